"""Alias of :mod:`lorax_amd.sgmv` under the module name the reference's importers use
(``lorax_server.utils.punica``; e.g. utils/layers.py:15, adapters/lora.py:13)."""

from lorax_amd.sgmv import *  # noqa: F401,F403
from lorax_amd.sgmv import (  # noqa: F401
    BGMV_MAX_RANK,
    HAS_SGMV,
    LORAX_PUNICA_TRITON_DISABLED,
    MAX_RANK_CUSTOM,
    MIN_RANK_CUSTOM,
    MIN_SGMV_RANK,
    SGMV_BLOCK_SIZE,
    _kernels,
)
