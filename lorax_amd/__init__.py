"""MI355X (gfx950) implementation of LoRAX's multi-adapter LoRA hot path.

``lorax_amd.sgmv`` (alias ``lorax_amd.punica``) is the kernel-facing API,
``lorax_amd.adapters`` builds the per-batch routing tables, ``lorax_amd.layers`` holds the
LoRA linear layers that call the kernels, ``lorax_amd.segments`` the run-length helpers.
"""

__version__ = "0.1.0"
