"""The reference's BGMV shape table as a test: every wide size it instantiates (bgmv/bgmv_config.h:12-80, 67 sizes)
times every narrow size (:82-87: 8, 16, 32, 64, 128), both directions where the reference's own dispatch would
take them (punica_ops.cc:291-334: both dims below 65536; the expand here also takes the wider LM-head sizes).
Three sizes are not multiples of 128 (1728, 2752, 6848) and six more not of 256 (640, 1152, 3456, 4480, 5504,
13696): they exercise the kernels' partial column blocks and the tails of their walks over the hidden dimension.  Each case is
3 tokens over 2 adapters, one token without adapter, against the oracle's bgmv_ref.  The SGMV kernels run the
sizes that are not multiples of 256.

Weights of all cases are views of one random pool (the cases differ in shape, not in data), so the table runs in
seconds."""

import pytest
import torch

from lorax_amd import sgmv
from oracle import lora_oracle as O
from tests.helpers import assert_close, ptr_table, randn

DEV = "cuda:0"

# FOR_BGMV_WIDE, bgmv_config.h:12-80
WIDE = [256, 512, 640, 768, 1024, 1152, 1280, 1536, 1728, 1792, 2048, 2304, 2560, 2752, 2816, 3072, 3456, 3584, 4096,
        4480, 4608, 5120, 5504, 5632, 6144, 6848, 6912, 7168, 7680, 8192, 8960, 9216, 9472, 10240, 11008, 12288,
        13696, 13824, 14336, 15360, 16384, 17920, 18944, 20480, 22016, 24576, 27392, 27648, 28672, 32000, 32256,
        32512, 32768, 33024, 35840, 36864, 43264, 49152, 64000, 64256, 64512, 102400, 102656, 102912, 128000, 128256,
        128512]
NARROW = [8, 16, 32, 64, 128]  # FOR_BGMV_WIDE_NARROW, bgmv_config.h:82-87
FP16_SUBSET = [256, 1728, 2752, 4096, 5504, 6848, 13696, 14336, 27392, 32256, 43264, 64512, 128512]


@pytest.fixture(scope="module")
def pools():
    gen = torch.Generator().manual_seed(77)
    out = {}
    for dtype in (torch.bfloat16, torch.float16):
        cpu = [(torch.randn((max(WIDE) * max(NARROW),), generator=gen) * 0.05).to(dtype) for _ in range(2)]
        out[dtype] = (cpu, [p.to(DEV) for p in cpu])
    return out


def test_the_table_has_the_references_67_sizes():
    assert len(WIDE) == 67 and len(set(WIDE)) == 67 and WIDE == sorted(WIDE) and all(w % 8 == 0 for w in WIDE)
    assert [w for w in WIDE if w % 128 != 0] == [1728, 2752, 6848]
    assert set(FP16_SUBSET) <= set(WIDE)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("r", NARROW)
def test_bgmv_reference_shape_table(pools, dtype, r):
    cpu_pool, dev_pool = pools[dtype]
    gen = torch.Generator().manual_seed(r)
    idx = [1, -1, 0]
    idx_d = torch.tensor(idx, dtype=torch.int64, device=DEV)
    failures = []
    for wide in WIDE if dtype == torch.bfloat16 else FP16_SUBSET:
        print(f"case dtype={dtype} r={r} wide={wide}", flush=True)
        n = r * wide
        # expand: B^T stacks [1, wide, r]; v [3, r]
        wb_cpu = [p[:n].view(1, wide, r) for p in cpu_pool]
        wb_dev = [p[:n].view(1, wide, r) for p in dev_pool]
        v = randn((3, r), 1.0, gen, dtype, DEV)
        y0 = randn((3, wide), 0.5, gen, dtype, DEV)
        y = y0.clone()
        sgmv.add_lora_b_bgmv(y, v, ptr_table(wb_dev, DEV), idx_d, 0)
        y_ref = O.bgmv_ref(y0.cpu().clone(), v.cpu(), wb_cpu, idx, 0)
        try:
            assert_close(y, y_ref, f"expand r={r} wide={wide}")
            assert torch.equal(y[1], y0[1]), f"expand r={r} wide={wide}: the token without adapter changed"
        except AssertionError as exc:
            failures.append(str(exc))
        if wide >= 65536:  # the shrink keeps the reference's limit (punica_ops.cc:310)
            continue
        wa_cpu = [p[:n].view(1, r, wide) for p in cpu_pool]
        wa_dev = [p[:n].view(1, r, wide) for p in dev_pool]
        x = randn((3, wide), 1.0, gen, dtype, DEV)
        u0 = randn((3, r), 0.5, gen, dtype, DEV)
        u = u0.clone()
        sgmv.add_lora_a_bgmv(u, x, ptr_table(wa_dev, DEV), idx_d, 0)
        u_ref = O.bgmv_ref(u0.cpu().clone(), x.cpu(), wa_cpu, idx, 0)
        try:
            # sums over up to 64512 products of N(0,1) x N(0,0.05) values reach |v| ~ 13: the roundings' spacing applies
            assert_close(u, u_ref, f"shrink r={r} wide={wide}", rounded=[u_ref])
            assert torch.equal(u[1], u0[1]), f"shrink r={r} wide={wide}: the token without adapter changed"
        except AssertionError as exc:
            failures.append(str(exc))
    torch.cuda.synchronize()
    assert not failures, "\n".join(failures)


@pytest.mark.gpu
@pytest.mark.parametrize("r", [16, 64])
@pytest.mark.parametrize("wide", [1728, 2752, 5504, 6848, 13696])
def test_sgmv_at_the_sizes_that_are_not_multiples_of_256(pools, r, wide):
    """Shrink (wide -> r) and expand (r -> wide, both B layouts) over ragged segments, one of them empty."""
    print(f"case r={r} wide={wide}", flush=True)
    dtype = torch.bfloat16
    cpu_pool, dev_pool = pools[dtype]
    gen = torch.Generator().manual_seed(wide + r)
    lens = [5, 40, 0, 530]  # more than 512 rows: past the streaming kernel, on the MFMA kernels
    starts, ends, pos = [], [], 2
    for n in lens:
        starts.append(pos)
        ends.append(pos + n)
        pos += n + 1
    T = pos + 3
    n = r * wide
    # four "adapters": two pool views, each at two offsets
    a_cpu = [cpu_pool[i % 2][(i // 2) * 64 : (i // 2) * 64 + n].view(1, r, wide) for i in range(4)]
    a_dev = [dev_pool[i % 2][(i // 2) * 64 : (i // 2) * 64 + n].view(1, r, wide) for i in range(4)]
    bt_cpu = [cpu_pool[i % 2][(i // 2) * 128 : (i // 2) * 128 + n].view(1, wide, r) for i in range(4)]
    bt_dev = [dev_pool[i % 2][(i // 2) * 128 : (i // 2) * 128 + n].view(1, wide, r) for i in range(4)]
    s_start = torch.tensor(starts, dtype=torch.int32, device=DEV)
    s_end = torch.tensor(ends, dtype=torch.int32, device=DEV)
    x = randn((T, wide), 1.0, gen, dtype, DEV)
    tmp = sgmv.get_tmp_tensor(torch.device(DEV))
    v = sgmv.lora_a_sgmv_cutlass(x, tmp, ptr_table(a_dev, DEV, null_at=[2]), s_start, s_end, 0, r)
    v_ref = torch.zeros((T, r), dtype=dtype)
    for i, (s, e) in enumerate(zip(starts, ends)):
        if e > s:
            v_ref[s:e] = x.cpu()[s:e] @ a_cpu[i][0].t()
    assert_close(v, v_ref, "shrink", rounded=[v_ref])

    vin = randn((T, r), 1.0, gen, dtype, DEV)
    y0 = randn((T, wide), 0.5, gen, dtype, DEV)
    tmp_e = sgmv.get_tmp_tensor_for_size(len(lens), torch.device(DEV))
    y_t = y0.clone()
    sgmv.lora_b_sgmv_cutlass_slice(y_t, vin, tmp_e, ptr_table(bt_dev, DEV, null_at=[2]), s_start, s_end, 0, 0, wide,
                                   transposed=True)
    b_dev = [w.transpose(1, 2).contiguous() for w in bt_dev]  # the reference's [L, r, h_out]
    y_r = y0.clone()
    sgmv.lora_b_sgmv_cutlass(y_r, vin, tmp_e, ptr_table(b_dev, DEV, null_at=[2]), s_start, s_end, 0)
    y_ref = y0.cpu().clone()
    for i, (s, e) in enumerate(zip(starts, ends)):
        if e > s:
            delta = (vin.cpu()[s:e] @ bt_cpu[i][0].t())
            y_ref[s:e] = (y_ref[s:e].float() + delta.float()).to(dtype)
    assert_close(y_t, y_ref, "expand, B^T stacks")
    assert_close(y_r, y_ref, "expand, reference layout")
    covered = torch.zeros(T, dtype=torch.bool)
    for s, e in zip(starts, ends):
        covered[s:e] = True
    assert torch.equal(y_t.cpu()[~covered], y0.cpu()[~covered])
    assert torch.equal(y_r.cpu()[~covered], y0.cpu()[~covered])
    assert torch.count_nonzero(v.cpu()[~covered]) == 0
