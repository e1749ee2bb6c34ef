"""GPU: the shapes the reference compiles its kernels for (python/cuda_attn.cu:13-31; d = 128),
run the way its own test does (python/test/test_extension.py:98-113): per shape dense attention,
dense attention with the fused row statistics, and sparse attention over a random permutation of
all keys - each through the reference-named torch.ops.cuda_attn operators and compared, on sampled
128-row q-blocks, with an fp32 softmax over all keys computed on the host (what the reference
compares with torch's scaled_dot_product_attention).  The sixth compiled shape, (1,24,75856) with
its hard-coded kv length, is tests/test_gpu_fullsize.py::test_reference_shape_75856_with_its_kv_length."""
import numpy as np
import pytest
import torch

from oracle import spattn_oracle as orc
from helpers import assert_close_o, assert_close_stat, f32

pytestmark = pytest.mark.gpu

SHAPES = [(1, 12, 32768), (1, 12, 32760), (1, 40, 32760), (1, 12, 75600), (1, 40, 75600)]


@pytest.mark.parametrize("B,H,S", SHAPES)
def test_reference_compiled_shape(dev, B, H, S):
    print("case reference shape", B, H, S, flush=True)
    import fgattn_tk_cuda_amd.spattn.cuda_attn  # noqa: F401

    ops = torch.ops.cuda_attn
    D = 128
    g = torch.Generator(device=dev).manual_seed(1000 + H + S)
    q, k, v = (torch.randn((B, H, S, D), generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16) for _ in range(3))
    Sp, SB = orc.padded_len(S), orc.ceil_div(S, 128)
    sf = np.float32(orc.LOG2E / np.sqrt(D))

    o_dense = torch.full_like(q, float("nan"))
    ops.full_attn(o_dense, q, k, v)
    o_stat = torch.full_like(q, float("nan"))
    mx = torch.full((B, H, 1, Sp), float("nan"), device=dev)
    dn = torch.full((B, H, 1, Sp), float("nan"), device=dev)
    ops.fullattn_maxq_denom(o_stat, mx, dn, q, k, v)
    # one random permutation of all keys for every q-block, the fill value behind it
    # (python/spattn/mask_utils.py: allindex_randompermutation_mask)
    row = torch.full((Sp,), Sp, dtype=torch.int32, device=dev)
    row[:S] = torch.randperm(S, generator=g, device=dev).int()
    kvi = row.expand(B, H, SB, Sp).contiguous()
    kvn = torch.full((B, H, SB), S, dtype=torch.int32, device=dev)
    o_sparse = torch.full_like(q, float("nan"))
    ops.sp_attn(o_sparse, q, k, v, kvi, kvn)
    torch.cuda.synchronize()
    del kvi
    for name, o in (("full_attn", o_dense), ("fullattn_maxq_denom", o_stat), ("sp_attn", o_sparse)):
        assert bool(torch.isfinite(o.float()).all()), name
    # pad rows of the statistics: max_q = 0, denom = -inf (include/maxq_denom.cuh:202-205)
    if Sp > S:
        assert bool((mx[..., S:] == 0).all()) and bool((dn[..., S:] == float("-inf")).all())

    rng = np.random.default_rng(S + H)
    blocks = [(int(rng.integers(H)), int(rng.integers(SB))) for _ in range(2)] + [(H - 1, SB - 1), (0, 0)]
    for h, i in blocks:
        r = slice(i * 128, min(S, (i + 1) * 128))
        qh, kh, vh = f32(q[0, h, r]), f32(k[0, h]), f32(v[0, h])
        s = qh @ kh.T
        m = s.max(1)
        p = np.exp2((s - m[:, None]) * sf)
        d = p.sum(1)
        want = (p @ vh) / d[:, None]
        assert_close_o(f32(o_dense[0, h, r]), want, "full_attn rows (%d,%d)" % (h, i))
        assert_close_o(f32(o_stat[0, h, r]), want, "fullattn_maxq_denom rows (%d,%d)" % (h, i))
        assert_close_o(f32(o_sparse[0, h, r]), want, "sp_attn rows (%d,%d)" % (h, i))
        assert_close_stat(f32(mx)[0, h, 0, r], m, "max_q", atol=1e-3)
        assert_close_stat(f32(dn)[0, h, 0, r], d, "denom")
