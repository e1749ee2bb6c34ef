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


def test_cached_refresh_at_the_largest_shape_respects_the_byte_budget(dev):
    """cached_attn_cuda at the reference's largest head count, (1,40,75600,128): the block-maxima
    buffer of the one-sweep refresh would take 7.2 GB, above the default budget, so the refresh step
    takes the reference's two sweeps and allocates no such buffer; with the budget raised it takes
    one sweep and caches the same key lists; the sparse step over them matches the host softmax on
    sampled q-blocks."""
    print("case refresh budget at 1x40x75600", flush=True)
    import fgattn_tk_cuda_amd.spattn.cuda_attn  # noqa: F401
    from fgattn_tk_cuda_amd.spattn import mask_utils as mu, sparseattn_functionals as fn

    B, H, S, D = 1, 40, 75600, 128
    g = torch.Generator(device=dev).manual_seed(4075)
    q, k, v = (torch.randn((B, H, S, D), generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16) for _ in range(3))
    thresh = 8.0 / S
    need = mu.blockmax_bytes(q)
    assert need > mu.BLOCKMAX_BUDGET_BYTES and not mu.use_onepass(q)
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats(dev)
    base = torch.cuda.memory_allocated(dev)
    cache2 = mu.NaiveMaskCache([0])
    o_fill = fn.cached_attn_cuda(q, k, v, 3, 0, thresh=thresh, blocksz=128, mask_cache=cache2)
    torch.cuda.synchronize()
    peak = torch.cuda.max_memory_allocated(dev) - base
    kvi2, kvn2 = cache2.get_mask_from_cache(3)
    lists_bytes = kvi2.numel() * 4
    # what the two-sweep refresh holds at its peak: O, the key lists, the bit-packed votes, statistics -
    # well short of the same plus the block maxima
    assert peak < lists_bytes + o_fill.numel() * 2 + need // 4, "the refresh step allocated %.2f GB" % (peak / 1e9)
    assert bool(torch.isfinite(o_fill.float()).all())
    cache1 = mu.NaiveMaskCache([0])
    fn.cached_attn_cuda(q, k, v, 3, 0, thresh=thresh, blocksz=128, mask_cache=cache1, blockmax_budget_bytes=8 << 30)
    kvi1, kvn1 = cache1.get_mask_from_cache(3)
    assert torch.equal(kvn1.view(-1), kvn2.view(-1)) and torch.equal(kvi1, kvi2)
    del kvi1, cache1
    assert 0 < float(kvn2.float().mean()) < S
    o_sp = fn.cached_attn_cuda(q, k, v, 3, 1, thresh=thresh, blocksz=128, mask_cache=cache2)
    torch.cuda.synchronize()
    sf = np.float32(orc.LOG2E / np.sqrt(D))
    SB = orc.ceil_div(S, 128)
    for h, i in ((0, 0), (17, 301), (H - 1, SB - 1)):
        r = slice(i * 128, min(S, (i + 1) * 128))
        lst = kvi2[0, h, i, : int(kvn2.view(B, H, SB)[0, h, i])].cpu().numpy()
        s = f32(q[0, h, r]) @ f32(k[0, h])[lst].T
        p = np.exp2((s - s.max(1, keepdims=True)) * sf)
        want = (p @ f32(v[0, h])[lst]) / p.sum(1, keepdims=True)
        assert_close_o(f32(o_sp[0, h, r]), want, "sparse step rows (%d,%d)" % (h, i))
