"""GPU: golden fixtures, the torch.ops.cuda_attn operator path and the functionals."""
import glob
import os

import numpy as np
import pytest
import torch

from fgattn_tk_cuda_amd import capi, workloads as wl
from oracle import spattn_oracle as orc
from helpers import assert_close_o, assert_close_stat, f32, to_dev

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _bf(x, dev):
    return torch.from_numpy(np.ascontiguousarray(x)).to(torch.bfloat16).to(dev)


@pytest.mark.parametrize("name", ["sparse_d64_q64", "sparse_d128_q128", "dense_d64"])
def test_sp_attn_golden(dev, name):
    print("case golden", name, flush=True)
    g = np.load(os.path.join(GOLD, name + ".npz"))
    q, k, v = (_bf(g[x][None, None], dev) for x in "qkv")
    idx = torch.from_numpy(g["kv_indices"]).to(dev)
    num = torch.from_numpy(g["kv_num_indices"]).to(dev)
    o = torch.full_like(q, float("nan"))
    lse = torch.full(q.shape[:3], float("nan"), device=dev)
    capi.sp_attn(o, q, k, v, idx, num, lse=lse, qblk=int(g["qblk"]))
    assert_close_o(f32(o)[0, 0], g["o"], name)
    assert_close_stat(f32(lse)[0, 0], g["lse"], name + " lse")
    if name == "dense_d64":
        o2 = torch.full_like(q, float("nan"))
        capi.full_attn(o2, q, k, v)
        assert_close_o(f32(o2)[0, 0], g["o"], "full_attn golden")


@pytest.mark.parametrize("name", ["prepass_d64", "prepass_d128"])
def test_prepass_golden(dev, name):
    print("case golden", name, flush=True)
    g = np.load(os.path.join(GOLD, name + ".npz"))
    q, k = (_bf(g[x][None, None], dev) for x in "qk")
    S = q.shape[2]
    Sp = orc.padded_len(S)
    mx = torch.empty((1, 1, 1, Sp), device=dev)
    dn = torch.empty((1, 1, 1, Sp), device=dev)
    capi.maxq_denom(mx, dn, q, k)
    assert_close_stat(f32(mx)[0, 0, 0, :S], g["max_q"], "max_q", atol=1e-4)
    assert_close_stat(f32(dn)[0, 0, 0, :S], g["denom"], "denom")
    mask = torch.zeros((1, 1, Sp // 128, Sp), dtype=torch.int32, device=dev)
    capi.booleanmask_128(mask, mx, dn, q, k, float(g["thresh"]))
    got = mask.cpu().numpy()
    near = np.abs(g["pmax"] - g["thresh"]) <= 1e-2 * g["thresh"]
    assert np.array_equal((got[..., :S] > 0) | near, (g["votes"][..., :S] > 0) | near)
    gm = torch.from_numpy(g["votes"]).to(dev)
    kvi = torch.full(gm.shape, Sp, dtype=torch.int32, device=dev)
    kvn = torch.zeros(gm.shape[:3], dtype=torch.int32, device=dev)
    capi.booleanmask_to_indexmask(kvi, kvn, gm, S)
    assert np.array_equal(kvi.cpu().numpy(), g["kv_indices"]) and np.array_equal(kvn.cpu().numpy(), g["kv_num_indices"])


def test_operator_extension_on_device(dev):
    """The seven torch.ops.cuda_attn ops, used the way the reference's callers use them."""
    print("case torch ops", flush=True)
    import fgattn_tk_cuda_amd.spattn.cuda_attn  # noqa: F401
    from fgattn_tk_cuda_amd.spattn import mask_utils as mu

    ops = torch.ops.cuda_attn
    B, H, S, D = 1, 2, 1000, 128
    q, k, v = to_dev(dev, *wl.clustered_qkv(B, H, S, D, seed=71, sigma=0.5))
    want = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float())
    o = torch.empty_like(q)
    ops.full_attn(o, q, k, v)
    assert_close_o(f32(o), f32(want), "ops.full_attn")
    Sp, SB = 1024, 8
    kvi = torch.zeros((B, H, SB, Sp), dtype=torch.int32, device=dev)
    kvn = torch.zeros((B, H, SB), dtype=torch.int32, device=dev)
    ops.all_index_mask(kvi, kvn, B, H, SB, S)
    o2 = torch.empty_like(q)
    ops.sp_attn(o2, q, k, v, kvi, kvn)
    assert_close_o(f32(o2), f32(want), "ops.sp_attn identity list")
    # a list per 64 rows is recognised by the number of q-blocks
    kvi64, kvn64 = to_dev(dev, *wl.permuted_all_index(B, H, S, qblk=64, seed=72))
    ops.sp_attn(o2, q, k, v, kvi64, kvn64)
    assert_close_o(f32(o2), f32(want), "ops.sp_attn 64-row lists")
    mx = torch.empty((B, H, 1, Sp), device=dev)
    dn = torch.empty((B, H, 1, Sp), device=dev)
    o3 = torch.empty_like(q)
    ops.fullattn_maxq_denom(o3, mx, dn, q, k, v)
    assert_close_o(f32(o3), f32(want), "ops.fullattn_maxq_denom")
    mx2, dn2 = torch.empty_like(mx), torch.empty_like(dn)
    ops.maxq_denom(mx2, dn2, q, k)
    assert_close_stat(f32(mx2), f32(mx), "max_q fused vs alone", atol=1e-4)
    assert_close_stat(f32(dn2), f32(dn), "denom fused vs alone")
    # the wrappers: torch definition of the mask vs the device path
    thr = 0.02
    dev_mask = mu.qk_bitmask_cuda(q, k, thr)[..., :S]
    ref_mask = mu.qk_bitmask(q.float(), k.float(), thr)
    _, pmax = orc.booleanmask_128(f32(mx2), f32(dn2), f32(q), f32(k), thr)
    near = torch.from_numpy(np.abs(pmax - thr) <= 1e-2 * thr).to(dev)
    assert torch.equal(dev_mask | near, ref_mask | near)
    idx_d, num_d = mu.qk_indexmask_cuda(q, k, thr)
    idx_r, num_r = mu.bitmask_to_indexmask(mu.qk_bitmask_cuda(q, k, thr))
    assert torch.equal(idx_d, idx_r) and torch.equal(num_d, num_r)
    # the bit-packed cache path: one kernel each way equals the torch-level pack / unpack + compaction
    votes = mu.qk_bitmask_from_maxq_denom_cuda(mx2, dn2, q, k, thr)
    packed = mu.pack_votes_cuda(votes)
    assert torch.equal(packed, mu.pack(votes > 0))
    idx_p, num_p = mu.packedmask_to_indexmask_cuda(packed, S)
    idx_u, num_u = mu.bitmask_to_indexmask_cuda(mu.unpack(packed).to(torch.int32), S)
    assert torch.equal(idx_p, idx_u) and torch.equal(num_p, num_u)
    cache = mu.CompressedBitMaskCache([0])
    cache.update_cache(3, votes, S)
    assert cache.cache[3][0].dtype == torch.uint8 and cache.cache[3][0].shape[-1] * 8 == votes.shape[-1]
    idx_c, num_c = cache.get_mask_from_cache(3)
    assert torch.equal(idx_c, idx_u) and torch.equal(num_c, num_u)
    # errors are raised, not swallowed
    with pytest.raises(RuntimeError):
        ops.full_attn(o, q.float(), k, v)
    with pytest.raises(RuntimeError):
        ops.sp_attn(o, q, k, v, kvi[:, :, :3].contiguous(), kvn)


def test_extended_operators_on_device(dev):
    """The operators beyond the reference's seven: kv length, scale and lse through torch.ops, the
    block-list attention, the bit-packed sweep, the block lists, the reusable work order.  Each
    against the oracle or, where an operator restates another, bit for bit against that one."""
    print("case extended torch ops", flush=True)
    import fgattn_tk_cuda_amd.spattn.cuda_attn  # noqa: F401
    from fgattn_tk_cuda_amd.spattn import mask_utils as mu

    ops = torch.ops.cuda_attn
    B, H, S, D = 1, 2, 1000, 64
    kv = 870
    q, k, v = to_dev(dev, *wl.clustered_qkv(B, H, S, D, seed=73, sigma=0.6))
    scale = 0.1
    # full_attn_ex: kv length + scale + lse against torch on the cut keys
    want = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float()[:, :, :kv], v.float()[:, :, :kv], scale=scale)
    wlse = torch.logsumexp(torch.einsum("bhsd,bhtd->bhst", q.float(), k.float()[:, :, :kv]) * scale, -1)
    o = torch.full_like(q, float("nan"))
    lse = torch.full((B, H, S), float("nan"), device=dev)
    ops.full_attn_ex(o, lse, q, k, v, scale, kv)
    assert_close_o(f32(o), f32(want), "full_attn_ex")
    assert_close_stat(f32(lse), f32(wlse), "full_attn_ex lse")
    o0 = torch.full_like(q, float("nan"))
    ops.full_attn_ex(o0, None, q, k, v, 0.0, 0)
    o1 = torch.full_like(q, float("nan"))
    ops.full_attn(o1, q, k, v)
    assert torch.equal(o0, o1)
    # statistics with a kv length, then the vote mask and the bit-packed sweep with it
    Sp, SB = 1024, 8
    mx = torch.empty((B, H, 1, Sp), device=dev)
    dn = torch.empty((B, H, 1, Sp), device=dev)
    ops.maxq_denom_ex(mx, dn, q, k, 0.0, kv)
    wmx, wdn = orc.maxq_denom(f32(q), f32(k), kv_len=kv)
    assert_close_stat(f32(mx)[..., :S], wmx[..., :S], "maxq_denom_ex max", atol=1e-3)
    assert_close_stat(f32(dn)[..., :S], wdn[..., :S], "maxq_denom_ex denom")
    o2 = torch.full_like(q, float("nan"))
    mx2, dn2 = torch.empty_like(mx), torch.empty_like(dn)
    ops.fullattn_maxq_denom_ex(o2, mx2, dn2, q, k, v, 0.0, kv)
    wo2 = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float()[:, :, :kv], v.float()[:, :, :kv])
    assert_close_o(f32(o2), f32(wo2), "fullattn_maxq_denom_ex")
    assert_close_stat(f32(dn2), f32(dn), "fused denom with kv_len")
    thr = 0.02
    votes = torch.zeros((B, H, SB, Sp), dtype=torch.int32, device=dev)
    ops.booleanmask_128_ex(votes, mx, dn, q, k, thr, 0.0, kv)
    assert not bool(votes[..., kv:].any()) and bool(votes.any())
    for qblk in (128, 64):
        nq = (S + qblk - 1) // qblk
        packed = torch.full((B, H, nq, Sp // 8), 0xA5, dtype=torch.uint8, device=dev)
        ops.booleanmask_packed(packed, mx, dn, q, k, thr, qblk, 0.0, kv)
        if qblk == 128:
            assert torch.equal(packed, mu.pack(votes > 0))
        else:
            assert torch.equal(packed[:, :, 0::2] | packed[:, :, 1::2], mu.pack(votes > 0))
        assert torch.equal(packed, mu.qk_packedmask_from_maxq_denom_cuda(mx, dn, q, k, thr, qblk, kv))
        # block lists: operator == oracle on the device's own bits; packed and votes sources agree
        blk_idx, blk_cnt, bm = mu.packedmask_to_blocklists_cuda(packed, kv, with_blockmask=True)
        wi, wn, wbm = orc.block_lists_from_mask(orc.unpack_mask(packed.cpu().numpy()), kv, fill=-1)
        assert np.array_equal(blk_idx.cpu().numpy(), wi) and np.array_equal(blk_cnt.cpu().numpy(), wn)
        assert np.array_equal(bm.cpu().numpy(), wbm.astype(np.uint8))
        if qblk == 128:
            bi2, bc2 = mu.bitmask_to_blocklists_cuda(votes, kv)
            assert torch.equal(bi2, blk_idx) and torch.equal(bc2, blk_cnt)
        # sp_attn_block with lse, scale, kv length and a work order
        order = mu.qblock_order_cuda(blk_cnt)
        assert np.array_equal(order.cpu().numpy(), orc.qblock_order(wn))
        ob = torch.full_like(q, float("nan"))
        lb = torch.full((B, H, S), float("nan"), device=dev)
        ops.sp_attn_block(ob, lb, q, k, v, blk_idx, blk_cnt, order, qblk, scale, kv)
        tok, num = orc.block_list_to_token_list(wi, wn, kv, mask_stride=Sp)
        wo, wl_ = orc.sp_attn(f32(q), f32(k), f32(v), tok, num, qblk=qblk, scale=scale)
        assert_close_o(f32(ob), wo, "sp_attn_block q%d" % qblk)
        assert_close_stat(f32(lb), wl_, "sp_attn_block lse q%d" % qblk)
        ob2 = torch.full_like(q, float("nan"))
        ops.sp_attn_block(ob2, None, q, k, v, blk_idx, blk_cnt, None, 0, scale, kv)     # no order, inferred q-block
        assert torch.equal(ob, ob2)
        # the same keys as token lists through sp_attn_ex: the operator's own cross-check
        tk, nm = torch.from_numpy(tok).to(dev), torch.from_numpy(num).to(dev)
        ot = torch.full_like(q, float("nan"))
        lt = torch.full((B, H, S), float("nan"), device=dev)
        ops.sp_attn_ex(ot, lt, q, k, v, tk, nm, mu.qblock_order_cuda(nm), scale, kv)
        assert_close_o(f32(ot), wo, "sp_attn_ex q%d" % qblk)
        assert_close_stat(f32(lt), wl_, "sp_attn_ex lse q%d" % qblk)
    # sp_attn_ex without extras == sp_attn
    kvi, kvn = mu.qk_indexmask_cuda(q, k, thr)
    oa, ob_ = torch.full_like(q, float("nan")), torch.full_like(q, float("nan"))
    ops.sp_attn(oa, q, k, v, kvi, kvn)
    ops.sp_attn_ex(ob_, None, q, k, v, kvi, kvn, None, 0.0, 0)
    assert torch.equal(oa, ob_)
    # the pure-torch definition of the block lists against the device path (kv length = S here)
    bi_d, bc_d = mu.qk_blocklists_cuda(q, k, thr, qblk=128)
    bi_r, bc_r, _ = mu.qk_blocklists(q.float(), k.float(), thr, qblk=128)
    mxs, dns = mu._stats_buffers(q)
    ops.maxq_denom(mxs, dns, q, k)
    _, pmax = orc.booleanmask_128(f32(mxs), f32(dns), f32(q), f32(k), thr)
    if not (np.abs(pmax - thr) <= 1e-2 * thr).any():
        assert torch.equal(bc_d, bc_r) and torch.equal(bi_d, bi_r)
    else:
        assert (bc_d - bc_r).abs().max().item() <= 2
    # bad arguments raise
    with pytest.raises(RuntimeError):
        ops.full_attn_ex(o, None, q, k, v, 0.0, S + 1)
    with pytest.raises(RuntimeError):
        ops.sp_attn_block(o, None, q, k, v, blk_idx, blk_cnt, order[:3].contiguous(), 64, 0.0, 0)
    with pytest.raises(RuntimeError):
        ops.booleanmask_packed(packed, mx, dn, q, k, thr, 32, 0.0, 0)


def test_block_maxima_operators_and_helpers(dev):
    """torch.ops.cuda_attn.maxq_denom_blockmax / fullattn_maxq_denom_blockmax / blockmax_to_blocklists
    against the C ABI (bit for bit), and the one-sweep helper against the two-sweep one: a superset
    of its block lists, the same except where a block's best key lies within the band around the
    threshold."""
    print("case blockmax operators", flush=True)
    from fgattn_tk_cuda_amd.spattn import mask_utils as mu

    ops = torch.ops.cuda_attn
    B, H, S, D, thr = 1, 2, 900, 64, 0.01
    q, k, v = to_dev(dev, *wl.clustered_qkv(B, H, S, D, seed=83, sigma=0.7))
    Sp = orc.padded_len(S)
    mx, dn, mx2, dn2 = (torch.empty((B, H, 1, Sp), device=dev) for _ in range(4))
    bmx, bmx2 = (torch.full((B, H, Sp // 64, Sp), -5.0, dtype=torch.bfloat16, device=dev) for _ in range(2))
    o, o2 = torch.empty_like(q), torch.empty_like(q)
    ops.fullattn_maxq_denom_blockmax(o, mx, dn, bmx, q, k, v, 0.0, 0)
    capi.fullattn_maxq_denom_blockmax(o2, mx2, dn2, bmx2, q, k, v)
    assert torch.equal(o, o2) and torch.equal(mx, mx2) and torch.equal(dn, dn2) and torch.equal(bmx, bmx2)
    bmx3 = torch.full_like(bmx, -5.0)
    ops.maxq_denom_blockmax(mx2, dn2, bmx3, q, k, 0.0, 0)
    assert torch.equal(mx, mx2) and torch.equal(dn, dn2) and torch.equal(bmx, bmx3)
    for qblk in (64, 128):
        nq, nb = orc.ceil_div(S, qblk), Sp // 64
        bi, bc, bm = mu.blockmax_to_blocklists_cuda(bmx, mx, dn, thr, S, D, qblk, with_blockmask=True)
        bi2 = torch.full((B, H, nq, nb), -1, dtype=torch.int32, device=dev)
        bc2 = torch.zeros((B, H, nq), dtype=torch.int32, device=dev)
        capi.blockmax_to_blocklists(bi2, bc2, bmx, mx, dn, thr, S, D, qblk=qblk)
        assert torch.equal(bi, bi2) and torch.equal(bc, bc2) and torch.equal(bm.sum(-1).int(), bc)
        b1, c1 = mu.qk_blocklists_onepass_cuda(q, k, thr, qblk)
        assert torch.equal(b1, bi) and torch.equal(c1, bc)
        # two sweeps (bit-packed threshold sweep) against one: equal outside the band
        _, _, bm_two = mu.packedmask_to_blocklists_cuda(mu.qk_packedmask_from_maxq_denom_cuda(mx, dn, q, k, thr, qblk), S,
                                                        with_blockmask=True)
        _, pmax = orc.booleanmask_rows(f32(mx), f32(dn), f32(q), f32(k), 1.0, qblk=qblk)
        pblk = np.zeros((B, H, nq, nb), np.float32)
        for J in range(orc.ceil_div(S, 64)):
            pblk[..., J] = pmax[..., 64 * J: min(64 * J + 64, S)].max(axis=-1)
        # the stored maxima are rounded up by at most 2^-7 |s|: the one-sweep mask holds every block of the
        # two-sweep mask and equals it outside the band widened downwards by that step
        lift = float(np.exp2(2.0 ** -7 * float(bmx[:, :, : orc.ceil_div(S, 64), :S].float().abs().max()) * orc.LOG2E / np.sqrt(D)))
        band = (pblk >= thr * (1 - 1e-2) / lift) & (pblk <= thr * (1 + 1e-2))
        one, two = bm.cpu().numpy().astype(bool), bm_two.cpu().numpy().astype(bool)
        assert not (two & ~one & ~band).any()
        assert np.array_equal(one | band, two | band)
        assert 0.05 < bm.float().mean().item() < 0.95
    # key lists with one full sweep: the reference's form of the lists.  The helpers take the blocks a
    # little below the threshold (a superset of the blocks that hold a passing key), so lists and
    # votes equal those of the two full sweeps exactly
    i1, n1 = mu.qk_indexmask_onepass_cuda(q, k, thr)
    i2, n2 = mu.qk_indexmask_cuda(q, k, thr)
    assert torch.equal(n1, n2) and torch.equal(i1, i2)
    m1 = mu.qk_bitmask_from_blockmax_cuda(bmx, mx, dn, q, k, thr)
    m2 = mu.qk_bitmask_from_maxq_denom_cuda(mx, dn, q, k, thr)
    assert torch.equal(m1, m2) and int(m1.max()) <= 8 and bool((m1 > 0).any())
    for qb in (128, 64):
        assert torch.equal(mu.qk_packedmask_from_blockmax_cuda(bmx, mx, dn, q, k, thr, qb),
                           mu.qk_packedmask_from_maxq_denom_cuda(mx, dn, q, k, thr, qb))
    pk1 = torch.empty((B, H, orc.ceil_div(S, 64), Sp // 8), dtype=torch.uint8, device=dev)
    b128, c128 = mu.blockmax_to_blocklists_cuda(bmx, mx, dn, thr, S, D, 128)
    ops.booleanmask_packed_blocks(pk1, mx, dn, q, k, b128, c128, thr, 64, 0.0, 0)
    pk2 = mu.qk_packedmask_from_maxq_denom_cuda(mx, dn, q, k, thr, 64)
    assert (pk1 != pk2).float().mean().item() < 1e-3
    with pytest.raises(RuntimeError):
        ops.booleanmask_128_blocks(m1, mx, dn, q, k, b128[:, :, :2].contiguous(), c128, thr, 0.0, 0)
    with pytest.raises(RuntimeError):
        ops.blockmax_to_blocklists(bi, bc, None, bmx[:, :, :3].contiguous(), mx, dn, thr, S, D, 128, 0.0, 0)
    with pytest.raises(RuntimeError):
        ops.blockmax_to_blocklists(bi, bc, None, bmx, mx, dn, thr, S, D, 32, 0.0, 0)


@pytest.mark.parametrize("seed", range(10))
def test_one_sweep_key_lists_equal_the_two_sweep_lists(dev, seed):
    """The reference's key lists through one full sweep (statistics with block maxima, blocks taken a
    little below the threshold, vote sweep over those blocks) against the two full sweeps: counts,
    lists and votes equal on every element, over random shapes, head dims, data spreads and thresholds."""
    from fgattn_tk_cuda_amd.spattn import mask_utils as mu

    rng = np.random.default_rng(1000 + seed)
    B, H = 1, int(rng.integers(1, 4))
    S = int(rng.integers(130, 2600))
    D = int(rng.choice([64, 128]))
    sigma = float(rng.choice([0.0, 0.4, 0.8, 1.5]))
    print("case one sweep vs two", seed, H, S, D, sigma, flush=True)
    q, k, _ = to_dev(dev, *wl.clustered_qkv(B, H, S, D, seed=2000 + seed, sigma=sigma))
    for thr in (float(rng.choice([3e-4, 1e-3, 3e-3, 1e-2, 5e-2])), 1.0 / S):
        i2, n2 = mu.qk_indexmask_cuda(q, k, thr)
        i1, n1 = mu.qk_indexmask_onepass_cuda(q, k, thr)
        assert torch.equal(n1, n2), "counts at threshold %g" % thr
        assert torch.equal(i1, i2), "lists at threshold %g" % thr
        assert int(n2.sum()) > 0


def test_functionals_with_mask_cache(dev):
    print("case functionals", flush=True)
    from fgattn_tk_cuda_amd.spattn import mask_utils as mu, sparseattn_functionals as fn

    B, H, S, D = 1, 2, 900, 64
    q, k, v = to_dev(dev, *wl.clustered_qkv(B, H, S, D, seed=81, sigma=0.7))
    dense = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float())
    assert_close_o(f32(fn.baseline_attn(q, k, v, 0, 0)), f32(dense), "baseline_attn")
    assert_close_o(f32(fn.baseline_attn_maxq_denom(q, k, v, 0, 0)), f32(dense), "baseline_attn_maxq_denom")
    with pytest.raises(NotImplementedError):
        fn.attn_lshmask_cuda(q, k, v, 0, 0, thresh=0.01, blocksz=128)
    seen_naive = False
    for cache in (mu.NaiveMaskCache([0]), mu.CompressMaskCache([0]), mu.OffloadMaskCache([0]), mu.BitMaskCache([0]),
                  mu.CompressedBitMaskCache([0]), mu.NaiveMaskCache([0])):
        f = fn.cached_attn_cuda if isinstance(cache, mu.NaiveMaskCache) else fn.bitmaskcached_attn_cuda
        extra = {"onepass": False} if type(cache) is mu.NaiveMaskCache and seen_naive else {}   # the reference's two sweeps
        seen_naive = seen_naive or type(cache) is mu.NaiveMaskCache
        o0 = f(q, k, v, 7, 0, thresh=0.01, blocksz=128, mask_cache=cache, **extra)   # step 0: dense + cache fill
        assert_close_o(f32(o0), f32(dense), "cache fill step")
        o1 = f(q, k, v, 7, 1, thresh=0.01, blocksz=128, mask_cache=cache)       # step 1: sparse from cache
        kvi, kvn = cache.get_mask_from_cache(7)
        want, _ = orc.sp_attn(f32(q), f32(k), f32(v), kvi.cpu().numpy(), kvn.cpu().numpy(), qblk=128)
        assert_close_o(f32(o1), want, "sparse step from %s" % type(cache).__name__)
        assert 0 < kvn.float().mean().item() < S
        if isinstance(cache, mu.NaiveMaskCache):
            assert cache.get_order(7) is not None and cache.get_order(7).numel() == kvn.numel()
        if isinstance(cache, mu.CompressMaskCache):
            # the compressed cache returns the lists it was given (as sets per q-block; here ascending both ways)
            ref_i, ref_n = mu.qk_indexmask_cuda(q, k, 0.01, blocksz=128)
            assert torch.equal(kvn.view_as(ref_n), ref_n) and torch.equal(kvi, ref_i)
    for qblk, onepass in ((64, True), (128, True), (64, False), (128, False)):
        cache = mu.BlockListCache([0])
        o0 = fn.blockcached_attn_cuda(q, k, v, 7, 0, thresh=0.01, qblk=qblk, mask_cache=cache, onepass=onepass)
        assert_close_o(f32(o0), f32(dense), "block cache fill step")
        o1 = fn.blockcached_attn_cuda(q, k, v, 7, 1, thresh=0.01, qblk=qblk, mask_cache=cache)
        bi, bc = cache.get_mask_from_cache(7)
        tok, num = orc.block_list_to_token_list(bi.cpu().numpy(), bc.cpu().numpy(), S)
        wb, _ = orc.sp_attn(f32(q), f32(k), f32(v), tok, num, qblk=qblk)
        assert_close_o(f32(o1), wb, "block sparse step q%d" % qblk)
        assert 0 < bc.float().mean().item() < (S + 63) // 64
    o2 = fn.attn_computed_with_sparse_mask_cuda(q, k, v, thresh=0.01, blocksz=128)
    assert_close_o(f32(o2), want, "attn_computed_with_sparse_mask_cuda")
    o3 = fn.attn_2xmask_cuda(q, k, v, 0, 0, blocksz=128)
    w3 = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float()[:, :, 0:2 * (S // 2):2], v.float()[:, :, 0:2 * (S // 2):2])
    assert_close_o(f32(o3), f32(w3), "attn_2xmask_cuda")


def test_sp_attn_operator_keeps_its_work_order(dev):
    """The reference-named operator has no argument for a work order: it computes one when it first sees a counts
    tensor or when that tensor was written to since, and otherwise launches the attention kernel alone - no
    allocation on repeated calls, the same bits as the C ABI, also after the counts changed in place and from a
    recorded graph."""
    print("case sp_attn operator work order", flush=True)
    import fgattn_tk_cuda_amd.spattn.cuda_attn  # noqa: F401

    ops = torch.ops.cuda_attn
    B, H, S, D = 1, 3, 2048, 128
    q, k, v = to_dev(dev, *wl.randn_qkv(B, H, S, D, seed=11))
    g = torch.Generator().manual_seed(5)
    SB, Sp = S // 128, S
    kvi = torch.full((B, H, SB, Sp), Sp, dtype=torch.int32)
    kvn = torch.zeros((B, H, SB), dtype=torch.int32)
    for b in range(B):
        for h in range(H):
            for i in range(SB):
                n = int(torch.randint(1, S // 2 if i % 3 else S, (1,), generator=g))   # very uneven lengths
                kvi[b, h, i, :n] = torch.randperm(S, generator=g)[:n].sort().values.int()
                kvn[b, h, i] = n
    kvi, kvn = kvi.to(dev), kvn.to(dev)

    def want_of(counts):
        w = torch.full_like(q, float("nan"))
        capi.sp_attn(w, q, k, v, kvi, counts, qblk=128)
        return w

    want = want_of(kvn)
    o = torch.full_like(q, float("nan"))
    ops.sp_attn(o, q, k, v, kvi, kvn)            # first sight of kvn: computes the order
    torch.cuda.synchronize()
    assert torch.equal(o, want)
    n0 = torch.cuda.memory_stats(dev)["allocation.all.allocated"]
    for _ in range(3):
        o.fill_(float("nan"))
        ops.sp_attn(o, q, k, v, kvi, kvn)
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats(dev)["allocation.all.allocated"] == n0, "repeated calls must not allocate"
    assert torch.equal(o, want)
    # the counts change in place (shorter lists): new order in the same buffer, same bits as the C ABI
    kvn.copy_(torch.clamp(kvn // 3, min=1))
    want2 = want_of(kvn)
    n1 = torch.cuda.memory_stats(dev)["allocation.all.allocated"]
    o.fill_(float("nan"))
    ops.sp_attn(o, q, k, v, kvi, kvn)
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats(dev)["allocation.all.allocated"] == n1, "a new version of known counts must not allocate"
    assert torch.equal(o, want2) and not torch.equal(want, want2)
    # recorded into a graph after the order exists: replays reproduce the eager result
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ops.sp_attn(o, q, k, v, kvi, kvn)         # this stream's own entry, made outside the capture
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        o.fill_(float("nan"))
        with torch.cuda.graph(graph, stream=side):
            ops.sp_attn(o, q, k, v, kvi, kvn)
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(3):
        o.fill_(float("nan"))
        _ = (q.float() @ k.float().transpose(-1, -2)).sum()   # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(o, want2), "replay %d" % rep
