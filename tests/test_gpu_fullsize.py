"""GPU: the benchmark configurations at (or near) full size, checked through properties
that do not need a full-size oracle run: sampled q-blocks against the oracle, agreement of
the two entry points, bitwise repeatability, and the pre-pass round trip."""
import numpy as np
import pytest
import torch

from fgattn_tk_cuda_amd import capi, workloads as wl
from oracle import spattn_oracle as orc
from helpers import assert_close_o, assert_close_stat, f32, to_dev

pytestmark = pytest.mark.gpu


def _oracle_block_rows(q, k, v, bi, bc, b, h, i, qblk, S):
    """Oracle O and lse for q-block i of head (b,h) from its block list (the oracle's own
    softmax on the gathered keys; avoids a full-size oracle call)."""
    D = q.shape[-1]
    blocks = bi[b, h, i, : int(bc[b, h, i])].numpy().astype(np.int64)
    lst = (blocks[:, None] * 64 + np.arange(64)[None]).reshape(-1)
    lst = lst[lst < S]
    r = slice(i * qblk, min(S, (i + 1) * qblk))
    scale = 1.0 / np.sqrt(D)
    s = f32(q[b, h, r]) @ f32(k[b, h])[lst].T
    p, den, m = orc._softmax_rows(s, scale, True)
    return (p @ f32(v[b, h])[lst]) / den[:, None], m * np.float32(scale) + np.log(den)


def test_cfg1_plumbing_case_against_dense_masked_softmax(dev):
    """B=1 H=4 N=1024 d=64, fp32 Q/K/V ~ N(0,1), 64x64 blocks, diagonal + random key blocks up
    to 25 % per q-block row: O = softmax(QK^T / 8 masked to -inf outside the kept blocks) V,
    computed densely in fp32 on the host, against the device kernel (block lists and token
    lists) on the same values rounded to bf16."""
    print("case cfg1 plumbing", flush=True)
    from oracle import cpu_masked_attention as cma

    c = wl.CONFIGS["cfg1_plumbing"]
    B, H, S, D, qblk, kvblk = c["B"], c["H"], c["S"], c["D"], c["qblk"], c["kvblk"]
    q32, k32, v32 = wl.randn_qkv(B, H, S, D, seed=101, dtype=torch.float32)
    q, k, v = q32.bfloat16(), k32.bfloat16(), v32.bfloat16()
    bi, bc = wl.uniform_block_lists(B, H, S, qblk, kvblk, int(round(c["density"] * (S // kvblk))), seed=102)
    qd, kd, vd, bid, bcd = to_dev(dev, q, k, v, bi, bc)
    o = torch.empty_like(qd)
    lse = torch.empty((B, H, S), device=dev)
    capi.sp_attn_blocks(o, qd, kd, vd, bid, bcd, lse=lse, qblk=qblk)
    tok, num = wl.blocks_to_tokens(bi, bc, S)
    o2 = torch.empty_like(qd)
    capi.sp_attn(o2, qd, kd, vd, tok.to(dev), num.to(dev), qblk=qblk)
    torch.cuda.synchronize()
    for h in range(H):
        want = cma.masked_attention_rows(q[0, h].float(), k[0, h].float(), v[0, h].float(), bi[0, h], bc[0, h], 0, S,
                                         qblk, kvblk)
        assert_close_o(f32(o[0, h]), f32(want), "cfg1 block lists, head %d" % h)
        assert_close_o(f32(o2[0, h]), f32(want), "cfg1 token lists, head %d" % h)
        # the bf16 rounding of the inputs is the only difference from the fp32 definition
        want32 = cma.masked_attention_rows(q32[0, h], k32[0, h], v32[0, h], bi[0, h], bc[0, h], 0, S, qblk, kvblk)
        assert np.abs(f32(o[0, h]) - f32(want32)).max() < 6e-2


def test_cfg3_headline_shape(dev):
    """B=2 H=32 N=16384 d=128, 26 of 256 blocks per 64-row q-block."""
    print("case cfg3 full size", flush=True)
    c = wl.CONFIGS["cfg3_sparse_16k"]
    B, H, S, D, qblk = c["B"], c["H"], c["S"], c["D"], c["qblk"]
    q, k, v = wl.randn_qkv(B, H, S, D, seed=0)
    bi, bc = wl.uniform_block_lists(B, H, S, qblk, 64, 26, seed=1)
    qd, kd, vd, bid, bcd = to_dev(dev, q, k, v, bi, bc)
    o = torch.full_like(qd, float("nan"))
    lse = torch.full((B, H, S), float("nan"), device=dev)
    capi.sp_attn_blocks(o, qd, kd, vd, bid, bcd, lse=lse, qblk=qblk)
    torch.cuda.synchronize()
    assert torch.isfinite(o.float()).all() and torch.isfinite(lse).all()
    rng = np.random.default_rng(2)
    for _ in range(12):
        b, h, i = int(rng.integers(B)), int(rng.integers(H)), int(rng.integers(S // qblk))
        wo, wlse = _oracle_block_rows(q, k, v, bi, bc, b, h, i, qblk, S)
        r = slice(i * qblk, (i + 1) * qblk)
        assert_close_o(f32(o[b, h, r]), wo, "cfg3 q-block (%d,%d,%d)" % (b, h, i))
        assert_close_stat(f32(lse[b, h, r]), wlse, "cfg3 lse")
    # bitwise repeatable: no atomics anywhere in the kernel
    o2 = torch.empty_like(o)
    capi.sp_attn_blocks(o2, qd, kd, vd, bid, bcd, qblk=qblk)
    assert torch.equal(o.view(torch.int16), o2.view(torch.int16))
    # the token-list operator on the same lists (one head, to bound the index tensor)
    tok, num = wl.blocks_to_tokens(bi[:1, :1], bc[:1, :1], S)
    o3 = torch.empty_like(qd[:1, :1])
    capi.sp_attn(o3, qd[:1, :1].contiguous(), kd[:1, :1].contiguous(), vd[:1, :1].contiguous(), tok.to(dev), num.to(dev), qblk=qblk)
    assert_close_o(f32(o3), f32(o[:1, :1]), "token path vs block path")


def test_cfg2_dense_shape(dev):
    print("case cfg2 full size", flush=True)
    c = wl.CONFIGS["cfg2_dense"]
    B, H, S, D = c["B"], c["H"], c["S"], c["D"]
    q, k, v = to_dev(dev, *wl.randn_qkv(B, H, S, D, seed=3))
    o = torch.empty_like(q)
    capi.full_attn(o, q, k, v)
    want = torch.nn.functional.scaled_dot_product_attention(q[:, :4].float(), k[:, :4].float(), v[:, :4].float())
    assert_close_o(f32(o[:, :4]), f32(want), "cfg2 vs SDPA")
    want = torch.nn.functional.scaled_dot_product_attention(q[:, 12:].float(), k[:, 12:].float(), v[:, 12:].float())
    assert_close_o(f32(o[:, 12:]), f32(want), "cfg2 vs SDPA (last heads)")


def test_cfg5_zipf_lists(dev):
    """Skewed per-row counts, q-block 128, kv-block 64 (two heads of the 64K configuration's shape, N=16384)."""
    print("case cfg5 zipf", flush=True)
    B, H, S, D, qblk = 1, 2, 16384, 128, 128
    q, k, v = wl.randn_qkv(B, H, S, D, seed=4)
    counts = wl.zipf_counts(B, H, S // qblk, s=1.2, lo=1, hi=256, seed=5)
    bi, bc = wl.ragged_block_lists(B, H, S, qblk, 64, counts, seed=6)
    qd, kd, vd, bid, bcd = to_dev(dev, q, k, v, bi, bc)
    o = torch.full_like(qd, float("nan"))
    lse = torch.full((B, H, S), float("nan"), device=dev)
    capi.sp_attn_blocks(o, qd, kd, vd, bid, bcd, lse=lse, qblk=qblk)
    assert torch.isfinite(o.float()).all()
    order = np.argsort(counts.reshape(-1))
    picks = list(order[:3]) + list(order[-3:]) + list(order[len(order) // 2: len(order) // 2 + 3])
    for flat in picks:
        h, i = divmod(int(flat), S // qblk)
        wo, wlse = _oracle_block_rows(q, k, v, bi, bc, 0, h, i, qblk, S)
        r = slice(i * qblk, (i + 1) * qblk)
        assert_close_o(f32(o[0, h, r]), wo, "zipf q-block (%d,%d) count %d" % (h, i, counts[0, h, i]))
        assert_close_stat(f32(lse[0, h, r]), wlse, "zipf lse")


@pytest.mark.parametrize("clip", [1024, 64])
def test_cfg5_full_size_work_order_changes_nothing(dev, clip):
    """B=1 H=8 N=65536 d=128, 128-row q-blocks, Zipf(1.2) counts in [1,clip] - the configuration's
    literal clip at 1024 blocks (mean 28 % of the keys) and the clip at 64 that gives its stated
    "mean about 3 %": the longest-first work order gives bit-identical O and lse; sampled q-blocks
    against the oracle."""
    print("case cfg5 full size, ordered, clip", clip, flush=True)
    c = wl.CONFIGS["cfg5_zipf_64k"]
    B, H, S, D, qblk = c["B"], c["H"], c["S"], c["D"], c["qblk"]
    assert clip <= c["max_blocks"]
    q, k, v = wl.randn_qkv(B, H, S, D, seed=14)
    counts = wl.zipf_counts(B, H, S // qblk, s=c["zipf_s"], lo=1, hi=clip, seed=15)
    bi, bc = wl.ragged_block_lists(B, H, S, qblk, 64, counts, seed=16)
    qd, kd, vd, bid, bcd = to_dev(dev, q, k, v, bi, bc)
    o1, o2 = torch.empty_like(qd), torch.empty_like(qd)
    l1 = torch.empty((B, H, S), device=dev)
    l2 = torch.empty((B, H, S), device=dev)
    order = torch.empty((bcd.numel(),), dtype=torch.int32, device=dev)
    capi.qblock_order(order, bcd)
    capi.sp_attn_blocks(o1, qd, kd, vd, bid, bcd, lse=l1, qblk=qblk)
    capi.sp_attn_blocks(o2, qd, kd, vd, bid, bcd, lse=l2, qblk=qblk, order=order)
    torch.cuda.synchronize()
    assert np.array_equal(order.cpu().numpy(), orc.qblock_order(counts))
    assert torch.equal(o1, o2) and torch.equal(l1, l2)
    flat = np.argsort(counts.reshape(-1))
    for pick in (flat[0], flat[-1], flat[len(flat) // 2]):
        h, i = divmod(int(pick), S // qblk)
        wo, wlse = _oracle_block_rows(q, k, v, bi, bc, 0, h, i, qblk, S)
        r = slice(i * qblk, (i + 1) * qblk)
        assert_close_o(f32(o2[0, h, r]), wo, "cfg5 q-block (%d,%d) count %d" % (h, i, counts[0, h, i]))
        assert_close_stat(f32(l2[0, h, r]), wlse, "cfg5 lse")


def test_cfg4_shape_topk_generator_sampled_rows(dev):
    """The top-k mask generator at B=1 H=24 N=32760 d=64, 2621 keys per 128-row q-block: sampled
    rows of the score matrix against the oracle, the selection of those rows bit-exact given
    the device's scores, counts and list order everywhere."""
    print("case cfg4 top-k", flush=True)
    c = wl.CONFIGS["cfg4_threshold_padded"]
    B, H, S, D = c["B"], c["H"], c["S"], c["D"]
    q, k, _ = wl.clustered_qkv(B, H, S, D, seed=17)
    SB, Sp, select_k = 256, 32768, int(round(c["keep"] * S))
    stride = 128 * orc.ceil_div(select_k, 128)
    kvi = torch.full((B, H, SB, stride), -7, dtype=torch.int32, device=dev)
    kvn = torch.zeros((B, H, SB), dtype=torch.int32, device=dev)
    score = torch.empty((B, H, SB, Sp), dtype=torch.bfloat16, device=dev)
    qmean = torch.empty((B, H, SB, D), dtype=torch.bfloat16, device=dev)
    capi.qk_topkmask_indices(kvi, kvn, score, qmean, q.to(dev), k.to(dev), select_k, blocksz=128)
    torch.cuda.synchronize()
    assert bool((kvn == select_k).all())
    lists = kvi[..., :select_k]
    assert bool((lists[..., 1:] > lists[..., :-1]).all()) and bool((lists >= 0).all()) and bool((lists < S).all())
    assert bool((kvi[..., select_k:] == -7).all())
    rng = np.random.default_rng(18)
    for h, m in [(int(rng.integers(H)), int(rng.integers(SB))) for _ in range(3)] + [(H - 1, SB - 1)]:
        want_qm, want_sc = orc.qblock_mean_scores(f32(q[:, h:h + 1, m * 128:(m + 1) * 128]), f32(k[:, h:h + 1]), 128)
        assert np.array_equal(f32(qmean[0, h, m]), want_qm[0, 0, 0])
        got = f32(score[0, h, m, :S])
        diff = got != want_sc[0, 0, 0]
        assert diff.mean() < 0.02
        assert np.all(np.abs(got - want_sc[0, 0, 0])[diff] <= np.abs(want_sc[0, 0, 0][diff]) * 2.0 ** -7 + 1e-5)
        assert np.array_equal(kvi[0, h, m, :select_k].cpu().numpy(), orc.topk_select(got[None], select_k)[0])


def test_cfg4_padded_threshold_pipeline(dev):
    """B=1 H=24 N=32760 (padded to 32768), d=64, clustered keys: statistics -> vote mask -> index
    lists -> sparse attention at the full head count.  The lists and counts of all 6144 mask rows
    are compared bit for bit (more rows than one round of the compaction grid), the bit-packed
    route must give the same lists, the other stages are checked on sampled q-blocks."""
    print("case cfg4 padded pipeline", flush=True)
    c = wl.CONFIGS["cfg4_threshold_padded"]
    B, H, S, D = c["B"], c["H"], c["S"], c["D"]
    assert (B, H, S, D) == (1, 24, 32760, 64)
    q, k, v = wl.clustered_qkv(B, H, S, D, seed=7)
    qd, kd, vd = to_dev(dev, q, k, v)
    Sp, SB = 32768, 256
    mx = torch.empty((B, H, 1, Sp), device=dev)
    dn = torch.empty((B, H, 1, Sp), device=dev)
    capi.maxq_denom(mx, dn, qd, kd)
    assert np.all(f32(mx)[..., S:] == 0) and np.all(np.isneginf(f32(dn)[..., S:]))
    rng = np.random.default_rng(8)
    blocks = [(int(rng.integers(H)), int(rng.integers(SB))) for _ in range(4)] + [(0, SB - 1), (H - 1, SB - 1)]   # incl. the ragged block
    kf = f32(k)
    for h, i in blocks:
        r = slice(i * 128, min(S, (i + 1) * 128))
        s = f32(q[0, h, r]) @ kf[0, h].T
        m = s.max(1)
        d = np.exp2((s - m[:, None]) * (orc.LOG2E / 8.0)).sum(1)
        assert_close_stat(f32(mx)[0, h, 0, r], m, "max_q", atol=1e-3)
        assert_close_stat(f32(dn)[0, h, 0, r], d, "denom")
    # threshold: keep about 8 % of the (q-block, 64-key block) pairs, from sampled q-blocks of three heads
    samp = []
    for h in (0, 11, 23):
        for i in range(0, SB, 32):
            r = slice(i * 128, min(S, (i + 1) * 128))
            s = f32(q[0, h, r]) @ kf[0, h].T
            p = np.exp2((s - f32(mx)[0, h, 0, r, None]) * (orc.LOG2E / 8.0)) / f32(dn)[0, h, 0, r, None]
            pm = np.concatenate([p.max(0), np.zeros(Sp - S, np.float32)]).reshape(-1, 64).max(1)
            samp.append(pm)
    thr = float(np.quantile(np.concatenate(samp), 0.92))
    mask = torch.zeros((B, H, SB, Sp), dtype=torch.int32, device=dev)
    capi.booleanmask_128(mask, mx, dn, qd, kd, thr)
    kvi = torch.full((B, H, SB, Sp), Sp, dtype=torch.int32, device=dev)
    kvn = torch.zeros((B, H, SB), dtype=torch.int32, device=dev)
    capi.booleanmask_to_indexmask(kvi, kvn, mask, S)
    # the bit-packed route (mask cache) over the same 6144 rows
    packed = torch.empty((B, H, SB, Sp // 8), dtype=torch.uint8, device=dev)
    capi.pack_mask(packed, mask)
    kvi2 = torch.full((B, H, SB, Sp), Sp, dtype=torch.int32, device=dev)
    kvn2 = torch.zeros((B, H, SB), dtype=torch.int32, device=dev)
    capi.packedmask_to_indexmask(kvi2, kvn2, packed, S)
    assert torch.equal(kvi, kvi2) and torch.equal(kvn, kvn2)
    del kvi2, kvn2
    assert int(mask.min()) >= 0 and int(mask.max()) <= 8 and not bool(mask[..., S:].any())
    blockmask = (mask > 0).view(B, H, SB, Sp // 64, 64).any(-1)
    dens = float(blockmask.float().mean())
    assert 0.06 < dens < 0.10, dens
    per_head = blockmask.float().mean(dim=(0, 2, 3)).cpu().numpy()
    assert per_head.min() > 0.04 and per_head.max() < 0.12, per_head
    # all 6144 rows: counts, ascending lists, fill, bit for bit against the plain loop
    mh = mask.cpu().numpy()
    assert np.array_equal(np.unpackbits(packed.cpu().numpy(), axis=-1, bitorder="little"), (mh > 0).astype(np.uint8))
    wi, wn = orc.booleanmask_to_indexmask(mh, S)
    assert np.array_equal(kvn.cpu().numpy(), wn) and np.array_equal(kvi.cpu().numpy(), wi)
    assert np.array_equal(orc.block_mask_from_votes(mh[:, :2], S), blockmask[:, :2, :, : orc.ceil_div(S, 64)].cpu().numpy())
    for h, i in blocks:
        r = slice(i * 128, min(S, (i + 1) * 128))
        s = f32(q[0, h, r]) @ kf[0, h].T
        p = np.exp2((s - f32(mx)[0, h, 0, r, None]) * (orc.LOG2E / 8.0)) / f32(dn)[0, h, 0, r, None]
        pmax = p.max(0)
        near = np.abs(pmax - thr) <= 1e-2 * thr
        assert np.array_equal((mh[0, h, i, :S] > 0) | near, (pmax > thr) | near), "mask row (%d,%d)" % (h, i)
    del mh
    # block route: the sweep with bit outputs equals the packed vote mask; block lists from the bits
    # and from the votes agree with each other and with the plain loop over the device's mask
    pk128 = torch.full_like(packed, 0xA5)
    capi.booleanmask_packed(pk128, mx, dn, qd, kd, thr, qblk=128)
    assert torch.equal(pk128, packed)
    nb = Sp // 64
    bi = torch.full((B, H, SB, nb), -1, dtype=torch.int32, device=dev)
    bc = torch.zeros((B, H, SB), dtype=torch.int32, device=dev)
    bm = torch.empty((B, H, SB, nb), dtype=torch.uint8, device=dev)
    capi.packedmask_to_blocklists(bi, bc, pk128, S, blockmask=bm)
    bi2 = torch.full_like(bi, -1)
    bc2 = torch.zeros_like(bc)
    capi.booleanmask_to_blocklists(bi2, bc2, mask, S)
    assert torch.equal(bi, bi2) and torch.equal(bc, bc2)
    assert torch.equal(bm.bool(), blockmask)
    assert torch.equal(bc, blockmask.sum(-1).int())
    ar = torch.arange(nb, device=dev, dtype=torch.int32)
    want_bi = torch.where(blockmask, ar, torch.full_like(ar, 1 << 20)).sort(-1).values
    want_bi = torch.where(want_bi == (1 << 20), torch.full_like(want_bi, -1), want_bi)
    assert torch.equal(bi, want_bi)
    # 64-row q-blocks: two bit rows per 128-row block that OR to it; block lists of 12288 rows
    n64 = orc.ceil_div(S, 64)
    pk64 = torch.full((B, H, n64, Sp // 8), 0xA5, dtype=torch.uint8, device=dev)
    capi.booleanmask_packed(pk64, mx, dn, qd, kd, thr, qblk=64)
    assert torch.equal(pk64[:, :, 0::2] | pk64[:, :, 1::2], packed)
    bi64 = torch.full((B, H, n64, nb), -1, dtype=torch.int32, device=dev)
    bc64 = torch.zeros((B, H, n64), dtype=torch.int32, device=dev)
    capi.packedmask_to_blocklists(bi64, bc64, pk64, S)
    dens64 = float(bc64.float().mean()) / orc.ceil_div(S, 64)
    assert 0.03 < dens64 < dens, (dens64, dens)
    bits64 = pk64.cpu().numpy()
    for h, i in blocks:
        for half in (0, 1):
            r = slice(i * 128 + 64 * half, min(S, i * 128 + 64 * half + 64))
            if r.start >= S:
                continue
            s = f32(q[0, h, r]) @ kf[0, h].T
            p = np.exp2((s - f32(mx)[0, h, 0, r, None]) * (orc.LOG2E / 8.0)) / f32(dn)[0, h, 0, r, None]
            pmax = p.max(0)
            near = np.abs(pmax - thr) <= 1e-2 * thr
            got = np.unpackbits(bits64[0, h, 2 * i + half], bitorder="little")[:S].astype(bool)
            assert np.array_equal(got | near, (pmax > thr) | near), "64-row bits (%d,%d,%d)" % (h, i, half)
            lst = bi64[0, h, 2 * i + half, : int(bc64[0, h, 2 * i + half])].cpu().numpy()
            assert np.array_equal(lst, np.flatnonzero(np.pad(got, (0, nb * 64 - S)).reshape(nb, 64).any(1)))
    del pk64, bits64, pk128, packed, mask
    ob = torch.full_like(qd, float("nan"))
    capi.sp_attn_blocks(ob, qd, kd, vd, bi, bc, qblk=128)
    ob64 = torch.full_like(qd, float("nan"))
    capi.sp_attn_blocks(ob64, qd, kd, vd, bi64, bc64, qblk=64)
    assert torch.isfinite(ob.float()).all() and torch.isfinite(ob64.float()).all()
    vf = f32(v)
    bih, bch, bi64h, bc64h = bi.cpu().numpy(), bc.cpu().numpy(), bi64.cpu().numpy(), bc64.cpu().numpy()
    for h, i in blocks:
        r = slice(i * 128, min(S, (i + 1) * 128))
        tok, num = orc.block_list_to_token_list(bih[:, h:h + 1, i:i + 1], bch[:, h:h + 1, i:i + 1], S)
        lst = tok[0, 0, 0, : num[0, 0, 0]]
        pp, den, _ = orc._softmax_rows(f32(q[0, h, r]) @ kf[0, h, lst].T, 0.125, True)
        assert_close_o(f32(ob[0, h, r]), (pp @ vf[0, h, lst]) / den[:, None], "cfg4 block rows (%d,%d)" % (h, i))
        for half in (0, 1):
            r = slice(i * 128 + 64 * half, min(S, i * 128 + 64 * half + 64))
            if r.start >= S:
                continue
            j = 2 * i + half
            tok, num = orc.block_list_to_token_list(bi64h[:, h:h + 1, j:j + 1], bc64h[:, h:h + 1, j:j + 1], S)
            lst = tok[0, 0, 0, : num[0, 0, 0]]
            if lst.size == 0:          # a q-block without a key: zeros
                assert not f32(ob64[0, h, r]).any()
                continue
            pp, den, _ = orc._softmax_rows(f32(q[0, h, r]) @ kf[0, h, lst].T, 0.125, True)
            assert_close_o(f32(ob64[0, h, r]), (pp @ vf[0, h, lst]) / den[:, None], "cfg4 block rows q64 (%d,%d)" % (h, j))
    del ob, ob64
    o = torch.full_like(qd, float("nan"))
    capi.sp_attn(o, qd, kd, vd, kvi, kvn)
    assert torch.isfinite(o.float()).all()
    vf = f32(v)
    for h, i in blocks:
        r = slice(i * 128, min(S, (i + 1) * 128))
        lst = wi[0, h, i, : wn[0, h, i]]
        s = f32(q[0, h, r]) @ kf[0, h, lst].T
        pp, den, _ = orc._softmax_rows(s, 0.125, True)
        assert_close_o(f32(o[0, h, r]), (pp @ vf[0, h, lst]) / den[:, None], "cfg4 sparse rows (%d,%d)" % (h, i))


def test_cfg4_block_maxima_route(dev):
    """cfg 4 at its size through the one-sweep block route: maxq_denom with the per-(row, key
    block) maxima (0.8 GB as bf16, rounded up), their threshold into block masks and lists for 128- and 64-row
    q-blocks (6144 / 12288 rows, every one compared with the same test done by torch on the
    device's own maxima), density, agreement with the per-key oracle on sampled q-blocks, and
    block-list attention over the result."""
    print("case cfg4 block maxima", flush=True)
    c = wl.CONFIGS["cfg4_threshold_padded"]
    B, H, S, D = c["B"], c["H"], c["S"], c["D"]
    q, k, v = wl.clustered_qkv(B, H, S, D, seed=7)
    qd, kd, vd = to_dev(dev, q, k, v)
    Sp, nb = 32768, 512
    sf = np.float32(orc.LOG2E / 8.0)
    mx, dn, mx0, dn0 = (torch.empty((B, H, 1, Sp), device=dev) for _ in range(4))
    bmx = torch.full((B, H, nb, Sp), float("nan"), dtype=torch.bfloat16, device=dev)
    capi.maxq_denom(mx0, dn0, qd, kd)
    capi.maxq_denom_blockmax(mx, dn, bmx, qd, kd)
    assert torch.equal(mx, mx0) and torch.equal(dn, dn0)
    del mx0, dn0
    assert torch.isfinite(bmx[..., :S]).all()
    # the largest stored maximum of a row is its max_q rounded up to bf16: not below it, less than a step above
    top = bmx[..., :S].max(dim=2).values.float()
    mrow = mx.view(B, H, Sp)[..., :S]
    assert bool((top >= mrow).all()) and bool((top <= mrow + mrow.abs() * 2.0 ** -7).all())
    assert torch.equal(top.cpu(), torch.from_numpy(orc.bf16_round_up(f32(mrow))))
    kf = f32(k)
    rng = np.random.default_rng(8)
    blocks = [(int(rng.integers(H)), int(rng.integers(256))) for _ in range(4)] + [(0, 255), (H - 1, 255)]
    samp = []
    for h, i in blocks + [(h, i) for h in (0, 11, 23) for i in range(0, 256, 32)]:
        r = slice(i * 128, min(S, (i + 1) * 128))
        s = f32(q[0, h, r]) @ kf[0, h].T
        sb = np.concatenate([s, np.full((s.shape[0], Sp - S), -np.inf, np.float32)], axis=1).reshape(s.shape[0], nb, 64).max(-1)
        got = f32(bmx[0, h, :, r]).T
        tol = 1e-3 + 1e-4 * np.abs(sb)
        assert np.all(got >= sb - tol) and np.all(got <= sb + tol + 2.0 ** -7 * np.abs(sb)), "blockmax (%d,%d)" % (h, i)
        p = np.exp2((s - f32(mx)[0, h, 0, r, None]) * sf) / f32(dn)[0, h, 0, r, None]
        samp.append(np.concatenate([p.max(0), np.zeros(Sp - S, np.float32)]).reshape(-1, 64).max(1))
    thr = float(np.quantile(np.concatenate(samp[len(blocks):]), 0.92))
    # what the threshold of the maxima must give, by torch on the device's own numbers
    t = (np.float32(np.log2(thr)) + (mx.view(B, H, Sp) * float(sf) + torch.log2(dn.view(B, H, Sp)))) / float(sf)
    t[..., S:] = float("inf")
    margin = (bmx.float() - t[:, :, None, :]) * float(sf)
    margin[..., S:] = float("-inf")
    lists = {}
    for qblk in (128, 64):
        nq = orc.ceil_div(S, qblk)
        mg = margin.view(B, H, nb, Sp // qblk, qblk)[:, :, :, :nq]
        want = (mg > 0).any(-1).transpose(2, 3)
        near = (mg.abs() <= 1e-4).any(-1).transpose(2, 3)
        bi = torch.full((B, H, nq, nb), -1, dtype=torch.int32, device=dev)
        bc = torch.full((B, H, nq), -3, dtype=torch.int32, device=dev)
        bm = torch.full((B, H, nq, nb), 9, dtype=torch.uint8, device=dev)
        capi.blockmax_to_blocklists(bi, bc, bmx, mx, dn, thr, S, D, qblk=qblk, blockmask=bm)
        assert int(bm.max()) <= 1
        got = bm.bool()
        assert torch.equal(got | near, want | near) and float(near.float().mean()) < 1e-3
        assert torch.equal(bc, got.sum(-1).int())
        ar = torch.arange(nb, device=dev, dtype=torch.int32)
        want_bi = torch.where(got, ar, torch.full_like(ar, 1 << 20)).sort(-1).values
        assert torch.equal(bi, torch.where(want_bi == (1 << 20), torch.full_like(want_bi, -1), want_bi))
        lists[qblk] = (bi, bc, got)
        del mg, want, near, bm, want_bi
    del margin, t
    dens = float(lists[128][2].float().mean())
    assert 0.06 < dens < 0.10, dens
    assert 0.03 < float(lists[64][2].float().mean()) < dens
    # the per-key oracle on the sampled q-blocks: every block it keeps is listed, and the lists equal it
    # outside the threshold band widened downwards by one bf16 step of the largest stored maximum
    lift = float(np.exp2(2.0 ** -7 * float(bmx[..., :S].float().abs().max()) * float(sf)))
    assert 1.0 < lift < 1.2
    for (h, i), pb in zip(blocks, samp):
        band = (pb >= thr * (1 - 1e-2) / lift) & (pb <= thr * (1 + 1e-2))
        got_row = lists[128][2][0, h, i].cpu().numpy()
        assert not ((pb > thr) & ~got_row & ~band).any(), "block row (%d,%d): a kept block is missing" % (h, i)
        assert np.array_equal(got_row | band, (pb > thr) | band), "block row (%d,%d)" % (h, i)
    vf = f32(v)
    for qblk in (128, 64):
        bi, bc, _ = lists[qblk]
        o = torch.full_like(qd, float("nan"))
        capi.sp_attn_blocks(o, qd, kd, vd, bi, bc, qblk=qblk)
        assert torch.isfinite(o.float()).all()
        bih, bch = bi.cpu().numpy(), bc.cpu().numpy()
        for h, i in blocks[:3] + blocks[-1:]:
            j = i * (128 // qblk)
            r = slice(j * qblk, min(S, (j + 1) * qblk))
            tok, num = orc.block_list_to_token_list(bih[:, h:h + 1, j:j + 1], bch[:, h:h + 1, j:j + 1], S)
            lst = tok[0, 0, 0, : num[0, 0, 0]]
            if lst.size == 0:
                assert not f32(o[0, h, r]).any()
                continue
            pp, den, _ = orc._softmax_rows(f32(q[0, h, r]) @ kf[0, h, lst].T, 0.125, True)
            assert_close_o(f32(o[0, h, r]), (pp @ vf[0, h, lst]) / den[:, None], "cfg4 blockmax route q%d (%d,%d)" % (qblk, h, j))
    # the threshold sweep over the listed blocks only gives the votes of the full sweep, bit for bit,
    # as int32 and as bits, and the key lists of both are the same
    print("case cfg4 block-restricted threshold sweep", flush=True)
    del bmx, o
    SB = Sp // 128
    bi, bc, _ = lists[128]
    full = torch.full((B, H, SB, Sp), 7, dtype=torch.int32, device=dev)
    part = torch.full((B, H, SB, Sp), 7, dtype=torch.int32, device=dev)
    capi.booleanmask_128(full, mx, dn, qd, kd, thr)
    capi.booleanmask_128_blocks(part, mx, dn, qd, kd, thr, bi, bc)
    assert torch.equal(full, part)
    assert 0 < int(full.count_nonzero()) < full.numel() // 50
    for qblk in (128, 64):
        nq = orc.ceil_div(S, qblk)
        pf = torch.full((B, H, nq, Sp // 8), 0xA5, dtype=torch.uint8, device=dev)
        pp_ = torch.full((B, H, nq, Sp // 8), 0xA5, dtype=torch.uint8, device=dev)
        capi.booleanmask_packed(pf, mx, dn, qd, kd, thr, qblk=qblk)
        capi.booleanmask_packed_blocks(pp_, mx, dn, qd, kd, thr, bi, bc, qblk=qblk)
        assert torch.equal(pf, pp_), "packed votes, q-blocks of %d" % qblk
    kvi_f = torch.full((B, H, SB, Sp), -5, dtype=torch.int32, device=dev)
    kvi_p = torch.full((B, H, SB, Sp), -5, dtype=torch.int32, device=dev)
    kvn_f, kvn_p = (torch.full((B, H, SB), -5, dtype=torch.int32, device=dev) for _ in range(2))
    capi.booleanmask_to_indexmask(kvi_f, kvn_f, full, S)
    del full
    pk = torch.empty((B, H, SB, Sp // 8), dtype=torch.uint8, device=dev)
    capi.booleanmask_packed_blocks(pk, mx, dn, qd, kd, thr, bi, bc, qblk=128)
    capi.packedmask_to_indexmask(kvi_p, kvn_p, pk, S)
    assert torch.equal(kvn_f, kvn_p)
    ar = torch.arange(Sp, device=dev, dtype=torch.int32)
    live = ar[None, None, None, :] < kvn_f[..., None]
    assert torch.equal(torch.where(live, kvi_f, 0), torch.where(live, kvi_p, 0))


def test_reference_shape_75856_with_its_kv_length(dev):
    """The largest shape the reference compiles, B=1 H=24 S=75856 d=128, with the kv length it
    hard-codes for it (75856 - 245, python/cuda_attn.cu:28-31): dense attention, fused statistics,
    the threshold pre-pass and sparse attention over its lists, sampled q-blocks against the
    oracle.  Keys 75611.. must not contribute anywhere."""
    print("case reference shape 75856", flush=True)
    B, H, S, D, kv = 1, 24, 75856, 128, 75856 - 245
    g = torch.Generator(device=dev).manual_seed(5)
    q, k, v = (torch.randn((B, H, S, D), generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16) for _ in range(3))
    k[:, :, kv:] = 50.0      # keys behind the kv length would dominate every row if they were read
    v[:, :, kv:] = -50.0
    Sp, SB = orc.padded_len(S), orc.ceil_div(S, 128)
    sf = np.float32(orc.LOG2E / np.sqrt(D))
    o = torch.full_like(q, float("nan"))
    lse = torch.full((B, H, S), float("nan"), device=dev)
    capi.full_attn(o, q, k, v, lse=lse, kv_len=kv)
    o2 = torch.full_like(q, float("nan"))
    mx = torch.full((B, H, 1, Sp), float("nan"), device=dev)
    dn = torch.full((B, H, 1, Sp), float("nan"), device=dev)
    capi.fullattn_maxq_denom(o2, mx, dn, q, k, v, kv_len=kv)
    assert torch.isfinite(o.float()).all() and torch.isfinite(o2.float()).all()
    rng = np.random.default_rng(6)
    blocks = [(int(rng.integers(H)), int(rng.integers(SB))) for _ in range(3)] + [(H - 1, SB - 1), (0, kv // 128)]
    per = {}
    for h, i in blocks:
        r = slice(i * 128, min(S, (i + 1) * 128))
        qh, kh, vh = f32(q[0, h, r]), f32(k[0, h, :kv]), f32(v[0, h, :kv])
        s = qh @ kh.T
        m = s.max(1)
        p = np.exp2((s - m[:, None]) * sf)
        d = p.sum(1)
        want = (orc.bf16_round(p) @ vh) / d[:, None]
        assert_close_o(f32(o[0, h, r]), want, "full_attn rows (%d,%d)" % (h, i))
        assert_close_o(f32(o2[0, h, r]), want, "fullattn_maxq_denom rows (%d,%d)" % (h, i))
        assert_close_stat(f32(lse[0, h, r]), (m * sf + np.log2(d)) * np.float32(np.log(2.0)), "lse", atol=1e-3)
        assert_close_stat(f32(mx)[0, h, 0, r], m, "max_q", atol=1e-3)
        assert_close_stat(f32(dn)[0, h, 0, r], d, "denom")
        per[(h, i)] = (p / d[:, None]).max(0)
    del o2
    thr = float(np.quantile(np.concatenate(list(per.values())), 0.98))
    mask = torch.zeros((B, H, SB, Sp), dtype=torch.int32, device=dev)
    capi.booleanmask_128(mask, mx, dn, q, k, thr, kv_len=kv)
    assert not bool(mask[..., kv:].any())
    kvi = torch.full((B, H, SB, Sp), Sp, dtype=torch.int32, device=dev)
    kvn = torch.zeros((B, H, SB), dtype=torch.int32, device=dev)
    capi.booleanmask_to_indexmask(kvi, kvn, mask, kv)
    assert torch.equal(kvn, (mask > 0).sum(-1).int()) and int(kvn.max()) <= kv
    for (h, i), pmax in per.items():
        near = np.abs(pmax - thr) <= 1e-2 * thr
        got = mask[0, h, i, :kv].cpu().numpy() > 0
        assert np.array_equal(got | near, (pmax > thr) | near), "mask row (%d,%d)" % (h, i)
        n = int(kvn[0, h, i])
        assert np.array_equal(kvi[0, h, i, :n].cpu().numpy(), np.flatnonzero(got))
    del mask
    o3 = torch.full_like(q, float("nan"))
    capi.sp_attn(o3, q, k, v, kvi, kvn, kv_len=kv)
    assert torch.isfinite(o3.float()).all()
    for h, i in blocks:
        r = slice(i * 128, min(S, (i + 1) * 128))
        lst = kvi[0, h, i, : int(kvn[0, h, i])].cpu().numpy()
        if lst.size == 0:
            assert not f32(o3[0, h, r]).any()
            continue
        pp, den, _ = orc._softmax_rows(f32(q[0, h, r]) @ f32(k[0, h])[lst].T, 1.0 / np.sqrt(D), True)
        assert_close_o(f32(o3[0, h, r]), (pp @ f32(v[0, h])[lst]) / den[:, None], "sp_attn rows (%d,%d)" % (h, i))
    # the same key lists through one full sweep: statistics with block maxima (4.3 GB at this shape), blocks
    # a little below the threshold, the vote sweep over those blocks as bits, key lists from the bits
    print("case reference shape 75856, one sweep", flush=True)
    del o3
    nb = Sp // 64
    bmx = torch.empty((B, H, nb, Sp), dtype=torch.bfloat16, device=dev)
    mx1 = torch.full((B, H, 1, Sp), float("nan"), device=dev)
    dn1 = torch.full((B, H, 1, Sp), float("nan"), device=dev)
    capi.maxq_denom_blockmax(mx1, dn1, bmx, q, k, kv_len=kv)
    assert torch.equal(mx1[..., :S], mx[..., :S]) and torch.equal(dn1[..., :S], dn[..., :S])
    bi = torch.full((B, H, SB, nb), -1, dtype=torch.int32, device=dev)
    bc = torch.zeros((B, H, SB), dtype=torch.int32, device=dev)
    capi.blockmax_to_blocklists(bi, bc, bmx, mx, dn, thr * (1.0 - 1e-3), S, D, qblk=128, kv_len=kv)
    del bmx
    assert 0 < int(bc.sum()) < bc.numel() * orc.ceil_div(kv, 64)      # unclustered keys: most blocks hold a passing key
    pk = torch.full((B, H, SB, Sp // 8), 0xA5, dtype=torch.uint8, device=dev)
    capi.booleanmask_packed_blocks(pk, mx, dn, q, k, thr, bi, bc, qblk=128, kv_len=kv)
    kvi1 = torch.full((B, H, SB, Sp), Sp, dtype=torch.int32, device=dev)
    kvn1 = torch.zeros((B, H, SB), dtype=torch.int32, device=dev)
    capi.packedmask_to_indexmask(kvi1, kvn1, pk, kv)
    assert torch.equal(kvn1, kvn) and torch.equal(kvi1, kvi)
