"""Seeded random shapes for the dense kernels and the pre-pass, against the CPU oracle.

Same checks as the hand-written cases of test_gpu_attention.py / test_gpu_prepass.py /
test_gpu_topk.py, on shapes drawn per seed: sequence lengths that are not multiples of any tile,
kv lengths from one key up, both head dims, masks with runs and bursts.
"""
import numpy as np
import pytest
import torch

from fgattn_tk_cuda_amd import capi, workloads as wl
from oracle import spattn_oracle as orc
from helpers import assert_close_o, assert_close_stat, f32, to_dev

pytestmark = pytest.mark.gpu

BAND = 1e-2   # relative band around the threshold inside which a vote may flip


@pytest.mark.parametrize("seed", range(16))
def test_dense_attention_and_statistics_random(dev, seed):
    rng = np.random.default_rng(3000 + seed)
    B, H = int(rng.integers(1, 3)), int(rng.integers(1, 4))
    S = int(rng.choice([1, 31, 64, 65, 127, 129, 200, 333, 512, 641]))
    D = int(rng.choice([64, 128]))
    kv_len = int(rng.choice([0, S, int(rng.integers(1, S + 1))]))
    kv = kv_len or S
    print("case random dense", seed, B, H, S, D, kv_len, flush=True)
    q, k, v = wl.randn_qkv(B, H, S, D, seed=seed)
    qd, kd, vd = to_dev(dev, q, k, v)
    want = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float()[:, :, :kv], v.float()[:, :, :kv])
    o = torch.full_like(qd, float("nan"))
    lse = torch.full(q.shape[:3], float("nan"), device=dev)
    capi.full_attn(o, qd, kd, vd, lse=lse, kv_len=kv_len)
    assert_close_o(f32(o), f32(want), "full_attn vs SDPA")
    s = torch.einsum("bhmd,bhnd->bhmn", q.float(), k.float()[:, :, :kv]) / D ** 0.5
    assert_close_stat(f32(lse), f32(torch.logsumexp(s, -1)), "lse", atol=1e-3)
    Sp = orc.padded_len(S)
    wmx, wdn = orc.maxq_denom(f32(q), f32(k), kv_len=kv)
    o2 = torch.full_like(qd, float("nan"))
    mx = torch.full((B, H, 1, Sp), float("nan"), device=dev)
    dn = torch.full((B, H, 1, Sp), float("nan"), device=dev)
    capi.fullattn_maxq_denom(o2, mx, dn, qd, kd, vd, kv_len=kv_len)
    assert_close_o(f32(o2), f32(want), "fullattn_maxq_denom O")
    assert_close_stat(f32(mx), wmx, "max_q (fused)", atol=1e-4)
    assert_close_stat(f32(dn), wdn, "denom (fused)")
    mx2 = torch.full((B, H, 1, Sp), float("nan"), device=dev)
    dn2 = torch.full((B, H, 1, Sp), float("nan"), device=dev)
    capi.maxq_denom(mx2, dn2, qd, kd, kv_len=kv_len)
    assert_close_stat(f32(mx2), wmx, "max_q", atol=1e-4)
    assert_close_stat(f32(dn2), wdn, "denom")
    assert np.all(f32(mx2)[..., S:] == 0) and np.all(np.isneginf(f32(dn2)[..., S:]))


@pytest.mark.parametrize("seed", range(10))
def test_vote_mask_random(dev, seed):
    rng = np.random.default_rng(4000 + seed)
    B, H = 1, int(rng.integers(1, 4))
    S = int(rng.choice([129, 200, 384, 500, 777, 1025]))
    D = int(rng.choice([64, 128]))
    kv_len = int(rng.choice([0, int(rng.integers(65, S + 1))]))
    kv = kv_len or S
    print("case random vote mask", seed, H, S, D, kv_len, flush=True)
    q, k, _ = wl.clustered_qkv(B, H, S, D, seed=seed, sigma=0.7)
    qd, kd = to_dev(dev, q, k)
    Sp = orc.padded_len(S)
    SB = Sp // 128
    mx = torch.empty((B, H, 1, Sp), device=dev)
    dn = torch.empty((B, H, 1, Sp), device=dev)
    capi.maxq_denom(mx, dn, qd, kd, kv_len=kv_len)
    _, pmax0 = orc.booleanmask_128(f32(mx), f32(dn), f32(q), f32(k), 1.0, kv_len=kv)
    thr = float(np.quantile(pmax0, float(rng.choice([0.3, 0.7, 0.95]))))
    mask = torch.full((B, H, SB, Sp), -7, dtype=torch.int32, device=dev)
    capi.booleanmask_128(mask, mx, dn, qd, kd, thr, kv_len=kv_len)
    got = mask.cpu().numpy()
    votes, pmax = orc.booleanmask_128(f32(mx), f32(dn), f32(q), f32(k), thr, kv_len=kv)
    assert got.min() >= 0 and got.max() <= 8
    assert np.all(got[..., kv:] == 0)
    near = np.abs(pmax - thr) <= BAND * thr
    dis = ((got[..., :kv] > 0) != (votes[..., :kv] > 0)) & ~near
    assert dis.sum() == 0, "%d mask mismatches outside the threshold band" % dis.sum()
    assert (got[..., :kv] == votes[..., :kv]).mean() > 0.995
    # and the lists made from the device's own mask, bit for bit
    kvi = torch.full((B, H, SB, Sp), Sp, dtype=torch.int32, device=dev)
    kvn = torch.full((B, H, SB), -1, dtype=torch.int32, device=dev)
    capi.booleanmask_to_indexmask(kvi, kvn, mask, kv)
    wi, wn = orc.booleanmask_to_indexmask(got, kv)
    assert np.array_equal(kvn.cpu().numpy(), wn) and np.array_equal(kvi.cpu().numpy(), wi)


@pytest.mark.parametrize("seed", range(16))
def test_compaction_and_packing_random(dev, seed):
    rng = np.random.default_rng(5000 + seed)
    B, H, SB = int(rng.integers(1, 3)), int(rng.integers(1, 4)), int(rng.integers(1, 6))
    ms = 128 * int(rng.choice([1, 2, 3, 7, 16, 33, 65, 130]))
    seq = int(rng.choice([0, 1, ms, ms - 1, int(rng.integers(0, ms + 1))]))
    density = float(rng.choice([0.0, 0.01, 0.08, 0.5, 1.0]))
    print("case random compaction", seed, B, H, SB, ms, seq, density, flush=True)
    mask = (rng.random((B, H, SB, ms)) < density).astype(np.int32) * rng.integers(1, 9, size=(B, H, SB, ms), dtype=np.int32)
    # runs: whole stretches kept or dropped
    for _ in range(int(rng.integers(0, 6))):
        a = int(rng.integers(0, ms))
        b = min(ms, a + int(rng.integers(1, 400)))
        mask[int(rng.integers(B)), int(rng.integers(H)), int(rng.integers(SB)), a:b] = int(rng.integers(0, 2)) * 3
    md = torch.from_numpy(mask).to(dev)
    kvi = torch.full((B, H, SB, ms), ms, dtype=torch.int32, device=dev)
    kvn = torch.full((B, H, SB), -1, dtype=torch.int32, device=dev)
    capi.booleanmask_to_indexmask(kvi, kvn, md, seq)
    wi, wn = orc.booleanmask_to_indexmask(mask, seq)
    assert np.array_equal(kvn.cpu().numpy(), wn)
    assert np.array_equal(kvi.cpu().numpy(), wi)
    packed = torch.full((B, H, SB, ms // 8), 0xA5, dtype=torch.uint8, device=dev)
    capi.pack_mask(packed, md)
    assert np.array_equal(packed.cpu().numpy(), orc.pack_mask(mask))
    kvi2 = torch.full((B, H, SB, ms), ms, dtype=torch.int32, device=dev)
    kvn2 = torch.full((B, H, SB), -1, dtype=torch.int32, device=dev)
    capi.packedmask_to_indexmask(kvi2, kvn2, packed, seq)
    assert torch.equal(kvi, kvi2) and torch.equal(kvn, kvn2)


@pytest.mark.parametrize("seed", range(12))
def test_topk_generator_random(dev, seed):
    rng = np.random.default_rng(6000 + seed)
    B, H = int(rng.integers(1, 3)), int(rng.integers(1, 4))
    S = int(rng.choice([130, 257, 640, 1000, 1500, 2300]))
    D = int(rng.choice([64, 128]))
    blk = int(rng.choice([64, 128]))
    kv_len = int(rng.choice([0, int(rng.integers(1, S + 1))]))
    kv = kv_len or S
    select_k = int(rng.choice([1, 7, 128, int(rng.integers(1, S + 1)), S + 5]))
    print("case random topk", seed, B, H, S, D, blk, kv_len, select_k, flush=True)
    q, k, _ = wl.randn_qkv(B, H, S, D, seed=seed)
    SB = orc.ceil_div(S, blk)
    idx_stride = 128 * orc.ceil_div(min(select_k, kv), 128)
    score_stride = orc.padded_len(S)
    fill = -7
    kvi = torch.full((B, H, SB, idx_stride), fill, dtype=torch.int32, device=dev)
    kvn = torch.full((B, H, SB), -1, dtype=torch.int32, device=dev)
    score = torch.full((B, H, SB, score_stride), float("nan"), dtype=torch.bfloat16, device=dev)
    qmean = torch.full((B, H, SB, D), float("nan"), dtype=torch.bfloat16, device=dev)
    capi.qk_topkmask_indices(kvi, kvn, score, qmean, q.to(dev), k.to(dev), select_k, blocksz=blk, kv_len=kv_len)
    torch.cuda.synchronize()
    kvi, kvn, score, qmean = kvi.cpu().numpy(), kvn.cpu().numpy(), f32(score), f32(qmean)
    want_qm, want_sc = orc.qblock_mean_scores(f32(q), f32(k), blk)
    assert np.array_equal(qmean, want_qm)
    got_sc = score[..., :kv]
    assert np.isfinite(got_sc).all()
    diff = got_sc != want_sc[..., :kv]
    assert diff.mean() < 0.02
    assert np.all(np.abs(got_sc - want_sc[..., :kv])[diff] <= np.abs(want_sc[..., :kv][diff]) * 2.0 ** -7 + 1e-5)
    kk = min(select_k, kv)
    want_sel = orc.topk_select(got_sc, select_k)
    assert np.all(kvn == kk)
    assert np.array_equal(kvi[..., :kk], want_sel)
    assert np.all(kvi[..., kk:] == fill)


@pytest.mark.parametrize("seed", range(12))
def test_block_maxima_route_random(dev, seed):
    """The one-sweep block route on drawn shapes (from one query row and one key up): block maxima
    against the oracle, their maximum over the blocks equal to max_q, the thresholded block mask
    against the threshold of the device's own maxima and against the per-key oracle outside the
    band, lists = the mask, for both q-block sizes."""
    rng = np.random.default_rng(9000 + seed)
    B, H = int(rng.integers(1, 3)), int(rng.integers(1, 4))
    S = int(rng.choice([1, 31, 64, 65, 127, 129, 200, 333, 512, 641, 900]))
    D = int(rng.choice([64, 128]))
    kv_len = int(rng.choice([0, S, int(rng.integers(1, S + 1))]))
    kv = kv_len or S
    with_v = bool(rng.integers(2))
    print("case random blockmax", seed, B, H, S, D, kv_len, with_v, flush=True)
    q, k, v = wl.clustered_qkv(B, H, S, D, seed=seed, sigma=0.8)
    qd, kd, vd = to_dev(dev, q, k, v)
    Sp = orc.padded_len(S)
    nb, nkb = Sp // 64, orc.ceil_div(kv, 64)
    mx = torch.full((B, H, 1, Sp), float("nan"), device=dev)
    dn = torch.full((B, H, 1, Sp), float("nan"), device=dev)
    bmx = torch.full((B, H, nb, Sp), float("nan"), dtype=torch.bfloat16, device=dev)
    if with_v:
        o = torch.full_like(qd, float("nan"))
        capi.fullattn_maxq_denom_blockmax(o, mx, dn, bmx, qd, kd, vd, kv_len=kv_len)
        want = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float()[:, :, :kv], v.float()[:, :, :kv])
        assert_close_o(f32(o), f32(want), "fullattn_maxq_denom_blockmax O")
    else:
        capi.maxq_denom_blockmax(mx, dn, bmx, qd, kd, kv_len=kv_len)
    wmx, wdn = orc.maxq_denom(f32(q), f32(k), kv_len=kv)
    assert_close_stat(f32(mx), wmx, "max_q", atol=1e-4)
    assert_close_stat(f32(dn), wdn, "denom")
    got = f32(bmx)
    assert np.isnan(got[:, :, nkb:]).all(), "blocks without a key are not written"
    g, w = got[:, :, :nkb, :S], orc.block_row_max(f32(q), f32(k), kv_len=kv)[:, :, :nkb, :S]
    tol = 1e-3 + 1e-4 * np.abs(w)
    # stored as bf16 rounded up: never below the oracle's maximum, less than one bf16 step above
    assert np.isfinite(g).all() and np.all(g >= w - tol) and np.all(g <= w + tol + 2.0 ** -7 * np.abs(w))
    assert np.array_equal(g.max(axis=2), orc.bf16_round_up(f32(mx).reshape(B, H, Sp)[..., :S]))
    dev_bmx = np.nan_to_num(got, nan=-np.inf)
    for qblk in (64, 128):
        nq = orc.ceil_div(S, qblk)
        _, pmax = orc.booleanmask_rows(f32(mx), f32(dn), f32(q), f32(k), 1.0, qblk=qblk, kv_len=kv)
        pblk = np.full((B, H, nq, nb), -np.inf, np.float32)
        for J in range(nkb):
            pblk[..., J] = pmax[..., 64 * J: min(64 * J + 64, kv)].max(axis=-1)
        thr = float(np.quantile(pblk[..., :nkb], 0.5)) if nkb > 2 else 0.5 * float(pblk[..., :nkb].min())
        bi = torch.full((B, H, nq, nb), -1, dtype=torch.int32, device=dev)
        bc = torch.full((B, H, nq), -9, dtype=torch.int32, device=dev)
        bm = torch.full((B, H, nq, nb), 7, dtype=torch.uint8, device=dev)
        capi.blockmax_to_blocklists(bi, bc, bmx, mx, dn, thr, S, D, qblk=qblk, blockmask=bm, kv_len=kv_len)
        got_bm = bm.cpu().numpy().astype(bool)
        assert int(bm.max()) <= 1 and not got_bm[..., nkb:].any()
        wi, wn = orc.block_lists_from_blockmask(got_bm, fill=-1)
        assert np.array_equal(bi.cpu().numpy(), wi) and np.array_equal(bc.cpu().numpy(), wn)
        want_bm, margin = orc.block_mask_from_blockmax(dev_bmx, f32(mx), f32(dn), thr, S, D, qblk=qblk, kv_len=kv)
        near = np.abs(margin) <= 1e-4
        assert np.array_equal(got_bm | near, want_bm | near)
        # a superset of the per-key oracle's block mask (the maxima are rounded up), equal outside the band
        lift = float(np.exp2(2.0 ** -7 * np.abs(dev_bmx[np.isfinite(dev_bmx)]).max() * orc.LOG2E / np.sqrt(D)))
        exact_bm = pblk > np.float32(thr)
        band = (pblk >= thr * (1 - BAND) / lift) & (pblk <= thr * (1 + BAND))
        assert not (exact_bm & ~got_bm & ~band).any()
        assert np.array_equal(got_bm | band, exact_bm | band)
