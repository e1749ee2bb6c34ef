"""Pins the CPU oracle: golden fixtures (independent fp64 loops), library routines that
special cases reduce to, invariants, and brute force.  Runs without a GPU."""
import glob
import math
import os

import numpy as np
import pytest
import torch

from fgattn_tk_cuda_amd import workloads as wl
from oracle import cpu_masked_attention as cma
from oracle import spattn_oracle as orc

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _qkv(B, H, S, D, seed):
    return tuple(t.float().numpy() for t in wl.randn_qkv(B, H, S, D, seed=seed))


def test_fixture_files_present():
    names = sorted(os.path.basename(p) for p in glob.glob(os.path.join(GOLD, "*.npz")))
    assert names == ["dense_d64.npz", "prepass_d128.npz", "prepass_d64.npz", "sparse_d128_q128.npz", "sparse_d64_q64.npz"]


@pytest.mark.parametrize("name", ["sparse_d64_q64", "sparse_d128_q128", "dense_d64"])
def test_sp_attn_matches_golden(name):
    g = np.load(os.path.join(GOLD, name + ".npz"))
    q, k, v = (g[x][None, None] for x in "qkv")
    o, lse = orc.sp_attn(q, k, v, g["kv_indices"], g["kv_num_indices"], qblk=int(g["qblk"]), round_p=False)
    assert np.allclose(o[0, 0], g["o"], atol=2e-5, rtol=1e-4)
    assert np.allclose(lse[0, 0], g["lse"], atol=1e-4, rtol=1e-5)
    # with P rounded to bf16 (what the kernels do) the result stays well inside the contract
    o2, _ = orc.sp_attn(q, k, v, g["kv_indices"], g["kv_num_indices"], qblk=int(g["qblk"]), round_p=True)
    assert np.abs(o2[0, 0] - g["o"]).max() < 5e-3


def test_full_attn_matches_golden_and_sdpa():
    g = np.load(os.path.join(GOLD, "dense_d64.npz"))
    q, k, v = (g[x][None, None] for x in "qkv")
    o, mx, dn = orc.full_attn(q, k, v, round_p=False)
    assert np.allclose(o[0, 0], g["o"], atol=2e-5, rtol=1e-4)
    q, k, v = _qkv(2, 2, 300, 64, 1)
    o, _, _ = orc.full_attn(q, k, v, round_p=False)
    want = torch.nn.functional.scaled_dot_product_attention(*(torch.from_numpy(x) for x in (q, k, v))).numpy()
    assert np.allclose(o, want, atol=2e-5, rtol=1e-4)
    o, _, _ = orc.full_attn(q, k, v, kv_len=250, round_p=False)
    want = torch.nn.functional.scaled_dot_product_attention(torch.from_numpy(q), torch.from_numpy(k[:, :, :250]), torch.from_numpy(v[:, :, :250])).numpy()
    assert np.allclose(o, want, atol=2e-5, rtol=1e-4)


@pytest.mark.parametrize("qblk", [64, 128])
def test_sp_attn_permuted_full_list_is_sdpa(qblk):
    """The reference's own sparse test: a permutation of all keys (python/test/test_extension.py:61-89)."""
    B, H, S, D = 1, 2, 333, 64
    q, k, v = _qkv(B, H, S, D, 2)
    idx, num = wl.permuted_all_index(B, H, S, qblk=qblk, seed=3)
    o, lse = orc.sp_attn(q, k, v, idx.numpy(), num.numpy(), qblk=qblk, round_p=False)
    tq, tk, tv = (torch.from_numpy(x) for x in (q, k, v))
    want = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv).numpy()
    assert np.allclose(o, want, atol=2e-5, rtol=1e-4)
    s = torch.einsum("bhmd,bhnd->bhmn", tq, tk) / math.sqrt(D)
    assert np.allclose(lse, torch.logsumexp(s, -1).numpy(), atol=1e-4)


def test_sp_attn_invariants():
    B, H, S, D = 1, 1, 256, 64
    q, k, v = _qkv(B, H, S, D, 4)
    rng = np.random.default_rng(5)
    ms = 256
    base = np.full((B, H, 2, ms), ms, np.int32)
    base[0, 0, 0, :100] = rng.permutation(S)[:100]
    base[0, 0, 1, :37] = rng.permutation(S)[:37]
    num = np.array([[[100, 37]]], np.int32)
    o0, l0 = orc.sp_attn(q, k, v, base, num, round_p=False)
    perm = base.copy()
    perm[0, 0, 0, :100] = perm[0, 0, 0, rng.permutation(100)]
    o1, _ = orc.sp_attn(q, k, v, perm, num, round_p=False)
    assert np.allclose(o0, o1, atol=1e-5)                       # order does not matter
    dup = base.copy()
    dup[0, 0, 0, 100:200] = base[0, 0, 0, :100]
    dup[0, 0, 1, 37:74] = base[0, 0, 1, :37]
    o2, l2 = orc.sp_attn(q, k, v, dup, num * 2, round_p=False)
    assert np.allclose(o0, o2, atol=1e-5)                       # a duplicated list changes nothing ...
    assert np.allclose(l2, l0 + math.log(2), atol=1e-5)         # ... but the log-sum-exp by log 2
    one = np.full((B, H, 2, ms), ms, np.int32)
    one[0, 0, :, 0] = [17, 200]
    o3, _ = orc.sp_attn(q, k, v, one, np.ones((B, H, 2), np.int32))
    assert np.array_equal(o3[0, 0, :128], np.repeat(v[0, 0, 17:18], 128, 0))   # a single key returns its V row
    assert np.array_equal(o3[0, 0, 128:], np.repeat(v[0, 0, 200:201], 128, 0))
    # entries past the count and entries >= S are ignored; an empty list gives zeros / -inf
    bad = base.copy()
    bad[0, 0, 0, 100:110] = 3
    bad[0, 0, 1, 5] = 9999
    num2 = np.array([[[100, 37]]], np.int32)
    o4, _ = orc.sp_attn(q, k, v, bad, num2, round_p=False)
    keep = [c for j, c in enumerate(base[0, 0, 1, :37]) if j != 5]
    ref = base.copy()
    ref[0, 0, 1, :36] = keep
    o5, _ = orc.sp_attn(q, k, v, ref, np.array([[[100, 36]]], np.int32), round_p=False)
    assert np.allclose(o4, o5, atol=1e-6)
    o6, l6 = orc.sp_attn(q, k, v, base, np.zeros((B, H, 2), np.int32))
    assert np.all(o6 == 0) and np.all(np.isneginf(l6))


def test_block_lists_expand_to_token_lists():
    B, H, S = 1, 2, 1000
    bi, bc = wl.ragged_block_lists(B, H, S, 64, 64, np.array([[3] * 16, [16] * 16]), seed=6)
    tok, num = orc.block_list_to_token_list(bi.numpy(), bc.numpy(), S)
    tok2, num2 = wl.blocks_to_tokens(bi, bc, S)
    assert np.array_equal(tok, tok2.numpy()) and np.array_equal(num, num2.numpy())
    for h in range(H):
        for i in range(16):
            want = sorted(t for j in bi[0, h, i, : bc[0, h, i]].tolist() for t in range(64 * j, min(S, 64 * j + 64)))
            assert tok[0, h, i, : num[0, h, i]].tolist() == want


def test_cpu_baseline_matches_oracle():
    B, H, S, D, qblk = 1, 1, 512, 64, 64
    q, k, v = wl.randn_qkv(B, H, S, D, seed=7, dtype=torch.float32)
    bi, bc = wl.uniform_block_lists(B, H, S, qblk, 64, 3, seed=8)
    got = cma.masked_attention_rows(q[0, 0], k[0, 0], v[0, 0], bi[0, 0], bc[0, 0], 64, 320, qblk, 64).numpy()
    tok, num = wl.blocks_to_tokens(bi, bc, S)
    want, _ = orc.sp_attn(q.numpy(), k.numpy(), v.numpy(), tok.numpy(), num.numpy(), qblk=qblk, round_p=False)
    assert np.allclose(got, want[0, 0, 64:320], atol=2e-5, rtol=1e-4)


@pytest.mark.parametrize("name", ["prepass_d64", "prepass_d128"])
def test_prepass_matches_golden(name):
    g = np.load(os.path.join(GOLD, name + ".npz"))
    q, k = g["q"][None, None], g["k"][None, None]
    S = q.shape[2]
    mx, dn = orc.maxq_denom(q, k)
    assert np.allclose(mx[0, 0, 0, :S], g["max_q"], rtol=1e-5, atol=1e-4)
    assert np.allclose(dn[0, 0, 0, :S], g["denom"], rtol=1e-4)
    assert np.all(mx[..., S:] == 0) and np.all(np.isneginf(dn[..., S:]))      # pad rows
    votes, pmax = orc.booleanmask_128(mx, dn, q, k, float(g["thresh"]))
    assert np.allclose(pmax, g["pmax"], rtol=1e-3, atol=1e-9)
    near = np.abs(g["pmax"] - g["thresh"]) <= 1e-3 * g["thresh"]
    assert np.array_equal((votes[..., :S] > 0) | near, (g["votes"][..., :S] > 0) | near)
    assert (votes == g["votes"]).mean() > 0.999
    idx, num = orc.booleanmask_to_indexmask(g["votes"], S)
    assert np.array_equal(idx, g["kv_indices"]) and np.array_equal(num, g["kv_num_indices"])


def test_maxq_denom_closed_forms():
    """The reference's own check (python/test/spattn/test_mask_utils.py:33-56)."""
    B, H, S, D = 1, 2, 300, 128
    q, k, _ = _qkv(B, H, S, D, 9)
    mx, dn = orc.maxq_denom(q, k)
    for h in range(H):
        s = torch.from_numpy(q[0, h]) @ torch.from_numpy(k[0, h]).T
        assert np.allclose(mx[0, h, 0, :S], s.max(-1).values.numpy(), atol=1e-4)
        d = torch.exp((s - s.max(-1, keepdim=True).values) / math.sqrt(D)).sum(-1)
        assert np.allclose(dn[0, h, 0, :S], d.numpy(), rtol=1e-4)
    mx2, dn2 = orc.maxq_denom(q, k, kv_len=200)
    s = torch.from_numpy(q[0, 0]) @ torch.from_numpy(k[0, 0, :200]).T
    assert np.allclose(mx2[0, 0, 0, :S], s.max(-1).values.numpy(), atol=1e-4)


def test_booleanmask_is_maxpooled_threshold():
    """>0 of the vote mask is the 128-row max-pool of softmax > thresh
    (python/spattn/mask_utils.py:126-142,206-222), here with torch's softmax and max_pool."""
    B, H, S, D = 1, 2, 300, 64
    q, k, _ = (t.float() for t in wl.clustered_qkv(B, H, S, D, seed=10, sigma=0.7))
    mx, dn = orc.maxq_denom(q.numpy(), k.numpy())
    thr = 0.02
    votes, pmax = orc.booleanmask_128(mx, dn, q.numpy(), k.numpy(), thr)
    for h in range(H):
        p = torch.softmax(q[0, h] @ k[0, h].T / math.sqrt(D), -1)
        hit = (p > thr).float()[None]
        pooled = torch.nn.functional.max_pool2d(torch.nn.functional.pad(hit, (0, 0, 0, (-S) % 128)), (128, 1))[0] > 0
        near = np.abs(pmax[0, h] - thr) <= 1e-3 * thr
        assert np.array_equal((votes[0, h, :, :S] > 0) | near, pooled.numpy() | near)
        # vote count = number of 16-row groups that hit
        cnt = torch.nn.functional.max_pool2d(torch.nn.functional.pad(hit, (0, 0, 0, (-S) % 16)), (16, 1))[0]
        cnt = torch.nn.functional.pad(cnt, (0, 0, 0, (-cnt.shape[0]) % 8)).view(-1, 8, S).sum(1)
        assert ((votes[0, h, :, :S] == cnt.numpy()) | near).all()
    assert np.all(votes[..., S:] == 0)


def test_booleanmask_to_indexmask_exact():
    rng = np.random.default_rng(11)
    mask = (rng.random((2, 2, 3, 256)) < 0.2) * rng.integers(1, 9, (2, 2, 3, 256))
    idx, num = orc.booleanmask_to_indexmask(mask, 200)
    for b in range(2):
        for h in range(2):
            for i in range(3):
                kept = [c for c in range(200) if mask[b, h, i, c] > 0]       # plain loop
                assert num[b, h, i] == len(kept)
                assert idx[b, h, i, : len(kept)].tolist() == kept
                assert np.all(idx[b, h, i, len(kept):] == 256)
    idx2, num2 = orc.booleanmask_to_indexmask(np.zeros((1, 1, 1, 128), np.int32), 128)
    assert num2[0, 0, 0] == 0 and np.all(idx2 == 128)


@pytest.mark.parametrize("S", [300, 330])
def test_booleanmask_rows_is_the_maxpooled_threshold_at_64_and_128_rows(S):
    """M[I,c] for 64-row q-blocks against torch softmax + max_pool over 64 rows; the two halves
    of a 128-row block OR to the 128-row mask, which is `booleanmask_128 > 0` exactly."""
    B, H, D = 1, 2, 64
    q, k, _ = (t.float() for t in wl.clustered_qkv(B, H, S, D, seed=12, sigma=0.7))
    mx, dn = orc.maxq_denom(q.numpy(), k.numpy())
    thr = 0.02
    m128, p128 = orc.booleanmask_rows(mx, dn, q.numpy(), k.numpy(), thr, qblk=128)
    m64, p64 = orc.booleanmask_rows(mx, dn, q.numpy(), k.numpy(), thr, qblk=64)
    votes, pmax = orc.booleanmask_128(mx, dn, q.numpy(), k.numpy(), thr)
    assert np.array_equal(m128, votes[..., :S] > 0) and np.array_equal(p128, pmax)
    n64, n128 = orc.ceil_div(S, 64), orc.ceil_div(S, 128)
    assert m64.shape == (B, H, n64, S) and m128.shape == (B, H, n128, S)
    both = np.zeros((B, H, 2 * n128, S), bool)
    both[:, :, :n64] = m64
    assert np.array_equal(both[:, :, 0::2] | both[:, :, 1::2], m128)
    for h in range(H):
        p = torch.softmax(q[0, h] @ k[0, h].T / math.sqrt(D), -1)
        hit = (p > thr).float()[None]
        pooled = torch.nn.functional.max_pool2d(torch.nn.functional.pad(hit, (0, 0, 0, (-S) % 64)), (64, 1))[0] > 0
        near = np.abs(p64[0, h] - thr) <= 1e-3 * thr
        assert np.array_equal(m64[0, h] | near, pooled.numpy() | near)
    # a short kv length cuts columns, nothing else
    mk, _ = orc.booleanmask_rows(*orc.maxq_denom(q.numpy(), k.numpy(), kv_len=200), q.numpy(), k.numpy(), thr, qblk=64, kv_len=200)
    assert mk.shape[-1] == 200


def test_block_mask_and_block_lists_by_brute_force():
    """MB[I,J] = OR of the keys of block J below seq; lists = ascending kept block ids, fill behind
    them, exact counts - against plain loops, with a ragged last block, set keys at and past seq,
    an empty row, a full row and a list cut off at max_blocks."""
    rng = np.random.default_rng(13)
    B, H, SB, MS, seq = 1, 2, 4, 384, 300
    mask = ((rng.random((B, H, SB, MS)) < 0.03) * rng.integers(1, 9, (B, H, SB, MS))).astype(np.int32)
    mask[0, 0, 0] = 0
    mask[0, 0, 1] = 3
    mask[0, 1, 2, :] = 0
    mask[0, 1, 2, 299] = 1          # the last key below seq: block 4 (keys 256..319) is kept
    mask[0, 1, 2, 300] = 1          # at seq: ignored
    mask[0, 1, 3, :] = 0
    mask[0, 1, 3, 320:] = 1         # only keys past seq: nothing is kept
    bm = orc.block_mask_from_votes(mask, seq)
    nb = orc.ceil_div(seq, 64)
    assert bm.shape == (B, H, SB, nb)
    for h in range(H):
        for i in range(SB):
            for J in range(nb):
                want = any(mask[0, h, i, c] > 0 for c in range(64 * J, min(64 * J + 64, seq)))
                assert bm[0, h, i, J] == want, (h, i, J)
    idx, cnt, full = orc.block_lists_from_mask(mask, seq, fill=-5)
    assert full.shape == (B, H, SB, MS // 64) and np.array_equal(full[..., :nb], bm) and not full[..., nb:].any()
    for h in range(H):
        for i in range(SB):
            kept = [J for J in range(nb) if bm[0, h, i, J]]
            assert cnt[0, h, i] == len(kept) and idx[0, h, i, : len(kept)].tolist() == kept
            assert np.all(idx[0, h, i, len(kept):] == -5)
    assert cnt[0, 0, 0] == 0 and cnt[0, 0, 1] == nb and idx[0, 1, 2, :1].tolist() == [4] and cnt[0, 1, 2] == 1 and cnt[0, 1, 3] == 0
    idx2, cnt2, _ = orc.block_lists_from_mask(mask, seq, max_blocks=2, fill=-5)
    assert np.array_equal(cnt2, cnt) and np.array_equal(idx2, idx[..., :2])
    # a bool mask and the packed form of the same mask give the same blocks
    assert np.array_equal(orc.block_mask_from_votes(orc.unpack_mask(orc.pack_mask(mask)), seq), bm)
    # block lists are the token lists of the reference restricted to aligned runs: expanding them
    # covers every kept key
    tok, num = orc.block_list_to_token_list(idx, cnt, seq, mask_stride=MS)
    ki, kn = orc.booleanmask_to_indexmask(mask, seq)
    for h in range(H):
        for i in range(SB):
            assert set(ki[0, h, i, : kn[0, h, i]]) <= set(tok[0, h, i, : num[0, h, i]])


def test_block_row_max_and_its_threshold_by_brute_force():
    """blockmax[J][r] = max of the raw scores of row r over the keys of block J below kv_len
    (plain loops), and thresholding it per row gives the block mask of the per-key threshold mask:
    a key of block J passes softmax(r, c) > tau exactly when the block's maximum passes
    s > t[r] - checked against block_mask_from_votes(booleanmask_rows(...)) outside a thin band
    around the threshold, and exactly in float64."""
    rng = np.random.default_rng(5)
    B, H, S, D, kv = 1, 2, 520, 64, 450
    q = orc.bf16_round(rng.standard_normal((B, H, S, D), dtype=np.float32))
    k = orc.bf16_round(rng.standard_normal((B, H, S, D), dtype=np.float32) + np.repeat(
        1.2 * rng.standard_normal((B, H, 13, D), dtype=np.float32), 40, axis=2))
    bmx = orc.block_row_max(q, k, kv_len=kv)
    sp = orc.padded_len(S)
    assert bmx.shape == (B, H, sp // 64, sp)
    for h in range(H):
        for r in (0, 17, 199):
            for J in range(sp // 64):
                cols = range(64 * J, min(64 * J + 64, kv))
                want = max((float(np.dot(q[0, h, r].astype(np.float64), k[0, h, c].astype(np.float64))) for c in cols),
                           default=-np.inf)
                assert bmx[0, h, J, r] == pytest.approx(want, rel=1e-5, abs=1e-5) or (want == -np.inf and bmx[0, h, J, r] == -np.inf)
    assert np.all(bmx[..., S:] == 0) and np.all(bmx[:, :, 8:, :S] == -np.inf)   # blocks 8.. hold no key below 450
    mx, dn = orc.maxq_denom(q, k, kv_len=kv)
    for qblk in (64, 128):
        mask, pmax = orc.booleanmask_rows(mx, dn, q, k, 1.0, qblk=qblk, kv_len=kv)
        thr = float(np.quantile(pmax, 0.985))
        want = orc.block_mask_from_votes((pmax > np.float32(thr)).astype(np.int32), kv)
        got, margin = orc.block_mask_from_blockmax(bmx, mx, dn, thr, S, D, qblk=qblk, kv_len=kv)
        nkb = orc.ceil_div(kv, 64)
        assert got.shape == (B, H, orc.ceil_div(S, qblk), sp // 64) and not got[..., nkb:].any()
        near = np.abs(margin[..., :nkb]) <= 1e-4
        assert np.array_equal(got[..., :nkb] | near, want | near)
        assert 0.02 < want.mean() < 0.98 and near.mean() < 0.01
        # the same statement in float64, where the two forms of the test are the same inequality
        # up to one rounding: compare the margins' signs away from zero
        s64 = np.einsum("bhrd,bhcd->bhrc", q.astype(np.float64), k[:, :, :kv].astype(np.float64))
        sf = orc.LOG2E / np.sqrt(D)
        mx64 = s64.max(-1); dn64 = np.exp2((s64 - mx64[..., None]) * sf).sum(-1)
        p64 = np.exp2((s64 - mx64[..., None]) * sf) / dn64[..., None]
        for i in range(orc.ceil_div(S, qblk)):
            rows = slice(i * qblk, min(S, (i + 1) * qblk))
            for J in range(nkb):
                cols = slice(64 * J, min(64 * J + 64, kv))
                by_key = (p64[:, :, rows, cols] > thr).any(axis=(-1, -2))
                t64 = (np.log2(thr) + mx64[:, :, rows] * sf + np.log2(dn64[:, :, rows])) / sf
                by_block = (s64[:, :, rows, cols].max(-1) > t64).any(-1)
                assert np.array_equal(by_key, by_block)
    idx, cnt = orc.block_lists_from_blockmask(got, max_blocks=3, fill=-2)
    for h in range(H):
        for i in range(got.shape[2]):
            kept = np.flatnonzero(got[0, h, i]).tolist()
            assert cnt[0, h, i] == len(kept) and idx[0, h, i, : min(3, len(kept))].tolist() == kept[:3]
            assert np.all(idx[0, h, i, len(kept):] == -2)


def test_all_index_mask():
    idx, num = orc.all_index_mask(1, 2, 3, 300, 384)
    assert idx.shape == (1, 2, 3, 384) and np.all(idx == np.arange(384)) and np.all(num == 300)


def test_bf16_round():
    x = np.array([1.0, 1.00390625, 1.01171875, -3.1415926, 1e-30, 65504.0], np.float32)
    want = torch.from_numpy(x).to(torch.bfloat16).float().numpy()
    assert np.array_equal(orc.bf16_round(x), want)


def test_pack_mask_matches_library_and_round_trips():
    """pack: 8 keys per byte, least significant bit first (numpy.packbits little); unpack inverts it
    (the reference's own round-trip test, python/test/spattn/test_mask_utils.py:86-97); the byte value of a
    hand-made pattern; the fused unpack+compaction equals compaction of the unpacked mask."""
    rng = np.random.default_rng(3)
    mask = (rng.random((1, 2, 3, 256)) < 0.2).astype(np.int32) * 5
    packed = orc.pack_mask(mask)
    assert packed.dtype == np.uint8 and packed.shape == (1, 2, 3, 32)
    assert np.array_equal(orc.unpack_mask(packed), mask > 0)
    one = np.zeros((1, 1, 1, 8), np.int32)
    one[..., 0] = 1
    one[..., 7] = 3
    assert orc.pack_mask(one).item() == 129
    # brute force, bit by bit
    for c in range(256):
        assert ((packed[0, 1, 2, c >> 3] >> (c & 7)) & 1) == (mask[0, 1, 2, c] > 0)
    wi, wn = orc.packedmask_to_indexmask(packed, 200)
    ri, rn = orc.booleanmask_to_indexmask(mask, 200)
    assert np.array_equal(wi, ri) and np.array_equal(wn, rn)


@pytest.mark.parametrize("S,D,blk", [(300, 64, 128), (256, 128, 64), (130, 128, 128)])
def test_topk_generator_scores_match_the_reference_expressions_in_bf16(S, D, blk):
    """qmean / score of the oracle against the reference's own torch expressions
    (python/spattn/mask_utils.py:390-410) evaluated in bf16 on the CPU: qmean exact, score
    equal except where another summation order moves a value across a bf16 rounding boundary."""
    g = torch.Generator().manual_seed(S + D)
    B, H = 1, 2
    q = torch.randn(B, H, S, D, generator=g).bfloat16()
    k = torch.randn(B, H, S, D, generator=g).bfloat16()
    qm, sc = orc.qblock_mean_scores(q.float().numpy(), k.float().numpy(), blk)
    fl = S // blk
    full = q[:, :, :fl * blk].view(B, H, fl, blk, D).mean(dim=3)
    parts = [full]
    if S % blk:
        parts.append(q[:, :, fl * blk:].mean(dim=2, keepdim=True))
    qs = torch.cat(parts, dim=2) * 1. / D ** 0.5
    ut = torch.einsum("bhmd,bhnd->bhmn", qs, k)
    assert np.array_equal(qm, qs.float().numpy())
    want = ut.float().numpy()
    diff = sc != want
    assert diff.mean() < 0.01
    assert np.all(np.abs(sc - want)[diff] <= np.abs(want[diff]) * 2.0 ** -7 + 1e-30)


def test_topk_select_matches_torch_topk_values_and_brute_force():
    rng = np.random.default_rng(4)
    # bf16-like scores with many ties
    sc = orc.bf16_round(rng.standard_normal((3, 5, 700)).astype(np.float32))
    for kk in (1, 37, 128, 700, 900):
        sel = orc.topk_select(sc, kk)
        k_eff = min(kk, 700)
        assert sel.shape == (3, 5, k_eff) and np.all(np.diff(sel, axis=-1) > 0)
        mine = np.take_along_axis(sc, sel.astype(np.int64), -1)
        want = torch.topk(torch.from_numpy(sc), k_eff, dim=-1).values.numpy()
        assert np.array_equal(np.sort(mine, -1), np.sort(want, -1))
    # ties go to the lower key; kv_len cuts the candidates
    row = np.array([[1.0, 3.0, 3.0, 2.0, 3.0, 3.0, 0.5, 9.0]], np.float32)
    assert orc.topk_select(row, 3).tolist() == [[1, 2, 7]]
    assert orc.topk_select(row, 3, kv_len=6).tolist() == [[1, 2, 4]]
    # brute force on tiny rows
    for _ in range(50):
        r = orc.bf16_round(rng.integers(-3, 4, size=(1, 12)).astype(np.float32))
        kk = int(rng.integers(1, 13))
        pairs = sorted(((-float(r[0, i]), i) for i in range(12)))[:kk]
        assert orc.topk_select(r, kk)[0].tolist() == sorted(i for _, i in pairs)


def test_cfg1_plumbing_case_oracle_equals_dense_masked_softmax():
    """The CPU-runnable configuration (B=1 H=4 N=1024 d=64 fp32, 64x64 blocks, diagonal plus
    random key blocks up to 25 %): the oracle's gathered form equals the dense definition
    softmax(QK^T * scale with -inf outside the kept blocks) V evaluated with torch in fp32."""
    c = wl.CONFIGS["cfg1_plumbing"]
    B, H, S, D, qblk, kvblk = c["B"], c["H"], c["S"], c["D"], c["qblk"], c["kvblk"]
    q, k, v = wl.randn_qkv(B, H, S, D, seed=101, dtype=torch.float32)
    bi, bc = wl.uniform_block_lists(B, H, S, qblk, kvblk, int(round(c["density"] * (S // kvblk))), seed=102)
    assert bi.shape[-1] == 4 and all(i in bi[0, 0, i].tolist() for i in range(S // qblk))
    tok, num = wl.blocks_to_tokens(bi, bc, S)
    got, lse = orc.sp_attn(q.numpy(), k.numpy(), v.numpy(), tok.numpy(), num.numpy(), qblk=qblk, round_p=False)
    for h in range(H):
        want = cma.masked_attention_rows(q[0, h], k[0, h], v[0, h], bi[0, h], bc[0, h], 0, S, qblk, kvblk)
        assert np.abs(got[0, h] - want.numpy()).max() < 2e-5
        s = (q[0, h] @ k[0, h].T) * D ** -0.5
        s.masked_fill_(~cma.block_mask_rows(bi[0, h], bc[0, h], 0, S, qblk, kvblk, S), float("-inf"))
        assert np.abs(lse[0, h] - torch.logsumexp(s, -1).numpy()).max() < 2e-5


def test_qblock_order_is_a_stable_class_sort():
    """Longest lists first in quarter-octave classes, stable inside a class; lists within a factor
    of two of each other keep the XCD-contiguous default order.  Checked against a pure-Python sort."""
    rng = np.random.default_rng(0)

    def cls(x):
        if x <= 0:
            return 89
        lg = x.bit_length() - 1
        below = ((x >> (lg - 2)) & 3) if lg >= 2 else ((x << (2 - lg)) & 3)
        return 88 - min(4 * lg + below, 88)

    for trial in range(200):
        n = int(rng.integers(1, 300))
        c = rng.integers(0, 5000, size=n)
        if trial % 5 == 0:
            c = c // 1000
        got = orc.qblock_order(c)
        assert sorted(got.tolist()) == list(range(n))
        lo, hi = int(c.min()), int(c.max())
        if hi <= 0 or hi < 2 * lo:
            assert got.tolist() == orc._xcd_remap(np.arange(n), n).tolist()
            continue
        assert got.tolist() == sorted(range(n), key=lambda i: (cls(int(c[i])), i))
    # equal lengths: the default order, every XCD a contiguous range
    d = orc.qblock_order(np.full(32, 7))
    assert d[:8].tolist() == [0, 4, 8, 12, 16, 20, 24, 28] and sorted(d.tolist()) == list(range(32))
    assert orc.qblock_order(np.array([1 << 30, 3, 1 << 24, 0])).tolist() == [0, 2, 1, 3]


def test_bf16_round_up_by_its_defining_property():
    """bf16_round_up(x) is the smallest bf16 >= x: it is a bf16 pattern, not below x, and the bf16
    just below it is below x; bf16 values, zeros and infinities map to themselves."""
    rng = np.random.default_rng(5)
    x = np.concatenate([rng.standard_normal(20000).astype(np.float32) * np.float32(40.0),
                        rng.standard_normal(2000).astype(np.float32) * np.float32(1e-3),
                        np.array([0.0, -0.0, 1.0, -1.0, 3.140625, -3.140625, np.inf, -np.inf, 1e30, -1e30], np.float32)])
    y = orc.bf16_round_up(x)
    yb = y.view(np.uint32)
    assert np.all((yb & 0xFFFF) == 0), "not a bf16 pattern"
    assert np.all(y >= x)
    fin = np.isfinite(x) & (y != 0)
    # the next bf16 towards -inf: one step of the upper 16 bits (down for positive, up for negative patterns)
    hi = (yb[fin] >> 16).astype(np.int64)
    below = np.where(y[fin] > 0, hi - 1, hi + 1).astype(np.uint32) << 16
    assert np.all(below.view(np.float32) < x[fin])
    exact = orc.bf16_round(x) == x
    assert np.array_equal(y[exact], x[exact])
    assert y[-4] == np.inf and y[-3] == -np.inf
    # against plain enumeration on a few values: candidates are the two bf16 neighbours
    for v in x[:200]:
        lo = np.float32(np.uint32(np.float32(v).view(np.uint32) & 0xFFFF0000).view(np.float32))   # truncation towards zero
        step = np.float32(np.uint32((np.float32(v).view(np.uint32) & 0xFFFF0000) + 0x10000).view(np.float32))
        cands = [c for c in (lo, step) if c >= v]
        assert orc.bf16_round_up(np.array([v], np.float32))[0] == min(cands)
