"""GPU parity of the top-k mask generator (q-block means, scores, radix select) through the C ABI."""
import numpy as np
import pytest
import torch

from fgattn_tk_cuda_amd import capi, workloads as wl
from oracle import spattn_oracle as orc
from helpers import assert_close_o, f32

pytestmark = pytest.mark.gpu


def _run(dev, q, k, select_k, blk, kv_len=0, idx_stride=None, score_stride=None):
    B, H, S, D = q.shape
    SB = orc.ceil_div(S, blk)
    kv = kv_len or S
    idx_stride = idx_stride or 128 * orc.ceil_div(min(select_k, kv), 128)
    score_stride = score_stride or orc.padded_len(S)
    fill = -7
    kvi = torch.full((B, H, SB, idx_stride), fill, dtype=torch.int32, device=dev)
    kvn = torch.full((B, H, SB), -1, dtype=torch.int32, device=dev)
    score = torch.full((B, H, SB, score_stride), float("nan"), dtype=torch.bfloat16, device=dev)
    qmean = torch.full((B, H, SB, D), float("nan"), dtype=torch.bfloat16, device=dev)
    capi.qk_topkmask_indices(kvi, kvn, score, qmean, q.to(dev), k.to(dev), select_k, blocksz=blk, kv_len=kv_len)
    torch.cuda.synchronize()
    return kvi.cpu().numpy(), kvn.cpu().numpy(), f32(score), f32(qmean), fill


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("blk", [64, 128])
@pytest.mark.parametrize("S,select_k,kv_len", [(1000, 100, 0), (4500, 512, 0), (777, 777, 0), (2048, 1, 0), (1000, 300, 900)])
def test_topk_generator_matches_oracle(dev, D, blk, S, select_k, kv_len):
    print("case topk", D, blk, S, select_k, kv_len, flush=True)
    B, H = 2, 3
    q, k, _ = wl.randn_qkv(B, H, S, D, seed=S + D)
    kvi, kvn, score, qmean, fill = _run(dev, q, k, select_k, blk, kv_len)
    kv = kv_len or S
    want_qm, want_sc = orc.qblock_mean_scores(f32(q), f32(k), blk)
    # q-block means: same order of summation, bit-exact
    assert np.array_equal(qmean, want_qm)
    # scores: fp32 accumulation inside the matrix unit may round differently by one bf16 step
    # (and, where the terms cancel, by the fp32 error of the sum itself: 1e-5 absolute)
    got_sc = score[..., :kv]
    assert np.isfinite(got_sc).all()
    diff = got_sc != want_sc[..., :kv]
    assert diff.mean() < 0.02
    assert np.all(np.abs(got_sc - want_sc[..., :kv])[diff] <= np.abs(want_sc[..., :kv][diff]) * 2.0 ** -7 + 1e-5)
    # the selection, given the scores the device produced, is integer work: bit-exact
    kk = min(select_k, kv)
    want_sel = orc.topk_select(got_sc, select_k)
    assert np.all(kvn == kk)
    assert np.array_equal(kvi[..., :kk], want_sel)
    assert np.all(kvi[..., kk:] == fill)


@pytest.mark.parametrize("S,select_k", [(4096, 300), (8200, 8100), (16001, 1300), (32757, 2621), (32768, 32768), (45003, 900),
                                        (72001, 6000), (73728, 73000)])
def test_topk_select_row_lengths_with_many_ties(dev, S, select_k):
    """Every row length class of the in-register select (1, 2, 4, 8, 12 and 18 vectors per lane), row
    ends inside a 16-byte vector, and keys on a coarse grid so that many scores are equal - also at
    the threshold, where the lower key wins."""
    print("case topk row lengths", S, select_k, flush=True)
    B, H, D, blk = 1, 1, 64, 128
    g = torch.Generator().manual_seed(S)
    q = (torch.randint(-2, 3, (B, H, S, D), generator=g).float() * 0.5).bfloat16()
    k = (torch.randint(-2, 3, (B, H, S, D), generator=g).float() * 0.25).bfloat16()
    kvi, kvn, score, _, fill = _run(dev, q, k, select_k, blk)
    SB = orc.ceil_div(S, blk)
    rows = sorted({0, 1, SB // 3, SB // 2, SB - 2, SB - 1})
    got_sc = score[0, 0, rows, :S]
    assert np.isfinite(got_sc).all()
    assert len(np.unique(got_sc[0])) < S // 4          # ties everywhere
    want_sel = orc.topk_select(got_sc, select_k)
    kk = min(select_k, S)
    assert np.all(kvn == kk)
    assert np.array_equal(kvi[0, 0, rows, :kk], want_sel)
    assert np.all(kvi[0, 0, :, kk:] == fill)
    # every row: ascending, in range, and no key left out has a higher score than a key taken
    lists = kvi[0, 0, :, :kk]
    assert np.all(np.diff(lists, axis=1) > 0) and lists.min() >= 0 and lists.max() < S
    for r in range(0, SB, max(1, SB // 16)):
        taken = np.zeros(S, bool)
        taken[lists[r]] = True
        if kk < S:
            assert score[0, 0, r, :S][taken].min() >= score[0, 0, r, :S][~taken].max()


def test_topk_rows_longer_than_the_register_path(dev):
    """More than 73728 keys per row: the select that re-reads its row from memory."""
    print("case topk long rows", flush=True)
    B, H, S, D, blk, select_k = 1, 1, 81000, 64, 128, 700
    q, k, _ = wl.randn_qkv(B, H, S, D, seed=5)
    kvi, kvn, score, qmean, fill = _run(dev, q, k, select_k, blk)
    want_qm, _ = orc.qblock_mean_scores(f32(q)[:, :, :256], f32(k)[:, :, :256], blk)
    assert np.array_equal(qmean[:, :, :2], want_qm[:, :, :2])
    rows = [0, 1, 317, 632]
    want_sel = orc.topk_select(score[0, 0, rows, :S], select_k)
    assert np.all(kvn == select_k)
    assert np.array_equal(kvi[0, 0, rows, :select_k], want_sel)


def test_topk_select_ties_and_wide_rows(dev):
    """Constant keys give equal scores everywhere: the lowest keys win; a second head with
    two score levels checks the boundary between the levels."""
    print("case topk ties", flush=True)
    B, H, S, D, blk = 1, 2, 3000, 64, 128
    q = torch.ones(B, H, S, D).bfloat16()
    k = torch.ones(B, H, S, D).bfloat16()
    k[0, 1, 1000:1100] = 2.0            # 100 keys with a higher score
    for select_k in (5, 150, 2999):
        kvi, kvn, score, _, _ = _run(dev, q, k, select_k, blk)
        assert np.all(kvn == select_k)
        assert np.array_equal(kvi[0, 0, :, :select_k], np.broadcast_to(np.arange(select_k), (24, select_k)))
        hi = np.arange(1000, 1100)
        lo = np.setdiff1d(np.arange(S), hi)
        want = np.sort(np.concatenate([hi[:select_k], lo[:max(0, select_k - 100)]]))
        assert np.array_equal(kvi[0, 1, :, :select_k], np.broadcast_to(want, (24, select_k)))


def test_attn_topkmask_functional_with_all_keys_is_dense(dev):
    """The model-facing call (python/spattn/sparseattn_functionals.py:39-48) with select_k = S
    keeps every key: dense attention."""
    print("case topk functional", flush=True)
    from fgattn_tk_cuda_amd.spattn import sparseattn_functionals as fn

    B, H, S, D = 1, 2, 640, 128
    q, k, v = (t.to(dev) for t in wl.randn_qkv(B, H, S, D, seed=21))
    o = fn.attn_topkmask_cuda(q, k, v, select_k=S, blocksz=128)
    want = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float())
    assert_close_o(f32(o), f32(want), "top-k with all keys vs SDPA")
    o2 = fn.attn_topkmask_cuda(q, k, v, select_k=200, blocksz=128)
    kvi, kvn = fn.mask_utils.qk_topkmask_indices_cuda(q, k, 200, blocksz=128)
    wo, _ = orc.sp_attn(f32(q), f32(k), f32(v), kvi.cpu().numpy(), kvn.cpu().numpy(), qblk=128)
    assert_close_o(f32(o2), wo, "top-k 200 vs oracle on the same lists")


def test_topk_argument_errors(dev):
    B, H, S, D = 1, 1, 256, 64
    q, k, _ = (t.to(dev) for t in wl.randn_qkv(B, H, S, D, seed=1))
    kvi = torch.zeros((B, H, 2, 128), dtype=torch.int32, device=dev)
    kvn = torch.zeros((B, H, 2), dtype=torch.int32, device=dev)
    score = torch.zeros((B, H, 2, 256), dtype=torch.bfloat16, device=dev)
    qmean = torch.zeros((B, H, 2, D), dtype=torch.bfloat16, device=dev)
    with pytest.raises(capi.SpattnError):
        capi.qk_topkmask_indices(kvi, kvn, score, qmean, q, k, 200, blocksz=128)      # lists too narrow
    with pytest.raises(capi.SpattnError):
        capi.qk_topkmask_indices(kvi, kvn, score[..., :200].contiguous(), qmean, q, k, 100, blocksz=128)  # score rows too short
    with pytest.raises(capi.SpattnError):
        capi.qk_topkmask_indices(kvi, kvn, score, qmean, q, k, 0, blocksz=128)
