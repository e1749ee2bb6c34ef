"""GPU parity of the attention kernels against the CPU oracle, through the C ABI."""
import numpy as np
import pytest
import torch

from fgattn_tk_cuda_amd import capi, workloads as wl
from oracle import spattn_oracle as orc
from helpers import assert_close_o, assert_close_stat, f32, to_dev

pytestmark = pytest.mark.gpu


def _run_tokens(dev, q, k, v, idx, num, qblk, kv_len=0):
    qd, kd, vd, idxd, numd = to_dev(dev, q, k, v, idx, num)
    o = torch.full_like(qd, float("nan"))
    lse = torch.full(q.shape[:3], float("nan"), device=dev)
    capi.sp_attn(o, qd, kd, vd, idxd, numd, lse=lse, qblk=qblk, kv_len=kv_len)
    torch.cuda.synchronize()
    return f32(o), f32(lse)


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("qblk", [64, 128])
@pytest.mark.parametrize("S", [256, 1000])
def test_sp_attn_permuted_all_keys_equals_sdpa(dev, D, qblk, S):
    """A permutation of all keys is dense attention (the reference's own sparse test)."""
    print("case sp_attn permuted", D, qblk, S, flush=True)
    B, H = 1, 2
    q, k, v = wl.randn_qkv(B, H, S, D, seed=1)
    idx, num = wl.permuted_all_index(B, H, S, qblk=qblk, seed=2)
    o, lse = _run_tokens(dev, q, k, v, idx, num, qblk)
    want = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float())
    assert_close_o(o, f32(want), "O vs SDPA")
    s = torch.einsum("bhmd,bhnd->bhmn", q.float(), k.float()) / D ** 0.5
    assert_close_stat(lse, f32(torch.logsumexp(s, -1)), "lse")


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("qblk", [64, 128])
def test_sp_attn_ragged_token_lists(dev, D, qblk):
    """Random token lists with counts that are not multiples of the 64-key tile."""
    print("case sp_attn ragged", D, qblk, flush=True)
    B, H, S = 2, 3, 777
    rng = np.random.default_rng(5)
    q, k, v = wl.randn_qkv(B, H, S, D, seed=3)
    ms = orc.padded_len(S)
    nq = orc.ceil_div(S, qblk)
    idx = np.full((B, H, nq, ms), ms, np.int32)
    num = np.zeros((B, H, nq), np.int32)
    for b in range(B):
        for h in range(H):
            for i in range(nq):
                c = int(rng.integers(1, S))
                if i == 0:
                    c = 1
                if i == 1:
                    c = 64
                if i == 2:
                    c = 65
                idx[b, h, i, :c] = rng.permutation(S)[:c]
                num[b, h, i] = c
    o, lse = _run_tokens(dev, q, k, v, torch.from_numpy(idx), torch.from_numpy(num), qblk)
    wo, wl_ = orc.sp_attn(f32(q), f32(k), f32(v), idx, num, qblk=qblk)
    assert_close_o(o, wo, "O vs oracle")
    assert_close_stat(lse, wl_, "lse vs oracle")


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("qblk", [64, 128])
def test_sp_attn_long_lists_with_entries_that_name_no_key(dev, D, qblk):
    """Lists of 13 to 25 tiles in which one entry in twelve is negative or past the end:
    such entries are skipped wherever they stand, also in the steady part of the tile loop."""
    print("case sp_attn holes", D, qblk, flush=True)
    B, H, S = 1, 3, 1600
    rng = np.random.default_rng(15)
    q, k, v = wl.randn_qkv(B, H, S, D, seed=16)
    ms = orc.padded_len(S)
    nq = orc.ceil_div(S, qblk)
    idx = np.full((B, H, nq, ms), ms, np.int32)
    num = np.zeros((B, H, nq), np.int32)
    for h in range(H):
        for i in range(nq):
            c = int(rng.integers(800, S))
            lst = rng.permutation(S)[:c].astype(np.int32)
            holes = rng.random(c) < 1.0 / 12
            lst[holes] = rng.choice(np.array([-1, -7, S, S + 5, 2 ** 30], np.int32), int(holes.sum()))
            idx[0, h, i, :c] = lst
            num[0, h, i] = c
    o, lse = _run_tokens(dev, q, k, v, torch.from_numpy(idx), torch.from_numpy(num), qblk)
    wo, wl_ = orc.sp_attn(f32(q), f32(k), f32(v), idx, num, qblk=qblk)
    assert_close_o(o, wo, "O vs oracle")
    assert_close_stat(lse, wl_, "lse vs oracle")


def test_sp_attn_single_key_returns_v_row(dev):
    print("case sp_attn single key", flush=True)
    B, H, S, D = 1, 1, 256, 128
    q, k, v = wl.randn_qkv(B, H, S, D, seed=7)
    ms = 256
    idx = np.full((B, H, 2, ms), ms, np.int32)
    idx[0, 0, 0, 0] = 17
    idx[0, 0, 1, 0] = 200
    num = np.ones((B, H, 2), np.int32)
    o, _ = _run_tokens(dev, q, k, v, torch.from_numpy(idx), torch.from_numpy(num), 128)
    want = np.concatenate([np.repeat(f32(v)[0, 0, 17:18], 128, 0), np.repeat(f32(v)[0, 0, 200:201], 128, 0)])
    assert np.array_equal(o[0, 0], want)


def test_sp_attn_empty_list_and_bad_indices(dev):
    """n = 0 gives O = 0 and lse = -inf; entries >= S inside the count are ignored."""
    print("case sp_attn empty", flush=True)
    B, H, S, D = 1, 2, 384, 64
    q, k, v = wl.randn_qkv(B, H, S, D, seed=8)
    ms = 384
    idx = np.full((B, H, 3, ms), ms, np.int32)
    num = np.zeros((B, H, 3), np.int32)
    idx[:, :, 1, :100] = np.arange(100)
    idx[:, :, 1, 10:20] = 5000          # out of range inside the count
    num[:, :, 1] = 100
    idx[:, :, 2, :300] = np.arange(300)
    num[:, :, 2] = 300
    o, lse = _run_tokens(dev, q, k, v, torch.from_numpy(idx), torch.from_numpy(num), 128)
    wo, wlse = orc.sp_attn(f32(q), f32(k), f32(v), idx, num, qblk=128)
    assert np.all(o[:, :, :128] == 0) and np.all(np.isneginf(lse[:, :, :128]))
    assert_close_o(o, wo, "O")
    assert_close_stat(lse, wlse, "lse")


def test_sp_attn_duplicate_and_permutation_invariance(dev):
    print("case sp_attn invariance", flush=True)
    B, H, S, D = 1, 2, 512, 128
    q, k, v = wl.randn_qkv(B, H, S, D, seed=9)
    rng = np.random.default_rng(10)
    ms = 512
    nq = 4
    base = np.full((B, H, nq, ms), ms, np.int32)
    num = np.full((B, H, nq), 150, np.int32)
    for i in range(nq):
        base[:, :, i, :150] = rng.permutation(S)[:150]
    perm = base.copy()
    for i in range(nq):
        perm[:, :, i, :150] = perm[:, :, i, rng.permutation(150)]
    dup = base.copy()
    dup[:, :, :, 150:300] = base[:, :, :, :150]
    o0, l0 = _run_tokens(dev, q, k, v, torch.from_numpy(base), torch.from_numpy(num), 128)
    o1, l1 = _run_tokens(dev, q, k, v, torch.from_numpy(perm), torch.from_numpy(num), 128)
    o2, l2 = _run_tokens(dev, q, k, v, torch.from_numpy(dup), torch.from_numpy(num * 2), 128)
    assert_close_o(o1, o0, "permuted list")
    assert_close_o(o2, o0, "duplicated list")
    assert_close_stat(l2, l0 + np.log(2.0), "lse of duplicated list")


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("qblk", [64, 128])
@pytest.mark.parametrize("S", [1024, 1000])
def test_sp_attn_blocks_matches_oracle_and_token_path(dev, D, qblk, S):
    print("case sp_attn blocks", D, qblk, S, flush=True)
    B, H = 1, 3
    q, k, v = wl.randn_qkv(B, H, S, D, seed=11)
    nk = orc.ceil_div(S, 64)
    counts = np.random.default_rng(12).integers(1, nk + 1, size=(B, H, orc.ceil_div(S, qblk)))
    bi, bc = wl.ragged_block_lists(B, H, S, qblk, 64, counts, seed=13)
    qd, kd, vd, bid, bcd = to_dev(dev, q, k, v, bi, bc)
    o = torch.full_like(qd, float("nan"))
    lse = torch.full(q.shape[:3], float("nan"), device=dev)
    capi.sp_attn_blocks(o, qd, kd, vd, bid, bcd, lse=lse, qblk=qblk)
    tok, num = wl.blocks_to_tokens(bi, bc, S)
    wo, wlse = orc.sp_attn(f32(q), f32(k), f32(v), tok.numpy(), num.numpy(), qblk=qblk)
    assert_close_o(f32(o), wo, "block path vs oracle")
    assert_close_stat(f32(lse), wlse, "lse")
    o2, _ = _run_tokens(dev, q, k, v, tok, num, qblk)
    assert_close_o(o2, f32(o), "token path vs block path")


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("qblk", [64, 128])
@pytest.mark.parametrize("growth", ["ramp", "jump"])
def test_sp_attn_scores_that_outgrow_the_running_maximum(dev, D, qblk, growth):
    """Keys whose scores grow along the list: the exponent reference has to move on later tiles
    (a moderate ramp), also after a jump large enough to overflow exp2 against the old reference."""
    print("case sp_attn growing scores", D, qblk, growth, flush=True)
    B, H, S = 1, 2, 1024
    q, k, v = wl.randn_qkv(B, H, S, D, seed=31)
    kf = k.float()
    blk = torch.arange(S) // 64
    if growth == "ramp":
        kf = kf * (1.0 + 0.75 * blk.float()).view(1, 1, S, 1)          # scores up to ~13x larger
    else:
        kf = kf * torch.where(blk >= 9, 600.0, 1.0).view(1, 1, S, 1)   # exponent jumps by thousands
    k = kf.to(torch.bfloat16)
    nk = S // 64
    counts = np.full((B, H, orc.ceil_div(S, qblk)), nk)
    bi, bc = wl.ragged_block_lists(B, H, S, qblk, 64, counts, seed=32)   # every block, ascending
    qd, kd, vd, bid, bcd = to_dev(dev, q, k, v, bi, bc)
    o = torch.full_like(qd, float("nan"))
    lse = torch.full(q.shape[:3], float("nan"), device=dev)
    capi.sp_attn_blocks(o, qd, kd, vd, bid, bcd, lse=lse, qblk=qblk)
    tok, num = wl.blocks_to_tokens(bi, bc, S)
    wo, wlse = orc.sp_attn(f32(q), f32(k), f32(v), tok.numpy(), num.numpy(), qblk=qblk)
    assert_close_o(f32(o), wo, "growing scores, block path")
    assert_close_stat(f32(lse), wlse, "lse", atol=1e-3)
    o2, _ = _run_tokens(dev, q, k, v, tok, num, qblk)
    assert_close_o(o2, wo, "growing scores, token path")
    od = torch.full_like(qd, float("nan"))
    capi.full_attn(od, qd, kd, vd)
    assert_close_o(f32(od), wo, "growing scores, dense path")


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("qblk", [64, 128])
def test_sp_attn_first_tiles_without_a_key(dev, D, qblk):
    """Lists that open with entries naming no key (ids beyond the sequence, or beyond a short kv
    length): the row gets its exponent reference from the first tile that has a key, and the keys
    of that tile and of every later one count."""
    print("case sp_attn keyless first tiles", D, qblk, flush=True)
    B, H, S = 1, 2, 512
    rng = np.random.default_rng(41)
    q, k, v = wl.randn_qkv(B, H, S, D, seed=40)
    nq = orc.ceil_div(S, qblk)
    ms = orc.padded_len(S)
    idx = np.full((B, H, nq, ms), ms, np.int32)
    num = np.zeros((B, H, nq), np.int32)
    for h in range(H):
        for i in range(nq):
            dead = 32 * int(rng.integers(1, 7))            # 32 .. 192 leading entries without a key
            live = int(rng.integers(1, 200))
            idx[0, h, i, :dead] = S + rng.integers(0, 100, size=dead)
            idx[0, h, i, dead:dead + live] = rng.integers(0, S, size=live)
            num[0, h, i] = dead + live
    o, lse = _run_tokens(dev, q, k, v, torch.from_numpy(idx), torch.from_numpy(num), qblk)
    wo, wlse = orc.sp_attn(f32(q), f32(k), f32(v), idx, num, qblk=qblk)
    assert_close_o(o, wo, "keyless first tiles, O")
    assert_close_stat(lse, wlse, "keyless first tiles, lse", atol=1e-3)
    # the same through a short kv length: most entries of a random list name no key
    idx2 = np.full((B, H, nq, ms), ms, np.int32)
    num2 = np.full((B, H, nq), 300, np.int32)
    idx2[..., :300] = rng.integers(0, S, size=(B, H, nq, 300))
    for kv_len in (39, 64, 65):
        o2, lse2 = _run_tokens(dev, q, k, v, torch.from_numpy(idx2), torch.from_numpy(num2), qblk, kv_len=kv_len)
        w2, wl2 = orc.sp_attn(f32(q), f32(k), f32(v), np.where(idx2 < kv_len, idx2, ms), num2, qblk=qblk)
        assert_close_o(o2, w2, "kv_len %d, O" % kv_len)
        assert_close_stat(lse2, wl2, "kv_len %d, lse" % kv_len, atol=1e-3)


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("S,kv_len", [(512, 0), (1000, 0), (1000, 900), (130, 0)])
def test_full_attn_and_stats(dev, D, S, kv_len):
    print("case full_attn", D, S, kv_len, flush=True)
    B, H = 2, 2
    q, k, v = wl.randn_qkv(B, H, S, D, seed=21)
    qd, kd, vd = to_dev(dev, q, k, v)
    kv = kv_len or S
    want = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float()[:, :, :kv], v.float()[:, :, :kv])
    o = torch.full_like(qd, float("nan"))
    lse = torch.full(q.shape[:3], float("nan"), device=dev)
    capi.full_attn(o, qd, kd, vd, lse=lse, kv_len=kv_len)
    assert_close_o(f32(o), f32(want), "full_attn vs SDPA")
    s = torch.einsum("bhmd,bhnd->bhmn", q.float(), k.float()[:, :, :kv]) / D ** 0.5
    assert_close_stat(f32(lse), f32(torch.logsumexp(s, -1)), "lse")

    Sp = orc.padded_len(S)
    o2 = torch.full_like(qd, float("nan"))
    mx = torch.full((B, H, 1, Sp), float("nan"), device=dev)
    dn = torch.full((B, H, 1, Sp), float("nan"), device=dev)
    capi.fullattn_maxq_denom(o2, mx, dn, qd, kd, vd, kv_len=kv_len)
    assert_close_o(f32(o2), f32(want), "fullattn_maxq_denom O")
    wmx, wdn = orc.maxq_denom(f32(q), f32(k), kv_len=kv)
    assert_close_stat(f32(mx), wmx, "max_q (fused)", atol=1e-4)
    assert_close_stat(f32(dn), wdn, "denom (fused)")

    mx2 = torch.full((B, H, 1, Sp), float("nan"), device=dev)
    dn2 = torch.full((B, H, 1, Sp), float("nan"), device=dev)
    capi.maxq_denom(mx2, dn2, qd, kd, kv_len=kv_len)
    assert_close_stat(f32(mx2), wmx, "max_q", atol=1e-4)
    assert_close_stat(f32(dn2), wdn, "denom")
    # pad rows: max 0, denominator -inf
    assert np.all(f32(mx2)[..., S:] == 0) and np.all(np.isneginf(f32(dn2)[..., S:]))


def test_reference_named_entry_points(dev):
    """The seven reference-named symbols run on the default stream with q-block 128."""
    print("case reference-named entry points", flush=True)
    B, H, S, D = 1, 2, 300, 128
    q, k, v = wl.randn_qkv(B, H, S, D, seed=31)
    qd, kd, vd = to_dev(dev, q, k, v)
    lib = capi.load()
    torch.cuda.synchronize()
    o = torch.zeros_like(qd)
    lib.attn_fwd_wg_impl(o.data_ptr(), qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), B, H, S, D)
    torch.cuda.synchronize()
    assert lib.spattn_last_status() == 0
    want = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float())
    assert_close_o(f32(o), f32(want), "attn_fwd_wg_impl")

    SB, ms = 3, 384
    idx = torch.zeros((B, H, SB, ms), dtype=torch.int32, device=dev)
    num = torch.zeros((B, H, SB), dtype=torch.int32, device=dev)
    lib.allindex_mask_impl(idx.data_ptr(), num.data_ptr(), B, H, SB, S)
    torch.cuda.synchronize()
    wi, wn = orc.all_index_mask(B, H, SB, S, ms)
    assert np.array_equal(idx.cpu().numpy(), wi) and np.array_equal(num.cpu().numpy(), wn)
    o2 = torch.zeros_like(qd)
    lib.attn_sparse_fwd_wg_impl(o2.data_ptr(), qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), idx.data_ptr(),
                                num.data_ptr(), ms, B, H, S, D)
    torch.cuda.synchronize()
    assert_close_o(f32(o2), f32(want), "identity list sparse == dense")

    Sp = 384
    mx = torch.zeros((B, H, 1, Sp), device=dev)
    dn = torch.zeros((B, H, 1, Sp), device=dev)
    o3 = torch.zeros_like(qd)
    lib.attn_maxq_denom_impl(o3.data_ptr(), mx.data_ptr(), dn.data_ptr(), qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), B, H, S, D)
    mx2 = torch.zeros_like(mx)
    dn2 = torch.zeros_like(dn)
    lib.maxq_denom_impl(mx2.data_ptr(), dn2.data_ptr(), qd.data_ptr(), kd.data_ptr(), B, H, S, D)
    torch.cuda.synchronize()
    wmx, wdn = orc.maxq_denom(f32(q), f32(k))
    assert_close_o(f32(o3), f32(want), "attn_maxq_denom_impl O")
    for a, b_ in ((mx, wmx), (mx2, wmx)):
        assert_close_stat(f32(a), b_, "max_q", atol=1e-4)
    for a, b_ in ((dn, wdn), (dn2, wdn)):
        assert_close_stat(f32(a), b_, "denom")

    thr = 1.0 / S
    mask = torch.zeros((B, H, SB, ms), dtype=torch.int32, device=dev)
    lib.booleanmask_128_impl(mask.data_ptr(), thr, ms, mx2.data_ptr(), dn2.data_ptr(), qd.data_ptr(), kd.data_ptr(), B, H, S, D)
    kvi = torch.full((B, H, SB, ms), ms, dtype=torch.int32, device=dev)
    kvn = torch.zeros((B, H, SB), dtype=torch.int32, device=dev)
    lib.booleanmask_to_indexmask_impl(kvi.data_ptr(), kvn.data_ptr(), mask.data_ptr(), B, H, S, SB, ms)
    torch.cuda.synchronize()
    wi, wn = orc.booleanmask_to_indexmask(mask.cpu().numpy(), S)
    assert np.array_equal(kvi.cpu().numpy(), wi) and np.array_equal(kvn.cpu().numpy(), wn)


def test_argument_errors(dev):
    print("case argument errors", flush=True)
    q = torch.zeros((1, 1, 128, 96), dtype=torch.bfloat16, device=dev)
    with pytest.raises(capi.SpattnError) as e:
        capi.full_attn(torch.zeros_like(q), q, q, q)
    assert e.value.status == -2
    q = torch.zeros((1, 1, 128, 64), dtype=torch.bfloat16, device=dev)
    idx = torch.zeros((1, 1, 1, 100), dtype=torch.int32, device=dev)
    num = torch.zeros((1, 1, 1), dtype=torch.int32, device=dev)
    with pytest.raises(capi.SpattnError) as e:
        capi.sp_attn(torch.zeros_like(q), q, q, q, idx, num)
    assert e.value.status == -3
    with pytest.raises(ValueError):
        capi.sp_attn(torch.zeros_like(q), q, q, q, idx.cpu(), num)
    with pytest.raises(ValueError):
        capi.full_attn(torch.zeros_like(q), q.float(), q, q)
