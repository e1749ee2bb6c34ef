"""Seeded random shapes and lists for the sparse-attention entry points, against the CPU oracle.

Every case draws its own B, H, S, D, q-block size, kv length and lists (empty lists, one-key
lists, duplicates, ids outside the sequence, a list as long as the sequence), on the token-list
and on the block-list entry point, with and without a caller-given work order.
"""
import numpy as np
import pytest
import torch

from fgattn_tk_cuda_amd import capi, workloads as wl
from oracle import spattn_oracle as orc
from helpers import assert_close_o, assert_close_stat, f32, to_dev

pytestmark = pytest.mark.gpu


def _draw_shape(rng):
    B = int(rng.integers(1, 3))
    H = int(rng.integers(1, 4))
    S = int(rng.choice([65, 100, 128, 191, 192, 257, 320, 449, 512, 700]))
    D = int(rng.choice([64, 128]))
    qblk = int(rng.choice([64, 128]))
    kv_len = int(rng.choice([0, 0, S, int(rng.integers(1, S + 1))]))
    return B, H, S, D, qblk, kv_len


@pytest.mark.parametrize("seed", range(24))
def test_token_lists_random(dev, seed):
    rng = np.random.default_rng(1000 + seed)
    B, H, S, D, qblk, kv_len = _draw_shape(rng)
    print("case random tokens", seed, B, H, S, D, qblk, kv_len, flush=True)
    kv = kv_len or S
    q, k, v = wl.randn_qkv(B, H, S, D, seed=seed)
    nq = orc.ceil_div(S, qblk)
    ms = orc.padded_len(S)
    idx = np.full((B, H, nq, ms), ms, np.int32)
    num = np.zeros((B, H, nq), np.int32)
    for b in range(B):
        for h in range(H):
            for i in range(nq):
                kind = int(rng.integers(6))
                if kind == 0:
                    c = 0
                elif kind == 1:
                    c = 1
                elif kind == 2:
                    c = min(ms, S)
                else:
                    c = int(rng.integers(1, min(ms, S) + 1))
                ids = rng.integers(0, S, size=c)
                if kind == 3 and c > 4:          # duplicates
                    ids[c // 2:] = ids[: c - c // 2]
                if kind == 4 and c > 2:          # ids outside the sequence / negative
                    ids[rng.integers(0, c, size=max(1, c // 8))] = S + int(rng.integers(0, 50))
                    ids[int(rng.integers(0, c))] = -1
                idx[b, h, i, :c] = ids
                num[b, h, i] = c
    idx_t, num_t = torch.from_numpy(idx), torch.from_numpy(num)
    qd, kd, vd, idxd, numd = to_dev(dev, q, k, v, idx_t, num_t)
    o = torch.full_like(qd, float("nan"))
    lse = torch.full(q.shape[:3], float("nan"), device=dev)
    order = None
    if seed % 3 == 0:
        order = torch.from_numpy(rng.permutation(B * H * nq).astype(np.int32)).to(dev)
    capi.sp_attn(o, qd, kd, vd, idxd, numd, lse=lse, qblk=qblk, kv_len=kv_len, order=order)
    torch.cuda.synchronize()
    # the oracle drops ids >= S; keys at or beyond kv_len do not exist either
    oidx = np.where((idx >= 0) & (idx < kv), idx, ms).astype(np.int32)
    wo, wlse = orc.sp_attn(f32(q), f32(k), f32(v), oidx, num, qblk=qblk)
    assert_close_o(f32(o), wo, "random token lists, O")
    assert_close_stat(f32(lse), wlse, "random token lists, lse", atol=2e-3)


@pytest.mark.parametrize("seed", range(24))
def test_block_lists_random(dev, seed):
    rng = np.random.default_rng(2000 + seed)
    B, H, S, D, qblk, kv_len = _draw_shape(rng)
    print("case random blocks", seed, B, H, S, D, qblk, kv_len, flush=True)
    kv = kv_len or S
    q, k, v = wl.randn_qkv(B, H, S, D, seed=100 + seed)
    nq = orc.ceil_div(S, qblk)
    nk = orc.ceil_div(S, 64)
    maxb = int(rng.integers(1, nk + 3))
    bi = np.zeros((B, H, nq, maxb), np.int32)
    bc = np.zeros((B, H, nq), np.int32)
    for b in range(B):
        for h in range(H):
            for i in range(nq):
                kind = int(rng.integers(5))
                c = 0 if kind == 0 else (1 if kind == 1 else int(rng.integers(1, maxb + 1)))
                ids = rng.integers(0, nk, size=c)
                if kind == 2 and c > 1:
                    ids = np.sort(ids)
                if kind == 3 and c > 1:          # block ids outside the sequence
                    ids[int(rng.integers(0, c))] = nk + int(rng.integers(0, 5))
                    ids[int(rng.integers(0, c))] = -2
                bi[b, h, i, :c] = ids
                bc[b, h, i] = c
    bi_t, bc_t = torch.from_numpy(bi), torch.from_numpy(bc)
    qd, kd, vd, bid, bcd = to_dev(dev, q, k, v, bi_t, bc_t)
    o = torch.full_like(qd, float("nan"))
    lse = torch.full(q.shape[:3], float("nan"), device=dev)
    order = None
    if seed % 3 == 1:
        order = torch.from_numpy(rng.permutation(B * H * nq).astype(np.int32)).to(dev)
    capi.sp_attn_blocks(o, qd, kd, vd, bid, bcd, lse=lse, qblk=qblk, kv_len=kv_len, order=order)
    torch.cuda.synchronize()
    # expected keys: the existing keys (< kv) of every listed block that lies inside the sequence
    ms = orc.padded_len(S)
    stride = max(ms, maxb * 64)
    tok = np.full((B, H, nq, stride), stride, np.int32)
    num = np.zeros((B, H, nq), np.int32)
    for b in range(B):
        for h in range(H):
            for i in range(nq):
                keys = []
                for j in bi[b, h, i, : bc[b, h, i]]:
                    if 0 <= j and j * 64 < kv:
                        keys.extend(range(j * 64, min(kv, j * 64 + 64)))
                tok[b, h, i, : len(keys)] = keys
                num[b, h, i] = len(keys)
    tok = np.where(tok < S, tok, S + 1)
    wo, wlse = orc.sp_attn(f32(q), f32(k), f32(v), tok, num, qblk=qblk)
    assert_close_o(f32(o), wo, "random block lists, O")
    assert_close_stat(f32(lse), wlse, "random block lists, lse", atol=2e-3)


@pytest.mark.parametrize("seed", range(6))
def test_operator_sp_attn_equals_the_c_abi_bit_for_bit(dev, seed):
    """torch.ops.cuda_attn.sp_attn (which orders the q-blocks by list length and launches the
    ordered entry point) against the plain C-ABI launch on the same ragged lists."""
    import fgattn_tk_cuda_amd.spattn.cuda_attn  # noqa: F401
    rng = np.random.default_rng(7000 + seed)
    B, H = int(rng.integers(1, 3)), int(rng.integers(1, 4))
    S = int(rng.choice([192, 449, 700, 1024]))
    D = int(rng.choice([64, 128]))
    qblk = int(rng.choice([64, 128]))
    print("case op vs C ABI", seed, B, H, S, D, qblk, flush=True)
    q, k, v = wl.randn_qkv(B, H, S, D, seed=200 + seed)
    nq = orc.ceil_div(S, qblk)
    ms = orc.padded_len(S)
    idx = np.full((B, H, nq, ms), ms, np.int32)
    num = np.zeros((B, H, nq), np.int32)
    for b in range(B):
        for h in range(H):
            for i in range(nq):
                # list lengths spread over more than a factor of two, so that the order is not the default one
                c = int(rng.choice([0, 1, 17, 64, 200, S])) if rng.random() < 0.5 else int(rng.integers(1, S + 1))
                c = min(c, ms)
                idx[b, h, i, :c] = rng.integers(0, S, size=c)
                num[b, h, i] = c
    qd, kd, vd, idxd, numd = to_dev(dev, q, k, v, torch.from_numpy(idx), torch.from_numpy(num))
    o_op = torch.full_like(qd, float("nan"))
    torch.ops.cuda_attn.sp_attn(o_op, qd, kd, vd, idxd, numd)
    o_c = torch.full_like(qd, float("nan"))
    capi.sp_attn(o_c, qd, kd, vd, idxd, numd, qblk=qblk)
    torch.cuda.synchronize()
    assert torch.equal(o_op.view(torch.int16), o_c.view(torch.int16))
    wo, _ = orc.sp_attn(f32(q), f32(k), f32(v), idx, num, qblk=qblk)
    assert_close_o(f32(o_op), wo, "operator sp_attn vs oracle")
