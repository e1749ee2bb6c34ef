"""Seeded synthetic inputs for the benchmark configurations.

Everything is generated on the host with numpy (one ``default_rng(seed)`` per call) and
returned as torch CPU tensors; callers move them to the device.  The five named
configurations are those the benchmark description lists; ``CONFIGS`` gives their shapes.
"""
from __future__ import annotations

import math

import numpy as np
import torch

CONFIGS = {
    # name: B, H, N, D, dtype, qblk, kvblk
    "cfg1_plumbing": dict(B=1, H=4, S=1024, D=64, qblk=64, kvblk=64, density=0.25),
    "cfg2_dense": dict(B=4, H=16, S=4096, D=64),
    "cfg3_sparse_16k": dict(B=2, H=32, S=16384, D=128, qblk=64, kvblk=64, density=0.10),
    "cfg4_threshold_padded": dict(B=1, H=24, S=32760, D=64, keep=0.08),
    "cfg5_zipf_64k": dict(B=1, H=8, S=65536, D=128, qblk=128, kvblk=64, zipf_s=1.2, max_blocks=1024),
}


def ceil_div(a: int, b: int) -> int:
    return (a + b - 1) // b


def randn_qkv(B, H, S, D, seed=0, dtype=torch.bfloat16):
    """Q, K, V ~ iid N(0,1), cast to dtype."""
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(3):
        x = rng.standard_normal((B, H, S, D), dtype=np.float32)
        out.append(torch.from_numpy(x).to(dtype))
    return tuple(out)


def clustered_qkv(B, H, S, D, seed=0, kvblk=64, sigma=1.5, dtype=torch.bfloat16):
    """Q, V ~ N(0,1); K = N(0,1) + mu_J with one offset vector mu_J ~ N(0, sigma^2 I) per
    kvblk-key block J, so that score mass clusters in a few key blocks."""
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((B, H, S, D), dtype=np.float32)
    k = rng.standard_normal((B, H, S, D), dtype=np.float32)
    v = rng.standard_normal((B, H, S, D), dtype=np.float32)
    nb = ceil_div(S, kvblk)
    mu = rng.standard_normal((B, H, nb, D), dtype=np.float32) * np.float32(sigma)
    k += np.repeat(mu, kvblk, axis=2)[:, :, :S]
    return tuple(torch.from_numpy(x).to(dtype) for x in (q, k, v))


def _diag_block(i: int, qblk: int, kvblk: int, nk: int) -> int:
    return min(nk - 1, (i * qblk) // kvblk)


def uniform_block_lists(B, H, S, qblk, kvblk, count, seed=0):
    """Per (b,h,q-block): a sorted list of `count` distinct key-block ids that contains the
    diagonal block; the others are uniform.  Returns (idx int32 [B,H,nq,count], cnt int32 [B,H,nq])."""
    rng = np.random.default_rng(seed)
    nq, nk = ceil_div(S, qblk), ceil_div(S, kvblk)
    count = max(1, min(count, nk))
    keys = rng.random((B * H, nq, nk), dtype=np.float32)
    diag = np.array([_diag_block(i, qblk, kvblk, nk) for i in range(nq)])
    keys[:, np.arange(nq), diag] = -1.0
    idx = np.argpartition(keys, count - 1, axis=-1)[..., :count]
    idx = np.sort(idx, axis=-1).astype(np.int32).reshape(B, H, nq, count)
    cnt = np.full((B, H, nq), count, np.int32)
    return torch.from_numpy(idx), torch.from_numpy(cnt)


def ragged_block_lists(B, H, S, qblk, kvblk, counts, seed=0):
    """Like uniform_block_lists with a per-row count array [B,H,nq]; rows are padded with -1."""
    rng = np.random.default_rng(seed)
    nq, nk = ceil_div(S, qblk), ceil_div(S, kvblk)
    counts = np.clip(np.asarray(counts).reshape(B * H, nq), 1, nk)
    width = int(counts.max())
    idx = np.full((B * H, nq, width), -1, np.int32)
    for r in range(B * H):
        keys = rng.random((nq, nk), dtype=np.float32)
        diag = np.array([_diag_block(i, qblk, kvblk, nk) for i in range(nq)])
        keys[np.arange(nq), diag] = -1.0
        order = np.argsort(keys, axis=-1)
        for i in range(nq):
            c = int(counts[r, i])
            idx[r, i, :c] = np.sort(order[i, :c])
    return (torch.from_numpy(idx.reshape(B, H, nq, width)),
            torch.from_numpy(counts.astype(np.int32).reshape(B, H, nq)))


def zipf_counts(B, H, nq, s=1.2, lo=1, hi=1024, seed=0):
    rng = np.random.default_rng(seed)
    return np.clip(rng.zipf(s, size=(B, H, nq)), lo, hi).astype(np.int32)


def blocks_to_tokens(blk_idx, blk_cnt, S, kvblk=64, mask_stride=None):
    """Expand block lists to the token lists of the reference API: block j -> tokens
    kvblk*j .. kvblk*j+kvblk-1 (clipped to S); tail filled with mask_stride."""
    bi = blk_idx.numpy()
    bc = blk_cnt.numpy()
    B, H, nq, width = bi.shape
    if mask_stride is None:
        mask_stride = 128 * ceil_div(S, 128)
    tok = np.full((B, H, nq, mask_stride), mask_stride, np.int32)
    num = np.zeros((B, H, nq), np.int32)
    ar = np.arange(kvblk)
    for b in range(B):
        for h in range(H):
            for i in range(nq):
                c = int(bc[b, h, i])
                t = (bi[b, h, i, :c].astype(np.int64)[:, None] * kvblk + ar[None]).reshape(-1)
                t = t[t < S]
                tok[b, h, i, : t.size] = t
                num[b, h, i] = t.size
    return torch.from_numpy(tok), torch.from_numpy(num)


def permuted_all_index(B, H, S, qblk=128, seed=0):
    """A random permutation of all keys, shared by every q-block, padded with the fill
    value mask_stride - the list the reference's own sparse test uses."""
    rng = np.random.default_rng(seed)
    ms = 128 * ceil_div(S, 128)
    nq = ceil_div(S, qblk)
    row = np.full((ms,), ms, np.int32)
    row[:S] = rng.permutation(S).astype(np.int32)
    idx = np.broadcast_to(row, (B, H, nq, ms)).copy()
    num = np.full((B, H, nq), S, np.int32)
    return torch.from_numpy(idx), torch.from_numpy(num)


def kept_block_flops(total_blocks: int, qblk: int, kvblk: int, D: int) -> float:
    """QK^T + PV, 2 flops per multiply-add, per kept (q-block, kv-block) pair."""
    return float(total_blocks) * 4.0 * qblk * kvblk * D


def default_scale(D: int) -> float:
    return 1.0 / math.sqrt(D)
