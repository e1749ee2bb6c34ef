"""Writes tests/golden/*.npz: small inputs with expected outputs computed here by plain
fp64 loops over the definitions (no oracle code, no library code), so that the oracle and
the GPU path are both checked against something independent.

    python tests/golden/make_fixtures.py

The reference repository holds no vectors of its own for these operators; its tests only
print differences against torch on random inputs.
"""
from __future__ import annotations

import math
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def bf16(x):
    """Round fp32 to bf16 (nearest even), as fp32."""
    u = np.asarray(x, np.float32).view(np.uint32)
    r = ((u >> 16) & 1) + 0x7FFF
    return ((u + r) & 0xFFFF0000).astype(np.uint32).view(np.float32)


def attention_rows(q, k, v, rows, keys, scale):
    """softmax(q_r . k_c * scale over c in keys) v, and its log-sum-exp, in fp64 loops."""
    D = q.shape[1]
    out = np.zeros((len(rows), D))
    lse = np.full(len(rows), -np.inf)
    for a, r in enumerate(rows):
        s = [sum(float(q[r, d]) * float(k[c, d]) for d in range(D)) * scale for c in keys]
        if not s:
            continue
        m = max(s)
        w = [math.exp(x - m) for x in s]
        z = sum(w)
        lse[a] = m + math.log(z)
        for wi, c in zip(w, keys):
            out[a] += wi / z * v[c].astype(np.float64)
    return out, lse


def make_sparse(seed, S, D, qblk, lists):
    rng = np.random.default_rng(seed)
    q, k, v = (bf16(rng.standard_normal((S, D), dtype=np.float32)) for _ in range(3))
    scale = 1.0 / math.sqrt(D)
    nq = (S + qblk - 1) // qblk
    ms = 128 * ((S + 127) // 128)
    idx = np.full((nq, ms), ms, np.int32)
    num = np.zeros((nq,), np.int32)
    o = np.zeros((S, D))
    lse = np.full((S,), -np.inf)
    for i in range(nq):
        lst = lists(rng, i)
        idx[i, : len(lst)] = lst
        num[i] = len(lst)
        rows = list(range(i * qblk, min(S, (i + 1) * qblk)))
        keys = [int(c) for c in lst if 0 <= c < S]
        oo, ll = attention_rows(q, k, v, rows, keys, scale)
        o[rows] = oo
        lse[rows] = ll
    return dict(q=q, k=k, v=v, kv_indices=idx[None, None], kv_num_indices=num[None, None], o=o.astype(np.float32),
                lse=lse.astype(np.float32), qblk=np.int32(qblk))


def make_prepass(seed, S, D, thresh_quantile):
    """max_q / denom (fp64), the vote mask of the eight 16-row groups, and the index lists."""
    rng = np.random.default_rng(seed)
    q = bf16(rng.standard_normal((S, D), dtype=np.float32))
    k = bf16(rng.standard_normal((S, D), dtype=np.float32) + np.repeat(rng.standard_normal((S // 16 + 1, D)), 16, 0)[:S].astype(np.float32))
    scale = 1.0 / math.sqrt(D)
    s = q.astype(np.float64) @ k.astype(np.float64).T
    max_q = s.max(1)
    denom = np.exp((s - max_q[:, None]) * scale).sum(1)
    p = np.exp((s - max_q[:, None]) * scale) / denom[:, None]
    SB = (S + 127) // 128
    ms = 128 * SB
    thresh = float(np.quantile(np.stack([p[i * 128:(i + 1) * 128].max(0) for i in range(SB)]), thresh_quantile))
    votes = np.zeros((SB, ms), np.int32)
    pmax = np.zeros((SB, S))
    for i in range(SB):
        blk = p[i * 128:(i + 1) * 128]
        pmax[i] = blk.max(0)
        for w in range(0, blk.shape[0], 16):
            votes[i, :S] += blk[w:w + 16].max(0) > thresh
    idx = np.full((SB, ms), ms, np.int32)
    num = np.zeros((SB,), np.int32)
    for i in range(SB):
        kept = [c for c in range(S) if votes[i, c] > 0]
        idx[i, : len(kept)] = kept
        num[i] = len(kept)
    return dict(q=q, k=k, max_q=max_q.astype(np.float32), denom=denom.astype(np.float32), thresh=np.float32(thresh),
                votes=votes[None, None], pmax=pmax.astype(np.float32)[None, None], kv_indices=idx[None, None],
                kv_num_indices=num[None, None])


def main():
    S = 200
    np.savez_compressed(os.path.join(HERE, "sparse_d64_q64.npz"),
                        **make_sparse(11, S, 64, 64, lambda rng, i: rng.permutation(S)[: [1, 70, 130, 199][i % 4]]))
    np.savez_compressed(os.path.join(HERE, "sparse_d128_q128.npz"),
                        **make_sparse(12, S, 128, 128, lambda rng, i: np.concatenate([rng.permutation(S)[:90], [S + 5, 10 ** 6]])))
    np.savez_compressed(os.path.join(HERE, "dense_d64.npz"),
                        **make_sparse(13, 130, 64, 128, lambda rng, i: np.arange(130)))
    np.savez_compressed(os.path.join(HERE, "prepass_d64.npz"), **make_prepass(14, 200, 64, 0.7))
    np.savez_compressed(os.path.join(HERE, "prepass_d128.npz"), **make_prepass(15, 136, 128, 0.5))


if __name__ == "__main__":
    main()
