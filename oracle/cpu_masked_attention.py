"""CPU baseline: the reference's dense-masked PyTorch attention.  TEST INFRASTRUCTURE ONLY.

Restates the algorithm of the reference's Python check (python/test_mask.py:37-54 and
python/spattn/mask_utils.py:225-245): per head, ``einsum('md,nd->mn')`` scores, softmax,
block mask, ``einsum('mn,nd->md')`` - in the renormalised form (scores outside the kept
blocks set to -inf before the softmax), which is what the sparse kernel computes
(include/sparseattn_asyncgatherload_padded.cuh:236-249).  Used only as the checker in tests
and as the timed ``cpu_baseline`` of bench.py; pinned against the numpy oracle in
tests/test_oracle.py.
"""
from __future__ import annotations

import torch


def block_mask_rows(blk_idx, blk_cnt, r0, r1, qblk, kvblk, S):
    """Boolean [r1-r0, S] mask of the kept keys for query rows r0..r1-1 of one head."""
    nk = (S + kvblk - 1) // kvblk
    mask = torch.zeros((r1 - r0, nk), dtype=torch.bool)
    for i in range(r0 // qblk, (r1 + qblk - 1) // qblk):
        c = int(blk_cnt[i])
        rows = slice(max(i * qblk, r0) - r0, min((i + 1) * qblk, r1) - r0)
        mask[rows, blk_idx[i, :c].long()] = True
    return mask.repeat_interleave(kvblk, dim=1)[:, :S]


def masked_attention_rows(q, k, v, blk_idx, blk_cnt, r0, r1, qblk, kvblk, scale=None):
    """O[r0:r1] of one head: q,k,v fp32 [S,D]; block lists of that head."""
    S, D = k.shape
    if scale is None:
        scale = D ** -0.5
    s = torch.einsum("md,nd->mn", q[r0:r1], k) * scale
    s.masked_fill_(~block_mask_rows(blk_idx, blk_cnt, r0, r1, qblk, kvblk, S), float("-inf"))
    p = torch.softmax(s, dim=-1)
    return torch.einsum("mn,nd->md", p, v)
