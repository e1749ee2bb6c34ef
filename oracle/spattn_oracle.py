"""CPU oracle for the block-sparse attention hot path.  TEST INFRASTRUCTURE ONLY.

This module restates, in numpy, what the reference kernels of
sankeerth95/fgattn_tk_cuda compute.  It is the checker used by ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py``; the
shipped library never imports it and has no CPU fallback.

Every function cites the reference file:line it follows.  How each function is
pinned (none of them is "parity unpinned"):

* ``sp_attn`` / ``full_attn``  - identity or permuted full lists reduce to
  ``torch.nn.functional.scaled_dot_product_attention`` (the reference's own
  check, python/test/test_extension.py:10-31,61-89); fp64 brute-force loops on
  tiny inputs; single-index list returns the V row; duplicated list and
  permuted list leave O unchanged.
* ``maxq_denom``               - closed forms of the reference's own test
  (python/test/spattn/test_mask_utils.py:33-56) recomputed with torch.
* ``booleanmask_128``          - equals max-pooling a thresholded torch softmax
  over 128 rows (python/spattn/mask_utils.py:126-142,206-222), vote count
  checked by brute force over the eight 16-row groups.
* ``booleanmask_to_indexmask`` - integer exact; ``np.flatnonzero`` per row and
  a pure-Python loop on small inputs.
* ``all_index_mask``           - ``arange`` closed form (include/utils.cuh:73-93).
* ``booleanmask_rows``          - for 128-row q-blocks it is ``booleanmask_128 > 0``; for 64-row
  q-blocks the OR of its two halves is the 128-row mask, and it equals max-pooling a
  thresholded torch softmax over 64 rows.
* ``block_mask_from_votes`` / ``block_lists_from_mask`` - integer exact; pure-Python loops over
  every (row, block, key) on small inputs, ragged last block and keys >= seq included.
* ``pack_mask`` / ``unpack_mask`` / ``packedmask_to_indexmask`` - ``numpy.packbits`` and round trips.
* ``qblock_mean_scores``       - the reference's own torch expressions
  (python/spattn/mask_utils.py:390-410) evaluated in bf16 on the CPU.
* ``topk_select``              - the multiset of selected scores equals
  ``torch.topk(...).values`` (python/spattn/mask_utils.py:412); brute force on tiny rows.
"""
from __future__ import annotations

import math

import numpy as np

QBLK_REF = 128          # q-block of the reference kernels (sparseattn_asyncgatherload_padded.cuh:82)
LOG2E = 1.4426950408889634


def bf16_round(x: np.ndarray) -> np.ndarray:
    """Round fp32 to the nearest bf16 (ties to even), returned as fp32."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    bias = ((u >> np.uint32(16)) & np.uint32(1)) + np.uint32(0x7FFF)
    out = ((u + bias) & np.uint32(0xFFFF0000)).view(np.float32)
    return np.where(np.isfinite(x), out, x)


def bf16_round_up(x: np.ndarray) -> np.ndarray:
    """The smallest bf16 that is not below x (round toward +infinity), returned as fp32; infinities
    stay.  The form in which the statistics sweeps of this library store their per-block maxima
    (no counterpart in the reference, whose second sweep recomputes the scores instead).  Pinned
    in tests/test_oracle.py by the defining property: the result has a bf16 bit pattern, is >= x,
    and the next bf16 below it is < x."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    neg = (u >> np.uint64(31)) != 0
    up = np.where(neg, u, u + np.uint64(0xFFFF)) & np.uint64(0xFFFF0000)
    out = up.astype(np.uint32).view(np.float32)
    return np.where(np.isfinite(x), out, x)


def ceil_div(a: int, b: int) -> int:
    return (a + b - 1) // b


def padded_len(seq: int, blk: int = 128) -> int:
    """Sp = 128*ceil(S/128) (python/spattn/mask_utils.py:314)."""
    return blk * ceil_div(seq, blk)


def _softmax_rows(scores: np.ndarray, scale: float, round_p: bool):
    """Online-softmax result of the reference, computed in one shot.

    Follows include/sparseattn_asyncgatherload_padded.cuh:211-249: the row max is
    taken on raw scores, p = exp2((s - m) * log2e * scale), the denominator sums
    fp32 p, and P is rounded to bf16 before the PV product.
    Returns (P_for_pv, denom, rowmax_raw).
    """
    m = scores.max(axis=-1, keepdims=True)
    m_safe = np.where(np.isfinite(m), m, 0.0)
    p = np.exp2((scores - m_safe) * np.float32(LOG2E * scale)).astype(np.float32)
    denom = p.sum(axis=-1, dtype=np.float32)
    if round_p:
        p = bf16_round(p)
    return p, denom, m[..., 0]


def sp_attn(q, k, v, kv_indices, kv_num_indices, *, qblk: int = QBLK_REF,
            scale: float | None = None, round_p: bool = True):
    """Gathered sparse attention (reference op ``sp_attn``).

    q, k, v: [B,H,S,D] float arrays holding bf16-representable values.
    kv_indices: int [B,H,SB,mask_stride] key-token ids; kv_num_indices: int with
    B*H*SB entries (python/extension.cpp:125-154).  For q-block I the key
    multiset is L = {idx[j] : j < n, idx[j] < S}
    (include/pad_utils.cuh:54-75, include/asyncloadutils.cuh:124-142) and
    O[r] = sum_{c in L} softmax_{c in L}(q_r.k_c * scale) v_c
    (include/sparseattn_asyncgatherload_padded.cuh:204-255).
    An empty L gives O = 0 and lse = -inf (the reference stores 0/0 there).
    Returns (O fp32 [B,H,S,D], lse fp32 [B,H,S]) with lse the natural-log
    log-sum-exp of the scaled scores over L.
    """
    q = np.asarray(q, np.float32)
    k = np.asarray(k, np.float32)
    v = np.asarray(v, np.float32)
    B, H, S, D = q.shape
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    SB = ceil_div(S, qblk)
    idx = np.asarray(kv_indices).reshape(B, H, SB, -1)
    num = np.asarray(kv_num_indices).reshape(B, H, SB)
    out = np.zeros((B, H, S, D), np.float32)
    lse = np.full((B, H, S), -np.inf, np.float32)
    for b in range(B):
        for h in range(H):
            for i in range(SB):
                r0, r1 = i * qblk, min(S, (i + 1) * qblk)
                lst = idx[b, h, i, : int(num[b, h, i])]
                lst = lst[(lst >= 0) & (lst < S)]
                if lst.size == 0:
                    continue
                s = q[b, h, r0:r1] @ k[b, h, lst].T
                p, denom, m = _softmax_rows(s, scale, round_p)
                out[b, h, r0:r1] = (p @ v[b, h, lst]) / denom[:, None]
                lse[b, h, r0:r1] = m * np.float32(scale) + np.log(denom)
    return out, lse


def block_list_to_token_list(blk_idx, blk_cnt, seq: int, kvblk: int = 64, mask_stride: int | None = None):
    """Expand KV-block lists into the reference's key-token lists.

    A kept block j of width kvblk is the token run kvblk*j .. kvblk*j+kvblk-1
    clipped to seq; the tail keeps the fill value mask_stride
    (python/spattn/mask_utils.py:329).
    """
    blk_idx = np.asarray(blk_idx)
    blk_cnt = np.asarray(blk_cnt)
    B, H, SB, _ = blk_idx.shape
    if mask_stride is None:
        mask_stride = padded_len(seq)
    tok = np.full((B, H, SB, mask_stride), mask_stride, np.int32)
    num = np.zeros((B, H, SB), np.int32)
    ar = np.arange(kvblk, dtype=np.int64)
    for b in range(B):
        for h in range(H):
            for i in range(SB):
                c = int(blk_cnt[b, h, i])
                t = (blk_idx[b, h, i, :c].astype(np.int64)[:, None] * kvblk + ar[None, :]).reshape(-1)
                t = t[t < seq]
                tok[b, h, i, : t.size] = t
                num[b, h, i] = t.size
    return tok, num


def full_attn(q, k, v, *, kv_len: int | None = None, scale: float | None = None, round_p: bool = True):
    """Dense attention (reference op ``full_attn``), keys limited to kv_len.

    include/fullattn_wgload_padded.cuh:190-232,244-265: softmax(QK^T*scale)V with
    keys >= kv_len masked to -inf and their V rows zero.
    Returns (O fp32, max_q raw [B,H,S], denom [B,H,S]).
    """
    q = np.asarray(q, np.float32)
    k = np.asarray(k, np.float32)
    v = np.asarray(v, np.float32)
    B, H, S, D = q.shape
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    kv = S if kv_len is None else kv_len
    out = np.zeros((B, H, S, D), np.float32)
    mx = np.zeros((B, H, S), np.float32)
    dn = np.zeros((B, H, S), np.float32)
    for b in range(B):
        for h in range(H):
            for r0 in range(0, S, 1024):
                r1 = min(S, r0 + 1024)
                s = q[b, h, r0:r1] @ k[b, h, :kv].T
                p, denom, m = _softmax_rows(s, scale, round_p)
                out[b, h, r0:r1] = (p @ v[b, h, :kv]) / denom[:, None]
                mx[b, h, r0:r1] = m
                dn[b, h, r0:r1] = denom
    return out, mx, dn


def maxq_denom(q, k, *, kv_len: int | None = None, scale: float | None = None):
    """Row statistics pre-pass (reference op ``maxq_denom``).

    include/maxq_denom.cuh:169-206: max_q[r] = max_c q_r.k_c on RAW scores,
    denom[r] = sum_c exp2((s - max_q) * log2e * scale); outputs are
    [B,H,1,Sp] fp32 with pad rows r in [S,Sp) holding max_q = 0, denom = -inf
    (include/maxq_denom.cuh:202-205).
    """
    q = np.asarray(q, np.float32)
    k = np.asarray(k, np.float32)
    B, H, S, D = q.shape
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    kv = S if kv_len is None else kv_len
    Sp = padded_len(S)
    mx = np.zeros((B, H, 1, Sp), np.float32)
    dn = np.full((B, H, 1, Sp), -np.inf, np.float32)
    for b in range(B):
        for h in range(H):
            for r0 in range(0, S, 1024):
                r1 = min(S, r0 + 1024)
                s = q[b, h, r0:r1] @ k[b, h, :kv].T
                _, denom, m = _softmax_rows(s, scale, False)
                mx[b, h, 0, r0:r1] = m
                dn[b, h, 0, r0:r1] = denom
    return mx, dn


def booleanmask_128(max_q, denom, q, k, thresh: float, *, kv_len: int | None = None,
                    scale: float | None = None, mask_stride: int | None = None):
    """Threshold vote mask (reference op ``booleanmask_128``).

    include/mask_utils.cuh:222-241: for q-block I of 128 rows and each of its
    eight 16-row groups W, p[r,c] = exp2((s - max_q[r]) * log2e*scale)/denom[r],
    cm_W[c] = max_{r in W} p[r,c]; mask[I,c] counts the groups with cm_W[c] > thresh
    (include/mask_utils.cuh:97-98,236-238).  Only columns c < kv_len are defined
    (python/spattn/mask_utils.py:269, include/mask_utils.cuh:297); others are 0 here.
    Returns (votes int32 [B,H,SB,mask_stride], pmax fp32 [B,H,SB,kv_len]) where pmax is
    max_{r in I} p[r,c], used by tests to leave out ties with the threshold.
    """
    q = np.asarray(q, np.float32)
    k = np.asarray(k, np.float32)
    B, H, S, D = q.shape
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    kv = S if kv_len is None else kv_len
    Sp = padded_len(S)
    SB = ceil_div(S, QBLK_REF)
    if mask_stride is None:
        mask_stride = Sp
    mx = np.asarray(max_q, np.float32).reshape(B, H, -1)
    dn = np.asarray(denom, np.float32).reshape(B, H, -1)
    votes = np.zeros((B, H, SB, mask_stride), np.int32)
    pmax = np.zeros((B, H, SB, kv), np.float32)
    for b in range(B):
        for h in range(H):
            for i in range(SB):
                r0, r1 = i * QBLK_REF, min(S, (i + 1) * QBLK_REF)
                s = q[b, h, r0:r1] @ k[b, h, :kv].T
                p = np.exp2((s - mx[b, h, r0:r1, None]) * np.float32(LOG2E * scale)) / dn[b, h, r0:r1, None]
                p = p.astype(np.float32)
                pmax[b, h, i] = p.max(axis=0)
                for w0 in range(0, r1 - r0, 16):
                    cm = p[w0:w0 + 16].max(axis=0)
                    votes[b, h, i, :kv] += (cm > np.float32(thresh)).astype(np.int32)
    return votes, pmax


def booleanmask_to_indexmask(booleanmask, seq: int, *, fill: int | None = None):
    """Mask -> index lists (reference op ``booleanmask_to_indexmask``), canonical order.

    include/mask_utils.cuh:292-300: count[I] = #{c < seq : mask[I,c] > 0}, the list
    holds exactly those c.  The reference order is whatever its atomics produce;
    the canonical form is ascending c followed by the caller's fill value
    (mask_stride, python/spattn/mask_utils.py:298), which is also what the
    reference's torch helper yields (python/spattn/mask_utils.py:152-167).
    """
    m = np.asarray(booleanmask)
    B, H, SB, MS = m.shape
    if fill is None:
        fill = MS
    idx = np.full((B, H, SB, MS), fill, np.int32)
    num = np.zeros((B, H, SB), np.int32)
    lim = min(seq, MS)
    for b in range(B):
        for h in range(H):
            for i in range(SB):
                nz = np.flatnonzero(m[b, h, i, :lim] > 0)
                idx[b, h, i, : nz.size] = nz
                num[b, h, i] = nz.size
    return idx, num


def all_index_mask(batch: int, heads: int, seqblocks: int, seq: int, mask_stride: int):
    """Identity lists (reference op ``all_index_mask``).

    include/utils.cuh:73-93: kv_indices[b,h,I,s] = s for every s < mask_stride and
    num = seq.
    """
    idx = np.broadcast_to(np.arange(mask_stride, dtype=np.int32), (batch, heads, seqblocks, mask_stride)).copy()
    num = np.full((batch, heads, seqblocks), seq, np.int32)
    return idx, num


def block_mask_from_votes(votes, seq: int, kvblk: int = 64):
    """MB[I,J] = OR_{c in J, c < seq} votes[I,c] > 0 - the block-level density measure."""
    m = np.asarray(votes)[..., :seq] > 0
    B, H, SB, _ = m.shape
    nb = ceil_div(seq, kvblk)
    pad = nb * kvblk - seq
    if pad:
        m = np.concatenate([m, np.zeros((B, H, SB, pad), bool)], axis=-1)
    return m.reshape(B, H, SB, nb, kvblk).any(axis=-1)


def booleanmask_rows(max_q, denom, q, k, thresh: float, *, qblk: int = 128, kv_len: int | None = None,
                     scale: float | None = None):
    """The `> 0` view of the threshold mask for q-blocks of qblk rows (64 or 128):
    M[I,c] = max_{r in I} p[r,c] > thresh with p as in ``booleanmask_128``
    (include/mask_utils.cuh:231-238; a q-block votes if one of its 16-row groups does, and the
    groups of a 64-row q-block are four of the eight of its 128-row block).
    Returns (mask bool [B,H,ceil(S/qblk),kv_len], pmax fp32 of the same shape)."""
    q = np.asarray(q, np.float32)
    k = np.asarray(k, np.float32)
    B, H, S, D = q.shape
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    kv = S if kv_len is None else kv_len
    nq = ceil_div(S, qblk)
    mx = np.asarray(max_q, np.float32).reshape(B, H, -1)
    dn = np.asarray(denom, np.float32).reshape(B, H, -1)
    pmax = np.zeros((B, H, nq, kv), np.float32)
    for b in range(B):
        for h in range(H):
            for i in range(nq):
                r0, r1 = i * qblk, min(S, (i + 1) * qblk)
                s = q[b, h, r0:r1] @ k[b, h, :kv].T
                p = np.exp2((s - mx[b, h, r0:r1, None]) * np.float32(LOG2E * scale)) / dn[b, h, r0:r1, None]
                pmax[b, h, i] = p.astype(np.float32).max(axis=0)
    return pmax > np.float32(thresh), pmax


def block_lists_from_mask(mask, seq: int, *, kvblk: int = 64, max_blocks: int | None = None, fill: int = -1):
    """Key mask -> ascending lists of kept key blocks: block J is kept when a key c in
    [kvblk*J, kvblk*J + kvblk) with c < seq is set (mask > 0).  The block form of
    ``booleanmask_to_indexmask`` (include/mask_utils.cuh:292-300 per key).
    Returns (blk_idx int32 [B,H,SB,max_blocks] with `fill` behind the kept ids,
    blk_cnt int32 [B,H,SB], blockmask bool [B,H,SB,ceil(mask_stride/kvblk)])."""
    m = np.asarray(mask)
    B, H, SB, MS = m.shape
    nb = ceil_div(MS, kvblk)
    bm = np.zeros((B, H, SB, nb), bool)
    lim = min(seq, MS)
    live = block_mask_from_votes(m, lim, kvblk) if lim > 0 else np.zeros((B, H, SB, 0), bool)
    bm[..., : live.shape[-1]] = live
    if max_blocks is None:
        max_blocks = nb
    idx = np.full((B, H, SB, max_blocks), fill, np.int32)
    cnt = np.zeros((B, H, SB), np.int32)
    for b in range(B):
        for h in range(H):
            for i in range(SB):
                nz = np.flatnonzero(bm[b, h, i])
                cnt[b, h, i] = nz.size
                w = min(nz.size, max_blocks)
                idx[b, h, i, :w] = nz[:w]
    return idx, cnt, bm


def block_row_max(q, k, *, kv_len: int | None = None, kvblk: int = 64):
    """Raw score maximum of every query row over every key block: out[b,h,J,r] = max over the
    keys c of block J with c < kv_len of q[r].k[c] (fp32), -inf for a block without such a key,
    laid out [B,H,Sp/kvblk,Sp] with Sp = 128*ceil(S/128); rows r >= S are left at 0.
    The per-block form of the row maximum of include/maxq_denom.cuh:182,203."""
    q = np.asarray(q, np.float32)
    k = np.asarray(k, np.float32)
    B, H, S, D = q.shape
    kv = S if kv_len is None else kv_len
    sp = padded_len(S)
    nb = sp // kvblk
    out = np.zeros((B, H, nb, sp), np.float32)
    for b in range(B):
        for h in range(H):
            s = q[b, h] @ k[b, h, :kv].T
            for j in range(nb):
                c0, c1 = j * kvblk, min(kv, (j + 1) * kvblk)
                out[b, h, j, :S] = s[:, c0:c1].max(axis=1) if c1 > c0 else -np.inf
    return out


def block_mask_from_blockmax(blockmax, max_q, denom, thresh: float, seq: int, D: int, *, qblk: int = 128,
                             kv_len: int | None = None, scale: float | None = None, kvblk: int = 64):
    """Block mask of the threshold test from per-(row, key block) score maxima:
    MB[I,J] = OR_{r in q-block I, r < seq} blockmax[J][r] > t[r] with
    t[r] = (log2 thresh + max_q[r] sf + log2 denom[r]) / sf - the test
    exp2((s - max_q) sf) / denom > thresh of include/mask_utils.cuh:231-238 solved for s; some key
    of a block passes it exactly when the block's maximum does.  Rows without a key (denom <= 0)
    do not vote.  Returns (MB bool [B,H,ceil(S/qblk),Sp/kvblk], margin fp32 of the same shape:
    max over the rows of (blockmax - t) sf, the log2 distance from the threshold)."""
    bm = np.asarray(blockmax, np.float32)
    B, H, nb, sp = bm.shape
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    sf = np.float32(LOG2E * scale)
    kv = seq if kv_len is None else kv_len
    nkb = ceil_div(kv, kvblk)
    mx = np.asarray(max_q, np.float32).reshape(B, H, -1)[..., :seq]
    dn = np.asarray(denom, np.float32).reshape(B, H, -1)[..., :seq]
    with np.errstate(divide="ignore", invalid="ignore"):
        t = np.where(dn > 0, (np.float32(np.log2(thresh)) + (mx * sf + np.log2(dn))) / sf, np.inf).astype(np.float32)
    nq = ceil_div(seq, qblk)
    mb = np.zeros((B, H, nq, nb), bool)
    margin = np.full((B, H, nq, nb), -np.inf, np.float32)
    for i in range(nq):
        r0, r1 = i * qblk, min(seq, (i + 1) * qblk)
        with np.errstate(invalid="ignore"):
            d = (bm[:, :, :nkb, r0:r1] - t[:, :, None, r0:r1]) * sf      # [B,H,nkb,rows]
        d = np.where(np.isnan(d), -np.inf, d)
        margin[:, :, i, :nkb] = d.max(axis=-1)
        mb[:, :, i, :nkb] = (bm[:, :, :nkb, r0:r1] > t[:, :, None, r0:r1]).any(axis=-1)
    return mb, margin


def block_lists_from_blockmask(bm, *, max_blocks: int | None = None, fill: int = -1):
    """Ascending kept-block ids per row of a block mask [B,H,SB,NB], then `fill`; counts."""
    bm = np.asarray(bm, bool)
    B, H, SB, nb = bm.shape
    if max_blocks is None:
        max_blocks = nb
    idx = np.full((B, H, SB, max_blocks), fill, np.int32)
    cnt = np.zeros((B, H, SB), np.int32)
    for b in range(B):
        for h in range(H):
            for i in range(SB):
                nz = np.flatnonzero(bm[b, h, i])
                cnt[b, h, i] = nz.size
                w = min(nz.size, max_blocks)
                idx[b, h, i, :w] = nz[:w]
    return idx, cnt


def pack_mask(mask):
    """Bit-packed form of a vote mask: bit (c & 7) of byte c >> 3 is set where mask[..., c] > 0
    (python/spattn/mask_utils.py:421-430, `pack`: 8 booleans per byte, least significant bit first).
    Pinned by numpy.packbits(bitorder='little'), a library routine, and by the round trip below."""
    mask = np.asarray(mask)
    assert mask.shape[-1] % 8 == 0
    return np.packbits(mask > 0, axis=-1, bitorder="little")


def unpack_mask(packed):
    """Inverse of pack_mask as booleans (python/spattn/mask_utils.py:432-439, `unpack`)."""
    return np.unpackbits(np.asarray(packed, np.uint8), axis=-1, bitorder="little").astype(bool)


def packedmask_to_indexmask(packed, seq, fill=None):
    """unpack followed by booleanmask_to_indexmask: what CompressedBitMaskCache.get_mask_from_cache
    computes (python/spattn/mask_utils.py:86-90)."""
    return booleanmask_to_indexmask(unpack_mask(packed).astype(np.int32), seq, fill=fill)


def qblock_mean_scores(q, k, blocksz: int = 128):
    """qmean and score of the top-k mask generator, with the roundings of the reference's bf16
    torch ops (python/spattn/mask_utils.py:390-410): block mean (fp32 sum * 1/rows -> bf16),
    divided by sqrt(D) (-> bf16), fp32 dot with every key (-> bf16).
    q, k: [B,H,S,D] holding bf16-representable values.  Returns (qmean [B,H,SB,D], score [B,H,SB,S])."""
    q = np.asarray(q, np.float32)
    k = np.asarray(k, np.float32)
    B, H, S, D = q.shape
    SB = ceil_div(S, blocksz)
    qmean = np.zeros((B, H, SB, D), np.float32)
    for m in range(SB):
        blk = q[:, :, m * blocksz:(m + 1) * blocksz]
        rows = blk.shape[2]
        # fp32 order of the device kernel: 512 / D interleaved row phases, each summed row
        # after row, then the phases added in order
        phases = 512 // D
        acc = None
        for j in range(phases):
            part = np.zeros((B, H, D), np.float32)
            for r in range(j, rows, phases):
                part = part + blk[:, :, r]
            acc = part if acc is None else acc + part
        qmean[:, :, m] = bf16_round(acc * (np.float32(1.0) / np.float32(rows)))
    qmean = bf16_round(qmean / np.float32(math.sqrt(D)))
    score = bf16_round(np.einsum("bhmd,bhnd->bhmn", qmean, k).astype(np.float32))
    return qmean, score


def topk_select(score, select_k: int, kv_len: int | None = None):
    """The select_k keys c < kv_len with the largest score per row, larger score first and the
    lower key first among equal scores (torch.topk, python/spattn/mask_utils.py:412, leaves
    the order among equal scores open), returned as ASCENDING key lists.
    score: [..., S].  Returns int32 [..., min(select_k, kv_len)]."""
    score = np.asarray(score, np.float32)
    S = score.shape[-1]
    kv_len = S if kv_len is None else kv_len
    kk = min(select_k, kv_len)
    flat = score.reshape(-1, S)[:, :kv_len]
    out = np.zeros((flat.shape[0], kk), np.int32)
    for i, row in enumerate(flat):
        order = np.lexsort((np.arange(kv_len), -row))   # by score descending, then key ascending
        out[i] = np.sort(order[:kk])
    return out.reshape(*score.shape[:-1], kk)


def _xcd_remap(i, n, xcds=8):
    per = n // xcds
    lim = per * xcds
    return np.where(i >= lim, i, (i % xcds) * per + i // xcds)


def qblock_order(counts, sub_bits: int = 2, octaves: int = 22):
    """Work order of the list-driven attention kernels (no counterpart in the reference, whose
    grid is fixed, include/sparseattn_asyncgatherload_padded.cuh:273): q-blocks by list length,
    longest first, in quarter-octave classes of the count (the leading one and the two bits
    below it), stable inside a class; if the longest list is less than twice the shortest the default order is kept
    (neighbouring q-blocks together on one XCD).
    Integer work; pinned by its defining properties (a permutation, class-monotone, stable) and
    by a brute-force sort in the tests."""
    c = np.asarray(counts).reshape(-1).astype(np.int64)
    n = c.size
    lo, hi = int(c.min()), int(c.max())
    if hi <= 0 or hi < 2 * lo:
        return _xcd_remap(np.arange(n), n).astype(np.int32)
    classes = (octaves << sub_bits) + 2
    lg = np.zeros(n, np.int64)
    pos = c > 0
    lg[pos] = np.frexp(c[pos].astype(np.float64))[1] - 1      # floor(log2 c), exact below 2^53
    m = (1 << sub_bits) - 1
    below = np.where(lg >= sub_bits, (c >> np.maximum(lg - sub_bits, 0)) & m, (c << np.maximum(sub_bits - lg, 0)) & m)
    fine = np.minimum((lg << sub_bits) + below, classes - 2)
    cls = np.where(pos, classes - 2 - fine, classes - 1)
    return np.argsort(cls, kind="stable").astype(np.int32)
