"""Mask helpers of the reference's ``spattn/mask_utils.py`` over the gfx950 operators.

Same names, argument meaning and tensor conventions as the reference
(python/spattn/mask_utils.py); the pure-torch functions are the semantic definition of
the masks, the ``*_cuda`` functions run the device operators.  Differences kept on
purpose: tensors are created on the device of their inputs instead of a hard-coded
'cuda', and ``seq`` of ``bitmask_to_indexmask_cuda`` defaults to the mask width instead
of a stale constant.
"""
from __future__ import annotations

import torch

from . import cuda_attn  # noqa: F401  (loading it registers torch.ops.cuda_attn)

spattn_interface = torch.ops.cuda_attn

BLOCKSZ = 128   # q-block of the threshold pre-pass (python/spattn/mask_utils.py:249,312)
BLOCKSZ_DEFAULT = BLOCKSZ


def _padded(seq: int, blk: int = BLOCKSZ) -> int:
    return blk * ((seq + blk - 1) // blk)


def _is_dev(t) -> bool:
    return isinstance(t, torch.Tensor) and t.is_cuda


# ----------------------------------------------------------------------------------
# mask caches (python/spattn/mask_utils.py:17-98)
# ----------------------------------------------------------------------------------
class NaiveMaskCache:
    """Index lists per layer, recomputed on the diffusion steps in ``compute_cache_at``.

    Next to the lists the cache keeps their work order (a function of the counts alone, see
    ``qblock_order_cuda``): it is computed when the lists are stored, so a step that reuses
    them is a single kernel launch.  ``get_order`` returns it (None for host tensors)."""

    def __init__(self, compute_cache_at):
        self.cache = {}
        self.order = {}
        self.compute_cache_at = compute_cache_at

    def run_fullattn(self, ditrun):
        return ditrun in self.compute_cache_at

    def get_mask_from_cache(self, layer):
        return self.cache[layer]

    def get_order(self, layer):
        return self.order.get(layer)

    def update_cache(self, layer, kv_indices, kv_num_indices):
        self.cache[layer] = (kv_indices, kv_num_indices)
        self.order[layer] = qblock_order_cuda(kv_num_indices) if _is_dev(kv_num_indices) else None


class BlockListCache(NaiveMaskCache):
    """KV-block lists ([B,H,ceil(S/qblk),max_blocks] ids of 64-key blocks, counts) per layer, for
    ``sp_attn_block``; same protocol as NaiveMaskCache.  No counterpart in the reference, whose
    lists are per key."""


class OffloadMaskCache(NaiveMaskCache):
    """Keeps the index lists in host memory between uses."""

    def get_mask_from_cache(self, layer, ditrun=0):
        kv_indices, kv_num_indices = self.cache[layer]
        return kv_indices.to(kv_num_indices.device), kv_num_indices

    def update_cache(self, layer, kv_indices, kv_num_indices):
        self.cache[layer] = (kv_indices.cpu(), kv_num_indices)
        self.order[layer] = qblock_order_cuda(kv_num_indices) if _is_dev(kv_num_indices) else None


class CompressMaskCache(NaiveMaskCache):
    """The reference's compressed list cache (python/spattn/mask_utils.py:46-67) keeps the index
    lists through nvcomp's BitComp codec.  Here the lists are kept as what they encode - one bit
    per (q-block, key), 1/32 of the int32 lists - and come back through the fused
    bits -> lists kernel: the same keys per q-block, in ascending order (the attention operators do
    not depend on the order), with the fill value the reference uses (the row length)."""

    def get_mask_from_cache(self, layer):
        packed, seq_len, kv_num_indices = self.cache[layer]
        kv_indices, counts = packedmask_to_indexmask_cuda(packed, seq_len)
        return kv_indices, counts.view_as(kv_num_indices)

    def update_cache(self, layer, kv_indices, kv_num_indices, seq_len=None):
        """seq_len: the number of keys the ids range over, rounded up to a multiple of 128 for the bit
        rows; default: the width of the lists, which is right for lists as wide as the sequence (what
        the threshold pre-pass returns).  Narrower lists (top-k) need it; an id that does not fit is an
        error, not a dropped key."""
        B, H, SB, stride = kv_indices.shape
        width = _padded(int(seq_len)) if seq_len is not None else int(stride)
        pos = torch.arange(stride, device=kv_indices.device).view(1, 1, 1, stride)
        live = (pos < kv_num_indices.reshape(B, H, SB, 1)) & (kv_indices >= 0)
        if bool((live & (kv_indices >= width)).any()):
            raise ValueError("CompressMaskCache: a listed key id does not fit %d keys; pass seq_len" % width)
        votes = torch.zeros((B, H, SB, width + 1), dtype=torch.int32, device=kv_indices.device)
        # entries behind the count are sent to a spare column
        votes.scatter_(3, torch.where(live, kv_indices, torch.full_like(kv_indices, width)).long(), 1)
        votes = votes[..., :width].contiguous()
        packed = pack_votes_cuda(votes) if votes.is_cuda and width % 128 == 0 else pack(votes > 0)
        self.cache[layer] = (packed, width, kv_num_indices)
        self.order[layer] = qblock_order_cuda(kv_num_indices) if _is_dev(kv_num_indices) else None


class BitMaskCache:
    """Stores the vote mask and re-expands it to index lists on every use."""

    def __init__(self, compute_cache_at):
        self.cache = {}
        self.compute_cache_at = compute_cache_at

    def run_fullattn(self, ditrun):
        return ditrun in self.compute_cache_at

    def get_mask_from_cache(self, layer):
        mask, seq_len = self.cache[layer]
        return bitmask_to_indexmask_cuda(mask, seq_len)

    def update_cache(self, layer, bytemask, seq_len):
        self.cache[layer] = (bytemask, seq_len)


class CompressedBitMaskCache(BitMaskCache):
    """Stores the mask bit-packed (8 keys per byte, least significant bit first).  On the device
    both directions are single kernels: the vote mask is packed without a boolean copy, and a
    reuse goes from the bits to the index lists without materialising the unpacked mask."""

    def get_mask_from_cache(self, layer):
        packed, seq_len = self.cache[layer]
        if packed.is_cuda and packed.dim() == 4:
            return packedmask_to_indexmask_cuda(packed, seq_len)
        return bitmask_to_indexmask_cuda(unpack(packed).to(torch.int32), seq_len)

    def update_cache(self, layer, bitmask, seq_len):
        if bitmask.is_cuda and bitmask.dim() == 4 and bitmask.dtype == torch.int32 and bitmask.shape[-1] % 128 == 0:
            self.cache[layer] = (pack_votes_cuda(bitmask), seq_len)
        else:
            self.cache[layer] = (pack(bitmask > 0), seq_len)


# ----------------------------------------------------------------------------------
# 2-D attention-map helpers (python/spattn/mask_utils.py:107-167)
# ----------------------------------------------------------------------------------
def _pool_rows(attnmap, block, reduce):
    rows, cols = attnmap.shape
    pad = (-rows) % block
    if pad:
        # a ragged last block is reduced over the rows it has: pad with copies of the last row
        attnmap = torch.cat([attnmap, attnmap[-1:].expand(pad, cols)], dim=0)
    return reduce(attnmap.view(-1, block, cols), 1)


def attnmapand(attnmap, BLOCK_SZ=128):
    """min over each block of BLOCK_SZ rows (python/spattn/mask_utils.py:107-123)."""
    return _pool_rows(attnmap, BLOCK_SZ, lambda t, d: t.min(dim=d).values)


def attnmapor(attnmap, BLOCK_SZ=128):
    """max over each block of BLOCK_SZ rows (python/spattn/mask_utils.py:126-142)."""
    return _pool_rows(attnmap, BLOCK_SZ, lambda t, d: t.max(dim=d).values)


def attnmapbroadcast(attnmapand_, BLOCK_SZ=128):
    """Repeat every row BLOCK_SZ times (python/spattn/mask_utils.py:145-149)."""
    return attnmapand_.repeat_interleave(BLOCK_SZ, dim=0)


def boolean_to_index_mask_2d(boolean_mask):
    """Rows of a boolean [R,N] mask -> ascending column lists padded with N, and counts
    (python/spattn/mask_utils.py:152-167)."""
    rows, n = boolean_mask.shape
    keep = boolean_mask != 0
    # a stable sort moves the kept columns to the front in ascending order
    order = torch.sort((~keep).to(torch.uint8), dim=1, stable=True).indices
    counts = keep.sum(dim=1)
    col = torch.arange(n, device=boolean_mask.device).expand(rows, n)
    index_mask = torch.where(col < counts[:, None], order, torch.full_like(order, n))
    return index_mask.to(torch.int32), counts.to(torch.int32)


# ----------------------------------------------------------------------------------
# index lists (python/spattn/mask_utils.py:175-203)
# ----------------------------------------------------------------------------------
def allindex_mask(B, H, max_stride, S, BLOCKSZ, device="cuda"):
    nb = (S + BLOCKSZ - 1) // BLOCKSZ
    kv_indices = torch.arange(max_stride, device=device, dtype=torch.int32).expand(B, H, nb, max_stride).contiguous()
    return kv_indices, torch.full((B, H, nb), S, device=device, dtype=torch.int32)


def halfindex_mask(B, H, S, BLOCKSZ, device="cuda"):
    nb = (S + BLOCKSZ - 1) // BLOCKSZ
    kv_indices = (2 * torch.arange(S // 2, device=device, dtype=torch.int32)).expand(B, H, nb, S // 2).contiguous()
    return kv_indices, torch.full((B, H, nb), S // 2, device=device, dtype=torch.int32)


def allindex_randompermutation_mask(B, H, max_stride, S, BLOCKSZ, device="cuda"):
    nb = (S + BLOCKSZ - 1) // BLOCKSZ
    row = torch.full((max_stride,), max_stride, device=device, dtype=torch.int32)
    row[:S] = torch.randperm(S, device=device).to(torch.int32)
    return row.expand(B, H, nb, max_stride).contiguous(), torch.full((B, H, nb), S, device=device, dtype=torch.int32)


# ----------------------------------------------------------------------------------
# pure-torch definition of the threshold mask (python/spattn/mask_utils.py:206-245)
# ----------------------------------------------------------------------------------
def qk_bitmask(q, k, thresh=0.001, blocksz=128):
    """mask[b,h,I,c] = any row r of q-block I has softmax(q k^T / sqrt(D))[r,c] > thresh."""
    B, H, S, D = q.shape
    out = []
    for b in range(B):
        per_head = []
        for h in range(H):
            p = torch.softmax((q[b, h] @ k[b, h].T) * (D ** -0.5), dim=-1)
            per_head.append(attnmapor(p > thresh, blocksz))
        out.append(torch.stack(per_head))
    return torch.stack(out)


def bitmask_to_indexmask(booleanmask):
    B, H, SB, MS = booleanmask.shape
    idx, cnt = boolean_to_index_mask_2d(booleanmask.reshape(B * H * SB, MS))
    return idx.view(B, H, SB, MS), cnt.view(B, H, SB)


def qk_indexmask(q, k, thresh=0.001, blocksz=128):
    return bitmask_to_indexmask(qk_bitmask(q, k, thresh, blocksz))


# ----------------------------------------------------------------------------------
# device path (python/spattn/mask_utils.py:248-382)
# ----------------------------------------------------------------------------------
def _stats_buffers(q):
    B, H, S, _ = q.shape
    sp = _padded(S)
    max_q = torch.empty((B, H, 1, sp), dtype=torch.float32, device=q.device)
    denom = torch.empty((B, H, 1, sp), dtype=torch.float32, device=q.device)
    return max_q, denom


def qk_bitmask_from_maxq_denom_cuda(max_q, denom, q, k, thresh, blocksz=128):
    """Vote mask int32 [B,H,ceil(S/128),Sp] from row statistics (python/spattn/mask_utils.py:337-355)."""
    assert blocksz == BLOCKSZ
    B, H, S, _ = q.shape
    booleanmask = torch.zeros((B, H, (S + blocksz - 1) // blocksz, max_q.shape[3]), dtype=torch.int32, device=q.device)
    spattn_interface.booleanmask_128(booleanmask, max_q.contiguous(), denom.contiguous(), q.contiguous(), k.contiguous(), thresh)
    return booleanmask


def qk_bitmask_cuda(q, k, thresh, blocksz=128):
    """Boolean mask via maxq_denom + booleanmask_128 (python/spattn/mask_utils.py:248-269)."""
    assert blocksz == BLOCKSZ
    max_q, denom = _stats_buffers(q)
    spattn_interface.maxq_denom(max_q, denom, q.contiguous(), k.contiguous())
    return qk_bitmask_from_maxq_denom_cuda(max_q, denom, q, k, thresh, blocksz) > 0


def bitmask_to_indexmask_cuda(booleanmask, seq=None):
    """Index lists (ascending, padded with mask_stride) and counts from a vote mask
    (python/spattn/mask_utils.py:293-303); ``seq`` is the kv length."""
    B, H, SB, MS = booleanmask.shape
    if seq is None:
        seq = MS
    kv_indices = torch.full((B, H, SB, MS), MS, dtype=torch.int32, device=booleanmask.device)
    num_kv_indices = torch.zeros((B, H, SB), dtype=torch.int32, device=booleanmask.device)
    spattn_interface.booleanmask_to_indexmask(kv_indices, num_kv_indices, booleanmask.to(torch.int32).contiguous(), seq)
    return kv_indices, num_kv_indices


def pack_votes_cuda(booleanmask):
    """uint8 [B,H,SB,mask_stride/8]: bit (c & 7) of byte c >> 3 set where the int32 vote mask is > 0;
    equals ``pack(booleanmask > 0)``."""
    B, H, SB, MS = booleanmask.shape
    packed = torch.empty((B, H, SB, MS // 8), dtype=torch.uint8, device=booleanmask.device)
    spattn_interface.pack_mask(packed, booleanmask.contiguous())
    return packed


def packedmask_to_indexmask_cuda(packed, seq=None):
    """Index lists and counts straight from a bit-packed mask; equals
    ``bitmask_to_indexmask_cuda(unpack(packed), seq)``."""
    B, H, SB, MB = packed.shape
    MS = MB * 8
    if seq is None:
        seq = MS
    kv_indices = torch.full((B, H, SB, MS), MS, dtype=torch.int32, device=packed.device)
    num_kv_indices = torch.zeros((B, H, SB), dtype=torch.int32, device=packed.device)
    spattn_interface.packedmask_to_indexmask(kv_indices, num_kv_indices, packed.contiguous(), seq)
    return kv_indices, num_kv_indices


def qk_indexmask_from_maxq_denom_cuda(max_q, denom, q, k, thresh, blocksz=128):
    """python/spattn/mask_utils.py:358-382."""
    booleanmask = qk_bitmask_from_maxq_denom_cuda(max_q, denom, q, k, thresh, blocksz)
    return bitmask_to_indexmask_cuda(booleanmask, q.shape[2])


def qk_indexmask_cuda(q, k, thresh, blocksz=128):
    """Statistics -> vote mask -> index lists (python/spattn/mask_utils.py:306-334)."""
    assert blocksz == BLOCKSZ
    max_q, denom = _stats_buffers(q)
    spattn_interface.maxq_denom(max_q, denom, q.contiguous(), k.contiguous())
    return qk_indexmask_from_maxq_denom_cuda(max_q, denom, q, k, thresh, blocksz)


def qblock_order_cuda(counts):
    """int32 [counts.numel()]: the q-blocks longest list first (the schedule of the list-driven
    attention operators); lists within a factor of two of each other keep the default order."""
    order = torch.empty((counts.numel(),), dtype=torch.int32, device=counts.device)
    spattn_interface.qblock_order(order, counts.contiguous())
    return order


# ----------------------------------------------------------------------------------
# KV-block lists: the threshold mask at the granularity of 64-key blocks.  The sweep writes
# one bit per (q-block, key) instead of an int32 vote count, and the lists hold block ids.
# ----------------------------------------------------------------------------------
KVBLK = 64


def qk_packedmask_from_maxq_denom_cuda(max_q, denom, q, k, thresh, qblk=128, kv_len=0):
    """uint8 [B,H,ceil(S/qblk),Sp/8], bit (c & 7) of byte c >> 3: some row of the q-block has
    softmax(row, c) > thresh.  For qblk = 128 equal to ``pack(qk_bitmask_from_maxq_denom_cuda(...) > 0)``."""
    B, H, S, _ = q.shape
    packed = torch.empty((B, H, (S + qblk - 1) // qblk, max_q.shape[3] // 8), dtype=torch.uint8, device=q.device)
    spattn_interface.booleanmask_packed(packed, max_q.contiguous(), denom.contiguous(), q.contiguous(), k.contiguous(),
                                        thresh, qblk, 0.0, kv_len)
    return packed


def packedmask_to_blocklists_cuda(packed, seq=None, max_blocks=None, with_blockmask=False):
    """Ascending lists of the 64-key blocks with a set key c < seq, padded with -1, and counts;
    optionally the block mask uint8 [B,H,SB,mask_stride/64] as a third result."""
    B, H, SB, MB = packed.shape
    nb = MB * 8 // KVBLK
    if seq is None:
        seq = MB * 8
    if max_blocks is None:
        max_blocks = nb
    blk_idx = torch.full((B, H, SB, max_blocks), -1, dtype=torch.int32, device=packed.device)
    blk_cnt = torch.zeros((B, H, SB), dtype=torch.int32, device=packed.device)
    blockmask = torch.empty((B, H, SB, nb), dtype=torch.uint8, device=packed.device) if with_blockmask else None
    spattn_interface.packedmask_to_blocklists(blk_idx, blk_cnt, blockmask, packed.contiguous(), seq)
    return (blk_idx, blk_cnt, blockmask) if with_blockmask else (blk_idx, blk_cnt)


def bitmask_to_blocklists_cuda(booleanmask, seq=None, max_blocks=None, with_blockmask=False):
    """The same from the int32 vote mask [B,H,SB,mask_stride]."""
    B, H, SB, MS = booleanmask.shape
    nb = MS // KVBLK
    if seq is None:
        seq = MS
    if max_blocks is None:
        max_blocks = nb
    blk_idx = torch.full((B, H, SB, max_blocks), -1, dtype=torch.int32, device=booleanmask.device)
    blk_cnt = torch.zeros((B, H, SB), dtype=torch.int32, device=booleanmask.device)
    blockmask = torch.empty((B, H, SB, nb), dtype=torch.uint8, device=booleanmask.device) if with_blockmask else None
    spattn_interface.booleanmask_to_blocklists(blk_idx, blk_cnt, blockmask, booleanmask.to(torch.int32).contiguous(), seq)
    return (blk_idx, blk_cnt, blockmask) if with_blockmask else (blk_idx, blk_cnt)


def qk_blocklists_from_maxq_denom_cuda(max_q, denom, q, k, thresh, qblk=128, kv_len=0):
    """Row statistics -> bit-packed threshold mask -> KV-block lists for q-blocks of qblk rows."""
    packed = qk_packedmask_from_maxq_denom_cuda(max_q, denom, q, k, thresh, qblk, kv_len)
    return packedmask_to_blocklists_cuda(packed, kv_len or q.shape[2])


def qk_blocklists_cuda(q, k, thresh, qblk=128, kv_len=0):
    """Statistics sweep -> threshold sweep -> KV-block lists (the block form of qk_indexmask_cuda)."""
    max_q, denom = _stats_buffers(q)
    spattn_interface.maxq_denom_ex(max_q, denom, q.contiguous(), k.contiguous(), 0.0, kv_len)
    return qk_blocklists_from_maxq_denom_cuda(max_q, denom, q, k, thresh, qblk, kv_len)


# Largest block-maxima buffer the one-sweep routes allocate without being told to (bytes).  The
# buffer takes 2 * Sp * Sp / 64 bytes per head: 0.81 GB at (1,24,32768), 1.5 GB at (1,12,75648),
# 4.3 GB at (1,24,75904), 7.2 GB at (1,40,75648).  Above the budget the callers fall back to the
# reference's two full sweeps, which need no such buffer.
BLOCKMAX_BUDGET_BYTES = 2 << 30


def blockmax_bytes(q):
    """Bytes of the block-maxima buffer for a statistics sweep over q [B,H,S,D]."""
    B, H, S, _ = q.shape
    sp = _padded(S)
    return 2 * B * H * (sp // KVBLK) * sp


def use_onepass(q, onepass=None, budget_bytes=None):
    """Whether a refresh step takes the one-sweep route (statistics sweep with block maxima, then the
    threshold on those) or the reference's two full sweeps.  onepass True / False decides outright;
    None decides by the size of the block-maxima buffer against budget_bytes (default
    BLOCKMAX_BUDGET_BYTES)."""
    if onepass is not None:
        return bool(onepass)
    budget = BLOCKMAX_BUDGET_BYTES if budget_bytes is None else int(budget_bytes)
    return blockmax_bytes(q) <= budget


def blockmax_buffer(q):
    """bf16 [B,H,Sp/64,Sp] for the per-(row, key block) score maxima of a statistics sweep (the
    sweep rounds them toward +inf)."""
    B, H, S, _ = q.shape
    sp = _padded(S)
    return torch.empty((B, H, sp // KVBLK, sp), dtype=torch.bfloat16, device=q.device)


def blockmax_to_blocklists_cuda(blockmax, max_q, denom, thresh, seq, head_dim, qblk=128, kv_len=0, max_blocks=None,
                                with_blockmask=False):
    """Threshold test on the block maxima -> KV-block lists (padded with -1), counts and, optionally,
    the block mask uint8 [B,H,ceil(S/qblk),Sp/64].  A new threshold needs no new sweep."""
    B, H, nb, _ = blockmax.shape
    nq = (seq + qblk - 1) // qblk
    if max_blocks is None:
        max_blocks = nb
    blk_idx = torch.full((B, H, nq, max_blocks), -1, dtype=torch.int32, device=blockmax.device)
    blk_cnt = torch.zeros((B, H, nq), dtype=torch.int32, device=blockmax.device)
    blockmask = torch.empty((B, H, nq, nb), dtype=torch.uint8, device=blockmax.device) if with_blockmask else None
    spattn_interface.blockmax_to_blocklists(blk_idx, blk_cnt, blockmask, blockmax, max_q.contiguous(), denom.contiguous(),
                                            thresh, seq, head_dim, qblk, 0.0, kv_len)
    return (blk_idx, blk_cnt, blockmask) if with_blockmask else (blk_idx, blk_cnt)


def qk_blocklists_onepass_cuda(q, k, thresh, qblk=128, kv_len=0):
    """KV-block lists from ONE sweep over Q K^T: the statistics sweep also writes the maximum of
    every row over every 64-key block (as bf16, rounded up), and the threshold test runs on those
    maxima.  The lists hold every block of qk_blocklists_cuda's and possibly a block whose best key
    misses the threshold by less than one bf16 step (2^-8) of its raw score."""
    max_q, denom = _stats_buffers(q)
    blockmax = blockmax_buffer(q)
    spattn_interface.maxq_denom_blockmax(max_q, denom, blockmax, q.contiguous(), k.contiguous(), 0.0, kv_len)
    return blockmax_to_blocklists_cuda(blockmax, max_q, denom, thresh, q.shape[2], q.shape[3], qblk, kv_len)


# The key-list route thresholds the block maxima a little below the vote threshold: the statistics
# sweep and the vote sweep round a score differently in fp32 (one rounds s and compares, the other
# accumulates s - t in the matrix unit), so a key whose margin is within that rounding could otherwise
# sit in a block the maxima leave out.  Two margins cover it: the stored maxima are rounded UP to bf16
# (up to 2^-8 of the score's own magnitude, so the margin grows with the scores), and tau (1 - 1e-3)
# moves the block test by about 0.01 raw score units whatever the magnitude.  The blocks either adds
# contribute zero votes.
_BLOCK_THRESH_SLACK = 1.0 - 1e-3


def _blocks_that_can_hold_a_key(blockmax, max_q, denom, thresh, S, D, kv_len):
    return blockmax_to_blocklists_cuda(blockmax, max_q, denom, thresh * _BLOCK_THRESH_SLACK, S, D, 128, kv_len)


def qk_bitmask_from_blockmax_cuda(blockmax, max_q, denom, q, k, thresh, blocksz=128, kv_len=0):
    """The vote mask of qk_bitmask_from_maxq_denom_cuda from the block maxima of the statistics sweep:
    their threshold gives the key blocks in which a key can pass, and the sweep then multiplies those
    blocks only (the rest of the mask is zero) - the same votes for a fraction of the work."""
    B, H, S, D = q.shape
    blk_idx, blk_cnt = _blocks_that_can_hold_a_key(blockmax, max_q, denom, thresh, S, D, kv_len)
    mask = torch.empty((B, H, (S + blocksz - 1) // blocksz, max_q.shape[3]), dtype=torch.int32, device=q.device)
    spattn_interface.booleanmask_128_blocks(mask, max_q.contiguous(), denom.contiguous(), q.contiguous(), k.contiguous(),
                                            blk_idx, blk_cnt, thresh, 0.0, kv_len)
    return mask


def qk_packedmask_from_blockmax_cuda(blockmax, max_q, denom, q, k, thresh, qblk=128, kv_len=0):
    """The same votes as bits (qk_packedmask_from_maxq_denom_cuda over the blocks that can hold a key)."""
    B, H, S, D = q.shape
    blk_idx, blk_cnt = _blocks_that_can_hold_a_key(blockmax, max_q, denom, thresh, S, D, kv_len)
    packed = torch.empty((B, H, (S + qblk - 1) // qblk, max_q.shape[3] // 8), dtype=torch.uint8, device=q.device)
    spattn_interface.booleanmask_packed_blocks(packed, max_q.contiguous(), denom.contiguous(), q.contiguous(), k.contiguous(),
                                               blk_idx, blk_cnt, thresh, qblk, 0.0, kv_len)
    return packed


def qk_indexmask_from_blockmax_cuda(blockmax, max_q, denom, q, k, thresh, blocksz=128, kv_len=0):
    """Key lists (the reference's form) from the block maxima: blocks that can hold a key, the sweep over
    those blocks with its votes as bits, the key lists decoded from the bits."""
    packed = qk_packedmask_from_blockmax_cuda(blockmax, max_q, denom, q, k, thresh, blocksz, kv_len)
    return packedmask_to_indexmask_cuda(packed, kv_len or q.shape[2])


def qk_indexmask_onepass_cuda(q, k, thresh, blocksz=128, kv_len=0):
    """qk_indexmask_cuda with one full sweep over Q K^T instead of two (statistics with block maxima,
    then the threshold sweep over the blocks that can hold a key)."""
    max_q, denom = _stats_buffers(q)
    blockmax = blockmax_buffer(q)
    spattn_interface.maxq_denom_blockmax(max_q, denom, blockmax, q.contiguous(), k.contiguous(), 0.0, kv_len)
    return qk_indexmask_from_blockmax_cuda(blockmax, max_q, denom, q, k, thresh, blocksz, kv_len)


def qk_blocklists(q, k, thresh=0.001, qblk=128):
    """Pure-torch definition of the block lists: block J of q-block I is kept when some row of I
    and some key of J have softmax > thresh.  Returns (blk_idx padded with -1, blk_cnt, blockmask)."""
    B, H, S, _ = q.shape
    m = qk_bitmask(q, k, thresh, qblk)                                   # [B,H,nq,S]
    pad = (-S) % KVBLK
    if pad:
        m = torch.cat([m, torch.zeros((*m.shape[:3], pad), dtype=m.dtype, device=m.device)], dim=-1)
    bm = m.view(*m.shape[:3], -1, KVBLK).any(dim=-1)
    nq, nb = bm.shape[2], bm.shape[3]
    idx, cnt = boolean_to_index_mask_2d(bm.reshape(B * H * nq, nb))
    idx = torch.where(idx == nb, torch.full_like(idx, -1), idx)
    return idx.view(B, H, nq, nb), cnt.view(B, H, nq), bm


def qk_lshmask_indices(query, key, thresh, blocksz=128):
    raise NotImplementedError   # as in the reference (python/spattn/mask_utils.py:385-386)


def qk_topkmask_indices(q, k, select_k, B=None, H=None, S=None, D=None, BLOCKSZ=None, blocksz=None):
    """Top-k keys per q-block by (block-mean query / sqrt(D)) . key, in the dtype of q like the
    reference (python/spattn/mask_utils.py:389-417).  Takes the reference's positional form
    ``(q, k, select_k, B, H, S, D, BLOCKSZ)`` as well as ``blocksz=`` alone, which is how the
    reference's own caller passes it (python/spattn/sparseattn_functionals.py:46); sizes that
    are not given are read from q."""
    B, H, S, D = (int(x) if x is not None else int(d) for x, d in zip((B, H, S, D), q.shape))
    blk = int(BLOCKSZ if BLOCKSZ is not None else (blocksz if blocksz is not None else BLOCKSZ_DEFAULT))
    nfull = S // blk
    parts = []
    if nfull:
        parts.append(q[:, :, : nfull * blk].reshape(B, H, nfull, blk, D).mean(dim=3))
    if S % blk:
        parts.append(q[:, :, nfull * blk:].mean(dim=2, keepdim=True))
    qmean = torch.cat(parts, dim=2) * 1.0 / D ** 0.5
    score = torch.einsum("bhmd,bhnd->bhmn", qmean, k)
    kv_indices = torch.topk(score, select_k, dim=-1, sorted=True).indices.to(torch.int32)
    nb = (S + blk - 1) // blk
    return kv_indices, torch.full((B, H, nb), select_k, device=q.device, dtype=torch.int32)


def qk_topkmask_indices_cuda(q, k, select_k, blocksz=128):
    """The same selection on the device in three kernels (q-block means, one [SB x D].[D x S]
    product per head, a radix select per row): kv_indices [B,H,SB,stride] int32 with the
    select_k keys of each q-block in ascending order, stride = select_k rounded up to 128 and
    the tail filled with stride, and kv_num_indices.  Every step is rounded to bf16 as the
    reference's bf16 torch ops are (python/spattn/mask_utils.py:390-413); among equal scores
    the lower key wins."""
    B, H, S, D = q.shape
    nb = (S + blocksz - 1) // blocksz
    select_k = min(int(select_k), S)
    stride = _padded(select_k)
    kv_indices = torch.full((B, H, nb, stride), stride, dtype=torch.int32, device=q.device)
    kv_num_indices = torch.empty((B, H, nb), dtype=torch.int32, device=q.device)
    score = torch.empty((B, H, nb, _padded(S)), dtype=torch.bfloat16, device=q.device)
    qmean = torch.empty((B, H, nb, D), dtype=torch.bfloat16, device=q.device)
    spattn_interface.qk_topkmask_indices(kv_indices, kv_num_indices, score, qmean, q.contiguous(), k.contiguous(),
                                         select_k, blocksz)
    return kv_indices, kv_num_indices


# ----------------------------------------------------------------------------------
# bit packing (python/spattn/mask_utils.py:421-439)
# ----------------------------------------------------------------------------------
def pack(bool_tensor):
    """8 booleans -> one uint8, least significant bit first; the last dim must be a multiple of 8."""
    w = torch.tensor([1, 2, 4, 8, 16, 32, 64, 128], dtype=torch.uint8, device=bool_tensor.device)
    grouped = bool_tensor.reshape(*bool_tensor.shape[:-1], bool_tensor.shape[-1] // 8, 8).to(torch.uint8)
    return (grouped * w).sum(dim=-1).to(torch.uint8)


def unpack(packed_tensor):
    w = torch.tensor([1, 2, 4, 8, 16, 32, 64, 128], dtype=torch.uint8, device=packed_tensor.device)
    bits = (packed_tensor.unsqueeze(-1) & w) != 0
    return bits.reshape(*packed_tensor.shape[:-1], packed_tensor.shape[-1] * 8)
