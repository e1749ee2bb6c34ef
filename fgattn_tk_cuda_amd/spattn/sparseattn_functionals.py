"""Model-facing attention functions of the reference's ``spattn/sparseattn_functionals.py``.

Each takes ``(query, key, value, current_layer, ditrun, **kwargs)`` with bf16 tensors
[B,H,S,D] and returns the bf16 output, like the reference
(python/spattn/sparseattn_functionals.py:10-154).  Outputs are allocated on the device
of ``query``.
"""
from __future__ import annotations

import torch

from . import mask_utils
from . import cuda_attn  # noqa: F401

spattn_interface = torch.ops.cuda_attn


def _out_like(query):
    return torch.empty(query.shape, device=query.device, dtype=torch.bfloat16)


def _c(*tensors):
    return tuple(t.contiguous() for t in tensors)


def baseline_attn(query, key, value, current_layer=None, ditrun=None, *args, **kwargs):
    """Dense attention (python/spattn/sparseattn_functionals.py:10-15)."""
    out = _out_like(query)
    spattn_interface.full_attn(out, *_c(query, key, value))
    return out


def _dense_with_stats(query, key, value):
    out = _out_like(query)
    max_q, denom = mask_utils._stats_buffers(query)
    spattn_interface.fullattn_maxq_denom(out, max_q, denom, *_c(query, key, value))
    return out, max_q, denom


def baseline_attn_maxq_denom(query, key, value, current_layer=None, ditrun=None, *args, **kwargs):
    """Dense attention through the fused statistics kernel (:18-26)."""
    return _dense_with_stats(query, key, value)[0]


def _sparse(query, key, value, kv_indices, kv_num_indices, order=None, cached=False):
    """order: the work order that a cache computed when it stored these lists.  With it, or with
    cached=True and no order (lists of even length), the step is one launch and allocates only
    the output; without, ``sp_attn`` derives the order from the counts on every call."""
    out = _out_like(query)
    if order is not None or cached:
        spattn_interface.sp_attn_ex(out, None, *_c(query, key, value, kv_indices, kv_num_indices), order, 0.0, 0)
    else:
        spattn_interface.sp_attn(out, *_c(query, key, value, kv_indices, kv_num_indices))
    return out


def _cached_order(mask_cache, layer):
    get = getattr(mask_cache, "get_order", None)
    return get(layer) if get is not None else None


def attn_computed_with_sparse_mask_python(query, key, value, current_layer=None, ditrun=None, *args, **kwargs):
    """Index lists from the pure-torch mask definition, then sparse attention (:29-36)."""
    kv_indices, kv_num_indices = mask_utils.qk_indexmask(query, key, kwargs["thresh"], blocksz=kwargs["blocksz"])
    return _sparse(query, key, value, kv_indices, kv_num_indices)


def attn_lshmask_cuda(query, key, value, current_layer=None, ditrun=None, *args, **kwargs):
    """LSH-selected key lists, then sparse attention (:51-58).  As in the reference the selector is
    not implemented (python/spattn/mask_utils.py:385-386): the call raises NotImplementedError."""
    kv_indices, kv_num_indices = mask_utils.qk_lshmask_indices(query, key, kwargs["thresh"], blocksz=kwargs["blocksz"])
    return _sparse(query, key, value, kv_indices, kv_num_indices)


def attn_topkmask_cuda(query, key, value, current_layer=None, ditrun=None, *args, **kwargs):
    """Top-k key lists per q-block, then sparse attention (:39-48).  The lists come from the
    device selector, padded to a multiple of 128 keys as the sparse operator needs."""
    select_k = kwargs.get("select_k") or query.shape[2]
    kv_indices, kv_num_indices = mask_utils.qk_topkmask_indices_cuda(query, key, select_k, blocksz=kwargs["blocksz"])
    return _sparse(query, key, value, kv_indices, kv_num_indices)


def attn_computed_with_sparse_mask_cuda(query, key, value, *args, **kwargs):
    """Threshold pre-pass on the device, then sparse attention (:62-70)."""
    kv_indices, kv_num_indices = mask_utils.qk_indexmask_cuda(query, key, kwargs["thresh"], blocksz=kwargs["blocksz"])
    return _sparse(query, key, value, kv_indices, kv_num_indices)


def compute_cache_and_attn_cuda(query, key, value, *args, **kwargs):
    """Dense attention plus the index lists for later steps (:75-85)."""
    out, max_q, denom = _dense_with_stats(query, key, value)
    kv_indices, kv_num_indices = mask_utils.qk_indexmask_from_maxq_denom_cuda(
        max_q, denom, query, key, kwargs["thresh"], blocksz=kwargs["blocksz"])
    return out, kv_indices, kv_num_indices


def sparse_attn_from_cache_cuda(query, key, value, *args, **kwargs):
    """Sparse attention from cached lists (:88-93)."""
    kv_indices, kv_num_indices = kwargs["mask_cache"].get_mask_from_cache(kwargs.get("current_layer"))
    return _sparse(query, key, value, kv_indices, kv_num_indices, _cached_order(kwargs["mask_cache"], kwargs.get("current_layer")))


def cached_attn_cuda(query, key, value, current_layer, ditrun, *args, **kwargs):
    """On the steps that refresh the cache: dense attention with statistics, then the mask
    pre-pass; on every other step: sparse attention from the cached lists (:95-114).
    Where the buffer for it fits the budget, the refresh step sweeps Q K^T once in full instead of
    twice: the dense pass also writes the score maximum of every row over every 64-key block (bf16,
    S*S/32 bytes per head, freed on return) and the threshold sweep then runs over the key blocks that
    can hold a key only; the lists are the same.  ``onepass=True`` / ``False`` forces one route
    (False: the reference's two full sweeps, no extra buffer); by default the route is the one-sweep
    one when the buffer is at most ``blockmax_budget_bytes`` (default
    ``mask_utils.BLOCKMAX_BUDGET_BYTES``, 2 GiB)."""
    mask_cache = kwargs["mask_cache"]
    if mask_cache.run_fullattn(ditrun):
        if mask_utils.use_onepass(query, kwargs.get("onepass"), kwargs.get("blockmax_budget_bytes")):
            # the dense pass also writes the block maxima; the threshold sweep then runs over the key
            # blocks that can hold a key only
            out = _out_like(query)
            max_q, denom = mask_utils._stats_buffers(query)
            blockmax = mask_utils.blockmax_buffer(query)
            spattn_interface.fullattn_maxq_denom_blockmax(out, max_q, denom, blockmax, *_c(query, key, value), 0.0, 0)
            kv_indices, kv_num_indices = mask_utils.qk_indexmask_from_blockmax_cuda(
                blockmax, max_q, denom, query, key, kwargs["thresh"], blocksz=kwargs["blocksz"])
        else:
            # the reference's two full sweeps; the votes of the second leave it as bits (1/32 of the
            # int32 mask of python/spattn/mask_utils.py:358-382, the same lists)
            out, max_q, denom = _dense_with_stats(query, key, value)
            packed = mask_utils.qk_packedmask_from_maxq_denom_cuda(max_q, denom, query, key, kwargs["thresh"], kwargs["blocksz"])
            kv_indices, kv_num_indices = mask_utils.packedmask_to_indexmask_cuda(packed, query.shape[2])
        mask_cache.update_cache(current_layer, kv_indices, kv_num_indices)
        return out
    kv_indices, kv_num_indices = mask_cache.get_mask_from_cache(current_layer)
    return _sparse(query, key, value, kv_indices, kv_num_indices, _cached_order(mask_cache, current_layer))


def blockcached_attn_cuda(query, key, value, current_layer, ditrun, *args, **kwargs):
    """cached_attn_cuda at the granularity of 64-key blocks (no counterpart in the reference):
    on the refresh steps dense attention with statistics and per-block score maxima, whose threshold
    gives the block lists for q-blocks of ``qblk`` rows (64 or 128, default 128) without a second
    sweep (``onepass=False``, or a block-maxima buffer above ``blockmax_budget_bytes`` as in
    ``cached_attn_cuda``: the bit-packed threshold sweep instead), kept in a
    ``mask_utils.BlockListCache``; on every other step ``sp_attn_block`` over the cached lists in
    their cached work order - one launch."""
    mask_cache = kwargs["mask_cache"]
    qblk = kwargs.get("qblk", 128)
    if mask_cache.run_fullattn(ditrun):
        if mask_utils.use_onepass(query, kwargs.get("onepass"), kwargs.get("blockmax_budget_bytes")):
            # the dense pass also writes the per-(row, key block) score maxima: the lists come from
            # thresholding those, without a second sweep over Q K^T
            out = _out_like(query)
            max_q, denom = mask_utils._stats_buffers(query)
            blockmax = mask_utils.blockmax_buffer(query)
            spattn_interface.fullattn_maxq_denom_blockmax(out, max_q, denom, blockmax, *_c(query, key, value), 0.0, 0)
            blk_idx, blk_cnt = mask_utils.blockmax_to_blocklists_cuda(blockmax, max_q, denom, kwargs["thresh"], query.shape[2],
                                                                    query.shape[3], qblk)
        else:
            out, max_q, denom = _dense_with_stats(query, key, value)
            blk_idx, blk_cnt = mask_utils.qk_blocklists_from_maxq_denom_cuda(max_q, denom, query, key, kwargs["thresh"], qblk)
        mask_cache.update_cache(current_layer, blk_idx, blk_cnt)
        return out
    blk_idx, blk_cnt = mask_cache.get_mask_from_cache(current_layer)
    out = _out_like(query)
    spattn_interface.sp_attn_block(out, None, *_c(query, key, value, blk_idx, blk_cnt), mask_cache.get_order(current_layer),
                                   qblk, 0.0, 0)
    return out


def bitmaskcached_attn_cuda(query, key, value, current_layer, ditrun, *args, **kwargs):
    """Like cached_attn_cuda with the vote mask (not the lists) kept in the cache (:117-134)."""
    mask_cache = kwargs["mask_cache"]
    if mask_cache.run_fullattn(ditrun):
        out, max_q, denom = _dense_with_stats(query, key, value)
        bitmask = mask_utils.qk_bitmask_from_maxq_denom_cuda(max_q, denom, query, key, kwargs["thresh"], blocksz=kwargs["blocksz"])
        mask_cache.update_cache(current_layer, bitmask, query.shape[2])
        return out
    kv_indices, kv_num_indices = mask_cache.get_mask_from_cache(current_layer)
    return _sparse(query, key, value, kv_indices, kv_num_indices)


def attn_2xmask_cuda(query, key, value, current_layer=None, ditrun=None, *args, **kwargs):
    """Every second key (:137-154)."""
    B, H, S, _ = query.shape
    blocksz = kwargs["blocksz"]
    nb = (S + blocksz - 1) // blocksz
    stride = mask_utils._padded(S)
    row = torch.full((stride,), stride, dtype=torch.int32, device=query.device)
    row[: S // 2] = 2 * torch.arange(S // 2, dtype=torch.int32, device=query.device)
    kv_indices = row.expand(B, H, nb, stride).contiguous()
    kv_num_indices = torch.full((B, H, nb), S // 2, dtype=torch.int32, device=query.device)
    return _sparse(query, key, value, kv_indices, kv_num_indices)
