"""ctypes binding of libspattn_hip.so (declared in include/spattn_hip.h).

Tensors are torch device tensors used only as owners of HBM; the calls pass raw
pointers and sizes.  There is no fallback: a missing library raises.
"""
from __future__ import annotations

import ctypes
import math
from pathlib import Path

import torch

_LIB_PATH = Path(__file__).resolve().parent / "libspattn_hip.so"
_lib = None

_c_int, _c_float, _c_void_p = ctypes.c_int, ctypes.c_float, ctypes.c_void_p

# name -> argtypes, for every symbol the header declares
_SIGNATURES = {
    # the reference's binding surface (void return)
    "attn_fwd_wg_impl": (None, [_c_void_p] * 4 + [_c_int] * 4),
    "attn_sparse_fwd_wg_impl": (None, [_c_void_p] * 6 + [_c_int] * 5),
    "allindex_mask_impl": (None, [_c_void_p] * 2 + [_c_int] * 4),
    "attn_maxq_denom_impl": (None, [_c_void_p] * 6 + [_c_int] * 4),
    "maxq_denom_impl": (None, [_c_void_p] * 4 + [_c_int] * 4),
    "booleanmask_128_impl": (None, [_c_void_p, _c_float, _c_int] + [_c_void_p] * 4 + [_c_int] * 4),
    "booleanmask_to_indexmask_impl": (None, [_c_void_p] * 3 + [_c_int] * 5),
    # extended entry points (status return)
    "spattn_full_attn": (_c_int, [_c_void_p] * 5 + [_c_int] * 5 + [_c_float, _c_void_p]),
    "spattn_sp_attn": (_c_int, [_c_void_p] * 7 + [_c_int] * 7 + [_c_float, _c_void_p]),
    "spattn_sp_attn_blocks": (_c_int, [_c_void_p] * 7 + [_c_int] * 7 + [_c_float, _c_void_p]),
    "spattn_sp_attn_ordered": (_c_int, [_c_void_p] * 8 + [_c_int] * 7 + [_c_float, _c_void_p]),
    "spattn_sp_attn_blocks_ordered": (_c_int, [_c_void_p] * 8 + [_c_int] * 7 + [_c_float, _c_void_p]),
    "spattn_sp_attn_blocks_balanced": (_c_int, [_c_void_p] * 7 + [_c_int] * 7 + [_c_float, _c_void_p]),
    "spattn_init": (_c_int, []),
    "spattn_qblock_order": (_c_int, [_c_void_p] * 2 + [_c_int, _c_void_p]),
    "spattn_all_index_mask": (_c_int, [_c_void_p] * 2 + [_c_int] * 5 + [_c_void_p]),
    "spattn_fullattn_maxq_denom": (_c_int, [_c_void_p] * 6 + [_c_int] * 5 + [_c_float, _c_void_p]),
    "spattn_maxq_denom": (_c_int, [_c_void_p] * 4 + [_c_int] * 5 + [_c_float, _c_void_p]),
    "spattn_booleanmask_128": (_c_int, [_c_void_p, _c_float, _c_int] + [_c_void_p] * 4 + [_c_int] * 5 + [_c_float, _c_void_p]),
    "spattn_booleanmask_to_indexmask": (_c_int, [_c_void_p] * 3 + [_c_int] * 5 + [_c_void_p]),
    "spattn_booleanmask_packed": (_c_int, [_c_void_p, _c_float, _c_int, _c_int] + [_c_void_p] * 4 + [_c_int] * 5 + [_c_float, _c_void_p]),
    "spattn_packedmask_to_blocklists": (_c_int, [_c_void_p] * 4 + [_c_int] * 6 + [_c_void_p]),
    "spattn_booleanmask_to_blocklists": (_c_int, [_c_void_p] * 4 + [_c_int] * 6 + [_c_void_p]),
    "spattn_maxq_denom_blockmax": (_c_int, [_c_void_p] * 5 + [_c_int] * 5 + [_c_float, _c_void_p]),
    "spattn_fullattn_maxq_denom_blockmax": (_c_int, [_c_void_p] * 7 + [_c_int] * 5 + [_c_float, _c_void_p]),
    "spattn_blockmax_to_blocklists": (_c_int, [_c_void_p] * 6 + [_c_float] + [_c_int] * 6 + [_c_float, _c_int, _c_void_p]),
    "spattn_booleanmask_128_blocks": (_c_int, [_c_void_p, _c_float, _c_int] + [_c_void_p] * 6 + [_c_int] * 6 + [_c_float, _c_void_p]),
    "spattn_booleanmask_packed_blocks": (_c_int, [_c_void_p, _c_float, _c_int, _c_int] + [_c_void_p] * 6 + [_c_int] * 6 + [_c_float, _c_void_p]),
    "spattn_pack_mask": (_c_int, [_c_void_p] * 2 + [_c_int] * 4 + [_c_void_p]),
    "spattn_packedmask_to_indexmask": (_c_int, [_c_void_p] * 3 + [_c_int] * 5 + [_c_void_p]),
    "spattn_qk_topkmask_indices": (_c_int, [_c_void_p] * 6 + [_c_int] * 9 + [_c_void_p]),
    "spattn_last_status": (_c_int, []),
    "spattn_status_string": (ctypes.c_char_p, [_c_int]),
    "spattn_version": (_c_int, []),
}


class SpattnError(RuntimeError):
    def __init__(self, status: int, text: str):
        super().__init__("spattn status %d: %s" % (status, text))
        self.status = status


def lib_path() -> Path:
    return _LIB_PATH


def exported_symbols():
    return sorted(_SIGNATURES)


def load() -> ctypes.CDLL:
    """Load libspattn_hip.so; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not _LIB_PATH.exists():
            raise RuntimeError(
                "%s is missing: build it with `python -m fgattn_tk_cuda_amd.build --lib-only`" % _LIB_PATH)
        lib = ctypes.CDLL(str(_LIB_PATH))
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def _check(status: int) -> None:
    if status != 0:
        raise SpattnError(status, load().spattn_status_string(status).decode())


def _ptr(t, dtype=None):
    if t is None:
        return None
    if not t.is_cuda:
        raise ValueError("expected a device tensor")
    if not t.is_contiguous():
        raise ValueError("expected a contiguous tensor")
    if dtype is not None and t.dtype != dtype:
        raise ValueError("expected dtype %s, got %s" % (dtype, t.dtype))
    return t.data_ptr()


def _stream(stream=None):
    if stream is None:
        stream = torch.cuda.current_stream()
    return stream.cuda_stream


def _bhsd(q):
    if q.dim() != 4:
        raise ValueError("q must be [B,H,S,D]")
    return tuple(int(x) for x in q.shape)


bf16, i32, f32 = torch.bfloat16, torch.int32, torch.float32


def full_attn(o, q, k, v, *, lse=None, kv_len=0, scale=0.0, stream=None):
    B, H, S, D = _bhsd(q)
    _check(load().spattn_full_attn(_ptr(o, bf16), _ptr(lse, f32), _ptr(q, bf16), _ptr(k, bf16), _ptr(v, bf16),
                                   B, H, S, D, kv_len, scale, _stream(stream)))


def sp_attn(o, q, k, v, kv_indices, kv_num_indices, *, lse=None, qblk=None, kv_len=0, scale=0.0, order=None,
            stream=None):
    """Token-list sparse attention.  qblk defaults to the value implied by kv_indices.shape[2].
    order: optional int32 [B*H*SB] work order from qblock_order (same results, better balance
    when the lists differ much in length)."""
    B, H, S, D = _bhsd(q)
    if kv_indices.dim() != 4:
        raise ValueError("kv_indices must be [B,H,SB,mask_stride]")
    if qblk is None:
        qblk = infer_qblk(S, int(kv_indices.shape[2]))
    if kv_num_indices.numel() != B * H * int(kv_indices.shape[2]):
        raise ValueError("kv_num_indices must have B*H*SB entries")
    if order is None:
        _check(load().spattn_sp_attn(_ptr(o, bf16), _ptr(lse, f32), _ptr(q, bf16), _ptr(k, bf16), _ptr(v, bf16),
                                     _ptr(kv_indices, i32), _ptr(kv_num_indices, i32), int(kv_indices.shape[3]), qblk,
                                     B, H, S, D, kv_len, scale, _stream(stream)))
        return
    if order.numel() != kv_num_indices.numel():
        raise ValueError("order must have B*H*SB entries")
    _check(load().spattn_sp_attn_ordered(_ptr(o, bf16), _ptr(lse, f32), _ptr(q, bf16), _ptr(k, bf16), _ptr(v, bf16),
                                         _ptr(kv_indices, i32), _ptr(kv_num_indices, i32), _ptr(order, i32),
                                         int(kv_indices.shape[3]), qblk, B, H, S, D, kv_len, scale, _stream(stream)))


def sp_attn_blocks(o, q, k, v, blk_indices, blk_counts, *, lse=None, qblk=None, kv_len=0, scale=0.0, order=None,
                   stream=None):
    """Block-list sparse attention over 64-key blocks.  order: as for sp_attn."""
    B, H, S, D = _bhsd(q)
    if blk_indices.dim() != 4:
        raise ValueError("blk_indices must be [B,H,SB,max_blocks]")
    if qblk is None:
        qblk = infer_qblk(S, int(blk_indices.shape[2]))
    if blk_counts.numel() != B * H * int(blk_indices.shape[2]):
        raise ValueError("blk_counts must have B*H*SB entries")
    if order is None:
        _check(load().spattn_sp_attn_blocks(_ptr(o, bf16), _ptr(lse, f32), _ptr(q, bf16), _ptr(k, bf16), _ptr(v, bf16),
                                            _ptr(blk_indices, i32), _ptr(blk_counts, i32), int(blk_indices.shape[3]),
                                            qblk, B, H, S, D, kv_len, scale, _stream(stream)))
        return
    if order.numel() != blk_counts.numel():
        raise ValueError("order must have B*H*SB entries")
    _check(load().spattn_sp_attn_blocks_ordered(_ptr(o, bf16), _ptr(lse, f32), _ptr(q, bf16), _ptr(k, bf16),
                                                _ptr(v, bf16), _ptr(blk_indices, i32), _ptr(blk_counts, i32),
                                                _ptr(order, i32), int(blk_indices.shape[3]), qblk, B, H, S, D, kv_len,
                                                scale, _stream(stream)))


BALANCED_MAX_QBLOCKS = 1 << 20


def sp_attn_blocks_balanced(o, q, k, v, blk_indices, blk_counts, *, lse=None, qblk=None, kv_len=0, scale=0.0, stream=None):
    """sp_attn_blocks in longest-list-first order with the order kept in the library's own device
    array: allocates nothing.  Calls that overlap on one device race on that array."""
    B, H, S, D = _bhsd(q)
    if blk_indices.dim() != 4:
        raise ValueError("blk_indices must be [B,H,SB,max_blocks]")
    if qblk is None:
        qblk = infer_qblk(S, int(blk_indices.shape[2]))
    if blk_counts.numel() != B * H * int(blk_indices.shape[2]):
        raise ValueError("blk_counts must have B*H*SB entries")
    _check(load().spattn_sp_attn_blocks_balanced(_ptr(o, bf16), _ptr(lse, f32), _ptr(q, bf16), _ptr(k, bf16), _ptr(v, bf16),
                                                 _ptr(blk_indices, i32), _ptr(blk_counts, i32), int(blk_indices.shape[3]),
                                                 qblk, B, H, S, D, kv_len, scale, _stream(stream)))


def init():
    """Sets up, on the current device, what a first call would otherwise set (the library's work-order
    array, the dynamic-LDS limit of every attention kernel): afterwards every entry point only launches."""
    _check(load().spattn_init())


def qblock_order(order, counts, *, stream=None):
    """order: int32 [n] <- the q-blocks (flat indices of counts) longest list first; lists within
    a factor of two of each other keep the default order."""
    if order.numel() != counts.numel():
        raise ValueError("order and counts must have the same number of entries")
    _check(load().spattn_qblock_order(_ptr(order, i32), _ptr(counts, i32), int(counts.numel()), _stream(stream)))


def all_index_mask(kv_indices, kv_num_indices, batch, heads, seqblocks, seq, *, stream=None):
    _check(load().spattn_all_index_mask(_ptr(kv_indices, i32), _ptr(kv_num_indices, i32), batch, heads, seqblocks, seq,
                                        int(kv_indices.shape[-1]), _stream(stream)))


def fullattn_maxq_denom(o, max_q, denom, q, k, v, *, kv_len=0, scale=0.0, stream=None):
    B, H, S, D = _bhsd(q)
    _need_padded(max_q, denom, B, H, S)
    _check(load().spattn_fullattn_maxq_denom(_ptr(o, bf16), _ptr(max_q, f32), _ptr(denom, f32), _ptr(q, bf16),
                                             _ptr(k, bf16), _ptr(v, bf16), B, H, S, D, kv_len, scale, _stream(stream)))


def maxq_denom(max_q, denom, q, k, *, kv_len=0, scale=0.0, stream=None):
    B, H, S, D = _bhsd(q)
    _need_padded(max_q, denom, B, H, S)
    _check(load().spattn_maxq_denom(_ptr(max_q, f32), _ptr(denom, f32), _ptr(q, bf16), _ptr(k, bf16), B, H, S, D,
                                    kv_len, scale, _stream(stream)))


def booleanmask_128(booleanmask, max_q, denom, q, k, threshold, *, kv_len=0, scale=0.0, stream=None):
    B, H, S, D = _bhsd(q)
    _need_padded(max_q, denom, B, H, S)
    if booleanmask.dim() != 4 or int(booleanmask.shape[2]) != (S + 127) // 128:
        raise ValueError("booleanmask must be [B,H,ceil(S/128),mask_stride]")
    _check(load().spattn_booleanmask_128(_ptr(booleanmask, i32), float(threshold), int(booleanmask.shape[3]),
                                         _ptr(max_q, f32), _ptr(denom, f32), _ptr(q, bf16), _ptr(k, bf16), B, H, S, D,
                                         kv_len, scale, _stream(stream)))


def booleanmask_to_indexmask(kv_indices, kv_num_indices, booleanmask, seq, *, stream=None):
    if booleanmask.dim() != 4:
        raise ValueError("booleanmask must be [B,H,SB,mask_stride]")
    B, H, SB, MS = (int(x) for x in booleanmask.shape)
    if tuple(kv_indices.shape) != (B, H, SB, MS) or kv_num_indices.numel() != B * H * SB:
        raise ValueError("kv_indices / kv_num_indices do not match booleanmask")
    _check(load().spattn_booleanmask_to_indexmask(_ptr(kv_indices, i32), _ptr(kv_num_indices, i32),
                                                  _ptr(booleanmask, i32), B, H, int(seq), SB, MS, _stream(stream)))


def booleanmask_packed(packed, max_q, denom, q, k, threshold, *, qblk=128, kv_len=0, scale=0.0, stream=None):
    """Threshold sweep with a bit-packed result: packed uint8 [B,H,ceil(S/qblk),mask_stride/8], bit
    (c & 7) of byte c >> 3 set where some row of the q-block has softmax(row, c) > threshold."""
    B, H, S, D = _bhsd(q)
    _need_padded(max_q, denom, B, H, S)
    if qblk not in (64, 128):
        raise ValueError("qblk must be 64 or 128")
    if packed.dim() != 4 or tuple(packed.shape[:3]) != (B, H, (S + qblk - 1) // qblk):
        raise ValueError("packed must be uint8 [B,H,ceil(S/qblk),mask_stride/8]")
    _check(load().spattn_booleanmask_packed(_ptr(packed, torch.uint8), float(threshold), int(packed.shape[3]) * 8,
                                            int(qblk), _ptr(max_q, f32), _ptr(denom, f32), _ptr(q, bf16), _ptr(k, bf16),
                                            B, H, S, D, kv_len, scale, _stream(stream)))


def _lists128(blk_indices, blk_counts, B, H, S):
    SB = (S + 127) // 128
    if blk_indices.dim() != 4 or tuple(blk_indices.shape[:3]) != (B, H, SB) or blk_counts.numel() != B * H * SB:
        raise ValueError("blk_indices must be [B,H,ceil(S/128),max_blocks] and blk_counts hold B*H*ceil(S/128) entries")


def booleanmask_128_blocks(booleanmask, max_q, denom, q, k, threshold, blk_indices, blk_counts, *, kv_len=0, scale=0.0,
                           stream=None):
    """booleanmask_128 restricted to the 64-key blocks listed per 128-row q-block; the rest of the mask is zeroed."""
    B, H, S, D = _bhsd(q)
    _need_padded(max_q, denom, B, H, S)
    _lists128(blk_indices, blk_counts, B, H, S)
    if booleanmask.dim() != 4 or int(booleanmask.shape[2]) != (S + 127) // 128:
        raise ValueError("booleanmask must be [B,H,ceil(S/128),mask_stride]")
    _check(load().spattn_booleanmask_128_blocks(_ptr(booleanmask, i32), float(threshold), int(booleanmask.shape[3]),
                                                _ptr(max_q, f32), _ptr(denom, f32), _ptr(q, bf16), _ptr(k, bf16),
                                                _ptr(blk_indices, i32), _ptr(blk_counts, i32), int(blk_indices.shape[3]),
                                                B, H, S, D, kv_len, scale, _stream(stream)))


def booleanmask_packed_blocks(packed, max_q, denom, q, k, threshold, blk_indices, blk_counts, *, qblk=128, kv_len=0,
                              scale=0.0, stream=None):
    """booleanmask_packed restricted to the listed blocks (lists per 128-row q-block for either qblk)."""
    B, H, S, D = _bhsd(q)
    _need_padded(max_q, denom, B, H, S)
    _lists128(blk_indices, blk_counts, B, H, S)
    if qblk not in (64, 128):
        raise ValueError("qblk must be 64 or 128")
    if packed.dim() != 4 or tuple(packed.shape[:3]) != (B, H, (S + qblk - 1) // qblk):
        raise ValueError("packed must be uint8 [B,H,ceil(S/qblk),mask_stride/8]")
    _check(load().spattn_booleanmask_packed_blocks(_ptr(packed, torch.uint8), float(threshold), int(packed.shape[3]) * 8,
                                                   int(qblk), _ptr(max_q, f32), _ptr(denom, f32), _ptr(q, bf16),
                                                   _ptr(k, bf16), _ptr(blk_indices, i32), _ptr(blk_counts, i32),
                                                   int(blk_indices.shape[3]), B, H, S, D, kv_len, scale, _stream(stream)))


def _blocklist_args(blk_indices, blk_counts, blockmask, B, H, SB, MS):
    if blk_indices.dim() != 4 or tuple(blk_indices.shape[:3]) != (B, H, SB) or blk_counts.numel() != B * H * SB:
        raise ValueError("blk_indices must be [B,H,SB,max_blocks] and blk_counts hold B*H*SB entries")
    if blockmask is not None and tuple(blockmask.shape) != (B, H, SB, MS // 64):
        raise ValueError("blockmask must be uint8 [B,H,SB,mask_stride/64]")


def packedmask_to_blocklists(blk_indices, blk_counts, packed, seq, *, blockmask=None, stream=None):
    """Ascending lists of the 64-key blocks that hold a set key c < seq, from a bit-packed mask
    (uint8 [B,H,SB,mask_stride/8]); blockmask: optional uint8 [B,H,SB,mask_stride/64] output."""
    if packed.dim() != 4:
        raise ValueError("packed must be [B,H,SB,mask_stride/8]")
    B, H, SB, MB = (int(x) for x in packed.shape)
    _blocklist_args(blk_indices, blk_counts, blockmask, B, H, SB, MB * 8)
    _check(load().spattn_packedmask_to_blocklists(_ptr(blk_indices, i32), _ptr(blk_counts, i32),
                                                  _ptr(blockmask, torch.uint8), _ptr(packed, torch.uint8), B, H,
                                                  int(seq), SB, MB * 8, int(blk_indices.shape[3]), _stream(stream)))


def booleanmask_to_blocklists(blk_indices, blk_counts, booleanmask, seq, *, blockmask=None, stream=None):
    """The same from the int32 vote mask [B,H,SB,mask_stride]."""
    if booleanmask.dim() != 4:
        raise ValueError("booleanmask must be [B,H,SB,mask_stride]")
    B, H, SB, MS = (int(x) for x in booleanmask.shape)
    _blocklist_args(blk_indices, blk_counts, blockmask, B, H, SB, MS)
    _check(load().spattn_booleanmask_to_blocklists(_ptr(blk_indices, i32), _ptr(blk_counts, i32),
                                                   _ptr(blockmask, torch.uint8), _ptr(booleanmask, i32), B, H, int(seq),
                                                   SB, MS, int(blk_indices.shape[3]), _stream(stream)))


def _need_blockmax(blockmax, B, H, S):
    sp = 128 * ((S + 127) // 128)
    if blockmax.numel() != B * H * (sp // 64) * sp:
        raise ValueError("blockmax must be bf16 [B,H,%d,%d]" % (sp // 64, sp))


def maxq_denom_blockmax(max_q, denom, blockmax, q, k, *, kv_len=0, scale=0.0, stream=None):
    """maxq_denom that also writes blockmax bf16 [B,H,Sp/64,Sp] (rounded toward +inf): [J][r] = max of q[r].k[c] over the keys c < kv_len
    of 64-key block J (blocks without such a key are left as they are)."""
    B, H, S, D = _bhsd(q)
    _need_padded(max_q, denom, B, H, S)
    _need_blockmax(blockmax, B, H, S)
    _check(load().spattn_maxq_denom_blockmax(_ptr(max_q, f32), _ptr(denom, f32), _ptr(blockmax, bf16), _ptr(q, bf16),
                                             _ptr(k, bf16), B, H, S, D, kv_len, scale, _stream(stream)))


def fullattn_maxq_denom_blockmax(o, max_q, denom, blockmax, q, k, v, *, kv_len=0, scale=0.0, stream=None):
    """fullattn_maxq_denom with the blockmax output of maxq_denom_blockmax."""
    B, H, S, D = _bhsd(q)
    _need_padded(max_q, denom, B, H, S)
    _need_blockmax(blockmax, B, H, S)
    _check(load().spattn_fullattn_maxq_denom_blockmax(_ptr(o, bf16), _ptr(max_q, f32), _ptr(denom, f32),
                                                      _ptr(blockmax, bf16), _ptr(q, bf16), _ptr(k, bf16), _ptr(v, bf16),
                                                      B, H, S, D, kv_len, scale, _stream(stream)))


def blockmax_to_blocklists(blk_indices, blk_counts, blockmax, max_q, denom, threshold, seq, D, *, qblk=128,
                           blockmask=None, kv_len=0, scale=0.0, stream=None):
    """Threshold test on the block maxima of a statistics sweep -> ascending 64-key block lists per
    q-block of qblk rows (and, optionally, the block mask uint8 [B,H,ceil(S/qblk),Sp/64])."""
    if blk_indices.dim() != 4:
        raise ValueError("blk_indices must be [B,H,ceil(S/qblk),max_blocks]")
    B, H, SB, MB = (int(x) for x in blk_indices.shape)
    S = int(seq)
    if qblk not in (64, 128) or SB != (S + qblk - 1) // qblk:
        raise ValueError("blk_indices must hold ceil(S/qblk) lists per head, qblk 64 or 128")
    _need_padded(max_q, denom, B, H, S)
    _need_blockmax(blockmax, B, H, S)
    _blocklist_args(blk_indices, blk_counts, blockmask, B, H, SB, 128 * ((S + 127) // 128))
    _check(load().spattn_blockmax_to_blocklists(_ptr(blk_indices, i32), _ptr(blk_counts, i32),
                                                _ptr(blockmask, torch.uint8), _ptr(blockmax, bf16), _ptr(max_q, f32),
                                                _ptr(denom, f32), float(threshold), int(qblk), B, H, S, int(D), kv_len,
                                                scale, MB, _stream(stream)))


def pack_mask(packed, booleanmask, *, stream=None):
    """packed: uint8 [B,H,SB,mask_stride/8]; bit (c & 7) of byte c >> 3 is set where booleanmask[..., c] > 0."""
    if booleanmask.dim() != 4:
        raise ValueError("booleanmask must be [B,H,SB,mask_stride]")
    B, H, SB, MS = (int(x) for x in booleanmask.shape)
    if tuple(packed.shape) != (B, H, SB, MS // 8) or MS % 8:
        raise ValueError("packed must be uint8 [B,H,SB,mask_stride/8]")
    _check(load().spattn_pack_mask(_ptr(packed, torch.uint8), _ptr(booleanmask, i32), B, H, SB, MS, _stream(stream)))


def packedmask_to_indexmask(kv_indices, kv_num_indices, packed, seq, *, stream=None):
    """Index lists straight from a bit-packed mask (uint8 [B,H,SB,mask_stride/8])."""
    if packed.dim() != 4:
        raise ValueError("packed must be [B,H,SB,mask_stride/8]")
    B, H, SB, MB = (int(x) for x in packed.shape)
    MS = MB * 8
    if tuple(kv_indices.shape) != (B, H, SB, MS) or kv_num_indices.numel() != B * H * SB:
        raise ValueError("kv_indices / kv_num_indices do not match the packed mask")
    _check(load().spattn_packedmask_to_indexmask(_ptr(kv_indices, i32), _ptr(kv_num_indices, i32),
                                                 _ptr(packed, torch.uint8), B, H, int(seq), SB, MS, _stream(stream)))


def qk_topkmask_indices(kv_indices, kv_num_indices, score, qmean, q, k, select_k, *, blocksz=128, kv_len=0,
                        stream=None):
    """Top-k keys per q-block by (block-mean query / sqrt(D)) . key; ascending key lists.
    score: bf16 [B,H,SB,score_stride] and qmean: bf16 [B,H,SB,D] are outputs as well."""
    B, H, S, D = (int(x) for x in q.shape)
    SB = (S + blocksz - 1) // blocksz
    if tuple(k.shape) != (B, H, S, D):
        raise ValueError("k must match q")
    if tuple(qmean.shape) != (B, H, SB, D) or score.dim() != 4 or tuple(score.shape[:3]) != (B, H, SB):
        raise ValueError("qmean must be [B,H,SB,D] and score [B,H,SB,score_stride]")
    if kv_indices.dim() != 4 or tuple(kv_indices.shape[:3]) != (B, H, SB) or kv_num_indices.numel() != B * H * SB:
        raise ValueError("kv_indices must be [B,H,SB,idx_stride] and kv_num_indices hold B*H*SB entries")
    bf = torch.bfloat16
    _check(load().spattn_qk_topkmask_indices(_ptr(kv_indices, i32), _ptr(kv_num_indices, i32), _ptr(score, bf),
                                             _ptr(qmean, bf), _ptr(q, bf), _ptr(k, bf), B, H, S, D, int(blocksz),
                                             int(kv_len), int(select_k), int(score.shape[3]),
                                             int(kv_indices.shape[3]), _stream(stream)))


def infer_qblk(seq: int, seqblocks: int) -> int:
    """Rows per q-block from the number of lists per head; 128 (the reference's) wins a tie."""
    if seqblocks == (seq + 127) // 128:
        return 128
    if seqblocks == (seq + 63) // 64:
        return 64
    raise ValueError("index tensor has %d q-blocks; expected ceil(S/128) or ceil(S/64)" % seqblocks)


def _need_padded(max_q, denom, B, H, S):
    sp = 128 * ((S + 127) // 128)
    for t in (max_q, denom):
        if t.numel() != B * H * sp:
            raise ValueError("max_q/denom must hold B*H*%d floats" % sp)


def default_scale(D: int) -> float:
    return 1.0 / math.sqrt(D)
