"""GPU: the allocation-free balanced block-list attention against the entry point it restates
(qblock_order + sp_attn_blocks_ordered), through the C ABI, bit for bit: two calls in a row on
one device, the second on a smaller input, so that what the first call left in the library's
work-order array lies behind the part the second one uses."""
import ctypes

import numpy as np
import pytest
import torch

from fgattn_tk_cuda_amd import capi, workloads as wl

pytestmark = pytest.mark.gpu


def _case(dev, B, H, S, D, qblk, seed):
    q, k, v = (t.to(dev) for t in wl.randn_qkv(B, H, S, D, seed=seed))
    nq = wl.ceil_div(S, qblk)
    cnt = wl.zipf_counts(B, H, nq, s=1.2, lo=1, hi=wl.ceil_div(S, 64), seed=seed + 1)
    bi, bc = (t.to(dev) for t in wl.ragged_block_lists(B, H, S, qblk, 64, cnt, seed=seed + 2))
    return q, k, v, bi, bc


def _both(dev, q, k, v, bi, bc, qblk):
    lib = capi.load()
    B, H, S, D = (int(x) for x in q.shape)
    st = torch.cuda.current_stream().cuda_stream
    o_new = torch.full_like(q, float("nan"))
    l_new = torch.full((B, H, S), float("nan"), device=dev)
    rc = lib.spattn_sp_attn_blocks_balanced(o_new.data_ptr(), l_new.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                            bi.data_ptr(), bc.data_ptr(), int(bi.shape[3]), qblk, B, H, S, D, 0,
                                            ctypes.c_float(0.0), st)
    assert rc == 0, lib.spattn_status_string(rc)
    order = torch.full((bc.numel(),), -1, dtype=torch.int32, device=dev)
    assert lib.spattn_qblock_order(order.data_ptr(), bc.data_ptr(), bc.numel(), st) == 0
    o_old = torch.full_like(q, float("nan"))
    l_old = torch.full((B, H, S), float("nan"), device=dev)
    rc = lib.spattn_sp_attn_blocks_ordered(o_old.data_ptr(), l_old.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                           bi.data_ptr(), bc.data_ptr(), order.data_ptr(), int(bi.shape[3]), qblk, B, H,
                                           S, D, 0, ctypes.c_float(0.0), st)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.isfinite(o_old.float()).all()
    assert torch.equal(o_new, o_old) and torch.equal(l_new, l_old)
    # the order really is a reordering here (uneven lists), so the array was used
    assert not np.array_equal(order.cpu().numpy(), np.arange(bc.numel()))


def test_balanced_block_attention_without_allocation_two_calls(dev):
    print("case balanced no-alloc", flush=True)
    lib = capi.load()
    assert lib.spattn_init() == 0
    big = _case(dev, 1, 3, 2048, 128, 64, seed=5)
    small = _case(dev, 1, 2, 640, 64, 128, seed=9)
    _both(dev, *big, 64)
    _both(dev, *small, 128)
    # more q-blocks than the array holds: rejected before anything is launched
    q, k, v, bi, bc = small
    rc = lib.spattn_sp_attn_blocks_balanced(q.data_ptr(), None, q.data_ptr(), k.data_ptr(), v.data_ptr(), bi.data_ptr(),
                                            bc.data_ptr(), 1, 64, 1, 1 << 15, 64 * 33, 64, 0, ctypes.c_float(0.0),
                                            torch.cuda.current_stream().cuda_stream)
    assert rc == -7 and b"q-blocks" in lib.spattn_status_string(rc)
