"""GPU: the longest-list-first work order and the attention entry points that take it."""
import numpy as np
import pytest
import torch

from fgattn_tk_cuda_amd import capi, workloads as wl
from oracle import spattn_oracle as orc

pytestmark = pytest.mark.gpu


def _order(dev, counts):
    c = torch.from_numpy(np.asarray(counts, np.int32)).to(dev)
    order = torch.full((c.numel(),), -1, dtype=torch.int32, device=dev)
    capi.qblock_order(order, c)
    torch.cuda.synchronize()
    return order.cpu().numpy()


@pytest.mark.parametrize("case", ["zipf", "uniform", "near_uniform", "zeros_and_ones", "tiny", "ragged_large", "powers"])
def test_qblock_order_bit_exact(dev, case):
    print("case order", case, flush=True)
    rng = np.random.default_rng(3)
    if case == "zipf":
        counts = wl.zipf_counts(1, 8, 512, s=1.2, lo=1, hi=1024, seed=3).reshape(-1)
    elif case == "uniform":
        counts = np.full(16384, 26)
    elif case == "near_uniform":
        counts = rng.integers(1500, 1650, size=3000)
    elif case == "zeros_and_ones":
        counts = rng.integers(0, 2, size=777)
    elif case == "tiny":
        counts = np.array([5, 900, 0, 17, 900, 3])
    elif case == "ragged_large":
        counts = rng.integers(0, 75000, size=100003)
    else:
        counts = np.array([1 << (i % 20) for i in range(1000)]) + rng.integers(0, 2, size=1000)
    got = _order(dev, counts)
    assert np.array_equal(np.sort(got), np.arange(len(counts)))
    assert np.array_equal(got, orc.qblock_order(counts))


@pytest.mark.parametrize("mode", ["blocks", "tokens"])
def test_ordered_attention_is_bit_identical(dev, mode):
    print("case ordered attention", mode, flush=True)
    B, H, S, D, qblk = 1, 3, 4096, 128, 64
    q, k, v = (t.to(dev) for t in wl.randn_qkv(B, H, S, D, seed=31))
    cnt = wl.zipf_counts(B, H, S // qblk, s=1.2, lo=1, hi=64, seed=32)
    bi, bc = wl.ragged_block_lists(B, H, S, qblk, 64, cnt, seed=33)
    o1, o2 = torch.empty_like(q), torch.empty_like(q)
    l1 = torch.empty((B, H, S), device=dev)
    l2 = torch.empty((B, H, S), device=dev)
    if mode == "blocks":
        idx, num = bi.to(dev), bc.to(dev)
        fn = capi.sp_attn_blocks
    else:
        tok, n = wl.blocks_to_tokens(bi, bc, S)
        idx, num = tok.to(dev), n.to(dev)
        fn = capi.sp_attn
    order = torch.empty((num.numel(),), dtype=torch.int32, device=dev)
    capi.qblock_order(order, num)
    fn(o1, q, k, v, idx, num, lse=l1, qblk=qblk)
    fn(o2, q, k, v, idx, num, lse=l2, qblk=qblk, order=order)
    torch.cuda.synchronize()
    assert not np.array_equal(order.cpu().numpy(), np.arange(num.numel()))
    assert torch.equal(o1, o2) and torch.equal(l1, l2)
