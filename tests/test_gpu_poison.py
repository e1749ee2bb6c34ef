"""GPU: the NaN-poisoning debug build of the library (libspattn_hip_poison.so, -DSPATTN_POISON_RING)
against the product library, bit for bit.  In that build every ring slot is filled with NaNs
between the barrier that frees it and the copy that refills it: a wave that read a tile after its
slot was released (a wait or a barrier too few, a wrong slot) would produce NaNs or different
bits.  Equal bits on lists long enough to go round the ring several times say that no kernel
reads a freed slot."""
import ctypes

import pytest
import torch

from fgattn_tk_cuda_amd import build as bld, capi, workloads as wl

pytestmark = pytest.mark.gpu


def _poison_lib():
    if not bld.POISON_LIB.exists():
        pytest.fail("%s is missing: build it with `python -m fgattn_tk_cuda_amd.build`" % bld.POISON_LIB)
    lib = ctypes.CDLL(str(bld.POISON_LIB))
    for name, (res, args) in capi._SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


def _st():
    return torch.cuda.current_stream().cuda_stream


@pytest.mark.parametrize("D,qblk,S,kv_len", [(128, 64, 1500, 0), (128, 128, 1100, 0), (64, 64, 2000, 1900), (64, 128, 900, 0)])
def test_list_attention_reads_no_freed_slot(dev, D, qblk, S, kv_len):
    print("case poison lists", D, qblk, S, kv_len, flush=True)
    good, bad = capi.load(), _poison_lib()
    B, H = 1, 3
    q, k, v = (t.to(dev) for t in wl.randn_qkv(B, H, S, D, seed=11))
    nq, nkb = wl.ceil_div(S, qblk), wl.ceil_div(S, 64)
    cnt = wl.zipf_counts(B, H, nq, s=1.1, lo=1, hi=nkb, seed=12)      # short and full lists
    bi, bc = wl.ragged_block_lists(B, H, S, qblk, 64, cnt, seed=13)
    bc[:, :, ::7] = 0                                                  # some q-blocks without a key
    bi, bc = bi.to(dev), bc.to(dev)
    tok, num = (t.to(dev) for t in wl.blocks_to_tokens(bi.cpu(), bc.cpu(), S))
    outs = []
    for lib in (good, bad):
        o1, o2 = torch.full_like(q, float("nan")), torch.full_like(q, float("nan"))
        l1, l2 = (torch.full((B, H, S), float("nan"), device=dev) for _ in range(2))
        assert lib.spattn_sp_attn_blocks(o1.data_ptr(), l1.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), bi.data_ptr(),
                                         bc.data_ptr(), int(bi.shape[3]), qblk, B, H, S, D, kv_len, 0.0, _st()) == 0
        assert lib.spattn_sp_attn(o2.data_ptr(), l2.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), tok.data_ptr(),
                                  num.data_ptr(), int(tok.shape[3]), qblk, B, H, S, D, kv_len, 0.0, _st()) == 0
        torch.cuda.synchronize()
        outs.append((o1, l1, o2, l2))
    assert torch.isfinite(outs[0][0].float()).all() and torch.isfinite(outs[0][2].float()).all()
    for a, b in zip(*outs):
        assert torch.equal(a.view(torch.int32) if a.dtype == torch.float32 else a.view(torch.int16),
                           b.view(torch.int32) if b.dtype == torch.float32 else b.view(torch.int16))
    assert int(bc.max()) > 12    # lists that go round the three K slots several times


@pytest.mark.parametrize("D,S,kv_len", [(128, 1300, 0), (64, 1700, 1601)])
def test_dense_kernels_read_no_freed_slot(dev, D, S, kv_len):
    print("case poison dense", D, S, kv_len, flush=True)
    good, bad = capi.load(), _poison_lib()
    B, H = 1, 2
    q, k, v = (t.to(dev) for t in wl.randn_qkv(B, H, S, D, seed=21))
    Sp = 128 * wl.ceil_div(S, 128)
    outs = []
    for lib in (good, bad):
        o1, o2 = torch.full_like(q, float("nan")), torch.full_like(q, float("nan"))
        lse = torch.full((B, H, S), float("nan"), device=dev)
        mx, dn, mx2, dn2 = (torch.full((B, H, 1, Sp), float("nan"), device=dev) for _ in range(4))
        assert lib.spattn_full_attn(o1.data_ptr(), lse.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), B, H, S, D, kv_len,
                                    0.0, _st()) == 0
        assert lib.spattn_fullattn_maxq_denom(o2.data_ptr(), mx.data_ptr(), dn.data_ptr(), q.data_ptr(), k.data_ptr(),
                                              v.data_ptr(), B, H, S, D, kv_len, 0.0, _st()) == 0
        assert lib.spattn_maxq_denom(mx2.data_ptr(), dn2.data_ptr(), q.data_ptr(), k.data_ptr(), B, H, S, D, kv_len, 0.0,
                                     _st()) == 0
        torch.cuda.synchronize()
        outs.append((o1.view(torch.int16), lse.view(torch.int32), o2.view(torch.int16), mx.view(torch.int32), dn.view(torch.int32),
                     mx2.view(torch.int32), dn2.view(torch.int32)))
    for a, b in zip(*outs):
        assert torch.equal(a, b)
