"""GPU: the entry points recorded into a HIP graph (torch.cuda.graph on the launch stream) and
replayed.  No entry point allocates, clears memory with a memset node or synchronises, so a
cache-refresh step (statistics with block maxima -> lists -> attention) and the steady-state
step are each capturable; every replay - with eager work and synchronisations between them -
must reproduce the eager results bit for bit."""
import os
import subprocess
import sys
import textwrap

import pytest
import torch

from fgattn_tk_cuda_amd import capi, workloads as wl

pytestmark = pytest.mark.gpu


def _buffers(dev, B, H, S, D):
    Sp = 128 * wl.ceil_div(S, 128)
    SB, nb = Sp // 128, Sp // 64
    f = dict(device=dev)
    return dict(
        mx=torch.empty((B, H, 1, Sp), **f), dn=torch.empty((B, H, 1, Sp), **f),
        bmx=torch.empty((B, H, nb, Sp), dtype=torch.bfloat16, **f),
        bi=torch.empty((B, H, SB, nb), dtype=torch.int32, **f), bc=torch.empty((B, H, SB), dtype=torch.int32, **f),
        pk=torch.empty((B, H, SB, Sp // 8), dtype=torch.uint8, **f),
        kvi=torch.empty((B, H, SB, Sp), dtype=torch.int32, **f), kvn=torch.empty((B, H, SB), dtype=torch.int32, **f),
        order=torch.empty((B * H * SB,), dtype=torch.int32, **f),
        o_dense=torch.empty((B, H, S, D), dtype=torch.bfloat16, **f), o_tok=torch.empty((B, H, S, D), dtype=torch.bfloat16, **f),
        o_blk=torch.empty((B, H, S, D), dtype=torch.bfloat16, **f), o_bal=torch.empty((B, H, S, D), dtype=torch.bfloat16, **f),
        lse=torch.empty((B, H, S), **f))


def _poison(buf):
    for t in buf.values():
        if t.dtype in (torch.float32, torch.bfloat16):
            t.fill_(float("nan"))
        else:
            t.fill_(-3 if t.dtype == torch.int32 else 0xA5)


@pytest.mark.parametrize("S,D", [(2000, 64), (1536, 128)])
def test_refresh_and_sparse_steps_replay_from_a_graph(dev, S, D):
    print("case graph replay", S, D, flush=True)
    B, H, tau = 1, 3, 2e-3
    q, k, v = (t.to(dev) for t in wl.clustered_qkv(B, H, S, D, seed=S, sigma=0.8))
    buf = _buffers(dev, B, H, S, D)

    def refresh():
        # dense attention with statistics and block maxima, block lists from the maxima, the per-key votes of the
        # kept blocks as bits, key lists from the bits, the work order of the key lists
        capi.fullattn_maxq_denom_blockmax(buf["o_dense"], buf["mx"], buf["dn"], buf["bmx"], q, k, v)
        capi.blockmax_to_blocklists(buf["bi"], buf["bc"], buf["bmx"], buf["mx"], buf["dn"], tau, S, D, qblk=128)
        capi.booleanmask_packed_blocks(buf["pk"], buf["mx"], buf["dn"], q, k, tau, buf["bi"], buf["bc"], qblk=128)
        capi.packedmask_to_indexmask(buf["kvi"], buf["kvn"], buf["pk"], S)
        capi.qblock_order(buf["order"], buf["kvn"])

    def steps():
        capi.sp_attn(buf["o_tok"], q, k, v, buf["kvi"], buf["kvn"], qblk=128, order=buf["order"], lse=buf["lse"])
        capi.sp_attn_blocks(buf["o_blk"], q, k, v, buf["bi"], buf["bc"], qblk=128)
        capi.sp_attn_blocks_balanced(buf["o_bal"], q, k, v, buf["bi"], buf["bc"], qblk=128)

    _poison(buf)
    refresh()
    steps()
    torch.cuda.synchronize()
    want = {name: t.clone() for name, t in buf.items()}
    assert int(want["bc"].sum()) > 0 and int(want["kvn"].sum()) > 0
    assert torch.isfinite(want["o_tok"].float()).all() and torch.isfinite(want["o_blk"].float()).all()
    assert torch.equal(want["o_blk"].view(torch.int16), want["o_bal"].view(torch.int16))

    side = torch.cuda.Stream()          # default priority
    side.wait_stream(torch.cuda.current_stream())
    g_refresh, g_steps = torch.cuda.CUDAGraph(), torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g_refresh, stream=side):
            refresh()
        with torch.cuda.graph(g_steps, stream=side):
            steps()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    def same(name):
        a, b = buf[name], want[name]
        if a.dtype in (torch.float32, torch.bfloat16):   # bit patterns: NaN pads compare equal to themselves
            a, b = a.view(torch.int32 if a.dtype == torch.float32 else torch.int16), b.view(
                torch.int32 if b.dtype == torch.float32 else torch.int16)
        return torch.equal(a, b)

    for rep in range(3):
        _poison(buf)
        torch.cuda.synchronize()
        g_refresh.replay()
        # eager work between the replays, on the lists the replay has just written
        eager = torch.full_like(buf["o_blk"], float("nan"))
        capi.sp_attn_blocks(eager, q, k, v, buf["bi"], buf["bc"], qblk=128)
        g_steps.replay()
        torch.cuda.synchronize()
        for name in buf:
            assert same(name), "replay %d: %s differs from the eager run" % (rep, name)
        assert torch.equal(eager.view(torch.int16), want["o_blk"].view(torch.int16))


def test_capture_right_after_init_in_a_fresh_process(dev):
    """A process whose first calls on the device are recorded into a graph: after spattn_init() no entry
    point changes a device setting, so the capture needs no eager warm-up of the library."""
    print("case graph capture after init", flush=True)
    code = textwrap.dedent("""
        import torch
        from fgattn_tk_cuda_amd import capi, workloads as wl
        dev = torch.device("cuda:0")
        B, H, S, D, qblk = 1, 2, 1100, 128, 64
        q, k, v = (t.to(dev) for t in wl.randn_qkv(B, H, S, D, seed=5))
        nq = wl.ceil_div(S, qblk)
        cnt = wl.zipf_counts(B, H, nq, s=1.2, lo=1, hi=wl.ceil_div(S, 64), seed=6)
        bi, bc = (t.to(dev) for t in wl.ragged_block_lists(B, H, S, qblk, 64, cnt, seed=7))
        o = torch.full_like(q, float("nan")); o2 = torch.full_like(q, float("nan")); od = torch.full_like(q, float("nan"))
        mx = torch.empty((B, H, 1, 1152), device=dev); dn = torch.empty((B, H, 1, 1152), device=dev)
        capi.init()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        g = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(g, stream=side):
                capi.sp_attn_blocks(o, q, k, v, bi, bc, qblk=qblk)
                capi.sp_attn_blocks_balanced(o2, q, k, v, bi, bc, qblk=qblk)
                capi.fullattn_maxq_denom(od, mx, dn, q, k, v)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        e = torch.full_like(q, float("nan")); ed = torch.full_like(q, float("nan"))
        capi.sp_attn_blocks(e, q, k, v, bi, bc, qblk=qblk)
        capi.fullattn_maxq_denom(ed, mx, dn, q, k, v)
        torch.cuda.synchronize()
        assert torch.isfinite(e.float()).all()
        assert torch.equal(o.view(torch.int16), e.view(torch.int16)) and torch.equal(o2.view(torch.int16), e.view(torch.int16))
        assert torch.equal(od.view(torch.int16), ed.view(torch.int16))
        print("captured-after-init ok")
        """)
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=110,
                       cwd=os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    assert r.returncode == 0 and "captured-after-init ok" in r.stdout, r.stdout[-2000:] + r.stderr[-4000:]


def test_balanced_entry_point_refuses_its_first_use_inside_a_capture(dev):
    """A process that records spattn_sp_attn_blocks_balanced into a graph without spattn_init() before: the
    address of the library's work-order array has not been looked up on the device yet, and the lookup is
    not made inside a capture - the call returns SPATTN_ERR_SCRATCH and launches nothing; after the capture
    has ended and spattn_init() has run, the same call works."""
    print("case balanced first use under capture", flush=True)
    code = textwrap.dedent("""
        import ctypes, torch
        from fgattn_tk_cuda_amd import capi, workloads as wl
        dev = torch.device("cuda:0")
        B, H, S, D, qblk = 1, 2, 640, 64, 64
        q, k, v = (t.to(dev) for t in wl.randn_qkv(B, H, S, D, seed=5))
        cnt = wl.zipf_counts(B, H, S // qblk, s=1.2, lo=1, hi=S // 64, seed=6)
        bi, bc = (t.to(dev) for t in wl.ragged_block_lists(B, H, S, qblk, 64, cnt, seed=7))
        o = torch.full_like(q, float("nan"))
        lib = capi.load()
        def call(stream):
            return lib.spattn_sp_attn_blocks_balanced(o.data_ptr(), None, q.data_ptr(), k.data_ptr(), v.data_ptr(), bi.data_ptr(),
                                                      bc.data_ptr(), int(bi.shape[3]), qblk, B, H, S, D, 0, ctypes.c_float(0.0), stream)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        g = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(g, stream=side):
                rc = call(side.cuda_stream)
                # something to record, so that the capture ends as a valid (if useless) graph
                q2 = q + 0
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        assert rc == -7, rc
        assert bool(torch.isnan(o.float()).all()), "nothing may have been launched"
        assert lib.spattn_init() == 0
        assert call(torch.cuda.current_stream().cuda_stream) == 0
        torch.cuda.synchronize()
        e = torch.full_like(q, float("nan"))
        capi.sp_attn_blocks(e, q, k, v, bi, bc, qblk=qblk)
        torch.cuda.synchronize()
        assert torch.equal(o.view(torch.int16), e.view(torch.int16))
        print("refused-under-capture ok")
        """)
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=110,
                       cwd=os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    assert r.returncode == 0 and "refused-under-capture ok" in r.stdout, r.stdout[-2000:] + r.stderr[-4000:]
