"""GPU: the entry points recorded into a HIP graph (torch.cuda.graph on the launch stream) and
replayed.  No entry point allocates, clears memory with a memset node or synchronises, so a
cache-refresh step (statistics with block maxima -> lists -> attention) and the steady-state
step are each capturable; every replay - with eager work and synchronisations between them -
must reproduce the eager results bit for bit."""
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
        bmx=torch.empty((B, H, nb, Sp), **f),
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
