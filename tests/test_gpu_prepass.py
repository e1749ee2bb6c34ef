"""GPU parity of the threshold pre-pass (statistics -> vote mask -> index lists)."""
import numpy as np
import pytest
import torch

from fgattn_tk_cuda_amd import capi, workloads as wl
from oracle import spattn_oracle as orc
from helpers import f32, to_dev

pytestmark = pytest.mark.gpu

BAND = 1e-2   # relative band around the threshold inside which a vote may flip


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("S,kv_len", [(512, 0), (1000, 0), (1000, 870)])
def test_booleanmask_votes(dev, D, S, kv_len):
    print("case booleanmask", D, S, kv_len, flush=True)
    B, H = 1, 3
    q, k, v = wl.clustered_qkv(B, H, S, D, seed=41, sigma=0.7)
    qd, kd = to_dev(dev, q, k)
    kv = kv_len or S
    Sp = orc.padded_len(S)
    SB = Sp // 128
    mx = torch.empty((B, H, 1, Sp), device=dev)
    dn = torch.empty((B, H, 1, Sp), device=dev)
    capi.maxq_denom(mx, dn, qd, kd, kv_len=kv_len)
    # threshold at the 70th percentile of the per-(q-block, key) peak probability
    _, pmax0 = orc.booleanmask_128(f32(mx), f32(dn), f32(q), f32(k), 1.0, kv_len=kv)
    thr = float(np.quantile(pmax0, 0.7))
    mask = torch.full((B, H, SB, Sp), -7, dtype=torch.int32, device=dev)
    capi.booleanmask_128(mask, mx, dn, qd, kd, thr, kv_len=kv_len)
    got = mask.cpu().numpy()
    votes, pmax = orc.booleanmask_128(f32(mx), f32(dn), f32(q), f32(k), thr, kv_len=kv)
    assert got.min() >= 0 and got.max() <= 8
    assert np.all(got[..., kv:] == 0)
    near = np.abs(pmax - thr) <= BAND * thr
    # outside the band the >0 masks must agree exactly
    dis = ((got[..., :kv] > 0) != (votes[..., :kv] > 0)) & ~near
    assert dis.sum() == 0, "%d mask mismatches outside the threshold band" % dis.sum()
    # vote counts agree wherever no group sits in the band: check the bulk
    frac_equal = (got[..., :kv] == votes[..., :kv]).mean()
    assert frac_equal > 0.999, frac_equal
    kept = (votes[..., :kv] > 0).mean()
    assert 0.01 < kept < 0.9, kept


@pytest.mark.parametrize("SB,ms,seq", [(3, 384, 300), (2, 2176, 2100), (5, 128, 128), (1, 4096, 1)])
@pytest.mark.parametrize("density", [0.0, 0.08, 1.0])
def test_compaction_bit_exact(dev, SB, ms, seq, density):
    print("case compaction", SB, ms, seq, density, flush=True)
    B, H = 2, 3
    rng = np.random.default_rng(50)
    mask = (rng.random((B, H, SB, ms)) < density).astype(np.int32) * rng.integers(1, 9, size=(B, H, SB, ms), dtype=np.int32)
    md = torch.from_numpy(mask).to(dev)
    kvi = torch.full((B, H, SB, ms), ms, dtype=torch.int32, device=dev)
    kvn = torch.full((B, H, SB), -1, dtype=torch.int32, device=dev)
    capi.booleanmask_to_indexmask(kvi, kvn, md, seq)
    wi, wn = orc.booleanmask_to_indexmask(mask, seq)
    assert np.array_equal(kvn.cpu().numpy(), wn)
    assert np.array_equal(kvi.cpu().numpy(), wi)


@pytest.mark.parametrize("SB,ms,seq,density", [(3, 128, 128, 0.3), (2, 1024, 1000, 0.08), (2, 8192 + 256, 8192 + 200, 0.08),
                                               (1, 16384, 16384, 1.0), (2, 2048, 0, 0.5), (2, 4096, 4096, 0.0),
                                               (1, 32768, 32760, 0.5)])
def test_packed_mask_round_trip_bit_exact(dev, SB, ms, seq, density):
    """pack_mask == numpy.packbits (LSB first); packedmask_to_indexmask == unpack + compaction, bit for bit;
    and on the device the packed path gives exactly what the int32 path gives."""
    print("case packed mask", SB, ms, seq, density, flush=True)
    B, H = 2, 2
    rng = np.random.default_rng(70)
    mask = (rng.random((B, H, SB, ms)) < density).astype(np.int32) * rng.integers(1, 9, size=(B, H, SB, ms), dtype=np.int32)
    md = torch.from_numpy(mask).to(dev)
    packed = torch.full((B, H, SB, ms // 8), 0xA5, dtype=torch.uint8, device=dev)
    capi.pack_mask(packed, md)
    assert np.array_equal(packed.cpu().numpy(), orc.pack_mask(mask))
    kvi = torch.full((B, H, SB, ms), ms, dtype=torch.int32, device=dev)
    kvn = torch.full((B, H, SB), -1, dtype=torch.int32, device=dev)
    capi.packedmask_to_indexmask(kvi, kvn, packed, seq)
    wi, wn = orc.packedmask_to_indexmask(orc.pack_mask(mask), seq)
    assert np.array_equal(kvn.cpu().numpy(), wn)
    assert np.array_equal(kvi.cpu().numpy(), wi)
    kvi2 = torch.full((B, H, SB, ms), ms, dtype=torch.int32, device=dev)
    kvn2 = torch.full((B, H, SB), -1, dtype=torch.int32, device=dev)
    capi.booleanmask_to_indexmask(kvi2, kvn2, md, seq)
    assert torch.equal(kvi, kvi2) and torch.equal(kvn, kvn2)


def _run_mask(rng, shape, density):
    """A 0..8 vote mask whose kept keys come in runs (what a threshold mask looks like)."""
    B, H, SB, ms = shape
    coarse = rng.random((B, H, SB, ms // 16)) < density
    fine = rng.random((B, H, SB, ms)) < 0.7
    keep = np.repeat(coarse, 16, axis=-1) & fine
    return keep.astype(np.int32) * rng.integers(1, 9, size=shape, dtype=np.int32)


def test_compaction_more_rows_than_one_round_of_the_grid(dev):
    """5120 mask rows: the compaction kernel's persistent waves (1024 workgroups x 4 rows) take
    a second row each; every list, count and fill value bit for bit."""
    print("case compaction many rows", flush=True)
    B, H, SB, ms, seq = 1, 40, 128, 256, 250
    rng = np.random.default_rng(81)
    mask = _run_mask(rng, (B, H, SB, ms), 0.12)
    mask[0, 3, 5] = 0                      # an empty row
    mask[0, 39, 127] = 1                   # a full row, the last one
    md = torch.from_numpy(mask).to(dev)
    kvi = torch.full((B, H, SB, ms), ms, dtype=torch.int32, device=dev)
    kvn = torch.full((B, H, SB), -1, dtype=torch.int32, device=dev)
    capi.booleanmask_to_indexmask(kvi, kvn, md, seq)
    wi, wn = orc.booleanmask_to_indexmask(mask, seq)
    assert np.array_equal(kvn.cpu().numpy(), wn)
    assert np.array_equal(kvi.cpu().numpy(), wi)
    assert wn[0, 3, 5] == 0 and wn[0, 39, 127] == seq


def test_bit_kernels_more_rows_than_one_round_of_the_grid(dev):
    """8960 mask rows: pack_mask and packedmask_to_indexmask both walk more than 8192 rows."""
    print("case bit kernels many rows", flush=True)
    B, H, SB, ms, seq = 1, 70, 128, 256, 256
    rng = np.random.default_rng(82)
    mask = _run_mask(rng, (B, H, SB, ms), 0.1)
    mask[0, 69, 127] = 2
    md = torch.from_numpy(mask).to(dev)
    packed = torch.full((B, H, SB, ms // 8), 0x5A, dtype=torch.uint8, device=dev)
    capi.pack_mask(packed, md)
    assert np.array_equal(packed.cpu().numpy(), orc.pack_mask(mask))
    kvi = torch.full((B, H, SB, ms), ms, dtype=torch.int32, device=dev)
    kvn = torch.full((B, H, SB), -1, dtype=torch.int32, device=dev)
    capi.packedmask_to_indexmask(kvi, kvn, packed, seq)
    wi, wn = orc.booleanmask_to_indexmask(mask, seq)
    assert np.array_equal(kvn.cpu().numpy(), wn)
    assert np.array_equal(kvi.cpu().numpy(), wi)


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("S,kv_len", [(512, 0), (1000, 0), (1000, 870), (200, 0), (1090, 1000)])
def test_booleanmask_packed_bits(dev, D, S, kv_len):
    """The sweep with bit outputs.  128-row q-blocks: bit for bit the packed form of the int32 vote
    mask of the same sweep.  64-row q-blocks: the two halves OR to the 128-row bits exactly, and
    each half agrees with the oracle outside the threshold band.  Every word is written."""
    print("case booleanmask packed", D, S, kv_len, flush=True)
    B, H = 1, 3
    q, k, v = wl.clustered_qkv(B, H, S, D, seed=43, sigma=0.7)
    qd, kd = to_dev(dev, q, k)
    kv = kv_len or S
    Sp = orc.padded_len(S)
    SB, n64 = Sp // 128, orc.ceil_div(S, 64)
    mx = torch.empty((B, H, 1, Sp), device=dev)
    dn = torch.empty((B, H, 1, Sp), device=dev)
    capi.maxq_denom(mx, dn, qd, kd, kv_len=kv_len)
    m64, p64 = orc.booleanmask_rows(f32(mx), f32(dn), f32(q), f32(k), 1.0, qblk=64, kv_len=kv)
    thr = float(np.quantile(p64, 0.75))
    mask = torch.full((B, H, SB, Sp), -7, dtype=torch.int32, device=dev)
    capi.booleanmask_128(mask, mx, dn, qd, kd, thr, kv_len=kv_len)
    want128 = orc.pack_mask(mask.cpu().numpy())
    p128 = torch.full((B, H, SB, Sp // 8), 0xA5, dtype=torch.uint8, device=dev)
    capi.booleanmask_packed(p128, mx, dn, qd, kd, thr, qblk=128, kv_len=kv_len)
    assert np.array_equal(p128.cpu().numpy(), want128)
    pk64 = torch.full((B, H, n64, Sp // 8), 0xA5, dtype=torch.uint8, device=dev)
    capi.booleanmask_packed(pk64, mx, dn, qd, kd, thr, qblk=64, kv_len=kv_len)
    g64 = pk64.cpu().numpy()
    both = np.zeros((B, H, 2 * SB, Sp // 8), np.uint8)
    both[:, :, :n64] = g64
    assert np.array_equal(both[:, :, 0::2] | both[:, :, 1::2], want128)
    bits = orc.unpack_mask(g64)
    assert not bits[..., kv:].any()
    m64 = p64 > np.float32(thr)
    near = np.abs(p64 - thr) <= BAND * thr
    dis = (bits[..., :kv] != m64) & ~near
    assert dis.sum() == 0, "%d mismatches outside the threshold band" % dis.sum()
    assert 0.01 < m64.mean() < 0.9


@pytest.mark.parametrize("SB,ms,seq,max_blocks,density", [
    (3, 384, 300, 6, 0.1), (2, 2176, 2100, 34, 0.05), (5, 128, 128, 2, 0.5), (1, 4096, 1, 64, 1.0),
    (2, 8192 + 256, 8192 + 200, 40, 0.08), (2, 1024, 0, 16, 0.5), (3, 4096, 4000, 64, 0.0), (2, 32768, 32760, 512, 0.02),
    (1, 4096, 4096, 5, 0.3)])
def test_block_lists_bit_exact(dev, SB, ms, seq, max_blocks, density):
    """Key mask -> block mask -> ascending block lists, from the bit-packed mask and from the int32
    votes: ids, counts, fill and the block mask bit for bit (incl. a list longer than max_blocks)."""
    print("case block lists", SB, ms, seq, max_blocks, density, flush=True)
    B, H = 2, 2
    rng = np.random.default_rng(90)
    mask = _run_mask(rng, (B, H, SB, ms), density) if density < 1.0 else np.ones((B, H, SB, ms), np.int32)
    wi, wn, wbm = orc.block_lists_from_mask(mask, seq, max_blocks=max_blocks, fill=-3)
    md = torch.from_numpy(mask).to(dev)
    pk = torch.from_numpy(orc.pack_mask(mask)).to(dev)
    for src in ("packed", "votes"):
        bi = torch.full((B, H, SB, max_blocks), -3, dtype=torch.int32, device=dev)
        bc = torch.full((B, H, SB), -1, dtype=torch.int32, device=dev)
        bm = torch.full((B, H, SB, ms // 64), 7, dtype=torch.uint8, device=dev)
        if src == "packed":
            capi.packedmask_to_blocklists(bi, bc, pk, seq, blockmask=bm)
        else:
            capi.booleanmask_to_blocklists(bi, bc, md, seq, blockmask=bm)
        assert np.array_equal(bc.cpu().numpy(), wn), src
        assert np.array_equal(bi.cpu().numpy(), wi), src
        assert np.array_equal(bm.cpu().numpy(), wbm.astype(np.uint8)), src
        bi2 = torch.full((B, H, SB, max_blocks), -3, dtype=torch.int32, device=dev)
        bc2 = torch.full((B, H, SB), -1, dtype=torch.int32, device=dev)
        (capi.packedmask_to_blocklists if src == "packed" else capi.booleanmask_to_blocklists)(
            bi2, bc2, pk if src == "packed" else md, seq)          # without the block mask output
        assert torch.equal(bi, bi2) and torch.equal(bc, bc2)


def test_block_lists_more_rows_than_one_round_of_the_grid(dev):
    """8960 rows: both block-list kernels walk more rows than their grid holds waves."""
    print("case block lists many rows", flush=True)
    B, H, SB, ms, seq = 1, 70, 128, 256, 250
    rng = np.random.default_rng(91)
    mask = _run_mask(rng, (B, H, SB, ms), 0.1)
    mask[0, 69, 127] = 2
    wi, wn, _ = orc.block_lists_from_mask(mask, seq, fill=-1)
    md = torch.from_numpy(mask).to(dev)
    pk = torch.from_numpy(orc.pack_mask(mask)).to(dev)
    for fn, src in ((capi.packedmask_to_blocklists, pk), (capi.booleanmask_to_blocklists, md)):
        bi = torch.full((B, H, SB, ms // 64), -1, dtype=torch.int32, device=dev)
        bc = torch.full((B, H, SB), -1, dtype=torch.int32, device=dev)
        fn(bi, bc, src, seq)
        assert np.array_equal(bc.cpu().numpy(), wn) and np.array_equal(bi.cpu().numpy(), wi)


@pytest.mark.parametrize("qblk", [64, 128])
@pytest.mark.parametrize("D,S", [(64, 1000), (128, 700)])
def test_block_threshold_pipeline_feeds_block_attention(dev, qblk, D, S):
    """maxq_denom -> bit-packed sweep -> block lists -> sp_attn_blocks: the block lists are those of
    the device's own bits (exact), and the attention over them matches the oracle over the
    expanded token lists."""
    print("case block pipeline", qblk, D, S, flush=True)
    B, H = 1, 2
    q, k, v = wl.clustered_qkv(B, H, S, D, seed=63, sigma=0.7)
    qd, kd, vd = to_dev(dev, q, k, v)
    Sp = orc.padded_len(S)
    nq = orc.ceil_div(S, qblk)
    mx = torch.empty((B, H, 1, Sp), device=dev)
    dn = torch.empty((B, H, 1, Sp), device=dev)
    capi.maxq_denom(mx, dn, qd, kd)
    pk = torch.empty((B, H, nq, Sp // 8), dtype=torch.uint8, device=dev)
    capi.booleanmask_packed(pk, mx, dn, qd, kd, 0.03, qblk=qblk)
    nb = Sp // 64
    bi = torch.full((B, H, nq, nb), -1, dtype=torch.int32, device=dev)
    bc = torch.zeros((B, H, nq), dtype=torch.int32, device=dev)
    capi.packedmask_to_blocklists(bi, bc, pk, S)
    wi, wn, _ = orc.block_lists_from_mask(orc.unpack_mask(pk.cpu().numpy()), S, fill=-1)
    assert np.array_equal(bi.cpu().numpy(), wi) and np.array_equal(bc.cpu().numpy(), wn)
    assert 0 < wn.mean() < nb
    o = torch.full_like(qd, float("nan"))
    lse = torch.empty((B, H, S), device=dev)
    capi.sp_attn_blocks(o, qd, kd, vd, bi, bc, lse=lse, qblk=qblk)
    tok, num = orc.block_list_to_token_list(wi, wn, S)
    want, wlse = orc.sp_attn(f32(q), f32(k), f32(v), tok, num, qblk=qblk)
    from helpers import assert_close_o, assert_close_stat
    assert_close_o(f32(o), want, "block pipeline O")
    assert_close_stat(f32(lse), wlse, "block pipeline lse")


@pytest.mark.parametrize("with_v", [False, True])
@pytest.mark.parametrize("D,S,kv_len", [(64, 1000, 0), (128, 700, 0), (64, 520, 450), (128, 64, 0), (64, 130, 1)])
def test_block_maxima_of_the_statistics_sweeps(dev, D, S, kv_len, with_v):
    """The statistics sweeps with the blockmax output: max_q / denom (and O) are bit for bit those of
    the plain sweeps, blockmax[J][r] is the oracle's per-block row maximum rounded up to bf16 (never
    below it, less than one bf16 step above), and its maximum over the blocks is max_q rounded up."""
    print("case blockmax sweep", D, S, kv_len, with_v, flush=True)
    B, H = 1, 3
    q, k, v = wl.clustered_qkv(B, H, S, D, seed=71, sigma=0.7)
    qd, kd, vd = to_dev(dev, q, k, v)
    kv = kv_len or S
    Sp = orc.padded_len(S)
    nb, nkb = Sp // 64, orc.ceil_div(kv, 64)
    mx, dn, mx2, dn2 = (torch.full((B, H, 1, Sp), 7.0, device=dev) for _ in range(4))
    bmx = torch.full((B, H, nb, Sp), 123.0, dtype=torch.bfloat16, device=dev)
    if with_v:
        o, o2 = torch.full_like(qd, float("nan")), torch.full_like(qd, float("nan"))
        capi.fullattn_maxq_denom(o, mx, dn, qd, kd, vd, kv_len=kv_len)
        capi.fullattn_maxq_denom_blockmax(o2, mx2, dn2, bmx, qd, kd, vd, kv_len=kv_len)
        assert torch.equal(o.view(torch.int16), o2.view(torch.int16))
    else:
        capi.maxq_denom(mx, dn, qd, kd, kv_len=kv_len)
        capi.maxq_denom_blockmax(mx2, dn2, bmx, qd, kd, kv_len=kv_len)
    assert torch.equal(mx, mx2) and torch.equal(dn, dn2)
    got = f32(bmx)
    want = orc.block_row_max(f32(q), f32(k), kv_len=kv)
    assert np.all(got[:, :, nkb:] == 123.0), "blocks without a key are not written"
    g, w = got[:, :, :nkb, :S], want[:, :, :nkb, :S]
    assert np.isfinite(g).all() and np.isfinite(w).all()
    tol = 1e-3 + 1e-4 * np.abs(w)        # the device's fp32 maximum against the oracle's
    assert np.all(g >= w - tol), "a stored maximum lies below the oracle's: %g" % (w - g).max()
    assert np.all(g <= w + tol + 2.0 ** -7 * np.abs(w)), "a stored maximum is more than one bf16 step above the oracle's"
    # rounding up is monotone: the largest stored maximum of a row is its max_q rounded up, exactly
    assert np.array_equal(g.max(axis=2), orc.bf16_round_up(f32(mx).reshape(B, H, Sp)[..., :S]))


@pytest.mark.parametrize("qblk", [64, 128])
@pytest.mark.parametrize("D,S,kv_len", [(64, 1000, 0), (128, 700, 0), (64, 520, 450), (64, 130, 1)])
def test_block_lists_from_block_maxima(dev, qblk, D, S, kv_len):
    """blockmax_to_blocklists: lists, counts and block mask are exactly the threshold of the device's
    own block maxima and statistics (outside a thin band where the device's log2 may round the
    other way).  Against the block mask of the per-key oracle and of the bit-packed sweep they are
    a superset - the stored maxima are rounded up - that is equal outside the threshold band widened
    downwards by one bf16 step of the largest score."""
    print("case blockmax lists", qblk, D, S, kv_len, flush=True)
    B, H = 1, 3
    q, k, v = wl.clustered_qkv(B, H, S, D, seed=73, sigma=0.7)
    qd, kd = to_dev(dev, q, k)
    kv = kv_len or S
    Sp = orc.padded_len(S)
    nb, nkb, nq = Sp // 64, orc.ceil_div(kv, 64), orc.ceil_div(S, qblk)
    mx = torch.empty((B, H, 1, Sp), device=dev)
    dn = torch.empty((B, H, 1, Sp), device=dev)
    bmx = torch.full((B, H, nb, Sp), float("nan"), dtype=torch.bfloat16, device=dev)
    capi.maxq_denom_blockmax(mx, dn, bmx, qd, kd, kv_len=kv_len)
    _, pmax = orc.booleanmask_rows(f32(mx), f32(dn), f32(q), f32(k), 1.0, qblk=qblk, kv_len=kv)
    pblk = np.full((B, H, nq, nb), -np.inf, np.float32)
    for J in range(nkb):
        pblk[..., J] = pmax[..., 64 * J: min(64 * J + 64, kv)].max(axis=-1)
    # about 40 % of the blocks pass; with one or two blocks per row, a threshold every row passes
    thr = float(np.quantile(pblk[..., :nkb], 0.6)) if nkb > 2 else 0.5 * float(pblk[..., :nkb].min())
    bi = torch.full((B, H, nq, nb), -1, dtype=torch.int32, device=dev)
    bc = torch.full((B, H, nq), -9, dtype=torch.int32, device=dev)
    bm = torch.full((B, H, nq, nb), 7, dtype=torch.uint8, device=dev)
    capi.blockmax_to_blocklists(bi, bc, bmx, mx, dn, thr, S, D, qblk=qblk, blockmask=bm, kv_len=kv_len)
    got_bm = bm.cpu().numpy().astype(bool)
    assert set(np.unique(bm.cpu().numpy())) <= {0, 1} and not got_bm[..., nkb:].any()
    # the lists are the block mask, ascending, exact counts, fill behind them
    wi, wn = orc.block_lists_from_blockmask(got_bm, fill=-1)
    assert np.array_equal(bi.cpu().numpy(), wi) and np.array_equal(bc.cpu().numpy(), wn)
    # the block mask is the threshold of the device's block maxima
    dev_bmx = np.nan_to_num(f32(bmx), nan=-np.inf)
    want_bm, margin = orc.block_mask_from_blockmax(dev_bmx, f32(mx), f32(dn), thr, S, D, qblk=qblk, kv_len=kv)
    near = np.abs(margin) <= 1e-4
    assert np.array_equal(got_bm | near, want_bm | near) and near.mean() < 0.01
    # ... and a superset of the block mask of the per-key threshold mask that equals it outside the
    # band: rounding a maximum up by at most 2^-7 |s| raises its softmax value by at most `lift`
    sf = orc.LOG2E / np.sqrt(D)
    lift = float(np.exp2(2.0 ** -7 * np.abs(dev_bmx[np.isfinite(dev_bmx)]).max() * sf))
    assert 1.0 < lift < 1.2
    exact_bm = pblk > np.float32(thr)
    assert not (exact_bm & ~got_bm & (pblk > thr * (1 + BAND))).any(), "a block of the exact mask is missing"
    assert not (got_bm & (pblk < thr * (1 - BAND) / lift)).any(), "a block far below the threshold is listed"
    band = (pblk >= thr * (1 - BAND) / lift) & (pblk <= thr * (1 + BAND))
    assert np.array_equal(got_bm | band, exact_bm | band)
    if nkb > 2:
        assert 0.1 < got_bm[..., :nkb].mean() < 0.9
    # the bit-packed sweep -> block lists route gives the same blocks where the oracle is clear
    pk = torch.empty((B, H, nq, Sp // 8), dtype=torch.uint8, device=dev)
    capi.booleanmask_packed(pk, mx, dn, qd, kd, thr, qblk=qblk, kv_len=kv_len)
    bi2 = torch.full((B, H, nq, nb), -1, dtype=torch.int32, device=dev)
    bc2 = torch.zeros((B, H, nq), dtype=torch.int32, device=dev)
    bm2 = torch.zeros((B, H, nq, nb), dtype=torch.uint8, device=dev)
    capi.packedmask_to_blocklists(bi2, bc2, pk, kv, blockmask=bm2)
    assert np.array_equal(got_bm | band, bm2.cpu().numpy().astype(bool) | band)
    # a list cut off at max_blocks keeps the first ids and the full count
    bi3 = torch.full((B, H, nq, 2), -1, dtype=torch.int32, device=dev)
    bc3 = torch.zeros((B, H, nq), dtype=torch.int32, device=dev)
    capi.blockmax_to_blocklists(bi3, bc3, bmx, mx, dn, thr, S, D, qblk=qblk, kv_len=kv_len)
    assert torch.equal(bc3, bc) and torch.equal(bi3, bi[..., :2])


@pytest.mark.parametrize("D,S,kv_len", [(64, 1000, 0), (128, 700, 0), (64, 520, 450), (128, 300, 130), (64, 130, 1)])
def test_threshold_sweep_restricted_to_block_lists(dev, D, S, kv_len):
    """The sweep over the listed key blocks only.  With every block listed it is the full sweep bit
    for bit (votes, and both bit forms); with the lists that the threshold of the block maxima
    gives, the mask differs from the full sweep at most where a block's best score lies within
    rounding of its row's threshold; a block left out of a list is zero in the output; garbage in
    the buffers beforehand does not show."""
    print("case sparse sweep", D, S, kv_len, flush=True)
    B, H = 1, 3
    q, k, v = wl.clustered_qkv(B, H, S, D, seed=91, sigma=0.7)
    qd, kd = to_dev(dev, q, k)
    kv = kv_len or S
    Sp = orc.padded_len(S)
    SB, nb, nkb, n64 = Sp // 128, Sp // 64, orc.ceil_div(kv, 64), orc.ceil_div(S, 64)
    mx = torch.empty((B, H, 1, Sp), device=dev)
    dn = torch.empty((B, H, 1, Sp), device=dev)
    bmx = torch.full((B, H, nb, Sp), float("nan"), dtype=torch.bfloat16, device=dev)
    capi.maxq_denom_blockmax(mx, dn, bmx, qd, kd, kv_len=kv_len)
    _, pmax = orc.booleanmask_rows(f32(mx), f32(dn), f32(q), f32(k), 1.0, qblk=128, kv_len=kv)
    pblk = np.stack([pmax[..., 64 * J: min(64 * J + 64, kv)].max(axis=-1) for J in range(nkb)], axis=-1)
    thr = float(np.quantile(pblk, 0.6)) if nkb > 2 else 0.5 * float(pblk.min())   # about 40 % of the blocks pass
    full = torch.full((B, H, SB, Sp), -7, dtype=torch.int32, device=dev)
    capi.booleanmask_128(full, mx, dn, qd, kd, thr, kv_len=kv_len)
    # every block listed: the same kernel walk in list order
    allb = torch.arange(nb, dtype=torch.int32, device=dev).expand(B, H, SB, nb).contiguous()
    alln = torch.full((B, H, SB), nb, dtype=torch.int32, device=dev)
    got = torch.full_like(full, 55)
    capi.booleanmask_128_blocks(got, mx, dn, qd, kd, thr, allb, alln, kv_len=kv_len)
    assert torch.equal(got, full)
    for qblk, rows in ((128, SB), (64, n64)):
        pf = torch.full((B, H, rows, Sp // 8), 0xA5, dtype=torch.uint8, device=dev)
        pg = torch.full((B, H, rows, Sp // 8), 0x5A, dtype=torch.uint8, device=dev)
        capi.booleanmask_packed(pf, mx, dn, qd, kd, thr, qblk=qblk, kv_len=kv_len)
        capi.booleanmask_packed_blocks(pg, mx, dn, qd, kd, thr, allb, alln, qblk=qblk, kv_len=kv_len)
        assert torch.equal(pf, pg)
    # the lists of the block maxima: same mask, except in blocks whose best key is within rounding of the threshold
    bi = torch.full((B, H, SB, nb), -1, dtype=torch.int32, device=dev)
    bc = torch.zeros((B, H, SB), dtype=torch.int32, device=dev)
    bm = torch.zeros((B, H, SB, nb), dtype=torch.uint8, device=dev)
    capi.blockmax_to_blocklists(bi, bc, bmx, mx, dn, thr, S, D, qblk=128, blockmask=bm, kv_len=kv_len)
    got = torch.full_like(full, 55)
    capi.booleanmask_128_blocks(got, mx, dn, qd, kd, thr, bi, bc, kv_len=kv_len)
    fm, gm, kept = full.cpu().numpy(), got.cpu().numpy(), bm.cpu().numpy().astype(bool)
    kept_keys = np.repeat(kept, 64, axis=-1)
    assert np.array_equal(gm[kept_keys], fm[kept_keys]), "votes of the listed blocks"
    assert not gm[~kept_keys].any(), "everything else is zero"
    _, margin = orc.block_mask_from_blockmax(np.nan_to_num(f32(bmx), nan=-np.inf), f32(mx), f32(dn), thr, S, D,
                                             qblk=128, kv_len=kv)
    clear = np.repeat(np.abs(margin) > 1e-4, 64, axis=-1)
    assert np.array_equal(gm[clear], fm[clear])
    assert (gm != fm).mean() < 1e-4
    if nkb > 2:
        assert 0.05 < kept[..., :nkb].mean() < 0.95 and fm.any()
    # a shorter list (first half of each) zeroes the blocks that were dropped
    half = torch.clamp(bc // 2, min=0)
    got2 = torch.full_like(full, 55)
    capi.booleanmask_128_blocks(got2, mx, dn, qd, kd, thr, bi, half, kv_len=kv_len)
    g2 = got2.cpu().numpy()
    bih, hh = bi.cpu().numpy(), half.cpu().numpy()
    for h in range(H):
        for i in range(SB):
            want = np.zeros(Sp, np.int32)
            for J in bih[0, h, i, : hh[0, h, i]]:
                want[64 * J: 64 * J + 64] = fm[0, h, i, 64 * J: 64 * J + 64]
            assert np.array_equal(g2[0, h, i], want), (h, i)
    # ids outside the row and counts beyond max_blocks are tolerated
    bad = bi.clone()
    bad[..., 0] = 10 ** 6
    got3 = torch.full_like(full, 55)
    capi.booleanmask_128_blocks(got3, mx, dn, qd, kd, thr, bad, bc + 1000, kv_len=kv_len)
    assert int(got3.min()) >= 0 and int(got3.max()) <= 8


def test_all_index_mask(dev):
    print("case all_index_mask", flush=True)
    B, H, SB, S, ms = 2, 3, 5, 600, 640
    kvi = torch.zeros((B, H, SB, ms), dtype=torch.int32, device=dev)
    kvn = torch.zeros((B, H, SB), dtype=torch.int32, device=dev)
    capi.all_index_mask(kvi, kvn, B, H, SB, S)
    wi, wn = orc.all_index_mask(B, H, SB, S, ms)
    assert np.array_equal(kvi.cpu().numpy(), wi) and np.array_equal(kvn.cpu().numpy(), wn)


def test_threshold_pipeline_feeds_sparse_attention(dev):
    """maxq_denom -> booleanmask_128 -> booleanmask_to_indexmask -> sp_attn on a padded length;
    with a tiny threshold every key is kept and the result is dense attention."""
    print("case pipeline", flush=True)
    B, H, S, D = 1, 2, 1000, 64
    q, k, v = wl.clustered_qkv(B, H, S, D, seed=61, sigma=0.7)
    qd, kd, vd = to_dev(dev, q, k, v)
    Sp = orc.padded_len(S)
    SB = Sp // 128
    mx = torch.empty((B, H, 1, Sp), device=dev)
    dn = torch.empty((B, H, 1, Sp), device=dev)
    capi.maxq_denom(mx, dn, qd, kd)
    for thr, dense in ((1e-30, True), (0.05, False)):
        mask = torch.zeros((B, H, SB, Sp), dtype=torch.int32, device=dev)
        capi.booleanmask_128(mask, mx, dn, qd, kd, thr)
        kvi = torch.full((B, H, SB, Sp), Sp, dtype=torch.int32, device=dev)
        kvn = torch.zeros((B, H, SB), dtype=torch.int32, device=dev)
        capi.booleanmask_to_indexmask(kvi, kvn, mask, S)
        o = torch.full_like(qd, float("nan"))
        capi.sp_attn(o, qd, kd, vd, kvi, kvn)
        if dense:
            assert np.all(kvn.cpu().numpy() == S)
            want = f32(torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float()))
        else:
            want, _ = orc.sp_attn(f32(q), f32(k), f32(v), kvi.cpu().numpy(), kvn.cpu().numpy(), qblk=128)
            assert 0 < kvn.float().mean().item() < S
        from helpers import assert_close_o
        assert_close_o(f32(o), want, "pipeline O (dense=%s)" % dense)
