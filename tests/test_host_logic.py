"""Host-side logic that needs no GPU: workload generators, the torch-level mask helpers
and the operator registration."""
import numpy as np
import pytest
import torch

from fgattn_tk_cuda_amd import capi, workloads as wl
from oracle import spattn_oracle as orc


def test_uniform_block_lists():
    B, H, S = 2, 3, 4096
    idx, cnt = wl.uniform_block_lists(B, H, S, 64, 64, 6, seed=1)
    assert idx.shape == (B, H, 64, 6) and idx.dtype == torch.int32 and torch.all(cnt == 6)
    a = idx.numpy()
    assert np.all(np.diff(a, axis=-1) > 0)                                  # sorted, unique
    assert np.all((a == np.arange(64)[None, None, :, None]).any(-1))        # diagonal kept
    idx2, _ = wl.uniform_block_lists(B, H, S, 64, 64, 6, seed=1)
    assert torch.equal(idx, idx2)                                           # seeded
    idx3, _ = wl.uniform_block_lists(1, 1, 1024, 128, 64, 4, seed=2)        # q-block 128: diagonal = block 2i
    assert np.all((idx3.numpy()[0, 0] == 2 * np.arange(8)[:, None]).any(-1))


def test_ragged_and_zipf_lists():
    counts = wl.zipf_counts(1, 2, 32, s=1.2, lo=1, hi=16, seed=3)
    assert counts.min() >= 1 and counts.max() <= 16
    idx, cnt = wl.ragged_block_lists(1, 2, 2048, 64, 64, counts, seed=4)
    assert np.array_equal(cnt.numpy(), counts)
    for h in range(2):
        for i in range(32):
            c = int(cnt[0, h, i])
            row = idx[0, h, i].numpy()
            assert np.all(np.diff(row[:c]) > 0) and i in row[:c] and np.all(row[c:] == -1)


def test_kept_block_flops_headline():
    # 26 of 256 blocks per row, 256 rows per head, 2*32 heads
    assert wl.kept_block_flops(2 * 32 * 256 * 26, 64, 64, 128) == pytest.approx(0.8934e12, rel=1e-3)


def test_infer_qblk():
    assert capi.infer_qblk(16384, 256) == 64 and capi.infer_qblk(16384, 128) == 128
    assert capi.infer_qblk(32760, 256) == 128 and capi.infer_qblk(100, 1) == 128
    with pytest.raises(ValueError):
        capi.infer_qblk(16384, 100)


def test_capi_rejects_host_tensors_without_touching_the_device():
    q = torch.zeros((1, 1, 128, 64), dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        capi.full_attn(torch.zeros_like(q), q, q, q)


def test_capi_rejects_a_work_order_of_the_wrong_size():
    """A work order names every q-block once: one that is shorter (or longer) than the count
    tensor never reaches the device."""
    q = torch.zeros((1, 2, 256, 64), dtype=torch.bfloat16)
    idx = torch.zeros((1, 2, 2, 256), dtype=torch.int32)
    cnt = torch.zeros((1, 2, 2), dtype=torch.int32)
    for bad in (torch.zeros(3, dtype=torch.int32), torch.zeros(5, dtype=torch.int32)):
        with pytest.raises(ValueError, match="order"):
            capi.sp_attn(q, q, q, q, idx, cnt, order=bad)
        with pytest.raises(ValueError, match="order"):
            capi.sp_attn_blocks(q, q, q, q, idx[..., :4].contiguous(), cnt, qblk=128, order=bad)


def test_torch_mask_helpers_match_oracle():
    from fgattn_tk_cuda_amd.spattn import mask_utils as mu

    rng = np.random.default_rng(5)
    mask = (rng.random((2, 2, 3, 256)) < 0.2).astype(np.int32)
    idx, cnt = mu.bitmask_to_indexmask(torch.from_numpy(mask))
    wi, wn = orc.booleanmask_to_indexmask(mask, 256)
    assert np.array_equal(idx.numpy(), wi) and np.array_equal(cnt.numpy(), wn)
    q, k, _ = (t.float() for t in wl.clustered_qkv(1, 2, 300, 64, seed=6, sigma=0.7))
    got = mu.qk_bitmask(q, k, thresh=0.02, blocksz=128).numpy()
    mx, dn = orc.maxq_denom(q.numpy(), k.numpy())
    votes, pmax = orc.booleanmask_128(mx, dn, q.numpy(), k.numpy(), 0.02)
    near = np.abs(pmax - 0.02) <= 1e-3 * 0.02
    assert np.array_equal(got | near, (votes[..., :300] > 0) | near)
    b = torch.from_numpy(rng.random((2, 3, 64)) < 0.5)
    assert torch.equal(mu.unpack(mu.pack(b)), b)
    assert mu.pack(torch.tensor([[True, False, False, False, False, False, False, True]])).item() == 129
    assert np.array_equal(mu.pack(b).numpy(), orc.pack_mask(b.numpy()))
    a = torch.rand(300, 8)
    assert torch.equal(mu.attnmapor(a, 128)[2], a[256:].max(0).values)
    assert torch.equal(mu.attnmapand(a, 128)[0], a[:128].min(0).values)
    assert mu.attnmapbroadcast(torch.rand(2, 4), 128).shape == (256, 4)
    cache = mu.NaiveMaskCache(compute_cache_at=[0, 5])
    assert cache.run_fullattn(5) and not cache.run_fullattn(1)
    cache.update_cache(3, "i", "n")
    assert cache.get_mask_from_cache(3) == ("i", "n")


def test_operator_extension_registers_the_seven_ops():
    import fgattn_tk_cuda_amd.spattn.cuda_attn as ext

    names = ["full_attn", "sp_attn", "all_index_mask", "maxq_denom", "booleanmask_128", "booleanmask_to_indexmask",
             "fullattn_maxq_denom"]
    for n in names:
        assert hasattr(ext, n) and hasattr(torch.ops.cuda_attn, n)
    # Meta kernels let fake tensors trace through the ops (python/extension.cpp:74-79)
    q = torch.zeros((1, 2, 256, 128), dtype=torch.bfloat16, device="meta")
    torch.ops.cuda_attn.full_attn(q, q, q, q)
    idx = torch.zeros((1, 2, 2, 256), dtype=torch.int32, device="meta")
    torch.ops.cuda_attn.sp_attn(q, q, q, q, idx, idx)
    schema = str(torch.ops.cuda_attn.sp_attn.default._schema)
    assert "Tensor(a!) o" in schema and "kv_num_indices" in schema
    # the seven reference schemas, character for character (python/extension.cpp:82,113,166,215,259,309,349)
    ref = {
        "full_attn": "cuda_attn::full_attn(Tensor(a!) o, Tensor q, Tensor k, Tensor v) -> ()",
        "all_index_mask": "cuda_attn::all_index_mask(Tensor(a!) kv_indices, Tensor(b!) kv_num_indices, int batch, int heads, int seqblocks, int seq) -> ()",
        "sp_attn": "cuda_attn::sp_attn(Tensor(a!) o, Tensor q, Tensor k, Tensor v, Tensor kv_indices, Tensor kv_num_indices) -> ()",
        "fullattn_maxq_denom": "cuda_attn::fullattn_maxq_denom(Tensor(a!) o, Tensor(b!) o_max_q, Tensor(c!) o_denom, Tensor q, Tensor k, Tensor v) -> ()",
        "maxq_denom": "cuda_attn::maxq_denom(Tensor(a!) o_max_q, Tensor(b!) o_denom, Tensor q, Tensor k) -> ()",
        "booleanmask_128": "cuda_attn::booleanmask_128(Tensor(a!) booleanmask, Tensor o_max_q, Tensor o_denom, Tensor q, Tensor k, float threshold) -> ()",
        "booleanmask_to_indexmask": "cuda_attn::booleanmask_to_indexmask(Tensor(a!) kv_indices, Tensor(b!) kv_numindices, Tensor booleanmask, int seq) -> ()",
    }
    for n, want in ref.items():
        assert str(getattr(torch.ops.cuda_attn, n).default._schema) == want


def test_extended_operators_are_registered_with_meta_kernels():
    import fgattn_tk_cuda_amd.spattn.cuda_attn as ext

    names = ["full_attn_ex", "sp_attn_ex", "sp_attn_block", "fullattn_maxq_denom_ex", "maxq_denom_ex", "booleanmask_128_ex",
             "booleanmask_packed", "packedmask_to_blocklists", "booleanmask_to_blocklists", "qblock_order"]
    for n in names:
        assert hasattr(ext, n) and hasattr(torch.ops.cuda_attn, n)
    q = torch.zeros((1, 2, 256, 128), dtype=torch.bfloat16, device="meta")
    i4 = torch.zeros((1, 2, 4, 8), dtype=torch.int32, device="meta")
    i3 = torch.zeros((1, 2, 4), dtype=torch.int32, device="meta")
    lse = torch.zeros((1, 2, 256), device="meta")
    torch.ops.cuda_attn.sp_attn_block(q, lse, q, q, q, i4, i3, None, 64, 0.0, 0)
    torch.ops.cuda_attn.sp_attn_block(q, None, q, q, q, i4, i3, i3.reshape(-1), 64, 0.0, 0)
    torch.ops.cuda_attn.full_attn_ex(q, None, q, q, q, 0.0, 100)
    pk = torch.zeros((1, 2, 4, 32), dtype=torch.uint8, device="meta")
    torch.ops.cuda_attn.packedmask_to_blocklists(i4, i3, None, pk, 256)
    assert "Tensor(b!)? lse" in str(torch.ops.cuda_attn.sp_attn_block.default._schema)


def test_topk_mask_definition_takes_the_reference_signature():
    """(q, k, select_k, B, H, S, D, BLOCKSZ) as the reference defines it, or blocksz= alone as its
    caller passes it; computed in the dtype of q."""
    from fgattn_tk_cuda_amd.spattn import mask_utils as mu

    q, k, _ = wl.randn_qkv(1, 2, 300, 64, seed=3)
    a_idx, a_num = mu.qk_topkmask_indices(q, k, 40, 1, 2, 300, 64, 128)
    b_idx, b_num = mu.qk_topkmask_indices(q, k, 40, blocksz=128)
    assert torch.equal(a_idx, b_idx) and torch.equal(a_num, b_num)
    assert a_idx.shape == (1, 2, 3, 40) and a_idx.dtype == torch.int32 and int(a_num[0, 0, 0]) == 40
    qm, sc = orc.qblock_mean_scores(q.float().numpy(), k.float().numpy(), 128)
    want = orc.topk_select(sc, 40)
    got = np.sort(a_idx.numpy(), axis=-1)
    # same keys wherever the 40th and 41st scores differ (ties may go either way in torch.topk)
    srt = np.sort(sc, axis=-1)
    clear = srt[..., -40] != srt[..., -41]
    assert clear.any() and np.array_equal(got[clear], want[clear])


def test_one_sweep_route_is_taken_only_within_the_byte_budget():
    """The refresh step of the cached functionals takes the one-sweep route when the block-maxima
    buffer (2 * Sp * Sp / 64 bytes per head) fits the budget, else the reference's two sweeps;
    onepass=True / False overrides.  Footprints at the shapes the reference compiles."""
    import torch

    from fgattn_tk_cuda_amd.spattn import mask_utils as mu

    def q_of(B, H, S, D=128):
        return torch.empty((B, H, S, D), dtype=torch.bfloat16, device="meta")

    assert mu.blockmax_bytes(q_of(1, 24, 32760, 64)) == 2 * 24 * 512 * 32768 == 805306368
    assert mu.blockmax_bytes(q_of(1, 12, 32768)) == 402653184
    assert mu.blockmax_bytes(q_of(1, 40, 32760)) == 1342177280
    assert mu.blockmax_bytes(q_of(1, 12, 75600)) == 2 * 12 * 1182 * 75648
    assert mu.blockmax_bytes(q_of(1, 24, 75856)) == 2 * 24 * 1186 * 75904 > 4e9
    assert mu.blockmax_bytes(q_of(1, 40, 75600)) == 2 * 40 * 1182 * 75648 > 7e9
    assert mu.BLOCKMAX_BUDGET_BYTES == 2 << 30
    # default budget: cfg 4 and the 32K shapes take one sweep, the 75K shapes with 24 or 40 heads two
    assert mu.use_onepass(q_of(1, 24, 32760, 64)) and mu.use_onepass(q_of(1, 40, 32760)) and mu.use_onepass(q_of(1, 12, 75600))
    assert not mu.use_onepass(q_of(1, 24, 75856)) and not mu.use_onepass(q_of(1, 40, 75600))
    # explicit choices and budgets
    assert mu.use_onepass(q_of(1, 40, 75600), True) and not mu.use_onepass(q_of(1, 12, 32768), False)
    assert mu.use_onepass(q_of(1, 40, 75600), None, 8 << 30) and not mu.use_onepass(q_of(1, 12, 32768), None, 1 << 20)
    assert mu.use_onepass(q_of(1, 12, 32768), None, 402653184) and not mu.use_onepass(q_of(1, 12, 32768), None, 402653183)


def test_compressed_list_cache_refuses_ids_that_do_not_fit():
    """Lists narrower than the sequence (top-k lists): without the sequence length an id beyond the
    list width is an error instead of a silently dropped key; with it the bits cover the sequence."""
    import torch

    from fgattn_tk_cuda_amd.spattn import mask_utils as mu

    kvi = torch.full((1, 1, 2, 128), 128, dtype=torch.int32)
    kvn = torch.tensor([[[3, 2]]], dtype=torch.int32)
    kvi[0, 0, 0, :3] = torch.tensor([5, 130, 400])
    kvi[0, 0, 1, :2] = torch.tensor([0, 511])
    cache = mu.CompressMaskCache([0])
    with pytest.raises(ValueError):
        cache.update_cache(0, kvi, kvn)
    cache.update_cache(0, kvi, kvn, seq_len=500)
    packed, width, counts = cache.cache[0]
    assert width == 512 and packed.shape == (1, 1, 2, 64) and counts is kvn
    bits = mu.unpack(packed)
    assert bits.shape[-1] == 512
    assert torch.nonzero(bits[0, 0, 0]).view(-1).tolist() == [5, 130, 400]
    assert torch.nonzero(bits[0, 0, 1]).view(-1).tolist() == [0, 511]
