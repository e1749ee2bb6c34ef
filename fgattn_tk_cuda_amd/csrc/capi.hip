// extern "C" surface of libspattn_hip.so: argument checks, parameter packing, dispatch.
#include "../../include/spattn_hip.h"

#include <math.h>

#include <atomic>
#include <mutex>

#include "dispatch.h"

namespace {

thread_local int g_last_status = SPATTN_OK;

inline int done(int st) {
  g_last_status = st;
  return st;
}
inline int from_hip(hipError_t e) { return done(e == hipSuccess ? SPATTN_OK : (int)e); }
inline bool misaligned(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) != 0; }
inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

int check_qkv(const void* q, const void* k, int B, int H, int S, int D) {
  if (!q || !k) return SPATTN_ERR_NULL;
  if (D != 64 && D != 128) return SPATTN_ERR_HEAD_DIM;
  // tile descriptors carry a row number in 24 bits
  if (B <= 0 || H <= 0 || S <= 0 || S >= (1 << 24)) return SPATTN_ERR_SHAPE;
  if (misaligned(q) || misaligned(k)) return SPATTN_ERR_ALIGN;
  return SPATTN_OK;
}

spattn::AttnParams base_params(const void* q, const void* k, const void* v, void* o, int B, int H, int S, int D,
                               int kv_len, float scale, int qblk) {
  spattn::AttnParams p{};
  p.q = static_cast<const uint16_t*>(q);
  p.k = static_cast<const uint16_t*>(k);
  p.v = static_cast<const uint16_t*>(v);
  p.o = static_cast<uint16_t*>(o);
  p.B = B;
  p.H = H;
  p.S = S;
  p.kv_len = (kv_len <= 0 || kv_len > S) ? S : kv_len;
  p.Sp = ((S + 127) / 128) * 128;
  p.nqblk = (S + qblk - 1) / qblk;
  p.scale = scale > 0.f ? scale : 1.0f / sqrtf((float)D);
  p.sf = spattn::kLog2e * p.scale;
  return p;
}

}  // namespace

extern "C" {

int spattn_full_attn(void* o, float* lse, const void* q, const void* k, const void* v, int B, int H, int S, int D,
                     int kv_len, float scale, void* stream) {
  if (int st = check_qkv(q, k, B, H, S, D)) return done(st);
  if (!o || !v) return done(SPATTN_ERR_NULL);
  if (misaligned(o) || misaligned(v)) return done(SPATTN_ERR_ALIGN);
  spattn::AttnParams p = base_params(q, k, v, o, B, H, S, D, kv_len, scale, 128);
  p.lse = lse;
  return from_hip(spattn::run_attn_dense(p, D, true, false, as_stream(stream)));
}

int spattn_sp_attn(void* o, float* lse, const void* q, const void* k, const void* v, const int* kv_indices,
                   const int* num_kv_indices, int mask_stride, int qblk, int B, int H, int S, int D, int kv_len,
                   float scale, void* stream) {
  if (int st = check_qkv(q, k, B, H, S, D)) return done(st);
  if (!o || !v || !kv_indices || !num_kv_indices) return done(SPATTN_ERR_NULL);
  if (misaligned(o) || misaligned(v) || misaligned(kv_indices)) return done(SPATTN_ERR_ALIGN);
  if (qblk != 64 && qblk != 128) return done(SPATTN_ERR_QBLK);
  // The reference asserts mask_stride % 128 == 0 (include/sparseattn_asyncgatherload_padded.cuh:269).
  if (mask_stride <= 0 || mask_stride % 128 != 0) return done(SPATTN_ERR_STRIDE);
  spattn::AttnParams p = base_params(q, k, v, o, B, H, S, D, kv_len, scale, qblk);
  p.lse = lse;
  p.idx = kv_indices;
  p.cnt = num_kv_indices;
  p.idx_stride = mask_stride;
  return from_hip(spattn::run_attn_tokens(p, D, qblk, as_stream(stream)));
}

int spattn_sp_attn_blocks(void* o, float* lse, const void* q, const void* k, const void* v, const int* blk_indices,
                          const int* blk_counts, int max_blocks, int qblk, int B, int H, int S, int D, int kv_len,
                          float scale, void* stream) {
  if (int st = check_qkv(q, k, B, H, S, D)) return done(st);
  if (!o || !v || !blk_indices || !blk_counts) return done(SPATTN_ERR_NULL);
  if (misaligned(o) || misaligned(v)) return done(SPATTN_ERR_ALIGN);
  if (qblk != 64 && qblk != 128) return done(SPATTN_ERR_QBLK);
  if (max_blocks <= 0) return done(SPATTN_ERR_SHAPE);
  spattn::AttnParams p = base_params(q, k, v, o, B, H, S, D, kv_len, scale, qblk);
  p.lse = lse;
  p.idx = blk_indices;
  p.cnt = blk_counts;
  p.idx_stride = max_blocks;
  return from_hip(spattn::run_attn_blocks(p, D, qblk, as_stream(stream)));
}

int spattn_all_index_mask(int* kv_indices, int* num_kv_indices, int B, int H, int seqblocks, int seq, int mask_stride,
                          void* stream) {
  if (!kv_indices || !num_kv_indices) return done(SPATTN_ERR_NULL);
  if (B <= 0 || H <= 0 || seqblocks <= 0 || seq <= 0) return done(SPATTN_ERR_SHAPE);
  if (mask_stride <= 0 || mask_stride % 128 != 0) return done(SPATTN_ERR_STRIDE);
  if (misaligned(kv_indices)) return done(SPATTN_ERR_ALIGN);
  return from_hip(spattn::run_all_index(kv_indices, num_kv_indices, B * H * seqblocks, mask_stride, seq, as_stream(stream)));
}

int spattn_fullattn_maxq_denom(void* o, float* max_q, float* denom, const void* q, const void* k, const void* v, int B,
                               int H, int S, int D, int kv_len, float scale, void* stream) {
  if (int st = check_qkv(q, k, B, H, S, D)) return done(st);
  if (!o || !v || !max_q || !denom) return done(SPATTN_ERR_NULL);
  if (misaligned(o) || misaligned(v)) return done(SPATTN_ERR_ALIGN);
  spattn::AttnParams p = base_params(q, k, v, o, B, H, S, D, kv_len, scale, 128);
  p.max_q = max_q;
  p.denom = denom;
  return from_hip(spattn::run_attn_dense(p, D, true, true, as_stream(stream)));
}

int spattn_maxq_denom(float* max_q, float* denom, const void* q, const void* k, int B, int H, int S, int D, int kv_len,
                      float scale, void* stream) {
  if (int st = check_qkv(q, k, B, H, S, D)) return done(st);
  if (!max_q || !denom) return done(SPATTN_ERR_NULL);
  spattn::AttnParams p = base_params(q, k, nullptr, nullptr, B, H, S, D, kv_len, scale, 128);
  p.max_q = max_q;
  p.denom = denom;
  return from_hip(spattn::run_attn_dense(p, D, false, true, as_stream(stream)));
}

int spattn_fullattn_maxq_denom_blockmax(void* o, float* max_q, float* denom, void* blockmax, const void* q, const void* k,
                                        const void* v, int B, int H, int S, int D, int kv_len, float scale, void* stream) {
  if (int st = check_qkv(q, k, B, H, S, D)) return done(st);
  if (!o || !v || !max_q || !denom || !blockmax) return done(SPATTN_ERR_NULL);
  if (misaligned(o) || misaligned(v)) return done(SPATTN_ERR_ALIGN);
  spattn::AttnParams p = base_params(q, k, v, o, B, H, S, D, kv_len, scale, 128);
  p.max_q = max_q;
  p.denom = denom;
  p.blockmax = static_cast<uint16_t*>(blockmax);
  return from_hip(spattn::run_attn_dense(p, D, true, true, as_stream(stream)));
}

int spattn_maxq_denom_blockmax(float* max_q, float* denom, void* blockmax, const void* q, const void* k, int B, int H,
                               int S, int D, int kv_len, float scale, void* stream) {
  if (int st = check_qkv(q, k, B, H, S, D)) return done(st);
  if (!max_q || !denom || !blockmax) return done(SPATTN_ERR_NULL);
  spattn::AttnParams p = base_params(q, k, nullptr, nullptr, B, H, S, D, kv_len, scale, 128);
  p.max_q = max_q;
  p.denom = denom;
  p.blockmax = static_cast<uint16_t*>(blockmax);
  return from_hip(spattn::run_attn_dense(p, D, false, true, as_stream(stream)));
}

int spattn_blockmax_to_blocklists(int* blk_indices, int* blk_counts, void* blockmask, const void* blockmax,
                                  const float* max_q, const float* denom, float threshold, int qblk, int B, int H, int S,
                                  int D, int kv_len, float scale, int max_blocks, void* stream) {
  if (!blk_indices || !blk_counts || !blockmax || !max_q || !denom) return done(SPATTN_ERR_NULL);
  if (misaligned(blockmax)) return done(SPATTN_ERR_ALIGN);
  if (D != 64 && D != 128) return done(SPATTN_ERR_HEAD_DIM);
  if (B <= 0 || H <= 0 || S <= 0 || S >= (1 << 24) || max_blocks <= 0) return done(SPATTN_ERR_SHAPE);
  if (qblk != 64 && qblk != 128) return done(SPATTN_ERR_QBLK);
  const int kv = (kv_len <= 0 || kv_len > S) ? S : kv_len;
  const float sc = scale > 0.f ? scale : 1.0f / sqrtf((float)D);
  return from_hip(spattn::run_blockmax_to_blocklists(blk_indices, blk_counts, static_cast<unsigned char*>(blockmask),
                                                     static_cast<const uint16_t*>(blockmax),
                                                     max_q, denom, threshold, spattn::kLog2e * sc, qblk, B * H, S, kv,
                                                     max_blocks, as_stream(stream)));
}

int spattn_booleanmask_128(int* booleanmask, float threshold, int mask_stride, const float* max_q, const float* denom,
                           const void* q, const void* k, int B, int H, int S, int D, int kv_len, float scale,
                           void* stream) {
  if (int st = check_qkv(q, k, B, H, S, D)) return done(st);
  if (!booleanmask || !max_q || !denom) return done(SPATTN_ERR_NULL);
  if (mask_stride <= 0 || mask_stride % 128 != 0) return done(SPATTN_ERR_STRIDE);
  const int kv = (kv_len <= 0 || kv_len > S) ? S : kv_len;
  const float sc = scale > 0.f ? scale : 1.0f / sqrtf((float)D);
  return from_hip(spattn::run_booleanmask(booleanmask, 0, threshold, mask_stride, max_q, denom,
                                          static_cast<const uint16_t*>(q), static_cast<const uint16_t*>(k), B, H, S, D,
                                          kv < mask_stride ? kv : mask_stride, sc, as_stream(stream)));
}

int spattn_booleanmask_packed(void* packed, float threshold, int mask_stride, int qblk, const float* max_q,
                              const float* denom, const void* q, const void* k, int B, int H, int S, int D, int kv_len,
                              float scale, void* stream) {
  if (int st = check_qkv(q, k, B, H, S, D)) return done(st);
  if (!packed || !max_q || !denom) return done(SPATTN_ERR_NULL);
  if (qblk != 64 && qblk != 128) return done(SPATTN_ERR_QBLK);
  if (mask_stride <= 0 || mask_stride % 128 != 0) return done(SPATTN_ERR_STRIDE);
  if (misaligned(packed)) return done(SPATTN_ERR_ALIGN);
  const int kv = (kv_len <= 0 || kv_len > S) ? S : kv_len;
  const float sc = scale > 0.f ? scale : 1.0f / sqrtf((float)D);
  return from_hip(spattn::run_booleanmask(packed, qblk, threshold, mask_stride, max_q, denom,
                                          static_cast<const uint16_t*>(q), static_cast<const uint16_t*>(k), B, H, S, D,
                                          kv < mask_stride ? kv : mask_stride, sc, as_stream(stream)));
}

int spattn_booleanmask_128_blocks(int* booleanmask, float threshold, int mask_stride, const float* max_q, const float* denom,
                                  const void* q, const void* k, const int* blk_indices, const int* blk_counts, int max_blocks,
                                  int B, int H, int S, int D, int kv_len, float scale, void* stream) {
  if (int st = check_qkv(q, k, B, H, S, D)) return done(st);
  if (!booleanmask || !max_q || !denom || !blk_indices || !blk_counts) return done(SPATTN_ERR_NULL);
  if (mask_stride <= 0 || mask_stride % 128 != 0) return done(SPATTN_ERR_STRIDE);
  if (max_blocks <= 0) return done(SPATTN_ERR_SHAPE);
  if (misaligned(booleanmask)) return done(SPATTN_ERR_ALIGN);
  const int kv = (kv_len <= 0 || kv_len > S) ? S : kv_len;
  const float sc = scale > 0.f ? scale : 1.0f / sqrtf((float)D);
  return from_hip(spattn::run_booleanmask(booleanmask, 0, threshold, mask_stride, max_q, denom,
                                          static_cast<const uint16_t*>(q), static_cast<const uint16_t*>(k), B, H, S, D,
                                          kv < mask_stride ? kv : mask_stride, sc, as_stream(stream), blk_indices, blk_counts,
                                          max_blocks));
}

int spattn_booleanmask_packed_blocks(void* packed, float threshold, int mask_stride, int qblk, const float* max_q,
                                     const float* denom, const void* q, const void* k, const int* blk_indices,
                                     const int* blk_counts, int max_blocks, int B, int H, int S, int D, int kv_len,
                                     float scale, void* stream) {
  if (int st = check_qkv(q, k, B, H, S, D)) return done(st);
  if (!packed || !max_q || !denom || !blk_indices || !blk_counts) return done(SPATTN_ERR_NULL);
  if (qblk != 64 && qblk != 128) return done(SPATTN_ERR_QBLK);
  if (mask_stride <= 0 || mask_stride % 128 != 0) return done(SPATTN_ERR_STRIDE);
  if (max_blocks <= 0) return done(SPATTN_ERR_SHAPE);
  if (misaligned(packed)) return done(SPATTN_ERR_ALIGN);
  const int kv = (kv_len <= 0 || kv_len > S) ? S : kv_len;
  const float sc = scale > 0.f ? scale : 1.0f / sqrtf((float)D);
  return from_hip(spattn::run_booleanmask(packed, qblk, threshold, mask_stride, max_q, denom,
                                          static_cast<const uint16_t*>(q), static_cast<const uint16_t*>(k), B, H, S, D,
                                          kv < mask_stride ? kv : mask_stride, sc, as_stream(stream), blk_indices, blk_counts,
                                          max_blocks));
}

int spattn_packedmask_to_blocklists(int* blk_indices, int* blk_counts, void* blockmask, const void* packed, int B, int H,
                                    int seq, int seqblocks, int mask_stride, int max_blocks, void* stream) {
  if (!blk_indices || !blk_counts || !packed) return done(SPATTN_ERR_NULL);
  if (B <= 0 || H <= 0 || seqblocks <= 0 || seq < 0 || max_blocks <= 0) return done(SPATTN_ERR_SHAPE);
  if (mask_stride <= 0 || mask_stride % 128 != 0) return done(SPATTN_ERR_STRIDE);
  if (misaligned(packed)) return done(SPATTN_ERR_ALIGN);
  return from_hip(spattn::run_packed_to_blocklists(blk_indices, blk_counts, static_cast<unsigned char*>(blockmask),
                                                   static_cast<const uint32_t*>(packed), B * H * seqblocks, mask_stride,
                                                   seq, max_blocks, as_stream(stream)));
}

int spattn_booleanmask_to_blocklists(int* blk_indices, int* blk_counts, void* blockmask, const int* booleanmask, int B,
                                     int H, int seq, int seqblocks, int mask_stride, int max_blocks, void* stream) {
  if (!blk_indices || !blk_counts || !booleanmask) return done(SPATTN_ERR_NULL);
  if (B <= 0 || H <= 0 || seqblocks <= 0 || seq < 0 || max_blocks <= 0) return done(SPATTN_ERR_SHAPE);
  if (mask_stride <= 0 || mask_stride % 128 != 0) return done(SPATTN_ERR_STRIDE);
  if (misaligned(booleanmask)) return done(SPATTN_ERR_ALIGN);
  return from_hip(spattn::run_votes_to_blocklists(blk_indices, blk_counts, static_cast<unsigned char*>(blockmask),
                                                  booleanmask, B * H * seqblocks, mask_stride, seq, max_blocks,
                                                  as_stream(stream)));
}

int spattn_booleanmask_to_indexmask(int* kv_indices, int* num_kv_indices, const int* booleanmask, int B, int H, int seq,
                                    int seqblocks, int mask_stride, void* stream) {
  if (!kv_indices || !num_kv_indices || !booleanmask) return done(SPATTN_ERR_NULL);
  if (B <= 0 || H <= 0 || seqblocks <= 0 || seq < 0) return done(SPATTN_ERR_SHAPE);
  if (mask_stride <= 0 || mask_stride % 128 != 0) return done(SPATTN_ERR_STRIDE);
  if (misaligned(kv_indices) || misaligned(booleanmask)) return done(SPATTN_ERR_ALIGN);
  return from_hip(spattn::run_compact(kv_indices, num_kv_indices, booleanmask, B * H * seqblocks, mask_stride, seq,
                                      as_stream(stream)));
}

int spattn_pack_mask(void* packed, const int* booleanmask, int B, int H, int seqblocks, int mask_stride, void* stream) {
  if (!packed || !booleanmask) return done(SPATTN_ERR_NULL);
  if (B <= 0 || H <= 0 || seqblocks <= 0) return done(SPATTN_ERR_SHAPE);
  if (mask_stride <= 0 || mask_stride % 128 != 0) return done(SPATTN_ERR_STRIDE);
  if (misaligned(packed) || misaligned(booleanmask)) return done(SPATTN_ERR_ALIGN);
  return from_hip(spattn::run_pack_mask(static_cast<uint32_t*>(packed), booleanmask, B * H * seqblocks, mask_stride,
                                        as_stream(stream)));
}

int spattn_packedmask_to_indexmask(int* kv_indices, int* num_kv_indices, const void* packed, int B, int H, int seq,
                                   int seqblocks, int mask_stride, void* stream) {
  if (!kv_indices || !num_kv_indices || !packed) return done(SPATTN_ERR_NULL);
  if (B <= 0 || H <= 0 || seqblocks <= 0 || seq < 0) return done(SPATTN_ERR_SHAPE);
  if (mask_stride <= 0 || mask_stride % 128 != 0) return done(SPATTN_ERR_STRIDE);
  if (misaligned(kv_indices) || misaligned(packed)) return done(SPATTN_ERR_ALIGN);
  return from_hip(spattn::run_packed_to_indexmask(kv_indices, num_kv_indices, static_cast<const uint32_t*>(packed),
                                                  B * H * seqblocks, mask_stride, seq, as_stream(stream)));
}

int spattn_qk_topkmask_indices(int* kv_indices, int* num_kv_indices, void* score, void* qmean, const void* q,
                               const void* k, int batch, int heads, int seq, int D, int blocksz, int kv_len,
                               int select_k, int score_stride, int idx_stride, void* stream) {
  if (!kv_indices || !num_kv_indices || !score || !qmean || !q || !k) return done(SPATTN_ERR_NULL);
  if (D != 64 && D != 128) return done(SPATTN_ERR_HEAD_DIM);
  if (batch <= 0 || heads <= 0 || seq <= 0 || select_k <= 0) return done(SPATTN_ERR_SHAPE);
  if (blocksz != 64 && blocksz != 128) return done(SPATTN_ERR_QBLK);
  if (kv_len < 0 || kv_len > seq) return done(SPATTN_ERR_SHAPE);
  const int kv = kv_len > 0 ? kv_len : seq;
  if (score_stride < kv || score_stride % 8 != 0) return done(SPATTN_ERR_STRIDE);
  if (idx_stride < (select_k < kv ? select_k : kv)) return done(SPATTN_ERR_STRIDE);
  if (misaligned(score) || misaligned(qmean) || misaligned(q) || misaligned(k)) return done(SPATTN_ERR_ALIGN);
  return from_hip(spattn::run_topk_mask(kv_indices, num_kv_indices, static_cast<uint16_t*>(score),
                                        static_cast<uint16_t*>(qmean), static_cast<const uint16_t*>(q),
                                        static_cast<const uint16_t*>(k), batch, heads, seq, D, blocksz, kv, select_k,
                                        score_stride, idx_stride, as_stream(stream)));
}

int spattn_qblock_order(int* order, const int* counts, int n, void* stream) {
  if (!order || !counts) return done(SPATTN_ERR_NULL);
  if (n <= 0) return done(SPATTN_ERR_SHAPE);
  return from_hip(spattn::run_qblock_order(order, counts, n, as_stream(stream)));
}

int spattn_sp_attn_ordered(void* o, float* lse, const void* q, const void* k, const void* v, const int* kv_indices,
                           const int* num_kv_indices, const int* order, int mask_stride, int qblk, int B, int H, int S,
                           int D, int kv_len, float scale, void* stream) {
  if (int st = check_qkv(q, k, B, H, S, D)) return done(st);
  if (!o || !v || !kv_indices || !num_kv_indices || !order) return done(SPATTN_ERR_NULL);
  if (misaligned(o) || misaligned(v) || misaligned(kv_indices)) return done(SPATTN_ERR_ALIGN);
  if (qblk != 64 && qblk != 128) return done(SPATTN_ERR_QBLK);
  if (mask_stride <= 0 || mask_stride % 128 != 0) return done(SPATTN_ERR_STRIDE);
  spattn::AttnParams p = base_params(q, k, v, o, B, H, S, D, kv_len, scale, qblk);
  p.lse = lse;
  p.idx = kv_indices;
  p.cnt = num_kv_indices;
  p.idx_stride = mask_stride;
  p.order = order;
  return from_hip(spattn::run_attn_tokens(p, D, qblk, as_stream(stream)));
}

int spattn_sp_attn_blocks_ordered(void* o, float* lse, const void* q, const void* k, const void* v,
                                  const int* blk_indices, const int* blk_counts, const int* order, int max_blocks,
                                  int qblk, int B, int H, int S, int D, int kv_len, float scale, void* stream) {
  if (int st = check_qkv(q, k, B, H, S, D)) return done(st);
  if (!o || !v || !blk_indices || !blk_counts || !order) return done(SPATTN_ERR_NULL);
  if (misaligned(o) || misaligned(v)) return done(SPATTN_ERR_ALIGN);
  if (qblk != 64 && qblk != 128) return done(SPATTN_ERR_QBLK);
  if (max_blocks <= 0) return done(SPATTN_ERR_SHAPE);
  spattn::AttnParams p = base_params(q, k, v, o, B, H, S, D, kv_len, scale, qblk);
  p.lse = lse;
  p.idx = blk_indices;
  p.cnt = blk_counts;
  p.idx_stride = max_blocks;
  p.order = order;
  return from_hip(spattn::run_attn_blocks(p, D, qblk, as_stream(stream)));
}

// ---- block-list attention in balanced order without a caller-provided order buffer -------------
// The work order (one int per q-block) lives in a device array that belongs to the library:
// every device the library runs on holds its own copy of it, at its own address, until the
// process ends.  Host code never uses the array's name as an address: the per-device address is
// looked up once with hipGetSymbolAddress and kept.

}  // extern "C"

namespace {

constexpr int kScratchInts = SPATTN_BALANCED_MAX_QBLOCKS;
static __device__ __align__(256) int scratch[kScratchInts];

std::mutex g_scratch_mu;
std::atomic<int*> g_scratch_ptr[spattn::kMaxDevices] = {};

// Address of `scratch` on the current device.  Looked up on the first call per device (under a
// lock, and never while `stream` is being captured into a graph: the lookup is a runtime call
// that may initialise the device's copy of the array); every later call is one atomic load.
int scratch_on_current_device(int** out, hipStream_t stream) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= spattn::kMaxDevices) return SPATTN_ERR_SHAPE;
  int* known = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (known == nullptr) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (stream != nullptr && hipStreamIsCapturing(stream, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone)
      return SPATTN_ERR_SCRATCH;   // call spattn_init() on this device before recording
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    known = g_scratch_ptr[dev].load(std::memory_order_relaxed);
    if (known == nullptr) {
      void* p = nullptr;
      e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
      if (e != hipSuccess) return (int)e;
      if (p == nullptr) return (int)hipErrorInvalidSymbol;
      known = static_cast<int*>(p);
      g_scratch_ptr[dev].store(known, std::memory_order_release);
    }
  }
  *out = known;
  return SPATTN_OK;
}

}  // namespace

extern "C" {

int spattn_init(void) {
  int* p = nullptr;
  if (int st = scratch_on_current_device(&p, nullptr)) return done(st);
  // what a first launch would otherwise set on this device: after this call every entry point only launches
  hipError_t e = spattn::prepare_attn_dense();
  if (e == hipSuccess) e = spattn::prepare_attn_blocks();
  if (e == hipSuccess) e = spattn::prepare_attn_tokens();
  return e == hipSuccess ? done(SPATTN_OK) : from_hip(e);
}

int spattn_sp_attn_blocks_balanced(void* o, float* lse, const void* q, const void* k, const void* v,
                                   const int* blk_indices, const int* blk_counts, int max_blocks, int qblk, int B, int H,
                                   int S, int D, int kv_len, float scale, void* stream) {
  if (int st = check_qkv(q, k, B, H, S, D)) return done(st);
  if (!o || !v || !blk_indices || !blk_counts) return done(SPATTN_ERR_NULL);
  if (misaligned(o) || misaligned(v)) return done(SPATTN_ERR_ALIGN);
  if (qblk != 64 && qblk != 128) return done(SPATTN_ERR_QBLK);
  if (max_blocks <= 0) return done(SPATTN_ERR_SHAPE);
  const long long nq = (long long)B * H * ((S + qblk - 1) / qblk);
  if (nq > kScratchInts) return done(SPATTN_ERR_SCRATCH);
  int* order = nullptr;
  if (int st = scratch_on_current_device(&order, as_stream(stream))) return done(st);
  // the order kernel writes all nq entries it is asked for: nothing of an earlier call is read
  const hipError_t e = spattn::run_qblock_order(order, blk_counts, (int)nq, as_stream(stream));
  if (e != hipSuccess) return from_hip(e);
  spattn::AttnParams p = base_params(q, k, v, o, B, H, S, D, kv_len, scale, qblk);
  p.lse = lse;
  p.idx = blk_indices;
  p.cnt = blk_counts;
  p.idx_stride = max_blocks;
  p.order = order;
  return from_hip(spattn::run_attn_blocks(p, D, qblk, as_stream(stream)));
}

// ---- the reference's binding surface: default stream, default scale, q-block 128 ----

void attn_fwd_wg_impl(void* o, void* q, void* k, void* v, int batch, int heads, int seq, int D) {
  spattn_full_attn(o, nullptr, q, k, v, batch, heads, seq, D, 0, 0.f, nullptr);
}

void attn_sparse_fwd_wg_impl(void* o, void* q, void* k, void* v, int* kv_indices, int* num_kv_indices, int mask_stride,
                             int batch, int heads, int seq, int D) {
  spattn_sp_attn(o, nullptr, q, k, v, kv_indices, num_kv_indices, mask_stride, 128, batch, heads, seq, D, 0, 0.f,
                 nullptr);
}

void allindex_mask_impl(int* kv_indices, int* num_kv_indices, int batch, int heads, int seqblocks, int seq) {
  spattn_all_index_mask(kv_indices, num_kv_indices, batch, heads, seqblocks, seq, ((seq + 127) / 128) * 128, nullptr);
}

void attn_maxq_denom_impl(void* d_o, float* d_o_max_q, float* d_o_norm, void* d_q, void* d_k, void* d_v, int batch,
                          int heads, int seq, int D) {
  spattn_fullattn_maxq_denom(d_o, d_o_max_q, d_o_norm, d_q, d_k, d_v, batch, heads, seq, D, 0, 0.f, nullptr);
}

void maxq_denom_impl(float* d_o_max_q, float* d_o_norm, void* d_q, void* d_k, int batch, int heads, int seq, int D) {
  spattn_maxq_denom(d_o_max_q, d_o_norm, d_q, d_k, batch, heads, seq, D, 0, 0.f, nullptr);
}

void booleanmask_128_impl(int* d_booleanmask, float threshold, int mask_stride, float* d_o_max_q, float* d_o_norm,
                          void* d_q, void* d_k, int batch, int heads, int seq, int D) {
  spattn_booleanmask_128(d_booleanmask, threshold, mask_stride, d_o_max_q, d_o_norm, d_q, d_k, batch, heads, seq, D, 0,
                         0.f, nullptr);
}

void booleanmask_to_indexmask_impl(int* d_indexmask, int* d_num_indices, int* d_booleanmask, int batch, int heads,
                                   int seq, int seqblocks, int mask_stride) {
  spattn_booleanmask_to_indexmask(d_indexmask, d_num_indices, d_booleanmask, batch, heads, seq, seqblocks, mask_stride,
                                  nullptr);
}

int spattn_last_status(void) { return g_last_status; }

const char* spattn_status_string(int status) {
  switch (status) {
    case SPATTN_OK: return "ok";
    case SPATTN_ERR_NULL: return "a required pointer is null";
    case SPATTN_ERR_HEAD_DIM: return "head dim must be 64 or 128";
    case SPATTN_ERR_STRIDE: return "mask_stride must be a positive multiple of 128";
    case SPATTN_ERR_QBLK: return "q-block must be 64 or 128";
    case SPATTN_ERR_ALIGN: return "pointer is not 16-byte aligned";
    case SPATTN_ERR_SHAPE: return "a size is not positive or is inconsistent";
    case SPATTN_ERR_SCRATCH:
      return "more q-blocks than the library's own work-order array holds, or its first use on a device inside a stream capture";
    default: return status > 0 ? hipGetErrorString((hipError_t)status) : "unknown status";
  }
}

int spattn_version(void) { return 2; }

}  // extern "C"
