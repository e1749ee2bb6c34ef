// PyTorch operator binding: registers the seven ops of the reference extension in the
// `cuda_attn` namespace (python/extension.cpp:81-358) and exposes the same seven functions
// as a pybind module (python/extension.cpp:362-370).  Operators under further names carry what
// the seven schemas cannot: a runtime kv length (the reference hard-codes one,
// python/cuda_attn.cu:28-31), a softmax scale, a log-sum-exp output, KV-block lists, bit-packed
// masks, and a work order computed once and reused.  Host code only: every op checks its
// arguments and forwards raw device pointers to the C ABI of libspattn_hip.so on the
// current HIP stream.  Unlike the reference, unsupported inputs raise instead of silently
// returning (python/cuda_attn.cu:33-36 under -DNDEBUG).
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <ATen/hip/HIPGraphsUtils.cuh>
#include <torch/extension.h>

#include <mutex>
#include <vector>

#include "spattn_hip.h"

namespace {

void check_status(int st, const char* op) {
  TORCH_CHECK(st == SPATTN_OK, "cuda_attn::", op, " failed: ", spattn_status_string(st), " (status ", st, ")");
}

void check_bhsd(const torch::Tensor& t, const char* name, const torch::Tensor& like) {
  TORCH_CHECK(t.is_cuda(), name, " must be a device tensor");
  TORCH_CHECK(t.scalar_type() == at::kBFloat16, name, " must be bfloat16");
  TORCH_CHECK(t.dim() == 4, name, " must be [B,H,S,D]");
  TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
  TORCH_CHECK(t.sizes() == like.sizes(), name, " must have the shape of q");
  TORCH_CHECK(t.device() == like.device(), name, " must be on the device of q");
}

void check_aux(const torch::Tensor& t, const char* name, at::ScalarType dt, const torch::Tensor& q) {
  TORCH_CHECK(t.is_cuda() && t.device() == q.device(), name, " must be on the device of q");
  TORCH_CHECK(t.scalar_type() == dt, name, " has the wrong dtype");
  TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
}

// PyTorch-ROCm presents HIP devices under the "cuda" device type; these are its guard and
// stream classes for that arrangement.
using DeviceGuard = c10::hip::HIPGuardMasqueradingAsCUDA;
void* cur_stream() { return static_cast<void*>(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()); }

int64_t padded128(int64_t s) { return ((s + 127) / 128) * 128; }

// rows per q-block implied by the number of lists per head; the reference's 128 wins a tie
int infer_qblk(int64_t seq, int64_t seqblocks) {
  if (seqblocks == (seq + 127) / 128) return 128;
  if (seqblocks == (seq + 63) / 64) return 64;
  TORCH_CHECK(false, "kv_indices has ", seqblocks, " q-blocks per head; expected ceil(S/128) or ceil(S/64)");
  return 0;
}

using OptTensor = c10::optional<torch::Tensor>;

// optional fp32 [B,H,S] log-sum-exp output
float* lse_ptr(const OptTensor& lse, const torch::Tensor& q) {
  if (!lse.has_value() || !lse->defined()) return nullptr;
  check_aux(*lse, "lse", at::kFloat, q);
  TORCH_CHECK(lse->numel() == q.size(0) * q.size(1) * q.size(2), "lse must hold B*H*S floats");
  return lse->data_ptr<float>();
}

// optional int32 work order with one entry per q-block
const int* order_ptr(const OptTensor& order, const torch::Tensor& counts) {
  if (!order.has_value() || !order->defined()) return nullptr;
  check_aux(*order, "order", at::kInt, counts);
  TORCH_CHECK(order->numel() == counts.numel(), "order must have one entry per q-block (B*H*SB)");
  return order->data_ptr<int>();
}

int checked_kv_len(int64_t kv_len, const torch::Tensor& q) {
  TORCH_CHECK(kv_len >= 0 && kv_len <= q.size(2), "kv_len must lie in [0, S] (0 = S)");
  return (int)kv_len;
}

}  // namespace

void full_attn_ex(torch::Tensor o, OptTensor lse, torch::Tensor q, torch::Tensor k, torch::Tensor v, double scale,
                  int64_t kv_len) {
  check_bhsd(q, "q", q);
  check_bhsd(k, "k", q);
  check_bhsd(v, "v", q);
  check_bhsd(o, "o", q);
  const DeviceGuard guard(q.device());
  check_status(spattn_full_attn(o.data_ptr(), lse_ptr(lse, q), q.data_ptr(), k.data_ptr(), v.data_ptr(), (int)q.size(0),
                                (int)q.size(1), (int)q.size(2), (int)q.size(3), checked_kv_len(kv_len, q), (float)scale,
                                cur_stream()),
               "full_attn");
}

void full_attn(torch::Tensor o, torch::Tensor q, torch::Tensor k, torch::Tensor v) {
  full_attn_ex(o, c10::nullopt, q, k, v, 0.0, 0);
}

void all_index_mask(torch::Tensor kv_indices, torch::Tensor kv_num_indices, int64_t batch, int64_t heads,
                    int64_t seqblocks, int64_t seq) {
  TORCH_CHECK(kv_indices.is_cuda() && kv_num_indices.is_cuda(), "index tensors must be device tensors");
  TORCH_CHECK(kv_indices.scalar_type() == at::kInt && kv_num_indices.scalar_type() == at::kInt, "index tensors must be int32");
  TORCH_CHECK(kv_indices.is_contiguous() && kv_num_indices.is_contiguous(), "index tensors must be contiguous");
  TORCH_CHECK(kv_indices.dim() == 4 && kv_indices.size(0) == batch && kv_indices.size(1) == heads &&
                  kv_indices.size(2) == seqblocks,
              "kv_indices must be [batch,heads,seqblocks,mask_stride]");
  TORCH_CHECK(kv_num_indices.numel() == batch * heads * seqblocks, "kv_num_indices must have batch*heads*seqblocks entries");
  const DeviceGuard guard(kv_indices.device());
  check_status(spattn_all_index_mask(kv_indices.data_ptr<int>(), kv_num_indices.data_ptr<int>(), (int)batch, (int)heads,
                                     (int)seqblocks, (int)seq, (int)kv_indices.size(3), cur_stream()),
               "all_index_mask");
}

// Token lists.  order: the work order of spattn_qblock_order for these counts, or none.
static void sp_attn_impl(torch::Tensor& o, const OptTensor& lse, torch::Tensor& q, torch::Tensor& k, torch::Tensor& v,
                         torch::Tensor& kv_indices, torch::Tensor& kv_num_indices, const int* order, double scale,
                         int64_t kv_len) {
  const int qblk = infer_qblk(q.size(2), kv_indices.size(2));
  const int B = (int)q.size(0), H = (int)q.size(1), S = (int)q.size(2), D = (int)q.size(3);
  const int kv = checked_kv_len(kv_len, q);
  if (order != nullptr) {
    check_status(spattn_sp_attn_ordered(o.data_ptr(), lse_ptr(lse, q), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                        kv_indices.data_ptr<int>(), kv_num_indices.data_ptr<int>(), order,
                                        (int)kv_indices.size(3), qblk, B, H, S, D, kv, (float)scale, cur_stream()),
                 "sp_attn");
  } else {
    check_status(spattn_sp_attn(o.data_ptr(), lse_ptr(lse, q), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                kv_indices.data_ptr<int>(), kv_num_indices.data_ptr<int>(), (int)kv_indices.size(3), qblk,
                                B, H, S, D, kv, (float)scale, cur_stream()),
                 "sp_attn");
  }
}

static void check_sp_attn_args(torch::Tensor& o, torch::Tensor& q, torch::Tensor& k, torch::Tensor& v,
                               torch::Tensor& kv_indices, torch::Tensor& kv_num_indices) {
  check_bhsd(q, "q", q);
  check_bhsd(k, "k", q);
  check_bhsd(v, "v", q);
  check_bhsd(o, "o", q);
  check_aux(kv_indices, "kv_indices", at::kInt, q);
  check_aux(kv_num_indices, "kv_num_indices", at::kInt, q);
  TORCH_CHECK(kv_indices.dim() == 4 && kv_indices.size(0) == q.size(0) && kv_indices.size(1) == q.size(1),
              "kv_indices must be [B,H,SB,mask_stride]");
  // the reference does not check the shape of kv_num_indices, only its element order
  TORCH_CHECK(kv_num_indices.numel() == q.size(0) * q.size(1) * kv_indices.size(2), "kv_num_indices must have B*H*SB entries");
}

// Work orders of the reference-named sp_attn, which has no argument to pass one in.  One entry per
// (device, stream, address and size of the counts tensor); the entry remembers the version counter
// of the counts it was computed from.  A call that finds its entry with the same version launches
// the attention kernel and nothing else; a new version recomputes the order into the entry's buffer
// (same stream, so launches that still read it are ahead in stream order); only the first sight of a
// counts tensor allocates.  Buffers are never freed or handed to another key, so a launch recorded
// into a graph keeps a valid pointer.  Any permutation of the q-blocks gives the same result: an
// entry that outlived its counts tensor (same address, size and version by coincidence) can cost
// balance, never correctness.
struct OrderEntry {
  int device;
  void* stream;
  const void* counts;
  int64_t numel;
  int64_t version;
  torch::Tensor order;
};
static std::mutex g_order_mu;
// never destroyed: the tensors must not be released after the HIP runtime has shut down at process exit
static std::vector<OrderEntry>& g_orders = *new std::vector<OrderEntry>();
constexpr size_t kMaxOrderEntries = 1024;

static int64_t counts_version(const torch::Tensor& t) {
  return t.is_inference() ? 0 : (int64_t)t._version();
}

// The work order for these counts on the current stream; computes it if the cache has none.
// Returns the tensor that owns the buffer (kept alive by the cache or, when the cache is full or
// the stream is being captured into a graph, by the caller for the length of the call).
static torch::Tensor cached_qblock_order(const torch::Tensor& counts) {
  const int dev = (int)counts.device().index();
  void* stream = cur_stream();
  const int64_t ver = counts_version(counts);
  auto compute = [&](torch::Tensor& order) {
    check_status(spattn_qblock_order(order.data_ptr<int>(), counts.data_ptr<int>(), (int)counts.numel(), stream),
                 "sp_attn (work order)");
  };
  const bool capturing =
      c10::hip::currentStreamCaptureStatusMayInitCtx() != c10::hip::CaptureStatus::None;
  std::lock_guard<std::mutex> lock(g_order_mu);
  for (auto& e : g_orders) {
    if (e.device == dev && e.stream == stream && e.counts == counts.data_ptr() && e.numel == counts.numel()) {
      if (e.version != ver) {
        compute(e.order);
        e.version = ver;
      }
      return e.order;
    }
  }
  torch::Tensor order = torch::empty({counts.numel()}, counts.options());
  compute(order);
  if (!capturing && g_orders.size() < kMaxOrderEntries)
    g_orders.push_back(OrderEntry{dev, stream, counts.data_ptr(), counts.numel(), ver, order});
  return order;
}

void sp_attn(torch::Tensor o, torch::Tensor q, torch::Tensor k, torch::Tensor v, torch::Tensor kv_indices,
             torch::Tensor kv_num_indices) {
  check_sp_attn_args(o, q, k, v, kv_indices, kv_num_indices);
  const DeviceGuard guard(q.device());
  // Threshold masks give lists of very different lengths: the q-blocks are handed to the
  // workgroups longest list first (lists within a factor of two of each other keep the default
  // order).  The order is computed when the counts tensor is first seen or has been written to
  // since (its version counter); every other call is the attention launch alone.
  const torch::Tensor order = cached_qblock_order(kv_num_indices);
  sp_attn_impl(o, c10::nullopt, q, k, v, kv_indices, kv_num_indices, order.data_ptr<int>(), 0.0, 0);
}

// sp_attn with an optional log-sum-exp output, an optional precomputed work order (none: the
// default order, one launch and no allocation), a softmax scale (0 = 1/sqrt(D)) and a kv length.
void sp_attn_ex(torch::Tensor o, OptTensor lse, torch::Tensor q, torch::Tensor k, torch::Tensor v,
                torch::Tensor kv_indices, torch::Tensor kv_num_indices, OptTensor order, double scale, int64_t kv_len) {
  check_sp_attn_args(o, q, k, v, kv_indices, kv_num_indices);
  const DeviceGuard guard(q.device());
  sp_attn_impl(o, lse, q, k, v, kv_indices, kv_num_indices, order_ptr(order, kv_num_indices), scale, kv_len);
}

// Sparse attention over lists of 64-key blocks: blk_idx int32 [B,H,ceil(S/qblk),max_blocks],
// blk_cnt int32 with B*H*ceil(S/qblk) entries, qblk 64 or 128 (0 = implied by blk_idx.size(2)).
void sp_attn_block(torch::Tensor o, OptTensor lse, torch::Tensor q, torch::Tensor k, torch::Tensor v,
                   torch::Tensor blk_idx, torch::Tensor blk_cnt, OptTensor order, int64_t qblk, double scale,
                   int64_t kv_len) {
  check_bhsd(q, "q", q);
  check_bhsd(k, "k", q);
  check_bhsd(v, "v", q);
  check_bhsd(o, "o", q);
  check_aux(blk_idx, "blk_idx", at::kInt, q);
  check_aux(blk_cnt, "blk_cnt", at::kInt, q);
  TORCH_CHECK(blk_idx.dim() == 4 && blk_idx.size(0) == q.size(0) && blk_idx.size(1) == q.size(1),
              "blk_idx must be [B,H,SB,max_blocks]");
  if (qblk == 0) qblk = infer_qblk(q.size(2), blk_idx.size(2));
  TORCH_CHECK(qblk == 64 || qblk == 128, "qblk must be 64 or 128");
  TORCH_CHECK(blk_idx.size(2) == (q.size(2) + qblk - 1) / qblk, "blk_idx must hold ceil(S/qblk) lists per head");
  TORCH_CHECK(blk_cnt.numel() == q.size(0) * q.size(1) * blk_idx.size(2), "blk_cnt must have B*H*SB entries");
  const DeviceGuard guard(q.device());
  const int B = (int)q.size(0), H = (int)q.size(1), S = (int)q.size(2), D = (int)q.size(3);
  const int kv = checked_kv_len(kv_len, q);
  const int* ord = order_ptr(order, blk_cnt);
  if (ord != nullptr) {
    check_status(spattn_sp_attn_blocks_ordered(o.data_ptr(), lse_ptr(lse, q), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                               blk_idx.data_ptr<int>(), blk_cnt.data_ptr<int>(), ord,
                                               (int)blk_idx.size(3), (int)qblk, B, H, S, D, kv, (float)scale,
                                               cur_stream()),
                 "sp_attn_block");
  } else {
    check_status(spattn_sp_attn_blocks(o.data_ptr(), lse_ptr(lse, q), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                       blk_idx.data_ptr<int>(), blk_cnt.data_ptr<int>(), (int)blk_idx.size(3), (int)qblk,
                                       B, H, S, D, kv, (float)scale, cur_stream()),
                 "sp_attn_block");
  }
}

// order int32 [n] <- the q-blocks of counts (int32, n entries) longest list first.
void qblock_order(torch::Tensor order, torch::Tensor counts) {
  TORCH_CHECK(counts.is_cuda() && counts.scalar_type() == at::kInt && counts.is_contiguous(),
              "counts must be a contiguous int32 device tensor");
  check_aux(order, "order", at::kInt, counts);
  TORCH_CHECK(order.numel() == counts.numel() && counts.numel() > 0, "order must have one entry per count");
  const DeviceGuard guard(counts.device());
  check_status(spattn_qblock_order(order.data_ptr<int>(), counts.data_ptr<int>(), (int)counts.numel(), cur_stream()),
               "qblock_order");
}

void fullattn_maxq_denom_ex(torch::Tensor o, torch::Tensor o_max_q, torch::Tensor o_denom, torch::Tensor q,
                            torch::Tensor k, torch::Tensor v, double scale, int64_t kv_len) {
  check_bhsd(q, "q", q);
  check_bhsd(k, "k", q);
  check_bhsd(v, "v", q);
  check_bhsd(o, "o", q);
  check_aux(o_max_q, "o_max_q", at::kFloat, q);
  check_aux(o_denom, "o_denom", at::kFloat, q);
  const int64_t need = q.size(0) * q.size(1) * padded128(q.size(2));
  TORCH_CHECK(o_max_q.numel() == need && o_denom.numel() == need, "o_max_q / o_denom must be [B,H,1,128*ceil(S/128)]");
  const DeviceGuard guard(q.device());
  check_status(spattn_fullattn_maxq_denom(o.data_ptr(), o_max_q.data_ptr<float>(), o_denom.data_ptr<float>(), q.data_ptr(),
                                          k.data_ptr(), v.data_ptr(), (int)q.size(0), (int)q.size(1), (int)q.size(2),
                                          (int)q.size(3), checked_kv_len(kv_len, q), (float)scale, cur_stream()),
               "fullattn_maxq_denom");
}

void fullattn_maxq_denom(torch::Tensor o, torch::Tensor o_max_q, torch::Tensor o_denom, torch::Tensor q, torch::Tensor k,
                         torch::Tensor v) {
  fullattn_maxq_denom_ex(o, o_max_q, o_denom, q, k, v, 0.0, 0);
}

void maxq_denom_ex(torch::Tensor o_max_q, torch::Tensor o_denom, torch::Tensor q, torch::Tensor k, double scale,
                   int64_t kv_len) {
  check_bhsd(q, "q", q);
  check_bhsd(k, "k", q);
  check_aux(o_max_q, "o_max_q", at::kFloat, q);
  check_aux(o_denom, "o_denom", at::kFloat, q);
  const int64_t need = q.size(0) * q.size(1) * padded128(q.size(2));
  TORCH_CHECK(o_max_q.numel() == need && o_denom.numel() == need, "o_max_q / o_denom must be [B,H,1,128*ceil(S/128)]");
  const DeviceGuard guard(q.device());
  check_status(spattn_maxq_denom(o_max_q.data_ptr<float>(), o_denom.data_ptr<float>(), q.data_ptr(), k.data_ptr(),
                                 (int)q.size(0), (int)q.size(1), (int)q.size(2), (int)q.size(3), checked_kv_len(kv_len, q),
                                 (float)scale, cur_stream()),
               "maxq_denom");
}

void maxq_denom(torch::Tensor o_max_q, torch::Tensor o_denom, torch::Tensor q, torch::Tensor k) {
  maxq_denom_ex(o_max_q, o_denom, q, k, 0.0, 0);
}

// The statistics sweeps with the per-(row, key block) score maxima as a further output, and the
// threshold test on those maxima: the block-level form of booleanmask_128 + booleanmask_to_indexmask
// (python/extension.cpp:229-340) that needs no second sweep over Q K^T.
void check_blockmax(const torch::Tensor& blockmax, const torch::Tensor& q_like, int64_t B, int64_t H, int64_t S) {
  check_aux(blockmax, "blockmax", at::kBFloat16, q_like);
  const int64_t sp = padded128(S);
  TORCH_CHECK(blockmax.numel() == B * H * (sp / 64) * sp, "blockmax must be bf16 [B,H,Sp/64,Sp] with Sp = 128*ceil(S/128)");
}

void fullattn_maxq_denom_blockmax(torch::Tensor o, torch::Tensor o_max_q, torch::Tensor o_denom, torch::Tensor blockmax,
                                  torch::Tensor q, torch::Tensor k, torch::Tensor v, double scale, int64_t kv_len) {
  check_bhsd(q, "q", q);
  check_bhsd(k, "k", q);
  check_bhsd(v, "v", q);
  check_bhsd(o, "o", q);
  check_aux(o_max_q, "o_max_q", at::kFloat, q);
  check_aux(o_denom, "o_denom", at::kFloat, q);
  const int64_t need = q.size(0) * q.size(1) * padded128(q.size(2));
  TORCH_CHECK(o_max_q.numel() == need && o_denom.numel() == need, "o_max_q / o_denom must be [B,H,1,128*ceil(S/128)]");
  check_blockmax(blockmax, q, q.size(0), q.size(1), q.size(2));
  const DeviceGuard guard(q.device());
  check_status(spattn_fullattn_maxq_denom_blockmax(o.data_ptr(), o_max_q.data_ptr<float>(), o_denom.data_ptr<float>(),
                                                   blockmax.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                                   (int)q.size(0), (int)q.size(1), (int)q.size(2), (int)q.size(3),
                                                   checked_kv_len(kv_len, q), (float)scale, cur_stream()),
               "fullattn_maxq_denom_blockmax");
}

void maxq_denom_blockmax(torch::Tensor o_max_q, torch::Tensor o_denom, torch::Tensor blockmax, torch::Tensor q,
                         torch::Tensor k, double scale, int64_t kv_len) {
  check_bhsd(q, "q", q);
  check_bhsd(k, "k", q);
  check_aux(o_max_q, "o_max_q", at::kFloat, q);
  check_aux(o_denom, "o_denom", at::kFloat, q);
  const int64_t need = q.size(0) * q.size(1) * padded128(q.size(2));
  TORCH_CHECK(o_max_q.numel() == need && o_denom.numel() == need, "o_max_q / o_denom must be [B,H,1,128*ceil(S/128)]");
  check_blockmax(blockmax, q, q.size(0), q.size(1), q.size(2));
  const DeviceGuard guard(q.device());
  check_status(spattn_maxq_denom_blockmax(o_max_q.data_ptr<float>(), o_denom.data_ptr<float>(), blockmax.data_ptr(),
                                          q.data_ptr(), k.data_ptr(), (int)q.size(0), (int)q.size(1), (int)q.size(2),
                                          (int)q.size(3), checked_kv_len(kv_len, q), (float)scale, cur_stream()),
               "maxq_denom_blockmax");
}

// blk_idx int32 [B,H,ceil(seq/qblk),max_blocks], blk_cnt int32 with B*H*ceil(seq/qblk) entries,
// blockmask optional uint8 [B,H,ceil(seq/qblk),Sp/64]; head_dim fixes the default scale (scale = 0).
void blockmax_to_blocklists(torch::Tensor blk_idx, torch::Tensor blk_cnt, OptTensor blockmask, torch::Tensor blockmax,
                            torch::Tensor o_max_q, torch::Tensor o_denom, double threshold, int64_t seq, int64_t head_dim,
                            int64_t qblk, double scale, int64_t kv_len) {
  TORCH_CHECK(blk_idx.is_cuda() && blk_idx.scalar_type() == at::kInt && blk_idx.is_contiguous() && blk_idx.dim() == 4,
              "blk_idx must be a contiguous int32 device tensor [B,H,ceil(seq/qblk),max_blocks]");
  TORCH_CHECK(qblk == 64 || qblk == 128, "qblk must be 64 or 128");
  TORCH_CHECK(seq > 0 && kv_len >= 0 && kv_len <= seq, "seq must be positive and kv_len lie in [0, seq]");
  const int64_t B = blk_idx.size(0), H = blk_idx.size(1), SB = blk_idx.size(2), sp = padded128(seq);
  TORCH_CHECK(SB == (seq + qblk - 1) / qblk, "blk_idx must hold ceil(seq/qblk) lists per head");
  check_aux(blk_cnt, "blk_cnt", at::kInt, blk_idx);
  TORCH_CHECK(blk_cnt.numel() == B * H * SB, "blk_cnt must have B*H*ceil(seq/qblk) entries");
  check_aux(o_max_q, "o_max_q", at::kFloat, blk_idx);
  check_aux(o_denom, "o_denom", at::kFloat, blk_idx);
  TORCH_CHECK(o_max_q.numel() == B * H * sp && o_denom.numel() == B * H * sp, "o_max_q / o_denom must be [B,H,1,128*ceil(S/128)]");
  check_blockmax(blockmax, blk_idx, B, H, seq);
  void* bm = nullptr;
  if (blockmask.has_value() && blockmask->defined()) {
    check_aux(*blockmask, "blockmask", at::kByte, blk_idx);
    TORCH_CHECK(blockmask->numel() == B * H * SB * (sp / 64), "blockmask must be uint8 [B,H,ceil(seq/qblk),Sp/64]");
    bm = blockmask->data_ptr();
  }
  const DeviceGuard guard(blk_idx.device());
  check_status(spattn_blockmax_to_blocklists(blk_idx.data_ptr<int>(), blk_cnt.data_ptr<int>(), bm, blockmax.data_ptr(),
                                             o_max_q.data_ptr<float>(), o_denom.data_ptr<float>(), (float)threshold, (int)qblk,
                                             (int)B, (int)H, (int)seq, (int)head_dim, (int)kv_len, (float)scale,
                                             (int)blk_idx.size(3), cur_stream()),
               "blockmax_to_blocklists");
}

void booleanmask_128_ex(torch::Tensor booleanmask, torch::Tensor o_max_q, torch::Tensor o_denom, torch::Tensor q,
                        torch::Tensor k, double threshold, double scale, int64_t kv_len) {
  check_bhsd(q, "q", q);
  check_bhsd(k, "k", q);
  check_aux(booleanmask, "booleanmask", at::kInt, q);
  check_aux(o_max_q, "o_max_q", at::kFloat, q);
  check_aux(o_denom, "o_denom", at::kFloat, q);
  TORCH_CHECK(booleanmask.dim() == 4 && booleanmask.size(0) == q.size(0) && booleanmask.size(1) == q.size(1) &&
                  booleanmask.size(2) == (q.size(2) + 127) / 128,
              "booleanmask must be [B,H,ceil(S/128),mask_stride]");
  const int64_t need = q.size(0) * q.size(1) * padded128(q.size(2));
  TORCH_CHECK(o_max_q.numel() == need && o_denom.numel() == need, "o_max_q / o_denom must be [B,H,1,128*ceil(S/128)]");
  const DeviceGuard guard(q.device());
  check_status(spattn_booleanmask_128(booleanmask.data_ptr<int>(), (float)threshold, (int)booleanmask.size(3),
                                      o_max_q.data_ptr<float>(), o_denom.data_ptr<float>(), q.data_ptr(), k.data_ptr(),
                                      (int)q.size(0), (int)q.size(1), (int)q.size(2), (int)q.size(3),
                                      checked_kv_len(kv_len, q), (float)scale, cur_stream()),
               "booleanmask_128");
}

void booleanmask_128(torch::Tensor booleanmask, torch::Tensor o_max_q, torch::Tensor o_denom, torch::Tensor q,
                     torch::Tensor k, double threshold) {
  booleanmask_128_ex(booleanmask, o_max_q, o_denom, q, k, threshold, 0.0, 0);
}

// The threshold sweep with a bit-packed result: packed uint8 [B,H,ceil(S/qblk),mask_stride/8],
// one bit per (q-block of qblk rows, key), least significant bit first.
// The sweeps restricted to the 64-key blocks listed per 128-row q-block (blk_idx int32
// [B,H,ceil(S/128),max_blocks], blk_cnt with B*H*ceil(S/128) entries): everything else is zeroed.
void check_lists128(const torch::Tensor& blk_idx, const torch::Tensor& blk_cnt, const torch::Tensor& q) {
  check_aux(blk_idx, "blk_idx", at::kInt, q);
  check_aux(blk_cnt, "blk_cnt", at::kInt, q);
  const int64_t SB = (q.size(2) + 127) / 128;
  TORCH_CHECK(blk_idx.dim() == 4 && blk_idx.size(0) == q.size(0) && blk_idx.size(1) == q.size(1) && blk_idx.size(2) == SB &&
                  blk_idx.size(3) > 0,
              "blk_idx must be [B,H,ceil(S/128),max_blocks]");
  TORCH_CHECK(blk_cnt.numel() == q.size(0) * q.size(1) * SB, "blk_cnt must have B*H*ceil(S/128) entries");
}

void booleanmask_128_blocks(torch::Tensor booleanmask, torch::Tensor o_max_q, torch::Tensor o_denom, torch::Tensor q,
                            torch::Tensor k, torch::Tensor blk_idx, torch::Tensor blk_cnt, double threshold, double scale,
                            int64_t kv_len) {
  check_bhsd(q, "q", q);
  check_bhsd(k, "k", q);
  check_aux(booleanmask, "booleanmask", at::kInt, q);
  check_aux(o_max_q, "o_max_q", at::kFloat, q);
  check_aux(o_denom, "o_denom", at::kFloat, q);
  check_lists128(blk_idx, blk_cnt, q);
  TORCH_CHECK(booleanmask.dim() == 4 && booleanmask.size(0) == q.size(0) && booleanmask.size(1) == q.size(1) &&
                  booleanmask.size(2) == (q.size(2) + 127) / 128,
              "booleanmask must be [B,H,ceil(S/128),mask_stride]");
  const int64_t need = q.size(0) * q.size(1) * padded128(q.size(2));
  TORCH_CHECK(o_max_q.numel() == need && o_denom.numel() == need, "o_max_q / o_denom must be [B,H,1,128*ceil(S/128)]");
  const DeviceGuard guard(q.device());
  check_status(spattn_booleanmask_128_blocks(booleanmask.data_ptr<int>(), (float)threshold, (int)booleanmask.size(3),
                                             o_max_q.data_ptr<float>(), o_denom.data_ptr<float>(), q.data_ptr(), k.data_ptr(),
                                             blk_idx.data_ptr<int>(), blk_cnt.data_ptr<int>(), (int)blk_idx.size(3),
                                             (int)q.size(0), (int)q.size(1), (int)q.size(2), (int)q.size(3),
                                             checked_kv_len(kv_len, q), (float)scale, cur_stream()),
               "booleanmask_128_blocks");
}

void booleanmask_packed_blocks(torch::Tensor packed, torch::Tensor o_max_q, torch::Tensor o_denom, torch::Tensor q,
                               torch::Tensor k, torch::Tensor blk_idx, torch::Tensor blk_cnt, double threshold, int64_t qblk,
                               double scale, int64_t kv_len) {
  check_bhsd(q, "q", q);
  check_bhsd(k, "k", q);
  check_aux(packed, "packed", at::kByte, q);
  check_aux(o_max_q, "o_max_q", at::kFloat, q);
  check_aux(o_denom, "o_denom", at::kFloat, q);
  check_lists128(blk_idx, blk_cnt, q);
  TORCH_CHECK(qblk == 64 || qblk == 128, "qblk must be 64 or 128");
  TORCH_CHECK(packed.dim() == 4 && packed.size(0) == q.size(0) && packed.size(1) == q.size(1) &&
                  packed.size(2) == (q.size(2) + qblk - 1) / qblk,
              "packed must be [B,H,ceil(S/qblk),mask_stride/8]");
  const int64_t need = q.size(0) * q.size(1) * padded128(q.size(2));
  TORCH_CHECK(o_max_q.numel() == need && o_denom.numel() == need, "o_max_q / o_denom must be [B,H,1,128*ceil(S/128)]");
  const DeviceGuard guard(q.device());
  check_status(spattn_booleanmask_packed_blocks(packed.data_ptr(), (float)threshold, (int)packed.size(3) * 8, (int)qblk,
                                                o_max_q.data_ptr<float>(), o_denom.data_ptr<float>(), q.data_ptr(), k.data_ptr(),
                                                blk_idx.data_ptr<int>(), blk_cnt.data_ptr<int>(), (int)blk_idx.size(3),
                                                (int)q.size(0), (int)q.size(1), (int)q.size(2), (int)q.size(3),
                                                checked_kv_len(kv_len, q), (float)scale, cur_stream()),
               "booleanmask_packed_blocks");
}

void booleanmask_packed(torch::Tensor packed, torch::Tensor o_max_q, torch::Tensor o_denom, torch::Tensor q,
                        torch::Tensor k, double threshold, int64_t qblk, double scale, int64_t kv_len) {
  check_bhsd(q, "q", q);
  check_bhsd(k, "k", q);
  check_aux(packed, "packed", at::kByte, q);
  check_aux(o_max_q, "o_max_q", at::kFloat, q);
  check_aux(o_denom, "o_denom", at::kFloat, q);
  TORCH_CHECK(qblk == 64 || qblk == 128, "qblk must be 64 or 128");
  TORCH_CHECK(packed.dim() == 4 && packed.size(0) == q.size(0) && packed.size(1) == q.size(1) &&
                  packed.size(2) == (q.size(2) + qblk - 1) / qblk,
              "packed must be [B,H,ceil(S/qblk),mask_stride/8]");
  const int64_t need = q.size(0) * q.size(1) * padded128(q.size(2));
  TORCH_CHECK(o_max_q.numel() == need && o_denom.numel() == need, "o_max_q / o_denom must be [B,H,1,128*ceil(S/128)]");
  const DeviceGuard guard(q.device());
  check_status(spattn_booleanmask_packed(packed.data_ptr(), (float)threshold, (int)packed.size(3) * 8, (int)qblk,
                                         o_max_q.data_ptr<float>(), o_denom.data_ptr<float>(), q.data_ptr(), k.data_ptr(),
                                         (int)q.size(0), (int)q.size(1), (int)q.size(2), (int)q.size(3),
                                         checked_kv_len(kv_len, q), (float)scale, cur_stream()),
               "booleanmask_packed");
}

// Key mask -> ascending lists of kept 64-key blocks (+ counts, + optional uint8 block mask
// [B,H,SB,mask_stride/64]); the source is the bit-packed mask or the int32 vote mask.
static void blocklists_common(torch::Tensor& blk_idx, torch::Tensor& blk_cnt, const OptTensor& blockmask,
                              const torch::Tensor& src, int64_t mask_stride, int64_t seq) {
  check_aux(blk_idx, "blk_idx", at::kInt, src);
  check_aux(blk_cnt, "blk_cnt", at::kInt, src);
  TORCH_CHECK(blk_idx.dim() == 4 && blk_idx.size(0) == src.size(0) && blk_idx.size(1) == src.size(1) &&
                  blk_idx.size(2) == src.size(2) && blk_idx.size(3) > 0,
              "blk_idx must be [B,H,SB,max_blocks]");
  TORCH_CHECK(blk_cnt.numel() == src.size(0) * src.size(1) * src.size(2), "blk_cnt must have B*H*SB entries");
  TORCH_CHECK(seq >= 0, "seq must not be negative");
  if (blockmask.has_value() && blockmask->defined()) {
    check_aux(*blockmask, "blockmask", at::kByte, src);
    TORCH_CHECK(blockmask->numel() == blk_cnt.numel() * (mask_stride / 64), "blockmask must be uint8 [B,H,SB,mask_stride/64]");
  }
}

void packedmask_to_blocklists(torch::Tensor blk_idx, torch::Tensor blk_cnt, OptTensor blockmask, torch::Tensor packed,
                              int64_t seq) {
  TORCH_CHECK(packed.is_cuda() && packed.scalar_type() == at::kByte && packed.is_contiguous() && packed.dim() == 4,
              "packed must be a contiguous uint8 device tensor [B,H,SB,mask_stride/8]");
  blocklists_common(blk_idx, blk_cnt, blockmask, packed, packed.size(3) * 8, seq);
  const DeviceGuard guard(packed.device());
  void* bm = (blockmask.has_value() && blockmask->defined()) ? blockmask->data_ptr() : nullptr;
  check_status(spattn_packedmask_to_blocklists(blk_idx.data_ptr<int>(), blk_cnt.data_ptr<int>(), bm, packed.data_ptr(),
                                               (int)packed.size(0), (int)packed.size(1), (int)seq, (int)packed.size(2),
                                               (int)packed.size(3) * 8, (int)blk_idx.size(3), cur_stream()),
               "packedmask_to_blocklists");
}

void booleanmask_to_blocklists(torch::Tensor blk_idx, torch::Tensor blk_cnt, OptTensor blockmask,
                               torch::Tensor booleanmask, int64_t seq) {
  TORCH_CHECK(booleanmask.is_cuda() && booleanmask.scalar_type() == at::kInt && booleanmask.is_contiguous() &&
                  booleanmask.dim() == 4,
              "booleanmask must be a contiguous int32 device tensor [B,H,SB,mask_stride]");
  blocklists_common(blk_idx, blk_cnt, blockmask, booleanmask, booleanmask.size(3), seq);
  const DeviceGuard guard(booleanmask.device());
  void* bm = (blockmask.has_value() && blockmask->defined()) ? blockmask->data_ptr() : nullptr;
  check_status(spattn_booleanmask_to_blocklists(blk_idx.data_ptr<int>(), blk_cnt.data_ptr<int>(), bm,
                                                booleanmask.data_ptr<int>(), (int)booleanmask.size(0),
                                                (int)booleanmask.size(1), (int)seq, (int)booleanmask.size(2),
                                                (int)booleanmask.size(3), (int)blk_idx.size(3), cur_stream()),
               "booleanmask_to_blocklists");
}

void booleanmask_to_indexmask(torch::Tensor kv_indices, torch::Tensor kv_numindices, torch::Tensor booleanmask, int64_t seq) {
  TORCH_CHECK(booleanmask.is_cuda() && booleanmask.scalar_type() == at::kInt && booleanmask.is_contiguous() &&
                  booleanmask.dim() == 4,
              "booleanmask must be a contiguous int32 device tensor [B,H,SB,mask_stride]");
  check_aux(kv_indices, "kv_indices", at::kInt, booleanmask);
  check_aux(kv_numindices, "kv_numindices", at::kInt, booleanmask);
  TORCH_CHECK(kv_indices.sizes() == booleanmask.sizes(), "kv_indices must have the shape of booleanmask");
  TORCH_CHECK(kv_numindices.numel() == booleanmask.size(0) * booleanmask.size(1) * booleanmask.size(2),
              "kv_numindices must have B*H*SB entries");
  TORCH_CHECK(seq >= 0, "seq must not be negative");
  const DeviceGuard guard(booleanmask.device());
  check_status(spattn_booleanmask_to_indexmask(kv_indices.data_ptr<int>(), kv_numindices.data_ptr<int>(),
                                               booleanmask.data_ptr<int>(), (int)booleanmask.size(0), (int)booleanmask.size(1),
                                               (int)seq, (int)booleanmask.size(2), (int)booleanmask.size(3), cur_stream()),
               "booleanmask_to_indexmask");
}

// Two operators beyond the reference's seven, for its bit-packed mask cache
// (python/spattn/mask_utils.py:74-98,421-439): the cache's torch-level pack / unpack become
// one kernel each way.
void pack_mask(torch::Tensor packed, torch::Tensor booleanmask) {
  TORCH_CHECK(booleanmask.is_cuda() && booleanmask.scalar_type() == at::kInt && booleanmask.is_contiguous() &&
                  booleanmask.dim() == 4,
              "booleanmask must be a contiguous int32 device tensor [B,H,SB,mask_stride]");
  check_aux(packed, "packed", at::kByte, booleanmask);
  TORCH_CHECK(packed.dim() == 4 && packed.size(0) == booleanmask.size(0) && packed.size(1) == booleanmask.size(1) &&
                  packed.size(2) == booleanmask.size(2) && packed.size(3) * 8 == booleanmask.size(3),
              "packed must be uint8 [B,H,SB,mask_stride/8]");
  const DeviceGuard guard(booleanmask.device());
  check_status(spattn_pack_mask(packed.data_ptr(), booleanmask.data_ptr<int>(), (int)booleanmask.size(0),
                                (int)booleanmask.size(1), (int)booleanmask.size(2), (int)booleanmask.size(3), cur_stream()),
               "pack_mask");
}

void packedmask_to_indexmask(torch::Tensor kv_indices, torch::Tensor kv_numindices, torch::Tensor packed, int64_t seq) {
  TORCH_CHECK(packed.is_cuda() && packed.scalar_type() == at::kByte && packed.is_contiguous() && packed.dim() == 4,
              "packed must be a contiguous uint8 device tensor [B,H,SB,mask_stride/8]");
  check_aux(kv_indices, "kv_indices", at::kInt, packed);
  check_aux(kv_numindices, "kv_numindices", at::kInt, packed);
  TORCH_CHECK(kv_indices.dim() == 4 && kv_indices.size(0) == packed.size(0) && kv_indices.size(1) == packed.size(1) &&
                  kv_indices.size(2) == packed.size(2) && kv_indices.size(3) == packed.size(3) * 8,
              "kv_indices must be [B,H,SB,mask_stride]");
  TORCH_CHECK(kv_numindices.numel() == packed.size(0) * packed.size(1) * packed.size(2),
              "kv_numindices must have B*H*SB entries");
  TORCH_CHECK(seq >= 0, "seq must not be negative");
  const DeviceGuard guard(packed.device());
  check_status(spattn_packedmask_to_indexmask(kv_indices.data_ptr<int>(), kv_numindices.data_ptr<int>(), packed.data_ptr(),
                                              (int)packed.size(0), (int)packed.size(1), (int)seq, (int)packed.size(2),
                                              (int)packed.size(3) * 8, cur_stream()),
               "packedmask_to_indexmask");
}

// The top-k mask generator of the reference's Python layer (python/spattn/mask_utils.py:389-417)
// as one operator: q-block means, their scores against every key, and the select_k best keys
// per q-block as ascending lists.  score and qmean are outputs too.
void qk_topkmask_indices(torch::Tensor kv_indices, torch::Tensor kv_numindices, torch::Tensor score, torch::Tensor qmean,
                         torch::Tensor q, torch::Tensor k, int64_t select_k, int64_t blocksz) {
  TORCH_CHECK(q.is_cuda() && q.scalar_type() == at::kBFloat16 && q.is_contiguous() && q.dim() == 4,
              "q must be a contiguous bf16 device tensor [B,H,S,D]");
  check_aux(k, "k", at::kBFloat16, q);
  check_aux(score, "score", at::kBFloat16, q);
  check_aux(qmean, "qmean", at::kBFloat16, q);
  check_aux(kv_indices, "kv_indices", at::kInt, q);
  check_aux(kv_numindices, "kv_numindices", at::kInt, q);
  TORCH_CHECK(k.sizes() == q.sizes(), "k must match q");
  TORCH_CHECK(blocksz > 0, "blocksz must be positive");
  const int64_t B = q.size(0), H = q.size(1), S = q.size(2), D = q.size(3);
  const int64_t SB = (S + blocksz - 1) / blocksz;
  TORCH_CHECK(qmean.dim() == 4 && qmean.size(0) == B && qmean.size(1) == H && qmean.size(2) == SB && qmean.size(3) == D,
              "qmean must be [B,H,SB,D]");
  TORCH_CHECK(score.dim() == 4 && score.size(0) == B && score.size(1) == H && score.size(2) == SB,
              "score must be [B,H,SB,score_stride]");
  TORCH_CHECK(kv_indices.dim() == 4 && kv_indices.size(0) == B && kv_indices.size(1) == H && kv_indices.size(2) == SB,
              "kv_indices must be [B,H,SB,idx_stride]");
  TORCH_CHECK(kv_numindices.numel() == B * H * SB, "kv_numindices must have B*H*SB entries");
  const DeviceGuard guard(q.device());
  check_status(spattn_qk_topkmask_indices(kv_indices.data_ptr<int>(), kv_numindices.data_ptr<int>(), score.data_ptr(),
                                          qmean.data_ptr(), q.data_ptr(), k.data_ptr(), (int)B, (int)H, (int)S, (int)D,
                                          (int)blocksz, 0, (int)select_k, (int)score.size(3), (int)kv_indices.size(3),
                                          cur_stream()),
               "qk_topkmask_indices");
}

// Meta kernels: shapes only, nothing to compute (all ops mutate their arguments in place).
void noop4(torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor) {}
void noop_all_index(torch::Tensor, torch::Tensor, int64_t, int64_t, int64_t, int64_t) {}
void noop6(torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor) {}
void noop_mask(torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, double) {}
void noop_b2i(torch::Tensor, torch::Tensor, torch::Tensor, int64_t) {}
void noop2(torch::Tensor, torch::Tensor) {}
void noop_topk(torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, int64_t, int64_t) {}
void noop_full_ex(torch::Tensor, OptTensor, torch::Tensor, torch::Tensor, torch::Tensor, double, int64_t) {}
void noop_sp_ex(torch::Tensor, OptTensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, OptTensor,
                double, int64_t) {}
void noop_sp_block(torch::Tensor, OptTensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
                   OptTensor, int64_t, double, int64_t) {}
void noop_fmd_ex(torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, double, int64_t) {}
void noop_md_ex(torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, double, int64_t) {}
void noop_mask_ex(torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, double, double, int64_t) {}
void noop_mask_packed(torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, double, int64_t, double,
                      int64_t) {}
void noop_blocklists(torch::Tensor, torch::Tensor, OptTensor, torch::Tensor, int64_t) {}
void noop_mask_blocks(torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, double,
                      double, int64_t) {}
void noop_mask_packed_blocks(torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
                             double, int64_t, double, int64_t) {}
void noop_fmd_bm(torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, double,
                 int64_t) {}
void noop_md_bm(torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, double, int64_t) {}
void noop_bm_lists(torch::Tensor, torch::Tensor, OptTensor, torch::Tensor, torch::Tensor, torch::Tensor, double, int64_t, int64_t,
                   int64_t, double, int64_t) {}

TORCH_LIBRARY_FRAGMENT(cuda_attn, m) {
  m.def("full_attn(Tensor(a!) o, Tensor q, Tensor k, Tensor v) -> ()");
  m.def("all_index_mask(Tensor(a!) kv_indices, Tensor(b!) kv_num_indices, int batch, int heads, int seqblocks, int seq) -> ()");
  m.def("sp_attn(Tensor(a!) o, Tensor q, Tensor k, Tensor v, Tensor kv_indices, Tensor kv_num_indices) -> ()");
  m.def("fullattn_maxq_denom(Tensor(a!) o, Tensor(b!) o_max_q, Tensor(c!) o_denom, Tensor q, Tensor k, Tensor v) -> ()");
  m.def("maxq_denom(Tensor(a!) o_max_q, Tensor(b!) o_denom, Tensor q, Tensor k) -> ()");
  m.def("booleanmask_128(Tensor(a!) booleanmask, Tensor o_max_q, Tensor o_denom, Tensor q, Tensor k, float threshold) -> ()");
  m.def("booleanmask_to_indexmask(Tensor(a!) kv_indices, Tensor(b!) kv_numindices, Tensor booleanmask, int seq) -> ()");
  m.def("pack_mask(Tensor(a!) packed, Tensor booleanmask) -> ()");
  m.def("packedmask_to_indexmask(Tensor(a!) kv_indices, Tensor(b!) kv_numindices, Tensor packed, int seq) -> ()");
  m.def("qk_topkmask_indices(Tensor(a!) kv_indices, Tensor(b!) kv_numindices, Tensor(c!) score, Tensor(d!) qmean, Tensor q, Tensor k, int select_k, int blocksz) -> ()");
  // scale 0 = 1/sqrt(D); kv_len 0 = S
  m.def("full_attn_ex(Tensor(a!) o, Tensor(b!)? lse, Tensor q, Tensor k, Tensor v, float scale, int kv_len) -> ()");
  m.def("sp_attn_ex(Tensor(a!) o, Tensor(b!)? lse, Tensor q, Tensor k, Tensor v, Tensor kv_indices, Tensor kv_num_indices, Tensor? order, float scale, int kv_len) -> ()");
  m.def("sp_attn_block(Tensor(a!) o, Tensor(b!)? lse, Tensor q, Tensor k, Tensor v, Tensor blk_idx, Tensor blk_cnt, Tensor? order, int qblk, float scale, int kv_len) -> ()");
  m.def("fullattn_maxq_denom_ex(Tensor(a!) o, Tensor(b!) o_max_q, Tensor(c!) o_denom, Tensor q, Tensor k, Tensor v, float scale, int kv_len) -> ()");
  m.def("maxq_denom_ex(Tensor(a!) o_max_q, Tensor(b!) o_denom, Tensor q, Tensor k, float scale, int kv_len) -> ()");
  m.def("booleanmask_128_ex(Tensor(a!) booleanmask, Tensor o_max_q, Tensor o_denom, Tensor q, Tensor k, float threshold, float scale, int kv_len) -> ()");
  m.def("booleanmask_packed(Tensor(a!) packed, Tensor o_max_q, Tensor o_denom, Tensor q, Tensor k, float threshold, int qblk, float scale, int kv_len) -> ()");
  m.def("packedmask_to_blocklists(Tensor(a!) blk_idx, Tensor(b!) blk_cnt, Tensor(c!)? blockmask, Tensor packed, int seq) -> ()");
  m.def("booleanmask_to_blocklists(Tensor(a!) blk_idx, Tensor(b!) blk_cnt, Tensor(c!)? blockmask, Tensor booleanmask, int seq) -> ()");
  m.def("qblock_order(Tensor(a!) order, Tensor counts) -> ()");
  m.def("booleanmask_128_blocks(Tensor(a!) booleanmask, Tensor o_max_q, Tensor o_denom, Tensor q, Tensor k, Tensor blk_idx, Tensor blk_cnt, float threshold, float scale, int kv_len) -> ()");
  m.def("booleanmask_packed_blocks(Tensor(a!) packed, Tensor o_max_q, Tensor o_denom, Tensor q, Tensor k, Tensor blk_idx, Tensor blk_cnt, float threshold, int qblk, float scale, int kv_len) -> ()");
  m.def("fullattn_maxq_denom_blockmax(Tensor(a!) o, Tensor(b!) o_max_q, Tensor(c!) o_denom, Tensor(d!) blockmax, Tensor q, Tensor k, Tensor v, float scale, int kv_len) -> ()");
  m.def("maxq_denom_blockmax(Tensor(a!) o_max_q, Tensor(b!) o_denom, Tensor(c!) blockmax, Tensor q, Tensor k, float scale, int kv_len) -> ()");
  m.def("blockmax_to_blocklists(Tensor(a!) blk_idx, Tensor(b!) blk_cnt, Tensor(c!)? blockmask, Tensor blockmax, Tensor o_max_q, Tensor o_denom, float threshold, int seq, int head_dim, int qblk, float scale, int kv_len) -> ()");
}

TORCH_LIBRARY_IMPL(cuda_attn, Meta, m) {
  m.impl("full_attn", noop4);
  m.impl("all_index_mask", noop_all_index);
  m.impl("sp_attn", noop6);
  m.impl("fullattn_maxq_denom", noop6);
  m.impl("maxq_denom", noop4);
  m.impl("booleanmask_128", noop_mask);
  m.impl("booleanmask_to_indexmask", noop_b2i);
  m.impl("pack_mask", noop2);
  m.impl("packedmask_to_indexmask", noop_b2i);
  m.impl("qk_topkmask_indices", noop_topk);
  m.impl("full_attn_ex", noop_full_ex);
  m.impl("sp_attn_ex", noop_sp_ex);
  m.impl("sp_attn_block", noop_sp_block);
  m.impl("fullattn_maxq_denom_ex", noop_fmd_ex);
  m.impl("maxq_denom_ex", noop_md_ex);
  m.impl("booleanmask_128_ex", noop_mask_ex);
  m.impl("booleanmask_packed", noop_mask_packed);
  m.impl("packedmask_to_blocklists", noop_blocklists);
  m.impl("booleanmask_to_blocklists", noop_blocklists);
  m.impl("qblock_order", noop2);
  m.impl("booleanmask_128_blocks", noop_mask_blocks);
  m.impl("booleanmask_packed_blocks", noop_mask_packed_blocks);
  m.impl("fullattn_maxq_denom_blockmax", noop_fmd_bm);
  m.impl("maxq_denom_blockmax", noop_md_bm);
  m.impl("blockmax_to_blocklists", noop_bm_lists);
}

// The CUDA dispatch key serves HIP tensors on PyTorch-ROCm.
TORCH_LIBRARY_IMPL(cuda_attn, CUDA, m) {
  m.impl("full_attn", full_attn);
  m.impl("all_index_mask", all_index_mask);
  m.impl("sp_attn", sp_attn);
  m.impl("fullattn_maxq_denom", fullattn_maxq_denom);
  m.impl("maxq_denom", maxq_denom);
  m.impl("booleanmask_128", booleanmask_128);
  m.impl("booleanmask_to_indexmask", booleanmask_to_indexmask);
  m.impl("pack_mask", pack_mask);
  m.impl("packedmask_to_indexmask", packedmask_to_indexmask);
  m.impl("qk_topkmask_indices", qk_topkmask_indices);
  m.impl("full_attn_ex", full_attn_ex);
  m.impl("sp_attn_ex", sp_attn_ex);
  m.impl("sp_attn_block", sp_attn_block);
  m.impl("fullattn_maxq_denom_ex", fullattn_maxq_denom_ex);
  m.impl("maxq_denom_ex", maxq_denom_ex);
  m.impl("booleanmask_128_ex", booleanmask_128_ex);
  m.impl("booleanmask_packed", booleanmask_packed);
  m.impl("packedmask_to_blocklists", packedmask_to_blocklists);
  m.impl("booleanmask_to_blocklists", booleanmask_to_blocklists);
  m.impl("qblock_order", qblock_order);
  m.impl("booleanmask_128_blocks", booleanmask_128_blocks);
  m.impl("booleanmask_packed_blocks", booleanmask_packed_blocks);
  m.impl("fullattn_maxq_denom_blockmax", fullattn_maxq_denom_blockmax);
  m.impl("maxq_denom_blockmax", maxq_denom_blockmax);
  m.impl("blockmax_to_blocklists", blockmax_to_blocklists);
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("full_attn", &full_attn, "Full attention");
  m.def("sp_attn", &sp_attn, "Sparse attention");
  m.def("all_index_mask", &all_index_mask, "all index mask");
  m.def("maxq_denom", &maxq_denom, "maxq_denom");
  m.def("booleanmask_128", &booleanmask_128, "booleanmask_128");
  m.def("booleanmask_to_indexmask", &booleanmask_to_indexmask, "booleanmask_to_indexmask");
  m.def("fullattn_maxq_denom", &fullattn_maxq_denom, "fullattn_maxq_denom");
  m.def("pack_mask", &pack_mask, "pack_mask");
  m.def("packedmask_to_indexmask", &packedmask_to_indexmask, "packedmask_to_indexmask");
  m.def("qk_topkmask_indices", &qk_topkmask_indices, "qk_topkmask_indices");
  m.def("full_attn_ex", &full_attn_ex, "full_attn with lse, scale, kv_len");
  m.def("sp_attn_ex", &sp_attn_ex, "sp_attn with lse, work order, scale, kv_len");
  m.def("sp_attn_block", &sp_attn_block, "sparse attention over KV-block lists");
  m.def("fullattn_maxq_denom_ex", &fullattn_maxq_denom_ex, "fullattn_maxq_denom with scale, kv_len");
  m.def("maxq_denom_ex", &maxq_denom_ex, "maxq_denom with scale, kv_len");
  m.def("booleanmask_128_ex", &booleanmask_128_ex, "booleanmask_128 with scale, kv_len");
  m.def("booleanmask_packed", &booleanmask_packed, "threshold sweep, bit-packed result");
  m.def("packedmask_to_blocklists", &packedmask_to_blocklists, "bit-packed mask -> KV-block lists");
  m.def("booleanmask_to_blocklists", &booleanmask_to_blocklists, "vote mask -> KV-block lists");
  m.def("qblock_order", &qblock_order, "work order, longest list first");
  m.def("booleanmask_128_blocks", &booleanmask_128_blocks, "threshold sweep over listed key blocks, int32 votes");
  m.def("booleanmask_packed_blocks", &booleanmask_packed_blocks, "threshold sweep over listed key blocks, bit-packed");
  m.def("fullattn_maxq_denom_blockmax", &fullattn_maxq_denom_blockmax, "fullattn_maxq_denom + per-block row maxima");
  m.def("maxq_denom_blockmax", &maxq_denom_blockmax, "maxq_denom + per-block row maxima");
  m.def("blockmax_to_blocklists", &blockmax_to_blocklists, "block maxima -> KV-block lists");
}
