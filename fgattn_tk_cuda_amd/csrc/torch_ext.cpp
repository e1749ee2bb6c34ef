// PyTorch operator binding: registers the seven ops of the reference extension in the
// `cuda_attn` namespace (python/extension.cpp:81-358) and exposes the same seven functions
// as a pybind module (python/extension.cpp:362-370).  Host code only: every op checks its
// arguments and forwards raw device pointers to the C ABI of libspattn_hip.so on the
// current HIP stream.  Unlike the reference, unsupported inputs raise instead of silently
// returning (python/cuda_attn.cu:33-36 under -DNDEBUG).
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/extension.h>

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

}  // namespace

void full_attn(torch::Tensor o, torch::Tensor q, torch::Tensor k, torch::Tensor v) {
  check_bhsd(q, "q", q);
  check_bhsd(k, "k", q);
  check_bhsd(v, "v", q);
  check_bhsd(o, "o", q);
  const DeviceGuard guard(q.device());
  check_status(spattn_full_attn(o.data_ptr(), nullptr, q.data_ptr(), k.data_ptr(), v.data_ptr(), (int)q.size(0),
                                (int)q.size(1), (int)q.size(2), (int)q.size(3), 0, 0.f, cur_stream()),
               "full_attn");
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

void sp_attn(torch::Tensor o, torch::Tensor q, torch::Tensor k, torch::Tensor v, torch::Tensor kv_indices,
             torch::Tensor kv_num_indices) {
  check_bhsd(q, "q", q);
  check_bhsd(k, "k", q);
  check_bhsd(v, "v", q);
  check_bhsd(o, "o", q);
  check_aux(kv_indices, "kv_indices", at::kInt, q);
  check_aux(kv_num_indices, "kv_num_indices", at::kInt, q);
  TORCH_CHECK(kv_indices.dim() == 4 && kv_indices.size(0) == q.size(0) && kv_indices.size(1) == q.size(1),
              "kv_indices must be [B,H,SB,mask_stride]");
  const int qblk = infer_qblk(q.size(2), kv_indices.size(2));
  // the reference does not check the shape of kv_num_indices, only its element order
  TORCH_CHECK(kv_num_indices.numel() == q.size(0) * q.size(1) * kv_indices.size(2), "kv_num_indices must have B*H*SB entries");
  const DeviceGuard guard(q.device());
  // Threshold masks give lists of very different lengths: the q-blocks are handed to the
  // workgroups longest list first (the order is a small device tensor from torch's caching
  // allocator; lists within a factor of two of each other keep the default order).
  torch::Tensor order = torch::empty({kv_num_indices.numel()}, kv_num_indices.options());
  check_status(spattn_qblock_order(order.data_ptr<int>(), kv_num_indices.data_ptr<int>(), (int)kv_num_indices.numel(),
                                   cur_stream()),
               "sp_attn (work order)");
  check_status(spattn_sp_attn_ordered(o.data_ptr(), nullptr, q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                      kv_indices.data_ptr<int>(), kv_num_indices.data_ptr<int>(), order.data_ptr<int>(),
                                      (int)kv_indices.size(3), qblk, (int)q.size(0), (int)q.size(1), (int)q.size(2),
                                      (int)q.size(3), 0, 0.f, cur_stream()),
               "sp_attn");
}

void fullattn_maxq_denom(torch::Tensor o, torch::Tensor o_max_q, torch::Tensor o_denom, torch::Tensor q, torch::Tensor k,
                         torch::Tensor v) {
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
                                          (int)q.size(3), 0, 0.f, cur_stream()),
               "fullattn_maxq_denom");
}

void maxq_denom(torch::Tensor o_max_q, torch::Tensor o_denom, torch::Tensor q, torch::Tensor k) {
  check_bhsd(q, "q", q);
  check_bhsd(k, "k", q);
  check_aux(o_max_q, "o_max_q", at::kFloat, q);
  check_aux(o_denom, "o_denom", at::kFloat, q);
  const int64_t need = q.size(0) * q.size(1) * padded128(q.size(2));
  TORCH_CHECK(o_max_q.numel() == need && o_denom.numel() == need, "o_max_q / o_denom must be [B,H,1,128*ceil(S/128)]");
  const DeviceGuard guard(q.device());
  check_status(spattn_maxq_denom(o_max_q.data_ptr<float>(), o_denom.data_ptr<float>(), q.data_ptr(), k.data_ptr(),
                                 (int)q.size(0), (int)q.size(1), (int)q.size(2), (int)q.size(3), 0, 0.f, cur_stream()),
               "maxq_denom");
}

void booleanmask_128(torch::Tensor booleanmask, torch::Tensor o_max_q, torch::Tensor o_denom, torch::Tensor q,
                     torch::Tensor k, double threshold) {
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
                                      (int)q.size(0), (int)q.size(1), (int)q.size(2), (int)q.size(3), 0, 0.f, cur_stream()),
               "booleanmask_128");
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
}
