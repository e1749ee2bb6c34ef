// Host-side entry points of the kernel translation units (internal, C++).
#pragma once
#include "common.h"

namespace spattn {

// attn_inst_tokens.hip / attn_inst_blocks.hip / attn_inst_dense.hip
hipError_t run_attn_tokens(const AttnParams& p, int D, int qblk, hipStream_t stream);
hipError_t run_attn_blocks(const AttnParams& p, int D, int qblk, hipStream_t stream);
hipError_t run_attn_dense(const AttnParams& p, int D, bool has_v, bool stats, hipStream_t stream);
// every instantiation's dynamic-LDS limit on the current device (idempotent)
hipError_t prepare_attn_tokens();
hipError_t prepare_attn_blocks();
hipError_t prepare_attn_dense();

// mask_kernels.hip
hipError_t run_booleanmask(void* out, int out_rows, float thresh, int mask_stride, const float* max_q,
                           const float* denom, const uint16_t* q, const uint16_t* k, int B, int H, int S, int D,
                           int kv_len, float scale, hipStream_t stream, const int* blk_idx = nullptr,
                           const int* blk_cnt = nullptr, int max_blocks = 0);
hipError_t run_compact(int* kv_indices, int* kv_num, const int* mask, int rows, int mask_stride, int kv_len,
                       hipStream_t stream);
hipError_t run_all_index(int* kv_indices, int* kv_num, int rows, int mask_stride, int seq, hipStream_t stream);

// bitmask_kernels.hip
hipError_t run_pack_mask(uint32_t* packed, const int* mask, int rows, int mask_stride, hipStream_t stream);
hipError_t run_packed_to_indexmask(int* kv_indices, int* kv_num, const uint32_t* packed, int rows, int mask_stride,
                                   int kv_len, hipStream_t stream);

// blocklist_kernels.hip
hipError_t run_packed_to_blocklists(int* blk_indices, int* blk_counts, unsigned char* blockmask, const uint32_t* packed,
                                    int rows, int mask_stride, int kv_len, int max_blocks, hipStream_t stream);
hipError_t run_votes_to_blocklists(int* blk_indices, int* blk_counts, unsigned char* blockmask, const int* votes,
                                   int rows, int mask_stride, int kv_len, int max_blocks, hipStream_t stream);

hipError_t run_blockmax_to_blocklists(int* blk_indices, int* blk_counts, unsigned char* blockmask, const uint16_t* blockmax,
                                      const float* max_q, const float* denom, float thresh, float sf, int qblk,
                                      int heads_total, int S, int kv_len, int max_blocks, hipStream_t stream);

// topk_kernels.hip
hipError_t run_topk_mask(int* kv_indices, int* kv_num, uint16_t* score, uint16_t* qmean, const uint16_t* q,
                         const uint16_t* k, int B, int H, int S, int D, int blk, int kv_len, int select_k,
                         int score_stride, int idx_stride, hipStream_t stream);

// order_kernels.hip
hipError_t run_qblock_order(int* order, const int* counts, int n, hipStream_t stream);

}  // namespace spattn
