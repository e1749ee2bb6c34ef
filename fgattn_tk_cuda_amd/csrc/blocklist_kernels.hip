// Key mask -> KV-block mask -> KV-block index lists, for gfx950.
//
// The reference's pre-pass ends in per-key lists (include/mask_utils.cuh:273-302).  The block
// form of the same step: key block J (64 keys) of a mask row is kept when any of its keys
// c < kv_len is set,
//   MB[row, J] = OR_{c in 64J .. 64J+63, c < kv_len} M[row, c],
// and the kept block ids of a row are written in ascending order, followed by the caller's
// fill, with the count next to them - what the block-list attention kernel walks.
//
// Two sources: the bit-packed mask (one 64-bit word is one block; 1/32 of the bytes) and the
// reference's int32 vote mask (a pure HBM stream like the per-key compaction).  One wave owns
// one row; a lane stands for one block of a group of 64, so the rank of a kept block is a
// wave ballot and a bit count - no atomics, deterministic, ascending.
#include <math.h>

#include "common.h"
#include "dispatch.h"

namespace spattn {

constexpr int kBlockListMaxGrid = 2048;   // workgroups of 4 waves; further rows in further rounds

// Appends the kept blocks of one group of 64 (lane = block J0 + lane) to the row's list.
__device__ __forceinline__ void append_blocks(bool keep, int J, int nblk, int& count, int* __restrict__ dst,
                                              unsigned char* __restrict__ mrow, int max_blocks) {
  const unsigned long long b = __ballot(keep);
  const int pos = count + __builtin_amdgcn_mbcnt_hi((unsigned)(b >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)b, 0));
  if (keep && pos < max_blocks) dst[pos] = J;
  if (mrow != nullptr && J < nblk) mrow[J] = keep ? 1 : 0;
  count += __popcll(b);
}

__global__ __launch_bounds__(256) void packed_to_blocklists_kernel(int* __restrict__ blk_indices,
                                                                   int* __restrict__ blk_counts,
                                                                   unsigned char* __restrict__ blockmask,
                                                                   const uint32_t* __restrict__ packed, int rows,
                                                                   int mask_stride, int kv_len, int max_blocks) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int nblk = mask_stride >> 6;
  const int lim = kv_len < mask_stride ? kv_len : mask_stride;
  for (int row = blockIdx.x * 4 + wave; row < rows; row += gridDim.x * 4) {
    const u32x2* __restrict__ src = reinterpret_cast<const u32x2*>(packed + (size_t)row * (mask_stride >> 5));
    int* __restrict__ dst = blk_indices + (size_t)row * max_blocks;
    unsigned char* mrow = blockmask ? blockmask + (size_t)row * nblk : nullptr;
    int count = 0;
    for (int J0 = 0; J0 < nblk; J0 += 64) {
      const int J = J0 + lane;
      u32x2 w = {0u, 0u};
      if (J < nblk) w = src[J];
      unsigned long long bits = ((unsigned long long)w[1] << 32) | w[0];
      const int valid = lim - J * 64;   // keys of this block below the kv length
      if (valid <= 0) bits = 0;
      else if (valid < 64) bits &= (1ull << valid) - 1ull;
      append_blocks(bits != 0, J, nblk, count, dst, mrow, max_blocks);
    }
    if (lane == 0) blk_counts[row] = count;
  }
}

// int32 votes: a wave step covers 64 blocks = 4096 keys with 16 loads of 16 bytes per lane, all
// requested before the first is looked at.  Load u of lane l holds keys 256u + 4l .. +3 of the
// step, so block 4u + b of the step is lanes 16b .. 16b+15 of load u: one ballot per load, four
// 16-bit fields per ballot.
__global__ __launch_bounds__(256) void votes_to_blocklists_kernel(int* __restrict__ blk_indices,
                                                                  int* __restrict__ blk_counts,
                                                                  unsigned char* __restrict__ blockmask,
                                                                  const int* __restrict__ votes, int rows,
                                                                  int mask_stride, int kv_len, int max_blocks) {
  constexpr int U = 16;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int nblk = mask_stride >> 6;
  const int lim = kv_len < mask_stride ? kv_len : mask_stride;
  for (int row = blockIdx.x * 4 + wave; row < rows; row += gridDim.x * 4) {
    const int* __restrict__ src = votes + (size_t)row * mask_stride;
    int* __restrict__ dst = blk_indices + (size_t)row * max_blocks;
    unsigned char* mrow = blockmask ? blockmask + (size_t)row * nblk : nullptr;
    int count = 0;
    for (int J0 = 0; J0 < nblk; J0 += 64) {
      const int e_base = J0 * 64 + 4 * lane;
      i32x4 v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int e0 = e_base + u * 256;
        const i32x4 z = {0, 0, 0, 0};
        // mask_stride is a multiple of 4: a vector that starts inside the row stays inside it
        v[u] = (e0 < lim) ? __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(src + e0)) : z;
      }
      unsigned long long word = 0;   // bit j: block J0 + j has a key
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int e0 = e_base + u * 256;
        const bool f = (v[u][0] > 0 && e0 < lim) || (v[u][1] > 0 && e0 + 1 < lim) || (v[u][2] > 0 && e0 + 2 < lim) ||
                       (v[u][3] > 0 && e0 + 3 < lim);
        const unsigned long long b = __ballot(f);
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if ((b >> (16 * j)) & 0xffffull) word |= 1ull << (4 * u + j);
      }
      append_blocks((word >> lane) & 1ull, J0 + lane, nblk, count, dst, mrow, max_blocks);
    }
    if (lane == 0) blk_counts[row] = count;
  }
}

// Block maxima -> block lists: the threshold test of the mask pre-pass on the per-(row, key block)
// score maxima that the statistics sweep writes next to max_q and denom (blockmax[b][h][J][r], raw
// scores as bf16 rounded toward +inf: never below the true maximum).  Some key c of block J passes
//   exp2((s[r,c] - max_q[r]) sf) / denom[r] > thresh      (include/mask_utils.cuh:231-238)
// exactly when the block's maximum does, so
//   MB[I, J] = OR_{r in q-block I, r < seq} ( blockmax[J][r] > t[r] ),
//   t[r] = (log2 thresh + max_q[r] sf + log2 denom[r]) / sf   (the sweep kernel's per-row constant),
// holds every block of the threshold sweep's block mask - and, because of the rounding, possibly a
// block whose maximum lies within one bf16 step (a factor 2^-8) below t[r] - without a second pass
// over Q K^T: one read of 2 Sp Sp/64 bytes per head instead of 2 Sp^2 D flops.  One wave owns one
// q-block.  A lane holds two neighbouring rows (one 32-bit load); with 128-row q-blocks a load
// covers one key block, with 64-row q-blocks the two halves of the wave take two neighbouring key
// blocks.  32 key blocks are in flight per step, the votes of a block are one ballot (or half of
// one), kept blocks are appended 64 at a time as in the kernels above.
template <int QB>
__global__ __launch_bounds__(256) void blockmax_to_blocklists_kernel(int* __restrict__ blk_indices,
                                                                    int* __restrict__ blk_counts,
                                                                    unsigned char* __restrict__ blockmask,
                                                                    const uint16_t* __restrict__ blockmax,
                                                                    const float* __restrict__ max_q,
                                                                    const float* __restrict__ denom, float log2_thresh,
                                                                    float sf, int heads_total, int S, int Sp, int kv_len,
                                                                    int max_blocks, int bm_stride) {
  constexpr int BPL = 128 / QB;  // key blocks per load instruction (1 or 2)
  constexpr int U = 32 / BPL;    // loads in flight per wave: 32 key blocks per step
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int nqb = (S + QB - 1) / QB;
  const int rows = heads_total * nqb;
  const int nblk = (kv_len + 63) >> 6;    // key blocks that hold a key
  const int nbs = Sp >> 6;                // block rows of a head in blockmax
  const float inv_sf = 1.f / sf;
  const int rl = (QB == 128) ? lane : (lane & 31);   // this lane's row pair within the q-block
  const int jl = (QB == 128) ? 0 : (lane >> 5);      // this lane's key block within a load
  for (int row = blockIdx.x * 4 + wave; row < rows; row += gridDim.x * 4) {
    const int bh = row / nqb, I = row - bh * nqb;
    const int r0 = I * QB + 2 * rl;       // rows r0, r0 + 1 (Sp is even: both inside the padded row)
    float t[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      t[j] = __builtin_huge_valf();   // a row that does not exist, or has no key, never votes
      if (r0 + j < S) {
        const float mq = max_q[(size_t)bh * Sp + r0 + j];
        const float dn = denom[(size_t)bh * Sp + r0 + j];
        if (dn > 0.f) t[j] = (log2_thresh + (mq * sf + __log2f(dn))) * inv_sf;
      }
    }
    const uint16_t* __restrict__ src = blockmax + (size_t)bh * nbs * Sp + r0;
    int* __restrict__ dst = blk_indices + (size_t)row * max_blocks;
    unsigned char* mrow = blockmask ? blockmask + (size_t)row * bm_stride : nullptr;
    int count = 0;
    for (int J0 = 0; J0 < nblk; J0 += 64) {
      unsigned long long word = 0;   // bit j: block J0 + j is kept
#pragma unroll 1
      for (int u0 = 0; u0 < 64 && J0 + u0 < nblk; u0 += 32) {
        uint32_t x[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int J = J0 + u0 + BPL * u + jl;
          const int Jc = J < nblk ? J : nblk - 1;
          x[u] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(src + (size_t)Jc * Sp));
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const float lo = __builtin_bit_cast(float, x[u] << 16);
          const float hi = __builtin_bit_cast(float, x[u] & 0xffff0000u);
          const unsigned long long b = __ballot(lo > t[0] || hi > t[1]);
          const int J = J0 + u0 + BPL * u;
          if constexpr (BPL == 1) {
            if (b != 0ull && J < nblk) word |= 1ull << (u0 + u);
          } else {
            if ((uint32_t)b != 0u && J < nblk) word |= 1ull << (u0 + 2 * u);
            if ((uint32_t)(b >> 32) != 0u && J + 1 < nblk) word |= 1ull << (u0 + 2 * u + 1);
          }
        }
      }
      append_blocks((word >> lane) & 1ull, J0 + lane, bm_stride, count, dst, mrow, max_blocks);
    }
    // block-mask entries behind the last key block of the head
    if (mrow != nullptr)
      for (int J = ((nblk + 63) & ~63) + lane; J < bm_stride; J += 64) mrow[J] = 0;
    if (lane == 0) blk_counts[row] = count;
  }
}

static int blocklist_grid(int rows) {
  int grid = (rows + 3) / 4;
  return grid > kBlockListMaxGrid ? kBlockListMaxGrid : grid;
}

hipError_t run_packed_to_blocklists(int* blk_indices, int* blk_counts, unsigned char* blockmask, const uint32_t* packed,
                                    int rows, int mask_stride, int kv_len, int max_blocks, hipStream_t stream) {
  if (rows <= 0) return hipSuccess;
  hipLaunchKernelGGL(packed_to_blocklists_kernel, dim3(blocklist_grid(rows)), dim3(256), 0, stream, blk_indices,
                     blk_counts, blockmask, packed, rows, mask_stride, kv_len, max_blocks);
  return hipGetLastError();
}

hipError_t run_votes_to_blocklists(int* blk_indices, int* blk_counts, unsigned char* blockmask, const int* votes,
                                   int rows, int mask_stride, int kv_len, int max_blocks, hipStream_t stream) {
  if (rows <= 0) return hipSuccess;
  hipLaunchKernelGGL(votes_to_blocklists_kernel, dim3(blocklist_grid(rows)), dim3(256), 0, stream, blk_indices,
                     blk_counts, blockmask, votes, rows, mask_stride, kv_len, max_blocks);
  return hipGetLastError();
}

hipError_t run_blockmax_to_blocklists(int* blk_indices, int* blk_counts, unsigned char* blockmask, const uint16_t* blockmax,
                                      const float* max_q, const float* denom, float thresh, float sf, int qblk,
                                      int heads_total, int S, int kv_len, int max_blocks, hipStream_t stream) {
  const int nqb = (S + qblk - 1) / qblk;
  const int rows = heads_total * nqb;
  if (rows <= 0) return hipSuccess;
  const int Sp = ((S + 127) / 128) * 128;
  const float lt = thresh > 0.f ? log2f(thresh) : -__builtin_huge_valf();
  const int grid = blocklist_grid(rows);
  if (qblk == 128)
    hipLaunchKernelGGL(blockmax_to_blocklists_kernel<128>, dim3(grid), dim3(256), 0, stream, blk_indices, blk_counts, blockmask,
                       blockmax, max_q, denom, lt, sf, heads_total, S, Sp, kv_len, max_blocks, Sp >> 6);
  else
    hipLaunchKernelGGL(blockmax_to_blocklists_kernel<64>, dim3(grid), dim3(256), 0, stream, blk_indices, blk_counts, blockmask,
                       blockmax, max_q, denom, lt, sf, heads_total, S, Sp, kv_len, max_blocks, Sp >> 6);
  return hipGetLastError();
}

}  // namespace spattn
