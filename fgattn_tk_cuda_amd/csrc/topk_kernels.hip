// Top-k mask generator: per q-block the select_k keys with the largest
//   (mean of the block's query rows / sqrt(D)) . key
// Reference: python/spattn/mask_utils.py:389-417 (qk_topkmask_indices), which runs, in bf16,
//   qmean = q.view(B,H,SB,BLOCKSZ,D).mean(3) (the last block over its remaining rows)   :390-405
//   score = einsum('bhmd,bhnd->bhmn', qmean * 1. / D**0.5, k)                             :407-410
//   torch.topk(score, select_k, dim=-1, sorted=True).indices                              :412-413
// Three kernels, one [SB x D].[D x S] product per head instead of the two S^2 sweeps of the
// threshold pre-pass:
//   qblock_mean_kernel   q -> qmean [B,H,SB,D] bf16 (fp32 sum, * 1/rows, bf16, / sqrt(D), bf16)
//   qmean_scores_kernel  qmean, k -> score [B,H,SB,score_stride] bf16 (MFMA, fp32 accumulate)
//   topk_select_kernel   score -> per row the select_k largest, as an ASCENDING key list
// The selection is a two-level radix select on the 16 score bits (two 256-bin histograms)
// followed by an ordered emit; among equal scores the lower key index wins.  The reference
// returns the same keys ordered by descending score (ties in whatever order torch.topk
// leaves them); the gathered attention that consumes the list does not depend on the order.
#include "common.h"
#include "dispatch.h"

namespace spattn {

__device__ __forceinline__ float bf16_to_f32(uint16_t x) { return __builtin_bit_cast(float, (uint32_t)x << 16); }
__device__ __forceinline__ uint16_t f32_to_bf16(float x) { return (uint16_t)(pack_bf16(x, 0.f) & 0xffffu); }

// ------------------------------------------------------------------------------------
// One workgroup of D lanes per (head, q-block); lane d sums column d over the rows.
// ------------------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(D) void qblock_mean_kernel(uint16_t* __restrict__ qmean, const uint16_t* __restrict__ q,
                                                         int S, int SB, int blk, float sqrt_d) {
  const int m = blockIdx.x % SB;
  const int bh = blockIdx.x / SB;
  const int d = threadIdx.x;
  const int r0 = m * blk;
  const int rows = (S - r0) < blk ? (S - r0) : blk;
  const uint16_t* src = q + ((size_t)bh * S + r0) * D + d;
  float sum = 0.f;
  for (int r = 0; r < rows; ++r) sum += bf16_to_f32(src[(size_t)r * D]);
  const float mean = bf16_to_f32(f32_to_bf16(sum * (1.f / (float)rows)));
  qmean[((size_t)bh * SB + m) * D + d] = f32_to_bf16(mean / sqrt_d);
}

// ------------------------------------------------------------------------------------
// score = qmean K^T.  A workgroup takes 64 q-blocks (two 32-row A operands per k-step, in
// registers) and a chunk of kKeysPerWg keys; each wave walks its own 32-key blocks with the
// keys as the B operand, loaded HBM -> registers one block ahead.  Accumulator register
// 4j+i of block mb in lane (n, g) is q-block 32mb + 8j + 4g + i against key n: for one
// register the 32 lanes of a half wave store 64 contiguous bytes.
// ------------------------------------------------------------------------------------
constexpr int kKeysPerWg = 4096;

template <int D>
__global__ __launch_bounds__(256) void qmean_scores_kernel(uint16_t* __restrict__ score,
                                                            const uint16_t* __restrict__ qmean,
                                                            const uint16_t* __restrict__ k, int S, int SB, int kv_len,
                                                            int score_stride) {
  constexpr int NT = D / 16;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int ln = lane & 31;
  const int g = lane >> 5;
  const int bh = blockIdx.z;
  const int m0 = blockIdx.y * 64;
  const int key0 = blockIdx.x * kKeysPerWg;
  const uint16_t* qh = qmean + (size_t)bh * SB * D;
  const uint16_t* kh = k + (size_t)bh * S * D;

  u32x4 qa[2][NT];
#pragma unroll
  for (int mb = 0; mb < 2; ++mb) {
    const int row = m0 + 32 * mb + ln;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const u32x4 z = {0, 0, 0, 0};
      qa[mb][t] = (row < SB) ? *reinterpret_cast<const u32x4*>(qh + (size_t)row * D + 16 * t + 8 * g) : z;
    }
  }
  auto load_keys = [&](int kb, u32x4 (&kf)[NT]) {
    int key = key0 + kb * 32 + ln;
    key = key < kv_len ? key : kv_len - 1;   // keys past the end re-read the last one; they are not stored
#pragma unroll
    for (int t = 0; t < NT; ++t) kf[t] = *reinterpret_cast<const u32x4*>(kh + (size_t)key * D + 16 * t + 8 * g);
  };
  const int nkb_all = (kv_len - key0 + 31) >> 5;
  const int nkb = nkb_all < kKeysPerWg / 32 ? nkb_all : kKeysPerWg / 32;
  u32x4 cur[NT], nxt[NT];
  if (wave < nkb) load_keys(wave, cur);
  for (int kb = wave; kb < nkb; kb += 4) {
    load_keys(kb + 4, nxt);
    f32x16 acc[2];
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) {
      const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      acc[mb] = zero;
#pragma unroll
      for (int t = 0; t < NT; ++t) acc[mb] = mfma32(qa[mb][t], cur[t], acc[mb]);
    }
    const int key = key0 + kb * 32 + ln;
    if (key < kv_len) {
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = m0 + 32 * mb + 8 * (r >> 2) + 4 * g + (r & 3);
          if (row < SB) score[((size_t)bh * SB + row) * score_stride + key] = f32_to_bf16(acc[mb][r]);
        }
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) cur[t] = nxt[t];
  }
}

// ------------------------------------------------------------------------------------
// Selection, one wave per score row.  bf16 bits map to 16-bit keys whose unsigned order is
// the order of the scores.  Pass 1 counts the high bytes and finds the byte b1 that holds
// the select_k-th largest score, pass 2 counts the low bytes among the scores with high
// byte b1: that fixes the threshold key T, how many scores lie above it and how many of
// those equal to it are still needed (r).  Pass 3 walks the row in key order and emits the
// keys with a score above T and the first r with a score equal to T.  The row is re-read
// in every pass (it is 2 bytes per key and stays in L2).
// ------------------------------------------------------------------------------------
__device__ __forceinline__ uint32_t order_key(uint32_t bits) {
  return (bits & 0x8000u) ? (~bits & 0xffffu) : (bits | 0x8000u);
}

// Exclusive prefix sum over the lanes of per-lane counts below 16, and their total: one
// ballot per bit of the count.
__device__ __forceinline__ void lane_prefix4(int cnt, int& before, int& total) {
  before = 0;
  total = 0;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const unsigned long long m = __ballot((cnt >> w) & 1);
    before += (int)__builtin_amdgcn_mbcnt_hi((unsigned)(m >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)m, 0)) << w;
    total += __popcll(m) << w;
  }
}

// hist[256] holds counts; returns the largest bin b with  sum_{j >= b} hist[j] >= need  and
// the count strictly above it.  need >= 1 and need <= sum of all bins.
__device__ __forceinline__ void find_bin(const unsigned* hist, int lane, int need, int& bin, int& above) {
  unsigned c[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) c[i] = hist[4 * lane + i];
  int own = (int)(c[0] + c[1] + c[2] + c[3]);
  int s = own;   // becomes the sum over lanes >= this one
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int t = __shfl_down(s, off, 64);
    if (lane + off < 64) s += t;
  }
  const unsigned long long m = __ballot(s >= need);
  const int L = 63 - __builtin_clzll(m);        // m != 0 because need <= total
  int a = s - own;                              // strictly above this lane's bins
  int b = 4 * lane + 3;
#pragma unroll
  for (int i = 3; i >= 0; --i) {
    if (a + (int)c[i] >= need) { b = 4 * lane + i; break; }
    a += (int)c[i];
  }
  bin = __shfl(b, L, 64);
  above = __shfl(a, L, 64);
}

__global__ __launch_bounds__(256) void topk_select_kernel(int* __restrict__ kv_indices, int* __restrict__ kv_num,
                                                           const uint16_t* __restrict__ score, int rows,
                                                           int score_stride, int kv_len, int select_k,
                                                           int idx_stride) {
  __shared__ unsigned hist_all[4][256];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  unsigned* hist = hist_all[wave];
  const int nvec = (kv_len + 7) >> 3;   // 16-byte vectors (8 scores) that hold keys below kv_len
  int want = select_k < kv_len ? select_k : kv_len;
  want = want < idx_stride ? want : idx_stride;

  for (int row = blockIdx.x * 4 + wave; row < rows; row += gridDim.x * 4) {
    const u32x4* __restrict__ src = reinterpret_cast<const u32x4*>(score + (size_t)row * score_stride);
    int* __restrict__ dst = kv_indices + (size_t)row * idx_stride;
    if (want <= 0) {
      if (lane == 0) kv_num[row] = 0;
      continue;
    }
    // the 16-bit keys of vector v, element e (key index 8v + e); keys past kv_len are skipped by the callers
    auto key_of = [](const u32x4& x, int e) -> uint32_t {
      const uint32_t w = x[e >> 1];
      return order_key((e & 1) ? (w >> 16) : (w & 0xffffu));
    };
    auto clear_hist = [&]() {
#pragma unroll
      for (int i = 0; i < 4; ++i) hist[64 * i + lane] = 0;
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
    };
    auto hist_done = [&]() {
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      __builtin_amdgcn_wave_barrier();
    };

    // pass 1: high bytes
    clear_hist();
    for (int v = lane; v < nvec; v += 64) {
      const u32x4 x = src[v];
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (8 * v + e < kv_len) atomicAdd(&hist[key_of(x, e) >> 8], 1u);
    }
    hist_done();
    int b1, gt1;
    find_bin(hist, lane, want, b1, gt1);
    __builtin_amdgcn_wave_barrier();

    // pass 2: low bytes of the scores whose high byte is b1
    clear_hist();
    for (int v = lane; v < nvec; v += 64) {
      const u32x4 x = src[v];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const uint32_t key = key_of(x, e);
        if (8 * v + e < kv_len && (int)(key >> 8) == b1) atomicAdd(&hist[key & 255u], 1u);
      }
    }
    hist_done();
    int b2, gt2;
    find_bin(hist, lane, want - gt1, b2, gt2);
    __builtin_amdgcn_wave_barrier();
    const uint32_t T = ((uint32_t)b1 << 8) | (uint32_t)b2;
    const int r = want - gt1 - gt2;   // scores equal to T that are still needed, in key order

    // pass 3: ordered emit
    int out_pos = 0, eq_seen = 0;
    for (int v0 = 0; v0 < nvec; v0 += 64) {
      const int v = v0 + lane;
      unsigned gt = 0, eq = 0;
      if (v < nvec) {
        const u32x4 x = src[v];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const uint32_t key = key_of(x, e);
          if (8 * v + e < kv_len) {
            gt |= (key > T ? 1u : 0u) << e;
            eq |= (key == T ? 1u : 0u) << e;
          }
        }
      }
      int eq_before, eq_total;
      lane_prefix4(__popc(eq), eq_before, eq_total);
      int keep = r - (eq_seen + eq_before);       // how many of this lane's equal scores are taken
      keep = keep < 0 ? 0 : keep;
      unsigned eq_kept = 0;
      while (eq && keep > 0) {
        eq_kept |= eq & (0u - eq);
        eq &= eq - 1;
        --keep;
      }
      unsigned sel = gt | eq_kept;
      int before, total;
      lane_prefix4(__popc(sel), before, total);
      int pos = out_pos + before;
      while (sel) {
        dst[pos++] = 8 * v + __builtin_ctz(sel);
        sel &= sel - 1;
      }
      out_pos += total;
      eq_seen += eq_total;
    }
    if (lane == 0) kv_num[row] = out_pos;
  }
}

hipError_t run_topk_mask(int* kv_indices, int* kv_num, uint16_t* score, uint16_t* qmean, const uint16_t* q,
                         const uint16_t* k, int B, int H, int S, int D, int blk, int kv_len, int select_k,
                         int score_stride, int idx_stride, hipStream_t stream) {
  const int SB = (S + blk - 1) / blk;
  const int rows = B * H * SB;
  if (rows <= 0) return hipSuccess;
  const float sqrt_d = (float)__builtin_sqrt((double)D);
  if (D == 64)
    hipLaunchKernelGGL(qblock_mean_kernel<64>, dim3(rows), dim3(64), 0, stream, qmean, q, S, SB, blk, sqrt_d);
  else
    hipLaunchKernelGGL(qblock_mean_kernel<128>, dim3(rows), dim3(128), 0, stream, qmean, q, S, SB, blk, sqrt_d);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  if (kv_len > 0) {
    const dim3 grid((kv_len + kKeysPerWg - 1) / kKeysPerWg, (SB + 63) / 64, B * H);
    if (D == 64)
      hipLaunchKernelGGL(qmean_scores_kernel<64>, grid, dim3(256), 0, stream, score, qmean, k, S, SB, kv_len,
                         score_stride);
    else
      hipLaunchKernelGGL(qmean_scores_kernel<128>, grid, dim3(256), 0, stream, score, qmean, k, S, SB, kv_len,
                         score_stride);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  int grid = (rows + 3) / 4;
  if (grid > 4096) grid = 4096;
  hipLaunchKernelGGL(topk_select_kernel, dim3(grid), dim3(256), 0, stream, kv_indices, kv_num, score, rows,
                     score_stride, kv_len, select_k, idx_stride);
  return hipGetLastError();
}

}  // namespace spattn
