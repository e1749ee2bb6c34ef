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
// One wave per (head, q-block).  A lane owns 8 neighbouring columns (one 16-byte load per
// row) of the rows r = j, j + P, j + 2P, ... with P = 512 / D row phases per wave-wide load;
// the P partial sums of a column are then added in the order of j.  The fp32 order of
// summation is thereby fixed: rows of one phase in increasing order, phases in increasing order.
// ------------------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(256) void qblock_mean_kernel(uint16_t* __restrict__ qmean, const uint16_t* __restrict__ q,
                                                           int S, int SB, int blk, int nblocks, float sqrt_d) {
  constexpr int CPR = D / 8;        // 16-byte chunks per row
  constexpr int P = 64 / CPR;       // row phases
  const int lane = threadIdx.x & 63;
  const int wb = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (wb >= nblocks) return;
  const int m = wb % SB;
  const int bh = wb / SB;
  const int c = lane % CPR;
  const int j = lane / CPR;
  const int r0 = m * blk;
  const int rows = (S - r0) < blk ? (S - r0) : blk;
  const uint16_t* src = q + ((size_t)bh * S + r0) * D + 8 * c;
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  constexpr int U = 4;   // loads in flight
  for (int r = j; r < rows; r += P * U) {
    u32x4 x[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const u32x4 z = {0, 0, 0, 0};
      x[u] = (r + P * u < rows) ? *reinterpret_cast<const u32x4*>(src + (size_t)(r + P * u) * D) : z;
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (r + P * u < rows) {
#pragma unroll
        for (int h = 0; h < 4; ++h) {
          acc[2 * h] += __builtin_bit_cast(float, x[u][h] << 16);
          acc[2 * h + 1] += __builtin_bit_cast(float, x[u][h] & 0xffff0000u);
        }
      }
  }
  float tot[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    tot[e] = __shfl(acc[e], c, 64);
#pragma unroll
    for (int ph = 1; ph < P; ++ph) tot[e] += __shfl(acc[e], ph * CPR + c, 64);
  }
  if (j == 0) {
    const float inv = 1.f / (float)rows;
    u32x4 out;
#pragma unroll
    for (int h = 0; h < 4; ++h) {
      const float a = bf16_to_f32(f32_to_bf16(tot[2 * h] * inv)) / sqrt_d;
      const float b2 = bf16_to_f32(f32_to_bf16(tot[2 * h + 1] * inv)) / sqrt_d;
      out[h] = pack_bf16(a, b2);
    }
    *reinterpret_cast<u32x4*>(qmean + ((size_t)bh * SB + m) * D + 8 * c) = out;
  }
}

// ------------------------------------------------------------------------------------
// score = qmean K^T.  A workgroup takes 64 q-blocks of one head (two 32-row A operands per
// k-step, in registers, the same in every wave) and a chunk of kKeysPerWg keys, 256 keys at
// a time: wave w multiplies the 64 keys 64w .. 64w+63 of those (two 32-key B operands, loaded
// HBM -> registers a few blocks ahead through rotating register sets; the product is tiny,
// what has to be covered is the latency of the loads).  Accumulator register 4j+i of block
// mb in lane (n, g) is q-block 32mb + 8j + 4g + i against key n.  The bf16 scores of the
// 64 x 256 piece are collected in LDS and leave row-wise, 512 contiguous bytes of a score row
// per half wave: stores in which every lane writes to a different row (rows are a power of
// two apart) ran an order of magnitude slower.
// Columns from kv_len to the next multiple of 8 receive unspecified values.
// ------------------------------------------------------------------------------------
constexpr int kKeysPerWg = 2048;
constexpr int kScorePitch = 512 + 16;   // bytes per staged row; rows 4 apart land 16 banks apart

template <int D>
__global__ __launch_bounds__(256) void qmean_scores_kernel(uint16_t* __restrict__ score,
                                                            const uint16_t* __restrict__ qmean,
                                                            const uint16_t* __restrict__ k, int S, int SB, int kv_len,
                                                            int score_stride) {
  constexpr int NT = D / 16;
  __shared__ __attribute__((aligned(16))) unsigned char tile[64 * kScorePitch];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
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
    key = key < kv_len ? key : kv_len - 1;   // keys past the end re-read the last one
#pragma unroll
    for (int t = 0; t < NT; ++t) kf[t] = *reinterpret_cast<const u32x4*>(kh + (size_t)key * D + 16 * t + 8 * g);
  };
  const int left = kv_len - key0;
  const int npiece_all = (left + 255) >> 8;
  const int npiece = npiece_all < kKeysPerWg / 256 ? npiece_all : kKeysPerWg / 256;

  // Step i of a wave is half (i & 1) of its 64 keys of piece i >> 1.
  constexpr int PF = (D == 64) ? 4 : 2;
  auto block_of = [&](int i) -> int { return 8 * (i >> 1) + 2 * wave + (i & 1); };
  u32x4 kf[PF][NT];
#pragma unroll
  for (int u = 0; u < PF - 1; ++u) load_keys(block_of(u), kf[u]);
  for (int i0 = 0; i0 < 2 * npiece; i0 += PF) {
#pragma unroll
    for (int u = 0; u < PF; ++u) {
      const int i = i0 + u;
      if (i < 2 * npiece) {   // wave-uniform and the same in every wave; a piece is never split (PF is even)
        const int half = u & 1;
        const int piece = i >> 1;
        load_keys(block_of(i + PF - 1), kf[(u + PF - 1) % PF]);
        f32x16 acc[2];
#pragma unroll
        for (int mb = 0; mb < 2; ++mb) {
          const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
          acc[mb] = zero;
#pragma unroll
          for (int t = 0; t < NT; ++t) acc[mb] = mfma32(qa[mb][t], kf[u][t], acc[mb]);
        }
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int row = 32 * mb + 8 * (r >> 2) + 4 * g + (r & 3);
            *reinterpret_cast<uint16_t*>(tile + row * kScorePitch + (64 * wave + 32 * half + ln) * 2) =
                f32_to_bf16(acc[mb][r]);
          }
        if (half == 1) {
          __syncthreads();
          // 32 lanes per row: 16 bytes each, rows tid / 32 + 8 j
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const int row = (tid >> 5) + 8 * j;
            const int col = 8 * (tid & 31);          // key within the piece
            const u32x4 v = *reinterpret_cast<const u32x4*>(tile + row * kScorePitch + 2 * col);
            if (m0 + row < SB && 256 * piece + col < left)
              *reinterpret_cast<u32x4*>(score + ((size_t)bh * SB + m0 + row) * score_stride + key0 + 256 * piece + col) = v;
          }
          __syncthreads();
        }
      }
    }
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

// The same for the two scores packed in one 32-bit word.
__device__ __forceinline__ uint32_t order_key2(uint32_t x) {
  const uint32_t sign = (x >> 15) & 0x00010001u;
  return x ^ (0x80008000u | (sign * 0x7fffu));
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
// Each bin is kept as SUBS partial counts (bin b at hist[b * SUBS .. b * SUBS + SUBS - 1]).
template <int SUBS>
__device__ __forceinline__ void find_bin(const unsigned* hist, int lane, int need, int& bin, int& above) {
  unsigned c[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    c[i] = 0;
#pragma unroll
    for (int s = 0; s < SUBS; ++s) c[i] += hist[(4 * lane + i) * SUBS + s];
  }
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
    find_bin<1>(hist, lane, want, b1, gt1);
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
    find_bin<1>(hist, lane, want - gt1, b2, gt2);
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

// The same selection with the row held in LDS: one workgroup per row reads its scores from
// HBM once, keeps them as 16-bit keys (2 bytes per key), and runs the passes out of LDS.  Wave w
// emits its contiguous part of the row; where its part of the list starts follows from the
// parts' counts of scores above and equal to the threshold.  Used while the row fits
// (kv_len <= kTopkLdsMaxKeys); longer rows take topk_select_kernel.
constexpr int kTopkLdsMaxKeys = 72000;
// A score row has few distinct exponents: most keys of a pass land in a handful of bins.  Every
// bin is therefore kept as 4 partial counts, one per lane & 3, next to each other (4
// different banks): the adds of a wave to one bin meet 16 to an address instead of 64.
constexpr int kTopkSubs = 4;
constexpr int kTopkThreads = 512;
constexpr int kTopkWaves = kTopkThreads / 64;
constexpr int kTopkLdsExtra = 256 * kTopkSubs * 4 + kTopkWaves * 2 * 4;   // histogram + per-wave counts

__global__ __launch_bounds__(kTopkThreads) void topk_select_lds_kernel(int* __restrict__ kv_indices, int* __restrict__ kv_num,
                                                               const uint16_t* __restrict__ score, int rows,
                                                               int score_stride, int kv_len, int select_k,
                                                               int idx_stride) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  const int nvec = (kv_len + 7) >> 3;
  u32x4* keys = reinterpret_cast<u32x4*>(smem_raw);                       // nvec vectors of 8 keys
  unsigned* hist = reinterpret_cast<unsigned*>(smem_raw + 16 * (size_t)nvec);
  int* wave_cnt = reinterpret_cast<int*>(hist + 256 * kTopkSubs);          // [waves][2]: above, equal
  constexpr int NTHR = kTopkThreads;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int sub = tid & (kTopkSubs - 1);
  int want = select_k < kv_len ? select_k : kv_len;
  want = want < idx_stride ? want : idx_stride;
  // wave w owns vectors [w * per, (w + 1) * per), per a multiple of 64
  const int per = ((nvec + NTHR - 1) / NTHR) << 6;
  const int v_lo = wave * per;
  const int v_hi = (v_lo + per) < nvec ? (v_lo + per) : nvec;

  auto key16 = [](const u32x4& x, int e) -> uint32_t {
    const uint32_t w = x[e >> 1];
    return (e & 1) ? (w >> 16) : (w & 0xffffu);
  };

  for (int row = blockIdx.x; row < rows; row += gridDim.x) {
    const u32x4* __restrict__ src = reinterpret_cast<const u32x4*>(score + (size_t)row * score_stride);
    int* __restrict__ dst = kv_indices + (size_t)row * idx_stride;
    if (want <= 0) {
      if (tid == 0) kv_num[row] = 0;
      continue;
    }
    for (int i = tid; i < 256 * kTopkSubs; i += NTHR) hist[i] = 0;
    __syncthreads();
    // Load, convert, pass 1 (high bytes).  Eight loads in flight per lane: the adds keep the
    // compiler from moving a load across them, and one load per trip would expose the memory
    // latency on every trip.  The up to 7 elements behind kv_len in the last vector get key
    // 0, the smallest, and are then treated like keys: with the largest indices of the row
    // they are the last candidates among equal keys, and want <= kv_len never reaches them.
    constexpr int U = 8;
    for (int v0 = tid; v0 < nvec; v0 += NTHR * U) {
      u32x4 xs[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int v = v0 + NTHR * u;
        const u32x4 z = {0, 0, 0, 0};
        xs[u] = v < nvec ? __builtin_nontemporal_load(src + v) : z;
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int v = v0 + NTHR * u;
        if (v < nvec) {
          u32x4 y;
#pragma unroll
          for (int h = 0; h < 4; ++h) y[h] = order_key2(xs[u][h]);
          if (8 * v + 8 > kv_len) {
#pragma unroll
            for (int h = 0; h < 4; ++h) {
              if (8 * v + 2 * h >= kv_len) y[h] &= 0xffff0000u;
              if (8 * v + 2 * h + 1 >= kv_len) y[h] &= 0x0000ffffu;
            }
          }
          keys[v] = y;
#pragma unroll
          for (int e = 0; e < 8; ++e) atomicAdd(&hist[(key16(y, e) >> 8) * kTopkSubs + sub], 1u);
        }
      }
    }
    __syncthreads();
    int b1, gt1;
    find_bin<kTopkSubs>(hist, lane, want, b1, gt1);   // every wave finds the same bin
    __syncthreads();
    for (int i = tid; i < 256 * kTopkSubs; i += NTHR) hist[i] = 0;
    __syncthreads();
    // pass 2 (low bytes under high byte b1)
    for (int v = tid; v < nvec; v += NTHR) {
      const u32x4 y = keys[v];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const uint32_t key = key16(y, e);
        if ((int)(key >> 8) == b1) atomicAdd(&hist[(key & 255u) * kTopkSubs + sub], 1u);
      }
    }
    __syncthreads();
    int b2, gt2;
    find_bin<kTopkSubs>(hist, lane, want - gt1, b2, gt2);
    const uint32_t T = ((uint32_t)b1 << 8) | (uint32_t)b2;
    const int r = want - gt1 - gt2;
    // counts of this wave's part
    int cg = 0, ce = 0;
    for (int v = v_lo + lane; v < v_hi; v += 64) {
      const u32x4 y = keys[v];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const uint32_t key = key16(y, e);
        cg += key > T ? 1 : 0;
        ce += key == T ? 1 : 0;
      }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      cg += __shfl_xor(cg, off, 64);
      ce += __shfl_xor(ce, off, 64);
    }
    if (lane == 0) {
      wave_cnt[2 * wave] = cg;
      wave_cnt[2 * wave + 1] = ce;
    }
    __syncthreads();
    int gt_start = 0, eq_seen = 0;
    for (int u = 0; u < wave; ++u) {
      gt_start += wave_cnt[2 * u];
      eq_seen += wave_cnt[2 * u + 1];
    }
    int out_pos = gt_start + (eq_seen < r ? eq_seen : r);
    // ordered emit of this wave's part
    for (int v0 = v_lo; v0 < v_hi; v0 += 64) {
      const int v = v0 + lane;
      unsigned gt = 0, eq = 0;
      if (v < v_hi) {
        const u32x4 y = keys[v];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const uint32_t key = key16(y, e);
          gt |= (key > T ? 1u : 0u) << e;
          eq |= (key == T ? 1u : 0u) << e;
        }
      }
      int eq_before, eq_total;
      lane_prefix4(__popc(eq), eq_before, eq_total);
      int keep = r - (eq_seen + eq_before);
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
    if (tid == 0) kv_num[row] = want;
    __syncthreads();   // the row buffer and the counts are reused
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
    hipLaunchKernelGGL(qblock_mean_kernel<64>, dim3((rows + 3) / 4), dim3(256), 0, stream, qmean, q, S, SB, blk, rows,
                       sqrt_d);
  else
    hipLaunchKernelGGL(qblock_mean_kernel<128>, dim3((rows + 3) / 4), dim3(256), 0, stream, qmean, q, S, SB, blk, rows,
                       sqrt_d);
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
  if (kv_len <= kTopkLdsMaxKeys) {
    const int lds = 16 * ((kv_len + 7) / 8) + kTopkLdsExtra;
    static bool attr_set[kMaxDevices] = {};
    e = raise_lds_limit(reinterpret_cast<const void*>(topk_select_lds_kernel),
                        16 * (kTopkLdsMaxKeys / 8) + kTopkLdsExtra, attr_set);
    if (e != hipSuccess) return e;
    const int grid = rows < 8192 ? rows : 8192;
    hipLaunchKernelGGL(topk_select_lds_kernel, dim3(grid), dim3(kTopkThreads), lds, stream, kv_indices, kv_num, score, rows,
                       score_stride, kv_len, select_k, idx_stride);
    return hipGetLastError();
  }
  int grid = (rows + 3) / 4;
  if (grid > 4096) grid = 4096;
  hipLaunchKernelGGL(topk_select_kernel, dim3(grid), dim3(256), 0, stream, kv_indices, kv_num, score, rows,
                     score_stride, kv_len, select_k, idx_stride);
  return hipGetLastError();
}

}  // namespace spattn
