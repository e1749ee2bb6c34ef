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
//   topk_select_reg_kernel / topk_select_kernel   score -> per row the select_k largest, as an ASCENDING key list
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
__global__ __launch_bounds__(256, 2) void qmean_scores_kernel(uint16_t* __restrict__ score,
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
  typedef short i16x2 __attribute__((ext_vector_type(2)));
  const i16x2 sign = __builtin_bit_cast(i16x2, x) >> 15;   // 0xffff under a set sign bit
  return x ^ (0x80008000u | __builtin_bit_cast(uint32_t, sign));
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

// ------------------------------------------------------------------------------------
// The same selection with the row held in registers: one workgroup of 512 lanes per row, every
// lane keeps VPL 16-byte vectors (8 keys each) of the row as packed 16-bit keys from the one HBM
// read to the emit.  Wave w owns the vectors [64 VPL w, 64 VPL (w + 1)), lane l of it the
// vectors 64 VPL w + 64 u + l: a wave-wide load is 1 KB contiguous, and (wave, u, lane, element)
// is the key order.  LDS holds only the histogram: every bin as 32 partial counts, one per
// lane & 31, next to each other - a wave's adds to one bin go to 32 different banks and meet at
// most two to an address, however few bins the row's exponents fill.  Two keys are handled per
// instruction wherever the 16-bit packed forms allow it (key order, pass-2 bin, the
// above / equal flags of the emit, which one dot product per register turns into a bit mask),
// and the lane prefix sums of the emit run on counts packed two to a register.
// ------------------------------------------------------------------------------------
constexpr int kRegThreads = 512;
constexpr int kRegSlots = 32;
constexpr int kRegSlotShift = 5;
constexpr int kRegMaxVpl = 18;
constexpr int kRegMaxKeys = kRegThreads * kRegMaxVpl * 8;   // 73728

__device__ __forceinline__ uint32_t pk_sub_sat_u16(uint32_t a, uint32_t b) {
  uint32_t d;
  asm("v_pk_sub_u16 %0, %1, %2 clamp" : "=v"(d) : "v"(a), "v"(b));
  return d;
}
__device__ __forceinline__ uint32_t pk_sub_u16(uint32_t a, uint32_t b) {
  uint32_t d;
  asm("v_pk_sub_u16 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
  return d;
}
__device__ __forceinline__ uint32_t pk_min_u16(uint32_t a, uint32_t b) {
  uint32_t d;
  asm("v_pk_min_u16 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
  return d;
}
__device__ __forceinline__ uint32_t pk_mad_u16(uint32_t a, uint32_t b, uint32_t c) {
  uint32_t d;
  asm("v_pk_mad_u16 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
  return d;
}
// adds 1 to the 32-bit LDS word at a byte address
__device__ __forceinline__ void lds_add_one(uint32_t byte_addr) {
  __hip_atomic_fetch_add((SPATTN_LDS unsigned*)(uintptr_t)byte_addr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
// acc + lo16(flags) * lo16(weights) + hi16(flags) * hi16(weights)
__device__ __forceinline__ uint32_t dot2_u16(uint32_t flags, uint32_t weights, uint32_t acc) {
  typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
  return __builtin_amdgcn_udot2(__builtin_bit_cast(u16x2, flags), __builtin_bit_cast(u16x2, weights), acc, false);
}
// Inclusive prefix sum over the 64 lanes (fields packed in x must not carry into each other).
__device__ __forceinline__ uint32_t lane_scan(uint32_t x) {
  int v = (int)x;
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, true);   // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, true);   // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, true);   // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, true);   // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);  // row_bcast:15 into rows 1 and 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);  // row_bcast:31 into rows 2 and 3
  return (uint32_t)v;
}

// find_bin on plain counts with the bins dealt to the lanes from the top (lane l holds bins
// 255 - 4l .. 252 - 4l): the sum over the bins at and above a lane's own is then an inclusive
// prefix sum over the lanes, six DPP adds instead of six cross-lane reads through LDS.
__device__ __forceinline__ void find_bin_top_down(const unsigned* tot, int lane, int need, int& bin, int& above) {
  const u32x4 c = *reinterpret_cast<const u32x4*>(tot + 252 - 4 * lane);   // c[3] is the highest bin of the four
  const int own = (int)(c[0] + c[1] + c[2] + c[3]);
  const int s = (int)lane_scan((uint32_t)own);
  const unsigned long long m = __ballot(s >= need);           // m != 0 because need <= total
  const int L = __builtin_ctzll(m);
  int a = s - own;                                            // strictly above this lane's bins
  int b = 252 - 4 * lane;
#pragma unroll
  for (int i = 3; i >= 0; --i) {
    if (a + (int)c[i] >= need) { b = 252 - 4 * lane + i; break; }
    a += (int)c[i];
  }
  bin = __builtin_amdgcn_readlane(b, L);
  above = __builtin_amdgcn_readlane(a, L);
}

// Sums the 32 partial counts of every bin into tot[256], clears what it read (and the overflow
// bin when asked), and finds the bin that holds the need-th largest key.  Two barriers inside;
// the caller has put one behind the last add.
template <bool CLEAR_OVERFLOW>
__device__ __forceinline__ void reduce_and_find(unsigned* hist, unsigned* tot, int tid, int lane, int need, int& bin,
                                                int& above) {
  u32x4* p = reinterpret_cast<u32x4*>(hist + (tid >> 1) * kRegSlots + (tid & 1) * (kRegSlots / 2));
  const u32x4 zero = {0, 0, 0, 0};
  unsigned s = 0;
  // a lane's 64 bytes start 16 banks from its neighbour's: neighbouring pairs of lanes take their
  // four 16-byte pieces in rotated order, so that 16 lanes cover all banks in every step
#pragma unroll
  for (int j = 0; j < kRegSlots / 8; ++j) {
    const int jj = (j + (tid >> 1)) & (kRegSlots / 8 - 1);
    const u32x4 c = p[jj];
    p[jj] = zero;
    s += c[0] + c[1] + c[2] + c[3];
  }
  s += __shfl_xor(s, 1, 64);
  if (!(tid & 1)) tot[tid >> 1] = s;
  if (CLEAR_OVERFLOW && tid < kRegSlots) hist[256 * kRegSlots + tid] = 0;
  __syncthreads();
  find_bin_top_down(tot, lane, need, bin, above);
  __syncthreads();   // tot is rewritten by the next reduction
}

template <int VPL>
__global__ __launch_bounds__(kRegThreads) __attribute__((amdgpu_waves_per_eu(VPL <= 8 ? 6 : (VPL <= 12 ? 4 : 2)))) void topk_select_reg_kernel(int* __restrict__ kv_indices, int* __restrict__ kv_num,
                                                                     const uint16_t* __restrict__ score, int rows,
                                                                     int score_stride, int kv_len, int select_k,
                                                                     int idx_stride) {
  __shared__ __attribute__((aligned(16))) unsigned hist[257 * kRegSlots];   // bin 256: pass-2 keys outside the pass-1 bin
  __shared__ __attribute__((aligned(16))) unsigned tot[256];
  __shared__ unsigned wave_cnt[kRegThreads / 64];
  constexpr int NP = (VPL + 1) / 2;   // registers of counts packed two to a register
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nvec = (kv_len + 7) >> 3;
  int want = select_k < kv_len ? select_k : kv_len;
  want = want < idx_stride ? want : idx_stride;
  const int vbase = wave * (VPL * 64) + lane;
  // the vector that holds key kv_len - 1, when elements behind kv_len share it: its wave, slot and lane
  const int tail_wave = (kv_len & 7) ? (nvec - 1) / (VPL * 64) : -1;
  const int tail_u = ((nvec - 1) % (VPL * 64)) >> 6;
  const int tail_lane = (nvec - 1) & 63;
  unsigned* const my_hist = hist + (lane & (kRegSlots - 1));
  SPATTN_LDS unsigned* const my_hist_lds = (SPATTN_LDS unsigned*)my_hist;
  const uint32_t one2 = 0x00010001u;

  {
    const u32x4 zero = {0, 0, 0, 0};
    for (int i = tid; i < 257 * kRegSlots / 4; i += kRegThreads) reinterpret_cast<u32x4*>(hist)[i] = zero;
  }
  for (int row = blockIdx.x; row < rows; row += gridDim.x) {
    const u32x4* __restrict__ src = reinterpret_cast<const u32x4*>(score + (size_t)row * score_stride);
    int* __restrict__ dst = kv_indices + (size_t)row * idx_stride;
    if (want <= 0) {
      if (tid == 0) kv_num[row] = 0;
      continue;
    }
    // Vectors behind the row hold the bit pattern whose key is 0, the smallest; so do the up to 7
    // elements behind kv_len in the last vector.  They count as keys: with the largest indices of
    // the row they are the last candidates among equal keys, and want <= kv_len never reaches them.
    u32x4 y[VPL];
    if ((wave + 1) * (VPL * 64) <= nvec) {
#pragma unroll
      for (int u = 0; u < VPL; ++u) y[u] = __builtin_nontemporal_load(src + vbase + 64 * u);
    } else {
#pragma unroll
      for (int u = 0; u < VPL; ++u) {
        const int v = vbase + 64 * u;
        const u32x4 lowest = {~0u, ~0u, ~0u, ~0u};
        y[u] = v < nvec ? __builtin_nontemporal_load(src + v) : lowest;
      }
    }
#pragma unroll
    for (int u = 0; u < VPL; ++u)
#pragma unroll
      for (int h = 0; h < 4; ++h) y[u][h] = order_key2(y[u][h]);
    if (wave == tail_wave) {
      const int left = kv_len & 7;   // elements of the vector that are keys
#pragma unroll
      for (int u = 0; u < VPL; ++u)
        if (u == tail_u) {
#pragma unroll
          for (int h = 0; h < 4; ++h) {
            const uint32_t keep = 2 * h + 1 < left ? ~0u : (2 * h < left ? 0x0000ffffu : 0u);
            y[u][h] &= lane == tail_lane ? keep : ~0u;
          }
        }
    }
    __syncthreads();   // the histogram is clear
    // pass 1: high bytes
#pragma unroll
    for (int u = 0; u < VPL; ++u)
#pragma unroll
      for (int h = 0; h < 4; ++h) {
        const uint32_t w = y[u][h];
        atomicAdd(my_hist + ((w >> 24) << kRegSlotShift), 1u);
        atomicAdd(my_hist + (((w >> 8) & 0xffu) << kRegSlotShift), 1u);
      }
    __syncthreads();
    int b1, gt1;
    reduce_and_find<false>(hist, tot, tid, lane, want, b1, gt1);
    // pass 2: low bytes under high byte b1; every other key goes to bin 256
    {
      const uint32_t base2 = (uint32_t)b1 * 0x01000100u;
      const uint32_t cap2 = 0x01000100u;
      const uint32_t stride2 = (4u * kRegSlots) * 0x00010001u;                       // bytes per bin
      const uint32_t slot2 = (uint32_t)(uintptr_t)my_hist_lds * 0x00010001u;          // this lane's count of bin 0
#pragma unroll
      for (int u = 0; u < VPL; ++u)
#pragma unroll
        for (int h = 0; h < 4; ++h) {
          // both LDS addresses of the register's two keys in one packed multiply-add (all below 64 KB)
          const uint32_t a2 = pk_mad_u16(pk_min_u16(pk_sub_u16(y[u][h], base2), cap2), stride2, slot2);
          lds_add_one(a2 & 0xffffu);
          lds_add_one(a2 >> 16);
        }
    }
    __syncthreads();
    int b2, gt2;
    reduce_and_find<true>(hist, tot, tid, lane, want - gt1, b2, gt2);
    const uint32_t T = ((uint32_t)b1 << 8) | (uint32_t)b2;
    const int r = want - gt1 - gt2;   // keys equal to T that are still needed, in key order

    // per vector: bit 2e of gtm / eqm says that element e lies above / at the threshold.  Both come
    // from one 2-bit field per element, min(key - (T - 1), 2) with the difference saturating at 0:
    // 0 below T, 1 at T, 2 above; one dot product per register puts its two fields in place.
    uint32_t gtm[VPL], eqm[VPL];
    {
      const uint32_t Tu = (uint32_t)__builtin_amdgcn_readfirstlane((int)T);
      const uint32_t two2 = 0x00020002u;
      const uint32_t below2 = (Tu - 1u) * 0x00010001u;
      if (Tu) {
#pragma unroll
        for (int u = 0; u < VPL; ++u) {
          uint32_t f = 0;
#pragma unroll
          for (int h = 0; h < 4; ++h)
            f = dot2_u16(pk_min_u16(pk_sub_sat_u16(y[u][h], below2), two2), (1u << (4 * h)) | (4u << (4 * h + 16)), f);
          gtm[u] = (f >> 1) & 0x5555u;
          eqm[u] = f & 0x5555u;
        }
      } else {   // every key is at or above a threshold of 0
#pragma unroll
        for (int u = 0; u < VPL; ++u) {
          uint32_t f = 0;
#pragma unroll
          for (int h = 0; h < 4; ++h)
            f = dot2_u16(pk_min_u16(y[u][h], one2) + one2, (1u << (4 * h)) | (4u << (4 * h + 16)), f);
          gtm[u] = (f >> 1) & 0x5555u;
          eqm[u] = f & 0x5555u;
        }
      }
    }
    // where this wave's part of the list starts: counts of the waves before it
    uint32_t mine = 0;
#pragma unroll
    for (int u = 0; u < VPL; ++u) mine += (uint32_t)__popc(gtm[u]) + ((uint32_t)__popc(eqm[u]) << 16);
    const uint32_t wave_total = (uint32_t)__builtin_amdgcn_readlane((int)lane_scan(mine), 63);
    if (lane == 0) wave_cnt[wave] = wave_total;
    __syncthreads();
    int out_pos = 0, eq_seen = 0;
    {
      uint32_t before = 0;
#pragma unroll
      for (int u = 0; u < kRegThreads / 64 - 1; ++u) before += u < wave ? wave_cnt[u] : 0u;
      out_pos = (int)(before & 0xffffu);
      eq_seen = (int)(before >> 16);
    }
    out_pos += eq_seen < r ? eq_seen : r;
    if (wave_total >> 16) {
      // keys equal to T in this wave: keep those whose rank among all such keys of the row is below r
      uint32_t ec[NP];
#pragma unroll
      for (int j = 0; j < NP; ++j) {
        ec[j] = (uint32_t)__popc(eqm[2 * j]);
        if (2 * j + 1 < VPL) ec[j] += (uint32_t)__popc(eqm[2 * j + 1]) << 16;
        ec[j] = lane_scan(ec[j]);
      }
#pragma unroll
      for (int u = 0; u < VPL; ++u) {
        const uint32_t incl = (ec[u >> 1] >> (16 * (u & 1))) & 0xffffu;
        const uint32_t total = ((uint32_t)__builtin_amdgcn_readlane((int)ec[u >> 1], 63) >> (16 * (u & 1))) & 0xffffu;
        uint32_t e = eqm[u];
        int keep = r - (eq_seen + (int)incl - __popc(e));
        uint32_t kept = 0;
        while (e && keep > 0) {
          kept |= e & (0u - e);
          e &= e - 1;
          --keep;
        }
        gtm[u] |= kept;
        eq_seen += (int)total;
      }
    }
    // ordered emit
    uint32_t sc[NP];
#pragma unroll
    for (int j = 0; j < NP; ++j) {
      sc[j] = (uint32_t)__popc(gtm[2 * j]);
      if (2 * j + 1 < VPL) sc[j] += (uint32_t)__popc(gtm[2 * j + 1]) << 16;
      sc[j] = lane_scan(sc[j]);
    }
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
      const uint32_t incl = (sc[u >> 1] >> (16 * (u & 1))) & 0xffffu;
      const uint32_t total = ((uint32_t)__builtin_amdgcn_readlane((int)sc[u >> 1], 63) >> (16 * (u & 1))) & 0xffffu;
      uint32_t sel = gtm[u];
      int pos = out_pos + (int)incl - __popc(sel);
      const int key0 = 8 * (vbase + 64 * u);
      while (sel) {
        dst[pos++] = key0 + (__builtin_ctz(sel) >> 1);
        sel &= sel - 1;
      }
      out_pos += (int)total;
    }
    if (tid == 0) kv_num[row] = want;
    // wave_cnt is rewritten only behind the barriers of the next row's passes
  }
}

template <int VPL>
static hipError_t launch_topk_select_reg(int* kv_indices, int* kv_num, const uint16_t* score, int rows, int score_stride,
                                         int kv_len, int select_k, int idx_stride, hipStream_t stream) {
  const int grid = rows < 16384 ? rows : 16384;
  hipLaunchKernelGGL(topk_select_reg_kernel<VPL>, dim3(grid), dim3(kRegThreads), 0, stream, kv_indices, kv_num, score, rows,
                     score_stride, kv_len, select_k, idx_stride);
  return hipGetLastError();
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
  if (kv_len <= kRegMaxKeys) {
    const int vpl = ((kv_len + 7) / 8 + kRegThreads - 1) / kRegThreads;
#define SPATTN_TOPK_REG(V) \
  if (vpl <= V) return launch_topk_select_reg<V>(kv_indices, kv_num, score, rows, score_stride, kv_len, select_k, idx_stride, stream)
    SPATTN_TOPK_REG(1);
    SPATTN_TOPK_REG(2);
    SPATTN_TOPK_REG(4);
    SPATTN_TOPK_REG(8);
    SPATTN_TOPK_REG(12);
    SPATTN_TOPK_REG(18);
#undef SPATTN_TOPK_REG
  }
  int grid = (rows + 3) / 4;
  if (grid > 4096) grid = 4096;
  hipLaunchKernelGGL(topk_select_kernel, dim3(grid), dim3(256), 0, stream, kv_indices, kv_num, score, rows,
                     score_stride, kv_len, select_k, idx_stride);
  return hipGetLastError();
}

}  // namespace spattn
