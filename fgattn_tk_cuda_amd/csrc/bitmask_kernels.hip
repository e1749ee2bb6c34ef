// Bit-packed vote masks for the mask cache.
//
// The reference keeps a cached mask as one bit per key, least significant bit first
// (python/spattn/mask_utils.py:421-439, `pack` / `unpack`), and on every reuse expands it
// with torch ops to an int32 mask that booleanmask_to_indexmask then compacts
// (CompressedBitMaskCache, python/spattn/mask_utils.py:74-98).  Here both directions are
// single kernels:
//   pack_mask_kernel            int32 vote mask -> bits            (reads 4 B per key, writes 1/8 B)
//   packed_to_indexmask_kernel  bits -> ascending index lists      (reads 1/8 B per key, writes 4 B per kept key)
// so that a reuse of a cached mask streams 1/32 of the bytes of the int32 path and never
// materialises the unpacked mask.
#include "common.h"
#include "dispatch.h"

namespace spattn {

// ------------------------------------------------------------------------------------
// pack: bit (c & 7) of byte c >> 3 of a row is set iff mask[row][c] > 0.
// One wave per step of 2048 keys (8 coalesced 16-byte loads per lane, the next step in
// flight).  A lane's four keys give a nibble; three shift-and-or exchanges with the lanes
// 1, 2 and 4 further on assemble the 32 keys of eight neighbouring lanes into one word,
// which every eighth lane stores.
// ------------------------------------------------------------------------------------
constexpr int kPackUnroll = 8;

__global__ __launch_bounds__(256) void pack_mask_kernel(uint32_t* __restrict__ packed, const int* __restrict__ mask,
                                                        int rows, int mask_stride) {
  constexpr int U = kPackUnroll;
  constexpr int SPAN = 256 * U;   // keys per wave step
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int words_per_row = mask_stride >> 5;
  const int nstep = (mask_stride + SPAN - 1) / SPAN;
  for (int row = blockIdx.x * 4 + wave; row < rows; row += gridDim.x * 4) {
    const int* __restrict__ src = mask + (size_t)row * mask_stride;
    uint32_t* __restrict__ dst = packed + (size_t)row * words_per_row;
    i32x4 cur[U], nxt[U];
    auto load = [&](int c, i32x4 (&v)[U]) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int e0 = c * SPAN + u * 256 + 4 * lane;
        const i32x4 z = {0, 0, 0, 0};
        v[u] = (e0 < mask_stride) ? __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(src + e0)) : z;
      }
    };
    load(0, cur);
    for (int c = 0; c < nstep; ++c) {
      if (c + 1 < nstep) load(c + 1, nxt);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        uint32_t x = (cur[u][0] > 0 ? 1u : 0u) | (cur[u][1] > 0 ? 2u : 0u) | (cur[u][2] > 0 ? 4u : 0u) |
                     (cur[u][3] > 0 ? 8u : 0u);
        // lanes l + 1, l + 2, l + 4 of the same 16-lane row (row_shl: data moves towards lane 0); only the
        // lanes with l % 8 == 0 use the result, and their partners lie in their own group of eight
        x |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x101, 0xf, 0xf, true) << 4;
        x |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x102, 0xf, 0xf, true) << 8;
        x |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x104, 0xf, 0xf, true) << 16;
        const int word = (c * SPAN + u * 256 + 4 * lane) >> 5;
        if ((lane & 7) == 0 && word < words_per_row) dst[word] = x;
      }
#pragma unroll
      for (int u = 0; u < U; ++u) cur[u] = nxt[u];
    }
  }
}

hipError_t run_pack_mask(uint32_t* packed, const int* mask, int rows, int mask_stride, hipStream_t stream) {
  if (rows <= 0) return hipSuccess;
  int grid = (rows + 3) / 4;
  if (grid > 2048) grid = 2048;
  hipLaunchKernelGGL(pack_mask_kernel, dim3(grid), dim3(256), 0, stream, packed, mask, rows, mask_stride);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------
// packed bits -> index lists, the fused form of unpack + booleanmask_to_indexmask
// (include/mask_utils.cuh:273-302 for the compaction): per row the keys c < kv_len whose
// bit is set, ascending, then the caller's fill; counts exact.
// One wave per row.  A step takes 1 KB of bits (8192 keys, one 16-byte load per lane, the
// next step in flight) into a wave-private LDS stage and walks it in eight sub-steps of
// 1024 keys: lane l owns the 16 keys 16 l .. 16 l + 15 of the sub-step, a wave prefix sum of
// the lanes' popcounts (five ballots) gives its place in the output, and it appends its keys to the same
// kind of ring that compact_kernel uses, written out 4 KB at a time.
// ------------------------------------------------------------------------------------
constexpr int kBitRing = 2048;    // ints; a sub-step appends at most 1024 to fewer than kBitFlush pending
constexpr int kBitFlush = 1024;

__global__ __launch_bounds__(256) void packed_to_indexmask_kernel(int* __restrict__ kv_indices, int* __restrict__ kv_num,
                                                                  const uint32_t* __restrict__ packed, int rows,
                                                                  int mask_stride, int kv_len) {
  constexpr int QN = kBitRing;
  constexpr int FL = kBitFlush;
  static_assert(FL + 1024 <= QN && FL % 256 == 0, "one sub-step must fit next to a pending flush");
  __shared__ __attribute__((aligned(16))) int ring[4][QN];
  __shared__ __attribute__((aligned(16))) uint16_t stage[4][512];   // 1 KB of bits per wave
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  int* q = ring[wave];
  uint16_t* st = stage[wave];
  const int lim = kv_len < mask_stride ? kv_len : mask_stride;
  const int vec_per_row = mask_stride >> 7;            // 16-byte vectors (128 keys) per row
  const int nstep = (lim + 8191) >> 13;                // steps that contain keys below lim

  for (int row = blockIdx.x * 4 + wave; row < rows; row += gridDim.x * 4) {
    const u32x4* __restrict__ src = reinterpret_cast<const u32x4*>(packed + (size_t)row * (mask_stride >> 5));
    int* __restrict__ dst = kv_indices + (size_t)row * mask_stride;
    int tail = 0, head = 0;
    auto load = [&](int c) -> u32x4 {
      const int v = c * 64 + lane;
      const u32x4 z = {0, 0, 0, 0};
      return (v < vec_per_row) ? src[v] : z;
    };
    u32x4 cur = {0, 0, 0, 0}, nxt = {0, 0, 0, 0};
    if (nstep > 0) cur = load(0);
    for (int c = 0; c < nstep; ++c) {
      if (c + 1 < nstep) nxt = load(c + 1);
      *reinterpret_cast<u32x4*>(st + 8 * lane) = cur;   // keys 128 l .. 128 l + 127 of the step
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
#pragma unroll 1
      for (int s = 0; s < 8; ++s) {
        const int key0 = c * 8192 + s * 1024 + 16 * lane;   // first key of this lane
        if (c * 8192 + s * 1024 >= lim) break;               // wave-uniform
        uint32_t bits = st[s * 64 + lane];
        const int valid = lim - key0;                        // keys of this lane below lim
        if (valid < 16) bits = valid <= 0 ? 0u : (bits & ((1u << valid) - 1u));
        // exclusive prefix sum of the lanes' counts (0..16) without any exchange: one ballot per
        // bit of the count, weighted by its place
        const int cnt = __popc(bits);
        int before = 0, total = 0;
#pragma unroll
        for (int w = 0; w < 5; ++w) {
          const unsigned long long m = __ballot((cnt >> w) & 1);
          before += (int)__builtin_amdgcn_mbcnt_hi((unsigned)(m >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)m, 0)) << w;
          total += __popcll(m) << w;
        }
        int pos = tail + before;
        while (bits) {
          const int b = __builtin_ctz(bits);
          q[pos & (QN - 1)] = key0 + b;
          ++pos;
          bits &= bits - 1;
        }
        tail += total;
        if (tail - head >= FL) {
#pragma unroll
          for (int w = 0; w < FL / 256; ++w)
            *reinterpret_cast<i32x4*>(dst + head + w * 256 + 4 * lane) =
                *reinterpret_cast<const i32x4*>(q + ((head + w * 256 + 4 * lane) & (QN - 1)));
          head += FL;
        }
      }
      __builtin_amdgcn_wave_barrier();
      cur = nxt;
    }
    for (; head < tail; head += 64)
      if (head + lane < tail) dst[head + lane] = q[(head + lane) & (QN - 1)];
    if (lane == 0) kv_num[row] = tail;
  }
}

hipError_t run_packed_to_indexmask(int* kv_indices, int* kv_num, const uint32_t* packed, int rows, int mask_stride,
                                   int kv_len, hipStream_t stream) {
  if (rows <= 0) return hipSuccess;
  int grid = (rows + 3) / 4;
  if (grid > 2048) grid = 2048;
  hipLaunchKernelGGL(packed_to_indexmask_kernel, dim3(grid), dim3(256), 0, stream, kv_indices, kv_num, packed, rows,
                     mask_stride, kv_len);
  return hipGetLastError();
}

}  // namespace spattn
