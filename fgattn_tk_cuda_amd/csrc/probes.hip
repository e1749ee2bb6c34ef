// Roofline probes for the attention kernels on gfx950 (libspattn_probes.so; not part of the
// product library).  spattn_probe_copy_stream times the gather of a block-list launch with
// nothing else running (the HBM / L2 -> LDS path at the lists' real L2 hit rate);
// spattn_probe_lds_mix measures what the LDS of a compute unit sustains for the three kinds
// of access the attention tile loop makes - HBM/L2 -> LDS copies (global_load_lds_dwordx4),
// ds_read_b128 of the K operands, ds_read_b64_tr_b16 of the V^T operands - alone and in the
// mix one 64-key tile of a 64-row q-block at d = 128 needs (32 KB copied, 32 KB + 32 KB read),
// with no matrix or vector work next to them: the time of that mix is a floor for the tile
// loop whatever its schedule.
//
// Launch shape of the attention kernel: 256 lanes per workgroup, 80 KB of LDS, two workgroups
// per compute unit.  The copies take their data from a 1 MB window (L2 resident), so neither
// HBM nor the L2 miss path is in the measurement.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
#define PROBE_LDS __attribute__((address_space(3)))

__device__ __forceinline__ void copy16(const void* sbase, uint32_t voff, uint32_t lds_base) {
  const uint64_t b = (uint64_t)(uintptr_t)sbase;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)b);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(b >> 32));
  const uint64_t sb = ((uint64_t)hi << 32) | lo;
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_base), "v"(voff), "s"(sb) : "memory");
}

enum : int {
  kCopy = 1,      // every wave copies 8 KB per step (32 KB per workgroup step)
  kReadK = 2,     // every wave reads 8 KB per step with ds_read_b128, K-operand pattern
  kReadV = 4,     // every wave reads 8 KB per step with ds_read_b64_tr_b16, V^T-operand pattern
  kWrite = 8,     // every wave writes 8 KB per step with ds_write_b128
  kBarrier = 16,  // one workgroup barrier per step, copies waited for as in the tile loop
};

// Ring of five 16 KB slots as in the attention kernel; step s copies into slots (2s, 2s+1) % 5
// and reads slots (2s+2, 2s+3) % 5.
template <int WHAT>
__global__ __launch_bounds__(256, 2) void lds_mix_kernel(const unsigned char* src, float* sink, int steps) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  const uint32_t base = (uint32_t)(uintptr_t)(PROBE_LDS unsigned char*)smem;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  for (int i = threadIdx.x; i < 81920 / 4; i += 256) reinterpret_cast<uint32_t*>(smem)[i] = i;
  __syncthreads();
  // K pattern: lane (row = lane & 31, half = lane >> 5) reads chunk (2t + half) ^ swz(row) of its row (256-byte rows)
  const int ln = lane & 31, g = lane >> 5;
  const int swk = ((ln & 3) << 2) | ((ln >> 2) & 3);
  const uint32_t k0 = base + (wave & 1) * 8192 + ln * 256;
  // V pattern: 16-lane groups address four rows; see the V^T reads of the attention kernel
  const int i16 = lane & 15, dhalf = (lane >> 4) & 1;
  const int r1 = 4 * g + (i16 >> 2);
  const int cb = 2 * dhalf + ((i16 & 3) >> 1);
  const int swv = ((r1 & 3) << 2) | ((r1 >> 2) & 3);
  const uint32_t v0 = base + (wave & 1) * 8192 + r1 * 256 + ((cb ^ swv) << 4) + ((i16 & 1) << 3);
  const unsigned char* s0 = src + (size_t)(blockIdx.x % 32) * 32768;
  const uint32_t voff = lane * 16;
  u32x4 acc = {0u, 0u, 0u, 0u};
  const u32x4 wv = {1u, 2u, 3u, (uint32_t)lane};
  for (int s = 0; s < steps; ++s) {
    const uint32_t cs = (uint32_t)((2 * s) % 5) * 16384;
    const uint32_t rs0 = (uint32_t)((2 * s + 2) % 5) * 16384;
    const uint32_t rs1 = (uint32_t)((2 * s + 3) % 5) * 16384;
    if constexpr ((WHAT & kBarrier) != 0) {
      asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
      __syncthreads();
    }
    if constexpr ((WHAT & kCopy) != 0) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        // parts 0-3 into the first slot, 4-7 into the second; wave w owns KB w of every 4 KB
        const uint32_t slot = (i < 4) ? cs : (uint32_t)((2 * s + 1) % 5) * 16384;
        copy16(s0 + (i & 3) * 4096 + wave * 1024 + (i >> 2) * 16384, voff, base + slot + (i & 3) * 4096 + wave * 1024);
      }
    }
    if constexpr ((WHAT & kWrite) != 0) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        asm volatile("ds_write_b128 %0, %1" ::"v"(base + cs + (uint32_t)(i * 4096 + wave * 1024 + lane * 16) % 32768u), "v"(wv) : "memory");
    }
    u32x4 xk[8];
    u32x2 xv[16];
    if constexpr ((WHAT & kReadK) != 0) {
#pragma unroll
      for (int t = 0; t < 8; ++t)
        asm volatile("ds_read_b128 %0, %1" : "=v"(xk[t]) : "v"(k0 + rs0 + (uint32_t)(((2 * t + g) ^ swk) << 4)) : "memory");
    }
    if constexpr ((WHAT & kReadV) != 0) {
#pragma unroll
      for (int t = 0; t < 16; ++t) {
        // 32-dim block t & 3, rows +8 with one swizzle bit flipped for odd t >> 2, rows +16 for t >= 8
        const uint32_t a = ((v0 + rs1) ^ (uint32_t)(((t & 3) << 6) | (((t >> 2) & 1) << 5))) + (uint32_t)(t >> 2) * 2048;
        asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(xv[t]) : "v"(a) : "memory");
      }
    }
    if constexpr ((WHAT & (kReadK | kReadV)) != 0) {
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      if constexpr ((WHAT & kReadK) != 0) {
#pragma unroll
        for (int t = 0; t < 8; ++t) {
          asm volatile("" : "+v"(xk[t]));
          acc ^= xk[t];
        }
      }
      if constexpr ((WHAT & kReadV) != 0) {
#pragma unroll
        for (int t = 0; t < 16; ++t) {
          asm volatile("" : "+v"(xv[t]));
          acc[0] ^= xv[t][0];
          acc[1] ^= xv[t][1];
        }
      }
    }
    if constexpr ((WHAT & kCopy) != 0 && (WHAT & kBarrier) == 0) asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
  }
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345u) sink[0] = 1.f;
}

template <int WHAT>
int run_mix(const unsigned char* src, float* sink, int steps, int reps, float* ms_out, hipStream_t stream) {
  auto kern = lds_mix_kernel<WHAT>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 81920);
  if (e != hipSuccess) return (int)e;
  int dev = 0, cus = 0;
  if ((e = hipGetDevice(&dev)) != hipSuccess) return (int)e;
  if ((e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev)) != hipSuccess) return (int)e;
  hipEvent_t a, b;
  if ((e = hipEventCreate(&a)) != hipSuccess) return (int)e;
  if ((e = hipEventCreate(&b)) != hipSuccess) return (int)e;
  const dim3 grid(2 * cus);
  for (int i = 0; i < 3; ++i) hipLaunchKernelGGL(kern, grid, dim3(256), 81920, stream, src, sink, steps);
  (void)hipEventRecord(a, stream);
  for (int i = 0; i < reps; ++i) hipLaunchKernelGGL(kern, grid, dim3(256), 81920, stream, src, sink, steps);
  (void)hipEventRecord(b, stream);
  e = hipEventSynchronize(b);
  float ms = 0.f;
  if (e == hipSuccess) e = hipEventElapsedTime(&ms, a, b);
  (void)hipEventDestroy(a);
  (void)hipEventDestroy(b);
  if (e != hipSuccess) return (int)e;
  *ms_out = ms / reps;
  return (int)hipGetLastError();
}

// The copy stream of block-list attention on its own: every workgroup walks the KV-block list of
// its q-block and copies the K and V tiles (64 rows of 256 bytes, d = 128) into a ring of five
// 16 KB LDS slots, four tiles in flight, one barrier per tile - no LDS reads, no arithmetic.
// Same grid, same q-block -> XCD mapping and same lists as the attention kernel, so the L2 hit
// rate of the gather is the real one.
__global__ __launch_bounds__(256, 2) void copy_stream_kernel(const unsigned char* k, const unsigned char* v, const int* lists,
                                                             int nlist, int nqblk, int seq, int total) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  const uint32_t base = (uint32_t)(uintptr_t)(PROBE_LDS unsigned char*)smem;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int per = total / 8;
  const int wg = (int)blockIdx.x < per * 8 ? ((int)blockIdx.x % 8) * per + (int)blockIdx.x / 8 : (int)blockIdx.x;
  const int bh = wg / nqblk;
  const size_t head_off = (size_t)bh * seq * 256;
  typedef const __attribute__((address_space(4))) int* cint_p;
  cint_p lst = (cint_p)(lists + (size_t)wg * nlist);
  const int ntiles = 2 * nlist;   // K0 V0 K1 V1 ...
  uint32_t go[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) go[i] = (uint32_t)((4 * (4 * i + wave) + lane / 16) * 256 + (lane % 16) * 16);
  auto issue = [&](int t) {
    const int blk = lst[t >> 1];
    const unsigned char* src = ((t & 1) ? v : k) + head_off + (size_t)blk * 64 * 256;
    const uint32_t lds = base + (uint32_t)(t % 5) * 16384 + wave * 1024;
#pragma unroll
    for (int i = 0; i < 4; ++i) copy16(src, go[i], lds + i * 4096);
  };
  for (int t = 0; t < 4 && t < ntiles; ++t) issue(t);
  for (int t = 0; t < ntiles; ++t) {
    const int younger = (ntiles - 1 - t) < 3 ? (ntiles - 1 - t) : 3;
    if (younger == 3) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
    else if (younger == 2) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    else if (younger == 1) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (t + 4 < ntiles) issue(t + 4);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

}  // namespace

extern "C" {

// Copy stream of block-list attention at d = 128 with 64-row q-blocks (see copy_stream_kernel):
// k, v bf16 [heads, seq, 128]; lists int32 [heads * seq/64, nlist] of valid 64-key block ids.
// Returns the average time of one launch in *ms_out.
int spattn_probe_copy_stream(const void* k, const void* v, const int* lists, int nlist, int heads, int seq, int reps,
                             float* ms_out, void* stream) {
  hipStream_t st = static_cast<hipStream_t>(stream);
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(copy_stream_kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, 81920);
  if (e != hipSuccess) return (int)e;
  const int nqblk = seq / 64, total = heads * nqblk;
  hipEvent_t a, b;
  if ((e = hipEventCreate(&a)) != hipSuccess) return (int)e;
  if ((e = hipEventCreate(&b)) != hipSuccess) return (int)e;
  auto launch = [&]() {
    hipLaunchKernelGGL(copy_stream_kernel, dim3(total), dim3(256), 81920, st, static_cast<const unsigned char*>(k),
                       static_cast<const unsigned char*>(v), lists, nlist, nqblk, seq, total);
  };
  for (int i = 0; i < 100; ++i) launch();
  (void)hipEventRecord(a, st);
  for (int i = 0; i < reps; ++i) launch();
  (void)hipEventRecord(b, st);
  e = hipEventSynchronize(b);
  float ms = 0.f;
  if (e == hipSuccess) e = hipEventElapsedTime(&ms, a, b);
  (void)hipEventDestroy(a);
  (void)hipEventDestroy(b);
  if (e != hipSuccess) return (int)e;
  *ms_out = ms / reps;
  return (int)hipGetLastError();
}


// Runs the access mix `what` (bit set: 1 copies, 2 K reads, 4 V^T reads, 8 ds_write_b128,
// 16 one barrier per step) for `steps` steps per workgroup on 2 workgroups per compute unit and
// returns the average time of one launch in *ms_out.  src: at least 1 MB + 32 KB of device
// memory; sink: one float.  Every wave moves 8 KB per step and kind of access, a workgroup
// 32 KB.  Returns 0 or a hipError_t; -1 for a mix that is not instantiated.
int spattn_probe_lds_mix(int what, const void* src, float* sink, int steps, int reps, float* ms_out, void* stream) {
  const unsigned char* s = static_cast<const unsigned char*>(src);
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (what) {
    case 1: return run_mix<1>(s, sink, steps, reps, ms_out, st);
    case 2: return run_mix<2>(s, sink, steps, reps, ms_out, st);
    case 4: return run_mix<4>(s, sink, steps, reps, ms_out, st);
    case 8: return run_mix<8>(s, sink, steps, reps, ms_out, st);
    case 3: return run_mix<3>(s, sink, steps, reps, ms_out, st);
    case 5: return run_mix<5>(s, sink, steps, reps, ms_out, st);
    case 6: return run_mix<6>(s, sink, steps, reps, ms_out, st);
    case 7: return run_mix<7>(s, sink, steps, reps, ms_out, st);
    case 23: return run_mix<23>(s, sink, steps, reps, ms_out, st);
    default: return -1;
  }
}

}  // extern "C"
