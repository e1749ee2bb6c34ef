// Shared declarations for the gfx950 sparse-attention kernels.
// Wave = 64 lanes; all matrix work uses v_mfma_f32_32x32x16_bf16.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace spattn {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((ext_vector_type(4))) int i32x4;

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// How the key rows of one 64-key tile are found.
enum KvMode : int {
  KV_DENSE = 0,   // tile t = rows 64t .. 64t+63, up to kv_len
  KV_TOKENS = 1,  // tile t = rows idx[64t .. 64t+63] of a per-q-block token list
  KV_BLOCKS = 2,  // tile t = rows 64*blk[t] .. 64*blk[t]+63 of a per-q-block block list
};

struct AttnParams {
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* v;
  uint16_t* o;        // bf16 [B,H,S,D]
  float* lse;         // optional fp32 [B,H,S], natural log
  float* max_q;       // optional fp32 [B,H,1,Sp], raw (unscaled) row max
  float* denom;       // optional fp32 [B,H,1,Sp]
  uint16_t* blockmax; // optional bf16 [B,H,Sp/64,Sp]: raw max of row r over the keys of block J at [J][r], rounded toward +inf (dense + statistics only)
  const int* idx;     // [B,H,SBq,idx_stride] token ids or block ids
  const int* cnt;     // [B*H*SBq]
  int idx_stride;
  const int* order;   // optional [B*H*nqblk]: the q-block (flat index) that workgroup i takes
  int B, H, S;
  int kv_len;         // keys with row >= kv_len never contribute
  int Sp;             // row stride of max_q / denom
  int nqblk;          // q-blocks per head
  float scale;        // softmax scale
  float sf;           // log2(e) * scale
};

__device__ __forceinline__ f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  f32x2 f = {lo, hi};
  bf16x2 b = __builtin_convertvector(f, bf16x2);   // v_cvt_pk_bf16_f32, round to nearest even
  return __builtin_bit_cast(uint32_t, b);
}

// The smallest bf16 that is not below x (x not NaN): negative values are truncated, positive ones
// rounded away from zero; -inf stays -inf.
__device__ __forceinline__ uint16_t bf16_round_up(float x) {
  const uint32_t b = __builtin_bit_cast(uint32_t, x);
  return (uint16_t)((b + ((b >> 31) ? 0u : 0xffffu)) >> 16);
}

// Largest of three floats in one instruction.  Written as asm: through fmaxf the compiler first
// passes every operand it cannot prove free of signalling NaNs (the accumulators of a matrix
// multiply among them) through a v_max_f32 x, x of its own, three instructions per two scores
// instead of one per two.  A NaN operand is skipped like in fmaxf.
__device__ __forceinline__ float max3_raw(float a, float b, float c) {
  float d;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
  return d;
}

__device__ __forceinline__ float max_raw(float a, float b) {
  float d;
  asm("v_max_f32 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
  return d;
}

// Max / sum of the values held by lanes l and l ^ 32, in both lanes.  v_permlane32_swap
// exchanges the upper half of its first operand with the lower half of its second: with
// the same value in both, each lane ends up holding its own and its partner's value.
// Written as asm: both operands are read and written, and the wait states cover a
// preceding vector-ALU write of either operand.
__device__ __forceinline__ void pair_values(float x, float& lo, float& hi) {
  lo = x;
  hi = x;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(lo), "+v"(hi));
}
__device__ __forceinline__ float pair_max(float x) {
  float a, b;
  pair_values(x, a, b);
  return max_raw(a, b);
}
__device__ __forceinline__ float pair_sum(float x) {
  float a, b;
  pair_values(x, a, b);
  return a + b;
}

// WGs are dealt to the 8 XCDs round-robin by launch order; give each XCD one
// contiguous range of logical work ids so that neighbouring q-blocks of a head
// share that XCD's L2.
__device__ __forceinline__ int xcd_remap(int wg, int total) {
  constexpr int kXcd = 8;
  int per = total / kXcd;
  int lim = per * kXcd;
  if (wg >= lim) return wg;
  return (wg % kXcd) * per + wg / kXcd;
}

#define SPATTN_LDS __attribute__((address_space(3)))
typedef SPATTN_LDS const unsigned char* lds_cptr;

// One wave-wide HBM -> LDS copy: lane l's 16 bytes land at lds_base + 16 l.
// Written as asm on purpose: the compiler does not count this load in its own vmcnt
// bookkeeping (with the builtin it drains every outstanding load before each LDS read),
// so the waits are placed by hand.  m0 cannot be named as clobbered (the compiler reserves it and
// warns that such a clobber is not honoured); tests/test_asm_inflight_loads.py checks on the
// listing that no compiler-generated instruction reads m0 across these statements.
__device__ __forceinline__ void dma16(const void* gptr, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_base), "v"(gptr) : "memory");
}
// Same with a wave-uniform base pointer and a 32-bit per-lane byte offset.
// The base goes through readfirstlane: under scalar-register pressure the compiler may keep
// a uniform pointer in vector registers, which the "s" constraint alone does not undo.
__device__ __forceinline__ void dma16(const void* sbase, uint32_t voff, uint32_t lds_base) {
  const uint64_t b = (uint64_t)(uintptr_t)sbase;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)b);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(b >> 32));
  const uint64_t sb = ((uint64_t)hi << 32) | lo;
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_base), "v"(voff), "s"(sb) : "memory");
}
// 16-byte global load that the compiler does not count either: the destination is valid only
// behind a hand-placed vmcnt wait, after which the caller ties the registers to that point with
// an empty asm ("+v") before their first use.
template <int OFF>
__device__ __forceinline__ void load16_uncounted(u32x4& dst, const void* ptr) {
  asm volatile("global_load_dwordx4 %0, %1, off offset:%2" : "=v"(dst) : "v"(ptr), "n"(OFF) : "memory");
}
// Q operands of the score product, k-steps T .. NT-1: 16 bytes every 32 from src.
template <int T, int NT>
__device__ __forceinline__ void load_q_uncounted(u32x4 (&qf)[NT], const void* src) {
  if constexpr (T < NT) {
    load16_uncounted<32 * T>(qf[T], src);
    load_q_uncounted<T + 1, NT>(qf, src);
  }
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// Raises a kernel's dynamic-LDS limit once per device (the attribute belongs to the device's
// copy of the kernel).  Host only; racing threads repeat a call that does no harm.
constexpr int kMaxDevices = 64;
inline hipError_t raise_lds_limit(const void* kernel, int bytes, bool (&done)[kMaxDevices]) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev >= 0 && dev < kMaxDevices && done[dev]) return hipSuccess;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) return e;
  if (dev >= 0 && dev < kMaxDevices) done[dev] = true;
  return hipSuccess;
}

}  // namespace spattn
