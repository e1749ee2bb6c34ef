// Work order for list-driven attention with very uneven list lengths.
//
// One workgroup per q-block, dispatched in index order, leaves the longest lists to whoever
// happens to get them last: with Zipf-distributed lengths a quarter of the run is spent
// waiting for a few stragglers.  qblock_order_kernel sorts the q-blocks by list length,
// longest first, in quarter-octave classes (stable inside a class, so the order is a function
// of the counts alone); the attention kernels then let workgroup i take q-block order[i].
// Lists whose lengths differ by less than a factor of two keep the default order, in which every XCD works on
// neighbouring q-blocks of one head.  The reference has no counterpart: its grid is fixed
// to (q-block, head, batch) (include/sparseattn_asyncgatherload_padded.cuh:273).
#include "common.h"
#include "dispatch.h"

namespace spattn {

constexpr int kOrderThreads = 128;
constexpr int kOrderSub = 2;                              // bits below the leading one that tell classes apart
constexpr int kOrderClasses = (22 << kOrderSub) + 2;      // 4 per octave up to 2^22 keys, one for longer lists, one for empty ones

// class 0 holds the longest lists
__device__ __forceinline__ int length_class(int c) {
  if (c <= 0) return kOrderClasses - 1;
  const int lg = 31 - __builtin_clz((unsigned)c);            // floor(log2 c), 0..30
  const int below = lg >= kOrderSub ? ((c >> (lg - kOrderSub)) & ((1 << kOrderSub) - 1))
                                    : ((c << (kOrderSub - lg)) & ((1 << kOrderSub) - 1));
  const int fine = (lg << kOrderSub) + below;
  return kOrderClasses - 2 - (fine < kOrderClasses - 2 ? fine : kOrderClasses - 2);
}

__global__ __launch_bounds__(kOrderThreads) void qblock_order_kernel(int* __restrict__ order,
                                                                      const int* __restrict__ counts, int n) {
  constexpr int T = kOrderThreads;
  __shared__ int cls_cnt[kOrderClasses * T];   // [class][thread]: members in that thread's segment, then offsets
  __shared__ int part[T];
  __shared__ int lo_hi[2];
  const int tid = threadIdx.x;
  // A thread owns a contiguous segment (the order inside a class is the index order), a multiple of
  // four counts long so that it is read with 16-byte loads, sixteen counts in flight at a time: one
  // count per load, each waiting for the one before, made this kernel 23 us of pure load latency.
  const int seg = (((n + T - 1) / T) + 3) & ~3;
  const int i0 = tid * seg < n ? tid * seg : n;
  const int i1 = (i0 + seg) < n ? (i0 + seg) : n;
  const bool vec_ok = ((uintptr_t)counts & 15) == 0;
  auto walk = [&](auto&& f) {
    for (int b = i0; b < i1; b += 16) {
      i32x4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int i = b + 4 * u;
        if (vec_ok && i + 4 <= i1) {
          v[u] = *reinterpret_cast<const i32x4*>(counts + i);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) v[u][e] = (i + e < i1) ? counts[i + e] : 0;
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (b + 4 * u + e < i1) f(b + 4 * u + e, v[u][e]);
    }
  };

  for (int c = 0; c < kOrderClasses; ++c) cls_cnt[c * T + tid] = 0;
  if (tid == 0) {
    lo_hi[0] = 0x7fffffff;
    lo_hi[1] = 0;
  }
  __syncthreads();
  int lo = 0x7fffffff, hi = 0;
  walk([&](int, int c) {
    lo = c < lo ? c : lo;
    hi = c > hi ? c : hi;
    cls_cnt[length_class(c) * T + tid] += 1;
  });
  atomicMin(&lo_hi[0], lo);
  atomicMax(&lo_hi[1], hi);
  __syncthreads();
  lo = lo_hi[0];
  hi = lo_hi[1];
  // the longest list less than twice the shortest: little to balance (measured: sorting such
  // lists costs 2 % through the lost locality), keep neighbours together
  if (hi <= 0 || hi < 2 * lo) {
    for (int i = i0; i < i1; ++i) order[i] = xcd_remap(i, n);
    return;
  }
  // exclusive prefix sum over cls_cnt in storage order (class-major, thread-minor)
  constexpr int PER = kOrderClasses;   // entries per scanning thread
  int sum = 0;
  for (int j = 0; j < PER; ++j) sum += cls_cnt[tid * PER + j];
  part[tid] = sum;
  __syncthreads();
  if (tid == 0) {
    int run = 0;
    for (int j = 0; j < T; ++j) {
      const int x = part[j];
      part[j] = run;
      run += x;
    }
  }
  __syncthreads();
  int run = part[tid];
  for (int j = 0; j < PER; ++j) {
    const int x = cls_cnt[tid * PER + j];
    cls_cnt[tid * PER + j] = run;
    run += x;
  }
  __syncthreads();
  walk([&](int i, int c) {
    const int slot = length_class(c) * T + tid;
    order[cls_cnt[slot]] = i;
    cls_cnt[slot] += 1;
  });
}

hipError_t run_qblock_order(int* order, const int* counts, int n, hipStream_t stream) {
  if (n <= 0) return hipSuccess;
  hipLaunchKernelGGL(qblock_order_kernel, dim3(1), dim3(kOrderThreads), 0, stream, order, counts, n);
  return hipGetLastError();
}

}  // namespace spattn
