// Flash-style attention forward for gfx950, one kernel template for the dense,
// token-list and block-list variants.
//
// What it computes follows the reference kernels
//   include/sparseattn_asyncgatherload_padded.cuh:204-255 (gathered sparse attention),
//   include/fullattn_wgload_padded.cuh:190-232          (dense attention),
//   include/maxq_denom_attn.cuh:196-252                 (dense attention + row statistics),
//   include/maxq_denom.cuh:169-206                      (row statistics only):
// running raw row max m, p = exp2((s - m) * log2e * scale), fp32 denominator, P rounded
// to bf16 before PV, O / l at the end.  Keys that are out of range (list position >= n,
// token id >= kv_len, row >= kv_len) are masked on every tile, a superset of the
// reference's "NaN row -> -inf on the last tile" (include/asyncloadutils.cuh:124-142,
// include/pad_utils.cuh:54-75).
//
// Layout.  A workgroup is 4 waves (256 lanes) and owns one q-block of QBLK rows.
// Scores are produced transposed, S^T = K Q^T, so that in the 32x32 MFMA accumulator a
// lane holds ONE query row (n = lane & 31) and 16 keys: every softmax statistic is a
// per-lane scalar and only lanes l and l^32 ever exchange data.  O is accumulated
// transposed too, O^T += V^T P^T, with P^T taken straight from the score accumulators.
//   QBLK = 128: wave w owns query rows 32w..32w+31 and all 64 keys of a tile.
//   QBLK =  64: wave w owns query rows 32(w&1).. and keys 32(w>>1).. of a tile; the two
//               key halves are merged through LDS at the end.
// LDS per stage: K tile [64][D] bf16 (16-byte chunks XOR-swizzled by row), V^T tile
// [D][64] bf16 (keys permuted so that the PV operand is one 16-byte read), 64 bias
// floats.  Two stages, one barrier per tile; the next tile's rows travel
// HBM -> registers while the current tile is multiplied.
#pragma once
#include "common.h"

namespace spattn {

template <int D, bool HAS_V>
struct AttnSmem {
  static constexpr int kKBytes = 64 * D * 2;
  static constexpr int kVBytes = HAS_V ? D * 64 * 2 : 0;
  static constexpr int kBiasBytes = 64 * 4;
  static constexpr int kStage = kKBytes + kVBytes + kBiasBytes;
  // The key-split merge needs 2 waves * (D/2 + 2) * 64 floats; it reuses the stages.
  static constexpr int kMerge = 2 * (D / 2 + 2) * 64 * 4;
  static constexpr int kTotal = (2 * kStage > kMerge) ? 2 * kStage : kMerge;
};

template <int D, int QBLK, int MODE, bool HAS_V, bool STATS>
__global__ __launch_bounds__(256, 2) void attn_fwd_kernel(const AttnParams p) {
  static_assert(D == 64 || D == 128, "head dim");
  static_assert(QBLK == 64 || QBLK == 128, "q-block");
  constexpr int NQW = QBLK / 32;     // waves along the query rows
  constexpr int KSPLIT = 4 / NQW;    // waves along the keys of a tile
  constexpr int KW = 64 / KSPLIT;    // keys of a tile per wave
  constexpr int NMB = KW / 32;       // 32-key score blocks per wave
  constexpr int NT = D / 16;         // k-steps of the QK^T product
  constexpr int NDB = D / 32;        // 32-wide blocks of the head dim
  constexpr int NKS = KW / 16;       // k-steps of the PV product
  constexpr int CPR = D / 8;         // 16-byte chunks per K row
  using Smem = AttnSmem<D, HAS_V>;
  constexpr float kNegInf = -__builtin_huge_valf();

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int ln = lane & 31;
  const int g = lane >> 5;
  const int qsub = wave % NQW;
  const int ksub = wave / NQW;

  const int total = p.nqblk * p.H * p.B;
  const int wg = xcd_remap(blockIdx.x, total);
  const int qb = wg % p.nqblk;
  const int bh = wg / p.nqblk;

  const size_t head_off = (size_t)bh * p.S * D;
  const uint16_t* __restrict__ qh = p.q + head_off;
  const uint16_t* __restrict__ kh = p.k + head_off;
  const uint16_t* __restrict__ vh = HAS_V ? p.v + head_off : nullptr;

  // ---- tile list of this q-block -------------------------------------------------
  const int* __restrict__ lst = nullptr;
  int n = 0, ntiles = 0;
  if constexpr (MODE == KV_DENSE) {
    ntiles = (p.kv_len + 63) >> 6;
  } else {
    const size_t lrow = (size_t)bh * p.nqblk + qb;
    lst = p.idx + lrow * p.idx_stride;
    n = p.cnt[lrow];
    n = n < 0 ? 0 : (n > p.idx_stride ? p.idx_stride : n);
    ntiles = (MODE == KV_TOKENS) ? ((n + 63) >> 6) : n;
  }

  // ---- loader role of this thread ------------------------------------------------
  constexpr bool SPLIT_ROLES = (D == 64);
  const int tt = SPLIT_ROLES ? (tid & 127) : tid;
  const bool k_loader = SPLIT_ROLES ? (tid < 128) : true;
  const bool v_loader = HAS_V && (SPLIT_ROLES ? (tid >= 128) : true);
  const int ld_c = tt % CPR;         // 16-byte chunk of the row
  const int ld_a = tt / CPR;         // rows 4*ld_a .. 4*ld_a+3 of the tile
  // V^T column of key 4*ld_a: the two low bits of ld_a swapped (see the PV operand below).
  const int ld_ap = (ld_a & ~3) | ((ld_a & 1) << 1) | ((ld_a >> 1) & 1);

  // Row sources of one tile for this thread.
  struct Rows {
    int row[4];
    bool ok[4];
  };
  auto raw_index = [&](int it) -> i32x4 {
    i32x4 r = {0, 0, 0, 0};
    if (it < ntiles) {
      if constexpr (MODE == KV_TOKENS) r = *reinterpret_cast<const i32x4*>(lst + it * 64 + 4 * ld_a);
      if constexpr (MODE == KV_BLOCKS) r[0] = lst[it];
    }
    return r;
  };
  auto resolve = [&](int it, i32x4 raw) -> Rows {
    Rows r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if constexpr (MODE == KV_DENSE) {
        r.row[i] = it * 64 + 4 * ld_a + i;
        r.ok[i] = r.row[i] < p.kv_len;
      } else if constexpr (MODE == KV_BLOCKS) {
        const int blk = raw[0];
        r.row[i] = blk * 64 + 4 * ld_a + i;
        r.ok[i] = blk >= 0 && blk <= (p.kv_len >> 6) && r.row[i] < p.kv_len;
      } else {
        r.row[i] = raw[i];
        r.ok[i] = (it * 64 + 4 * ld_a + i) < n && (unsigned)raw[i] < (unsigned)p.kv_len;
      }
    }
    return r;
  };

  u32x4 kr[4], vr[4];
  float bias_r[4];
  auto issue_loads = [&](const Rows& r) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const u32x4 z = {0, 0, 0, 0};
      kr[i] = z;
      vr[i] = z;
      bias_r[i] = r.ok[i] ? 0.f : kNegInf;
      if (r.ok[i]) {
        const size_t off = (size_t)r.row[i] * D + 8 * ld_c;
        if (k_loader) kr[i] = *reinterpret_cast<const u32x4*>(kh + off);
        if (v_loader) vr[i] = *reinterpret_cast<const u32x4*>(vh + off);
      }
    }
  };
  auto store_tile = [&](int stage) {
    unsigned char* kb = smem + stage * Smem::kStage;
    if (k_loader) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 4 * ld_a + i;
        *reinterpret_cast<u32x4*>(kb + r * (D * 2) + ((ld_c ^ (r & (CPR - 1))) << 4)) = kr[i];
      }
      if (MODE == KV_TOKENS && ld_c == 0) {
        float* bias = reinterpret_cast<float*>(kb + Smem::kKBytes + Smem::kVBytes);
        *reinterpret_cast<float4*>(bias + 4 * ld_a) = make_float4(bias_r[0], bias_r[1], bias_r[2], bias_r[3]);
      }
    }
    if constexpr (HAS_V) {
      if (v_loader) {
        unsigned char* vb = kb + Smem::kKBytes;
        // Transpose the 4 keys x 8 dims held in registers into 8 dims x 4 keys.
#pragma unroll
        for (int w = 0; w < 4; ++w) {
#pragma unroll
          for (int hl = 0; hl < 2; ++hl) {
            const uint32_t sel = hl ? 0x07060302u : 0x05040100u;
            u32x2 out;
            out[0] = __builtin_amdgcn_perm(vr[1][w], vr[0][w], sel);
            out[1] = __builtin_amdgcn_perm(vr[3][w], vr[2][w], sel);
            const int d = 8 * ld_c + 2 * w + hl;
            const int unit = (ld_ap >> 1) ^ ((d ^ (d >> 3)) & 7);
            *reinterpret_cast<u32x2*>(vb + d * 128 + (unit << 4) + ((ld_ap & 1) << 3)) = out;
          }
        }
      }
    }
  };

  // ---- prologue ------------------------------------------------------------------
  const int q0 = qb * QBLK + qsub * 32;
  const int qrow = q0 + ln;
  const bool qrow_ok = qrow < p.S;

  float m_run = kNegInf;   // running raw row max
  float l_run = 0.f;       // running denominator, this lane's keys only
  f32x16 oacc[HAS_V ? NDB : 1];
#pragma unroll
  for (int db = 0; db < (HAS_V ? NDB : 1); ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;

  u32x4 qf[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const u32x4 z = {0, 0, 0, 0};
    qf[t] = qrow_ok ? *reinterpret_cast<const u32x4*>(qh + (size_t)qrow * D + 16 * t + 8 * g) : z;
  }

  if (ntiles > 0) {
    i32x4 raw_cur = raw_index(0);
    i32x4 raw_nxt = raw_index(1);
    int tile_row0 = 0;   // dense/block: first key row of the current tile
    {
      Rows r0 = resolve(0, raw_cur);
      issue_loads(r0);
      store_tile(0);
    }
    __syncthreads();

    for (int it = 0; it < ntiles; ++it) {
      const int cur = it & 1;
      if constexpr (MODE == KV_DENSE) tile_row0 = it * 64;
      if constexpr (MODE == KV_BLOCKS) {
        const int blk = raw_cur[0];
        tile_row0 = (blk >= 0 && blk <= (p.kv_len >> 6)) ? blk * 64 : p.kv_len;
      }
      const bool has_next = (it + 1) < ntiles;
      if (has_next) {
        Rows rn = resolve(it + 1, raw_nxt);
        issue_loads(rn);
      }
      raw_cur = raw_nxt;
      raw_nxt = raw_index(it + 2);

      // ---- S^T = K Q^T for this wave's keys ----
      const unsigned char* kb = smem + cur * Smem::kStage;
      f32x16 s[NMB];
#pragma unroll
      for (int mb = 0; mb < NMB; ++mb) {
#pragma unroll
        for (int r = 0; r < 16; ++r) s[mb][r] = 0.f;
        const int krow = ksub * KW + mb * 32 + ln;
        const unsigned char* krp = kb + krow * (D * 2);
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          const u32x4 a = *reinterpret_cast<const u32x4*>(krp + (((2 * t + g) ^ (krow & (CPR - 1))) << 4));
          s[mb] = mfma32(a, qf[t], s[mb]);
        }
      }

      // ---- mask keys that do not exist ----
      // Accumulator register 4j+i of block mb is key ksub*KW + 32mb + 8j + 4g + i of the tile.
      if constexpr (MODE == KV_TOKENS) {
        const float* bias = reinterpret_cast<const float*>(kb + Smem::kKBytes + Smem::kVBytes);
#pragma unroll
        for (int mb = 0; mb < NMB; ++mb)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float4 bv = *reinterpret_cast<const float4*>(bias + ksub * KW + 32 * mb + 8 * j + 4 * g);
            s[mb][4 * j + 0] += bv.x;
            s[mb][4 * j + 1] += bv.y;
            s[mb][4 * j + 2] += bv.z;
            s[mb][4 * j + 3] += bv.w;
          }
      } else {
        if (tile_row0 + 64 > p.kv_len) {
#pragma unroll
          for (int mb = 0; mb < NMB; ++mb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const int key = tile_row0 + ksub * KW + 32 * mb + 8 * (r >> 2) + 4 * g + (r & 3);
              if (key >= p.kv_len) s[mb][r] = kNegInf;
            }
        }
      }

      // ---- online softmax; one query row per lane ----
      float mloc = s[0][0];
#pragma unroll
      for (int mb = 0; mb < NMB; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) mloc = fmaxf(mloc, s[mb][r]);
      mloc = fmaxf(mloc, xor32(mloc));
      const float m_new = fmaxf(m_run, mloc);
      const float msf = (m_new == kNegInf) ? 0.f : m_new * p.sf;
      const float alpha = __builtin_amdgcn_exp2f(m_run * p.sf - msf);
      m_run = m_new;
      float psum = 0.f;
#pragma unroll
      for (int mb = 0; mb < NMB; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(s[mb][r], p.sf, -msf));
          s[mb][r] = e;
          psum += e;
        }
      l_run = l_run * alpha + psum;

      if constexpr (HAS_V) {
        if (__any(alpha != 1.f)) {
#pragma unroll
          for (int db = 0; db < NDB; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;
        }
        // P^T operand: registers 8h..8h+7 of block mb are the 8 keys this lane feeds to
        // k-step 2mb+h; the V^T tile stores those keys at columns 16(2mb+h) + 8g + 0..7.
        u32x4 pb[NKS];
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
          const int mb = ks >> 1, h8 = (ks & 1) * 8;
          pb[ks][0] = pack_bf16(s[mb][h8 + 0], s[mb][h8 + 1]);
          pb[ks][1] = pack_bf16(s[mb][h8 + 2], s[mb][h8 + 3]);
          pb[ks][2] = pack_bf16(s[mb][h8 + 4], s[mb][h8 + 5]);
          pb[ks][3] = pack_bf16(s[mb][h8 + 6], s[mb][h8 + 7]);
        }
        const unsigned char* vb = kb + Smem::kKBytes;
#pragma unroll
        for (int db = 0; db < NDB; ++db) {
          const int d = 32 * db + ln;
          const unsigned char* vrp = vb + d * 128;
          const int hsw = (d ^ (d >> 3)) & 7;
#pragma unroll
          for (int ks = 0; ks < NKS; ++ks) {
            const int unit = (ksub * KW + 16 * ks + 8 * g) >> 3;
            const u32x4 a = *reinterpret_cast<const u32x4*>(vrp + ((unit ^ hsw) << 4));
            oacc[db] = mfma32(a, pb[ks], oacc[db]);
          }
        }
      }

      if (has_next) store_tile(cur ^ 1);
      __syncthreads();
    }
  }

  // ---- combine the two 32-lane halves, then the two key halves -------------------
  float l_tot = l_run + xor32(l_run);
  if constexpr (KSPLIT == 2) {
    float* mg = reinterpret_cast<float*>(smem) + qsub * ((HAS_V ? D / 2 : 0) + 2) * 64;
    if (ksub == 1) {
      mg[lane] = m_run;
      mg[64 + lane] = l_tot;
      if constexpr (HAS_V) {
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
          for (int r = 0; r < 16; ++r) mg[(2 + db * 16 + r) * 64 + lane] = oacc[db][r];
      }
    }
    __syncthreads();
    if (ksub == 1) return;
    const float m2 = mg[lane];
    const float l2 = mg[64 + lane];
    const float m_new = fmaxf(m_run, m2);
    const float msf = (m_new == kNegInf) ? 0.f : m_new * p.sf;
    const float a1 = __builtin_amdgcn_exp2f(m_run * p.sf - msf);
    const float a2 = __builtin_amdgcn_exp2f(m2 * p.sf - msf);
    l_tot = l_tot * a1 + l2 * a2;
    m_run = m_new;
    if constexpr (HAS_V) {
#pragma unroll
      for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[db][r] = oacc[db][r] * a1 + mg[(2 + db * 16 + r) * 64 + lane] * a2;
    }
  }

  // ---- epilogue --------------------------------------------------------------------
  if constexpr (HAS_V) {
    if (qrow_ok) {
      const float inv = (l_tot > 0.f) ? 1.f / l_tot : 0.f;
      uint16_t* orow = p.o + head_off + (size_t)qrow * D;
#pragma unroll
      for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          u32x2 w;
          w[0] = pack_bf16(oacc[db][4 * j + 0] * inv, oacc[db][4 * j + 1] * inv);
          w[1] = pack_bf16(oacc[db][4 * j + 2] * inv, oacc[db][4 * j + 3] * inv);
          *reinterpret_cast<u32x2*>(orow + 32 * db + 8 * j + 4 * g) = w;
        }
    }
  }
  if (g == 0) {
    if (p.lse != nullptr && qrow_ok) {
      p.lse[(size_t)bh * p.S + qrow] = (l_tot > 0.f) ? (m_run * p.scale + __logf(l_tot)) : kNegInf;
    }
    if constexpr (STATS) {
      // Pad rows keep the reference convention max_q = 0, denom = -inf
      // (include/maxq_denom.cuh:202-205).
      if (qrow < p.Sp) {
        const size_t so = (size_t)bh * p.Sp + qrow;
        p.max_q[so] = (qrow_ok && m_run != kNegInf) ? m_run : 0.f;
        p.denom[so] = qrow_ok ? l_tot : kNegInf;
      }
    }
  }
}

// Host launcher; returns hipError_t of the launch.
template <int D, int QBLK, int MODE, bool HAS_V, bool STATS>
inline hipError_t launch_attn_fwd(const AttnParams& p, hipStream_t stream) {
  using Smem = AttnSmem<D, HAS_V>;
  auto kern = attn_fwd_kernel<D, QBLK, MODE, HAS_V, STATS>;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, Smem::kTotal);
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  const int total = p.nqblk * p.H * p.B;
  if (total <= 0) return hipSuccess;
  hipLaunchKernelGGL(kern, dim3(total), dim3(256), Smem::kTotal, stream, p);
  return hipGetLastError();
}

}  // namespace spattn
