// Flash-style attention forward for gfx950, one kernel template for the dense,
// token-list and block-list variants.
//
// What it computes follows the reference kernels
//   include/sparseattn_asyncgatherload_padded.cuh:204-255 (gathered sparse attention),
//   include/fullattn_wgload_padded.cuh:190-232          (dense attention),
//   include/maxq_denom_attn.cuh:196-252                 (dense attention + row statistics),
//   include/maxq_denom.cuh:169-206                      (row statistics only):
// running row max, p = exp2((s - m) * log2e * scale), fp32 denominator, P rounded to bf16
// before PV, O / l at the end.  Keys that do not exist (list position >= n, token id >=
// kv_len, row >= kv_len) are masked on every tile, a superset of the reference's "NaN row
// -> -inf on the last tile" (include/asyncloadutils.cuh:124-142, include/pad_utils.cuh:54-75).
//
// Work split.  A workgroup is 4 waves (256 lanes) and owns one q-block of QBLK rows.
// Scores are produced transposed, S^T = K Q^T, so that in the 32x32 MFMA accumulator a
// lane holds ONE query row (n = lane & 31) and 16 keys: every softmax statistic is a
// per-lane scalar and only lanes l and l^32 ever exchange data.  O is accumulated
// transposed too, O^T += V^T P^T, with P^T taken straight from the score accumulators.
//   QBLK = 128: wave w owns query rows 32w..32w+31 and all 64 keys of a tile.
//   QBLK =  64: wave w owns query rows 32(w&1).. and keys 32(w>>1).. of a tile; the two
//               key halves are merged through LDS at the end.
//
// Data movement.  K and V tiles (64 rows x D bf16, row-major as in HBM) go HBM -> LDS with
// global_load_lds_dwordx4: no staging registers, no LDS stores.  Each lane picks which
// 16-byte chunk of its row it fetches so that the tile lands XOR-swizzled (chunk ^ swz(row),
// one swizzle for K and V).  K is read back as the MFMA A operand with ds_read_b128; the
// V^T operand comes from ds_read_b64_tr_b16, which hands lane j of a 16-lane group the
// j-th 16-bit column of the 4 rows the group addressed.
//
// Schedule.  Tiles are consumed in "phases" K0 | K1 V0 | K2 V1 | ... : the scores of tile
// i+1 are multiplied while the softmax of tile i runs on the vector ALU, and the row
// maxima of tile i+1 are reduced while P_i V_i is multiplied.  Phase j lives in ring slot
// j & 3; every phase is  wait (own loads of this phase) -> barrier -> issue phase j+3 into
// the slot the barrier just freed -> multiply.  The steady-state loop is unrolled over two
// tiles so that every slot is a compile-time constant: LDS addresses are a per-lane base
// plus an instruction immediate, the wait counts are literals, and the loop carries almost
// no scalar or address arithmetic - the instruction issue rate, not the matrix pipe, is
// what bounds this kernel.
#pragma once
#include <type_traits>

#include "common.h"

namespace spattn {

typedef __attribute__((ext_vector_type(4))) short s16x4;
#define SPATTN_LDS __attribute__((address_space(3)))
typedef SPATTN_LDS const unsigned char* lds_cptr;

template <int D, int MODE, bool HAS_V>
struct AttnCfg {
  static constexpr int kTileBytes = 64 * D * 2;
  static constexpr int kSlots = 4;
  static constexpr int kBiasRing = 8;                         // tiles of key-validity bias (token lists)
  static constexpr int kBiasBytes = (MODE == KV_TOKENS) ? kBiasRing * 64 * 4 : 0;
  static constexpr int kRing = kSlots * kTileBytes;
  static constexpr int kMerge = 2 * (D / 2 + 3) * 64 * 4;     // key-split merge, overlays the ring
  static constexpr int kTotal = ((kRing > kMerge) ? kRing : kMerge) + kBiasBytes;
  static constexpr int kRowsPerLoad = 1024 / (D * 2);         // rows one wave-wide 1 KB load covers
  static constexpr int kLoadsPerTile = kTileBytes / 1024 / 4;   // per wave
};

// One wave-wide HBM -> LDS copy: lane l's 16 bytes land at lds_base + 16 l.
// Written as asm on purpose: the compiler does not count this load in its own vmcnt
// bookkeeping (with the builtin it drains every outstanding load before each LDS read),
// so the waits are placed by hand.
__device__ __forceinline__ void dma16(const void* gptr, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_base), "v"(gptr) : "memory");
}
// Same with a wave-uniform base pointer and a 32-bit per-lane byte offset.
__device__ __forceinline__ void dma16(const void* sbase, uint32_t voff, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_base), "v"(voff), "s"(sbase) : "memory");
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

template <int D, int QBLK, int MODE, bool HAS_V, bool STATS>
__global__ __launch_bounds__(256, 2) void attn_fwd_kernel(const AttnParams p) {
  static_assert(D == 64 || D == 128, "head dim");
  static_assert(QBLK == 64 || QBLK == 128, "q-block");
  using Cfg = AttnCfg<D, MODE, HAS_V>;
  constexpr int NQW = QBLK / 32;     // waves along the query rows
  constexpr int KSPLIT = 4 / NQW;    // waves along the keys of a tile
  constexpr int KW = 64 / KSPLIT;    // keys of a tile per wave
  constexpr int NMB = KW / 32;       // 32-key score blocks per wave
  constexpr int NT = D / 16;         // k-steps of the QK^T product
  constexpr int NDB = D / 32;        // 32-wide blocks of the head dim
  constexpr int CPR = D / 8;         // 16-byte chunks per row
  constexpr int ROWB = D * 2;        // bytes per row
  constexpr int TILE = Cfg::kTileBytes;
  constexpr int LPT = Cfg::kLoadsPerTile;
  constexpr int RPL = Cfg::kRowsPerLoad;
  constexpr float kNegInf = -__builtin_huge_valf();

  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  const lds_cptr smem_l = (lds_cptr)smem;
  const uint32_t smem_base = (uint32_t)(uintptr_t)smem_l;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
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
  const unsigned char* __restrict__ kh = reinterpret_cast<const unsigned char*>(p.k + head_off);
  const unsigned char* __restrict__ vh = HAS_V ? reinterpret_cast<const unsigned char*>(p.v + head_off) : nullptr;

  // ---- tile list of this q-block -------------------------------------------------
  // The lists are read through the constant address space: with a wave-uniform address
  // that makes them scalar loads, which stay out of the vector-memory counter that the
  // tile pipeline waits on.
  typedef const __attribute__((address_space(4))) int* cint_p;
  cint_p lst = nullptr;
  int n = 0, ntiles = 0;
  if constexpr (MODE == KV_DENSE) {
    ntiles = (p.kv_len + 63) >> 6;
  } else {
    const size_t lrow = (size_t)bh * p.nqblk + qb;
    lst = (cint_p)(p.idx + lrow * p.idx_stride);
    n = ((cint_p)p.cnt)[lrow];
    n = n < 0 ? 0 : (n > p.idx_stride ? p.idx_stride : n);
    ntiles = (MODE == KV_TOKENS) ? ((n + 63) >> 6) : n;
  }
  const int last_row = p.kv_len - 1;
  // Phase numbers: with V, 0 = K0, 2i+1 = K(i+1), 2i+2 = V(i); phase 2*ntiles-1 would be a
  // K tile past the end and is never issued.  Without V, phase j = K(j).
  const int last_phase = HAS_V ? 2 * ntiles : ntiles - 1;

  // ---- loader role: load i of a tile covers rows RPL*(4i + wave) .. +RPL-1 ----------
  const int ld_sub = lane / CPR;       // row within the load
  const int ld_slot = lane % CPR;      // 16-byte position within the row in LDS
  // Row r of a tile stores its 16-byte chunk c at position c ^ swz(r).  The swizzle has a
  // period of 16 rows and is chosen so that (K reads, ds_read_b128) one chunk of 16
  // consecutive rows covers all sixteen 16-byte bank groups, and (transposing V reads) the
  // two 32-byte windows that a read takes from each of four consecutive rows cover all
  // eight 32-byte windows: both reads then run at the full LDS rate (measured: twice,
  // resp. 1.45 times, the rate of a swizzle that only separates 8 rows).
  auto swz = [](int r) -> int {
    return D == 128 ? (((r & 3) << 2) | ((r >> 2) & 3)) : ((((r >> 1) & 1) << 2) | ((r >> 2) & 3));
  };
  auto ld_row = [&](int i) -> int { return RPL * (4 * i + wave) + ld_sub; };
  auto ld_off = [&](int i) -> int { return (ld_slot ^ swz(ld_row(i))) << 4; };   // chunk offset within the row
  uint32_t ld_go[LPT];                 // lane offset within a contiguous 64-row tile
#pragma unroll
  for (int i = 0; i < LPT; ++i) ld_go[i] = ld_row(i) * ROWB + ld_off(i);

  // First key row of a tile (dense / block lists) from its id; kv_len marks "no such block".
  // The id of tile t is t itself (dense) or the t-th list entry (block lists).
  auto tile_id = [&](int t) -> int {
    if constexpr (MODE == KV_BLOCKS) return lst[t];
    return t;
  };
  auto id_row0 = [&](int blk) -> int {
    if constexpr (MODE == KV_DENSE) return blk * 64;
    if constexpr (MODE == KV_BLOCKS) return (blk >= 0 && blk <= (last_row >> 6)) ? blk * 64 : p.kv_len;
    return 0;
  };
  // Same, for a tile that may lie past the end of the list (prefetched ids that are never used).
  auto tile_id_clamped = [&](int t) -> int {
    if constexpr (MODE == KV_BLOCKS) return lst[t < p.idx_stride ? t : p.idx_stride - 1];
    return t;
  };

  // Token lists: the RPL token ids behind one load are wave-uniform, so they are fetched
  // as scalars (tok_raw) one tile ahead and turned into this lane's row (tok_row) just
  // before the K load of that tile is issued; V tiles are issued one tile later and take
  // their rows from a two-deep queue.
  int tok_raw[MODE == KV_TOKENS ? LPT : 1][MODE == KV_TOKENS ? RPL : 1];
  int tok_row[MODE == KV_TOKENS ? LPT : 1];      // rows of the next K tile to issue
  int tok_row_v0[MODE == KV_TOKENS ? LPT : 1];   // rows of the next V tile to issue
  int tok_row_v1[MODE == KV_TOKENS ? LPT : 1];   // rows of the V tile after that
  bool tok_ok[MODE == KV_TOKENS ? LPT : 1];
  auto tok_fetch = [&](int t) {
    if constexpr (MODE == KV_TOKENS) {
#pragma unroll
      for (int i = 0; i < LPT; ++i)
#pragma unroll
        for (int s = 0; s < RPL; ++s) tok_raw[i][s] = (t < ntiles) ? lst[t * 64 + RPL * (4 * i + wave) + s] : 0;
    }
  };
  auto tok_resolve = [&](int t) {
    if constexpr (MODE == KV_TOKENS) {
#pragma unroll
      for (int i = 0; i < LPT; ++i) {
        int tok = 0;
#pragma unroll
        for (int s = 0; s < RPL; ++s) {
          int v = tok_raw[i][s];
          v = __builtin_amdgcn_readfirstlane(v);   // keeps the list a scalar load (no per-lane reload)
          tok = (ld_sub == s) ? v : tok;
        }
        tok_ok[i] = (t * 64 + ld_row(i)) < n && (unsigned)tok <= (unsigned)last_row;
        tok_row[i] = tok_ok[i] ? tok : 0;
      }
    }
  };

  // Loads of one K or V tile into ring slot `slot`: prepare() resolves the wave-uniform
  // base and this lane's byte offsets, load(i) issues the i-th of the LPT wave-wide copies.
  // Issue order of the tiles is K0 K1 V0 K2 V1 ..., which the token-row queue relies on.
  struct TileLoad {
    const unsigned char* base;
    uint32_t lds;
    uint32_t go[LPT];
  };
  auto prepare_tile = [&](int t, int id, int slot, bool is_v) -> TileLoad {
    TileLoad tl;
    tl.lds = smem_base + (uint32_t)slot * TILE + wave * 1024;
    const unsigned char* src = is_v ? vh : kh;
    if constexpr (MODE == KV_TOKENS) {
      tl.base = src;
      float* bias = reinterpret_cast<float*>(smem + Cfg::kTotal - Cfg::kBiasBytes) + (t % Cfg::kBiasRing) * 64;
#pragma unroll
      for (int i = 0; i < LPT; ++i) {
        const int row = is_v ? tok_row_v0[i] : tok_row[i];
        tl.go[i] = (uint32_t)row * ROWB + ld_off(i);
        if (!is_v && ld_slot == 0) bias[ld_row(i)] = tok_ok[i] ? 0.f : kNegInf;
      }
      if (is_v) {
#pragma unroll
        for (int i = 0; i < LPT; ++i) tok_row_v0[i] = tok_row_v1[i];
      } else {
#pragma unroll
        for (int i = 0; i < LPT; ++i) {
          if (t == 0) tok_row_v0[i] = tok_row[i];
          tok_row_v1[i] = tok_row[i];
        }
        tok_resolve(t + 1);
        tok_fetch(t + 2);
      }
    } else {
      const int r0 = id_row0(id);
      if (r0 + 64 <= p.kv_len) {
        tl.base = src + (size_t)r0 * ROWB;   // whole tile in range
#pragma unroll
        for (int i = 0; i < LPT; ++i) tl.go[i] = ld_go[i];
      } else {
        // ragged last tile: rows past the end re-read the last row and are masked later
        tl.base = src;
#pragma unroll
        for (int i = 0; i < LPT; ++i) {
          int row = r0 + ld_row(i);
          row = row > last_row ? last_row : row;
          tl.go[i] = (uint32_t)row * ROWB + ld_off(i);
        }
      }
    }
    return tl;
  };
  auto load_part = [&](const TileLoad& tl, int i) { dma16(tl.base, tl.go[i], tl.lds + i * 4096); };
  auto issue_tile = [&](int t, int slot, bool is_v) {
    const TileLoad tl = prepare_tile(t, tile_id(t), slot, is_v);
#pragma unroll
    for (int i = 0; i < LPT; ++i) load_part(tl, i);
  };
  auto phase_exists = [&](int j) -> bool {
    if (j > last_phase) return false;
    if constexpr (HAS_V) return j != 2 * ntiles - 1;
    return true;
  };
  // Generic form: issue phase j if it exists.
  auto issue_phase = [&](int j) {
    if (!phase_exists(j)) return;
    if constexpr (HAS_V) {
      if (j == 0) issue_tile(0, 0, false);
      else if (j & 1) issue_tile((j + 1) / 2, j & 3, false);
      else issue_tile(j / 2 - 1, j & 3, true);
    } else {
      issue_tile(j, j & 3, false);
    }
  };
  // Generic wait for phase j: phases j+1 and j+2, if they exist, may stay in flight.
  auto wait_generic = [&](int j) {
    const int later = (phase_exists(j + 1) ? 1 : 0) + (phase_exists(j + 2) ? 1 : 0);
    if (later == 2) wait_vmcnt<2 * LPT>();
    else if (later == 1) wait_vmcnt<LPT>();
    else wait_vmcnt<0>();
  };

  // ---- prologue ------------------------------------------------------------------
  const int q0 = qb * QBLK + qsub * 32;
  const int qrow = q0 + ln;
  const bool qrow_ok = qrow < p.S;

  tok_fetch(0);
  tok_resolve(0);
  tok_fetch(1);
  issue_phase(0);
  // The Q loads are the only compiler-visible vector loads of the kernel.  They go out
  // between the first copies so that their latency overlaps that of tile 0, and must have
  // retired before the first counted wait.
  u32x4 qf[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const u32x4 z = {0, 0, 0, 0};
    qf[t] = qrow_ok ? *reinterpret_cast<const u32x4*>(qh + (size_t)qrow * D + 16 * t + 8 * g) : z;
  }
  issue_phase(1);
  issue_phase(2);
#pragma unroll
  for (int t = 0; t < NT; ++t) asm volatile("" ::"v"(qf[t]));

  // Softmax state of this lane's query row.  Exponents are taken against a reference
  // mr_sf (in log2 units, = raw max * sf at the time it was set) that is only moved when
  // some row of the wave outgrows it by more than kSlack: p = exp2(s*sf - mr_sf) may then
  // exceed 1 (by at most 2^kSlack), which fp32 sums and bf16 P hold without loss, and the
  // O / l rescale is skipped on most tiles.  m_true tracks the true raw max for the
  // statistics outputs.
  constexpr float kSlack = 8.f;
  float mr_sf = kNegInf;
  float m_true = kNegInf;
  float l_run = 0.f;       // running denominator, this lane's keys only
  f32x16 oacc[HAS_V ? NDB : 1];
#pragma unroll
  for (int db = 0; db < (HAS_V ? NDB : 1); ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;

  u32x4 pb[HAS_V ? 2 * NMB : 1];   // P^T operands, k-step 2mb + h

  // Per-lane LDS addresses inside slot 0; slot, score block and k-step offsets are added
  // as constants (instruction immediates in the unrolled loop).
  lds_cptr k_lo[NT];       // A operand of QK^T, k-step t, score block 0
  {
    const int krow = ksub * KW + ln;
#pragma unroll
    for (int t = 0; t < NT; ++t) k_lo[t] = smem_l + krow * ROWB + (((2 * t + g) ^ swz(krow)) << 4);
  }
  // Transposing V read: in each 16-lane group, lane i addresses 4 dims of key (i>>2);
  // lane j receives dim j of those 4 keys.  Keys 4g..4g+3 (+8 for the second read) of
  // each 16-key step, dims 32db + 16*dhalf + 4*(i&3)..+3.
  lds_cptr v_lo[HAS_V ? NDB : 1];    // keys 4g..4g+3 of a step
  lds_cptr v_lo2[HAS_V ? NDB : 1];   // keys 8+4g..8+4g+3 of a step (their rows have another swizzle)
  if constexpr (HAS_V) {
    const int i16 = lane & 15;
    const int dhalf = (lane >> 4) & 1;
    const int r1 = ksub * KW + 4 * g + (i16 >> 2);
    const int cb = 2 * dhalf + ((i16 & 3) >> 1);
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
      v_lo[db] = smem_l + r1 * ROWB + (((4 * db + cb) ^ swz(r1)) << 4) + ((i16 & 1) << 3);
      v_lo2[db] = smem_l + (r1 + 8) * ROWB + (((4 * db + cb) ^ swz(r1 + 8)) << 4) + ((i16 & 1) << 3);
    }
  }

  // ---- building blocks --------------------------------------------------------------
  // Keys of tile `it` that do not exist get -inf.  Accumulator register 4j+i of block mb
  // is key ksub*KW + 32mb + 8j + 4g + i of the tile.
  auto mask_tile = [&](int it, int id, f32x16 (&s)[NMB]) {
    if constexpr (MODE == KV_TOKENS) {
      const float* bias = reinterpret_cast<const float*>(smem + Cfg::kTotal - Cfg::kBiasBytes) + (it % Cfg::kBiasRing) * 64;
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
      const int r0 = id_row0(id);
      if (r0 + 64 > p.kv_len) {
#pragma unroll
        for (int mb = 0; mb < NMB; ++mb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int key = r0 + ksub * KW + 32 * mb + 8 * (r >> 2) + 4 * g + (r & 3);
            if (key >= p.kv_len) s[mb][r] = kNegInf;
          }
      }
    }
  };
  // Row max of a score tile (both 32-lane halves); returns max * sf.
  auto row_stats = [&](const f32x16 (&s)[NMB]) -> float {
    float mloc = s[0][0];
#pragma unroll
    for (int mb = 0; mb < NMB; ++mb)
#pragma unroll
      for (int r = 0; r < 16; ++r) mloc = fmaxf(mloc, s[mb][r]);
    mloc = pair_max(mloc);
    m_true = fmaxf(m_true, mloc);
    return mloc * p.sf;
  };
  // Move the exponent reference if some row of the wave outgrew it; rescales O and l.
  auto maybe_rescale = [&](float mloc_sf) {
    if (__any(mloc_sf > mr_sf + kSlack)) {
      const float new_sf = fmaxf(mr_sf, mloc_sf);
      const float alpha = (new_sf == kNegInf) ? 1.f : __builtin_amdgcn_exp2f(mr_sf - new_sf);
      mr_sf = new_sf;
      l_run *= alpha;
      if constexpr (HAS_V) {
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
          for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;
      }
    }
  };
  // p = exp2(s*sf - reference) for registers r0..r0+cnt-1 of block mb; adds to the row sum
  // and leaves P^T as bf16 MFMA operands (k-step 2mb+h takes registers 8h..8h+7 of block
  // mb, i.e. keys 32mb + 16h + {4g..4g+3} and 32mb + 16h + 8 + {4g..4g+3}).
  auto softmax_chunk = [&](f32x16 (&s)[NMB], float base, int mb, int r0, int cnt) {
#pragma unroll
    for (int r = r0; r < r0 + cnt; r += 2) {
      const float e0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[mb][r], p.sf, -base));
      const float e1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[mb][r + 1], p.sf, -base));
      l_run += e0;
      l_run += e1;
      if constexpr (HAS_V) pb[2 * mb + (r >> 3)][(r & 7) >> 1] = pack_bf16(e0, e1);
    }
  };
  // Pin the softmax results where they are produced; otherwise the compiler sinks the
  // whole softmax to the first use of P, behind the next barrier, and nothing overlaps
  // the MFMAs.
  auto pin_softmax = [&]() {
    asm volatile("" : "+v"(l_run));
    if constexpr (HAS_V) {
#pragma unroll
      for (int ks = 0; ks < 2 * NMB; ++ks)
#pragma unroll
        for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(pb[ks][i]));
    }
  };
  auto softmax_only = [&](f32x16 (&s)[NMB]) {
    const float base = (mr_sf == kNegInf) ? 0.f : mr_sf;
#pragma unroll
    for (int mb = 0; mb < NMB; ++mb) softmax_chunk(s, base, mb, 0, 16);
  };
  // s_out^T = K Q^T from the K tile at ring offset kofs (bytes), one 32-key block at a
  // time; if WITH_SM, the softmax of s_in is interleaved: one MFMA, then the vector-ALU
  // work of 16/NT score registers.
  auto qk_tile = [&](auto with_sm, uint32_t kofs, f32x16 (&s_out)[NMB], f32x16 (&s_in)[NMB], const TileLoad* tl) {
    constexpr bool WITH_SM = decltype(with_sm)::value;
    constexpr int EPM = 16 / NT;
    const float base = (mr_sf == kNegInf) ? 0.f : mr_sf;
#pragma unroll
    for (int mb = 0; mb < NMB; ++mb) {
      u32x4 ka[NT];
#pragma unroll
      for (int t = 0; t < NT; ++t) ka[t] = *(SPATTN_LDS const u32x4*)(k_lo[t] + kofs + mb * 32 * ROWB);
      __builtin_amdgcn_sched_barrier(0);   // all reads in flight before the first multiply
#pragma unroll
      for (int r = 0; r < 16; ++r) s_out[mb][r] = 0.f;
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        s_out[mb] = mfma32(ka[t], qf[t], s_out[mb]);
        if constexpr (WITH_SM) softmax_chunk(s_in, base, mb, t * EPM, EPM);
        // the next tile's copies are spread over the multiplies: issued in one burst they
        // queue behind the other waves' copies and stall this wave
        if (tl != nullptr) {
          constexpr int STEP = (NMB * NT) / LPT;
          const int m = mb * NT + t;
          if (m % STEP == STEP - 1) load_part(*tl, m / STEP);
        }
      }
      if constexpr (WITH_SM) {
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);            // one MFMA
          __builtin_amdgcn_sched_group_barrier(0x002, EPM * 7 / 2, 0);  // its share of the softmax
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (WITH_SM) pin_softmax();
  };
  // O^T += V^T P^T from the V tile at ring offset vofs, two 16-key steps at a time.
  auto pv_tile = [&](uint32_t vofs, const TileLoad* tl) {
    if constexpr (HAS_V) {
#pragma unroll
      for (int mb = 0; mb < NMB; ++mb) {
        u32x2 va[2][NDB][2];
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int db = 0; db < NDB; ++db) {
            const lds_cptr a1 = v_lo[db] + vofs + (2 * mb + h) * 16 * ROWB;
            const lds_cptr a2 = v_lo2[db] + vofs + (2 * mb + h) * 16 * ROWB;
            va[h][db][0] = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((SPATTN_LDS s16x4*)a1));
            va[h][db][1] = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((SPATTN_LDS s16x4*)a2));
          }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int db = 0; db < NDB; ++db) {
            const u32x4 a = {va[h][db][0][0], va[h][db][0][1], va[h][db][1][0], va[h][db][1][1]};
            oacc[db] = mfma32(a, pb[2 * mb + h], oacc[db]);
            if (tl != nullptr) {   // the next tile's copies, spread over the multiplies
              constexpr int STEP = (NMB * 2 * NDB) / LPT;
              const int m = (mb * 2 + h) * NDB + db;
              if (m % STEP == STEP - 1) load_part(*tl, m / STEP);
            }
          }
      }
    }
  };

  // One tile of the pipeline: K phase of tile it+1 (ring slot KS) with the softmax of tile
  // it (scores in s_a), then V phase of tile it (ring slot VS) with the row maxima of tile
  // it+1 (scores in s_b).  In the steady state every later phase exists, so waits and
  // issues are unconditional.
  // id_v / id_k: ids of tiles it+1 and it+3 (it+4 without V), fetched ahead of time by the
  // steady loop so that no list load sits between a barrier and the copies behind it;
  // the generic form looks them up itself.
  auto tile_body = [&](auto ks_c, auto vs_c, auto steady_c, int it, f32x16 (&s_a)[NMB], f32x16 (&s_b)[NMB], int id_v, int id_k) {
    constexpr int KS = decltype(ks_c)::value;
    constexpr int VS = decltype(vs_c)::value;
    constexpr bool STEADY = decltype(steady_c)::value;
    {
      const int j = HAS_V ? 2 * it + 1 : it + 1;
      if constexpr (STEADY) wait_vmcnt<2 * LPT>(); else wait_generic(j);
      __syncthreads();
      // phase j+3 is V(it+1) (with V) or K(it+4)
      if constexpr (STEADY) {
        const TileLoad tl = HAS_V ? prepare_tile(it + 1, id_v, (VS + 2) & 3, true) : prepare_tile(it + 4, id_k, (KS + 3) & 3, false);
        qk_tile(std::true_type{}, KS * TILE, s_b, s_a, &tl);
      } else {
        if constexpr (HAS_V) {
          if (it + 1 < ntiles) issue_tile(it + 1, (VS + 2) & 3, true);
        } else {
          if (it + 4 < ntiles) issue_tile(it + 4, (KS + 3) & 3, false);
        }
        qk_tile(std::true_type{}, KS * TILE, s_b, s_a, nullptr);
      }
      mask_tile(it + 1, STEADY ? id_v : tile_id(it + 1), s_b);
    }
    if constexpr (HAS_V) {
      const int j = 2 * it + 2;
      if constexpr (STEADY) wait_vmcnt<2 * LPT>(); else wait_generic(j);
      __syncthreads();
      // phase j+3 is K(it+3)
      if constexpr (STEADY) {
        const TileLoad tl = prepare_tile(it + 3, id_k, KS, false);
        pv_tile(VS * TILE, &tl);
      } else {
        if (it + 3 < ntiles) issue_tile(it + 3, KS, false);
        pv_tile(VS * TILE, nullptr);
      }
    }
    maybe_rescale(row_stats(s_b));
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;

  if (ntiles > 0) {
    f32x16 s_e[NMB], s_o[NMB];   // scores of even / odd tiles
    // phase 0: scores of tile 0
    wait_generic(0);
    __syncthreads();
    issue_phase(3);
    qk_tile(std::false_type{}, 0, s_e, s_e, nullptr);
    mask_tile(0, tile_id(0), s_e);
    maybe_rescale(row_stats(s_e));

    int it = 0;
    if constexpr (HAS_V) {
      // tile `it` has its next K tile in slot (2it+1)&3 and its V tile in slot (2it+2)&3
      // w1..w3: ids of tiles it+1..it+3; two more are fetched per round, a round ahead
      int w1 = 0, w2 = 0, w3 = 0;
      if (4 < ntiles) {
        w1 = tile_id(1);
        w2 = tile_id(2);
        w3 = tile_id(3);
      }
      for (; it + 4 < ntiles; it += 2) {
        const int w4 = tile_id(it + 4);
        const int w5 = tile_id_clamped(it + 5);
        tile_body(I1{}, I2{}, std::true_type{}, it, s_e, s_o, w1, w3);
        tile_body(I3{}, I0{}, std::true_type{}, it + 1, s_o, s_e, w2, w4);
        w1 = w3;
        w2 = w4;
        w3 = w5;
      }
      for (; it + 1 < ntiles; ++it) {
        if (it & 1) tile_body(I3{}, I0{}, std::false_type{}, it, s_o, s_e, 0, 0);
        else tile_body(I1{}, I2{}, std::false_type{}, it, s_e, s_o, 0, 0);
      }
      if (it & 1) softmax_only(s_o); else softmax_only(s_e);
      wait_vmcnt<0>();
      __syncthreads();
      pv_tile((uint32_t)((2 * ntiles) & 3) * TILE, nullptr);
    } else {
      // tile it+1 sits in K slot (it+1)&3
      for (; it + 1 < ntiles; ++it) {
        switch ((it + 1) & 3) {
          case 0: tile_body(I0{}, I0{}, std::false_type{}, it, s_e, s_o, 0, 0); break;
          case 1: tile_body(I1{}, I0{}, std::false_type{}, it, s_e, s_o, 0, 0); break;
          case 2: tile_body(I2{}, I0{}, std::false_type{}, it, s_e, s_o, 0, 0); break;
          default: tile_body(I3{}, I0{}, std::false_type{}, it, s_e, s_o, 0, 0); break;
        }
#pragma unroll
        for (int mb = 0; mb < NMB; ++mb) s_e[mb] = s_o[mb];
      }
      softmax_only(s_e);
    }
  }
  __syncthreads();   // every wave is done with the ring

  // ---- combine the two 32-lane halves, then the two key halves -------------------
  float l_tot = pair_sum(l_run);
  if constexpr (KSPLIT == 2) {
    float* mg = reinterpret_cast<float*>(smem) + qsub * ((HAS_V ? D / 2 : 0) + 3) * 64;
    if (ksub == 1) {
      mg[lane] = mr_sf;
      mg[64 + lane] = l_tot;
      mg[128 + lane] = m_true;
      if constexpr (HAS_V) {
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
          for (int r = 0; r < 16; ++r) mg[(3 + db * 16 + r) * 64 + lane] = oacc[db][r];
      }
    }
    __syncthreads();
    if (ksub == 1) return;
    const float m2 = mg[lane];
    const float l2 = mg[64 + lane];
    m_true = fmaxf(m_true, mg[128 + lane]);
    const float new_sf = fmaxf(mr_sf, m2);
    const float a1 = (mr_sf == kNegInf) ? 0.f : __builtin_amdgcn_exp2f(mr_sf - new_sf);
    const float a2 = (m2 == kNegInf) ? 0.f : __builtin_amdgcn_exp2f(m2 - new_sf);
    l_tot = l_tot * a1 + l2 * a2;
    mr_sf = new_sf;
    if constexpr (HAS_V) {
#pragma unroll
      for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[db][r] = oacc[db][r] * a1 + mg[(3 + db * 16 + r) * 64 + lane] * a2;
    }
  }

  // ---- epilogue --------------------------------------------------------------------
  // The wave's 32 x D output tile is one contiguous piece of O.  It is turned from "a lane
  // holds a row" into "a lane holds 16 consecutive bytes" through a wave-private piece of
  // LDS (row pitch + 8 bytes: conflict-free both ways), so that every store instruction
  // writes whole cache lines.
  if constexpr (HAS_V) {
    constexpr int RS = ROWB + 8;
    constexpr int EP0 = (KSPLIT == 2) ? Cfg::kMerge : 0;
    static_assert(EP0 + NQW * 32 * RS <= Cfg::kRing, "output staging must fit the ring");
    unsigned char* ep = smem + EP0 + qsub * 32 * RS;
    const float inv = (l_tot > 0.f) ? 1.f / l_tot : 0.f;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        u32x2 w;
        w[0] = pack_bf16(oacc[db][4 * j + 0] * inv, oacc[db][4 * j + 1] * inv);
        w[1] = pack_bf16(oacc[db][4 * j + 2] * inv, oacc[db][4 * j + 3] * inv);
        *reinterpret_cast<u32x2*>(ep + ln * RS + (32 * db + 8 * j + 4 * g) * 2) = w;
      }
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
    constexpr int RPI = 64 / CPR;     // rows per store instruction
    const int er = lane / CPR, ec = lane % CPR;
    uint16_t* otile = p.o + head_off + (size_t)q0 * D;
#pragma unroll
    for (int i = 0; i < 32 / RPI; ++i) {
      const int row = i * RPI + er;
      const u32x2 lo = *reinterpret_cast<const u32x2*>(ep + row * RS + ec * 16);
      const u32x2 hi = *reinterpret_cast<const u32x2*>(ep + row * RS + ec * 16 + 8);
      const u32x4 w = {lo[0], lo[1], hi[0], hi[1]};
      if (q0 + row < p.S) *reinterpret_cast<u32x4*>(otile + (size_t)row * D + ec * 8) = w;
    }
  }
  if (g == 0) {
    if (p.lse != nullptr && qrow_ok) {
      p.lse[(size_t)bh * p.S + qrow] = (l_tot > 0.f) ? (mr_sf + __log2f(l_tot)) * kLn2 : kNegInf;
    }
    if constexpr (STATS) {
      // Pad rows keep the reference convention max_q = 0, denom = -inf
      // (include/maxq_denom.cuh:202-205).
      if (qrow < p.Sp) {
        const size_t so = (size_t)bh * p.Sp + qrow;
        // the denominator is reported against the true row max
        const bool any_key = qrow_ok && m_true != kNegInf;
        p.max_q[so] = any_key ? m_true : 0.f;
        p.denom[so] = qrow_ok ? (any_key ? l_tot * __builtin_amdgcn_exp2f(mr_sf - m_true * p.sf) : 0.f) : kNegInf;
      }
    }
  }
}

// Host launcher; returns hipError_t of the launch.
template <int D, int QBLK, int MODE, bool HAS_V, bool STATS>
inline hipError_t launch_attn_fwd(const AttnParams& p, hipStream_t stream) {
  using Cfg = AttnCfg<D, MODE, HAS_V>;
  auto kern = attn_fwd_kernel<D, QBLK, MODE, HAS_V, STATS>;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::kTotal);
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  const int total = p.nqblk * p.H * p.B;
  if (total <= 0) return hipSuccess;
  hipLaunchKernelGGL(kern, dim3(total), dim3(256), Cfg::kTotal, stream, p);
  return hipGetLastError();
}

}  // namespace spattn
