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
// Schedule.  One barrier per tile.  Between the barriers of tile i a wave multiplies the
// scores of tile i+1 while the softmax of tile i runs on the vector ALU, then P_i V_i while
// the row maxima of tile i+1 are reduced; the V^T operands are requested from LDS while
// the last score multiplies run, so the 16 (or 32) multiplies of a tile form one
// uninterrupted run.  The ring has three K slots and two V slots (5 x 16 KB at d = 128: two
// workgroups fill the 160 KB of a CU): the barrier of tile i frees the slots of K(i) and
// V(i-1), and V(i+1) and K(i+3) are copied into them, their issue spread between the
// multiplies.  The steady-state loop is unrolled over six tiles so that every slot is a
// compile-time constant: LDS addresses are a per-lane base plus an instruction immediate,
// the wait counts are literals, and the loop carries almost no scalar or address
// arithmetic - instruction issue and latency, not the matrix pipe, bound this kernel.
#pragma once
#include <type_traits>

#include "common.h"

namespace spattn {

typedef __attribute__((ext_vector_type(4))) short s16x4;

template <int D, int MODE, bool HAS_V>
struct AttnCfg {
  static constexpr int kTileBytes = 64 * D * 2;
  // Ring slots: K tiles are copied three tiles ahead, V tiles one ahead; 80 KB at d = 128,
  // which lets two workgroups share a CU.
  static constexpr int kKSlots = 3;
  static constexpr int kVSlots = HAS_V ? 2 : 0;
  static constexpr int kSlots = kKSlots + kVSlots;
  static constexpr int kRing = kSlots * kTileBytes;
  static constexpr int kMerge = 2 * (D / 2 + 3) * 64 * 4;     // key-split merge, overlays the ring
  static constexpr int kTotal = (kRing > kMerge) ? kRing : kMerge;
  static constexpr int kRowsPerLoad = 1024 / (D * 2);         // rows one wave-wide 1 KB load covers
  static constexpr int kLoadsPerTile = kTileBytes / 1024 / 4;   // per wave
};

// Waves per SIMD the register allocation aims at.  Two everywhere (256 registers), except for block lists at
// d = 64 with 128-row q-blocks: that instantiation fits 168 registers with a handful of spills outside the
// tile loop, its 40 KB ring lets three workgroups share a CU, and it is bound by the vector ALU, which a
// third wave keeps fed (measured side by side on one board: -7 %; the dense and token-list forms of the same
// shape need 40-50 spills for it and lose).
template <int D, int QBLK, int MODE>
constexpr int attn_waves_per_simd() {
  return (D == 64 && QBLK == 128 && MODE == KV_BLOCKS) ? 3 : 2;
}

template <int D, int QBLK, int MODE, bool HAS_V, bool STATS>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(attn_waves_per_simd<D, QBLK, MODE>())))
void attn_fwd_kernel(const AttnParams p) {
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
  constexpr int NK = Cfg::kKSlots;
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
  // a caller-given work order (longest lists first) replaces the XCD-contiguous default
  const int wg = p.order ? ((const __attribute__((address_space(4))) int*)p.order)[blockIdx.x]
                         : xcd_remap(blockIdx.x, total);
  // an entry of a work order that names no q-block: nothing is addressed (wave-uniform, ahead
  // of every copy and barrier)
  if ((unsigned)wg >= (unsigned)total) return;
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
  // The loads of a tile are 4 RPL rows apart, a multiple of the swizzle period: one chunk
  // offset serves all of them.
  static_assert((4 * RPL) % 16 == 0, "loads of one wave must share the swizzle");
  const int ld_row0 = RPL * wave + ld_sub;
  const int ld_off0 = (ld_slot ^ swz(ld_row0)) << 4;   // chunk offset within the row
  auto ld_row = [&](int i) -> int { return ld_row0 + 4 * RPL * i; };
  auto ld_off = [&](int) -> int { return ld_off0; };
  uint32_t ld_go[LPT];                 // lane offset within a contiguous 64-row tile
#pragma unroll
  for (int i = 0; i < LPT; ++i) {
    // a key sequence shorter than one tile: rows past its end re-read the last row
    const int row = ld_row(i) > last_row ? last_row : ld_row(i);
    ld_go[i] = row * ROWB + ld_off0;
  }

  // Dense / block lists: a tile is described by the first row that is copied and by how
  // many of its 64 keys exist, packed as  start | keys << 24  (wave-uniform, one SGPR).
  // A tile that runs past kv_len is copied as the LAST 64 rows of the sequence, so that no
  // lane needs a row clamp of its own: its keys then sit at the end of the tile and the
  // rows in front of them (keys of the previous block) are masked.  A sequence shorter than
  // one tile is copied from row 0 with the clamped lane offsets above.  A block id outside
  // the sequence describes a tile with no keys.
  // The id of tile t is t itself (dense) or the t-th list entry (block lists); positions
  // past the end of the list may be asked for (prefetch), their descriptors are never used.
  const bool kv_short = p.kv_len < 64;
  auto tile_desc = [&](int t) -> int {
    int id = t;
    if constexpr (MODE == KV_BLOCKS) id = lst[t < p.idx_stride ? t : p.idx_stride - 1];
    const bool valid = id >= 0 && id <= (last_row >> 6);
    const int r0 = valid ? id * 64 : 0;
    int keys = valid ? p.kv_len - r0 : 0;
    keys = keys > 64 ? 64 : keys;
    const int start = (keys < 64 && !kv_short) ? p.kv_len - 64 : r0;
    return start | (keys << 24);
  };

  // Token lists: lane l of every wave fetches entry 64t + l of the list, one tile further
  // ahead than the K copies (ids_load: a vector load written as asm, so that it is counted
  // by hand like the tile copies).  When the K copy of tile t is prepared, the entries that
  // name a key (position < n, id < kv_len) are balloted into the tile's 64-bit key mask,
  // the others are pointed at row 0, and each copy takes the row of its lane from the
  // lane that holds it (ds_bpermute).  idr / idw / idh hold ids and mask halves of tile j
  // at index j % 6.
  int idr[6] = {};   // used with token lists only
  uint64_t lst_addr = 0;
  if constexpr (MODE == KV_TOKENS) {
    const uint64_t a = (uint64_t)(uintptr_t)(p.idx + ((size_t)bh * p.nqblk + qb) * p.idx_stride);
    // readfirstlane returns a signed int: without the casts the low word would be sign-extended
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)a);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
    lst_addr = ((uint64_t)hi << 32) | lo;
  }
  auto ids_load = [&](int t, int& dst) {
    if constexpr (MODE == KV_TOKENS) {
      int pos = t * 64 + lane;
      pos = pos < p.idx_stride ? pos : p.idx_stride - 1;
      asm volatile("global_load_dword %0, %1, %2" : "=v"(dst) : "v"(pos * 4), "s"(lst_addr) : "memory");
    }
  };
  auto ids_resolve = [&](int t, int& ids, int& mlo, int& mhi) {
    if constexpr (MODE == KV_TOKENS) {
      const bool ok = (t * 64 + lane) < n && (unsigned)ids <= (unsigned)last_row;
      const unsigned long long m = __ballot(ok);
      mlo = (int)(unsigned)m;
      mhi = (int)(unsigned)(m >> 32);
      ids = ok ? ids : 0;
    }
  };

  // Loads of one K or V tile into ring slot `slot`: prepare() resolves the wave-uniform
  // base and this lane's byte offsets, load(i) issues the i-th of the LPT wave-wide copies.
  struct TileLoad {
    const unsigned char* base;
    uint32_t lds;
    uint32_t go[LPT];
  };
  // desc: tile descriptor (dense / block lists) or the resolved ids of the tile (token lists).
  // Token lists with a 64-row q-block (registers to spare): the byte offsets found for the K
  // copy of tile j are kept in gor[j % 3] and serve its V copy two tiles later.
  constexpr bool GO_RING = (MODE == KV_TOKENS) && HAS_V && QBLK == 64;
  uint32_t gor[GO_RING ? 3 : 1][GO_RING ? LPT : 1];
  auto prepare_tile = [&](int desc, int slot, bool is_v, auto gic) -> TileLoad {
    constexpr int GI = decltype(gic)::value;
    TileLoad tl;
    tl.lds = smem_base + (uint32_t)slot * TILE + wave * 1024;
    const unsigned char* src = is_v ? vh : kh;
    if constexpr (MODE == KV_TOKENS) {
      tl.base = src;
#pragma unroll
      for (int i = 0; i < LPT; ++i) {
        if (GO_RING && is_v) {
          tl.go[i] = gor[GO_RING ? GI : 0][GO_RING ? i : 0];
        } else {
          const int row = __builtin_amdgcn_ds_bpermute(ld_row(i) * 4, desc);
          tl.go[i] = (uint32_t)row * ROWB + ld_off(i);
          if constexpr (GO_RING) gor[GI][i] = tl.go[i];
        }
      }
    } else {
      tl.base = src + (size_t)(desc & 0xffffff) * ROWB;
#pragma unroll
      for (int i = 0; i < LPT; ++i) tl.go[i] = ld_go[i];
    }
    return tl;
  };
  auto load_part = [&](const TileLoad& tl, int i) { dma16(tl.base, tl.go[i], tl.lds + i * 4096); };
  auto issue_tile = [&](int desc, int slot, bool is_v, auto gic) {
    const TileLoad tl = prepare_tile(desc, slot, is_v, gic);
#pragma unroll
    for (int i = 0; i < LPT; ++i) load_part(tl, i);
  };

  // ---- prologue ------------------------------------------------------------------
  const int q0 = qb * QBLK + qsub * 32;
  const int qrow = q0 + ln;
  const bool qrow_ok = qrow < p.S;

  auto kslot = [](int t) -> int { return t % NK; };
  auto vslot = [](int t) -> int { return NK + (t & 1); };

  // Copies go out in the order K0 K1 V0 K2 | V1 K3 | V2 K4 | ...
  int idw[6] = {0, 0, 0, 0, 0, 0};   // descriptors (key mask, low half) of the tiles in flight, tile j in idw[j % 6]
  int idh[6] = {0, 0, 0, 0, 0, 0};   // token lists: key mask, high half
  if constexpr (MODE == KV_TOKENS) {
#pragma unroll
    for (int j = 0; j < 4; ++j) ids_load(j, idr[j]);
    wait_vmcnt<0>();
#pragma unroll
    for (int j = 0; j < 4; ++j) asm volatile("" : "+v"(idr[j]));
#pragma unroll
    for (int j = 0; j < 3; ++j) ids_resolve(j, idr[j], idw[j], idh[j]);
  }
  // What prepare_tile takes for tile j (a prologue tile: j < 3).  Block lists: the first three
  // entries are fetched before anything depends on the count (list positions are clamped, an
  // entry past the count is simply not used), so that the count and the entries travel
  // together instead of one scalar-load latency after the other.
  int hd[3] = {0, 0, 0};
  if constexpr (MODE != KV_TOKENS) {
#pragma unroll
    for (int j = 0; j < 3; ++j) hd[j] = tile_desc(j);
  }
  auto head_desc = [&](int j) -> int {
    if constexpr (MODE == KV_TOKENS) return idr[j];
    else return hd[j];
  };
  using G0 = std::integral_constant<int, 0>;
  using G1 = std::integral_constant<int, 1>;
  using G2 = std::integral_constant<int, 2>;
  // The Q loads go out first - their address does not wait for the list - and are counted by
  // hand like the copies (a load the compiler sees makes it wait for every copy issued before
  // the first use of Q): the wait for K0, issued behind them, covers them.  Rows past the end of
  // the sequence read the last row and are zeroed.
  u32x4 qf[NT];
  {
    const uint16_t* qsrc = qh + (size_t)(qrow_ok ? qrow : p.S - 1) * D + 8 * g;
    load_q_uncounted<0, NT>(qf, qsrc);
  }
  if (ntiles > 0) issue_tile(head_desc(0), kslot(0), false, G0{});
  int head_pending = 0;   // tile copies behind K0 when the first phase waits
  if (ntiles > 0) {
    if (1 < ntiles) { issue_tile(head_desc(1), kslot(1), false, G1{}); ++head_pending; }
    if constexpr (HAS_V) { issue_tile(head_desc(0), vslot(0), true, G0{}); ++head_pending; }
    if (NK == 3 && 2 < ntiles) { issue_tile(head_desc(2), kslot(2), false, G2{}); ++head_pending; }
  }

  // Softmax state of this lane's query row.  Exponents are taken against a reference
  // mr_sf (in log2 units, = raw max * sf at the time it was set) that is only moved when
  // some row of the wave outgrows it by more than kSlack: p = exp2(s*sf - mr_sf) may then
  // exceed 1 (by at most 2^kSlack), which fp32 sums and bf16 P hold without loss, and the
  // O / l rescale is skipped on most tiles.  m_true tracks the true raw max for the
  // statistics outputs.
  // Without statistics outputs the row maxima are not even computed per tile (LAZY_MAX):
  // a row that outgrew the reference shows in the tile's own sum of p (above 2^kSlack, inf
  // or NaN), and only then are the maxima taken, the reference moved and the tile's
  // exponentials redone.
  constexpr float kSlack = 8.f;
  constexpr float kTrigger = 256.f;   // 2^kSlack
  constexpr bool LAZY_MAX = !STATS;
  float mr_sf = kNegInf;
  // What the exponentials subtract: mr_sf once a key has been seen.  Before that, 0 where the
  // row maxima are taken on every tile (every key so far was masked, p = exp2(-inf) = 0), but
  // -inf with LAZY_MAX: a tile with a key then gives p = inf (NaN for its masked keys), the
  // tile's sum trips the check below and the row gets its reference from that tile's true
  // maximum, instead of keys being accumulated against a reference that was never recorded.
  constexpr float kNoRef = LAZY_MAX ? kNegInf : 0.f;
  float base_eff = kNoRef;
  float m_true = kNegInf;
  float l_run = 0.f;       // running denominator, this lane's keys only
  float l_tile = 0.f;      // sum of p over the tile whose softmax is in progress
  f32x16 oacc[HAS_V ? NDB : 1];
#pragma unroll
  for (int db = 0; db < (HAS_V ? NDB : 1); ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;

  // SPLIT_SM: the exponentials of a tile are taken in two halves, score registers 0-7 of every
  // block under the P V multiplies of the tile before, registers 8-15 under the QK^T multiplies
  // of the tile after, so that every multiply has the same vector-ALU work next to it (all of
  // it under QK^T leaves the vector ALU the bottleneck there and idle under P V).  Needs the
  // reference fixed before the tile's scores exist, which LAZY_MAX gives.
  constexpr bool SPLIT_SM = LAZY_MAX && HAS_V;
  u32x4 pb[SPLIT_SM ? 2 : 1][HAS_V ? 2 * NMB : 1];   // P^T operands, k-step 2mb + h; SPLIT_SM: by tile parity

  // Per-lane LDS addresses inside slot 0; slot, score block and k-step offsets are added
  // as constants (instruction immediates in the unrolled loop).
  // A operand of QK^T, k-step t, score block 0.  K_XOR (d=128 with 128-row q-blocks, where the
  // registers do not reach and two Q operands were reloaded from scratch on every tile, each
  // reload waiting for every tile copy in flight): only the address of k-step 0 is kept, that
  // of k-step t is the same with t XORed into chunk bits 1-3.
  constexpr bool K_XOR = (D == 128 && QBLK == 128);
  lds_cptr k_lo[K_XOR ? 1 : NT];
  {
    const int krow = ksub * KW + ln;
#pragma unroll
    for (int t = 0; t < (K_XOR ? 1 : NT); ++t) k_lo[t] = smem_l + krow * ROWB + (((2 * t + g) ^ swz(krow)) << 4);
  }
  // Transposing V read: in each 16-lane group, lane i addresses 4 dims of key (i>>2);
  // lane j receives dim j of those 4 keys.  Keys 4g..4g+3 (+8 for the second read) of
  // each 16-key step, dims 32db + 16*dhalf + 4*(i&3)..+3.
  // All V addresses of a lane derive from one: the 32-dim block db sits in chunk bits 2-3,
  // which the swizzle only XORs (address ^ (db << 6)), and rows r and r+8 differ in one
  // swizzle bit (address ^ 32, + 8 rows).  They are re-derived per tile instead of being
  // kept in eight registers.
  uint32_t v_base = 0, v_cur = 0;
  if constexpr (HAS_V) {
    const int i16 = lane & 15;
    const int dhalf = (lane >> 4) & 1;
    const int r1 = ksub * KW + 4 * g + (i16 >> 2);
    const int cb = 2 * dhalf + ((i16 & 3) >> 1);
    static_assert(NDB <= 4, "db must fit chunk bits 2-3");
    // relative to the first V slot: instruction offsets reach 64 KB, the ring is larger
    v_base = smem_base + NK * TILE + r1 * ROWB + ((cb ^ swz(r1)) << 4) + ((i16 & 1) << 3);
  }
  // Called once per tile: hides v_base from loop-invariant code motion.
  // With a 64-row q-block there are registers to spare and the compiler may keep all of them.
  uint32_t k_cur = 0;
  auto v_addr_refresh = [&]() {
    v_cur = v_base;
    if constexpr (QBLK != 64) asm volatile("" : "+v"(v_cur));
    if constexpr (K_XOR) {
      k_cur = (uint32_t)(uintptr_t)k_lo[0];
      asm volatile("" : "+v"(k_cur));
    }
  };

  // ---- building blocks --------------------------------------------------------------
  // Keys of tile `it` that do not exist get -inf.  Accumulator register 4j+i of block mb
  // is key ksub*KW + 32mb + 8j + 4g + i of the tile.
  auto mask_tile = [&](int desc, int desc_hi, f32x16 (&s)[NMB]) {
    if constexpr (MODE == KV_TOKENS) {
      if ((desc & desc_hi) != -1) {   // wave-uniform: some key of the tile does not exist
        const unsigned long long m = ((unsigned long long)(unsigned)desc_hi << 32) | (unsigned)desc;
        const unsigned long long mine = m >> (ksub * KW + 4 * g);   // bit c: this lane's key c
#pragma unroll
        for (int mb = 0; mb < NMB; ++mb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int c = 32 * mb + 8 * (r >> 2) + (r & 3);
            if (!((mine >> c) & 1)) s[mb][r] = kNegInf;
          }
      }
    } else {
      const int keys = desc >> 24;
      if (keys < 64) {
        // existing keys are tile rows lo .. hi-1 (wave-uniform)
        const int lo = kv_short ? 0 : 64 - keys;
        const int hi = kv_short ? keys : 64;
        const int kb = ksub * KW + 4 * g;    // this lane's first key
#pragma unroll
        for (int mb = 0; mb < NMB; ++mb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int c = 32 * mb + 8 * (r >> 2) + (r & 3);
            if (kb < lo - c || kb >= hi - c) s[mb][r] = kNegInf;
          }
      }
    }
  };
  // Row max of a score tile in NP pieces (so that they can be placed between multiplies),
  // then the exchange between the two 32-lane halves; returns max * sf.
  constexpr int NP = 4 * NMB;
  auto stat_piece = [&](const f32x16 (&s)[NMB], int k, float& mloc) {
    const int mb = k >> 2, r = 4 * (k & 3);
    if (k == 0) mloc = s[0][0];
    mloc = max3_raw(mloc, s[mb][r], s[mb][r + 1]);
    mloc = max3_raw(mloc, s[mb][r + 2], s[mb][r + 3]);
  };
  // tile: the key block the maxima belong to.  With the statistics outputs a caller may also ask
  // for them per key block (blockmax[J][row], raw like max_q): the threshold test of the mask
  // pre-pass, softmax(r, c) > tau, holds for some key of block J exactly when the block's maximum
  // passes it, so these S x S/64 numbers replace the second score sweep for block-level masks.
  auto stat_finish = [&](float mloc, int tile) -> float {
    mloc = pair_max(mloc);
    if constexpr (STATS && KSPLIT == 1 && MODE == KV_DENSE) {
      if (p.blockmax != nullptr && g == 0) p.blockmax[((size_t)bh * (p.Sp >> 6) + tile) * p.Sp + qrow] = bf16_round_up(mloc);
    }
    m_true = max_raw(m_true, mloc);
    return mloc * p.sf;
  };
  auto row_stats = [&](const f32x16 (&s)[NMB], int tile) -> float {
    float mloc;
#pragma unroll
    for (int k = 0; k < NP; ++k) stat_piece(s, k, mloc);
    return stat_finish(mloc, tile);
  };
  // Move the exponent reference if some row of the wave outgrew it; rescales O and l.
  auto maybe_rescale = [&](float mloc_sf) {
    if (__any(mloc_sf > mr_sf + kSlack)) {
      const float new_sf = max_raw(mr_sf, mloc_sf);
      const float alpha = (new_sf == kNegInf) ? 1.f : __builtin_amdgcn_exp2f(mr_sf - new_sf);
      mr_sf = new_sf;
      base_eff = (new_sf == kNegInf) ? kNoRef : new_sf;
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
  auto softmax_chunk = [&](const f32x16 (&s)[NMB], float base, int mb, int r0, int cnt, int par) {
#pragma unroll
    for (int r = r0; r < r0 + cnt; r += 2) {
      const float e0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[mb][r], p.sf, -base));
      const float e1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[mb][r + 1], p.sf, -base));
      l_tile = (mb == 0 && r == 0) ? e0 : l_tile + e0;
      l_tile += e1;
      if constexpr (HAS_V) pb[SPLIT_SM ? par : 0][2 * mb + (r >> 3)][(r & 7) >> 1] = pack_bf16(e0, e1);
    }
  };
  // Pin the softmax results where they are produced; otherwise the compiler sinks the
  // whole softmax to the first use of P and nothing overlaps the MFMAs.
  // half: 0 = the operands of registers 0-7, 1 = of registers 8-15, 2 = both
  auto pin_softmax = [&](int par, int half) {
    asm volatile("" : "+v"(l_tile));
    if constexpr (HAS_V) {
#pragma unroll
      for (int ks = 0; ks < 2 * NMB; ++ks)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (half == 2 || (ks & 1) == half) asm volatile("" : "+v"(pb[SPLIT_SM ? par : 0][ks][i]));
    }
  };
  auto softmax_only = [&](const f32x16 (&s)[NMB], int par, float base) {
#pragma unroll
    for (int mb = 0; mb < NMB; ++mb) softmax_chunk(s, base, mb, 0, 16, par);
  };
  auto softmax_half = [&](const f32x16 (&s)[NMB], int par, int half) {
#pragma unroll
    for (int mb = 0; mb < NMB; ++mb) softmax_chunk(s, base_eff, mb, 8 * half, 8, par);
  };
  // Closes the softmax of a tile: adds its sum to the denominator.  LAZY_MAX: first redoes
  // the tile against a new reference if some row of the wave outgrew the old one.
  auto softmax_close = [&](const f32x16 (&s)[NMB], int par) {
    if constexpr (LAZY_MAX) {
      if (__any(!(l_tile <= kTrigger))) {
        maybe_rescale(row_stats(s, 0));
        // a row that still has no reference has seen masked keys only: p = exp2(-inf - 0) = 0
        softmax_only(s, par, mr_sf == kNegInf ? 0.f : mr_sf);
      }
    }
    l_run += l_tile;
  };

  // V^T operands of one 16-key step (PV group gi = 2mb + h), double-buffered over groups; where
  // the registers do not reach (K_XOR) one buffer, the operand of block db refilled for the
  // next group as soon as its multiply of this group has been issued.
  constexpr int NG = 2 * NMB;
  constexpr int VB = K_XOR ? 1 : 2;
  u32x2 va[HAS_V ? VB : 1][HAS_V ? NDB : 1][2];
  auto v_read_db = [&](uint32_t vofs, int gi, int db) {
    if constexpr (HAS_V) {
      const uint32_t x1 = v_cur ^ (uint32_t)(db << 6);
      const uint32_t x2 = x1 ^ 32u;
      const lds_cptr a1 = (lds_cptr)(uintptr_t)x1 + vofs + gi * 16 * ROWB;
      const lds_cptr a2 = (lds_cptr)(uintptr_t)x2 + vofs + gi * 16 * ROWB + 8 * ROWB;
      va[gi % VB][db][0] = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((SPATTN_LDS s16x4*)a1));
      va[gi % VB][db][1] = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((SPATTN_LDS s16x4*)a2));
    }
  };
  auto v_reads = [&](uint32_t vofs, int gi) {
#pragma unroll
    for (int db = 0; db < (HAS_V ? NDB : 0); ++db) v_read_db(vofs, gi, db);
  };

  // s_out^T = K Q^T from the K tile at ring offset kofs (bytes), one 32-key block at a
  // time.  WITH_SM: the softmax of s_in is interleaved, one MFMA then the vector-ALU work of
  // 16/NT score registers.  tl: a tile copy whose parts are issued between the multiplies
  // if `live` (in one burst they queue behind the other waves' copies and stall this wave).
  // EARLY_V: the V^T operands of the first PV group are requested before the last multiply,
  // so that PV does not start by waiting for LDS.
  constexpr int kEarly = 1;
  auto qk_tile = [&](auto with_sm, auto early_v, uint32_t kofs, uint32_t vofs, f32x16 (&s_out)[NMB], f32x16 (&s_in)[NMB],
                     int par_in, const TileLoad* tl, bool live) {
    constexpr bool WITH_SM = decltype(with_sm)::value;
    constexpr bool EARLY_V = decltype(early_v)::value;
    constexpr int EPM = 16 / NT;
    constexpr int MPP = NT / 4;   // SPLIT_SM: multiplies per pair of score registers 8-15
    const float base = base_eff;
#pragma unroll
    for (int mb = 0; mb < NMB; ++mb) {
      u32x4 ka[NT];
      auto k_reads = [&](int t0, int t1) {
#pragma unroll
        for (int t = t0; t < t1; ++t) {
          if constexpr (K_XOR) {
            const uint32_t a0 = k_cur ^ (uint32_t)(t << 5);
            ka[t] = *(SPATTN_LDS const u32x4*)((lds_cptr)(uintptr_t)a0 + kofs + mb * 32 * ROWB);
          } else {
            ka[t] = *(SPATTN_LDS const u32x4*)(k_lo[t] + kofs + mb * 32 * ROWB);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      };
      // the operands arrive in two batches, to bound the registers they hold
      k_reads(0, NT / 2);
      const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      auto steps = [&](int t0, int t1) {
#pragma unroll
        for (int t = t0; t < t1; ++t) {
          s_out[mb] = mfma32(ka[t], qf[t], t == 0 ? zero : s_out[mb]);
          if constexpr (WITH_SM && SPLIT_SM) {
            if (t % MPP == 0) softmax_chunk(s_in, base, mb, 8 + 2 * (t / MPP), 2, par_in);
          } else if constexpr (WITH_SM) {
            softmax_chunk(s_in, base, mb, t * EPM, EPM, par_in);
          }
          if (tl != nullptr && live) {
            constexpr int STEP = (NMB * NT) / LPT;
            const int m = mb * NT + t;
            if (m % STEP == STEP - 1) load_part(*tl, m / STEP);
          }
        }
        if constexpr (WITH_SM) {
#pragma unroll
          for (int t = t0; t < t1; ++t) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);            // one MFMA
            // its share of the softmax: seven instructions per pair of score registers
            if constexpr (!SPLIT_SM) __builtin_amdgcn_sched_group_barrier(0x002, EPM * 7 / 2, 0);
            else if constexpr (MPP == 1) __builtin_amdgcn_sched_group_barrier(0x002, 7, 0);
            else if (t % 2 == 0) __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
            else __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      };
      steps(0, NT / 4);
      k_reads(NT / 2, NT);
      if (EARLY_V && mb == NMB - 1) {
        steps(NT / 4, NT - kEarly);
        v_reads(vofs, 0);
        __builtin_amdgcn_sched_barrier(0);
        steps(NT - kEarly, NT);
      } else {
        steps(NT / 4, NT);
      }
    }
    if constexpr (WITH_SM) pin_softmax(par_in, SPLIT_SM ? 1 : 2);
  };
  // O^T += V^T P^T from the V tile at offset vofs from the first V slot, one 16-key step (NDB multiplies) at
  // a time; the operands of step 0 are in flight or here already (FIRST_LOADED), those of
  // step gi+1 are requested before step gi is multiplied.  STAT: the row maxima of s_next
  // are reduced between the multiplies; returns them (times sf).
  // EARLY_SM: the exponentials of registers 0-7 of s_next (the tile after, parity par ^ 1) are
  // taken between the multiplies.
  auto pv_tile = [&](auto first_loaded, auto stat_c, uint32_t vofs, const TileLoad* tl, bool live, const f32x16 (&s_next)[NMB],
                     int par, auto early_sm, int tile_next = 0) -> float {
    constexpr bool STAT = decltype(stat_c)::value;
    constexpr bool EARLY_SM = decltype(early_sm)::value;
    constexpr int MPP = NDB / 2;   // EARLY_SM: multiplies per pair of score registers
    const float base = base_eff;
    float mloc = 0.f;
    if constexpr (HAS_V) {
      if constexpr (!decltype(first_loaded)::value) v_reads(vofs, 0);
#pragma unroll
      for (int gi = 0; gi < NG; ++gi) {
        if (VB == 2 && gi + 1 < NG) v_reads(vofs, gi + 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int db = 0; db < NDB; ++db) {
          const u32x4 a = {va[gi % VB][db][0][0], va[gi % VB][db][0][1], va[gi % VB][db][1][0], va[gi % VB][db][1][1]};
          oacc[db] = mfma32(a, pb[SPLIT_SM ? par : 0][gi], oacc[db]);
          if (VB == 1 && gi + 1 < NG) v_read_db(vofs, gi + 1, db);
          const int m = gi * NDB + db;
          if constexpr (EARLY_SM) {
            if (m % MPP == 0) softmax_chunk(s_next, base, (m / MPP) / 4, 2 * ((m / MPP) % 4), 2, par ^ 1);
          }
          if constexpr (STAT) {
            constexpr int PPM = (NP + NG * NDB - 1) / (NG * NDB);   // pieces per multiply
#pragma unroll
            for (int k = m * PPM; k < (m + 1) * PPM && k < NP; ++k) stat_piece(s_next, k, mloc);
          }
          if (tl != nullptr && live) {   // a tile copy, spread over the multiplies
            constexpr int STEP = (NG * NDB) / LPT;
            if (m % STEP == STEP - 1) load_part(*tl, m / STEP);
          }
        }
        if constexpr (EARLY_SM) {
#pragma unroll
          for (int db = 0; db < NDB; ++db) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if constexpr (MPP == 1) __builtin_amdgcn_sched_group_barrier(0x002, 7, 0);
            else if (db % 2 == 0) __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
            else __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (EARLY_SM) pin_softmax(par ^ 1, 0);
    } else if constexpr (STAT) {
#pragma unroll
      for (int k = 0; k < NP; ++k) stat_piece(s_next, k, mloc);
    }
    if constexpr (STAT) return stat_finish(mloc, tile_next);
    return 0.f;
  };

  f32x16 s_e[NMB], s_o[NMB];   // scores of even / odd tiles

  // One tile of the pipeline, between two barriers: the scores of tile it+1 are multiplied
  // (K slot (it+1) % NK) while the softmax of tile it runs on the vector ALU, then P V of
  // tile it (V slot NK + it % 2) is multiplied while the row maxima of tile it+1 are
  // reduced.  The barrier frees the slots of K(it) and V(it-1): V(it+1) and, if it exists,
  // K(it+NK) are copied into them.  KC = it % 6 fixes every slot at compile time.
  auto tile_body = [&](auto kc, int it) {
    constexpr int KC = decltype(kc)::value;
    // KS, KN: ring slots of K(it+1), K(it+NK); VS: V slot of tile it counted from the first
    // V slot; VN: ring slot of V(it+1)
    constexpr int KS = (KC + 1) % NK, VS = KC % 2, KN = KC % NK, VN = NK + (KC + 1) % 2;
    auto& s_a = (KC & 1) ? s_o : s_e;   // tile it
    auto& s_b = (KC & 1) ? s_e : s_o;   // tile it+1
    const bool has_kn = it + NK < ntiles;
    // behind K(it+1) and V(it) only K(it+2) can be in flight (three K slots)
    if (NK == 3 && it + 2 < ntiles) wait_vmcnt<LPT>(); else wait_vmcnt<0>();
    if constexpr (MODE == KV_TOKENS) {
      // the ids of tile it+NK, requested one tile ago, are behind the wait above
      asm volatile("" : "+v"(idr[(KC + NK) % 6]));
      ids_resolve(it + NK, idr[(KC + NK) % 6], idw[(KC + NK) % 6], idh[(KC + NK) % 6]);
    }
    __syncthreads();
    v_addr_refresh();
    // what the copies of V(it+1) and K(it+NK) are prepared from, and the key mask of tile it+1
    const int d_v = (MODE == KV_TOKENS) ? idr[(KC + 1) % 6] : idw[(KC + 1) % 6];
    const int d_k = (MODE == KV_TOKENS) ? idr[(KC + NK) % 6] : idw[(KC + NK) % 6];
    const int m_lo = idw[(KC + 1) % 6], m_hi = idh[(KC + 1) % 6];
    constexpr bool K_FIRST = !HAS_V;
    using GK = std::integral_constant<int, (KC + NK) % 3>;    // tile it+NK
    using GV = std::integral_constant<int, (KC + 1) % 3>;     // tile it+1
    const TileLoad tl_first = K_FIRST ? prepare_tile(d_k, KN, false, GK{}) : prepare_tile(d_v, VN, true, GV{});
#ifdef SPATTN_POISON_RING
    // Debug build of the copy pipeline: the two ring slots this barrier has freed are filled with
    // bf16 NaNs before the copies of V(it+1) and K(it+NK) are issued into them (each wave the
    // parts it copies itself, the stores complete before the copies go out).  A wave that still
    // reads the old tile from a freed slot - a missing wait, a barrier too few, a wrong slot
    // number - then sees NaNs instead of stale but plausible keys, and the output shows it.
    {
      const u32x4 nan4 = {0x7fc07fc0u, 0x7fc07fc0u, 0x7fc07fc0u, 0x7fc07fc0u};
      auto poison = [&](int slot) {
        unsigned char* base = smem + slot * TILE + wave * 1024 + lane * 16;
#pragma unroll
        for (int i = 0; i < LPT; ++i) *reinterpret_cast<u32x4*>(base + i * 4096) = nan4;
      };
      if constexpr (HAS_V) poison(VN);
      if (has_kn) poison(KN);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
#endif
    constexpr int PAR = KC & 1;
    qk_tile(std::true_type{}, std::integral_constant<bool, HAS_V>{}, KS * TILE, VS * TILE, s_b, s_a, PAR, &tl_first,
            K_FIRST ? has_kn : true);
    // ids of tile it+NK+1: between the copies of V(it+1) and K(it+NK) in the order of issue.
    // Issued whether or not that tile exists (the position is clamped to the list): the wait
    // counts stay the same on every tile, and the registers are held until the final wait.
    if constexpr (MODE == KV_TOKENS) ids_load(it + NK + 1, idr[(KC + NK + 1) % 6]);
    softmax_close(s_a, PAR);
    mask_tile(m_lo, m_hi, s_b);
    if constexpr (MODE != KV_TOKENS) idw[(KC + NK + 1) % 6] = tile_desc(it + NK + 1);
    float mloc_sf;
    using stat_t = std::integral_constant<bool, !LAZY_MAX>;
    if constexpr (HAS_V) {
      const TileLoad tl_second = K_FIRST ? prepare_tile(d_v, VN, true, GV{}) : prepare_tile(d_k, KN, false, GK{});
      mloc_sf = pv_tile(std::true_type{}, stat_t{}, VS * TILE, &tl_second, K_FIRST ? true : has_kn, s_b, PAR,
                        std::integral_constant<bool, SPLIT_SM>{}, it + 1);
    } else {
      mloc_sf = pv_tile(std::true_type{}, stat_t{}, 0, nullptr, false, s_b, PAR, std::false_type{}, it + 1);
    }
    if constexpr (!LAZY_MAX) maybe_rescale(mloc_sf);
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;
  using I4 = std::integral_constant<int, 4>;
  using I5 = std::integral_constant<int, 5>;

  if (ntiles > 0) {
    // head: scores of tile 0
    if (head_pending == 3) wait_vmcnt<3 * LPT>();
    else if (head_pending == 2) wait_vmcnt<2 * LPT>();
    else if (head_pending == 1) wait_vmcnt<LPT>();
    else wait_vmcnt<0>();
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      asm volatile("" : "+v"(qf[t]));
      if (!qrow_ok) qf[t] = u32x4{0, 0, 0, 0};
    }
    __syncthreads();
    v_addr_refresh();
    qk_tile(std::false_type{}, std::false_type{}, 0, 0, s_e, s_e, 0, nullptr, false);
    if constexpr (MODE == KV_TOKENS) mask_tile(idw[0], idh[0], s_e);
    else mask_tile(hd[0], 0, s_e);
    maybe_rescale(row_stats(s_e, 0));
    if constexpr (SPLIT_SM) softmax_half(s_e, 0, 0);   // nothing to hide these under

    int it = 0;
    if constexpr (MODE != KV_TOKENS) {
#pragma unroll
      for (int j = 1; j <= NK; ++j) idw[j] = j < 3 ? hd[j] : tile_desc(j);
    }
    // Rounds of six tiles without side exits (the register allocator handles one plain
    // back-edge far better than six exits), then up to five single tiles.
    while (it + 6 < ntiles) {
      tile_body(I0{}, it);
      tile_body(I1{}, it + 1);
      tile_body(I2{}, it + 2);
      tile_body(I3{}, it + 3);
      tile_body(I4{}, it + 4);
      tile_body(I5{}, it + 5);
      it += 6;
    }
    if (it + 1 < ntiles) {
      tile_body(I0{}, it++);
      if (it + 1 < ntiles) {
        tile_body(I1{}, it++);
        if (it + 1 < ntiles) {
          tile_body(I2{}, it++);
          if (it + 1 < ntiles) {
            tile_body(I3{}, it++);
            if (it + 1 < ntiles) tile_body(I4{}, it++);
          }
        }
      }
    }
    // tail: softmax and P V of the last tile
    if (it & 1) {
      if constexpr (SPLIT_SM) softmax_half(s_o, 1, 1); else softmax_only(s_o, 1, base_eff);
      softmax_close(s_o, 1);
      if constexpr (SPLIT_SM) {
#pragma unroll
        for (int ks = 0; ks < 2 * NMB; ++ks) pb[0][ks] = pb[1][ks];
      }
    } else {
      if constexpr (SPLIT_SM) softmax_half(s_e, 0, 1); else softmax_only(s_e, 0, base_eff);
      softmax_close(s_e, 0);
    }
    wait_vmcnt<0>();
    if constexpr (MODE == KV_TOKENS) {
      // the id registers stay allocated until every id load has landed
#pragma unroll
      for (int j = 0; j < 6; ++j) asm volatile("" ::"v"(idr[j]));
    }
    if constexpr (HAS_V) {
      __syncthreads();
      v_addr_refresh();
      pv_tile(std::false_type{}, std::false_type{}, (uint32_t)(it & 1) * TILE, nullptr, false, s_e, 0, std::false_type{});
    }
  } else {
    // the Q loads still own their registers
    wait_vmcnt<0>();
#pragma unroll
    for (int t = 0; t < NT; ++t) asm volatile("" ::"v"(qf[t]));
  }
  __syncthreads();   // every wave is done with the ring

  // ---- combine the two 32-lane halves, then the two key halves -------------------
  float l_tot = pair_sum(l_run);
  if constexpr (KSPLIT == 2) {
    // per row half: three rows of 64 floats (reference, sum, true max), then the accumulators
    // four registers at a time, 16 bytes per lane
    float* mg = reinterpret_cast<float*>(smem) + qsub * ((HAS_V ? D / 2 : 0) + 3) * 64;
    typedef __attribute__((ext_vector_type(4))) float f32x4;
    f32x4* mg4 = reinterpret_cast<f32x4*>(mg + 3 * 64);
    if (ksub == 1) {
      mg[lane] = mr_sf;
      mg[64 + lane] = l_tot;
      mg[128 + lane] = m_true;
      if constexpr (HAS_V) {
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const f32x4 x = {oacc[db][4 * j], oacc[db][4 * j + 1], oacc[db][4 * j + 2], oacc[db][4 * j + 3]};
            mg4[(db * 4 + j) * 64 + lane] = x;
          }
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
        for (int j = 0; j < 4; ++j) {
          const f32x4 x = mg4[(db * 4 + j) * 64 + lane];
#pragma unroll
          for (int i = 0; i < 4; ++i) oacc[db][4 * j + i] = oacc[db][4 * j + i] * a1 + x[i] * a2;
        }
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

// Raises the dynamic-LDS limit of one instantiation on the current device (once per device; the
// launcher does it on the first launch, a caller that is about to record launches into a graph
// does it beforehand through spattn_init).
template <int D, int QBLK, int MODE, bool HAS_V, bool STATS>
inline hipError_t prepare_attn_fwd() {
  using Cfg = AttnCfg<D, MODE, HAS_V>;
  static bool attr_set[kMaxDevices] = {};
  return raise_lds_limit(reinterpret_cast<const void*>(attn_fwd_kernel<D, QBLK, MODE, HAS_V, STATS>), Cfg::kTotal, attr_set);
}

// Host launcher; returns hipError_t of the launch.
template <int D, int QBLK, int MODE, bool HAS_V, bool STATS>
inline hipError_t launch_attn_fwd(const AttnParams& p, hipStream_t stream) {
  using Cfg = AttnCfg<D, MODE, HAS_V>;
  auto kern = attn_fwd_kernel<D, QBLK, MODE, HAS_V, STATS>;
  const hipError_t ea = prepare_attn_fwd<D, QBLK, MODE, HAS_V, STATS>();
  if (ea != hipSuccess) return ea;
  const int total = p.nqblk * p.H * p.B;
  if (total <= 0) return hipSuccess;
  hipLaunchKernelGGL(kern, dim3(total), dim3(256), Cfg::kTotal, stream, p);
  return hipGetLastError();
}

}  // namespace spattn
