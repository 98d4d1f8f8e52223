// Forward attention with a whole head's K and V resident in LDS (head dim 64, up to 512 keys).
//
// Same arithmetic as the pipelined forward (fmha_fwd_pipe.h: transposed products, the extra
// contraction step that applies the per-key mask and the softmax reference, the lazily raised
// reference, row sums over the rounded probabilities) -- what differs is who shares what:
//
//   * one workgroup of EIGHT waves owns a whole (head, 512 queries) item; a wave owns 64 queries
//     (two 32-query blocks, so every LDS operand feeds two matrix instructions);
//   * all of the head's K and V rows (up to 512 keys x 64: 64 KB each) sit in LDS at once, copied
//     there directly from global memory exactly once per head, so the steady-state loop contains
//     no copy, no wait for a copy and no barrier: the waves run free and fall out of phase by
//     themselves;
//   * a wave's item is sixteen 32-key tiles long instead of eight 64-key tiles, of which the same
//     two (the first product and the last second product) run outside the interleaved stream, and
//     the first tile's softmax is interleaved with the second tile's first product.
//
// Workgroups are persistent (one per compute unit: 144 KB of LDS).  While an item is being computed,
// the next item's K and V rows are copied, a few tiles at a time, into the LDS that tiles which every
// wave has left behind have freed.  Five points of an item therefore carry a wait and a barrier
// ("hooks"): its start and the tops of its iterations 3, 7, 11 and 15.
//
// Tile t of K (keys 32 t .. +31) lives at byte 4096 t of the K area in the swizzled panel layout of
// fmha_common.h; V likewise.  A copy instruction of the workgroup (512 lanes x 16 bytes) moves 64
// rows, a "pair" of tiles.
#pragma once
#include <type_traits>

#include "fmha_fwd_kernel.h"

namespace fmha {

// tuning knobs (development builds override them on the command line)
#ifndef FMHA_HEAD_AHEAD
#define FMHA_HEAD_AHEAD 2 // LDS operands requested ahead of their matrix instructions
#endif

// QB: 32-query blocks per wave.  2: eight waves (two per SIMD), every LDS operand feeds two matrix instructions.
// 1: sixteen waves (four per SIMD, 128 registers each): twice the LDS operand traffic, but four instruction
// streams per SIMD instead of two to fill its issue slots.
template <int QB_> struct HeadCfgT {
  static constexpr int D = 64, QB = QB_, NW = 16 / QB_, BK = 32, KS = 4, DB = 2;
  static constexpr int NT = NW * 64;       // threads
  static constexpr int QT = NW * QB * 32;  // queries per item
  static constexpr int MAXK = 512;         // keys that fit
  static constexpr int NTILE = MAXK / BK;
  static constexpr int TILEB = BK * kPanelRowB;
  static constexpr int UT = NT / 8 / BK;   // tiles per "unit": the rows one copy instruction of the workgroup moves
  static constexpr int UNITB = UT * TILEB;
  static constexpr int NUNIT = NTILE / UT;
  // The extra-contraction-step rows: eight elements per key, read by the lanes that hold contraction indices 0-7;
  // the other half-wave reads zeros from an area of their own.  Two buffers: the next item's rows are written while
  // the current item's are in use.
  static constexpr int XROWB = 16, XTILEB = BK * XROWB, XBUFB = MAXK * XROWB, ZEROB = 2048;
  static constexpr int LDS_K = 0, LDS_V = MAXK * kPanelRowB, LDS_X = 2 * MAXK * kPanelRowB;
  static constexpr int LDS_ZERO = LDS_X + 2 * XBUFB;
  static constexpr int LDS_TRIM = LDS_ZERO + ZEROB; // per item parity: each wave's count of keys up to its last live one
  static constexpr int LDS_TL = LDS_TRIM + 2 * 16 * 4; // development builds: cycle-counter stamps
#ifdef FMHA_HEAD_TIMELINE
  static constexpr int LDS_BYTES = LDS_TL + NW * 64 * 8;
#else
  static constexpr int LDS_BYTES = LDS_TL;
#endif
};
using HeadCfg = HeadCfgT<2>;

// LDS operands of one iteration in issue order (kind 0: V^T block (c, db) of the second product;
// 1: K rows of contraction step ks; 2: the extra-step rows).  The second product goes first: by the
// time the first product of the next tile claims its accumulators, half of the current tile's
// scores have been turned into probabilities and their registers are free again -- with the two
// products alternating, both score buffers, both probability buffers, the outputs and Q' are all
// live at once, a few registers more than two waves per SIMD have.  (A matrix instruction that
// accumulates onto its predecessor's result issues back to back at full rate on this chip, so
// nothing is lost by not alternating accumulators.)
struct HeadOperandList {
  int n;
  int kind[12], a0[12], a1[12];
};
template <bool HAS_PV, bool HAS_S> constexpr HeadOperandList head_operand_list() {
  constexpr int kDB = 2, kKS = 4;
  HeadOperandList L{};
  int n = 0;
  if (HAS_PV)
    for (int c = 0; c < 2; ++c)
      for (int db = 0; db < kDB; ++db) {
        L.kind[n] = 0; L.a0[n] = c; L.a1[n] = db;
        ++n;
      }
  if (HAS_S)
    for (int i = 0; i <= kKS; ++i) {
      L.kind[n] = i < kKS ? 1 : 2; L.a0[n] = i; L.a1[n] = 0;
      ++n;
    }
  L.n = n;
  return L;
}

FMHA_DEV void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
template <int N> FMHA_DEV void vm_wait() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

// STRIDED: the rows of q, k, v and o lie where the argument block's row maps say ([B,S,H,D] views, packed
// projections) instead of in folded [bh, s, 64] tensors.
template <typename T, int QBW, int MASK, int DROP, bool STRIDED = false>
__global__ __launch_bounds__(HeadCfgT<QBW>::NT) __attribute__((amdgpu_waves_per_eu(4 / QBW, 4 / QBW))) void fmha_fwd_head_kernel(const FwdArgs a) {
  using E = Elem<T>;
  using v8 = typename E::v8;
  using C = HeadCfgT<QBW>;
  constexpr int UT = C::UT, NUNIT = C::NUNIT;
  constexpr int D = C::D, QB = C::QB, BK = C::BK, KS = C::KS, DB = C::DB, TILEB = C::TILEB;
  constexpr int QT = C::QT, XTILEB = C::XTILEB;
  static_assert(MASK == kMaskNone || MASK == kMaskPerKey, "full mask tensors have kernels of their own");
  static_assert(DROP == 0 || DROP == 1, "tensor dropout has kernels of its own");
  constexpr float NEG_INF = -__builtin_inff();
  constexpr float WINDOW = 16384.f;
  constexpr float kHardMask = -9000.f * FMHA_LOG2E; // see fmha_fwd_pipe.h: keys masked this hard weigh exactly zero

  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int tid = threadIdx.x;
  const int w = tid >> 6;
  const int l = tid & 63;
  const int ql = l & 31;
  const int h = l >> 5;

  const bool probe = a.clock_probe != nullptr && blockIdx.x == 0 && tid == 0;
  if (probe) {
    a.clock_probe[0] = __builtin_readcyclecounter();
    a.clock_probe[1] = __builtin_amdgcn_s_memrealtime();
  }

  const int G = gridDim.x;
  const int nitems = a.bh * a.nqt; // nqt: 512-query chunks per head
#ifdef FMHA_HEAD_TIMELINE
  // development aid: cycle-counter stamps of every wave of a few workgroups, kept in LDS and written behind the
  // four clock-probe words at the end (the caller's buffer must hold 4 + grid * waves * 64 words)
  unsigned long long *tl_lds = (unsigned long long *)(lds + C::LDS_TL) + w * 64;
  int tl_n = 0;
#define FMHA_TL()                                                        \
  do {                                                                   \
    if (l == 0 && tl_n < 64) tl_lds[tl_n] = __builtin_readcyclecounter(); \
    ++tl_n;                                                              \
  } while (0)
#else
#define FMHA_TL() do { } while (0)
#endif

  // A per-key mask that ends in hard-masked keys (a padded batch) leaves those keys with a weight of exactly
  // zero: the key tiles that hold nothing else are not visited (bit-identical results; kFwdFlagNoTrim turns it off).
  const bool trimming = MASK == kMaskPerKey && !(a.flags & kFwdFlagNoTrim);

  struct Item {
    int bh, qc, kend; // kend: keys this head may see at all (its valid count); the mask may shorten the item further
  };
  auto make_item = [&](int idx) {
    Item it;
    it.bh = a.nqt == 1 ? idx : idx / a.nqt; // (one chunk per head: no division on the way to the first requests)
    it.qc = idx - it.bh * a.nqt;
    it.kend = visible_keys<STRIDED>(a, it.bh, 0);
    return it;
  };
  // tiles an item of n keys visits: an even number, so that the x / P buffers keep fixed roles
  auto tiles2 = [&](int n) {
    int nkt = (n + BK - 1) / BK;
    if (nkt < 1) nkt = 1;
    return (nkt + 1) & ~1;
  };

  // ---- copies: unit u (rows 32 UT u .. of a head's K or V: what one copy instruction of the workgroup moves) into
  // its place in LDS.  Rows at or past kend re-read the last valid row (finite values that meet a probability of
  // zero).
  const uint32_t lds_base = lds_address(lds);
  const uint32_t wave_dst = (uint32_t)__builtin_amdgcn_readfirstlane(w) * 1024u;
  const int crow = tid >> 3;                                        // the lane's row within a unit
  const uint32_t ccolb = (uint32_t)(((tid & 7) ^ ((crow >> 1) & 7)) * 16); // byte offset of the 16-byte chunk that belongs at the lane's slot
  auto dma_unit = [&](const void *tensor, const Item &it, int u, uint32_t area) {
    const uint32_t dst = lds_base + area + (uint32_t)u * C::UNITB + wave_dst;
    int r = u * (UT * BK) + crow;
    const int last = it.kend > 0 ? it.kend - 1 : 0;
    r = r < last ? r : last;
    if constexpr (!STRIDED) {
      dma_global_to_lds_b128((const T *)tensor + (size_t)it.bh * (size_t)a.sk * D, (uint32_t)r * (D * 2) + ccolb, dst);
    } else {
      const RowMap &map = area == (uint32_t)C::LDS_K ? a.mk : a.mv;
      dma_global_to_lds_b128((const T *)tensor + map.head(it.bh), (uint32_t)r * ((uint32_t)map.ss * 2u) + ccolb, dst);
    }
  };
  auto dmaK = [&](const Item &it, int u) { dma_unit(a.k, it, u, (uint32_t)C::LDS_K); };
  auto dmaV = [&](const Item &it, int u) { dma_unit(a.v, it, u, (uint32_t)C::LDS_V); };
  auto units_of = [&](const Item &it) { return (it.kend + UT * BK - 1) / (UT * BK); }; // units that hold any of its rows

  // ---- the extra-step rows (validity and per-key mask of each key): thread = key
  auto load_xm = [&](const Item &it) -> T {
    if (MASK != kMaskPerKey) return (T)0.f;
    const int last = it.kend > 0 ? it.kend - 1 : 0;
    return ((const T *)a.mask + (size_t)(it.bh / a.mask_div) * a.mask_sb)[tid < last ? tid : last]; // (threads past the 512th: unused)
  };
  // writes key tid's row into buffer xb and this wave's count of keys up to its last live one (0: none) beside it
  auto storeX = [&](T mraw, int kend, int xb) {
    float mk = 0.f;
    if (MASK == kMaskPerKey) mk = fmaf((float)mraw, a.mask_a, a.mask_b);
    if (!(tid < kend)) mk = NEG_INF;
    const T hi = (T)mk;
    const bool fin = (float)hi != NEG_INF;
    const T lo = fin ? (T)(mk - (float)hi) : (T)0.f;
    v8 x0;
#pragma unroll
    for (int j = 0; j < 8; ++j) x0[j] = (T)0.f;
    x0[0] = (T)1.f;
    x0[1] = hi;
    x0[2] = lo;
    x0[3] = (T)1.f;
    if (tid < C::MAXK) *(v8 *)(lds + C::LDS_X + xb * C::XBUFB + tid * C::XROWB) = x0;
    if (MASK == kMaskPerKey) {
      const unsigned long long live = __builtin_amdgcn_ballot_w64(tid < kend && mk > kHardMask);
      if (l == 0 && w < C::MAXK / 64) ((int *)(lds + C::LDS_TRIM))[xb * 16 + w] = live ? w * 64 + 64 - (int)__builtin_clzll(live) : 0;
    }
  };
  // keys of the item whose rows are in buffer xb: up to its last live key (all of them if none is live)
  auto trimmed_keys = [&](int kend, int xb) {
    if (MASK != kMaskPerKey || !trimming) return kend;
    const int *tr = (const int *)(lds + C::LDS_TRIM) + xb * 16;
    int n = 0;
#pragma unroll
    for (int i = 0; i < C::MAXK / 64; ++i) {
      const int c = tr[i];
      n = c > n ? c : n;
    }
    n = __builtin_amdgcn_readfirstlane(n);
    return n > 0 && n < kend ? n : kend;
  };

  // ---- Q rows: lane (ql, h) owns chunks [16 ks + 8 h, +8) of rows q0w + 32 qb + ql
  auto q_row = [&](const Item &it, int qb) {
    int q = it.qc * QT + w * (QB * 32) + qb * 32 + ql;
    q = q < a.sq ? q : a.sq - 1; // rows past the end repeat the last valid row and are never stored
    if constexpr (!STRIDED) return (const T *)a.q + ((size_t)it.bh * (size_t)a.sq + (size_t)q) * D + h * 8;
    else return (const T *)a.q + a.mq.head(it.bh) + (size_t)q * (size_t)a.mq.ss + h * 8;
  };
  u32x4 qraw[QB][KS];
  // (real = false: a request that must exist for the registers' sake but whose rows nobody will use -- every
  // lane reads the tensor's first row, one cache line instead of the wave's 8 KB)
  auto loadQ = [&](const Item &it, bool real = true) {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      const T *row = real ? q_row(it, qb) : (const T *)a.q + h * 8;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) qraw[qb][ks] = *(const u32x4 *)(row + ks * 16);
    }
  };

  // ---- LDS operand addresses.  Each lane keeps the byte offsets of what it reads of the tiles the current loop
  // trip starts at (K: its row's four chunk pairs; V: its transposed read; extra rows: its key's row, or the
  // zeros) and the tiles of a trip are fixed distances from there, so every read is base register + immediate and
  // the bases move once per trip.
  PanelLane pl;
  pl.init(l);
  uint32_t kofs[4], vofs, xofs;
  const uint32_t xstep = h ? 0u : (uint32_t)XTILEB;
  auto cursors_to_tile0 = [&](int xb) {
#pragma unroll
    for (int j = 0; j < 4; ++j) kofs[j] = (uint32_t)C::LDS_K + pl.rowofs[j];
    vofs = (uint32_t)C::LDS_V + pl.trofs;
    xofs = h ? (uint32_t)C::LDS_ZERO : (uint32_t)(C::LDS_X + xb * C::XBUFB + ql * C::XROWB);
  };
  auto pin_cursors = [&]() { // (keeps the compiler from re-deriving them from the loop counter, one add per read)
#pragma unroll
    for (int j = 0; j < 4; ++j) asm volatile("" : "+v"(kofs[j]));
    asm volatile("" : "+v"(vofs), "+v"(xofs));
  };
  auto advance_cursors = [&](int tiles) {
#pragma unroll
    for (int j = 0; j < 4; ++j) kofs[j] += (uint32_t)(tiles * TILEB);
    vofs += (uint32_t)(tiles * TILEB);
    xofs += (uint32_t)tiles * xstep;
    pin_cursors();
  };
  auto readK = [&](int off, int ks) -> v8 { return as_v8<T>(*(const u32x4 *)(lds + kofs[ks] + off)); };
  auto readX = [&](int off) -> v8 { return as_v8<T>(*(const u32x4 *)(lds + xofs + off)); };
  auto readV = [&](int off, int db, int c) -> v8 {
    const char *p0 = lds + vofs + off + 16 * c * kPanelRowB;
    const u32x2 lo = lds_read_tr16(p0 + (db & 1) * 64);
    const u32x2 hi = lds_read_tr16(p0 + 8 * kPanelRowB + ((db & 1) ^ 1) * 64);
    const u32x4 both = {lo.x, lo.y, hi.x, hi.y};
    return as_v8<T>(both);
  };

  // ---- running state (see fmha_fwd_pipe.h for the bookkeeping of the lazily raised reference)
  f32x16 o[QB][DB];
  float mref[QB], lsum[QB];
  bool seen[QB];
  v8 bx[QB];
  v8 qreg[QB][KS];
  f32x16 xA[QB], xB[QB];
  float bkA[QB], bkB[QB];   // the reference baked into each score buffer
  float limA[QB], limB[QB]; // the row-sum limit that goes with it: the 2^14 window, or -1 once the reference has moved on
  float lim_now[QB];        // what a buffer baked now would get: -1 until a row has a reference
  v8 pA[QB][2], pB[QB][2];
  int bh = 0, q0w = 0;

  // first product of the tile koff / xoff bytes past the cursors
  auto g1 = [&](int koff, int xoff, f32x16 (&x)[QB], float (&bk)[QB], float (&lim)[QB]) {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      bk[qb] = mref[qb];
      lim[qb] = lim_now[qb];
#pragma unroll
      for (int r = 0; r < 16; ++r) x[qb][r] = 0.f;
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const v8 ka = readK(koff, ks);
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) x[qb] = E::mfma(ka, qreg[qb][ks], x[qb]);
    }
    const v8 xa = readX(xoff);
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) x[qb] = E::mfma(xa, bx[qb], x[qb]);
  };
  auto g2 = [&](int voff, const v8 (&p)[QB][2]) {
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const v8 va = readV(voff, db, c);
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) o[qb][db] = E::mfma(va, p[qb][c], o[qb][db]);
      }
  };

  // One iteration's matrix work and softmax arithmetic as ONE hand-ordered stream: the second
  // product of the tile voff past the V cursor (probabilities p; HAS_PV), the first product of the tile
  // koff / xoff past the K / extra-row cursors into x (HAS_S) and P = exp2(xc [+ shift]) rounded into pc
  // with its row sums rs -- groups of {request operand j + 2, matrix instructions of operand j, a share
  // of the softmax arithmetic}, each closed by a scheduling barrier.
  auto fused_step = [&](auto pv_tag, auto s_tag, auto shift_tag, int voff, const v8 (&p)[QB][2], int koff, int xoff,
                        f32x16 (&x)[QB], float (&bk)[QB], float (&lim)[QB], const f32x16 (&xc)[QB],
                        const float (&shift)[QB], v8 (&pc)[QB][2], float (&rs)[QB]) {
    constexpr bool HAS_PV = decltype(pv_tag)::value, HAS_S = decltype(s_tag)::value;
    constexpr bool SHIFTED = decltype(shift_tag)::value;
    constexpr HeadOperandList ops = head_operand_list<HAS_PV, HAS_S>();
    constexpr int kAhead = FMHA_HEAD_AHEAD; // LDS operands in flight
    constexpr int NSL = QB * 8; // slices: two exponentials, one pack, one dot2 each
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      if (HAS_S) {
        bk[qb] = mref[qb];
        lim[qb] = lim_now[qb];
      }
    }
    auto fetch = [&](int j) -> v8 {
      if (ops.kind[j] == 0) return readV(voff, ops.a1[j], ops.a0[j]);
      if (ops.kind[j] == 1) return readK(koff, ops.a0[j]);
      return readX(xoff);
    };
    // The softmax arithmetic of a slice is a chain of three dependent steps -- two exponentials, their packing
    // into the element type, the addition of the rounded pair to the row sum -- and a wave issues in order:
    // written as a chain, every step waits out the latency of the one before it.  The steps therefore run as
    // a three-stage pipeline over the groups of the stream: a group starts the exponentials of its slices,
    // packs the slices that the previous group started and sums the slices that the group before that packed,
    // so nothing in a group depends on anything else in it.  The row sum runs on two accumulators.
    float ex[NSL][2];
    float rsa[QB][2];
    auto stage_exp = [&](int sidx) {
      const int qb = sidx / 8, pr = sidx % 8;
      float y0 = xc[qb][2 * pr], y1 = xc[qb][2 * pr + 1];
      if (SHIFTED) {
        y0 += shift[qb];
        y1 += shift[qb];
      }
      ex[sidx][0] = fast_exp2(y0), ex[sidx][1] = fast_exp2(y1);
    };
    auto stage_pack = [&](int sidx) {
      const int qb = sidx / 8, pr = sidx % 8, c = pr / 4, j = pr % 4;
      pc[qb][c][2 * j] = (T)ex[sidx][0];
      pc[qb][c][2 * j + 1] = (T)ex[sidx][1];
    };
    auto stage_sum = [&](int sidx) {
      // fp32 sums of the rounded pair (see sum_pair: not a packed dot product)
      const int qb = sidx / 8, pr = sidx % 8, c = pr / 4, j = pr % 4;
      if (pr == 0) rsa[qb][0] = rsa[qb][1] = 0.f;
      sum_pair<T>(pc[qb][c], j, rsa[qb][0], rsa[qb][1]);
      // (the sums are only needed after the last group, and the compiler would gather them all there)
      asm volatile("" : "+v"(rsa[qb][0]), "+v"(rsa[qb][1]));
    };
    // slices whose exponentials have been started once group j is through: all of them one group before the last
    auto started = [&](int j) { return j < 0 ? 0 : (j + 1 >= ops.n - 1 ? NSL : (j + 1) * NSL / (ops.n - 1)); };
    v8 opnd[ops.n];
#pragma unroll
    for (int j = 0; j < kAhead && j < ops.n; ++j) opnd[j] = fetch(j);
#pragma unroll
    for (int j = 0; j < ops.n; ++j) {
      if (j + kAhead < ops.n) opnd[j + kAhead] = fetch(j + kAhead);
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        if (ops.kind[j] == 0) {
          o[qb][ops.a1[j]] = E::mfma(opnd[j], p[qb][ops.a0[j]], o[qb][ops.a1[j]]);
        } else {
          f32x16 acc;
          if (ops.a0[j] == 0) {
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[r] = 0.f;
          } else {
            acc = x[qb];
          }
          x[qb] = E::mfma(opnd[j], ops.kind[j] == 1 ? qreg[qb][ops.a0[j]] : bx[qb], acc);
        }
      }
#pragma unroll
      for (int sidx = started(j - 1); sidx < started(j); ++sidx) stage_exp(sidx);
#pragma unroll
      for (int sidx = started(j - 2); sidx < started(j - 1); ++sidx) stage_pack(sidx);
#pragma unroll
      for (int sidx = started(j - 3); sidx < started(j - 2); ++sidx) stage_sum(sidx);
      __builtin_amdgcn_sched_barrier(0);
    }
    // what the pipeline still owes: the sums of the slices that the last group packed
#pragma unroll
    for (int sidx = started(ops.n - 3); sidx < NSL; ++sidx) stage_sum(sidx);
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) rs[qb] = rsa[qb][0] + rsa[qb][1];
  };

  // P = exp2(x + shift) rounded to T, and the row sum of the rounded values (the rare re-base path)
  auto exp_pack = [&](const f32x16 &x, float shift, v8 (&pk)[2]) -> float {
    float rs0 = 0.f, rs1 = 0.f;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
#pragma unroll
      for (int j = 0; j < 8; ++j) pk[c][j] = (T)fast_exp2(x[8 * c + j] + shift);
#pragma unroll
      for (int j = 0; j < 4; ++j) sum_pair<T>(pk[c], j, rs0, rs1);
    }
    return rs0 + rs1;
  };
  // move the reference of query block qb to this tile's maximum (x is relative to bk); returns the
  // shift that re-bases x onto the new reference
  auto rebase = [&](int qb, const f32x16 &x, float bk) -> float {
    float mx = NEG_INF;
#pragma unroll
    for (int r = 0; r < 16; r += 2) mx = max3(mx, x[r], x[r + 1]);
    mx = xhalf_max(mx);
    const float shift0 = bk - mref[qb];
    float mnew = mref[qb];
    if (mx != NEG_INF) {
      const float cand = (float)(T)(bk + mx);
      mnew = seen[qb] ? fmaxf(mref[qb], cand) : cand;
      seen[qb] = true;
      lim_now[qb] = WINDOW;
    }
    const float up = mref[qb] - mnew;
    if (up != 0.f) {
      const float alpha = fast_exp2(up);
      lsum[qb] *= alpha;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[qb][db][r] *= alpha;
    }
    mref[qb] = mnew;
    if (h == 0) bx[qb][0] = (T)(-mnew);
    return shift0 + up;
  };
  auto dropout = [&](int tile, int qb, v8 (&pk)[2]) {
    if (DROP == 1) {
      const int q = q0w + qb * 32 + ql;
      uint32_t wd[4];
      drop_words_q(a.drop, (uint32_t)bh, (uint32_t)q, (uint32_t)(tile * BK), h, l, wd);
      const uint32_t thr2 = ((a.drop.thr - 1u) & 0xffffu) * 0x00010001u; // thr = 0 gives -1: everything kept
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        Pack16 pp;
        if constexpr (std::is_same<T, _Float16>::value) pp.h = pk[c];
        else pp.b = pk[c];
        uint32_t r0 = pp.u.x, r1 = pp.u.y, r2 = pp.u.z, r3 = pp.u.w;
        drop_apply_pk4(wd[2 * c], thr2, r0, r1);
        drop_apply_pk4(wd[2 * c + 1], thr2, r2, r3);
        pp.u = u32x4{r0, r1, r2, r3};
        if constexpr (std::is_same<T, _Float16>::value) pk[c] = pp.h;
        else pk[c] = pp.b;
      }
    }
  };

  using Yes = std::true_type;
  using No = std::false_type;
  const float no_shift[QB] = {};

  // Steady-state iteration t, the SECOND-th (0 / 1) of its loop trip (LAST: there is no next tile): second product
  // of tile t - 1, first product of tile t + 1, softmax of tile t.  The trip's cursors stand at tile t - SECOND of K
  // and of the extra rows and one tile below that of V.
  auto steady = [&](int t, auto second_tag, auto last_tag, f32x16 (&xc)[QB], float (&bkc)[QB], float (&limc)[QB],
                    f32x16 (&xn)[QB], float (&bkn)[QB], float (&limn)[QB], v8 (&pprev)[QB][2], v8 (&pcur)[QB][2]) {
    constexpr int SECOND = decltype(second_tag)::value;
    constexpr bool LAST = decltype(last_tag)::value;
    float rs[QB];
    fused_step(Yes{}, std::integral_constant<bool, !LAST>{}, No{}, SECOND * TILEB, pprev, (SECOND + 1) * TILEB,
               (SECOND + 1) * XTILEB, xn, bkn, limn, xc, no_shift, pcur, rs);
    // The probabilities are good if the rounded row sum stayed inside the window that belongs to the buffer's
    // reference; otherwise (rare) the tile is redone on a new reference.
    bool unfit = false;
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) unfit = unfit | !(rs[qb] < limc[qb]); // no short circuit: keep one basic block
    if (__builtin_amdgcn_ballot_w64(unfit) != 0ull) {
      // The scores are formed again (tile t's K rows are still in LDS), relative to the reference that is current
      // now: keeping the first copy for this path would hold 32 registers through every iteration that does not
      // take it.
      f32x16 xr[QB];
      float bkr[QB], limr[QB];
      g1(SECOND * TILEB, SECOND * XTILEB, xr, bkr, limr);
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        const float shift = rebase(qb, xr[qb], bkr[qb]);
        rs[qb] = exp_pack(xr[qb], shift, pcur[qb]);
        if (!LAST && bkn[qb] != mref[qb]) limn[qb] = -1.f; // the next buffer was baked with the old reference
      }
    }
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      lsum[qb] += rs[qb];
      dropout(t, qb, pcur[qb]);
    }
  };

  // ---- the items
  // Hooks: before iterations 3, 7, 11 and 15 every wave waits for the copies it has issued, meets the others at a
  // barrier and requests the next item's rows for the tiles that all waves have now left.  Iteration t reads tiles
  // t + 1 (first product) and t (the rare re-base) of K and t - 1 of V, so before iteration T the tiles up to T - 1 of
  // K and T - 2 of V are free: pair 0 at T = 3, pairs 1-2 at 7, 3-4 at 11, 5-6 at 15; what is left (pair 7) follows
  // at the next item's own hook 3, by when every wave has left this item.  The copies thus leave in even portions
  // instead of one burst per item that every compute unit would issue at the same moment.  The next item's
  // extra-step rows are written into the other buffer at hook 7 (mask values requested at hook 3); from hook 11 on
  // they are visible to every wave, and an item whose predecessor got that far starts WITHOUT a barrier: each wave
  // walks on into it as soon as its own Q rows are there.  Otherwise (first item of a workgroup, or a very short
  // predecessor) the item starts cold: barrier, first tiles, barrier, and its rows arrive while it computes -- its
  // hook 3 waits only for those that iterations 3-6 read (tiles 4-7 of K, 2-5 of V).
  // Q' = Q * scale * log2(e), rounded once, as B-operand registers.  The conversion must happen where this is called:
  // left alone the compiler sinks it towards the first use of Q' -- below copies issued in between, and its wait for
  // the raw rows, counted without those copies, then waits for all of them.
  auto convertQ = [&]() {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const v8 raw = as_v8<T>(qraw[qb][ks]);
#pragma unroll
        for (int j = 0; j < 8; ++j) qreg[qb][ks][j] = (T)((float)raw[j] * a.scale_l2);
        asm volatile("" : "+v"(qreg[qb][ks]));
      }
  };
  int pf = 0;        // pairs of the current item's K and V that its predecessor requested
  bool xready = false; // ... and whether it wrote the item's extra-step rows
  int xb = 0;        // the extra-row buffer of the current item
  T xm = (T)0.f;     // a mask value on its way from memory to an extra-step row
  Item cur = make_item(blockIdx.x);
  if (tid < C::ZEROB / 4) ((uint32_t *)(lds + C::LDS_ZERO))[tid] = 0u;
  static_assert(C::ZEROB / 4 <= C::NT, "one word per thread clears the zero area");
  for (int idx = blockIdx.x;;) {
    const int nidx = idx + G;
    const bool more = nidx < nitems;
    bh = cur.bh;
    q0w = cur.qc * QT + w * (QB * 32);
    const bool cold = !(xready && pf >= (8 + UT - 1) / UT); // (tiles 0-7 are read before the item's own hook 3 copies could land)

    FMHA_TL(); // 0: item start
    if (cold) {
      // Every wave has left the previous item (its tiles and extra rows are about to be overwritten).  Tiles 0-3
      // of K and 0-1 of V and the mask values go first, the Q rows behind them: the barrier below needs every
      // wave's part of the former, but a wave's Q rows are its own business, so it comes BEFORE the wait for them
      // and a wave starts computing as soon as its own rows are there.
      if (idx != (int)blockIdx.x) lds_barrier();
      dmaK(cur, 0);
      dmaV(cur, 0);
      if (UT == 2) dmaK(cur, 1);
      xm = load_xm(cur);
      loadQ(cur);
      __builtin_amdgcn_sched_barrier(0);
      storeX(xm, cur.kend, xb); // (the compiler's wait for the mask value leaves the QB * KS loads behind it in flight)
      __builtin_amdgcn_sched_barrier(0);
      vm_wait<QB * KS>();       // this wave's part of the first tiles is in LDS
      lds_barrier();            // ... and everybody's, and the extra rows
    }
    // (A warm item has nothing to wait for: its Q rows were converted at the end of the previous item, before that
    // item's output stores went out -- a wait for them here would also wait for those stores -- and its first tiles
    // were confirmed by the previous item's hooks.)
    __builtin_amdgcn_sched_barrier(0);
    const Item nxt = make_item(more ? nidx : idx);
    FMHA_TL(); // 1: requests out and first tiles in (cold)
    if (cold) convertQ();
    if (cold) {
      __builtin_amdgcn_sched_barrier(0);
      // (the Q rows have been consumed: nothing of this wave's is in flight)  The rest of the item's rows in the
      // order of their use; hook 3 waits for the first of them
      if (UT == 2) {
        dmaV(cur, 1);
        dmaK(cur, 2);
        dmaK(cur, 3);
        dmaV(cur, 2);
        dmaV(cur, 3);
      } else {
        dmaK(cur, 1);
        dmaV(cur, 1);
      }
#pragma unroll
      for (int u = 8 / UT; u < NUNIT; ++u) {
        dmaK(cur, u);
        dmaV(cur, u);
      }
    }
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      mref[qb] = 0.f;
      seen[qb] = false;
      lim_now[qb] = -1.f;
      lsum[qb] = 0.f;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[qb][db][r] = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) bx[qb][j] = (T)0.f;
      if (h == 0) {
        bx[qb][1] = (T)1.f;
        bx[qb][2] = (T)1.f;
      }
    }
    FMHA_TL(); // 2: Q converted, state cleared
    FMHA_TL(); // 3
    const int nkt2 = tiles2(trimmed_keys(cur.kend, xb));
    const int np = units_of(cur), npn = units_of(nxt);
    // copies a cold item still has in flight at its hook 3 once those that iterations 3-6 read have landed
    constexpr int kColdLeft3 = UT == 2 ? 9 : 4;

    int pfn = 0;
    bool xnext = false;
    auto hook = [&](int t) {
      if ((t & 3) != 3) return;
      if (cold && t == 3) vm_wait<kColdLeft3>();
      else vm_wait<0>();
      lds_barrier();
      // (a load the compiler knows about is consumed before any copy goes out behind it: its wait for that load
      // would also wait for those copies)
      if (more && t == 7) {
        storeX(xm, nxt.kend, xb ^ 1);
        xnext = true;
      }
      __builtin_amdgcn_sched_barrier(0);
      if (t == 3 && !cold)
        for (int p = pf; p < np; ++p) { // what the predecessor's hooks did not get to: first read in iteration 9 or later
          dmaK(cur, p);
          dmaV(cur, p);
        }
      if (more) {
        const int free_pairs = (t - 1) / UT; // whole units among the tiles 0 .. t - 2
        for (int p = pfn; p < free_pairs; ++p)
          if (p < npn) {
            dmaK(nxt, p);
            dmaV(nxt, p);
          }
        pfn = free_pairs;
        if (t == 3) xm = load_xm(nxt);
      }
    };

    cursors_to_tile0(xb);
    pin_cursors();
    g1(0, 0, xA, bkA, limA);
    FMHA_TL(); // 4: first product of tile 0
    { // t = 0: the reference from tile 0, then its softmax inside the first product of tile 1
      float shift[QB], rs[QB];
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) shift[qb] = rebase(qb, xA[qb], bkA[qb]);
      fused_step(No{}, Yes{}, Yes{}, 0, pB, TILEB, XTILEB, xB, bkB, limB, xA, shift, pA, rs);
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        lsum[qb] += rs[qb];
        dropout(0, qb, pA[qb]);
      }
    }
    // from here on the cursors stand at the trip's first tile for K and the extra rows and one tile below for V
#pragma unroll
    for (int j = 0; j < 4; ++j) kofs[j] += (uint32_t)TILEB;
    xofs += xstep;
    pin_cursors();
    FMHA_TL(); // 5: iteration 0
#ifdef FMHA_HEAD_LOOPX
    // development aid (wrong results): the steady-state iterations FMHA_HEAD_LOOPX times over, without hooks
    for (int rep = 1; rep < FMHA_HEAD_LOOPX; ++rep)
      for (int t = 1; t < nkt2 - 1; t += 2) {
        steady(t, std::integral_constant<int, 0>{}, No{}, xB, bkB, limB, xA, bkA, limA, pA, pB);
        steady(t + 1, std::integral_constant<int, 1>{}, No{}, xA, bkA, limA, xB, bkB, limB, pB, pA);
      }
#endif
    for (int t = 1; t < nkt2 - 1; t += 2) {
      hook(t);
      FMHA_TL(); // 6, 9, ...: hook
      steady(t, std::integral_constant<int, 0>{}, No{}, xB, bkB, limB, xA, bkA, limA, pA, pB);
      FMHA_TL(); // 7, 10, ...: odd iteration
      steady(t + 1, std::integral_constant<int, 1>{}, No{}, xA, bkA, limA, xB, bkB, limB, pB, pA);
      advance_cursors(2);
      FMHA_TL(); // 8, 11, ...: even iteration
    }
    {
      const int t = nkt2 - 1;
      hook(t);
      // The Q registers have had their last use: request the next item's rows.  (Unconditionally, so that the
      // raw rows are not a value that has to survive the whole item on the path that would not load them; an
      // item that starts cold loads them again, and after the last item the request is for one row only.)
      loadQ(nxt, more);
      FMHA_TL(); // last hook and Q request
      steady(t, std::integral_constant<int, 0>{}, Yes{}, xB, bkB, limB, xA, bkA, limA, pA, pB);
      FMHA_TL(); // last iteration
      g2(TILEB, pB);
      FMHA_TL(); // last second product
    }
    if (more && xnext && pfn < (8 + UT - 1) / UT) {
      // A short item (fewer than twelve tiles) has not reached the hooks that request the middle of the next
      // item's rows, which that item's first iterations read.  They go out now, behind a barrier: every wave
      // has finished this item's tiles (and the copies of hook 7 have landed).
      vm_wait<0>();
      lds_barrier();
      for (int p = pfn; p < npn; ++p) {
        dmaK(nxt, p);
        dmaV(nxt, p);
      }
      pfn = NUNIT;
    }

    // ---- item epilogue
    // The next item's Q rows (requested at the last hook) become Q' before this item's outputs are stored: the
    // wait for them covers only older requests, and the next item starts without a wait.
    if (more) convertQ();
    T *Ob = (T *)a.o + (STRIDED ? a.mo.head(bh) : (size_t)bh * (size_t)a.sq * D);
    const size_t o_pitch = STRIDED ? (size_t)a.mo.ss : (size_t)D;
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      const int q = q0w + qb * 32 + ql;
      const float lt = xhalf_sum(lsum[qb]);
      const float inv = lt > 0.f ? a.drop_scale / lt : 0.f;
      if (q < a.sq) {
#pragma unroll
        for (int db = 0; db < DB; ++db) store_acc_block_row<T>(Ob + (size_t)q * o_pitch + db * 32, o[qb][db], inv, h);
        if (a.lse && h == 0) a.lse[(size_t)bh * a.sq + q] = lt > 0.f ? (mref[qb] + fast_log2(lt)) * FMHA_LN2 : NEG_INF;
      }
    }
    FMHA_TL(); // stores issued
    if (!more) break;
    idx = nidx;
    cur = nxt;
    pf = pfn;
    xready = xnext;
    xb ^= 1;
  }
  vm_wait<0>(); // no copy may still be on its way into LDS when the wave ends
#ifdef FMHA_HEAD_TIMELINE
  if (a.clock_probe != nullptr && l == 0)
    for (int i = 0; i < 64; ++i) a.clock_probe[4 + ((size_t)blockIdx.x * C::NW + w) * 64 + i] = i < tl_n ? tl_lds[i] : 0ull;
#endif
  if (probe) {
    a.clock_probe[2] = __builtin_readcyclecounter();
    a.clock_probe[3] = __builtin_amdgcn_s_memrealtime();
  }
}

} // namespace fmha
