// Software-pipelined forward attention kernel for gfx950 (no dropout-tensor / save pass;
// those stay on fmha_fwd_kernel).  Same data layout, same MFMA formulation and the same
// softmax bookkeeping as fmha_fwd_kernel (see the header of fmha_fwd_kernel.h); what
// changes is the ORDER of work inside a wave.
//
// On this hardware a wave issues in order, and MFMA and VALU work overlap only when
// they are interleaved in the instruction stream of one wave (two waves on a SIMD
// overlap them only partially).  The loop is therefore skewed so that every iteration
// holds three mutually independent pieces in one basic block:
//     O^T    += V(t-1)^T . P(t-1)^T          MFMA   (second product of the previous tile)
//     x(t+1)  = K(t+1) . Q'^T + extra step    MFMA   (first product of the next tile)
//     P(t)    = exp2(x(t)), row sums           VALU   (softmax of the current tile)
// and the scheduler is told to interleave them.  Iteration t needs K(t+1) and V(t-1) in
// LDS and fetches K(t+2) and V(t); both still fit two stages each because the stage a
// fetch overwrites was last read one iteration earlier.
//
// K and V tiles go from global memory straight into LDS (global_load_lds_dwordx4: every
// lane names a 16-byte global chunk and the wave's 64 chunks land in 1 KiB of consecutive
// LDS), issued at the top of an iteration and awaited at its end, so no registers and no
// VALU/LDS-write issue slots are spent on staging; the tiles use the swizzled panel layout
// of fmha_common.h.
//
// Workgroups are persistent: the grid holds as many workgroups as the chip keeps resident
// and each walks a strided list of (head, query tile) items.  The K and extra-row streams
// simply run on into the next item's first tiles, and the next item's Q rows are copied
// into an LDS buffer of their own as soon as the current Q has been read, so that only the
// first item of a workgroup waits for global memory before it can start computing.
//
// x(t+1) is started before the softmax of tile t may raise the reference exponent, so
// each x buffer remembers the reference that was baked into it; a mismatch sends that
// tile through the (rare) correction path, which re-bases the exponentials.
#pragma once
#include <type_traits>

#include "fmha_fwd_kernel.h"

namespace fmha {

template <int D, int QB> struct PipeCfg {
  // keys per LDS tile: the two in-flight score buffers of a wave hold QB x BK/32 accumulator
  // tiles each, which is what the register file can carry
  static constexpr int BK = 64 / QB;
  static constexpr int NSB = BK / 32; // 32-key sub-blocks per tile
  static constexpr int KS = D / 16;   // contraction steps of K.Q^T
  static constexpr int DB = D / 32;   // 32-row blocks of O^T
  static constexpr int TILEB = BK * D * 2; // swizzled panel layout, no padding
  static constexpr int XROWB = 32;    // pitch of the extra-contraction-step rows (16 elements)
  // The next item's Q rows are prefetched into LDS where that still leaves room for two
  // workgroups per CU; otherwise Q is loaded from global memory when the item starts.
  static constexpr bool QLDS = (D == 64);
  static constexpr int LDS_BYTES = 4 * TILEB + 2 * BK * XROWB; // {K,V} x 2 stages + extra rows x 2 stages
  static constexpr int TRIM_BYTES = 256; // per-item key counts derived from a per-key mask, at the very end
  static constexpr int lds_bytes(int nw) { return LDS_BYTES + (QLDS ? nw * QB * 32 * D * 2 : 0) + TRIM_BYTES; }
};

// The LDS operands of one steady-state iteration in issue order.  kind 0: V^T block of the
// second product (sb, c, db); kind 1: K rows of contraction step ks for sub-block sb; kind 2: the
// extra-step rows of sub-block sb.  The two products alternate so that consecutive MFMAs never
// share an accumulator: a dependent MFMA cannot start until its predecessor has drained the
// matrix pipe (about twice the issue interval).
struct FwdOperandList {
  int n;
  int kind[48], a0[48], a1[48], a2[48];
};
template <int NSB, int KS, int DB, bool WITH_FIRST_PRODUCT> constexpr FwdOperandList fwd_operand_list() {
  FwdOperandList L{};
  int n = 0;
  constexpr int S2 = NSB * 2, S1 = WITH_FIRST_PRODUCT ? KS + 1 : 0, S = S2 > S1 ? S2 : S1;
  for (int i = 0; i < S; ++i) {
    if (i < S2)
      for (int db = 0; db < DB; ++db) {
        L.kind[n] = 0; L.a0[n] = i / 2; L.a1[n] = i % 2; L.a2[n] = db;
        ++n;
      }
    if (i < S1)
      for (int sb = 0; sb < NSB; ++sb) {
        L.kind[n] = i < KS ? 1 : 2; L.a0[n] = i; L.a1[n] = sb; L.a2[n] = 0;
        ++n;
      }
  }
  L.n = n;
  return L;
}

// (Two query blocks per wave, head dim 128, and the staged values of a full mask tensor under a
// causal mask need more than the 256 registers of a two-waves-per-SIMD budget by a few; the occupancy attribute makes the compiler spill those
// few instead of settling for one wave per SIMD, which measures 8-30 % faster.)
template <typename T, int D, int QB, int NW, int MASK, bool CAUSAL, int DROP, bool STRIDED>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu((QB == 2 || D == 128 || MASK == kMaskFull || DROP == 2) ? 2 : 1, 2))) void fmha_fwd_pipe_kernel(const FwdArgs a) {
  using RW = Rows<STRIDED, D>;
  using E = Elem<T>;
  using v8 = typename E::v8;
  using v4 = typename E::v4;
  using C = PipeCfg<D, QB>;
  constexpr int BK = C::BK, NSB = C::NSB, KS = C::KS, DB = C::DB, XROWB = C::XROWB;
  constexpr int TILEB = C::TILEB;
  constexpr int NT = NW * 64;
  constexpr int QT = NW * QB * 32;
  static_assert(NT >= BK, "the extra rows are staged by the first BK threads");
  static_assert(DROP == 0 || DROP == 1 || (DROP == 2 && D == 64 && !CAUSAL),
                "the save pass, and tensor dropout at head dim 128, use fmha_fwd_kernel");
  static_assert(D % 64 == 0, "tiles are stored as panels of 64 columns");
  constexpr float NEG_INF = -__builtin_inff();
  constexpr float WINDOW = 16384.f;

  extern __shared__ __attribute__((aligned(16))) char lds[];
  // layout: K stage 0, K stage 1, V stage 0, V stage 1, extra rows stage 0, stage 1
  char *ldsKb = lds;
  char *ldsVb = lds + 2 * TILEB;
  char *ldsXb = lds + 4 * TILEB;

  const int tid = threadIdx.x;
  const int w = tid >> 6;
  const int l = tid & 63;
  const int ql = l & 31;
  const int h = l >> 5;

  // diagnostic: core clock counter and constant 100 MHz counter when the first workgroup starts
  // (and, at the end of the kernel, when it finishes)
  const bool probe = a.clock_probe != nullptr && blockIdx.x == 0 && tid == 0;
  if (probe) {
    a.clock_probe[0] = __builtin_readcyclecounter();
    a.clock_probe[1] = __builtin_amdgcn_s_memrealtime();
  }

  // ---- persistent schedule: this workgroup handles items lb, lb + G, lb + 2G, ...
  // Workgroups are dealt round-robin to the 8 XCDs; lb is chosen so that one XCD (one L2)
  // works on a contiguous run of items at any time, i.e. on the query tiles of few heads.
  const int G = gridDim.x;
  const int nitems = a.bh * a.nqt;
  int lb = blockIdx.x;
  if ((G & 7) == 0) lb = (lb & 7) * (G >> 3) + (lb >> 3);

  // A per-key mask that ends in "hard" masked keys (a padded batch: -10000 or -inf on the tail of
  // every sequence) leaves those keys with a weight of exactly zero, so the key tiles that hold
  // nothing else need not be visited -- the same saving as valid key counts, for callers who only
  // have the mask.  The workgroup looks at the mask rows of its (few) items once, in its prologue,
  // sharing the trip to memory with the first item's Q and K tiles: one wave per row loads the
  // whole row up front, a ballot per 64-key chunk gives the last key that is not hard-masked.  A
  // row without any such key keeps its full range (a fully masked row is a plain softmax over all
  // keys, reference fmha/fmha_manual.cpp:70).
  // "Hard" means a mask term of -9000 or below (-10000 is -9984 in bf16): such a key's weight is
  // exactly zero in fp32 unless its score exceeds every visible key's by more than 8800, a spread
  // at which a -10000 mask would not mask in the reference either.  kFwdFlagNoTrim turns it off.
  constexpr bool TRIM = MASK == kMaskPerKey;
  constexpr int kTrimSlots = 4, kTrimChunks = 16; // items per workgroup (one wave each), 64-key chunks per row
  static_assert(NW >= kTrimSlots, "one wave per item looks at its mask row");
  constexpr float kHardMask = -9000.f * FMHA_LOG2E;
  static_assert(kTrimSlots * 4 <= C::TRIM_BYTES, "key counts do not fit their LDS area");
  int *trim_kend = (int *)(lds + C::lds_bytes(NW) - C::TRIM_BYTES); // exchanged through the dynamic LDS block
  // The counts of the workgroup's items, by their order (item lb + n * G has ordinal n), as scalars:
  // with one wave per SIMD an LDS read or a division per item would be paid in full.  They start
  // at "no trimming" and are set by the workgroup prologue once the mask rows have been looked at.
  int trim_n[kTrimSlots];
#pragma unroll
  for (int i = 0; i < kTrimSlots; ++i) trim_n[i] = a.sk;
  // The mask rows are requested first of all (wave n: the row of the workgroup's n-th item, 64 keys
  // per instruction), so that the item set-up and the first copies below run in their shadow.
  const int ws = __builtin_amdgcn_readfirstlane(w);
  // Balanced mode (set up by the host when the shape allows it, see FwdArgs::bal_rows): every
  // workgroup looks at ALL mask rows (16 bytes per lane and instruction, wave n takes every NW-th
  // row or half row of 512 keys), so that all workgroups know every row's key count and can agree,
  // without talking to each other, on a dealing of the rows that evens out their work: a
  // workgroup's items come from one mask row per round; the first round keeps its row (its copies
  // start before the counts are known), the later rounds hand the remaining rows out by their
  // length, longest to the least loaded, in alternating order.
  const bool bal = TRIM && !CAUSAL && a.bal_rows > 0 && lb < nitems;
  const bool trim = TRIM && !bal && lb < nitems && lb + kTrimSlots * G >= nitems && a.sk > 2 * BK && // (two tiles are the least)
                    a.sk <= 64 * kTrimChunks && !(a.flags & kFwdFlagNoTrim); // workgroup-uniform
  constexpr int kBalSlots = 16; // (half) rows per wave
  static_assert(kBalSlots * NW * 4 <= C::TRIM_BYTES, "row counts do not fit their LDS area");
  u32x4 bal_mv[kBalSlots];
  const int bal_halves = a.sk > 512 ? 2 : 1; // 512-key pieces per row
  if (TRIM && bal) {
    auto bal_load = [&](int sidx) {
      const int gs = sidx * NW + ws; // which (row, half) this wave's slot covers
      int row = bal_halves == 2 ? gs >> 1 : gs;
      const int half = bal_halves == 2 ? gs & 1 : 0;
      row = row < a.bal_rows ? row : a.bal_rows - 1;
      int key0 = half * 512 + l * 8;
      key0 = key0 < a.sk ? key0 : 0;
      bal_mv[sidx] = *(const u32x4 *)((const T *)a.mask + (size_t)row * a.mask_sb + key0);
    };
#pragma unroll
    for (int i = 0; i < kBalSlots / 2; ++i) bal_load(i);
    if (a.bal_rows * bal_halves > kBalSlots / 2 * NW) {
#pragma unroll
      for (int i = kBalSlots / 2; i < kBalSlots; ++i) bal_load(i);
    }
  }
  int bal_row[kTrimSlots]; // balanced mode: the mask row (= group of bal_ipr items) of the n-th item
  int bal_h0 = 0, bal_qt0 = 0; // ... and the item's head and query tile within its row
#pragma unroll
  for (int i = 0; i < kTrimSlots; ++i) bal_row[i] = 0;
  T trim_mv[kTrimChunks];
#pragma unroll
  for (int c = 0; c < kTrimChunks; ++c) trim_mv[c] = (T)0.f;
  if (TRIM && trim && ws < kTrimSlots) {
    const int idx = lb + ws * G < nitems ? lb + ws * G : lb;
    const T *mk = (const T *)a.mask + (size_t)(idx / (a.nqt * a.mask_div)) * a.mask_sb; // (idx / nqt) / mask_div
#pragma unroll
    for (int c = 0; c < kTrimChunks / 2; ++c) {
      const int key = c * 64 + l;
      trim_mv[c] = mk[key < a.sk ? key : a.sk - 1];
    }
    if (a.sk > 64 * kTrimChunks / 2) {
#pragma unroll
      for (int c = kTrimChunks / 2; c < kTrimChunks; ++c) {
        const int key = c * 64 + l;
        trim_mv[c] = mk[key < a.sk ? key : a.sk - 1];
      }
    }
  }

  // Everything that depends on the item.  Keys: tiles [0, nkt), keys [0, kend); the tile count
  // is padded to even (nkt2) with an all-masked phantom tile so that the two x / P buffers and
  // the two LDS stages alternate with fixed roles across items as well.
  struct Item {
    int bh, rh, qt, nkt2, kend; // rh: the head q, k and v belong to (= bh unless the key range is cut into pieces)
    const T *Kb, *Vb, *mkey;
  };
  auto make_item = [&](int idx, int ord) {
    Item it;
    int mrow; // the item's mask row
    if (TRIM && bal) {
      // the dealing decides which row's item this is; its head and query tile within the row are the
      // workgroup's own (no division: with one wave per SIMD its latency would be paid in full)
      mrow = ord == 0 ? bal_row[0] : ord == 1 ? bal_row[1] : ord == 2 ? bal_row[2] : bal_row[3];
      it.bh = mrow * a.mask_div + bal_h0;
      it.qt = bal_qt0;
    } else {
      it.bh = idx / a.nqt;
      it.qt = idx - it.bh * a.nqt;
      mrow = MASK == kMaskPerKey ? it.bh / a.mask_div : 0;
    }
    // Causal items grow with the query tile.  A workgroup's items are G apart, which is often a
    // multiple of the tiles per head, so the order of the tiles is reversed in every other
    // round: long and short items then alternate within each workgroup.  (Within a round the
    // map stays one-to-one, so every item is still visited exactly once.)
    if (CAUSAL && ((idx / G) & 1) == 0) it.qt = a.nqt - 1 - it.qt;
    // keys this head may see at all: [0, sk) or its valid count (possibly 0: then every key is
    // treated as past the end, which yields O = 0 and LSE = -inf)
    int piece;
    real_head<STRIDED>(a, it.bh, it.rh, piece);
    const int sk = visible_keys<STRIDED>(a, it.rh, piece);
    int nkt = (sk + BK - 1) / BK;
    if (nkt < 1) nkt = 1;
    if (CAUSAL) {
      int qmax = it.qt * QT + QT - 1;
      if (qmax > a.sq - 1) qmax = a.sq - 1;
      const int need = qmax / BK + 1;
      if (need < nkt) nkt = need;
    }
    it.kend = nkt * BK < sk ? nkt * BK : sk;
    it.nkt2 = (nkt + 1) & ~1;
    const size_t poff = STRIDED ? (size_t)piece * (size_t)a.piece_stride : 0;
    it.Kb = (const T *)a.k + RW::head(a.mk, it.rh, a.sk) + poff;
    it.Vb = (const T *)a.v + RW::head(a.mv, it.rh, a.sk) + poff;
    it.mkey = (MASK == kMaskPerKey) ? (const T *)a.mask + (size_t)mrow * a.mask_sb : nullptr;
    return it;
  };
  // The mask's own trailing hard-masked keys shorten an item after the fact: with n >= 1 live keys
  // the range becomes [0, min(kend, n)) and the tile count follows from it (kend always lies in
  // the item's last tile).
  auto trim_count = [&](int ord) { return ord == 0 ? trim_n[0] : ord == 1 ? trim_n[1] : ord == 2 ? trim_n[2] : trim_n[3]; };
  auto trimmed = [&](Item it, int ord) {
    if (TRIM) {
      const int n = trim_count(ord);
      if (n < it.kend) {
        it.kend = n;
        it.nkt2 = ((n + BK - 1) / BK + 1) & ~1;
      }
    }
    return it;
  };
  if (TRIM && bal) { // until the dealing is known: every round keeps its own row
    const int grp = (int)(((float)lb + 0.5f) * a.bal_inv_ipr);
    const int r0 = lb - grp * a.bal_ipr; // the item's place within its row: head r0 / nqt, query tile r0 % nqt
    bal_h0 = r0 / a.nqt;
    bal_qt0 = r0 - bal_h0 * a.nqt;
#pragma unroll
    for (int i = 0; i < kTrimSlots; ++i) bal_row[i] = grp + i * a.bal_R;
  }
  Item cur = make_item(lb, 0);
  Item nxt = make_item(lb + G < nitems ? lb + G : lb, lb + G < nitems ? 1 : 0); // without a successor the streams harmlessly re-read the item
  int bh = cur.bh, q0w = cur.qt * QT + w * (QB * 32); // of the current item

  // ---- staging
  const uint32_t lds_base = lds_address(lds);
  const uint32_t wave_dst = (uint32_t)__builtin_amdgcn_readfirstlane(w) * 1024u;
  // Copy tile `tile` of `base` (K or V of a head) into stage (tile & 1) of the LDS area at byte
  // offset area_off.  Rows past kend re-read the last valid row: their scores get -inf through
  // the extra step, and finite garbage in V is multiplied by P = 0.
  TileCopy<T, D, BK, NT> tcopy;
  tcopy.init(tid, RW::ss(a.mk)); // K and V rows are equally far apart
  auto dma_tile = [&](const T *base, int kend, int tile, uint32_t area_off) {
    tcopy.issue(base, tile * BK, kend > 0 ? kend : 1, lds_base + area_off + (uint32_t)(tile & 1) * TILEB, tid, RW::cols(a));
  };
  // K tile u of the stream that runs from the current item on into the next one (u may reach
  // past the current item's last tile; nkt2 is even, so the stage parity carries over)
  auto dmaK = [&](int u) {
    const bool here = u < cur.nkt2;
    dma_tile(here ? cur.Kb : nxt.Kb, here ? cur.kend : nxt.kend, here ? u : u - cur.nkt2, 0u);
  };
  auto dmaV = [&](int tile) { dma_tile(cur.Vb, cur.kend, tile, 2u * TILEB); };

  // Q rows of an item: lane (ql, h) of wave w owns chunks [16*ks + 8*h, +8) of row q0 + 32*qb + ql.
  // Each wave copies its own rows into its own part of the Q buffer, exactly where its lanes
  // read them back, so the buffer needs no synchronisation beyond the wave's own wait.
  char *ldsQb = lds + C::LDS_BYTES;
  auto q_row = [&](const Item &it, int qb) {
    int q = it.qt * QT + w * (QB * 32) + qb * 32 + ql;
    q = q < a.sq ? q : a.sq - 1; // rows past the end repeat the last valid row and are never stored
    return (const T *)a.q + RW::head(a.mq, it.rh, a.sq) + (size_t)q * RW::ss(a.mq) + h * 8;
  };
  auto dmaQ = [&](const Item &it) {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      const T *row = q_row(it, qb);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) // (chunks past a narrower head's end come from the zero chunk)
        dma_global_to_lds_b128(ks * 16 + h * 8 < RW::cols(a) ? row + ks * 16 : (const T *)g_zero_chunk,
                               lds_base + C::LDS_BYTES + (uint32_t)((qb * KS + ks) * NT * 16) + wave_dst);
    }
  };

  // The extra-step rows (validity and per-key mask of each key) take the register path.
  struct XStage {
    T mraw;      // raw per-key mask element (converted when it is written to LDS, so that the
    bool mvalid; // conversion does not wait on the load)
  };
  XStage xs; // extra rows of the tile after next, in flight across iterations
  int nn_kend = cur.kend;      // key range and per-key mask of the item after next
  const T *nn_mkey = cur.mkey;
  auto set_after_next = [&](int idx, int ord) {
    const bool has = idx + 2 * G < nitems;
    const Item it = trimmed(make_item(has ? idx + 2 * G : idx, has ? ord + 2 : ord), has ? ord + 2 : ord);
    nn_kend = it.kend;
    nn_mkey = it.mkey;
  };
  // u: position in the tile stream, as for dmaK; it runs up to three tiles ahead, which can
  // reach the first tile of the item after next when the next item has only two tiles
  auto gloadX = [&](int u, XStage &st) {
    int tile = u, kend = cur.kend;
    const T *mk = cur.mkey;
    if (tile >= cur.nkt2) {
      tile -= cur.nkt2;
      kend = nxt.kend;
      mk = nxt.mkey;
      if (tile >= nxt.nkt2) {
        tile -= nxt.nkt2;
        kend = nn_kend;
        mk = nn_mkey;
      }
    }
    const int kr = tile * BK + (tid & (BK - 1));
    st.mvalid = kr < kend;
    st.mraw = (T)0.f;
    if (MASK == kMaskPerKey) st.mraw = mk[st.mvalid ? kr : (kend > 0 ? kend - 1 : 0)];
  };
  auto lstoreX = [&](int tile, const XStage &st) {
    if (tid < BK) {
      float mk = 0.f;
      if (MASK == kMaskPerKey) mk = fmaf((float)st.mraw, a.mask_a, a.mask_b);
      if (!st.mvalid) mk = NEG_INF;
      const T hi = (T)mk;
      const bool fin = (float)hi != NEG_INF;
      const T lo = fin ? (T)(mk - (float)hi) : (T)0.f;
      v8 x0, x1;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        x0[j] = (T)0.f;
        x1[j] = (T)0.f;
      }
      x0[0] = (T)1.f;
      x0[1] = hi;
      x0[2] = lo;
      x0[3] = (T)1.f;
      v8 *dst = (v8 *)(ldsXb + (tile & 1) * BK * XROWB + tid * XROWB);
      dst[0] = x0;
      dst[1] = x1;
    }
  };

  PanelLane pl;
  pl.init(l);
  auto readK = [&](const char *ldsK, int sb, int ks) -> v8 { return panel_read_rows<T, BK>(ldsK, pl, sb, ks); };
  auto readV = [&](const char *ldsV, int sb, int db, int c) -> v8 {
    return panel_read_transposed<T, BK>(ldsV, pl, sb, db, c);
  };

  // A full mask tensor takes the register path, one tile ahead: this lane's 32 mask values of the
  // next tile are requested right after the current tile's have been consumed, so the load has a
  // whole iteration to land (requested and consumed in the same iteration, it left the wave
  // waiting on memory in every tile: 135 instead of 85 us at the headline shape).
  // (At head dim 128 the registers for that are not there: the values are requested where they
  // are consumed, as they come.)
  constexpr bool MASK_AHEAD = MASK == kMaskFull && D == 64;
  const T *mrow[QB];     // this lane's rows of the mask tensor for the current item
  const T *mrow_nxt[QB]; // ... and for the next item, whose first tile is requested by the last iteration
  v4 mreg[QB][NSB][4];
  auto mask_rows = [&](const Item &it, const T *(&rows)[QB]) {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      int q = it.qt * QT + w * (QB * 32) + qb * 32 + ql;
      if (q > a.sq - 1) q = a.sq - 1;
      rows[qb] = (const T *)a.mask + (size_t)(it.bh / a.mask_div) * a.mask_sb + (size_t)q * a.mask_sq;
    }
  };
  auto mload = [&](const T *const (&mrow)[QB], int tile) {
    const int k0 = tile * BK;
    const bool vec_ok = a.mask_vec && (k0 + BK <= a.sk);
#pragma unroll
    for (int qb = 0; qb < QB; ++qb)
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int kk = k0 + sb * 32 + 8 * g + 4 * h;
          if (vec_ok) {
            mreg[qb][sb][g] = as_v4<T>(*(const u32x2 *)(mrow[qb] + kk));
          } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) mreg[qb][sb][g][i] = (kk + i < a.sk) ? mrow[qb][kk + i] : (T)0.f;
          }
        }
  };

  // A dropout tensor (the reference's train operators: 0/1 values in the element type, shaped like
  // the scores) takes the same register path, one tile BEHIND: tile t's values are requested in
  // iteration t and multiply P(t) at the top of iteration t+1, just before the second product
  // consumes it, so they too have a whole iteration to land and need one set of registers.
  const T *drow[QB];
  v4 dreg[QB][NSB][4];
  auto dload = [&](int tile) {
    const int k0 = tile * BK;
    const bool vec_ok = a.mask_vec && (k0 + BK <= a.sk);
#pragma unroll
    for (int qb = 0; qb < QB; ++qb)
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int kk = k0 + sb * 32 + 8 * g + 4 * h;
          if (vec_ok) {
            dreg[qb][sb][g] = as_v4<T>(*(const u32x2 *)(drow[qb] + kk));
          } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) dreg[qb][sb][g][i] = (kk + i < a.sk) ? drow[qb][kk + i] : (T)0.f;
          }
        }
  };
  auto apply_drop = [&](v8 (&p)[QB][NSB][2]) {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb)
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
          for (int t = 0; t < 4; ++t)
            p[qb][sb][g >> 1][4 * (g & 1) + t] =
                (T)((float)p[qb][sb][g >> 1][4 * (g & 1) + t] * (float)dreg[qb][sb][g][t]);
  };

  // ---- running state
  f32x16 o[QB][DB];
  float mref[QB], lsum[QB];
  bool seen[QB];
  v8 bx[QB];
  v8 qreg[QB][KS]; // Q' = Q * scale * log2(e) as B-operand registers

  // x buffers (accumulators of the first product) with the reference baked into each,
  // and the rounded probabilities of the previous / current tile
  f32x16 xA[QB][NSB], xB[QB][NSB];
  float bkA[QB], bkB[QB];
  // Row-sum limit that goes with each x buffer: the 2^14 window while the buffer's baked
  // reference is current, -1 (every sum fails) when the buffer was baked before a reference
  // existed or has been overtaken by a change of the reference.  lim_now is what a buffer baked
  // now would get.
  float limA[QB], limB[QB], lim_now[QB];
  v8 pA[QB][NSB][2], pB[QB][NSB][2];

  // first product of `tile` into x, baking the current reference
  auto g1 = [&](int tile, f32x16 (&x)[QB][NSB], float (&bk)[QB], float (&lim)[QB]) {
    const char *ldsK = ldsKb + (tile & 1) * TILEB;
    const char *ldsX = ldsXb + (tile & 1) * BK * XROWB;
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      bk[qb] = mref[qb];
      lim[qb] = lim_now[qb];
    }
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
      for (int qb = 0; qb < QB; ++qb)
#pragma unroll
        for (int r = 0; r < 16; ++r) x[qb][sb][r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb) {
        const v8 ka = readK(ldsK, sb, ks);
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) x[qb][sb] = E::mfma(ka, qreg[qb][ks], x[qb][sb]);
      }
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb) {
      const v8 xa = as_v8<T>(*(const u32x4 *)(ldsX + (sb * 32 + ql) * XROWB + h * 16));
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) x[qb][sb] = E::mfma(xa, bx[qb], x[qb][sb]);
    }
  };
  // second product of `tile`
  auto g2 = [&](int tile, const v8 (&p)[QB][NSB][2]) {
    const char *ldsV = ldsVb + (tile & 1) * TILEB;
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const v8 va = readV(ldsV, sb, db, c);
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) o[qb][db] = E::mfma(va, p[qb][sb][c], o[qb][db]);
        }
  };

  // One steady-state iteration's matrix work and softmax arithmetic as ONE hand-ordered
  // instruction stream: second product of tile tprev (probabilities p), first product of tile
  // tnext into x (skipped when LASTT), and P = exp2(xc) rounded into pc with its row sums rs.
  // MFMA and VALU work overlap only when they alternate inside one wave, and an LDS operand
  // must be requested a few MFMAs before its use, so the stream is built as groups of
  // {request operand j+kAhead, MFMAs of operand j, a slice of the exponentials} and every
  // group is closed by a scheduling barrier that nothing may cross.
  auto fused_step = [&](auto last_tag, int tprev, const v8 (&p)[QB][NSB][2], int tnext, f32x16 (&x)[QB][NSB],
                        float (&bk)[QB], float (&lim)[QB], const f32x16 (&xc)[QB][NSB], v8 (&pc)[QB][NSB][2],
                        float (&rs)[QB]) {
    constexpr bool LASTT = decltype(last_tag)::value;
    constexpr FwdOperandList ops = fwd_operand_list<NSB, KS, DB, !LASTT>();
    constexpr int kAhead = QB == 1 ? 3 : 2; // operands in flight; two query blocks leave fewer registers
    constexpr int NSL = QB * NSB * 8; // slices: two exponentials, one pack, one dot2 each
    const char *ldsV = ldsVb + (tprev & 1) * TILEB;
    const char *ldsK = ldsKb + (tnext & 1) * TILEB;
    const char *ldsX = ldsXb + (tnext & 1) * BK * XROWB;
    float rs2[QB]; // the row sum runs on two accumulators
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      bk[qb] = mref[qb];
      lim[qb] = lim_now[qb];
      rs[qb] = 0.f;
      rs2[qb] = 0.f;
    }
    auto fetch = [&](int j) -> v8 {
      if (ops.kind[j] == 0) return readV(ldsV, ops.a0[j], ops.a2[j], ops.a1[j]);
      if (ops.kind[j] == 1) return readK(ldsK, ops.a1[j], ops.a0[j]);
      return as_v8<T>(*(const u32x4 *)(ldsX + (ops.a1[j] * 32 + ql) * XROWB + h * 16));
    };
    auto slice = [&](int sidx) {
      const int qb = sidx / (NSB * 8), sb = (sidx / 8) % NSB, pr = sidx % 8;
      const float e0 = fast_exp2(xc[qb][sb][2 * pr]), e1 = fast_exp2(xc[qb][sb][2 * pr + 1]);
      const int c = pr / 4, j = pr % 4;
      pc[qb][sb][c][2 * j] = (T)e0;
      pc[qb][sb][c][2 * j + 1] = (T)e1;
      sum_pair<T>(pc[qb][sb][c], j, rs[qb], rs2[qb]); // (fp32 sums of the rounded pair, not a packed dot product)
    };
    v8 opnd[ops.n];
#pragma unroll
    for (int j = 0; j < kAhead && j < ops.n; ++j) opnd[j] = fetch(j);
    int done = 0;
#pragma unroll
    for (int j = 0; j < ops.n; ++j) {
      if (j + kAhead < ops.n) opnd[j + kAhead] = fetch(j + kAhead);
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        if (ops.kind[j] == 0) {
          o[qb][ops.a2[j]] = E::mfma(opnd[j], p[qb][ops.a0[j]][ops.a1[j]], o[qb][ops.a2[j]]);
        } else {
          f32x16 acc;
          if (ops.a0[j] == 0) {
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[r] = 0.f;
          } else {
            acc = x[qb][ops.a1[j]];
          }
          x[qb][ops.a1[j]] = E::mfma(opnd[j], ops.kind[j] == 1 ? qreg[qb][ops.a0[j]] : bx[qb], acc);
        }
      }
      const int upto = (j + 1) * NSL / ops.n;
#pragma unroll
      for (; done < upto; ++done) slice(done);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) rs[qb] += rs2[qb];
  };

  // per-element work that cannot go through the matrix pipe: a full mask tensor, the causal test
  auto adjust = [&](int tile, f32x16 (&x)[QB][NSB], auto guarded_tag) {
    constexpr bool GUARDED = decltype(guarded_tag)::value;
    if (MASK == kMaskFull || GUARDED) {
      const int k0 = tile * BK;
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        const int q = q0w + qb * 32 + ql;
#pragma unroll
        for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int kk = k0 + sb * 32 + 8 * g + 4 * h;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
              float xv = x[qb][sb][4 * g + t];
              if (MASK == kMaskFull) xv = fmaf((float)mreg[qb][sb][g][t], a.mask_a, xv);
              if (GUARDED) xv = (kk + t <= q) ? xv : NEG_INF;
              x[qb][sb][4 * g + t] = xv;
            }
          }
      }
    }
  };

  // P = exp2(x + shift) rounded to T, and the row sum of the rounded values
  auto exp_pack = [&](const f32x16 (&x)[NSB], float shift, v8 (&pk)[NSB][2]) -> float {
    float rs = 0.f, rs2 = 0.f;
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb) {
      float p[16];
#pragma unroll
      for (int r = 0; r < 16; ++r) p[r] = fast_exp2(x[sb][r] + shift);
#pragma unroll
      for (int c = 0; c < 2; ++c) {
#pragma unroll
        for (int j = 0; j < 8; ++j) pk[sb][c][j] = (T)p[8 * c + j];
#pragma unroll
        for (int j = 0; j < 4; ++j) sum_pair<T>(pk[sb][c], j, rs, rs2);
      }
    }
    return rs + rs2;
  };
  // move the reference of query block qb to this tile's maximum (x is relative to bk);
  // returns the shift that re-bases x onto the new reference
  auto rebase = [&](int qb, const f32x16 (&x)[NSB], float bk) -> float {
    float mx = NEG_INF;
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
      for (int r = 0; r < 16; r += 2) mx = max3(mx, x[sb][r], x[sb][r + 1]);
    mx = xhalf_max(mx);
    const float shift0 = bk - mref[qb]; // x + shift0 is relative to the current reference
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

  auto dropout = [&](int tile, int qb, v8 (&pk)[NSB][2]) {
    if (DROP == 1) {
      const int q = q0w + qb * 32 + ql;
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb) {
        uint32_t wd[4];
        drop_words_q(a.drop, (uint32_t)bh, (uint32_t)q, (uint32_t)(tile * BK + sb * 32), h, l, wd);
        const uint32_t thr2 = ((a.drop.thr - 1u) & 0xffffu) * 0x00010001u; // thr = 0 gives -1: everything kept
#pragma unroll
        for (int c = 0; c < 2; ++c) {
          Pack16 pp;
          if constexpr (std::is_same<T, _Float16>::value) pp.h = pk[sb][c];
          else pp.b = pk[sb][c];
          uint32_t r0 = pp.u.x, r1 = pp.u.y, r2 = pp.u.z, r3 = pp.u.w;
          drop_apply_pk4(wd[2 * c], thr2, r0, r1);
          drop_apply_pk4(wd[2 * c + 1], thr2, r2, r3);
          pp.u = u32x4{r0, r1, r2, r3};
          if constexpr (std::is_same<T, _Float16>::value) pk[sb][c] = pp.h;
          else pk[sb][c] = pp.b;
        }
      }
    }
  };

  // One iteration.  FIRST: tile t is the first tile (no previous second product; the
  // reference is set from this tile before the next first product bakes it).
  // LAST: there is no next tile.
  // K(t+2) and V(t) are requested at the top and awaited by tile_sync() after the body; past
  // the item's last tile, "K(t+2)" is one of the first two tiles of the next item.
  // The extra rows of tile t+2 are written first, from the registers `xs` that the previous
  // iteration loaded (so the load has certainly landed: tile_sync() waited for it), and `xs`
  // is refilled for tile t+3 -- all before the copies are issued, because the compiler's own
  // wait for a load it knows about also waits for every copy issued ahead of it.
  auto body = [&](int t, auto first_tag, auto last_tag, auto guarded_tag, f32x16 (&xc)[QB][NSB], float (&bkc)[QB],
                  float (&limc)[QB], f32x16 (&xn)[QB][NSB], float (&bkn)[QB], float (&limn)[QB],
                  v8 (&pprev)[QB][NSB][2], v8 (&pcur)[QB][NSB][2]) {
    constexpr bool FIRST = decltype(first_tag)::value;
    constexpr bool LAST = decltype(last_tag)::value;
    lstoreX(t + 2, xs);
    gloadX(t + 3, xs);
    if (MASK_AHEAD) {
      // consume this tile's mask values and request the next tile's before the copies go out: the
      // compiler's wait for these loads, in the next iteration, then finds nothing younger in flight
      adjust(t, xc, guarded_tag);
      if (t + 1 < cur.nkt2) mload(mrow, t + 1);
      else mload(mrow_nxt, 0); // without a successor: this item's rows again, harmlessly
    }
    if (DROP == 2) {
      if (!FIRST) apply_drop(pprev); // with tile t-1's values, requested one iteration ago
      dload(t);
    }
    dmaK(t + 2);
    dmaV(t);
    if (!MASK_AHEAD) {
      if (MASK == kMaskFull) mload(mrow, t);
      adjust(t, xc, guarded_tag);
    }
    if (FIRST) {
      float shift[QB];
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) shift[qb] = rebase(qb, xc[qb], bkc[qb]);
      if (!LAST) g1(t + 1, xn, bkn, limn);
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        lsum[qb] += exp_pack(xc[qb], shift[qb], pcur[qb]);
        dropout(t, qb, pcur[qb]);
      }
    } else {
      float rs[QB];
      fused_step(last_tag, t - 1, pprev, t + 1, xn, bkn, limn, xc, pcur, rs);
      bool unfit = false;
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) unfit = unfit | !(rs[qb] < limc[qb]); // no short circuit: keep one basic block
      if (__builtin_amdgcn_ballot_w64(unfit) != 0ull) {
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
          const float shift = rebase(qb, xc[qb], bkc[qb]);
          rs[qb] = exp_pack(xc[qb], shift, pcur[qb]);
          if (bkn[qb] != mref[qb]) limn[qb] = -1.f; // the next buffer was baked with the old reference
        }
      }
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        lsum[qb] += rs[qb];
        dropout(t, qb, pcur[qb]);
      }
    }
  };
  auto tile_sync = [&]() {
    dma_wait_all();
    __syncthreads();
  };

  using Yes = std::true_type;
  using No = std::false_type;
  // A tile crosses the causal diagonal of this wave iff its last key exceeds the wave's first query.
  auto diag = [&](int t) { return CAUSAL && (t * BK + BK - 1 > q0w); };

  // ---- workgroup prologue: the first item's Q, K(0), K(1) and extra rows
  if (C::QLDS) dmaQ(cur);
  dmaK(0);
  dmaK(1);
  {
    XStage x0, x1;
    gloadX(0, x0);
    gloadX(1, x1);
    // The third tile of the stream is the first item's tile 2 or, if trimming leaves it only two
    // tiles, the next item's tile 0: both candidates are requested now, so that the choice does
    // not cost a second trip to memory.
    T xs_here = (T)0.f, xs_next = (T)0.f;
    set_after_next(lb, 0);
    if (TRIM) {
      const int last = a.sk > 0 ? a.sk - 1 : 0;
      const int ka = 2 * BK + (tid & (BK - 1)), kb = tid & (BK - 1);
      xs_here = cur.mkey[ka < last ? ka : last];
      xs_next = nxt.mkey[kb < last ? kb : last];
    } else {
      gloadX(2, xs);
    }
    // Up to here the items had their untrimmed key ranges: the tiles just requested hold real
    // rows where a trimmed range would repeat its last row, which makes no difference to keys
    // that are marked as past the end below.
    if (TRIM && bal) {
      // ---- every row's count: a lane's eight keys are all hard-masked iff the smallest of their bit
      // patterns, read as unsigned, is not below that of the threshold (negative numbers grow with
      // their magnitude; anything non-negative is smaller)
      const unsigned hard = __builtin_bit_cast(unsigned short, (T)(-9000.f));
      int *part = trim_kend; // [kBalSlots * NW] keys up to the last live one, per (half) row
      auto bal_count = [&](int sidx) {
        const int gs = sidx * NW + ws;
        const int half = bal_halves == 2 ? gs & 1 : 0;
        const u32x4 r = bal_mv[sidx];
        unsigned lo = 0xffffu;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const unsigned e0 = r[j] & 0xffffu, e1 = r[j] >> 16;
          lo = e0 < lo ? e0 : lo;
          lo = e1 < lo ? e1 : lo;
        }
        const bool live = half * 512 + l * 8 < a.sk && lo < hard;
        const unsigned long long bl = __builtin_amdgcn_ballot_w64(live);
        const int n = bl ? half * 512 + (64 - __builtin_clzll(bl)) * 8 : 0; // rounded up to the lane's 8 keys
        if (l == 0) part[gs] = n;
      };
#pragma unroll
      for (int i = 0; i < kBalSlots / 2; ++i) bal_count(i);
      if (a.bal_rows * bal_halves > kBalSlots / 2 * NW) {
#pragma unroll
        for (int i = kBalSlots / 2; i < kBalSlots; ++i) bal_count(i);
      }
      __syncthreads();
      // ---- lane i: row i.  (Every wave does the same arithmetic and arrives at the same scalars.)
      const bool row_ok = l < a.bal_rows;
      int len = 0;
      if (row_ok) {
        len = bal_halves == 2 ? (part[2 * l + 1] ? part[2 * l + 1] : part[2 * l]) : part[l];
        len = len == 0 || len > a.sk ? a.sk : len; // no live key: a plain softmax over all keys
      }
      const int cls = (len + 2 * BK - 1) / (2 * BK); // work of an item: its tile pairs (1 .. 8)
      const int R = a.bal_R;
      const int grp = bal_row[0];
      // position of each lane's row among the first round's rows (l < R) / the other rows, longest first
      const unsigned long long below = l ? ~0ull >> (64 - l) : 0ull;
      int pos = 0, above_first = 0, above_rest = 0;
      for (int c = (a.sk + 2 * BK - 1) / (2 * BK); c >= 1; --c) { // the classes this key range can have
        const unsigned long long bf = __builtin_amdgcn_ballot_w64(row_ok && l < R && cls == c);
        const unsigned long long br = __builtin_amdgcn_ballot_w64(row_ok && l >= R && cls == c);
        if (cls == c) pos = l < R ? above_first + __builtin_popcountll(bf & below) : above_rest + __builtin_popcountll(br & below);
        above_first += __builtin_popcountll(bf);
        above_rest += __builtin_popcountll(br);
      }
      const int my_rank = __builtin_amdgcn_readlane(pos, grp); // 0: the longest first-round row
      trim_n[0] = __builtin_amdgcn_readlane(len, grp);
      const int rounds = a.bal_rows / R;
#pragma unroll
      for (int n = 1; n < kTrimSlots; ++n) {
        // round n hands every (rounds-1)-th row of the sorted rest to the groups (so that each round
        // spans all lengths), the longest to the group with the shortest first-round row in odd
        // rounds, the other way round in even ones
        const int want = ((n & 1) ? R - 1 - my_rank : my_rank) * (rounds - 1) + (n - 1);
        const unsigned long long hit = __builtin_amdgcn_ballot_w64(row_ok && l >= R && pos == want);
        const int row = n < rounds && hit ? __builtin_ctzll(hit) : grp;
        bal_row[n] = row;
        trim_n[n] = __builtin_amdgcn_readlane(len, row);
      }
      __syncthreads(); // the counts' LDS area is not written again, but keep the waves together as the other path does
      cur = trimmed(cur, 0);
      nxt = trimmed(make_item(0, lb + G < nitems ? 1 : 0), lb + G < nitems ? 1 : 0);
      x0.mvalid = (tid & (BK - 1)) < cur.kend;
      x1.mvalid = BK + (tid & (BK - 1)) < cur.kend;
      const bool here = 2 < cur.nkt2;
      xs.mraw = xs_here;
      xs.mvalid = 2 * BK + (tid & (BK - 1)) < cur.kend;
      if (!here) { // (rare: at most two tiles) the stream's third tile is the next item's first, known only now
        const int kr = tid & (BK - 1);
        xs.mvalid = kr < nxt.kend;
        xs.mraw = nxt.mkey[xs.mvalid ? kr : (nxt.kend > 0 ? nxt.kend - 1 : 0)];
      }
      set_after_next(lb, 0);
    } else if (TRIM) {
      if (trim) {
        if (ws < kTrimSlots) {
          int last = -1;
          auto chunk = [&](int c) {
            const int key = c * 64 + l;
            const bool live = key < a.sk && fmaf((float)trim_mv[c], a.mask_a, a.mask_b) > kHardMask;
            const unsigned long long bal = __builtin_amdgcn_ballot_w64(live);
            if (bal) last = c * 64 + 63 - __builtin_clzll(bal); // chunks ascend: the last hit wins
          };
#pragma unroll
          for (int c = 0; c < kTrimChunks / 2; ++c) chunk(c);
          if (a.sk > 64 * kTrimChunks / 2) {
#pragma unroll
            for (int c = kTrimChunks / 2; c < kTrimChunks; ++c) chunk(c);
          }
          if (l == 0) trim_kend[ws] = last < 0 ? a.sk : last + 1;
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < kTrimSlots; ++i) trim_n[i] = __builtin_amdgcn_readfirstlane(trim_kend[i]);
        cur = trimmed(cur, 0);
        nxt = trimmed(nxt, lb + G < nitems ? 1 : 0);
        const int nn = trim_count(lb + 2 * G < nitems ? 2 : 0);
        nn_kend = nn < nn_kend ? nn : nn_kend;
        x0.mvalid = (tid & (BK - 1)) < cur.kend;
        x1.mvalid = BK + (tid & (BK - 1)) < cur.kend;
      }
      const bool here = 2 < cur.nkt2;
      xs.mraw = here ? xs_here : xs_next;
      xs.mvalid = here ? 2 * BK + (tid & (BK - 1)) < cur.kend : (tid & (BK - 1)) < nxt.kend;
    }
    lstoreX(0, x0);
    lstoreX(1, x1);
  }

  for (int idx = lb, ord = 0;;) {
    const int nidx = idx + G;
    const bool more = nidx < nitems;
    nxt = trimmed(make_item(more ? nidx : idx, more ? ord + 1 : ord), more ? ord + 1 : ord);
    set_after_next(idx, ord);
    bh = cur.bh;
    q0w = cur.qt * QT + w * (QB * 32);
    if (DROP == 2) {
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        int q = q0w + qb * 32 + ql;
        if (q > a.sq - 1) q = a.sq - 1;
        drow[qb] = (const T *)a.drop_mask + ((size_t)bh * a.sq + q) * a.sk;
      }
    }
    if (MASK == kMaskFull) {
      mask_rows(cur, mrow);
      if (MASK_AHEAD) {
        mask_rows(nxt, mrow_nxt);
        if (idx == lb) mload(mrow, 0); // later items: requested by the previous item's last iteration
      }
    }

    // ---- item prologue: Q' registers, state, first product of tile 0
    // Only the first item has copies in flight here (Q, K(0), K(1)) and extra rows that other
    // waves have not seen yet.  For later items all of that was awaited inside the previous
    // item, and waiting again would only stall on the output stores just issued.
    if (idx == lb) tile_sync();
    if (C::QLDS) {
#pragma unroll
      for (int qb = 0; qb < QB; ++qb)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const v8 raw = as_v8<T>(*(const u32x4 *)(ldsQb + ((qb * KS + ks) * NT + tid) * 16));
#pragma unroll
          for (int j = 0; j < 8; ++j) qreg[qb][ks][j] = (T)((float)raw[j] * a.scale_l2);
        }
    } else {
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        const T *row = q_row(cur, qb);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const bool live = ks * 16 + h * 8 < RW::cols(a);
          const v8 raw = as_v8<T>(chunk_or_zero(*(const u32x4 *)(live ? row + ks * 16 : row), live));
#pragma unroll
          for (int j = 0; j < 8; ++j) qreg[qb][ks][j] = (T)((float)raw[j] * a.scale_l2);
        }
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
        if (MASK == kMaskFull) bx[qb][3] = (T)a.mask_b;
      }
    }
    g1(0, xA, bkA, limA);
    __syncthreads(); // tile 0's K stage is refilled during the first iteration
    // The next item's Q rows are requested here rather than earlier so that the wait they end
    // up in is the one at the end of the first iteration.  The Q buffer has been read (the
    // first product used the registers made from it).
    if (C::QLDS && more) dmaQ(nxt);

    const int nkt2 = cur.nkt2;
    // t = 0
    if (diag(0)) body(0, Yes{}, No{}, Yes{}, xA, bkA, limA, xB, bkB, limB, pB, pA);
    else body(0, Yes{}, No{}, No{}, xA, bkA, limA, xB, bkB, limB, pB, pA);
    tile_sync();
    // steady state, two tiles per trip so that the buffers keep fixed roles
    for (int t = 1; t < nkt2 - 1; t += 2) {
      if (diag(t)) body(t, No{}, No{}, Yes{}, xB, bkB, limB, xA, bkA, limA, pA, pB);
      else body(t, No{}, No{}, No{}, xB, bkB, limB, xA, bkA, limA, pA, pB);
      tile_sync();
      if (diag(t + 1)) body(t + 1, No{}, No{}, Yes{}, xA, bkA, limA, xB, bkB, limB, pB, pA);
      else body(t + 1, No{}, No{}, No{}, xA, bkA, limA, xB, bkB, limB, pB, pA);
      tile_sync();
    }
    // last tile (odd index) and the second product that is still owed
    {
      const int t = nkt2 - 1;
      if (diag(t)) body(t, No{}, Yes{}, Yes{}, xB, bkB, limB, xA, bkA, limA, pA, pB);
      else body(t, No{}, Yes{}, No{}, xB, bkB, limB, xA, bkA, limA, pA, pB);
      tile_sync();
      if (DROP == 2) apply_drop(pB);
      g2(t, pB);
    }

    // ---- item epilogue
    T *Ob = (T *)a.o + RW::head(a.mo, bh, a.sq);
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      const int q = q0w + qb * 32 + ql;
      const float lt = xhalf_sum(lsum[qb]);
      const float inv = lt > 0.f ? a.drop_scale / lt : 0.f;
      if (q < a.sq) {
#pragma unroll
        for (int db = 0; db < DB; ++db) store_acc_block_row<T>(Ob + (size_t)q * RW::ss(a.mo) + db * 32, o[qb][db], inv, h, RW::cols(a) - db * 32);
        const float cfix = (MASK == kMaskFull) ? a.mask_b - (float)(T)a.mask_b : 0.f;
        if (a.lse && h == 0)
          a.lse[(size_t)bh * a.sq + q] = lt > 0.f ? (mref[qb] + cfix + fast_log2(lt)) * FMHA_LN2 : NEG_INF;
      }
    }
    if (!more) break;
    idx = nidx;
    ++ord;
    cur = nxt;
  }
  if (probe) {
    a.clock_probe[2] = __builtin_readcyclecounter();
    a.clock_probe[3] = __builtin_amdgcn_s_memrealtime();
  }
}

} // namespace fmha
