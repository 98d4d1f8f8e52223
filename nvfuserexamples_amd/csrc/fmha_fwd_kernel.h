// Forward attention kernel for gfx950 (wave64, MFMA 32x32x16).
//
// Takes the place of the three nvFuser-scheduled kernels of the reference
// (fmha/fmha_manual.cpp:20-409, :411-807, :809-1214).  Where the reference keeps a
// whole key row of 128 in one CTA (fmha_manual.cpp:107-111) and moves the score
// tile through shared memory twice (:160,165,274,322), this kernel walks the keys
// in LDS tiles of 64 with an online softmax and keeps scores and probabilities in
// registers from the first product to the second.
//
// Work decomposition
//   workgroup = NW waves, one (bh, query tile of NW*QB*32 rows); wave = QB blocks of
//   32 queries.  K and V tiles of 64 keys are staged in LDS (double buffered, padded
//   rows); Q lives in registers as the B operand for the whole kernel.
// Products are computed transposed so that every lane owns one query column:
//   X^T[key][q] = K . Q'^T      A = K rows from LDS (ds_read_b128), B = Q' registers
//   O^T[d][q]   = V^T . P^T     A = V^T via the LDS transpose read, B = P registers
// The accumulator layout of X^T (lane = query, registers = keys) is exactly the B
// operand layout of the second product under a fixed permutation of the key index,
// and V is fetched with that same permutation, so P never leaves registers.
//
// The softmax is VALU-bound at head dim 64 (one v_exp per score against ~16 MFMA
// flops per score), so everything except the exponential and the rounding is pushed
// into the matrix pipe:
//   * Q' = Q * scale * log2(e), rounded once to the element type, so the product is
//     already in log2 units;
//   * the product gets one extra contraction step whose A rows are
//     (1, mask_hi[key], mask_lo[key], 1, 0, ...) and whose B columns are
//     (-m[q], 1, 1, c, 0, ...): the accumulator comes out as
//         x = score + mask[key] - m[q]
//     i.e. the per-key additive mask (split hi+lo so it keeps 2x the element type's
//     precision; -inf for keys past the end) and the per-query reference exponent m are
//     applied by the MFMA, and P = exp2(x) needs no further arithmetic;
//   * m is kept representable in the element type so the subtraction is exact, and it
//     is NOT the running maximum: it is only raised when a tile's probabilities would
//     leave a 2^14 window (detected from the tile's row sum, which is needed anyway),
//     so the common tile computes no maximum and rescales nothing;
//   * the row sum is taken over the ROUNDED probabilities with v_dot2 on the packed
//     pairs, so the denominator matches what the second product sums.
// The two half-wave partial sums are combined once in the epilogue.
#pragma once
#include <type_traits>

#include "fmha_common.h"

namespace fmha {

struct FwdArgs {
  const void *q, *k, *v;
  void *o;
  float *lse;
  const void *mask;
  const void *drop_mask;
  void *save_softmax, *save_dropout;
  int64_t mask_sb, mask_sq;
  int32_t mask_div;
  int32_t mask_vec;  // 1: 8-byte accesses to [.., sk] rows (mask, drop mask, saves) are aligned
  float mask_a, mask_b; // mask term in log2 units = mask_value * mask_a + mask_b
  int32_t bh, sq, sk;
  int32_t nqt;       // query tiles per head
  float scale_l2;    // scale * log2(e)
  float inv_scale_l2; // 1 / scale_l2
  float drop_scale;
  DropCtx drop;
  int32_t flags;
  const int32_t *kv_len; // optional valid key count per group of kv_div heads (not with tensor dropout / saved outputs)
  int32_t kv_div;
  // A key range cut into pieces that run as heads of their own (run-time layouts only; pieces <= 1: off).
  // Head index = real head * pieces + piece; q, k, v (and kv_len) belong to the real head, piece c starts
  // piece_stride * c elements into the real head's k and v rows and covers sk of the sk_whole keys; o, lse
  // and the mask are indexed by the head index as always.
  int32_t pieces;
  uint32_t pieces_rcp;   // floor(2^32 / pieces) + 1
  int32_t sk_whole;
  int64_t piece_stride;
  unsigned long long *clock_probe; // optional: counters at the start and end of workgroup 0 (pipelined kernel only)
  RowMap mq, mk, mv, mo; // row layout of q, k, v, o (mk.ss == mv.ss)
  int32_t dcols;         // elements per row that exist (<= the kernel's head dim; run-time layouts only)
  // Balanced dealing of a per-key mask's rows over the persistent workgroups (pipelined kernel; set
  // by its launch code, 0 rows = off).  It applies when every workgroup has the same number of items
  // (2 to 4), one per round, and a round's items of one mask row (bal_ipr = heads per row x query
  // tiles) fill whole groups of bal_ipr workgroups: round n of workgroup g * bal_ipr + r is item r of
  // row g + n * bal_R.  Then the rows can be dealt to the groups by length without breaking that shape.
  int32_t bal_rows;   // mask rows (= bh / mask_div)
  int32_t bal_ipr;    // items per mask row
  int32_t bal_R;      // rows per round = grid size / bal_ipr
  float bal_inv_ipr;  // 1 / bal_ipr
};

// FwdArgs::flags
enum { kFwdFlagNoTrim = 1 }; // visit every key tile even where a per-key mask hard-masks the tail

// how the mask tensor is read
enum { kMaskNone = 0, kMaskPerKey = 1, kMaskFull = 2 };

// Head index -> (real head, first key of its piece); see FwdArgs::pieces.
template <bool STRIDED> FMHA_DEV void real_head(const FwdArgs &a, int bh, int &head, int &piece) {
  head = bh;
  piece = 0;
  if constexpr (STRIDED) {
    if (a.pieces > 1) {
      head = (int)__umulhi((uint32_t)bh, a.pieces_rcp);
      piece = bh - head * a.pieces;
    }
  }
}
// Keys a head may see at all: all sk, or the real head's valid count (possibly 0); of a piece: what is left
// of either in it.
template <bool STRIDED> FMHA_DEV int visible_keys(const FwdArgs &a, int head, int piece) {
  int n = a.sk;
  if constexpr (STRIDED) {
    if (a.pieces > 1) n = a.sk_whole;
  }
  if (a.kv_len) {
    const int m = a.kv_len[head / a.kv_div];
    n = m < 0 ? 0 : (m < n ? m : n);
  }
  n -= piece * a.sk;
  return n < 0 ? 0 : (n < a.sk ? n : a.sk);
}

template <int D> struct FwdCfg {
  static constexpr int BK = 64;           // keys per LDS tile
  static constexpr int NSB = BK / 32;     // 32-key sub-blocks per tile
  static constexpr int KS = D / 16;       // contraction steps of K.Q^T
  static constexpr int DB = D / 32;       // 32-row blocks of O^T
  // LDS row pitches in bytes.  K rows are read 16 bytes per lane, a row per lane: a pad of 16 bytes puts sixteen
  // consecutive rows on the sixteen 16-byte bank groups.  V rows are read by the transpose read, 8 bytes per lane,
  // four lanes per row and four rows per sixteen lanes: a pad of 32 bytes sets consecutive rows 32 bytes apart in
  // the banks, so the sixteen lanes cover 128 contiguous bytes (with the 16-byte pad rows overlapped pairwise and
  // every such read took two passes).
  static constexpr int ROWB = D * 2 + 16;
  static constexpr int ROWBV = D * 2 + 32;
  static constexpr int TILEB = BK * ROWBV; // (one size for both tiles)
  static constexpr int XROWB = 32;        // pitch of the extra-contraction-step rows (16 elements)
  static constexpr int LDS_BYTES = 4 * TILEB + 2 * BK * XROWB; // {K,V} x 2 stages + extra rows x 2 stages
};

template <typename T> FMHA_DEV float dot2_ones(typename Elem<T>::v8 v, int pair, float acc);
template <> FMHA_DEV float dot2_ones<_Float16>(f16x8 v, int pair, float acc) {
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  const h2 one = {(_Float16)1.f, (_Float16)1.f};
  const h2 x = {v[2 * pair], v[2 * pair + 1]};
  return __builtin_amdgcn_fdot2(x, one, acc, false);
}
template <> FMHA_DEV float dot2_ones<__bf16>(bf16x8 v, int pair, float acc) {
  typedef __bf16 b2 __attribute__((ext_vector_type(2)));
  const b2 one = {(__bf16)1.f, (__bf16)1.f};
  const b2 x = {v[2 * pair], v[2 * pair + 1]};
  return __builtin_amdgcn_fdot2_f32_bf16(x, one, acc, false);
}

// lo += v[2 pair], hi += v[2 pair + 1] in fp32: the row sums of the ROUNDED probabilities, so that the denominator
// matches what the second product sums (a row with one visible key reproduces that key's value exactly).  Not the
// packed dot product that would do both in one instruction: next to matrix instructions v_dot2c costs about twenty
// cycles apiece on this chip (measured: one matrix instruction + 2 / 4 / 6 v_dot2c_f32_f16 55 / 63 / 71 cycles;
// + 2 / 4 / 6 v_fma_mix_f32 35 / 36 / 40; + 2 / 4 / 6 v_add_f32 34 / 35 / 37), while these disappear in the matrix
// instruction's shadow.
template <typename T> FMHA_DEV void sum_pair(typename Elem<T>::v8 v, int pair, float &lo, float &hi);
template <> FMHA_DEV void sum_pair<_Float16>(f16x8 v, int pair, float &lo, float &hi) {
  const uint32_t u = as_u32x4(v)[pair];
  asm("v_fma_mix_f32 %0, %1, 1.0, %0 op_sel_hi:[1,0,0]" : "+v"(lo) : "v"(u));
  asm("v_fma_mix_f32 %0, %1, 1.0, %0 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "+v"(hi) : "v"(u));
}
template <> FMHA_DEV void sum_pair<__bf16>(bf16x8 v, int pair, float &lo, float &hi) {
  const uint32_t u = as_u32x4(v)[pair];
  lo += __uint_as_float(u << 16);
  hi += __uint_as_float(u & 0xffff0000u);
}

template <typename T, int D, int QB, int NW, int MASK, bool CAUSAL, int DROP, bool STRIDED = false>
__global__ __launch_bounds__(NW * 64) void fmha_fwd_kernel(const FwdArgs a) {
  using RW = Rows<STRIDED, D>; // (run-time row layouts are built at head dim 256 only, where this is the only forward)
  using E = Elem<T>;
  using v8 = typename E::v8;
  using v4 = typename E::v4;
  using C = FwdCfg<D>;
  constexpr int BK = C::BK, NSB = C::NSB, KS = C::KS, DB = C::DB, ROWB = C::ROWB, ROWBV = C::ROWBV, XROWB = C::XROWB;
  constexpr int TILEB = C::TILEB;
  constexpr int NT = NW * 64;
  constexpr int QT = NW * QB * 32;
  constexpr int CPR = D / 8;                 // 16-byte chunks per row
  constexpr int CPT = BK * CPR / NT;         // chunks per thread per tile
  static_assert(BK * CPR % NT == 0, "tile must divide evenly over the workgroup");
  static_assert(NT >= BK, "the extra rows are staged by the first BK threads");
  constexpr float NEG_INF = -__builtin_inff();
  constexpr float WINDOW = 16384.f; // a tile whose rounded row sum reaches 2^14 raises the reference

  extern __shared__ __attribute__((aligned(16))) char lds[];
  char *ldsX = lds + 4 * TILEB;

  const int tid = threadIdx.x;
  const int w = tid >> 6;
  const int l = tid & 63;
  const int ql = l & 31;
  const int h = l >> 5;

  // Workgroups are dealt round-robin to the 8 XCDs; remap so that one XCD (one L2)
  // owns a contiguous range of (head, query tile) pairs and the query tiles of a head
  // re-read that head's K/V from the same L2.
  int bid = blockIdx.x;
  const int nb = gridDim.x;
  if ((nb & 7) == 0) bid = (bid & 7) * (nb >> 3) + (bid >> 3);
  const int bh = bid / a.nqt;
  int qt = bid - bh * a.nqt;
  if (CAUSAL) qt = a.nqt - 1 - qt; // longest rows first
  const int q0w = qt * QT + w * (QB * 32);

  int rh, piece;
  real_head<STRIDED>(a, bh, rh, piece);
  const T *Qb = (const T *)a.q + RW::head(a.mq, rh, a.sq);
  const T *Kb = (const T *)a.k + RW::head(a.mk, rh, a.sk) + (STRIDED ? (size_t)piece * (size_t)a.piece_stride : 0);
  const T *Vb = (const T *)a.v + RW::head(a.mv, rh, a.sk) + (STRIDED ? (size_t)piece * (size_t)a.piece_stride : 0);
  const T *mkey = (MASK == kMaskPerKey) ? (const T *)a.mask + (size_t)(bh / a.mask_div) * a.mask_sb : nullptr;

  // ---- Q' = Q * scale * log2(e) as B-operand registers
  v8 qreg[QB][KS];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int q = q0w + qb * 32 + ql;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      // rows past the end re-read the last row (never stored); unconditional loads do not stall on each other
      const int qc = q < a.sq ? q : a.sq - 1;
      const bool live = ks * 16 + h * 8 < RW::cols(a);
      const u32x4 t = *(const u32x4 *)(Qb + (size_t)qc * RW::ss(a.mq) + (live ? ks * 16 + h * 8 : 0));
      const v8 raw = as_v8<T>(chunk_or_zero(t, live));
#pragma unroll
      for (int j = 0; j < 8; ++j) qreg[qb][ks][j] = (T)((float)raw[j] * a.scale_l2);
    }
  }

  // ---- key range: all sk keys, or the head's valid count (keys at or past it get a -inf mask term, whole
  // tiles past it are not visited; a count of 0 visits one tile that is masked throughout: O = 0, LSE = -inf)
  const int skv = visible_keys<STRIDED>(a, rh, piece);
  int nkt = (skv + BK - 1) / BK;
  if (nkt < 1) nkt = 1;
  if (CAUSAL) {
    int qmax = qt * QT + QT - 1;
    if (qmax > a.sq - 1) qmax = a.sq - 1;
    int need = qmax / BK + 1;
    if (need < nkt) nkt = need;
  }

  // rows of K and V that exist from Kb / Vb on: all sk, or what the whole key range leaves for this piece (>= 1)
  int krows = a.sk;
  if constexpr (STRIDED) {
    if (a.pieces > 1 && a.sk_whole - piece * a.sk < krows) krows = a.sk_whole - piece * a.sk;
  }

  // ---- tile staging: global -> registers -> LDS
  u32x4 kst[CPT], vst[CPT];
  T mraw = (T)0.f;     // raw per-key mask element in flight (converted when it is written to LDS,
  bool mvalid = false; // so that the conversion does not wait on the loads issued with it)
  auto gload = [&](int k0) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = tid + i * NT;
      const int row = c / CPR, col = c % CPR;
      // keys past the end re-read the last row: their scores get -inf through the extra step, so P = 0
      // meets finite values of V (unconditional loads do not stall on each other)
      int kr = k0 + row;
      kr = kr < krows ? kr : krows - 1;
      const int cc = col * 8 < RW::cols(a) ? col * 8 : 0; // padding chunks: zeroed when they are written to LDS
      kst[i] = *(const u32x4 *)(Kb + (size_t)kr * RW::ss(a.mk) + cc);
      vst[i] = *(const u32x4 *)(Vb + (size_t)kr * RW::ss(a.mv) + cc);
    }
    {
      const int kr = k0 + (tid & (BK - 1));
      mvalid = kr < skv;
      if (MASK == kMaskPerKey) mraw = mkey[kr < a.sk ? kr : a.sk - 1];
    }
  };
  auto lstore = [&](int stage) {
    char *kd = lds + stage * 2 * TILEB;
    char *vd = kd + TILEB;
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = tid + i * NT;
      const int row = c / CPR, col = c % CPR;
      const bool live = col * 8 < RW::cols(a);
      *(u32x4 *)(kd + row * ROWB + col * 16) = chunk_or_zero(kst[i], live);
      *(u32x4 *)(vd + row * ROWBV + col * 16) = chunk_or_zero(vst[i], live);
    }
    if (tid < BK) {
      // extra contraction step, A side: (1, mask_hi, mask_lo, 1, 0 ...); keys past the end get
      // mask = -inf, which is all the ragged last tile needs
      float mk = 0.f;
      if (MASK == kMaskPerKey) mk = fmaf((float)mraw, a.mask_a, a.mask_b);
      if (!mvalid) mk = NEG_INF;
      const T hi = (T)mk;
      const T lo = mvalid ? (T)(mk - (float)hi) : (T)0.f;
      v8 x0, x1;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        x0[j] = (T)0.f;
        x1[j] = (T)0.f;
      }
      x0[0] = (T)1.f;
      x0[1] = hi;
      x0[2] = (hi == hi && (float)hi != NEG_INF) ? lo : (T)0.f;
      x0[3] = (T)1.f;
      v8 *dst = (v8 *)(ldsX + stage * BK * XROWB + tid * XROWB);
      dst[0] = x0;
      dst[1] = x1;
    }
  };

  // ---- per-row base pointers of [.., sk]-shaped tensors
  const T *mrow[QB];
  const T *drow[QB];
  size_t srow[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    int q = q0w + qb * 32 + ql;
    if (q > a.sq - 1) q = a.sq - 1;
    mrow[qb] = nullptr;
    drow[qb] = nullptr;
    if (MASK == kMaskFull)
      mrow[qb] = (const T *)a.mask + (size_t)(bh / a.mask_div) * a.mask_sb + (size_t)q * a.mask_sq;
    srow[qb] = ((size_t)bh * a.sq + q) * a.sk;
    if (DROP == 2 && a.drop_mask) drow[qb] = (const T *)a.drop_mask + srow[qb];
  }

  // four consecutive elements of a [.., sk] row starting at key kk (kk % 4 == 0), as floats.
  // safe = the whole group is known to be in range and 8-byte aligned.
  auto load4 = [&](const T *row, int kk, bool safe, float out[4]) {
    if (safe) {
      v4 t = as_v4<T>(*(const u32x2 *)(row + kk));
#pragma unroll
      for (int i = 0; i < 4; ++i) out[i] = (float)t[i];
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) out[i] = (kk + i < a.sk) ? (float)row[kk + i] : 0.f;
    }
  };
  auto store4 = [&](T *row, int kk, const float in[4]) {
    if (a.mask_vec && kk + 3 < a.sk) {
      v4 t;
#pragma unroll
      for (int i = 0; i < 4; ++i) t[i] = (T)in[i];
      *(v4 *)(row + kk) = t;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (kk + i < a.sk) row[kk + i] = (T)in[i];
    }
  };

  // ---- running state.  mref: reference exponent (log2 units, representable in T); seen: a
  // finite score has set it; lsum: this lane's part of the denominator; o: unnormalised O^T.
  f32x16 o[QB][DB];
  float mref[QB], lsum[QB];
  bool seen[QB];
  v8 bx[QB]; // extra contraction step, B side: (-mref, 1, 1, c, 0 ...) on the lower half-wave
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    mref[qb] = 0.f;
    seen[qb] = false;
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
      if (MASK == kMaskFull) bx[qb][3] = (T)a.mask_b; // constant part of a full mask's term
    }
  }
  float inv_l[QB]; // used by the save pass

  const bool saving = (DROP == 2) && (a.save_softmax != nullptr || a.save_dropout != nullptr);
  const int npass = saving ? 2 : 1;

  for (int pass = 0; pass < npass; ++pass) {
    if (pass == 1) {
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        const float lt = xhalf_sum(lsum[qb]);
        inv_l[qb] = lt > 0.f ? 1.f / lt : 0.f;
      }
    }
    gload(0);
    lstore(0);
    __syncthreads();

    for (int kt = 0; kt < nkt; ++kt) {
      const int cur = kt & 1;
      const int k0 = kt * BK;
      if (kt + 1 < nkt) gload(k0 + BK);

      const char *ldsK = lds + cur * 2 * TILEB;
      const char *ldsV = ldsK + TILEB;
      const char *ldsXc = ldsX + cur * BK * XROWB;

      const bool active = !CAUSAL || (k0 <= q0w + QB * 32 - 1);
      if (active) {
        // ---- x^T = K . Q'^T  + (mask[key] - mref[q]) through the extra step
        f32x16 x[QB][NSB];
#pragma unroll
        for (int sb = 0; sb < NSB; ++sb) {
#pragma unroll
          for (int qb = 0; qb < QB; ++qb)
#pragma unroll
            for (int r = 0; r < 16; ++r) x[qb][sb][r] = 0.f;
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            const v8 ka = as_v8<T>(*(const u32x4 *)(ldsK + (sb * 32 + ql) * ROWB + ks * 32 + h * 16));
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) x[qb][sb] = E::mfma(ka, qreg[qb][ks], x[qb][sb]);
          }
          const v8 xa = as_v8<T>(*(const u32x4 *)(ldsXc + (sb * 32 + ql) * XROWB + h * 16));
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) x[qb][sb] = E::mfma(xa, bx[qb], x[qb][sb]);
        }

        // Only tiles crossing the causal diagonal need a per-element test (the ragged tail is
        // handled by the -inf mask terms of the extra step).
        const bool diag = CAUSAL && (k0 + BK - 1 > q0w);
        const bool vec_ok = a.mask_vec && (k0 + BK <= a.sk);
        v8 pfrag[QB][NSB][2];

        auto softmax_block = [&](int qb, auto guarded_tag) {
          constexpr bool GUARDED = decltype(guarded_tag)::value;
          const int q = q0w + qb * 32 + ql;
          if (MASK == kMaskFull || GUARDED) {
#pragma unroll
            for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
              for (int g = 0; g < 4; ++g) {
                const int kk = k0 + sb * 32 + 8 * g + 4 * h;
                float mv[4] = {0.f, 0.f, 0.f, 0.f};
                if (MASK == kMaskFull) load4(mrow[qb], kk, vec_ok, mv);
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                  float xv = x[qb][sb][4 * g + t];
                  if (MASK == kMaskFull) xv = fmaf(mv[t], a.mask_a, xv);
                  if (GUARDED) xv = (kk + t <= q) ? xv : NEG_INF;
                  x[qb][sb][4 * g + t] = xv;
                }
              }
          }

          // ---- P = exp2(x), rounded to the element type; row sum of the rounded values
          float p[NSB][16];
          v8 pk[NSB][2];
          float rs = 0.f;
          auto exp_pack = [&](float shift) {
            rs = 0.f;
#pragma unroll
            for (int sb = 0; sb < NSB; ++sb) {
#pragma unroll
              for (int r = 0; r < 16; ++r) p[sb][r] = fast_exp2(x[qb][sb][r] + shift);
#pragma unroll
              for (int c = 0; c < 2; ++c) {
#pragma unroll
                for (int j = 0; j < 8; ++j) pk[sb][c][j] = (T)p[sb][8 * c + j];
#pragma unroll
                for (int j = 0; j < 4; ++j) rs = dot2_ones<T>(pk[sb][c], j, rs);
              }
            }
          };
          exp_pack(0.f);

          if (pass == 1) {
            // save-intermediates pass: normalised softmax and its dropped/scaled version
            T *ssm = a.save_softmax ? (T *)a.save_softmax + srow[qb] : nullptr;
            T *sdr = a.save_dropout ? (T *)a.save_dropout + srow[qb] : nullptr;
            if (q < a.sq) {
#pragma unroll
              for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                  const int kk = k0 + sb * 32 + 8 * g + 4 * h;
                  if (kk >= a.sk) continue;
                  float pv[4], dm[4] = {1.f, 1.f, 1.f, 1.f};
#pragma unroll
                  for (int t = 0; t < 4; ++t) pv[t] = p[sb][4 * g + t] * inv_l[qb];
                  if (ssm) store4(ssm, kk, pv);
                  if (sdr) {
                    if (drow[qb]) load4(drow[qb], kk, vec_ok, dm);
#pragma unroll
                    for (int t = 0; t < 4; ++t) pv[t] = pv[t] * (dm[t] * a.drop_scale);
                    store4(sdr, kk, pv);
                  }
                }
            }
            return;
          }

          // ---- rare path: the reference exponent is unset or this tile left the window.
          // Take the tile maximum, move the reference there (kept representable in T),
          // rescale the running sums and redo the exponentials.
          const bool unfit = !(rs < WINDOW) || !seen[qb];
          if (__builtin_amdgcn_ballot_w64(unfit) != 0ull) {
            float mx = NEG_INF;
#pragma unroll
            for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
              for (int r = 0; r < 16; r += 2) mx = max3(mx, x[qb][sb][r], x[qb][sb][r + 1]);
            mx = xhalf_max(mx);
            float mnew = mref[qb];
            const bool had_ref = seen[qb];
            if (mx != NEG_INF) {
              const float cand = (float)(T)(mref[qb] + mx);
              mnew = seen[qb] ? fmaxf(mref[qb], cand) : cand;
              seen[qb] = true;
            }
            const float shift = mref[qb] - mnew;
            // Nothing has been accumulated before the first reference is set, and that first move can be
            // upwards by thousands (a first tile under a -10000 mask): 0 * 2^shift would be 0 * inf.
            if (shift != 0.f && had_ref) {
              const float alpha = fast_exp2(shift);
              lsum[qb] *= alpha;
#pragma unroll
              for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int r = 0; r < 16; ++r) o[qb][db][r] *= alpha;
            }
            mref[qb] = mnew;
            if (h == 0) bx[qb][0] = (T)(-mnew);
            exp_pack(shift);
          }
          lsum[qb] += rs;

          // ---- dropout acts on the numerator only
          if (DROP == 1) {
#pragma unroll
            for (int sb = 0; sb < NSB; ++sb) {
              uint32_t wd[4];
              drop_words_q(a.drop, (uint32_t)bh, (uint32_t)q, (uint32_t)(k0 + sb * 32), h, l, wd);
#pragma unroll
              for (int g = 0; g < 4; ++g)
#pragma unroll
                for (int t = 0; t < 4; ++t)
                  if (!drop_keep_byte(wd[g], t, a.drop.thr)) pk[sb][g >> 1][4 * (g & 1) + t] = (T)0.f;
            }
          } else if (DROP == 2) {
            if (drow[qb]) {
#pragma unroll
              for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                  const int kk = k0 + sb * 32 + 8 * g + 4 * h;
                  float dm[4];
                  load4(drow[qb], kk, vec_ok, dm);
#pragma unroll
                  for (int t = 0; t < 4; ++t)
                    pk[sb][g >> 1][4 * (g & 1) + t] = (T)((float)pk[sb][g >> 1][4 * (g & 1) + t] * dm[t]);
                }
            }
          }
#pragma unroll
          for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
            for (int c = 0; c < 2; ++c) pfrag[qb][sb][c] = pk[sb][c];
        };

        if (diag) {
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) softmax_block(qb, std::true_type{});
        } else {
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) softmax_block(qb, std::false_type{});
        }

        if (pass == 0) {
          // ---- O^T += V^T . P^T
#pragma unroll
          for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
              for (int c = 0; c < 2; ++c) {
                const v8 va = lds_load_a_transposed<T, ROWBV>(ldsV, sb * 32, db * 32, c, l);
#pragma unroll
                for (int qb = 0; qb < QB; ++qb) o[qb][db] = E::mfma(va, pfrag[qb][sb][c], o[qb][db]);
              }
        }
      }

      if (kt + 1 < nkt) lstore(cur ^ 1);
      __syncthreads();
    }
  }

  // ---- epilogue: normalise, round, store O and the row log-sum-exp
  T *Ob = (T *)a.o + RW::head(a.mo, bh, a.sq);
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int q = q0w + qb * 32 + ql;
    const float lt = xhalf_sum(lsum[qb]);
    const float inv = lt > 0.f ? a.drop_scale / lt : 0.f;
    if (q < a.sq) {
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          v4 t;
#pragma unroll
          for (int i = 0; i < 4; ++i) t[i] = (T)(o[qb][db][4 * g + i] * inv);
          if (db * 32 + 8 * g + 4 * h < RW::cols(a)) *(v4 *)(Ob + (size_t)q * RW::ss(a.mo) + db * 32 + 8 * g + 4 * h) = t;
        }
      // the constant part of a full mask's term entered the product rounded to T; the
      // difference cancels in O but belongs in the log-sum-exp
      const float cfix = (MASK == kMaskFull) ? a.mask_b - (float)(T)a.mask_b : 0.f;
      if (a.lse && h == 0)
        a.lse[(size_t)bh * a.sq + q] = lt > 0.f ? (mref[qb] + cfix + fast_log2(lt)) * FMHA_LN2 : NEG_INF;
    }
  }
}

} // namespace fmha
