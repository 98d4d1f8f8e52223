// Backward attention kernels for gfx950 (wave64, MFMA 32x32x16).  The reference has no
// backward (its README states forward only); the formulas are the analytic gradient of
//   O = (softmax(scale Q K^T + mask) o Z) V ,  Z = dropout factor (0 or drop_scale):
//   dV = (P o Z)^T dO ;  dPz = dO V^T ;  dP = dPz o Z ;  delta_i = sum_d dO_id O_id
//   dS = P o (dP - delta) ;  dQ = scale dS K ;  dK = scale dS^T Q
// with P recomputed from the saved row log-sum-exp: P = exp(score - LSE).
//
// Two kernels, no atomics, deterministic:
//   fmha_bwd_dq_kernel    one workgroup per (bh, query tile), walks the key tiles;
//                         lane = query, like the forward: x^T = K.Q'^T, g^T = V.dO^T,
//                         dQ^T += K^T.dS^T (K^T through the LDS transpose read).  Also
//                         computes delta for its rows and writes it out.
//   fmha_bwd_dkdv_kernel  one workgroup per (bh, key tile), walks the query tiles with
//                         dK^T / dV^T accumulators resident in registers; lane = key:
//                         x = Q.K'^T, g = dO.V^T, dV^T += dO^T.(P o Z), dK^T += Q^T.dS
//                         (dO^T and Q^T through the LDS transpose read).
// In both, the 32x32 accumulator tile of the score product is converted in registers
// into the B operand of the next product (see fmha_common.h), so P and dS never travel
// through LDS.  The price of avoiding atomics and LDS transposes of dS is that the score
// and dP products are formed in both kernels (7 tile products instead of 5).
//
// As in the forward, the per-element VALU work is what bounds these kernels at head dim
// 64, so everything that is a rank-one term rides in one extra contraction step:
//   x = score*scale*log2e + mask[key] - LSE[q]*log2e     (K' or Q' pre-scaled; mask and LSE
//                                                         split hi+lo in the element type)
//   g = drop_scale * dO.V^T - delta[q]                 (the register-resident operand of that
//                                                        product, dO or V, is pre-multiplied by drop_scale)
// leaving  P = exp2(x)  and  dS = P * (kept ? g : -delta)  (= P*g without dropout).
// "Minus infinity" terms are entered as a large finite negative number, because the same
// extra rows also meet zeros in the other operand of the second product.
#pragma once
#include "fmha_common.h"
#include "fmha_fwd_kernel.h"

namespace fmha {

struct BwdArgs {
  const void *q, *k, *v, *o, *dout;
  const float *lse;
  float *delta;
  void *dq, *dk, *dv;
  const void *mask;
  int64_t mask_sb, mask_sq;
  int32_t mask_div;
  int32_t mask_vec;
  float mask_a, mask_b;
  int32_t bh, sq, sk;
  int32_t ntile; // tiles per head of the kernel being launched
  int32_t pair;  // causal only: a workgroup takes the tile pair (i, ntile-1-i) instead of one tile
  float scale_l2, scale, drop_scale;
  DropCtx drop;
  int32_t flags;
  const int32_t *kv_len; // optional valid key count per group of kv_div heads
  int32_t kv_div;
  RowMap mq, mk, mv, mo, mdo, mdq, mdk, mdv; // row layouts (mk.ss == mv.ss)
  float *ws; // the caller's workspace pointer: no kernel of a release build reads it (development builds: cycle stamps)
  int32_t dcols; // elements per row that exist (<= the kernel's head dim; run-time layouts only)
};

// BT: rows per LDS tile (keys in the dQ kernel, queries in the dK/dV kernel).  The dK/dV kernel
// at head dim 128 holds 128 accumulator registers; walking the queries 32 at a time brings its
// score / dP tiles and their fragments close enough to a two-waves-per-SIMD register budget
// that forcing that occupancy pays (+11 % measured) -- for the plain variant only: with a causal
// mask the shorter tiles lose more to the uneven tile counts, and the dropout variant spills
// too much, so those keep 64-row tiles at one wave per SIMD.
template <int D> constexpr int bwd_dq_tile_rows() { return 64; }
// (Head dim 256 has a dK/dV kernel of its own, fmha_bwd_wide.h.)
template <int D, bool CAUSAL, int DROP> constexpr bool bwd_dkdv_small_tiles() { return D == 128 && !CAUSAL && DROP == 0; }
template <int D, bool CAUSAL, int DROP> constexpr int bwd_dkdv_tile_rows() {
  return bwd_dkdv_small_tiles<D, CAUSAL, DROP>() ? 32 : 64;
}

template <int D, int BT_> struct BwdCfg {
  static constexpr int BT = BT_;          // rows per LDS tile
  static constexpr int NSB = BT / 32;
  static constexpr int KS = D / 16;
  static constexpr int DB = D / 32;
  static constexpr int TILEB = BT * D * 2; // swizzled panel layout of fmha_common.h, no padding
  static constexpr int XROWB = 32;        // extra-step rows: 16 elements
  // two tiles x 2 stages + two sets of extra rows x 2 stages + {delta} x 2 stages
  static constexpr int LDS_BYTES = 4 * TILEB + 2 * 2 * BT * XROWB + 2 * BT * 4;
  // dK/dV kernel with a full mask tensor: [stage][BT queries][128 keys of the workgroup + 8] mask values
  static constexpr int MASK_PITCH = 128 + 8;
  static constexpr int MASK_BYTES = 2 * BT * MASK_PITCH * 2;
};

// Keys a head may see at all: [0, sk) or its valid count (possibly 0).
FMHA_DEV int bwd_valid_keys(const BwdArgs &a, int bh) {
  if (!a.kv_len) return a.sk;
  const int n = a.kv_len[bh / a.kv_div];
  return n < 0 ? 0 : (n < a.sk ? n : a.sk);
}

// BwdArgs::flags
enum { kBwdFlagNoTrim = 1 }; // visit every key tile even where a per-key mask hard-masks the tail

// The mask's own say on how many keys a head sees.  A per-key mask that ends in hard-masked keys
// (mask term of -9000 or below: the -10000 or -inf tail of a padded sequence) gives those keys
// P = exp(score + mask - LSE) = 0 exactly, hence dS = 0: their tiles need not be visited and their
// dK, dV rows are zero.  A workgroup loads its head's mask row when it starts (`issue`, NT threads,
// rows of up to 1024 keys) and turns it into a key count once its own operand loads, issued behind
// it, have been consumed (`finish`), so that the row costs no trip to memory of its own.  A row
// without any live key keeps all its keys (its softmax is a plain one over all of them).
template <typename T, int NT> struct MaskTail {
  static constexpr int kMaxKeys = 1024, NCH = kMaxKeys / NT;
  T v[NCH];
  FMHA_DEV static bool enabled(const BwdArgs &a) { return a.sk > 128 && a.sk <= kMaxKeys && !(a.flags & kBwdFlagNoTrim); } // (128 keys or fewer: nothing to leave out)
  FMHA_DEV void issue(const BwdArgs &a, const T *mkey, int tid) {
#pragma unroll
    for (int c = 0; c < NCH; ++c) v[c] = (T)0.f;
    if (enabled(a)) { // uniform
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        const int key = c * NT + tid;
        v[c] = mkey[key < a.sk ? key : a.sk - 1];
      }
    }
  }
  // `red`: NT / 64 ints of LDS that nothing else uses until this returns (two barriers inside)
  FMHA_DEV int finish(const BwdArgs &a, int *red, int tid) {
    if (!enabled(a)) return a.sk;
    constexpr float kHardMask = -9000.f * FMHA_LOG2E;
    int last = -1;
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const int key = c * NT + tid;
      const bool live = key < a.sk && fmaf((float)v[c], a.mask_a, a.mask_b) > kHardMask;
      const unsigned long long bal = __builtin_amdgcn_ballot_w64(live);
      if (bal) last = c * NT + (tid & ~63) + 63 - __builtin_clzll(bal); // chunks ascend: the last hit wins
    }
    if ((tid & 63) == 0) red[tid >> 6] = last;
    __syncthreads();
    int top = -1;
#pragma unroll
    for (int ww = 0; ww < NT / 64; ++ww) top = red[ww] > top ? red[ww] : top;
    top = __builtin_amdgcn_readfirstlane(top);
    __syncthreads();
    return top < 0 ? a.sk : top + 1;
  }
};

// A value as hi + lo in the element type (|error| ~ 2^-2p relative), clamped to a large finite
// negative number so that it may be multiplied by zero.
template <typename T> FMHA_DEV void split_hi_lo(float v, T &hi, T &lo) {
  constexpr float BIG = sizeof(T) == 2 && std::is_same<T, _Float16>::value ? -60000.f : -1.0e30f;
  v = v > BIG ? v : BIG;
  hi = (T)v;
  lo = (T)(v - (float)hi);
}

// ------------------------------------------------------------------------------ dQ
// (At head dim 128, and with a full mask tensor under a causal mask and dropout, some variants need
// a few registers more than a two-waves-per-SIMD budget: spill those few rather than drop to one
// wave per SIMD, +10 % measured.)
template <typename T, int D, int QB, int NW, int MASK, bool CAUSAL, int DROP, bool STRIDED>
__global__ __launch_bounds__(NW * 64)
    __attribute__((amdgpu_waves_per_eu((D == 128 || MASK == kMaskFull) ? 2 : 1, 2))) void fmha_bwd_dq_kernel(const BwdArgs a) {
  using RW = Rows<STRIDED, D>;
  using E = Elem<T>;
  using v8 = typename E::v8;
  using v4 = typename E::v4;
  using C = BwdCfg<D, bwd_dq_tile_rows<D>()>;
  constexpr int BK = C::BT, NSB = C::NSB, KS = C::KS, DB = C::DB, TILEB = C::TILEB;
  constexpr int XROWB = C::XROWB;
  constexpr int NT = NW * 64;
  constexpr int QT = NW * QB * 32;
  constexpr float NEG_INF = -__builtin_inff();
  constexpr float BIGNEG = -60000.f;

  extern __shared__ __attribute__((aligned(16))) char lds[];
  char *ldsXb = lds + 4 * TILEB; // extra rows per key: (1, 1, mask_hi, mask_lo, 1, 1, 0 ...)

  const int tid = threadIdx.x;
  const int w = tid >> 6, l = tid & 63, ql = l & 31, h = l >> 5;

  int bid = blockIdx.x;
  const int nb = gridDim.x;
  if ((nb & 7) == 0) bid = (bid & 7) * (nb >> 3) + (bid >> 3);
  // With a causal mask the work of a query tile grows with its index, so a workgroup takes a
  // pair of tiles (i, n-1-i), one after the other: every workgroup then has the same amount of
  // work (the host launches ceil(n/2) workgroups per head; it does so when that still fills the
  // device, otherwise one tile per workgroup, longest first).
  const bool paired = CAUSAL && a.pair;
  const int npair = paired ? (a.ntile + 1) / 2 : a.ntile;
  const int bh = bid / npair;
  const int pi = bid - bh * npair;
  const int npass = (paired && a.ntile - 1 - pi != pi) ? 2 : 1;
  MaskTail<T, NT> tail;
  int live_keys = a.sk; // the mask's own count of keys worth visiting
  if (MASK == kMaskPerKey) tail.issue(a, (const T *)a.mask + (size_t)(bh / a.mask_div) * a.mask_sb, tid);
  for (int pass = 0; pass < npass; ++pass) {
  const int qt = CAUSAL ? (pass == 0 ? a.ntile - 1 - pi : pi) : pi;
  const int q0w = qt * QT + w * (QB * 32);

  const T *Qb = (const T *)a.q + RW::head(a.mq, bh, a.sq);
  const T *Ob = (const T *)a.o + RW::head(a.mo, bh, a.sq);
  const T *dOb = (const T *)a.dout + RW::head(a.mdo, bh, a.sq);
  const T *Kb = (const T *)a.k + RW::head(a.mk, bh, a.sk);
  const T *Vb = (const T *)a.v + RW::head(a.mv, bh, a.sk);
  const T *mkey = (MASK == kMaskPerKey) ? (const T *)a.mask + (size_t)(bh / a.mask_div) * a.mask_sb : nullptr;

  // ---- per-row operands: Q' and dO as B operands, the extra-step columns, delta
  v8 qreg[QB][KS], doreg[QB][KS];
  v8 bxs[QB], bxd[QB]; // (-L_hi, -L_lo, 1, 1, c_hi, c_lo, 0, 0) and (-d_hi, -d_lo, 0 ...) on the lower half-wave
  float delta[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int q = q0w + qb * 32 + ql;
    // Rows past the end re-read the last row (nothing of theirs is stored and their P is forced to 0).
    // The loads are unconditional on purpose: a load under a lane condition is merged with its "else"
    // value right behind it, so the compiler waits for it on the spot and the twelve loads below would
    // take four round trips to memory instead of one.
    const int qc = q < a.sq ? q : a.sq - 1;
    u32x4 tq[KS], td[KS], to[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const size_t col = ks * 16 + h * 8 < RW::cols(a) ? ks * 16 + h * 8 : 0; // padding chunks are zeroed below
      tq[ks] = *(const u32x4 *)(Qb + (size_t)qc * RW::ss(a.mq) + col);
      td[ks] = *(const u32x4 *)(dOb + (size_t)qc * RW::ss(a.mdo) + col);
      to[ks] = *(const u32x4 *)(Ob + (size_t)qc * RW::ss(a.mo) + col);
    }
    const float lse_q = a.lse[(size_t)bh * a.sq + qc];
    float dsum = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const bool live = ks * 16 + h * 8 < RW::cols(a);
      const v8 qraw = as_v8<T>(chunk_or_zero(tq[ks], live));
      const v8 doraw = as_v8<T>(chunk_or_zero(td[ks], live));
      const v8 ov = as_v8<T>(to[ks]);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        qreg[qb][ks][j] = (T)((float)qraw[j] * a.scale_l2);
        doreg[qb][ks][j] = DROP == 1 ? (T)((float)doraw[j] * a.drop_scale) : doraw[j];
        dsum = fmaf((float)doraw[j], (float)ov[j], dsum);
      }
    }
    dsum = xhalf_sum(dsum);
    delta[qb] = dsum;
    float nl = BIGNEG; // rows past the end and fully masked rows get P = 0
    if (q < a.sq) {
      if (lse_q != NEG_INF) nl = -lse_q * FMHA_LOG2E;
      if (h == 0) a.delta[(size_t)bh * a.sq + q] = dsum;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      bxs[qb][j] = (T)0.f;
      bxd[qb][j] = (T)0.f;
    }
    if (h == 0) {
      T hi, lo;
      split_hi_lo<T>(nl, hi, lo);
      bxs[qb][0] = hi;
      bxs[qb][1] = lo;
      bxs[qb][2] = (T)1.f;
      bxs[qb][3] = (T)1.f;
      if (MASK == kMaskFull) { // constant part of a full mask's term
        split_hi_lo<T>(a.mask_b, hi, lo);
        bxs[qb][4] = hi;
        bxs[qb][5] = lo;
      }
      split_hi_lo<T>(-dsum, hi, lo);
      bxd[qb][0] = hi;
      bxd[qb][1] = lo;
    }
  }

  // (the tile area of LDS is idle here in the first pass: nothing has been copied yet)
  if (MASK == kMaskPerKey && pass == 0) live_keys = tail.finish(a, (int *)lds, tid);
  int skv = bwd_valid_keys(a, bh);
  skv = live_keys < skv ? live_keys : skv;
  int nkt = (skv + BK - 1) / BK;
  if (nkt < 1) nkt = 1; // no valid key at all: one tile of keys that are all "past the end"
  if (CAUSAL) {
    int qmax = qt * QT + QT - 1;
    if (qmax > a.sq - 1) qmax = a.sq - 1;
    const int need = qmax / BK + 1;
    if (need < nkt) nkt = need;
  }
  const int kend = nkt * BK < skv ? nkt * BK : skv;
  const int kclamp = kend > 0 ? kend : 1; // row bound for addresses

  // ---- staging.  K and V tiles are copied from global memory straight into LDS (rows past the
  // end re-read the last valid row; their scores are pushed to -60000 by the extra step, so
  // P = dS = 0 for them).  The extra rows take the register path, one tile further ahead, so
  // that their load has long landed when it is used: the compiler's wait for a load it knows
  // about also waits for every copy issued before it.
  const uint32_t lds_base = lds_address(lds);
  PanelLane pl;
  pl.init(l);
  TileCopy<T, D, BK, NT> tcopy;
  tcopy.init(tid, RW::ss(a.mk)); // K and V rows are equally far apart
  auto dma_kv = [&](int kt) {
    const uint32_t dst = lds_base + (uint32_t)(kt & 1) * 2 * TILEB;
    tcopy.issue(Kb, kt * BK, kclamp, dst, tid, RW::cols(a));
    tcopy.issue(Vb, kt * BK, kclamp, dst + TILEB, tid, RW::cols(a));
  };
  T mraw = (T)0.f;
  bool mvalid = false;
  auto gloadX = [&](int kt) {
    const int kr = kt * BK + (tid & (BK - 1));
    mvalid = kr < kend;
    if (MASK == kMaskPerKey) mraw = mkey[mvalid ? kr : kclamp - 1];
  };
  auto lstoreX = [&](int stage) {
    if (tid < BK) {
      float mk = 0.f;
      if (MASK == kMaskPerKey) mk = fmaf((float)mraw, a.mask_a, a.mask_b);
      if (!mvalid) mk = BIGNEG;
      T hi, lo;
      split_hi_lo<T>(mk, hi, lo);
      v8 x0, x1;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        x0[j] = (T)0.f;
        x1[j] = (T)0.f;
      }
      x0[0] = (T)1.f;
      x0[1] = (T)1.f;
      x0[2] = hi;
      x0[3] = lo;
      x0[4] = (T)1.f;
      x0[5] = (T)1.f;
      v8 *dst = (v8 *)(ldsXb + stage * BK * XROWB + tid * XROWB);
      dst[0] = x0;
      dst[1] = x1;
    }
  };

  const T *mrow[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    int q = q0w + qb * 32 + ql;
    if (q > a.sq - 1) q = a.sq - 1;
    mrow[qb] = nullptr;
    if (MASK == kMaskFull)
      mrow[qb] = (const T *)a.mask + (size_t)(bh / a.mask_div) * a.mask_sb + (size_t)q * a.mask_sq;
  }
  // A full mask tensor takes the register path, one tile ahead (at head dim 64, where the
  // registers are there): this lane's 32 mask values of the next tile are requested as soon as
  // the current tile's have been consumed -- they seed the score accumulators, so that happens at
  // the top of the iteration, before the copies go out.
  constexpr bool MASK_AHEAD = MASK == kMaskFull && D == 64;
  v4 mreg[QB][NSB][4];
  auto mload = [&](int tile) {
    const int mk0 = tile * BK;
    const bool vec_ok = a.mask_vec && (mk0 + BK <= a.sk);
#pragma unroll
    for (int qb = 0; qb < QB; ++qb)
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int kk = mk0 + sb * 32 + 8 * g + 4 * h;
          if (vec_ok) {
            mreg[qb][sb][g] = as_v4<T>(*(const u32x2 *)(mrow[qb] + kk));
          } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) mreg[qb][sb][g][i] = (kk + i < a.sk) ? mrow[qb][kk + i] : (T)0.f;
          }
        }
  };

  f32x16 dq[QB][DB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb)
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) dq[qb][db][r] = 0.f;

  if (MASK_AHEAD) mload(0);
  dma_kv(0);
  gloadX(0);
  lstoreX(0);
  gloadX(1);
  dma_wait_all();
  __syncthreads();

  for (int kt = 0; kt < nkt; ++kt) {
    const int cur = kt & 1;
    const int k0 = kt * BK;
    // x^T = K.Q'^T + (mask - LSE) ; g^T = drop_scale*V.dO^T - delta   (accumulators visited round-robin)
    // A full mask tensor's term seeds the score accumulators.
    f32x16 x[QB][NSB], g[QB][NSB];
    if (MASK == kMaskFull && !MASK_AHEAD) mload(kt);
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
      for (int qb = 0; qb < QB; ++qb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          x[qb][sb][r] = MASK == kMaskFull ? (float)mreg[qb][sb][r / 4][r % 4] * a.mask_a : 0.f;
          g[qb][sb][r] = 0.f;
        }
    if (MASK_AHEAD && kt + 1 < nkt) mload(kt + 1);
    if (kt + 1 < nkt) {
      lstoreX(cur ^ 1); // rows of tile kt+1, loaded one iteration ago
      gloadX(kt + 2);
      dma_kv(kt + 1);
    }
    const char *ldsK = lds + cur * 2 * TILEB;
    const char *ldsV = ldsK + TILEB;
    const char *ldsX = ldsXb + cur * BK * XROWB;

#pragma unroll
    for (int ks = 0; ks <= KS; ++ks)
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb) {
        if (ks < KS) {
          const v8 ka = panel_read_rows<T, BK>(ldsK, pl, sb, ks);
          const v8 va = panel_read_rows<T, BK>(ldsV, pl, sb, ks);
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) {
            x[qb][sb] = E::mfma(ka, qreg[qb][ks], x[qb][sb]);
            g[qb][sb] = E::mfma(va, doreg[qb][ks], g[qb][sb]);
          }
        } else {
          const v8 xa = as_v8<T>(*(const u32x4 *)(ldsX + (sb * 32 + ql) * XROWB + h * 16));
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) {
            x[qb][sb] = E::mfma(xa, bxs[qb], x[qb][sb]);
            g[qb][sb] = E::mfma(xa, bxd[qb], g[qb][sb]);
          }
        }
      }

    const bool diag = CAUSAL && (k0 + BK - 1 > q0w);
    v8 dsfrag[QB][NSB][2];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      const int q = q0w + qb * 32 + ql;
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb) {
        uint32_t wd[4] = {0u, 0u, 0u, 0u};
        if (DROP == 1) drop_words_q(a.drop, (uint32_t)bh, (uint32_t)q, (uint32_t)(k0 + sb * 32), h, l, wd);
        float ds[16];
#pragma unroll
        for (int gq = 0; gq < 4; ++gq) {
          const int kk = k0 + sb * 32 + 8 * gq + 4 * h;
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            float xv = x[qb][sb][4 * gq + t];
            if (diag) xv = (kk + t <= q) ? xv : BIGNEG;
            const float p = fast_exp2(xv);
            float gv = g[qb][sb][4 * gq + t];
            if (DROP == 1) gv = drop_keep_byte(wd[gq], t, a.drop.thr) ? gv : -delta[qb];
            ds[4 * gq + t] = p * gv;
          }
        }
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
          for (int j = 0; j < 8; ++j) dsfrag[qb][sb][c][j] = (T)ds[8 * c + j];
      }
    }

    // dQ^T += K^T . dS^T
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const v8 kt_a = panel_read_transposed<T, BK>(ldsK, pl, sb, db, c);
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) dq[qb][db] = E::mfma(kt_a, dsfrag[qb][sb][c], dq[qb][db]);
        }

    dma_wait_all();
    __syncthreads();
  }

  T *dQb = (T *)a.dq + RW::head(a.mdq, bh, a.sq);
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int q = q0w + qb * 32 + ql;
    if (q < a.sq) {
#pragma unroll
      for (int db = 0; db < DB; ++db) store_acc_block_row<T>(dQb + (size_t)q * RW::ss(a.mdq) + db * 32, dq[qb][db], a.scale, h, RW::cols(a) - db * 32);
    }
  }
  __syncthreads(); // the next pass refills the tiles
  } // pass
}

// --------------------------------------------------------------------------- dK, dV
template <typename T, int D, int KB, int NW, int MASK, bool CAUSAL, int DROP, bool STRIDED>
__global__ __launch_bounds__(NW * 64)
    __attribute__((amdgpu_waves_per_eu(bwd_dkdv_small_tiles<D, CAUSAL, DROP>() ? 2 : 1, 2))) void fmha_bwd_dkdv_kernel(const BwdArgs a) {
  using RW = Rows<STRIDED, D>;
  using E = Elem<T>;
  using v8 = typename E::v8;
  using v4 = typename E::v4;
  using C = BwdCfg<D, bwd_dkdv_tile_rows<D, CAUSAL, DROP>()>;
  constexpr int BQ = C::BT, NSB = C::NSB, KS = C::KS, DB = C::DB, TILEB = C::TILEB;
  constexpr int XROWB = C::XROWB;
  constexpr int NT = NW * 64;
  constexpr int KT = NW * KB * 32;
  constexpr float NEG_INF = -__builtin_inff();
  constexpr float BIGNEG = -60000.f;
  static_assert(NT >= BQ, "row statistics are staged by the first BQ threads");

  extern __shared__ __attribute__((aligned(16))) char lds[];
  // extra rows per query: [stage][{score row (-L_hi,-L_lo,1,1,1,1,0..), dP row (-d_hi,-d_lo,0..)}][BQ]
  char *ldsXb = lds + 4 * TILEB;
  float *ldsDl = (float *)(ldsXb + 2 * 2 * BQ * XROWB); // [stage][BQ] delta (dropout path)

  const int tid = threadIdx.x;
  const int w = tid >> 6, l = tid & 63, kl = l & 31, h = l >> 5;

#ifdef FMHA_BWD_TIMELINE
  // development aid: per wave, the 100 MHz counter at start and end and the cycle counter at the start, at the
  // loop's entry, after every query tile and at the end, written to a.ws (32 words of 8 bytes per wave)
  unsigned long long *tl = (unsigned long long *)a.ws + ((size_t)blockIdx.x * NW + w) * 32;
  int tl_n = 0;
  auto stamp = [&]() {
    if (a.ws != nullptr && l == 0 && tl_n < 30) tl[2 + tl_n++] = __builtin_readcyclecounter();
  };
  if (a.ws != nullptr && l == 0) tl[0] = __builtin_amdgcn_s_memrealtime();
  stamp();
#endif
  int bid = blockIdx.x;
  const int nb = gridDim.x;
  if ((nb & 7) == 0) bid = (bid & 7) * (nb >> 3) + (bid >> 3);
  // causal: a pair of key tiles (i, n-1-i) per workgroup, as in the dQ kernel
  const bool paired = CAUSAL && a.pair;
  const int npair = paired ? (a.ntile + 1) / 2 : a.ntile;
  const int bh = bid / npair;
  const int pi = bid - bh * npair;
  const int npass = (paired && a.ntile - 1 - pi != pi) ? 2 : 1;
  MaskTail<T, NT> tail;
  int live_keys = a.sk; // the mask's own count of keys worth visiting
  if (MASK == kMaskPerKey) tail.issue(a, (const T *)a.mask + (size_t)(bh / a.mask_div) * a.mask_sb, tid);
  for (int pass = 0; pass < npass; ++pass) {
  const int ktile = pass == 0 ? pi : a.ntile - 1 - pi;
  const int k0w = ktile * KT + w * (KB * 32);

  const T *Qb = (const T *)a.q + RW::head(a.mq, bh, a.sq);
  const T *dOb = (const T *)a.dout + RW::head(a.mdo, bh, a.sq);
  const T *Kb = (const T *)a.k + RW::head(a.mk, bh, a.sk);
  const T *Vb = (const T *)a.v + RW::head(a.mv, bh, a.sk);
  const float *lseb = a.lse + (size_t)bh * a.sq;
  const float *delb = a.delta + (size_t)bh * a.sq;

  // ---- per-key operands: K' and V rows as B operands, the extra-step columns
  v8 kreg[KB][KS], vreg[KB][KS];
  const int skv = bwd_valid_keys(a, bh); // keys at or past it are invalid: their dK, dV rows are zero
  v8 bxs[KB], bxd[KB]; // (1, 1, mask_hi, mask_lo, c_hi, c_lo, 0, 0) and (1, 1, 0 ...) on the lower half-wave
#pragma unroll
  for (int kb = 0; kb < KB; ++kb) {
    const int key = k0w + kb * 32 + kl;
    // Unconditional loads (a load under a lane condition makes the compiler wait for it on the spot:
    // four round trips to memory instead of one).  Keys past the end re-read the last row; invalid keys
    // get P = dS = 0 through their mask term, whatever their K and V rows hold.
    const int kc = key < a.sk ? key : a.sk - 1;
    u32x4 tk[KS], tv[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const size_t col = ks * 16 + h * 8 < RW::cols(a) ? ks * 16 + h * 8 : 0; // padding chunks are zeroed below
      tk[ks] = *(const u32x4 *)(Kb + (size_t)kc * RW::ss(a.mk) + col);
      tv[ks] = *(const u32x4 *)(Vb + (size_t)kc * RW::ss(a.mv) + col);
    }
    T mraw_key = (T)0.f;
    if (MASK == kMaskPerKey) mraw_key = ((const T *)a.mask)[(size_t)(bh / a.mask_div) * a.mask_sb + kc];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const bool live = ks * 16 + h * 8 < RW::cols(a);
      const v8 kraw = as_v8<T>(chunk_or_zero(tk[ks], live));
      const v8 vraw = as_v8<T>(chunk_or_zero(tv[ks], live));
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        kreg[kb][ks][j] = (T)((float)kraw[j] * a.scale_l2);
        vreg[kb][ks][j] = DROP == 1 ? (T)((float)vraw[j] * a.drop_scale) : vraw[j];
      }
    }
    float mk = 0.f;
    if (MASK == kMaskPerKey) mk = fmaf((float)mraw_key, a.mask_a, a.mask_b);
    if (key >= skv) mk = BIGNEG;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      bxs[kb][j] = (T)0.f;
      bxd[kb][j] = (T)0.f;
    }
    if (h == 0) {
      T hi, lo;
      bxs[kb][0] = (T)1.f;
      bxs[kb][1] = (T)1.f;
      split_hi_lo<T>(mk, hi, lo);
      bxs[kb][2] = hi;
      bxs[kb][3] = lo;
      if (MASK == kMaskFull) {
        split_hi_lo<T>(a.mask_b, hi, lo);
        bxs[kb][4] = hi;
        bxs[kb][5] = lo;
      }
      bxd[kb][0] = (T)1.f;
      bxd[kb][1] = (T)1.f;
    }
  }
  // A full mask tensor reaches the lanes (one key each) through LDS: the [BQ queries x 128 keys]
  // tile is loaded row-wise, 8 bytes per thread and load, one tile ahead like the extra rows, and
  // each lane then reads its key's column.  (Read straight from global memory, two bytes per lane
  // and element, the mask made this kernel five times slower.)
  const T *mbase = (MASK == kMaskFull) ? (const T *)a.mask + (size_t)(bh / a.mask_div) * a.mask_sb : nullptr;
  constexpr int MP = C::MASK_PITCH;
  constexpr int MLOADS = BQ * 32 / NT; // 8-byte pieces per thread: the tile has BQ rows of 32
  static_assert(MASK != kMaskFull || (KT == 128 && (BQ * 32) % NT == 0), "mask tile staging assumes 128 keys per workgroup");
  T *ldsM = (T *)(lds + C::LDS_BYTES);
  u32x2 mraw[MASK == kMaskFull ? MLOADS : 1];

  const int nqt = (a.sq + BQ - 1) / BQ;
  // first query tile that sees any of these keys; none at all if the whole key tile is invalid
  // (hard-masked keys already have P = 0 through their mask term; the count only decides whether the
  // whole key tile can be left out.  LDS is idle here in the first pass.)
  if (MASK == kMaskPerKey && pass == 0) live_keys = tail.finish(a, (int *)lds, tid);
  const int qt0 = ktile * KT >= (live_keys < skv ? live_keys : skv) ? nqt : (CAUSAL ? (ktile * KT) / BQ : 0);

  // ---- staging: Q and dO tiles copied straight into LDS (rows past the end repeat the last
  // valid row); the per-query extra rows take the register path one tile further ahead, as in
  // the dQ kernel.
  const uint32_t lds_base = lds_address(lds);
  PanelLane pl;
  pl.init(l);
  TileCopy<T, D, BQ, NT> tcopy, tcopy_do; // Q and dO rows need not be equally far apart
  tcopy.init(tid, RW::ss(a.mq));
  tcopy_do.init(tid, RW::ss(a.mdo));
  auto dma_qdo = [&](int qt) {
    const uint32_t dst = lds_base + (uint32_t)(qt & 1) * 2 * TILEB;
    tcopy.issue(Qb, qt * BQ, a.sq, dst, tid, RW::cols(a));
    tcopy_do.issue(dOb, qt * BQ, a.sq, dst + TILEB, tid, RW::cols(a));
  };
  float lraw = 0.f, draw = 0.f;
  bool qvalid = false;
  auto gloadX = [&](int qt) {
    int qr = qt * BQ + (tid & (BQ - 1));
    qvalid = qr < a.sq;
    qr = qvalid ? qr : a.sq - 1;
    lraw = lseb[qr];
    draw = delb[qr];
    if (MASK == kMaskFull) {
      const int kbase = ktile * KT;
      const bool vec_ok = a.mask_vec && (kbase + KT <= a.sk);
#pragma unroll
      for (int i = 0; i < MLOADS; ++i) {
        const int c = i * NT + tid, row = c >> 5, col = (c & 31) * 4;
        int q = qt * BQ + row;
        q = q < a.sq ? q : a.sq - 1;
        const T *src = mbase + (size_t)q * a.mask_sq + kbase + col;
        if (vec_ok) {
          mraw[i] = *(const u32x2 *)src;
        } else { // ragged or unaligned: element by element, inside the row
          v4 t;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int kc = kbase + col + j < a.sk ? kbase + col + j : a.sk - 1;
            t[j] = mbase[(size_t)q * a.mask_sq + kc];
          }
          union { v4 v; u32x2 u; } cv;
          cv.v = t;
          mraw[i] = cv.u;
        }
      }
    }
  };
  auto lstoreX = [&](int stage) {
    if (MASK == kMaskFull) {
#pragma unroll
      for (int i = 0; i < MLOADS; ++i) {
        const int c = i * NT + tid, row = c >> 5, col = (c & 31) * 4;
        *(u32x2 *)(ldsM + (stage * BQ + row) * MP + col) = mraw[i];
      }
    }
    if (tid < BQ) {
      // rows past the end (whose Q/dO rows repeat the last valid row) and fully masked rows: P = 0
      float nl = BIGNEG, dl = 0.f;
      if (qvalid && lraw != NEG_INF) {
        nl = -lraw * FMHA_LOG2E;
        dl = draw;
      }
      v8 xs, xd, z;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        xs[j] = (T)0.f;
        xd[j] = (T)0.f;
        z[j] = (T)0.f;
      }
      T hi, lo;
      split_hi_lo<T>(nl, hi, lo);
      xs[0] = hi;
      xs[1] = lo;
      xs[2] = (T)1.f;
      xs[3] = (T)1.f;
      xs[4] = (T)1.f;
      xs[5] = (T)1.f;
      split_hi_lo<T>(-dl, hi, lo);
      xd[0] = hi;
      xd[1] = lo;
      v8 *ds_ = (v8 *)(ldsXb + (stage * 2 + 0) * BQ * XROWB + tid * XROWB);
      v8 *dd_ = (v8 *)(ldsXb + (stage * 2 + 1) * BQ * XROWB + tid * XROWB);
      ds_[0] = xs;
      ds_[1] = z;
      dd_[0] = xd;
      dd_[1] = z;
      ldsDl[stage * BQ + tid] = dl;
    }
  };

  f32x16 dk[KB][DB], dv[KB][DB];
#pragma unroll
  for (int kb = 0; kb < KB; ++kb)
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        dk[kb][db][r] = 0.f;
        dv[kb][db][r] = 0.f;
      }

  if (qt0 < nqt) {
    dma_qdo(qt0);
    gloadX(qt0);
    lstoreX(qt0 & 1);
    gloadX(qt0 + 1); // row indices are clamped, so looking past the last tile is harmless
  }
  dma_wait_all();
  __syncthreads();
#ifdef FMHA_BWD_TIMELINE
  stamp();
#endif

  for (int qt = qt0; qt < nqt; ++qt) {
    const int cur = qt & 1;
    const int q0 = qt * BQ;
    if (qt + 1 < nqt) {
      lstoreX(cur ^ 1); // rows of tile qt+1, loaded one iteration ago
      gloadX(qt + 2);
      dma_qdo(qt + 1);
    }
    const char *ldsQ = lds + cur * 2 * TILEB;
    const char *ldsDO = ldsQ + TILEB;
    const char *ldsXs = ldsXb + (cur * 2 + 0) * BQ * XROWB;
    const char *ldsXd = ldsXb + (cur * 2 + 1) * BQ * XROWB;
    const float *ldsD = ldsDl + cur * BQ;

    // x = Q.K'^T + (mask - LSE) ; g = drop_scale*dO.V^T - delta
    // (The phases of a tile run one after the other: products, then exponentials and dropout, then the gradient
    // products.  A hand-ordered stream that skewed the two 32-query blocks -- the second block's products beside the
    // first block's exponentials, the first block's gradient products beside the second block's exponentials, the
    // Philox calls beside the products -- measured the same time to within 0.5 %, with and without dropout: with
    // two waves per SIMD the other wave's vector work already falls into this wave's matrix phases, and what the
    // kernel's time follows is the count of vector instructions, not their order.)
    f32x16 x[KB][NSB], g[KB][NSB];
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          // a full mask tensor's term seeds the score accumulators: row = query 8*(r/4) + 4h + r%4 of
          // the 32-query block, column = this lane's key
          x[kb][sb][r] = MASK == kMaskFull
                             ? (float)ldsM[(cur * BQ + sb * 32 + 8 * (r / 4) + 4 * h + r % 4) * MP + w * (KB * 32) + kb * 32 + kl] * a.mask_a
                             : 0.f;
          g[kb][sb][r] = 0.f;
        }
#pragma unroll
    for (int ks = 0; ks <= KS; ++ks)
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb) {
        if (ks < KS) {
          const v8 qa = panel_read_rows<T, BQ>(ldsQ, pl, sb, ks);
          const v8 da = panel_read_rows<T, BQ>(ldsDO, pl, sb, ks);
#pragma unroll
          for (int kb = 0; kb < KB; ++kb) {
            x[kb][sb] = E::mfma(qa, kreg[kb][ks], x[kb][sb]);
            g[kb][sb] = E::mfma(da, vreg[kb][ks], g[kb][sb]);
          }
        } else {
          const int off = (sb * 32 + kl) * XROWB + h * 16;
          const v8 xsa = as_v8<T>(*(const u32x4 *)(ldsXs + off));
          const v8 xda = as_v8<T>(*(const u32x4 *)(ldsXd + off));
#pragma unroll
          for (int kb = 0; kb < KB; ++kb) {
            x[kb][sb] = E::mfma(xsa, bxs[kb], x[kb][sb]);
            g[kb][sb] = E::mfma(xda, bxd[kb], g[kb][sb]);
          }
        }
      }

    const bool diag = CAUSAL && (k0w + KB * 32 - 1 > q0);
    v8 pfrag[KB][NSB][2], dsfrag[KB][NSB][2];
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      const int key = k0w + kb * 32 + kl;
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb) {
        uint32_t rb[4]; // rb[t], byte gq: the random byte of (query 8 gq + 4h + t of the block, this lane's key)
        if (DROP == 1) drop_bytes_k(a.drop, (uint32_t)bh, (uint32_t)(q0 + sb * 32), (uint32_t)key, h, l, rb);
        float pz[16], ds[16];
#pragma unroll
        for (int gq = 0; gq < 4; ++gq) {
          const int qq = sb * 32 + 8 * gq + 4 * h; // row in tile of t = 0
          f32x4 Dl = {0.f, 0.f, 0.f, 0.f};
          if (DROP == 1) Dl = *(const f32x4 *)(ldsD + qq);
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const int q = q0 + qq + t;
            float xv = x[kb][sb][4 * gq + t];
            if (diag) xv = (key <= q) ? xv : BIGNEG;
            const float p = fast_exp2(xv);
            float gv = g[kb][sb][4 * gq + t];
            float pzv = p;
            if (DROP == 1) {
              const bool keep = drop_keep_byte(rb[t], gq, a.drop.thr);
              gv = keep ? gv : -Dl[t];
              pzv = keep ? p : 0.f; // (drop_scale multiplies dV once, on store)
              // keep the selection in fp32: left alone the compiler converts first and selects halves, which costs
              // a conversion per element and a pack per pair instead of one packed conversion per pair
              asm volatile("" : "+v"(pzv));
            }
            pz[4 * gq + t] = pzv;
            ds[4 * gq + t] = p * gv;
          }
        }
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            pfrag[kb][sb][c][j] = (T)pz[8 * c + j];
            dsfrag[kb][sb][c][j] = (T)ds[8 * c + j];
          }
      }
    }

    // dV^T += dO^T . (P o Z) ;  dK^T += Q^T . dS
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const v8 dot = panel_read_transposed<T, BQ>(ldsDO, pl, sb, db, c);
          const v8 qtr = panel_read_transposed<T, BQ>(ldsQ, pl, sb, db, c);
#pragma unroll
          for (int kb = 0; kb < KB; ++kb) {
            dv[kb][db] = E::mfma(dot, pfrag[kb][sb][c], dv[kb][db]);
            dk[kb][db] = E::mfma(qtr, dsfrag[kb][sb][c], dk[kb][db]);
          }
        }

    dma_wait_all();
    __syncthreads();
#ifdef FMHA_BWD_TIMELINE
    stamp();
#endif
  }

  T *dKb = (T *)a.dk + RW::head(a.mdk, bh, a.sk);
  T *dVb = (T *)a.dv + RW::head(a.mdv, bh, a.sk);
#pragma unroll
  for (int kb = 0; kb < KB; ++kb) {
    const int key = k0w + kb * 32 + kl;
    if (key < a.sk) {
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        store_acc_block_row<T>(dKb + (size_t)key * RW::ss(a.mdk) + db * 32, dk[kb][db], a.scale, h, RW::cols(a) - db * 32);
        store_acc_block_row<T>(dVb + (size_t)key * RW::ss(a.mdv) + db * 32, dv[kb][db], DROP == 1 ? a.drop_scale : 1.f, h, RW::cols(a) - db * 32);
      }
    }
  }
  __syncthreads(); // the next pass refills the tiles
  } // pass
#ifdef FMHA_BWD_TIMELINE
  stamp();
  if (a.ws != nullptr && l == 0) tl[1] = __builtin_amdgcn_s_memrealtime();
#endif
}

} // namespace fmha
