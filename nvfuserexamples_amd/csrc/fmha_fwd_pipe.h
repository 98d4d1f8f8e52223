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
// x(t+1) is started before the softmax of tile t may raise the reference exponent, so
// each x buffer remembers the reference that was baked into it; a mismatch sends that
// tile through the (rare) correction path, which re-bases the exponentials.
#pragma once
#include <type_traits>

#include "fmha_fwd_kernel.h"

namespace fmha {

template <typename T, int D, int QB, int NW, int MASK, bool CAUSAL, int DROP>
__global__ __launch_bounds__(NW * 64) void fmha_fwd_pipe_kernel(const FwdArgs a) {
  using E = Elem<T>;
  using v8 = typename E::v8;
  using v4 = typename E::v4;
  using C = FwdCfg<D>;
  constexpr int BK = C::BK, NSB = C::NSB, KS = C::KS, DB = C::DB, ROWB = C::ROWB, XROWB = C::XROWB;
  constexpr int TILEB = C::TILEB;
  constexpr int NT = NW * 64;
  constexpr int QT = NW * QB * 32;
  constexpr int CPR = D / 8;
  constexpr int CPT = BK * CPR / NT;
  static_assert(BK * CPR % NT == 0, "tile must divide evenly over the workgroup");
  static_assert(NT >= BK, "the extra rows are staged by the first BK threads");
  static_assert(DROP == 0 || DROP == 1, "tensor dropout and the save pass use fmha_fwd_kernel");
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

  int bid = blockIdx.x;
  const int nb = gridDim.x;
  if ((nb & 7) == 0) bid = (bid & 7) * (nb >> 3) + (bid >> 3); // one XCD (one L2) per run of tiles
  const int bh = bid / a.nqt;
  int qt = bid - bh * a.nqt;
  if (CAUSAL) qt = a.nqt - 1 - qt;
  const int q0w = qt * QT + w * (QB * 32);

  const T *Qb = (const T *)a.q + (size_t)bh * a.sq * D;
  const T *Kb = (const T *)a.k + (size_t)bh * a.sk * D;
  const T *Vb = (const T *)a.v + (size_t)bh * a.sk * D;
  const T *mkey = (MASK == kMaskPerKey) ? (const T *)a.mask + (size_t)(bh / a.mask_div) * a.mask_sb : nullptr;

  // Q rows are loaded unconditionally (rows past the end repeat the last valid row and are
  // never stored) and converted only after the first K/V tiles have been requested, so that
  // the whole prologue costs one global round trip instead of three.
  u32x4 qraw[QB][KS];
  v8 qreg[QB][KS]; // filled in the prologue
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    int q = q0w + qb * 32 + ql;
    q = q < a.sq ? q : a.sq - 1;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qraw[qb][ks] = *(const u32x4 *)(Qb + (size_t)q * D + ks * 16 + h * 8);
  }

  // ---- key range: tiles [0, nkt), keys [0, kend); the count is padded to even with an
  // all-masked phantom tile so that the two x / P buffers alternate with fixed roles
  int nkt = (a.sk + BK - 1) / BK;
  if (CAUSAL) {
    int qmax = qt * QT + QT - 1;
    if (qmax > a.sq - 1) qmax = a.sq - 1;
    const int need = qmax / BK + 1;
    if (need < nkt) nkt = need;
  }
  const int kend = nkt * BK < a.sk ? nkt * BK : a.sk;
  const int nkt2 = (nkt + 1) & ~1;

  // ---- staging
  // Two register sets: a tile's global loads are issued two iterations before its data is
  // written to LDS, so that their latency (of the order of an iteration) stays hidden.
  struct Stage {
    u32x4 k[CPT], v[CPT];
    T mraw;      // raw per-key mask element (converted when it is written to LDS, so that the
    bool mvalid; // conversion does not wait on the loads issued with it)
  };
  Stage st0, st1;
  st0.mraw = (T)0.f; st0.mvalid = false;
  st1.mraw = (T)0.f; st1.mvalid = false;
  auto gloadK = [&](int tile, Stage &st) {
    const int k0 = tile * BK;
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = tid + i * NT;
      const int row = c / CPR, col = c % CPR;
      // Loads are unconditional (rows past the end re-read the last valid row) so that the
      // number of loads in flight is known at compile time and the wait before the LDS write
      // can leave the younger set outstanding.  Rows past the end need no zeroing: their scores
      // get -inf through the extra step, and finite garbage in V is multiplied by P = 0.
      int kr = k0 + row;
      kr = kr < kend ? kr : kend - 1;
      st.k[i] = *(const u32x4 *)(Kb + (size_t)kr * D + col * 8);
    }
    {
      const int kr = k0 + (tid & (BK - 1));
      st.mvalid = kr < kend;
      if (MASK == kMaskPerKey) st.mraw = mkey[st.mvalid ? kr : kend - 1];
    }
  };
  auto gloadV = [&](int tile, Stage &st) {
    const int k0 = tile * BK;
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = tid + i * NT;
      const int row = c / CPR, col = c % CPR;
      int kr = k0 + row;
      kr = kr < kend ? kr : kend - 1;
      st.v[i] = *(const u32x4 *)(Vb + (size_t)kr * D + col * 8);
    }
  };
  auto lstoreK = [&](int tile, const Stage &st) {
    char *kd = ldsKb + (tile & 1) * TILEB;
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = tid + i * NT;
      const int row = c / CPR, col = c % CPR;
      *(u32x4 *)(kd + row * ROWB + col * 16) = st.k[i];
    }
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
  auto lstoreV = [&](int tile, const Stage &st) {
    char *vd = ldsVb + (tile & 1) * TILEB;
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = tid + i * NT;
      const int row = c / CPR, col = c % CPR;
      *(u32x4 *)(vd + row * ROWB + col * 16) = st.v[i];
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

  // ---- running state
  f32x16 o[QB][DB];
  float mref[QB], lsum[QB];
  bool seen[QB];
  v8 bx[QB];
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
      if (MASK == kMaskFull) bx[qb][3] = (T)a.mask_b;
    }
  }

  // x buffers (accumulators of the first product) with the reference baked into each,
  // and the rounded probabilities of the previous / current tile
  f32x16 xA[QB][NSB], xB[QB][NSB];
  float bkA[QB], bkB[QB];
  v8 pA[QB][NSB][2], pB[QB][NSB][2];

  // first product of `tile` into x, baking the current reference
  auto g1 = [&](int tile, f32x16 (&x)[QB][NSB], float (&bk)[QB]) {
    const char *ldsK = ldsKb + (tile & 1) * TILEB;
    const char *ldsX = ldsXb + (tile & 1) * BK * XROWB;
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) bk[qb] = mref[qb];
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
        const v8 ka = as_v8<T>(*(const u32x4 *)(ldsK + (sb * 32 + ql) * ROWB + ks * 32 + h * 16));
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
          const v8 va = lds_load_a_transposed<T, ROWB>(ldsV, sb * 32, db * 32, c, l);
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) o[qb][db] = E::mfma(va, p[qb][sb][c], o[qb][db]);
        }
  };

  // Both products of one iteration, issued so that consecutive MFMAs never share an
  // accumulator: a dependent MFMA cannot start until its predecessor has drained the
  // matrix pipe (about twice the issue interval), so the four accumulator chains
  // o[.][0], o[.][1], x[.][0], x[.][1] are visited round-robin.
  auto g12 = [&](int tprev, const v8 (&p)[QB][NSB][2], int tnext, f32x16 (&x)[QB][NSB], float (&bk)[QB]) {
    const char *ldsV = ldsVb + (tprev & 1) * TILEB;
    const char *ldsK = ldsKb + (tnext & 1) * TILEB;
    const char *ldsX = ldsXb + (tnext & 1) * BK * XROWB;
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) bk[qb] = mref[qb];
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
      for (int qb = 0; qb < QB; ++qb)
#pragma unroll
        for (int r = 0; r < 16; ++r) x[qb][sb][r] = 0.f;
    constexpr int STEPS2 = NSB * 2;                    // second product: (sb, c) pairs, DB MFMAs each
    constexpr int STEPS1 = KS + 1;                     // first product: contraction steps, NSB MFMAs each
    constexpr int STEPS = STEPS1 > STEPS2 ? STEPS1 : STEPS2;
#pragma unroll
    for (int i = 0; i < STEPS; ++i) {
      if (i < STEPS2) {
        const int sb = i / 2, c = i % 2;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const v8 va = lds_load_a_transposed<T, ROWB>(ldsV, sb * 32, db * 32, c, l);
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) o[qb][db] = E::mfma(va, p[qb][sb][c], o[qb][db]);
        }
      }
      if (i < STEPS1) {
#pragma unroll
        for (int sb = 0; sb < NSB; ++sb) {
          if (i < KS) {
            const v8 ka = as_v8<T>(*(const u32x4 *)(ldsK + (sb * 32 + ql) * ROWB + i * 32 + h * 16));
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) x[qb][sb] = E::mfma(ka, qreg[qb][i], x[qb][sb]);
          } else {
            const v8 xa = as_v8<T>(*(const u32x4 *)(ldsX + (sb * 32 + ql) * XROWB + h * 16));
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) x[qb][sb] = E::mfma(xa, bx[qb], x[qb][sb]);
          }
        }
      }
    }
  };

  // per-element work that cannot go through the matrix pipe: a full mask tensor, the causal test
  auto adjust = [&](int tile, f32x16 (&x)[QB][NSB], auto guarded_tag) {
    constexpr bool GUARDED = decltype(guarded_tag)::value;
    if (MASK == kMaskFull || GUARDED) {
      const int k0 = tile * BK;
      const bool vec_ok = a.mask_vec && (k0 + BK <= a.sk);
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        const int q = q0w + qb * 32 + ql;
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
    }
  };

  // P = exp2(x + shift) rounded to T, and the row sum of the rounded values
  auto exp_pack = [&](const f32x16 (&x)[NSB], float shift, v8 (&pk)[NSB][2]) -> float {
    float rs = 0.f;
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
        for (int j = 0; j < 4; ++j) rs = dot2_ones<T>(pk[sb][c], j, rs);
      }
    }
    return rs;
  };
  auto exp_pack0 = [&](const f32x16 (&x)[NSB], v8 (&pk)[NSB][2]) -> float {
    float rs = 0.f;
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb) {
      float p[16];
#pragma unroll
      for (int r = 0; r < 16; ++r) p[r] = fast_exp2(x[sb][r]);

#pragma unroll
      for (int c = 0; c < 2; ++c) {
#pragma unroll
        for (int j = 0; j < 8; ++j) pk[sb][c][j] = (T)p[8 * c + j];
#pragma unroll
        for (int j = 0; j < 4; ++j) rs = dot2_ones<T>(pk[sb][c], j, rs);
      }
    }
    return rs;
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
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
          for (int t = 0; t < 4; ++t)
            if (!drop_keep_byte(wd[g], t, a.drop.thr)) pk[sb][g >> 1][4 * (g & 1) + t] = (T)0.f;
      }
    }
  };

  // One iteration.  FIRST: tile t is the first tile (no previous second product; the
  // reference is set from this tile before the next first product bakes it).
  // LAST: there is no next tile.
  // stl: register set to load into (K(t+3), V(t+1)); sts: set loaded one iteration ago,
  // written to LDS at the end (K(t+2), V(t)).
  auto body = [&](int t, auto first_tag, auto last_tag, auto guarded_tag, f32x16 (&xc)[QB][NSB], float (&bkc)[QB],
                  f32x16 (&xn)[QB][NSB], float (&bkn)[QB], const v8 (&pprev)[QB][NSB][2], v8 (&pcur)[QB][NSB][2],
                  Stage &stl, const Stage &sts) {
    constexpr bool FIRST = decltype(first_tag)::value;
    constexpr bool LAST = decltype(last_tag)::value;
    if (!LAST) {
      gloadK(t + 3, stl);
      gloadV(t + 1, stl);
    }
    adjust(t, xc, guarded_tag);
    if (FIRST) {
      float shift[QB];
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) shift[qb] = rebase(qb, xc[qb], bkc[qb]);
      if (!LAST) g1(t + 1, xn, bkn);
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        lsum[qb] += exp_pack(xc[qb], shift[qb], pcur[qb]);
        dropout(t, qb, pcur[qb]);
      }
    } else {
      if (LAST) g2(t - 1, pprev);
      else g12(t - 1, pprev, t + 1, xn, bkn);
      float rs[QB];
      bool unfit = false;
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        rs[qb] = exp_pack0(xc[qb], pcur[qb]);
        unfit = unfit | !(rs[qb] < WINDOW) | !seen[qb] | (bkc[qb] != mref[qb]); // no short circuit: keep one basic block
      }
      // Shape of this block for the scheduler: operand reads run a few MFMAs ahead of their
      // use (LDS latency), and every MFMA is followed by a slice of the softmax VALU work.
      {
        constexpr int kMfma = QB * (DB * NSB * 2 + (LAST ? 0 : NSB * (KS + 1)));
        constexpr int kReads = DB * NSB * 2 * 2 + (LAST ? 0 : NSB * (KS + 1));
        constexpr int kValu = QB * NSB * (16 + 8 + 8) + 8;
        constexpr int kAhead = 6;
        constexpr int kValuPer = (kValu + kMfma - 1) / kMfma;
        __builtin_amdgcn_sched_group_barrier(0x100, kAhead, 0);
#pragma unroll
        for (int i = 0; i < kMfma; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          if (kAhead + 2 * i < kReads) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, kValuPer, 0);
        }
      }
      if (__builtin_amdgcn_ballot_w64(unfit) != 0ull) {
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
          const float shift = rebase(qb, xc[qb], bkc[qb]);
          rs[qb] = exp_pack(xc[qb], shift, pcur[qb]);
        }
      }
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        lsum[qb] += rs[qb];
        dropout(t, qb, pcur[qb]);
      }
    }
    if (!LAST) lstoreK(t + 2, sts);
    lstoreV(t, sts);
  };

  // ---- prologue: K(0), K(1) into LDS, first product of tile 0
  gloadK(0, st0);
  gloadK(1, st1);
  gloadV(0, st1);
  // Q' = Q * scale * log2(e) as B-operand registers
#pragma unroll
  for (int qb = 0; qb < QB; ++qb)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const v8 raw = as_v8<T>(qraw[qb][ks]);
#pragma unroll
      for (int j = 0; j < 8; ++j) qreg[qb][ks][j] = (T)((float)raw[j] * a.scale_l2);
    }
  lstoreK(0, st0);
  lstoreK(1, st1);
  gloadK(2, st1); // K(2) joins V(0) in the set that the first iteration writes to LDS
  __syncthreads();
  g1(0, xA, bkA);
  __syncthreads(); // tile 0's K stage is refilled during the first iteration

  using Yes = std::true_type;
  using No = std::false_type;
  // A tile crosses the causal diagonal of this wave iff its last key exceeds the wave's first query.
  auto diag = [&](int t) { return CAUSAL && (t * BK + BK - 1 > q0w); };

  // t = 0
  if (diag(0)) body(0, Yes{}, No{}, Yes{}, xA, bkA, xB, bkB, pB, pA, st0, st1);
  else body(0, Yes{}, No{}, No{}, xA, bkA, xB, bkB, pB, pA, st0, st1);
  __syncthreads();
  // steady state, two tiles per trip so that the buffers keep fixed roles
  for (int t = 1; t < nkt2 - 1; t += 2) {
    if (diag(t)) body(t, No{}, No{}, Yes{}, xB, bkB, xA, bkA, pA, pB, st1, st0);
    else body(t, No{}, No{}, No{}, xB, bkB, xA, bkA, pA, pB, st1, st0);
    __syncthreads();
    if (diag(t + 1)) body(t + 1, No{}, No{}, Yes{}, xA, bkA, xB, bkB, pB, pA, st0, st1);
    else body(t + 1, No{}, No{}, No{}, xA, bkA, xB, bkB, pB, pA, st0, st1);
    __syncthreads();
  }
  // last tile (odd index) and the second product that is still owed
  {
    const int t = nkt2 - 1;
    if (diag(t)) body(t, No{}, Yes{}, Yes{}, xB, bkB, xA, bkA, pA, pB, st1, st0);
    else body(t, No{}, Yes{}, No{}, xB, bkB, xA, bkA, pA, pB, st1, st0);
    __syncthreads();
    g2(t, pB);
  }

  // ---- epilogue
  T *Ob = (T *)a.o + (size_t)bh * a.sq * D;
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
          *(v4 *)(Ob + (size_t)q * D + db * 32 + 8 * g + 4 * h) = t;
        }
      const float cfix = (MASK == kMaskFull) ? a.mask_b - (float)(T)a.mask_b : 0.f;
      if (a.lse && h == 0)
        a.lse[(size_t)bh * a.sq + q] = lt > 0.f ? (mref[qb] + cfix + fast_log2(lt)) * FMHA_LN2 : NEG_INF;
    }
  }
}

} // namespace fmha
