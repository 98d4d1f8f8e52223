// Backward attention kernels for gfx950 (wave64, MFMA 32x32x16).  The reference has no
// backward (its README states forward only); the formulas are the analytic gradient of
//   O = (softmax(scale Q K^T + mask) o Z) V ,  Z = dropout factor (0 or drop_scale):
//   dV = (P o Z)^T dO ;  dPz = dO V^T ;  dP = dPz o Z ;  delta_i = sum_d dO_id O_id
//   dS = P o (dP - delta) ;  dQ = scale dS K ;  dK = scale dS^T Q
// with P recomputed from the saved row log-sum-exp: P = exp(score - LSE).
//
// Two kernels, no atomics, deterministic:
//   fmha_bwd_dq_kernel    one workgroup per (bh, query tile), walks the key tiles;
//                         lane = query, like the forward: S^T = K.Q^T, dP^T = V.dO^T,
//                         dQ^T += K^T.dS^T (K^T through the LDS transpose read).  Also
//                         computes delta for its rows and writes it out.
//   fmha_bwd_dkdv_kernel  one workgroup per (bh, key tile), walks the query tiles with
//                         dK^T / dV^T accumulators resident in registers; lane = key:
//                         S = Q.K^T, dP = dO.V^T, dV^T += dO^T.(P o Z), dK^T += Q^T.dS
//                         (dO^T and Q^T through the LDS transpose read).
// In both, the 32x32 accumulator tile of the score product is converted in registers
// into the B operand of the next product (see fmha_common.h), so P and dS never travel
// through LDS.  The price of avoiding atomics and LDS transposes of dS is that the score
// and dP products are formed in both kernels (7 tile products instead of 5).
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
  float scale_l2, scale, drop_scale;
  DropCtx drop;
  int32_t flags;
};

template <int D> struct BwdCfg {
  static constexpr int BT = 64;           // rows per LDS tile
  static constexpr int NSB = BT / 32;
  static constexpr int KS = D / 16;
  static constexpr int DB = D / 32;
  static constexpr int ROWB = D * 2 + 16;
  static constexpr int TILEB = BT * ROWB;
  static constexpr int LDS_BYTES = 4 * TILEB + 2 * 2 * BT * 4; // two tiles x 2 stages + {lse, delta} x 2 stages
};

// ------------------------------------------------------------------------------ dQ
template <typename T, int D, int QB, int NW, bool MASK, bool CAUSAL, int DROP>
__global__ __launch_bounds__(NW * 64) void fmha_bwd_dq_kernel(const BwdArgs a) {
  using E = Elem<T>;
  using v8 = typename E::v8;
  using v4 = typename E::v4;
  using C = BwdCfg<D>;
  constexpr int BK = C::BT, NSB = C::NSB, KS = C::KS, DB = C::DB, ROWB = C::ROWB, TILEB = C::TILEB;
  constexpr int NT = NW * 64;
  constexpr int QT = NW * QB * 32;
  constexpr int CPR = D / 8;
  constexpr int CPT = BK * CPR / NT;
  constexpr float NEG_INF = -__builtin_inff();
  constexpr float POS_INF = __builtin_inff();

  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int tid = threadIdx.x;
  const int w = tid >> 6, l = tid & 63, ql = l & 31, h = l >> 5;

  int bid = blockIdx.x;
  const int nb = gridDim.x;
  if ((nb & 7) == 0) bid = (bid & 7) * (nb >> 3) + (bid >> 3);
  const int bh = bid / a.ntile;
  int qt = bid - bh * a.ntile;
  if (CAUSAL) qt = a.ntile - 1 - qt;
  const int q0w = qt * QT + w * (QB * 32);

  const T *Qb = (const T *)a.q + (size_t)bh * a.sq * D;
  const T *Ob = (const T *)a.o + (size_t)bh * a.sq * D;
  const T *dOb = (const T *)a.dout + (size_t)bh * a.sq * D;
  const T *Kb = (const T *)a.k + (size_t)bh * a.sk * D;
  const T *Vb = (const T *)a.v + (size_t)bh * a.sk * D;

  // ---- per-row operands: Q and dO as B operands, delta, LSE
  v8 qreg[QB][KS], doreg[QB][KS];
  float delta[QB], lse2[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int q = q0w + qb * 32 + ql;
    float dsum = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      u32x4 tq = {0u, 0u, 0u, 0u}, td = {0u, 0u, 0u, 0u}, to = {0u, 0u, 0u, 0u};
      if (q < a.sq) {
        const size_t off = (size_t)q * D + ks * 16 + h * 8;
        tq = *(const u32x4 *)(Qb + off);
        td = *(const u32x4 *)(dOb + off);
        to = *(const u32x4 *)(Ob + off);
      }
      qreg[qb][ks] = as_v8<T>(tq);
      doreg[qb][ks] = as_v8<T>(td);
      const v8 ov = as_v8<T>(to);
#pragma unroll
      for (int j = 0; j < 8; ++j) dsum = fmaf((float)doreg[qb][ks][j], (float)ov[j], dsum);
    }
    dsum = xhalf_sum(dsum);
    delta[qb] = dsum;
    float ls = POS_INF; // rows past the end and fully masked rows get P = 0
    if (q < a.sq) {
      const float v = a.lse[(size_t)bh * a.sq + q];
      if (v != NEG_INF) ls = v * FMHA_LOG2E;
      if (h == 0) a.delta[(size_t)bh * a.sq + q] = dsum;
    }
    lse2[qb] = ls;
  }

  int nkt = (a.sk + BK - 1) / BK;
  if (CAUSAL) {
    int qmax = qt * QT + QT - 1;
    if (qmax > a.sq - 1) qmax = a.sq - 1;
    const int need = qmax / BK + 1;
    if (need < nkt) nkt = need;
  }

  u32x4 kst[CPT], vst[CPT];
  auto gload = [&](int k0) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = tid + i * NT;
      const int row = c / CPR, col = c % CPR;
      const int kr = k0 + row;
      u32x4 kk = {0u, 0u, 0u, 0u}, vv = {0u, 0u, 0u, 0u};
      if (kr < a.sk) {
        kk = *(const u32x4 *)(Kb + (size_t)kr * D + col * 8);
        vv = *(const u32x4 *)(Vb + (size_t)kr * D + col * 8);
      }
      kst[i] = kk;
      vst[i] = vv;
    }
  };
  auto lstore = [&](int stage) {
    char *kd = lds + stage * 2 * TILEB;
    char *vd = kd + TILEB;
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = tid + i * NT;
      const int row = c / CPR, col = c % CPR;
      *(u32x4 *)(kd + row * ROWB + col * 16) = kst[i];
      *(u32x4 *)(vd + row * ROWB + col * 16) = vst[i];
    }
  };

  const T *mrow[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    int q = q0w + qb * 32 + ql;
    if (q > a.sq - 1) q = a.sq - 1;
    mrow[qb] = nullptr;
    if (MASK) mrow[qb] = (const T *)a.mask + (size_t)(bh / a.mask_div) * a.mask_sb + (size_t)q * a.mask_sq;
  }
  auto load4 = [&](const T *row, int kk, float out[4]) {
    if (a.mask_vec && kk + 3 < a.sk) {
      v4 t = as_v4<T>(*(const u32x2 *)(row + kk));
#pragma unroll
      for (int i = 0; i < 4; ++i) out[i] = (float)t[i];
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) out[i] = (kk + i < a.sk) ? (float)row[kk + i] : 0.f;
    }
  };

  f32x16 dq[QB][DB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb)
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) dq[qb][db][r] = 0.f;

  gload(0);
  lstore(0);
  __syncthreads();

  for (int kt = 0; kt < nkt; ++kt) {
    const int cur = kt & 1;
    const int k0 = kt * BK;
    if (kt + 1 < nkt) gload(k0 + BK);
    const char *ldsK = lds + cur * 2 * TILEB;
    const char *ldsV = ldsK + TILEB;

    const bool active = !CAUSAL || (k0 <= q0w + QB * 32 - 1);
    if (active) {
      f32x16 s[QB][NSB], dp[QB][NSB];
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb) {
#pragma unroll
        for (int qb = 0; qb < QB; ++qb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            s[qb][sb][r] = 0.f;
            dp[qb][sb][r] = 0.f;
          }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const int off = (sb * 32 + ql) * ROWB + ks * 32 + h * 16;
          const v8 ka = as_v8<T>(*(const u32x4 *)(ldsK + off));
          const v8 va = as_v8<T>(*(const u32x4 *)(ldsV + off));
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) {
            s[qb][sb] = E::mfma(ka, qreg[qb][ks], s[qb][sb]);
            dp[qb][sb] = E::mfma(va, doreg[qb][ks], dp[qb][sb]);
          }
        }
      }

      const bool pred = (k0 + BK > a.sk) || (CAUSAL && (k0 + BK - 1 > q0w));
      v8 dsfrag[QB][NSB][2];
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        const int q = q0w + qb * 32 + ql;
#pragma unroll
        for (int sb = 0; sb < NSB; ++sb) {
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int kk = k0 + sb * 32 + 8 * g + 4 * h;
            float mv[4] = {0.f, 0.f, 0.f, 0.f};
            if (MASK) {
              load4(mrow[qb], kk, mv);
#pragma unroll
              for (int t = 0; t < 4; ++t) mv[t] = fmaf(mv[t], a.mask_a, a.mask_b);
            }
            uint32_t wd = 0;
            if (DROP == 1) wd = drop_word(a.drop, (uint32_t)bh, (uint32_t)q, (uint32_t)(kk >> 2));
#pragma unroll
            for (int t = 0; t < 4; ++t) {
              float x = fmaf(s[qb][sb][4 * g + t], a.scale_l2, mv[t]);
              if (pred) {
                const int k = kk + t;
                const bool ok = (k < a.sk) && (!CAUSAL || k <= q);
                x = ok ? x : NEG_INF;
              }
              const float p = fast_exp2(x - lse2[qb]);
              float dpe = dp[qb][sb][4 * g + t];
              if (DROP == 1) dpe = drop_keep_byte(wd, t, a.drop.thr) ? dpe * a.drop_scale : 0.f;
              s[qb][sb][4 * g + t] = p * (dpe - delta[qb]);
            }
          }
        }
#pragma unroll
        for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
          for (int c = 0; c < 2; ++c)
#pragma unroll
            for (int j = 0; j < 8; ++j) dsfrag[qb][sb][c][j] = (T)s[qb][sb][8 * c + j];
      }

      // dQ^T += K^T . dS^T
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
          for (int c = 0; c < 2; ++c) {
            const v8 kt_a = lds_load_a_transposed<T, ROWB>(ldsK, sb * 32, db * 32, c, l);
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) dq[qb][db] = E::mfma(kt_a, dsfrag[qb][sb][c], dq[qb][db]);
          }
    }

    if (kt + 1 < nkt) lstore(cur ^ 1);
    __syncthreads();
  }

  T *dQb = (T *)a.dq + (size_t)bh * a.sq * D;
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int q = q0w + qb * 32 + ql;
    if (q < a.sq) {
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          v4 t;
#pragma unroll
          for (int i = 0; i < 4; ++i) t[i] = (T)(dq[qb][db][4 * g + i] * a.scale);
          *(v4 *)(dQb + (size_t)q * D + db * 32 + 8 * g + 4 * h) = t;
        }
    }
  }
}

// --------------------------------------------------------------------------- dK, dV
template <typename T, int D, int KB, int NW, bool MASK, bool CAUSAL, int DROP>
__global__ __launch_bounds__(NW * 64) void fmha_bwd_dkdv_kernel(const BwdArgs a) {
  using E = Elem<T>;
  using v8 = typename E::v8;
  using v4 = typename E::v4;
  using C = BwdCfg<D>;
  constexpr int BQ = C::BT, NSB = C::NSB, KS = C::KS, DB = C::DB, ROWB = C::ROWB, TILEB = C::TILEB;
  constexpr int NT = NW * 64;
  constexpr int KT = NW * KB * 32;
  constexpr int CPR = D / 8;
  constexpr int CPT = BQ * CPR / NT;
  constexpr float NEG_INF = -__builtin_inff();
  constexpr float POS_INF = __builtin_inff();
  static_assert(NT >= 2 * BQ, "row statistics are staged by the first 2*BQ threads");

  extern __shared__ __attribute__((aligned(16))) char lds[];
  float *ldsStat = (float *)(lds + 4 * TILEB); // [stage][{lse2, delta}][BQ]

  const int tid = threadIdx.x;
  const int w = tid >> 6, l = tid & 63, kl = l & 31, h = l >> 5;

  int bid = blockIdx.x;
  const int nb = gridDim.x;
  if ((nb & 7) == 0) bid = (bid & 7) * (nb >> 3) + (bid >> 3);
  const int bh = bid / a.ntile;
  const int ktile = bid - bh * a.ntile;
  const int k0w = ktile * KT + w * (KB * 32);

  const T *Qb = (const T *)a.q + (size_t)bh * a.sq * D;
  const T *dOb = (const T *)a.dout + (size_t)bh * a.sq * D;
  const T *Kb = (const T *)a.k + (size_t)bh * a.sk * D;
  const T *Vb = (const T *)a.v + (size_t)bh * a.sk * D;
  const float *lseb = a.lse + (size_t)bh * a.sq;
  const float *delb = a.delta + (size_t)bh * a.sq;

  // ---- per-key operands: K and V rows as B operands
  v8 kreg[KB][KS], vreg[KB][KS];
  float mcol[KB];
#pragma unroll
  for (int kb = 0; kb < KB; ++kb) {
    const int key = k0w + kb * 32 + kl;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      u32x4 tk = {0u, 0u, 0u, 0u}, tv = {0u, 0u, 0u, 0u};
      if (key < a.sk) {
        const size_t off = (size_t)key * D + ks * 16 + h * 8;
        tk = *(const u32x4 *)(Kb + off);
        tv = *(const u32x4 *)(Vb + off);
      }
      kreg[kb][ks] = as_v8<T>(tk);
      vreg[kb][ks] = as_v8<T>(tv);
    }
    mcol[kb] = 0.f;
    if (MASK && a.mask_sq == 0 && key < a.sk) // mask constant along queries: one value per lane
      mcol[kb] = fmaf((float)((const T *)a.mask)[(size_t)(bh / a.mask_div) * a.mask_sb + key], a.mask_a, a.mask_b);
  }
  const T *mbase = MASK ? (const T *)a.mask + (size_t)(bh / a.mask_div) * a.mask_sb : nullptr;

  const int nqt = (a.sq + BQ - 1) / BQ;
  const int qt0 = CAUSAL ? (ktile * KT) / BQ : 0; // first query tile that sees any of these keys

  u32x4 qst[CPT], dst[CPT];
  float stat = 0.f;
  auto gload = [&](int q0) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = tid + i * NT;
      const int row = c / CPR, col = c % CPR;
      const int qr = q0 + row;
      u32x4 qq = {0u, 0u, 0u, 0u}, dd = {0u, 0u, 0u, 0u};
      if (qr < a.sq) {
        qq = *(const u32x4 *)(Qb + (size_t)qr * D + col * 8);
        dd = *(const u32x4 *)(dOb + (size_t)qr * D + col * 8);
      }
      qst[i] = qq;
      dst[i] = dd;
    }
    if (tid < BQ) {
      const int qr = q0 + tid;
      float v = POS_INF;
      if (qr < a.sq) {
        const float t = lseb[qr];
        if (t != NEG_INF) v = t * FMHA_LOG2E;
      }
      stat = v;
    } else if (tid < 2 * BQ) {
      const int qr = q0 + tid - BQ;
      stat = qr < a.sq ? delb[qr] : 0.f;
    }
  };
  auto lstore = [&](int stage) {
    char *qd = lds + stage * 2 * TILEB;
    char *dd = qd + TILEB;
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = tid + i * NT;
      const int row = c / CPR, col = c % CPR;
      *(u32x4 *)(qd + row * ROWB + col * 16) = qst[i];
      *(u32x4 *)(dd + row * ROWB + col * 16) = dst[i];
    }
    if (tid < 2 * BQ) ldsStat[stage * 2 * BQ + tid] = stat;
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
    gload(qt0 * BQ);
    lstore(qt0 & 1);
  }
  __syncthreads();

  for (int qt = qt0; qt < nqt; ++qt) {
    const int cur = qt & 1;
    const int q0 = qt * BQ;
    if (qt + 1 < nqt) gload(q0 + BQ);
    const char *ldsQ = lds + cur * 2 * TILEB;
    const char *ldsDO = ldsQ + TILEB;
    const float *ldsL = ldsStat + cur * 2 * BQ;
    const float *ldsDl = ldsL + BQ;

    // queries of this tile all precede this wave's keys: nothing visible under the causal mask
    const bool active = !CAUSAL || (q0 + BQ - 1 >= k0w);
    if (active) {
      f32x16 s[KB][NSB], dp[KB][NSB];
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb) {
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            s[kb][sb][r] = 0.f;
            dp[kb][sb][r] = 0.f;
          }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const int off = (sb * 32 + kl) * ROWB + ks * 32 + h * 16;
          const v8 qa = as_v8<T>(*(const u32x4 *)(ldsQ + off));
          const v8 da = as_v8<T>(*(const u32x4 *)(ldsDO + off));
#pragma unroll
          for (int kb = 0; kb < KB; ++kb) {
            s[kb][sb] = E::mfma(qa, kreg[kb][ks], s[kb][sb]);
            dp[kb][sb] = E::mfma(da, vreg[kb][ks], dp[kb][sb]);
          }
        }
      }

      const bool pred = (q0 + BQ > a.sq) || (k0w + KB * 32 > a.sk) || (CAUSAL && (k0w + KB * 32 - 1 > q0));
      v8 pfrag[KB][NSB][2], dsfrag[KB][NSB][2];
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        const int key = k0w + kb * 32 + kl;
#pragma unroll
        for (int sb = 0; sb < NSB; ++sb) {
          f32x16 pd;
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int qq = sb * 32 + 8 * g + 4 * h; // row in tile of t = 0
            const f32x4 L = *(const f32x4 *)(ldsL + qq);
            const f32x4 Dl = *(const f32x4 *)(ldsDl + qq);
            uint32_t o4[4] = {0u, 0u, 0u, 0u};
            if (DROP == 1) drop_block(a.drop, (uint32_t)bh, (uint32_t)((q0 + qq) >> 2), (uint32_t)(key >> 2), o4);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
              const int q = q0 + qq + t;
              float mv = mcol[kb];
              if (MASK && a.mask_sq != 0) {
                const int qc = q < a.sq ? q : a.sq - 1;
                const int kc = key < a.sk ? key : a.sk - 1;
                mv = fmaf((float)mbase[(size_t)qc * a.mask_sq + kc], a.mask_a, a.mask_b);
              }
              float x = fmaf(s[kb][sb][4 * g + t], a.scale_l2, mv);
              if (pred) {
                const bool ok = (q < a.sq) && (key < a.sk) && (!CAUSAL || key <= q);
                x = ok ? x : NEG_INF;
              }
              const float p = fast_exp2(x - L[t]);
              float dpe = dp[kb][sb][4 * g + t];
              float pz = p;
              if (DROP == 1) {
                const bool keep = drop_keep_byte(o4[t], key & 3, a.drop.thr);
                dpe = keep ? dpe * a.drop_scale : 0.f;
                pz = keep ? p * a.drop_scale : 0.f;
              }
              pd[4 * g + t] = pz;
              s[kb][sb][4 * g + t] = p * (dpe - Dl[t]);
            }
          }
#pragma unroll
          for (int c = 0; c < 2; ++c)
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              pfrag[kb][sb][c][j] = (T)pd[8 * c + j];
              dsfrag[kb][sb][c][j] = (T)s[kb][sb][8 * c + j];
            }
        }
      }

      // dV^T += dO^T . (P o Z) ;  dK^T += Q^T . dS
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
          for (int c = 0; c < 2; ++c) {
            const v8 dot = lds_load_a_transposed<T, ROWB>(ldsDO, sb * 32, db * 32, c, l);
            const v8 qtr = lds_load_a_transposed<T, ROWB>(ldsQ, sb * 32, db * 32, c, l);
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
              dv[kb][db] = E::mfma(dot, pfrag[kb][sb][c], dv[kb][db]);
              dk[kb][db] = E::mfma(qtr, dsfrag[kb][sb][c], dk[kb][db]);
            }
          }
    }

    if (qt + 1 < nqt) lstore(cur ^ 1);
    __syncthreads();
  }

  T *dKb = (T *)a.dk + (size_t)bh * a.sk * D;
  T *dVb = (T *)a.dv + (size_t)bh * a.sk * D;
#pragma unroll
  for (int kb = 0; kb < KB; ++kb) {
    const int key = k0w + kb * 32 + kl;
    if (key < a.sk) {
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          v4 tk, tv;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            tk[i] = (T)(dk[kb][db][4 * g + i] * a.scale);
            tv[i] = (T)dv[kb][db][4 * g + i];
          }
          const size_t off = (size_t)key * D + db * 32 + 8 * g + 4 * h;
          *(v4 *)(dKb + off) = tk;
          *(v4 *)(dVb + off) = tv;
        }
    }
  }
}

} // namespace fmha
