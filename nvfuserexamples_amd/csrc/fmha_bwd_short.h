// Backward kernel for short sequences (sq and sk <= 128, or <= 256; head dim 64; no mask, a per-key mask
// and / or the causal mask): one workgroup per
// head, one launch, every tensor crosses HBM once.
//
// At these shapes the backward is mostly memory time (BH 512, S 128: 5.4 GFLOP against 67 MB), and a head's
// Q, K, V and dO fit in LDS together (64 KB; 128 KB at 256 rows).  The general path launches two kernels that each
// read the head again; here the workgroup copies the four matrices into LDS once and then runs the
// same two computations back to back on them:
//   phase 1  lane = query (a wave owns 32 queries, walks the key blocks):
//            x^T = K.Q^T, g^T = V.dO^T, dS^T, dQ^T += K^T.dS^T   -> dQ complete per wave
//   phase 2  lane = key (a wave owns 32 keys, walks the query blocks):
//            x = Q.K^T, g = dO.V^T, dV^T += dO^T.(P o Z), dK^T += Q^T.dS   -> dK, dV complete per wave
// so no partial result ever leaves a wave: no atomics, no reduction through LDS, deterministic.
// The score and dP products are formed twice (7 tile products instead of 5), which costs matrix
// time the memory system leaves idle anyway.  Scale, mask, log-sum-exp and delta are applied in
// fp32 on the accumulators (no extra contraction step: the VALU is not what bounds this kernel).
// Formulas and the dropout rule as in fmha_bwd_kernel.h.
#pragma once
#include "fmha_bwd_kernel.h"

namespace fmha {

// SMAX_: queries and keys per head, 128 (4 waves, 66 KB of LDS: two workgroups per CU) or 256 (8 waves,
// 131 KB: one workgroup per CU).
template <int SMAX_> struct BwdShortCfg {
  static constexpr int D = 64;
  static constexpr int SMAX = SMAX_;
  static constexpr int NW = SMAX / 32;              // a wave per 32 queries (phase 1) / 32 keys (phase 2)
  static constexpr int NB = SMAX / 32;              // 32-row blocks per matrix
  static constexpr int BT = 64;                     // rows per swizzled LDS tile
  static constexpr int NTL = SMAX / BT;             // tiles per matrix
  static constexpr int TILEB = BT * D * 2;
  static constexpr int LDS_BYTES = 4 * NTL * TILEB + 3 * SMAX * 4; // Q, K, V, dO; delta, LSE, mask term
};

template <typename T, int DROP, int SMAX, bool CAUSAL, bool STRIDED>
__global__ __launch_bounds__(BwdShortCfg<SMAX>::NW * 64) __attribute__((amdgpu_waves_per_eu(2, 2)))
void fmha_bwd_short_kernel(const BwdArgs a) {
  using RW = Rows<STRIDED, BwdShortCfg<SMAX>::D>;
  using E = Elem<T>;
  using v8 = typename E::v8;
  using C = BwdShortCfg<SMAX>;
  constexpr int D = C::D, KS = D / 16, DB = D / 32, NT = C::NW * 64, TILEB = C::TILEB, BT = C::BT, NTL = C::NTL;
  constexpr float NEG_INF = -__builtin_inff();
  constexpr float BIG = 3.0e38f;

  extern __shared__ __attribute__((aligned(16))) char lds[];
  char *ldsQ = lds, *ldsK = lds + NTL * TILEB, *ldsV = lds + 2 * NTL * TILEB, *ldsDO = lds + 3 * NTL * TILEB;
  float *fD = (float *)(lds + 4 * NTL * TILEB); // delta[q]
  float *fL = fD + C::SMAX;               // LSE[q] in log2 units; +BIG for rows that must give P = 0
  float *fM = fL + C::SMAX;               // mask term of key k in log2 units; -inf past the valid keys

  const int tid = threadIdx.x;
  const int w = tid >> 6;
  const int l = tid & 63;
  const int ql = l & 31;
  const int h = l >> 5;
  const int bh = blockIdx.x;
  const int kend = bwd_valid_keys(a, bh);

  const T *Qb = (const T *)a.q + RW::head(a.mq, bh, a.sq);
  const T *Kb = (const T *)a.k + RW::head(a.mk, bh, a.sk);
  const T *Vb = (const T *)a.v + RW::head(a.mv, bh, a.sk);
  const T *Ob = (const T *)a.o + RW::head(a.mo, bh, a.sq);
  const T *dOb = (const T *)a.dout + RW::head(a.mdo, bh, a.sq);

  // ---- the head's four matrices: global -> LDS, all requests up front
  TileCopy<T, D, BT, NT> cq, ck, cdo; // rows of Q, of K and V (equally far apart), of dO
  cq.init(tid, RW::ss(a.mq));
  ck.init(tid, RW::ss(a.mk));
  cdo.init(tid, RW::ss(a.mdo));
  const uint32_t lds0 = lds_address(lds);
#pragma unroll
  for (int t = 0; t < NTL; ++t) {
    if (t * BT < a.sq) {
      cq.issue(Qb, t * BT, a.sq, lds0 + t * TILEB, tid);
      cdo.issue(dOb, t * BT, a.sq, lds0 + (3 * NTL + t) * TILEB, tid);
    }
    if (t * BT < a.sk) {
      ck.issue(Kb, t * BT, a.sk, lds0 + (NTL + t) * TILEB, tid);
      ck.issue(Vb, t * BT, a.sk, lds0 + (2 * NTL + t) * TILEB, tid);
    }
  }
  // this lane's part of its query's O row (for delta), in the layout of a B operand
  const int q1 = w * 32 + ql; // phase 1: the lane's query
  v8 oreg[KS];
  {
    const int q = q1 < a.sq ? q1 : a.sq - 1;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) oreg[ks] = as_v8<T>(*(const u32x4 *)(Ob + (size_t)q * RW::ss(a.mo) + ks * 16 + h * 8));
  }
  if (tid < C::SMAX) {
    float lq = BIG; // rows past the end and rows that saw no key: P = 0
    if (tid < a.sq) {
      const float ls = a.lse[(size_t)bh * a.sq + tid];
      if (ls != NEG_INF) lq = ls * FMHA_LOG2E;
    }
    fL[tid] = lq;
    float mk = NEG_INF;
    if (tid < kend) {
      mk = 0.f;
      if (a.mask) mk = fmaf((float)((const T *)a.mask)[(size_t)(bh / a.mask_div) * a.mask_sb + tid], a.mask_a, a.mask_b);
    }
    fM[tid] = mk;
  }
  dma_wait_all();
  __syncthreads();

  PanelLane pl;
  pl.init(l);

  // =============================================================== phase 1: dQ (lane = query)
  float delta = 0.f;
  if (w * 32 < a.sq) { // wave-uniform
    const char *tQ = ldsQ + (w >> 1) * TILEB, *tDO = ldsDO + (w >> 1) * TILEB;
    v8 qreg[KS], doreg[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      qreg[ks] = panel_read_rows<T, BT>(tQ, pl, w & 1, ks);
      doreg[ks] = panel_read_rows<T, BT>(tDO, pl, w & 1, ks);
#pragma unroll
      for (int j = 0; j < 8; ++j) delta = fmaf((float)oreg[ks][j], (float)doreg[ks][j], delta);
    }
    delta = xhalf_sum(delta);
    const float lq = fL[q1];
    f32x16 dq[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) dq[db][r] = 0.f;

#pragma unroll
    for (int sb = 0; sb < C::NB; ++sb) {
      // causal (key <= query): key blocks above the wave's queries contribute nothing
      if (sb * 32 < a.sk && (!CAUSAL || sb <= w)) {
        const char *tK = ldsK + (sb >> 1) * TILEB, *tV = ldsV + (sb >> 1) * TILEB;
        f32x16 x, g;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          x[r] = 0.f;
          g[r] = 0.f;
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          x = E::mfma(panel_read_rows<T, BT>(tK, pl, sb & 1, ks), qreg[ks], x);
          g = E::mfma(panel_read_rows<T, BT>(tV, pl, sb & 1, ks), doreg[ks], g);
        }
        uint32_t wd[4] = {0u, 0u, 0u, 0u};
        if (DROP == 1) drop_words_q(a.drop, (uint32_t)bh, (uint32_t)q1, (uint32_t)(sb * 32), h, l, wd);
        v8 dsfrag[2];
#pragma unroll
        for (int gq = 0; gq < 4; ++gq) {
          const f32x4 mk = *(const f32x4 *)(fM + sb * 32 + 8 * gq + 4 * h);
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            float p = fast_exp2(fmaf(x[4 * gq + t], a.scale_l2, mk[t]) - lq);
            if (CAUSAL) p = (sb * 32 + 8 * gq + 4 * h + t <= q1) ? p : 0.f;
            float gv = g[4 * gq + t] - delta;
            if (DROP == 1)
              gv = drop_keep_byte(wd[gq], t, a.drop.thr) ? fmaf(g[4 * gq + t], a.drop_scale, -delta) : -delta;
            dsfrag[gq >> 1][4 * (gq & 1) + t] = (T)(p * gv);
          }
        }
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
          for (int db = 0; db < DB; ++db)
            dq[db] = E::mfma(panel_read_transposed<T, BT>(tK, pl, sb & 1, db, c), dsfrag[c], dq[db]);
      }
    }
    if (q1 < a.sq) {
      T *dQr = (T *)a.dq + RW::head(a.mdq, bh, a.sq) + (size_t)q1 * RW::ss(a.mdq);
#pragma unroll
      for (int db = 0; db < DB; ++db) store_acc_block_row<T>(dQr + db * 32, dq[db], a.scale, h);
      if (h == 0) a.delta[(size_t)bh * a.sq + q1] = delta;
    }
  }
  if (h == 0) fD[q1] = delta; // (zero for waves without queries; those rows have P = 0 anyway)
  __syncthreads();

  // =============================================================== phase 2: dK, dV (lane = key)
  const int key = w * 32 + ql;
  if (w * 32 < a.sk) { // wave-uniform
    const char *tK = ldsK + (w >> 1) * TILEB, *tV = ldsV + (w >> 1) * TILEB;
    v8 kreg[KS], vreg[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      kreg[ks] = panel_read_rows<T, BT>(tK, pl, w & 1, ks);
      vreg[ks] = panel_read_rows<T, BT>(tV, pl, w & 1, ks);
    }
    const float mk = fM[key];
    f32x16 dk[DB], dv[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        dk[db][r] = 0.f;
        dv[db][r] = 0.f;
      }
#pragma unroll
    for (int qb = 0; qb < C::NB; ++qb) {
      // causal: query blocks below the wave's keys see none of them
      if (qb * 32 < a.sq && (!CAUSAL || qb >= w)) {
        const char *tQ = ldsQ + (qb >> 1) * TILEB, *tDO = ldsDO + (qb >> 1) * TILEB;
        f32x16 x, g;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          x[r] = 0.f;
          g[r] = 0.f;
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          x = E::mfma(panel_read_rows<T, BT>(tQ, pl, qb & 1, ks), kreg[ks], x);
          g = E::mfma(panel_read_rows<T, BT>(tDO, pl, qb & 1, ks), vreg[ks], g);
        }
        uint32_t rb[4]; // rb[t], byte gq: the random byte of (query 8 gq + 4h + t of the block, this lane's key)
        if (DROP == 1) drop_bytes_k(a.drop, (uint32_t)bh, (uint32_t)(qb * 32), (uint32_t)key, h, l, rb);
        v8 pfrag[2], dsfrag[2];
#pragma unroll
        for (int gq = 0; gq < 4; ++gq) {
          const int qq = qb * 32 + 8 * gq + 4 * h;
          const f32x4 Dl = *(const f32x4 *)(fD + qq);
          const f32x4 Ll = *(const f32x4 *)(fL + qq);
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            float p = fast_exp2(fmaf(x[4 * gq + t], a.scale_l2, mk) - Ll[t]);
            if (CAUSAL) p = (key <= qq + t) ? p : 0.f;
            float gv = g[4 * gq + t] - Dl[t];
            float pz = p;
            if (DROP == 1) {
              const bool keep = drop_keep_byte(rb[t], gq, a.drop.thr);
              gv = keep ? fmaf(g[4 * gq + t], a.drop_scale, -Dl[t]) : -Dl[t];
              pz = keep ? p : 0.f; // (drop_scale multiplies dV once, on store)
            }
            pfrag[gq >> 1][4 * (gq & 1) + t] = (T)pz;
            dsfrag[gq >> 1][4 * (gq & 1) + t] = (T)(p * gv);
          }
        }
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
          for (int db = 0; db < DB; ++db) {
            dv[db] = E::mfma(panel_read_transposed<T, BT>(tDO, pl, qb & 1, db, c), pfrag[c], dv[db]);
            dk[db] = E::mfma(panel_read_transposed<T, BT>(tQ, pl, qb & 1, db, c), dsfrag[c], dk[db]);
          }
      }
    }
    if (key < a.sk) {
      T *dKr = (T *)a.dk + RW::head(a.mdk, bh, a.sk) + (size_t)key * RW::ss(a.mdk);
      T *dVr = (T *)a.dv + RW::head(a.mdv, bh, a.sk) + (size_t)key * RW::ss(a.mdv);
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        store_acc_block_row<T>(dKr + db * 32, dk[db], a.scale, h);
        store_acc_block_row<T>(dVr + db * 32, dv[db], DROP == 1 ? a.drop_scale : 1.f, h);
      }
    }
  }
}

} // namespace fmha
