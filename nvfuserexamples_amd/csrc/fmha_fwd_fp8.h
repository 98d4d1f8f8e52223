// Forward attention on 8-bit floating point inputs (OCP e4m3, the format of gfx950's fp8 matrix
// instructions): q, k, v hold e4m3 bytes with one dequantisation factor per tensor, both products run on
// v_mfma_f32_32x32x16_fp8_fp8 with fp32 accumulation, the softmax is fp32, and the probabilities are
// rounded to e4m3 -- unnormalised, in (0, 1] relative to the running row maximum, where e4m3 keeps its
// three mantissa bits down to 2^-6 -- before the second product.  O leaves as fp16 or bf16.  The reference
// is fp16 only (fmha/fmha_manual.cpp:120, Ampere_16_8_16); this is a first, plain (not software-pipelined)
// kernel of the same transposed-product design as the 16-bit ones:
//   S^T = K.Q^T   A = K rows from LDS (8 bytes per lane), B = Q in registers; lane = query
//   O^T = V^T.P^T A = V^T rows from an LDS tile that is written transposed, B = the accumulator tile of
//                 the first product, rounded in place
// Feeding the accumulator tile back needs the eight contraction indices of a lane to be the rows
// {0..3, 8..11} + 4h + 16c of the tile; the first product therefore reads its K rows permuted (row i of
// the tile holds key i with bits 2 and 3 exchanged), which makes those eight rows the CONSECUTIVE keys
// 16c + 8h .. +7: one 8-byte LDS read per operand of the second product, and register r of a lane is key
// 16 (r / 8) + 8h + r % 8 of its 32-key block.
#pragma once
#include "fmha_common.h"

namespace fmha {

struct Fp8Args {
  const uint8_t *q, *k, *v; // e4m3 bytes, [bh, s, d] contiguous
  void *o;                  // [bh, sq, d] fp16 / bf16
  float *lse;               // optional [bh, sq]
  const void *mask;         // optional per-key additive mask in O's element type: mask[(bh / mask_div) * mask_sb + key]
  int64_t mask_sb;
  int32_t mask_div;
  int32_t bh, sq, sk;
  float score_scale_l2;     // scale * descale_q * descale_k * log2(e)
  float out_scale;          // descale_v
};

typedef long i64x1;

template <int D> struct Fp8Cfg {
  static constexpr int NW = 4, NT = NW * 64, QT = NW * 32, BK = 64;
  static constexpr int KPITCH = D + 16;            // bytes per key row of the K tile
  static constexpr int VPITCH = BK + 16;           // bytes per head-dim row of the transposed V tile
  static constexpr int OFF_V = BK * KPITCH;
  static constexpr int OFF_M = OFF_V + D * VPITCH; // mask terms of the tile, fp32
  static constexpr int LDS_BYTES = OFF_M + BK * 4;
};

FMHA_DEV f32x16 mfma_fp8(long a, long b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(a, b, c, 0, 0, 0); }

// Eight floats to eight e4m3 bytes (round to nearest even), element 0 in the lowest byte.
FMHA_DEV long pack8_e4m3(const float *p) {
  int lo = 0, hi = 0;
  lo = __builtin_amdgcn_cvt_pk_fp8_f32(p[0], p[1], lo, false);
  lo = __builtin_amdgcn_cvt_pk_fp8_f32(p[2], p[3], lo, true);
  hi = __builtin_amdgcn_cvt_pk_fp8_f32(p[4], p[5], hi, false);
  hi = __builtin_amdgcn_cvt_pk_fp8_f32(p[6], p[7], hi, true);
  return (long)(((unsigned long)(uint32_t)hi << 32) | (uint32_t)lo);
}

template <typename TO, int D, bool CAUSAL, bool MASK>
__global__ __launch_bounds__(Fp8Cfg<D>::NT) void fmha_fwd_fp8_kernel(const Fp8Args a) {
  using C = Fp8Cfg<D>;
  constexpr int NT = C::NT, QT = C::QT, BK = C::BK, KS = D / 16, DB = D / 32;
  constexpr int CPR = D / 16;            // 16-byte chunks per row
  constexpr int CPT = BK * CPR / NT;     // chunks per thread and tile
  static_assert(CPT >= 1, "tile must cover the workgroup");
  constexpr float NEG_INF = -__builtin_inff();

  extern __shared__ __attribute__((aligned(16))) char lds[];
  char *ldsK = lds;
  char *ldsV = lds + C::OFF_V;
  float *ldsM = (float *)(lds + C::OFF_M);

  const int tid = threadIdx.x;
  const int w = tid >> 6, l = tid & 63, ql = l & 31, h = l >> 5;
  const int nqt = (a.sq + QT - 1) / QT;
  const int bh = blockIdx.x / nqt, qt = blockIdx.x % nqt;
  const int q = qt * QT + w * 32 + ql;
  const int qc = q < a.sq ? q : a.sq - 1;

  const uint8_t *Qb = a.q + (size_t)bh * a.sq * D;
  const uint8_t *Kb = a.k + (size_t)bh * a.sk * D;
  const uint8_t *Vb = a.v + (size_t)bh * a.sk * D;
  const TO *mkey = MASK ? (const TO *)a.mask + (size_t)(bh / a.mask_div) * a.mask_sb : nullptr;

  // Q as the B operand: column = this lane's query, contraction bytes 16 ks + 8h .. +7
  long qreg[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) qreg[ks] = *(const long *)(Qb + (size_t)qc * D + ks * 16 + h * 8);

  int nkt = (a.sk + BK - 1) / BK;
  if (CAUSAL) {
    int qmax = qt * QT + QT - 1;
    if (qmax > a.sq - 1) qmax = a.sq - 1;
    const int need = qmax / BK + 1;
    if (need < nkt) nkt = need;
  }

  // tile staging: global -> registers -> LDS (K as it is, V transposed byte by byte)
  u32x4 kst[CPT], vst[CPT];
  float mst = 0.f;
  auto gload = [&](int k0) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = tid + i * NT, row = c / CPR, col = c % CPR;
      int kr = k0 + row;
      kr = kr < a.sk ? kr : a.sk - 1; // keys past the end re-read the last row; their scores are -inf
      kst[i] = *(const u32x4 *)(Kb + (size_t)kr * D + col * 16);
      vst[i] = *(const u32x4 *)(Vb + (size_t)kr * D + col * 16);
    }
    if (tid < BK) {
      const int kr = k0 + tid;
      mst = kr < a.sk ? 0.f : NEG_INF;
      if (MASK && kr < a.sk) mst = (float)mkey[kr] * FMHA_LOG2E;
    }
  };
  auto lstore = [&]() {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = tid + i * NT, row = c / CPR, col = c % CPR;
      *(u32x4 *)(ldsK + row * C::KPITCH + col * 16) = kst[i];
      union { u32x4 u; uint8_t b[16]; } cv;
      cv.u = vst[i];
#pragma unroll
      for (int j = 0; j < 16; ++j) ldsV[(col * 16 + j) * C::VPITCH + row] = (char)cv.b[j];
    }
    if (tid < BK) ldsM[tid] = mst;
  };

  // row i of a 32-key block of the first product holds key i with bits 2 and 3 exchanged
  const int krow = (ql & 0x13) | ((ql & 4) << 1) | ((ql & 8) >> 1);

  f32x16 oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;
  float m_run = NEG_INF, l_run = 0.f;

  gload(0);
  for (int kt = 0; kt < nkt; ++kt) {
    const int k0 = kt * BK;
    __syncthreads(); // the previous tile has been consumed
    lstore();
    __syncthreads();
    if (kt + 1 < nkt) gload(k0 + BK);

    // S^T = K.Q^T for the two 32-key blocks of the tile
    f32x16 x[2];
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
#pragma unroll
      for (int r = 0; r < 16; ++r) x[sb][r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const long ka = *(const long *)(ldsK + (sb * 32 + krow) * C::KPITCH + ks * 16 + h * 8);
        x[sb] = mfma_fp8(ka, qreg[ks], x[sb]);
      }
    }
    // scores in log2 units plus the mask term; register r of block sb is key k0 + 32 sb + 16 (r / 8) + 8h + r % 8
    float mx = NEG_INF;
#pragma unroll
    for (int sb = 0; sb < 2; ++sb)
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        const int kk = sb * 32 + 16 * c + 8 * h;
        const f32x4 m0 = *(const f32x4 *)(ldsM + kk), m1 = *(const f32x4 *)(ldsM + kk + 4);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float v = fmaf(x[sb][8 * c + e], a.score_scale_l2, e < 4 ? m0[e] : m1[e - 4]);
          if (CAUSAL) v = (k0 + kk + e <= q) ? v : NEG_INF;
          x[sb][8 * c + e] = v;
          mx = fmaxf(mx, v);
        }
      }
    mx = xhalf_max(mx);
    const float m_new = fmaxf(m_run, mx);
    // a row that has seen no key yet keeps everything at zero (exp2(-inf - -inf) must not appear)
    const float m_use = m_new == NEG_INF ? 0.f : m_new;
    const float alpha = fast_exp2(m_run - m_use); // 0 on the first live tile
    float psum = 0.f;
    long pb[2][2];
#pragma unroll
    for (int sb = 0; sb < 2; ++sb)
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        float p[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          p[e] = fast_exp2(x[sb][8 * c + e] - m_use);
          psum += p[e];
        }
        pb[sb][c] = pack8_e4m3(p);
      }
    psum = xhalf_sum(psum);
    l_run = l_run * alpha + psum;
    m_run = m_new;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;
    // O^T += V^T.P^T
#pragma unroll
    for (int sb = 0; sb < 2; ++sb)
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const long va = *(const long *)(ldsV + (db * 32 + ql) * C::VPITCH + sb * 32 + 16 * c + 8 * h);
          oacc[db] = mfma_fp8(va, pb[sb][c], oacc[db]);
        }
  }

  // normalise and store: in the accumulator layout lane (q, h) holds head-dim columns 8g + 4h .. +3 of each 32-block
  if (q < a.sq) {
    const float inv = l_run > 0.f ? a.out_scale / l_run : 0.f;
    TO *Or = (TO *)a.o + ((size_t)bh * a.sq + q) * D;
#pragma unroll
    for (int db = 0; db < DB; ++db) store_acc_block_row<TO>(Or + db * 32, oacc[db], inv, h);
    if (a.lse && h == 0) a.lse[(size_t)bh * a.sq + q] = l_run > 0.f ? (m_run + fast_log2(l_run)) * FMHA_LN2 : NEG_INF;
  }
}

} // namespace fmha
