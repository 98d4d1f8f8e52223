// Forward attention on 8-bit floating point inputs (OCP e4m3): q, k, v hold e4m3 bytes with one
// dequantisation factor per tensor, both products run on v_mfma_f32_32x32x64_f8f6f4 (the K = 64 form, the
// only fp8 matrix instruction that runs at twice the 16-bit rate) with fp32 accumulation, the softmax is
// fp32, and the probabilities are rounded to e4m3 -- unnormalised, relative to an integer reference exponent
// near the row maximum, where e4m3 keeps its three mantissa bits down to 2^-6 -- before the second product.  O leaves as
// fp16 or bf16.  The reference is fp16 only (fmha/fmha_manual.cpp:120, Ampere_16_8_16).  Same
// transposed-product design as the 16-bit kernels, on a plain double-buffered loop:
//   S^T = K.Q^T   A = K rows from LDS (32 bytes per lane: keys l % 32, head-dim bytes 32 (l / 32) .. +31),
//                 B = Q in registers; lane = query
//   O^T = V^T.P^T A = V^T through the 8-bit LDS transpose read (ds_read_b64_tr_b8) from a V tile kept as it
//                 is in memory, B = the two accumulator tiles of the first product, rounded in place
// Feeding the accumulator tiles back: a lane's 32 contraction bytes are its 16 registers of key block 0, then
// of key block 1; register r of a lane (q, h) is key 8 (r / 4) + 4h + r % 4 of its block, so contraction byte
// j = 16 b + r of half-wave h stands for key 32 b + 8 (r / 4) + 4 h + r % 4, and the V^T operand is fetched in
// that order: transpose read (b, gp) covers the rows 32 b + 16 gp + 4 h + {0,1,2,3, 8,9,10,11}.
// As in the 16-bit kernels the per-element vector work is what bounds the kernel (the fp8 products take a
// quarter of its time), so everything that is a rank-one term rides in the matrix pipe: after the fp8 product
// one bf16 32x32x16 step adds  (mask[key] - M[q]) / s  to the raw scores, with
//   A row of a key   (1, 1, 1, mk_hi, mk_mid, mk_lo, 0, 0)      mk = mask term / s, "-inf" for keys past the end
//   B col of a query (-Mr_hi, -Mr_mid, -Mr_lo, 1, 1, 1, 0, 0)   Mr = M / s
// (three bf16 pieces each: exact to fp32), s = scale * descale_q * descale_k * log2(e).  Then P = exp2(s x): one
// multiply, one exponential and half a conversion per element.  The row sums come out of the matrix pipe too:
// one more fp8 product of the rounded tile with an operand of ones gives every lane the sum of ITS row's
// rounded probabilities, so O = sum P~ v / sum P~ is a convex combination of the values (a row with one
// dominant key reproduces that key's value exactly, whatever the rounding did to its probability).  The row
// log-sum-exp, where the caller wants it, is accumulated from the unrounded probabilities (one add per element,
// in that case only).  M is the row's reference exponent, an INTEGER in log2 units, so that changing it
// rescales every probability by an exact power of two and the e4m3 rounding of P does not depend on when a
// maximum was met.  It is not a running maximum: it is set from the first tile a row sees (ceil of that tile's
// maximum) and raised only when a tile's row sum leaves the range in which no probability can exceed the e4m3
// range (sum of the rounded values > 256; a saturated 448 or a NaN fails the same test), the rare slow path
// that also rescales the accumulators; a common tile computes no maximum at all.
// ds_read_b64_tr_b8, as measured on the device: the 16 lanes of a group cover 8 rows x 16 byte columns; lane i
// supplies the address of row i / 2, byte columns 8 (i % 2) .. +7, and receives column i, rows 0..7.
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
  float score_scale_l2;     // s = scale * descale_q * descale_k * log2(e)
  float inv_score_scale_l2; // 1 / s
  float out_scale;          // descale_v
};

typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef int i32x2v __attribute__((ext_vector_type(2)));

template <int D> struct Fp8Cfg {
  static constexpr int NW = 4, NT = NW * 64, QT = NW * 32, BK = 64;
  static constexpr int PITCH = D + 16;              // bytes per key row of the K and V tiles (16 rows, 16 bank groups)
  static constexpr int TILEB = BK * PITCH;
  static constexpr int XROWB = 32;                   // extra-step row of a key: 16 bf16
  static constexpr int STAGEB = 2 * TILEB + BK * XROWB; // K tile, V tile, extra-step rows of the tile
  static constexpr int LDS_BYTES = 2 * STAGEB;
};

// 32x32 += (32 x 64 e4m3) . (64 x 32 e4m3); format selectors 0 = e4m3 for both operands, no block scaling
FMHA_DEV f32x16 mfma_fp8_k64(i32x8 a, i32x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}
FMHA_DEV i32x2v lds_read_tr8(const char *lds_ptr) {
  typedef __attribute__((address_space(3))) i32x2v lds_vec;
  return __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_vec *)(lds_ptr));
}

// Four floats to four e4m3 bytes (round to nearest even), element 0 in the lowest byte.
FMHA_DEV int pack4_e4m3(float a, float b, float c, float d) {
  int w = 0;
  w = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, w, false);
  w = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, w, true);
  return w;
}

// v = hi + mid + lo in bf16 pieces (24 bits together)
FMHA_DEV void split3_bf16(float v, __bf16 &hi, __bf16 &mid, __bf16 &lo) {
  hi = (__bf16)v;
  const float r = v - (float)hi;
  mid = (__bf16)r;
  lo = (__bf16)(r - (float)mid);
}

template <typename TO, int D, bool CAUSAL, bool MASK>
__global__ __launch_bounds__(Fp8Cfg<D>::NT) void fmha_fwd_fp8_kernel(const Fp8Args a) {
  using C = Fp8Cfg<D>;
  constexpr int NT = C::NT, QT = C::QT, BK = C::BK, DS = D / 64, DB = D / 32, PITCH = C::PITCH, XROWB = C::XROWB;
  constexpr int CPR = D / 16;            // 16-byte chunks per row
  constexpr int CPT = BK * CPR / NT;     // chunks per thread and tile
  static_assert(CPT >= 1, "tile must cover the workgroup");
  constexpr float NEG_INF = -__builtin_inff();
  constexpr float SUM_LIMIT = 256.f;     // a row sum up to here: every probability fits e4m3 (maximum 448)

  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int tid = threadIdx.x;
  const int w = tid >> 6, l = tid & 63, ql = l & 31, h = l >> 5;
  const int nqt = (a.sq + QT - 1) / QT;
  const int bh = blockIdx.x / nqt, qt = blockIdx.x % nqt;
  const int q = qt * QT + w * 32 + ql;
  const int qc = q < a.sq ? q : a.sq - 1;
  const float s = a.score_scale_l2, inv_s = a.inv_score_scale_l2;
  // a masked key's term in raw score units: -1e25 in log2 units whatever the scale (kept inside the bf16 range)
  const float BIGNEG_RAW = -fminf(1e25f * inv_s, 1e37f);

  const uint8_t *Qb = a.q + (size_t)bh * a.sq * D;
  const uint8_t *Kb = a.k + (size_t)bh * a.sk * D;
  const uint8_t *Vb = a.v + (size_t)bh * a.sk * D;
  const TO *mkey = MASK ? (const TO *)a.mask + (size_t)(bh / a.mask_div) * a.mask_sb : nullptr;

  // Q as the B operand: column = this lane's query, contraction bytes 64 ds + 32 h .. +31
  i32x8 qreg[DS];
#pragma unroll
  for (int ds = 0; ds < DS; ++ds) {
    const u32x4 lo = *(const u32x4 *)(Qb + (size_t)qc * D + ds * 64 + h * 32);
    const u32x4 hi = *(const u32x4 *)(Qb + (size_t)qc * D + ds * 64 + h * 32 + 16);
    qreg[ds] = i32x8{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
  }

  int nkt = (a.sk + BK - 1) / BK;
  if (CAUSAL) {
    int qmax = qt * QT + QT - 1;
    if (qmax > a.sq - 1) qmax = a.sq - 1;
    const int need = qmax / BK + 1;
    if (need < nkt) nkt = need;
  }

  // tile staging: global -> registers -> LDS, both tiles as they are in memory; two LDS stages
  u32x4 kst[CPT], vst[CPT];
  float mst = 0.f; // mask term of this thread's key in raw score units
  auto gload = [&](int k0) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = tid + i * NT, row = c / CPR, col = c % CPR;
      int kr = k0 + row;
      kr = kr < a.sk ? kr : a.sk - 1; // keys past the end re-read the last row; their mask term is "-inf"
      kst[i] = *(const u32x4 *)(Kb + (size_t)kr * D + col * 16);
      vst[i] = *(const u32x4 *)(Vb + (size_t)kr * D + col * 16);
    }
    if (tid < BK) {
      const int kr = k0 + tid;
      mst = kr < a.sk ? 0.f : BIGNEG_RAW;
      if (MASK && kr < a.sk) {
        const float mk = (float)mkey[kr];
        mst = mk == NEG_INF ? BIGNEG_RAW : fmaxf(mk * (FMHA_LOG2E * inv_s), BIGNEG_RAW);
      }
    }
  };
  auto lstore = [&](int stage) {
    char *kd = lds + stage * C::STAGEB;
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = tid + i * NT, row = c / CPR, col = c % CPR;
      *(u32x4 *)(kd + row * PITCH + col * 16) = kst[i];
      *(u32x4 *)(kd + C::TILEB + row * PITCH + col * 16) = vst[i];
    }
    if (tid < BK) { // (1, 1, 1, mk_hi, mk_mid, mk_lo, 0 ...)
      bf16x8 r0, z;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        r0[j] = (__bf16)0.f;
        z[j] = (__bf16)0.f;
      }
      r0[0] = r0[1] = r0[2] = (__bf16)1.f;
      __bf16 hi, mid, lo;
      split3_bf16(mst, hi, mid, lo);
      r0[3] = hi;
      r0[4] = mid;
      r0[5] = lo;
      bf16x8 *dst = (bf16x8 *)(kd + 2 * C::TILEB + tid * XROWB);
      dst[0] = r0;
      dst[1] = z;
    }
  };

  // transpose-read address of this lane inside a V tile: row 4h + {0,1,2,3, 8,9,10,11}[i16 / 2], byte column
  // (ql & 16) + 8 (i16 % 2) of a 32-column block
  const int i16 = l & 15;
  const int trofs = (4 * h + (i16 >> 1) + ((i16 >> 1) >= 4 ? 4 : 0)) * PITCH + (ql & 16) + 8 * (i16 & 1);

  f32x16 oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;
  float M = 0.f, l_run = 0.f, l_true = 0.f; // reference exponent (an integer); sums of the rounded / unrounded probabilities relative to it
  bool seen = false;          // M has been set from a tile with a live key
  bf16x8 bx;                  // extra-step column of this lane's query
  auto set_bx = [&]() {
#pragma unroll
    for (int j = 0; j < 8; ++j) bx[j] = (__bf16)0.f;
    if (h == 0) {
      __bf16 hi, mid, lo;
      split3_bf16(-M * inv_s, hi, mid, lo);
      bx[0] = hi;
      bx[1] = mid;
      bx[2] = lo;
      bx[3] = bx[4] = bx[5] = (__bf16)1.f;
    }
  };
  set_bx();

  gload(0);
  lstore(0);
  if (nkt > 1) gload(BK);
  __syncthreads();

  for (int kt = 0; kt < nkt; ++kt) {
    const int k0 = kt * BK;
    const char *ldsK = lds + (kt & 1) * C::STAGEB;
    const char *ldsV = ldsK + C::TILEB;
    const char *ldsX = ldsK + 2 * C::TILEB;

    // x = K.Q^T + (mask[key] - M[q]) / s  for the two 32-key blocks of the tile
    f32x16 x[2];
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
#pragma unroll
      for (int r = 0; r < 16; ++r) x[sb][r] = 0.f;
#pragma unroll
      for (int ds = 0; ds < DS; ++ds) {
        const char *kp = ldsK + (sb * 32 + ql) * PITCH + ds * 64 + h * 32;
        const u32x4 lo = *(const u32x4 *)kp, hi = *(const u32x4 *)(kp + 16);
        const i32x8 ka = {(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
        x[sb] = mfma_fp8_k64(ka, qreg[ds], x[sb]);
      }
      const bf16x8 xa = as_v8<__bf16>(*(const u32x4 *)(ldsX + (sb * 32 + ql) * XROWB + h * 16));
      x[sb] = Elem<__bf16>::mfma(xa, bx, x[sb]);
    }
    // the next tile goes to the other stage while this one is worked on (its last readers passed the barrier
    // that ended the previous iteration)
    if (kt + 1 < nkt) {
      lstore((kt + 1) & 1);
      if (kt + 2 < nkt) gload(k0 + 2 * BK);
    }
    // register r of block sb is key k0 + 32 sb + 8 (r / 4) + 4 h + r % 4
    const bool diag = CAUSAL && (k0 + BK - 1 > qt * QT + w * 32);
    const bool want_lse = a.lse != nullptr;
    float psum = 0.f; // unrounded row sum of the tile, only where the LSE is wanted
#pragma unroll
    for (int sb = 0; sb < 2; ++sb)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float p = fast_exp2(x[sb][r] * s);
        if (diag) p = (k0 + sb * 32 + 8 * (r / 4) + 4 * h + r % 4 <= q) ? p : 0.f;
        x[sb][r] = p;
      }
    if (want_lse) {
#pragma unroll
      for (int sb = 0; sb < 2; ++sb)
#pragma unroll
        for (int r = 0; r < 16; ++r) psum += x[sb][r];
    }
    i32x8 pb;
#pragma unroll
    for (int sb = 0; sb < 2; ++sb)
#pragma unroll
      for (int g = 0; g < 4; ++g) pb[sb * 4 + g] = pack4_e4m3(x[sb][4 * g], x[sb][4 * g + 1], x[sb][4 * g + 2], x[sb][4 * g + 3]);
    // sum of the rounded probabilities of this lane's row over the tile: ones . P~ (every row of the result alike)
    const i32x8 ones = {0x38383838, 0x38383838, 0x38383838, 0x38383838, 0x38383838, 0x38383838, 0x38383838, 0x38383838};
    f32x16 zero;
#pragma unroll
    for (int r = 0; r < 16; ++r) zero[r] = 0.f;
    float tsum = mfma_fp8_k64(ones, pb, zero)[0];
    // Slow path, wave-uniform: the first tile of a row (no reference yet), or a row sum beyond the range that
    // guarantees representable probabilities (compared as bit patterns: the sum is never negative, and a NaN
    // from a saturated conversion must take this path although the build tells the compiler that NaNs do not
    // occur).  The scores are recomputed from the operands (the fast path has
    // overwritten them), the reference becomes ceil(max), everything is rescaled by the exact power of two.
    // Only the rows that need it change their reference (and take the recomputed probabilities): a row's result
    // depends on that row alone, whatever rows share its wave.
    const bool need = !seen || __float_as_uint(tsum) > __float_as_uint(SUM_LIMIT);
    if (__builtin_amdgcn_ballot_w64(need)) {
      f32x16 y[2];
      float mx = NEG_INF;
#pragma unroll
      for (int sb = 0; sb < 2; ++sb) {
#pragma unroll
        for (int r = 0; r < 16; ++r) y[sb][r] = 0.f;
#pragma unroll
        for (int ds = 0; ds < DS; ++ds) {
          const char *kp = ldsK + (sb * 32 + ql) * PITCH + ds * 64 + h * 32;
          const u32x4 lo = *(const u32x4 *)kp, hi = *(const u32x4 *)(kp + 16);
          const i32x8 ka = {(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
          y[sb] = mfma_fp8_k64(ka, qreg[ds], y[sb]);
        }
        const bf16x8 xa = as_v8<__bf16>(*(const u32x4 *)(ldsX + (sb * 32 + ql) * XROWB + h * 16));
        y[sb] = Elem<__bf16>::mfma(xa, bx, y[sb]);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          float v = fmaf(y[sb][r], s, M); // the score in log2 units (plus mask term)
          if (diag) v = (k0 + sb * 32 + 8 * (r / 4) + 4 * h + r % 4 <= q) ? v : NEG_INF;
          y[sb][r] = v;
          mx = fmaxf(mx, v);
        }
      }
      mx = xhalf_max(mx);
      const bool live = mx > -1e20f; // this tile shows the row a key that is not masked out
      float Mn = M;
      if (need && live) Mn = seen ? fmaxf(M, __builtin_ceilf(mx)) : __builtin_ceilf(mx);
      const float alpha = seen ? fast_exp2(M - Mn) : 1.f; // (nothing has been accumulated before the first live tile; 1 where the reference stays)
      float psum_new = 0.f;
#pragma unroll
      for (int sb = 0; sb < 2; ++sb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float p = live ? fast_exp2(y[sb][r] - Mn) : 0.f;
          y[sb][r] = p;
          psum_new += p;
        }
      psum = need ? psum_new : psum;
#pragma unroll
      for (int sb = 0; sb < 2; ++sb)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int pn = pack4_e4m3(y[sb][4 * g], y[sb][4 * g + 1], y[sb][4 * g + 2], y[sb][4 * g + 3]);
          pb[sb * 4 + g] = need ? pn : pb[sb * 4 + g]; // (both half-waves of a row decide alike: the sums they test are the row's)
        }
      tsum = mfma_fp8_k64(ones, pb, zero)[0];
      l_run *= alpha;
      l_true *= alpha;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;
      M = Mn;
      seen = seen || (need && live);
      set_bx();
    }
    l_run += tsum;
    if (want_lse) l_true += xhalf_sum(psum);
    // O^T += V^T.P^T: one K = 64 product per 32 head-dim columns
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      i32x8 va;
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int gp = 0; gp < 2; ++gp) {
          const i32x2v t = lds_read_tr8(ldsV + trofs + (32 * b + 16 * gp) * PITCH + db * 32);
          va[4 * b + 2 * gp] = t.x;
          va[4 * b + 2 * gp + 1] = t.y;
        }
      oacc[db] = mfma_fp8_k64(va, pb, oacc[db]);
    }
    __syncthreads(); // this stage is free again, the next one is complete
  }

  // normalise and store: in the accumulator layout lane (q, h) holds head-dim columns 8g + 4h .. +3 of each 32-block
  if (q < a.sq) {
    const float inv = l_run > 0.f ? a.out_scale / l_run : 0.f;
    TO *Or = (TO *)a.o + ((size_t)bh * a.sq + q) * D;
#pragma unroll
    for (int db = 0; db < DB; ++db) store_acc_block_row<TO>(Or + db * 32, oacc[db], inv, h);
    if (a.lse && h == 0) a.lse[(size_t)bh * a.sq + q] = l_true > 0.f ? (M + fast_log2(l_true)) * FMHA_LN2 : NEG_INF;
  }
}

} // namespace fmha
