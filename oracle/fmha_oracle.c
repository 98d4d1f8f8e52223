/*
 * CPU oracle for the fused multi-head-attention path.  TEST INFRASTRUCTURE ONLY:
 * nothing that ships (the HIP library, the torch extension, the package) may
 * call, link or import this file; it exists so tests, the smoke check and the
 * benchmark's CPU-baseline leg have an independent statement of the answer.
 *
 * It restates, in plain C with double accumulation, the eager composition the
 * reference treats as ground truth:
 *   inference  reference test.py:12-18         p = q k^T ; p/8 + (1-amask)*-10000 ;
 *                                              softmax(-1) ; @ v ; cast half
 *   train      reference test_train_mha.py:14-21   q k^T * scale + pad_mask ; softmax ;
 *                                              (x / dropout_prob) * dropout_mask ; @ v
 *   op order and the half casts of the fused kernels:
 *              reference fmha/fmha_manual.cpp:55-97 (inference), :452-492 (train),
 *              :891-897 (saved softmax / dropout outputs)
 * plus two things the reference does not have and this build defines: seeded
 * Philox4x32-10 dropout and the analytic backward (dQ, dK, dV).
 *
 * Pinning (see tests/test_oracle_*.py): forward against torch CPU matmul/softmax
 * in fp32/fp64 and closed forms; Philox against the Random123 known-answer
 * vectors; backward against central finite differences in fp64 and torch
 * autograd through an eager composition.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ rounding */

static float round_f16(float x) {
  /* round-to-nearest-even to IEEE binary16, returned as float */
  if (isnan(x) || isinf(x)) return x;
  float ax = fabsf(x);
  if (ax >= 65520.0f) return copysignf(INFINITY, x);
  if (ax < 6.103515625e-05f) { /* subnormal half: spacing 2^-24 */
    float r = nearbyintf(ax * 16777216.0f) / 16777216.0f;
    return copysignf(r, x);
  }
  int e;
  frexpf(ax, &e);                 /* ax = f * 2^e, f in [0.5,1) */
  float ulp = ldexpf(1.0f, e - 11); /* 11 significant bits */
  float r = nearbyintf(ax / ulp) * ulp;
  return copysignf(r, x);
}

static float round_bf16(float x) {
  if (isnan(x) || isinf(x)) return x;
  uint32_t u;
  memcpy(&u, &x, 4);
  uint32_t lsb = (u >> 16) & 1u;
  u += 0x7fffu + lsb;
  u &= 0xffff0000u;
  float r;
  memcpy(&r, &u, 4);
  return r;
}

static float round_e4m3(float x) {
  /* round-to-nearest-even to OCP e4m3 (4 exponent bits, bias 7, 3 mantissa bits, no infinities),
   * saturating at the largest finite value 448; subnormal spacing 2^-9 below 2^-6 */
  if (isnan(x)) return x;
  float ax = fabsf(x);
  if (ax >= 448.0f) return copysignf(448.0f, x);
  if (ax < 0.015625f) return copysignf(nearbyintf(ax * 512.0f) / 512.0f, x);
  int e;
  frexpf(ax, &e);
  float ulp = ldexpf(1.0f, e - 4); /* 4 significant bits */
  float r = nearbyintf(ax / ulp) * ulp;
  if (r > 448.0f) r = 448.0f;
  return copysignf(r, x);
}

static float round_to(float x, int kind) {
  if (kind == 1) return round_f16(x);
  if (kind == 2) return round_bf16(x);
  if (kind == 3) return round_e4m3(x);
  return x;
}

float fmha_oracle_round(float x, int kind) { return round_to(x, kind); }

/* -------------------------------------------------------------------- Philox */
/* Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3",
 * SC'11).  Same constants and round function as Random123 and as ATen's
 * philox_engine. */

void fmha_oracle_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
  uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3];
  uint32_t k0 = key[0], k1 = key[1];
  for (int r = 0; r < 10; ++r) {
    uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    uint32_t n1 = (uint32_t)p1;
    uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    uint32_t n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

/* Dropout keep rule of this build (integer only).
 * Elements are grouped in 4x4 (query x key) blocks; one Philox call serves a block:
 *   key  = (seed_lo, seed_hi)
 *   ctr  = (offset_lo, offset_hi, blk_lo, blk_hi),
 *          blk = (bh * ceil(Sq/4) + q/4) * ceil(Sk/4) + k/4
 *   byte = (out[q%4] >> 8*(k%4)) & 0xff ;  keep iff byte >= thr,  thr = round(p*256)
 * Kept values are scaled by 256 / (256 - thr), the reciprocal of the keep probability that the 8-bit
 * threshold realises (not of the nominal 1 - p), so that dropout preserves the mean exactly;
 * thr == 0 keeps everything (scale 1).
 */
uint32_t fmha_oracle_drop_threshold(float p) {
  double t = floor((double)p * 256.0 + 0.5);
  if (t < 0) t = 0;
  if (t > 255) t = 255;
  return (uint32_t)t;
}

float fmha_oracle_drop_scale(float p) {
  uint32_t thr = fmha_oracle_drop_threshold(p);
  return (float)(256.0 / (256.0 - (double)thr));
}

int fmha_oracle_keep(uint64_t seed, uint64_t offset, uint32_t thr, int64_t bh, int64_t q,
                     int64_t k, int64_t sq, int64_t sk) {
  uint64_t qb4 = (uint64_t)((sq + 3) / 4), kb4 = (uint64_t)((sk + 3) / 4);
  uint64_t blk = ((uint64_t)bh * qb4 + (uint64_t)(q / 4)) * kb4 + (uint64_t)(k / 4);
  uint32_t ctr[4] = {(uint32_t)offset, (uint32_t)(offset >> 32), (uint32_t)blk,
                     (uint32_t)(blk >> 32)};
  uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  uint32_t out[4];
  fmha_oracle_philox4x32_10(ctr, key, out);
  uint32_t byte = (out[q & 3] >> (8 * (k & 3))) & 0xffu;
  return byte >= thr;
}

void fmha_oracle_keep_mask(uint64_t seed, uint64_t offset, float p, int64_t bh, int64_t sq,
                           int64_t sk, uint8_t *out /* [bh,sq,sk] */) {
  uint32_t thr = fmha_oracle_drop_threshold(p);
  for (int64_t b = 0; b < bh; ++b)
    for (int64_t q = 0; q < sq; ++q)
      for (int64_t k = 0; k < sk; ++k)
        out[(b * sq + q) * sk + k] = (uint8_t)fmha_oracle_keep(seed, offset, thr, b, q, k, sq, sk);
}

/* -------------------------------------------------------------------- params */

typedef struct {
  int64_t bh, sq, sk, d;
  const float *q, *k, *v; /* [bh,sq,d], [bh,sk,d], [bh,sk,d] */
  /* mask: element (bh,q,k) at mask[(bh / mask_bh_div) * mask_sb + q * mask_sq + k] */
  const float *mask;
  int64_t mask_bh_div, mask_sb, mask_sq;
  int32_t mask_kind; /* 0 none, 1 additive, 2 keep01: adds (1-m)*mask_neg */
  float mask_neg;
  int32_t causal;    /* 1: key k visible to query q iff k <= q */
  float scale;
  /* dropout: 0 none, 1 explicit multiplicative mask [bh,sq,sk], 2 Philox */
  int32_t drop_kind;
  const float *drop_mask;
  float p_drop;      /* Philox threshold source */
  float drop_scale;  /* multiplies kept probabilities (2.0 legacy, 1/(1-p) seeded) */
  uint64_t seed, offset;
  int32_t round_p;   /* 0: none, 1: fp16, 2: bf16 -- rounding of P before P.V (fmha_manual.cpp:87);
                      * 3: e4m3, the rounding model of the 8-bit forward (which the reference lacks): applied to
                      * the UNNORMALISED 2^(y - M), y the score in log2 units and M = ceil(max_j y_j), an integer,
                      * so that any other integer reference gives the same rounded values up to a power of two;
                      * the weights are the rounded values over THEIR sum (a convex combination: a row with one
                      * dominant key reproduces that key's value exactly); the LSE stays unrounded */
  int32_t round_o;   /* rounding of outputs (fmha_manual.cpp:95) */
  /* outputs (any may be NULL) */
  float *o;          /* [bh,sq,d] */
  float *lse;        /* [bh,sq] natural log of the softmax denominator incl. max */
  float *softmax;    /* [bh,sq,sk] P */
  float *dropout;    /* [bh,sq,sk] P*dropmask*drop_scale */
  /* backward */
  const float *dout; /* [bh,sq,d] */
  float *dq, *dk, *dv;
  /* head b of these tensors is head bh_offset + b of the full problem as far as the Philox block
   * index is concerned (a sample of the heads of a larger batch keeps its dropout decisions) */
  int64_t bh_offset;
} fmha_oracle_params;

static double score_at(const fmha_oracle_params *p, int64_t b, int64_t i, int64_t j) {
  const float *qi = p->q + (b * p->sq + i) * p->d;
  const float *kj = p->k + (b * p->sk + j) * p->d;
  double s = 0.0;
  for (int64_t c = 0; c < p->d; ++c) s += (double)qi[c] * (double)kj[c];
  s *= (double)p->scale;
  if (p->mask_kind) {
    double m = (double)p->mask[(b / p->mask_bh_div) * p->mask_sb + i * p->mask_sq + j];
    s += (p->mask_kind == 2) ? (1.0 - m) * (double)p->mask_neg : m;
  }
  if (p->causal && j > i) s = -INFINITY;
  return s;
}

static double drop_factor(const fmha_oracle_params *p, uint32_t thr, int64_t b, int64_t i,
                          int64_t j) {
  if (p->drop_kind == 1)
    return (double)p->drop_mask[(b * p->sq + i) * p->sk + j] * (double)p->drop_scale;
  if (p->drop_kind == 2)
    return fmha_oracle_keep(p->seed, p->offset, thr, p->bh_offset + b, i, j, p->sq, p->sk)
               ? (double)p->drop_scale : 0.0;
  return 1.0;
}

/* One softmax row: fills prob[0..sk) and returns log-sum-exp; *sum_out (if given) receives
 * sum_j exp(s_j - max), the factor between prob and the unnormalised exponentials. */
static double softmax_row_sum(const fmha_oracle_params *p, int64_t b, int64_t i, double *prob, double *sum_out);
static double softmax_row(const fmha_oracle_params *p, int64_t b, int64_t i, double *prob) {
  return softmax_row_sum(p, b, i, prob, NULL);
}
static double softmax_row_sum(const fmha_oracle_params *p, int64_t b, int64_t i, double *prob, double *sum_out) {
  double mx = -INFINITY;
  for (int64_t j = 0; j < p->sk; ++j) {
    prob[j] = score_at(p, b, i, j);
    if (prob[j] > mx) mx = prob[j];
  }
  if (sum_out) *sum_out = 1.0;
  if (mx == -INFINITY) { /* fully masked row: defined as all-zero probabilities */
    for (int64_t j = 0; j < p->sk; ++j) prob[j] = 0.0;
    return -INFINITY;
  }
  double sum = 0.0;
  for (int64_t j = 0; j < p->sk; ++j) {
    prob[j] = exp(prob[j] - mx);
    sum += prob[j];
  }
  for (int64_t j = 0; j < p->sk; ++j) prob[j] /= sum;
  if (sum_out) *sum_out = sum;
  return mx + log(sum);
}

int fmha_oracle_fwd(const fmha_oracle_params *p) {
  double *prob = (double *)malloc(sizeof(double) * (size_t)p->sk);
  double *acc = (double *)malloc(sizeof(double) * (size_t)p->d);
  if (!prob || !acc) return -1;
  uint32_t thr = fmha_oracle_drop_threshold(p->p_drop);
  for (int64_t b = 0; b < p->bh; ++b) {
    for (int64_t i = 0; i < p->sq; ++i) {
      double rowsum = 1.0;
      double lse = softmax_row_sum(p, b, i, prob, &rowsum);
      if (p->lse) p->lse[b * p->sq + i] = (float)lse;
      for (int64_t c = 0; c < p->d; ++c) acc[c] = 0.0;
      double e4_factor = 1.0, e4_den = 1.0;
      if (p->round_p == 3 && lse > -INFINITY) {
        const double yl2 = (lse - log(rowsum)) * 1.4426950408889634; /* row maximum in log2 units */
        e4_factor = rowsum * exp2(yl2 - ceil(yl2));
        e4_den = 0.0;
        for (int64_t j = 0; j < p->sk; ++j) e4_den += (double)round_to((float)(prob[j] * e4_factor), 3);
        if (e4_den == 0.0) e4_den = 1.0;
      }
      for (int64_t j = 0; j < p->sk; ++j) {
        double pj = prob[j];
        double pd = pj * drop_factor(p, thr, b, i, j);
        if (p->softmax) p->softmax[(b * p->sq + i) * p->sk + j] = round_to((float)pj, p->round_o);
        if (p->dropout) p->dropout[(b * p->sq + i) * p->sk + j] = round_to((float)pd, p->round_o);
        double w = p->round_p == 3 ? (double)round_to((float)(pd * e4_factor), 3) / e4_den
                                   : (double)round_to((float)pd, p->round_p);
        const float *vj = p->v + (b * p->sk + j) * p->d;
        for (int64_t c = 0; c < p->d; ++c) acc[c] += w * (double)vj[c];
      }
      if (p->o)
        for (int64_t c = 0; c < p->d; ++c)
          p->o[(b * p->sq + i) * p->d + c] = round_to((float)acc[c], p->round_o);
    }
  }
  free(prob);
  free(acc);
  return 0;
}

/* Analytic backward of O = (softmax(S) o Z) V, S = scale q k^T + mask, Z = dropout factor:
 *   dV = (P o Z)^T dO ;  dPz = dO V^T ;  dP = dPz o Z ;  delta_i = sum_j P_ij dP_ij
 *   dS = P o (dP - delta) ;  dQ = scale dS K ;  dK = scale dS^T Q            */
int fmha_oracle_bwd(const fmha_oracle_params *p) {
  double *prob = (double *)malloc(sizeof(double) * (size_t)p->sk);
  double *dp = (double *)malloc(sizeof(double) * (size_t)p->sk);
  size_t nk = (size_t)(p->bh * p->sk * p->d), nq = (size_t)(p->bh * p->sq * p->d);
  double *dk = (double *)calloc(nk, sizeof(double));
  double *dv = (double *)calloc(nk, sizeof(double));
  double *dq = (double *)calloc(nq, sizeof(double));
  if (!prob || !dp || !dk || !dv || !dq) return -1;
  uint32_t thr = fmha_oracle_drop_threshold(p->p_drop);
  for (int64_t b = 0; b < p->bh; ++b) {
    for (int64_t i = 0; i < p->sq; ++i) {
      softmax_row(p, b, i, prob);
      const float *doi = p->dout + (b * p->sq + i) * p->d;
      const float *qi = p->q + (b * p->sq + i) * p->d;
      double delta = 0.0;
      for (int64_t j = 0; j < p->sk; ++j) {
        double z = drop_factor(p, thr, b, i, j);
        const float *vj = p->v + (b * p->sk + j) * p->d;
        double dpz = 0.0;
        for (int64_t c = 0; c < p->d; ++c) dpz += (double)doi[c] * (double)vj[c];
        double w = prob[j] * z;
        double *dvj = dv + (b * p->sk + j) * p->d;
        for (int64_t c = 0; c < p->d; ++c) dvj[c] += w * (double)doi[c];
        dp[j] = dpz * z;
        delta += prob[j] * dp[j];
      }
      double *dqi = dq + (b * p->sq + i) * p->d;
      for (int64_t j = 0; j < p->sk; ++j) {
        double ds = prob[j] * (dp[j] - delta) * (double)p->scale;
        if (ds == 0.0) continue;
        const float *kj = p->k + (b * p->sk + j) * p->d;
        double *dkj = dk + (b * p->sk + j) * p->d;
        for (int64_t c = 0; c < p->d; ++c) {
          dqi[c] += ds * (double)kj[c];
          dkj[c] += ds * (double)qi[c];
        }
      }
    }
  }
  for (size_t t = 0; t < nq; ++t)
    if (p->dq) p->dq[t] = round_to((float)dq[t], p->round_o);
  for (size_t t = 0; t < nk; ++t) {
    if (p->dk) p->dk[t] = round_to((float)dk[t], p->round_o);
    if (p->dv) p->dv[t] = round_to((float)dv[t], p->round_o);
  }
  free(prob); free(dp); free(dk); free(dv); free(dq);
  return 0;
}
