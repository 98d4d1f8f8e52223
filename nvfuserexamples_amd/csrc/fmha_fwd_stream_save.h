// The reference's save-intermediates operator (fmha/fmha_manual.cpp:891-897: context, normalised
// softmax and its dropped, scaled copy) for key ranges of 129 to 512 keys in ONE launch that reads
// every input once.
//
// The streaming forward followed by the kernel that derives the saved outputs from the row
// log-sum-exp reads the mask and the dropout tensor twice: two of the six [.., sq, sk]-sized
// transfers of the operator.  Here a wave keeps what the second launch would re-read: per 64-key
// tile the unnormalised probabilities exp2(s - m_t) of its 32 queries, rounded to the element type
// (16 registers), the tile's dropout rows as loaded (16 registers) and the running maximum m_t they
// were formed under.  Eight tiles make 264 registers, so the kernel runs one wave per SIMD with the
// whole 512-entry register file (the key loop is unrolled: register arrays are indexed by constants).
// After the last tile the row's log-sum-exp L is known and a second, store-only, phase writes
//   softmax = round(p_t * exp2(m_t - L)),   dropout = round(p_t * exp2(m_t - L) * d * scale)
// tile by tile through the wave's LDS scratch as whole 128-byte row segments.
//
// Rounding: the saved softmax is rounded twice (p_t to the element type, then the product), at most
// 2^-10 relative for fp16 instead of 2^-11; the second product O += P V takes exactly the operands
// of the streaming forward, so the context is bit-identical to that kernel's.
#pragma once
#include "fmha_fwd_stream.h"

namespace fmha {

struct StreamSaveCfg : StreamCfg {
  static constexpr int MAXT = 8;                   // 64-key tiles whose probabilities a wave can hold
  static constexpr int SKMAX = MAXT * BK;
};

template <typename T>
__global__ __launch_bounds__(StreamSaveCfg::NW * 64) __attribute__((amdgpu_waves_per_eu(1, 1)))
void fmha_fwd_stream_save_kernel(const FwdArgs a) {
  using E = Elem<T>;
  using v8 = typename E::v8;
  using v4 = typename E::v4;
  using C = StreamSaveCfg;
  constexpr int D = C::D, KS = D / 16, DB = D / 32, BK = C::BK, NSB = BK / 32, NT = C::NW * 64, ROWB = C::ROWB;
  constexpr int TILEB = C::TILEB, MAXT = C::MAXT;
  constexpr int CPR = D / 8, CPT = BK * CPR / NT;
  constexpr float NEG_INF = -__builtin_inff();

  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int tid = threadIdx.x;
  const int w = tid >> 6;
  const int l = tid & 63;
  const int ql = l & 31;
  const int h = l >> 5;

  int bid = blockIdx.x;
  const int nb = gridDim.x;
  if ((nb & 7) == 0) bid = (bid & 7) * (nb >> 3) + (bid >> 3);
  const int bh = bid / a.nqt;
  const int qt = bid - bh * a.nqt;
  const int q0w = qt * C::QT + w * 32;

  const T *Qb = (const T *)a.q + (size_t)bh * a.sq * D;
  const T *Kb = (const T *)a.k + (size_t)bh * a.sk * D;
  const T *Vb = (const T *)a.v + (size_t)bh * a.sk * D;

  v8 qreg[KS];
  {
    int q = q0w + ql;
    q = q < a.sq ? q : a.sq - 1;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qreg[ks] = as_v8<T>(*(const u32x4 *)(Qb + (size_t)q * D + ks * 16 + h * 8));
  }

  // ---- staging, as in the streaming forward.  K, V: global -> registers -> LDS (two stages).  [.., sq, sk]
  // rows: instruction i covers rows 8i .. 8i+7 of the wave's 32, eight lanes per row, 8 keys per lane.
  typename C::Scratch scr;
  scr.init(lds + 4 * TILEB + w * C::Scratch::BYTES, l);
  const int rsub = scr.rsub, chunk = scr.chunk;
  int qrow[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int q = q0w + 8 * i + rsub;
    qrow[i] = q < a.sq ? q : a.sq - 1;
  }
  const T *mb = (const T *)a.mask + (size_t)(bh / a.mask_div) * a.mask_sb;
  const T *db_ = (const T *)a.drop_mask + (size_t)bh * a.sq * a.sk;
  struct Stage {
    u32x4 k[CPT], v[CPT], m[4], d[4];
  };
  // every load is unconditional: key rows past the end re-read the last row, chunks past sk the row's first
  // chunk; those keys' scores are forced to -inf and their columns are never stored
  auto gload = [&](int k0, Stage &st) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = tid + i * NT;
      int kr = k0 + c / CPR;
      kr = kr < a.sk ? kr : a.sk - 1;
      st.k[i] = *(const u32x4 *)(Kb + (size_t)kr * D + (c % CPR) * 8);
      st.v[i] = *(const u32x4 *)(Vb + (size_t)kr * D + (c % CPR) * 8);
    }
    const int koff = k0 + chunk * 8 < a.sk ? k0 + chunk * 8 : 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      st.m[i] = *(const u32x4 *)(mb + (size_t)qrow[i] * a.mask_sq + koff);
      st.d[i] = *(const u32x4 *)(db_ + (size_t)qrow[i] * a.sk + koff);
    }
  };
  auto lstore = [&](int stage, const Stage &st) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = tid + i * NT;
      *(u32x4 *)(lds + stage * 2 * TILEB + (c / CPR) * ROWB + (c % CPR) * 16) = st.k[i];
      *(u32x4 *)(lds + stage * 2 * TILEB + TILEB + (c / CPR) * ROWB + (c % CPR) * 16) = st.v[i];
    }
  };

  // ---- running state, and what the store phase needs of every tile
  float m = NEG_INF, lsum = 0.f;
  f32x16 o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[db][r] = 0.f;
  v8 psave[MAXT][NSB][2];
  u32x4 dsave[MAXT][4];
  float msave[MAXT];

  // (Requests run one tile ahead of their use.  Two tiles ahead -- the registers would allow it -- measured
  // 5-7 % slower at BH 512, S 256 to 512: the operator is bound by the mixed read / write stream of the
  // whole device, not by one workgroup's latency.)
  const int nkt = (a.sk + BK - 1) / BK; // <= MAXT (checked by the host)
  Stage cur;
  gload(0, cur);
  lstore(0, cur);
  __syncthreads();

#pragma unroll
  for (int t = 0; t < MAXT; ++t) {
    if (t < nkt) { // workgroup-uniform
      const int k0 = t * BK;
      const char *ldsK = lds + (t & 1) * 2 * TILEB;
      const char *ldsV = ldsK + TILEB;
      Stage nxt;
      const bool more = t + 1 < nkt;
      if (more) gload(k0 + BK, nxt);

      // ---- scores in log2 units: x * scale + mask
      f32x16 x[NSB];
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb) {
#pragma unroll
        for (int r = 0; r < 16; ++r) x[sb][r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
          x[sb] = E::mfma(as_v8<T>(*(const u32x4 *)(ldsK + (sb * 32 + ql) * ROWB + ks * 32 + h * 16)), qreg[ks], x[sb]);
      }
      scr.rows_in(cur.m);
      scr.turn();
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const v4 mv = as_v4<T>(scr.piece(sb, g));
#pragma unroll
          for (int i = 0; i < 4; ++i)
            x[sb][4 * g + i] = fmaf(x[sb][4 * g + i], a.scale_l2, fmaf((float)mv[i], a.mask_a, a.mask_b));
        }
      scr.turn();
      if (k0 + BK > a.sk) { // only a partly filled last tile has keys to switch off (workgroup-uniform)
#pragma unroll
        for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int kk = k0 + sb * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
            x[sb][r] = kk < a.sk ? x[sb][r] : NEG_INF;
          }
      }
      float tmax = NEG_INF;
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
        for (int r = 0; r < 16; r += 2) tmax = max3(tmax, x[sb][r], x[sb][r + 1]);

      // ---- online softmax
      tmax = xhalf_max(tmax);
      const float mnew = fmaxf(m, tmax);
      const float muse = mnew == NEG_INF ? 0.f : mnew;
      const float alpha = m == NEG_INF ? 0.f : fast_exp2(m - mnew);
      m = mnew;
      msave[t] = mnew; // -inf while the row has seen no key: the tile's probabilities are zeros and stay zeros
      float rs = 0.f;
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float p = fast_exp2(x[sb][r] - muse);
          x[sb][r] = p;
          rs += p;
        }
      lsum = fmaf(lsum, alpha, rs);
      if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) { // (exactly one wherever the maximum stayed)
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[db][r] *= alpha;
      }

      // ---- dropped probabilities in the element type (B operand of the second product); undropped ones kept
      scr.rows_in(cur.d);
      scr.turn();
      v8 pfrag[NSB][2];
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const v4 dm = as_v4<T>(scr.piece(sb, g));
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            pfrag[sb][g >> 1][4 * (g & 1) + i] = (T)(x[sb][4 * g + i] * (float)dm[i]);
            psave[t][sb][g >> 1][4 * (g & 1) + i] = (T)x[sb][4 * g + i];
          }
        }
      scr.turn();
#pragma unroll
      for (int i = 0; i < 4; ++i) dsave[t][i] = cur.d[i];

      // ---- O^T += V^T . P^T
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
          for (int db = 0; db < DB; ++db)
            o[db] = E::mfma(lds_load_a_transposed<T, ROWB>(ldsV, sb * 32, db * 32, c, l), pfrag[sb][c], o[db]);

      if (more) {
        lstore((t + 1) & 1, nxt);
        cur = nxt;
      }
      __syncthreads();
    }
  }

  // ---- context and log-sum-exp
  const int q = q0w + ql;
  const float lt = xhalf_sum(lsum);
  const float inv = lt > 0.f ? a.drop_scale / lt : 0.f;
  if (q < a.sq) {
    T *Ob = (T *)a.o + ((size_t)bh * a.sq + q) * D;
#pragma unroll
    for (int db = 0; db < DB; ++db) store_acc_block_row<T>(Ob + db * 32, o[db], inv, h);
    if (a.lse && h == 0) a.lse[(size_t)bh * a.sq + q] = lt > 0.f ? (m + fast_log2(lt)) * FMHA_LN2 : NEG_INF;
  }

  // ---- the saved outputs.  m_t <= m <= L wherever m_t is finite, so the factors are at most one; a tile the
  // row entered with no key seen (m_t = -inf) and a row that never saw one (L = +big) give factor zero.
  const float L = lt > 0.f ? m + fast_log2(lt) : 3.0e38f;
  auto rows_out = [&](void *out, int k0) {
    const bool cvalid = k0 + chunk * 8 < a.sk;
    T *ob = (T *)out + (size_t)bh * a.sq * a.sk + k0 + chunk * 8;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int qq = q0w + 8 * i + rsub;
      const u32x4 tt = scr.row_out(i);
      if (cvalid && qq < a.sq) *(u32x4 *)(ob + (size_t)qq * a.sk) = tt;
    }
  };
#pragma unroll
  for (int t = 0; t < MAXT; ++t) {
    if (t < nkt) {
      const int k0 = t * BK;
      const float f = fast_exp2(msave[t] - L);
      float x[NSB][16];
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
        for (int r = 0; r < 16; ++r) x[sb][r] = (float)psave[t][sb][r >> 3][r & 7] * f;
      if (a.save_softmax) {
#pragma unroll
        for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            v4 s4;
#pragma unroll
            for (int i = 0; i < 4; ++i) s4[i] = (T)x[sb][4 * g + i];
            scr.template put_piece<T>(sb, g, s4);
          }
        scr.turn();
        rows_out(a.save_softmax, k0);
        scr.turn();
      }
      if (a.save_dropout) {
        scr.rows_in(dsave[t]);
        scr.turn();
        v4 d4[NSB][4];
#pragma unroll
        for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const v4 dm = as_v4<T>(scr.piece(sb, g));
#pragma unroll
            for (int i = 0; i < 4; ++i) d4[sb][g][i] = (T)(x[sb][4 * g + i] * ((float)dm[i] * a.drop_scale));
          }
        scr.turn();
#pragma unroll
        for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
          for (int g = 0; g < 4; ++g) scr.template put_piece<T>(sb, g, d4[sb][g]);
        scr.turn();
        rows_out(a.save_dropout, k0);
        scr.turn();
      }
    }
  }
}

} // namespace fmha
