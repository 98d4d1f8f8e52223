// Writes the two saved outputs of the reference's save-intermediates operator -- the normalised
// softmax and its dropped, scaled copy (reference fmha/fmha_manual.cpp:891-897) -- for key ranges
// beyond the one-pass kernel's 128 keys, given the row log-sum-exp that the forward kernel has
// just produced:  P = exp(score + mask - LSE) needs no second sweep for the normalisation.
//
// This is a streaming kernel: per 64-key tile a workgroup reads 16 KB of mask and 16 KB of dropout
// rows and writes 32 KB, against 8 KB of K and 16 MFMAs.  It is built like the one-pass kernel for
// short key ranges: [.., sq, sk] rows move as whole 128-byte row segments (16 bytes per lane, 8
// lanes per row) and a wave-private LDS scratch turns them into the accumulator layout and back.
// K tiles and the next tile's mask / dropout rows are requested at the top of an iteration, before
// the iteration's stores, so that waiting for them never waits for a store.
#pragma once
#include "fmha_fwd_kernel.h"

namespace fmha {

struct SaveCfg {
  static constexpr int D = 64;
  static constexpr int NW = 4;
  static constexpr int QT = NW * 32;
  static constexpr int BK = 64;
  static constexpr int ROWB = D * 2 + 16;          // padded K rows: conflict-free 16-byte reads
  static constexpr int KTILEB = BK * ROWB;
  using Scratch = RowScratch<BK>;                  // wave-private: rows of a [.., sq, sk] tensor <-> accumulator layout
  static constexpr int LDS_BYTES = 2 * KTILEB + NW * Scratch::BYTES;
};

template <typename T>
__global__ __launch_bounds__(SaveCfg::NW * 64) __attribute__((amdgpu_waves_per_eu(2, 2)))
void fmha_fwd_save_kernel(const FwdArgs a) {
  using E = Elem<T>;
  using v8 = typename E::v8;
  using v4 = typename E::v4;
  using C = SaveCfg;
  constexpr int D = C::D, KS = D / 16, BK = C::BK, NSB = BK / 32, NT = C::NW * 64, ROWB = C::ROWB;
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

  v8 qreg[KS];
  float lq; // the lane's row log-sum-exp in log2 units; rows that saw no key give P = 0
  {
    int q = q0w + ql;
    q = q < a.sq ? q : a.sq - 1;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qreg[ks] = as_v8<T>(*(const u32x4 *)(Qb + (size_t)q * D + ks * 16 + h * 8));
    const float ls = a.lse[(size_t)bh * a.sq + q];
    lq = ls == NEG_INF ? 3.0e38f : ls * FMHA_LOG2E;
  }

  // ---- staging.  K: global -> registers -> LDS (two stages).  [.., sq, sk] rows: instruction i covers
  // rows 8i .. 8i+7 of the wave's 32, eight lanes per row, 8 keys (16 bytes) per lane.
  typename C::Scratch scr;
  scr.init(lds + 2 * C::KTILEB + w * C::Scratch::BYTES, l);
  const int rsub = scr.rsub, chunk = scr.chunk;
  int qrow[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int q = q0w + 8 * i + rsub;
    qrow[i] = q < a.sq ? q : a.sq - 1;
  }
  const T *mb = (const T *)a.mask + (size_t)(bh / a.mask_div) * a.mask_sb;
  const T *db_ = (const T *)a.drop_mask + (size_t)bh * a.sq * a.sk;
  u32x4 kst[CPT], mreg[4], dreg[4];
  // Every load is unconditional (a load under a lane condition makes the compiler wait for it on the
  // spot): rows past the end re-read the last row, chunks past sk re-read the row's first chunk; neither
  // is ever used (those keys get P = 0 and are not stored).
  auto gload = [&](int k0, u32x4 (&kd)[CPT], u32x4 (&md)[4], u32x4 (&dd)[4]) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = tid + i * NT;
      int kr = k0 + c / CPR;
      kr = kr < a.sk ? kr : a.sk - 1;
      kd[i] = *(const u32x4 *)(Kb + (size_t)kr * D + (c % CPR) * 8);
    }
    const int koff = k0 + chunk * 8 < a.sk ? k0 + chunk * 8 : 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      md[i] = *(const u32x4 *)(mb + (size_t)qrow[i] * a.mask_sq + koff);
      dd[i] = *(const u32x4 *)(db_ + (size_t)qrow[i] * a.sk + koff);
    }
  };
  auto lstore = [&](int stage, const u32x4 (&kd)[CPT]) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = tid + i * NT;
      *(u32x4 *)(lds + stage * C::KTILEB + (c / CPR) * ROWB + (c % CPR) * 16) = kd[i];
    }
  };

  auto rows_out = [&](void *out, int k0) {
    const bool cvalid = k0 + chunk * 8 < a.sk;
    T *ob = (T *)out + (size_t)bh * a.sq * a.sk + k0 + chunk * 8;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int q = q0w + 8 * i + rsub;
      const u32x4 t = scr.row_out(i);
      if (cvalid && q < a.sq) *(u32x4 *)(ob + (size_t)q * a.sk) = t;
    }
  };

  const int nkt = (a.sk + BK - 1) / BK;
  gload(0, kst, mreg, dreg);
  lstore(0, kst);
  __syncthreads();

  for (int t = 0; t < nkt; ++t) {
    const int k0 = t * BK;
    const char *ldsK = lds + (t & 1) * C::KTILEB;
    u32x4 kst_n[CPT], mreg_n[4], dreg_n[4];
    const bool more = t + 1 < nkt; // workgroup-uniform
    if (more) gload(k0 + BK, kst_n, mreg_n, dreg_n);

    // ---- P = exp2(score * scale + mask - LSE)
    f32x16 x[NSB];
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb) {
#pragma unroll
      for (int r = 0; r < 16; ++r) x[sb][r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        x[sb] = E::mfma(as_v8<T>(*(const u32x4 *)(ldsK + (sb * 32 + ql) * ROWB + ks * 32 + h * 16)), qreg[ks], x[sb]);
    }
    scr.rows_in(mreg);
    scr.turn();
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const v4 mv = as_v4<T>(scr.piece(sb, g));
#pragma unroll
        for (int i = 0; i < 4; ++i)
          x[sb][4 * g + i] = fast_exp2(fmaf(x[sb][4 * g + i], a.scale_l2, fmaf((float)mv[i], a.mask_a, a.mask_b)) - lq);
      }
    scr.turn();
    if (k0 + BK > a.sk) { // only a partly filled last tile has keys to switch off (workgroup-uniform)
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int kk = k0 + sb * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
          x[sb][r] = kk < a.sk ? x[sb][r] : 0.f;
        }
    }

    // ---- softmax out
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

    // ---- dropped, scaled copy out
    if (a.save_dropout) {
      scr.rows_in(dreg);
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

    if (more) {
      lstore((t + 1) & 1, kst_n);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        mreg[i] = mreg_n[i];
        dreg[i] = dreg_n[i];
      }
    }
    __syncthreads();
  }
}

} // namespace fmha
