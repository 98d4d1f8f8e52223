// Forward kernel for long key ranges under a full [.., sq, sk] mask tensor (and, optionally, a dropout
// tensor of the same shape): the reference's operators beyond their own 128-key shape.
//
// With such tensors the forward is memory time at head dim 64 (BH 512, S 512: 34 GFLOP against
// 402 MB with the mask, 671 MB with mask and dropout tensor), so the kernel is built for streaming,
// like the kernel that writes the saved outputs: [.., sq, sk] rows arrive as whole 128-byte row
// segments (16 bytes per lane, 8 lanes per row), one tile ahead, and a wave-private LDS scratch
// turns them into the accumulator layout; K and V tiles are staged through registers with them, so
// every request of an iteration is in flight for a whole iteration.  The softmax is the textbook
// online one (running row maximum, rescale on every tile, fp32 row sum): at two waves per SIMD the
// vector work hides under the memory time, which the lazily re-based, matrix-pipe-assisted softmax
// of the pipelined kernel is not needed for.
#pragma once
#include "fmha_fwd_kernel.h"

namespace fmha {

struct StreamCfg {
  static constexpr int D = 64;
  static constexpr int NW = 4;
  static constexpr int QT = NW * 32;
  static constexpr int BK = 64;
  static constexpr int ROWB = D * 2 + 16;          // padded K / V rows: conflict-free 16-byte and transpose reads
  static constexpr int TILEB = BK * ROWB;
  using Scratch = RowScratch<BK>;                  // wave-private: rows of a [.., sq, sk] tensor <-> accumulator layout
  static constexpr int LDS_BYTES = 4 * TILEB + NW * Scratch::BYTES; // {K, V} x 2 stages + one scratch per wave
};

template <typename T, bool DROPT>
__global__ __launch_bounds__(StreamCfg::NW * 64) __attribute__((amdgpu_waves_per_eu(2, 2)))
void fmha_fwd_stream_kernel(const FwdArgs a) {
  using E = Elem<T>;
  using v8 = typename E::v8;
  using v4 = typename E::v4;
  using C = StreamCfg;
  constexpr int D = C::D, KS = D / 16, DB = D / 32, BK = C::BK, NSB = BK / 32, NT = C::NW * 64, ROWB = C::ROWB;
  constexpr int TILEB = C::TILEB;
  constexpr int CPR = D / 8, CPT = BK * CPR / NT;
  constexpr float NEG_INF = -__builtin_inff();
  constexpr bool PF2 = !DROPT; // mask rows two tiles ahead

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

  // ---- staging.  K, V: global -> registers -> LDS (two stages).  [.., sq, sk] rows: instruction i covers
  // rows 8i .. 8i+7 of the wave's 32, eight lanes per row, 8 keys (16 bytes) per lane.
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
  const T *db_ = DROPT ? (const T *)a.drop_mask + (size_t)bh * a.sq * a.sk : nullptr;
  struct Stage {
    u32x4 k[CPT], v[CPT], m[4], d[4];
  };
  // Every load is unconditional (a load under a lane condition makes the compiler wait for it on the
  // spot): key rows past the end re-read the last row, chunks past sk re-read the row's first chunk;
  // those keys' scores are forced to -inf, so P = 0 meets finite values of V.
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
      if (!PF2) st.m[i] = *(const u32x4 *)(mb + (size_t)qrow[i] * a.mask_sq + koff);
      if (DROPT) st.d[i] = *(const u32x4 *)(db_ + (size_t)qrow[i] * a.sk + koff);
    }
  };
  // Without a dropout tensor the registers allow the mask rows -- the larger half of an iteration's bytes -- to be
  // requested two tiles ahead (BH 512, S 512: 99.6 -> 93.0 us; with the dropout tensor it measured level).
  auto gload_mask = [&](int k0, u32x4 (&mm)[4]) {
    const int koff = k0 + chunk * 8 < a.sk ? k0 + chunk * 8 : 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) mm[i] = *(const u32x4 *)(mb + (size_t)qrow[i] * a.mask_sq + koff);
  };
  auto lstore = [&](int stage, const Stage &st) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = tid + i * NT;
      *(u32x4 *)(lds + stage * 2 * TILEB + (c / CPR) * ROWB + (c % CPR) * 16) = st.k[i];
      *(u32x4 *)(lds + stage * 2 * TILEB + TILEB + (c / CPR) * ROWB + (c % CPR) * 16) = st.v[i];
    }
  };

  // ---- running state: row maximum m (log2 units), this lane's part of the row sum, unnormalised O^T
  float m = NEG_INF, lsum = 0.f;
  f32x16 o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[db][r] = 0.f;

  const int nkt = (a.sk + BK - 1) / BK;
  Stage cur;
  gload(0, cur);
  u32x4 m_next[4];
  if (PF2) {
    gload_mask(0, cur.m);
    gload_mask(nkt > 1 ? BK : 0, m_next);
  }
  lstore(0, cur);
  __syncthreads();

  for (int t = 0; t < nkt; ++t) {
    const int k0 = t * BK;
    const char *ldsK = lds + (t & 1) * 2 * TILEB;
    const char *ldsV = ldsK + TILEB;
    Stage nxt;
    const bool more = t + 1 < nkt; // workgroup-uniform
    if (more) gload(k0 + BK, nxt);
    u32x4 m_after[4];
    if (PF2) gload_mask(t + 2 < nkt ? k0 + 2 * BK : k0, m_after); // (unconditional: past the last tile it re-reads this one)

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

    // ---- online softmax: raise the maximum, rescale what has been accumulated under the old one
    tmax = xhalf_max(tmax);
    const float mnew = fmaxf(m, tmax);
    const float muse = mnew == NEG_INF ? 0.f : mnew;
    const float alpha = m == NEG_INF ? 0.f : fast_exp2(m - mnew);
    m = mnew;
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
    // (alpha is exactly one in every lane whose maximum stayed: the products are skipped when no lane's moved;
    // with the range check of the scores left to the one tile that needs it: BH 512 S 512 99.8 -> 95.3 us under
    // the mask alone, 136.9 -> 130.2 with the dropout tensor, BH 64 S 2048 167.3 -> 150.5 / 217.7 -> 199.2)
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[db][r] *= alpha;
    }

    // ---- (dropped) probabilities in the element type: B operand of the second product
    if (DROPT) {
      scr.rows_in(cur.d);
      scr.turn();
    }
    v8 pfrag[NSB][2];
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        float keep[4] = {1.f, 1.f, 1.f, 1.f};
        if (DROPT) {
          const v4 dm = as_v4<T>(scr.piece(sb, g));
#pragma unroll
          for (int i = 0; i < 4; ++i) keep[i] = (float)dm[i];
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) pfrag[sb][g >> 1][4 * (g & 1) + i] = (T)(x[sb][4 * g + i] * keep[i]);
      }
    if (DROPT) scr.turn();

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
      if (PF2) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          cur.m[i] = m_next[i];
          m_next[i] = m_after[i];
        }
      }
    }
    __syncthreads();
  }

  // ---- epilogue
  const int q = q0w + ql;
  const float lt = xhalf_sum(lsum);
  const float inv = lt > 0.f ? a.drop_scale / lt : 0.f;
  if (q < a.sq) {
    T *Ob = (T *)a.o + ((size_t)bh * a.sq + q) * D;
#pragma unroll
    for (int db = 0; db < DB; ++db) store_acc_block_row<T>(Ob + db * 32, o[db], inv, h);
    if (a.lse && h == 0) a.lse[(size_t)bh * a.sq + q] = lt > 0.f ? (m + fast_log2(lt)) * FMHA_LN2 : NEG_INF;
  }
}

} // namespace fmha
