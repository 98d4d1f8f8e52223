// Forward kernel for short key ranges (sk <= 128) under a full [.., sq, sk] mask tensor: the shape
// class of the reference's three operators, which take [512,128,64] tensors with [512,128,128]
// masks (reference fmha/fmha_manual.cpp:39-47, test.py:20-23) and optionally return the
// normalised softmax and its dropped copy (fmha/fmha_manual.cpp:891-897).
//
// At these shapes the operators move 50-100 MB for 2 GFLOP: the time is memory time, and most of
// the bytes are the [.., sq, sk] tensors (mask, dropout mask, the two saved outputs).  So this
// kernel is organised around them rather than around the matrix pipe:
//   * one pass: the scores of a wave's 32 queries against ALL keys stay in registers (4 accumulator
//     blocks), so the softmax is exact (true row maximum, fp32 sum) and nothing is read twice;
//   * every load of the workgroup is requested up front (K and V as global->LDS copies, then Q, mask
//     and dropout rows into registers) and consumed in that order: the first product runs while the
//     mask rows arrive, the softmax while the dropout rows arrive, and stores start only after the
//     last load has been used;
//   * mask and dropout rows are read, and the saved outputs written, as whole 256-byte rows
//     (16 bytes per lane, 16 lanes per row).  The MFMA accumulator layout wants the opposite
//     (lane = query row, 8-byte pieces), which as a global access pattern touches 32 different
//     cache lines per instruction; a wave-private LDS scratch turns one layout into the other.
// The same one-pass organisation serves short key ranges WITHOUT a full mask tensor (no mask, a per-key
// [B,1,1,S] mask, valid key counts; no dropout or the Philox rule): MASK / DROP below.  The mask term of
// every key then sits in a 128-float LDS row that the workgroup fills once, nothing passes through the
// row scratch, and P goes into the second product unnormalised.  These builds also exist for run-time row layouts.
// The second product takes the dropped, normalised probabilities -- the very values of the
// saved "dropout" output -- as its operand, as the reference does (fmha/fmha_manual.cpp:478-490).
#pragma once
#include "fmha_fwd_kernel.h"

namespace fmha {

struct ShortCfg {
  static constexpr int D = 64;
  static constexpr int NW = 4;                      // waves per workgroup, 32 queries each (two-wave workgroups measured 15-20 % slower)
  static constexpr int QT = NW * 32;
  static constexpr int SKMAX = 128;
  static constexpr int NSB = SKMAX / 32;            // 32-key accumulator blocks
  static constexpr int BT = 64;                     // rows per swizzled LDS tile
  static constexpr int TILEB = BT * D * 2;
  using Scratch = RowScratch<SKMAX>;              // wave-private: rows of a [.., sq, sk] tensor <-> accumulator layout
  static constexpr int LDS_BYTES = 4 * TILEB + NW * Scratch::BYTES; // K, V (two tiles each) + one scratch per wave
  static constexpr int LDS_BYTES_KEYMASK = 4 * TILEB + SKMAX * 4;   // K, V + the per-key mask terms (no scratch)
};

// FULL: more than 96 keys, so all four 32-key blocks and both 64-row tiles exist (the reference's 128 keys).  The
// products then run without conditions around their blocks: under a condition every block's accumulators are
// merged with their "block skipped" values afterwards, 32 register copies per block of the second product.
// MASK: kMaskFull (the operators' [.., sq, sk] tensor), kMaskPerKey or kMaskNone.  DROP: 0 none, 1 the Philox
// rule, 2 a [.., sq, sk] dropout tensor (kMaskFull only).  SAVE: kMaskFull with a dropout tensor only.
template <typename T, int MASK, int DROP, bool SAVE, bool FULL, bool STRIDED = false> FMHA_DEV void fwd_short_body(const FwdArgs &a) {
  constexpr bool DROPT = DROP == 2;
  static_assert(!STRIDED || MASK != kMaskFull, "run-time row layouts: the builds without a full mask tensor only");
  constexpr bool ROWS = MASK == kMaskFull; // [.., sq, sk] tensors move through the row scratch
  static_assert(ROWS || (!DROPT && !SAVE), "dropout tensors and saved outputs come with the full mask tensor");
  using E = Elem<T>;
  using v8 = typename E::v8;
  using v4 = typename E::v4;
  using C = ShortCfg;
  constexpr int D = C::D, KS = D / 16, DB = D / 32, NSB = C::NSB, NT = C::NW * 64;
  constexpr int TILEB = C::TILEB;
  constexpr float NEG_INF = -__builtin_inff();

  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int tid = threadIdx.x;
  const int w = tid >> 6;
  const int l = tid & 63;
  const int ql = l & 31;
  const int h = l >> 5;

  // one XCD (one L2) owns a contiguous range of (head, query tile) pairs
  int bid = blockIdx.x;
  const int nb = gridDim.x;
  if ((nb & 7) == 0) bid = (bid & 7) * (nb >> 3) + (bid >> 3);
  // (a.nqt = 1 at the reference's own 128 queries: no division there; the same for masks that are not shared)
  const int bh = a.nqt == 1 ? bid : bid / a.nqt;
  const int qt = a.nqt == 1 ? 0 : bid - bh * a.nqt;
  const int q0w = qt * C::QT + w * 32;

  using RW = Rows<STRIDED, D>; // folded [bh, s, 64] tensors, or the row maps of the argument block
  const T *Qb = (const T *)a.q + RW::head(a.mq, bh, a.sq);
  const T *Kb = (const T *)a.k + RW::head(a.mk, bh, a.sk);
  const T *Vb = (const T *)a.v + RW::head(a.mv, bh, a.sk);

  // ---- every request of this workgroup, up front
  // (per-key mask: one value per thread, requested ahead of the copies so that the wait for the copies covers it)
  float *fM = (float *)(lds + 4 * TILEB); // !ROWS: mask term of key k in log2 units, -inf from the first invisible key on
  const int kend = ROWS ? a.sk : visible_keys<STRIDED>(a, bh, 0);
  T mraw = (T)0.f;
  if (MASK == kMaskPerKey && tid < C::SKMAX) {
    const int mhead = a.mask_div == 1 ? bh : bh / a.mask_div;
    mraw = ((const T *)a.mask + (size_t)mhead * a.mask_sb)[tid < a.sk ? tid : a.sk - 1];
  }
  TileCopy<T, D, C::BT, NT> tcopy;
  tcopy.init(tid, RW::ss(a.mk));
  const uint32_t lds0 = lds_address(lds);
  const bool two_tiles = FULL || a.sk > C::BT;
  tcopy.issue(Kb, 0, a.sk, lds0, tid);
  if (two_tiles) tcopy.issue(Kb, C::BT, a.sk, lds0 + TILEB, tid);
  tcopy.issue(Vb, 0, a.sk, lds0 + 2 * TILEB, tid);
  if (two_tiles) tcopy.issue(Vb, C::BT, a.sk, lds0 + 3 * TILEB, tid);

  v8 qreg[KS];
  {
    // Row addresses are a per-head base (uniform) plus a 32-bit byte offset: one multiply per row instead of
    // 64-bit arithmetic ahead of every request (the host keeps sq * row pitch below 2^30 elements on this path).
    int q = q0w + ql;
    q = q < a.sq ? q : a.sq - 1;
    const char *qb8 = (const char *)Qb;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      qreg[ks] = as_v8<T>(*(const u32x4 *)(qb8 + ((uint32_t)q * RW::ss(a.mq) + (uint32_t)(ks * 16 + h * 8)) * 2u));
  }

  // [.., sq, sk] rows as the wave reads and writes them: instruction i covers rows 4i .. 4i+3 of the
  // wave's 32, sixteen lanes per row, 8 keys (16 bytes) per lane
  typename C::Scratch scr;
  scr.init(lds + 4 * TILEB + w * C::Scratch::BYTES, l);
  const int rsub = scr.rsub, chunk = scr.chunk;
  const bool cvalid = chunk * 8 < a.sk;
  u32x4 mreg[8], dreg[8];
  if (ROWS) {
    // Lanes whose chunk lies past sk read chunk 0 instead (their values are never used: those keys'
    // scores are forced to -inf).  Unconditional loads matter: a load under a lane condition is merged
    // with its "else" value right behind it, which makes the compiler wait for it on the spot.
    const int ch8 = cvalid ? chunk * 8 : 0;
    const int mhead = a.mask_div == 1 ? bh : bh / a.mask_div;
    const char *mb = (const char *)((const T *)a.mask + (size_t)mhead * a.mask_sb);
    const char *db_ = DROPT ? (const char *)((const T *)a.drop_mask + (size_t)bh * a.sq * a.sk) : nullptr;
    int qrow[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int q = q0w + 4 * i + rsub;
      qrow[i] = q < a.sq ? q : a.sq - 1;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) mreg[i] = *(const u32x4 *)(mb + (uint32_t)(qrow[i] * (int)a.mask_sq + ch8) * 2u);
    if (DROPT) {
#pragma unroll
      for (int i = 0; i < 8; ++i) dreg[i] = *(const u32x4 *)(db_ + (uint32_t)(qrow[i] * a.sk + ch8) * 2u);
    }
  }
  // Loads complete in the order they were requested.  The K and V copies went out first: once at most
  // the 4 Q, 8 mask and 8 dropout-row loads requested after them are outstanding, they have landed;
  // the first product then runs while the [.., sq, sk] rows are still on their way.  (A test compiles
  // this kernel to assembly and checks that count.)
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(4 + (ROWS ? 8 : 0) + (DROPT ? 8 : 0)) : "memory");
  if (!ROWS && tid < C::SKMAX) {
    float mt = 0.f;
    if (MASK == kMaskPerKey) mt = fmaf((float)mraw, a.mask_a, a.mask_b);
    fM[tid] = tid < kend ? mt : NEG_INF;
  }
  __syncthreads();

  PanelLane pl;
  pl.init(l);
  // ---- x^T = K . Q^T for all keys (lane = query, registers = keys 32 sb + 8g + 4h + t)
  f32x16 x[NSB];
#pragma unroll
  for (int sb = 0; sb < NSB; ++sb) {
#pragma unroll
    for (int r = 0; r < 16; ++r) x[sb][r] = 0.f;
    if (FULL || sb * 32 < a.sk) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        x[sb] = E::mfma(panel_read_rows<T, C::BT>(lds + (sb >> 1) * TILEB, pl, sb & 1, ks), qreg[ks], x[sb]);
    }
  }

  // ---- scale and mask (log2 units); keys past the end drop out
  if (ROWS) {
    scr.rows_in(mreg);
    scr.turn();
  }
#pragma unroll
  for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      if (ROWS) {
        const v4 mv = as_v4<T>(scr.piece(sb, g));
#pragma unroll
        for (int t = 0; t < 4; ++t)
          x[sb][4 * g + t] = fmaf(x[sb][4 * g + t], a.scale_l2, fmaf((float)mv[t], a.mask_a, a.mask_b));
      } else {
        const f32x4 mk = *(const f32x4 *)(fM + sb * 32 + 8 * g + 4 * h);
#pragma unroll
        for (int t = 0; t < 4; ++t) x[sb][4 * g + t] = fmaf(x[sb][4 * g + t], a.scale_l2, mk[t]);
      }
    }
  if (ROWS) scr.turn();
  if (ROWS && a.sk < C::SKMAX) { // (workgroup-uniform: the reference's own 128 keys skip it; !ROWS: fM holds -inf there)
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int kk = sb * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
        x[sb][r] = kk < a.sk ? x[sb][r] : NEG_INF;
      }
  }
  float mx = NEG_INF;
#pragma unroll
  for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
    for (int r = 0; r < 16; r += 2) mx = max3(mx, x[sb][r], x[sb][r + 1]);
  mx = xhalf_max(mx);
  const float mref = mx == NEG_INF ? 0.f : mx;

  // ---- exact softmax of the row
  float sum = 0.f;
#pragma unroll
  for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float p = fast_exp2(x[sb][r] - mref);
      x[sb][r] = p;
      sum += p;
    }
  const float lt = xhalf_sum(sum);
  const float inv = lt > 0.f ? 1.f / lt : 0.f;

  // rows of the scratch leave as whole rows of a [.., sq, sk] output
  auto store_rows = [&](void *out) {
    char *ob = (char *)((T *)out + (size_t)bh * a.sq * a.sk);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int q = q0w + 4 * i + rsub;
      const u32x4 t = scr.row_out(i);
      if (cvalid && q < a.sq) *(u32x4 *)(ob + (uint32_t)(q * a.sk + chunk * 8) * 2u) = t;
    }
  };
  // ---- dropped, normalised probabilities in the element type: second operand and saved output.
  // (The dropout rows are the last loads to arrive; nothing is stored before they are consumed, so
  // that waiting for them never waits for a store.)
  if (DROPT) {
    scr.rows_in(dreg);
    scr.turn();
  }
  // (With a dropout tensor the products are formed as (x / sum) * (d * scale) whether the outputs are saved or
  // not -- the saving and the plain operator then give the same O bit for bit; without one, 1 / sum and the scale
  // are one factor per row, applied to the 64 values of O instead of the 128 of P.)
  v8 pfrag[NSB][2];
  uint32_t wd[4] = {0u, 0u, 0u, 0u};
  const float inv_scaled = inv * a.drop_scale;
#pragma unroll
  for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      if (DROPT) {
        const v4 dm = as_v4<T>(scr.piece(sb, g));
#pragma unroll
        for (int t = 0; t < 4; ++t)
          pfrag[sb][g >> 1][4 * (g & 1) + t] = (T)((x[sb][4 * g + t] * inv) * ((float)dm[t] * a.drop_scale));
      } else if (DROP == 1) { // Philox rule: unnormalised, dropped elements zero; O takes scale / sum on its way out
        if (g == 0) drop_words_q(a.drop, (uint32_t)bh, (uint32_t)(q0w + ql), (uint32_t)(sb * 32), h, l, wd);
        v4 s4;
#pragma unroll
        for (int t = 0; t < 4; ++t) s4[t] = (T)x[sb][4 * g + t];
        Pack8 pk;
        if constexpr (__is_same(T, _Float16)) pk.h = s4;
        else pk.b = s4;
        uint32_t r0 = pk.u.x, r1 = pk.u.y;
        drop_apply_pk4(wd[g], ((a.drop.thr - 1u) & 0xffffu) * 0x00010001u, r0, r1); // (thr = 0 gives -1: everything kept)
        pk.u = u32x2{r0, r1};
        if constexpr (__is_same(T, _Float16)) s4 = pk.h;
        else s4 = pk.b;
#pragma unroll
        for (int t = 0; t < 4; ++t) pfrag[sb][g >> 1][4 * (g & 1) + t] = s4[t];
      } else { // unnormalised (values in (0, 1]); O takes the factor on its way out
#pragma unroll
        for (int t = 0; t < 4; ++t) pfrag[sb][g >> 1][4 * (g & 1) + t] = (T)x[sb][4 * g + t];
      }
    }
  if (ROWS) scr.turn();

  if (SAVE && a.save_softmax) {
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        v4 s4;
#pragma unroll
        for (int t = 0; t < 4; ++t) s4[t] = (T)(x[sb][4 * g + t] * inv);
        scr.template put_piece<T>(sb, g, s4);
      }
    scr.turn();
    store_rows(a.save_softmax);
    scr.turn();
  }
  if (SAVE && a.save_dropout) {
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        v4 d4;
#pragma unroll
        for (int t = 0; t < 4; ++t) d4[t] = pfrag[sb][g >> 1][4 * (g & 1) + t];
        scr.template put_piece<T>(sb, g, d4);
      }
    scr.turn();
    store_rows(a.save_dropout);
  }

  // ---- O^T = V^T . P^T
  f32x16 o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[db][r] = 0.f;
#pragma unroll
  for (int sb = 0; sb < NSB; ++sb) {
    if (FULL || sb * 32 < a.sk) {
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int db = 0; db < DB; ++db)
          o[db] = E::mfma(panel_read_transposed<T, C::BT>(lds + (2 + (sb >> 1)) * TILEB, pl, sb & 1, db, c),
                          pfrag[sb][c], o[db]);
    }
  }

  const int q = q0w + ql;
  if (q < a.sq) {
    T *Ob = (T *)a.o + RW::head(a.mo, bh, a.sq) + (size_t)q * RW::ss(a.mo);
#pragma unroll
    for (int db = 0; db < DB; ++db) store_acc_block_row<T>(Ob + db * 32, o[db], DROPT ? 1.f : inv_scaled, h);
    if (a.lse && h == 0) a.lse[(size_t)bh * a.sq + q] = lt > 0.f ? (mref + fast_log2(lt)) * FMHA_LN2 : NEG_INF;
  }
}

// Under a full mask tensor: two workgroups per compute unit (the row scratch and up to 185 registers).
template <typename T, int DROP, bool SAVE, bool FULL>
__global__ __launch_bounds__(ShortCfg::NW * 64) __attribute__((amdgpu_waves_per_eu(2, 2)))
void fmha_fwd_short_kernel(const FwdArgs a) {
  fwd_short_body<T, kMaskFull, DROP, SAVE, FULL>(a);
}
// Without one: four workgroups per compute unit (33 KB of LDS, at most 128 registers), which is what keeps launches
// of more heads than the device holds at once level with the persistent pipelined kernel.
template <typename T, int MASK, int DROP, bool FULL, bool STRIDED>
__global__ __launch_bounds__(ShortCfg::NW * 64) __attribute__((amdgpu_waves_per_eu(4, 4)))
void fmha_fwd_short_kernel_keymask(const FwdArgs a) {
  static_assert(MASK != kMaskFull, "the build for full mask tensors is fmha_fwd_short_kernel");
  fwd_short_body<T, MASK, DROP, false, FULL, STRIDED>(a);
}

} // namespace fmha
