// dK / dV kernel for wide heads (head dim 256).  A lane that owns one key cannot hold that key's K and V
// rows as register operands AND both of its gradient rows as accumulators: 2 x 64 + 2 x 128 registers
// before any score tile.  Here the two halves of the work go to two waves that own the SAME 32 keys:
//   wave P ("probabilities")  x = Q.K'^T + (mask - LSE),  P = exp2(x), dropout decisions,  dV^T += dO^T.(P o Z)
//   wave G ("gradients")      g = drop_scale dO.V^T - delta,  dS = P o (kept ? g : -delta),  dK^T += Q^T.dS
// Each holds one operand row (64 registers) and one accumulator row (128 registers): one wave per SIMD,
// no spills, and no tile product is formed twice inside the kernel.  P crosses from wave P to wave G
// through LDS once per 32 x 32 block, already rounded to the element type and in the register layout of
// the product that consumes it (16 bytes per lane and half block), with the dropout decision in its sign
// bit (P >= 0).  Everything else -- the swizzled Q / dO tiles copied straight into LDS, the extra
// contraction step that carries mask, LSE and delta, the mask tail, the causal tile pairing -- is
// fmha_bwd_dkdv_kernel's (fmha_bwd_kernel.h), whose comments describe it.
//
// One workgroup = 2 wave pairs = 64 keys, walking 64-query tiles; two barriers per tile: tiles ready /
// P written.  A full mask tensor's [64 queries x 64 keys] tile has ONE LDS buffer (two would not fit
// beside four 32 KB tiles): it is written in the second half of the previous iteration, after wave P has
// finished with the old one.
#pragma once
#include "fmha_bwd_kernel.h"

namespace fmha {

// Waves per workgroup and workgroup waves per SIMD: one operand row and one accumulator row are 3 D / 4
// registers, so head dim 256 runs one wave per SIMD (4 waves, 64 keys per workgroup) and the narrower
// heads two (8 waves, 128 keys).
template <int D> constexpr int bwd_wide_threads() { return D == 256 ? 256 : 512; }
template <int D> constexpr int bwd_wide_occupancy() { return D == 256 ? 1 : 2; }
template <int D, int MASK> struct BwdWideCfg {
  static constexpr int NT = bwd_wide_threads<D>(), NW = NT / 64, BQ = 64, NSB = BQ / 32, NPAIR = NW / 2, KT = NPAIR * 32;
  using Base = BwdCfg<D, BQ>;
  static constexpr int OFF_EXCH = Base::LDS_BYTES;
  static constexpr int EXCH_BYTES = NPAIR * NSB * 2 * 64 * 16; // [pair][query block][half block][lane] x 16 B
  static constexpr int OFF_MASK = OFF_EXCH + EXCH_BYTES;
  static constexpr int MASK_PITCH = KT + 8;
  static constexpr int MASK_BYTES = MASK == kMaskFull ? BQ * MASK_PITCH * 2 : 0;
  static constexpr int LDS_BYTES = OFF_MASK + MASK_BYTES;
};

template <typename T, int D, int MASK, bool CAUSAL, int DROP, bool STRIDED>
__global__ __launch_bounds__(bwd_wide_threads<D>()) __attribute__((amdgpu_waves_per_eu(bwd_wide_occupancy<D>(), bwd_wide_occupancy<D>()))) void fmha_bwd_dkdv_wide_kernel(const BwdArgs a) {
  using RW = Rows<STRIDED, D>;
  using E = Elem<T>;
  using v8 = typename E::v8;
  using v4 = typename E::v4;
  using W = BwdWideCfg<D, MASK>;
  using C = typename W::Base;
  constexpr int BQ = W::BQ, NSB = W::NSB, KS = C::KS, DB = C::DB, TILEB = C::TILEB, XROWB = C::XROWB;
  constexpr int NT = W::NT, KT = W::KT, MP = W::MASK_PITCH;
  constexpr float NEG_INF = -__builtin_inff();
  constexpr float BIGNEG = -60000.f;

  extern __shared__ __attribute__((aligned(16))) char lds[];
  char *ldsXb = lds + 4 * TILEB;                        // [stage][{score row, dP row}][BQ] extra-step rows
  float *ldsDl = (float *)(ldsXb + 2 * 2 * BQ * XROWB); // [stage][BQ] delta (dropout path)
  T *ldsM = (T *)(lds + W::OFF_MASK);

  const int tid = threadIdx.x;
  const int w = tid >> 6, l = tid & 63, kl = l & 31, h = l >> 5;
  const int pairi = w >> 1;
  const bool roleG = (w & 1) != 0; // wave-uniform
  u32x4 *exch = (u32x4 *)(lds + W::OFF_EXCH) + pairi * (NSB * 2 * 64) + l;

  int bid = blockIdx.x;
  const int nb = gridDim.x;
  if ((nb & 7) == 0) bid = (bid & 7) * (nb >> 3) + (bid >> 3);
  const bool paired = CAUSAL && a.pair;
  const int npair = paired ? (a.ntile + 1) / 2 : a.ntile;
  const int bh = bid / npair;
  const int pi = bid - bh * npair;
  const int npass = (paired && a.ntile - 1 - pi != pi) ? 2 : 1;
  MaskTail<T, NT> tail;
  int live_keys = a.sk;
  if (MASK == kMaskPerKey) tail.issue(a, (const T *)a.mask + (size_t)(bh / a.mask_div) * a.mask_sb, tid);

  for (int pass = 0; pass < npass; ++pass) {
    const int ktile = pass == 0 ? pi : a.ntile - 1 - pi;
    const int k0w = ktile * KT + pairi * 32;
    const int key = k0w + kl;

    const T *Qb = (const T *)a.q + RW::head(a.mq, bh, a.sq);
    const T *dOb = (const T *)a.dout + RW::head(a.mdo, bh, a.sq);
    const float *lseb = a.lse + (size_t)bh * a.sq;
    const float *delb = a.delta + (size_t)bh * a.sq;
    const int skv = bwd_valid_keys(a, bh);

    // ---- this wave's per-key operand: K' rows (wave P) or V rows (wave G), and its extra-step column
    v8 oreg[KS], bx;
    {
      const T *src = roleG ? (const T *)a.v + RW::head(a.mv, bh, a.sk) : (const T *)a.k + RW::head(a.mk, bh, a.sk);
      const int64_t ss = roleG ? RW::ss(a.mv) : RW::ss(a.mk);
      const float f = roleG ? (DROP == 1 ? a.drop_scale : 1.f) : a.scale_l2;
      const int kc = key < a.sk ? key : a.sk - 1; // keys past the end re-read the last row; their mask term is "-inf"
      u32x4 raw[KS];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) // (padding chunks of a narrower head: chunk 0 instead, zeroed below)
        raw[ks] = *(const u32x4 *)(src + (size_t)kc * ss + (ks * 16 + h * 8 < RW::cols(a) ? ks * 16 + h * 8 : 0));
      T mraw_key = (T)0.f;
      if (MASK == kMaskPerKey) mraw_key = ((const T *)a.mask)[(size_t)(bh / a.mask_div) * a.mask_sb + kc];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const v8 r = as_v8<T>(chunk_or_zero(raw[ks], ks * 16 + h * 8 < RW::cols(a)));
#pragma unroll
        for (int j = 0; j < 8; ++j) oreg[ks][j] = (T)((float)r[j] * f);
      }
      float mk = 0.f;
      if (MASK == kMaskPerKey) mk = fmaf((float)mraw_key, a.mask_a, a.mask_b);
      if (key >= skv) mk = BIGNEG;
#pragma unroll
      for (int j = 0; j < 8; ++j) bx[j] = (T)0.f;
      if (h == 0) {
        bx[0] = (T)1.f;
        bx[1] = (T)1.f;
        if (!roleG) { // (1, 1, mask_hi, mask_lo, c_hi, c_lo, 0, 0)
          T hi, lo;
          split_hi_lo<T>(mk, hi, lo);
          bx[2] = hi;
          bx[3] = lo;
          if (MASK == kMaskFull) {
            split_hi_lo<T>(a.mask_b, hi, lo);
            bx[4] = hi;
            bx[5] = lo;
          }
        }
      }
    }

    const T *mbase = (MASK == kMaskFull) ? (const T *)a.mask + (size_t)(bh / a.mask_div) * a.mask_sb : nullptr;
    constexpr int MPR = KT / 4;             // 8-byte pieces per mask row of the tile
    constexpr int MLOADS = BQ * MPR / NT;   // pieces per thread
    static_assert((BQ * MPR) % NT == 0 && NT >= BQ, "staging assumes the workgroup covers the tile evenly");
    u32x2 mraw[MASK == kMaskFull ? MLOADS : 1];

    const int nqt = (a.sq + BQ - 1) / BQ;
    if (MASK == kMaskPerKey && pass == 0) live_keys = tail.finish(a, (int *)lds, tid);
    const int qt0 = ktile * KT >= (live_keys < skv ? live_keys : skv) ? nqt : (CAUSAL ? (ktile * KT) / BQ : 0);

    const uint32_t lds_base = lds_address(lds);
    PanelLane pl;
    pl.init(l);
    TileCopy<T, D, BQ, NT> tcopy, tcopy_do;
    tcopy.init(tid, RW::ss(a.mq));
    tcopy_do.init(tid, RW::ss(a.mdo));
    auto dma_qdo = [&](int qt) {
      const uint32_t dst = lds_base + (uint32_t)(qt & 1) * 2 * TILEB;
      tcopy.issue(Qb, qt * BQ, a.sq, dst, tid, RW::cols(a));
      tcopy_do.issue(dOb, qt * BQ, a.sq, dst + TILEB, tid, RW::cols(a));
    };
    float lraw = 0.f, draw = 0.f;
    bool qvalid = false;
    auto gloadX = [&](int qt) {
      int qr = qt * BQ + (tid & (BQ - 1));
      qvalid = qr < a.sq;
      qr = qvalid ? qr : a.sq - 1;
      lraw = lseb[qr];
      draw = delb[qr];
      if (MASK == kMaskFull) {
        const int kbase = ktile * KT;
        const bool vec_ok = a.mask_vec && (kbase + KT <= a.sk);
#pragma unroll
        for (int i = 0; i < MLOADS; ++i) {
          const int c = i * NT + tid, row = c / MPR, col = (c % MPR) * 4;
          int q = qt * BQ + row;
          q = q < a.sq ? q : a.sq - 1;
          const T *src = mbase + (size_t)q * a.mask_sq + kbase + col;
          if (vec_ok) {
            mraw[i] = *(const u32x2 *)src;
          } else {
            v4 t;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const int kc = kbase + col + j < a.sk ? kbase + col + j : a.sk - 1;
              t[j] = mbase[(size_t)q * a.mask_sq + kc];
            }
            union { v4 v; u32x2 u; } cv;
            cv.v = t;
            mraw[i] = cv.u;
          }
        }
      }
    };
    auto lstoreM = [&]() {
      if (MASK == kMaskFull) {
#pragma unroll
        for (int i = 0; i < MLOADS; ++i) {
          const int c = i * NT + tid, row = c / MPR, col = (c % MPR) * 4;
          *(u32x2 *)(ldsM + row * MP + col) = mraw[i];
        }
      }
    };
    auto lstoreX = [&](int stage) {
      if (tid < BQ) {
        float nl = BIGNEG, dl = 0.f; // rows past the end and fully masked rows: P = 0
        if (qvalid && lraw != NEG_INF) {
          nl = -lraw * FMHA_LOG2E;
          dl = draw;
        }
        v8 xs, xd, z;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          xs[j] = (T)0.f;
          xd[j] = (T)0.f;
          z[j] = (T)0.f;
        }
        T hi, lo;
        split_hi_lo<T>(nl, hi, lo);
        xs[0] = hi;
        xs[1] = lo;
        xs[2] = (T)1.f;
        xs[3] = (T)1.f;
        xs[4] = (T)1.f;
        xs[5] = (T)1.f;
        split_hi_lo<T>(-dl, hi, lo);
        xd[0] = hi;
        xd[1] = lo;
        v8 *ds_ = (v8 *)(ldsXb + (stage * 2 + 0) * BQ * XROWB + tid * XROWB);
        v8 *dd_ = (v8 *)(ldsXb + (stage * 2 + 1) * BQ * XROWB + tid * XROWB);
        ds_[0] = xs;
        ds_[1] = z;
        dd_[0] = xd;
        dd_[1] = z;
        ldsDl[stage * BQ + tid] = dl;
      }
    };

    f32x16 acc[DB]; // dV^T (wave P) or dK^T (wave G) of this lane's key
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[db][r] = 0.f;

    if (qt0 < nqt) {
      dma_qdo(qt0);
      gloadX(qt0);
      lstoreX(qt0 & 1);
      lstoreM();
      gloadX(qt0 + 1); // row indices are clamped: looking past the last tile is harmless
    }
    dma_wait_all();
    __syncthreads();

    for (int qt = qt0; qt < nqt; ++qt) {
      const int cur = qt & 1;
      const int q0 = qt * BQ;
      if (qt + 1 < nqt) dma_qdo(qt + 1);
      const char *ldsQ = lds + cur * 2 * TILEB;
      const char *ldsDO = ldsQ + TILEB;
      const char *ldsRow = roleG ? ldsDO : ldsQ; // rows of the first product
      const char *ldsTr = roleG ? ldsQ : ldsDO;  // read transposed by the second
      const char *ldsX = ldsXb + (cur * 2 + (roleG ? 1 : 0)) * BQ * XROWB;
      const float *ldsD = ldsDl + cur * BQ;

      // ---- first product of this wave: x (wave P) or g (wave G)
      f32x16 y[NSB];
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          y[sb][r] = (MASK == kMaskFull && !roleG)
                         ? (float)ldsM[(sb * 32 + 8 * (r / 4) + 4 * h + r % 4) * MP + pairi * 32 + kl] * a.mask_a
                         : 0.f;
#pragma unroll
      for (int ks = 0; ks <= KS; ++ks)
#pragma unroll
        for (int sb = 0; sb < NSB; ++sb) {
          if (ks < KS) {
            y[sb] = E::mfma(panel_read_rows<T, BQ>(ldsRow, pl, sb, ks), oreg[ks], y[sb]);
          } else {
            const v8 xa = as_v8<T>(*(const u32x4 *)(ldsX + (sb * 32 + kl) * XROWB + h * 16));
            y[sb] = E::mfma(xa, bx, y[sb]);
          }
        }

      v8 frag[NSB][2];
      if (!roleG) {
        const bool diag = CAUSAL && (k0w + 31 > q0);
#pragma unroll
        for (int sb = 0; sb < NSB; ++sb) {
          uint32_t rb[4]; // rb[t], byte gq: the random byte of (query 8 gq + 4h + t of the block, this lane's key)
          if (DROP == 1) drop_bytes_k(a.drop, (uint32_t)bh, (uint32_t)(q0 + sb * 32), (uint32_t)key, h, l, rb);
          v8 send[2];
#pragma unroll
          for (int gq = 0; gq < 4; ++gq)
#pragma unroll
            for (int t = 0; t < 4; ++t) {
              const int q = q0 + sb * 32 + 8 * gq + 4 * h + t;
              float xv = y[sb][4 * gq + t];
              if (diag) xv = (key <= q) ? xv : BIGNEG;
              const float p = fast_exp2(xv);
              const int r = 4 * gq + t;
              if (DROP == 1) {
                const bool keep = drop_keep_byte(rb[t], gq, a.drop.thr);
                frag[sb][r >> 3][r & 7] = (T)(keep ? p : 0.f); // (drop_scale multiplies dV once, on store)
                send[r >> 3][r & 7] = (T)(keep ? p : -p);
              } else {
                frag[sb][r >> 3][r & 7] = (T)p;
              }
            }
#pragma unroll
          for (int c = 0; c < 2; ++c) exch[(sb * 2 + c) * 64] = as_u32x4(DROP == 1 ? send[c] : frag[sb][c]);
        }
      }
      __syncthreads(); // P has been written (and every first product has read the old mask tile)
      if (roleG) {
#pragma unroll
        for (int sb = 0; sb < NSB; ++sb) {
          v8 pv[2];
#pragma unroll
          for (int c = 0; c < 2; ++c) pv[c] = as_v8<T>(exch[(sb * 2 + c) * 64]);
#pragma unroll
          for (int gq = 0; gq < 4; ++gq) {
            f32x4 Dl = {0.f, 0.f, 0.f, 0.f};
            if (DROP == 1) Dl = *(const f32x4 *)(ldsD + sb * 32 + 8 * gq + 4 * h);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
              const int r = 4 * gq + t;
              const float pf = (float)pv[r >> 3][r & 7];
              float gv = y[sb][r];
              float p = pf;
              if (DROP == 1) {
                gv = pf < 0.f ? -Dl[t] : gv; // (a dropped P of exactly zero arrives as -0: either branch gives 0)
                p = __builtin_fabsf(pf);
              }
              frag[sb][r >> 3][r & 7] = (T)(p * gv);
            }
          }
        }
      }
      if (qt + 1 < nqt) {
        lstoreX(cur ^ 1); // rows of tile qt+1, loaded one iteration ago
        lstoreM();
        gloadX(qt + 2);
      }

      // ---- second product: dV^T += dO^T.(P o Z)  /  dK^T += Q^T.dS
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
          for (int db = 0; db < DB; ++db)
            acc[db] = E::mfma(panel_read_transposed<T, BQ>(ldsTr, pl, sb, db, c), frag[sb][c], acc[db]);

      dma_wait_all();
      __syncthreads();
    }

    if (key < a.sk) {
      T *dst = roleG ? (T *)a.dk + RW::head(a.mdk, bh, a.sk) + (size_t)key * RW::ss(a.mdk)
                     : (T *)a.dv + RW::head(a.mdv, bh, a.sk) + (size_t)key * RW::ss(a.mdv);
      const float f = roleG ? a.scale : (DROP == 1 ? a.drop_scale : 1.f);
#pragma unroll
      for (int db = 0; db < DB; ++db) store_acc_block_row<T>(dst + db * 32, acc[db], f, h, RW::cols(a) - db * 32);
    }
    __syncthreads(); // the next pass refills the tiles
  }
}

} // namespace fmha
