// One-pass backward for heads of up to 512 keys at head dim 64 (no mask, a per-key mask, valid
// key counts; Philox dropout or none): dQ, dK and dV from ONE evaluation of the scores.
//
// The general path (fmha_bwd_kernel.h) runs a dQ kernel and a dK/dV kernel that each form the
// score and dP products, the exponentials and the dropout decisions: per-element vector work,
// which is what bounds those kernels, done twice.  Here one workgroup of eight waves owns a head.
// Keys are taken 256 at a time (a chunk: 32 keys per wave, lane = key, dK^T / dV^T accumulators
// resident in registers as in the dK/dV kernel) and the workgroup walks the 64-query tiles:
//   x = Q.K'^T + (mask - LSE), g = drop_scale*dO.V^T - delta        (rank-one terms ride in an extra
//   P = exp2(x), dS = P * (kept ? g : -delta)                        contraction step, as in fmha_bwd_kernel.h)
//   dV^T += dO^T.(P o Z), dK^T += Q^T.dS                             (P, dS fed back from the accumulators)
// and each wave also writes its rounded dS block into an LDS tile [256 keys][64 queries].  One
// iteration later -- after the barrier that ends every iteration anyway -- the eight waves split
//   dQ^T[64 d x 64 q] (+)= K^T[64 d x 256 keys] . dS^T[256 keys x 64 q]
// into eight [32 d x 16 q] pieces (v_mfma_f32_16x16x32: two accumulator blocks per wave), with
// both operands fetched by LDS transpose reads from the chunk's K tile and the dS tile, so a
// piece is complete over the chunk's keys inside one wave: no atomics, no reduction between
// waves, deterministic.  With more than 256 live keys the second chunk adds to fp32 partial sums
// that the first one left in a caller-provided workspace (written and re-read by the same lanes,
// in a layout of whole 16-byte pieces per lane).
//
// delta_i = sum_d dO_id O_id is computed by the workgroup itself, two tiles ahead, while the first
// chunk runs (eight threads per query row) and written out for the second chunk.
#pragma once
#include "fmha_bwd_kernel.h"

namespace fmha {

struct BwdFusedCfg {
  static constexpr int D = 64;
  static constexpr int NW = 8;            // waves per workgroup
  static constexpr int NT = NW * 64;
  static constexpr int KC = NW * 32;      // keys per chunk
  static constexpr int BQ = 64;           // queries per tile
  static constexpr int MAX_KEYS = 2 * KC; // longer heads stay on the two-kernel path
  static constexpr int TILEB = BQ * D * 2;     // one Q or dO tile
  static constexpr int KTILEB = KC * D * 2;    // the chunk's K rows
  static constexpr int DSTILEB = KC * BQ * 2;  // dS of one query tile against the chunk's keys
  static constexpr int XROWB = 32;
  static constexpr int OFF_K = 4 * TILEB;                   // Q, dO x 2 stages
  static constexpr int OFF_DS = OFF_K + KTILEB;             // 2 buffers
  static constexpr int OFF_X = OFF_DS + 2 * DSTILEB;        // extra rows [stage][2][BQ]
  static constexpr int OFF_DL = OFF_X + 2 * 2 * BQ * XROWB; // delta [stage][BQ]
  static constexpr int LDS_BYTES = OFF_DL + 2 * BQ * 4;
  // fp32 partial dQ of one query tile: 8 waves x 2 blocks x 64 lanes x 16 bytes
  static constexpr int WS_TILE_BYTES = NW * 2 * 64 * 16;
};


template <typename T> struct Mfma16;
template <> struct Mfma16<_Float16> {
  static FMHA_DEV f32x4 run(f16x8 a, f16x8 b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
};
template <> struct Mfma16<__bf16> {
  static FMHA_DEV f32x4 run(bf16x8 a, bf16x8 b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
};

// Operand of v_mfma_f32_16x16x32 whose 16 rows (columns, for the B operand) are 16 consecutive
// COLUMNS of a swizzled row-major LDS tile (fmha_common.h: 128-byte rows, 16-byte chunk c of row r
// at position c ^ ((r >> 1) & 7)) and whose 32 contraction indices are 32 consecutive tile ROWS:
// lane l (i = l % 16, group g = l / 16) receives column i, rows 8g .. 8g+7, through two transpose
// reads (rows 8g + i/4 and 8g + 4 + i/4, eight bytes at column 4 (i % 4)).  `lo`, `hi` are the
// lane's byte offsets for 16-column group 0 of the tile; a group 2j further right is an xor with
// j << 5 (the swizzle works on whole 16-byte chunks and 16 columns are two of them).
struct TrLane16 {
  uint32_t lo, hi;
  FMHA_DEV void init(int l) {
    const int i = l & 15, g = l >> 4;
    const int r0 = 8 * g + (i >> 2), r1 = r0 + 4;
    const int x = (i & 3) >> 1;
    lo = (uint32_t)(r0 * kPanelRowB + ((x ^ ((r0 >> 1) & 7)) << 4) + 8 * (i & 1));
    hi = (uint32_t)(r1 * kPanelRowB + ((x ^ ((r1 >> 1) & 7)) << 4) + 8 * (i & 1));
  }
};
template <typename T> FMHA_DEV typename Elem<T>::v8 tr16_read(const char *tile_rows, uint32_t lo, uint32_t hi) {
  const u32x2 a = lds_read_tr16(tile_rows + lo);
  const u32x2 b = lds_read_tr16(tile_rows + hi);
  const u32x4 both = {a.x, a.y, b.x, b.y};
  return as_v8<T>(both);
}

// Sum over aligned groups of eight lanes (all eight end up with it).
FMHA_DEV float sum_over_8_lanes(float v) {
  v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xf, 0xf, true));  // lane ^ 1
  v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xf, 0xf, true));  // lane ^ 2
  v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x141, 0xf, 0xf, true)); // mirror inside 8 lanes
  return v;
}

template <typename T, int MASK, int DROP, bool STRIDED>
__global__ __launch_bounds__(BwdFusedCfg::NT) __attribute__((amdgpu_waves_per_eu(2, 2)))
void fmha_bwd_fused_kernel(const BwdArgs a) {
  using C = BwdFusedCfg;
  constexpr int D = C::D, NT = C::NT, KC = C::KC, BQ = C::BQ, NSB = BQ / 32, KS = D / 16, DB = D / 32;
  constexpr int TILEB = C::TILEB, XROWB = C::XROWB;
  using RW = Rows<STRIDED, D>;
  using E = Elem<T>;
  using v8 = typename E::v8;
  using v4 = typename E::v4;
  constexpr float NEG_INF = -__builtin_inff();
  constexpr float BIGNEG = -60000.f;
  static_assert(MASK == kMaskNone || MASK == kMaskPerKey, "full mask tensors stay on the two-kernel path");

  extern __shared__ __attribute__((aligned(16))) char lds[];
  char *ldsK = lds + C::OFF_K;
  char *ldsDS = lds + C::OFF_DS;
  char *ldsXb = lds + C::OFF_X;
  float *ldsDl = (float *)(lds + C::OFF_DL);

  const int tid = threadIdx.x;
  const int w = tid >> 6, l = tid & 63, kl = l & 31, h = l >> 5;
  const int bh = blockIdx.x;

  const T *Qb = (const T *)a.q + RW::head(a.mq, bh, a.sq);
  const T *Ob = (const T *)a.o + RW::head(a.mo, bh, a.sq);
  const T *dOb = (const T *)a.dout + RW::head(a.mdo, bh, a.sq);
  const T *Kb = (const T *)a.k + RW::head(a.mk, bh, a.sk);
  const T *Vb = (const T *)a.v + RW::head(a.mv, bh, a.sk);
  const float *lseb = a.lse + (size_t)bh * a.sq;
  float *delb = a.delta + (size_t)bh * a.sq;
  const T *mkey = (MASK == kMaskPerKey) ? (const T *)a.mask + (size_t)(bh / a.mask_div) * a.mask_sb : nullptr;

  // keys worth visiting: the valid count and what a hard-masked tail of the mask row leaves
  MaskTail<T, NT> tail;
  int live_keys = a.sk;
  if (MASK == kMaskPerKey) {
    tail.issue(a, mkey, tid);
    live_keys = tail.finish(a, (int *)lds, tid);
  }
  const int skv = bwd_valid_keys(a, bh); // keys at or past it are invalid: P = 0 through their mask term
  const int kvis = live_keys < skv ? live_keys : skv;
  const int nchunk = kvis > KC ? 2 : 1;
  const int nqt = (a.sq + BQ - 1) / BQ;

  const uint32_t lds_base = lds_address(lds);
  PanelLane pl;
  pl.init(l);
  TrLane16 tl;
  tl.init(l);
  TileCopy<T, D, BQ, NT> tcopy, tcopy_do;
  tcopy.init(tid, RW::ss(a.mq));
  tcopy_do.init(tid, RW::ss(a.mdo));
  TileCopy<T, D, KC, NT> tcopy_k;
  tcopy_k.init(tid, RW::ss(a.mk));

  // dQ pieces: wave w takes queries 16 (w / 2) .. +15 of the tile and head-dim columns 32 (w % 2) .. +31
  const int dq_q = 16 * (w >> 1) + (l & 15);
  const int dq_d = 32 * (w & 1) + 4 * (l >> 4); // + 16 blk + r
  const uint32_t ds_lo = tl.lo ^ (uint32_t)((w >> 1) << 5), ds_hi = tl.hi ^ (uint32_t)((w >> 1) << 5);
  uint32_t kt_lo[2], kt_hi[2];
#pragma unroll
  for (int blk = 0; blk < 2; ++blk) {
    kt_lo[blk] = tl.lo ^ (uint32_t)((2 * (w & 1) + blk) << 5);
    kt_hi[blk] = tl.hi ^ (uint32_t)((2 * (w & 1) + blk) << 5);
  }
  float *wsb = a.ws + ((size_t)bh * nqt * C::NW + w) * 128 * 4 + (size_t)l * 4;
  T *dQb = (T *)a.dq + RW::head(a.mdq, bh, a.sq);
  T *dKb = (T *)a.dk + RW::head(a.mdk, bh, a.sk);
  T *dVb = (T *)a.dv + RW::head(a.mdv, bh, a.sk);

  // delta_i = sum_d dO_id O_id for every query of the head: eight threads per row hold 16 bytes each of
  // its O and dO rows (all loads go out together, beside the first chunk's operand loads)
  {
    constexpr int RPP = NT / 8; // rows per pass
    const int part = tid & 7;
    for (int r0 = 0; r0 < a.sq; r0 += 4 * RPP) {
      u32x4 ov[4], dv_[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        int qr = r0 + i * RPP + (tid >> 3);
        qr = qr < a.sq ? qr : a.sq - 1;
        ov[i] = *(const u32x4 *)(Ob + (size_t)qr * RW::ss(a.mo) + part * 8);
        dv_[i] = *(const u32x4 *)(dOb + (size_t)qr * RW::ss(a.mdo) + part * 8);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const v8 o8 = as_v8<T>(ov[i]), d8 = as_v8<T>(dv_[i]);
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) sum = fmaf((float)o8[j], (float)d8[j], sum);
        sum = sum_over_8_lanes(sum);
        const int qr = r0 + i * RPP + (tid >> 3);
        if (part == 0 && qr < a.sq) delb[qr] = sum;
      }
    }
    __syncthreads(); // (a workgroup-wide fence as well: the chunks read delta back)
  }

  for (int chunk = 0; chunk < nchunk; ++chunk) {
    const int kbase = chunk * KC;
    const int k0w = kbase + w * 32;
    const int key = k0w + kl;
    // 32-key blocks of this chunk that hold a visible key; waves past them only take part in the
    // copies, the barriers and the dQ pieces
    int nblk = (kvis - kbase + 31) / 32;
    nblk = nblk < 0 ? 0 : (nblk > C::NW ? C::NW : nblk);
    const bool wave_live = w < nblk;
    const bool last_chunk = chunk == nchunk - 1;

    // ---- per-key operands: K' and V rows as B operands, the extra-step columns
    v8 kreg[KS], vreg[KS];
    v8 bxs; // (1, 1, mask_hi, mask_lo, 0 ...) on the lower half-wave; the dP step's rows (-d_hi, -d_lo, 0 ...) meet its two ones
    {
      const int kc = key < a.sk ? key : a.sk - 1;
      u32x4 tk[KS], tv[KS];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const size_t col = ks * 16 + h * 8;
        tk[ks] = *(const u32x4 *)(Kb + (size_t)kc * RW::ss(a.mk) + col);
        tv[ks] = *(const u32x4 *)(Vb + (size_t)kc * RW::ss(a.mv) + col);
      }
      T mraw_key = (T)0.f;
      if (MASK == kMaskPerKey) mraw_key = mkey[kc];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const v8 kraw = as_v8<T>(tk[ks]);
        const v8 vraw = as_v8<T>(tv[ks]);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          kreg[ks][j] = (T)((float)kraw[j] * a.scale_l2);
          vreg[ks][j] = DROP == 1 ? (T)((float)vraw[j] * a.drop_scale) : vraw[j];
        }
      }
      float mk = 0.f;
      if (MASK == kMaskPerKey) mk = fmaf((float)mraw_key, a.mask_a, a.mask_b);
      if (key >= skv) mk = BIGNEG;
#pragma unroll
      for (int j = 0; j < 8; ++j) bxs[j] = (T)0.f;
      if (h == 0) {
        T hi, lo;
        bxs[0] = (T)1.f;
        bxs[1] = (T)1.f;
        split_hi_lo<T>(mk, hi, lo);
        bxs[2] = hi;
        bxs[3] = lo;
      }
    }

    // ---- staging.  Q and dO tiles and the chunk's K rows are copied straight into LDS; the
    // per-query extra rows take the register path two tiles ahead.  In the first chunk eight
    // threads per query row hold 16 bytes each of its O and dO rows and form delta; the second
    // chunk reads delta back.
    auto dma_qdo = [&](int qt) {
      const uint32_t dst = lds_base + (uint32_t)(qt & 1) * 2 * TILEB;
      tcopy.issue(Qb, qt * BQ, a.sq, dst, tid);
      tcopy_do.issue(dOb, qt * BQ, a.sq, dst + TILEB, tid);
    };
    const int xrow = tid;
    float lraw = 0.f, draw = 0.f;
    bool qvalid = false;
    auto gloadX = [&](int qt) {
      int qr = qt * BQ + (xrow & (BQ - 1));
      qvalid = qr < a.sq;
      qr = qvalid ? qr : a.sq - 1;
      lraw = lseb[qr];
      draw = delb[qr];
    };
    auto lstoreX = [&](int stage) {
      if (xrow < BQ) {
        // rows past the end (whose Q/dO rows repeat the last valid row) and fully masked rows: P = 0
        float nl = BIGNEG, dl = 0.f;
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
        split_hi_lo<T>(-dl, hi, lo);
        xd[0] = hi;
        xd[1] = lo;
        v8 *ds_ = (v8 *)(ldsXb + (stage * 2 + 0) * BQ * XROWB + xrow * XROWB);
        v8 *dd_ = (v8 *)(ldsXb + (stage * 2 + 1) * BQ * XROWB + xrow * XROWB);
        ds_[0] = xs;
        ds_[1] = z;
        dd_[0] = xd;
        dd_[1] = z;
        ldsDl[stage * BQ + xrow] = dl;
      }
    };

    f32x16 dk[DB], dv[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        dk[db][r] = 0.f;
        dv[db][r] = 0.f;
      }

    {
      const int kclamp = a.sk; // rows past the end re-read the last row; their dS is zero
      tcopy_k.issue(Kb, kbase, kclamp, lds_base + C::OFF_K, tid);
    }
    dma_qdo(0);
    gloadX(0);
    lstoreX(0);
    gloadX(1); // row indices are clamped, so looking past the last tile is harmless
    dma_wait_all();
    __syncthreads();

    // ---- pieces of one iteration, for a 32-query block b of the tile:
    //   X(b)  score product (5 MFMAs)            E(b)  exponentials, keep decisions, rounding  (vector ALU)
    //   G(b)  dP product (5; 4 with dropout)     D(b)  dS, rounding, the lane's row of the dS tile (vector ALU)
    //   V(b), K(b)  dV and dK products (4 each)  PH(b) the block's Philox call (vector ALU)
    //   DQ    the dQ pieces of the previous tile (16 small MFMAs)
    // The matrix pipe and the vector ALU only overlap when their instructions alternate inside one
    // wave's stream, so an iteration is laid out as six steps that each pair matrix work with vector
    // work that does not depend on it:
    //   X(0) | PH(0)     G(0) | E(0)     X(1) V(0) | D(0) PH(1)     G(1) K(0) | E(1)     V(1) DQ | D(1)     K(1)
    // With dropout the dP product leaves delta out (u = drop_scale dO.V^T) and
    //   dS = (P o keep) u - P delta
    // needs no keep decision a second time; without dropout delta rides in the product's extra step and dS = P g.
    const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    auto px = [&](int sb, int cur, f32x16 &x) {
      const char *ldsQ = lds + cur * 2 * TILEB;
      const char *ldsXs = ldsXb + (cur * 2 + 0) * BQ * XROWB;
      x = zero16;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) x = E::mfma(panel_read_rows<T, BQ>(ldsQ, pl, sb, ks), kreg[ks], x);
      x = E::mfma(as_v8<T>(*(const u32x4 *)(ldsXs + (sb * 32 + kl) * XROWB + h * 16)), bxs, x);
    };
    auto pg = [&](int sb, int cur, f32x16 &g) {
      const char *ldsDO = lds + cur * 2 * TILEB + TILEB;
      const char *ldsXd = ldsXb + (cur * 2 + 1) * BQ * XROWB;
      g = zero16;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) g = E::mfma(panel_read_rows<T, BQ>(ldsDO, pl, sb, ks), vreg[ks], g);
      if (DROP == 0) g = E::mfma(as_v8<T>(*(const u32x4 *)(ldsXd + (sb * 32 + kl) * XROWB + h * 16)), bxs, g);
    };
    // Dropout: lane i of a quad evaluates the 4x4 block of query group g = i (fmha_common.h, drop_words_k)
    // and keeps its four words; where an element's byte is needed the word comes over from the
    // owning lane with the other bytes masked away in the same instruction.
    const uint32_t byte_mask = 0xffu << (8 * (key & 3));
    const uint32_t thr_in_place = a.drop.thr << (8 * (key & 3));
    auto ph = [&](int sb, int q0, uint32_t (&o)[4]) {
      if (DROP == 1)
        drop_block(a.drop, (uint32_t)bh, (uint32_t)((q0 + sb * 32) >> 2) + (uint32_t)h + 2u * ((uint32_t)l & 3u),
                   (uint32_t)key >> 2, o);
    };
    auto keep_of = [&](const uint32_t (&o)[4], int gq, int t) -> bool {
      const uint32_t wd = gq == 0 ? quad_perm<0x00>(o[t]) : gq == 1 ? quad_perm<0x55>(o[t])
                        : gq == 2 ? quad_perm<0xAA>(o[t]) : quad_perm<0xFF>(o[t]);
      return (wd & byte_mask) >= thr_in_place;
    };
    // E(b): P = exp2(x) rounded (pp), and with the dropped elements zeroed (pz; the same without dropout)
    auto pe = [&](const f32x16 &x, const uint32_t (&o)[4], v8 (&pz)[2], v8 (&pp)[2]) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float p = fast_exp2(x[r]);
        pp[r >> 3][r & 7] = (T)p;
        if (DROP == 1) pz[r >> 3][r & 7] = keep_of(o, r >> 2, r & 3) ? (T)p : (T)0.f;
      }
      if (DROP == 0) {
        pz[0] = pp[0];
        pz[1] = pp[1];
      }
    };
    // D(b): dS rounded (df), and the lane's key row of the dS tile
    auto pd = [&](int sb, int cur, const f32x16 &g, const v8 (&pz)[2], const v8 (&pp)[2], v8 (&df)[2]) {
      const float *ldsD = ldsDl + cur * BQ;
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        f32x4 Dl = {0.f, 0.f, 0.f, 0.f};
        if (DROP == 1) Dl = *(const f32x4 *)(ldsD + sb * 32 + 8 * gq + 4 * h);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const int r = 4 * gq + t;
          if (DROP == 1)
            df[r >> 3][r & 7] = (T)fmaf((float)pz[r >> 3][r & 7], g[r], -((float)pp[r >> 3][r & 7] * Dl[t]));
          else
            df[r >> 3][r & 7] = (T)((float)pp[r >> 3][r & 7] * g[r]);
        }
      }
      // queries 32 sb + 8 gq + 4h .. +3 are half of the row's 16-byte chunk 4 sb + gq
      char *dsW = ldsDS + cur * C::DSTILEB + (w * 32 + kl) * kPanelRowB + 8 * h;
      const int swz = ((w * 32 + kl) >> 1) & 7;
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        union { v8 v; u32x4 u; } cv;
        cv.v = df[gq >> 1];
        const u32x2 piece = (gq & 1) ? u32x2{cv.u.z, cv.u.w} : u32x2{cv.u.x, cv.u.y};
        *(u32x2 *)(dsW + (((4 * sb + gq) ^ swz) << 4)) = piece;
      }
    };
    auto pv = [&](int sb, int cur, const v8 (&pz)[2]) {
      const char *ldsDO = lds + cur * 2 * TILEB + TILEB;
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int db = 0; db < DB; ++db) dv[db] = E::mfma(panel_read_transposed<T, BQ>(ldsDO, pl, sb, db, c), pz[c], dv[db]);
    };
    auto pk = [&](int sb, int cur, const v8 (&df)[2]) {
      const char *ldsQ = lds + cur * 2 * TILEB;
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int db = 0; db < DB; ++db) dk[db] = E::mfma(panel_read_transposed<T, BQ>(ldsQ, pl, sb, db, c), df[c], dk[db]);
    };
    auto dq_products = [&](int qt, bool all_blocks, f32x4 (&acc)[2]) {
      const char *dsT = ldsDS + (qt & 1) * C::DSTILEB;
      acc[0] = f32x4{0.f, 0.f, 0.f, 0.f};
      acc[1] = f32x4{0.f, 0.f, 0.f, 0.f};
      if (all_blocks) { // (wave-uniform) straight-line code that the scheduler can weave into the rest
#pragma unroll
        for (int s = 0; s < C::NW; ++s) {
          const v8 b = tr16_read<T>(dsT + s * 32 * kPanelRowB, ds_lo, ds_hi);
          const v8 a0 = tr16_read<T>(ldsK + s * 32 * kPanelRowB, kt_lo[0], kt_hi[0]);
          const v8 a1 = tr16_read<T>(ldsK + s * 32 * kPanelRowB, kt_lo[1], kt_hi[1]);
          acc[0] = Mfma16<T>::run(a0, b, acc[0]);
          acc[1] = Mfma16<T>::run(a1, b, acc[1]);
        }
      } else {
        for (int s = 0; s < nblk; ++s) {
          const v8 b = tr16_read<T>(dsT + s * 32 * kPanelRowB, ds_lo, ds_hi);
          const v8 a0 = tr16_read<T>(ldsK + s * 32 * kPanelRowB, kt_lo[0], kt_hi[0]);
          const v8 a1 = tr16_read<T>(ldsK + s * 32 * kPanelRowB, kt_lo[1], kt_hi[1]);
          acc[0] = Mfma16<T>::run(a0, b, acc[0]);
          acc[1] = Mfma16<T>::run(a1, b, acc[1]);
        }
      }
    };
    auto dq_part_load = [&](int qt, f32x4 (&part)[2]) {
      const float *wst = wsb + (size_t)qt * (C::WS_TILE_BYTES / 4);
      part[0] = *(const f32x4 *)(wst);
      part[1] = *(const f32x4 *)(wst + 64 * 4);
    };
    auto dq_store = [&](int qt, const f32x4 (&sums)[2]) {
      float *wst = wsb + (size_t)qt * (C::WS_TILE_BYTES / 4);
      const int q = qt * BQ + dq_q;
#pragma unroll
      for (int blk = 0; blk < 2; ++blk) {
        const f32x4 sum = sums[blk];
        if (last_chunk) {
          if (q < a.sq) {
            v4 o;
#pragma unroll
            for (int r = 0; r < 4; ++r) o[r] = (T)(sum[r] * a.scale);
            union { v4 v; u32x2 u; } cv;
            cv.v = o;
            *(u32x2 *)(dQb + (size_t)q * RW::ss(a.mdq) + dq_d + 16 * blk) = cv.u;
          }
        } else {
          *(f32x4 *)(wst + blk * 64 * 4) = sum;
        }
      }
    };
    // Scheduling pattern of one step: the step's first LDS reads go out together, then matrix
    // instructions alternate with slices of the vector work and the remaining reads.
#define FMHA_SGB(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)
#define FMHA_STEP_PATTERN(lead_reads, nmfma, valu_per, trans_per)                                                    \
  FMHA_SGB(0x100, lead_reads);                                                                                      \
  _Pragma("unroll") for (int i_ = 0; i_ < (nmfma); ++i_) {                                                          \
    FMHA_SGB(0x008, 1);                                                                                             \
    FMHA_SGB(0x100, 2);                                                                                             \
    FMHA_SGB(0x002, valu_per);                                                                                      \
    FMHA_SGB(0x400, trans_per);                                                                                     \
    FMHA_SGB(0x200, 1);                                                                                             \
  }

    // iteration qt: dQ pieces of tile qt-1 (from the dS tile written one iteration ago) woven into
    // scores / dS / dK / dV of tile qt; one more round of dQ pieces after the last tile
    const bool all_blocks = nblk == C::NW;
    f32x4 pend[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    for (int qt = 0; qt < nqt; ++qt) {
      const int cur = qt & 1;
      const int q0 = qt * BQ;
      // The dQ pieces finished in the previous iteration leave now, ahead of this iteration's loads: the
      // wait that ends an iteration is for all of the wave's memory operations, and a store issued just
      // before it would be waited for at its full latency.
      if (qt > 1) dq_store(qt - 2, pend);
      if (qt + 1 < nqt) {
        lstoreX(cur ^ 1); // rows of tile qt+1, loaded one iteration ago
        gloadX(qt + 2);
        dma_qdo(qt + 1);
      }
      f32x4 part[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
      f32x4 acc[2];
      if (wave_live && all_blocks) {
        // One hand-ordered stream.  Slot j holds: the LDS fetch of the operand of product j+2, product j, a
        // slice of vector work that does not depend on it -- closed by a scheduling barrier so that
        // the order stands.  Products, in order (b = 32-query block):
        //   X(0) | G(0) | X(1) and V(0) alternating | G(1) and K(0) alternating | V(1) | dQ pieces | K(1)
        // vector slices beside them:
        //   PH(0) | E(0)  | D(0), PH(1)               | E(1)                      | D(1) ...           |
        // (the first iteration forms dQ pieces from whatever the dS buffer holds and drops them)
        constexpr int NG = DROP == 1 ? KS : KS + 1;  // products of G(b)
        constexpr int J_G0 = KS + 1, J_S3 = J_G0 + NG, J_S4 = J_S3 + (KS + 1) + 4, J_S5 = J_S4 + NG + 4, NM = J_S5 + 4 + 4;
        f32x16 x = zero16, g = zero16;
        v8 pz[2][2], pp[2][2], df[2][2];
        v8 op[3];
        const char *ldsQ = lds + cur * 2 * TILEB;
        const char *ldsDO = ldsQ + TILEB;
        const char *ldsXs = ldsXb + (cur * 2 + 0) * BQ * XROWB;
        const char *ldsXd = ldsXb + (cur * 2 + 1) * BQ * XROWB;
        // product j: kind 0 X, 1 G, 2 V, 3 K; block sb; index within the product group
        auto kind_of = [&](int j, int &sb, int &idx) -> int {
          if (j < J_G0) { sb = 0; idx = j; return 0; }
          if (j < J_S3) { sb = 0; idx = j - J_G0; return 1; }
          if (j < J_S4) { // X(1) x5 and V(0) x4 alternating, X first
            const int k = j - J_S3;
            if ((k & 1) == 0) { sb = 1; idx = k >> 1; return 0; }
            sb = 0; idx = k >> 1; return 2;
          }
          if (j < J_S5) { // G(1) and K(0) alternating while both last
            const int k = j - J_S4;
            if (k < 2 * 4) {
              if ((k & 1) == 0) { sb = 1; idx = k >> 1; return 1; }
              sb = 0; idx = k >> 1; return 3;
            }
            sb = 1; idx = k - 4; return 1; // (the extra step of G without dropout)
          }
          if (j < J_S5 + 4) { sb = 1; idx = j - J_S5; return 2; }
          sb = 1; idx = j - J_S5 - 4; return 3;
        };
        auto fetch = [&](int j) -> v8 {
          int sb = 0, idx = 0;
          const int kind = kind_of(j, sb, idx);
          if (kind == 0)
            return idx < KS ? panel_read_rows<T, BQ>(ldsQ, pl, sb, idx)
                            : as_v8<T>(*(const u32x4 *)(ldsXs + (sb * 32 + kl) * XROWB + h * 16));
          if (kind == 1)
            return idx < KS ? panel_read_rows<T, BQ>(ldsDO, pl, sb, idx)
                            : as_v8<T>(*(const u32x4 *)(ldsXd + (sb * 32 + kl) * XROWB + h * 16));
          // V, K: idx = 2 c + db
          return panel_read_transposed<T, BQ>(kind == 2 ? ldsDO : ldsQ, pl, sb, idx & 1, idx >> 1);
        };
        auto product = [&](int j, const v8 &aop) {
          int sb = 0, idx = 0;
          const int kind = kind_of(j, sb, idx);
          if (kind == 0) x = E::mfma(aop, idx < KS ? kreg[idx < KS ? idx : 0] : bxs, idx == 0 ? zero16 : x);
          else if (kind == 1) g = E::mfma(aop, idx < KS ? vreg[idx < KS ? idx : 0] : bxs, idx == 0 ? zero16 : g);
          else if (kind == 2) dv[idx & 1] = E::mfma(aop, pz[sb][idx >> 1], dv[idx & 1]);
          else dk[idx & 1] = E::mfma(aop, df[sb][idx >> 1], dk[idx & 1]);
        };
        // ---- vector slices
        uint32_t c0 = 0, c1 = 0, c2 = 0, c3 = 0, k0 = 0, k1 = 0; // Philox state of the call in flight
        uint32_t o[2][4];
        auto ph_start = [&](int sb) {
          const uint64_t blk = ((uint64_t)bh * a.drop.qb4 + ((uint32_t)((q0 + sb * 32) >> 2) + (uint32_t)h + 2u * ((uint32_t)l & 3u))) * a.drop.kb4 + ((uint32_t)key >> 2);
          c0 = a.drop.off_lo; c1 = a.drop.off_hi; c2 = (uint32_t)blk; c3 = (uint32_t)(blk >> 32);
          k0 = a.drop.seed_lo; k1 = a.drop.seed_hi;
        };
        auto ph_rounds = [&](int n) {
#pragma unroll
          for (int r = 0; r < n; ++r) {
            const uint64_t p0 = (uint64_t)Philox::M0 * c0, p1 = (uint64_t)Philox::M1 * c2;
            const uint32_t n0 = __builtin_amdgcn_bitop3_b32((uint32_t)(p1 >> 32), c1, k0, 0x96);
            const uint32_t n2 = __builtin_amdgcn_bitop3_b32((uint32_t)(p0 >> 32), c3, k1, 0x96);
            c1 = (uint32_t)p1; c3 = (uint32_t)p0; c0 = n0; c2 = n2;
            k0 += Philox::W0; k1 += Philox::W1;
          }
        };
        auto ph_done = [&](int sb) { o[sb][0] = c0; o[sb][1] = c1; o[sb][2] = c2; o[sb][3] = c3; };
        auto e_slice = [&](int sb, int gq) { // four elements: P, P o keep, both rounded
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const int r = 4 * gq + t;
            const float p = fast_exp2(x[r]);
            pp[sb][r >> 3][r & 7] = (T)p;
            if (DROP == 1) pz[sb][r >> 3][r & 7] = keep_of(o[sb], gq, t) ? (T)p : (T)0.f;
          }
          if (DROP == 0 && (gq & 1)) pz[sb][gq >> 1] = pp[sb][gq >> 1];
        };
        f32x4 dl_ring[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
        auto dl_fetch = [&](int sb, int gq) { // delta of the four queries of D slice (sb, gq), one slot ahead
          if (DROP == 1) dl_ring[gq & 1] = *(const f32x4 *)(ldsDl + cur * BQ + sb * 32 + 8 * gq + 4 * h);
        };
        auto d_slice = [&](int sb, int gq) { // four elements of dS and their 8 bytes of the dS tile
          const f32x4 Dl = dl_ring[gq & 1];
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const int r = 4 * gq + t;
            if (DROP == 1)
              df[sb][r >> 3][r & 7] = (T)fmaf((float)pz[sb][r >> 3][r & 7], g[r], -((float)pp[sb][r >> 3][r & 7] * Dl[t]));
            else
              df[sb][r >> 3][r & 7] = (T)((float)pp[sb][r >> 3][r & 7] * g[r]);
          }
          char *dsW = ldsDS + cur * C::DSTILEB + (w * 32 + kl) * kPanelRowB + 8 * h;
          const int swz = ((w * 32 + kl) >> 1) & 7;
          union { v8 v; u32x4 u; } cv;
          cv.v = df[sb][gq >> 1];
          const u32x2 piece = (gq & 1) ? u32x2{cv.u.z, cv.u.w} : u32x2{cv.u.x, cv.u.y};
          *(u32x2 *)(dsW + (((4 * sb + gq) ^ swz) << 4)) = piece;
        };
        auto slice = [&](int j) {
          if (j < J_G0) { // beside X(0): the Philox call of block 0, two rounds a slot
            if (DROP == 1) {
              if (j == 0) ph_start(0);
              ph_rounds(2);
              if (j == J_G0 - 1) ph_done(0);
            }
          } else if (j < J_S3) { // beside G(0): E(0)
            const int k = j - J_G0;
            if (k < 4) e_slice(0, k);
          } else if (j < J_S4) { // beside X(1), V(0): D(0), then the Philox call of block 1
            const int k = j - J_S3;
            if (k < 4) d_slice(0, k);
            else if (DROP == 1) {
              if (k == 4) ph_start(1);
              ph_rounds(2);
              if (k == 8) ph_done(1);
            }
          } else if (j < J_S5) { // beside G(1), K(0): E(1), on every other slot
            const int k = j - J_S4;
            if ((k & 1) == 0 && (k >> 1) < 4) e_slice(1, k >> 1);
          } else if (j < J_S5 + 4) { // beside V(1): D(1)
            d_slice(1, j - J_S5);
          }
        };

        __builtin_amdgcn_sched_barrier(0);
        op[0] = fetch(0);
        op[1] = fetch(1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < J_S5 + 4; ++j) {
          // (the D slices sit in slots J_S3 .. J_S3+3 and J_S5 .. J_S5+3)
          if (j + 1 >= J_S3 && j + 1 < J_S3 + 4) dl_fetch(0, j + 1 - J_S3);
          if (j + 1 >= J_S5 && j + 1 < J_S5 + 4) dl_fetch(1, j + 1 - J_S5);
          if (j + 2 < NM) op[(j + 2) % 3] = fetch(j + 2);
          product(j, op[j % 3]);
          slice(j);
          __builtin_amdgcn_sched_barrier(0);
        }
        // dQ pieces of the previous tile, operands one step ahead; the last two operands of K(1) are already in flight
        {
          const char *dsT = ldsDS + (cur ^ 1) * C::DSTILEB;
          if (chunk > 0 && qt > 0) dq_part_load(qt - 1, part);
          acc[0] = f32x4{0.f, 0.f, 0.f, 0.f};
          acc[1] = f32x4{0.f, 0.f, 0.f, 0.f};
          v8 tb[2], ta0[2], ta1[2];
          tb[0] = tr16_read<T>(dsT, ds_lo, ds_hi);
          ta0[0] = tr16_read<T>(ldsK, kt_lo[0], kt_hi[0]);
          ta1[0] = tr16_read<T>(ldsK, kt_lo[1], kt_hi[1]);
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int s_ = 0; s_ < C::NW; ++s_) {
            if (s_ + 1 < C::NW) {
              tb[(s_ + 1) & 1] = tr16_read<T>(dsT + (s_ + 1) * 32 * kPanelRowB, ds_lo, ds_hi);
              ta0[(s_ + 1) & 1] = tr16_read<T>(ldsK + (s_ + 1) * 32 * kPanelRowB, kt_lo[0], kt_hi[0]);
              ta1[(s_ + 1) & 1] = tr16_read<T>(ldsK + (s_ + 1) * 32 * kPanelRowB, kt_lo[1], kt_hi[1]);
            }
            acc[0] = Mfma16<T>::run(ta0[s_ & 1], tb[s_ & 1], acc[0]);
            acc[1] = Mfma16<T>::run(ta1[s_ & 1], tb[s_ & 1], acc[1]);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
#pragma unroll
        for (int j = J_S5 + 4; j < NM; ++j) {
          if (j + 2 < NM) op[(j + 2) % 3] = fetch(j + 2);
          product(j, op[j % 3]);
          __builtin_amdgcn_sched_barrier(0);
        }
      } else {
        if (chunk > 0 && qt > 0) dq_part_load(qt - 1, part);
        if (qt > 0) dq_products(qt - 1, all_blocks, acc);
        if (wave_live) {
#pragma unroll
          for (int sb = 0; sb < NSB; ++sb) {
            f32x16 x, g;
            uint32_t o[4];
            v8 pz[2], pp[2], df[2];
            px(sb, cur, x);
            pg(sb, cur, g);
            ph(sb, q0, o);
            pe(x, o, pz, pp);
            pd(sb, cur, g, pz, pp, df);
            pv(sb, cur, pz);
            pk(sb, cur, df);
          }
        }
      }
      if (qt > 0) {
        pend[0] = acc[0] + part[0];
        pend[1] = acc[1] + part[1];
      }

      dma_wait_all();
      __syncthreads();
    }
    {
      f32x4 part[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
      f32x4 acc[2];
      if (nqt > 1) dq_store(nqt - 2, pend);
      if (chunk > 0) dq_part_load(nqt - 1, part);
      dq_products(nqt - 1, all_blocks, acc);
      pend[0] = acc[0] + part[0];
      pend[1] = acc[1] + part[1];
      dq_store(nqt - 1, pend);
    }
#undef FMHA_STEP_PATTERN
#undef FMHA_SGB

    const float dv_scale = DROP == 1 ? a.drop_scale : 1.f;
    if (key < a.sk) {
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        store_acc_block_row<T>(dKb + (size_t)key * RW::ss(a.mdk) + db * 32, dk[db], a.scale, h);
        store_acc_block_row<T>(dVb + (size_t)key * RW::ss(a.mdv) + db * 32, dv[db], dv_scale, h);
      }
    }
    __syncthreads(); // the next chunk refills the K rows and the dS tiles
  }

  // keys past the chunks that were visited: zero gradient rows
  for (int i = nchunk * KC * 8 + tid; i < a.sk * 8; i += NT) {
    const int row = i >> 3, piece = i & 7;
    const u32x4 z = {0u, 0u, 0u, 0u};
    *(u32x4 *)(dKb + (size_t)row * RW::ss(a.mdk) + piece * 8) = z;
    *(u32x4 *)(dVb + (size_t)row * RW::ss(a.mdv) + piece * 8) = z;
  }
}

} // namespace fmha
