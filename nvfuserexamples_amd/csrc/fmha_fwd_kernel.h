// Forward attention kernel for gfx950 (wave64, MFMA 32x32x16).
//
// Takes the place of the three nvFuser-scheduled kernels of the reference
// (fmha/fmha_manual.cpp:20-409, :411-807, :809-1214).  Where the reference keeps a
// whole key row of 128 in one CTA (fmha_manual.cpp:107-111) and moves the score
// tile through shared memory twice (:160,165,274,322), this kernel walks the keys
// in LDS tiles of 64 with an online (running max / running sum) softmax and keeps
// scores and probabilities in registers from the first product to the second.
//
// Work decomposition
//   workgroup = NW waves, one (bh, query tile of NW*QB*32 rows); wave = QB blocks of
//   32 queries.  K and V tiles of 64 keys are staged in LDS (double buffered, padded
//   rows); Q lives in registers as the B operand for the whole kernel.
// Products are computed transposed so that every lane owns one query column:
//   S^T[key][q] = K . Q^T       A = K rows from LDS (ds_read_b128), B = Q registers
//   O^T[d][q]   = V^T . P^T     A = V^T via the LDS transpose read, B = P registers
// The accumulator layout of S^T (lane = query, registers = keys) is exactly the B
// operand layout of the second product under a fixed permutation of the key index,
// and V is fetched with that same permutation, so P never leaves registers.
//
// Softmax bookkeeping per lane (one query): a reference exponent m, a partial sum l
// of the ROUNDED probabilities (accumulated with v_dot2 on the packed pairs, so the
// denominator matches what the second product actually sums) and the unnormalised
// accumulator O^T.  The reference m is raised -- and l, O rescaled -- only when a
// tile's maximum exceeds it by more than 2^8, which keeps every probability below
// 256 (exact in fp16/bf16 range) and removes the rescale from almost every tile.
// Row max needs one exchange between lane l and l^32 per tile; the two half-wave
// partial sums are combined once in the epilogue.
#pragma once
#include <type_traits>

#include "fmha_common.h"

namespace fmha {

struct FwdArgs {
  const void *q, *k, *v;
  void *o;
  float *lse;
  const void *mask;
  const void *drop_mask;
  void *save_softmax, *save_dropout;
  int64_t mask_sb, mask_sq;
  int32_t mask_div;
  int32_t mask_vec;  // 1: 8-byte accesses to [.., sk] rows (mask, drop mask, saves) are aligned
  float mask_a, mask_b; // mask term in log2 units = mask_value * mask_a + mask_b
  int32_t bh, sq, sk;
  int32_t nqt;       // query tiles per head
  float scale_l2;    // scale * log2(e)
  float inv_scale_l2; // 1 / scale_l2
  float drop_scale;
  DropCtx drop;
  int32_t flags;
};

// how the mask tensor is read
enum { kMaskNone = 0, kMaskPerKey = 1, kMaskFull = 2 };

template <int D> struct FwdCfg {
  static constexpr int BK = 64;           // keys per LDS tile
  static constexpr int NSB = BK / 32;     // 32-key sub-blocks per tile
  static constexpr int KS = D / 16;       // contraction steps of K.Q^T
  static constexpr int DB = D / 32;       // 32-row blocks of O^T
  static constexpr int ROWB = D * 2 + 16; // LDS row pitch in bytes (16 B pad: conflict-free b128 reads)
  static constexpr int TILEB = BK * ROWB;
  static constexpr int LDS_BYTES = 4 * TILEB + 2 * BK * 4; // {K,V} x 2 stages + per-key mask terms x 2 stages
};

template <typename T> FMHA_DEV float dot2_ones(typename Elem<T>::v8 v, int pair, float acc);
template <> FMHA_DEV float dot2_ones<_Float16>(f16x8 v, int pair, float acc) {
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  const h2 one = {(_Float16)1.f, (_Float16)1.f};
  const h2 x = {v[2 * pair], v[2 * pair + 1]};
  return __builtin_amdgcn_fdot2(x, one, acc, false);
}
template <> FMHA_DEV float dot2_ones<__bf16>(bf16x8 v, int pair, float acc) {
  typedef __bf16 b2 __attribute__((ext_vector_type(2)));
  const b2 one = {(__bf16)1.f, (__bf16)1.f};
  const b2 x = {v[2 * pair], v[2 * pair + 1]};
  return __builtin_amdgcn_fdot2_f32_bf16(x, one, acc, false);
}

template <typename T, int D, int QB, int NW, int MASK, bool CAUSAL, int DROP>
__global__ __launch_bounds__(NW * 64) void fmha_fwd_kernel(const FwdArgs a) {
  using E = Elem<T>;
  using v8 = typename E::v8;
  using v4 = typename E::v4;
  using C = FwdCfg<D>;
  constexpr int BK = C::BK, NSB = C::NSB, KS = C::KS, DB = C::DB, ROWB = C::ROWB;
  constexpr int TILEB = C::TILEB;
  constexpr int NT = NW * 64;
  constexpr int QT = NW * QB * 32;
  constexpr int CPR = D / 8;                 // 16-byte chunks per row
  constexpr int CPT = BK * CPR / NT;         // chunks per thread per tile
  static_assert(BK * CPR % NT == 0, "tile must divide evenly over the workgroup");
  static_assert(NT >= BK, "per-key mask terms are staged by the first BK threads");
  constexpr float NEG_INF = -__builtin_inff();
  constexpr float RESCALE_TH = 8.f; // log2 units

  extern __shared__ __attribute__((aligned(16))) char lds[];
  float *ldsMask = (float *)(lds + 4 * TILEB);

  const int tid = threadIdx.x;
  const int w = tid >> 6;
  const int l = tid & 63;
  const int ql = l & 31;
  const int h = l >> 5;

  // Workgroups are dealt round-robin to the 8 XCDs; remap so that one XCD (one L2)
  // owns a contiguous range of (head, query tile) pairs and the query tiles of a head
  // re-read that head's K/V from the same L2.
  int bid = blockIdx.x;
  const int nb = gridDim.x;
  if ((nb & 7) == 0) bid = (bid & 7) * (nb >> 3) + (bid >> 3);
  const int bh = bid / a.nqt;
  int qt = bid - bh * a.nqt;
  if (CAUSAL) qt = a.nqt - 1 - qt; // longest rows first
  const int q0w = qt * QT + w * (QB * 32);

  const T *Qb = (const T *)a.q + (size_t)bh * a.sq * D;
  const T *Kb = (const T *)a.k + (size_t)bh * a.sk * D;
  const T *Vb = (const T *)a.v + (size_t)bh * a.sk * D;
  const T *mkey = (MASK == kMaskPerKey) ? (const T *)a.mask + (size_t)(bh / a.mask_div) * a.mask_sb : nullptr;

  // ---- Q operand registers
  v8 qreg[QB][KS];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int q = q0w + qb * 32 + ql;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      u32x4 t = {0u, 0u, 0u, 0u};
      if (q < a.sq) t = *(const u32x4 *)(Qb + (size_t)q * D + ks * 16 + h * 8);
      qreg[qb][ks] = as_v8<T>(t);
    }
  }

  // ---- key range
  int nkt = (a.sk + BK - 1) / BK;
  if (CAUSAL) {
    int qmax = qt * QT + QT - 1;
    if (qmax > a.sq - 1) qmax = a.sq - 1;
    int need = qmax / BK + 1;
    if (need < nkt) nkt = need;
  }

  // ---- tile staging: global -> registers -> LDS
  u32x4 kst[CPT], vst[CPT];
  float mst = 0.f;
  auto gload = [&](int k0) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = tid + i * NT;
      const int row = c / CPR, col = c % CPR;
      const int kr = k0 + row;
      u32x4 kk = {0u, 0u, 0u, 0u}, vv = {0u, 0u, 0u, 0u};
      if (kr < a.sk) {
        kk = *(const u32x4 *)(Kb + (size_t)kr * D + col * 8);
        vv = *(const u32x4 *)(Vb + (size_t)kr * D + col * 8);
      }
      kst[i] = kk;
      vst[i] = vv;
    }
    if (MASK == kMaskPerKey && tid < BK) {
      // additive term of key k0+tid, divided by the score scale so that it can seed the
      // accumulator of K.Q^T (the product then comes out as score + term/scale and one fma
      // finishes it); keys past the end get -inf, which also covers the ragged last tile
      const int kr = k0 + tid;
      mst = kr < a.sk ? fmaf((float)mkey[kr], a.mask_a, a.mask_b) * a.inv_scale_l2 : NEG_INF;
    }
  };
  auto lstore = [&](int stage) {
    char *kd = lds + stage * 2 * TILEB;
    char *vd = kd + TILEB;
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = tid + i * NT;
      const int row = c / CPR, col = c % CPR;
      *(u32x4 *)(kd + row * ROWB + col * 16) = kst[i];
      *(u32x4 *)(vd + row * ROWB + col * 16) = vst[i];
    }
    if (MASK == kMaskPerKey && tid < BK) ldsMask[stage * BK + tid] = mst;
  };

  // ---- per-row base pointers of [.., sk]-shaped tensors
  const T *mrow[QB];
  const T *drow[QB];
  size_t srow[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    int q = q0w + qb * 32 + ql;
    if (q > a.sq - 1) q = a.sq - 1;
    mrow[qb] = nullptr;
    drow[qb] = nullptr;
    if (MASK == kMaskFull)
      mrow[qb] = (const T *)a.mask + (size_t)(bh / a.mask_div) * a.mask_sb + (size_t)q * a.mask_sq;
    srow[qb] = ((size_t)bh * a.sq + q) * a.sk;
    if (DROP == 2 && a.drop_mask) drow[qb] = (const T *)a.drop_mask + srow[qb];
  }

  // four consecutive elements of a [.., sk] row starting at key kk (kk % 4 == 0), as floats.
  // SAFE = the whole group is known to be in range and 8-byte aligned.
  auto load4 = [&](const T *row, int kk, bool safe, float out[4]) {
    if (safe) {
      v4 t = as_v4<T>(*(const u32x2 *)(row + kk));
#pragma unroll
      for (int i = 0; i < 4; ++i) out[i] = (float)t[i];
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) out[i] = (kk + i < a.sk) ? (float)row[kk + i] : 0.f;
    }
  };
  auto store4 = [&](T *row, int kk, const float in[4]) {
    if (a.mask_vec && kk + 3 < a.sk) {
      v4 t;
#pragma unroll
      for (int i = 0; i < 4; ++i) t[i] = (T)in[i];
      *(v4 *)(row + kk) = t;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (kk + i < a.sk) row[kk + i] = (T)in[i];
    }
  };

  // ---- running state
  f32x16 o[QB][DB];
  float mref[QB], lsum[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    mref[qb] = NEG_INF;
    lsum[qb] = 0.f;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[qb][db][r] = 0.f;
  }
  float inv_l[QB]; // used by the save pass

  const bool saving = (DROP == 2) && (a.save_softmax != nullptr || a.save_dropout != nullptr);
  const int npass = saving ? 2 : 1;

  for (int pass = 0; pass < npass; ++pass) {
    if (pass == 1) {
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        const float lt = xhalf_sum(lsum[qb]);
        inv_l[qb] = lt > 0.f ? 1.f / lt : 0.f;
      }
    }
    gload(0);
    lstore(0);
    __syncthreads();

    for (int kt = 0; kt < nkt; ++kt) {
      const int cur = kt & 1;
      const int k0 = kt * BK;
      if (kt + 1 < nkt) gload(k0 + BK);

      const char *ldsK = lds + cur * 2 * TILEB;
      const char *ldsV = ldsK + TILEB;
      const float *ldsM = ldsMask + cur * BK;

      const bool active = !CAUSAL || (k0 <= q0w + QB * 32 - 1);
      if (active) {
        // ---- S^T = K . Q^T
        f32x16 s[QB][NSB];
#pragma unroll
        for (int sb = 0; sb < NSB; ++sb) {
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) {
            if (MASK == kMaskPerKey) {
              // row r of the accumulator is key 8*(r/4) + 4h + r%4: seed it with that key's term
#pragma unroll
              for (int g = 0; g < 4; ++g) {
                const f32x4 t4 = *(const f32x4 *)(ldsM + sb * 32 + 8 * g + 4 * h);
#pragma unroll
                for (int t = 0; t < 4; ++t) s[qb][sb][4 * g + t] = t4[t];
              }
            } else {
#pragma unroll
              for (int r = 0; r < 16; ++r) s[qb][sb][r] = 0.f;
            }
          }
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            const v8 ka = as_v8<T>(*(const u32x4 *)(ldsK + (sb * 32 + ql) * ROWB + ks * 32 + h * 16));
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) s[qb][sb] = E::mfma(ka, qreg[qb][ks], s[qb][sb]);
          }
        }

        // Tiles that need a per-element bounds / causal test take the guarded path; the
        // per-key mask path encodes the ragged tail in its -inf terms and needs none.
        const bool ragged = (MASK != kMaskPerKey) && (k0 + BK > a.sk);
        const bool diag = CAUSAL && (k0 + BK - 1 > q0w);
        const bool vec_ok = a.mask_vec && !ragged;
        v8 pfrag[QB][NSB][2];

        auto softmax_block = [&](int qb, auto guarded_tag) {
          constexpr bool GUARDED = decltype(guarded_tag)::value;
          const int q = q0w + qb * 32 + ql;
          // ---- raw scores (per-key mask term already inside), bounds, running max.
          // With a full mask tensor the scaled+masked score x is formed here; otherwise the
          // scale is folded into the exponent's fma below (scale > 0 keeps the max monotone).
          float mx = NEG_INF;
#pragma unroll
          for (int sb = 0; sb < NSB; ++sb) {
            if (MASK == kMaskFull || GUARDED) {
#pragma unroll
              for (int g = 0; g < 4; ++g) {
                const int kk = k0 + sb * 32 + 8 * g + 4 * h;
                float mv[4] = {0.f, 0.f, 0.f, 0.f};
                if (MASK == kMaskFull) {
                  load4(mrow[qb], kk, vec_ok, mv);
#pragma unroll
                  for (int t = 0; t < 4; ++t) mv[t] = fmaf(mv[t], a.mask_a, a.mask_b);
                }
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                  float x = s[qb][sb][4 * g + t];
                  if (MASK == kMaskFull) x = fmaf(x, a.scale_l2, mv[t]);
                  if (GUARDED) {
                    const int k = kk + t;
                    const bool ok = (k < a.sk) && (!CAUSAL || k <= q);
                    x = ok ? x : NEG_INF;
                  }
                  s[qb][sb][4 * g + t] = x;
                }
              }
            }
            mx = max3(mx, s[qb][sb][0], s[qb][sb][1]);
#pragma unroll
            for (int r = 2; r < 16; r += 2) mx = max3(mx, s[qb][sb][r], s[qb][sb][r + 1]);
          }
          constexpr bool PRESCALED = (MASK == kMaskFull);
          const float cs = PRESCALED ? 1.f : a.scale_l2;

          if (pass == 0) {
            mx = xhalf_max(mx) * cs;
            // raise the reference exponent only when this tile would overflow the 2^8 headroom
            // (with mref = -inf the test reads mx > -inf: the first finite maximum always raises it)
            if (__builtin_amdgcn_ballot_w64(mx > mref[qb] + RESCALE_TH) != 0ull) {
              const float mnew = fmaxf(mref[qb], mx);
              const float ms = (mnew == NEG_INF) ? 0.f : mnew;
              const float alpha = fast_exp2(mref[qb] - ms);
              mref[qb] = mnew;
              lsum[qb] *= alpha;
#pragma unroll
              for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int r = 0; r < 16; ++r) o[qb][db][r] *= alpha;
            }
          }
          const float nmsafe = (mref[qb] == NEG_INF) ? 0.f : -mref[qb];

#pragma unroll
          for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
            for (int r = 0; r < 16; ++r)
              s[qb][sb][r] = fast_exp2(PRESCALED ? s[qb][sb][r] + nmsafe : fmaf(s[qb][sb][r], cs, nmsafe));

          if (pass == 1) {
            // save-intermediates pass: normalised softmax and its dropped/scaled version
            T *ssm = a.save_softmax ? (T *)a.save_softmax + srow[qb] : nullptr;
            T *sdr = a.save_dropout ? (T *)a.save_dropout + srow[qb] : nullptr;
            if (q < a.sq) {
#pragma unroll
              for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                  const int kk = k0 + sb * 32 + 8 * g + 4 * h;
                  if (kk >= a.sk) continue;
                  float pv[4], dm[4] = {1.f, 1.f, 1.f, 1.f};
#pragma unroll
                  for (int t = 0; t < 4; ++t) pv[t] = s[qb][sb][4 * g + t] * inv_l[qb];
                  if (ssm) store4(ssm, kk, pv);
                  if (sdr) {
                    if (drow[qb]) load4(drow[qb], kk, vec_ok, dm);
#pragma unroll
                    for (int t = 0; t < 4; ++t) pv[t] = pv[t] * (dm[t] * a.drop_scale);
                    store4(sdr, kk, pv);
                  }
                }
            }
            return;
          }

          // ---- round to the element type, sum the rounded values (softmax denominator)
          float rs = 0.f;
          v8 pk[NSB][2];
#pragma unroll
          for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
            for (int c = 0; c < 2; ++c) {
#pragma unroll
              for (int j = 0; j < 8; ++j) pk[sb][c][j] = (T)s[qb][sb][8 * c + j];
#pragma unroll
              for (int j = 0; j < 4; ++j) rs = dot2_ones<T>(pk[sb][c], j, rs);
            }
          lsum[qb] += rs;

          // ---- dropout acts on the numerator only
          if (DROP == 1) {
#pragma unroll
            for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
              for (int g = 0; g < 4; ++g) {
                const int kk = k0 + sb * 32 + 8 * g + 4 * h;
                const uint32_t wd = drop_word(a.drop, (uint32_t)bh, (uint32_t)q, (uint32_t)(kk >> 2));
#pragma unroll
                for (int t = 0; t < 4; ++t)
                  if (!drop_keep_byte(wd, t, a.drop.thr)) pk[sb][g >> 1][4 * (g & 1) + t] = (T)0.f;
              }
          } else if (DROP == 2) {
            if (drow[qb]) {
#pragma unroll
              for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                  const int kk = k0 + sb * 32 + 8 * g + 4 * h;
                  float dm[4];
                  load4(drow[qb], kk, vec_ok, dm);
#pragma unroll
                  for (int t = 0; t < 4; ++t)
                    pk[sb][g >> 1][4 * (g & 1) + t] = (T)((float)pk[sb][g >> 1][4 * (g & 1) + t] * dm[t]);
                }
            }
          }
#pragma unroll
          for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
            for (int c = 0; c < 2; ++c) pfrag[qb][sb][c] = pk[sb][c];
        };

        if (ragged || diag) {
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) softmax_block(qb, std::true_type{});
        } else {
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) softmax_block(qb, std::false_type{});
        }

        if (pass == 0) {
          // ---- O^T += V^T . P^T
#pragma unroll
          for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
              for (int c = 0; c < 2; ++c) {
                const v8 va = lds_load_a_transposed<T, ROWB>(ldsV, sb * 32, db * 32, c, l);
#pragma unroll
                for (int qb = 0; qb < QB; ++qb) o[qb][db] = E::mfma(va, pfrag[qb][sb][c], o[qb][db]);
              }
        }
      }

      if (kt + 1 < nkt) lstore(cur ^ 1);
      __syncthreads();
    }
  }

  // ---- epilogue: normalise, round, store O and the row log-sum-exp
  T *Ob = (T *)a.o + (size_t)bh * a.sq * D;
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int q = q0w + qb * 32 + ql;
    const float lt = xhalf_sum(lsum[qb]);
    const float inv = lt > 0.f ? a.drop_scale / lt : 0.f;
    if (q < a.sq) {
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          v4 t;
#pragma unroll
          for (int i = 0; i < 4; ++i) t[i] = (T)(o[qb][db][4 * g + i] * inv);
          *(v4 *)(Ob + (size_t)q * D + db * 32 + 8 * g + 4 * h) = t;
        }
      if (a.lse && h == 0)
        a.lse[(size_t)bh * a.sq + q] = lt > 0.f ? (mref[qb] + fast_log2(lt)) * FMHA_LN2 : NEG_INF;
    }
  }
}

} // namespace fmha
