// Decode steps: one to four query rows per head against a long key range.
//
// Such a forward is memory time -- K and V are read once, 4*D bytes per key against 4*D flops per query row --
// so this kernel is built around the loads, not around the matrix pipe: a wave reads whole rows with 16-byte
// loads (D / 8 neighbouring lanes cover one row, so a load instruction fetches 64 / (D / 8) complete rows),
// keeps eight K loads and eight V loads in flight (up to 16 KB per wave, 128 KB per compute unit),
// and does the arithmetic on the vector pipe in fp32: dot products on v_dot2c_f32_f16 / _bf16 (exact products of
// the packed elements, fp32 sums; multiply-adds on unpacked elements for e4m3 rows), summed over the lanes of a
// row by three or four DPP additions, an online softmax per lane group, P.V by multiply-add.
// Nothing is staged in LDS and nothing is rounded on the way (scores, probabilities and sums are fp32).
//
// Work split: a workgroup of four waves owns one (head, piece of the key range); its waves take the piece's
// blocks of keys in turn, and inside a wave the 64 / (D / 8) lane groups take every such-th key.  Each lane
// group runs its own online softmax over the keys it sees (running maximum m, sum l, 8 output columns per
// lane and query row); the 4 waves x lane groups meet once, at the end, through LDS.  With the key range in
// pieces (few heads: see the launch code) the piece's normalised output and log-sum-exp go to the caller's
// workspace as fp32 and a second kernel merges the pieces; otherwise O and the LSE are written directly.
#pragma once
#include "fmha_common.h"

namespace fmha {

// q, k and v may also hold e4m3 bytes (element type uint8_t here; o and the mask then have a 16-bit type of
// their own): the same kernel with 8-byte row loads, twice as many of them in flight, and the dequantisation
// factors folded into scale_l2 and out_scale.
struct DecodeArgs {
  const void *q, *k, *v;
  void *o;          // final output (element type), used when pieces == 1
  float *lse;       // optional final LSE [bh, sq], used when pieces == 1
  float *o_part;    // pieces > 1: [bh * pieces, sq, D] fp32
  float *lse_part;  // pieces > 1: [bh * pieces, sq]
  const void *mask; // optional per-key mask, element (b, j) at mask[(b / mask_div) * mask_sb + j]
  int64_t mask_sb;
  int32_t mask_div;
  float mask_a, mask_b; // mask term in log2 units = value * mask_a + mask_b
  const int32_t *kv_len;
  int32_t kv_div;
  int32_t bh, sq, sk;
  int32_t pieces, chunk; // pieces of `chunk` keys each (pieces == 1: chunk >= sk)
  float scale_l2;   // scale * log2(e) (times the dequantisation factors of q and k)
  float out_scale;  // 1 (the dequantisation factor of v)
  RowMap mq, mk, mv, mo;
};

constexpr int kDecodeWaves = 4;

// A lane's eight elements of a row: one 16-byte load of 16-bit elements, one 8-byte load of e4m3 bytes; and how
// many K (and V) loads a wave keeps in flight per block (the same bytes either way).
template <typename TI> struct DecodeIn {
  using Load = u32x4;
  static constexpr int LOADS = 8;
};
template <> struct DecodeIn<uint8_t> {
  using Load = u32x2;
  static constexpr int LOADS = 16;
};

template <typename T> FMHA_DEV void unpack8(u32x4 w, float (&x)[8]) {
  if constexpr (__is_same(T, _Float16)) {
    Pack16 p;
    p.u = w;
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = (float)p.h[e];
  } else { // bf16: the upper half of an fp32
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x[2 * i] = __uint_as_float(w[i] << 16);
      x[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
}
template <typename T> FMHA_DEV void unpack8(u32x2 w, float (&x)[8]) { // e4m3
  static_assert(__is_same(T, uint8_t), "8-byte loads hold e4m3 bytes");
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const auto lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[i], false), hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[i], true);
    x[4 * i] = lo[0];
    x[4 * i + 1] = lo[1];
    x[4 * i + 2] = hi[0];
    x[4 * i + 3] = hi[1];
  }
}

// c + a.x * b.x + a.y * b.y on a pair of 16-bit elements (fp32 products and sum).
template <typename T> FMHA_DEV float dot2(uint32_t a, uint32_t b, float c) {
  if constexpr (__is_same(T, _Float16)) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, a), __builtin_bit_cast(h2, b), c, false);
  } else {
    typedef __bf16 b2 __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(b2, a), __builtin_bit_cast(b2, b), c, false);
  }
}

// Sum over the LPR (8 or 16) neighbouring lanes that hold one row; every lane gets the total.
template <int LPR> FMHA_DEV float row_sum(float x) {
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0xB1, 0xf, 0xf, true));  // quad_perm [1,0,3,2]
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x4E, 0xf, 0xf, true));  // quad_perm [2,3,0,1]
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x141, 0xf, 0xf, true)); // row_half_mirror
  if constexpr (LPR == 16)
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x140, 0xf, 0xf, true)); // row_mirror
  return x;
}

// TI: element type of q, k, v (fp16, bf16 or uint8_t = e4m3); TO: of o and the mask (= TI unless TI is e4m3).
template <typename TI, typename TO, int D, int NQ, bool MASK>
__global__ __launch_bounds__(kDecodeWaves * 64) void fmha_fwd_decode_kernel(const DecodeArgs a) {
  using T = TI;
  using Load = typename DecodeIn<TI>::Load;
  constexpr int LPR = D / 8;       // lanes per row
  constexpr int NG = 64 / LPR;     // lane groups per wave = rows per load instruction
  constexpr int U = NQ >= 4 ? 8 : DecodeIn<TI>::LOADS; // (four query rows: fewer loads in flight, for the registers)
  constexpr int BLK = U * NG;      // keys per wave and block
  constexpr int NS = kDecodeWaves * NG; // softmax states per workgroup
  constexpr float NEG_INF = -__builtin_inff();
  static_assert(D == 64 || D == 128, "rows of 8 or 16 lanes");

  constexpr int RG = NQ < 4 ? NQ : 4; // query rows that meet in LDS at a time
  __shared__ float s_m[NS][RG], s_l[NS][RG];
  __shared__ float s_acc[NS][RG][D];

  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63;
  const int g = l / LPR, c8 = l % LPR; // the lane's group and its 8 columns
  const int head = blockIdx.x / a.pieces, piece = blockIdx.x - head * a.pieces;

  // keys of this piece: [k0, k1)
  int n = a.sk;
  if (a.kv_len) {
    const int m = a.kv_len[head / a.kv_div];
    n = m < 0 ? 0 : (m < n ? m : n);
  }
  const int k0 = piece * a.chunk;
  int k1 = k0 + a.chunk;
  k1 = k1 < n ? k1 : n;

  const T *Kb = (const T *)a.k + a.mk.head(head) + c8 * 8;
  const T *Vb = (const T *)a.v + a.mv.head(head) + c8 * 8;
  const size_t kss = (size_t)a.mk.ss, vss = (size_t)a.mv.ss;
  const TO *mrow = MASK ? (const TO *)a.mask + (size_t)(head / a.mask_div) * (size_t)a.mask_sb : nullptr;

  // the lane's 8 columns of every query row: 16-bit rows stay packed (the dot products run on v_dot2c_f32_*, exact
  // products summed in fp32, and the score is scaled afterwards); e4m3 rows are unpacked and scaled here
  constexpr bool DOT2 = sizeof(TI) == 2;
  Load qp[DOT2 ? NQ : 1];
  float qf[DOT2 ? 1 : NQ][8];
#pragma unroll
  for (int r = 0; r < NQ; ++r) {
    const int qr = r < a.sq ? r : a.sq - 1;
    const Load t = *(const Load *)((const T *)a.q + a.mq.head(head) + (size_t)qr * (size_t)a.mq.ss + c8 * 8);
    if constexpr (DOT2) {
      qp[r] = t;
    } else {
      unpack8<T>(t, qf[r]);
#pragma unroll
      for (int e = 0; e < 8; ++e) qf[r][e] *= a.scale_l2;
    }
  }

  float m_run[NQ], l_run[NQ], acc[NQ][8];
#pragma unroll
  for (int r = 0; r < NQ; ++r) {
    m_run[r] = NEG_INF;
    l_run[r] = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[r][e] = 0.f;
  }

  // blocks of the piece: wave w takes blocks w, w + 4, ...; load j of a block covers keys kb + j*NG + g
  const int nblk = k1 > k0 ? (k1 - k0 + BLK - 1) / BLK : 0;
  // One set of registers per stream: the K loads of the wave's next block are issued as soon as this block's
  // scores are formed, its V loads as soon as this block's P.V is done, so that 8-16 loads per wave (and the other
  // waves of the SIMD) cover the trip to memory.
  Load kc[U], vc[U];
  float mc[U];
  auto key_of = [&](int b, int j) {
    const int key = k0 + b * BLK + j * NG + g;
    return key < k1 ? key : k1 - 1; // keys past the end repeat the last one (their scores are set to -inf)
  };
  auto issue_k = [&](int b) {
#pragma unroll
    for (int j = 0; j < U; ++j) {
      const int key = key_of(b, j);
      kc[j] = *(const Load *)(Kb + (size_t)key * kss);
      if constexpr (MASK) mc[j] = (float)mrow[key];
    }
  };
  auto issue_v = [&](int b) {
#pragma unroll
    for (int j = 0; j < U; ++j) vc[j] = *(const Load *)(Vb + (size_t)key_of(b, j) * vss);
  };
  if (w < nblk) {
    issue_k(w);
    issue_v(w);
  }
  for (int b = w; b < nblk; b += kDecodeWaves) {
    const bool more = b + kDecodeWaves < nblk;
    const int kb = k0 + b * BLK;
    // scores of the group's U keys, all query rows
    float s[NQ][U];
#pragma unroll
    for (int j = 0; j < U; ++j) {
      const bool live = kb + j * NG + g < k1;
      float x[8];
      if constexpr (!DOT2) unpack8<T>(kc[j], x);
#pragma unroll
      for (int r = 0; r < NQ; ++r) {
        float d = 0.f;
        if constexpr (DOT2) {
#pragma unroll
          for (int i = 0; i < 4; ++i) d = dot2<T>(qp[r][i], kc[j][i], d);
          d = row_sum<LPR>(d) * a.scale_l2;
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) d = fmaf(qf[r][e], x[e], d);
          d = row_sum<LPR>(d);
        }
        if constexpr (MASK) d += fmaf(mc[j], a.mask_a, a.mask_b);
        s[r][j] = live ? d : NEG_INF;
      }
    }
    if (more) issue_k(b + kDecodeWaves);
    // online softmax: raise the reference, rescale, turn the scores into probabilities
#pragma unroll
    for (int r = 0; r < NQ; ++r) {
      float bm = s[r][0];
#pragma unroll
      for (int j = 1; j < U; ++j) bm = fmaxf(bm, s[r][j]);
      const float m_new = fmaxf(m_run[r], bm);
      const float m_use = m_new == NEG_INF ? 0.f : m_new; // nothing visible yet: every probability is 0
      const float alpha = fast_exp2(m_run[r] - m_use);    // (2^-inf = 0 at the start)
      m_run[r] = m_new;
      float ps = 0.f;
#pragma unroll
      for (int j = 0; j < U; ++j) {
        s[r][j] = fast_exp2(s[r][j] - m_use);
        ps += s[r][j];
      }
      l_run[r] = l_run[r] * alpha + ps;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[r][e] *= alpha;
    }
#pragma unroll
    for (int j = 0; j < U; ++j) {
      float x[8];
      unpack8<T>(vc[j], x);
#pragma unroll
      for (int r = 0; r < NQ; ++r) {
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[r][e] = fmaf(s[r][j], x[e], acc[r][e]);
      }
    }
    if (more) issue_v(b + kDecodeWaves);
  }

  // ---- the workgroup's NS partial softmaxes meet in LDS (up to four query rows at a time: RG)
  const int st = w * NG + g;
#pragma unroll
  for (int r0 = 0; r0 < NQ; r0 += RG) {
    if (r0 > 0) __syncthreads(); // the previous rows have been read
#pragma unroll
    for (int rr = 0; rr < RG; ++rr) {
      if (c8 == 0) {
        s_m[st][rr] = m_run[r0 + rr];
        s_l[st][rr] = l_run[r0 + rr];
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) s_acc[st][rr][c8 * 8 + e] = acc[r0 + rr][e];
    }
    __syncthreads();
    // thread t: query row r0 + t / LPR, columns 8 * (t % LPR) .. +7
    const int rr = tid / LPR, r = r0 + rr;
    if (rr < RG && r < a.sq) {
      float M = NEG_INF;
#pragma unroll
      for (int i = 0; i < NS; ++i) M = fmaxf(M, s_m[i][rr]);
      float tot = 0.f, out[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      if (M != NEG_INF) {
#pragma unroll
        for (int i = 0; i < NS; ++i) {
          const float f = fast_exp2(s_m[i][rr] - M); // (an empty state: 2^-inf = 0)
          tot = fmaf(s_l[i][rr], f, tot);
#pragma unroll
          for (int e = 0; e < 8; ++e) out[e] = fmaf(s_acc[i][rr][c8 * 8 + e], f, out[e]);
        }
      }
      const float inv = tot > 0.f ? a.out_scale / tot : 0.f; // no visible key: O = 0, LSE = -inf
      const float lse = tot > 0.f ? (M + fast_log2(tot)) * FMHA_LN2 : NEG_INF;
      if (a.pieces > 1) {
        float *dst = a.o_part + ((size_t)blockIdx.x * a.sq + r) * D + c8 * 8;
        f32x4 lo = {out[0] * inv, out[1] * inv, out[2] * inv, out[3] * inv};
        f32x4 hi = {out[4] * inv, out[5] * inv, out[6] * inv, out[7] * inv};
        *(f32x4 *)dst = lo;
        *(f32x4 *)(dst + 4) = hi;
        if (c8 == 0) a.lse_part[(size_t)blockIdx.x * a.sq + r] = lse;
      } else {
        Pack16 y;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          if constexpr (__is_same(TO, _Float16)) y.h[e] = (_Float16)(out[e] * inv);
          else y.b[e] = (__bf16)(out[e] * inv);
        }
        *(u32x4 *)((TO *)a.o + a.mo.head(head) + (size_t)r * (size_t)a.mo.ss + c8 * 8) = y.u;
        if (a.lse && c8 == 0) a.lse[(size_t)head * a.sq + r] = lse;
      }
    }
  }
}

// Return 0 on success, 1 if the shape is not built, 2 if the launch failed.
int fwd_decode_dispatch(const DecodeArgs &a, int d, bool bf16, hipStream_t s);
// The same for e4m3 q, k, v (o and mask fp16 or bf16).
int fwd_decode_fp8_dispatch(const DecodeArgs &a, int d, bool out_bf16, hipStream_t s);

} // namespace fmha
