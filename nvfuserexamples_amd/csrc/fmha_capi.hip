// C-ABI entry points of libfmha_hip.so: argument validation, variant selection and
// launch.  Declared in include/fmha_capi.h.  No allocation, no synchronisation.
#include "../../include/fmha_capi.h"
#include "fmha_launch.h"
#include "fmha_fwd_fp8.h"
#include "fmha_fwd_decode.h"

#include <atomic>
#include <cmath>
#include <cstddef>
#include <cstring>
#include <cstdlib>
#include <mutex>
#include <type_traits>

using namespace fmha;

namespace {

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
bool aligned8(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 7u) == 0; }

__global__ void philox_keep_mask_kernel(DropCtx c, int sq, int sk, long long total, uint8_t *out) {
  // one thread per (bh, q, 4-key group): writes up to four bytes
  const long long kg = (sk + 3) / 4;
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const long long k4 = idx % kg;
  const long long row = idx / kg;
  const int q = (int)(row % sq);
  const long long bh = row / sq;
  const uint32_t wd = drop_word(c, (uint32_t)bh, (uint32_t)q, (uint32_t)k4);
  uint8_t *dst = out + row * sk + k4 * 4;
  for (int t = 0; t < 4; ++t)
    if (k4 * 4 + t < sk) dst[t] = drop_keep_byte(wd, t, c.thr) ? 1 : 0;
}

DropCtx make_drop_ctx(uint64_t seed, uint64_t offset, float p, int sq, int sk) {
  DropCtx c;
  c.seed_lo = (uint32_t)seed;
  c.seed_hi = (uint32_t)(seed >> 32);
  c.off_lo = (uint32_t)offset;
  c.off_hi = (uint32_t)(offset >> 32);
  c.thr = fmha_drop_threshold(p);
  c.qb4 = (uint32_t)((sq + 3) / 4);
  c.kb4 = (uint32_t)((sk + 3) / 4);
  return c;
}

// Tuning overrides for experiments and tests: FMHA_FWD_QB=1|2 forces the query blocks per wave of
// the forward, FMHA_FWD_STREAM=0 keeps full-mask forwards on the pipelined kernel, FMHA_FWD_SAVE_ONCE=0 /
// FMHA_FWD_SAVE_SPLIT=0 keep the save-intermediates operator beyond 128 keys off its one-launch kernel / off the
// forward-then-save pair of launches,
// FMHA_FWD_SHORT=0 / FMHA_BWD_SHORT=0 keep short key ranges / short sequences off their
// one-pass kernels (FMHA_FWD_SHORT=2: only the forwards without a full mask tensor) (FMHA_BWD_SHORT=128 limits the backward one to 128 rows), FMHA_BWD_PAIR=0|1 sets the
// pairing of causal tiles in the backward, FMHA_MASK_TRIM=0 makes forward and backward visit the key tiles
// that a per-key mask hard-masks (as FMHA_FLAG_NO_MASK_TRIM does per call), FMHA_FWD_SPLIT=0 never cuts a
// forward's key range into pieces, FMHA_FWD_SPLIT=n (2..64) cuts it into about n wherever pieces are possible,
// FMHA_FWD_DECODE=0 keeps forwards of one to four query rows on the matrix-pipe kernels, FMHA_FWD_HEAD=0|1 keeps
// forwards off / puts them on the whole-head kernel wherever it applies.
// The environment is read once per process (on the first launch); fmha_reload_overrides() reads it again.
struct Overrides {
  int mask_trim, fwd_short, fwd_save_split, fwd_save_once, fwd_stream, fwd_qb, fwd_split, fwd_decode, fwd_head, bwd_pair, bwd_short;
};
int env_int(const char *name, int dflt) {
  const char *e = std::getenv(name);
  return e ? std::atoi(e) : dflt;
}
Overrides read_overrides() {
  Overrides o;
  o.mask_trim = env_int("FMHA_MASK_TRIM", 1);
  o.fwd_short = env_int("FMHA_FWD_SHORT", 1);
  o.fwd_save_split = env_int("FMHA_FWD_SAVE_SPLIT", 1);
  o.fwd_save_once = env_int("FMHA_FWD_SAVE_ONCE", 1);
  o.fwd_stream = env_int("FMHA_FWD_STREAM", 1);
  o.fwd_qb = env_int("FMHA_FWD_QB", 0);
  o.fwd_split = env_int("FMHA_FWD_SPLIT", -1);
  o.fwd_decode = env_int("FMHA_FWD_DECODE", 1);
  o.fwd_head = env_int("FMHA_FWD_HEAD", -1);
  o.bwd_pair = env_int("FMHA_BWD_PAIR", -1);
  o.bwd_short = env_int("FMHA_BWD_SHORT", 1);
  return o;
}
Overrides &overrides() {
  static Overrides o = read_overrides();
  return o;
}

constexpr int kMaxDevices = 64;

// Compute units of the current device (0 if it cannot be asked), looked up once per device.
int cu_count() {
  static std::atomic<int> cached[kMaxDevices];
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 0;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 0) n = 0;
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

// ---- A forward whose key range is cut into pieces (few heads, long key ranges: decode steps) ----
// With one to a few query rows per head and fewer heads than the chip has room for workgroups, a launch
// by head leaves most compute units idle while each busy one streams a whole K and V.  Such a forward
// runs as `pieces` forwards over `chunk` keys each (the kernels see bh * pieces heads: FwdArgs::pieces), which write normalised partial outputs and their log-sum-exps into the caller's workspace,
// and a second launch merges them:  O = sum_c w_c O_c,  w_c = exp(LSE_c - LSE),  LSE = log sum_c exp(LSE_c).
constexpr int kMaxPieces = 64; // what the merge kernel holds in LDS
struct SplitPlan {
  int pieces, chunk;
  size_t off_lse, off_mask, bytes; // the partial outputs start at offset 0
};

size_t round256(size_t x) { return (x + 255u) & ~(size_t)255u; }

// Forwards the decode kernel serves (fmha_fwd_decode.h): one to four query rows, head dim 64 or 128, no causal
// mask, dropout or saved outputs, no mask or one that is constant along the queries.
bool decode_eligible(const fmha_fwd_params *p) {
  return overrides().fwd_decode != 0 && p->sq <= 4 && (p->d == 64 || p->d == 128) && !p->causal &&
         p->drop_kind == FMHA_DROP_NONE && !p->save_softmax && !p->save_dropout &&
         (p->mask_kind == FMHA_MASK_NONE || p->mask_stride_q == 0);
}

// Whether the forward described by p (already validated) runs in pieces, and where its intermediates go.
// The decode kernel's pieces are fp32 and read the caller's mask where it is; the matrix-pipe kernels' pieces
// have the element type and a regrouped copy of the mask.
bool plan_split(const fmha_fwd_params *p, SplitPlan &pl) {
  const bool decode = decode_eligible(p);
  const int force = overrides().fwd_split;
  if (force == 0) return false;
  if (p->causal || p->drop_kind != FMHA_DROP_NONE || p->save_softmax || p->save_dropout) return false;
  if (p->mask_kind != FMHA_MASK_NONE && p->mask_stride_q != 0) return false; // a [.., sq, sk] mask tensor
  const long long sk = p->sk, sq = p->sq;
  long long chunk;
  if (force >= 2) {
    const long long n = force > kMaxPieces ? kMaxPieces : force;
    chunk = ((sk + n - 1) / n + 127) / 128 * 128;
  } else {
    const int cus = cu_count();
    const long long items = (long long)p->bh * ((sq + 127) / 128); // workgroups of the plain launch
    // Worth it while the plain launch has fewer workgroups than the chip has compute units (with one per
    // unit it already streams at 0.66 of the HBM peak, measured) and the key range is long enough to cut.
    if (cus <= 0 || items >= cus || sk < 2048) return false;
    // Measured best (one to sixteen heads per compute unit's worth of work, 4k to 128k keys): about two
    // workgroups per compute unit, pieces of at least 1024 keys.
    const long long want = (2LL * cus + items - 1) / items;
    chunk = ((sk + want - 1) / want + 127) / 128 * 128;
    const long long least = (4 * sq + 127) / 128 * 128;         // partial outputs stay under an eighth of the K/V bytes
    if (chunk < least) chunk = least;
    if (chunk < 1024) chunk = 1024;
    const long long cap = ((sk + kMaxPieces - 1) / kMaxPieces + 127) / 128 * 128;
    if (chunk < cap) chunk = cap;
  }
  const long long pieces = (sk + chunk - 1) / chunk;
  if (pieces < 2 || pieces > kMaxPieces || (long long)p->bh * pieces >= (1ll << 24)) return false;
  pl.pieces = (int)pieces;
  pl.chunk = (int)chunk;
  const size_t vh = (size_t)p->bh * (size_t)pieces;
  size_t off = round256(vh * (size_t)sq * (size_t)p->d * (decode ? 4u : 2u));
  pl.off_lse = off;
  off += round256(vh * (size_t)sq * sizeof(float));
  pl.off_mask = off;
  if (p->mask_kind != FMHA_MASK_NONE && !decode) off += round256(vh * (size_t)chunk * 2u);
  pl.bytes = off;
  return true;
}

// A per-key mask's rows regrouped by piece (the kernels index mask rows by head): piece c of head i gets keys
// [c * chunk, (c + 1) * chunk) of row i / mask_div.  One thread per (head, piece, group of 8 keys).
__global__ void split_mask_kernel(uint16_t *mask_out, const uint16_t *mask_in, int64_t mask_sb, int32_t mask_div,
                                  int32_t bh, int32_t sk, int32_t pieces, int32_t chunk) {
  const int gpp = chunk / 8; // threads per piece
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long long)bh * pieces * gpp) return;
  const int g = (int)(idx % gpp);
  const long long vh = idx / gpp;
  const int c = (int)(vh % pieces);
  const int i = (int)(vh / pieces);
  const uint16_t *src = mask_in + (size_t)(i / mask_div) * (size_t)mask_sb;
  uint16_t *dst = mask_out + (size_t)vh * (size_t)chunk + g * 8;
  for (int t = 0; t < 8; ++t) {
    const int key = c * chunk + g * 8 + t;
    dst[t] = key < sk ? src[key] : (uint16_t)0; // (keys past the end are excluded by the pieces' key counts)
  }
}

// Merges the pieces: one workgroup of kMergeThreads per (head, query row).  Thread t owns 8 output columns
// (t % cpr) and every (kMergeThreads / cpr)-th piece, so that the loads of all pieces are in flight together
// (a thread walking the pieces one after the other pays a trip to memory per piece); the threads' sums meet in LDS.
constexpr int kMergeThreads = 256;
template <typename T, typename TP>
__global__ void __launch_bounds__(kMergeThreads)
split_merge_kernel(const TP *o_part, const float *lse_part, T *o, float *lse, RowMap mo, int32_t sq, int32_t d,
                   int32_t pieces) {
  __shared__ float s_lse[kMaxPieces];
  __shared__ float s_acc[kMergeThreads][9];
  const int t = threadIdx.x;
  const int cpr = d / 8;          // 16-byte column groups per row (1..32)
  const int lanes = kMergeThreads / cpr; // threads per column group
  const int c8 = t % cpr, pl = t / cpr;  // (threads with pl >= lanes have no work)
  const int h = blockIdx.x / sq, q = blockIdx.x - h * sq;
  const size_t row0 = (size_t)h * pieces * sq + q; // piece c: row0 + c * sq
  if (t < pieces) s_lse[t] = lse_part[row0 + (size_t)t * sq];
  __syncthreads();
  float m = -INFINITY;
  for (int c = 0; c < pieces; ++c) m = fmaxf(m, s_lse[c]);
  float acc[9] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}; // eight columns and the sum of the weights
  if (m != -INFINITY && pl < lanes) { // (a head without any visible key: O = 0, LSE = -inf, like the plain launch)
    for (int c = pl; c < pieces; c += lanes) {
      const float l = s_lse[c];
      if (l == -INFINITY) continue; // an empty piece
      const float w = expf(l - m);
      const TP *src = o_part + (row0 + (size_t)c * sq) * d + c8 * 8;
      float xv[8];
      if constexpr (__is_same(TP, float)) {
        const f32x4 lo = *(const f32x4 *)src, hi = *(const f32x4 *)(src + 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          xv[e] = lo[e];
          xv[4 + e] = hi[e];
        }
      } else {
        unpack8<TP>(*(const u32x4 *)src, xv);
      }
      acc[8] += w;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += w * xv[e];
    }
  }
#pragma unroll
  for (int e = 0; e < 9; ++e) s_acc[t][e] = acc[e];
  __syncthreads();
  if (pl != 0) return;
  for (int j = 1; j < lanes; ++j) {
#pragma unroll
    for (int e = 0; e < 9; ++e) acc[e] += s_acc[j * cpr + c8][e];
  }
  const float tot = acc[8];
  const float inv = tot > 0.f ? 1.f / tot : 0.f;
  Pack16 y;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    if constexpr (__is_same(T, _Float16)) y.h[e] = (_Float16)(acc[e] * inv);
    else y.b[e] = (__bf16)(acc[e] * inv);
  }
  *(u32x4 *)(o + mo.head(h) + (size_t)q * (size_t)mo.ss + c8 * 8) = y.u;
  if (lse && c8 == 0) lse[(size_t)h * sq + q] = tot > 0.f ? m + logf(tot) : -INFINITY;
}

} // namespace

extern "C" {

uint32_t fmha_drop_threshold(float p_drop) {
  double t = std::floor((double)p_drop * 256.0 + 0.5);
  if (t < 0) t = 0;
  if (t > 255) t = 255;
  return (uint32_t)t;
}

float fmha_drop_scale(float p_drop) {
  const uint32_t thr = fmha_drop_threshold(p_drop);
  return (float)(256.0 / (256.0 - (double)thr));
}

const char *fmha_strerror(int code) {
  switch (code) {
  case FMHA_OK: return "ok";
  case FMHA_E_NULL: return "a required pointer is NULL";
  case FMHA_E_DTYPE: return "unknown dtype (0 = fp16, 1 = bf16)";
  case FMHA_E_SHAPE: return "bad shape: sizes must be positive, the head dim a multiple of 8 up to 256, and one head's rows must span less than 2^31 elements";
  case FMHA_E_ALIGN: return "q/k/v/o/gradient pointers must be 16-byte aligned and their strides multiples of 8 elements";
  case FMHA_E_ARG: return "argument out of range (struct_bytes must be set to the size of the parameter struct, scale must be > 0, p_drop in [0,1), mask_bh_div >= 1, mask_neg finite and <= 0, known mask/drop kind)";
  case FMHA_E_UNSUPPORTED: return "combination not built (tensor dropout / saved intermediates exclude causal, Philox, valid key counts and strided layouts; the backward takes Philox dropout only; k and v rows must be equally far apart)";
  case FMHA_E_LAUNCH: return "HIP launch failed";
  case FMHA_E_SCRATCH: return "fmha_bwd_launch_noalloc: bh * sq exceeds fmha_bwd_noalloc_max_rows() (the library's own scratch holds one float per query row); use fmha_bwd_launch with caller-provided delta";
  default: return "unknown error code";
  }
}

const char *fmha_version(void) { return "0.2"; }

void fmha_reload_overrides(void) { overrides() = read_overrides(); }

int fmha_philox_keep_mask(uint64_t seed, uint64_t offset, float p_drop, int32_t bh, int32_t sq,
                          int32_t sk, uint8_t *out, void *hip_stream) {
  if (!out) return FMHA_E_NULL;
  if (bh <= 0 || sq <= 0 || sk <= 0) return FMHA_E_SHAPE;
  if (!(p_drop >= 0.f && p_drop < 1.f)) return FMHA_E_ARG;
  const DropCtx c = make_drop_ctx(seed, offset, p_drop, sq, sk);
  const long long total = (long long)bh * sq * ((sk + 3) / 4);
  const int nt = 256;
  const long long nb = (total + nt - 1) / nt;
  if (nb > 0x7fffffffLL) return FMHA_E_SHAPE;
  hipLaunchKernelGGL(philox_keep_mask_kernel, dim3((unsigned)nb), dim3(nt), 0, (hipStream_t)hip_stream, c,
                     sq, sk, total, out);
  return hipGetLastError() == hipSuccess ? FMHA_OK : FMHA_E_LAUNCH;
}

} // extern "C"

// Head dims the kernels are built for: 64, 128 and 256.  Anything else (a multiple of 8) runs on the next
// built size through the run-time-layout kernels, which never read or write the missing columns.
static int built_head_dim(int d) { return d <= 64 ? 64 : d <= 128 ? 128 : 256; }

// Row layout of one tensor from the caller's (heads, strides); see fmha_capi.h.  `strided` is
// set when the layout is not the folded contiguous one (it is never cleared).
static int make_row_map(RowMap &m, int32_t heads, const int64_t st[3], int32_t bh, int32_t rows, int32_t d,
                        bool &strided) {
  m.heads_rcp = 0;
  if (heads == 0) {
    m.sb = (int64_t)rows * d;
    m.sh = 0;
    m.ss = d;
    m.heads = 1;
    return (int64_t)rows * d < (1ll << 31) ? FMHA_OK : FMHA_E_SHAPE; // offsets inside a head are 31-bit
  }
  if (heads < 0 || bh % heads != 0) return FMHA_E_ARG;
  for (int i = 0; i < 3; ++i)
    if (st[i] < 0 || (st[i] & 7) != 0) return FMHA_E_ALIGN;
  if (st[2] < d || st[2] >= (1ll << 24)) return FMHA_E_ARG;
  if ((int64_t)(rows - 1) * st[2] + d >= (1ll << 31) || (int64_t)bh * heads >= (1ll << 32)) return FMHA_E_SHAPE;
  m.heads_rcp = (uint32_t)((1ull << 32) / (uint64_t)heads) + 1u; // unused when heads == 1
  m.sb = st[0];
  m.sh = st[1];
  m.ss = st[2];
  m.heads = heads;
  if (!(st[2] == d && st[1] == (int64_t)rows * d && st[0] == (int64_t)heads * rows * d)) strided = true;
  return FMHA_OK;
}

static int fwd_dispatch_strided(FwdArgs &a, const FwdVariant &v, int dtype, int D, hipStream_t s) {
  if (dtype == FMHA_DTYPE_F16)
    return D == 64 ? fwd_dispatch_f16_d64_strided(a, v, s) : D == 128 ? fwd_dispatch_f16_d128_strided(a, v, s) : fwd_dispatch_f16_d256_strided(a, v, s);
  return D == 64 ? fwd_dispatch_bf16_d64_strided(a, v, s) : D == 128 ? fwd_dispatch_bf16_d128_strided(a, v, s) : fwd_dispatch_bf16_d256_strided(a, v, s);
}

// The merge of `pieces` partial results (fp32 from the decode kernel, element type otherwise) into o and lse.
template <bool F32> static int merge_launch(int dtype, void *o, float *lse, int bh, int sq, int d, const void *o_part,
                                            const float *lse_part, const RowMap &mo, int pieces, hipStream_t s) {
  if ((long long)bh * sq > 0x7fffffffLL) return 2; // one workgroup per output row
  const dim3 grid((unsigned)((long long)bh * sq)), block(kMergeThreads);
  if (dtype == FMHA_DTYPE_F16) {
    using TP = std::conditional_t<F32, float, _Float16>;
    hipLaunchKernelGGL((split_merge_kernel<_Float16, TP>), grid, block, 0, s, (const TP *)o_part, lse_part,
                       (_Float16 *)o, lse, mo, sq, d, pieces);
  } else {
    using TP = std::conditional_t<F32, float, __bf16>;
    hipLaunchKernelGGL((split_merge_kernel<__bf16, TP>), grid, block, 0, s, (const TP *)o_part, lse_part, (__bf16 *)o,
                       lse, mo, sq, d, pieces);
  }
  return hipGetLastError() == hipSuccess ? 0 : 2;
}

// One to four query rows (decode_eligible): the decode kernel on the whole key range, or -- with a plan -- on its
// pieces, followed by the merge.
static int fwd_decode_launch(const fmha_fwd_params *p, const FwdArgs &a, const SplitPlan *pl, hipStream_t s) {
  DecodeArgs d;
  d.q = a.q; d.k = a.k; d.v = a.v;
  d.o = a.o;
  d.lse = a.lse;
  d.o_part = nullptr;
  d.lse_part = nullptr;
  d.mask = a.mask;
  d.mask_sb = a.mask_sb;
  d.mask_div = a.mask_div;
  d.mask_a = a.mask_a;
  d.mask_b = a.mask_b;
  d.kv_len = a.kv_len;
  d.kv_div = a.kv_div;
  d.bh = p->bh; d.sq = p->sq; d.sk = p->sk;
  d.pieces = 1;
  d.chunk = p->sk;
  d.scale_l2 = a.scale_l2;
  d.out_scale = 1.f;
  d.mq = a.mq; d.mk = a.mk; d.mv = a.mv; d.mo = a.mo;
  if (pl) {
    unsigned char *ws = (unsigned char *)p->workspace;
    d.pieces = pl->pieces;
    d.chunk = pl->chunk;
    d.o_part = (float *)ws;
    d.lse_part = (float *)(ws + pl->off_lse);
  }
  const int rc = fwd_decode_dispatch(d, p->d, p->dtype == FMHA_DTYPE_BF16, s);
  if (rc != 0) return rc == 1 ? FMHA_E_UNSUPPORTED : FMHA_E_LAUNCH;
  if (pl && merge_launch<true>(p->dtype, p->o, p->lse, p->bh, p->sq, p->d, d.o_part, d.lse_part, a.mo, pl->pieces, s) != 0)
    return FMHA_E_LAUNCH;
  return FMHA_OK;
}

// The forward in pieces (plan_split): a per-key mask's rows regrouped by piece, the forward kernels over bh * pieces
// heads of `chunk` keys on the run-time-layout code path, then the merge.  `a` describes the whole launch.
static int fwd_split_launch(const fmha_fwd_params *p, const FwdArgs &a, const SplitPlan &pl, int D, hipStream_t s) {
  unsigned char *ws = (unsigned char *)p->workspace;
  float *lse_part = (float *)(ws + pl.off_lse);
  uint16_t *mask_part = a.mask ? (uint16_t *)(ws + pl.off_mask) : nullptr;
  const long long vh = (long long)p->bh * pl.pieces;
  if (vh > 0x7fffffffLL) return FMHA_E_SHAPE; // the kernels see bh * pieces heads
  if (a.mask) {
    const long long threads = vh * (pl.chunk / 8);
    const int nt = 256;
    if ((threads + nt - 1) / nt > 0x7fffffffLL) return FMHA_E_SHAPE;
    hipLaunchKernelGGL(split_mask_kernel, dim3((unsigned)((threads + nt - 1) / nt)), dim3(nt), 0, s, mask_part,
                       (const uint16_t *)a.mask, a.mask_sb, a.mask_div, p->bh, p->sk, pl.pieces, pl.chunk);
    if (hipGetLastError() != hipSuccess) return FMHA_E_LAUNCH;
  }
  FwdArgs b = a;
  b.o = ws;
  b.lse = lse_part;
  b.sk_whole = p->sk; // the kernels work out each piece's own key count (from the head's valid count, if any)
  if (a.mask) {
    b.mask = mask_part;
    b.mask_sb = pl.chunk;
    b.mask_sq = 0;
    b.mask_div = 1;
  }
  b.mask_vec = 1; // pieces are multiples of 128 keys and start on 256-byte boundaries
  b.bh = (int32_t)vh;
  b.sk = pl.chunk;
  b.drop = make_drop_ctx(0, 0, 0.f, p->sq, pl.chunk);
  b.clock_probe = nullptr;
  b.pieces = pl.pieces;
  b.pieces_rcp = (uint32_t)((1ull << 32) / (uint64_t)pl.pieces) + 1u;
  b.piece_stride = (int64_t)pl.chunk * a.mk.ss; // (k and v rows are equally far apart)
  b.mo.heads = 1; // the partial outputs: [bh * pieces, sq, d] contiguous
  b.mo.heads_rcp = 0;
  b.mo.sb = (int64_t)p->sq * p->d;
  b.mo.sh = 0;
  b.mo.ss = p->d;
  FwdVariant v;
  v.qb = 1;
  v.mask = a.mask ? kMaskPerKey : kMaskNone;
  v.causal = false;
  v.drop = 0;
  v.saving = v.save_split = v.save_once = v.stream = v.short_keys = v.head = false;
  const int rc = fwd_dispatch_strided(b, v, p->dtype, D, s);
  if (rc != 0) return rc == 1 ? FMHA_E_UNSUPPORTED : FMHA_E_LAUNCH;
  {
    if (merge_launch<false>(p->dtype, p->o, p->lse, p->bh, p->sq, p->d, ws, lse_part, a.mo, pl.pieces, s) != 0)
      return FMHA_E_LAUNCH;
  }
  return FMHA_OK;
}

extern "C" {

uint64_t fmha_fwd_workspace_bytes(const fmha_fwd_params *caller) {
  if (!caller || caller->struct_bytes < offsetof(fmha_fwd_params, kv_len)) return 0;
  fmha_fwd_params local;
  std::memset(&local, 0, sizeof local);
  std::memcpy(&local, caller, caller->struct_bytes < sizeof local ? (size_t)caller->struct_bytes : sizeof local);
  if (local.bh <= 0 || local.sq <= 0 || local.sk <= 0 || local.d < 8 || local.d > 256 || (local.d & 7) != 0) return 0;
  if (local.drop_kind == FMHA_DROP_PHILOX && fmha_drop_threshold(local.p_drop) == 0) local.drop_kind = FMHA_DROP_NONE;
  if (local.sq == 1) local.mask_stride_q = 0;
  SplitPlan pl;
  return plan_split(&local, pl) ? (uint64_t)pl.bytes : 0;
}

int fmha_fwd_launch(const fmha_fwd_params *caller, void *hip_stream) {
  // the caller's struct may be shorter (older header) or longer (newer) than this library's
  if (!caller) return FMHA_E_NULL;
  if (caller->struct_bytes < offsetof(fmha_fwd_params, kv_len)) return FMHA_E_ARG;
  fmha_fwd_params local;
  std::memset(&local, 0, sizeof local);
  std::memcpy(&local, caller, caller->struct_bytes < sizeof local ? (size_t)caller->struct_bytes : sizeof local);
  const fmha_fwd_params *p = &local;
  if (!p->q || !p->k || !p->v || !p->o) return FMHA_E_NULL;
  if (p->dtype != FMHA_DTYPE_F16 && p->dtype != FMHA_DTYPE_BF16) return FMHA_E_DTYPE;
  if (p->bh <= 0 || p->sq <= 0 || p->sk <= 0) return FMHA_E_SHAPE;
  if (p->d < 8 || p->d > 256 || (p->d & 7) != 0) return FMHA_E_SHAPE;
  const int D = built_head_dim(p->d); // the kernels' head dim; rows of fewer elements count as zero-padded
  if (!aligned16(p->q) || !aligned16(p->k) || !aligned16(p->v) || !aligned16(p->o)) return FMHA_E_ALIGN;
  if (!(p->scale > 0.f) || !std::isfinite(p->scale)) return FMHA_E_ARG;
  if (p->mask_kind < FMHA_MASK_NONE || p->mask_kind > FMHA_MASK_KEEP01) return FMHA_E_ARG;
  if (p->drop_kind < FMHA_DROP_NONE || p->drop_kind > FMHA_DROP_TENSOR) return FMHA_E_ARG;
  if (p->mask_kind != FMHA_MASK_NONE) {
    if (!p->mask) return FMHA_E_NULL;
    if (p->mask_bh_div < 1 || p->mask_stride_b < 0 || p->mask_stride_q < 0) return FMHA_E_ARG;
  }
  if (p->mask_kind == FMHA_MASK_KEEP01 && !(std::isfinite(p->mask_neg) && p->mask_neg <= 0.f)) return FMHA_E_ARG;
  if (p->drop_kind == FMHA_DROP_PHILOX && !(p->p_drop >= 0.f && p->p_drop < 1.f)) return FMHA_E_ARG;
  if (p->drop_kind == FMHA_DROP_TENSOR && !p->drop_mask) return FMHA_E_NULL;
  if (p->drop_kind != FMHA_DROP_NONE && !std::isfinite(p->drop_scale)) return FMHA_E_ARG;
  if (p->drop_kind == FMHA_DROP_PHILOX) {
    // a threshold of 0 drops nothing: no dropout at all (and no factor on the probabilities)
    if (fmha_drop_threshold(p->p_drop) == 0) local.drop_kind = FMHA_DROP_NONE;
    else if (p->drop_scale == 0.f) local.drop_scale = fmha_drop_scale(p->p_drop);
  }
  if (p->sq == 1) local.mask_stride_q = 0; // one query row: any mask is a per-key mask
  const bool saving = p->save_softmax || p->save_dropout;
  if (saving && (p->drop_kind == FMHA_DROP_PHILOX || p->causal)) return FMHA_E_UNSUPPORTED;
  if (p->drop_kind == FMHA_DROP_TENSOR && p->causal) return FMHA_E_UNSUPPORTED;
  if (p->kv_len) {
    if (p->kv_len_bh_div < 1 || ((uintptr_t)p->kv_len & 3u)) return FMHA_E_ARG;
    if (saving || p->drop_kind == FMHA_DROP_TENSOR) return FMHA_E_UNSUPPORTED;
  }
  if ((uintptr_t)p->clock_probe & 7u) return FMHA_E_ARG;

  FwdArgs a;
  a.q = p->q; a.k = p->k; a.v = p->v; a.o = p->o; a.lse = p->lse;
  a.mask = p->mask_kind ? p->mask : nullptr;
  a.drop_mask = p->drop_kind == FMHA_DROP_TENSOR ? p->drop_mask : nullptr;
  a.save_softmax = p->save_softmax;
  a.save_dropout = p->save_dropout;
  a.mask_sb = p->mask_stride_b;
  a.mask_sq = p->mask_stride_q;
  a.mask_div = p->mask_kind ? (int32_t)p->mask_bh_div : 1;
  if (p->mask_kind == FMHA_MASK_KEEP01) {
    a.mask_a = -p->mask_neg * FMHA_LOG2E;
    a.mask_b = p->mask_neg * FMHA_LOG2E;
  } else {
    a.mask_a = FMHA_LOG2E;
    a.mask_b = 0.f;
  }
  // 8-byte vector accesses to [.., sk] rows need every row start on an 8-byte boundary
  bool vec = (p->sk % 4) == 0;
  if (a.mask) vec = vec && aligned8(a.mask) && (a.mask_sb % 4) == 0 && (a.mask_sq % 4) == 0;
  if (a.drop_mask) vec = vec && aligned8(a.drop_mask);
  if (a.save_softmax) vec = vec && aligned8(a.save_softmax);
  if (a.save_dropout) vec = vec && aligned8(a.save_dropout);
  a.mask_vec = vec ? 1 : 0;
  a.bh = p->bh; a.sq = p->sq; a.sk = p->sk;
  a.nqt = 0;
  a.scale_l2 = p->scale * FMHA_LOG2E;
  a.inv_scale_l2 = 1.f / a.scale_l2;
  a.drop_scale = p->drop_kind == FMHA_DROP_NONE ? 1.f : p->drop_scale;
  a.drop = make_drop_ctx(p->seed, p->offset, p->drop_kind == FMHA_DROP_PHILOX ? p->p_drop : 0.f, p->sq, p->sk);
  a.flags = p->flags;
  if (!overrides().mask_trim) a.flags |= kFwdFlagNoTrim;
  a.kv_len = p->kv_len;
  a.kv_div = p->kv_len ? p->kv_len_bh_div : 1;
  a.pieces = 0;
  a.pieces_rcp = 0;
  a.sk_whole = 0;
  a.piece_stride = 0;
  a.clock_probe = (unsigned long long *)p->clock_probe;
  int mrc;
  bool strided = false;
  if ((mrc = make_row_map(a.mq, p->heads, p->q_stride, p->bh, p->sq, p->d, strided)) != FMHA_OK) return mrc;
  if ((mrc = make_row_map(a.mk, p->heads, p->k_stride, p->bh, p->sk, p->d, strided)) != FMHA_OK) return mrc;
  if ((mrc = make_row_map(a.mv, p->heads, p->v_stride, p->bh, p->sk, p->d, strided)) != FMHA_OK) return mrc;
  if ((mrc = make_row_map(a.mo, p->heads, p->o_stride, p->bh, p->sq, p->d, strided)) != FMHA_OK) return mrc;
  if (p->d != D) strided = true;
  a.dcols = p->d;
  if (a.mk.ss != a.mv.ss) return FMHA_E_UNSUPPORTED;
  if (strided && (saving || p->drop_kind == FMHA_DROP_TENSOR)) return FMHA_E_UNSUPPORTED;

  hipStream_t s = (hipStream_t)hip_stream;
  SplitPlan pl;
  const bool split = p->workspace && ((uintptr_t)p->workspace & 15u) == 0 && plan_split(p, pl) &&
                     p->workspace_bytes >= pl.bytes;
  if (decode_eligible(p)) return fwd_decode_launch(p, a, split ? &pl : nullptr, s);
  if (split) return fwd_split_launch(p, a, pl, D, s);

  FwdVariant v;
  v.mask = a.mask == nullptr ? kMaskNone : (a.mask_sq == 0 ? kMaskPerKey : kMaskFull);
  v.causal = p->causal != 0;
  v.drop = (p->drop_kind == FMHA_DROP_TENSOR || saving) ? 2 : (p->drop_kind == FMHA_DROP_PHILOX ? 1 : 0);
  v.saving = saving;
  // Short key ranges under a full mask tensor run in one pass with whole-row accesses to the
  // [.., sq, sk] tensors, which must then start on 16-byte boundaries row by row.
  v.short_keys = !strided && p->d == 64 && p->sk <= 128 && (p->sk % 8) == 0 && v.mask == kMaskFull && !v.causal &&
                 v.drop != 1 && !p->kv_len && aligned16(a.mask) && (a.mask_sb % 8) == 0 && (a.mask_sq % 8) == 0 &&
                 (!a.drop_mask || aligned16(a.drop_mask)) && (!a.save_softmax || aligned16(a.save_softmax)) &&
                 (!a.save_dropout || aligned16(a.save_dropout)) && (!saving || a.drop_mask) &&
                 (long long)p->sq * (a.mask_sq > 128 ? a.mask_sq : 128) < (1LL << 30) && // (the kernel forms 32-bit byte offsets within a head: mask rows, and [.., sq, sk] rows of up to 128 keys)
                 overrides().fwd_short != 0;
  // The same one-pass kernel without a full mask tensor: no mask, a per-key mask or valid key counts, no dropout or
  // the Philox rule (FMHA_FWD_SHORT=2 keeps these on the pipelined kernel while the operators' shape stays here).
  // Measured against the pipelined kernel at S 128 with a padding mask: BH 96 4.4-4.7 against 6.6-6.7 us, BH 512 8.7
  // against 10.2 (10.2-10.5 against 11.9 with Philox dropout), BH 1 024 13.7 against 16.1 (16.7 against 18.4), level
  // from BH 2 048 on -- and 5 % behind there with Philox dropout, which therefore stays on the persistent kernel
  // once the launch has more than six items per compute unit.
  if (!v.short_keys) {
    const long long items = (long long)p->bh * ((p->sq + 127) / 128);
    const long long qpitch = strided ? (a.mq.ss > a.mo.ss ? a.mq.ss : a.mo.ss) : 64; // (folded or run-time row layouts)
    v.short_keys = p->d == 64 && p->sk <= 128 && v.mask != kMaskFull && !v.causal && v.drop != 2 && !saving &&
                   (long long)p->sq * qpitch < (1LL << 30) && (v.drop != 1 || items <= 6LL * cu_count()) &&
                   overrides().fwd_short == 1 && overrides().fwd_head != 1;
  }
  // Longer key ranges: where the caller provides an LSE buffer, the save-intermediates operator is the forward
  // launch followed by a streaming kernel that derives both saved outputs from that LSE (instead of a second
  // sweep inside a slower forward).  Same alignment needs as above.
  v.save_split = saving && !v.short_keys && !strided && p->d == 64 && p->lse && (p->sk % 8) == 0 &&
                 v.mask == kMaskFull && !v.causal && a.drop_mask && aligned16(a.mask) && (a.mask_sb % 8) == 0 &&
                 (a.mask_sq % 8) == 0 && aligned16(a.drop_mask) && (!a.save_softmax || aligned16(a.save_softmax)) &&
                 (!a.save_dropout || aligned16(a.save_dropout)) && overrides().fwd_save_split != 0;
  // Up to 512 keys one launch does it all: a wave keeps its probabilities and dropout rows in registers until the
  // row's log-sum-exp is known, so the mask and the dropout tensor are read once (no LSE buffer needed).
  v.save_once = saving && !v.short_keys && !strided && p->d == 64 && p->sk <= 512 && (p->sk % 8) == 0 &&
                v.mask == kMaskFull && !v.causal && !p->kv_len && a.drop_mask && aligned16(a.mask) &&
                (a.mask_sb % 8) == 0 && (a.mask_sq % 8) == 0 && aligned16(a.drop_mask) &&
                (!a.save_softmax || aligned16(a.save_softmax)) && (!a.save_dropout || aligned16(a.save_dropout)) &&
                overrides().fwd_save_once != 0 && overrides().fwd_stream != 0; // (it is the streaming forward's arithmetic)
  if (v.save_once) v.save_split = false;
  if (v.save_split || v.save_once) v.saving = false; // (save_split: the forward launch itself saves nothing)
  // Other forwards under an aligned full mask tensor (with or without a dropout tensor) are memory time at
  // head dim 64: the streaming kernel.
  v.stream = !v.short_keys && !v.saving && !strided && p->d == 64 && (p->sk % 8) == 0 && v.mask == kMaskFull &&
             !v.causal && v.drop != 1 && !p->kv_len && aligned16(a.mask) && (a.mask_sb % 8) == 0 &&
             (a.mask_sq % 8) == 0 && (v.drop != 2 || (a.drop_mask && aligned16(a.drop_mask))) &&
             overrides().fwd_stream != 0;
  // Two 32-query blocks per wave (on tiles of 32 keys) halve the LDS operand traffic per
  // flop.  That pays (4-6 % measured) for the unmasked variant at head dim 64 on long key
  // ranges when there is enough work for every resident workgroup to get several 256-query
  // items; with dropout or any mask the per-element work dominates (a per-key mask measures
  // 4-7 % slower with two blocks), and on short key ranges the longer per-item prologue does,
  // so one block per wave is faster there.
  v.qb = 1;
  if (p->d == 64 && !v.causal && v.drop == 0 && v.mask == kMaskNone) {
    const int cus = cu_count();
    const int tiles2 = (p->sq + 255) / 256;
    const long long items2 = (long long)p->bh * tiles2;
    const bool little_padding = tiles2 * 256 - p->sq <= p->sq / 8;
    if (cus > 0 && items2 >= 4LL * cus && little_padding && p->sk >= 1024) v.qb = 2;
  }
  const int force = overrides().fwd_qb; // tuning override: 1 or 2
  if (force == 1 || (force == 2 && p->d == 64 && !v.causal && v.drop == 0 && v.mask != kMaskFull)) v.qb = force;
  if (strided) v.qb = 1; // the two-block variant is built for the folded layout only
  // Key ranges of 257 to 512 keys at head dim 64: a whole head's K and V fit in LDS, and one workgroup of
  // eight waves per (head, 512 queries) runs without copies or barriers in its loop.  Taken when the
  // 512-query items fill the compute units evenly (FMHA_FWD_HEAD=0 never, =1 wherever the kernel applies).
  v.head = false;
  // (run-time row layouts too, where a head's rows stay within 32-bit byte offsets of its first one)
  const bool head_rows_ok = !strided || ((long long)p->sk * a.mk.ss < (1LL << 30) && (long long)p->sq * a.mq.ss < (1LL << 40));
  if (head_rows_ok && p->d == 64 && p->sk <= 512 && !v.causal && v.drop != 2 && v.mask != kMaskFull && !v.saving &&
      overrides().fwd_head != 0) {
    const int cus = cu_count();
    const int chunks = (p->sq + 511) / 512;
    const long long items = (long long)p->bh * chunks;
    const bool full = chunks * 512 - p->sq <= 128; // at most two of the eight waves of a head's last item idle
    const bool even = cus > 0 && (items % cus == 0 || items >= 4LL * cus);
    v.head = overrides().fwd_head == 1 || (p->sk > 256 && full && even);
  }

  int rc;
  if (strided) rc = fwd_dispatch_strided(a, v, p->dtype, D, s);
  else if (p->dtype == FMHA_DTYPE_F16)
    rc = D == 64 ? fwd_dispatch_f16_d64(a, v, s) : D == 128 ? fwd_dispatch_f16_d128(a, v, s) : fwd_dispatch_f16_d256(a, v, s);
  else
    rc = D == 64 ? fwd_dispatch_bf16_d64(a, v, s) : D == 128 ? fwd_dispatch_bf16_d128(a, v, s) : fwd_dispatch_bf16_d256(a, v, s);
  return rc == 0 ? FMHA_OK : (rc == 1 ? FMHA_E_UNSUPPORTED : FMHA_E_LAUNCH);
}

uint64_t fmha_bwd_workspace_bytes(int32_t, int32_t, int32_t, int32_t) { return 0; } // no backward kernel uses one

} // extern "C"

// The library's own scratch memory, for fmha_bwd_launch_noalloc: delta (bh*sq floats).  Every GPU holds its own
// copy of the array; its device address is looked up once per device (the array's name is only a host-side handle).
namespace {
constexpr size_t kScratchBytes = 8u << 20;
} // namespace
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
namespace {
void *g_scratch_ptr[kMaxDevices];
std::mutex g_scratch_mutex;

// Device address of `scratch` on the current device, or nullptr.
void *scratch_on_current_device() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void *ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess) return nullptr;
    g_scratch_ptr[dev] = ptr;
  }
  return g_scratch_ptr[dev];
}

int bwd_launch_impl(const fmha_bwd_params *caller, void *hip_stream, bool own_scratch);
} // namespace

// Whether an e4m3 forward (validated) runs on the decode kernel; `shape` then describes it to plan_split.
static bool fp8_decode_shape(const fmha_fwd_fp8_params *p, fmha_fwd_params &shape) {
  std::memset(&shape, 0, sizeof shape);
  shape.bh = p->bh; shape.sq = p->sq; shape.sk = p->sk; shape.d = p->d;
  shape.causal = p->causal;
  shape.mask_kind = p->mask ? FMHA_MASK_ADDITIVE : FMHA_MASK_NONE;
  return decode_eligible(&shape);
}

extern "C" {

uint64_t fmha_fwd_fp8_workspace_bytes(const fmha_fwd_fp8_params *caller) {
  if (!caller || caller->struct_bytes < offsetof(fmha_fwd_fp8_params, causal) + sizeof(int32_t)) return 0;
  fmha_fwd_fp8_params local;
  std::memset(&local, 0, sizeof local);
  std::memcpy(&local, caller, caller->struct_bytes < sizeof local ? (size_t)caller->struct_bytes : sizeof local);
  if (local.bh <= 0 || local.sq <= 0 || local.sk <= 0 || (local.d != 64 && local.d != 128)) return 0;
  fmha_fwd_params shape;
  SplitPlan pl;
  return fp8_decode_shape(&local, shape) && plan_split(&shape, pl) ? (uint64_t)pl.bytes : 0;
}

int fmha_fwd_fp8_launch(const fmha_fwd_fp8_params *caller, void *hip_stream) {
  if (!caller) return FMHA_E_NULL;
  if (caller->struct_bytes < offsetof(fmha_fwd_fp8_params, causal) + sizeof(int32_t)) return FMHA_E_ARG;
  fmha_fwd_fp8_params local;
  std::memset(&local, 0, sizeof local);
  std::memcpy(&local, caller, caller->struct_bytes < sizeof local ? (size_t)caller->struct_bytes : sizeof local);
  const fmha_fwd_fp8_params *p = &local;
  if (!p->q || !p->k || !p->v || !p->o) return FMHA_E_NULL;
  if (p->out_dtype != FMHA_DTYPE_F16 && p->out_dtype != FMHA_DTYPE_BF16) return FMHA_E_DTYPE;
  if (p->bh <= 0 || p->sq <= 0 || p->sk <= 0) return FMHA_E_SHAPE;
  if (p->d != 64 && p->d != 128) return FMHA_E_SHAPE;
  if ((int64_t)p->sq * p->d >= (1ll << 31) || (int64_t)p->sk * p->d >= (1ll << 31)) return FMHA_E_SHAPE;
  if (!aligned16(p->q) || !aligned16(p->k) || !aligned16(p->v) || !aligned16(p->o)) return FMHA_E_ALIGN;
  if (!(p->scale > 0.f) || !std::isfinite(p->scale)) return FMHA_E_ARG;
  for (float f : {p->descale_q, p->descale_k, p->descale_v})
    if (!(f > 0.f) || !std::isfinite(f)) return FMHA_E_ARG;
  if (p->mask && (p->mask_bh_div < 1 || p->mask_stride_b < 0)) return FMHA_E_ARG;
  if (p->kv_len && (p->kv_len_bh_div < 1 || ((uintptr_t)p->kv_len & 3u))) return FMHA_E_ARG;
  fmha_fwd_params shape; // what the piece planning looks at
  if (fp8_decode_shape(p, shape)) {
    // one to four query rows: the streaming decode kernel on e4m3 rows, whole key range or pieces
    DecodeArgs d;
    d.q = p->q; d.k = p->k; d.v = p->v;
    d.o = p->o;
    d.lse = p->lse;
    d.o_part = nullptr;
    d.lse_part = nullptr;
    d.mask = p->mask;
    d.mask_sb = p->mask_stride_b;
    d.mask_div = p->mask ? (int32_t)p->mask_bh_div : 1;
    d.mask_a = FMHA_LOG2E;
    d.mask_b = 0.f;
    d.kv_len = p->kv_len;
    d.kv_div = p->kv_len ? p->kv_len_bh_div : 1;
    d.bh = p->bh; d.sq = p->sq; d.sk = p->sk;
    d.pieces = 1;
    d.chunk = p->sk;
    d.scale_l2 = p->scale * p->descale_q * p->descale_k * FMHA_LOG2E;
    d.out_scale = p->descale_v;
    bool strided = false;
    int mrc;
    if ((mrc = make_row_map(d.mq, 0, nullptr, p->bh, p->sq, p->d, strided)) != FMHA_OK) return mrc;
    if ((mrc = make_row_map(d.mk, 0, nullptr, p->bh, p->sk, p->d, strided)) != FMHA_OK) return mrc;
    d.mv = d.mk;
    d.mo = d.mq;
    SplitPlan pl;
    const bool split = p->workspace && ((uintptr_t)p->workspace & 15u) == 0 && plan_split(&shape, pl) &&
                       p->workspace_bytes >= pl.bytes;
    if (split) {
      unsigned char *ws = (unsigned char *)p->workspace;
      d.pieces = pl.pieces;
      d.chunk = pl.chunk;
      d.o_part = (float *)ws;
      d.lse_part = (float *)(ws + pl.off_lse);
    }
    hipStream_t s = (hipStream_t)hip_stream;
    const int rc = fwd_decode_fp8_dispatch(d, p->d, p->out_dtype == FMHA_DTYPE_BF16, s);
    if (rc != 0) return rc == 1 ? FMHA_E_UNSUPPORTED : FMHA_E_LAUNCH;
    if (split && merge_launch<true>(p->out_dtype, p->o, p->lse, p->bh, p->sq, p->d, d.o_part, d.lse_part, d.mo,
                                    pl.pieces, s) != 0)
      return FMHA_E_LAUNCH;
    return FMHA_OK;
  }
  if (p->kv_len) return FMHA_E_UNSUPPORTED; // the matrix-pipe e4m3 kernel takes no key counts
  Fp8Args a;
  a.q = (const uint8_t *)p->q; a.k = (const uint8_t *)p->k; a.v = (const uint8_t *)p->v;
  a.o = p->o; a.lse = p->lse;
  a.mask = p->mask; a.mask_sb = p->mask_stride_b; a.mask_div = p->mask ? (int32_t)p->mask_bh_div : 1;
  a.bh = p->bh; a.sq = p->sq; a.sk = p->sk;
  a.score_scale_l2 = p->scale * p->descale_q * p->descale_k * FMHA_LOG2E;
  a.inv_score_scale_l2 = 1.f / a.score_scale_l2;
  a.out_scale = p->descale_v;
  const int rc = fwd_fp8_dispatch(a, p->d, p->out_dtype == FMHA_DTYPE_BF16, p->causal != 0, (hipStream_t)hip_stream);
  return rc == 0 ? FMHA_OK : (rc == 1 ? FMHA_E_UNSUPPORTED : FMHA_E_LAUNCH);
}

int fmha_bwd_launch(const fmha_bwd_params *caller, void *hip_stream) { return bwd_launch_impl(caller, hip_stream, false); }

int fmha_bwd_launch_noalloc(const fmha_bwd_params *caller, void *hip_stream) { return bwd_launch_impl(caller, hip_stream, true); }

uint64_t fmha_bwd_noalloc_max_rows(void) { return kScratchBytes / sizeof(float); }

} // extern "C"

namespace {

int bwd_launch_impl(const fmha_bwd_params *caller, void *hip_stream, bool own_scratch) {
  if (!caller) return FMHA_E_NULL;
  if (caller->struct_bytes < offsetof(fmha_bwd_params, kv_len)) return FMHA_E_ARG;
  fmha_bwd_params local;
  std::memset(&local, 0, sizeof local);
  std::memcpy(&local, caller, caller->struct_bytes < sizeof local ? (size_t)caller->struct_bytes : sizeof local);
  if (own_scratch) {
    // delta comes out of the library's array; what the caller put there is not looked at
    local.delta = nullptr;
    if (local.bh <= 0 || local.sq <= 0) return FMHA_E_SHAPE;
    const uint64_t rows = (uint64_t)local.bh * (uint64_t)local.sq;
    if (rows * sizeof(float) > kScratchBytes) return FMHA_E_SCRATCH;
    unsigned char *base = (unsigned char *)scratch_on_current_device();
    if (!base) return FMHA_E_LAUNCH;
    local.delta = (float *)base;
  }
  const fmha_bwd_params *p = &local;
  if (!p->q || !p->k || !p->v || !p->o || !p->dout || !p->lse || !p->delta || !p->dq || !p->dk || !p->dv)
    return FMHA_E_NULL;
  if (p->dtype != FMHA_DTYPE_F16 && p->dtype != FMHA_DTYPE_BF16) return FMHA_E_DTYPE;
  if (p->bh <= 0 || p->sq <= 0 || p->sk <= 0) return FMHA_E_SHAPE;
  if (p->d < 8 || p->d > 256 || (p->d & 7) != 0) return FMHA_E_SHAPE;
  const int D = built_head_dim(p->d); // the kernels' head dim; rows of fewer elements count as zero-padded
  if (!aligned16(p->q) || !aligned16(p->k) || !aligned16(p->v) || !aligned16(p->o) || !aligned16(p->dout) ||
      !aligned16(p->dq) || !aligned16(p->dk) || !aligned16(p->dv))
    return FMHA_E_ALIGN;
  if (!(p->scale > 0.f) || !std::isfinite(p->scale)) return FMHA_E_ARG;
  if (p->mask_kind < FMHA_MASK_NONE || p->mask_kind > FMHA_MASK_KEEP01) return FMHA_E_ARG;
  if (p->drop_kind < FMHA_DROP_NONE || p->drop_kind > FMHA_DROP_TENSOR) return FMHA_E_ARG;
  if (p->mask_kind != FMHA_MASK_NONE) {
    if (!p->mask) return FMHA_E_NULL;
    if (p->mask_bh_div < 1 || p->mask_stride_b < 0 || p->mask_stride_q < 0) return FMHA_E_ARG;
  }
  if (p->mask_kind == FMHA_MASK_KEEP01 && !(std::isfinite(p->mask_neg) && p->mask_neg <= 0.f)) return FMHA_E_ARG;
  if (p->drop_kind == FMHA_DROP_PHILOX && !(p->p_drop >= 0.f && p->p_drop < 1.f)) return FMHA_E_ARG;
  if (p->drop_kind == FMHA_DROP_PHILOX && !std::isfinite(p->drop_scale)) return FMHA_E_ARG;
  if (p->drop_kind == FMHA_DROP_PHILOX) {
    if (fmha_drop_threshold(p->p_drop) == 0) local.drop_kind = FMHA_DROP_NONE;
    else if (p->drop_scale == 0.f) local.drop_scale = fmha_drop_scale(p->p_drop);
  }
  if (p->drop_kind == FMHA_DROP_TENSOR) return FMHA_E_UNSUPPORTED; // backward regenerates Philox decisions only
  if (p->kv_len && (p->kv_len_bh_div < 1 || ((uintptr_t)p->kv_len & 3u))) return FMHA_E_ARG;

  BwdArgs a;
  a.q = p->q; a.k = p->k; a.v = p->v; a.o = p->o; a.dout = p->dout;
  a.lse = p->lse; a.delta = p->delta;
  a.dq = p->dq; a.dk = p->dk; a.dv = p->dv;
  a.mask = p->mask_kind ? p->mask : nullptr;
  a.mask_sb = p->mask_stride_b;
  a.mask_sq = p->mask_stride_q;
  a.mask_div = p->mask_kind ? (int32_t)p->mask_bh_div : 1;
  if (p->mask_kind == FMHA_MASK_KEEP01) {
    a.mask_a = -p->mask_neg * FMHA_LOG2E;
    a.mask_b = p->mask_neg * FMHA_LOG2E;
  } else {
    a.mask_a = FMHA_LOG2E;
    a.mask_b = 0.f;
  }
  bool vec = (p->sk % 4) == 0;
  if (a.mask) vec = vec && aligned8(a.mask) && (a.mask_sb % 4) == 0 && (a.mask_sq % 4) == 0;
  a.mask_vec = vec ? 1 : 0;
  a.bh = p->bh; a.sq = p->sq; a.sk = p->sk;
  a.ntile = 0;
  a.scale = p->scale;
  a.scale_l2 = p->scale * FMHA_LOG2E;
  a.drop_scale = p->drop_kind == FMHA_DROP_NONE ? 1.f : p->drop_scale;
  if (!(a.drop_scale > 0.f)) return FMHA_E_ARG;
  a.drop = make_drop_ctx(p->seed, p->offset, p->drop_kind == FMHA_DROP_PHILOX ? p->p_drop : 0.f, p->sq, p->sk);
  a.flags = p->flags;
  if (!overrides().mask_trim) a.flags |= kBwdFlagNoTrim;
  a.kv_len = p->kv_len;
  a.kv_div = p->kv_len ? p->kv_len_bh_div : 1;
  int mrc;
  bool strided = false;
  if ((mrc = make_row_map(a.mq, p->heads, p->q_stride, p->bh, p->sq, p->d, strided)) != FMHA_OK) return mrc;
  if ((mrc = make_row_map(a.mk, p->heads, p->k_stride, p->bh, p->sk, p->d, strided)) != FMHA_OK) return mrc;
  if ((mrc = make_row_map(a.mv, p->heads, p->v_stride, p->bh, p->sk, p->d, strided)) != FMHA_OK) return mrc;
  if ((mrc = make_row_map(a.mo, p->heads, p->o_stride, p->bh, p->sq, p->d, strided)) != FMHA_OK) return mrc;
  if ((mrc = make_row_map(a.mdo, p->heads, p->do_stride, p->bh, p->sq, p->d, strided)) != FMHA_OK) return mrc;
  if ((mrc = make_row_map(a.mdq, p->heads, p->dq_stride, p->bh, p->sq, p->d, strided)) != FMHA_OK) return mrc;
  if ((mrc = make_row_map(a.mdk, p->heads, p->dk_stride, p->bh, p->sk, p->d, strided)) != FMHA_OK) return mrc;
  if ((mrc = make_row_map(a.mdv, p->heads, p->dv_stride, p->bh, p->sk, p->d, strided)) != FMHA_OK) return mrc;
  if (p->d != D) strided = true;
  a.dcols = p->d;
  if (a.mk.ss != a.mv.ss) return FMHA_E_UNSUPPORTED;

  BwdVariant v;
  v.mask = a.mask == nullptr ? kMaskNone : (a.mask_sq == 0 ? kMaskPerKey : kMaskFull);
  v.causal = p->causal != 0;
  v.drop = p->drop_kind == FMHA_DROP_PHILOX ? 1 : 0;
  v.pair = overrides().bwd_pair; // tuning / test override: 0 or 1
  // Heads whose Q, K, V and dO fit in LDS together (up to 256 queries and keys) take one launch instead of two.
  int short_rows = overrides().bwd_short; // 0: never; 1: up to 256 rows; other values: that many rows
  if (short_rows == 1) short_rows = 256;
  v.short_seq = p->d == 64 && p->sq <= short_rows && p->sk <= short_rows && p->sq <= 256 && p->sk <= 256 &&
                v.mask != kMaskFull;
  a.ws = (float *)p->workspace; // no kernel of a release build reads it (development builds: cycle stamps)
  hipStream_t s = (hipStream_t)hip_stream;
  int rc;
  if (strided) {
    if (p->dtype == FMHA_DTYPE_F16)
      rc = D == 64 ? bwd_dispatch_f16_d64_strided(a, v, s) : D == 128 ? bwd_dispatch_f16_d128_strided(a, v, s) : bwd_dispatch_f16_d256_strided(a, v, s);
    else
      rc = D == 64 ? bwd_dispatch_bf16_d64_strided(a, v, s) : D == 128 ? bwd_dispatch_bf16_d128_strided(a, v, s) : bwd_dispatch_bf16_d256_strided(a, v, s);
  } else if (p->dtype == FMHA_DTYPE_F16)
    rc = D == 64 ? bwd_dispatch_f16_d64(a, v, s) : D == 128 ? bwd_dispatch_f16_d128(a, v, s) : bwd_dispatch_f16_d256(a, v, s);
  else
    rc = D == 64 ? bwd_dispatch_bf16_d64(a, v, s) : D == 128 ? bwd_dispatch_bf16_d128(a, v, s) : bwd_dispatch_bf16_d256(a, v, s);
  return rc == 0 ? FMHA_OK : (rc == 1 ? FMHA_E_UNSUPPORTED : FMHA_E_LAUNCH);
}

} // namespace
