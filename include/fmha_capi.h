/*
 * C ABI of the gfx950 fused multi-head-attention library (libfmha_hip.so).
 *
 * Plain pointers and sizes only -- no torch / ATen types -- so the library can be
 * bound from C, C++, ctypes or any FFI.
 *
 * Input contract: q, k, v, dout and mask values are finite numbers or, for masks, -inf.  NaN or +inf
 * inputs are not detected and do not propagate in any defined way (the kernels are compiled without
 * NaN handling: they use -inf on purpose and never produce a NaN from finite inputs).  All tensor pointers are DEVICE pointers;
 * the library never allocates, frees or synchronises: kernels are enqueued on the
 * HIP stream the caller passes and the call returns immediately.
 *
 * What each entry point replaces in the reference (shmsong/NvFuserExamples):
 * the reference has no C ABI; its boundary is the torch dispatcher
 * (fmha/fmha_manual.cpp:1240-1250) and behind it NVFuserOpBase<T>::run
 * (common/manual_scheduled_kernel.h:13-19), which JIT-compiles and launches one
 * nvFuser-generated kernel per op.  The launch functions below take the place of
 * that run() call for the three fused kernels
 *   FMHAKernel                       fmha/fmha_manual.cpp:20-409
 *   FMHATrainKernel                  fmha/fmha_manual.cpp:411-807
 *   FMHATrainKernelSaveIntermediate  fmha/fmha_manual.cpp:809-1214
 * with shapes, scale, mask layout and dropout as run-time arguments instead of
 * compile-time constants (fmha/fmha_manual.cpp:24-29,68,421).
 */
#ifndef FMHA_CAPI_H_
#define FMHA_CAPI_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element types of q/k/v/o, masks and gradients */
enum { FMHA_DTYPE_F16 = 0, FMHA_DTYPE_BF16 = 1 };

/* how the mask tensor enters the scores */
enum {
  FMHA_MASK_NONE = 0,
  FMHA_MASK_ADDITIVE = 1, /* score += mask                    (train ops, fmha_manual.cpp:463) */
  FMHA_MASK_KEEP01 = 2    /* score += (1 - mask) * mask_neg   (inference op, fmha_manual.cpp:64-71) */
};

/* dropout source */
enum {
  FMHA_DROP_NONE = 0,
  FMHA_DROP_PHILOX = 1,  /* keep decisions from Philox4x32-10 keyed by (seed, offset) */
  FMHA_DROP_TENSOR = 2   /* caller supplies a multiplicative [bh,sq,sk] tensor (fmha_manual.cpp:478-480) */
};

/* fmha_fwd_params.flags, fmha_bwd_params.flags.
 * A [.., 1, sk] mask whose tail is hard-masked (mask term <= -9000, e.g. the -10000 or -inf of a
 * padded batch; rows of up to 1024 keys are looked at) lets forward and backward skip the key tiles
 * that hold nothing else; the skipped keys' weights are exactly zero unless a masked key's score
 * exceeds every visible key's by more than 8800.  FMHA_FLAG_NO_MASK_TRIM makes them visit every tile
 * regardless. */
enum {
  FMHA_FLAG_NO_MASK_TRIM = 1
  /* (value 2 asked for a one-pass backward kernel in earlier versions; it never beat the default and was
   * removed: the bit is accepted and ignored) */
};

/* return codes */
enum {
  FMHA_OK = 0,
  FMHA_E_NULL = -1,        /* a required pointer is NULL */
  FMHA_E_DTYPE = -2,       /* unknown dtype */
  FMHA_E_SHAPE = -3,       /* non-positive size or unsupported head dim (multiples of 8 up to 256) */
  FMHA_E_ALIGN = -4,       /* q/k/v/o/gradient base pointer not 16-byte aligned */
  FMHA_E_ARG = -5,         /* scale / p_drop / mask description out of range */
  FMHA_E_UNSUPPORTED = -6, /* combination not built (see fmha_strerror) */
  FMHA_E_LAUNCH = -7,      /* the HIP runtime refused the launch */
  FMHA_E_SCRATCH = -8      /* fmha_bwd_launch_noalloc: the sizes exceed the library's own scratch memory */
};

/*
 * Forward.  Layout (as the reference, fmha/fmha_manual.cpp:39-47): heads folded into
 * dim 0, everything contiguous:
 *   q [bh,sq,d]   k [bh,sk,d]   v [bh,sk,d]   o [bh,sq,d]
 * Mask element (b,i,j) is read at
 *   mask[(b / mask_bh_div) * mask_stride_b + i * mask_stride_q + j]
 * so [bh,sq,sk] is (div 1, stride_b sq*sk, stride_q sk), a [B,1,1,sk] padding mask
 * over bh = B*H is (div H, stride_b sk, stride_q 0).
 * Head dim d: 64 in the reference (fmha_manual.cpp:24-29); here any multiple of 8 up to 256.  The kernels
 * are built for 64, 128 and 256; other head dims run at the next of those and neither read nor write
 * the columns a row does not have (no padded copies), on the run-time-layout code path.  Tensor dropout
 * and the saved outputs exist at d = 64, 128 and 256 only.
 * Computes  O = (dropout(softmax(scale * q k^T + mask_term [+ causal]))) v
 * with fp32 accumulation and fp32 softmax, the probabilities rounded to the
 * element type before the second product (fmha_manual.cpp:87) and O rounded on
 * store (fmha_manual.cpp:95).
 */
typedef struct fmha_fwd_params {
  /* sizeof(fmha_fwd_params) as the caller was compiled.  Fields are only ever appended: the library
   * reads that many bytes and takes every field beyond them as zero, so a caller built against an
   * older header keeps working.  Zero-initialise the struct (`= {}`) and set this first. */
  uint64_t struct_bytes;
  const void *q, *k, *v;
  void *o;
  float *lse; /* optional [bh,sq]: log(sum_j exp(score_ij)), saved for the backward */

  const void *mask; /* optional, element type = dtype */
  int32_t mask_kind;
  int32_t causal; /* 1: key j is visible to query i iff j <= i (no tensor involved) */
  int64_t mask_bh_div, mask_stride_b, mask_stride_q;
  float mask_neg; /* used by FMHA_MASK_KEEP01; -10000 in the reference; must be finite and <= 0 */

  int32_t drop_kind;
  const void *drop_mask; /* FMHA_DROP_TENSOR: [bh,sq,sk], element type = dtype */
  float p_drop;          /* FMHA_DROP_PHILOX: drop probability in [0,1), realised as round(256 p) / 256;
                          * below 1/512 nothing is dropped and the call is one without dropout */
  float drop_scale;      /* factor on kept probabilities: 2 on the legacy ops; with FMHA_DROP_PHILOX, 0 selects
                          * fmha_drop_scale(p_drop), which keeps the mean */
  uint64_t seed, offset; /* FMHA_DROP_PHILOX */

  /* optional [bh,sq,sk] outputs of the save-intermediates op (fmha_manual.cpp:891-897):
   * softmax before dropout and after dropout*scale, element type = dtype.
   * Only with FMHA_DROP_TENSOR or FMHA_DROP_NONE.  Beyond 128 keys, also pass `lse`: with the row
   * log-sum-exp at hand both tensors are written by one streaming launch after the forward
   * instead of by a second sweep over the keys (about 40 % less time at sk = 512). */
  void *save_softmax, *save_dropout;

  int32_t bh, sq, sk, d;
  int32_t dtype;
  float scale; /* > 0; 1/8 in the reference (fmha_manual.cpp:68) */
  int32_t flags; /* 0 or FMHA_FLAG_NO_MASK_TRIM */

  /* Optional valid key counts (the "padded version" the reference leaves as a TODO,
   * fmha_manual.cpp:110,178): head b attends keys [0, kv_len[b / kv_len_bh_div]) only, exactly
   * as if the others carried a -inf mask, and whole key tiles past the count are never touched.
   * Device pointer to int32, or NULL for all sk keys.  Not with FMHA_DROP_TENSOR / the save outputs. */
  const int32_t *kv_len;
  int32_t kv_len_bh_div;

  /* Optional diagnostic (no counterpart in the reference): device pointer to four uint64, or NULL.
   * The first workgroup of the pipelined forward kernel writes {core clock counter at its start,
   * constant 100 MHz counter at its start, core clock counter at its end, 100 MHz counter at its
   * end}; (c_end - c_start) / (t_end - t_start) * 100 is the effective core clock in MHz while
   * the kernel ran, which on a power-limited board is well below the maximum clock that the
   * published MFMA peak assumes.  Left untouched by the non-pipelined kernel. */
  uint64_t *clock_probe;

  /* Optional row layout of q, k, v and o (no counterpart in the reference: its operators take
   * folded, contiguous [bh, s, d] tensors and its perf scripts exclude the permute that produces
   * them, perf_measurement.py:52).  heads == 0: that layout, strides ignored.  heads = H > 0:
   * bh = B*H, head index i means (batch i / H, head i % H), and row r of that head of tensor x
   * starts at element (i / H) * x_stride[0] + (i % H) * x_stride[1] + r * x_stride[2]; rows are d
   * contiguous elements.  Every stride must be a non-negative multiple of 8 elements, stride[2]
   * at least d and below 2^24, and k and v must share stride[2].  E.g. a [B, s, H, d] tensor:
   * {s*H*d, d, H*d}; the q part of a packed [B, s, 3, H, d] tensor: {s*3*H*d, d, 3*H*d}.
   * lse (and delta) stay [bh, sq] contiguous.  Outputs must not overlap inputs. */
  int32_t heads;
  int64_t q_stride[3], k_stride[3], v_stride[3], o_stride[3];

  /* Optional device memory for a forward whose key range is cut into pieces (no counterpart in the
   * reference, whose shapes are fixed at 128 x 128 per head, fmha_manual.cpp:24-29).  A decode step -- one
   * or a few query rows per head against a long key range -- on fewer heads than the chip has compute units
   * would leave most of them idle while each busy one streams a whole K and V.  Given a workspace of at
   * least fmha_fwd_workspace_bytes(p) bytes (16-byte aligned), such a launch runs every piece of the key
   * range as a workgroup (or head) of its own, keeps the pieces' normalised outputs and log-sum-exps in the
   * workspace and merges them in a second launch:
   *   O = sum_c exp(LSE_c - LSE) O_c,   LSE = log sum_c exp(LSE_c).
   * Launches of one to four query rows at head dim 64 or 128 (which have a streaming kernel of their own,
   * with or without pieces) keep their pieces in fp32; other shapes keep them in the element type, so their
   * results differ from the plain launch by one more rounding to that type.  Pieces are used without a
   * causal mask, dropout or saved outputs, with no mask or a mask that is constant along the queries, with
   * or without kv_len; everything else, a NULL or too small workspace included, takes the plain launch.
   * The workspace may be reused by the next launch on the same stream. */
  void *workspace;
  uint64_t workspace_bytes;
} fmha_fwd_params;

/* Enqueue the forward kernel on `hip_stream` (a hipStream_t; NULL = default stream). */
int fmha_fwd_launch(const fmha_fwd_params *p, void *hip_stream);

/* Bytes of `workspace` with which fmha_fwd_launch(p) would run its key range in pieces on the current
 * device, or 0 where it would not (p as for the launch; the pointers are not looked at). */
uint64_t fmha_fwd_workspace_bytes(const fmha_fwd_params *p);

/*
 * Forward on 8-bit floating point inputs (no counterpart in the reference, which is fp16 only:
 * fmha/fmha_manual.cpp:120).  q, k, v hold OCP e4m3 bytes (torch.float8_e4m3fn), [bh, s, d] contiguous,
 * with one dequantisation factor per tensor (x = descale_x * x8); both products run on the fp8 matrix
 * instructions with fp32 accumulation, the softmax is fp32, the probabilities -- unnormalised, relative to
 * an INTEGER reference exponent M (in log2 units) near the row maximum, so that the rounding does not depend
 * on the order in which the keys are visited -- are rounded to e4m3 before the second product, and O is that
 * product over the sum of the ROUNDED probabilities (a convex combination of the value rows):
 *   P~ = round_e4m3(2^(y - M)),  y = log2(e) * (scale * descale_q * descale_k * q8 k8^T + mask),  M = ceil(rowmax y)
 *   O  = descale_v * (P~ v8) / rowsum(P~)
 * o (and the optional per-key additive mask, mask[(b / mask_bh_div) * mask_stride_b + j]) are fp16 or
 * bf16 (out_dtype); lse (optional) is the exact row log-sum-exp, from the unrounded probabilities.  Head dim 64
 * or 128.  e4m3 carries three mantissa bits, so outputs agree with the 16-bit path to a few per cent of their
 * magnitude, not to 2e-3.
 */
typedef struct fmha_fwd_fp8_params {
  uint64_t struct_bytes; /* sizeof(fmha_fwd_fp8_params); see fmha_fwd_params */
  const void *q, *k, *v;
  void *o;
  float *lse;
  const void *mask;
  int64_t mask_bh_div, mask_stride_b;
  int32_t bh, sq, sk, d;
  int32_t out_dtype; /* FMHA_DTYPE_F16 / FMHA_DTYPE_BF16 */
  float scale, descale_q, descale_k, descale_v;
  int32_t causal;
  /* Decode steps on an e4m3 K/V cache: launches of one to four query rows without a causal mask run on the
   * streaming kernel of the 16-bit decode steps (8-byte row loads, fp32 arithmetic), which keeps the
   * probabilities in fp32 -- no e4m3 rounding of P~, so O = descale_v * softmax(y) v8 up to fp32 rounding --
   * and moves half the bytes of the fp16 cache.  Such launches (and only they) also take valid key counts
   * (kv_len, kv_len_bh_div) and a workspace (workspace, workspace_bytes, fmha_fwd_fp8_workspace_bytes), all
   * as in fmha_fwd_params. */
  const int32_t *kv_len;
  int32_t kv_len_bh_div;
  void *workspace;
  uint64_t workspace_bytes;
} fmha_fwd_fp8_params;

int fmha_fwd_fp8_launch(const fmha_fwd_fp8_params *p, void *hip_stream);

/* As fmha_fwd_workspace_bytes, for fmha_fwd_fp8_launch. */
uint64_t fmha_fwd_fp8_workspace_bytes(const fmha_fwd_fp8_params *p);

/*
 * Backward (no counterpart in the reference, which has no backward kernel:
 * README.md:1).  Inputs are those of the forward plus the upstream gradient
 * `dout`, the forward output `o` and the saved `lse`; the dropout decisions are
 * regenerated from (seed, offset) or re-read from drop_mask, never stored.
 *   dv = (P o Z)^T dout ; dP = (dout v^T) o Z ; delta_i = sum_d dout_id o_id
 *   dS = P o (dP - delta) ; dq = scale dS k ; dk = scale dS^T q
 * `delta` is caller-provided scratch of bh*sq floats (written, then read).
 */
typedef struct fmha_bwd_params {
  uint64_t struct_bytes; /* sizeof(fmha_bwd_params) as the caller was compiled; see fmha_fwd_params */
  const void *q, *k, *v, *o, *dout;
  const float *lse;
  float *delta;
  void *dq, *dk, *dv;

  const void *mask;
  int32_t mask_kind;
  int32_t causal;
  int64_t mask_bh_div, mask_stride_b, mask_stride_q;
  float mask_neg;

  int32_t drop_kind;
  const void *drop_mask;
  float p_drop;
  float drop_scale;
  uint64_t seed, offset;

  int32_t bh, sq, sk, d;
  int32_t dtype;
  float scale;
  int32_t flags; /* 0 or FMHA_FLAG_NO_MASK_TRIM */

  const int32_t *kv_len; /* as in fmha_fwd_params; dk and dv rows at or past the count are zero */
  int32_t kv_len_bh_div;

  /* Optional row layouts, as in fmha_fwd_params, of q, k, v, o, dout and of the outputs dq, dk, dv. */
  int32_t heads;
  int64_t q_stride[3], k_stride[3], v_stride[3], o_stride[3], do_stride[3];
  int64_t dq_stride[3], dk_stride[3], dv_stride[3];

  /* Reserved (earlier versions' one-pass backward kept partial sums there): no backward kernel uses a
   * workspace; leave NULL / 0. */
  void *workspace;
  uint64_t workspace_bytes;
} fmha_bwd_params;

int fmha_bwd_launch(const fmha_bwd_params *p, void *hip_stream);

/*
 * The backward for callers that cannot allocate (no counterpart in the reference): code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  Same as fmha_bwd_launch, except that
 * `delta` of the struct is ignored: it comes out of an array of
 * 4 * fmha_bwd_noalloc_max_rows() bytes (8 MiB) that the library holds in the memory of every GPU it
 * runs on until the process ends.  bh * sq beyond fmha_bwd_noalloc_max_rows() is refused
 * (FMHA_E_SCRATCH).  The call allocates nothing and synchronises nothing.  All calls on one GPU share
 * that GPU's array: calls that may overlap there (different streams or threads) race on it; serialise
 * them or use fmha_bwd_launch with buffers of the caller's own.  Results are bit-identical to
 * fmha_bwd_launch's.  Under stream capture: the FIRST call on a device (it looks up the array's address) and the
 * first launch of each kernel variant in the process (it sets the kernel's LDS size) are not stream operations
 * and must have happened before the capture begins -- make one eager call with the same shape class first.
 */
int fmha_bwd_launch_noalloc(const fmha_bwd_params *p, void *hip_stream);
uint64_t fmha_bwd_noalloc_max_rows(void);

/* Workspace the backward can make use of for these sizes: always 0 (kept for callers of earlier versions). */
uint64_t fmha_bwd_workspace_bytes(int32_t bh, int32_t sq, int32_t sk, int32_t d);

/*
 * Materialise the Philox keep decisions the kernels use for (seed, offset, p_drop)
 * as a [bh,sq,sk] tensor of bytes (1 keep, 0 drop) in device memory.  For tests and
 * for callers that need the mask itself; the fused kernels never read such a tensor.
 * (No counterpart in the reference, whose dropout mask is a caller-made tensor:
 * test_train_mha.py:28.)
 */
int fmha_philox_keep_mask(uint64_t seed, uint64_t offset, float p_drop, int32_t bh, int32_t sq,
                          int32_t sk, uint8_t *out, void *hip_stream);

/* 8-bit threshold the keep rule compares against: keep iff random_byte >= threshold. */
uint32_t fmha_drop_threshold(float p_drop);

/* 256 / (256 - threshold): the reciprocal of the keep probability that the 8-bit threshold realises
 * (230/256 at p_drop = 0.1, not 0.9), so that E[dropout(x)] = x exactly; 1 when nothing is dropped. */
float fmha_drop_scale(float p_drop);

/* Static description of a return code. */
const char *fmha_strerror(int code);

/* The FMHA_* environment variables -- tuning and test overrides of the variant selection: FMHA_MASK_TRIM,
 * FMHA_FWD_QB, FMHA_FWD_SHORT, FMHA_FWD_STREAM, FMHA_FWD_SAVE_ONCE, FMHA_FWD_SAVE_SPLIT, FMHA_FWD_SPLIT, FMHA_FWD_DECODE, FMHA_FWD_HEAD, FMHA_BWD_SHORT, FMHA_BWD_PAIR
 * -- are read once per process, on the first launch.  This reads them again; not to be
 * called while another thread is launching.  (No counterpart in the reference.) */
void fmha_reload_overrides(void);

/*
 * Pipe-ceiling microbenchmarks of the compute units (no counterpart in the reference; diagnostic only).
 * mode: 0 exponentials only; 1 matrix instructions (32x32x16 fp16) only, four independent accumulators;
 * 2 both in one wave's instruction stream, nexp (2, 4 or 6) exponentials behind every matrix instruction;
 * 3 matrix instructions on one accumulator (a dependent chain); 4 the two waves of a SIMD split the work,
 * one matrix only, one exponentials only (waves_per_simd must be 2); 5 matrix instructions whose A operand
 * is read from LDS every time; 6 those LDS reads alone; 7 as 2, but the exponentials read registers that the
 * matrix instructions of the previous trip wrote; 8 as 2, but the B operand of every matrix instruction is packed
 * from exponentials of the previous trip; 9-11 the attention kernels' mix of two exponentials, a packing conversion,
 * a packed dot product and an integer add behind every matrix instruction (on registers of their own / reading what
 * the matrix instructions wrote / also feeding their B operand); 12-35 nexp instructions of ONE kind behind every
 * matrix instruction: 12 v_dot2c_f32_f16, 13 v_cvt_f16_f32 + v_pack_b32_f16, 14 v_add_f32, 15 v_pk_add_f16,
 * 16 v_cvt_pk_f16_f32, 17 v_exp_f32, 18 (nexp = 5) two exponentials + one packing conversion + two adds,
 * 19 v_fma_mix_f32, 20 v_mad_u64_u32, 21 v_bitop3_b32, 22 v_mov_b32 with a DPP quad permutation, 23 v_pk_sub_i16,
 * 24 v_perm_b32, 25 v_cndmask_b32, 26 v_mul_f32, 27 v_fma_f32, 28 v_pk_mul_f16, 29 v_max3_f32,
 * 30 v_permlane32_swap_b32, 31 v_cvt_f32_f16, 32 v_dot2_f32_f16, 33 v_sub_f32, 34 v_and_b32, 35 v_pk_ashrrev_i16;
 * 36 nexp v_xor_b32 behind every matrix instruction and 37 the same v_xor_b32 alone (these two also take
 * nexp = 8, 16 and 32: how much vector work a matrix instruction hides, and the plain vector issue rate).
 * random_data: 0 all-zero operands, 1 pseudo-random
 * ones in [-1, 1) -- the board's power management sets the core clock by what the data toggles.
 * Runs `launches` launches (the second half timed with events) of `iters` loop trips -- 4 matrix
 * instructions and / or 4 * nexp exponentials per trip and wave -- with waves_per_simd (1 or 2) waves on
 * every SIMD of the current device and writes
 *   result[0] microseconds per launch, result[1] mean core clock in MHz as the waves saw it,
 *   result[2] matrix TFLOP/s (0 without matrix work), result[3] exponentials (modes 36, 37: v_xor_b32 lane results)
 *   per nanosecond over the chip.
 * Unlike the launch functions it allocates and frees buffers of its own and synchronises the device.
 * Returns 0, or -1 on a bad argument or a HIP error.
 */
int fmha_pipe_probe(int mode, int nexp, int random_data, int waves_per_simd, int iters, int launches,
                    double *result);

/* Library version, "major.minor". */
const char *fmha_version(void);

#ifdef __cplusplus
}
#endif
#endif /* FMHA_CAPI_H_ */
