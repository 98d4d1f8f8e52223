// Internal interface between the C-ABI translation unit and the per-(element type,
// head dim) kernel translation units.  Each kernel TU is compiled once per
// combination with -DFMHA_TU_BF16={0,1} -DFMHA_TU_D={64,128,256} -DFMHA_TU_STRIDED={0,1} and exports
// one dispatcher per pass (the _strided ones read the row maps of the argument block; the
// others assume folded contiguous tensors).
#pragma once
#include <hip/hip_runtime.h>
#include "fmha_fwd_kernel.h"
#include "fmha_bwd_kernel.h"

namespace fmha {

struct FwdVariant {
  int qb;       // 32-query blocks per wave (1 or 2)
  int mask;     // kMaskNone / kMaskPerKey (constant along queries) / kMaskFull
  bool causal;
  int drop;     // 0 none, 1 Philox, 2 tensor / save-intermediates
  bool saving;  // drop == 2: the save-intermediates pass is wanted (plain kernel only)
  bool save_split; // saving beyond the one-pass kernel's range with a caller-provided LSE buffer: forward, then a save kernel
  bool save_once;  // saving for 129 to 512 keys: one launch that keeps a wave's probabilities in registers (head dim 64, folded layout)
  bool stream;     // full mask tensor on aligned rows beyond the one-pass range: the streaming forward (head dim 64, folded layout)
  bool head;       // up to 512 keys, no / per-key mask, no causal mask: the whole-head kernel (head dim 64, folded layout)
  bool short_keys; // sk <= 128 under an aligned full mask tensor: the one-pass kernel (head dim 64, folded layout)
};

// Return 0 on success, 1 if the variant is not built, 2 if the launch failed.
int fwd_dispatch_f16_d64(FwdArgs &a, const FwdVariant &v, hipStream_t s);
int fwd_dispatch_f16_d128(FwdArgs &a, const FwdVariant &v, hipStream_t s);
int fwd_dispatch_bf16_d64(FwdArgs &a, const FwdVariant &v, hipStream_t s);
int fwd_dispatch_bf16_d128(FwdArgs &a, const FwdVariant &v, hipStream_t s);
int fwd_dispatch_f16_d256(FwdArgs &a, const FwdVariant &v, hipStream_t s);
int fwd_dispatch_bf16_d256(FwdArgs &a, const FwdVariant &v, hipStream_t s);
int fwd_dispatch_f16_d256_strided(FwdArgs &a, const FwdVariant &v, hipStream_t s);
int fwd_dispatch_bf16_d256_strided(FwdArgs &a, const FwdVariant &v, hipStream_t s);
int fwd_dispatch_f16_d64_strided(FwdArgs &a, const FwdVariant &v, hipStream_t s);
int fwd_dispatch_f16_d128_strided(FwdArgs &a, const FwdVariant &v, hipStream_t s);
int fwd_dispatch_bf16_d64_strided(FwdArgs &a, const FwdVariant &v, hipStream_t s);
int fwd_dispatch_bf16_d128_strided(FwdArgs &a, const FwdVariant &v, hipStream_t s);

struct BwdVariant {
  int mask;  // kMaskNone / kMaskPerKey / kMaskFull
  bool causal;
  int drop; // 0 none, 1 Philox
  int pair; // causal tile pairing: -1 decide from the amount of work, 0 off, 1 on
  bool short_seq; // sq, sk <= 256 without a full mask tensor: the one-launch kernel (head dim 64)
};

int bwd_dispatch_f16_d64(BwdArgs &a, const BwdVariant &v, hipStream_t s);
int bwd_dispatch_f16_d128(BwdArgs &a, const BwdVariant &v, hipStream_t s);
int bwd_dispatch_bf16_d64(BwdArgs &a, const BwdVariant &v, hipStream_t s);
int bwd_dispatch_bf16_d128(BwdArgs &a, const BwdVariant &v, hipStream_t s);
int bwd_dispatch_f16_d256(BwdArgs &a, const BwdVariant &v, hipStream_t s);
int bwd_dispatch_bf16_d256(BwdArgs &a, const BwdVariant &v, hipStream_t s);
int bwd_dispatch_f16_d256_strided(BwdArgs &a, const BwdVariant &v, hipStream_t s);
int bwd_dispatch_bf16_d256_strided(BwdArgs &a, const BwdVariant &v, hipStream_t s);
int bwd_dispatch_f16_d64_strided(BwdArgs &a, const BwdVariant &v, hipStream_t s);
int bwd_dispatch_f16_d128_strided(BwdArgs &a, const BwdVariant &v, hipStream_t s);
int bwd_dispatch_bf16_d64_strided(BwdArgs &a, const BwdVariant &v, hipStream_t s);
int bwd_dispatch_bf16_d128_strided(BwdArgs &a, const BwdVariant &v, hipStream_t s);

// e4m3 forward (fmha_fwd_fp8.hip): 0 ok, 1 not built, 2 launch failed
struct Fp8Args;
int fwd_fp8_dispatch(const Fp8Args &a, int d, bool out_bf16, bool causal, hipStream_t s);

} // namespace fmha
