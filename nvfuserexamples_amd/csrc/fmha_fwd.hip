// Instantiates the forward kernel for one (element type, head dim, row layout kind) triple, chosen
// with -DFMHA_TU_BF16={0,1} -DFMHA_TU_D={64,128,256} -DFMHA_TU_STRIDED={0,1}, and exports its dispatcher.
#include "fmha_launch.h"
#include "fmha_fwd_pipe.h"
#ifndef FMHA_TU_STRIDED
#define FMHA_TU_STRIDED 0
#endif
#if FMHA_TU_D == 64 && !FMHA_TU_STRIDED
#define FMHA_TU_SHORT 1
#include "fmha_fwd_short.h"
#include "fmha_fwd_save.h"
#include "fmha_fwd_stream.h"
#include "fmha_fwd_stream_save.h"
#include "fmha_fwd_head.h"
#else
#define FMHA_TU_SHORT 0
#if FMHA_TU_D == 64
#include "fmha_fwd_short.h" // run-time row layouts: its builds without a full mask tensor
#include "fmha_fwd_head.h"  // and the whole-head kernel
#endif
#endif

#if FMHA_TU_BF16
#define FMHA_TU_T __bf16
#define FMHA_TU_TNAME bf16
#else
#define FMHA_TU_T _Float16
#define FMHA_TU_TNAME f16
#endif
#if FMHA_TU_STRIDED
#define FMHA_CAT3(a, b, c) a##b##_d##c##_strided
#else
#define FMHA_CAT3(a, b, c) a##b##_d##c
#endif
#define FMHA_NAME(t, d) FMHA_CAT3(fwd_dispatch_, t, d)

namespace fmha {
namespace {

#ifndef FMHA_FWD_NW
#define FMHA_FWD_NW 4
#endif
constexpr int kNW = FMHA_FWD_NW;
constexpr bool kStrided = FMHA_TU_STRIDED != 0;

template <int QB, int MASK, bool CAUSAL, int DROP, bool kPipe = (DROP != 2)> int launch(FwdArgs &a, hipStream_t s) {
  constexpr int kLds = kPipe ? PipeCfg<FMHA_TU_D, QB>::lds_bytes(kNW) : FwdCfg<FMHA_TU_D>::LDS_BYTES;
  // the save pass (and tensor dropout at head dim 128) runs on the plain loop; everything else is
  // software-pipelined
  auto kern = [] {
    if constexpr (!kPipe) return fmha_fwd_kernel<FMHA_TU_T, FMHA_TU_D, QB, kNW, MASK, CAUSAL, DROP, kStrided && FMHA_TU_D == 256>;
    else return fmha_fwd_pipe_kernel<FMHA_TU_T, FMHA_TU_D, QB, kNW, MASK, CAUSAL, DROP, kStrided>;
  }();
  // once per kernel: allow the dynamic LDS size, and for the persistent kernel find how many
  // workgroups the device keeps resident (that is its grid size)
  static const int resident = [&]() -> int {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, kLds) !=
        hipSuccess)
      return -1;
    if (!kPipe) return 0;
    int dev = 0, cus = 0, per_cu = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void *>(kern), kNW * 64, kLds) !=
            hipSuccess ||
        cus <= 0 || per_cu <= 0)
      return -1;
    return cus * per_cu;
  }();
  if (resident < 0) return 2;
  constexpr int QT = kNW * QB * 32;
  a.nqt = (a.sq + QT - 1) / QT;
  long long nblk = (long long)a.bh * a.nqt;
  if (nblk > 0x7fffffffLL) return 2;
  if (kPipe && nblk > resident) nblk = resident;
  a.bal_rows = 0;
  if (kPipe && MASK == kMaskPerKey && !CAUSAL && a.mask_div > 0 && a.bh % a.mask_div == 0) {
    // shapes whose mask rows can be dealt to the workgroups by length (see FwdArgs::bal_rows): an
    // additive mask (its values are compared as they are), rows of whole 16-byte pieces, at most 64
    // pieces of 512 keys in all
    const long long items = (long long)a.bh * a.nqt, ipr = (long long)a.mask_div * a.nqt, rows = a.bh / a.mask_div;
    const bool shape = nblk % ipr == 0 && items % nblk == 0 && items / nblk >= 2 && items / nblk <= 4 &&
                       rows == items / nblk * (nblk / ipr);
    const bool mask_ok = a.mask_a == FMHA_LOG2E && a.mask_b == 0.f && a.sk % 8 == 0 && a.sk > 128 && a.sk <= 1024 &&
                         rows * ((a.sk + 511) / 512) <= 64 && a.mask_sb % 8 == 0 &&
                         (reinterpret_cast<uintptr_t>(a.mask) & 15) == 0;
    if (shape && mask_ok && !a.kv_len && a.sk_whole == 0 && !(a.flags & kFwdFlagNoTrim)) {
      a.bal_rows = (int32_t)rows;
      a.bal_ipr = (int32_t)ipr;
      a.bal_R = (int32_t)(nblk / ipr);
      a.bal_inv_ipr = 1.f / (float)ipr;
    }
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)nblk), dim3(kNW * 64), kLds, s, a);
  return hipGetLastError() == hipSuccess ? 0 : 2;
}

#if FMHA_TU_D == 64
// short key ranges in one pass: under a full mask tensor (the reference's operators at their own shape), and under
// no mask / a per-key mask / valid key counts, without dropout or with the Philox rule
template <int MASK, int DROP, bool SAVE, bool FULL> int launch_short_as(FwdArgs &a, hipStream_t s) {
  static_assert(MASK != kMaskFull || !kStrided, "full mask tensors: folded layout only");
  auto kern = [] {
    if constexpr (MASK == kMaskFull) return fmha_fwd_short_kernel<FMHA_TU_T, DROP, SAVE, FULL>;
    else return fmha_fwd_short_kernel_keymask<FMHA_TU_T, MASK, DROP, FULL, kStrided>;
  }();
  constexpr int kLds = MASK == kMaskFull ? ShortCfg::LDS_BYTES : ShortCfg::LDS_BYTES_KEYMASK;
  static const bool ready = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                                hipFuncAttributeMaxDynamicSharedMemorySize, kLds) == hipSuccess;
  if (!ready) return 2;
  a.nqt = (a.sq + ShortCfg::QT - 1) / ShortCfg::QT;
  const long long nblk = (long long)a.bh * a.nqt;
  if (nblk > 0x7fffffffLL) return 2;
  hipLaunchKernelGGL(kern, dim3((unsigned)nblk), dim3(ShortCfg::NW * 64), kLds, s, a);
  return hipGetLastError() == hipSuccess ? 0 : 2;
}
// (more than 96 keys: every 32-key block exists, and the kernel is built without the conditions around them)
template <int MASK, int DROP, bool SAVE> int launch_short(FwdArgs &a, hipStream_t s) {
  return a.sk > ShortCfg::SKMAX - 32 ? launch_short_as<MASK, DROP, SAVE, true>(a, s)
                                     : launch_short_as<MASK, DROP, SAVE, false>(a, s);
}
#endif

#if FMHA_TU_SHORT
// the saved outputs of the save-intermediates operator, from the row log-sum-exp of a forward launch
int launch_save(FwdArgs &a, hipStream_t s) {
  auto kern = fmha_fwd_save_kernel<FMHA_TU_T>;
  a.nqt = (a.sq + SaveCfg::QT - 1) / SaveCfg::QT;
  const long long nblk = (long long)a.bh * a.nqt;
  if (nblk > 0x7fffffffLL) return 2;
  hipLaunchKernelGGL(kern, dim3((unsigned)nblk), dim3(SaveCfg::NW * 64), SaveCfg::LDS_BYTES, s, a);
  return hipGetLastError() == hipSuccess ? 0 : 2;
}
#endif

#if FMHA_TU_SHORT
// long key ranges under a full mask tensor (and a dropout tensor): the streaming forward
template <bool DROPT> int launch_stream(FwdArgs &a, hipStream_t s) {
  auto kern = fmha_fwd_stream_kernel<FMHA_TU_T, DROPT>;
  a.nqt = (a.sq + StreamCfg::QT - 1) / StreamCfg::QT;
  const long long nblk = (long long)a.bh * a.nqt;
  if (nblk > 0x7fffffffLL) return 2;
  hipLaunchKernelGGL(kern, dim3((unsigned)nblk), dim3(StreamCfg::NW * 64), StreamCfg::LDS_BYTES, s, a);
  return hipGetLastError() == hipSuccess ? 0 : 2;
}
#endif

#if FMHA_TU_SHORT
// the save-intermediates operator for 129 to 512 keys in one launch (one wave per SIMD: the whole register file)
int launch_stream_save(FwdArgs &a, hipStream_t s) {
  auto kern = fmha_fwd_stream_save_kernel<FMHA_TU_T>;
  if (a.sk > StreamSaveCfg::SKMAX) return 1;
  a.nqt = (a.sq + StreamSaveCfg::QT - 1) / StreamSaveCfg::QT;
  const long long nblk = (long long)a.bh * a.nqt;
  if (nblk > 0x7fffffffLL) return 2;
  hipLaunchKernelGGL(kern, dim3((unsigned)nblk), dim3(StreamSaveCfg::NW * 64), StreamSaveCfg::LDS_BYTES, s, a);
  return hipGetLastError() == hipSuccess ? 0 : 2;
}
#endif

#if FMHA_TU_D == 64
// a whole head's K and V resident in LDS: one persistent workgroup per compute unit
#ifndef FMHA_HEAD_QB
#define FMHA_HEAD_QB 2
#endif
template <int MASK, int DROP> int launch_head(FwdArgs &a, hipStream_t s) {
  using HC = HeadCfgT<FMHA_HEAD_QB>;
  auto kern = fmha_fwd_head_kernel<FMHA_TU_T, FMHA_HEAD_QB, MASK, DROP, kStrided>;
  static const int resident = [&]() -> int {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            HC::LDS_BYTES) != hipSuccess)
      return -1;
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      return -1;
    return cus;
  }();
  if (resident < 0) return 2;
  if (a.sk > HC::MAXK) return 1;
  a.nqt = (a.sq + HC::QT - 1) / HC::QT;
  long long nblk = (long long)a.bh * a.nqt;
  if (nblk > 0x7fffffffLL) return 2;
  if (nblk > resident) nblk = resident;
  hipLaunchKernelGGL(kern, dim3((unsigned)nblk), dim3(HC::NT), HC::LDS_BYTES, s, a);
  return hipGetLastError() == hipSuccess ? 0 : 2;
}
#endif

template <int QB, int MASK, bool CAUSAL> int by_drop(FwdArgs &a, int drop, hipStream_t s) {
  if (drop == 0) return launch<QB, MASK, CAUSAL, 0>(a, s);
  if (drop == 1) return launch<QB, MASK, CAUSAL, 1>(a, s);
  return 1;
}

template <int QB, int MASK> int by_causal(FwdArgs &a, const FwdVariant &v, hipStream_t s) {
  return v.causal ? by_drop<QB, MASK, true>(a, v.drop, s) : by_drop<QB, MASK, false>(a, v.drop, s);
}

#ifdef FMHA_DEV_MINIMAL
// development builds: only the variants the headline benchmark uses
template <int QB> int by_mask(FwdArgs &a, const FwdVariant &v, hipStream_t s) {
  if (v.causal || v.drop) return 1;
  if (v.mask == kMaskPerKey) return launch<1, kMaskPerKey, false, 0>(a, s);
  if (v.mask == kMaskNone) return launch<1, kMaskNone, false, 0>(a, s);
  return 1;
}
#else
template <int QB> int by_mask(FwdArgs &a, const FwdVariant &v, hipStream_t s) {
  if (v.mask == kMaskPerKey) return by_causal<QB, kMaskPerKey>(a, v, s);
  if (v.mask == kMaskFull) return by_causal<QB, kMaskFull>(a, v, s);
  return by_causal<QB, kMaskNone>(a, v, s);
}
#endif

} // namespace

#if FMHA_TU_D == 256
// Head dim 256: built for coverage, not tuned.  Every variant runs on the plain (not software-pipelined)
// loop at one wave per SIMD: the output accumulators alone take 128 registers per lane.
namespace { // (per translation unit: the element type differs between units of the same name)
template <int MASK, bool CAUSAL> int plain_by_drop(FwdArgs &a, int drop, hipStream_t s) {
  if (drop == 0) return launch<1, MASK, CAUSAL, 0, false>(a, s);
  if (drop == 1) return launch<1, MASK, CAUSAL, 1, false>(a, s);
  if (drop == 2 && !CAUSAL) return launch<1, MASK, false, 2, false>(a, s);
  return 1;
}
} // namespace

int FMHA_NAME(FMHA_TU_TNAME, FMHA_TU_D)(FwdArgs &a, const FwdVariant &v, hipStream_t s) {
  if (v.qb == 2 || v.short_keys || v.save_split || v.save_once || v.stream || v.head || (kStrided && v.drop == 2)) return 1;
  if (v.mask == kMaskPerKey)
    return v.causal ? plain_by_drop<kMaskPerKey, true>(a, v.drop, s) : plain_by_drop<kMaskPerKey, false>(a, v.drop, s);
  if (v.mask == kMaskFull)
    return v.causal ? plain_by_drop<kMaskFull, true>(a, v.drop, s) : plain_by_drop<kMaskFull, false>(a, v.drop, s);
  return v.causal ? plain_by_drop<kMaskNone, true>(a, v.drop, s) : plain_by_drop<kMaskNone, false>(a, v.drop, s);
}
#else
int FMHA_NAME(FMHA_TU_TNAME, FMHA_TU_D)(FwdArgs &a, const FwdVariant &v, hipStream_t s) {
#if defined(FMHA_DEV_MINIMAL) || FMHA_TU_STRIDED
  if (v.drop == 2 || v.qb == 2) return 1; // folded layout only
#endif
#if FMHA_TU_D == 64 && FMHA_TU_STRIDED
  if (v.head && !v.short_keys) { // run-time row layouts: the whole-head kernel
    if (v.causal || v.drop == 2 || v.mask == kMaskFull) return 1;
    if (v.mask == kMaskPerKey) return v.drop ? launch_head<kMaskPerKey, 1>(a, s) : launch_head<kMaskPerKey, 0>(a, s);
    return v.drop ? launch_head<kMaskNone, 1>(a, s) : launch_head<kMaskNone, 0>(a, s);
  }
  if (v.short_keys) { // run-time row layouts: the one-pass kernel's builds without a full mask tensor
    if (v.causal || v.mask == kMaskFull || v.drop == 2 || v.saving) return 1;
    if (v.mask == kMaskPerKey)
      return v.drop == 1 ? launch_short<kMaskPerKey, 1, false>(a, s) : launch_short<kMaskPerKey, 0, false>(a, s);
    return v.drop == 1 ? launch_short<kMaskNone, 1, false>(a, s) : launch_short<kMaskNone, 0, false>(a, s);
  }
#endif
#if FMHA_TU_SHORT
  if (v.short_keys) {
    if (v.causal) return 1;
    if (v.mask == kMaskFull) {
      if (v.drop == 1) return 1;
      if (v.saving) return launch_short<kMaskFull, 2, true>(a, s);
      return v.drop == 2 ? launch_short<kMaskFull, 2, false>(a, s) : launch_short<kMaskFull, 0, false>(a, s);
    }
    if (v.drop == 2 || v.saving) return 1;
    if (v.mask == kMaskPerKey)
      return v.drop == 1 ? launch_short<kMaskPerKey, 1, false>(a, s) : launch_short<kMaskPerKey, 0, false>(a, s);
    return v.drop == 1 ? launch_short<kMaskNone, 1, false>(a, s) : launch_short<kMaskNone, 0, false>(a, s);
  }
  if (v.save_once) return launch_stream_save(a, s);
  if (v.save_split) { // forward with LSE, then the saved outputs from that LSE
    const int rc = v.stream ? launch_stream<true>(a, s) : launch<1, kMaskFull, false, 2, true>(a, s);
    return rc ? rc : launch_save(a, s);
  }
  if (v.stream) return v.drop == 2 ? launch_stream<true>(a, s) : launch_stream<false>(a, s);
  if (v.head) {
    if (v.causal || v.drop == 2 || v.mask == kMaskFull) return 1;
    if (v.mask == kMaskPerKey) return v.drop ? launch_head<kMaskPerKey, 1>(a, s) : launch_head<kMaskPerKey, 0>(a, s);
    return v.drop ? launch_head<kMaskNone, 1>(a, s) : launch_head<kMaskNone, 0>(a, s);
  }
#else
  if (v.short_keys || v.save_split || v.save_once || v.stream || v.head) return 1;
#endif
  if (v.drop == 2) { // tensor dropout / save-intermediates: the legacy ops' shape class
    if (v.causal) return 1;
#if FMHA_TU_D == 64
    if (!v.saving) { // dropout tensor alone: pipelined kernel
      if (v.mask == kMaskPerKey) return launch<1, kMaskPerKey, false, 2, true>(a, s);
      if (v.mask == kMaskFull) return launch<1, kMaskFull, false, 2, true>(a, s);
      return launch<1, kMaskNone, false, 2, true>(a, s);
    }
#endif
    if (v.mask == kMaskPerKey) return launch<1, kMaskPerKey, false, 2>(a, s);
    if (v.mask == kMaskFull) return launch<1, kMaskFull, false, 2>(a, s);
    return launch<1, kMaskNone, false, 2>(a, s);
  }
#if FMHA_TU_D == 64
  // two query blocks per wave: only where their accumulators fit the register file and only
  // for the variants the host ever selects them for
  if (v.qb == 2) {
    if (v.causal || v.drop != 0 || v.mask == kMaskFull) return 1;
    return v.mask == kMaskPerKey ? launch<2, kMaskPerKey, false, 0>(a, s) : launch<2, kMaskNone, false, 0>(a, s);
  }
#endif
  return by_mask<1>(a, v, s);
}
#endif

} // namespace fmha
