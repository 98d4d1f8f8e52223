// Instantiates the backward kernels for one (element type, head dim, row layout kind) triple, chosen
// with -DFMHA_TU_BF16={0,1} -DFMHA_TU_D={64,128,256} -DFMHA_TU_STRIDED={0,1}, and exports their dispatcher.
#include "fmha_launch.h"
#ifndef FMHA_TU_STRIDED
#define FMHA_TU_STRIDED 0
#endif
#if FMHA_TU_D == 64
#define FMHA_TU_SHORT 1
#include "fmha_bwd_short.h"
#else
#define FMHA_TU_SHORT 0
#endif
#if FMHA_TU_D == 256 || defined(FMHA_BWD_FORCE_WIDE) // (the second: development builds, to measure the wave-pair kernel at narrower heads)
#define FMHA_TU_WIDE 1
#include "fmha_bwd_wide.h"
#else
#define FMHA_TU_WIDE 0
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
#define FMHA_NAME(t, d) FMHA_CAT3(bwd_dispatch_, t, d)

namespace fmha {
namespace {

constexpr int kNW = 4;
constexpr int kQB = 1; // 32-query blocks per wave in the dQ kernel
constexpr int kKB = 1; // 32-key blocks per wave in the dK/dV kernel
constexpr bool kStrided = FMHA_TU_STRIDED != 0;

template <typename K> int set_lds(K kern, int bytes) {
  return hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                             bytes) == hipSuccess ? 0 : 2;
}

template <int MASK, bool CAUSAL, int DROP> int launch(BwdArgs &a, int pair, hipStream_t s) {
  constexpr int kLdsQ = BwdCfg<FMHA_TU_D, bwd_dq_tile_rows<FMHA_TU_D>()>::LDS_BYTES;
  auto kq = fmha_bwd_dq_kernel<FMHA_TU_T, FMHA_TU_D, kQB, kNW, MASK, CAUSAL, DROP, kStrided>;
#if FMHA_TU_WIDE
  // head dim 256: the dK / dV work of a key block is split between two waves (fmha_bwd_wide.h; at head
  // dims 128 and 64 the same kernel measured level with and a third slower than the one-wave kernel)
  using CfgK = BwdWideCfg<FMHA_TU_D, MASK>;
  constexpr int kLdsK = CfgK::LDS_BYTES;
  constexpr int kNWK = CfgK::NW, KT = CfgK::KT;
  auto kk = fmha_bwd_dkdv_wide_kernel<FMHA_TU_T, FMHA_TU_D, MASK, CAUSAL, DROP, kStrided>;
#else
  using CfgK = BwdCfg<FMHA_TU_D, bwd_dkdv_tile_rows<FMHA_TU_D, CAUSAL, DROP>()>;
  constexpr int kLdsK = CfgK::LDS_BYTES + (MASK == kMaskFull ? CfgK::MASK_BYTES : 0);
  constexpr int kNWK = kNW, KT = kNW * kKB * 32;
  auto kk = fmha_bwd_dkdv_kernel<FMHA_TU_T, FMHA_TU_D, kKB, kNW, MASK, CAUSAL, DROP, kStrided>;
#endif
  static_assert(kLdsQ <= 160 * 1024 && kLdsK <= 160 * 1024, "tiles do not fit the LDS of a compute unit");
  static const int attr = set_lds(kq, kLdsQ) | set_lds(kk, kLdsK);
  if (attr) return 2;
  constexpr int QT = kNW * kQB * 32;
  // dQ first: it also writes delta, which the dK/dV kernel reads (same stream => ordered)
  // causal: workgroups take pairs of tiles (see the kernels) when that leaves at least two
  // rounds of workgroups for the device
  static const int cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
      n = 0;
    return n;
  }();
  a.ntile = (a.sq + QT - 1) / QT;
  auto want_pair = [&](int ntile) {
    if (!CAUSAL) return false;
    return pair >= 0 ? pair != 0 : (long long)a.bh * ((ntile + 1) / 2) >= 4LL * cus;
  };
  a.pair = want_pair(a.ntile);
  long long nblk = (long long)a.bh * (a.pair ? (a.ntile + 1) / 2 : a.ntile);
  if (nblk > 0x7fffffffLL) return 2;
  hipLaunchKernelGGL(kq, dim3((unsigned)nblk), dim3(kNW * 64), kLdsQ, s, a);
  if (hipGetLastError() != hipSuccess) return 2;
  a.ntile = (a.sk + KT - 1) / KT;
  a.pair = want_pair(a.ntile);
  nblk = (long long)a.bh * (a.pair ? (a.ntile + 1) / 2 : a.ntile);
  if (nblk > 0x7fffffffLL) return 2;
  hipLaunchKernelGGL(kk, dim3((unsigned)nblk), dim3(kNWK * 64), kLdsK, s, a);
  return hipGetLastError() == hipSuccess ? 0 : 2;
}

#if FMHA_TU_SHORT
// sq, sk <= 128: one workgroup per head computes dQ, dK and dV from one copy of the head in LDS
template <int DROP, int SMAX, bool CAUSAL> int launch_short(BwdArgs &a, hipStream_t s) {
  using Cfg = BwdShortCfg<SMAX>;
  auto kern = fmha_bwd_short_kernel<FMHA_TU_T, DROP, SMAX, CAUSAL, kStrided>;
  static const int attr = set_lds(kern, Cfg::LDS_BYTES);
  if (attr) return 2;
  hipLaunchKernelGGL(kern, dim3((unsigned)a.bh), dim3(Cfg::NW * 64), Cfg::LDS_BYTES, s, a);
  return hipGetLastError() == hipSuccess ? 0 : 2;
}
#endif

template <int MASK, bool CAUSAL> int by_drop(BwdArgs &a, const BwdVariant &v, hipStream_t s) {
  if (v.drop == 0) return launch<MASK, CAUSAL, 0>(a, v.pair, s);
  if (v.drop == 1) return launch<MASK, CAUSAL, 1>(a, v.pair, s);
  return 1;
}

} // namespace

int FMHA_NAME(FMHA_TU_TNAME, FMHA_TU_D)(BwdArgs &a, const BwdVariant &v, hipStream_t s) {
#if FMHA_TU_SHORT
  if (v.short_seq) {
    const bool small = a.sq <= 128 && a.sk <= 128;
    if (v.causal) {
      if (small) return v.drop == 1 ? launch_short<1, 128, true>(a, s) : launch_short<0, 128, true>(a, s);
      return v.drop == 1 ? launch_short<1, 256, true>(a, s) : launch_short<0, 256, true>(a, s);
    }
    if (small) return v.drop == 1 ? launch_short<1, 128, false>(a, s) : launch_short<0, 128, false>(a, s);
    return v.drop == 1 ? launch_short<1, 256, false>(a, s) : launch_short<0, 256, false>(a, s);
  }
#else
  if (v.short_seq) return 1;
#endif
  if (v.mask == kMaskPerKey)
    return v.causal ? by_drop<kMaskPerKey, true>(a, v, s) : by_drop<kMaskPerKey, false>(a, v, s);
  if (v.mask == kMaskFull)
    return v.causal ? by_drop<kMaskFull, true>(a, v, s) : by_drop<kMaskFull, false>(a, v, s);
  return v.causal ? by_drop<kMaskNone, true>(a, v, s) : by_drop<kMaskNone, false>(a, v, s);
}

} // namespace fmha
