// The e4m3 forward kernels (head dim 64 and 128, fp16 / bf16 output) and their dispatcher.
#include "fmha_fwd_fp8.h"
#include "fmha_launch.h"

namespace fmha {
namespace {

template <typename K> int set_lds(K kern, int bytes) {
  return hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                             bytes) == hipSuccess ? 0 : 2;
}

template <typename TO, int D, bool CAUSAL, bool MASK> int launch(const Fp8Args &a, hipStream_t s) {
  using C = Fp8Cfg<D>;
  auto kern = fmha_fwd_fp8_kernel<TO, D, CAUSAL, MASK>;
  static const int attr = set_lds(kern, C::LDS_BYTES);
  if (attr) return 2;
  const long long nblk = (long long)a.bh * ((a.sq + C::QT - 1) / C::QT);
  if (nblk > 0x7fffffffLL) return 2;
  hipLaunchKernelGGL(kern, dim3((unsigned)nblk), dim3(C::NT), C::LDS_BYTES, s, a);
  return hipGetLastError() == hipSuccess ? 0 : 2;
}

template <typename TO, int D> int by_variant(const Fp8Args &a, bool causal, hipStream_t s) {
  if (a.mask) return causal ? launch<TO, D, true, true>(a, s) : launch<TO, D, false, true>(a, s);
  return causal ? launch<TO, D, true, false>(a, s) : launch<TO, D, false, false>(a, s);
}

} // namespace

int fwd_fp8_dispatch(const Fp8Args &a, int d, bool out_bf16, bool causal, hipStream_t s) {
  if (d == 64) return out_bf16 ? by_variant<__bf16, 64>(a, causal, s) : by_variant<_Float16, 64>(a, causal, s);
  if (d == 128) return out_bf16 ? by_variant<__bf16, 128>(a, causal, s) : by_variant<_Float16, 128>(a, causal, s);
  return 1;
}

} // namespace fmha
