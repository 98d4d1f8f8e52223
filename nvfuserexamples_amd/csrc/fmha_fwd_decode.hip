// The decode-step forward kernels (head dim 64 and 128; fp16, bf16 or e4m3 inputs; 1 / 2 / 4 query rows) and their
// dispatchers.
#include "fmha_fwd_decode.h"

namespace fmha {
namespace {

template <typename T, typename TO, int D, int NQ, bool MASK> int launch(const DecodeArgs &a, hipStream_t s) {
  const long long nblk = (long long)a.bh * a.pieces;
  if (nblk > 0x7fffffffLL) return 2;
  hipLaunchKernelGGL((fmha_fwd_decode_kernel<T, TO, D, NQ, MASK>), dim3((unsigned)nblk), dim3(kDecodeWaves * 64), 0, s, a);
  return hipGetLastError() == hipSuccess ? 0 : 2;
}

template <typename T, typename TO, int D, int NQ> int by_mask(const DecodeArgs &a, hipStream_t s) {
  return a.mask ? launch<T, TO, D, NQ, true>(a, s) : launch<T, TO, D, NQ, false>(a, s);
}

template <typename T, typename TO, int D> int by_rows(const DecodeArgs &a, hipStream_t s) {
  if (a.sq == 1) return by_mask<T, TO, D, 1>(a, s);
  if (a.sq == 2) return by_mask<T, TO, D, 2>(a, s);
  if (a.sq <= 4) return by_mask<T, TO, D, 4>(a, s);
  return 1; // (measured with eight rows: 0.38-0.53 of the HBM peak where the matrix-pipe kernels reach 0.43-0.73)
}

} // namespace

int fwd_decode_dispatch(const DecodeArgs &a, int d, bool bf16, hipStream_t s) {
  if (d == 64) return bf16 ? by_rows<__bf16, __bf16, 64>(a, s) : by_rows<_Float16, _Float16, 64>(a, s);
  if (d == 128) return bf16 ? by_rows<__bf16, __bf16, 128>(a, s) : by_rows<_Float16, _Float16, 128>(a, s);
  return 1;
}

int fwd_decode_fp8_dispatch(const DecodeArgs &a, int d, bool out_bf16, hipStream_t s) {
  if (d == 64) return out_bf16 ? by_rows<uint8_t, __bf16, 64>(a, s) : by_rows<uint8_t, _Float16, 64>(a, s);
  if (d == 128) return out_bf16 ? by_rows<uint8_t, __bf16, 128>(a, s) : by_rows<uint8_t, _Float16, 128>(a, s);
  return 1;
}

} // namespace fmha
