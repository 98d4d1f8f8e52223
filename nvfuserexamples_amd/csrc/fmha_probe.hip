// Pipe-ceiling microbenchmarks of the gfx950 compute unit, exported through the C ABI as
// fmha_pipe_probe.  They answer, on the board the library runs on, what the attention kernels can
// reach at best: the matrix pipe alone, the exponential alone, both in one wave's instruction
// stream, both on different waves of one SIMD, and LDS operand reads beside the matrix pipe -- each
// on all-zero and on pseudo-random operands, because the board's power management sets the core
// clock by what the data toggles.  Diagnostic only: no attention kernel depends on this file.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fmha_common.h"

namespace fmha {
namespace {

// out[3 * workgroup + {0,1,2}] = core clock cycles, 100 MHz ticks, a value that keeps the work alive
template <int MODE, int NEXP>
__global__ __launch_bounds__(512) void pipe_probe_kernel(unsigned long long *out, const _Float16 *src, int iters) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int tid = threadIdx.x;
  const int w = tid >> 6;
  const size_t lane = (size_t)blockIdx.x * blockDim.x + tid;
  f16x8 a, b;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    a[j] = src[lane * 16 + j];
    b[j] = src[lane * 16 + 8 + j];
  }
  // LDS operand area: every lane's 16 bytes of four 1 KiB-per-wave slabs
  if (MODE == 5 || MODE == 6) {
#pragma unroll
    for (int i = 0; i < 4; ++i) *(f16x8 *)(lds + (w * 4 + i) * 1024 + (tid & 63) * 16) = i & 1 ? b : a;
    __syncthreads();
  }
  f32x16 acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
  float v[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = (float)a[j];
  // MODE 4: the waves of a SIMD split the work, waves 0-3 matrix only, waves 4-7 exponentials only
  const bool do_mfma = MODE == 1 || (MODE == 4 && w < 4);
  const bool do_exp = MODE == 0 || MODE == 2 || (MODE == 4 && w >= 4);
  f16x8 la[4] = {a, b, a, b};
  f16x8 bw[2] = {b, a};
  float pe[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, rsum = 0.f;
  typedef _Float16 h2p __attribute__((ext_vector_type(2)));
  h2p ppk[4] = {{a[0], a[1]}, {a[2], a[3]}, {b[0], b[1]}, {b[2], b[3]}};
  uint32_t cnt = (uint32_t)tid;
  uint32_t iv[8];
  unsigned long long lv[4] = {1ull, 2ull, 3ull, 4ull};
#pragma unroll
  for (int j = 0; j < 8; ++j) iv[j] = (uint32_t)tid * 2654435761u + (uint32_t)j;
  const unsigned long long r0 = __builtin_amdgcn_s_memrealtime(), c0 = __builtin_readcyclecounter();
  for (int it = 0; it < iters; ++it) {
    if (MODE == 3) { // dependent chain: one accumulator
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[0], 0, 0, 0);
    } else if (MODE == 2) { // one stream: NEXP exponentials behind every matrix instruction
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[i], 0, 0, 0);
#pragma unroll
        for (int j = 0; j < NEXP; ++j) v[(i * NEXP + j) & 7] = __builtin_amdgcn_exp2f(v[(i * NEXP + j) & 7] * 0.5f - 1.0f);
        __builtin_amdgcn_sched_barrier(0);
      }
    } else if (MODE == 36 || MODE == 37) {
      // NEXP full-rate vector instructions (v_xor_b32) behind every matrix instruction (36) or alone (37)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (MODE == 36) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[i], 0, 0, 0);
#pragma unroll
        for (int j = 0; j < NEXP; ++j) {
          const int r = (i * NEXP + j) & 7;
          asm volatile("v_xor_b32 %0, %0, %1" : "+v"(iv[r]) : "v"(iv[(r + 3) & 7]));
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    } else if (MODE >= 20 && MODE <= 35) {
      // NEXP instructions of one kind (inline assembly, registers of their own) behind every matrix instruction
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[i], 0, 0, 0);
#pragma unroll
        for (int j = 0; j < NEXP; ++j) {
          const int r = (i * NEXP + j) & 7;
          uint32_t &x = iv[r], &y = iv[(r + 3) & 7];
          if (MODE == 20) asm volatile("v_mad_u64_u32 %0, vcc, %1, %2, %0" : "+v"(lv[r & 3]) : "v"(x), "v"(y) : "vcc");
          if (MODE == 21) asm volatile("v_bitop3_b32 %0, %0, %1, %2 bitop3:0x96" : "+v"(x) : "v"(y), "v"(iv[(r + 5) & 7]));
          if (MODE == 22) asm volatile("v_mov_b32_dpp %0, %1 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf" : "+v"(x) : "v"(y));
          if (MODE == 23) asm volatile("v_pk_sub_i16 %0, %0, %1" : "+v"(x) : "v"(y));
          if (MODE == 24) asm volatile("v_perm_b32 %0, %0, %1, %2" : "+v"(x) : "v"(y), "v"(iv[(r + 5) & 7]));
          if (MODE == 25) asm volatile("v_cndmask_b32 %0, %0, %1, vcc" : "+v"(x) : "v"(y) : "vcc");
          if (MODE == 26) asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x) : "v"(y));
          if (MODE == 27) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x) : "v"(y), "v"(iv[(r + 5) & 7]));
          if (MODE == 28) asm volatile("v_pk_mul_f16 %0, %0, %1" : "+v"(x) : "v"(y));
          if (MODE == 29) asm volatile("v_max3_f32 %0, %0, %1, %2" : "+v"(x) : "v"(y), "v"(iv[(r + 5) & 7]));
          if (MODE == 30) asm volatile("v_permlane32_swap_b32 %0, %1" : "+v"(x), "+v"(y));
          if (MODE == 31) asm volatile("v_cvt_f32_f16 %0, %1" : "=v"(x) : "v"(y));
          if (MODE == 32) asm volatile("v_dot2_f32_f16 %0, %1, %2, %0" : "+v"(x) : "v"(y), "v"(iv[(r + 5) & 7]));
          if (MODE == 33) asm volatile("v_sub_f32 %0, %0, %1" : "+v"(x) : "v"(y));
          if (MODE == 34) asm volatile("v_and_b32 %0, %0, %1" : "+v"(x) : "v"(y));
          if (MODE == 35) asm volatile("v_pk_ashrrev_i16 %0, 15, %0" : "+v"(x));
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    } else if (MODE >= 12 && MODE <= 19) {
      // NEXP instructions of one kind behind every matrix instruction, on registers of their own: 12 packed dot
      // product (v_dot2c_f32_f16), 13 packing conversion (v_cvt_pk_f16_f32), 14 fp32 add, 15 packed fp16 add,
      // 16 packing conversion of two fp32 (v_cvt_pk_f16_f32), 17 exponential alone, 18 (with n = 5) the softmax mix
      // without a dot product: two exponentials, one packing conversion, two fp32 adds; 19 fp32 += one half of a
      // packed fp16 pair (v_fma_mix_f32)
      typedef _Float16 h2 __attribute__((ext_vector_type(2)));
      const h2 one = {(_Float16)1.f, (_Float16)1.f};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[i], 0, 0, 0);
#pragma unroll
        for (int j = 0; j < NEXP; ++j) {
          const int r = (i * NEXP + j) & 7;
          if (MODE == 12) v[r] = __builtin_amdgcn_fdot2(ppk[r & 3], one, v[r], false);
          if (MODE == 13) {
            const h2 t = {(_Float16)v[r], (_Float16)pe[r]};
            ppk[r & 3] = t;
            asm volatile("" : "+v"(ppk[r & 3]));
          }
          if (MODE == 14) v[r] = v[r] + pe[r];
          if (MODE == 15) ppk[r & 3] = ppk[r & 3] + one;
          if (MODE == 16) asm volatile("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(ppk[r & 3]) : "v"(v[r]), "v"(pe[r]));
          if (MODE == 17) v[r] = __builtin_amdgcn_exp2f(v[r]);
          if (MODE == 19) { // fp32 += one half of a packed fp16 pair (v_fma_mix_f32), alternating halves
            if (j & 1) asm volatile("v_fma_mix_f32 %0, %1, 1.0, %0 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "+v"(v[r]) : "v"(ppk[r & 3]));
            else asm volatile("v_fma_mix_f32 %0, %1, 1.0, %0 op_sel_hi:[1,0,0]" : "+v"(v[r]) : "v"(ppk[r & 3]));
          }
          if (MODE == 18) { // the softmax mix without the dot product: two exponentials, one packing conversion, two adds
            if (j % 5 < 2) v[r] = __builtin_amdgcn_exp2f(v[r]);
            else if (j % 5 == 2) asm volatile("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(ppk[r & 3]) : "v"(v[r]), "v"(pe[r]));
            else v[r] = v[r] + pe[r];
          }
          asm volatile("" : "+v"(v[r]));
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    } else if (MODE >= 9 && MODE <= 11) {
      // the attention kernels' mix behind every matrix instruction: two exponentials, one packing conversion, one
      // packed dot product, one integer add.  9: on registers of their own; 10: the exponentials read what the
      // matrix instructions of the previous trip wrote; 11: as 10, and the packed values are the B operand of the
      // matrix instructions of the next trip.
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float y0 = MODE == 9 ? v[2 * i] : acc[(i + 2) & 3][2 * i], y1 = MODE == 9 ? v[2 * i + 1] : acc[(i + 2) & 3][2 * i + 1];
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, MODE == 11 ? bw[0] : b, acc[i], 0, 0, 0);
        const float e0 = __builtin_amdgcn_exp2f(y0), e1 = __builtin_amdgcn_exp2f(y1);
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        const h2 one = {(_Float16)1.f, (_Float16)1.f};
        const h2 pk = {(_Float16)pe[2 * i], (_Float16)pe[2 * i + 1]}; // packs what the previous group computed
        rsum = __builtin_amdgcn_fdot2(ppk[i], one, rsum, false);       // sums what the previous group packed
        ppk[i] = pk;
        bw[1][2 * i] = pk[0];
        bw[1][2 * i + 1] = pk[1];
        pe[2 * i] = e0;
        pe[2 * i + 1] = e1;
        cnt += i;
        asm volatile("" : "+v"(pe[2 * i]), "+v"(pe[2 * i + 1]), "+v"(rsum), "+v"(cnt));
        __builtin_amdgcn_sched_barrier(0);
      }
      bw[0] = bw[1];
      if (MODE == 9) {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = pe[j] * 0.5f;
      }
    } else if (MODE == 7) { // as 2, but the exponentials read what the matrix instructions of the previous trip wrote
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const f32x16 src = acc[(i + 2) & 3];
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[i], 0, 0, 0);
#pragma unroll
        for (int j = 0; j < NEXP; ++j) v[(i * NEXP + j) & 7] = __builtin_amdgcn_exp2f(src[(i * NEXP + j) & 15] * 0.5f - 1.0f);
        __builtin_amdgcn_sched_barrier(0);
      }
    } else if (MODE == 8) { // as 2, but the B operand of every matrix instruction is packed from exponentials of the previous trip
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, bw[i & 1], acc[i], 0, 0, 0);
#pragma unroll
        for (int j = 0; j < NEXP; ++j) v[(i * NEXP + j) & 7] = __builtin_amdgcn_exp2f(v[(i * NEXP + j) & 7] * 0.5f - 1.0f);
        bw[(i + 1) & 1][(2 * i) & 7] = (_Float16)v[(2 * i) & 7];
        bw[(i + 1) & 1][(2 * i + 1) & 7] = (_Float16)v[(2 * i + 1) & 7];
        __builtin_amdgcn_sched_barrier(0);
      }
    } else if (MODE == 5 || MODE == 6) { // every matrix instruction takes its A operand from LDS, requested one trip ahead
      uint32_t ofs = (uint32_t)(w * 4096 + (tid & 63) * 16);
      asm volatile("" : "+v"(ofs)); // the compiler must not take the reads out of the loop
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (MODE == 5) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(la[i], b, acc[i], 0, 0, 0);
        else v[i] += (float)la[i][0]; // reads alone
        la[i] = *(const f16x8 *)(lds + ofs + i * 1024);
      }
    } else {
      if (do_mfma) {
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[i], 0, 0, 0);
      }
      if (do_exp) {
#pragma unroll
        for (int j = 0; j < 4 * NEXP; ++j) v[j & 7] = __builtin_amdgcn_exp2f(v[j & 7] * 0.5f - 1.0f);
      }
    }
  }
  const unsigned long long c1 = __builtin_readcyclecounter(), r1 = __builtin_amdgcn_s_memrealtime();
  float s = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[i][r];
#pragma unroll
  for (int j = 0; j < 8; ++j) s += v[j] + (float)bw[0][j] + (float)bw[1][j] + pe[j];
#pragma unroll
  for (int j = 0; j < 8; ++j) s += (float)iv[j];
  s += (float)(lv[0] + lv[1] + lv[2] + lv[3]);
  s += rsum + (float)cnt + (float)ppk[0][0] + (float)ppk[1][0] + (float)ppk[2][0] + (float)ppk[3][0];
  if ((tid & 63) == 0 && (w == 0 || w == 4)) {
    unsigned long long *o = out + ((size_t)blockIdx.x * 2 + (w >> 2)) * 3;
    o[0] = c1 - c0;
    o[1] = r1 - r0;
    o[2] = (unsigned long long)s;
  }
}

__global__ void probe_fill_kernel(_Float16 *p, size_t n, int random) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  uint32_t x = (uint32_t)i * 2654435761u + 12345u;
  x ^= x >> 15;
  x *= 2246822519u;
  x ^= x >> 13;
  p[i] = random ? (_Float16)(((int)(x & 0x7ff) - 1024) * (1.f / 1024.f)) : (_Float16)0.f;
}

template <int MODE, int NEXP> void launch_probe(int grid, int threads, unsigned long long *out, const _Float16 *src,
                                                int iters, hipStream_t s) {
  hipLaunchKernelGGL((pipe_probe_kernel<MODE, NEXP>), dim3(grid), dim3(threads), 32768, s, out, src, iters);
}

} // namespace
} // namespace fmha

// mode: 0 exponentials only; 1 matrix instructions only (four independent accumulators); 2 both in one
// stream (nexp exponentials per matrix instruction, nexp = 2, 4 or 6); 3 matrix instructions on ONE accumulator
// (a dependent chain); 4 waves 0-3 matrix only, waves 4-7 exponentials only (needs waves_per_simd = 2);
// 5 matrix instructions with the A operand read from LDS each time; 6 those LDS reads alone; 7 as 2, the
// exponentials reading registers that the matrix instructions of the previous trip wrote; 8 as 2, the B operand of
// the matrix instructions packed from the exponentials of the previous trip.
// 20-35: nexp instructions of one kind behind every matrix instruction, on registers of their own: 20 v_mad_u64_u32,
// 21 v_bitop3_b32, 22 v_mov_b32 with a DPP quad permutation, 23 v_pk_sub_i16, 24 v_perm_b32, 25 v_cndmask_b32,
// 26 v_mul_f32, 27 v_fma_f32, 28 v_pk_mul_f16, 29 v_max3_f32, 30 v_permlane32_swap_b32, 31 v_cvt_f32_f16,
// 32 v_dot2_f32_f16, 33 v_sub_f32, 34 v_and_b32, 35 v_pk_ashrrev_i16.  36: nexp v_xor_b32 behind every matrix
// instruction; 37: those v_xor_b32 alone (both also with nexp = 8, 16, 32).
// random_data: 0 all-zero operands, 1 pseudo-random in [-1, 1).  waves_per_simd: 1 or 2.
// Runs `launches` launches of `iters` loop trips (4 matrix instructions and/or 4 * nexp exponentials per trip and
// wave) on every compute unit, times the second half of them with events, and writes
//   result[0] = microseconds per launch, result[1] = mean core clock in MHz seen by the waves (cycle counter over
//   the 100 MHz counter), result[2] = matrix TFLOP/s (0 where no matrix work), result[3] = exponentials per
//   nanosecond over the chip.
// Allocates and frees its own buffers and synchronises the device.  Returns 0, or -1 on a bad argument / HIP error.
extern "C" int fmha_pipe_probe(int mode, int nexp, int random_data, int waves_per_simd, int iters, int launches,
                               double *result) {
  using namespace fmha;
  if (!result || mode < 0 || mode > 37 || (waves_per_simd != 1 && waves_per_simd != 2) || iters <= 0 || launches < 2)
    return -1;
  const bool wide = mode >= 36; // these two modes also take 8, 16 and 32 instructions per group
  if (nexp != 2 && nexp != 4 && nexp != 6 && nexp != 5 && !(wide && (nexp == 8 || nexp == 16 || nexp == 32))) return -1;
  if (mode == 4 && waves_per_simd != 2) return -1;
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    return -1;
  const int threads = 256 * waves_per_simd, grid = cus;
  const size_t nsrc = (size_t)grid * threads * 16;
  _Float16 *src = nullptr;
  unsigned long long *out = nullptr;
  if (hipMalloc(&src, nsrc * 2) != hipSuccess) return -1;
  if (hipMalloc(&out, (size_t)grid * 2 * 3 * 8) != hipSuccess) {
    (void)hipFree(src);
    return -1;
  }
  hipStream_t s = nullptr;
  hipLaunchKernelGGL(probe_fill_kernel, dim3((unsigned)((nsrc + 255) / 256)), dim3(256), 0, s, src, nsrc, random_data);
  (void)hipMemsetAsync(out, 0, (size_t)grid * 2 * 3 * 8, s);
  hipEvent_t e0, e1;
  (void)hipEventCreate(&e0);
  (void)hipEventCreate(&e1);
  auto go = [&]() {
#define FMHA_PROBE_CASE(M)                                                                  \
  case M:                                                                                   \
    if (nexp == 2) launch_probe<M, 2>(grid, threads, out, src, iters, s);                   \
    else if (nexp == 5) launch_probe<M, 5>(grid, threads, out, src, iters, s);              \
    else if (nexp == 4) launch_probe<M, 4>(grid, threads, out, src, iters, s);              \
    else launch_probe<M, 6>(grid, threads, out, src, iters, s);                             \
    break;
    switch (mode) {
      FMHA_PROBE_CASE(0)
      FMHA_PROBE_CASE(1)
      FMHA_PROBE_CASE(2)
      FMHA_PROBE_CASE(3)
      FMHA_PROBE_CASE(4)
      FMHA_PROBE_CASE(5)
      FMHA_PROBE_CASE(6)
      FMHA_PROBE_CASE(7)
      FMHA_PROBE_CASE(8)
      FMHA_PROBE_CASE(9)
      FMHA_PROBE_CASE(10)
      FMHA_PROBE_CASE(11)
      FMHA_PROBE_CASE(12)
      FMHA_PROBE_CASE(13)
      FMHA_PROBE_CASE(14)
      FMHA_PROBE_CASE(15)
      FMHA_PROBE_CASE(16)
      FMHA_PROBE_CASE(17)
      FMHA_PROBE_CASE(18)
      FMHA_PROBE_CASE(19)
      FMHA_PROBE_CASE(20)
      FMHA_PROBE_CASE(21)
      FMHA_PROBE_CASE(22)
      FMHA_PROBE_CASE(23)
      FMHA_PROBE_CASE(24)
      FMHA_PROBE_CASE(25)
      FMHA_PROBE_CASE(26)
      FMHA_PROBE_CASE(27)
      FMHA_PROBE_CASE(28)
      FMHA_PROBE_CASE(29)
      FMHA_PROBE_CASE(30)
      FMHA_PROBE_CASE(31)
      FMHA_PROBE_CASE(32)
      FMHA_PROBE_CASE(33)
      FMHA_PROBE_CASE(34)
      FMHA_PROBE_CASE(35)
#define FMHA_PROBE_WIDE(M)                                                                  \
  case M:                                                                                   \
    if (nexp == 2) launch_probe<M, 2>(grid, threads, out, src, iters, s);                   \
    else if (nexp == 4) launch_probe<M, 4>(grid, threads, out, src, iters, s);              \
    else if (nexp == 5) launch_probe<M, 5>(grid, threads, out, src, iters, s);              \
    else if (nexp == 6) launch_probe<M, 6>(grid, threads, out, src, iters, s);              \
    else if (nexp == 8) launch_probe<M, 8>(grid, threads, out, src, iters, s);              \
    else if (nexp == 16) launch_probe<M, 16>(grid, threads, out, src, iters, s);            \
    else launch_probe<M, 32>(grid, threads, out, src, iters, s);                            \
    break;
      FMHA_PROBE_WIDE(36)
      FMHA_PROBE_WIDE(37)
#undef FMHA_PROBE_WIDE
    }
#undef FMHA_PROBE_CASE
  };
  const int warm = launches / 2, timed = launches - warm;
  for (int i = 0; i < warm; ++i) go();
  (void)hipEventRecord(e0, s);
  for (int i = 0; i < timed; ++i) go();
  (void)hipEventRecord(e1, s);
  int rc = hipDeviceSynchronize() == hipSuccess && hipGetLastError() == hipSuccess ? 0 : -1;
  float ms = 0.f;
  if (rc == 0 && hipEventElapsedTime(&ms, e0, e1) != hipSuccess) rc = -1;
  static unsigned long long host[2048 * 6];
  const int nrec = grid * 2 <= 2048 * 2 ? grid * 2 : 2048 * 2;
  if (rc == 0 && hipMemcpy(host, out, (size_t)nrec * 3 * 8, hipMemcpyDeviceToHost) != hipSuccess) rc = -1;
  if (rc == 0) {
    double cyc = 0, tick = 0;
    for (int i = 0; i < nrec; ++i) {
      if (waves_per_simd == 1 && (i & 1)) continue;
      cyc += (double)host[3 * i];
      tick += (double)host[3 * i + 1];
    }
    const double us = (double)ms * 1e3 / timed;
    const bool has_mfma = mode != 0 && mode != 6 && mode != 37;
    const bool has_exp = mode == 0 || mode == 2 || mode == 4 || mode >= 7; // (modes 36, 37: the v_xor_b32 count)
    const double mfma_waves = (double)grid * (mode == 4 ? 4 : 4 * waves_per_simd);
    const double exp_waves = (double)grid * (mode == 4 ? 4 : 4 * waves_per_simd);
    result[0] = us;
    result[1] = tick > 0 ? cyc / tick * 100.0 : 0.0;
    result[2] = has_mfma ? mfma_waves * iters * 4.0 * 32768.0 / (us * 1e-6) * 1e-12 : 0.0;
    result[3] = has_exp ? exp_waves * iters * 4.0 * nexp * 64.0 / (us * 1e3) : 0.0;
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  (void)hipFree(src);
  (void)hipFree(out);
  return rc;
}
