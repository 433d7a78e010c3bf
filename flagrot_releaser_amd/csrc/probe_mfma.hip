// Measurement aid, not part of the drop-in boundary: what the matrix pipe of this GPU gives a kernel that does nothing
// but v_mfma_f32_32x32x16_f16 (the instruction of the multi-query prefill kernels), back to back on registers, and the
// same with one operand of every instruction read from LDS (a 1 KB tile row per wavefront and instruction, as in the
// prefill kernels' block step).  bench.py times both beside the prefill kernel: the dense-fp16 ceiling that is
// actually reachable on the box, next to the nominal 2.5 PFLOP/s.
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdio>

#include "../../include/flagrot_probe.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
constexpr int PROBE_WAVES = 8;      // wavefronts per workgroup: two per SIMD, as the prefill kernel runs
constexpr int PROBE_CHAINS = 4;     // independent accumulators per wavefront

// MODE 0: both operands stay in registers.  MODE 1: the A operand of every instruction comes from LDS.
template <int MODE>
__global__ void __launch_bounds__(64 * PROBE_WAVES) k_probe_mfma(int iters, uint32_t* __restrict__ sink) {
  __shared__ uint4 tile[PROBE_WAVES][PROBE_CHAINS * 64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // small exact values: sums stay finite whatever the iteration count
  const _Float16 av = static_cast<_Float16>(0.0009765625f * static_cast<float>((lane & 7) - 3));
  const _Float16 bv = static_cast<_Float16>(0.0009765625f * static_cast<float>((lane & 3) - 1));
  half8 a{av, av, av, av, av, av, av, av}, b{bv, bv, bv, bv, bv, bv, bv, bv};
  for (int k = 0; k < PROBE_CHAINS; ++k) tile[wave][k * 64 + lane] = __builtin_bit_cast(uint4, a);
  __syncthreads();
  f32x16 acc[PROBE_CHAINS];
#pragma unroll
  for (int k = 0; k < PROBE_CHAINS; ++k)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[k][i] = 0.f;
  const uint4* row = &tile[wave][lane];
  if constexpr (MODE == 0) {
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int k = 0; k < PROBE_CHAINS; ++k) acc[k] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[k], 0, 0, 0);
    }
  } else {
    // software-pipelined as a real kernel would be: the operands of step it + 1 are requested before the products of
    // step it are issued, so that what is measured is the LDS feed and not the latency of one read
    half8 x[PROBE_CHAINS], y[PROBE_CHAINS];
#pragma unroll
    for (int k = 0; k < PROBE_CHAINS; ++k) x[k] = __builtin_bit_cast(half8, row[k * 64]);
    for (int it = 0; it < iters; it += 2) {
      asm volatile("" : "+v"(row));      // the reads stay inside the loop
#pragma unroll
      for (int k = 0; k < PROBE_CHAINS; ++k) y[k] = __builtin_bit_cast(half8, row[k * 64]);
#pragma unroll
      for (int k = 0; k < PROBE_CHAINS; ++k) acc[k] = __builtin_amdgcn_mfma_f32_32x32x16_f16(x[k], b, acc[k], 0, 0, 0);
      asm volatile("" : "+v"(row));
#pragma unroll
      for (int k = 0; k < PROBE_CHAINS; ++k) x[k] = __builtin_bit_cast(half8, row[k * 64]);
#pragma unroll
      for (int k = 0; k < PROBE_CHAINS; ++k) acc[k] = __builtin_amdgcn_mfma_f32_32x32x16_f16(y[k], b, acc[k], 0, 0, 0);
    }
  }
  float s = 0.f;
#pragma unroll
  for (int k = 0; k < PROBE_CHAINS; ++k)
#pragma unroll
    for (int i = 0; i < 16; ++i) s += acc[k][i];
  if (s == 12345.678f) sink[0] = __float_as_uint(s);           // keeps the products alive; practically never taken
}

}  // namespace

extern "C" {

long long fr_probe_mfma_flops(int iters, int workgroups) {
  iters += iters & 1;
  return 2LL * 32 * 32 * 16 * PROBE_CHAINS * PROBE_WAVES * static_cast<long long>(iters) * workgroups;
}

int fr_probe_mfma(int mode, int iters, int workgroups, uint32_t* sink, void* stream) {
  if (iters <= 0 || workgroups <= 0) return 0;
  iters += iters & 1;      // mode 1 works through the steps in pairs
  if (mode != 0 && mode != 1) return -2;
  if (mode == 0) hipLaunchKernelGGL(k_probe_mfma<0>, dim3(workgroups), dim3(64 * PROBE_WAVES), 0, static_cast<hipStream_t>(stream), iters, sink);
  else hipLaunchKernelGGL(k_probe_mfma<1>, dim3(workgroups), dim3(64 * PROBE_WAVES), 0, static_cast<hipStream_t>(stream), iters, sink);
  return hipPeekAtLastError() == hipSuccess ? 0 : -1;
}

}  // extern "C"
