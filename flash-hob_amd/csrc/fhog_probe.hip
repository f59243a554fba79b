// Measurement aid: the bf16 MFMA rate the device sustains, as a function of the operand data.
// The published dense peak assumes the nominal clock; under a power limit the clock the chip holds depends on how many
// operand bits toggle, so a loop of nothing but v_mfma_f32_32x32x16_bf16 runs measurably slower on random operands
// than on zeros. bench.py reports both figures next to the kernels' own throughput.
#include "fhog_common.h"

namespace fhog {
namespace {

__device__ __forceinline__ uint32_t xorshift(uint32_t& s) {
  s ^= s << 13;
  s ^= s >> 17;
  s ^= s << 5;
  return s;
}

// 8 waves per CU (two per SIMD), four independent accumulators per wave, 32 MFMAs per loop trip.
// data_mode 0: all operands zero; 1: random values in (-2, 2).
__global__ void __launch_bounds__(512) mfma_rate_kernel(float* out, int trips, int data_mode) {
  const int l = threadIdx.x;
  bf16x8_t a[4], b[4];
  uint32_t st = 1234567u * (blockIdx.x * 512 + l + 1);
  for (int i = 0; i < 4; i++)
    for (int e = 0; e < 8; e++) {
      const float va = data_mode ? ((int)(xorshift(st) & 0xffff) - 32768) / 16384.0f : 0.f;
      const float vb = data_mode ? ((int)(xorshift(st) & 0xffff) - 32768) / 16384.0f : 0.f;
      a[i][e] = (__bf16)va;
      b[i][e] = (__bf16)vb;
    }
  f32x16_t c[4] = {f32x16_t{0}, f32x16_t{0}, f32x16_t{0}, f32x16_t{0}};
  for (int it = 0; it < trips; it++) {
#pragma unroll
    for (int u = 0; u < 8; u++)
#pragma unroll
      for (int i = 0; i < 4; i++) c[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[i], c[i], 0, 0, 0);
    if ((it & 63) == 63)  // keep the accumulators bounded
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) c[i][r] *= 1e-3f;
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) s += c[i][r];
  out[blockIdx.x * 512 + l] = s;
}

}  // namespace

// Launches the loop on `blocks` workgroups of 512 threads; `out` needs blocks * 512 floats. FLOPs issued:
// blocks * 8 waves * trips * 32 MFMAs * 32768.
hipError_t launch_mfma_rate(float* out, int blocks, int trips, int data_mode, hipStream_t s) {
  hipLaunchKernelGGL(mfma_rate_kernel, dim3((unsigned)blocks), dim3(512), 0, s, out, trips, data_mode);
  return hipGetLastError();
}

}  // namespace fhog
