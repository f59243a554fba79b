// Measurement aid: the bf16 MFMA rate the device sustains, as a function of the operand data and of what else the
// instruction stream carries.
// The published dense peak assumes the nominal clock; under a power limit the clock the chip holds depends on how many
// operand bits toggle, so a loop of nothing but v_mfma_f32_32x32x16_bf16 runs measurably slower on random operands
// than on zeros - and slower again when the same loop also reads its A operands from LDS or carries VALU instructions,
// although the matrix pipe never waits for either. bench.py reports these figures next to the kernels' own throughput:
// they are the practical ceilings for a kernel with that instruction mix.
#include "fhog_common.h"

namespace fhog {
namespace {

__device__ __forceinline__ uint32_t xorshift(uint32_t& s) {
  s ^= s << 13;
  s ^= s >> 17;
  s ^= s << 5;
  return s;
}

// 8 waves per CU (two per SIMD; launched with 256 threads: four waves, one per SIMD, and every instruction of a wave then
// has only that wave's own MFMAs to hide behind), four independent accumulators per wave, 32 MFMAs per loop trip.
// MODE 0: all operands zero; 1: random values in (-2, 2), operands in registers;
//      2: as 1, every MFMA takes its A operand from LDS (one ds_read_b128 per MFMA, fetched one group of four ahead);
//      3: as 2 with every operand read feeding two MFMAs (the ratio of a wave that keeps 64 stationary rows);
//      4: as 1 plus three independent v_fma_f32 per MFMA;
//      5: 2 and 4 together (one LDS read and three VALU instructions per MFMA: the mix of the recomputation sweeps).
template <int MODE, int WAVES>
__global__ void __launch_bounds__(64 * WAVES) mfma_rate_kernel(float* out, int trips) {
  constexpr bool RANDOM = MODE != 0, LDS = MODE == 2 || MODE == 3 || MODE == 5, VALU = MODE == 4 || MODE == 5;
  constexpr int LDS_BYTES = 32 * 1024;
  __shared__ __attribute__((aligned(16))) char pool[LDS ? LDS_BYTES : 16];
  const int l = threadIdx.x, lane = l & 63;
  bf16x8_t a[4], b[4];
  uint32_t st = 1234567u * (blockIdx.x * 512 + l + 1);
  for (int i = 0; i < 4; i++)
    for (int e = 0; e < 8; e++) {
      const float va = RANDOM ? ((int)(xorshift(st) & 0xffff) - 32768) / 16384.0f : 0.f;
      const float vb = RANDOM ? ((int)(xorshift(st) & 0xffff) - 32768) / 16384.0f : 0.f;
      a[i][e] = (__bf16)va;
      b[i][e] = (__bf16)vb;
    }
  if (LDS) {   // 32 KiB of random bf16 values in (-2, 2): 32 tiles of 1 KiB, one per operand read
    for (int o = l * 16; o < LDS_BYTES; o += 64 * WAVES * 16) {
      bf16x8_t v;
      for (int e = 0; e < 8; e++) v[e] = (__bf16)(((int)(xorshift(st) & 0xffff) - 32768) / 16384.0f);
      *reinterpret_cast<bf16x8_t*>(pool + o) = v;
    }
    __syncthreads();
  }
  f32x16_t c[4] = {f32x16_t{0}, f32x16_t{0}, f32x16_t{0}, f32x16_t{0}};
  float x[12];   // VALU side work: independent of the MFMAs, kept alive through `out`
  for (int k = 0; k < 12; k++) x[k] = 1.0f + 0.001f * (lane + k);
  const float fa = 0.999f, fb = 0.001f;
  const char* mine = pool + lane * 16;
  constexpr int PER = MODE == 3 ? 2 : 4;   // operand reads per group of four MFMAs
  for (int it = 0; it < trips; it++) {
    bf16x8_t buf[2][4];
    if (LDS) {
#pragma unroll
      for (int i = 0; i < PER; i++) buf[0][i] = *reinterpret_cast<const bf16x8_t*>(mine + ((it * 8 * PER + i) & 31) * 1024);
    }
#pragma unroll
    for (int u = 0; u < 8; u++) {
      if (LDS && u + 1 < 8) {
#pragma unroll
        for (int i = 0; i < PER; i++)
          buf[(u + 1) & 1][i] = *reinterpret_cast<const bf16x8_t*>(mine + ((it * 8 * PER + (u + 1) * PER + i) & 31) * 1024);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const bf16x8_t av = LDS ? buf[u & 1][MODE == 3 ? i / 2 : i] : a[i];
        c[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, b[i], c[i], 0, 0, 0);
        if (VALU) {   // from inline asm, so that the instructions stay where they are, behind their MFMA
#pragma unroll
          for (int k = 0; k < 3; k++) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x[3 * i + k]) : "v"(fa), "v"(fb));
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
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
  for (int k = 0; k < 12; k++) s += 1e-30f * x[k];
  out[blockIdx.x * 512 + l] = s;
}

}  // namespace

// Launches the loop on `blocks` workgroups of `waves` (4 or 8) waves; `out` needs blocks * 512 floats. FLOPs issued:
// blocks * waves * trips * 32 MFMAs * 32768.
hipError_t launch_mfma_rate(float* out, int blocks, int trips, int data_mode, int waves, hipStream_t s) {
  const dim3 grid((unsigned)blocks), block(64u * (unsigned)waves);
#define FHOG_PROBE(M)                                                                                  \
  case M:                                                                                              \
    if (waves == 8) hipLaunchKernelGGL((mfma_rate_kernel<M, 8>), grid, block, 0, s, out, trips);       \
    else hipLaunchKernelGGL((mfma_rate_kernel<M, 4>), grid, block, 0, s, out, trips);                  \
    break;
  if (waves != 4 && waves != 8) return hipErrorInvalidValue;
  switch (data_mode) {
    FHOG_PROBE(0) FHOG_PROBE(1) FHOG_PROBE(2) FHOG_PROBE(3) FHOG_PROBE(4) FHOG_PROBE(5)
    default: return hipErrorInvalidValue;
  }
#undef FHOG_PROBE
  return hipGetLastError();
}

}  // namespace fhog
