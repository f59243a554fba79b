// Device helpers shared by the fp32-MFMA kernels (v_mfma_f32_32x32x2_f32): element loads and stores for fp32, bf16 and
// fp16 tensors, the padded fp32 LDS tile, first- and second-level products on 32 x 32 blocks.
#pragma once
#include "fhog_common.h"

namespace fhog {
namespace f32k {

constexpr int TR = 32;   // rows per tile on both sides

template <typename T>
__device__ inline f32x4_t load4(const T* p);
template <>
__device__ inline f32x4_t load4<float>(const float* p) {
  return *reinterpret_cast<const f32x4_t*>(p);
}
template <>
__device__ inline f32x4_t load4<__bf16>(const __bf16* p) {
  bf16x4_t v = *reinterpret_cast<const bf16x4_t*>(p);
  f32x4_t r = {(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
  return r;
}
template <>
__device__ inline f32x4_t load4<_Float16>(const _Float16* p) {
  typedef __attribute__((__vector_size__(4 * sizeof(_Float16)))) _Float16 f16x4_t;
  f16x4_t v = *reinterpret_cast<const f16x4_t*>(p);
  f32x4_t r = {(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
  return r;
}
template <typename T>
__device__ inline void store4(T* p, f32x4_t x);
template <>
__device__ inline void store4<float>(float* p, f32x4_t x) {
  *reinterpret_cast<f32x4_t*>(p) = x;
}
template <>
__device__ inline void store4<__bf16>(__bf16* p, f32x4_t x) {
  bf16x4_t v = {(__bf16)x[0], (__bf16)x[1], (__bf16)x[2], (__bf16)x[3]};
  *reinterpret_cast<bf16x4_t*>(p) = v;
}
template <>
__device__ inline void store4<_Float16>(_Float16* p, f32x4_t x) {
  typedef __attribute__((__vector_size__(4 * sizeof(_Float16)))) _Float16 f16x4_t;
  f16x4_t v = {(_Float16)x[0], (_Float16)x[1], (_Float16)x[2], (_Float16)x[3]};
  *reinterpret_cast<f16x4_t*>(p) = v;
}

// LDS tiles: 32 rows of D floats, row stride D + 4 (rows stay 16-byte aligned; 16 consecutive rows
// at the same column fall into 16 different 16-byte bank groups).
template <int D>
struct Tile {
  static constexpr int LD = D + 4;
  static constexpr int FLOATS = TR * LD;
};

// rows row0..row0+31 of two (n, D) matrices -> two LDS tiles as fp32, by the 256 threads of the workgroup; rows >= n
// read as 0. All loads are issued before the first LDS write, so the step pays one memory latency, not one per chunk.
template <typename T, int D>
__device__ inline void load_tile_pair(float* dst0, float* dst1, const T* src0, const T* src1, int64_t ld, int row0, int n, int tid) {
  constexpr int C4 = D / 4, PER = TR * C4 / 256;
  f32x4_t x[2][PER];
#pragma unroll
  for (int c = 0; c < PER; c++) {
    const int v = tid + c * 256, r = v / C4, col = (v % C4) * 4;
    x[0][c] = x[1][c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    if (row0 + r < n) {
      x[0][c] = load4<T>(src0 + (int64_t)(row0 + r) * ld + col);
      x[1][c] = load4<T>(src1 + (int64_t)(row0 + r) * ld + col);
    }
  }
#pragma unroll
  for (int c = 0; c < PER; c++) {
    const int v = tid + c * 256, r = v / C4, col = (v % C4) * 4;
    *reinterpret_cast<f32x4_t*>(dst0 + r * Tile<D>::LD + col) = x[0][c];
    *reinterpret_cast<f32x4_t*>(dst1 + r * Tile<D>::LD + col) = x[1][c];
  }
}

// Operands of one stationary row for the first-level products. The MFMA contracts two columns per
// instruction (k = lane / 32); the columns are dealt so that each half-wave owns whole 16-byte chunks:
// instruction 4j + e contracts columns 8j + e (lanes 0-31) and 8j + 4 + e (lanes 32-63).
template <typename T, int D>
__device__ inline void load_resident(f32x4_t* dst, const T* src, int64_t ld, int row, int n, int h) {
#pragma unroll
  for (int j = 0; j < D / 8; j++) {
    f32x4_t x = {0.f, 0.f, 0.f, 0.f};
    if (row < n) x = load4<T>(src + (int64_t)row * ld + 8 * j + 4 * h);
    dst[j] = x;
  }
}

// acc[m][n] += sum_c A[m][c] * B[n][c]: A = streamed LDS tile (m = tile row), B = stationary row n = lane % 32.
// Result layout: acc[r] holds (m = 8*(r/4) + 4*(lane/32) + r%4, n = lane%32).
// The LDS operand of group j + 1 is fetched before the four MFMAs of group j and the scheduler is kept from
// hoisting more than that: one group in flight hides the LDS latency behind 256 matrix-pipe cycles, and the
// stationary operands need the registers.
template <int D>
__device__ inline f32x16_t mma_first(f32x16_t acc, const float* A, const f32x4_t* B, int lane) {
  const float* ap = A + (lane & 31) * Tile<D>::LD + 4 * (lane >> 5);
  f32x4_t a = *reinterpret_cast<const f32x4_t*>(ap);
#pragma unroll
  for (int j = 0; j < D / 8; j++) {
    f32x4_t nxt = a;
    if (j + 1 < D / 8) nxt = *reinterpret_cast<const f32x4_t*>(ap + 8 * (j + 1));
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int e = 0; e < 4; e++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], B[j][e], acc, 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    a = nxt;
  }
  return acc;
}
// same with the stationary operand in an LDS tile of its own (row = lane % 32)
template <int D>
__device__ inline f32x16_t mma_first_lds(f32x16_t acc, const float* A, const float* B, int lane) {
  const float* ap = A + (lane & 31) * Tile<D>::LD + 4 * (lane >> 5);
  const float* bp = B + (lane & 31) * Tile<D>::LD + 4 * (lane >> 5);
  f32x4_t a = *reinterpret_cast<const f32x4_t*>(ap), b = *reinterpret_cast<const f32x4_t*>(bp);
#pragma unroll
  for (int j = 0; j < D / 8; j++) {
    f32x4_t na = a, nb = b;
    if (j + 1 < D / 8) {
      na = *reinterpret_cast<const f32x4_t*>(ap + 8 * (j + 1));
      nb = *reinterpret_cast<const f32x4_t*>(bp + 8 * (j + 1));
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int e = 0; e < 4; e++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], b[e], acc, 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    a = na;
    b = nb;
  }
  return acc;
}

// acc[cb][c][n] += sum_m X[m][cb*32 + c] * W[m][n], W being a first-level accumulator (m over its registers):
// instruction 4g + e contracts the streamed rows 8g + e (lanes 0-31) and 8g + 4 + e (lanes 32-63), which is
// where register 4g + e of W holds them.
template <int D>
__device__ inline void mma_second(f32x16_t* acc, const f32x16_t& w, const float* X, int lane) {
  const float* xp = X + 4 * (lane >> 5) * Tile<D>::LD + (lane & 31);
  constexpr int NG = 4 * (D / 32);   // groups of four instructions: (cb, g)
  float a[4];
#pragma unroll
  for (int e = 0; e < 4; e++) a[e] = xp[e * Tile<D>::LD];
#pragma unroll
  for (int i = 0; i < NG; i++) {
    const int cb = i / 4, g = i % 4;
    float nxt[4];
#pragma unroll
    for (int e = 0; e < 4; e++)
      nxt[e] = (i + 1 < NG) ? xp[(8 * ((i + 1) % 4) + e) * Tile<D>::LD + ((i + 1) / 4) * 32] : 0.f;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int e = 0; e < 4; e++) acc[cb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], w[4 * g + e], acc[cb], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int e = 0; e < 4; e++) a[e] = nxt[e];
  }
}

// acc[cb][r] holds column cb*32 + 8*(r/4) + 4*(lane/32) + r%4 of stationary row lane % 32
template <typename T, int D>
__device__ inline void store_acc(T* dst, int64_t ld, int row, int n, const f32x16_t* acc, int h) {
  if (row >= n) return;
#pragma unroll
  for (int cb = 0; cb < D / 32; cb++)
#pragma unroll
    for (int g = 0; g < 4; g++) {
      const f32x4_t x = {acc[cb][4 * g], acc[cb][4 * g + 1], acc[cb][4 * g + 2], acc[cb][4 * g + 3]};
      store4<T>(dst + (int64_t)row * ld + cb * 32 + 8 * g + 4 * h, x);
    }
}

}  // namespace f32k
}  // namespace fhog
