// fp32-MFMA kernels of the attention double-backward: every product and every
// intermediate in fp32 (v_mfma_f32_32x32x2_f32). This family serves fp32 inputs (bf16
// MFMA cannot reach 1e-4) and any shape the bf16 family does not take (ragged N, d=32).
// One wave64 per workgroup owns a 32-row tile; the opposite side streams through LDS in
// 32-row tiles. No atomics, nothing of shape (N_Q, N_K) leaves the chip.
//
// Math per tile pair (fhog/triton_bwdbwd.py:194-202, 229-243, 266-288, 485-507):
//   S = scale Q K^T, P = exp(S - L), dP = dO V^T, ddS = scale (ddQ K^T + Q ddK^T), E = dO ddV^T
//   dP' = E - dP dd - ddS d + dP ddS
//   dS = scale P (dP - d), dS' = scale P (dP' - b), ddP = P (ddS - dd)
#include "fhog_common.h"

namespace fhog {
namespace {

constexpr int TR = 32;   // rows per tile on both sides
constexpr int SB = 33;   // row stride (floats) of the S-shaped LDS buffers

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
__device__ inline void store1(T* p, float x) {
  *p = (T)x;
}

// rows row0..row0+31 of a (n, D) matrix -> LDS floats with row stride D+1; rows >= n read as 0.
template <typename T, int D>
__device__ inline void load_tile(float* dst, const T* src, int64_t ld, int row0, int n, int lane) {
  constexpr int C4 = D / 4;
  for (int v = lane; v < TR * C4; v += 64) {
    const int r = v / C4, c = (v % C4) * 4;
    f32x4_t x = {0.f, 0.f, 0.f, 0.f};
    if (row0 + r < n) x = load4<T>(src + (int64_t)(row0 + r) * ld + c);
    float* d = dst + r * (D + 1) + c;
    d[0] = x[0];
    d[1] = x[1];
    d[2] = x[2];
    d[3] = x[3];
  }
}

// acc[m][n] += sum_c A[m][c] * B[n][c]; A, B are 32 x D LDS tiles (row stride D+1).
// Result layout: acc[r] holds (m = 8*(r/4) + 4*(lane/32) + r%4, n = lane%32).
template <int D>
__device__ inline f32x16_t mma_nt(f32x16_t acc, const float* A, const float* B, int lane) {
  const float* ap = A + (lane & 31) * (D + 1) + (lane >> 5);
  const float* bp = B + (lane & 31) * (D + 1) + (lane >> 5);
#pragma unroll 8
  for (int c = 0; c < D; c += 2) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ap[c], bp[c], acc, 0, 0, 0);
  return acc;
}

struct TileVals {
  f32x16_t p, ds, ds2, ddp;
  float dd_part, b_part;
};

// Everything elementwise for one 32(query) x 32(key) tile pair. Lane owns query (lane%32);
// register r owns key 8*(r/4) + 4*(lane/32) + r%4.  LEVEL: 1 = dd only, 2 = + b, 3 = all.
template <int D, int LEVEL, bool CAUSAL>
__device__ inline TileVals tile_math(const float* Qs, const float* dOs, const float* ddQs, const float* Ks,
                                     const float* Vs, const float* ddKs, const float* ddVs, int lane, int q0,
                                     int k0, int n_q, int n_k, float scale, float L, float dsum, float dd, float b,
                                     int mask_off, int window) {
  TileVals t;
  const f32x16_t zero = {0};
  f32x16_t s = mma_nt<D>(zero, Ks, Qs, lane);
  f32x16_t dds = mma_nt<D>(zero, Ks, ddQs, lane);
  dds = mma_nt<D>(dds, ddKs, Qs, lane);
  f32x16_t dp = zero, e = zero;
  if (LEVEL >= 2) {
    dp = mma_nt<D>(zero, Vs, dOs, lane);
    e = mma_nt<D>(zero, ddVs, dOs, lane);
  }
  const int qi = q0 + (lane & 31);
  t.dd_part = 0.f;
  t.b_part = 0.f;
#pragma unroll
  for (int r = 0; r < 16; r++) {
    const int kj = k0 + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
    bool valid = (qi < n_q) && (kj < n_k);
    // band mask: key visible iff 0 <= (qi + mask_off) - kj < window (fhog/jax_refs/jax_impl.py:110-115)
    if (CAUSAL) valid = valid && (kj <= qi + mask_off) && (qi + mask_off - kj < window);
    const float p = valid ? expf(s[r] * scale - L) : 0.f;
    const float ddsv = dds[r] * scale;
    t.p[r] = p;
    t.dd_part += p * ddsv;
    if (LEVEL >= 2) {
      const float dpv = dp[r];
      const float dp2 = e[r] - dpv * dd - ddsv * dsum + dpv * ddsv;
      t.b_part += p * dp2;
      if (LEVEL >= 3) {
        t.ds[r] = scale * p * (dpv - dsum);
        t.ds2[r] = scale * p * (dp2 - b);
        t.ddp[r] = p * (ddsv - dd);
      }
    }
  }
  return t;
}

// S-shaped register tile -> LDS buffer laid out [query][key], row stride SB.
__device__ inline void spill_tile(float* buf, const f32x16_t& x, int lane) {
#pragma unroll
  for (int r = 0; r < 16; r++) buf[(lane & 31) * SB + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4)] = x[r];
}

// acc[cb][i][c] += sum_j W[i][j] * X[j][cb*32 + c]   (W: [query][key] buffer, X: 32 x D tile)
template <int D>
__device__ inline void mma_wx(f32x16_t* acc, const float* W, const float* X, int lane) {
  const float* wp = W + (lane & 31) * SB + (lane >> 5);
#pragma unroll
  for (int cb = 0; cb < D / 32; cb++) {
    const float* xp = X + (lane >> 5) * (D + 1) + cb * 32 + (lane & 31);
#pragma unroll 8
    for (int j = 0; j < TR; j += 2) acc[cb] = __builtin_amdgcn_mfma_f32_32x32x2f32(wp[j], xp[j * (D + 1)], acc[cb], 0, 0, 0);
  }
}

// acc[cb][j][c] += sum_i W[i][j] * X[i][cb*32 + c]   (contraction over the buffer's rows)
template <int D>
__device__ inline void mma_wtx(f32x16_t* acc, const float* W, const float* X, int lane) {
  const float* wp = W + (lane >> 5) * SB + (lane & 31);
#pragma unroll
  for (int cb = 0; cb < D / 32; cb++) {
    const float* xp = X + (lane >> 5) * (D + 1) + cb * 32 + (lane & 31);
#pragma unroll 8
    for (int i = 0; i < TR; i += 2) acc[cb] = __builtin_amdgcn_mfma_f32_32x32x2f32(wp[i * SB], xp[i * (D + 1)], acc[cb], 0, 0, 0);
  }
}

template <typename T, int D>
__device__ inline void store_acc(T* dst, int64_t ld, int row0, int n, const f32x16_t* acc, int lane) {
#pragma unroll
  for (int cb = 0; cb < D / 32; cb++) {
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int row = row0 + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
      if (row < n) store1<T>(dst + (int64_t)row * ld + cb * 32 + (lane & 31), acc[cb][r]);
    }
  }
}

template <int D>
struct SmemLayout {
  static constexpr int TILE = TR * (D + 1);
  static constexpr int BUF = TR * SB;
  static constexpr size_t BYTES = (size_t)(7 * TILE + 4 * BUF) * sizeof(float);
};

// Passes 1..3: one wave owns 32 query rows and sweeps all key tiles.
template <typename T, int D, int PASS, bool CAUSAL>
__global__ void __launch_bounds__(64) q_sweep_fp32(Params p) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  using SL = SmemLayout<D>;
  float* Qs = smem;
  float* dOs = Qs + SL::TILE;
  float* ddQs = dOs + SL::TILE;
  float* Ks = ddQs + SL::TILE;
  float* Vs = Ks + SL::TILE;
  float* ddKs = Vs + SL::TILE;
  float* ddVs = ddKs + SL::TILE;
  float* Wds = ddVs + SL::TILE;
  float* Wds2 = Wds + SL::BUF;
  float* Wddp = Wds2 + SL::BUF;
  float* Wp = Wddp + SL::BUF;

  const int lane = threadIdx.x;
  const int q0 = blockIdx.x * TR;
  const int bh = blockIdx.y;
  const int64_t qoff = (int64_t)bh * p.stride_qb, koff = (int64_t)bh * p.stride_kb;
  const T* Q = (const T*)p.q + qoff;
  const T* dO = (const T*)p.dO + qoff;
  const T* ddQ = (const T*)p.ddq + qoff;
  const T* K = (const T*)p.k + koff;
  const T* V = (const T*)p.v + koff;
  const T* ddK = (const T*)p.ddk + koff;
  const T* ddV = (const T*)p.ddv + koff;

  load_tile<T, D>(Qs, Q, p.stride_qn, q0, p.n_q, lane);
  load_tile<T, D>(ddQs, ddQ, p.stride_qn, q0, p.n_q, lane);
  if (PASS >= 2) load_tile<T, D>(dOs, dO, p.stride_qn, q0, p.n_q, lane);

  const int qi = q0 + (lane & 31);
  const bool qok = qi < p.n_q;
  const int64_t row = (int64_t)bh * p.n_q + qi;
  const float L = qok ? p.lse[row] : 0.f;
  const float dsum = (PASS >= 2 && qok) ? p.ws_d[row] : 0.f;
  const float dd = (PASS >= 2 && qok) ? p.ws_dd[row] : 0.f;
  const float b = (PASS >= 3 && qok) ? p.ws_b[row] : 0.f;

  float red = 0.f;
  f32x16_t acc_dq[D / 32], acc_ddo[D / 32];
#pragma unroll
  for (int cb = 0; cb < D / 32; cb++) {
    acc_dq[cb] = f32x16_t{0};
    acc_ddo[cb] = f32x16_t{0};
  }

  // key tiles that hold a visible key for some query of this tile
  int k_begin = 0, k_end = p.n_k;
  if (CAUSAL) {
    k_end = min(p.n_k, q0 + TR + p.mask_off);
    k_begin = max(0, q0 + p.mask_off - p.window + 1) / TR * TR;
  }
  for (int k0 = k_begin; k0 < k_end; k0 += TR) {
    __syncthreads();
    load_tile<T, D>(Ks, K, p.stride_kn, k0, p.n_k, lane);
    load_tile<T, D>(ddKs, ddK, p.stride_kn, k0, p.n_k, lane);
    if (PASS >= 2) {
      load_tile<T, D>(Vs, V, p.stride_kn, k0, p.n_k, lane);
      load_tile<T, D>(ddVs, ddV, p.stride_kn, k0, p.n_k, lane);
    }
    __syncthreads();
    TileVals t = tile_math<D, PASS, CAUSAL>(Qs, dOs, ddQs, Ks, Vs, ddKs, ddVs, lane, q0, k0, p.n_q, p.n_k, p.scale, L,
                                            dsum, dd, b, p.mask_off, p.window);
    if (PASS == 1) red += t.dd_part;
    if (PASS == 2) red += t.b_part;
    if (PASS == 3) {
      spill_tile(Wds, t.ds, lane);
      spill_tile(Wds2, t.ds2, lane);
      spill_tile(Wddp, t.ddp, lane);
      spill_tile(Wp, t.p, lane);
      __syncthreads();
      mma_wx<D>(acc_dq, Wds, ddKs, lane);
      mma_wx<D>(acc_dq, Wds2, Ks, lane);
      mma_wx<D>(acc_ddo, Wddp, Vs, lane);
      mma_wx<D>(acc_ddo, Wp, ddVs, lane);
    }
  }

  if (PASS == 1 || PASS == 2) {
    red += __shfl_xor(red, 32);
    if (lane < 32 && qok) (PASS == 1 ? p.ws_dd : p.ws_b)[row] = red;
  } else {
    store_acc<T, D>((T*)p.dq2 + qoff, p.stride_qn, q0, p.n_q, acc_dq, lane);
    store_acc<T, D>((T*)p.ddo + qoff, p.stride_qn, q0, p.n_q, acc_ddo, lane);
  }
}

// Pass 4: one wave owns 32 key rows and sweeps all query tiles.
template <typename T, int D, bool CAUSAL>
__global__ void __launch_bounds__(64) k_sweep_fp32(Params p) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  using SL = SmemLayout<D>;
  float* Qs = smem;
  float* dOs = Qs + SL::TILE;
  float* ddQs = dOs + SL::TILE;
  float* Ks = ddQs + SL::TILE;
  float* Vs = Ks + SL::TILE;
  float* ddKs = Vs + SL::TILE;
  float* ddVs = ddKs + SL::TILE;
  float* Wds = ddVs + SL::TILE;
  float* Wds2 = Wds + SL::BUF;
  float* Wddp = Wds2 + SL::BUF;

  const int lane = threadIdx.x;
  const int k0 = blockIdx.x * TR;
  const int bh = blockIdx.y;
  const int64_t qoff = (int64_t)bh * p.stride_qb, koff = (int64_t)bh * p.stride_kb;
  const T* Q = (const T*)p.q + qoff;
  const T* dO = (const T*)p.dO + qoff;
  const T* ddQ = (const T*)p.ddq + qoff;
  const T* K = (const T*)p.k + koff;
  const T* V = (const T*)p.v + koff;
  const T* ddK = (const T*)p.ddk + koff;
  const T* ddV = (const T*)p.ddv + koff;

  load_tile<T, D>(Ks, K, p.stride_kn, k0, p.n_k, lane);
  load_tile<T, D>(Vs, V, p.stride_kn, k0, p.n_k, lane);
  load_tile<T, D>(ddKs, ddK, p.stride_kn, k0, p.n_k, lane);
  load_tile<T, D>(ddVs, ddV, p.stride_kn, k0, p.n_k, lane);

  f32x16_t acc_dk[D / 32], acc_dv[D / 32];
#pragma unroll
  for (int cb = 0; cb < D / 32; cb++) {
    acc_dk[cb] = f32x16_t{0};
    acc_dv[cb] = f32x16_t{0};
  }

  // query tiles that hold a query seeing some key of this tile: k - mask_off <= i < k - mask_off + window
  int q_begin = 0, q_end = p.n_q;
  if (CAUSAL) {
    q_begin = max(0, k0 - p.mask_off) / TR * TR;
    q_end = (int)min((int64_t)p.n_q, (int64_t)k0 + TR - 1 - p.mask_off + p.window);
  }
  for (int q0 = q_begin; q0 < q_end; q0 += TR) {
    __syncthreads();
    load_tile<T, D>(Qs, Q, p.stride_qn, q0, p.n_q, lane);
    load_tile<T, D>(dOs, dO, p.stride_qn, q0, p.n_q, lane);
    load_tile<T, D>(ddQs, ddQ, p.stride_qn, q0, p.n_q, lane);
    const int qi = q0 + (lane & 31);
    const bool qok = qi < p.n_q;
    const int64_t row = (int64_t)bh * p.n_q + qi;
    const float L = qok ? p.lse[row] : 0.f;
    const float dsum = qok ? p.ws_d[row] : 0.f;
    const float dd = qok ? p.ws_dd[row] : 0.f;
    const float b = qok ? p.ws_b[row] : 0.f;
    __syncthreads();
    TileVals t = tile_math<D, 3, CAUSAL>(Qs, dOs, ddQs, Ks, Vs, ddKs, ddVs, lane, q0, k0, p.n_q, p.n_k, p.scale, L, dsum,
                                         dd, b, p.mask_off, p.window);
    spill_tile(Wds, t.ds, lane);
    spill_tile(Wds2, t.ds2, lane);
    spill_tile(Wddp, t.ddp, lane);
    __syncthreads();
    mma_wtx<D>(acc_dk, Wds, ddQs, lane);
    mma_wtx<D>(acc_dk, Wds2, Qs, lane);
    mma_wtx<D>(acc_dv, Wddp, dOs, lane);
  }
  store_acc<T, D>((T*)p.dk2 + koff, p.stride_kn, k0, p.n_k, acc_dk, lane);
  store_acc<T, D>((T*)p.dv2 + koff, p.stride_kn, k0, p.n_k, acc_dv, lane);
}

// Pass 0: d_i = sum_c O_ic dO_ic  (fhog/triton_bwdbwd.py:580), fp32 result. 16 lanes per row.
template <typename T, int D>
__global__ void __launch_bounds__(256) rowdot_kernel(Params p) {
  const int64_t rows = (int64_t)p.batch * p.n_q;
  const int64_t r = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  const int sub = threadIdx.x & 15;
  float acc = 0.f;
  if (r < rows) {
    const int64_t bh = r / p.n_q, i = r % p.n_q;
    const T* o = (const T*)p.o + bh * p.stride_qb + i * p.stride_qn;
    const T* g = (const T*)p.dO + bh * p.stride_qb + i * p.stride_qn;
#pragma unroll
    for (int c = sub * 4; c < D; c += 64) {
      f32x4_t a = load4<T>(o + c), b = load4<T>(g + c);
      acc += a[0] * b[0] + a[1] * b[1] + a[2] * b[2] + a[3] * b[3];
    }
  }
  acc += __shfl_xor(acc, 8);
  acc += __shfl_xor(acc, 4);
  acc += __shfl_xor(acc, 2);
  acc += __shfl_xor(acc, 1);
  if (r < rows && sub == 0) p.ws_d[r] = acc;
}

template <typename T, int D>
hipError_t launch_pass_td(const Params& p, int pass, hipStream_t s) {
  const size_t smem = SmemLayout<D>::BYTES;
  const dim3 block(64);
  const dim3 gq((p.n_q + TR - 1) / TR, p.batch), gk((p.n_k + TR - 1) / TR, p.batch);
#define FHOG_LAUNCH(kern, grid)                                                                            \
  do {                                                                                                     \
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem); \
    if (e != hipSuccess) return e;                                                                         \
    hipLaunchKernelGGL(kern, grid, block, smem, s, p);                                                     \
  } while (0)
  if (p.causal) {
    switch (pass) {
      case FHOG_PASS_DD: FHOG_LAUNCH((q_sweep_fp32<T, D, 1, true>), gq); break;
      case FHOG_PASS_B: FHOG_LAUNCH((q_sweep_fp32<T, D, 2, true>), gq); break;
      case FHOG_PASS_DQ_DDO: FHOG_LAUNCH((q_sweep_fp32<T, D, 3, true>), gq); break;
      case FHOG_PASS_DK_DV: FHOG_LAUNCH((k_sweep_fp32<T, D, true>), gk); break;
      default: return hipErrorInvalidValue;
    }
  } else {
    switch (pass) {
      case FHOG_PASS_DD: FHOG_LAUNCH((q_sweep_fp32<T, D, 1, false>), gq); break;
      case FHOG_PASS_B: FHOG_LAUNCH((q_sweep_fp32<T, D, 2, false>), gq); break;
      case FHOG_PASS_DQ_DDO: FHOG_LAUNCH((q_sweep_fp32<T, D, 3, false>), gq); break;
      case FHOG_PASS_DK_DV: FHOG_LAUNCH((k_sweep_fp32<T, D, false>), gk); break;
      default: return hipErrorInvalidValue;
    }
  }
#undef FHOG_LAUNCH
  return hipGetLastError();
}

template <typename T>
hipError_t launch_pass_t(const Params& p, int pass, hipStream_t s) {
  switch (p.d) {
    case 32: return launch_pass_td<T, 32>(p, pass, s);
    case 64: return launch_pass_td<T, 64>(p, pass, s);
    case 128: return launch_pass_td<T, 128>(p, pass, s);
    default: return hipErrorInvalidValue;
  }
}

template <typename T>
hipError_t launch_rowdot_t(const Params& p, hipStream_t s) {
  const int64_t rows = (int64_t)p.batch * p.n_q;
  const dim3 grid((unsigned)((rows + 15) / 16)), block(256);
  switch (p.d) {
    case 32: hipLaunchKernelGGL((rowdot_kernel<T, 32>), grid, block, 0, s, p); break;
    case 64: hipLaunchKernelGGL((rowdot_kernel<T, 64>), grid, block, 0, s, p); break;
    case 128: hipLaunchKernelGGL((rowdot_kernel<T, 128>), grid, block, 0, s, p); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

}  // namespace

hipError_t launch_rowdot(const Params& p, int dtype, hipStream_t s) {
  if (dtype == FHOG_DTYPE_FP32) return launch_rowdot_t<float>(p, s);
  return dtype == FHOG_DTYPE_FP16 ? launch_rowdot_t<_Float16>(p, s) : launch_rowdot_t<__bf16>(p, s);
}

hipError_t launch_fp32_pass(const Params& p, int dtype, int pass, hipStream_t s) {
  if (dtype == FHOG_DTYPE_FP32) return launch_pass_t<float>(p, pass, s);
  return dtype == FHOG_DTYPE_FP16 ? launch_pass_t<_Float16>(p, pass, s) : launch_pass_t<__bf16>(p, pass, s);
}

}  // namespace fhog
