// First-order attention on the fp32-MFMA skeleton (v_mfma_f32_32x32x2_f32, every product and intermediate in fp32):
// forward (O and the fp32 log-sum-exp L, online soft-max; fhog/triton_flash.py:12-133, 252-258) and backward
// (dQ; dK and dV; the arithmetic of fhog/triton_flash.py:201-220 without the (batch, N_Q, N_K) tensors and without
// atomics). Serves fp32 tensors and d = 32, the shapes the 16-bit kernels of fhog_attn.hip do not take; bf16 and fp16
// tensors of any supported head dim go through as well.
//
// Same shape as the double-backward kernels of fhog_fp32.hip: a workgroup of 4 wave64 owns 32 stationary rows per
// wave (queries; keys in the K-tiled backward) with their operands in registers, the other side streams through LDS in
// 32-row fp32 tiles. First-level products have the streamed rows as M and the stationary rows as N: a lane owns ONE
// stationary row, its accumulator registers run over the streamed rows, and such an accumulator is as it stands the B
// operand of the second-level products. In the forward the running maximum, the running sum and the rescaling factor
// of a query are therefore per-lane scalars.
#include "fhog_bf16_util.h"   // XCD-aware grid decode
#include "fhog_fp32_util.h"

namespace fhog {
using namespace f32k;
namespace {

constexpr int MODE_FWD = 0, MODE_BWD_Q = 1, MODE_BWD_K = 2;

template <typename T, int D, int MODE, bool MASKED>
__global__ void __launch_bounds__(256) attn_fp32(AttnParams p) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  constexpr bool KSIDE = MODE == MODE_BWD_K;                 // the stationary rows are keys
  constexpr int NR = MODE == MODE_FWD ? 1 : 2;               // stationary tensors: Q | Q, dO | K, V
  constexpr int J = D / 8, CB = D / 32, TF = Tile<D>::FLOATS, nw = 4;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, h = lane >> 5;
  const int n_sta = KSIDE ? p.n_k : p.n_q, n_str = KSIDE ? p.n_q : p.n_k;
  // with a mask the work of a tile grows (or falls) with its index: a workgroup takes tiles u and n_tiles - 1 - u in turn
  const int n_tiles = (n_sta + TR * nw - 1) / (TR * nw);
  int bh, unit;
  if (!bf16k::decode_block(MASKED ? (n_tiles + 1) / 2 : n_tiles, p.batch, false, false, bh, unit)) return;
  const int64_t qoff = (int64_t)bh * p.stride_qb, koff = (int64_t)bh * p.stride_kb;
  const int64_t sta_ld = KSIDE ? p.stride_kn : p.stride_qn, str_ld = KSIDE ? p.stride_qn : p.stride_kn;
  const T* sta[2] = {(const T*)(KSIDE ? p.k : p.q) + (KSIDE ? koff : qoff), (const T*)(KSIDE ? p.v : p.dO) + (KSIDE ? koff : qoff)};
  const T* str[2] = {(const T*)(KSIDE ? p.q : p.k) + (KSIDE ? qoff : koff), (const T*)(KSIDE ? p.dO : p.v) + (KSIDE ? qoff : koff)};
  float* tiles = smem;            // two streamed tiles: K, V | Q, dO
  float* stat = tiles + 2 * TF;   // K-tiled backward: L and d of the 32 streamed queries
  const int64_t srow = (int64_t)bh * p.n_q;
  const float c_log2 = p.scale * kLog2e;

#pragma unroll 1
  for (int half = 0; half < (MASKED ? 2 : 1); half++) {
    const int tile = half ? n_tiles - 1 - unit : unit;
    if (half && tile == unit) break;   // odd number of tiles: the middle one stands alone
    const int r0 = tile * TR * nw, rw = r0 + TR * wave, ri = rw + n;
    const bool rok = ri < n_sta;

    f32x4_t res[NR][J];
#pragma unroll
    for (int x = 0; x < NR; x++) load_resident<T, D>(res[x], sta[x], sta_ld, ri, n_sta, h);
    float L = 0.f, dsum = 0.f;
    if (MODE == MODE_BWD_Q && rok) L = p.lse[srow + ri], dsum = p.ws_d[srow + ri];
    float m_run = -INFINITY, l_run = 0.f;   // forward: running maximum (base-2 units) and running sum of the lane's query
    f32x16_t acc0[CB], acc1[CB];            // O | dQ | dK, and dV
#pragma unroll
    for (int cb = 0; cb < CB; cb++) acc0[cb] = f32x16_t{0}, acc1[cb] = f32x16_t{0};

    // streamed tiles that hold a visible pair for some stationary row of this workgroup; key j is visible to
    // query i iff 0 <= i + mask_off - j < window (fhog/jax_refs/jax_impl.py:110-115)
    const int rows = TR * nw;
    int s_begin = 0, s_end = n_str;
    if (MASKED) {
      if (!KSIDE) {
        s_end = (int)min((int64_t)n_str, (int64_t)r0 + rows + p.mask_off);
        s_begin = (int)(max((int64_t)0, (int64_t)r0 + p.mask_off - p.window + 1) / TR * TR);
      } else {
        s_begin = max(0, r0 - p.mask_off) / TR * TR;
        s_end = (int)min((int64_t)n_str, (int64_t)r0 + rows - 1 - p.mask_off + p.window);
      }
    }

    for (int s0 = s_begin; s0 < s_end; s0 += TR) {
      __syncthreads();   // the previous tile is no longer read
      load_tile_pair<T, D>(tiles, tiles + TF, str[0], str[1], str_ld, s0, n_str, tid);
      if (KSIDE && tid < 2 * TR) {
        const int qi = s0 + (tid & 31);
        stat[tid] = qi < p.n_q ? (tid < TR ? p.lse : p.ws_d)[srow + qi] : 0.f;
      }
      __syncthreads();
      // every pair of this wave's rows with this tile hidden, or a wave without rows: nothing to add
      bool dead = rw >= n_sta;
      if (MASKED) {
        const int64_t q_lo = KSIDE ? s0 : rw, q_hi = (KSIDE ? s0 : rw) + TR - 1;   // queries of the block
        const int64_t k_lo = KSIDE ? rw : s0, k_hi = (KSIDE ? rw : s0) + TR - 1;   // keys of the block
        dead = dead || k_lo > q_hi + p.mask_off || q_lo + p.mask_off - k_hi >= p.window;
      }
      if (dead) continue;

      const f32x16_t zero = {0};
      f32x16_t sv = mma_first<D>(zero, tiles, res[0], lane);   // K Q^T | Q K^T: register r <-> streamed row m(r)
      bool valid[16];
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int m = 8 * (r / 4) + 4 * h + (r % 4);
        const int qi = KSIDE ? s0 + m : ri, kj = KSIDE ? ri : s0 + m;
        valid[r] = qi < p.n_q && kj < p.n_k;
        if (MASKED) valid[r] = valid[r] && (kj <= qi + p.mask_off) && (qi + p.mask_off - kj < p.window);
      }
      f32x16_t pv;
      if (MODE == MODE_FWD) {
        float tmax = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; r++) {
          sv[r] = valid[r] ? sv[r] * c_log2 : -INFINITY;
          tmax = fmaxf(tmax, sv[r]);
        }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32));   // the other half of the wave holds the other 16 keys of the row
        const float m_new = fmaxf(m_run, tmax);
        // a row that has seen no key yet (window starting in a later tile, or a row past the end) keeps its state
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);   // exp2(-inf) = 0 on the first visible tile
        float psum = 0.f;
#pragma unroll
        for (int r = 0; r < 16; r++) {
          pv[r] = __builtin_amdgcn_exp2f(sv[r] - m_use);
          psum += pv[r];
        }
        l_run = l_run * alpha + psum;
        m_run = m_new;
#pragma unroll
        for (int cb = 0; cb < CB; cb++)
#pragma unroll
          for (int r = 0; r < 16; r++) acc0[cb][r] *= alpha;
        mma_second<D>(acc0, pv, tiles + TF, lane);                 // O += P V
      } else {
        f32x16_t dp = mma_first<D>(zero, tiles + TF, res[1], lane);   // V dO^T | dO V^T
        f32x16_t ds;
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int m = 8 * (r / 4) + 4 * h + (r % 4);
          const float Lr = KSIDE ? stat[m] : L, dr = KSIDE ? stat[TR + m] : dsum;
          pv[r] = valid[r] ? __builtin_amdgcn_exp2f((sv[r] * p.scale - Lr) * kLog2e) : 0.f;
          ds[r] = p.scale * pv[r] * (dp[r] - dr);
        }
        if (KSIDE) {
          mma_second<D>(acc1, pv, tiles + TF, lane);               // dV += P^T dO
          mma_second<D>(acc0, ds, tiles, lane);                    // dK += dS^T Q
        } else {
          mma_second<D>(acc0, ds, tiles, lane);                    // dQ += dS K
        }
      }
    }

    if (MODE == MODE_FWD) {
      l_run += __shfl_xor(l_run, 32);
      const float inv = 1.f / l_run;
#pragma unroll
      for (int cb = 0; cb < CB; cb++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc0[cb][r] *= inv;
      store_acc<T, D>((T*)p.o + qoff, p.stride_qn, ri, p.n_q, acc0, h);
      if (h == 0 && rok) p.lse[srow + ri] = (m_run + __builtin_amdgcn_logf(l_run)) * 0.6931471805599453f;   // v_log_f32 is log2
    } else if (MODE == MODE_BWD_Q) {
      store_acc<T, D>((T*)p.dq + qoff, p.stride_qn, ri, p.n_q, acc0, h);
    } else {
      store_acc<T, D>((T*)p.dk + koff, p.stride_kn, ri, p.n_k, acc0, h);
      store_acc<T, D>((T*)p.dv + koff, p.stride_kn, ri, p.n_k, acc1, h);
    }
  }
}

template <typename T, int D, int MODE, bool MASKED>
hipError_t launch_mode(const AttnParams& p, hipStream_t s) {
  constexpr bool KSIDE = MODE == MODE_BWD_K;
  const int64_t n_rows = KSIDE ? p.n_k : p.n_q;
  const int smem = (int)((2 * Tile<D>::FLOATS + (KSIDE ? 2 * TR : 0)) * sizeof(float));
  const int n_tiles = (int)((n_rows + TR * 4 - 1) / (TR * 4));
  const dim3 grid(bf16k::grid_blocks(MASKED ? (n_tiles + 1) / 2 : n_tiles, p.batch)), block(256);
  const hipError_t e = allow_dynamic_lds<attn_fp32<T, D, MODE, MASKED>>(smem);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL((attn_fp32<T, D, MODE, MASKED>), grid, block, smem, s, p);
  return hipGetLastError();
}

template <typename T, int D>
hipError_t launch_td(const AttnParams& p, int which, hipStream_t s) {
  switch (which) {
    case 0: return p.causal ? launch_mode<T, D, MODE_FWD, true>(p, s) : launch_mode<T, D, MODE_FWD, false>(p, s);
    case 1: return p.causal ? launch_mode<T, D, MODE_BWD_Q, true>(p, s) : launch_mode<T, D, MODE_BWD_Q, false>(p, s);
    case 2: return p.causal ? launch_mode<T, D, MODE_BWD_K, true>(p, s) : launch_mode<T, D, MODE_BWD_K, false>(p, s);
    default: return hipErrorInvalidValue;
  }
}

template <typename T>
hipError_t launch_t(const AttnParams& p, int which, hipStream_t s) {
  switch (p.d) {
    case 32: return launch_td<T, 32>(p, which, s);
    case 64: return launch_td<T, 64>(p, which, s);
    case 128: return launch_td<T, 128>(p, which, s);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace

// 0 forward, 1 dQ, 2 dK and dV; dtype: FHOG_DTYPE_*
hipError_t launch_attn_fp32(const AttnParams& p, int dtype, int which, hipStream_t s) {
  if (dtype == FHOG_DTYPE_FP32) return launch_t<float>(p, which, s);
  return dtype == FHOG_DTYPE_FP16 ? launch_t<_Float16>(p, which, s) : launch_t<__bf16>(p, which, s);
}

}  // namespace fhog
