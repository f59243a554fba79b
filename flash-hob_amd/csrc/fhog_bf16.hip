// bf16 MFMA kernels of the attention double-backward for gfx950 (v_mfma_f32_32x32x16_bf16,
// fp32 accumulation). Four recomputation passes, no atomics, nothing of shape (N_Q, N_K)
// leaves the chip:
//   pass 1  dd_i        Q-tiled   (fhog/triton_bwdbwd.py:185-211)   this file
//   pass 2  b_i         Q-tiled   (fhog/triton_bwdbwd.py:217-251)   this file
//   pass 3  dQ2, ddO    Q-tiled   (fhog/triton_bwdbwd.py:257-313)   fhog_bf16_pc.hip
//   pass 4  dK2, dV2    K-tiled   (fhog/triton_bwdbwd.py:467-535)   fhog_bf16_pc.hip
//
// Fused statistics sweep (PASS = 5, what fhog_bwdbwd launches): b_i = sum_j P (E + ddS (dP - d)) - dd_i sum_j P dP
// needs dd_i only as a factor of a row sum, so dd and b come out of ONE sweep with the five products of pass 2
// and three running sums per query; the three products of a separate pass 1 are saved.
//
// Passes 1, 2 and 5 (row statistics only): a workgroup is 256 threads = 4 wave64 owning 128 queries,
// two workgroups per CU. Each wave keeps its 32 query rows in registers as MFMA B operands
// (Q, ddQ and, in pass 2, dO); K-side tiles of 32 keys stream through a two-stage LDS ring filled by
// direct global->LDS loads. Products are computed transposed (keys = M, queries = N), so every lane
// owns ONE query: L, d, dd are per-lane scalars and the row sum is a per-lane partial sum, reduced
// once at the end with a single cross-half shuffle.
#include "fhog_bf16_util.h"

namespace fhog {
using namespace bf16k;
namespace {

template <bool F16, int D, int PASS, int MASK>
__global__ void __launch_bounds__(256, 2) q_stats_bf16(Params p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int NT = (PASS == 1) ? 2 : 4;  // streamed tensors: K, ddK (, V, ddV)
  constexpr int TILE = TS * 2 * D;
  constexpr int STAGE = NT * TILE;
  constexpr int KK = D / 16;

  int bh, tile;
  if (!decode_block((p.n_q + WG_ROWS - 1) / WG_ROWS, p.batch, MASK != MASK_NONE, bh, tile)) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: lets the compiler branch on scalars
  const int n = lane & 31, h = lane >> 5;
  const int q0 = tile * WG_ROWS, qw = q0 + 32 * wave, qi = qw + n;
  const int qr = min(qi, p.n_q - 1);  // queries past the end compute on a copy of the last row and store nothing
  const int64_t qoff = (int64_t)bh * p.stride_qb, koff = (int64_t)bh * p.stride_kb;
  const __bf16* src[4] = {(const __bf16*)p.k + koff, (const __bf16*)p.ddk + koff, (const __bf16*)p.v + koff,
                          (const __bf16*)p.ddv + koff};

  bf16x8_t Qb[KK], ddQb[KK], dOb[KK];
  load_resident<D>(Qb, (const __bf16*)p.q + qoff, p.stride_qn, qr, h);
  load_resident<D>(ddQb, (const __bf16*)p.ddq + qoff, p.stride_qn, qr, h);
  if (PASS != 1) load_resident<D>(dOb, (const __bf16*)p.dO + qoff, p.stride_qn, qr, h);

  const int64_t row = (int64_t)bh * p.n_q + qr;
  const float l_log2 = p.lse[row] * kLog2e;
  const float c_scale_log2 = p.scale * kLog2e;
  float dsum = 0.f;
  if (PASS == 2) {
    dsum = p.ws_d[row];
  } else {
    // The first statistics sweep of a chain also produces d_i = sum_c O_ic dO_ic (fhog/triton_bwdbwd.py:580) for the
    // sweeps behind it: each lane holds half of its query's row of O and dO, one cross-half shuffle completes the sum.
    bf16x8_t Ob[KK];
    load_resident<D>(Ob, (const __bf16*)p.o + qoff, p.stride_qn, qr, h);
    if (PASS == 1) load_resident<D>(dOb, (const __bf16*)p.dO + qoff, p.stride_qn, qr, h);
#pragma unroll
    for (int kk = 0; kk < KK; kk++)
#pragma unroll
      for (int e = 0; e < 8; e++) dsum = __builtin_fmaf(to_f32<F16>(Ob[kk][e]), to_f32<F16>(dOb[kk][e]), dsum);
    dsum += __shfl_xor(dsum, 32);
    if (h == 0 && qi < p.n_q) p.ws_d[row] = dsum;
  }
  const float dd = PASS == 2 ? p.ws_dd[row] : 0.f;
  float red = 0.f, red_dd = 0.f, red_pdp = 0.f;  // the last two: fused sweep only
  // All register loads land here. The staging loads below are issued from inline asm, which the compiler's
  // wait-count bookkeeping does not see: without this explicit wait it would keep "vmcnt(n)" waits for the
  // resident operands inside the loop, where they would stall every iteration on the tile being staged.
  wait_vm0();

  int aoff[KK];
#pragma unroll
  for (int kk = 0; kk < KK; kk++) aoff[kk] = tile_off<D>(n, 2 * kk + h);

  const StreamKeys<MASK> geo(p.mask_off, p.window, p.n_k);
  int j_begin, j_end;  // key tiles this workgroup visits
  geo.tile_range(q0, WG_ROWS, j_begin, j_end);
  Dma<D> dma;
  dma.init(p.stride_kn, wave, lane);
  const uint32_t ring_lds = lds_addr(smem);
  dma.template issue_all<NT>(ring_lds + (j_begin & 1) * STAGE, TILE, src, (int64_t)j_begin * TS * p.stride_kn, wave, p.n_k - j_begin * TS);
  dma_wait();
  __syncthreads();

  for (int j = j_begin; j < j_end; j++) {
    if (j + 1 < j_end) {
      const uint32_t dst = ring_lds + ((j + 1) & 1) * STAGE;
      const int64_t adv = (int64_t)(j + 1) * TS * p.stride_kn;
      dma.template issue_all<NT>(dst, TILE, src, adv, wave, p.n_k - (j + 1) * TS);
    }
    const int k0 = j * TS;
    const bool masked = geo.partial(k0, qw);  // wave-uniform: the block holds hidden keys (mask edge or tensor end)
    int lo = 0, hi = 0;                       // key k0 + 8g + 4h + e is visible iff lo <= 8g + e <= hi
    if (masked) keep_branch(), geo.limits(k0, qi, h, lo, hi);
    if (!geo.dead(k0, qw)) {  // else every key of the tile is hidden from this wave
      const char* stage = smem + (j & 1) * STAGE;
      // The products are issued as a stream of NT*KK k-steps (K, then V, ddK, ddV); the elementwise work
      // is cut into small pieces placed right behind the MFMAs of the same wave, where it runs in the
      // shadow of the matrix pipe. LDS operands are fetched PF steps ahead.
      //   K  : S += K Q^T, ddS += K ddQ^T
      //   V  : dP += V dO^T            + P = exp2(S c - L)                       (pass 2)
      //   ddK: ddS += ddK Q^T          + P (pass 1) | u = (dP - d) scale, t = dP dd   (pass 2; fused: u only)
      //   ddV: E += ddV dO^T           + acc += P (ddS u - t)                      (pass 2)
      //                                | acc_dd += P ddS, acc_pdp += P dP, w = ddS u   (fused)
      //   tail: acc += P ddS (pass 1) | acc += P E (pass 2) | acc += P (w + E) (fused)
      constexpr int kTensorOfPhase[4] = {0, PASS == 1 ? 1 : 2, 1, 3};
      constexpr int NSTEP = NT * KK, PF = 2, NB = PF + 1, EPK = 16 / KK;
      f32x16_t s = {0}, dds = {0}, dp = {0}, e = {0}, pv, us, tt;
      bf16x8_t a[NB];
#pragma unroll
      for (int i = 0; i < PF; i++) a[i] = lds_read128(stage + kTensorOfPhase[i / KK] * TILE, aoff[i % KK]);
#pragma unroll
      for (int i = 0; i < NSTEP; i++) {
        const int ph = (PASS == 1 && i >= KK) ? 2 : i / KK, kk = i % KK, c = i % NB;
        if (i + PF < NSTEP)
          a[(i + PF) % NB] = lds_read128(stage + kTensorOfPhase[(i + PF) / KK] * TILE, aoff[(i + PF) % KK]);
        __builtin_amdgcn_sched_barrier(0);
        if (ph == 0) {
          s = mfma<F16>(a[c], Qb[kk], s);
          dds = mfma<F16>(a[c], ddQb[kk], dds);
        } else if (ph == 1) {
          dp = mfma<F16>(a[c], dOb[kk], dp);
#pragma unroll
          for (int r = EPK * kk; r < EPK * (kk + 1); r++) pv[r] = __builtin_amdgcn_exp2f(s[r] * c_scale_log2 - l_log2);
        } else if (ph == 2) {
          dds = mfma<F16>(a[c], Qb[kk], dds);
#pragma unroll
          for (int r = EPK * kk; r < EPK * (kk + 1); r++) {
            if (PASS == 1) {
              pv[r] = __builtin_amdgcn_exp2f(s[r] * c_scale_log2 - l_log2);
            } else {
              us[r] = (dp[r] - dsum) * p.scale;
              if (PASS == 2) tt[r] = dp[r] * dd;
            }
          }
        } else {
          e = mfma<F16>(a[c], dOb[kk], e);
          if (kk == 0 && masked) {
            keep_branch();
#pragma unroll
            for (int r = 0; r < 16; r++) pv[r] = in_limits(r, lo, hi) ? pv[r] : 0.f;
          }
#pragma unroll
          for (int r = EPK * kk; r < EPK * (kk + 1); r++) {
            if (PASS == 2) {
              red = __builtin_fmaf(pv[r], __builtin_fmaf(dds[r], us[r], -tt[r]), red);
            } else {
              red_dd = __builtin_fmaf(pv[r], dds[r], red_dd);
              red_pdp = __builtin_fmaf(pv[r], dp[r], red_pdp);
              us[r] *= dds[r];
            }
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      if (PASS == 1) {
        if (masked) {
          keep_branch();
#pragma unroll
          for (int r = 0; r < 16; r++) pv[r] = in_limits(r, lo, hi) ? pv[r] : 0.f;
        }
#pragma unroll
        for (int r = 0; r < 16; r++) red = __builtin_fmaf(pv[r], dds[r], red);   // scale applied once at the end
      } else if (PASS == 2) {
#pragma unroll
        for (int r = 0; r < 16; r++) red = __builtin_fmaf(pv[r], e[r], red);
      } else {
#pragma unroll
        for (int r = 0; r < 16; r++) red = __builtin_fmaf(pv[r], us[r] + e[r], red);
      }
    }
    dma_wait();
    __syncthreads();
  }
  red += __shfl_xor(red, 32);
  if (PASS == 1) red *= p.scale;
  if (PASS == 5) {
    red_dd += __shfl_xor(red_dd, 32);
    red_pdp += __shfl_xor(red_pdp, 32);
    const float dd_i = red_dd * p.scale;
    if (h == 0 && qi < p.n_q) {
      p.ws_dd[row] = dd_i;
      p.ws_b[row] = __builtin_fmaf(-dd_i, red_pdp, red);
    }
  } else if (h == 0 && qi < p.n_q) {
    (PASS == 1 ? p.ws_dd : p.ws_b)[row] = red;
  }
}

template <bool F16, int D, int MASK>
hipError_t launch_stats_d(const Params& p, int pass, hipStream_t s) {
  const dim3 block(256);
  const dim3 grid(grid_blocks((p.n_q + WG_ROWS - 1) / WG_ROWS, p.batch));
  const int tile = TS * 2 * D;
  hipError_t e;
  if (pass == FHOG_PASS_DD) {
    const int smem = 2 * 2 * tile;
    e = hipFuncSetAttribute((const void*)q_stats_bf16<F16, D, 1, MASK>, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((q_stats_bf16<F16, D, 1, MASK>), grid, block, smem, s, p);
  } else if (pass == FHOG_PASS_B) {
    const int smem = 2 * 4 * tile;
    e = hipFuncSetAttribute((const void*)q_stats_bf16<F16, D, 2, MASK>, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((q_stats_bf16<F16, D, 2, MASK>), grid, block, smem, s, p);
  } else {
    const int smem = 2 * 4 * tile;
    e = hipFuncSetAttribute((const void*)q_stats_bf16<F16, D, 5, MASK>, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((q_stats_bf16<F16, D, 5, MASK>), grid, block, smem, s, p);
  }
  return hipGetLastError();
}

}  // namespace

hipError_t launch_bf16_pc_pass(const Params& p, int pass, hipStream_t s);

bool bf16_shape_supported(int64_t n_q, int64_t n_k, int64_t d, int causal) {
  (void)causal;
  return (d == 64 || d == 128) && n_q >= 1 && n_k >= 1;
}

hipError_t launch_bf16_pass(const Params& p, int pass, hipStream_t s) {
  if (!bf16_shape_supported(p.n_q, p.n_k, p.d, p.causal)) return hipErrorInvalidValue;
  if (pass == FHOG_PASS_DQ_DDO || pass == FHOG_PASS_DK_DV) return launch_bf16_pc_pass(p, pass, s);
  if (pass != FHOG_PASS_DD && pass != FHOG_PASS_B && pass != FHOG_PASS_DD_B) return hipErrorInvalidValue;
  const int mask = mask_mode(p);
#define FHOG_STATS(F, DD)                                                             \
  (mask == MASK_NONE ? launch_stats_d<F, DD, MASK_NONE>(p, pass, s)                   \
                     : mask == MASK_CAUSAL ? launch_stats_d<F, DD, MASK_CAUSAL>(p, pass, s) : launch_stats_d<F, DD, MASK_BAND>(p, pass, s))
  if (p.f16) return p.d == 128 ? FHOG_STATS(true, 128) : FHOG_STATS(true, 64);
  return p.d == 128 ? FHOG_STATS(false, 128) : FHOG_STATS(false, 64);
#undef FHOG_STATS
}

}  // namespace fhog
