// bf16 MFMA kernels of the attention double-backward for gfx950 (v_mfma_f32_32x32x16_bf16,
// fp32 accumulation). Four recomputation passes, no atomics, nothing of shape (N_Q, N_K)
// leaves the chip:
//   pass 1  dd_i        Q-tiled   (fhog/triton_bwdbwd.py:185-211)
//   pass 2  b_i         Q-tiled   (fhog/triton_bwdbwd.py:217-251)
//   pass 3  dQ2, ddO    Q-tiled   (fhog/triton_bwdbwd.py:257-313)
//   pass 4  dK2, dV2    K-tiled   (fhog/triton_bwdbwd.py:467-535)
//
// Layout of one workgroup (256 threads = 4 wave64, one wave per SIMD):
//   * the stationary side (128 rows, 32 per wave) lives in registers as MFMA B operands;
//   * the streamed side moves through LDS in 32-row tiles, double buffered, XOR-swizzled in
//     16-byte chunks so that both the row-wise ds_read_b128 (first-level A operands) and
//     the transposing ds_read_b64_tr_b16 (second-level B operands) are bank-conflict free;
//   * first-level products are computed transposed (streamed rows = M, stationary rows = N),
//     so each lane owns ONE stationary row: its row statistics are scalars, and the
//     accumulator registers of the S-shaped tiles are directly the K-slots of the
//     second-level MFMA operand (no shuffle, no LDS round trip).
#include <stdlib.h>

#include "fhog_bf16_util.h"

namespace fhog {
using namespace bf16k;
namespace {

// S-shaped results of one (32 streamed rows) x (32 stationary rows) block, as second-level operands.
struct Ops {
  bf16x8_t p[2], ds[2], ds2[2], ddp[2];
};

// First-level products and the elementwise math for one block.
//   tile pointers: streamed-side tiles in LDS (A operands, row-wise reads)
//   xb/yb/zb: stationary-side B operands.
// Q-sweeps (KSIDE_STREAMED): streamed = K, ddK, V, ddV; stationary = Q, ddQ, dO; lane <-> query.
template <int D, int LEVEL, bool MASK>
__device__ __forceinline__ void block_q(const char* tK, const char* tddK, const char* tV, const char* tddV,
                                        const bf16x8_t* Qb, const bf16x8_t* ddQb, const bf16x8_t* dOb, int lane,
                                        int q_idx, int k_base, float c_scale_log2, float l_log2, float scale, float dsum,
                                        float dd, float b, float& red, Ops& ops) {
  const int n = lane & 31, h = lane >> 5;
  f32x16_t s = {0}, dds = {0}, dp = {0}, e = {0};
#pragma unroll
  for (int kk = 0; kk < D / 16; kk++) {
    const int off = tile_off<D>(n, 2 * kk + h);
    const bf16x8_t ak = lds_read128(tK, off);
    const bf16x8_t addk = lds_read128(tddK, off);
    s = mfma(ak, Qb[kk], s);
    dds = mfma(ak, ddQb[kk], dds);
    dds = mfma(addk, Qb[kk], dds);
    if (LEVEL >= 2) {
      const bf16x8_t av = lds_read128(tV, off);
      const bf16x8_t addv = lds_read128(tddV, off);
      dp = mfma(av, dOb[kk], dp);
      e = mfma(addv, dOb[kk], e);
    }
  }
  f32x16_t pv, dsv, ds2v, ddpv;
#pragma unroll
  for (int r = 0; r < 16; r++) {
    float p = __builtin_amdgcn_exp2f(s[r] * c_scale_log2 - l_log2);
    if (MASK) {
      const int key = k_base + 8 * (r / 4) + 4 * h + (r % 4);
      p = (key <= q_idx) ? p : 0.f;
    }
    const float ddsv = dds[r] * scale;
    if (LEVEL == 1) {
      red += p * ddsv;
    } else {
      const float t1 = ddsv - dd;
      const float dp2 = __builtin_fmaf(-ddsv, dsum, __builtin_fmaf(dp[r], t1, e[r]));
      if (LEVEL == 2) {
        red += p * dp2;
      } else {
        pv[r] = p;
        ddpv[r] = p * t1;
        dsv[r] = p * (dp[r] - dsum);
        ds2v[r] = p * (dp2 - b);
      }
    }
  }
  if (LEVEL >= 3) {
#pragma unroll
    for (int t = 0; t < 2; t++) {
      ops.p[t] = pack8(pv, t);
      ops.ds[t] = pack8(dsv, t);
      ops.ds2[t] = pack8(ds2v, t);
      ops.ddp[t] = pack8(ddpv, t);
    }
  }
}

// ---- passes 1..3 ---------------------------------------------------------------------------------
template <int D, int PASS, bool CAUSAL>
__global__ void __launch_bounds__(256) q_sweep_bf16(Params p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int NT = (PASS == 1) ? 2 : 4;  // streamed tensors: K, ddK (, V, ddV)
  constexpr int TILE = TS * 2 * D;
  constexpr int STAGE = NT * TILE;
  constexpr int NC = D / 32;

  int bh, tile;
  if (!decode_block(p.n_q / WG_ROWS, p.batch, CAUSAL, bh, tile)) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = lane & 31, h = lane >> 5;
  const int q0 = tile * WG_ROWS, qw = q0 + 32 * wave, qi = qw + n;
  const int64_t qoff = (int64_t)bh * p.stride_qb, koff = (int64_t)bh * p.stride_kb;

  const __bf16* src[4] = {(const __bf16*)p.k + koff, (const __bf16*)p.ddk + koff, (const __bf16*)p.v + koff,
                          (const __bf16*)p.ddv + koff};

  bf16x8_t Qb[D / 16], ddQb[D / 16], dOb[D / 16];
  load_resident<D>(Qb, (const __bf16*)p.q + qoff, p.stride_qn, qi, h);
  load_resident<D>(ddQb, (const __bf16*)p.ddq + qoff, p.stride_qn, qi, h);
  if (PASS >= 2) load_resident<D>(dOb, (const __bf16*)p.dO + qoff, p.stride_qn, qi, h);

  const int64_t row = (int64_t)bh * p.n_q + qi;
  const float l_log2 = p.lse[row] * kLog2e;
  const float c_scale_log2 = p.scale * kLog2e;
  const float dsum = PASS >= 2 ? p.ws_d[row] : 0.f;
  const float dd = PASS >= 2 ? p.ws_dd[row] : 0.f;
  const float b = PASS >= 3 ? p.ws_b[row] : 0.f;

  float red = 0.f;
  f32x16_t acc_dq[NC], acc_ddo[NC];
#pragma unroll
  for (int cb = 0; cb < NC; cb++) {
    acc_dq[cb] = f32x16_t{0};
    acc_ddo[cb] = f32x16_t{0};
  }

  const int n_tiles = CAUSAL ? (q0 + WG_ROWS) / TS : p.n_k / TS;
  Stage<D, NT> st;
  st.load(src, p.stride_kn, 0, tid);
  st.store(smem, tid);
  __syncthreads();

  for (int kt = 0; kt < n_tiles; kt++) {
    const char* cur = smem + (kt & 1) * STAGE;
    const bool more = kt + 1 < n_tiles;
    if (more) st.load(src, p.stride_kn, (kt + 1) * TS, tid);

    const int k0 = kt * TS;
    const bool active = !CAUSAL || k0 <= qw;      // else every key of the tile is masked for this wave
    const bool diag = CAUSAL && k0 == qw;
    if (active) {
      Ops ops;
      const char* tK = cur;
      const char* tddK = cur + TILE;
      const char* tV = cur + 2 * TILE;
      const char* tddV = cur + 3 * TILE;
      if (diag)
        block_q<D, PASS, true>(tK, tddK, tV, tddV, Qb, ddQb, dOb, lane, qi, k0, c_scale_log2, l_log2, p.scale, dsum, dd, b,
                               red, ops);
      else
        block_q<D, PASS, false>(tK, tddK, tV, tddV, Qb, ddQb, dOb, lane, qi, k0, c_scale_log2, l_log2, p.scale, dsum, dd,
                                b, red, ops);
      if (PASS == 3) {
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
          for (int cb = 0; cb < NC; cb++) {
            acc_dq[cb] = mfma(ops.ds[t], lds_read_tr<D>(tddK, t, cb, lane), acc_dq[cb]);
            acc_dq[cb] = mfma(ops.ds2[t], lds_read_tr<D>(tK, t, cb, lane), acc_dq[cb]);
            acc_ddo[cb] = mfma(ops.ddp[t], lds_read_tr<D>(tV, t, cb, lane), acc_ddo[cb]);
            acc_ddo[cb] = mfma(ops.p[t], lds_read_tr<D>(tddV, t, cb, lane), acc_ddo[cb]);
          }
      }
    }
    if (more) st.store(smem + ((kt + 1) & 1) * STAGE, tid);
    __syncthreads();
  }

  if (PASS == 1 || PASS == 2) {
    red += __shfl_xor(red, 32);
    if (h == 0) (PASS == 1 ? p.ws_dd : p.ws_b)[row] = red;
  } else {
    // acc[cb][r] holds (query qw + 8*(r/4) + 4h + r%4, column cb*32 + n)
    __bf16* odq = (__bf16*)p.dq2 + qoff;
    __bf16* oddo = (__bf16*)p.ddo + qoff;
#pragma unroll
    for (int cb = 0; cb < NC; cb++)
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int64_t o = (int64_t)(qw + 8 * (r / 4) + 4 * h + (r % 4)) * p.stride_qn + cb * 32 + n;
        odq[o] = (__bf16)(acc_dq[cb][r] * p.scale);
        oddo[o] = (__bf16)acc_ddo[cb][r];
      }
  }
}

// ---- pass 4 --------------------------------------------------------------------------------------
// Stationary = 32 keys per wave (K, ddK, V, ddV as B operands), streamed = query tiles
// (Q, ddQ, dO through LDS + L, d, dd, b). First-level products are S[i][j] with the query as M:
// lane <-> key, registers <-> queries, so dS^T, dS'^T, ddP^T come out as A operands over queries.
template <int D, bool MASK>
__device__ __forceinline__ void block_k(const char* tQ, const char* tddQ, const char* tdO, const float* stat,
                                        const bf16x8_t* Kb, const bf16x8_t* ddKb, const bf16x8_t* Vb, const bf16x8_t* ddVb,
                                        int lane, int k_idx, int q_base, float c_scale_log2, float scale, Ops& ops) {
  const int n = lane & 31, h = lane >> 5;
  f32x16_t s = {0}, dds = {0}, dp = {0}, e = {0};
#pragma unroll
  for (int kk = 0; kk < D / 16; kk++) {
    const int off = tile_off<D>(n, 2 * kk + h);
    const bf16x8_t aq = lds_read128(tQ, off);
    const bf16x8_t addq = lds_read128(tddQ, off);
    const bf16x8_t ado = lds_read128(tdO, off);
    s = mfma(aq, Kb[kk], s);
    dds = mfma(addq, Kb[kk], dds);
    dds = mfma(aq, ddKb[kk], dds);
    dp = mfma(ado, Vb[kk], dp);
    e = mfma(ado, ddVb[kk], e);
  }
  f32x16_t dsv, ds2v, ddpv;
#pragma unroll
  for (int g = 0; g < 4; g++) {
    // rows 8g + 4h + 0..3 of the query tile: four consecutive floats of each statistic
    const f32x4_t l4 = *reinterpret_cast<const f32x4_t*>(stat + 0 * TS + 8 * g + 4 * h);
    const f32x4_t d4 = *reinterpret_cast<const f32x4_t*>(stat + 1 * TS + 8 * g + 4 * h);
    const f32x4_t dd4 = *reinterpret_cast<const f32x4_t*>(stat + 2 * TS + 8 * g + 4 * h);
    const f32x4_t b4 = *reinterpret_cast<const f32x4_t*>(stat + 3 * TS + 8 * g + 4 * h);
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int r = 4 * g + j;
      float p = __builtin_amdgcn_exp2f(s[r] * c_scale_log2 - l4[j]);
      if (MASK) {
        const int qrow = q_base + 8 * g + 4 * h + j;
        p = (k_idx <= qrow) ? p : 0.f;
      }
      const float ddsv = dds[r] * scale;
      const float t1 = ddsv - dd4[j];
      const float dp2 = __builtin_fmaf(-ddsv, d4[j], __builtin_fmaf(dp[r], t1, e[r]));
      ddpv[r] = p * t1;
      dsv[r] = p * (dp[r] - d4[j]);
      ds2v[r] = p * (dp2 - b4[j]);
    }
  }
#pragma unroll
  for (int t = 0; t < 2; t++) {
    ops.ds[t] = pack8(dsv, t);
    ops.ds2[t] = pack8(ds2v, t);
    ops.ddp[t] = pack8(ddpv, t);
  }
}

template <int D, bool CAUSAL>
__global__ void __launch_bounds__(256) k_sweep_bf16(Params p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int NT = 3;  // streamed tensors: Q, ddQ, dO
  constexpr int TILE = TS * 2 * D;
  constexpr int STAGE = NT * TILE + 4 * TS * (int)sizeof(float);  // + L*log2e, d, dd, b of the 32 rows
  constexpr int NC = D / 32;

  int bh, tile;
  if (!decode_block(p.n_k / WG_ROWS, p.batch, false, bh, tile)) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = lane & 31, h = lane >> 5;
  const int k0 = tile * WG_ROWS, kw = k0 + 32 * wave, kj = kw + n;
  const int64_t qoff = (int64_t)bh * p.stride_qb, koff = (int64_t)bh * p.stride_kb;

  const __bf16* src[3] = {(const __bf16*)p.q + qoff, (const __bf16*)p.ddq + qoff, (const __bf16*)p.dO + qoff};
  const float* stat_src[4] = {p.lse + (int64_t)bh * p.n_q, p.ws_d + (int64_t)bh * p.n_q, p.ws_dd + (int64_t)bh * p.n_q,
                              p.ws_b + (int64_t)bh * p.n_q};

  bf16x8_t Kb[D / 16], ddKb[D / 16], Vb[D / 16], ddVb[D / 16];
  load_resident<D>(Kb, (const __bf16*)p.k + koff, p.stride_kn, kj, h);
  load_resident<D>(ddKb, (const __bf16*)p.ddk + koff, p.stride_kn, kj, h);
  load_resident<D>(Vb, (const __bf16*)p.v + koff, p.stride_kn, kj, h);
  load_resident<D>(ddVb, (const __bf16*)p.ddv + koff, p.stride_kn, kj, h);

  const float c_scale_log2 = p.scale * kLog2e;
  f32x16_t acc_dk[NC], acc_dv[NC];
#pragma unroll
  for (int cb = 0; cb < NC; cb++) {
    acc_dk[cb] = f32x16_t{0};
    acc_dv[cb] = f32x16_t{0};
  }

  // causal: query tiles before this workgroup's first key see none of its keys
  const int t_begin = CAUSAL ? k0 / TS : 0;
  const int n_tiles = p.n_q / TS;
  Stage<D, NT> st;
  float stat_reg = 0.f;  // threads 0..127: one statistic value of the next tile
  auto load_stat = [&](int q_base) {
    if (tid < 4 * TS) {
      const float v = stat_src[tid / TS][q_base + (tid % TS)];
      stat_reg = (tid < TS) ? v * kLog2e : v;
    }
  };
  auto store_stat = [&](char* stage_base) {
    if (tid < 4 * TS) reinterpret_cast<float*>(stage_base + NT * TILE)[tid] = stat_reg;
  };
  st.load(src, p.stride_qn, t_begin * TS, tid);
  load_stat(t_begin * TS);
  st.store(smem + (t_begin & 1) * STAGE, tid);
  store_stat(smem + (t_begin & 1) * STAGE);
  __syncthreads();

  for (int qt = t_begin; qt < n_tiles; qt++) {
    const char* cur = smem + (qt & 1) * STAGE;
    const bool more = qt + 1 < n_tiles;
    if (more) {
      st.load(src, p.stride_qn, (qt + 1) * TS, tid);
      load_stat((qt + 1) * TS);
    }
    const int qb = qt * TS;
    const bool active = !CAUSAL || qb + TS - 1 >= kw;  // some query of the tile sees some key of this wave
    const bool diag = CAUSAL && qb == kw;
    if (active) {
      Ops ops;
      const char* tQ = cur;
      const char* tddQ = cur + TILE;
      const char* tdO = cur + 2 * TILE;
      const float* stat = reinterpret_cast<const float*>(cur + NT * TILE);
      if (diag)
        block_k<D, true>(tQ, tddQ, tdO, stat, Kb, ddKb, Vb, ddVb, lane, kj, qb, c_scale_log2, p.scale, ops);
      else
        block_k<D, false>(tQ, tddQ, tdO, stat, Kb, ddKb, Vb, ddVb, lane, kj, qb, c_scale_log2, p.scale, ops);
#pragma unroll
      for (int t = 0; t < 2; t++)
#pragma unroll
        for (int cb = 0; cb < NC; cb++) {
          acc_dk[cb] = mfma(ops.ds[t], lds_read_tr<D>(tddQ, t, cb, lane), acc_dk[cb]);
          acc_dk[cb] = mfma(ops.ds2[t], lds_read_tr<D>(tQ, t, cb, lane), acc_dk[cb]);
          acc_dv[cb] = mfma(ops.ddp[t], lds_read_tr<D>(tdO, t, cb, lane), acc_dv[cb]);
        }
    }
    if (more) {
      st.store(smem + ((qt + 1) & 1) * STAGE, tid);
      store_stat(smem + ((qt + 1) & 1) * STAGE);
    }
    __syncthreads();
  }

  __bf16* odk = (__bf16*)p.dk2 + koff;
  __bf16* odv = (__bf16*)p.dv2 + koff;
#pragma unroll
  for (int cb = 0; cb < NC; cb++)
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int64_t o = (int64_t)(kw + 8 * (r / 4) + 4 * h + (r % 4)) * p.stride_kn + cb * 32 + n;
      odk[o] = (__bf16)(acc_dk[cb][r] * p.scale);
      odv[o] = (__bf16)acc_dv[cb][r];
    }
}

template <int D, bool CAUSAL>
hipError_t launch_d(const Params& p, int pass, hipStream_t s) {
  const dim3 block(256);
  const int heads8 = (p.batch + 7) / 8 * 8;
  const dim3 gq((unsigned)(heads8 * (p.n_q / WG_ROWS))), gk((unsigned)(heads8 * (p.n_k / WG_ROWS)));
  const size_t tile = (size_t)TS * 2 * D;
#define FHOG_LAUNCH(kern, grid, smem)                                                                             \
  do {                                                                                                            \
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)(smem)); \
    if (e != hipSuccess) return e;                                                                                \
    hipLaunchKernelGGL(kern, grid, block, (smem), s, p);                                                          \
  } while (0)
  switch (pass) {
    case FHOG_PASS_DD: FHOG_LAUNCH((q_sweep_bf16<D, 1, CAUSAL>), gq, NSTAGE * 2 * tile); break;
    case FHOG_PASS_B: FHOG_LAUNCH((q_sweep_bf16<D, 2, CAUSAL>), gq, NSTAGE * 4 * tile); break;
    case FHOG_PASS_DQ_DDO: FHOG_LAUNCH((q_sweep_bf16<D, 3, CAUSAL>), gq, NSTAGE * 4 * tile); break;
    case FHOG_PASS_DK_DV: FHOG_LAUNCH((k_sweep_bf16<D, CAUSAL>), gk, NSTAGE * (3 * tile + 4 * TS * sizeof(float))); break;
    default: return hipErrorInvalidValue;
  }
#undef FHOG_LAUNCH
  return hipGetLastError();
}

}  // namespace

bool bf16_shape_supported(int64_t n_q, int64_t n_k, int64_t d, int causal) {
  (void)causal;
  return (d == 64 || d == 128) && n_q % WG_ROWS == 0 && n_k % WG_ROWS == 0;
}

hipError_t launch_bf16_pc_pass(const Params& p, int pass, hipStream_t s);

hipError_t launch_bf16_pass(const Params& p, int pass, hipStream_t s) {
  if (!bf16_shape_supported(p.n_q, p.n_k, p.d, p.causal)) return hipErrorInvalidValue;
  static const bool old_variant = getenv("FHOG_OLD34") != nullptr;
  if (!old_variant && (pass == FHOG_PASS_DQ_DDO || pass == FHOG_PASS_DK_DV)) return launch_bf16_pc_pass(p, pass, s);
  if (p.d == 128) return p.causal ? launch_d<128, true>(p, pass, s) : launch_d<128, false>(p, pass, s);
  return p.causal ? launch_d<64, true>(p, pass, s) : launch_d<64, false>(p, pass, s);
}

}  // namespace fhog
