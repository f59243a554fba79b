// 16-bit MFMA kernels of the attention double-backward for gfx950 (v_mfma_f32_32x32x16_bf16 / _f16,
// fp32 accumulation). Four recomputation passes, no atomics, nothing of shape (N_Q, N_K)
// leaves the chip:
//   pass 1  d_i, dd_i   Q-tiled   (fhog/triton_bwdbwd.py:580, 185-211)   q_sweep_bf16<PASS=1>
//   pass 2  b_i         Q-tiled   (fhog/triton_bwdbwd.py:217-251)        q_sweep_bf16<PASS=2>
//   pass 3  dQ2, ddO    Q-tiled   (fhog/triton_bwdbwd.py:257-313)        d=64: q_sweep_bf16<PASS=3>; d=128: fhog_bf16_pc.hip
//   pass 4  dK2, dV2    K-tiled   (fhog/triton_bwdbwd.py:467-535)        d=64: k_sweep_bf16;         d=128: fhog_bf16_pc.hip
//
// Fused statistics sweep (PASS = 5, opt-in): b_i = sum_j P (E + ddS (dP - d)) - dd_i sum_j P dP
// needs dd_i only as a factor of a row sum, so dd and b come out of ONE sweep with the five products of pass 2
// and three running sums per query; the three products of a separate pass 1 are saved.
// PASS = 7 (opt-in schedules whose second sweep already produced ddO, fhog_bf16_ddo.hip): pass 3 for dQ2 alone, d = 64.
//
// The kernels of this file are single-role: a workgroup is 256 threads = 4 wave64 owning 128 stationary rows,
// two workgroups per CU (the b sweeps at d = 128 also exist with 8 waves and 256 rows, one workgroup per CU, for
// launches with enough workgroups: half the staging loads per row). Each wave keeps its 32 rows in registers as
// MFMA B operands (Q, ddQ and, from pass 2 on, dO; K, ddK, V, ddV in pass 4); the other side streams through a
// two-stage LDS ring of 32-row tiles filled by direct global->LDS loads. First-level products are computed with the
// streamed rows as M and the stationary rows as N, so every lane owns ONE stationary row: in the Q-tiled sweeps L, d, dd, b are per-lane scalars and a
// row sum is a per-lane partial sum, reduced once at the end with a single cross-half shuffle.
// Passes 3 and 4 at d = 64 fit the second-level products into the same wave (256 registers): the S-shaped
// accumulators, rounded to 16 bits, are the B operands of those products as they stand (contraction over the
// streamed rows), the A operands are transposing reads of the staged tiles in the same row order. At d = 128
// the output accumulators alone take 128 registers and the work is split over producer and consumer waves.

#include "fhog_bf16_util.h"

namespace fhog {
using namespace bf16k;
namespace {

// Finishes a statistics pass that ran split: sums the partial row sums in a fixed order.
template <int PASS>
__global__ void __launch_bounds__(256) combine_stats(Params p) {
  const int64_t rows = (int64_t)p.batch * p.n_q, row = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (row >= rows) return;
  float a = 0.f, b = 0.f, c = 0.f;
  for (int s = 0; s < p.n_split; s++) {
    const float* ps = p.part + (int64_t)s * 3 * rows + row;
    if (PASS != 2) a += ps[0];
    if (PASS != 1) b += ps[rows];
    if (PASS == 5) c += ps[2 * rows];
  }
  if (PASS != 2) p.ws_dd[row] = a;
  if (PASS == 2) p.ws_b[row] = b;
  if (PASS == 5) p.ws_b[row] = __builtin_fmaf(-a, c, b);
}

// Finishes pass 3 or 4 that ran split: out0 = scale * sum of the first partial tensor, out1 = sum of the second,
// rounded to the tensor type. One thread per four columns of a row.
template <bool F16, int D>
__global__ void __launch_bounds__(256) combine_out(const float* part, int n_split, int batch, int n, int64_t stride_b,
                                                   int64_t stride_n, uint16_t* out0, uint16_t* out1, float scale) {
  const int64_t rows = (int64_t)batch * n, idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t row = idx / (D / 4);
  const int col = (int)(idx % (D / 4)) * 4;
  if (row >= rows) return;
  f32x4_t a = {0.f, 0.f, 0.f, 0.f}, b = {0.f, 0.f, 0.f, 0.f};
  for (int s = 0; s < n_split; s++) {
    const float* ps = part + ((int64_t)s * 2 * rows + row) * D + col;
    a += *reinterpret_cast<const f32x4_t*>(ps);
    b += *reinterpret_cast<const f32x4_t*>(ps + rows * D);
  }
  const int64_t o = (row / n) * stride_b + (row % n) * stride_n + col;
  *reinterpret_cast<u32x2_t*>(out0 + o) = pack4<F16>(a[0] * scale, a[1] * scale, a[2] * scale, a[3] * scale);
  *reinterpret_cast<u32x2_t*>(out1 + o) = pack4<F16>(b[0], b[1], b[2], b[3]);
}

// Row statistics of the wave's queries handed from one sweep to the next inside a launch that runs several of them for
// its tile (q_stage1_bf16): every lane of a query's pair holds the value.
struct RowChain {
  float d, dd, b;
};

// One Q-tiled sweep for the tile (bh, tile, split). CHAIN: the sweep is one of several that a launch runs for its tile;
// it takes d, dd, b from `chain` where a sweep before it left them, and leaves there what it produces (it still writes
// them to the workspace for the launches behind it).
template <bool F16, int D, int PASS, int MASK, int NW, int SUB, bool CHAIN>
__device__ __forceinline__ void q_sweep_run(const Params& p, char* smem, int bh, int tile, int split, RowChain& chain) {
  constexpr int ROWS = 32 * NW;
  constexpr int NT = (PASS == 1) ? 2 : 4;  // streamed tensors: K, ddK (, V, ddV)
  // PASS 7 is pass 3 without its ddO half (dQ2 alone, for the schedules whose earlier sweep already produced ddO)
  constexpr bool P3 = PASS == 3 || PASS == 7, WITH_DDO = PASS == 3;
  constexpr int TILE = TS * 2 * D;
  constexpr int STAGE = NT * TILE;
  constexpr int KK = D / 16;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: lets the compiler branch on scalars
  const int n = lane & 31, h = lane >> 5;
  const int q0 = tile * ROWS, qw = q0 + 32 * wave, qi = qw + n;
  const int qr = min(qi, p.n_q - 1);  // queries past the end compute on a copy of the last row and store nothing
  const int64_t qoff = (int64_t)bh * p.stride_qb, koff = (int64_t)bh * p.stride_kb;
  const __bf16* src[4] = {(const __bf16*)p.k + koff, (const __bf16*)p.ddk + koff, (const __bf16*)p.v + koff,
                          (const __bf16*)p.ddv + koff};

  // The first streamed tile is requested before the resident operands: the two round trips to memory overlap instead of
  // following each other (a workgroup that visits four tiles spends most of its time in this prologue).
  const StreamKeys<MASK> geo(p.mask_off, p.window, p.n_k);
  int j_begin, j_end;  // key tiles this workgroup visits
  geo.tile_range(q0, ROWS, j_begin, j_end);
  if (p.n_split > 1) split_range(split, p.n_split, j_begin, j_end);
  // staging: four waves share the rows of a tile; with eight waves each group of four takes half of the tensors
  constexpr int NLD = NW == 8 ? NT / 2 : NT;
  const int half = NW == 8 ? wave >> 2 : 0;
  const __bf16* srcl[NLD];
#pragma unroll
  for (int x = 0; x < NLD; x++) {   // wave-uniform, and the staging instruction wants it in scalar registers
    const uint64_t a = (uint64_t)(NW == 8 ? (half ? src[NT / 2 + x < NT ? NT / 2 + x : 0] : src[x]) : src[x]);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a), hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
    srcl[x] = (const __bf16*)(((uint64_t)hi << 32) | lo);
  }
  Dma<D> dma;
  dma.init(p.stride_kn, wave & 3, lane);
  const uint32_t ring_lds = lds_addr(smem) + half * NLD * TILE;
  // the ring holds 2 * SUB tiles; tile j lives in slot (j - j_begin) mod (2 * SUB)
  const auto stage_tile = [&](int j) {
    const uint32_t dst = ring_lds + ((j - j_begin) & (2 * SUB - 1)) * STAGE;
    dma.template issue_all<NLD>(dst, TILE, srcl, (int64_t)j * TS * p.stride_kn, wave & 3, p.n_k - j * TS);
  };
#pragma unroll
  for (int u = 0; u < SUB; u++)
    if (j_begin + u < j_end) stage_tile(j_begin + u);

  bf16x8_t Qb[KK], ddQb[KK], dOb[KK];
  load_resident<D>(Qb, (const __bf16*)p.q + qoff, p.stride_qn, qr, h);
  load_resident<D>(ddQb, (const __bf16*)p.ddq + qoff, p.stride_qn, qr, h);
  if (PASS != 1) load_resident<D>(dOb, (const __bf16*)p.dO + qoff, p.stride_qn, qr, h);

  const int64_t row = (int64_t)bh * p.n_q + qr;
  const float l_log2 = p.lse[row] * kLog2e;
  const float c_scale_log2 = p.scale * kLog2e;
  float dsum = 0.f;
  if (PASS == 2 || P3) {
    dsum = CHAIN ? chain.d : p.ws_d[row];
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
    if (h == 0 && qi < p.n_q && split == 0) p.ws_d[row] = dsum;
    if (CHAIN) chain.d = dsum;
  }
  const float dd = (PASS == 2 || P3) ? (CHAIN ? chain.dd : p.ws_dd[row]) : 0.f;
  const float b = P3 ? (CHAIN ? chain.b : p.ws_b[row]) : 0.f;
  const float kc = __builtin_fmaf(dd, dsum, b);   // per-row constant of dP' = E + (ddS - dd)(dP - d) - kc (passes 2, 3)
  float red = 0.f, red_dd = 0.f, red_pdp = 0.f;  // the last two: fused sweep only
  // PASS 3 (d = 64): the second-level products follow in the same wave, with the S-shaped tiles as B operands
  // straight from the registers; lane = query, registers = output columns
  constexpr int NC = D / 32;
  f32x16_t acc_dq[NC], acc_ddo[NC];
  int troff[NC][2];
  if (P3) {
#pragma unroll
    for (int cb = 0; cb < NC; cb++) {
      acc_dq[cb] = f32x16_t{0};
      acc_ddo[cb] = f32x16_t{0};
      troff[cb][0] = tr_lane_off_acc<D>(cb, 0, lane);
      troff[cb][1] = tr_lane_off_acc<D>(cb, 1, lane);
    }
  }
  // All register loads land here. The staging loads below are issued from inline asm, which the compiler's
  // wait-count bookkeeping does not see: without this explicit wait it would keep "vmcnt(n)" waits for the
  // resident operands inside the loop, where they would stall every iteration on the tile being staged.
  wait_vm0();

  int aoff[KK];
#pragma unroll
  for (int kk = 0; kk < KK; kk++) aoff[kk] = tile_off<D>(n, 2 * kk + h);

  dma_wait();
  __syncthreads();

  for (int jj = j_begin; jj < j_end; jj += SUB) {
#pragma unroll
    for (int u = 0; u < SUB; u++)
      if (jj + SUB + u < j_end) stage_tile(jj + SUB + u);
#pragma unroll
    for (int u = 0; u < SUB; u++) {
      const int j = jj + u;
      if (SUB > 1 && j >= j_end) continue;
      const int k0 = j * TS;
      const bool masked = geo.partial(k0, qw);  // wave-uniform: the block holds hidden keys (mask edge or tensor end)
      int lo = 0, hi = 0;                       // key k0 + 8g + 4h + e is visible iff lo <= 8g + e <= hi
      if (masked) keep_branch(), geo.limits(k0, qi, h, lo, hi);
      if (!geo.dead(k0, qw)) {  // else every key of the tile is hidden from this wave
        const char* stage = smem + (((jj - j_begin) & SUB) + u) * STAGE;
        // The products are issued as a stream of NT*KK k-steps (K, then V, ddK, ddV); the elementwise work
        // is cut into small pieces placed right behind the MFMAs of the same wave, where it runs in the
        // shadow of the matrix pipe. LDS operands are fetched PF steps ahead.
        //   K  : S += K Q^T, ddS += K ddQ^T
        //   V  : dP += V dO^T            + P = exp2(S c - L)                       (pass 2)
        //   ddK: ddS += ddK Q^T          + P (pass 1) | u = (dP - d) scale (fused)
        //   ddV: E += ddV dO^T           + acc += P (ddS - dd) u   (pass 2: u = dP - d and E' = E - dd d come from
        //                                  accumulators that start at the row constants; with the tail, acc ends as
        //                                  sum P (E' + (ddS - dd) u) = sum P (E + ddS u - dP dd))
        //                                | acc_dd += P ddS, acc_pdp += P dP, w = ddS u   (fused)
        //   tail: acc += P ddS (pass 1) | acc += P E (pass 2) | acc += P (w + E) (fused)
        // Pass 3 (d = 64) runs the same stream with the elementwise work of the producer/consumer kernel (dS = P u behind
        // ddK; w = ddS scale - dd, ddP = P w, z = P (w u - dd d - b) behind ddV; dS' = P E + z in the tail), packs the four
        // tiles to 16 bits and goes on to the second-level products.
        constexpr int kTensorOfPhase[4] = {0, PASS == 1 ? 1 : 2, 1, 3};
        constexpr int NSTEP = NT * KK, PF = 2, NB = PF + 1, EPK = 16 / KK;
        f32x16_t s = {0}, dds = {0}, dp = {0}, e = {0}, pv, us, tt;
        if (PASS == 2) {   // u = dP - d and E' = E - kc straight from the matrix pipe (in pass 3 this measured slower)
#pragma unroll
          for (int r = 0; r < 16; r++) dp[r] = -dsum, e[r] = -kc;
        }
        uint32_t pk_ds[8], pk_ds2[8], pk_ddp[8], pk_p[8];   // PASS 3: packed dS, dS', ddP, P (registers 2i, 2i+1)
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
            if (P3 && kk == 0 && masked) {
              keep_branch();
#pragma unroll
              for (int r = 0; r < 16; r++) pv[r] = in_limits(r, lo, hi) ? pv[r] : 0.f;
            }
#pragma unroll
            for (int r = EPK * kk; r < EPK * (kk + 1); r++) {
              if (PASS == 1) {
                pv[r] = __builtin_amdgcn_exp2f(s[r] * c_scale_log2 - l_log2);
              } else if (P3) {
                dp[r] -= dsum;                           // u
                us[r] = pv[r] * dp[r];                   // dS = P u (scale applied to the accumulator at the end)
              } else if (PASS == 5) {
                us[r] = (dp[r] - dsum) * p.scale;
              }
            }
          } else {
            e = mfma<F16>(a[c], dOb[kk], e);
            if (!P3 && kk == 0 && masked) {
              keep_branch();
#pragma unroll
              for (int r = 0; r < 16; r++) pv[r] = in_limits(r, lo, hi) ? pv[r] : 0.f;
            }
#pragma unroll
            for (int r = EPK * kk; r < EPK * (kk + 1); r++) {
              if (PASS == 2) {
                red = __builtin_fmaf(pv[r] * __builtin_fmaf(dds[r], p.scale, -dd), dp[r], red);   // P w u
              } else if (P3) {
                const float w = __builtin_fmaf(dds[r], p.scale, -dd);
                const float ddp = pv[r] * w;
                tt[r] = pv[r] * __builtin_fmaf(w, dp[r], -kc);   // z = P (w u - kc)
                if (r & 1) {
                  if (WITH_DDO) pk_ddp[r / 2] = pack2<F16>(dds[r - 1], ddp);   // dds[r - 1] holds ddP of the even register by now
                  pk_ds[r / 2] = pack2<F16>(us[r - 1], us[r]);
                  if (WITH_DDO) pk_p[r / 2] = pack2<F16>(pv[r - 1], pv[r]);
                } else if (WITH_DDO) {
                  dds[r] = ddp;
                }
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
        } else if (P3) {
#pragma unroll
          for (int r = 0; r < 16; r += 2)
            pk_ds2[r / 2] = pack2<F16>(__builtin_fmaf(pv[r], e[r], tt[r]), __builtin_fmaf(pv[r + 1], e[r + 1], tt[r + 1]));
          // dQ2^T += ddK^T dS^T + K^T dS'^T ; ddO^T += V^T ddP^T + ddV^T P^T  (stage order K, ddK, V, ddV)
          constexpr int NIT = 2 * NC;
          const auto opnd = [](const uint32_t* pk, int t) {
            return __builtin_bit_cast(bf16x8_t, u32x4_t{pk[4 * t], pk[4 * t + 1], pk[4 * t + 2], pk[4 * t + 3]});
          };
          constexpr int NX = WITH_DDO ? 4 : 2;   // staged tensors the second level reads: K, ddK (, V, ddV)
          bf16x8_t ta[2][NX];
#pragma unroll
          for (int x = 0; x < NX; x++) ta[0][x] = lds_read_tr_pre(stage + troff[0][0], stage + troff[0][1], x * TILE);
          if (WITH_DDO) {
#pragma unroll
            for (int it = 0; it < NIT; it++) {
              const int t = it / NC, cb = it % NC, c = it & 1;
              if (it + 1 < NIT) {
                const int t1 = (it + 1) / NC, cb1 = (it + 1) % NC;
#pragma unroll
                for (int x = 0; x < NX; x++)
                  ta[c ^ 1][x] = lds_read_tr_pre(stage + troff[cb1][0], stage + troff[cb1][1], x * TILE + t1 * 16 * 2 * D);
              }
              __builtin_amdgcn_sched_barrier(0);
              acc_dq[cb] = mfma<F16>(ta[c][1], opnd(pk_ds, t), acc_dq[cb]);
              acc_ddo[cb] = mfma<F16>(ta[c][NX - 2], opnd(pk_ddp, t), acc_ddo[cb]);
              acc_dq[cb] = mfma<F16>(ta[c][0], opnd(pk_ds2, t), acc_dq[cb]);
              acc_ddo[cb] = mfma<F16>(ta[c][NX - 1], opnd(pk_p, t), acc_ddo[cb]);
              __builtin_amdgcn_sched_barrier(0);
            }
          } else {
            // dQ2 alone: two column blocks per round, so that the MFMAs on one accumulator are two instructions apart
            constexpr int NP = NC / 2;
            bf16x8_t tb[2][2][2];   // [buffer][column block of the pair][K | ddK]
            const auto read_tb = [&](int buf, int it) {
              const int t1 = it / NP, cp1 = it % NP;
#pragma unroll
              for (int cl = 0; cl < 2; cl++)
#pragma unroll
                for (int x = 0; x < 2; x++)
                  tb[buf][cl][x] = lds_read_tr_pre(stage + troff[2 * cp1 + cl][0], stage + troff[2 * cp1 + cl][1], x * TILE + t1 * 16 * 2 * D);
            };
#pragma unroll
            for (int x = 0; x < 2; x++) tb[0][0][x] = ta[0][x];
#pragma unroll
            for (int x = 0; x < 2; x++) tb[0][1][x] = lds_read_tr_pre(stage + troff[1][0], stage + troff[1][1], x * TILE);
#pragma unroll
            for (int it = 0; it < 2 * NP; it++) {
              const int t = it / NP, cp = it % NP, c = it & 1;
              if (it + 1 < 2 * NP) read_tb(c ^ 1, it + 1);
              __builtin_amdgcn_sched_barrier(0);
              acc_dq[2 * cp] = mfma<F16>(tb[c][0][1], opnd(pk_ds, t), acc_dq[2 * cp]);
              acc_dq[2 * cp + 1] = mfma<F16>(tb[c][1][1], opnd(pk_ds, t), acc_dq[2 * cp + 1]);
              acc_dq[2 * cp] = mfma<F16>(tb[c][0][0], opnd(pk_ds2, t), acc_dq[2 * cp]);
              acc_dq[2 * cp + 1] = mfma<F16>(tb[c][1][0], opnd(pk_ds2, t), acc_dq[2 * cp + 1]);
              __builtin_amdgcn_sched_barrier(0);
            }
          }
        } else {
#pragma unroll
          for (int r = 0; r < 16; r++) red = __builtin_fmaf(pv[r], us[r] + e[r], red);
        }
      }
    }
    dma_wait();
    __syncthreads();
  }
  if (WITH_DDO && p.n_split > 1) {   // fp32 partial rows [split][dQ2 | ddO][batch * n_q][D]
    if (qi >= p.n_q) return;
    const int64_t rows = (int64_t)p.batch * p.n_q;
    float* pq = p.part + ((int64_t)split * 2 * rows + (int64_t)bh * p.n_q + qi) * D;
    float* po = pq + rows * D;
#pragma unroll
    for (int cb = 0; cb < NC; cb++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const f32x16_t& x = acc_dq[cb];
        const f32x16_t& y = acc_ddo[cb];
        *reinterpret_cast<f32x4_t*>(pq + 32 * cb + 8 * g + 4 * h) = f32x4_t{x[4 * g], x[4 * g + 1], x[4 * g + 2], x[4 * g + 3]};
        *reinterpret_cast<f32x4_t*>(po + 32 * cb + 8 * g + 4 * h) = f32x4_t{y[4 * g], y[4 * g + 1], y[4 * g + 2], y[4 * g + 3]};
      }
    return;
  }
  if (P3) {
    if (qi >= p.n_q) return;
    uint16_t* odq = (uint16_t*)p.dq2 + qoff + (int64_t)qi * p.stride_qn;
    uint16_t* oddo = (uint16_t*)p.ddo + qoff + (int64_t)qi * p.stride_qn;
#pragma unroll
    for (int cb = 0; cb < NC; cb++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const f32x16_t& x = acc_dq[cb];
        const f32x16_t& y = acc_ddo[cb];
        *reinterpret_cast<u32x2_t*>(odq + 32 * cb + 8 * g + 4 * h) =
            pack4<F16>(x[4 * g] * p.scale, x[4 * g + 1] * p.scale, x[4 * g + 2] * p.scale, x[4 * g + 3] * p.scale);
        if (WITH_DDO) *reinterpret_cast<u32x2_t*>(oddo + 32 * cb + 8 * g + 4 * h) = pack4<F16>(y[4 * g], y[4 * g + 1], y[4 * g + 2], y[4 * g + 3]);
      }
    return;
  }
  red += __shfl_xor(red, 32);
  if (PASS == 1) red *= p.scale;
  if (PASS == 5) {
    red_dd += __shfl_xor(red_dd, 32);
    red_pdp += __shfl_xor(red_pdp, 32);
  }
  if (p.n_split > 1) {   // partial sums [split][dd | b | sum P dP][batch * n_q]; combine_stats finishes the pass
    if (h == 0 && qi < p.n_q) {
      const int64_t rows = (int64_t)p.batch * p.n_q;
      float* ps = p.part + (int64_t)split * 3 * rows + row;
      if (PASS == 1) ps[0] = red;
      if (PASS == 2) ps[rows] = red;
      if (PASS == 5) ps[0] = red_dd * p.scale, ps[rows] = red, ps[2 * rows] = red_pdp;
    }
    return;
  }
  if (PASS == 5) {
    const float dd_i = red_dd * p.scale;
    if (h == 0 && qi < p.n_q) {
      p.ws_dd[row] = dd_i;
      p.ws_b[row] = __builtin_fmaf(-dd_i, red_pdp, red);
    }
  } else {
    if (h == 0 && qi < p.n_q) (PASS == 1 ? p.ws_dd : p.ws_b)[row] = red;
    if (CHAIN) (PASS == 1 ? chain.dd : chain.b) = red;
  }
}

// SUB: 32-row tiles staged and consumed per barrier. SUB = 2 is a 64-row stage: one barrier, one round of staging
// issues and one set of stage addresses per two blocks (twice the LDS), for the head dim whose blocks are short.
template <bool F16, int D, int PASS, int MASK, int NW = 4, int SUB = 1>
__global__ void __launch_bounds__(64 * NW, NW == 8 ? 1 : 2) q_sweep_bf16(Params p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  // with a split, n_split consecutive "slices" share one (batch*head) slice and take its streamed tiles in turn
  int bh, tile, split = 0;
  if (!decode_block((p.n_q + 32 * NW - 1) / (32 * NW), p.batch * p.n_split, MASK != MASK_NONE, p.tile_major, bh, tile)) return;
  if (p.n_split > 1) split = bh % p.n_split, bh /= p.n_split;
  RowChain unused;
  q_sweep_run<F16, D, PASS, MASK, NW, SUB, false>(p, smem, bh, tile, split, unused);
}

// The reference's first kernel (bwdbwd_kernel_stage1, fhog/triton_bwdbwd.py:185-313) as it stands there: ONE launch
// whose workgroups run the dd sweep, the b sweep and the dQ2 / ddO sweep one after the other for their query tile, dd
// and b staying in registers in between. Same sweeps, same 25 products, two launches and two sets of resident loads
// fewer. For the head dim whose three sweeps have the same workgroup shape (d = 64: 128 queries, four waves).
template <bool F16, int D, int MASK>
__global__ void __launch_bounds__(256, 2) q_stage1_bf16(Params p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  int bh, tile;
  if (!decode_block((p.n_q + WG_ROWS - 1) / WG_ROWS, p.batch, MASK != MASK_NONE, p.tile_major, bh, tile)) return;
  RowChain chain;
  q_sweep_run<F16, D, 1, MASK, 4, 1, true>(p, smem, bh, tile, 0, chain);   // every sweep ends on a barrier: the ring is free
  q_sweep_run<F16, D, 2, MASK, 4, 1, true>(p, smem, bh, tile, 0, chain);
  q_sweep_run<F16, D, 3, MASK, 4, 1, true>(p, smem, bh, tile, 0, chain);
}

// ---- pass 1 with 64 stationary rows per wave -----------------------------------------------------------------------
// The dd sweep keeps only Q and ddQ resident, so a wave has the registers for TWO 32-query blocks (128 resident
// registers at d = 128, 64 for the two S-shaped accumulators of each block): every K or ddK operand read from LDS then
// feeds twice the MFMAs (16 reads per 48 instead of per 24), and a staged tile serves twice the rows.
// One 32-key step of such a wave; A0 / A1: the query block takes part (a block whose queries see no key of the tile
// is left out at compile time). P overwrites S in place.
template <bool F16, int D, bool A0, bool A1>
__device__ __forceinline__ void dd_block64(const char* stage, const int* aoff, const bf16x8_t (&Qb)[2][D / 16],
                                           const bf16x8_t (&ddQb)[2][D / 16], float c_scale_log2, const float* l_log2,
                                           const bool* masked, const int* lo, const int* hi, float* red) {
  constexpr int KK = D / 16, TILE = TS * 2 * D, NSTEP = 2 * KK, PF = 2, NB = PF + 1, EPK = 16 / KK;
  constexpr bool act[2] = {A0, A1};
  f32x16_t sc[2] = {{0}, {0}}, dds[2] = {{0}, {0}};
  bf16x8_t a[NB];
#pragma unroll
  for (int i = 0; i < PF; i++) a[i] = lds_read128(stage + (i / KK) * TILE, aoff[i % KK]);
#pragma unroll
  for (int i = 0; i < NSTEP; i++) {
    const int ph = i / KK, kk = i % KK, c = i % NB;
    if (i + PF < NSTEP) a[(i + PF) % NB] = lds_read128(stage + ((i + PF) / KK) * TILE, aoff[(i + PF) % KK]);
    __builtin_amdgcn_sched_barrier(0);
    if (ph == 0) {   // A = K: S += K Q^T, ddS += K ddQ^T
#pragma unroll
      for (int rb = 0; rb < 2; rb++)
        if (act[rb]) sc[rb] = mfma<F16>(a[c], Qb[rb][kk], sc[rb]);
#pragma unroll
      for (int rb = 0; rb < 2; rb++)
        if (act[rb]) dds[rb] = mfma<F16>(a[c], ddQb[rb][kk], dds[rb]);
    } else {         // A = ddK: ddS += ddK Q^T, and P = exp2(S c - L) behind the MFMAs
#pragma unroll
      for (int rb = 0; rb < 2; rb++)
        if (act[rb]) dds[rb] = mfma<F16>(a[c], Qb[rb][kk], dds[rb]);
#pragma unroll
      for (int rb = 0; rb < 2; rb++)
        if (act[rb]) {
#pragma unroll
          for (int r = EPK * kk; r < EPK * (kk + 1); r++) sc[rb][r] = __builtin_amdgcn_exp2f(sc[rb][r] * c_scale_log2 - l_log2[rb]);
        }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
#pragma unroll
  for (int rb = 0; rb < 2; rb++)
    if (act[rb]) {
      if (masked[rb]) {   // wave-uniform: the block holds hidden keys (mask edge or tensor end)
        keep_branch();
#pragma unroll
        for (int r = 0; r < 16; r++) sc[rb][r] = in_limits(r, lo[rb], hi[rb]) ? sc[rb][r] : 0.f;
      }
#pragma unroll
      for (int r = 0; r < 16; r++) red[rb] = __builtin_fmaf(sc[rb][r], dds[rb][r], red[rb]);   // scale applied once at the end
    }
}

// Four waves of 64 queries each: 256 queries per workgroup, two workgroups per CU. (Two-wave workgroups of 128 queries,
// four per CU, measured 20-40 % slower than these.)
template <bool F16, int D, int MASK>
__global__ void __launch_bounds__(256, 2) dd_sweep64_bf16(Params p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int ROWS = 256, NT = 2, TILE = TS * 2 * D, STAGE = NT * TILE, KK = D / 16;
  int bh, tile;
  if (!decode_block((p.n_q + ROWS - 1) / ROWS, p.batch, MASK != MASK_NONE, p.tile_major, bh, tile)) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, h = lane >> 5;
  const int q0 = tile * ROWS, qw = q0 + 64 * wave;
  const int64_t qoff = (int64_t)bh * p.stride_qb, koff = (int64_t)bh * p.stride_kb;
  const __bf16* src[NT] = {(const __bf16*)p.k + koff, (const __bf16*)p.ddk + koff};

  // the first streamed tile is requested before anything else is loaded: the round trips to memory overlap
  const StreamKeys<MASK> geo(p.mask_off, p.window, p.n_k);
  int j_begin, j_end;
  geo.tile_range(q0, ROWS, j_begin, j_end);
  Dma<D> dma;
  dma.init(p.stride_kn, wave, lane);
  const uint32_t ring_lds = lds_addr(smem);
  const auto stage_tile = [&](int j) {
    dma.template issue_all<NT>(ring_lds + (j & 1) * STAGE, TILE, src, (int64_t)j * TS * p.stride_kn, wave, p.n_k - j * TS);
  };
  if (j_begin < j_end) stage_tile(j_begin);

  // d_i = sum_c O_ic dO_ic for the sweeps behind this one (fhog/triton_bwdbwd.py:580), before the resident operands
  // are loaded: its operands are dead by then
  int qi[2];
  int64_t row[2];
  float l_log2[2];
#pragma unroll
  for (int rb = 0; rb < 2; rb++) {
    qi[rb] = qw + 32 * rb + n;
    const int qr = min(qi[rb], p.n_q - 1);  // queries past the end compute on a copy of the last row and store nothing
    row[rb] = (int64_t)bh * p.n_q + qr;
    bf16x8_t Ob[KK], dOb[KK];
    load_resident<D>(Ob, (const __bf16*)p.o + qoff, p.stride_qn, qr, h);
    load_resident<D>(dOb, (const __bf16*)p.dO + qoff, p.stride_qn, qr, h);
    float dsum = 0.f;
#pragma unroll
    for (int kk = 0; kk < KK; kk++)
#pragma unroll
      for (int e = 0; e < 8; e++) dsum = __builtin_fmaf(to_f32<F16>(Ob[kk][e]), to_f32<F16>(dOb[kk][e]), dsum);
    dsum += __shfl_xor(dsum, 32);
    if (h == 0 && qi[rb] < p.n_q) p.ws_d[row[rb]] = dsum;
    l_log2[rb] = p.lse[row[rb]] * kLog2e;
  }
  bf16x8_t Qb[2][KK], ddQb[2][KK];
#pragma unroll
  for (int rb = 0; rb < 2; rb++) {
    const int qr = min(qi[rb], p.n_q - 1);
    load_resident<D>(Qb[rb], (const __bf16*)p.q + qoff, p.stride_qn, qr, h);
    load_resident<D>(ddQb[rb], (const __bf16*)p.ddq + qoff, p.stride_qn, qr, h);
  }
  const float c_scale_log2 = p.scale * kLog2e;
  wait_vm0();   // the staging loads below are invisible to the compiler's wait counts (see q_sweep_bf16)

  int aoff[KK];
#pragma unroll
  for (int kk = 0; kk < KK; kk++) aoff[kk] = tile_off<D>(n, 2 * kk + h);
  dma_wait();
  __syncthreads();

  float red[2] = {0.f, 0.f};
  for (int j = j_begin; j < j_end; j++) {
    if (j + 1 < j_end) stage_tile(j + 1);
    const int k0 = j * TS;
    bool act[2], masked[2];
    int lo[2] = {0, 0}, hi[2] = {0, 0};   // key k0 + 8g + 4h + e is visible to the lane's query of block rb iff lo <= 8g + e <= hi
#pragma unroll
    for (int rb = 0; rb < 2; rb++) {
      act[rb] = !geo.dead(k0, qw + 32 * rb);
      masked[rb] = act[rb] && geo.partial(k0, qw + 32 * rb);
      if (masked[rb]) keep_branch(), geo.limits(k0, qi[rb], h, lo[rb], hi[rb]);
    }
    const char* stage = smem + (j & 1) * STAGE;
    if (act[0] && act[1]) dd_block64<F16, D, true, true>(stage, aoff, Qb, ddQb, c_scale_log2, l_log2, masked, lo, hi, red);
    else if (act[1]) dd_block64<F16, D, false, true>(stage, aoff, Qb, ddQb, c_scale_log2, l_log2, masked, lo, hi, red);
    else if (MASK == MASK_BAND && act[0]) dd_block64<F16, D, true, false>(stage, aoff, Qb, ddQb, c_scale_log2, l_log2, masked, lo, hi, red);
    dma_wait();
    __syncthreads();
  }
#pragma unroll
  for (int rb = 0; rb < 2; rb++) {
    float r = red[rb];
    r += __shfl_xor(r, 32);
    if (h == 0 && qi[rb] < p.n_q) p.ws_dd[row[rb]] = r * p.scale;
  }
}

// Pass 4 (dK2, dV2) at d = 64 as a single-role kernel: 256 threads = 4 waves own 128 keys (K, ddK, V, ddV rows in
// registers), Q-side tiles of 32 queries stream through a two-stage LDS ring together with the four row statistics of
// those queries. First-level products have the queries as M and the keys as N, so a lane owns one key and its
// accumulator registers run over the queries; rounded to 16 bits they are the B operands of the second-level
// products (contraction over the queries), whose A operands are transposing reads of the staged Q-side tiles.
// At d = 64 everything fits 256 registers, so no S-shaped tile passes through LDS.
// SUB: 32-query tiles staged and consumed per barrier (see q_sweep_bf16).
template <bool F16, int D, int MASK, int SUB = 1>
__global__ void __launch_bounds__(256, 2) k_sweep_bf16(Params p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int KK = D / 16, NC = D / 32, TILE = TS * 2 * D;
  constexpr int STAT = 4 * TS * 4;         // L log2(e), -d, dd, -(dd d + b) of the 32 staged queries
  constexpr int STAGE = 3 * TILE + STAT;   // Q, ddQ, dO tiles, statistics

  int bh, tile, split = 0;
  if (!decode_block((p.n_k + WG_ROWS - 1) / WG_ROWS, p.batch * p.n_split, false, p.tile_major, bh, tile)) return;
  if (p.n_split > 1) split = bh % p.n_split, bh /= p.n_split;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, h = lane >> 5;
  const int k0 = tile * WG_ROWS, kw = k0 + 32 * wave, kj = kw + n;
  const int kr = min(kj, p.n_k - 1);  // keys past the end compute on a copy of the last row and store nothing
  const int64_t qoff = (int64_t)bh * p.stride_qb, koff = (int64_t)bh * p.stride_kb;
  const __bf16* src[3] = {(const __bf16*)p.q + qoff, (const __bf16*)p.ddq + qoff, (const __bf16*)p.dO + qoff};
  const float* stat_src = p.lse;   // thread t < 128 carries statistic t / 32 of staged query t % 32
  if ((tid >> 5) == 1) stat_src = p.ws_d;
  if ((tid >> 5) == 2) stat_src = p.ws_dd;
  if ((tid >> 5) == 3) stat_src = p.ws_b;
  stat_src += (int64_t)bh * p.n_q;

  bf16x8_t Kb[KK], ddKb[KK], Vb[KK], ddVb[KK];
  load_resident<D>(Kb, (const __bf16*)p.k + koff, p.stride_kn, kr, h);
  load_resident<D>(ddKb, (const __bf16*)p.ddk + koff, p.stride_kn, kr, h);
  load_resident<D>(Vb, (const __bf16*)p.v + koff, p.stride_kn, kr, h);
  load_resident<D>(ddVb, (const __bf16*)p.ddv + koff, p.stride_kn, kr, h);
  const float c_scale_log2 = p.scale * kLog2e;

  int aoff[KK], troff[NC][2];
#pragma unroll
  for (int kk = 0; kk < KK; kk++) aoff[kk] = tile_off<D>(n, 2 * kk + h);
#pragma unroll
  for (int cb = 0; cb < NC; cb++) {
    troff[cb][0] = tr_lane_off_acc<D>(cb, 0, lane);
    troff[cb][1] = tr_lane_off_acc<D>(cb, 1, lane);
  }
  f32x16_t acc_dk[NC], acc_dv[NC];  // dK2^T, dV2^T: lane = key, registers = columns
#pragma unroll
  for (int cb = 0; cb < NC; cb++) {
    acc_dk[cb] = f32x16_t{0};
    acc_dv[cb] = f32x16_t{0};
  }
  const StreamQueries<MASK> geo(p.mask_off, p.window, p.n_q);
  int t_begin, t_end;  // query tiles that hold a query seeing some key of this workgroup
  geo.tile_range(k0, WG_ROWS, t_begin, t_end);
  if (p.n_split > 1) split_range(split, p.n_split, t_begin, t_end);
  Dma<D> dma;
  dma.init(p.stride_qn, wave, lane);
  const uint32_t ring_lds = lds_addr(smem);
  float stat_reg[SUB] = {}, stat_d[SUB] = {}, stat_dd[SUB] = {};   // one set per tile of a group
  // The statistic is loaded (a global, not generic, load) before the staging loads of a step and first touched at
  // the end of the step, so the wave never waits for it in between. Staged per query: L log2(e), -d, dd and
  // -(dd d + b), the values the accumulators of dP and E start from (the threads of the last group load d and dd too).
  auto load_stat = [&](int u, int q_base) {
    if (tid < 4 * TS) {
      const int q = min(q_base + (tid & (TS - 1)), p.n_q - 1);
      stat_reg[u] = *(global_f32_ptr)(stat_src + q);
      if (tid >= 3 * TS) {
        stat_d[u] = *(global_f32_ptr)(p.ws_d + (int64_t)bh * p.n_q + q);
        stat_dd[u] = *(global_f32_ptr)(p.ws_dd + (int64_t)bh * p.n_q + q);
      }
    }
  };
  auto store_stat = [&](int u, char* stage_base) {
    if (tid < 4 * TS) {
      const int g = tid / TS;
      reinterpret_cast<float*>(stage_base + 3 * TILE)[tid] =
          g == 0 ? stat_reg[u] * kLog2e : g == 1 ? -stat_reg[u] : g == 2 ? stat_reg[u] : -__builtin_fmaf(stat_dd[u], stat_d[u], stat_reg[u]);
    }
  };
  // the ring holds two groups of SUB tiles; tile j lives in slot (j - t_begin) mod (2 * SUB)
  const auto stage_tile = [&](int j) {
    const uint32_t dst = ring_lds + ((j - t_begin) & (2 * SUB - 1)) * STAGE;
    dma.template issue_all<3>(dst, TILE, src, (int64_t)j * TS * p.stride_qn, wave, p.n_q - j * TS);
  };
#pragma unroll
  for (int u = 0; u < SUB; u++)
    if (t_begin + u < t_end) {
      load_stat(u, (t_begin + u) * TS);
      stage_tile(t_begin + u);
    }
  if (t_begin < t_end) {
    wait_vm0();
#pragma unroll
    for (int u = 0; u < SUB; u++)
      if (t_begin + u < t_end) store_stat(u, smem + u * STAGE);
  }
  dma_wait();
  __syncthreads();

  for (int jj = t_begin; jj < t_end; jj += SUB) {
    const int grp = (jj - t_begin) & SUB;   // first ring slot of this group; the other group starts at grp ^ SUB
#pragma unroll
    for (int u = 0; u < SUB; u++)
      if (jj + SUB + u < t_end) {
        load_stat(u, (jj + SUB + u) * TS);
        stage_tile(jj + SUB + u);
      }
#pragma unroll
    for (int u = 0; u < SUB; u++) {
      const int j = jj + u;
      if (SUB > 1 && j >= t_end) continue;
      const int qb = j * TS;
      if (!geo.dead(qb, kw)) {  // else no query of the tile sees a key of this wave
        const char* stage = smem + (grp + u) * STAGE;
        const float* stat = reinterpret_cast<const float*>(stage + 3 * TILE);
        // five first-level products in one stream of KK k-steps; the three staged operands of step kk + 1 are
        // fetched before the MFMAs of step kk: S = Q K^T, ddS = ddQ K^T + Q ddK^T, dP = dO V^T, E = dO ddV^T
        // register 4g + i belongs to query qb + 8g + 4h + i: its statistics come from the staged arrays. The accumulators
        // of dP and E start at -d and -(dd d + b): u = dP - d and E' = E - dd d - b come straight from the matrix pipe.
        f32x16_t s = {0}, dds = {0}, dp, e;
#pragma unroll
        for (int g = 0; g < 4; g++) {
          const f32x4_t md4 = *reinterpret_cast<const f32x4_t*>(stat + 1 * TS + 8 * g + 4 * h);
          const f32x4_t mk4 = *reinterpret_cast<const f32x4_t*>(stat + 3 * TS + 8 * g + 4 * h);
#pragma unroll
          for (int i = 0; i < 4; i++) dp[4 * g + i] = md4[i], e[4 * g + i] = mk4[i];
        }
        bf16x8_t a[2][3];
#pragma unroll
        for (int x = 0; x < 3; x++) a[0][x] = lds_read128(stage + x * TILE, aoff[0]);
#pragma unroll
        for (int kk = 0; kk < KK; kk++) {
          const int c = kk & 1;
          if (kk + 1 < KK) {
#pragma unroll
            for (int x = 0; x < 3; x++) a[c ^ 1][x] = lds_read128(stage + x * TILE, aoff[kk + 1]);
          }
          __builtin_amdgcn_sched_barrier(0);
          s = mfma<F16>(a[c][0], Kb[kk], s);
          dds = mfma<F16>(a[c][1], Kb[kk], dds);
          dp = mfma<F16>(a[c][2], Vb[kk], dp);
          dds = mfma<F16>(a[c][0], ddKb[kk], dds);
          e = mfma<F16>(a[c][2], ddVb[kk], e);
          __builtin_amdgcn_sched_barrier(0);
        }
        f32x16_t pv;
#pragma unroll
        for (int g = 0; g < 4; g++) {
          const f32x4_t l4 = *reinterpret_cast<const f32x4_t*>(stat + 0 * TS + 8 * g + 4 * h);
#pragma unroll
          for (int i = 0; i < 4; i++) pv[4 * g + i] = __builtin_amdgcn_exp2f(s[4 * g + i] * c_scale_log2 - l4[i]);
        }
        if (geo.partial(qb, kw)) {  // wave-uniform: the block holds hidden (query, key) pairs (mask edge or tensor end)
          int lo, hi;                // query row 8g + 4h + i of the tile counts iff lo <= 8g + i <= hi
          geo.limits(qb, kj, h, lo, hi);
          keep_branch();
#pragma unroll
          for (int r = 0; r < 16; r++) pv[r] = in_limits(r, lo, hi) ? pv[r] : 0.f;
        }
        // dS -> s, dS' -> e, ddP -> dds (in place; scale on dS, dS' is applied to the accumulators at the end)
#pragma unroll
        for (int g = 0; g < 4; g++) {
          const f32x4_t dd4 = *reinterpret_cast<const f32x4_t*>(stat + 2 * TS + 8 * g + 4 * h);
#pragma unroll
          for (int i = 0; i < 4; i++) {
            const int r = 4 * g + i;
            const float pr = pv[r];
            dds[r] = pr * __builtin_fmaf(dds[r], p.scale, -dd4[i]);   // ddP = P (ddS - dd)
            s[r] = pr * dp[r];                                         // dS = P u
            e[r] = __builtin_fmaf(pr, e[r], dds[r] * dp[r]);           // dS' = P (E' + (ddS - dd) u)
          }
        }
        const bf16x8_t op_ds[2] = {pack_operand<F16>(s, 0), pack_operand<F16>(s, 1)};
        const bf16x8_t op_ds2[2] = {pack_operand<F16>(e, 0), pack_operand<F16>(e, 1)};
        const bf16x8_t op_ddp[2] = {pack_operand<F16>(dds, 0), pack_operand<F16>(dds, 1)};
        // dK2^T += ddQ^T dS + Q^T dS' ; dV2^T += dO^T ddP   (stage order Q, ddQ, dO)
        constexpr int NIT = 2 * NC;
        bf16x8_t ta[2][3];
#pragma unroll
        for (int x = 0; x < 3; x++) ta[0][x] = lds_read_tr_pre(stage + troff[0][0], stage + troff[0][1], x * TILE);
#pragma unroll
        for (int it = 0; it < NIT; it++) {
          const int t = it / NC, cb = it % NC, c = it & 1;
          if (it + 1 < NIT) {
            const int t1 = (it + 1) / NC, cb1 = (it + 1) % NC;
#pragma unroll
            for (int x = 0; x < 3; x++)
              ta[c ^ 1][x] = lds_read_tr_pre(stage + troff[cb1][0], stage + troff[cb1][1], x * TILE + t1 * 16 * 2 * D);
          }
          __builtin_amdgcn_sched_barrier(0);
          acc_dk[cb] = mfma<F16>(ta[c][1], op_ds[t], acc_dk[cb]);
          acc_dv[cb] = mfma<F16>(ta[c][2], op_ddp[t], acc_dv[cb]);
          acc_dk[cb] = mfma<F16>(ta[c][0], op_ds2[t], acc_dk[cb]);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    if (jj + SUB < t_end) {
      wait_vm0();
#pragma unroll
      for (int u = 0; u < SUB; u++)
        if (jj + SUB + u < t_end) store_stat(u, smem + ((grp ^ SUB) + u) * STAGE);
    }
    dma_wait();
    __syncthreads();
  }
  if (kj >= p.n_k) return;
  if (p.n_split > 1) {   // fp32 partial rows [split][dK2 | dV2][batch * n_k][D]
    const int64_t rows = (int64_t)p.batch * p.n_k;
    float* pk = p.part + ((int64_t)split * 2 * rows + (int64_t)bh * p.n_k + kj) * D;
    float* pv2 = pk + rows * D;
#pragma unroll
    for (int cb = 0; cb < NC; cb++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const f32x16_t& x = acc_dk[cb];
        const f32x16_t& y = acc_dv[cb];
        *reinterpret_cast<f32x4_t*>(pk + 32 * cb + 8 * g + 4 * h) = f32x4_t{x[4 * g], x[4 * g + 1], x[4 * g + 2], x[4 * g + 3]};
        *reinterpret_cast<f32x4_t*>(pv2 + 32 * cb + 8 * g + 4 * h) = f32x4_t{y[4 * g], y[4 * g + 1], y[4 * g + 2], y[4 * g + 3]};
      }
    return;
  }
  uint16_t* odk = (uint16_t*)p.dk2 + koff + (int64_t)kj * p.stride_kn;
  uint16_t* odv = (uint16_t*)p.dv2 + koff + (int64_t)kj * p.stride_kn;
#pragma unroll
  for (int cb = 0; cb < NC; cb++)
#pragma unroll
    for (int g = 0; g < 4; g++) {
      const f32x16_t& x = acc_dk[cb];
      const f32x16_t& y = acc_dv[cb];
      *reinterpret_cast<u32x2_t*>(odk + 32 * cb + 8 * g + 4 * h) =
          pack4<F16>(x[4 * g] * p.scale, x[4 * g + 1] * p.scale, x[4 * g + 2] * p.scale, x[4 * g + 3] * p.scale);
      *reinterpret_cast<u32x2_t*>(odv + 32 * cb + 8 * g + 4 * h) = pack4<F16>(y[4 * g], y[4 * g + 1], y[4 * g + 2], y[4 * g + 3]);
    }
}

template <auto Kernel>
hipError_t launch_sweep(unsigned grid, int smem, hipStream_t s, const Params& p, unsigned threads = 256) {
  const hipError_t e = allow_dynamic_lds<Kernel>(smem);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(Kernel, dim3(grid), dim3(threads), smem, s, p);
  return hipGetLastError();
}

template <bool F16, int D, int MASK>
hipError_t launch_single_d(const Params& p, int pass, hipStream_t s) {
  const int tile = TS * 2 * D, slices = p.batch * p.n_split;
  const unsigned gq = grid_blocks((p.n_q + WG_ROWS - 1) / WG_ROWS, slices);
  const unsigned gk = grid_blocks((p.n_k + WG_ROWS - 1) / WG_ROWS, slices);
  const bool split = p.n_split > 1;
  const int64_t rows_q = (int64_t)p.batch * p.n_q, rows_k = (int64_t)p.batch * p.n_k;
  hipError_t e;
  // Passes 2 and 5 with plenty of workgroups run 256 rows per workgroup (8 waves, one workgroup per CU): each staged
  // tile then serves twice the rows, i.e. half the staging loads per row (cfg2: pass 2 -7 %). Pass 1 (two tensors,
  // three workgroups per CU), d = 64 (measured slower or equal) and small launches keep 128 rows.
  const unsigned g8 = grid_blocks((p.n_q + 255) / 256, slices);
  if constexpr (D == 128) {
    const int b8 = tuning().b8;
    if (!split && (b8 < 0 ? g8 >= 512 : b8 == 1) && (pass == FHOG_PASS_B || pass == FHOG_PASS_DD_B)) {
      if (pass == FHOG_PASS_B) return launch_sweep<q_sweep_bf16<F16, D, 2, MASK, 8>>(g8, 2 * 4 * tile, s, p, 512);
      return launch_sweep<q_sweep_bf16<F16, D, 5, MASK, 8>>(g8, 2 * 4 * tile, s, p, 512);
    }
  }
  // Pass 1 at d = 128 with 64 queries per wave (256 per workgroup) once the launch has 2048 such workgroups (four rounds of
  // two per CU): half the LDS operand reads per MFMA, 4.7 % faster on 32 x 16384 rows. Smaller masked launches lose more
  // to the coarser balance than the reads gain (32 x 4096 rows: 512 workgroups, all resident at once, +9 %), and at
  // d = 64 the 32-query kernel with its three waves per SIMD is faster.
  if constexpr (D == 128) {
    const int dd64 = tuning().dd64;
    if (pass == FHOG_PASS_DD && !split && (dd64 < 0 ? g8 >= 2048 : dd64 == 1))
      return launch_sweep<dd_sweep64_bf16<F16, D, MASK>>(g8, 2 * 2 * tile, s, p, 256);
  }
  // d = 64: a block is half as long as at d = 128 while the work per barrier, staging issue and set of stage addresses
  // stays; FHOG_TUNE stage64=1 lets the sweeps stage and consume two 32-row tiles per barrier (SUB = 2, twice the LDS).
  // Off by default: it removes instructions and barriers, but kernel times stay within 1 % either way.
  constexpr int S2 = D == 64 ? 2 : 1;
  const bool two = D == 64 && tuning().stage64 != 0;
  switch (pass) {
    case FHOG_PASS_DD:
      e = two ? launch_sweep<q_sweep_bf16<F16, D, 1, MASK, 4, S2>>(gq, 2 * S2 * 2 * tile, s, p)
              : launch_sweep<q_sweep_bf16<F16, D, 1, MASK>>(gq, 2 * 2 * tile, s, p);
      if (e == hipSuccess && split) hipLaunchKernelGGL(combine_stats<1>, dim3((unsigned)((rows_q + 255) / 256)), dim3(256), 0, s, p);
      break;
    case FHOG_PASS_B:
      e = two ? launch_sweep<q_sweep_bf16<F16, D, 2, MASK, 4, S2>>(gq, 2 * S2 * 4 * tile, s, p)
              : launch_sweep<q_sweep_bf16<F16, D, 2, MASK>>(gq, 2 * 4 * tile, s, p);
      if (e == hipSuccess && split) hipLaunchKernelGGL(combine_stats<2>, dim3((unsigned)((rows_q + 255) / 256)), dim3(256), 0, s, p);
      break;
    case FHOG_PASS_DD_B:
      e = two ? launch_sweep<q_sweep_bf16<F16, D, 5, MASK, 4, S2>>(gq, 2 * S2 * 4 * tile, s, p)
              : launch_sweep<q_sweep_bf16<F16, D, 5, MASK>>(gq, 2 * 4 * tile, s, p);
      if (e == hipSuccess && split) hipLaunchKernelGGL(combine_stats<5>, dim3((unsigned)((rows_q + 255) / 256)), dim3(256), 0, s, p);
      break;
    case FHOG_PASS_DQ_DDO:
      if constexpr (D == 64) {
        e = two ? launch_sweep<q_sweep_bf16<F16, D, 3, MASK, 4, S2>>(gq, 2 * S2 * 4 * tile, s, p)
                : launch_sweep<q_sweep_bf16<F16, D, 3, MASK>>(gq, 2 * 4 * tile, s, p);
        if (e == hipSuccess && split)
          hipLaunchKernelGGL((combine_out<F16, D>), dim3((unsigned)((rows_q * (D / 4) + 255) / 256)), dim3(256), 0, s, p.part, p.n_split,
                             p.batch, p.n_q, p.stride_qb, p.stride_qn, (uint16_t*)p.dq2, (uint16_t*)p.ddo, p.scale);
      } else {
        return hipErrorInvalidValue;
      }
      break;
    case FHOG_PASS_STAGE1:
      if constexpr (D == 64) {
        if (split) return hipErrorInvalidValue;
        e = launch_sweep<q_stage1_bf16<F16, D, MASK>>(gq, 2 * 4 * tile, s, p);
      } else {
        return hipErrorInvalidValue;
      }
      break;
    case FHOG_PASS_DQ:
      if constexpr (D == 64) {
        e = two ? launch_sweep<q_sweep_bf16<F16, D, 7, MASK, 4, S2>>(gq, 2 * S2 * 4 * tile, s, p)
                : launch_sweep<q_sweep_bf16<F16, D, 7, MASK>>(gq, 2 * 4 * tile, s, p);
      } else {
        return hipErrorInvalidValue;
      }
      break;
    case FHOG_PASS_DK_DV:
      if constexpr (D == 64) {
        e = two ? launch_sweep<k_sweep_bf16<F16, D, MASK, S2>>(gk, 2 * S2 * (3 * tile + 4 * TS * 4), s, p)
                : launch_sweep<k_sweep_bf16<F16, D, MASK>>(gk, 2 * (3 * tile + 4 * TS * 4), s, p);
        if (e == hipSuccess && split)
          hipLaunchKernelGGL((combine_out<F16, D>), dim3((unsigned)((rows_k * (D / 4) + 255) / 256)), dim3(256), 0, s, p.part, p.n_split,
                             p.batch, p.n_k, p.stride_kb, p.stride_kn, (uint16_t*)p.dk2, (uint16_t*)p.dv2, p.scale);
      } else {
        return hipErrorInvalidValue;
      }
      break;
    default: return hipErrorInvalidValue;
  }
  return e != hipSuccess ? e : hipGetLastError();
}

}  // namespace

hipError_t launch_bf16_pc_pass(const Params& p, int pass, hipStream_t s);
hipError_t launch_bf16_ddo_pass(const Params& p, int pass, hipStream_t s);

bool bf16_shape_supported(int64_t n_q, int64_t n_k, int64_t d, int causal) {
  (void)causal;
  return (d == 64 || d == 128) && n_q >= 1 && n_k >= 1;
}

hipError_t launch_bf16_pass(const Params& p, int pass, hipStream_t s) {
  if (!bf16_shape_supported(p.n_q, p.n_k, p.d, p.causal)) return hipErrorInvalidValue;
  if (pass == FHOG_PASS_B_DDO || pass == FHOG_PASS_DD_B_DDO) return launch_bf16_ddo_pass(p, pass, s);
  if (pass == FHOG_PASS_DQ && p.d == 128) return launch_bf16_pc_pass(p, pass, s);
  // d = 128: passes 3 and 4 need the producer/consumer split to fit the registers; d = 64: single-role kernels throughout
  if (p.d == 128 && (pass == FHOG_PASS_DQ_DDO || pass == FHOG_PASS_DK_DV)) {
    const hipError_t e = launch_bf16_pc_pass(p, pass, s);
    if (e != hipSuccess || p.n_split == 1) return e;
    const bool kside = pass == FHOG_PASS_DK_DV;
    const int n = kside ? p.n_k : p.n_q;
    const dim3 grid((unsigned)(((int64_t)p.batch * n * (128 / 4) + 255) / 256));
    uint16_t* out0 = (uint16_t*)(kside ? p.dk2 : p.dq2);
    uint16_t* out1 = (uint16_t*)(kside ? p.dv2 : p.ddo);
    const int64_t sb = kside ? p.stride_kb : p.stride_qb, sn = kside ? p.stride_kn : p.stride_qn;
    if (p.f16) hipLaunchKernelGGL((combine_out<true, 128>), grid, dim3(256), 0, s, p.part, p.n_split, p.batch, n, sb, sn, out0, out1, p.scale);
    else hipLaunchKernelGGL((combine_out<false, 128>), grid, dim3(256), 0, s, p.part, p.n_split, p.batch, n, sb, sn, out0, out1, p.scale);
    return hipGetLastError();
  }
  if (pass != FHOG_PASS_STAGE1 && (pass < FHOG_PASS_DD || pass > FHOG_PASS_DQ || pass == FHOG_PASS_B_DDO)) return hipErrorInvalidValue;
  const int mask = mask_mode(p);
#define FHOG_SINGLE(F, DD)                                                             \
  (mask == MASK_NONE ? launch_single_d<F, DD, MASK_NONE>(p, pass, s)                   \
                     : mask == MASK_CAUSAL ? launch_single_d<F, DD, MASK_CAUSAL>(p, pass, s) : launch_single_d<F, DD, MASK_BAND>(p, pass, s))
  if (p.f16) return p.d == 128 ? FHOG_SINGLE(true, 128) : FHOG_SINGLE(true, 64);
  return p.d == 128 ? FHOG_SINGLE(false, 128) : FHOG_SINGLE(false, 64);
#undef FHOG_SINGLE
}

}  // namespace fhog
