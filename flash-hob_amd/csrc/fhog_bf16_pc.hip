// Passes 3 (dQ2, ddO) and 4 (dK2, dV2) of the 16-bit MFMA family at d = 128 as producer/consumer kernels (at d = 64 one
// wave holds everything and the single-role kernels of fhog_bf16.hip are faster).
//
// A workgroup is 512 threads = 8 wave64, two per SIMD, owning 128 stationary rows:
//   producers (4 waves, 32 stationary rows each): first-level products of one 32x32 block
//     (S, dP, ddS, dO ddV^T on MFMA), the softmax / dP' / dS / dS' / ddP arithmetic on the VALU,
//     and the hand-off of the bf16 S-shaped operands through LDS;
//   consumers (4 waves, same rows): the second-level products of the PREVIOUS block on MFMA
//     (4 contractions in pass 3, 3 in pass 4) into the fp32 output accumulators, plus all
//     global -> LDS staging of the streamed tiles.
// The consumer runs one block behind the producer, so the VALU-heavy end of the producer's block and the MFMAs of
// the consumer on the same SIMD can overlap; each wave fits 256 registers.
// One barrier per 32-row step. LDS: 3-stage ring of streamed tiles + double-buffered operand tiles.
#include "fhog_bf16_util.h"

namespace fhog {
using namespace bf16k;
namespace {

constexpr int PC_THREADS = 512;
constexpr int RING = 3;

template <int D, bool PASS4>
struct PCSmem {
  static constexpr int NT = PASS4 ? 3 : 4;      // streamed tensors per stage
  static constexpr int NSOP = PASS4 ? 3 : 4;    // operand tensors handed over per block
  static constexpr int TILE = TS * 2 * D;
  static constexpr int STAT = PASS4 ? 4 * TS * (int)sizeof(float) : 0;
  static constexpr int STAGE = NT * TILE + STAT;
  static constexpr int SOP_WAVE = NSOP * SOP_TILE;
  static constexpr int SOP_BUF = 4 * SOP_WAVE;
  static constexpr int SOP_BASE = RING * STAGE;
  static constexpr int TOTAL = SOP_BASE + 2 * SOP_BUF;
};

// ---- pass 3 ------------------------------------------------------------------------------------------
// One 32-key x 32-query block of pass 3 on a producer wave.
// The five first-level products are issued as a stream of 32 k-steps (8 each for K, V, ddK, ddV);
// the elementwise work of the block is cut into 2-element pieces that are placed right behind the
// MFMAs in the SAME wave's instruction stream, where they execute in the shadow of the matrix pipe
// (VALU work of another wave overlaps an MFMA only in part: both go through the SIMD's one vector issue port, and a
// pure-MFMA wave next to a pure-VALU wave of the same length takes 1.35x the time of either):
//   steps  0.. 7  A = K  : S += K Q^T, ddS += K ddQ^T
//   steps  8..15  A = V  : dP += V dO^T          + P = exp2(S c - L)
//   steps 16..23  A = ddK: ddS += ddK Q^T        + dS = P u
//   steps 24..31  A = ddV: E' += ddV dO^T        + w = ddS - dd, ddP = P w, z = ddP u
//   tail                                          dS' = P E' + z     [= P (E + dP (ddS - dd) - ddS d - b)]
// with u = dP - d and E' = E - (dd d + b) straight from the matrix pipe: the accumulators of dP and E start at the
// (per-lane) row constants -d and -(dd d + b) instead of zero.
// LDS operands are fetched PF steps ahead. Results go to the operand tiles dS, dS', ddP, P.

// registers 8t .. 8t+7 of one S-shaped tile, given as packed pairs pk[4t] .. pk[4t+3]: one ds_write_b128, so that the
// hand-off writes can be spread over the stream
__device__ __forceinline__ void sop_write_pk(char* tile, const uint32_t* pk, int t, int lane) {
  sop_write_step(tile, u32x4_t{pk[4 * t], pk[4 * t + 1], pk[4 * t + 2], pk[4 * t + 3]}, t, lane);
}

// KSIDE = false: pass 3 as described (stationary rows = queries: rs = Q, rdds = ddQ, rdp = re = dO; streamed K, V, ddK,
// ddV). KSIDE = true: pass 4 with the same stream: stationary rows = keys (rs = K, rdds = ddK, rdp = V, re = ddV),
// streamed Q, dO, ddQ, dO again; the resident operand goes first in the MFMA, so that a lane still owns one QUERY (a
// streamed row) and the row statistics stay per-lane scalars, reloaded for every tile; registers run over the keys.
// DQ_ONLY (pass 3 without its ddO half, FHOG_PASS_DQ): ddP and P are not handed over.
template <bool F16, int D, bool KSIDE, bool DQ_ONLY = false>
__device__ __forceinline__ void produce_q(const char* stage, char* sop, const bf16x8_t* rs, const bf16x8_t* rdds,
                                          const bf16x8_t* rdp, const bf16x8_t* re, int lane, int lo, int hi, bool mask,
                                          float c_scale_log2, float l_log2, float scale, float dsum, float dd, float b) {
  constexpr int TILE = TS * 2 * D;
  constexpr int KK = D / 16, NSTEP = 4 * KK, PF = 2, NB = PF + 1;
  const int n = lane & 31, h = lane >> 5;
  int aoff[KK];
#pragma unroll
  for (int kk = 0; kk < KK; kk++) aoff[kk] = tile_off<D>(n, 2 * kk + h);
  // stream order of the staged operands: K, V, ddK, ddV (stage order K, ddK, V, ddV) | Q, dO, ddQ, dO (stage order Q, ddQ, dO)
  constexpr int kTensorOfPhase[4] = {0, 2, 1, KSIDE ? 2 : 3};
  const auto mm = [](bf16x8_t staged, bf16x8_t resident, f32x16_t acc) {
    return KSIDE ? mfma<F16>(resident, staged, acc) : mfma<F16>(staged, resident, acc);
  };
  f32x16_t s = {0}, dds = {0}, dp, e, pv, z;   // dp holds u, e holds E'
  const float kc = __builtin_fmaf(dd, dsum, b);   // dS' = P (E + w u - kc) with u = dP - d, w = ddS - dd
#pragma unroll
  for (int r = 0; r < 16; r++) dp[r] = -dsum, e[r] = -kc;
  uint32_t pk_ds[8], pk_ds2[8], pk_ddp[8], pk_p[8];
  bf16x8_t a[NB];
#pragma unroll
  for (int i = 0; i < PF; i++) a[i] = lds_read128(stage + kTensorOfPhase[i / KK] * TILE, aoff[i % KK]);

  constexpr int EPK = 16 / KK;  // elements of the 16-register tiles handled per k-step (2 at d=128, 4 at d=64)
#pragma unroll
  for (int i = 0; i < NSTEP; i++) {
    const int ph = i / KK, kk = i % KK, c = i % NB;
    if (i + PF < NSTEP) a[(i + PF) % NB] = lds_read128(stage + kTensorOfPhase[(i + PF) / KK] * TILE, aoff[(i + PF) % KK]);
    __builtin_amdgcn_sched_barrier(0);
    if (ph == 0) {
      s = mm(a[c], rs[kk], s);
      dds = mm(a[c], rdds[kk], dds);
    } else if (ph == 1) {
      dp = mm(a[c], rdp[kk], dp);
#pragma unroll
      for (int r = EPK * kk; r < EPK * (kk + 1); r++) pv[r] = __builtin_amdgcn_exp2f(s[r] * c_scale_log2 - l_log2);
    } else if (ph == 2) {
      dds = mm(a[c], rs[kk], dds);
      if (kk == 0 && mask) {  // wave-uniform: the block holds hidden pairs (mask edge or end of a tensor)
        keep_branch();
#pragma unroll
        for (int r = 0; r < 16; r++) pv[r] = in_limits(r, lo, hi) ? pv[r] : 0.f;
      }
#pragma unroll
      for (int r = EPK * kk; r < EPK * (kk + 1); r += 2) pk_ds[r / 2] = pack2<F16>(pv[r] * dp[r], pv[r + 1] * dp[r + 1]);
      // the eight registers of a k-step are complete every 8 / EPK steps: hand them off right away, so that the
      // writes travel while the matrix pipe is busy instead of queueing up behind the consumers' reads at the end
      if ((EPK * (kk + 1)) % 8 == 0) sop_write_pk(sop + 0 * SOP_TILE, pk_ds, (EPK * kk) / 8, lane);
    } else {
      e = mm(a[c], re[kk], e);
#pragma unroll
      for (int r = EPK * kk; r < EPK * (kk + 1); r += 2) {
        const float ddp0 = pv[r] * __builtin_fmaf(dds[r], scale, -dd), ddp1 = pv[r + 1] * __builtin_fmaf(dds[r + 1], scale, -dd);
        if (!DQ_ONLY) pk_ddp[r / 2] = pack2<F16>(ddp0, ddp1);
        if (!DQ_ONLY && !KSIDE) pk_p[r / 2] = pack2<F16>(pv[r], pv[r + 1]);
        z[r] = ddp0 * dp[r];
        z[r + 1] = ddp1 * dp[r + 1];
      }
      if (!DQ_ONLY && (EPK * (kk + 1)) % 8 == 0) {
        sop_write_pk(sop + 2 * SOP_TILE, pk_ddp, (EPK * kk) / 8, lane);
        if (!KSIDE) sop_write_pk(sop + 3 * SOP_TILE, pk_p, (EPK * kk) / 8, lane);   // pass 4 has no use for P
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
#pragma unroll
  for (int r = 0; r < 16; r += 2)
    pk_ds2[r / 2] = pack2<F16>(__builtin_fmaf(pv[r], e[r], z[r]), __builtin_fmaf(pv[r + 1], e[r + 1], z[r + 1]));
  sop_write_pk(sop + 1 * SOP_TILE, pk_ds2, 0, lane);
  sop_write_pk(sop + 1 * SOP_TILE, pk_ds2, 1, lane);
}


// Consumer wave of pass 3: the second-level products of one output, OUT = 0: dQ2 = dS ddK + dS' K, OUT = 1:
// ddO = ddP V + P ddV, for the 64 queries of the pair qp = wq / 2 and all D columns (eight 32 x 32 accumulators). Per
// 32-key block it reads two of the four operand tiles of its two query blocks and two of the four staged tensors: each
// transposed K-side operand feeds two MFMAs (one per query block), each S-shaped operand D / 32 of them (one per column
// block), 24 KiB of LDS reads per block where a 64 x 64 block of BOTH outputs takes 32 KiB. The wave also issues the
// staging loads of its quarter of every tile.
template <bool F16, int D, int MASK, int OUT>
__device__ __forceinline__ void consume_q(const Params& p, char* smem, const StreamKeys<MASK>& geo, int j_begin, int j_end,
                                          int q0, int wq, int lane, int split, int bh) {
  using SM = PCSmem<D, false>;
  constexpr int NC = D / 32;
  // operand tiles: dS, dS', ddP, P; staged tensors: K, ddK, V, ddV
  constexpr int A0 = OUT ? 2 : 0, A1 = OUT ? 3 : 1, B0 = OUT ? 2 : 1, B1 = OUT ? 3 : 0;
  const int n = lane & 31, h = lane >> 5, qp = wq >> 1;
  const int64_t qoff = (int64_t)bh * p.stride_qb, koff = (int64_t)bh * p.stride_kb;
  const __bf16* src[4] = {(const __bf16*)p.k + koff, (const __bf16*)p.ddk + koff, (const __bf16*)p.v + koff,
                          (const __bf16*)p.ddv + koff};
  f32x16_t acc[2][NC];  // [query block of the pair][32-column block]
#pragma unroll
  for (int qb = 0; qb < 2; qb++)
#pragma unroll
    for (int cb = 0; cb < NC; cb++) acc[qb][cb] = f32x16_t{0};
  int troff[NC][2];
#pragma unroll
  for (int cb = 0; cb < NC; cb++) {
    troff[cb][0] = tr_lane_off_acc<D>(cb, 0, lane);
    troff[cb][1] = tr_lane_off_acc<D>(cb, 1, lane);
  }
  const int qw0 = q0 + 64 * qp;            // first query of the pair
  const char* sop_pair = smem + SM::SOP_BASE + (2 * qp) * SM::SOP_WAVE;
  Dma<D> dma;
  dma.init(p.stride_kn, wq, lane);
  const uint32_t ring_lds = lds_addr(smem);
  if (j_begin < j_end)
    dma.template issue_all<4>(ring_lds, SM::TILE, src, (int64_t)j_begin * TS * p.stride_kn, wq, p.n_k - j_begin * TS);
  dma_wait();
  __syncthreads();
  int sc = RING - 1, sn = 1;  // ring slots of tile j-1 (read here) and tile j+1 (filled here)
  for (int j = j_begin; j <= j_end; j++) {
    if (j + 1 < j_end) {
      const uint32_t dst = ring_lds + sn * SM::STAGE;
      const int64_t adv = (int64_t)(j + 1) * TS * p.stride_kn;
      dma.template issue_all<4>(dst, SM::TILE, src, adv, wq, p.n_k - (j + 1) * TS);
    }
    // block j-1: query block qb of the pair took part iff the tile held a key visible to it
    const bool act0 = j > j_begin && !geo.dead((j - 1) * TS, qw0);
    const bool act1 = j > j_begin && !geo.dead((j - 1) * TS, qw0 + 32);
    const bool act = act0 || act1;
    const char* stage = smem + sc * SM::STAGE;
    const char* sop = sop_pair + ((j - 1) & 1) * SM::SOP_BUF;
    // two column blocks per iteration (k-step t, column pair cp): the four MFMAs on one accumulator are four instructions apart
    constexpr int NIT = 2 * (NC / 2);
    bf16x8_t bop[2][2][2];   // [buffer][column block of the pair][product]
    bf16x8_t a_op[2][2][2];  // [k-step][query block][product]
    const auto read_b = [&](int buf, int it) {
      const int t = it / (NC / 2), cp = it % (NC / 2);
#pragma unroll
      for (int cl = 0; cl < 2; cl++) {
        const char* b0 = stage + troff[2 * cp + cl][0];
        const char* b1 = stage + troff[2 * cp + cl][1];
        bop[buf][cl][0] = lds_read_tr_pre(b0, b1, B0 * SM::TILE + t * 16 * 2 * D);
        bop[buf][cl][1] = lds_read_tr_pre(b0, b1, B1 * SM::TILE + t * 16 * 2 * D);
      }
    };
    if (act) {
      read_b(0, 0);
#pragma unroll
      for (int t = 0; t < 2; t++)
#pragma unroll
        for (int qb = 0; qb < 2; qb++) {
          a_op[t][qb][0] = sop_read(sop + qb * SM::SOP_WAVE + A0 * SOP_TILE, t, lane);
          a_op[t][qb][1] = sop_read(sop + qb * SM::SOP_WAVE + A1 * SOP_TILE, t, lane);
        }
#pragma unroll
      for (int it = 0; it < NIT; it++) {
        const int t = it / (NC / 2), cp = it % (NC / 2), c = it & 1;
        if (it + 1 < NIT) read_b(c ^ 1, it + 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int pr = 0; pr < 2; pr++)
#pragma unroll
          for (int cl = 0; cl < 2; cl++) {
            if (act0) acc[0][2 * cp + cl] = mfma<F16>(a_op[t][0][pr], bop[c][cl][pr], acc[0][2 * cp + cl]);
            // with a plain causal mask (or none) a tile that block 0 takes part in is also one for block 1
            if (MASK != MASK_BAND || act1) acc[1][2 * cp + cl] = mfma<F16>(a_op[t][1][pr], bop[c][cl][pr], acc[1][2 * cp + cl]);
          }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    dma_wait();
    __syncthreads();
    sc = (sc == RING - 1) ? 0 : sc + 1;
    sn = (sn == RING - 1) ? 0 : sn + 1;
  }
  // acc[qb][cb][r] holds (query qw0 + 32 qb + 8*(r/4) + 4h + r%4, column 32 cb + n)
  if (p.n_split > 1) {   // fp32 partial rows [split][dQ2 | ddO][batch * n_q][D]; combine_out finishes the pass
    const int64_t rows = (int64_t)p.batch * p.n_q;
    float* pq = p.part + ((int64_t)split * 2 * rows + (OUT ? rows : 0) + (int64_t)bh * p.n_q) * D;
#pragma unroll
    for (int qb = 0; qb < 2; qb++)
#pragma unroll
      for (int cb = 0; cb < NC; cb++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int qrow = qw0 + 32 * qb + 8 * (r / 4) + 4 * h + (r % 4);
          if (qrow < p.n_q) pq[(int64_t)qrow * D + 32 * cb + n] = acc[qb][cb][r];
        }
    return;
  }
  uint16_t* o = (uint16_t*)(OUT ? p.ddo : p.dq2) + qoff;
  const float f = OUT ? 1.f : p.scale;
#pragma unroll
  for (int qb = 0; qb < 2; qb++)
#pragma unroll
    for (int cb = 0; cb < NC; cb++)
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int qrow = qw0 + 32 * qb + 8 * (r / 4) + 4 * h + (r % 4);
        if (qrow < p.n_q) o[(int64_t)qrow * p.stride_qn + 32 * cb + n] = to_elem<F16>(acc[qb][cb][r] * f);
      }
}

// Consumer wave of the dQ2-only sweep (FHOG_PASS_DQ): dQ2 = dS ddK + dS' K for the 32 queries of producer wave wq and
// all D columns (D / 32 accumulators), from the operand tiles dS, dS' of that producer and the staged K and ddK.
template <bool F16, int D, int MASK>
__device__ __forceinline__ void consume_dq(const Params& p, char* smem, const StreamKeys<MASK>& geo, int j_begin, int j_end,
                                           int q0, int wq, int lane, int bh) {
  using SM = PCSmem<D, false>;
  constexpr int NC = D / 32, NP = NC / 2, NIT = 2 * NP;
  const int n = lane & 31, h = lane >> 5;
  const int64_t qoff = (int64_t)bh * p.stride_qb, koff = (int64_t)bh * p.stride_kb;
  const __bf16* src[4] = {(const __bf16*)p.k + koff, (const __bf16*)p.ddk + koff, (const __bf16*)p.v + koff,
                          (const __bf16*)p.ddv + koff};
  f32x16_t acc[NC];
  int troff[NC][2];
#pragma unroll
  for (int cb = 0; cb < NC; cb++) {
    acc[cb] = f32x16_t{0};
    troff[cb][0] = tr_lane_off_acc<D>(cb, 0, lane);
    troff[cb][1] = tr_lane_off_acc<D>(cb, 1, lane);
  }
  const int qw0 = q0 + 32 * wq;
  const char* sop_wave = smem + SM::SOP_BASE + wq * SM::SOP_WAVE;
  Dma<D> dma;
  dma.init(p.stride_kn, wq, lane);
  const uint32_t ring_lds = lds_addr(smem);
  if (j_begin < j_end)
    dma.template issue_all<4>(ring_lds, SM::TILE, src, (int64_t)j_begin * TS * p.stride_kn, wq, p.n_k - j_begin * TS);
  dma_wait();
  __syncthreads();
  int sc = RING - 1, sn = 1;  // ring slots of tile j-1 (read here) and tile j+1 (filled here)
  for (int j = j_begin; j <= j_end; j++) {
    if (j + 1 < j_end) {
      const uint32_t dst = ring_lds + sn * SM::STAGE;
      dma.template issue_all<4>(dst, SM::TILE, src, (int64_t)(j + 1) * TS * p.stride_kn, wq, p.n_k - (j + 1) * TS);
    }
    if (j > j_begin && !geo.dead((j - 1) * TS, qw0)) {   // block j-1 took part
      const char* stage = smem + sc * SM::STAGE;
      const char* sop = sop_wave + ((j - 1) & 1) * SM::SOP_BUF;
      bf16x8_t bop[2][2][2];   // [buffer][column block of the pair][ddK | K]
      bf16x8_t a_op[2][2];     // [k-step][dS | dS']
      const auto read_b = [&](int buf, int it) {
        const int t = it / NP, cp = it % NP;
#pragma unroll
        for (int cl = 0; cl < 2; cl++) {
          const char* b0 = stage + troff[2 * cp + cl][0];
          const char* b1 = stage + troff[2 * cp + cl][1];
          bop[buf][cl][0] = lds_read_tr_pre(b0, b1, 1 * SM::TILE + t * 16 * 2 * D);
          bop[buf][cl][1] = lds_read_tr_pre(b0, b1, 0 * SM::TILE + t * 16 * 2 * D);
        }
      };
      read_b(0, 0);
#pragma unroll
      for (int t = 0; t < 2; t++) {
        a_op[t][0] = sop_read(sop + 0 * SOP_TILE, t, lane);
        a_op[t][1] = sop_read(sop + 1 * SOP_TILE, t, lane);
      }
#pragma unroll
      for (int it = 0; it < NIT; it++) {
        const int t = it / NP, cp = it % NP, c = it & 1;
        if (it + 1 < NIT) read_b(c ^ 1, it + 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int pr = 0; pr < 2; pr++)
#pragma unroll
          for (int cl = 0; cl < 2; cl++) acc[2 * cp + cl] = mfma<F16>(a_op[t][pr], bop[c][cl][pr], acc[2 * cp + cl]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    dma_wait();
    __syncthreads();
    sc = (sc == RING - 1) ? 0 : sc + 1;
    sn = (sn == RING - 1) ? 0 : sn + 1;
  }
  // acc[cb][r] holds (query qw0 + 8*(r/4) + 4h + r%4, column 32 cb + n)
  uint16_t* o = (uint16_t*)p.dq2 + qoff;
#pragma unroll
  for (int cb = 0; cb < NC; cb++)
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int qrow = qw0 + 8 * (r / 4) + 4 * h + (r % 4);
      if (qrow < p.n_q) o[(int64_t)qrow * p.stride_qn + 32 * cb + n] = to_elem<F16>(acc[cb][r] * p.scale);
    }
}

template <bool F16, int D, int MASK, bool DQ_ONLY = false>
__global__ void __launch_bounds__(PC_THREADS) q_sweep3_pc(Params p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  using SM = PCSmem<D, false>;
  constexpr int NC = D / 32;

  // with a split, n_split consecutive "slices" share one (batch*head) slice and take its streamed tiles in turn
  int bh, tile, split = 0;
  if (!decode_block((p.n_q + WG_ROWS - 1) / WG_ROWS, p.batch * p.n_split, MASK != MASK_NONE, p.tile_major, bh, tile)) return;
  if (p.n_split > 1) split = bh % p.n_split, bh /= p.n_split;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: lets the compiler branch on scalars
  const bool producer = wave < 4;
  const int wq = wave & 3;
  const int n = lane & 31, h = lane >> 5;
  const int q0 = tile * WG_ROWS, qw = q0 + 32 * wq, qi = qw + n;
  const int64_t qoff = (int64_t)bh * p.stride_qb, koff = (int64_t)bh * p.stride_kb;
  const StreamKeys<MASK> geo(p.mask_off, p.window, p.n_k);
  int j_begin, j_end;  // key tiles this workgroup visits
  geo.tile_range(q0, WG_ROWS, j_begin, j_end);
  if (p.n_split > 1) split_range(split, p.n_split, j_begin, j_end);
  char* sop_base = smem + SM::SOP_BASE + wq * SM::SOP_WAVE;

  if (producer) {
    bf16x8_t Qb[D / 16], ddQb[D / 16], dOb[D / 16];
    const int qr = min(qi, p.n_q - 1);  // queries past the end compute on a copy of the last row; nothing of them is stored
    load_resident<D>(Qb, (const __bf16*)p.q + qoff, p.stride_qn, qr, h);
    load_resident<D>(ddQb, (const __bf16*)p.ddq + qoff, p.stride_qn, qr, h);
    load_resident<D>(dOb, (const __bf16*)p.dO + qoff, p.stride_qn, qr, h);
    const int64_t row = (int64_t)bh * p.n_q + qr;
    const float l_log2 = p.lse[row] * kLog2e;
    const float c_scale_log2 = p.scale * kLog2e;
    const float dsum = p.ws_d[row], dd = p.ws_dd[row], b = p.ws_b[row];
    __syncthreads();
    int sp = 0;  // ring slot of tile j
    for (int j = j_begin; j <= j_end; j++) {
      const int k0 = j * TS;
      if (j < j_end && !geo.dead(k0, qw)) {
        const char* stage = smem + sp * SM::STAGE;
        char* sop = sop_base + (j & 1) * SM::SOP_BUF;
        const bool masked = geo.partial(k0, qw);
        int lo = 0, hi = 0;  // key k0 + 8g + 4h + e is visible iff lo <= 8g + e <= hi
        if (masked) keep_branch(), geo.limits(k0, qi, h, lo, hi);
        produce_q<F16, D, false, DQ_ONLY>(stage, sop, Qb, ddQb, dOb, dOb, lane, lo, hi, masked, c_scale_log2, l_log2, p.scale, dsum, dd, b);
      }
      __syncthreads();
      sp = (sp == RING - 1) ? 0 : sp + 1;
    }
  } else {
    // dQ2 alone: consumer wave wq owns the 32 queries of producer wave wq
    if (DQ_ONLY) consume_dq<F16, D, MASK>(p, smem, geo, j_begin, j_end, q0, wq, lane, bh);
    // consumer wave (qp, out) owns the 64-query x D-column block of ONE output for the query pair qp
    else if (wq & 1) consume_q<F16, D, MASK, 1>(p, smem, geo, j_begin, j_end, q0, wq, lane, split, bh);
    else consume_q<F16, D, MASK, 0>(p, smem, geo, j_begin, j_end, q0, wq, lane, split, bh);
  }
}

// ---- pass 4 ------------------------------------------------------------------------------------------
// The producers run the pass 3 stream with the roles of the two sides exchanged (produce_q<KSIDE = true>): a lane
// owns a staged query, its registers run over the wave's 32 keys. The operand tiles therefore hold rows = queries,
// columns = keys, and the consumer, which contracts over the queries, reads them with transposing loads.
// Per-lane part of the address of such a read: lane (key = lane % 32, h = lane / 32) receives, for k-step t, the queries
// 16t + 4h + 0..3 (s = 0) and 16t + 8 + 4h + 0..3 (s = 1) at column `key`, the order tr_lane_off_acc gives the
// staged Q-side tiles. Within a 16-lane group lane i addresses query row (i >> 2) and the four keys 4 (i & 3) .. + 3,
// which the tile keeps in chunk 2b + (cg & 1), half cg >> 1 (b = key / 16, cg = i & 3).
__device__ __forceinline__ int sop_tr_lane_off(int s, int lane) {
  const int i = lane & 15, b = (lane >> 4) & 1, h = lane >> 5, cg = i & 3;
  const int r = 8 * s + 4 * h + (i >> 2);
  return r * 64 + (((2 * b + (cg & 1)) ^ sop_swz(r)) << 4) + 8 * (cg >> 1);
}

template <bool F16, int D, int MASK>
__global__ void __launch_bounds__(PC_THREADS) k_sweep_pc(Params p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  using SM = PCSmem<D, true>;
  constexpr int NC = D / 32;

  int bh, tile, split = 0;
  if (!decode_block((p.n_k + WG_ROWS - 1) / WG_ROWS, p.batch * p.n_split, false, p.tile_major, bh, tile)) return;
  if (p.n_split > 1) split = bh % p.n_split, bh /= p.n_split;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: lets the compiler branch on scalars
  const bool producer = wave < 4;
  const int wq = wave & 3;
  const int n = lane & 31, h = lane >> 5;
  const int k0 = tile * WG_ROWS, kw = k0 + 32 * wq, kj = kw + n;
  const int kr = min(kj, p.n_k - 1);  // keys past the end compute on a copy of the last row; nothing of them is stored
  const int64_t qoff = (int64_t)bh * p.stride_qb, koff = (int64_t)bh * p.stride_kb;
  const StreamQueries<MASK> geo(p.mask_off, p.window, p.n_q);
  int t_begin, t_end;  // query tiles that hold a query seeing some key of this workgroup
  geo.tile_range(k0, WG_ROWS, t_begin, t_end);
  if (p.n_split > 1) split_range(split, p.n_split, t_begin, t_end);
  char* sop_base = smem + SM::SOP_BASE + wq * SM::SOP_WAVE;

  if (producer) {
    bf16x8_t Kb[D / 16], ddKb[D / 16], Vb[D / 16], ddVb[D / 16];
    load_resident<D>(Kb, (const __bf16*)p.k + koff, p.stride_kn, kr, h);
    load_resident<D>(ddKb, (const __bf16*)p.ddk + koff, p.stride_kn, kr, h);
    load_resident<D>(Vb, (const __bf16*)p.v + koff, p.stride_kn, kr, h);
    load_resident<D>(ddVb, (const __bf16*)p.ddv + koff, p.stride_kn, kr, h);
    const float c_scale_log2 = p.scale * kLog2e;
    const StreamKeys<MASK> kgeo(p.mask_off, p.window, p.n_k);
    __syncthreads();
    int sp = 0;  // ring slot of tile j (slot 0 holds tile t_begin)
    for (int j = t_begin; j <= t_end; j++) {
      const int qb = j * TS;
      if (j < t_end && !geo.dead(qb, kw)) {
        const char* stage = smem + sp * SM::STAGE;
        char* sop = sop_base + (j & 1) * SM::SOP_BUF;
        const bool masked = geo.partial(qb, kw);
        const int qi = qb + n;   // the lane's query
        int lo = 0, hi = 0;      // key kw + 8g + 4h + e counts for it iff lo <= 8g + e <= hi
        if (masked) {
          keep_branch();
          kgeo.limits(kw, qi, h, lo, hi);
          if (qi >= p.n_q) hi = -2 * TS;   // a row past the end of the tensor (a copy of its last row)
        }
        const float* stat = reinterpret_cast<const float*>(stage + 3 * SM::TILE);
        produce_q<F16, D, true>(stage, sop, Kb, ddKb, Vb, ddVb, lane, lo, hi, masked, c_scale_log2, stat[n], p.scale,
                                stat[TS + n], stat[2 * TS + n], stat[3 * TS + n]);
      }
      __syncthreads();
      sp = (sp == RING - 1) ? 0 : sp + 1;
    }
  } else {
    const int ctid = tid - 256;
    const __bf16* src[3] = {(const __bf16*)p.q + qoff, (const __bf16*)p.ddq + qoff, (const __bf16*)p.dO + qoff};
    const float* stat_src[4] = {p.lse + (int64_t)bh * p.n_q, p.ws_d + (int64_t)bh * p.n_q, p.ws_dd + (int64_t)bh * p.n_q,
                                p.ws_b + (int64_t)bh * p.n_q};
    // consumer wave (kp, ch) owns the keys of the producer waves 2 kp and 2 kp + 1 and the column half ch of both outputs
    // (eight 32 x 32 accumulators): every transposed Q-side operand read from LDS feeds the MFMAs of two key blocks, every
    // S-shaped operand those of two column blocks - 24 KiB of LDS reads per block where one key block with all columns
    // takes 30 KiB
    constexpr int NCL = NC / 2;   // 32-column blocks per consumer wave
    const int kp = wq >> 1, ch = wq & 1;
    const int kw2 = k0 + 64 * kp;   // first key of the pair
    f32x16_t acc_dk[2][NCL], acc_dv[2][NCL];   // [key block of the pair][column block of the half]
#pragma unroll
    for (int kb = 0; kb < 2; kb++)
#pragma unroll
      for (int cl = 0; cl < NCL; cl++) {
        acc_dk[kb][cl] = f32x16_t{0};
        acc_dv[kb][cl] = f32x16_t{0};
      }
    int troff[NCL][2];
#pragma unroll
    for (int cl = 0; cl < NCL; cl++) {
      troff[cl][0] = tr_lane_off_acc<D>(NCL * ch + cl, 0, lane);
      troff[cl][1] = tr_lane_off_acc<D>(NCL * ch + cl, 1, lane);
    }
    const char* sop_pair = smem + SM::SOP_BASE + (2 * kp) * SM::SOP_WAVE;
    const int sopoff[2] = {sop_tr_lane_off(0, lane), sop_tr_lane_off(1, lane)};
    Dma<D> dma;
    dma.init(p.stride_qn, wq, lane);
    const uint32_t ring_lds = lds_addr(smem);
    float stat_reg = 0.f;  // consumer threads 0..127: one statistic value of the staged tile
    // A global (not generic) load, so that it does not tie up the LDS wait counter; issued before the staging
    // loads of the step, so that reusing its destination register never waits for those.
    // The loaded value is first touched in store_stat, at the end of the step: a use right after the load would
    // make the wave wait there for the load and, with it, for every staging load issued before it.
    auto load_stat = [&](int q_base) {
      if (ctid < 4 * TS) stat_reg = *(global_f32_ptr)(stat_src[ctid / TS] + min(q_base + (ctid % TS), p.n_q - 1));
    };
    auto store_stat = [&](char* stage_base) {
      if (ctid < 4 * TS) reinterpret_cast<float*>(stage_base + 3 * SM::TILE)[ctid] = (ctid < TS) ? stat_reg * kLog2e : stat_reg;
    };
    if (t_begin < t_end) {
      const int64_t adv = (int64_t)t_begin * TS * p.stride_qn;
      dma.template issue_all<3>(ring_lds, SM::TILE, src, adv, wq, p.n_q - t_begin * TS);
      load_stat(t_begin * TS);
      store_stat(smem);
    }
    dma_wait();
    __syncthreads();
    int sc = RING - 1, sn = 1;  // ring slots of tile j-1 (read here) and tile j+1 (filled here)
    for (int j = t_begin; j <= t_end; j++) {
      if (j + 1 < t_end) {
        const uint32_t dst = ring_lds + sn * SM::STAGE;
        const int64_t adv = (int64_t)(j + 1) * TS * p.stride_qn;
        load_stat((j + 1) * TS);
        dma.template issue_all<3>(dst, SM::TILE, src, adv, wq, p.n_q - (j + 1) * TS);
      }
      // block j-1: key block kb of the pair took part iff the tile held a query that sees one of its keys
      const bool act0 = j > t_begin && !geo.dead((j - 1) * TS, kw2);
      const bool act1 = j > t_begin && !geo.dead((j - 1) * TS, kw2 + 32);
      if (act0 || act1) {
        const char* stage = smem + sc * SM::STAGE;
        const char* sop = sop_pair + ((j - 1) & 1) * SM::SOP_BUF;
        const char* bp[NCL][2];
#pragma unroll
        for (int cl = 0; cl < NCL; cl++) {
          bp[cl][0] = stage + troff[cl][0];
          bp[cl][1] = stage + troff[cl][1];
        }
        // operand tiles: dS, dS', ddP; staged tensors: Q, ddQ, dO.  dK2^T += ddQ^T dS + Q^T dS' ; dV2^T += dO^T ddP
        bf16x8_t bop[2][3];
        bop[0][0] = lds_read_tr_pre(bp[0][0], bp[0][1], 1 * SM::TILE + 0 * 16 * 2 * D);
        bop[0][1] = lds_read_tr_pre(bp[0][0], bp[0][1], 0 * SM::TILE + 0 * 16 * 2 * D);
        bop[0][2] = lds_read_tr_pre(bp[0][0], bp[0][1], 2 * SM::TILE + 0 * 16 * 2 * D);
        bf16x8_t a_op[2][2][3];   // [key block][k-step][tile]
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
          for (int t = 0; t < 2; t++)
#pragma unroll
            for (int x = 0; x < 3; x++)
              a_op[kb][t][x] = lds_read_tr_pre(sop + kb * SM::SOP_WAVE + sopoff[0], sop + kb * SM::SOP_WAVE + sopoff[1], x * SOP_TILE + t * 16 * 64);
#pragma unroll
        for (int it = 0; it < 2 * NCL; it++) {
          const int t = it / NCL, cl = it % NCL, c = it & 1;
          if (it + 1 < 2 * NCL) {
            const int t1 = (it + 1) / NCL, cl1 = (it + 1) % NCL;
            bop[c ^ 1][0] = lds_read_tr_pre(bp[cl1][0], bp[cl1][1], 1 * SM::TILE + t1 * 16 * 2 * D);
            bop[c ^ 1][1] = lds_read_tr_pre(bp[cl1][0], bp[cl1][1], 0 * SM::TILE + t1 * 16 * 2 * D);
            bop[c ^ 1][2] = lds_read_tr_pre(bp[cl1][0], bp[cl1][1], 2 * SM::TILE + t1 * 16 * 2 * D);
          }
          __builtin_amdgcn_sched_barrier(0);
          if (act0) {
            acc_dk[0][cl] = mfma<F16>(a_op[0][t][0], bop[c][0], acc_dk[0][cl]);
            acc_dv[0][cl] = mfma<F16>(a_op[0][t][2], bop[c][2], acc_dv[0][cl]);
          }
          if (act1) {
            acc_dk[1][cl] = mfma<F16>(a_op[1][t][0], bop[c][0], acc_dk[1][cl]);
            acc_dv[1][cl] = mfma<F16>(a_op[1][t][2], bop[c][2], acc_dv[1][cl]);
          }
          if (act0) acc_dk[0][cl] = mfma<F16>(a_op[0][t][1], bop[c][1], acc_dk[0][cl]);
          if (act1) acc_dk[1][cl] = mfma<F16>(a_op[1][t][1], bop[c][1], acc_dk[1][cl]);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      if (j + 1 < t_end) store_stat(smem + sn * SM::STAGE);
      dma_wait();
      __syncthreads();
      sc = (sc == RING - 1) ? 0 : sc + 1;
      sn = (sn == RING - 1) ? 0 : sn + 1;
    }
    // acc[kb][cl][r] holds (key kw2 + 32 kb + 8*(r/4) + 4h + r%4, column 32 (NCL ch + cl) + n)
    if (p.n_split > 1) {   // fp32 partial rows [split][dK2 | dV2][batch * n_k][D]
      const int64_t rows = (int64_t)p.batch * p.n_k;
      float* pk = p.part + ((int64_t)split * 2 * rows + (int64_t)bh * p.n_k) * D;
#pragma unroll
      for (int kb = 0; kb < 2; kb++)
#pragma unroll
        for (int cl = 0; cl < NCL; cl++)
#pragma unroll
          for (int r = 0; r < 16; r++) {
            const int krow = kw2 + 32 * kb + 8 * (r / 4) + 4 * h + (r % 4);
            if (krow < p.n_k) {
              const int64_t o = (int64_t)krow * D + 32 * (NCL * ch + cl) + n;
              pk[o] = acc_dk[kb][cl][r];
              pk[rows * D + o] = acc_dv[kb][cl][r];
            }
          }
      return;
    }
    uint16_t* odk = (uint16_t*)p.dk2 + koff;
    uint16_t* odv = (uint16_t*)p.dv2 + koff;
#pragma unroll
    for (int kb = 0; kb < 2; kb++)
#pragma unroll
      for (int cl = 0; cl < NCL; cl++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int krow = kw2 + 32 * kb + 8 * (r / 4) + 4 * h + (r % 4);
          if (krow < p.n_k) {
            const int64_t o = (int64_t)krow * p.stride_kn + 32 * (NCL * ch + cl) + n;
            odk[o] = to_elem<F16>(acc_dk[kb][cl][r] * p.scale);
            odv[o] = to_elem<F16>(acc_dv[kb][cl][r]);
          }
        }
  }
}

// ---- first-order backward, K-tiled (dK, dV) at d = 128 -------------------------------------------------------------
// The arithmetic of fhog/triton_flash.py:201-220 for one key tile, as a producer/consumer kernel of the same shape as
// pass 4: a single wave does not hold two 32 x 128 fp32 accumulators, two resident tensors and the S-shaped tiles in 256
// registers (the single-role kernel of fhog_attn.hip keeps 24-37 registers per lane in scratch memory at d = 128).
//   producers: S = K Q^T, dP = V dO^T (resident operand first: a lane owns one staged query), P = exp2(S c - L),
//              dS = P (dP - d); operand tiles dS, P
//   consumers: dK^T += dS^T Q, dV^T += P^T dO from transposing reads of the operand and the staged tiles
template <int D>
struct PCSmemAttn {
  static constexpr int NT = 2;      // streamed tensors per stage: Q, dO
  static constexpr int NSOP = 2;    // operand tensors handed over per block: dS, P
  static constexpr int TILE = TS * 2 * D;
  static constexpr int STAT = 2 * TS * (int)sizeof(float);   // L log2(e), d of the 32 staged queries
  static constexpr int STAGE = NT * TILE + STAT;
  static constexpr int SOP_WAVE = NSOP * SOP_TILE;
  static constexpr int SOP_BUF = 4 * SOP_WAVE;
  static constexpr int SOP_BASE = RING * STAGE;
  static constexpr int TOTAL = SOP_BASE + 2 * SOP_BUF;
};

template <bool F16, int D>
__device__ __forceinline__ void produce_first(const char* stage, char* sop, const bf16x8_t* Kb, const bf16x8_t* Vb, int lane,
                                              int lo, int hi, bool mask, float c_scale_log2, float l_log2, float dsum) {
  constexpr int TILE = TS * 2 * D;
  constexpr int KK = D / 16, NSTEP = 2 * KK, PF = 2, NB = PF + 1, EPK = 16 / KK;
  const int n = lane & 31, h = lane >> 5;
  int aoff[KK];
#pragma unroll
  for (int kk = 0; kk < KK; kk++) aoff[kk] = tile_off<D>(n, 2 * kk + h);
  f32x16_t s = {0}, dp, pv;   // the accumulator of dP starts at -d: dp ends as dP - d
#pragma unroll
  for (int r = 0; r < 16; r++) dp[r] = -dsum;
  bf16x8_t a[NB];
#pragma unroll
  for (int i = 0; i < PF; i++) a[i] = lds_read128(stage + (i / KK) * TILE, aoff[i % KK]);
#pragma unroll
  for (int i = 0; i < NSTEP; i++) {
    const int ph = i / KK, kk = i % KK, c = i % NB;
    if (i + PF < NSTEP) a[(i + PF) % NB] = lds_read128(stage + ((i + PF) / KK) * TILE, aoff[(i + PF) % KK]);
    __builtin_amdgcn_sched_barrier(0);
    if (ph == 0) {
      s = mfma<F16>(Kb[kk], a[c], s);
    } else {
      dp = mfma<F16>(Vb[kk], a[c], dp);
#pragma unroll
      for (int r = EPK * kk; r < EPK * (kk + 1); r++) pv[r] = __builtin_amdgcn_exp2f(s[r] * c_scale_log2 - l_log2);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  if (mask) {  // wave-uniform: the block holds hidden pairs (mask edge or end of a tensor)
    keep_branch();
#pragma unroll
    for (int r = 0; r < 16; r++) pv[r] = in_limits(r, lo, hi) ? pv[r] : 0.f;
  }
  uint32_t pk_ds[8], pk_p[8];
#pragma unroll
  for (int r = 0; r < 16; r += 2) {
    pk_ds[r / 2] = pack2<F16>(pv[r] * dp[r], pv[r + 1] * dp[r + 1]);
    pk_p[r / 2] = pack2<F16>(pv[r], pv[r + 1]);
  }
#pragma unroll
  for (int t = 0; t < 2; t++) {
    sop_write_pk(sop + 0 * SOP_TILE, pk_ds, t, lane);
    sop_write_pk(sop + 1 * SOP_TILE, pk_p, t, lane);
  }
}

template <bool F16, int D, int MASK>
__global__ void __launch_bounds__(PC_THREADS) attn_bwd_k_pc(AttnParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  using SM = PCSmemAttn<D>;
  constexpr int NC = D / 32;

  int bh, tile;
  if (!decode_block((p.n_k + WG_ROWS - 1) / WG_ROWS, p.batch, false, p.tile_major_k != 0, bh, tile)) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool producer = wave < 4;
  const int wq = wave & 3;
  const int n = lane & 31, h = lane >> 5;
  const int k0 = tile * WG_ROWS, kw = k0 + 32 * wq, kj = kw + n;
  const int kr = min(kj, p.n_k - 1);  // keys past the end compute on a copy of the last row; nothing of them is stored
  const int64_t qoff = (int64_t)bh * p.stride_qb, koff = (int64_t)bh * p.stride_kb;
  const StreamQueries<MASK> geo(p.mask_off, p.window, p.n_q);
  int t_begin, t_end;  // query tiles that hold a query seeing some key of this workgroup
  geo.tile_range(k0, WG_ROWS, t_begin, t_end);
  char* sop_base = smem + SM::SOP_BASE + wq * SM::SOP_WAVE;

  if (producer) {
    bf16x8_t Kb[D / 16], Vb[D / 16];
    load_resident<D>(Kb, (const __bf16*)p.k + koff, p.stride_kn, kr, h);
    load_resident<D>(Vb, (const __bf16*)p.v + koff, p.stride_kn, kr, h);
    const float c_scale_log2 = p.scale * kLog2e;
    const StreamKeys<MASK> kgeo(p.mask_off, p.window, p.n_k);
    __syncthreads();
    int sp = 0;  // ring slot of tile j (slot 0 holds tile t_begin)
    for (int j = t_begin; j <= t_end; j++) {
      const int qb = j * TS;
      if (j < t_end && !geo.dead(qb, kw)) {
        const char* stage = smem + sp * SM::STAGE;
        char* sop = sop_base + (j & 1) * SM::SOP_BUF;
        const bool masked = geo.partial(qb, kw);
        const int qi = qb + n;   // the lane's query
        int lo = 0, hi = 0;      // key kw + 8g + 4h + e counts for it iff lo <= 8g + e <= hi
        if (masked) {
          keep_branch();
          kgeo.limits(kw, qi, h, lo, hi);
          if (qi >= p.n_q) hi = -2 * TS;   // a row past the end of the tensor (a copy of its last row)
        }
        const float* stat = reinterpret_cast<const float*>(stage + SM::NT * SM::TILE);
        produce_first<F16, D>(stage, sop, Kb, Vb, lane, lo, hi, masked, c_scale_log2, stat[n], stat[TS + n]);
      }
      __syncthreads();
      sp = (sp == RING - 1) ? 0 : sp + 1;
    }
  } else {
    const int ctid = tid - 256;
    const __bf16* src[2] = {(const __bf16*)p.q + qoff, (const __bf16*)p.dO + qoff};
    const float* stat_src = (ctid < TS ? p.lse : p.ws_d) + (int64_t)bh * p.n_q;
    f32x16_t acc_dk[NC], acc_dv[NC];
#pragma unroll
    for (int cb = 0; cb < NC; cb++) {
      acc_dk[cb] = f32x16_t{0};
      acc_dv[cb] = f32x16_t{0};
    }
    int troff[NC][2];
#pragma unroll
    for (int cb = 0; cb < NC; cb++) {
      troff[cb][0] = tr_lane_off_acc<D>(cb, 0, lane);
      troff[cb][1] = tr_lane_off_acc<D>(cb, 1, lane);
    }
    const int sopoff[2] = {sop_tr_lane_off(0, lane), sop_tr_lane_off(1, lane)};
    Dma<D> dma;
    dma.init(p.stride_qn, wq, lane);
    const uint32_t ring_lds = lds_addr(smem);
    float stat_reg = 0.f;  // consumer threads 0..63: one statistic value of the staged tile
    // a global (not generic) load issued before the staging loads of the step and first touched at its end
    auto load_stat = [&](int q_base) {
      if (ctid < 2 * TS) stat_reg = *(global_f32_ptr)(stat_src + min(q_base + (ctid % TS), p.n_q - 1));
    };
    auto store_stat = [&](char* stage_base) {
      if (ctid < 2 * TS) reinterpret_cast<float*>(stage_base + SM::NT * SM::TILE)[ctid] = (ctid < TS) ? stat_reg * kLog2e : stat_reg;
    };
    if (t_begin < t_end) {
      const int64_t adv = (int64_t)t_begin * TS * p.stride_qn;
      dma.template issue_all<2>(ring_lds, SM::TILE, src, adv, wq, p.n_q - t_begin * TS);
      load_stat(t_begin * TS);
      store_stat(smem);
    }
    dma_wait();
    __syncthreads();
    int sc = RING - 1, sn = 1;  // ring slots of tile j-1 (read here) and tile j+1 (filled here)
    for (int j = t_begin; j <= t_end; j++) {
      if (j + 1 < t_end) {
        const uint32_t dst = ring_lds + sn * SM::STAGE;
        const int64_t adv = (int64_t)(j + 1) * TS * p.stride_qn;
        load_stat((j + 1) * TS);
        dma.template issue_all<2>(dst, SM::TILE, src, adv, wq, p.n_q - (j + 1) * TS);
      }
      if (j > t_begin && !geo.dead((j - 1) * TS, kw)) {
        const char* stage = smem + sc * SM::STAGE;
        const char* sop = sop_base + ((j - 1) & 1) * SM::SOP_BUF;
        bf16x8_t a_op[2][2];   // [k-step][dS | P]
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
          for (int x = 0; x < 2; x++) a_op[t][x] = lds_read_tr_pre(sop + sopoff[0], sop + sopoff[1], x * SOP_TILE + t * 16 * 64);
        bf16x8_t bop[2][2];    // [buffer][Q | dO]
#pragma unroll
        for (int x = 0; x < 2; x++) bop[0][x] = lds_read_tr_pre(stage + troff[0][0], stage + troff[0][1], x * SM::TILE);
#pragma unroll
        for (int it = 0; it < 2 * NC; it++) {
          const int t = it / NC, cb = it % NC, c = it & 1;
          if (it + 1 < 2 * NC) {
            const int t1 = (it + 1) / NC, cb1 = (it + 1) % NC;
#pragma unroll
            for (int x = 0; x < 2; x++)
              bop[c ^ 1][x] = lds_read_tr_pre(stage + troff[cb1][0], stage + troff[cb1][1], x * SM::TILE + t1 * 16 * 2 * D);
          }
          __builtin_amdgcn_sched_barrier(0);
          acc_dk[cb] = mfma<F16>(a_op[t][0], bop[c][0], acc_dk[cb]);
          acc_dv[cb] = mfma<F16>(a_op[t][1], bop[c][1], acc_dv[cb]);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      if (j + 1 < t_end) store_stat(smem + sn * SM::STAGE);
      dma_wait();
      __syncthreads();
      sc = (sc == RING - 1) ? 0 : sc + 1;
      sn = (sn == RING - 1) ? 0 : sn + 1;
    }
    // acc[cb][r] holds (key kw + 8*(r/4) + 4h + r%4, column 32 cb + n)
    uint16_t* odk = (uint16_t*)p.dk + koff;
    uint16_t* odv = (uint16_t*)p.dv + koff;
#pragma unroll
    for (int cb = 0; cb < NC; cb++)
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int krow = kw + 8 * (r / 4) + 4 * h + (r % 4);
        if (krow < p.n_k) {
          const int64_t o = (int64_t)krow * p.stride_kn + cb * 32 + n;
          odk[o] = to_elem<F16>(acc_dk[cb][r] * p.scale);
          odv[o] = to_elem<F16>(acc_dv[cb][r]);
        }
      }
  }
}

template <bool F16, int D, int MASK>
hipError_t launch_attn_bwd_k_pc_d(const AttnParams& p, hipStream_t s) {
  const int smem = PCSmemAttn<D>::TOTAL;
  const hipError_t e = allow_dynamic_lds<attn_bwd_k_pc<F16, D, MASK>>(smem);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL((attn_bwd_k_pc<F16, D, MASK>), dim3(grid_blocks((p.n_k + WG_ROWS - 1) / WG_ROWS, p.batch)), dim3(PC_THREADS), smem, s, p);
  return hipGetLastError();
}

template <bool F16, int D, int MASK>
hipError_t launch_pc_d(const Params& p, int pass, hipStream_t s) {
  const dim3 block(PC_THREADS);
  hipError_t e;
  if (pass == FHOG_PASS_DQ) {
    const int smem = PCSmem<D, false>::TOTAL;
    e = allow_dynamic_lds<q_sweep3_pc<F16, D, MASK, true>>(smem);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((q_sweep3_pc<F16, D, MASK, true>), dim3(grid_blocks((p.n_q + WG_ROWS - 1) / WG_ROWS, p.batch)), block, smem, s, p);
  } else if (pass == FHOG_PASS_DQ_DDO) {
    const int smem = PCSmem<D, false>::TOTAL;
    e = allow_dynamic_lds<q_sweep3_pc<F16, D, MASK>>(smem);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((q_sweep3_pc<F16, D, MASK>), dim3(grid_blocks((p.n_q + WG_ROWS - 1) / WG_ROWS, p.batch * p.n_split)), block, smem, s, p);
  } else {
    const int smem = PCSmem<D, true>::TOTAL;
    e = allow_dynamic_lds<k_sweep_pc<F16, D, MASK>>(smem);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((k_sweep_pc<F16, D, MASK>), dim3(grid_blocks((p.n_k + WG_ROWS - 1) / WG_ROWS, p.batch * p.n_split)), block, smem, s, p);
  }
  return hipGetLastError();
}

}  // namespace

// first-order backward, K-tiled, d = 128 (the other head dims run on the single-role kernel of fhog_attn.hip)
hipError_t launch_attn_bwd_k_pc(const AttnParams& p, hipStream_t s) {
  if (p.d != 128) return hipErrorInvalidValue;
  const int mask = mask_mode(p);
#define FHOG_BWDK(F)                                                                     \
  (mask == MASK_NONE ? launch_attn_bwd_k_pc_d<F, 128, MASK_NONE>(p, s)                   \
                     : mask == MASK_CAUSAL ? launch_attn_bwd_k_pc_d<F, 128, MASK_CAUSAL>(p, s) : launch_attn_bwd_k_pc_d<F, 128, MASK_BAND>(p, s))
  return p.f16 ? FHOG_BWDK(true) : FHOG_BWDK(false);
#undef FHOG_BWDK
}

hipError_t launch_bf16_pc_pass(const Params& p, int pass, hipStream_t s) {
  const int mask = mask_mode(p);
#define FHOG_PC(F, DD)                                                          \
  (mask == MASK_NONE ? launch_pc_d<F, DD, MASK_NONE>(p, pass, s)                \
                     : mask == MASK_CAUSAL ? launch_pc_d<F, DD, MASK_CAUSAL>(p, pass, s) : launch_pc_d<F, DD, MASK_BAND>(p, pass, s))
  if (p.d != 128) return hipErrorInvalidValue;   // d = 64 runs on the single-role kernels
  return p.f16 ? FHOG_PC(true, 128) : FHOG_PC(false, 128);
#undef FHOG_PC
}

}  // namespace fhog
