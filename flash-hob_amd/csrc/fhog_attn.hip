// First-order attention on gfx950 bf16 MFMA: the callers on either side of the double-backward.
//   attn_fwd_bf16     O and fp32 L = logsumexp        (fhog/triton_flash.py:12-133; L also replaces produce_L, :252-258)
//   attn_bwd_q_bf16   dQ                 Q-tiled      (fhog/triton_flash.py:201-220: P, dP, dS, dQ)
//   attn_bwd_k_bf16   dK, dV             K-tiled      (fhog/triton_flash.py:201-220: dV, dK)
// No atomics and nothing of shape (N_Q, N_K) in memory: like the double-backward, the backward recomputes
// S and dP once per tiling direction.
//
// A workgroup is 256 threads = 4 wave64 owning 128 stationary rows (queries, or keys in the K-tiled kernel);
// tiles of 32 streamed rows go through a two-stage LDS ring filled by direct global->LDS loads. First-level
// products are computed transposed (streamed rows = M, stationary rows = N), so a lane owns ONE stationary row
// and the soft-max statistics are per-lane scalars. The accumulator layout of such a product (lane = column,
// registers = streamed rows 8g + 4h + j) is, after rounding to bf16, already a valid B operand of the
// second-level MFMA whose contraction runs over the streamed rows: slot e of k-step t stands for streamed row
// 16t + 8(e/4) + 4h + e%4, and the A operand (the transposed value tile) is fetched from LDS with transposing
// reads that use the same row order. Second-level operands therefore never pass through LDS.
#include "fhog_bf16_util.h"

namespace fhog {
using namespace bf16k;
namespace {

// acc[cb] += tile^T (columns 32cb..32cb+31) x operand, for both k-steps and all column blocks of the tile
template <bool F16, int D, int NOP>
__device__ __forceinline__ void second_level(const char* const (&tile)[NOP], const int (&troff)[D / 32][2],
                                             const bf16x8_t (&op)[NOP][2], f32x16_t (&acc)[NOP][D / 32]) {
  constexpr int NC = D / 32, NIT = 2 * NC;
  bf16x8_t a[2][NOP];
#pragma unroll
  for (int x = 0; x < NOP; x++) a[0][x] = lds_read_tr_pre(tile[x] + troff[0][0], tile[x] + troff[0][1], 0);
#pragma unroll
  for (int it = 0; it < NIT; it++) {
    const int t = it / NC, cb = it % NC, c = it & 1;
    if (it + 1 < NIT) {
      const int t1 = (it + 1) / NC, cb1 = (it + 1) % NC;
#pragma unroll
      for (int x = 0; x < NOP; x++)
        a[c ^ 1][x] = lds_read_tr_pre(tile[x] + troff[cb1][0], tile[x] + troff[cb1][1], t1 * 16 * 2 * D);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int x = 0; x < NOP; x++) acc[x][cb] = mfma<F16>(a[c][x], op[x][t], acc[x][cb]);
    __builtin_amdgcn_sched_barrier(0);
  }
}

// first-level product of one streamed tile with resident rows: out += tile x res^T (streamed rows = M)
template <bool F16, int D, int NRES>
__device__ __forceinline__ void first_level(const char* tile, const int (&aoff)[D / 16], const bf16x8_t* const (&res)[NRES],
                                            f32x16_t (&out)[NRES]) {
  constexpr int KK = D / 16, PF = 2, NB = PF + 1;
  bf16x8_t a[NB];
#pragma unroll
  for (int i = 0; i < PF; i++) a[i] = lds_read128(tile, aoff[i]);
#pragma unroll
  for (int kk = 0; kk < KK; kk++) {
    if (kk + PF < KK) a[(kk + PF) % NB] = lds_read128(tile, aoff[kk + PF]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int x = 0; x < NRES; x++) out[x] = mfma<F16>(a[kk % NB], res[x][kk], out[x]);
    __builtin_amdgcn_sched_barrier(0);
  }
}

// ---- forward -----------------------------------------------------------------------------------------
template <bool F16, int D, int MASK>
__global__ void __launch_bounds__(256, 2) attn_fwd_bf16(AttnParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int KK = D / 16, NC = D / 32, TILE = TS * 2 * D, STAGE = 2 * TILE;

  int bh, tile;
  // the forward keeps the tile-major order at every length: one slice after the other measures 2 % slower on 32 x 16384 rows
  if (!decode_block((p.n_q + WG_ROWS - 1) / WG_ROWS, p.batch, MASK != MASK_NONE, MASK != MASK_NONE, bh, tile)) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, h = lane >> 5;
  const int q0 = tile * WG_ROWS, qw = q0 + 32 * wave, qi = qw + n;
  const int qr = min(qi, p.n_q - 1);  // queries past the end compute on a copy of the last row and store nothing
  const int64_t qoff = (int64_t)bh * p.stride_qb, koff = (int64_t)bh * p.stride_kb;
  const __bf16* src[2] = {(const __bf16*)p.k + koff, (const __bf16*)p.v + koff};

  bf16x8_t Qb[KK];
  load_resident<D>(Qb, (const __bf16*)p.q + qoff, p.stride_qn, qr, h);
  wait_vm0();
  const float c_scale_log2 = p.scale * kLog2e;

  int aoff[KK], troff[NC][2];
#pragma unroll
  for (int kk = 0; kk < KK; kk++) aoff[kk] = tile_off<D>(n, 2 * kk + h);
#pragma unroll
  for (int cb = 0; cb < NC; cb++) {
    troff[cb][0] = tr_lane_off_acc<D>(cb, 0, lane);
    troff[cb][1] = tr_lane_off_acc<D>(cb, 1, lane);
  }
  float m = -INFINITY, l = 0.f;  // running maximum (log2 units) of the row; this lane's half of the row sum
  f32x16_t acc[1][NC];           // O^T: acc[0][cb][r] = (column 32cb + 8(r/4) + 4h + r%4, query qi)
#pragma unroll
  for (int cb = 0; cb < NC; cb++) acc[0][cb] = f32x16_t{0};

  const StreamKeys<MASK> geo(p.mask_off, p.window, p.n_k);
  int j_begin, j_end;  // key tiles this workgroup visits
  geo.tile_range(q0, WG_ROWS, j_begin, j_end);
  Dma<D> dma;
  dma.init(p.stride_kn, wave, lane);
  const uint32_t ring_lds = lds_addr(smem);
  dma.template issue_all<2>(ring_lds + (j_begin & 1) * STAGE, TILE, src, (int64_t)j_begin * TS * p.stride_kn, wave, p.n_k - j_begin * TS);
  dma_wait();
  __syncthreads();

  for (int j = j_begin; j < j_end; j++) {
    if (j + 1 < j_end) {
      const uint32_t dst = ring_lds + ((j + 1) & 1) * STAGE;
      const int64_t adv = (int64_t)(j + 1) * TS * p.stride_kn;
      dma.template issue_all<2>(dst, TILE, src, adv, wave, p.n_k - (j + 1) * TS);
    }
    const int k0 = j * TS;
    const bool masked = geo.partial(k0, qw);  // wave-uniform: the block holds hidden keys (mask edge or tensor end)
    int lo = 0, hi = 0;                       // key k0 + 8g + 4h + e is visible iff lo <= 8g + e <= hi
    if (masked) keep_branch(), geo.limits(k0, qi, h, lo, hi);
    if (!geo.dead(k0, qw)) {  // else every key of the tile is hidden from this wave
      const char* stage = smem + (j & 1) * STAGE;
      f32x16_t s[1] = {f32x16_t{0}};
      const bf16x8_t* const res[1] = {Qb};
      first_level<F16, D, 1>(stage, aoff, res, s);  // S^T: s[r] = (key k0 + 8(r/4) + 4h + r%4, query qi)
      f32x16_t x = s[0];   // raw scores; the scale (positive) goes into the exponent's FMA, maxima commute with it
      if (masked) {
        keep_branch();
#pragma unroll
        for (int r = 0; r < 16; r++) x[r] = in_limits(r, lo, hi) ? x[r] : -INFINITY;
      }
      float tmax = fmaxf(fmaxf(x[0], x[1]), x[2]);
#pragma unroll
      for (int r = 3; r < 15; r += 2) tmax = fmaxf(fmaxf(tmax, x[r]), x[r + 1]);
      tmax = fmaxf(tmax, x[15]) * c_scale_log2;
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
      // The running maximum follows the row maximum only in jumps of more than kMaxSlack (in log2 units): P may then
      // reach 2^kMaxSlack instead of 1, which costs no precision in a 16-bit float or in the fp32 sums, and the output
      // accumulators are rescaled only in the rare steps where some row jumps (else on about every second tile).
      constexpr float kMaxSlack = 8.f;
      const float m_new = tmax > m + kMaxSlack ? tmax : m;
      // a row whose window starts in a later tile has seen no key yet: keep exp2(-inf - (-inf)) out of it
      const float m_ref = m_new == -INFINITY ? 0.f : m_new;
      const float alpha = __builtin_amdgcn_exp2f(m - m_ref);
      float rs = 0.f;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        x[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(x[r], c_scale_log2, -m_ref));
        rs += x[r];
      }
      l = __builtin_fmaf(l, alpha, rs);
      if (__builtin_amdgcn_ballot_w64(m_new > m) != 0) {  // rescale only when some row's maximum moved
#pragma unroll
        for (int cb = 0; cb < NC; cb++)
#pragma unroll
          for (int r = 0; r < 16; r++) acc[0][cb][r] *= alpha;
      }
      m = m_new;
      const bf16x8_t op[1][2] = {{pack_operand<F16>(x, 0), pack_operand<F16>(x, 1)}};
      const char* const vt[1] = {stage + TILE};
      second_level<F16, D, 1>(vt, troff, op, acc);  // O^T += V^T P^T
    }
    dma_wait();
    __syncthreads();
  }
  l += __shfl_xor(l, 32);
  const float inv = 1.f / l;
  if (qi >= p.n_q) return;
  __bf16* o = (__bf16*)p.o + qoff + (int64_t)qi * p.stride_qn;
#pragma unroll
  for (int cb = 0; cb < NC; cb++)
#pragma unroll
    for (int g = 0; g < 4; g++) {
      const f32x16_t& a = acc[0][cb];
      *reinterpret_cast<u32x2_t*>(o + 32 * cb + 8 * g + 4 * h) =
          pack4<F16>(a[4 * g] * inv, a[4 * g + 1] * inv, a[4 * g + 2] * inv, a[4 * g + 3] * inv);
    }
  if (h == 0) p.lse[(int64_t)bh * p.n_q + qi] = (m + __builtin_amdgcn_logf(l)) * 0.6931471805599453f;  // v_log_f32 is log2
}

// ---- backward, Q-tiled: dQ -----------------------------------------------------------------------------
template <bool F16, int D, int MASK>
__global__ void __launch_bounds__(256, 2) attn_bwd_q_bf16(AttnParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int KK = D / 16, NC = D / 32, TILE = TS * 2 * D, STAGE = 2 * TILE;

  int bh, tile;
  if (!decode_block((p.n_q + WG_ROWS - 1) / WG_ROWS, p.batch, MASK != MASK_NONE, p.tile_major_q != 0, bh, tile)) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, h = lane >> 5;
  const int q0 = tile * WG_ROWS, qw = q0 + 32 * wave, qi = qw + n;
  const int qr = min(qi, p.n_q - 1);  // queries past the end compute on a copy of the last row and store nothing
  const int64_t qoff = (int64_t)bh * p.stride_qb, koff = (int64_t)bh * p.stride_kb;
  const __bf16* src[2] = {(const __bf16*)p.k + koff, (const __bf16*)p.v + koff};

  bf16x8_t Qb[KK], dOb[KK];
  load_resident<D>(Qb, (const __bf16*)p.q + qoff, p.stride_qn, qr, h);
  load_resident<D>(dOb, (const __bf16*)p.dO + qoff, p.stride_qn, qr, h);
  const int64_t row = (int64_t)bh * p.n_q + qr;
  const float l_log2 = p.lse[row] * kLog2e, dsum = p.ws_d[row];
  wait_vm0();
  const float c_scale_log2 = p.scale * kLog2e;

  int aoff[KK], troff[NC][2];
#pragma unroll
  for (int kk = 0; kk < KK; kk++) aoff[kk] = tile_off<D>(n, 2 * kk + h);
#pragma unroll
  for (int cb = 0; cb < NC; cb++) {
    troff[cb][0] = tr_lane_off_acc<D>(cb, 0, lane);
    troff[cb][1] = tr_lane_off_acc<D>(cb, 1, lane);
  }
  f32x16_t acc[1][NC];  // dQ^T
#pragma unroll
  for (int cb = 0; cb < NC; cb++) acc[0][cb] = f32x16_t{0};

  const StreamKeys<MASK> geo(p.mask_off, p.window, p.n_k);
  int j_begin, j_end;  // key tiles this workgroup visits
  geo.tile_range(q0, WG_ROWS, j_begin, j_end);
  Dma<D> dma;
  dma.init(p.stride_kn, wave, lane);
  const uint32_t ring_lds = lds_addr(smem);
  dma.template issue_all<2>(ring_lds + (j_begin & 1) * STAGE, TILE, src, (int64_t)j_begin * TS * p.stride_kn, wave, p.n_k - j_begin * TS);
  dma_wait();
  __syncthreads();

  for (int j = j_begin; j < j_end; j++) {
    if (j + 1 < j_end) {
      const uint32_t dst = ring_lds + ((j + 1) & 1) * STAGE;
      const int64_t adv = (int64_t)(j + 1) * TS * p.stride_kn;
      dma.template issue_all<2>(dst, TILE, src, adv, wave, p.n_k - (j + 1) * TS);
    }
    const int k0 = j * TS;
    const bool masked = geo.partial(k0, qw);  // wave-uniform: the block holds hidden keys (mask edge or tensor end)
    int lo = 0, hi = 0;                       // key k0 + 8g + 4h + e is visible iff lo <= 8g + e <= hi
    if (masked) keep_branch(), geo.limits(k0, qi, h, lo, hi);
    if (!geo.dead(k0, qw)) {
      const char* stage = smem + (j & 1) * STAGE;
      f32x16_t s[1] = {f32x16_t{0}}, dp[1];
#pragma unroll
      for (int r = 0; r < 16; r++) dp[0][r] = -dsum;        // the accumulator ends as dP - d
      const bf16x8_t* const rq[1] = {Qb};
      const bf16x8_t* const rdo[1] = {dOb};
      first_level<F16, D, 1>(stage, aoff, rq, s);           // S^T  = K Q^T
      first_level<F16, D, 1>(stage + TILE, aoff, rdo, dp);  // dP^T = V dO^T - d
      f32x16_t ds;
#pragma unroll
      for (int r = 0; r < 16; r++) ds[r] = __builtin_amdgcn_exp2f(s[0][r] * c_scale_log2 - l_log2) * dp[0][r];
      if (masked) {
        keep_branch();
#pragma unroll
        for (int r = 0; r < 16; r++) ds[r] = in_limits(r, lo, hi) ? ds[r] : 0.f;
      }
      const bf16x8_t op[1][2] = {{pack_operand<F16>(ds, 0), pack_operand<F16>(ds, 1)}};
      const char* const kt[1] = {stage};
      second_level<F16, D, 1>(kt, troff, op, acc);  // dQ^T += K^T dS^T
    }
    dma_wait();
    __syncthreads();
  }
  if (qi >= p.n_q) return;
  __bf16* o = (__bf16*)p.dq + qoff + (int64_t)qi * p.stride_qn;
#pragma unroll
  for (int cb = 0; cb < NC; cb++)
#pragma unroll
    for (int g = 0; g < 4; g++) {
      const f32x16_t& a = acc[0][cb];
      *reinterpret_cast<u32x2_t*>(o + 32 * cb + 8 * g + 4 * h) =
          pack4<F16>(a[4 * g] * p.scale, a[4 * g + 1] * p.scale, a[4 * g + 2] * p.scale, a[4 * g + 3] * p.scale);
    }
}

// ---- backward, K-tiled: dK, dV (d = 64; at d = 128 attn_bwd_k_pc of fhog_bf16_pc.hip) ---------------------------------
template <bool F16, int D, int MASK>
__global__ void __launch_bounds__(256, 2) attn_bwd_k_bf16(AttnParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int KK = D / 16, NC = D / 32, TILE = TS * 2 * D;
  constexpr int STAT = 2 * TS * 4;         // L log2(e) and d of the 32 staged queries
  constexpr int STAGE = 2 * TILE + STAT;   // Q tile, dO tile, statistics

  int bh, tile;
  if (!decode_block((p.n_k + WG_ROWS - 1) / WG_ROWS, p.batch, false, p.tile_major_k != 0, bh, tile)) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, h = lane >> 5;
  const int k0 = tile * WG_ROWS, kw = k0 + 32 * wave, kj = kw + n;
  const int kr = min(kj, p.n_k - 1);  // keys past the end compute on a copy of the last row and store nothing
  const int64_t qoff = (int64_t)bh * p.stride_qb, koff = (int64_t)bh * p.stride_kb;
  const __bf16* src[2] = {(const __bf16*)p.q + qoff, (const __bf16*)p.dO + qoff};
  const float* stat_src = (tid < TS ? p.lse : p.ws_d) + (int64_t)bh * p.n_q;

  bf16x8_t Kb[KK], Vb[KK];
  load_resident<D>(Kb, (const __bf16*)p.k + koff, p.stride_kn, kr, h);
  load_resident<D>(Vb, (const __bf16*)p.v + koff, p.stride_kn, kr, h);
  const float c_scale_log2 = p.scale * kLog2e;

  int aoff[KK], troff[NC][2];
#pragma unroll
  for (int kk = 0; kk < KK; kk++) aoff[kk] = tile_off<D>(n, 2 * kk + h);
#pragma unroll
  for (int cb = 0; cb < NC; cb++) {
    troff[cb][0] = tr_lane_off_acc<D>(cb, 0, lane);
    troff[cb][1] = tr_lane_off_acc<D>(cb, 1, lane);
  }
  f32x16_t acc[2][NC];  // [0]: dK^T, [1]: dV^T
#pragma unroll
  for (int cb = 0; cb < NC; cb++) {
    acc[0][cb] = f32x16_t{0};
    acc[1][cb] = f32x16_t{0};
  }
  const StreamQueries<MASK> geo(p.mask_off, p.window, p.n_q);
  int t_begin, t_end;  // query tiles that hold a query seeing some key of this workgroup
  geo.tile_range(k0, WG_ROWS, t_begin, t_end);
  Dma<D> dma;
  dma.init(p.stride_qn, wave, lane);
  const uint32_t ring_lds = lds_addr(smem);
  float stat_reg = 0.f;  // threads 0..63: one statistic of the tile being staged
  // The statistic is loaded before the staging loads of a step and first touched at the end of the step, so the
  // wave never waits for it in between.
  auto load_stat = [&](int q_base) {
    if (tid < 2 * TS) stat_reg = *(global_f32_ptr)(stat_src + min(q_base + (tid & (TS - 1)), p.n_q - 1));
  };
  auto store_stat = [&](char* stage_base) {
    if (tid < 2 * TS) reinterpret_cast<float*>(stage_base + 2 * TILE)[tid] = (tid < TS) ? stat_reg * kLog2e : stat_reg;
  };
  {
    load_stat(t_begin * TS);
    const int64_t adv = (int64_t)t_begin * TS * p.stride_qn;
    dma.template issue_all<2>(ring_lds, TILE, src, adv, wave, p.n_q - t_begin * TS);
    wait_vm0();
    store_stat(smem);
  }
  __syncthreads();

  for (int j = t_begin; j < t_end; j++) {
    const int st = (j - t_begin) & 1;
    if (j + 1 < t_end) {
      load_stat((j + 1) * TS);
      const uint32_t dst = ring_lds + (st ^ 1) * STAGE;
      const int64_t adv = (int64_t)(j + 1) * TS * p.stride_qn;
      dma.template issue_all<2>(dst, TILE, src, adv, wave, p.n_q - (j + 1) * TS);
    }
    const int qb = j * TS;
    if (!geo.dead(qb, kw)) {  // else no query of the tile sees a key of this wave
      const char* stage = smem + st * STAGE;
      const float* stat = reinterpret_cast<const float*>(stage + 2 * TILE);
      f32x16_t s[1] = {f32x16_t{0}}, dp[1] = {f32x16_t{0}};
      const bf16x8_t* const rk[1] = {Kb};
      const bf16x8_t* const rv[1] = {Vb};
      first_level<F16, D, 1>(stage, aoff, rk, s);           // S  = Q K^T : s[r] = (query qb + 8(r/4) + 4h + r%4, key kj)
      first_level<F16, D, 1>(stage + TILE, aoff, rv, dp);   // dP = dO V^T
      f32x16_t pv, ds;
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const f32x4_t l4 = *reinterpret_cast<const f32x4_t*>(stat + 8 * g + 4 * h);
        const f32x4_t d4 = *reinterpret_cast<const f32x4_t*>(stat + TS + 8 * g + 4 * h);
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int r = 4 * g + e;
          pv[r] = __builtin_amdgcn_exp2f(s[0][r] * c_scale_log2 - l4[e]);
          ds[r] = dp[0][r] - d4[e];
        }
      }
      if (geo.partial(qb, kw)) {  // wave-uniform: the block holds hidden (query, key) pairs
        int lo, hi;                // query row 8g + 4h + e of the tile counts iff lo <= 8g + e <= hi: it exists and sees key kj
        geo.limits(qb, kj, h, lo, hi);
        keep_branch();
#pragma unroll
        for (int r = 0; r < 16; r++) pv[r] = in_limits(r, lo, hi) ? pv[r] : 0.f;
      }
#pragma unroll
      for (int r = 0; r < 16; r++) ds[r] *= pv[r];
      const bf16x8_t op[2][2] = {{pack_operand<F16>(ds, 0), pack_operand<F16>(ds, 1)}, {pack_operand<F16>(pv, 0), pack_operand<F16>(pv, 1)}};
      const char* const tl[2] = {stage, stage + TILE};
      second_level<F16, D, 2>(tl, troff, op, acc);  // dK^T += Q^T dS ; dV^T += dO^T P
    }
    if (j + 1 < t_end) {
      wait_vm0();
      store_stat(smem + (st ^ 1) * STAGE);
    }
    dma_wait();
    __syncthreads();
  }
  if (kj >= p.n_k) return;
  __bf16* odk = (__bf16*)p.dk + koff + (int64_t)kj * p.stride_kn;
  __bf16* odv = (__bf16*)p.dv + koff + (int64_t)kj * p.stride_kn;
#pragma unroll
  for (int cb = 0; cb < NC; cb++)
#pragma unroll
    for (int g = 0; g < 4; g++) {
      const f32x16_t& a = acc[0][cb];
      const f32x16_t& b = acc[1][cb];
      *reinterpret_cast<u32x2_t*>(odk + 32 * cb + 8 * g + 4 * h) =
          pack4<F16>(a[4 * g] * p.scale, a[4 * g + 1] * p.scale, a[4 * g + 2] * p.scale, a[4 * g + 3] * p.scale);
      *reinterpret_cast<u32x2_t*>(odv + 32 * cb + 8 * g + 4 * h) = pack4<F16>(b[4 * g], b[4 * g + 1], b[4 * g + 2], b[4 * g + 3]);
    }
}

template <auto Kernel>
hipError_t launch(unsigned grid, int smem, hipStream_t s, const AttnParams& p) {
  const hipError_t e = allow_dynamic_lds<Kernel>(smem);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(Kernel, dim3(grid), dim3(256), smem, s, p);
  return hipGetLastError();
}

template <bool F16, int D, int MASK>
hipError_t launch_attn_d(const AttnParams& p, int which, hipStream_t s) {
  constexpr int TILE = TS * 2 * D;
  switch (which) {
    case 0: return launch<attn_fwd_bf16<F16, D, MASK>>(grid_blocks((p.n_q + WG_ROWS - 1) / WG_ROWS, p.batch), 2 * 2 * TILE, s, p);
    case 1: return launch<attn_bwd_q_bf16<F16, D, MASK>>(grid_blocks((p.n_q + WG_ROWS - 1) / WG_ROWS, p.batch), 2 * 2 * TILE, s, p);
    default:
      if constexpr (D == 64)
        return launch<attn_bwd_k_bf16<F16, D, MASK>>(grid_blocks((p.n_k + WG_ROWS - 1) / WG_ROWS, p.batch), 2 * (2 * TILE + 2 * TS * 4), s, p);
      else
        return hipErrorInvalidValue;   // d = 128 is dispatched to the producer/consumer kernel before this point
  }
}

}  // namespace

// which: 0 forward, 1 backward Q-tiled (dQ), 2 backward K-tiled (dK, dV)
hipError_t launch_attn_bf16(const AttnParams& p, int which, hipStream_t s) {
  if (!bf16_shape_supported(p.n_q, p.n_k, p.d, p.causal)) return hipErrorInvalidValue;
  if (which == 2 && p.d == 128) return launch_attn_bwd_k_pc(p, s);   // one wave does not hold this sweep at d = 128
  const int mask = mask_mode(p);
#define FHOG_ATTN(F, DD)                                                            \
  (mask == MASK_NONE ? launch_attn_d<F, DD, MASK_NONE>(p, which, s)                 \
                     : mask == MASK_CAUSAL ? launch_attn_d<F, DD, MASK_CAUSAL>(p, which, s) : launch_attn_d<F, DD, MASK_BAND>(p, which, s))
  if (p.f16) return p.d == 128 ? FHOG_ATTN(true, 128) : FHOG_ATTN(true, 64);
  return p.d == 128 ? FHOG_ATTN(false, 128) : FHOG_ATTN(false, 64);
#undef FHOG_ATTN
}

}  // namespace fhog
