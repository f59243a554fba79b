// Q-tiled sweep of the opt-in schedules that take ddO out of the third sweep (16-bit MFMA family, gfx950).
//
// The reference's second sweep recomputes five first-level products to form b_i = sum_j P_ij dP'_ij
// (fhog/triton_bwdbwd.py:217-251) and its third sweep forms ddO = P ddV + ddP V (fhog/triton_bwdbwd.py:284-288).
// Since sum_j P_ij dP_ij = d_i, the row statistic is a row dot of that output:
//     b_i = dO_i . ddO_i - d_i dd_i,
// so ONE sweep with the three first-level products of S and ddS and the two second-level products of ddO yields ddO
// and b together (five products; the sweep for dQ2 behind it then needs seven instead of nine):
//     KNOWN_DD = true   dd_i comes from the dd sweep in front: ddP = P (ddS - dd_i)                 (FHOG_PASS_B_DDO)
//     KNOWN_DD = false  dd_i = sum_j P_ij ddS_ij is accumulated in the same sweep and taken out at the end of the
//                       row, ddO_i = (P ddV)_i + ((P o ddS) V)_i - dd_i O_i, using sum_j P_ij V_j = O_i
//                       (FHOG_PASS_DD_B_DDO; it also writes d_i = O_i . dO_i for the sweeps behind it)
//
// Single-role kernel of the shape of the statistics sweeps: 256 threads = 4 wave64 own 128 queries, two workgroups per
// CU (NW = 8: 512 threads own 256 queries, one workgroup per CU, for launches with plenty of workgroups: every staged
// tile then serves twice the rows, i.e. half the staging loads per row). A wave keeps Q and ddQ of its 32 queries in
// registers as MFMA B operands; K, ddK, V, ddV stream through a two-stage LDS ring of 32-key tiles filled by direct
// global->LDS loads. First-level products have the keys as M and
// the queries as N, so a lane owns one query; P and ddP, rounded to 16 bits, are the B operands of the second-level
// products as they stand in the registers (contraction over the keys), whose A operands are transposing reads of the
// staged V and ddV tiles: nothing S-shaped passes through LDS, and one 32 x D fp32 accumulator (ddO^T: lane = query,
// registers = columns) fits next to the two resident tensors.
#include "fhog_bf16_util.h"

namespace fhog {
using namespace bf16k;
namespace {

template <bool F16, int D, int MASK, bool KNOWN_DD, int NW = 4>
__global__ void __launch_bounds__(64 * NW, NW == 8 ? 1 : 2) q_sweep_ddo(Params p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int NT = 4, TILE = TS * 2 * D, STAGE = NT * TILE, KK = D / 16, NC = D / 32, ROWS = 32 * NW;

  int bh, tile;
  if (!decode_block((p.n_q + ROWS - 1) / ROWS, p.batch, MASK != MASK_NONE, p.tile_major, bh, tile)) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: lets the compiler branch on scalars
  const int n = lane & 31, h = lane >> 5;
  const int q0 = tile * ROWS, qw = q0 + 32 * wave, qi = qw + n;
  const int qr = min(qi, p.n_q - 1);  // queries past the end compute on a copy of the last row and store nothing
  const int64_t qoff = (int64_t)bh * p.stride_qb, koff = (int64_t)bh * p.stride_kb;
  const __bf16* src[NT] = {(const __bf16*)p.k + koff, (const __bf16*)p.ddk + koff, (const __bf16*)p.v + koff,
                           (const __bf16*)p.ddv + koff};

  // the first streamed tile is requested before the resident operands: the two round trips to memory overlap
  const StreamKeys<MASK> geo(p.mask_off, p.window, p.n_k);
  int j_begin, j_end;  // key tiles this workgroup visits
  geo.tile_range(q0, ROWS, j_begin, j_end);
  // staging: four waves share the rows of a tile; with eight waves each group of four takes two of the four tensors
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
  const auto stage_tile = [&](int j) {
    dma.template issue_all<NLD>(ring_lds + (j & 1) * STAGE, TILE, srcl, (int64_t)j * TS * p.stride_kn, wave & 3, p.n_k - j * TS);
  };
  if (j_begin < j_end) stage_tile(j_begin);

  bf16x8_t Qb[KK], ddQb[KK];
  load_resident<D>(Qb, (const __bf16*)p.q + qoff, p.stride_qn, qr, h);
  load_resident<D>(ddQb, (const __bf16*)p.ddq + qoff, p.stride_qn, qr, h);
  const int64_t row = (int64_t)bh * p.n_q + qr;
  const float l_log2 = p.lse[row] * kLog2e;
  const float c_scale_log2 = p.scale * kLog2e;
  const float dd_in = KNOWN_DD ? p.ws_dd[row] : 0.f;
  const float d_in = KNOWN_DD ? p.ws_d[row] : 0.f;

  f32x16_t acc[NC];   // ddO^T: lane = query, register 4g + i of block cb = column 32 cb + 8g + 4h + i
  int troff[NC][2];
#pragma unroll
  for (int cb = 0; cb < NC; cb++) {
    acc[cb] = f32x16_t{0};
    troff[cb][0] = tr_lane_off_acc<D>(cb, 0, lane);
    troff[cb][1] = tr_lane_off_acc<D>(cb, 1, lane);
  }
  // All register loads land here: the staging loads are issued from inline asm, which the compiler's wait-count
  // bookkeeping does not see; without this wait it would keep waits for the resident operands inside the loop.
  wait_vm0();
  int aoff[KK];
#pragma unroll
  for (int kk = 0; kk < KK; kk++) aoff[kk] = tile_off<D>(n, 2 * kk + h);
  dma_wait();
  __syncthreads();

  float red = 0.f;   // KNOWN_DD = false: this lane's share of sum_j P_ij ddS_ij scale
  for (int j = j_begin; j < j_end; j++) {
    if (j + 1 < j_end) stage_tile(j + 1);
    const int k0 = j * TS;
    const bool masked = geo.partial(k0, qw);  // wave-uniform: the block holds hidden keys (mask edge or tensor end)
    int lo = 0, hi = 0;                       // key k0 + 8g + 4h + e is visible iff lo <= 8g + e <= hi
    if (masked) keep_branch(), geo.limits(k0, qi, h, lo, hi);
    if (!geo.dead(k0, qw)) {  // else every key of the tile is hidden from this wave
      const char* stage = smem + (j & 1) * STAGE;
      // first level, a stream of 2 KK k-steps with the LDS operands fetched PF steps ahead (stage order K, ddK, V, ddV):
      //   K  : S += K Q^T, ddS += K ddQ^T
      //   ddK: ddS += ddK Q^T          + P = exp2(S c - L) behind the MFMAs (in place of S)
      constexpr int NSTEP = 2 * KK, PF = 2, NB = PF + 1, EPK = 16 / KK;
      f32x16_t s = {0}, dds = {0};
      bf16x8_t a[NB];
#pragma unroll
      for (int i = 0; i < PF; i++) a[i] = lds_read128(stage + (i / KK) * TILE, aoff[i % KK]);
#pragma unroll
      for (int i = 0; i < NSTEP; i++) {
        const int ph = i / KK, kk = i % KK, c = i % NB;
        if (i + PF < NSTEP) a[(i + PF) % NB] = lds_read128(stage + ((i + PF) / KK) * TILE, aoff[(i + PF) % KK]);
        __builtin_amdgcn_sched_barrier(0);
        if (ph == 0) {
          s = mfma<F16>(a[c], Qb[kk], s);
          dds = mfma<F16>(a[c], ddQb[kk], dds);
        } else {
          dds = mfma<F16>(a[c], Qb[kk], dds);
#pragma unroll
          for (int r = EPK * kk; r < EPK * (kk + 1); r++) s[r] = __builtin_amdgcn_exp2f(s[r] * c_scale_log2 - l_log2);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      // second level: ddO^T += V^T ddP^T + ddV^T P^T, two column blocks per round so that the MFMAs on one accumulator
      // are two instructions apart; the first transposed operands are requested before the elementwise work
      constexpr int NP = NC / 2, NIT = 2 * NP;
      bf16x8_t ta[2][2][2];   // [buffer][column block of the pair][V | ddV]
      const auto read_ta = [&](int buf, int it) {
        const int t = it / NP, cp = it % NP;
#pragma unroll
        for (int cl = 0; cl < 2; cl++)
#pragma unroll
          for (int x = 0; x < 2; x++)
            ta[buf][cl][x] = lds_read_tr_pre(stage + troff[2 * cp + cl][0], stage + troff[2 * cp + cl][1], (2 + x) * TILE + t * 16 * 2 * D);
      };
      read_ta(0, 0);
      if (masked) {
        keep_branch();
#pragma unroll
        for (int r = 0; r < 16; r++) s[r] = in_limits(r, lo, hi) ? s[r] : 0.f;
      }
      // ddP = P (ddS scale - dd) [or P ddS scale, with dd taken out at the end of the row]; P and ddP packed to 16 bits
      uint32_t pk_p[8], pk_ddp[8];
      const auto elementwise = [&](int r0, int r1) {
#pragma unroll
        for (int r = r0; r < r1; r += 2) {
          const float w0 = KNOWN_DD ? __builtin_fmaf(dds[r], p.scale, -dd_in) : dds[r] * p.scale;
          const float w1 = KNOWN_DD ? __builtin_fmaf(dds[r + 1], p.scale, -dd_in) : dds[r + 1] * p.scale;
          const float ddp0 = s[r] * w0, ddp1 = s[r + 1] * w1;
          if (!KNOWN_DD) red += ddp0 + ddp1;
          pk_ddp[r / 2] = pack2<F16>(ddp0, ddp1);
          pk_p[r / 2] = pack2<F16>(s[r], s[r + 1]);
        }
      };
      const auto opnd = [](const uint32_t* pk, int t) {
        return __builtin_bit_cast(bf16x8_t, u32x4_t{pk[4 * t], pk[4 * t + 1], pk[4 * t + 2], pk[4 * t + 3]});
      };
      elementwise(0, 8);   // registers 0..7: the keys of the first second-level k-step
      constexpr int EPI = 8 / NP;   // registers 8..15 follow in pieces behind the MFMAs of that step
#pragma unroll
      for (int it = 0; it < NIT; it++) {
        const int t = it / NP, cp = it % NP, c = it & 1;
        if (it + 1 < NIT) read_ta(c ^ 1, it + 1);
        __builtin_amdgcn_sched_barrier(0);
        acc[2 * cp] = mfma<F16>(ta[c][0][0], opnd(pk_ddp, t), acc[2 * cp]);
        acc[2 * cp + 1] = mfma<F16>(ta[c][1][0], opnd(pk_ddp, t), acc[2 * cp + 1]);
        acc[2 * cp] = mfma<F16>(ta[c][0][1], opnd(pk_p, t), acc[2 * cp]);
        acc[2 * cp + 1] = mfma<F16>(ta[c][1][1], opnd(pk_p, t), acc[2 * cp + 1]);
        if (t == 0) elementwise(8 + EPI * cp, 8 + EPI * (cp + 1));
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    dma_wait();
    __syncthreads();
  }

  // end of the row: dd, d, ddO and b = dO . ddO - d dd. Each lane holds half of its query's columns.
  float dd = dd_in, dsum = d_in;
  if (!KNOWN_DD) {
    red += __shfl_xor(red, 32);
    dd = red;
  }
  const __bf16* orow = (const __bf16*)p.o + qoff + (int64_t)qr * p.stride_qn;
  const __bf16* dorow = (const __bf16*)p.dO + qoff + (int64_t)qr * p.stride_qn;
  uint16_t* oddo = (uint16_t*)p.ddo + qoff + (int64_t)qr * p.stride_qn;
  float dot = 0.f, od = 0.f;
#pragma unroll
  for (int cb = 0; cb < NC; cb++)
#pragma unroll
    for (int g = 0; g < 4; g++) {
      const int col = 32 * cb + 8 * g + 4 * h;
      const bf16x4_t do4 = *reinterpret_cast<const bf16x4_t*>(dorow + col);
      bf16x4_t o4 = do4;
      if (!KNOWN_DD) o4 = *reinterpret_cast<const bf16x4_t*>(orow + col);
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const float dof = to_f32<F16>(do4[i]);
        float v = acc[cb][4 * g + i];
        if (!KNOWN_DD) {
          const float of = to_f32<F16>(o4[i]);
          od = __builtin_fmaf(of, dof, od);
          v = __builtin_fmaf(-dd, of, v);   // (P o ddS) V - dd O = ddP V
        }
        dot = __builtin_fmaf(dof, v, dot);
        acc[cb][4 * g + i] = v;
      }
    }
  // the stores in a run of their own, so that the eight-byte pieces of a row reach the memory side together
  if (qi < p.n_q) {
#pragma unroll
    for (int cb = 0; cb < NC; cb++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const f32x16_t& y = acc[cb];
        *reinterpret_cast<u32x2_t*>(oddo + 32 * cb + 8 * g + 4 * h) = pack4<F16>(y[4 * g], y[4 * g + 1], y[4 * g + 2], y[4 * g + 3]);
      }
  }
  dot += __shfl_xor(dot, 32);
  if (!KNOWN_DD) {
    od += __shfl_xor(od, 32);
    dsum = od;
  }
  if (h == 0 && qi < p.n_q) {
    p.ws_b[row] = __builtin_fmaf(-dsum, dd, dot);
    if (!KNOWN_DD) {
      p.ws_dd[row] = dd;
      p.ws_d[row] = dsum;
    }
  }
}

template <auto Kernel>
hipError_t launch(unsigned grid, unsigned threads, int smem, hipStream_t s, const Params& p) {
  const hipError_t e = allow_dynamic_lds<Kernel>(smem);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(Kernel, dim3(grid), dim3(threads), smem, s, p);
  return hipGetLastError();
}

template <bool F16, int D, int MASK>
hipError_t launch_ddo_d(const Params& p, int pass, hipStream_t s) {
  const unsigned grid = grid_blocks((p.n_q + WG_ROWS - 1) / WG_ROWS, p.batch);
  constexpr int smem = 2 * 4 * TS * 2 * D;
  // with plenty of workgroups, 256 queries per workgroup of eight waves (one per CU), as the b sweep does at d = 128
  const unsigned g8 = grid_blocks((p.n_q + 255) / 256, p.batch);
  const int w8 = tuning().b8;
  if (D == 128 && (w8 < 0 ? g8 >= 512 : w8 == 1)) {
    if (pass == FHOG_PASS_B_DDO) return launch<q_sweep_ddo<F16, D, MASK, true, 8>>(g8, 512, smem, s, p);
    return launch<q_sweep_ddo<F16, D, MASK, false, 8>>(g8, 512, smem, s, p);
  }
  if (pass == FHOG_PASS_B_DDO) return launch<q_sweep_ddo<F16, D, MASK, true>>(grid, 256, smem, s, p);
  return launch<q_sweep_ddo<F16, D, MASK, false>>(grid, 256, smem, s, p);
}

}  // namespace

// FHOG_PASS_B_DDO and FHOG_PASS_DD_B_DDO, d in {64, 128}
hipError_t launch_bf16_ddo_pass(const Params& p, int pass, hipStream_t s) {
  if (pass != FHOG_PASS_B_DDO && pass != FHOG_PASS_DD_B_DDO) return hipErrorInvalidValue;
  if (p.d != 64 && p.d != 128) return hipErrorInvalidValue;
  const int mask = mask_mode(p);
#define FHOG_DDO(F, DD)                                                        \
  (mask == MASK_NONE ? launch_ddo_d<F, DD, MASK_NONE>(p, pass, s)              \
                     : mask == MASK_CAUSAL ? launch_ddo_d<F, DD, MASK_CAUSAL>(p, pass, s) : launch_ddo_d<F, DD, MASK_BAND>(p, pass, s))
  if (p.f16) return p.d == 128 ? FHOG_DDO(true, 128) : FHOG_DDO(true, 64);
  return p.d == 128 ? FHOG_DDO(false, 128) : FHOG_DDO(false, 64);
#undef FHOG_DDO
}

}  // namespace fhog
