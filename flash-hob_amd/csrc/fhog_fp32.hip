// fp32-MFMA kernels of the attention double-backward: every product and every
// intermediate in fp32 (v_mfma_f32_32x32x2_f32). This family serves fp32 tensors (16-bit
// MFMA cannot reach 1e-4) and d = 32; it takes bf16 and fp16 tensors of any shape too.
// No atomics, nothing of shape (N_Q, N_K) leaves the chip.
//
// One kernel template for the four sweeps. A workgroup of 4 wave64 owns 32 stationary rows per wave
// (queries in passes 1-3, keys in pass 4) and keeps their operands in registers; the other side
// streams through LDS in 32-row tiles shared by the waves. Small launches (WS = 2 or 4) put WS waves
// on the same 32 rows instead: each takes every WS-th streamed tile and the partial results are
// added through LDS in a fixed order, so a short problem is spread over WS times the workgroups. First-level products are
// computed with the streamed rows as M and the stationary rows as N, so a lane owns ONE stationary
// row and its registers run over the streamed rows. Such an accumulator is, as it stands, the B
// operand of the second-level products (contraction over the streamed rows; the A operand is read
// from the streamed LDS tile in the same row order), so nothing S-shaped passes through LDS.
//
// Math per tile pair (fhog/triton_bwdbwd.py:194-202, 229-243, 266-288, 485-507):
//   S = scale Q K^T, P = exp(S - L), dP = dO V^T, ddS = scale (ddQ K^T + Q ddK^T), E = dO ddV^T
//   dP' = E - dP dd - ddS d + dP ddS
//   dS = scale P (dP - d), dS' = scale P (dP' - b), ddP = P (ddS - dd)
#include "fhog_bf16_util.h"   // XCD-aware grid decode
#include "fhog_fp32_util.h"

namespace fhog {
using namespace f32k;
namespace {

// PASS 1: dd (Q-tiled), 2: b (Q-tiled), 3: dQ2 and ddO (Q-tiled), 4: dK2 and dV2 (K-tiled).
template <typename T, int D, int PASS, bool MASKED, int WS = 1>
__global__ void __launch_bounds__(256) sweep_fp32(Params p) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  constexpr bool KSIDE = PASS == 4;                          // the stationary rows are keys
  constexpr int NT = PASS == 1 ? 2 : (KSIDE ? 3 : 4);        // streamed tensors
  constexpr int NR = KSIDE ? 4 : (PASS == 1 ? 2 : 3);        // stationary tensors
  constexpr bool LAST_IN_LDS = KSIDE && D == 128;            // the fourth stationary tensor does not fit the registers
  constexpr int NREG = LAST_IN_LDS ? 3 : NR;
  constexpr int J = D / 8, CB = D / 32, TF = Tile<D>::FLOATS;

  static_assert(WS == 1 || D <= 64, "wave split needs WS staged tiles per tensor in LDS");
  constexpr int nthr = 256;        // 4 waves (waves without rows still help with the loads)
  constexpr int nw = 4 / WS;       // groups of 32 stationary rows per workgroup, WS waves on each
  const int tid = threadIdx.x, lane = tid & 63;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave = wv / WS, ws = wv % WS;   // row group of the wave, and which of its streamed tiles it takes
  const int n = lane & 31, h = lane >> 5;
  const int n_sta = KSIDE ? p.n_k : p.n_q, n_str = KSIDE ? p.n_q : p.n_k;
  // All tiles of a slice on one XCD (one L2 streams the slice's other side). With a mask the work of a tile grows (or
  // falls) with its index, so a workgroup takes tiles u and n_tiles - 1 - u in turn: every workgroup of a slice
  // then does the same amount of work, whatever their number.
  const int n_tiles = (n_sta + TR * nw - 1) / (TR * nw);
  int bh, unit;
  if (!bf16k::decode_block(MASKED ? (n_tiles + 1) / 2 : n_tiles, p.batch, false, false, bh, unit)) return;
  const int64_t qoff = (int64_t)bh * p.stride_qb, koff = (int64_t)bh * p.stride_kb;
  const int64_t sta_ld = KSIDE ? p.stride_kn : p.stride_qn, str_ld = KSIDE ? p.stride_qn : p.stride_kn;
  // stationary tensors: Q, ddQ, dO | K, ddK, V, ddV; streamed tensors: K, ddK, V, ddV | Q, ddQ, dO
  const T* sta[4] = {(const T*)(KSIDE ? p.k : p.q) + (KSIDE ? koff : qoff), (const T*)(KSIDE ? p.ddk : p.ddq) + (KSIDE ? koff : qoff),
                     (const T*)(KSIDE ? p.v : p.dO) + (KSIDE ? koff : qoff), (const T*)p.ddv + koff};
  const T* str[4] = {(const T*)(KSIDE ? p.q : p.k) + (KSIDE ? qoff : koff), (const T*)(KSIDE ? p.ddq : p.ddk) + (KSIDE ? qoff : koff),
                     (const T*)(KSIDE ? p.dO : p.v) + (KSIDE ? qoff : koff), (const T*)p.ddv + koff};

  float* tiles = smem;                                // WS stages of NT streamed tiles
  float* stat = tiles + WS * NT * TF;                 // pass 4: L, d, dd, b of the 32 streamed queries of each stage
  float* sta_lds = stat + (KSIDE ? WS * 4 * TR : 0);  // pass 4, d = 128: ddV rows of each wave
  const int64_t srow = (int64_t)bh * p.n_q;

#pragma unroll 1
  for (int half = 0; half < (MASKED ? 2 : 1); half++) {
  const int tile = half ? n_tiles - 1 - unit : unit;
  if (half && tile == unit) break;   // odd number of tiles: the middle one stands alone
  const int r0 = tile * TR * nw, rw = r0 + TR * wave, ri = rw + n;

  f32x4_t res[NREG][J];
#pragma unroll
  for (int x = 0; x < NREG; x++) load_resident<T, D>(res[x], sta[x], sta_ld, ri, n_sta, h);
  if (LAST_IN_LDS) {
    float* mine = sta_lds + wave * TF;
    for (int v = lane; v < TR * (D / 4); v += 64) {
      const int r = v / (D / 4), c = (v % (D / 4)) * 4;
      f32x4_t x = {0.f, 0.f, 0.f, 0.f};
      if (rw + r < n_sta) x = load4<T>(sta[3] + (int64_t)(rw + r) * sta_ld + c);
      *reinterpret_cast<f32x4_t*>(mine + r * Tile<D>::LD + c) = x;
    }
  }

  // row statistics of a query: per lane in passes 1-3, per register (from LDS) in pass 4
  const bool rok = ri < n_sta;
  float L = 0.f, dsum = 0.f, dd = 0.f, b = 0.f;
  if (!KSIDE && rok) {
    L = p.lse[srow + ri];
    if (PASS >= 2) dsum = p.ws_d[srow + ri], dd = p.ws_dd[srow + ri];
    if (PASS >= 3) b = p.ws_b[srow + ri];
  }

  float red = 0.f;
  f32x16_t acc0[CB], acc1[CB];   // dQ2, ddO | dK2, dV2
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

  // Streaming: up to d = 64 the next tile is fetched into registers while this one is computed on and written to
  // LDS behind the step (PRE f32x4 per tensor and thread); at d = 128 the registers are taken and the tile is
  // loaded between two barriers.
  constexpr bool PREFETCH = D <= 64 && WS == 1;
  constexpr int C4 = D / 4, PRE = PREFETCH ? TR * C4 / nthr : 1;
  f32x4_t pre[NT][PRE];
  float pre_stat = 0.f;
  // pass 4: thread t < 128 carries statistic t / 32 (L, d, dd, b) of streamed query t % 32
  const float* stat_src = p.lse;
  if ((tid >> 5) == 1) stat_src = p.ws_d;
  if ((tid >> 5) == 2) stat_src = p.ws_dd;
  if ((tid >> 5) == 3) stat_src = p.ws_b;
  stat_src += srow;
  auto fetch = [&](int s0) {
#pragma unroll
    for (int x = 0; x < NT; x++)
#pragma unroll
      for (int c = 0; c < PRE; c++) {
        const int v = tid + c * nthr, r = v / C4, col = (v % C4) * 4;
        f32x4_t val = {0.f, 0.f, 0.f, 0.f};
        if (s0 + r < n_str) val = load4<T>(str[x] + (int64_t)(s0 + r) * str_ld + col);
        pre[x][c] = val;
      }
    if (KSIDE && tid < 4 * TR) {
      const int qi = s0 + (tid & 31);
      pre_stat = qi < p.n_q ? stat_src[qi] : 0.f;
    }
  };
  auto publish = [&]() {
#pragma unroll
    for (int x = 0; x < NT; x++)
#pragma unroll
      for (int c = 0; c < PRE; c++) {
        const int v = tid + c * nthr, r = v / C4, col = (v % C4) * 4;
        *reinterpret_cast<f32x4_t*>(tiles + x * TF + r * Tile<D>::LD + col) = pre[x][c];
      }
    if (KSIDE && tid < 4 * TR) stat[tid] = pre_stat;
  };
  if (PREFETCH && s_begin < s_end) {
    __syncthreads();   // the tiles of the other half are no longer read
    fetch(s_begin);
    publish();
  }

  for (int sb = s_begin; sb < s_end; sb += WS * TR) {
    __syncthreads();
    if (PREFETCH) {
      if (sb + TR < s_end) fetch(sb + TR);
    } else {
#pragma unroll
      for (int g = 0; g < WS; g++) {   // stage g holds the tile of the waves with ws == g
        float* tg = tiles + g * NT * TF;
        load_tile_pair<T, D>(tg, tg + TF, str[0], str[1], str_ld, sb + g * TR, n_str, tid);
        if (NT > 2) load_tile_pair<T, D>(tg + 2 * TF, tg + (NT - 1) * TF, str[2], str[NT - 1], str_ld, sb + g * TR, n_str, tid);
        if (KSIDE && tid < 4 * TR) {
          const int qi = sb + g * TR + (tid & 31);
          stat[g * 4 * TR + tid] = qi < p.n_q ? stat_src[qi] : 0.f;
        }
      }
      __syncthreads();
    }
    const int s0 = sb + ws * TR;
    const float* const tiles = smem + ws * NT * TF;
    const float* const stat = smem + WS * NT * TF + ws * 4 * TR;
    [&]() {
    if (WS > 1 && s0 >= s_end) return;   // the last round of tiles may be short
    // Every pair of this wave's rows with this tile hidden: nothing to add. Not at d = 128, where the extra loop
    // edge makes the register allocator spill; there the element mask alone zeroes the block.
    bool dead = false;
    if (MASKED && D < 128) {
      const int64_t q_lo = KSIDE ? s0 : rw, q_hi = (KSIDE ? s0 : rw) + TR - 1;   // queries of the block
      const int64_t k_lo = KSIDE ? rw : s0, k_hi = (KSIDE ? rw : s0) + TR - 1;   // keys of the block
      dead = k_lo > q_hi + p.mask_off || q_lo + p.mask_off - k_hi >= p.window;
    }
    if (D < 128 && rw >= n_sta) dead = true;   // a wave without rows
    if (dead) return;

    const f32x16_t zero = {0};
    const float* t0 = tiles;            // K   | Q
    const float* t1 = tiles + TF;       // ddK | ddQ
    const float* t2 = tiles + 2 * TF;   // V   | dO
    const float* t3 = tiles + 3 * TF;   // ddV | -
    f32x16_t sv, dds, pv;
    if (!KSIDE) {
      sv = mma_first<D>(zero, t0, res[0], lane);                 // K Q^T
      dds = mma_first<D>(zero, t0, res[1], lane);                // K ddQ^T
      dds = mma_first<D>(dds, t1, res[0], lane);                 // + ddK Q^T
    } else {
      sv = mma_first<D>(zero, t0, res[0], lane);                 // Q K^T
      dds = mma_first<D>(zero, t1, res[0], lane);                // ddQ K^T
      dds = mma_first<D>(dds, t0, res[1], lane);                 // + Q ddK^T
    }
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int m = 8 * (r / 4) + 4 * h + (r % 4);
      const int qi = KSIDE ? s0 + m : ri, kj = KSIDE ? ri : s0 + m;
      bool valid = qi < p.n_q && kj < p.n_k;
      if (MASKED) valid = valid && (kj <= qi + p.mask_off) && (qi + p.mask_off - kj < p.window);
      const float Lr = KSIDE ? stat[m] : L;
      pv[r] = valid ? __builtin_amdgcn_exp2f((sv[r] * p.scale - Lr) * kLog2e) : 0.f;
      dds[r] *= p.scale;
    }
    if (PASS == 1) {
#pragma unroll
      for (int r = 0; r < 16; r++) red += pv[r] * dds[r];
      return;
    }
    f32x16_t w;
    if (PASS >= 3) {
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const float ddr = KSIDE ? stat[2 * TR + 8 * (r / 4) + 4 * h + (r % 4)] : dd;
        w[r] = pv[r] * (dds[r] - ddr);                            // ddP
      }
      mma_second<D>(acc1, w, t2, lane);                          // ddO += ddP V | dV2 += ddP^T dO
      if (!KSIDE) mma_second<D>(acc1, pv, t3, lane);             // ddO += P ddV
    }
    f32x16_t dp = KSIDE ? mma_first<D>(zero, t2, res[2], lane)    // dO V^T
                        : mma_first<D>(zero, t2, res[2], lane);   // V dO^T
    if (PASS >= 3) {
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const float dr = KSIDE ? stat[TR + 8 * (r / 4) + 4 * h + (r % 4)] : dsum;
        w[r] = p.scale * pv[r] * (dp[r] - dr);                    // dS
      }
      mma_second<D>(acc0, w, t1, lane);                          // dQ2 += dS ddK | dK2 += dS^T ddQ
    }
    f32x16_t e;
    if (!KSIDE) e = mma_first<D>(zero, t3, res[2], lane);         // ddV dO^T
    else if (LAST_IN_LDS) e = mma_first_lds<D>(zero, t2, sta_lds + wave * TF, lane);
    else e = mma_first<D>(zero, t2, res[NREG - 1], lane);         // dO ddV^T
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int m = 8 * (r / 4) + 4 * h + (r % 4);
      const float dr = KSIDE ? stat[TR + m] : dsum, ddr = KSIDE ? stat[2 * TR + m] : dd, br = KSIDE ? stat[3 * TR + m] : b;
      const float dp2 = e[r] - dp[r] * ddr - dds[r] * dr + dp[r] * dds[r];
      if (PASS == 2) red += pv[r] * dp2;
      else w[r] = p.scale * pv[r] * (dp2 - br);                   // dS'
    }
    if (PASS >= 3) mma_second<D>(acc0, w, t0, lane);             // dQ2 += dS' K | dK2 += dS'^T Q
    }();
    if (PREFETCH && sb + TR < s_end) {
      __syncthreads();   // every wave is done reading the tile
      publish();
    }
  }

  if (WS > 1) {
    // the WS waves of a row group add their partial results through LDS in the order of ws; the wave with ws == 0
    // holds the sum and stores it
    __syncthreads();   // the streamed tiles are no longer read
    float* xch = smem + ((wave * (WS - 1) + (ws - 1)) * (PASS <= 2 ? 1 : 2 * CB * 16)) * 64 + lane;
    if (ws > 0) {
      if (PASS <= 2) {
        xch[0] = red;
      } else {
#pragma unroll
        for (int cb = 0; cb < CB; cb++)
#pragma unroll
          for (int r = 0; r < 16; r++) xch[(cb * 16 + r) * 64] = acc0[cb][r], xch[((CB + cb) * 16 + r) * 64] = acc1[cb][r];
      }
    }
    __syncthreads();
    if (ws > 0) continue;
#pragma unroll
    for (int o = 1; o < WS; o++) {
      const float* src = smem + ((wave * (WS - 1) + (o - 1)) * (PASS <= 2 ? 1 : 2 * CB * 16)) * 64 + lane;
      if (PASS <= 2) {
        red += src[0];
      } else {
#pragma unroll
        for (int cb = 0; cb < CB; cb++)
#pragma unroll
          for (int r = 0; r < 16; r++) acc0[cb][r] += src[(cb * 16 + r) * 64], acc1[cb][r] += src[((CB + cb) * 16 + r) * 64];
      }
    }
  }

  if (PASS == 1 || PASS == 2) {
    red += __shfl_xor(red, 32);
    if (h == 0 && rok) (PASS == 1 ? p.ws_dd : p.ws_b)[srow + ri] = red;
  } else if (PASS == 3) {
    store_acc<T, D>((T*)p.dq2 + qoff, p.stride_qn, ri, p.n_q, acc0, h);
    store_acc<T, D>((T*)p.ddo + qoff, p.stride_qn, ri, p.n_q, acc1, h);
  } else {
    store_acc<T, D>((T*)p.dk2 + koff, p.stride_kn, ri, p.n_k, acc0, h);
    store_acc<T, D>((T*)p.dv2 + koff, p.stride_kn, ri, p.n_k, acc1, h);
  }
  }  // half
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

template <typename T, int D, int PASS, bool MASKED, int WS>
hipError_t launch_sweep_ws(const Params& p, hipStream_t s) {
  constexpr bool KSIDE = PASS == 4;
  constexpr int NT = PASS == 1 ? 2 : (KSIDE ? 3 : 4);
  const int64_t n_rows = KSIDE ? p.n_k : p.n_q;
  constexpr int nw = 4 / WS;   // 32-row groups per workgroup
  size_t floats = (size_t)WS * NT * Tile<D>::FLOATS + (KSIDE ? WS * 4 * TR : 0);
  if (KSIDE && D == 128) floats += (size_t)nw * Tile<D>::FLOATS;
  const int smem = (int)(floats * sizeof(float));
  const int n_tiles = (int)((n_rows + TR * nw - 1) / (TR * nw));
  const dim3 grid(bf16k::grid_blocks(MASKED ? (n_tiles + 1) / 2 : n_tiles, p.batch)), block(256);
  const hipError_t e = allow_dynamic_lds<sweep_fp32<T, D, PASS, MASKED, WS>>(smem);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL((sweep_fp32<T, D, PASS, MASKED, WS>), grid, block, smem, s, p);
  return hipGetLastError();
}

// Four waves on 128 stationary rows is the best shape whenever that fills the GPU (the waves share the streamed tiles
// and their loads). A launch with fewer than 128 such workgroups (256 CUs) puts two or four waves on the same 32 rows
// instead (d <= 64: the stages of all waves have to fit the LDS): a 256-token problem of two heads is 4 workgroups
// otherwise, each running its eight streamed tiles one after the other.
template <typename T, int D, int PASS, bool MASKED>
hipError_t launch_sweep(const Params& p, hipStream_t s) {
  if constexpr (D <= 64) {
    const int64_t n_rows = PASS == 4 ? p.n_k : p.n_q, n_str = PASS == 4 ? p.n_q : p.n_k;
    const int64_t groups = (n_rows + 127) / 128 * p.batch / (MASKED ? 2 : 1);
    if (groups < 64 && n_str > 2 * TR) return launch_sweep_ws<T, D, PASS, MASKED, 4>(p, s);
    if (groups < 128 && n_str > TR) return launch_sweep_ws<T, D, PASS, MASKED, 2>(p, s);
  }
  return launch_sweep_ws<T, D, PASS, MASKED, 1>(p, s);
}

template <typename T, int D>
hipError_t launch_pass_td(const Params& p, int pass, hipStream_t s) {
  switch (pass) {
    case FHOG_PASS_DD: return p.causal ? launch_sweep<T, D, 1, true>(p, s) : launch_sweep<T, D, 1, false>(p, s);
    case FHOG_PASS_B: return p.causal ? launch_sweep<T, D, 2, true>(p, s) : launch_sweep<T, D, 2, false>(p, s);
    case FHOG_PASS_DQ_DDO: return p.causal ? launch_sweep<T, D, 3, true>(p, s) : launch_sweep<T, D, 3, false>(p, s);
    case FHOG_PASS_DK_DV: return p.causal ? launch_sweep<T, D, 4, true>(p, s) : launch_sweep<T, D, 4, false>(p, s);
    default: return hipErrorInvalidValue;
  }
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
