// Device helpers shared by the bf16 MFMA kernels (gfx950): LDS tile addressing with the 16-byte
// XOR swizzle, row-wise and transposing LDS operand reads, global->LDS staging, XCD-aware grid decode.
#pragma once
#include "fhog_common.h"

namespace fhog {
namespace bf16k {

constexpr int WG_ROWS = 128;  // stationary rows per workgroup (4 waves x 32)
constexpr int TS = 32;        // streamed rows per LDS stage

typedef __attribute__((address_space(3))) bf16x4_t* lds_bf16x4_ptr;

// ---- LDS tile addressing ------------------------------------------------------------------
// A tile holds TS rows of D bf16 (2*D bytes per row, no padding). The 16-byte chunk `ch` of row
// `r` is stored at chunk position ch ^ swz(r).
template <int D>
__device__ __forceinline__ int swz(int r) {
  if (D == 128) return ((r & 3) << 2) | ((r >> 2) & 3);
  return (((r >> 1) & 1) << 2) | ((r >> 2) & 3);
}
template <int D>
__device__ __forceinline__ int tile_off(int r, int ch) {
  return r * (2 * D) + ((ch ^ swz<D>(r)) << 4);
}

__device__ __forceinline__ bf16x8_t lds_read128(const char* smem, int off) {
  return *reinterpret_cast<const bf16x8_t*>(smem + off);
}

// Transposed (second-level) operand of the 32-column block `cb`, read with ds_read_b64_tr_b16 from a 32-row tile:
// two 8-byte transposing reads, one per group of 4 rows; within a 16-lane group lane i addresses row (i>>2), columns
// 4*(i&3)..+3, and receives column i of the 4 x 16 block. The other operand of such a contraction is always an
// S-shaped accumulator (in registers, or handed over through an operand tile), whose k-step t holds, in lane half h,
// the streamed rows 16t + 4h + 0..3 and then 16t + 8 + 4h + 0..3 (accumulator registers 8t .. 8t+7). So lane
// (col = lane%32, h = lane/32) fetches rows 4h + 0..3 with the first read (s = 0) and rows 8 + 4h + 0..3 with the
// second (s = 1) of the 16-row step, at column cb*32 + col. The per-lane part of the address does not depend on t and
// is precomputed; step t adds 16 rows.
template <int D>
__device__ __forceinline__ int tr_lane_off_acc(int cb, int s, int lane) {
  const int i = lane & 15, b = (lane >> 4) & 1, h = lane >> 5;
  const int col = cb * 32 + 16 * b + 4 * (i & 3);
  const int r = 8 * s + 4 * h + (i >> 2);
  return tile_off<D>(r, col >> 3) + ((col >> 2) & 1) * 8;
}
// p0 / p1: stage base + tr_lane_off_acc(cb, 0 / 1); `imm` = tensor offset + t * 16 rows (compile-time)
__device__ __forceinline__ bf16x8_t lds_read_tr_pre(const char* p0, const char* p1, int imm) {
  bf16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4_ptr)(p0 + imm));
  bf16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4_ptr)(p1 + imm));
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// ---- fp32 -> 16-bit tensor type (bf16, or fp16 when F16), round to nearest even ---------------------------
template <bool F16>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  if constexpr (F16) {
    typedef __attribute__((__vector_size__(2 * sizeof(_Float16)))) _Float16 f16x2_t;
    f16x2_t v = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(uint32_t, v);
  } else {
    typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
    bf16x2_t v = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, v);
  }
}
template <bool F16>
__device__ __forceinline__ u32x2_t pack4(float a, float b, float c, float d) {
  return u32x2_t{pack2<F16>(a, b), pack2<F16>(c, d)};
}
template <bool F16>
__device__ __forceinline__ uint16_t to_elem(float x) {
  if constexpr (F16) return __builtin_bit_cast(uint16_t, (_Float16)x);
  else return __builtin_bit_cast(uint16_t, (__bf16)x);
}

// element of a 16-bit carrier vector (bf16 bits, or fp16 bits when F16) as fp32
template <bool F16>
__device__ __forceinline__ float to_f32(__bf16 x) {
  if constexpr (F16) return (float)__builtin_bit_cast(_Float16, x);
  else return (float)x;
}

// registers 8t .. 8t+7 of an S-shaped fp32 tile as the 16-bit B operand of second-level k-step t (in registers)
template <bool F16>
__device__ __forceinline__ bf16x8_t pack_operand(const f32x16_t& x, int t) {
  u32x4_t u = {pack2<F16>(x[8 * t + 0], x[8 * t + 1]), pack2<F16>(x[8 * t + 2], x[8 * t + 3]),
               pack2<F16>(x[8 * t + 4], x[8 * t + 5]), pack2<F16>(x[8 * t + 6], x[8 * t + 7])};
  return __builtin_bit_cast(bf16x8_t, u);
}

// ---- S-shaped bf16 operand tiles handed from producer to consumer waves through LDS ------------
// 32 stationary rows x 32 streamed rows, 64 bytes per row, 16-byte chunks XOR-swizzled by sop_swz(row).
// Chunk 2t + h of row n holds accumulator registers 8t .. 8t+7 of lane (n, h), i.e. the streamed rows
// 16t + 4h + 0..3 and 16t + 8 + 4h + 0..3: one 128-bit write per k-step on the producer side, one 128-bit read on
// the consumer side, whose other operand enumerates the streamed rows in the same order (tr_lane_off_acc).
// The swizzle keeps both free of bank conflicts, as measured on gfx950 with pairs of active lanes: a 128-bit LDS
// write serves 8 consecutive lanes per cycle and addresses 128 bytes apart collide, so the rows n, n+2, n+4, n+6 of
// such a group need four different chunk positions; a 128-bit read serves the lanes {0-3, 12-15, 20-23, 24-27} (and
// {4-11, 16-19, 28-31}) of a half-wave together, with addresses 256 bytes apart colliding, so rows with equal n % 4
// need different positions across n / 4 in {0, 3, 5, 6} and in {1, 2, 4, 7}.
constexpr int SOP_TILE = 32 * 64;
__device__ __forceinline__ int sop_swz(int n) { return ((n >> 2) & 3) ^ (n & 2); }
// producer: registers 8t .. 8t+7 of stationary row n as four packed pairs
__device__ __forceinline__ void sop_write_step(char* tile, u32x4_t pk, int t, int lane) {
  const int n = lane & 31, h = lane >> 5;
  *reinterpret_cast<u32x4_t*>(tile + n * 64 + (((2 * t + h) ^ sop_swz(n)) << 4)) = pk;
}
// consumer: A operand of second-level step t: stationary row n, streamed rows in the order given above
__device__ __forceinline__ bf16x8_t sop_read(const char* tile, int t, int lane) {
  const int n = lane & 31, h = lane >> 5;
  return *reinterpret_cast<const bf16x8_t*>(tile + n * 64 + (((2 * t + h) ^ sop_swz(n)) << 4));
}

// The kernels carry 16-bit operands as bf16x8_t whatever the tensor type; F16 selects the instruction.
template <bool F16>
__device__ __forceinline__ f32x16_t mfma(bf16x8_t a, bf16x8_t b, f32x16_t c) {
  if constexpr (F16) {
    typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8_t;
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
}

// ---- direct global -> LDS staging (no registers): global_load_lds_dwordx4 ------------------------
// One wave instruction moves 64 x 16 bytes to 1 KiB of contiguous LDS at M0 (lane l lands at
// M0 + 16*l). The destination is therefore linear; the swizzle is applied on the SOURCE side: the lane
// that lands on chunk position pc of row r fetches chunk pc ^ swz(r) of that row.
// The load is issued from inline asm, so the compiler does not track it: the caller must execute
// dma_wait() before the barrier that publishes the tile.
template <int D>
struct Dma {
  static constexpr int CPR = D / 8;             // 16-byte chunks per row
  static constexpr int RPI = 64 / CPR;          // rows per instruction (4 at d=128, 8 at d=64)
  static constexpr int IPT = TS / RPI;          // instructions per 32-row tile (8 or 4)
  static constexpr int PER_WAVE = IPT / 4;      // instructions per tile for each of 4 loader waves (2 or 1)
  uint32_t voff[PER_WAVE];                      // per-lane byte offset from the tile's first row
  int64_t ld_;
  int lw_, lane_;

  __device__ __forceinline__ uint32_t lane_offset(int u, int rows_valid) const {
    const int q = lw_ + 4 * u;
    const int r = q * RPI + lane_ / CPR, pc = lane_ % CPR;
    const int rs = r < rows_valid ? r : rows_valid - 1;  // rows past the end of the tensor re-read its last row
    return (uint32_t)((rs * ld_ + ((pc ^ swz<D>(r)) << 3)) * 2);
  }
  __device__ __forceinline__ void init(int64_t ld, int lw, int lane) {
    ld_ = ld;
    lw_ = lw;
    lane_ = lane;
#pragma unroll
    for (int u = 0; u < PER_WAVE; u++) voff[u] = lane_offset(u, TS);
  }
  // tile_lds: LDS byte address of the destination tile (wave-uniform); src + adv: first row of the source tile;
  // rows_valid: rows of the tensor from that row on (>= TS for a full tile). A partial tile is filled up with copies of
  // the tensor's last row, so that no load leaves the tensor; the kernels mask those rows.
  // N tiles of the same rows from N tensors: tensor x goes to tile_lds + x * tile_stride and starts at src[x] + adv.
  // ONE scalar branch decides between the precomputed offsets and the clamped ones of a partial tile, so the common
  // case costs no vector work.
  template <int N, int NSRC>
  __device__ __forceinline__ void issue_all(uint32_t tile_lds, int tile_stride, const __bf16* const (&src)[NSRC], int64_t adv,
                                            int lw, int rows_valid) const {
    static_assert(N <= NSRC, "more tiles than tensors");
    if (__builtin_amdgcn_readfirstlane(rows_valid) >= TS) {
#pragma unroll
      for (int x = 0; x < N; x++)
#pragma unroll
        for (int u = 0; u < PER_WAVE; u++) issue_one(tile_lds + x * tile_stride + (lw + 4 * u) * 1024, voff[u], src[x] + adv);
    } else {
      uint32_t off[PER_WAVE];
#pragma unroll
      for (int u = 0; u < PER_WAVE; u++) off[u] = lane_offset(u, rows_valid);
#pragma unroll
      for (int x = 0; x < N; x++)
#pragma unroll
        for (int u = 0; u < PER_WAVE; u++) issue_one(tile_lds + x * tile_stride + (lw + 4 * u) * 1024, off[u], src[x] + adv);
    }
  }
  // M0 is on the clobber list: the compiler never allocates it, but it does write it ahead of instructions of its own
  // that read it and may share one such write between several of them; the list tells it that this statement changes
  // the register in between (clang warns about any reserved register on a clobber list; the warning is switched off here).
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
  __device__ __forceinline__ static void issue_one(uint32_t lds, uint32_t off, const __bf16* src_) {
    const uint32_t m0 = __builtin_amdgcn_readfirstlane(lds);
    // the base address is wave-uniform; say so, or the "s" operand may be handed a vector register pair
    // (the builtin returns a signed int: the halves are kept unsigned)
    const uint64_t a = (uint64_t)src_;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a), hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
    const __bf16* src = (const __bf16*)(((uint64_t)hi << 32) | lo);
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2\n\t" ::"s"(m0), "v"(off), "s"(src) : "memory", "m0");
  }
#pragma clang diagnostic pop
};
__device__ __forceinline__ void dma_wait() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
// s_waitcnt vmcnt(0) as a builtin (gfx9 encoding: vmcnt 0, expcnt 7, lgkmcnt 15), which the compiler's wait-count
// pass takes into account: register loads issued before it are known to have landed.
__device__ __forceinline__ void wait_vm0() { __builtin_amdgcn_s_waitcnt(0x0F70); }
typedef const __attribute__((address_space(1))) float* global_f32_ptr;
__device__ __forceinline__ uint32_t lds_addr(const char* p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)p;
}

// B operands of the stationary rows: lane (n = lane%32, h) holds row n, elements 16kk + 8h .. +7.
template <int D>
__device__ __forceinline__ void load_resident(bf16x8_t* dst, const __bf16* base, int64_t ld, int row, int h) {
  const __bf16* p = base + (int64_t)row * ld + 8 * h;
#pragma unroll
  for (int kk = 0; kk < D / 16; kk++) dst[kk] = *reinterpret_cast<const bf16x8_t*>(p + 16 * kk);
}

// ---- mask geometry ------------------------------------------------------------------------------------------
// Key j is visible to query i iff 0 <= i + off - j < win (off = 0: top-left causal, off = n_k - n_q: bottom-right;
// win >= n_q + n_k: no window), and rows past the end of a tensor never count.
// The kernels are compiled for three mask modes, so that the common cases carry no arithmetic they do not need:
constexpr int MASK_NONE = 0;    // only the tensor ends
constexpr int MASK_CAUSAL = 1;  // off = 0 and no window, known at compile time (the square causal mask)
constexpr int MASK_BAND = 2;    // off and win from the arguments
// "Streamed" rows come in 32-row tiles starting at t0; "stationary" rows are the 32 rows of a wave starting at r0
// (or the rows [r0, r0 + nrows) of a workgroup for the tile range).
//
// StreamKeys: stationary rows are queries, streamed tiles are keys (statistics sweeps, pass 3, forward, dQ).
template <int MASK>
struct StreamKeys {
  int off, win, n_k;
  __device__ __forceinline__ StreamKeys(int off_, int win_, int n_k_)
      : off(MASK == MASK_BAND ? off_ : 0), win(MASK == MASK_BAND ? win_ : (1 << 28)), n_k(n_k_) {}
  // tiles [lo, hi) hold a visible key for some query of [r0, r0 + nrows)
  __device__ __forceinline__ void tile_range(int r0, int nrows, int& lo, int& hi) const {
    const int k_tiles = (n_k + TS - 1) / TS;
    lo = MASK == MASK_BAND ? max(0, r0 + off - win + 1) / TS : 0;
    hi = MASK != MASK_NONE ? min(k_tiles, (r0 + nrows - 1 + off) / TS + 1) : k_tiles;
  }
  // no key of tile t0 is visible to any query of [r0, r0 + 32)
  __device__ __forceinline__ bool dead(int t0, int r0) const {
    if (MASK == MASK_NONE) return false;
    return t0 > r0 + 31 + off || (MASK == MASK_BAND && t0 + TS - 1 < r0 + off - win + 1);
  }
  // some key of tile t0 is hidden from some query of [r0, r0 + 32)
  __device__ __forceinline__ bool partial(int t0, int r0) const {
    if (t0 + TS > n_k) return true;
    if (MASK == MASK_NONE) return false;
    return t0 + TS - 1 > r0 + off || (MASK == MASK_BAND && t0 < r0 + 31 + off - win + 1);
  }
  // key t0 + 8g + 4h + e is visible to query i iff lo <= 8g + e <= hi
  __device__ __forceinline__ void limits(int t0, int i, int h, int& lo, int& hi) const {
    hi = min(MASK != MASK_NONE ? i + off - t0 : TS, n_k - 1 - t0) - 4 * h;
    lo = MASK == MASK_BAND ? i + off - win + 1 - t0 - 4 * h : -TS;
  }
};
// StreamQueries: stationary rows are keys, streamed tiles are queries (pass 4, dK and dV).
template <int MASK>
struct StreamQueries {
  int off, win, n_q;
  __device__ __forceinline__ StreamQueries(int off_, int win_, int n_q_)
      : off(MASK == MASK_BAND ? off_ : 0), win(MASK == MASK_BAND ? win_ : (1 << 28)), n_q(n_q_) {}
  __device__ __forceinline__ void tile_range(int r0, int nrows, int& lo, int& hi) const {
    const int q_tiles = (n_q + TS - 1) / TS;
    lo = MASK != MASK_NONE ? max(0, r0 - off) / TS : 0;
    hi = MASK == MASK_BAND ? (int)min((int64_t)q_tiles, ((int64_t)r0 + nrows - 1 - off + win - 1) / TS + 1) : q_tiles;
    hi = max(hi, lo);
  }
  __device__ __forceinline__ bool dead(int t0, int r0) const {
    if (MASK == MASK_NONE) return false;
    return t0 + TS - 1 < r0 - off || (MASK == MASK_BAND && t0 > r0 + 31 - off + win - 1);
  }
  __device__ __forceinline__ bool partial(int t0, int r0) const {
    if (t0 + TS > n_q) return true;
    if (MASK == MASK_NONE) return false;
    return t0 < r0 + 31 - off || (MASK == MASK_BAND && t0 + TS - 1 > r0 - off + win - 1);
  }
  // query t0 + 8g + 4h + e sees key j iff lo <= 8g + e <= hi
  __device__ __forceinline__ void limits(int t0, int j, int h, int& lo, int& hi) const {
    lo = MASK != MASK_NONE ? j - off - t0 - 4 * h : -TS;
    hi = min(MASK == MASK_BAND ? j - off + win - 1 - t0 : TS, n_q - 1 - t0) - 4 * h;
  }
};
// part `split` of `n` equal parts of the streamed tile range [lo, hi) (the last parts may be empty)
__device__ __forceinline__ void split_range(int split, int n, int& lo, int& hi) {
  const int chunk = (hi - lo + n - 1) / n;
  lo = min(hi, lo + split * chunk);
  hi = min(hi, lo + chunk);
}
// mask mode of a launch (Params or AttnParams)
template <typename P>
inline int mask_mode(const P& p) {
  if (!p.causal) return MASK_NONE;
  return (p.mask_off == 0 && p.window >= p.n_q + p.n_k) ? MASK_CAUSAL : MASK_BAND;
}

// Placed at the top of a rarely taken wave-uniform branch: keeps the compiler from turning the branch into
// unconditional selects that every step would pay for.
__device__ __forceinline__ void keep_branch() { asm volatile("" ::: "memory"); }
__device__ __forceinline__ bool in_limits(int r, int lo, int hi) {  // r: register index of an S-shaped tile
  const int x = 8 * (r / 4) + (r % 4);
  return x >= lo && x <= hi;
}

// XCD-aware 1-D grid. Workgroup ids go round-robin over the 8 XCDs (id % 8 = XCD), each with its own L2.
// With 8 or more (batch*head) slices every slice is pinned to one XCD, so that all its tiles stream the slice's
// other side through ONE L2. With fewer slices a slice is spread over 8/batch (rounded down to a power of two)
// XCDs, tiles interleaved, so that a single long head still fills the chip.
//   xcds_per_slice XS = 8, 4, 2, 2, 1, ... for batch = 1, 2, 3, 4, >= 5;  slices per round = 8 / XS
__host__ __device__ __forceinline__ int xcds_per_slice(int batch) { return batch >= 5 ? 1 : batch >= 3 ? 2 : batch == 2 ? 4 : 8; }
// number of workgroups to launch for n_tiles tiles per slice
__host__ __forceinline__ unsigned grid_blocks(int n_tiles, int batch) {
  const int xs = xcds_per_slice(batch), per_round = 8 / xs;
  const int rounds = (batch + per_round - 1) / per_round, tiles_per_xcd = (n_tiles + xs - 1) / xs;
  return (unsigned)(rounds * 8 * tiles_per_xcd);
}
// Returns false when the id falls beyond the last slice or tile.
// tile_major: the slices that share an XCD advance through their tiles together (ids enumerate tile 0 of every
// slice, then tile 1 of every slice, ...) instead of one slice after the other. With a mask the work of a tile grows
// with its index; heaviest-first over ALL workgroups of the XCD is what lets the light tiles at the end fill the
// gaps (one slice after the other leaves the last slice's heavy tiles alone at the end whenever the XCD holds more
// resident workgroups than a slice has tiles). All workgroups stream the other side from its first tile on, so the
// slices still move through L2 together.
__device__ __forceinline__ bool decode_block(int n_tiles, int batch, bool heavy_first, bool tile_major, int& bh, int& tile) {
  const int id = blockIdx.x;
  const int xcd = id & 7, slot = id >> 3;
  const int xs = xcds_per_slice(batch), per_round = 8 / xs, tiles_per_xcd = (n_tiles + xs - 1) / xs;
  const int rounds = (batch + per_round - 1) / per_round;   // slices this XCD (group) serves
  const int r = tile_major ? slot % rounds : slot / tiles_per_xcd;
  const int t = tile_major ? slot / rounds : slot % tiles_per_xcd;
  bh = xcd / xs + per_round * r;
  tile = t * xs + xcd % xs;
  if (bh >= batch || tile >= n_tiles) return false;
  if (heavy_first) tile = n_tiles - 1 - tile;
  return true;
}

}  // namespace bf16k
}  // namespace fhog
