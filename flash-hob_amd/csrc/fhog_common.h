// Shared device/host declarations of libfhog_hip.so (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "fhog_hip.h"

namespace fhog {

typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4_t;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t u32x2_t;

constexpr float kLog2e = 1.4426950408889634f;

// Kernel-side view of fhog_bwdbwd_args (same fields, typed for device code).
struct Params {
  const void* q;
  const void* k;
  const void* v;
  const void* o;
  const void* dO;
  const void* ddq;
  const void* ddk;
  const void* ddv;
  const float* lse;
  void* dq2;
  void* dk2;
  void* dv2;
  void* ddo;
  float* ws_d;   // (batch, n_q)
  float* ws_dd;  // (batch, n_q)
  float* ws_b;   // (batch, n_q)
  int64_t stride_qb, stride_qn, stride_kb, stride_kn;
  int32_t batch, n_q, n_k, d;
  float scale;
  int32_t causal;    // some mask is set
  int32_t f16;       // 16-bit tensors are fp16 (else bf16); read by the 16-bit MFMA family only
  int32_t mask_off;  // key j is visible to query i iff 0 <= i + mask_off - j < window
  int32_t window;
  // Streamed side split over n_split workgroups per stationary tile (1 = no split): each writes fp32 partial results
  // to `part` and a combining kernel finishes the pass. Set per pass by the caller of the launchers (16-bit kernels,
  // both head dims).
  int32_t n_split;
  float* part;
  // Workgroup ids of one XCD enumerate its tiles (decode_block). tile_major: the slices that share the XCD advance
  // through their tiles together instead of one slice after the other (the default with a mask).
  int32_t tile_major;
};

// Launch choices that can be overridden for experiments through the environment variable FHOG_TUNE, a comma-separated
// list of key=value (read once, on the host, at the first launch; never in a timed path):
//   b8=0|1             b / dd+b sweeps at d = 128: 128-row workgroups of 4 waves | 256-row workgroups of 8 waves
//                      (default: 8 waves when that still gives 512 workgroups)
//   order=slice|tile   workgroup order within an XCD (default: tile-major with a mask, slice after slice without)
//   split=0|1          let launches too small to fill the GPU split their streamed side over several workgroups (default 1)
//   dd64=0|1           dd sweep at d = 128: 32 | 64 queries per wave (default: 64 when that still gives 2048 workgroups)
//   stage64=0|1        single-role sweeps at d = 64: one | two 32-row tiles staged and consumed per barrier (default 0: measured equal within 1 %)
//   stage1=0|1         d = 64, reference schedule: sweeps 1-3 as three launches | as one launch whose workgroups run them one
//                      after the other for their tile (FHOG_PASS_STAGE1)
struct Tuning {
  int b8 = -1, order = -1, split = 1, dd64 = -1, stage64 = 0, stage1 = 0;
};
const Tuning& tuning();

// Kernel-side view of fhog_attn_args (first-order forward and backward).
struct AttnParams {
  const void* q;
  const void* k;
  const void* v;
  void* o;        // forward: written; backward: read
  float* lse;     // forward: written; backward: read
  const void* dO; // backward only
  void* dq;
  void* dk;
  void* dv;
  float* ws_d;    // backward: (batch, n_q) row sums of O * dO
  int64_t stride_qb, stride_qn, stride_kb, stride_kn;
  int32_t batch, n_q, n_k, d;
  float scale;
  int32_t causal;    // some mask is set
  int32_t f16;       // tensors are fp16 (else bf16)
  int32_t mask_off;  // key j is visible to query i iff 0 <= i + mask_off - j < window
  int32_t window;
  // Workgroup order within an XCD for the Q-tiled kernels (forward, dQ) and the K-tiled one (dK, dV): see Params
  int32_t tile_major_q, tile_major_k;
};

// A kernel that uses more than 64 KiB of dynamic LDS needs its limit raised before the first launch. Done once per
// kernel and device (not per launch: the call takes a lock in the runtime and must not run under stream capture, so
// the first launch of a kernel on a device has to happen outside a capture).
template <auto Kernel>
inline hipError_t allow_dynamic_lds(int bytes) {
  constexpr int kDevices = 64;
  static std::atomic<int> granted[kDevices];   // zero-initialised: nothing granted yet
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const bool memo = dev >= 0 && dev < kDevices;
  if (memo && granted[dev].load(std::memory_order_acquire) >= bytes) return hipSuccess;
  e = hipFuncSetAttribute((const void*)Kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess && memo) granted[dev].store(bytes, std::memory_order_release);
  return e;
}

// Launchers implemented in the kernel translation units. Each returns hipGetLastError().
hipError_t launch_rowdot(const Params& p, int dtype, hipStream_t s);                 // pass 0
hipError_t launch_fp32_pass(const Params& p, int dtype, int pass, hipStream_t s);   // passes 1..4, fp32 MFMA
hipError_t launch_bf16_pass(const Params& p, int pass, hipStream_t s);              // passes 1..4, bf16 MFMA
hipError_t launch_attn_bf16(const AttnParams& p, int which, hipStream_t s);         // 0 forward, 1 dQ, 2 dK and dV
hipError_t launch_attn_fp32(const AttnParams& p, int dtype, int which, hipStream_t s);  // same, fp32 MFMA (fp32 tensors, d = 32)
hipError_t launch_attn_bwd_k_pc(const AttnParams& p, hipStream_t s);                // dK and dV at d = 128 (producer/consumer)
hipError_t launch_mfma_rate(float* out, int blocks, int trips, int data_mode, int waves, hipStream_t s);  // measurement aid
bool bf16_shape_supported(int64_t n_q, int64_t n_k, int64_t d, int causal);

}  // namespace fhog
