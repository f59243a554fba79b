/*
 * fhog_hip.h - C ABI of libfhog_hip.so, the MI355X (gfx950) attention double-backward.
 *
 * One call replaces the body of the reference's host wrapper
 *   flash_bwdbwd(Q, K, V, O, dO, ddQ, ddK, ddV, L, scale) -> (dQ2, dK2, dV2, ddO)
 *   (fhog/triton_bwdbwd.py:557-648): the row reduction D = sum(dO*O) (:580), the launch
 *   of bwdbwd_kernel_stage1 (:586-612, kernels :33-313) and of bwdbwd_kernel_stage2
 *   (:620-646, kernels :316-535).
 *
 * Rules of the boundary
 *   - plain C: pointers, integers, floats; no C++ or torch types.
 *   - the library never allocates or frees device memory; the caller owns inputs,
 *     outputs and the workspace (fhog_bwdbwd_workspace_bytes).
 *   - every function returns 0 on success or a negative FHOG_E_* code; nothing throws
 *     or exits; fhog_last_error() gives a thread-local message for the last failure.
 *   - kernels are enqueued on the caller's hipStream_t (passed as void*); the library
 *     never synchronises.
 *   - all tensors are row-major (batch, N, d) with the last dimension contiguous;
 *     the row stride and batch stride (in elements) are given per tensor group.
 */
#ifndef FHOG_HIP_H
#define FHOG_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FHOG_ABI_VERSION 5

/* element types of Q,K,V,O,dO,ddQ,ddK,ddV and of the four outputs */
#define FHOG_DTYPE_BF16 0
#define FHOG_DTYPE_FP32 1
#define FHOG_DTYPE_FP16 2 /* the dtype of the reference's benchmark sweep (fhog/benchhhh.py:15-110) */

/* error codes */
#define FHOG_OK 0
#define FHOG_E_NULL (-1)      /* a required pointer is NULL */
#define FHOG_E_SHAPE (-2)     /* batch/n_q/n_k/d not supported */
#define FHOG_E_DTYPE (-3)     /* unknown dtype */
#define FHOG_E_STRIDE (-4)    /* stride smaller than the row / not a multiple of the vector width / row stride > 2^24 */
#define FHOG_E_ALIGN (-5)     /* pointer not 16-byte aligned */
#define FHOG_E_CAUSAL (-6)    /* mask not applicable: top-left causal with n_q != n_k, bottom-right with n_k < n_q,
                                 a negative window, or a window without a causal mask */
#define FHOG_E_PASS (-7)      /* unknown pass id */
#define FHOG_E_LAUNCH (-8)    /* HIP reported an error at launch */
#define FHOG_E_SCALE (-9)     /* scale is not finite (fhog_attn_fwd / fhog_attn_bwd: not finite or not positive) */
#define FHOG_E_IMPL (-10)     /* unknown kernel family (fhog_bwdbwd_args.impl) */
#define FHOG_E_SCHEDULE (-11) /* unknown pass schedule (fhog_bwdbwd_args.schedule) */

/* pass ids for fhog_bwdbwd_pass */
#define FHOG_PASS_D 0      /* d_i  = sum_c O_ic dO_ic                         (fhog/triton_bwdbwd.py:580)     */
#define FHOG_PASS_DD 1     /* dd_i = sum_j ddS_ij P_ij                        (fhog/triton_bwdbwd.py:185-211);
                              the 16-bit kernels of passes 1 and 5 also write d_i, so fhog_bwdbwd launches pass 0
                              only for the fp32-MFMA family */
#define FHOG_PASS_B 2      /* b_i  = sum_j dP'_ij P_ij                        (fhog/triton_bwdbwd.py:217-251) */
#define FHOG_PASS_DQ_DDO 3 /* dQ2 = dS ddK + dS' K ; ddO = P ddV + ddP V      (fhog/triton_bwdbwd.py:257-313) */
#define FHOG_PASS_DK_DV 4  /* dK2 = dS^T ddQ + dS'^T Q ; dV2 = ddP^T dO       (fhog/triton_bwdbwd.py:467-535) */
#define FHOG_PASS_DD_B 5   /* passes 1 and 2 in one sweep: b_i = sum_j P (E + ddS (dP - d)) - dd_i sum_j P dP
                              (same quantities as fhog/triton_bwdbwd.py:185-251, three recomputed products fewer) */

/* passes of the opt-in schedules that take ddO out of the third sweep (16-bit MFMA family; see FHOG_SCHEDULE_*) */
#define FHOG_PASS_B_DDO 6    /* second sweep as S, ddS, P ddV, ddP V: writes ddO and b_i = dO_i . ddO_i - d_i dd_i (an
                                identity of the reference's quantities: sum_j P_ij dP_ij = d_i); reads d, dd */
#define FHOG_PASS_DQ 7       /* third sweep for dQ2 alone (ddO is already there): seven products instead of nine */
#define FHOG_PASS_DD_B_DDO 8 /* passes 1 and 6 in one sweep: dd_i is accumulated next to (P ddV)_i and ((P o ddS) V)_i
                                and taken out at the end of the row, ddO_i = ... - dd_i O_i (sum_j P_ij V_j = O_i);
                                writes d, dd, b, ddO */
#define FHOG_PASS_STAGE1 9     /* passes 1, 2 and 3 in ONE launch whose workgroups run the three sweeps one after the other
                                for their query tile, dd and b staying in registers: the reference's first kernel as it
                                stands there (bwdbwd_kernel_stage1, fhog/triton_bwdbwd.py:185-313). 16-bit family, d = 64,
                                streamed side not split; writes d, dd, b, dQ2, ddO */

/* kernel families (fhog_bwdbwd_args.impl) */
#define FHOG_IMPL_AUTO 0   /* 16-bit MFMA kernels for bf16/fp16 tensors when the shape allows, else the fp32-MFMA kernels */
#define FHOG_IMPL_FP32 1   /* force the fp32-MFMA kernels (any dtype; every intermediate in fp32) */
#define FHOG_IMPL_BF16 2   /* force the 16-bit MFMA kernels (bf16 or fp16 tensors, products in the tensor type);
                              error if the shape/dtype does not fit */

/* masks (fhog_bwdbwd_args.causal). With a window W > 0 key j is visible to query i iff 0 <= i' - j < W, where i' = i
   (top-left) or i' = i + n_k - n_q (bottom-right: fhog/jax_refs/jax_impl.py:110-115); W = 0 means no window.
   Both kernel families implement all of them and skip the tiles outside the band. */
#define FHOG_MASK_NONE 0
#define FHOG_MASK_TOP_LEFT 1     /* j <= i; needs n_q == n_k (fhog/triton_flash.py:86-92) */
#define FHOG_MASK_BOTTOM_RIGHT 2 /* j <= i + n_k - n_q; needs n_k >= n_q, so that every query sees a key */

/* pass schedules of fhog_bwdbwd (fhog_bwdbwd_args.schedule) */
#define FHOG_SCHEDULE_FOUR_PASS 0   /* the reference's schedule: d, then dd, b, dQ2+ddO, dK2+dV2 as four sweeps
                                       (fhog/triton_bwdbwd.py:185-313, 467-535); 25 recomputed products */
#define FHOG_SCHEDULE_FUSED_STATS 1 /* opt-in: dd and b from one sweep (FHOG_PASS_DD_B), 22 recomputed products;
                                       b differs from the four-pass value only by fp32 summation order */
#define FHOG_SCHEDULE_DDO_EARLY 2   /* opt-in, still four sweeps in the reference's order: dd; b together with ddO
                                       (FHOG_PASS_B_DDO); dQ2 alone (FHOG_PASS_DQ); dK2+dV2. 23 recomputed products.
                                       b inherits the 16-bit rounding of the P and ddP operands of ddO */
#define FHOG_SCHEDULE_THREE_SWEEP 3 /* opt-in, three sweeps: dd, b and ddO (FHOG_PASS_DD_B_DDO); dQ2 (FHOG_PASS_DQ);
                                       dK2+dV2. 20 recomputed products. ddP V is formed as (P o ddS) V - dd O with the
                                       caller's 16-bit O: accurate as long as dd_i does not dominate ddS_ij - dd_i.
                                       Schedules 2 and 3 exist in the 16-bit MFMA family; the fp32-MFMA family runs the
                                       four-pass schedule for them. Passes 6, 7 and 8 have no split form: a launch too
                                       small to fill the GPU whose workspace allows a split (ws_bytes) runs the four
                                       passes (schedule 2) or the fused statistics sweep and passes 3, 4 (schedule 3) */

/* Launch choices (the counterpart of the reference's autotune list, fhog/triton_bwdbwd.py:12-36) are fixed functions of
 * the launch size. For experiments they can be overridden through the environment variable FHOG_TUNE, a comma-separated
 * list of key=value read once, on the host, at the first launch of the process (never in a timed path):
 *   b8=0|1            b and dd+b sweeps at d = 128: 128-row workgroups of 4 waves | 256-row workgroups of 8 waves
 *   order=slice|tile  workgroup order within an XCD: one (batch*head) slice after the other | the slices of an XCD advance
 *                     through their tiles together (also read by the first-order dQ and dK, dV kernels)
 *   split=0|1         small launches may split their streamed side over several workgroups (needs the workspace of
 *                     fhog_bwdbwd_workspace_hint)
 *   dd64=0|1          dd sweep at d = 128 with 32 | 64 queries per wave
 *   stage64=0|1       single-role sweeps at d = 64: one | two 32-row tiles staged and consumed per barrier
 *   stage1=0|1        d = 64, four-pass schedule: sweeps 1-3 as three launches | as one launch (FHOG_PASS_STAGE1)
 * Results do not depend on any of them beyond fp32 summation order (split) - the others are bit-identical. Unknown keys
 * and values are reported on stderr and ignored. */
typedef struct fhog_bwdbwd_args {
  /* inputs (device pointers); q, o, dO, ddq: (batch, n_q, d); k, v, ddk, ddv: (batch, n_k, d) */
  const void* q;
  const void* k;
  const void* v;
  const void* o;
  const void* dO;
  const void* ddq;
  const void* ddk;
  const void* ddv;
  const float* lse; /* (batch, n_q) fp32, contiguous: L_i = logsumexp_j(scale * q_i . k_j) over unmasked j */
  /* outputs (device pointers), same dtype and strides as the matching input group */
  void* dq2; /* like q */
  void* dk2; /* like k */
  void* dv2; /* like k */
  void* ddo; /* like q */
  /* workspace: at least 3 * batch * n_q floats, laid out d | dd | b, each (batch, n_q) contiguous; whatever follows
     (see ws_bytes) holds partial results of launches whose streamed side is split */
  float* ws;
  int64_t batch, n_q, n_k, d;
  /* element strides. The q group (q, o, dO, ddq, dq2, ddo) shares stride_qb/stride_qn,
     the k group (k, v, ddk, ddv, dk2, dv2) shares stride_kb/stride_kn; last-dim stride is 1. */
  int64_t stride_qb, stride_qn, stride_kb, stride_kn;
  float scale;
  int32_t dtype;  /* FHOG_DTYPE_* */
  int32_t causal; /* FHOG_MASK_* */
  int32_t impl;   /* FHOG_IMPL_* */
  int32_t schedule; /* FHOG_SCHEDULE_* */
  int64_t window; /* sliding window length in keys, 0 = none; needs a causal mask */
  int64_t ws_bytes; /* size of ws in bytes; 0 = the minimum, fhog_bwdbwd_workspace_bytes(batch, n_q). With
                       fhog_bwdbwd_workspace_hint(args) bytes, launches too small to fill the GPU (few batch*head
                       slices, short sequences; 16-bit kernels) split the streamed side over several workgroups,
                       which write fp32 partial results behind d | dd | b; a second kernel adds them in a fixed
                       order (no atomics). Anything in between gives as much of that as fits. */
} fhog_bwdbwd_args;

/* Version of this header the library was built from. */
int fhog_abi_version(void);

/* sizeof(fhog_bwdbwd_args) as the library sees it, so that a foreign-language binding can check its mirror. */
size_t fhog_bwdbwd_args_size(void);

/* Bytes of workspace fhog_bwdbwd needs: 3 * batch * n_q * sizeof(float).
   Replaces the torch allocations of D, dD, B at fhog/triton_bwdbwd.py:580-584. */
size_t fhog_bwdbwd_workspace_bytes(int64_t batch, int64_t n_q);

/* Workspace size that lets every pass of these arguments use the split it would like (>= the minimum, and equal to
   it when no pass would split); 0 if the arguments are not valid. Host-only. No counterpart in the reference, whose
   kernels are always tiled over (batch*head, N / BLOCK) alone (fhog/triton_bwdbwd.py:586-646). */
size_t fhog_bwdbwd_workspace_hint(const fhog_bwdbwd_args* args);

/* Host-only argument check (no HIP call is made; works without a GPU).
   Returns FHOG_OK or the FHOG_E_* code fhog_bwdbwd would return for these arguments. */
int fhog_validate(const fhog_bwdbwd_args* args);

/* Which kernel family fhog_bwdbwd would use for these arguments: FHOG_IMPL_FP32 or
   FHOG_IMPL_BF16, or a negative FHOG_E_* code. Host-only. */
int fhog_select_impl(const fhog_bwdbwd_args* args);

/* All passes in order (d, dd, b, dQ2+ddO, dK2+dV2) on `hip_stream` (a hipStream_t); with
   schedule = FHOG_SCHEDULE_FUSED_STATS, dd and b come from one sweep (FHOG_PASS_DD_B) instead.
   Drop-in for the two launches + reduction of flash_bwdbwd (fhog/triton_bwdbwd.py:580-646). */
int fhog_bwdbwd(const fhog_bwdbwd_args* args, void* hip_stream);

/* fhog_bwdbwd for callers that cannot allocate device memory (code under HIP-graph capture, tight serving loops,
   harnesses that forbid hipMalloc): the same passes, with the workspace (d | dd | b and the partial results of split
   launches) in a device array of FHOG_STATIC_WS_BYTES that is part of the loaded library, one copy per GPU, held until
   the process ends. args->ws and args->ws_bytes are not read; inputs and outputs stay the caller's. It has no
   counterpart in the reference, which allocates D, dD and B with torch on every call (fhog/triton_bwdbwd.py:580-584).
   Limits: batch * n_q <= FHOG_STATIC_WS_BYTES / 12 rows (FHOG_E_SHAPE beyond); launches split only as far as the array
   has room. Every call on a GPU uses that GPU's one array: calls that overlap on the same GPU (two streams, two
   threads) race on it; calls ordered on one stream do not. Nothing in the array has to start at zero: every word a
   pass reads was written earlier in the same call. The first call on a device looks the array's address up
   (hipGetSymbolAddress) and raises the dynamic-LDS limit of the kernels it launches (hipFuncSetAttribute): make one call
   per device and tensor configuration OUTSIDE a stream capture before capturing the entry point into a HIP graph.
   No call allocates, frees or synchronises. */
#ifndef FHOG_STATIC_WS_BYTES   /* a build of the library may size the array differently (hipcc -DFHOG_STATIC_WS_BYTES=...) */
#define FHOG_STATIC_WS_BYTES (16 << 20)
#endif
int fhog_bwdbwd_static_ws(const fhog_bwdbwd_args* args, void* hip_stream);

/* Size in bytes of that array in the loaded library (FHOG_STATIC_WS_BYTES of its build). Host-only. */
size_t fhog_static_ws_bytes(void);

/* One pass only (FHOG_PASS_*), for per-pass tests and profiling. Passes read the
   workspace rows written by earlier passes (stage 2 of the reference reads dD, B, D the
   same way: fhog/triton_bwdbwd.py:474-482). */
int fhog_bwdbwd_pass(const fhog_bwdbwd_args* args, int pass, void* hip_stream);

/* ---- first-order attention: the callers on either side of the double-backward ---------------------------
 * bf16, fp16 or fp32 tensors, d in {32, 64, 128}, any n_q and n_k (fhog_attn_validate tells); the layout rules
 * above apply. bf16 / fp16 tensors with d in {64, 128} run on 16-bit MFMA kernels (they need scale > 0), fp32
 * tensors and d = 32 on fp32-MFMA kernels. O and dO/dQ share the q strides, dK/dV the k strides. */
typedef struct fhog_attn_args {
  const void* q;   /* (batch, n_q, d) */
  const void* k;   /* (batch, n_k, d) */
  const void* v;   /* (batch, n_k, d) */
  void* o;         /* (batch, n_q, d): written by fhog_attn_fwd, read by fhog_attn_bwd */
  float* lse;      /* (batch, n_q) fp32 contiguous: written by fhog_attn_fwd, read by fhog_attn_bwd */
  const void* dO;  /* backward only */
  void* dq;        /* backward only, like q */
  void* dk;        /* backward only, like k */
  void* dv;        /* backward only, like k */
  float* ws;       /* backward only: batch * n_q floats */
  int64_t batch, n_q, n_k, d;
  int64_t stride_qb, stride_qn, stride_kb, stride_kn;
  float scale;
  int32_t dtype;   /* FHOG_DTYPE_* */
  int32_t causal;  /* FHOG_MASK_*, as in fhog_bwdbwd_args */
  int32_t window;  /* sliding window length in keys, 0 = none; needs a causal mask */
} fhog_attn_args;

size_t fhog_attn_args_size(void);

/* Host-only: FHOG_OK if fhog_attn_fwd / fhog_attn_bwd cover these arguments (backward != 0 also checks the
   backward-only pointers), else the FHOG_E_* code they would return. */
int fhog_attn_validate(const fhog_attn_args* args, int backward);

/* O = softmax(scale q k^T [causal]) v and L = logsumexp of the scaled scores over visible keys, one sweep,
   online soft-max. Replaces flash_kernel (fhog/triton_flash.py:12-133) and, through L, produce_L
   (fhog/triton_flash.py:252-258). */
int fhog_attn_fwd(const fhog_attn_args* args, void* hip_stream);

/* dQ, dK, dV of the forward above from (q, k, v, o, dO, lse): the arithmetic of flash_backward_torch
   (fhog/triton_flash.py:201-220) as three launches (row sums of o*dO, a Q-tiled sweep for dQ, a K-tiled
   sweep for dK and dV), without the (batch, n_q, n_k) tensors. */
int fhog_attn_bwd(const fhog_attn_args* args, void* hip_stream);

/* Measurement aid (no counterpart in the reference): enqueue a loop of bf16 32x32x16 MFMAs on `blocks` workgroups of 8
   waves (one per CU fills the chip), `trips` x 32 MFMAs per wave. data_mode: 0 operands all zero; 1 random operands in
   registers (nothing but MFMAs); 2 random, every A operand read from LDS (one 128-bit read per MFMA, prefetched: the
   matrix pipe never waits); 3 as 2 with one read per two MFMAs; 4 as 1 plus three independent v_fma_f32 per MFMA; 5 one LDS
   read and three VALU instructions per MFMA, the mix of the recomputation sweeps; data_mode + 8 (8..13): the same loops on
   workgroups of 4 waves, one wave per SIMD, where nothing but a wave's own MFMAs can hide its other instructions. `out`:
   device buffer of blocks * 512 floats. Returns the MFMA FLOPs issued through *flops. Timing it gives the MFMA rate the device sustains at the clock it
   holds for that data and instruction mix, the practical ceiling next to the published peak. */
int fhog_probe_mfma_rate(float* out, int blocks, int trips, int data_mode, double* flops, void* hip_stream);

/* Message for the last failing call on this thread ("" if none). */
const char* fhog_last_error(void);

#ifdef __cplusplus
}
#endif
#endif /* FHOG_HIP_H */
