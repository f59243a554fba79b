// C ABI of libfhog_hip.so: argument validation, kernel-family selection, pass sequencing.
// Replaces the host side of flash_bwdbwd (fhog/triton_bwdbwd.py:557-648).
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <atomic>

#include "fhog_common.h"

// Workspace of fhog_bwdbwd_static_ws: device memory that belongs to the loaded library, so that the entry point never
// allocates. Every GPU the library runs on holds its own copy at its own address until the process ends; the name below
// is only a host-side handle, the address on the current device comes from hipGetSymbolAddress (scratch_on_device).
static __device__ __align__(256) unsigned char scratch[FHOG_STATIC_WS_BYTES];

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

// the staging loads address a 32-row tile with 32-bit byte offsets per lane: 32 rows * stride * 2 bytes must fit
constexpr int64_t kMaxRowStride = (int64_t)1 << 24;

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// FHOG_OK or the error for a mask that does not apply to the shape
int check_mask(int32_t causal, int64_t window, int64_t n_q, int64_t n_k) {
  if (causal < FHOG_MASK_NONE || causal > FHOG_MASK_BOTTOM_RIGHT) return fail(FHOG_E_CAUSAL, "causal must be 0, 1 or 2");
  if (causal == FHOG_MASK_TOP_LEFT && n_q != n_k)
    return fail(FHOG_E_CAUSAL, "causal (top-left) needs n_q == n_k (got %lld, %lld)", (long long)n_q, (long long)n_k);
  if (causal == FHOG_MASK_BOTTOM_RIGHT && n_k < n_q)
    return fail(FHOG_E_CAUSAL, "causal (bottom-right) needs n_k >= n_q (got %lld, %lld)", (long long)n_k, (long long)n_q);
  if (window < 0) return fail(FHOG_E_CAUSAL, "window must be >= 0");
  if (window > 0 && causal == FHOG_MASK_NONE) return fail(FHOG_E_CAUSAL, "a window needs a causal mask");
  return FHOG_OK;
}
// kernel-side mask parameters: key j is visible to query i iff 0 <= i + off - j < win
void mask_params(int32_t causal, int64_t window, int64_t n_q, int64_t n_k, int32_t* off, int32_t* win) {
  *off = causal == FHOG_MASK_BOTTOM_RIGHT ? (int32_t)(n_k - n_q) : 0;
  const int64_t reach = n_q + n_k;  // a window this long hides nothing
  *win = (int32_t)((window == 0 || window > reach) ? reach : window);
}

int validate(const fhog_bwdbwd_args* a) {
  if (!a) return fail(FHOG_E_NULL, "args is NULL");
  const void* ptrs[] = {a->q, a->k, a->v, a->o, a->dO, a->ddq, a->ddk, a->ddv, a->lse, a->dq2, a->dk2, a->dv2, a->ddo, a->ws};
  const char* names[] = {"q", "k", "v", "o", "dO", "ddq", "ddk", "ddv", "lse", "dq2", "dk2", "dv2", "ddo", "ws"};
  for (int i = 0; i < 14; i++)
    if (!ptrs[i]) return fail(FHOG_E_NULL, "pointer '%s' is NULL", names[i]);
  if (a->dtype != FHOG_DTYPE_BF16 && a->dtype != FHOG_DTYPE_FP32 && a->dtype != FHOG_DTYPE_FP16)
    return fail(FHOG_E_DTYPE, "unknown dtype %d", a->dtype);
  if (a->impl != FHOG_IMPL_AUTO && a->impl != FHOG_IMPL_FP32 && a->impl != FHOG_IMPL_BF16)
    return fail(FHOG_E_IMPL, "unknown impl %d", a->impl);
  if (a->schedule < FHOG_SCHEDULE_FOUR_PASS || a->schedule > FHOG_SCHEDULE_THREE_SWEEP)
    return fail(FHOG_E_SCHEDULE, "unknown schedule %d", a->schedule);
  if (a->batch < 1 || a->n_q < 1 || a->n_k < 1)
    return fail(FHOG_E_SHAPE, "batch, n_q, n_k must be >= 1 (got %lld, %lld, %lld)", (long long)a->batch, (long long)a->n_q,
                (long long)a->n_k);
  if (a->batch > 65535) return fail(FHOG_E_SHAPE, "batch %lld above 65535 (batch * head slices) is not supported", (long long)a->batch);
  if (a->n_q > (1 << 24) || a->n_k > (1 << 24)) return fail(FHOG_E_SHAPE, "n_q/n_k above 2^24 not supported");
  if (a->batch * a->n_q >= (int64_t)1 << 31) return fail(FHOG_E_SHAPE, "batch*n_q must be below 2^31");
  if (a->d != 32 && a->d != 64 && a->d != 128) return fail(FHOG_E_SHAPE, "head dim %lld not in {32, 64, 128}", (long long)a->d);
  if (const int rc = check_mask(a->causal, a->window, a->n_q, a->n_k)) return rc;
  if (!isfinite(a->scale)) return fail(FHOG_E_SCALE, "scale is not finite");
  if (a->ws_bytes != 0 && a->ws_bytes < (int64_t)(3 * a->batch * a->n_q * sizeof(float)))
    return fail(FHOG_E_SHAPE, "ws_bytes %lld is below the minimum of 3 * batch * n_q floats", (long long)a->ws_bytes);
  const int vec = a->dtype == FHOG_DTYPE_FP32 ? 4 : 8;  // elements per 16 bytes
  if (a->stride_qn < a->d || a->stride_kn < a->d) return fail(FHOG_E_STRIDE, "row stride smaller than d");
  if (a->stride_qn > kMaxRowStride || a->stride_kn > kMaxRowStride) return fail(FHOG_E_STRIDE, "row stride above 2^24 elements");
  if (a->stride_qn % vec || a->stride_kn % vec || a->stride_qb % vec || a->stride_kb % vec)
    return fail(FHOG_E_STRIDE, "strides must be multiples of %d elements (16 bytes)", vec);
  if (a->batch > 1 && (a->stride_qb < a->n_q * a->stride_qn || a->stride_kb < a->n_k * a->stride_kn))
    return fail(FHOG_E_STRIDE, "batch stride smaller than one (n, d) slice");
  for (int i = 0; i < 14; i++)
    if (!aligned16(ptrs[i])) return fail(FHOG_E_ALIGN, "pointer '%s' is not 16-byte aligned", names[i]);
  if (a->impl == FHOG_IMPL_BF16) {
    if (a->dtype == FHOG_DTYPE_FP32) return fail(FHOG_E_DTYPE, "impl=bf16 needs bf16 or fp16 tensors");
    if (!fhog::bf16_shape_supported(a->n_q, a->n_k, a->d, a->causal))
      return fail(FHOG_E_SHAPE, "impl=bf16 needs d in {64,128}");
  }
  return FHOG_OK;
}

int select_impl(const fhog_bwdbwd_args* a) {
  if (a->impl == FHOG_IMPL_FP32) return FHOG_IMPL_FP32;
  if (a->impl == FHOG_IMPL_BF16) return FHOG_IMPL_BF16;
  if (a->dtype != FHOG_DTYPE_FP32 && fhog::bf16_shape_supported(a->n_q, a->n_k, a->d, a->causal)) return FHOG_IMPL_BF16;
  return FHOG_IMPL_FP32;
}

fhog::Params to_params(const fhog_bwdbwd_args* a) {
  fhog::Params p;
  p.q = a->q;
  p.k = a->k;
  p.v = a->v;
  p.o = a->o;
  p.dO = a->dO;
  p.ddq = a->ddq;
  p.ddk = a->ddk;
  p.ddv = a->ddv;
  p.lse = a->lse;
  p.dq2 = a->dq2;
  p.dk2 = a->dk2;
  p.dv2 = a->dv2;
  p.ddo = a->ddo;
  const int64_t rows = a->batch * a->n_q;
  p.ws_d = a->ws;
  p.ws_dd = a->ws + rows;
  p.ws_b = a->ws + 2 * rows;
  p.stride_qb = a->stride_qb;
  p.stride_qn = a->stride_qn;
  p.stride_kb = a->stride_kb;
  p.stride_kn = a->stride_kn;
  p.batch = (int32_t)a->batch;
  p.n_q = (int32_t)a->n_q;
  p.n_k = (int32_t)a->n_k;
  p.d = (int32_t)a->d;
  p.scale = a->scale;
  p.causal = a->causal != FHOG_MASK_NONE;
  p.f16 = a->dtype == FHOG_DTYPE_FP16;
  mask_params(a->causal, a->window, a->n_q, a->n_k, &p.mask_off, &p.window);
  p.n_split = 1;
  p.part = nullptr;
  const int order = fhog::tuning().order;
  p.tile_major = order < 0 ? p.causal : order;
  return p;
}

// ---- splitting the streamed side of small launches (16-bit kernels) -------------------------------------------
// Bytes of d | dd | b, rounded up so that what follows stays 16-byte aligned.
size_t stats_bytes(const fhog_bwdbwd_args* a) { return ((size_t)3 * a->batch * a->n_q * sizeof(float) + 15) & ~(size_t)15; }
// fp32 partial results one split of a pass writes
size_t split_bytes(const fhog_bwdbwd_args* a, int pass) {
  if (pass == FHOG_PASS_DQ_DDO) return (size_t)2 * a->batch * a->n_q * a->d * sizeof(float);
  if (pass == FHOG_PASS_DK_DV) return (size_t)2 * a->batch * a->n_k * a->d * sizeof(float);
  return (size_t)3 * a->batch * a->n_q * sizeof(float);
}
// Splits a pass would like: enough workgroups for two per CU, every split keeping at least 8 streamed tiles.
int wanted_split(const fhog_bwdbwd_args* a, int impl, int pass) {
  if (impl != FHOG_IMPL_BF16 || pass == FHOG_PASS_D || pass > FHOG_PASS_DD_B) return 1;   // passes 6-8 never split
  const bool kside = pass == FHOG_PASS_DK_DV;
  const int64_t groups = ((kside ? a->n_k : a->n_q) + 127) / 128 * a->batch;
  const int64_t streamed = ((kside ? a->n_q : a->n_k) + 31) / 32;
  int s = 1;
  if (!fhog::tuning().split) return s;
  while (groups * s < 512 && s < 16 && streamed / (2 * s) >= 8) s *= 2;
  return s;
}
// ... and what of that the workspace has room for
int granted_split(const fhog_bwdbwd_args* a, int impl, int pass) {
  int s = wanted_split(a, impl, pass);
  const size_t have = a->ws_bytes > 0 ? (size_t)a->ws_bytes : 0;
  while (s > 1 && stats_bytes(a) + (size_t)s * split_bytes(a, pass) > have) s /= 2;
  return s;
}

int run_pass(const fhog_bwdbwd_args* a, const fhog::Params& base, int impl, int pass, hipStream_t s) {
  fhog::Params p = base;
  p.n_split = granted_split(a, impl, pass);
  // Workgroup order within an XCD. With a mask, tile-major (the slices of an XCD advance together, heaviest tiles of all
  // of them first) balances the end of a launch; from 16384 stationary rows on a slice alone has tiles enough for that
  // and one slice after the other keeps the fetched bytes near the algorithmic ones (measured on N = 16384: 2.2-2.6x
  // instead of 4-10x, sweeps b, 3 and 4 0.1-3 % faster, the dd sweep with its three workgroups per CU 4 % slower).
  if (fhog::tuning().order < 0 && p.causal && pass != FHOG_PASS_DD && (pass == FHOG_PASS_DK_DV ? a->n_k : a->n_q) >= 16384)
    p.tile_major = 0;
  p.part = reinterpret_cast<float*>(reinterpret_cast<char*>(a->ws) + stats_bytes(a));
  hipError_t e;
  if (pass > FHOG_PASS_DD_B && impl != FHOG_IMPL_BF16)
    return fail(FHOG_E_PASS, "pass %d exists in the 16-bit MFMA family only (bf16 / fp16 tensors, d in {64, 128})", pass);
  if (pass == FHOG_PASS_STAGE1 && a->d != 64)
    return fail(FHOG_E_PASS, "pass %d (three sweeps in one launch) exists for d = 64 only", pass);
  if (pass == FHOG_PASS_D)
    e = fhog::launch_rowdot(p, a->dtype, s);
  else if (impl == FHOG_IMPL_BF16)
    e = fhog::launch_bf16_pass(p, pass, s);
  else if (pass == FHOG_PASS_DD_B) {
    e = fhog::launch_fp32_pass(p, a->dtype, FHOG_PASS_DD, s);
    if (e == hipSuccess) e = fhog::launch_fp32_pass(p, a->dtype, FHOG_PASS_B, s);
  } else
    e = fhog::launch_fp32_pass(p, a->dtype, pass, s);
  if (e != hipSuccess) return fail(FHOG_E_LAUNCH, "pass %d: HIP error %d (%s)", pass, (int)e, hipGetErrorString(e));
  return FHOG_OK;
}

// bf16 / fp16 tensors with d in {64, 128} run on the 16-bit MFMA kernels, everything else (fp32 tensors, d = 32) on the
// fp32-MFMA ones
bool attn_on_16bit_kernels(const fhog_attn_args* a) { return a->dtype != FHOG_DTYPE_FP32 && (a->d == 64 || a->d == 128); }

int validate_attn(const fhog_attn_args* a, int backward) {
  if (!a) return fail(FHOG_E_NULL, "args is NULL");
  const void* ptrs[] = {a->q, a->k, a->v, a->o, a->lse, a->dO, a->dq, a->dk, a->dv, a->ws};
  const char* names[] = {"q", "k", "v", "o", "lse", "dO", "dq", "dk", "dv", "ws"};
  const int n_ptr = backward ? 10 : 5;
  for (int i = 0; i < n_ptr; i++) {
    if (!ptrs[i]) return fail(FHOG_E_NULL, "pointer '%s' is NULL", names[i]);
    if (!aligned16(ptrs[i])) return fail(FHOG_E_ALIGN, "pointer '%s' is not 16-byte aligned", names[i]);
  }
  if (a->dtype != FHOG_DTYPE_BF16 && a->dtype != FHOG_DTYPE_FP16 && a->dtype != FHOG_DTYPE_FP32)
    return fail(FHOG_E_DTYPE, "unknown dtype %d", a->dtype);
  if (a->batch < 1 || a->batch > 65535) return fail(FHOG_E_SHAPE, "batch %lld outside 1..65535", (long long)a->batch);
  if (a->n_q < 1 || a->n_k < 1 || a->n_q > (1 << 24) || a->n_k > (1 << 24) || a->batch * a->n_q >= (int64_t)1 << 31)
    return fail(FHOG_E_SHAPE, "n_q/n_k out of range");
  if (const int rc = check_mask(a->causal, a->window, a->n_q, a->n_k)) return rc;
  if (a->d != 32 && a->d != 64 && a->d != 128) return fail(FHOG_E_SHAPE, "head dim %lld not in {32, 64, 128}", (long long)a->d);
  if (!isfinite(a->scale)) return fail(FHOG_E_SCALE, "scale is not finite");
  // the 16-bit forward takes the running maximum of the raw scores and scales it afterwards, which needs scale > 0
  if (attn_on_16bit_kernels(a) && a->scale <= 0.f)
    return fail(FHOG_E_SCALE, "the 16-bit kernels need a positive scale (got %g)", (double)a->scale);
  const int vec = a->dtype == FHOG_DTYPE_FP32 ? 4 : 8;  // elements per 16 bytes
  if (a->stride_qn < a->d || a->stride_kn < a->d) return fail(FHOG_E_STRIDE, "row stride smaller than d");
  if (a->stride_qn > kMaxRowStride || a->stride_kn > kMaxRowStride) return fail(FHOG_E_STRIDE, "row stride above 2^24 elements");
  if (a->stride_qn % vec || a->stride_kn % vec || a->stride_qb % vec || a->stride_kb % vec)
    return fail(FHOG_E_STRIDE, "strides must be multiples of %d elements (16 bytes)", vec);
  if (a->batch > 1 && (a->stride_qb < a->n_q * a->stride_qn || a->stride_kb < a->n_k * a->stride_kn))
    return fail(FHOG_E_STRIDE, "batch stride smaller than one (n, d) slice");
  return FHOG_OK;
}

fhog::AttnParams to_attn_params(const fhog_attn_args* a) {
  fhog::AttnParams p;
  p.q = a->q;
  p.k = a->k;
  p.v = a->v;
  p.o = a->o;
  p.lse = a->lse;
  p.dO = a->dO;
  p.dq = a->dq;
  p.dk = a->dk;
  p.dv = a->dv;
  p.ws_d = a->ws;
  p.stride_qb = a->stride_qb;
  p.stride_qn = a->stride_qn;
  p.stride_kb = a->stride_kb;
  p.stride_kn = a->stride_kn;
  p.batch = (int32_t)a->batch;
  p.n_q = (int32_t)a->n_q;
  p.n_k = (int32_t)a->n_k;
  p.d = (int32_t)a->d;
  p.scale = a->scale;
  p.causal = a->causal != FHOG_MASK_NONE;
  p.f16 = a->dtype == FHOG_DTYPE_FP16;
  mask_params(a->causal, a->window, a->n_q, a->n_k, &p.mask_off, &p.window);
  // as in run_pass: tile-major with a mask, until a slice alone has tiles enough to balance the end of a launch
  const int order = fhog::tuning().order;
  p.tile_major_q = order < 0 ? (p.causal && a->n_q < 16384) : order;
  p.tile_major_k = order < 0 ? (p.causal && a->n_k < 16384) : order;
  return p;
}

// Address of `scratch` on the current device, looked up once per device (the first call there) and kept.
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

int scratch_on_device(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(FHOG_E_LAUNCH, "hipGetDevice: HIP error %d (%s)", (int)e, hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail(FHOG_E_LAUNCH, "device ordinal %d outside 0..%d", dev, kMaxDevices - 1);
  void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!ptr) {
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr)
      return fail(FHOG_E_LAUNCH, "hipGetSymbolAddress(scratch) on device %d: HIP error %d (%s)", dev, (int)e, hipGetErrorString(e));
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);   // concurrent first calls store the same address
  }
  *out = ptr;
  return FHOG_OK;
}

}  // namespace

namespace fhog {
const Tuning& tuning() {
  static const Tuning t = [] {
    Tuning r;
    const char* env = getenv("FHOG_TUNE");
    if (!env) return r;
    char buf[256];
    if (strlen(env) >= sizeof(buf)) fprintf(stderr, "libfhog_hip: FHOG_TUNE is longer than %zu characters; the rest is ignored\n", sizeof(buf) - 1);
    strncpy(buf, env, sizeof(buf) - 1);
    buf[sizeof(buf) - 1] = 0;
    // 0 / 1 switches; anything else is reported and ignored
    const auto flag = [](const char* key, const char* val, int* out) {
      if (!strcmp(val, "0") || !strcmp(val, "1")) *out = val[0] - '0';
      else fprintf(stderr, "libfhog_hip: FHOG_TUNE: value '%s' of '%s' is not 0 or 1; ignored\n", val, key);
    };
    char* save = nullptr;
    for (char* tok = strtok_r(buf, ",", &save); tok; tok = strtok_r(nullptr, ",", &save)) {
      char* eq = strchr(tok, '=');
      if (!eq) {
        fprintf(stderr, "libfhog_hip: FHOG_TUNE: '%s' is not key=value; ignored\n", tok);
        continue;
      }
      *eq = 0;
      const char* val = eq + 1;
      if (!strcmp(tok, "b8")) flag(tok, val, &r.b8);
      else if (!strcmp(tok, "split")) flag(tok, val, &r.split);
      else if (!strcmp(tok, "dd64")) flag(tok, val, &r.dd64);
      else if (!strcmp(tok, "stage64")) flag(tok, val, &r.stage64);
      else if (!strcmp(tok, "stage1")) flag(tok, val, &r.stage1);
      else if (!strcmp(tok, "order")) {
        if (!strcmp(val, "tile")) r.order = 1;
        else if (!strcmp(val, "slice")) r.order = 0;
        else fprintf(stderr, "libfhog_hip: FHOG_TUNE: order is 'slice' or 'tile', not '%s'; ignored\n", val);
      } else {
        fprintf(stderr, "libfhog_hip: FHOG_TUNE: unknown key '%s'; ignored\n", tok);
      }
    }
    return r;
  }();
  return t;
}
}  // namespace fhog

extern "C" {

size_t fhog_attn_args_size(void) { return sizeof(fhog_attn_args); }

int fhog_attn_validate(const fhog_attn_args* args, int backward) { return validate_attn(args, backward); }

int fhog_attn_fwd(const fhog_attn_args* args, void* hip_stream) {
  const int rc = validate_attn(args, 0);
  if (rc != FHOG_OK) return rc;
  const hipError_t e = attn_on_16bit_kernels(args) ? fhog::launch_attn_bf16(to_attn_params(args), 0, (hipStream_t)hip_stream)
                                                   : fhog::launch_attn_fp32(to_attn_params(args), args->dtype, 0, (hipStream_t)hip_stream);
  if (e != hipSuccess) return fail(FHOG_E_LAUNCH, "attention forward: HIP error %d (%s)", (int)e, hipGetErrorString(e));
  return FHOG_OK;
}

int fhog_attn_bwd(const fhog_attn_args* args, void* hip_stream) {
  const int rc = validate_attn(args, 1);
  if (rc != FHOG_OK) return rc;
  const fhog::AttnParams p = to_attn_params(args);
  fhog::Params rd = {};  // row sums d_i = sum_c o_ic dO_ic with the kernel of pass 0
  rd.o = args->o;
  rd.dO = args->dO;
  rd.ws_d = args->ws;
  rd.stride_qb = p.stride_qb;
  rd.stride_qn = p.stride_qn;
  rd.batch = p.batch;
  rd.n_q = p.n_q;
  rd.d = p.d;
  hipError_t e = fhog::launch_rowdot(rd, args->dtype, (hipStream_t)hip_stream);
  for (int which = 1; which <= 2 && e == hipSuccess; which++)
    e = attn_on_16bit_kernels(args) ? fhog::launch_attn_bf16(p, which, (hipStream_t)hip_stream)
                                    : fhog::launch_attn_fp32(p, args->dtype, which, (hipStream_t)hip_stream);
  if (e != hipSuccess) return fail(FHOG_E_LAUNCH, "attention backward: HIP error %d (%s)", (int)e, hipGetErrorString(e));
  return FHOG_OK;
}


int fhog_abi_version(void) { return FHOG_ABI_VERSION; }

size_t fhog_bwdbwd_args_size(void) { return sizeof(fhog_bwdbwd_args); }

size_t fhog_bwdbwd_workspace_bytes(int64_t batch, int64_t n_q) {
  if (batch < 0 || n_q < 0) return 0;
  return (size_t)3 * (size_t)batch * (size_t)n_q * sizeof(float);
}

size_t fhog_bwdbwd_workspace_hint(const fhog_bwdbwd_args* args) {
  if (validate(args) != FHOG_OK) return 0;
  const int impl = select_impl(args);
  size_t extra = 0;
  for (int pass = FHOG_PASS_DD; pass <= FHOG_PASS_DD_B; pass++) {
    const int s = wanted_split(args, impl, pass);
    if (s > 1 && (size_t)s * split_bytes(args, pass) > extra) extra = (size_t)s * split_bytes(args, pass);
  }
  return extra ? stats_bytes(args) + extra : fhog_bwdbwd_workspace_bytes(args->batch, args->n_q);
}

int fhog_validate(const fhog_bwdbwd_args* args) { return validate(args); }

int fhog_select_impl(const fhog_bwdbwd_args* args) {
  const int rc = validate(args);
  if (rc != FHOG_OK) return rc;
  return select_impl(args);
}

int fhog_bwdbwd_pass(const fhog_bwdbwd_args* args, int pass, void* hip_stream) {
  const int rc = validate(args);
  if (rc != FHOG_OK) return rc;
  if (pass < FHOG_PASS_D || pass > FHOG_PASS_STAGE1) return fail(FHOG_E_PASS, "unknown pass %d", pass);
  const fhog::Params p = to_params(args);
  return run_pass(args, p, select_impl(args), pass, (hipStream_t)hip_stream);
}

int fhog_bwdbwd(const fhog_bwdbwd_args* args, void* hip_stream) {
  const int rc = validate(args);
  if (rc != FHOG_OK) return rc;
  const fhog::Params p = to_params(args);
  const int impl = select_impl(args);
  // Pass sequences. The first statistics sweep of the 16-bit family writes d_i itself: no separate launch for it there.
  // The schedules that take ddO out of the third sweep exist in the 16-bit family; the fp32-MFMA family runs the
  // reference's four passes for them.
  static const int four[] = {FHOG_PASS_D, FHOG_PASS_DD, FHOG_PASS_B, FHOG_PASS_DQ_DDO, FHOG_PASS_DK_DV};
  static const int fused[] = {FHOG_PASS_D, FHOG_PASS_DD_B, FHOG_PASS_DQ_DDO, FHOG_PASS_DK_DV};
  static const int ddo_early[] = {FHOG_PASS_DD, FHOG_PASS_B_DDO, FHOG_PASS_DQ, FHOG_PASS_DK_DV};
  static const int three[] = {FHOG_PASS_DD_B_DDO, FHOG_PASS_DQ, FHOG_PASS_DK_DV};
  const int* order = four;
  int first = impl == FHOG_IMPL_BF16 ? 1 : 0, n_pass = 5;
  // d = 64, launch large enough to fill the GPU: the reference's own arrangement of its four passes, sweeps 1-3 in one launch
  static const int stage1[] = {FHOG_PASS_STAGE1, FHOG_PASS_DK_DV};
  if (args->schedule == FHOG_SCHEDULE_FOUR_PASS && impl == FHOG_IMPL_BF16 && args->d == 64 && fhog::tuning().stage1 != 0 &&
      granted_split(args, impl, FHOG_PASS_DQ_DDO) == 1 && granted_split(args, impl, FHOG_PASS_DD) == 1)
    order = stage1, first = 0, n_pass = 2;
  if (args->schedule == FHOG_SCHEDULE_FUSED_STATS) order = fused, n_pass = 4;
  // Passes 6-8 have no split form: a launch too small to fill the GPU whose workspace lets the reference's passes split
  // their streamed side runs the nearest schedule that can (three sweeps -> fused statistics, ddO early -> four passes).
  const bool small = granted_split(args, impl, FHOG_PASS_DQ_DDO) > 1;
  if (args->schedule == FHOG_SCHEDULE_THREE_SWEEP && small) order = fused, n_pass = 4;
  if (args->schedule == FHOG_SCHEDULE_DDO_EARLY && impl == FHOG_IMPL_BF16 && !small) order = ddo_early, first = 0, n_pass = 4;
  if (args->schedule == FHOG_SCHEDULE_THREE_SWEEP && impl == FHOG_IMPL_BF16 && !small) order = three, first = 0, n_pass = 3;
  for (int i = first; i < n_pass; i++) {
    const int r = run_pass(args, p, impl, order[i], (hipStream_t)hip_stream);
    if (r != FHOG_OK) return r;
  }
  return FHOG_OK;
}

int fhog_bwdbwd_static_ws(const fhog_bwdbwd_args* args, void* hip_stream) {
  if (!args) return fail(FHOG_E_NULL, "args is NULL");
  void* ws = nullptr;
  if (const int rc = scratch_on_device(&ws)) return rc;
  fhog_bwdbwd_args a = *args;   // the caller's ws / ws_bytes are not read
  a.ws = static_cast<float*>(ws);
  a.ws_bytes = 0;
  if (const int rc = validate(&a)) return rc;
  const size_t need = fhog_bwdbwd_workspace_bytes(a.batch, a.n_q);
  if (need > (size_t)FHOG_STATIC_WS_BYTES)
    return fail(FHOG_E_SHAPE,
                "fhog_bwdbwd_static_ws: batch*n_q = %lld rows need %zu bytes of row statistics, the static workspace holds %zu "
                "(at most %zu rows); use fhog_bwdbwd with a caller-owned workspace",
                (long long)(a.batch * a.n_q), need, (size_t)FHOG_STATIC_WS_BYTES, (size_t)FHOG_STATIC_WS_BYTES / 12);
  a.ws_bytes = FHOG_STATIC_WS_BYTES;   // small launches split their streamed side as far as the rest of the array allows
  return fhog_bwdbwd(&a, hip_stream);
}

size_t fhog_static_ws_bytes(void) { return (size_t)FHOG_STATIC_WS_BYTES; }

int fhog_probe_mfma_rate(float* out, int blocks, int trips, int data_mode, double* flops, void* hip_stream) {
  if (!out || !flops) return fail(FHOG_E_NULL, "out or flops is NULL");
  const int mix = data_mode & 7, waves = (data_mode & 8) ? 4 : 8;
  if (blocks < 1 || blocks > 65535 || trips < 1 || data_mode < 0 || data_mode > 13 || mix > 5)
    return fail(FHOG_E_SHAPE, "blocks in 1..65535, trips >= 1, data_mode 0..5 or 8..13");
  const hipError_t e = fhog::launch_mfma_rate(out, blocks, trips, mix, waves, (hipStream_t)hip_stream);
  if (e != hipSuccess) return fail(FHOG_E_LAUNCH, "MFMA rate probe: HIP error %d (%s)", (int)e, hipGetErrorString(e));
  *flops = (double)blocks * waves * trips * 32.0 * 32768.0;
  return FHOG_OK;
}

const char* fhog_last_error(void) { return g_err; }

}  // extern "C"
