"""Host wrapper of the attention double-backward: same entry point as the reference's
``flash_bwdbwd`` (``fhog/triton_bwdbwd.py:557-648``), backed by ``libfhog_hip.so``.
"""
from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import torch

from . import _lib

_DTYPES = {torch.bfloat16: _lib.DTYPE_BF16, torch.float32: _lib.DTYPE_FP32, torch.float16: _lib.DTYPE_FP16}
_IMPLS = {None: _lib.IMPL_AUTO, "auto": _lib.IMPL_AUTO, "fp32": _lib.IMPL_FP32, "bf16": _lib.IMPL_BF16}
_SCHEDULES = {None: _lib.SCHEDULE_FOUR_PASS, "four_pass": _lib.SCHEDULE_FOUR_PASS, "fused_stats": _lib.SCHEDULE_FUSED_STATS,
              "ddo_early": _lib.SCHEDULE_DDO_EARLY, "three_sweep": _lib.SCHEDULE_THREE_SWEEP}


def schedule_code(schedule, fused_stats: bool = False) -> int:
    """FHOG_SCHEDULE_* of the C ABI for the Python-level arguments (``fused_stats=True`` is ``schedule="fused_stats"``)."""
    if schedule not in _SCHEDULES:
        raise ValueError(f"schedule must be one of {sorted(k for k in _SCHEDULES if k)} or None, got {schedule!r}")
    if fused_stats:
        if schedule not in (None, "fused_stats"):
            raise ValueError(f"fused_stats=True contradicts schedule={schedule!r}")
        return _lib.SCHEDULE_FUSED_STATS
    return _SCHEDULES[schedule]


def _flatten(t: torch.Tensor, name: str) -> torch.Tensor:
    """(batch, N, d) stays; (B, H, N, d) becomes (B*H, N, d) (a view when possible)."""
    if t.dim() == 3:
        return t
    if t.dim() == 4:
        return t.reshape(t.shape[0] * t.shape[1], t.shape[2], t.shape[3])
    raise ValueError(f"{name}: expected a 3-D (batch, N, d) or 4-D (B, H, N, d) tensor, got shape {tuple(t.shape)}")


def _same_layout(ts) -> bool:
    s0 = ts[0].stride()
    return all(t.stride() == s0 for t in ts)


def _prepare_group(ts, names):
    """Tensors of one group must share (batch stride, row stride) and have a contiguous last dim."""
    vec = 16 // ts[0].element_size()
    ok = (_same_layout(ts) and ts[0].stride(2) == 1 and ts[0].stride(1) >= ts[0].shape[2]
          and ts[0].stride(1) % vec == 0 and ts[0].stride(0) % vec == 0
          and (ts[0].shape[0] == 1 or ts[0].stride(0) >= ts[0].shape[1] * ts[0].stride(1))
          and all(t.data_ptr() % 16 == 0 for t in ts))
    if ok:
        return list(ts)
    return [t.contiguous() for t in ts]


def workspace_floats(batch: int, n_q: int) -> int:
    return _lib.lib().fhog_bwdbwd_workspace_bytes(batch, n_q) // 4


def mask_code(causal, window, n_q: int, n_k: int):
    """(FHOG_MASK_* code, window) of the C ABI for the Python-level mask arguments.

    ``causal``: False | True (top-left, N_Q == N_K) | "bottom_right" (key j visible iff j <= i + N_K - N_Q,
    ``fhog/jax_refs/jax_impl.py:110-115``); ``window``: None or the sliding-window length in keys."""
    if causal is None or causal is False or causal == 0:
        if window is not None:
            raise ValueError("a sliding window needs a causal mask")
        return _lib.MASK_NONE, 0
    if causal is True or causal == 1:
        if n_q != n_k:
            raise ValueError(f"causal needs N_Q == N_K, got {n_q} and {n_k} (causal='bottom_right' aligns the diagonal "
                             "to the last key)")
        code = _lib.MASK_TOP_LEFT
    elif causal == "bottom_right":
        if n_k < n_q:
            raise ValueError(f"causal='bottom_right' needs N_K >= N_Q, got {n_k} and {n_q}")
        code = _lib.MASK_BOTTOM_RIGHT
    else:
        raise ValueError(f"causal must be False, True or 'bottom_right', got {causal!r}")
    if window is None:
        return code, 0
    if int(window) < 1:
        raise ValueError(f"window must be >= 1, got {window}")
    return code, int(window)


def _workspace(args: "_lib.BwdBwdArgs", device, split: bool) -> torch.Tensor:
    """Allocate the workspace of a call and enter it into ``args``: the three row statistics ``d | dd | b`` and, with
    ``split``, room for the partial results of launches that split their streamed side (``fhog_bwdbwd_workspace_hint``)."""
    batch, n_q = args.batch, args.n_q
    nbytes = 3 * batch * n_q * 4
    if split:
        args.ws, args.ws_bytes = args.q, 0      # any valid pointer: the hint is computed on the host
        nbytes = max(nbytes, int(_lib.lib().fhog_bwdbwd_workspace_hint(ctypes.byref(args))))
    ws = torch.empty((nbytes + 3) // 4, dtype=torch.float32, device=device)
    args.ws, args.ws_bytes = ws.data_ptr(), nbytes
    return ws


def _build_args(Q, K, V, O, dO, ddQ, ddK, ddV, L, scale, causal, impl, outs, ws, schedule=0,
                window=None) -> _lib.BwdBwdArgs:
    """``ws``: a workspace tensor of the minimum size, or None when :func:`_workspace` fills it in afterwards."""
    a = _lib.BwdBwdArgs()
    a.q, a.k, a.v, a.o, a.dO = Q.data_ptr(), K.data_ptr(), V.data_ptr(), O.data_ptr(), dO.data_ptr()
    a.ddq, a.ddk, a.ddv = ddQ.data_ptr(), ddK.data_ptr(), ddV.data_ptr()
    a.lse = L.data_ptr()
    a.dq2, a.dk2, a.dv2, a.ddo = (t.data_ptr() for t in outs)
    a.ws = ws.data_ptr() if ws is not None else 0
    a.batch, a.n_q, a.d = Q.shape
    a.n_k = K.shape[1]
    a.stride_qb, a.stride_qn = Q.stride(0), Q.stride(1)
    a.stride_kb, a.stride_kn = K.stride(0), K.stride(1)
    a.scale = float(scale)
    a.dtype = _DTYPES[Q.dtype]
    a.causal, a.window = mask_code(causal, window, Q.shape[1], K.shape[1])
    a.impl = impl
    a.schedule = int(schedule)
    return a


def flash_bwdbwd(Q, K, V, O, dO, ddQ, ddK, ddV, L, scale, *, causal=False, window: Optional[int] = None,
                 impl: Optional[str] = None, fused_stats: bool = False, schedule: Optional[str] = None,
                 return_stats: bool = False, only_pass: Optional[int] = None, split: bool = True):
    """Flash Higher-Order-Gradients: VJP of the attention backward pass.

    Same positional signature and return order as the reference
    (``fhog/triton_bwdbwd.py:558,648``)::

        dQ2, dK2, dV2, ddO = flash_bwdbwd(Q, K, V, O, dO, ddQ, ddK, ddV, L, scale)

    Args:
        Q, O, dO, ddQ: (batch, N_Q, d) or (B, H, N_Q, d); K, V, ddK, ddV: (batch, N_K, d) or (B, H, N_K, d).
            bf16, fp16 or fp32 (all the same dtype), on a ROCm device.
        L: (batch, N_Q) / (B, H, N_Q) log-sum-exp of ``scale * Q K^T`` over visible keys. Used in fp32
            (any other dtype is up-cast; the reference passes it in the input dtype,
            ``fhog/triton_flash.py:255-257``).
        scale: python float.
        causal: keyword only. True: top-left mask (key j visible to query i iff j <= i), needs N_Q == N_K.
            "bottom_right": j <= i + N_K - N_Q, needs N_K >= N_Q. (The reference's Triton path has no causal
            double-backward; its JAX specification has the bottom-right form, ``fhog/jax_refs/jax_impl.py:110-115``.)
        window: sliding-window length in keys on top of a causal mask (same function of the specification):
            only the ``window`` most recent visible keys stay visible. Both kernel families take every mask and
            skip the tiles outside the band.
        impl: None/"auto" | "fp32" | "bf16" - kernel family; "auto" takes the 16-bit MFMA kernels ("bf16": products
            in the tensor type, bf16 or fp16) for 16-bit tensors whose shape they support, the fp32-MFMA kernels
            otherwise.
        fused_stats: opt-in schedule that takes ``dd`` and ``b`` from one sweep instead of the reference's two
            (``fhog/triton_bwdbwd.py:185-251``): 22 instead of 25 recomputed products; ``b`` then differs from the
            default schedule's value only by fp32 summation order.
        schedule: None / "four_pass" (the reference's four sweeps, 25 recomputed products) or one of the opt-in
            schedules "fused_stats" (22), "ddo_early" (23: four sweeps, the second one yields ``ddO`` together with
            ``b_i = dO_i . ddO_i - d_i dd_i``, the third ``dQ2`` alone) and "three_sweep" (20: ``dd``, ``b`` and ``ddO``
            from one sweep, then ``dQ2``, then ``dK2`` and ``dV2``). The last two exist in the 16-bit kernels; fp32
            tensors run the reference schedule whatever is asked, and a launch too small to fill the GPU (with
            ``split=True``) runs the nearest schedule whose passes can split their streamed side.
        return_stats: also return the fp32 row vectors ``(d, dd, b)`` of shape like ``L``.
        only_pass: run a single pass (0..5, see fhog._lib.PASS_*) instead of the whole chain; for tests and profiling.
        split: allocate the larger workspace that lets launches too small to fill the GPU split their streamed side over
            several workgroups (fp32 partial results, added in a fixed order by a second kernel); False keeps the
            minimum workspace of three row statistics.

    Returns:
        dQ2, dK2, dV2, ddO shaped and typed like Q, K, V, O (+ ``(d, dd, b)`` if ``return_stats``).
    """
    tensors = dict(Q=Q, K=K, V=V, O=O, dO=dO, ddQ=ddQ, ddK=ddK, ddV=ddV)
    for n, t in tensors.items():
        if not isinstance(t, torch.Tensor):
            raise TypeError(f"{n} must be a torch.Tensor, got {type(t).__name__}")
    if not isinstance(L, torch.Tensor):
        raise TypeError(f"L must be a torch.Tensor, got {type(L).__name__}")
    if Q.dtype not in _DTYPES:
        raise TypeError(f"unsupported dtype {Q.dtype}; expected torch.bfloat16, torch.float16 or torch.float32")
    for n, t in tensors.items():
        if t.dtype != Q.dtype:
            raise TypeError(f"{n} has dtype {t.dtype}, expected {Q.dtype} like Q")
        if t.device != Q.device:
            raise ValueError(f"{n} is on {t.device}, expected {Q.device} like Q")
    if impl not in _IMPLS:
        raise ValueError(f"impl must be one of {sorted(k for k in _IMPLS if k)} or None, got {impl!r}")
    out_shape_q, out_shape_k = Q.shape, K.shape
    q3, k3, v3, o3, do3, ddq3, ddk3, ddv3 = (_flatten(t, n) for n, t in tensors.items())
    batch, n_q, d = q3.shape
    n_k = k3.shape[1]
    for n, t in (("O", o3), ("dO", do3), ("ddQ", ddq3)):
        if t.shape != q3.shape:
            raise ValueError(f"{n} has shape {tuple(t.shape)}, expected {tuple(q3.shape)} like Q")
    if k3.shape[0] != batch or k3.shape[2] != d:
        raise ValueError(f"K has shape {tuple(k3.shape)}, expected ({batch}, N_K, {d})")
    for n, t in (("V", v3), ("ddK", ddk3), ("ddV", ddv3)):
        if t.shape != k3.shape:
            raise ValueError(f"{n} has shape {tuple(t.shape)}, expected {tuple(k3.shape)} like K")
    if L.numel() != batch * n_q:
        raise ValueError(f"L has {L.numel()} elements, expected batch*N_Q = {batch * n_q}")
    if d not in (32, 64, 128):
        raise ValueError(f"head dim {d} not supported (32, 64 or 128)")
    mask_code(causal, window, n_q, n_k)  # raises on an inapplicable mask
    sched = schedule_code(schedule, fused_stats)
    if not Q.is_cuda:
        raise ValueError("flash_bwdbwd runs on the GPU only: tensors must be on a ROCm device (there is no CPU path)")
    lse = L.reshape(batch, n_q)
    if lse.dtype != torch.float32 or not lse.is_contiguous():
        lse = lse.to(torch.float32).contiguous()

    q3, o3, do3, ddq3 = _prepare_group([q3, o3, do3, ddq3], "q")
    k3, v3, ddk3, ddv3 = _prepare_group([k3, v3, ddk3, ddv3], "k")

    with torch.cuda.device(Q.device):
        dq2 = torch.empty_strided(q3.shape, q3.stride(), dtype=Q.dtype, device=Q.device)
        ddo = torch.empty_strided(q3.shape, q3.stride(), dtype=Q.dtype, device=Q.device)
        dk2 = torch.empty_strided(k3.shape, k3.stride(), dtype=Q.dtype, device=Q.device)
        dv2 = torch.empty_strided(k3.shape, k3.stride(), dtype=Q.dtype, device=Q.device)
        args = _build_args(q3, k3, v3, o3, do3, ddq3, ddk3, ddv3, lse, scale, causal, _IMPLS[impl],
                           (dq2, dk2, dv2, ddo), None, sched, window)
        ws = _workspace(args, Q.device, split)
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        L_ = _lib.lib()
        if only_pass is None:
            _lib.check(L_.fhog_bwdbwd(ctypes.byref(args), stream))
        else:
            _lib.check(L_.fhog_bwdbwd_pass(ctypes.byref(args), int(only_pass), stream))
    res = (dq2.view(out_shape_q) if dq2.is_contiguous() else dq2.reshape(out_shape_q),
           dk2.view(out_shape_k) if dk2.is_contiguous() else dk2.reshape(out_shape_k),
           dv2.view(out_shape_k) if dv2.is_contiguous() else dv2.reshape(out_shape_k),
           ddo.view(out_shape_q) if ddo.is_contiguous() else ddo.reshape(out_shape_q))
    if return_stats:
        st = ws[:3 * batch * n_q].view(3, *L.shape)
        return res + ((st[0], st[1], st[2]),)
    return res


class BwdBwdPlan:
    """Pre-validated call with caller-owned outputs and workspace (no allocation per call).

    For benchmark loops and per-pass profiling; ``flash_bwdbwd`` is the drop-in entry point.
    """

    def __init__(self, Q, K, V, O, dO, ddQ, ddK, ddV, L, scale, *, causal=False, window=None, impl=None,
                 fused_stats=False, schedule=None, split=True):
        ts = [_flatten(t, "tensor") for t in (Q, K, V, O, dO, ddQ, ddK, ddV)]
        q3, k3, v3, o3, do3, ddq3, ddk3, ddv3 = ts
        q3, o3, do3, ddq3 = _prepare_group([q3, o3, do3, ddq3], "q")
        k3, v3, ddk3, ddv3 = _prepare_group([k3, v3, ddk3, ddv3], "k")
        batch, n_q, _ = q3.shape
        lse = L.reshape(batch, n_q).to(torch.float32).contiguous()
        self.keep = (q3, k3, v3, o3, do3, ddq3, ddk3, ddv3, lse)
        self.outs = (torch.empty_like(q3), torch.empty_like(k3), torch.empty_like(v3), torch.empty_like(q3))
        self.args = _build_args(q3, k3, v3, o3, do3, ddq3, ddk3, ddv3, lse, scale, causal, _IMPLS[impl], self.outs, None, schedule_code(schedule, fused_stats), window)
        with torch.cuda.device(Q.device):
            self.ws_all = _workspace(self.args, Q.device, split)   # d | dd | b, then partial results of split launches
        self.ws = self.ws_all[:3 * batch * n_q]
        self.lib = _lib.lib()
        _lib.check(self.lib.fhog_validate(ctypes.byref(self.args)))
        self.impl = self.lib.fhog_select_impl(ctypes.byref(self.args))

    def run(self, stream: Optional[int] = None, only_pass: Optional[int] = None, static_ws: bool = False):
        """Enqueue the call. ``static_ws``: through ``fhog_bwdbwd_static_ws``, which keeps the row statistics and partial
        results in the library's own device array instead of this plan's workspace (``self.ws`` is then not written)."""
        s = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream if stream is None else stream)
        if static_ws:
            if only_pass is not None:
                raise ValueError("static_ws runs the whole chain")
            _lib.check(self.lib.fhog_bwdbwd_static_ws(ctypes.byref(self.args), s))
        elif only_pass is None:
            _lib.check(self.lib.fhog_bwdbwd(ctypes.byref(self.args), s))
        else:
            _lib.check(self.lib.fhog_bwdbwd_pass(ctypes.byref(self.args), int(only_pass), s))
        return self.outs
