"""Autograd surface around the double-backward kernels.

The reference sketches this chain but never finishes it: ``FlashAttention2`` saves
``(q, k, v, output, L)`` and ``is_causal`` (``fhog/triton_flash.py:136-198``) and the
``Bwd`` Function that would route ``create_graph=True`` into ``flash_bwdbwd`` is a
commented stub (``fhog/triton_bwdbwd.py:538-554``).  Here it is wired:

    FlashAttention.forward   -> O, saves (q, k, v, O, L)
    FlashAttention.backward  -> AttnBwd.apply(q, k, v, O, dO, L, scale, causal)
    AttnBwd.forward          -> dQ, dK, dV   (first-order backward)
    AttnBwd.backward         -> flash_bwdbwd(...) -> dQ', dK', dV', ddO

The forward and the first-order backward are the callers on either side of the hot path.  They run as HIP
kernels of the same library (``fhog_attn_fwd`` / ``fhog_attn_bwd``): 16-bit MFMA kernels for bf16 and fp16 tensors
with d in {64, 128}, fp32-MFMA kernels for fp32 tensors and d = 32.  A linear-memory torch composition on the GPU
(blocked over heads and query rows, fp32 accumulation) remains for arguments the kernels reject (a non-positive
scale on 16-bit tensors) and as the second implementation the tests compare with (``use_hip=False``).
The double-backward is always the HIP library.
"""
from __future__ import annotations

import math
import warnings
from typing import Optional, Tuple

import ctypes

import torch

from . import _lib
from .bwdbwd import flash_bwdbwd, mask_code

_HIP_DTYPES = {torch.bfloat16: _lib.DTYPE_BF16, torch.float16: _lib.DTYPE_FP16, torch.float32: _lib.DTYPE_FP32}
_BLOCK_ELEMS = 1 << 26  # fp32 elements of one materialised (heads, rows, N_K) block (256 MiB)


def _blocks(batch: int, n_q: int, n_k: int):
    """Yield (head slice, row slice) so that heads*rows*n_k stays below the block budget."""
    rows = max(1, min(n_q, _BLOCK_ELEMS // max(1, n_k)))
    heads = max(1, min(batch, _BLOCK_ELEMS // (rows * n_k)))
    for b0 in range(0, batch, heads):
        for r0 in range(0, n_q, rows):
            yield slice(b0, min(batch, b0 + heads)), slice(r0, min(n_q, r0 + rows))


def _scores(q, k, scale, causal, r0, n_q=None, window=None):
    """fp32 scores of query rows r0.. against all keys, masked entries at -inf."""
    s = torch.matmul(q.float(), k.float().transpose(-1, -2)) * scale
    if causal:
        n_r, n_k = s.shape[-2], s.shape[-1]
        shift = (n_k - n_q) if causal == "bottom_right" else 0
        qi = torch.arange(r0, r0 + n_r, device=s.device)[:, None] + shift
        kj = torch.arange(n_k, device=s.device)[None, :]
        hidden = kj > qi
        if window is not None:
            hidden = hidden | (qi - kj >= window)
        s = s.masked_fill(hidden, float("-inf"))
    return s



class _NotCovered(Exception):
    """The HIP first-order kernels do not take these arguments; the message says why."""


def _hip_args(q, k, v, scale, causal, window=None) -> _lib.AttnArgs:
    """Arguments for the HIP first-order kernels; raises _NotCovered when they do not cover these tensors."""
    if not q.is_cuda:
        raise _NotCovered("the tensors are not on a ROCm device")
    if q.dtype not in _HIP_DTYPES or not (k.dtype == v.dtype == q.dtype):
        raise _NotCovered(f"dtypes {q.dtype}, {k.dtype}, {v.dtype}: need one of bf16, fp16, fp32 for all tensors")
    a = _lib.AttnArgs()
    a.q, a.k, a.v = q.data_ptr(), k.data_ptr(), v.data_ptr()
    a.batch, a.n_q, a.d = q.shape
    a.n_k = k.shape[1]
    a.stride_qb, a.stride_qn = q.stride(0), q.stride(1)
    a.stride_kb, a.stride_kn = k.stride(0), k.stride(1)
    a.scale, a.dtype = float(scale), _HIP_DTYPES[q.dtype]
    a.causal, a.window = mask_code(causal, window, q.shape[1], k.shape[1])
    return a


def _same_layout(ts) -> bool:
    return all(t.stride() == ts[0].stride() and t.stride(-1) == 1 for t in ts)


def _attention_forward_hip(q, k, v, scale, causal, window=None):
    """O and L from ``fhog_attn_fwd``; raises _NotCovered when the kernels do not cover the arguments."""
    q, k, v = (t if t.stride(-1) == 1 else t.contiguous() for t in (q, k, v))
    if not _same_layout([k, v]):
        k, v = k.contiguous(), v.contiguous()
    a = _hip_args(q, k, v, scale, causal, window)
    L_ = _lib.lib()
    with torch.cuda.device(q.device):
        o = torch.empty_strided(q.shape, q.stride(), dtype=q.dtype, device=q.device)
        lse = torch.empty(q.shape[0], q.shape[1], dtype=torch.float32, device=q.device)
        a.o, a.lse = o.data_ptr(), lse.data_ptr()
        if L_.fhog_attn_validate(ctypes.byref(a), 0) != 0:
            raise _NotCovered(L_.fhog_last_error().decode())
        _lib.check(L_.fhog_attn_fwd(ctypes.byref(a), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    return o, lse


def _attention_backward_hip(q, k, v, o, do, L, scale, causal, window=None):
    ts_q = [t if t.stride(-1) == 1 else t.contiguous() for t in (q, o, do)]
    if not _same_layout(ts_q):
        ts_q = [t.contiguous() for t in ts_q]
    ts_k = [t if t.stride(-1) == 1 else t.contiguous() for t in (k, v)]
    if not _same_layout(ts_k):
        ts_k = [t.contiguous() for t in ts_k]
    (q, o, do), (k, v) = ts_q, ts_k
    a = _hip_args(q, k, v, scale, causal, window)
    if o.dtype != q.dtype or do.dtype != q.dtype:
        raise _NotCovered(f"O and dO have dtypes {o.dtype}, {do.dtype}: need {q.dtype} like Q")
    L_ = _lib.lib()
    with torch.cuda.device(q.device):
        lse = L.reshape(q.shape[0], q.shape[1]).to(torch.float32).contiguous()
        dq = torch.empty_strided(q.shape, q.stride(), dtype=q.dtype, device=q.device)
        dk = torch.empty_strided(k.shape, k.stride(), dtype=k.dtype, device=k.device)
        dv = torch.empty_strided(k.shape, k.stride(), dtype=k.dtype, device=k.device)
        ws = torch.empty(q.shape[0] * q.shape[1], dtype=torch.float32, device=q.device)
        a.o, a.lse, a.dO = o.data_ptr(), lse.data_ptr(), do.data_ptr()
        a.dq, a.dk, a.dv, a.ws = dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), ws.data_ptr()
        if L_.fhog_attn_validate(ctypes.byref(a), 1) != 0:
            raise _NotCovered(L_.fhog_last_error().decode())
        _lib.check(L_.fhog_attn_bwd(ctypes.byref(a), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    return dq, dk, dv


class TorchCompositionWarning(RuntimeWarning):
    """A first-order call left the HIP kernels for the blocked torch composition (10-100x slower)."""


def _second_path(func: str, entry: str, why: Exception, use_hip: Optional[bool]) -> None:
    """The HIP kernel refused the arguments: an error under ``use_hip=True``, else a warning that names the reason
    before the caller goes on to the blocked torch composition (never silently: the composition is 10-100x slower)."""
    if use_hip:
        raise ValueError(f"{entry} does not cover these arguments: {why}")
    warnings.warn(f"fhog.{func}: {entry} does not cover these arguments ({why}); running the blocked torch composition "
                  "instead, which is far slower. Pass use_hip=False to choose it on purpose.",
                  TorchCompositionWarning, stacklevel=3)


def attention_forward(q, k, v, scale: Optional[float] = None, causal=False, *, window: Optional[int] = None,
                      use_hip: Optional[bool] = None):
    """O (dtype of q) and fp32 L = logsumexp_j(scale q.k_j) for (batch, N, d) tensors.

    Takes the place of the reference's forward kernel outputs (``fhog/triton_flash.py:123-133``)
    and of ``produce_L`` (``fhog/triton_flash.py:252-258``), with causal support and without an
    (batch, N_Q, N_K) allocation.

    ``use_hip``: None = the HIP kernel; when it refuses the arguments (a non-positive scale with 16-bit tensors, strides
    that are not multiples of 16 bytes, CPU tensors), a ``TorchCompositionWarning`` names the reason and the blocked
    torch composition runs instead. True = the HIP kernel or a ``ValueError``; False = the torch composition.
    """
    if q.dim() == 4:
        B, H = q.shape[:2]
        o, L = attention_forward(q.flatten(0, 1), k.flatten(0, 1), v.flatten(0, 1), scale, causal, window=window,
                                 use_hip=use_hip)
        return o.view(q.shape), L.view(B, H, -1)
    batch, n_q, d = q.shape
    n_k = k.shape[1]
    mask_code(causal, window, n_q, n_k)  # raises on an inapplicable mask
    scale = d ** -0.5 if scale is None else scale
    if use_hip is not False:
        try:
            return _attention_forward_hip(q, k, v, scale, causal, window)
        except _NotCovered as why:
            _second_path("attention_forward", "fhog_attn_fwd", why, use_hip)
    o = torch.empty_like(q)
    L = torch.empty(batch, n_q, dtype=torch.float32, device=q.device)
    for hs, rs in _blocks(batch, n_q, n_k):
        s = _scores(q[hs, rs], k[hs], scale, causal, rs.start, n_q, window)
        lse = torch.logsumexp(s, dim=-1)
        p = torch.exp(s - lse[..., None])
        o[hs, rs] = torch.matmul(p, v[hs].float()).to(q.dtype)
        L[hs, rs] = lse
    return o, L


def produce_L(Q, K, is_causal: bool = False):
    """fp32 log-sum-exp of ``Q K^T / sqrt(d)``; same call as ``fhog/triton_flash.py:252-258``
    (which raises on causal and returns the input dtype)."""
    return attention_forward(Q, K, K, None, is_causal)[1]


def attention_backward(q, k, v, o, do, L, scale: float, causal, *, window: Optional[int] = None,
                       use_hip: Optional[bool] = None):
    """First-order backward (dQ, dK, dV); the arithmetic of ``fhog/triton_flash.py:201-220`` without the
    (batch, N_Q, N_K) tensors. ``use_hip`` as in :func:`attention_forward`."""
    batch, n_q, d = q.shape
    n_k = k.shape[1]
    if use_hip is not False:
        try:
            return _attention_backward_hip(q, k, v, o, do, L, scale, causal, window)
        except _NotCovered as why:
            _second_path("attention_backward", "fhog_attn_bwd", why, use_hip)
    dq = torch.empty_like(q)
    dk = torch.zeros(k.shape, dtype=torch.float32, device=k.device)
    dv = torch.zeros(v.shape, dtype=torch.float32, device=v.device)
    for hs, rs in _blocks(batch, n_q, n_k):
        qf, dof = q[hs, rs].float(), do[hs, rs].float()
        s = _scores(q[hs, rs], k[hs], scale, causal, rs.start, n_q, window)
        p = torch.exp(s - L[hs, rs].float()[..., None])
        dsum = (o[hs, rs].float() * dof).sum(-1, keepdim=True)
        dp = torch.matmul(dof, v[hs].float().transpose(-1, -2))
        ds = p * (dp - dsum) * scale
        dq[hs, rs] = torch.matmul(ds, k[hs].float()).to(q.dtype)
        dk[hs] += torch.matmul(ds.transpose(-1, -2), qf)
        dv[hs] += torch.matmul(p.transpose(-1, -2), dof)
    return dq, dk.to(k.dtype), dv.to(v.dtype)


class AttnBwd(torch.autograd.Function):
    """First-order attention backward as a differentiable node; its backward is the HIP double-backward.

    Signature follows the reference's stub ``Bwd.forward(ctx, Q, K, V, dO, L, scale)``
    (``fhog/triton_bwdbwd.py:538-554``) plus the cached ``O`` and the causal flag.
    """

    @staticmethod
    def forward(ctx, q, k, v, o, do, L, scale, causal, window=None, schedule=None):
        ctx.save_for_backward(q, k, v, o, do, L)
        ctx.scale = scale
        ctx.causal = causal
        ctx.window = window
        ctx.schedule = schedule
        sq = q.shape
        f = (lambda t: t.flatten(0, 1)) if q.dim() == 4 else (lambda t: t)
        dq, dk, dv = attention_backward(f(q), f(k), f(v), f(o), f(do), f(L), scale, causal, window=window)
        return dq.view(sq), dk.view(k.shape), dv.view(v.shape)

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, ddq, ddk, ddv):
        q, k, v, o, do, L = ctx.saved_tensors
        dq2, dk2, dv2, ddo = flash_bwdbwd(q, k, v, o, do, ddq.contiguous(), ddk.contiguous(), ddv.contiguous(), L,
                                          ctx.scale, causal=ctx.causal, window=ctx.window, schedule=ctx.schedule)
        # O and L are caches of (q, k, v): the four results are already total derivatives.
        return dq2, dk2, dv2, None, ddo, None, None, None, None, None


class FlashAttention(torch.autograd.Function):
    """``FlashAttention.apply(q, k, v, is_causal)`` - call-compatible with the reference's
    ``FlashAttention2`` (``fhog/triton_flash.py:136-198``), twice differentiable."""

    @staticmethod
    def forward(ctx, q, k, v, is_causal=False, window=None, schedule=None):
        scale = q.shape[-1] ** -0.5
        o, L = attention_forward(q, k, v, scale, is_causal, window=window)
        ctx.save_for_backward(q, k, v, o, L)
        ctx.is_causal = is_causal
        ctx.window = window
        ctx.schedule = schedule
        ctx.scale = scale
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, o, L = ctx.saved_tensors
        dq, dk, dv = AttnBwd.apply(q, k, v, o, do.contiguous(), L, ctx.scale, ctx.is_causal, ctx.window, ctx.schedule)
        return dq, dk, dv, None, None, None


def attention(q, k, v, is_causal=False, window: Optional[int] = None, schedule: Optional[str] = None):
    """Twice-differentiable scaled-dot-product attention (scale = d^-1/2). ``is_causal``: False | True |
    "bottom_right"; ``window``: sliding-window length on top of a causal mask; ``schedule``: pass schedule of the
    double-backward (see :func:`fhog.flash_bwdbwd`; None = the reference's four passes)."""
    return FlashAttention.apply(q, k, v, is_causal, window, schedule)
