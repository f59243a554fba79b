"""CPU oracle for the attention double-backward (Flash Hog) path.

THIS IS TEST INFRASTRUCTURE.  Nothing in the shipped package may import it; only
``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` do, and there only as the checker / reported baseline.

Two independent statements of the same function live here:

* :func:`closed_form` - the materialised formulas of the reference in numpy
  float64.  Follows ``fhog/jax_refs/jax_impl.py:286-354`` (``attn_bwd_bwd_stats``,
  the function that generated the reference's golden tensors),
  ``fhog/jax_refs/torch_impl.py:14-79`` and the per-tile arithmetic of the Triton
  kernels ``fhog/triton_bwdbwd.py:194-202,229-243,266-288,485-507``.
  It also returns the per-row intermediates ``L, d, dd, b`` so that every pass
  of the device path can be checked on its own.
* :func:`autograd_double_backward` - ``torch.autograd.grad(create_graph=True)``
  applied twice to materialised softmax attention: a library routine that does
  not share a single formula with :func:`closed_form`.  This is the parity
  definition of the build (fp32 on the GPU tier, fp64 on the CPU tier).

Mask conventions: ``causal=True`` is top-left, ``P_ij = 0`` for ``j > i`` (what
``fhog/triton_flash.py:86-92`` and ``F.scaled_dot_product_attention(is_causal=True)``
use).  ``causal="bottom_right"`` with an optional ``window`` is the mask of
``fhog/jax_refs/jax_impl.py:110-115`` (key j visible iff ``0 <= i + N_K - N_Q - j < window``);
for ``N_Q == N_K`` and no window the two are the same.

Pinning status (tests/test_oracle.py):
  closed_form          pinned: == autograd (fp64, <=1e-10), == reference golden
                       tensors (bf16 tolerance, all four outputs), brute-force
                       scalar loops, adjoint identity vs central differences,
                       SDPA special case, row identities.
  autograd_double_backward  pinned by the same cross-checks (it is the other side).
  causal, d=128, N>256, fp32 inputs: no reference-held vector exists (the
  reference implements none of them); pinned by autograd == closed_form and the
  mathematical checks only.
  bottom-right / sliding-window masks: no reference-held vector either; pinned by
  closed_form == autograd == brute force on the same mask, by the mask itself
  against the index formula of jax_impl.py:110-115, and by the reductions to known
  cases (window >= N: plain causal; N_Q == N_K: top-left; window = 1: one key per
  query, for which every gradient through the soft-max vanishes).
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import numpy as np
import torch

__all__ = [
    "closed_form",
    "autograd_double_backward",
    "forward_o_lse",
    "first_backward",
    "brute_force",
    "normalised_max_error",
]


def _mask(n_q: int, n_k: int, causal=True, window: Optional[int] = None) -> Optional[np.ndarray]:
    """Visibility mask: True where key j may be attended by query i; None when nothing is masked.

    ``causal``: False | True (top-left: j <= i) | "bottom_right" (j <= i + N_K - N_Q, the mask of
    ``fhog/jax_refs/jax_impl.py:110-115``).  ``window`` adds the sliding-window bound of the same
    function: (shifted i) - j < window.
    """
    if not causal:
        if window is not None:
            raise ValueError("a sliding window needs a causal mask")
        return None
    if causal not in (True, "bottom_right"):
        raise ValueError(f"unknown mask {causal!r}")
    qi = np.arange(n_q)[:, None] + ((n_k - n_q) if causal == "bottom_right" else 0)
    kj = np.arange(n_k)[None, :]
    m = qi >= kj
    if window is not None:
        m &= (qi - kj) < window
    return m


def forward_o_lse(q, k, v, scale: float, causal=False, window: Optional[int] = None):
    """Materialised forward in float64: returns (O, L) with L = logsumexp_j(scale q.k).

    ``L`` is what ``fhog/triton_flash.py:252-258`` (``produce_L``) and the forward
    kernel (``fhog/triton_flash.py:123-133``) hand to the double-backward.
    Shapes: q (..., N_Q, d), k/v (..., N_K, d).
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    s = scale * np.einsum("...id,...jd->...ij", q, k)
    m_ = _mask(q.shape[-2], k.shape[-2], causal, window)
    if m_ is not None:
        s = np.where(m_, s, -np.inf)
    m = s.max(axis=-1, keepdims=True)
    e = np.exp(s - m)
    l = e.sum(axis=-1, keepdims=True)
    lse = (m + np.log(l))[..., 0]
    o = np.einsum("...ij,...jd->...id", e / l, v)
    return o, lse


def first_backward(q, k, v, do, scale: float, causal=False, window: Optional[int] = None):
    """Materialised first-order attention backward (dQ, dK, dV) in float64.

    Same arithmetic as ``fhog/triton_flash.py:201-220``; used by the adjoint test.
    """
    q, k, v, do = (np.asarray(t, dtype=np.float64) for t in (q, k, v, do))
    o, lse = forward_o_lse(q, k, v, scale, causal, window)
    s = scale * np.einsum("...id,...jd->...ij", q, k)
    p = np.exp(s - lse[..., None])
    m_ = _mask(q.shape[-2], k.shape[-2], causal, window)
    if m_ is not None:
        p = np.where(m_, p, 0.0)
    d = np.einsum("...id,...id->...i", o, do)
    dp = np.einsum("...id,...jd->...ij", do, v)
    ds = scale * p * (dp - d[..., None])
    dq = np.einsum("...ij,...jd->...id", ds, k)
    dk = np.einsum("...ij,...id->...jd", ds, q)
    dv = np.einsum("...ij,...id->...jd", p, do)
    return dq, dk, dv


def closed_form(q, k, v, do, ddq, ddk, ddv, scale: float, causal=False,
                o: Optional[np.ndarray] = None, lse: Optional[np.ndarray] = None,
                window: Optional[int] = None) -> Dict[str, np.ndarray]:
    """Materialised double-backward in float64.

    Inputs broadcast over leading dims; q, do, ddq: (..., N_Q, d); k, v, ddk, ddv: (..., N_K, d).
    ``o`` / ``lse`` may be supplied (the device path receives them as caches); when
    omitted they are recomputed exactly.

    Returns dict with dq2, dk2, dv2, ddo and the row vectors L, d, dd, b and o.
    """
    q, k, v, do, ddq, ddk, ddv = (np.asarray(t, dtype=np.float64) for t in (q, k, v, do, ddq, ddk, ddv))
    if o is None or lse is None:
        o_x, lse_x = forward_o_lse(q, k, v, scale, causal, window)
        o = o_x if o is None else np.asarray(o, dtype=np.float64)
        lse = lse_x if lse is None else np.asarray(lse, dtype=np.float64)
    else:
        o = np.asarray(o, dtype=np.float64)
        lse = np.asarray(lse, dtype=np.float64)

    s = scale * np.einsum("...id,...jd->...ij", q, k)            # jax_impl.py:314-319
    p = np.exp(s - lse[..., None])                               # jax_impl.py:326
    m_ = _mask(q.shape[-2], k.shape[-2], causal, window)
    if m_ is not None:
        p = np.where(m_, p, 0.0)   # jax_impl.py:321-324
    dp = np.einsum("...id,...jd->...ij", do, v)                  # jax_impl.py:328
    dds = scale * (np.einsum("...id,...jd->...ij", ddq, k)
                   + np.einsum("...id,...jd->...ij", q, ddk))    # jax_impl.py:329
    d = np.einsum("...id,...id->...i", o, do)                    # jax_impl.py:336, triton_bwdbwd.py:580
    dd = np.einsum("...ij,...ij->...i", dds, p)                  # jax_impl.py:337, triton_bwdbwd.py:203
    dp2 = (np.einsum("...id,...jd->...ij", do, ddv)
           - dp * dd[..., None] - dds * d[..., None] + dp * dds)  # jax_impl.py:340, triton_bwdbwd.py:232-237
    b = np.einsum("...ij,...ij->...i", dp2, p)                   # jax_impl.py:343, triton_bwdbwd.py:238
    ddp = p * (dds - dd[..., None])                              # jax_impl.py:341
    ds2 = scale * p * (dp2 - b[..., None])                       # jax_impl.py:343
    ds = scale * p * (dp - d[..., None])                         # jax_impl.py:345
    dq2 = np.einsum("...ij,...jd->...id", ds, ddk) + np.einsum("...ij,...jd->...id", ds2, k)   # :347
    dk2 = np.einsum("...ij,...id->...jd", ds, ddq) + np.einsum("...ij,...id->...jd", ds2, q)   # :348
    dv2 = np.einsum("...ij,...id->...jd", ddp, do)                                              # :350
    ddo = np.einsum("...ij,...jd->...id", p, ddv) + np.einsum("...ij,...jd->...id", ddp, v)     # :352
    return dict(dq2=dq2, dk2=dk2, dv2=dv2, ddo=ddo, L=lse, d=d, dd=dd, b=b, o=o)


def autograd_double_backward(q, k, v, do, ddq, ddk, ddv, scale: float, causal=False,
                             dtype: torch.dtype = torch.float64, head_chunk: int = 1, window: Optional[int] = None):
    """Double backward through materialised softmax attention with torch autograd.

    Accepts torch tensors or numpy arrays of shape (batch, N, d) (or (N, d)); loops
    over the batch dim in chunks of ``head_chunk`` so that only ``head_chunk``
    (N_Q, N_K) graphs are alive at once.  Returns (dq2, dk2, dv2, ddo) as torch
    tensors of ``dtype`` on the input device.
    """
    ts = [torch.as_tensor(t) for t in (q, k, v, do, ddq, ddk, ddv)]
    squeeze = ts[0].dim() == 2
    if squeeze:
        ts = [t.unsqueeze(0) for t in ts]
    ts = [t.to(dtype) for t in ts]
    q_, k_, v_, do_, ddq_, ddk_, ddv_ = ts
    batch, n_q, _ = q_.shape
    n_k = k_.shape[1]
    outs = [torch.empty_like(q_), torch.empty_like(k_), torch.empty_like(v_), torch.empty_like(do_)]
    mask = _mask(n_q, n_k, causal, window)
    if mask is not None:
        mask = torch.from_numpy(mask).to(q_.device)
    for b0 in range(0, batch, head_chunk):
        sl = slice(b0, min(batch, b0 + head_chunk))
        qh = q_[sl].detach().clone().requires_grad_(True)
        kh = k_[sl].detach().clone().requires_grad_(True)
        vh = v_[sl].detach().clone().requires_grad_(True)
        doh = do_[sl].detach().clone().requires_grad_(True)
        s = torch.matmul(qh, kh.transpose(-1, -2)) * scale
        if mask is not None:
            s = s.masked_fill(~mask, float("-inf"))
        p = torch.softmax(s, dim=-1)
        o = torch.matmul(p, vh)
        dq, dk, dv = torch.autograd.grad(o, (qh, kh, vh), doh, create_graph=True)
        g = torch.autograd.grad((dq, dk, dv), (qh, kh, vh, doh), (ddq_[sl], ddk_[sl], ddv_[sl]))
        for dst, src in zip(outs, g):
            dst[sl] = src.detach()
    if squeeze:
        outs = [t[0] for t in outs]
    return tuple(outs)


def brute_force(q, k, v, do, ddq, ddk, ddv, scale: float, causal=False, window: Optional[int] = None):
    """Scalar-loop evaluation for tiny single-head inputs (N <= 8, d <= 4).

    Written index by index from the handwritten equations
    (``assets/handwritten_equations.png``), without einsum, so that a transposed
    operand or a dropped term in :func:`closed_form` cannot also hide here.
    Returns (dq2, dk2, dv2, ddo) as nested float64 arrays.
    """
    q, k, v, do, ddq, ddk, ddv = (np.asarray(t, dtype=np.float64) for t in (q, k, v, do, ddq, ddk, ddv))
    nq, dh = q.shape
    nk = k.shape[0]
    P = np.zeros((nq, nk)); dP = np.zeros((nq, nk)); ddS = np.zeros((nq, nk)); E = np.zeros((nq, nk))
    O = np.zeros((nq, dh))
    for i in range(nq):
        srow = []
        for j in range(nk):
            sij = 0.0
            for c in range(dh):
                sij += q[i, c] * k[j, c]
            srow.append(scale * sij)
        shift = (nk - nq) if causal == "bottom_right" else 0
        allowed = [j for j in range(nk)
                   if (not causal) or (j <= i + shift and (window is None or i + shift - j < window))]
        mx = max(srow[j] for j in allowed)
        z = sum(math.exp(srow[j] - mx) for j in allowed)
        for j in allowed:
            P[i, j] = math.exp(srow[j] - mx) / z
        for j in range(nk):
            for c in range(dh):
                dP[i, j] += do[i, c] * v[j, c]
                ddS[i, j] += scale * (ddq[i, c] * k[j, c] + q[i, c] * ddk[j, c])
                E[i, j] += do[i, c] * ddv[j, c]
                O[i, c] += P[i, j] * v[j, c]
    dq2 = np.zeros_like(q); dk2 = np.zeros_like(k); dv2 = np.zeros_like(v); ddo = np.zeros_like(do)
    for i in range(nq):
        d_i = sum(O[i, c] * do[i, c] for c in range(dh))
        dd_i = sum(ddS[i, j] * P[i, j] for j in range(nk))
        dP2 = [E[i, j] - dP[i, j] * dd_i - ddS[i, j] * d_i + dP[i, j] * ddS[i, j] for j in range(nk)]
        b_i = sum(dP2[j] * P[i, j] for j in range(nk))
        for j in range(nk):
            ddP = P[i, j] * (ddS[i, j] - dd_i)
            dS2 = scale * P[i, j] * (dP2[j] - b_i)
            dS = scale * P[i, j] * (dP[i, j] - d_i)
            for c in range(dh):
                dq2[i, c] += dS * ddk[j, c] + dS2 * k[j, c]
                dk2[j, c] += dS * ddq[i, c] + dS2 * q[i, c]
                dv2[j, c] += ddP * do[i, c]
                ddo[i, c] += P[i, j] * ddv[j, c] + ddP * v[j, c]
    return dq2, dk2, dv2, ddo


def normalised_max_error(x, ref) -> float:
    """max|x - ref| / max|ref| - the error metric of the parity gates."""
    x = torch.as_tensor(x).detach().double().cpu()
    ref = torch.as_tensor(ref).detach().double().cpu()
    den = ref.abs().max().item()
    return (x - ref).abs().max().item() / (den if den > 0 else 1.0)
