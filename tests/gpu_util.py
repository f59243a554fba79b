"""Helpers of the GPU tier: seeded cases, references, error metric. Imports the oracle as the checker."""
import math

import torch

from oracle.bwdbwd_oracle import autograd_double_backward, closed_form, normalised_max_error  # noqa: F401

NAMES = ("dq2", "dk2", "dv2", "ddo")
TOL = {torch.float32: 1e-4, torch.bfloat16: 2e-2}   # north-star gates: normalised max error


def require_gpu():
    assert torch.cuda.is_available(), "GPU tier needs a ROCm device"
    torch.backends.cuda.matmul.allow_tf32 = False
    return torch.device("cuda:0")


def make_case(batch, n_q, n_k, d, dtype, seed, grad_std=1.0, k_row_scale=False, device="cuda:0"):
    g = torch.Generator(device="cpu").manual_seed(seed)
    qs, ks = (batch, n_q, d), (batch, n_k, d)
    x = {}
    for name, shape, std in (("Q", qs, 1.0), ("K", ks, 1.0), ("V", ks, 1.0), ("dO", qs, grad_std), ("ddQ", qs, grad_std),
                             ("ddK", ks, grad_std), ("ddV", ks, grad_std)):
        x[name] = torch.randn(shape, generator=g, dtype=torch.float32) * std
    if k_row_scale:
        x["K"] = x["K"] * (torch.rand((batch, n_k, 1), generator=g) * 1.5 + 0.5)
    return {n: t.to(dtype).to(device) for n, t in x.items()}


def with_caches(x, scale, causal, window=None):
    """Add O (input dtype) and fp32 L from an fp32 forward on the rounded inputs."""
    import fhog
    o, L = fhog.attention_forward(x["Q"], x["K"], x["V"], scale, causal, window=window,
                                  use_hip=False)  # fp32 forward on the rounded inputs
    return dict(x, O=o, L=L)


def run_fhog(x, scale, causal, impl=None, **kw):
    import fhog
    return fhog.flash_bwdbwd(x["Q"], x["K"], x["V"], x["O"], x["dO"], x["ddQ"], x["ddK"], x["ddV"], x["L"], scale,
                             causal=causal, impl=impl, **kw)


def reference_fp32_gpu(x, scale, causal, heads=None, head_chunk=1, window=None):
    """fp32 torch autograd double-backward on materialised attention, on the GPU, head-chunked."""
    sel = (lambda t: t) if heads is None else (lambda t: t[heads])
    return autograd_double_backward(sel(x["Q"]), sel(x["K"]), sel(x["V"]), sel(x["dO"]), sel(x["ddQ"]), sel(x["ddK"]),
                                    sel(x["ddV"]), scale, causal, dtype=torch.float32, head_chunk=head_chunk, window=window)


def reference_fp64_cpu(x, scale, causal, window=None, heads=None):
    """fp64 closed form on the CPU (outputs and the row vectors d, dd, b), optionally on a few (batch*head) slices."""
    sel = (lambda t: t) if heads is None else (lambda t: t[heads])
    c = {n: sel(t).detach().double().cpu().numpy() for n, t in x.items()}
    return closed_form(c["Q"], c["K"], c["V"], c["dO"], c["ddQ"], c["ddK"], c["ddV"], scale, causal, window=window)


def errors(outs, refs):
    return {n: normalised_max_error(o, r) for n, o, r in zip(NAMES, outs, refs)}
