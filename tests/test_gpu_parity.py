"""GPU tier: the HIP path (through the C ABI) against the oracle.

Gates (normalised max error, max|x-ref| / max|ref|): 1e-4 for fp32 tensors, 2e-2 for bf16.
Small cases are checked against the fp64 closed form on the CPU (including the row vectors
d, dd, b of each pass); full-size cases against the fp32 torch-autograd double-backward on the
GPU and through size-independent properties.
"""
import math

import numpy as np
import pytest
import torch

from gpu_util import (NAMES, TOL, errors, make_case, normalised_max_error, reference_fp32_gpu, reference_fp64_cpu,
                      require_gpu, run_fhog, with_caches)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _dev():
    return require_gpu()


def test_library_is_the_hip_one():
    from fhog import _lib
    assert _lib.LIB_PATH.exists()
    assert _lib.lib().fhog_abi_version() == 1


# ---------------------------------------------------------------- reference golden tensors
@pytest.mark.parametrize("impl", ["fp32", None])
def test_reference_fixture_bf16(golden, impl):
    """Restates fhog/test_bwdbwd.py:27-82: fixture -> bf16, O and L recomputed, all four outputs compared
    (the reference asserts dv2 only)."""
    g = {k: torch.tensor(v) for k, v in golden.items()}
    x = {n: g[k][None].to(torch.bfloat16).cuda() for n, k in (("Q", "q"), ("K", "k"), ("V", "v"), ("dO", "do"),
                                                               ("ddQ", "ddq"), ("ddK", "ddk"), ("ddV", "ddv"))}
    scale = 1 / math.sqrt(64)
    x = with_caches(x, scale, False)
    outs = run_fhog(x, scale, False, impl=impl)
    for n, o in zip(NAMES, outs):
        assert o.dtype == torch.bfloat16 and o.shape[0] == 1
        err = normalised_max_error(o[0], g[n])
        assert err < 2e-2, (n, err)
    torch.testing.assert_close(outs[2][0].float().cpu(), g["dv2"].to(torch.bfloat16).float(), rtol=1.6e-2, atol=2e-2)


def test_reference_fixture_fp32_tensors(golden):
    """Same tensors kept in fp32 through the fp32-MFMA family, against the fp64 closed form."""
    g = {k: torch.tensor(v) for k, v in golden.items()}
    x = {n: g[k][None].cuda() for n, k in (("Q", "q"), ("K", "k"), ("V", "v"), ("dO", "do"), ("ddQ", "ddq"),
                                            ("ddK", "ddk"), ("ddV", "ddv"))}
    scale = 1 / math.sqrt(64)
    x = with_caches(x, scale, False)
    outs = run_fhog(x, scale, False)
    ref = reference_fp64_cpu(x, scale, False)
    for n, o in zip(NAMES, outs):
        assert normalised_max_error(o, ref[n]) < 1e-4, n


# ---------------------------------------------------------------- fp32 family, small and ragged
@pytest.mark.parametrize("seed", [0, 1, 2])
def test_cfg0_fp32_noncausal(seed):
    """configs[0]: fp32 non-causal B=1 H=2 N=256 d=64, all seven tensors N(0,1)."""
    x = make_case(2, 256, 256, 64, torch.float32, seed)
    scale = 64 ** -0.5
    x = with_caches(x, scale, False)
    outs = run_fhog(x, scale, False, return_stats=True)
    ref = reference_fp64_cpu(x, scale, False)
    e = errors(outs[:4], [ref[n] for n in NAMES])
    assert max(e.values()) < 1e-4, e
    for got, name in zip(outs[4], ("d", "dd", "b")):
        assert normalised_max_error(got, ref[name]) < 1e-4, name
    ag = reference_fp32_gpu(x, scale, False)
    e2 = errors(outs[:4], ag)
    assert max(e2.values()) < 1e-4, e2


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", [(3, 100, 77, 32), (2, 33, 129, 64), (2, 160, 160, 128), (1, 1, 1, 64), (1, 31, 31, 128)])
def test_fp32_family_ragged(shape, causal, dtype):
    batch, n_q, n_k, d = shape
    if causal:
        n_k = n_q
    x = make_case(batch, n_q, n_k, d, dtype, seed=3)
    scale = d ** -0.5
    x = with_caches(x, scale, causal)
    outs = run_fhog(x, scale, causal, impl="fp32", return_stats=True)
    ref = reference_fp64_cpu(x, scale, causal)
    e = errors(outs[:4], [ref[n] for n in NAMES])
    assert max(e.values()) < TOL[dtype], e
    stat_tol = 1e-4 if dtype == torch.float32 else 5e-3   # bf16: O is rounded before d = rowsum(O*dO)
    for got, name in zip(outs[4], ("d", "dd", "b")):
        assert normalised_max_error(got, ref[name]) < stat_tol, name


def test_strided_and_4d_inputs():
    """(B, H, N, d) views with a padded row stride go through without a copy and give the same numbers."""
    B, H, n, d = 2, 3, 64, 64
    scale = d ** -0.5
    x = make_case(B * H, n, n, d, torch.float32, seed=4)
    x = with_caches(x, scale, True)
    base = run_fhog(x, scale, True)
    padded = {}
    for k_, t in x.items():
        if k_ == "L":
            padded[k_] = t.view(B, H, n)
            continue
        buf = torch.zeros(B, H, n, d + 8, dtype=t.dtype, device=t.device)
        buf[..., :d] = t.view(B, H, n, d)
        padded[k_] = buf[..., :d]
    outs = run_fhog(padded, scale, True)
    for a, b in zip(outs, base):
        assert a.shape == (B, H, n, d)
        torch.testing.assert_close(a.reshape(B * H, n, d), b, rtol=0, atol=0)
