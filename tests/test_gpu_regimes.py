"""GPU tier: the regimes either side of the benchmark configurations.

* the reference's own benchmark sweep far beyond its first point (fhog/benchhhh.py:15-27,93-108: one head, d = 64,
  fp16, non-causal, N up to 2097152), pinned at N = 131072 by quantities that stay affordable there: sampled query rows
  against the fp64 closed form (non-causal rows are independent), the zero column sums of the key-side outputs, and the
  fp32-MFMA kernels on the same tensors;
* `fhog.produce_L` (fhog/triton_flash.py:252-258) against the oracle's log-sum-exp;
* the launch choices behind FHOG_TUNE, each forced in a child process (the variable is read once per process), on a shape
  the defaults would never give them.
"""
import os
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

from gpu_util import (NAMES, errors, make_case, normalised_max_error, reference_fp64_cpu, require_gpu, run_fhog,
                      with_caches)
from oracle.bwdbwd_oracle import closed_form, forward_o_lse

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent


@pytest.fixture(scope="module", autouse=True)
def _dev():
    return require_gpu()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_reference_sweep_regime_long_n_131072(dtype):
    """N = 131072, one head, d = 64, non-causal: P = exp(S - L) is of the order 1 / N = 8e-6, below fp16's smallest
    normal number (6e-5) and in the middle of bf16's range."""
    import fhog
    n, d, rows = 131072, 64, 64
    scale = d ** -0.5
    x = make_case(1, n, n, d, dtype, seed=43, grad_std=0.1)
    o, L = fhog.attention_forward(x["Q"], x["K"], x["V"], scale, False, use_hip=True)   # linear memory, fp32 L
    x = dict(x, O=o, L=L)
    dq2, dk2, dv2, ddo, (dsum, dd, b) = run_fhog(x, scale, False, return_stats=True)
    for t in (dq2, dk2, dv2, ddo, dsum, dd, b):
        assert torch.isfinite(t.float()).all()

    # (1) 64 query rows spread over the sequence against the fp64 closed form on those rows and ALL keys
    sel = torch.linspace(0, n - 1, rows).long()
    c = {k_: (v_[0, sel] if k_ in ("Q", "dO", "ddQ") else v_[0]).double().cpu().numpy() for k_, v_ in x.items()
         if k_ in ("Q", "K", "V", "dO", "ddQ", "ddK", "ddV")}
    ref = closed_form(c["Q"], c["K"], c["V"], c["dO"], c["ddQ"], c["ddK"], c["ddV"], scale, False)
    sel_dev = sel.to(dq2.device)
    assert normalised_max_error(L[0, sel_dev], ref["L"]) < 1e-3
    e_rows = {"dq2": normalised_max_error(dq2[0, sel_dev], ref["dq2"]), "ddo": normalised_max_error(ddo[0, sel_dev], ref["ddo"])}
    e_stat = {"d": normalised_max_error(dsum[0, sel_dev], ref["d"]), "dd": normalised_max_error(dd[0, sel_dev], ref["dd"]),
              "b": normalised_max_error(b[0, sel_dev], ref["b"])}
    print(f"long-N {dtype}: sampled rows {e_rows}, statistics {e_stat}")
    assert max(e_rows.values()) < 2e-2, e_rows
    assert max(e_stat.values()) < 1e-2, e_stat

    # (2) sum_j dK2_j = sum_j dV2_j = 0 for the exact quantities (tests/test_oracle.py::test_row_identities). On the device
    # every output element carries a rounding error of at most 2^-8 of its size; N of them add up like a random walk.
    # A systematic loss (probabilities flushed to zero, a biased P) grows like N instead and breaks the bound.
    for name, t in (("dk2", dk2), ("dv2", dv2)):
        col = t[0].double().sum(0).abs().max().item()
        bound = 1e-2 * t.float().abs().max().item() * n ** 0.5
        print(f"long-N {dtype}: |sum_j {name}_j| = {col:.3e}, bound {bound:.3e}")
        assert col < bound, (name, col, bound)

    # (3) the key-side outputs against the fp32-MFMA kernels on the same tensors (every product and intermediate in fp32)
    _, dk2_32, dv2_32, _ = run_fhog(x, scale, False, impl="fp32")
    e_k = {"dk2": normalised_max_error(dk2, dk2_32.float()), "dv2": normalised_max_error(dv2, dv2_32.float())}
    print(f"long-N {dtype}: against the fp32-MFMA family {e_k}")
    assert max(e_k.values()) < 2e-2, e_k


def test_produce_L_is_the_oracle_logsumexp():
    """`fhog.produce_L(Q, K)` (the reference's helper, fhog/triton_flash.py:252-258) in fp32 from the HIP forward."""
    import fhog
    x = make_case(3, 200, 333, 64, torch.bfloat16, seed=44)
    L = fhog.produce_L(x["Q"], x["K"])
    assert L.dtype == torch.float32 and L.shape == (3, 200)
    q, k = (x[n_].double().cpu().numpy() for n_ in ("Q", "K"))
    want = forward_o_lse(q, k, k, 64 ** -0.5, False)[1]
    assert np.abs(L.cpu().numpy() - want).max() < 2e-3
    Lc = fhog.produce_L(x["Q"][:, :, :], x["K"][:, :200], True)
    want_c = forward_o_lse(q, k[:, :200], k[:, :200], 64 ** -0.5, True)[1]
    assert np.abs(Lc.cpu().numpy() - want_c).max() < 2e-3


_CHILD = r"""
import sys, torch
sys.path[:0] = [{root!r} + "/flash-hob_amd", {root!r}, {root!r} + "/tests"]
from gpu_util import make_case, run_fhog, with_caches
out = {{}}
for tag, (shape, causal, window) in {cases!r}.items():
    batch, n_q, n_k, d = shape
    x = with_caches(make_case(batch, n_q, n_k, d, torch.bfloat16, seed=45, grad_std=0.1), d ** -0.5, causal, window)
    res = run_fhog(x, d ** -0.5, causal, window=window, return_stats=True)
    out[tag] = [t.cpu() for t in res[:4]] + [t.cpu() for t in res[4]]
    res = run_fhog(x, d ** -0.5, causal, window=window, return_stats=True, schedule="three_sweep", split=False)
    out[tag + "/three_sweep"] = [t.cpu() for t in res[:4]] + [t.cpu() for t in res[4]]
torch.save(out, sys.argv[1])
"""
# small, ragged and masked, d = 128: the 8-wave b and ddO sweeps, the 64-queries-per-wave dd sweep and both workgroup orders on
# launches of a handful of workgroups (each case under the default and under the three-sweep schedule); the last shape is
# one whose passes split their streamed side by default; d64_many: d = 64 with workgroups enough not to split (the one-launch
# form of sweeps 1-3 and the 64-row stage apply)
_TUNE_CASES = {"ragged_causal": ((3, 333, 333, 128), True, None), "window": ((2, 300, 400, 128), "bottom_right", 200),
               "d64_many": ((180, 384, 300, 64), False, None), "split": ((2, 700, 700, 128), True, None)}


def _run_child(tmp_path, tune):
    f = tmp_path / (tune.replace("=", "_").replace(",", "__") or "default")
    env = dict(os.environ, FHOG_TUNE=tune)
    r = subprocess.run([sys.executable, "-c", _CHILD.format(root=str(ROOT), cases=_TUNE_CASES), str(f)], env=env,
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    return torch.load(f, weights_only=True), r.stderr


def test_launch_choices_forced_through_FHOG_TUNE(tmp_path):
    """b8, dd64, order, stage64 and stage1 change which kernel, which workgroup order or how many launches run, never a bit
    of the results; split=0 changes the fp32 summation order of the launches that would split. Unknown keys are reported,
    not obeyed."""
    base, _ = _run_child(tmp_path, "")
    for tune in ("b8=1,dd64=1,order=slice,stage1=1", "b8=0,dd64=0,order=tile,stage64=1"):
        got, err = _run_child(tmp_path, tune)
        assert "FHOG_TUNE" not in err, err
        for tag in base:
            for i, (a, b_) in enumerate(zip(got[tag], base[tag])):
                assert torch.equal(a, b_), (tune, tag, i)
    got, err = _run_child(tmp_path, "split=0,b9=1,order=diagonal,dd64")
    assert "unknown key 'b9'" in err and "not 'diagonal'" in err and "not key=value" in err, err
    for tag in base:          # nothing splits there (the three-sweep runs were made with the minimum workspace)
        if tag != "split":
            for a, b_ in zip(got[tag], base[tag]):
                assert torch.equal(a, b_), tag
    for i, (a, b_) in enumerate(zip(got["split"], base["split"])):
        assert normalised_max_error(a, b_.float()) < (1e-5 if i >= 4 else 8e-3), i   # row statistics in fp32, outputs rounded to bf16
