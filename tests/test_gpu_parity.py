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
    assert _lib.lib().fhog_abi_version() == _lib.ABI_VERSION


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


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", [(2, 256, 256, 64), (70, 128, 200, 32), (130, 128, 96, 64), (40, 300, 300, 64), (3, 100, 40, 64)])
def test_fp32_family_launch_sizes(shape, causal):
    """The fp32-MFMA kernels put one, two or four waves on the same 32 stationary rows depending on how many workgroups
    the launch has (four, each taking every fourth streamed tile, for a problem as small as the first benchmark
    configuration): every regime against the fp64 closed form at the fp32 gate, row statistics included."""
    batch, n_q, n_k, d = shape
    if causal:
        n_k = n_q
    x = make_case(batch, n_q, n_k, d, torch.float32, seed=27)
    scale = d ** -0.5
    x = with_caches(x, scale, causal)
    outs = run_fhog(x, scale, causal, return_stats=True)
    ref = reference_fp64_cpu(x, scale, causal)
    e = errors(outs[:4], [ref[n] for n in NAMES])
    assert max(e.values()) < 1e-4, e
    for got, name in zip(outs[4], ("d", "dd", "b")):
        assert normalised_max_error(got, ref[name]) < 1e-4, name


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mask", [("bottom_right", None, 100, 177), ("bottom_right", 40, 100, 177), (True, 33, 160, 160),
                                  ("bottom_right", 1, 64, 96), ("bottom_right", 500, 31, 31), (True, 7, 256, 256)])
def test_bottom_right_and_sliding_window_masks(mask, dtype):
    """The masks of the reference's specification (fhog/jax_refs/jax_impl.py:110-115), which its Triton path lacks:
    bottom-right alignment for N_Q != N_K and a sliding window; fp32 tensors take the fp32-MFMA kernels, bf16 tensors
    the 16-bit ones."""
    causal, window, n_q, n_k = mask
    d = 64
    x = make_case(2, n_q, n_k, d, dtype, seed=15)
    scale = d ** -0.5
    x = with_caches(x, scale, causal, window)
    outs = run_fhog(x, scale, causal, window=window, return_stats=True)
    ref = reference_fp64_cpu(x, scale, causal, window)
    e = errors(outs[:4], [ref[n] for n in NAMES])
    assert max(e.values()) < TOL[dtype], e
    stat_tol = 1e-4 if dtype == torch.float32 else 5e-3
    for got, name in zip(outs[4], ("d", "dd", "b")):
        assert normalised_max_error(got, ref[name]) < stat_tol, name


@pytest.mark.parametrize("mask", [("bottom_right", None, 200, 456, 128), ("bottom_right", 100, 300, 300, 128),
                                  (True, 2, 160, 160, 64), ("bottom_right", 33, 257, 700, 64), (True, 129, 512, 512, 128),
                                  ("bottom_right", 1000, 96, 1500, 64)])
def test_band_masks_agree_between_the_kernel_families(mask):
    """Longer shapes: both kernel families (the 16-bit one with tile skipping on both edges of the band and partial
    tiles) against the fp64 oracle, and against each other on the same bf16 tensors."""
    causal, window, n_q, n_k, d = mask
    x = make_case(3, n_q, n_k, d, torch.bfloat16, seed=19, grad_std=0.1)
    scale = d ** -0.5
    x = with_caches(x, scale, causal, window)
    fast = run_fhog(x, scale, causal, window=window, impl="bf16", return_stats=True)
    slow = run_fhog(x, scale, causal, window=window, impl="fp32", return_stats=True)
    fused = run_fhog(x, scale, causal, window=window, impl="bf16", fused_stats=True)
    # first against the oracle (fp64 closed form): outputs at the 2e-2 gate, row statistics of every family
    ref = reference_fp64_cpu(x, scale, causal, window)
    for outs, gate in ((fast[:4], 2e-2), (fused, 2e-2), (slow[:4], 2e-2)):
        e = errors(outs, [ref[n] for n in NAMES])
        assert max(e.values()) < gate, e
    for stats in (fast[4], slow[4]):
        for got, name in zip(stats, ("d", "dd", "b")):
            assert normalised_max_error(got, ref[name]) < 1e-2, name
    # then between the two kernel families, far inside the gate
    e = errors(fast[:4], slow[:4])
    assert max(e.values()) < 1.5e-2, e
    for a, b, name in zip(fast[4], slow[4], ("d", "dd", "b")):
        assert normalised_max_error(a, b) < 1e-2, name
    e = errors(fused, slow[:4])
    assert max(e.values()) < 1.5e-2, e


def test_masks_that_hide_nothing_more_give_the_same_bits():
    """Square bottom-right == top-left, and a window as long as the sequence: same results bit for bit."""
    from fhog import BwdBwdPlan
    x = with_caches(make_case(2, 256, 256, 64, torch.bfloat16, seed=16, grad_std=0.1), 0.125, True)
    base = run_fhog(x, 0.125, True)
    for kw in (dict(causal="bottom_right"), dict(causal=True, window=256), dict(causal="bottom_right", window=4096)):
        plan = BwdBwdPlan(x["Q"], x["K"], x["V"], x["O"], x["dO"], x["ddQ"], x["ddK"], x["ddV"], x["L"], 0.125, **kw)
        assert plan.impl == 2
        outs = plan.run()
        torch.cuda.synchronize()
        for a, b in zip(outs, base):
            assert torch.equal(a, b)


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


# ---------------------------------------------------------------- bf16 MFMA family
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", [(2, 128, 128, 64), (3, 256, 256, 128), (2, 128, 384, 64), (9, 384, 128, 128),
                                   (1, 512, 512, 128)])
@pytest.mark.parametrize("fused_stats", [False, True])
def test_bf16_family_small(shape, causal, fused_stats):
    """bf16 MFMA kernels against the fp64 closed form, including the row vectors of passes 0..2, under the
    four-pass schedule and the opt-in fused statistics sweep."""
    batch, n_q, n_k, d = shape
    if causal:
        n_k = n_q
    x = make_case(batch, n_q, n_k, d, torch.bfloat16, seed=5, grad_std=0.1)
    scale = d ** -0.5
    x = with_caches(x, scale, causal)
    outs = run_fhog(x, scale, causal, impl="bf16", return_stats=True, fused_stats=fused_stats)
    ref = reference_fp64_cpu(x, scale, causal)
    e = errors(outs[:4], [ref[n] for n in NAMES])
    assert max(e.values()) < 2e-2, e
    for got, name in zip(outs[4], ("d", "dd", "b")):
        assert normalised_max_error(got, ref[name]) < 1e-2, name
    # the two kernel families agree far inside the gate
    outs32 = run_fhog(x, scale, causal, impl="fp32")
    e2 = errors(outs[:4], outs32)
    assert max(e2.values()) < 1.5e-2, e2


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("d", [64, 128])
def test_bf16_fused_statistics_match_separate_passes(d, causal):
    """The fused dd+b sweep (pass id 5, what the whole chain runs) against passes 1 and 2 run on their own."""
    from fhog import BwdBwdPlan
    x = with_caches(make_case(3, 384, 384, d, torch.bfloat16, seed=12, grad_std=0.1), d ** -0.5, causal)
    plan = BwdBwdPlan(x["Q"], x["K"], x["V"], x["O"], x["dO"], x["ddQ"], x["ddK"], x["ddV"], x["L"], d ** -0.5,
                      causal=causal, impl="bf16")
    plan.ws.fill_(float("nan"))
    for i in (0, 1, 2):
        plan.run(only_pass=i)
    torch.cuda.synchronize()
    separate = plan.ws.clone()
    plan.ws[plan.ws.numel() // 3:].fill_(float("nan"))
    plan.run(only_pass=5)
    torch.cuda.synchronize()
    fused = plan.ws.view(3, -1)
    separate = separate.view(3, -1)
    assert torch.isfinite(fused).all()
    assert torch.equal(fused[0], separate[0])
    assert normalised_max_error(fused[1], separate[1]) < 1e-6      # same sums, same order
    assert normalised_max_error(fused[2], separate[2]) < 1e-3      # dd_i * sum_j P dP taken out of the sum


@pytest.mark.parametrize("fused_stats", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(3, 333, 333, 128), (2, 100, 77, 64)])
def test_bf16_chain_writes_row_sums_d_itself(shape, dtype, fused_stats):
    """The 16-bit chain launches no separate kernel for d = rowsum(O * dO) (fhog/triton_bwdbwd.py:580): its first
    statistics sweep writes it. Checked on a NaN-filled workspace against fp64 and against the stand-alone pass 0."""
    from fhog import BwdBwdPlan
    batch, n_q, n_k, d = shape
    x = with_caches(make_case(batch, n_q, n_k, d, dtype, seed=21, grad_std=0.1), d ** -0.5, False)
    plan = BwdBwdPlan(x["Q"], x["K"], x["V"], x["O"], x["dO"], x["ddQ"], x["ddK"], x["ddV"], x["L"], d ** -0.5,
                      impl="bf16", fused_stats=fused_stats)
    plan.ws.fill_(float("nan"))
    plan.run()
    torch.cuda.synchronize()
    got = plan.ws.view(3, -1)[0].clone()
    want = (x["O"].double() * x["dO"].double()).sum(-1).flatten()
    assert torch.isfinite(plan.ws).all()
    assert normalised_max_error(got, want) < 1e-5
    plan.run(only_pass=0)
    torch.cuda.synchronize()
    assert normalised_max_error(plan.ws.view(3, -1)[0], got) < 1e-5


@pytest.mark.parametrize("fused_stats", [False, True])
@pytest.mark.parametrize("case", [((1, 2048, 2048, 64), False, None, torch.bfloat16), ((1, 2048, 2048, 64), True, None, torch.float16),
                                  ((2, 1000, 1500, 64), "bottom_right", None, torch.bfloat16),
                                  ((1, 1536, 1536, 64), True, 300, torch.bfloat16), ((1, 130, 4100, 64), False, None, torch.bfloat16),
                                  ((1, 2048, 2048, 128), True, None, torch.bfloat16), ((2, 1000, 1500, 128), False, None, torch.float16),
                                  ((1, 1536, 1536, 128), "bottom_right", 700, torch.bfloat16)])
def test_split_streamed_side_matches_the_unsplit_launch(case, fused_stats):
    """Few (batch*head) slices: with the workspace of fhog_bwdbwd_workspace_hint every pass splits its
    streamed side over several workgroups (fp32 partial results, added by a second kernel). Same gate against the
    fp64 oracle as the unsplit launch, row statistics equal up to summation order, outputs within a 16-bit rounding."""
    import os
    from fhog import BwdBwdPlan, _lib
    if "split=0" in os.environ.get("FHOG_TUNE", ""):
        pytest.skip("FHOG_TUNE switches the split launches off")
    (batch, n_q, n_k, d), causal, window, dtype = case
    scale = d ** -0.5
    x = with_caches(make_case(batch, n_q, n_k, d, dtype, seed=23, grad_std=0.1), scale, causal, window)
    plans = [BwdBwdPlan(x["Q"], x["K"], x["V"], x["O"], x["dO"], x["ddQ"], x["ddK"], x["ddV"], x["L"], scale, causal=causal,
                        window=window, impl="bf16", fused_stats=fused_stats, split=sp) for sp in (True, False)]
    assert plans[0].args.ws_bytes > plans[1].args.ws_bytes == _lib.lib().fhog_bwdbwd_workspace_bytes(batch, n_q)
    res = []
    for plan in plans:
        plan.ws_all.fill_(float("nan"))
        outs = [o.clone() for o in plan.run()]
        torch.cuda.synchronize()
        assert torch.isfinite(plan.ws).all()
        res.append((outs, plan.ws.clone().view(3, -1)))
    ref = reference_fp64_cpu(x, scale, causal, window)
    order = ("dq2", "dk2", "dv2", "ddo")   # the plan's output order
    for outs, _ in res:
        e = {n: normalised_max_error(o.view_as(x["Q"] if n in ("dq2", "ddo") else x["K"]), ref[n]) for n, o in zip(order, outs)}
        assert max(e.values()) < 2e-2, e
    for a, b in zip(res[0][1], res[1][1]):
        assert normalised_max_error(a, b) < 1e-5
    for a, b in zip(res[0][0], res[1][0]):
        assert normalised_max_error(a, b) < 1e-2


@pytest.mark.parametrize("seed", range(12))
def test_split_launches_on_random_shapes_against_the_fp32_family(seed):
    """Random ragged lengths, masks, head dims and row strides in the range where launches split (few slices, at least
    16 streamed tiles): the 16-bit kernels with partial results and the fp32-MFMA kernels against the oracle (fp32
    autograd for the outputs, fp64 closed form for the row statistics), then against each other."""
    import random
    rnd = random.Random(1000 + seed)
    d = rnd.choice([64, 128])
    batch = rnd.choice([1, 2, 3])
    n_q, n_k = rnd.randint(520, 2300), rnd.randint(520, 2300)
    kind = rnd.choice(["none", "causal", "bottom_right", "band"])
    causal, window = False, None
    if kind == "causal":
        causal, n_k = True, n_q
    elif kind in ("bottom_right", "band"):
        causal, n_k = "bottom_right", max(n_k, n_q)
        if kind == "band":
            window = rnd.randint(40, 900)
    pad = rnd.choice([0, 8, 64])   # row stride d + pad
    dtype = rnd.choice([torch.bfloat16, torch.float16])
    x = make_case(batch, n_q, n_k, d, dtype, seed=200 + seed, grad_std=0.1)
    if pad:
        for name in list(x):
            t = x[name]
            wide = torch.zeros(t.shape[0], t.shape[1], d + pad, dtype=t.dtype, device=t.device)
            wide[..., :d] = t
            x[name] = wide[..., :d]
    scale = d ** -0.5
    x = with_caches(x, scale, causal, window)
    if pad:
        wide = torch.zeros(batch, n_q, d + pad, dtype=x["O"].dtype, device="cuda")
        wide[..., :d] = x["O"]
        x["O"] = wide[..., :d]
    fast = run_fhog(x, scale, causal, window=window, impl="bf16", return_stats=True)
    slow = run_fhog(x, scale, causal, window=window, impl="fp32", return_stats=True)
    what = (d, batch, n_q, n_k, kind, window, pad, dtype)
    # the oracle first: fp32 autograd double-backward on the GPU for the outputs of every slice, the fp64 closed form
    # on the CPU for the row statistics of slice 0
    ref = reference_fp32_gpu(x, scale, causal, window=window)
    for outs in (fast[:4], slow[:4]):
        e = errors(outs, ref)
        assert max(e.values()) < 2e-2, (e, what)
    ref0 = reference_fp64_cpu(x, scale, causal, window, heads=[0])
    for stats in (fast[4], slow[4]):
        for got, name in zip(stats, ("d", "dd", "b")):
            assert normalised_max_error(got[:1], ref0[name]) < 1e-2, (name, what)
    e = errors(fast[:4], slow[:4])
    assert max(e.values()) < 1.5e-2, (e, what)
    for a, b, name in zip(fast[4], slow[4], ("d", "dd", "b")):
        assert normalised_max_error(a, b) < 1e-2, name


@pytest.mark.parametrize("fused_stats", [False, True])
@pytest.mark.parametrize("case", [(130, 1000, 1000, "causal", None, torch.bfloat16), (128, 1025, 700, "none", None, torch.float16),
                                  (171, 770, 1100, "bottom_right", 300, torch.bfloat16), (64, 2050, 520, "none", None, torch.bfloat16)])
def test_many_slices_d128_statistics_in_256_row_workgroups(case, fused_stats):
    """At d = 128, launches of the b and dd+b sweeps with at least 512 workgroups of 256 query rows use those (8 waves)
    instead of 128-row workgroups: ragged lengths (last workgroup partly or, for its upper waves, wholly past the end),
    masks and dtypes against the oracle on sampled slices and against the fp32-MFMA kernels, statistics included."""
    batch, n_q, n_k, kind, window, dtype = case
    causal = {"none": False, "causal": True, "bottom_right": "bottom_right"}[kind]
    x = make_case(batch, n_q, n_k, 128, dtype, seed=77, grad_std=0.1)
    scale = 128 ** -0.5
    x = with_caches(x, scale, causal, window)
    fast = run_fhog(x, scale, causal, window=window, impl="bf16", fused_stats=fused_stats, return_stats=True)
    slow = run_fhog(x, scale, causal, window=window, impl="fp32", return_stats=True)
    # the oracle on four sampled slices, the last one included (its last workgroup is the ragged one): fp32 autograd
    # for the outputs, fp64 closed form for the row statistics
    heads = [0, batch // 3, (2 * batch) // 3, batch - 1]
    ref = reference_fp32_gpu(x, scale, causal, heads=heads, window=window)
    ref64 = reference_fp64_cpu(x, scale, causal, window, heads=heads[-2:])
    for res in (fast, slow):
        e = errors([o[heads] for o in res[:4]], ref)
        assert max(e.values()) < 2e-2, e
        for got, name in zip(res[4], ("d", "dd", "b")):
            assert normalised_max_error(got[heads[-2:]], ref64[name]) < 1e-2, name
    e = errors(fast[:4], slow[:4])
    assert max(e.values()) < 1.5e-2, e
    for a, b, name in zip(fast[4], slow[4], ("d", "dd", "b")):
        assert normalised_max_error(a, b) < 1e-2, name


@pytest.mark.parametrize("case", [(520, 1000, 1000, "causal", None, torch.bfloat16), (512, 1021, 515, "none", None, torch.float16),
                                  (700, 770, 1100, "bottom_right", 300, torch.bfloat16)])
def test_many_rows_d128_dd_sweep_with_64_queries_per_wave(case):
    """At d = 128 a dd sweep of at least 2048 workgroups of 256 query rows runs 64 queries per wave (two 32-query blocks,
    either of which a mask can leave out of a step): ragged ends, masks and dtypes; d and dd against the fp64 closed form
    on sampled slices and against the fp32-MFMA kernels on all of them, outputs against fp32 autograd on sampled slices."""
    batch, n_q, n_k, kind, window, dtype = case
    causal = {"none": False, "causal": True, "bottom_right": "bottom_right"}[kind]
    x = make_case(batch, n_q, n_k, 128, dtype, seed=78, grad_std=0.1)
    scale = 128 ** -0.5
    x = with_caches(x, scale, causal, window)
    fast = run_fhog(x, scale, causal, window=window, impl="bf16", return_stats=True)
    slow = run_fhog(x, scale, causal, window=window, impl="fp32", return_stats=True)
    heads = [0, batch // 2, batch - 1]
    ref = reference_fp32_gpu(x, scale, causal, heads=heads, window=window)
    ref64 = reference_fp64_cpu(x, scale, causal, window, heads=heads[-2:])
    e = errors([o[heads] for o in fast[:4]], ref)
    assert max(e.values()) < 2e-2, e
    for got, name in zip(fast[4], ("d", "dd", "b")):
        assert normalised_max_error(got[heads[-2:]], ref64[name]) < 1e-2, name
    for a, b, name in zip(fast[4], slow[4], ("d", "dd", "b")):
        assert normalised_max_error(a, b) < 1e-2, name


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("impl", ["bf16", "fp32"])
@pytest.mark.parametrize("shape", [(2, 256, 128, 64), (3, 384, 384, 128)])
def test_fp16_tensors_both_families(shape, impl, causal):
    """fp16 tensors (the dtype of the reference's benchmark sweep, fhog/benchhhh.py:15-26) through the 16-bit MFMA
    kernels (products in fp16) and through the fp32-MFMA kernels."""
    batch, n_q, n_k, d = shape
    if causal:
        n_k = n_q
    x = make_case(batch, n_q, n_k, d, torch.float16, seed=13, grad_std=0.1)
    scale = d ** -0.5
    x = with_caches(x, scale, causal)
    outs = run_fhog(x, scale, causal, impl=impl, return_stats=True)
    ref = reference_fp64_cpu(x, scale, causal)
    e = errors(outs[:4], [ref[n] for n in NAMES])
    assert all(o.dtype == torch.float16 for o in outs[:4])
    assert max(e.values()) < (5e-3 if impl == "bf16" else 1e-3), e   # fp16 carries 3 more mantissa bits than bf16
    for got, name in zip(outs[4], ("d", "dd", "b")):
        assert normalised_max_error(got, ref[name]) < 2e-3, name


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_reference_sweep_regime_one_head_8192(dtype):
    """The first point of the reference's benchmark sweep (fhog/benchhhh.py:15-27,93-110: one head, d = 64, fp16,
    non-causal, N = 8192), where every pass splits its streamed side: against the fp32 autograd double-backward, with L
    and O from a real forward (the reference's script draws them at random: timing only). fp16 keeps three more
    mantissa bits than bf16 but P = exp(S - L) ~ 1/N already sits near the bottom of its normal range here."""
    from fhog import BwdBwdPlan
    n, d = 8192, 64
    scale = d ** -0.5
    x = with_caches(make_case(1, n, n, d, dtype, seed=41, grad_std=0.1), scale, False)
    plan = BwdBwdPlan(x["Q"], x["K"], x["V"], x["O"], x["dO"], x["ddQ"], x["ddK"], x["ddV"], x["L"], scale, impl="bf16")
    assert plan.args.ws_bytes > 3 * n * 4          # room for partial results: the passes split
    outs = run_fhog(x, scale, False, return_stats=True)
    ref = reference_fp32_gpu(x, scale, False)
    e = errors(outs[:4], ref)
    assert max(e.values()) < 2e-2, e
    ref64 = reference_fp64_cpu({k_: v_[:, :256] if k_ in ("Q", "dO", "ddQ", "O", "L") else v_ for k_, v_ in x.items()}, scale, False)
    for got, name in zip(outs[4], ("d", "dd", "b")):   # row statistics of the first 256 queries against fp64
        assert normalised_max_error(got[:, :256], ref64[name]) < 1e-2, name


def test_single_head_spreads_over_the_chip():
    """batch = 1 (the reference's sweep shape): tiles of the one slice are dealt to all XCDs; results unchanged."""
    x = with_caches(make_case(1, 1024, 1024, 64, torch.bfloat16, seed=14, grad_std=0.1), 0.125, True)
    outs = run_fhog(x, 0.125, True, impl="bf16")
    ref = reference_fp64_cpu(x, 0.125, True)
    e = errors(outs, [ref[n] for n in NAMES])
    assert max(e.values()) < 2e-2, e


@pytest.mark.parametrize("fused_stats", [False, True])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", [(3, 100, 77, 64), (2, 33, 129, 128), (2, 333, 333, 128), (1, 1, 1, 64), (2, 31, 31, 128),
                                   (2, 129, 257, 64), (1, 1000, 1000, 128), (5, 160, 96, 64)])
def test_bf16_family_ragged_lengths(shape, causal, fused_stats):
    """Sequence lengths that are no multiple of the 128-row workgroup tile or of the 32-row stage: rows past the end
    are computed on copies of the last row and masked / not stored."""
    batch, n_q, n_k, d = shape
    if causal:
        n_k = n_q
    x = make_case(batch, n_q, n_k, d, torch.bfloat16, seed=18, grad_std=0.1)
    scale = d ** -0.5
    x = with_caches(x, scale, causal)
    canary = 7.0
    outs = run_fhog(x, scale, causal, impl="bf16", return_stats=True, fused_stats=fused_stats)
    ref = reference_fp64_cpu(x, scale, causal)
    e = errors(outs[:4], [ref[n] for n in NAMES])
    assert max(e.values()) < 2e-2, e
    for got, name in zip(outs[4], ("d", "dd", "b")):
        assert normalised_max_error(got, ref[name]) < 1e-2, name
    # nothing is written past the end of a tensor: outputs are views into larger canary-filled buffers
    from fhog import BwdBwdPlan
    plan = BwdBwdPlan(x["Q"], x["K"], x["V"], x["O"], x["dO"], x["ddQ"], x["ddK"], x["ddV"], x["L"], scale, causal=causal,
                      impl="bf16", fused_stats=fused_stats)
    big = [torch.full((t.numel() + 4096,), canary, dtype=t.dtype, device=t.device) for t in plan.outs]
    ws_floats = (plan.args.ws_bytes + 3) // 4   # d | dd | b and, for a split launch, the partial results
    assert ws_floats <= plan.ws_all.numel()
    ws_big = torch.full((ws_floats + 1024,), canary, dtype=torch.float32, device="cuda")
    for name, buf, t in zip(("dq2", "dk2", "dv2", "ddo"), big, plan.outs):
        setattr(plan.args, name, buf.data_ptr())
    plan.args.ws = ws_big.data_ptr()
    plan.run()
    torch.cuda.synchronize()
    for buf, t, o in zip(big, plan.outs, outs[:4]):
        assert torch.equal(buf[:t.numel()].view(t.shape), o.reshape(t.shape))
        assert (buf[t.numel():] == canary).all()
    assert (ws_big[ws_floats:] == canary).all()


def test_bf16_auto_dispatch():
    from fhog import BwdBwdPlan
    x = with_caches(make_case(2, 256, 256, 64, torch.bfloat16, seed=6), 0.125, False)
    plan = BwdBwdPlan(x["Q"], x["K"], x["V"], x["O"], x["dO"], x["ddQ"], x["ddK"], x["ddV"], x["L"], 0.125)
    assert plan.impl == 2
    y = with_caches(make_case(2, 200, 256, 64, torch.bfloat16, seed=6), 0.125, False)
    plan = BwdBwdPlan(y["Q"], y["K"], y["V"], y["O"], y["dO"], y["ddQ"], y["ddK"], y["ddV"], y["L"], 0.125)
    assert plan.impl == 2          # ragged lengths stay on the 16-bit kernels
    z = with_caches(make_case(2, 128, 128, 32, torch.bfloat16, seed=6), 32 ** -0.5, False)
    plan = BwdBwdPlan(z["Q"], z["K"], z["V"], z["O"], z["dO"], z["ddQ"], z["ddK"], z["ddV"], z["L"], 32 ** -0.5)
    assert plan.impl == 1          # d = 32 is served by the fp32-MFMA kernels


def _full_config(name, seed, heads=None, fused_stats=False):
    from fhog.workloads import WORKLOADS, make_inputs
    w = WORKLOADS[name]
    x = make_inputs(w, seed, device="cuda:0")
    x = {n: t.flatten(0, 1) for n, t in x.items()}
    x = with_caches(x, w.scale, w.causal)
    outs = run_fhog(x, w.scale, w.causal, fused_stats=fused_stats)
    hs = list(range(w.batch)) if heads is None else heads
    worst = {}
    for h0 in range(0, len(hs), 4):
        sel = hs[h0:h0 + 4]
        ref = reference_fp32_gpu(x, w.scale, w.causal, heads=sel)
        e = errors([o[sel] for o in outs], ref)
        worst = {n: max(worst.get(n, 0.0), v) for n, v in e.items()}
    for o in outs:
        assert torch.isfinite(o.float()).all()
    return w, worst


@pytest.mark.parametrize("seed", [0, 1])
def test_cfg1_bf16_noncausal_2048_d64(seed):
    w, e = _full_config("cfg1_bf16_nc_2048_d64", seed)
    assert max(e.values()) < 2e-2, e


@pytest.mark.parametrize("seed", [0, 1])
def test_cfg2_bf16_causal_4096_d128_headline(seed):
    w, e = _full_config("cfg2_bf16_causal_4096_d128", seed)
    assert max(e.values()) < 2e-2, e


@pytest.mark.parametrize("name,heads", [("cfg1_bf16_nc_2048_d64", None), ("cfg2_bf16_causal_4096_d128", None),
                                        ("cfg3_bf16_causal_16384_d128", [3, 30]), ("cfg4_bf16_cross_1024x8192_d64", None)])
def test_full_size_configs_fused_statistics_schedule(name, heads):
    """The opt-in schedule (dd and b from one sweep) on every 16-bit benchmark configuration at full size."""
    w, e = _full_config(name, 2, heads=heads, fused_stats=True)
    assert max(e.values()) < 2e-2, e


def test_cfg3_bf16_causal_16384_d128_sampled_heads():
    """configs[3]: all 32 heads run through the HIP path; 4 sampled heads are compared with the fp32 reference."""
    w, e = _full_config("cfg3_bf16_causal_16384_d128", 0, heads=[0, 9, 18, 27])
    assert max(e.values()) < 2e-2, e


def test_cfg4_bf16_cross_attention_scaled_keys():
    w, e = _full_config("cfg4_bf16_cross_1024x8192_d64", 0)
    assert max(e.values()) < 2e-2, e


# ---------------------------------------------------------------- size-independent properties at full size
def test_headline_properties_linearity_zero_and_sdpa_case():
    from fhog.workloads import WORKLOADS, make_inputs
    w = WORKLOADS["cfg2_bf16_causal_4096_d128"]
    x = {n: t.flatten(0, 1)[:8] for n, t in make_inputs(w, 2, device="cuda:0").items()}
    x = with_caches(x, w.scale, True)
    # zero cotangents -> exact zeros
    z = dict(x, ddQ=torch.zeros_like(x["ddQ"]), ddK=torch.zeros_like(x["ddK"]), ddV=torch.zeros_like(x["ddV"]))
    for o in run_fhog(z, w.scale, True):
        assert o.float().abs().max().item() == 0.0
    # linearity in the cotangents: f(2 t) == 2 f(t) exactly (powers of two commute with every rounding)
    base = run_fhog(x, w.scale, True)
    dbl = run_fhog(dict(x, ddQ=x["ddQ"] * 2, ddK=x["ddK"] * 2, ddV=x["ddV"] * 2), w.scale, True)
    for a, b in zip(base, dbl):
        torch.testing.assert_close(b.float(), a.float() * 2, rtol=0, atol=0)
    # ddQ = ddK = 0: dV' = 0, ddO = attention(Q, K, ddV), (dQ', dK') = first-order grads with V := ddV
    y = dict(x, ddQ=torch.zeros_like(x["ddQ"]), ddK=torch.zeros_like(x["ddK"]))
    dq2, dk2, dv2, ddo = run_fhog(y, w.scale, True)
    assert dv2.float().abs().max().item() == 0.0
    q = x["Q"].float().requires_grad_(True)
    k = x["K"].float().requires_grad_(True)
    out = torch.nn.functional.scaled_dot_product_attention(q, k, x["ddV"].float(), is_causal=True, scale=w.scale)
    gq, gk = torch.autograd.grad(out, (q, k), x["dO"].float())
    assert normalised_max_error(ddo, out) < 2e-2
    assert normalised_max_error(dq2, gq) < 2e-2
    assert normalised_max_error(dk2, gk) < 2e-2
    # causal row 0 sees only key 0: dQ'[0] = 0, ddO[0] = ddV[0]
    assert base[0][:, 0].float().abs().max().item() < 1e-6
    torch.testing.assert_close(base[3][:, 0].float(), x["ddV"][:, 0].float(), rtol=1e-2, atol=1e-3)


@pytest.mark.parametrize("name", ["cfg2_bf16_causal_4096_d128", "cfg4_bf16_cross_1024x8192_d64", "cfg3_bf16_causal_16384_d128"])
def test_full_size_statistic_b_is_the_row_dot_of_dO_and_ddO(name):
    """b_i = dO_i . ddO_i - d_i dd_i holds for the exact quantities, whatever the size: the row statistic the second sweep
    leaves in the workspace against an output of the third sweep, at the full benchmark sizes (every slice, every row)."""
    from fhog.workloads import WORKLOADS, make_inputs
    w = WORKLOADS[name]
    x = {n: t.flatten(0, 1) for n, t in make_inputs(w, 3, device="cuda:0").items()}
    x = with_caches(x, w.scale, w.causal)
    dq2, dk2, dv2, ddo, (d, dd, b) = run_fhog(x, w.scale, w.causal, return_stats=True)
    rowdot = torch.zeros_like(b)
    for h0 in range(0, ddo.shape[0], 8):   # in slices: the fp32 copies of a whole tensor are large at N = 16384
        rowdot[h0:h0 + 8] = (x["dO"][h0:h0 + 8].float() * ddo[h0:h0 + 8].float()).sum(-1)
    want = rowdot - d * dd
    # ddO is rounded to bf16 (2^-9 relative) before the row dot: the bound scales with sum_c |dO ddO| of the row
    assert normalised_max_error(b, want) < 1e-2, normalised_max_error(b, want)


def test_peak_memory_is_linear_in_n():
    """Workspace + outputs only: 4 output tensors and 3 fp32 row vectors, nothing of size N_Q x N_K. The larger
    workspace for split launches adds partial results of fewer than 2 * 131072 * d floats, whatever N (the number of
    splits falls as the number of workgroups grows)."""
    import fhog
    sizes = {}
    for n in (2048, 8192):
        x = with_caches(make_case(4, n, n, 128, torch.bfloat16, seed=7, grad_std=0.1), 128 ** -0.5, True)
        for split in (False, True):
            torch.cuda.synchronize()
            torch.cuda.reset_peak_memory_stats()
            before = torch.cuda.memory_allocated()
            outs = run_fhog(x, 128 ** -0.5, True, split=split)
            torch.cuda.synchronize()
            used = torch.cuda.max_memory_allocated() - before
            expect = 4 * 4 * n * 128 * 2 + 3 * 4 * n * 4
            if split:
                assert used <= expect * 1.05 + (1 << 20) + 2 * 131072 * 128 * 4, (n, used, expect)
            else:
                sizes[n] = used
                assert used <= expect * 1.05 + (1 << 20), (n, used, expect)
            del outs
        del x
    assert sizes[8192] <= 4.2 * sizes[2048]


@pytest.mark.parametrize("batch,n", [(4, 512), (128, 1024)])
def test_hip_graph_capture_and_replay(batch, n):
    """The library only enqueues kernels on the caller's stream: a captured call replays to the same bits, also after
    the inputs changed in place and with eager work in between. The small case runs split launches with their combine
    kernels, the large one the 256-row statistics workgroups."""
    from fhog import BwdBwdPlan
    x = with_caches(make_case(batch, n, n, 128, torch.bfloat16, seed=17, grad_std=0.1), 128 ** -0.5, True)
    plan = BwdBwdPlan(x["Q"], x["K"], x["V"], x["O"], x["dO"], x["ddQ"], x["ddK"], x["ddV"], x["L"], 128 ** -0.5, causal=True)
    eager = [t.clone() for t in plan.run()]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        plan.run()                       # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        plan.run()
    for rep in range(3):
        for o in plan.outs:
            o.fill_(float("nan"))
        plan.ws.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip(plan.outs, eager):
            assert torch.equal(a, b), rep
        _ = (x["Q"].float() @ x["K"].float().transpose(-1, -2)).sum().item()   # unrelated eager work between replays
    # the graph reads the plan's input buffers: new values in place, same graph
    q_in = plan.keep[7]                  # ddV as the plan holds it
    q_in.mul_(2.0)
    graph.replay()
    torch.cuda.synchronize()
    fresh = BwdBwdPlan(x["Q"], x["K"], x["V"], x["O"], x["dO"], x["ddQ"], x["ddK"], q_in, x["L"], 128 ** -0.5, causal=True)
    want = fresh.run()
    torch.cuda.synchronize()
    for a, b in zip(plan.outs, want):
        assert torch.equal(a, b)


def test_mfma_rate_probe_runs():
    """The measurement aid of bench.py: launches, reports the FLOPs it issued, leaves finite sums."""
    import ctypes
    from fhog import _lib
    L = _lib.lib()
    out = torch.full((8 * 512,), float("nan"), device="cuda:0")
    flops = ctypes.c_double()
    # zeros; random; random with LDS operand reads and / or VALU side work in the stream; + 8: one wave per SIMD
    for mode in list(range(6)) + list(range(8, 14)):
        waves = 4 if mode & 8 else 8
        out.fill_(float("nan"))
        _lib.check(L.fhog_probe_mfma_rate(out.data_ptr(), 8, 100, mode, ctypes.byref(flops),
                                          ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
        torch.cuda.synchronize()
        assert flops.value == 8 * waves * 100 * 32 * 32768
        written = out.view(8, 512)[:, :64 * waves]
        assert torch.isfinite(written).all()
        assert mode & 7 == 0 or written.abs().max() > 1e-20   # random operands leave non-zero sums


def test_autograd_chain_with_a_sliding_window():
    """attention(..., 'bottom_right', window) twice differentiated against torch autograd on the same mask."""
    import fhog
    g = torch.Generator().manual_seed(9)
    mk = lambda *s: torch.randn(*s, generator=g).cuda()
    q, k, v, w = mk(2, 96, 64), mk(2, 160, 64), mk(2, 160, 64), mk(2, 96, 64)
    qi = torch.arange(96, device="cuda")[:, None] + 64
    kj = torch.arange(160, device="cuda")[None, :]
    visible = (kj <= qi) & (qi - kj < 50)

    def penalty(attn):
        qq, kk, vv = (t.clone().requires_grad_(True) for t in (q, k, v))
        out = attn(qq, kk, vv)
        gq, gk, gv = torch.autograd.grad((out * w).sum(), (qq, kk, vv), create_graph=True)
        loss = gq.square().sum() + (gk * gv).sum()
        return torch.autograd.grad(loss, (qq, kk, vv))

    ours = penalty(lambda a, b, c: fhog.attention(a, b, c, "bottom_right", 50))
    ref = penalty(lambda a, b, c: torch.nn.functional.scaled_dot_product_attention(a, b, c, attn_mask=visible))
    for a, b in zip(ours, ref):
        assert normalised_max_error(a, b) < 1e-4


# ---------------------------------------------------------------- autograd chain
@pytest.mark.parametrize("causal", [False, True])
def test_autograd_chain_reaches_hip_double_backward(causal):
    """create_graph=True through FlashAttention -> AttnBwd -> flash_bwdbwd (the wiring the reference only
    sketches, fhog/triton_bwdbwd.py:538-554) against plain torch attention."""
    import fhog
    g = torch.Generator().manual_seed(8)
    mk = lambda *s: torch.randn(*s, generator=g).cuda()
    q, k, v = mk(2, 128, 64), mk(2, 128, 64), mk(2, 128, 64)
    w = mk(2, 128, 64)

    def penalty(attn):
        qq, kk, vv = (t.clone().requires_grad_(True) for t in (q, k, v))
        out = attn(qq, kk, vv)
        gq, gk, gv = torch.autograd.grad((out * w).sum(), (qq, kk, vv), create_graph=True)
        loss = gq.square().sum() + (gk * gv).sum()
        return torch.autograd.grad(loss, (qq, kk, vv))

    ours = penalty(lambda a, b, c: fhog.attention(a, b, c, causal))
    ref = penalty(lambda a, b, c: torch.nn.functional.scaled_dot_product_attention(a, b, c, is_causal=causal))
    for a, b in zip(ours, ref):
        assert normalised_max_error(a, b) < 1e-4
