"""GPU tier: the opt-in schedules that take ddO out of the third sweep (FHOG_SCHEDULE_DDO_EARLY, FHOG_SCHEDULE_THREE_SWEEP).

The reference forms ddO next to dQ2 in its third sweep (fhog/triton_bwdbwd.py:257-313) and b in a sweep of five
first-level products (:217-251). Here the second sweep produces ddO and takes b from it, b_i = dO_i . ddO_i - d_i dd_i
(pinned for the exact quantities in tests/test_oracle.py::test_row_identities), and the third produces dQ2 alone. Same
gates as the default schedule: outputs within 2e-2 of the fp64 closed form (normalised max error), row statistics
d, dd, b read back from the workspace.
"""
import ctypes

import pytest
import torch

from gpu_util import (NAMES, errors, make_case, normalised_max_error, reference_fp32_gpu, reference_fp64_cpu, require_gpu,
                      run_fhog, with_caches)

pytestmark = pytest.mark.gpu
SCHEDULES = ["ddo_early", "three_sweep"]


@pytest.fixture(scope="module", autouse=True)
def _dev():
    return require_gpu()


def _check(x, scale, causal, schedule, window=None, tol=2e-2, stat_tol=1e-2):
    outs = run_fhog(x, scale, causal, schedule=schedule, window=window, return_stats=True)
    ref = reference_fp64_cpu(x, scale, causal, window=window)
    e = errors(outs[:4], [ref[n] for n in NAMES])
    assert max(e.values()) < tol, (schedule, e)
    for got, name in zip(outs[4], ("d", "dd", "b")):
        err = normalised_max_error(got, ref[name])
        assert err < stat_tol, (schedule, name, err)
    return outs


@pytest.mark.parametrize("schedule", SCHEDULES)
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", [(2, 128, 128, 64), (3, 256, 256, 128), (2, 128, 384, 64), (9, 384, 128, 128),
                                   (3, 100, 77, 64), (2, 33, 129, 128), (2, 333, 333, 128), (1, 1, 1, 64), (2, 31, 31, 128)])
def test_schedules_small_and_ragged(shape, causal, schedule):
    batch, n_q, n_k, d = shape
    if causal and n_q != n_k:
        causal = "bottom_right" if n_k > n_q else False
    x = with_caches(make_case(batch, n_q, n_k, d, torch.bfloat16, seed=51, grad_std=0.1), d ** -0.5, causal)
    _check(x, d ** -0.5, causal, schedule)


@pytest.mark.parametrize("schedule", SCHEDULES)
@pytest.mark.parametrize("mask", [("bottom_right", None, 200, 456, 128), ("bottom_right", 100, 300, 300, 128), (True, 65, 257, 257, 64),
                                  ("bottom_right", 1, 96, 160, 64)])
def test_schedules_band_masks(mask, schedule):
    causal, window, n_q, n_k, d = mask
    x = with_caches(make_case(3, n_q, n_k, d, torch.bfloat16, seed=52, grad_std=0.1), d ** -0.5, causal, window)
    _check(x, d ** -0.5, causal, schedule, window=window)


@pytest.mark.parametrize("schedule", SCHEDULES)
@pytest.mark.parametrize("d", [64, 128])
def test_schedules_fp16_and_unit_cotangents(d, schedule):
    """fp16 tensors (the reference's sweep dtype), and cotangents of the size of the inputs (the fixture's regime)."""
    x = with_caches(make_case(2, 320, 200, d, torch.float16, seed=53, grad_std=1.0), d ** -0.5, False)
    _check(x, d ** -0.5, False, schedule)


@pytest.mark.parametrize("schedule", SCHEDULES)
@pytest.mark.parametrize("split", [True, False])
def test_schedules_on_a_launch_too_small_to_fill_the_gpu(schedule, split):
    """One head of 4096 tokens is 32 workgroups: with the larger workspace the library runs the nearest schedule whose
    passes can split their streamed side, with the minimum workspace the schedule itself, unsplit. Same gates either way."""
    x = with_caches(make_case(1, 4096, 4096, 64, torch.bfloat16, seed=58, grad_std=0.1), 0.125, False)
    outs = run_fhog(x, 0.125, False, schedule=schedule, split=split, return_stats=True)
    ref = reference_fp32_gpu(x, 0.125, False)
    e = errors(outs[:4], ref)
    assert max(e.values()) < 2e-2, e
    d, dd, b = outs[4]
    rowdot = (x["dO"].float() * outs[3].float()).sum(-1)
    assert normalised_max_error(b, rowdot - d * dd) < 1e-2


@pytest.mark.parametrize("schedule", SCHEDULES)
def test_schedules_against_the_default_one(schedule):
    """Same tensors through the reference schedule and an opt-in one: dK2, dV2 and dQ2 depend on the row statistics
    (dd, b) only, so they move by no more than the statistics' own rounding; ddO is rounded once in both."""
    x = with_caches(make_case(5, 640, 640, 128, torch.bfloat16, seed=54, grad_std=0.1), 128 ** -0.5, True)
    base = run_fhog(x, 128 ** -0.5, True, return_stats=True)
    alt = run_fhog(x, 128 ** -0.5, True, schedule=schedule, return_stats=True)
    for name, a, b_ in zip(NAMES, alt[:4], base[:4]):
        assert normalised_max_error(a, b_.float()) < 8e-3, name
    for name, a, b_ in zip(("d", "dd", "b"), alt[4], base[4]):
        assert normalised_max_error(a, b_) < 4e-3, name


@pytest.mark.parametrize("schedule", SCHEDULES)
def test_schedules_fp32_tensors_run_the_reference_schedule(schedule):
    x = with_caches(make_case(2, 96, 160, 64, torch.float32, seed=55), 0.125, False)
    base = run_fhog(x, 0.125, False)
    alt = run_fhog(x, 0.125, False, schedule=schedule)
    for a, b_ in zip(alt, base):
        assert torch.equal(a, b_)


def test_new_passes_exist_in_the_16_bit_family_only():
    from fhog import BwdBwdPlan, _lib
    x = with_caches(make_case(2, 128, 128, 64, torch.bfloat16, seed=56), 0.125, False)
    plan = BwdBwdPlan(x["Q"], x["K"], x["V"], x["O"], x["dO"], x["ddQ"], x["ddK"], x["ddV"], x["L"], 0.125, impl="fp32")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for pass_id in (_lib.PASS_B_DDO, _lib.PASS_DQ, _lib.PASS_DD_B_DDO, _lib.PASS_STAGE1):
        assert plan.lib.fhog_bwdbwd_pass(ctypes.byref(plan.args), pass_id, stream) == -7
        assert "16-bit" in plan.lib.fhog_last_error().decode()
    assert plan.lib.fhog_bwdbwd_pass(ctypes.byref(plan.args), 10, stream) == -7
    # the one-launch form of sweeps 1-3 exists where the three sweeps share a workgroup shape: d = 64
    y = with_caches(make_case(2, 128, 128, 128, torch.bfloat16, seed=56), 128 ** -0.5, False)
    plan = BwdBwdPlan(y["Q"], y["K"], y["V"], y["O"], y["dO"], y["ddQ"], y["ddK"], y["ddV"], y["L"], 128 ** -0.5)
    assert plan.lib.fhog_bwdbwd_pass(ctypes.byref(plan.args), _lib.PASS_STAGE1, stream) == -7
    assert "d = 64" in plan.lib.fhog_last_error().decode()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("case", [(5, 640, 640, True, None), (3, 300, 777, "bottom_right", 200), (70, 256, 1000, False, None),
                                  (2, 33, 129, False, None)])
def test_three_sweeps_in_one_launch_equal_the_three_launches(case, dtype):
    """FHOG_PASS_STAGE1, the reference's own arrangement (bwdbwd_kernel_stage1 runs its three sweeps inside one kernel,
    fhog/triton_bwdbwd.py:185-313): same sweeps with dd and b handed over in registers, so d, dd, b, dQ2 and ddO come out
    bit for bit as from passes 1, 2, 3 launched one by one."""
    from fhog import BwdBwdPlan, _lib
    batch, n_q, n_k, causal, window = case
    x = with_caches(make_case(batch, n_q, n_k, 64, dtype, seed=61, grad_std=0.1), 0.125, causal, window)
    plans = [BwdBwdPlan(x["Q"], x["K"], x["V"], x["O"], x["dO"], x["ddQ"], x["ddK"], x["ddV"], x["L"], 0.125, causal=causal,
                        window=window, split=False) for _ in range(2)]
    for p in plans:
        for t in p.outs:
            t.fill_(float("nan"))
        p.ws.fill_(float("nan"))
    for pass_id in (_lib.PASS_DD, _lib.PASS_B, _lib.PASS_DQ_DDO):
        plans[0].run(only_pass=pass_id)
    plans[1].run(only_pass=_lib.PASS_STAGE1)
    torch.cuda.synchronize()
    assert torch.equal(plans[0].ws, plans[1].ws) and torch.isfinite(plans[0].ws).all()
    for a, b in ((plans[0].outs[0], plans[1].outs[0]), (plans[0].outs[3], plans[1].outs[3])):   # dQ2, ddO
        assert torch.equal(a, b) and torch.isfinite(a.float()).all()


def _full_config(name, seed, schedule, heads=None):
    from fhog.workloads import WORKLOADS, make_inputs
    w = WORKLOADS[name]
    x = {n: t.flatten(0, 1) for n, t in make_inputs(w, seed, device="cuda:0").items()}
    x = with_caches(x, w.scale, w.causal)
    outs = run_fhog(x, w.scale, w.causal, schedule=schedule, return_stats=True)
    hs = list(range(w.batch)) if heads is None else heads
    worst = {}
    for h0 in range(0, len(hs), 4):
        sel = hs[h0:h0 + 4]
        ref = reference_fp32_gpu(x, w.scale, w.causal, heads=sel)
        e = errors([o[sel] for o in outs[:4]], ref)
        worst = {n: max(worst.get(n, 0.0), v) for n, v in e.items()}
    for o in outs[:4]:
        assert torch.isfinite(o.float()).all()
    # b against the identity it is taken from, with the device's own ddO (rounded to 16 bits), on every row
    d, dd, b = outs[4]
    rowdot = torch.zeros_like(b)
    for h0 in range(0, w.batch, 8):
        rowdot[h0:h0 + 8] = (x["dO"][h0:h0 + 8].float() * outs[3][h0:h0 + 8].float()).sum(-1)
    worst["b_identity"] = normalised_max_error(b, rowdot - d * dd)
    return worst


@pytest.mark.parametrize("schedule", SCHEDULES)
@pytest.mark.parametrize("name,heads", [("cfg1_bf16_nc_2048_d64", None), ("cfg2_bf16_causal_4096_d128", None),
                                        ("cfg3_bf16_causal_16384_d128", [5, 26]), ("cfg4_bf16_cross_1024x8192_d64", None)])
def test_schedules_full_size_configs(name, heads, schedule):
    e = _full_config(name, 4, schedule, heads=heads)
    print(f"{name} {schedule}: {e}")
    assert max(e.values()) < 2e-2, e


@pytest.mark.parametrize("schedule", SCHEDULES)
def test_schedules_through_the_autograd_chain(schedule):
    """`fhog.attention(..., schedule=...)`: create_graph=True through FlashAttention -> AttnBwd -> flash_bwdbwd with an
    opt-in schedule, bf16 tensors, against plain torch attention in fp32 on the same (rounded) tensors."""
    import fhog
    g = torch.Generator().manual_seed(57)
    mk = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16).cuda()
    q, k, v, w = mk(2, 256, 128), mk(2, 256, 128), mk(2, 256, 128), mk(2, 256, 128) * 0.1

    def penalty(attn, cast):
        qq, kk, vv = (cast(t).clone().requires_grad_(True) for t in (q, k, v))
        out = attn(qq, kk, vv)
        gq, gk, gv = torch.autograd.grad((out * cast(w)).sum(), (qq, kk, vv), create_graph=True)
        loss = gq.float().square().sum() + (gk.float() * gv.float()).sum()
        return torch.autograd.grad(loss, (qq, kk, vv))

    ours = penalty(lambda a, b, c: fhog.attention(a, b, c, True, schedule=schedule), lambda t: t)
    ref = penalty(lambda a, b, c: torch.nn.functional.scaled_dot_product_attention(a, b, c, is_causal=True), lambda t: t.float())
    for a, b in zip(ours, ref):
        assert normalised_max_error(a, b) < 3e-2   # three bf16 kernels in a row (forward, first backward, double-backward)
