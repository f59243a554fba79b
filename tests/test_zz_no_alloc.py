"""GPU tier, collected last: the entry point that allocates nothing (fhog_bwdbwd_static_ws) against fhog_bwdbwd.

Both run the same kernels; the only difference is where the workspace lives (the library's own device array against a
caller-owned tensor of the same size), so with equal workspace sizes the outputs agree bit for bit, and both stay
inside the 2e-2 gate against the fp64 oracle. Two calls in a row, the second on a smaller input, share the array.
"""
import ctypes

import pytest
import torch

from gpu_util import NAMES, errors, make_case, reference_fp64_cpu, require_gpu, with_caches

pytestmark = pytest.mark.gpu


def _plan(x, scale, causal):
    from fhog import BwdBwdPlan, _lib
    plan = BwdBwdPlan(x["Q"], x["K"], x["V"], x["O"], x["dO"], x["ddQ"], x["ddK"], x["ddV"], x["L"], scale, causal=causal,
                      impl="bf16", split=False)
    # a caller-owned workspace exactly as large as the library's array: same split decisions in both entry points
    plan.ws_all = torch.empty(_lib.lib().fhog_static_ws_bytes() // 4, dtype=torch.float32, device="cuda")
    plan.args.ws, plan.args.ws_bytes = plan.ws_all.data_ptr(), _lib.lib().fhog_static_ws_bytes()
    return plan


def test_static_workspace_entry_point_matches_fhog_bwdbwd_on_two_calls_in_a_row():
    require_gpu()
    from fhog import _lib
    L = _lib.lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # first a launch whose passes split their streamed side (few slices), then a smaller, ragged one that does not
    cases = [((4, 1024, 1024, 128), True), ((2, 300, 200, 64), False)]
    for (batch, n_q, n_k, d), causal in cases:
        scale = d ** -0.5
        x = with_caches(make_case(batch, n_q, n_k, d, torch.bfloat16, seed=31, grad_std=0.1), scale, causal)
        plan = _plan(x, scale, causal)
        plan.ws_all.fill_(float("nan"))
        want = [o.clone() for o in plan.run()]
        torch.cuda.synchronize()
        for o in plan.outs:
            o.fill_(float("nan"))
        plan.ws_all.fill_(float("nan"))          # the static entry point must not need the caller's workspace
        before = torch.cuda.memory_allocated()
        _lib.check(L.fhog_bwdbwd_static_ws(ctypes.byref(plan.args), stream))
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        assert torch.isnan(plan.ws_all).all()    # ... and does not touch it
        for name, got, ref in zip(("dq2", "dk2", "dv2", "ddo"), plan.outs, want):
            assert torch.isfinite(got.float()).all(), name
            assert torch.equal(got, ref), name
        oracle = reference_fp64_cpu(x, scale, causal)
        dq2, dk2, dv2, ddo = plan.outs
        e = errors((dq2, dk2, dv2, ddo), [oracle[n] for n in NAMES])
        assert max(e.values()) < 2e-2, e
        # args.ws / ws_bytes are not read at all
        plan.args.ws, plan.args.ws_bytes = 0, 0
        for o in plan.outs:
            o.fill_(float("nan"))
        _lib.check(L.fhog_bwdbwd_static_ws(ctypes.byref(plan.args), stream))
        torch.cuda.synchronize()
        for got, ref in zip(plan.outs, want):
            assert torch.equal(got, ref)


def test_static_workspace_entry_point_rejects_what_does_not_fit():
    require_gpu()
    from fhog import _lib
    L = _lib.lib()
    rows_max = _lib.lib().fhog_static_ws_bytes() // 12
    x = with_caches(make_case(1, 128, 128, 64, torch.bfloat16, seed=32, grad_std=0.1), 0.125, False)
    from fhog import BwdBwdPlan
    plan = BwdBwdPlan(x["Q"], x["K"], x["V"], x["O"], x["dO"], x["ddQ"], x["ddK"], x["ddV"], x["L"], 0.125)
    plan.args.batch = rows_max // 128 + 1      # one slice too many for the array; rejected on the host, nothing is launched
    plan.args.stride_qb = plan.args.stride_kb = 128 * 64
    rc = L.fhog_bwdbwd_static_ws(ctypes.byref(plan.args), None)
    assert rc == -2, rc
    msg = L.fhog_last_error().decode()
    assert "static workspace" in msg and str(_lib.lib().fhog_static_ws_bytes()) in msg
    assert L.fhog_bwdbwd_static_ws(None, None) == -1


def test_static_workspace_entry_point_under_hip_graph_capture():
    """One eager call first (it looks the array's address up and raises the kernels' LDS limit, neither of which may
    run under capture), then the entry point is captured into a HIP graph and replayed: every replay gives the bits of
    the eager call, with the program's own eager work and synchronisations in between."""
    require_gpu()
    from fhog import _lib
    L = _lib.lib()
    x = with_caches(make_case(4, 512, 512, 128, torch.bfloat16, seed=33, grad_std=0.1), 128 ** -0.5, True)
    plan = _plan(x, 128 ** -0.5, True)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        _lib.check(L.fhog_bwdbwd_static_ws(ctypes.byref(plan.args), ctypes.c_void_p(side.cuda_stream)))   # warm-up, eager
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    eager = [o.clone() for o in plan.outs]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        _lib.check(L.fhog_bwdbwd_static_ws(ctypes.byref(plan.args), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    for rep in range(3):
        for o in plan.outs:
            o.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        for name, got, ref in zip(("dq2", "dk2", "dv2", "ddo"), plan.outs, eager):
            assert torch.equal(got, ref), (rep, name)
        _ = (x["Q"].float() @ x["K"].float().transpose(-1, -2)).sum().item()   # unrelated eager work between replays
