"""CPU tier: pin the oracle (oracle/bwdbwd_oracle.py) before anything is compared with it.

Each test is built so that a plausible mistake (dropped term, wrong sign, transposed
operand, wrong mask) in one statement of the math fails against an independent one.
"""
import math

import numpy as np
import pytest
import torch

from oracle.bwdbwd_oracle import (autograd_double_backward, brute_force, closed_form, first_backward,
                                  forward_o_lse, normalised_max_error)

NAMES = ("dq2", "dk2", "dv2", "ddo")


def rand_inputs(rng, n_q, n_k, d, batch=()):
    qs, ks = batch + (n_q, d), batch + (n_k, d)
    return dict(q=rng.standard_normal(qs), k=rng.standard_normal(ks), v=rng.standard_normal(ks),
                do=rng.standard_normal(qs), ddq=rng.standard_normal(qs), ddk=rng.standard_normal(ks),
                ddv=rng.standard_normal(ks))


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", [(24, 24, 8), (40, 40, 16), (17, 33, 8)])
def test_closed_form_equals_autograd_fp64(shape, causal):
    n_q, n_k, d = shape
    if causal and n_q != n_k:
        pytest.skip("causal is defined for N_Q == N_K")
    rng = np.random.default_rng(0)
    x = rand_inputs(rng, n_q, n_k, d, batch=(3,))
    scale = 1 / math.sqrt(d)
    cf = closed_form(**x, scale=scale, causal=causal)
    ag = autograd_double_backward(x["q"], x["k"], x["v"], x["do"], x["ddq"], x["ddk"], x["ddv"], scale, causal)
    for n, a in zip(NAMES, ag):
        assert normalised_max_error(cf[n], a) < 1e-10, n


@pytest.mark.parametrize("causal", [False, True])
def test_brute_force_scalar_loops(causal):
    rng = np.random.default_rng(1)
    n_q, n_k, d = (4, 4, 2) if causal else (3, 4, 2)
    x = rand_inputs(rng, n_q, n_k, d)
    cf = closed_form(**x, scale=0.7, causal=causal)
    bf = brute_force(x["q"], x["k"], x["v"], x["do"], x["ddq"], x["ddk"], x["ddv"], 0.7, causal)
    for n, b in zip(NAMES, bf):
        np.testing.assert_allclose(cf[n], b, rtol=1e-11, atol=1e-12, err_msg=n)


def test_reference_golden_tensors(golden):
    """The reference's own fixture (test_data.zip; asserted on dv2 by fhog/test_bwdbwd.py:82 and on
    dq2, ddo by fhog/jax_refs/torch_impl.py:225-226). It was generated with bf16 matmuls, so it pins
    the oracle at bf16 tolerance: measured 2.6e-3..4.2e-3, gate 2e-2 on all four outputs."""
    g = golden
    scale = 1 / math.sqrt(64)
    cf = closed_form(g["q"], g["k"], g["v"], g["do"], g["ddq"], g["ddk"], g["ddv"], scale, causal=False)
    for n in NAMES:
        err = normalised_max_error(cf[n], g[n])
        assert err < 2e-2, (n, err)
        assert err < 6e-3, (n, err)  # what was measured, with margin: a dropped term gives O(1)
    # the caches stored with the fixture agree with a recomputation at bf16 accuracy
    assert np.abs(cf["L"] - g["L"]).max() < 1e-2
    assert np.abs(cf["o"] - g["o"]).max() < 2e-2
    # feeding the fixture's own (bf16-grade) O and L changes nothing beyond that accuracy
    cf2 = closed_form(g["q"], g["k"], g["v"], g["do"], g["ddq"], g["ddk"], g["ddv"], scale, o=g["o"], lse=g["L"])
    for n in NAMES:
        assert normalised_max_error(cf2[n], g[n]) < 2e-2, n


@pytest.mark.parametrize("causal", [False, True])
def test_row_identities(causal):
    rng = np.random.default_rng(2)
    n, d = 24, 8
    x = rand_inputs(rng, n, n, d)
    scale = 0.3
    cf = closed_form(**x, scale=scale, causal=causal)
    o, lse = forward_o_lse(x["q"], x["k"], x["v"], scale, causal)
    s = scale * x["q"] @ x["k"].T
    p = np.exp(s - lse[:, None])
    if causal:
        p = np.tril(p)
    np.testing.assert_allclose(p.sum(-1), 1.0, atol=1e-13)
    dp = x["do"] @ x["v"].T
    dds = scale * (x["ddq"] @ x["k"].T + x["q"] @ x["ddk"].T)
    np.testing.assert_allclose(cf["d"], (p * dp).sum(-1), atol=1e-12)               # d = sum_j P dP
    b_alt = np.einsum("id,id->i", x["do"], p @ x["ddv"]) - 2 * cf["d"] * cf["dd"] + (p * dp * dds).sum(-1)
    np.testing.assert_allclose(cf["b"], b_alt, atol=1e-12)
    # b_i = dO_i . ddO_i - d_i dd_i: the statistic of the second sweep is a row dot of an OUTPUT of the third
    # (ddO = P ddV + P (ddS - dd) V and sum_j P_ij dP_ij = d_i), which ties the two passes together
    np.testing.assert_allclose(cf["b"], np.einsum("id,id->i", x["do"], cf["ddo"]) - cf["d"] * cf["dd"], atol=1e-12)
    if causal:  # row 0 sees only key 0
        np.testing.assert_allclose(cf["dq2"][0], 0.0, atol=1e-13)
        np.testing.assert_allclose(cf["ddo"][0], x["ddv"][0], atol=1e-13)
    # The key-side outputs sum to zero over the keys: dK2 = dS^T ddQ + dS'^T Q and dV2 = ddP^T dO, and every row of dS,
    # dS' and ddP sums to zero over j. A probability that underflows on the device breaks exactly this (the long-N GPU
    # test bounds the column sums of the device outputs with it).
    np.testing.assert_allclose(cf["dk2"].sum(0), 0.0, atol=1e-12 * n)
    np.testing.assert_allclose(cf["dv2"].sum(0), 0.0, atol=1e-12 * n)
    # ... and a result with that property broken by a constant offset in P is caught by the same check
    bad = closed_form(**x, scale=scale, causal=causal, lse=lse + 1e-3)
    assert np.abs(bad["dv2"].sum(0)).max() > 1e-6


def test_ddo_is_forward_jvp():
    """ddO is the JVP of the attention output in direction (ddQ, ddK, ddV); it does not depend on dO."""
    rng = np.random.default_rng(3)
    n_q, n_k, d = 12, 20, 8
    x = rand_inputs(rng, n_q, n_k, d)
    scale = 0.4
    t = {k: torch.tensor(v) for k, v in x.items()}

    def attn(q, k, v):
        return torch.softmax(q @ k.T * scale, -1) @ v

    _, jvp = torch.func.jvp(attn, (t["q"], t["k"], t["v"]), (t["ddq"], t["ddk"], t["ddv"]))
    cf = closed_form(**x, scale=scale)
    np.testing.assert_allclose(cf["ddo"], jvp.numpy(), atol=1e-12)
    x2 = dict(x, do=rng.standard_normal(x["do"].shape))
    np.testing.assert_allclose(closed_form(**x2, scale=scale)["ddo"], cf["ddo"], atol=1e-13)


@pytest.mark.parametrize("causal", [False, True])
def test_ddv_only_reduces_to_sdpa(causal):
    """ddQ = ddK = 0: dV' = 0, ddO = SDPA(Q, K, ddV), (dQ', dK') = SDPA first-order grads with V := ddV."""
    rng = np.random.default_rng(4)
    n, d = 16, 8
    x = rand_inputs(rng, n, n, d)
    x["ddq"][:] = 0
    x["ddk"][:] = 0
    scale = 1 / math.sqrt(d)
    cf = closed_form(**x, scale=scale, causal=causal)
    q = torch.tensor(x["q"], requires_grad=True)
    k = torch.tensor(x["k"], requires_grad=True)
    w = torch.tensor(x["ddv"])
    out = torch.nn.functional.scaled_dot_product_attention(q[None], k[None], w[None], is_causal=causal, scale=scale)[0]
    gq, gk = torch.autograd.grad(out, (q, k), torch.tensor(x["do"]))
    np.testing.assert_allclose(cf["dv2"], 0.0, atol=1e-13)
    np.testing.assert_allclose(cf["ddo"], out.detach().numpy(), atol=1e-12)
    np.testing.assert_allclose(cf["dq2"], gq.numpy(), atol=1e-12)
    np.testing.assert_allclose(cf["dk2"], gk.numpy(), atol=1e-12)


@pytest.mark.parametrize("causal", [False, True])
def test_adjoint_identity_vs_central_differences(causal):
    """<(ddQ,ddK,ddV), J t> == <J^T (ddQ,ddK,ddV), t>, with J t from central differences of the
    first backward (a different code path: no double-backward formula involved)."""
    rng = np.random.default_rng(5)
    n, d = 10, 4
    x = rand_inputs(rng, n, n, d)
    scale = 0.5
    t = [rng.standard_normal(x[k].shape) for k in ("q", "k", "v", "do")]
    eps = 1e-6
    plus = first_backward(*(x[k] + eps * tk for k, tk in zip(("q", "k", "v", "do"), t)), scale, causal)
    minus = first_backward(*(x[k] - eps * tk for k, tk in zip(("q", "k", "v", "do"), t)), scale, causal)
    jt = [(a - b) / (2 * eps) for a, b in zip(plus, minus)]
    lhs = sum((w * j).sum() for w, j in zip((x["ddq"], x["ddk"], x["ddv"]), jt))
    cf = closed_form(**x, scale=scale, causal=causal)
    rhs = sum((cf[n] * tk).sum() for n, tk in zip(("dq2", "dk2", "dv2", "ddo"), t))
    assert abs(lhs - rhs) < 1e-6 * max(1.0, abs(lhs)), (lhs, rhs)


def test_linearity_and_zero():
    rng = np.random.default_rng(6)
    n_q, n_k, d = 9, 14, 4
    x = rand_inputs(rng, n_q, n_k, d)
    y = rand_inputs(rng, n_q, n_k, d)
    base = {k: x[k] for k in ("q", "k", "v", "do")}
    f = lambda ddq, ddk, ddv: closed_form(**base, ddq=ddq, ddk=ddk, ddv=ddv, scale=0.6)
    a, b = 0.7, -1.3
    lhs = f(a * x["ddq"] + b * y["ddq"], a * x["ddk"] + b * y["ddk"], a * x["ddv"] + b * y["ddv"])
    r1, r2 = f(x["ddq"], x["ddk"], x["ddv"]), f(y["ddq"], y["ddk"], y["ddv"])
    z = f(0 * x["ddq"], 0 * x["ddk"], 0 * x["ddv"])
    for n in NAMES:
        np.testing.assert_allclose(lhs[n], a * r1[n] + b * r2[n], atol=1e-11)
        np.testing.assert_allclose(z[n], 0.0, atol=0)


def test_key_permutation_equivariance():
    rng = np.random.default_rng(7)
    n_q, n_k, d = 8, 12, 4
    x = rand_inputs(rng, n_q, n_k, d)
    perm = rng.permutation(n_k)
    xp = dict(x, k=x["k"][perm], v=x["v"][perm], ddk=x["ddk"][perm], ddv=x["ddv"][perm])
    a, b = closed_form(**x, scale=0.5), closed_form(**xp, scale=0.5)
    np.testing.assert_allclose(b["dq2"], a["dq2"], atol=1e-12)
    np.testing.assert_allclose(b["ddo"], a["ddo"], atol=1e-12)
    np.testing.assert_allclose(b["dk2"], a["dk2"][perm], atol=1e-12)
    np.testing.assert_allclose(b["dv2"], a["dv2"][perm], atol=1e-12)


def test_autograd_fp32_head_chunking_matches_fp64():
    rng = np.random.default_rng(8)
    x = rand_inputs(rng, 32, 32, 16, batch=(5,))
    args = (x["q"], x["k"], x["v"], x["do"], x["ddq"], x["ddk"], x["ddv"], 0.25, True)
    a64 = autograd_double_backward(*args, dtype=torch.float64, head_chunk=1)
    a32 = autograd_double_backward(*args, dtype=torch.float32, head_chunk=2)
    for u, w in zip(a32, a64):
        assert normalised_max_error(u, w) < 1e-5


# ---------------------------------------------------------------- bottom-right and sliding-window masks
def test_mask_follows_the_reference_index_formula():
    """The mask itself against fhog/jax_refs/jax_impl.py:110-115, index by index."""
    from oracle.bwdbwd_oracle import _mask
    for n_q, n_k, w in [(3, 5, None), (4, 4, 2), (2, 7, 3), (5, 5, 1), (6, 9, 100)]:
        m = _mask(n_q, n_k, "bottom_right", w)
        for i in range(n_q):
            for j in range(n_k):
                qi = i + n_k - n_q
                assert bool(m[i, j]) == (qi >= j and (w is None or qi - j < w)), (n_q, n_k, w, i, j)
        assert m.any(axis=1).all()   # with N_K >= N_Q every query sees at least one key
    assert np.array_equal(_mask(6, 6, "bottom_right"), _mask(6, 6, True))
    assert np.array_equal(_mask(6, 6, True, 100), _mask(6, 6, True))
    assert _mask(4, 9, False) is None


@pytest.mark.parametrize("spec", [("bottom_right", None, 12, 20), ("bottom_right", 5, 12, 20), (True, 4, 16, 16),
                                  ("bottom_right", 7, 16, 16)])
def test_band_masks_closed_form_equals_autograd_and_brute_force(spec):
    causal, window, n_q, n_k = spec
    rng = np.random.default_rng(5)
    x = rand_inputs(rng, n_q, n_k, 8, batch=(2,))
    scale = 8 ** -0.5
    cf = closed_form(**x, scale=scale, causal=causal, window=window)
    ag = autograd_double_backward(x["q"], x["k"], x["v"], x["do"], x["ddq"], x["ddk"], x["ddv"], scale, causal,
                                  window=window)
    for n, a in zip(NAMES, ag):
        assert normalised_max_error(cf[n], a) < 1e-10, n
    y = rand_inputs(rng, 4, 6 if causal == "bottom_right" else 4, 2)
    w_small = None if window is None else 2
    cf = closed_form(**y, scale=0.7, causal=causal, window=w_small)
    bf = brute_force(y["q"], y["k"], y["v"], y["do"], y["ddq"], y["ddk"], y["ddv"], 0.7, causal, w_small)
    for n, b in zip(NAMES, bf):
        np.testing.assert_allclose(cf[n], b, rtol=1e-11, atol=1e-12, err_msg=n)


def test_band_mask_reductions_to_known_cases():
    rng = np.random.default_rng(6)
    x = rand_inputs(rng, 10, 10, 4)
    base = closed_form(**x, scale=0.5, causal=True)
    for other in (closed_form(**x, scale=0.5, causal="bottom_right"), closed_form(**x, scale=0.5, causal=True, window=10)):
        for n in NAMES:
            np.testing.assert_allclose(other[n], base[n], rtol=0, atol=0)
    # window 1: every query sees exactly one key, P = 1 there: no gradient flows through the soft-max
    one = closed_form(**x, scale=0.5, causal=True, window=1)
    np.testing.assert_allclose(one["dq2"], 0, atol=1e-12)
    np.testing.assert_allclose(one["dk2"], 0, atol=1e-12)
    np.testing.assert_allclose(one["dv2"], 0, atol=1e-12)
    np.testing.assert_allclose(one["ddo"], x["ddv"], atol=1e-12)   # O_i = V_i, so ddO_i = ddV_i


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", [(24, 24, 8), (33, 33, 16), (17, 40, 8)])
def test_first_backward_and_forward_equal_sdpa_autograd(shape, causal):
    """forward_o_lse and first_backward (the oracle of the first-order kernels and of the adjoint test) against a
    library routine: torch's scaled_dot_product_attention and its autograd, in float64."""
    n_q, n_k, d = shape
    if causal and n_q != n_k:
        pytest.skip("causal is defined for N_Q == N_K")
    rng = np.random.default_rng(11)
    x = rand_inputs(rng, n_q, n_k, d, batch=(2,))
    scale = 0.37
    q, k, v = (torch.tensor(x[n], dtype=torch.float64, requires_grad=True) for n in ("q", "k", "v"))
    out = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=causal, scale=scale)
    want = torch.autograd.grad(out, (q, k, v), torch.tensor(x["do"]))
    o, lse = forward_o_lse(x["q"], x["k"], x["v"], scale, causal)
    assert normalised_max_error(o, out.detach()) < 1e-12
    s = scale * torch.einsum("bid,bjd->bij", q.detach(), k.detach())
    if causal:
        s = s.masked_fill(~torch.ones(n_q, n_k, dtype=torch.bool).tril(), float("-inf"))
    assert normalised_max_error(lse, torch.logsumexp(s, -1)) < 1e-12
    got = first_backward(x["q"], x["k"], x["v"], x["do"], scale, causal)
    for name, a, b in zip(("dq", "dk", "dv"), got, want):
        assert normalised_max_error(a, b) < 1e-12, name
