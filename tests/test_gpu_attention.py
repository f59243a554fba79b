"""GPU tier: the HIP first-order kernels (fhog_attn_fwd / fhog_attn_bwd) against the fp64 oracle, the blocked
torch composition and torch autograd, and the whole bf16 autograd chain running on HIP kernels only."""
import pytest
import torch

from gpu_util import make_case, normalised_max_error, require_gpu
from oracle.bwdbwd_oracle import first_backward, forward_o_lse

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _gpu():
    require_gpu()


def _np(t):
    return t.detach().double().cpu().numpy()


SHAPES = [(2, 128, 128, 64), (3, 256, 384, 128), (2, 384, 128, 64), (9, 128, 256, 128), (1, 512, 512, 128),
          (2, 100, 77, 64), (3, 333, 333, 128), (1, 1, 1, 64), (2, 129, 257, 128)]   # the last four: ragged lengths


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", SHAPES)
def test_forward_against_fp64_oracle(shape, causal):
    import fhog
    batch, n_q, n_k, d = shape
    if causal:
        n_k = n_q
    x = make_case(batch, n_q, n_k, d, torch.bfloat16, seed=21)
    scale = d ** -0.5
    o, L = fhog.attention_forward(x["Q"], x["K"], x["V"], scale, causal, use_hip=True)
    o_ref, l_ref = forward_o_lse(_np(x["Q"]), _np(x["K"]), _np(x["V"]), scale, causal)
    assert o.dtype == torch.bfloat16 and L.dtype == torch.float32 and L.shape == (batch, n_q)
    assert normalised_max_error(o, o_ref) < 1e-2           # bf16 P and bf16 output rounding
    assert (L.double().cpu() - torch.from_numpy(l_ref)).abs().max() < 2e-3
    # the blocked torch composition (fp32 P) is the other implementation of the same call
    o_t, l_t = fhog.attention_forward(x["Q"], x["K"], x["V"], scale, causal, use_hip=False)
    assert normalised_max_error(o, o_t) < 1e-2
    assert (L - l_t).abs().max() < 2e-3


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", SHAPES)
def test_backward_against_fp64_oracle(shape, causal):
    import fhog
    from fhog.attention import attention_backward
    batch, n_q, n_k, d = shape
    if causal:
        n_k = n_q
    x = make_case(batch, n_q, n_k, d, torch.bfloat16, seed=22)
    scale = d ** -0.5
    o, L = fhog.attention_forward(x["Q"], x["K"], x["V"], scale, causal, use_hip=True)
    dq, dk, dv = attention_backward(x["Q"], x["K"], x["V"], o, x["dO"], L, scale, causal, use_hip=True)
    ref = first_backward(_np(x["Q"]), _np(x["K"]), _np(x["V"]), _np(x["dO"]), scale, causal)
    for name, got, want in zip(("dq", "dk", "dv"), (dq, dk, dv), ref):
        assert got.dtype == torch.bfloat16
        assert normalised_max_error(got, want) < 2e-2, name
    blocked = attention_backward(x["Q"], x["K"], x["V"], o, x["dO"], L, scale, causal, use_hip=False)
    for name, got, want in zip(("dq", "dk", "dv"), (dq, dk, dv), blocked):
        assert normalised_max_error(got, want) < 2e-2, name


@pytest.mark.parametrize("causal", [False, True])
def test_fp16_forward_and_backward(causal):
    import fhog
    from fhog.attention import attention_backward
    x = make_case(3, 256, 256, 128, torch.float16, seed=27)
    scale = 128 ** -0.5
    o, L = fhog.attention_forward(x["Q"], x["K"], x["V"], scale, causal, use_hip=True)
    o_ref, l_ref = forward_o_lse(_np(x["Q"]), _np(x["K"]), _np(x["V"]), scale, causal)
    assert o.dtype == torch.float16
    assert normalised_max_error(o, o_ref) < 2e-3
    assert (L.double().cpu() - torch.from_numpy(l_ref)).abs().max() < 2e-3
    got = attention_backward(x["Q"], x["K"], x["V"], o, x["dO"], L, scale, causal, use_hip=True)
    ref = first_backward(_np(x["Q"]), _np(x["K"]), _np(x["V"]), _np(x["dO"]), scale, causal)
    for name, a, b in zip(("dq", "dk", "dv"), got, ref):
        assert a.dtype == torch.float16
        assert normalised_max_error(a, b) < 5e-3, name


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("mask", [("bottom_right", None, 100, 177, 64), ("bottom_right", 40, 300, 300, 128), (True, 1, 160, 160, 64),
                                  ("bottom_right", 33, 257, 700, 128), (True, 129, 512, 512, 128)])
def test_band_masks_forward_and_backward(mask, dtype):
    """Bottom-right alignment and sliding windows (fhog/jax_refs/jax_impl.py:110-115) in the HIP first-order kernels:
    rows whose window starts in a later tile, tiles skipped on both edges of the band."""
    import fhog
    from fhog.attention import attention_backward
    causal, window, n_q, n_k, d = mask
    x = make_case(2, n_q, n_k, d, dtype, seed=28)
    scale = d ** -0.5
    o, L = fhog.attention_forward(x["Q"], x["K"], x["V"], scale, causal, window=window, use_hip=True)
    o_ref, l_ref = forward_o_lse(_np(x["Q"]), _np(x["K"]), _np(x["V"]), scale, causal, window)
    assert torch.isfinite(o.float()).all() and torch.isfinite(L).all()
    assert normalised_max_error(o, o_ref) < 1e-2
    assert (L.double().cpu() - torch.from_numpy(l_ref)).abs().max() < 2e-3
    got = attention_backward(x["Q"], x["K"], x["V"], o, x["dO"], L, scale, causal, window=window, use_hip=True)
    ref = first_backward(_np(x["Q"]), _np(x["K"]), _np(x["V"]), _np(x["dO"]), scale, causal, window)
    for name, a, b in zip(("dq", "dk", "dv"), got, ref):
        assert normalised_max_error(a, b) < 2e-2, name


def test_strided_rows_and_4d_input():
    """Row stride larger than d (q, k, v as slices of one packed (batch, N, 3d) tensor) and (B, H, N, d) input."""
    import fhog
    from fhog.attention import attention_backward
    batch, N, d = 4, 256, 64
    g = torch.Generator().manual_seed(23)
    packed = torch.randn(batch, N, 3 * d, generator=g).to(torch.bfloat16).cuda()
    q, k, v = packed[..., :d], packed[..., d:2 * d], packed[..., 2 * d:]
    do = torch.randn(batch, N, d, generator=g).to(torch.bfloat16).cuda()
    scale = d ** -0.5
    o, L = fhog.attention_forward(q, k, v, scale, True, use_hip=True)
    o_ref, l_ref = forward_o_lse(_np(q), _np(k), _np(v), scale, True)
    assert normalised_max_error(o, o_ref) < 1e-2
    assert (L.double().cpu() - torch.from_numpy(l_ref)).abs().max() < 2e-3
    dq, dk, dv = attention_backward(q, k, v, o, do, L, scale, True, use_hip=True)
    ref = first_backward(_np(q), _np(k), _np(v), _np(do), scale, True)
    for got, want in zip((dq, dk, dv), ref):
        assert normalised_max_error(got, want) < 2e-2
    q4, k4, v4 = (t.reshape(2, 2, N, d) for t in (q, k, v))
    o4, L4 = fhog.attention_forward(q4, k4, v4, scale, True, use_hip=True)
    assert o4.shape == (2, 2, N, d) and L4.shape == (2, 2, N)
    assert torch.equal(o4.flatten(0, 1), o) and torch.equal(L4.flatten(0, 1), L)


@pytest.mark.parametrize("causal", [False, True, "bottom_right"])
@pytest.mark.parametrize("case", [(torch.float32, 2, 256, 256, 64), (torch.float32, 3, 100, 177, 128), (torch.float32, 2, 33, 129, 32),
                                  (torch.bfloat16, 2, 200, 200, 32), (torch.float16, 1, 300, 300, 32), (torch.float32, 1, 1, 1, 64)])
def test_fp32_mfma_first_order_kernels(case, causal):
    """fp32 tensors (the producer of O and L for the first benchmark configuration) and d = 32 run on the fp32-MFMA
    first-order kernels: O, L, dQ, dK, dV against the fp64 oracle, at the fp32 gate for fp32 tensors."""
    import fhog
    from fhog.attention import attention_backward
    dtype, batch, n_q, n_k, d = case
    window = None
    if causal is True:
        n_k = n_q
    elif causal == "bottom_right":
        n_k, window = max(n_k, n_q), 40
    x = make_case(batch, n_q, n_k, d, dtype, seed=29)
    scale = d ** -0.5
    o, L = fhog.attention_forward(x["Q"], x["K"], x["V"], scale, causal, window=window, use_hip=True)
    o_ref, l_ref = forward_o_lse(_np(x["Q"]), _np(x["K"]), _np(x["V"]), scale, causal, window)
    tol = 1e-4 if dtype == torch.float32 else 1e-2
    assert o.dtype == dtype and L.dtype == torch.float32
    assert normalised_max_error(o, o_ref) < tol
    assert (L.double().cpu() - torch.from_numpy(l_ref)).abs().max() < (1e-4 if dtype == torch.float32 else 2e-3)
    got = attention_backward(x["Q"], x["K"], x["V"], o, x["dO"], L, scale, causal, window=window, use_hip=True)
    ref = first_backward(_np(x["Q"]), _np(x["K"]), _np(x["V"]), _np(x["dO"]), scale, causal, window)
    for name, a, b in zip(("dq", "dk", "dv"), got, ref):
        assert a.dtype == dtype
        assert normalised_max_error(a, b) < (1e-4 if dtype == torch.float32 else 2e-2), name


def test_fp32_kernels_take_a_negative_scale_and_16_bit_ones_fall_back():
    """The fp32-MFMA forward scales the scores before it takes their maximum: any sign of the scale. The 16-bit forward
    needs a positive one: use_hip=True raises, the default warns and takes the torch composition."""
    import fhog
    y = make_case(2, 128, 160, 64, torch.float32, seed=24)
    o, L = fhog.attention_forward(y["Q"], y["K"], y["V"], -0.2, False, use_hip=True)
    o_ref, l_ref = forward_o_lse(_np(y["Q"]), _np(y["K"]), _np(y["V"]), -0.2, False)
    assert normalised_max_error(o, o_ref) < 1e-4
    assert (L.double().cpu() - torch.from_numpy(l_ref)).abs().max() < 1e-4
    x = make_case(2, 128, 160, 64, torch.bfloat16, seed=24)
    with pytest.raises(ValueError, match="positive scale"):
        fhog.attention_forward(x["Q"], x["K"], x["V"], -0.2, False, use_hip=True)
    from fhog.attention import TorchCompositionWarning
    with pytest.warns(TorchCompositionWarning, match="positive scale"):   # never silently: the warning carries the library's reason
        o, L = fhog.attention_forward(x["Q"], x["K"], x["V"], -0.2, False)
    o_ref, l_ref = forward_o_lse(_np(x["Q"]), _np(x["K"]), _np(x["V"]), -0.2, False)
    assert normalised_max_error(o, o_ref) < 1e-2


def test_fp32_autograd_chain_runs_on_hip_kernels_only():
    """attention() on fp32 tensors: forward, first backward and double-backward are all kernels of the library (the torch
    composition is switched off for the duration of the test)."""
    import sys
    import fhog
    A = sys.modules["fhog.attention"]   # the module (fhog.attention the attribute is the function of that name)
    g = torch.Generator().manual_seed(30)
    mk = lambda *s: torch.randn(*s, generator=g).cuda()
    q, k, v, w = mk(2, 160, 64), mk(2, 160, 64), mk(2, 160, 64), mk(2, 160, 64)
    saved = A._blocks
    A._blocks = None   # any use of the blocked torch composition would now raise

    def penalty(attn):
        qq, kk, vv = (t.clone().requires_grad_(True) for t in (q, k, v))
        out = attn(qq, kk, vv)
        gq, gk, gv = torch.autograd.grad((out * w).sum(), (qq, kk, vv), create_graph=True)
        loss = gq.square().sum() + (gk * gv).sum()
        return torch.autograd.grad(loss, (qq, kk, vv))

    try:
        ours = penalty(lambda a, b, c: fhog.attention(a, b, c, True))
    finally:
        A._blocks = saved
    ref = penalty(lambda a, b, c: torch.nn.functional.scaled_dot_product_attention(a, b, c, is_causal=True))
    for a, b in zip(ours, ref):
        assert normalised_max_error(a, b) < 1e-4


@pytest.mark.parametrize("causal", [False, True])
def test_headline_shape_sampled_heads(causal):
    """B=2 H=16 N=4096 d=128: every head through the HIP kernels, three heads against fp32 torch."""
    import fhog
    from fhog.attention import attention_backward
    x = make_case(32, 4096, 4096, 128, torch.bfloat16, seed=25, grad_std=0.1)
    scale = 128 ** -0.5
    o, L = fhog.attention_forward(x["Q"], x["K"], x["V"], scale, causal, use_hip=True)
    dq, dk, dv = attention_backward(x["Q"], x["K"], x["V"], o, x["dO"], L, scale, causal, use_hip=True)
    for t in (o, L, dq, dk, dv):
        assert torch.isfinite(t.float()).all()
    for hd in (0, 13, 31):
        q, k, v = (x[n][hd:hd + 1].float().requires_grad_(True) for n in ("Q", "K", "V"))
        s = torch.matmul(q, k.transpose(-1, -2)) * scale
        if causal:
            s = s.masked_fill(torch.ones(4096, 4096, dtype=torch.bool, device=s.device).triu(1), float("-inf"))
        ref_o = torch.matmul(torch.softmax(s, -1), v)
        ref_L = torch.logsumexp(s, -1)
        gq, gk, gv = torch.autograd.grad(ref_o, (q, k, v), x["dO"][hd:hd + 1].float())
        assert normalised_max_error(o[hd:hd + 1], ref_o) < 1e-2
        assert (L[hd:hd + 1] - ref_L).abs().max() < 2e-3
        for got, want in zip((dq, dk, dv), (gq, gk, gv)):
            assert normalised_max_error(got[hd:hd + 1], want) < 2e-2


@pytest.mark.parametrize("causal", [False, True])
def test_bf16_autograd_chain_runs_on_hip_kernels(causal):
    """attention() on bf16 tensors: forward, first backward and double-backward are all HIP kernels; the
    gradient of a gradient penalty is compared with fp32 torch autograd on the same rounded inputs."""
    import fhog
    g = torch.Generator().manual_seed(26)
    mk = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16).cuda()
    q, k, v, w = mk(2, 256, 128), mk(2, 256, 128), mk(2, 256, 128), mk(2, 256, 128) * 0.1

    def penalty(attn, cast):
        qq, kk, vv = (cast(t).clone().requires_grad_(True) for t in (q, k, v))
        out = attn(qq, kk, vv)
        gq, gk, gv = torch.autograd.grad((out * cast(w)).sum(), (qq, kk, vv), create_graph=True)
        loss = gq.float().square().sum() + (gk.float() * gv.float()).sum()
        return torch.autograd.grad(loss, (qq, kk, vv))

    ours = penalty(lambda a, b, c: fhog.attention(a, b, c, causal), lambda t: t)
    ref = penalty(lambda a, b, c: torch.nn.functional.scaled_dot_product_attention(a, b, c, is_causal=causal),
                  lambda t: t.float())
    for a, b in zip(ours, ref):
        assert a.dtype == torch.bfloat16
        assert normalised_max_error(a, b) < 3e-2   # three bf16 stages chained (forward caches, dQ/dK/dV, double-backward)
