"""CPU tier: the C-ABI library loads, exports every symbol the header declares, and rejects bad
arguments on the host before any launch. No compute call is made here (no GPU needed)."""
import ctypes
import re
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent


@pytest.fixture(scope="module")
def L():
    from fhog import _lib
    return _lib.lib()


def good_args():
    from fhog import _lib
    a = _lib.BwdBwdArgs()
    for i, (name, _) in enumerate(_lib.BwdBwdArgs._fields_[:14]):
        setattr(a, name, 0x10000 * (i + 1))  # fake, 16-byte aligned device addresses (never dereferenced)
    a.batch, a.n_q, a.n_k, a.d = 4, 256, 512, 64
    a.stride_qn = a.stride_kn = 64
    a.stride_qb, a.stride_kb = 256 * 64, 512 * 64
    a.scale, a.dtype, a.causal, a.impl = 0.125, 0, 0, 0
    return a


def test_header_symbols_exported(L):
    header = (ROOT / "include" / "fhog_hip.h").read_text()
    names = re.findall(r"^\s*(?:int|size_t|const char\*)\s+(fhog_\w+)\s*\(", header, flags=re.M)
    assert set(names) >= {"fhog_abi_version", "fhog_bwdbwd_args_size", "fhog_bwdbwd_workspace_bytes", "fhog_validate", "fhog_select_impl",
                          "fhog_bwdbwd", "fhog_bwdbwd_pass", "fhog_last_error",
                          "fhog_attn_args_size", "fhog_attn_validate", "fhog_attn_fwd", "fhog_attn_bwd",
                          "fhog_probe_mfma_rate", "fhog_bwdbwd_workspace_hint", "fhog_bwdbwd_static_ws"}
    for n in names:
        assert hasattr(L, n), n


def _header_fields(struct_name):
    header = (ROOT / "include" / "fhog_hip.h").read_text()
    body = header[header.index(f"typedef struct {struct_name}"):header.index(f"}} {struct_name};")]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    fields = []
    for decl in body.split("{", 1)[1].split(";"):
        decl = decl.strip()
        if not decl:
            continue
        for piece in decl.split(","):
            fields.append(re.findall(r"(\w+)\s*$", piece.strip())[0])
    return fields


def test_struct_mirror_matches_header():
    from fhog import _lib
    assert _header_fields("fhog_bwdbwd_args") == [f[0] for f in _lib.BwdBwdArgs._fields_]
    assert ctypes.sizeof(_lib.BwdBwdArgs) == _lib.lib().fhog_bwdbwd_args_size() == 216
    assert _header_fields("fhog_attn_args") == [f[0] for f in _lib.AttnArgs._fields_]
    assert ctypes.sizeof(_lib.AttnArgs) == _lib.lib().fhog_attn_args_size() == 160


def good_attn_args():
    from fhog import _lib
    a = _lib.AttnArgs()
    for i, (name, _) in enumerate(_lib.AttnArgs._fields_[:10]):
        setattr(a, name, 0x10000 * (i + 1))
    a.batch, a.n_q, a.n_k, a.d = 4, 256, 512, 64
    a.stride_qn = a.stride_kn = 64
    a.stride_qb, a.stride_kb = 256 * 64, 512 * 64
    a.scale, a.dtype, a.causal = 0.125, 0, 0
    return a


@pytest.mark.parametrize("mutate, backward, code, word", [
    (lambda a: None, 1, 0, ""),
    (lambda a: setattr(a, "dO", 0), 0, 0, ""),            # forward does not look at the backward-only pointers
    (lambda a: setattr(a, "dO", 0), 1, -1, "dO"),
    (lambda a: setattr(a, "lse", 0), 0, -1, "lse"),
    (lambda a: setattr(a, "dtype", 1), 0, 0, ""),             # fp32 tensors: the fp32-MFMA first-order kernels
    (lambda a: setattr(a, "dtype", 5), 0, -3, "dtype"),
    (lambda a: (setattr(a, "dtype", 1), setattr(a, "stride_kn", 68), setattr(a, "stride_kb", 512 * 68)), 1, 0, ""),   # 16 bytes = 4 floats
    (lambda a: (setattr(a, "dtype", 1), setattr(a, "scale", -0.125)), 0, 0, ""),   # any sign of the scale there
    (lambda a: setattr(a, "d", 32), 1, 0, ""),                # d = 32 as well
    (lambda a: setattr(a, "d", 96), 0, -2, "head dim"),
    (lambda a: setattr(a, "n_q", 200), 0, 0, ""),           # ragged lengths are fine
    (lambda a: setattr(a, "causal", 1), 0, -6, "causal"),   # top-left needs n_q == n_k
    (lambda a: setattr(a, "causal", 2), 0, 0, ""),
    (lambda a: (setattr(a, "causal", 2), setattr(a, "window", 17)), 1, 0, ""),
    (lambda a: setattr(a, "window", 17), 0, -6, "window"),
    (lambda a: setattr(a, "stride_kn", 60), 0, -4, "stride"),
    (lambda a: (setattr(a, "stride_qn", (1 << 24) + 8), setattr(a, "stride_qb", 1 << 40)), 0, -4, "2^24"),
    (lambda a: setattr(a, "v", 0x30008), 0, -5, "aligned"),
    (lambda a: setattr(a, "scale", float("inf")), 0, -9, "scale"),
    (lambda a: setattr(a, "scale", -0.125), 0, -9, "positive"),   # the forward's running maximum needs scale > 0
    (lambda a: setattr(a, "scale", 0.0), 1, -9, "positive"),
])
def test_attn_validate(L, mutate, backward, code, word):
    a = good_attn_args()
    mutate(a)
    assert L.fhog_attn_validate(ctypes.byref(a), backward) == code
    if code:
        assert word in L.fhog_last_error().decode()
        # the compute entry points refuse the same way, before any launch
        assert (L.fhog_attn_bwd if backward else L.fhog_attn_fwd)(ctypes.byref(a), None) == code


def test_version_and_workspace(L):
    assert L.fhog_abi_version() == 5
    assert L.fhog_bwdbwd_workspace_bytes(32, 4096) == 3 * 32 * 4096 * 4
    assert L.fhog_bwdbwd_workspace_bytes(-1, 5) == 0


def test_validate_accepts_good(L):
    a = good_args()
    assert L.fhog_validate(ctypes.byref(a)) == 0
    assert L.fhog_select_impl(ctypes.byref(a)) in (1, 2)
    a.dtype = 1
    a.stride_qn = a.stride_kn = 64
    assert L.fhog_select_impl(ctypes.byref(a)) == 1  # fp32 tensors always take the fp32-MFMA family


@pytest.mark.parametrize("mutate, code, word", [
    (lambda a: setattr(a, "q", 0), -1, "q"),
    (lambda a: setattr(a, "ws", 0), -1, "ws"),
    (lambda a: setattr(a, "d", 96), -2, "head dim"),
    (lambda a: setattr(a, "n_k", 0), -2, "n_k"),
    (lambda a: setattr(a, "batch", 70000), -2, "batch"),
    (lambda a: setattr(a, "dtype", 7), -3, "dtype"),
    (lambda a: setattr(a, "impl", 9), -10, "impl"),
    (lambda a: setattr(a, "schedule", 9), -11, "schedule"),
    (lambda a: setattr(a, "stride_qn", 32), -4, "stride"),
    (lambda a: setattr(a, "stride_kn", 68), -4, "multiples"),
    (lambda a: (setattr(a, "stride_kn", (1 << 24) + 8), setattr(a, "stride_kb", 1 << 40)), -4, "2^24"),
    (lambda a: setattr(a, "stride_qb", 64), -4, "batch stride"),
    (lambda a: setattr(a, "k", 0x20004), -5, "aligned"),
    (lambda a: setattr(a, "causal", 1), -6, "top-left"),          # n_q != n_k
    (lambda a: setattr(a, "causal", 3), -6, "causal"),
    (lambda a: (setattr(a, "causal", 2), setattr(a, "n_k", 128), setattr(a, "stride_kb", 128 * 64)), -6, "bottom-right"),
    (lambda a: setattr(a, "window", 16), -6, "window needs"),
    (lambda a: (setattr(a, "causal", 2), setattr(a, "window", -1)), -6, "window"),
    (lambda a: setattr(a, "scale", float("nan")), -9, "scale"),
    (lambda a: setattr(a, "ws_bytes", 3 * 4 * 256 * 4 - 4), -2, "ws_bytes"),
])
def test_validate_rejects(L, mutate, code, word):
    a = good_args()
    mutate(a)
    assert L.fhog_validate(ctypes.byref(a)) == code
    assert word in L.fhog_last_error().decode()
    # the compute entry points refuse the same way, before any launch
    assert L.fhog_bwdbwd(ctypes.byref(a), None) == code
    assert L.fhog_bwdbwd_pass(ctypes.byref(a), 1, None) == code


def test_workspace_hint(L):
    """The hint is the minimum where no pass would split, and grows by the partial results of the widest split
    where the launch is too small to fill the GPU (16-bit kernels at d = 64 only)."""
    a = good_args()                           # bf16, batch 4, 256 x 512, d = 64: 8 workgroups of 128 rows
    minimum = L.fhog_bwdbwd_workspace_bytes(4, 256)
    assert minimum == 3 * 4 * 256 * 4
    # 16 key tiles: one split in two keeps 8 tiles each -> pass 3 wants 2 x (2 * batch * n_q * d) floats
    assert L.fhog_bwdbwd_workspace_hint(ctypes.byref(a)) == minimum + 2 * (2 * 4 * 256 * 64 * 4)
    a.ws_bytes = minimum
    assert L.fhog_validate(ctypes.byref(a)) == 0
    a.ws_bytes = 0
    a.batch = 4096                            # plenty of workgroups: nothing to split
    a.stride_qb, a.stride_kb = 256 * 64, 512 * 64
    assert L.fhog_bwdbwd_workspace_hint(ctypes.byref(a)) == L.fhog_bwdbwd_workspace_bytes(4096, 256)
    a = good_args()
    a.dtype = 1                               # fp32 tensors: the fp32-MFMA family does not split
    assert L.fhog_bwdbwd_workspace_hint(ctypes.byref(a)) == minimum
    a.d = 96
    assert L.fhog_bwdbwd_workspace_hint(ctypes.byref(a)) == 0   # invalid arguments


@pytest.mark.parametrize("d", [64, 128])
def test_workspace_hint_stays_below_its_stated_bound(L, d):
    """Whatever batch and N: the partial results of split launches take fewer than 2 * 131072 * d floats (a pass stops
    doubling its split once it has 512 workgroups), so the workspace stays linear in N plus a constant."""
    worst = 0
    for batch in (1, 2, 3, 4, 5, 7, 8, 15, 16, 31, 32, 33, 64):
        for n in [128 * k + r for k in (1, 2, 3, 5, 8, 13, 16, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 511, 512, 1023, 1024)
                  for r in (-127, 0)]:
            a = good_args()
            a.batch, a.n_q, a.n_k, a.d = batch, n, n, d
            a.stride_qn = a.stride_kn = d
            a.stride_qb = a.stride_kb = n * d
            hint = L.fhog_bwdbwd_workspace_hint(ctypes.byref(a))
            stats = (3 * batch * n * 4 + 15) // 16 * 16
            assert hint >= L.fhog_bwdbwd_workspace_bytes(batch, n)
            worst = max(worst, hint - stats)
    assert 0 < worst < 2 * 131072 * d * 4
    assert worst > 2 * 65536 * d * 4      # the bound is not slack by a factor of two: some shape comes close


def test_probe_rejects_bad_arguments(L):
    flops = ctypes.c_double()
    assert L.fhog_probe_mfma_rate(None, 256, 10, 0, ctypes.byref(flops), None) == -1
    assert L.fhog_probe_mfma_rate(0x10000, 0, 10, 0, ctypes.byref(flops), None) == -2
    for mode in (6, 7, 14, 15, 16):
        assert L.fhog_probe_mfma_rate(0x10000, 256, 10, mode, ctypes.byref(flops), None) == -2
    assert L.fhog_probe_mfma_rate(0x10000, 256, 10, -1, ctypes.byref(flops), None) == -2


def test_every_mask_runs_on_both_kernel_families(L):
    a = good_args()                       # bf16, 256 x 512, d = 64
    for causal, window in ((0, 0), (2, 0), (2, 64), (2, 10 ** 9)):
        a.causal, a.window = causal, window
        assert L.fhog_validate(ctypes.byref(a)) == 0
        a.impl = 0
        assert L.fhog_select_impl(ctypes.byref(a)) == 2
        for forced in (1, 2):
            a.impl = forced
            assert L.fhog_validate(ctypes.byref(a)) == 0 and L.fhog_select_impl(ctypes.byref(a)) == forced


def test_null_args(L):
    assert L.fhog_validate(None) == -1


def test_impl_bf16_needs_bf16_shape(L):
    a = good_args()
    a.impl = 2
    a.dtype = 1
    assert L.fhog_validate(ctypes.byref(a)) == -3
    a.dtype = 0
    a.n_q = 100                      # ragged lengths are taken by the 16-bit kernels
    a.stride_qb = 100 * 64
    assert L.fhog_validate(ctypes.byref(a)) == 0
    a.d = 32                         # d = 32 is not
    a.stride_qn = a.stride_kn = 32
    assert L.fhog_validate(ctypes.byref(a)) == -2


def test_python_wrapper_errors():
    import fhog
    t = lambda *s, dt=torch.bfloat16: torch.zeros(*s, dtype=dt)
    q, k = t(2, 64, 64), t(2, 128, 64)
    L = torch.zeros(2, 64)
    with pytest.raises(TypeError):
        fhog.flash_bwdbwd(q, k, k, q, q, q, k, k.float(), L, 0.125)
    with pytest.raises(TypeError):
        d64 = lambda x: x.double()   # fp64 tensors are not taken (bf16, fp16, fp32 are)
        fhog.flash_bwdbwd(d64(q), d64(k), d64(k), d64(q), d64(q), d64(q), d64(k), d64(k), L, 0.125)
    with pytest.raises(ValueError):
        fhog.flash_bwdbwd(q, k, k, q, q, q, k, t(2, 64, 64), L, 0.125)
    with pytest.raises(ValueError):
        fhog.flash_bwdbwd(q, k, k, q, q, q, k, k, L, 0.125, causal=True)      # top-left needs N_Q == N_K
    with pytest.raises(ValueError):
        fhog.flash_bwdbwd(k, q, q, k, k, k, q, q, torch.zeros(2, 128), 0.125, causal="bottom_right")  # N_K < N_Q
    with pytest.raises(ValueError):
        fhog.flash_bwdbwd(q, k, k, q, q, q, k, k, L, 0.125, window=8)         # window without a causal mask
    with pytest.raises(ValueError):
        fhog.flash_bwdbwd(q, k, k, q, q, q, k, k, L, 0.125, causal="upper")
    with pytest.raises(ValueError):
        fhog.flash_bwdbwd(q, k, k, q, q, q, k, k, torch.zeros(2, 63), 0.125)
    with pytest.raises(ValueError, match="GPU only"):
        fhog.flash_bwdbwd(q, k, k, q, q, q, k, k, L, 0.125)  # CPU tensors: no CPU path exists
    with pytest.raises(ValueError):
        fhog.produce_L(q, t(2, 128, 64), is_causal=True)


def test_product_does_not_import_oracle():
    """The shipped package must not reach into oracle/ (it is the checker, not the product)."""
    for f in (ROOT / "flash-hob_amd").rglob("*.py"):
        assert "oracle" not in f.read_text(), f
    for f in (ROOT / "flash-hob_amd" / "csrc").glob("*"):
        assert "oracle" not in f.read_text(), f


def test_workload_flop_counts():
    from fhog.workloads import WORKLOADS
    w = WORKLOADS["cfg2_bf16_causal_4096_d128"]
    assert w.pairs == 32 * 4096 * 4097 // 2
    assert abs(w.flops_algorithmic - 8.248e11) / 8.248e11 < 1e-3
    assert abs(WORKLOADS["cfg1_bf16_nc_2048_d64"].flops_algorithmic - 4.123e11) / 4.123e11 < 1e-3
    assert w.bytes_algorithmic == (256 * 2**20 + 32 * 4096 * 4) + 128 * 2**20
