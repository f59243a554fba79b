"""Seeded synthetic workloads: the five benchmark configurations and their generator.

Tensor creation order is fixed (Q, K, V, dO, ddQ, ddK, ddV, then the K-row scales of the
cross-attention case), fp32 on the CPU from ``torch.Generator().manual_seed(seed)``, then
cast and copied to the device, so that a configuration and a seed name one set of tensors
on every machine.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict

import torch


@dataclass(frozen=True)
class Workload:
    name: str
    dtype: torch.dtype
    causal: bool
    B: int
    H: int
    n_q: int
    n_k: int
    d: int
    grad_std: float = 1.0       # std of dO and of the cotangents ddQ, ddK, ddV
    k_row_scale: bool = False   # multiply each K row by U(0.5, 2)

    @property
    def batch(self) -> int:
        return self.B * self.H

    @property
    def scale(self) -> float:
        return self.d ** -0.5

    @property
    def pairs(self) -> int:
        """(query, key) pairs that carry probability mass."""
        if self.causal:
            return self.batch * self.n_q * (self.n_q + 1) // 2
        return self.batch * self.n_q * self.n_k

    @property
    def flops_algorithmic(self) -> int:
        """12 (N_Q x N_K x d) contractions of the materialised formula, 2 FLOP per MAC."""
        return 24 * self.d * self.pairs

    @property
    def flops_executed(self) -> int:
        """25 contractions issued by the four recomputation passes (3 + 5 + 9 + 8); the opt-in fused
        statistics sweep issues 22 (5 + 9 + 8)."""
        return 50 * self.d * self.pairs

    @property
    def bytes_algorithmic(self) -> int:
        es = 2 if self.dtype == torch.bfloat16 else 4
        inputs = (4 * self.n_q + 4 * self.n_k) * self.d * es * self.batch + 4 * self.n_q * self.batch
        outputs = (2 * self.n_q + 2 * self.n_k) * self.d * es * self.batch
        return inputs + outputs


WORKLOADS: Dict[str, Workload] = {
    "cfg0_fp32_nc_256_d64": Workload("cfg0_fp32_nc_256_d64", torch.float32, False, 1, 2, 256, 256, 64, 1.0),
    "cfg1_bf16_nc_2048_d64": Workload("cfg1_bf16_nc_2048_d64", torch.bfloat16, False, 4, 16, 2048, 2048, 64, 0.1),
    "cfg2_bf16_causal_4096_d128": Workload("cfg2_bf16_causal_4096_d128", torch.bfloat16, True, 2, 16, 4096, 4096, 128, 0.1),
    "cfg3_bf16_causal_16384_d128": Workload("cfg3_bf16_causal_16384_d128", torch.bfloat16, True, 1, 32, 16384, 16384, 128, 0.1),
    "cfg4_bf16_cross_1024x8192_d64": Workload("cfg4_bf16_cross_1024x8192_d64", torch.bfloat16, False, 8, 8, 1024, 8192, 64, 0.1, True),
}
HEADLINE = "cfg2_bf16_causal_4096_d128"


def make_inputs(w: Workload, seed: int = 0, device="cpu") -> Dict[str, torch.Tensor]:
    """Q, K, V, dO, ddQ, ddK, ddV of shape (B, H, N, d), rounded to ``w.dtype``, on ``device``."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    qs, ks = (w.B, w.H, w.n_q, w.d), (w.B, w.H, w.n_k, w.d)
    out = {}
    for name, shape, std in (("Q", qs, 1.0), ("K", ks, 1.0), ("V", ks, 1.0), ("dO", qs, w.grad_std),
                             ("ddQ", qs, w.grad_std), ("ddK", ks, w.grad_std), ("ddV", ks, w.grad_std)):
        out[name] = torch.randn(shape, generator=g, dtype=torch.float32) * std
    if w.k_row_scale:
        out["K"] = out["K"] * (torch.rand((w.B, w.H, w.n_k, 1), generator=g, dtype=torch.float32) * 1.5 + 0.5)
    return {n: t.to(w.dtype).to(device) for n, t in out.items()}
