"""MI355X-native Flash Hog: attention double-backward on hand-written gfx950 kernels.

Public entry point mirrors the reference package (``fhog/__init__.py:1-3``).
"""
from .bwdbwd import BwdBwdPlan, flash_bwdbwd
from .attention import AttnBwd, FlashAttention, attention, attention_backward, attention_forward, produce_L

__all__ = ["flash_bwdbwd", "BwdBwdPlan", "FlashAttention", "AttnBwd", "attention", "attention_forward", "attention_backward",
           "produce_L"]
