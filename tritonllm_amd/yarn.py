"""YaRN rotary parameters on the host.

The kernels compute cos/sin in registers as ``cos(float(pos) * inv_freq[i]) * concentration``;
``inv_freq`` and ``concentration`` are fixed per model and are computed here once, with the
same fp32 operation order as the reference's ``RotaryEmbedding._compute_concentration_and_inv_freq``
(``gpt_oss/triton/model.py:267-305``) so that the fp32 angles agree with its tables.
"""
from __future__ import annotations

import ctypes as C
import math
from dataclasses import dataclass, field

import torch

from ._lib import MAX_ROPE_FREQS, TllmYarn
from ._lib import require as _require


@dataclass(frozen=True)
class YarnParams:
    head_dim: int
    base: float
    initial_context_length: int = 4096
    scaling_factor: float = 1.0
    ntk_alpha: float = 1.0
    ntk_beta: float = 32.0
    concentration: float = field(init=False)
    inv_freq: tuple = field(init=False)          # head_dim/2 python floats (exact fp32 values)

    def __post_init__(self):
        if self.head_dim <= 0 or self.head_dim % 2:
            raise ValueError(f"head_dim {self.head_dim} must be even and positive")
        if self.head_dim // 2 > MAX_ROPE_FREQS:
            raise ValueError(f"head_dim {self.head_dim} exceeds {2 * MAX_ROPE_FREQS}")
        conc, inv = _concentration_and_inv_freq(
            self.head_dim, self.base, self.initial_context_length, self.scaling_factor, self.ntk_alpha, self.ntk_beta
        )
        object.__setattr__(self, "concentration", conc)
        object.__setattr__(self, "inv_freq", tuple(inv.tolist()))

    def c_struct(self) -> TllmYarn:
        s = getattr(self, "_c", None)
        if s is None:
            s = TllmYarn()
            for i, f in enumerate(self.inv_freq):
                s.inv_freq[i] = f
            s.concentration = self.concentration
            s.n_freq = len(self.inv_freq)
            object.__setattr__(self, "_c", s)
        return s

    def c_pointer(self):
        return C.pointer(self.c_struct())


def _concentration_and_inv_freq(head_dim, base, initial_context_length, scaling_factor, ntk_alpha, ntk_beta):
    # fp32 tensor arithmetic on the CPU, in the reference's order of operations
    freq = base ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim)
    if scaling_factor > 1.0:
        concentration = 0.1 * math.log(scaling_factor) + 1.0
        d_half = head_dim / 2
        low = d_half * math.log(initial_context_length / (ntk_beta * 2 * math.pi)) / math.log(base)
        high = d_half * math.log(initial_context_length / (ntk_alpha * 2 * math.pi)) / math.log(base)
        _require(0 < low < high < d_half - 1)
        interpolation = 1.0 / (scaling_factor * freq)
        extrapolation = 1.0 / freq
        ramp = (torch.arange(d_half, dtype=torch.float32) - low) / (high - low)
        mask = 1 - ramp.clamp(0, 1)
        inv_freq = interpolation * (1 - mask) + extrapolation * mask
    else:
        concentration = 1.0
        inv_freq = 1.0 / freq
    return concentration, inv_freq


def gpt_oss_yarn() -> YarnParams:
    """The gpt-oss-20b/120b rotary configuration (model.py:36-53 defaults)."""
    return YarnParams(head_dim=64, base=150000.0, initial_context_length=4096, scaling_factor=32.0, ntk_alpha=1.0, ntk_beta=32.0)
