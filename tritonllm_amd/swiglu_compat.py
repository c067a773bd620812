"""The second SwiGLU call signature the reference exposes (``triton_kernels/swiglu.py``):
``swiglu(a, alpha, precision_config, routing_data=None)`` with the limit carried by a
``PrecisionConfig``. Flexpoint scales are not part of the bf16 path (they are ``None`` -- i.e.
1.0 -- everywhere the gpt-oss model calls it), so only ``limit`` is honoured."""
from __future__ import annotations

from dataclasses import dataclass

import torch

from . import ops
from ._lib import require as _require


@dataclass(frozen=True)
class PrecisionConfig:
    limit: float | None


def swiglu(a: torch.Tensor, alpha: float, precision_config: PrecisionConfig, routing_data=None) -> torch.Tensor:
    """triton_kernels/swiglu.py:85-86. Always the interleaved layout; returns a fresh tensor."""
    if routing_data is not None:
        raise NotImplementedError("routing_data (ragged expert batches) is outside the bf16 layer-kernel path")
    _require(a.stride()[-1] == 1)
    _require(a.shape[-1] % 2 == 0)
    return ops.swiglu(a, alpha=alpha, limit=precision_config.limit, interleaved=True)
