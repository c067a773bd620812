"""Shape-keyed pool of reusable output buffers.

Same contract as the reference's ``gpt_oss/triton/scratch_pool.py:17-22``: one
buffer per (shape, dtype, device); a later call with the same key returns the
same memory, so results are *borrowed* until the next such call. This is what
keeps a decode step free of allocations and therefore capturable in a HIP graph.
"""
from __future__ import annotations

from typing import Any

import torch

_pool: dict[tuple, torch.Tensor] = {}


def get(shape: tuple, dtype: torch.dtype, device: torch.device) -> torch.Tensor:
    key = (tuple(shape), dtype, torch.device(device))
    buf = _pool.get(key)
    if buf is None:
        buf = torch.empty(tuple(shape), dtype=dtype, device=device)
        _pool[key] = buf
    return buf


def clear() -> None:
    _pool.clear()


def stats() -> dict[str, Any]:
    return {"num_buffers": len(_pool), "total_bytes": sum(t.numel() * t.element_size() for t in _pool.values())}
