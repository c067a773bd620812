"""Checkpoint reader with the reference's interface (``Checkpoint``, weights.py:29-117): a directory of
``.safetensors`` files, ``get(name)`` returning a tensor on the requested device, and the MoE weights -- stored as
MXFP4 ``.blocks`` / ``.scales`` pairs -- expanded to bf16.

The expansion runs as one HIP kernel over the packed bytes on the GPU (17 bytes read and 64 written per block)
instead of the reference's chunked lookup-table indexing, so the checkpoint's packed form is all that crosses PCIe and
no int32 index temporaries are made. ``get(name, out=...)`` expands straight into a preallocated parameter slice.
There is no CPU expansion: an MXFP4 tensor can only be fetched to a GPU device.
"""
from __future__ import annotations

import os

import torch
from safetensors import safe_open

from . import ops
from ._lib import require as _require

# Bytes per MXFP4 block: 32 FP4 numbers in 16 bytes (weights.py:8-9)
BYTES_PER_BLOCK = 16
N_BLOCKS_MAX = 36   # the reference maps MoE names for up to 36 transformer blocks (weights.py:17-26)

_MXFP4_PARAMS = ("mlp1_weight", "mlp2_weight")


def _param_names(name: str):
    """The checkpoint key(s) behind a parameter name (PARAM_NAME_MAP, weights.py:17-26): the MoE weights of blocks
    0..35 are (blocks, scales) pairs, every other name is stored under itself."""
    parts = name.split(".")
    if len(parts) == 4 and parts[0] == "block" and parts[2] == "mlp" and parts[3] in _MXFP4_PARAMS and parts[1].isdigit() \
            and str(int(parts[1])) == parts[1] and int(parts[1]) < N_BLOCKS_MAX:
        return name + ".blocks", name + ".scales"
    return name


class Checkpoint:
    def __init__(self, path: str, device: torch.device):
        device = torch.device(device)
        self.device_str = device.type if device.index is None else f"{device.type}:{device.index}"
        self.tensor_name_to_file: dict[str, str] = {}
        for fname in sorted(os.listdir(path)):
            if not fname.endswith(".safetensors"):
                continue
            fpath = os.path.join(path, fname)
            with safe_open(fpath, framework="pt", device="cpu") as f:
                for key in f.keys():
                    self.tensor_name_to_file[key] = fpath

    def get(self, name: str, out: torch.Tensor | None = None) -> torch.Tensor:
        names = _param_names(name)
        if isinstance(names, tuple):
            return self._get_mxfp4_tensor(*names, out=out)
        t = self._get_tensor(names)
        if out is not None:
            out.copy_(t)
            return out
        return t

    def _get_tensor(self, name: str) -> torch.Tensor:
        _require(name in self.tensor_name_to_file, f"Tensor {name} not found in checkpoint.")
        with safe_open(self.tensor_name_to_file[name], framework="pt", device=self.device_str) as f:
            return f.get_tensor(name)

    def _get_mxfp4_tensor(self, blocks_name: str, scales_name: str, *, dtype: torch.dtype = torch.bfloat16,
                          out: torch.Tensor | None = None) -> torch.Tensor:
        _require(blocks_name in self.tensor_name_to_file, f"Blocks tensor {blocks_name} not found in checkpoint.")
        _require(scales_name in self.tensor_name_to_file, f"Scales tensor {scales_name} not found in checkpoint.")
        if dtype != torch.bfloat16:
            raise NotImplementedError("MXFP4 tensors expand to bfloat16 only")
        blocks = self._get_tensor(blocks_name)
        scales = self._get_tensor(scales_name)
        _require(blocks.shape[:-1] == scales.shape, f"{blocks.shape=} does not match {scales.shape=}")
        return ops.mxfp4_dequant(blocks, scales, out=out)
