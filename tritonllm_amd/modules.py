"""Leaf modules with the constructor and forward signatures of the reference's
``gpt_oss/triton/model.py``: ``RMSNorm`` (:55-68), ``QKV`` (:119-167), ``OUT`` (:170-216), ``UnEmbedding`` (:70-117),
``RotaryEmbedding`` (:218-337) and the token ``Embedding`` (``torch.nn.Embedding``
at :906-908). A model file written against the reference can import these instead.

Unlike the reference modules there is no torch fallback branch: inputs must be bf16
tensors on the GPU, and the HIP library must be present.
"""
from __future__ import annotations

import ctypes as C
import os

import torch

from . import ops
from ._lib import check, lib
from ._lib import require as _require
from .yarn import YarnParams


class RMSNorm(torch.nn.Module):
    def __init__(self, num_features: int, eps: float = 1e-05, device: torch.device | None = None):
        super().__init__()
        self.num_features = num_features
        self.eps = eps
        self.scale = torch.nn.Parameter(torch.ones(num_features, device=device, dtype=torch.float32))

    def forward(self, x: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
        return ops.rmsnorm_forward(x, self.scale, self.eps, out=out)


class QKV(torch.nn.Module):
    def __init__(self, hidden_size: int, qkv_dim: int, device: torch.device | None = None):
        super().__init__()
        self.weight = torch.nn.Parameter(torch.empty((qkv_dim, hidden_size), device=device, dtype=torch.bfloat16))
        self.bias = torch.nn.Parameter(torch.empty((qkv_dim), device=device, dtype=torch.bfloat16))
        # model.py:130-134: ATTN_FP8 switches the decode path to a per-row quantised fp8 copy of the weight
        self._use_fp8 = os.getenv("ATTN_FP8", "0").strip().lower() not in {"0", "false", "no", "off"}
        self._weight_fp8: torch.Tensor | None = None
        self._weight_scale: torch.Tensor | None = None

    @property
    def _fp8_weight(self):
        """``(weight_fp8, weight_scale)``, quantised on first use (model.py:160-167); ``(None, None)`` unless ATTN_FP8 is set."""
        if not self._use_fp8:
            return None, None
        if self._weight_fp8 is None:
            self._weight_fp8, self._weight_scale = ops.quantize_fp8_rows(self.weight.detach())
        return self._weight_fp8, self._weight_scale

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """``F.linear(x, weight, bias)``: one dense ``[..., qkv_dim]`` tensor."""
        return ops.linear_qkv_forward(x, self.weight, self.bias)

    def decode(self, x: torch.Tensor, q_dim: int, kv_dim: int):
        return ops.qkv_decode_forward(x, self.weight, self.bias, q_dim, kv_dim)

    def forward_rope(self, x: torch.Tensor, rope: "RotaryEmbedding", num_q_heads: int, num_kv_heads: int,
                     offset: torch.Tensor | None = None, positions: torch.Tensor | None = None):
        """Fused projection + bias + rotary for ``x [B, T, H]``: returns
        ``q [B,T,Hq,D]``, ``k [B,T,Hkv,D]`` (rotated) and ``v [B,T,Hkv,D]`` without the
        split / contiguous / rope_forward round trips of the reference's prefill path."""
        b, t, h = x.shape
        d = rope.head_dim
        q, k, v = ops.qkv_rope_forward(x.reshape(b * t, h), self.weight, self.bias, num_q_heads, num_kv_heads, d, yarn=rope.yarn,
                                       positions=positions, offset=offset, tokens_per_batch=t,
                                       max_context_length=rope.max_context_length)
        return q.view(b, t, num_q_heads, d), k.view(b, t, num_kv_heads, d), v.view(b, t, num_kv_heads, d)


class OUT(torch.nn.Module):
    """Attention out-projection (model.py:170-216): ``weight [hidden_size, out_dim]``, ``bias [hidden_size]``.
    ``decode_residual`` is the HIP kernel; ``forward`` is, as in the reference, the library GEMM."""

    def __init__(self, out_dim: int, hidden_size: int, device: torch.device | None = None):
        super().__init__()
        self.weight = torch.nn.Parameter(torch.empty((hidden_size, out_dim), device=device, dtype=torch.bfloat16))
        self.bias = torch.nn.Parameter(torch.empty((hidden_size), device=device, dtype=torch.bfloat16))
        self._use_fp8 = os.getenv("ATTN_FP8", "0").strip().lower() not in {"0", "false", "no", "off"}
        self._weight_fp8: torch.Tensor | None = None
        self._weight_scale: torch.Tensor | None = None

    @property
    def _fp8_weight(self):
        if not self._use_fp8:
            return None, None
        if self._weight_fp8 is None:
            self._weight_fp8, self._weight_scale = ops.quantize_fp8_rows(self.weight.detach())
        return self._weight_fp8, self._weight_scale

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return torch.nn.functional.linear(x, self.weight, self.bias)

    def decode_residual(self, x: torch.Tensor, residual: torch.Tensor) -> torch.Tensor:
        """``residual + x @ W.T + b`` for ``x [B,1,out_dim]``, written into ``residual`` (model.py:199-216)."""
        if self._use_fp8:
            w_fp8, w_scale = self._fp8_weight
            return ops.out_residual_decode_forward(x, w_fp8, self.bias, residual, weight_scale=w_scale)
        return ops.out_residual_decode_forward(x, self.weight, self.bias, residual)


class UnEmbedding(torch.nn.Module):
    """Output projection onto the vocabulary (model.py:70-117): ``weight [vocab_size, hidden_size]`` bf16.
    One token per batch row goes through the HIP stream kernels (fp8 copy of the weight under ``UNEMBED_FP8``);
    anything else is, as in the reference, the library GEMM."""

    def __init__(self, hidden_size: int, vocab_size: int, device: torch.device | None = None):
        super().__init__()
        self.weight = torch.nn.Parameter(torch.empty((vocab_size, hidden_size), device=device, dtype=torch.bfloat16))
        self._use_fp8 = os.getenv("UNEMBED_FP8", "0").strip().lower() not in {"0", "false", "no", "off"}
        self._weight_fp8: torch.Tensor | None = None
        self._weight_scale: torch.Tensor | None = None

    def _fp8(self):
        if self._weight_fp8 is None:
            self._weight_fp8, self._weight_scale = ops.quantize_fp8_rows(self.weight.detach())
        return self._weight_fp8, self._weight_scale

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if x.is_cuda and x.ndim == 3 and x.shape[1] == 1 and x.dtype == torch.bfloat16:
            if self._use_fp8:
                return ops.unembedding_decode_forward(x, *self._fp8())
            return ops.unembedding_decode_forward(x, self.weight)
        return torch.nn.functional.linear(x, self.weight, bias=None)

    def forward_argmax(self, x: torch.Tensor) -> torch.Tensor:
        if x.is_cuda and x.ndim == 3 and x.shape[1] == 1 and x.dtype == torch.bfloat16:
            if self._use_fp8:
                return ops.unembedding_decode_argmax_forward(x, *self._fp8())
            return ops.unembedding_decode_argmax_forward(x, self.weight)
        return self.forward(x)[-1].argmax(dim=-1)


class RotaryEmbedding(torch.nn.Module):
    """YaRN rotary embedding. ``.cos`` / ``.sin`` are the fp32 ``[max_ctx, head_dim/2]`` tables of
    the reference (built once per configuration by the HIP table kernel and shared), and they
    carry the YaRN parameters so that every kernel they are passed to computes cos/sin in
    registers rather than reading 33 MB of tables."""

    _cos_sin_cache: dict[tuple, tuple[torch.Tensor, torch.Tensor]] = {}

    def __init__(self, head_dim: int, base: int, dtype: torch.dtype, initial_context_length: int = 4096,
                 max_context_length: int = 131072, scaling_factor: float = 1.0, ntk_alpha: float = 1.0, ntk_beta: float = 32.0,
                 device: torch.device | None = None) -> None:
        super().__init__()
        self.head_dim = head_dim
        self.base = base
        self.dtype = dtype
        self.initial_context_length = initial_context_length
        self.max_context_length = max_context_length
        self.scaling_factor = scaling_factor
        self.ntk_alpha = ntk_alpha
        self.ntk_beta = ntk_beta
        self.device = torch.device(device) if device is not None else torch.device("cuda")
        self.yarn = YarnParams(head_dim=head_dim, base=float(base), initial_context_length=initial_context_length,
                               scaling_factor=scaling_factor, ntk_alpha=ntk_alpha, ntk_beta=ntk_beta)
        self.cos, self.sin = self._get_or_create_cos_sin()

    def _cache_key(self) -> tuple:
        return (self.device.type, self.device.index, self.head_dim, self.base, self.dtype, self.initial_context_length,
                self.max_context_length, self.scaling_factor, self.ntk_alpha, self.ntk_beta)

    def _get_or_create_cos_sin(self):
        key = self._cache_key()
        cached = self._cos_sin_cache.get(key)
        if cached is None:
            cached = self._compute_cos_sin(0, self.max_context_length)
            self._cos_sin_cache[key] = cached
        return cached

    def _compute_cos_sin(self, start: int, num_tokens: int):
        n_freq = self.head_dim // 2
        cos = torch.empty((num_tokens, n_freq), dtype=torch.float32, device=self.device)
        sin = torch.empty((num_tokens, n_freq), dtype=torch.float32, device=self.device)
        rc = lib().tllm_yarn_table_f32(cos.data_ptr(), sin.data_ptr(), start, num_tokens, C.byref(self.yarn.c_struct()),
                                       torch.cuda.current_stream().cuda_stream)
        check(rc, "yarn_table")
        if start == 0:
            cos._tllm_yarn = self.yarn   # lets the ops recognise these tables and skip reading them
            sin._tllm_yarn = self.yarn
        return cos, sin

    def forward(self, query: torch.Tensor, key: torch.Tensor, offset: torch.Tensor):
        ops.rope_forward(query, key, self.sin, self.cos, self.max_context_length, offset)
        return query, key


class Embedding(torch.nn.Module):
    """``torch.nn.Embedding(num_embeddings, embedding_dim, device=, dtype=torch.bfloat16)`` forward as a HIP gather."""

    def __init__(self, num_embeddings: int, embedding_dim: int, device: torch.device | None = None, dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        _require(dtype == torch.bfloat16)
        self.num_embeddings = num_embeddings
        self.embedding_dim = embedding_dim
        self.weight = torch.nn.Parameter(torch.empty((num_embeddings, embedding_dim), device=device, dtype=dtype))
        self._oob = None

    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        if self._oob is None or self._oob.device != self.weight.device:
            self._oob = torch.zeros((), dtype=torch.int32, device=self.weight.device)
        return ops.embedding_forward(ids, self.weight, oob_flag=self._oob)

    def check_ids(self) -> None:
        """Synchronising check: raise IndexError if any id seen so far was out of range."""
        if self._oob is not None and int(self._oob.item()) != 0:
            self._oob.zero_()
            raise IndexError("index out of range in Embedding")
