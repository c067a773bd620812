"""The per-token layer-kernel stack of a gpt-oss-shaped model: the kernels of this package in the order the
reference's decode step calls them, with everything between them (attention, out-projection, expert GEMMs) left out.

Call order followed (paths under ``tritonllm/gpt_oss/triton/``):

    Transformer._forward_hidden   model.py:918-923   for block in blocks: x = block(x);  then the final norm
    AttentionBlock.forward        model.py:471-526   t = norm(x);  q, k, v = fused QKV + bias + rotary of t
    MLPBlock.forward              model.py:751-757   t = norm(x);  ... the experts' clamped SwiGLU (moe.py:25-33)

Per layer: attention RMSNorm + QKV + bias + YaRN rotary (one launch up to 16 rows -- the norm runs inside the QKV
kernel --, two launches above), the MLP block's RMSNorm, SwiGLU on the ``[4 * B, 5760]`` activations of the four
routed experts; after the last layer the final RMSNorm. The residual stream ``x`` is not updated between layers (what
would update it is not part of this path), so every layer normalises the same ``x`` with its own scales and projects
it with its own weight and bias.

The stack owns its output buffers and allocates nothing in ``token_step``, so a step can be captured in a HIP graph
and replayed with new ``x`` / ``positions`` / ``swiglu_x`` contents.
"""
from __future__ import annotations

import torch

from . import ops
from ._lib import require as _require
from .yarn import YarnParams


class LayerKernelStack:
    def __init__(self, weights, biases, attn_scales, mlp_scales, final_scale, yarn: YarnParams, batch: int, *,
                 num_q_heads: int = 64, num_kv_heads: int = 8, head_dim: int = 64, eps: float = 1e-5,
                 keep_layers: bool = False, fuse_norm: bool = True):
        """``weights[l] [qkv_dim, hidden]``, ``biases[l] [qkv_dim]``, ``attn_scales[l]`` / ``mlp_scales[l]`` /
        ``final_scale`` ``[hidden]`` (fp32 or bf16), all on the GPU. ``keep_layers``: every layer writes its own
        q / k / v / MLP-norm / SwiGLU buffers (``[L, ...]``; for checking), otherwise one set is reused by all layers.
        ``fuse_norm=False`` runs the attention norm as its own launch at every row count."""
        self.n_layers = len(weights)
        _require(len(biases) == len(attn_scales) == len(mlp_scales) == self.n_layers)
        self.weights, self.biases, self.attn_scales, self.mlp_scales, self.final_scale = weights, biases, attn_scales, mlp_scales, final_scale
        self.yarn, self.batch, self.eps, self.fuse_norm = yarn, batch, eps, fuse_norm
        self.nq, self.nkv, self.hd = num_q_heads, num_kv_heads, head_dim
        dev, hidden = weights[0].device, weights[0].shape[1]
        self.hidden = hidden
        n = self.n_layers if keep_layers else 1
        mk = lambda *shape: torch.empty(*shape, dtype=torch.bfloat16, device=dev)
        self.q, self.k, self.v = mk(n, batch, num_q_heads * head_dim), mk(n, batch, num_kv_heads * head_dim), mk(n, batch, num_kv_heads * head_dim)
        self.attn_normed = mk(batch, hidden)                 # used only when the norm is its own launch
        self.mlp_normed = mk(n, batch, hidden)
        self.swiglu_out = mk(n, 4 * batch, hidden)
        self.final = mk(batch, hidden)
        self._n = n

    def launches_per_step(self) -> int:
        fused = self.fuse_norm and ops._norm_fusable("decode", self.batch, self.hidden, self.hd)
        return self.n_layers * (3 if fused else 4) + 1

    def token_step(self, x: torch.Tensor, positions: torch.Tensor, swiglu_x: torch.Tensor) -> torch.Tensor:
        """``x [B, hidden]`` bf16 (the residual stream), ``positions [B]`` int64 on the device, ``swiglu_x [4 * B,
        2 * hidden]`` bf16 (interleaved gate / linear). Returns the final-norm output ``[B, hidden]`` (owned by the stack)."""
        _require(x.shape == (self.batch, self.hidden) and swiglu_x.shape == (4 * self.batch, 2 * self.hidden))
        for l in range(self.n_layers):
            i = l % self._n
            out = (self.q[i], self.k[i], self.v[i])
            if self.fuse_norm:
                ops.qkv_rope_forward(x, self.weights[l], self.biases[l], self.nq, self.nkv, self.hd, yarn=self.yarn, positions=positions,
                                     mode="decode", out=out, norm_scale=self.attn_scales[l], norm_eps=self.eps)
            else:
                ops.rmsnorm_forward(x, self.attn_scales[l], self.eps, out=self.attn_normed)
                ops.qkv_rope_forward(self.attn_normed, self.weights[l], self.biases[l], self.nq, self.nkv, self.hd, yarn=self.yarn,
                                     positions=positions, mode="decode", out=out)
            ops.rmsnorm_forward(x, self.mlp_scales[l], self.eps, out=self.mlp_normed[i])
            ops.swiglu(swiglu_x, out=self.swiglu_out[i])
        return ops.rmsnorm_forward(x, self.final_scale, self.eps, out=self.final)
