"""The gpt-oss layer ops, with the call signatures the reference model code uses.

Each function validates its tensors the way the reference does (``assert`` on shape
preconditions, ``.contiguous()`` on a strided last dim), takes raw device pointers and
hands them to ``libtllm_hip.so`` on the current PyTorch HIP stream. PyTorch is plumbing
here -- memory, streams, dtypes; all arithmetic happens in the HIP kernels. There is no
CPU path: tensors must live on the GPU and the shared library must be built.

Reference signatures (paths under ``tritonllm/gpt_oss/triton/``):

    rmsnorm_forward(x, scale, eps, out=None)                         triton_kernels.py:28
    rope_forward(query, key, sin, cos, max_context_length, offset)   triton_kernels.py:90
    qkv_decode_forward(hidden, weight, bias, q_dim, kv_dim)          triton_kernels.py:615
    qkv_rope_cache_decode_forward(hidden, weight, bias, sin, cos, max_context_length,
        cache_k, cache_v, offset, num_q_heads, num_kv_heads, head_dim,
        weight_scale=None)                                           triton_kernels.py:1109
    swiglu(x, alpha=1.702, limit=7.0, interleaved=True)              moe.py:25
    embedding: torch.nn.Embedding.forward                            model.py:906-920

Outputs that the reference takes from its scratch pool are taken from
``tritonllm_amd.scratch_pool`` here, with the same borrowed-buffer semantics.
"""
from __future__ import annotations

import ctypes as C
import math

import torch

from . import scratch_pool
from ._lib import TllmRope, check, lib
from ._lib import require as _require
from .yarn import YarnParams

_BF16 = torch.bfloat16

# rows at or below this use the weight-streaming decode kernel, above it the MFMA GEMM
DECODE_MAX_ROWS = 64
# At the gpt-oss shape the weight is read once whatever the row count (above 32 rows a kernel holds its share of the
# weight and streams the rows past it: ~6.5 us + 0.09 us per row -- 96 rows 16 us, 192 rows 24 us, 384 rows 38-42 us),
# where the GEMM's one round of tiles costs 50-56 us however few rows there are: they meet near 500 rows.
DECODE_MAX_ROWS_2880 = 448


def _decode_max_rows(hidden: int, head_dim: int) -> int:
    return DECODE_MAX_ROWS_2880 if hidden == 2880 and head_dim == 64 else DECODE_MAX_ROWS


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _on_gpu(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("tritonllm_amd ops run on the GPU only (got a CPU tensor); there is no CPU fallback")


def _overlaps(a: torch.Tensor, b: torch.Tensor) -> bool:
    a0, b0 = a.data_ptr(), b.data_ptr()
    return a0 < b0 + b.numel() * b.element_size() and b0 < a0 + a.numel() * a.element_size()


def _pooled_output(shape: tuple, dtype, device, *inputs) -> torch.Tensor:
    """A scratch-pool buffer for an output the kernel writes while other workgroups still read ``inputs``. The pool
    hands out one buffer per (shape, dtype, device), so an input that is itself a borrowed pool buffer of the same
    shape (the normalised activations, when hidden == n_q_heads * head_dim) would be that very memory: then the
    output is a fresh tensor instead."""
    buf = scratch_pool.get(shape, dtype, device)
    for t in inputs:
        if t is not None and t.numel() and buf.numel() and _overlaps(buf, t):
            return torch.empty(shape, dtype=dtype, device=device)
    return buf


def _yarn_of(t) -> YarnParams | None:
    return getattr(t, "_tllm_yarn", None)


def _rope_desc(cos, sin, yarn, positions, offset, tokens_per_batch, max_ctx, keep: list, rows: int) -> TllmRope:
    """Fill the C descriptor of where the rotary angles come from. ``keep`` collects
    objects that must stay alive until the launch call has returned. ``rows`` is the number of rows the kernel
    will rotate: it reads ``positions[row]`` for each of them, and only the host can check that they exist."""
    r = TllmRope()
    if yarn is None and cos is not None:
        yarn = _yarn_of(cos)
        if yarn is not None and _yarn_of(sin) is not yarn:
            yarn = None
    if yarn is not None:
        r.yarn = yarn.c_pointer()
        keep.append(yarn)
    else:
        _require(cos is not None and sin is not None, "rotary needs YaRN parameters or cos/sin tables")
        _require(cos.dtype == torch.float32 and sin.dtype == torch.float32)
        _require(cos.ndim == 2 and cos.shape == sin.shape)
        if cos.stride(-1) != 1:
            cos = cos.contiguous()
        if sin.stride(-1) != 1 or sin.stride(0) != cos.stride(0):
            sin = sin.contiguous()
            cos = cos.contiguous()
        _require(cos.shape[0] >= max_ctx, "cos/sin tables shorter than max_context_length")
        keep += [cos, sin]
        r.cos_table = cos.data_ptr()
        r.sin_table = sin.data_ptr()
        r.table_row_stride = cos.stride(0)
    # The kernels read positions[row] for every row and offset[0] from device memory: these checks are what keeps
    # those reads in bounds, so they raise (an `assert` disappears under `python -O`).
    if positions is not None:
        if not (positions.is_cuda and positions.dtype == torch.int64 and positions.is_contiguous()):
            raise ValueError("positions must be a contiguous int64 tensor on the GPU")
        if positions.numel() != rows:
            raise ValueError(f"positions holds {positions.numel()} entries for {rows} rows")
        r.positions = positions.data_ptr()
    if offset is not None:
        if not (offset.is_cuda and offset.dtype == torch.int64 and offset.numel() == 1):
            raise ValueError("offset must be an int64 tensor of one element on the GPU")
        r.offset = offset.data_ptr()
    r.tokens_per_batch = int(tokens_per_batch)
    r.max_ctx = int(max_ctx)
    return r


# --------------------------------------------------------------------------------------- RMSNorm
def rmsnorm_forward(x: torch.Tensor, scale: torch.Tensor, eps: float, out: torch.Tensor | None = None) -> torch.Tensor:
    """``y = x * rsqrt(mean(x^2) + eps) * scale`` over the last dim; ``out`` may alias ``x``."""
    _on_gpu(x, scale, out)
    _require(x.dtype == _BF16, "rmsnorm_forward: x must be bfloat16")
    _require(scale.dtype in (torch.float32, _BF16), "rmsnorm_forward: scale must be float32 or bfloat16")
    hidden = x.shape[-1]
    _require(scale.shape == (hidden,))
    if not x.is_contiguous():
        x = x.contiguous()
    if not scale.is_contiguous():
        scale = scale.contiguous()
    if out is None:
        out = scratch_pool.get(tuple(x.shape), x.dtype, x.device)
    _require(out.shape == x.shape and out.dtype == x.dtype and out.is_contiguous())
    rows = x.numel() // hidden if hidden else 0
    rc = lib().tllm_rmsnorm_bf16(x.data_ptr(), scale.data_ptr(), int(scale.dtype == _BF16), out.data_ptr(), rows, hidden,
                                 float(eps), _stream())
    check(rc, "rmsnorm_forward")
    return out


# --------------------------------------------------------------------------------------- embedding
def embedding_forward(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor | None = None,
                      oob_flag: torch.Tensor | None = None) -> torch.Tensor:
    """``out[..., :] = table[ids[...], :]`` (bit-exact). ids int32 or int64, any shape.

    An id outside ``[0, vocab)`` produces a zero row and sets ``oob_flag`` (int32 device
    scalar) to 1 when one is given -- never a device fault."""
    _on_gpu(ids, table, out, oob_flag)
    _require(table.dtype == _BF16 and table.ndim == 2 and table.is_contiguous())
    _require(ids.dtype in (torch.int32, torch.int64))
    if not ids.is_contiguous():
        ids = ids.contiguous()
    vocab, hidden = table.shape
    shape = (*ids.shape, hidden)
    if out is None:
        out = torch.empty(shape, dtype=table.dtype, device=table.device)   # a fresh tensor, as nn.Embedding returns
    _require(tuple(out.shape) == shape and out.dtype == table.dtype and out.is_contiguous())
    if oob_flag is not None:
        _require(oob_flag.dtype == torch.int32 and oob_flag.numel() == 1)
    rc = lib().tllm_embedding_bf16(table.data_ptr(), ids.data_ptr(), int(ids.dtype == torch.int64), out.data_ptr(), ids.numel(),
                                   hidden, vocab, oob_flag.data_ptr() if oob_flag is not None else None, _stream())
    check(rc, "embedding_forward")
    return out


def embedding_rmsnorm_forward(ids: torch.Tensor, table: torch.Tensor, scale: torch.Tensor, eps: float,
                              x_out: torch.Tensor | None = None, out: torch.Tensor | None = None,
                              oob_flag: torch.Tensor | None = None) -> tuple[torch.Tensor, torch.Tensor]:
    """``x = table[ids]`` (model.py:906-908, 920) and ``RMSNorm(x)`` of the first block (model.py:476) in one launch.
    Returns ``(x, normed)``, both ``[*ids.shape, hidden]``: ``x`` bit-exact like ``embedding_forward`` (a fresh tensor
    unless ``x_out`` is given), ``normed`` identical to ``rmsnorm_forward(x, scale, eps)`` (pooled unless ``out`` is given).
    Hidden sizes the fused kernel does not cover take the two separate calls."""
    _on_gpu(ids, table, scale, x_out, out, oob_flag)
    _require(table.dtype == _BF16 and table.ndim == 2 and table.is_contiguous())
    _require(ids.dtype in (torch.int32, torch.int64))
    _require(scale.dtype in (torch.float32, _BF16), "embedding_rmsnorm_forward: scale must be float32 or bfloat16")
    vocab, hidden = table.shape
    _require(scale.shape == (hidden,))
    if hidden % 8 != 0 or hidden > 8192:
        x = embedding_forward(ids, table, out=x_out, oob_flag=oob_flag)
        return x, rmsnorm_forward(x, scale, eps, out=out)
    if not ids.is_contiguous():
        ids = ids.contiguous()
    if not scale.is_contiguous():
        scale = scale.contiguous()
    shape = (*ids.shape, hidden)
    if x_out is None:
        x_out = torch.empty(shape, dtype=table.dtype, device=table.device)
    if out is None:
        out = scratch_pool.get(shape, table.dtype, table.device)
    for t in (x_out, out):
        _require(tuple(t.shape) == shape and t.dtype == table.dtype and t.is_contiguous())
    _require(x_out.data_ptr() != out.data_ptr())
    if oob_flag is not None:
        _require(oob_flag.dtype == torch.int32 and oob_flag.numel() == 1)
    rc = lib().tllm_embed_rmsnorm_bf16(table.data_ptr(), ids.data_ptr(), int(ids.dtype == torch.int64), x_out.data_ptr(), scale.data_ptr(),
                                       int(scale.dtype == _BF16), out.data_ptr(), ids.numel(), hidden, vocab, float(eps),
                                       oob_flag.data_ptr() if oob_flag is not None else None, _stream())
    check(rc, "embedding_rmsnorm_forward")
    return x_out, out


# --------------------------------------------------------------------------------------- SwiGLU
def swiglu(x: torch.Tensor, alpha: float = 1.702, limit: float | None = 7.0, interleaved: bool = True,
           out: torch.Tensor | None = None) -> torch.Tensor:
    """Clamped SwiGLU over the last dim: ``[..., 2n] -> [..., n]``."""
    _on_gpu(x, out)
    _require(x.dtype == _BF16, "swiglu: x must be bfloat16")
    _require(x.shape[-1] % 2 == 0)
    n_out = x.shape[-1] // 2
    if x.stride(-1) != 1:
        x = x.contiguous()
    x2 = x.reshape(-1, x.shape[-1]) if x.ndim != 2 else x
    if x2.ndim == 2 and x2.shape[0] > 1 and x2.stride(0) < x2.shape[1]:
        x2 = x2.contiguous()
    rows = x2.shape[0]
    shape = (*x.shape[:-1], n_out)
    if out is None:
        out = torch.empty(shape, dtype=x.dtype, device=x.device)
    _require(tuple(out.shape) == shape and out.dtype == x.dtype and out.is_contiguous())
    row_stride = x2.stride(0) if rows > 1 else 2 * n_out
    rc = lib().tllm_swiglu_bf16(x2.data_ptr(), out.data_ptr(), rows, n_out, row_stride, float(alpha),
                                float(limit) if limit is not None else 0.0, int(limit is not None), int(bool(interleaved)), _stream())
    check(rc, "swiglu")
    return out


# --------------------------------------------------------------------------------------- rotary
def rope_forward(query: torch.Tensor, key: torch.Tensor, sin: torch.Tensor | None, cos: torch.Tensor | None,
                 max_context_length: int, offset: torch.Tensor | None, *, yarn: YarnParams | None = None,
                 positions: torch.Tensor | None = None) -> None:
    """In-place rotary on ``query [B, T, Hq, D]`` and ``key [B, T, Hkv, D]``.

    Token ``t`` of every batch row sits at position ``(t + offset) % max_context_length``.
    ``sin``/``cos`` are the fp32 ``[max_ctx, D/2]`` tables; tables produced by
    :class:`tritonllm_amd.modules.RotaryEmbedding` carry their YaRN parameters and the
    kernel then computes cos/sin in registers instead of reading them. Extensions over
    the reference: ``yarn=`` to pass parameters without tables, ``positions=`` (int64
    ``[B*T]``) for an independent position per row."""
    _on_gpu(query, key, offset, positions)
    batch_size, num_tokens, num_heads, head_dim = query.shape
    kb, kt, num_key_value_heads, khd = key.shape
    _require((kb, kt, khd) == (batch_size, num_tokens, head_dim))
    _require(query.dtype == _BF16 and key.dtype == _BF16)
    _require(query.is_contiguous() and key.is_contiguous(), "rope_forward rotates in place and needs dense q/k")
    keep: list = []
    desc = _rope_desc(cos, sin, yarn, positions, offset, num_tokens, max_context_length, keep, batch_size * num_tokens)
    rc = lib().tllm_rope_bf16(query.data_ptr(), key.data_ptr(), batch_size * num_tokens, num_heads, num_key_value_heads, head_dim,
                              C.byref(desc), _stream())
    check(rc, "rope_forward")


# --------------------------------------------------------------------------------------- fused QKV
def _norm_fusable(kind: str, rows: int, hidden: int, hd: int) -> bool:
    """The decode kernel can normalise its own activations for the gpt-oss shape; beyond 16 rows
    its 32-row variant is out of registers and the two launches are the faster form."""
    return kind == "decode" and hidden == 2880 and hd == 64 and rows <= 16


def _launch_qkv(kind: str, x2, weight, bias, q, k, v, q_rs, k_rs, v_rs, kv_slot_stride, n_q, n_kv, hd, desc, norm=None, w_scale=None):
    """``norm = (scale, eps)``: x2 is the raw hidden state and is RMS-normalised first -- inside
    the decode kernel where it can, by a preceding rmsnorm launch otherwise.
    ``w_scale``: ``weight`` is fp8 e4m3 with one fp32 scale per output row (decode kernel, gpt-oss shape only)."""
    ptr = lambda t: t.data_ptr() if t is not None else None
    rope = C.byref(desc) if desc is not None else None
    if norm is not None:
        scale, eps = norm
        _require(scale.dtype in (torch.float32, _BF16) and scale.shape == (x2.shape[1],))
        if not scale.is_contiguous():
            scale = scale.contiguous()
        if w_scale is None and _norm_fusable(kind, x2.shape[0], x2.shape[1], hd):
            rc = lib().tllm_norm_qkv_rope_decode_bf16(
                x2.data_ptr(), scale.data_ptr(), int(scale.dtype == _BF16), float(eps), weight.data_ptr(), ptr(bias), ptr(q), ptr(k),
                ptr(v), q_rs, k_rs, v_rs, kv_slot_stride, x2.shape[0], x2.shape[1], n_q, n_kv, hd, rope, _stream())
            check(rc, "norm_qkv_rope_decode")
            return
        if w_scale is None or not _norm_fusable(kind, x2.shape[0], x2.shape[1], hd):
            x2 = rmsnorm_forward(x2, scale, eps)
            norm = None
    if w_scale is not None:
        if kind != "decode" or x2.shape[1] % 32 != 0 or hd % 16 != 0:
            raise NotImplementedError("fp8 weights with per-row scales: the HIP path has decode kernels only, for hidden a multiple "
                                      "of 32 and head_dim a multiple of 16")
        scale, eps = norm if norm is not None else (None, 0.0)
        rc = lib().tllm_qkv_rope_decode_w8_bf16(
            x2.data_ptr(), ptr(scale), int(scale is not None and scale.dtype == _BF16), float(eps), weight.data_ptr(),
            w_scale.data_ptr(), ptr(bias), ptr(q), ptr(k), ptr(v), q_rs, k_rs, v_rs, kv_slot_stride, x2.shape[0], x2.shape[1], n_q,
            n_kv, hd, rope, _stream())
        check(rc, "qkv_rope_decode_w8")
        return
    fn = lib().tllm_qkv_rope_decode_bf16 if kind == "decode" else lib().tllm_qkv_rope_prefill_bf16
    rc = fn(x2.data_ptr(), weight.data_ptr(), ptr(bias), ptr(q), ptr(k), ptr(v), q_rs, k_rs, v_rs, kv_slot_stride, x2.shape[0],
            x2.shape[1], n_q, n_kv, hd, rope, _stream())
    check(rc, f"qkv_rope_{kind}")


_FP8 = torch.float8_e4m3fn


def quantize_fp8_rows(weight: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """Per-row fp8 e4m3 quantisation of a bf16 weight, as ``_quantize_unembed_fp8`` (triton_kernels.py:261-268):
    returns ``(weight_fp8 [n, k] float8_e4m3fn, scale [n] float32)`` on the weight's device."""
    w = weight.to(torch.float32)
    amax = w.abs().max(dim=1, keepdim=True).values.clamp(min=1e-12)
    scale = (amax / torch.finfo(_FP8).max).squeeze(1).to(torch.float32)
    return (w / scale[:, None].clamp(min=1e-12)).to(_FP8), scale


def _prep_weight_scale(weight, weight_scale):
    _require(weight.dtype == _FP8, "weight_scale goes with a float8_e4m3fn weight")
    _require(weight_scale.dtype == torch.float32 and weight_scale.shape == (weight.shape[0],))
    return weight_scale if weight_scale.is_contiguous() else weight_scale.contiguous()


def _prep_linear(hidden2, weight, bias):
    _require(hidden2.dtype == _BF16 and weight.dtype in (_BF16, _FP8) and (bias is None or bias.dtype == _BF16))
    if not hidden2.is_contiguous():
        hidden2 = hidden2.contiguous()
    if not weight.is_contiguous():
        weight = weight.contiguous()
    if bias is not None and not bias.is_contiguous():
        bias = bias.contiguous()
    return hidden2, weight, bias


def qkv_rope_forward(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, num_q_heads: int, num_kv_heads: int,
                     head_dim: int, *, yarn: YarnParams | None = None, cos: torch.Tensor | None = None,
                     sin: torch.Tensor | None = None, positions: torch.Tensor | None = None, offset: torch.Tensor | None = None,
                     tokens_per_batch: int | None = None, max_context_length: int = 131072, rotate: bool = True,
                     mode: str = "auto", out: tuple | None = None, norm_scale: torch.Tensor | None = None,
                     norm_eps: float = 1e-5, weight_scale: torch.Tensor | None = None):
    """RMS-normed activations ``x [rows, hidden]`` -> ``(q [rows, Hq*D], k [rows, Hkv*D], v [rows, Hkv*D])``.

    With ``norm_scale`` given, ``x`` is the raw hidden state and the call also performs the
    ``RMSNorm(x)`` of model.py:476 (inside the same kernel for decode-sized gpt-oss shapes).
    With ``weight_scale`` the weight is float8_e4m3fn with per-row scales (see ``quantize_fp8_rows``).

    One fused kernel: projection, bias, rotary on q/k (fp32 accumulator, one rounding),
    outputs written to three dense tensors. ``mode``: "decode" (weight streaming),
    "prefill" (MFMA GEMM) or "auto" (by row count). No reference twin as a single call:
    it is F.linear + split + contiguous + rope_forward of model.py:506-522 in one launch."""
    _on_gpu(x, weight, bias, positions, offset, cos, sin, norm_scale, weight_scale)
    _require(x.ndim == 2)
    _require((weight.dtype == _FP8) == (weight_scale is not None), "a float8 weight needs weight_scale, a bfloat16 one takes none")
    rows, hidden = x.shape
    total_out, hidden_w = weight.shape
    _require(hidden == hidden_w)
    _require(total_out == (num_q_heads + 2 * num_kv_heads) * head_dim)
    _require(bias is None or bias.shape == (total_out,))
    x, weight, bias = _prep_linear(x, weight, bias)
    q_dim, kv_dim = num_q_heads * head_dim, num_kv_heads * head_dim
    if out is None:
        # keyed by the 3-D shape the reference's pool uses for q (triton_kernels.py:1196-1199), never a [rows, hidden] key
        q = _pooled_output((rows, num_q_heads, head_dim), x.dtype, x.device, x).view(rows, q_dim)
        kv = _pooled_output((2, rows, kv_dim), x.dtype, x.device, x)   # k and v share a shape: one buffer, two halves
        k, v = kv[0], kv[1]
    else:
        q, k, v = out
        _require(q.shape == (rows, q_dim) and k.shape == (rows, kv_dim) and v.shape == (rows, kv_dim))
        _require(q.stride(1) == 1 and k.stride(1) == 1 and v.stride(1) == 1)
    keep: list = []
    desc = None
    if rotate:
        desc = _rope_desc(cos, sin, yarn, positions, offset, tokens_per_batch if tokens_per_batch else max(rows, 1),
                          max_context_length, keep, rows)
    if mode == "auto":
        mode = "decode" if rows <= _decode_max_rows(x.shape[-1], head_dim) else "prefill"
    _require(mode in ("decode", "prefill"))
    _launch_qkv(mode, x, weight, bias, q, k, v, q.stride(0), k.stride(0), v.stride(0), 0, num_q_heads, num_kv_heads, head_dim, desc,
                norm=None if norm_scale is None else (norm_scale, norm_eps),
                w_scale=None if weight_scale is None else _prep_weight_scale(weight, weight_scale))
    return q, k, v


EMBED_FUSED_MAX_ROWS = 16


def embed_qkv_rope_forward(ids: torch.Tensor, table: torch.Tensor, norm_scale: torch.Tensor, norm_eps: float, weight: torch.Tensor,
                           bias: torch.Tensor | None, num_q_heads: int, num_kv_heads: int, head_dim: int, *,
                           yarn: YarnParams | None = None, cos: torch.Tensor | None = None, sin: torch.Tensor | None = None,
                           positions: torch.Tensor | None = None, offset: torch.Tensor | None = None,
                           tokens_per_batch: int | None = None, max_context_length: int = 131072, rotate: bool = True,
                           out: tuple | None = None, x_out: torch.Tensor | None = None, weight_scale: torch.Tensor | None = None,
                           oob_flag: torch.Tensor | None = None):
    """The first layer of a decode step: ``x = table[ids]`` (torch.nn.Embedding, model.py:906-908, 920), then the first
    block's ``RMSNorm(x)`` + QKV + bias + rotary (model.py:476, 489-503). Returns ``(x, q, k, v)`` with ``x [rows, hidden]``
    the gathered rows (bit-exact; the residual stream), q / k / v as ``qkv_rope_forward(x, ..., norm_scale=...)`` gives them.

    Up to 16 ids at the gpt-oss shape this is ONE launch (the gather rides in the QKV kernel's activation loads);
    otherwise it is the gather followed by ``qkv_rope_forward``. Either way an id outside the table produces a zero
    row of ``x`` (and the q / k / v that follow from it) and sets ``oob_flag``."""
    _on_gpu(ids, table, norm_scale, weight, bias, positions, offset, cos, sin, weight_scale, x_out, oob_flag)
    _require(ids.ndim == 1 and ids.dtype in (torch.int32, torch.int64))
    _require(table.dtype == _BF16 and table.ndim == 2 and table.is_contiguous())
    rows, (vocab, hidden) = ids.shape[0], table.shape
    # (the one-launch kernel addresses table rows with 32-bit byte offsets: tables of 4 GiB and more take the two launches)
    fused = 0 < rows <= EMBED_FUSED_MAX_ROWS and hidden == 2880 and head_dim == 64 and vocab * hidden * 2 < 2 ** 32
    if x_out is None:
        x_out = torch.empty(rows, hidden, dtype=_BF16, device=table.device)
    _require(x_out.shape == (rows, hidden) and x_out.dtype == _BF16 and x_out.is_contiguous())
    if not fused:
        embedding_forward(ids, table, out=x_out, oob_flag=oob_flag)
        q, k, v = qkv_rope_forward(x_out, weight, bias, num_q_heads, num_kv_heads, head_dim, yarn=yarn, cos=cos, sin=sin,
                                   positions=positions, offset=offset, tokens_per_batch=tokens_per_batch,
                                   max_context_length=max_context_length, rotate=rotate, out=out, norm_scale=norm_scale,
                                   norm_eps=norm_eps, weight_scale=weight_scale)
        return x_out, q, k, v
    _require((weight.dtype == _FP8) == (weight_scale is not None), "a float8 weight needs weight_scale, a bfloat16 one takes none")
    total_out, hidden_w = weight.shape
    _require(hidden == hidden_w and total_out == (num_q_heads + 2 * num_kv_heads) * head_dim)
    _require(bias is None or bias.shape == (total_out,))
    _require(norm_scale.dtype in (torch.float32, _BF16) and norm_scale.shape == (hidden,))
    if oob_flag is not None:
        _require(oob_flag.dtype == torch.int32 and oob_flag.numel() == 1)
    ids = ids if ids.is_contiguous() else ids.contiguous()
    norm_scale = norm_scale if norm_scale.is_contiguous() else norm_scale.contiguous()
    _, weight, bias = _prep_linear(x_out, weight, bias)
    w_scale = None if weight_scale is None else _prep_weight_scale(weight, weight_scale)
    q_dim, kv_dim = num_q_heads * head_dim, num_kv_heads * head_dim
    if out is None:
        q = _pooled_output((rows, num_q_heads, head_dim), _BF16, table.device, x_out).view(rows, q_dim)
        kv = _pooled_output((2, rows, kv_dim), _BF16, table.device, x_out)
        k, v = kv[0], kv[1]
    else:
        q, k, v = out
        _require(q.shape == (rows, q_dim) and k.shape == (rows, kv_dim) and v.shape == (rows, kv_dim))
        _require(q.stride(1) == 1 and k.stride(1) == 1 and v.stride(1) == 1)
    keep: list = []
    desc = None
    if rotate:
        desc = _rope_desc(cos, sin, yarn, positions, offset, tokens_per_batch if tokens_per_batch else rows, max_context_length, keep, rows)
    ptr = lambda t: t.data_ptr() if t is not None else None
    rc = lib().tllm_embed_norm_qkv_rope_decode_bf16(
        ids.data_ptr(), int(ids.dtype == torch.int64), table.data_ptr(), vocab, x_out.data_ptr(), ptr(oob_flag), norm_scale.data_ptr(),
        int(norm_scale.dtype == _BF16), float(norm_eps), weight.data_ptr(), ptr(w_scale), ptr(bias), q.data_ptr(), k.data_ptr(),
        v.data_ptr(), q.stride(0), k.stride(0), v.stride(0), 0, rows, hidden, num_q_heads, num_kv_heads, head_dim,
        C.byref(desc) if desc is not None else None, _stream())
    check(rc, "embed_norm_qkv_rope_decode")
    return x_out, q, k, v


def _split_head_dim(q_dim: int, kv_dim: int) -> int:
    """A head size that tiles both q_dim and kv_dim (no rotation: any even tiling will do)."""
    if q_dim % 64 == 0 and kv_dim % 64 == 0:
        return 64
    g = math.gcd(q_dim, kv_dim)
    _require(g % 2 == 0, "q_dim and kv_dim need a common even divisor")
    return g


def qkv_decode_forward(hidden: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, q_dim: int, kv_dim: int):
    """Unfused decode projection: ``[B,1,H] -> q [B,1,q_dim], k, v [B,1,kv_dim]`` (no rotary)."""
    _on_gpu(hidden, weight, bias)
    batch, num_tokens, hidden_size = hidden.shape
    total_out, hidden_size_weight = weight.shape
    _require(num_tokens == 1)
    _require(hidden_size == hidden_size_weight)
    _require(bias.shape == (total_out,))
    _require(total_out == q_dim + 2 * kv_dim)
    _require(weight.dtype == _BF16)
    x2, weight, bias = _prep_linear(hidden.reshape(batch, hidden_size), weight, bias)
    hd = _split_head_dim(q_dim, kv_dim)
    q = _pooled_output((batch, q_dim), hidden.dtype, hidden.device, x2)
    kv = _pooled_output((2, batch, kv_dim), hidden.dtype, hidden.device, x2)
    k, v = kv[0], kv[1]
    _launch_qkv("decode", x2, weight, bias, q, k, v, q_dim, kv_dim, kv_dim, 0, q_dim // hd, kv_dim // hd, hd, None)
    return q[:, None, :], k[:, None, :], v[:, None, :]


def qkv_rope_cache_decode_forward(hidden, weight, bias, sin, cos, max_context_length, cache_k, cache_v, offset, num_q_heads,
                                  num_kv_heads, head_dim, weight_scale=None, *, yarn: YarnParams | None = None,
                                  positions: torch.Tensor | None = None, norm_scale: torch.Tensor | None = None,
                                  norm_eps: float = 1e-5):
    """Fused decode step: projection + bias + rotary; the rotated k and the raw v of the
    new token are written into the KV cache at slot ``offset``; q ``[B,1,Hq*D]`` is returned
    (a borrowed pool buffer). ``offset`` is an int64 device tensor of shape (1,) and is read
    on the device, so the call can be replayed from a HIP graph. With ``norm_scale`` the
    block's input RMSNorm (model.py:476) runs inside the same kernel on the raw ``hidden``."""
    _on_gpu(hidden, weight, bias, cache_k, cache_v, offset, positions, norm_scale, weight_scale)
    _require((weight.dtype == _FP8) == (weight_scale is not None), "a float8 weight needs weight_scale, a bfloat16 one takes none")
    batch, num_tokens, hidden_size = hidden.shape
    total_out, hidden_size_weight = weight.shape
    _require(num_tokens == 1)
    _require(hidden_size == hidden_size_weight)
    _require(total_out == (num_q_heads + 2 * num_kv_heads) * head_dim)
    _require(bias.shape == (total_out,))
    _require(cache_k.shape == cache_v.shape)
    _require(cache_k.shape[0] == batch)
    _require(cache_k.shape[2] == num_kv_heads)
    _require(cache_k.shape[3] == head_dim)
    _require(offset.shape == (1,))
    _require(cache_k.dtype == _BF16 and cache_v.dtype == _BF16)
    _require(cache_k.stride() == cache_v.stride())
    _require(cache_k.stride(3) == 1 and cache_k.stride(2) == head_dim, "KV cache must be dense over (heads, head_dim)")
    x2, weight, bias = _prep_linear(hidden.reshape(batch, hidden_size), weight, bias)
    q = _pooled_output((batch, num_q_heads, head_dim), hidden.dtype, hidden.device, x2)
    keep: list = []
    desc = _rope_desc(cos, sin, yarn, positions, offset, 1, max_context_length, keep, batch)
    _launch_qkv("decode", x2, weight, bias, q, cache_k, cache_v, num_q_heads * head_dim, cache_k.stride(0), cache_v.stride(0),
                cache_k.stride(1), num_q_heads, num_kv_heads, head_dim, desc,
                norm=None if norm_scale is None else (norm_scale, norm_eps),
                w_scale=None if weight_scale is None else _prep_weight_scale(weight, weight_scale))
    return q.reshape(batch, 1, num_q_heads * head_dim)


def linear_qkv_forward(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None) -> torch.Tensor:
    """``F.linear(x, weight, bias)`` for the QKV weight (model.py:136-138): ``[..., H] -> [..., qkv_dim]``
    through the MFMA kernel (or the streaming kernel for few rows), writing one dense output."""
    _on_gpu(x, weight, bias)
    total_out, hidden = weight.shape
    _require(x.shape[-1] == hidden and weight.dtype == _BF16)
    x2, weight, bias = _prep_linear(x.reshape(-1, hidden), weight, bias)
    rows = x2.shape[0]
    hd = 64 if total_out % 64 == 0 else 2
    _require(total_out % hd == 0)
    out = torch.empty((*x.shape[:-1], total_out), dtype=x.dtype, device=x.device)
    o2 = out.view(rows, total_out)
    mode = "decode" if rows <= _decode_max_rows(hidden, hd) else "prefill"
    # all columns as "q heads" of one dense output row
    _launch_qkv(mode, x2, weight, bias, o2, None, None, total_out, 0, 0, 0, total_out // hd, 0, hd, None)
    return out


# --------------------------------------------------------------------------------------- out-projection (decode)
def out_residual_decode_forward(hidden: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, residual: torch.Tensor,
                                weight_scale: torch.Tensor | None = None) -> torch.Tensor:
    """``residual + hidden @ weight.T + bias`` for one token per batch row (triton_kernels.py:1470-1517):
    ``hidden [B,1,out_dim]``, ``weight [hidden_size, out_dim]`` (bf16, or float8_e4m3fn with ``weight_scale
    [hidden_size]``), ``bias [hidden_size]``, ``residual [B,1,hidden_size]``. Like the reference the result is
    written into ``residual``'s storage (when its last dimension is dense) and returned as ``[B,1,hidden_size]``."""
    _on_gpu(hidden, weight, bias, residual, weight_scale)
    batch, num_tokens, out_dim_hidden = hidden.shape
    hidden_size, out_dim_weight = weight.shape
    _require(num_tokens == 1)
    _require(out_dim_hidden == out_dim_weight)
    _require(bias.shape == (hidden_size,))
    _require(residual.shape == (batch, 1, hidden_size))
    _require(hidden.dtype == _BF16 and bias.dtype == _BF16 and residual.dtype == _BF16)
    _require((weight.dtype == _FP8) == (weight_scale is not None), "a float8 weight needs weight_scale, a bfloat16 one takes none")
    _require(weight.dtype in (_BF16, _FP8))
    x2 = hidden.reshape(batch, out_dim_hidden)
    res2 = residual.reshape(batch, hidden_size)
    if not x2.is_contiguous():
        x2 = x2.contiguous()
    if not weight.is_contiguous():
        weight = weight.contiguous()
    if not bias.is_contiguous():
        bias = bias.contiguous()
    if res2.stride(-1) != 1:
        res2 = res2.contiguous()
    ws = None if weight_scale is None else _prep_weight_scale(weight, weight_scale)
    out = res2
    rc = lib().tllm_out_residual_decode_bf16(x2.data_ptr(), weight.data_ptr(), ws.data_ptr() if ws is not None else None, bias.data_ptr(),
                                             res2.data_ptr(), out.data_ptr(), res2.stride(0), out.stride(0), batch, out_dim_hidden,
                                             hidden_size, _stream())
    check(rc, "out_residual_decode_forward")
    return out[:, None, :]


# --------------------------------------------------------------------------------------- unembedding (decode)
def _unembed_prep(hidden, weight, weight_scale):
    _on_gpu(hidden, weight, weight_scale)
    batch, num_tokens, hidden_size = hidden.shape
    vocab_size, hidden_size_weight = weight.shape
    _require(num_tokens == 1)
    _require(hidden_size == hidden_size_weight)
    _require(hidden.dtype == _BF16)
    _require((weight.dtype == _FP8) == (weight_scale is not None), "a float8 weight needs weight_scale, a bfloat16 one takes none")
    _require(weight.dtype in (_BF16, _FP8))
    x2 = hidden.reshape(batch, hidden_size)
    if not x2.is_contiguous():
        x2 = x2.contiguous()
    if not weight.is_contiguous():
        weight = weight.contiguous()
    ws = None if weight_scale is None else _prep_weight_scale(weight, weight_scale)
    return x2, weight, ws, batch, hidden_size, vocab_size


def unembedding_decode_forward(hidden: torch.Tensor, weight: torch.Tensor, weight_scale: torch.Tensor | None = None) -> torch.Tensor:
    """``hidden [B,1,H] @ weight[V,H].T -> logits [B,1,V]`` (a borrowed pool buffer), triton_kernels.py:163-197;
    with ``weight_scale`` the fp8 form :271-302."""
    x2, weight, ws, batch, hidden_size, vocab_size = _unembed_prep(hidden, weight, weight_scale)
    logits = scratch_pool.get((batch, vocab_size), hidden.dtype, hidden.device)
    rc = lib().tllm_unembedding_decode_bf16(x2.data_ptr(), weight.data_ptr(), ws.data_ptr() if ws is not None else None,
                                            logits.data_ptr(), logits.stride(0), batch, hidden_size, vocab_size, _stream())
    check(rc, "unembedding_decode_forward")
    return logits[:, None, :]


def unembedding_decode_fp8_forward(hidden, weight_fp8, weight_scale):
    """triton_kernels.py:271-302."""
    return unembedding_decode_forward(hidden, weight_fp8, weight_scale)


def unembedding_decode_argmax_forward(hidden: torch.Tensor, weight: torch.Tensor, weight_scale: torch.Tensor | None = None) -> torch.Tensor:
    """Greedy token per batch row without materialising the logits: ``int32 [B]`` (triton_kernels.py:363-401;
    with ``weight_scale`` :470-512). The candidates of the wavefronts travel through a pooled workspace."""
    x2, weight, ws, batch, hidden_size, vocab_size = _unembed_prep(hidden, weight, weight_scale)
    nbytes = lib().tllm_unembedding_argmax_workspace_bytes(batch)
    work = scratch_pool.get((max(nbytes // 4, 1),), torch.float32, hidden.device)
    ids = scratch_pool.get((batch,), torch.int32, hidden.device)
    rc = lib().tllm_unembedding_argmax_bf16(x2.data_ptr(), weight.data_ptr(), ws.data_ptr() if ws is not None else None, work.data_ptr(),
                                            work.numel() * 4, ids.data_ptr(), batch, hidden_size, vocab_size, _stream())
    check(rc, "unembedding_decode_argmax_forward")
    return ids


def unembedding_decode_argmax_noalloc(hidden: torch.Tensor, weight: torch.Tensor, token_ids: torch.Tensor,
                                      weight_scale: torch.Tensor | None = None) -> torch.Tensor:
    """``unembedding_decode_argmax_forward`` for callers that must not allocate: the caller passes ``token_ids``
    (int32 ``[B]``), the candidates go through a device array the library owns, and nothing is taken from the scratch
    pool or from PyTorch's allocator. At most ``tllm_unembedding_argmax_noalloc_max_rows()`` (16) batch rows. Calls on
    one GPU share that array: do not overlap them on different streams. A caller that captures this call in a graph
    runs ``unembedding_decode_argmax_noalloc_init()`` on the device first (the library looks the array's address up
    once per device, which a capturing stream does not allow). No counterpart in the reference."""
    x2, weight, ws, batch, hidden_size, vocab_size = _unembed_prep(hidden, weight, weight_scale)
    _on_gpu(token_ids)
    # the kernel writes token_ids[0 .. batch): checked with exceptions, which `python -O` keeps
    if token_ids.dtype != torch.int32 or tuple(token_ids.shape) != (batch,) or not token_ids.is_contiguous():
        raise ValueError(f"token_ids must be a contiguous int32 tensor of shape ({batch},), got {token_ids.dtype} {tuple(token_ids.shape)}")
    rc = lib().tllm_unembedding_argmax_noalloc_bf16(x2.data_ptr(), weight.data_ptr(), ws.data_ptr() if ws is not None else None,
                                                    token_ids.data_ptr(), batch, hidden_size, vocab_size, _stream())
    check(rc, "unembedding_decode_argmax_noalloc")
    return token_ids


def unembedding_decode_argmax_noalloc_init(device=None) -> None:
    """Look up the library-owned candidate array of ``unembedding_decode_argmax_noalloc`` on ``device`` (default: the
    current one). Call once per device, outside any stream capture, before capturing that op in a graph."""
    with torch.cuda.device(device if device is not None else torch.cuda.current_device()):
        check(lib().tllm_unembedding_argmax_noalloc_init(), "unembedding_decode_argmax_noalloc_init")


def unembedding_forward(hidden: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """triton_kernels.py:515-525: the stream kernel for one bf16 token per batch row on the GPU, the library GEMM otherwise."""
    if hidden.is_cuda and hidden.ndim == 3 and hidden.shape[1] == 1 and hidden.dtype == _BF16 and weight.dtype == _BF16:
        return unembedding_decode_forward(hidden, weight)
    return torch.nn.functional.linear(hidden, weight, bias=None)


def unembedding_decode_fp8_argmax_forward(hidden, weight_fp8, weight_scale):
    """triton_kernels.py:470-512."""
    return unembedding_decode_argmax_forward(hidden, weight_fp8, weight_scale)


# --------------------------------------------------------------------------------------- decode attention
def attention_decode(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, sinks: torch.Tensor | None, sm_scale: float,
                     bandwidth: int | None, start_q: torch.Tensor, kv_len_hint: int | None = None) -> torch.Tensor:
    """One new token per batch row against the KV cache, with sinks and an optional sliding window
    (attention_tt_decode.py:290-408): ``q [bs, 1, n_kv_heads, repeat_kv, 64]``, ``k, v [bs, n_kv_ctx, n_kv_heads, 64]``,
    ``sinks [n_kv_heads * repeat_kv]`` bf16, ``start_q`` a device tensor of one int32/int64 element (read on the
    device), ``bandwidth`` the sliding window (``None`` / 0: none). Returns ``[bs, 1, n_heads * 64]`` (pooled).

    ``k`` / ``v`` are usually the whole preallocated cache; the launch is planned from its size and the kernels then use
    only the splits the context at ``start_q`` needs. ``kv_len_hint`` (an extension; the host's idea of how many keys
    are visible, e.g. the decode loop's position + 1) plans the launch for that length instead, which is faster when
    the context is far shorter than the cache; the result never depends on it."""
    _on_gpu(q, k, v, sinks, start_q)
    _require(len(start_q) == 1 and start_q.dtype in (torch.int32, torch.int64))
    bs, n_ctx, n_kv_heads, repeat_kv, head_dim_q = q.shape
    bs_k, n_kv_ctx, n_kv_heads_k, head_dim_k = k.shape
    bs_v, n_kv_ctx_v, n_kv_heads_v, head_dim_v = v.shape
    _require(n_ctx == 1)
    _require(bs == bs_k == bs_v and n_kv_ctx == n_kv_ctx_v)
    _require(n_kv_heads == n_kv_heads_k == n_kv_heads_v)
    _require(head_dim_q == head_dim_k == head_dim_v)
    _require(head_dim_q in {16, 32, 64, 128, 256})
    if head_dim_q != 64 or repeat_kv > 16:
        raise NotImplementedError("attention_decode: the HIP kernel is built for head_dim 64 and up to 16 query heads per KV head")
    _require(q.dtype == _BF16 and k.dtype == _BF16 and v.dtype == _BF16 and (sinks is None or sinks.dtype == _BF16))
    n_heads = n_kv_heads * repeat_kv
    q2 = q[:, 0].reshape(bs, n_heads * 64)
    if not q2.is_contiguous():
        q2 = q2.contiguous()

    def dense_heads(t):
        return t if (t.stride(3) == 1 and t.stride(2) == 64 and t.stride(1) % 8 == 0 and t.stride(0) % 8 == 0) else t.contiguous()

    k, v = dense_heads(k), dense_heads(v)
    if k.stride() != v.stride():
        k, v = k.contiguous(), v.contiguous()
    if sinks is not None:
        _require(sinks.shape == (n_heads,))
        sinks = sinks if sinks.is_contiguous() else sinks.contiguous()
    window = int(bandwidth) if bandwidth else 0
    o = scratch_pool.get((bs, n_heads * 64), q.dtype, q.device)
    hint = 0 if kv_len_hint is None else max(int(kv_len_hint), 1)
    plan_ctx = min(hint, n_kv_ctx) if hint else n_kv_ctx
    nbytes = lib().tllm_attention_decode_workspace_bytes(bs, n_heads, n_kv_heads, plan_ctx, window)
    work = scratch_pool.get((max(nbytes // 4, 1),), torch.float32, q.device) if nbytes else None
    rc = lib().tllm_attention_decode_bf16(q2.data_ptr(), k.data_ptr(), v.data_ptr(), sinks.data_ptr() if sinks is not None else None,
                                          o.data_ptr(), q2.stride(0), o.stride(0), k.stride(0), k.stride(1), bs, n_kv_ctx, n_kv_heads,
                                          repeat_kv, 64, float(sm_scale), window, start_q.data_ptr(), int(start_q.dtype == torch.int64),
                                          hint, work.data_ptr() if work is not None else None, nbytes, _stream())
    check(rc, "attention_decode")
    return o.view(bs, 1, n_heads * 64)


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, sinks: torch.Tensor | None, sm_scale: float,
              bandwidth: int | None, start_q: torch.Tensor) -> torch.Tensor:
    """Prefill attention with sinks and an optional sliding window (attention, attention_tt.py:167-242):
    ``q [bs, n_ctx, n_kv_heads, repeat_kv, 64]``, ``k, v [bs, n_kv_ctx, n_kv_heads, 64]``, ``sinks [n_heads]`` bf16,
    ``start_q`` a device tensor of one int32/int64 element (query ``i`` sits at position ``start_q + i``; read on the
    device), ``bandwidth`` the sliding window (``None`` / 0: none). Returns ``[bs, n_ctx, n_heads * 64]`` (pooled).

    ``q`` may be a view into the fused QKV output and ``k`` / ``v`` views of the cache: the kernel takes batch and
    token strides, so none of the reference's transposed, padded copies (:180-191) is made."""
    _on_gpu(q, k, v, sinks, start_q)
    _require(len(start_q) == 1 and start_q.dtype in (torch.int32, torch.int64))
    bs, n_ctx, n_kv_heads, repeat_kv, head_dim_q = q.shape
    bs_k, n_kv_ctx, n_kv_heads_k, head_dim_k = k.shape
    bs_v, n_kv_ctx_v, n_kv_heads_v, head_dim_v = v.shape
    _require(bs == bs_k == bs_v and n_kv_ctx == n_kv_ctx_v)
    _require(n_kv_heads == n_kv_heads_k == n_kv_heads_v)
    _require(head_dim_q == head_dim_k == head_dim_v)
    _require(head_dim_q in {16, 32, 64, 128, 256})
    if head_dim_q != 64:
        raise NotImplementedError("attention: the HIP kernel is built for head_dim 64")
    _require(q.dtype == _BF16 and k.dtype == _BF16 and v.dtype == _BF16 and (sinks is None or sinks.dtype == _BF16))
    n_heads = n_kv_heads * repeat_kv

    def dense_q(t):
        ok = t.stride(4) == 1 and t.stride(3) == 64 and t.stride(2) == 64 * repeat_kv and t.stride(1) % 8 == 0 and t.stride(0) % 8 == 0
        return t if ok and t.data_ptr() % 16 == 0 else t.contiguous()

    def dense_heads(t):
        ok = t.stride(3) == 1 and t.stride(2) == 64 and t.stride(1) % 8 == 0 and t.stride(0) % 8 == 0
        return t if ok and t.data_ptr() % 16 == 0 else t.contiguous()

    q = dense_q(q)
    k, v = dense_heads(k), dense_heads(v)
    if k.stride() != v.stride():
        k, v = k.contiguous(), v.contiguous()
    if sinks is not None:
        _require(sinks.shape == (n_heads,))
        sinks = sinks if sinks.is_contiguous() else sinks.contiguous()
    window = int(bandwidth) if bandwidth else 0
    o = scratch_pool.get((bs, n_ctx, n_heads * 64), q.dtype, q.device)
    rc = lib().tllm_attention_prefill_bf16(q.data_ptr(), k.data_ptr(), v.data_ptr(), sinks.data_ptr() if sinks is not None else None,
                                           o.data_ptr(), q.stride(0), q.stride(1), o.stride(0), o.stride(1), k.stride(0), k.stride(1),
                                           bs, n_ctx, n_kv_ctx, n_kv_heads, repeat_kv, 64, float(sm_scale), window, start_q.data_ptr(),
                                           int(start_q.dtype == torch.int64), _stream())
    check(rc, "attention")
    return o


def mxfp4_dequant(blocks: torch.Tensor, scales: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """Expand MXFP4 checkpoint data to bf16 (Checkpoint._get_mxfp4_tensor, weights.py:68-117).

    ``blocks`` uint8 ``[..., G, 16]`` holds 32 e2m1 values per 16 bytes, low nibble first; ``scales`` uint8
    ``[..., G]`` holds the shared power-of-two exponent, biased by 127. Returns ``[..., G * 32]`` bf16; ``out``, if
    given, must be a contiguous bf16 tensor of that many elements (it is filled in place, so a caller can expand
    straight into a slice of a preallocated parameter)."""
    _on_gpu(blocks, scales, out)
    _require(blocks.dtype == torch.uint8 and scales.dtype == torch.uint8, "MXFP4 blocks and scales are uint8")
    _require(blocks.shape[:-1] == scales.shape, f"{blocks.shape=} does not match {scales.shape=}")
    _require(blocks.shape[-1] == 16, "an MXFP4 block is 16 bytes")
    *prefix, G, B = blocks.shape
    blocks = blocks.contiguous()
    scales = scales.contiguous()
    n_blocks = scales.numel()
    shape = (*prefix, G * B * 2)
    if out is None:
        out = torch.empty(shape, dtype=_BF16, device=blocks.device)
    else:
        _require(out.dtype == _BF16 and out.is_contiguous() and out.numel() == n_blocks * 32, "out must be contiguous bf16 of 32 values per block")
    check(lib().tllm_mxfp4_dequant_bf16(blocks.data_ptr(), scales.data_ptr(), out.data_ptr(), n_blocks, _stream()), "mxfp4_dequant")
    return out.view(shape) if out.shape != torch.Size(shape) else out
