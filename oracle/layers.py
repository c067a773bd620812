"""CPU oracle: a plain-PyTorch restatement of the reference's gpt-oss layer ops.

TEST INFRASTRUCTURE ONLY -- imported by ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py``; the product package never imports
it and has no CPU fallback.

Two families live here:

* ``*_ref``   -- the *fp32-upcast* closed forms the bf16 kernels are judged
  against (rtol 1.6e-2 / atol 1e-2), and the bit-exact gather.
* ``*_eager`` -- the reference's own eager torch op chain in the tensors' own
  dtype (bf16), which is what the reference would run on a CPU; used only as
  the timed CPU baseline and as a looser cross-check.

Each function cites the reference lines it restates (paths relative to the
reference checkout, ``tritonllm/gpt_oss/triton/...`` unless stated).

Pinning status: the reference ships no test, fixture or golden vector for any
function on this path, so parity with the reference's *implementation* is
pinned only through mathematics -- closed forms, invariants, float64 brute
force and special cases -- in ``tests/test_oracle_pins.py``:

    yarn_concentration_and_inv_freq   closed-form constants, band structure
    yarn_cos_sin                      float64 recomputation, position 0
    rmsnorm_ref                       float64 brute force, scale/constant-row invariants
    embedding_ref                     index_select equality
    linear_ref                        float64 brute force, one-hot selector rows
    rope_rotate_ref                   norm preservation, relative-position property,
                                      additivity, textbook RoPE at scaling_factor=1,
                                      half-split (not interleaved) layout
    qkv_rope_ref                      composition of the above, v slice un-rotated
    swiglu_ref                        float64 brute force, edge grid, l=-1 => 0,
                                      interleaved == chunked under permutation
    attention_decode_ref              float64 brute force per head, causal / window key ranges, sink limits
                                      (-> -inf: plain softmax; -> +inf: zero output), equal keys => mean of values
    attention_ref                     every query row equals attention_decode_ref at position start_q + i; float64 brute
                                      force with a window and a key count below the last position; no visible key => 0
    out_residual_ref                  linear_ref + an fp32 add; float64 brute force
    quantize_fp8_rows_ref /           all 256 e4m3 codes against the OCP bit formula, row maxima map to
    dequant_fp8_ref                   +-448, round-trip error within half a step of the format
    mxfp4_dequant_ref                 every (byte, scale) pair against the e2m1 bit formula times an exact power of
                                      two in float64, torch.ldexp on the looked-up bf16 table, nibble order by
                                      planted bytes, the reference's second formulation (stack + view interleave)

The third-party arithmetic underneath (torch.cos/sin/pow/rsqrt, F.linear) is
PyTorch's, un-pinned by the reference (its README leaves torch unversioned);
no reference test covers those call sites, so against the reference's own
binaries this path stays "parity unpinned" beyond the stated tolerance.
"""
from __future__ import annotations

import math

import torch

# gpt-oss-20b defaults, model.py:36-53
HIDDEN = 2880
HEAD_DIM = 64
N_Q_HEADS = 64
N_KV_HEADS = 8
VOCAB = 201088
ROPE_THETA = 150000.0
ROPE_SCALING = 32.0
ROPE_NTK_ALPHA = 1.0
ROPE_NTK_BETA = 32.0
INITIAL_CTX = 4096
MAX_CTX = 131072
SWIGLU_ALPHA = 1.702
SWIGLU_LIMIT = 7.0
RMS_EPS = 1e-5


# --------------------------------------------------------------------------- YaRN
def yarn_concentration_and_inv_freq(
    head_dim: int = HEAD_DIM,
    base: float = ROPE_THETA,
    initial_context_length: int = INITIAL_CTX,
    scaling_factor: float = ROPE_SCALING,
    ntk_alpha: float = ROPE_NTK_ALPHA,
    ntk_beta: float = ROPE_NTK_BETA,
) -> tuple[float, torch.Tensor]:
    """model.py:267-305 (RotaryEmbedding._compute_concentration_and_inv_freq).

    Same torch fp32 ops in the same order, on the CPU.
    """
    freq = base ** (torch.arange(0, head_dim, 2, dtype=torch.float) / head_dim)
    if scaling_factor > 1.0:
        concentration = 0.1 * math.log(scaling_factor) + 1.0
        d_half = head_dim / 2
        low = d_half * math.log(initial_context_length / (ntk_beta * 2 * math.pi)) / math.log(base)
        high = d_half * math.log(initial_context_length / (ntk_alpha * 2 * math.pi)) / math.log(base)
        assert 0 < low < high < d_half - 1
        interpolation = 1.0 / (scaling_factor * freq)
        extrapolation = 1.0 / freq
        ramp = (torch.arange(d_half, dtype=torch.float32) - low) / (high - low)
        mask = 1 - ramp.clamp(0, 1)
        inv_freq = interpolation * (1 - mask) + extrapolation * mask
    else:
        concentration = 1.0
        inv_freq = 1.0 / freq
    return concentration, inv_freq


def yarn_cos_sin(positions: torch.Tensor, **yarn) -> tuple[torch.Tensor, torch.Tensor]:
    """model.py:307-313 (_compute_cos_sin) evaluated at arbitrary integer positions.

    angle = fp32(position) * inv_freq as one fp32 product (the reference's
    einsum "i,j->ij"); cos/sin in fp32, then scaled by the concentration.
    Returns fp32 ``[n, head_dim/2]`` each.
    """
    concentration, inv_freq = yarn_concentration_and_inv_freq(**yarn)
    t = positions.to(torch.float32)
    freqs = torch.einsum("i,j->ij", t, inv_freq)
    return freqs.cos() * concentration, freqs.sin() * concentration


def token_positions(batch: int, tokens: int, offset: int, max_ctx: int = MAX_CTX) -> torch.Tensor:
    """triton_kernels.py:57-59: every batch row uses (t + offset) % max_ctx."""
    pos = (torch.arange(tokens, dtype=torch.int64) + int(offset)) % max_ctx
    return pos.repeat(batch)


# --------------------------------------------------------------------------- fp32-upcast oracles
def rmsnorm_ref(x: torch.Tensor, scale: torch.Tensor, eps: float = RMS_EPS) -> torch.Tensor:
    """model.py:55-68 / triton_kernels.py:9-35 as the fp32 closed form.

    y = x * rsqrt(mean(x^2) + eps) * scale with everything upcast to fp32 (the
    Triton kernel's habit of squaring in bf16 is a quirk, not the contract).
    Returns fp32.
    """
    t = x.to(torch.float32)
    ms = t.pow(2).mean(dim=-1, keepdim=True)
    return t * torch.rsqrt(ms + eps) * scale.to(torch.float32)


def embedding_ref(table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
    """model.py:906-908, 920 (torch.nn.Embedding forward): a row gather."""
    return torch.index_select(table, 0, ids.reshape(-1).to(torch.int64)).reshape(*ids.shape, table.shape[1])


def linear_ref(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None) -> torch.Tensor:
    """model.py:136-138 (F.linear) on fp32-upcast operands. Returns fp32."""
    out = x.to(torch.float32) @ weight.to(torch.float32).t()
    if bias is not None:
        out = out + bias.to(torch.float32)
    return out


def out_residual_ref(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, residual: torch.Tensor | None) -> torch.Tensor:
    """triton_kernels.py:1470-1517 (kernel :1340-1416, reduce :1419-1467): ``x @ W.T + bias + residual`` with every
    operand upcast to fp32 (pass the dequantised weight for the fp8 form). Returns fp32."""
    out = linear_ref(x, weight, bias)
    if residual is not None:
        out = out + residual.to(torch.float32)
    return out


def attention_decode_ref(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, sinks: torch.Tensor | None, sm_scale: float = 0.125,
                         sliding_window: int | None = None, start_q: int = 0) -> torch.Tensor:
    """attention_ref.py:4-42 for one query position (the decode case), fp32, returned as fp32 ``[bs, 1, heads*hd]``.

    query ``[bs, 1, kv_heads, groups, hd]``, key/value ``[bs, n_keys, kv_heads, hd]``, sinks ``[kv_heads*groups]``
    (``None``: logit 0 for every head, attention_tt_decode.py:55-58). Keys after position ``start_q`` are masked
    (:20-23), keys older than ``start_q - sliding_window + 1`` too (:25-27); the sink joins the softmax
    denominator but contributes no value (:32-37)."""
    bs, nq, n_kv, groups, hd = query.shape
    n_keys = key.shape[1]
    assert nq == 1
    sink = torch.zeros(n_kv * groups) if sinks is None else sinks.to(torch.float32)
    sink = sink.view(1, n_kv, groups, 1)
    pos = torch.arange(n_keys)
    masked = pos > start_q
    if sliding_window:
        masked = masked | (pos < start_q - sliding_window + 1)
    logits = torch.einsum("bhmd,bkhd->bhmk", query[:, 0].to(torch.float32), key.to(torch.float32)) * sm_scale
    logits = logits.masked_fill(masked[None, None, None, :], float("-inf"))
    top = torch.maximum(sink, logits.max(dim=-1, keepdim=True).values)
    w = torch.exp(logits - top)
    z = w.sum(dim=-1, keepdim=True) + torch.exp(sink - top)
    out = torch.einsum("bhmk,bkhd->bhmd", w / z, value.to(torch.float32))
    return out.reshape(bs, 1, n_kv * groups * hd)


def attention_ref(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, sinks: torch.Tensor | None, sm_scale: float = 0.125,
                  sliding_window: int | None = None, start_q: int = 0) -> torch.Tensor:
    """attention_ref.py:4-42 for any number of query positions (the prefill case), fp32, returned as fp32
    ``[bs, n_queries, heads*hd]``.

    query ``[bs, n_queries, kv_heads, groups, hd]``, key/value ``[bs, n_keys, kv_heads, hd]``, sinks ``[kv_heads*groups]``
    (``None``: logit 0, attention_tt.py:100-104). Query ``i`` sits at position ``start_q + i`` (:21); keys after that
    position are masked (:22-23), keys older than ``position - sliding_window + 1`` too (:25-27); the sink joins the
    softmax denominator but contributes no value (:31-37). A query that sees no key yields zeros."""
    bs, nq, n_kv, groups, hd = query.shape
    n_keys = key.shape[1]
    sink = torch.zeros(n_kv * groups) if sinks is None else sinks.to(torch.float32)
    sink = sink.view(1, n_kv, groups, 1, 1)
    pos_k = torch.arange(n_keys)
    pos_q = torch.arange(nq) + int(start_q)
    masked = pos_k[None, :] > pos_q[:, None]
    if sliding_window:
        masked = masked | (pos_k[None, :] < pos_q[:, None] - sliding_window + 1)
    logits = torch.einsum("bqhmd,bkhd->bhmqk", query.to(torch.float32), key.to(torch.float32)) * sm_scale
    logits = logits.masked_fill(masked[None, None, None, :, :], float("-inf"))
    top = torch.maximum(sink, logits.max(dim=-1, keepdim=True).values)
    w = torch.exp(logits - top)
    z = w.sum(dim=-1, keepdim=True) + torch.exp(sink - top)
    out = torch.einsum("bhmqk,bkhd->bqhmd", w / z, value.to(torch.float32))
    return out.reshape(bs, nq, n_kv * groups * hd)


def quantize_fp8_rows_ref(weight: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """triton_kernels.py:261-268 (``_quantize_unembed_fp8``): per-row e4m3 quantisation.

    scale[n] = max_k |W[n,k]| / 448 (fp32, floor 1e-12); W8 = fp8_e4m3fn(W / scale). Returns
    (W8 ``[n, k]`` float8_e4m3fn, scale ``[n]`` fp32)."""
    w = weight.to(torch.float32)
    max_fp8 = torch.finfo(torch.float8_e4m3fn).max
    amax = w.abs().max(dim=1, keepdim=True).values.clamp(min=1e-12)
    scale = (amax / max_fp8).squeeze(1).to(torch.float32)
    w8 = (w / scale[:, None].clamp(min=1e-12)).to(torch.float8_e4m3fn)
    return w8, scale


def dequant_fp8_ref(w8: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """triton_kernels.py:963-965: the weight the fp8 kernels multiply with, ``fp32(W8) * scale[row]``. fp32."""
    return w8.to(torch.float32) * scale.to(torch.float32)[:, None]


def rope_rotate_ref(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """triton_kernels.py:72-88 / model.py:315-327: half-split rotation in fp32.

    x ``[n, heads, head_dim]`` (any float dtype), cos/sin fp32 ``[n, head_dim/2]``.
    Pairs are (d, d + head_dim/2). Returns fp32.
    """
    xf = x.to(torch.float32)
    x1, x2 = torch.chunk(xf, 2, dim=-1)
    c = cos[:, None, :]
    s = sin[:, None, :]
    return torch.cat((x1 * c - x2 * s, x2 * c + x1 * s), dim=-1)


def qkv_rope_ref(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: torch.Tensor,
    positions: torch.Tensor,
    n_q_heads: int = N_Q_HEADS,
    n_kv_heads: int = N_KV_HEADS,
    head_dim: int = HEAD_DIM,
    round_qkv_first: bool = False,
    **yarn,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """QKV projection + bias + YaRN rotary on q/k, fp32.

    ``round_qkv_first=False`` follows the fused decode path, which rotates the
    fp32 accumulator (triton_kernels.py:1029-1054); ``True`` follows the
    prefill path, which rounds the F.linear result to bf16 before rope_forward
    (model.py:506-522). x ``[rows, hidden]``; returns fp32 q ``[rows, n_q*hd]``,
    k ``[rows, n_kv*hd]`` (both rotated) and v ``[rows, n_kv*hd]`` (untouched).
    """
    rows = x.shape[0]
    qkv = linear_ref(x, weight, bias)
    if round_qkv_first:
        qkv = qkv.to(torch.bfloat16).to(torch.float32)
    q_dim, kv_dim = n_q_heads * head_dim, n_kv_heads * head_dim
    q, k, v = torch.split(qkv, (q_dim, kv_dim, kv_dim), dim=-1)
    cos, sin = yarn_cos_sin(positions, head_dim=head_dim, **yarn)
    q = rope_rotate_ref(q.reshape(rows, n_q_heads, head_dim), cos, sin).reshape(rows, q_dim)
    k = rope_rotate_ref(k.reshape(rows, n_kv_heads, head_dim), cos, sin).reshape(rows, kv_dim)
    return q, k, v.contiguous()


def swiglu_ref(
    x: torch.Tensor, alpha: float = SWIGLU_ALPHA, limit: float | None = SWIGLU_LIMIT, interleaved: bool = True
) -> torch.Tensor:
    """moe.py:25-33 / triton_kernels/swiglu.py:89-100 on fp32-upcast input.

    gate = even columns (or first half), linear = odd columns (or second half);
    gate clamped from above only, linear clamped both sides;
    out = gate * sigmoid(alpha * gate) * (linear + 1). Returns fp32.
    """
    xf = x.to(torch.float32)
    if interleaved:
        g, l = xf[..., ::2], xf[..., 1::2]
    else:
        g, l = torch.chunk(xf, 2, dim=-1)
    if limit is not None:
        g = g.clamp(min=None, max=limit)
        l = l.clamp(min=-limit, max=limit)
    return g * torch.sigmoid(alpha * g) * (l + 1)


# --------------------------------------------------------------------------- eager twins (CPU baseline)
def rmsnorm_eager(x: torch.Tensor, scale: torch.Tensor, eps: float = RMS_EPS) -> torch.Tensor:
    """The torch RMSNorm the reference family uses on CPU: fp32 inside, cast back (model.py:55-68)."""
    t = x.float()
    t = t * torch.rsqrt(torch.mean(t**2, dim=-1, keepdim=True) + eps)
    return (t * scale).to(x.dtype)


def qkv_rope_eager(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: torch.Tensor,
    cos_table: torch.Tensor,
    sin_table: torch.Tensor,
    positions: torch.Tensor,
    n_q_heads: int = N_Q_HEADS,
    n_kv_heads: int = N_KV_HEADS,
    head_dim: int = HEAD_DIM,
):
    """model.py:506-522 with the torch `_rotate` twin (model.py:315-327): bf16 F.linear,
    split + contiguous, cos/sin rows looked up in the fp32 tables and cast to bf16."""
    rows = x.shape[0]
    qkv = torch.nn.functional.linear(x, weight, bias)
    q_dim, kv_dim = n_q_heads * head_dim, n_kv_heads * head_dim
    q, k, v = torch.split(qkv, (q_dim, kv_dim, kv_dim), dim=-1)
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    cos = cos_table[positions][:, None, :].to(x.dtype)
    sin = sin_table[positions][:, None, :].to(x.dtype)

    def rot(t, heads):
        t = t.view(rows, heads, head_dim)
        x1, x2 = torch.chunk(t, 2, dim=-1)
        return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin), dim=-1).view(rows, heads * head_dim)

    return rot(q, n_q_heads), rot(k, n_kv_heads), v


def swiglu_eager(x: torch.Tensor, alpha: float = SWIGLU_ALPHA, limit: float = SWIGLU_LIMIT, interleaved: bool = True):
    """moe.py:25-33 verbatim semantics in the input dtype."""
    if interleaved:
        x_glu, x_linear = x[..., ::2], x[..., 1::2]
    else:
        x_glu, x_linear = torch.chunk(x, 2, dim=-1)
    x_glu = x_glu.clamp(min=None, max=limit)
    x_linear = x_linear.clamp(min=-limit, max=limit)
    out_glu = x_glu * torch.sigmoid(alpha * x_glu)
    return out_glu * (x_linear + 1)


def embedding_eager(table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
    """model.py:920: torch.nn.functional.embedding."""
    return torch.nn.functional.embedding(ids.to(torch.int64), table)


# --------------------------------------------------------------------------- seeded inputs shared by tests / bench
def make_inputs(rows: int, swiglu_rows: int = 0, seed: int = 0, hidden: int = HIDDEN, norm_scale_dtype=torch.bfloat16,
                n_q_heads: int = N_Q_HEADS, n_kv_heads: int = N_KV_HEADS, head_dim: int = HEAD_DIM,
                prefill: bool = False, max_pos: int = 8192) -> dict:
    """Synthetic inputs of the benchmark configurations: everything drawn in fp32
    from a seeded CPU generator, then rounded to bf16."""
    g = torch.Generator().manual_seed(seed)
    qkv_dim = (n_q_heads + 2 * n_kv_heads) * head_dim
    d = {
        "x": torch.randn(rows, hidden, generator=g).bfloat16(),
        "norm_scale": (1 + 0.1 * torch.randn(hidden, generator=g)).to(norm_scale_dtype),
        "w": (0.02 * torch.randn(qkv_dim, hidden, generator=g)).bfloat16(),
        "b": (0.02 * torch.randn(qkv_dim, generator=g)).bfloat16(),
    }
    if prefill:
        d["positions"] = torch.arange(rows, dtype=torch.int64)
    else:
        d["positions"] = torch.randint(0, max_pos, (rows,), generator=g, dtype=torch.int64)
    if swiglu_rows:
        d["swiglu_x"] = (2.0 * torch.randn(swiglu_rows, 2 * hidden, generator=g)).bfloat16()
    return d


# ---- MXFP4 checkpoint expansion (weights.py:11-14, 68-117) ----------------------------------------------------------

FP4_VALUES = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0)


def mxfp4_dequant_ref(blocks: torch.Tensor, scales: torch.Tensor) -> torch.Tensor:
    """Checkpoint._get_mxfp4_tensor (weights.py:68-117): blocks uint8 [..., G, B], scales uint8 [..., G] ->
    bf16 [..., G * B * 2]. Byte k of a block gives element 2k from its low nibble and 2k+1 from its high nibble
    (weights.py:105-110); each element is table[nibble] * 2^(scale - 127) (weights.py:86, 112). The reference forms
    the product with torch.ldexp on a bf16 tensor, which multiplies by pow(2.0, e) in fp32 and rounds once to bf16;
    the same two steps are written out here."""
    assert blocks.dtype == torch.uint8 and scales.dtype == torch.uint8
    assert blocks.shape[:-1] == scales.shape
    *prefix, G, B = blocks.shape
    lut = torch.tensor(FP4_VALUES, dtype=torch.float32)
    b = blocks.reshape(-1, B).to(torch.int64)
    vals = torch.empty(b.shape[0], 2 * B, dtype=torch.float32)
    vals[:, 0::2] = lut[b & 0x0F]
    vals[:, 1::2] = lut[b >> 4]
    e = scales.reshape(-1, 1).to(torch.int32) - 127
    p = torch.pow(torch.tensor(2.0, dtype=torch.float32), e.to(torch.float32))   # fp32: denormal below -126, inf at 128
    return (vals * p).to(torch.bfloat16).reshape(*prefix, G * B * 2)
