"""MI355X-native gpt-oss layer kernels: RMSNorm, fused QKV + bias + YaRN rotary,
clamped SwiGLU and the token-embedding gather, as hand-written HIP for gfx950 behind a
C ABI (``include/tllm_hip.h``) with the reference model's Python call signatures on top."""
from . import scratch_pool
from .modules import OUT, QKV, Embedding, RMSNorm, RotaryEmbedding, UnEmbedding
from .ops import (
    attention,
    attention_decode,
    embed_qkv_rope_forward,
    embedding_forward,
    embedding_rmsnorm_forward,
    linear_qkv_forward,
    mxfp4_dequant,
    out_residual_decode_forward,
    qkv_decode_forward,
    qkv_rope_cache_decode_forward,
    qkv_rope_forward,
    quantize_fp8_rows,
    rmsnorm_forward,
    rope_forward,
    swiglu,
    unembedding_decode_argmax_forward,
    unembedding_decode_argmax_noalloc,
    unembedding_decode_argmax_noalloc_init,
    unembedding_decode_forward,
    unembedding_decode_fp8_argmax_forward,
    unembedding_decode_fp8_forward,
    unembedding_forward,
)
from .weights import Checkpoint
from .yarn import YarnParams, gpt_oss_yarn

__all__ = [
    "Checkpoint", "OUT", "QKV", "Embedding", "RMSNorm", "RotaryEmbedding", "YarnParams", "gpt_oss_yarn", "scratch_pool",
    "attention", "attention_decode", "embed_qkv_rope_forward", "embedding_forward", "embedding_rmsnorm_forward", "linear_qkv_forward", "mxfp4_dequant", "out_residual_decode_forward", "qkv_decode_forward", "qkv_rope_cache_decode_forward",
    "qkv_rope_forward", "quantize_fp8_rows", "rmsnorm_forward", "rope_forward", "swiglu", "UnEmbedding", "unembedding_decode_forward", "unembedding_decode_argmax_forward", "unembedding_decode_argmax_noalloc", "unembedding_decode_argmax_noalloc_init",
    "unembedding_decode_fp8_forward", "unembedding_decode_fp8_argmax_forward", "unembedding_forward",
]
