"""ctypes binding of ``libtllm_hip.so`` (the C ABI declared in ``include/tllm_hip.h``).

There is no fallback: if the shared library has not been built, importing a kernel
entry point raises. Build it with ``python -m tritonllm_amd.build``.
"""
from __future__ import annotations

import ctypes as C
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "lib", "libtllm_hip.so")

MAX_ROPE_FREQS = 128
ABI_VERSION = 1


class TllmYarn(C.Structure):
    _fields_ = [("inv_freq", C.c_float * MAX_ROPE_FREQS), ("concentration", C.c_float), ("n_freq", C.c_int32)]


class TllmRope(C.Structure):
    _fields_ = [
        ("yarn", C.POINTER(TllmYarn)),
        ("cos_table", C.c_void_p),
        ("sin_table", C.c_void_p),
        ("table_row_stride", C.c_int64),
        ("positions", C.c_void_p),
        ("offset", C.c_void_p),
        ("tokens_per_batch", C.c_int64),
        ("max_ctx", C.c_int64),
    ]


_vp, _i64, _i32, _f32 = C.c_void_p, C.c_int64, C.c_int, C.c_float
_QKV_SIG = [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i32, _i32, _i32, C.POINTER(TllmRope), _vp]

# name -> (restype, argtypes); every symbol include/tllm_hip.h declares
SIGNATURES = {
    "tllm_abi_version": (_i32, []),
    "tllm_last_error": (C.c_char_p, []),
    "tllm_rmsnorm_bf16": (_i32, [_vp, _vp, _i32, _vp, _i64, _i64, _f32, _vp]),
    "tllm_embedding_bf16": (_i32, [_vp, _vp, _i32, _vp, _i64, _i64, _i64, _vp, _vp]),
    "tllm_swiglu_bf16": (_i32, [_vp, _vp, _i64, _i64, _i64, _f32, _f32, _i32, _i32, _vp]),
    "tllm_yarn_table_f32": (_i32, [_vp, _vp, _i64, _i64, C.POINTER(TllmYarn), _vp]),
    "tllm_rope_bf16": (_i32, [_vp, _vp, _i64, _i32, _i32, _i32, C.POINTER(TllmRope), _vp]),
    "tllm_qkv_rope_decode_bf16": (_i32, _QKV_SIG),
    "tllm_qkv_rope_prefill_bf16": (_i32, _QKV_SIG),
    "tllm_norm_qkv_rope_decode_bf16": (_i32, [_vp, _vp, _i32, _f32] + _QKV_SIG[1:]),
    "tllm_qkv_decode_wait_expired": (_i32, [_vp]),
    "tllm_embed_norm_qkv_rope_decode_bf16": (_i32, [_vp, _i32, _vp, _i64, _vp, _vp, _vp, _i32, _f32, _vp, _vp] + _QKV_SIG[2:]),
    "tllm_out_residual_decode_bf16": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp]),
    "tllm_unembedding_decode_bf16": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "tllm_unembedding_argmax_workspace_bytes": (_i64, [_i64]),
    "tllm_unembedding_argmax_bf16": (_i32, [_vp, _vp, _vp, _vp, _i64, _vp, _i64, _i64, _i64, _vp]),
    "tllm_unembedding_argmax_noalloc_max_rows": (_i64, []),
    "tllm_unembedding_argmax_noalloc_init": (_i32, []),
    "tllm_unembedding_argmax_noalloc_bf16": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "tllm_attention_decode_splits": (_i32, [_i64, _i32, _i64, _i32]),
    "tllm_attention_decode_heads_per_workgroup": (_i32, [_i64, _i32, _i64, _i32]),
    "tllm_attention_decode_workspace_bytes": (_i64, [_i64, _i32, _i32, _i64, _i32]),
    "tllm_attention_decode_bf16": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i32, _i32, _i32, _f32, _i32, _vp,
                                          _i32, _i64, _vp, _i64, _vp]),
    "tllm_embed_rmsnorm_bf16": (_i32, [_vp, _vp, _i32, _vp, _vp, _i32, _vp, _i64, _i64, _i64, _f32, _vp, _vp]),
    "tllm_attention_prefill_bf16": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i32, _i32, _i32,
                                           _f32, _i32, _vp, _i32, _vp]),
    "tllm_mxfp4_dequant_bf16": (_i32, [_vp, _vp, _vp, _i64, _vp]),
    "tllm_qkv_rope_decode_w8_bf16": (_i32, [_vp, _vp, _i32, _f32, _vp, _vp] + _QKV_SIG[2:]),
}

_lib = None


def lib() -> C.CDLL:
    """Load the shared library once; raise loudly when it is missing or stale."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: the HIP extension is not built (python -m tritonllm_amd.build). "
                "There is no CPU or PyTorch fallback."
            )
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)   # AttributeError if the library does not export it
            fn.restype = res
            fn.argtypes = args
        got = handle.tllm_abi_version()
        if got != ABI_VERSION:
            raise RuntimeError(f"libtllm_hip.so has ABI version {got}, this package expects {ABI_VERSION}: rebuild it")
        _lib = handle
    return _lib


def require(cond, msg: str = "") -> None:
    """The reference's argument checks are `assert` statements (triton_kernels.py:1086-1106 and the other op wrappers); these
    raise the same AssertionError but survive `python -O`, since several of them guard device memory accesses."""
    if not cond:
        raise AssertionError(msg)


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = lib().tllm_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{what} failed (code {rc}): {msg}")
