"""Compile the HIP sources into ``tritonllm_amd/lib/libtllm_hip.so`` for gfx950.

``hipcc`` cross-compiles without a GPU, so this runs anywhere the ROCm toolchain
is installed. Usage: ``python -m tritonllm_amd.build``.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_DIR = os.path.join(PKG_DIR, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libtllm_hip.so")
INCLUDE = os.path.join(ROOT, "include")

SOURCES = ["abi.hip", "rmsnorm.hip", "embedding.hip", "swiglu.hip", "rope.hip", "qkv_decode.hip", "qkv_decode_r8.hip", "qkv_decode_r32.hip", "qkv_decode_rows.hip", "qkv_prefill.hip", "out_decode.hip", "out_decode_r8.hip", "out_decode_r32.hip", "unembed.hip", "attn_decode.hip", "attn_prefill.hip", "mxfp4.hip"]

# -packed-fp32-ops: keep the compiler from forming v_pk_*_f32 from ordinary float code.
HIPCC_FLAGS = [
    "-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
] + os.environ.get("TLLM_EXTRA_HIPCC_FLAGS", "").split()


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the ROCm toolchain is required to build libtllm_hip.so")
    return exe


def _compile(src: str, obj_dir: str) -> str:
    obj = os.path.join(obj_dir, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, "-I", INCLUDE, "-I", CSRC, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{r.stdout}\n{r.stderr}")
    return obj


def build_library(verbose: bool = False) -> str:
    obj_dir = os.path.join(PKG_DIR, "build")
    os.makedirs(obj_dir, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(lambda s: _compile(s, obj_dir), SOURCES))
    tmp = LIB_PATH + ".tmp"
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH} ({os.path.getsize(LIB_PATH)} bytes)")
    return LIB_PATH


if __name__ == "__main__":
    build_library(verbose=True)
    sys.exit(0)
