"""CPU-side checks of the C-ABI boundary: the library loads, exports every symbol the
header declares, and rejects bad arguments on the host before anything is launched."""
import ctypes as C
import os
import re

import pytest
import torch

from tritonllm_amd import _lib
from tritonllm_amd.yarn import YarnParams, gpt_oss_yarn

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _header_symbols():
    text = open(os.path.join(ROOT, "include", "tllm_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tllm_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.lib()
    declared = _header_symbols()
    assert declared, "no declarations parsed"
    assert sorted(_lib.SIGNATURES) == declared
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.tllm_abi_version() == _lib.ABI_VERSION


def test_struct_layout_matches_header():
    assert C.sizeof(_lib.TllmYarn) == 128 * 4 + 4 + 4
    assert C.sizeof(_lib.TllmRope) == 8 * 8


def _err():
    return _lib.lib().tllm_last_error().decode()


def test_argument_errors_are_reported_not_launched():
    lib = _lib.lib()
    assert lib.tllm_rmsnorm_bf16(None, None, 0, None, 4, 2880, 1e-5, None) == -1
    assert "null" in _err()
    assert lib.tllm_rmsnorm_bf16(None, None, 0, None, -1, 2880, 1e-5, None) == -1
    assert lib.tllm_rmsnorm_bf16(None, None, 0, None, 0, 2880, 1e-5, None) == 0     # empty input is a no-op
    assert lib.tllm_embedding_bf16(None, None, 0, None, 0, 2880, 10, None, None) == 0
    assert lib.tllm_embedding_bf16(None, None, 0, None, 3, 2880, 10, None, None) == -1
    assert lib.tllm_swiglu_bf16(None, None, 0, 2880, 5760, 1.702, 7.0, 1, 1, None) == 0
    assert lib.tllm_swiglu_bf16(None, None, 2, 2880, 100, 1.702, 7.0, 1, 1, None) == -1
    assert "x_row_stride" in _err()
    rope = _lib.TllmRope()
    assert lib.tllm_rope_bf16(None, None, 0, 64, 8, 64, C.byref(rope), None) == -1   # no yarn, no tables, max_ctx 0
    y = gpt_oss_yarn()
    rope.yarn = y.c_pointer()
    rope.max_ctx = 131072
    rope.tokens_per_batch = 1
    assert lib.tllm_rope_bf16(None, None, 0, 64, 8, 64, C.byref(rope), None) == 0
    assert lib.tllm_rope_bf16(None, None, 0, 64, 8, 128, C.byref(rope), None) == -2  # head_dim vs yarn.n_freq
    assert "n_freq" in _err()
    assert lib.tllm_rope_bf16(None, None, 0, 64, 8, 63, C.byref(rope), None) == -2
    qkv = lib.tllm_qkv_rope_decode_bf16
    assert qkv(None, None, None, None, None, None, 4096, 512, 512, 0, 8, 2880, 64, 8, 64, None, None) == -1
    assert qkv(None, None, None, None, None, None, 4096, 512, 512, 0, 8, 2880, 64, 8, 63, None, None) == -2
    assert lib.tllm_yarn_table_f32(None, None, 0, 0, None, None) == -1


def test_yarn_params_match_closed_form():
    y = gpt_oss_yarn()
    assert y.concentration == pytest.approx(1.3465735902799727, abs=1e-15)
    assert len(y.inv_freq) == 32 and y.inv_freq[0] == 1.0
    for i in (1, 5, 8):
        assert y.inv_freq[i] == pytest.approx(150000.0 ** (-i / 32), rel=2e-6)
    for i in (18, 25, 31):
        assert y.inv_freq[i] == pytest.approx(150000.0 ** (-i / 32) / 32, rel=2e-6)
    s = y.c_struct()
    assert s.n_freq == 32 and s.inv_freq[3] == torch.tensor(y.inv_freq[3], dtype=torch.float32).item()
    plain = YarnParams(head_dim=128, base=10000.0)
    assert plain.concentration == 1.0 and plain.inv_freq[1] == pytest.approx(10000.0 ** (-2 / 128), rel=2e-6)
    with pytest.raises(ValueError):
        YarnParams(head_dim=63, base=10000.0)


def test_yarn_params_agree_with_oracle_bitwise():
    from oracle import layers as O

    conc, inv = O.yarn_concentration_and_inv_freq()
    y = gpt_oss_yarn()
    assert conc == y.concentration
    assert inv.tolist() == list(y.inv_freq)


def test_ops_refuse_cpu_tensors():
    import tritonllm_amd as T

    x = torch.zeros(2, 2880, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU only"):
        T.rmsnorm_forward(x, torch.ones(2880), 1e-5)
    with pytest.raises(RuntimeError, match="GPU only"):
        T.swiglu(torch.zeros(2, 8, dtype=torch.bfloat16))


def test_scratch_pool_returns_same_buffer():
    from tritonllm_amd import scratch_pool

    scratch_pool.clear()
    a = scratch_pool.get((2, 3), torch.float32, torch.device("cpu"))
    b = scratch_pool.get((2, 3), torch.float32, torch.device("cpu"))
    c = scratch_pool.get((2, 4), torch.float32, torch.device("cpu"))
    assert a.data_ptr() == b.data_ptr() and a.data_ptr() != c.data_ptr()
    assert scratch_pool.stats()["num_buffers"] == 2
    scratch_pool.clear()


def test_checkpoint_names_and_plain_tensors(tmp_path):
    """Host logic of the checkpoint reader (reference weights.py:17-66): key discovery over several files, the MoE
    name mapping, plain tensors on the CPU, and no CPU expansion of MXFP4 data."""
    from safetensors.torch import save_file

    from tritonllm_amd.weights import Checkpoint, _param_names

    assert _param_names("block.0.mlp.mlp1_weight") == ("block.0.mlp.mlp1_weight.blocks", "block.0.mlp.mlp1_weight.scales")
    assert _param_names("block.35.mlp.mlp2_weight") == ("block.35.mlp.mlp2_weight.blocks", "block.35.mlp.mlp2_weight.scales")
    assert _param_names("block.36.mlp.mlp2_weight") == "block.36.mlp.mlp2_weight"       # the reference maps 36 blocks
    assert _param_names("block.3.mlp.mlp1_bias") == "block.3.mlp.mlp1_bias"
    assert _param_names("block.3.attn.qkv.weight") == "block.3.attn.qkv.weight"
    assert _param_names("embedding.weight") == "embedding.weight"

    g = torch.Generator().manual_seed(0)
    a = torch.randn(4, 8, generator=g).bfloat16()
    b = torch.randn(3, generator=g)
    save_file({"embedding.weight": a}, str(tmp_path / "one.safetensors"))
    save_file({"block.0.mlp.mlp1_bias": b,
               "block.0.mlp.mlp1_weight.blocks": torch.zeros(2, 4, 3, 16, dtype=torch.uint8),
               "block.0.mlp.mlp1_weight.scales": torch.full((2, 4, 3), 127, dtype=torch.uint8)}, str(tmp_path / "two.safetensors"))
    (tmp_path / "ignored.txt").write_text("not a tensor file")
    ck = Checkpoint(str(tmp_path), torch.device("cpu"))
    assert sorted(ck.tensor_name_to_file) == ["block.0.mlp.mlp1_bias", "block.0.mlp.mlp1_weight.blocks", "block.0.mlp.mlp1_weight.scales",
                                              "embedding.weight"]
    assert torch.equal(ck.get("embedding.weight"), a)
    assert torch.equal(ck.get("block.0.mlp.mlp1_bias"), b)
    dst = torch.empty(3)
    assert ck.get("block.0.mlp.mlp1_bias", out=dst) is dst and torch.equal(dst, b)
    with pytest.raises(AssertionError, match="not found"):
        ck.get("block.1.mlp.mlp1_bias")
    with pytest.raises(AssertionError, match="not found"):
        ck.get("block.1.mlp.mlp1_weight")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ck.get("block.0.mlp.mlp1_weight")


def test_mxfp4_argument_errors():
    lib = _lib.lib()
    assert lib.tllm_mxfp4_dequant_bf16(None, None, None, 0, None) == 0
    assert lib.tllm_mxfp4_dequant_bf16(None, None, None, 5, None) == -1
    assert lib.tllm_mxfp4_dequant_bf16(None, None, None, -1, None) == -1
    assert lib.tllm_mxfp4_dequant_bf16(C.c_void_p(8), C.c_void_p(1), C.c_void_p(16), 5, None) != 0   # blocks not 16-byte aligned
    assert "aligned" in _err()


def test_attention_prefill_argument_errors():
    """Argument checks of the prefill attention entry point happen before anything touches the GPU."""
    f = _lib.lib().tllm_attention_prefill_bf16
    p = C.c_void_p(4096)

    def call(q=p, k=p, v=p, out=p, q_ts=4096, kv_ts=512, batch=1, n_q=16, n_kv=16, kvh=8, group=8, hd=64, scale=0.125, window=0, start=p):
        return f(q, k, v, None, out, n_q * q_ts, q_ts, n_q * 4096, 4096, n_kv * kv_ts, kv_ts, batch, n_q, n_kv, kvh, group, hd, scale, window,
                 start, 0, None)

    assert call(batch=0) == 0 and call(n_q=0) == 0                      # nothing to do
    assert call(hd=128) != 0 and "head_dim" in _err()
    assert call(scale=0.0) != 0 and "sm_scale" in _err()
    assert call(window=-1) != 0
    assert call(n_kv=0) != 0
    assert call(q=None) != 0 and "NULL" in _err()
    assert call(start=None) != 0
    assert call(k=C.c_void_p(4104)) != 0 and "aligned" in _err()
    assert call(q_ts=4000) != 0                                         # heads do not fit into a token's stride
    assert call(kv_ts=256) != 0


def test_attention_decode_shape_planning():
    """The host-side choice of workgroup shape and splits (no launch): small batches keep one KV head per workgroup."""
    hpw = _lib.lib().tllm_attention_decode_heads_per_workgroup
    splits = _lib.lib().tllm_attention_decode_splits
    assert [hpw(b, 8, 4096, 0) for b in (1, 4)] == [0, 0]
    assert hpw(8, 8, 4096, 0) == 4 and splits(8, 8, 4096, 0) == 16               # splits of 256 keys, few enough of them
    assert hpw(16, 8, 4096, 0) == 4 and splits(16, 8, 4096, 0) == 8
    assert hpw(32, 8, 4096, 0) == 4 and splits(32, 8, 4096, 0) == 4
    assert hpw(8, 8, 32768, 0) == 4 and splits(8, 8, 32768, 0) == 16             # the longer splits win over the wider workgroup
    assert hpw(8, 8, 131072, 0) == 8 and splits(8, 8, 131072, 0) == 32           # ... and the wider one a tie
    assert hpw(12, 8, 20000, 0) == 4 and splits(12, 8, 20000, 0) == 10           # 24 x 10 workgroups rather than 24 x 11 = 264
    assert hpw(3, 8, 4096, 0) == 0 and splits(3, 8, 4096, 0) == 10               # 24 x 10 here as well
    assert hpw(4, 8, 32768, 0) == 4 and splits(4, 8, 32768, 0) == 32
    assert hpw(2, 8, 32768, 0) == 4 and splits(2, 8, 32768, 0) == 64
    assert hpw(2, 8, 16384, 0) == 0
    assert hpw(1, 8, 131072, 0) == 0
    assert hpw(64, 8, 131072, 128) == 0 and splits(64, 8, 131072, 128) == 1      # a sliding window bounds the context
    for b in (1, 3, 8, 100):
        for ctx in (1, 127, 128, 129, 5000, 131072):
            s = splits(b, 8, ctx, 0)
            assert 1 <= s <= 64 and (s == 1 or ctx >= 128 * (s - 1))
