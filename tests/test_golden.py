"""Drift guards: the CPU oracle against the fixtures it wrote earlier (tests/golden/make_golden.py), and -- on the
GPU -- the HIP kernels against the same fixtures. The fixtures are data (inputs by seed, expected outputs as arrays)."""
import os

import numpy as np
import pytest
import torch

from oracle import layers as O

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _load(name):
    return np.load(os.path.join(GOLDEN, name), allow_pickle=False)


def test_oracle_yarn_tables_match_fixture():
    g = _load("yarn_tables.npz")
    conc, inv_freq = O.yarn_concentration_and_inv_freq()
    assert abs(conc - float(g["concentration"])) < 1e-15
    np.testing.assert_array_equal(inv_freq.numpy(), g["inv_freq"])           # fp32 pow/div: the same bits or the tables move
    cos, sin = O.yarn_cos_sin(torch.from_numpy(g["positions"]))
    np.testing.assert_allclose(cos.numpy(), g["cos"], rtol=0, atol=2e-7)      # another libm may differ in the last place
    np.testing.assert_allclose(sin.numpy(), g["sin"], rtol=0, atol=2e-7)


def test_oracle_b1_chain_matches_fixture():
    g = _load("chain_b1.npz")
    d = O.make_inputs(1, swiglu_rows=4, seed=0)
    sums = [float(d[key].double().sum()) for key in ("x", "norm_scale", "w", "b", "swiglu_x")] + [float(d["positions"][0])]
    np.testing.assert_allclose(np.array(sums), g["input_sums"], rtol=1e-12, atol=0, err_msg="the seeded inputs themselves changed")
    t = O.rmsnorm_ref(d["x"], d["norm_scale"].float(), 1e-5)
    q, k, v = O.qkv_rope_ref(t.bfloat16(), d["w"], d["b"], d["positions"])
    np.testing.assert_allclose(t.numpy(), g["normed"], rtol=1e-6, atol=1e-6)
    for got, name in ((q, "q"), (k, "k"), (v, "v")):
        np.testing.assert_allclose(got.numpy(), g[name], rtol=1e-5, atol=2e-5)   # fp32 GEMM: summation order may differ between builds
    np.testing.assert_allclose(O.swiglu_ref(d["swiglu_x"]).numpy(), g["swiglu"], rtol=1e-6, atol=1e-6)


@pytest.mark.gpu
def test_hip_b1_chain_matches_fixture(gpu):
    """The B = 1 configuration on the HIP kernels against the stored oracle outputs, at the path's tolerance."""
    import tritonllm_amd as T

    g = _load("chain_b1.npz")
    d = O.make_inputs(1, swiglu_rows=4, seed=0)
    tol = dict(rtol=1.6e-2, atol=1e-2)
    t = T.rmsnorm_forward(d["x"].to(gpu), d["norm_scale"].to(gpu), 1e-5)
    torch.testing.assert_close(t.float().cpu(), torch.from_numpy(g["normed"]), **tol)
    for fused in (False, True):
        x = d["x"].to(gpu) if fused else t
        q, k, v = T.qkv_rope_forward(x, d["w"].to(gpu), d["b"].to(gpu), 64, 8, 64, yarn=T.gpt_oss_yarn(), positions=d["positions"].to(gpu),
                                     mode="decode", norm_scale=d["norm_scale"].to(gpu) if fused else None)
        for got, name in ((q, "q"), (k, "k"), (v, "v")):
            torch.testing.assert_close(got.float().cpu(), torch.from_numpy(g[name]), **tol)
    torch.testing.assert_close(T.swiglu(d["swiglu_x"].to(gpu)).float().cpu(), torch.from_numpy(g["swiglu"]), **tol)


@pytest.mark.gpu
def test_hip_yarn_rows_match_fixture(gpu):
    import ctypes

    import tritonllm_amd as T
    from tritonllm_amd import _lib

    g = _load("yarn_tables.npz")
    yp = T.gpt_oss_yarn()
    np.testing.assert_array_equal(np.array(yp.inv_freq, dtype=np.float32), g["inv_freq"])
    for i, pos in enumerate(g["positions"].tolist()):
        cos = torch.empty(1, 32, dtype=torch.float32, device=gpu)
        sin = torch.empty(1, 32, dtype=torch.float32, device=gpu)
        rc = _lib.lib().tllm_yarn_table_f32(cos.data_ptr(), sin.data_ptr(), pos, 1, ctypes.byref(yp.c_struct()), torch.cuda.current_stream().cuda_stream)
        assert rc == 0
        np.testing.assert_allclose(cos.cpu().numpy()[0], g["cos"][i], rtol=0, atol=4e-7 * yp.concentration)
        np.testing.assert_allclose(sin.cpu().numpy()[0], g["sin"][i], rtol=0, atol=4e-7 * yp.concentration)
