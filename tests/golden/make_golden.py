#!/usr/bin/env python3
"""Writes the drift-guard fixtures of this directory from the repository's own CPU oracle (oracle/layers.py).

They pin nothing against the reference -- the reference ships no vectors for this path -- but they freeze what the
oracle produced when they were made, so that a change of the PyTorch build under the tests (its cos/sin/pow, its
seeded random streams, its bf16 rounding) shows up as a failing CPU test instead of silently moving every parity
target. Run from the repository root:  python tests/golden/make_golden.py

    yarn_tables.npz   inv_freq[32] and the concentration of the gpt-oss YaRN configuration; cos/sin rows of the fp32
                      tables at positions {0, 1, 4095, 4096, 8191, 131071}
    chain_b1.npz      one seeded single-token chain (make_inputs(1, seed=0), the B = 1 configuration):
                      RMSNorm -> QKV + bias -> YaRN rotary, and the clamped SwiGLU of a [4, 5760] input, all fp32;
                      plus a checksum of the seeded inputs themselves
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import layers as O  # noqa: E402

POSITIONS = [0, 1, 4095, 4096, 8191, 131071]


def chain_b1():
    d = O.make_inputs(1, swiglu_rows=4, seed=0)
    t = O.rmsnorm_ref(d["x"], d["norm_scale"].float(), 1e-5)
    q, k, v = O.qkv_rope_ref(t.bfloat16(), d["w"], d["b"], d["positions"])
    s = O.swiglu_ref(d["swiglu_x"])
    sums = np.array([float(d[key].double().sum()) for key in ("x", "norm_scale", "w", "b", "swiglu_x")] + [float(d["positions"][0])])
    return {"normed": t.numpy(), "q": q.numpy(), "k": k.numpy(), "v": v.numpy(), "swiglu": s.numpy(), "input_sums": sums}


def main():
    conc, inv_freq = O.yarn_concentration_and_inv_freq()
    cos, sin = O.yarn_cos_sin(torch.tensor(POSITIONS))
    np.savez(os.path.join(HERE, "yarn_tables.npz"), inv_freq=inv_freq.numpy(), concentration=np.float64(conc),
             positions=np.array(POSITIONS), cos=cos.numpy(), sin=sin.numpy())
    np.savez(os.path.join(HERE, "chain_b1.npz"), **chain_b1())
    print("wrote yarn_tables.npz, chain_b1.npz with torch", torch.__version__)


if __name__ == "__main__":
    main()
