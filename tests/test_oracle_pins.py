"""Pins for the CPU oracle: closed forms, invariants and float64 brute force.

None of these retype the oracle's formula in the oracle's own arithmetic: the
brute-force twins are numpy float64 loops / expressions written from the
mathematical definition, and the rest are properties the mathematics fixes.
"""
import math

import numpy as np
import pytest
import torch

from oracle import layers as O


# ----------------------------------------------------------------------------- YaRN parameters
def test_yarn_constants_closed_form():
    conc, inv = O.yarn_concentration_and_inv_freq()
    assert conc == pytest.approx(1.3465735902799727, abs=1e-15)
    assert inv.dtype == torch.float32 and inv.shape == (32,)
    low = 32 * math.log(4096 / (32 * 2 * math.pi)) / math.log(150000.0)
    high = 32 * math.log(4096 / (2 * math.pi)) / math.log(150000.0)
    assert low == pytest.approx(8.092779, abs=1e-5)
    assert high == pytest.approx(17.398024, abs=1e-5)
    inv64 = inv.double().numpy()
    assert inv64[0] == 1.0
    for i in range(32):
        f = 150000.0 ** (-i / 32)
        if i <= 8:      # pure extrapolation below `low`
            assert inv64[i] == pytest.approx(f, rel=2e-6)
        elif i >= 18:   # pure interpolation above `high`
            assert inv64[i] == pytest.approx(f / 32, rel=2e-6)
        else:           # blended band
            m = 1 - min(max((i - low) / (high - low), 0.0), 1.0)
            assert inv64[i] == pytest.approx(f / 32 * (1 - m) + f * m, rel=5e-6)
    assert np.all(np.diff(inv64) < 0)  # strictly decreasing frequencies


def test_yarn_scaling_one_is_textbook_rope():
    conc, inv = O.yarn_concentration_and_inv_freq(scaling_factor=1.0, base=10000.0, head_dim=128)
    assert conc == 1.0
    expect = 10000.0 ** (-np.arange(0, 128, 2) / 128)
    np.testing.assert_allclose(inv.double().numpy(), expect, rtol=2e-6)


def test_yarn_cos_sin_vs_float64():
    pos = torch.tensor([0, 1, 4095, 4096, 8191, 131071], dtype=torch.int64)
    cos, sin = O.yarn_cos_sin(pos)
    conc, inv = O.yarn_concentration_and_inv_freq()
    # angle is the *fp32* product; evaluate cos/sin of that fp32 angle in float64
    ang32 = (pos.float()[:, None] * inv[None, :]).double().numpy()
    np.testing.assert_allclose(cos.double().numpy(), np.cos(ang32) * conc, atol=4e-7)
    np.testing.assert_allclose(sin.double().numpy(), np.sin(ang32) * conc, atol=4e-7)
    assert torch.all(cos[0] == np.float32(conc)) and torch.all(sin[0] == 0)


def test_token_positions_wrap():
    p = O.token_positions(2, 3, 131071, 131072)
    assert p.tolist() == [131071, 0, 1, 131071, 0, 1]


# ----------------------------------------------------------------------------- RMSNorm
def test_rmsnorm_bruteforce_float64():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(3, 40, generator=g).bfloat16()
    s = (1 + 0.1 * torch.randn(40, generator=g)).bfloat16()
    ref = np.empty((3, 40))
    xn, sn = x.double().numpy(), s.double().numpy()
    for r in range(3):
        acc = 0.0
        for c in range(40):
            acc += xn[r, c] * xn[r, c]
        inv = 1.0 / math.sqrt(acc / 40 + 1e-5)
        for c in range(40):
            ref[r, c] = xn[r, c] * inv * sn[c]
    np.testing.assert_allclose(O.rmsnorm_ref(x, s, 1e-5).double().numpy(), ref, rtol=2e-6, atol=1e-7)


def test_rmsnorm_invariants():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(4, 2880, generator=g)
    one = torch.ones(2880)
    y = O.rmsnorm_ref(x, one, 1e-5)
    ms = x.pow(2).mean(-1)
    torch.testing.assert_close(y.pow(2).mean(-1).sqrt(), 1 / torch.sqrt(1 + 1e-5 / ms), rtol=1e-5, atol=0)
    torch.testing.assert_close(O.rmsnorm_ref(8 * x, one, 1e-5), y, rtol=1e-4, atol=1e-6)   # scale invariance up to eps
    c, s = -3.0, torch.linspace(0.5, 1.5, 2880)
    const = O.rmsnorm_ref(torch.full((1, 2880), c), s, 1e-5)
    torch.testing.assert_close(const[0], -s / math.sqrt(1 + 1e-5 / c**2), rtol=1e-6, atol=0)
    assert torch.all(O.rmsnorm_ref(torch.zeros(2, 2880), s, 1e-5) == 0)


# ----------------------------------------------------------------------------- embedding / linear
def test_embedding_is_row_gather():
    g = torch.Generator().manual_seed(3)
    table = torch.randn(97, 16, generator=g).bfloat16()
    ids = torch.tensor([[0, 96, 5, 5, 0]], dtype=torch.int32)
    out = O.embedding_ref(table, ids)
    assert out.shape == (1, 5, 16)
    for j, i in enumerate(ids[0].tolist()):
        assert torch.equal(out[0, j], table[i])


def test_linear_bruteforce_and_selectors():
    g = torch.Generator().manual_seed(4)
    x = torch.randn(3, 24, generator=g).bfloat16()
    w = torch.randn(10, 24, generator=g).bfloat16()
    b = torch.randn(10, generator=g).bfloat16()
    ref = x.double().numpy() @ w.double().numpy().T + b.double().numpy()
    np.testing.assert_allclose(O.linear_ref(x, w, b).double().numpy(), ref, rtol=1e-5, atol=1e-5)
    e = torch.zeros(1, 24)
    e[0, 7] = 1.0
    torch.testing.assert_close(O.linear_ref(e, w, b)[0], w.float()[:, 7] + b.float())


# ----------------------------------------------------------------------------- rotary
def _rot(x, pos, **kw):
    cos, sin = O.yarn_cos_sin(torch.as_tensor(pos, dtype=torch.int64), **kw)
    return O.rope_rotate_ref(x, cos, sin)


def test_rope_layout_is_half_split():
    x = torch.zeros(1, 1, 64)
    x[0, 0, 3] = 1.0
    y = _rot(x, [5])
    nz = torch.nonzero(y[0, 0]).flatten().tolist()
    assert nz == [3, 35]   # partner of d is d+32, not d^1
    cos, sin = O.yarn_cos_sin(torch.tensor([5]))
    assert y[0, 0, 3] == cos[0, 3] and y[0, 0, 35] == sin[0, 3]


def test_rope_norm_and_position_zero():
    g = torch.Generator().manual_seed(5)
    x = torch.randn(6, 8, 64, generator=g)
    conc, _ = O.yarn_concentration_and_inv_freq()
    y = _rot(x, [0, 1, 77, 4096, 8191, 100000])
    n_in = x[..., :32] ** 2 + x[..., 32:] ** 2
    n_out = y[..., :32] ** 2 + y[..., 32:] ** 2
    torch.testing.assert_close(n_out, conc**2 * n_in, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(y[0], np.float32(conc) * x[0], rtol=1e-6, atol=0)


def test_rope_relative_position_property():
    g = torch.Generator().manual_seed(6)
    q = torch.randn(1, 1, 64, generator=g).double()
    k = torch.randn(1, 1, 64, generator=g).double()

    def dot(m, n):
        return float((_rot(q, [m]).double() * _rot(k, [n]).double()).sum())

    # positions small enough that fp32 angles carry ~1e-6 absolute error
    assert dot(10, 3) == pytest.approx(dot(107, 100), rel=2e-4, abs=2e-4)
    assert dot(50, 50) == pytest.approx(dot(0, 0), rel=2e-4, abs=2e-4)


def test_rope_additivity():
    g = torch.Generator().manual_seed(7)
    x = torch.randn(1, 2, 64, generator=g)
    conc, _ = O.yarn_concentration_and_inv_freq()
    ab = _rot(_rot(x, [40]), [60])
    torch.testing.assert_close(ab, np.float32(conc) * _rot(x, [100]), rtol=1e-4, atol=1e-4)


def test_rope_textbook_when_unscaled():
    g = torch.Generator().manual_seed(8)
    x = torch.randn(2, 1, 8, generator=g)
    y = _rot(x, [3, 9], head_dim=8, base=10000.0, scaling_factor=1.0).double().numpy()
    xn = x.double().numpy()
    for r, p in enumerate([3, 9]):
        for d in range(4):
            th = p * 10000.0 ** (-2 * d / 8)
            a, b = xn[r, 0, d], xn[r, 0, d + 4]
            assert y[r, 0, d] == pytest.approx(a * math.cos(th) - b * math.sin(th), abs=2e-6)
            assert y[r, 0, d + 4] == pytest.approx(b * math.cos(th) + a * math.sin(th), abs=2e-6)


def test_qkv_rope_composition():
    d = O.make_inputs(3, seed=9)
    q, k, v = O.qkv_rope_ref(d["x"], d["w"], d["b"], d["positions"])
    qkv = O.linear_ref(d["x"], d["w"], d["b"])
    assert torch.equal(v, qkv[:, 4608:])            # v is the raw slice
    cos, sin = O.yarn_cos_sin(d["positions"])
    # head 5 of q, pair (d=7, d+32)
    a, b = qkv[:, 5 * 64 + 7], qkv[:, 5 * 64 + 39]
    torch.testing.assert_close(q[:, 5 * 64 + 7], a * cos[:, 7] - b * sin[:, 7])
    torch.testing.assert_close(k[:, 2 * 64 + 39], qkv[:, 4096 + 2 * 64 + 39] * cos[:, 7] + qkv[:, 4096 + 2 * 64 + 7] * sin[:, 7])
    qa, ka, va = O.qkv_rope_ref(d["x"], d["w"], d["b"], d["positions"], round_qkv_first=True)
    torch.testing.assert_close(qa, q, rtol=1.6e-2, atol=1e-2)
    torch.testing.assert_close(ka, k, rtol=1.6e-2, atol=1e-2)


# ----------------------------------------------------------------------------- SwiGLU
def test_swiglu_bruteforce_float64_edge_grid():
    gs = [-30.0, -7.0, 0.0, 6.99, 7.0, 7.01, 30.0]
    ls = [-30.0, -7.01, -7.0, -1.0, 0.0, 7.0, 30.0]
    rows = []
    for gv in gs:
        row = []
        for lv in ls:
            row += [gv, lv]
        rows.append(row)
    x = torch.tensor(rows, dtype=torch.float32)
    out = O.swiglu_ref(x).double().numpy()
    for i, gv in enumerate(gs):
        for j, lv in enumerate(ls):
            gg = min(gv, 7.0)
            ll = min(max(lv, -7.0), 7.0)
            expect = gg / (1 + math.exp(-1.702 * gg)) * (ll + 1)
            assert out[i, j] == pytest.approx(expect, rel=2e-6, abs=1e-12), (gv, lv)
    j1 = ls.index(-1.0)
    assert np.all(out[:, j1] == 0)                          # l = -1  =>  exact zero
    sat = 7.0 / (1 + math.exp(-1.702 * 7.0))
    assert out[gs.index(30.0), ls.index(0.0)] == pytest.approx(sat, rel=1e-6)
    assert out[gs.index(-30.0), ls.index(0.0)] < 0 and out[gs.index(-30.0), ls.index(0.0)] > -1e-18  # no lower clamp on gate


def test_swiglu_interleaved_equals_chunked_under_permutation():
    g = torch.Generator().manual_seed(10)
    x = (2 * torch.randn(5, 64, generator=g)).bfloat16()
    perm = torch.cat((x[:, ::2], x[:, 1::2]), dim=-1)
    assert torch.equal(O.swiglu_ref(x, interleaved=True), O.swiglu_ref(perm, interleaved=False))


def test_eager_twins_within_tolerance_of_upcast_oracle():
    d = O.make_inputs(8, swiglu_rows=32, seed=0)
    torch.testing.assert_close(O.rmsnorm_eager(d["x"], d["norm_scale"]).float(), O.rmsnorm_ref(d["x"], d["norm_scale"]), rtol=1.6e-2, atol=1e-2)
    torch.testing.assert_close(O.swiglu_eager(d["swiglu_x"]).float(), O.swiglu_ref(d["swiglu_x"]), rtol=5e-2, atol=5e-2)
    cos_t, sin_t = O.yarn_cos_sin(torch.arange(8192))
    q, k, v = O.qkv_rope_eager(d["x"], d["w"], d["b"], cos_t, sin_t, d["positions"])
    qr, kr, vr = O.qkv_rope_ref(d["x"], d["w"], d["b"], d["positions"])
    torch.testing.assert_close(q.float(), qr, rtol=5e-2, atol=5e-2)
    torch.testing.assert_close(v.float(), vr, rtol=1.6e-2, atol=1e-2)


def test_fp8_rows_quantisation_pins():
    """e4m3fn decode against the OCP bit formula for all 256 codes; the row maximum lands on +-448; the round trip
    stays within half a step of the format (3 mantissa bits: relative 2^-4 for normals)."""
    codes = torch.arange(256, dtype=torch.uint8)
    dec = codes.view(torch.float8_e4m3fn).to(torch.float32)
    for c in range(256):
        s, e, m = c >> 7, (c >> 3) & 15, c & 7
        if e == 15 and m == 7:
            assert math.isnan(dec[c].item())
            continue
        val = (m / 8.0) * 2.0 ** -6 if e == 0 else (1 + m / 8.0) * 2.0 ** (e - 7)
        assert dec[c].item() == (-val if s else val), c
    g = torch.Generator().manual_seed(5)
    w = (0.02 * torch.randn(64, 256, generator=g)).bfloat16()
    w[3] = 0                                                    # an all-zero row must not divide by zero
    w8, scale = O.quantize_fp8_rows_ref(w)
    assert w8.dtype == torch.float8_e4m3fn and scale.dtype == torch.float32 and scale.shape == (64,)
    amax = w.float().abs().max(dim=1).values
    torch.testing.assert_close(scale[amax > 0], (amax / 448.0)[amax > 0], rtol=1e-6, atol=0)
    assert scale[3].item() == pytest.approx(1e-12 / 448.0, rel=1e-5)
    assert torch.all(w8.float().abs().max(dim=1).values[amax > 0] == 448.0)
    deq = O.dequant_fp8_ref(w8, scale)
    assert torch.all(deq[3] == 0)
    err = (deq - w.float()).abs()
    # half a step: normals 2^-4 relative; below 2^-6 (in units of scale) the step is fixed at 2^-9
    bound = torch.maximum(w.float().abs() * 2.0 ** -4, scale[:, None] * 2.0 ** -10) * 1.0001
    assert torch.all(err <= bound)


def test_out_residual_ref_brute_force():
    g = torch.Generator().manual_seed(9)
    x = torch.randn(3, 40, generator=g).bfloat16()
    w = (0.1 * torch.randn(7, 40, generator=g)).bfloat16()
    b = (0.1 * torch.randn(7, generator=g)).bfloat16()
    r = torch.randn(3, 7, generator=g).bfloat16()
    want = torch.zeros(3, 7, dtype=torch.float64)
    for i in range(3):
        for n in range(7):
            want[i, n] = sum(float(x[i, k]) * float(w[n, k]) for k in range(40)) + float(b[n]) + float(r[i, n])
    torch.testing.assert_close(O.out_residual_ref(x, w, b, r).double(), want, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(O.out_residual_ref(x, w, None, None), O.linear_ref(x, w, None))


def test_attention_decode_ref_pins():
    g = torch.Generator().manual_seed(11)
    bs, n_keys, n_kv, groups, hd = 2, 40, 2, 3, 16
    q = torch.randn(bs, 1, n_kv, groups, hd, generator=g).bfloat16()
    k = torch.randn(bs, n_keys, n_kv, hd, generator=g).bfloat16()
    v = torch.randn(bs, n_keys, n_kv, hd, generator=g).bfloat16()
    sinks = torch.randn(n_kv * groups, generator=g).bfloat16()
    for window, start in ((None, 39), (None, 7), (8, 20), (8, 3), (100, 25)):
        got = O.attention_decode_ref(q, k, v, sinks, 0.25, window, start).view(bs, n_kv, groups, hd)
        lo = max(0, start - window + 1) if window else 0
        for b in range(bs):
            for h in range(n_kv):
                for m in range(groups):
                    s = [0.25 * sum(float(q[b, 0, h, m, d]) * float(k[b, n, h, d]) for d in range(hd)) for n in range(lo, start + 1)]
                    sk = float(sinks[h * groups + m])
                    top = max(max(s), sk)
                    wts = [math.exp(x - top) for x in s]
                    z = sum(wts) + math.exp(sk - top)
                    want = [sum(wts[i] * float(v[b, lo + i, h, d]) for i in range(len(s))) / z for d in range(hd)]
                    torch.testing.assert_close(got[b, h, m].double(), torch.tensor(want, dtype=torch.float64), rtol=1e-4, atol=1e-5)
    # sink -> -inf: plain causal softmax; sink -> +inf: nothing is left for the values; no sinks = logit 0
    plain = O.attention_decode_ref(q, k, v, torch.full((6,), -1e4), 0.25, None, 39).view(bs, n_kv, groups, hd)
    sm = torch.softmax(torch.einsum("bhmd,bkhd->bhmk", q[:, 0].float(), k.float()) * 0.25, dim=-1)
    torch.testing.assert_close(plain, torch.einsum("bhmk,bkhd->bhmd", sm, v.float()), rtol=1e-5, atol=1e-6)
    assert O.attention_decode_ref(q, k, v, torch.full((6,), 1e4), 0.25, None, 39).abs().max() < 1e-6
    torch.testing.assert_close(O.attention_decode_ref(q, k, v, None, 0.25, None, 39), O.attention_decode_ref(q, k, v, torch.zeros(6), 0.25, None, 39))
    # all keys equal: every weight is the same, output = mean of the values times the non-sink share
    ke = k[:, :1].expand(-1, n_keys, -1, -1)
    out = O.attention_decode_ref(q, ke, v, torch.full((6,), -1e4), 0.25, None, 39).view(bs, n_kv, groups, hd)
    torch.testing.assert_close(out, v.float().mean(dim=1)[:, :, None, :].expand(-1, -1, groups, -1), rtol=1e-5, atol=1e-6)


def test_attention_ref_pins():
    g = torch.Generator().manual_seed(12)
    bs, n_keys, n_kv, groups, hd, nq = 2, 24, 2, 3, 16, 9
    q = torch.randn(bs, nq, n_kv, groups, hd, generator=g).bfloat16()
    k = torch.randn(bs, n_keys, n_kv, hd, generator=g).bfloat16()
    v = torch.randn(bs, n_keys, n_kv, hd, generator=g).bfloat16()
    sinks = torch.randn(n_kv * groups, generator=g).bfloat16()
    # row i of the many-query form is the one-query form at position start + i (which is pinned by brute force above)
    for window, start in ((None, 0), (None, 15), (5, 0), (5, 11), (100, 3)):
        got = O.attention_ref(q, k, v, sinks, 0.25, window, start)
        for i in range(nq):
            one = O.attention_decode_ref(q[:, i : i + 1], k, v, sinks, 0.25, window, start + i)
            torch.testing.assert_close(got[:, i : i + 1], one, rtol=1e-5, atol=1e-6)
    # float64 brute force where the last positions lie beyond the keys (start + i >= n_keys) and a window cuts the front
    window, start = 6, 18
    got = O.attention_ref(q, k, v, sinks, 0.25, window, start).view(bs, nq, n_kv, groups, hd)
    for b in range(bs):
        for i in range(nq):
            p = start + i
            vis = [n for n in range(n_keys) if n <= p and n >= p - window + 1]
            for h in range(n_kv):
                for m in range(groups):
                    sk = float(sinks[h * groups + m])
                    sc = [0.25 * sum(float(q[b, i, h, m, d]) * float(k[b, n, h, d]) for d in range(hd)) for n in vis]
                    top = max(sc + [sk])
                    wts = [math.exp(x - top) for x in sc]
                    z = sum(wts) + math.exp(sk - top)
                    want = [sum(w * float(v[b, n, h, d]) for w, n in zip(wts, vis)) / z for d in range(hd)]
                    torch.testing.assert_close(got[b, i, h, m].double(), torch.tensor(want, dtype=torch.float64), rtol=1e-4, atol=1e-5)
    # positions past the keys by more than the window see nothing: zeros (only the sink is left)
    assert O.attention_ref(q, k, v, sinks, 0.25, 4, 40).abs().max() == 0
    # no sinks = logit 0
    torch.testing.assert_close(O.attention_ref(q, k, v, None, 0.25, None, 2), O.attention_ref(q, k, v, torch.zeros(6), 0.25, None, 2))


def _e2m1(nib: int) -> float:
    """OCP MX e2m1: sign bit 3, two exponent bits (bias 1), one mantissa bit; exponent 0 is subnormal (0 or 0.5)."""
    s, e, m = nib >> 3, (nib >> 1) & 3, nib & 1
    mag = 0.5 * m if e == 0 else (1 + 0.5 * m) * 2.0 ** (e - 1)
    return -mag if s else mag


def test_mxfp4_dequant_ref_pins():
    # the table is the e2m1 format
    assert [_e2m1(n) for n in range(16)] == list(O.FP4_VALUES)
    # every (byte, scale) pair with a finite result: element 2k = low nibble, 2k+1 = high nibble, times an exact power of two
    bytes_ = torch.arange(256, dtype=torch.uint8)
    blocks = bytes_.reshape(1, 16, 16).repeat(255, 1, 1)               # [scale, G=16, B=16]: all 256 byte values per scale
    scales = torch.arange(255, dtype=torch.uint8).reshape(255, 1).repeat(1, 16)
    got = O.mxfp4_dequant_ref(blocks, scales)
    assert got.shape == (255, 512) and got.dtype == torch.bfloat16
    want = np.empty((255, 512), dtype=np.float64)
    for s in range(255):
        for byte in range(256):
            want[s, 2 * byte] = _e2m1(byte & 15) * 2.0 ** (s - 127)
            want[s, 2 * byte + 1] = _e2m1(byte >> 4) * 2.0 ** (s - 127)
    # finite products are exactly representable in bf16 (one mantissa bit, exponents -128..129); 6 * 2^127 and
    # 4 * 2^127 overflow fp32 / bf16 to inf
    bf16_max = float(torch.finfo(torch.bfloat16).max)
    want_t = torch.from_numpy(want)
    finite = want_t.abs() <= bf16_max
    assert torch.equal(got.double()[finite], want_t[finite])
    assert torch.isinf(got.double()[~finite]).all() and (torch.sign(got.double()[~finite]) == torch.sign(want_t[~finite])).all()
    assert (~finite).sum() > 0
    # signed zeros survive
    assert torch.signbit(O.mxfp4_dequant_ref(torch.full((1, 16), 0x88, dtype=torch.uint8), torch.tensor([127], dtype=torch.uint8))).all()
    # torch.ldexp on the looked-up bf16 values, the library call the reference makes (weights.py:112), scale 255 included
    blocks = torch.randint(0, 256, (3, 7, 16), dtype=torch.uint8, generator=torch.Generator().manual_seed(5))
    scales = torch.randint(0, 256, (3, 7), dtype=torch.uint8, generator=torch.Generator().manual_seed(6))
    scales[0, 0] = 255
    scales[0, 1] = 0
    lut = torch.tensor(O.FP4_VALUES, dtype=torch.bfloat16)
    # second formulation (weights.py:119-139): stack (lo, hi) on a new last axis and flatten it
    idx = torch.stack((blocks & 0x0F, blocks >> 4), dim=-1).reshape(3, 7, 32).int()
    alt = torch.ldexp(lut[idx], (scales.int() - 127).unsqueeze(-1)).reshape(3, 7 * 32)
    got = O.mxfp4_dequant_ref(blocks, scales)
    assert got.shape == alt.shape
    assert torch.equal(got.view(torch.int16)[~torch.isnan(alt)], alt.view(torch.int16)[~torch.isnan(alt)])
    assert torch.equal(torch.isnan(got), torch.isnan(alt)) and torch.isnan(alt).any()    # 0 * 2^128 = nan in both
    # nibble order by a planted byte: 0x21 -> (0.5, 1.0)
    one = torch.zeros(1, 16, dtype=torch.uint8)
    one[0, 3] = 0x21
    out = O.mxfp4_dequant_ref(one, torch.tensor([128], dtype=torch.uint8))
    assert out[6].item() == 1.0 and out[7].item() == 2.0 and out.count_nonzero() == 2
