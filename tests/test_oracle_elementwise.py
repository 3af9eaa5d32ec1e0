"""Pins the oracle's restatements of the ops either side of a Linear (RmsNorm, RmsNormAdd,
GatedAct, GatedActFused, Add) with closed forms, special cases and layout constructions rather
than with the oracle's own formulas."""
import math

import numpy as np
import pytest

from oracle import oracle as orc


def test_activation_special_values_and_closed_forms():
    assert orc.act(orc.SILU, 0.0) == 0.0 and orc.act(orc.GELU, 0.0) == 0.0
    assert orc.act(orc.SIGMOID, 0.0) == np.float32(0.5)
    rng = np.random.default_rng(1)
    for g in rng.normal(0, 3, 200).astype(np.float32):
        g64 = float(g)
        sig = 1.0 / (1.0 + math.exp(-g64))
        assert abs(float(orc.act(orc.SIGMOID, g)) - sig) <= 2e-7
        assert abs(float(orc.act(orc.SILU, g)) - g64 * sig) <= 4e-7 * max(1.0, abs(g64))
        gelu = 0.5 * g64 * (1.0 + math.tanh(math.sqrt(2.0 / math.pi) * (g64 + 0.044715 * g64 ** 3)))
        assert abs(float(orc.act(orc.GELU, g)) - gelu) <= 1e-6 * max(1.0, abs(g64))
    # saturation: silu(g) -> g, sigmoid -> 1 for large g; -> 0 for very negative g
    assert orc.act(orc.SILU, 40.0) == np.float32(40.0) and orc.act(orc.SIGMOID, 40.0) == np.float32(1.0)
    assert abs(float(orc.act(orc.SILU, -40.0))) < 1e-15


def test_gated_act_clamp_is_one_sided_on_the_gate_and_symmetric_on_up():
    silu = lambda g: float(orc.act(orc.SILU, g))
    assert orc.gated_act_fn(orc.SILU, None, 1.5, 2.0) == np.float32(silu(1.5)) * np.float32(2.0)
    # gate above the limit is cut BEFORE the activation; a gate far below -limit is left alone
    assert orc.gated_act_fn(orc.SILU, 1.0, 5.0, 0.5) == np.float32(silu(1.0)) * np.float32(0.5)
    assert orc.gated_act_fn(orc.SILU, 1.0, -5.0, 0.5) == np.float32(silu(-5.0)) * np.float32(0.5)
    # up is clamped on both sides
    assert orc.gated_act_fn(orc.SILU, 1.0, 0.5, 7.0) == np.float32(silu(0.5)) * np.float32(1.0)
    assert orc.gated_act_fn(orc.SILU, 1.0, 0.5, -7.0) == np.float32(silu(0.5)) * np.float32(-1.0)


def test_rms_norm_closed_forms():
    # constant rows, power-of-two dim: every partial sum is exact, so the closed form must hold bit for bit
    for c, dim in [(2.0, 8), (-0.5, 256), (3.0, 4096)]:
        w = np.arange(1, dim + 1, dtype=np.float32)
        out = orc.rms_norm(np.full(dim, c, np.float32), w, 1, dim, 0.0)
        s = np.float32(1.0) / np.sqrt(np.float32(c * c))
        assert np.array_equal(out[0], np.float32(c) * s * w)
    # eps enters under the root: x = 0 gives 0 * (1/sqrt(eps)) * w = 0, not NaN
    assert not orc.rms_norm(np.zeros(16, np.float32), np.ones(16, np.float32), 1, 16, 1e-6).any()
    # one-hot row: ss = a^2 / dim
    x = np.zeros(64, np.float32)
    x[5] = 8.0
    out = orc.rms_norm(x, np.ones(64, np.float32), 1, 64, 0.0)
    assert out[0, 5] == np.float32(8.0) and np.count_nonzero(out) == 1


def test_rms_norm_properties_on_random_rows():
    rng = np.random.default_rng(2)
    rows, dim = 3, 1000
    x = rng.normal(0, 2, rows * dim).astype(np.float32)
    w = rng.normal(1, 0.1, dim).astype(np.float32)
    out = orc.rms_norm(x, w, rows, dim, 1e-6)
    x64 = x.reshape(rows, dim).astype(np.float64)
    ref = x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + 1e-6) * w
    assert np.abs(out - ref).max() <= 2e-6 * np.abs(ref).max()
    # rows are independent and the mean square of out / w is 1
    assert np.allclose(((out / w).astype(np.float64) ** 2).mean(axis=1), 1.0, atol=1e-5)
    one = orc.rms_norm(x[dim:2 * dim], w, 1, dim, 1e-6)
    assert np.array_equal(one[0], out[1])
    # RmsNormAdd accumulates into dst
    base = rng.normal(0, 1, (rows, dim)).astype(np.float32)
    assert np.array_equal(orc.rms_norm(x, w, rows, dim, 1e-6, into=base), base + out)


def test_rms_norm_sums_squares_in_index_order():
    # 1 followed by many tiny squares: added one at a time to a running sum of 1 they vanish
    # (each is below half an ulp of 1.0); a pairwise or reversed sum would keep them
    dim = 4096
    x = np.full(dim, 2.0 ** -13, np.float32)   # squares 2^-26; 4095 of them sum to ~6.1e-5
    x[0] = 1.0
    out = orc.rms_norm(x, np.ones(dim, np.float32), 1, dim, 0.0)
    s_seq = np.float32(1.0) / np.sqrt(np.float32(1.0) / np.float32(dim))
    assert out[0, 0] == s_seq


def test_gated_act_layouts():
    rng = np.random.default_rng(3)
    rows, nff = 3, 64
    g = rng.normal(0, 2, (rows, nff)).astype(np.float32)
    u = rng.normal(0, 2, (rows, nff)).astype(np.float32)
    plain = orc.gated_act(g, u, rows, nff)
    want = np.array([[orc.gated_act_fn(orc.SILU, None, g[r, i], u[r, i]) for i in range(nff)] for r in range(rows)])
    assert np.array_equal(plain, want)
    # up embedded in a wider row-major tensor at a column offset
    wide = rng.normal(0, 1, (rows, 200)).astype(np.float32)
    wide[:, 17:17 + nff] = u
    assert np.array_equal(orc.gated_act(g, wide, rows, nff, up_off=17, up_stride=200), plain)
    # gate interleaved with queries in blocks of 2*hd: [q(hd) | g(hd)] per head
    hd = 16
    inter = np.empty((rows, 2 * nff), np.float32)
    for h in range(nff // hd):
        inter[:, h * 2 * hd:h * 2 * hd + hd] = 99.0
        inter[:, h * 2 * hd + hd:(h + 1) * 2 * hd] = g[:, h * hd:(h + 1) * hd]
    assert np.array_equal(orc.gated_act(inter, u, rows, nff, gate_stride=2 * nff, gate_block_width=2 * hd), plain)
    # combined [rows, 2*nff] buffer, gate half first
    assert np.array_equal(orc.gated_act_fused(np.concatenate([g, u], axis=1), rows, nff), plain)
    # other activations and the clamp go through the same element function
    got = orc.gated_act(g, u, rows, nff, orc.GELU, clamp=1.25)
    assert got[1, 7] == orc.gated_act_fn(orc.GELU, 1.25, g[1, 7], u[1, 7])


def test_add():
    a = np.array([1.0, 2.5, -3.0, 1e20], np.float32)
    b = np.array([0.5, -2.5, 1.0, 1.0], np.float32)
    assert np.array_equal(orc.add(a, b), np.array([1.5, 0.0, -2.0, 1e20], np.float32))
