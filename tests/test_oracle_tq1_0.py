"""Pins the oracle's restatement of TQ1_0: the reference's single-block known answer
(crates/infr-gguf/src/dequant.rs:1365-1378); the digit extraction against the format's definition -
a byte holds five ternary digits as ceil(v * 256 / 243), v their base-3 value with the first digit
most significant (ggml's quantize_row_tq1_0), so every one of the 243 digit strings must come back,
and the four-digit qh bytes likewise; the element order against its published description; the
integer stage as an int64 sum; the f32 expression evaluated independently; dot(dequant) at the
reference's 1e-3."""
import itertools

import numpy as np
import pytest

from oracle import oracle as orc


def f16(b0, b1):
    return np.float32(np.frombuffer(bytes([int(b0), int(b1)]), np.float16)[0])


def pack5(trits):
    """Five digits (first = most significant) -> the byte ggml stores: ceil(v * 256 / 243)."""
    v = 0
    for t in trits:
        v = v * 3 + int(t)
    return (v * 256 + 242) // 243


def element_source(e):
    """(byte index in the block, digit index) of element e: 32 bytes x 5 digits, 16 bytes x 5, 4 x 4."""
    if e < 160:
        return e % 32, e // 32
    if e < 240:
        return 32 + (e - 160) % 16, (e - 160) // 16
    return 48 + (e - 240) % 4, (e - 240) // 4


def test_reference_known_answer():
    b = np.zeros(54, np.uint8)                      # tq1_0_single_block
    b[52:54] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    y = orc.dequant_block(orc.TQ1_0, b)
    assert y.size == 256 and np.all(y == -1.0)
    assert orc.block_layout(orc.TQ1_0) == (256, 54)


def test_every_digit_string_comes_back():
    blk = np.zeros(54, np.uint8)
    for trits in itertools.product(range(3), repeat=5):
        blk[7] = pack5(trits)                       # a byte of the first run: digit n -> element 32 n + 7
        blk[40] = pack5(trits)                      # of the second: element 160 + 16 n + 8
        assert [orc.tq1_0_digit(blk, 32 * n + 7) for n in range(5)] == list(trits)
        assert [orc.tq1_0_digit(blk, 160 + 16 * n + 8) for n in range(5)] == list(trits)
    for trits in itertools.product(range(3), repeat=4):
        blk[50] = pack5(trits + (0,))               # qh holds four digits, packed as five with a zero last
        assert [orc.tq1_0_digit(blk, 240 + 4 * n + 2) for n in range(4)] == list(trits)


def test_element_order_and_dequant():
    rng = np.random.default_rng(5)
    trits = rng.integers(0, 3, 256)
    blk = np.zeros(54, np.uint8)
    per_byte = {}
    for e in range(256):
        byte, n = element_source(e)
        per_byte.setdefault(byte, [0] * 5)[n] = int(trits[e])
    for byte, t in per_byte.items():
        blk[byte] = pack5(t)
    blk[52:54] = np.frombuffer(np.float16(0.25).tobytes(), np.uint8)
    y = orc.dequant_block(orc.TQ1_0, blk)
    assert np.array_equal(y, (trits - 1).astype(np.float32) * np.float32(0.25))


@pytest.mark.parametrize("in_f", [256, 1024])
def test_stage_and_terms(in_f):
    rng = np.random.default_rng(6 + in_f)
    row = orc.synth_weight(orc.TQ1_0, in_f, 0x9E)    # arbitrary bytes: every byte value decodes to digits 0..2
    assert f16(row[52], row[53]) == np.float32(np.float16(0.05))
    x = rng.standard_normal(in_f).astype(np.float32)
    q8 = orc.quantize_q8(x)
    y, ip = orc.vec_dot_tq1_0(row, q8, in_f, stages=True)
    acc = np.float32(0.0)
    for b in range(in_f // 256):
        blk = row[54 * b:54 * (b + 1)]
        digits = np.empty(256, np.int64)
        for e in range(256):
            byte, n = element_source(e)
            q = (int(blk[byte]) * 3 ** n) & 0xFF
            digits[e] = (q * 3) >> 8
        assert digits.min() >= 0 and digits.max() <= 2
        q = q8.qs[256 * b:256 * (b + 1)].astype(np.int64)
        want = int(((digits - 1) * q).sum())
        assert ip[b] == want
        acc = np.float32(acc + np.float32(np.float32(f16(blk[52], blk[53]) * q8.d[b]) * np.float32(want)))
    assert np.float32(y).view(np.uint32) == acc.view(np.uint32)


def test_dot_matches_dequant_reference_and_linear_dispatch():
    dtype, in_f, out_f, m = orc.TQ1_0, 1024, 9, 3
    rng = np.random.default_rng(78)
    w = orc.synth_weight(dtype, out_f * in_f, 0x62)
    x = rng.uniform(-1, 1, m * in_f).astype(np.float32)
    y = orc.linear(dtype, w, x, m, in_f, out_f)
    bpr = w.size // out_f
    wf = orc.dequant_block(dtype, w).reshape(out_f, in_f).astype(np.float64)
    for r in range(m):
        q8 = orc.quantize_q8(x[r * in_f:(r + 1) * in_f])
        xq = q8.qs.astype(np.float64) * np.repeat(q8.d.astype(np.float64), 256)
        for o in range(out_f):
            one = orc.vec_dot_tq1_0(w[o * bpr:(o + 1) * bpr], q8, in_f)
            assert np.float32(y[r, o]).view(np.uint32) == np.float32(one).view(np.uint32)   # batch == single
            ref = float(wf[o] @ xq)
            assert abs(float(one) - ref) <= 1e-3 * max(1.0, abs(ref))
    f64 = orc.ref_linear_f64(x, wf.astype(np.float32), m, in_f, out_f)
    yr = orc.linear(dtype, w, x, m, in_f, out_f, reference_mode=True)
    assert np.abs(y - f64).max() <= 2e-2 * np.abs(f64).max()
    assert np.abs(yr - f64).max() <= 1e-5 * max(1.0, np.abs(f64).max()) + 1e-4
    a, b = orc.linear_int_stages(dtype, w, x, m, in_f, out_f)
    assert a.shape == (m, out_f, in_f // 256) and b is None
