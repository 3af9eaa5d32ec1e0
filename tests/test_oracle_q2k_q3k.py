"""Pins the oracle's restatement of Q2_K and Q3_K: the reference's single-block known answers
(crates/infr-gguf/src/dequant.rs:1615-1720), hand blocks built from the published ggml layouts that
exercise every sub-block, shift and bit plane, independent element-at-a-time numpy decoders on random
bytes, brute-force int64 integer stages, the per-block f32 expression evaluated independently, and
dot(dequant) at the reference's 1e-3."""
import numpy as np
import pytest

from oracle import oracle as orc


def h16(v):
    return np.frombuffer(np.float16(v).tobytes(), np.uint8)


def f16(b0, b1):
    return np.float32(np.frombuffer(bytes([int(b0), int(b1)]), np.float16)[0])


def test_reference_known_answers():
    b = np.zeros(84, np.uint8)                      # q2k_single_block
    b[0] = b[1] = 0x23
    b[16:80] = 0x55
    b[80:82], b[82:84] = h16(1.0), h16(2.0)
    y = orc.dequant_block(orc.Q2_K, b)
    assert y.size == 256 and np.all(y[:32] == -1.0)
    b = np.zeros(110, np.uint8)                     # q3k_single_block
    b[108:110] = h16(1.0)
    y = orc.dequant_block(orc.Q3_K, b)
    assert y.size == 256 and np.all(y == 128.0)


# ───────────── independent decoders: element e of a block, straight from the ggml layout ─────────────
# Element e = 128 n + 32 j + 16 half + l (n < 2, j < 4, half < 2, l < 16) of both formats reads the
# two-bit field j of byte qs[32 n + 16 half + l]; its 16-element sub-block is e // 16.

def q2k_element(blk, e):
    n, j, half, l = e // 128, (e // 32) % 4, (e // 16) % 2, e % 16
    sc = int(blk[e // 16])
    code = (int(blk[16 + 32 * n + 16 * half + l]) >> (2 * j)) & 3
    d, dmin = f16(blk[80], blk[81]), f16(blk[82], blk[83])
    return np.float32(np.float32(d * np.float32(sc & 15)) * np.float32(code) + np.float32(dmin * np.float32(-(sc >> 4)))), code


def q3k_scale(blk, i):
    """Sub-block i's 6-bit scale: low nibble i < 8 / high nibble i >= 8 of scales[i % 8], two more bits
    from scales[8 + i % 4] at bit position 2 (i // 4); minus 32."""
    s = blk[96:108]
    low = (int(s[i % 8]) >> (4 * (i // 8))) & 15
    high = (int(s[8 + i % 4]) >> (2 * (i // 4))) & 3
    return (low | (high << 4)) - 32


def q3k_element(blk, e):
    n, j, half, l = e // 128, (e // 32) % 4, (e // 16) % 2, e % 16
    low2 = (int(blk[32 + 32 * n + 16 * half + l]) >> (2 * j)) & 3
    high = (int(blk[16 * half + l]) >> (4 * n + j)) & 1
    code = low2 | (high << 2)
    s = q3k_scale(blk, e // 16)
    d = f16(blk[108], blk[109])
    return np.float32(np.float32(d * np.float32(s)) * np.float32(code) + np.float32(d * np.float32(-4 * s))), code


def test_q3k_scale_fields_against_the_bit_layout():
    rng = np.random.default_rng(11)
    for _ in range(200):
        blk = rng.integers(0, 256, 110, dtype=np.uint8)
        got = orc.q3k_scales(blk[96:108])
        assert [int(v) for v in got] == [q3k_scale(blk, i) for i in range(16)]
    # one field at a time: scale 5's low nibble is scales[5] & 15, its top bits scales[9] bits 2-3
    blk = np.zeros(110, np.uint8)
    blk[96 + 5], blk[96 + 9] = 0x0B, 0b1000
    want = [-32] * 16
    want[5] = (0x0B | (2 << 4)) - 32
    assert [int(v) for v in orc.q3k_scales(blk[96:108])] == want


def test_hand_blocks_touch_every_subblock_shift_and_plane():
    # Q2_K: scale byte of sub-block s = (s + 1) | ((15 - s) << 4); every qs byte 0b11100100: field j = j
    b = np.zeros(84, np.uint8)
    for s in range(16):
        b[s] = (s + 1 if s < 15 else 15) | ((15 - s) << 4)
    b[16:80] = 0b11100100
    b[80:82], b[82:84] = h16(0.5), h16(0.25)
    y = orc.dequant_block(orc.Q2_K, b)
    for e in range(256):
        s, j = e // 16, (e // 32) % 4
        want = np.float32(0.5 * (int(b[s]) & 15)) * np.float32(j) + np.float32(0.25 * -(int(b[s]) >> 4))
        assert y[e] == np.float32(want), e
    # Q3_K: all scales 33 (field 1 -> s = 1: low nibbles 1, top bits 2 -> byte 0b10101010), low two
    # bits 0b00011011 (field j = 3 - j), plane bit (4 n + j) set for odd l only
    b = np.zeros(110, np.uint8)
    b[96:104] = 0x11
    b[104:108] = 0b10101010
    b[32:96] = 0b00011011
    b[0:32] = np.where(np.arange(32) % 2 == 1, 0xFF, 0x00)
    b[108:110] = h16(2.0)
    y = orc.dequant_block(orc.Q3_K, b)
    for e in range(256):
        j, l = (e // 32) % 4, e % 16
        code = (3 - j) | (4 if l % 2 else 0)
        assert y[e] == np.float32(2.0 * 1 * code + 2.0 * -4), e


@pytest.mark.parametrize("dtype", [orc.Q2_K, orc.Q3_K])
def test_dequant_block_matches_independent_decoder_bit_for_bit(dtype):
    bpb = orc.block_layout(dtype)[1]
    w = orc.synth_weight(dtype, 256 * 6, 0x31 + dtype)
    y = orc.dequant_block(dtype, w)
    el = q2k_element if dtype == orc.Q2_K else q3k_element
    for b in range(6):
        blk = w[b * bpb:(b + 1) * bpb]
        want = np.array([el(blk, e)[0] for e in range(256)], np.float32)
        assert np.array_equal(y[b * 256:(b + 1) * 256].view(np.uint32), want.view(np.uint32)), b


def test_synth_scale_slots():
    w = orc.synth_weight(orc.Q2_K, 512, 7)
    for b in range(2):
        assert f16(w[84 * b + 80], w[84 * b + 81]) == np.float32(np.float16(0.05))
        assert f16(w[84 * b + 82], w[84 * b + 83]) == np.float32(np.float16(0.10))
    w = orc.synth_weight(orc.Q3_K, 512, 7)
    for b in range(2):
        assert f16(w[110 * b + 108], w[110 * b + 109]) == np.float32(np.float16(0.03))


@pytest.mark.parametrize("in_f", [256, 1024])
def test_q2k_stages_and_terms(in_f):
    rng = np.random.default_rng(5 + in_f)
    row = orc.synth_weight(orc.Q2_K, in_f, 0x99)
    x = rng.standard_normal(in_f).astype(np.float32)
    q8 = orc.quantize_q8(x)
    y, sd, sm = orc.vec_dot_q2k(row, q8, in_f, stages=True)
    acc = np.float32(0.0)
    for b in range(in_f // 256):
        blk = row[84 * b:84 * (b + 1)]
        codes = np.array([q2k_element(blk, e)[1] for e in range(256)], np.int64)
        q = q8.qs[256 * b:256 * (b + 1)].astype(np.int64)
        want_sd = sum((int(blk[s]) & 15) * int((codes[16 * s:16 * s + 16] * q[16 * s:16 * s + 16]).sum()) for s in range(16))
        want_sm = sum((int(blk[s]) >> 4) * int(q[16 * s:16 * s + 16].sum()) for s in range(16))
        assert sd[b] == want_sd and sm[b] == want_sm
        d, dmin = f16(blk[80], blk[81]), f16(blk[82], blk[83])
        acc = np.float32(acc + np.float32(q8.d[b] * np.float32(np.float32(d * np.float32(want_sd)) - np.float32(dmin * np.float32(want_sm)))))
    assert np.float32(y).view(np.uint32) == acc.view(np.uint32)


@pytest.mark.parametrize("in_f", [256, 1024])
def test_q3k_stage_and_terms(in_f):
    rng = np.random.default_rng(6 + in_f)
    row = orc.synth_weight(orc.Q3_K, in_f, 0x9A)
    x = rng.standard_normal(in_f).astype(np.float32)
    q8 = orc.quantize_q8(x)
    y, isum = orc.vec_dot_q3k(row, q8, in_f, stages=True)
    acc = np.float32(0.0)
    for b in range(in_f // 256):
        blk = row[110 * b:110 * (b + 1)]
        codes = np.array([q3k_element(blk, e)[1] for e in range(256)], np.int64)
        q = q8.qs[256 * b:256 * (b + 1)].astype(np.int64)
        # sum over elements of s * (code - 4) * q8: the same integer as sc * (iprod - 4 bsum16)
        want = sum(q3k_scale(blk, s) * int(((codes[16 * s:16 * s + 16] - 4) * q[16 * s:16 * s + 16]).sum()) for s in range(16))
        assert isum[b] == want
        d = f16(blk[108], blk[109])
        acc = np.float32(acc + np.float32(np.float32(d * q8.d[b]) * np.float32(want)))
    assert np.float32(y).view(np.uint32) == acc.view(np.uint32)


@pytest.mark.parametrize("dtype", [orc.Q2_K, orc.Q3_K])
def test_dot_matches_dequant_reference(dtype):
    # the int8 kernel against dot(dequant(w), dequant(q8)) at the reference's 1e-3
    in_f = 1024
    rng = np.random.default_rng(40 + dtype)
    row = orc.synth_weight(dtype, in_f, 0x51)
    x = rng.uniform(-1, 1, in_f).astype(np.float32)
    q8 = orc.quantize_q8(x)
    y = orc.vec_dot_q2k(row, q8, in_f) if dtype == orc.Q2_K else orc.vec_dot_q3k(row, q8, in_f)
    wf = orc.dequant_block(dtype, row).astype(np.float64)
    xq = q8.qs.astype(np.float64) * np.repeat(q8.d.astype(np.float64), 256)
    ref = float(wf @ xq)
    assert abs(float(y) - ref) <= 1e-3 * max(1.0, abs(ref))


@pytest.mark.parametrize("dtype", [orc.Q2_K, orc.Q3_K])
def test_linear_dispatch(dtype):
    # production arm = the per-256 int8 kernel row by row (batch == single); reference mode = f32 dot of
    # the decoded row; the two agree to the reference's 2e-2 of max|f64 oracle|
    in_f, out_f, m = 512, 9, 3
    rng = np.random.default_rng(70 + dtype)
    w = orc.synth_weight(dtype, out_f * in_f, 0x61)
    x = rng.standard_normal(m * in_f).astype(np.float32)
    y = orc.linear(dtype, w, x, m, in_f, out_f)
    bpr = w.size // out_f
    for r in range(m):
        q8 = orc.quantize_q8(x[r * in_f:(r + 1) * in_f])
        for o in range(out_f):
            row = w[o * bpr:(o + 1) * bpr]
            one = orc.vec_dot_q2k(row, q8, in_f) if dtype == orc.Q2_K else orc.vec_dot_q3k(row, q8, in_f)
            assert np.float32(y[r, o]).view(np.uint32) == np.float32(one).view(np.uint32)
    y1 = orc.linear(dtype, w, x[:in_f], 1, in_f, out_f)
    assert np.array_equal(y1.view(np.uint32), y[:1].view(np.uint32))
    wf = orc.dequant_block(dtype, w).reshape(out_f, in_f)
    f64 = orc.ref_linear_f64(x, wf, m, in_f, out_f)
    yr = orc.linear(dtype, w, x, m, in_f, out_f, reference_mode=True)
    bound = 2e-2 * np.abs(f64).max()
    assert np.abs(y - f64).max() <= bound and np.abs(yr - f64).max() <= 1e-5 * max(1.0, np.abs(f64).max()) + 1e-4
    a, b = orc.linear_int_stages(dtype, w, x, m, in_f, out_f)
    assert a.shape == (m, out_f, in_f // 256) and ((b is not None) == (dtype == orc.Q2_K))
