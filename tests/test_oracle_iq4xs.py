"""Pins the oracle's restatement of IQ4_XS: the reference's single-block known answer
(crates/infr-gguf/src/dequant.rs:1257-1277), hand blocks built from the published ggml layout that
give every sub-block its own scale and every nibble position its own code, an independent
element-at-a-time numpy decoder on random bytes, a brute-force int64 integer stage, the
per-superblock f32 expression evaluated independently, and dot(dequant) at the reference's 1e-3."""
import numpy as np
import pytest

from oracle import oracle as orc

# kvalues_iq4nl as ggml-common.h publishes it (the reference quotes the same table,
# crates/infr-gguf/src/dequant.rs:439-441)
KV = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], np.int64)


def h16(v):
    return np.frombuffer(np.float16(v).tobytes(), np.uint8)


def f16(b0, b1):
    return np.float32(np.frombuffer(bytes([int(b0), int(b1)]), np.float16)[0])


def scale(blk, ib):
    """Sub-block ib's 6-bit scale: nibble ib of the four scales_l bytes, two more bits from the
    16-bit scales_h at bit 2 ib; minus 32."""
    sh = int(blk[2]) | (int(blk[3]) << 8)
    lo = (int(blk[4 + ib // 2]) >> (4 * (ib % 2))) & 15
    return (lo | (((sh >> (2 * ib)) & 3) << 4)) - 32


def element(blk, e):
    """Element e = 32 ib + 16 hi + j reads nibble hi of qs[16 ib + j]."""
    ib, hi, j = e // 32, (e // 16) % 2, e % 16
    code = int(KV[(int(blk[8 + 16 * ib + j]) >> (4 * hi)) & 15])
    d = f16(blk[0], blk[1])
    return np.float32(np.float32(d * np.float32(scale(blk, ib))) * np.float32(code)), code


def test_reference_known_answer():
    b = np.zeros(136, np.uint8)                     # iq4xs_single_block: ls = 0, every code 0
    b[0:2] = h16(1.0)
    y = orc.dequant_block(orc.IQ4_XS, b)
    assert y.size == 256 and np.all(y == 4064.0)     # -32 * -127


def test_scale_fields_against_the_bit_layout():
    rng = np.random.default_rng(3)
    for _ in range(200):
        blk = rng.integers(0, 256, 136, dtype=np.uint8)
        sh = int(blk[2]) | (int(blk[3]) << 8)
        assert [orc.iq4xs_scale(sh, blk[4:8], ib) for ib in range(8)] == [scale(blk, ib) for ib in range(8)]
    # one field at a time: sub-block 5 = high nibble of scales_l[2], bits 10-11 of scales_h
    assert orc.iq4xs_scale(0b10 << 10, np.array([0, 0, 0xB0, 0], np.uint8), 5) == (0x0B | (2 << 4)) - 32
    assert orc.iq4xs_scale(0b10 << 10, np.array([0, 0, 0xB0, 0], np.uint8), 4) == -32


def test_hand_block_gives_every_subblock_and_nibble_its_own_value():
    # sub-block ib: ls = 33 + ib (low nibble 1 + ib, top bits 2), so ls - 32 = 1 + ib;
    # qs[16 ib + j] = j | ((15 - j) << 4): element j has code j, element 16 + j code 15 - j
    b = np.zeros(136, np.uint8)
    b[0:2] = h16(0.5)
    sh = 0
    for ib in range(8):
        sh |= 2 << (2 * ib)
        b[4 + ib // 2] |= (1 + ib) << (4 * (ib % 2))
        b[8 + 16 * ib:8 + 16 * ib + 16] = [j | ((15 - j) << 4) for j in range(16)]
    b[2], b[3] = sh & 0xFF, sh >> 8
    y = orc.dequant_block(orc.IQ4_XS, b)
    for e in range(256):
        ib, hi, j = e // 32, (e // 16) % 2, e % 16
        assert y[e] == np.float32(0.5 * (1 + ib) * KV[15 - j if hi else j]), e


def test_dequant_block_matches_independent_decoder_bit_for_bit():
    w = orc.synth_weight(orc.IQ4_XS, 256 * 6, 0x41)
    y = orc.dequant_block(orc.IQ4_XS, w)
    for b in range(6):
        blk = w[b * 136:(b + 1) * 136]
        want = np.array([element(blk, e)[0] for e in range(256)], np.float32)
        assert np.array_equal(y[b * 256:(b + 1) * 256].view(np.uint32), want.view(np.uint32)), b


def test_synth_scale_slot():
    w = orc.synth_weight(orc.IQ4_XS, 512, 7)
    for b in range(2):
        assert f16(w[136 * b], w[136 * b + 1]) == np.float32(np.float16(0.06))
    assert orc.block_layout(orc.IQ4_XS) == (256, 136)


@pytest.mark.parametrize("in_f", [256, 1024])
def test_stage_and_terms(in_f):
    rng = np.random.default_rng(6 + in_f)
    row = orc.synth_weight(orc.IQ4_XS, in_f, 0x9B)
    x = rng.standard_normal(in_f).astype(np.float32)
    q8 = orc.quantize_q8(x)
    y, isum = orc.vec_dot_iq4xs(row, q8, in_f, stages=True)
    acc = np.float32(0.0)
    for b in range(in_f // 256):
        blk = row[136 * b:136 * (b + 1)]
        codes = np.array([element(blk, e)[1] for e in range(256)], np.int64)
        q = q8.qs[256 * b:256 * (b + 1)].astype(np.int64)
        want = sum(scale(blk, ib) * int((codes[32 * ib:32 * ib + 32] * q[32 * ib:32 * ib + 32]).sum()) for ib in range(8))
        assert isum[b] == want
        d = f16(blk[0], blk[1])
        acc = np.float32(acc + np.float32(np.float32(d * q8.d[b]) * np.float32(want)))
    assert np.float32(y).view(np.uint32) == acc.view(np.uint32)


def test_dot_matches_dequant_reference():
    in_f = 1024
    rng = np.random.default_rng(63)
    row = orc.synth_weight(orc.IQ4_XS, in_f, 0x51)
    x = rng.uniform(-1, 1, in_f).astype(np.float32)
    q8 = orc.quantize_q8(x)
    y = orc.vec_dot_iq4xs(row, q8, in_f)
    wf = orc.dequant_block(orc.IQ4_XS, row).astype(np.float64)
    xq = q8.qs.astype(np.float64) * np.repeat(q8.d.astype(np.float64), 256)
    ref = float(wf @ xq)
    assert abs(float(y) - ref) <= 1e-3 * max(1.0, abs(ref))


def test_linear_dispatch():
    # production arm = the per-256 int8 kernel row by row (batch == single); reference mode = f32 dot of
    # the decoded row; the two agree to the reference's 2e-2 of max|f64 oracle|
    dtype, in_f, out_f, m = orc.IQ4_XS, 512, 9, 3
    rng = np.random.default_rng(93)
    w = orc.synth_weight(dtype, out_f * in_f, 0x61)
    x = rng.standard_normal(m * in_f).astype(np.float32)
    y = orc.linear(dtype, w, x, m, in_f, out_f)
    bpr = w.size // out_f
    for r in range(m):
        q8 = orc.quantize_q8(x[r * in_f:(r + 1) * in_f])
        for o in range(out_f):
            one = orc.vec_dot_iq4xs(w[o * bpr:(o + 1) * bpr], q8, in_f)
            assert np.float32(y[r, o]).view(np.uint32) == np.float32(one).view(np.uint32)
    y1 = orc.linear(dtype, w, x[:in_f], 1, in_f, out_f)
    assert np.array_equal(y1.view(np.uint32), y[:1].view(np.uint32))
    wf = orc.dequant_block(dtype, w).reshape(out_f, in_f)
    f64 = orc.ref_linear_f64(x, wf, m, in_f, out_f)
    yr = orc.linear(dtype, w, x, m, in_f, out_f, reference_mode=True)
    bound = 2e-2 * np.abs(f64).max()
    assert np.abs(y - f64).max() <= bound and np.abs(yr - f64).max() <= 1e-5 * max(1.0, np.abs(f64).max()) + 1e-4
    a, b = orc.linear_int_stages(dtype, w, x, m, in_f, out_f)
    assert a.shape == (m, out_f, in_f // 256) and b is None
    with pytest.raises(Exception):
        orc.linear(dtype, w[:136], x[:128], 1, 128, 1)      # rows are whole superblocks
