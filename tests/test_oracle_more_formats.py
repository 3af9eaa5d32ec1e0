"""Pins the oracle's restatement of Q5_K, Q4_0, Q4_1, Q5_0, Q5_1 and IQ4_NL: the reference's own
single-block known answers (crates/infr-gguf/src/dequant.rs:1229-1246, 1736-1843), independent
element-at-a-time numpy decoders on random bytes, brute-force int64 integer stages, the per-block
f32 expression evaluated independently, and dot(dequant) at the reference's 1e-3
(crates/infr-cpu/src/kernels.rs:6700-6730)."""
import numpy as np
import pytest

from oracle import oracle as orc

BLK32 = [orc.Q4_0, orc.Q4_1, orc.Q5_0, orc.Q5_1, orc.IQ4_NL]
NAMES = {orc.Q4_0: "q4_0", orc.Q4_1: "q4_1", orc.Q5_0: "q5_0", orc.Q5_1: "q5_1", orc.IQ4_NL: "iq4_nl",
         orc.Q5_K: "q5_k"}


def h16(v):
    return np.frombuffer(np.float16(v).tobytes(), np.uint8)


def f16(b0, b1):
    return np.float32(np.frombuffer(bytes([int(b0), int(b1)]), np.float16)[0])


# ───────────── the reference's single-block known answers ─────────────

def test_reference_known_answers():
    b = np.zeros(18, np.uint8)                      # q4_0_single_block
    b[0:2], b[2], b[3:] = h16(2.0), 0x89, 0x88
    y = orc.dequant_block(orc.Q4_0, b)
    assert y.size == 32 and y[0] == 2.0 and y[16] == 0.0 and y[1] == 0.0

    b = np.zeros(20, np.uint8)                      # q4_1_single_block
    b[0:2], b[2:4], b[4] = h16(1.0), h16(0.5), 0x30
    y = orc.dequant_block(orc.Q4_1, b)
    assert y[0] == 0.5 and y[16] == 3.5

    b = np.zeros(22, np.uint8)                      # q5_0_single_block
    b[0:2], b[2], b[6] = h16(1.0), 0x01, 0x0F
    y = orc.dequant_block(orc.Q5_0, b)
    assert y[0] == 15.0 and y[16] == -16.0

    b = np.zeros(24, np.uint8)                      # q5_1_single_block
    b[0:2], b[2:4], b[8] = h16(2.0), h16(-1.0), 0x1F
    y = orc.dequant_block(orc.Q5_1, b)
    assert y[0] == 29.0 and y[16] == 1.0

    b = np.zeros(18, np.uint8)                      # iq4nl_single_block
    b[0:2], b[2] = h16(1.0), 0x80
    y = orc.dequant_block(orc.IQ4_NL, b)
    assert y.size == 32 and y[0] == -127.0 and y[16] == 1.0


def test_q5_0_high_bits_reach_both_halves():
    # qh bit j is element j's 5th bit, qh bit j+16 element j+16's: set bit 3 and bit 16+5 only
    b = np.zeros(22, np.uint8)
    b[0:2] = h16(1.0)
    b[2:6] = np.frombuffer(((1 << 3) | (1 << 21)).to_bytes(4, "little"), np.uint8)
    y = orc.dequant_block(orc.Q5_0, b)
    want = np.full(32, -16.0, np.float32)
    want[3] = want[21] = 0.0
    assert np.array_equal(y, want)


def test_q5_k_hand_block():
    # d=1, dmin=.5; scales bytes 0..3 = 1 (sc of sub-blocks 0..3), bytes 4..7 = 2 (m of 0..3), the
    # rest 0x11 / so sub-blocks 4..7 take sc = 1, m = 1 from bytes 8..11 (low / high nibble).
    b = np.zeros(176, np.uint8)
    b[0:2], b[2:4] = h16(1.0), h16(0.5)
    b[4:8], b[8:12], b[12:16] = 1, 2, 0x11
    b[48:176] = 0x23                                # low nibble 3 (even sub-blocks), high 2 (odd)
    b[16:48] = 0b00000110                           # qh: bit 1 (sub-block 1) and bit 2 (sub-block 2)
    y = orc.dequant_block(orc.Q5_K, b)
    code = {0: 3, 1: 2 + 16, 2: 3 + 16, 3: 2, 4: 3, 5: 2, 6: 3, 7: 2}
    m = {s: 2 if s < 4 else 1 for s in range(8)}
    for s in range(8):
        assert np.all(y[s * 32:(s + 1) * 32] == 1.0 * code[s] - 0.5 * m[s]), s


# ───────────── independent decoders on random bytes ─────────────

def k4_independent(j, q):
    if j < 4:
        return q[j] & 63, q[j + 4] & 63
    return (q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4), (q[j + 4] >> 4) | ((q[j] >> 6) << 4)


def codes_blk32(dtype, blk):
    """The 32 integer code values of one block, element order (IQ4_NL: codebook values)."""
    affine, five = dtype in (orc.Q4_1, orc.Q5_1), dtype in (orc.Q5_0, orc.Q5_1)
    p = 4 if affine else 2
    qh = int.from_bytes(bytes(blk[p:p + 4]), "little") if five else 0
    qs = blk[p + (4 if five else 0):]
    out = []
    for e in range(32):
        byte = int(qs[e % 16])
        c = byte >> 4 if e >= 16 else byte & 15
        if five:
            c |= ((qh >> e) & 1) << 4
        out.append(orc.KVALUES_IQ4NL[c] if dtype == orc.IQ4_NL else c)
    return np.array(out, np.int64)


def codes_q5k(blk):
    out = np.empty(256, np.int64)
    for e in range(256):
        s, l = divmod(e, 32)
        byte = int(blk[48 + (s // 2) * 32 + l])
        out[e] = (byte >> 4 if s % 2 else byte & 15) + 16 * ((int(blk[16 + l]) >> s) & 1)
    return out


def decode_independent(dtype, blk):
    if dtype == orc.Q5_K:
        d, dmin = f16(blk[0], blk[1]), f16(blk[2], blk[3])
        c = codes_q5k(blk)
        out = np.empty(256, np.float32)
        for e in range(256):
            sc, m = k4_independent(e // 32, [int(v) for v in blk[4:16]])
            out[e] = np.float32(d * np.float32(sc)) * np.float32(c[e]) + np.float32(dmin * np.float32(-m))
        return out
    d = f16(blk[0], blk[1])
    c = codes_blk32(dtype, blk)
    if dtype == orc.IQ4_NL:
        return np.array([d * np.float32(v) for v in c], np.float32)
    if dtype in (orc.Q4_1, orc.Q5_1):
        mn = np.float32(f16(blk[2], blk[3]) * np.float32(1))
    else:
        mn = np.float32(d * np.float32(-16 if dtype == orc.Q5_0 else -8))
    return np.array([np.float32(d * np.float32(1)) * np.float32(v) + mn for v in c], np.float32)


@pytest.mark.parametrize("dtype", BLK32 + [orc.Q5_K], ids=lambda d: NAMES[d])
def test_dequant_block_matches_independent_decoder_bit_for_bit(dtype):
    e, b = orc.block_layout(dtype)
    raw = orc.synth_weight(dtype, e * 6, 0x5EED)
    got = orc.dequant_block(dtype, raw)
    for i in range(6):
        want = decode_independent(dtype, raw[i * b:(i + 1) * b])
        assert np.array_equal(got[i * e:(i + 1) * e].view(np.uint32), want.view(np.uint32)), f"block {i}"


def test_synth_scale_slots():
    # crates/infr-testkit/src/lib.rs:73-93
    for dt, d, mn in ((orc.Q4_0, 0.04, None), (orc.Q5_0, 0.04, None), (orc.Q4_1, 0.04, -0.30),
                      (orc.Q5_1, 0.04, -0.30), (orc.Q5_K, 0.05, 0.10), (orc.IQ4_NL, 0.004, None)):
        e, b = orc.block_layout(dt)
        w = orc.synth_weight(dt, 2 * e, 9)
        assert np.array_equal(w[b:b + 2], h16(d))
        if mn is not None:
            assert np.array_equal(w[b + 2:b + 4], h16(mn))
        skip = 4 if mn is not None else 2
        assert np.array_equal(w[b + skip:2 * b], orc.lcg_bytes(9 ^ 1, b)[skip:])


# ───────────── integer stages and the per-block f32 expression ─────────────

@pytest.mark.parametrize("dtype", BLK32, ids=lambda d: NAMES[d])
@pytest.mark.parametrize("in_f", [32, 96, 1024])
def test_blk32_stages_and_terms(dtype, in_f):
    e, b = orc.block_layout(dtype)
    w = orc.synth_weight(dtype, in_f, 77 + in_f)
    x = orc.det_x(in_f, 5 + dtype)
    q = orc.quantize_q8_32(x)
    y, ip = orc.vec_dot_blk32(dtype, w, q, in_f, stages=True)
    sumf = np.float32(0)
    for k in range(in_f // 32):
        blk = w[k * b:(k + 1) * b]
        c = codes_blk32(dtype, blk)
        want_ip = int((c * q.qs[k * 32:(k + 1) * 32].astype(np.int64)).sum())
        assert ip[k] == want_ip
        d, d8 = f16(blk[0], blk[1]), q.d[k]
        ipf, bsf = np.float32(want_ip), np.float32(q.bsum[k])
        if dtype in (orc.Q4_1, orc.Q5_1):
            term = d8 * np.float32(np.float32(d * ipf) + np.float32(f16(blk[2], blk[3]) * bsf))
        elif dtype == orc.IQ4_NL:
            term = np.float32(d * d8) * ipf
        else:
            off = np.float32(16.0 if dtype == orc.Q5_0 else 8.0)
            term = np.float32(d * d8) * np.float32(ipf - np.float32(off * bsf))
        sumf = np.float32(sumf + np.float32(term))
    assert np.float32(y).view(np.uint32) == sumf.view(np.uint32)


@pytest.mark.parametrize("in_f", [256, 1024])
def test_q5k_stages_and_terms(in_f):
    w = orc.synth_weight(orc.Q5_K, in_f, 1234)
    x = orc.det_x(in_f, 42)
    q = orc.quantize_q8(x)
    y, sd, sm = orc.vec_dot_q5k(w, q, in_f, stages=True)
    sumf = np.float32(0)
    for k in range(in_f // 256):
        blk = w[k * 176:(k + 1) * 176]
        c = codes_q5k(blk)
        sdw = smw = 0
        for s in range(8):
            sc, m = k4_independent(s, [int(v) for v in blk[4:16]])
            sdw += sc * int((c[s * 32:(s + 1) * 32] * q.qs[k * 256 + s * 32:k * 256 + (s + 1) * 32].astype(np.int64)).sum())
            smw += m * int(q.bsums[k * 8 + s])
        assert (sd[k], sm[k]) == (sdw, smw)
        d, dmin = f16(blk[0], blk[1]), f16(blk[2], blk[3])
        term = q.d[k] * np.float32(np.float32(d * np.float32(sdw)) - np.float32(dmin * np.float32(smw)))
        sumf = np.float32(sumf + np.float32(term))
    assert np.float32(y).view(np.uint32) == sumf.view(np.uint32)


@pytest.mark.parametrize("dtype", BLK32 + [orc.Q5_K], ids=lambda d: NAMES[d])
def test_dot_matches_dequant_reference(dtype):
    """The integer kernel equals dot(dequant(w), dequant(q8)) up to f32 summation order: the
    activation rounding is common to both sides (kernels.rs:6700-6730, tolerance 1e-3)."""
    in_f = 1024
    w = orc.synth_weight(dtype, in_f, 31)
    x = orc.det_x(in_f, 3)
    wf = orc.dequant_block(dtype, w).astype(np.float64)
    if dtype == orc.Q5_K:
        q = orc.quantize_q8(x)
        xq = q.qs.astype(np.float64) * np.repeat(q.d.astype(np.float64), 256)
        y = orc.vec_dot_q5k(w, q, in_f)
    else:
        q = orc.quantize_q8_32(x)
        xq = q.qs.astype(np.float64) * np.repeat(q.d.astype(np.float64), 32)
        y = orc.vec_dot_blk32(dtype, w, q, in_f)
    want = float(wf @ xq)
    assert abs(float(y) - want) <= 1e-3 * max(1.0, abs(want))


# ───────────── Op::Linear dispatch ─────────────

@pytest.mark.parametrize("dtype", BLK32 + [orc.Q5_K], ids=lambda d: NAMES[d])
def test_linear_dispatch(dtype):
    in_f, out_f = 512, 6
    w = orc.synth_weight(dtype, in_f * out_f, 8)
    x = orc.gen_f32(3 * in_f, 2)
    y3 = orc.linear(dtype, w, x, 3, in_f, out_f)
    y1 = orc.linear(dtype, w, x[:in_f], 1, in_f, out_f)
    yr = orc.linear(dtype, w, x[:in_f], 1, in_f, out_f, reference_mode=True)
    if dtype == orc.Q5_0:
        # no one-token int8 arm: decode takes dequant + f32 dot (lib.rs:1165); m >= 2 the int8 kernel
        assert np.array_equal(y1, yr) and not np.array_equal(y3[0], y1[0])
        q = orc.quantize_q8_32(x[:in_f])
        e, b = orc.block_layout(dtype)
        assert y3[0, 1] == orc.vec_dot_blk32(dtype, w[in_f // e * b:2 * in_f // e * b], q, in_f)
    else:
        assert np.array_equal(y3[0], y1[0])            # batch == single, bit for bit
    wf = orc.dequant_block(dtype, w).reshape(out_f, in_f)
    want = orc.ref_linear_f64(x, wf, 3, in_f, out_f)
    assert np.abs(y3 - want).max() <= 2e-2 * max(1.0, np.abs(want).max())
    bad = 48 if dtype != orc.Q5_K else 128
    with pytest.raises(ValueError):
        orc.linear(dtype, w[:10 * orc.block_layout(dtype)[1]], x, 1, bad, 1)
    ia, ib = orc.linear_int_stages(dtype, w, x, 2, in_f, out_f)
    assert ia.shape == (2, out_f, in_f // (256 if dtype == orc.Q5_K else 32))
    assert (ib is not None) == (dtype == orc.Q5_K)
