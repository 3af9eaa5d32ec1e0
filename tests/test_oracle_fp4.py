"""Pins the oracle's restatement of MXFP4 and NVFP4: the reference's single-block known answers
(crates/infr-gguf/src/dequant.rs:1307-1345), the two scale decoders against their definitions
(every E8M0 byte is 2^(x - 128); every UE4M3 byte against the OCP FP8 E4M3 value, halved),
hand blocks that give every nibble position its own code, independent element-at-a-time numpy
decoders on random bytes, brute-force int64 integer stages, the per-block f32 expression
evaluated independently, and dot(dequant) at the reference's 1e-3."""
import numpy as np
import pytest

from oracle import oracle as orc

# the E2M1 values 0, 0.5, 1, 1.5, 2, 3, 4, 6 and their negatives, doubled (ggml-common.h
# kvalues_mxfp4; the reference quotes the same table, crates/infr-gguf/src/dequant.rs:405)
KV = np.array([0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12], np.int64)
assert [int(2 * v) for v in (0, .5, 1, 1.5, 2, 3, 4, 6)] == list(KV[:8]) and list(-KV[:8]) == list(KV[8:])


def test_reference_known_answers():
    b = np.zeros(17, np.uint8)                      # mxfp4_single_block
    b[0], b[1] = 128, 0x21
    y = orc.dequant_block(orc.MXFP4, b)
    assert y.size == 32 and y[0] == 1.0 and y[16] == 2.0 and np.all(y[1:16] == 0.0) and np.all(y[17:] == 0.0)
    y = orc.dequant_block(orc.NVFP4, np.zeros(36, np.uint8))     # nvfp4_single_block
    assert y.size == 64 and np.all(y == 0.0)
    assert orc.block_layout(orc.MXFP4) == (32, 17) and orc.block_layout(orc.NVFP4) == (64, 36)


def test_e8m0_is_a_power_of_two_halved():
    for x in range(256):
        assert float(orc.e8m0_half(x)) == 2.0 ** (x - 128), x      # exact in f32, subnormals included


def test_ue4m3_against_the_fp8_definition():
    """E4M3 without a sign: exponent bias 7, subnormals m/8 * 2^-6, then halved. 0x7F (the NaN
    pattern of the signed format's positive half) decodes to 0 like 0; bit 7 is ignored."""
    for x in range(256):
        e, m = (x >> 3) & 15, x & 7
        want = 0.0 if x in (0, 0x7F) else 0.5 * ((m / 8) * 2.0 ** -6 if e == 0 else (1 + m / 8) * 2.0 ** (e - 7))
        assert float(orc.ue4m3_half(x)) == want, x
    assert float(orc.ue4m3_half(0x38)) == 0.5 and float(orc.ue4m3_half(0x7E)) == 224.0


def mxfp4_element(blk, e):
    code = int(KV[(int(blk[1 + e % 16]) >> (4 * (e // 16))) & 15])
    return np.float32(np.float32(code) * orc.e8m0_half(blk[0])), code


def nvfp4_element(blk, e):
    sb, hi, j = e // 16, (e // 8) % 2, e % 8
    code = int(KV[(int(blk[4 + 8 * sb + j]) >> (4 * hi)) & 15])
    return np.float32(np.float32(code) * orc.ue4m3_half(blk[sb])), code


def test_hand_blocks_give_every_nibble_position_its_own_code():
    b = np.zeros(17, np.uint8)
    b[0] = 127                                              # d = 0.5
    b[1:17] = [j | ((15 - j) << 4) for j in range(16)]
    y = orc.dequant_block(orc.MXFP4, b)
    for e in range(32):
        assert y[e] == 0.5 * KV[e if e < 16 else 15 - (e - 16)], e
    b = np.zeros(36, np.uint8)
    b[0:4] = [0x38, 0x40, 0x30, 0x3C]                       # 0.5, 1.0, 0.25, 0.75
    for sb in range(4):
        b[4 + 8 * sb:12 + 8 * sb] = [((j + 2 * sb) % 16) | (((15 - j - sb) % 16) << 4) for j in range(8)]
    y = orc.dequant_block(orc.NVFP4, b)
    for e in range(64):
        sb, hi, j = e // 16, (e // 8) % 2, e % 8
        code = (15 - j - sb) % 16 if hi else (j + 2 * sb) % 16
        assert y[e] == (0.5, 1.0, 0.25, 0.75)[sb] * KV[code], e


@pytest.mark.parametrize("dtype", [orc.MXFP4, orc.NVFP4])
def test_dequant_block_matches_independent_decoder_bit_for_bit(dtype):
    e, bpb = orc.block_layout(dtype)
    rng = np.random.default_rng(dtype)
    w = rng.integers(0, 256, bpb * 24, dtype=np.uint8)      # every scale byte value is finite for both
    y = orc.dequant_block(dtype, w)
    el = mxfp4_element if dtype == orc.MXFP4 else nvfp4_element
    for b in range(24):
        blk = w[b * bpb:(b + 1) * bpb]
        want = np.array([el(blk, i)[0] for i in range(e)], np.float32)
        assert np.array_equal(y[b * e:(b + 1) * e].view(np.uint32), want.view(np.uint32)), b


def test_synth_scale_slots():
    w = orc.synth_weight(orc.MXFP4, 64, 7)
    assert w[0] == 125 and w[17] == 125                     # 2^-2 = 0.25 as 2^(e - 127); decoded halved
    w = orc.synth_weight(orc.NVFP4, 128, 7)
    for b in range(2):
        got = [2 * float(orc.ue4m3_half(w[36 * b + i])) for i in range(4)]
        assert got == [0.5 * (0.625 + 0.125 * i) for i in range(4)]


@pytest.mark.parametrize("dtype", [orc.MXFP4, orc.NVFP4])
@pytest.mark.parametrize("in_f", [64, 1024])
def test_stages_and_terms(dtype, in_f):
    rng = np.random.default_rng(6 + in_f + dtype)
    row = orc.synth_weight(dtype, in_f, 0x9C)
    x = rng.standard_normal(in_f).astype(np.float32)
    q8 = orc.quantize_q8_32(x)
    y, ip = orc.vec_dot_fp4(dtype, row, q8, in_f, stages=True)
    e, bpb = orc.block_layout(dtype)
    acc = np.float32(0.0)
    for b in range(in_f // e):
        blk = row[bpb * b:bpb * (b + 1)]
        el = mxfp4_element if dtype == orc.MXFP4 else nvfp4_element
        codes = np.array([el(blk, i)[1] for i in range(e)], np.int64)
        q = q8.qs[e * b:e * (b + 1)].astype(np.int64)
        if dtype == orc.MXFP4:
            want = int((codes * q).sum())
            assert ip[b] == want
            acc = np.float32(acc + np.float32(np.float32(orc.e8m0_half(blk[0]) * q8.d[b]) * np.float32(want)))
        else:
            for sb in range(4):
                want = int((codes[16 * sb:16 * sb + 16] * q[16 * sb:16 * sb + 16]).sum())
                assert ip[4 * b + sb] == want
                acc = np.float32(acc + np.float32(np.float32(orc.ue4m3_half(blk[sb]) * q8.d[2 * b + sb // 2]) * np.float32(want)))
    assert np.float32(y).view(np.uint32) == acc.view(np.uint32)


@pytest.mark.parametrize("dtype", [orc.MXFP4, orc.NVFP4])
def test_dot_matches_dequant_reference(dtype):
    in_f = 1024
    rng = np.random.default_rng(63 + dtype)
    row = orc.synth_weight(dtype, in_f, 0x51)
    x = rng.uniform(-1, 1, in_f).astype(np.float32)
    q8 = orc.quantize_q8_32(x)
    y = orc.vec_dot_fp4(dtype, row, q8, in_f)
    wf = orc.dequant_block(dtype, row).astype(np.float64)
    xq = q8.qs.astype(np.float64) * np.repeat(q8.d.astype(np.float64), 32)
    ref = float(wf @ xq)
    assert abs(float(y) - ref) <= 1e-3 * max(1.0, abs(ref))


@pytest.mark.parametrize("dtype", [orc.MXFP4, orc.NVFP4])
def test_linear_dispatch(dtype):
    # the per-32 int8 kernel row by row at every token count, one token included
    # (crates/infr-cpu/src/lib.rs:1066-1076, 1145-1160, 1394-1432); reference mode = f32 dot of the decoded row
    in_f, out_f, m = 512, 9, 3
    rng = np.random.default_rng(93 + dtype)
    w = orc.synth_weight(dtype, out_f * in_f, 0x61)
    x = rng.standard_normal(m * in_f).astype(np.float32)
    y = orc.linear(dtype, w, x, m, in_f, out_f)
    bpr = w.size // out_f
    for r in range(m):
        q8 = orc.quantize_q8_32(x[r * in_f:(r + 1) * in_f])
        for o in range(out_f):
            one = orc.vec_dot_fp4(dtype, w[o * bpr:(o + 1) * bpr], q8, in_f)
            assert np.float32(y[r, o]).view(np.uint32) == np.float32(one).view(np.uint32)
    y1 = orc.linear(dtype, w, x[:in_f], 1, in_f, out_f)
    assert np.array_equal(y1.view(np.uint32), y[:1].view(np.uint32))
    wf = orc.dequant_block(dtype, w).reshape(out_f, in_f)
    f64 = orc.ref_linear_f64(x, wf, m, in_f, out_f)
    yr = orc.linear(dtype, w, x, m, in_f, out_f, reference_mode=True)
    bound = 2e-2 * np.abs(f64).max()
    assert np.abs(y - f64).max() <= bound and np.abs(yr - f64).max() <= 1e-5 * max(1.0, np.abs(f64).max()) + 1e-4
    a, b = orc.linear_int_stages(dtype, w, x, m, in_f, out_f)
    assert a.shape == (m, out_f, in_f // (32 if dtype == orc.MXFP4 else 16)) and b is None
    with pytest.raises(Exception):
        orc.linear(dtype, w, x, 1, in_f - 16, 1)            # rows are whole blocks
