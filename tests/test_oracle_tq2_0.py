"""Pins the oracle's restatement of TQ2_0: the reference's single-block known answer
(crates/infr-gguf/src/dequant.rs:1385-1398), a hand block with a different code in every bit pair,
an independent element-at-a-time numpy decoder on random bytes, the integer stage as an int64 sum
(and through the identity sum (q - 1) a = sum q a - sum a), the f32 expression evaluated
independently, and dot(dequant) at the reference's 1e-3."""
import numpy as np
import pytest

from oracle import oracle as orc


def f16(b0, b1):
    return np.float32(np.frombuffer(bytes([int(b0), int(b1)]), np.float16)[0])


def element(blk, e):
    """Element e = 128 chunk + 32 l + m reads bit pair l of qs[32 chunk + m]; value (q - 1) d."""
    chunk, l, m = e // 128, (e // 32) % 4, e % 32
    q = (int(blk[32 * chunk + m]) >> (2 * l)) & 3
    return np.float32(np.float32(q - 1) * f16(blk[64], blk[65])), q - 1


def test_reference_known_answer_and_hand_block():
    b = np.zeros(66, np.uint8)                      # tq2_0_single_block
    b[64:66] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    y = orc.dequant_block(orc.TQ2_0, b)
    assert y.size == 256 and np.all(y == -1.0)
    b[0:64] = 0b11100100                            # bit pair l holds l
    b[64:66] = np.frombuffer(np.float16(0.5).tobytes(), np.uint8)
    y = orc.dequant_block(orc.TQ2_0, b)
    for e in range(256):
        assert y[e] == 0.5 * ((e // 32) % 4 - 1), e
    assert orc.block_layout(orc.TQ2_0) == (256, 66)


def test_dequant_block_matches_independent_decoder_bit_for_bit():
    w = orc.synth_weight(orc.TQ2_0, 256 * 6, 0x43)
    assert f16(w[64], w[65]) == np.float32(np.float16(0.05))
    y = orc.dequant_block(orc.TQ2_0, w)
    for b in range(6):
        blk = w[b * 66:(b + 1) * 66]
        want = np.array([element(blk, e)[0] for e in range(256)], np.float32)
        assert np.array_equal(y[b * 256:(b + 1) * 256].view(np.uint32), want.view(np.uint32)), b


@pytest.mark.parametrize("in_f", [256, 1024])
def test_stage_and_terms(in_f):
    rng = np.random.default_rng(6 + in_f)
    row = orc.synth_weight(orc.TQ2_0, in_f, 0x9D)
    x = rng.standard_normal(in_f).astype(np.float32)
    q8 = orc.quantize_q8(x)
    y, ip = orc.vec_dot_tq2_0(row, q8, in_f, stages=True)
    acc = np.float32(0.0)
    for b in range(in_f // 256):
        blk = row[66 * b:66 * (b + 1)]
        codes = np.array([element(blk, e)[1] for e in range(256)], np.int64)
        q = q8.qs[256 * b:256 * (b + 1)].astype(np.int64)
        want = int((codes * q).sum())
        assert ip[b] == want == int(((codes + 1) * q).sum()) - int(q8.bsums[8 * b:8 * b + 8].sum())
        acc = np.float32(acc + np.float32(np.float32(f16(blk[64], blk[65]) * q8.d[b]) * np.float32(want)))
    assert np.float32(y).view(np.uint32) == acc.view(np.uint32)


def test_dot_matches_dequant_reference_and_linear_dispatch():
    dtype, in_f, out_f, m = orc.TQ2_0, 1024, 9, 3
    rng = np.random.default_rng(77)
    w = orc.synth_weight(dtype, out_f * in_f, 0x61)
    x = rng.uniform(-1, 1, m * in_f).astype(np.float32)
    y = orc.linear(dtype, w, x, m, in_f, out_f)
    bpr = w.size // out_f
    wf = orc.dequant_block(dtype, w).reshape(out_f, in_f).astype(np.float64)
    for r in range(m):
        q8 = orc.quantize_q8(x[r * in_f:(r + 1) * in_f])
        xq = q8.qs.astype(np.float64) * np.repeat(q8.d.astype(np.float64), 256)
        for o in range(out_f):
            one = orc.vec_dot_tq2_0(w[o * bpr:(o + 1) * bpr], q8, in_f)
            assert np.float32(y[r, o]).view(np.uint32) == np.float32(one).view(np.uint32)   # batch == single
            ref = float(wf[o] @ xq)
            assert abs(float(one) - ref) <= 1e-3 * max(1.0, abs(ref))
    f64 = orc.ref_linear_f64(x, wf.astype(np.float32), m, in_f, out_f)
    yr = orc.linear(dtype, w, x, m, in_f, out_f, reference_mode=True)
    assert np.abs(y - f64).max() <= 2e-2 * np.abs(f64).max()
    assert np.abs(yr - f64).max() <= 1e-5 * max(1.0, np.abs(f64).max()) + 1e-4
    a, b = orc.linear_int_stages(dtype, w, x, m, in_f, out_f)
    assert a.shape == (m, out_f, in_f // 256) and b is None
