"""Pins the CPU oracle's format layer (f16, k4, block geometry, host decode) against evidence that
does not come from the oracle's own code: the reference's known-answer test, hand-derived block
vectors, ggml's size formulas, numpy's IEEE float16, and independent byte-at-a-time decoders
written here from the format descriptions (a second decoder, the way the reference cross-checks
its kernel decode against dequant_block, crates/infr-cpu/tests/decode_parity.rs:7-11).
"""
import numpy as np
import pytest

from oracle import oracle as orc


# ───────────── f16 ─────────────

def test_f16_widening_matches_ieee_for_all_65536_patterns():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([orc.f16_bits_to_f32(int(b)) for b in bits], np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f16_narrowing_round_trip_and_rne():
    # every finite f16 survives f16 -> f32 -> f16
    bits = np.arange(65536, dtype=np.uint16)
    vals = bits.view(np.float16).astype(np.float32)
    for b, v in zip(bits[::7], vals[::7]):
        if np.isfinite(v):
            assert orc.f32_to_f16_bits(float(v)) == int(b)
    # round-to-nearest-even against numpy on a spread of magnitudes (incl. subnormal, overflow)
    rng = np.random.default_rng(0)
    xs = np.concatenate([rng.standard_normal(4000) * s for s in (1e-8, 1e-5, 1e-3, 1.0, 100.0, 7e4)])
    xs = xs.astype(np.float32)
    want = xs.astype(np.float16).view(np.uint16)
    got = np.array([orc.f32_to_f16_bits(float(x)) for x in xs], np.uint16)
    assert np.array_equal(got, want)
    # exact ties: 1 + 2^-11 is halfway between two f16 values -> even mantissa
    assert orc.f32_to_f16_bits(1.0 + 2.0 ** -11) == 0x3C00
    assert orc.f32_to_f16_bits(1.0 + 3 * 2.0 ** -11) == 0x3C02


# ───────────── geometry ─────────────

def test_block_bytes_match_the_ggml_formulas():
    # crates/infr-core/src/decode_spec.rs:455-504 restates them as formulas; so does this.
    QK_K = 256
    assert orc.block_layout(orc.Q8_0) == (32, 2 + 32)
    assert orc.block_layout(orc.Q4_K) == (QK_K, 2 * 2 + 12 + QK_K // 2)
    assert orc.block_layout(orc.Q6_K) == (QK_K, QK_K // 2 + QK_K // 4 + QK_K // 16 + 2)
    assert orc.block_layout(orc.Q2_0) == (64, 2 + 64 // 4)


# ───────────── k4 ─────────────

def k4_independent(j, q):
    """llama.cpp get_scale_min_k4 written from the bit layout: six low bits of bytes 0-3 / 4-7
    for j < 4; for j >= 4 the low nibble / high nibble of byte j+4 plus the top two bits of
    bytes j-4 / j as bits 4-5."""
    if j < 4:
        return q[j] % 64, q[j + 4] % 64
    return (q[j + 4] % 16) + 16 * (q[j - 4] // 64), (q[j + 4] // 16) + 16 * (q[j] // 64)


def test_k4_hand_vector_with_split_high_bits():
    scales = bytes.fromhex("81000000C200000025000000")
    got = [orc.k4(j, np.frombuffer(scales, np.uint8)) for j in range(8)]
    assert got[0] == (1, 2)
    assert got[4] == (37, 50)      # 5 | (2 << 4), 2 | (3 << 4)
    assert all(g == (0, 0) for i, g in enumerate(got) if i not in (0, 4))


def test_k4_matches_independent_restatement_on_random_bytes():
    rng = np.random.default_rng(1)
    for _ in range(500):
        q = rng.integers(0, 256, 12, dtype=np.uint8)
        for j in range(8):
            assert orc.k4(j, q) == k4_independent(j, [int(v) for v in q])


# ───────────── host decode: known answers ─────────────

def test_q2_0_single_block_reference_known_answer():
    # crates/infr-gguf/src/dequant.rs:1405-1428
    blk = np.zeros(18, np.uint8)
    blk[0:2] = np.frombuffer(np.float16(0.5).tobytes(), np.uint8)
    blk[2] = 0b11100100
    y = orc.dequant_block(orc.Q2_0, blk)
    assert y.shape == (64,)
    assert np.allclose(y[:4], [-0.5, 0.0, 0.5, 1.0], atol=1e-4)
    assert np.allclose(y[4:], -0.5, atol=1e-4)


HAND_BLOCKS = {
    # every decoded weight is exactly 2.0 (derivations in the test names below)
    orc.Q4_K: bytes.fromhex("003C" "0038" "010101010202020221212121") + b"\x33" * 128,
    orc.Q6_K: b"\x11" * 128 + b"\xAA" * 64 + b"\x02" * 16 + bytes.fromhex("003C"),
    orc.Q8_0: (bytes.fromhex("0038") + b"\x04" * 32) * 8,
    orc.Q2_0: (bytes.fromhex("003C") + b"\xFF" * 16) * 4,
}


@pytest.mark.parametrize("dtype", list(HAND_BLOCKS))
def test_hand_derived_blocks_decode_to_two(dtype):
    # Q4_K: d=1, dmin=.5, sc=1, m=2, code 3 -> 1*1*3 - .5*2;  Q6_K: d=1, sc=2, q=33 -> 2*(33-32)
    # Q8_0: d=.5, q=4;  Q2_0: d=1, code 3 -> (3-1)*1
    y = orc.dequant_block(dtype, np.frombuffer(HAND_BLOCKS[dtype], np.uint8))
    assert y.size == 256 and np.all(y == 2.0)


# ───────────── host decode: independent decoders on random bytes ─────────────

def f16(b0, b1):
    return float(np.frombuffer(bytes([b0, b1]), np.float16)[0])


def decode_q4k_elementwise(blk):
    d, dmin = np.float32(f16(blk[0], blk[1])), np.float32(f16(blk[2], blk[3]))
    out = np.empty(256, np.float32)
    for e in range(256):
        s, l = divmod(e, 32)
        sc, m = k4_independent(s, [int(v) for v in blk[4:16]])
        byte = int(blk[16 + (s // 2) * 32 + l])
        q = byte >> 4 if s % 2 else byte & 15
        out[e] = np.float32(d * np.float32(sc)) * np.float32(q) + np.float32(dmin * np.float32(-m))
    return out


def decode_q6k_elementwise(blk):
    d = np.float32(f16(blk[208], blk[209]))
    out = np.empty(256, np.float32)
    for e in range(256):
        half, r = divmod(e, 128)
        col, l = divmod(r, 32)                      # col 0..3 = the four 32-element groups
        lo_byte = int(blk[half * 64 + (col % 2) * 32 + l])
        lo = lo_byte >> 4 if col >= 2 else lo_byte & 15
        hi = (int(blk[128 + half * 32 + l]) >> (2 * col)) & 3
        q = lo | (hi << 4)
        sc = int(np.int8(blk[192 + half * 8 + 2 * col + l // 16]))
        out[e] = np.float32(d * np.float32(sc)) * np.float32(q) + np.float32(d * np.float32(-32 * sc))
    return out


def decode_q8_0_elementwise(blk):
    d = np.float32(f16(blk[0], blk[1]))
    q = blk[2:34].view(np.int8).astype(np.int32)
    # host decode biases the code by 128: (d*1)*(q+128) + d*(-128)
    return np.array([np.float32(d * np.float32(1)) * np.float32(v + 128) + np.float32(d * np.float32(-128))
                     for v in q], np.float32)


def decode_q2_0_elementwise(blk):
    d = np.float32(f16(blk[0], blk[1]))
    return np.array([np.float32(((int(blk[2 + j // 4]) >> (2 * (j % 4))) & 3) - 1) * d
                     for j in range(64)], np.float32)


@pytest.mark.parametrize("dtype,dec", [(orc.Q4_K, decode_q4k_elementwise), (orc.Q6_K, decode_q6k_elementwise),
                                       (orc.Q8_0, decode_q8_0_elementwise), (orc.Q2_0, decode_q2_0_elementwise)])
def test_dequant_block_matches_independent_decoder_bit_for_bit(dtype, dec):
    e, b = orc.block_layout(dtype)
    raw = orc.synth_weight(dtype, e * 6, 0x5EED)  # aperiodic LCG payload, sane f16 scales
    got = orc.dequant_block(dtype, raw)
    for i in range(6):
        want = dec(raw[i * b:(i + 1) * b])
        assert np.array_equal(got[i * e:(i + 1) * e].view(np.uint32), want.view(np.uint32)), f"block {i}"


# ───────────── the reference's input recipes ─────────────

def test_lcg_bytes_recipe():
    # crates/infr-testkit/src/lib.rs:49-56: seed = seed*1664525 + 1013904223 (mod 2^32), byte = seed >> 16
    seed, want = 0x201, []
    for _ in range(8):
        seed = (seed * 1664525 + 1013904223) % 2 ** 32
        want.append((seed >> 16) & 0xFF)
    assert list(orc.lcg_bytes(0x201, 8)) == want


def test_gen_f32_recipe():
    got = orc.gen_f32(64, 7)
    # f32 arithmetic, as the reference: ((i*13+salt)%29) as f32 - 14.0) * 0.05
    want = np.array([(np.float32((i * 13 + 7) % 29) - np.float32(14.0)) * np.float32(0.05) for i in range(64)], np.float32)
    assert np.array_equal(got, want)


def test_synth_weight_scale_slots_are_the_real_scales():
    # crates/infr-testkit/src/lib.rs:529-555: after synthesis the declared slots hold f16(d), f16(min)
    h = lambda v: np.frombuffer(np.float16(v).tobytes(), np.uint8)
    w = orc.synth_weight(orc.Q4_K, 512, 9)
    for b in range(2):
        assert np.array_equal(w[b * 144:b * 144 + 2], h(0.05)) and np.array_equal(w[b * 144 + 2:b * 144 + 4], h(0.10))
    # payload = LCG(seed ^ b) everywhere else
    assert np.array_equal(w[144 + 4:288], orc.lcg_bytes(9 ^ 1, 144)[4:])
    w = orc.synth_weight(orc.Q6_K, 256, 9)
    assert np.array_equal(w[208:210], h(0.03))
    w = orc.synth_weight(orc.Q8_0, 64, 9)
    assert np.array_equal(w[34:36], h(0.01))
    w = orc.synth_weight(orc.Q2_0, 128, 9)
    assert np.array_equal(w[18:20], h(0.05))


def test_det_generators_recipe():
    # crates/infr-cpu/src/kernels.rs:6611-6624
    s, bs, xs = 1, [], []
    for _ in range(5):
        s = (s * 6364136223846793005 + 1442695040888963407) % 2 ** 64
        bs.append((s >> 33) & 0xFF)
    assert list(orc.det_bytes(5, 1)) == bs
    s = 2
    for _ in range(5):
        s = (s * 6364136223846793005 + 1442695040888963407) % 2 ** 64
        xs.append(np.float32(np.float32(s >> 40) / np.float32(2 ** 24)) * np.float32(2.0) - np.float32(1.0))
    assert np.array_equal(orc.det_x(5, 2), np.array(xs, np.float32))
