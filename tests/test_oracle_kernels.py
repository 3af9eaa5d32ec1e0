"""Pins the CPU oracle's quantizers, integer dots, f32 epilogues and Op::Linear dispatch.

Evidence used (none of it is the oracle's own formula retyped):
  * hand-derived known answers (all-127 activation x all-2.0 weights -> 65024 with the integer
    stages spelled out; the half-away-from-zero tie vector; zero and one-hot blocks),
  * invariants the reference states (bsums identities quant.rs:51, |q| <= 127, reconstruction
    error <= d/2 kernels.rs:6629-6646),
  * brute-force int64 dots over codes extracted by an independent byte-wise decoder,
  * the reference's own kernel tests restated with its input generators and tolerances
    (kernels.rs:6653-6697, 7115-7150: int8 dot vs dot(dequant(w), dequant(q8)) at 1e-3),
  * the reference's op-level sweep (decode_parity.rs: production <= 2e-2 of max|f64 oracle|,
    reference mode <= 1e-5, production vs reference mode <= 2e-2) with testkit's recipes and seeds,
  * batch == single bit-identical (kernels.rs:9297-9405).
"""
import numpy as np
import pytest

from oracle import oracle as orc
from tests.test_oracle_formats import HAND_BLOCKS, k4_independent

X127 = np.full(256, 127.0, np.float32)


# ───────────── activation quantizers ─────────────

def test_quantize_q8_all_127():
    q = orc.quantize_q8(X127)
    assert q.d[0] == 1.0 and np.all(q.qs == 127)
    assert np.all(q.bsums == 4064) and np.all(q.bsums16 == 2032)
    q32 = orc.quantize_q8_32(X127)
    assert np.all(q32.d == 1.0) and np.all(q32.bsum == 4064) and q32.d.size == 8


def test_quantize_ties_round_half_away_from_zero():
    x = np.zeros(256, np.float32)
    x[:6] = [0.5, 1.5, 2.5, -0.5, -1.5, 127.0]
    q = orc.quantize_q8(x)
    assert q.d[0] == 1.0
    assert list(q.qs[:6]) == [1, 2, 3, -1, -2, 127]      # round-to-even would give 0, 2, 2, 0, -2
    assert q.bsums[0] == 130 and q.bsums16[0] == 130 and not q.bsums[1:].any() and not q.bsums16[1:].any()
    q32 = orc.quantize_q8_32(x[:32])
    assert list(q32.qs[:6]) == [1, 2, 3, -1, -2, 127] and q32.bsum[0] == 130


def test_quantize_zero_block_and_one_hot():
    q = orc.quantize_q8(np.zeros(512, np.float32))
    assert not q.d.any() and not q.qs.any() and not q.bsums.any()
    x = np.zeros(256, np.float32)
    x[17] = -3.25
    q = orc.quantize_q8(x)
    assert q.qs[17] == -127 and np.count_nonzero(q.qs) == 1
    assert q.d[0] == np.float32(3.25) / np.float32(127.0)
    assert q.bsums[0] == -127 and q.bsums16[1] == -127


def test_quantize_invariants_on_random_rows():
    rng = np.random.default_rng(3)
    x = (rng.standard_normal(4096) * rng.choice([1e-3, 1.0, 50.0], 4096)).astype(np.float32)
    q = orc.quantize_q8(x)
    qs = q.qs.astype(np.int64)
    assert np.abs(qs).max() <= 127
    assert np.array_equal(q.bsums16, qs.reshape(-1, 16).sum(1))
    assert np.array_equal(q.bsums, q.bsums16.reshape(-1, 2).sum(1))          # quant.rs:51
    amax = np.abs(x.reshape(-1, 256)).max(1)
    assert np.array_equal(q.d, (amax / np.float32(127.0)).astype(np.float32))
    recon = (q.d[:, None] * q.qs.reshape(-1, 256).astype(np.float32)).ravel()
    assert np.all(np.abs(recon - x) <= np.repeat(q.d, 256) * 0.5000001)      # kernels.rs:6629-6646
    q32 = orc.quantize_q8_32(x)
    assert np.array_equal(q32.bsum, q32.qs.astype(np.int64).reshape(-1, 32).sum(1))
    amax32 = np.abs(x.reshape(-1, 32)).max(1)
    assert np.array_equal(q32.d, (amax32 / np.float32(127.0)).astype(np.float32))
    # a sub-256 tail is dropped by the per-256 quantizer (quant.rs:28)
    assert orc.quantize_q8(x[:300]).qs.size == 256


# ───────────── known-answer dots ─────────────

def test_hand_derived_dots_give_65024():
    q8, q32 = orc.quantize_q8(X127), orc.quantize_q8_32(X127)
    y, sd, sm = orc.vec_dot_q4k(np.frombuffer(HAND_BLOCKS[orc.Q4_K], np.uint8), q8, 256, True)
    assert (y, sd[0], sm[0]) == (65024.0, 8 * 12192, 8 * 2 * 4064)
    y, isum = orc.vec_dot_q6k(np.frombuffer(HAND_BLOCKS[orc.Q6_K], np.uint8), q8, 256, True)
    assert (y, isum[0]) == (65024.0, 16 * 2 * (16 * 33 * 127 - 32 * 2032))
    y, ip = orc.vec_dot_q8_0(np.frombuffer(HAND_BLOCKS[orc.Q8_0], np.uint8), q8, 256, True)
    assert y == 65024.0 and np.all(ip == 32 * 4 * 127)
    y, ip = orc.vec_dot_q2_0(np.frombuffer(HAND_BLOCKS[orc.Q2_0], np.uint8), q32, 256, True)
    assert y == 65024.0 and np.all(ip == 32 * 3 * 127)


def test_q4k_split_scale_bits_vector():
    # scales 81.. C2.. 25..: k4(0) = (1, 2), k4(4) = (37, 50); d = 1, dmin = 0, all codes 1
    blk = bytes.fromhex("003C" "0000" "81000000C200000025000000") + b"\x11" * 128
    y, sd, sm = orc.vec_dot_q4k(np.frombuffer(blk, np.uint8), orc.quantize_q8(X127), 256, True)
    assert sd[0] == (1 + 37) * 32 * 127 and y == 154432.0
    assert sm[0] == (2 + 50) * 4064


# ───────────── brute-force integer stages ─────────────

def codes_q4k(blk):
    return np.array([(int(blk[16 + (e // 64) * 32 + e % 32]) >> (4 * ((e // 32) % 2))) & 15 for e in range(256)])


def codes_q6k(blk):
    out = np.empty(256, np.int64)
    for e in range(256):
        half, r = divmod(e, 128)
        col, l = divmod(r, 32)
        lo_byte = int(blk[half * 64 + (col % 2) * 32 + l])
        lo = lo_byte >> 4 if col >= 2 else lo_byte & 15
        out[e] = lo | (((int(blk[128 + half * 32 + l]) >> (2 * col)) & 3) << 4)
    return out


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_integer_stages_match_brute_force(seed):
    in_f = 512
    x = orc.det_x(in_f, 100 + seed) * np.float32(3.0)
    q8, q32 = orc.quantize_q8(x), orc.quantize_q8_32(x)
    xi = q8.qs.astype(np.int64)
    # Q4_K
    w = orc.synth_weight(orc.Q4_K, in_f, seed)
    _, sd, sm = orc.vec_dot_q4k(w, q8, in_f, True)
    for b in range(2):
        blk = w[b * 144:(b + 1) * 144]
        c = codes_q4k(blk)
        scm = [k4_independent(s, [int(v) for v in blk[4:16]]) for s in range(8)]
        xb = xi[b * 256:(b + 1) * 256]
        assert sd[b] == sum(scm[s][0] * int((c[s * 32:(s + 1) * 32] * xb[s * 32:(s + 1) * 32]).sum()) for s in range(8))
        assert sm[b] == sum(scm[s][1] * int(xb[s * 32:(s + 1) * 32].sum()) for s in range(8))
    # Q6_K: isum = sum_sub sc * sum (q - 32) * x over each 16-element group
    w = orc.synth_weight(orc.Q6_K, in_f, seed)
    _, isum = orc.vec_dot_q6k(w, q8, in_f, True)
    for b in range(2):
        blk = w[b * 210:(b + 1) * 210]
        c = codes_q6k(blk) - 32
        xb = xi[b * 256:(b + 1) * 256]
        sc = blk[192:208].view(np.int8).astype(np.int64)
        assert isum[b] == sum(int(sc[g]) * int((c[g * 16:(g + 1) * 16] * xb[g * 16:(g + 1) * 16]).sum()) for g in range(16))
    # Q8_0
    w = orc.synth_weight(orc.Q8_0, in_f, seed)
    _, ip = orc.vec_dot_q8_0(w, q8, in_f, True)
    for k in range(in_f // 32):
        qw = w[k * 34 + 2:(k + 1) * 34].view(np.int8).astype(np.int64)
        assert ip[k] == int((qw * xi[k * 32:(k + 1) * 32]).sum())
    # Q2_0 (per-32 activation)
    xi32 = q32.qs.astype(np.int64)
    w = orc.synth_weight(orc.Q2_0, in_f, seed)
    _, ip = orc.vec_dot_q2_0(w, q32, in_f, True)
    for s in range(in_f // 32):
        b, sub = divmod(s, 2)
        qs = w[b * 18 + 2:(b + 1) * 18]
        c = np.array([(int(qs[(sub * 32 + p) // 4]) >> (2 * (p % 4))) & 3 for p in range(32)])
        assert ip[s] == int((c * xi32[s * 32:(s + 1) * 32]).sum())


def test_all_ones_q8_0_weights_reduce_to_bsums():
    in_f = 256
    w = (bytes.fromhex("003C") + b"\x01" * 32) * 8
    x = orc.det_x(in_f, 5)
    q8 = orc.quantize_q8(x)
    _, ip = orc.vec_dot_q8_0(np.frombuffer(w, np.uint8), q8, in_f, True)
    assert np.array_equal(ip, q8.bsums)


# ───────────── the reference's kernel tests, restated ─────────────

def rel_err(got, want):
    return abs(float(got) - float(want)) / max(abs(float(want)), 1.0)


def put_f16(w, off, v):
    w[off:off + 2] = np.frombuffer(np.float16(v).tobytes(), np.uint8)


def dequant_q8(q):
    return (np.repeat(q.d, 256) * q.qs.astype(np.float32)).astype(np.float32)


def test_q4k_q6k_q8_0_dot_matches_dequant_reference():
    # kernels.rs:6653-6697
    in_f = 768
    w = orc.det_bytes(3 * 144, 1)
    for k in range(3):
        put_f16(w, k * 144, 0.05)
        put_f16(w, k * 144 + 2, 0.015)
    q8 = orc.quantize_q8(orc.det_x(in_f, 2))
    assert rel_err(orc.vec_dot_q4k(w, q8, in_f), orc.dot(orc.dequant_block(orc.Q4_K, w), dequant_q8(q8))) < 1e-3
    w = orc.det_bytes(3 * 210, 3)
    for k in range(3):
        put_f16(w, k * 210 + 208, 0.04)
    q8 = orc.quantize_q8(orc.det_x(in_f, 4))
    assert rel_err(orc.vec_dot_q6k(w, q8, in_f), orc.dot(orc.dequant_block(orc.Q6_K, w), dequant_q8(q8))) < 1e-3
    in_f = 512
    w = orc.det_bytes(16 * 34, 9)
    for k in range(16):
        put_f16(w, k * 34, 0.03)
    q8 = orc.quantize_q8(orc.det_x(in_f, 10))
    assert rel_err(orc.vec_dot_q8_0(w, q8, in_f), orc.dot(orc.dequant_block(orc.Q8_0, w), dequant_q8(q8))) < 1e-3


@pytest.mark.parametrize("in_f", [64, 256, 704])
def test_q2_0_matches_dequant_reference(in_f):
    # kernels.rs:7115-7150
    nb = in_f // 64
    w = orc.det_bytes(nb * 18, 210)
    for k in range(nb):
        put_f16(w, k * 18, 0.03)
    wref = orc.dequant_block(orc.Q2_0, w)
    assert np.any(wref[:64] != 0)
    for i in range(4):
        x = orc.det_x(in_f, 211 + i)
        q = orc.quantize_q8_32(x)
        got = orc.vec_dot_q2_0(w, q, in_f)
        deq = (np.repeat(q.d, 32) * q.qs.astype(np.float32)).astype(np.float32)
        assert rel_err(got, orc.dot(wref, deq)) < 1e-3
        assert rel_err(got, orc.dot(wref, x)) < 2e-2


def test_dot_is_eight_lane_fma():
    # kernels.rs:6557-6573: lane j accumulates elements j, j+8, ... with fused multiply-add
    rng = np.random.default_rng(0)
    a, b = rng.standard_normal(67).astype(np.float32), rng.standard_normal(67).astype(np.float32)
    acc = [np.float64(0)] * 8
    acc32 = [np.float32(0)] * 8
    for c in range(8):
        for j in range(8):
            # fma: exact product + acc, rounded once (f64 holds the f32 product exactly)
            acc32[j] = np.float32(np.float64(a[c * 8 + j]) * np.float64(b[c * 8 + j]) + np.float64(acc32[j]))
    s = np.float32(0)
    for j in range(8):
        s = np.float32(s + acc32[j])
    for i in range(64, 67):
        s = np.float32(np.float64(a[i]) * np.float64(b[i]) + np.float64(s))
    assert orc.dot(a, b) == s


@pytest.mark.parametrize("m", [1, 3])
def test_linear_over_plain_rows_is_dot_over_the_widened_row(m):
    # lib.rs:1162-1164, 1443-1462: F32 / F16 / BF16 weights go through dot / dot_f16 / dot_bf16, which
    # widen each weight exactly (kernels.rs:6505-6549) and run dot's chains. Widened here by numpy
    # (float16 -> float32) and by bit arithmetic (bf16 = the top half of the f32 pattern), then fed
    # to the eight-chain restatement pinned above: the three dtypes must give those bits.
    in_f, out_f = 104, 5      # 13 chunks of eight: chains and no tail; a tail is covered above
    rng = np.random.default_rng(5)
    w = (rng.standard_normal(out_f * in_f) * 0.05).astype(np.float32)
    x = rng.standard_normal(m * in_f).astype(np.float32)
    f16 = w.astype(np.float16)
    bf16 = (w.view(np.uint32) >> 16).astype(np.uint16)
    cases = [(orc.F32, w.view(np.uint8), w),
             (orc.F16, f16.view(np.uint8), f16.astype(np.float32)),
             (orc.BF16, bf16.view(np.uint8), (bf16.astype(np.uint32) << 16).view(np.float32))]
    for dtype, raw, widened in cases:
        got = orc.linear(dtype, raw, x, m, in_f, out_f).reshape(m, out_f)
        for r in range(m):
            for o in range(out_f):
                assert got[r, o] == orc.dot(widened[o * in_f:(o + 1) * in_f], x[r * in_f:(r + 1) * in_f])


# ───────────── Op::Linear: the reference's op-level sweep ─────────────

# position of each format in WEIGHT_QUANTS (decode_spec.rs:255-280) -> testkit seed 0x201 + i
SWEEP = [(orc.Q8_0, 4), (orc.Q4_K, 7), (orc.Q6_K, 9), (orc.Q2_0, 21)]


@pytest.mark.parametrize("dtype,pos", SWEEP)
@pytest.mark.parametrize("m", [1, 2])
def test_linear_sweep_against_f64_oracle(dtype, pos, m):
    in_f, out_f, seed = 256, 8, 0x201 + pos
    w = orc.synth_weight(dtype, in_f * out_f, seed)
    x = orc.gen_f32(m * in_f, seed ^ 0x9E37)
    want = orc.ref_linear_f64(x, orc.dequant_block(dtype, w), m, in_f, out_f)
    ref_mag = np.abs(want).max()
    assert ref_mag > 1e-3                                             # testkit: vacuous cases fail
    prod = orc.linear(dtype, w, x, m, in_f, out_f)
    refm = orc.linear(dtype, w, x, m, in_f, out_f, reference_mode=True)
    assert np.abs(prod - want).max() / ref_mag < 2e-2                 # decode_parity.rs:57
    assert np.abs(refm - want).max() / ref_mag < 1e-5                 # decode_parity.rs:93-102
    assert np.abs(prod - refm).max() / np.abs(refm).max() < 2e-2      # decode_parity.rs:133-159


@pytest.mark.parametrize("dtype", [orc.Q4_K, orc.Q6_K, orc.Q8_0, orc.Q2_0])
def test_linear_batch_is_bit_identical_to_single_rows(dtype):
    in_f, out_f, m = 1024, 19, 5
    w = orc.synth_weight(dtype, in_f * out_f, 77)
    x = orc.det_x(m * in_f, 78)
    y = orc.linear(dtype, w, x, m, in_f, out_f, threads=3)
    for r in range(m):
        yr = orc.linear(dtype, w, x[r * in_f:(r + 1) * in_f], 1, in_f, out_f, threads=1)
        assert np.array_equal(y[r].view(np.uint32), yr.ravel().view(np.uint32))


def test_linear_w_off_slices_rows_of_a_concatenated_weight():
    in_f, rows = 256, 24
    w = orc.synth_weight(orc.Q4_K, in_f * rows, 5)
    x = orc.det_x(in_f, 6)
    full = orc.linear(orc.Q4_K, w, x, 1, in_f, rows)
    part = orc.linear(orc.Q4_K, w, x, 1, in_f, 8, w_numel=rows * in_f, w_off=8 * in_f)
    assert np.array_equal(part, full[:, 8:16])
    with pytest.raises(ValueError):
        orc.linear(orc.Q4_K, w, x, 1, in_f, 8, w_numel=rows * in_f, w_off=100)   # not row-aligned


def test_linear_int_stages_agree_with_row_kernels():
    in_f, out_f, m = 512, 6, 2
    w = orc.synth_weight(orc.Q4_K, in_f * out_f, 11)
    x = orc.det_x(m * in_f, 12)
    a, b = orc.linear_int_stages(orc.Q4_K, w, x, m, in_f, out_f)
    for r in range(m):
        q8 = orc.quantize_q8(x[r * in_f:(r + 1) * in_f])
        for o in range(out_f):
            _, sd, sm = orc.vec_dot_q4k(w[o * 288:(o + 1) * 288], q8, in_f, True)
            assert np.array_equal(a[r, o], sd) and np.array_equal(b[r, o], sm)


def test_linear_rejects_ragged_in_f():
    # a row must be a whole number of weight blocks: Q4_K needs 256s (a per-256 quantizer would
    # silently drop the tail, quant.rs:28), Q2_0 whole 64s
    w = orc.synth_weight(orc.Q4_K, 256 * 4, 1)
    with pytest.raises(ValueError):
        orc.linear(orc.Q4_K, w, np.zeros(128, np.float32), 1, 128, 8)
    w = orc.synth_weight(orc.Q2_0, 64 * 4, 1)
    with pytest.raises(ValueError):
        orc.linear(orc.Q2_0, w, np.zeros(32, np.float32), 1, 32, 8)


# ───────────── the committed known-answer fixture, through Op::Linear ─────────────

def _golden():
    import json
    import os
    with open(os.path.join(os.path.dirname(__file__), "golden", "known_answers.json")) as f:
        return json.load(f)


@pytest.mark.parametrize("case", _golden()["dots"], ids=lambda c: c["name"])
def test_golden_known_answers_through_linear(case):
    row = np.frombuffer(b"".join(bytes.fromhex(h) * n for h, n in case["parts"]), np.uint8)
    w = np.tile(row, 3)
    x = np.full(2 * case["in_f"], 127.0, np.float32)
    y = orc.linear(case["dtype"], w, x, 2, case["in_f"], 3)
    assert np.all(y == np.float32(case["y"]))
    a, b = orc.linear_int_stages(case["dtype"], w, x, 2, case["in_f"], 3)
    assert np.array_equal(np.asarray(a).reshape(6, -1), np.tile(np.array(case["int_a"], np.int32), (6, 1)))
    if "int_b" in case:
        assert np.array_equal(np.asarray(b).reshape(6, -1), np.tile(np.array(case["int_b"], np.int32), (6, 1)))


# ───────────── Q8_0 rows that are a multiple of 32 only: the per-32 arm ─────────────

@pytest.mark.parametrize("in_f", [32, 96, 1152])
def test_q8_0_per32_arm_against_brute_force_and_dequant(in_f):
    out_f = 5
    w = orc.synth_weight(orc.Q8_0, in_f * out_f, 0x231)
    x = orc.gen_f32(in_f, 7)
    y = orc.linear(orc.Q8_0, w, x, 1, in_f, out_f).ravel()
    ia, _ = orc.linear_int_stages(orc.Q8_0, w, x, 1, in_f, out_f)
    q = orc.quantize_q8_32(x)
    blocks = w.reshape(out_f, in_f // 32, 34)
    for o in range(out_f):
        acc = np.float32(0.0)
        for b in range(in_f // 32):
            qw = blocks[o, b, 2:].view(np.int8).astype(np.int64)
            ip = int(qw @ q.qs[b * 32:(b + 1) * 32].astype(np.int64))
            assert ia.reshape(out_f, -1)[o, b] == ip
            d_w = np.float32(orc.f16_bits_to_f32(int(blocks[o, b, 0]) | int(blocks[o, b, 1]) << 8))
            acc = np.float32(acc + np.float32(np.float32(d_w * q.d[b]) * np.float32(ip)))
        assert y[o] == acc
    # and against the decoded weights in f64, at the reference's production bound
    wf = np.concatenate([orc.dequant_block(orc.Q8_0, blocks[o].ravel()) for o in range(out_f)]).reshape(out_f, in_f)
    ref = wf.astype(np.float64) @ x.astype(np.float64)
    assert np.abs(y - ref).max() <= 2e-2 * np.abs(ref).max()
