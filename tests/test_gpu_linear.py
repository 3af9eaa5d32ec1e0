"""GPU parity of Op::Linear against the CPU oracle, through the C ABI.

Bars: activation quantization and per-block integer stages bit-exact; Q4_K / Q6_K decode outputs
bit-identical to the oracle (same per-block expression, same accumulation order); Q8_0 / Q2_0 and
every m > 1 output within rel-L2 <= 1e-4 and max-abs <= 1e-3 * max|y|.
"""
import numpy as np
import pytest

from infr_amd import DType, synth_normal_f32, synth_weight
from oracle import oracle as orc

pytestmark = pytest.mark.gpu

REL_L2 = 1e-4
MAX_ABS = 1e-3


def gate(y, want):
    y, want = np.asarray(y, np.float64).ravel(), np.asarray(want, np.float64).ravel()
    assert np.abs(want).max() > 1e-3, "vacuous case: oracle output is all zero"
    rel = np.linalg.norm(y - want) / np.linalg.norm(want)
    mx = np.abs(y - want).max() / np.abs(want).max()
    assert rel <= REL_L2 and mx <= MAX_ABS, f"rel-L2 {rel:.3e} max-abs/|y|inf {mx:.3e}"
    return rel, mx


def close(got, want, rel_bar=2e-6, mx_bar=1e-5):
    """The bar of the contracted Q4_K prefill epilogue (128 tokens and more on the strip kernel): fused
    multiply-adds where infr-cpu rounds every product, ~1e-7 relative; exact integers either way."""
    g, t = np.asarray(got, np.float64).ravel(), np.asarray(want, np.float64).ravel()
    rel = np.linalg.norm(g - t) / np.linalg.norm(t)
    mx = np.abs(g - t).max() / np.abs(t).max()
    assert rel <= rel_bar and mx <= mx_bar, f"rel-L2 {rel:.3e} max-abs/|y|inf {mx:.3e}"


def run_linear(be, dtype, w, x, m, in_f, out_f, w_off=0, w_numel=None):
    wb, xb = be.upload_new(w), be.upload_new(x)
    yb = be.alloc(m * out_f * 4)
    be.linear(dtype, wb, xb, yb, m, in_f, out_f, w_numel=w_numel, w_off=w_off)
    return be.download(yb, np.empty((m, out_f), np.float32))


@pytest.mark.parametrize("m,k", [(1, 256), (1, 4096), (3, 768), (8, 12288)])
def test_quantize_q8_bit_exact(be, m, k):
    x = synth_normal_f32(11 + k, m * k)
    x[:7] = [0.5, 1.5, 2.5, -0.5, -1.5, 127.0, 0.0]  # exact ties: half away from zero
    if m > 1:
        x[k:2 * k] = 0.0  # an all-zero row: d = 0, id = 0
    qs, d, bs, bs16 = be.quantize_q8(be.upload_new(x), m, k)
    for r in range(m):
        o = orc.quantize_q8(x[r * k:(r + 1) * k])
        assert np.array_equal(qs[r], o.qs)
        assert np.array_equal(d[r].view(np.uint32), o.d.view(np.uint32))
        assert np.array_equal(bs[r], o.bsums)
        assert np.array_equal(bs16[r], o.bsums16)


@pytest.mark.parametrize("m,k", [(1, 64), (1, 4096), (5, 96), (2, 12288)])
def test_quantize_q8_32_bit_exact(be, m, k):
    x = synth_normal_f32(5 + k, m * k)
    x[:6] = [0.5, 1.5, 2.5, -0.5, -1.5, 127.0]
    qs, d, bs = be.quantize_q8_32(be.upload_new(x), m, k)
    for r in range(m):
        o = orc.quantize_q8_32(x[r * k:(r + 1) * k])
        assert np.array_equal(qs[r], o.qs)
        assert np.array_equal(d[r].view(np.uint32), o.d.view(np.uint32))
        assert np.array_equal(bs[r], o.bsum)


def test_quantizers_round_every_code_boundary_like_the_cpu(be):
    """round() is half away from zero (crates/infr-cpu/src/quant.rs:27-58, 97-117). With amax = 127 the
    scale is exactly 1, so the codes are round(x) itself: every boundary k + 0.5 for k = 0 .. 126, the
    floats just below and just above it, and their negatives, in both quantizers. (The device rounds
    by adding copysign(0.5 - 2^-25, x) and truncating, which must agree at all of them.)"""
    ks = np.arange(0, 127, dtype=np.float32) + np.float32(0.5)
    vals = np.concatenate([ks, np.nextafter(ks, np.float32(0)), np.nextafter(ks, np.float32(200)),
                           np.float32([0.0, 1e-30, 0.25, 126.99999, 127.0])]).astype(np.float32)
    vals = np.concatenate([vals, -vals])
    n = -(-vals.size // 256) * 256
    x = np.zeros(n, np.float32)
    x[:vals.size] = vals
    x[255::256] = 127.0                       # every 256-block (and below: every 32-block) has amax = 127
    qs, d, bs, bs16 = be.quantize_q8(be.upload_new(x), 1, n)
    o = orc.quantize_q8(x)
    assert np.all(o.d == 1.0)
    assert np.array_equal(qs[0], o.qs) and np.array_equal(bs[0], o.bsums) and np.array_equal(bs16[0], o.bsums16)
    x32 = x.copy()
    x32[31::32] = 127.0
    qs, d, bs = be.quantize_q8_32(be.upload_new(x32), 1, n)
    o = orc.quantize_q8_32(x32)
    assert np.all(o.d == 1.0)
    assert np.array_equal(qs[0], o.qs) and np.array_equal(bs[0], o.bsum)


DECODE_SHAPES = [(256, 8), (768, 37), (4096, 1024), (12288, 512), (2048, 100), (5120, 64)]


def test_headline_configuration_q4k_4096x4096(be):
    """The benchmark's own CPU-runnable case: W[4096, 4096] ~ N(0, 0.02^2) from seed 0 as Q4_K, x[1, 4096]
    ~ N(0, 1) from seed 1; activation codes and block integers bit-exact, y bit-identical."""
    n = k = 4096
    w = synth_weight(DType.Q4K, 0, n, k, 0.02)
    x = synth_normal_f32(1, k)
    qs, d, bs, _ = be.quantize_q8(be.upload_new(x), 1, k)
    o = orc.quantize_q8(x)
    assert np.array_equal(qs[0], o.qs) and np.array_equal(d[0].view(np.uint32), o.d.view(np.uint32))
    assert np.array_equal(bs[0], o.bsums)
    a, b = be.linear_int_stages(DType.Q4K, be.upload_new(w), be.upload_new(x), 1, k, n)
    oa, ob = orc.linear_int_stages(DType.Q4K, w, x, 1, k, n)
    assert np.array_equal(a, oa) and np.array_equal(b, ob)
    y = run_linear(be, DType.Q4K, w, x, 1, k, n)
    want = orc.linear(DType.Q4K, w, x, 1, k, n)
    gate(y, want)
    assert np.array_equal(y.view(np.uint32), want.view(np.uint32)), "not bit-identical"


# the decode set at Qwen3-8B layer shapes, batch 1 and 8 (rows cut to 256: a row's arithmetic does not
# depend on how many rows there are, and the oracle stays within seconds)
@pytest.mark.parametrize("dtype", [DType.Q4K, DType.Q6K, DType.Q8_0])
@pytest.mark.parametrize("m", [1, 8])
@pytest.mark.parametrize("in_f", [4096, 12288])
def test_decode_set_shapes_batch_1_and_8(be, dtype, m, in_f):
    out_f = 256
    w = synth_weight(dtype, 0, out_f, in_f, 0.02)
    x = synth_normal_f32(1, m * in_f)
    y = run_linear(be, dtype, w, x, m, in_f, out_f)
    want = orc.linear(dtype, w, x, m, in_f, out_f)
    gate(y, want)
    if dtype in (DType.Q4K, DType.Q6K):
        assert np.array_equal(y.view(np.uint32), want.view(np.uint32)), "not bit-identical"


@pytest.mark.parametrize("dtype", [DType.Q4K, DType.Q6K, DType.Q8_0, DType.Q2_0])
@pytest.mark.parametrize("in_f,out_f", DECODE_SHAPES)
def test_decode_gemv_vs_oracle(be, dtype, in_f, out_f):
    w = synth_weight(dtype, 100 + in_f, out_f, in_f)
    x = synth_normal_f32(200 + out_f, in_f)
    y = run_linear(be, dtype, w, x, 1, in_f, out_f)
    want = orc.linear(dtype, w, x, 1, in_f, out_f)
    gate(y, want)
    if dtype in (DType.Q4K, DType.Q6K):
        assert np.array_equal(y.view(np.uint32), want.view(np.uint32)), "not bit-identical"


@pytest.mark.parametrize("dtype,in_f", [(DType.Q4K, 1024), (DType.Q5K, 768), (DType.Q4K, 2560)])
@pytest.mark.parametrize("noalloc", [False, True])
def test_one_token_over_an_output_head_sized_matrix(be, dtype, in_f, noalloc):
    """A single one-token op with a vocabulary's worth of rows (Qwen3's 151936) is many rounds of
    workgroups by itself and takes the streamed-row form of the decode GEMV through the direct entry
    points (no tile table: the descriptor travels as a kernel argument); the last tile is partial.
    The integer-stage entry point keeps the direct-load form: same bits."""
    out_f = 151936 + 5
    w = orc.synth_weight(dtype, out_f * in_f, 0x77 + in_f)
    x = synth_normal_f32(0x78, in_f)
    yb = be.alloc(out_f * 4)
    (be.linear_noalloc if noalloc else be.linear)(dtype, be.upload_new(w), be.upload_new(x), yb, 1, in_f, out_f)
    got = be.download(yb, np.empty(out_f, np.float32))
    want = orc.linear(dtype, w, x, 1, in_f, out_f).ravel()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("dtype", [DType.Q4K, DType.Q6K, DType.Q8_0, DType.Q2_0])
def test_decode_int_stages_bit_exact(be, dtype):
    in_f, out_f = 1024, 24
    # full-range payload bytes (the reference's synth_weight recipe) stress every code value
    w = orc.synth_weight(dtype, in_f * out_f, 0x201)
    x = orc.gen_f32(in_f, 0x201 ^ 0x9E37)
    a, b = be.linear_int_stages(dtype, be.upload_new(w), be.upload_new(x), 1, in_f, out_f)
    oa, ob = orc.linear_int_stages(dtype, w, x, 1, in_f, out_f)
    assert np.array_equal(a, oa)
    if dtype == DType.Q4K:
        assert np.array_equal(b, ob)


@pytest.mark.parametrize("dtype", [DType.Q4K, DType.Q6K, DType.Q8_0, DType.Q2_0])
@pytest.mark.parametrize("m", [2, 8])
def test_small_batch_vs_oracle(be, dtype, m):
    in_f, out_f = 1024, 96
    w = synth_weight(dtype, 7, out_f, in_f)
    x = synth_normal_f32(8, m * in_f)
    y = run_linear(be, dtype, w, x, m, in_f, out_f)
    gate(y, orc.linear(dtype, w, x, m, in_f, out_f))


@pytest.mark.parametrize("dtype", [DType.Q4K, DType.Q6K, DType.Q8_0, DType.Q5_0])
@pytest.mark.parametrize("noalloc", [False, True])
def test_one_row_linear_in_place_on_its_input(be, dtype, noalloc):
    # dst == x is a legal graph (the CPU arm builds its result in a fresh vector, lib.rs:985-1492):
    # every output row must see the x from before the op. 4096 rows span many workgroups.
    n = 4096
    w = synth_weight(dtype, 0x51, n, n, sigma=0.02)
    x = synth_normal_f32(0x52, n)
    wb, xb = be.upload_new(w), be.upload_new(x)
    (be.linear_noalloc if noalloc else be.linear)(dtype, wb, xb, xb, 1, n, n)
    y = be.download(xb, np.empty((1, n), np.float32))
    want = orc.linear(dtype, w, x, 1, n, n)
    gate(y, want)
    if dtype in (DType.Q4K, DType.Q6K):
        assert np.array_equal(y.view(np.uint32), want.view(np.uint32)), "not bit-identical"


def test_w_off_selects_rows_of_a_concatenated_weight(be):
    in_f, rows = 512, 48
    w = synth_weight(DType.Q4K, 3, rows, in_f)
    x = synth_normal_f32(4, in_f)
    y = run_linear(be, DType.Q4K, w, x, 1, in_f, 16, w_off=16 * in_f, w_numel=rows * in_f)
    want = orc.linear(DType.Q4K, w, x, 1, in_f, 16, w_numel=rows * in_f, w_off=16 * in_f)
    assert np.array_equal(y.view(np.uint32), want.view(np.uint32))


# ───────────── prefill (m >= 2): int8 MFMA path for Q4_K ─────────────

# from 128 tokens: the 16-token K-split kernel (rows of two blocks and more, up to 640 K outputs), the
# 128-token tiles (batches that fill little of their 256-token groups) or the strips (ragged last tiles in
# both directions)
PREFILL_SHAPES = [(2, 256, 8), (8, 1024, 96), (33, 512, 200), (64, 1024, 256), (130, 768, 130), (257, 2048, 384),
                  (800, 256, 64), (900, 256, 64), (1024, 256, 64), (1200, 512, 72), (2100, 256, 40)]


@pytest.mark.parametrize("m,in_f,out_f", PREFILL_SHAPES)
def test_prefill_q4k_matches_the_oracle(be, m, in_f, out_f):
    """Bit-identical below 128 tokens; from 128 on the route may be the strips, whose contracted f32
    epilogue is held to 2e-6 (the integers behind it are checked exactly elsewhere)."""
    w = synth_weight(DType.Q4K, 300 + m, out_f, in_f)
    x = synth_normal_f32(400 + m, m * in_f)
    x[:in_f] *= 37.0            # rows with very different scales
    if m > 2:
        x[2 * in_f:3 * in_f] = 0.0   # an all-zero row
    y = run_linear(be, DType.Q4K, w, x, m, in_f, out_f)
    want = orc.linear(DType.Q4K, w, x, m, in_f, out_f)
    gate(y, want)
    if m < 128:
        assert np.array_equal(y.view(np.uint32), want.view(np.uint32)), "not bit-identical"
    else:
        close(y, want)


# 2..16 tokens on rows of an even number of blocks: 16 x 16 MFMA tiles, K split over the waves of a
# workgroup in passes of eight blocks (one pass, several, a ragged last one, waves past the end),
# 8- and 16-token tiles, a ragged last row tile
@pytest.mark.parametrize("m,in_f,out_f", [(3, 4096, 48), (8, 5632, 40), (7, 8192, 24), (9, 512, 16),
                                          (12, 2048, 100), (16, 4096, 33), (16, 6144, 64)])
@pytest.mark.parametrize("dtype", [DType.Q4K, DType.Q5K, DType.Q6K])
def test_small_batch_kquant_mfma_is_bit_identical_to_oracle(be, dtype, m, in_f, out_f):
    w = synth_weight(dtype, 500 + m, out_f, in_f)
    x = synth_normal_f32(600 + m, m * in_f)
    x[:in_f] *= 37.0
    x[(m - 1) * in_f:] *= 0.01
    y = run_linear(be, dtype, w, x, m, in_f, out_f)
    want = orc.linear(dtype, w, x, m, in_f, out_f)
    assert np.array_equal(y.view(np.uint32), want.view(np.uint32)), "not bit-identical"


@pytest.mark.parametrize("m,in_f,out_f", [(9, 4096, 48), (13, 512, 40), (16, 5632, 24), (12, 1024, 70), (10, 8192, 40),
                                          (15, 12288, 33)])
def test_q8_0_on_the_sixteen_token_mfma_kernel_is_bit_identical_to_oracle(be, m, in_f, out_f):
    """9..16 tokens of Q8_0 take the K-split MFMA kernel (eight waves per workgroup on the two long-row shapes): one
    exact iprod per 34-byte block and the CPU's chain `sumf += (q8.d * d_w) * iprod` block by block
    (crates/infr-cpu/src/kernels.rs:1170-1187) handed from wave to wave, so unlike the dot4 batches
    these outputs equal the scalar kernel's bits; the per-block integers are exact as everywhere."""
    w = orc.synth_weight(DType.Q8_0, in_f * out_f, 0x20C)
    x = orc.gen_f32(m * in_f, 0x20C ^ 0x9E37)
    y = run_linear(be, DType.Q8_0, w, x, m, in_f, out_f)
    want = orc.linear(DType.Q8_0, w, x, m, in_f, out_f)
    assert np.array_equal(y.view(np.uint32), want.reshape(m, out_f).view(np.uint32)), "not bit-identical"
    a, _ = be.linear_int_stages(DType.Q8_0, be.upload_new(w), be.upload_new(x), m, in_f, out_f)
    oa, _ = orc.linear_int_stages(DType.Q8_0, w, x, m, in_f, out_f)
    assert np.array_equal(a, oa)


@pytest.mark.parametrize("m,in_f,out_f", [(9, 4096, 48), (13, 512, 40), (16, 5632, 24), (12, 1024, 70), (11, 12288, 33)])
def test_q2_0_on_the_sixteen_token_mfma_kernel_is_bit_identical_to_oracle(be, m, in_f, out_f):
    """9..16 tokens of Q2_0 on the K-split MFMA kernel: one exact iprod per 32-element half against
    the per-32 activation, the CPU's term `(d * q8.d[s]) * (iprod - bsum[s])` per half and its chain
    in block order (crates/infr-cpu/src/kernels.rs:5641-5668): the scalar kernel's bits."""
    w = orc.synth_weight(DType.Q2_0, in_f * out_f, 0x20D)
    x = orc.gen_f32(m * in_f, 0x20D ^ 0x9E37)
    y = run_linear(be, DType.Q2_0, w, x, m, in_f, out_f)
    want = orc.linear(DType.Q2_0, w, x, m, in_f, out_f)
    assert np.array_equal(y.view(np.uint32), want.reshape(m, out_f).view(np.uint32)), "not bit-identical"
    a, _ = be.linear_int_stages(DType.Q2_0, be.upload_new(w), be.upload_new(x), m, in_f, out_f)
    oa, _ = orc.linear_int_stages(DType.Q2_0, w, x, m, in_f, out_f)
    assert np.array_equal(a, oa)


@pytest.mark.parametrize("m", [17, 31, 33, 48, 64, 96, 128])
@pytest.mark.parametrize("dtype", [DType.Q4K, DType.Q5K, DType.Q6K, DType.Q8_0, DType.Q2_0])
def test_batches_beyond_sixteen_tokens_on_the_k_split_kernel(be, dtype, m):
    """The 16-token K-split MFMA kernel walks larger batches 16 tokens at a time (up to 32..128
    tokens by format, row length and matrix size): every output still equals the oracle's bit for
    bit - the token tile a row falls into changes nothing about its arithmetic - and the per-block
    integers are exact. A small matrix, which keeps the route for the longest, and a long-row one."""
    if m > {DType.Q4K: 127, DType.Q5K: 96, DType.Q6K: 128, DType.Q8_0: 64, DType.Q2_0: 128}[dtype]:
        pytest.skip("beyond this format's range the 128-token MFMA tiles take over (their own tests)")
    for in_f, out_f in ((1024, 70), (8192, 40)):
        w = orc.synth_weight(dtype, in_f * out_f, 0x20E)
        x = orc.gen_f32(m * in_f, 0x20E ^ 0x9E37)
        x[in_f:2 * in_f] = 0.0                      # an all-zero token inside the first tile
        y = run_linear(be, dtype, w, x, m, in_f, out_f)
        want = orc.linear(dtype, w, x, m, in_f, out_f).reshape(m, out_f)
        assert np.array_equal(y.view(np.uint32), want.view(np.uint32)), f"not bit-identical at {in_f} x {out_f}"
    a, b = be.linear_int_stages(dtype, be.upload_new(w), be.upload_new(x), m, in_f, out_f)
    oa, ob = orc.linear_int_stages(dtype, w, x, m, in_f, out_f)
    assert np.array_equal(a, oa)
    if dtype in (DType.Q4K, DType.Q5K):
        assert np.array_equal(b, ob)


@pytest.mark.parametrize("m", [3, 8, 16, 24, 40, 64])
@pytest.mark.parametrize("dtype", [DType.Q4K, DType.Q5K, DType.Q8_0, DType.Q4_0, DType.Q5_1])
def test_k_split_kernel_on_rows_of_an_odd_number_of_blocks(be, dtype, m):
    """Rows of 3, 9 and 43 blocks of 256 (768, 2304 and 11008 columns: Llama-2-7B's and Qwen2.5's
    down projections are such rows): the kernel stages weights two blocks at a time and the last,
    single block of a row arrives in a stage that starts a block early. Outputs bit-identical to the
    oracle's scalar kernels, the per-block integers exact (the last block's included)."""
    if dtype in (DType.Q8_0, DType.Q4_0, DType.Q5_1) and m <= 8:
        pytest.skip("these formats take the dot4 batches up to eight tokens")
    for in_f, out_f in ((768, 70), (2304, 33), (11008, 40)):
        w = orc.synth_weight(dtype, in_f * out_f, 0x30D + in_f)
        x = orc.gen_f32(m * in_f, 0x30D ^ 0x9E37)
        x[in_f:2 * in_f] = 0.0
        y = run_linear(be, dtype, w, x, m, in_f, out_f)
        want = orc.linear(dtype, w, x, m, in_f, out_f).reshape(m, out_f)
        assert np.array_equal(y.view(np.uint32), want.view(np.uint32)), f"not bit-identical at {in_f} x {out_f}"
        a, b = be.linear_int_stages(dtype, be.upload_new(w), be.upload_new(x), m, in_f, out_f)
        oa, ob = orc.linear_int_stages(dtype, w, x, m, in_f, out_f)
        assert np.array_equal(a, oa), f"first integer stage at {in_f} x {out_f}"
        if dtype in (DType.Q4K, DType.Q5K):
            assert np.array_equal(b, ob), f"second integer stage at {in_f} x {out_f}"


@pytest.mark.parametrize("m,in_f,out_f", [(6, 4608, 40), (13, 1024, 50)])
@pytest.mark.parametrize("dtype,seed", [(DType.Q4K, 0x209), (DType.Q5K, 0x20A), (DType.Q6K, 0x20B)])
def test_small_batch_kquant_mfma_int_stages_bit_exact(be, dtype, seed, m, in_f, out_f):
    # full-range payload bytes and saturated activation rows: every scale, min and code value,
    # block sums up to +-4064
    w = orc.synth_weight(dtype, in_f * out_f, seed)
    x = synth_normal_f32(78, m * in_f) * np.float32(3.0)
    x[in_f:2 * in_f] = 1e4
    x[2 * in_f:3 * in_f] = -1e4
    a, b = be.linear_int_stages(dtype, be.upload_new(w), be.upload_new(x), m, in_f, out_f)
    oa, ob = orc.linear_int_stages(dtype, w, x, m, in_f, out_f)
    assert np.array_equal(a, oa)
    if dtype != DType.Q6K:      # Q6_K has one integer stage (isum)
        assert np.array_equal(b, ob)


@pytest.mark.parametrize("m,in_f,out_f", [(5, 512, 40), (70, 768, 150), (200, 512, 40), (1030, 256, 70)])
def test_prefill_q4k_int_stages_bit_exact(be, m, in_f, out_f):
    # full-range payload bytes: every scale, min and code value occurs (sc up to 63 exercises the
    # split-scale operands, large |bsums| the split sums)
    w = orc.synth_weight(DType.Q4K, in_f * out_f, 0x208)
    x = synth_normal_f32(77, m * in_f) * np.float32(3.0)
    x[in_f:2 * in_f] = 1e4      # saturates every code to +127: bsums reach +4064
    x[2 * in_f:3 * in_f] = -1e4
    a, b = be.linear_int_stages(DType.Q4K, be.upload_new(w), be.upload_new(x), m, in_f, out_f)
    oa, ob = orc.linear_int_stages(DType.Q4K, w, x, m, in_f, out_f)
    assert np.array_equal(a, oa)
    assert np.array_equal(b, ob)


@pytest.mark.parametrize("dtype", [DType.Q6K, DType.Q8_0, DType.Q2_0])
def test_prefill_other_formats_vs_oracle(be, dtype):
    m, in_f, out_f = 5, 1024, 72
    w = synth_weight(dtype, 9, out_f, in_f)
    x = synth_normal_f32(10, m * in_f)
    y = run_linear(be, dtype, w, x, m, in_f, out_f)
    gate(y, orc.linear(dtype, w, x, m, in_f, out_f))


# ───────────── prefill of Q6_K from 33 tokens: its own int8 MFMA kernel ─────────────

@pytest.mark.parametrize("m,in_f,out_f", [(33, 512, 40), (128, 256, 32), (130, 768, 130), (257, 2048, 384),
                                         (600, 1024, 100)])
def test_prefill_q6k_mfma_is_bit_identical_to_oracle(be, m, in_f, out_f):
    w = synth_weight(DType.Q6K, 310 + m, out_f, in_f)
    x = synth_normal_f32(410 + m, m * in_f)
    x[:in_f] *= 37.0
    x[2 * in_f:3 * in_f] = 0.0
    y = run_linear(be, DType.Q6K, w, x, m, in_f, out_f)
    want = orc.linear(DType.Q6K, w, x, m, in_f, out_f)
    gate(y, want)
    assert np.array_equal(y.view(np.uint32), want.view(np.uint32)), "not bit-identical"


def test_prefill_q6k_mfma_int_stage_bit_exact(be):
    # full-range payload: every 6-bit code, every int8 group scale (-128 included), saturated rows
    m, in_f, out_f = 140, 768, 70
    w = orc.synth_weight(DType.Q6K, in_f * out_f, 0x20A)
    x = synth_normal_f32(78, m * in_f) * np.float32(3.0)
    x[in_f:2 * in_f] = 1e4
    x[2 * in_f:3 * in_f] = -1e4
    a, _ = be.linear_int_stages(DType.Q6K, be.upload_new(w), be.upload_new(x), m, in_f, out_f)
    oa, _ = orc.linear_int_stages(DType.Q6K, w, x, m, in_f, out_f)
    assert np.array_equal(a, oa)


def test_full_size_prefill_q6k(be):
    """4096 x 12288 (a Q4_K_M file's ffn_down) at 512 tokens: sampled rows bit-identical to the oracle
    and to each token's own one-token result."""
    m, in_f, out_f = 512, 12288, 4096
    w = synth_weight(DType.Q6K, 930, out_f, in_f)
    x = synth_normal_f32(931, m * in_f)
    wb = be.upload_new(w)
    yb = be.alloc(m * out_f * 4)
    be.linear(DType.Q6K, wb, be.upload_new(x), yb, m, in_f, out_f)
    y = be.download(yb, np.empty((m, out_f), np.float32))
    toks = [0, 1, 255, 511]
    xs = x[np.concatenate([np.arange(t * in_f, (t + 1) * in_f) for t in toks])]
    for row0 in (0, 2000, out_f - 32):
        want = _oracle_rows(DType.Q6K, w, xs, len(toks), in_f, out_f, row0, 32)
        assert np.array_equal(y[toks, row0:row0 + 32].view(np.uint32), want.view(np.uint32)), "not bit-identical"
    y1 = be.alloc(out_f * 4)
    for t in toks[:2]:
        be.linear(DType.Q6K, wb, be.upload_new(x[t * in_f:(t + 1) * in_f]), y1, 1, in_f, out_f)
        single = be.download(y1, np.empty((1, out_f), np.float32))
        assert np.array_equal(single[0].view(np.uint32), y[t].view(np.uint32)), "batch != single"


# ───────────── prefill of Q5_K from 33 tokens: its own int8 MFMA kernel ─────────────

@pytest.mark.parametrize("m,in_f,out_f", [(33, 512, 40), (128, 256, 32), (130, 768, 130), (257, 2048, 384),
                                         (600, 1024, 100)])
def test_prefill_q5k_mfma_is_bit_identical_to_oracle(be, m, in_f, out_f):
    w = synth_weight(DType.Q5K, 330 + m, out_f, in_f)
    x = synth_normal_f32(430 + m, m * in_f)
    x[:in_f] *= 37.0
    x[2 * in_f:3 * in_f] = 0.0
    y = run_linear(be, DType.Q5K, w, x, m, in_f, out_f)
    want = orc.linear(DType.Q5K, w, x, m, in_f, out_f)
    gate(y, want)
    assert np.array_equal(y.view(np.uint32), want.view(np.uint32)), "not bit-identical"


def test_prefill_q5k_mfma_int_stages_bit_exact(be):
    # full-range payload: every 5-bit code, every 6-bit scale and min, saturated rows (|bsums| up to 4064)
    m, in_f, out_f = 140, 768, 70
    w = orc.synth_weight(DType.Q5K, in_f * out_f, 0x209)
    x = synth_normal_f32(80, m * in_f) * np.float32(3.0)
    x[in_f:2 * in_f] = 1e4
    x[2 * in_f:3 * in_f] = -1e4
    a, b = be.linear_int_stages(DType.Q5K, be.upload_new(w), be.upload_new(x), m, in_f, out_f)
    oa, ob = orc.linear_int_stages(DType.Q5K, w, x, m, in_f, out_f)
    assert np.array_equal(a, oa)
    assert np.array_equal(b, ob)


# ───────────── prefill of Q8_0 (rows of whole 256s) from 33 tokens: its own int8 MFMA kernel ─────────────

@pytest.mark.parametrize("m,in_f,out_f", [(33, 512, 40), (128, 256, 32), (130, 768, 130), (257, 2048, 384),
                                         (600, 1024, 100), (70, 1056, 64)])      # 1056: the per-32 arm, dot4
def test_prefill_q8_0_mfma_vs_oracle(be, m, in_f, out_f):
    w = synth_weight(DType.Q8_0, 320 + m, out_f, in_f)
    x = synth_normal_f32(420 + m, m * in_f)
    x[:in_f] *= 37.0
    x[2 * in_f:3 * in_f] = 0.0
    y = run_linear(be, DType.Q8_0, w, x, m, in_f, out_f)
    want = orc.linear(DType.Q8_0, w, x, m, in_f, out_f)
    assert np.all(y[2] == 0.0)
    gate(y, want)
    rel = np.linalg.norm(y.astype(np.float64) - want) / np.linalg.norm(want)
    assert rel < 2e-6, rel            # the same terms in another association: rounding level


def test_prefill_q8_0_mfma_int_stage_bit_exact(be):
    m, in_f, out_f = 140, 768, 70
    w = orc.synth_weight(DType.Q8_0, in_f * out_f, 0x205)          # full-range int8 codes
    x = synth_normal_f32(79, m * in_f) * np.float32(3.0)
    x[in_f:2 * in_f] = 1e4
    x[2 * in_f:3 * in_f] = -1e4
    a, _ = be.linear_int_stages(DType.Q8_0, be.upload_new(w), be.upload_new(x), m, in_f, out_f)
    oa, _ = orc.linear_int_stages(DType.Q8_0, w, x, m, in_f, out_f)
    assert np.array_equal(a, oa)


# ───────────── prefill of Q2_0 (rows of whole 256s) from 65 tokens: its own int8 MFMA kernel ─────────────

@pytest.mark.parametrize("m,in_f,out_f", [(65, 512, 40), (130, 768, 130), (257, 2048, 384), (600, 1024, 100),
                                         (70, 320, 64)])                        # 320: not whole 256s, dot4
def test_prefill_q2_0_mfma_vs_oracle(be, m, in_f, out_f):
    w = synth_weight(DType.Q2_0, 340 + m, out_f, in_f)
    x = synth_normal_f32(440 + m, m * in_f)
    x[:in_f] *= 37.0
    x[2 * in_f:3 * in_f] = 0.0
    y = run_linear(be, DType.Q2_0, w, x, m, in_f, out_f)
    want = orc.linear(DType.Q2_0, w, x, m, in_f, out_f)
    assert np.all(y[2] == 0.0)
    gate(y, want)
    rel = np.linalg.norm(y.astype(np.float64) - want) / np.linalg.norm(want)
    assert rel < 3e-6, rel


def test_prefill_q2_0_mfma_int_stage_bit_exact(be):
    m, in_f, out_f = 140, 768, 70
    w = orc.synth_weight(DType.Q2_0, in_f * out_f, 0x216)          # all four code values
    x = synth_normal_f32(82, m * in_f) * np.float32(3.0)
    x[in_f:2 * in_f] = 1e4
    x[2 * in_f:3 * in_f] = -1e4
    a, _ = be.linear_int_stages(DType.Q2_0, be.upload_new(w), be.upload_new(x), m, in_f, out_f)
    oa, _ = orc.linear_int_stages(DType.Q2_0, w, x, m, in_f, out_f)
    assert np.array_equal(a, oa)


# ───────────── hand-derived known answers (tests/golden/known_answers.json), no oracle involved ─────────────

def _golden():
    import json
    import os
    with open(os.path.join(os.path.dirname(__file__), "golden", "known_answers.json")) as f:
        return json.load(f)


@pytest.mark.parametrize("case", _golden()["dots"], ids=lambda c: c["name"])
@pytest.mark.parametrize("m", [1, 3, 40, 130])
def test_known_answer_dots_on_the_device(be, case, m):
    """Every kernel route (decode GEMV, batch GEMV, skinny / tiled / shared MFMA) against values
    derived on paper: out_f copies of the row, m copies of the all-127 activation."""
    row = b"".join(bytes.fromhex(h) * n for h, n in case["parts"])
    out_f, in_f, dtype = 37, case["in_f"], case["dtype"]
    w = np.frombuffer(row * out_f, np.uint8)
    x = np.full(m * in_f, 127.0, np.float32)
    y = run_linear(be, dtype, w, x, m, in_f, out_f)
    assert np.all(y == np.float32(case["y"]))
    a, b = be.linear_int_stages(dtype, be.upload_new(w), be.upload_new(x), m, in_f, out_f)
    assert np.array_equal(a.reshape(m * out_f, -1), np.tile(np.array(case["int_a"], np.int32), (m * out_f, 1)))
    if "int_b" in case:
        assert np.array_equal(b.reshape(m * out_f, -1), np.tile(np.array(case["int_b"], np.int32), (m * out_f, 1)))


def test_known_answer_quantizer_ties_on_the_device(be):
    g = _golden()["quantize_q8"]
    x = np.zeros(g["k"], np.float32)
    x[:len(g["x_head"])] = g["x_head"]
    qs, d, bs, bs16 = be.quantize_q8(be.upload_new(x), 1, g["k"])
    assert d[0, 0] == g["d"] and list(qs[0, :len(g["q_head"])]) == g["q_head"]
    assert not qs[0, len(g["q_head"]):].any()
    assert bs[0, 0] == g["bsums0"] and bs16[0, 0] == g["bsums16_0"] and not bs[0, 1:].any() and not bs16[0, 1:].any()


# ───────────── full benchmark sizes: sampled rows against the oracle + batch == single ─────────────

def _oracle_rows(dtype, w, x, m, in_f, out_f, row0, n):
    """Oracle output for weight rows [row0, row0 + n) only (Op::Linear's w_off slicing)."""
    return orc.linear(dtype, w, x, m, in_f, n, w_numel=out_f * in_f, w_off=row0 * in_f)


@pytest.mark.parametrize("dtype", [DType.Q4K, DType.Q6K, DType.Q8_0, DType.Q2_0])
@pytest.mark.parametrize("in_f,out_f", [(4096, 12288), (12288, 4096)])
def test_full_size_decode_rows_vs_oracle(be, dtype, in_f, out_f):
    w = synth_weight(dtype, 900 + in_f, out_f, in_f)
    x = synth_normal_f32(901, in_f)
    y = run_linear(be, dtype, w, x, 1, in_f, out_f)
    for row0 in (0, out_f // 2 - 7, out_f - 48):
        want = _oracle_rows(dtype, w, x, 1, in_f, out_f, row0, 48)
        got = y[:, row0:row0 + 48]
        gate(got, want)
        if dtype in (DType.Q4K, DType.Q6K):
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), "not bit-identical"


@pytest.mark.parametrize("m", [8, 64, 512, 1024, 1100, 2048])
def test_full_size_prefill_q4k(be, m):
    """K = 4096 -> N = 12288 at the benchmark's token counts (every Q4_K kernel route; 512, 1024 and
    2048 tokens fill whole rounds of 96-row strips, 1100 takes 64-row strips): sampled rows against the
    oracle and every token's row against its own m = 1 result - bit-identical below 128 tokens, within
    the contracted epilogue's 2e-6 from there on (the per-block integers of those routes are checked
    exactly in the strip tests below)."""
    in_f, out_f = 4096, 12288
    w = synth_weight(DType.Q4K, 910, out_f, in_f)
    x = synth_normal_f32(911 + m, m * in_f)
    wb = be.upload_new(w)
    yb = be.alloc(m * out_f * 4)
    be.linear(DType.Q4K, wb, be.upload_new(x), yb, m, in_f, out_f)
    y = be.download(yb, np.empty((m, out_f), np.float32))
    toks = sorted({0, 1, m // 2, m - 1})
    for row0 in (0, 6000, out_f - 32):
        want = _oracle_rows(DType.Q4K, w, x[np.concatenate([np.arange(t * in_f, (t + 1) * in_f) for t in toks])],
                            len(toks), in_f, out_f, row0, 32)
        got = y[toks, row0:row0 + 32]
        if m < 128:
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), "not bit-identical"
        else:
            close(got, want)
    y1 = be.alloc(out_f * 4)
    for t in toks:
        be.linear(DType.Q4K, wb, be.upload_new(x[t * in_f:(t + 1) * in_f]), y1, 1, in_f, out_f)
        single = be.download(y1, np.empty((1, out_f), np.float32))
        if m < 128:
            assert np.array_equal(single[0].view(np.uint32), y[t].view(np.uint32)), "batch != single"
        else:
            close(y[t], single[0])


@pytest.mark.parametrize("m,in_f,out_f", [(2560, 256, 2304), (2400, 768, 2300), (512, 512, 12288), (512, 1024, 4096),
                                          (700, 512, 3000), (1024, 768, 4100), (300, 2304, 2500)])
def test_q4k_strip_route_is_exact(be, m, in_f, out_f):
    """The prefill strips (256 tokens x 32, 64 or 96 rows per workgroup, the height chosen for the grid):
    ragged last strip and token group, one and several blocks per row, odd block counts (the two lower
    heights unroll their block loop by two). Per-block sd / sm exact on sampled tokens and y within the
    contracted epilogue's bar, full-range payloads."""
    w = orc.synth_weight(DType.Q4K, in_f * out_f, 0x300 + in_f)      # full-range payload bytes
    x = synth_normal_f32(778 + m, m * in_f) * np.float32(3.0)
    x[in_f:2 * in_f] = 1e4      # saturates every code to +127: bsums reach +4064
    x[2 * in_f:3 * in_f] = -1e4
    wb, xb = be.upload_new(w), be.upload_new(x)
    yb = be.alloc(m * out_f * 4)
    be.linear(DType.Q4K, wb, xb, yb, m, in_f, out_f)
    y = be.download(yb, np.empty((m, out_f), np.float32))
    toks = sorted({0, 1, 2, 31, 32, 255, 256, m // 2 + 3, m - 33, m - 1})
    xs = x.reshape(m, in_f)[toks].ravel()
    want = orc.linear(DType.Q4K, w, xs, len(toks), in_f, out_f)
    close(y[toks], want)
    sd, sm = be.linear_int_stages(DType.Q4K, wb, xb, m, in_f, out_f)
    osd, osm = orc.linear_int_stages(DType.Q4K, w, xs, len(toks), in_f, out_f)
    assert np.array_equal(sd[toks], osd) and np.array_equal(sm[toks], osm)


def test_q4k_strips_at_sixteen_blocks_on_4096_rows(be):
    """1280 tokens x 4096 rows: five token groups of 64- or 32-row strips, 16 blocks per row (the
    double-buffered activation fragments at the benchmark's K)."""
    m, in_f, out_f = 1280, 4096, 4096
    w = synth_weight(DType.Q4K, 930, out_f, in_f)
    x = synth_normal_f32(931, m * in_f)
    y = run_linear(be, DType.Q4K, w, x, m, in_f, out_f)
    toks = [0, 255, 256, 640, 1279]
    for row0 in (0, 2040, out_f - 32):
        want = _oracle_rows(DType.Q4K, w, x.reshape(m, in_f)[toks].ravel(), len(toks), in_f, out_f, row0, 32)
        close(y[toks, row0:row0 + 32], want)


@pytest.mark.parametrize("dtype", [DType.Q6K, DType.Q8_0])
@pytest.mark.parametrize("in_f,out_f", [(4096, 12288), (12288, 4096)])
def test_full_size_batch8_rows_vs_oracle(be, dtype, in_f, out_f):
    """Eight tokens at the full Qwen3-8B grids (the tile heights a grid of 12288 or 4096 rows gets
    differ from a 256-row one's): sampled rows against the oracle."""
    m = 8
    w = synth_weight(dtype, 940 + in_f, out_f, in_f)
    x = synth_normal_f32(941, m * in_f)
    y = run_linear(be, dtype, w, x, m, in_f, out_f)
    for row0 in (0, out_f // 2 - 5, out_f - 40):
        want = _oracle_rows(dtype, w, x, m, in_f, out_f, row0, 40)
        got = y[:, row0:row0 + 40]
        gate(got, want)
        if dtype == DType.Q6K:
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), "not bit-identical"


def test_ternary_output_head_rows_vs_oracle(be):
    in_f, out_f = 4096, 151936
    w = synth_weight(DType.Q2_0, 920, out_f, in_f)
    x = synth_normal_f32(921, in_f)
    y = run_linear(be, DType.Q2_0, w, x, 1, in_f, out_f)
    for row0 in (0, 77777, out_f - 64):
        gate(y[:, row0:row0 + 64], _oracle_rows(DType.Q2_0, w, x, 1, in_f, out_f, row0, 64))


# ───────────── Q8_0 rows that are whole 32s but not whole 256s: the per-32 arm ─────────────

@pytest.mark.parametrize("m", [1, 3, 8, 20])
@pytest.mark.parametrize("in_f,out_f", [(96, 40), (1152, 300), (2080, 64), (4128, 33)])
def test_q8_0_per32_rows_vs_oracle(be, m, in_f, out_f):
    w = synth_weight(DType.Q8_0, 70 + in_f, out_f, in_f)
    x = synth_normal_f32(71 + m, m * in_f)
    y = run_linear(be, DType.Q8_0, w, x, m, in_f, out_f)
    gate(y, orc.linear(DType.Q8_0, w, x, m, in_f, out_f))
    a, _ = be.linear_int_stages(DType.Q8_0, be.upload_new(w), be.upload_new(x), m, in_f, out_f)
    oa, _ = orc.linear_int_stages(DType.Q8_0, w, x, m, in_f, out_f)
    assert np.array_equal(a, oa)
