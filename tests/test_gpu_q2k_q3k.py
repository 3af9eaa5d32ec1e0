"""GPU parity of Q2_K, Q3_K, IQ4_XS, TQ2_0 and TQ1_0 weights against the CPU oracle, through the C ABI: Op::Linear
(one token and batches), Op::EmbedGather tables and Op::MoeFfn expert banks.

infr-cpu multiplies these formats with a per-256 int8 activation (crates/infr-cpu/src/lib.rs:1043-1124,
vec_dot_q2k / vec_dot_q3k / vec_dot_iq4xs / vec_dot_tq2_0 in crates/infr-cpu/src/kernels.rs): the integer stages must be equal and,
since the device adds the per-superblock f32 terms in block order like the CPU, every output must
be bit-identical. Weights are the oracle's full-range payloads (every 2-/3-bit code, all 6-bit
scale patterns, both signs of the Q3_K scales)."""
import numpy as np
import pytest

from infr_amd import Bindings, DType, Graph, InfrError, Linear, Status, TensorDesc, synth_normal_f32
from oracle import oracle as orc
from tests.test_gpu_linear import _oracle_rows, gate, run_linear
from tests.test_gpu_moe import check, run_moe

pytestmark = pytest.mark.gpu

BOTH = [DType.Q2K, DType.Q3K, DType.IQ4XS, DType.TQ2_0, DType.TQ1_0]
ids = lambda d: DType(d).name


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


@pytest.mark.parametrize("dtype", BOTH, ids=ids)
@pytest.mark.parametrize("in_f,out_f", [(256, 8), (768, 37), (2048, 100), (4096, 256), (5120, 64), (12288, 96),
                                        (32768, 20), (1280, 1)])
def test_decode_is_bit_identical_to_the_oracle(be, dtype, in_f, out_f):
    w = orc.synth_weight(dtype, in_f * out_f, 0x51 + in_f)
    x = synth_normal_f32(200 + out_f, in_f)
    y = run_linear(be, dtype, w, x, 1, in_f, out_f)
    want = orc.linear(dtype, w, x, 1, in_f, out_f)
    gate(y, want)
    assert np.array_equal(bits(y).ravel(), bits(want).ravel()), f"not bit-identical at {in_f} x {out_f}"


@pytest.mark.parametrize("dtype", BOTH, ids=ids)
@pytest.mark.parametrize("m", [1, 3, 8, 19])
def test_int_stages_bit_exact(be, dtype, m):
    in_f, out_f = 1024, 24
    w = orc.synth_weight(dtype, in_f * out_f, 0x301 + dtype)
    x = orc.gen_f32(m * in_f, 0x9E37 + dtype)
    a, b = be.linear_int_stages(dtype, be.upload_new(w), be.upload_new(x), m, in_f, out_f)
    oa, ob = orc.linear_int_stages(dtype, w, x, m, in_f, out_f)
    assert np.array_equal(a, oa)
    if dtype == DType.Q2K:
        assert np.array_equal(b, ob)         # the dmin stage: sum of (scale >> 4) * bsums16


@pytest.mark.parametrize("dtype", BOTH, ids=ids)
@pytest.mark.parametrize("m", [2, 5, 8, 9, 19, 40, 130])
def test_batches_are_bit_identical_to_the_oracle(be, dtype, m):
    """Two tokens share one pass of the dot4 kernel over the weights; from three the 16-token K-split
    MFMA kernel takes rows of two superblocks and more (an even number of them for Q3_K and TQ2_0),
    16 tokens at a time; other rows, and TQ1_0 at every token count, keep the dot4 kernel, eight
    tokens per pass. Every token's value is the one-token value."""
    in_f, out_f = 1024, 96
    w = orc.synth_weight(dtype, in_f * out_f, 0x77 + m)
    x = synth_normal_f32(8 + m, m * in_f)
    x[:in_f] *= 29.0
    x[in_f:2 * in_f] = 0.0           # an all-zero row
    y = run_linear(be, dtype, w, x, m, in_f, out_f)
    want = orc.linear(dtype, w, x, m, in_f, out_f).reshape(m, out_f)
    assert np.all(y[1] == 0.0)
    gate(y, want)
    assert np.array_equal(bits(y), bits(want)), "not bit-identical"


@pytest.mark.parametrize("dtype", BOTH, ids=ids)
def test_batch_on_long_rows_and_many_rows(be, dtype):
    for m, in_f, out_f in ((4, 8192, 40), (7, 4096, 1031), (3, 256, 5), (5, 768, 33), (16, 1280, 50), (12, 2048, 17)):
        w = orc.synth_weight(dtype, in_f * out_f, 0x99 + m)
        x = orc.gen_f32(m * in_f, 0x1234 + m)
        y = run_linear(be, dtype, w, x, m, in_f, out_f)
        want = orc.linear(dtype, w, x, m, in_f, out_f).reshape(m, out_f)
        assert np.array_equal(bits(y), bits(want)), f"not bit-identical at m {m}, {in_f} x {out_f}"


@pytest.mark.parametrize("dtype", BOTH, ids=ids)
def test_full_size_rows_vs_oracle(be, dtype):
    in_f, out_f = 4096, 12288
    w = orc.synth_weight(dtype, in_f * out_f, 900 + int(dtype))
    x = synth_normal_f32(901, in_f)
    y = run_linear(be, dtype, w, x, 1, in_f, out_f)
    for row0 in (0, out_f // 2 - 7, out_f - 48):
        want = _oracle_rows(dtype, w, x, 1, in_f, out_f, row0, 48)
        got = y[:, row0:row0 + 48]
        gate(got, want)
        assert np.array_equal(bits(got), bits(want)), "not bit-identical"


@pytest.mark.parametrize("dtype", BOTH, ids=ids)
def test_w_off_selects_rows_of_a_concatenated_weight(be, dtype):
    """Q2_K rows are 84 bytes per 256 weights, Q3_K rows 110, IQ4_XS rows 136: row starts fall on
    4-, 2- and 8-byte boundaries only."""
    in_f, rows = 768, 40
    w = orc.synth_weight(dtype, in_f * rows, 3)
    x = synth_normal_f32(4, in_f)
    for row0, n in ((0, 40), (7, 16), (33, 7)):
        y = run_linear(be, dtype, w, x, 1, in_f, n, w_off=row0 * in_f, w_numel=rows * in_f)
        want = orc.linear(dtype, w, x, 1, in_f, n, w_numel=rows * in_f, w_off=row0 * in_f)
        assert np.array_equal(bits(y).ravel(), bits(want).ravel())


@pytest.mark.parametrize("dtype", BOTH, ids=ids)
def test_rows_that_are_not_whole_superblocks_are_refused(be, dtype):
    in_f, out_f = 256 + 32, 4
    w = np.zeros(2 * out_f * orc.block_layout(dtype)[1], np.uint8)
    with pytest.raises(InfrError) as e:
        run_linear(be, dtype, w, np.zeros(in_f, np.float32), 1, in_f, out_f)
    assert e.value.status == Status.Unsupported


def test_a_plan_mixes_them_with_other_formats(be):
    """One decode step's worth of Linears over one activation, each in its own format: the plan
    groups by (format, in_f) and every output equals the single-op value."""
    in_f = 2048
    outs = [(DType.Q2K, 96), (DType.Q3K, 80), (DType.Q4K, 64), (DType.Q2K, 33), (DType.Q3K, 130), (DType.IQ4XS, 70),
            (DType.IQ4XS, 9), (DType.TQ2_0, 45), (DType.TQ1_0, 77)]
    g = Graph()
    x = g.input(TensorDesc((1, in_f), DType.F32))
    ws, ys = [], []
    for dt, out_f in outs:
        ws.append(g.weight(TensorDesc((out_f, in_f), dt)))
        ys.append(g.output(TensorDesc((1, out_f), DType.F32)))
        g.push(Linear(x, ws[-1], ys[-1], 1, in_f, out_f))
    xv = synth_normal_f32(77, in_f)
    wv = [orc.synth_weight(dt, in_f * out_f, 0x600 + i) for i, (dt, out_f) in enumerate(outs)]
    binds = Bindings().bind(x, be.upload_new(xv))
    ybs = []
    for i, (dt, out_f) in enumerate(outs):
        ybs.append(be.alloc(out_f * 4))
        binds.bind(ws[i], be.upload_new(wv[i])).bind(ys[i], ybs[-1])
    plan = be.compile(g)
    for _ in range(2):
        be.execute(plan, binds)
        for i, (dt, out_f) in enumerate(outs):
            got = be.download(ybs[i], np.empty(out_f, np.float32))
            want = orc.linear(dt, wv[i], xv, 1, in_f, out_f)
            assert np.array_equal(bits(got), bits(want).ravel()), f"op {i} ({DType(dt).name}) differs"


@pytest.mark.parametrize("m", [6, 24])
def test_a_batch_plan_groups_them(be, m):
    """Linears of one level over one activation tensor at several tokens: the plan shares one
    quantized activation and one launch per (format, in_f) group."""
    in_f = 2048
    outs = [(DType.Q2K, 96), (DType.Q2K, 40), (DType.Q3K, 80), (DType.Q3K, 33), (DType.Q4K, 64), (DType.IQ4XS, 50),
            (DType.IQ4XS, 31), (DType.TQ2_0, 45), (DType.TQ2_0, 8), (DType.TQ1_0, 21)]
    g = Graph()
    x = g.input(TensorDesc((m, in_f), DType.F32))
    ws, ys = [], []
    for dt, out_f in outs:
        ws.append(g.weight(TensorDesc((out_f, in_f), dt)))
        ys.append(g.output(TensorDesc((m, out_f), DType.F32)))
        g.push(Linear(x, ws[-1], ys[-1], m, in_f, out_f))
    xv = synth_normal_f32(78, m * in_f)
    wv = [orc.synth_weight(dt, in_f * out_f, 0x610 + i) for i, (dt, out_f) in enumerate(outs)]
    binds = Bindings().bind(x, be.upload_new(xv))
    ybs = []
    for i, (dt, out_f) in enumerate(outs):
        ybs.append(be.alloc(m * out_f * 4))
        binds.bind(ws[i], be.upload_new(wv[i])).bind(ys[i], ybs[-1])
    plan = be.compile(g)
    for _ in range(2):
        be.execute(plan, binds)
        for i, (dt, out_f) in enumerate(outs):
            got = be.download(ybs[i], np.empty((m, out_f), np.float32))
            want = orc.linear(dt, wv[i], xv, m, in_f, out_f).reshape(m, out_f)
            assert np.array_equal(bits(got), bits(want)), f"op {i} ({DType(dt).name}) differs"


@pytest.mark.parametrize("rows", [1, 5])
@pytest.mark.parametrize("dtype", BOTH, ids=ids)
def test_moe_banks(be, dtype, rows):
    """expert_acts_kind (crates/infr-cpu/src/moe.rs:42-53) has no int8 arm for these formats:
    their expert rows are decoded and multiplied with the raw activation row at every row count."""
    ne, n_expert, n_used, nff = 512, 8, 2, 256
    gate_w = orc.synth_weight(dtype, n_expert * nff * ne, 0x700)
    up_w = orc.synth_weight(dtype, n_expert * nff * ne, 0x701)
    down_w = orc.synth_weight(dtype, n_expert * ne * nff, 0x702)
    x = synth_normal_f32(230 + rows, rows * ne)
    router = synth_normal_f32(231, n_expert * ne, sigma=0.05)
    got = run_moe(be, x, router, gate_w, up_w, down_w, rows, ne, n_expert, n_used, nff, 1.0, dtype)
    want = orc.moe_ffn(x, router, gate_w, up_w, down_w, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff,
                       gate_dtype=int(dtype), up_dtype=int(dtype), down_dtype=int(dtype))
    check(*got, *want)


TILED = [DType.Q2K, DType.Q3K, DType.IQ4XS, DType.TQ2_0, DType.TQ1_0]


@pytest.mark.parametrize("dtype", TILED, ids=ids)
@pytest.mark.parametrize("m,in_f,out_f", [(97, 4096, 8224), (161, 1024, 96), (200, 2048, 70), (300, 768, 33), (512, 4096, 64),
                                          (300, 256, 1), (170, 8192, 40), (190, 1280, 50)])
def test_prefill_tiles_are_bit_identical_to_the_oracle(be, dtype, m, in_f, out_f):
    """Beyond the 16-token kernel's reach these formats take 128-token x 32-row tiles on the int8
    matrix cores: IQ4_XS a product per 32-weight sub-block scaled by ls - 32 in integers; Q2_K, Q3_K
    and TQ2_0 scaled codes (code x scale fits a byte), so a block is one chain of eight MFMAs, Q2_K's
    mins an f16 MFMA against per-16 sums formed in the kernel; TQ1_0 the same chain over its base-3
    digits minus one. Same per-block integers and f32
    expression as the one-token kernels, blocks in ascending order - every output bit-identical;
    ragged token and row counts and an odd number of blocks per row included."""
    w = orc.synth_weight(dtype, in_f * out_f, 0x4A + m)
    x = synth_normal_f32(30 + m, m * in_f)
    x[:in_f] *= 17.0
    x[in_f:2 * in_f] = 0.0
    y = run_linear(be, dtype, w, x, m, in_f, out_f)
    rows = np.unique(np.r_[0, 1, m // 2, m - 1, np.arange(0, m, max(1, m // 9))])
    for r in rows:                                    # (a sample of tokens keeps the oracle's time down at the large case)
        want = orc.linear(dtype, w, x[r * in_f:(r + 1) * in_f], 1, in_f, out_f).ravel()
        assert np.array_equal(bits(y[r]), bits(want)), f"token {r} differs"
    assert np.all(y[1] == 0.0)


@pytest.mark.parametrize("dtype", TILED, ids=ids)
def test_prefill_tiles_int_stages_are_exact(be, dtype):
    m, in_f, out_f = 200, 1024, 40
    w = orc.synth_weight(dtype, in_f * out_f, 0x4B)
    x = orc.gen_f32(m * in_f, 0x77AA)
    a, b = be.linear_int_stages(dtype, be.upload_new(w), be.upload_new(x), m, in_f, out_f)
    oa, ob = orc.linear_int_stages(dtype, w, x, m, in_f, out_f)
    assert np.array_equal(a, oa)
    if dtype == DType.Q2K:
        assert np.array_equal(b, ob)
