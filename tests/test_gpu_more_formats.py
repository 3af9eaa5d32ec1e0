"""GPU parity of Op::Linear for Q5_K, Q4_0, Q4_1, Q5_0, Q5_1 and IQ4_NL against the CPU oracle,
through the C ABI. Integer stages bit-exact; Q5_K outputs bit-identical (same per-block expression
and the CPU's accumulation order); the 32-weight-block formats within rel-L2 <= 1e-4 and
max-abs <= 1e-3 * max|y| (their per-block terms are added in a different order than the CPU's).
One token of Q5_0 multiplies f32 activations, as infr-cpu does."""
import numpy as np
import pytest

from infr_amd import (Bindings, DType, Graph, InfrError, Linear, Status, TensorDesc, synth_normal_f32,
                      synth_weight)
from oracle import oracle as orc
from tests.test_gpu_linear import _oracle_rows, gate, run_linear

pytestmark = pytest.mark.gpu

BLK32 = [DType.Q4_0, DType.Q4_1, DType.Q5_0, DType.Q5_1, DType.IQ4NL]
ALL = BLK32 + [DType.Q5K]
ids = lambda d: DType(d).name


def shapes(dtype):
    if dtype == DType.Q5K:
        return [(256, 8), (768, 37), (4096, 256), (12288, 96), (5120, 64)]
    return [(32, 8), (96, 37), (2048, 100), (4096, 256), (4128, 33), (12288, 96), (1152, 300)]


@pytest.mark.parametrize("dtype", ALL, ids=ids)
def test_decode_vs_oracle(be, dtype):
    for in_f, out_f in shapes(dtype):
        w = synth_weight(dtype, 100 + in_f, out_f, in_f)
        x = synth_normal_f32(200 + out_f, in_f)
        y = run_linear(be, dtype, w, x, 1, in_f, out_f)
        want = orc.linear(dtype, w, x, 1, in_f, out_f)
        gate(y, want)
        if dtype == DType.Q5K:
            assert np.array_equal(y.view(np.uint32), want.view(np.uint32)), f"not bit-identical at {in_f}x{out_f}"


@pytest.mark.parametrize("dtype", ALL, ids=ids)
@pytest.mark.parametrize("m", [1, 3])
def test_int_stages_bit_exact(be, dtype, m):
    in_f, out_f = 1024, 24
    # full-range payload bytes (the reference's synth_weight recipe): every code and 5th-bit pattern
    w = orc.synth_weight(dtype, in_f * out_f, 0x301 + dtype)
    x = orc.gen_f32(m * in_f, 0x9E37 + dtype)
    if dtype == DType.Q5_0 and m == 1:
        with pytest.raises(InfrError) as e:
            be.linear_int_stages(dtype, be.upload_new(w), be.upload_new(x), 1, in_f, out_f)
        assert e.value.status == Status.Unsupported       # one token of Q5_0 has no integer stage
        return
    a, b = be.linear_int_stages(dtype, be.upload_new(w), be.upload_new(x), m, in_f, out_f)
    oa, ob = orc.linear_int_stages(dtype, w, x, m, in_f, out_f)
    assert np.array_equal(a, oa)
    if dtype == DType.Q5K:
        assert np.array_equal(b, ob)


@pytest.mark.parametrize("dtype", ALL, ids=ids)
def test_full_range_payload_decode(be, dtype):
    """LCG payload bytes with the reference's scale magnitudes: all 16 / 32 code values, both nibble
    halves, odd and even block alignment."""
    in_f, out_f = 2048 if dtype != DType.Q5K else 2304, 50
    w = orc.synth_weight(dtype, in_f * out_f, 0x77)
    x = synth_normal_f32(5, in_f)
    gate(run_linear(be, dtype, w, x, 1, in_f, out_f), orc.linear(dtype, w, x, 1, in_f, out_f))


@pytest.mark.parametrize("dtype", ALL, ids=ids)
@pytest.mark.parametrize("m", [2, 8, 40, 130])
def test_batches_vs_oracle(be, dtype, m):
    in_f, out_f = 1024, 96
    w = synth_weight(dtype, 7, out_f, in_f)
    x = synth_normal_f32(8 + m, m * in_f)
    x[:in_f] *= 29.0
    x[in_f:2 * in_f] = 0.0           # an all-zero row
    y = run_linear(be, dtype, w, x, m, in_f, out_f)
    want = orc.linear(dtype, w, x, m, in_f, out_f)
    assert np.all(y[1] == 0.0)
    gate(y, want)
    if dtype == DType.Q5K and m <= 8:
        assert np.array_equal(y.view(np.uint32), want.view(np.uint32)), "not bit-identical"


@pytest.mark.parametrize("dtype", BLK32, ids=ids)
@pytest.mark.parametrize("m", [9, 16, 17, 40, 64, 100, 128])
def test_nine_tokens_and_up_on_the_k_split_kernel_are_bit_identical(be, dtype, m):
    """From nine tokens the 32-weight-block formats take the 16-token K-split MFMA kernel (16 tokens
    at a time beyond that): one exact iprod per block and the CPU's f32 term per block, added in
    block order by the wave-to-wave chain (oracle orc_vec_dot_blk32 = infr-cpu's
    vec_dot_*_32_batch_scalar) - so, unlike the dot4 batches and the 128-token tiles, these outputs
    equal the scalar kernel's bits. Full-range payloads; a small matrix and one of long rows."""
    for in_f, out_f in ((1024, 70), (8192, 40)):
        w = orc.synth_weight(dtype, in_f * out_f, 0x30A)
        x = orc.gen_f32(m * in_f, 0x30A ^ 0x9E37)
        x[in_f:2 * in_f] = 0.0
        y = run_linear(be, dtype, w, x, m, in_f, out_f)
        want = orc.linear(dtype, w, x, m, in_f, out_f).reshape(m, out_f)
        assert np.array_equal(y.view(np.uint32), want.view(np.uint32)), f"not bit-identical at {in_f} x {out_f}"
    a, _ = be.linear_int_stages(dtype, be.upload_new(w), be.upload_new(x), m, in_f, out_f)
    oa, _ = orc.linear_int_stages(dtype, w, x, m, in_f, out_f)
    assert np.array_equal(a, oa)


def test_q5_0_one_token_is_the_f32_path_not_the_int8_one(be):
    in_f, out_f = 2048, 64
    w = synth_weight(DType.Q5_0, 31, out_f, in_f)
    x = synth_normal_f32(32, 2 * in_f)
    y1 = run_linear(be, DType.Q5_0, w, x[:in_f], 1, in_f, out_f)
    y2 = run_linear(be, DType.Q5_0, w, x, 2, in_f, out_f)
    exact = orc.linear(DType.Q5_0, w, x[:in_f], 1, in_f, out_f, reference_mode=True)
    gate(y1, exact)                                   # f32 activations: 1e-4 against decode + dot
    gate(y2, orc.linear(DType.Q5_0, w, x, 2, in_f, out_f))
    # and the int8 result really is a different number, so the gate above tells the arms apart
    rel = np.linalg.norm(y2[0] - exact[0]) / np.linalg.norm(exact[0])
    assert rel > 3e-4, rel


@pytest.mark.parametrize("dtype", ALL, ids=ids)
def test_full_size_rows_vs_oracle(be, dtype):
    in_f, out_f = 4096, 12288
    w = synth_weight(dtype, 900 + int(dtype), out_f, in_f)
    x = synth_normal_f32(901, in_f)
    y = run_linear(be, dtype, w, x, 1, in_f, out_f)
    for row0 in (0, out_f // 2 - 7, out_f - 48):
        want = _oracle_rows(dtype, w, x, 1, in_f, out_f, row0, 48)
        got = y[:, row0:row0 + 48]
        gate(got, want)
        if dtype == DType.Q5K:
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), "not bit-identical"


def test_w_off_on_2_mod_4_strides(be):
    """Row slices of a concatenated Q4_0 weight whose row stride (in_f/32*18) is 2 mod 4: rows start
    on both alignments."""
    in_f, rows = 32 * 9, 40                             # bpr = 162
    w = synth_weight(DType.Q4_0, 3, rows, in_f)
    x = synth_normal_f32(4, in_f)
    for row0, n in ((0, 40), (7, 16), (33, 7)):
        y = run_linear(be, DType.Q4_0, w, x, 1, in_f, n, w_off=row0 * in_f, w_numel=rows * in_f)
        gate(y, orc.linear(DType.Q4_0, w, x, 1, in_f, n, w_numel=rows * in_f, w_off=row0 * in_f))


def test_plan_with_mixed_formats_replays(be):
    """One plan holding a decode Linear of every format (Q5_0 as a launch of its own beside the
    grouped ones) and a small-batch pair, executed twice with fresh inputs."""
    in_f, out_f, m = 1024, 64, 4
    g = Graph()
    x1 = g.input(TensorDesc((1, in_f), DType.F32))
    xm = g.input(TensorDesc((m, in_f), DType.F32))
    binds = Bindings()
    ws, outs = {}, []
    for dt in ALL + [DType.Q4K]:
        wt = g.weight(TensorDesc((out_f, in_f), dt))
        ws[dt] = synth_weight(dt, 50 + int(dt), out_f, in_f)
        binds.bind(wt, be.upload_new(ws[dt]))
        y = g.output(TensorDesc((1, out_f), DType.F32))
        g.push(Linear(x1, wt, y, 1, in_f, out_f))
        yb = be.alloc(out_f * 4)
        binds.bind(y, yb)
        outs.append((dt, 1, yb))
        if dt in (DType.Q5_0, DType.Q5K):
            ym = g.output(TensorDesc((m, out_f), DType.F32))
            g.push(Linear(xm, wt, ym, m, in_f, out_f))
            ymb = be.alloc(m * out_f * 4)
            binds.bind(ym, ymb)
            outs.append((dt, m, ymb))
    plan = be.compile(g)
    x1b, xmb = be.alloc(in_f * 4), be.alloc(m * in_f * 4)
    binds.bind(x1, x1b).bind(xm, xmb)
    for rep in range(2):
        a, b = synth_normal_f32(70 + rep, in_f), synth_normal_f32(80 + rep, m * in_f)
        be.upload(x1b, a)
        be.upload(xmb, b)
        be.execute(plan, binds)
        for dt, rows, yb in outs:
            got = be.download(yb, np.empty((rows, out_f), np.float32))
            gate(got, orc.linear(dt, ws[dt], a if rows == 1 else b, rows, in_f, out_f))


def test_ragged_rows_are_refused(be):
    w = be.upload_new(np.zeros(4096, np.uint8))
    x = be.upload_new(np.zeros(4096, np.float32))
    y = be.alloc(4096)
    for dt, in_f in ((DType.Q4_0, 48), (DType.Q5_1, 16), (DType.Q5K, 128), (DType.IQ4NL, 40)):
        with pytest.raises(InfrError) as e:
            be.linear(dt, w, x, y, 1, in_f, 2, w_numel=2 * in_f)
        assert e.value.status == Status.Unsupported


def test_rows_beyond_eight_wave_steps(be):
    """in_f above the decode kernels' bound (32768; 16384 for Q8_0 / Q4_1 / Q5_1): rows of whole 256s
    run the prefill kernels at any token count - same integers, same results - and other lengths are
    Unsupported, never truncated. The bound itself still takes the decode kernel."""
    for dt, in_f in ((DType.Q8_0, 16384 + 32), (DType.Q4_1, 16384 + 32), (DType.Q5_0, 32768 + 256)):
        w = be.alloc(block_bytes(dt, in_f) * 2)
        x = be.alloc(in_f * 4)
        y = be.alloc(8)
        with pytest.raises(InfrError) as e:
            be.linear(dt, w, x, y, 1, in_f, 2)      # (one token of Q5_0 multiplies f32 activations: no int8 arm)
        assert e.value.status == Status.Unsupported
    in_f, out_f = 16384, 24
    w = synth_weight(DType.Q8_0, 77, out_f, in_f)
    x = synth_normal_f32(78, in_f)
    gate(run_linear(be, DType.Q8_0, w, x, 1, in_f, out_f), orc.linear(DType.Q8_0, w, x, 1, in_f, out_f))
    for dt, in_f in ((DType.Q4K, 33024), (DType.Q5K, 33024), (DType.Q6K, 33024), (DType.Q8_0, 16640),
                     (DType.Q4_0, 33024), (DType.Q4_1, 16640), (DType.Q2_0, 33024)):
        out_f = 40
        w = synth_weight(dt, 90 + int(dt), out_f, in_f)
        for m in (1, 5, 40):
            x = synth_normal_f32(91 + m, m * in_f)
            y = run_linear(be, dt, w, x, m, in_f, out_f)
            want = orc.linear(dt, w, x, m, in_f, out_f)
            gate(y, want)
            if dt in (DType.Q4K, DType.Q5K, DType.Q6K):
                assert np.array_equal(y.view(np.uint32), want.view(np.uint32)), (dt, m)


def test_long_rows_inside_a_plan(be):
    in_f, out_f = 33024, 32
    g, binds = Graph(), Bindings()
    x1 = g.input(TensorDesc((1, in_f), DType.F32))
    xs = synth_normal_f32(5, in_f)
    binds.bind(x1, be.upload_new(xs))
    outs = []
    for dt in (DType.Q4K, DType.Q6K):
        w = synth_weight(dt, 60 + int(dt), out_f, in_f)
        wt = g.weight(TensorDesc((out_f, in_f), dt))
        binds.bind(wt, be.upload_new(w))
        yt = g.output(TensorDesc((1, out_f), DType.F32))
        yb = be.alloc(out_f * 4)
        binds.bind(yt, yb)
        g.push(Linear(x1, wt, yt, 1, in_f, out_f))
        outs.append((dt, w, yb))
    plan = be.compile(g)
    for _ in range(2):
        be.execute(plan, binds)
        for dt, w, yb in outs:
            got = be.download(yb, np.empty((1, out_f), np.float32))
            want = orc.linear(dt, w, xs, 1, in_f, out_f)
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), dt


def block_bytes(dt, in_f):
    from infr_amd import block_layout
    e, b = block_layout(dt)
    return in_f // e * b


@pytest.mark.parametrize("dtype", BLK32, ids=ids)
def test_prefill_mfma_blk32_formats(be, dtype):
    """From 65 tokens, rows of whole 256s: the int8-MFMA kernel of the 32-weight-block formats. iprod
    per block bit-exact on full-range payloads; outputs at rounding level of the oracle (the same
    terms in another association)."""
    for m, in_f, out_f in ((65, 512, 40), (130, 768, 130), (257, 2048, 96), (70, 1056, 64)):   # 1056: a ragged last step
        w = synth_weight(dtype, 500 + m, out_f, in_f)
        x = synth_normal_f32(600 + m, m * in_f)
        x[:in_f] *= 37.0
        x[2 * in_f:3 * in_f] = 0.0
        y = run_linear(be, dtype, w, x, m, in_f, out_f)
        want = orc.linear(dtype, w, x, m, in_f, out_f)
        assert np.all(y[2] == 0.0)
        gate(y, want)
        rel = np.linalg.norm(y.astype(np.float64) - want) / np.linalg.norm(want)
        assert rel < 3e-6, (m, in_f, rel)
    m, in_f, out_f = 140, 768, 70
    w = orc.synth_weight(dtype, in_f * out_f, 0x310 + dtype)
    x = synth_normal_f32(81, m * in_f) * np.float32(3.0)
    x[in_f:2 * in_f] = 1e4
    x[2 * in_f:3 * in_f] = -1e4
    a, _ = be.linear_int_stages(dtype, be.upload_new(w), be.upload_new(x), m, in_f, out_f)
    oa, _ = orc.linear_int_stages(dtype, w, x, m, in_f, out_f)
    assert np.array_equal(a, oa)
    gate(run_linear(be, dtype, w, x, m, in_f, out_f), orc.linear(dtype, w, x, m, in_f, out_f))


@pytest.mark.parametrize("dtype", BLK32 + [DType.Q8_0, DType.Q2_0], ids=ids)
def test_prefill_mfma_rows_that_are_not_whole_256s(be, dtype):
    """Rows of whole 32-weight blocks that end inside a 256-element step (the gemma widths the
    reference calls out, crates/infr-cpu/src/lib.rs:1037-1042; Q8_0 rows of that kind multiply the
    per-32 activation like the nibble formats; Q2_0 needs whole 64s) take the same int8-MFMA
    kernel, the last step padded with zero blocks: iprod of every real block bit-exact, outputs at
    the rounding level of the oracle."""
    q2 = dtype == DType.Q2_0
    for m, in_f, out_f in ((100, 1152, 96), (65, 1056 if not q2 else 1088, 40), (200, 2112, 70),
                           (129, 96 if not q2 else 64, 33), (70, 4128 if not q2 else 4160, 48)):
        w = synth_weight(dtype, 700 + m, out_f, in_f)
        x = synth_normal_f32(800 + m, m * in_f)
        x[:in_f] *= 37.0
        x[2 * in_f:3 * in_f] = 0.0
        y = run_linear(be, dtype, w, x, m, in_f, out_f)
        want = orc.linear(dtype, w, x, m, in_f, out_f)
        assert np.all(y[2] == 0.0)
        gate(y, want)
        rel = np.linalg.norm(y.astype(np.float64) - want) / np.linalg.norm(want)
        assert rel < 3e-6, (m, in_f, rel)
    m, in_f, out_f = 70, 1184 if not q2 else 1216, 50
    w = orc.synth_weight(dtype, in_f * out_f, 0x320 + dtype)     # full-range payload bytes
    x = synth_normal_f32(82, m * in_f) * np.float32(3.0)
    x[in_f:2 * in_f] = 1e4
    a, _ = be.linear_int_stages(dtype, be.upload_new(w), be.upload_new(x), m, in_f, out_f)
    oa, _ = orc.linear_int_stages(dtype, w, x, m, in_f, out_f)
    assert np.array_equal(a, oa)
    gate(run_linear(be, dtype, w, x, m, in_f, out_f), orc.linear(dtype, w, x, m, in_f, out_f))


def test_q5_0_one_token_linears_of_a_level_share_a_launch(be):
    """One-token Q5_0 Linears multiply f32 activations (no int8 arm on the CPU): inside a plan the
    ops of a level run as one launch per row length - sixteen-wave workgroups from 8192 columns -
    over distinct activations, ragged row counts and a w_off slice, each within 1e-4 of decode + dot;
    a second level reads the first one's output."""
    spec = [(4096, 100, "x0"), (4096, 37, "x0"), (4096, 1, "x1"), (12288, 130, "x2"), (12288, 16, "x2"),
            (256, 9, "x3"), (13824, 21, "x4")]
    g, binds = Graph(), Bindings()
    xs, host = {}, {}
    for name, n in (("x0", 4096), ("x1", 4096), ("x2", 12288), ("x3", 256), ("x4", 13824)):
        xs[name] = g.input(TensorDesc((1, n), DType.F32))
        host[name] = synth_normal_f32(len(xs) + 500, n)
        binds.bind(xs[name], be.upload_new(host[name]))
    outs = []
    for i, (in_f, out_f, xn) in enumerate(spec):
        rows = out_f + 5                                  # the op takes rows 3 .. 3 + out_f of a taller weight
        w = synth_weight(DType.Q5_0, 300 + i, rows, in_f)
        wid = g.weight(TensorDesc((rows, in_f), DType.Q5_0))
        binds.bind(wid, be.upload_new(w))
        y = g.output(TensorDesc((1, out_f), DType.F32))
        yb = be.alloc(out_f * 4)
        binds.bind(y, yb)
        g.push(Linear(xs[xn], wid, y, 1, in_f, out_f, w_off=3 * in_f))
        outs.append((w, in_f, out_f, xn, yb, rows, y))
    # and a chain over two levels: x3 -> [256 x 256] -> [64 x 256]
    w1, w2 = synth_weight(DType.Q5_0, 400, 256, 256), synth_weight(DType.Q5_0, 401, 64, 256)
    a, b = g.weight(TensorDesc((256, 256), DType.Q5_0)), g.weight(TensorDesc((64, 256), DType.Q5_0))
    binds.bind(a, be.upload_new(w1)).bind(b, be.upload_new(w2))
    h, z = g.output(TensorDesc((1, 256), DType.F32)), g.output(TensorDesc((1, 64), DType.F32))
    hb, zb = be.alloc(256 * 4), be.alloc(64 * 4)
    binds.bind(h, hb).bind(z, zb)
    g.push(Linear(xs["x3"], a, h, 1, 256, 256))
    g.push(Linear(h, b, z, 1, 256, 64))
    plan = be.compile(g)
    for rep in range(2):
        be.execute(plan, binds)
        assert plan.launches() == 5, plan.launches()      # 4096, 12288, 256, 13824 on the first level; 256 on the second
        for w, in_f, out_f, xn, yb, rows, _ in outs:
            got = be.download(yb, np.empty((1, out_f), np.float32))
            gate(got, orc.linear(DType.Q5_0, w, host[xn], 1, in_f, out_f, w_numel=rows * in_f, w_off=3 * in_f,
                                 reference_mode=True))
        hv = be.download(hb, np.empty((1, 256), np.float32))
        gate(hv, orc.linear(DType.Q5_0, w1, host["x3"], 1, 256, 256, reference_mode=True))
        gate(be.download(zb, np.empty((1, 64), np.float32)), orc.linear(DType.Q5_0, w2, hv, 1, 256, 64, reference_mode=True))


@pytest.mark.parametrize("dtype", [DType.Q5K, DType.Q6K, DType.Q8_0, DType.IQ4XS, DType.Q4_0, DType.Q5_1, DType.IQ4NL, DType.Q2_0],
                         ids=lambda d: DType(d).name)
@pytest.mark.parametrize("m,out_f", [(300, 200), (512, 1024), (1000, 96)])
def test_narrow_matrices_keep_the_16_token_kernel_at_any_token_count(be, dtype, m, out_f):
    """A 128-token tile kernel walks whole rows per workgroup and has a floor however few rows there
    are, so matrices with few outputs (tokens x rows) stay on the 16-token K-split kernel, 16 tokens
    per pass, beyond its usual token range. Same integers and block order as at 16 tokens: the
    super-block formats and Q8_0 bit-identical to the oracle, the others within the path's 1e-4."""
    in_f = 1024
    w = synth_weight(dtype, 0x510 + int(dtype), out_f, in_f, 0.05)
    x = synth_normal_f32(0x520 + m, m * in_f)
    x[in_f:2 * in_f] = 0.0
    y = run_linear(be, dtype, w, x, m, in_f, out_f)
    toks = np.unique(np.r_[0, 1, 15, 16, m // 2, m - 17, m - 1])
    want = orc.linear(dtype, w, x.reshape(m, in_f)[toks].ravel(), len(toks), in_f, out_f).reshape(len(toks), out_f)
    if dtype in (DType.Q5K, DType.Q6K, DType.Q8_0, DType.IQ4XS):
        assert np.array_equal(y[toks].view(np.uint32), want.view(np.uint32))
    else:
        gate(y[toks], want)
    assert np.all(y[1] == 0.0)
