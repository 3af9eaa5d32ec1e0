"""GPU parity of MXFP4 and NVFP4 weights against the CPU oracle, through the C ABI: Op::Linear (one
token and batches), Op::EmbedGather tables and Op::MoeFfn expert banks.

infr-cpu multiplies both with the per-32 int8 activation at every token count, one token included
(crates/infr-cpu/src/lib.rs:1066-1076, 1145-1160, 1394-1432): MXFP4's per-block integers must be
equal; the f32 outputs are the same per-block terms added in another order than the CPU's
`sumf +=` chain, held to rel-L2 <= 1e-4 and max-abs <= 1e-3 * max|y| like the other 32-weight
formats. MXFP4's 17-byte blocks sit at every byte alignment."""
import numpy as np
import pytest

from infr_amd import Bindings, DType, Graph, InfrError, Linear, Status, TensorDesc, synth_normal_f32, synth_weight
from oracle import oracle as orc
from tests.test_gpu_linear import _oracle_rows, gate, run_linear
from tests.test_gpu_moe import check, run_moe

pytestmark = pytest.mark.gpu

BOTH = [DType.MXFP4, DType.NVFP4]
ids = lambda d: DType(d).name


@pytest.mark.parametrize("dtype", BOTH, ids=ids)
@pytest.mark.parametrize("in_f,out_f", [(64, 8), (96 * 2, 37), (2048, 100), (4096, 256), (4160, 33), (12288, 96),
                                        (16384, 20), (1280, 1), (1152, 300)])
def test_decode_vs_oracle(be, dtype, in_f, out_f):
    for w in (orc.synth_weight(dtype, in_f * out_f, 0x51 + in_f), synth_weight(dtype, 100 + in_f, out_f, in_f)):
        x = synth_normal_f32(200 + out_f, in_f)
        gate(run_linear(be, dtype, w, x, 1, in_f, out_f), orc.linear(dtype, w, x, 1, in_f, out_f))


@pytest.mark.parametrize("m", [1, 3, 8, 19])
def test_mxfp4_int_stages_bit_exact(be, m):
    in_f, out_f = 1024, 24
    w = orc.synth_weight(DType.MXFP4, in_f * out_f, 0x327)
    x = orc.gen_f32(m * in_f, 0x9E5E)
    a, _ = be.linear_int_stages(DType.MXFP4, be.upload_new(w), be.upload_new(x), m, in_f, out_f)
    oa, _ = orc.linear_int_stages(DType.MXFP4, w, x, m, in_f, out_f)
    assert np.array_equal(a, oa)


def test_nvfp4_has_no_integer_stage_entry(be):
    in_f, out_f = 256, 4
    w = orc.synth_weight(DType.NVFP4, in_f * out_f, 1)
    with pytest.raises(InfrError) as e:
        be.linear_int_stages(DType.NVFP4, be.upload_new(w), be.upload_new(np.zeros(in_f, np.float32)), 1, in_f, out_f)
    assert e.value.status == Status.Unsupported


@pytest.mark.parametrize("dtype", BOTH, ids=ids)
@pytest.mark.parametrize("m", [2, 5, 8, 9, 19, 40])
def test_batches_vs_oracle(be, dtype, m):
    in_f, out_f = 1024, 96
    w = orc.synth_weight(dtype, in_f * out_f, 0x77 + m)
    x = synth_normal_f32(8 + m, m * in_f)
    x[:in_f] *= 29.0
    x[in_f:2 * in_f] = 0.0           # an all-zero row
    y = run_linear(be, dtype, w, x, m, in_f, out_f)
    assert np.all(y[1] == 0.0)
    gate(y, orc.linear(dtype, w, x, m, in_f, out_f))


@pytest.mark.parametrize("dtype", BOTH, ids=ids)
def test_full_size_rows_vs_oracle(be, dtype):
    in_f, out_f = 4096, 12288
    w = synth_weight(dtype, 900 + int(dtype), out_f, in_f)
    x = synth_normal_f32(901, in_f)
    y = run_linear(be, dtype, w, x, 1, in_f, out_f)
    for row0 in (0, out_f // 2 - 7, out_f - 48):
        gate(y[:, row0:row0 + 48], _oracle_rows(dtype, w, x, 1, in_f, out_f, row0, 48))


def test_mxfp4_rows_start_at_every_byte_alignment(be):
    """in_f = 32 * 9: rows are 153 bytes, so consecutive rows start at every residue mod 4; w_off
    slices of a concatenated weight start anywhere too."""
    in_f, rows = 32 * 9, 41
    w = orc.synth_weight(DType.MXFP4, in_f * rows, 3)
    x = synth_normal_f32(4, in_f)
    for row0, n in ((0, 41), (7, 16), (33, 8), (2, 1)):
        y = run_linear(be, DType.MXFP4, w, x, 1, in_f, n, w_off=row0 * in_f, w_numel=rows * in_f)
        gate(y, orc.linear(DType.MXFP4, w, x, 1, in_f, n, w_numel=rows * in_f, w_off=row0 * in_f))
    y = run_linear(be, DType.MXFP4, w, np.tile(x, 3), 3, in_f, 16, w_off=7 * in_f, w_numel=rows * in_f)
    gate(y, orc.linear(DType.MXFP4, w, np.tile(x, 3), 3, in_f, 16, w_numel=rows * in_f, w_off=7 * in_f))


def test_mxfp4_weight_that_ends_on_a_page_boundary(be):
    """4096 rows of 128 blocks are 2176 pages exactly: the last block's codes end with the buffer, and
    nothing past them may be read."""
    in_f, out_f = 4096, 4096
    w = orc.synth_weight(DType.MXFP4, in_f * out_f, 9)
    assert w.size % 4096 == 0
    x = synth_normal_f32(5, in_f)
    y = run_linear(be, DType.MXFP4, w, x, 1, in_f, out_f)
    gate(y[:, -64:], _oracle_rows(DType.MXFP4, w, x, 1, in_f, out_f, out_f - 64, 64))


@pytest.mark.parametrize("dtype", BOTH, ids=ids)
def test_ragged_rows_are_refused(be, dtype):
    in_f, out_f = (32 if dtype == DType.MXFP4 else 64) + 16, 4
    w = np.zeros(2 * out_f * orc.block_layout(dtype)[1], np.uint8)
    with pytest.raises(InfrError) as e:
        run_linear(be, dtype, w, np.zeros(in_f, np.float32), 1, in_f, out_f)
    assert e.value.status == Status.Unsupported


@pytest.mark.parametrize("m", [1, 6])
def test_a_plan_mixes_them_with_other_formats(be, m):
    in_f = 2048
    outs = [(DType.MXFP4, 96), (DType.NVFP4, 80), (DType.Q4K, 64), (DType.MXFP4, 33), (DType.NVFP4, 130)]
    g = Graph()
    x = g.input(TensorDesc((m, in_f), DType.F32))
    ws, ys = [], []
    for dt, out_f in outs:
        ws.append(g.weight(TensorDesc((out_f, in_f), dt)))
        ys.append(g.output(TensorDesc((m, out_f), DType.F32)))
        g.push(Linear(x, ws[-1], ys[-1], m, in_f, out_f))
    xv = synth_normal_f32(77, m * in_f)
    wv = [orc.synth_weight(dt, in_f * out_f, 0x600 + i) for i, (dt, out_f) in enumerate(outs)]
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
            gate(got, orc.linear(dt, wv[i], xv, m, in_f, out_f))


@pytest.mark.parametrize("rows", [1, 5])
@pytest.mark.parametrize("dtype", BOTH, ids=ids)
def test_moe_banks(be, dtype, rows):
    """expert_acts_kind (crates/infr-cpu/src/moe.rs:42-53) has no int8 arm for these formats: expert
    rows are decoded and multiplied with the raw activation row at every row count (MXFP4 expert
    banks are what gpt-oss files carry)."""
    ne, n_expert, n_used, nff = 512, 8, 2, 256
    gate_w = synth_weight(dtype, 0x700, n_expert * nff, ne, 0.05)
    up_w = synth_weight(dtype, 0x701, n_expert * nff, ne, 0.05)
    down_w = synth_weight(dtype, 0x702, n_expert * ne, nff, 0.05)
    x = synth_normal_f32(230 + rows, rows * ne)
    router = synth_normal_f32(231, n_expert * ne, sigma=0.05)
    got = run_moe(be, x, router, gate_w, up_w, down_w, rows, ne, n_expert, n_used, nff, 1.0, dtype)
    want = orc.moe_ffn(x, router, gate_w, up_w, down_w, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff,
                       gate_dtype=int(dtype), up_dtype=int(dtype), down_dtype=int(dtype))
    check(*got, *want)


@pytest.mark.parametrize("rows", [1, 9, 40])
@pytest.mark.parametrize("dts", [(DType.MXFP4, DType.MXFP4, DType.Q4K), (DType.Q2K, DType.Q3K, DType.IQ4XS),
                                 (DType.Q4K, DType.Q4K, DType.NVFP4), (DType.TQ2_0, DType.TQ2_0, DType.TQ2_0)],
                         ids=lambda d: "-".join(DType(x).name for x in d))
def test_moe_banks_mixed_with_the_int8_formats(be, dts, rows):
    """Each bank of an op takes its own kind (expert_acts_kind, crates/infr-cpu/src/moe.rs:42-53):
    per-256 int8 activations for a Q4_K bank from two rows up, decoded rows for the others; rows
    beyond the bucketing thresholds too."""
    from tests.test_gpu_moe import run_moe_mixed
    ne, n_expert, n_used, nff = 1024, 16, 4, 512
    gate_w = synth_weight(dts[0], 0x710, n_expert * nff, ne, 0.05)
    up_w = synth_weight(dts[1], 0x711, n_expert * nff, ne, 0.05)
    down_w = synth_weight(dts[2], 0x712, n_expert * ne, nff, 0.05)
    x = synth_normal_f32(240 + rows, rows * ne)
    router = synth_normal_f32(241, n_expert * ne, sigma=0.05)
    got = run_moe_mixed(be, x, router, gate_w, up_w, down_w, rows, ne, n_expert, n_used, nff, dts)
    want = orc.moe_ffn(x, router, gate_w, up_w, down_w, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff,
                       gate_dtype=int(dts[0]), up_dtype=int(dts[1]), down_dtype=int(dts[2]))
    check(*got, *want)


@pytest.mark.parametrize("m,in_f,out_f", [(41, 1024, 96), (64, 4096, 8200), (130, 2048, 70), (300, 288, 33), (200, 1280, 50),
                                          (70, 8192, 40), (512, 4096, 64)])
def test_mxfp4_prefill_tiles(be, m, in_f, out_f):
    """From 33..65 tokens (by shape) MXFP4 takes the 32-weight-block formats' 128-token tiles on the
    int8 matrix cores: one MFMA per block over the doubled E2M1 table values, scaled by the halved
    E8M0 scale and the per-32 activation scale - per-block integers equal to the oracle's, y within
    the path's 1e-4 (another association of the same f32 terms); rows that are not whole 256s and
    17-byte blocks at every byte alignment included."""
    w = orc.synth_weight(DType.MXFP4, in_f * out_f, 0x5A + m)
    x = synth_normal_f32(40 + m, m * in_f)
    x[in_f:2 * in_f] = 0.0
    y = run_linear(be, DType.MXFP4, w, x, m, in_f, out_f)
    toks = np.unique(np.r_[0, 1, 31, 32, m // 2, m - 1])
    want = orc.linear(DType.MXFP4, w, x.reshape(m, in_f)[toks].ravel(), len(toks), in_f, out_f)
    gate(y[toks], want)
    assert np.all(y[1] == 0.0)
    if out_f <= 96:
        a, _ = be.linear_int_stages(DType.MXFP4, be.upload_new(w), be.upload_new(x), m, in_f, out_f)
        oa, _ = orc.linear_int_stages(DType.MXFP4, w, x, m, in_f, out_f)
        assert np.array_equal(a, oa)


@pytest.mark.parametrize("m,in_f,out_f", [(25, 1024, 96), (9, 4096, 8200), (130, 2048, 70), (300, 320, 33), (200, 1280, 50),
                                          (70, 8192, 40), (512, 4096, 64)])
def test_nvfp4_prefill_tiles(be, m, in_f, out_f):
    """From 9..41 tokens (by shape) NVFP4 takes the same tiles with a K = 16 MFMA per 16-weight
    sub-block (lane swaps put the activation halves in operand order), each scaled by its halved
    UE4M3 scale and the per-32 activation scale: y within the path's 1e-4 of the oracle; rows that
    are not whole 256s included."""
    w = orc.synth_weight(DType.NVFP4, in_f * out_f, 0x5B + m)
    x = synth_normal_f32(50 + m, m * in_f)
    x[in_f:2 * in_f] = 0.0
    y = run_linear(be, DType.NVFP4, w, x, m, in_f, out_f)
    toks = np.unique(np.r_[0, 1, m // 2, m - 1, min(31, m - 1), min(32, m - 1)])
    want = orc.linear(DType.NVFP4, w, x.reshape(m, in_f)[toks].ravel(), len(toks), in_f, out_f)
    gate(y[toks], want)
    assert np.all(y[1] == 0.0)
