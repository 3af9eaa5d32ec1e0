"""Op::Linear over unquantized weight rows - F32, F16, BF16 - against the CPU oracle, through the C
ABI. infr-cpu multiplies such rows with dot / dot_f16 / dot_bf16
(crates/infr-cpu/src/lib.rs:1162-1164, 1443-1462; kernels.rs:6505-6573): every weight widened
exactly, eight FMA chains over the columns i mod 8, the chains added in order. The device runs the
same chains (the MoE router's kernels), so every output must equal the oracle's bit for bit at
every token count."""
import numpy as np
import pytest

from infr_amd import Bindings, DType, Graph, InfrError, Linear, Status, TensorDesc, synth_normal_f32, synth_weight
from oracle import oracle as orc

pytestmark = pytest.mark.gpu

PLAIN = [DType.F32, DType.F16, DType.BF16]
ids = lambda d: DType(d).name


def plain_rows(dtype, seed, n, sigma=0.05):
    w = synth_normal_f32(seed, n, sigma=sigma)
    if dtype == DType.F16:
        return w.astype(np.float16).view(np.uint8)
    if dtype == DType.BF16:
        return (w.view(np.uint32) >> 16).astype(np.uint16).view(np.uint8)
    return w.view(np.uint8)


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


@pytest.mark.parametrize("dtype", PLAIN, ids=ids)
@pytest.mark.parametrize("m", [1, 2, 5, 40, 300])
@pytest.mark.parametrize("in_f,out_f", [(512, 100), (4096, 130), (96, 7), (10240, 33)])
def test_plain_rows_are_bit_identical_to_the_oracle(be, dtype, m, in_f, out_f):
    w = plain_rows(dtype, 0x900 + in_f, out_f * in_f)
    x = synth_normal_f32(0x901 + m, m * in_f)
    yb = be.alloc(m * out_f * 4)
    be.linear(dtype, be.upload_new(w), be.upload_new(x), yb, m, in_f, out_f)
    got = be.download(yb, np.empty((m, out_f), np.float32))
    want = orc.linear(dtype, w, x, m, in_f, out_f).reshape(m, out_f)
    assert np.abs(want).max() > 1e-3
    assert np.array_equal(bits(got), bits(want))


@pytest.mark.parametrize("dtype", PLAIN, ids=ids)
def test_row_window_in_place_and_without_allocating(be, dtype):
    # rows 5 .. 1028 of a taller matrix, y written over x, through both entry points
    n, before, after = 1024, 5, 3
    w = plain_rows(dtype, 0x910, (before + n + after) * n)
    x = synth_normal_f32(0x911, n)
    want = orc.linear(dtype, w, x, 1, n, n, w_numel=(before + n + after) * n, w_off=before * n).ravel()
    wb = be.upload_new(w)
    for call in (be.linear, be.linear_noalloc):
        xb = be.upload_new(x)
        call(dtype, wb, xb, xb, 1, n, n, w_numel=(before + n + after) * n, w_off=before * n)
        assert np.array_equal(bits(be.download(xb, np.empty(n, np.float32))), bits(want))


def test_plain_rows_inside_a_plan_beside_quantized_ones(be):
    # h = W16 x (F16); y = Wq h (Q4_K, one token: a decode GEMV group); z = W32 h (F32)
    n = 512
    g, binds = Graph(), Bindings()
    xid = g.input(TensorDesc((1, n), DType.F32))
    hid, yid, zid = (g.output(TensorDesc((1, n), DType.F32)) for _ in range(3))
    w16, wq, w32 = plain_rows(DType.F16, 0x920, n * n), synth_weight(DType.Q4K, 0x921, n, n, 0.05), plain_rows(DType.F32, 0x922, n * n)
    ids_ = [g.weight(TensorDesc((n, n), d)) for d in (DType.F16, DType.Q4K, DType.F32)]
    x = synth_normal_f32(0x923, n)
    bufs = {t: be.alloc(n * 4) for t in (hid, yid, zid)}
    binds.bind(xid, be.upload_new(x))
    for t, b in bufs.items():
        binds.bind(t, b)
    for t, w in zip(ids_, (w16, wq, w32)):
        binds.bind(t, be.upload_new(w))
    g.push(Linear(xid, ids_[0], hid, 1, n, n))
    g.push(Linear(hid, ids_[1], yid, 1, n, n))
    g.push(Linear(hid, ids_[2], zid, 1, n, n))
    plan = be.compile(g)
    for _ in range(2):
        be.execute(plan, binds)
        h = orc.linear(DType.F16, w16, x, 1, n, n).ravel()
        assert np.array_equal(bits(be.download(bufs[hid], np.empty(n, np.float32))), bits(h))
        assert np.array_equal(bits(be.download(bufs[yid], np.empty(n, np.float32))), bits(orc.linear(DType.Q4K, wq, h, 1, n, n).ravel()))
        assert np.array_equal(bits(be.download(bufs[zid], np.empty(n, np.float32))), bits(orc.linear(DType.F32, w32, h, 1, n, n).ravel()))


def test_rows_that_are_not_whole_32s_are_refused(be):
    w = plain_rows(DType.F32, 0x930, 8 * 40)
    with pytest.raises(InfrError) as e:
        be.linear(DType.F32, be.upload_new(w), be.upload_new(synth_normal_f32(1, 40)), be.alloc(32), 1, 40, 8)
    assert e.value.status == Status.Unsupported
