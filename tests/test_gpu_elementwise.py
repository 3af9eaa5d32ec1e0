"""GPU parity of the ops either side of a Linear (RmsNorm, RmsNormAdd, GatedAct, GatedActFused, Add)
against the CPU oracle, through compile / execute of the C ABI.

Add is bit-exact. The gated activations use the device's expf / tanhf (last-bit differences from
the host libm) and RmsNorm sums the squares as a tree rather than in index order: both are gated
at 2e-6 relative to the row's largest output, two orders inside the path's 1e-4 bar."""
import numpy as np
import pytest

from infr_amd import (Activation, Add, Bindings, DType, GatedAct, GatedActFused, Graph, RmsNorm, RmsNormAdd,
                      TensorDesc, synth_normal_f32)
from oracle import oracle as orc

pytestmark = pytest.mark.gpu


def close(got, want, tol=2e-6):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    assert np.abs(want).max() > 1e-3
    assert np.abs(got - want).max() <= tol * np.abs(want).max(), np.abs(got - want).max() / np.abs(want).max()


def run_one(be, op_factory, inputs, out_shape):
    """inputs: list of (array, kind) with kind 'input'/'weight'; op_factory(ids..., dst_id) -> op."""
    g, binds = Graph(), Bindings()
    ids = []
    for arr in inputs:
        t = g.input(TensorDesc(arr.shape, DType.F32))
        binds.bind(t, be.upload_new(np.ascontiguousarray(arr, np.float32)))
        ids.append(t)
    dst = g.output(TensorDesc(out_shape, DType.F32))
    ob = be.alloc(int(np.prod(out_shape)) * 4)
    binds.bind(dst, ob)
    g.push(op_factory(*ids, dst))
    be.execute(be.compile(g), binds)
    return be.download(ob, np.empty(out_shape, np.float32))


@pytest.mark.parametrize("rows,dim", [(1, 4096), (3, 1000), (16, 2048), (1, 12288)])
def test_rms_norm(be, rows, dim):
    x = synth_normal_f32(1 + dim, rows * dim).reshape(rows, dim) * np.float32(3.0)
    w = (synth_normal_f32(2, dim) * np.float32(0.1) + np.float32(1.0))
    got = run_one(be, lambda xi, wi, d: RmsNorm(xi, wi, d, rows, dim, 1e-6), [x, w], (rows, dim))
    close(got, orc.rms_norm(x, w, rows, dim, 1e-6))


def test_rms_norm_add_accumulates_in_place(be):
    rows, dim = 4, 1536
    x = synth_normal_f32(3, rows * dim).reshape(rows, dim)
    w = synth_normal_f32(4, dim) + np.float32(1.0)
    base = synth_normal_f32(5, rows * dim).reshape(rows, dim)
    g, binds = Graph(), Bindings()
    xi, wi = g.input(TensorDesc(x.shape, DType.F32)), g.input(TensorDesc(w.shape, DType.F32))
    di = g.output(TensorDesc(base.shape, DType.F32))
    db = be.upload_new(base)
    binds.bind(xi, be.upload_new(x)).bind(wi, be.upload_new(w)).bind(di, db)
    g.push(RmsNormAdd(xi, wi, di, rows, dim, 1e-5))
    be.execute(be.compile(g), binds)
    close(be.download(db, np.empty(base.shape, np.float32)), orc.rms_norm(x, w, rows, dim, 1e-5, into=base))


@pytest.mark.parametrize("act", [Activation.Silu, Activation.Gelu, Activation.Sigmoid])
@pytest.mark.parametrize("clamp", [None, 1.5])
def test_gated_act(be, act, clamp):
    if clamp is not None and act == Activation.Sigmoid:
        pytest.skip("the reference refuses a clamped sigmoid (lib.rs:1903-1907)")
    rows, nff = 5, 768
    gt = synth_normal_f32(6, rows * nff).reshape(rows, nff) * np.float32(2.5)
    up = synth_normal_f32(7, rows * nff).reshape(rows, nff) * np.float32(2.5)
    got = run_one(be, lambda gi, ui, d: GatedAct(gi, ui, d, rows, nff, act, swiglu_clamp=clamp), [gt, up], (rows, nff))
    close(got, orc.gated_act(gt, up, rows, nff, int(act), clamp=clamp))
    gu = np.concatenate([gt, up], axis=1)
    got = run_one(be, lambda gi, d: GatedActFused(gi, d, rows, nff, act, swiglu_clamp=clamp), [gu], (rows, nff))
    close(got, orc.gated_act_fused(gu, rows, nff, int(act), clamp=clamp))


def test_gated_act_strided_and_interleaved_layouts(be):
    rows, nff, hd = 3, 256, 64
    gt = synth_normal_f32(8, rows * nff).reshape(rows, nff)
    up = synth_normal_f32(9, rows * nff).reshape(rows, nff)
    wide = synth_normal_f32(10, rows * 700).reshape(rows, 700)
    wide[:, 33:33 + nff] = up
    inter = np.full((rows, 2 * nff), 7.0, np.float32)
    for h in range(nff // hd):
        inter[:, h * 2 * hd + hd:(h + 1) * 2 * hd] = gt[:, h * hd:(h + 1) * hd]
    want = orc.gated_act(gt, up, rows, nff)
    got = run_one(be, lambda gi, ui, d: GatedAct(gi, ui, d, rows, nff, up_off=33, up_stride=700), [gt, wide], (rows, nff))
    close(got, want)
    got = run_one(be, lambda gi, ui, d: GatedAct(gi, ui, d, rows, nff, gate_stride=2 * nff, gate_block_width=2 * hd),
                  [inter, up], (rows, nff))
    close(got, want)


def test_add_is_bit_exact_and_in_place(be):
    n = 5000
    a, b = synth_normal_f32(11, n), synth_normal_f32(12, n) * np.float32(1e-3)
    got = run_one(be, lambda ai, bi, d: Add(ai, bi, d, n), [a, b], (n,))
    assert np.array_equal(got.view(np.uint32), orc.add(a, b).view(np.uint32))
    g, binds = Graph(), Bindings()
    ai, bi = g.input(TensorDesc((n,), DType.F32)), g.input(TensorDesc((n,), DType.F32))
    ab = be.upload_new(a)
    binds.bind(ai, ab).bind(bi, be.upload_new(b))
    g.push(Add(ai, bi, ai, n))
    g.push(Add(ai, bi, ai, n))  # ordered after the first: reads what it wrote
    be.execute(be.compile(g), binds)
    want = orc.add(orc.add(a, b), b)
    assert np.array_equal(be.download(ab, np.empty(n, np.float32)).view(np.uint32), want.view(np.uint32))


def test_shape_and_binding_errors(be):
    from infr_amd import InfrError
    g, binds = Graph(), Bindings()
    xi = g.input(TensorDesc((4, 64), DType.F32))
    wi = g.input(TensorDesc((64,), DType.F32))
    di = g.output(TensorDesc((4, 64), DType.F32))
    g.push(RmsNorm(xi, wi, di, 4, 64, 1e-6))
    plan = be.compile(g)
    binds.bind(xi, be.alloc(4 * 64 * 4)).bind(wi, be.alloc(64 * 4)).bind(di, be.alloc(100))  # dst too small
    with pytest.raises(InfrError):
        be.execute(plan, binds)
    g2 = Graph()
    a = g2.input(TensorDesc((8,), DType.F32))
    g2.push(GatedActFused(a, a, 1, 4, Activation.Sigmoid, swiglu_clamp=1.0))
    with pytest.raises(InfrError):
        be.compile(g2)


def test_measurement_probes_report_sane_rates(be):
    """The two measurement aids (no counterpart in the reference): a register-only int8 MFMA loop and
    a read-only streaming pass. Both must finish and report a positive rate below the published peaks
    (5 POP/s int8, 8 TB/s); bad arguments are refused."""
    from infr_amd import InfrError
    for random_data in (False, True):
        tops = be.mfma_i8_peak_tops(2, 256, random_data)
        assert 10.0 < tops < 5200.0, tops
    with pytest.raises(InfrError):
        be.mfma_i8_peak_tops(0, 256, True)
    with pytest.raises(InfrError):
        be.mfma_i8_peak_tops(2, 0, True)
    buf = be.alloc(64 << 20)
    for nt in (False, True):
        gbs = be.stream_read_gbs(buf, reps=3, nontemporal=nt)
        assert 100.0 < gbs < 8200.0, (nt, gbs)
    buf.free()
