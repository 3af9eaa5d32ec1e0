"""Backend::compile / execute over a graph of Op::Linear: grouped decode launches, dependency
ordering and replay, checked against the CPU oracle through the C ABI."""
import numpy as np
import pytest

from infr_amd import Bindings, DType, Graph, Linear, TensorDesc, synth_normal_f32, synth_weight
from oracle import oracle as orc

pytestmark = pytest.mark.gpu


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def test_layer_shaped_plan_matches_oracle_and_replays(be):
    # A decoder layer's dependency structure at reduced width: {q,k,v}(x) -> o(q) -> {gate,up}(o)
    # -> down(gate), Q4_K except Q6_K for v and down (as Q4_K_M files mix them).
    H, KV, FF = 512, 256, 1536
    spec = [("q", DType.Q4K, H, H, "x"), ("k", DType.Q4K, KV, H, "x"), ("v", DType.Q6K, KV, H, "x"),
            ("o", DType.Q4K, H, H, "q"), ("gate", DType.Q4K, FF, H, "o"), ("up", DType.Q4K, FF, H, "o"),
            ("down", DType.Q6K, H, FF, "gate")]
    g, binds = Graph(), Bindings()
    tid = {"x": g.input(TensorDesc((1, H), DType.F32))}
    xb = be.alloc(H * 4)
    binds.bind(tid["x"], xb)
    weights, outs = {}, {}
    for i, (name, dt, out_f, in_f, src) in enumerate(spec):
        w = synth_weight(dt, 40 + i, out_f, in_f)
        weights[name] = w
        wid = g.weight(TensorDesc((out_f, in_f), dt))
        binds.bind(wid, be.upload_new(w))
        tid[name] = g.output(TensorDesc((1, out_f), DType.F32))
        outs[name] = be.alloc(out_f * 4)
        binds.bind(tid[name], outs[name])
        g.push(Linear(tid[src], wid, tid[name], 1, in_f, out_f))
    plan = be.compile(g)
    for rep in range(3):  # first execute records, the others replay with new input contents
        x = synth_normal_f32(900 + rep, H)
        be.upload(xb, x)
        be.execute(plan, binds)
        want = {"x": x}
        for name, dt, out_f, in_f, src in spec:
            want[name] = orc.linear(dt, weights[name], want[src], 1, in_f, out_f).ravel()
            got = be.download(outs[name], np.empty(out_f, np.float32))
            assert np.array_equal(bits(got), bits(want[name])), f"{name} differs on execute {rep}"


def test_independent_ops_of_mixed_formats_share_launches(be):
    in_f = 1024
    g, binds = Graph(), Bindings()
    xid = g.input(TensorDesc((1, in_f), DType.F32))
    x = synth_normal_f32(5, in_f)
    binds.bind(xid, be.upload_new(x))
    cases = []
    for i, (dt, out_f) in enumerate([(DType.Q4K, 40), (DType.Q8_0, 33), (DType.Q4K, 7), (DType.Q2_0, 64),
                                     (DType.Q6K, 129), (DType.Q4K, 300), (DType.Q2_0, 5)]):
        w = synth_weight(dt, 70 + i, out_f, in_f)
        wid = g.weight(TensorDesc((out_f, in_f), dt))
        yid = g.output(TensorDesc((1, out_f), DType.F32))
        yb = be.alloc(out_f * 4)
        binds.bind(wid, be.upload_new(w)).bind(yid, yb)
        g.push(Linear(xid, wid, yid, 1, in_f, out_f))
        cases.append((dt, out_f, w, yb))
    plan = be.compile(g)
    be.execute(plan, binds)
    be.execute(plan, binds)
    for dt, out_f, w, yb in cases:
        got = be.download(yb, np.empty(out_f, np.float32))
        want = orc.linear(dt, w, x, 1, in_f, out_f).ravel()
        if dt in (DType.Q4K, DType.Q6K):
            assert np.array_equal(bits(got), bits(want))
        else:
            assert np.linalg.norm(got - want) <= 1e-4 * np.linalg.norm(want)


def test_in_place_chain_is_ordered(be):
    # Two ops writing the same dst and a reader in between: levels must follow program order.
    in_f = 256
    g, binds = Graph(), Bindings()
    xid = g.input(TensorDesc((1, in_f), DType.F32))
    yid = g.output(TensorDesc((1, in_f), DType.F32))
    zid = g.output(TensorDesc((1, in_f), DType.F32))
    x = synth_normal_f32(1, in_f)
    wa, wb_, wc = (synth_weight(DType.Q4K, s, in_f, in_f, sigma=0.05) for s in (1, 2, 3))
    ids = [g.weight(TensorDesc((in_f, in_f), DType.Q4K)) for _ in range(3)]
    yb, zb = be.alloc(in_f * 4), be.alloc(in_f * 4)
    binds.bind(xid, be.upload_new(x)).bind(yid, yb).bind(zid, zb)
    for i, w in zip(ids, (wa, wb_, wc)):
        binds.bind(i, be.upload_new(w))
    g.push(Linear(xid, ids[0], yid, 1, in_f, in_f))   # y = A x
    g.push(Linear(yid, ids[1], zid, 1, in_f, in_f))   # z = B y
    g.push(Linear(xid, ids[2], yid, 1, in_f, in_f))   # y = C x  (must wait for the read of y)
    plan = be.compile(g)
    be.execute(plan, binds)
    y1 = orc.linear(DType.Q4K, wa, x, 1, in_f, in_f).ravel()
    z = orc.linear(DType.Q4K, wb_, y1, 1, in_f, in_f).ravel()
    y2 = orc.linear(DType.Q4K, wc, x, 1, in_f, in_f).ravel()
    assert np.array_equal(bits(be.download(zb, np.empty(in_f, np.float32))), bits(z))
    assert np.array_equal(bits(be.download(yb, np.empty(in_f, np.float32))), bits(y2))


@pytest.mark.parametrize("m", [2, 5, 8, 19])
def test_small_batch_ops_run_as_groups(be, m):
    """m = 2..32 inside a plan: ops of a level that share (dtype, in_f, m) become one quantize
    launch over the distinct activation tensors plus one GEMM launch over a tile table. q/k/v
    share x, a second level consumes the first, and every replay is checked against the oracle."""
    H, KV, FF = 512, 256, 1024
    fmts = [DType.Q4K] if m > 8 else [DType.Q4K, DType.Q6K, DType.Q8_0, DType.Q2_0]
    for dt in fmts:
        spec = [("q", dt, H, H, "x"), ("k", dt, KV, H, "x"), ("v", dt, KV + 40, H, "x2"),
                ("o", dt, H, H, "q"), ("up", dt, FF, H, "q"), ("down", dt, 200, FF, "up")]
        g, binds = Graph(), Bindings()
        tid, bufs = {}, {}
        for name in ("x", "x2"):
            tid[name] = g.input(TensorDesc((m, H), DType.F32))
            bufs[name] = be.alloc(m * H * 4)
            binds.bind(tid[name], bufs[name])
        weights = {}
        for i, (name, d, out_f, in_f, src) in enumerate(spec):
            weights[name] = synth_weight(d, 60 + i, out_f, in_f, 0.05)
            wid = g.weight(TensorDesc((out_f, in_f), d))
            binds.bind(wid, be.upload_new(weights[name]))
            tid[name] = g.output(TensorDesc((m, out_f), DType.F32))
            bufs[name] = be.alloc(m * out_f * 4)
            binds.bind(tid[name], bufs[name])
            g.push(Linear(tid[src], wid, tid[name], m, in_f, out_f))
        plan = be.compile(g)
        for rep in range(2):
            want = {"x": synth_normal_f32(700 + rep, m * H), "x2": synth_normal_f32(710 + rep, m * H)}
            be.upload(bufs["x"], want["x"])
            be.upload(bufs["x2"], want["x2"])
            be.execute(plan, binds)
            assert plan.launches() == 6, plan.launches()  # three levels x (quantize + GEMM)
            for name, d, out_f, in_f, src in spec:
                got = be.download(bufs[name], np.empty((m, out_f), np.float32))
                # each op is checked on the device's own input, so one op's rounding does not leak
                src_dev = want[src] if src in want else be.download(bufs[src], np.empty(m * in_f, np.float32))
                ref = orc.linear(d, weights[name], src_dev, m, in_f, out_f)
                if d in (DType.Q4K, DType.Q6K):
                    assert np.array_equal(bits(got), bits(ref)), f"{name} {d} differs on execute {rep}"
                else:
                    a, b = got.astype(np.float64).ravel(), ref.astype(np.float64).ravel()
                    assert np.linalg.norm(a - b) <= 1e-4 * np.linalg.norm(b), f"{name} {d}"
