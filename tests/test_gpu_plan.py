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


@pytest.mark.parametrize("dtype", [DType.Q4K, DType.Q8_0])
@pytest.mark.parametrize("y_first", [True, False])
def test_add_in_place_on_the_linear_output_is_absorbed(be, dtype, y_first):
    # y = W x; y = y + r: the absorbed Add's dst is the Linear's own dst, which then holds the sum
    from infr_amd import Add
    n = 1024
    g, binds = Graph(), Bindings()
    xid, rid = (g.input(TensorDesc((1, n), DType.F32)) for _ in range(2))
    yid = g.output(TensorDesc((1, n), DType.F32))
    wid = g.weight(TensorDesc((n, n), dtype))
    x, r = synth_normal_f32(0x71, n), synth_normal_f32(0x72, n)
    w = synth_weight(dtype, 0x73, n, n, sigma=0.03)
    yb = be.alloc(n * 4)
    binds.bind(xid, be.upload_new(x)).bind(rid, be.upload_new(r)).bind(yid, yb).bind(wid, be.upload_new(w))
    g.push(Linear(xid, wid, yid, 1, n, n))
    g.push(Add(yid, rid, yid, n) if y_first else Add(rid, yid, yid, n))
    plan = be.compile(g)
    for _ in range(2):
        be.execute(plan, binds)
        got = be.download(yb, np.empty(n, np.float32))
        want = orc.linear(dtype, w, x, 1, n, n).ravel() + r
        assert plan.launches() == 1
        if dtype == DType.Q4K:
            assert np.array_equal(bits(got), bits(want))
        else:
            assert _rel(got, want) < 1e-5


def test_one_row_linear_in_place_inside_a_plan(be):
    # y = A y next to a sibling z = B y that reads the old y first (program order), then y = C y
    # again: the in-place ops must neither join a group nor overtake the reader.
    n = 2048
    g, binds = Graph(), Bindings()
    yid = g.output(TensorDesc((1, n), DType.F32))
    zid = g.output(TensorDesc((1, n), DType.F32))
    y0 = synth_normal_f32(0x61, n)
    ws = [synth_weight(DType.Q4K, s, n, n, sigma=0.03) for s in (0x62, 0x63, 0x64)]
    ids = [g.weight(TensorDesc((n, n), DType.Q4K)) for _ in ws]
    yb, zb = be.upload_new(y0), be.alloc(n * 4)
    binds.bind(yid, yb).bind(zid, zb)
    for i, w in zip(ids, ws):
        binds.bind(i, be.upload_new(w))
    g.push(Linear(yid, ids[0], zid, 1, n, n))   # z = B y0
    g.push(Linear(yid, ids[1], yid, 1, n, n))   # y = A y0   (in place)
    g.push(Linear(yid, ids[2], yid, 1, n, n))   # y = C y    (in place again)
    plan = be.compile(g)
    be.execute(plan, binds)
    z = orc.linear(DType.Q4K, ws[0], y0, 1, n, n).ravel()
    y1 = orc.linear(DType.Q4K, ws[1], y0, 1, n, n).ravel()
    y2 = orc.linear(DType.Q4K, ws[2], y1, 1, n, n).ravel()
    assert np.array_equal(bits(be.download(zb, np.empty(n, np.float32))), bits(z))
    assert np.array_equal(bits(be.download(yb, np.empty(n, np.float32))), bits(y2))


@pytest.mark.parametrize("m", [2, 5, 8, 12, 16, 19])
def test_small_batch_ops_run_as_groups(be, m):
    """m = 2..32 inside a plan: ops of a level that share (dtype, in_f, m) become one quantize
    launch over the distinct activation tensors plus one GEMM launch over a tile table. q/k/v
    share x, a second level consumes the first, and every replay is checked against the oracle."""
    H, KV, FF = 512, 256, 1024
    fmts = ([DType.Q4K] if m > 16 else [DType.Q4K, DType.Q5K, DType.Q6K]) if m > 8 else [DType.Q4K, DType.Q5K, DType.Q6K, DType.Q8_0, DType.Q2_0]
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
                if d in (DType.Q4K, DType.Q5K, DType.Q6K):
                    assert np.array_equal(bits(got), bits(ref)), f"{name} {d} differs on execute {rep}"
                else:
                    a, b = got.astype(np.float64).ravel(), ref.astype(np.float64).ravel()
                    assert np.linalg.norm(a - b) <= 1e-4 * np.linalg.norm(b), f"{name} {d}"


def _rel(a, b):
    a, b = np.asarray(a, np.float64).ravel(), np.asarray(b, np.float64).ravel()
    return np.linalg.norm(a - b) / np.linalg.norm(b)


@pytest.mark.parametrize("combined_gu", [False, True])
def test_decoder_layer_without_attention_fuses_into_four_launches(be, combined_gu):
    """RmsNorm -> {q, k, v}; o(q) -> Add; RmsNorm -> gate/up -> GatedAct -> down -> Add at m = 1.
    The norms, the gated activation and the residual adds are absorbed by the decode GEMVs: four
    launches instead of nine, every intermediate tensor still written, each stage within the
    path's 1e-4 of the oracle fed with the device's own upstream tensors."""
    from infr_amd import Add, GatedAct, GatedActFused, RmsNorm
    H, KV, FF = 1024, 256, 2816
    rng_w = lambda seed, n: synth_normal_f32(seed, n) * np.float32(0.1) + np.float32(1.0)
    g, binds, bufs, host = Graph(), Bindings(), {}, {}

    def tensor(name, shape, data=None, kind="input"):
        t = (g.input if kind == "input" else g.output)(TensorDesc(shape, DType.F32))
        n = int(np.prod(shape))
        bufs[name] = be.upload_new(data) if data is not None else be.alloc(n * 4)
        host[name] = data
        binds.bind(t, bufs[name])
        return t

    def weight(name, dt, out_f, in_f, seed):
        host[name] = synth_weight(dt, seed, out_f, in_f, 0.05)
        t = g.weight(TensorDesc((out_f, in_f), dt))
        binds.bind(t, be.upload_new(host[name]))
        return t

    x = tensor("x", (1, H))
    n1w, n2w = tensor("n1w", (H,), rng_w(1, H)), tensor("n2w", (H,), rng_w(2, H))
    h1, q, k, v, o = (tensor(nm, (1, d), kind="output") for nm, d in
                      [("h1", H), ("q", H), ("k", KV), ("v", KV), ("o", H)])
    h2, act, down = tensor("h2", (1, H), kind="output"), tensor("act", (1, FF), kind="output"), tensor("down", (1, H), kind="output")
    wq, wk, wv = weight("wq", DType.Q4K, H, H, 11), weight("wk", DType.Q4K, KV, H, 12), weight("wv", DType.Q6K, KV, H, 13)
    wo, wd = weight("wo", DType.Q4K, H, H, 14), weight("wd", DType.Q6K, H, FF, 15)
    g.push(RmsNorm(x, n1w, h1, 1, H, 1e-6))
    g.push(Linear(h1, wq, q, 1, H, H))
    g.push(Linear(h1, wk, k, 1, H, KV))
    g.push(Linear(h1, wv, v, 1, H, KV))
    g.push(Linear(q, wo, o, 1, H, H))
    g.push(Add(o, x, x, H))                      # residual in place: x = o + x
    g.push(RmsNorm(x, n2w, h2, 1, H, 1e-6))
    if combined_gu:
        wgu = weight("wgu", DType.Q4K, 2 * FF, H, 16)
        gu = tensor("gu", (1, 2 * FF), kind="output")
        g.push(Linear(h2, wgu, gu, 1, H, 2 * FF))
        g.push(GatedActFused(gu, act, 1, FF))
    else:
        wg, wu = weight("wg", DType.Q4K, FF, H, 16), weight("wu", DType.Q4K, FF, H, 17)
        gt, up = tensor("gate", (1, FF), kind="output"), tensor("up", (1, FF), kind="output")
        g.push(Linear(h2, wg, gt, 1, H, FF))
        g.push(Linear(h2, wu, up, 1, H, FF))
        g.push(GatedAct(gt, up, act, 1, FF))
    g.push(Linear(act, wd, down, 1, FF, H))
    g.push(Add(down, x, x, H))
    plan = be.compile(g)
    get = lambda nm, n: be.download(bufs[nm], np.empty(n, np.float32))
    for rep in range(3):
        x0 = synth_normal_f32(800 + rep, H)
        be.upload(bufs["x"], x0)
        be.execute(plan, binds)
        # q/k (Q4_K) and v (Q6_K) are separate launches; o; gate/up; down -> 5 groups here
        assert plan.launches() == 5, plan.launches()
        d = {nm: get(nm, n) for nm, n in [("h1", H), ("q", H), ("k", KV), ("v", KV), ("o", H), ("h2", H),
                                          ("act", FF), ("down", H), ("x", H)]}
        assert _rel(d["h1"], orc.rms_norm(x0, host["n1w"], 1, H, 1e-6)) < 1e-6
        assert _rel(d["q"], orc.linear(DType.Q4K, host["wq"], d["h1"], 1, H, H)) < 1e-4
        assert _rel(d["k"], orc.linear(DType.Q4K, host["wk"], d["h1"], 1, H, KV)) < 1e-4
        assert _rel(d["v"], orc.linear(DType.Q6K, host["wv"], d["h1"], 1, H, KV)) < 1e-4
        o_want = orc.linear(DType.Q4K, host["wo"], d["q"], 1, H, H).ravel()
        assert np.array_equal(bits(d["o"]), bits(o_want))      # no absorbed producer: bit-identical
        x1 = orc.add(d["o"], x0)
        assert _rel(d["h2"], orc.rms_norm(x1, host["n2w"], 1, H, 1e-6)) < 1e-6
        if combined_gu:
            gu_d = get("gu", 2 * FF)
            assert _rel(gu_d, orc.linear(DType.Q4K, host["wgu"], d["h2"], 1, H, 2 * FF)) < 1e-4
            act_want = orc.gated_act_fused(gu_d, 1, FF)
        else:
            g_d, u_d = get("gate", FF), get("up", FF)
            assert _rel(g_d, orc.linear(DType.Q4K, host["wg"], d["h2"], 1, H, FF)) < 1e-4
            assert _rel(u_d, orc.linear(DType.Q4K, host["wu"], d["h2"], 1, H, FF)) < 1e-4
            act_want = orc.gated_act(g_d, u_d, 1, FF)
        assert _rel(d["act"], act_want) < 1e-6
        assert _rel(d["down"], orc.linear(DType.Q6K, host["wd"], d["act"], 1, FF, H)) < 1e-4
        assert np.array_equal(bits(d["x"]), bits(orc.add(d["down"], x1)))   # both adds are exact


def test_fusion_is_refused_when_it_would_reorder_a_dependency(be):
    """A reader of the norm's output that is not a decode Linear, and a writer of the residual
    between a Linear and its Add, both keep the ops separate; results follow program order."""
    from infr_amd import Add, RmsNorm
    H = 512
    g, binds = Graph(), Bindings()
    ids = {}
    for nm in ("x", "w", "h", "h_copy", "y", "r", "zero"):
        ids[nm] = g.input(TensorDesc((H,), DType.F32))
    wq = g.weight(TensorDesc((H, H), DType.Q4K))
    w_host = synth_weight(DType.Q4K, 5, H, H, 0.05)
    x0, nw = synth_normal_f32(1, H), synth_normal_f32(2, H) + np.float32(1.0)
    r0 = synth_normal_f32(3, H)
    b = {"x": be.upload_new(x0), "w": be.upload_new(nw), "h": be.alloc(H * 4), "h_copy": be.alloc(H * 4),
         "y": be.alloc(H * 4), "r": be.upload_new(r0), "zero": be.alloc(H * 4)}
    for nm, buf in b.items():
        binds.bind(ids[nm], buf)
    binds.bind(wq, be.upload_new(w_host))
    g.push(RmsNorm(ids["x"], ids["w"], ids["h"], 1, H, 1e-6))
    g.push(Add(ids["h"], ids["zero"], ids["h_copy"], H))       # a non-Linear reader of h: no absorption
    g.push(Linear(ids["h"], wq, ids["y"], 1, H, H))
    g.push(Add(ids["r"], ids["r"], ids["r"], H))               # r *= 2 between the Linear and its Add
    g.push(Add(ids["y"], ids["r"], ids["r"], H))               # must see the doubled r
    plan = be.compile(g)
    be.execute(plan, binds)
    assert plan.launches() == 5
    h = be.download(b["h"], np.empty(H, np.float32))
    assert np.array_equal(bits(be.download(b["h_copy"], np.empty(H, np.float32))), bits(h))
    y = be.download(b["y"], np.empty(H, np.float32))
    assert np.array_equal(bits(y), bits(orc.linear(DType.Q4K, w_host, h, 1, H, H).ravel()))
    want_r = orc.add(y, orc.add(r0, r0))
    assert np.array_equal(bits(be.download(b["r"], np.empty(H, np.float32))), bits(want_r))


def test_in_place_producers_are_not_absorbed(be):
    """The runner emits in-place producers at decode (GatedAct{gate: g, dst: g} followed by
    Linear{x: g}, crates/infr-llama/src/seam/runner.rs:4305-4326). Every workgroup of an
    absorbing GEMV would re-read the producer's input while the first one overwrites it, so such
    producers run as their own launch: outputs equal the oracle's on the first execute and on replays."""
    from infr_amd import Activation, GatedAct, RmsNorm
    H, KV, FF = 1024, 256, 4096
    g, binds = Graph(), Bindings()
    x, nw = g.input(TensorDesc((1, H), DType.F32)), g.input(TensorDesc((H,), DType.F32))
    gate, up = g.input(TensorDesc((1, FF), DType.F32)), g.input(TensorDesc((1, FF), DType.F32))
    xb, gb = be.alloc(H * 4), be.alloc(FF * 4)
    nw_h = synth_normal_f32(2, H) * np.float32(0.1) + np.float32(1.0)
    up_h = synth_normal_f32(3, FF)
    binds.bind(x, xb).bind(nw, be.upload_new(nw_h)).bind(gate, gb).bind(up, be.upload_new(up_h))
    ws, outs = {}, {}
    for nm, dt, out_f, in_f in [("q", DType.Q4K, H, H), ("k", DType.Q4K, KV, H), ("v", DType.Q6K, KV, H),
                                ("down", DType.Q4K, 3072, FF)]:
        ws[nm] = synth_weight(dt, 20 + len(ws), out_f, in_f, 0.05)
        wid = g.weight(TensorDesc((out_f, in_f), dt))
        oid = g.output(TensorDesc((1, out_f), DType.F32))
        outs[nm] = (dt, out_f, in_f, be.alloc(out_f * 4))
        binds.bind(wid, be.upload_new(ws[nm])).bind(oid, outs[nm][3])
        outs[nm] += (wid, oid)
    g.push(RmsNorm(x, nw, x, 1, H, 1e-6))                       # in place: x = rmsnorm(x) * w
    for nm in ("q", "k", "v"):
        g.push(Linear(x, outs[nm][4], outs[nm][5], 1, H, outs[nm][1]))
    g.push(GatedAct(gate, up, gate, 1, FF, act=int(Activation.Gelu)))   # in place: gate = gelu(gate) * up
    g.push(Linear(gate, outs["down"][4], outs["down"][5], 1, FF, 3072))  # 3072 rows: many workgroups
    plan = be.compile(g)
    for rep in range(3):
        x0, g0 = synth_normal_f32(40 + rep, H), synth_normal_f32(50 + rep, FF)
        be.upload(xb, x0)
        be.upload(gb, g0)
        be.execute(plan, binds)
        assert plan.launches() == 5, plan.launches()             # norm, {q, k}, v, act, down
        h = be.download(xb, np.empty(H, np.float32))
        a = be.download(gb, np.empty(FF, np.float32))
        assert _rel(h, orc.rms_norm(x0, nw_h, 1, H, 1e-6)) < 2e-6
        assert _rel(a, orc.gated_act(g0, up_h, 1, FF, int(Activation.Gelu))) < 2e-6
        for nm, src in (("q", h), ("k", h), ("v", h), ("down", a)):
            dt, out_f, in_f, buf = outs[nm][:4]
            got = be.download(buf, np.empty(out_f, np.float32))
            want = orc.linear(dt, ws[nm], src, 1, in_f, out_f).ravel()
            assert np.array_equal(bits(got), bits(want)), f"{nm} differs on execute {rep}"


def test_two_layers_sharing_scratch_tensors_still_fuse(be):
    """The runner reuses the norm / gate / act scratch tensors from layer to layer
    (crates/infr-core/src/graph.rs:10-14). A producer's readers are those up to the next op that
    overwrites its dst, so each layer's norm and gated activation are absorbed: two layers of
    norm -> {gate, up} -> act -> down -> add run in four launches, not ten."""
    from infr_amd import Add, GatedAct, RmsNorm
    H, FF, L = 512, 1536, 2
    g, binds, host = Graph(), Bindings(), {}
    x = g.input(TensorDesc((1, H), DType.F32))
    xb = be.alloc(H * 4)
    binds.bind(x, xb)
    scratch = {}
    for nm, n in (("xn", H), ("gate", FF), ("up", FF), ("act", FF), ("down", H)):
        scratch[nm] = (g.output(TensorDesc((1, n), DType.F32)), be.alloc(n * 4))
        binds.bind(*scratch[nm])
    for l in range(L):
        host[l] = {"nw": synth_normal_f32(100 + l, H) * np.float32(0.1) + np.float32(1.0)}
        nw = g.input(TensorDesc((H,), DType.F32))
        binds.bind(nw, be.upload_new(host[l]["nw"]))
        wid = {}
        for nm, out_f, in_f in (("wg", FF, H), ("wu", FF, H), ("wd", H, FF)):
            host[l][nm] = synth_weight(DType.Q4K, 110 + 10 * l + len(wid), out_f, in_f, 0.05)
            wid[nm] = g.weight(TensorDesc((out_f, in_f), DType.Q4K))
            binds.bind(wid[nm], be.upload_new(host[l][nm]))
        g.push(RmsNorm(x, nw, scratch["xn"][0], 1, H, 1e-6))
        g.push(Linear(scratch["xn"][0], wid["wg"], scratch["gate"][0], 1, H, FF))
        g.push(Linear(scratch["xn"][0], wid["wu"], scratch["up"][0], 1, H, FF))
        g.push(GatedAct(scratch["gate"][0], scratch["up"][0], scratch["act"][0], 1, FF))
        g.push(Linear(scratch["act"][0], wid["wd"], scratch["down"][0], 1, FF, H))
        g.push(Add(scratch["down"][0], x, x, H))
    plan = be.compile(g)
    for rep in range(3):
        x0 = synth_normal_f32(300 + rep, H)
        be.upload(xb, x0)
        be.execute(plan, binds)
        assert plan.launches() == 2 * L, plan.launches()
        # the oracle chain, each stage fed the previous stage's oracle value: the absorbed norm and
        # activation differ from the stand-alone ops by ~1e-7 relative, the gate is 1e-4 end to end
        xr = x0
        for l in range(L):
            xn = orc.rms_norm(xr, host[l]["nw"], 1, H, 1e-6)
            gt = orc.linear(DType.Q4K, host[l]["wg"], xn, 1, H, FF)
            up = orc.linear(DType.Q4K, host[l]["wu"], xn, 1, H, FF)
            act = orc.gated_act(gt, up, 1, FF)
            dn = orc.linear(DType.Q4K, host[l]["wd"], act, 1, FF, H)
            xr = orc.add(dn, xr)
        got = be.download(xb, np.empty(H, np.float32))
        assert _rel(got, xr) < 1e-4, _rel(got, xr)
        # the scratch tensors hold the LAST layer's values, as in program order
        assert _rel(be.download(scratch["act"][1], np.empty(FF, np.float32)), act) < 1e-4
        assert _rel(be.download(scratch["xn"][1], np.empty(H, np.float32)), xn) < 1e-4


def test_plans_survive_backend_scratch_regrowth(be):
    """A recorded plan carries the backend's scratch addresses. Compiling a plan that needs far more
    scratch reallocates it, so the first plan must be recorded again instead of replaying launches
    that point at freed memory (Internal scratch is the backend's to keep valid,
    crates/infr-core/src/backend.rs:8-13)."""
    from infr_amd import HipBackend, MoeFfn
    own = HipBackend(0)          # a backend of its own, so the scratch starts small
    try:
        ne, n_expert, n_used, nff, rows = 512, 16, 4, 256, 2
        in_f, out_f, m = 512, 384, 8
        w = synth_weight(DType.Q6K, 1, out_f, in_f, 0.05)
        router = synth_normal_f32(2, n_expert * ne, sigma=0.05)
        gate = synth_weight(DType.Q4K, 3, n_expert * nff, ne, 0.05)
        up = synth_weight(DType.Q4K, 4, n_expert * nff, ne, 0.05)
        down = synth_weight(DType.Q4K, 5, n_expert * ne, nff, 0.05)
        g, binds = Graph(), Bindings()
        x = g.input(TensorDesc((m, in_f), DType.F32))
        mx = g.input(TensorDesc((rows, ne), DType.F32))
        xb, mxb = own.alloc(m * in_f * 4), own.alloc(rows * ne * 4)
        y, my = g.output(TensorDesc((m, out_f), DType.F32)), g.output(TensorDesc((rows, ne), DType.F32))
        yb, myb = own.alloc(m * out_f * 4), own.alloc(rows * ne * 4)
        wid, rid = g.weight(TensorDesc((out_f, in_f), DType.Q6K)), g.weight(TensorDesc((n_expert, ne), DType.F32))
        gid, uid = (g.weight(TensorDesc((n_expert, nff, ne), DType.Q4K)) for _ in range(2))
        did = g.weight(TensorDesc((n_expert, ne, nff), DType.Q4K))
        binds.bind(x, xb).bind(mx, mxb).bind(y, yb).bind(my, myb).bind(wid, own.upload_new(w))
        binds.bind(rid, own.upload_new(router)).bind(gid, own.upload_new(gate)).bind(uid, own.upload_new(up))
        binds.bind(did, own.upload_new(down))
        g.push(Linear(x, wid, y, m, in_f, out_f))
        g.push(MoeFfn(mx, mx, rid, gid, uid, did, my, ne, n_expert, n_used, nff))
        plan_a = own.compile(g)

        def run_a(seed):
            x0, mx0 = synth_normal_f32(seed, m * in_f), synth_normal_f32(seed + 1, rows * ne)
            own.upload(xb, x0)
            own.upload(mxb, mx0)
            own.execute(plan_a, binds)
            got = own.download(yb, np.empty((m, out_f), np.float32))
            assert np.array_equal(bits(got), bits(orc.linear(DType.Q6K, w, x0, m, in_f, out_f)))
            want, _, _ = orc.moe_ffn(mx0, router, gate, up, down, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff)
            assert _rel(own.download(myb, np.empty((rows, ne), np.float32)), want) < 1e-4

        run_a(10)
        run_a(20)                                            # a replay
        # plan B: 600 tokens of a longer row and a 300-row MoE need far larger scratch
        gB, bB = Graph(), Bindings()
        mB, kB, nB, rB = 600, 2048, 256, 300
        wB = synth_weight(DType.Q4K, 7, nB, kB, 0.05)
        xB, yB = gB.input(TensorDesc((mB, kB), DType.F32)), gB.output(TensorDesc((mB, nB), DType.F32))
        xBh = synth_normal_f32(8, mB * kB)
        yBb = own.alloc(mB * nB * 4)
        wBid = gB.weight(TensorDesc((nB, kB), DType.Q4K))
        mxB, myB = gB.input(TensorDesc((rB, ne), DType.F32)), gB.output(TensorDesc((rB, ne), DType.F32))
        mxBh = synth_normal_f32(9, rB * ne)
        myBb = own.alloc(rB * ne * 4)
        bB.bind(xB, own.upload_new(xBh)).bind(yB, yBb).bind(wBid, own.upload_new(wB))
        bB.bind(mxB, own.upload_new(mxBh)).bind(myB, myBb)
        ids = []
        for arr, shape, dt in ((router, (n_expert, ne), DType.F32), (gate, (n_expert, nff, ne), DType.Q4K),
                               (up, (n_expert, nff, ne), DType.Q4K), (down, (n_expert, ne, nff), DType.Q4K)):
            ids.append(gB.weight(TensorDesc(shape, dt)))
            bB.bind(ids[-1], own.upload_new(arr))
        gB.push(Linear(xB, wBid, yB, mB, kB, nB))
        gB.push(MoeFfn(mxB, mxB, ids[0], ids[1], ids[2], ids[3], myB, ne, n_expert, n_used, nff))
        plan_b = own.compile(gB)
        own.execute(plan_b, bB)
        gotB = own.download(yBb, np.empty((mB, nB), np.float32))
        rows_chk = [0, 1, 31, 32, 299, 599]
        wantB = orc.linear(DType.Q4K, wB, xBh.reshape(mB, kB)[rows_chk].ravel(), len(rows_chk), kB, nB)
        assert np.array_equal(bits(gotB[rows_chk]), bits(wantB))
        run_a(30)                                            # plan A after the scratch moved
        run_a(40)
        own.execute(plan_b, bB)                              # and B again, replayed
        assert np.array_equal(bits(own.download(yBb, np.empty((mB, nB), np.float32))[rows_chk]), bits(wantB))
    finally:
        own.close()


def test_capabilities_advertise_the_ops_that_are_built(be):
    caps = be.capabilities()
    assert caps["combined_gu"] == 1 and caps["embed_gather"] == 1 and caps["decode_replay"] == 1
    assert caps["gpu_sample"] == 0 and caps["argmax_rows"] == 0 and caps["gated_rmsnorm"] == 0


@pytest.mark.parametrize("rows", [1, 3])
@pytest.mark.parametrize("resid_first", [True, False])
def test_moe_residual_add_rides_in_the_last_moe_kernel(be, rows, resid_first):
    """MoeFfn -> Add(residual) (crates/infr-core/src/fusion.rs:155-200): the Add is produced by the
    kernel that accumulates the experts, in place on the residual stream, with the un-added MoE
    output still stored; the sum is the CPU's `a + b` bit for bit."""
    from infr_amd import Add, MoeFfn
    ne, n_expert, n_used, nff = 512, 16, 4, 256
    router = synth_normal_f32(2, n_expert * ne, sigma=0.05)
    gate = synth_weight(DType.Q4K, 3, n_expert * nff, ne, 0.05)
    up = synth_weight(DType.Q4K, 4, n_expert * nff, ne, 0.05)
    down = synth_weight(DType.Q6K, 5, n_expert * ne, nff, 0.05)
    g, binds = Graph(), Bindings()
    xn = g.input(TensorDesc((rows, ne), DType.F32))
    h = g.input(TensorDesc((rows, ne), DType.F32))
    y = g.output(TensorDesc((rows, ne), DType.F32))
    xnb, hb, yb = (be.alloc(rows * ne * 4) for _ in range(3))
    rid = g.weight(TensorDesc((n_expert, ne), DType.F32))
    gid, uid = (g.weight(TensorDesc((n_expert, nff, ne), DType.Q4K)) for _ in range(2))
    did = g.weight(TensorDesc((n_expert, ne, nff), DType.Q6K))
    binds.bind(xn, xnb).bind(h, hb).bind(y, yb).bind(rid, be.upload_new(router))
    binds.bind(gid, be.upload_new(gate)).bind(uid, be.upload_new(up)).bind(did, be.upload_new(down))
    g.push(MoeFfn(xn, xn, rid, gid, uid, did, y, ne, n_expert, n_used, nff))
    g.push(Add(h, y, h, rows * ne) if resid_first else Add(y, h, h, rows * ne))
    plan = be.compile(g)
    for seed in (10, 20, 30):                               # the second and third are replays
        xn0, h0 = synth_normal_f32(seed, rows * ne), synth_normal_f32(seed + 1, rows * ne)
        be.upload(xnb, xn0)
        be.upload(hb, h0)
        be.execute(plan, binds)
        got_y = be.download(yb, np.empty(rows * ne, np.float32))
        got_h = be.download(hb, np.empty(rows * ne, np.float32))
        want, _, _ = orc.moe_ffn(xn0, router, gate, up, down, ne=ne, n_expert=n_expert, n_used=n_used,
                                 n_ff_exp=nff, down_dtype=DType.Q6K)
        assert _rel(got_y, want.ravel()) < 1e-4
        assert np.array_equal(bits(got_h), bits(h0 + got_y))
    # rows >= 2: router, selection (+ the quantizer), gate and up in one launch, activation + down + sum in one
    assert plan.launches() == (3 if rows == 1 else 4)       # no launch of its own for the Add


def test_single_row_rms_norm_rides_in_the_moe_router_kernel(be):
    """RmsNorm -> MoeFfn(rows == 1) reading the normalised row as x and router_x
    (crates/infr-core/src/fusion.rs:58-73, `moe_ok`) -> Add(residual): three launches for the whole
    sublayer. The router kernel normalises with the stand-alone kernel's own arithmetic, so the MoE
    output equals, bit for bit, that of a plan in which a second reader of the normalised row keeps
    the RmsNorm a launch of its own."""
    from infr_amd import Add, MoeFfn, RmsNorm
    ne, n_expert, n_used, nff = 1024, 16, 4, 256
    router = synth_normal_f32(2, n_expert * ne, sigma=0.05)
    gate = synth_weight(DType.Q4K, 3, n_expert * nff, ne, 0.05)
    up = synth_weight(DType.Q4K, 4, n_expert * nff, ne, 0.05)
    down = synth_weight(DType.Q4K, 5, n_expert * ne, nff, 0.05)
    nw = synth_normal_f32(6, ne, mean=1.0, sigma=0.1)
    shared = [be.upload_new(a) for a in (router, gate, up, down, nw)]

    def build(extra_reader):
        g, binds = Graph(), Bindings()
        h = g.input(TensorDesc((1, ne), DType.F32))
        xn, y, junk = (g.output(TensorDesc((1, ne), DType.F32)) for _ in range(3))
        bufs = {t: be.alloc(ne * 4) for t in (h, xn, y, junk)}
        for t, b in bufs.items():
            binds.bind(t, b)
        rid = g.weight(TensorDesc((n_expert, ne), DType.F32))
        gid, uid = (g.weight(TensorDesc((n_expert, nff, ne), DType.Q4K)) for _ in range(2))
        did = g.weight(TensorDesc((n_expert, ne, nff), DType.Q4K))
        wid = g.weight(TensorDesc((ne,), DType.F32))
        for t, b in zip((rid, gid, uid, did, wid), shared):
            binds.bind(t, b)
        g.push(RmsNorm(h, wid, xn, 1, ne, 1e-6))
        g.push(MoeFfn(xn, xn, rid, gid, uid, did, y, ne, n_expert, n_used, nff))
        g.push(Add(h, y, h, ne))
        if extra_reader:
            g.push(Add(xn, xn, junk, ne))
        return be.compile(g), binds, bufs[h], bufs[xn], bufs[y]

    fused, plain = build(False), build(True)
    for seed in (10, 20, 30):
        h0 = synth_normal_f32(seed, ne)
        outs = []
        for plan, binds, hb, xnb, yb in (fused, plain):
            be.upload(hb, h0)
            be.execute(plan, binds)
            outs.append([be.download(b, np.empty(ne, np.float32)) for b in (hb, xnb, yb)])
        for a, b in zip(*outs):
            assert np.array_equal(bits(a), bits(b))
        h1, xn1, y1 = outs[0]
        xn_ref = orc.rms_norm(h0, nw, 1, ne, 1e-6)
        assert _rel(xn1, xn_ref) < 2e-6
        want, _, _ = orc.moe_ffn(xn_ref, router, gate, up, down, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff)
        assert _rel(y1, want.ravel()) < 1e-4
        assert np.array_equal(bits(h1), bits(h0 + y1))
    assert fused[0].launches() == 3 and plain[0].launches() == 5


@pytest.mark.parametrize("m", [2, 8, 16, 24])
def test_norm_and_gated_activation_ride_in_the_small_batch_quantizer(be, m):
    """A decode batch through RmsNorm -> {q (Q4_K), v (Q6_K)} and GatedAct -> down: the norm and the
    activation are evaluated by the quantizer launches of the Linears that read them (stand-alone
    arithmetic, so the same bits), their outputs are still stored, and the plan is four launches
    shorter than one per op - two quantizers (one per weight format) compute the norm, which is
    allowed because they sit on one level."""
    from infr_amd import GatedAct, RmsNorm
    H, FF = 1024, 1536
    wq, wv = synth_weight(DType.Q4K, 1, H, H, 0.05), synth_weight(DType.Q6K, 2, 256, H, 0.05)
    wd = synth_weight(DType.Q4K, 3, H, FF, 0.05)
    nw = synth_normal_f32(4, H, mean=1.0, sigma=0.1)
    g, binds = Graph(), Bindings()
    x, gt, up = (g.input(TensorDesc((m, d), DType.F32)) for d in (H, FF, FF))
    nwid = g.input(TensorDesc((H,), DType.F32))
    h, q, v, act, dn = (g.output(TensorDesc((m, d), DType.F32)) for d in (H, H, 256, FF, H))
    bufs = {t: be.alloc(m * d * 4) for t, d in ((x, H), (gt, FF), (up, FF), (h, H), (q, H), (v, 256), (act, FF), (dn, H))}
    for t, b in bufs.items():
        binds.bind(t, b)
    binds.bind(nwid, be.upload_new(nw))
    wqid, wvid, wdid = (g.weight(TensorDesc(s, dt)) for s, dt in (((H, H), DType.Q4K), ((256, H), DType.Q6K),
                                                                 ((H, FF), DType.Q4K)))
    binds.bind(wqid, be.upload_new(wq)).bind(wvid, be.upload_new(wv)).bind(wdid, be.upload_new(wd))
    g.push(RmsNorm(x, nwid, h, m, H, 1e-6))
    g.push(Linear(h, wqid, q, m, H, H))
    g.push(Linear(h, wvid, v, m, H, 256))
    g.push(GatedAct(gt, up, act, m, FF))
    g.push(Linear(act, wdid, dn, m, FF, H))
    plan = be.compile(g)
    for seed in (10, 20):                                   # the second is a replay
        x0, g0, u0 = synth_normal_f32(seed, m * H), synth_normal_f32(seed + 1, m * FF), synth_normal_f32(seed + 2, m * FF)
        be.upload(bufs[x], x0)
        be.upload(bufs[gt], g0)
        be.upload(bufs[up], u0)
        be.execute(plan, binds)
        got_h = be.download(bufs[h], np.empty(m * H, np.float32))
        got_act = be.download(bufs[act], np.empty(m * FF, np.float32))
        # the folded ops' own outputs: the stand-alone kernels' values (each op alone in a plan)
        alone = Graph()
        ax, aw, ah = alone.input(TensorDesc((m, H), DType.F32)), alone.input(TensorDesc((H,), DType.F32)), alone.output(TensorDesc((m, H), DType.F32))
        alone.push(RmsNorm(ax, aw, ah, m, H, 1e-6))
        hb = be.alloc(m * H * 4)
        be.execute(be.compile(alone), Bindings().bind(ax, bufs[x]).bind(aw, binds.get(nwid)).bind(ah, hb))
        assert np.array_equal(bits(got_h), bits(be.download(hb, np.empty(m * H, np.float32))))
        assert _rel(got_h, orc.rms_norm(x0, nw, m, H, 1e-6).ravel()) < 1e-6
        assert _rel(got_act, orc.gated_act(g0, u0, m, FF).ravel()) < 1e-6
        # the Linears multiply exactly those stored rows
        for buf, w, dt, src, k, n in ((q, wq, DType.Q4K, got_h, H, H), (v, wv, DType.Q6K, got_h, H, 256),
                                      (dn, wd, DType.Q4K, got_act, FF, H)):
            got = be.download(bufs[buf], np.empty((m, n), np.float32))
            assert np.array_equal(bits(got), bits(orc.linear(dt, w, src, m, k, n).reshape(m, n)))
    # quantize + GEMM for each of the three (format, row length) groups; the norm and the activation add none
    assert plan.launches() == 6


@pytest.mark.parametrize("m,in_f", [(4, 1024), (4, 8192), (12, 1024), (24, 1024), (40, 8192)])
@pytest.mark.parametrize("dtype", [DType.Q4K, DType.Q8_0])
def test_residual_add_rides_in_the_small_batch_launch(be, dtype, m, in_f):
    """Linear (two rows and more) -> Add(residual), in place on the residual stream: every
    small-batch kernel (the dot4 batches in their one-wave and K-split forms, the 16- and
    32-token MFMA kernels) stores `y + residual` beside y, so the Add has no launch of its own;
    the sum is the CPU's `a + b` on the stored y, bit for bit."""
    from infr_amd import Add
    out_f = 96
    w = synth_weight(dtype, 5, out_f, in_f, 0.05)
    g, binds = Graph(), Bindings()
    x, h = g.input(TensorDesc((m, in_f), DType.F32)), g.input(TensorDesc((m, out_f), DType.F32))
    y = g.output(TensorDesc((m, out_f), DType.F32))
    xb, hb, yb = be.alloc(m * in_f * 4), be.alloc(m * out_f * 4), be.alloc(m * out_f * 4)
    wid = g.weight(TensorDesc((out_f, in_f), dtype))
    binds.bind(x, xb).bind(h, hb).bind(y, yb).bind(wid, be.upload_new(w))
    g.push(Linear(x, wid, y, m, in_f, out_f))
    g.push(Add(y, h, h, m * out_f))
    plan = be.compile(g)
    for seed in (10, 20):
        x0, h0 = synth_normal_f32(seed, m * in_f), synth_normal_f32(seed + 1, m * out_f)
        be.upload(xb, x0)
        be.upload(hb, h0)
        be.execute(plan, binds)
        got_y = be.download(yb, np.empty(m * out_f, np.float32))
        got_h = be.download(hb, np.empty(m * out_f, np.float32))
        assert _rel(got_y, orc.linear(dtype, w, x0, m, in_f, out_f).ravel()) < 1e-5
        assert np.array_equal(bits(got_h), bits(h0 + got_y))
    assert plan.launches() == 2                             # the quantizer and the GEMM


@pytest.mark.parametrize("m", [3, 16])
def test_combined_gate_up_activation_rides_in_the_small_batch_quantizer(be, m):
    """Op::GatedActFused on a [rows, 2 * nff] buffer (gate half first) in front of a small-batch
    Linear, with a clamp and the GELU form: folded into that Linear's quantizer launch, same bits
    as the op alone."""
    from infr_amd import GatedActFused
    FF, H = 1024, 512
    wd = synth_weight(DType.Q5K, 3, H, FF, 0.05)
    g, binds = Graph(), Bindings()
    gu = g.input(TensorDesc((m, 2 * FF), DType.F32))
    act, dn = g.output(TensorDesc((m, FF), DType.F32)), g.output(TensorDesc((m, H), DType.F32))
    gub, actb, dnb = be.alloc(m * 2 * FF * 4), be.alloc(m * FF * 4), be.alloc(m * H * 4)
    wid = g.weight(TensorDesc((H, FF), DType.Q5K))
    binds.bind(gu, gub).bind(act, actb).bind(dn, dnb).bind(wid, be.upload_new(wd))
    g.push(GatedActFused(gu, act, m, FF, act=1, swiglu_clamp=1.5))
    g.push(Linear(act, wid, dn, m, FF, H))
    plan = be.compile(g)
    alone = Graph()
    agu, aact = alone.input(TensorDesc((m, 2 * FF), DType.F32)), alone.output(TensorDesc((m, FF), DType.F32))
    alone.push(GatedActFused(agu, aact, m, FF, act=1, swiglu_clamp=1.5))
    alone_plan, alone_out = be.compile(alone), be.alloc(m * FF * 4)
    for seed in (10, 20):
        gu0 = synth_normal_f32(seed, m * 2 * FF) * np.float32(1.5)
        be.upload(gub, gu0)
        be.execute(plan, binds)
        be.execute(alone_plan, Bindings().bind(agu, gub).bind(aact, alone_out))
        got_act = be.download(actb, np.empty(m * FF, np.float32))
        assert np.array_equal(bits(got_act), bits(be.download(alone_out, np.empty(m * FF, np.float32))))
        got = be.download(dnb, np.empty((m, H), np.float32))
        assert np.array_equal(bits(got), bits(orc.linear(DType.Q5K, wd, got_act, m, FF, H).reshape(m, H)))
    assert plan.launches() == 2


@pytest.mark.parametrize("wide_first", [False, True])
@pytest.mark.parametrize("shared_x", [True, False])
def test_small_and_large_batch_ops_of_one_shape_class_on_one_level(be, wide_first, shared_x):
    """Whether a batch counts as small depends on out_f as well (Q4_K at 33..128 tokens: a 1024-row matrix
    takes the 16-token K-split kernel, a 12288-row one the 32-token tiles). Two such Linears of one dtype,
    row length and token count on one level: the narrow one runs in a small-batch group, the wide one alone,
    whichever comes first; with distinct activations the group's scratch is sized when it is scheduled."""
    m, in_f = 48, 4096
    shapes = [(1024, 70), (12288, 71)]
    if wide_first:
        shapes.reverse()
    g, binds = Graph(), Bindings()
    xs, ws, ybs = [], [], []
    for i, (out_f, seed) in enumerate(shapes):
        if i == 0 or not shared_x:
            x = synth_normal_f32(80 + i, m * in_f)
            xid = g.input(TensorDesc((m, in_f), DType.F32))
            binds.bind(xid, be.upload_new(x))
        xs.append(x)
        w = synth_weight(DType.Q4K, seed, out_f, in_f)
        ws.append(w)
        wid = g.weight(TensorDesc((out_f, in_f), DType.Q4K))
        yid = g.output(TensorDesc((m, out_f), DType.F32))
        yb = be.alloc(m * out_f * 4)
        ybs.append(yb)
        binds.bind(wid, be.upload_new(w)).bind(yid, yb)
        g.push(Linear(xid, wid, yid, m, in_f, out_f))
    plan = be.compile(g)
    for _ in range(2):
        be.execute(plan, binds)
        for (out_f, _), x, w, yb in zip(shapes, xs, ws, ybs):
            got = be.download(yb, np.empty((m, out_f), np.float32))
            rows = 64                                                # sampled weight rows against the oracle
            for row0 in (0, out_f - rows):
                want = orc.linear(DType.Q4K, w[row0 * 2304:(row0 + rows) * 2304], x, m, in_f, rows)
                assert np.array_equal(bits(got[:, row0:row0 + rows]), bits(want)), (out_f, row0)


def test_prefill_linears_of_one_level_share_the_activation_quantization(be):
    """q / k / v of a prefill chunk multiply one activation tensor: the plan quantizes it once per layout
    and level. Five Linears over one x at 300 tokens - Q4_K strips, a Q6_K tile kernel (same tiled layout:
    shared), a narrow Q4_K matrix on the 16-token kernel (row-major layout: quantized again), then strips
    again (tiled once more) and a Linear over another tensor - each against the oracle on sampled rows,
    on the recording execute and on a replay with new activations."""
    m, in_f = 300, 1024
    specs = [(DType.Q4K, 2304, 0), (DType.Q6K, 640, 0), (DType.Q4K, 512, 0), (DType.Q4K, 2600, 0), (DType.Q4K, 2304, 1)]
    g, binds = Graph(), Bindings()
    xids, xbs = [], []
    for i in range(2):
        xids.append(g.input(TensorDesc((m, in_f), DType.F32)))
        xbs.append(be.alloc(m * in_f * 4))
        binds.bind(xids[i], xbs[i])
    ws, ybs = [], []
    for i, (dt, out_f, xi) in enumerate(specs):
        w = synth_weight(dt, 600 + i, out_f, in_f, 0.05)
        ws.append(w)
        wid = g.weight(TensorDesc((out_f, in_f), dt))
        yid = g.output(TensorDesc((m, out_f), DType.F32))
        ybs.append(be.alloc(m * out_f * 4))
        binds.bind(wid, be.upload_new(w)).bind(yid, ybs[i])
        g.push(Linear(xids[xi], wid, yid, m, in_f, out_f))
    plan = be.compile(g)
    for rep in range(2):
        xs = [synth_normal_f32(610 + 2 * rep + i, m * in_f) for i in range(2)]
        for xb, x in zip(xbs, xs):
            be.upload(xb, x)
        be.execute(plan, binds)
        toks = [0, 37, 255, 256, m - 1]
        for (dt, out_f, xi), w, yb in zip(specs, ws, ybs):
            got = be.download(yb, np.empty((m, out_f), np.float32))[toks]
            want = orc.linear(dt, w, xs[xi].reshape(m, in_f)[toks].ravel(), len(toks), in_f, out_f)
            rel = np.linalg.norm(got.astype(np.float64) - want) / np.linalg.norm(want)
            assert rel <= 2e-6, (rep, int(dt), out_f, rel)


@pytest.mark.parametrize("dtype,in_f", [(DType.Q4K, 256), (DType.Q4K, 768), (DType.Q4K, 1024), (DType.Q4K, 1536), (DType.Q4K, 4096), (DType.Q4K, 5120),
                                        (DType.Q4K, 8192), (DType.Q4K, 12288), (DType.Q5K, 1536), (DType.Q5K, 4096),
                                        (DType.Q5K, 12288), (DType.Q6K, 4096)])
def test_many_round_decode_groups_stream_their_rows_through_lds(be, dtype, in_f):
    # A level of one-token Q4_K / Q5_K Linears (and Q6_K, which keeps the direct loads) with enough rows for many rounds of workgroups (over 131072)
    # takes the form whose waves fetch their rows as whole lines into LDS rings. Row counts that are
    # not multiples of the tile height, rows of 1.125, 3.375, 4.5 and 6.75 lines (waves start at every
    # 16-byte offset of a line), rows
    # shorter than a wave step, rows of two and three wave steps with a short last step; two
    # activations. Ordered sums: every output equals the oracle's bits.
    rows_each = [16387, 20011, 9001] if in_f <= 4096 else [6007, 4001, 3003]
    reps = -(-140000 // sum(rows_each))
    g, binds = Graph(), Bindings()
    xs = [synth_normal_f32(31 + i, in_f) for i in range(2)]
    xids = [g.input(TensorDesc((1, in_f), DType.F32)) for _ in xs]
    for xid, x in zip(xids, xs):
        binds.bind(xid, be.upload_new(x))
    ws = [synth_weight(dtype, 500 + i, r, in_f) for i, r in enumerate(rows_each)]
    wbufs = [be.upload_new(w) for w in ws]
    cases = []
    for rep in range(reps):
        for i, r in enumerate(rows_each):
            wid = g.weight(TensorDesc((r, in_f), dtype))
            yid = g.output(TensorDesc((1, r), DType.F32))
            yb = be.alloc(r * 4)
            binds.bind(wid, wbufs[i]).bind(yid, yb)
            xi = (rep + i) % 2
            g.push(Linear(xids[xi], wid, yid, 1, in_f, r))
            cases.append((i, xi, yb))
    plan = be.compile(g)
    want = {(i, xi): orc.linear(dtype, ws[i], xs[xi], 1, in_f, rows_each[i]).ravel()
            for i in range(len(ws)) for xi in range(2)}
    for _ in range(2):  # record, then replay
        be.execute(plan, binds)
        for i, xi, yb in cases:
            got = be.download(yb, np.empty(rows_each[i], np.float32))
            assert np.array_equal(bits(got), bits(want[(i, xi)])), (i, xi)


def test_streamed_decode_group_with_an_absorbed_norm_and_absorbed_adds(be):
    # RmsNorm -> many one-token Q4_K Linears on one level (enough rows for the streamed form), each
    # followed by a residual Add: the norm runs in every workgroup's prologue, the adds in the row
    # flush (residuals of a wave's rows prefetched by its lanes). Row counts leave partial tiles.
    from infr_amd import Add, RmsNorm
    H, n_ops = 2048, 12
    rows_each = [12291, 11777, 12800]
    g, binds = Graph(), Bindings()
    x = synth_normal_f32(77, H)
    nw = synth_normal_f32(78, H) * np.float32(0.1) + np.float32(1.0)
    xid, nwid = g.input(TensorDesc((1, H), DType.F32)), g.input(TensorDesc((H,), DType.F32))
    hid = g.output(TensorDesc((1, H), DType.F32))
    hb = be.alloc(H * 4)
    binds.bind(xid, be.upload_new(x)).bind(nwid, be.upload_new(nw)).bind(hid, hb)
    g.push(RmsNorm(xid, nwid, hid, 1, H, 1e-6))
    ws = [synth_weight(DType.Q4K, 600 + i, r, H) for i, r in enumerate(rows_each)]
    wbufs = [be.upload_new(w) for w in ws]
    cases = []
    for k in range(n_ops):
        i = k % len(rows_each)
        r = rows_each[i]
        wid = g.weight(TensorDesc((r, H), DType.Q4K))
        yid, zid = g.output(TensorDesc((1, r), DType.F32)), g.output(TensorDesc((1, r), DType.F32))
        resid = synth_normal_f32(900 + k, r)
        rid = g.input(TensorDesc((1, r), DType.F32))
        yb, zb = be.alloc(r * 4), be.alloc(r * 4)
        binds.bind(wid, wbufs[i]).bind(yid, yb).bind(zid, zb).bind(rid, be.upload_new(resid))
        g.push(Linear(hid, wid, yid, 1, H, r))
        g.push(Add(yid, rid, zid, r))
        cases.append((i, resid, yb, zb))
    assert sum(rows_each[k % 3] for k in range(n_ops)) > 139264
    plan = be.compile(g)
    for _ in range(2):
        be.execute(plan, binds)
        assert plan.launches() == 1, plan.launches()
        h = be.download(hb, np.empty(H, np.float32))
        assert _rel(h, orc.rms_norm(x, nw, 1, H, 1e-6)) < 1e-6
        want = [orc.linear(DType.Q4K, w, h, 1, H, r).ravel() for w, r in zip(ws, rows_each)]
        for i, resid, yb, zb in cases:
            y = be.download(yb, np.empty(rows_each[i], np.float32))
            z = be.download(zb, np.empty(rows_each[i], np.float32))
            assert np.array_equal(bits(y), bits(want[i]))
            assert np.array_equal(bits(z), bits(orc.add(y, resid)))


def test_streamed_decode_group_of_two_step_rows_behind_an_absorbed_gated_activation(be):
    # GatedAct -> many one-token Q4_K Linears over 8192 columns (two wave steps a row, chunks of four
    # load instructions) on one level: the activation is evaluated and quantized in every workgroup's
    # prologue, over the LDS that the rings take afterwards.
    from infr_amd import GatedAct
    FF, n_ops = 8192, 18
    rows_each = [9001, 8000, 7203]
    g, binds = Graph(), Bindings()
    gate, up = synth_normal_f32(41, FF), synth_normal_f32(42, FF)
    gid, uid = g.input(TensorDesc((1, FF), DType.F32)), g.input(TensorDesc((1, FF), DType.F32))
    aid = g.output(TensorDesc((1, FF), DType.F32))
    ab = be.alloc(FF * 4)
    binds.bind(gid, be.upload_new(gate)).bind(uid, be.upload_new(up)).bind(aid, ab)
    g.push(GatedAct(gid, uid, aid, 1, FF))
    ws = [synth_weight(DType.Q4K, 700 + i, r, FF) for i, r in enumerate(rows_each)]
    wbufs = [be.upload_new(w) for w in ws]
    cases = []
    for k in range(n_ops):
        i = k % len(rows_each)
        wid = g.weight(TensorDesc((rows_each[i], FF), DType.Q4K))
        yid = g.output(TensorDesc((1, rows_each[i]), DType.F32))
        yb = be.alloc(rows_each[i] * 4)
        binds.bind(wid, wbufs[i]).bind(yid, yb)
        g.push(Linear(aid, wid, yid, 1, FF, rows_each[i]))
        cases.append((i, yb))
    assert sum(rows_each[k % 3] for k in range(n_ops)) > 139264
    plan = be.compile(g)
    for _ in range(2):
        be.execute(plan, binds)
        assert plan.launches() == 1, plan.launches()
        act = be.download(ab, np.empty(FF, np.float32))
        assert _rel(act, orc.gated_act(gate, up, 1, FF)) < 1e-6
        want = [orc.linear(DType.Q4K, w, act, 1, FF, r).ravel() for w, r in zip(ws, rows_each)]
        for i, yb in cases:
            y = be.download(yb, np.empty(rows_each[i], np.float32))
            assert np.array_equal(bits(y), bits(want[i]))


def _gated_ffn(be, dt, H, FF, *, combined, up_first=False, act=0, clamp=None, norm=False, reader_between=False,
               down_dt=None, seed=0):
    """x [-> RmsNorm] -> gate / up (or one Linear onto [gate | up]) -> GatedAct -> down. Returns
    (plan, run) where run(x) executes and returns every tensor of the chain from the device."""
    from infr_amd import Add, GatedAct, GatedActFused, RmsNorm
    down_dt = dt if down_dt is None else down_dt
    g, binds, bufs, host = Graph(), Bindings(), {}, {}

    def tensor(name, n, data=None):
        t = g.output(TensorDesc((1, n), DType.F32)) if data is None else g.input(TensorDesc((1, n), DType.F32))
        bufs[name] = be.upload_new(data) if data is not None else be.alloc(n * 4)
        binds.bind(t, bufs[name])
        return t

    def weight(name, d, out_f, in_f, s):
        host[name] = synth_weight(d, s, out_f, in_f, 0.05)
        t = g.weight(TensorDesc((out_f, in_f), d))
        binds.bind(t, be.upload_new(host[name]))
        return t

    x = tensor("x", H, np.zeros(H, np.float32))
    h = x
    if norm:
        host["nw"] = synth_normal_f32(seed + 3, H) * np.float32(0.1) + np.float32(1.0)
        nw = tensor("nw", H, host["nw"])
        h = tensor("h", H)
        g.push(RmsNorm(x, nw, h, 1, H, 1e-6))
    a = tensor("act", FF)
    if combined:
        wgu, gu = weight("wgu", dt, 2 * FF, H, seed + 10), tensor("gu", 2 * FF)
        g.push(Linear(h, wgu, gu, 1, H, 2 * FF))
        g.push(GatedActFused(gu, a, 1, FF, act=act, swiglu_clamp=clamp))
    else:
        wg, wu = weight("wg", dt, FF, H, seed + 10), weight("wu", dt, FF, H, seed + 11)
        gt, up = tensor("gate", FF), tensor("up", FF)
        lin = [Linear(h, wg, gt, 1, H, FF), Linear(h, wu, up, 1, H, FF)]
        for op in (reversed(lin) if up_first else lin):
            g.push(op)
        if reader_between:   # someone still reads the activation's dst after the projections
            zero, cp = tensor("zero", FF, np.zeros(FF, np.float32)), tensor("copy", FF)
            g.push(Add(a, zero, cp, FF))
        g.push(GatedAct(gt, up, a, 1, FF, act=act, swiglu_clamp=clamp))
    if FF % 256 == 0:    # (the narrow cases end at the activation)
        wd, y = weight("wd", down_dt, H, FF, seed + 12), tensor("y", H)
        g.push(Linear(a, wd, y, 1, FF, H))
    plan = be.compile(g)

    def run(xv, act_before=None):
        be.upload(bufs["x"], xv)
        if act_before is not None:
            be.upload(bufs["act"], act_before)
        be.execute(plan, binds)
        return {nm: be.download(b, np.empty(b.len_bytes() // 4, np.float32)) for nm, b in bufs.items()}
    return plan, run, host


@pytest.mark.parametrize("dt", [DType.Q4K, DType.Q6K, DType.Q8_0, DType.Q4_0, DType.Q3K, DType.MXFP4],
                         ids=lambda d: DType(d).name)
@pytest.mark.parametrize("combined", [False, True])
@pytest.mark.parametrize("H,FF", [(512, 100), (1024, 2816), (4096, 1000), (256, 4)])
def test_gated_activation_is_evaluated_where_gate_and_up_are_produced(be, dt, combined, H, FF):
    """Op::GatedAct / GatedActFused behind one-token gate and up projections of one shape: the
    workgroups that produce a row of both also store act(gate) * up, so the chain is two launches
    and the down projection (where the test has one) starts from the finished vector. Gate, up and the activation equal
    what the ops give one by one: the projections bit for bit where the format's decode is
    bit-identical, the activation within 1e-6 of the CPU's expf form."""
    plan, run, host = _gated_ffn(be, dt, H, FF, combined=combined, norm=H >= 1024, seed=H + FF)
    exact = dt in (DType.Q4K, DType.Q6K, DType.Q3K)
    for rep in range(2):
        xv = synth_normal_f32(50 + rep, H)
        d = run(xv)
        assert plan.launches() == (2 if "y" in d else 1), plan.launches()
        h = d["h"] if "h" in d else xv
        if "h" in d:
            assert _rel(h, orc.rms_norm(xv, host["nw"], 1, H, 1e-6)) < 1e-6
        if combined:
            gu = orc.linear(dt, host["wgu"], h, 1, H, 2 * FF).ravel()
            want_g, want_u, got_g, got_u = gu[:FF], gu[FF:], d["gu"][:FF], d["gu"][FF:]
        else:
            want_g = orc.linear(dt, host["wg"], h, 1, H, FF).ravel()
            want_u = orc.linear(dt, host["wu"], h, 1, H, FF).ravel()
            got_g, got_u = d["gate"], d["up"]
        if exact and "h" not in d:
            assert np.array_equal(bits(got_g), bits(want_g)) and np.array_equal(bits(got_u), bits(want_u))
        else:
            assert _rel(got_g, want_g) < 1e-4 and _rel(got_u, want_u) < 1e-4
        assert _rel(d["act"], orc.gated_act(got_g, got_u, 1, FF)) < 1e-6
        if "y" not in d:
            continue
        y_want = orc.linear(dt, host["wd"], d["act"], 1, FF, H).ravel()
        if exact:
            assert np.array_equal(bits(d["y"]), bits(y_want))       # down sees the stored vector itself
        else:
            assert _rel(d["y"], y_want) < 1e-4


@pytest.mark.parametrize("act,clamp", [(1, None), (2, None), (0, 0.75), (1, 1.5)])
def test_paired_gated_activation_kinds_and_clamp(be, act, clamp):
    """GELU, sigmoid and the clamped forms through the paired launch, with the up projection first
    in program order behind an absorbed RmsNorm (whose vector the pair's tiles must still store)."""
    H, FF = 1024, 1536
    plan, run, host = _gated_ffn(be, DType.Q4K, H, FF, combined=False, up_first=True, act=act, clamp=clamp, norm=True,
                                 down_dt=DType.Q6K, seed=7)
    xv = synth_normal_f32(61, H) * np.float32(3.0)
    d = run(xv)
    assert plan.launches() == 2
    assert _rel(d["h"], orc.rms_norm(xv, host["nw"], 1, H, 1e-6)) < 1e-6
    assert _rel(d["gate"], orc.linear(DType.Q4K, host["wg"], d["h"], 1, H, FF)) < 1e-4
    assert _rel(d["act"], orc.gated_act(d["gate"], d["up"], 1, FF, act, clamp=clamp)) < 1e-6
    assert np.array_equal(bits(d["y"]), bits(orc.linear(DType.Q6K, host["wd"], d["act"], 1, FF, H).ravel()))


def test_pairing_is_refused_when_the_activations_dst_is_still_read(be):
    """An op between the projections and the GatedAct reads the activation's dst (its previous
    contents): the activation may not be stored early, and it goes into the down projection's
    prologue instead."""
    H, FF = 512, 768
    plan, run, host = _gated_ffn(be, DType.Q4K, H, FF, combined=False, reader_between=True, seed=9)
    before = synth_normal_f32(71, FF)
    d = run(synth_normal_f32(70, H), act_before=before)
    assert np.array_equal(bits(d["copy"]), bits(before))            # the reader saw the old contents
    assert _rel(d["act"], orc.gated_act(d["gate"], d["up"], 1, FF)) < 1e-6
    assert _rel(d["y"], orc.linear(DType.Q4K, host["wd"], d["act"], 1, FF, H)) < 1e-4


@pytest.mark.parametrize("combined", [False, True])
@pytest.mark.parametrize("H", [1024, 5120])
def test_paired_gated_activation_in_a_many_round_group(be, combined, H):
    """66,000 gate rows and as many up rows: the group is many rounds of workgroups, whose rows go
    through the per-wave LDS rings; a paired tile's two wave sets stream their own matrix each."""
    FF = 66000
    norm = H == 5120 and not combined          # one case also behind an absorbed RmsNorm
    plan, run, host = _gated_ffn(be, DType.Q4K, H, FF, combined=combined, norm=norm, seed=31)
    xv = synth_normal_f32(90, H)
    d = run(xv)
    assert plan.launches() == 1
    if norm:
        assert _rel(d["h"], orc.rms_norm(xv, host["nw"], 1, H, 1e-6)) < 1e-6
        xv = d["h"]
    if combined:
        gu = orc.linear(DType.Q4K, host["wgu"], xv, 1, H, 2 * FF).ravel()
        want_g, want_u, got_g, got_u = gu[:FF], gu[FF:], d["gu"][:FF], d["gu"][FF:]
    else:
        want_g = orc.linear(DType.Q4K, host["wg"], xv, 1, H, FF).ravel()
        want_u = orc.linear(DType.Q4K, host["wu"], xv, 1, H, FF).ravel()
        got_g, got_u = d["gate"], d["up"]
    if norm:       # (the device normalises in registers; its stored vector is what the oracle multiplies)
        assert _rel(got_g, want_g) < 1e-4 and _rel(got_u, want_u) < 1e-4
    else:
        assert np.array_equal(bits(got_g), bits(want_g)) and np.array_equal(bits(got_u), bits(want_u))
    assert _rel(d["act"], orc.gated_act(got_g, got_u, 1, FF)) < 1e-6


@pytest.mark.parametrize("m", [130, 200, 512, 700])
def test_q4k_prefill_linears_over_one_tensor_run_as_one_strip_launch(be, m):
    """q / k / v of a prefill chunk: Q4_K Linears of a level that read one activation tensor are one
    quantization plus one strip launch over all their rows (a 256-row k or v on its own would fill
    a fraction of the machine), from the token counts the strip kernel takes, when the rows together
    are past the 16-token kernel's reach. Every output equals the same op run alone - same kernel, same per-row
    arithmetic - and the oracle within the route's 1e-4; a Linear over another tensor and a Q6_K
    one over the same tensor stay out of the group."""
    in_f = 1024
    specs = [(DType.Q4K, 1024, 0), (DType.Q4K, 256, 0), (DType.Q4K, 300, 0), (DType.Q6K, 256, 0), (DType.Q4K, 1100, 1)]
    g, binds = Graph(), Bindings()
    xids, xbs = [], []
    for i in range(2):
        xids.append(g.input(TensorDesc((m, in_f), DType.F32)))
        xbs.append(be.alloc(m * in_f * 4))
        binds.bind(xids[i], xbs[i])
    ws, wbs, ybs = [], [], []
    for i, (dt, out_f, xi) in enumerate(specs):
        w = synth_weight(dt, 640 + i, out_f, in_f, 0.05)
        ws.append(w)
        wbs.append(be.upload_new(w))
        wid = g.weight(TensorDesc((out_f, in_f), dt))
        yid = g.output(TensorDesc((m, out_f), DType.F32))
        ybs.append(be.alloc(m * out_f * 4))
        binds.bind(wid, wbs[i]).bind(yid, ybs[i])
        g.push(Linear(xids[xi], wid, yid, m, in_f, out_f))
    plan = be.compile(g)
    grouped = m >= 512      # (130: under 0.6 of a 256-token group; 200: the three are within the 16-token kernel's reach)
    for rep in range(2):
        xs = [synth_normal_f32(650 + 2 * rep + i, m * in_f) for i in range(2)]
        for xb, x in zip(xbs, xs):
            be.upload(xb, x)
        be.execute(plan, binds)
        if rep == 0:
            # grouped: (quantize + strips) + Q6_K's (quantize + tiles) + the other tensor's (quantize + GEMM)
            assert not grouped or plan.launches() == 6, plan.launches()
        toks = [0, 37, m // 2, m - 1]
        alone = be.alloc(m * 1100 * 4)
        for (dt, out_f, xi), w, wb, yb in zip(specs, ws, wbs, ybs):
            got = be.download(yb, np.empty((m, out_f), np.float32))
            be.linear(dt, wb, xbs[xi], alone, m, in_f, out_f)
            one = be.download(alone, np.empty((m, out_f), np.float32))
            # (alone, a narrow op may take the 16-token kernel, whose y is infr-cpu's bit for bit; the
            # strips contract the f32 epilogue: the route's 1e-4, in practice ~1e-7)
            assert _rel(got, one) <= 1e-6, (rep, int(dt), out_f)
            want = orc.linear(dt, w, xs[xi].reshape(m, in_f)[toks].ravel(), len(toks), in_f, out_f)
            assert _rel(got[toks], want) <= 2e-6, (rep, int(dt), out_f)
        alone.free()
