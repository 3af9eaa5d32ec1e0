"""GPU parity of the fields of Op::MoeFfn beyond qwen3moe's setting (crates/infr-core/src/graph.rs:932-1010;
CPU arm crates/infr-cpu/src/lib.rs:2293-2309, 2426-2543, 2833-2861, 2932-2945, 2976), through the C ABI
against the CPU oracle: gating function, norm_w, weight_before, the expert activation and its clamp, fused
gate|up banks, per-expert down scale, selection bias, group-limited routing and supplied expert ids - each on
every route the op takes (one row on the factored kernels, one row on the decode-and-dot kernels, a few rows
with the one-launch down stage, a few rows without it, pairs bucketed by expert) - and the refusals: a
setting the kernels do not implement must come back Unsupported, never as another setting's numbers.
Bars as in test_gpu_moe.py: identical selection, rel-L2 <= 1e-4, max-abs <= 1e-3 * max|y|.
"""
import numpy as np
import pytest

from infr_amd import DType, InfrError, Status, synth_normal_f32, synth_weight
from infr_amd.backend import Activation, MoeGating
from oracle import oracle as orc

pytestmark = pytest.mark.gpu

# (rows, ne, n_expert, n_used, nff, gate/up dtype, down dtype): one shape per route
ROUTES = {
    "one_row_factored": (1, 512, 16, 4, 256, DType.Q4K, DType.Q4K),
    "one_row_decode_and_dot": (1, 512, 16, 4, 256, DType.Q4_0, DType.Q4K),
    "few_rows_fused_down": (5, 512, 16, 4, 256, DType.Q4K, DType.Q6K),
    "few_rows_q8_0": (3, 512, 8, 2, 256, DType.Q8_0, DType.Q8_0),
    "few_rows_raw_banks": (3, 512, 8, 2, 256, DType.Q4_1, DType.Q5_0),
    "bucketed_by_expert": (40, 512, 8, 2, 256, DType.Q4K, DType.Q4K),
}


def make(route, seed, fused=False):
    rows, ne, n_expert, n_used, nff, gdt, ddt = ROUTES[route]
    if fused:
        gate = synth_weight(gdt, seed, n_expert * 2 * nff, ne, 0.05)
        up = None
    else:
        gate = synth_weight(gdt, seed, n_expert * nff, ne, 0.05)
        up = synth_weight(gdt, seed + 1, n_expert * nff, ne, 0.05)
    down = synth_weight(ddt, seed + 2, n_expert * ne, nff, 0.05)
    x = synth_normal_f32(seed + 3, rows * ne)
    router = synth_normal_f32(seed + 4, n_expert * ne, sigma=0.05)
    return x, router, gate, up, down


def run_both(be, route, x, router, gate, up, down, scale=1.0, **opts):
    """The op on the device and on the oracle with the same options; returns (got, want) triples."""
    rows, ne, n_expert, n_used, nff, gdt, ddt = ROUTES[route]
    xb, rb, gb, db = be.upload_new(x), be.upload_new(router), be.upload_new(gate), be.upload_new(down)
    ub = be.upload_new(up) if up is not None else None
    yb = be.alloc(rows * ne * 4)
    ib, wb = be.alloc(rows * n_used * 4), be.alloc(rows * n_used * 4)
    dev = dict(opts)
    held = []
    for k in ("down_scale", "exp_probs_b", "expert_ids"):
        if dev.get(k) is not None:
            dev[k] = be.upload_new(np.ascontiguousarray(dev[k]))
            held.append(dev[k])
    try:
        be.moe_ffn(xb, rb, gb, ub, db, yb, rows=rows, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff,
                   scale=scale, gate_dtype=gdt, up_dtype=gdt, down_dtype=ddt, sel_idx=ib, sel_w=wb,
                   fused_gate_up=up is None, **dev)
        got = (be.download(yb, np.empty((rows, ne), np.float32)), be.download(ib, np.empty((rows, n_used), np.int32)),
               be.download(wb, np.empty((rows, n_used), np.float32)))
    finally:
        for b in [xb, rb, gb, db, yb, ib, wb] + held + ([ub] if ub is not None else []):
            b.free()
    ok = {k: (int(v) if k in ("act", "gating") else v) for k, v in opts.items()}
    want = orc.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff, scale=scale,
                       gate_dtype=int(gdt), up_dtype=int(gdt), down_dtype=int(ddt), fused_gate_up=up is None, **ok)
    return got, want


def check(got, want):
    y, idx, w = got
    oy, oidx, ow = want
    assert np.array_equal(idx, oidx), "expert selection differs"
    assert np.allclose(w, ow, rtol=2e-5, atol=0)
    a, b = y.astype(np.float64).ravel(), oy.astype(np.float64).ravel()
    assert np.abs(b).max() > 1e-6
    rel = np.linalg.norm(a - b) / np.linalg.norm(b)
    mx = np.abs(a - b).max() / np.abs(b).max()
    assert rel <= 1e-4 and mx <= 1e-3, f"rel-L2 {rel:.3e} max-abs {mx:.3e}"


@pytest.mark.parametrize("route", list(ROUTES))
@pytest.mark.parametrize("opts", [
    dict(gating=MoeGating.Sigmoid, norm_w=False),
    dict(gating=MoeGating.SqrtSoftplus),
    dict(gating=MoeGating.Sigmoid, norm_w=False, weight_before=True),      # llama4's setting (graph.rs:956-967)
    dict(weight_before=True),
    dict(act=Activation.Gelu),
    dict(act=Activation.Sigmoid),
    dict(swiglu_clamp=0.05),
    dict(act=Activation.Gelu, swiglu_clamp=0.04),
], ids=["sigmoid_raw_w", "sqrt_softplus", "llama4", "weight_before", "gelu", "sigmoid_act", "clamp", "gelu_clamp"])
def test_gating_activation_and_weight_side(be, route, opts):
    got, want = run_both(be, route, *make(route, 300), scale=1.5, **opts)
    check(got, want)


@pytest.mark.parametrize("route", list(ROUTES))
def test_fused_gate_up_bank(be, route):
    got, want = run_both(be, route, *make(route, 310, fused=True))
    check(got, want)


@pytest.mark.parametrize("route", list(ROUTES))
def test_down_scale(be, route):
    n_expert = ROUTES[route][2]
    ds = np.linspace(0.25, 2.0, n_expert).astype(np.float32)
    got, want = run_both(be, route, *make(route, 320), down_scale=ds)
    check(got, want)
    plain = run_both(be, route, *make(route, 320))[0][0]
    assert not np.array_equal(plain, got[0])


@pytest.mark.parametrize("route", list(ROUTES))
def test_selection_bias(be, route):
    n_expert = ROUTES[route][2]
    bias = (synth_normal_f32(331, n_expert, sigma=0.2)).astype(np.float32)
    got, want = run_both(be, route, *make(route, 330), exp_probs_b=bias)
    check(got, want)
    assert not np.array_equal(got[1], run_both(be, route, *make(route, 330))[0][1])       # the bias moved a selection


@pytest.mark.parametrize("route", list(ROUTES))
@pytest.mark.parametrize("groups,used", [(4, 2), (2, 1), (4, 4)])
def test_group_limited_routing(be, route, groups, used):
    rows, ne, n_expert, n_used = ROUTES[route][:4]
    if n_expert // groups * used < n_used:
        pytest.skip("fewer experts kept than selected: refused (see the refusals test)")
    got, want = run_both(be, route, *make(route, 340), n_expert_groups=groups, n_expert_groups_used=used,
                         gating=MoeGating.Sigmoid, exp_probs_b=synth_normal_f32(341, n_expert, sigma=0.1))
    check(got, want)
    per = n_expert // groups
    assert all(len({int(e) // per for e in row}) <= used for row in got[1])


@pytest.mark.parametrize("route", list(ROUTES))
def test_supplied_expert_ids(be, route):
    rows, ne, n_expert, n_used = ROUTES[route][:4]
    rng = np.random.default_rng(350)
    ids = np.stack([rng.permutation(n_expert)[:n_used] for _ in range(rows)]).astype(np.int32)
    got, want = run_both(be, route, *make(route, 351), expert_ids=ids, gating=MoeGating.SqrtSoftplus)
    check(got, want)
    assert np.array_equal(got[1], ids)


def test_refusals_are_unsupported_not_wrong_numbers(be):
    """ep_band needs another GPU; a clamp with Sigmoid or weight_before and supplied ids with a bias or groups are
    what the CPU arm asserts against (lib.rs:2293-2309); groups must divide the experts and keep n_used of them."""
    route = "one_row_factored"
    x, router, gate, up, down = make(route, 360)
    n_expert, n_used = ROUTES[route][2], ROUTES[route][3]
    ids = np.zeros((1, n_used), np.int32)
    bias = np.zeros(n_expert, np.float32)
    for bad in (dict(ep_band=(0, 8)), dict(swiglu_clamp=1.0, act=Activation.Sigmoid), dict(swiglu_clamp=1.0, weight_before=True),
                dict(expert_ids=ids, exp_probs_b=bias), dict(expert_ids=ids, n_expert_groups=2, n_expert_groups_used=1),
                dict(n_expert_groups=3, n_expert_groups_used=1), dict(n_expert_groups=8, n_expert_groups_used=1),
                dict(act=7), dict(gating=5)):
        with pytest.raises(InfrError) as e:
            # (the oracle leg is never reached: the device call raises first)
            run_both(be, route, x, router, gate, up, down, **bad)
        assert e.value.status == Status.Unsupported, bad


def test_params_in_a_plan(be):
    """The same fields through compile / execute: a llama4-style op and one with every optional operand."""
    from infr_amd import Bindings, Graph, MoeFfn, TensorDesc
    route = "few_rows_fused_down"
    rows, ne, n_expert, n_used, nff, gdt, ddt = ROUTES[route]
    x, router, gate, up, down = make(route, 370)
    ds = np.linspace(0.5, 1.5, n_expert).astype(np.float32)
    bias = synth_normal_f32(371, n_expert, sigma=0.2)
    g, binds = Graph(), Bindings()
    xid = g.input(TensorDesc((rows, ne), DType.F32))
    rid = g.weight(TensorDesc((n_expert, ne), DType.F32))
    gid, uid = (g.weight(TensorDesc((n_expert, nff, ne), gdt)) for _ in range(2))
    did = g.weight(TensorDesc((n_expert, ne, nff), ddt))
    sid, bid = (g.weight(TensorDesc((n_expert,), DType.F32)) for _ in range(2))
    y1, y2 = (g.output(TensorDesc((rows, ne), DType.F32)) for _ in range(2))
    for t, a in ((xid, x), (rid, router), (gid, gate), (uid, up), (did, down), (sid, ds), (bid, bias)):
        binds.bind(t, be.upload_new(a))
    yb1, yb2 = be.alloc(rows * ne * 4), be.alloc(rows * ne * 4)
    binds.bind(y1, yb1).bind(y2, yb2)
    g.push(MoeFfn(xid, xid, rid, gid, uid, did, y1, ne, n_expert, n_used, nff, 1.0, gating=MoeGating.Sigmoid,
                  norm_w=False, weight_before=True))
    g.push(MoeFfn(xid, xid, rid, gid, uid, did, y2, ne, n_expert, n_used, nff, 2.0, act=Activation.Gelu,
                  down_scale=sid, exp_probs_b=bid, n_expert_groups=4, n_expert_groups_used=2))
    plan = be.compile(g)
    kw = dict(ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff, gate_dtype=int(gdt), up_dtype=int(gdt), down_dtype=int(ddt))
    w1 = orc.moe_ffn(x, router, gate, up, down, gating=1, norm_w=False, weight_before=True, **kw)[0]
    w2 = orc.moe_ffn(x, router, gate, up, down, scale=2.0, act=1, down_scale=ds, exp_probs_b=bias, n_expert_groups=4,
                     n_expert_groups_used=2, **kw)[0]
    for _ in range(2):                          # the second execute replays the recorded launches
        be.execute(plan, binds)
        for yb, want in ((yb1, w1), (yb2, w2)):
            got = be.download(yb, np.empty((rows, ne), np.float32))
            rel = np.linalg.norm(got.astype(np.float64) - want) / np.linalg.norm(want)
            assert rel <= 1e-4, rel
