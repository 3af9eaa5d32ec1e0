"""GPU parity of Op::MoeFfn against the CPU oracle, through the C ABI.

rows == 1 takes the f32 (decoded weights x unquantized activation) path like infr-cpu; rows >= 2
the int8 path. Router logits are evaluated in the CPU's FMA order, so the selected experts must
be identical; outputs are gated at rel-L2 <= 1e-4 and max-abs <= 1e-3 * max|y| (SiLU/softmax use
the platform's expf on either side, so the last bits may differ).
"""
import numpy as np
import pytest

from infr_amd import DType, synth_normal_f32, synth_weight
from oracle import oracle as orc

pytestmark = pytest.mark.gpu


def banks(seed, ne, n_expert, nff, dtype=DType.Q4K, sigma=0.02):
    gate = synth_weight(dtype, seed, n_expert * nff, ne, sigma)
    up = synth_weight(dtype, seed + 1, n_expert * nff, ne, sigma)
    down = synth_weight(dtype, seed + 2, n_expert * ne, nff, sigma)
    return gate, up, down


def run_moe(be, x, router, gate, up, down, rows, ne, n_expert, n_used, nff, scale, dtype=DType.Q4K):
    xb, rb = be.upload_new(x), be.upload_new(router)
    gb, ub, db = be.upload_new(gate), be.upload_new(up), be.upload_new(down)
    yb = be.alloc(rows * ne * 4)
    ib, wb = be.alloc(rows * n_used * 4), be.alloc(rows * n_used * 4)
    be.moe_ffn(xb, rb, gb, ub, db, yb, rows=rows, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff,
               scale=scale, gate_dtype=dtype, up_dtype=dtype, down_dtype=dtype, sel_idx=ib, sel_w=wb)
    return (be.download(yb, np.empty((rows, ne), np.float32)),
            be.download(ib, np.empty((rows, n_used), np.int32)),
            be.download(wb, np.empty((rows, n_used), np.float32)))


def check(y, idx, w, oy, oidx, ow):
    assert np.array_equal(idx, oidx), "expert selection differs"
    assert np.allclose(w, ow, rtol=1e-5, atol=0)
    a, b = y.astype(np.float64).ravel(), oy.astype(np.float64).ravel()
    assert np.abs(b).max() > 1e-4
    rel = np.linalg.norm(a - b) / np.linalg.norm(b)
    mx = np.abs(a - b).max() / np.abs(b).max()
    assert rel <= 1e-4 and mx <= 1e-3, f"rel-L2 {rel:.3e} max-abs {mx:.3e}"


@pytest.mark.parametrize("rows", [1, 2, 5])
@pytest.mark.parametrize("ne,n_expert,n_used,nff", [(512, 16, 4, 256), (1024, 8, 2, 768)])
def test_moe_small_shapes(be, rows, ne, n_expert, n_used, nff):
    gate, up, down = banks(50 + rows, ne, n_expert, nff, sigma=0.05)
    x = synth_normal_f32(60 + rows, rows * ne)
    router = synth_normal_f32(61, n_expert * ne, sigma=0.05)
    got = run_moe(be, x, router, gate, up, down, rows, ne, n_expert, n_used, nff, 1.25)
    want = orc.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff, scale=1.25)
    check(*got, *want)


@pytest.mark.parametrize("rows", [1, 16])
def test_moe_qwen3_30b_a3b_shape(be, rows):
    # 128 experts, top-8, hidden 2048, expert FFN 768, Q4_K banks
    ne, n_expert, n_used, nff = 2048, 128, 8, 768
    gate, up, down = banks(7, ne, n_expert, nff)
    x = synth_normal_f32(8 + rows, rows * ne)
    router = synth_normal_f32(9, n_expert * ne, sigma=0.03)   # logits ~ N(0, ~1.4^2)
    got = run_moe(be, x, router, gate, up, down, rows, ne, n_expert, n_used, nff, 1.0)
    want = orc.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff)
    check(*got, *want)


def test_moe_router_ties_go_to_the_lower_index(be):
    ne, n_expert, n_used, nff = 256, 6, 3, 256
    gate, up, down = banks(90, ne, n_expert, nff, sigma=0.05)
    x = np.ones(ne, np.float32)
    router = np.zeros((n_expert, ne), np.float32)
    router[4] = 0.01
    _, idx, _ = run_moe(be, x, router, gate, up, down, 1, ne, n_expert, n_used, nff, 1.0)
    assert list(idx[0]) == [4, 0, 1]


@pytest.mark.parametrize("dtype", [DType.Q6K, DType.Q8_0, DType.Q5K])
def test_moe_int8_path_other_bank_formats(be, dtype):
    rows, ne, n_expert, n_used, nff = 3, 512, 8, 2, 256
    gate, up, down = banks(120, ne, n_expert, nff, dtype, sigma=0.05)
    x = synth_normal_f32(121, rows * ne)
    router = synth_normal_f32(122, n_expert * ne, sigma=0.05)
    got = run_moe(be, x, router, gate, up, down, rows, ne, n_expert, n_used, nff, 1.0, dtype)
    want = orc.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff,
                       gate_dtype=int(dtype), up_dtype=int(dtype), down_dtype=int(dtype))
    check(*got, *want)


@pytest.mark.parametrize("rows", [1, 6, 72])     # 72: the expert-bucketed prefill path, captured and replayed
def test_moe_in_a_plan_replays(be, rows):
    """Two Op::MoeFfn separated by a Linear in one compiled plan (the second routes the first's
    output), executed three times with fresh inputs: every replay must match the oracle chain."""
    from infr_amd import Bindings, Graph, Linear, MoeFfn, TensorDesc
    ne, n_expert, n_used, nff = 512, 16, 4, 256
    router = synth_normal_f32(31, n_expert * ne, sigma=0.05)
    b1, b2 = banks(32, ne, n_expert, nff, sigma=0.05), banks(36, ne, n_expert, nff, sigma=0.05)
    wmid = synth_weight(DType.Q4K, 40, ne, ne, 0.05)
    g, binds = Graph(), Bindings()
    xid = g.input(TensorDesc((rows, ne), DType.F32))
    xb = be.alloc(rows * ne * 4)
    rid = g.weight(TensorDesc((n_expert, ne), DType.F32))
    binds.bind(xid, xb).bind(rid, be.upload_new(router))

    def bank_ids(bk):
        ids = []
        for i, w in enumerate(bk):
            shape = (n_expert, nff, ne) if i < 2 else (n_expert, ne, nff)
            wid = g.weight(TensorDesc(shape, DType.Q4K))
            binds.bind(wid, be.upload_new(w))
            ids.append(wid)
        return ids

    outs = []
    for _ in range(3):
        t = g.output(TensorDesc((rows, ne), DType.F32))
        outs.append((t, be.alloc(rows * ne * 4)))
        binds.bind(t, outs[-1][1])
    i1, i2 = bank_ids(b1), bank_ids(b2)
    mid = g.weight(TensorDesc((ne, ne), DType.Q4K))
    binds.bind(mid, be.upload_new(wmid))
    g.push(MoeFfn(xid, xid, rid, i1[0], i1[1], i1[2], outs[0][0], ne, n_expert, n_used, nff, 1.5))
    g.push(Linear(outs[0][0], mid, outs[1][0], rows, ne, ne))
    g.push(MoeFfn(outs[1][0], outs[1][0], rid, i2[0], i2[1], i2[2], outs[2][0], ne, n_expert, n_used, nff, 1.0))
    plan = be.compile(g)
    def gate_out(got, want):
        a, b = got.astype(np.float64).ravel(), np.asarray(want, np.float64).ravel()
        assert np.abs(b).max() > 1e-4
        rel = np.linalg.norm(a - b) / np.linalg.norm(b)
        mx = np.abs(a - b).max() / np.abs(b).max()
        assert rel <= 1e-4 and mx <= 1e-3, f"rel-L2 {rel:.3e} max-abs {mx:.3e}"

    kw = dict(ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff)
    for rep in range(3):
        x = synth_normal_f32(500 + rep, rows * ne)
        be.upload(xb, x)
        be.execute(plan, binds)
        got = [be.download(b, np.empty((rows, ne), np.float32)) for _, b in outs]
        # each stage is gated on its own: downstream oracles are fed the device's upstream output
        gate_out(got[0], orc.moe_ffn(x, router, *b1, scale=1.5, **kw)[0])
        gate_out(got[1], orc.linear(DType.Q4K, wmid, got[0].ravel(), rows, ne, ne))
        gate_out(got[2], orc.moe_ffn(got[1].ravel(), router, *b2, scale=1.0, **kw)[0])


@pytest.mark.parametrize("gu_dtype,down_dtype", [(DType.Q6K, DType.Q6K), (DType.Q8_0, DType.Q8_0),
                                                 (DType.Q5K, DType.Q5K), (DType.Q5K, DType.Q6K),
                                                 (DType.Q4K, DType.Q6K), (DType.Q8_0, DType.Q4K)])
@pytest.mark.parametrize("ne,nff", [(512, 256), (2048, 768)])
def test_moe_one_token_other_bank_formats(be, gu_dtype, down_dtype, ne, nff):
    """rows == 1 (decoded-f32-weights path) for Q6_K / Q8_0 banks and the mixed layouts real files
    use (Q4_K gate/up with a Q6_K down)."""
    n_expert, n_used = 16, 4
    gate = synth_weight(gu_dtype, 130, n_expert * nff, ne, 0.05)
    up = synth_weight(gu_dtype, 131, n_expert * nff, ne, 0.05)
    down = synth_weight(down_dtype, 132, n_expert * ne, nff, 0.05)
    x = synth_normal_f32(133, ne)
    router = synth_normal_f32(134, n_expert * ne, sigma=0.05)
    xb, rb = be.upload_new(x), be.upload_new(router)
    gb, ub, db = be.upload_new(gate), be.upload_new(up), be.upload_new(down)
    yb, ib, wb = be.alloc(ne * 4), be.alloc(n_used * 4), be.alloc(n_used * 4)
    be.moe_ffn(xb, rb, gb, ub, db, yb, rows=1, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff, scale=1.0,
               gate_dtype=gu_dtype, up_dtype=gu_dtype, down_dtype=down_dtype, sel_idx=ib, sel_w=wb)
    got = (be.download(yb, np.empty((1, ne), np.float32)), be.download(ib, np.empty((1, n_used), np.int32)),
           be.download(wb, np.empty((1, n_used), np.float32)))
    want = orc.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff,
                       gate_dtype=int(gu_dtype), up_dtype=int(gu_dtype), down_dtype=int(down_dtype))
    check(*got, *want)


@pytest.mark.parametrize("rows,ne,n_expert,n_used,nff", [(64, 512, 16, 4, 256), (40, 1024, 8, 2, 768),
                                                         (200, 512, 16, 4, 512),
                                                         (400, 512, 8, 2, 256)])     # the tiled router (rows >= 256), ~100 pairs per expert
def test_moe_prefill_buckets_vs_oracle(be, rows, ne, n_expert, n_used, nff):
    """Prefill-sized batches of all-Q4_K banks: pairs bucketed by expert, int8-MFMA GEMM per (expert,
    32 pairs) tile. Same integers and epilogue as the per-pair GEMVs: the first two tokens of the
    batch, run again as a batch of two (per-pair path), give the same bits."""
    gate, up, down = banks(70 + rows, ne, n_expert, nff, sigma=0.05)
    x = synth_normal_f32(71 + rows, rows * ne)
    router = synth_normal_f32(72, n_expert * ne, sigma=0.05)
    got = run_moe(be, x, router, gate, up, down, rows, ne, n_expert, n_used, nff, 1.0)
    want = orc.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff, scale=1.0)
    check(*got, *want)
    two = run_moe(be, x[:2 * ne], router, gate, up, down, 2, ne, n_expert, n_used, nff, 1.0)
    assert np.array_equal(two[1], got[1][:2])
    assert np.array_equal(two[0].view(np.uint32), got[0][:2].view(np.uint32)), "bucketed != per-pair"


def test_moe_prefill_buckets_with_idle_and_crowded_experts(be):
    """A router that sends every token to the same two experts plus one of two others: buckets of
    0, a few and > 32 pairs (several tiles per expert, a ragged last tile)."""
    rows, ne, n_expert, n_used, nff = 75, 512, 16, 3, 256
    gate, up, down = banks(90, ne, n_expert, nff, sigma=0.05)
    x = np.abs(synth_normal_f32(91, rows * ne)) + np.float32(0.1)     # all-positive activations
    router = np.zeros((n_expert, ne), np.float32)
    router[3], router[11] = 0.05, 0.04                                 # always the top two
    router[5, :ne // 2], router[6, ne // 2:] = 0.06, 0.06              # third place depends on the token
    x = x.reshape(rows, ne)
    x[::7, :ne // 2] *= 3.0
    x = x.ravel()
    got = run_moe(be, x, router.ravel(), gate, up, down, rows, ne, n_expert, n_used, nff, 1.0)
    want = orc.moe_ffn(x, router.ravel(), gate, up, down, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff,
                       scale=1.0)
    assert set(np.unique(got[1])) <= {3, 5, 6, 11} and np.bincount(got[1].ravel(), minlength=16)[3] == rows
    check(*got, *want)


def test_moe_qwen3_30b_a3b_prefill(be):
    """512 tokens at the Qwen3-30B-A3B shape (4096 pairs over 128 experts), sampled rows against the
    oracle run on those rows alone (each token's output is independent of the rest of the batch)."""
    ne, n_expert, n_used, nff, rows = 2048, 128, 8, 768, 512
    gate, up, down = banks(7, ne, n_expert, nff)
    x = synth_normal_f32(8, rows * ne)
    router = synth_normal_f32(9, n_expert * ne, sigma=0.05)
    y, idx, w = run_moe(be, x, router, gate, up, down, rows, ne, n_expert, n_used, nff, 1.0)
    pick = [0, 1, 255, 256, 510, 511]
    xs = np.concatenate([x[r * ne:(r + 1) * ne] for r in pick])
    want = orc.moe_ffn(xs, router, gate, up, down, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff, scale=1.0)
    check(y[pick], idx[pick], w[pick], *want)
    assert np.isfinite(y).all() and len(np.unique(idx)) > 100        # most experts are touched


@pytest.mark.parametrize("gu,down", [(DType.Q4K, DType.Q6K), (DType.Q6K, DType.Q4K), (DType.Q6K, DType.Q6K),
                                     (DType.Q4K, DType.Q8_0), (DType.Q5K, DType.Q5K), (DType.Q5K, DType.Q6K),
                                     (DType.Q8_0, DType.Q8_0)])
def test_moe_prefill_buckets_with_mixed_bank_formats(be, gu, down):
    """A Q4_K_M file's mix (Q4_K gate / up beside a Q6_K down bank), its mirror, a Q5_K_M file's mix,
    and all-Q6_K / Q5_K / Q8_0: every bank takes its format's bucketed MFMA GEMM in one op - and the
    first two tokens, run again as a batch of two (per-pair GEMVs throughout), give the same bits in
    the formats whose sums are ordered."""
    rows, ne, n_expert, n_used, nff = 96, 512, 16, 4, 256          # 24 pairs per expert
    gate_w = synth_weight(gu, 201, n_expert * nff, ne, 0.05)
    up_w = synth_weight(gu, 202, n_expert * nff, ne, 0.05)
    down_w = synth_weight(down, 203, n_expert * ne, nff, 0.05)
    x = synth_normal_f32(204, rows * ne)
    router = synth_normal_f32(205, n_expert * ne, sigma=0.05)
    yb, ib, wb = be.alloc(rows * ne * 4), be.alloc(rows * n_used * 4), be.alloc(rows * n_used * 4)
    be.moe_ffn(be.upload_new(x), be.upload_new(router), be.upload_new(gate_w), be.upload_new(up_w),
               be.upload_new(down_w), yb, rows=rows, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff,
               scale=1.0, gate_dtype=gu, up_dtype=gu, down_dtype=down, sel_idx=ib, sel_w=wb)
    got = (be.download(yb, np.empty((rows, ne), np.float32)), be.download(ib, np.empty((rows, n_used), np.int32)),
           be.download(wb, np.empty((rows, n_used), np.float32)))
    want = orc.moe_ffn(x, router, gate_w, up_w, down_w, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff,
                       scale=1.0, gate_dtype=int(gu), up_dtype=int(gu), down_dtype=int(down))
    check(*got, *want)
    y2 = be.alloc(2 * ne * 4)
    be.moe_ffn(be.upload_new(x[:2 * ne]), be.upload_new(router), be.upload_new(gate_w), be.upload_new(up_w),
               be.upload_new(down_w), y2, rows=2, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff,
               scale=1.0, gate_dtype=gu, up_dtype=gu, down_dtype=down)
    two = be.download(y2, np.empty((2, ne), np.float32))
    if DType.Q8_0 not in (gu, down):       # the ordered formats: bit-identical whichever kernel ran
        assert np.array_equal(two.view(np.uint32), got[0][:2].view(np.uint32)), "bucketed != per-pair"


def run_moe_mixed(be, x, router, gate, up, down, rows, ne, n_expert, n_used, nff, dts):
    xb, rb = be.upload_new(x), be.upload_new(router)
    gb, ub, db = be.upload_new(gate), be.upload_new(up), be.upload_new(down)
    yb = be.alloc(rows * ne * 4)
    ib, wb = be.alloc(rows * n_used * 4), be.alloc(rows * n_used * 4)
    be.moe_ffn(xb, rb, gb, ub, db, yb, rows=rows, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff,
               gate_dtype=dts[0], up_dtype=dts[1], down_dtype=dts[2], sel_idx=ib, sel_w=wb)
    return (be.download(yb, np.empty((rows, ne), np.float32)),
            be.download(ib, np.empty((rows, n_used), np.int32)),
            be.download(wb, np.empty((rows, n_used), np.float32)))


@pytest.mark.parametrize("rows", [1, 5])
@pytest.mark.parametrize("dtype", [DType.Q4_0, DType.Q4_1, DType.Q5_0, DType.Q5_1, DType.IQ4NL, DType.Q2_0])
def test_moe_banks_in_the_32_block_formats(be, dtype, rows):
    """expert_acts_kind (crates/infr-cpu/src/moe.rs:42-53): Q5_0 banks take per-32 int8 activations
    from two rows up (Blk32), the other 32-block formats and every single-row call multiply decoded
    f32 weights with the raw activation row (Raw)."""
    ne, n_expert, n_used, nff = 512, 8, 2, 256
    gate, up, down = banks(200 + int(dtype), ne, n_expert, nff, dtype, sigma=0.05)
    x = synth_normal_f32(230 + rows, rows * ne)
    router = synth_normal_f32(231, n_expert * ne, sigma=0.05)
    got = run_moe(be, x, router, gate, up, down, rows, ne, n_expert, n_used, nff, 1.0, dtype)
    want = orc.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff,
                       gate_dtype=int(dtype), up_dtype=int(dtype), down_dtype=int(dtype))
    check(*got, *want)


@pytest.mark.parametrize("rows", [1, 6])
@pytest.mark.parametrize("dtype", [DType.F32, DType.F16, DType.BF16])
def test_moe_banks_of_plain_float_rows(be, dtype, rows):
    """Unquantized expert banks take expert_acts_kind's Raw arm at every row count
    (crates/infr-cpu/src/moe.rs:42-53: anything without an int8 arm), decoded by
    crates/infr-gguf/src/dequant.rs:13-22 and multiplied in `dot`'s order."""
    ne, n_expert, n_used, nff = 512, 8, 2, 256

    def rows_of(seed, n):
        w = synth_normal_f32(seed, n, sigma=0.05)
        if dtype == DType.F16:
            return w.astype(np.float16).view(np.uint8)
        if dtype == DType.BF16:
            return (w.view(np.uint32) >> 16).astype(np.uint16).view(np.uint8)
        return w.view(np.uint8)

    gate, up, down = rows_of(401, n_expert * nff * ne), rows_of(402, n_expert * nff * ne), rows_of(403, n_expert * ne * nff)
    x = synth_normal_f32(404 + rows, rows * ne)
    router = synth_normal_f32(405, n_expert * ne, sigma=0.05)
    got = run_moe_mixed(be, x, router, gate, up, down, rows, ne, n_expert, n_used, nff, (dtype,) * 3)
    want = orc.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff,
                       gate_dtype=int(dtype), up_dtype=int(dtype), down_dtype=int(dtype))
    check(*got, *want)


def test_moe_one_expert_per_token_with_tall_down_tiles(be):
    """n_used == 1 gives the fused down launch one wave per workgroup; with 130 tokens of a 4096-wide
    model its tiles are 128 output rows tall, more than that workgroup has threads: the weighted
    sum has to walk them."""
    rows, ne, n_expert, n_used, nff = 130, 4096, 72, 1, 256
    gate, up, down = banks(420, ne, n_expert, nff, sigma=0.05)
    x = synth_normal_f32(421, rows * ne)
    router = synth_normal_f32(422, n_expert * ne, sigma=0.02)
    got = run_moe(be, x, router, gate, up, down, rows, ne, n_expert, n_used, nff, 1.0)
    want = orc.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff)
    check(*got, *want)


@pytest.mark.parametrize("rows", [1, 3, 300])      # 300: the register-tiled router
@pytest.mark.parametrize("router_dtype", [DType.F16, DType.BF16])
def test_moe_router_weights_in_half_precision(be, router_dtype, rows):
    """The router matrix is one more bank to the CPU arm (expert_gemm over router_dtype,
    crates/infr-cpu/src/lib.rs:2376-2395): f16 / bf16 rows are widened exactly and multiplied in
    `dot`'s order, so the selection still equals the oracle's."""
    ne, n_expert, n_used, nff = 512, 16, 4, 256
    gate, up, down = banks(410, ne, n_expert, nff, sigma=0.05)
    r32 = synth_normal_f32(413, n_expert * ne, sigma=0.05)
    router = (r32.astype(np.float16) if router_dtype == DType.F16
              else (r32.view(np.uint32) >> 16).astype(np.uint16)).view(np.uint8)
    x = synth_normal_f32(414 + rows, rows * ne)
    xb, rb = be.upload_new(x), be.upload_new(router)
    gb, ub, db = be.upload_new(gate), be.upload_new(up), be.upload_new(down)
    yb, ib, wb = be.alloc(rows * ne * 4), be.alloc(rows * n_used * 4), be.alloc(rows * n_used * 4)
    be.moe_ffn(xb, rb, gb, ub, db, yb, rows=rows, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff,
               router_dtype=router_dtype, sel_idx=ib, sel_w=wb)
    got = (be.download(yb, np.empty((rows, ne), np.float32)), be.download(ib, np.empty((rows, n_used), np.int32)),
           be.download(wb, np.empty((rows, n_used), np.float32)))
    want = orc.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff,
                       router_dtype=int(router_dtype))
    check(*got, *want)


@pytest.mark.parametrize("rows", [1, 4, 40])     # 40 rows of 8 experts: the bucketed Q4_K gate beside the rest
def test_moe_banks_of_three_different_kinds(be, rows):
    """gate Q4_K (per-256 activations), up Q5_0 (per-32), down Q4_0 (raw f32 rows) in one op: every
    bank takes the activation form its own format asks for."""
    ne, n_expert, n_used, nff = 512, 8, 2, 256
    dts = (DType.Q4K, DType.Q5_0, DType.Q4_0)
    gate = synth_weight(dts[0], 301, n_expert * nff, ne, 0.05)
    up = synth_weight(dts[1], 302, n_expert * nff, ne, 0.05)
    down = synth_weight(dts[2], 303, n_expert * ne, nff, 0.05)
    x = synth_normal_f32(304 + rows, rows * ne)
    router = synth_normal_f32(305, n_expert * ne, sigma=0.05)
    got = run_moe_mixed(be, x, router, gate, up, down, rows, ne, n_expert, n_used, nff, dts)
    want = orc.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff,
                       gate_dtype=int(dts[0]), up_dtype=int(dts[1]), down_dtype=int(dts[2]))
    check(*got, *want)


@pytest.mark.parametrize("rows", [1, 3])
@pytest.mark.parametrize("dtype", [DType.Q4K, DType.Q6K])
def test_moe_hidden_size_above_4096(be, dtype, rows):
    """One token: a lane of the factored kernels keeps 64 activations of a row in registers, rows of
    more than 4096 columns go round by round. Two rows and more run the id-gathered int8 GEMVs at any
    length their wave steps reach."""
    ne, n_expert, n_used, nff = 8192, 4, 2, 512
    gate, up, down = banks(400, ne, n_expert, nff, dtype, sigma=0.03)
    x = synth_normal_f32(401, rows * ne)
    router = synth_normal_f32(402, n_expert * ne, sigma=0.02)
    got = run_moe(be, x, router, gate, up, down, rows, ne, n_expert, n_used, nff, 1.0, dtype)
    want = orc.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff,
                       gate_dtype=int(dtype), up_dtype=int(dtype), down_dtype=int(dtype))
    check(*got, *want)


@pytest.mark.parametrize("dtype", [DType.Q4K, DType.Q5K, DType.Q6K, DType.Q8_0])
@pytest.mark.parametrize("ne,nff", [(5120, 256), (6144, 1024), (7168, 768), (256, 14336), (512, 4352), (768, 12288), (8192, 8192)])
def test_moe_one_token_rows_in_several_rounds(be, dtype, ne, nff):
    """Hidden sizes and expert widths beyond 4096 at one token (5120 x 8192, 6144 x 16384, 7168 x 2048,
    4096 x 14336 in files): 80, 96, 112, 224, 68, 192 and 128 units of 64 weights per row run as 4 x 20,
    3 x 32, 2 x 56, 4 x 56, 17 x 4, 3 x 64 and 2 x 64 lanes."""
    n_expert, n_used = 3, 2
    gate, up, down = banks(410, ne, n_expert, nff, dtype, sigma=0.03)
    x = synth_normal_f32(411, ne)
    router = synth_normal_f32(412, n_expert * ne, sigma=0.02)
    got = run_moe(be, x, router, gate, up, down, 1, ne, n_expert, n_used, nff, 1.0, dtype)
    want = orc.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff,
                       gate_dtype=int(dtype), up_dtype=int(dtype), down_dtype=int(dtype))
    check(*got, *want)


@pytest.mark.parametrize("rows", [1, 4])
@pytest.mark.parametrize("dtype", [DType.Q4K, DType.Q6K])
def test_moe_router_reads_another_row_than_the_experts(be, dtype, rows):
    """`router_x` distinct from `x`: the selection comes from one tensor, the expert inputs from
    another (at one token the expert kernels read their row in an order of their own, which the
    router kernel cannot leave for them when its row is a different one)."""
    ne, n_expert, n_used, nff = 1024, 8, 2, 512
    gate, up, down = banks(420, ne, n_expert, nff, dtype, sigma=0.03)
    x = synth_normal_f32(421, rows * ne)
    rx = synth_normal_f32(422, rows * ne)
    router = synth_normal_f32(423, n_expert * ne, sigma=0.05)
    xb, rxb, rb = be.upload_new(x), be.upload_new(rx), be.upload_new(router)
    gb, ub, db = be.upload_new(gate), be.upload_new(up), be.upload_new(down)
    yb, ib, wb = be.alloc(rows * ne * 4), be.alloc(rows * n_used * 4), be.alloc(rows * n_used * 4)
    be.moe_ffn(xb, rb, gb, ub, db, yb, rows=rows, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff, scale=1.0,
               gate_dtype=dtype, up_dtype=dtype, down_dtype=dtype, router_x=rxb, sel_idx=ib, sel_w=wb)
    got = (be.download(yb, np.empty((rows, ne), np.float32)), be.download(ib, np.empty((rows, n_used), np.int32)),
           be.download(wb, np.empty((rows, n_used), np.float32)))
    want = orc.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff,
                       gate_dtype=int(dtype), up_dtype=int(dtype), down_dtype=int(dtype), router_x=rx)
    check(*got, *want)
