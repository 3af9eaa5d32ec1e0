"""Pins the CPU oracle's Op::MoeFfn against a textbook f32 MoE (the reference's own `moe_ref`
test helper, crates/infr-llama/tests/seam_op_parity.rs:1224-1322, restated with numpy) at the
reference's tolerance (1e-4 at rows == 1, :1407-1412), plus routing invariants."""
import numpy as np
import pytest

from oracle import oracle as orc


def moe_ref(x, router, gate, up, down, ne, n_expert, n_used, n_ff, scale):
    """Softmax gating, stable descending top-k, renormalised weights, silu(gate.x)*(up.x), down."""
    f = np.float32
    logits = (router.reshape(n_expert, ne) @ x).astype(f)
    p = np.exp(logits - logits.max()).astype(f)
    p = (p / p.sum(dtype=f)).astype(f)
    idx = sorted(range(n_expert), key=lambda e: -p[e])[:n_used]      # sorted() is stable
    wsum = max(f(sum(p[e] for e in idx)), f(1e-20))
    out = np.zeros(ne, f)
    for e in idx:
        g = gate.reshape(n_expert, n_ff, ne)[e] @ x
        u = up.reshape(n_expert, n_ff, ne)[e] @ x
        act = (g / (1.0 + np.exp(-g)) * u).astype(f)
        out += (p[e] / wsum * scale) * (down.reshape(n_expert, ne, n_ff)[e] @ act)
    return out, idx


def make_banks(seed, ne, n_expert, n_ff, dtype):
    from infr_amd import synth_weight
    gate = synth_weight(dtype, seed, n_expert * n_ff, ne, sigma=0.05)
    up = synth_weight(dtype, seed + 1, n_expert * n_ff, ne, sigma=0.05)
    down = synth_weight(dtype, seed + 2, n_expert * ne, n_ff, sigma=0.05)
    return gate, up, down


@pytest.mark.parametrize("dtype", [orc.Q4_K, orc.Q6_K, orc.Q8_0, orc.Q5_K])
def test_rows1_matches_textbook_moe(dtype):
    ne, n_expert, n_used, n_ff = 256, 8, 2, 256
    rng = np.random.default_rng(4)
    x = rng.standard_normal(ne).astype(np.float32)
    router = (rng.standard_normal(n_expert * ne) * 0.1).astype(np.float32)
    gate, up, down = make_banks(10, ne, n_expert, n_ff, dtype)
    y, idx, w = orc.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=n_expert, n_used=n_used,
                            n_ff_exp=n_ff, scale=1.5, gate_dtype=dtype, up_dtype=dtype, down_dtype=dtype)
    gf, uf, df = (orc.dequant_block(dtype, b) for b in (gate, up, down))
    want, want_idx = moe_ref(x, router, gf, uf, df, ne, n_expert, n_used, n_ff, np.float32(1.5))
    assert list(idx[0]) == want_idx
    assert np.abs(y[0] - want).max() < 1e-4
    # routing invariants: distinct experts, descending probabilities, weights sum to scale
    assert len(set(idx[0])) == n_used and np.all(np.diff(w[0]) <= 0)
    assert abs(float(w[0].sum()) - 1.5) < 1e-5


def test_rows_ge_2_take_the_int8_path_and_stay_close_to_textbook():
    # lib.rs:2359: int8_ok = rows >= 2; the int8 activation error is the reference's ~4e-3 class
    ne, n_expert, n_used, n_ff, rows = 256, 16, 4, 256, 5
    rng = np.random.default_rng(5)
    x = rng.standard_normal(rows * ne).astype(np.float32)
    router = (rng.standard_normal(n_expert * ne) * 0.1).astype(np.float32)
    gate, up, down = make_banks(20, ne, n_expert, n_ff, orc.Q4_K)
    y, idx, w = orc.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=n_ff)
    yref, idx_ref, _ = orc.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=n_expert, n_used=n_used,
                                   n_ff_exp=n_ff, reference_mode=True)
    assert np.array_equal(idx, idx_ref)                   # the f32 router is the same in both modes
    gf, uf, df = (orc.dequant_block(orc.Q4_K, b) for b in (gate, up, down))
    for r in range(rows):
        want, want_idx = moe_ref(x[r * ne:(r + 1) * ne], router, gf, uf, df, ne, n_expert, n_used, n_ff, np.float32(1))
        assert list(idx[r]) == want_idx
        assert np.abs(yref[r] - want).max() < 1e-4                                   # exact mode
        assert np.abs(y[r] - want).max() < 2e-2 * np.abs(want).max()                 # int8 mode
    # and the two modes differ (the int8 path really ran)
    assert not np.array_equal(y, yref)


def test_rows1_is_the_exact_mode():
    ne, n_expert, n_used, n_ff = 256, 8, 2, 256
    rng = np.random.default_rng(6)
    x = rng.standard_normal(ne).astype(np.float32)
    router = (rng.standard_normal(n_expert * ne) * 0.1).astype(np.float32)
    gate, up, down = make_banks(30, ne, n_expert, n_ff, orc.Q4_K)
    a = orc.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=n_ff)[0]
    b = orc.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=n_ff,
                    reference_mode=True)[0]
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_ties_go_to_the_lower_expert_index():
    ne, n_expert, n_used, n_ff = 256, 6, 3, 256
    x = np.ones(ne, np.float32)
    router = np.zeros((n_expert, ne), np.float32)
    router[4] = 0.01          # one clear winner, everything else tied
    gate, up, down = make_banks(40, ne, n_expert, n_ff, orc.Q4_K)
    _, idx, _ = orc.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=n_ff)
    assert list(idx[0]) == [4, 0, 1]


def test_expert_acts_kind_dispatch():
    # crates/infr-cpu/src/moe.rs:42-53
    assert orc.expert_acts_kind(orc.Q4_K, 2048, True) == orc.ACTS_SUPER
    assert orc.expert_acts_kind(orc.Q4_K, 2048, False) == orc.ACTS_RAW
    assert orc.expert_acts_kind(orc.Q8_0, 704, True) == orc.ACTS_BLK32
    assert orc.expert_acts_kind(orc.Q5_K, 2048, True) == orc.ACTS_SUPER
    assert orc.expert_acts_kind(orc.Q5_0, 704, True) == orc.ACTS_BLK32
    assert orc.expert_acts_kind(orc.Q5_0, 704, False) == orc.ACTS_RAW
    assert orc.expert_acts_kind(orc.Q4_0, 2048, True) == orc.ACTS_RAW
    assert orc.expert_acts_kind(orc.Q2_0, 2048, True) == orc.ACTS_RAW
    assert orc.expert_acts_kind(orc.F32, 2048, True) == orc.ACTS_RAW


@pytest.mark.parametrize("dtype,int8", [(orc.Q5_0, True), (orc.Q4_0, False), (orc.Q4_1, False), (orc.Q5_1, False),
                                        (orc.IQ4_NL, False), (orc.Q2_0, False)])
def test_32_block_bank_formats_against_textbook(dtype, int8):
    """moe.rs:42-53 at rows >= 2: Q5_0 banks take per-32 int8 activations (the reference's ~4e-3
    class of error, and a result that differs from the exact mode); the other 32-block formats
    stay on decoded f32 weights x raw activations, i.e. the exact mode bit for bit."""
    ne, n_expert, n_used, n_ff, rows = 256, 8, 2, 256, 3
    rng = np.random.default_rng(7)
    x = rng.standard_normal(rows * ne).astype(np.float32)
    router = (rng.standard_normal(n_expert * ne) * 0.1).astype(np.float32)
    gate, up, down = make_banks(50, ne, n_expert, n_ff, dtype)
    kw = dict(ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=n_ff, gate_dtype=dtype, up_dtype=dtype, down_dtype=dtype)
    y, idx, _ = orc.moe_ffn(x, router, gate, up, down, **kw)
    yref = orc.moe_ffn(x, router, gate, up, down, reference_mode=True, **kw)[0]
    gf, uf, df = (orc.dequant_block(dtype, b) for b in (gate, up, down))
    for r in range(rows):
        want, want_idx = moe_ref(x[r * ne:(r + 1) * ne], router, gf, uf, df, ne, n_expert, n_used, n_ff, np.float32(1))
        assert list(idx[r]) == want_idx
        assert np.abs(yref[r] - want).max() < 1e-4
        assert np.abs(y[r] - want).max() < (2e-2 * np.abs(want).max() if int8 else 1e-4)
    assert np.array_equal(y, yref) != int8
