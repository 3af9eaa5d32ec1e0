"""Op::MoeFfn on random shapes and bank formats against the CPU oracle: row counts on both sides of
every route's threshold (one row; a few rows: per-pair kernels and the fused down launch; from an
average of two or four pairs per expert the bucketed int8-MFMA tiles), every bank format in every
position, hidden sizes and expert widths of one to several 256-blocks (one case in four beyond
4096 columns, where the one-token kernels walk a row in rounds), up to 32 experts per token.

Bars: the expert selection equals the oracle's, its weights agree to 1e-5 relative, outputs within
rel-L2 <= 1e-4 and max-abs <= 1e-3 * max|y| (crates/infr-cpu/src/lib.rs:2334-2541, moe.rs:42-53).

There is one bar for every case. From two rows up the gated activation is quantized to int8 for the
down bank (lib.rs:2824-2892), so a gate / up output that differed from the CPU's in its last bit could
move one activation across a rounding boundary and with it a code - 1 / 127 of its chunk's maximum in
every output of that pair, 1e-4..7e-4 of the whole output. The device therefore adds the per-block
terms of every int8 bank format in the scalar CPU kernel's order (ascending blocks, kernels.rs:1170-1187):
K-quants through their ordered sums, Q8_0 and Q5_0 through a per-lane ordered sum in the per-pair
kernels and block-by-block accumulation in the bucketed tiles. The directed seeds below are cases of
a sweep of seeds 80..4300 that sat at 1.0e-4..8.6e-4 while Q8_0 / Q5_0 terms were added in a tree
(twenty of 460 such cases; none of 1015 up to seed 9000 with the ordered sums).
"""
import numpy as np
import pytest

from infr_amd import DType, synth_normal_f32, synth_weight
from oracle import oracle as orc

pytestmark = pytest.mark.gpu

BANK_FORMATS = (DType.Q4K, DType.Q4K, DType.Q5K, DType.Q6K, DType.Q8_0, DType.Q5_0, DType.Q4_0, DType.Q4_1,
                DType.Q5_1, DType.IQ4NL, DType.Q2_0, DType.F32, DType.F16, DType.BF16)


def bank(dtype, seed, rows, in_f):
    """N(0, 0.05^2) rows as raw bytes of `dtype`; the float formats are plain arrays (f16 rounded to
    nearest, bf16 the top half of the f32 pattern, crates/infr-gguf/src/dequant.rs:19-22)."""
    if dtype in (DType.F32, DType.F16, DType.BF16):
        w = synth_normal_f32(seed, rows * in_f, sigma=0.05)
        if dtype == DType.F16:
            return w.astype(np.float16).view(np.uint8)
        if dtype == DType.BF16:
            return (w.view(np.uint32) >> 16).astype(np.uint16).view(np.uint8)
        return w.view(np.uint8)
    return synth_weight(dtype, seed, rows, in_f, 0.05)


def draw_case(rng):
    while True:
        ne = int(rng.choice([256, 512, 768, 1024, 1024, 2048, 4096]))
        nff = 256 * int(rng.integers(1, 4))
        long_rows = int(rng.integers(8))        # one case in four: rows beyond 4096 columns on one side
        if long_rows == 0:
            ne = int(rng.choice([4352, 5120, 6144, 7168, 8192]))
        elif long_rows == 1:
            ne, nff = int(rng.choice([256, 512])), int(rng.choice([4352, 5120, 8192, 14336]))
        n_expert = int(rng.choice([2, 4, 8, 16, 32, 48, 72, 128]))
        if n_expert * nff * ne <= 1 << 24:      # banks of at most 16 M weights each
            break
    n_used = int(rng.choice([u for u in (1, 1, 2, 3, 4, 8, 20, 32) if u <= n_expert]))
    rows = int(rng.choice([1, 1, 2, 3, 4, 5, 8, 9, 16, 17, 31, 33, 48, 64, 70, 130, 200]))
    if rng.integers(2):
        dts = (BANK_FORMATS[rng.integers(len(BANK_FORMATS))],) * 3          # one format, as most files have
    else:
        dts = tuple(BANK_FORMATS[rng.integers(len(BANK_FORMATS))] for _ in range(3))
    scale = float(rng.choice([1.0, 1.0, 2.5]))
    return rows, ne, n_expert, n_used, nff, dts, scale


# seeds of the wide sweep whose Q8_0 / Q5_0 gate / up sums used to flip an activation code (see above)
DIRECTED_SEEDS = (207, 524, 750, 841, 1103, 1929, 2027, 2242, 2462, 2564, 2588, 2834, 3113, 3188, 3513, 3549, 3764, 3816,
                  4108, 4205,
                  4219, 5853, 5940)     # and three with 14336-wide Q8_0 / Q5_0 down rows (seven wave steps per row)


@pytest.mark.parametrize("seed", list(range(80)) + list(DIRECTED_SEEDS))
def test_moe_ffn_on_a_random_shape_matches_the_oracle(be, seed):
    rng = np.random.default_rng(0xB0A + seed)
    rows, ne, n_expert, n_used, nff, dts, scale = draw_case(rng)
    case = f"rows {rows} ne {ne} experts {n_expert} top-{n_used} nff {nff} banks {[int(d) for d in dts]} scale {scale}"
    gate = bank(dts[0], 3 * seed + 1, n_expert * nff, ne)
    up = bank(dts[1], 3 * seed + 2, n_expert * nff, ne)
    down = bank(dts[2], 3 * seed + 3, n_expert * ne, nff)
    x = synth_normal_f32(0xC0 + seed, rows * ne)
    router = synth_normal_f32(0xD0 + seed, n_expert * ne, sigma=0.05)
    xb, rb = be.upload_new(x), be.upload_new(router)
    gb, ub, db = be.upload_new(gate), be.upload_new(up), be.upload_new(down)
    yb = be.alloc(rows * ne * 4)
    ib, wb = be.alloc(rows * n_used * 4), be.alloc(rows * n_used * 4)
    be.moe_ffn(xb, rb, gb, ub, db, yb, rows=rows, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff, scale=scale,
               gate_dtype=dts[0], up_dtype=dts[1], down_dtype=dts[2], sel_idx=ib, sel_w=wb)
    y = be.download(yb, np.empty((rows, ne), np.float32))
    idx = be.download(ib, np.empty((rows, n_used), np.int32))
    w = be.download(wb, np.empty((rows, n_used), np.float32))
    oy, oidx, ow = orc.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff,
                               scale=scale, gate_dtype=int(dts[0]), up_dtype=int(dts[1]), down_dtype=int(dts[2]))
    assert np.array_equal(idx, oidx), f"expert selection differs: {case}"
    assert np.allclose(w, ow, rtol=1e-5, atol=0), f"selection weights differ: {case}"
    a, b = y.astype(np.float64).ravel(), oy.astype(np.float64).ravel()
    assert np.abs(b).max() > 1e-6, f"vacuous: {case}"
    rel = np.linalg.norm(a - b) / np.linalg.norm(b)
    mx = np.abs(a - b).max() / np.abs(b).max()
    assert rel <= 1e-4 and mx <= 1e-3, f"rel-L2 {rel:.2e} max-abs {mx:.2e}: {case}"
