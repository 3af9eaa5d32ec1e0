"""Op::Linear on random shapes against the CPU oracle: every format, token counts on both sides of
every route's threshold (1, 2..16, 17..32, 33..127, 128.., the per-32 formats' 65), row lengths
that are and are not whole 256s, weight-row windows (`w_off`) into a larger matrix.

The directed tests pin each kernel at the sizes it was written for; this one is for the seams
between them: a threshold off by one, a tile that assumes a multiple it is not given, a row window
that starts inside a tile. Bars are the path's: K-quant outputs bit-identical to the oracle
(same per-block expression, same order), the other formats within rel-L2 <= 1e-4 and
max-abs <= 1e-3 * max|y|. One K-quant route is not bit-identical by design: Q4_K from 128 tokens up may
take the prefill strips, whose f32 epilogue is contracted into fused
multiply-adds (the integers stay exact); it is held to rel-L2 <= 2e-6, fifty times inside the path's bar
and far from what a wrong block, scale or row would give.
"""
import numpy as np
import pytest

from infr_amd import DType, block_layout, synth_normal_f32
from oracle import oracle as orc

pytestmark = pytest.mark.gpu

FORMATS = (DType.Q4K, DType.Q5K, DType.Q6K, DType.Q8_0, DType.Q2_0, DType.Q4_0, DType.Q4_1, DType.Q5_0, DType.Q5_1,
           DType.IQ4NL, DType.F32, DType.F16, DType.BF16, DType.Q2K, DType.Q3K, DType.IQ4XS, DType.TQ2_0, DType.MXFP4,
           DType.NVFP4, DType.TQ1_0)
PLAIN = (DType.F32, DType.F16, DType.BF16)
BIT_IDENTICAL = (DType.Q4K, DType.Q5K, DType.Q6K, DType.Q2K, DType.Q3K, DType.IQ4XS, DType.TQ2_0, DType.TQ1_0) + PLAIN
TOKENS = (1, 1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 24, 31, 32, 33, 40, 63, 64, 65, 66, 96, 127, 128, 129, 130, 200,
          255, 256, 257, 300)


def draw_case(rng):
    dtype = FORMATS[rng.integers(len(FORMATS))]
    unit = 32 if dtype in PLAIN else block_layout(dtype)[0]
    # row lengths: whole 256s mostly, for the 32- and 64-element formats also rows that end inside one
    if unit < 256 and rng.integers(3) == 0:
        in_f = unit * int(rng.integers(1, 1 + 2304 // unit))
    else:
        in_f = 256 * int(rng.integers(1, 10))
    m = int(TOKENS[rng.integers(len(TOKENS))])
    out_f = int(rng.choice([1, 7, 16, 31, 32, 33, 64, 96, 100, 128, 130, 257, 384]))
    if dtype == DType.Q4K and m >= 128 and rng.integers(2):
        out_f = int(rng.choice([2304, 2600, 5100, 6144]))        # enough outputs for the prefill strips
        in_f = 256 * int(rng.integers(1, 5))
    if dtype in (DType.Q2K, DType.Q3K, DType.IQ4XS, DType.TQ2_0, DType.Q5K, DType.Q6K) and m >= 96 and rng.integers(2):
        out_f = int(rng.choice([2304, 2600, 5100]))              # enough outputs for the 128-token tiles
        in_f = 256 * int(rng.integers(1, 5))
    extra_before, extra_after = (int(rng.integers(0, 40)) if rng.integers(2) else 0 for _ in range(2))
    return dtype, m, in_f, out_f, extra_before, extra_after


@pytest.mark.parametrize("seed", range(320))
def test_linear_on_a_random_shape_matches_the_oracle(be, seed):
    rng = np.random.default_rng(0xF00D + seed)
    dtype, m, in_f, out_f, before, after = draw_case(rng)
    rows = before + out_f + after
    # full-range payload bytes (the reference's synth_weight recipe): every code value, every scale
    if dtype in PLAIN:
        w32 = synth_normal_f32(0x5EED + seed, rows * in_f, sigma=0.05)
        w = (w32 if dtype == DType.F32 else w32.astype(np.float16) if dtype == DType.F16
             else (w32.view(np.uint32) >> 16).astype(np.uint16)).view(np.uint8)
    else:
        w = orc.synth_weight(dtype, rows * in_f, 0x5EED + seed)
    x = synth_normal_f32(0xACE + seed, m * in_f)
    if m > 2:
        x[in_f:2 * in_f] = 0.0                     # an all-zero token: scale 0, inverse 0
    case = f"dtype {int(dtype)} m {m} in_f {in_f} out_f {out_f} rows {before}+{out_f}+{after}"
    yb = be.alloc(m * out_f * 4)
    # every third case goes through the entry point that allocates nothing (same kernels, static scratch)
    call = be.linear_noalloc if seed % 3 == 0 else be.linear
    call(dtype, be.upload_new(w), be.upload_new(x), yb, m, in_f, out_f, w_numel=rows * in_f, w_off=before * in_f)
    got = be.download(yb, np.empty((m, out_f), np.float32))
    want = orc.linear(dtype, w, x, m, in_f, out_f, w_numel=rows * in_f, w_off=before * in_f).reshape(m, out_f)
    assert np.isfinite(want).all(), case
    contracted = dtype == DType.Q4K and m >= 128        # (the routes that are still bit-identical pass this bar too)
    if contracted:
        g, t = got.astype(np.float64), want.astype(np.float64)
        rel = np.linalg.norm(g - t) / max(np.linalg.norm(t), 1e-30)
        assert rel <= 2e-6 and np.abs(g - t).max() <= 1e-5 * np.abs(t).max(), f"rel-L2 {rel:.2e}: {case}"
    elif dtype in BIT_IDENTICAL:
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), f"not bit-identical: {case}"
    else:
        g, t = got.astype(np.float64), want.astype(np.float64)
        rel = np.linalg.norm(g - t) / max(np.linalg.norm(t), 1e-30)
        mx = np.abs(g - t).max() / max(np.abs(t).max(), 1e-30)
        assert rel <= 1e-4 and mx <= 1e-3, f"rel-L2 {rel:.2e} max-abs {mx:.2e}: {case}"
    # every fourth quantized case: the per-block integers behind those outputs, exact on every route
    # (one token of Q5_0 multiplies f32 activations: it has no integer stage, as on the CPU; NVFP4 has
    # four integers per block and no stage entry)
    if seed % 4 == 1 and dtype not in PLAIN and dtype != DType.NVFP4 and not (dtype == DType.Q5_0 and m == 1):
        a, b = be.linear_int_stages(dtype, be.upload_new(w), be.upload_new(x), m, in_f, out_f, w_numel=rows * in_f,
                                    w_off=before * in_f)
        oa, ob = orc.linear_int_stages(dtype, w, x, m, in_f, out_f, w_numel=rows * in_f, w_off=before * in_f)
        assert np.array_equal(a, oa), f"first integer stage differs: {case}"
        if dtype in (DType.Q4K, DType.Q5K, DType.Q2K):
            assert np.array_equal(b, ob), f"second integer stage differs: {case}"
