"""infr_hip_linear_noalloc: Op::Linear over the library's static device scratch, for callers that
cannot allocate device memory. Its kernels and results are those of infr_hip_linear, so every output
must equal that entry point's bit for bit, on consecutive calls that reuse the scratch (the second
with a smaller input), and the oracle's to the path's bar."""
import numpy as np
import pytest

from infr_amd import DType, InfrError, Status, synth_normal_f32, synth_weight
from oracle import oracle as orc

pytestmark = pytest.mark.gpu


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def both(be, dt, w, x, m, in_f, out_f):
    wb, xb = be.upload_new(w), be.upload_new(x)
    ya, yb = be.alloc(m * out_f * 4), be.alloc(m * out_f * 4)
    be.linear_noalloc(dt, wb, xb, ya, m, in_f, out_f)
    be.linear(dt, wb, xb, yb, m, in_f, out_f)
    return (be.download(ya, np.empty((m, out_f), np.float32)),
            be.download(yb, np.empty((m, out_f), np.float32)))


# (m, in_f, out_f) pairs: the second call of each pair is smaller than the first and lands in the
# scratch the first one left behind. 512 / 40 / 8 / 1 tokens take the four Q4_K routes.
CASES = [
    (DType.Q4K, [(512, 1024, 320), (200, 512, 96)]),
    (DType.Q4K, [(40, 2048, 256), (8, 1024, 64)]),
    (DType.Q4K, [(8, 1024, 64), (1, 1024, 64)]),
    (DType.Q6K, [(96, 1024, 192), (33, 512, 64)]),
    (DType.Q8_0, [(70, 1024, 128), (5, 256, 40)]),
    (DType.Q2_0, [(130, 512, 96), (66, 256, 32)]),
]


@pytest.mark.parametrize("dt,calls", CASES, ids=[f"{c[0].name}-{c[1][0][0]}-{c[1][1][0]}" for c in CASES])
def test_noalloc_equals_linear_on_consecutive_calls(be, dt, calls):
    for i, (m, in_f, out_f) in enumerate(calls):
        w = synth_weight(dt, 500 + i, out_f, in_f, 0.05)
        x = synth_normal_f32(510 + i, m * in_f)
        got, ref = both(be, dt, w, x, m, in_f, out_f)
        assert np.array_equal(bits(got), bits(ref)), f"call {i}: differs from infr_hip_linear"
        rows = sorted({0, m // 2, m - 1})
        want = orc.linear(dt, w, x.reshape(m, in_f)[rows].ravel(), len(rows), in_f, out_f)
        if dt in (DType.Q4K, DType.Q6K) and not (dt == DType.Q4K and m >= 128):
            assert np.array_equal(bits(got[rows]), bits(want)), f"call {i}: differs from the oracle"
        else:
            a, b = got[rows].astype(np.float64).ravel(), want.astype(np.float64).ravel()
            assert np.linalg.norm(a - b) <= 1e-4 * np.linalg.norm(b)
            assert np.abs(a - b).max() <= 1e-3 * np.abs(b).max()


def test_noalloc_rejects_what_the_static_scratch_cannot_hold(be):
    in_f, out_f = 4096, 32
    w = be.upload_new(synth_weight(DType.Q4K, 1, out_f, in_f))
    m_ok, m_big = 1024, 1025                       # 1025 tokens round up to 1056 x 4096 > 4 Mi elements
    x = be.alloc(m_big * in_f * 4)
    y = be.alloc(m_big * out_f * 4)
    be.linear_noalloc(DType.Q4K, w, x, y, m_ok, in_f, out_f)
    with pytest.raises(InfrError) as e:
        be.linear_noalloc(DType.Q4K, w, x, y, m_big, in_f, out_f)
    assert e.value.status == Status.Unsupported and "static scratch" in e.value.msg
    be.sync()


def _free_device_bytes():
    """hipMemGetInfo through the HIP runtime the library itself is linked against."""
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    free, total = ctypes.c_size_t(), ctypes.c_size_t()
    assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
    return free.value


def test_noalloc_leaves_free_device_memory_unchanged(be):
    """A call far larger than any before it on this route must not take device memory: the grow-on-demand
    scratch of infr_hip_linear would have to grow by several MB for it (and does, in the control below)."""
    in_f, out_f = 4096, 64
    w = be.upload_new(synth_weight(DType.Q4K, 2, out_f, in_f))
    m_small, m_big = 128, 1000
    x = be.upload_new(synth_normal_f32(3, m_big * in_f))
    y = be.alloc(m_big * out_f * 4)
    be.linear_noalloc(DType.Q4K, w, x, y, m_small, in_f, out_f)    # the route's kernels are loaded now
    be.sync()
    before = _free_device_bytes()
    be.linear_noalloc(DType.Q4K, w, x, y, m_big, in_f, out_f)
    be.sync()
    assert _free_device_bytes() == before
    got = be.download(y, np.empty((m_big, out_f), np.float32))
    want = orc.linear(DType.Q4K, synth_weight(DType.Q4K, 2, out_f, in_f), synth_normal_f32(3, m_big * in_f)[:2 * in_f], 2, in_f, out_f)
    assert np.array_equal(bits(got[:2]), bits(want))
