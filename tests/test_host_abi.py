"""CPU-side checks of the drop-in boundary: the shared library loads, exports every symbol the
public header declares, and its host-only pieces (shutdown latch, synthesizers, geometry) behave.
No compute entry point is called here: those need a GPU and fail loudly without one."""
import ctypes
import os
import re

import numpy as np
import pytest

import infr_amd
from infr_amd import backend as B

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    names = set()
    for header in ("infr_hip.h", "infr_gguf.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(infr_(?:hip|synth|block|gguf)_\w+)\s*\(", text))
    return sorted(names)


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(B.LIB_PATH)
    names = declared_symbols()
    assert len(names) >= 60
    for n in names:
        assert hasattr(lib, n), f"{n} is declared under include/ but not exported"
    # and the Python mirror binds exactly that set
    assert sorted(B.SYMBOLS) == names


def test_no_gpu_means_a_loud_backend_error_not_a_fallback():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    with pytest.raises(infr_amd.InfrError) as e:
        infr_amd.HipBackend(0)
    assert e.value.status == infr_amd.Status.Backend
    assert "HIP device" in e.value.msg


def test_shutdown_latch_is_monotonic_and_reports_the_first_signal():
    # crates/infr-core/src/shutdown.rs:61-80
    B.reset_shutdown()
    assert not B.shutdown_requested() and B.shutdown_signal() is None
    assert B.request_shutdown(2) is True
    assert B.request_shutdown(15) is False          # second signal does not re-latch
    assert B.shutdown_requested() and B.shutdown_signal() == 2
    B.reset_shutdown()
    assert not B.shutdown_requested()


def test_block_layouts():
    assert B.block_layout(B.DType.Q8_0) == (32, 34)
    assert B.block_layout(B.DType.Q4K) == (256, 144)
    assert B.block_layout(B.DType.Q6K) == (256, 210)
    assert B.block_layout(B.DType.Q2_0) == (64, 18)
    with pytest.raises(infr_amd.InfrError):
        B.block_layout(99)


def test_synth_is_deterministic_and_thread_count_independent():
    a = infr_amd.synth_weight(B.DType.Q4K, 0, 64, 1024)
    b = infr_amd.synth_weight(B.DType.Q4K, 0, 64, 1024)
    assert np.array_equal(a, b)
    # rows are keyed by (seed, row): a prefix of rows is a prefix of bytes
    c = infr_amd.synth_weight(B.DType.Q4K, 0, 8, 1024)
    assert np.array_equal(a[:c.size], c)
    assert not np.array_equal(a, infr_amd.synth_weight(B.DType.Q4K, 1, 64, 1024))
    x = infr_amd.synth_normal_f32(1, 100_000)
    assert abs(float(x.mean())) < 0.02 and abs(float(x.std()) - 1.0) < 0.02
    with pytest.raises(infr_amd.InfrError):
        infr_amd.synth_weight(B.DType.Q4K, 0, 4, 100)       # ragged in_f is rejected


@pytest.mark.parametrize("dtype,tol", [(B.DType.Q4K, 0.09), (B.DType.Q6K, 0.03), (B.DType.Q8_0, 0.01)])
def test_synth_encoders_reproduce_their_input_distribution(dtype, tol):
    """The encoders are nearest-code quantizers of N(0, 0.02^2): decoding (with the CPU oracle's
    host decode) must give that distribution back within the format's step size."""
    from oracle import oracle as orc
    w = infr_amd.synth_weight(dtype, 3, 32, 2048, sigma=0.02)
    f = orc.dequant_block(int(dtype), w)
    assert abs(float(f.std()) - 0.02) < 0.02 * tol * 2
    assert abs(float(f.mean())) < 2e-4
    assert np.isfinite(f).all()


def test_synth_q2_0_codes_are_ternary():
    w = infr_amd.synth_weight(B.DType.Q2_0, 5, 16, 1024).reshape(-1, 18)
    codes = np.stack([(w[:, 2:] >> s) & 3 for s in (0, 2, 4, 6)])
    assert codes.max() == 2 and set(np.unique(codes)) == {0, 1, 2}
    frac = [(codes == v).mean() for v in (0, 1, 2)]
    assert all(abs(f - 1 / 3) < 0.02 for f in frac)
