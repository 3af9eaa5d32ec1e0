"""The C++ host side (include/infr_hip.hpp) and its seam tests (tests/cpp/op_parity.cpp: the
reference's op-parity sweeps restated over infr::HipBackend, scored against the CPU oracle).
Without a GPU: the test program builds against the C ABI, lists its tests, and exits with the
"no device" status instead of computing anything. With one: every test of the program passes."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CPP = os.path.join(ROOT, "tests", "cpp")
EXE = os.path.join(CPP, "_build", "op_parity")

TESTS = [
    "hip_backend_honours_the_seam_contract",
    "hip_linear_all_weight_quants_match_the_host_oracle",
    "hip_linear_matches_the_cpu_production_arm",
    "hip_linear_batch_rows_equal_single_rows",
    "hip_linear_w_off_slices_a_concatenated_weight",
    "hip_decoder_layer_graph_matches_the_cpu_arms",
    "hip_moe_ffn_matches_the_cpu_arm",
    "hip_embed_gather_equals_the_host_decode",
]


def exe():
    if not os.path.exists(EXE):   # built by __graft_entry__.build(); here only if nothing is
        import infr_amd
        from oracle import oracle  # noqa: F401  (builds the oracle library when it is missing)
        infr_amd.load_library()
        subprocess.run(["make", "-C", CPP], check=True, capture_output=True)
    return EXE


def test_program_builds_and_lists_its_tests():
    out = subprocess.run([exe(), "--list"], capture_output=True, text=True, check=True).stdout.split()
    assert out == TESTS


def test_without_a_device_it_refuses_to_run():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    r = subprocess.run([exe()], capture_output=True, text=True)
    assert r.returncode == 99 and "no usable gfx950 device" in r.stdout


@pytest.fixture(scope="module")
def run():
    print("running", EXE, flush=True)
    r = subprocess.run([exe()], capture_output=True, text=True, timeout=600)
    return r


@pytest.mark.gpu
@pytest.mark.parametrize("name", TESTS)
def test_cpp_seam(run, name):
    assert f"test {name} ... ok" in run.stdout, run.stdout[-6000:] + run.stderr[-2000:]


@pytest.mark.gpu
def test_cpp_seam_exit_status(run):
    assert run.returncode == 0, run.stdout[-6000:] + run.stderr[-2000:]
    assert f"{len(TESTS)} passed; 0 failed" in run.stdout
