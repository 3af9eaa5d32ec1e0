"""Build the gfx950 shared library ``infr_amd/libinfr_hip.so`` with hipcc.

One translation unit per kernel family plus the C-ABI layer and the host-side input
synthesizers, linked into a single shared object whose exported symbols are exactly the ones
``include/infr_hip.h`` declares. hipcc cross-compiles for gfx950 without a GPU present.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libinfr_hip.so")
OBJ = os.path.join(HERE, "build")

SOURCES = ["backend.hip", "quant_act.hip", "gemv.hip", "gemv_fmt_kquant.hip", "gemv_fmt_blk32.hip", "gemv_fmt_q5k.hip", "gemv_fmt_q23k.hip", "gemv_fmt_tq.hip", "gemv_fmt_iq4xs_fp4.hip", "gemv_fmt_nib4.hip", "gemv_fmt_nib5.hip", "gemv_fmt_pair.hip", "gemv_f32act.hip", "mmq.hip", "mmq_q4k_strip.hip", "mmq_q5k.hip", "mmq_iq4xs.hip", "mmq_q2k.hip", "mmq_q3k.hip", "mmq_q6k.hip", "mmq_q8_0.hip", "mmq_nib32.hip", "mmq_gathered.hip", "moe.hip", "elementwise.hip", "embed.hip", "synth.cpp", "gguf.cpp"]

# -ffp-contract=off: the f32 epilogues restate infr-cpu's expressions, which never fuse a multiply
# into an add; -packed-fp32-ops off: packed FP32 forms are not used on this hardware pool.
DEVICE_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wno-unused-function",
    # keep MFMA accumulators in VGPRs: the epilogues read every accumulator with VALU
    # instructions, and AGPR-resident results would each cost a v_accvgpr_read first
    "-mllvm", "-amdgpu-mfma-vgpr-form",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the gfx950 library cannot be built")
    return exe


def _compile(src: str, extra_flags: tuple = (), obj_dir: str = OBJ) -> str:
    obj = os.path.join(obj_dir, os.path.splitext(src)[0] + ".o")
    cmd = [hipcc(), *DEVICE_FLAGS, *extra_flags, "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{r.stderr[-4000:]}")
    return obj


def build(verbose: bool = False, lib: str = LIB, extra_flags: tuple = (), obj_dir: str = OBJ) -> str:
    """Compiles every source and links ``lib``. ``extra_flags`` / ``obj_dir`` serve builds of a
    variant of the library beside the product's (the defaults are the product)."""
    os.makedirs(obj_dir, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(lambda src: _compile(src, tuple(extra_flags), obj_dir), SOURCES))
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr[-4000:]}")
    if verbose:
        print(f"built {lib}")
    return lib


if __name__ == "__main__":
    build(verbose=True)
    sys.exit(0)
