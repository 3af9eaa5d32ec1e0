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


@pytest.mark.parametrize("dtype,tol", [(B.DType.Q4K, 0.09), (B.DType.Q6K, 0.03), (B.DType.Q8_0, 0.01),
                                       (B.DType.Q2K, 0.06), (B.DType.Q3K, 0.02), (B.DType.IQ4XS, 0.03),
                                       (B.DType.MXFP4, 0.08), (B.DType.NVFP4, 0.06)])
def test_synth_encoders_reproduce_their_input_distribution(dtype, tol):
    """The encoders are nearest-code quantizers of N(0, 0.02^2): decoding (with the CPU oracle's
    host decode) must give that distribution back within the format's step size."""
    from oracle import oracle as orc
    w = infr_amd.synth_weight(dtype, 3, 32, 2048, sigma=0.02)
    f = orc.dequant_block(int(dtype), w)
    assert abs(float(f.std()) - 0.02) < 0.02 * tol * 2
    assert abs(float(f.mean())) < 2e-4
    assert np.isfinite(f).all()


def test_synth_tq1_0_digits_are_uniform():
    from oracle import oracle as orc
    w = infr_amd.synth_weight(B.DType.TQ1_0, 5, 16, 1024)
    f = orc.dequant_block(orc.TQ1_0, w).reshape(-1, 256)
    d = np.abs(f).max(axis=1, keepdims=True)
    digits = np.rint(f / d).astype(int) + 1
    assert set(np.unique(digits)) == {0, 1, 2}
    assert all(abs((digits == v).mean() - 1 / 3) < 0.02 for v in (0, 1, 2))


@pytest.mark.parametrize("dtype", [B.DType.Q2_0, B.DType.TQ2_0])
def test_synth_ternary_codes(dtype):
    w = infr_amd.synth_weight(dtype, 5, 16, 1024)
    w = w.reshape(-1, 18)[:, 2:] if dtype == B.DType.Q2_0 else w.reshape(-1, 66)[:, :64]
    codes = np.stack([(w >> s) & 3 for s in (0, 2, 4, 6)])
    assert codes.max() == 2 and set(np.unique(codes)) == {0, 1, 2}
    frac = [(codes == v).mean() for v in (0, 1, 2)]
    assert all(abs(f - 1 / 3) < 0.02 for f in frac)


# ---- the Rust mirror in the binding notes against the C header's layout ----

BINDING_NOTES = "INTEGRATION.md"  # the file that holds the reference-side shim's source text

_RUST_TYPES = {"i32": (4, 4), "u32": (4, 4), "f32": (4, 4), "u64": (8, 8), "i64": (8, 8), "usize": (8, 8)}


def _rust_repr_c_structs():
    """name -> [(field, size, align)] for every `#[repr(C)] ... pub struct` of the shim's source text."""
    text = open(os.path.join(ROOT, BINDING_NOTES)).read()
    out = {}
    for name, body in re.findall(r"#\[repr\(C\)\][^{;]*?pub struct (\w+)\s*\{(.*?)\}", text, flags=re.S):
        body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
        body = re.sub(r"//[^\n]*", "", body)
        fields = []
        for decl in [d.strip() for d in body.split(",") if d.strip()]:
            fname, ftype = [t.strip() for t in decl.split(":", 1)]
            arr = re.fullmatch(r"\[(\w+);\s*(\d+)\]", ftype)
            if arr:
                size, align = (1, 1) if arr.group(1) in ("c_char", "u8", "i8") else _RUST_TYPES[arr.group(1)]
                fields.append((fname, size * int(arr.group(2)), align))
            elif ftype in _RUST_TYPES:
                fields.append((fname, *_RUST_TYPES[ftype]))
            else:
                fields.append((fname, ftype, None))        # a nested struct, resolved below
        out[name] = fields
    return out


def _repr_c_layout(structs, name):
    """offsets, size and alignment of a #[repr(C)] struct: C's rules, which repr(C) promises."""
    off, max_align, offsets = 0, 1, {}
    for fname, size, align in structs[name]:
        if align is None:
            _, size, align = _repr_c_layout(structs, size)
        off = (off + align - 1) // align * align
        offsets[fname] = off
        off += size
        max_align = max(max_align, align)
    return offsets, (off + max_align - 1) // max_align * max_align, max_align


def _c_layout(tmp_path, ctype, fields):
    """offsetof of every field and sizeof, as gcc lays out the public header's struct."""
    import subprocess
    src = tmp_path / f"layout_{ctype}.c"
    lines = "\n".join(f'    printf("{f} %zu\\n", offsetof({ctype}, {f}));' for f in fields)
    src.write_text(f'#include <stddef.h>\n#include <stdio.h>\n#include "infr_hip.h"\nint main(void) {{\n{lines}\n'
                   f'    printf("sizeof %zu\\n", sizeof({ctype}));\n    return 0;\n}}\n')
    exe = tmp_path / f"layout_{ctype}"
    subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()
    return dict(zip(out[0::2], map(int, out[1::2])))


@pytest.mark.parametrize("rust,ctype", [("HipOp", "infr_hip_op_t"), ("HipMoe", "infr_hip_moe_params_t"),
                                        ("HipCaps", "infr_hip_caps_t")])
def test_rust_mirror_structs_match_the_c_header(tmp_path, rust, ctype):
    """The `impl Backend for HipBackend` shim cannot be compiled here (no Rust toolchain); what can be
    checked is that its #[repr(C)] structs still describe the header's structs field by field."""
    structs = _rust_repr_c_structs()
    assert rust in structs, f"{BINDING_NOTES} no longer declares {rust}"
    offsets, size, _ = _repr_c_layout(structs, rust)
    c = _c_layout(tmp_path, ctype, list(offsets))          # a field the header lacks fails to compile
    assert c.pop("sizeof") == size, f"{rust} and {ctype} differ in size"
    assert c == offsets
    # and the header has no field the mirror lacks: the ctypes mirror lists them all
    ct = {"HipOp": B._Op, "HipMoe": B._MoeParams, "HipCaps": B._Caps}[rust]
    assert [f[0] for f in ct._fields_] == list(offsets)
    assert ctypes.sizeof(ct) == size


def test_shim_moe_arm_names_every_field_of_the_op():
    """The shim's `Op::MoeFfn { .. }` pattern must bind every field of the reference's op
    (crates/infr-core/src/graph.rs:918-1011) and carry each into `HipMoe` or a tensor id: a `..` in the
    pattern would let a field that changes the arithmetic (gating, weight_before, act, ...) vanish on the
    way to the library, which can only refuse what it is told about."""
    import re
    text = open(os.path.join(ROOT, BINDING_NOTES)).read()
    m = re.search(r"Op::MoeFfn \{([^}]*)\} => ops\.push\(HipOp \{(.*?)\.\.Default::default\(\) \}\),", text, re.S)
    assert m, f"{BINDING_NOTES} no longer holds the MoeFfn arm"
    pattern, body = m.group(1), m.group(2)
    assert ".." not in pattern, "the MoeFfn pattern skips fields with `..`"
    bound = {f.strip().split(":")[0].strip() for f in pattern.split(",") if f.strip()}
    op_fields = {"x", "router_x", "router", "gate_exps", "up_exps", "down_exps", "down_scale", "fused_gate_up", "dst",
                 "ne", "n_expert", "n_used", "n_ff_exp", "scale", "act", "swiglu_clamp", "gating", "norm_w",
                 "weight_before", "ep_band", "exp_probs_b", "n_expert_groups", "n_expert_groups_used", "expert_ids"}
    assert bound == op_fields
    for f in op_fields:                          # and each one is used on the right-hand side
        assert re.search(rf"\b{f}\b", body), f"{f} is bound but not passed on"
    # the header documents what each flag means and that unsupported settings are refused
    header = open(os.path.join(ROOT, "include", "infr_hip.h")).read()
    for f in ("act", "gating", "norm_w", "weight_before", "fused_gate_up", "has_clamp", "n_expert_groups",
              "n_expert_groups_used", "has_down_scale", "has_exp_probs_b", "has_expert_ids", "has_ep_band"):
        assert re.search(rf"\b{f}\b", header), f
