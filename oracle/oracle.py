"""ctypes/numpy front end of the CPU oracle (``libinfr_cpu_oracle.so``).

TEST INFRASTRUCTURE ONLY: a restatement of infr-cpu's quantized Op::Linear / Op::MoeFfn path used
as the checker by the tests, the smoke check and the benchmark's CPU-baseline leg. The GPU library
never imports this module. Each wrapper maps 1:1 onto a C function whose header comment cites the
reference file:line it follows.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from dataclasses import dataclass

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libinfr_cpu_oracle.so")

F32, F16, Q8_0, Q4_K, Q6_K, Q2_0 = 0, 1, 8, 12, 14, 42
Q4_0, Q4_1, Q5_0, Q5_1, Q5_K, IQ4_NL = 2, 3, 6, 7, 13, 20
Q2_K, Q3_K = 10, 11
IQ4_XS = 23
MXFP4, NVFP4 = 39, 40
TQ1_0, TQ2_0 = 34, 35
BF16 = 30
KVALUES_IQ4NL = (-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113)
ACTS_SUPER, ACTS_BLK32, ACTS_RAW = 0, 1, 2


def build() -> str:
    """Compile the oracle with its Makefile (gcc, -ffp-contract=off)."""
    subprocess.run(["make", "-C", _HERE, "-B"], check=True, capture_output=True)
    return _LIB_PATH


def _load() -> C.CDLL:
    if not os.path.exists(_LIB_PATH):
        build()
    return C.CDLL(_LIB_PATH)


_lib = _load()

_u8p = C.POINTER(C.c_uint8)
_i8p = C.POINTER(C.c_int8)
_i32p = C.POINTER(C.c_int32)
_f32p = C.POINTER(C.c_float)


def _p(a, t):
    return None if a is None else a.ctypes.data_as(t)


def _sig(name, res, *args):
    f = getattr(_lib, name)
    f.restype = res
    f.argtypes = list(args)
    return f


_block_layout = _sig("orc_block_layout", C.c_int, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int))
_f16_to_f32 = _sig("orc_f16_bits_to_f32", C.c_float, C.c_uint16)
_f32_to_f16 = _sig("orc_f32_to_f16_bits", C.c_uint16, C.c_float)
_k4 = _sig("orc_k4", None, C.c_int, _u8p, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32))
_dequant = _sig("orc_dequant_block", C.c_int, C.c_int, _u8p, C.c_size_t, _f32p)
_qq8 = _sig("orc_quantize_q8", None, _f32p, C.c_size_t, _i8p, _f32p, _i32p, _i32p)
_qq832 = _sig("orc_quantize_q8_32", None, _f32p, C.c_size_t, _i8p, _f32p, _i32p)
_vd_q4k = _sig("orc_vec_dot_q4k", C.c_float, _u8p, _i8p, _f32p, _i32p, C.c_size_t, _i32p, _i32p)
_vd_q6k = _sig("orc_vec_dot_q6k", C.c_float, _u8p, _i8p, _f32p, C.c_size_t, _i32p)
_vd_q80 = _sig("orc_vec_dot_q8_0", C.c_float, _u8p, _i8p, _f32p, C.c_size_t, _i32p)
_vd_q20 = _sig("orc_vec_dot_q2_0", C.c_float, _u8p, _i8p, _f32p, _i32p, C.c_size_t, _i32p)
_vd_q5k = _sig("orc_vec_dot_q5k", C.c_float, _u8p, _i8p, _f32p, _i32p, C.c_size_t, _i32p, _i32p)
_vd_q2k = _sig("orc_vec_dot_q2k", C.c_float, _u8p, _i8p, _f32p, _i32p, C.c_size_t, _i32p, _i32p)
_vd_q3k = _sig("orc_vec_dot_q3k", C.c_float, _u8p, _i8p, _f32p, _i32p, C.c_size_t, _i32p)
_q3k_scales = _sig("orc_q3k_scales", None, _u8p, C.POINTER(C.c_int16))
_vd_iq4xs = _sig("orc_vec_dot_iq4xs", C.c_float, _u8p, _i8p, _f32p, C.c_size_t, _i32p)
_iq4xs_scale = _sig("orc_iq4xs_scale", C.c_int, C.c_uint32, _u8p, C.c_int)
_vd_tq1_0 = _sig("orc_vec_dot_tq1_0", C.c_float, _u8p, _i8p, _f32p, C.c_size_t, _i32p)
_tq1_digit = _sig("orc_tq1_0_digit", C.c_int, _u8p, C.c_int)
_vd_tq2_0 = _sig("orc_vec_dot_tq2_0", C.c_float, _u8p, _i8p, _f32p, C.c_size_t, _i32p)
_vd_mxfp4 = _sig("orc_vec_dot_mxfp4", C.c_float, _u8p, _i8p, _f32p, C.c_size_t, _i32p)
_vd_nvfp4 = _sig("orc_vec_dot_nvfp4", C.c_float, _u8p, _i8p, _f32p, C.c_size_t, _i32p)
_e8m0 = _sig("orc_e8m0_half", C.c_float, C.c_uint8)
_ue4m3 = _sig("orc_ue4m3_half", C.c_float, C.c_uint8)
_vd_b32 = _sig("orc_vec_dot_blk32", C.c_float, C.c_int, _u8p, _i8p, _f32p, _i32p, C.c_size_t, _i32p)
_embed = _sig("orc_embed_gather", C.c_int, C.c_int, _u8p, C.c_size_t, C.c_size_t, _i32p, C.c_size_t, C.c_size_t,
              C.c_float, _f32p)
_dot = _sig("orc_dot", C.c_float, _f32p, _f32p, C.c_size_t)
_silu = _sig("orc_silu", C.c_float, C.c_float)
_linear = _sig("orc_linear", C.c_int, C.c_int, _u8p, C.c_size_t, C.c_size_t, C.c_size_t, _f32p,
               _f32p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_int, C.c_int)
_linear_int = _sig("orc_linear_int_stages", C.c_int, C.c_int, _u8p, C.c_size_t, C.c_size_t,
                   C.c_size_t, _f32p, C.c_size_t, C.c_size_t, C.c_size_t, _i32p, _i32p)
_ref_f64 = _sig("orc_ref_linear_f64", None, _f32p, _f32p, C.c_size_t, C.c_size_t, C.c_size_t, _f32p)
_acts_kind = _sig("orc_expert_acts_kind", C.c_int, C.c_int, C.c_size_t, C.c_int)
_lcg = _sig("orc_lcg_bytes", None, C.c_uint32, C.c_size_t, _u8p)
_gen = _sig("orc_gen_f32", None, C.c_size_t, C.c_size_t, _f32p)
_synth = _sig("orc_synth_weight", C.c_size_t, C.c_int, C.c_size_t, C.c_uint32, _u8p)
_detb = _sig("orc_det_bytes", None, C.c_size_t, C.c_uint64, _u8p)
_detx = _sig("orc_det_x", None, C.c_size_t, C.c_uint64, _f32p)
_maxthr = _sig("orc_max_threads", C.c_int)


class _MoeParams(C.Structure):
    _fields_ = [("ne", C.c_uint32), ("n_expert", C.c_uint32), ("n_used", C.c_uint32),
                ("n_ff_exp", C.c_uint32), ("rows", C.c_uint32), ("scale", C.c_float),
                ("router_dtype", C.c_int), ("gate_dtype", C.c_int), ("up_dtype", C.c_int),
                ("down_dtype", C.c_int), ("reference_mode", C.c_int),
                ("act", C.c_int), ("gating", C.c_int), ("norm_w", C.c_int), ("weight_before", C.c_int),
                ("fused_gate_up", C.c_int), ("has_clamp", C.c_int), ("clamp", C.c_float),
                ("n_expert_groups", C.c_uint32), ("n_expert_groups_used", C.c_uint32)]


GATING_SOFTMAX, GATING_SIGMOID, GATING_SQRT_SOFTPLUS = 0, 1, 2

_moe = _sig("orc_moe_ffn", C.c_int, C.POINTER(_MoeParams), _f32p, _f32p, _u8p, C.c_size_t, _u8p,
            C.c_size_t, _u8p, C.c_size_t, _u8p, C.c_size_t, _f32p, _i32p, _f32p, C.c_int, _f32p, _f32p, _i32p)


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


def block_layout(dtype: int) -> tuple[int, int]:
    e, b = C.c_int(), C.c_int()
    if not _block_layout(dtype, C.byref(e), C.byref(b)):
        raise ValueError(f"unknown dtype {dtype}")
    return e.value, b.value


def f16_bits_to_f32(h: int) -> float:
    return float(_f16_to_f32(h))


def f32_to_f16_bits(f: float) -> int:
    return int(_f32_to_f16(np.float32(f)))


def k4(j: int, scales) -> tuple[int, int]:
    s = _c(scales, np.uint8)
    sc, m = C.c_uint32(), C.c_uint32()
    _k4(j, _p(s, _u8p), C.byref(sc), C.byref(m))
    return sc.value, m.value


def dequant_block(dtype: int, raw) -> np.ndarray:
    raw = _c(raw, np.uint8)
    e, b = block_layout(dtype)
    out = np.empty(raw.size // b * e, np.float32)
    if _dequant(dtype, _p(raw, _u8p), raw.size, _p(out, _f32p)) != 0:
        raise ValueError(f"dequant_block: unsupported dtype {dtype}")
    return out


@dataclass
class Q8:
    """crates/infr-cpu/src/quant.rs:8-25"""
    qs: np.ndarray
    d: np.ndarray
    bsums: np.ndarray
    bsums16: np.ndarray


@dataclass
class Q8x32:
    """crates/infr-cpu/src/quant.rs:90-95"""
    qs: np.ndarray
    d: np.ndarray
    bsum: np.ndarray


def quantize_q8(x) -> Q8:
    x = _c(x, np.float32).ravel()
    nb = x.size // 256
    q = Q8(np.empty(nb * 256, np.int8), np.empty(nb, np.float32), np.empty(nb * 8, np.int32),
           np.empty(nb * 16, np.int32))
    _qq8(_p(x, _f32p), x.size, _p(q.qs, _i8p), _p(q.d, _f32p), _p(q.bsums, _i32p),
         _p(q.bsums16, _i32p))
    return q


def quantize_q8_32(x) -> Q8x32:
    x = _c(x, np.float32).ravel()
    nb = x.size // 32
    q = Q8x32(np.empty(nb * 32, np.int8), np.empty(nb, np.float32), np.empty(nb, np.int32))
    _qq832(_p(x, _f32p), x.size, _p(q.qs, _i8p), _p(q.d, _f32p), _p(q.bsum, _i32p))
    return q


def vec_dot_q4k(row, q8: Q8, in_f: int, stages: bool = False):
    row = _c(row, np.uint8)
    nb = in_f // 256
    sd = np.empty(nb, np.int32) if stages else None
    sm = np.empty(nb, np.int32) if stages else None
    y = _vd_q4k(_p(row, _u8p), _p(q8.qs, _i8p), _p(q8.d, _f32p), _p(q8.bsums, _i32p), in_f,
                _p(sd, _i32p), _p(sm, _i32p))
    return (np.float32(y), sd, sm) if stages else np.float32(y)


def vec_dot_q6k(row, q8: Q8, in_f: int, stages: bool = False):
    row = _c(row, np.uint8)
    isum = np.empty(in_f // 256, np.int32) if stages else None
    y = _vd_q6k(_p(row, _u8p), _p(q8.qs, _i8p), _p(q8.d, _f32p), in_f, _p(isum, _i32p))
    return (np.float32(y), isum) if stages else np.float32(y)


def vec_dot_q8_0(row, q8: Q8, in_f: int, stages: bool = False):
    row = _c(row, np.uint8)
    ip = np.empty(in_f // 32, np.int32) if stages else None
    y = _vd_q80(_p(row, _u8p), _p(q8.qs, _i8p), _p(q8.d, _f32p), in_f, _p(ip, _i32p))
    return (np.float32(y), ip) if stages else np.float32(y)


def vec_dot_q2_0(row, q8: Q8x32, in_f: int, stages: bool = False):
    row = _c(row, np.uint8)
    ip = np.empty(in_f // 32, np.int32) if stages else None
    y = _vd_q20(_p(row, _u8p), _p(q8.qs, _i8p), _p(q8.d, _f32p), _p(q8.bsum, _i32p), in_f,
                _p(ip, _i32p))
    return (np.float32(y), ip) if stages else np.float32(y)


def vec_dot_q5k(row, q8: Q8, in_f: int, stages: bool = False):
    row = _c(row, np.uint8)
    nb = in_f // 256
    sd = np.empty(nb, np.int32) if stages else None
    sm = np.empty(nb, np.int32) if stages else None
    y = _vd_q5k(_p(row, _u8p), _p(q8.qs, _i8p), _p(q8.d, _f32p), _p(q8.bsums, _i32p), in_f,
                _p(sd, _i32p), _p(sm, _i32p))
    return (np.float32(y), sd, sm) if stages else np.float32(y)


def vec_dot_q2k(row, q8: Q8, in_f: int, stages: bool = False):
    row = _c(row, np.uint8)
    nb = in_f // 256
    sd = np.empty(nb, np.int32) if stages else None
    sm = np.empty(nb, np.int32) if stages else None
    y = _vd_q2k(_p(row, _u8p), _p(q8.qs, _i8p), _p(q8.d, _f32p), _p(q8.bsums16, _i32p), in_f,
                _p(sd, _i32p), _p(sm, _i32p))
    return (np.float32(y), sd, sm) if stages else np.float32(y)


def vec_dot_q3k(row, q8: Q8, in_f: int, stages: bool = False):
    row = _c(row, np.uint8)
    isum = np.empty(in_f // 256, np.int32) if stages else None
    y = _vd_q3k(_p(row, _u8p), _p(q8.qs, _i8p), _p(q8.d, _f32p), _p(q8.bsums16, _i32p), in_f, _p(isum, _i32p))
    return (np.float32(y), isum) if stages else np.float32(y)


def vec_dot_iq4xs(row, q8: Q8, in_f: int, stages: bool = False):
    row = _c(row, np.uint8)
    isum = np.empty(in_f // 256, np.int32) if stages else None
    y = _vd_iq4xs(_p(row, _u8p), _p(q8.qs, _i8p), _p(q8.d, _f32p), in_f, _p(isum, _i32p))
    return (np.float32(y), isum) if stages else np.float32(y)


def vec_dot_tq1_0(row, q8: Q8, in_f: int, stages: bool = False):
    row = _c(row, np.uint8)
    ip = np.empty(in_f // 256, np.int32) if stages else None
    y = _vd_tq1_0(_p(row, _u8p), _p(q8.qs, _i8p), _p(q8.d, _f32p), in_f, _p(ip, _i32p))
    return (np.float32(y), ip) if stages else np.float32(y)


def tq1_0_digit(blk, i: int) -> int:
    return int(_tq1_digit(_p(_c(blk, np.uint8), _u8p), i))


def vec_dot_tq2_0(row, q8: Q8, in_f: int, stages: bool = False):
    row = _c(row, np.uint8)
    ip = np.empty(in_f // 256, np.int32) if stages else None
    y = _vd_tq2_0(_p(row, _u8p), _p(q8.qs, _i8p), _p(q8.d, _f32p), in_f, _p(ip, _i32p))
    return (np.float32(y), ip) if stages else np.float32(y)


def vec_dot_fp4(dtype: int, row, q8: "Q8x32", in_f: int, stages: bool = False):
    """MXFP4 / NVFP4 against the per-32 activation; stages: iprod per 32 (MXFP4) or per 16 (NVFP4)."""
    row = _c(row, np.uint8)
    ip = np.empty(in_f // (32 if dtype == MXFP4 else 16), np.int32) if stages else None
    fn = _vd_mxfp4 if dtype == MXFP4 else _vd_nvfp4
    y = fn(_p(row, _u8p), _p(q8.qs, _i8p), _p(q8.d, _f32p), in_f, _p(ip, _i32p))
    return (np.float32(y), ip) if stages else np.float32(y)


def e8m0_half(x: int) -> np.float32:
    return np.float32(_e8m0(int(x)))


def ue4m3_half(x: int) -> np.float32:
    return np.float32(_ue4m3(int(x)))


def iq4xs_scale(scales_h: int, scales_l, ib: int) -> int:
    """Sub-block ib's 6-bit scale of an IQ4_XS block, minus 32."""
    return int(_iq4xs_scale(int(scales_h), _p(_c(scales_l, np.uint8), _u8p), ib))


def q3k_scales(scales_raw) -> np.ndarray:
    """The sixteen signed sub-block scales (sc6 - 32) of one Q3_K block from its 12 scale bytes."""
    r = _c(scales_raw, np.uint8)
    out = np.empty(16, np.int16)
    _q3k_scales(_p(r, _u8p), out.ctypes.data_as(C.POINTER(C.c_int16)))
    return out


def vec_dot_blk32(dtype: int, row, q8: Q8x32, in_f: int, stages: bool = False):
    """Q4_0 / Q4_1 / Q5_0 / Q5_1 / IQ4_NL against the per-32 activation."""
    row = _c(row, np.uint8)
    ip = np.empty(in_f // 32, np.int32) if stages else None
    y = _vd_b32(dtype, _p(row, _u8p), _p(q8.qs, _i8p), _p(q8.d, _f32p), _p(q8.bsum, _i32p), in_f,
                _p(ip, _i32p))
    return (np.float32(y), ip) if stages else np.float32(y)


def embed_gather(dtype: int, table, table_numel: int, ids, ne: int, scale: float = 1.0) -> np.ndarray:
    """Op::EmbedGather on the CPU oracle: rows of ``table`` (raw blocks) decoded and scaled."""
    table = _c(table, np.uint8).ravel() if np.asarray(table).dtype == np.uint8 else np.ascontiguousarray(table).view(np.uint8).ravel()
    ids = _c(ids, np.int32).ravel()
    out = np.empty((ids.size, ne), np.float32)
    rc = _embed(dtype, _p(table, _u8p), table.size, table_numel, _p(ids, _i32p), ids.size, ne, scale, _p(out, _f32p))
    if rc != 0:
        raise ValueError(f"oracle embed_gather failed rc={rc}")
    return out


def dot(a, b) -> np.float32:
    a, b = _c(a, np.float32), _c(b, np.float32)
    return np.float32(_dot(_p(a, _f32p), _p(b, _f32p), min(a.size, b.size)))


def silu(g: float) -> np.float32:
    return np.float32(_silu(np.float32(g)))


SILU, GELU, SIGMOID = 0, 1, 2
_act = _sig("orc_act", C.c_float, C.c_int, C.c_float)
_gated = _sig("orc_gated_act", C.c_float, C.c_int, C.c_int, C.c_float, C.c_float, C.c_float)
_rms = _sig("orc_rms_norm", None, _f32p, _f32p, _f32p, C.c_size_t, C.c_size_t, C.c_float, C.c_int)
_gact = _sig("orc_gated_act_op", None, _f32p, _f32p, _f32p, C.c_size_t, C.c_size_t, C.c_int, C.c_size_t,
             C.c_size_t, C.c_size_t, C.c_size_t, C.c_int, C.c_float)
_gactf = _sig("orc_gated_act_fused", None, _f32p, _f32p, C.c_size_t, C.c_size_t, C.c_int, C.c_int, C.c_float)
_addop = _sig("orc_add", None, _f32p, _f32p, _f32p, C.c_size_t)


def act(kind: int, g: float) -> np.float32:
    """act_fn (kernels.rs:6578-6585)."""
    return np.float32(_act(kind, np.float32(g)))


def gated_act_fn(kind: int, clamp, gate: float, up: float) -> np.float32:
    """gated_act_fn (kernels.rs:6591-6597); ``clamp`` is None or the limit."""
    return np.float32(_gated(kind, clamp is not None, np.float32(clamp or 0.0), np.float32(gate), np.float32(up)))


def rms_norm(x, w, rows: int, dim: int, eps: float, into=None) -> np.ndarray:
    """Op::RmsNorm; with ``into`` (a [rows, dim] array) Op::RmsNormAdd: into += rmsnorm(x) * w."""
    x, w = _c(x, np.float32).ravel(), _c(w, np.float32).ravel()
    out = np.zeros(rows * dim, np.float32) if into is None else _c(into, np.float32).ravel().copy()
    _rms(_p(x, _f32p), _p(w, _f32p), _p(out, _f32p), rows, dim, np.float32(eps), into is not None)
    return out.reshape(rows, dim)


def gated_act(gate, up, rows: int, nff: int, kind: int = SILU, *, up_off: int = 0, up_stride: int = 0,
              gate_stride: int = 0, gate_block_width: int = 0, clamp=None) -> np.ndarray:
    """Op::GatedAct (lib.rs:1890-1944)."""
    gate, up = _c(gate, np.float32).ravel(), _c(up, np.float32).ravel()
    out = np.empty(rows * nff, np.float32)
    _gact(_p(gate, _f32p), _p(up, _f32p), _p(out, _f32p), rows, nff, kind, up_off, up_stride, gate_stride,
          gate_block_width, clamp is not None, np.float32(clamp or 0.0))
    return out.reshape(rows, nff)


def gated_act_fused(gu, rows: int, nff: int, kind: int = SILU, *, clamp=None) -> np.ndarray:
    """Op::GatedActFused (lib.rs:1945-1971)."""
    gu = _c(gu, np.float32).ravel()
    out = np.empty(rows * nff, np.float32)
    _gactf(_p(gu, _f32p), _p(out, _f32p), rows, nff, kind, clamp is not None, np.float32(clamp or 0.0))
    return out.reshape(rows, nff)


def add(a, b) -> np.ndarray:
    """Op::Add (lib.rs:1972-1988)."""
    a, b = _c(a, np.float32).ravel(), _c(b, np.float32).ravel()
    out = np.empty(a.size, np.float32)
    _addop(_p(a, _f32p), _p(b, _f32p), _p(out, _f32p), a.size)
    return out


def linear(dtype: int, w, x, m: int, in_f: int, out_f: int, *, w_numel: int | None = None,
           w_off: int = 0, reference_mode: bool = False, threads: int = 0) -> np.ndarray:
    """Op::Linear on the CPU oracle. ``w`` is the whole bound weight buffer (raw GGUF blocks)."""
    w = _c(w, np.uint8).ravel()
    x = _c(x, np.float32).ravel()
    if w_numel is None:
        e, b = block_layout(dtype)
        w_numel = w.size // b * e
    y = np.empty(m * out_f, np.float32)
    rc = _linear(dtype, _p(w, _u8p), w.size, w_numel, w_off, _p(x, _f32p), _p(y, _f32p), m, in_f,
                 out_f, int(reference_mode), threads)
    if rc != 0:
        raise ValueError(f"oracle linear failed rc={rc}")
    return y.reshape(m, out_f)


def linear_int_stages(dtype: int, w, x, m: int, in_f: int, out_f: int, *,
                      w_numel: int | None = None, w_off: int = 0):
    w = _c(w, np.uint8).ravel()
    x = _c(x, np.float32).ravel()
    if w_numel is None:
        e, b = block_layout(dtype)
        w_numel = w.size // b * e
    blocks = in_f // 256 if dtype in (Q4_K, Q5_K, Q6_K, Q2_K, Q3_K, IQ4_XS, TQ2_0, TQ1_0) else (in_f // 16 if dtype == NVFP4 else in_f // 32)
    a = np.empty((m, out_f, blocks), np.int32)
    b_ = np.empty((m, out_f, blocks), np.int32) if dtype in (Q4_K, Q5_K, Q2_K) else None
    rc = _linear_int(dtype, _p(w, _u8p), w.size, w_numel, w_off, _p(x, _f32p), m, in_f, out_f,
                     _p(a, _i32p), _p(b_, _i32p))
    if rc != 0:
        raise ValueError(f"oracle linear_int_stages failed rc={rc}")
    return a, b_


def ref_linear_f64(x, w_f32, m: int, in_f: int, out_f: int) -> np.ndarray:
    x, w_f32 = _c(x, np.float32).ravel(), _c(w_f32, np.float32).ravel()
    out = np.empty(m * out_f, np.float32)
    _ref_f64(_p(x, _f32p), _p(w_f32, _f32p), m, in_f, out_f, _p(out, _f32p))
    return out.reshape(m, out_f)


def expert_acts_kind(dtype: int, in_f: int, int8_ok: bool) -> int:
    return int(_acts_kind(dtype, in_f, int(int8_ok)))


def moe_ffn(x, router, gate, up, down, *, ne: int, n_expert: int, n_used: int, n_ff_exp: int,
            scale: float = 1.0, router_dtype: int = F32, gate_dtype: int = Q4_K,
            up_dtype: int = Q4_K, down_dtype: int = Q4_K, router_x=None,
            reference_mode: bool = False, threads: int = 0, act: int = 0, gating: int = 0,
            norm_w: bool = True, weight_before: bool = False, fused_gate_up: bool = False,
            swiglu_clamp=None, n_expert_groups: int = 0, n_expert_groups_used: int = 0,
            down_scale=None, exp_probs_b=None, expert_ids=None):
    """Op::MoeFfn on the CPU oracle; the keyword defaults are qwen3moe's setting. With
    ``fused_gate_up`` the ``gate`` bank holds gate rows then up rows per expert and ``up`` is ignored."""
    x = _c(x, np.float32).ravel()
    rows = x.size // ne
    rx = x if router_x is None else _c(router_x, np.float32).ravel()
    def raw(a):  # banks arrive as raw bytes (quantized) or as f32 arrays (router)
        a = np.ascontiguousarray(a)
        return a.view(np.uint8).ravel()

    router, gate, down = raw(router), raw(gate), raw(down)
    up = gate if fused_gate_up or up is None else raw(up)
    p = _MoeParams(ne, n_expert, n_used, n_ff_exp, rows, scale, router_dtype, gate_dtype, up_dtype,
                   down_dtype, int(reference_mode), act, gating, int(norm_w), int(weight_before),
                   int(fused_gate_up), int(swiglu_clamp is not None), float(swiglu_clamp or 0.0),
                   n_expert_groups, n_expert_groups_used)
    ds = None if down_scale is None else _c(down_scale, np.float32).ravel()
    eb = None if exp_probs_b is None else _c(exp_probs_b, np.float32).ravel()
    ids = None if expert_ids is None else _c(expert_ids, np.int32).ravel()
    y = np.empty(rows * ne, np.float32)
    idx = np.empty(rows * n_used, np.int32)
    w = np.empty(rows * n_used, np.float32)
    rc = _moe(C.byref(p), _p(x, _f32p), _p(rx, _f32p), _p(router, _u8p), router.size,
              _p(gate, _u8p), gate.size, _p(up, _u8p), up.size, _p(down, _u8p), down.size,
              _p(y, _f32p), _p(idx, _i32p), _p(w, _f32p), threads, _p(ds, _f32p), _p(eb, _f32p), _p(ids, _i32p))
    if rc != 0:
        raise ValueError(f"oracle moe_ffn failed rc={rc}")
    return y.reshape(rows, ne), idx.reshape(rows, n_used), w.reshape(rows, n_used)


def lcg_bytes(seed: int, n: int) -> np.ndarray:
    out = np.empty(n, np.uint8)
    _lcg(seed & 0xFFFFFFFF, n, _p(out, _u8p))
    return out


def gen_f32(n: int, salt: int) -> np.ndarray:
    out = np.empty(n, np.float32)
    _gen(n, salt, _p(out, _f32p))
    return out


def synth_weight(dtype: int, n_elem: int, seed: int) -> np.ndarray:
    e, b = block_layout(dtype)
    out = np.empty(n_elem // e * b, np.uint8)
    if _synth(dtype, n_elem, seed & 0xFFFFFFFF, _p(out, _u8p)) == 0:
        raise ValueError("synth_weight: unsupported dtype or ragged n_elem")
    return out


def det_bytes(n: int, seed: int) -> np.ndarray:
    out = np.empty(n, np.uint8)
    _detb(n, seed, _p(out, _u8p))
    return out


def det_x(n: int, seed: int) -> np.ndarray:
    out = np.empty(n, np.float32)
    _detx(n, seed, _p(out, _f32p))
    return out


def max_threads() -> int:
    return int(_maxthr())
