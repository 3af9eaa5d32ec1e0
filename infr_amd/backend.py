"""Host-side mirror of infr-core's backend seam over the C ABI of ``libinfr_hip.so``.

Names follow the reference (crates/infr-core/src/backend.rs:387-662, graph.rs): ``HipBackend``
implements ``alloc / alloc_uninit / upload / download / copy_buffer / compile / execute / sync``,
``Graph`` holds ``TensorDesc`` handles and ``Op`` records, ``Bindings`` maps ``TensorId`` to
``Buffer``. Everything computes on the GPU through the shared library; there is no host
fallback, and loading fails loudly when the library is missing.
"""
from __future__ import annotations

import ctypes as C
import os
from dataclasses import dataclass, field
from enum import IntEnum

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libinfr_hip.so")


class DType(IntEnum):
    """GGML type ids (crates/infr-gguf/src/lib.rs:330-354)."""
    F32 = 0
    F16 = 1      # plain rows: embedding tables, Linear weights, MoE router and banks
    Q4_0 = 2
    Q4_1 = 3
    Q5_0 = 6
    Q5_1 = 7
    Q8_0 = 8
    Q2K = 10
    Q3K = 11
    Q4K = 12
    Q5K = 13
    Q6K = 14
    IQ4NL = 20
    IQ4XS = 23
    TQ1_0 = 34
    TQ2_0 = 35
    MXFP4 = 39
    NVFP4 = 40
    BF16 = 30    # plain rows, as F16
    I32 = 26     # token ids (never a weight here)
    Q2_0 = 42


class BufferUsage(IntEnum):
    """crates/infr-core/src/backend.rs:358-380"""
    Weights = 0
    Activations = 1
    KvCache = 2
    Staging = 3
    Readback = 4
    HostWeights = 5


class Status(IntEnum):
    Ok = 0
    Backend = 1
    Loader = 2
    Model = 3
    Unsupported = 4
    Aborted = 5
    Io = 6
    Other = 7
    Invalid = 8


class InfrError(RuntimeError):
    """infr_core::error::Error (crates/infr-core/src/error.rs:5-25) with its variant in ``status``."""

    def __init__(self, status: int, msg: str):
        super().__init__(f"{Status(status).name}: {msg}")
        self.status = Status(status)
        self.msg = msg


class _MoeParams(C.Structure):
    _fields_ = [("ne", C.c_uint32), ("n_expert", C.c_uint32), ("n_used", C.c_uint32),
                ("n_ff_exp", C.c_uint32), ("rows", C.c_uint32), ("scale", C.c_float),
                ("router_dtype", C.c_int), ("gate_dtype", C.c_int), ("up_dtype", C.c_int),
                ("down_dtype", C.c_int),
                ("act", C.c_int), ("gating", C.c_int), ("norm_w", C.c_int), ("weight_before", C.c_int),
                ("fused_gate_up", C.c_int), ("has_clamp", C.c_int), ("clamp", C.c_float),
                ("n_expert_groups", C.c_uint32), ("n_expert_groups_used", C.c_uint32),
                ("has_down_scale", C.c_int), ("has_exp_probs_b", C.c_int), ("has_expert_ids", C.c_int),
                ("has_ep_band", C.c_int)]


class _MoeOptional(C.Structure):
    _fields_ = [("down_scale", C.c_void_p), ("exp_probs_b", C.c_void_p), ("expert_ids", C.c_void_p)]


def _moe_params(ne, n_expert, n_used, n_ff_exp, rows, scale, router_dtype, gate_dtype, up_dtype, down_dtype, act,
                gating, norm_w, weight_before, fused_gate_up, swiglu_clamp, n_expert_groups, n_expert_groups_used,
                has_down_scale, has_exp_probs_b, has_expert_ids, has_ep_band) -> "_MoeParams":
    return _MoeParams(ne, n_expert, n_used, n_ff_exp, rows, scale, router_dtype, gate_dtype, up_dtype, down_dtype,
                      int(act), int(gating), int(bool(norm_w)), int(bool(weight_before)), int(bool(fused_gate_up)),
                      int(swiglu_clamp is not None), float(swiglu_clamp or 0.0), n_expert_groups,
                      n_expert_groups_used, int(has_down_scale), int(has_exp_probs_b), int(has_expert_ids),
                      int(has_ep_band))


class _Op(C.Structure):
    _fields_ = [("kind", C.c_int), ("x", C.c_uint32), ("weight", C.c_uint32), ("dst", C.c_uint32),
                ("m", C.c_uint32), ("in_f", C.c_uint32), ("out_f", C.c_uint32),
                ("w_off", C.c_uint64), ("w_numel", C.c_uint64), ("w_dtype", C.c_int),
                ("router_x", C.c_uint32), ("router", C.c_uint32), ("gate_exps", C.c_uint32),
                ("up_exps", C.c_uint32), ("down_exps", C.c_uint32),
                ("down_scale", C.c_uint32), ("exp_probs_b", C.c_uint32), ("expert_ids", C.c_uint32),
                ("moe", _MoeParams),
                ("aux", C.c_uint32), ("eps", C.c_float), ("act", C.c_int), ("up_off", C.c_uint32),
                ("up_stride", C.c_uint32), ("gate_stride", C.c_uint32), ("gate_block_width", C.c_uint32),
                ("has_clamp", C.c_int), ("clamp", C.c_float), ("scale", C.c_float)]


class _Caps(C.Structure):
    _fields_ = [("i8", C.c_int), ("i8_dot", C.c_int), ("coopmat_i8_m", C.c_int),
                ("coopmat_i8_n", C.c_int), ("coopmat_i8_k", C.c_int), ("decode_replay", C.c_int),
                ("combined_gu", C.c_int), ("embed_gather", C.c_int), ("gpu_sample", C.c_int),
                ("argmax_rows", C.c_int), ("gated_rmsnorm", C.c_int),
                ("graph_input_inplace", C.c_int), ("unified_memory", C.c_int),
                ("device_memory_bytes", C.c_uint64), ("compute_units", C.c_int),
                ("device_name", C.c_char * 64)]


_vp = C.c_void_p
# Every symbol include/infr_hip.h declares: (restype, argtypes).
SYMBOLS = {
    "infr_hip_create": (C.c_int, [C.c_int, C.POINTER(_vp)]),
    "infr_hip_destroy": (None, [_vp]),
    "infr_hip_name": (C.c_char_p, [_vp]),
    "infr_hip_capabilities": (C.c_int, [_vp, C.POINTER(_Caps)]),
    "infr_hip_last_error": (C.c_char_p, [_vp]),
    "infr_hip_alloc": (C.c_int, [_vp, C.c_size_t, C.c_int, C.POINTER(_vp)]),
    "infr_hip_alloc_uninit": (C.c_int, [_vp, C.c_size_t, C.c_int, C.POINTER(_vp)]),
    "infr_hip_wrap": (C.c_int, [_vp, _vp, C.c_size_t, C.POINTER(_vp)]),
    "infr_hip_free": (None, [_vp, _vp]),
    "infr_hip_buffer_len": (C.c_size_t, [_vp]),
    "infr_hip_buffer_device_addr": (C.c_uint64, [_vp]),
    "infr_hip_upload": (C.c_int, [_vp, _vp, _vp, C.c_size_t]),
    "infr_hip_download": (C.c_int, [_vp, _vp, _vp, C.c_size_t]),
    "infr_hip_upload_at": (C.c_int, [_vp, _vp, C.c_size_t, _vp, C.c_size_t]),
    "infr_hip_download_at": (C.c_int, [_vp, _vp, C.c_size_t, _vp, C.c_size_t]),
    "infr_hip_copy_buffer": (C.c_int, [_vp, _vp, _vp, C.c_size_t]),
    "infr_hip_sync": (C.c_int, [_vp]),
    "infr_hip_linear": (C.c_int, [_vp, C.c_int, _vp, C.c_size_t, C.c_size_t, _vp, _vp, C.c_size_t,
                                  C.c_size_t, C.c_size_t]),
    "infr_hip_linear_noalloc": (C.c_int, [_vp, C.c_int, _vp, C.c_size_t, C.c_size_t, _vp, _vp, C.c_size_t,
                                          C.c_size_t, C.c_size_t]),
    "infr_hip_quantize_q8": (C.c_int, [_vp, _vp, C.c_size_t, C.c_size_t, _vp, _vp, _vp, _vp]),
    "infr_hip_quantize_q8_32": (C.c_int, [_vp, _vp, C.c_size_t, C.c_size_t, _vp, _vp, _vp]),
    "infr_hip_linear_int_stages": (C.c_int, [_vp, C.c_int, _vp, C.c_size_t, C.c_size_t, _vp,
                                             C.c_size_t, C.c_size_t, C.c_size_t, _vp, _vp]),
    "infr_hip_moe_ffn": (C.c_int, [_vp, C.POINTER(_MoeParams), _vp, _vp, _vp, _vp, _vp, _vp,
                                   C.POINTER(_MoeOptional), _vp, _vp, _vp]),
    "infr_hip_embed_gather": (C.c_int, [_vp, C.c_int, _vp, C.c_size_t, _vp, C.c_size_t, C.c_size_t, C.c_float, _vp]),
    "infr_hip_compile": (C.c_int, [_vp, C.POINTER(_Op), C.c_size_t, C.POINTER(_vp)]),
    "infr_hip_plan_free": (None, [_vp, _vp]),
    "infr_hip_execute": (C.c_int, [_vp, _vp, C.POINTER(_vp), C.c_size_t]),
    "infr_hip_plan_launches": (C.c_size_t, [_vp]),
    "infr_hip_request_shutdown": (C.c_int, [C.c_int]),
    "infr_hip_shutdown_requested": (C.c_int, []),
    "infr_hip_shutdown_signal": (C.c_int, []),
    "infr_hip_reset_shutdown": (None, []),
    "infr_hip_timer_begin": (C.c_int, [_vp]),
    "infr_hip_timer_end": (C.c_int, [_vp, C.POINTER(C.c_float)]),
    "infr_hip_stream_read": (C.c_int, [_vp, _vp, C.c_size_t, C.c_int, C.c_int, C.POINTER(C.c_float)]),
    "infr_hip_mfma_i8_peak": (C.c_int, [_vp, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_float), C.POINTER(C.c_double)]),
    "infr_synth_normal_f32": (None, [C.c_uint64, C.c_float, C.c_float, C.c_size_t, _vp]),
    "infr_synth_weight": (C.c_size_t, [C.c_int, C.c_uint64, C.c_float, C.c_size_t, C.c_size_t, _vp]),
    "infr_block_layout": (C.c_int, [C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int)]),
}


class _GgufTensor(C.Structure):
    _fields_ = [("name", C.c_char_p), ("ggml_type", C.c_int), ("n_dims", C.c_int),
                ("shape", C.c_uint64 * 4), ("numel", C.c_uint64), ("offset", C.c_uint64),
                ("nbytes", C.c_size_t)]


# Every symbol include/infr_gguf.h declares.
SYMBOLS.update({
    "infr_gguf_open": (C.c_int, [C.c_char_p, C.POINTER(_vp)]),
    "infr_gguf_close": (None, [_vp]),
    "infr_gguf_last_error": (C.c_char_p, []),
    "infr_gguf_n_tensors": (C.c_size_t, [_vp]),
    "infr_gguf_tensor": (C.c_int, [_vp, C.c_size_t, C.POINTER(_GgufTensor)]),
    "infr_gguf_find": (C.c_int64, [_vp, C.c_char_p]),
    "infr_gguf_tensor_bytes": (C.c_int, [_vp, C.c_char_p, C.POINTER(_vp), C.POINTER(C.c_size_t)]),
    "infr_gguf_tensor_file_range": (C.c_int, [_vp, C.c_char_p, C.POINTER(C.c_uint64), C.POINTER(C.c_size_t)]),
    "infr_gguf_n_shards": (C.c_size_t, [_vp]),
    "infr_gguf_shard": (C.c_int, [_vp, C.c_size_t, C.POINTER(C.c_char_p), C.POINTER(C.c_uint64)]),
    "infr_gguf_n_meta": (C.c_size_t, [_vp]),
    "infr_gguf_meta_key": (C.c_char_p, [_vp, C.c_size_t]),
    "infr_gguf_meta_get": (_vp, [_vp, C.c_char_p]),
    "infr_gguf_value_kind": (C.c_int, [_vp]),
    "infr_gguf_value_u64": (C.c_int, [_vp, C.POINTER(C.c_uint64)]),
    "infr_gguf_value_i64": (C.c_int, [_vp, C.POINTER(C.c_int64)]),
    "infr_gguf_value_f64": (C.c_int, [_vp, C.POINTER(C.c_double)]),
    "infr_gguf_value_bool": (C.c_int, [_vp, C.POINTER(C.c_int)]),
    "infr_gguf_value_str": (C.c_int, [_vp, C.POINTER(_vp), C.POINTER(C.c_size_t)]),
    "infr_gguf_value_arr_len": (C.c_int, [_vp, C.POINTER(C.c_size_t)]),
    "infr_gguf_value_arr_at": (_vp, [_vp, C.c_size_t]),
    "infr_gguf_chat_template": (C.c_char_p, [_vp]),
    "infr_gguf_block_layout": (C.c_int, [C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "infr_gguf_nbytes": (C.c_size_t, [C.c_int, C.c_uint64, C.POINTER(C.c_int)]),
    "infr_gguf_parse_shard": (C.c_int, [C.c_char_p, C.c_char_p, C.c_size_t, C.POINTER(C.c_size_t),
                                        C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.POINTER(C.c_size_t)]),
    "infr_gguf_shard_set": (C.c_size_t, [C.c_char_p, C.c_size_t, C.c_char_p, C.c_size_t]),
    "infr_gguf_upload": (C.c_int, [_vp, C.c_char_p, _vp, C.POINTER(_vp)]),
    "infr_gguf_upload_concat": (C.c_int, [_vp, C.POINTER(C.c_char_p), C.c_size_t, _vp, C.POINTER(_vp),
                                          C.POINTER(C.c_size_t)]),
})

_lib = None


def load_library() -> C.CDLL:
    """Load ``libinfr_hip.so`` (built in-tree by ``infr_amd.build``) and bind every symbol."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise InfrError(Status.Backend, f"{LIB_PATH} is not built; run `python -m infr_amd.build`")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def block_layout(dtype: int) -> tuple[int, int]:
    e, b = C.c_int(), C.c_int()
    if not load_library().infr_block_layout(int(dtype), C.byref(e), C.byref(b)):
        raise InfrError(Status.Unsupported, f"unknown dtype {dtype}")
    return e.value, b.value


def synth_normal_f32(seed: int, n: int, mean: float = 0.0, sigma: float = 1.0) -> np.ndarray:
    out = np.empty(n, np.float32)
    load_library().infr_synth_normal_f32(seed, mean, sigma, n, out.ctypes.data)
    return out


def synth_weight(dtype: int, seed: int, rows: int, in_f: int, sigma: float = 0.02) -> np.ndarray:
    """N(0, sigma^2) weights [rows, in_f] encoded as raw blocks of ``dtype``."""
    e, b = block_layout(dtype)
    if rows <= 0 or in_f <= 0 or in_f % e != 0:
        raise InfrError(Status.Invalid, f"synth_weight: in_f {in_f} is not a whole number of {e}-element blocks")
    out = np.empty(rows * (in_f // e) * b, np.uint8)
    n = load_library().infr_synth_weight(int(dtype), seed, sigma, rows, in_f, out.ctypes.data)
    if n != out.size:
        raise InfrError(Status.Invalid, f"synth_weight({dtype}, rows={rows}, in_f={in_f}) rejected")
    return out


# ───────────────────────────── graph mirror ─────────────────────────────

@dataclass(frozen=True)
class TensorId:
    id: int


@dataclass
class TensorDesc:
    """crates/infr-core/src/tensor.rs: shape + dtype."""
    shape: tuple
    dtype: DType

    def numel(self) -> int:
        n = 1
        for s in self.shape:
            n *= s
        return n


@dataclass
class Linear:
    """Op::Linear (crates/infr-core/src/graph.rs:177-191)."""
    x: TensorId
    weight: TensorId
    dst: TensorId
    m: int
    in_f: int
    out_f: int
    w_off: int = 0


class Activation(IntEnum):
    """crates/infr-core/src/graph.rs Activation; act_fn, crates/infr-cpu/src/kernels.rs:6578-6585."""
    Silu = 0
    Gelu = 1
    Sigmoid = 2


class MoeGating(IntEnum):
    """crates/infr-core/src/graph.rs:76-85."""
    Softmax = 0
    Sigmoid = 1
    SqrtSoftplus = 2


@dataclass
class MoeFfn:
    """Op::MoeFfn (graph.rs:911-1011), every field under the reference's name; the defaults are what
    qwen3moe emits (crates/infr-llama/src/seam/runner.rs:3971-3997)."""
    x: TensorId
    router_x: TensorId
    router: TensorId
    gate_exps: TensorId
    up_exps: TensorId
    down_exps: TensorId
    dst: TensorId
    ne: int
    n_expert: int
    n_used: int
    n_ff_exp: int
    scale: float = 1.0
    act: Activation = Activation.Silu
    gating: MoeGating = MoeGating.Softmax
    norm_w: bool = True
    weight_before: bool = False
    fused_gate_up: bool = False
    swiglu_clamp: float | None = None
    down_scale: TensorId | None = None
    exp_probs_b: TensorId | None = None
    n_expert_groups: int = 0
    n_expert_groups_used: int = 0
    expert_ids: TensorId | None = None
    ep_band: tuple | None = None


@dataclass
class RmsNorm:
    """Op::RmsNorm (graph.rs:139-148): dst = rmsnorm(x) * weight over the last `dim` of each row."""
    x: TensorId
    weight: TensorId
    dst: TensorId
    rows: int
    dim: int
    eps: float


@dataclass
class RmsNormAdd:
    """Op::RmsNormAdd (graph.rs:149-158): dst += rmsnorm(x) * weight."""
    x: TensorId
    weight: TensorId
    dst: TensorId
    rows: int
    dim: int
    eps: float


@dataclass
class GatedAct:
    """Op::GatedAct (graph.rs:697-735): dst[r, i] = act(gate[r, i]) * up[r, i + up_off]."""
    gate: TensorId
    up: TensorId
    dst: TensorId
    rows: int
    nff: int
    act: int = 0
    up_off: int = 0
    up_stride: int = 0
    gate_stride: int = 0
    gate_block_width: int = 0
    swiglu_clamp: float | None = None


@dataclass
class GatedActFused:
    """Op::GatedActFused (graph.rs:736-748): gu is [rows, 2*nff], gate half first."""
    gu: TensorId
    dst: TensorId
    rows: int
    nff: int
    act: int = 0
    swiglu_clamp: float | None = None


@dataclass
class Add:
    """Op::Add (graph.rs:749-755): dst[i] = a[i] + b[i]; in place when dst == a."""
    a: TensorId
    b: TensorId
    dst: TensorId
    n: int


@dataclass
class EmbedGather:
    """Op::EmbedGather (graph.rs:853-865): dst[r, :] = decode(table[ids[r], :]) * scale."""
    ids: TensorId
    table: TensorId
    dst: TensorId
    rows: int
    ne: int
    scale: float = 1.0


@dataclass
class Graph:
    """Ordered op list over declared tensors (crates/infr-core/src/graph.rs:1317-1460)."""
    tensors: list = field(default_factory=list)
    kinds: list = field(default_factory=list)
    ops: list = field(default_factory=list)

    def _decl(self, desc: TensorDesc, kind: str) -> TensorId:
        self.tensors.append(desc)
        self.kinds.append(kind)
        return TensorId(len(self.tensors) - 1)

    def input(self, desc: TensorDesc) -> TensorId:
        return self._decl(desc, "Input")

    def weight(self, desc: TensorDesc) -> TensorId:
        return self._decl(desc, "Weight")

    def output(self, desc: TensorDesc) -> TensorId:
        return self._decl(desc, "Output")

    def desc(self, t: TensorId) -> TensorDesc:
        return self.tensors[t.id]

    def push(self, op) -> None:
        self.ops.append(op)


class Buffer:
    """Opaque device-memory handle owned by the caller (backend.rs:387-416)."""

    def __init__(self, be: "HipBackend", handle: int):
        self._be = be
        self._h = handle

    def len_bytes(self) -> int:
        return load_library().infr_hip_buffer_len(self._h)

    def device_addr(self) -> int:
        return load_library().infr_hip_buffer_device_addr(self._h)

    def free(self) -> None:
        if self._h and self._be._h:
            load_library().infr_hip_free(self._be._h, self._h)
        self._h = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Bindings:
    """TensorId -> Buffer for one execute (backend.rs:448-483)."""

    def __init__(self):
        self.slots: list = []

    def bind(self, tid: TensorId, buf: Buffer) -> "Bindings":
        if tid.id >= len(self.slots):
            self.slots.extend([None] * (tid.id + 1 - len(self.slots)))
        self.slots[tid.id] = buf
        return self

    def get(self, tid: TensorId):
        return self.slots[tid.id] if tid.id < len(self.slots) else None


class Plan:
    def __init__(self, be: "HipBackend", handle: int, graph: Graph):
        self._be, self._h, self.graph = be, handle, graph

    def launches(self) -> int:
        """Kernel launches per execute for the bindings last run with."""
        return load_library().infr_hip_plan_launches(self._h)

    def __del__(self):
        try:
            if self._h and self._be._h:
                load_library().infr_hip_plan_free(self._be._h, self._h)
        except Exception:
            pass
        self._h = None


class HipBackend:
    """``impl Backend`` for one MI355X (crates/infr-core/src/backend.rs:486-662)."""

    def __init__(self, device: int = 0):
        self._lib = load_library()
        h = _vp()
        self._h = None
        rc = self._lib.infr_hip_create(device, C.byref(h))
        if rc != 0:
            raise InfrError(rc, (self._lib.infr_hip_last_error(None) or b"").decode())
        self._h = h.value

    # -- plumbing --
    def _check(self, rc: int) -> None:
        if rc != 0:
            raise InfrError(rc, (self._lib.infr_hip_last_error(self._h) or b"").decode())

    def close(self) -> None:
        if self._h:
            self._lib.infr_hip_destroy(self._h)
        self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # -- Backend --
    def name(self) -> str:
        return self._lib.infr_hip_name(self._h).decode()

    def capabilities(self) -> dict:
        caps = _Caps()
        self._check(self._lib.infr_hip_capabilities(self._h, C.byref(caps)))
        out = {n: getattr(caps, n) for n, _ in _Caps._fields_}
        out["device_name"] = caps.device_name.decode()
        return out

    def alloc(self, nbytes: int, usage: BufferUsage = BufferUsage.Activations) -> Buffer:
        h = _vp()
        self._check(self._lib.infr_hip_alloc(self._h, nbytes, int(usage), C.byref(h)))
        return Buffer(self, h.value)

    def alloc_uninit(self, nbytes: int, usage: BufferUsage = BufferUsage.Activations) -> Buffer:
        h = _vp()
        self._check(self._lib.infr_hip_alloc_uninit(self._h, nbytes, int(usage), C.byref(h)))
        return Buffer(self, h.value)

    def wrap(self, device_ptr: int, nbytes: int) -> Buffer:
        h = _vp()
        self._check(self._lib.infr_hip_wrap(self._h, device_ptr, nbytes, C.byref(h)))
        return Buffer(self, h.value)

    def upload(self, dst: Buffer, src, offset: int = 0) -> None:
        a = np.ascontiguousarray(src)
        self._check(self._lib.infr_hip_upload_at(self._h, dst._h, offset, a.ctypes.data, a.nbytes))

    def download(self, src: Buffer, dst: np.ndarray, offset: int = 0) -> np.ndarray:
        assert dst.flags["C_CONTIGUOUS"]
        self._check(self._lib.infr_hip_download_at(self._h, src._h, offset, dst.ctypes.data, dst.nbytes))
        return dst

    def copy_buffer(self, src: Buffer, dst: Buffer, nbytes: int) -> None:
        self._check(self._lib.infr_hip_copy_buffer(self._h, src._h, dst._h, nbytes))

    def sync(self) -> None:
        self._check(self._lib.infr_hip_sync(self._h))

    def compile(self, g: Graph) -> Plan:
        ops = (_Op * max(1, len(g.ops)))()
        for i, op in enumerate(g.ops):
            o = ops[i]
            if isinstance(op, Linear):
                o.kind = 1
                o.x, o.weight, o.dst = op.x.id, op.weight.id, op.dst.id
                o.m, o.in_f, o.out_f, o.w_off = op.m, op.in_f, op.out_f, op.w_off
                o.w_numel = g.desc(op.weight).numel()
                o.w_dtype = int(g.desc(op.weight).dtype)
            elif isinstance(op, MoeFfn):
                o.kind = 2
                o.x, o.dst = op.x.id, op.dst.id
                o.router_x, o.router = op.router_x.id, op.router.id
                o.gate_exps, o.up_exps, o.down_exps = op.gate_exps.id, op.up_exps.id, op.down_exps.id
                rows = g.desc(op.x).numel() // op.ne
                o.moe = _moe_params(op.ne, op.n_expert, op.n_used, op.n_ff_exp, rows, op.scale,
                                    int(g.desc(op.router).dtype), int(g.desc(op.gate_exps).dtype),
                                    int(g.desc(op.up_exps).dtype), int(g.desc(op.down_exps).dtype), op.act,
                                    op.gating, op.norm_w, op.weight_before, op.fused_gate_up, op.swiglu_clamp,
                                    op.n_expert_groups, op.n_expert_groups_used, op.down_scale is not None,
                                    op.exp_probs_b is not None, op.expert_ids is not None, op.ep_band is not None)
                o.down_scale = op.down_scale.id if op.down_scale is not None else 0
                o.exp_probs_b = op.exp_probs_b.id if op.exp_probs_b is not None else 0
                o.expert_ids = op.expert_ids.id if op.expert_ids is not None else 0
            elif isinstance(op, (RmsNorm, RmsNormAdd)):
                o.kind = 3 if isinstance(op, RmsNorm) else 4
                o.x, o.weight, o.dst = op.x.id, op.weight.id, op.dst.id
                o.m, o.in_f, o.eps = op.rows, op.dim, op.eps
            elif isinstance(op, GatedAct):
                o.kind = 5
                o.x, o.aux, o.dst = op.gate.id, op.up.id, op.dst.id
                o.m, o.in_f, o.act = op.rows, op.nff, int(op.act)
                o.up_off, o.up_stride = op.up_off, op.up_stride
                o.gate_stride, o.gate_block_width = op.gate_stride, op.gate_block_width
                o.has_clamp, o.clamp = op.swiglu_clamp is not None, op.swiglu_clamp or 0.0
            elif isinstance(op, GatedActFused):
                o.kind = 6
                o.x, o.dst = op.gu.id, op.dst.id
                o.m, o.in_f, o.act = op.rows, op.nff, int(op.act)
                o.has_clamp, o.clamp = op.swiglu_clamp is not None, op.swiglu_clamp or 0.0
            elif isinstance(op, Add):
                o.kind = 7
                o.x, o.aux, o.dst = op.a.id, op.b.id, op.dst.id
                o.m, o.in_f = 1, op.n
            elif isinstance(op, EmbedGather):
                o.kind = 8
                o.x, o.weight, o.dst = op.ids.id, op.table.id, op.dst.id
                o.m, o.in_f, o.scale = op.rows, op.ne, op.scale
                o.w_numel = g.desc(op.table).numel()
                o.w_dtype = int(g.desc(op.table).dtype)
            else:
                raise InfrError(Status.Unsupported, f"op {type(op).__name__} is not on this path")
        h = _vp()
        self._check(self._lib.infr_hip_compile(self._h, ops, len(g.ops), C.byref(h)))
        return Plan(self, h.value, g)

    def execute(self, plan: Plan, bindings: Bindings) -> None:
        n = len(bindings.slots)
        arr = (_vp * max(1, n))()
        for i, b in enumerate(bindings.slots):
            arr[i] = b._h if b is not None else None
        self._check(self._lib.infr_hip_execute(self._h, plan._h, arr, n))

    # -- the ops, directly --
    def linear(self, dtype: int, w: Buffer, x: Buffer, dst: Buffer, m: int, in_f: int, out_f: int,
               w_numel: int | None = None, w_off: int = 0) -> None:
        if w_numel is None:
            e, b = block_layout(dtype)
            w_numel = w.len_bytes() // b * e
        self._check(self._lib.infr_hip_linear(self._h, int(dtype), w._h, w_numel, w_off, x._h,
                                              dst._h, m, in_f, out_f))

    def linear_noalloc(self, dtype: int, w: Buffer, x: Buffer, dst: Buffer, m: int, in_f: int, out_f: int,
                       w_numel: int | None = None, w_off: int = 0) -> None:
        """infr_hip_linear over the library's static device scratch: allocates nothing."""
        if w_numel is None:
            e, b = block_layout(dtype)
            w_numel = w.len_bytes() // b * e
        self._check(self._lib.infr_hip_linear_noalloc(self._h, int(dtype), w._h, w_numel, w_off, x._h,
                                                      dst._h, m, in_f, out_f))

    def linear_int_stages(self, dtype: int, w: Buffer, x: Buffer, m: int, in_f: int, out_f: int,
                          w_numel: int | None = None, w_off: int = 0):
        if w_numel is None:
            e, b = block_layout(dtype)
            w_numel = w.len_bytes() // b * e
        blocks = in_f // 256 if dtype in (DType.Q4K, DType.Q5K, DType.Q6K, DType.Q2K, DType.Q3K, DType.IQ4XS, DType.TQ2_0, DType.TQ1_0) else in_f // 32
        a = self.alloc(m * out_f * blocks * 4)
        b_ = self.alloc(m * out_f * blocks * 4) if dtype in (DType.Q4K, DType.Q5K, DType.Q2K) else None
        self._check(self._lib.infr_hip_linear_int_stages(
            self._h, int(dtype), w._h, w_numel, w_off, x._h, m, in_f, out_f, a._h,
            b_._h if b_ else None))
        ra = self.download(a, np.empty((m, out_f, blocks), np.int32))
        rb = self.download(b_, np.empty((m, out_f, blocks), np.int32)) if b_ else None
        return ra, rb

    def quantize_q8(self, x: Buffer, m: int, k: int):
        """quantize_q8 (crates/infr-cpu/src/quant.rs:27-58) -> (qs, d, bsums, bsums16) arrays."""
        qs, d = self.alloc(m * k), self.alloc(m * k // 256 * 4)
        bs, bs16 = self.alloc(m * k // 32 * 4), self.alloc(m * k // 16 * 4)
        self._check(self._lib.infr_hip_quantize_q8(self._h, x._h, m, k, qs._h, d._h, bs._h, bs16._h))
        return (self.download(qs, np.empty((m, k), np.int8)),
                self.download(d, np.empty((m, k // 256), np.float32)),
                self.download(bs, np.empty((m, k // 32), np.int32)),
                self.download(bs16, np.empty((m, k // 16), np.int32)))

    def quantize_q8_32(self, x: Buffer, m: int, k: int):
        """quantize_q8_32 (quant.rs:97-117) -> (qs, d, bsum) arrays."""
        qs, d, bs = self.alloc(m * k), self.alloc(m * k // 32 * 4), self.alloc(m * k // 32 * 4)
        self._check(self._lib.infr_hip_quantize_q8_32(self._h, x._h, m, k, qs._h, d._h, bs._h))
        return (self.download(qs, np.empty((m, k), np.int8)),
                self.download(d, np.empty((m, k // 32), np.float32)),
                self.download(bs, np.empty((m, k // 32), np.int32)))

    def embed_gather(self, dtype: int, table: Buffer, table_numel: int, ids: Buffer, rows: int, ne: int,
                     dst: Buffer, scale: float = 1.0) -> None:
        self._check(self._lib.infr_hip_embed_gather(self._h, int(dtype), table._h, table_numel, ids._h, rows,
                                                    ne, scale, dst._h))

    def moe_ffn(self, x: Buffer, router: Buffer, gate: Buffer, up: Buffer, down: Buffer,
                dst: Buffer, *, rows: int, ne: int, n_expert: int, n_used: int, n_ff_exp: int,
                scale: float = 1.0, router_dtype: int = DType.F32, gate_dtype: int = DType.Q4K,
                up_dtype: int = DType.Q4K, down_dtype: int = DType.Q4K, router_x: Buffer | None = None,
                sel_idx: Buffer | None = None, sel_w: Buffer | None = None,
                act: int = Activation.Silu, gating: int = MoeGating.Softmax, norm_w: bool = True,
                weight_before: bool = False, fused_gate_up: bool = False, swiglu_clamp: float | None = None,
                n_expert_groups: int = 0, n_expert_groups_used: int = 0, down_scale: Buffer | None = None,
                exp_probs_b: Buffer | None = None, expert_ids: Buffer | None = None,
                ep_band: tuple | None = None) -> None:
        """Op::MoeFfn; the keyword defaults are qwen3moe's setting. With ``fused_gate_up`` the ``gate``
        bank holds gate rows then up rows per expert and ``up`` may be None."""
        p = _moe_params(ne, n_expert, n_used, n_ff_exp, rows, scale, int(router_dtype), int(gate_dtype),
                        int(up_dtype), int(down_dtype), act, gating, norm_w, weight_before, fused_gate_up,
                        swiglu_clamp, n_expert_groups, n_expert_groups_used, down_scale is not None,
                        exp_probs_b is not None, expert_ids is not None, ep_band is not None)
        opt = _MoeOptional(down_scale._h if down_scale else None, exp_probs_b._h if exp_probs_b else None,
                           expert_ids._h if expert_ids else None)
        rx = router_x if router_x is not None else x
        self._check(self._lib.infr_hip_moe_ffn(
            self._h, C.byref(p), x._h, rx._h, router._h, gate._h, up._h if up is not None else None, down._h,
            C.byref(opt), dst._h, sel_idx._h if sel_idx else None, sel_w._h if sel_w else None))

    # -- measurement --
    def stream_read_gbs(self, buf: Buffer, nbytes: int | None = None, reps: int = 10, nontemporal: bool = False) -> float:
        """GB/s of a read-only streaming kernel over ``buf`` (what fetching alone reaches), with plain
        or non-temporal loads."""
        n = buf.len_bytes() if nbytes is None else nbytes
        ms = C.c_float()
        self._check(self._lib.infr_hip_stream_read(self._h, buf._h, n, reps, 1 if nontemporal else 0, C.byref(ms)))
        return n * reps / (ms.value * 1e-3) / 1e9

    def mfma_i8_peak_tops(self, waves_per_simd: int = 4, iters: int = 4096, random_data: bool = True) -> float:
        """TOP/s of a register-only int8 MFMA loop (the matrix rate the device sustains by itself)."""
        ms, ops = C.c_float(), C.c_double()
        self._check(self._lib.infr_hip_mfma_i8_peak(self._h, waves_per_simd, iters, int(random_data),
                                                    C.byref(ms), C.byref(ops)))
        return ops.value / (ms.value * 1e-3) / 1e12

    def timer_begin(self) -> None:
        self._check(self._lib.infr_hip_timer_begin(self._h))

    def timer_end(self) -> float:
        ms = C.c_float()
        self._check(self._lib.infr_hip_timer_end(self._h, C.byref(ms)))
        return ms.value

    # -- convenience used by tests and the benchmark --
    def upload_new(self, arr, usage: BufferUsage = BufferUsage.Activations) -> Buffer:
        a = np.ascontiguousarray(arr)
        b = self.alloc_uninit(max(a.nbytes, 4), usage)
        self.upload(b, a)
        return b


def request_shutdown(signo: int) -> bool:
    return bool(load_library().infr_hip_request_shutdown(signo))


def shutdown_requested() -> bool:
    return bool(load_library().infr_hip_shutdown_requested())


def shutdown_signal() -> int | None:
    s = load_library().infr_hip_shutdown_signal()
    return s or None


def reset_shutdown() -> None:
    load_library().infr_hip_reset_shutdown()
