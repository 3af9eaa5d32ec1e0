// infr_hip.hpp — C++17 host side over the C ABI of infr_hip.h: the types a caller of infr-core's
// `Backend` seam handles (crates/infr-core/src/backend.rs:486-662), under the names they have
// there, for the ops of the quantized-matmul path. Header-only; link libinfr_hip.so.
//
//   reference (Rust)                               here (namespace infr)
//   DType, TensorDesc        tensor.rs:7-57        DType, TensorDesc
//   TensorId, TensorKind     graph.rs:100-122      TensorId, TensorKind
//   Op::{Linear, MoeFfn, RmsNorm, RmsNormAdd,      op::Linear ... op::EmbedGather (same field names),
//        GatedAct, GatedActFused, Add,             Op = std::variant of them
//        EmbedGather}        graph.rs:139-1011
//   Graph::{input, weight, internal, output,       Graph, same methods
//           push, desc, kind} graph.rs:1365-1460
//   BufferUsage              backend.rs:358-380    BufferUsage
//   Box<dyn Buffer>          backend.rs:387-416    Buffer (move-only; freed by its owner, never by
//                                                  the backend)
//   Box<dyn Plan>            backend.rs:418-446    Plan
//   Bindings                 backend.rs:448-483    Bindings (borrows buffers for one execute)
//   Error                    error.rs:5-25         Error (ErrorKind mirrors the enum; where the
//                                                  reference panics on a programmer error this
//                                                  throws ErrorKind::Invalid instead)
//   trait Backend            backend.rs:486-662    HipBackend: name, capabilities, alloc,
//                                                  alloc_uninit, upload, download, copy_buffer,
//                                                  compile, execute, sync
//
// Nothing here computes: every method is one call across the C ABI, and construction fails when no
// gfx950 device is usable.
#ifndef INFR_HIP_HPP
#define INFR_HIP_HPP

#include <cstdint>
#include <cstring>
#include <optional>
#include <stdexcept>
#include <string>
#include <utility>
#include <variant>
#include <vector>

#include "infr_hip.h"

namespace infr {

// crates/infr-core/src/tensor.rs:7-57; numbered as GGML type ids.
enum class DType : int {
    F32 = INFR_DTYPE_F32, F16 = INFR_DTYPE_F16, Q4_0 = INFR_DTYPE_Q4_0, Q4_1 = INFR_DTYPE_Q4_1,
    Q5_0 = INFR_DTYPE_Q5_0, Q5_1 = INFR_DTYPE_Q5_1, Q8_0 = INFR_DTYPE_Q8_0, Q2K = INFR_DTYPE_Q2_K,
    Q3K = INFR_DTYPE_Q3_K, Q4K = INFR_DTYPE_Q4_K,
    Q5K = INFR_DTYPE_Q5_K, Q6K = INFR_DTYPE_Q6_K, IQ4NL = INFR_DTYPE_IQ4_NL, IQ4XS = INFR_DTYPE_IQ4_XS, TQ1_0 = INFR_DTYPE_TQ1_0, TQ2_0 = INFR_DTYPE_TQ2_0, MXFP4 = INFR_DTYPE_MXFP4, NVFP4 = INFR_DTYPE_NVFP4, I32 = 26,
    BF16 = INFR_DTYPE_BF16, Q2_0 = INFR_DTYPE_Q2_0,
};

inline const char* dtype_name(DType d) {
    switch (d) {
    case DType::F32: return "F32";
    case DType::F16: return "F16";
    case DType::Q4_0: return "Q4_0";
    case DType::Q4_1: return "Q4_1";
    case DType::Q5_0: return "Q5_0";
    case DType::Q5_1: return "Q5_1";
    case DType::Q8_0: return "Q8_0";
    case DType::Q2K: return "Q2K";
    case DType::Q3K: return "Q3K";
    case DType::Q4K: return "Q4K";
    case DType::Q5K: return "Q5K";
    case DType::Q6K: return "Q6K";
    case DType::IQ4NL: return "IQ4NL";
    case DType::IQ4XS: return "IQ4XS";
    case DType::TQ1_0: return "TQ1_0";
    case DType::TQ2_0: return "TQ2_0";
    case DType::MXFP4: return "MXFP4";
    case DType::NVFP4: return "NVFP4";
    case DType::I32: return "I32";
    case DType::BF16: return "BF16";
    case DType::Q2_0: return "Q2_0";
    }
    return "?";
}

// (elements, bytes) of one block; crates/infr-core/src/decode_spec.rs:255-381.
inline std::pair<size_t, size_t> block_layout(DType d) {
    if (d == DType::I32) return {1, 4};
    int e = 0, b = 0;
    if (!infr_block_layout((int)d, &e, &b)) throw std::invalid_argument("unknown dtype");
    return {(size_t)e, (size_t)b};
}

enum class ErrorKind : int {
    Backend = INFR_HIP_ERR_BACKEND, Loader = INFR_HIP_ERR_LOADER, Model = INFR_HIP_ERR_MODEL,
    Unsupported = INFR_HIP_ERR_UNSUPPORTED, Aborted = INFR_HIP_ERR_ABORTED, Io = INFR_HIP_ERR_IO,
    Other = INFR_HIP_ERR_OTHER, Invalid = INFR_HIP_ERR_INVALID,
};

// crates/infr-core/src/error.rs:5-25
class Error : public std::runtime_error {
public:
    Error(ErrorKind k, const std::string& msg) : std::runtime_error(msg), kind(k) {}
    ErrorKind kind;
};

// crates/infr-core/src/backend.rs:358-380
enum class BufferUsage : int {
    Weights = INFR_USAGE_WEIGHTS, Activations = INFR_USAGE_ACTIVATIONS, KvCache = INFR_USAGE_KV_CACHE,
    Staging = INFR_USAGE_STAGING, Readback = INFR_USAGE_READBACK, HostWeights = INFR_USAGE_HOST_WEIGHTS,
};

struct TensorId {
    uint32_t v = 0;
    bool operator==(TensorId o) const { return v == o.v; }
};

enum class TensorKind { Input, Weight, Internal, Output };

struct TensorDesc {
    std::vector<size_t> shape;
    DType dtype = DType::F32;
    size_t numel() const {
        size_t n = 1;
        for (size_t s : shape) n *= s;
        return n;
    }
    // bytes of the raw tensor: whole blocks of `dtype`
    size_t nbytes() const {
        const auto [e, b] = block_layout(dtype);
        return numel() / e * b;
    }
};

// crates/infr-core/src/graph.rs Activation; act_fn, crates/infr-cpu/src/kernels.rs:6578-6585
enum class Activation : int { Silu = INFR_ACT_SILU, Gelu = INFR_ACT_GELU, Sigmoid = INFR_ACT_SIGMOID };
// crates/infr-core/src/graph.rs:76-85
enum class MoeGating : int { Softmax = INFR_GATING_SOFTMAX, Sigmoid = INFR_GATING_SIGMOID, SqrtSoftplus = INFR_GATING_SQRT_SOFTPLUS };

namespace op {
// graph.rs:177-191
struct Linear { TensorId x, weight, dst; uint32_t m, in_f, out_f; uint64_t w_off = 0; };
// graph.rs:911-1011, every field under the reference's name; the defaults after `scale` are what
// qwen3moe emits (softmax gating, renormalised weights on the output, split banks, SiLU)
struct MoeFfn {
    TensorId x, router_x, router, gate_exps, up_exps, down_exps, dst;
    uint32_t ne, n_expert, n_used, n_ff_exp;
    float scale = 1.0f;
    Activation act = Activation::Silu;
    MoeGating gating = MoeGating::Softmax;
    bool norm_w = true;
    bool weight_before = false;
    bool fused_gate_up = false;
    std::optional<float> swiglu_clamp;
    std::optional<TensorId> down_scale, exp_probs_b, expert_ids;
    uint32_t n_expert_groups = 0, n_expert_groups_used = 0;
    std::optional<std::pair<uint32_t, uint32_t>> ep_band;
};
// graph.rs:139-148 / 149-158
struct RmsNorm { TensorId x, weight, dst; uint32_t rows, dim; float eps; };
struct RmsNormAdd { TensorId x, weight, dst; uint32_t rows, dim; float eps; };
// graph.rs:697-735
struct GatedAct {
    TensorId gate, up, dst; uint32_t rows, nff; Activation act = Activation::Silu;
    uint32_t up_off = 0, up_stride = 0, gate_stride = 0, gate_block_width = 0;
    std::optional<float> swiglu_clamp;
};
// graph.rs:736-748
struct GatedActFused {
    TensorId gu, dst; uint32_t rows, nff; Activation act = Activation::Silu;
    std::optional<float> swiglu_clamp;
};
// graph.rs:749-755 (element count taken from dst's declaration)
struct Add { TensorId a, b, dst; };
// graph.rs:853-865
struct EmbedGather { TensorId ids, table, dst; uint32_t rows, ne; float scale = 1.0f; };
}  // namespace op

using Op = std::variant<op::Linear, op::MoeFfn, op::RmsNorm, op::RmsNormAdd, op::GatedAct,
                        op::GatedActFused, op::Add, op::EmbedGather>;

// crates/infr-core/src/graph.rs:1317-1460: ordered op list over declared tensors.
class Graph {
public:
    struct TensorDecl { TensorDesc desc; TensorKind kind; std::string label; };
    std::vector<TensorDecl> tensors;
    std::vector<Op> ops;

    TensorId input(TensorDesc d) { return decl(std::move(d), TensorKind::Input); }
    TensorId weight(TensorDesc d) { return decl(std::move(d), TensorKind::Weight); }
    TensorId internal(TensorDesc d) { return decl(std::move(d), TensorKind::Internal); }
    TensorId output(TensorDesc d) { return decl(std::move(d), TensorKind::Output); }
    TensorId label(TensorId id, std::string s) { tensors.at(id.v).label = std::move(s); return id; }
    void push(Op o) { ops.push_back(std::move(o)); }
    const TensorDesc& desc(TensorId id) const { return tensors.at(id.v).desc; }
    TensorKind kind(TensorId id) const { return tensors.at(id.v).kind; }

private:
    TensorId decl(TensorDesc d, TensorKind k) {
        tensors.push_back({std::move(d), k, {}});
        return TensorId{(uint32_t)tensors.size() - 1};
    }
};

class HipBackend;

// Box<dyn Buffer>: owned by whoever allocated it; dropping it frees the device memory.
class Buffer {
public:
    Buffer() = default;
    Buffer(Buffer&& o) noexcept : be_(o.be_), h_(o.h_) { o.h_ = nullptr; }
    Buffer& operator=(Buffer&& o) noexcept {
        if (this != &o) { reset(); be_ = o.be_; h_ = o.h_; o.h_ = nullptr; }
        return *this;
    }
    Buffer(const Buffer&) = delete;
    Buffer& operator=(const Buffer&) = delete;
    ~Buffer() { reset(); }
    size_t len_bytes() const { return h_ ? infr_hip_buffer_len(h_) : 0; }
    uint64_t device_addr() const { return h_ ? infr_hip_buffer_device_addr(h_) : 0; }
    infr_hip_buffer_t* raw() const { return h_; }

private:
    friend class HipBackend;
    Buffer(infr_hip_t* be, infr_hip_buffer_t* h) : be_(be), h_(h) {}
    void reset() { if (h_) infr_hip_free(be_, h_); h_ = nullptr; }
    infr_hip_t* be_ = nullptr;
    infr_hip_buffer_t* h_ = nullptr;
};

// Box<dyn Plan>
class Plan {
public:
    Plan() = default;
    Plan(Plan&& o) noexcept : be_(o.be_), h_(o.h_) { o.h_ = nullptr; }
    Plan& operator=(Plan&& o) noexcept {
        if (this != &o) { reset(); be_ = o.be_; h_ = o.h_; o.h_ = nullptr; }
        return *this;
    }
    Plan(const Plan&) = delete;
    Plan& operator=(const Plan&) = delete;
    ~Plan() { reset(); }
    // kernel launches one execute issued for the bindings it last ran with
    size_t launches() const { return h_ ? infr_hip_plan_launches(h_) : 0; }

private:
    friend class HipBackend;
    Plan(infr_hip_t* be, infr_hip_plan_t* h) : be_(be), h_(h) {}
    void reset() { if (h_) infr_hip_plan_free(be_, h_); h_ = nullptr; }
    infr_hip_t* be_ = nullptr;
    infr_hip_plan_t* h_ = nullptr;
};

// Bindings (backend.rs:448-483): buffers borrowed for one execute, indexed by TensorId.
class Bindings {
public:
    Bindings& bind(TensorId id, const Buffer& b) {
        if (slots_.size() <= id.v) slots_.resize(id.v + 1, nullptr);
        slots_[id.v] = b.raw();
        return *this;
    }
    infr_hip_buffer_t* get(TensorId id) const { return id.v < slots_.size() ? slots_[id.v] : nullptr; }
    const std::vector<infr_hip_buffer_t*>& slots() const { return slots_; }

private:
    std::vector<infr_hip_buffer_t*> slots_;
};

using Capabilities = infr_hip_caps_t;

// impl Backend for the gfx950 library.
class HipBackend {
public:
    explicit HipBackend(int device = 0) {
        const int rc = infr_hip_create(device, &h_);
        if (rc != INFR_HIP_OK) throw Error((ErrorKind)rc, infr_hip_last_error(nullptr));
    }
    ~HipBackend() { if (h_) infr_hip_destroy(h_); }
    HipBackend(const HipBackend&) = delete;
    HipBackend& operator=(const HipBackend&) = delete;

    std::string name() const { return infr_hip_name(h_); }
    Capabilities capabilities() const {
        Capabilities c{};
        check(infr_hip_capabilities(h_, &c));
        return c;
    }
    // zero-initialised (backend.rs:491-496)
    Buffer alloc(size_t bytes, BufferUsage usage) {
        infr_hip_buffer_t* b = nullptr;
        check(infr_hip_alloc(h_, bytes, (int)usage, &b));
        return Buffer(h_, b);
    }
    Buffer alloc_uninit(size_t bytes, BufferUsage usage) {
        infr_hip_buffer_t* b = nullptr;
        check(infr_hip_alloc_uninit(h_, bytes, (int)usage, &b));
        return Buffer(h_, b);
    }
    void upload(const Buffer& dst, const void* src, size_t n) { check(infr_hip_upload(h_, dst.raw(), src, n)); }
    template <typename T>
    void upload(const Buffer& dst, const std::vector<T>& src) { upload(dst, src.data(), src.size() * sizeof(T)); }
    void download(const Buffer& src, void* dst, size_t n) { check(infr_hip_download(h_, src.raw(), dst, n)); }
    template <typename T>
    void download(const Buffer& src, std::vector<T>& dst) { download(src, dst.data(), dst.size() * sizeof(T)); }
    void copy_buffer(const Buffer& src, const Buffer& dst, size_t bytes) {
        check(infr_hip_copy_buffer(h_, src.raw(), dst.raw(), bytes));
    }
    void sync() { check(infr_hip_sync(h_)); }

    // Validates and stores the op list; weight element counts and types come from the graph's
    // tensor declarations, as in the reference.
    Plan compile(const Graph& g) {
        std::vector<infr_hip_op_t> ops(g.ops.size());
        for (size_t i = 0; i < g.ops.size(); ++i) ops[i] = lower(g, g.ops[i]);
        infr_hip_plan_t* p = nullptr;
        check(infr_hip_compile(h_, ops.data(), ops.size(), &p));
        return Plan(h_, p);
    }
    // Asynchronous; results are visible after sync() or a download.
    void execute(const Plan& plan, const Bindings& b) {
        check(infr_hip_execute(h_, plan.h_, b.slots().data(), b.slots().size()));
    }

    infr_hip_t* raw() const { return h_; }
    void check(int rc) const {
        if (rc != INFR_HIP_OK) throw Error((ErrorKind)rc, infr_hip_last_error(h_));
    }

private:
    static infr_hip_op_t lower(const Graph& g, const Op& o) {
        infr_hip_op_t c;
        std::memset(&c, 0, sizeof c);
        std::visit([&](const auto& v) { fill(g, v, c); }, o);
        return c;
    }
    static void fill(const Graph& g, const op::Linear& v, infr_hip_op_t& c) {
        c.kind = INFR_OP_LINEAR;
        c.x = v.x.v; c.weight = v.weight.v; c.dst = v.dst.v;
        c.m = v.m; c.in_f = v.in_f; c.out_f = v.out_f; c.w_off = v.w_off;
        c.w_numel = g.desc(v.weight).numel();
        c.w_dtype = (int)g.desc(v.weight).dtype;
    }
    static void fill(const Graph& g, const op::MoeFfn& v, infr_hip_op_t& c) {
        c.kind = INFR_OP_MOE_FFN;
        c.x = v.x.v; c.dst = v.dst.v; c.router_x = v.router_x.v; c.router = v.router.v;
        c.gate_exps = v.gate_exps.v; c.up_exps = v.up_exps.v; c.down_exps = v.down_exps.v;
        c.moe.ne = v.ne; c.moe.n_expert = v.n_expert; c.moe.n_used = v.n_used; c.moe.n_ff_exp = v.n_ff_exp;
        c.moe.rows = (uint32_t)(g.desc(v.x).numel() / (v.ne ? v.ne : 1));
        c.moe.scale = v.scale;
        c.moe.router_dtype = (int)g.desc(v.router).dtype;
        c.moe.gate_dtype = (int)g.desc(v.gate_exps).dtype;
        c.moe.up_dtype = (int)g.desc(v.up_exps).dtype;
        c.moe.down_dtype = (int)g.desc(v.down_exps).dtype;
        c.moe.act = (int)v.act; c.moe.gating = (int)v.gating;
        c.moe.norm_w = v.norm_w; c.moe.weight_before = v.weight_before; c.moe.fused_gate_up = v.fused_gate_up;
        c.moe.has_clamp = v.swiglu_clamp.has_value(); c.moe.clamp = v.swiglu_clamp.value_or(0.0f);
        c.moe.n_expert_groups = v.n_expert_groups; c.moe.n_expert_groups_used = v.n_expert_groups_used;
        c.moe.has_down_scale = v.down_scale.has_value(); c.down_scale = v.down_scale ? v.down_scale->v : 0;
        c.moe.has_exp_probs_b = v.exp_probs_b.has_value(); c.exp_probs_b = v.exp_probs_b ? v.exp_probs_b->v : 0;
        c.moe.has_expert_ids = v.expert_ids.has_value(); c.expert_ids = v.expert_ids ? v.expert_ids->v : 0;
        c.moe.has_ep_band = v.ep_band.has_value();
    }
    static void fill(const Graph&, const op::RmsNorm& v, infr_hip_op_t& c) {
        c.kind = INFR_OP_RMS_NORM;
        c.x = v.x.v; c.weight = v.weight.v; c.dst = v.dst.v; c.m = v.rows; c.in_f = v.dim; c.eps = v.eps;
    }
    static void fill(const Graph&, const op::RmsNormAdd& v, infr_hip_op_t& c) {
        c.kind = INFR_OP_RMS_NORM_ADD;
        c.x = v.x.v; c.weight = v.weight.v; c.dst = v.dst.v; c.m = v.rows; c.in_f = v.dim; c.eps = v.eps;
    }
    static void fill(const Graph&, const op::GatedAct& v, infr_hip_op_t& c) {
        c.kind = INFR_OP_GATED_ACT;
        c.x = v.gate.v; c.aux = v.up.v; c.dst = v.dst.v; c.m = v.rows; c.in_f = v.nff; c.act = (int)v.act;
        c.up_off = v.up_off; c.up_stride = v.up_stride; c.gate_stride = v.gate_stride;
        c.gate_block_width = v.gate_block_width;
        c.has_clamp = v.swiglu_clamp.has_value(); c.clamp = v.swiglu_clamp.value_or(0.0f);
    }
    static void fill(const Graph&, const op::GatedActFused& v, infr_hip_op_t& c) {
        c.kind = INFR_OP_GATED_ACT_FUSED;
        c.x = v.gu.v; c.dst = v.dst.v; c.m = v.rows; c.in_f = v.nff; c.act = (int)v.act;
        c.has_clamp = v.swiglu_clamp.has_value(); c.clamp = v.swiglu_clamp.value_or(0.0f);
    }
    static void fill(const Graph& g, const op::Add& v, infr_hip_op_t& c) {
        c.kind = INFR_OP_ADD;
        c.x = v.a.v; c.aux = v.b.v; c.dst = v.dst.v; c.m = 1; c.in_f = (uint32_t)g.desc(v.dst).numel();
    }
    static void fill(const Graph& g, const op::EmbedGather& v, infr_hip_op_t& c) {
        c.kind = INFR_OP_EMBED_GATHER;
        c.x = v.ids.v; c.weight = v.table.v; c.dst = v.dst.v; c.m = v.rows; c.in_f = v.ne; c.scale = v.scale;
        c.w_numel = g.desc(v.table).numel();
        c.w_dtype = (int)g.desc(v.table).dtype;
    }

    infr_hip_t* h_ = nullptr;
};

}  // namespace infr
#endif  // INFR_HIP_HPP
