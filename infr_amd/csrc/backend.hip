// C-ABI layer (include/infr_hip.h): buffers, stream, argument checking, op dispatch and the
// plan/execute replay. Mirrors infr-core's Backend trait (crates/infr-core/src/backend.rs:486-662)
// for Op::Linear and Op::MoeFfn. Nothing here computes on the host: with no usable gfx950 device
// infr_hip_create fails and no other entry point can be reached.
#include "../../include/infr_hip.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "kernels.hpp"

struct infr_hip_buffer {
    void* ptr = nullptr;
    size_t len = 0;
    bool owned = false;
};

struct infr_hip_plan {
    std::vector<infr_hip_op_t> ops;
    uint32_t max_tensor = 0;
    // decode replay: launch sequence recorded for one set of bound device addresses
    hipGraphExec_t exec = nullptr;
    std::vector<void*> bound;
    uint64_t scratch_epoch = 0;  // the backend's scratch epoch the recording was made under
    size_t recorded_nodes = 0;   // nodes of the recorded graph: the launches of one execute
    // Launch schedule for the bound addresses: ops ordered by dependency level; the m == 1 ops
    // of a level that share (dtype, in_f) form one grouped decode launch.
    struct Step {
        int level = 0;
        int op = -1;              // ungrouped op (MoeFfn, larger m): index into ops
        int dtype = 0;            // group
        size_t in_f = 0;
        size_t m = 1;             // 1: decode group; 2..32: small-batch group
        bool f32act = false;      // decode group of the f32-activation kernel (Q5_0 at one token)
        bool strips = false;      // prefill group: Q4_K Linears over one activation tensor, one strip launch
        const float* x = nullptr; // strips: the shared activation tensor
        int first = 0, n = 0;     // slice of descs
        size_t tile_first = 0;    // slice of tiles (decode) / btiles (small batch)
        infr::GemvGroupPlan gp;
        infr::BatchGroupPlan bp;
        size_t qtile_first = 0, qtile_n = 0;  // small batch: slice of qtiles
    };
    std::vector<Step> steps;
    // per op: the Op::Add a MoeFfn's last kernel also produces (-1: none), and whether that
    // Add's residual is its first operand
    std::vector<int> moe_add;
    std::vector<char> moe_add_resid_is_a;
    // per op: the single-row Op::RmsNorm a MoeFfn's router kernel also computes (-1: none)
    std::vector<int> moe_norm;
    std::vector<infr::GemvOpDesc> descs;
    // per-workgroup tile tables of the grouped launches, back to back (tile_first per step)
    std::vector<infr::GemvTile> tiles;
    infr::GemvTile* tiles_dev = nullptr;
    size_t tiles_cap = 0;
    // prefill strip groups: one entry per strip (tile_first per step)
    std::vector<infr::StripSeg> ssegs;
    infr::StripSeg* ssegs_dev = nullptr;
    size_t ssegs_cap = 0;
    // small-batch groups: quantizer and GEMM tile tables
    std::vector<infr::QuantTile> qtiles;
    std::vector<infr::BatchTile> btiles;
    infr::QuantTile* qtiles_dev = nullptr;
    infr::BatchTile* btiles_dev = nullptr;
    size_t qtiles_cap = 0, btiles_cap = 0;
};

struct infr_hip {
    int device = 0;
    hipStream_t stream = nullptr;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    hipDeviceProp_t props;
    std::string err;
    std::string name;
    // Transient scratch for the quantized activation (TensorKind::Internal in the reference's
    // terms: backend-allocated, graph.rs:109-122). Grow-only.
    infr::ActQ8 act;
    size_t act_cap_elems = 0;
    // The same four arrays inside this device's static scratch (infr_hip_linear_noalloc).
    infr::ActQ8 static_act;
    // MoE scratch
    void* moe_ws = nullptr;
    size_t moe_ws_bytes = 0;
    // Counts reallocations of the scratch above. A recorded launch sequence carries the scratch
    // addresses in its kernel arguments, so a plan replays only while the epoch it was recorded
    // under is still current (Internal scratch is the backend's to keep valid, backend.rs:8-13).
    uint64_t scratch_epoch = 0;
};

// ---- static device scratch of the allocation-free Op::Linear entry point ----
// Quantized activation of up to kStaticActElems elements (tokens rounded up to 32, times in_f
// rounded up to 256):
// codes, then per-32 scales, per-32 sums and per-16 sums, the four arrays of infr::ActQ8 back to
// back. Every device the library runs on holds its own copy of this array at its own address
// until the process ends; the name below is only a host-side handle for hipGetSymbolAddress.
constexpr size_t kStaticActElems = (size_t)4 << 20;
constexpr size_t kStaticActBytes = kStaticActElems + kStaticActElems / 32 * 4 * 2 + kStaticActElems / 16 * 4;
static __device__ __align__(256) unsigned char scratch[kStaticActBytes];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
unsigned char* g_scratch_ptr[kMaxDevices] = {};  // device address of `scratch` per device, 0 = not asked yet

// The device address of this device's copy of `scratch`; `device` must be current.
hipError_t static_scratch_ptr(int device, unsigned char** out) {
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[device]) {
        void* p = nullptr;
        hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        g_scratch_ptr[device] = static_cast<unsigned char*>(p);
    }
    *out = g_scratch_ptr[device];
    return hipSuccess;
}

thread_local std::string g_create_err;
std::atomic<int> g_shutdown_signo{0};

int fail(infr_hip_t* be, int code, const std::string& msg) {
    if (be) be->err = msg;
    else g_create_err = msg;
    return code;
}

#define HIP_TRY(be, expr)                                                                     \
    do {                                                                                      \
        hipError_t e__ = (expr);                                                              \
        if (e__ != hipSuccess)                                                                \
            return fail((be), INFR_HIP_ERR_BACKEND,                                           \
                        std::string(#expr) + ": " + hipGetErrorString(e__));                 \
    } while (0)

// Weight formats Op::Linear has kernels for.
bool is_quant(int dt) {
    switch (dt) {
    case INFR_DTYPE_Q4_0: case INFR_DTYPE_Q4_1: case INFR_DTYPE_Q5_0: case INFR_DTYPE_Q5_1:
    case INFR_DTYPE_Q8_0: case INFR_DTYPE_Q4_K: case INFR_DTYPE_Q5_K: case INFR_DTYPE_Q6_K:
    case INFR_DTYPE_Q2_K: case INFR_DTYPE_Q3_K: case INFR_DTYPE_IQ4_XS: case INFR_DTYPE_MXFP4: case INFR_DTYPE_NVFP4:
    case INFR_DTYPE_TQ1_0: case INFR_DTYPE_TQ2_0: case INFR_DTYPE_IQ4_NL: case INFR_DTYPE_Q2_0: return true;
    default: return false;
    }
}
// Formats Op::MoeFfn's expert banks may hold: every Linear weight format, and plain f32 / f16 / bf16
// rows (expert_acts_kind's Raw arm decodes any of them, crates/infr-cpu/src/moe.rs:42-53).
bool is_moe_quant(int dt) {
    switch (dt) {
    case INFR_DTYPE_Q4_K: case INFR_DTYPE_Q5_K: case INFR_DTYPE_Q6_K: case INFR_DTYPE_Q8_0:
    case INFR_DTYPE_Q4_0: case INFR_DTYPE_Q4_1: case INFR_DTYPE_Q5_0: case INFR_DTYPE_Q5_1:
    case INFR_DTYPE_IQ4_NL: case INFR_DTYPE_Q2_0: case INFR_DTYPE_Q2_K: case INFR_DTYPE_Q3_K:
    case INFR_DTYPE_IQ4_XS: case INFR_DTYPE_MXFP4: case INFR_DTYPE_NVFP4: case INFR_DTYPE_TQ2_0:
    case INFR_DTYPE_TQ1_0:
    case INFR_DTYPE_F32: case INFR_DTYPE_F16: case INFR_DTYPE_BF16:
        return true;
    default: return false;
    }
}
bool act_per32(int dt, size_t in_f) { return infr::act_is_per32(dt, in_f); }
// Row lengths a format accepts: whole weight blocks.
// Unquantized weight rows: Op::Linear multiplies them with dot / dot_f16 / dot_bf16
// (crates/infr-cpu/src/lib.rs:1162-1165, 1443-1462).
bool is_plain(int dt) { return dt == INFR_DTYPE_F32 || dt == INFR_DTYPE_F16 || dt == INFR_DTYPE_BF16; }
size_t in_f_multiple(int dt) {
    if (is_plain(dt)) return 32;  // the row-dot kernel stages whole groups of 32 columns
    int e = 0, b = 0;
    return infr_block_layout(dt, &e, &b) ? (size_t)e : 256;
}
// Blocks per row of the per-block integer stage outputs: per 256 for the K-quants, per 32 otherwise.
size_t stage_blocks(int dt, size_t in_f) {
    return (dt == INFR_DTYPE_Q4_K || dt == INFR_DTYPE_Q5_K || dt == INFR_DTYPE_Q6_K || dt == INFR_DTYPE_Q2_K ||
            dt == INFR_DTYPE_Q3_K || dt == INFR_DTYPE_IQ4_XS || dt == INFR_DTYPE_TQ2_0 || dt == INFR_DTYPE_TQ1_0)
               ? in_f / 256
               : in_f / 32;
}
bool has_two_stages(int dt) { return dt == INFR_DTYPE_Q4_K || dt == INFR_DTYPE_Q5_K || dt == INFR_DTYPE_Q2_K; }

// Activation scratch for m rows: the prefill kernels read tokens in groups of 32.
// Tokens rounded up to the 32 of a tile, rows to the 256 of a step (the tiled per-32 quantizer pads
// rows that end inside a step).
static size_t act_scratch_elems(size_t m, size_t in_f) { return (m + 31) / 32 * 32 * ((in_f + 255) / 256 * 256); }
// What an Op::Linear needs of it: unquantized weights quantize nothing, but an op in place on its x
// parks a copy of x there (4 bytes per element).
static size_t linear_scratch_elems(int dtype, size_t m, size_t in_f) {
    return is_plain(dtype) ? m * in_f * sizeof(float) : act_scratch_elems(m, in_f);
}

static bool is_elementwise(int kind) { return kind >= INFR_OP_RMS_NORM && kind <= INFR_OP_ADD; }

// Bound f32 operands of an elementwise op, validated against the sizes the op addresses.
struct ElementwiseArgs {
    const float* x = nullptr;    // RmsNorm x / GatedAct gate / GatedActFused gu / Add a
    const float* aux = nullptr;  // RmsNorm weight / GatedAct up / Add b
    float* dst = nullptr;
    size_t x_elems = 0, aux_elems = 0, dst_elems = 0;
};

static int check_elementwise(infr_hip_t* be, const infr_hip_op_t& op, infr_hip_buffer_t* const* bindings,
                             ElementwiseArgs* a) {
    const size_t rows = op.m, n = op.in_f;
    const infr_hip_buffer_t* xb = bindings[op.x];
    const infr_hip_buffer_t* db = bindings[op.dst];
    const infr_hip_buffer_t* ab = nullptr;
    a->dst_elems = rows * n;
    switch (op.kind) {
    case INFR_OP_RMS_NORM:
    case INFR_OP_RMS_NORM_ADD:
        ab = bindings[op.weight];
        a->x_elems = rows * n;
        a->aux_elems = n;
        break;
    case INFR_OP_GATED_ACT: {
        ab = bindings[op.aux];
        const size_t grow = (op.gate_block_width > 0 || op.gate_stride > 0) ? op.gate_stride : n;
        // last gate element addressed: the interleaved layout reaches 2x the row's width
        const size_t glast = op.gate_block_width > 0 ? (n / (op.gate_block_width / 2)) * op.gate_block_width : n;
        a->x_elems = (rows - 1) * grow + glast;
        a->aux_elems = (rows - 1) * (op.up_stride ? op.up_stride : n) + op.up_off + n;
        if (op.gate_block_width > 0 && n % (op.gate_block_width / 2) != 0)
            return fail(be, INFR_HIP_ERR_UNSUPPORTED, "gated_act: nff is not a whole number of gate blocks");
        break;
    }
    case INFR_OP_GATED_ACT_FUSED:
        a->x_elems = rows * 2 * n;
        break;
    default:  // Add
        ab = bindings[op.aux];
        a->x_elems = a->aux_elems = rows * n;
        break;
    }
    if (!xb || !db || (a->aux_elems && !ab)) return fail(be, INFR_HIP_ERR_INVALID, "elementwise op: unbound buffer");
    if (xb->len < a->x_elems * 4 || db->len < a->dst_elems * 4 || (ab && ab->len < a->aux_elems * 4))
        return fail(be, INFR_HIP_ERR_INVALID, "elementwise op: buffer too small for the shape");
    a->x = static_cast<const float*>(xb->ptr);
    a->aux = ab ? static_cast<const float*>(ab->ptr) : nullptr;
    a->dst = static_cast<float*>(db->ptr);
    return INFR_HIP_OK;
}

static int enqueue_elementwise(infr_hip_t* be, const infr_hip_op_t& op, const ElementwiseArgs& a) {
    switch (op.kind) {
    case INFR_OP_RMS_NORM:
    case INFR_OP_RMS_NORM_ADD:
        infr::launch_rms_norm(a.x, a.aux, a.dst, op.m, op.in_f, op.eps, op.kind == INFR_OP_RMS_NORM_ADD, be->stream);
        break;
    case INFR_OP_GATED_ACT:
        infr::launch_gated_act(a.x, a.aux, a.dst,
                               infr::GatedActShape{op.m, op.in_f, op.act, op.up_off, op.up_stride, op.gate_stride,
                                                   op.gate_block_width, op.has_clamp, op.clamp},
                               be->stream);
        break;
    case INFR_OP_GATED_ACT_FUSED:
        // the combined buffer is the strided form of the same kernel: gate rows 2*nff apart, up at +nff
        infr::launch_gated_act(a.x, a.x, a.dst,
                               infr::GatedActShape{op.m, op.in_f, op.act, op.in_f, 2 * op.in_f, 2 * op.in_f, 0,
                                                   op.has_clamp, op.clamp},
                               be->stream);
        break;
    default:
        infr::launch_add(a.x, a.aux, a.dst, (size_t)op.m * op.in_f, be->stream);
        break;
    }
    HIP_TRY(be, hipGetLastError());
    return INFR_HIP_OK;
}

// Linears that are launched on their own, outside the fused / grouped decode and small-batch
// launches: one token of a format whose CPU arm multiplies f32 activations, and rows too long for
// the decode mapping (those go to the prefill kernels at any m).
static bool runs_alone(int dtype, size_t m, size_t in_f) {
    return is_plain(dtype) || infr::gemv_takes_f32_activations(dtype, m) || infr::gemv_row_too_long(dtype, in_f);
}

// Ops that run in small-batch groups inside plans: the K-split MFMA kernels take Q4_K up to 32
// rows, and Q4_K, Q5_K, Q6_K, Q8_0 and Q2_0 as far as their 16-token kernel is the route
// (mmq_skinny16_takes: up to 32..128 rows by format and shape); the dot4 batch kernel the other
// formats up to 8.
static bool small_batch(const infr_hip_op_t& op) {
    if (op.m < 2 || is_plain(op.w_dtype) || infr::gemv_row_too_long(op.w_dtype, op.in_f)) return false;
    if (op.w_dtype == INFR_DTYPE_Q4_K && op.m <= 32) return true;
    return op.m <= 8 || infr::mmq_skinny16_takes(op.w_dtype, op.m, op.in_f, op.out_f);
}

// (Re)allocates a device table when it grew and enqueues the copy on the backend stream.
template <typename T>
static int upload_table(infr_hip_t* be, const std::vector<T>& host, T** dev, size_t* cap) {
    if (host.empty()) return INFR_HIP_OK;
    if (host.size() > *cap) {
        if (*dev) (void)hipFree(*dev);
        *dev = nullptr;
        *cap = 0;
        HIP_TRY(be, hipMalloc((void**)dev, sizeof(T) * host.size()));
        *cap = host.size();
    }
    HIP_TRY(be, hipMemcpyAsync(*dev, host.data(), sizeof(T) * host.size(), hipMemcpyHostToDevice, be->stream));
    return INFR_HIP_OK;
}

int ensure_act(infr_hip_t* be, size_t elems) {
    if (elems <= be->act_cap_elems) return INFR_HIP_OK;
    HIP_TRY(be, hipStreamSynchronize(be->stream));
    ++be->scratch_epoch;
    if (be->act.qs) {
        (void)hipFree(be->act.qs);
        (void)hipFree(be->act.d);
        (void)hipFree(be->act.bsums);
        (void)hipFree(be->act.bsums16);
        be->act = infr::ActQ8{};
        be->act_cap_elems = 0;
    }
    const size_t cap = (elems + 4095) / 4096 * 4096;
    HIP_TRY(be, hipMalloc((void**)&be->act.qs, cap));
    HIP_TRY(be, hipMalloc((void**)&be->act.d, cap / 32 * sizeof(float)));
    HIP_TRY(be, hipMalloc((void**)&be->act.bsums, cap / 32 * sizeof(int32_t)));
    HIP_TRY(be, hipMalloc((void**)&be->act.bsums16, cap / 16 * sizeof(int32_t)));
    be->act_cap_elems = cap;
    return INFR_HIP_OK;
}

struct LinearArgs {
    const uint8_t* wrows;  // first selected row
    size_t bpr;
};

// Shape/size validation shared by linear and linear_int_stages
// (crates/infr-cpu/src/lib.rs:1003-1008 for the row slicing).
int check_linear(infr_hip_t* be, int dtype, const infr_hip_buffer_t* w, size_t w_numel,
                 size_t w_off, const infr_hip_buffer_t* x, size_t m, size_t in_f, size_t out_f,
                 LinearArgs* out) {
    if (!w || !x) return fail(be, INFR_HIP_ERR_INVALID, "linear: unbound buffer");
    if (!is_quant(dtype) && !is_plain(dtype))
        return fail(be, INFR_HIP_ERR_UNSUPPORTED,
                    "linear: weight dtype " + std::to_string(dtype) + " has no kernel");
    if (m == 0 || in_f == 0 || out_f == 0) return fail(be, INFR_HIP_ERR_INVALID, "linear: empty shape");
    int qpb = 0, bpb = 0;
    infr_block_layout(dtype, &qpb, &bpb);
    // The per-256 activation quantizer drops a sub-256 tail (quant.rs:28); reject, never truncate.
    const size_t need = in_f_multiple(dtype);
    if (in_f % need != 0)
        return fail(be, INFR_HIP_ERR_UNSUPPORTED,
                    "linear: in_f " + std::to_string(in_f) + " is not a multiple of " +
                        std::to_string(need) + " for dtype " + std::to_string(dtype));
    if (w_numel == 0 || w_numel % in_f != 0 || w_off % in_f != 0)
        return fail(be, INFR_HIP_ERR_INVALID, "linear: w_numel / w_off not row-aligned");
    const size_t total_rows = w_numel / in_f;
    const size_t bpr = in_f / (size_t)qpb * (size_t)bpb;
    if (w->len < total_rows * bpr)
        return fail(be, INFR_HIP_ERR_INVALID, "linear: weight buffer smaller than its declared shape");
    const size_t row0 = w_off / in_f;
    if (row0 + out_f > total_rows)
        return fail(be, INFR_HIP_ERR_INVALID, "linear: w_off + out_f exceeds the weight's rows");
    if (x->len < m * in_f * sizeof(float))
        return fail(be, INFR_HIP_ERR_INVALID, "linear: x buffer too small");
    if (in_f > 0x7FFFFFFFull || out_f > 0x7FFFFFFFull || m > 0x7FFFFFFFull)
        return fail(be, INFR_HIP_ERR_UNSUPPORTED, "linear: dimension exceeds 2^31");
    out->wrows = static_cast<const uint8_t*>(w->ptr) + row0 * bpr;
    out->bpr = bpr;
    // The kernels fetch blocks with 2-, 4- or 16-byte loads according to the block stride and
    // assume the first row starts where a row stride of that alignment would put it.
    // (MXFP4's 17-byte blocks sit at any byte: its kernels fetch the aligned dwords around a block)
    const uintptr_t align = dtype == INFR_DTYPE_MXFP4 ? 1 : (bpr % 16 == 0 ? 16 : (bpr % 4 == 0 ? 4 : 2));
    if (reinterpret_cast<uintptr_t>(out->wrows) % align != 0)
        return fail(be, INFR_HIP_ERR_INVALID,
                    "linear: weight rows start at an address that is not " + std::to_string(align) + "-byte aligned");
    return INFR_HIP_OK;
}

// A Linear whose dst overlaps its x (the CPU arm computes into a fresh vector first, lib.rs:985-1492,
// so that is a legal graph). The one-launch decode kernels read x in every workgroup while others
// already store y, so such an op takes a path that consumes x before anything is written.
static bool floats_overlap(const float* a, size_t na, const float* b, size_t nb) {
    return a < b + nb && b < a + na;
}

int enqueue_linear(infr_hip_t* be, int dtype, const LinearArgs& la, const float* x, float* y,
                   size_t m, size_t in_f, size_t out_f, const infr::IntStages& st, const infr::ActQ8& act,
                   infr::QuantCache* qc = nullptr) {
    bool ok;
    // (the branches that do not quantize may park a copy of x in the scratch)
    if (qc && (is_plain(dtype) || infr::gemv_takes_f32_activations(dtype, m))) *qc = infr::QuantCache{};
    if (is_plain(dtype)) {
        if (st.a) return fail(be, INFR_HIP_ERR_UNSUPPORTED, "int_stages: unquantized weights have no integer stage");
        if (floats_overlap(x, m * in_f, y, m * out_f)) {
            // in place: every workgroup reads x while others store y; multiply a copy of x
            float* copy = reinterpret_cast<float*>(act.qs);
            HIP_TRY(be, hipMemcpyAsync(copy, x, m * in_f * sizeof(float), hipMemcpyDeviceToDevice, be->stream));
            x = copy;
        }
        ok = infr::launch_linear_plain_rows(dtype, la.wrows, x, y, m, in_f, out_f, be->stream);
    } else if (infr::gemv_takes_f32_activations(dtype, m)) {
        if (st.a)
            return fail(be, INFR_HIP_ERR_UNSUPPORTED,
                        "int_stages: one token of dtype " + std::to_string(dtype) + " has no integer stage");
        if (floats_overlap(x, m * in_f, y, m * out_f)) {
            // in place: the kernel reads a copy of x parked in the activation scratch
            float* copy = reinterpret_cast<float*>(act.qs);
            HIP_TRY(be, hipMemcpyAsync(copy, x, m * in_f * sizeof(float), hipMemcpyDeviceToDevice, be->stream));
            x = copy;
        }
        ok = infr::launch_gemv_f32act(dtype, la.wrows, la.bpr, x, y, in_f, out_f, be->stream);
    } else {
        // quantizes x into the scratch in the layout its kernel reads, then multiplies
        ok = infr::launch_mmq(dtype, la.wrows, la.bpr, x, act, y, m, in_f, out_f, st, be->props.multiProcessorCount, be->stream, qc);
        if (qc && floats_overlap(x, m * in_f, y, m * out_f)) *qc = infr::QuantCache{};  // x is overwritten
    }
    if (!ok)
        return fail(be, INFR_HIP_ERR_UNSUPPORTED,
                    "linear: no kernel for dtype " + std::to_string(dtype) + " at in_f " +
                        std::to_string(in_f) + ", m " + std::to_string(m));
    HIP_TRY(be, hipGetLastError());
    return INFR_HIP_OK;
}

// One fused decode launch (quantize x in LDS + GEMV) for a single m == 1 Linear.
int enqueue_gemv_single(infr_hip_t* be, int dtype, size_t in_f, const infr::GemvOpDesc& op) {
    infr::GemvGroupPlan gp;
    if (!infr::plan_gemv_group(dtype, in_f, &op, 1, &gp) ||
        !infr::launch_gemv_fused(dtype, in_f, &op, 1, nullptr, gp, be->stream))
        return fail(be, INFR_HIP_ERR_UNSUPPORTED,
                    "linear: no decode kernel for dtype " + std::to_string(dtype) + " at in_f " +
                        std::to_string(in_f));
    HIP_TRY(be, hipGetLastError());
    return INFR_HIP_OK;
}

struct EmbedArgs {
    const uint8_t* table;
    size_t bpr, total_rows;
};

// Shape/size validation of an Op::EmbedGather (table rows as lib.rs:2099-2100 derives them).
int check_embed(infr_hip_t* be, int dtype, const infr_hip_buffer_t* table, size_t table_numel,
                const infr_hip_buffer_t* ids, size_t rows, size_t ne, const infr_hip_buffer_t* dst,
                EmbedArgs* out) {
    if (!table || !ids || !dst) return fail(be, INFR_HIP_ERR_INVALID, "embed_gather: unbound buffer");
    int qpb = 0, bpb = 0;
    if (!infr::embed_gather_supported(dtype) || !infr_block_layout(dtype, &qpb, &bpb))
        return fail(be, INFR_HIP_ERR_UNSUPPORTED, "embed_gather: table dtype " + std::to_string(dtype) + " has no decoder");
    if (rows == 0 || ne == 0 || ne % (size_t)qpb != 0 || table_numel == 0 || table_numel % ne != 0)
        return fail(be, INFR_HIP_ERR_UNSUPPORTED, "embed_gather: rows must be whole blocks and the table whole rows");
    if (ne > 0x7FFFFFFFull || rows > 65535 || table_numel / ne > 0x7FFFFFFFull)
        return fail(be, INFR_HIP_ERR_UNSUPPORTED, "embed_gather: dimension out of range");
    out->total_rows = table_numel / ne;
    out->bpr = ne / (size_t)qpb * (size_t)bpb;
    out->table = static_cast<const uint8_t*>(table->ptr);
    if (table->len < out->total_rows * out->bpr)
        return fail(be, INFR_HIP_ERR_INVALID, "embed_gather: table buffer smaller than its declared shape");
    if (ids->len < rows * sizeof(int32_t) || dst->len < rows * ne * sizeof(float))
        return fail(be, INFR_HIP_ERR_INVALID, "embed_gather: ids or dst buffer too small");
    if (reinterpret_cast<uintptr_t>(out->table) % 2 != 0)
        return fail(be, INFR_HIP_ERR_INVALID, "embed_gather: table is not 2-byte aligned");
    return INFR_HIP_OK;
}

int check_latch(infr_hip_t* be) {
    if (g_shutdown_signo.load(std::memory_order_relaxed) != 0)
        return fail(be, INFR_HIP_ERR_ABORTED, "shutdown requested");
    return INFR_HIP_OK;
}

}  // namespace

extern "C" {

int infr_hip_create(int device, infr_hip_t** out) {
    if (!out) return fail(nullptr, INFR_HIP_ERR_INVALID, "create: out is null");
    *out = nullptr;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0)
        return fail(nullptr, INFR_HIP_ERR_BACKEND,
                    std::string("no HIP device: ") + (e != hipSuccess ? hipGetErrorString(e) : "count is 0"));
    if (device < 0 || device >= n || device >= kMaxDevices)
        return fail(nullptr, INFR_HIP_ERR_INVALID, "create: device index out of range");
    infr_hip_t* be = new (std::nothrow) infr_hip();
    if (!be) return fail(nullptr, INFR_HIP_ERR_OTHER, "create: out of host memory");
    be->device = device;
    auto bail = [&](const char* what, hipError_t err) {
        std::string msg = std::string(what) + ": " + hipGetErrorString(err);
        infr_hip_destroy(be);
        return fail(nullptr, INFR_HIP_ERR_BACKEND, msg);
    };
    if ((e = hipSetDevice(device)) != hipSuccess) return bail("hipSetDevice", e);
    if ((e = hipGetDeviceProperties(&be->props, device)) != hipSuccess)
        return bail("hipGetDeviceProperties", e);
    if (std::strncmp(be->props.gcnArchName, "gfx950", 6) != 0) {
        std::string msg = std::string("device is ") + be->props.gcnArchName +
                          ", this library carries gfx950 code only";
        infr_hip_destroy(be);
        return fail(nullptr, INFR_HIP_ERR_UNSUPPORTED, msg);
    }
    // this device's copy of the static scratch (the device is current here)
    unsigned char* sp = nullptr;
    if ((e = static_scratch_ptr(device, &sp)) != hipSuccess) return bail("hipGetSymbolAddress(scratch)", e);
    be->static_act.qs = reinterpret_cast<int8_t*>(sp);
    be->static_act.d = reinterpret_cast<float*>(sp + kStaticActElems);
    be->static_act.bsums = reinterpret_cast<int32_t*>(sp + kStaticActElems + kStaticActElems / 32 * 4);
    be->static_act.bsums16 = reinterpret_cast<int32_t*>(sp + kStaticActElems + kStaticActElems / 32 * 4 * 2);
    if ((e = hipStreamCreateWithFlags(&be->stream, hipStreamNonBlocking)) != hipSuccess)
        return bail("hipStreamCreate", e);
    if ((e = hipEventCreate(&be->ev0)) != hipSuccess) return bail("hipEventCreate", e);
    if ((e = hipEventCreate(&be->ev1)) != hipSuccess) return bail("hipEventCreate", e);
    be->name = std::string("hip:") + be->props.gcnArchName;
    *out = be;
    return INFR_HIP_OK;
}

void infr_hip_destroy(infr_hip_t* be) {
    if (!be) return;
    (void)hipSetDevice(be->device);
    if (be->stream) (void)hipStreamSynchronize(be->stream);
    if (be->act.qs) {
        (void)hipFree(be->act.qs);
        (void)hipFree(be->act.d);
        (void)hipFree(be->act.bsums);
        (void)hipFree(be->act.bsums16);
    }
    if (be->moe_ws) (void)hipFree(be->moe_ws);
    if (be->ev0) (void)hipEventDestroy(be->ev0);
    if (be->ev1) (void)hipEventDestroy(be->ev1);
    if (be->stream) (void)hipStreamDestroy(be->stream);
    delete be;
}

const char* infr_hip_name(const infr_hip_t* be) { return be ? be->name.c_str() : "hip"; }

int infr_hip_capabilities(const infr_hip_t* be, infr_hip_caps_t* out) {
    if (!be || !out) return INFR_HIP_ERR_INVALID;
    std::memset(out, 0, sizeof *out);
    out->i8 = 1;
    out->i8_dot = 1;
    out->coopmat_i8_m = 32;
    out->coopmat_i8_n = 32;
    out->coopmat_i8_k = 32;
    out->decode_replay = 1;
    out->combined_gu = 1;   // a Linear onto [gate | up] followed by Op::GatedActFused is a plan op here
    out->embed_gather = 1;  // Op::EmbedGather decodes table rows on the device
    out->graph_input_inplace = 1;
    out->unified_memory = 0;
    out->device_memory_bytes = be->props.totalGlobalMem;
    out->compute_units = be->props.multiProcessorCount;
    std::snprintf(out->device_name, sizeof out->device_name, "%s", be->props.name);
    return INFR_HIP_OK;
}

const char* infr_hip_last_error(const infr_hip_t* be) {
    return be ? be->err.c_str() : g_create_err.c_str();
}

static int alloc_impl(infr_hip_t* be, size_t bytes, bool zero, infr_hip_buffer_t** out) {
    if (!be || !out) return fail(be, INFR_HIP_ERR_INVALID, "alloc: null argument");
    *out = nullptr;
    infr_hip_buffer_t* b = new (std::nothrow) infr_hip_buffer();
    if (!b) return fail(be, INFR_HIP_ERR_OTHER, "alloc: out of host memory");
    const size_t n = bytes ? bytes : 4;  // the reference's harness allocs max(len, 4)
    hipError_t e = hipMalloc(&b->ptr, n);
    if (e != hipSuccess) {
        delete b;
        return fail(be, INFR_HIP_ERR_BACKEND,
                    "hipMalloc(" + std::to_string(n) + "): " + hipGetErrorString(e));
    }
    if (zero) {
        e = hipMemsetAsync(b->ptr, 0, n, be->stream);
        if (e != hipSuccess) {
            (void)hipFree(b->ptr);
            delete b;
            return fail(be, INFR_HIP_ERR_BACKEND, std::string("hipMemsetAsync: ") + hipGetErrorString(e));
        }
    }
    b->len = bytes;
    b->owned = true;
    *out = b;
    return INFR_HIP_OK;
}

int infr_hip_alloc(infr_hip_t* be, size_t bytes, int /*usage*/, infr_hip_buffer_t** out) {
    return alloc_impl(be, bytes, true, out);
}
int infr_hip_alloc_uninit(infr_hip_t* be, size_t bytes, int /*usage*/, infr_hip_buffer_t** out) {
    return alloc_impl(be, bytes, false, out);
}

int infr_hip_wrap(infr_hip_t* be, void* device_ptr, size_t bytes, infr_hip_buffer_t** out) {
    if (!be || !out || !device_ptr) return fail(be, INFR_HIP_ERR_INVALID, "wrap: null argument");
    infr_hip_buffer_t* b = new (std::nothrow) infr_hip_buffer();
    if (!b) return fail(be, INFR_HIP_ERR_OTHER, "wrap: out of host memory");
    b->ptr = device_ptr;
    b->len = bytes;
    b->owned = false;
    *out = b;
    return INFR_HIP_OK;
}

void infr_hip_free(infr_hip_t* be, infr_hip_buffer_t* buf) {
    if (!buf) return;
    if (buf->owned && buf->ptr) {
        if (be && be->stream) (void)hipStreamSynchronize(be->stream);
        (void)hipFree(buf->ptr);
    }
    delete buf;
}

size_t infr_hip_buffer_len(const infr_hip_buffer_t* buf) { return buf ? buf->len : 0; }
uint64_t infr_hip_buffer_device_addr(const infr_hip_buffer_t* buf) {
    return buf ? (uint64_t)(uintptr_t)buf->ptr : 0;
}

int infr_hip_upload_at(infr_hip_t* be, infr_hip_buffer_t* dst, size_t dst_off, const void* src,
                       size_t n) {
    if (!be || !dst || (!src && n)) return fail(be, INFR_HIP_ERR_INVALID, "upload: null argument");
    if (dst_off > dst->len || n > dst->len - dst_off)
        return fail(be, INFR_HIP_ERR_BACKEND,
                    "upload of " + std::to_string(n) + " bytes at " + std::to_string(dst_off) +
                        " exceeds the " + std::to_string(dst->len) + "-byte buffer");
    if (n == 0) return INFR_HIP_OK;
    HIP_TRY(be, hipMemcpyAsync(static_cast<uint8_t*>(dst->ptr) + dst_off, src, n,
                               hipMemcpyHostToDevice, be->stream));
    HIP_TRY(be, hipStreamSynchronize(be->stream));  // src may be reused as soon as we return
    return INFR_HIP_OK;
}
int infr_hip_upload(infr_hip_t* be, infr_hip_buffer_t* dst, const void* src, size_t n) {
    return infr_hip_upload_at(be, dst, 0, src, n);
}

int infr_hip_download_at(infr_hip_t* be, const infr_hip_buffer_t* src, size_t src_off, void* dst,
                         size_t n) {
    if (!be || !src || (!dst && n)) return fail(be, INFR_HIP_ERR_INVALID, "download: null argument");
    if (src_off > src->len || n > src->len - src_off)
        return fail(be, INFR_HIP_ERR_BACKEND,
                    "download of " + std::to_string(n) + " bytes at " + std::to_string(src_off) +
                        " exceeds the " + std::to_string(src->len) + "-byte buffer");
    if (n) {
        HIP_TRY(be, hipMemcpyAsync(dst, static_cast<const uint8_t*>(src->ptr) + src_off, n,
                                   hipMemcpyDeviceToHost, be->stream));
    }
    HIP_TRY(be, hipStreamSynchronize(be->stream));
    return INFR_HIP_OK;
}
int infr_hip_download(infr_hip_t* be, const infr_hip_buffer_t* src, void* dst, size_t n) {
    return infr_hip_download_at(be, src, 0, dst, n);
}

int infr_hip_copy_buffer(infr_hip_t* be, const infr_hip_buffer_t* src, infr_hip_buffer_t* dst,
                         size_t bytes) {
    if (!be || !src || !dst) return fail(be, INFR_HIP_ERR_INVALID, "copy_buffer: null argument");
    // check_copy_bytes (backend.rs:23-30): an oversize copy is an error, not a fault.
    if (bytes > src->len || bytes > dst->len)
        return fail(be, INFR_HIP_ERR_BACKEND,
                    "copy_buffer: " + std::to_string(bytes) + " bytes exceeds src (" +
                        std::to_string(src->len) + ") or dst (" + std::to_string(dst->len) + ")");
    if (bytes)
        HIP_TRY(be, hipMemcpyAsync(dst->ptr, src->ptr, bytes, hipMemcpyDeviceToDevice, be->stream));
    return INFR_HIP_OK;
}

int infr_hip_sync(infr_hip_t* be) {
    if (!be) return INFR_HIP_ERR_INVALID;
    HIP_TRY(be, hipStreamSynchronize(be->stream));
    return INFR_HIP_OK;
}

int infr_hip_linear(infr_hip_t* be, int dtype, const infr_hip_buffer_t* w, size_t w_numel,
                    size_t w_off, const infr_hip_buffer_t* x, infr_hip_buffer_t* dst, size_t m,
                    size_t in_f, size_t out_f) {
    if (!be) return INFR_HIP_ERR_INVALID;
    if (int rc = check_latch(be)) return rc;
    LinearArgs la;
    if (int rc = check_linear(be, dtype, w, w_numel, w_off, x, m, in_f, out_f, &la)) return rc;
    if (!dst || dst->len < m * out_f * sizeof(float))
        return fail(be, INFR_HIP_ERR_INVALID, "linear: dst buffer missing or too small");
    const bool in_place = floats_overlap(static_cast<const float*>(x->ptr), m * in_f, static_cast<float*>(dst->ptr), m * out_f);
    if (m == 1 && !runs_alone(dtype, m, in_f) && !in_place) {
        // decode: one fused launch (quantize x in LDS + GEMV)
        const infr::GemvOpDesc op{la.wrows, static_cast<const float*>(x->ptr),
                                  static_cast<float*>(dst->ptr), la.bpr, (int32_t)out_f};
        return enqueue_gemv_single(be, dtype, in_f, op);
    }
    if (int rc = ensure_act(be, linear_scratch_elems(dtype, m, in_f))) return rc;
    return enqueue_linear(be, dtype, la, static_cast<const float*>(x->ptr),
                          static_cast<float*>(dst->ptr), m, in_f, out_f, infr::IntStages{}, be->act);
}

int infr_hip_linear_noalloc(infr_hip_t* be, int dtype, const infr_hip_buffer_t* w, size_t w_numel,
                            size_t w_off, const infr_hip_buffer_t* x, infr_hip_buffer_t* dst, size_t m,
                            size_t in_f, size_t out_f) {
    if (!be) return INFR_HIP_ERR_INVALID;
    if (int rc = check_latch(be)) return rc;
    LinearArgs la;
    if (int rc = check_linear(be, dtype, w, w_numel, w_off, x, m, in_f, out_f, &la)) return rc;
    if (!dst || dst->len < m * out_f * sizeof(float))
        return fail(be, INFR_HIP_ERR_INVALID, "linear_noalloc: dst buffer missing or too small");
    const bool in_place = floats_overlap(static_cast<const float*>(x->ptr), m * in_f, static_cast<float*>(dst->ptr), m * out_f);
    if (m == 1 && !runs_alone(dtype, m, in_f) && !in_place) {
        // decode: the fused launch keeps the quantized activation in LDS and needs no scratch
        const infr::GemvOpDesc op{la.wrows, static_cast<const float*>(x->ptr),
                                  static_cast<float*>(dst->ptr), la.bpr, (int32_t)out_f};
        return enqueue_gemv_single(be, dtype, in_f, op);
    }
    if (linear_scratch_elems(dtype, m, in_f) > kStaticActElems)
        return fail(be, INFR_HIP_ERR_UNSUPPORTED,
                    "linear_noalloc: " + std::to_string(linear_scratch_elems(dtype, m, in_f)) +
                        " activation elements (tokens rounded up to 32, times in_f rounded up to 256) exceed the static scratch of " +
                        std::to_string(kStaticActElems));
    return enqueue_linear(be, dtype, la, static_cast<const float*>(x->ptr), static_cast<float*>(dst->ptr), m,
                          in_f, out_f, infr::IntStages{}, be->static_act);
}

int infr_hip_embed_gather(infr_hip_t* be, int dtype, const infr_hip_buffer_t* table, size_t table_numel,
                          const infr_hip_buffer_t* ids, size_t rows, size_t ne, float scale,
                          infr_hip_buffer_t* dst) {
    if (!be) return INFR_HIP_ERR_INVALID;
    if (int rc = check_latch(be)) return rc;
    EmbedArgs ea;
    if (int rc = check_embed(be, dtype, table, table_numel, ids, rows, ne, dst, &ea)) return rc;
    infr::launch_embed_gather(dtype, ea.table, ea.bpr, ea.total_rows, static_cast<const int32_t*>(ids->ptr), rows,
                              ne, scale, static_cast<float*>(dst->ptr), be->stream);
    HIP_TRY(be, hipGetLastError());
    return INFR_HIP_OK;
}

int infr_hip_linear_int_stages(infr_hip_t* be, int dtype, const infr_hip_buffer_t* w,
                               size_t w_numel, size_t w_off, const infr_hip_buffer_t* x, size_t m,
                               size_t in_f, size_t out_f, infr_hip_buffer_t* a,
                               infr_hip_buffer_t* b) {
    if (!be) return INFR_HIP_ERR_INVALID;
    if (int rc = check_latch(be)) return rc;
    LinearArgs la;
    if (int rc = check_linear(be, dtype, w, w_numel, w_off, x, m, in_f, out_f, &la)) return rc;
    if (dtype == INFR_DTYPE_NVFP4)
        return fail(be, INFR_HIP_ERR_UNSUPPORTED, "int_stages: NVFP4 has four integers per block, not one");
    const size_t blocks = stage_blocks(dtype, in_f);
    const size_t need = m * out_f * blocks * sizeof(int32_t);
    if (!a || a->len < need) return fail(be, INFR_HIP_ERR_INVALID, "int_stages: buffer a too small");
    if (has_two_stages(dtype) && (!b || b->len < need))
        return fail(be, INFR_HIP_ERR_INVALID, "int_stages: Q4_K / Q5_K need buffer b");
    if (int rc = ensure_act(be, act_scratch_elems(m, in_f))) return rc;
    // y is not wanted here; use a transient output
    float* y = nullptr;
    HIP_TRY(be, hipMalloc((void**)&y, m * out_f * sizeof(float)));
    infr::IntStages st;
    st.a = static_cast<int32_t*>(a->ptr);
    st.b = b ? static_cast<int32_t*>(b->ptr) : nullptr;
    int rc;
    if (m == 1 && !runs_alone(dtype, m, in_f)) {
        // one token: the decode kernel infr_hip_linear launches, writing its integers as well
        infr::GemvOpDesc op{la.wrows, static_cast<const float*>(x->ptr), y, la.bpr, (int32_t)out_f};
        op.st_a = st.a;
        op.st_b = st.b;
        rc = enqueue_gemv_single(be, dtype, in_f, op);
    } else {
        rc = enqueue_linear(be, dtype, la, static_cast<const float*>(x->ptr), y, m, in_f, out_f, st, be->act);
    }
    (void)hipStreamSynchronize(be->stream);
    (void)hipFree(y);
    return rc;
}

static int quantize_impl(infr_hip_t* be, bool per32, const infr_hip_buffer_t* x, size_t m, size_t k,
                         infr_hip_buffer_t* qs, infr_hip_buffer_t* d, infr_hip_buffer_t* bsums,
                         infr_hip_buffer_t* bsums16) {
    if (!be) return INFR_HIP_ERR_INVALID;
    if (int rc = check_latch(be)) return rc;
    if (!x || !qs || !d || !bsums) return fail(be, INFR_HIP_ERR_INVALID, "quantize: unbound buffer");
    const size_t blk = per32 ? 32 : 256;
    if (m == 0 || k == 0 || k % blk != 0)
        return fail(be, INFR_HIP_ERR_UNSUPPORTED,
                    "quantize: k " + std::to_string(k) + " is not a multiple of " + std::to_string(blk));
    const size_t n = m * k;
    if (x->len < n * 4 || qs->len < n || d->len < n / blk * 4 || bsums->len < n / 32 * 4 ||
        (bsums16 && bsums16->len < n / 16 * 4))
        return fail(be, INFR_HIP_ERR_INVALID, "quantize: a buffer is too small");
    infr::ActQ8 out;
    out.qs = static_cast<int8_t*>(qs->ptr);
    out.d = static_cast<float*>(d->ptr);
    out.bsums = static_cast<int32_t*>(bsums->ptr);
    out.bsums16 = bsums16 ? static_cast<int32_t*>(bsums16->ptr) : nullptr;
    infr::launch_quantize_q8(static_cast<const float*>(x->ptr), m, k, per32, out, be->stream);
    HIP_TRY(be, hipGetLastError());
    return INFR_HIP_OK;
}

int infr_hip_quantize_q8(infr_hip_t* be, const infr_hip_buffer_t* x, size_t m, size_t k,
                         infr_hip_buffer_t* qs, infr_hip_buffer_t* d, infr_hip_buffer_t* bsums,
                         infr_hip_buffer_t* bsums16) {
    return quantize_impl(be, false, x, m, k, qs, d, bsums, bsums16);
}
int infr_hip_quantize_q8_32(infr_hip_t* be, const infr_hip_buffer_t* x, size_t m, size_t k,
                            infr_hip_buffer_t* qs, infr_hip_buffer_t* d, infr_hip_buffer_t* bsum) {
    return quantize_impl(be, true, x, m, k, qs, d, bsum, nullptr);
}

static int ensure_moe_ws(infr_hip_t* be, size_t bytes) {
    if (bytes <= be->moe_ws_bytes) return INFR_HIP_OK;
    HIP_TRY(be, hipStreamSynchronize(be->stream));
    ++be->scratch_epoch;
    if (be->moe_ws) (void)hipFree(be->moe_ws);
    be->moe_ws = nullptr;
    be->moe_ws_bytes = 0;
    HIP_TRY(be, hipMalloc(&be->moe_ws, bytes));
    // the router's ticket counters live at the start and must read zero before the first op;
    // every op leaves them at zero again
    HIP_TRY(be, hipMemset(be->moe_ws, 0, bytes));
    be->moe_ws_bytes = bytes;
    return INFR_HIP_OK;
}

static size_t expert_bank_bytes(int dtype, size_t rows, size_t in_f) {
    int qpb = 0, bpb = 0;
    if (!infr_block_layout(dtype, &qpb, &bpb) || in_f % (size_t)qpb != 0) return 0;
    return rows * (in_f / (size_t)qpb) * (size_t)bpb;
}

// Validates an Op::MoeFfn and fills the launch structures. Every field of the op is either carried
// into the launch or refused here: none is read as another setting.
static int check_moe(infr_hip_t* be, const infr_hip_moe_params_t* p, const infr_hip_buffer_t* x,
                     const infr_hip_buffer_t* router_x, const infr_hip_buffer_t* router,
                     const infr_hip_buffer_t* gate, const infr_hip_buffer_t* up,
                     const infr_hip_buffer_t* down, const infr_hip_moe_optional_t* opt, infr_hip_buffer_t* dst,
                     infr_hip_buffer_t* sel_idx, infr_hip_buffer_t* sel_w, infr::MoeShape* s,
                     infr::MoeBuffers* b) {
    if (!p) return fail(be, INFR_HIP_ERR_INVALID, "moe_ffn: null parameters");
    const bool fused = p->fused_gate_up != 0;
    if (!x || !router_x || !router || !gate || (!up && !fused) || !down || !dst)
        return fail(be, INFR_HIP_ERR_INVALID, "moe_ffn: unbound buffer");
    if (!p->ne || !p->n_expert || !p->n_used || !p->n_ff_exp || !p->rows || p->n_used > p->n_expert)
        return fail(be, INFR_HIP_ERR_INVALID, "moe_ffn: empty or inconsistent shape");
    if (p->has_ep_band)
        return fail(be, INFR_HIP_ERR_UNSUPPORTED, "moe_ffn: ep_band (an expert-parallel shard) needs more than one GPU");
    if (p->act < INFR_ACT_SILU || p->act > INFR_ACT_SIGMOID || p->gating < INFR_GATING_SOFTMAX ||
        p->gating > INFR_GATING_SQRT_SOFTPLUS)
        return fail(be, INFR_HIP_ERR_UNSUPPORTED, "moe_ffn: unknown activation or gating");
    // the two combinations the CPU arm asserts against (lib.rs:2293-2309)
    if (p->has_clamp && (p->act == INFR_ACT_SIGMOID || p->weight_before))
        return fail(be, INFR_HIP_ERR_UNSUPPORTED, "moe_ffn: swiglu_clamp is defined for SiLU / GELU with output-side weighting only");
    if (p->has_expert_ids && (p->has_exp_probs_b || p->n_expert_groups > 1))
        return fail(be, INFR_HIP_ERR_UNSUPPORTED, "moe_ffn: expert_ids supplies the selection; exp_probs_b and expert groups must be absent");
    const bool grouped = p->n_expert_groups > 1 && p->n_expert_groups_used > 0;
    if (grouped && (p->n_expert_groups > 64 || p->n_expert % p->n_expert_groups != 0 ||
                    p->n_expert_groups_used > p->n_expert_groups ||
                    (uint64_t)p->n_expert / p->n_expert_groups * p->n_expert_groups_used < p->n_used))
        return fail(be, INFR_HIP_ERR_UNSUPPORTED, "moe_ffn: expert groups must divide n_expert (at most 64 groups) and keep at least n_used experts");
    const infr_hip_buffer_t* down_scale = opt ? opt->down_scale : nullptr;
    const infr_hip_buffer_t* exp_probs_b = opt ? opt->exp_probs_b : nullptr;
    const infr_hip_buffer_t* expert_ids = opt ? opt->expert_ids : nullptr;
    if ((p->has_down_scale != 0) != (down_scale != nullptr) || (p->has_exp_probs_b != 0) != (exp_probs_b != nullptr) ||
        (p->has_expert_ids != 0) != (expert_ids != nullptr))
        return fail(be, INFR_HIP_ERR_INVALID, "moe_ffn: an optional operand does not match its has_* flag");
    const int up_dtype = fused ? p->gate_dtype : p->up_dtype;
    const size_t gb = expert_bank_bytes(p->gate_dtype, (size_t)p->n_expert * p->n_ff_exp * (fused ? 2 : 1), p->ne);
    const size_t ub = fused ? gb : expert_bank_bytes(up_dtype, (size_t)p->n_expert * p->n_ff_exp, p->ne);
    const size_t db = expert_bank_bytes(p->down_dtype, (size_t)p->n_expert * p->ne, p->n_ff_exp);
    if (!gb || !ub || !db || !is_moe_quant(p->gate_dtype) || !is_moe_quant(up_dtype) ||
        !is_moe_quant(p->down_dtype) || !is_plain(p->router_dtype))
        return fail(be, INFR_HIP_ERR_UNSUPPORTED, "moe_ffn: expert bank dtype/shape has no kernel");
    const size_t act_bytes = (size_t)p->rows * p->ne * sizeof(float);
    if (gate->len < gb || (!fused && up->len < ub) || down->len < db ||
        router->len < (size_t)p->n_expert * p->ne * (p->router_dtype == INFR_DTYPE_F32 ? 4 : 2) || x->len < act_bytes ||
        router_x->len < act_bytes || dst->len < act_bytes)
        return fail(be, INFR_HIP_ERR_INVALID, "moe_ffn: a buffer is smaller than its declared shape");
    const size_t sel_bytes = (size_t)p->rows * p->n_used * 4;
    if ((sel_idx && sel_idx->len < sel_bytes) || (sel_w && sel_w->len < sel_bytes))
        return fail(be, INFR_HIP_ERR_INVALID, "moe_ffn: selection output buffer too small");
    if ((down_scale && down_scale->len < (size_t)p->n_expert * 4) || (exp_probs_b && exp_probs_b->len < (size_t)p->n_expert * 4) ||
        (expert_ids && expert_ids->len < sel_bytes))
        return fail(be, INFR_HIP_ERR_INVALID, "moe_ffn: an optional operand is smaller than its declared shape");
    *s = infr::MoeShape{(int)p->ne, (int)p->n_expert, (int)p->n_used, (int)p->n_ff_exp, (int)p->rows,
                        p->scale, p->router_dtype, p->gate_dtype, up_dtype, p->down_dtype};
    s->route.gating = p->gating;
    s->route.norm_w = p->norm_w != 0;
    s->route.n_groups = grouped ? (int)p->n_expert_groups : 0;
    s->route.n_groups_used = grouped ? (int)p->n_expert_groups_used : 0;
    s->route.bias = exp_probs_b ? static_cast<const float*>(exp_probs_b->ptr) : nullptr;
    s->route.ids = expert_ids ? static_cast<const int32_t*>(expert_ids->ptr) : nullptr;
    s->act.act = p->act;
    s->act.has_clamp = p->has_clamp != 0;
    s->act.clamp = p->clamp;
    s->act.weight_before = p->weight_before != 0;
    s->fused_gate_up = fused;
    b->x = static_cast<const float*>(x->ptr);
    b->router_x = static_cast<const float*>(router_x->ptr);
    b->router = static_cast<const float*>(router->ptr);
    b->gate = static_cast<const uint8_t*>(gate->ptr);
    b->up = fused ? b->gate : static_cast<const uint8_t*>(up->ptr);
    b->down = static_cast<const uint8_t*>(down->ptr);
    // expert e = the e-th equal byte slice of the bound bank (lib.rs:2345-2347)
    b->gate_stride = gate->len / p->n_expert;
    b->up_stride = fused ? b->gate_stride : up->len / p->n_expert;
    b->down_stride = down->len / p->n_expert;
    b->dst = static_cast<float*>(dst->ptr);
    b->sel_idx = sel_idx ? static_cast<int32_t*>(sel_idx->ptr) : nullptr;
    b->sel_w = sel_w ? static_cast<float*>(sel_w->ptr) : nullptr;
    b->down_scale = down_scale ? static_cast<const float*>(down_scale->ptr) : nullptr;
    return INFR_HIP_OK;
}

// The optional operands of a plan's MoeFfn op, from the bindings.
static infr_hip_moe_optional_t moe_optional(const infr_hip_op_t& op, infr_hip_buffer_t* const* bindings) {
    infr_hip_moe_optional_t o{nullptr, nullptr, nullptr};
    if (op.moe.has_down_scale) o.down_scale = bindings[op.down_scale];
    if (op.moe.has_exp_probs_b) o.exp_probs_b = bindings[op.exp_probs_b];
    if (op.moe.has_expert_ids) o.expert_ids = bindings[op.expert_ids];
    return o;
}

static int enqueue_moe(infr_hip_t* be, const infr::MoeShape& s, const infr::MoeBuffers& b) {
    const char* msg = infr::launch_moe_ffn(s, b, be->moe_ws, be->stream);
    if (msg) return fail(be, INFR_HIP_ERR_UNSUPPORTED, std::string("moe_ffn: ") + msg);
    HIP_TRY(be, hipGetLastError());
    return INFR_HIP_OK;
}

int infr_hip_moe_ffn(infr_hip_t* be, const infr_hip_moe_params_t* p, const infr_hip_buffer_t* x,
                     const infr_hip_buffer_t* router_x, const infr_hip_buffer_t* router,
                     const infr_hip_buffer_t* gate_exps, const infr_hip_buffer_t* up_exps,
                     const infr_hip_buffer_t* down_exps, const infr_hip_moe_optional_t* opt, infr_hip_buffer_t* dst,
                     infr_hip_buffer_t* sel_idx, infr_hip_buffer_t* sel_w) {
    if (!be) return INFR_HIP_ERR_INVALID;
    if (int rc = check_latch(be)) return rc;
    infr::MoeShape s;
    infr::MoeBuffers b;
    if (int rc = check_moe(be, p, x, router_x, router, gate_exps, up_exps, down_exps, opt, dst, sel_idx, sel_w, &s, &b))
        return rc;
    if (int rc = ensure_moe_ws(be, infr::moe_workspace_bytes(s))) return rc;
    return enqueue_moe(be, s, b);
}

// ---- plan / execute ----

int infr_hip_compile(infr_hip_t* be, const infr_hip_op_t* ops, size_t n_ops, infr_hip_plan_t** out) {
    if (!be || !out || (!ops && n_ops)) return fail(be, INFR_HIP_ERR_INVALID, "compile: null argument");
    *out = nullptr;
    infr_hip_plan_t* p = new (std::nothrow) infr_hip_plan();
    if (!p) return fail(be, INFR_HIP_ERR_OTHER, "compile: out of host memory");
    p->ops.assign(ops, ops + n_ops);
    // batch_need: one small-batch op's activations; a group of several distinct activation tensors
    // grows the scratch when it is scheduled (the levels depend on the bound addresses)
    size_t act_need = 0, moe_need = 0, batch_need = 0;
    for (const auto& op : p->ops) {
        if (op.kind == INFR_OP_LINEAR) {
            if ((!is_quant(op.w_dtype) && !is_plain(op.w_dtype)) || op.m == 0 || op.in_f == 0 || op.out_f == 0 ||
                op.in_f % in_f_multiple(op.w_dtype) != 0 || op.w_numel % op.in_f != 0 ||
                op.w_off % op.in_f != 0) {
                delete p;
                return fail(be, INFR_HIP_ERR_UNSUPPORTED, "compile: Linear op with unsupported dtype/shape");
            }
            p->max_tensor = std::max({p->max_tensor, op.x, op.weight, op.dst});
            act_need = std::max(act_need, linear_scratch_elems(op.w_dtype, op.m, op.in_f));
            if (small_batch(op)) batch_need = std::max(batch_need, ((size_t)op.m * op.in_f + 255) / 256 * 256);
        } else if (op.kind == INFR_OP_MOE_FFN) {
            const auto& mp = op.moe;
            if (!mp.ne || !mp.n_expert || !mp.n_used || !mp.n_ff_exp || !mp.rows) {
                delete p;
                return fail(be, INFR_HIP_ERR_UNSUPPORTED, "compile: MoeFfn op with empty shape");
            }
            p->max_tensor = std::max({p->max_tensor, op.x, op.dst, op.router_x, op.router,
                                      op.gate_exps, mp.fused_gate_up ? op.gate_exps : op.up_exps, op.down_exps,
                                      mp.has_down_scale ? op.down_scale : 0u, mp.has_exp_probs_b ? op.exp_probs_b : 0u,
                                      mp.has_expert_ids ? op.expert_ids : 0u});
            const infr::MoeShape ms{(int)mp.ne, (int)mp.n_expert, (int)mp.n_used, (int)mp.n_ff_exp,
                                    (int)mp.rows, mp.scale, mp.router_dtype, mp.gate_dtype,
                                    mp.up_dtype, mp.down_dtype};
            moe_need = std::max(moe_need, infr::moe_workspace_bytes(ms));
        } else if (is_elementwise(op.kind)) {
            const bool clamp_ok = !op.has_clamp || op.act != INFR_ACT_SIGMOID;  // lib.rs:1903-1907
            const bool act_ok = op.act >= INFR_ACT_SILU && op.act <= INFR_ACT_SIGMOID;
            if (op.m == 0 || op.in_f == 0 || !clamp_ok || !act_ok ||
                (op.kind == INFR_OP_GATED_ACT && op.gate_block_width % 2 != 0)) {
                delete p;
                return fail(be, INFR_HIP_ERR_UNSUPPORTED, "compile: elementwise op with unsupported shape or mode");
            }
            p->max_tensor = std::max({p->max_tensor, op.x, op.dst});
            if (op.kind == INFR_OP_RMS_NORM || op.kind == INFR_OP_RMS_NORM_ADD)
                p->max_tensor = std::max(p->max_tensor, op.weight);
            if (op.kind == INFR_OP_GATED_ACT || op.kind == INFR_OP_ADD)
                p->max_tensor = std::max(p->max_tensor, op.aux);
        } else if (op.kind == INFR_OP_EMBED_GATHER) {
            int qpb = 0, bpb = 0;
            if (!infr::embed_gather_supported(op.w_dtype) || !infr_block_layout(op.w_dtype, &qpb, &bpb) ||
                op.m == 0 || op.in_f == 0 || op.in_f % (uint32_t)qpb != 0 || op.w_numel == 0 ||
                op.w_numel % op.in_f != 0) {
                delete p;
                return fail(be, INFR_HIP_ERR_UNSUPPORTED, "compile: EmbedGather op with unsupported dtype/shape");
            }
            p->max_tensor = std::max({p->max_tensor, op.x, op.weight, op.dst});
        } else {
            delete p;
            return fail(be, INFR_HIP_ERR_UNSUPPORTED, "compile: op kind " + std::to_string(op.kind));
        }
    }
    // Scratch is sized here so that execute never allocates (it records launches for replay).
    if (int rc = ensure_act(be, std::max(act_need, batch_need))) {
        delete p;
        return rc;
    }
    if (int rc = ensure_moe_ws(be, moe_need)) {
        delete p;
        return rc;
    }
    *out = p;
    return INFR_HIP_OK;
}

size_t infr_hip_plan_launches(const infr_hip_plan_t* plan) {
    if (!plan) return 0;
    if (plan->recorded_nodes) return plan->recorded_nodes;
    // nothing recorded (direct submission): the common forms' counts
    size_t n = 0;
    for (const auto& st : plan->steps) {
        if (st.op < 0) n += st.m > 1 ? 2 : 1;                              // grouped launch (+ grouped quantize)
        else if (plan->ops[st.op].kind == INFR_OP_MOE_FFN) n += plan->ops[st.op].moe.rows == 1 ? 3 : 4;
        else if (is_elementwise(plan->ops[st.op].kind) || plan->ops[st.op].kind == INFR_OP_EMBED_GATHER) n += 1;
        else n += 2;                                                       // quantize + GEMM
    }
    return n;
}

void infr_hip_plan_free(infr_hip_t* be, infr_hip_plan_t* plan) {
    if (!plan) return;
    if (be && be->stream) (void)hipStreamSynchronize(be->stream);
    if (plan->exec) (void)hipGraphExecDestroy(plan->exec);
    if (plan->tiles_dev) (void)hipFree(plan->tiles_dev);
    if (plan->ssegs_dev) (void)hipFree(plan->ssegs_dev);
    if (plan->qtiles_dev) (void)hipFree(plan->qtiles_dev);
    if (plan->btiles_dev) (void)hipFree(plan->btiles_dev);
    delete plan;
}

// Orders the plan's ops for the currently bound device addresses. Two ops conflict when one
// writes memory the other reads or writes (the read/write sets of Op::io, graph.rs:1128); an op's
// level is one more than the highest level among earlier conflicting ops, so ops of one level are
// mutually independent and running levels in ascending order preserves every dependency.
static int schedule_plan(infr_hip_t* be, infr_hip_plan_t* plan, infr_hip_buffer_t* const* bindings) {
    const size_t n = plan->ops.size();
    struct Span { const uint8_t* lo; const uint8_t* hi; };
    auto span = [](const infr_hip_buffer_t* b, size_t bytes) {
        const uint8_t* p = static_cast<const uint8_t*>(b->ptr);
        return Span{p, p + bytes};
    };
    auto fspan = [](const float* p, size_t elems) {
        return Span{reinterpret_cast<const uint8_t*>(p), reinterpret_cast<const uint8_t*>(p + elems)};
    };
    auto overlap = [](const Span& a, const Span& b) { return a.lo < b.hi && b.lo < a.hi; };
    auto any_overlap = [&](const std::vector<Span>& a, const std::vector<Span>& b) {
        for (const auto& x : a)
            for (const auto& y : b)
                if (overlap(x, y)) return true;
        return false;
    };
    // reads / writes: device ranges an op reads (activations and weights) and writes
    std::vector<std::vector<Span>> rd(n), wr(n);
    std::vector<int> level(n, 0);
    std::vector<LinearArgs> la(n);
    std::vector<ElementwiseArgs> ea(n);
    for (size_t i = 0; i < n; ++i) {
        const auto& op = plan->ops[i];
        if (op.kind == INFR_OP_MOE_FFN) {
            infr::MoeShape ms;
            infr::MoeBuffers mb;
            const infr_hip_moe_optional_t mo = moe_optional(op, bindings);
            if (int rc = check_moe(be, &op.moe, bindings[op.x], bindings[op.router_x], bindings[op.router],
                                   bindings[op.gate_exps], op.moe.fused_gate_up ? nullptr : bindings[op.up_exps],
                                   bindings[op.down_exps], &mo, bindings[op.dst], nullptr, nullptr, &ms, &mb))
                return rc;
            const size_t abytes = (size_t)ms.rows * ms.ne * sizeof(float);
            rd[i] = {span(bindings[op.x], abytes), span(bindings[op.router_x], abytes)};
            if (mo.expert_ids) rd[i].push_back(span(mo.expert_ids, (size_t)ms.rows * ms.n_used * 4));
            if (mo.down_scale) rd[i].push_back(span(mo.down_scale, (size_t)ms.n_expert * 4));
            if (mo.exp_probs_b) rd[i].push_back(span(mo.exp_probs_b, (size_t)ms.n_expert * 4));
            wr[i] = {span(bindings[op.dst], abytes)};
        } else if (op.kind == INFR_OP_EMBED_GATHER) {
            EmbedArgs eg;
            if (int rc = check_embed(be, op.w_dtype, bindings[op.weight], op.w_numel, bindings[op.x], op.m, op.in_f,
                                     bindings[op.dst], &eg))
                return rc;
            rd[i] = {span(bindings[op.x], (size_t)op.m * sizeof(int32_t)),
                     Span{eg.table, eg.table + eg.total_rows * eg.bpr}};
            wr[i] = {span(bindings[op.dst], (size_t)op.m * op.in_f * sizeof(float))};
        } else if (is_elementwise(op.kind)) {
            if (int rc = check_elementwise(be, op, bindings, &ea[i])) return rc;
            rd[i] = {fspan(ea[i].x, ea[i].x_elems)};
            if (ea[i].aux) rd[i].push_back(fspan(ea[i].aux, ea[i].aux_elems));
            wr[i] = {fspan(ea[i].dst, ea[i].dst_elems)};
        } else {
            if (int rc = check_linear(be, op.w_dtype, bindings[op.weight], op.w_numel, op.w_off,
                                      bindings[op.x], op.m, op.in_f, op.out_f, &la[i]))
                return rc;
            const size_t ybytes = (size_t)op.m * op.out_f * sizeof(float);
            if (!bindings[op.dst] || bindings[op.dst]->len < ybytes)
                return fail(be, INFR_HIP_ERR_INVALID, "execute: dst buffer missing or too small");
            rd[i] = {span(bindings[op.x], (size_t)op.m * op.in_f * sizeof(float)),
                     Span{la[i].wrows, la[i].wrows + (size_t)op.out_f * la[i].bpr}};
            wr[i] = {span(bindings[op.dst], ybytes)};
        }
    }

    // ---- absorb the ops around m == 1 Linears into the decode GEMV (see infr::GemvFusion) ----
    // pre[i]  >= 0: Linear i computes its x from op pre[i]'s inputs (GatedAct / GatedActFused / RmsNorm)
    // post[i] >= 0: Linear i also writes Op::Add post[i]
    // absorbed[k]: op k runs inside some Linear and is not scheduled on its own
    std::vector<int> pre(n, -1), post(n, -1);
    std::vector<char> absorbed(n, 0), publishes(n, 0);
    plan->moe_norm.assign(n, -1);
    // INFR_HIP_FUSE=0: every op a launch of its own (for comparing against the absorbed form)
    static const int env_fuse = getenv("INFR_HIP_FUSE") ? atoi(getenv("INFR_HIP_FUSE")) : 1;
    // (a one-row Linear in place on its x runs alone, through the quantize-then-multiply path)
    // (taken from the ops as written: absorbing an Add later puts the residual among the Linear's spans)
    std::vector<char> in_place(n, 0);
    for (size_t i = 0; i < n; ++i)
        in_place[i] = plan->ops[i].kind == INFR_OP_LINEAR && any_overlap(rd[i], wr[i]);
    auto self_alias = [&](size_t i) { return in_place[i] != 0; };
    auto decode_linear = [&](size_t i) {
        return plan->ops[i].kind == INFR_OP_LINEAR && plan->ops[i].m == 1 &&
               !runs_alone(plan->ops[i].w_dtype, 1, plan->ops[i].in_f) && !self_alias(i);
    };
    // pair_act[i] >= 0: Linear i is the gate projection of gated activation pair_act[i], evaluated by
    // the workgroups that produce its operands; pair_up[i] is the up projection (i itself when one
    // Linear writes [gate | up]) and pair_follower marks an up projection that rides in i's tiles.
    std::vector<int> pair_act(n, -1), pair_up(n, -1);
    std::vector<char> pair_follower(n, 0);
    struct PairUndo {
        size_t k, gate, up;
        std::vector<Span> gate_wr;
    };
    std::vector<PairUndo> pairs;
    // INFR_HIP_PAIR=0: gated activations go into their consumer's prologue only
    static const int env_pair = getenv("INFR_HIP_PAIR") ? atoi(getenv("INFR_HIP_PAIR")) : 1;
    auto try_pair = [&](size_t k) {
        const auto& p = plan->ops[k];
        const size_t nff = p.in_f;
        const bool one = p.kind == INFR_OP_GATED_ACT_FUSED;
        const float* G = ea[k].x;
        const float* U = one ? ea[k].x + nff : ea[k].aux + p.up_off;
        const std::vector<Span> gs{fspan(G, nff)}, us{fspan(U, nff)};
        int ig = -1, iu = -1;  // the last writers of the two operands
        for (size_t j = 0; j < k; ++j) {
            if (any_overlap(wr[j], gs)) ig = (int)j;
            if (any_overlap(wr[j], us)) iu = (int)j;
        }
        if (ig < 0 || iu < 0 || (ig == iu) != one) return false;
        const auto &og = plan->ops[ig], &ou = plan->ops[iu];
        if (!decode_linear(ig) || !decode_linear(iu) || absorbed[ig] || absorbed[iu]) return false;
        if (pair_act[ig] >= 0 || pair_act[iu] >= 0 || pair_follower[ig] || pair_follower[iu]) return false;
        if (static_cast<const float*>(bindings[og.dst]->ptr) != G || og.out_f != (one ? 2 * nff : nff)) return false;
        if (!one && (static_cast<const float*>(bindings[ou.dst]->ptr) != U || ou.out_f != nff ||
                     ou.w_dtype != og.w_dtype || ou.in_f != og.in_f || la[iu].bpr != la[ig].bpr ||
                     bindings[ou.x]->ptr != bindings[og.x]->ptr || pre[iu] != pre[ig]))
            return false;
        if (pre[ig] >= 0 && plan->ops[pre[ig]].kind != INFR_OP_RMS_NORM) return false;
        // dst is stored where the operands are produced: nothing from there up to the activation
        // may touch it, and the producers' own inputs must not lie in it
        for (size_t j = (size_t)std::min(ig, iu); j < k; ++j)
            if (any_overlap(wr[j], wr[k]) || any_overlap(rd[j], wr[k])) return false;
        pairs.push_back(PairUndo{k, (size_t)ig, (size_t)iu, wr[ig]});
        pair_act[ig] = (int)k;
        pair_up[ig] = iu;
        if (!one) pair_follower[iu] = 1;
        absorbed[k] = 1;
        wr[ig].push_back(wr[k][0]);
        return true;
    };
    for (size_t k = 0; env_fuse && k < n; ++k) {
        const auto& p = plan->ops[k];
        const bool gated = (p.kind == INFR_OP_GATED_ACT && p.gate_block_width == 0) || p.kind == INFR_OP_GATED_ACT_FUSED;
        if (!(gated || p.kind == INFR_OP_RMS_NORM) || p.m != 1 || p.in_f % 4 != 0) continue;
        // A producer that runs in place (dst overlapping one of its inputs) cannot be absorbed:
        // every workgroup of the consumer re-reads the producer's inputs while the first one
        // stores dst, so later workgroups would apply the op to its own result.
        if (any_overlap(wr[k], rd[k])) continue;
        if (gated && env_pair && try_pair(k)) continue;
        // The definition's live range ends at the next op that overwrites dst (scratch tensors
        // are reused from layer to layer, graph.rs:10-14): readers beyond it see that op's value.
        // An op that overwrites only part of dst keeps the whole plan as the range.
        size_t end = n - 1;
        for (size_t j = k + 1; j < n; ++j) {
            if (!any_overlap(wr[j], wr[k])) continue;
            bool covers = false;
            for (const auto& w : wr[j]) covers = covers || (w.lo <= wr[k][0].lo && w.hi >= wr[k][0].hi);
            if (covers) end = j;
            break;
        }
        // every reader of this definition must be a decode Linear taking exactly that vector as
        // x, with the producer's inputs and dst untouched up to the last of them
        std::vector<size_t> users;
        bool ok = true;
        int moe_user = -1;  // a single-row MoeFfn reading dst as both x and router_x (fusion.rs:58-73)
        for (size_t i = k + 1; ok && i <= end; ++i) {
            if (!any_overlap(rd[i], wr[k])) continue;
            const auto& u = plan->ops[i];
            if (p.kind == INFR_OP_RMS_NORM && u.kind == INFR_OP_MOE_FFN && u.moe.rows == 1 && u.moe.ne == p.in_f &&
                static_cast<const float*>(bindings[u.x]->ptr) == ea[k].dst &&
                static_cast<const float*>(bindings[u.router_x]->ptr) == ea[k].dst && moe_user < 0 && users.empty()) {
                moe_user = (int)i;
                continue;
            }
            ok = moe_user < 0 && decode_linear(i) && u.in_f == p.in_f &&
                 static_cast<const float*>(bindings[u.x]->ptr) == ea[k].dst;
            if (ok) users.push_back(i);
        }
        if (ok && moe_user >= 0) {
            // the MoeFfn is the definition's only reader: its router kernel normalises the row and
            // stores dst; nothing up to it may touch the norm's inputs or dst
            for (size_t j = k + 1; ok && j < (size_t)moe_user; ++j)
                ok = !any_overlap(wr[j], rd[k]) && !any_overlap(wr[j], wr[k]);
            // the op's own output must not land on the norm's inputs (its kernels re-read them)
            ok = ok && !any_overlap(wr[moe_user], rd[k]);
            if (!ok) continue;
            absorbed[k] = 1;
            plan->moe_norm[moe_user] = (int)k;
            for (const auto& r : rd[k]) rd[moe_user].push_back(r);
            wr[moe_user].push_back(wr[k][0]);
            continue;
        }
        if (!ok || users.empty()) continue;
        for (size_t j = k + 1; ok && j <= users.back(); ++j)
            ok = !any_overlap(wr[j], rd[k]) && (!any_overlap(wr[j], wr[k]));
        if (!ok) continue;
        for (size_t u : users) ok = ok && pre[u] < 0;
        if (!ok) continue;
        absorbed[k] = 1;
        for (size_t u : users) {
            pre[u] = (int)k;
            // the consumer reads the producer's inputs instead of its dst; the first one stores dst
            rd[u][0] = rd[k][0];
            for (size_t q = 1; q < rd[k].size(); ++q) rd[u].push_back(rd[k][q]);
        }
        publishes[users.front()] = 1;
        wr[users.front()].push_back(wr[k][0]);
    }
    // Op::Add after its producer (fusion.rs:155-260): one operand is the output of an earlier decode
    // Linear or MoeFfn of the same length, the other is the residual; the producer's last kernel
    // then also writes the sum (f32 addition commutes, so either operand order gives the CPU's bits).
    std::vector<const float*> resid(n, nullptr);
    plan->moe_add.assign(n, -1);
    plan->moe_add_resid_is_a.assign(n, 0);
    for (size_t k = 0; env_fuse && k < n; ++k) {
        const auto& a = plan->ops[k];
        if (a.kind != INFR_OP_ADD || ea[k].x == ea[k].aux) continue;
        const size_t n_add = (size_t)a.m * a.in_f;
        // nothing between the producer and the Add may touch the Add's dst or write the residual
        // or the producer's dst (the sum is produced at the producer's place in the order)
        for (size_t i = 0; i < k; ++i) {
            const auto& pr = plan->ops[i];
            // (a small-batch Linear's grouped launch stores the sum with each output as well)
            const bool lin = (decode_linear(i) && pr.out_f == n_add) ||
                             (pr.kind == INFR_OP_LINEAR && pr.m >= 2 && small_batch(pr) && !self_alias(i) &&
                              (size_t)pr.m * pr.out_f == n_add);
            const bool moe = pr.kind == INFR_OP_MOE_FFN && (size_t)pr.moe.rows * pr.moe.ne == n_add;
            if ((!lin && !moe) || post[i] >= 0 || pair_act[i] >= 0 || pair_follower[i]) continue;
            const float* pdst = static_cast<const float*>(bindings[pr.dst]->ptr);
            if (pdst != ea[k].x && pdst != ea[k].aux) continue;
            const bool resid_is_a = pdst == ea[k].aux;
            bool ok = true;
            const std::vector<Span> b_span{fspan(resid_is_a ? ea[k].x : ea[k].aux, n_add)};
            for (size_t j = i + 1; ok && j < k; ++j)
                ok = !any_overlap(wr[j], wr[k]) && !any_overlap(rd[j], wr[k]) && !any_overlap(wr[j], b_span) &&
                     !any_overlap(wr[j], wr[i]);
            // a Linear's own inputs must not alias the Add's destination (its workgroups read them
            // while others already store); a MoeFfn reads its inputs in launches that finish before
            // the one that stores
            ok = ok && (moe || !any_overlap(rd[i], wr[k]));
            if (!ok) continue;
            post[i] = (int)k;
            resid[i] = resid_is_a ? ea[k].x : ea[k].aux;
            if (moe) {
                plan->moe_add[i] = (int)k;
                plan->moe_add_resid_is_a[i] = resid_is_a;
            }
            absorbed[k] = 1;
            rd[i].push_back(b_span[0]);
            wr[i].push_back(wr[k][0]);
            break;
        }
    }

    // Two rows and more: a RmsNorm or a gated activation whose output only feeds small-batch
    // Linears of the same shape is evaluated by those Linears' quantizer launch (a workgroup
    // applies the op to the floats it is about to quantize, with the stand-alone kernel's
    // arithmetic, and stores them): one launch less per op, same bits. The users must end up on
    // one level - the quantizers of a level all run before anything later - which is checked once
    // the levels are known; a fold that fails the check is undone.
    struct QuantFold {
        size_t k;
        std::vector<size_t> users;
        std::vector<std::vector<Span>> users_rd;
        std::vector<Span> front_wr;
    };
    std::vector<QuantFold> folds;
    std::vector<int> qpre(n, -1);
    for (size_t k = 0; env_fuse && k < n; ++k) {
        const auto& p = plan->ops[k];
        const bool gated = (p.kind == INFR_OP_GATED_ACT && p.gate_block_width == 0) || p.kind == INFR_OP_GATED_ACT_FUSED;
        if (!(gated || p.kind == INFR_OP_RMS_NORM) || p.m < 2 || p.in_f % 256 != 0 || absorbed[k]) continue;
        if (p.kind == INFR_OP_GATED_ACT && (p.up_off % 4 != 0 || p.up_stride % 4 != 0 || p.gate_stride % 4 != 0)) continue;
        if (any_overlap(wr[k], rd[k])) continue;
        size_t end = n - 1;
        for (size_t j = k + 1; j < n; ++j) {
            if (!any_overlap(wr[j], wr[k])) continue;
            bool covers = false;
            for (const auto& w : wr[j]) covers = covers || (w.lo <= wr[k][0].lo && w.hi >= wr[k][0].hi);
            if (covers) end = j;
            break;
        }
        std::vector<size_t> users;
        bool ok = true;
        for (size_t i = k + 1; ok && i <= end; ++i) {
            if (!any_overlap(rd[i], wr[k])) continue;
            const auto& u = plan->ops[i];
            ok = u.kind == INFR_OP_LINEAR && small_batch(u) && u.m == p.m && u.in_f == p.in_f && !self_alias(i) &&
                 qpre[i] < 0 && static_cast<const float*>(bindings[u.x]->ptr) == ea[k].dst;
            if (ok) users.push_back(i);
        }
        if (!ok || users.empty()) continue;
        for (size_t j = k + 1; ok && j <= users.back(); ++j)
            ok = !any_overlap(wr[j], rd[k]) && !any_overlap(wr[j], wr[k]);
        if (!ok) continue;
        QuantFold f;
        f.k = k;
        f.users = users;
        for (size_t u : users) f.users_rd.push_back(rd[u]);
        f.front_wr = wr[users.front()];
        absorbed[k] = 1;
        for (size_t u : users) {
            qpre[u] = (int)k;
            rd[u][0] = rd[k][0];
            for (size_t q = 1; q < rd[k].size(); ++q) rd[u].push_back(rd[k][q]);
        }
        wr[users.front()].push_back(wr[k][0]);
        folds.push_back(std::move(f));
    }

    int max_level = 0;
    for (;;) {
        max_level = 0;
        std::fill(level.begin(), level.end(), 0);
        for (size_t i = 0; i < n; ++i) {
            if (absorbed[i]) continue;
            for (size_t j = 0; j < i; ++j) {
                if (absorbed[j]) continue;
                if (any_overlap(wr[j], rd[i]) || any_overlap(wr[j], wr[i]) || any_overlap(rd[j], wr[i]))
                    level[i] = std::max(level[i], level[j] + 1);
            }
            max_level = std::max(max_level, level[i]);
        }
        bool undone = false;
        for (auto& f : folds) {
            if (f.users.empty()) continue;
            bool same = true;
            for (size_t u : f.users) same = same && level[u] == level[f.users.front()];
            if (same) continue;
            absorbed[f.k] = 0;
            for (size_t q = 0; q < f.users.size(); ++q) {
                rd[f.users[q]] = f.users_rd[q];
                qpre[f.users[q]] = -1;
            }
            wr[f.users.front()] = f.front_wr;
            f.users.clear();
            undone = true;
        }
        // a pair's two projections share one launch: they must have come out on one level
        for (auto& pr : pairs) {
            if (pair_act[pr.gate] < 0 || level[pr.gate] == level[pr.up]) continue;
            pair_act[pr.gate] = pair_up[pr.gate] = -1;
            pair_follower[pr.up] = 0;
            absorbed[pr.k] = 0;
            wr[pr.gate] = pr.gate_wr;
            undone = true;
        }
        if (!undone) break;
    }
    auto fusion_of = [&](size_t k) {
        infr::GemvFusion f;
        if (pair_act[k] >= 0) {
            const auto& p = plan->ops[pair_act[k]];
            const ElementwiseArgs& e = ea[pair_act[k]];
            const bool one = (size_t)pair_up[k] == k;
            f.pair_w = one ? la[k].wrows + (size_t)p.in_f * la[k].bpr : la[pair_up[k]].wrows;
            f.pair_y = const_cast<float*>(one ? e.x + p.in_f : e.aux + p.up_off);
            f.pair_dst = e.dst;
            f.act = p.act;
            f.has_clamp = p.has_clamp;
            f.clamp = p.clamp;
        }
        if (pre[k] >= 0) {
            const auto& p = plan->ops[pre[k]];
            const ElementwiseArgs& e = ea[pre[k]];
            if (p.kind == INFR_OP_RMS_NORM) {
                f.pre = 2;
                f.x2 = e.aux;
                f.eps = p.eps;
            } else {
                f.pre = 1;
                f.x2 = p.kind == INFR_OP_GATED_ACT_FUSED ? e.x + p.in_f : e.aux + p.up_off;
                f.act = p.act;
                f.has_clamp = p.has_clamp;
                f.clamp = p.clamp;
            }
            // (a paired up projection that was to publish the vector hands that to its gate's tiles)
            const bool pub = publishes[k] || (pair_act[k] >= 0 && publishes[pair_up[k]]);
            f.pre_dst = pub ? e.dst : nullptr;
        }
        if (post[k] >= 0) {
            f.add_b = resid[k];
            f.add_dst = ea[post[k]].dst;
        }
        return f;
    };
    plan->steps.clear();
    plan->descs.clear();
    plan->tiles.clear();
    plan->ssegs.clear();
    plan->qtiles.clear();
    plan->btiles.clear();
    for (int lv = 0; lv <= max_level; ++lv) {
        std::vector<char> taken(n, 0);
        for (size_t i = 0; i < n; ++i) {
            if (level[i] != lv || taken[i] || absorbed[i]) continue;
            const auto& op = plan->ops[i];
            infr_hip_plan::Step st;
            st.level = lv;
            // Q4_K Linears of a prefill chunk that read one activation tensor (q / k / v, gate / up):
            // one quantization and one strip launch over all their rows, so that a narrow projection
            // (k, v) shares the grid instead of running on a fraction of the machine.
            auto strip_op = [&](size_t k) {
                const auto& o2 = plan->ops[k];
                return o2.kind == INFR_OP_LINEAR && o2.w_dtype == INFR_DTYPE_Q4_K && o2.m == op.m && o2.in_f == op.in_f &&
                       bindings[o2.x]->ptr == bindings[op.x]->ptr && !self_alias(k) && la[k].bpr == la[i].bpr;
            };
            if (op.kind == INFR_OP_LINEAR && op.w_dtype == INFR_DTYPE_Q4_K && op.m >= 128 && !self_alias(i)) {
                size_t total = 0, count = 0;
                for (size_t k = i; k < n; ++k)
                    if (level[k] == lv && !taken[k] && !absorbed[k] && strip_op(k)) total += plan->ops[k].out_f, ++count;
                if (count >= 2 && infr::mmq_q4k_strip_group_takes(op.m, op.in_f, total)) {
                    st.dtype = op.w_dtype;
                    st.in_f = op.in_f;
                    st.m = op.m;
                    st.strips = true;
                    st.x = static_cast<const float*>(bindings[op.x]->ptr);
                    st.first = (int)plan->descs.size();
                    const int tiles = infr::mmq_strip_q4k_tiles(op.m, total, op.in_f, be->props.multiProcessorCount);
                    const int rows = infr::mmq_strip_q4k_rows(tiles);
                    st.gp.rows_per_wg = tiles;
                    st.tile_first = plan->ssegs.size();
                    for (size_t k = i; k < n; ++k) {
                        if (level[k] != lv || taken[k] || absorbed[k] || !strip_op(k)) continue;
                        taken[k] = 1;
                        const auto& o2 = plan->ops[k];
                        float* yk = static_cast<float*>(bindings[o2.dst]->ptr);
                        plan->descs.push_back(infr::GemvOpDesc{la[k].wrows, st.x, yk, la[k].bpr, (int32_t)o2.out_f,
                                                               infr::GemvFusion{}});
                        for (size_t r = 0; r < o2.out_f; r += (size_t)rows)
                            plan->ssegs.push_back(infr::StripSeg{la[k].wrows + r * la[k].bpr, yk + r, (int32_t)o2.out_f,
                                                                 (int32_t)std::min<size_t>((size_t)rows, o2.out_f - r)});
                    }
                    st.n = (int)plan->descs.size() - st.first;
                    st.gp.total_wgs = (int)(plan->ssegs.size() - st.tile_first);
                    plan->steps.push_back(st);
                    continue;
                }
            }
            if (op.kind == INFR_OP_LINEAR && small_batch(op)) {
                // small-batch group: same (dtype, in_f, m) in this level -> one quantize launch over
                // the distinct activation tensors + one GEMM launch over a tile table
                st.dtype = op.w_dtype;
                st.in_f = op.in_f;
                st.m = op.m;
                st.first = (int)plan->descs.size();
                std::vector<const float*> xs;
                std::vector<int> xs_pre;  // per activation tensor: the op folded into its quantizer tiles (-1: none)
                std::vector<uint32_t> elem0;
                const size_t x_elems = ((size_t)op.m * op.in_f + 255) / 256 * 256;
                for (size_t k = i; k < n; ++k) {
                    const auto& o2 = plan->ops[k];
                    // (small_batch depends on out_f too: an op of the same dtype, rows and row length that
                    // is not a small batch runs alone, as it does when it comes first)
                    if (level[k] != lv || taken[k] || absorbed[k] || o2.kind != INFR_OP_LINEAR || o2.m != op.m ||
                        o2.w_dtype != op.w_dtype || o2.in_f != op.in_f || !small_batch(o2))
                        continue;
                    taken[k] = 1;
                    const float* x = static_cast<const float*>(bindings[o2.x]->ptr);
                    size_t xi = 0;
                    while (xi < xs.size() && xs[xi] != x) ++xi;
                    if (xi == xs.size()) {
                        xs.push_back(x);
                        xs_pre.push_back(qpre[k]);
                    }
                    elem0.push_back((uint32_t)(xi * x_elems));
                    infr::GemvOpDesc desc{la[k].wrows, x, static_cast<float*>(bindings[o2.dst]->ptr), la[k].bpr,
                                          (int32_t)o2.out_f};
                    if (post[k] >= 0) {  // an Op::Add on this output rides in the launch
                        desc.fus.add_b = resid[k];
                        desc.fus.add_dst = ea[post[k]].dst;
                    }
                    plan->descs.push_back(desc);
                }
                st.n = (int)plan->descs.size() - st.first;
                // the group's distinct activation tensors side by side in the scratch (a regrow here is
                // before anything of this schedule is recorded; it bumps the scratch epoch for other plans)
                if (int rc = ensure_act(be, xs.size() * x_elems)) return rc;
                if (!infr::plan_batch_group(st.dtype, st.m, st.in_f, &plan->descs[st.first], st.n, &st.bp))
                    return fail(be, INFR_HIP_ERR_UNSUPPORTED,
                                "execute: no small-batch kernel for dtype " + std::to_string(st.dtype) +
                                    " at in_f " + std::to_string(st.in_f));
                st.tile_first = plan->btiles.size();
                plan->btiles.resize(st.tile_first + st.bp.total_wgs);
                infr::fill_batch_tiles(&plan->descs[st.first], elem0.data(), st.n, st.bp, &plan->btiles[st.tile_first]);
                st.qtile_first = plan->qtiles.size();
                const size_t n_elems = (size_t)op.m * op.in_f;
                for (size_t xi = 0; xi < xs.size(); ++xi) {
                    if (xs_pre[xi] < 0) {
                        for (size_t e = 0; e < n_elems; e += 1024)
                            plan->qtiles.push_back(infr::QuantTile{xs[xi] + e, (uint32_t)((xi * x_elems + e) / 256),
                                                                   (uint32_t)std::min<size_t>(1024, n_elems - e)});
                        continue;
                    }
                    // the folded op's rows, tiles inside a row (in_f is whole 256s here)
                    const auto& p = plan->ops[xs_pre[xi]];
                    const ElementwiseArgs& e = ea[xs_pre[xi]];
                    for (size_t r = 0; r < op.m; ++r) {
                        const float *src, *src2;
                        if (p.kind == INFR_OP_RMS_NORM) {
                            src = e.x + r * op.in_f;
                            src2 = e.aux;
                        } else if (p.kind == INFR_OP_GATED_ACT_FUSED) {
                            src = e.x + r * 2 * op.in_f;
                            src2 = src + op.in_f;
                        } else {
                            src = e.x + r * (p.gate_stride > 0 ? (size_t)p.gate_stride : op.in_f);
                            src2 = e.aux + r * (p.up_stride > 0 ? (size_t)p.up_stride : op.in_f) + p.up_off;
                        }
                        for (size_t c = 0; c < op.in_f; c += 1024) {
                            infr::QuantTile t{src + c, (uint32_t)((xi * x_elems + r * op.in_f + c) / 256),
                                              (uint32_t)std::min<size_t>(1024, op.in_f - c)};
                            t.pre = p.kind == INFR_OP_RMS_NORM ? 2 : 1;
                            t.x2 = src2 + c;
                            t.pre_dst = e.dst + r * op.in_f + c;
                            t.row = src;
                            t.dim = (uint32_t)op.in_f;
                            t.eps = p.eps;
                            t.act = p.act;
                            t.has_clamp = p.has_clamp;
                            t.clamp = p.clamp;
                            plan->qtiles.push_back(t);
                        }
                    }
                }
                st.qtile_n = plan->qtiles.size() - st.qtile_first;
                plan->steps.push_back(st);
                continue;
            }
            // One token of a format that multiplies f32 activations: the level's ops of one row
            // length share a launch (no absorbed neighbours: decode_linear() excludes them).
            auto f32act_op = [&](size_t k) {
                const auto& o2 = plan->ops[k];
                return o2.kind == INFR_OP_LINEAR && o2.m == 1 && infr::gemv_takes_f32_activations(o2.w_dtype, 1) &&
                       infr::gemv_f32act_groups(o2.w_dtype, o2.in_f) && !self_alias(k);
            };
            if (f32act_op(i)) {
                st.dtype = op.w_dtype;
                st.in_f = op.in_f;
                st.f32act = true;
                st.first = (int)plan->descs.size();
                size_t total_rows = 0;
                for (size_t k = i; k < n; ++k) {
                    const auto& o2 = plan->ops[k];
                    if (level[k] != lv || taken[k] || absorbed[k] || !f32act_op(k) || o2.w_dtype != op.w_dtype ||
                        o2.in_f != op.in_f || la[k].bpr > 0xFFFFFFFFull)
                        continue;
                    taken[k] = 1;
                    plan->descs.push_back(infr::GemvOpDesc{la[k].wrows, static_cast<const float*>(bindings[o2.x]->ptr),
                                                           static_cast<float*>(bindings[o2.dst]->ptr), la[k].bpr,
                                                           (int32_t)o2.out_f, infr::GemvFusion{}});
                    total_rows += o2.out_f;
                }
                st.n = (int)plan->descs.size() - st.first;
                if (st.n > 0) {
                    st.gp.rows_per_wg = infr::gemv_f32act_group_rows(total_rows, op.in_f);
                    st.tile_first = plan->tiles.size();
                    for (int q = st.first; q < st.first + st.n; ++q) {
                        const auto& d = plan->descs[q];
                        for (int r = 0; r < d.out_f; r += st.gp.rows_per_wg) {
                            infr::GemvTile tl{};
                            tl.w = d.w + (size_t)r * d.bpr;
                            tl.x = d.x;
                            tl.y = d.y + r;
                            tl.bpr = (uint32_t)d.bpr;
                            tl.rows = std::min(st.gp.rows_per_wg, d.out_f - r);
                            plan->tiles.push_back(tl);
                        }
                    }
                    st.gp.total_wgs = (int)(plan->tiles.size() - st.tile_first);
                    plan->steps.push_back(st);
                    continue;
                }
                st = infr_hip_plan::Step{};   // (a row too long for the table: the op runs alone below)
                st.level = lv;
            }
            if (op.kind != INFR_OP_LINEAR || op.m != 1 || runs_alone(op.w_dtype, op.m, op.in_f) || self_alias(i)) {
                st.op = (int)i;
                taken[i] = 1;
                plan->steps.push_back(st);
                continue;
            }
            st.dtype = op.w_dtype;
            st.in_f = op.in_f;
            st.first = (int)plan->descs.size();
            for (size_t k = i; k < n; ++k) {
                const auto& o2 = plan->ops[k];
                if (level[k] != lv || taken[k] || absorbed[k] || o2.kind != INFR_OP_LINEAR || o2.m != 1 ||
                    o2.w_dtype != op.w_dtype || o2.in_f != op.in_f || self_alias(k) ||
                    (op.w_dtype == INFR_DTYPE_Q8_0 && (o2.in_f % 256 == 0) != (op.in_f % 256 == 0)))
                    continue;
                taken[k] = 1;
                if (pair_follower[k]) continue;  // its rows ride in the gate projection's tiles
                // with an absorbed producer the GEMV starts from the producer's first input
                const float* xsrc = pre[k] >= 0 ? ea[pre[k]].x : static_cast<const float*>(bindings[o2.x]->ptr);
                // (one Linear onto [gate | up]: the op's rows are the gate half, the pair the other)
                const size_t rows = pair_act[k] >= 0 && (size_t)pair_up[k] == k ? o2.out_f / 2 : o2.out_f;
                plan->descs.push_back(infr::GemvOpDesc{la[k].wrows, xsrc, static_cast<float*>(bindings[o2.dst]->ptr),
                                                       la[k].bpr, (int32_t)rows, fusion_of(k)});
            }
            st.n = (int)plan->descs.size() - st.first;
            if (!infr::plan_gemv_group(st.dtype, st.in_f, &plan->descs[st.first], st.n, &st.gp))
                return fail(be, INFR_HIP_ERR_UNSUPPORTED,
                            "execute: no decode kernel for dtype " + std::to_string(st.dtype) +
                                " at in_f " + std::to_string(st.in_f));
            st.tile_first = plan->tiles.size();
            plan->tiles.resize(st.tile_first + (size_t)st.gp.total_wgs);
            infr::fill_gemv_tiles(&plan->descs[st.first], st.n, st.gp, &plan->tiles[st.tile_first]);
            plan->steps.push_back(st);
        }
    }
    if (int rc = upload_table(be, plan->tiles, &plan->tiles_dev, &plan->tiles_cap)) return rc;
    if (int rc = upload_table(be, plan->ssegs, &plan->ssegs_dev, &plan->ssegs_cap)) return rc;
    if (int rc = upload_table(be, plan->qtiles, &plan->qtiles_dev, &plan->qtiles_cap)) return rc;
    if (int rc = upload_table(be, plan->btiles, &plan->btiles_dev, &plan->btiles_cap)) return rc;
    HIP_TRY(be, hipStreamSynchronize(be->stream));
    return INFR_HIP_OK;
}

// Enqueues the scheduled launches (this is what gets recorded for replay: kernels only).
static int enqueue_plan(infr_hip_t* be, infr_hip_plan_t* plan, infr_hip_buffer_t* const* bindings) {
    // Linears of one level that multiply the same activation tensor (q / k / v, gate / up of a prefill
    // chunk) quantize it once: the scratch keeps it until the level ends or another step writes the
    // scratch. (Ops of one level neither write what another reads nor each other's outputs.)
    infr::QuantCache qc;
    int qc_level = -1;
    for (const auto& st : plan->steps) {
        const bool lone_linear = st.op >= 0 && plan->ops[st.op].kind == INFR_OP_LINEAR;
        if (!lone_linear || st.level != qc_level) qc = infr::QuantCache{};
        qc_level = st.level;
        if (st.op >= 0 && plan->ops[st.op].kind == INFR_OP_MOE_FFN) {
            const auto& op = plan->ops[st.op];
            infr::MoeShape ms;
            infr::MoeBuffers mb;
            const infr_hip_moe_optional_t mo = moe_optional(op, bindings);
            if (int rc = check_moe(be, &op.moe, bindings[op.x], bindings[op.router_x], bindings[op.router],
                                   bindings[op.gate_exps], op.moe.fused_gate_up ? nullptr : bindings[op.up_exps],
                                   bindings[op.down_exps], &mo, bindings[op.dst], nullptr, nullptr, &ms, &mb))
                return rc;
            if (plan->moe_norm[st.op] >= 0) {
                const auto& nop = plan->ops[plan->moe_norm[st.op]];
                ElementwiseArgs norm;
                if (int rc = check_elementwise(be, nop, bindings, &norm)) return rc;
                mb.router_x = norm.x;
                mb.norm_w = norm.aux;
                mb.norm_dst = norm.dst;
                mb.norm_eps = nop.eps;
            }
            if (plan->moe_add[st.op] >= 0) {
                ElementwiseArgs add;
                if (int rc = check_elementwise(be, plan->ops[plan->moe_add[st.op]], bindings, &add)) return rc;
                mb.add_b = plan->moe_add_resid_is_a[st.op] ? add.x : add.aux;
                mb.add_dst = add.dst;
            }
            if (int rc = enqueue_moe(be, ms, mb)) return rc;
        } else if (st.op >= 0 && plan->ops[st.op].kind == INFR_OP_EMBED_GATHER) {
            const auto& op = plan->ops[st.op];
            EmbedArgs eg;
            if (int rc = check_embed(be, op.w_dtype, bindings[op.weight], op.w_numel, bindings[op.x], op.m, op.in_f,
                                     bindings[op.dst], &eg))
                return rc;
            infr::launch_embed_gather(op.w_dtype, eg.table, eg.bpr, eg.total_rows,
                                      static_cast<const int32_t*>(bindings[op.x]->ptr), op.m, op.in_f, op.scale,
                                      static_cast<float*>(bindings[op.dst]->ptr), be->stream);
            HIP_TRY(be, hipGetLastError());
        } else if (st.op >= 0 && is_elementwise(plan->ops[st.op].kind)) {
            ElementwiseArgs ea;
            if (int rc = check_elementwise(be, plan->ops[st.op], bindings, &ea)) return rc;
            if (int rc = enqueue_elementwise(be, plan->ops[st.op], ea)) return rc;
        } else if (st.op >= 0) {
            const auto& op = plan->ops[st.op];
            LinearArgs la;
            if (int rc = check_linear(be, op.w_dtype, bindings[op.weight], op.w_numel, op.w_off,
                                      bindings[op.x], op.m, op.in_f, op.out_f, &la))
                return rc;
            if (int rc = enqueue_linear(be, op.w_dtype, la, static_cast<const float*>(bindings[op.x]->ptr),
                                        static_cast<float*>(bindings[op.dst]->ptr), op.m, op.in_f,
                                        op.out_f, infr::IntStages{}, be->act, &qc))
                return rc;
        } else if (st.strips) {
            infr::launch_quantize_q8_tiled(st.x, st.m, st.in_f, be->act, be->stream);
            infr::launch_mmq_strip_q4k_group(plan->descs[st.first].bpr, be->act, st.m, st.in_f, st.gp.rows_per_wg,
                                             plan->ssegs_dev + st.tile_first, st.gp.total_wgs, be->stream);
            HIP_TRY(be, hipGetLastError());
        } else if (st.m > 1) {
            infr::launch_quantize_q8_group(plan->qtiles_dev + st.qtile_first, st.qtile_n, act_per32(st.dtype, st.in_f),
                                           be->act, be->stream);
            if (st.bp.kind == 1)
                infr::launch_mmq_skinny_group(st.dtype, st.m, st.in_f, plan->btiles_dev + st.tile_first, st.bp, be->act,
                                              be->stream);
            else if (!infr::launch_gemv_batch_group(st.dtype, st.m, st.in_f, plan->btiles_dev + st.tile_first,
                                                    st.bp, be->act, be->stream))
                return fail(be, INFR_HIP_ERR_UNSUPPORTED, "execute: small-batch launch rejected");
            HIP_TRY(be, hipGetLastError());
        } else if (st.f32act) {
            if (!infr::launch_gemv_f32act_group(st.dtype, st.in_f, plan->tiles_dev + st.tile_first, st.gp.total_wgs,
                                                be->stream))
                return fail(be, INFR_HIP_ERR_UNSUPPORTED, "execute: f32-activation decode launch rejected");
            HIP_TRY(be, hipGetLastError());
        } else {
            if (!infr::launch_gemv_fused(st.dtype, st.in_f, &plan->descs[st.first], st.n,
                                         plan->tiles_dev + st.tile_first, st.gp, be->stream))
                return fail(be, INFR_HIP_ERR_UNSUPPORTED, "execute: decode launch rejected");
            HIP_TRY(be, hipGetLastError());
        }
    }
    return INFR_HIP_OK;
}

int infr_hip_execute(infr_hip_t* be, infr_hip_plan_t* plan, infr_hip_buffer_t* const* bindings,
                     size_t n_bindings) {
    if (!be || !plan || (!bindings && n_bindings)) return fail(be, INFR_HIP_ERR_INVALID, "execute: null argument");
    if (int rc = check_latch(be)) return rc;
    if (plan->ops.empty()) return INFR_HIP_OK;
    if (plan->max_tensor >= n_bindings)
        return fail(be, INFR_HIP_ERR_INVALID, "execute: a tensor id has no binding slot");
    // Replay when every bound device address is what the recording saw.
    std::vector<void*> now(n_bindings);
    for (size_t i = 0; i < n_bindings; ++i) now[i] = bindings[i] ? bindings[i]->ptr : nullptr;
    if (plan->exec && now == plan->bound && plan->scratch_epoch == be->scratch_epoch) {
        HIP_TRY(be, hipGraphLaunch(plan->exec, be->stream));
        return INFR_HIP_OK;
    }
    if (plan->exec) {
        HIP_TRY(be, hipStreamSynchronize(be->stream));
        (void)hipGraphExecDestroy(plan->exec);
        plan->exec = nullptr;
    }
    // Validate and schedule before recording so a bad binding cannot leave a capture open.
    for (const auto& op : plan->ops) {
        const bool moe = op.kind == INFR_OP_MOE_FFN;
        // elementwise ops name their second operand per kind; check_elementwise validates it
        if (!bindings[op.x] || !bindings[op.dst] || ((op.kind == INFR_OP_LINEAR || op.kind == INFR_OP_EMBED_GATHER) && !bindings[op.weight]) ||
            (moe && (!bindings[op.router_x] || !bindings[op.router] || !bindings[op.gate_exps] ||
                     (!op.moe.fused_gate_up && !bindings[op.up_exps]) || !bindings[op.down_exps])))
            return fail(be, INFR_HIP_ERR_INVALID, "execute: unbound tensor");
    }
    if (int rc = schedule_plan(be, plan, bindings)) return rc;
    // INFR_HIP_GRAPH=0: enqueue the launches directly on every execute instead of replaying a
    // recorded graph (for comparing the two submission paths).
    static const int env_graph = getenv("INFR_HIP_GRAPH") ? atoi(getenv("INFR_HIP_GRAPH")) : 1;
    if (!env_graph) return enqueue_plan(be, plan, bindings);
    hipGraph_t graph = nullptr;
    HIP_TRY(be, hipStreamBeginCapture(be->stream, hipStreamCaptureModeThreadLocal));
    int rc = enqueue_plan(be, plan, bindings);
    hipError_t e = hipStreamEndCapture(be->stream, &graph);
    if (rc != INFR_HIP_OK) {
        if (graph) (void)hipGraphDestroy(graph);
        return rc;
    }
    if (e != hipSuccess) return fail(be, INFR_HIP_ERR_BACKEND, std::string("hipStreamEndCapture: ") + hipGetErrorString(e));
    size_t n_nodes = 0;
    plan->recorded_nodes = hipGraphGetNodes(graph, nullptr, &n_nodes) == hipSuccess ? n_nodes : 0;
    e = hipGraphInstantiate(&plan->exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) {
        plan->exec = nullptr;
        return fail(be, INFR_HIP_ERR_BACKEND, std::string("hipGraphInstantiate: ") + hipGetErrorString(e));
    }
    plan->bound = now;
    plan->scratch_epoch = be->scratch_epoch;
    HIP_TRY(be, hipGraphLaunch(plan->exec, be->stream));
    return INFR_HIP_OK;
}

// ---- shutdown latch ----
int infr_hip_request_shutdown(int signo) {
    int expected = 0;
    return g_shutdown_signo.compare_exchange_strong(expected, signo, std::memory_order_relaxed) ? 1 : 0;
}
int infr_hip_shutdown_requested(void) { return g_shutdown_signo.load(std::memory_order_relaxed) != 0; }
int infr_hip_shutdown_signal(void) { return g_shutdown_signo.load(std::memory_order_relaxed); }
void infr_hip_reset_shutdown(void) { g_shutdown_signo.store(0, std::memory_order_relaxed); }

// ---- timing ----
int infr_hip_timer_begin(infr_hip_t* be) {
    if (!be) return INFR_HIP_ERR_INVALID;
    HIP_TRY(be, hipEventRecord(be->ev0, be->stream));
    return INFR_HIP_OK;
}
int infr_hip_timer_end(infr_hip_t* be, float* elapsed_ms) {
    if (!be || !elapsed_ms) return INFR_HIP_ERR_INVALID;
    HIP_TRY(be, hipEventRecord(be->ev1, be->stream));
    HIP_TRY(be, hipEventSynchronize(be->ev1));
    HIP_TRY(be, hipEventElapsedTime(elapsed_ms, be->ev0, be->ev1));
    return INFR_HIP_OK;
}

int infr_hip_stream_read(infr_hip_t* be, const infr_hip_buffer_t* src, size_t bytes, int reps, int nontemporal,
                         float* elapsed_ms) {
    if (!be || !src || !elapsed_ms || reps <= 0) return fail(be, INFR_HIP_ERR_INVALID, "stream_read: bad argument");
    if (bytes > src->len || bytes < 16) return fail(be, INFR_HIP_ERR_INVALID, "stream_read: size outside the buffer");
    if (int rc = check_latch(be)) return rc;
    const int wgs = std::max(1, be->props.multiProcessorCount) * 64;
    int* out = nullptr;
    HIP_TRY(be, hipMalloc((void**)&out, sizeof(int) * (size_t)wgs));
    infr::launch_stream_read(src->ptr, bytes, out, wgs, nontemporal != 0, be->stream);  // untimed first pass
    hipError_t e = hipEventRecord(be->ev0, be->stream);
    for (int r = 0; r < reps && e == hipSuccess; ++r)
        infr::launch_stream_read(src->ptr, bytes, out, wgs, nontemporal != 0, be->stream);
    if (e == hipSuccess) e = hipEventRecord(be->ev1, be->stream);
    if (e == hipSuccess) e = hipEventSynchronize(be->ev1);
    if (e == hipSuccess) e = hipEventElapsedTime(elapsed_ms, be->ev0, be->ev1);
    if (e == hipSuccess) e = hipGetLastError();
    (void)hipFree(out);
    if (e != hipSuccess) return fail(be, INFR_HIP_ERR_BACKEND, std::string("stream_read: ") + hipGetErrorString(e));
    return INFR_HIP_OK;
}

int infr_hip_mfma_i8_peak(infr_hip_t* be, int waves_per_simd, int iters, int random_data, float* elapsed_ms, double* ops) {
    if (!be || !elapsed_ms || !ops || waves_per_simd <= 0 || waves_per_simd > 8 || iters <= 0 || iters > (1 << 20))
        return fail(be, INFR_HIP_ERR_INVALID, "mfma_i8_peak: bad argument");
    if (int rc = check_latch(be)) return rc;
    const int wgs = std::max(1, be->props.multiProcessorCount) * waves_per_simd;  // four waves each: one per SIMD
    int* out = nullptr;
    HIP_TRY(be, hipMalloc((void**)&out, sizeof(int) * (size_t)wgs));
    infr::launch_mfma_i8_peak(out, wgs, iters, random_data, be->stream);  // untimed first pass
    hipError_t e = hipEventRecord(be->ev0, be->stream);
    if (e == hipSuccess) infr::launch_mfma_i8_peak(out, wgs, iters, random_data, be->stream);
    if (e == hipSuccess) e = hipEventRecord(be->ev1, be->stream);
    if (e == hipSuccess) e = hipEventSynchronize(be->ev1);
    if (e == hipSuccess) e = hipEventElapsedTime(elapsed_ms, be->ev0, be->ev1);
    if (e == hipSuccess) e = hipGetLastError();
    (void)hipFree(out);
    if (e != hipSuccess) return fail(be, INFR_HIP_ERR_BACKEND, std::string("mfma_i8_peak: ") + hipGetErrorString(e));
    *ops = 2.0 * 32 * 32 * 32 * 4.0 * (double)iters * 4.0 * (double)wgs;
    return INFR_HIP_OK;
}

}  // extern "C"
