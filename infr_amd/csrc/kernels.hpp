// Host-side launch interface of the device kernels. Launchers validate nothing: the C-ABI layer
// (backend.hip) checks shapes, alignment and buffer sizes before calling in here.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace infr {

// Device-resident quantized activation of m rows of k elements, laid out row-major per field.
// per-256 `Q8`   (crates/infr-cpu/src/quant.rs:8-25):  d[m][k/256], bsums[m][k/32], bsums16[m][k/16]
// per-32 `Q8x32` (quant.rs:90-95): d[m][k/32], bsums[m][k/32]; bsums16 unused.
struct ActQ8 {
    int8_t* qs = nullptr;
    float* d = nullptr;
    int32_t* bsums = nullptr;
    int32_t* bsums16 = nullptr;
};

// quantize_q8 / quantize_q8_32 over m*k contiguous floats.
void launch_quantize_q8(const float* x, size_t m, size_t k, bool per32, const ActQ8& out,
                        hipStream_t stream);
// Several activation tensors in one launch (plans): workgroup i quantizes `n_chunks` <= 4
// consecutive 256-float chunks of `x` into chunk slots chunk0.. of the shared scratch.
struct QuantTile {
    const float* x;      // first float of the workgroup's chunks
    uint32_t chunk0;     // destination chunk index
    uint32_t n_elems;    // floats to quantize (<= 1024; a per-32 input may end inside a chunk)
    // An op of two rows and more that a plan folded into the quantizer of the Linears reading it
    // (tiles then stay inside one row): the workgroup evaluates the op on its floats with the
    // stand-alone kernel's arithmetic, stores them to `pre_dst` and quantizes them.
    //   1  gated activation: act(x[e]) * x2[e]
    //   2  RmsNorm of the row `row` (dim floats): x[e] * scale * x2[e], x2 = the weight from the tile's first column on
    uint32_t pre = 0;
    const float* x2 = nullptr;
    float* pre_dst = nullptr;
    const float* row = nullptr;
    uint32_t dim = 0;
    float eps = 0.0f;
    int32_t act = 0, has_clamp = 0;
    float clamp = 0.0f;
};
void launch_quantize_q8_group(const QuantTile* tiles_dev, size_t n_tiles, bool per32, const ActQ8& out,
                              hipStream_t stream);
// Per-256 quantizer writing MFMA A-operand order (token groups of 32) into the same buffers.
void launch_quantize_q8_tiled(const float* x, size_t m, size_t k, const ActQ8& out, hipStream_t stream);
// Per-32 quantizer in the tiled code order (k % 32 == 0; a row is padded with zero blocks to whole
// 256-element steps, nb = ceil(k / 256)): out.d f32 [(g*nb + b)*32 + token%32][8],
// out.bsums the code sums in the same order, as f32. transposed16: every 16-element group's codes 4 x 4
// transposed (dword i = elements i, 4 + i, 8 + i, 12 + i), the order Q2_0's prefill kernel multiplies in.
void launch_quantize_q8_32_tiled(const float* x, size_t m, size_t k, bool transposed16, const ActQ8& out,
                                 hipStream_t stream);

// Optional per-block integer-stage outputs, i32 [m][out_f][blocks] (nullptr = not wanted).
struct IntStages {
    int32_t* a = nullptr;
    int32_t* b = nullptr;
};

// Small-batch GEMV: m activation rows (already quantized) against every weight row, the weights
// streamed once per chunk of up to 8 rows. y is [m][out_f]; stages [m][out_f][blocks].
bool launch_gemv_batch(int dtype, const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m,
                       size_t in_f, size_t out_f, const IntStages& st, hipStream_t stream);

// One m == 1 Op::Linear of a fused, grouped decode launch: the kernel quantizes x itself (into
// LDS) and produces y. All ops of a group share (dtype, in_f).
// What the decode GEMV can absorb from the ops around an m == 1 Linear (plans fuse them):
//   before: x = gated_act(gate, up) (Op::GatedAct / GatedActFused) or x = rmsnorm(x_in) * w
//           (Op::RmsNorm), computed by every workgroup in its quantization prologue; the first
//           workgroup of the op also stores that f32 vector to `pre_dst` (the absorbed op's dst)
//   after:  add_dst[row] = y[row] + add_b[row] (Op::Add), next to the plain y store
//   paired: the op is the gate projection of a gated activation whose up projection has the same
//           shape and input; a workgroup computes the same rows of both matrices (half of its
//           waves each) and then also stores pair_dst[row] = act(y[row]) * pair_y[row]
//           (Op::GatedAct / GatedActFused evaluated where its operands are produced)
struct GemvFusion {
    const float* x2 = nullptr;   // GatedAct: up; RmsNorm: weight
    float* pre_dst = nullptr;    // nullptr: computed but not stored
    const float* add_b = nullptr;
    float* add_dst = nullptr;    // nullptr: no Add
    const uint8_t* pair_w = nullptr;  // first row of the up matrix; nullptr: not paired
    float* pair_y = nullptr;          // the up projection's output
    float* pair_dst = nullptr;        // the gated activation's output
    int32_t pre = 0;             // 0 none, 1 gated activation, 2 RmsNorm
    int32_t act = 0;             // gated activation kind (0 SiLU, 1 GELU, 2 sigmoid), of pre == 1 or of the pair
    int32_t has_clamp = 0;
    float clamp = 0.0f;
    float eps = 0.0f;
};

struct GemvOpDesc {
    const uint8_t* w;  // first selected weight row
    const float* x;    // f32 [in_f] (gate / un-normalised input when fus.pre != 0)
    float* y;          // f32 [out_f]
    uint64_t bpr;      // bytes per weight row
    int32_t out_f;
    GemvFusion fus;
    // optional per-block integer stages, i32 [out_f][blocks] (single-op launches only)
    int32_t* st_a = nullptr;
    int32_t* st_b = nullptr;
};

// What one workgroup of a grouped launch works on: `rows` consecutive weight rows of one op.
// The launcher keeps a table of these in device memory, indexed by blockIdx.x, so a workgroup
// finds its work with one run of scalar loads.
struct GemvTile {
    const uint8_t* w;  // first row of the tile
    const float* x;
    float* y;          // output of the tile's first row
    uint32_t bpr;
    int32_t rows;
    GemvFusion fus;    // add_b / add_dst already offset to the tile's first row; pre_dst only in
                       // the op's first tile
};

struct GemvGroupPlan {
    int total_wgs = 0;
    int waves_per_wg = 0;
    int rows_per_wg = 0;
    size_t lds_bytes = 0;
    bool streamed = false;  // the weight bytes go through per-wave LDS rings (gemv_rows_streamed)
};

// Chooses workgroup shape and rows per wave for a group. false = no kernel for (dtype, in_f).
bool plan_gemv_group(int dtype, size_t in_f, const GemvOpDesc* ops, int n, GemvGroupPlan* plan);
// Writes the plan's total_wgs tiles for ops[0..n).
void fill_gemv_tiles(const GemvOpDesc* ops, int n, const GemvGroupPlan& plan, GemvTile* tiles);

// Launches a planned group. `tiles_dev` is the device copy of the tile table; it may be null when
// n == 1 (the single op's descriptor then travels as a kernel argument).
bool launch_gemv_fused(int dtype, size_t in_f, const GemvOpDesc* ops, int n, const GemvTile* tiles_dev,
                       const GemvGroupPlan& plan, hipStream_t stream);

// m >= 2: GEMM over on-device quantized activations. y is [m][out_f] row-major.
// m >= 2: quantizes x [m, in_f] into `act` (sized for m rounded up to 32 rows) in the layout the
// chosen kernel reads, then multiplies.
// `cus`: the device's compute units (the prefill kernels size their grids in rounds of them).
// What the activation scratch currently holds: the quantization of the m x in_f floats at `x` in
// `layout` (0: nothing known). A caller that runs several Linears over one activation tensor with
// nothing in between that writes the scratch or x (q / k / v, gate / up of a prefill chunk) passes
// the same QuantCache to each: the quantizer then runs once.
struct QuantCache {
    const float* x = nullptr;
    size_t m = 0, in_f = 0;
    int layout = 0;  // 1 row-major per-256, 2 row-major per-32, 3 tiled per-256, 4 tiled per-32, 5 tiled per-32 transposed
};
bool launch_mmq(int dtype, const uint8_t* w, size_t bpr, const float* x, const ActQ8& act, float* y,
                size_t m, size_t in_f, size_t out_f, const IntStages& st, int cus, hipStream_t stream,
                QuantCache* qc = nullptr);

// Small-batch ops of one dependency level that share (dtype, in_f, m), as ONE launch: the
// workgroups index a tile table. `act_elem0` is where the op's quantized activation rows start
// in the scratch (elements; a multiple of 256).
struct BatchTile {
    const uint8_t* w;    // first weight row of the tile
    float* y;            // y + first row
    uint32_t act_elem0;
    uint32_t out_f;      // row stride of y
    uint32_t rows;       // weight rows in this tile
    uint32_t bpr;
    // an Op::Add on the op's output that the plan folded into this launch (both at the tile's
    // first row, strided like y): add_dst = y + add_b; null: none
    const float* add_b = nullptr;
    float* add_dst = nullptr;
};
struct BatchGroupPlan {
    int kind = 0;          // 0: dot4 batch GEMV, 1: K-split MFMA kernel (Q4_K)
    int rows_per_wg = 0;
    int rows_per_wave = 0; // kind 0
    int waves = 4;         // kind 1: waves per workgroup (4 or 8)
    size_t total_wgs = 0;
};
bool plan_batch_group(int dtype, size_t m, size_t in_f, const GemvOpDesc* ops, int n, BatchGroupPlan* plan);
void fill_batch_tiles(const GemvOpDesc* ops, const uint32_t* act_elem0, int n, const BatchGroupPlan& plan,
                      BatchTile* out);
bool launch_gemv_batch_group(int dtype, size_t m, size_t in_f, const BatchTile* tiles_dev,
                             const BatchGroupPlan& plan, const ActQ8& act, hipStream_t stream);
void launch_mmq_skinny_group(int dtype, size_t m, size_t in_f, const BatchTile* tiles_dev,
                             const BatchGroupPlan& plan, const ActQ8& act, hipStream_t stream);
// Small and middle batches on rows of whole 256-blocks (an even number of them for Q6_K and Q2_0):
// whether the K-split MFMA kernel with 16 x 16 tiles (mmq.hip) takes them, alone or as a plan's
// group of 32-row tiles; the thresholds are per format, row length and matrix size.
bool mmq_skinny16_takes(int dtype, size_t m, size_t in_f, size_t out_f);

// Which activation quantizer infr-cpu's dispatch pairs with a weight format
// (crates/infr-cpu/src/lib.rs:1037-1076, 1322-1412): per-32 `Q8x32` for the 32-weight-block
// formats and Q2_0, and for Q8_0 rows that are not whole 256s; per-256 `Q8` otherwise.
inline bool act_is_per32(int dtype, size_t in_f) {
    switch (dtype) {
    case 2: case 3: case 6: case 7: case 20: case 42: case 39: case 40: return true;
    case 8: return in_f % 256 != 0;
    default: return false;
    }
}

// One token of a format without an int8 decode arm multiplies f32 activations (gemv_f32act.hip).
bool gemv_takes_f32_activations(int dtype, size_t m);
bool launch_gemv_f32act(int dtype, const uint8_t* w, size_t bpr, const float* x, float* y, size_t in_f,
                        size_t out_f, hipStream_t stream);
// Plans: the one-token Linears of a level that take this kernel and share (dtype, in_f) run as one
// launch over a tile table (GemvTile: w, x, y, bpr, rows; no fusion fields are read).
bool gemv_f32act_groups(int dtype, size_t in_f);
int gemv_f32act_group_rows(size_t total_rows, size_t in_f);
bool launch_gemv_f32act_group(int dtype, size_t in_f, const GemvTile* tiles_dev, int n_tiles, hipStream_t stream);

// Op::EmbedGather: dst[r, :] = decode(table[ids[r], :]) * scale, rows decoded from the raw blocks.
bool embed_gather_supported(int dtype);
void launch_embed_gather(int dtype, const uint8_t* table, size_t bpr, size_t total_rows, const int32_t* ids,
                         size_t rows, size_t ne, float scale, float* dst, hipStream_t stream);

// Read-only streaming pass (measurement aid): `out` holds one int per workgroup.
void launch_stream_read(const void* src, size_t bytes, int* out, int workgroups, bool nontemporal, hipStream_t stream);
void launch_mfma_i8_peak(int* out, int workgroups, int iters, int random_data, hipStream_t stream);

// The decode-GEMV launchers of one weight format. Each format's kernels are instantiated in one
// translation unit, which also defines its accessor below.
struct GemvFormatOps {
    int elems_per_step = 0;  // K elements one wave step covers
    bool (*batch)(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m, size_t in_f,
                  size_t out_f, const IntStages& st, hipStream_t stream) = nullptr;
    bool (*batch_group)(const BatchTile* tiles, const BatchGroupPlan& plan, const ActQ8& act, size_t m,
                        size_t in_f, hipStream_t stream) = nullptr;
    bool (*plan_group)(size_t in_f, const GemvOpDesc* ops, int n, GemvGroupPlan* plan) = nullptr;
    bool (*fused)(size_t in_f, const GemvOpDesc& op, const GemvTile* tiles_dev, const GemvGroupPlan& plan,
                  hipStream_t stream) = nullptr;
};
// Rows longer than eight wave steps of the format's decode mapping have no decode or small-batch
// kernel; when they are whole 256s the prefill kernels (which walk the blocks) take them at any m.
bool gemv_row_too_long(int dtype, size_t in_f);
const GemvFormatOps& gemv_ops_q4k();
const GemvFormatOps& gemv_ops_q6k();
const GemvFormatOps& gemv_ops_q8_0();
const GemvFormatOps& gemv_ops_q8_0_32();
const GemvFormatOps& gemv_ops_q8_0_32_aligned();  // rows of whole 64s
const GemvFormatOps& gemv_ops_q2_0();
const GemvFormatOps& gemv_ops_q2_0_aligned();  // rows of whole 128s
const GemvFormatOps& gemv_ops_q5k();
const GemvFormatOps& gemv_ops_q2k();
const GemvFormatOps& gemv_ops_q3k();
const GemvFormatOps& gemv_ops_iq4xs();
const GemvFormatOps& gemv_ops_tq1_0();
const GemvFormatOps& gemv_ops_tq2_0();
const GemvFormatOps& gemv_ops_mxfp4();
const GemvFormatOps& gemv_ops_nvfp4();
const GemvFormatOps& gemv_ops_q4_0();
const GemvFormatOps& gemv_ops_q4_1();
const GemvFormatOps& gemv_ops_q5_0();  // batch launchers only: one token takes the f32 kernel
const GemvFormatOps& gemv_ops_q5_1();
const GemvFormatOps& gemv_ops_iq4nl();
// rows of whole 64s: two 2-mod-4-stride blocks per lane
const GemvFormatOps& gemv_ops_q4_0_pair();
const GemvFormatOps& gemv_ops_iq4nl_pair();
const GemvFormatOps& gemv_ops_q5_0_pair();

// Elementwise ops either side of a Linear (elementwise.hip).
struct GatedActShape {
    uint32_t rows, nff;
    int act;  // 0 SiLU, 1 GELU (tanh form), 2 sigmoid
    uint32_t up_off, up_stride, gate_stride, gate_block_width;
    int has_clamp;
    float clamp;
};
void launch_rms_norm(const float* x, const float* w, float* out, size_t rows, size_t dim, float eps,
                     bool accumulate, hipStream_t stream);
void launch_gated_act(const float* gate, const float* up, float* out, const GatedActShape& s,
                      hipStream_t stream);
void launch_add(const float* a, const float* b, float* out, size_t n, hipStream_t stream);

// Op::MoeFfn. Expert e of a bank starts at bank + e * stride.
// Routing (crates/infr-core/src/graph.rs:956-1010): how logits become probabilities, what the
// selection ranks, how the selected probabilities become weights.
struct MoeRoute {
    int gating = 0;  // 0 softmax, 1 sigmoid, 2 sqrt(softplus)
    int norm_w = 1;  // w = p / max(sum_sel p, 1e-20) * scale, else p * scale
    int n_groups = 0, n_groups_used = 0;  // group-limited routing when n_groups > 1 and n_groups_used > 0
    const float* bias = nullptr;          // exp_probs_b [n_expert]: added for the selection only
    const int32_t* ids = nullptr;         // expert_ids [rows, n_used]: the selection itself
};
// The experts' gated activation (graph.rs:948-967).
struct MoeAct {
    int act = 0;  // 0 SiLU, 1 GELU (tanh form), 2 sigmoid
    int has_clamp = 0;
    float clamp = 0.0f;
    int weight_before = 0;  // the routing weight on gate / up in front of the activation, not on the output
};
struct MoeShape {
    int ne, n_expert, n_used, n_ff, rows;
    float scale;
    int router_dtype, gate_dtype, up_dtype, down_dtype;
    MoeRoute route;
    MoeAct act;
    int fused_gate_up = 0;  // `gate` holds [gate rows | up rows] per expert; `up` is not read
};
struct MoeBuffers {
    const float* x;         // [rows, ne]
    const float* router_x;  // [rows, ne]
    const float* router;    // f32 [n_expert, ne]
    const uint8_t* gate;
    const uint8_t* up;
    const uint8_t* down;
    size_t gate_stride, up_stride, down_stride;
    float* dst;             // [rows, ne]
    int32_t* sel_idx;       // optional [rows, n_used]
    float* sel_w;           // optional [rows, n_used]
    const float* down_scale = nullptr;  // optional f32 [n_expert]: y_e * down_scale[e] before the weighted sum
    // absorbed Op::Add (fusion.rs:155-200): add_dst[i] = dst[i] + add_b[i] from the kernel that
    // produces dst; add_dst may be add_b (each element is read and written by one thread)
    const float* add_b = nullptr;
    float* add_dst = nullptr;
    // absorbed single-row Op::RmsNorm in front (fusion.rs:58-73, `moe_ok`): router_x is then the
    // norm's input; the router kernel normalises it (rms_norm_kernel's arithmetic and order), its
    // first workgroup stores the result to `norm_dst`, and x must be that same `norm_dst`
    const float* norm_w = nullptr;
    float* norm_dst = nullptr;
    float norm_eps = 0.0f;
};
// Q6_K prefill GEMM on the int8 matrix cores (any m; used from 33 tokens): activations in the tiled quantizer's layout
// (launch_quantize_q8_tiled); st.a, when set, receives isum per (token, row, 256-block).
void launch_mmq_shared_q6k(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m, size_t in_f,
                           size_t out_f, const IntStages& st, hipStream_t stream);
// The same for Q8_0 rows that are whole 256s; st.a receives iprod per (token, row, 32-block).
void launch_mmq_shared_q8_0(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m, size_t in_f,
                            size_t out_f, const IntStages& st, hipStream_t stream);
// The same for Q5_K; st.a / st.b receive sd / sm per (token, row, 256-block).
void launch_mmq_shared_q5k(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m, size_t in_f,
                           size_t out_f, const IntStages& st, hipStream_t stream);
// The same for Q2_K; st.a / st.b receive sd / sm per (token, row, 256-block).
void launch_mmq_shared_q2k(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m, size_t in_f,
                           size_t out_f, const IntStages& st, hipStream_t stream);
// The same for Q3_K, TQ2_0 and TQ1_0; st.a receives isum / iprod per (token, row, 256-block).
void launch_mmq_shared_q3k(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m, size_t in_f,
                           size_t out_f, const IntStages& st, hipStream_t stream);
void launch_mmq_shared_tq2_0(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m, size_t in_f,
                             size_t out_f, const IntStages& st, hipStream_t stream);
void launch_mmq_shared_tq1_0(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m, size_t in_f,
                             size_t out_f, const IntStages& st, hipStream_t stream);
// The same for IQ4_XS; st.a receives isum per (token, row, 256-block).
void launch_mmq_shared_iq4xs(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m, size_t in_f,
                             size_t out_f, const IntStages& st, hipStream_t stream);
// The same for Q4_0 / Q4_1 / Q5_0 / Q5_1 / IQ4_NL (and Q2_0: transposed16 activations) rows that are whole
// 256s, against the per-32 activation in the tiled order (launch_quantize_q8_32_tiled); st.a receives
// iprod per (token, row, 32-element block).
bool launch_mmq_shared_nib32(int dtype, const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m,
                             size_t in_f, size_t out_f, const IntStages& st, hipStream_t stream);
// Q4_K strip form (mmq_q4k_strip.hip): 256 tokens x (32 * tiles) rows per workgroup, activations in
// the tiled quantizer's layout. mmq_strip_q4k_tiles picks the strip height (1..3 row tiles) for a device
// of `cus` compute units.
// exact: the f32 epilogue as infr-cpu writes it (y bit-identical) instead of the contracted one.
// One strip of a grouped launch: `rows` (at most the strip height) rows of one op, whose outputs
// go to y[token * ldy + row].
struct StripSeg {
    const uint8_t* w;  // the strip's first weight row
    float* y;          // the op's output at the strip's first row
    int32_t ldy;       // the op's out_f
    int32_t rows;
};
int mmq_strip_q4k_tiles(size_t m, size_t out_f, size_t in_f, int cus);
int mmq_strip_q4k_rows(int tiles);
bool mmq_q4k_strip_group_takes(size_t m, size_t in_f, size_t total_out_f);
// Several Q4_K Linears over one quantized activation tensor as one launch (the 1e-4 form).
void launch_mmq_strip_q4k_group(size_t bpr, const ActQ8& act, size_t m, size_t in_f, int tiles, const StripSeg* segs_dev,
                                int n_segs, hipStream_t stream);
void launch_mmq_strip_q4k(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m, size_t in_f,
                          size_t out_f, const IntStages& st, int tiles, bool exact, hipStream_t stream);
// Routed pairs bucketed by expert, in tiles of at most 32 pairs of one expert each (device arrays;
// `*n_tiles` of the `max_tiles` entries exist). `perm` lists the pairs expert by expert.
struct MoeTileTable {
    const int32_t* n_tiles;
    const int32_t* expert;
    const int32_t* slot0;
    const int32_t* count;
    const int32_t* perm;
    int max_tiles;
};
// Q4_K int8-MFMA GEMM over such tiles: tile i multiplies rows perm[slot0[i]..] / act_div of the
// quantized activations with expert[i]'s slice of `bank` and writes y[perm[..], :]. Same integers
// and f32 epilogue as the dense kernel, so every output equals the per-pair GEMV's bit for bit.
void launch_mmq_q4k_gathered(const uint8_t* bank, size_t expert_stride, size_t bpr, const ActQ8& act, int act_div,
                             const MoeTileTable& t, float* y, size_t in_f, size_t out_f, hipStream_t stream);
// The same by bank format: Q4_K through the call above, Q5_K / Q6_K / Q8_0 through their tile kernels
// (mmq_gathered.hip). false: the format has no bucketed kernel.
bool launch_mmq_gathered(int dtype, const uint8_t* bank, size_t expert_stride, size_t bpr, const ActQ8& act,
                         int act_div, const MoeTileTable& t, float* y, size_t in_f, size_t out_f,
                         hipStream_t stream);
size_t moe_workspace_bytes(const MoeShape& s);
// Enqueues the whole op; returns nullptr or a message naming what is unsupported.
const char* launch_moe_ffn(const MoeShape& s, const MoeBuffers& b, void* workspace, hipStream_t stream);
// Op::Linear over plain f32 (dtype 0), f16 (1) or bf16 (30) weight rows: y[t, o] = dot(w[o], x[t]) in
// infr-cpu's `dot` order (in_f a multiple of 32). False when the shape has no launch.
bool launch_linear_plain_rows(int dtype, const void* w, const float* x, float* y, size_t m, size_t in_f, size_t out_f,
                              hipStream_t stream);

}  // namespace infr
