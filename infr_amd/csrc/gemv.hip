// Decode GEMV (m == 1) for GGUF block-quantized weights against the int8-quantized activation,
// hand-written for gfx950 wave64. The per-format lane mappings are in gemv_formats.hpp.
//
// Common shape. One wavefront owns `rows_per_wave` consecutive weight rows. The K dimension is
// spread over the 64 lanes with a FIXED lane -> K-range mapping, so the int8 activation bytes a lane
// needs are loaded once into registers and reused for every row the wave processes. Weight bytes
// stream from HBM exactly once, with 16-byte loads that are contiguous across the wave; the next
// row's loads are issued before the current row is reduced. The kernels are HBM-bound: algorithmic
// traffic is the weight bytes (144 B / 210 B per 256 weights, 34 B per 32, 18 B per 64).
//
// Two entry kernels share that body:
//   gemv_kernel        activation already quantized in device memory (m >= 2 by rows, debug stages)
//   gemv_fused_kernel  the m == 1 product path: each workgroup quantizes x into LDS itself
//                      (quant_chunk.hpp, bit-exact with infr-cpu) while its first weight loads are
//                      in flight, and one launch serves a whole group of independent Op::Linear
//                      (descriptor table; blockIdx -> op by binary search), so a decode step needs
//                      one launch per dependency level instead of two per projection.
//
// Integer stages (v_dot4_i32_i8 sums, 6-bit scale products) are exact. The f32 epilogue evaluates
// the CPU expression per block with separate multiplies and adds. For Q4_K and Q6_K the per-block
// terms are then added in ascending block order (16 v_readlane + v_add per 16 blocks), which is
// the CPU's accumulation order, so y matches infr-cpu's scalar kernel bit for bit. For Q8_0 and
// Q2_0 (128 terms per 4096 columns) the lanes' terms are added with a fixed butterfly instead:
// deterministic, but rounded in a different order than the CPU's sequential sum.
#include "gemv_impl.hpp"

namespace infr {

// One table per format; each is defined in the gemv_fmt_*.hip that instantiates the format.
static const GemvFormatOps* format_ops(int dtype, size_t in_f) {
    switch (dtype) {
    case 12: return &gemv_ops_q4k();
    case 14: return &gemv_ops_q6k();
    case 8: return in_f % 256 == 0 ? &gemv_ops_q8_0() : (in_f % 64 == 0 ? &gemv_ops_q8_0_32_aligned() : &gemv_ops_q8_0_32());
    case 42: return in_f % 128 == 0 ? &gemv_ops_q2_0_aligned() : &gemv_ops_q2_0();
    case 13: return &gemv_ops_q5k();
    case 10: return &gemv_ops_q2k();
    case 11: return &gemv_ops_q3k();
    case 23: return &gemv_ops_iq4xs();
    case 34: return &gemv_ops_tq1_0();
    case 35: return &gemv_ops_tq2_0();
    case 39: return &gemv_ops_mxfp4();
    case 40: return &gemv_ops_nvfp4();
    case 2: return in_f % 64 == 0 ? &gemv_ops_q4_0_pair() : &gemv_ops_q4_0();
    case 3: return &gemv_ops_q4_1();
    case 6: return in_f % 64 == 0 ? &gemv_ops_q5_0_pair() : &gemv_ops_q5_0();
    case 7: return &gemv_ops_q5_1();
    case 20: return in_f % 64 == 0 ? &gemv_ops_iq4nl_pair() : &gemv_ops_iq4nl();
    default: return nullptr;
    }
}

bool gemv_row_too_long(int dtype, size_t in_f) {
    const GemvFormatOps* o = format_ops(dtype, in_f);
    return o != nullptr && in_f > (size_t)8 * (size_t)o->elems_per_step;
}

bool launch_gemv_batch_group(int dtype, size_t m, size_t in_f, const BatchTile* tiles_dev,
                             const BatchGroupPlan& plan, const ActQ8& act, hipStream_t stream) {
    const GemvFormatOps* f = format_ops(dtype, in_f);
    return f && f->batch_group(tiles_dev, plan, act, m, in_f, stream);
}

bool plan_batch_group(int dtype, size_t m, size_t in_f, const GemvOpDesc* ops, int n, BatchGroupPlan* plan) {
    size_t total_rows = 0;
    for (int i = 0; i < n; ++i) total_rows += (size_t)ops[i].out_f;
    BatchGroupPlan gp;
    size_t max_out_f = 0;
    for (int i = 0; i < n; ++i) max_out_f = std::max(max_out_f, (size_t)ops[i].out_f);
    // (Q8_0 at 5..8 tokens on rows of 8192 columns and more: only when the group fills the device twice over)
    const bool q8_0_long = dtype == 8 && m >= 5 && m <= 8 && in_f % 256 == 0 && in_f >= 8192 && total_rows >= 8192;
    if ((dtype != 12 || m > 32) &&
        (q8_0_long || mmq_skinny16_takes(dtype, m, in_f, max_out_f))) {  // the K-split MFMA kernel
        gp.kind = 1;
        gp.rows_per_wg = 32;
    } else if (dtype == 12 && m > 2) {  // Q4_K from three tokens: the K-split MFMA kernels, 32 rows per workgroup
        if (in_f % 256 != 0 || m > 32) return false;
        gp.kind = 1;
        gp.rows_per_wg = 32;
        const size_t wgs = (total_rows + 31) / 32;
        gp.waves = (in_f >= 8192 || (wgs * 4 < 1024 && in_f >= 2048)) ? 8 : 4;
    } else {
        const GemvFormatOps* f = format_ops(dtype, in_f);
        if (!f) return false;
        const size_t per_step = (size_t)f->elems_per_step;
        const size_t steps = (in_f + per_step - 1) / per_step;
        if (steps < 1 || steps > 8 || m > 8) return false;
        gp.kind = 0;
        if (steps == 1) {
            size_t rpw = (total_rows + 4095) / 4096;
            rpw = rpw < 2 ? 2 : (rpw > 16 ? 16 : rpw);
            gp.rows_per_wave = (int)rpw;
            gp.rows_per_wg = (int)rpw * 4;
        } else {
            // K-split form: a tile is one workgroup's rows, whole flush groups of 64 / MB rows
            const size_t rb = 64 / (m > 4 ? 8 : (m > 2 ? 4 : 2));
            size_t r = ((total_rows + 4095) / 4096 + rb - 1) / rb * rb;
            gp.rows_per_wave = 0;
            gp.rows_per_wg = (int)(r < rb ? rb : (r > 32 && rb <= 32 ? 32 : r));
        }
    }
    gp.total_wgs = 0;
    for (int i = 0; i < n; ++i) gp.total_wgs += ((size_t)ops[i].out_f + gp.rows_per_wg - 1) / gp.rows_per_wg;
    *plan = gp;
    return true;
}

void fill_batch_tiles(const GemvOpDesc* ops, const uint32_t* act_elem0, int n, const BatchGroupPlan& plan,
                      BatchTile* out) {
    size_t k = 0;
    for (int i = 0; i < n; ++i)
        for (int r0 = 0; r0 < ops[i].out_f; r0 += plan.rows_per_wg) {
            BatchTile t{ops[i].w + (size_t)r0 * ops[i].bpr, ops[i].y + r0, act_elem0[i],
                        (uint32_t)ops[i].out_f, (uint32_t)std::min(plan.rows_per_wg, ops[i].out_f - r0),
                        (uint32_t)ops[i].bpr};
            if (ops[i].fus.add_dst) {  // an Op::Add folded into the launch
                t.add_b = ops[i].fus.add_b + r0;
                t.add_dst = ops[i].fus.add_dst + r0;
            }
            out[k++] = t;
        }
}

bool launch_gemv_batch(int dtype, const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m,
                       size_t in_f, size_t out_f, const IntStages& st, hipStream_t stream) {
    if (out_f == 0 || m == 0) return true;
    const GemvFormatOps* f = format_ops(dtype, in_f);
    return f && f->batch(w, bpr, act, y, m, in_f, out_f, st, stream);
}

bool plan_gemv_group(int dtype, size_t in_f, const GemvOpDesc* ops, int n, GemvGroupPlan* plan) {
    if (n <= 0) return false;
    const GemvFormatOps* f = format_ops(dtype, in_f);
    return f && f->plan_group && f->plan_group(in_f, ops, n, plan);
}

void fill_gemv_tiles(const GemvOpDesc* ops, int n, const GemvGroupPlan& plan, GemvTile* tiles) {
    int t = 0;
    for (int i = 0; i < n; ++i) {
        // a paired op's workgroup takes half of its rows from each of the two matrices
        const int per_wg = ops[i].fus.pair_w ? plan.rows_per_wg / 2 : plan.rows_per_wg;
        for (int r = 0; r < ops[i].out_f; r += per_wg) {
            GemvTile& tl = tiles[t++];
            tl.w = ops[i].w + (size_t)r * ops[i].bpr;
            tl.x = ops[i].x;
            tl.y = ops[i].y + r;
            tl.bpr = (uint32_t)ops[i].bpr;
            tl.rows = ops[i].out_f - r < per_wg ? ops[i].out_f - r : per_wg;
            tl.fus = ops[i].fus;
            if (tl.fus.add_dst) {
                tl.fus.add_b += r;
                tl.fus.add_dst += r;
            }
            if (tl.fus.pair_w) {
                tl.fus.pair_w += (size_t)r * ops[i].bpr;
                tl.fus.pair_y += r;
                tl.fus.pair_dst += r;
            }
            if (r != 0) tl.fus.pre_dst = nullptr;
        }
    }
}

bool launch_gemv_fused(int dtype, size_t in_f, const GemvOpDesc* ops, int n, const GemvTile* tiles_dev,
                       const GemvGroupPlan& plan, hipStream_t stream) {
    if (n <= 0 || plan.total_wgs <= 0) return n == 0;
    if (n > 1 && tiles_dev == nullptr) return false;
    for (int i = 0; i < n; ++i)  // paired ops need the table, and carry neither an Add nor a gated producer
        if (ops[i].fus.pair_w && (tiles_dev == nullptr || ops[i].fus.add_dst || ops[i].fus.pre == 1 || ops[i].st_a))
            return false;
    if (bpr_too_big(ops, n)) return false;
    const GemvFormatOps* f = format_ops(dtype, in_f);
    return f && f->fused && f->fused(in_f, ops[0], tiles_dev, plan, stream);
}

}  // namespace infr
