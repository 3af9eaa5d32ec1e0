// Templates of the decode GEMV kernels and their launchers, parameterised by a format policy
// (gemv_formats.hpp). gemv.hip describes the kernels and holds the per-dtype dispatch; each
// gemv_fmt_*.hip instantiates this header for a few formats, so the formats compile in parallel.
#pragma once

#include <algorithm>
#include <cstdlib>

#include "gemv_formats.hpp"
#include "gemv_rows.hpp"
#include "kernels.hpp"
#include "quant_chunk.hpp"

namespace infr {

// Small batch (2..8 activation rows already quantized in device memory): weights stream once.
// With `tiles` (plans) a workgroup takes one table entry - some rows of one of several ops - and
// blockIdx.y selects the pass of MB activation rows; `m_valid` is then the op's total row count.
template <typename F, int STEPS, int MB, bool STAGES>
__global__ __launch_bounds__(256) void gemv_batch_kernel(const uint8_t* __restrict__ w, size_t bpr,
                                                         ActPtrs act, int m_valid, int in_f,
                                                         float* y, int out_f,
                                                         int rows_per_wave, StagePtrs st,
                                                         const BatchTile* __restrict__ tiles) {
    const int lane = threadIdx.x & 63;
    int wave = blockIdx.x * 4 + (threadIdx.x >> 6);
    int n_rows = out_f;
    size_t act_elem0 = 0;
    BatchAdd add;
    if (tiles) {
        const BatchTile t = tiles[blockIdx.x];
        const int pass = blockIdx.y;
        w = t.w;
        bpr = t.bpr;
        out_f = (int)t.out_f;
        n_rows = (int)t.rows;
        y = t.y + (size_t)pass * MB * out_f;
        if (t.add_dst) add = BatchAdd{t.add_b + (size_t)pass * MB * out_f, t.add_dst + (size_t)pass * MB * out_f};
        act_elem0 = (size_t)t.act_elem0 + (size_t)pass * MB * in_f;
        m_valid = min(MB, m_valid - pass * MB);
        wave = threadIdx.x >> 6;
    }
    const int row0 = wave * rows_per_wave;
    if (row0 >= n_rows) return;
    const int row_end = min(row0 + rows_per_wave, n_rows);
    const int n_units = F::units(in_f);
    typename F::Acts acts[MB][STEPS];
    typename F::Row first;
    bool ok[STEPS];
#pragma unroll
    for (int t = 0; t < STEPS; ++t) ok[t] = F::valid(t, lane, n_units);
    F::load_row(first, w + (size_t)row0 * bpr, 0, lane, ok[0]);
#pragma unroll
    for (int mi = 0; mi < MB; ++mi) {
        const int r = mi < m_valid ? mi : 0;  // padding rows reuse row 0; their outputs are dropped
        const size_t e = act_elem0 + (size_t)r * in_f;
        const ActPtrs a{act.qs + e, act.d + e / (F::kPer32 ? 32 : 256), act.bsums + e / 32,
                        act.bsums16 + e / 16};
#pragma unroll
        for (int t = 0; t < STEPS; ++t) F::load_acts(acts[mi][t], a, t, lane, ok[t]);
    }
    __shared__ __attribute__((aligned(16))) float osum[F::kOrdered ? 4 * OrderedSum<STEPS>::kFloatsPerWave : 4];
    const size_t st_stride = (size_t)out_f * (F::kBlockElems == 64 ? 2 * n_units : n_units);
    gemv_rows_batch<F, STEPS, MB, STAGES>(
        w, bpr, first, acts, ok, y, (size_t)out_f, m_valid, n_units, row0, row_end, lane, st, st_stride,
        osum + (threadIdx.x >> 6) * (F::kOrdered ? OrderedSum<STEPS>::kFloatsPerWave : 0), add);
}

// Small batch over rows longer than one wave step: K split over the waves of a workgroup. Wave w
// owns wave step w of every row of the workgroup's tile, so the activations of all MB tokens for
// that step fit its registers and the weights stream ONCE for the whole batch (the one-wave form
// above has to re-stream them once per 8 / STEPS tokens). Per row every wave leaves its share in
// LDS - for the ordered formats the per-block terms themselves, otherwise four partial sums - and after
// each group of rows the workgroup's threads finish one (row, token) output each: the terms in
// ascending block order, i.e. the CPU's `sumf +=` chain (bit-identical for Q4_K / Q5_K / Q6_K), or
// the waves' sums in wave order. Two LDS buffers alternate, so one barrier per group suffices.
// blockDim.x = 64 * (wave steps of a row), at most 512. Loads run two rows ahead.
template <int MB>
struct BatchKs {
    static constexpr int kRowsPerFlush = 64 / MB;  // 64 (row, token) outputs per flush
    // floats per (row, token): the waves' per-block terms (ordered) or their four row-of-16 sums
    __host__ __device__ static constexpr int row_stride(bool ordered, int nw) { return ordered ? nw * 16 + 4 : nw * 4; }
    __host__ __device__ static constexpr size_t lds_bytes(bool ordered, int nw) {
        return (size_t)2 * 64 * row_stride(ordered, nw) * sizeof(float);
    }
};

template <typename F, int MB, bool STAGES>
__global__ __launch_bounds__(512) void gemv_batch_ks_kernel(const uint8_t* __restrict__ w, size_t bpr,
                                                            ActPtrs act, int m_valid, int in_f,
                                                            float* y, int out_f,
                                                            int rows_per_wg, StagePtrs st,
                                                            const BatchTile* __restrict__ tiles) {
    extern __shared__ __attribute__((aligned(16))) float ks_lds[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    int row0 = blockIdx.x * rows_per_wg, n_rows = out_f;
    size_t act_elem0 = 0;
    BatchAdd add;
    if (tiles) {
        const BatchTile t = tiles[blockIdx.x];
        const int pass = blockIdx.y;
        w = t.w;
        bpr = t.bpr;
        out_f = (int)t.out_f;
        n_rows = (int)t.rows;
        y = t.y + (size_t)pass * MB * out_f;
        if (t.add_dst) add = BatchAdd{t.add_b + (size_t)pass * MB * out_f, t.add_dst + (size_t)pass * MB * out_f};
        act_elem0 = (size_t)t.act_elem0 + (size_t)pass * MB * in_f;
        m_valid = min(MB, m_valid - pass * MB);
        row0 = 0;
        rows_per_wg = n_rows;
    }
    if (row0 >= n_rows) return;
    const int row_end = min(row0 + rows_per_wg, n_rows);
    const int n_units = F::units(in_f);
    const bool ok = F::valid(wave, lane, n_units);
    typename F::Row q0, q1;  // this wave's step of the current row and of the next
    F::load_row(q0, w + (size_t)row0 * bpr, wave, lane, ok);
    F::load_row(q1, w + (size_t)(row0 + 1) * bpr, wave, lane, ok && row0 + 1 < row_end);
    typename F::Acts acts[MB];
#pragma unroll
    for (int mi = 0; mi < MB; ++mi) {
        const int r = mi < m_valid ? mi : 0;  // padding rows reuse row 0; their outputs are dropped
        const size_t e = act_elem0 + (size_t)r * in_f;
        const ActPtrs a{act.qs + e, act.d + e / (F::kPer32 ? 32 : 256), act.bsums + e / 32,
                        act.bsums16 + e / 16};
        F::load_acts(acts[mi], a, wave, lane, ok);
    }
    constexpr int RB = BatchKs<MB>::kRowsPerFlush;
    const int ls = BatchKs<MB>::row_stride(F::kOrdered, nw);
    const size_t st_stride = (size_t)out_f * (F::kBlockElems == 64 ? 2 * n_units : n_units);
    int buf = 0;
    for (int batch0 = row0; batch0 < row_end; batch0 += RB, buf ^= 1) {
        float* B = ks_lds + (size_t)buf * 64 * ls;
        const int nr = min(RB, row_end - batch0);
        for (int r = 0; r < nr; ++r) {
            const int row = batch0 + r;
            typename F::Row q2;
            F::load_row(q2, w + (size_t)(row + 2) * bpr, wave, lane, ok && row + 2 < row_end);
            float terms[MB];
#pragma unroll
            for (int mi = 0; mi < MB; ++mi) {
                const StagePtrs sm{STAGES ? st.a + mi * st_stride : nullptr,
                                   STAGES && st.b ? st.b + mi * st_stride : nullptr};
                terms[mi] = term_shared<F, STAGES>(q0, acts[mi], wave, lane, ok && mi < m_valid, sm,
                                                   (size_t)row * n_units);
                if (F::kOrdered) {
                    if ((lane & 3) == 0) B[(r * MB + mi) * ls + wave * 16 + (lane >> 2)] = terms[mi];
                }
            }
            if (!F::kOrdered) {
                // all MB tokens' lane terms reduced together: lane L ends with token L % MB summed
                // over its row of 16 lanes, and the first MB lanes of each row park that
                if constexpr (MB == 2 || MB == 4 || MB == 8) {
                    const float part = row16_transpose_sum<MB>(terms, lane);
                    if ((lane & 15) < MB) B[(r * MB + (lane & (MB - 1))) * ls + wave * 4 + (lane >> 4)] = part;
                } else {
#pragma unroll
                    for (int mi = 0; mi < MB; ++mi) {
                        const float tot = wave_sum_f(terms[mi]);
                        if (lane < 4) B[(r * MB + mi) * ls + wave * 4 + lane] = lane == 0 ? tot : 0.0f;
                    }
                }
            }
            q0 = q1;
            q1 = q2;
        }
        __syncthreads();
        for (int task = threadIdx.x; task < nr * MB; task += blockDim.x) {
            const float* tr = B + (size_t)task * ls;
            float acc = 0.0f;
            if (F::kOrdered) {
                for (int k = 0; k < 4 * nw; ++k) {
                    const v4f v = reinterpret_cast<const v4f*>(tr)[k];
                    acc += v.x;
                    acc += v.y;
                    acc += v.z;
                    acc += v.w;
                }
            } else {
                for (int k = 0; k < 4 * nw; ++k) acc += tr[k];
            }
            const int mi = task % MB;
            if (mi < m_valid) store_batch_out(y, add, (size_t)mi * out_f + batch0 + task / MB, acc);
        }
    }
}

// Rows per side of a paired tile at most (the workgroup keeps both sides' outputs in LDS).
constexpr int kPairRows = 128;

// act(gate) * up with the optional clamp, as Op::GatedAct evaluates one element
// (gated_act_fn, crates/infr-cpu/src/kernels.rs:6591-6597).
__device__ __forceinline__ float fused_gated_act(int act, bool has_clamp, float l, float gate, float up) {
    if (has_clamp) {
        gate = gate < l ? gate : l;
        up = up < -l ? -l : (up > l ? l : up);
    }
    // Every workgroup of the consuming GEMV recomputes the whole vector, so the transcendental is
    // the hardware's (v_exp_f32 on a log2(e)-scaled argument, v_rcp_f32): a dozen instructions per
    // element instead of forty, within 1e-6 relative of the library expf / tanhf forms
    // (tanh(z) = 1 - 2 / (1 + e^{2z})).
    float a;
    switch (act) {
    case 1: {
        const float z = 0.7978846f * (gate + 0.044715f * gate * gate * gate);
        const float th = 1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + __expf(2.0f * z));
        a = 0.5f * gate * (1.0f + th);
        break;
    }
    case 2: a = __builtin_amdgcn_rcpf(1.0f + __expf(-gate)); break;
    default: a = gate * __builtin_amdgcn_rcpf(1.0f + __expf(-gate)); break;
    }
    return a * up;
}

// Fused + grouped form. LDS: qs[in_f] | d[in_f/32] | bsums[in_f/32] | bsums16[in_f/16] | per-wave
// ordered-sum scratch.
// STAGES: the per-block integers of every row also go to single.st_a / st_b (single-op launches only).
// STREAMED: the weight rows go through per-wave LDS rings (gemv_rows_streamed). LDS is then
// rings[NW] | per-wave ordered-sum scratch, and the activation arrays lie over the start of the
// rings: they are dead once every wave holds its activation registers (a second barrier).
template <typename F, int STEPS, int NW, bool STAGES, bool STREAMED = false>
__global__ __launch_bounds__(NW * 64) void gemv_fused_kernel(GemvOpDesc single, int single_rows,
                                                             const GemvTile* __restrict__ tiles,
                                                             int in_f) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int lane = threadIdx.x & 63;
    // (as a scalar, so that the row, tile and chunk bookkeeping runs on the scalar unit)
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

    // This workgroup's rows: one table entry, or computed from the single op's descriptor.
    GemvTile tile;
    int first_row = 0;
    if (tiles != nullptr) {
        tile = tiles[blockIdx.x];
    } else {
        const int first = (int)blockIdx.x * single_rows;
        first_row = first;
        tile.w = single.w + (size_t)first * single.bpr;
        tile.x = single.x;
        tile.y = single.y + first;
        tile.bpr = (uint32_t)single.bpr;
        tile.rows = min(single_rows, single.out_f - first);
        tile.fus = single.fus;
        if (tile.fus.add_dst) {
            tile.fus.add_b += first;
            tile.fus.add_dst += first;
        }
        if (blockIdx.x != 0) tile.fus.pre_dst = nullptr;
    }
    // A paired tile (workgroup-uniform): the second half of the waves takes the same rows of the up matrix.
    const bool paired = tile.fus.pair_w != nullptr;
    const bool second = paired && wave >= NW / 2;
    const int side_waves = paired ? NW / 2 : NW;
    const uint8_t* const wrows = second ? tile.fus.pair_w : tile.w;
    float* const yrows = second ? tile.fus.pair_y : tile.y;
    // the two halves' outputs, kept for the gated activation at the end (a side has at most kPairRows rows)
    __shared__ float pair_out[2][kPairRows];
    float* const pair_lds = paired ? pair_out[second ? 1 : 0] : nullptr;
    const int rpw = (tile.rows + side_waves - 1) / side_waves;
    const int n_units = F::units(in_f);
    const int row0 = (second ? wave - NW / 2 : wave) * rpw;
    const int row_end = min(row0 + rpw, tile.rows);

    int8_t* l_qs = reinterpret_cast<int8_t*>(lds);
    float* l_d = reinterpret_cast<float*>(lds + in_f);
    int32_t* l_bs = reinterpret_cast<int32_t*>(lds + in_f + in_f / 8);
    int32_t* l_bs16 = reinterpret_cast<int32_t*>(lds + in_f + in_f / 4);

    // The wave's share of x (256-float chunks w, w+NW, ...) is requested first, then the first
    // weight row: the row streams in from HBM while x is quantized.
    const int n_chunks = (in_f + 255) / 256;
    constexpr int kMaxChunks = (STEPS * F::kElemsPerStep / 256 + NW - 1) / NW;
    v4f xv[kMaxChunks];
#pragma unroll
    for (int i = 0; i < kMaxChunks; ++i) {
        const int c = wave + i * NW;
        xv[i] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
        if (c < n_chunks && c * 256 + lane * 4 < in_f)
            xv[i] = gload<v4f>(tile.x + (size_t)c * 256 + lane * 4);
    }
    // An absorbed producer's second operand and an absorbed Add's residual are requested here as
    // well, so that they arrive with x instead of costing a memory round trip each later on.
    v4f ov[kMaxChunks];
    if (tile.fus.pre != 0) {
#pragma unroll
        for (int i = 0; i < kMaxChunks; ++i) {
            const int c = wave + i * NW;
            ov[i] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
            if (c < n_chunks && c * 256 + lane * 4 < in_f) ov[i] = gload<v4f>(tile.fus.x2 + (size_t)c * 256 + lane * 4);
        }
    }
    float add_first = 0.0f;  // add_b[row0 + lane]
    if (tile.fus.add_dst && row0 + lane < row_end) add_first = gload<float>(tile.fus.add_b + row0 + lane);
    const bool has_rows = row0 < tile.rows;
    // Rows of two or three wave steps: the rest of the first row is requested once x has arrived
    // (in front of the quantization), so that its round trips are spent under the prologue's
    // arithmetic and not one after the other behind it.
    constexpr bool kFirstWhole = STEPS == 2 || STEPS == 3;
    typename F::Row first[kFirstWhole ? STEPS : 1];
    bool ok[STEPS];
#pragma unroll
    for (int t = 0; t < STEPS; ++t) ok[t] = has_rows && F::valid(t, lane, n_units);
    // STREAMED: the image of this wave's rows starts at the line that holds their first byte
    const uint8_t* span = wrows + (size_t)row0 * tile.bpr;
    const uint32_t head = (uint32_t)(reinterpret_cast<uintptr_t>(span) & 127);
    const uint32_t total = has_rows ? (head + (uint32_t)(row_end - row0) * tile.bpr + 127) & ~127u : 0;
    typename std::conditional<STREAMED, RingChunk<ring_instr<F, STEPS, STREAMED>()>, int>::type chunks_ahead;
    if constexpr (STREAMED) {
        if (has_rows) ring_issue(span - head, 0, total, lane, chunks_ahead.v);  // (wave-uniform)
    }
    else F::load_row(first[0], wrows + (size_t)row0 * tile.bpr, 0, lane, ok[0]);
    // An absorbed producer of x (workgroup-uniform branch): every workgroup recomputes the vector
    // from the producer's inputs - cheaper than a launch of its own - and the op's first
    // workgroup stores it where the producer would have.
    if (tile.fus.pre != 0) {
        float scale = 1.0f;
        if (tile.fus.pre == 2) {  // RmsNorm: mean square over the row, tree order fixed by NW
            __shared__ float part[NW];
            float sq = 0.0f;
#pragma unroll
            for (int i = 0; i < kMaxChunks; ++i)
                sq += (xv[i].x * xv[i].x + xv[i].y * xv[i].y) + (xv[i].z * xv[i].z + xv[i].w * xv[i].w);
            sq = wave_sum_f(sq);
            if (lane == 0) part[wave] = sq;
            __syncthreads();
            float tot = 0.0f;
#pragma unroll
            for (int wv = 0; wv < NW; ++wv) tot += part[wv];
            scale = 1.0f / sqrtf(tot / (float)in_f + tile.fus.eps);
        }
#pragma unroll
        for (int i = 0; i < kMaxChunks; ++i) {
            const int c = wave + i * NW;
            if (c < n_chunks && c * 256 + lane * 4 < in_f) {
                const v4f o = ov[i];
                v4f r;
                if (tile.fus.pre == 2) {
                    r = v4f{xv[i].x * scale * o.x, xv[i].y * scale * o.y, xv[i].z * scale * o.z, xv[i].w * scale * o.w};
                } else {
                    const bool hc = tile.fus.has_clamp != 0;
                    r.x = fused_gated_act(tile.fus.act, hc, tile.fus.clamp, xv[i].x, o.x);
                    r.y = fused_gated_act(tile.fus.act, hc, tile.fus.clamp, xv[i].y, o.y);
                    r.z = fused_gated_act(tile.fus.act, hc, tile.fus.clamp, xv[i].z, o.z);
                    r.w = fused_gated_act(tile.fus.act, hc, tile.fus.clamp, xv[i].w, o.w);
                }
                xv[i] = r;
                if (tile.fus.pre_dst)
                    gstore<v4f>(tile.fus.pre_dst + (size_t)c * 256 + lane * 4, r);
            }
        }
    }
    if constexpr (kFirstWhole && !STREAMED) {
        asm volatile("" ::: "memory");  // not before the loads above have been waited for
#pragma unroll
        for (int t = 1; t < STEPS; ++t) F::load_row(first[t], wrows + (size_t)row0 * tile.bpr, t, lane, ok[t]);
    }
#pragma unroll
    for (int i = 0; i < kMaxChunks; ++i) {
        const int c = wave + i * NW;
        if (c < n_chunks)
            quantize_chunk<F::kPer32>(xv[i], c * 256 + lane * 4 < in_f, lane, (size_t)c, l_qs, l_d,
                                      l_bs, F::kPer32 ? nullptr : l_bs16);
    }
    __syncthreads();
    if (!STREAMED && !has_rows && !paired) return;

    ActPtrs act{l_qs, l_d, l_bs, l_bs16};
    typename F::Acts acts[STEPS];
#pragma unroll
    for (int t = 0; t < STEPS; ++t) F::load_acts(acts[t], act, t, lane, ok[t]);
    // stage outputs are indexed by the op's row: offset them to the tile's first
    const size_t st_off = (size_t)first_row * (F::kBlockElems == 64 ? 2 * n_units : n_units);
    const StagePtrs st{STAGES ? single.st_a + st_off : nullptr, STAGES && single.st_b ? single.st_b + st_off : nullptr};
    if constexpr (STREAMED) {
        __syncthreads();  // the rings lie over the activation arrays
        if (!has_rows && !paired) return;
        float* osum = reinterpret_cast<float*>(lds + (size_t)NW * WeightRingOf<F, STEPS>::kBytes) +
                      wave * RowSumScratch<F, STEPS>::kFloatsPerWave;
        if (has_rows)
            gemv_rows_streamed<F, STEPS, STAGES>(span - head, head, total, tile.bpr, chunks_ahead,
                                                 lds + (size_t)wave * WeightRingOf<F, STEPS>::kBytes, acts, ok, yrows, n_units,
                                                 row0, row_end, lane, st, osum, tile.fus.add_dst, add_first,
                                                 pair_lds);
    } else {
        float* osum = reinterpret_cast<float*>(lds + in_f + in_f / 2) + wave * RowSumScratch<F, STEPS>::kFloatsPerWave;
        if (has_rows)
            gemv_rows<F, STEPS, STAGES, kFirstWhole>(wrows, tile.bpr, first, acts, ok, yrows, n_units, row0, row_end, lane,
                                                     st, osum, tile.fus.add_b, tile.fus.add_dst, add_first, pair_lds);
    }
    if (paired) {
        // Both halves' outputs of this tile are in LDS once every wave is here: one gated activation per row.
        __syncthreads();
        const bool hc = tile.fus.has_clamp != 0;
        for (int i = (int)threadIdx.x; i < tile.rows; i += NW * 64)
            gstore<float>(tile.fus.pair_dst + i,
                          fused_gated_act(tile.fus.act, hc, tile.fus.clamp, pair_out[0][i], pair_out[1][i]));
    }
}

// ───────────────────────────────────── launch ─────────────────────────────────────

template <typename F, int STEPS, int MB>
static void launch_batch_one(const uint8_t* w, size_t bpr, const ActPtrs& act, int m_valid, size_t in_f,
                             float* y, size_t out_f, const StagePtrs& st, hipStream_t stream) {
    size_t rpw = (out_f + 4095) / 4096;
    rpw = rpw < 2 ? 2 : (rpw > 16 ? 16 : rpw);
    const size_t waves = (out_f + rpw - 1) / rpw;
    const dim3 grid((unsigned)((waves + 3) / 4)), block(256);
    if (st.a)
        hipLaunchKernelGGL((gemv_batch_kernel<F, STEPS, MB, true>), grid, block, 0, stream, w, bpr, act,
                           m_valid, (int)in_f, y, (int)out_f, (int)rpw, st, (const BatchTile*)nullptr);
    else
        hipLaunchKernelGGL((gemv_batch_kernel<F, STEPS, MB, false>), grid, block, 0, stream, w, bpr, act,
                           m_valid, (int)in_f, y, (int)out_f, (int)rpw, st, (const BatchTile*)nullptr);
}

// Activation rows per pass of the batch kernels (they live in registers): the K-split form keeps
// one wave step per wave, so it takes eight whatever the row length.
static int batch_rows_per_pass(int steps) {
    (void)steps;
    return 8;
}

// Rows per workgroup of the K-split form: whole flush groups; 8 to 16 rows measured best for eight
// tokens (larger tiles leave too few workgroups, and the one-wave form with several passes was no
// faster on any shape tried).
template <int MB>
static int batch_ks_rows_per_wg(size_t total_rows) {
    constexpr int RB = BatchKs<MB>::kRowsPerFlush;
    size_t r = (total_rows + 4095) / 4096;  // about 4096 workgroups for a large group of rows
    r = (r + RB - 1) / RB * RB;
    return (int)(r < (size_t)RB ? RB : (r > 32 && RB <= 32 ? 32 : r));
}

template <typename F, int MB, bool STAGES>
static void launch_batch_ks(const uint8_t* w, size_t bpr, const ActPtrs& act, int m_valid, size_t in_f,
                            float* y, size_t out_f, const StagePtrs& st, int steps, const BatchTile* tiles,
                            dim3 grid, int rows_per_wg, hipStream_t stream) {
    hipLaunchKernelGGL((gemv_batch_ks_kernel<F, MB, STAGES>), grid, dim3((unsigned)steps * 64),
                       BatchKs<MB>::lds_bytes(F::kOrdered, steps), stream, w, bpr, act, m_valid, (int)in_f, y,
                       (int)out_f, rows_per_wg, st, tiles);
}

template <typename F, int STEPS, int MB>
static void launch_batch_group_one(const BatchTile* tiles, const BatchGroupPlan& gp, const ActPtrs& act,
                                   int m, size_t in_f, hipStream_t stream) {
    const dim3 grid((unsigned)gp.total_wgs, (unsigned)((m + MB - 1) / MB)), block(256);
    hipLaunchKernelGGL((gemv_batch_kernel<F, STEPS, MB, false>), grid, block, 0, stream,
                       (const uint8_t*)nullptr, (size_t)0, act, m, (int)in_f, (float*)nullptr, 0,
                       gp.rows_per_wave, StagePtrs{nullptr, nullptr}, tiles);
}

template <typename F>
static bool launch_batch_group_fmt(const BatchTile* tiles, const BatchGroupPlan& gp, const ActQ8& a,
                                   size_t m, size_t in_f, hipStream_t stream) {
    const int steps = (int)((in_f + F::kElemsPerStep - 1) / F::kElemsPerStep);
    const ActPtrs act{a.qs, a.d, a.bsums, a.bsums16};
    if (steps < 1 || steps > 8) return false;
    const int mb = std::min((int)m, batch_rows_per_pass(steps));
    if (steps == 1) {
        if (mb > 4) launch_batch_group_one<F, 1, 8>(tiles, gp, act, (int)m, in_f, stream);
        else if (mb > 2) launch_batch_group_one<F, 1, 4>(tiles, gp, act, (int)m, in_f, stream);
        else launch_batch_group_one<F, 1, 2>(tiles, gp, act, (int)m, in_f, stream);
        return true;
    }
    // rows longer than a wave step: K split over the workgroup's waves, one tile per workgroup
    const StagePtrs none{nullptr, nullptr};
#define INFR_G(MB)                                                                                         \
    launch_batch_ks<F, MB, false>(nullptr, 0, act, (int)m, in_f, nullptr, 0, none, steps, tiles,           \
                                  dim3((unsigned)gp.total_wgs, (unsigned)((m + MB - 1) / MB)), 0, stream)
    if (mb > 4) INFR_G(8); else if (mb > 2) INFR_G(4); else INFR_G(2);
#undef INFR_G
    return true;
}

// m activation rows in chunks of MB <= 8 / STEPS (the activations live in registers).
template <typename F>
static bool launch_batch_fmt(const uint8_t* w, size_t bpr, const ActQ8& a, float* y, size_t m,
                             size_t in_f, size_t out_f, const IntStages& st, hipStream_t stream) {
    const int steps = (int)((in_f + F::kElemsPerStep - 1) / F::kElemsPerStep);
    if (steps < 1 || steps > 8) return false;
    const size_t dper = F::kPer32 ? in_f / 32 : in_f / 256;
    const size_t blocks = (F::kBlockElems == 64 ? 2 : 1) * (in_f / F::kBlockElems);
    const size_t mb_max = (size_t)batch_rows_per_pass(steps);
    for (size_t r0 = 0; r0 < m; r0 += mb_max) {
        const int mv = (int)std::min(mb_max, m - r0);
        const ActPtrs act{a.qs + r0 * in_f, a.d + r0 * dper, a.bsums + r0 * (in_f / 32),
                          a.bsums16 ? a.bsums16 + r0 * (in_f / 16) : nullptr};
        const StagePtrs sp{st.a ? st.a + r0 * out_f * blocks : nullptr,
                           st.b ? st.b + r0 * out_f * blocks : nullptr};
        float* yo = y + r0 * out_f;
        if (steps == 1) {
            if (mv > 4) launch_batch_one<F, 1, 8>(w, bpr, act, mv, in_f, yo, out_f, sp, stream);
            else if (mv > 2) launch_batch_one<F, 1, 4>(w, bpr, act, mv, in_f, yo, out_f, sp, stream);
            else if (mv > 1) launch_batch_one<F, 1, 2>(w, bpr, act, mv, in_f, yo, out_f, sp, stream);
            else launch_batch_one<F, 1, 1>(w, bpr, act, mv, in_f, yo, out_f, sp, stream);
            continue;
        }
#define INFR_B(MB)                                                                                          \
    do {                                                                                                    \
        const int rpw = batch_ks_rows_per_wg<MB>(out_f);                                                    \
        const dim3 grid((unsigned)((out_f + rpw - 1) / rpw));                                               \
        if (st.a) launch_batch_ks<F, MB, true>(w, bpr, act, mv, in_f, yo, out_f, sp, steps, nullptr, grid, rpw, stream); \
        else launch_batch_ks<F, MB, false>(w, bpr, act, mv, in_f, yo, out_f, sp, steps, nullptr, grid, rpw, stream);     \
    } while (0)
        if (mv > 4) INFR_B(8); else if (mv > 2) INFR_B(4); else if (mv > 1) INFR_B(2); else INFR_B(1);
#undef INFR_B
    }
    return true;
}


// Workgroups of the fused kernel that one compute unit holds at once (registers, LDS, wave slots),
// as the runtime computes it for the exact instantiation; 0 if the query fails.
template <typename F, int NW>
static int fused_wgs_per_cu_nw(int steps, size_t lds_bytes) {
    int nblk = 0;
#define INFR_CASE(N)                                                                                  \
    case N:                                                                                           \
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(                                             \
                &nblk, reinterpret_cast<const void*>(&gemv_fused_kernel<F, N, NW, false>), NW * 64, lds_bytes) != hipSuccess) \
            nblk = 0;                                                                                 \
        break;
    switch (steps) {
        INFR_CASE(1) INFR_CASE(2) INFR_CASE(3) INFR_CASE(4)
        INFR_CASE(5) INFR_CASE(6) INFR_CASE(7) INFR_CASE(8)
    default: break;
    }
#undef INFR_CASE
    return nblk;
}
template <typename F>
static int fused_wgs_per_cu(int steps, int nw, size_t lds_bytes) {
    switch (nw) {
    case 4: return fused_wgs_per_cu_nw<F, 4>(steps, lds_bytes);
    case 8: return fused_wgs_per_cu_nw<F, 8>(steps, lds_bytes);
    case 16: return fused_wgs_per_cu_nw<F, 16>(steps, lds_bytes);
    default: return 0;
    }
}
inline int device_cu_count() {
    static const int cus = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
            n = 0;
        return n;
    }();
    return cus;
}

template <typename F>
static bool plan_group_fmt(size_t in_f, const GemvOpDesc* ops, int n, GemvGroupPlan* plan) {
    const int steps = (int)((in_f + F::kElemsPerStep - 1) / F::kElemsPerStep);
    if (steps < 1 || steps > 8) return false;
    // (a paired op stands for the rows of two matrices: its workgroups take rows_per_wg / 2 of each)
    size_t total_rows = 0;
    for (int i = 0; i < n; ++i) total_rows += (size_t)ops[i].out_f * (ops[i].fus.pair_w ? 2 : 1);
    // Every workgroup re-quantizes x (about the arithmetic of eleven weight rows at in_f 4096), so
    // big groups take up to 128 rows per workgroup (more than that loses to the uneven tail);
    // small ones keep at least ~512 workgroups in flight. The workgroup is always as wide as the register budget allows, so that the
    // quantization is spread over the most waves; waves beyond the tile's rows retire after it.
    int nw = steps <= F::kWide16Steps ? 16 : 8;
    if (steps >= 3 && nw > 8) nw = 8;  // long rows: 8-wave workgroups measured faster
    size_t rows_per_wg = (total_rows + 511) / 512;
    rows_per_wg = rows_per_wg < 4 ? 4 : (rows_per_wg > 128 ? 128 : rows_per_wg);
    // activations, then every wave's row-sum scratch (OrderedSum<steps> or LaneSums)
    const size_t lds_bytes = in_f + in_f / 2 +
                             (size_t)nw * (F::kOrdered ? 16 * (16 * steps + 4) : (F::kLaneSums ? LaneSums::kFloatsPerWave : 0)) * sizeof(float);
    // Grids of only a few rounds: a grid that needs a little more than a whole number of rounds
    // idles most of the machine during the last one, and workgroups that share a compute unit
    // share its pipes, so what counts is workgroups per compute unit. For those grids take, among
    // tile heights near the one above, the one with the least modelled time
    // ceil(workgroups / CUs) x (rows + fixed cost); the fixed cost is the per-workgroup prologue
    // in units of a weight row: about eleven for quantizing x, more when the prologue also
    // evaluates an absorbed gated activation (expf per element) or RmsNorm. Grids of many rounds
    // keep the 128-row tiles: their tail is small and taller tiles measured slower.
    const int resident = device_cu_count() * fused_wgs_per_cu<F>(steps, nw, lds_bytes);
    const int cus = device_cu_count();
    double fixed = 11.0;
    for (int i = 0; i < n; ++i)
        fixed = std::max(fixed, ops[i].fus.pre == 1 ? 32.0 : (ops[i].fus.pre == 2 ? 15.0 : 11.0));
    auto wgs_at = [&](size_t r) {
        size_t w = 0;
        for (int i = 0; i < n; ++i) {
            const size_t per = ops[i].fus.pair_w ? r / 2 : r;
            w += ((size_t)ops[i].out_f + per - 1) / per;
        }
        return w;
    };
    if (resident > 0 && wgs_at(rows_per_wg) < (size_t)resident * 4) {
        const size_t lo = std::max<size_t>(4, rows_per_wg / 2), hi = std::max<size_t>(rows_per_wg * 2, 160);
        double best = 1e300;
        size_t best_r = rows_per_wg;
        for (size_t r = lo; r <= hi; ++r) {
            const size_t rounds = (wgs_at(r) + cus - 1) / cus;
            const double cost = (double)rounds * ((double)r + fixed);
            if (cost < best * 0.999) {  // ties go to the smaller tile
                best = cost;
                best_r = r;
            }
        }
        rows_per_wg = best_r;
    }
    int wg = (int)wgs_at(rows_per_wg);
    // A single round of workgroups: nothing else on the compute unit covers the prologue, so it is
    // spread over the widest workgroup that fits the registers (18.1 -> 15.4 us for a 4096 x 12288
    // Q4_K matrix behind an absorbed gated activation).
    if (steps <= F::kWide16Steps && cus > 0 && wg <= cus) nw = 16;
    // Many rounds of one-step rows: eight-wave workgroups of 64 rows or more, so that two or three of them
    // share a compute unit and one's prologue runs under the others' streaming (16-wave workgroups
    // fill the registers alone). Measured on the 216-matrix in_f 4096 group: Q4_K 6.05 -> 6.19 TB/s,
    // Q6_K 4.84 -> 5.25 and 5.35 -> 5.80 on its two shapes, Q5_K +3 %, the 32-weight-block formats
    // and Q2_0 unchanged; 32-row tiles cost those up to 15 % (more prologues per weight byte).
    if (steps == 1 && cus > 0 && wg > 4 * cus) {
        nw = 8;
        // (at least 64 rows and ~144 KB of weights per prologue: Q2_0's 1152-byte rows take 128 -
        // its sweep runs at 5.3 TB/s so, 4.9 with 64)
        const size_t cap = std::max<size_t>(64, (size_t)147456 / std::max<size_t>(1, ops[0].bpr));
        rows_per_wg = std::min<size_t>(rows_per_wg, cap);
        wg = (int)wgs_at(rows_per_wg);
    }
    const size_t sum_scratch =
        (size_t)nw * (F::kOrdered ? 16 * (16 * steps + 4) : (F::kLaneSums ? LaneSums::kFloatsPerWave : 0)) * sizeof(float);
    for (int i = 0; i < n; ++i)
        if (ops[i].fus.pair_w && rows_per_wg / 2 > (size_t)kPairRows) return false;
    plan->total_wgs = wg;
    plan->waves_per_wg = nw;
    plan->rows_per_wg = (int)rows_per_wg;
    // qs + d + bsums + bsums16, then the ordered-sum scratch of every wave
    plan->lds_bytes = in_f + in_f / 2 + sum_scratch;
    // Many rounds of workgroups: the weight bytes go through per-wave LDS rings as whole lines,
    // non-temporally (gemv_rows_streamed), 64 rows per eight-wave workgroup. Launches of a few rounds
    // measured slower that way - the ring adds a trip through LDS to every wave's start-up - and keep
    // the direct loads.
    plan->streamed = false;
    if constexpr (HasRingLoads<F>::value) {
        bool aligned = true;  // the ring's 16-byte pieces need 16-byte-aligned rows
        for (int i = 0; i < n; ++i)
            aligned = aligned && reinterpret_cast<uintptr_t>(ops[i].w) % 16 == 0 && ops[i].bpr % 16 == 0 && ops[i].st_a == nullptr;
        // (measured crossover: 139264 rows of 4096 columns, 98304 rows of 12288)
        const size_t wg64 = wgs_at(64);
        const size_t ring_bytes = ring_alloc_bytes<F>(steps);
        if (aligned && steps <= F::kRingMaxSteps && cus > 0 && wg64 > (size_t)8 * cus &&
            in_f + in_f / 2 <= (size_t)8 * ring_bytes) {
            plan->streamed = true;
            plan->waves_per_wg = 8;
            plan->rows_per_wg = 64;
            plan->total_wgs = (int)wg64;
            plan->lds_bytes = (size_t)8 * ring_bytes + (size_t)8 * 16 * (16 * steps + 4) * sizeof(float);
        }
    }
    return true;
}

static bool bpr_too_big(const GemvOpDesc* ops, int n) {
    for (int i = 0; i < n; ++i)
        if (ops[i].bpr > 0xFFFFFFFFull) return true;
    return false;
}

template <typename F, int NW, bool STAGES>
static bool launch_fused_nw(int steps, size_t in_f, const GemvOpDesc& op, const GemvTile* tiles_dev,
                            const GemvGroupPlan& plan, hipStream_t stream) {
    const dim3 grid((unsigned)plan.total_wgs), block(NW * 64);
#define INFR_CASE(N)                                                                                  \
    case N:                                                                                           \
        hipLaunchKernelGGL((gemv_fused_kernel<F, N, NW, STAGES>), grid, block, plan.lds_bytes, stream, \
                           op, plan.rows_per_wg, tiles_dev, (int)in_f);                             \
        return true;
    switch (steps) {
        INFR_CASE(1) INFR_CASE(2) INFR_CASE(3) INFR_CASE(4)
        INFR_CASE(5) INFR_CASE(6) INFR_CASE(7) INFR_CASE(8)
    default: return false;
    }
#undef INFR_CASE
}

template <typename F>
static bool launch_fused_fmt(size_t in_f, const GemvOpDesc& op, const GemvTile* tiles_dev,
                             const GemvGroupPlan& plan, hipStream_t stream) {
    const int steps = (int)((in_f + F::kElemsPerStep - 1) / F::kElemsPerStep);
    if constexpr (HasRingLoads<F>::value) {
        if (plan.streamed) {
            if (plan.waves_per_wg != 8 || steps > F::kRingMaxSteps || op.st_a != nullptr) return false;
            const dim3 grid((unsigned)plan.total_wgs), block(512);
#define INFR_STREAMED(N)                                                                                          \
    do {                                                                                                          \
        if (plan.lds_bytes > 64 * 1024)                                                                           \
            (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&gemv_fused_kernel<F, N, 8, false, true>),    \
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)plan.lds_bytes);           \
        hipLaunchKernelGGL((gemv_fused_kernel<F, N, 8, false, true>), grid, block, plan.lds_bytes, stream, op,    \
                           plan.rows_per_wg, tiles_dev, (int)in_f);                                               \
    } while (0)
            if (steps == 1) INFR_STREAMED(1);
            if constexpr (F::kRingMaxSteps >= 3) {
                if (steps == 2) INFR_STREAMED(2);
                if (steps == 3) INFR_STREAMED(3);
            }
#undef INFR_STREAMED
            return true;
        }
    }
    if (op.st_a != nullptr) {
        // the integer-stage outputs: the same kernel, single-op launches only
        if (tiles_dev != nullptr) return false;
        switch (plan.waves_per_wg) {
        case 4: return launch_fused_nw<F, 4, true>(steps, in_f, op, tiles_dev, plan, stream);
        case 8: return launch_fused_nw<F, 8, true>(steps, in_f, op, tiles_dev, plan, stream);
        case 16: return launch_fused_nw<F, 16, true>(steps, in_f, op, tiles_dev, plan, stream);
        default: return false;
        }
    }
    switch (plan.waves_per_wg) {
    case 4: return launch_fused_nw<F, 4, false>(steps, in_f, op, tiles_dev, plan, stream);
    case 8: return launch_fused_nw<F, 8, false>(steps, in_f, op, tiles_dev, plan, stream);
    case 16: return launch_fused_nw<F, 16, false>(steps, in_f, op, tiles_dev, plan, stream);
    default: return false;
    }
}


// The launchers of one format, as the per-dtype dispatch calls them.
template <typename F, bool DECODE = true>
GemvFormatOps make_gemv_format_ops() {
    GemvFormatOps o;
    o.elems_per_step = F::kElemsPerStep;
    o.batch = &launch_batch_fmt<F>;
    o.batch_group = &launch_batch_group_fmt<F>;
    if constexpr (DECODE) {
        o.plan_group = &plan_group_fmt<F>;
        o.fused = &launch_fused_fmt<F>;
    }
    return o;
}

}  // namespace infr
