// The row loop shared by every decode-GEMV entry kernel (plain, fused/grouped, id-gathered).
#pragma once

#include <type_traits>

#include "gemv_formats.hpp"

namespace infr {

// Per-wave LDS scratch for the ordered sum: 16 rows x (16*STEPS block terms + 4 pad) floats. The
// row stride 4*(4*STEPS+1) dwords makes the 16 lanes' 16-byte reads hit distinct banks.
template <int STEPS>
struct OrderedSum {
    static constexpr int kRowStride = 16 * STEPS + 4;
    static constexpr int kFloatsPerWave = 16 * kRowStride;
};

// The per-block term of one weight row when the same row meets several activation rows in
// registers: the format's shared-unpack form where it has one.
template <typename F, typename = void>
struct HasSharedTerm : std::false_type {};
template <typename F>
struct HasSharedTerm<F, std::void_t<decltype(&F::template term_shared<false>)>> : std::true_type {};
template <typename F, bool STAGES>
__device__ __forceinline__ float term_shared(const typename F::Row& r, const typename F::Acts& a, int t, int lane,
                                             bool ok, const StagePtrs& st, size_t row_units) {
    if constexpr (HasSharedTerm<F>::value) return F::template term_shared<STAGES>(r, a, t, lane, ok, st, row_units);
    else return F::template term<STAGES>(r, a, t, lane, ok, st, row_units);
}

// Per-wave LDS scratch of the butterfly formats: the lanes' sums of 8 rows, 64 + 4 pad floats per row
// (the pad spreads the flush's 16-byte reads over the banks).
struct LaneSums {
    static constexpr int kRows = 8, kRowStride = 68;
    static constexpr int kFloatsPerWave = kRows * kRowStride;
};
// Per-wave LDS scratch of the one-block-per-lane formats (Q8_0, the 32-weight-block formats) when
// their per-block terms must be added in ascending block order as infr-cpu's scalar kernels add them
// (kernels.rs:1170-1187: `sumf += d8 * d_w * iprod` block by block): every lane parks its block's
// term, 8 (long rows: 4) rows x (64 * STEPS terms + 4 pad) floats, and lane i then adds row i's terms in order.
template <int STEPS>
struct LaneOrderedSum {
    static constexpr int kRows = STEPS > 4 ? 4 : 8, kRowStride = 64 * STEPS + 4;  // (at most 33 KB for four waves)
    static constexpr int kFloatsPerWave = kRows * kRowStride;
};
// What gemv_rows needs per wave, by format.
template <typename F, int STEPS, bool LANE_ORDERED = false>
struct RowSumScratch {
    static constexpr int kFloatsPerWave =
        F::kOrdered ? OrderedSum<STEPS>::kFloatsPerWave
                    : (LANE_ORDERED ? LaneOrderedSum<STEPS>::kFloatsPerWave : (F::kLaneSums ? LaneSums::kFloatsPerWave : 1));
};

// Step 0 of a row known to be readable, through the format's unpredicated loader where it has one.
template <typename F>
__device__ __forceinline__ void load_row_clamped(typename F::Row& r, const uint8_t* rowp, int lane, bool ok) {
    if constexpr (F::kClampedLoads) F::load_row_clamped(r, rowp, 0, lane, ok);
    else F::load_row(r, rowp, 0, lane, ok);
}
// Whether the loop that runs one step ahead uses the unpredicated loader too (the loop that runs a
// whole row ahead always does): a format says kClampedOneAhead = false when its predicated loads
// measured faster there.
template <typename F, typename = void>
struct ClampedOneAhead : std::integral_constant<bool, F::kClampedLoads> {};
template <typename F>
struct ClampedOneAhead<F, std::void_t<decltype(F::kClampedOneAhead)>> : std::integral_constant<bool, F::kClampedOneAhead> {};

// The longest rows (in wave steps) that the loop running a whole row ahead takes: a format says
// kRowAheadMaxSteps when two register sets of longer rows cost it more than the lead buys.
template <typename F, typename = void>
struct RowAheadMaxSteps : std::integral_constant<int, 8> {};
template <typename F>
struct RowAheadMaxSteps<F, std::void_t<decltype(F::kRowAheadMaxSteps)>> : std::integral_constant<int, F::kRowAheadMaxSteps> {};

// Rows [row0, row_end) of one weight matrix against activation registers `acts`. `first` already
// holds step 0 of row0 - every step of it when FIRST_WHOLE - (the caller issues those loads as
// early as it can). The loads run one wave
// step (16 or 64 blocks) ahead of the arithmetic, across row boundaries, so a wave always has one
// step's bytes in flight (two and three steps ahead measured 3-10 % slower on the small-block
// formats, whose occupancy already covers the latency).
//
// Ordered formats (Q4_K, Q6_K): the CPU adds a row's per-block terms in ascending block order
// (`sumf +=`). The quad leaders park each row's terms in LDS (`osum`, this wave's private
// scratch) and, every 16 rows, lane i adds row i's terms in that order: the same rounding
// sequence as the CPU at about two instructions per row instead of a 16-deep v_readlane chain
// per step. Lanes past a row's last block contribute +0.0, which leaves the sum unchanged.
//
// `add_first` is add_b[row0 + lane], requested by the caller ahead of its prologue (an absorbed
// Op::Add); rows 64 and up of a wave read add_b when they are stored.
//
// LANE_ORDERED (formats that are not kOrdered, one block per lane): instead of a tree over the lanes,
// every lane parks its block's term in LDS (LaneOrderedSum) and every eight rows lane i adds row i's
// 64 * STEPS terms in ascending block order - the scalar CPU kernel's `sumf +=` chain, so the output
// equals its bit for bit. Lanes past a row's last block park +0.0. The routed-expert GEMVs take this
// form: their outputs are re-quantized to int8 for the down bank, where a last-bit difference in one
// activation can flip a code.
template <typename F, int STEPS, bool STAGES, bool FIRST_WHOLE = false, bool LANE_ORDERED = false>
__device__ __forceinline__ void gemv_rows(const uint8_t* __restrict__ w, size_t bpr,
                                          const typename F::Row (&first)[FIRST_WHOLE ? STEPS : 1],
                                          const typename F::Acts (&acts)[STEPS],
                                          const bool (&ok)[STEPS], float* __restrict__ y, int n_units,
                                          int row0, int row_end, int lane, const StagePtrs& st,
                                          float* osum, const float* add_b = nullptr,
                                          float* add_dst = nullptr, float add_first = 0.0f,
                                          float* y_lds = nullptr) {
    // y_lds: an LDS image of y (same row index) for a workgroup that reads its outputs back.
    // The residual of row r for an absorbed Add, from the lanes' prefetched values while
    // r - row0 < 64 (every lane of the wave must call this; `wanted` guards the late read).
    auto residual = [&](int r, bool wanted) {
        const float pf = __shfl(add_first, (r - row0) & 63, kWave);
        if (r - row0 < 64) return pf;
        return wanted ? gload<float>(add_b + r) : 0.0f;
    };
    // An absorbed Add may name this op's own dst as its dst (y = y + b as the graph writes it):
    // then only the sum is stored, through add_dst alone.
    const bool plain_y = y != add_dst;
    constexpr int LS = OrderedSum<STEPS>::kRowStride;
    constexpr int LSO = LaneOrderedSum<STEPS>::kRowStride;
    static_assert(!(LANE_ORDERED && F::kOrdered), "the ordered formats already add their blocks in order");
    int in_batch = 0, batch_row0 = row0;
    // A row's step-t term: parked for the ordered sum, or added to the lane's partial sum.
    auto take_term = [&](int t, float term, float& s) {
        if (LANE_ORDERED) {
            osum[in_batch * LSO + t * 64 + lane] = term;
        } else if (F::kOrdered) {
            if ((lane & 3) == 0) osum[in_batch * LS + t * 16 + (lane >> 2)] = term;
        } else {
            s += term;
        }
    };
    auto finish_row = [&](int row, float s) {
        if (LANE_ORDERED) {
            if (++in_batch == LaneOrderedSum<STEPS>::kRows || row + 1 == row_end) {
                const float resid = add_dst ? residual(batch_row0 + lane, lane < in_batch) : 0.0f;
                if (lane < in_batch) {
                    const v4f* tr = reinterpret_cast<const v4f*>(osum + lane * LSO);
                    float acc = 0.0f;
#pragma unroll 4
                    for (int k = 0; k < 16 * STEPS; ++k) {
                        const v4f v = tr[k];
                        acc += v.x;
                        acc += v.y;
                        acc += v.z;
                        acc += v.w;
                    }
                    if (plain_y) gstore<float>(y + batch_row0 + lane, acc);
                    if (y_lds) y_lds[batch_row0 + lane] = acc;
                    if (add_dst) gstore<float>(add_dst + batch_row0 + lane, acc + resid);
                }
                batch_row0 = row + 1;
                in_batch = 0;
            }
        } else if (F::kOrdered) {
            if (++in_batch == 16 || row + 1 == row_end) {
                const float resid = add_dst ? residual(batch_row0 + lane, lane < in_batch) : 0.0f;
                if (lane < in_batch) {
                    const v4f* tr = reinterpret_cast<const v4f*>(osum + lane * LS);
                    float acc = 0.0f;
#pragma unroll
                    for (int k = 0; k < 4 * STEPS; ++k) {
                        const v4f v = tr[k];
                        acc += v.x;
                        acc += v.y;
                        acc += v.z;
                        acc += v.w;
                    }
                    if (plain_y) gstore<float>(y + batch_row0 + lane, acc);
                    if (y_lds) y_lds[batch_row0 + lane] = acc;
                    // an absorbed Op::Add: dst = a + b with a = this output
                    if (add_dst) gstore<float>(add_dst + batch_row0 + lane, acc + resid);
                }
                batch_row0 = row + 1;
                in_batch = 0;
            }
        } else if (!F::kLaneSums) {
            s = wave_sum_f(s);
            const float resid = add_dst ? residual(row, lane == 0) : 0.0f;
            if (lane == 0) {
                if (plain_y) gstore<float>(y + row, s);
                if (y_lds) y_lds[row] = s;
                if (add_dst) gstore<float>(add_dst + row, s + resid);
            }
        } else {
            // The lanes' sums of up to eight rows are parked in LDS and reduced together: lane L
            // adds eighth L / 8 of row L % 8, then the eighths meet over lanes L ^ 8, ^ 16, ^ 32 -
            // about two instructions per row where a whole-wave reduction per row costs twelve.
            osum[in_batch * LaneSums::kRowStride + lane] = s;
            if (++in_batch == LaneSums::kRows || row + 1 == row_end) {
                const v4f* tr = reinterpret_cast<const v4f*>(osum + (lane & 7) * LaneSums::kRowStride + (lane >> 3) * 8);
                const v4f a = tr[0], b = tr[1];
                float acc = ((a.x + a.y) + (a.z + a.w)) + ((b.x + b.y) + (b.z + b.w));
                acc += __shfl_xor(acc, 8, kWave);
                acc += __shfl_xor(acc, 16, kWave);
                acc += __shfl_xor(acc, 32, kWave);
                const float resid = add_dst ? residual(batch_row0 + lane, lane < in_batch) : 0.0f;
                if (lane < in_batch) {
                    if (plain_y) gstore<float>(y + batch_row0 + lane, acc);
                    if (y_lds) y_lds[batch_row0 + lane] = acc;
                    if (add_dst) gstore<float>(add_dst + batch_row0 + lane, acc + resid);
                }
                batch_row0 = row + 1;
                in_batch = 0;
            }
        }
    };
    if constexpr (STEPS > 1 && F::kRowAhead && STEPS <= RowAheadMaxSteps<F>::value) {
        // Long rows run in eight-wave workgroups, where one step ahead is too few bytes in flight:
        // the loads run a whole row ahead - step t of the next row is requested before step t of
        // this one is computed.
        if (row0 >= row_end) return;
        typename F::Row cur[STEPS];
        cur[0] = first[0];
#pragma unroll
        for (int t = 1; t < STEPS; ++t) {
            if constexpr (FIRST_WHOLE) cur[t] = first[t];
            else F::load_row(cur[t], w + (size_t)row0 * bpr, t, lane, ok[t]);
        }
        for (int row = row0; row < row_end; ++row) {
            const uint8_t* rowp = w + (size_t)row * bpr;
            const bool more = row + 1 < row_end;
            typename F::Row nxt[STEPS];
            float s = 0.0f;
#pragma unroll
            for (int t = 0; t < STEPS; ++t) {
                // unpredicated where the format can: the wave's last row requests itself again
                if constexpr (F::kClampedLoads) F::load_row_clamped(nxt[t], more ? rowp + bpr : rowp, t, lane, ok[t]);
                else F::load_row(nxt[t], rowp + bpr, t, lane, ok[t] && more);
                take_term(t, F::template term<STAGES>(cur[t], acts[t], t, lane, ok[t], st, (size_t)row * n_units), s);
            }
            finish_row(row, s);
#pragma unroll
            for (int t = 0; t < STEPS; ++t) cur[t] = nxt[t];
        }
        return;
    }
    // One row: `cur0` holds its step 0; the loads of step t + 1 are issued before step t is
    // computed, and the last step's prefetch - step 0 of the next row - lands in `next0`.
    auto do_row = [&](int row, const typename F::Row& cur0, typename F::Row& next0) {
        const uint8_t* rowp = w + (size_t)row * bpr;
        float s = 0.0f;
        typename F::Row cur = cur0;
#pragma unroll
        for (int t = 0; t < STEPS; ++t) {
            typename F::Row nxt;
            if (t + 1 < STEPS) F::load_row(nxt, rowp, t + 1, lane, ok[t + 1 < STEPS ? t + 1 : 0]);
            else if (ClampedOneAhead<F>::value)  // the wave's last row prefetches itself again: no predicate
                load_row_clamped<F>(next0, row + 1 < row_end ? rowp + bpr : rowp, lane, ok[0]);
            else F::load_row(next0, rowp + bpr, 0, lane, ok[0] && row + 1 < row_end);
            take_term(t, F::template term<STAGES>(cur, acts[t], t, lane, ok[t], st, (size_t)row * n_units), s);
            if (t + 1 < STEPS) cur = nxt;
        }
        finish_row(row, s);
    };
    typename F::Row cur = first[0];
    int row = row0;
    if constexpr (FIRST_WHOLE && STEPS > 1) {
        if (row < row_end) {  // every step of the first row is here already
            const uint8_t* rowp = w + (size_t)row * bpr;
            if (ClampedOneAhead<F>::value) load_row_clamped<F>(cur, row + 1 < row_end ? rowp + bpr : rowp, lane, ok[0]);
            else F::load_row(cur, rowp + bpr, 0, lane, ok[0] && row + 1 < row_end);
            float s = 0.0f;
#pragma unroll
            for (int t = 0; t < STEPS; ++t)
                take_term(t, F::template term<STAGES>(first[t], acts[t], t, lane, ok[t], st, (size_t)row * n_units), s);
            finish_row(row, s);
            ++row;
        }
    }
    for (; row < row_end; ++row) {
        typename F::Row nxt;
        do_row(row, cur, nxt);
        cur = nxt;
    }
}

// ───────────────────────────── rows streamed through LDS ─────────────────────────────
// A wave's rows [row0, row_end) are one contiguous span of the weight matrix. gemv_rows reads it the
// way the lanes consume it - 16 bytes of a block header here, 32 bytes of nibbles there - so every
// load instruction touches a part of many 128-byte lines and every line is touched by three or more
// instructions. That access pattern must not be non-temporal (a line is dropped after its first
// touch and fetched again: 4.9 TB/s measured), and plain loads stop at 6.2-6.5 TB/s on this device.
// Here the span is instead fetched as it lies in memory: whole lines, 1024 contiguous bytes per load
// instruction, non-temporal (7.1-7.3 TB/s measured for this shape of kernel), in chunks of a few
// instructions into a ring in LDS that belongs to the wave alone; the lanes then pick their block
// pieces out of the ring with the format's load_row_ring. One chunk is in flight in registers while
// the previous one is consumed. No barrier is involved: a wave's LDS operations execute in order.
//
// The image in the ring starts at `origin`, the 128-byte line that holds the span's first byte
// (`head` bytes into it), and ends with the line that holds its last byte (`total` bytes in all):
// bytes outside the span but inside those two lines are fetched and never looked at (a line never
// crosses a page, so they are readable). Ring offsets are image offsets modulo the ring size: a chunk
// is written when less than one wave step of older bytes is still to be consumed, so a ring of a step
// plus a chunk never overwrites bytes that are still wanted.
template <typename F, typename = void>
struct HasRingLoads : std::false_type {};
template <typename F>
struct HasRingLoads<F, std::void_t<decltype(&F::load_row_ring)>> : std::true_type {};
// Ring geometry of a format at a row length of STEPS wave steps.
// kInstr: 1024-byte load instructions per chunk. One-step rows: two and three measured alike (6.74 TB/s
// on 216 Q4_K matrices of 4096 columns) and four 6 % slower at 64 rows per workgroup; two keeps the ring
// smallest (three workgroups per compute unit). Longer rows hold more activation registers and fit two
// workgroups per compute unit, which leaves too few bytes in flight at two instructions: 36 Q4_K
// matrices of 4096 x 12288 ran at 5.61 / 5.72 / 5.82 TB/s with two / three / four; the format says how
// many its ring can afford there (F::kRingLongInstr: two workgroups must still fit the LDS).
// kBytes: a chunk is written only when less than one wave step of older bytes is still to be consumed,
// so a step plus a chunk always fit. The lanes' pieces must be 16-byte aligned in the row (Q4_K's and
// Q5_K's are): a ring of whole pieces then never splits one at its end. Q6_K's pieces sit at any even
// offset; a form that kept a second copy of the ring's first 16 bytes behind its end and read the
// pieces with misaligned 16-byte LDS loads gave the right bits and ran 7-9 % slower than the direct
// loads (5.28 against 5.67 TB/s at 4096 x 4096), and is not kept.
template <typename F, int STEPS>
struct WeightRingOf {
    static constexpr int kInstr = STEPS == 1 ? 2 : F::kRingLongInstr;
    static constexpr uint32_t kChunk = kInstr * 1024;
    static constexpr uint32_t kBytes = F::kStepBytes + kChunk;
    static_assert(kBytes % 16 == 0, "chunk pieces are 16 bytes");
};
// The ring of a row of `steps` wave steps, for host code that sizes LDS by the step count.
template <typename F>
inline size_t ring_alloc_bytes(int steps) {
    return steps == 1 ? WeightRingOf<F, 1>::kBytes : WeightRingOf<F, 2>::kBytes;
}
// (kInstr for a kernel that may be instantiated for formats without ring loads)
template <typename F, int STEPS, bool STREAMED>
constexpr int ring_instr() {
    if constexpr (STREAMED) return WeightRingOf<F, STEPS>::kInstr;
    else return 1;
}
template <int INSTR>
struct RingChunk {
    v4i v[INSTR];
};

// Chunk `c` of the image: lane l takes bytes [16 l, 16 l + 16) of each of its 1024-byte pieces.
// Pieces past the image's end read its last piece again instead of being masked off (total >= 128):
// with every load unconditional the compiler can count how many are in flight and wait for the
// oldest chunk alone; behind a per-lane branch it waits for all of them.
template <int INSTR>
__device__ __forceinline__ void ring_issue(const uint8_t* origin, uint32_t c, uint32_t total, int lane, v4i (&v)[INSTR]) {
#pragma unroll
    for (int k = 0; k < INSTR; ++k) {
        const uint32_t o = c * (INSTR * 1024) + k * 1024 + lane * 16;
        v[k] = gload_stream<v4i>(origin + (o < total ? o : total - 16));
    }
}
// gemv_rows for an ordered format with load_row_ring, fed from the ring. `rc` holds chunk 0 of the
// image (the caller requests it ahead of its prologue). A chunk's registers are written to the ring
// and at once reloaded with the next chunk, which is then in flight while the rows that the ring now
// holds are computed (a second register set would have to be copied into the first, and a copy
// waits for the load it reads). row0, row_end, head and total must be wave-uniform scalars.
// Every output equals gemv_rows' bit for bit: the per-block terms and the order in which they are
// added are the same code.
template <typename F, int STEPS, bool STAGES>
__device__ __forceinline__ void gemv_rows_streamed(const uint8_t* origin, uint32_t head, uint32_t total, size_t bpr,
                                                   RingChunk<WeightRingOf<F, STEPS>::kInstr>& rc, uint8_t* ring,
                                                   const typename F::Acts (&acts)[STEPS], const bool (&ok)[STEPS],
                                                   float* __restrict__ y, int n_units, int row0, int row_end,
                                                   int lane, const StagePtrs& st, float* osum,
                                                   float* add_dst = nullptr, float add_first = 0.0f,
                                                   float* y_lds = nullptr) {
    static_assert(F::kOrdered, "the streamed loop adds per-block terms in block order");
    // (a wave has at most 64 rows here: every residual is among the lanes' prefetched values, and
    // the loop holds no load but the chunks' - one more would be waited for together with them)
    auto residual = [&](int r) { return __shfl(add_first, (r - row0) & 63, kWave); };
    const bool plain_y = y != add_dst;
    constexpr int LS = OrderedSum<STEPS>::kRowStride;
    constexpr uint32_t kRing = WeightRingOf<F, STEPS>::kBytes;
    constexpr int kInstr = WeightRingOf<F, STEPS>::kInstr;
    constexpr uint32_t kChunk = WeightRingOf<F, STEPS>::kChunk;
    uint32_t chunks = 0;  // chunks of the image written to the ring so far
    uint32_t wpos = 0;    // ring position of the next chunk (image offset modulo the ring size)
    auto advance = [&]() {
#pragma unroll
        for (int k = 0; k < kInstr; ++k) {
            uint32_t o = wpos + k * 1024 + lane * 16;
            o = o >= kRing ? o - kRing : o;
            *reinterpret_cast<v4i*>(ring + o) = rc.v[k];
        }
        ++chunks;
        ring_issue(origin, chunks, total, lane, rc.v);
        wpos += kChunk;
        wpos = wpos >= kRing ? wpos - kRing : wpos;
    };
    int in_batch = 0, batch_row0 = row0;
    uint32_t rpos = head;  // ring position of the current row's first byte
    for (int row = row0; row < row_end; ++row) {
        const uint32_t roff = head + (uint32_t)(row - row0) * (uint32_t)bpr;
#pragma unroll
        for (int t = 0; t < STEPS; ++t) {
            const uint32_t step_end = (uint32_t)(t + 1) * F::kStepBytes < (uint32_t)bpr ? (uint32_t)(t + 1) * F::kStepBytes : (uint32_t)bpr;
            while (chunks * kChunk < roff + step_end) advance();
            typename F::Row r;
            uint32_t spos = rpos + (uint32_t)t * (F::kStepBytes % kRing);
            while (spos >= kRing) spos -= kRing;
            F::load_row_ring(r, ring, spos, kRing, lane, ok[t]);
            const float term = F::template term<STAGES>(r, acts[t], t, lane, ok[t], st, (size_t)row * n_units);
            if ((lane & 3) == 0) osum[in_batch * LS + t * 16 + (lane >> 2)] = term;
        }
        rpos += (uint32_t)(bpr % kRing);
        rpos = rpos >= kRing ? rpos - kRing : rpos;
        if (++in_batch == 16 || row + 1 == row_end) {
            const float resid = add_dst ? residual(batch_row0 + lane) : 0.0f;
            if (lane < in_batch) {
                const v4f* tr = reinterpret_cast<const v4f*>(osum + lane * LS);
                float acc = 0.0f;
#pragma unroll
                for (int k = 0; k < 4 * STEPS; ++k) {
                    const v4f v = tr[k];
                    acc += v.x;
                    acc += v.y;
                    acc += v.z;
                    acc += v.w;
                }
                if (plain_y) gstore<float>(y + batch_row0 + lane, acc);
                if (y_lds) y_lds[batch_row0 + lane] = acc;
                if (add_dst) gstore<float>(add_dst + batch_row0 + lane, acc + resid);
            }
            batch_row0 = row + 1;
            in_batch = 0;
        }
    }
}

// Folded form for short rows of the 16-blocks-per-step formats (Q4_K, Q6_K) with nb <= 8 blocks
// per row: consecutive weight rows are contiguous in memory, so one wave step takes
// rps = 16 / nb whole rows at once (block slot q = lane / 4 -> row q / nb, block q % nb) instead of
// leaving the lanes past the row's end idle. `acts` must hold activation block q % nb for this
// lane. Per-(row, block) terms are the same code as the unfolded loop and are added per row in
// ascending block order, so every output equals the unfolded result bit for bit.
// `osum` is this wave's OrderedSum<1> scratch.
// Y_GLOBAL = false: `y` is not device memory (a caller's LDS row); `first`, when given, is the
// step at row0, requested by the caller ahead of its own prologue.
template <typename F, bool Y_GLOBAL = true>
__device__ __forceinline__ void gemv_rows_folded(const uint8_t* __restrict__ w, size_t bpr, int nb,
                                                 const typename F::Acts& acts,
                                                 float* __restrict__ y, int row0, int row_end,
                                                 int lane, float* osum, const typename F::Row* first = nullptr) {
    static_assert(F::kOrdered, "folded rows exist for the ordered 16-block formats");
    constexpr int LS = OrderedSum<1>::kRowStride;
    const int q = lane >> 2, rps = 16 / nb;
    const int rq = q / nb, bq = q - rq * nb;
    const bool lane_ok = rq < rps;
    // columns nb..15 of a scratch row are never written: zero them once so the flush can add all 16
    for (int i = lane; i < OrderedSum<1>::kFloatsPerWave; i += 64) osum[i] = 0.0f;
    typename F::Row cur;
    if (first) cur = *first;
    else F::load_row(cur, w + (size_t)row0 * bpr, 0, lane, lane_ok && row0 + rq < row_end);
    int in_batch = 0, batch_row0 = row0;
    for (int row = row0; row < row_end; row += rps) {
        const int nr = row + rps;
        typename F::Row nxt;
        F::load_row(nxt, w + (size_t)nr * bpr, 0, lane, lane_ok && nr + rq < row_end);
        const bool ok = lane_ok && row + rq < row_end;
        const float term = F::template term<false>(cur, acts, 0, lane, ok, StagePtrs{nullptr, nullptr}, 0);
        if ((lane & 3) == 0 && lane_ok) osum[(in_batch + rq) * LS + bq] = ok ? term : 0.0f;
        in_batch += rps;
        cur = nxt;
        if (in_batch + rps > 16 || nr >= row_end) {
            if (lane < in_batch && batch_row0 + lane < row_end) {
                const v4f* tr = reinterpret_cast<const v4f*>(osum + lane * LS);
                float acc = 0.0f;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const v4f v = tr[k];
                    acc += v.x;
                    acc += v.y;
                    acc += v.z;
                    acc += v.w;
                }
                if (Y_GLOBAL) gstore<float>(y + batch_row0 + lane, acc);
                else y[batch_row0 + lane] = acc;
            }
            batch_row0 = nr;
            in_batch = 0;
        }
    }
}

// Small-batch form: MB activation rows against each weight row, so the weights stream once for
// up to eight tokens. Every (weight row, activation) pair runs the same per-block code and the
// same ordered sum as the single-activation loop, so each output equals the m == 1 result bit
// for bit (the CPU's batch kernels have the same property, kernels.rs:9297-9405).
template <typename F, int STEPS, int MB, bool STAGES>
__device__ __forceinline__ void gemv_rows_batch(const uint8_t* __restrict__ w, size_t bpr,
                                                const typename F::Row& first,
                                                const typename F::Acts (&acts)[MB][STEPS],
                                                const bool (&ok)[STEPS], float* y,
                                                size_t y_stride, int m_valid, int n_units, int row0,
                                                int row_end, int lane, const StagePtrs& st,
                                                size_t st_stride, float* osum, const BatchAdd& add = BatchAdd{}) {
    constexpr int LS = OrderedSum<STEPS>::kRowStride;
    constexpr int RB = 16 / MB;  // weight rows per ordered-sum flush
    typename F::Row cur = first;
    int in_batch = 0, batch_row0 = row0;
    for (int row = row0; row < row_end; ++row) {
        const uint8_t* rowp = w + (size_t)row * bpr;
        float s[MB];
#pragma unroll
        for (int mi = 0; mi < MB; ++mi) s[mi] = 0.0f;
#pragma unroll
        for (int t = 0; t < STEPS; ++t) {
            typename F::Row nxt;
            if (t + 1 < STEPS) F::load_row(nxt, rowp, t + 1, lane, ok[t + 1 < STEPS ? t + 1 : 0]);
            else F::load_row(nxt, rowp + bpr, 0, lane, ok[0] && row + 1 < row_end);
#pragma unroll
            for (int mi = 0; mi < MB; ++mi) {
                const StagePtrs sm{STAGES ? st.a + mi * st_stride : nullptr,
                                   STAGES && st.b ? st.b + mi * st_stride : nullptr};
                const float term = term_shared<F, STAGES>(cur, acts[mi][t], t, lane,
                                                            ok[t] && mi < m_valid, sm,
                                                            (size_t)row * n_units);
                if (F::kOrdered) {
                    if ((lane & 3) == 0) osum[(in_batch * MB + mi) * LS + t * 16 + (lane >> 2)] = term;
                } else {
                    s[mi] += term;
                }
            }
            cur = nxt;
        }
        if (F::kOrdered) {
            if (++in_batch == RB || row + 1 == row_end) {
                if (lane < in_batch * MB) {
                    const v4f* tr = reinterpret_cast<const v4f*>(osum + lane * LS);
                    float acc = 0.0f;
#pragma unroll
                    for (int k = 0; k < 4 * STEPS; ++k) {
                        const v4f v = tr[k];
                        acc += v.x;
                        acc += v.y;
                        acc += v.z;
                        acc += v.w;
                    }
                    const int mi = lane % MB;
                    if (mi < m_valid) store_batch_out(y, add, (size_t)mi * y_stride + batch_row0 + lane / MB, acc);
                }
                batch_row0 = row + 1;
                in_batch = 0;
            }
        } else {
            if constexpr (MB == 2 || MB == 4 || MB == 8) {
                // the MB tokens' lane sums reduced together: lane L carries token L % MB summed over
                // its row of 16 lanes; two cross-row exchanges finish it
                float part = row16_transpose_sum<MB>(s, lane);
                part += __shfl_xor(part, 16, kWave);
                part += __shfl_xor(part, 32, kWave);
                if (lane < MB && lane < m_valid) store_batch_out(y, add, (size_t)lane * y_stride + row, part);
            } else {
#pragma unroll
                for (int mi = 0; mi < MB; ++mi) {
                    const float tot = wave_sum_f(s[mi]);
                    if (lane == 0 && mi < m_valid) store_batch_out(y, add, (size_t)mi * y_stride + row, tot);
                }
            }
        }
    }
}

}  // namespace infr
