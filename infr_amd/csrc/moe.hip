// Op::MoeFfn on the device. Mirrors infr-cpu's staged pipeline (crates/infr-cpu/src/lib.rs:2264-2984,
// crates/infr-cpu/src/moe.rs); the list below is qwen3moe's setting (softmax gating, renormalised
// top-k, split gate/up banks, SiLU, weights on the expert outputs), the op's other fields - gating
// function, selection bias, group-limited routing, supplied expert ids, activation and clamp, the
// weight on the expert input, fused gate|up banks, per-expert down scale - are MoeRoute / MoeAct below:
//
//   router   f32 router rows . router_x with infr-cpu's `dot` (8 FMA accumulators by index mod 8,
//            summed in order, kernels.rs:6557-6573), evaluated in that exact order so the logits -
//            and with them the expert selection - match the CPU bit for bit
//   select   softmax with max-subtraction, probabilities summed in index order, stable top-n_used
//            (ties to the lower expert index), w = p / max(sum_sel p, 1e-20) * scale  (lib.rs:2421-2543)
//   rows == 1   the CPU multiplies DECODED f32 weights with the UNQUANTIZED activation
//            (ActsKind::Raw, moe.rs:42-53,142-173): gate/up rows of Q4_K / Q6_K / Q8_0 banks are
//            applied to f32 x in registers (sc * sum(code*x) + mn * sum(x) per scale group, all
//            f32), SiLU fused; the down kernel does likewise and adds the experts in rank order
//   rows >= 2   int8 path: x rows quantized per 256 once, id-gathered Q4_K/Q6_K/Q8_0 GEMVs per
//            (row, expert) pair (the decode GEMV body, bit-identical to the CPU's batch kernels),
//            SiLU + re-quantization, id-gathered down GEMV, rank-ordered accumulate
// Only the selected experts' blocks are addressed: every weight pointer is
// bank + ids[slot] * expert_stride, read on the device.
#include <algorithm>

#include "gemv_formats.hpp"
#include "gemv_rows.hpp"
#include "kernels.hpp"
#include "decode_element.hpp"
#include "elementwise_fn.hpp"
#include "quant_chunk.hpp"

namespace infr {

// ───────────────────────────── router + selection ─────────────────────────────

// LDS of one selection: probabilities, the values the selection ranks (the probabilities plus an
// optional bias, masked by group), their ranks, the ranked winners with their weights, reduction slots.
struct SelectLds {
    float p[1024];
    float sv[1024];
    int rank[1024];
    float top_p[64];
    float top_w[64];
    int top_e[64];
    float gscore[64];
    int gkeep[64];
    float red[8];
};

// Quad-major activation rows, [quad][unit][4]: unit = the 64 weights of a row that one lane of the
// one-token expert kernels owns, quad q = the floats in its registers 4q .. 4q+3, so consecutive
// lanes read consecutive 16 bytes. Unit and quad of the quad that starts at element e (a multiple
// of 4): 64 consecutive elements per unit for Q4_K, Q5_K and Q8_0; for Q6_K a unit is four groups
// of 16, 32 apart, of one half of a 256-block (the decode GEMV's mapping).
__device__ __forceinline__ void quad_place_linear(int e, int& u, int& q) {
    u = e >> 6;
    q = (e & 63) >> 2;
}
__device__ __forceinline__ void quad_place_q6k(int e, int& u, int& q) {
    const int r = e & 255, r2 = r & 127, r3 = r2 & 31;
    u = (e >> 8) * 4 + (r >> 7) * 2 + (r3 >> 4);
    q = 4 * (r2 >> 5) + ((r3 & 15) >> 2);
}

// Gating probabilities, selection and weights of one row (lib.rs:2421-2543), run by a whole
// 256-thread workgroup. n_expert <= 1024, n_used <= 64, at most 64 groups.
//   probabilities  softmax with max-subtraction, summed in index order by one thread; or a per-expert
//                  sigmoid; or sqrt(softplus) with the CPU's v > 20 shortcut
//   selection      on a copy: + bias (exp_probs_b), then group-limited routing - a group's score is the
//                  sum of its two best values, the best `n_groups_used` groups (ties to the lower group)
//                  keep their values, the others become -inf - then the stable descending sort,
//                  realised by counting rank(e) = #{j : v[j] > v[e] or (v[j] == v[e] and j < e)} (for
//                  softmax on the NORMALISED probabilities: normalising can create ties that the raw
//                  exponentials do not have). Supplied ids replace all of it, in their own order.
//   weights        from the unbiased probabilities, summed in rank order:
//                  norm_w ? p / max(sum, 1e-20) * scale : p * scale
// Leaves s.top_e / s.top_p / s.top_w (all threads may read them on return) and stores the ranked
// experts and weights when out_idx is given.
// COHERENT: the logits were written by other workgroups of the same launch (with device-scope
// stores) and are read past this compute unit's and this die's caches.
template <bool COHERENT = false>
__device__ __forceinline__ void moe_select_block(const float* __restrict__ l, SelectLds& s,
                                                 int n_expert, int n_used, float scale, int tid,
                                                 int32_t* __restrict__ out_idx,
                                                 float* __restrict__ out_w, const MoeRoute& rt, size_t row) {
    const int lane = tid & 63, wave = tid >> 6;
    float lv[4];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int e = tid + 256 * i;
        lv[i] = e >= n_expert ? -INFINITY
                : COHERENT   ? __hip_atomic_load(l + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                             : l[e];
        mx = __builtin_fmaxf(mx, lv[i]);
    }
    if (rt.gating == 0) {
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) mx = __builtin_fmaxf(mx, __shfl_xor(mx, off, kWave));
        if (lane == 0) s.red[wave] = mx;
        __syncthreads();
        mx = __builtin_fmaxf(__builtin_fmaxf(s.red[0], s.red[1]), __builtin_fmaxf(s.red[2], s.red[3]));
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int e = tid + 256 * i;
            if (e < n_expert) {
                lv[i] = expf(lv[i] - mx);
                s.p[e] = lv[i];
                s.rank[e] = 0;
            }
        }
        __syncthreads();
        if (tid == 0) {  // `p.iter().sum()`: index order; 32 LDS values per wait
            float sum = 0.0f;
            int e = 0;
            for (; e + 32 <= n_expert; e += 32) {
                v4f q[8];
#pragma unroll
                for (int k = 0; k < 8; ++k) q[k] = *reinterpret_cast<const v4f*>(s.p + e + 4 * k);
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    sum += q[k].x; sum += q[k].y; sum += q[k].z; sum += q[k].w;
                }
            }
            for (; e < n_expert; ++e) sum += s.p[e];
            s.red[4] = sum;
        }
        __syncthreads();
        const float psum = s.red[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int e = tid + 256 * i;
            if (e < n_expert) s.p[e] = lv[i] / psum;
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int e = tid + 256 * i;
            if (e < n_expert) {
                const float v = lv[i];
                s.p[e] = rt.gating == 1 ? 1.0f / (1.0f + expf(-v)) : sqrtf(v > 20.0f ? v : logf(1.0f + expf(v)));
                s.rank[e] = 0;
            }
        }
    }
    __syncthreads();
    if (rt.ids) {  // the selection is given; the weights still come from the probabilities
        if (tid < n_used) {
            const int e = min(max(rt.ids[row * n_used + tid], 0), n_expert - 1);
            s.top_e[tid] = e;
            s.top_p[tid] = s.p[e];
        }
    } else {
        const float* v = s.p;  // what the selection ranks
        const bool grouped = rt.n_groups > 1 && rt.n_groups_used > 0;
        if (rt.bias || grouped) {
            for (int e = tid; e < n_expert; e += 256) s.sv[e] = rt.bias ? s.p[e] + rt.bias[e] : s.p[e];
            __syncthreads();
            if (grouped) {
                const int per = n_expert / rt.n_groups;
                if (tid < rt.n_groups) {
                    float b0 = -INFINITY, b1 = -INFINITY;
                    for (int i = 0; i < per; ++i) {
                        const float x = s.sv[tid * per + i];
                        if (x > b0) { b1 = b0; b0 = x; } else if (x > b1) { b1 = x; }
                    }
                    s.gscore[tid] = b0 + b1;
                }
                __syncthreads();
                if (tid < rt.n_groups) {
                    const float g = s.gscore[tid];
                    int cnt = 0;
                    for (int j = 0; j < rt.n_groups; ++j) {
                        const float q = s.gscore[j];
                        cnt += (q > g ? 1 : 0) + ((q == g && j < tid) ? 1 : 0);
                    }
                    s.gkeep[tid] = cnt < rt.n_groups_used;
                }
                __syncthreads();
                for (int e = tid; e < n_expert; e += 256)
                    if (!s.gkeep[e / per]) s.sv[e] = -INFINITY;
                __syncthreads();
            }
            v = s.sv;
        }
        // rank by counting: `parts` threads share an expert when n_expert < 256
        const int parts = n_expert <= 128 ? 256 / n_expert : 1;
        const int span = ((n_expert + parts - 1) / parts + 3) & ~3;
        for (int item = tid; item < n_expert * parts; item += 256) {
            const int e = item % n_expert, part = item / n_expert;
            const float ve = v[e];
            const int j0 = part * span, j1 = min(n_expert, j0 + span);
            int cnt = 0, j = j0;
            for (; j + 4 <= j1; j += 4) {
                const v4f q = *reinterpret_cast<const v4f*>(v + j);
                cnt += (q.x > ve ? 1 : 0) + ((q.x == ve && j + 0 < e) ? 1 : 0);
                cnt += (q.y > ve ? 1 : 0) + ((q.y == ve && j + 1 < e) ? 1 : 0);
                cnt += (q.z > ve ? 1 : 0) + ((q.z == ve && j + 2 < e) ? 1 : 0);
                cnt += (q.w > ve ? 1 : 0) + ((q.w == ve && j + 3 < e) ? 1 : 0);
            }
            for (; j < j1; ++j) {
                const float q = v[j];
                cnt += (q > ve ? 1 : 0) + ((q == ve && j < e) ? 1 : 0);
            }
            if (parts > 1) atomicAdd(&s.rank[e], cnt);
            else s.rank[e] = cnt;
        }
        __syncthreads();
        for (int e = tid; e < n_expert; e += 256) {
            const int r = s.rank[e];
            if (r < n_used) {
                s.top_e[r] = e;
                s.top_p[r] = s.p[e];
            }
        }
    }
    __syncthreads();
    if (tid < n_used) {
        float wsum = 0.0f;  // summed in rank order, as the CPU sums its selection
        for (int k = 0; k < n_used; ++k) wsum += s.top_p[k];
        wsum = __builtin_fmaxf(wsum, 1e-20f);
        const float w = rt.norm_w ? s.top_p[tid] / wsum * scale : s.top_p[tid] * scale;
        s.top_w[tid] = w;
        if (out_idx) {
            out_idx[tid] = s.top_e[tid];
            out_w[tid] = w;
        }
    }
    __syncthreads();
}

// One workgroup per row (used when there are several rows; a single row is selected by the
// router kernel itself).
// When x is given, the workgroup first quantizes its row of the expert input (per-256 `Q8`, the
// layout of quantize_q8_kernel; ne a multiple of 256): one launch less in front of the expert GEMVs.
__global__ __launch_bounds__(256) void moe_select_kernel(const float* __restrict__ logits,
                                                         int32_t* __restrict__ sel_idx,
                                                         float* __restrict__ sel_w, int n_expert,
                                                         int n_used, float scale,
                                                         const float* __restrict__ x, int ne,
                                                         int8_t* __restrict__ qs, float* __restrict__ qd,
                                                         int32_t* __restrict__ bsums,
                                                         int32_t* __restrict__ bsums16, MoeRoute rt) {
    __shared__ __attribute__((aligned(16))) SelectLds s;
    const size_t r = blockIdx.x;
    if (x) {
        const int lane = threadIdx.x & 63, nchunk = ne / 256;
        for (int c = threadIdx.x >> 6; c < nchunk; c += 4) {  // wave-uniform
            const size_t chunk = r * nchunk + c;
            const v4f v = *reinterpret_cast<const v4f*>(x + chunk * 256 + (size_t)lane * 4);
            quantize_chunk<false>(v, true, lane, chunk, qs, qd, bsums, bsums16);
        }
    }
    moe_select_block(logits + r * n_expert, s, n_expert, n_used, scale, threadIdx.x, sel_idx + r * n_used,
                     sel_w + r * n_used, rt, r);
}

// infr-cpu's `dot` keeps 8 FMA accumulators (element i goes to accumulator i mod 8) and adds them
// in order; each accumulator is a strictly sequential chain, so the order cannot be parallelised
// beyond the 8 accumulators without changing the rounding. A workgroup takes `epw` expert rows
// (1, 4 or 8) and 32 / epw activation rows: all 256 threads stage K-chunks of them into LDS with
// coalesced 16-byte loads, and eight lanes per (expert, token) pair - one accumulator each - run
// the chains from LDS, carrying them across chunks. A row sits in LDS accumulator-major (element i
// at [i % 8][i / 8]), so a lane reads four steps of its chain with one 16-byte access.
// A single row of banks in the factored kernels' formats leaves only logits here (one expert per
// workgroup; the gate / up kernel selects in its prologue). For any other single row (tickets !=
// nullptr) the last workgroup to finish - a ticket counter, left at zero again - runs the
// selection too, which saves a launch; eight experts per workgroup keep that to a handful of
// tickets (atomics on one address complete one after another, ~65 ns each).
// ne % 32 == 0 is required.
// Four consecutive elements of a plain row of f32 (WT 0), f16 (1) or bf16 (30) as f32, widened
// exactly (crates/infr-gguf/src/dequant.rs:13-22): what dot / dot_f16 / dot_bf16 multiply
// (crates/infr-cpu/src/kernels.rs:6505-6573).
template <int WT>
__device__ __forceinline__ v4f row_load4(const void* row, size_t elem) {
    if constexpr (WT == 0) {
        return *reinterpret_cast<const v4f*>(static_cast<const float*>(row) + elem);
    } else {
        const v2i raw = *reinterpret_cast<const v2i*>(static_cast<const uint16_t*>(row) + elem);
        const uint32_t lo = (uint32_t)raw.x, hi = (uint32_t)raw.y;
        if constexpr (WT == 1)
            return v4f{f16_bits_to_f32(lo & 0xFFFFu), f16_bits_to_f32(lo >> 16), f16_bits_to_f32(hi & 0xFFFFu),
                       f16_bits_to_f32(hi >> 16)};
        else
            return v4f{__builtin_bit_cast(float, lo << 16), __builtin_bit_cast(float, lo & 0xFFFF0000u),
                       __builtin_bit_cast(float, hi << 16), __builtin_bit_cast(float, hi & 0xFFFF0000u)};
    }
}
template <int WT>
__host__ __device__ constexpr size_t row_elem_bytes() { return WT == 0 ? 4 : 2; }

constexpr int kRouterPairs = 32, kRouterChunk = 512;
// floats between two staged rows of kc elements: eight accumulator rows of kc / 8 + 4
__host__ __device__ constexpr int router_row_floats(int kc) { return 8 * (kc / 8 + 4); }

// NL: 16-byte loads a thread has in flight while staging (24 at a single row: the nine rows of a
// workgroup arrive in one round trip)
template <int NL, int WT = 0>
__global__ __launch_bounds__(256) void moe_router_kernel(
    const void* __restrict__ router, const float* __restrict__ rx, float* __restrict__ logits,
    int* __restrict__ tickets, int32_t* __restrict__ sel_idx, float* __restrict__ sel_w, int ne,
    int n_expert, int rows, int n_used, float scale, int kc, int epw, int tpw, const float* __restrict__ norm_w,
    float* __restrict__ norm_dst, float norm_eps, float* __restrict__ xt, int xt_q6k, MoeRoute rt) {
    extern __shared__ __attribute__((aligned(16))) float rl[];  // [epw] rows | [32 / epw] rows
    __shared__ __attribute__((aligned(16))) SelectLds sel;
    __shared__ int s_last;
    const int tid = threadIdx.x;
    // An absorbed RmsNorm of the single activation row: the scale with rms_norm_kernel's own
    // reduction (stride-256 partial sums, wave sums, ((p0 + p1) + (p2 + p3))), applied while the
    // row is staged; the first workgroup stores the normalised row for the expert kernels.
    float nscale = 1.0f;
    if (norm_w) {
        float s = 0.0f;
        for (int i = tid; i < ne; i += 256) s += rx[i] * rx[i];
        s = wave_sum_f(s);
        if ((tid & 63) == 0) sel.red[tid >> 6] = s;
        __syncthreads();
        const float ss = ((sel.red[0] + sel.red[1]) + (sel.red[2] + sel.red[3])) / (float)ne;
        nscale = 1.0f / sqrtf(ss + norm_eps);
    }
    const int e0 = blockIdx.x * epw, t0 = blockIdx.y * tpw;
    const int n_e = min(epw, n_expert - e0), n_t = min(tpw, rows - t0);
    const int ld = router_row_floats(kc), la = kc / 8 + 4;  // row and accumulator-row strides
    float* lw = rl;
    float* lx = rl + epw * ld;
    const int pair = tid >> 3, j = tid & 7;
    const int e = pair % epw, t = pair / epw;
    const bool active = e < n_e && t < n_t;
    float acc = 0.0f;  // accumulator j
    for (int k0 = 0; k0 < ne; k0 += kc) {
        const int n = min(kc, ne - k0), n4 = n / 4;
        const int total = (n_e + n_t) * n4;
        if (k0) __syncthreads();
        for (int base = 0; base < total; base += 256 * NL) {  // NL loads in flight per thread
            v4f tmp[NL];
            float* dst[NL];
#pragma unroll
            for (int u = 0; u < NL; ++u) {
                const int i = base + u * 256 + tid;
                const int row = i / n4, q = i % n4;
                // elements 4q .. 4q+3 are accumulators 4(q & 1) .. +3 at step q / 2
                dst[u] = (row < n_e ? lw + row * ld : lx + (row - n_e) * ld) + 4 * (q & 1) * la + (q >> 1);
                if (i < total) {
                    if (row < n_e)
                        tmp[u] = row_load4<WT>(static_cast<const uint8_t*>(router) + (size_t)(e0 + row) * ne * row_elem_bytes<WT>(),
                                               (size_t)k0 + 4 * q);
                    else
                        tmp[u] = reinterpret_cast<const v4f*>(rx + (size_t)(t0 + row - n_e) * ne + k0)[q];
                    if (norm_w && row >= n_e) {
                        const v4f wv = reinterpret_cast<const v4f*>(norm_w + k0)[q];
                        tmp[u] = v4f{tmp[u].x * nscale * wv.x, tmp[u].y * nscale * wv.y, tmp[u].z * nscale * wv.z,
                                     tmp[u].w * nscale * wv.w};
                        if (norm_dst && blockIdx.x == 0) reinterpret_cast<v4f*>(norm_dst + k0)[q] = tmp[u];
                    }
                    // a single row for the one-token expert kernels: the first workgroup leaves it
                    // quad-major, [quad][unit][4] of the gate / up format's lane mapping
                    if (xt && row >= n_e && blockIdx.x == 0) {
                        int xu, xq;
                        if (xt_q6k) quad_place_q6k(k0 + 4 * q, xu, xq);
                        else quad_place_linear(k0 + 4 * q, xu, xq);
                        *reinterpret_cast<v4f*>(xt + ((size_t)xq * (ne / 64) + xu) * 4) = tmp[u];
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < NL; ++u)
                if (base + u * 256 + tid < total) {
                    dst[u][0] = tmp[u].x;
                    dst[u][la] = tmp[u].y;
                    dst[u][2 * la] = tmp[u].z;
                    dst[u][3 * la] = tmp[u].w;
                }
        }
        __syncthreads();
        if (active) {
            const v4f* a = reinterpret_cast<const v4f*>(lw + e * ld + j * la);
            const v4f* xx = reinterpret_cast<const v4f*>(lx + t * ld + j * la);
#pragma unroll 8
            for (int c = 0; c < n / 32; ++c) {
                const v4f av = a[c], xv = xx[c];
                acc = __builtin_fmaf(av.x, xv.x, acc);
                acc = __builtin_fmaf(av.y, xv.y, acc);
                acc = __builtin_fmaf(av.z, xv.z, acc);
                acc = __builtin_fmaf(av.w, xv.w, acc);
            }
        }
    }
    // s = acc[0] + acc[1] + ... + acc[7] in order
    float sum = 0.0f;
#pragma unroll
    for (int q = 0; q < 8; ++q) sum += __shfl(acc, (tid & ~7) + q, kWave);
    if (!tickets) {
        if (active && j == 0) logits[(size_t)(t0 + t) * n_expert + e0 + e] = sum;
        return;
    }
    // ticket: the workgroup that sees every other one done selects. The logits go to memory with
    // device-scope stores and come back with device-scope loads, and each thread waits for its
    // store before the barrier in front of the ticket: a device-wide fence pair instead (write
    // back and invalidate the whole L2 of the die) costs several microseconds per workgroup.
    if (active && j == 0)
        __hip_atomic_store(logits + (size_t)(t0 + t) * n_expert + e0 + e, sum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) s_last = atomicAdd(tickets, 1) == (int)gridDim.x - 1;
    __syncthreads();
    if (!s_last) return;
    moe_select_block<true>(logits, sel, n_expert, n_used, scale, tid, sel_idx, sel_w, rt, 0);
    if (tid == 0) *tickets = 0;
}

// Prefill form of the router (rows >= kRtMinRows): the same eight accumulator chains per
// (expert, token) dot, register-tiled so that LDS is read half a word per FMA instead of two. A
// workgroup of two wavefronts takes 16 experts x 16 tokens; its 16 groups of eight lanes each own
// a 4 x 4 tile of pairs - experts eg + 4i, tokens tg + 4i, so that the lanes of a wavefront read 32
// distinct banks - and lane j of a group carries accumulator j of all 16 pairs. The next K-chunk
// is fetched into registers while the current one is multiplied.
constexpr int kRtE = 16, kRtT = 16, kRtK = 256, kRtThreads = 128, kRtMinRows = 256;
constexpr int kRtLoads = (kRtE + kRtT) * (kRtK / 4) / kRtThreads;  // 16-byte loads per thread and chunk

template <int WT = 0>
__global__ __launch_bounds__(kRtThreads) void moe_router_tile_kernel(const void* __restrict__ router,
                                                                     const float* __restrict__ rx,
                                                                     float* __restrict__ logits, int ne,
                                                                     int n_expert, int rows) {
    __shared__ __attribute__((aligned(16))) float lrow[kRtE + kRtT][kRtK + 8];  // experts, then tokens
    const int tid = threadIdx.x, j = tid & 7, tile = tid >> 3;
    const int eg = tile & 3, tg = tile >> 2;
    const int e0 = blockIdx.x * kRtE, t0 = blockIdx.y * kRtT;
    // this thread's pieces of a chunk: row (i * kRtThreads + tid) / 64, float4 column % 64;
    // rows past the last expert / token repeat it (computed, never stored)
    const void* src[kRtLoads];  // the row each piece comes from: a weight row (WT) or an activation row (f32)
#pragma unroll
    for (int i = 0; i < kRtLoads; ++i) {
        const int idx = i * kRtThreads + tid, row = idx / (kRtK / 4);
        src[i] = row < kRtE ? static_cast<const void*>(static_cast<const uint8_t*>(router) +
                                                       (size_t)min(e0 + row, n_expert - 1) * ne * row_elem_bytes<WT>())
                            : static_cast<const void*>(rx + (size_t)min(t0 + row - kRtE, rows - 1) * ne);
    }
    v4f stage[kRtLoads];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < kRtLoads; ++i) {
            const int idx = i * kRtThreads + tid, row = idx / (kRtK / 4), q = idx % (kRtK / 4);
            if (k0 + 4 * q >= ne) stage[i] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
            else if (row < kRtE) stage[i] = row_load4<WT>(src[i], (size_t)k0 + 4 * q);
            else stage[i] = row_load4<0>(src[i], (size_t)k0 + 4 * q);
        }
    };
    float acc[4][4];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b) acc[a][b] = 0.0f;
    fetch(0);
    for (int k0 = 0; k0 < ne; k0 += kRtK) {
        const int n = min(kRtK, ne - k0);
        if (k0) __syncthreads();  // the previous chunk's readers are done
#pragma unroll
        for (int i = 0; i < kRtLoads; ++i) {
            const int idx = i * kRtThreads + tid;
            reinterpret_cast<v4f*>(&lrow[idx / (kRtK / 4)][0])[idx % (kRtK / 4)] = stage[i];
        }
        __syncthreads();
        if (k0 + kRtK < ne) fetch(k0 + kRtK);
#pragma unroll 4
        for (int c = 0; c < n / 8; ++c) {
            float a[4], x[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                a[i] = lrow[eg + 4 * i][c * 8 + j];
                x[i] = lrow[kRtE + tg + 4 * i][c * 8 + j];
            }
#pragma unroll
            for (int ie = 0; ie < 4; ++ie)
#pragma unroll
                for (int it = 0; it < 4; ++it) acc[ie][it] = __builtin_fmaf(a[ie], x[it], acc[ie][it]);
        }
    }
#pragma unroll
    for (int ie = 0; ie < 4; ++ie)
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            float sum = 0.0f;  // acc[0] + acc[1] + ... + acc[7] in order
#pragma unroll
            for (int q = 0; q < 8; ++q) sum += __shfl(acc[ie][it], (tid & 63 & ~7) + q, kWave);
            const int e = e0 + eg + 4 * ie, t = t0 + tg + 4 * it;
            if (j == 0 && e < n_expert && t < rows) logits[(size_t)t * n_expert + e] = sum;
        }
}

// ───────────────────────────── rows == 1: f32 (ActsKind::Raw) path ─────────────────────────────
// A lane owns 64 consecutive-or-strided weights of a row ("unit" u of the row's in_f / 64) and
// keeps the matching 64 activation floats in registers; S = in_f / 64 lanes cover a weight row and
// 64 / S rows run per wave step. The CPU decodes each weight to f32 (dequant_block) and runs an
// f32 dot; here the same sum is factored per scale group as sc * sum(code * x) + mn * sum(x)
// (one conversion and one FMA per weight), which moves the result by f32 rounding only - orders
// of magnitude inside the 1e-4 relative bound this path is held to. One policy per bank format:
//   Row / load_row(r, row pointer, u, ok)      the lane's bytes of a weight row
//   X   / load_x(x, source, u)                 its activation floats and the group sums it needs
//   partial(r, x, u)                           sum over the lane's 64 weights of w * x

// Where a lane's 64 activation floats come from, four at a time: quad q (0..15) of unit u is the
// four floats from element `e` of the row on.
//   XLinear    the row as the caller holds it: a lane's quads are 256 bytes apart from its
//              neighbour's, so one load instruction touches 64 cache lines
//   XLds       a round of the row staged in LDS by the whole workgroup (coalesced), four floats of
//              padding per 64 so that the lanes' 16-byte reads spread over the banks
//   XByQuad    a row stored quad-major, [q][unit][4]: consecutive lanes read consecutive 16 bytes.
//              The gate / up kernel writes the activations in this order for the down kernel.
struct XLinear {
    const float* x;
    __device__ v4f get(int, int, int e) const { return *reinterpret_cast<const v4f*>(x + e); }
};
struct XLds {
    const float* xs;
    int e0;  // first element of the staged round
    __device__ static int pad(int i) { return i + (i >> 6) * 4; }
    __device__ v4f get(int, int, int e) const { return *reinterpret_cast<const v4f*>(xs + pad(e - e0)); }
};
struct XByQuad {
    const float* xt;
    int n_units;
    __device__ v4f get(int u, int q, int) const {
        return *reinterpret_cast<const v4f*>(xt + ((size_t)q * n_units + u) * 4);
    }
};

// Keeps a masked dword whole in the compiler's eyes: byte k of it then converts with one
// v_cvt_f32_ubyte<k>, where a mask folded into each byte's extraction costs a bit-field extract more.
__device__ __forceinline__ uint32_t whole_dword(uint32_t v) {
    asm("" : "+v"(v));
    return v;
}

// Q4_K: unit u = (block u/4, nibble pair u%4): sub-block 2p in the low nibbles of the pair's
// 32 bytes, 2p+1 in the high ones. w = (d*sc)*code - dmin*m.
struct RawQ4K {
    static constexpr int kBlockBytes = 144;
    struct Row {
        v4i hdr, qa, qb;
    };
    struct X {
        float x[64];
        float sum_lo, sum_hi;  // sum of x[0..32), x[32..64)
    };
    __device__ static void load_row(Row& r, const uint8_t* rowp, int u, bool ok) {
        if (ok) {
            const uint8_t* blk = rowp + (size_t)(u >> 2) * 144;
            const int p = u & 3;
            r.hdr = load16(blk);
            r.qa = load16(blk + 16 + p * 32);
            r.qb = load16(blk + 32 + p * 32);
        } else {
            r.hdr = r.qa = r.qb = v4i{0, 0, 0, 0};
        }
    }
    // element of the row that quad q of unit u starts at (quad_place_linear is the way back)
    __device__ static int quad_elem(int u, int q) { return u * 64 + q * 4; }
    template <typename Src>
    __device__ static void load_x(X& a, const Src& src, int u) {
        float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            const v4f v = src.get(u, k, quad_elem(u, k));
            a.x[4 * k + 0] = v.x; a.x[4 * k + 1] = v.y; a.x[4 * k + 2] = v.z; a.x[4 * k + 3] = v.w;
            if (k < 8) { s0 += v.x + v.y; s1 += v.z + v.w; } else { s2 += v.x + v.y; s3 += v.z + v.w; }
        }
        a.sum_lo = s0 + s1;
        a.sum_hi = s2 + s3;
    }
    __device__ static float partial(const Row& r, const X& a, int u) {
        const int p = u & 3;
        uint32_t sc8[2], mn8[2];
        k4_all((uint32_t)r.hdr.y, (uint32_t)r.hdr.z, (uint32_t)r.hdr.w, sc8, mn8);
        const uint32_t scw = (p & 2) ? sc8[1] : sc8[0];
        const uint32_t mnw = (p & 2) ? mn8[1] : mn8[0];
        const int sh = (p & 1) * 16;
        const float d = f16_bits_to_f32((uint32_t)r.hdr.x & 0xFFFFu);
        const float dmin = f16_bits_to_f32((uint32_t)r.hdr.x >> 16);
        const float fs_lo = d * (float)(int)((scw >> sh) & 0xFF), fs_hi = d * (float)(int)((scw >> (sh + 8)) & 0xFF);
        const float fm_lo = dmin * (float)(int)((mnw >> sh) & 0xFF), fm_hi = dmin * (float)(int)((mnw >> (sh + 8)) & 0xFF);
        const int wq[8] = {r.qa.x, r.qa.y, r.qa.z, r.qa.w, r.qb.x, r.qb.y, r.qb.z, r.qb.w};
        float lo0 = 0.0f, lo1 = 0.0f, hi0 = 0.0f, hi1 = 0.0f;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const uint32_t w = (uint32_t)wq[k];
            const uint32_t l = whole_dword(w & 0x0F0F0F0Fu), h = whole_dword((w >> 4) & 0x0F0F0F0Fu);
            lo0 = __builtin_fmaf((float)(l & 0xFF), a.x[4 * k + 0], lo0);
            lo1 = __builtin_fmaf((float)((l >> 8) & 0xFF), a.x[4 * k + 1], lo1);
            lo0 = __builtin_fmaf((float)((l >> 16) & 0xFF), a.x[4 * k + 2], lo0);
            lo1 = __builtin_fmaf((float)(l >> 24), a.x[4 * k + 3], lo1);
            hi0 = __builtin_fmaf((float)(h & 0xFF), a.x[32 + 4 * k + 0], hi0);
            hi1 = __builtin_fmaf((float)((h >> 8) & 0xFF), a.x[32 + 4 * k + 1], hi1);
            hi0 = __builtin_fmaf((float)((h >> 16) & 0xFF), a.x[32 + 4 * k + 2], hi0);
            hi1 = __builtin_fmaf((float)(h >> 24), a.x[32 + 4 * k + 3], hi1);
        }
        return (fs_lo * (lo0 + lo1) - fm_lo * a.sum_lo) + (fs_hi * (hi0 + hi1) - fm_hi * a.sum_hi);
    }
};

// Q5_K: RawQ4K's mapping on the 176-byte block; the 5th code bit of sub-block s, element l, is
// bit s of qh[l], so pair p adds bits 2p / 2p+1 of the block's 32 qh bytes to its two nibbles.
struct RawQ5K {
    static constexpr int kBlockBytes = 176;
    struct Row {
        v4i hdr, ha, hb, qa, qb;
    };
    typedef RawQ4K::X X;
    __device__ static void load_row(Row& r, const uint8_t* rowp, int u, bool ok) {
        if (ok) {
            const uint8_t* blk = rowp + (size_t)(u >> 2) * 176;
            const int p = u & 3;
            r.hdr = load16(blk);
            r.ha = load16(blk + 16);
            r.hb = load16(blk + 32);
            r.qa = load16(blk + 48 + p * 32);
            r.qb = load16(blk + 64 + p * 32);
        } else {
            r.hdr = v4i{0, 0, 0, 0};
            r.ha = v4i{0, 0, 0, 0};
            r.hb = v4i{0, 0, 0, 0};
            r.qa = v4i{0, 0, 0, 0};
            r.qb = v4i{0, 0, 0, 0};
        }
    }
    __device__ static int quad_elem(int u, int q) { return RawQ4K::quad_elem(u, q); }
    template <typename Src>
    __device__ static void load_x(X& a, const Src& src, int u) { RawQ4K::load_x(a, src, u); }
    __device__ static float partial(const Row& r, const X& a, int u) {
        const int p = u & 3;
        uint32_t sc8[2], mn8[2];
        k4_all((uint32_t)r.hdr.y, (uint32_t)r.hdr.z, (uint32_t)r.hdr.w, sc8, mn8);
        const uint32_t scw = (p & 2) ? sc8[1] : sc8[0];
        const uint32_t mnw = (p & 2) ? mn8[1] : mn8[0];
        const int sh = (p & 1) * 16;
        const float d = f16_bits_to_f32((uint32_t)r.hdr.x & 0xFFFFu);
        const float dmin = f16_bits_to_f32((uint32_t)r.hdr.x >> 16);
        const float fs_lo = d * (float)(int)((scw >> sh) & 0xFF), fs_hi = d * (float)(int)((scw >> (sh + 8)) & 0xFF);
        const float fm_lo = dmin * (float)(int)((mnw >> sh) & 0xFF), fm_hi = dmin * (float)(int)((mnw >> (sh + 8)) & 0xFF);
        const int wq[8] = {r.qa.x, r.qa.y, r.qa.z, r.qa.w, r.qb.x, r.qb.y, r.qb.z, r.qb.w};
        const int hq[8] = {r.ha.x, r.ha.y, r.ha.z, r.ha.w, r.hb.x, r.hb.y, r.hb.z, r.hb.w};
        float lo0 = 0.0f, lo1 = 0.0f, hi0 = 0.0f, hi1 = 0.0f;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const uint32_t w = (uint32_t)wq[k], hb = (uint32_t)hq[k] >> (2 * p);
            const uint32_t l = (w & 0x0F0F0F0Fu) | ((hb & 0x01010101u) << 4);
            const uint32_t h = ((w >> 4) & 0x0F0F0F0Fu) | (((hb >> 1) & 0x01010101u) << 4);
            lo0 = __builtin_fmaf((float)(l & 0xFF), a.x[4 * k + 0], lo0);
            lo1 = __builtin_fmaf((float)((l >> 8) & 0xFF), a.x[4 * k + 1], lo1);
            lo0 = __builtin_fmaf((float)((l >> 16) & 0xFF), a.x[4 * k + 2], lo0);
            lo1 = __builtin_fmaf((float)(l >> 24), a.x[4 * k + 3], lo1);
            hi0 = __builtin_fmaf((float)(h & 0xFF), a.x[32 + 4 * k + 0], hi0);
            hi1 = __builtin_fmaf((float)((h >> 8) & 0xFF), a.x[32 + 4 * k + 1], hi1);
            hi0 = __builtin_fmaf((float)((h >> 16) & 0xFF), a.x[32 + 4 * k + 2], hi0);
            hi1 = __builtin_fmaf((float)(h >> 24), a.x[32 + 4 * k + 3], hi1);
        }
        return (fs_lo * (lo0 + lo1) - fm_lo * a.sum_lo) + (fs_hi * (hi0 + hi1) - fm_hi * a.sum_hi);
    }
};

// Q6_K: unit u = (block u/4, half h = (u%4)/2, c = u%2) as in the decode GEMV: the lane decodes
// the four 16-element groups {l, l+32, l+64, l+96}, l in [16c, 16c+16), of its 128-element half;
// group k has scale index h*8 + c + 2k. w = d * sc * (q - 32).
struct RawQ6K {
    static constexpr int kBlockBytes = 210;
    typedef FmtQ6K::Row Row;
    struct X {
        float x[64];    // x[16k + j] = element 128h + 32k + 16c + j of the block
        float gsum[4];  // sum over each group's 16 activations
    };
    __device__ static void load_row(Row& r, const uint8_t* rowp, int u, bool ok) {
        FmtQ6K::load_row(r, rowp, 0, u, ok);
    }
    __device__ static int quad_elem(int u, int q) {
        const int h = (u >> 1) & 1, c = u & 1;
        return (u >> 2) * 256 + h * 128 + c * 16 + 32 * (q >> 2) + 4 * (q & 3);
    }
    template <typename Src>
    __device__ static void load_x(X& a, const Src& src, int u) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            float s0 = 0.0f, s1 = 0.0f;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const v4f v = src.get(u, 4 * k + q, quad_elem(u, 4 * k + q));
                a.x[16 * k + 4 * q + 0] = v.x; a.x[16 * k + 4 * q + 1] = v.y;
                a.x[16 * k + 4 * q + 2] = v.z; a.x[16 * k + 4 * q + 3] = v.w;
                s0 += v.x + v.y;
                s1 += v.z + v.w;
            }
            a.gsum[k] = s0 + s1;
        }
    }
    __device__ static float partial(const Row& r, const X& a, int u) {
        const int c = u & 1;
        const uint32_t m4 = 0x0F0F0F0Fu, m2 = 0x30303030u;
        const int la[4] = {r.qla.x, r.qla.y, r.qla.z, r.qla.w};
        const int lb[4] = {r.qlb.x, r.qlb.y, r.qlb.z, r.qlb.w};
        const int hh[4] = {r.qh.x, r.qh.y, r.qh.z, r.qh.w};
        float dotq[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t lo = (uint32_t)la[j], hi = (uint32_t)lb[j], hb = (uint32_t)hh[j];
            const uint32_t w[4] = {(lo & m4) | ((hb << 4) & m2), (hi & m4) | ((hb << 2) & m2),
                                   ((lo >> 4) & m4) | (hb & m2), ((hi >> 4) & m4) | ((hb >> 2) & m2)};
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                dotq[k] = __builtin_fmaf((float)(w[k] & 0xFF), a.x[16 * k + 4 * j + 0], dotq[k]);
                dotq[k] = __builtin_fmaf((float)((w[k] >> 8) & 0xFF), a.x[16 * k + 4 * j + 1], dotq[k]);
                dotq[k] = __builtin_fmaf((float)((w[k] >> 16) & 0xFF), a.x[16 * k + 4 * j + 2], dotq[k]);
                dotq[k] = __builtin_fmaf((float)(w[k] >> 24), a.x[16 * k + 4 * j + 3], dotq[k]);
            }
        }
        const uint32_t lo = (uint32_t)r.sc.x >> (8 * c), hi = (uint32_t)r.sc.y >> (8 * c);
        const float sc[4] = {(float)(int)(int8_t)(lo & 0xFF), (float)(int)(int8_t)((lo >> 16) & 0xFF),
                             (float)(int)(int8_t)(hi & 0xFF), (float)(int)(int8_t)((hi >> 16) & 0xFF)};
        const float d = f16_bits_to_f32(r.d);
        float acc = 0.0f;
#pragma unroll
        for (int k = 0; k < 4; ++k) acc += (d * sc[k]) * (dotq[k] - 32.0f * a.gsum[k]);
        return acc;
    }
};

// Q8_0: unit u = the two 32-blocks 2u, 2u+1. w = d * q.
struct RawQ8_0 {
    static constexpr int kBlockBytes = 8 * 34;  // per 256 elements
    struct Row {
        FmtQ8_0::Row b0, b1;
    };
    struct X {
        float x[64];
    };
    __device__ static void load_row(Row& r, const uint8_t* rowp, int u, bool ok) {
        FmtQ8_0::load_row(r.b0, rowp, 0, 2 * u, ok);
        FmtQ8_0::load_row(r.b1, rowp, 0, 2 * u + 1, ok);
    }
    __device__ static int quad_elem(int u, int q) { return RawQ4K::quad_elem(u, q); }
    template <typename Src>
    __device__ static void load_x(X& a, const Src& src, int u) {
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            const v4f v = src.get(u, k, quad_elem(u, k));
            a.x[4 * k + 0] = v.x; a.x[4 * k + 1] = v.y; a.x[4 * k + 2] = v.z; a.x[4 * k + 3] = v.w;
        }
    }
    __device__ static float block_dot(const FmtQ8_0::Row& b, const float* x) {
        const int q[8] = {b.qa.x, b.qa.y, b.qa.z, b.qa.w, b.qb.x, b.qb.y, b.qb.z, b.qb.w};
        float s0 = 0.0f, s1 = 0.0f;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            s0 = __builtin_fmaf((float)(int)(int8_t)(q[k] & 0xFF), x[4 * k + 0], s0);
            s1 = __builtin_fmaf((float)(int)(int8_t)((q[k] >> 8) & 0xFF), x[4 * k + 1], s1);
            s0 = __builtin_fmaf((float)(int)(int8_t)((q[k] >> 16) & 0xFF), x[4 * k + 2], s0);
            s1 = __builtin_fmaf((float)(q[k] >> 24), x[4 * k + 3], s1);
        }
        return f16_bits_to_f32(b.d) * (s0 + s1);
    }
    __device__ static float partial(const Row& r, const X& a, int) {
        return block_dot(r.b0, a.x) + block_dot(r.b1, a.x + 32);
    }
};

// Sum over the S lanes (a multiple of 4) of a row segment; every lane of the segment gets the total.
__device__ __forceinline__ float seg_sum(float v, int seg_base, int S) {
    v += __builtin_bit_cast(float, quad_xor1(__builtin_bit_cast(int, v)));
    v += __builtin_bit_cast(float, quad_xor2(__builtin_bit_cast(int, v)));
    if ((S & (S - 1)) == 0) {  // a power of two: the rest of the butterfly
        for (int o = 4; o < S; o <<= 1) v += __shfl_xor(v, o, kWave);
        return v;
    }
    float s = 0.0f;
    for (int i = 0; i < S / 4; ++i) s += __shfl(v, seg_base + 4 * i, kWave);
    return s;
}

// gate/up at one token: act[slot][o] = silu(gate_e[o] . x) * (up_e[o] . x), e = the expert of rank `slot`.
// A wave takes SPW consecutive row steps and requests all their rows before it computes the
// first: at one token the kernel is a few memory round trips deep, so every request it can make
// up front is a round trip less.
template <typename P, int SPW>
__global__ __launch_bounds__(256) void moe_gate_up_f32_kernel(
    const uint8_t* __restrict__ gate, const uint8_t* __restrict__ up, size_t gate_stride,
    size_t up_stride, const float* __restrict__ logits, int n_expert, int n_used, float scale,
    int32_t* __restrict__ sel_idx, float* __restrict__ sel_w, const float* __restrict__ x,
    float* __restrict__ act, int ne, int nff, int S, int chunks, int down_q6k, MoeRoute rt, MoeAct ma) {
    __shared__ __attribute__((aligned(16))) SelectLds sel;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int rps = 64 / S;  // S lanes per weight row (each on `chunks` units of it), rows per wave step
    const int seg = lane / S, u = lane % S;
    const bool lane_ok = seg < rps;
    const int slot = blockIdx.y;
    const int steps_total = (nff + rps - 1) / rps;
    const int st0 = (blockIdx.x * 4 + wave) * SPW;
    // the activation does not depend on the routing: requested first, it arrives under the selection
    // (every lane loads: idle lanes and rows past the end sit on valid units of row 0 and drop
    // their results, which keeps branches and zero fills out of the load sequence)
    // `x` is the row in quad-major order (the router kernel leaves it so): consecutive lanes read
    // consecutive 16 bytes
    const XByQuad xsrc{x, ne / 64};
    typename P::X xa;
    P::load_x(xa, xsrc, u);
    // Every workgroup selects for itself from the router's logits (a few hundred bytes and a few
    // barriers) instead of waiting for a selection kernel in between; the first one also leaves
    // the ranked experts and weights for the down kernel.
    const bool first = blockIdx.x == 0 && blockIdx.y == 0;
    moe_select_block(logits, sel, n_expert, n_used, scale, threadIdx.x, first ? sel_idx : nullptr,
                     first ? sel_w : nullptr, rt, 0);
    if (st0 >= steps_total) return;
    const int e = sel.top_e[slot];
    // the routing weight on the expert input (`weight_before`): gate and up are linear in x, so it
    // multiplies their outputs in front of the activation (lib.rs:2833-2857)
    const float wp = ma.weight_before ? sel.top_w[slot] : 1.0f;
    const size_t bpr = (size_t)(ne / 256) * P::kBlockBytes;
    const uint8_t* gw = gate + (size_t)e * gate_stride;
    const uint8_t* uw = up + (size_t)e * up_stride;
    float gp[SPW], upp[SPW];
#pragma unroll
    for (int i = 0; i < SPW; ++i) gp[i] = upp[i] = 0.0f;
    // rows longer than 64 lanes x 64 weights: unit c * S + u in round c, the partial sums added per lane
    for (int c = 0; c < chunks; ++c) {
        const int uc = c * S + u;
        if (c) P::load_x(xa, xsrc, uc);
        typename P::Row g[SPW], up_r[SPW];
#pragma unroll
        for (int i = 0; i < SPW; ++i) {
            const int o = (st0 + i) * rps + seg;
            const bool ok = lane_ok && o < nff;
            P::load_row(g[i], gw + (size_t)(ok ? o : 0) * bpr, uc, true);
            P::load_row(up_r[i], uw + (size_t)(ok ? o : 0) * bpr, uc, true);
        }
#pragma unroll
        for (int i = 0; i < SPW; ++i) {
            gp[i] += P::partial(g[i], xa, uc);
            upp[i] += P::partial(up_r[i], xa, uc);
        }
    }
#pragma unroll
    for (int i = 0; i < SPW; ++i) {
        const int o = (st0 + i) * rps + seg;
        const bool ok = lane_ok && o < nff;
        const float gs = seg_sum(gp[i], seg * S, S);
        const float us = seg_sum(upp[i], seg * S, S);
        if (ok && u == 0) {
            // stored in the order the down kernel's lanes read: [quad][unit][4] of its format
            int du, dq;
            if (down_q6k) quad_place_q6k(o, du, dq);
            else quad_place_linear(o, du, dq);
            act[(size_t)slot * nff + ((size_t)dq * (nff / 64) + du) * 4 + (o & 3)] =
                gated_act_fn(ma.act, ma.has_clamp != 0, ma.clamp, wp * gs, wp * us);
        }
    }
}

// down + accumulate at one token: out[o] = sum_k w_k * (down_{ids[k]}[o] . act[k]), k in rank
// order. One wave per selected expert (up to eight at a time: 512 threads leave every wave the 256
// registers that four row steps in flight need), every wave of a workgroup on the same STEPS row
// steps, all requested up front; the per-expert results meet in LDS and are added in rank order
// with a separate multiply and add, as the CPU's `*o += w_e * yv`.
constexpr int kDownMaxSteps = 4, kDownMaxWaves = 8;
// (2048 against 1024: 25.3 against 27.8 us per layer at 128 experts x 768 x 2048, top-8 - one row step per
// wave there; the shapes with many more steps per expert keep four steps per wave either way)
constexpr int kMoeWavesWanted = 2048;

template <typename P, int STEPS>
__global__ __launch_bounds__(64 * kDownMaxWaves) void moe_down_f32_kernel(
    const uint8_t* __restrict__ down, size_t down_stride, const int32_t* __restrict__ ids,
    const float* __restrict__ wts, const float* __restrict__ act, float* __restrict__ out,
    const float* add_b, float* add_dst, int nff, int ne, int n_used, int S, int chunks, int unit_w,
    const float* __restrict__ down_scale) {
    __shared__ float ys[kDownMaxSteps][kDownMaxWaves][16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const int rps = 64 / S;
    const int seg = lane / S, u = lane % S;
    const bool lane_ok = seg < rps;
    const size_t bpr = (size_t)(nff / 256) * P::kBlockBytes;
    const int st0 = blockIdx.x * STEPS;
    const int own_s = threadIdx.x / rps, own_seg = threadIdx.x % rps;  // output this thread adds up
    const bool owner = (int)threadIdx.x < STEPS * rps;
    float acc = 0.0f;
    for (int k0 = 0; k0 < n_used; k0 += nw) {
        const int k = k0 + wave;
        if (k0) __syncthreads();
        if (k < n_used) {
            const uint8_t* dw = down + (size_t)ids[k] * down_stride;
            const float ds = down_scale ? down_scale[ids[k]] : 1.0f;  // `y = raw * s_e` (lib.rs:2932-2938)
            float part[STEPS];
#pragma unroll
            for (int s = 0; s < STEPS; ++s) part[s] = 0.0f;
            for (int c = 0; c < chunks; ++c) {
                const int uc = c * S + u;
                typename P::Row row[STEPS];
#pragma unroll
                for (int s = 0; s < STEPS; ++s) {
                    const int o = (st0 + s) * rps + seg;
                    const bool ok = lane_ok && o < ne;
                    P::load_row(row[s], dw + (size_t)(ok ? o : 0) * bpr, uc, true);
                }
                typename P::X xa;
                P::load_x(xa, XByQuad{act + (size_t)k * nff, nff / 64}, uc);
#pragma unroll
                for (int s = 0; s < STEPS; ++s) part[s] += P::partial(row[s], xa, uc);
            }
#pragma unroll
            for (int s = 0; s < STEPS; ++s) {
                const float yk = seg_sum(part[s], seg * S, S);
                if (lane_ok && u == 0) ys[s][wave][seg] = down_scale ? yk * ds : yk;
            }
        }
        __syncthreads();
        if (owner) {
            const int kn = min(nw, n_used - k0);
            // (`weight_before`: the weight is inside the activation already, w_e = 1.0, lib.rs:2976)
            for (int j = 0; j < kn; ++j) acc += (unit_w ? 1.0f : wts[k0 + j]) * ys[own_s][j][own_seg];
        }
    }
    if (owner) {
        const int o = (st0 + own_s) * rps + own_seg;
        if (o < ne) {
            if (out != add_dst) out[o] = acc;  // an Add in place on this op's dst stores the sum only
            if (add_dst) add_dst[o] = acc + add_b[o];
        }
    }
}

// ───────────────────────────── rows >= 2: int8 path ─────────────────────────────

// gated_act_fn(act, clamp, wp * gate, wp * up) for four elements (lib.rs:2836-2857): wp is the pair's
// routing weight under `weight_before`, else 1.0 (an exact identity).
__device__ __forceinline__ v4f moe_gated4(const MoeAct& ma, float wp, const v4f& g, const v4f& u) {
    const bool c = ma.has_clamp != 0;
    return v4f{gated_act_fn(ma.act, c, ma.clamp, wp * g.x, wp * u.x), gated_act_fn(ma.act, c, ma.clamp, wp * g.y, wp * u.y),
               gated_act_fn(ma.act, c, ma.clamp, wp * g.z, wp * u.z), gated_act_fn(ma.act, c, ma.clamp, wp * g.w, wp * u.w)};
}

// id-gathered decode GEMV over pre-quantized activation rows: pair = blockIdx.y,
// weights = bank + ids[pair] * expert_stride, activation row = pair / n_used.
template <typename F, int STEPS>
__global__ __launch_bounds__(256) void gemv_id_kernel(const uint8_t* __restrict__ bank,
                                                      size_t expert_stride, size_t bpr,
                                                      const int32_t* __restrict__ ids, ActPtrs act,
                                                      int in_f, int n_used, float* __restrict__ y,
                                                      int out_f, int rows_per_wave) {
    const int lane = threadIdx.x & 63;
    const int wave = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int row0 = wave * rows_per_wave;
    if (row0 >= out_f) return;
    const int row_end = min(row0 + rows_per_wave, out_f);
    const int pair = blockIdx.y, r = pair / n_used;
    const uint8_t* w = bank + (size_t)ids[pair] * expert_stride;
    const int n_units = F::units(in_f);
    ActPtrs a;
    a.qs = act.qs + (size_t)r * in_f;
    a.d = act.d + (size_t)r * (in_f / (F::kPer32 ? 32 : 256));
    a.bsums = act.bsums + (size_t)r * (in_f / 32);
    a.bsums16 = F::kPer32 ? nullptr : act.bsums16 + (size_t)r * (in_f / 16);
    typename F::Acts acts[STEPS];
    typename F::Row first[1];
    bool ok[STEPS];
#pragma unroll
    for (int t = 0; t < STEPS; ++t) ok[t] = F::valid(t, lane, n_units);
    F::load_row(first[0], w + (size_t)row0 * bpr, 0, lane, ok[0]);
#pragma unroll
    for (int t = 0; t < STEPS; ++t) F::load_acts(acts[t], a, t, lane, ok[t]);
    // same body as the decode GEMV: per-block exact integers, and the f32 terms added in ascending
    // block order for every format (the one-block-per-lane formats through LANE_ORDERED), so each
    // output equals the scalar CPU kernel's bit for bit and the int8 codes of the gated activation
    // that the down bank multiplies equal the CPU's
    constexpr bool kLaneOrdered = !F::kOrdered;
    __shared__ __attribute__((aligned(16))) float osum[4 * RowSumScratch<F, STEPS, kLaneOrdered>::kFloatsPerWave];
    gemv_rows<F, STEPS, false, false, kLaneOrdered>(w, bpr, first, acts, ok, y + (size_t)pair * out_f, n_units, row0,
                                                    row_end, lane, StagePtrs{nullptr, nullptr},
                                                    osum + (threadIdx.x >> 6) *
                                                               RowSumScratch<F, STEPS, kLaneOrdered>::kFloatsPerWave);
}

// The same for short rows (in_f <= 2048) of Q4_K / Q6_K banks: 16 / nb rows per wave step.
// blockIdx.z selects one of two same-shaped banks (gate and up share a launch).
template <typename F>
__global__ __launch_bounds__(256) void gemv_id_folded_kernel(const uint8_t* __restrict__ bank0,
                                                             const uint8_t* __restrict__ bank1,
                                                             size_t expert_stride0,
                                                             size_t expert_stride1, size_t bpr,
                                                             const int32_t* __restrict__ ids,
                                                             ActPtrs act, int in_f, int n_used,
                                                             float* __restrict__ y0,
                                                             float* __restrict__ y1, int out_f,
                                                             int rows_per_wave) {
    const int lane = threadIdx.x & 63;
    const int wave = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int row0 = wave * rows_per_wave;
    if (row0 >= out_f) return;
    const int row_end = min(row0 + rows_per_wave, out_f);
    const int pair = blockIdx.y, r = pair / n_used;
    const bool second = blockIdx.z != 0;
    const uint8_t* w = (second ? bank1 : bank0) + (size_t)ids[pair] * (second ? expert_stride1 : expert_stride0);
    float* y = second ? y1 : y0;
    const int nb = in_f / 256, q = lane >> 2;
    const int shift = q - q % nb;  // load_acts addresses block q; this lane wants block q % nb
    ActPtrs a;
    a.qs = act.qs + (size_t)r * in_f - (size_t)shift * 256;
    a.d = act.d + (size_t)r * nb - shift;
    a.bsums = act.bsums + (size_t)r * (in_f / 32) - shift * 8;
    a.bsums16 = act.bsums16 + (size_t)r * (in_f / 16) - shift * 16;
    typename F::Acts acts;
    F::load_acts(acts, a, 0, lane, q / nb < 16 / nb);
    __shared__ __attribute__((aligned(16))) float osum[4 * OrderedSum<1>::kFloatsPerWave];
    gemv_rows_folded<F>(w, bpr, nb, acts, y + (size_t)pair * out_f, row0, row_end, lane,
                        osum + (threadIdx.x >> 6) * OrderedSum<1>::kFloatsPerWave);
}

// act = silu(g) * u per pair row, quantized per 256 for the down bank (lib.rs:2824-2892).
// One wavefront per 256-float chunk.
template <bool PER32>
__global__ __launch_bounds__(256) void moe_act_quant_kernel(const float* __restrict__ g,
                                                            const float* __restrict__ u,
                                                            int8_t* __restrict__ qs,
                                                            float* __restrict__ d,
                                                            int32_t* __restrict__ bsums,
                                                            int32_t* __restrict__ bsums16,
                                                            size_t n_elems, int nff, MoeAct ma,
                                                            const float* __restrict__ pair_w) {
    const int lane = threadIdx.x & 63;
    const size_t chunk = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (chunk * 256 >= n_elems) return;
    const v4f gv = *reinterpret_cast<const v4f*>(g + chunk * 256 + (size_t)lane * 4);
    const v4f uv = *reinterpret_cast<const v4f*>(u + chunk * 256 + (size_t)lane * 4);
    const float wp = ma.weight_before ? pair_w[chunk * 256 / (size_t)nff] : 1.0f;
    const v4f a = moe_gated4(ma, wp, gv, uv);
    quantize_chunk<PER32>(a, true, lane, chunk, qs, d, bsums, PER32 ? nullptr : bsums16);
}

// A few rows, short expert rows (n_ff <= 2048) of a 16-block format: activation, down projection
// and the weighted sum over a token's experts in one launch. A workgroup is a token and a tile of
// output rows; wave k takes the token's k-th expert: it requests its first weight step, builds
// act = silu(g) * u of its pair and quantizes it per 256 into its own LDS (the stand-alone kernel's
// arithmetic), runs the folded decode body into an LDS row, and after a barrier thread o adds
// w_k * y_k[o] over the experts in rank order with a separate multiply and add - the values and
// the order of moe_act_quant_kernel, the id-gathered GEMV and moe_accumulate_kernel, without the
// two launches in between and without the per-pair outputs going through memory.
// LDS per wave: qs[nff] | d[nff / 256, padded to 4] | bsums[nff / 32] | bsums16[nff / 16] | ordered-sum scratch | y[rows_per_wg]
__host__ __device__ constexpr size_t moe_down_fused_y_offset(int nff) {
    return (size_t)nff + (size_t)((nff / 256 + 3) / 4 * 4 + nff / 32 + nff / 16 + OrderedSum<1>::kFloatsPerWave) * 4;
}
__host__ __device__ constexpr size_t moe_down_fused_wave_bytes(int nff, int rows_per_wg) {
    return (moe_down_fused_y_offset(nff) + (size_t)rows_per_wg * 4 + 15) / 16 * 16;
}
template <typename F>
__global__ __launch_bounds__(1024) void moe_down_fused_kernel(
    const uint8_t* __restrict__ bank, size_t expert_stride, size_t bpr, const int32_t* __restrict__ ids,
    const float* __restrict__ wts, const float* __restrict__ g, const float* __restrict__ u,
    float* __restrict__ out, const float* add_b, float* add_dst, int nff, int ne, int n_used, int rows_per_wg,
    MoeAct ma, const float* __restrict__ down_scale) {
    extern __shared__ __attribute__((aligned(16))) uint8_t dlds[];
    const int lane = threadIdx.x & 63, k = threadIdx.x >> 6;
    const int token = blockIdx.y, pair = token * n_used + k;
    const int row0 = blockIdx.x * rows_per_wg, row_end = min(row0 + rows_per_wg, ne);
    const int nb = nff / 256;
    const size_t wave_bytes = moe_down_fused_wave_bytes(nff, rows_per_wg);
    uint8_t* mine = dlds + (size_t)k * wave_bytes;
    int8_t* qs = reinterpret_cast<int8_t*>(mine);
    float* d = reinterpret_cast<float*>(mine + nff);
    int32_t* bsums = reinterpret_cast<int32_t*>(d + (nb + 3) / 4 * 4);
    int32_t* bsums16 = bsums + nff / 32;
    float* osum = reinterpret_cast<float*>(bsums16 + nff / 16);
    const size_t y_off = moe_down_fused_y_offset(nff);
    float* yk = reinterpret_cast<float*>(mine + y_off);
    const uint8_t* w = bank + (size_t)ids[pair] * expert_stride;
    const int q = lane >> 2, rq = q / nb;
    typename F::Row first;
    F::load_row(first, w + (size_t)row0 * bpr, 0, lane, rq < 16 / nb && row0 + rq < row_end);
    const float wp = ma.weight_before ? wts[pair] : 1.0f;
    for (int c = 0; c < nb; ++c) {
        const v4f gv = *reinterpret_cast<const v4f*>(g + (size_t)pair * nff + c * 256 + lane * 4);
        const v4f uv = *reinterpret_cast<const v4f*>(u + (size_t)pair * nff + c * 256 + lane * 4);
        const v4f a = moe_gated4(ma, wp, gv, uv);
        quantize_chunk<false>(a, true, lane, (size_t)c, qs, d, bsums, bsums16);
    }
    __syncthreads();
    const int shift = q - q % nb;  // load_acts addresses block q; this lane wants block q % nb
    ActPtrs a;
    a.qs = qs - (ptrdiff_t)shift * 256;
    a.d = d - shift;
    a.bsums = bsums - shift * 8;
    a.bsums16 = bsums16 - shift * 16;
    typename F::Acts acts;
    F::load_acts(acts, a, 0, lane, q / nb < 16 / nb);
    gemv_rows_folded<F, false>(w, bpr, nb, acts, yk - row0, row0, row_end, lane, osum, &first);
    __syncthreads();
    for (int o = (int)threadIdx.x; o < row_end - row0; o += (int)blockDim.x) {  // (one expert per token: 64 threads)
        float acc = 0.0f;
        for (int j = 0; j < n_used; ++j) {
            const float* yj = reinterpret_cast<const float*>(dlds + (size_t)j * wave_bytes + y_off);
            const float yv = down_scale ? yj[o] * down_scale[ids[token * n_used + j]] : yj[o];
            acc += (ma.weight_before ? 1.0f : wts[token * n_used + j]) * yv;
        }
        const size_t i = (size_t)token * ne + row0 + o;
        if (out != add_dst) out[i] = acc;  // an Add in place on this op's dst stores the sum only
        if (add_dst) add_dst[i] = acc + add_b[i];
    }
}

// The same activation kept in f32 (in place over g) for a down bank that multiplies raw rows.
__global__ __launch_bounds__(256) void moe_act_f32_kernel(float* __restrict__ g, const float* __restrict__ u,
                                                          size_t n_elems, int nff, MoeAct ma,
                                                          const float* __restrict__ pair_w) {
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= n_elems) return;
    const v4f gv = *reinterpret_cast<const v4f*>(g + i), uv = *reinterpret_cast<const v4f*>(u + i);
    const float wp = ma.weight_before ? pair_w[i / (size_t)nff] : 1.0f;
    *reinterpret_cast<v4f*>(g + i) = moe_gated4(ma, wp, gv, uv);
}

// `ActsKind::Raw` for any bank format (crates/infr-cpu/src/moe.rs:143-172): the weight row is decoded
// to f32 as the host decode does and multiplied with `dot` (kernels.rs:6557-6573) - eight FMA chains
// by element index mod 8, added in order - against the f32 activation row, so every output equals
// the CPU's bit for bit. Eight lanes per output row, one chain each; pair = blockIdx.y,
// activation row = pair / act_div. This is the arm of the formats infr-cpu has no int8 expert
// kernel for, and of single rows of shapes the factored one-token kernels do not take: a fallback
// there as here (one byte load and a dozen instructions per weight).
__global__ __launch_bounds__(256) void moe_raw_dot_kernel(int dtype, const uint8_t* __restrict__ bank,
                                                          size_t expert_stride, size_t bpr,
                                                          const int32_t* __restrict__ ids,
                                                          const float* __restrict__ acts, int act_div,
                                                          int in_f, float* __restrict__ y, int out_f) {
    const int pair = blockIdx.y, j = threadIdx.x & 7;
    const int o = (int)blockIdx.x * 32 + ((int)threadIdx.x >> 3);
    const bool live = o < out_f;
    const uint8_t* rowp = bank + (size_t)ids[pair] * expert_stride + (size_t)(live ? o : 0) * bpr;
    const float* x = acts + (size_t)(pair / act_div) * in_f;
    float acc = 0.0f;
    for (int i = j; i < in_f; i += 8) acc = __builtin_fmaf(decode_element(dtype, rowp, i), x[i], acc);
    float sum = 0.0f;
#pragma unroll
    for (int q = 0; q < 8; ++q) sum += __shfl(acc, ((int)threadIdx.x & ~7) + q, kWave);
    if (live && j == 0) y[(size_t)pair * out_f + o] = sum;
}

// out[r][o] = sum_k w[r][k] * yp[r*n_used + k][o], k in rank order (lib.rs:2967-2983)
__global__ __launch_bounds__(256) void moe_accumulate_kernel(const float* __restrict__ yp,
                                                             const float* __restrict__ wts,
                                                             float* __restrict__ out,
                                                             const float* add_b, float* add_dst,
                                                             int ne, int n_used, int rows, int unit_w,
                                                             const float* __restrict__ down_scale,
                                                             const int32_t* __restrict__ ids) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)rows * ne) return;
    const size_t r = i / ne, o = i % ne;
    float acc = 0.0f;
    for (int k = 0; k < n_used; ++k) {
        // `y = raw * s_e` per pair (lib.rs:2932-2938), then `*o += w_e * y`, w_e = 1.0 under weight_before
        const float yv = yp[(r * n_used + k) * ne + o];
        acc += (unit_w ? 1.0f : wts[r * n_used + k]) * (down_scale ? yv * down_scale[ids[r * n_used + k]] : yv);
    }
    if (out != add_dst) out[i] = acc;  // an Add in place on this op's dst stores the sum only
    if (add_dst) add_dst[i] = acc + add_b[i];
}

// Buckets the routed pairs by expert for the prefill path: perm = pair ids grouped by expert,
// plus one tile entry per 32 pairs of an expert. One workgroup; the order of pairs inside a bucket
// depends on the order the atomics land in and does not matter (each pair's outputs are its own).
constexpr int kBucketThreads = 1024;
__global__ __launch_bounds__(kBucketThreads) void moe_bucket_kernel(
    const int32_t* __restrict__ sel_idx, int pairs, int n_expert, int32_t* __restrict__ perm,
    int32_t* __restrict__ tile_expert, int32_t* __restrict__ tile_slot0, int32_t* __restrict__ tile_count,
    int32_t* __restrict__ n_tiles) {
    constexpr int tile_rows = 32;  // 64-pair tiles measured slower (704 us against 554 at 2048 tokens)
    __shared__ int cnt[kBucketThreads], off[kBucketThreads], toff[kBucketThreads], cursor[kBucketThreads];
    const int tid = threadIdx.x;
    cnt[tid] = 0;
    cursor[tid] = 0;
    __syncthreads();
    for (int p = tid; p < pairs; p += kBucketThreads) atomicAdd(&cnt[sel_idx[p]], 1);
    __syncthreads();
    const int mine = tid < n_expert ? cnt[tid] : 0, my_tiles = (mine + tile_rows - 1) / tile_rows;
    off[tid] = mine;
    toff[tid] = my_tiles;
    __syncthreads();
    for (int d = 1; d < kBucketThreads; d <<= 1) {  // inclusive scans of both arrays
        const int a = tid >= d ? off[tid - d] : 0, b = tid >= d ? toff[tid - d] : 0;
        __syncthreads();
        off[tid] += a;
        toff[tid] += b;
        __syncthreads();
    }
    const int first_slot = off[tid] - mine, first_tile = toff[tid] - my_tiles;
    if (tid == kBucketThreads - 1) *n_tiles = toff[tid];
    for (int k = 0; k < my_tiles; ++k) {
        tile_expert[first_tile + k] = tid;
        tile_slot0[first_tile + k] = first_slot + tile_rows * k;
        tile_count[first_tile + k] = min(tile_rows, mine - tile_rows * k);
    }
    __syncthreads();
    off[tid] = first_slot;
    __syncthreads();
    for (int p = tid; p < pairs; p += kBucketThreads) {
        const int e = sel_idx[p];
        perm[off[e] + atomicAdd(&cursor[e], 1)] = p;
    }
}

// ───────────────────────────── launch ─────────────────────────────

// `bank1`/`y1` (optional): a second bank of the same dtype and shape against the same activations.
template <typename F>
static bool launch_gemv_id_fmt(const uint8_t* bank, size_t expert_stride, size_t bpr,
                               const int32_t* ids, const ActQ8& act, size_t in_f, int n_used,
                               int pairs, float* y, size_t out_f, hipStream_t stream,
                               const uint8_t* bank1 = nullptr, size_t expert_stride1 = 0,
                               float* y1 = nullptr) {
    const int steps = (int)((in_f + F::kElemsPerStep - 1) / F::kElemsPerStep);
    const ActPtrs a{act.qs, act.d, act.bsums, act.bsums16};
    if constexpr (F::kOrdered) {
        if (in_f <= 2048) {  // short rows: fold 16 / nb rows into each wave step
            const int rps = 16 / (int)(in_f / 256);
            int wave_steps = 8;
            while (wave_steps > 1 && ((out_f + rps * wave_steps - 1) / (rps * wave_steps) + 3) / 4 * (size_t)pairs < 1024)
                wave_steps /= 2;
            const int rpw = rps * wave_steps;
            const size_t waves = (out_f + rpw - 1) / rpw;
            hipLaunchKernelGGL((gemv_id_folded_kernel<F>),
                               dim3((unsigned)((waves + 3) / 4), (unsigned)pairs, bank1 ? 2u : 1u), dim3(256), 0,
                               stream, bank, bank1, expert_stride, expert_stride1, bpr, ids, a, (int)in_f,
                               n_used, y, y1, (int)out_f, rpw);
            return true;
        }
    }
    if (bank1)  // long rows: one launch per bank
        return launch_gemv_id_fmt<F>(bank, expert_stride, bpr, ids, act, in_f, n_used, pairs, y, out_f, stream) &&
               launch_gemv_id_fmt<F>(bank1, expert_stride1, bpr, ids, act, in_f, n_used, pairs, y1, out_f, stream);
    // enough rows per wave to amortise loading the activation registers, while keeping the grid
    // (row tiles x pairs) well above the CU count
    int rpw = 8;
    while (rpw > 2 && ((out_f + rpw - 1) / rpw + 3) / 4 * (size_t)pairs < 1024) rpw /= 2;
    const size_t waves = (out_f + rpw - 1) / rpw;
    const dim3 grid((unsigned)((waves + 3) / 4), (unsigned)pairs), block(256);
#define INFR_CASE(N)                                                                               \
    case N:                                                                                        \
        hipLaunchKernelGGL((gemv_id_kernel<F, N>), grid, block, 0, stream, bank, expert_stride, bpr, \
                           ids, a, (int)in_f, n_used, y, (int)out_f, rpw);                         \
        return true;
    switch (steps) {
        INFR_CASE(1) INFR_CASE(2) INFR_CASE(3) INFR_CASE(4)
    default: break;
    }
    // rows of five to eight wave steps of the one-block-per-lane formats (2048 columns a step: up to
    // 16384, Mixtral's 14336-wide experts); the K-quants' four steps already reach 16384
    if constexpr (!F::kOrdered) {
        switch (steps) {
            INFR_CASE(5) INFR_CASE(6) INFR_CASE(7) INFR_CASE(8)
        default: break;
        }
    }
    return false;
#undef INFR_CASE
}

static bool launch_gemv_id(int dtype, const uint8_t* bank, size_t expert_stride, size_t bpr,
                           const int32_t* ids, const ActQ8& act, size_t in_f, int n_used, int pairs,
                           float* y, size_t out_f, hipStream_t stream, const uint8_t* bank1 = nullptr,
                           size_t expert_stride1 = 0, float* y1 = nullptr) {
    switch (dtype) {
    case 12: return launch_gemv_id_fmt<FmtQ4K>(bank, expert_stride, bpr, ids, act, in_f, n_used, pairs, y, out_f, stream, bank1, expert_stride1, y1);
    case 13: return launch_gemv_id_fmt<FmtQ5K>(bank, expert_stride, bpr, ids, act, in_f, n_used, pairs, y, out_f, stream, bank1, expert_stride1, y1);
    case 14: return launch_gemv_id_fmt<FmtQ6K>(bank, expert_stride, bpr, ids, act, in_f, n_used, pairs, y, out_f, stream, bank1, expert_stride1, y1);
    case 8: return launch_gemv_id_fmt<FmtQ8_0>(bank, expert_stride, bpr, ids, act, in_f, n_used, pairs, y, out_f, stream, bank1, expert_stride1, y1);
    case 6: return launch_gemv_id_fmt<FmtNib32<Nib32::Q5_0>>(bank, expert_stride, bpr, ids, act, in_f, n_used, pairs, y, out_f, stream, bank1, expert_stride1, y1);
    default: return false;
    }
}

// Activation + down + accumulate in one launch (moe_down_fused_kernel) where that form exists:
// a 16-block bank format, whole expert rows of at most 2048, up to 16 experts per token, 64 KB of LDS.
template <typename F>
static bool launch_moe_down_fused_fmt(const uint8_t* bank, size_t stride, size_t bpr, const int32_t* ids,
                                      const float* wts, const float* g, const float* u, float* out,
                                      const float* add_b, float* add_dst, int nff, int ne, int n_used, int rows,
                                      const MoeAct& ma, const float* down_scale, hipStream_t stream) {
    const int rps = 16 / (nff / 256);
    int wave_steps = 8;  // rows per workgroup: enough waves in all (as the id-gathered launches size theirs)
    while (wave_steps > 1 && (size_t)((ne + rps * wave_steps - 1) / (rps * wave_steps)) * rows * n_used < 4096)
        wave_steps /= 2;
    const int rows_per_wg = rps * wave_steps;
    const size_t lds = moe_down_fused_wave_bytes(nff, rows_per_wg) * n_used;
    if (lds > 64 * 1024) return false;
    hipLaunchKernelGGL((moe_down_fused_kernel<F>), dim3((unsigned)((ne + rows_per_wg - 1) / rows_per_wg), (unsigned)rows),
                       dim3((unsigned)(64 * n_used)), lds, stream, bank, stride, bpr, ids, wts, g, u, out, add_b, add_dst,
                       nff, ne, n_used, rows_per_wg, ma, down_scale);
    return true;
}
static bool launch_moe_down_fused(int dtype, const uint8_t* bank, size_t stride, size_t bpr, const int32_t* ids,
                                  const float* wts, const float* g, const float* u, float* out, const float* add_b,
                                  float* add_dst, int nff, int ne, int n_used, int rows, const MoeAct& ma,
                                  const float* down_scale, hipStream_t stream) {
    if (nff > 2048 || nff % 256 != 0 || n_used > 16 || rows > 65535) return false;
    switch (dtype) {
    case 12: return launch_moe_down_fused_fmt<FmtQ4K>(bank, stride, bpr, ids, wts, g, u, out, add_b, add_dst, nff, ne, n_used, rows, ma, down_scale, stream);
    case 13: return launch_moe_down_fused_fmt<FmtQ5K>(bank, stride, bpr, ids, wts, g, u, out, add_b, add_dst, nff, ne, n_used, rows, ma, down_scale, stream);
    case 14: return launch_moe_down_fused_fmt<FmtQ6K>(bank, stride, bpr, ids, wts, g, u, out, add_b, add_dst, nff, ne, n_used, rows, ma, down_scale, stream);
    default: return false;
    }
}

// logits[t * n_rows_w + r] = dot(w[r], x[t]) in infr-cpu's `dot` order, for `n_rows_w` plain rows of
// `ne` f32 (WT 0), f16 (1) or bf16 (30) weights against `rows` activation rows: the MoE router, and
// Op::Linear over unquantized weights. With a single row and `logits_only` unset the last workgroup
// also selects (tickets, sel_idx, sel_w).
template <int WT>
static void launch_row_dots(const void* w, const float* x, float* logits, int ne, int n_rows_w, int rows,
                            bool logits_only, int* tickets, int32_t* sel_idx, float* sel_w, int n_used, float scale,
                            const float* norm_w, float* norm_dst, float norm_eps, float* xt, int xt_q6k,
                            const MoeRoute& rt, hipStream_t stream) {
    // One weight row per workgroup when only logits are wanted of a single row (nothing to wait
    // for); eight at a single row that ends in the selection (few tickets), four once rows fill the
    // pairs; whole rows in one chunk when they fit the LDS a workgroup may have, else kRouterChunk
    // columns at a time
    constexpr size_t kRouterLdsMax = 144 * 1024;
    int epw = logits_only ? 1 : (rows == 1 ? 8 : 4);
    int tpw = kRouterPairs / epw;
    if (rows > 1) {
        // a few rows: fewer (expert, token) pairs per workgroup, so that about 256 workgroups share
        // the staging (16 tokens x 128 experts: 2 x 4 pairs each instead of 4 x 8 on 64 workgroups)
        int per_wg = 1;
        while (per_wg < kRouterPairs && (size_t)n_rows_w * rows > (size_t)256 * per_wg) per_wg *= 2;
        epw = per_wg >= 16 ? 4 : (per_wg >= 4 ? 2 : 1);
        tpw = per_wg / epw;
    }
    while (epw > 1 && (size_t)(epw + 1) * router_row_floats(ne) * sizeof(float) > kRouterLdsMax) epw /= 2;
    const int n_t = std::min(rows, tpw);
    // (whole rows also for a few rows, while the grid is a single round of one workgroup per compute unit)
    const bool one_round = (size_t)((n_rows_w + epw - 1) / epw) * ((rows + tpw - 1) / tpw) <= 256;
    const bool whole_rows = (size_t)(epw + n_t) * router_row_floats(ne) * sizeof(float) <= (one_round ? kRouterLdsMax : 64 * 1024);
    const int kc = whole_rows ? ne : kRouterChunk;
    const size_t router_lds = (size_t)(epw + n_t) * router_row_floats(kc) * sizeof(float);
    if (router_lds > 64 * 1024)
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&moe_router_kernel<24, WT>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)router_lds);
    if (rows >= kRtMinRows)
        hipLaunchKernelGGL(moe_router_tile_kernel<WT>,
                           dim3((unsigned)((n_rows_w + kRtE - 1) / kRtE), (unsigned)((rows + kRtT - 1) / kRtT)),
                           dim3(kRtThreads), 0, stream, w, x, logits, ne, n_rows_w, rows);
    else if (rows == 1)
        hipLaunchKernelGGL((moe_router_kernel<24, WT>), dim3((unsigned)((n_rows_w + epw - 1) / epw), 1), dim3(256), router_lds,
                           stream, w, x, logits, logits_only ? (int*)nullptr : tickets, sel_idx, sel_w, ne,
                           n_rows_w, rows, n_used, scale, kc, epw, tpw, norm_w, norm_dst, norm_eps, xt, xt_q6k, rt);
    else if (whole_rows && router_lds > 64 * 1024)
        hipLaunchKernelGGL((moe_router_kernel<24, WT>),
                           dim3((unsigned)((n_rows_w + epw - 1) / epw), (unsigned)((rows + tpw - 1) / tpw)),
                           dim3(256), router_lds, stream, w, x, logits, (int*)nullptr, sel_idx, sel_w,
                           ne, n_rows_w, rows, n_used, scale, kc, epw, tpw, (const float*)nullptr, (float*)nullptr,
                           0.0f, (float*)nullptr, 0, rt);
    else
        hipLaunchKernelGGL((moe_router_kernel<8, WT>),
                           dim3((unsigned)((n_rows_w + epw - 1) / epw), (unsigned)((rows + tpw - 1) / tpw)),
                           dim3(256), router_lds, stream, w, x, logits, (int*)nullptr, sel_idx, sel_w,
                           ne, n_rows_w, rows, n_used, scale, kc, epw, tpw, (const float*)nullptr, (float*)nullptr,
                           0.0f, (float*)nullptr, 0, rt);
}

// Op::Linear over plain f32 / f16 / bf16 weight rows (crates/infr-cpu/src/lib.rs:1162-1165,
// 1443-1462: dot / dot_f16 / dot_bf16 per output): y[t, o] = dot(w[o], x[t]), the CPU's bits.
bool launch_linear_plain_rows(int dtype, const void* w, const float* x, float* y, size_t m, size_t in_f, size_t out_f,
                              hipStream_t stream) {
    if (in_f % 32 != 0 || in_f > (size_t)1 << 30 || out_f > (size_t)1 << 30 || m > (size_t)1 << 30) return false;
    switch (dtype) {
    case 0: launch_row_dots<0>(w, x, y, (int)in_f, (int)out_f, (int)m, true, nullptr, nullptr, nullptr, 0, 0.0f, nullptr, nullptr, 0.0f, nullptr, 0, MoeRoute{}, stream); break;
    case 1: launch_row_dots<1>(w, x, y, (int)in_f, (int)out_f, (int)m, true, nullptr, nullptr, nullptr, 0, 0.0f, nullptr, nullptr, 0.0f, nullptr, 0, MoeRoute{}, stream); break;
    case 30: launch_row_dots<30>(w, x, y, (int)in_f, (int)out_f, (int)m, true, nullptr, nullptr, nullptr, 0, 0.0f, nullptr, nullptr, 0.0f, nullptr, 0, MoeRoute{}, stream); break;
    default: return false;
    }
    return hipGetLastError() == hipSuccess;
}

// A row into quad-major order (the expert input when it is not the row the router reads).
__global__ __launch_bounds__(256) void moe_quad_major_kernel(const float* __restrict__ x, float* __restrict__ xt, int ne,
                                                            int q6k) {
    const int e = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (e >= ne) return;
    int u, q;
    if (q6k) quad_place_q6k(e, u, q);
    else quad_place_linear(e, u, q);
    *reinterpret_cast<v4f*>(xt + ((size_t)q * (ne / 64) + u) * 4) = *reinterpret_cast<const v4f*>(x + e);
}

size_t moe_workspace_bytes(const MoeShape& s) {
    const size_t pairs = (size_t)s.rows * s.n_used;
    size_t n = 0;
    auto add = [&n](size_t bytes) { n += (bytes + 255) / 256 * 256; };
    add(4);                                       // router ticket (first: zero between ops)
    add((size_t)s.rows * s.n_expert * 4);        // logits
    add(pairs * 4);                               // sel_idx
    add(pairs * 4);                               // sel_w
    add(pairs * s.n_ff * 4);                      // gate out / act (rows == 1: act)
    add(pairs * s.n_ff * 4);                      // up out
    add(pairs * s.ne * 4);                        // per-pair down outputs
    const size_t qmax = std::max((size_t)s.rows * s.ne, pairs * s.n_ff);
    add(qmax);                                    // int8 activations
    add(qmax / 32 * 4);                           // d (sized for either quantizer)
    add(qmax / 32 * 4);                           // bsums
    add(qmax / 16 * 4);                           // bsums16
    add(qmax);                                    // per-32 int8 activations (Q5_0 banks)
    add(qmax / 32 * 4);                           // their d
    add(qmax / 32 * 4);                           // their bsums
    const size_t max_tiles = pairs / 32 + std::min((size_t)s.n_expert, pairs);
    add(4);                                       // n_tiles
    add(pairs * 4);                               // perm
    add(max_tiles * 4);                           // tile expert
    add(max_tiles * 4);                           // tile slot0
    add(max_tiles * 4);                           // tile count
    return n;
}

const char* launch_moe_ffn(const MoeShape& shape, const MoeBuffers& bufs, void* ws, hipStream_t stream) {
    MoeShape s = shape;
    MoeBuffers b = bufs;
    const MoeRoute& rt = s.route;
    const MoeAct& ma = s.act;
    if (s.fused_gate_up) {
        // [gate rows | up rows] inside each expert's slice (graph.rs:936-941): the up bank is the
        // gate bank from row n_ff of every slice on, same format and expert stride
        s.up_dtype = s.gate_dtype;
        b.up_stride = b.gate_stride;
    }
    if (ma.act < 0 || ma.act > 2 || rt.gating < 0 || rt.gating > 2) return "unknown activation or gating";
    if (ma.has_clamp && (ma.act == 2 || ma.weight_before)) return "swiglu_clamp with Sigmoid or weight_before (the CPU arm asserts against it)";
    if (rt.ids && (rt.bias || rt.n_groups > 1)) return "expert_ids with exp_probs_b or expert groups (the CPU arm asserts against it)";
    if (rt.n_groups > 1 && rt.n_groups_used > 0 &&
        (rt.n_groups > 64 || s.n_expert % rt.n_groups != 0 || rt.n_groups_used > rt.n_groups))
        return "expert groups: n_expert must be a multiple of at most 64 groups, groups_used <= groups";
    if (s.router_dtype != 0 && s.router_dtype != 1 && s.router_dtype != 30) return "router dtype must be F32, F16 or BF16";
    if (b.norm_w && (s.rows != 1 || b.x != b.norm_dst)) return "an absorbed RmsNorm needs a single row read from its dst";
    if (s.n_used > 64 || s.n_expert > 1024 || s.n_used > s.n_expert) return "n_used <= 64 and n_expert <= 1024 required";
    if (s.ne % 256 != 0 || s.n_ff % 256 != 0) return "ne and n_ff_exp must be multiples of 256";
    const size_t pairs = (size_t)s.rows * s.n_used;
    uint8_t* p = static_cast<uint8_t*>(ws);
    auto take = [&p](size_t bytes) {
        uint8_t* r = p;
        p += (bytes + 255) / 256 * 256;
        return r;
    };
    int* tickets = (int*)take(4);
    float* logits = (float*)take((size_t)s.rows * s.n_expert * 4);
    int32_t* sel_idx = (int32_t*)take(pairs * 4);
    float* sel_w = (float*)take(pairs * 4);
    float* gbuf = (float*)take(pairs * s.n_ff * 4);
    float* ubuf = (float*)take(pairs * s.n_ff * 4);
    float* yp = (float*)take(pairs * s.ne * 4);
    const size_t qmax = std::max((size_t)s.rows * s.ne, pairs * s.n_ff);
    ActQ8 aq;
    aq.qs = (int8_t*)take(qmax);
    aq.d = (float*)take(qmax / 32 * 4);
    aq.bsums = (int32_t*)take(qmax / 32 * 4);
    aq.bsums16 = (int32_t*)take(qmax / 16 * 4);
    ActQ8 aq32;
    aq32.qs = (int8_t*)take(qmax);
    aq32.d = (float*)take(qmax / 32 * 4);
    aq32.bsums = (int32_t*)take(qmax / 32 * 4);
    aq32.bsums16 = nullptr;
    const size_t max_tiles = pairs / 32 + std::min((size_t)s.n_expert, pairs);
    int32_t* n_tiles = (int32_t*)take(4);
    int32_t* perm = (int32_t*)take(pairs * 4);
    int32_t* tile_expert = (int32_t*)take(max_tiles * 4);
    int32_t* tile_slot0 = (int32_t*)take(max_tiles * 4);
    int32_t* tile_count = (int32_t*)take(max_tiles * 4);

    // One row in the formats of the factored kernels: the gate / up kernel selects in its own
    // prologue, so the router only leaves the logits - one expert per workgroup, nothing to wait for.
    auto raw_ok = [](int dt) { return dt == 12 || dt == 13 || dt == 14 || dt == 8; };
    const bool fast1 = s.rows == 1 && raw_ok(s.gate_dtype) && s.up_dtype == s.gate_dtype && raw_ok(s.down_dtype);
    // (one token on the factored kernels: the router's first workgroup also leaves the row
    // quad-major for them, in the space of the per-pair down outputs that path does not use)
    float* xt = fast1 ? yp : nullptr;
    const bool router_row_is_x = b.x == b.router_x || b.norm_w;
    if (fast1 && !router_row_is_x)
        hipLaunchKernelGGL(moe_quad_major_kernel, dim3((unsigned)((s.ne / 4 + 255) / 256)), dim3(256), 0, stream, b.x, xt,
                           s.ne, s.gate_dtype == 14 ? 1 : 0);
    float* router_xt = router_row_is_x ? xt : nullptr;
    switch (s.router_dtype) {
    case 0: launch_row_dots<0>(b.router, b.router_x, logits, s.ne, s.n_expert, s.rows, fast1, tickets, sel_idx, sel_w, s.n_used, s.scale, b.norm_w, b.norm_dst, b.norm_eps, router_xt, s.gate_dtype == 14 ? 1 : 0, rt, stream); break;
    case 1: launch_row_dots<1>(b.router, b.router_x, logits, s.ne, s.n_expert, s.rows, fast1, tickets, sel_idx, sel_w, s.n_used, s.scale, b.norm_w, b.norm_dst, b.norm_eps, router_xt, s.gate_dtype == 14 ? 1 : 0, rt, stream); break;
    default: launch_row_dots<30>(b.router, b.router_x, logits, s.ne, s.n_expert, s.rows, fast1, tickets, sel_idx, sel_w, s.n_used, s.scale, b.norm_w, b.norm_dst, b.norm_eps, router_xt, s.gate_dtype == 14 ? 1 : 0, rt, stream); break;
    }
    auto bytes_per_row = [](int dtype, size_t in_f) -> size_t {
        switch (dtype) {
        case 12: return in_f / 256 * 144;
        case 13: return in_f / 256 * 176;
        case 10: return in_f / 256 * 84;
        case 11: return in_f / 256 * 110;
        case 23: return in_f / 256 * 136;
        case 34: return in_f / 256 * 54;
        case 35: return in_f / 256 * 66;
        case 39: return in_f / 32 * 17;
        case 40: return in_f / 64 * 36;
        case 14: return in_f / 256 * 210;
        case 8: return in_f / 32 * 34;
        case 2: case 20: return in_f / 32 * 18;
        case 3: return in_f / 32 * 20;
        case 6: return in_f / 32 * 22;
        case 7: return in_f / 32 * 24;
        case 42: return in_f / 64 * 18;
        case 0: return in_f * 4;
        case 1: case 30: return in_f * 2;
        default: return 0;
        }
    };
    const size_t gbpr = bytes_per_row(s.gate_dtype, s.ne), ubpr = bytes_per_row(s.up_dtype, s.ne);
    const size_t dbpr = bytes_per_row(s.down_dtype, s.n_ff);
    if (!gbpr || !ubpr || !dbpr) return "expert bank format has no kernel";
    if (s.fused_gate_up) b.up = b.gate + (size_t)s.n_ff * gbpr;
    const int unit_w = ma.weight_before ? 1 : 0;
    // expert_acts_kind (moe.rs:42-53) with whole-256 rows: per-256 int8 activations (Super) for the
    // K-quants and Q8_0, per-32 (Blk32) for Q5_0, f32 rows (Raw) for everything else - and for
    // every bank when there is a single row (int8_ok = rows >= 2, lib.rs:2359).
    enum { kSuper = 0, kBlk32 = 1, kRaw = 2 };
    auto acts_kind = [&](int dt) {
        if (s.rows < 2) return (int)kRaw;
        return dt == 12 || dt == 13 || dt == 14 || dt == 8 ? (int)kSuper : (dt == 6 ? (int)kBlk32 : (int)kRaw);
    };
    const int kg = acts_kind(s.gate_dtype), ku = acts_kind(s.up_dtype), kd = acts_kind(s.down_dtype);
    auto launch_raw = [&](int dt, const uint8_t* bank, size_t stride, size_t bpr_, const float* acts, int act_div,
                          size_t in_f, float* out, size_t out_f) {
        hipLaunchKernelGGL(moe_raw_dot_kernel, dim3((unsigned)((out_f + 31) / 32), (unsigned)pairs), dim3(256), 0,
                           stream, dt, bank, stride, bpr_, sel_idx, acts, act_div, (int)in_f, out, (int)out_f);
    };
    // the expert input is quantized per 256 by the selection kernel's workgroups (one per row)
    const bool quant_in_select = s.rows > 1 && (kg == kSuper || ku == kSuper);
    if (s.rows > 1)
        hipLaunchKernelGGL(moe_select_kernel, dim3((unsigned)s.rows), dim3(256), 0, stream, logits, sel_idx,
                           sel_w, s.n_expert, s.n_used, s.scale, quant_in_select ? b.x : (const float*)nullptr,
                           s.ne, aq.qs, aq.d, aq.bsums, aq.bsums16, rt);
    auto export_selection = [&] {
        if (b.sel_idx) (void)hipMemcpyAsync(b.sel_idx, sel_idx, pairs * 4, hipMemcpyDeviceToDevice, stream);
        if (b.sel_w) (void)hipMemcpyAsync(b.sel_w, sel_w, pairs * 4, hipMemcpyDeviceToDevice, stream);
    };
    if (!fast1) export_selection();

    if (s.rows == 1) {
        // ActsKind::Raw for every bank (lib.rs:2359: int8_ok = rows >= 2)
        if (!fast1) {
            // other formats, mixed gate / up formats: the decode-and-dot form of every stage
            launch_raw(s.gate_dtype, b.gate, b.gate_stride, gbpr, b.x, s.n_used, s.ne, gbuf, s.n_ff);
            launch_raw(s.up_dtype, b.up, b.up_stride, ubpr, b.x, s.n_used, s.ne, ubuf, s.n_ff);
            const size_t n_act1 = pairs * s.n_ff;
            hipLaunchKernelGGL(moe_act_f32_kernel, dim3((unsigned)((n_act1 / 4 + 255) / 256)), dim3(256), 0, stream,
                               gbuf, ubuf, n_act1, s.n_ff, ma, sel_w);
            launch_raw(s.down_dtype, b.down, b.down_stride, dbpr, gbuf, 1, s.n_ff, yp, s.ne);
            hipLaunchKernelGGL(moe_accumulate_kernel, dim3((unsigned)((s.ne + 255) / 256)), dim3(256), 0, stream, yp,
                               sel_w, b.dst, b.add_b, b.add_dst, s.ne, s.n_used, s.rows, unit_w, b.down_scale, sel_idx);
            return hipGetLastError() == hipSuccess ? nullptr : "kernel launch failed";
        }
        // row steps per wave: amortise the 64 activation registers while keeping >= ~1024 waves
        auto steps_per_wave = [](int wave_steps) { return std::max(1, std::min(4, wave_steps / kMoeWavesWanted)); };
        // lanes per weight row: every 64-weight unit its own lane up to 4096 columns; longer rows
        // in rounds of the widest lane count that divides the units and leaves at most 8 lanes idle
        auto row_lanes = [](int units) {
            if (units <= 64) return units;
            int l = 64;
            while (units % l != 0 || 64 / l * l < 56) l -= 4;
            return l;
        };
        const int lanes_g = row_lanes(s.ne / 64), chunks_g = s.ne / 64 / lanes_g;
        const int rps_g = 64 / lanes_g;
        const int steps_g = (s.n_ff + rps_g - 1) / rps_g;
        // (Q8_0 rows are 1.9x the bytes of Q4_K's: four steps of gate and up rows in flight leave
        // one wave per SIMD, two steps three)
        int spw = std::min(s.gate_dtype == 8 ? 2 : 4, steps_per_wave(steps_g * s.n_used));
        if (s.gate_dtype == 14 && spw == 3) spw = 2;  // (three steps of Q6_K rows compile to one wave per SIMD, two to three)
        const dim3 grid_g((unsigned)((steps_g + 4 * spw - 1) / (4 * spw)), (unsigned)s.n_used);
#define INFR_GATE_UP_N(P, N)                                                                                  \
    hipLaunchKernelGGL((moe_gate_up_f32_kernel<P, N>), grid_g, dim3(256), 0, stream, b.gate, b.up, b.gate_stride, \
                       b.up_stride, logits, s.n_expert, s.n_used, s.scale, sel_idx, sel_w, xt, gbuf, s.ne, s.n_ff, \
                       lanes_g, chunks_g, s.down_dtype == 14 ? 1 : 0, rt, ma)
#define INFR_GATE_UP(P)                 \
    switch (spw) {                      \
    case 1: INFR_GATE_UP_N(P, 1); break; \
    case 2: INFR_GATE_UP_N(P, 2); break; \
    case 3: INFR_GATE_UP_N(P, 3); break; \
    default: INFR_GATE_UP_N(P, 4); break; \
    }
        if (s.gate_dtype == 12) INFR_GATE_UP(RawQ4K)
        else if (s.gate_dtype == 13) INFR_GATE_UP(RawQ5K)
        else if (s.gate_dtype == 14) INFR_GATE_UP(RawQ6K)
        else INFR_GATE_UP(RawQ8_0)
#undef INFR_GATE_UP
#undef INFR_GATE_UP_N
        export_selection();
        const int lanes_d = row_lanes(s.n_ff / 64), chunks_d = s.n_ff / 64 / lanes_d;
        const int rps_d = 64 / lanes_d;
        const int steps_d = (s.ne + rps_d - 1) / rps_d;
        const int spw_d = std::min(kDownMaxSteps, steps_per_wave(steps_d * s.n_used));
        const int nw_d = std::min(s.n_used, kDownMaxWaves);
        const dim3 grid_d((unsigned)((steps_d + spw_d - 1) / spw_d));
#define INFR_DOWN_N(P, N)                                                                                   \
    hipLaunchKernelGGL((moe_down_f32_kernel<P, N>), grid_d, dim3((unsigned)(64 * nw_d)), 0, stream, b.down,   \
                       b.down_stride, sel_idx, sel_w, gbuf, b.dst, b.add_b, b.add_dst, s.n_ff, s.ne, s.n_used, \
                       lanes_d, chunks_d, unit_w, b.down_scale)
#define INFR_DOWN(P)                 \
    switch (spw_d) {                 \
    case 1: INFR_DOWN_N(P, 1); break; \
    case 2: INFR_DOWN_N(P, 2); break; \
    case 3: INFR_DOWN_N(P, 3); break; \
    default: INFR_DOWN_N(P, 4); break; \
    }
        if (s.down_dtype == 12) INFR_DOWN(RawQ4K)
        else if (s.down_dtype == 13) INFR_DOWN(RawQ5K)
        else if (s.down_dtype == 14) INFR_DOWN(RawQ6K)
        else INFR_DOWN(RawQ8_0)
#undef INFR_DOWN
#undef INFR_DOWN_N
        return hipGetLastError() == hipSuccess ? nullptr : "kernel launch failed";
    }

    // rows >= 2
    if ((kg == kSuper || ku == kSuper) && !quant_in_select) launch_quantize_q8(b.x, s.rows, s.ne, false, aq, stream);
    if (kg == kBlk32 || ku == kBlk32) launch_quantize_q8(b.x, s.rows, s.ne, true, aq32, stream);
    const size_t n_act = pairs * s.n_ff, n_out = (size_t)s.rows * s.ne;
    // Prefill-sized batches: the pairs are bucketed by expert and every bank runs its format's
    // int8-MFMA GEMM per (expert, 32 pairs) tile, so an expert's weights are read once per 32 of
    // its pairs instead of once per pair. From an average of `bucket_min` pairs per expert up: the
    // tiles' time is flat in the number of pairs there (Q4_K banks, 128 experts, top-8: 125-130 us per
    // layer from 32 to 96 tokens) while the per-pair GEMVs grow by ~2.6 us per token (126 us at 32
    // tokens, 168 at 48); with one pair per expert the tiles lose (103 against 87 us at 16 tokens).
    constexpr int bucket_min = 2;
    // (a Q6_K tile costs more than the others': at four pairs per expert its per-pair GEMVs tie with
    // the tiles, 313 us per layer either way, so it is bucketed from four)
    auto has_mfma = [&](int dt) {
        return ((dt == 12 || dt == 13 || dt == 8) && pairs >= (size_t)bucket_min * s.n_expert) ||
               (dt == 14 && pairs >= (size_t)2 * bucket_min * s.n_expert);
    };
    auto launch_gathered = [&](int dt, const uint8_t* bank, size_t stride, size_t bpr_, int act_div, const MoeTileTable& t,
                               float* out, size_t in_f, size_t out_f) {
        (void)launch_mmq_gathered(dt, bank, stride, bpr_, aq, act_div, t, out, in_f, out_f, stream);
    };
    const bool bucketed = bucket_min > 0 && pairs >= (size_t)bucket_min * s.n_expert && pairs <= (size_t)1 << 24 &&
                          (has_mfma(s.gate_dtype) || has_mfma(s.up_dtype) || has_mfma(s.down_dtype));
    const MoeTileTable tt{n_tiles, tile_expert, tile_slot0, tile_count, perm, (int)max_tiles};
    if (bucketed)
        hipLaunchKernelGGL(moe_bucket_kernel, dim3(1), dim3(kBucketThreads), 0, stream, sel_idx, (int)pairs,
                           s.n_expert, perm, tile_expert, tile_slot0, tile_count, n_tiles);
    const bool gate_mfma = bucketed && has_mfma(s.gate_dtype), up_mfma = bucketed && has_mfma(s.up_dtype);
    if (gate_mfma) launch_gathered(s.gate_dtype, b.gate, b.gate_stride, gbpr, s.n_used, tt, gbuf, s.ne, s.n_ff);
    if (up_mfma) launch_gathered(s.up_dtype, b.up, b.up_stride, ubpr, s.n_used, tt, ubuf, s.ne, s.n_ff);
    bool gate_up_ok = true;
    if (!gate_mfma && !up_mfma && s.gate_dtype == s.up_dtype && kg != kRaw) {
        gate_up_ok = launch_gemv_id(s.gate_dtype, b.gate, b.gate_stride, gbpr, sel_idx, kg == kBlk32 ? aq32 : aq, s.ne,
                                    s.n_used, (int)pairs, gbuf, s.n_ff, stream, b.up, b.up_stride, ubuf);
    } else {
        if (kg == kRaw)
            launch_raw(s.gate_dtype, b.gate, b.gate_stride, gbpr, b.x, s.n_used, s.ne, gbuf, s.n_ff);
        else if (!gate_mfma)
            gate_up_ok = launch_gemv_id(s.gate_dtype, b.gate, b.gate_stride, gbpr, sel_idx, kg == kBlk32 ? aq32 : aq,
                                        s.ne, s.n_used, (int)pairs, gbuf, s.n_ff, stream);
        if (ku == kRaw)
            launch_raw(s.up_dtype, b.up, b.up_stride, ubpr, b.x, s.n_used, s.ne, ubuf, s.n_ff);
        else if (!up_mfma)
            gate_up_ok = gate_up_ok && launch_gemv_id(s.up_dtype, b.up, b.up_stride, ubpr, sel_idx,
                                                      ku == kBlk32 ? aq32 : aq, s.ne, s.n_used, (int)pairs, ubuf,
                                                      s.n_ff, stream);
    }
    if (!gate_up_ok) return "no id-gathered kernel for this gate/up shape";
    // a few rows: activation, down projection and the sum over a token's experts in one launch
    if (kd == kSuper && !(bucketed && has_mfma(s.down_dtype)) &&
        launch_moe_down_fused(s.down_dtype, b.down, b.down_stride, dbpr, sel_idx, sel_w, gbuf, ubuf, b.dst, b.add_b,
                              b.add_dst, s.n_ff, s.ne, s.n_used, s.rows, ma, b.down_scale, stream))
        return hipGetLastError() == hipSuccess ? nullptr : "kernel launch failed";
    // act = silu(g) * u in the form the down bank multiplies: per-256 codes, per-32 codes, or f32
    if (kd == kSuper)
        hipLaunchKernelGGL(moe_act_quant_kernel<false>, dim3((unsigned)((n_act / 256 + 3) / 4)), dim3(256), 0, stream,
                           gbuf, ubuf, aq.qs, aq.d, aq.bsums, aq.bsums16, n_act, s.n_ff, ma, sel_w);
    else if (kd == kBlk32)
        hipLaunchKernelGGL(moe_act_quant_kernel<true>, dim3((unsigned)((n_act / 256 + 3) / 4)), dim3(256), 0, stream,
                           gbuf, ubuf, aq32.qs, aq32.d, aq32.bsums, (int32_t*)nullptr, n_act, s.n_ff, ma, sel_w);
    else
        hipLaunchKernelGGL(moe_act_f32_kernel, dim3((unsigned)((n_act / 4 + 255) / 256)), dim3(256), 0, stream, gbuf,
                           ubuf, n_act, s.n_ff, ma, sel_w);
    // the down projection's activation row is the pair itself: n_used = 1
    if (kd == kRaw)
        launch_raw(s.down_dtype, b.down, b.down_stride, dbpr, gbuf, 1, s.n_ff, yp, s.ne);
    else if (bucketed && has_mfma(s.down_dtype))
        launch_gathered(s.down_dtype, b.down, b.down_stride, dbpr, 1, tt, yp, s.n_ff, s.ne);
    else if (!launch_gemv_id(s.down_dtype, b.down, b.down_stride, dbpr, sel_idx, kd == kBlk32 ? aq32 : aq, s.n_ff, 1,
                             (int)pairs, yp, s.ne, stream))
        return "no id-gathered kernel for this down shape";
    hipLaunchKernelGGL(moe_accumulate_kernel, dim3((unsigned)((n_out + 255) / 256)), dim3(256), 0, stream,
                       yp, sel_w, b.dst, b.add_b, b.add_dst, s.ne, s.n_used, s.rows, unit_w, b.down_scale, sel_idx);
    return hipGetLastError() == hipSuccess ? nullptr : "kernel launch failed";
}

}  // namespace infr
