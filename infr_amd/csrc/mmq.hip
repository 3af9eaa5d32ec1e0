// Prefill GEMM (m >= 2) of block-quantized weights against on-device int8-quantized activations.
//
// Q4_K runs on the int8 matrix cores. Per 256-element block infr-cpu computes, per output,
//     sd = sum_s sc_s * (sum_l q4 * q8)     sm = sum_s m_s * bsums_s
//     y += q8.d[b] * (d * (f32)sd - dmin * (f32)sm)            (crates/infr-cpu/src/kernels.rs:151-184)
// with 6-bit sc_s, m_s per 32-element sub-block. The MFMA accumulates over K inside the
// instruction, so a per-sub-block scale has to be inside the operand. q4 * sc_s needs 10 bits, so
// the scale is split sc = 8 * sc_hi + sc_lo (3 bits each): q4 * sc_lo and q4 * sc_hi both fit int8,
// two v_mfma_i32_32x32x32_i8 chains run over the whole block, and sd = lo + 8 * hi exactly.
// (The alternative, one K=32 MFMA per sub-block followed by a VALU multiply, runs the legacy
// half-rate instruction and needs eight integer multiply-adds per output per block.)
// sm is a K = 16 product of the mins with the activation's per-32 sums split as bsum = lo + 64*hi
// (both exact in f16): one v_mfma_f32_32x32x16_f16 whose f32 result is the exact integer.
// The f32 epilogue then evaluates the CPU expression with separate multiplies and adds, and each
// output accumulates its blocks in ascending order, so y is bit-identical to infr-cpu's batch
// kernel (and to this library's m == 1 GEMV).
//
// Tiling. Tokens are the MFMA's M (rows of C), weight rows its N (columns): a lane's 16
// accumulators then share one weight row, so d, dmin and the pre-scaled operand are per lane.
// A workgroup (4 waves) covers BM tokens x 128 weight rows; each wave owns 32 weight rows for all
// BM tokens, loads and unpacks its rows' blocks straight from global memory into MFMA B operands
// (no LDS for weights, no redundant unpacking), and reads the activation tile, shared by the four
// waves, from LDS. Per 256-block and 32x32 output tile: 16 int8 MFMAs + 1 f16 MFMA against
// 7 VALU instructions per output for the epilogue.
//
// This tiled kernel serves 33..127 tokens; fewer take the skinny kernel and more the shared-operand
// kernel, both further down. The other formats take the multi-activation dot4 GEMV (gemv.hip).
#include <cstdlib>

#include "device_common.hpp"
#include "gemv_formats.hpp"
#include "kernels.hpp"
#include "mmq_tiles.hpp"

namespace infr {

typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

struct Q4kRaw {
    v4i hdr, q[4];
};

__device__ __forceinline__ void q4k_load_raw(Q4kRaw& r, const uint8_t* blk, int h, bool ok) {
    if (ok) {
        r.hdr = load16(blk);
#pragma unroll
        for (int p = 0; p < 4; ++p) r.q[p] = load16(blk + 16 + p * 32 + h * 16);
    } else {
        r.hdr = v4i{0, 0, 0, 0};
#pragma unroll
        for (int p = 0; p < 4; ++p) r.q[p] = v4i{0, 0, 0, 0};
    }
}

// Packed byte-wise multiply of four codes (<= 15) by a scale digit (<= 7): no byte overflows, so
// two 16-bit lane multiplies do it.
__device__ __forceinline__ int scale_codes(uint32_t codes, uint32_t digit) {
    typedef unsigned short us2 __attribute__((ext_vector_type(2)));
    const us2 c = __builtin_bit_cast(us2, codes);
    const us2 s = {(unsigned short)digit, (unsigned short)digit};
    return __builtin_bit_cast(int, (us2)(c * s));
}

template <int BM, bool STAGES, typename TILES>
__global__ __launch_bounds__(256) void mmq_q4k_kernel(const uint8_t* __restrict__ w, size_t bpr,
                                                      const int8_t* __restrict__ qs,
                                                      const float* __restrict__ d8,
                                                      const int32_t* __restrict__ bsums,
                                                      float* __restrict__ y, TILES tiles, int out_f, int nb,
                                                      int32_t* __restrict__ st_sd,
                                                      int32_t* __restrict__ st_sm) {
    constexpr int TB = BM / 32;  // token blocks of 32
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];  // two MmqLds<BM> buffers
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, h = lane >> 5;
    const int tile_y = blockIdx.y;
    size_t w_off = 0;
    if (!tiles.select(tile_y, w_off)) return;  // uniform over the workgroup, before any barrier
    const int n_slots = tiles.count(tile_y, BM);
    const int tok0 = tile_y * BM;  // dense tiles only (the integer stages)
    const int wrow = blockIdx.x * 128 + wave * 32 + col;
    const bool row_ok = wrow < out_f;
    const uint8_t* wrowp = w + w_off + (size_t)(row_ok ? wrow : 0) * bpr;

    v16f acc[TB];
#pragma unroll
    for (int tb = 0; tb < TB; ++tb)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[tb][i] = 0.0f;

    ActStage<BM> stage;
    stage.resolve(tid, [&](int t) { return tiles.act_row(tile_y, BM, t); });
    stage.fetch(qs, d8, bsums, nb, 0, tid);
    Q4kRaw raw;
    q4k_load_raw(raw, wrowp, h, row_ok);
    stage.store(lds, tid);
    __syncthreads();

    for (int b = 0; b < nb; ++b) {
        const uint8_t* tile = lds + (b & 1) * MmqLds<BM>::bytes;
        // ---- request block b+1: activation tile into registers, this wave's weight rows ----
        const Q4kRaw cur = raw;
        if (b + 1 < nb) {
            stage.fetch(qs, d8, bsums, nb, b + 1, tid);
            q4k_load_raw(raw, wrowp + (size_t)(b + 1) * 144, h, row_ok);
        }

        // ---- this wave's 32 weight rows of block b -> MFMA B operands (registers) ----
        uint32_t sc8[2], mn8[2];
        k4_all((uint32_t)cur.hdr.y, (uint32_t)cur.hdr.z, (uint32_t)cur.hdr.w, sc8, mn8);
        const float d = f16_bits_to_f32((uint32_t)cur.hdr.x & 0xFFFFu);
        const float dmin = f16_bits_to_f32((uint32_t)cur.hdr.x >> 16);
        v4i blo[8], bhi[8];
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const int qw[4] = {cur.q[p].x, cur.q[p].y, cur.q[p].z, cur.q[p].w};
#pragma unroll
            for (int e = 0; e < 2; ++e) {  // e = 0: sub-block 2p (low nibbles), 1: 2p+1 (high)
                const int s = 2 * p + e;
                const uint32_t sc = (sc8[s >> 2] >> (8 * (s & 3))) & 0xFFu;
                const uint32_t lo3 = sc & 7u, hi3 = sc >> 3;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t codes = ((uint32_t)qw[k] >> (4 * e)) & 0x0F0F0F0Fu;
                    blo[s][k] = scale_codes(codes, lo3);
                    bhi[s][k] = scale_codes(codes, hi3);
                }
            }
        }
        // mins as f16 for the K=16 product: k-slots 0..7 pair with bsum lo, 8..15 with 64*hi
        v8h bm;
#pragma unroll
        for (int s = 0; s < 8; ++s) bm[s] = (_Float16)(int)((mn8[s >> 2] >> (8 * (s & 3))) & 0xFFu);

#pragma unroll
        for (int tb = 0; tb < TB; ++tb) {
            const v16i zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            const v16f zf = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            const uint8_t* arow = tile + MmqLds<BM>::qs_off + (tb * 32 + col) * kActRowBytes + h * 16;
            v4i a = *reinterpret_cast<const v4i*>(arow);
            v16i alo = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, blo[0], zi, 0, 0, 0);
            v16i ahi = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, bhi[0], zi, 0, 0, 0);
#pragma unroll
            for (int s = 1; s < 8; ++s) {
                a = *reinterpret_cast<const v4i*>(arow + s * 32);
                alo = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, blo[s], alo, 0, 0, 0);
                ahi = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, bhi[s], ahi, 0, 0, 0);
            }
            const v8h abs_ = *reinterpret_cast<const v8h*>(tile + MmqLds<BM>::bs_off + (tb * 32 + col) * 32 + h * 16);
            const v16f smf = __builtin_amdgcn_mfma_f32_32x32x16_f16(abs_, bm, zf, 0, 0, 0);
            // epilogue: accumulator i of this lane is token 8*(i/4) + 4*h + i%4 of the block
            const float* dtile = reinterpret_cast<const float*>(tile + MmqLds<BM>::d_off) + tb * 32 + 4 * h;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const v4f dq = *reinterpret_cast<const v4f*>(dtile + 8 * j);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int r = 4 * j + i;
                    const int sd = alo[r] + (ahi[r] << 3);
                    if (STAGES) {
                        const int slot = tb * 32 + 8 * j + 4 * h + i, tok = tok0 + slot;
                        if (row_ok && slot < n_slots) {
                            st_sd[((size_t)tok * out_f + wrow) * nb + b] = sd;
                            st_sm[((size_t)tok * out_f + wrow) * nb + b] = (int)smf[r];
                        }
                    }
                    // sumf += q8.d[b] * (d * sd as f32 - dmin * sm as f32)
                    acc[tb][r] += dq[i] * (d * (float)sd - dmin * smf[r]);
                }
            }
        }

        // ---- publish block b+1 in the other buffer (its last readers passed the previous barrier)
        if (b + 1 < nb) stage.store(lds + ((b + 1) & 1) * MmqLds<BM>::bytes, tid);
        __syncthreads();
    }

    if (!row_ok) return;
#pragma unroll
    for (int tb = 0; tb < TB; ++tb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int slot = tb * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
            if (slot < n_slots) y[(size_t)tiles.out_row(tile_y, BM, slot) * out_f + wrow] = acc[tb][r];
        }
}

// ───────────────────────────── shared-operand form: 128 tokens x 32*T rows per workgroup ─────────────────────────────
// The tiled kernel above unpacks a weight block once per 32*TB tokens and is bound by that VALU
// work. Here the four waves of a workgroup own 32 tokens each and share the unpacked rows through
// LDS: wave w unpacks nibble pair w (sub-blocks 2w, 2w+1) of every row of the block - a quarter of
// the work - into MFMA B-operand order, double-buffered so that block b+1 is unpacked while block
// b is multiplied, one barrier per block. The unpack cost per 32x32 output tile falls from ~250
// (or ~125 at 64-token tiles) to ~60 VALU instructions, each wave carries one or two accumulator
// tiles only, and the activation fragments go from global memory (L2) straight to registers.
// Integers, epilogue expression and block order are those of the tiled kernel: same bits.
template <int T>
struct SharedLds {
    static constexpr int b_bytes = 8 * 2 * T * 1024;   // [sub-block][plane][row tile][lane] x 16 B
    static constexpr int mn_off = b_bytes;             // [row tile][row][8] f16 mins
    static constexpr int dd_off = mn_off + T * 32 * 16;  // [row tile][row] (d, dmin)
    static constexpr int bytes = dd_off + T * 32 * 8;
};

template <int T, bool STAGES, int NW = 4>
__global__ __launch_bounds__(NW * 64) void mmq_shared_q4k_kernel(
    const uint8_t* __restrict__ w, size_t bpr, const int8_t* __restrict__ qs,
    const float* __restrict__ d8, const _Float16* __restrict__ bsh, float* __restrict__ y, int m,
    int out_f, int nb, int32_t* __restrict__ st_sd, int32_t* __restrict__ st_sm) {
    typedef SharedLds<T> L;
    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * L::bytes];
    __shared__ __attribute__((aligned(16))) float dql[NW][32];  // per wave: its tokens' activation scales
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, h = lane >> 5;
    const int tok0 = blockIdx.y * (32 * NW) + wave * 32;
    const int row0 = blockIdx.x * (32 * T);
    // the nibble pair this wave unpacks; with eight waves (T = 2) the upper four take the second
    // row tile, so a wave unpacks one tile's pair instead of both
    static_assert(NW == 4 || (NW == 8 && T == 2), "eight waves split the unpack of two row tiles");
    const int p = wave & 3;
    constexpr int TU = NW == 8 ? 1 : T;      // row tiles a wave unpacks
    const int tu0 = NW == 8 ? wave >> 2 : 0;  // the first of them

    const uint8_t* wrowp[T];
    bool row_ok[T];
#pragma unroll
    for (int t = 0; t < T; ++t) {
        row_ok[t] = row0 + 32 * t + col < out_f;
        wrowp[t] = w + (size_t)(row_ok[t] ? row0 + 32 * t + col : 0) * bpr;
    }
    v16f acc[T];
#pragma unroll
    for (int t = 0; t < T; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[t][i] = 0.0f;

    v4i hdr[TU], qv[TU];  // raw bytes of the block to unpack next
    const uint8_t* urowp[TU];
#pragma unroll
    for (int u = 0; u < TU; ++u) urowp[u] = NW == 8 ? (tu0 ? wrowp[T - 1] : wrowp[0]) : wrowp[u];
    auto request_rows = [&](int b) {
#pragma unroll
        for (int u = 0; u < TU; ++u) {
            const uint8_t* blk = urowp[u] + (size_t)b * 144;
            hdr[u] = load16(blk);
            qv[u] = load16(blk + 16 + p * 32 + h * 16);
        }
    };
    auto unpack_to = [&](uint8_t* buf) {
#pragma unroll
        for (int u = 0; u < TU; ++u) {
            const int t = tu0 + u;
            uint32_t sc8[2], mn8[2];
            k4_all((uint32_t)hdr[u].y, (uint32_t)hdr[u].z, (uint32_t)hdr[u].w, sc8, mn8);
            const uint32_t scw = (p & 2) ? sc8[1] : sc8[0], mnw = (p & 2) ? mn8[1] : mn8[0];
            const int sh = (p & 1) * 16;
            const int qw[4] = {qv[u].x, qv[u].y, qv[u].z, qv[u].w};
#pragma unroll
            for (int e = 0; e < 2; ++e) {  // e = 0: sub-block 2p (low nibbles), 1: 2p+1 (high)
                const uint32_t sc = (scw >> (sh + 8 * e)) & 0xFFu;
                const uint32_t lo3 = sc & 7u, hi3 = sc >> 3;
                v4i blo, bhi;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t codes = ((uint32_t)qw[k] >> (4 * e)) & 0x0F0F0F0Fu;
                    blo[k] = scale_codes(codes, lo3);
                    bhi[k] = scale_codes(codes, hi3);
                }
                uint8_t* dst = buf + (size_t)(((2 * p + e) * 2) * T + t) * 1024 + lane * 16;
                *reinterpret_cast<v4i*>(dst) = blo;
                *reinterpret_cast<v4i*>(dst + T * 1024) = bhi;
            }
            if (h == 0) {
                // the two mins of this pair as f16, k-slots 2p and 2p+1 of the row's eight
                typedef _Float16 h2 __attribute__((ext_vector_type(2)));
                const h2 mn = {(_Float16)(int)((mnw >> sh) & 0xFFu), (_Float16)(int)((mnw >> (sh + 8)) & 0xFFu)};
                *reinterpret_cast<h2*>(buf + L::mn_off + (t * 32 + col) * 16 + p * 4) = mn;
                if (p == 0) {
                    float* dd = reinterpret_cast<float*>(buf + L::dd_off) + (t * 32 + col) * 2;
                    dd[0] = f16_bits_to_f32((uint32_t)hdr[u].x & 0xFFFFu);
                    dd[1] = f16_bits_to_f32((uint32_t)hdr[u].x >> 16);
                }
            }
        }
    };
    // activation fragments in the tiled quantizer's order: every load is a contiguous kilobyte
    v4i a[8];
    v8h abs_;  // split per-32 sums: the h = 0 lanes carry bsum & 63, the h = 1 lanes the rest
    float dtok;
    // this wave's group of 32 tokens; a wave wholly past m recomputes the last group (nothing is stored)
    const size_t g = min((size_t)blockIdx.y * NW + wave, (size_t)(m - 1) / 32);
    auto request_acts = [&](int b) {
        const size_t gb = g * nb + b;
        const int8_t* ap = qs + gb * (8 * 1024) + lane * 16;
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) a[sb] = *reinterpret_cast<const v4i*>(ap + sb * 1024);
        abs_ = *reinterpret_cast<const v8h*>(bsh + (gb * 64 + lane) * 8);
        dtok = d8[gb * 32 + col];
    };

    // Requests past the last block are clamped to it (redundant loads, never consumed) so that the
    // loop body is straight-line code and every wait covers exactly the loads it needs.
    // The prologue leaves the same loads pending, in the same order (weight rows older than the
    // activation fragments), as the loop's back edge does.
    request_rows(0);
    unpack_to(lds);
    request_rows(min(1, nb - 1));
    request_acts(0);
    __syncthreads();

    for (int b = 0; b < nb; ++b) {
        const uint8_t* cur = lds + (b & 1) * L::bytes;
        // ---- unpack block b+1 into the other buffer, then ask for block b+2's bytes ----
        unpack_to(lds + ((b + 1) & 1) * L::bytes);
        request_rows(min(b + 2, nb - 1));
        // ---- this wave's 32 tokens of block b ----
        const v8h abs_b = abs_;
        if (h == 0) dql[wave][col] = dtok;
        v16i alo[T], ahi[T];
        const v16i zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        const v16f zf = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        __builtin_amdgcn_s_setprio(1);  // matrix work first: the other waves' VALU fills the gaps
        // B fragments run one sub-block ahead of the MFMAs that consume them
        v4i flo[T], fhi[T];
#pragma unroll
        for (int t = 0; t < T; ++t) {
            const uint8_t* src = cur + (size_t)t * 1024 + lane * 16;
            flo[t] = *reinterpret_cast<const v4i*>(src);
            fhi[t] = *reinterpret_cast<const v4i*>(src + T * 1024);
        }
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) {
            v4i nlo[T], nhi[T];
            if (sb < 7) {
#pragma unroll
                for (int t = 0; t < T; ++t) {
                    const uint8_t* src = cur + (size_t)(((sb + 1) * 2) * T + t) * 1024 + lane * 16;
                    nlo[t] = *reinterpret_cast<const v4i*>(src);
                    nhi[t] = *reinterpret_cast<const v4i*>(src + T * 1024);
                }
            }
#pragma unroll
            for (int t = 0; t < T; ++t) {
                alo[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[sb], flo[t], sb ? alo[t] : zi, 0, 0, 0);
                ahi[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[sb], fhi[t], sb ? ahi[t] : zi, 0, 0, 0);
            }
            if (sb < 7) {
#pragma unroll
                for (int t = 0; t < T; ++t) {
                    flo[t] = nlo[t];
                    fhi[t] = nhi[t];
                }
            }
        }
        // issue order: the LDS reads of sub-block s+1 go out before the MFMAs of sub-block s
        __builtin_amdgcn_sched_group_barrier(0x100, 2 * T, 0);
#pragma unroll
        for (int sb = 0; sb < 7; ++sb) {
            __builtin_amdgcn_sched_group_barrier(0x100, 2 * T, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 2 * T, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 2 * T, 0);
        __builtin_amdgcn_s_setprio(0);
        // the activation registers are free: fetch block b+1 while the epilogue runs
        const int b_this = b;
        request_acts(min(b + 1, nb - 1));
#pragma unroll
        for (int t = 0; t < T; ++t) {
            const v8h bm = *reinterpret_cast<const v8h*>(cur + L::mn_off + (t * 32 + col) * 16);
            const v16f smf = __builtin_amdgcn_mfma_f32_32x32x16_f16(abs_b, bm, zf, 0, 0, 0);
            const float* dd = reinterpret_cast<const float*>(cur + L::dd_off) + (t * 32 + col) * 2;
            const float d = dd[0], dmin = dd[1];
            const int wrow = row0 + 32 * t + col;
            // accumulator i of this lane is token 8*(i/4) + 4*h + i%4 of the wave's 32
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const v4f dq = *reinterpret_cast<const v4f*>(&dql[wave][8 * j + 4 * h]);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int r = 4 * j + i;
                    const int sd = alo[t][r] + (ahi[t][r] << 3);
                    if (STAGES) {
                        const int tok = tok0 + 8 * j + 4 * h + i;
                        if (row_ok[t] && tok < m) {
                            st_sd[((size_t)tok * out_f + wrow) * nb + b_this] = sd;
                            st_sm[((size_t)tok * out_f + wrow) * nb + b_this] = (int)smf[r];
                        }
                    }
                    // sumf += q8.d[b] * (d * sd as f32 - dmin * sm as f32)
                    acc[t][r] += dq[i] * (d * (float)sd - dmin * smf[r]);
                }
            }
        }
        __syncthreads();
    }

#pragma unroll
    for (int t = 0; t < T; ++t) {
        if (!row_ok[t]) continue;
        const int wrow = row0 + 32 * t + col;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int tok = tok0 + 8 * (r >> 2) + 4 * h + (r & 3);
            if (tok < m) y[(size_t)tok * out_f + wrow] = acc[t][r];
        }
    }
}

template <int T, int NW = 4>
static void launch_mmq_shared_q4k(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m,
                                  size_t in_f, size_t out_f, const IntStages& st, hipStream_t stream) {
    const dim3 grid((unsigned)((out_f + 32 * T - 1) / (32 * T)), (unsigned)((m + 32 * NW - 1) / (32 * NW))), block(NW * 64);
    const int nb = (int)(in_f / 256);
    if (st.a)
        hipLaunchKernelGGL((mmq_shared_q4k_kernel<T, true, NW>), grid, block, 0, stream, w, bpr, act.qs, act.d,
                           reinterpret_cast<const _Float16*>(act.bsums), y, (int)m, (int)out_f, nb, st.a, st.b);
    else
        hipLaunchKernelGGL((mmq_shared_q4k_kernel<T, false, NW>), grid, block, 0, stream, w, bpr, act.qs, act.d,
                           reinterpret_cast<const _Float16*>(act.bsums), y, (int)m, (int)out_f, nb, (int32_t*)nullptr, (int32_t*)nullptr);
}

// ───────────────────────────── skinny form: up to 32 tokens per workgroup ─────────────────────────────
// With few tokens there are too few 32 x 128 output tiles to fill the chip, and a wave that walks
// all of K alone is serial for nb blocks. Here a workgroup owns 32 weight rows x 32 tokens and
// splits K over its NW waves: in every round wave w takes block round*NW + w - loads its weight
// rows and the activation fragments straight from global memory (L2), unpacks, runs the same 17
// MFMAs - and parks the exact per-block integers (sd, sm) in LDS. After a barrier all NW*64
// threads run the f32 epilogue, each for 16/NW of a lane position's outputs, walking the round's
// blocks in ascending order: the same operations in the same order as the CPU, so the result is
// bit-identical to the tiled kernel and the GEMV, at NW-fold K parallelism.
template <int NW, bool STAGES>
__global__ __launch_bounds__(NW * 64) void mmq_skinny_q4k_kernel(
    const uint8_t* __restrict__ w, size_t bpr, const int8_t* __restrict__ qs,
    const float* __restrict__ d8, const int32_t* __restrict__ bsums, float* y, int m,
    int out_f, int nb, int32_t* __restrict__ st_sd, int32_t* __restrict__ st_sm,
    const BatchTile* __restrict__ tiles) {
    constexpr int RG = 16 / NW;  // accumulators per epilogue thread
    typedef int vrgi __attribute__((ext_vector_type(RG)));
    typedef float vrgf __attribute__((ext_vector_type(RG)));
    __shared__ __attribute__((aligned(16))) int sd_l[NW][NW][64][RG];    // [writer][reader group][lane]
    __shared__ __attribute__((aligned(16))) float sm_l[NW][NW][64][RG];
    __shared__ float dd_l[NW][32][2];                                    // d, dmin per writer and row
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, h = lane >> 5;
    const int tok0 = blockIdx.y * 32;
    const size_t in_f = (size_t)nb * 256;
    // This workgroup's 32 weight rows: a table entry (plans: rows of one of several ops, whose
    // activation rows start at act_elem0 of the scratch) or computed from the single op.
    int wrow = blockIdx.x * 32 + col;  // output column relative to y
    bool row_ok = wrow < out_f;
    BatchAdd add;
    if (tiles) {
        const BatchTile t = tiles[blockIdx.x];
        w = t.w;
        bpr = t.bpr;
        y = t.y;
        add = BatchAdd{t.add_b, t.add_dst};
        out_f = (int)t.out_f;
        wrow = col;
        row_ok = col < (int)t.rows;
        qs += t.act_elem0;
        d8 += t.act_elem0 / 256;
        bsums += t.act_elem0 / 32;
    }
    const uint8_t* wrowp = w + (size_t)(row_ok ? wrow : 0) * bpr;
    const int atok = min(tok0 + col, m - 1);  // this lane's activation row as MFMA A operand
    // tokens of this thread's epilogue outputs: accumulator r = RG*wave + i of lane position `lane`
    int etok[RG];
#pragma unroll
    for (int i = 0; i < RG; ++i) {
        const int r = RG * wave + i;
        etok[i] = tok0 + 8 * (r >> 2) + 4 * h + (r & 3);
    }
    float acc[RG];
#pragma unroll
    for (int i = 0; i < RG; ++i) acc[i] = 0.0f;

    // Everything a round reads from global memory is requested one round ahead: the weight rows
    // (HBM), the activation fragments, per-32 sums and scales (L2).
    struct RoundIn {
        Q4kRaw raw;
        v4i a[8], bs0, bs1;
        float dq[NW][RG];
    };
    auto request = [&](RoundIn& in, int round) {
        const int b = round * NW + wave;
        const bool has = b < nb;
        const int bc = has ? b : 0;
        const int8_t* ap = qs + (size_t)atok * in_f + (size_t)bc * 256 + h * 16;
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) in.a[sb] = *reinterpret_cast<const v4i*>(ap + sb * 32);
        in.bs0 = *reinterpret_cast<const v4i*>(bsums + (size_t)atok * (nb * 8) + bc * 8);
        in.bs1 = *reinterpret_cast<const v4i*>(bsums + (size_t)atok * (nb * 8) + bc * 8 + 4);
#pragma unroll
        for (int j = 0; j < NW; ++j)
#pragma unroll
            for (int i = 0; i < RG; ++i) {
                const int bj = min(round * NW + j, nb - 1);
                in.dq[j][i] = d8[(size_t)min(etok[i], m - 1) * nb + bj];
            }
        q4k_load_raw(in.raw, wrowp + (size_t)bc * 144, h, row_ok && has);
    };
    RoundIn nxt;
    request(nxt, 0);
    const int rounds = (nb + NW - 1) / NW;
    for (int round = 0; round < rounds; ++round) {
        const int b = round * NW + wave;
        const bool has = b < nb;
        const RoundIn in = nxt;
        if (round + 1 < rounds) request(nxt, round + 1);
        const Q4kRaw& cur = in.raw;
        const v4i (&a)[8] = in.a;
        const float (&dq)[NW][RG] = in.dq;
        if (has) {
            const v4i bs0 = in.bs0, bs1 = in.bs1;

            uint32_t sc8[2], mn8[2];
            k4_all((uint32_t)cur.hdr.y, (uint32_t)cur.hdr.z, (uint32_t)cur.hdr.w, sc8, mn8);
            v4i blo[8], bhi[8];
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const int qw[4] = {cur.q[p].x, cur.q[p].y, cur.q[p].z, cur.q[p].w};
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const int sb = 2 * p + e;
                    const uint32_t sc = (sc8[sb >> 2] >> (8 * (sb & 3))) & 0xFFu;
                    const uint32_t lo3 = sc & 7u, hi3 = sc >> 3;
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const uint32_t codes = ((uint32_t)qw[k] >> (4 * e)) & 0x0F0F0F0Fu;
                        blo[sb][k] = scale_codes(codes, lo3);
                        bhi[sb][k] = scale_codes(codes, hi3);
                    }
                }
            }
            v8h bm;
#pragma unroll
            for (int sb = 0; sb < 8; ++sb) bm[sb] = (_Float16)(int)((mn8[sb >> 2] >> (8 * (sb & 3))) & 0xFFu);
            // per-32 sums split bsum = lo + 64*hi': the h = 0 lanes carry lo, the h = 1 lanes bsum - lo
            const int bsv[8] = {bs0.x, bs0.y, bs0.z, bs0.w, bs1.x, bs1.y, bs1.z, bs1.w};
            v8h abs_;
#pragma unroll
            for (int sb = 0; sb < 8; ++sb) {
                const int lo = bsv[sb] & 63;
                abs_[sb] = (_Float16)(h ? bsv[sb] - lo : lo);
            }
            const v16i zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            const v16f zf = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            v16i alo = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[0], blo[0], zi, 0, 0, 0);
            v16i ahi = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[0], bhi[0], zi, 0, 0, 0);
#pragma unroll
            for (int sb = 1; sb < 8; ++sb) {
                alo = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[sb], blo[sb], alo, 0, 0, 0);
                ahi = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[sb], bhi[sb], ahi, 0, 0, 0);
            }
            const v16f smf = __builtin_amdgcn_mfma_f32_32x32x16_f16(abs_, bm, zf, 0, 0, 0);
#pragma unroll
            for (int g = 0; g < NW; ++g) {
                vrgi sdv;
                vrgf smv;
#pragma unroll
                for (int i = 0; i < RG; ++i) {
                    const int r = RG * g + i;
                    sdv[i] = alo[r] + (ahi[r] << 3);
                    smv[i] = smf[r];
                    if (STAGES) {
                        const int tok = tok0 + 8 * (r >> 2) + 4 * h + (r & 3);
                        if (row_ok && tok < m) {
                            st_sd[((size_t)tok * out_f + wrow) * nb + b] = sdv[i];
                            st_sm[((size_t)tok * out_f + wrow) * nb + b] = (int)smv[i];
                        }
                    }
                }
                *reinterpret_cast<vrgi*>(&sd_l[wave][g][lane][0]) = sdv;
                *reinterpret_cast<vrgf*>(&sm_l[wave][g][lane][0]) = smv;
            }
            if (h == 0) {
                dd_l[wave][col][0] = f16_bits_to_f32((uint32_t)cur.hdr.x & 0xFFFFu);
                dd_l[wave][col][1] = f16_bits_to_f32((uint32_t)cur.hdr.x >> 16);
            }
        }
        __syncthreads();
        // f32 epilogue, blocks in ascending order: sumf += q8.d[b] * (d * sd as f32 - dmin * sm as f32)
#pragma unroll
        for (int j = 0; j < NW; ++j) {
            if (round * NW + j < nb) {
                const vrgi sdv = *reinterpret_cast<const vrgi*>(&sd_l[j][wave][lane][0]);
                const vrgf smv = *reinterpret_cast<const vrgf*>(&sm_l[j][wave][lane][0]);
                const float d = dd_l[j][col][0], dmin = dd_l[j][col][1];
#pragma unroll
                for (int i = 0; i < RG; ++i) acc[i] += dq[j][i] * (d * (float)sdv[i] - dmin * smv[i]);
            }
        }
        __syncthreads();
    }
    if (!row_ok) return;
#pragma unroll
    for (int i = 0; i < RG; ++i)
        if (etok[i] < m) store_batch_out(y, add, (size_t)etok[i] * out_f + wrow, acc[i]);
}

template <int NW>
static void launch_mmq_skinny_q4k(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m,
                                  size_t in_f, size_t out_f, const IntStages& st, hipStream_t stream) {
    const dim3 grid((unsigned)((out_f + 31) / 32), (unsigned)((m + 31) / 32)), block(NW * 64);
    const int nb = (int)(in_f / 256);
    if (st.a)
        hipLaunchKernelGGL((mmq_skinny_q4k_kernel<NW, true>), grid, block, 0, stream, w, bpr, act.qs, act.d,
                           act.bsums, y, (int)m, (int)out_f, nb, st.a, st.b, (const BatchTile*)nullptr);
    else
        hipLaunchKernelGGL((mmq_skinny_q4k_kernel<NW, false>), grid, block, 0, stream, w, bpr, act.qs, act.d,
                           act.bsums, y, (int)m, (int)out_f, nb, (int32_t*)nullptr, (int32_t*)nullptr,
                           (const BatchTile*)nullptr);
}

// ───────────────────────────── up to 16 tokens: 16 x 16 tiles, K split over waves, no exchange of integers ─────────────────────────────
// Decode batches (2..16 tokens) are bound by memory instructions and by VALU work per weight byte,
// not by the matrix cores. v_mfma_i32_16x16x64_i8 tiles of 16 tokens x 16 weight rows waste little
// on absent tokens, and one 64-byte run of a row feeds four lanes: lane (row r, K quarter kq)
// fetches bytes 64c + 16kq .. + 15 of the block's codes for c = 0, 1 and both nibbles of every byte
// are operands - the low nibbles of chunk c are one K = 64 step (sub-blocks 4c + 2(kq/2), elements
// 16(kq%2)..), the high nibbles the next (sub-blocks 4c + 2(kq/2) + 1) - so nothing is fetched
// twice. A workgroup covers 16 rows (half of a 32-row tile, blockIdx.y) and splits K over its NW
// waves in contiguous ranges of BPW blocks: a wave asks for all its weight bytes at once, keeps the
// exact integers (sd, sm) of its blocks in registers, and the f32 epilogue - the CPU's expression,
// blocks in ascending order - is handed from wave to wave through LDS (four floats per lane,
// NW - 1 barriers). A block's activations (MT tokens x 256 codes, their per-32 sums) come in with
// whole-line loads, one block ahead, and pass through a wave-private LDS tile into operand order:
// fetching the operands lane by lane took twice the memory instructions and kept the address
// units 80 % busy. The weights take the same route, two blocks (288 contiguous bytes of each of
// the 16 rows) at a time: neighbouring lanes then fetch neighbouring 16-byte pieces of one row and
// the loads leave the first-level cache as 64-byte requests, where a lane per row made every
// request 32 bytes - half of a DRAM burst. Same integers and the same f32 operations in the same
// order as the kernels above: bit-identical results.
//
// The format supplies one block's integers: block() reads this lane's row (weight row r16 of the
// half tile, staged in LDS), token r16's codes and per-32 sums as A operands, and returns
// sd = sum_s sc_s * (q . q8) and sm = sum_s m_s * bsum_s for tokens 4kq .. 4kq + 3 of row r16.
struct Skinny16Q4K {
    static constexpr bool kPer32Acts = false, kTranspose16 = false;
    static constexpr bool kSubScales = false;
    static constexpr int kBlockBytes = 144;
    // Q4_K: the scale split sc = 8 hi + lo folded into two operand sets, two chains of four K = 64 steps
    static constexpr int kRowStride = 2 * kBlockBytes + 16;  // two blocks, padded: eight rows' 16-byte reads cover all banks
    // sumf += q8.d[b] * (d * sd as f32 - dmin * sm as f32)
    __device__ static float accumulate(float acc, float dq, uint32_t ddm, int sd, float sm) {
        const float d = f16_bits_to_f32(ddm & 0xFFFFu), dmin = f16_bits_to_f32(ddm >> 16);
        return acc + dq * (d * (float)sd - dmin * sm);
    }
    __device__ static void block(const uint8_t* wrow, int jj, const uint8_t* arow, const uint8_t* zrow,
                                 const uint8_t* bsrow, int kq, int (&sd)[4], float (&sm)[4], uint32_t& ddm) {
        const uint8_t* wblk = wrow + jj * kBlockBytes;
        const int g = kq >> 1, hh = kq & 1;
        const v4i hdr = *reinterpret_cast<const v4i*>(wblk);
        v4i q[2];
        q[0] = *reinterpret_cast<const v4i*>(wblk + 16 + 16 * kq);
        q[1] = *reinterpret_cast<const v4i*>(wblk + 16 + 64 + 16 * kq);
        ddm = (uint32_t)hdr.x;
        uint32_t sc8[2], mn8[2];
        k4_all((uint32_t)hdr.y, (uint32_t)hdr.z, (uint32_t)hdr.w, sc8, mn8);
        v4i alo = {0, 0, 0, 0}, ahi = {0, 0, 0, 0};
#pragma unroll
        for (int s = 0; s < 4; ++s) {  // step s: chunk c = s / 2, nibble e = s % 2
            const int c = s >> 1, e = s & 1;
            const uint32_t sc = (sc8[c] >> (8 * (2 * g + e))) & 0xFFu;
            const uint32_t lo3 = sc & 7u, hi3 = sc >> 3;
            const int qw[4] = {q[c].x, q[c].y, q[c].z, q[c].w};
            v4i blo, bhi;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t codes = ((uint32_t)qw[k] >> (4 * e)) & 0x0F0F0F0Fu;
                blo[k] = scale_codes(codes, lo3);
                bhi[k] = scale_codes(codes, hi3);
            }
            const v4i a = *reinterpret_cast<const v4i*>(arow + (4 * c + 2 * g + e) * 32 + 16 * hh);
            alo = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, blo, alo, 0, 0, 0);
            ahi = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, bhi, ahi, 0, 0, 0);
        }
        const v4f smf = mins_dot_sums(mn8[hh], bsrow, g, hh);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            sd[i] = alo[i] + (ahi[i] << 3);
            sm[i] = smf[i];
        }
    }
    // sm as a K = 16 f16 product: slots = (bsum & 63 | the rest) x sub-blocks 0..7; lane (., kq) carries
    // slots 4kq..4kq+3: sub-blocks 4hh..4hh+3 (their mins are the bytes of `mnw`) of part g
    __device__ static v4f mins_dot_sums(uint32_t mnw, const uint8_t* bsrow, int g, int hh) {
        typedef _Float16 v4h __attribute__((ext_vector_type(4)));
        const v4h bm = {(_Float16)(int)(mnw & 0xFFu), (_Float16)(int)((mnw >> 8) & 0xFFu),
                        (_Float16)(int)((mnw >> 16) & 0xFFu), (_Float16)(int)(mnw >> 24)};
        const v4i bs = *reinterpret_cast<const v4i*>(bsrow + 16 * hh);
        const int bsv[4] = {bs.x, bs.y, bs.z, bs.w};
        v4h abs_;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int lo = bsv[k] & 63;
            abs_[k] = (_Float16)(g ? bsv[k] - lo : lo);
        }
        return __builtin_amdgcn_mfma_f32_16x16x16f16(abs_, bm, v4f{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
    }
};

// Q5_K (176-byte block: d, dmin, scales[12], qh[32], qs[128]; crates/infr-cpu/src/kernels.rs q5_k dot):
// a 5-bit code times a 6-bit scale has no int8 split of two digits, so a sub-block is one
// v_mfma_i32_16x16x32_i8 (lane (., kq): elements 8kq .. 8kq + 7) scaled into sd by a 24-bit
// multiply-add; sm and the epilogue are Q4_K's.
struct Skinny16Q5K {
    static constexpr bool kPer32Acts = false, kTranspose16 = false;
    static constexpr bool kSubScales = false;
    static constexpr int kBlockBytes = 176;
    static constexpr int kRowStride = 2 * kBlockBytes + 16;
    __device__ static float accumulate(float acc, float dq, uint32_t ddm, int sd, float sm) {
        return Skinny16Q4K::accumulate(acc, dq, ddm, sd, sm);
    }
    __device__ static void block(const uint8_t* wrow, int jj, const uint8_t* arow, const uint8_t* zrow,
                                 const uint8_t* bsrow, int kq, int (&sd)[4], float (&sm)[4], uint32_t& ddm) {
        typedef int v2i __attribute__((ext_vector_type(2)));
        const uint8_t* wblk = wrow + jj * kBlockBytes;
        const int g = kq >> 1, hh = kq & 1;
        const v4i hdr = *reinterpret_cast<const v4i*>(wblk);
        const v2i qh = *reinterpret_cast<const v2i*>(wblk + 16 + 8 * kq);
        v2i qs[4];
#pragma unroll
        for (int p = 0; p < 4; ++p) qs[p] = *reinterpret_cast<const v2i*>(wblk + 48 + 32 * p + 8 * kq);
        ddm = (uint32_t)hdr.x;
        uint32_t sc8[2], mn8[2];
        k4_all((uint32_t)hdr.y, (uint32_t)hdr.z, (uint32_t)hdr.w, sc8, mn8);
#pragma unroll
        for (int i = 0; i < 4; ++i) sd[i] = 0;
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) {
            const int p = sb >> 1, e = sb & 1;
            v2i b;
#pragma unroll
            for (int k = 0; k < 2; ++k) {
                const uint32_t nib = ((uint32_t)qs[p][k] >> (4 * e)) & 0x0F0F0F0Fu;
                const uint32_t hb = ((uint32_t)qh[k] >> sb) & 0x01010101u;
                b[k] = (int)((hb << 4) | nib);
            }
            const v2i a = *reinterpret_cast<const v2i*>(arow + sb * 32 + 8 * kq);
            const v4i r = __builtin_amdgcn_mfma_i32_16x16x32_i8(__builtin_bit_cast(long, a), __builtin_bit_cast(long, b),
                                                                v4i{0, 0, 0, 0}, 0, 0, 0);
            const int sc = (int)((sc8[sb >> 2] >> (8 * (sb & 3))) & 0xFFu);
#pragma unroll
            for (int i = 0; i < 4; ++i) sd[i] += __mul24(r[i], sc);
        }
        const v4f smf = Skinny16Q4K::mins_dot_sums(mn8[hh], bsrow, g, hh);
#pragma unroll
        for (int i = 0; i < 4; ++i) sm[i] = smf[i];
    }
};

// Q6_K (210-byte block: ql[128], qh[64], int8 scales[16], d; crates/infr-cpu/src/kernels.rs:487-526):
// isum = sum_g sc_g * (sum over the group's 16 of (q - 32) * q8), y += (d * q8.d[b]) * isum. A K = 32
// step holds two groups of 16 (lanes kq 0, 1 and kq 2, 3); each is multiplied alone - the other
// group's activation lanes read a row of zero bytes - and scaled into isum by a 24-bit
// multiply-add. A stage of two blocks is 420 bytes from a 4-byte boundary, so its second block sits
// 2 bytes off a boundary in LDS: it is read as aligned words and shifted in registers.
struct Skinny16Q6K {
    static constexpr bool kPer32Acts = false, kTranspose16 = false;
    static constexpr bool kSubScales = false;
    typedef int v2i __attribute__((ext_vector_type(2)));
    static constexpr int kBlockBytes = 210;
    static constexpr int kRowStride = 432;  // 420 rounded up to 16: 108 words, eight rows' reads cover all banks
    // sumf += d * q8.d[b] * (isum as f32), evaluated (d * q8.d[b]) * isum
    __device__ static float accumulate(float acc, float dq, uint32_t ddm, int sd, float) {
        return acc + (f16_bits_to_f32(ddm) * dq) * (float)sd;
    }
    template <bool ODD>
    __device__ static v2i read8(const uint8_t* blk, int o) {
        if (!ODD) return *reinterpret_cast<const v2i*>(blk + o);
        const uint8_t* p = blk - 2 + o;
        const v2i lo = *reinterpret_cast<const v2i*>(p);
        const int hi = *reinterpret_cast<const int*>(p + 8);
        return v2i{(int)__builtin_amdgcn_alignbyte((uint32_t)lo.y, (uint32_t)lo.x, 2),
                   (int)__builtin_amdgcn_alignbyte((uint32_t)hi, (uint32_t)lo.y, 2)};
    }
    template <bool ODD>
    __device__ static void block_at(const uint8_t* blk, const uint8_t* arow, const uint8_t* zrow, int kq, int (&sd)[4],
                                    uint32_t& ddm) {
        v2i ql[2][2], qh[2];
#pragma unroll
        for (int n = 0; n < 2; ++n) {
            ql[n][0] = read8<ODD>(blk, 64 * n + 8 * kq);
            ql[n][1] = read8<ODD>(blk, 64 * n + 32 + 8 * kq);
            qh[n] = read8<ODD>(blk, 128 + 32 * n + 8 * kq);
        }
        const v2i s01 = read8<ODD>(blk, 192), s23 = read8<ODD>(blk, 200);
        const int scw[4] = {s01.x, s01.y, s23.x, s23.y};
        ddm = *reinterpret_cast<const uint16_t*>(blk + 208);
        // group 2s in the K-slots of lanes kq 0, 1, group 2s+1 in those of kq 2, 3
        const uint8_t* a0p = (kq < 2 ? arow : zrow) + 8 * kq;
        const uint8_t* a1p = (kq < 2 ? zrow : arow) + 8 * kq;
#pragma unroll
        for (int i = 0; i < 4; ++i) sd[i] = 0;
#pragma unroll
        for (int s = 0; s < 8; ++s) {  // elements 32s .. 32s + 31: half n, quarter t of the half
            const int n = s >> 2, t = s & 3;
            v2i b;
#pragma unroll
            for (int k = 0; k < 2; ++k) {
                const uint32_t nib = ((uint32_t)ql[n][t & 1][k] >> (4 * (t >> 1))) & 0x0F0F0F0Fu;
                const uint32_t hb = ((uint32_t)qh[n][k] >> (2 * t)) & 0x03030303u;
                b[k] = (int)((((hb << 4) | nib) + 0x60606060u) ^ 0x80808080u);  // q - 32 as int8
            }
            const long bl = __builtin_bit_cast(long, b);
            const v2i a0 = *reinterpret_cast<const v2i*>(a0p + 32 * s);
            const v2i a1 = *reinterpret_cast<const v2i*>(a1p + 32 * s);
            const v4i r0 = __builtin_amdgcn_mfma_i32_16x16x32_i8(__builtin_bit_cast(long, a0), bl, v4i{0, 0, 0, 0}, 0, 0, 0);
            const v4i r1 = __builtin_amdgcn_mfma_i32_16x16x32_i8(__builtin_bit_cast(long, a1), bl, v4i{0, 0, 0, 0}, 0, 0, 0);
            const int g0 = 2 * s, g1 = 2 * s + 1;
            const int sc0 = __builtin_amdgcn_sbfe(scw[g0 >> 2], 8 * (g0 & 3), 8);
            const int sc1 = __builtin_amdgcn_sbfe(scw[g1 >> 2], 8 * (g1 & 3), 8);
#pragma unroll
            for (int i = 0; i < 4; ++i) sd[i] += __mul24(r0[i], sc0) + __mul24(r1[i], sc1);
        }
    }
    __device__ static void block(const uint8_t* wrow, int jj, const uint8_t* arow, const uint8_t* zrow,
                                 const uint8_t*, int kq, int (&sd)[4], float (&sm)[4], uint32_t& ddm) {
        if (jj & 1) block_at<true>(wrow + jj * kBlockBytes, arow, zrow, kq, sd, ddm);
        else block_at<false>(wrow + jj * kBlockBytes, arow, zrow, kq, sd, ddm);
#pragma unroll
        for (int i = 0; i < 4; ++i) sm[i] = 0.0f;
    }
};

// Q2_K (84-byte block: scales[16] (scale | min << 4 per 16 weights), qs[64], d, dmin;
// crates/infr-cpu/src/kernels.rs:315-361): sd = sum_g sc_g * (q . q8)_g, sm = sum_g mn_g * bsum16_g,
// y += q8.d[b] * (d * sd - dmin * sm). Lane (., kq = 2 n + half) owns bytes qs[16 kq .. 16 kq + 15]:
// their bit pairs j = 0..3 are elements 128 n + 32 j + 16 half .. + 15, sub-block 8 n + 2 j + half,
// so a K = 64 step takes bit pair j of every lane's 16 bytes and each lane's 16 K-slots are one
// sub-block. A 2-bit code times a 4-bit scale fits a byte: the scaled codes are the operand and
// four steps chain into sd; a second chain against bytes that all hold the sub-block's min sums
// min * q8 over the sub-block - mn_g * bsum16_g without the sums. Exact integers either way.
struct Skinny16Q2K {
    static constexpr bool kPer32Acts = false, kTranspose16 = false;
    static constexpr bool kSubScales = false;
    static constexpr int kBlockBytes = 84;
    static constexpr int kRowStride = 176;  // two blocks (168 bytes) padded: 44 words, eight rows' 16-byte reads cover all banks
    __device__ static float accumulate(float acc, float dq, uint32_t ddm, int sd, float sm) {
        return Skinny16Q4K::accumulate(acc, dq, ddm, sd, sm);
    }
    __device__ static void block(const uint8_t* wrow, int jj, const uint8_t* arow, const uint8_t*, const uint8_t*,
                                 int kq, int (&sd)[4], float (&sm)[4], uint32_t& ddm) {
        const uint8_t* wblk = wrow + jj * kBlockBytes;  // blocks are word-aligned, not 16-byte aligned
        const int n = kq >> 1, half = kq & 1;
        const int* qp = reinterpret_cast<const int*>(wblk + 16 + 16 * kq);
        const int qw[4] = {qp[0], qp[1], qp[2], qp[3]};
        const int* sp = reinterpret_cast<const int*>(wblk + 8 * n);
        const uint32_t scw[2] = {(uint32_t)sp[0] >> (8 * half), (uint32_t)sp[1] >> (8 * half)};
        ddm = *reinterpret_cast<const uint32_t*>(wblk + 80);
        v4i ad = {0, 0, 0, 0}, am = {0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t sb = (scw[j >> 1] >> (16 * (j & 1))) & 0xFFu;  // byte half + 2 j of scales[8 n ..]
            const uint32_t s4 = sb & 15u;
            const int mw = (int)((sb >> 4) * 0x01010101u);
            v4i b;
#pragma unroll
            for (int k = 0; k < 4; ++k) b[k] = scale_codes(((uint32_t)qw[k] >> (2 * j)) & 0x03030303u, s4);
            const v4i a = *reinterpret_cast<const v4i*>(arow + 128 * n + 32 * j + 16 * half);
            ad = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, ad, 0, 0, 0);
            am = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, v4i{mw, mw, mw, mw}, am, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            sd[i] = ad[i];
            sm[i] = (float)am[i];  // |sm| <= 15 * 127 * 256: exact
        }
    }
};

// Q3_K (110-byte block: hmask[32], qs[64], scales[12], d; crates/infr-cpu/src/kernels.rs:812-852,
// scales by :764-783): isum = sum_g (sc6_g - 32) * sum (code - 4) * q8, y += (d * q8.d[b]) * isum.
// Lanes own bytes and sub-blocks as for Q2_K; the third code bit of bit pair j is bit 4 n + j of
// hmask[16 half + l]. (4 - code) * (sc6 - 32) lies in [-128, 124]: the lane builds that product's
// eight values for its sub-block as a byte table - (4 - v) u - 32 (4 - v) for v < 4 and
// (v - 4) (64 - u) - 32 (v - 4) above, u = sc6, each a packed multiply and a byte-wise subtract -
// and one v_perm_b32 per word looks four codes up in it. Four K = 64 steps chain into -isum. A
// stage of two blocks is 220 bytes: the second block sits 2 bytes off a word boundary in LDS and is
// read as aligned words and shifted; rows are an even number of blocks.
struct Skinny16Q3K {
    static constexpr bool kPer32Acts = false, kTranspose16 = false;
    static constexpr bool kSubScales = false;
    static constexpr int kBlockBytes = 110;
    static constexpr int kRowStride = 240;  // 220 rounded up: 60 words, eight rows' 16-byte reads cover all banks
    __device__ static float accumulate(float acc, float dq, uint32_t ddm, int sd, float) {
        return acc + (f16_bits_to_f32(ddm) * dq) * (float)sd;
    }
    template <bool ODD, int N>
    __device__ static void words(const uint8_t* blk, int o, uint32_t (&out)[N]) {
        if (!ODD) {
#pragma unroll
            for (int i = 0; i < N; ++i) out[i] = *reinterpret_cast<const uint32_t*>(blk + o + 4 * i);
        } else {
            uint32_t w[N + 1];
#pragma unroll
            for (int i = 0; i <= N; ++i) w[i] = *reinterpret_cast<const uint32_t*>(blk - 2 + o + 4 * i);
#pragma unroll
            for (int i = 0; i < N; ++i) out[i] = __builtin_amdgcn_alignbyte(w[i + 1], w[i], 2);
        }
    }
    // x - y on each byte, modulo 256, without borrows between bytes
    __device__ static uint32_t sub_bytes(uint32_t x, uint32_t y_low7, uint32_t not_y_top) {
        return ((x | 0x80808080u) - y_low7) ^ (x & 0x80808080u) ^ not_y_top;
    }
    __device__ static uint32_t mul_bytes(uint32_t halves, uint32_t f) {
        typedef unsigned short us2 __attribute__((ext_vector_type(2)));
        const us2 s = {(unsigned short)f, (unsigned short)f};
        return __builtin_bit_cast(uint32_t, (us2)(__builtin_bit_cast(us2, halves) * s));
    }
    template <bool ODD>
    __device__ static void block_at(const uint8_t* blk, const uint8_t* arow, int kq, int (&sd)[4], uint32_t& ddm) {
        const int n = kq >> 1, half = kq & 1;
        uint32_t qw[4], hw[4], scw[3];
        words<ODD, 4>(blk, 32 + 16 * kq, qw);
        words<ODD, 4>(blk, 16 * half, hw);
        words<ODD, 3>(blk, 96, scw);
        ddm = *reinterpret_cast<const uint16_t*>(blk + 108);
        // field 8 n + 2 j + half: low nibble in nibble n of byte 2 j + half of the first eight, top
        // two bits at bit 4 n + 2 (j / 2) of byte 8 + 2 (j % 2) + half
        const int sh = 8 * half + 4 * n;
        const uint32_t a0 = scw[0] >> sh, a1 = scw[1] >> sh, tt = scw[2] >> sh;
        v4i acc = {0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t u = (((j < 2 ? a0 : a1) >> (16 * (j & 1))) & 15u) | (((tt >> (16 * (j & 1) + 2 * (j >> 1))) & 3u) << 4);
            // table[v] = (4 - v) * (u - 32) as int8, v = 0..3 in t_lo, 4..7 in t_hi
            const uint32_t t_lo = sub_bytes(mul_bytes(0x01020304u, u), 0x20406000u, 0x80808000u);
            const uint32_t t_hi = sub_bytes(mul_bytes(0x03020100u, 64u - u), 0x60402000u, 0x80808080u);
            v4i b;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t low2 = (qw[k] >> (2 * j)) & 0x03030303u;
                const uint32_t high = (hw[k] >> (4 * n + j)) & 0x01010101u;
                b[k] = (int)__builtin_amdgcn_perm(t_hi, t_lo, low2 | (high << 2));
            }
            const v4i a = *reinterpret_cast<const v4i*>(arow + 128 * n + 32 * j + 16 * half);
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) sd[i] = -acc[i];
    }
    __device__ static void block(const uint8_t* wrow, int jj, const uint8_t* arow, const uint8_t*, const uint8_t*,
                                 int kq, int (&sd)[4], float (&sm)[4], uint32_t& ddm) {
        if (jj & 1) block_at<true>(wrow + jj * kBlockBytes, arow, kq, sd, ddm);
        else block_at<false>(wrow + jj * kBlockBytes, arow, kq, sd, ddm);
#pragma unroll
        for (int i = 0; i < 4; ++i) sm[i] = 0.0f;
    }
};

// TQ2_0 (66-byte block: qs[64], d; crates/infr-cpu/src/kernels.rs:3066-3126): the ternary weights
// q - 1 are the operand as they are - lanes and bit pairs as for Q2_K, four K = 64 steps chain into
// the block's iprod - and y += (d * q8.d[b]) * iprod. A stage of two blocks is 132 bytes: the second
// sits 2 bytes off a word boundary in LDS (read as aligned words and shifted); rows are an even
// number of blocks.
struct Skinny16TQ2_0 {
    static constexpr bool kPer32Acts = false, kTranspose16 = false;
    static constexpr bool kSubScales = false;
    static constexpr int kBlockBytes = 66;
    static constexpr int kRowStride = 144;  // 132 rounded up: 36 words, eight rows' 16-byte reads cover all banks
    __device__ static float accumulate(float acc, float dq, uint32_t ddm, int sd, float) {
        return acc + (f16_bits_to_f32(ddm) * dq) * (float)sd;
    }
    __device__ static void block(const uint8_t* wrow, int jj, const uint8_t* arow, const uint8_t*, const uint8_t*,
                                 int kq, int (&sd)[4], float (&sm)[4], uint32_t& ddm) {
        const uint8_t* blk = wrow + jj * kBlockBytes;
        const int n = kq >> 1, half = kq & 1;
        uint32_t qw[4];
        if (jj & 1) Skinny16Q3K::words<true, 4>(blk, 16 * kq, qw);
        else Skinny16Q3K::words<false, 4>(blk, 16 * kq, qw);
        ddm = *reinterpret_cast<const uint16_t*>(blk + 64);
        v4i acc = {0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            v4i b;
#pragma unroll
            for (int k = 0; k < 4; ++k)  // q - 1 on every byte: q + 0x7F stays inside the byte, flipping bit 7 gives q - 1
                b[k] = (int)((((qw[k] >> (2 * j)) & 0x03030303u) + 0x7F7F7F7Fu) ^ 0x80808080u);
            const v4i a = *reinterpret_cast<const v4i*>(arow + 128 * n + 32 * j + 16 * half);
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            sd[i] = acc[i];
            sm[i] = 0.0f;
        }
    }
};

// IQ4_XS (136-byte block: d, scales_h, scales_l[4], qs[128]; crates/infr-cpu/src/kernels.rs:995-1036):
// isum = sum_ib (ls_ib - 32) * (table[q] . q8) over eight sub-blocks of 32, y += (d * q8.d[b]) * isum.
// A table value times a 6-bit scale does not fit a byte, so a sub-block is one
// v_mfma_i32_16x16x32_i8 (lane (., kq): elements 8 kq .. 8 kq + 7 - nibble kq / 2 of bytes
// 8 (kq % 2) .. + 7 of the sub-block's 16, looked up in IQ4_NL's table) scaled into isum by a 24-bit
// multiply-add. Blocks are 8-byte aligned; a stage of two is 272 bytes.
struct Skinny16IQ4XS {
    typedef int v2i __attribute__((ext_vector_type(2)));
    static constexpr bool kPer32Acts = false, kTranspose16 = false;
    static constexpr bool kSubScales = false;
    static constexpr int kBlockBytes = 136;
    static constexpr int kRowStride = 2 * kBlockBytes + 16;
    __device__ static float accumulate(float acc, float dq, uint32_t ddm, int sd, float) {
        return acc + (f16_bits_to_f32(ddm & 0xFFFFu) * dq) * (float)sd;
    }
    __device__ static int lookup(uint32_t nib) {  // IQ4_NL's table (crates/infr-gguf/src/dequant.rs:439-441)
        const uint32_t sel = nib & 0x07070707u;
        const uint32_t lo = __builtin_amdgcn_perm(0xF6EADDCFu, 0xBFAD9881u, sel);
        const uint32_t hi = __builtin_amdgcn_perm(0x71594535u, 0x26190D01u, sel);
        const uint32_t pick = ((nib >> 3) & 0x01010101u) * 0xFFu;
        return (int)((hi & pick) | (lo & ~pick));
    }
    __device__ static void block(const uint8_t* wrow, int jj, const uint8_t* arow, const uint8_t*, const uint8_t*,
                                 int kq, int (&sd)[4], float (&sm)[4], uint32_t& ddm) {
        const uint8_t* wblk = wrow + jj * kBlockBytes;
        const v2i hdr = *reinterpret_cast<const v2i*>(wblk);
        ddm = (uint32_t)hdr.x;
        const uint32_t sl = (uint32_t)hdr.y, sh = (uint32_t)hdr.x >> 16;
        const int shift = 4 * (kq >> 1);
#pragma unroll
        for (int i = 0; i < 4; ++i) sd[i] = 0;
#pragma unroll
        for (int ib = 0; ib < 8; ++ib) {
            const v2i q = *reinterpret_cast<const v2i*>(wblk + 8 + 16 * ib + 8 * (kq & 1));
            v2i b;
            b.x = lookup(((uint32_t)q.x >> shift) & 0x0F0F0F0Fu);
            b.y = lookup(((uint32_t)q.y >> shift) & 0x0F0F0F0Fu);
            const v2i a = *reinterpret_cast<const v2i*>(arow + ib * 32 + 8 * kq);
            const v4i r = __builtin_amdgcn_mfma_i32_16x16x32_i8(__builtin_bit_cast(long, a), __builtin_bit_cast(long, b),
                                                                v4i{0, 0, 0, 0}, 0, 0, 0);
            const int ls = (int)(((sl >> (4 * ib)) & 15u) | (((sh >> (2 * ib)) & 3u) << 4)) - 32;
#pragma unroll
            for (int i = 0; i < 4; ++i) sd[i] += __mul24(r[i], ls);  // |r| <= 32 * 127 * 127
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) sm[i] = 0.0f;
    }
};

// Q8_0 (34-byte blocks: f16 d, 32 int8 codes; crates/infr-cpu/src/kernels.rs:1170-1187): a 256-element
// step is eight blocks, 272 bytes, each with a scale of its own. The stored codes are the operand:
// one v_mfma_i32_16x16x32_i8 per block gives its exact iprod, and the f32 side is the CPU's chain
// `sumf += (q8.d[b] * d_w) * (iprod as f32)` block by block - so these outputs equal infr-cpu's
// scalar kernel bit for bit, which the dot4 batches (a fixed tree over the lanes) do not.
// kSubScales: a step's integers are 8 x 4 (block s, output i at [4 s + i]) and `ddm` its eight
// scales, two to a word. Blocks start 2 bytes off a word boundary on every other block: those codes
// are read as aligned words and shifted.
struct Skinny16Q8_0 {
    static constexpr bool kPer32Acts = false, kTranspose16 = false;
    typedef int v2i __attribute__((ext_vector_type(2)));
    static constexpr bool kSubScales = true;
    static constexpr int kBlockBytes = 272;
    static constexpr int kRowStride = 2 * kBlockBytes + 16;  // 140 words: eight rows' 16-byte reads cover all banks
    __device__ static void block(const uint8_t* wrow, int jj, const uint8_t* arow, int kq, int (&ip)[32],
                                 uint32_t (&dw)[4]) {
        const uint8_t* blk = wrow + jj * kBlockBytes;
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const uint8_t* sb = blk + s * 34;
            v2i b;
            if (s & 1) {  // codes at 34 s + 2 + 8 kq: a word boundary
                b.x = *reinterpret_cast<const int*>(sb + 2 + 8 * kq);
                b.y = *reinterpret_cast<const int*>(sb + 6 + 8 * kq);
            } else {      // two bytes past one
                const int w0 = *reinterpret_cast<const int*>(sb + 8 * kq);
                const int w1 = *reinterpret_cast<const int*>(sb + 4 + 8 * kq);
                const int w2 = *reinterpret_cast<const int*>(sb + 8 + 8 * kq);
                b.x = (int)__builtin_amdgcn_alignbyte((uint32_t)w1, (uint32_t)w0, 2);
                b.y = (int)__builtin_amdgcn_alignbyte((uint32_t)w2, (uint32_t)w1, 2);
            }
            const v2i a = *reinterpret_cast<const v2i*>(arow + s * 32 + 8 * kq);
            const v4i r = __builtin_amdgcn_mfma_i32_16x16x32_i8(__builtin_bit_cast(long, a), __builtin_bit_cast(long, b),
                                                                v4i{0, 0, 0, 0}, 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 4; ++i) ip[4 * s + i] = r[i];
            const uint32_t d16 = *reinterpret_cast<const uint16_t*>(sb);
            if (s & 1) dw[s >> 1] |= d16 << 16;
            else dw[s >> 1] = d16;
        }
    }
    // sumf += (q8.d[b] * d_w) * (iprod as f32), the step's eight blocks in order
    __device__ static void accumulate(float (&acc)[4], const float (&dq)[4], const uint32_t (&dw)[4], const int (&ip)[32]) {
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const float d = f16_bits_to_f32((dw[s >> 1] >> (16 * (s & 1))) & 0xFFFFu);
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] += (dq[i] * d) * (float)ip[4 * s + i];
        }
    }
};

// Q2_0 (18-byte blocks of 64: f16 d, 16 bytes of 2-bit codes; crates/infr-cpu/src/kernels.rs:5641-5668)
// against the per-32 activation: a 256-element step is four blocks, 72 bytes, and eight 32-element
// halves, each with its own activation scale and code sum. `(word >> 2 i) & 0x03030303` is codes
// i, 4 + i, 8 + i, 12 + i of a word's sixteen, so the activation tile holds every 16 codes 4 x 4
// transposed (kTranspose16: done in registers on the way into LDS) and a half is one
// v_mfma_i32_16x16x32_i8 after two shifts and two masks. The lane turns each half's exact integer
// into the CPU's f32 term `(d * q8.d[s]) * (iprod - bsum[s]) as f32` at once (both integers and their
// difference are exact in f32) - the scales and sums of its four output tokens are in LDS then -
// and the wave-to-wave chain adds the terms in block order: infr-cpu's bits. `ip` carries the
// terms' bit patterns; `raw` the integers for the stage outputs.
struct Skinny16Q2_0 {
    typedef int v2i __attribute__((ext_vector_type(2)));
    static constexpr bool kSubScales = true, kPer32Acts = true, kTranspose16 = true;
    static constexpr int kBlockBytes = 72;
    static constexpr int kRowStride = 2 * kBlockBytes;  // 36 words: eight rows' 16-byte reads cover all banks
    template <int MT, int DQ_STRIDE>
    __device__ static void block(const uint8_t* wrow, int jj, const uint8_t* arow, const uint8_t* bs_base,
                                 const float* dq_base, int kq, int (&ip)[32], int (&raw)[32]) {
        const uint8_t* blk = wrow + jj * kBlockBytes;
        const int i0 = 2 * (kq & 1);
        // this lane's output tokens 4 kq .. 4 kq + 3: their eight scales and eight code sums of the step
        v4f dq[4][2];
        v4i bs[4][2];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int tok = (4 * kq + i) & (MT - 1);
            dq[i][0] = *reinterpret_cast<const v4f*>(dq_base + tok * DQ_STRIDE + jj * 8);
            dq[i][1] = *reinterpret_cast<const v4f*>(dq_base + tok * DQ_STRIDE + jj * 8 + 4);
            bs[i][0] = *reinterpret_cast<const v4i*>(bs_base + tok * 32);
            bs[i][1] = *reinterpret_cast<const v4i*>(bs_base + tok * 32 + 16);
        }
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const int q = s >> 1;  // the half's 64-block
            const int off = 18 * q + 2 + 8 * (s & 1) + 4 * (kq >> 1);  // this lane's word of the half's codes
            uint32_t cw;
            if (q & 1) {
                cw = *reinterpret_cast<const uint32_t*>(blk + off);
            } else {  // 2 bytes past a word boundary
                const uint32_t w0 = *reinterpret_cast<const uint32_t*>(blk + off - 2);
                const uint32_t w1 = *reinterpret_cast<const uint32_t*>(blk + off + 2);
                cw = __builtin_amdgcn_alignbyte(w1, w0, 2);
            }
            v2i b;
            b.x = (int)((cw >> (2 * i0)) & 0x03030303u);
            b.y = (int)((cw >> (2 * i0 + 2)) & 0x03030303u);
            const v2i a = *reinterpret_cast<const v2i*>(arow + s * 32 + 8 * kq);
            const v4i r = __builtin_amdgcn_mfma_i32_16x16x32_i8(__builtin_bit_cast(long, a), __builtin_bit_cast(long, b),
                                                                v4i{0, 0, 0, 0}, 0, 0, 0);
            const float d = f16_bits_to_f32(*reinterpret_cast<const uint16_t*>(blk + 18 * q));
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                raw[4 * s + i] = r[i];
                const float term = (d * dq[i][s >> 2][s & 3]) * (float)(r[i] - bs[i][s >> 2][s & 3]);
                ip[4 * s + i] = __builtin_bit_cast(int, term);
            }
        }
    }
    // sumf += term, the step's eight halves in order
    __device__ static void accumulate(float (&acc)[4], const float (&)[4], const uint32_t (&)[4], const int (&ip)[32]) {
#pragma unroll
        for (int s = 0; s < 8; ++s)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] += __builtin_bit_cast(float, ip[4 * s + i]);
    }
};

// Q4_0 / Q4_1 / Q5_0 / Q5_1 / IQ4_NL (32-weight blocks of 18..24 bytes; crates/infr-cpu/src/kernels.rs
// vec_dot_*_32_batch, restated in the oracle's orc_vec_dot_blk32) against the per-32 activation: a
// 256-element step is eight blocks. Byte j of a block's 16 holds element j in its low nibble and
// element 16 + j in its high one, so the lane that supplies elements 8 kq .. 8 kq + 7 reads eight
// bytes and takes one nibble of each (plus, for the Q5 kinds, eight bits of the mask spread to bit 4;
// IQ4_NL's nibbles go through its table); one v_mfma_i32_16x16x32_i8 per block gives the exact
// iprod, and the lane forms the CPU's f32 term at once - `(d * q8.d) * (iprod - 8 or 16 * bsum)`,
// `(d * q8.d) * iprod` for IQ4_NL, `q8.d * (d * iprod + m * bsum)` for the affine kinds - for the
// wave-to-wave chain to add in block order: infr-cpu's bits. Blocks of 18 and 22 bytes start two
// bytes off a word boundary every other block: read as aligned words and shifted.
template <Nib32 K>
struct Skinny16Nib32 {
    typedef int v2i __attribute__((ext_vector_type(2)));
    static constexpr bool kAffine = K == Nib32::Q4_1 || K == Nib32::Q5_1;
    static constexpr bool kFive = K == Nib32::Q5_0 || K == Nib32::Q5_1;
    static constexpr bool kSubScales = true, kPer32Acts = true, kTranspose16 = false;
    static constexpr int kB = 18 + (kAffine ? 2 : 0) + (kFive ? 4 : 0);  // bytes of a 32-weight block
    static constexpr int kBlockBytes = 8 * kB;
    static constexpr int kRowStride = 2 * kBlockBytes + 16;  // (stride / 4) mod 32 = 12, 20, 28, 4: eight rows' 16-byte reads cover all banks
    // a word at `off` bytes into the row's stage, where off is 0 or 2 mod 4 (`odd`: known at compile time)
    template <bool ODD>
    __device__ static uint32_t word_at(const uint8_t* p) {
        if (!ODD) return *reinterpret_cast<const uint32_t*>(p);
        const uint32_t w0 = *reinterpret_cast<const uint32_t*>(p - 2), w1 = *reinterpret_cast<const uint32_t*>(p + 2);
        return __builtin_amdgcn_alignbyte(w1, w0, 2);
    }
    template <int MT, int DQ_STRIDE>
    __device__ static void block(const uint8_t* wrow, int jj, const uint8_t* arow, const uint8_t* bs_base,
                                 const float* dq_base, int kq, int (&ip)[32], int (&raw)[32]) {
        const uint8_t* blk = wrow + jj * kBlockBytes;
        v4f dq[4][2];
        v4i bs[4][2];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int tok = (4 * kq + i) & (MT - 1);
            dq[i][0] = *reinterpret_cast<const v4f*>(dq_base + tok * DQ_STRIDE + jj * 8);
            dq[i][1] = *reinterpret_cast<const v4f*>(dq_base + tok * DQ_STRIDE + jj * 8 + 4);
            bs[i][0] = *reinterpret_cast<const v4i*>(bs_base + tok * 32);
            bs[i][1] = *reinterpret_cast<const v4i*>(bs_base + tok * 32 + 16);
        }
        constexpr int kQhOff = 2 + (kAffine ? 2 : 0), kQsOff = kQhOff + (kFive ? 4 : 0);
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const uint8_t* sb = blk + s * kB;
            // (s * kB + kQsOff) mod 4 is 2 for the even blocks of the 18- and 22-byte kinds, else 0
            constexpr bool kOddStride = kB % 4 == 2;
            const uint8_t* qp = sb + kQsOff + 8 * (kq & 1);
            uint32_t c0, c1;
            if (kOddStride && (s & 1) == 0) {
                const uint32_t w0 = *reinterpret_cast<const uint32_t*>(qp - 2), w1 = *reinterpret_cast<const uint32_t*>(qp + 2);
                const uint32_t w2 = *reinterpret_cast<const uint32_t*>(qp + 6);
                c0 = __builtin_amdgcn_alignbyte(w1, w0, 2);
                c1 = __builtin_amdgcn_alignbyte(w2, w1, 2);
            } else {
                c0 = *reinterpret_cast<const uint32_t*>(qp);
                c1 = *reinterpret_cast<const uint32_t*>(qp + 4);
            }
            const int sh = 4 * (kq >> 1);
            c0 = (c0 >> sh) & 0x0F0F0F0Fu;
            c1 = (c1 >> sh) & 0x0F0F0F0Fu;
            if (K == Nib32::IQ4_NL) {
                c0 = (uint32_t)iq4nl_lookup(c0);
                c1 = (uint32_t)iq4nl_lookup(c1);
            }
            if (kFive) {
                const uint32_t qh = (kOddStride && (s & 1) == 0) ? word_at<true>(sb + kQhOff) : word_at<false>(sb + kQhOff);
                const uint32_t h = qh >> (8 * kq);
                c0 |= spread4_to_bit4(h);
                c1 |= spread4_to_bit4(h >> 4);
            }
            const v2i b = {(int)c0, (int)c1};
            const v2i a = *reinterpret_cast<const v2i*>(arow + s * 32 + 8 * kq);
            const v4i r = __builtin_amdgcn_mfma_i32_16x16x32_i8(__builtin_bit_cast(long, a), __builtin_bit_cast(long, b),
                                                                v4i{0, 0, 0, 0}, 0, 0, 0);
            const float d = f16_bits_to_f32(*reinterpret_cast<const uint16_t*>(sb));
            const float mw = kAffine ? f16_bits_to_f32(*reinterpret_cast<const uint16_t*>(sb + 2)) : 0.0f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                raw[4 * s + i] = r[i];
                const float d8 = dq[i][s >> 2][s & 3];
                const int bsum = bs[i][s >> 2][s & 3];
                float term;
                if (kAffine) term = d8 * (d * (float)r[i] + mw * (float)bsum);
                else if (K == Nib32::IQ4_NL) term = (d * d8) * (float)r[i];
                else term = (d * d8) * (float)(r[i] - (kFive ? 16 : 8) * bsum);  // both integers and the difference are exact in f32
                ip[4 * s + i] = __builtin_bit_cast(int, term);
            }
        }
    }
    __device__ static void accumulate(float (&acc)[4], const float (&)[4], const uint32_t (&)[4], const int (&ip)[32]) {
#pragma unroll
        for (int s = 0; s < 8; ++s)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] += __builtin_bit_cast(float, ip[4 * s + i]);
    }
};

// NVFP4 (36-byte blocks of 64 weights [UE4M3 d[4]][qs[32]], four to a 256-element step: 144 bytes, like
// Q4_K's; crates/infr-cpu/src/kernels.rs:6472-6500): sub-block sb of a block (16 weights: the low
// nibbles of qs[8 sb .. 8 sb + 7] elements 0..7, the high nibbles 8..15) has its own halved UE4M3
// scale and meets half of a per-32 activation block, term d_sb * q8.d * iprod_sb. The K = 32 step of
// a 32-element activation block therefore runs twice, once with the operand bytes of the second
// sub-block zeroed and once with the first's: lanes kq = 0, 1 hold the first sub-block's K slots,
// kq = 2, 3 the second's. The two terms of a 32 are added before they join the chain.
struct Skinny16NVFP4 {
    typedef int v2i __attribute__((ext_vector_type(2)));
    static constexpr bool kSubScales = true, kPer32Acts = true, kTranspose16 = false;
    static constexpr int kBlockBytes = 144;
    static constexpr int kRowStride = 2 * kBlockBytes + 16;  // 76 words: eight rows' 16-byte reads cover all banks
    template <int MT, int DQ_STRIDE>
    __device__ static void block(const uint8_t* wrow, int jj, const uint8_t* arow, const uint8_t*,
                                 const float* dq_base, int kq, int (&ip)[32], int (&raw)[32]) {
        const uint8_t* blk = wrow + jj * kBlockBytes;
        v4f dq[4][2];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int tok = (4 * kq + i) & (MT - 1);
            dq[i][0] = *reinterpret_cast<const v4f*>(dq_base + tok * DQ_STRIDE + jj * 8);
            dq[i][1] = *reinterpret_cast<const v4f*>(dq_base + tok * DQ_STRIDE + jj * 8 + 4);
        }
        const bool second = kq >= 2;
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const uint8_t* nv = blk + 36 * (s >> 1);
            const int sb0 = 2 * (s & 1);  // the 32's sub-blocks sb0, sb0 + 1; this lane's own: sb0 + (kq >> 1)
            const uint8_t* qp = nv + 4 + 8 * (sb0 + (kq >> 1));
            const int sh = 4 * (kq & 1);
            const uint32_t c0 = (uint32_t)mxfp4_lookup((*reinterpret_cast<const uint32_t*>(qp) >> sh) & 0x0F0F0F0Fu);
            const uint32_t c1 = (uint32_t)mxfp4_lookup((*reinterpret_cast<const uint32_t*>(qp + 4) >> sh) & 0x0F0F0F0Fu);
            const v2i b0 = {second ? 0 : (int)c0, second ? 0 : (int)c1}, b1 = {second ? (int)c0 : 0, second ? (int)c1 : 0};
            const v2i a = *reinterpret_cast<const v2i*>(arow + s * 32 + 8 * kq);
            const v4i r0 = __builtin_amdgcn_mfma_i32_16x16x32_i8(__builtin_bit_cast(long, a), __builtin_bit_cast(long, b0),
                                                                 v4i{0, 0, 0, 0}, 0, 0, 0);
            const v4i r1 = __builtin_amdgcn_mfma_i32_16x16x32_i8(__builtin_bit_cast(long, a), __builtin_bit_cast(long, b1),
                                                                 v4i{0, 0, 0, 0}, 0, 0, 0);
            const uint32_t dw = *reinterpret_cast<const uint32_t*>(nv);
            const float w0 = ue4m3_half((dw >> (8 * sb0)) & 0xFFu), w1 = ue4m3_half((dw >> (8 * sb0 + 8)) & 0xFFu);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                raw[4 * s + i] = r0[i];
                const float d8 = dq[i][s >> 2][s & 3];
                const float term = (w0 * d8) * (float)r0[i] + (w1 * d8) * (float)r1[i];
                ip[4 * s + i] = __builtin_bit_cast(int, term);
            }
        }
    }
    __device__ static void accumulate(float (&acc)[4], const float (&)[4], const uint32_t (&)[4], const int (&ip)[32]) {
#pragma unroll
        for (int s = 0; s < 8; ++s)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] += __builtin_bit_cast(float, ip[4 * s + i]);
    }
};

template <typename F, int NW, int BPW, int MT, bool STAGES>
__global__ __launch_bounds__(NW * 64) void mmq_skinny16_kernel(
    const uint8_t* __restrict__ w, size_t bpr, const int8_t* __restrict__ qs,
    const float* __restrict__ d8, const int32_t* __restrict__ bsums, float* y, int m,
    int out_f, int nb, int32_t* __restrict__ st_sd, int32_t* __restrict__ st_sm,
    const BatchTile* __restrict__ tiles) {
    constexpr int kBlk = F::kBlockBytes;
    constexpr int kTokStride = 256 + 16;            // one token's codes of a block, padded against bank conflicts
    constexpr int kBsOff = MT * kTokStride;         // [token][8] per-32 sums
    constexpr int kZeroOff = kBsOff + MT * 32;      // 256 zero bytes: the codes of a token that is not there
    constexpr int kTileBytes = kZeroOff + 256;
    constexpr int kPh = BPW;                        // blocks of weights staged at a time: the wave's share of a pass
    constexpr int kRowStride = BPW == 2 ? F::kRowStride : kPh * kBlk + 16;
    // a row's stage in 16-byte pieces, and a last piece of one to three words (Q6_K: 420 = 26 x 16 + 4)
    constexpr int kFull = kPh * kBlk / 16, kTail = kPh * kBlk % 16;
    static_assert(kTail % 4 == 0, "a stage is whole 16-byte pieces plus at most three words");
    constexpr int kPieces = kFull + (kTail ? 1 : 0), kIt = (kPieces + 3) / 4;
    __shared__ __attribute__((aligned(16))) uint8_t w_l[NW][16 * kRowStride];
    __shared__ __attribute__((aligned(16))) uint8_t act_l[NW][kTileBytes];
    constexpr int kDq = BPW * (F::kPer32Acts ? 8 : 1);  // activation scales per token and pass: per 256 or per 32
    __shared__ __attribute__((aligned(16))) float dq_l[NW][MT][kDq];
    __shared__ __attribute__((aligned(16))) float chain_l[64][4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r16 = lane & 15, kq = lane >> 4;
    const int tok0 = (int)blockIdx.z * 16;  // batches beyond 16 tokens: one pass over the weights per 16
    const int rt = blockIdx.y * 16 + r16;  // row inside the 32-row tile
    const size_t in_f = (size_t)nb * 256;
    int wrow = blockIdx.x * 32 + rt;
    bool row_ok = wrow < out_f;
    bool any_row = (int)blockIdx.x * 32 + (int)blockIdx.y * 16 < out_f;
    BatchAdd add;
    if (tiles) {
        const BatchTile t = tiles[blockIdx.x];
        w = t.w;
        bpr = t.bpr;
        y = t.y;
        add = BatchAdd{t.add_b, t.add_dst};
        out_f = (int)t.out_f;
        wrow = rt;
        row_ok = rt < (int)t.rows;
        any_row = (int)blockIdx.y * 16 < (int)t.rows;
        qs += t.act_elem0;
        d8 += t.act_elem0 / (F::kPer32Acts ? 32 : 256);
        bsums += t.act_elem0 / 32;
    }
    if (!any_row) return;  // uniform over the workgroup, before any barrier
    // K in passes of NW * BPW blocks; in a pass wave w owns blocks (pass * NW + w) * BPW .. + BPW - 1
    const int n_pass = (nb + NW * BPW - 1) / (NW * BPW);
    // Weight stage: lane (row = lane / 4, pq = lane % 4) takes the 16-byte pieces pq, pq + 4, .. of its
    // row's BPW blocks - a quad of lanes fetches 64 contiguous bytes - so every address is one
    // per-lane offset plus a constant; rows past the matrix repeat the half's first row (their
    // outputs are never stored).
    const int rows_here = (tiles ? (int)tiles[blockIdx.x].rows : out_f - (int)blockIdx.x * 32) - (int)blockIdx.y * 16;
    const uint8_t* wbase = w + (size_t)(wrow - r16) * bpr;  // first row of this half
    const int srow = lane >> 2, pq = lane & 3;
    const uint32_t goff = (uint32_t)((srow < rows_here ? srow : 0) * bpr) + pq * 16;
    const uint32_t loff = srow * kRowStride + pq * 16;
    v4i wreg[kIt];
    auto request_rows = [&](int b) {  // blocks b .. b + BPW - 1; past the end: a redundant stage, never used
        const uint8_t* src = wbase + (size_t)min(b, nb - kPh) * kBlk;
#pragma unroll
        for (int it = 0; it < kIt; ++it) {
            if (pq + 4 * it < kFull) wreg[it] = kBlk % 16 == 0 ? load16(src + goff + 64 * it) : load16_a4(src + goff + 64 * it);
            else if (kTail && pq + 4 * it == kFull) {
                wreg[it].x = load_u32(src + goff + 64 * it);
                if (kTail >= 8) wreg[it].y = load_u32(src + goff + 64 * it + 4);
                if (kTail >= 12) wreg[it].z = load_u32(src + goff + 64 * it + 8);
            }
        }
    };
    uint8_t* wl = w_l[wave];
    auto publish_rows = [&]() {
#pragma unroll
        for (int it = 0; it < kIt; ++it) {
            if (pq + 4 * it < kFull) *reinterpret_cast<v4i*>(wl + loff + 64 * it) = wreg[it];
            else if (kTail && pq + 4 * it == kFull) {
                int* dst = reinterpret_cast<int*>(wl + loff + 64 * it);
                dst[0] = wreg[it].x;
                if (kTail >= 8) dst[1] = wreg[it].y;
                if (kTail >= 12) dst[2] = wreg[it].z;
            }
        }
    };
    const uint8_t* wfrag = wl + r16 * kRowStride;
    // a block's activations: 16-byte piece `chunk & 15` of token `chunk >> 4` (absent tokens repeat the
    // last one: their products land in accumulators that are never stored)
    v4i areg[MT / 4], bsreg = {0, 0, 0, 0};
    uint32_t aoff[MT / 4];
#pragma unroll
    for (int it = 0; it < MT / 4; ++it) aoff[it] = (uint32_t)min(tok0 + (lane >> 4) + 4 * it, m - 1) * (uint32_t)in_f + (lane & 15) * 16;
    const uint32_t boff = (uint32_t)min(tok0 + (lane >> 1), m - 1) * (uint32_t)(nb * 32) + (lane & 1) * 16;
    auto request_acts = [&](int b_) {
        const int b = min(b_, nb - 1);
        const int8_t* src = qs + (size_t)b * 256;
        const uint8_t* bsrc = reinterpret_cast<const uint8_t*>(bsums) + (size_t)b * 32;
#pragma unroll
        for (int it = 0; it < MT / 4; ++it) areg[it] = *reinterpret_cast<const v4i*>(src + aoff[it]);
        if (lane < MT * 2) bsreg = *reinterpret_cast<const v4i*>(bsrc + boff);
    };
    uint8_t* tile = act_l[wave];
    auto publish_acts = [&]() {
#pragma unroll
        for (int it = 0; it < MT / 4; ++it) {
            const int chunk = lane + 64 * it;
            v4i piece = areg[it];
            if constexpr (F::kTranspose16) {
                // the piece's 16 codes 4 x 4 transposed: word i = codes i, 4 + i, 8 + i, 12 + i
                const uint32_t d0 = (uint32_t)piece.x, d1 = (uint32_t)piece.y, d2 = (uint32_t)piece.z, d3 = (uint32_t)piece.w;
                const uint32_t a = __builtin_amdgcn_perm(d1, d0, 0x05010400u), b = __builtin_amdgcn_perm(d1, d0, 0x07030602u);
                const uint32_t c = __builtin_amdgcn_perm(d3, d2, 0x05010400u), d = __builtin_amdgcn_perm(d3, d2, 0x07030602u);
                piece = v4i{(int)__builtin_amdgcn_perm(c, a, 0x05040100u), (int)__builtin_amdgcn_perm(c, a, 0x07060302u),
                            (int)__builtin_amdgcn_perm(d, b, 0x05040100u), (int)__builtin_amdgcn_perm(d, b, 0x07060302u)};
            }
            *reinterpret_cast<v4i*>(tile + (chunk >> 4) * kTokStride + (chunk & 15) * 16) = piece;
        }
        if (lane < MT * 2) *reinterpret_cast<v4i*>(tile + kBsOff + lane * 16) = bsreg;
    };
    // the wave's lanes exchange data through its own LDS tiles: order the tiles' writes and reads
    auto wave_sync = [&]() {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    // this lane as A operand: token r16 (rows of absent tokens hold another token's codes)
    const uint8_t* afrag = tile + (r16 & (MT - 1)) * kTokStride;
    const uint8_t* bsfrag = tile + kBsOff + (r16 & (MT - 1)) * 32;
    const uint8_t* zrow = tile + kZeroOff;
    *reinterpret_cast<int*>(tile + kZeroOff + lane * 4) = 0;  // ordered before the first read by the loop's wave_sync

    uint32_t dqoff[(MT * BPW + 63) / 64];
#pragma unroll
    for (int it = 0; it < (MT * BPW + 63) / 64; ++it) {
        const int i = lane + 64 * it;
        dqoff[it] = (uint32_t)min(tok0 + i / BPW, m - 1) * (uint32_t)nb + i % BPW;
    }
    // per-32 activations: a pass's scales of a token are 8 BPW consecutive floats, four to a lane
    constexpr int kDqQuads = BPW * 2;  // 16-byte pieces per token and pass
    const uint32_t dq32off = (uint32_t)min(tok0 + lane / kDqQuads, m - 1) * (uint32_t)(nb * 8) + (lane % kDqQuads) * 4;
    static_assert(!F::kPer32Acts || MT * kDqQuads <= 64, "one 16-byte piece of scales per lane");
    request_rows(wave * BPW);
    request_acts(wave * BPW);
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};  // this lane's outputs: tokens 4kq .. 4kq + 3 of row r16
    for (int pass = 0; pass < n_pass; ++pass) {
        const int b0 = (pass * NW + wave) * BPW;
        const int b0_next = b0 + NW * BPW;  // next pass (past the end: clamped, never used)
        // A row of an odd number of blocks ends in a stage of one block: that stage starts a block
        // early (request_rows), so block b0 + j sits in slot (j + 1) % BPW of the weight tile and of
        // the scales; the slot that holds the block before is never summed (b0 + j < nb below).
        const int slot0 = BPW == 2 && b0 == nb - 1 ? 1 : 0;
        // the activation scales of the wave's blocks: dq_l[token][j]
        if constexpr (F::kPer32Acts) {
            if (lane < MT * kDqQuads)
                *reinterpret_cast<v4f*>(&dq_l[wave][0][0] + lane * 4) =
                    *reinterpret_cast<const v4f*>(d8 + (size_t)min(b0, nb - BPW) * 8 + dq32off);
        } else {
            const float* dsrc = d8 + min(b0, nb - BPW);
#pragma unroll
            for (int it = 0; it < (MT * BPW + 63) / 64; ++it)
                if (lane + 64 * it < MT * BPW) (&dq_l[wave][0][0])[lane + 64 * it] = dsrc[dqoff[it]];
        }
        constexpr bool kSub = F::kSubScales;  // a step's integers: one per output, or one per 32-block and output
        int sd[BPW][kSub ? 32 : 4];
        float sm[BPW][4];
        uint32_t ddm[BPW][kSub ? 4 : 1];  // (d, dmin) of this lane's row, or the step's eight block scales
#pragma unroll
        for (int j = 0; j < BPW; ++j) {
            wave_sync();  // the previous block's operand reads are done
            publish_acts();
            if (j + 1 < BPW) request_acts(b0 + j + 1);
            else if (pass + 1 < n_pass) request_acts(b0_next);
            if (j == 0) {
                publish_rows();
                if (pass + 1 < n_pass) request_rows(b0_next);
            }
            wave_sync();
            int raw[kSub && F::kPer32Acts ? 32 : 1];  // the integers behind a policy's f32 terms (stage outputs)
            const int slot = (j + slot0) % kPh;
            if constexpr (kSub && F::kPer32Acts)
                F::template block<MT, kDq>(wfrag, slot, afrag, tile + kBsOff, &dq_l[wave][0][0], kq, sd[j], raw);
            else if constexpr (kSub) F::block(wfrag, slot, afrag, kq, sd[j], ddm[j]);
            else F::block(wfrag, slot, afrag, zrow, bsfrag, kq, sd[j], sm[j], ddm[j][0]);
            if (STAGES) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int tok = tok0 + 4 * kq + i;
                    if (row_ok && tok < m && b0 + j < nb) {
                        if constexpr (kSub) {
#pragma unroll
                            for (int s8 = 0; s8 < 8; ++s8)
                                st_sd[((size_t)tok * out_f + wrow) * ((size_t)nb * 8) + (size_t)(b0 + j) * 8 + s8] =
                                    F::kPer32Acts ? raw[F::kPer32Acts ? 4 * s8 + i : 0] : sd[j][4 * s8 + i];
                        } else {
                            st_sd[((size_t)tok * out_f + wrow) * nb + b0 + j] = sd[j][i];
                            if (st_sm) st_sm[((size_t)tok * out_f + wrow) * nb + b0 + j] = (int)sm[j][i];
                        }
                    }
                }
            }
        }
        wave_sync();  // dq_l was written by this wave's lanes

        // f32 epilogue handed down the waves: the format's CPU expression per block, b ascending
#pragma unroll
        for (int k = 0; k < NW; ++k) {
            if (wave == k) {
                if (k > 0 || pass > 0) {
                    const v4f prev = *reinterpret_cast<const v4f*>(&chain_l[lane][0]);
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[i] = prev[i];
                }
#pragma unroll
                for (int j = 0; j < BPW; ++j) {
                    if (b0 + j < nb) {
                        if constexpr (kSub) {
                            float dqv[4];
#pragma unroll
                            for (int i = 0; i < 4; ++i) dqv[i] = dq_l[wave][(4 * kq + i) & (MT - 1)][(j + slot0) % BPW];
                            F::accumulate(acc, dqv, ddm[j], sd[j]);
                        } else {
#pragma unroll
                            for (int i = 0; i < 4; ++i)
                                acc[i] = F::accumulate(acc[i], dq_l[wave][(4 * kq + i) & (MT - 1)][(j + slot0) % BPW], ddm[j][0], sd[j][i], sm[j][i]);
                        }
                    }
                }
                if (k + 1 < NW || pass + 1 < n_pass)
                    *reinterpret_cast<v4f*>(&chain_l[lane][0]) = v4f{acc[0], acc[1], acc[2], acc[3]};
            }
            if (k + 1 < NW || pass + 1 < n_pass) __syncthreads();
        }
    }
    if (wave != NW - 1 || !row_ok) return;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int tok = tok0 + 4 * kq + i;
        if (tok < m) store_batch_out(y, add, (size_t)tok * out_f + wrow, acc[i]);
    }
}

// Which batches the 16-token K-split kernel takes: rows (of any quantized format) of two 256-blocks
// and more. Weights are staged two blocks at a time; a row of an odd number ends in a stage that starts
// a block early, which needs every block 16-byte aligned in every row - not so for Q6_K (210 bytes) and
// Q2_0 (72): their rows must be an even number of blocks. Four waves per workgroup;
// (eight measured no faster, and four blocks per wave and pass - 576-byte, 64-byte-aligned runs per
// row - measured 20-25 % slower: a wave then computes for longer before it asks for more).
constexpr int kSkinny16Waves = 4, kSkinny16Blocks = 2;
static bool skinny16_shape(int dtype, int nb, size_t m, size_t out_f) {
    const bool nib32 = dtype == 2 || dtype == 3 || dtype == 6 || dtype == 7 || dtype == 20;
    if (dtype != 12 && dtype != 13 && dtype != 14 && dtype != 8 && dtype != 42 && dtype != 10 && dtype != 11 && dtype != 23 && dtype != 35 && dtype != 40 && !nib32)
        return false;
    if (nb < kSkinny16Blocks || (nb % kSkinny16Blocks != 0 && (dtype == 14 || dtype == 42 || dtype == 11 || dtype == 35))) return false;
    // Q2_K, Q3_K, IQ4_XS, TQ2_0 up to 16 tokens: the dot4 batches are the only other kernel there, eight tokens per
    // pass over the weights; beyond, their 128-token tile kernels take over as measured below
    // IQ4_XS has a 128-token tile kernel whose time is flat up to 128 tokens (30 / 59 / 22 us at 12288 x 4096,
    // 4096 x 12288, 4096 x 4096) where a 16-token pass here costs 8.2 / 8.0 / 2.8: it takes over at 49 tokens
    // on large matrices of 4096-column rows, at 113 on long rows and small matrices
    // Narrow matrices at any token count: a 128-token tile kernel walks a whole row per workgroup,
    // so its time has a floor however few rows there are (26-29 us at 4096 columns for Q5_K, Q8_0 and
    // IQ4_XS, 41 for Q6_K: a 1024-row projection at 128..512 tokens is 32..128 workgroups), while a
    // pass here costs its share of the outputs. The two meet at about 700 K outputs for Q5_K, 1 M for
    // Q6_K, 600 K for IQ4_XS and Q2_K, 700 K for Q3_K and TQ2_0, 640 K for Q8_0 (1024 x 4096 at 128 / 256 / 512 tokens: Q5_K 26.7 / 27.8 /
    // 29.5 us on the tiles, 5.7 / 10.2 / 19.0 here; Q6_K 7.9 / 41.4 / 43.1 and 7.8 / 9.5 / 17.6), 768 K for
    // the 32-weight-block formats (Q4_0 at 256 / 512 tokens: 62 / 65 us on the tiles), 600 K for Q2_0 (44 / 47). Independent of the row length: both scale with it.
    if (m > (size_t)16 * 65535) return false;  // (the grid's third dimension walks the batch 16 tokens at a time)
    // NVFP4: from nine tokens (the dot4 batches take eight a pass) up to where its tiles take over - a 16-token
    // pass costs 34 / 31 / 12 us (12288 x 4096, 4096 x 12288, 4096 x 4096: two half-empty MFMAs per 32 weights),
    // the tiles a flat 69 / 166 / 55
    if (dtype == 40)
        return m >= 9 && (out_f == 0 || m <= ((out_f * (size_t)nb <= (size_t)4096 * 16 || nb >= 32) ? 80u : 32u));
    if (m > 16 && out_f == 0 && dtype != 12) return true;  // (a plan's group: its ops were taken one by one)
    if (m > 16) {
        const size_t outputs = m * out_f;
        if ((dtype == 13 && outputs <= (size_t)700 * 1024) || (dtype == 14 && outputs <= (size_t)1024 * 1024) ||
            ((dtype == 23 || dtype == 10) && outputs <= (size_t)600 * 1024) ||
            ((dtype == 11 || dtype == 35) && nb % kSkinny16Blocks == 0 && outputs <= (size_t)700 * 1024) || (dtype == 8 && outputs <= (size_t)640 * 1024) ||
            (nib32 && outputs <= (size_t)768 * 1024) || (dtype == 42 && outputs <= (size_t)600 * 1024))
            return true;
    }
    // Q2_K's 128-token tiles (mmq_q2k.hip) are flat up to 128 tokens at 23 / 45 / 18 us (12288 x 4096, 4096 x 12288,
    // 4096 x 4096) where a 16-token pass here costs 5.8 / 5.4 / 2.0: they take over at 65 tokens on large matrices
    // of 4096-column rows, at 129 on long rows and small matrices
    // Q3_K and TQ2_0 (mmq_q3k.hip): tiles flat at 36 / 70 / 25 us and 23 / 44 / 17 us up to 128 tokens, a 16-token
    // pass here 6.6 / 6.3 / 2.3 and 4.4 / 4.4 / 1.6: from 97 (Q3_K) and 81 (TQ2_0) tokens on large matrices of
    // 4096-column rows, from 161 on long rows and small matrices
    if ((dtype == 11 || dtype == 35) && m > 16)
        return m <= ((out_f == 0 || out_f * (size_t)nb <= (size_t)4096 * 16 || nb >= 32) ? 160u : (dtype == 11 ? 96u : 80u));
    if (dtype == 10 && m > 16) return m <= ((out_f == 0 || out_f * (size_t)nb <= (size_t)4096 * 16 || nb >= 32) ? 128u : 64u);
    if (dtype == 23 && m > 16) return m <= ((out_f == 0 || out_f * (size_t)nb <= (size_t)4096 * 16 || nb >= 32) ? 112u : 48u);
    if (dtype == 10 || dtype == 11 || dtype == 23 || dtype == 35) return m >= 3;
    if (m <= 16) {
        // the dot4 batch kernels, which unpack a weight once per two or four tokens, stay ahead at the
        // bottom: Q4_K at two tokens (4.3 / 4.0 / 5.5 / 5.6 against 3.7 / 3.4 / 4.2 / 4.2 TB/s on the four
        // layer shapes; level from three), Q5_K at two (4.3-5.3 against 3.8-4.4), Q6_K up to four
        // (3.6-4.5 against 3.3-3.9)
        if ((dtype == 12 && m < 3) || (dtype == 13 && m < 3) || (dtype == 14 && m < 5)) return false;
        // Q8_0: the dot4 batches stay ahead up to eight tokens (4.2 / 3.8 / 4.8 against 3.8 / 3.3 / 4.2 TB/s
        // at eight tokens on the 4096-column shapes, 5.1-5.9 at two to four; on rows of 8192 columns and
        // more this kernel is ahead by a tenth when forty such ops share a launch, 4.4 against 3.95 TB/s,
        // but a single 4096 x 12288 op - what a layer has - takes 29 us here against 19 there: a plan's
        // group of 8192 rows and more comes here from five tokens, out_f == 0); this kernel takes
        // 9..16 tokens (one pass over the weights instead of two)
        if (dtype == 8 && m <= 8 && !(out_f == 0 && m >= 5 && nb >= 32)) return false;
        // Q2_0: 72 bytes a step make this kernel compute-bound (1.0-1.3 TB/s at any token count, what the
        // dot4 batches reach at eight tokens): it takes 9 tokens and more, where they would need two passes
        if (dtype == 42 && m <= 8) return false;
        // the 32-weight-block formats: as Q2_0 (12288 x 4096 at eight tokens: 10-12 us on the dot4 batches, 14-15 here)
        if (nib32 && m <= 8) return false;
        return true;
    }
    // Beyond 16 tokens the grid's third dimension walks the batch 16 tokens at a time (the weights
    // then come once per 16 tokens, the later times from cache): taken while that beats what else
    // the format has - dot4 passes of eight tokens up to 32 / 64 tokens, then a 128-token MFMA tile
    // whose time is flat in the token count and has a floor of 26-42 us however small the matrix.
    // Per op, us, at 12288 x 4096 / 4096 x 12288 / 4096 x 4096 / 1024 x 4096:
    //   Q6_K  a 16-token pass 10.6 / 10.4 / 3.3 / 0.95; before: 68-114 at 17..32, then 61 / 102 / 40 / 40
    //   Q5_K  9.2 / 8.8 / 2.9 / 0.8; 52-85, then 35 / 65 / 26 / 26
    //   Q8_0  15.4 / 15.2 / 6.1 / 1.8; 51-71, then 46-50 / 73 / 30 / 28
    //   Q2_0  12.5 / 10.7 / 4.1 / 1.2; 44-74 at 17..32, 79-144 at 33..64, then 51 / 120 / 42 / 41
    // out_f == 0: the caller has decided already.
    const bool long_rows = nb >= 32;                                          // 8192 columns and more
    const bool small = out_f == 0 || out_f * (size_t)nb <= (size_t)4096 * 16;  // up to 4096 x 4096 weights
    if (dtype == 12) {
        // Q4_K keeps its 32-token K-split kernel up to 32 tokens (10.6-12.9 against 16 us at 12288 x 4096)
        // and its 32-token tiles on large matrices of 4096-column rows (31 us flat from 33 to 127
        // tokens; this kernel 29 at 33..48, 36 at 64). Those tiles cost 80 us on 4096 x 12288 and have a
        // floor of 26 us on small matrices: there this kernel takes 33 tokens and up (4096 x 12288:
        // 24 / 32 / 48 us at 33 / 64 / 96 tokens; 4096 x 4096: 7.6 / 9.8 / 14; 1024 x 4096: 2.7 / 3.3 / 4.4).
        if (m <= 32) return false;
        if (out_f == 0) return true;
        // Beyond that this kernel runs at ~225 TOP/s whatever the shape (it unpacks a block once per
        // 16 tokens), while the tiled kernels have a floor: a workgroup walks a whole row, ~1.6 us per
        // 256-block, however few workgroups there are. The two meet at about 640 K outputs (measured at
        // 1024 / 2048 / 4096 x 4096 and 4096 x 12288, 128 to 1024 tokens: 1024 x 4096 at 512 tokens takes
        // 19 us here and 27 on the tiles, 4096 x 4096 at 192 tokens 29 against 25).
        return m * out_f <= (size_t)640 * 1024;
    }
    //   Q4_0, Q4_1, Q5_0, Q5_1, IQ4_NL  14-16 / 12-14 / 5.0-5.7; before: 41 at 16 tokens, 76 at 32, 147 at 64,
    //         then 59-71 / 130-180 / 50-64
    if (nib32) return m <= (small || long_rows ? 128 : 64);
    const size_t top = dtype == 13   ? (small || long_rows ? 96 : 48)
                       : dtype == 14 ? (small || long_rows ? 128 : 80)
                       : dtype == 8  ? (small || long_rows ? 64 : 32)
                                     : (small || long_rows ? 128 : 64);
    return m <= top;
}

bool mmq_skinny16_takes(int dtype, size_t m, size_t in_f, size_t out_f) {
    return in_f % 256 == 0 && skinny16_shape(dtype, (int)(in_f / 256), m, out_f);
}

template <typename F, bool STAGES>
static void launch_mmq_skinny16_fmt(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m, int nb,
                                    size_t out_f, size_t wgs, const IntStages& st, const BatchTile* tiles,
                                    hipStream_t stream) {
    const dim3 grid((unsigned)wgs, 2, (unsigned)((m + 15) / 16)), block(kSkinny16Waves * 64);
    // At most one workgroup per compute unit (one op of up to 4096 rows and 16 tokens: a down
    // projection on its own level of a plan) and long rows: eight waves share a row's blocks
    // instead of four, twice the requests in flight (4096 x 12288 at 8 tokens, per call with its
    // quantizer: Q4_K 17.4 -> 15.3 us, Q8_0 at 16 tokens 29.2 -> 27.3). With more workgroups than
    // that the four-wave form is as fast or faster (512 workgroups: 33 against 49 us).
    if constexpr (!STAGES) {
        if (wgs * 2 * grid.z <= 256 && nb >= 32) {
            if (m <= 8)
                hipLaunchKernelGGL((mmq_skinny16_kernel<F, 8, kSkinny16Blocks, 8, false>), grid, dim3(512), 0, stream,
                                   w, bpr, act.qs, act.d, act.bsums, y, (int)m, (int)out_f, nb, st.a, st.b, tiles);
            else
                hipLaunchKernelGGL((mmq_skinny16_kernel<F, 8, kSkinny16Blocks, 16, false>), grid, dim3(512), 0, stream,
                                   w, bpr, act.qs, act.d, act.bsums, y, (int)m, (int)out_f, nb, st.a, st.b, tiles);
            return;
        }
    }
    if (m <= 8)
        hipLaunchKernelGGL((mmq_skinny16_kernel<F, kSkinny16Waves, kSkinny16Blocks, 8, STAGES>), grid, block, 0, stream,
                           w, bpr, act.qs, act.d, act.bsums, y, (int)m, (int)out_f, nb, st.a, st.b, tiles);
    else
        hipLaunchKernelGGL((mmq_skinny16_kernel<F, kSkinny16Waves, kSkinny16Blocks, 16, STAGES>), grid, block, 0, stream,
                           w, bpr, act.qs, act.d, act.bsums, y, (int)m, (int)out_f, nb, st.a, st.b, tiles);
}

template <bool STAGES>
static bool launch_mmq_skinny16(int dtype, const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m,
                                size_t in_f, size_t out_f, size_t wgs, const IntStages& st, const BatchTile* tiles,
                                hipStream_t stream) {
    const int nb = (int)(in_f / 256);
    if (in_f % 256 != 0 || !skinny16_shape(dtype, nb, m, out_f)) return false;
    if (dtype == 12)
        launch_mmq_skinny16_fmt<Skinny16Q4K, STAGES>(w, bpr, act, y, m, nb, out_f, wgs, st, tiles, stream);
    else if (dtype == 13)
        launch_mmq_skinny16_fmt<Skinny16Q5K, STAGES>(w, bpr, act, y, m, nb, out_f, wgs, st, tiles, stream);
    else if (dtype == 8)
        launch_mmq_skinny16_fmt<Skinny16Q8_0, STAGES>(w, bpr, act, y, m, nb, out_f, wgs, st, tiles, stream);
    else if (dtype == 42)
        launch_mmq_skinny16_fmt<Skinny16Q2_0, STAGES>(w, bpr, act, y, m, nb, out_f, wgs, st, tiles, stream);
    else if (dtype == 2)
        launch_mmq_skinny16_fmt<Skinny16Nib32<Nib32::Q4_0>, STAGES>(w, bpr, act, y, m, nb, out_f, wgs, st, tiles, stream);
    else if (dtype == 3)
        launch_mmq_skinny16_fmt<Skinny16Nib32<Nib32::Q4_1>, STAGES>(w, bpr, act, y, m, nb, out_f, wgs, st, tiles, stream);
    else if (dtype == 6)
        launch_mmq_skinny16_fmt<Skinny16Nib32<Nib32::Q5_0>, STAGES>(w, bpr, act, y, m, nb, out_f, wgs, st, tiles, stream);
    else if (dtype == 7)
        launch_mmq_skinny16_fmt<Skinny16Nib32<Nib32::Q5_1>, STAGES>(w, bpr, act, y, m, nb, out_f, wgs, st, tiles, stream);
    else if (dtype == 20)
        launch_mmq_skinny16_fmt<Skinny16Nib32<Nib32::IQ4_NL>, STAGES>(w, bpr, act, y, m, nb, out_f, wgs, st, tiles, stream);
    else if (dtype == 40)
        launch_mmq_skinny16_fmt<Skinny16NVFP4, STAGES>(w, bpr, act, y, m, nb, out_f, wgs, st, tiles, stream);
    else if (dtype == 10)
        launch_mmq_skinny16_fmt<Skinny16Q2K, STAGES>(w, bpr, act, y, m, nb, out_f, wgs, st, tiles, stream);
    else if (dtype == 11)
        launch_mmq_skinny16_fmt<Skinny16Q3K, STAGES>(w, bpr, act, y, m, nb, out_f, wgs, st, tiles, stream);
    else if (dtype == 23)
        launch_mmq_skinny16_fmt<Skinny16IQ4XS, STAGES>(w, bpr, act, y, m, nb, out_f, wgs, st, tiles, stream);
    else if (dtype == 35)
        launch_mmq_skinny16_fmt<Skinny16TQ2_0, STAGES>(w, bpr, act, y, m, nb, out_f, wgs, st, tiles, stream);
    else
        launch_mmq_skinny16_fmt<Skinny16Q6K, STAGES>(w, bpr, act, y, m, nb, out_f, wgs, st, tiles, stream);
    return true;
}

void launch_mmq_skinny_group(int dtype, size_t m, size_t in_f, const BatchTile* tiles_dev,
                             const BatchGroupPlan& plan, const ActQ8& act, hipStream_t stream) {
    if (launch_mmq_skinny16<false>(dtype, nullptr, 0, act, nullptr, m, in_f, 0, plan.total_wgs, IntStages{}, tiles_dev,
                                   stream))
        return;
    const dim3 grid((unsigned)plan.total_wgs, (unsigned)((m + 31) / 32));
    const int nb = (int)(in_f / 256);
    if (plan.waves == 8)
        hipLaunchKernelGGL((mmq_skinny_q4k_kernel<8, false>), grid, dim3(512), 0, stream, (const uint8_t*)nullptr,
                           (size_t)0, act.qs, act.d, act.bsums, (float*)nullptr, (int)m, 0, nb,
                           (int32_t*)nullptr, (int32_t*)nullptr, tiles_dev);
    else
        hipLaunchKernelGGL((mmq_skinny_q4k_kernel<4, false>), grid, dim3(256), 0, stream, (const uint8_t*)nullptr,
                           (size_t)0, act.qs, act.d, act.bsums, (float*)nullptr, (int)m, 0, nb,
                           (int32_t*)nullptr, (int32_t*)nullptr, tiles_dev);
}

template <int BM>
static void launch_mmq_q4k(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m,
                           size_t in_f, size_t out_f, const IntStages& st, hipStream_t stream) {
    const dim3 grid((unsigned)((out_f + 127) / 128), (unsigned)((m + BM - 1) / BM)), block(256);
    const int nb = (int)(in_f / 256);
    if (st.a)
        hipLaunchKernelGGL((mmq_q4k_kernel<BM, true, DenseTiles>), grid, block, 2 * MmqLds<BM>::bytes, stream, w,
                           bpr, act.qs, act.d, act.bsums, y, DenseTiles{(int)m}, (int)out_f, nb, st.a, st.b);
    else
        hipLaunchKernelGGL((mmq_q4k_kernel<BM, false, DenseTiles>), grid, block, 2 * MmqLds<BM>::bytes, stream, w,
                           bpr, act.qs, act.d, act.bsums, y, DenseTiles{(int)m}, (int)out_f, nb, (int32_t*)nullptr,
                           (int32_t*)nullptr);
}

void launch_mmq_q4k_gathered(const uint8_t* bank, size_t expert_stride, size_t bpr, const ActQ8& act, int act_div,
                             const MoeTileTable& t, float* y, size_t in_f, size_t out_f, hipStream_t stream) {
    const dim3 grid((unsigned)((out_f + 127) / 128), (unsigned)t.max_tiles), block(256);
    const GatheredTiles g{t.n_tiles, t.expert, t.slot0, t.count, t.perm, expert_stride, act_div};
    hipLaunchKernelGGL((mmq_q4k_kernel<32, false, GatheredTiles>), grid, block, 2 * MmqLds<32>::bytes, stream, bank,
                       bpr, act.qs, act.d, act.bsums, y, g, (int)out_f, (int)(in_f / 256), (int32_t*)nullptr,
                       (int32_t*)nullptr);
}

// Whether Q4_K Linears of `m` tokens over one activation tensor, `total_out_f` rows between them, run
// as one grouped strip launch inside a plan: the token counts launch_mmq sends to the strip kernel,
// on rows the decode mapping covers, when the rows together are past the 16-token kernel's reach.
bool mmq_q4k_strip_group_takes(size_t m, size_t in_f, size_t total_out_f) {
    if (in_f % 256 != 0 || gemv_row_too_long(12, in_f) || m < 128) return false;
    const size_t groups256 = (m + 255) / 256;
    if ((double)m < 0.6 * (double)(groups256 * 256)) return false;
    return !mmq_skinny16_takes(12, m, in_f, total_out_f);
}

bool launch_mmq(int dtype, const uint8_t* w, size_t bpr, const float* x, const ActQ8& act, float* y,
                size_t m, size_t in_f, size_t out_f, const IntStages& st, int cus, hipStream_t stream,
                QuantCache* qc) {
    // the activation quantizers, skipped when the scratch already holds this tensor in this layout
    auto have = [&](int layout) {
        if (qc && qc->x == x && qc->m == m && qc->in_f == in_f && qc->layout == layout) return true;
        if (qc) *qc = QuantCache{x, m, in_f, layout};
        return false;
    };
    auto quantize_rows = [&](bool per32) {
        if (!have(per32 ? 2 : 1)) launch_quantize_q8(x, m, in_f, per32, act, stream);
    };
    auto quantize_tiled = [&] {
        if (!have(3)) launch_quantize_q8_tiled(x, m, in_f, act, stream);
    };
    auto quantize_32_tiled = [&](bool transposed16) {
        if (!have(transposed16 ? 5 : 4)) launch_quantize_q8_32_tiled(x, m, in_f, transposed16, act, stream);
    };
    // Q4_K routes by token count (thresholds from sweeps at K = 4096, N = 12288):
    //   2..32      skinny kernel, K split over the waves of a workgroup
    //   33..127    tiled kernel, 32 tokens x 128 rows per workgroup (most workgroups for few tokens)
    //   128..      shared-operand kernel, 128 tokens x 32 rows (x 64 rows from 1024 tokens up)
    // Q5_K, Q6_K from 33 tokens, Q8_0 (33) and the 32-weight-block formats (65) on rows of whole 256s:
    // their own shared-operand MFMA kernels (mmq_q5k.hip, mmq_q6k.hip, mmq_q8_0.hip,
    // mmq_nib32.hip). Otherwise the other
    // formats take the dot4 GEMV with the activations of up to eight rows in registers (weights
    // re-streamed once per eight rows beyond that).
    // rows beyond the decode / small-batch kernels' length, when whole 256s, take the MFMA kernel of
    // their format at any token count (a 128-token tile for one token: slow, but exact and bounded)
    const bool long_row = gemv_row_too_long(dtype, in_f) && in_f % 256 == 0;
    // the 16-token K-split kernel where it is ahead beyond 16 tokens (up to 32..128 by format and shape)
    if (!long_row && (dtype != 12 || m > 32) && mmq_skinny16_takes(dtype, m, in_f, out_f)) {
        quantize_rows(act_is_per32(dtype, in_f));
        const size_t wgs = (out_f + 31) / 32;
        return st.a ? launch_mmq_skinny16<true>(dtype, w, bpr, act, y, m, in_f, out_f, wgs, st, nullptr, stream)
                    : launch_mmq_skinny16<false>(dtype, w, bpr, act, y, m, in_f, out_f, wgs, st, nullptr, stream);
    }
    if (dtype == 12 && (m >= 128 || long_row)) {
        quantize_tiled();
        // From 128 tokens up y is held to 1e-4 of infr-cpu, not to its bits (the integers stay exact):
        // the strip kernel contracts the f32 epilogue. The integer-stage entry point keeps the exact form.
        // Strips are 256 tokens wide: a batch that fills less than ~0.6 of its 256-token groups (128..153,
        // 257..307 tokens) takes the 128-token tiles of the shared-operand kernel instead.
        const size_t groups256 = (m + 255) / 256;
        int tiles = (double)m >= 0.6 * (double)(groups256 * 256) ? mmq_strip_q4k_tiles(m, out_f, in_f, cus) : 0;
        // One-tile strips that cover at most half of the compute units (4096 rows at up to 256 tokens): the
        // 128-token tiles are twice the workgroups (4096 x 12288 at 200 / 256 tokens: 64 / 66 us against 78 / 79;
        // 4096 x 4096: 26 against 30).
        if (tiles == 1 && ((out_f + 31) / 32) * groups256 * 2 <= (size_t)(cus > 0 ? cus : 256)) tiles = 0;
        if (tiles > 0) launch_mmq_strip_q4k(w, bpr, act, y, m, in_f, out_f, st, tiles, st.a != nullptr, stream);
        else launch_mmq_shared_q4k<1>(w, bpr, act, y, m, in_f, out_f, st, stream);
        return true;
    }
    // Q6_K: the MFMA kernel's time is flat up to 128 tokens (63 / 103 / 39 us at 12288 x 4096,
    // 4096 x 12288, 1024 x 4096) and the dot4 batches cost ~3.5 / 3.2 / 1.1 us per token there, so
    // it takes over from 33 tokens
    if (dtype == 14 && (m >= 33 || long_row)) {
        quantize_tiled();
        launch_mmq_shared_q6k(w, bpr, act, y, m, in_f, out_f, st, stream);
        return true;
    }
    if (dtype == 13 && (m >= 33 || long_row)) {
        quantize_tiled();
        launch_mmq_shared_q5k(w, bpr, act, y, m, in_f, out_f, st, stream);
        return true;
    }
    if (dtype == 10 && in_f % 256 == 0 && (m >= 17 || long_row)) {  // (what the 16-token kernel left)
        quantize_tiled();
        launch_mmq_shared_q2k(w, bpr, act, y, m, in_f, out_f, st, stream);
        return true;
    }
    // TQ1_0 has no 16-token kernel: its dot4 batches cost 2.6 / 2.3 / 1.3 us per token (12288 x 4096, 4096 x 12288,
    // 4096 x 4096), the tiles - whose unpack takes the base-3 digits out - a flat 44 / 106 / 39 us up to 128 tokens
    const size_t tq1_tile_tokens = in_f < 8192 && out_f * in_f >= ((size_t)32 << 20) ? 17 : 33;
    if (dtype == 34 && in_f % 256 == 0 && (m >= tq1_tile_tokens || long_row)) {
        quantize_tiled();
        launch_mmq_shared_tq1_0(w, bpr, act, y, m, in_f, out_f, st, stream);
        return true;
    }
    if ((dtype == 11 || dtype == 35) && in_f % 256 == 0 && (m >= 17 || long_row)) {  // (what the 16-token kernel left)
        quantize_tiled();
        if (dtype == 11) launch_mmq_shared_q3k(w, bpr, act, y, m, in_f, out_f, st, stream);
        else launch_mmq_shared_tq2_0(w, bpr, act, y, m, in_f, out_f, st, stream);
        return true;
    }
    if (dtype == 23 && in_f % 256 == 0 && (m >= 17 || long_row)) {  // (what the 16-token kernel left: 49 / 113 tokens and up)
        quantize_tiled();
        launch_mmq_shared_iq4xs(w, bpr, act, y, m, in_f, out_f, st, stream);
        return true;
    }
    // MXFP4 has no 16-token kernel: its dot4 batches cost 2.1 / 2.2 / 1.3 us per token (12288 x 4096, 4096 x 12288,
    // 4096 x 4096) against the tiles' flat 61 / 149 / 51 us
    const size_t mxfp4_tile_tokens = in_f >= 8192 ? 65 : (out_f * in_f >= ((size_t)32 << 20) ? 33 : 41);
    // NVFP4 likewise: 4.5 / 4.5 / 2.3 us per token against a flat 69 / 165 / 55 us
    const size_t nvfp4_tile_tokens = in_f >= 8192 ? 41 : (out_f * in_f >= ((size_t)32 << 20) ? 9 : 25);
    // (their kernel's flat time up to 128 tokens, ~145 us at 4096 x 12288, meets the dot4 batches'
    // ~2.1 us per token at 64 tokens)
    // (rows that are not whole 256s included: the kernel pads the last step; Q8_0 rows of that kind
    // multiply the per-32 activation like these formats, crates/infr-cpu/src/lib.rs:1037-1042)
    if ((dtype == 2 || dtype == 3 || dtype == 6 || dtype == 7 || dtype == 20 || (dtype == 8 && in_f % 256 != 0) ||
         (dtype == 39 && m >= mxfp4_tile_tokens) ||
         (dtype == 40 && st.a == nullptr && in_f % 64 == 0 && m >= nvfp4_tile_tokens)) &&
        in_f % 32 == 0 && (m >= 65 || long_row || dtype == 39 || dtype == 40)) {
        quantize_32_tiled(false);
        return launch_mmq_shared_nib32(dtype, w, bpr, act, y, m, in_f, out_f, st, stream);
    }
    if (dtype == 42 && in_f % 64 == 0 && (m >= 65 || long_row)) {
        quantize_32_tiled(true);
        return launch_mmq_shared_nib32(dtype, w, bpr, act, y, m, in_f, out_f, st, stream);
    }
    if (dtype == 8 && in_f % 256 == 0 && (m >= 33 || long_row)) {
        quantize_tiled();
        launch_mmq_shared_q8_0(w, bpr, act, y, m, in_f, out_f, st, stream);
        return true;
    }
    quantize_rows(act_is_per32(dtype, in_f));
    if (mmq_skinny16_takes(dtype, m, in_f, out_f)) {
        const size_t wgs = (out_f + 31) / 32;
        return st.a ? launch_mmq_skinny16<true>(dtype, w, bpr, act, y, m, in_f, out_f, wgs, st, nullptr, stream)
                    : launch_mmq_skinny16<false>(dtype, w, bpr, act, y, m, in_f, out_f, wgs, st, nullptr, stream);
    }
    if (dtype != 12 || m == 2) return launch_gemv_batch(dtype, w, bpr, act, y, m, in_f, out_f, st, stream);
    if (m <= 32) {
        // four blocks per round; eight for long rows or when four would leave most SIMDs without a wave
        const size_t wgs = (out_f + 31) / 32 * ((m + 31) / 32);
        if (in_f >= 8192 || (wgs * 4 < 1024 && in_f >= 2048))
            launch_mmq_skinny_q4k<8>(w, bpr, act, y, m, in_f, out_f, st, stream);
        else
            launch_mmq_skinny_q4k<4>(w, bpr, act, y, m, in_f, out_f, st, stream);
        return true;
    }
    launch_mmq_q4k<32>(w, bpr, act, y, m, in_f, out_f, st, stream);
    return true;
}

}  // namespace infr
