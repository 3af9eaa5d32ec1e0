// Routed-expert prefill GEMM (Op::MoeFfn with pairs bucketed by expert) for Q5_K, Q6_K and Q8_0 banks
// on the int8 matrix cores; Q4_K banks run the tiled kernel of mmq.hip through the same tile map.
//
// Tiles of up to 32 pairs of one expert (mmq_tiles.hpp). A workgroup covers the tile's pairs x 128 rows
// of the expert; every wave unpacks its own 32 rows - lane (row, h) the 16-element halves 16h..16h+15
// of all eight 32-element sub-blocks of a 256-element step - into B operands held in registers, and
// the activation tile (row-major per-256 quantized rows, gathered through `perm`) sits in
// double-buffered LDS. One policy per format supplies the bytes to load, the operands and what a
// step adds to the 16 accumulators; integers, f32 expressions and block order are those of the
// formats' dense prefill kernels (mmq_q5k.hip, mmq_q6k.hip) and, for Q8_0, of the scalar CPU kernel, so every
// pair equals the per-pair GEMV bit for bit.
#include "device_common.hpp"
#include "kernels.hpp"
#include "mmq_tiles.hpp"

namespace infr {

typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kGatherBM = 32;

// What a policy's step() sees of the tile: this lane's activation row as MFMA A operand (token
// `col`, K half `h`), the tile's per-token scales, its split per-32 sums, and 16 zero bytes.
struct GatherCtx {
    const uint8_t* arow;   // + sb * 32: 16 activation bytes of sub-block sb
    const float* dtile;    // + 8 * j: scales of tokens 8j + 4h .. + 3 (the lane's accumulators 4j .. 4j+3)
    const uint8_t* bsrow;  // 8 f16: bsum & 63 (h = 0 lanes) / the rest (h = 1 lanes) of token `col`
    const uint8_t* zero;
    int h;
};

// Q6_K (210-byte block; kernels.rs:487-526): a group of 16 is multiplied alone - the activations of
// the sub-block's other half are read from the zero bytes - and scaled into isum by its int8 scale.
struct GatherQ6K {
    static constexpr int kStepBytes = 210;
    struct Raw {
        v4i ql[4], qh[2], sc;  // ql[2 * half + (qd & 1)], qh[half]: this lane's 16 bytes of each
        uint32_t d;
    };
    __device__ static void load(Raw& r, const uint8_t* blk, int h) {  // 2-byte aligned
#pragma unroll
        for (int k = 0; k < 4; ++k) r.ql[k] = load16_a2(blk + 32 * k + 16 * h);
        r.qh[0] = load16_a2(blk + 128 + 16 * h);
        r.qh[1] = load16_a2(blk + 160 + 16 * h);
        r.sc = load16_a2(blk + 192);
        r.d = load_u16(blk + 208);
    }
    __device__ static void step(const Raw& cur, const GatherCtx& c, float (&acc)[16]) {
        const int scw[4] = {cur.sc.x, cur.sc.y, cur.sc.z, cur.sc.w};
        const float d = f16_bits_to_f32(cur.d);
        const v16i zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        v16i isum;
#pragma unroll
        for (int i = 0; i < 16; ++i) isum[i] = 0;
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) {
            const int half = sb >> 2, qd = sb & 3;
            v4i bf;  // q - 32 as int8: (q + 0x60) ^ 0x80 per byte
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t nib = ((uint32_t)cur.ql[2 * half + (qd & 1)][k] >> (4 * (qd >> 1))) & 0x0F0F0F0Fu;
                const uint32_t hb = ((uint32_t)cur.qh[half][k] >> (2 * qd)) & 0x03030303u;
                bf[k] = (int)((((hb << 4) | nib) + 0x60606060u) ^ 0x80808080u);
            }
            const v4i a0 = *reinterpret_cast<const v4i*>(c.h == 0 ? c.arow + sb * 32 : c.zero);
            const v4i a1 = *reinterpret_cast<const v4i*>(c.h == 1 ? c.arow + sb * 32 : c.zero);
            const v16i r0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, bf, zi, 0, 0, 0);
            const v16i r1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, bf, zi, 0, 0, 0);
            const int g0 = 2 * sb, g1 = 2 * sb + 1;
            const int sc0 = __builtin_amdgcn_sbfe(scw[g0 >> 2], 8 * (g0 & 3), 8);
            const int sc1 = __builtin_amdgcn_sbfe(scw[g1 >> 2], 8 * (g1 & 3), 8);
#pragma unroll
            for (int i = 0; i < 16; ++i) isum[i] += __mul24(r0[i], sc0) + __mul24(r1[i], sc1);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const v4f dq = *reinterpret_cast<const v4f*>(c.dtile + 8 * j);
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[4 * j + i] += (d * dq[i]) * (float)isum[4 * j + i];
        }
    }
};

// Q5_K (176-byte block): one MFMA per 32-element sub-block, scaled into sd by its 6-bit scale; sm is
// the f16 MFMA of the mins against the split per-32 sums; q8.d[b] * (d * sd - dmin * sm).
struct GatherQ5K {
    static constexpr int kStepBytes = 176;
    struct Raw {
        v4i hdr, qh, ql[4];
    };
    __device__ static void load(Raw& r, const uint8_t* blk, int h) {  // 16-byte aligned
        r.hdr = load16(blk);
        r.qh = load16(blk + 16 + 16 * h);
#pragma unroll
        for (int p = 0; p < 4; ++p) r.ql[p] = load16(blk + 48 + 32 * p + 16 * h);
    }
    __device__ static void step(const Raw& cur, const GatherCtx& c, float (&acc)[16]) {
        uint32_t sc8[2], mn8[2];
        k4_all((uint32_t)cur.hdr.y, (uint32_t)cur.hdr.z, (uint32_t)cur.hdr.w, sc8, mn8);
        const float d = f16_bits_to_f32((uint32_t)cur.hdr.x & 0xFFFFu);
        const float dmin = f16_bits_to_f32((uint32_t)cur.hdr.x >> 16);
        const v16i zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        const v16f zf = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        int sd[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) sd[i] = 0;
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) {
            const int p = sb >> 1, e = sb & 1;  // low / high nibbles of pair p, bit sb of qh
            v4i bf;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t nib = ((uint32_t)cur.ql[p][k] >> (4 * e)) & 0x0F0F0F0Fu;
                const uint32_t hb = ((uint32_t)cur.qh[k] >> sb) & 0x01010101u;
                bf[k] = (int)((hb << 4) | nib);
            }
            const v4i a = *reinterpret_cast<const v4i*>(c.arow + sb * 32);
            const v16i r = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, bf, zi, 0, 0, 0);
            const int sc = (int)((sc8[sb >> 2] >> (8 * (sb & 3))) & 0xFFu);
#pragma unroll
            for (int i = 0; i < 16; ++i) sd[i] += __mul24(r[i], sc);
        }
        v8h bm;
#pragma unroll
        for (int s = 0; s < 8; ++s) bm[s] = (_Float16)(int)((mn8[s >> 2] >> (8 * (s & 3))) & 0xFFu);
        const v8h abs_ = *reinterpret_cast<const v8h*>(c.bsrow);
        const v16f smf = __builtin_amdgcn_mfma_f32_32x32x16_f16(abs_, bm, zf, 0, 0, 0);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const v4f dq = *reinterpret_cast<const v4f*>(c.dtile + 8 * j);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int r = 4 * j + i;
                acc[r] += dq[i] * (d * (float)sd[r] - dmin * smf[r]);
            }
        }
    }
};

// Q8_0 (eight 34-byte blocks per step): the stored codes are the operand; every 32-block adds
// (d8 * d_w) * (f32)iprod to the output, blocks ascending and without FMA - the scalar CPU kernel's
// `sumf += d8 * d_w * iprod as f32` (kernels.rs:1170-1187) - so a pair's gate / up outputs, and with
// them the int8 codes of its gated activation, equal the CPU's bit for bit.
struct GatherQ8_0 {
    static constexpr int kStepBytes = 8 * 34;
    struct Raw {
        v4i q[8];
        uint32_t d[8];
    };
    __device__ static void load(Raw& r, const uint8_t* blk, int h) {  // 2-byte aligned
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) {
            r.q[sb] = load16_a2(blk + sb * 34 + 2 + 16 * h);
            r.d[sb] = load_u16(blk + sb * 34);
        }
    }
    __device__ static void step(const Raw& cur, const GatherCtx& c, float (&acc)[16]) {
        const v16i zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        float dq[16];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const v4f q = *reinterpret_cast<const v4f*>(c.dtile + 8 * j);
            dq[4 * j + 0] = q.x; dq[4 * j + 1] = q.y; dq[4 * j + 2] = q.z; dq[4 * j + 3] = q.w;
        }
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) {
            const v4i a = *reinterpret_cast<const v4i*>(c.arow + sb * 32);
            const v16i r = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, cur.q[sb], zi, 0, 0, 0);
            const float dw = f16_bits_to_f32(cur.d[sb]);
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[i] += (dq[i] * dw) * (float)r[i];
        }
    }
};

template <typename P>
__global__ __launch_bounds__(256) void mmq_gathered_kernel(const uint8_t* __restrict__ w, size_t bpr,
                                                           const int8_t* __restrict__ qs,
                                                           const float* __restrict__ d8,
                                                           const int32_t* __restrict__ bsums,
                                                           float* __restrict__ y, GatheredTiles tiles, int out_f,
                                                           int nb) {
    constexpr int BM = kGatherBM;
    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * MmqLds<BM>::bytes];
    __shared__ __attribute__((aligned(16))) int zero16[4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, h = lane >> 5;
    const int tile_y = blockIdx.y;
    size_t w_off = 0;
    if (!tiles.select(tile_y, w_off)) return;  // uniform over the workgroup, before any barrier
    const int n_slots = tiles.count(tile_y, BM);
    const int wrow = blockIdx.x * 128 + wave * 32 + col;
    const bool row_ok = wrow < out_f;
    const uint8_t* wrowp = w + w_off + (size_t)(row_ok ? wrow : 0) * bpr;
    if (tid < 4) zero16[tid] = 0;

    float acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;

    ActStage<BM> stage;
    stage.resolve(tid, [&](int t) { return tiles.act_row(tile_y, BM, t); });
    stage.fetch(qs, d8, bsums, nb, 0, tid);
    typename P::Raw raw;
    P::load(raw, wrowp, h);
    stage.store(lds, tid);
    __syncthreads();

    for (int b = 0; b < nb; ++b) {
        const uint8_t* tile = lds + (b & 1) * MmqLds<BM>::bytes;
        const typename P::Raw cur = raw;
        if (b + 1 < nb) {
            stage.fetch(qs, d8, bsums, nb, b + 1, tid);
            P::load(raw, wrowp + (size_t)(b + 1) * P::kStepBytes, h);
        }
        const GatherCtx ctx{tile + MmqLds<BM>::qs_off + col * kActRowBytes + h * 16,
                            reinterpret_cast<const float*>(tile + MmqLds<BM>::d_off) + 4 * h,
                            tile + MmqLds<BM>::bs_off + col * 32 + h * 16,
                            reinterpret_cast<const uint8_t*>(zero16), h};
        P::step(cur, ctx, acc);
        if (b + 1 < nb) stage.store(lds + ((b + 1) & 1) * MmqLds<BM>::bytes, tid);
        __syncthreads();
    }

    if (!row_ok) return;
    // accumulator r of this lane is slot 8*(r/4) + 4*h + r%4 of the tile
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int slot = 8 * (r >> 2) + 4 * h + (r & 3);
        if (slot < n_slots) y[(size_t)tiles.out_row(tile_y, BM, slot) * out_f + wrow] = acc[r];
    }
}

bool launch_mmq_gathered(int dtype, const uint8_t* bank, size_t expert_stride, size_t bpr, const ActQ8& act,
                         int act_div, const MoeTileTable& t, float* y, size_t in_f, size_t out_f,
                         hipStream_t stream) {
    const dim3 grid((unsigned)((out_f + 127) / 128), (unsigned)t.max_tiles), block(256);
    const GatheredTiles g{t.n_tiles, t.expert, t.slot0, t.count, t.perm, expert_stride, act_div};
    const int nb = (int)(in_f / 256);
#define INFR_GATHER(P)                                                                                          \
    hipLaunchKernelGGL((mmq_gathered_kernel<P>), grid, block, 0, stream, bank, bpr, act.qs, act.d, act.bsums, y, g, \
                       (int)out_f, nb)
    switch (dtype) {
    case 12: launch_mmq_q4k_gathered(bank, expert_stride, bpr, act, act_div, t, y, in_f, out_f, stream); return true;
    case 13: INFR_GATHER(GatherQ5K); return true;
    case 14: INFR_GATHER(GatherQ6K); return true;
    case 8: INFR_GATHER(GatherQ8_0); return true;
    default: return false;
    }
#undef INFR_GATHER
}

}  // namespace infr
