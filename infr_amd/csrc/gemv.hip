// Decode GEMV (m == 1) for GGUF block-quantized weights against the int8-quantized activation,
// hand-written for gfx950 wave64. Follows infr-cpu's scalar kernels per block:
//   Q4_K  crates/infr-cpu/src/kernels.rs:151-184     Q6_K  kernels.rs:487-526
//   Q8_0  kernels.rs:1170-1187                       Q2_0  kernels.rs:5641-5668
//
// Common shape. One wavefront owns `rows_per_wave` consecutive weight rows. The K dimension is
// spread over the 64 lanes with a FIXED lane -> K-range mapping, so the int8 activation bytes a lane
// needs are loaded once into registers and reused for every row the wave processes (no LDS).
// Weight bytes stream from HBM exactly once, with 16-byte loads that are contiguous across the
// wave; the next row's loads are issued before the current row is reduced. The kernels are
// HBM-bound: algorithmic traffic is the weight bytes (144 B / 210 B per 256 weights, 34 B per
// 32, 18 B per 64); the activation (K bytes + scales) is re-read per wave from L2.
//
// Integer stages (v_dot4_i32_i8 sums, 6-bit scale products) are exact. The f32 epilogue evaluates
// the CPU expression per block with separate multiplies and adds. For Q4_K and Q6_K the per-block
// terms are then added in ascending block order (16 v_readlane + v_add per 16 blocks), which is
// the CPU's accumulation order, so y matches infr-cpu's scalar kernel bit for bit. For Q8_0 and
// Q2_0 (128 terms per 4096 columns) the lanes' terms are added with a fixed butterfly instead:
// deterministic, but rounded in a different order than the CPU's sequential sum.
#include "device_common.hpp"
#include "kernels.hpp"

namespace infr {

// ───────────────────────────────────── Q4_K ─────────────────────────────────────
// Lane l: block-in-step q = l/4, nibble pair p = l%4. Pair p's 32 bytes hold sub-block 2p in the
// low nibbles and 2p+1 in the high nibbles, so `w & 0x0F0F0F0F` / `(w >> 4) & 0x0F0F0F0F` are
// ready v_dot4 operands against 64 consecutive activation bytes. 16 blocks (4096 weights,
// 2304 B) per wave step.
struct Q4kRow {
    v4i hdr, qa, qb;
};

template <int STEPS>
struct Q4kActs {
    int xa[STEPS][16];
    int bs0[STEPS], bs1[STEPS];
    float dact[STEPS];
};

__device__ __forceinline__ void q4k_load_row(const uint8_t* rowp, int b, int p, bool valid,
                                             Q4kRow& r) {
    if (valid) {
        const uint8_t* blk = rowp + (size_t)b * 144;
        r.hdr = load16(blk);
        r.qa = load16(blk + 16 + p * 32);
        r.qb = load16(blk + 32 + p * 32);
    } else {
        r.hdr = r.qa = r.qb = v4i{0, 0, 0, 0};
    }
}

// Per-block term for one lane quad; sd/sm are the exact per-block integers (all four lanes of
// the quad return the same values).
__device__ __forceinline__ float q4k_block_term(const Q4kRow& r, const int* xa, int bs0, int bs1,
                                                float dact, int p, int& sd, int& sm) {
    const uint32_t m4 = 0x0F0F0F0Fu;
    int ip_e = 0, ip_o = 0;
    const int wq[8] = {r.qa.x, r.qa.y, r.qa.z, r.qa.w, r.qb.x, r.qb.y, r.qb.z, r.qb.w};
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const uint32_t w = (uint32_t)wq[k];
        ip_e = dot4((int)(w & m4), xa[k], ip_e);
        ip_o = dot4((int)((w >> 4) & m4), xa[8 + k], ip_o);
    }
    uint32_t sc8[2], mn8[2];
    k4_all((uint32_t)r.hdr.y, (uint32_t)r.hdr.z, (uint32_t)r.hdr.w, sc8, mn8);
    const uint32_t scw = (p & 2) ? sc8[1] : sc8[0];
    const uint32_t mnw = (p & 2) ? mn8[1] : mn8[0];
    const int sh = (p & 1) * 16;
    const int sc_e = (scw >> sh) & 0xFF, sc_o = (scw >> (sh + 8)) & 0xFF;
    const int m_e = (mnw >> sh) & 0xFF, m_o = (mnw >> (sh + 8)) & 0xFF;
    sd = quad_sum(__mul24(sc_e, ip_e) + __mul24(sc_o, ip_o));
    sm = quad_sum(__mul24(m_e, bs0) + __mul24(m_o, bs1));
    const float d = f16_bits_to_f32((uint32_t)r.hdr.x & 0xFFFFu);
    const float dmin = f16_bits_to_f32((uint32_t)r.hdr.x >> 16);
    // sumf += q8.d[b] * (d * sd as f32 - dmin * sm as f32)
    return dact * (d * (float)sd - dmin * (float)sm);
}

template <int STEPS, bool STAGES>
__global__ __launch_bounds__(256) void gemv_q4k_kernel(
    const uint8_t* __restrict__ w, size_t bpr, const int8_t* __restrict__ qs,
    const float* __restrict__ d8, const int32_t* __restrict__ bsums, float* __restrict__ y, int nb,
    int out_f, int rows_per_wave, int32_t* __restrict__ st_sd, int32_t* __restrict__ st_sm) {
    const int lane = threadIdx.x & 63;
    const int q = lane >> 2, p = lane & 3;
    const int wave = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int row0 = wave * rows_per_wave;
    if (row0 >= out_f) return;
    const int row_end = min(row0 + rows_per_wave, out_f);

    Q4kActs<STEPS> a;
    bool valid[STEPS];
#pragma unroll
    for (int t = 0; t < STEPS; ++t) {
        const int b = t * 16 + q;
        valid[t] = b < nb;
        if (valid[t]) {
            const v4i* xp = reinterpret_cast<const v4i*>(qs + (size_t)b * 256 + p * 64);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const v4i v = xp[k];
                a.xa[t][4 * k + 0] = v.x;
                a.xa[t][4 * k + 1] = v.y;
                a.xa[t][4 * k + 2] = v.z;
                a.xa[t][4 * k + 3] = v.w;
            }
            const v2i bs = *reinterpret_cast<const v2i*>(bsums + (size_t)b * 8 + 2 * p);
            a.bs0[t] = bs.x;
            a.bs1[t] = bs.y;
            a.dact[t] = d8[b];
        } else {
#pragma unroll
            for (int k = 0; k < 16; ++k) a.xa[t][k] = 0;
            a.bs0[t] = a.bs1[t] = 0;
            a.dact[t] = 0.0f;
        }
    }

    Q4kRow cur[STEPS], nxt[STEPS];
    {
        const uint8_t* rowp = w + (size_t)row0 * bpr;
#pragma unroll
        for (int t = 0; t < STEPS; ++t) q4k_load_row(rowp, t * 16 + q, p, valid[t], cur[t]);
    }
    for (int row = row0; row < row_end; ++row) {
        if (row + 1 < row_end) {
            const uint8_t* rowp = w + (size_t)(row + 1) * bpr;
#pragma unroll
            for (int t = 0; t < STEPS; ++t) q4k_load_row(rowp, t * 16 + q, p, valid[t], nxt[t]);
        }
        float s = 0.0f;
#pragma unroll
        for (int t = 0; t < STEPS; ++t) {
            int sd, sm;
            const float term =
                q4k_block_term(cur[t], a.xa[t], a.bs0[t], a.bs1[t], a.dact[t], p, sd, sm);
            if (STAGES && valid[t] && p == 0) {
                st_sd[(size_t)row * nb + t * 16 + q] = sd;
                st_sm[(size_t)row * nb + t * 16 + q] = sm;
            }
            // Ascending block order, one add per block: the CPU's `sumf +=` chain. Lanes past
            // the row's last block hold +0.0, which leaves the sum unchanged.
#pragma unroll
            for (int i = 0; i < 16; ++i) s += readlane_f(term, 4 * i);
        }
        if (lane == 0) y[row] = s;
#pragma unroll
        for (int t = 0; t < STEPS; ++t) cur[t] = nxt[t];
    }
}

// ───────────────────────────────────── Q6_K ─────────────────────────────────────
// Lane l: block-in-step q = l/4, half h = (l%4)/2, c = l%2 selects l in [16c, 16c+16). The lane
// decodes the four 16-element groups {l, l+32, l+64, l+96} of its half: 64 weights, scale indices
// h*8 + c + {0,2,4,6}. Codes stay biased (0..63) and the -32 offset is applied through the
// activation's per-16 sums, exactly the CPU's `sc * (sumi - 32*bsum)`. 16 blocks (3360 B) per
// wave step. Block stride 210 B is 2 mod 4: loads are 2-byte aligned.
struct Q6kRow {
    v4i qla, qlb, qh;
    v2i sc;
    uint32_t d;
};

__device__ __forceinline__ void q6k_load_row(const uint8_t* rowp, int b, int h, int c, bool valid,
                                             Q6kRow& r) {
    if (valid) {
        const uint8_t* blk = rowp + (size_t)b * 210;
        r.qla = load16_a2(blk + h * 64 + c * 16);
        r.qlb = load16_a2(blk + h * 64 + 32 + c * 16);
        r.qh = load16_a2(blk + 128 + h * 32 + c * 16);
        __builtin_memcpy(&r.sc, __builtin_assume_aligned(blk + 192 + h * 8, 2), 8);
        r.d = load_u16(blk + 208);
    } else {
        r.qla = r.qlb = r.qh = v4i{0, 0, 0, 0};
        r.sc = v2i{0, 0};
        r.d = 0;
    }
}

__device__ __forceinline__ float q6k_block_term(const Q6kRow& r, const int* xa, const int* bs16,
                                                float dact, int c, int& isum) {
    const uint32_t m4 = 0x0F0F0F0Fu, m2 = 0x30303030u;
    const int la[4] = {r.qla.x, r.qla.y, r.qla.z, r.qla.w};
    const int lb[4] = {r.qlb.x, r.qlb.y, r.qlb.z, r.qlb.w};
    const int hh[4] = {r.qh.x, r.qh.y, r.qh.z, r.qh.w};
    int sumi[4] = {0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t a = (uint32_t)la[j], b = (uint32_t)lb[j], h = (uint32_t)hh[j];
        sumi[0] = dot4((int)((a & m4) | ((h << 4) & m2)), xa[0 + j], sumi[0]);
        sumi[1] = dot4((int)((b & m4) | ((h << 2) & m2)), xa[4 + j], sumi[1]);
        sumi[2] = dot4((int)(((a >> 4) & m4) | (h & m2)), xa[8 + j], sumi[2]);
        sumi[3] = dot4((int)(((b >> 4) & m4) | ((h >> 2) & m2)), xa[12 + j], sumi[3]);
    }
    // scales[h*8 + c + 2k]: byte (c + 2k) of the 8 bytes loaded at scales + h*8
    const uint32_t lo = (uint32_t)r.sc.x >> (8 * c), hi = (uint32_t)r.sc.y >> (8 * c);
    const int sc0 = (int)(int8_t)(lo & 0xFF), sc1 = (int)(int8_t)((lo >> 16) & 0xFF);
    const int sc2 = (int)(int8_t)(hi & 0xFF), sc3 = (int)(int8_t)((hi >> 16) & 0xFF);
    int part = __mul24(sc0, sumi[0] - 32 * bs16[0]);
    part += __mul24(sc1, sumi[1] - 32 * bs16[1]);
    part += __mul24(sc2, sumi[2] - 32 * bs16[2]);
    part += __mul24(sc3, sumi[3] - 32 * bs16[3]);
    isum = quad_sum(part);
    const float d = f16_bits_to_f32(r.d);
    // sumf += d * q8.d[b] * isum as f32
    return d * dact * (float)isum;
}

template <int STEPS, bool STAGES>
__global__ __launch_bounds__(256) void gemv_q6k_kernel(
    const uint8_t* __restrict__ w, size_t bpr, const int8_t* __restrict__ qs,
    const float* __restrict__ d8, const int32_t* __restrict__ bsums16, float* __restrict__ y,
    int nb, int out_f, int rows_per_wave, int32_t* __restrict__ st_isum) {
    const int lane = threadIdx.x & 63;
    const int q = lane >> 2, h = (lane >> 1) & 1, c = lane & 1;
    const int wave = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int row0 = wave * rows_per_wave;
    if (row0 >= out_f) return;
    const int row_end = min(row0 + rows_per_wave, out_f);

    int xa[STEPS][16], bs16[STEPS][4];
    float dact[STEPS];
    bool valid[STEPS];
#pragma unroll
    for (int t = 0; t < STEPS; ++t) {
        const int b = t * 16 + q;
        valid[t] = b < nb;
        if (valid[t]) {
            const int8_t* xb = qs + (size_t)b * 256 + h * 128 + c * 16;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const v4i v = *reinterpret_cast<const v4i*>(xb + 32 * k);
                xa[t][4 * k + 0] = v.x;
                xa[t][4 * k + 1] = v.y;
                xa[t][4 * k + 2] = v.z;
                xa[t][4 * k + 3] = v.w;
                bs16[t][k] = bsums16[(size_t)b * 16 + h * 8 + c + 2 * k];
            }
            dact[t] = d8[b];
        } else {
#pragma unroll
            for (int k = 0; k < 16; ++k) xa[t][k] = 0;
#pragma unroll
            for (int k = 0; k < 4; ++k) bs16[t][k] = 0;
            dact[t] = 0.0f;
        }
    }

    Q6kRow cur[STEPS], nxt[STEPS];
    {
        const uint8_t* rowp = w + (size_t)row0 * bpr;
#pragma unroll
        for (int t = 0; t < STEPS; ++t) q6k_load_row(rowp, t * 16 + q, h, c, valid[t], cur[t]);
    }
    for (int row = row0; row < row_end; ++row) {
        if (row + 1 < row_end) {
            const uint8_t* rowp = w + (size_t)(row + 1) * bpr;
#pragma unroll
            for (int t = 0; t < STEPS; ++t) q6k_load_row(rowp, t * 16 + q, h, c, valid[t], nxt[t]);
        }
        float s = 0.0f;
#pragma unroll
        for (int t = 0; t < STEPS; ++t) {
            int isum;
            const float term = q6k_block_term(cur[t], xa[t], bs16[t], dact[t], c, isum);
            if (STAGES && valid[t] && (lane & 3) == 0)
                st_isum[(size_t)row * nb + t * 16 + q] = isum;
#pragma unroll
            for (int i = 0; i < 16; ++i) s += readlane_f(term, 4 * i);
        }
        if (lane == 0) y[row] = s;
#pragma unroll
        for (int t = 0; t < STEPS; ++t) cur[t] = nxt[t];
    }
}

// ───────────────────────────────────── Q8_0 ─────────────────────────────────────
// Lane l owns 32-weight block t*64 + l of the row: 34 B = f16 scale + 32 int8, 2-byte aligned.
// 64 blocks (2048 weights, 2176 B) per wave step; the activation scale is per 256 (8 lanes).
struct Q80Row {
    v4i qa, qb;
    uint32_t d;
};

__device__ __forceinline__ void q80_load_row(const uint8_t* rowp, int wb, bool valid, Q80Row& r) {
    if (valid) {
        const uint8_t* blk = rowp + (size_t)wb * 34;
        r.d = load_u16(blk);
        r.qa = load16_a2(blk + 2);
        r.qb = load16_a2(blk + 18);
    } else {
        r.qa = r.qb = v4i{0, 0, 0, 0};
        r.d = 0;
    }
}

template <int STEPS, bool STAGES>
__global__ __launch_bounds__(256) void gemv_q8_0_kernel(
    const uint8_t* __restrict__ w, size_t bpr, const int8_t* __restrict__ qs,
    const float* __restrict__ d8, float* __restrict__ y, int nblk32, int out_f, int rows_per_wave,
    int32_t* __restrict__ st_iprod) {
    const int lane = threadIdx.x & 63;
    const int wave = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int row0 = wave * rows_per_wave;
    if (row0 >= out_f) return;
    const int row_end = min(row0 + rows_per_wave, out_f);

    int xa[STEPS][8];
    float dact[STEPS];
    bool valid[STEPS];
#pragma unroll
    for (int t = 0; t < STEPS; ++t) {
        const int wb = t * 64 + lane;
        valid[t] = wb < nblk32;
        if (valid[t]) {
            const v4i v0 = *reinterpret_cast<const v4i*>(qs + (size_t)wb * 32);
            const v4i v1 = *reinterpret_cast<const v4i*>(qs + (size_t)wb * 32 + 16);
            xa[t][0] = v0.x; xa[t][1] = v0.y; xa[t][2] = v0.z; xa[t][3] = v0.w;
            xa[t][4] = v1.x; xa[t][5] = v1.y; xa[t][6] = v1.z; xa[t][7] = v1.w;
            dact[t] = d8[wb >> 3];
        } else {
#pragma unroll
            for (int k = 0; k < 8; ++k) xa[t][k] = 0;
            dact[t] = 0.0f;
        }
    }

    Q80Row cur[STEPS], nxt[STEPS];
    {
        const uint8_t* rowp = w + (size_t)row0 * bpr;
#pragma unroll
        for (int t = 0; t < STEPS; ++t) q80_load_row(rowp, t * 64 + lane, valid[t], cur[t]);
    }
    for (int row = row0; row < row_end; ++row) {
        if (row + 1 < row_end) {
            const uint8_t* rowp = w + (size_t)(row + 1) * bpr;
#pragma unroll
            for (int t = 0; t < STEPS; ++t) q80_load_row(rowp, t * 64 + lane, valid[t], nxt[t]);
        }
        float s = 0.0f;
#pragma unroll
        for (int t = 0; t < STEPS; ++t) {
            const Q80Row& r = cur[t];
            int ip = 0;
            ip = dot4(r.qa.x, xa[t][0], ip);
            ip = dot4(r.qa.y, xa[t][1], ip);
            ip = dot4(r.qa.z, xa[t][2], ip);
            ip = dot4(r.qa.w, xa[t][3], ip);
            ip = dot4(r.qb.x, xa[t][4], ip);
            ip = dot4(r.qb.y, xa[t][5], ip);
            ip = dot4(r.qb.z, xa[t][6], ip);
            ip = dot4(r.qb.w, xa[t][7], ip);
            if (STAGES && valid[t]) st_iprod[(size_t)row * nblk32 + t * 64 + lane] = ip;
            // sumf += d8 * d_w * iprod as f32
            s += dact[t] * f16_bits_to_f32(r.d) * (float)ip;
        }
        s = wave_sum_f(s);
        if (lane == 0) y[row] = s;
#pragma unroll
        for (int t = 0; t < STEPS; ++t) cur[t] = nxt[t];
    }
}

// ───────────────────────────────────── Q2_0 ─────────────────────────────────────
// Lane l owns 64-weight block t*64 + l: 18 B = f16 scale + 16 bytes of 2-bit codes, 2-byte
// aligned. `(w >> 2s) & 0x03030303` pulls the codes of elements {4i+s} of a 16-element group into
// the four bytes of a word; the activation bytes are transposed once per wave (v_perm_b32) into
// that order, so each extracted word is a ready v_dot4 operand. 64 blocks (4096 weights,
// 1152 B) per wave step. Codes stay 0..3; the -1 offset is applied as `iprod - bsum` like the CPU.
struct Q20Row {
    v4i codes;
    uint32_t d;
};

__device__ __forceinline__ void q20_load_row(const uint8_t* rowp, int b, bool valid, Q20Row& r) {
    if (valid) {
        const uint8_t* blk = rowp + (size_t)b * 18;
        r.d = load_u16(blk);
        r.codes = load16_a2(blk + 2);
    } else {
        r.codes = v4i{0, 0, 0, 0};
        r.d = 0;
    }
}

// 4x4 byte transpose: out[s] byte i = in[i] byte s.
__device__ __forceinline__ void transpose4x4(const int in[4], int out[4]) {
    // v_perm_b32(hi, lo, sel): result byte k = byte sel[k] of the 8-byte value {hi:lo} (lo = 0..3).
    const uint32_t a = (uint32_t)in[0], b = (uint32_t)in[1], c = (uint32_t)in[2], d = (uint32_t)in[3];
    const uint32_t ab_lo = __builtin_amdgcn_perm(b, a, 0x05010400u);  // a0 b0 a1 b1
    const uint32_t ab_hi = __builtin_amdgcn_perm(b, a, 0x07030602u);  // a2 b2 a3 b3
    const uint32_t cd_lo = __builtin_amdgcn_perm(d, c, 0x05010400u);  // c0 d0 c1 d1
    const uint32_t cd_hi = __builtin_amdgcn_perm(d, c, 0x07030602u);  // c2 d2 c3 d3
    out[0] = (int)__builtin_amdgcn_perm(cd_lo, ab_lo, 0x05040100u);   // a0 b0 c0 d0
    out[1] = (int)__builtin_amdgcn_perm(cd_lo, ab_lo, 0x07060302u);   // a1 b1 c1 d1
    out[2] = (int)__builtin_amdgcn_perm(cd_hi, ab_hi, 0x05040100u);   // a2 b2 c2 d2
    out[3] = (int)__builtin_amdgcn_perm(cd_hi, ab_hi, 0x07060302u);   // a3 b3 c3 d3
}

template <int STEPS, bool STAGES>
__global__ __launch_bounds__(256) void gemv_q2_0_kernel(
    const uint8_t* __restrict__ w, size_t bpr, const int8_t* __restrict__ qs,
    const float* __restrict__ d32, const int32_t* __restrict__ bsum, float* __restrict__ y, int nb64,
    int out_f, int rows_per_wave, int32_t* __restrict__ st_iprod) {
    const int lane = threadIdx.x & 63;
    const int wave = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int row0 = wave * rows_per_wave;
    if (row0 >= out_f) return;
    const int row_end = min(row0 + rows_per_wave, out_f);

    int xt[STEPS][16];  // xt[4j + s] = bytes {x[16j + 4i + s]}, i = 0..3
    float da0[STEPS], da1[STEPS], fb0[STEPS], fb1[STEPS];
    bool valid[STEPS];
#pragma unroll
    for (int t = 0; t < STEPS; ++t) {
        const int b = t * 64 + lane;
        valid[t] = b < nb64;
        if (valid[t]) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const v4i v = *reinterpret_cast<const v4i*>(qs + (size_t)b * 64 + 16 * j);
                const int in[4] = {v.x, v.y, v.z, v.w};
                transpose4x4(in, &xt[t][4 * j]);
            }
            da0[t] = d32[2 * b];
            da1[t] = d32[2 * b + 1];
            fb0[t] = (float)bsum[2 * b];
            fb1[t] = (float)bsum[2 * b + 1];
        } else {
#pragma unroll
            for (int k = 0; k < 16; ++k) xt[t][k] = 0;
            da0[t] = da1[t] = fb0[t] = fb1[t] = 0.0f;
        }
    }

    Q20Row cur[STEPS], nxt[STEPS];
    {
        const uint8_t* rowp = w + (size_t)row0 * bpr;
#pragma unroll
        for (int t = 0; t < STEPS; ++t) q20_load_row(rowp, t * 64 + lane, valid[t], cur[t]);
    }
    for (int row = row0; row < row_end; ++row) {
        if (row + 1 < row_end) {
            const uint8_t* rowp = w + (size_t)(row + 1) * bpr;
#pragma unroll
            for (int t = 0; t < STEPS; ++t) q20_load_row(rowp, t * 64 + lane, valid[t], nxt[t]);
        }
        float s = 0.0f;
#pragma unroll
        for (int t = 0; t < STEPS; ++t) {
            const Q20Row& r = cur[t];
            const uint32_t cw[4] = {(uint32_t)r.codes.x, (uint32_t)r.codes.y, (uint32_t)r.codes.z,
                                    (uint32_t)r.codes.w};
            int ip0 = 0, ip1 = 0;
#pragma unroll
            for (int sft = 0; sft < 4; ++sft) {
                ip0 = dot4((int)((cw[0] >> (2 * sft)) & 0x03030303u), xt[t][0 + sft], ip0);
                ip0 = dot4((int)((cw[1] >> (2 * sft)) & 0x03030303u), xt[t][4 + sft], ip0);
                ip1 = dot4((int)((cw[2] >> (2 * sft)) & 0x03030303u), xt[t][8 + sft], ip1);
                ip1 = dot4((int)((cw[3] >> (2 * sft)) & 0x03030303u), xt[t][12 + sft], ip1);
            }
            if (STAGES && valid[t]) {
                st_iprod[(size_t)row * nb64 * 2 + 2 * (t * 64 + lane)] = ip0;
                st_iprod[(size_t)row * nb64 * 2 + 2 * (t * 64 + lane) + 1] = ip1;
            }
            const float d = f16_bits_to_f32(r.d);
            // sumf += d * q8.d[s] * (iprod as f32 - bsum[s] as f32), sub-block 2b then 2b+1
            s += d * da0[t] * ((float)ip0 - fb0[t]);
            s += d * da1[t] * ((float)ip1 - fb1[t]);
        }
        s = wave_sum_f(s);
        if (lane == 0) y[row] = s;
#pragma unroll
        for (int t = 0; t < STEPS; ++t) cur[t] = nxt[t];
    }
}

// ───────────────────────────────────── launch ─────────────────────────────────────

// Rows per wavefront: enough waves to cover the machine several times over (256 CUs x 4 SIMDs),
// few enough that the per-wave activation load is amortised.
static int pick_rows_per_wave(size_t out_f) {
    const size_t target_waves = 256 * 4 * 4;
    size_t r = (out_f + target_waves - 1) / target_waves;
    if (r < 2) r = 2;
    if (r > 16) r = 16;
    return (int)r;
}

int g_gemv_rows_per_wave_override = 0;  // tuning hook (0 = automatic)

// Instantiates KERNEL<STEPS, STAGES> for 1..8 wave steps per row; more steps than that (in_f
// beyond 32768 for Q4_K/Q6_K/Q2_0, 16384 for Q8_0) has no kernel and is reported as unsupported.
#define INFR_CASE(KERNEL, N, ST, ...) \
    case N: hipLaunchKernelGGL((KERNEL<N, ST>), grid, block, 0, stream, __VA_ARGS__); break;
#define INFR_LAUNCH_STEPS(KERNEL, ST, STEPS_EXPR, ...)  \
    do {                                                \
        switch (STEPS_EXPR) {                           \
            INFR_CASE(KERNEL, 1, ST, __VA_ARGS__)       \
            INFR_CASE(KERNEL, 2, ST, __VA_ARGS__)       \
            INFR_CASE(KERNEL, 3, ST, __VA_ARGS__)       \
            INFR_CASE(KERNEL, 4, ST, __VA_ARGS__)       \
            INFR_CASE(KERNEL, 5, ST, __VA_ARGS__)       \
            INFR_CASE(KERNEL, 6, ST, __VA_ARGS__)       \
            INFR_CASE(KERNEL, 7, ST, __VA_ARGS__)       \
            INFR_CASE(KERNEL, 8, ST, __VA_ARGS__)       \
        default: return false;                          \
        }                                               \
    } while (0)

bool launch_gemv(int dtype, const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t in_f,
                 size_t out_f, const IntStages& st, hipStream_t stream) {
    if (out_f == 0) return true;
    const int rpw = g_gemv_rows_per_wave_override > 0 ? g_gemv_rows_per_wave_override
                                                      : pick_rows_per_wave(out_f);
    const size_t waves = (out_f + rpw - 1) / rpw;
    const dim3 grid((unsigned)((waves + 3) / 4)), block(256);
    const int n_out = (int)out_f;
    int32_t* const no_st = nullptr;
    switch (dtype) {
    case 12: {  // Q4_K
        const int nb = (int)(in_f / 256);
        const int steps = (nb + 15) / 16;
        if (st.a)
            INFR_LAUNCH_STEPS(gemv_q4k_kernel, true, steps, w, bpr, act.qs, act.d, act.bsums, y, nb,
                              n_out, rpw, st.a, st.b);
        else
            INFR_LAUNCH_STEPS(gemv_q4k_kernel, false, steps, w, bpr, act.qs, act.d, act.bsums, y,
                              nb, n_out, rpw, no_st, no_st);
        return true;
    }
    case 14: {  // Q6_K
        const int nb = (int)(in_f / 256);
        const int steps = (nb + 15) / 16;
        if (st.a)
            INFR_LAUNCH_STEPS(gemv_q6k_kernel, true, steps, w, bpr, act.qs, act.d, act.bsums16, y,
                              nb, n_out, rpw, st.a);
        else
            INFR_LAUNCH_STEPS(gemv_q6k_kernel, false, steps, w, bpr, act.qs, act.d, act.bsums16, y,
                              nb, n_out, rpw, no_st);
        return true;
    }
    case 8: {  // Q8_0
        const int nblk = (int)(in_f / 32);
        const int steps = (nblk + 63) / 64;
        if (st.a)
            INFR_LAUNCH_STEPS(gemv_q8_0_kernel, true, steps, w, bpr, act.qs, act.d, y, nblk, n_out,
                              rpw, st.a);
        else
            INFR_LAUNCH_STEPS(gemv_q8_0_kernel, false, steps, w, bpr, act.qs, act.d, y, nblk, n_out,
                              rpw, no_st);
        return true;
    }
    case 42: {  // Q2_0
        const int nb64 = (int)(in_f / 64);
        const int steps = (nb64 + 63) / 64;
        if (st.a)
            INFR_LAUNCH_STEPS(gemv_q2_0_kernel, true, steps, w, bpr, act.qs, act.d, act.bsums, y,
                              nb64, n_out, rpw, st.a);
        else
            INFR_LAUNCH_STEPS(gemv_q2_0_kernel, false, steps, w, bpr, act.qs, act.d, act.bsums, y,
                              nb64, n_out, rpw, no_st);
        return true;
    }
    default:
        return false;
    }
}

}  // namespace infr
