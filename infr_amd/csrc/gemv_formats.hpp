// Per-format lane mappings of the decode GEMV: what a lane loads of a weight row, which
// activation bytes it keeps in registers, and the per-block integer stage + f32 term.
// Each format follows infr-cpu's scalar kernel for one block:
//   Q4_K  crates/infr-cpu/src/kernels.rs:151-184     Q6_K  kernels.rs:487-526
//   Q8_0  kernels.rs:1170-1187                       Q2_0  kernels.rs:5641-5668
//   Q5_K  kernels.rs:1286-1327                      Q2_K  kernels.rs:315-361    Q3_K  :764-852
//   Q4_0  kernels.rs:5496-5520   Q4_1  :5793-5822    Q5_0  :5350-5377   Q5_1  :5948-5980
//   IQ4_NL  kernels.rs:6128-6152
//
// Interface of a format policy F (all members static, `t` = wave step, `lane` = 0..63):
//   kElemsPerStep         K elements one wave step covers
//   kPer32                activation quantizer: per-32 (true) or per-256 (false)
//   kOrdered              per-block terms are added in ascending block order (bit-exact with the
//                         CPU's `sumf +=` chain) instead of a butterfly
//   kWide16Steps          up to this many wave steps per row the fused kernel fits 16 waves per
//                         workgroup (128 VGPRs per lane) without spilling; beyond it, 8 waves
//   kRowAhead             rows of several wave steps request step t of the next row before step t
//                         of this one is computed (a whole row in flight) instead of one step ahead
//   kClampedLoads         has load_row_clamped: for a row known to be readable, lanes without
//                         work read block 0 instead of being masked off
//   kLaneSums             butterfly formats: the lanes' row sums of eight rows are parked in LDS and
//                         reduced together instead of one whole-wave reduction per row (Q4_0
//                         +14 % at 4096 x 4096, IQ4_NL +6 % at 4096 x 12288, Q8_0 +1-2 %; Q2_0
//                         measured 12-17 % slower that way and keeps the per-row reduction)
//   units(in_f)           number of lane work units in a row (blocks for Q4_K/Q6_K ...)
//   Row / Acts            registers for one step of a weight row / of the activation
//   valid(t, lane, n)     does this lane have work in step t
//   load_row, load_acts   fill them (acts from any address space: global or LDS pointers)
//   term(...)             exact integer stage + f32 term of the lane's unit; writes stage outputs
//   term_shared(...)      optional: the same when one weight row meets several activation rows
#pragma once

#include "device_common.hpp"

namespace infr {

// Pointers to a quantized activation row (global memory or LDS).
struct ActPtrs {
    const int8_t* qs;
    const float* d;
    const int32_t* bsums;    // per 32
    const int32_t* bsums16;  // per 16 (per-256 quantizer only)
};

struct StagePtrs {
    int32_t* a;
    int32_t* b;
};

// ───────────────────────────────────── Q4_K ─────────────────────────────────────
// Lane l: block-in-step q = l/4, nibble pair p = l%4. Pair p's 32 bytes hold sub-block 2p in the
// low nibbles and 2p+1 in the high nibbles, so `w & 0x0F0F0F0F` / `(w >> 4) & 0x0F0F0F0F` are
// ready v_dot4 operands against 64 consecutive activation bytes. 16 blocks (4096 weights,
// 2304 B) per wave step; the quad's partial integers are combined with two DPP adds.
struct FmtQ4K {
    static constexpr int kElemsPerStep = 4096;
    static constexpr bool kPer32 = false;
    static constexpr bool kOrdered = true;
    static constexpr int kBlockBytes = 144, kBlockElems = 256;
    static constexpr int kWide16Steps = 3;
    static constexpr bool kClampedLoads = false;
    static constexpr bool kLaneSums = true;
    static constexpr bool kRowAhead = false;
    struct Row {
        v4i hdr, qa, qb;
    };
    struct Acts {
        int xa[16];
        int bs0, bs1;
        float dact;
    };
    __device__ static int units(int in_f) { return in_f / 256; }
    __device__ static bool valid(int t, int lane, int n) { return t * 16 + (lane >> 2) < n; }
    __device__ static void load_row(Row& r, const uint8_t* rowp, int t, int lane, bool ok) {
        if (ok) {
            const uint8_t* blk = rowp + (size_t)(t * 16 + (lane >> 2)) * 144;
            const int p = lane & 3;
            r.hdr = load16(blk);
            r.qa = load16(blk + 16 + p * 32);
            r.qb = load16(blk + 32 + p * 32);
        } else {
            r.hdr = r.qa = r.qb = v4i{0, 0, 0, 0};
        }
    }
    // The same pieces out of a wave's LDS ring of the weight bytes: `pos` is the ring position of the
    // step's first byte (below `ring_bytes`). Blocks are whole 16-byte pieces at 16-byte boundaries
    // and the ring is a whole number of pieces, so no piece straddles the wrap.
    static constexpr uint32_t kStepBytes = 16 * 144;
    static constexpr int kRingMaxSteps = 3, kRingLongInstr = 4;
    __device__ static void load_row_ring(Row& r, const uint8_t* ring, uint32_t pos, uint32_t ring_bytes, int lane, bool ok) {
        const int p = lane & 3;
        uint32_t o0 = pos + (uint32_t)(lane >> 2) * 144;
        uint32_t o1 = o0 + 16 + p * 32, o2 = o0 + 32 + p * 32;
        o0 = o0 >= ring_bytes ? o0 - ring_bytes : o0;
        o1 = o1 >= ring_bytes ? o1 - ring_bytes : o1;
        o2 = o2 >= ring_bytes ? o2 - ring_bytes : o2;
        const v4i hdr = *reinterpret_cast<const v4i*>(ring + o0);
        const v4i qa = *reinterpret_cast<const v4i*>(ring + o1);
        const v4i qb = *reinterpret_cast<const v4i*>(ring + o2);
        // a lane without a block: d = dmin = 0 makes its term +0.0 whatever the other bytes are
        r.hdr = hdr;
        r.hdr.x = ok ? hdr.x : 0;
        r.qa = qa;
        r.qb = qb;
    }
    __device__ static void load_acts(Acts& a, const ActPtrs& s, int t, int lane, bool ok) {
        if (ok) {
            const int b = t * 16 + (lane >> 2), p = lane & 3;
            const v4i* xp = reinterpret_cast<const v4i*>(s.qs + (size_t)b * 256 + p * 64);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const v4i v = xp[k];
                a.xa[4 * k + 0] = v.x;
                a.xa[4 * k + 1] = v.y;
                a.xa[4 * k + 2] = v.z;
                a.xa[4 * k + 3] = v.w;
            }
            const v2i bs = *reinterpret_cast<const v2i*>(s.bsums + (size_t)b * 8 + 2 * p);
            a.bs0 = bs.x;
            a.bs1 = bs.y;
            a.dact = s.d[b];
        } else {
#pragma unroll
            for (int k = 0; k < 16; ++k) a.xa[k] = 0;
            a.bs0 = a.bs1 = 0;
            a.dact = 0.0f;
        }
    }
    // sd/sm are exact per-block integers, identical in the four lanes of a quad.
    template <bool STAGES>
    __device__ static float term(const Row& r, const Acts& a, int t, int lane, bool ok,
                                 const StagePtrs& st, size_t row_units) {
        const int p = lane & 3;
        const uint32_t m4 = 0x0F0F0F0Fu;
        int ip_e = 0, ip_o = 0;
        const int wq[8] = {r.qa.x, r.qa.y, r.qa.z, r.qa.w, r.qb.x, r.qb.y, r.qb.z, r.qb.w};
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const uint32_t w = (uint32_t)wq[k];
            ip_e = dot4((int)(w & m4), a.xa[k], ip_e);
            ip_o = dot4((int)((w >> 4) & m4), a.xa[8 + k], ip_o);
        }
        uint32_t sc8[2], mn8[2];
        k4_all((uint32_t)r.hdr.y, (uint32_t)r.hdr.z, (uint32_t)r.hdr.w, sc8, mn8);
        const uint32_t scw = (p & 2) ? sc8[1] : sc8[0];
        const uint32_t mnw = (p & 2) ? mn8[1] : mn8[0];
        const int sh = (p & 1) * 16;
        const int sc_e = (scw >> sh) & 0xFF, sc_o = (scw >> (sh + 8)) & 0xFF;
        const int m_e = (mnw >> sh) & 0xFF, m_o = (mnw >> (sh + 8)) & 0xFF;
        const int sd = quad_sum(__mul24(sc_e, ip_e) + __mul24(sc_o, ip_o));
        const int sm = quad_sum(__mul24(m_e, a.bs0) + __mul24(m_o, a.bs1));
        if (STAGES && ok && p == 0) {
            st.a[row_units + t * 16 + (lane >> 2)] = sd;
            st.b[row_units + t * 16 + (lane >> 2)] = sm;
        }
        const float d = f16_bits_to_f32((uint32_t)r.hdr.x & 0xFFFFu);
        const float dmin = f16_bits_to_f32((uint32_t)r.hdr.x >> 16);
        // sumf += q8.d[b] * (d * sd as f32 - dmin * sm as f32)
        return a.dact * (d * (float)sd - dmin * (float)sm);
    }
};

// ───────────────────────────────────── Q6_K ─────────────────────────────────────
// Lane l: block-in-step q = l/4, half h = (l%4)/2, c = l%2 selects l in [16c, 16c+16). The lane
// decodes the four 16-element groups {l, l+32, l+64, l+96} of its half: 64 weights, scale indices
// h*8 + c + {0,2,4,6}. Codes stay biased (0..63) and the -32 offset is applied through the
// activation's per-16 sums, exactly the CPU's `sc * (sumi - 32*bsum)`. 16 blocks (3360 B) per
// wave step. Block stride 210 B is 2 mod 4: loads are 2-byte aligned.
struct FmtQ6K {
    static constexpr int kElemsPerStep = 4096;
    static constexpr bool kPer32 = false;
    static constexpr bool kOrdered = true;
    static constexpr int kBlockBytes = 210, kBlockElems = 256;
    static constexpr int kWide16Steps = 1;
    static constexpr bool kClampedLoads = false;
    static constexpr bool kLaneSums = true;
    static constexpr bool kRowAhead = true;  // rows of two and three wave steps run a whole row ahead: 4096 x 12288 5.28 -> 5.57 TB/s,
    static constexpr int kRowAheadMaxSteps = 3;  // 1024 x 12288 5.20 -> 5.48, 8192 columns +2.5 %; four steps lose 1.6 %
    struct Row {
        v4i qla, qlb, qh;
        v2i sc;
        uint32_t d;
    };
    struct Acts {
        int xa[16];
        int bs16[4];
        float dact;
    };
    __device__ static int units(int in_f) { return in_f / 256; }
    __device__ static bool valid(int t, int lane, int n) { return t * 16 + (lane >> 2) < n; }
    __device__ static void load_row(Row& r, const uint8_t* rowp, int t, int lane, bool ok) {
        if (ok) {
            const int h = (lane >> 1) & 1, c = lane & 1;
            const uint8_t* blk = rowp + (size_t)(t * 16 + (lane >> 2)) * 210;
            r.qla = load16_a2(blk + h * 64 + c * 16);
            r.qlb = load16_a2(blk + h * 64 + 32 + c * 16);
            r.qh = load16_a2(blk + 128 + h * 32 + c * 16);
            r.sc = gload<v2i_a2>(blk + 192 + h * 8);
            r.d = load_u16(blk + 208);
        } else {
            r.qla = r.qlb = r.qh = v4i{0, 0, 0, 0};
            r.sc = v2i{0, 0};
            r.d = 0;
        }
    }
    __device__ static void load_acts(Acts& a, const ActPtrs& s, int t, int lane, bool ok) {
        if (ok) {
            const int b = t * 16 + (lane >> 2), h = (lane >> 1) & 1, c = lane & 1;
            const int8_t* xb = s.qs + (size_t)b * 256 + h * 128 + c * 16;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const v4i v = *reinterpret_cast<const v4i*>(xb + 32 * k);
                a.xa[4 * k + 0] = v.x;
                a.xa[4 * k + 1] = v.y;
                a.xa[4 * k + 2] = v.z;
                a.xa[4 * k + 3] = v.w;
                a.bs16[k] = s.bsums16[(size_t)b * 16 + h * 8 + c + 2 * k];
            }
            a.dact = s.d[b];
        } else {
#pragma unroll
            for (int k = 0; k < 16; ++k) a.xa[k] = 0;
#pragma unroll
            for (int k = 0; k < 4; ++k) a.bs16[k] = 0;
            a.dact = 0.0f;
        }
    }
    template <bool STAGES>
    __device__ static float term(const Row& r, const Acts& a, int t, int lane, bool ok,
                                 const StagePtrs& st, size_t row_units) {
        const int c = lane & 1;
        const uint32_t m4 = 0x0F0F0F0Fu, m2 = 0x30303030u;
        const int la[4] = {r.qla.x, r.qla.y, r.qla.z, r.qla.w};
        const int lb[4] = {r.qlb.x, r.qlb.y, r.qlb.z, r.qlb.w};
        const int hh[4] = {r.qh.x, r.qh.y, r.qh.z, r.qh.w};
        int sumi[4] = {0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t lo = (uint32_t)la[j], hi = (uint32_t)lb[j], h = (uint32_t)hh[j];
            sumi[0] = dot4((int)((lo & m4) | ((h << 4) & m2)), a.xa[0 + j], sumi[0]);
            sumi[1] = dot4((int)((hi & m4) | ((h << 2) & m2)), a.xa[4 + j], sumi[1]);
            sumi[2] = dot4((int)(((lo >> 4) & m4) | (h & m2)), a.xa[8 + j], sumi[2]);
            sumi[3] = dot4((int)(((hi >> 4) & m4) | ((h >> 2) & m2)), a.xa[12 + j], sumi[3]);
        }
        // scales[h*8 + c + 2k]: byte (c + 2k) of the 8 bytes loaded at scales + h*8
        const uint32_t lo = (uint32_t)r.sc.x >> (8 * c), hi = (uint32_t)r.sc.y >> (8 * c);
        const int sc0 = (int)(int8_t)(lo & 0xFF), sc1 = (int)(int8_t)((lo >> 16) & 0xFF);
        const int sc2 = (int)(int8_t)(hi & 0xFF), sc3 = (int)(int8_t)((hi >> 16) & 0xFF);
        int part = __mul24(sc0, sumi[0] - 32 * a.bs16[0]);
        part += __mul24(sc1, sumi[1] - 32 * a.bs16[1]);
        part += __mul24(sc2, sumi[2] - 32 * a.bs16[2]);
        part += __mul24(sc3, sumi[3] - 32 * a.bs16[3]);
        const int isum = quad_sum(part);
        if (STAGES && ok && (lane & 3) == 0) st.a[row_units + t * 16 + (lane >> 2)] = isum;
        // sumf += d * q8.d[b] * isum as f32
        return f16_bits_to_f32(r.d) * a.dact * (float)isum;
    }
};

// ───────────────────────────────────── Q8_0 ─────────────────────────────────────
// Lane l owns 32-weight block t*64 + l of the row: 34 B = f16 scale + 32 int8, 2-byte aligned.
// 64 blocks (2048 weights, 2176 B) per wave step. Rows of whole 256s take the per-256 activation
// (scale shared by 8 lanes, kernels.rs:1170-1187); rows that are a multiple of 32 only take the
// per-32 activation, one scale per block (P32; kernels.rs:4972-4991, lib.rs:1037-1042).
// ALIGNED (rows of whole 64s: an even number of blocks, so rows start on a dword and the block
// parity gives the alignment): the last dword is fetched whole - an even block's runs 2 bytes into
// its odd neighbour, inside the row - which saves the second, conditional 2-byte load.
template <bool P32, bool ALIGNED = false>
struct FmtQ8_0T {
    static constexpr int kElemsPerStep = 2048;
    static constexpr bool kPer32 = P32;
    static constexpr bool kOrdered = false;
    static constexpr int kBlockBytes = 34, kBlockElems = 32;
    static constexpr int kWide16Steps = 4;
    static constexpr bool kClampedLoads = false;
    static constexpr bool kLaneSums = true;
    static constexpr bool kRowAhead = false;
    struct Row {
        v4i qa, qb;
        uint32_t d;
    };
    struct Acts {
        int xa[8];
        float dact;
    };
    __device__ static int units(int in_f) { return in_f / 32; }
    __device__ static bool valid(int t, int lane, int n) { return t * 64 + lane < n; }
    // Dword-aligned loads + register realignment (see realign2): a block 2 bytes past a 4-byte
    // boundary reads the 2 bytes before it (the previous block of the row or buffer) and never
    // past its own end.
    __device__ static void load_row(Row& r, const uint8_t* rowp, int t, int lane, bool ok) {
        if (ok) {
            const uint8_t* blk = rowp + (size_t)(t * 64 + lane) * 34;
            const bool odd = ALIGNED ? (lane & 1) != 0 : (reinterpret_cast<uintptr_t>(blk) & 2) != 0;
            const uint8_t* a = blk - (odd ? 2 : 0);
            const v4i lo = load16_a4(a), hi = load16_a4(a + 16);
            // last dword: bytes 32..33 always belong to the block, 34..35 only to an odd one
            uint32_t tail;
            if (ALIGNED) {
                tail = (uint32_t)load_u32(a + 32);
            } else {
                tail = load_u16(a + 32);
                if (odd) tail |= load_u16(a + 34) << 16;
            }
            const uint32_t sel = realign2_selector(odd);
            r.d = odd ? (uint32_t)lo.x >> 16 : (uint32_t)lo.x & 0xFFFFu;
            r.qa.x = realign2(lo.x, lo.y, sel);
            r.qa.y = realign2(lo.y, lo.z, sel);
            r.qa.z = realign2(lo.z, lo.w, sel);
            r.qa.w = realign2(lo.w, hi.x, sel);
            r.qb.x = realign2(hi.x, hi.y, sel);
            r.qb.y = realign2(hi.y, hi.z, sel);
            r.qb.z = realign2(hi.z, hi.w, sel);
            r.qb.w = realign2(hi.w, (int)tail, sel);
        } else {
            r.qa = r.qb = v4i{0, 0, 0, 0};
            r.d = 0;
        }
    }
    __device__ static void load_acts(Acts& a, const ActPtrs& s, int t, int lane, bool ok) {
        if (ok) {
            const int wb = t * 64 + lane;
            const v4i v0 = *reinterpret_cast<const v4i*>(s.qs + (size_t)wb * 32);
            const v4i v1 = *reinterpret_cast<const v4i*>(s.qs + (size_t)wb * 32 + 16);
            a.xa[0] = v0.x; a.xa[1] = v0.y; a.xa[2] = v0.z; a.xa[3] = v0.w;
            a.xa[4] = v1.x; a.xa[5] = v1.y; a.xa[6] = v1.z; a.xa[7] = v1.w;
            a.dact = s.d[P32 ? wb : wb >> 3];
        } else {
#pragma unroll
            for (int k = 0; k < 8; ++k) a.xa[k] = 0;
            a.dact = 0.0f;
        }
    }
    template <bool STAGES>
    __device__ static float term(const Row& r, const Acts& a, int t, int lane, bool ok,
                                 const StagePtrs& st, size_t row_units) {
        int ip = 0;
        ip = dot4(r.qa.x, a.xa[0], ip);
        ip = dot4(r.qa.y, a.xa[1], ip);
        ip = dot4(r.qa.z, a.xa[2], ip);
        ip = dot4(r.qa.w, a.xa[3], ip);
        ip = dot4(r.qb.x, a.xa[4], ip);
        ip = dot4(r.qb.y, a.xa[5], ip);
        ip = dot4(r.qb.z, a.xa[6], ip);
        ip = dot4(r.qb.w, a.xa[7], ip);
        if (STAGES && ok) st.a[row_units + t * 64 + lane] = ip;
        // sumf += d8 * d_w * iprod as f32   (per-32: d_w * d_x[b] * iprod - the same product)
        return a.dact * f16_bits_to_f32(r.d) * (float)ip;
    }
};
using FmtQ8_0 = FmtQ8_0T<false>;        // any row alignment (expert banks)
using FmtQ8_0A = FmtQ8_0T<false, true>;  // per-256 activation: rows are whole 256s, always aligned
using FmtQ8_0_32 = FmtQ8_0T<true>;
using FmtQ8_0_32A = FmtQ8_0T<true, true>;

// ───────────────────────────────────── Q2_0 ─────────────────────────────────────
// Lane l owns 64-weight block t*64 + l: 18 B = f16 scale + 16 bytes of 2-bit codes, 2-byte
// aligned. `(w >> 2s) & 0x03030303` pulls the codes of elements {4i+s} of a 16-element group into
// the four bytes of a word; the activation bytes are transposed once per wave (v_perm_b32) into
// that order, so each extracted word is a ready v_dot4 operand. 64 blocks (4096 weights,
// 1152 B) per wave step. Codes stay 0..3; the -1 offset is applied as `iprod - bsum` like the CPU.

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

// ALIGNED: rows of whole 128s have an even number of blocks, so every row starts on a dword and
// blocks alternate between a dword boundary and 2 bytes past one. Each lane then fetches its block
// with two dword-aligned loads (5 dwords from the boundary at or below the block; an even block's
// last dword runs 2 bytes into its odd neighbour, which is always inside the row) and realigns in
// registers, instead of one 16-byte load at 2-byte alignment, which runs well below full rate.
template <bool ALIGNED>
struct FmtQ2_0T {
    static constexpr int kElemsPerStep = 4096;
    static constexpr bool kPer32 = true;
    static constexpr bool kOrdered = false;
    static constexpr int kBlockBytes = 18, kBlockElems = 64;
    static constexpr int kWide16Steps = 3;
    static constexpr bool kClampedLoads = true;
    static constexpr bool kLaneSums = false;
    static constexpr bool kRowAhead = true;
    struct Row {
        v4i codes;
        uint32_t d;
    };
    struct Acts {
        int xt[16];  // xt[4j + s] = bytes {x[16j + 4i + s]}, i = 0..3
        float da0, da1, fb0, fb1;
    };
    __device__ static int units(int in_f) { return in_f / 64; }
    __device__ static bool valid(int t, int lane, int n) { return t * 64 + lane < n; }
    __device__ static void load_row(Row& r, const uint8_t* rowp, int t, int lane, bool ok) {
        if (ok) {
            load_row_clamped(r, rowp, t, lane, true);
        } else {
            r.codes = v4i{0, 0, 0, 0};
            r.d = 0;
        }
    }
    // For a `rowp` that is a readable row whatever `ok` says: lanes past the row's last block read
    // block 0 instead of being masked off (their activations are zero, so what they load
    // contributes +0.0), and the loads carry no predicate.
    __device__ static void load_row_clamped(Row& r, const uint8_t* rowp, int t, int lane, bool ok) {
        const int idx = ok ? t * 64 + lane : 0;
        const uint8_t* blk = rowp + (size_t)idx * 18;
        if (ALIGNED) {
            const bool odd = (idx & 1) != 0;
            const uint8_t* a = blk - (odd ? 2 : 0);
            const v4i lo = load16_a4(a);
            const int w4 = load_u32(a + 16);
            const uint32_t sel = realign2_selector(odd);
            r.d = odd ? (uint32_t)lo.x >> 16 : (uint32_t)lo.x & 0xFFFFu;
            r.codes = v4i{realign2(lo.x, lo.y, sel), realign2(lo.y, lo.z, sel), realign2(lo.z, lo.w, sel),
                          realign2(lo.w, w4, sel)};
        } else {
            r.d = load_u16(blk);
            r.codes = load16_a2(blk + 2);
        }
    }
    __device__ static void load_acts(Acts& a, const ActPtrs& s, int t, int lane, bool ok) {
        if (ok) {
            const int b = t * 64 + lane;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const v4i v = *reinterpret_cast<const v4i*>(s.qs + (size_t)b * 64 + 16 * j);
                const int in[4] = {v.x, v.y, v.z, v.w};
                transpose4x4(in, &a.xt[4 * j]);
            }
            a.da0 = s.d[2 * b];
            a.da1 = s.d[2 * b + 1];
            a.fb0 = (float)s.bsums[2 * b];
            a.fb1 = (float)s.bsums[2 * b + 1];
        } else {
#pragma unroll
            for (int k = 0; k < 16; ++k) a.xt[k] = 0;
            a.da0 = 0.0f;
            a.da1 = 0.0f;
            a.fb0 = 0.0f;
            a.fb1 = 0.0f;
        }
    }
    template <bool STAGES>
    __device__ static float term(const Row& r, const Acts& a, int t, int lane, bool ok,
                                 const StagePtrs& st, size_t row_units) {
        return term_impl<STAGES, false>(r, a, t, lane, ok, st, row_units);
    }
    // One weight row against several activation rows: the unpacked code words are shared by all
    // of them, so the plain four-shift unpack with one accumulator per sub-block is cheaper there
    // than the two-accumulator form below.
    template <bool STAGES>
    __device__ static float term_shared(const Row& r, const Acts& a, int t, int lane, bool ok,
                                        const StagePtrs& st, size_t row_units) {
        return term_impl<STAGES, true>(r, a, t, lane, ok, st, row_units);
    }
    template <bool STAGES, bool SHARED>
    __device__ static float term_impl(const Row& r, const Acts& a, int t, int lane, bool ok,
                                      const StagePtrs& st, size_t row_units) {
        const uint32_t cw[4] = {(uint32_t)r.codes.x, (uint32_t)r.codes.y, (uint32_t)r.codes.z,
                                (uint32_t)r.codes.w};
        int ip0 = 0, ip1 = 0;
        if (SHARED) {
#pragma unroll
            for (int sft = 0; sft < 4; ++sft) {
                ip0 = dot4((int)((cw[0] >> (2 * sft)) & 0x03030303u), a.xt[0 + sft], ip0);
                ip0 = dot4((int)((cw[1] >> (2 * sft)) & 0x03030303u), a.xt[4 + sft], ip0);
                ip1 = dot4((int)((cw[2] >> (2 * sft)) & 0x03030303u), a.xt[8 + sft], ip1);
                ip1 = dot4((int)((cw[3] >> (2 * sft)) & 0x03030303u), a.xt[12 + sft], ip1);
            }
        } else {
            // Code k of every byte (bits 2k, 2k+1): k = 0 and 1 are masked out of w and w >> 2 as
            // they are; k = 2 and 3 are masked in place at bits 4-5 of the same two words, i.e.
            // 16 x code (<= 48, still a positive int8), and their dot is divided by 16 afterwards
            // (exact). One shift per word instead of three.
            int lo[2] = {0, 0}, hi[2] = {0, 0};
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const uint32_t c = cw[w], c2 = c >> 2;
                lo[w >> 1] = dot4((int)(c & 0x03030303u), a.xt[4 * w + 0], lo[w >> 1]);
                lo[w >> 1] = dot4((int)(c2 & 0x03030303u), a.xt[4 * w + 1], lo[w >> 1]);
                hi[w >> 1] = dot4((int)(c & 0x30303030u), a.xt[4 * w + 2], hi[w >> 1]);
                hi[w >> 1] = dot4((int)(c2 & 0x30303030u), a.xt[4 * w + 3], hi[w >> 1]);
            }
            ip0 = lo[0] + (hi[0] >> 4);
            ip1 = lo[1] + (hi[1] >> 4);
        }
        if (STAGES && ok) {
            // stage layout is per 32-element sub-block: two per unit
            st.a[2 * row_units + 2 * (t * 64 + lane)] = ip0;
            st.a[2 * row_units + 2 * (t * 64 + lane) + 1] = ip1;
        }
        const float d = f16_bits_to_f32(r.d);
        // sumf += d * q8.d[s] * (iprod as f32 - bsum[s] as f32), sub-block 2b then 2b+1
        float s = d * a.da0 * ((float)ip0 - a.fb0);
        s += d * a.da1 * ((float)ip1 - a.fb1);
        return s;
    }
};
using FmtQ2_0 = FmtQ2_0T<false>;
using FmtQ2_0A = FmtQ2_0T<true>;

// ───────────────────────────────────── Q5_K ─────────────────────────────────────
// Q4_K's lane mapping (block-in-step q = l/4, nibble pair p = l%4) on the 176-byte block
// [f16 d][f16 dmin][u8 scales[12]][u8 qh[32]][u8 ql[128]]: the 5th code bit of sub-block s,
// element l, is bit s of qh[l], so pair p takes bits 2p (even sub-block) and 2p+1 (odd) of the 32
// qh bytes, which all four lanes of the quad load (same cache lines). Block stride 176 B is a
// multiple of 16: every load is 16-byte aligned.
struct FmtQ5K {
    static constexpr int kElemsPerStep = 4096;
    static constexpr bool kPer32 = false;
    static constexpr bool kOrdered = true;
    static constexpr int kBlockBytes = 176, kBlockElems = 256;
    static constexpr int kWide16Steps = 2;
    static constexpr bool kClampedLoads = false;
    static constexpr bool kLaneSums = true;
    static constexpr bool kRowAhead = false;
    struct Row {
        v4i hdr, ha, hb, qa, qb;
    };
    typedef FmtQ4K::Acts Acts;
    __device__ static int units(int in_f) { return in_f / 256; }
    __device__ static bool valid(int t, int lane, int n) { return t * 16 + (lane >> 2) < n; }
    __device__ static void load_row(Row& r, const uint8_t* rowp, int t, int lane, bool ok) {
        if (ok) {
            const uint8_t* blk = rowp + (size_t)(t * 16 + (lane >> 2)) * 176;
            const int p = lane & 3;
            r.hdr = load16(blk);
            r.ha = load16(blk + 16);
            r.hb = load16(blk + 32);
            r.qa = load16(blk + 48 + p * 32);
            r.qb = load16(blk + 64 + p * 32);
        } else {
            r.hdr = r.ha = r.hb = r.qa = r.qb = v4i{0, 0, 0, 0};
        }
    }
    // The same pieces out of a wave's LDS ring (see FmtQ4K::load_row_ring).
    static constexpr uint32_t kStepBytes = 16 * 176;
    static constexpr int kRingMaxSteps = 3, kRingLongInstr = 3;  // (two: 5.79 TB/s, three: 5.83, four: one workgroup per compute unit, 5.21)
    __device__ static void load_row_ring(Row& r, const uint8_t* ring, uint32_t pos, uint32_t ring_bytes, int lane, bool ok) {
        const int p = lane & 3;
        uint32_t o[5];
        o[0] = pos + (uint32_t)(lane >> 2) * 176;
        o[1] = o[0] + 16;
        o[2] = o[0] + 32;
        o[3] = o[0] + 48 + p * 32;
        o[4] = o[0] + 64 + p * 32;
#pragma unroll
        for (int i = 0; i < 5; ++i) o[i] = o[i] >= ring_bytes ? o[i] - ring_bytes : o[i];
        r.hdr = *reinterpret_cast<const v4i*>(ring + o[0]);
        r.ha = *reinterpret_cast<const v4i*>(ring + o[1]);
        r.hb = *reinterpret_cast<const v4i*>(ring + o[2]);
        r.qa = *reinterpret_cast<const v4i*>(ring + o[3]);
        r.qb = *reinterpret_cast<const v4i*>(ring + o[4]);
        r.hdr.x = ok ? r.hdr.x : 0;  // d = dmin = 0: a lane without a block contributes +0.0
    }
    __device__ static void load_acts(Acts& a, const ActPtrs& s, int t, int lane, bool ok) {
        FmtQ4K::load_acts(a, s, t, lane, ok);
    }
    template <bool STAGES>
    __device__ static float term(const Row& r, const Acts& a, int t, int lane, bool ok,
                                 const StagePtrs& st, size_t row_units) {
        const int p = lane & 3;
        const uint32_t m4 = 0x0F0F0F0Fu, b1 = 0x01010101u;
        int ip_e = 0, ip_o = 0;
        const int wq[8] = {r.qa.x, r.qa.y, r.qa.z, r.qa.w, r.qb.x, r.qb.y, r.qb.z, r.qb.w};
        const int hq[8] = {r.ha.x, r.ha.y, r.ha.z, r.ha.w, r.hb.x, r.hb.y, r.hb.z, r.hb.w};
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const uint32_t w = (uint32_t)wq[k], h = (uint32_t)hq[k] >> (2 * p);
            ip_e = dot4((int)((w & m4) | ((h & b1) << 4)), a.xa[k], ip_e);
            ip_o = dot4((int)(((w >> 4) & m4) | (((h >> 1) & b1) << 4)), a.xa[8 + k], ip_o);
        }
        uint32_t sc8[2], mn8[2];
        k4_all((uint32_t)r.hdr.y, (uint32_t)r.hdr.z, (uint32_t)r.hdr.w, sc8, mn8);
        const uint32_t scw = (p & 2) ? sc8[1] : sc8[0];
        const uint32_t mnw = (p & 2) ? mn8[1] : mn8[0];
        const int sh = (p & 1) * 16;
        const int sc_e = (scw >> sh) & 0xFF, sc_o = (scw >> (sh + 8)) & 0xFF;
        const int m_e = (mnw >> sh) & 0xFF, m_o = (mnw >> (sh + 8)) & 0xFF;
        // |ip| <= 32 * 31 * 127 < 2^17 and sc < 2^6: the 24-bit multiply is exact
        const int sd = quad_sum(__mul24(sc_e, ip_e) + __mul24(sc_o, ip_o));
        const int sm = quad_sum(__mul24(m_e, a.bs0) + __mul24(m_o, a.bs1));
        if (STAGES && ok && p == 0) {
            st.a[row_units + t * 16 + (lane >> 2)] = sd;
            st.b[row_units + t * 16 + (lane >> 2)] = sm;
        }
        const float d = f16_bits_to_f32((uint32_t)r.hdr.x & 0xFFFFu);
        const float dmin = f16_bits_to_f32((uint32_t)r.hdr.x >> 16);
        // sumf += q8.d[b] * (d * sd as f32 - dmin * sm as f32)
        return a.dact * (d * (float)sd - dmin * (float)sm);
    }
};

// ───────────────────────────────────── Q2_K / Q3_K ─────────────────────────────────────
// Both keep a block's 2-bit fields in qs[64]: element 128 n + 32 j + 16 half + l is field j of byte
// qs[32 n + 16 half + l], and its 16-element sub-block 8 n + 2 j + half has a scale of its own. Lane l:
// block-in-step q = l/4, p = l%4 = 2 n + half: the lane owns the 16 bytes qs[16 p ..], i.e. the four
// sub-blocks 8 n + half + 2 j, and their 64 activation bytes (FmtQ6K's activation mapping: groups of
// 16 at 128 n + 16 half + 32 j, per-16 sums at 8 n + half + 2 j). 16 blocks per wave step.
//
// Q2_K (84-byte block, 4-byte aligned: [u8 scales[16]][u8 qs[64]][f16 d][f16 dmin]): a scale byte is a
// 4-bit scale (low) and a 4-bit min (high); sd = sum scale * (q2 . q8), sm = sum min * bsum16, and the
// CPU's term q8.d[b] * (d * sd - dmin * sm) (kernels.rs:315-361), blocks in ascending order.
struct FmtQ2K {
    static constexpr int kElemsPerStep = 4096;
    static constexpr bool kPer32 = false;
    static constexpr bool kOrdered = true;
    static constexpr int kBlockBytes = 84, kBlockElems = 256;
    static constexpr int kWide16Steps = 3;
    static constexpr bool kClampedLoads = true;
    static constexpr bool kLaneSums = true;
    static constexpr bool kRowAhead = false;
    struct Row {
        v4i q;
        v2i sc;       // scales[8 n .. 8 n + 8)
        uint32_t dm;  // d | dmin << 16
    };
    typedef FmtQ6K::Acts Acts;
    __device__ static int units(int in_f) { return in_f / 256; }
    __device__ static bool valid(int t, int lane, int n) { return t * 16 + (lane >> 2) < n; }
    // For a `rowp` that is a readable row whatever `ok` says: lanes past the row's last block read
    // block 0 (their activations and activation scale are zero: a term of +0.0 that nothing adds),
    // and the loads carry no predicate.
    __device__ static void load_row_clamped(Row& r, const uint8_t* rowp, int t, int lane, bool ok) {
        const uint8_t* blk = rowp + (size_t)(ok ? t * 16 + (lane >> 2) : 0) * 84;
        const int p = lane & 3;
        r.q = load16_a4(blk + 16 + 16 * p);
        r.sc = gload<v2i_a4>(blk + 8 * (p >> 1));
        r.dm = (uint32_t)load_u32(blk + 80);
    }
    __device__ static void load_row(Row& r, const uint8_t* rowp, int t, int lane, bool ok) {
        if (ok) {
            load_row_clamped(r, rowp, t, lane, true);
        } else {
            r.q = v4i{0, 0, 0, 0};
            r.sc = v2i{0, 0};
            r.dm = 0;
        }
    }
    __device__ static void load_acts(Acts& a, const ActPtrs& s, int t, int lane, bool ok) {
        FmtQ6K::load_acts(a, s, t, lane, ok);
    }
    template <bool STAGES>
    __device__ static float term(const Row& r, const Acts& a, int t, int lane, bool ok,
                                 const StagePtrs& st, size_t row_units) {
        const int half = lane & 1;
        const int qw[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
        int pd = 0, pm = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            // bit pairs 1 and 2 are multiplied where they sit (4 and 16 times the code still fit a
            // signed byte) and the exact sum is shifted back
            int ip = 0;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t c = j == 3 ? ((uint32_t)qw[k] >> 6) & 0x03030303u : (uint32_t)qw[k] & (0x03030303u << (2 * j));
                ip = dot4((int)c, a.xa[4 * j + k], ip);
            }
            if (j == 1 || j == 2) ip >>= 2 * j;
            // sub-block 8 n + half + 2 j: byte half + 2 j of the eight scale bytes
            const uint32_t sb = ((uint32_t)(j < 2 ? r.sc.x : r.sc.y) >> (8 * (half + 2 * (j & 1)))) & 0xFFu;
            pd += __mul24((int)(sb & 15u), ip);  // |ip| <= 16 * 3 * 127: the 24-bit multiply is exact
            pm += __mul24((int)(sb >> 4), a.bs16[j]);
        }
        const int sd = quad_sum(pd), sm = quad_sum(pm);
        if (STAGES && ok && (lane & 3) == 0) {
            st.a[row_units + t * 16 + (lane >> 2)] = sd;
            st.b[row_units + t * 16 + (lane >> 2)] = sm;
        }
        const float d = f16_bits_to_f32(r.dm & 0xFFFFu), dmin = f16_bits_to_f32(r.dm >> 16);
        // sumf += q8.d[b] * (d * sd as f32 - dmin * sm as f32)
        return a.dact * (d * (float)sd - dmin * (float)sm);
    }
};

// TQ1_0 (54-byte block, 2-byte aligned: [u8 qs[48]][u8 qh[4]][f16 d]): base-3 packed ternary. A byte
// holds five digits (qh: four): digit n is the high byte of three times (byte * 3^n mod 256), i.e.
// repeated "times three, take the carry". Elements come in three runs - qs[0..32) x 5 digits ->
// 32 n + m, qs[32..48) x 5 -> 160 + 16 n + m, qh[0..4) x 4 -> 240 + 4 n + j - and a weight is
// (digit - 1) d: iprod = sum digit * q8 - (the activation's code sum), term d * q8.d[b] * iprod
// (crates/infr-cpu/src/kernels.rs:3167-3240), blocks in ascending order. Lane p of a block's four owns
// qs[8 p .. 8 p + 8), qs[32 + 4 p .. + 4) and qh[p]: 64 weights, whose activations are gathered to
// match (digit n of word k of the first run meets bytes 32 n + 8 p + 4 k .. + 3). Four bytes are
// unpacked at a time, even and odd bytes in the two halves of a word (three times a byte fits 16 bits).
struct FmtTQ1_0 {
    static constexpr int kElemsPerStep = 4096;
    static constexpr bool kPer32 = false;
    static constexpr bool kOrdered = true;
    static constexpr int kBlockBytes = 54, kBlockElems = 256;
    static constexpr int kWide16Steps = 3;
    static constexpr bool kClampedLoads = false;
    static constexpr bool kLaneSums = true;
    static constexpr bool kRowAhead = false;
    struct Row {
        v2i a;       // qs[8 p .. 8 p + 8)
        uint32_t b;  // qs[32 + 4 p .. + 4)
        v2i tail;    // bytes 46 .. 53: qs[46], qs[47], qh[0..4), d
    };
    struct Acts {
        int xa[16];  // 2 n + k: first run, digit n, word k; 10 + n: second run, digit n; 15: third run
        int bs;      // code sum of the 64 activations this lane's index p stands for (two per-32 sums)
        float dact;
    };
    __device__ static int units(int in_f) { return in_f / 256; }
    __device__ static bool valid(int t, int lane, int n) { return t * 16 + (lane >> 2) < n; }
    __device__ static void load_row(Row& r, const uint8_t* rowp, int t, int lane, bool ok) {
        if (ok) {
            const uint8_t* blk = rowp + (size_t)(t * 16 + (lane >> 2)) * 54;
            const int p = lane & 3;
            r.a = gload<v2i_a2>(blk + 8 * p);
            r.b = (uint32_t)gload<int_a2>(blk + 32 + 4 * p);
            r.tail = gload<v2i_a2>(blk + 46);
        } else {
            r.a = r.tail = v2i{0, 0};
            r.b = 0;
        }
    }
    __device__ static void load_acts(Acts& a, const ActPtrs& s, int t, int lane, bool ok) {
        if (ok) {
            const int b = t * 16 + (lane >> 2), p = lane & 3;
            const int8_t* base = s.qs + (size_t)b * 256;
#pragma unroll
            for (int n = 0; n < 5; ++n) {
                const v2i v = *reinterpret_cast<const v2i*>(base + 32 * n + 8 * p);
                a.xa[2 * n] = v.x;
                a.xa[2 * n + 1] = v.y;
                a.xa[10 + n] = *reinterpret_cast<const int*>(base + 160 + 16 * n + 4 * p);
            }
            // elements 240 + 4 n + p: byte p of each of the last four words
            const v4i last = *reinterpret_cast<const v4i*>(base + 240);
            const int sh = 8 * p;
            a.xa[15] = (int)((((uint32_t)last.x >> sh) & 0xFFu) | ((((uint32_t)last.y >> sh) & 0xFFu) << 8) |
                             ((((uint32_t)last.z >> sh) & 0xFFu) << 16) | ((((uint32_t)last.w >> sh) & 0xFFu) << 24));
            a.bs = s.bsums[(size_t)b * 8 + 2 * p] + s.bsums[(size_t)b * 8 + 2 * p + 1];
            a.dact = s.d[b];
        } else {
#pragma unroll
            for (int k = 0; k < 16; ++k) a.xa[k] = 0;
            a.bs = 0;
            a.dact = 0.0f;
        }
    }
    // The five digits of each of a word's four bytes: out[n] holds digit n of byte k in byte k.
    __device__ static void digits5(uint32_t w, uint32_t (&out)[5]) {
        uint32_t e = w & 0x00FF00FFu, o = (w >> 8) & 0x00FF00FFu;
#pragma unroll
        for (int n = 0; n < 5; ++n) {
            const uint32_t te = e * 3u, to = o * 3u;  // per 16-bit half: at most 765
            out[n] = ((te >> 8) & 0x00FF00FFu) | (to & 0xFF00FF00u);
            e = te & 0x00FF00FFu;
            o = to & 0x00FF00FFu;
        }
    }
    template <bool STAGES>
    __device__ static float term(const Row& r, const Acts& a, int t, int lane, bool ok,
                                 const StagePtrs& st, size_t row_units) {
        const int p = lane & 3;
        uint32_t d0[5], d1[5], d2[5];
        digits5((uint32_t)r.a.x, d0);
        digits5((uint32_t)r.a.y, d1);
        digits5(r.b, d2);
        int ip = 0;
#pragma unroll
        for (int n = 0; n < 5; ++n) {
            ip = dot4((int)d0[n], a.xa[2 * n], ip);
            ip = dot4((int)d1[n], a.xa[2 * n + 1], ip);
            ip = dot4((int)d2[n], a.xa[10 + n], ip);
        }
        // qh[p]: four digits, digit n to byte n
        const uint32_t qh = ((uint32_t)r.tail.x >> 16) | ((uint32_t)r.tail.y << 16);
        uint32_t q = (qh >> (8 * p)) & 0xFFu, dq = 0;
#pragma unroll
        for (int n = 0; n < 4; ++n) {
            const uint32_t tq = q * 3u;
            dq |= (tq >> 8) << (8 * n);
            q = tq & 0xFFu;
        }
        ip = dot4((int)dq, a.xa[15], ip);
        const int iprod = quad_sum(ip - a.bs);
        if (STAGES && ok && p == 0) st.a[row_units + t * 16 + (lane >> 2)] = iprod;
        return f16_bits_to_f32((uint32_t)r.tail.y >> 16) * a.dact * (float)iprod;  // sumf += d * q8.d[b] * iprod as f32
    }
};

// TQ2_0 (66-byte block, 2-byte aligned: [u8 qs[64]][f16 d]): the bit pairs are laid out as Q2_K's, a
// code q is the ternary weight q - 1 with one scale per superblock: iprod = sum (q - 1) * q8 =
// sum q * q8 - (the activation's code sum), term d * q8.d[b] * iprod
// (crates/infr-cpu/src/kernels.rs:3066-3126), blocks in ascending order. Lanes as for Q2_K.
struct FmtTQ2_0 {
    static constexpr int kElemsPerStep = 4096;
    static constexpr bool kPer32 = false;
    static constexpr bool kOrdered = true;
    static constexpr int kBlockBytes = 66, kBlockElems = 256;
    static constexpr int kWide16Steps = 3;
    static constexpr bool kClampedLoads = false;
    static constexpr bool kLaneSums = true;
    // rows of two and three wave steps run a whole row ahead (4096 x 12288: 4.4 -> 4.8 TB/s, 1024 x 12288:
    // 4.2 -> 4.6; 8192 columns the same); four steps lose a fifth that way (two sets of four rows' registers)
    static constexpr bool kRowAhead = true;
    static constexpr int kRowAheadMaxSteps = 3;
    struct Row {
        v4i q;
        uint32_t d;
    };
    typedef FmtQ6K::Acts Acts;
    __device__ static int units(int in_f) { return in_f / 256; }
    __device__ static bool valid(int t, int lane, int n) { return t * 16 + (lane >> 2) < n; }
    __device__ static void load_row(Row& r, const uint8_t* rowp, int t, int lane, bool ok) {
        if (ok) {
            const uint8_t* blk = rowp + (size_t)(t * 16 + (lane >> 2)) * 66;
            r.q = load16_a2(blk + 16 * (lane & 3));
            r.d = load_u16(blk + 64);
        } else {
            r.q = v4i{0, 0, 0, 0};
            r.d = 0;
        }
    }
    __device__ static void load_acts(Acts& a, const ActPtrs& s, int t, int lane, bool ok) {
        FmtQ6K::load_acts(a, s, t, lane, ok);
    }
    template <bool STAGES>
    __device__ static float term(const Row& r, const Acts& a, int t, int lane, bool ok,
                                 const StagePtrs& st, size_t row_units) {
        const int qw[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
        int part = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int ip = 0;  // (bit pairs 1 and 2 multiplied where they sit, as for Q2_K)
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t c = j == 3 ? ((uint32_t)qw[k] >> 6) & 0x03030303u : (uint32_t)qw[k] & (0x03030303u << (2 * j));
                ip = dot4((int)c, a.xa[4 * j + k], ip);
            }
            if (j == 1 || j == 2) ip >>= 2 * j;
            part += ip - a.bs16[j];
        }
        const int iprod = quad_sum(part);
        if (STAGES && ok && (lane & 3) == 0) st.a[row_units + t * 16 + (lane >> 2)] = iprod;
        return f16_bits_to_f32(r.d) * a.dact * (float)iprod;  // sumf += d * q8.d[b] * iprod as f32
    }
};

// Q3_K (110-byte block, 2-byte aligned: [u8 hmask[32]][u8 qs[64]][u8 scales[12]][f16 d]): a code is
// the 2-bit field plus bit 4 n + j of hmask[16 half + l] as its third bit; sixteen 6-bit scales are
// packed as low nibbles, high nibbles and a word of top bit pairs (q3k_scales, kernels.rs:764-783),
// and enter as sc6 - 32. isum = sum (sc6 - 32) * (q3 . q8 - 4 bsum16), term d * q8.d[b] * isum
// (kernels.rs:812-852), blocks in ascending order.
struct FmtQ3K {
    static constexpr int kElemsPerStep = 4096;
    static constexpr bool kPer32 = false;
    static constexpr bool kOrdered = true;
    static constexpr int kBlockBytes = 110, kBlockElems = 256;
    static constexpr int kWide16Steps = 2;
    static constexpr bool kClampedLoads = true;
    // (one-step rows: 4.45 TB/s with predicated loads against 4.27; three-step rows a whole row ahead:
    // 4.13 unpredicated against 3.97)
    static constexpr bool kClampedOneAhead = false;
    static constexpr bool kLaneSums = true;
    static constexpr bool kRowAhead = true;
    // A quad's lanes split the fields they all need and exchange them in registers (term): lane p
    // fetches hmask bytes 8 p .. 8 p + 7 and one word of the block's last 16 bytes - scale words 0..2
    // for p < 3, the word at byte 106 (two scale bytes and d) for p = 3 - so a block's 110 bytes are
    // requested once (112 with the overlap) instead of 184 over the quad.
    struct Row {
        v4i q;
        v2i hm8;
        uint32_t tail;
    };
    typedef FmtQ6K::Acts Acts;
    __device__ static int units(int in_f) { return in_f / 256; }
    __device__ static bool valid(int t, int lane, int n) { return t * 16 + (lane >> 2) < n; }
    // (lanes past the row's last block read block 0 of a readable row, as for Q2_K)
    __device__ static void load_row_clamped(Row& r, const uint8_t* rowp, int t, int lane, bool ok) {
        const uint8_t* blk = rowp + (size_t)(ok ? t * 16 + (lane >> 2) : 0) * 110;
        const int p = lane & 3;
        r.hm8 = gload<v2i_a2>(blk + 8 * p);
        r.q = load16_a2(blk + 32 + 16 * p);
        r.tail = (uint32_t)gload<int_a2>(blk + (p < 3 ? 96 + 4 * p : 106));
    }
    __device__ static void load_row(Row& r, const uint8_t* rowp, int t, int lane, bool ok) {
        if (ok) {
            load_row_clamped(r, rowp, t, lane, true);
        } else {
            r.q = v4i{0, 0, 0, 0};
            r.hm8 = v2i{0, 0};
            r.tail = 0;
        }
    }
    __device__ static void load_acts(Acts& a, const ActPtrs& s, int t, int lane, bool ok) {
        FmtQ6K::load_acts(a, s, t, lane, ok);
    }
    template <bool STAGES>
    __device__ static float term(const Row& r, const Acts& a, int t, int lane, bool ok,
                                 const StagePtrs& st, size_t row_units) {
        const int n = (lane >> 1) & 1, half = lane & 1;
        const int qw[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
        // hmask[16 half ..]: the two words of lane 2 half, then those of lane 2 half + 1
        const int hw[4] = {__builtin_amdgcn_mov_dpp(r.hm8.x, 0x88, 0xF, 0xF, true),   // quad_perm [0,2,0,2]
                           __builtin_amdgcn_mov_dpp(r.hm8.y, 0x88, 0xF, 0xF, true),
                           __builtin_amdgcn_mov_dpp(r.hm8.x, 0xDD, 0xF, 0xF, true),   // quad_perm [1,3,1,3]
                           __builtin_amdgcn_mov_dpp(r.hm8.y, 0xDD, 0xF, 0xF, true)};
        const uint32_t sc_x = (uint32_t)__builtin_amdgcn_mov_dpp((int)r.tail, 0x00, 0xF, 0xF, true);  // lane 0's word
        const uint32_t sc_y = (uint32_t)__builtin_amdgcn_mov_dpp((int)r.tail, 0x55, 0xF, 0xF, true);  // lane 1's
        const uint32_t sc_z = (uint32_t)__builtin_amdgcn_mov_dpp((int)r.tail, 0xAA, 0xF, 0xF, true);  // lane 2's
        const uint32_t d16 = (uint32_t)__builtin_amdgcn_mov_dpp((int)r.tail, 0xFF, 0xF, 0xF, true) >> 16;  // lane 3's: d on top
        // scales 8 n .. 8 n + 7 as two words of bytes: nibbles of the first eight bytes (low for
        // n = 0, high for n = 1) with two more bits each from the last four
        const uint32_t k1 = 0x03030303u, k2 = 0x0F0F0F0Fu, tt = sc_z >> (4 * n);
        const uint32_t w0 = ((sc_x >> (4 * n)) & k2) | ((tt & k1) << 4);
        const uint32_t w1 = ((sc_y >> (4 * n)) & k2) | (((tt >> 2) & k1) << 4);
        // hmask bits 4 n .. 4 n + 3 of every byte moved to bits 2 .. 5: bit pair j's third bit then
        // sits 2 + j above bit 0
        uint32_t hs[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) hs[k] = ((uint32_t)hw[k] >> (4 * n)) << 2;
        int part = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            // bit pairs 1 and 2 are multiplied where they sit, with the third bit moved next to them
            // (4 and 16 times a code of 0..7 still fit a signed byte); the exact sum is shifted back
            int ip = 0;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                uint32_t c;
                if (j == 0) c = ((uint32_t)qw[k] & 0x03030303u) | (hs[k] & 0x04040404u);
                else if (j == 1) c = ((uint32_t)qw[k] & 0x0C0C0C0Cu) | ((hs[k] << 1) & 0x10101010u);
                else if (j == 2) c = ((uint32_t)qw[k] & 0x30303030u) | ((hs[k] << 2) & 0x40404040u);
                else c = (((uint32_t)qw[k] >> 6) & 0x03030303u) | ((hs[k] >> 3) & 0x04040404u);
                ip = dot4((int)c, a.xa[4 * j + k], ip);
            }
            if (j == 1 || j == 2) ip >>= 2 * j;
            const int s = (int)(((j < 2 ? w0 : w1) >> (8 * (half + 2 * (j & 1)))) & 0xFFu) - 32;
            part += __mul24(s, ip - 4 * a.bs16[j]);  // |.| <= 16 * 11 * 127: the 24-bit multiply is exact
        }
        const int isum = quad_sum(part);
        if (STAGES && ok && (lane & 3) == 0) st.a[row_units + t * 16 + (lane >> 2)] = isum;
        // sumf += d * q8.d[b] * isum as f32
        return f16_bits_to_f32(d16) * a.dact * (float)isum;
    }
};

// ───────────────── Q4_0 / Q4_1 / Q5_0 / Q5_1 / IQ4_NL: 32 weights per block ─────────────────
// Lane l owns block t*64 + l of the row: an f16 scale (plus an f16 min for the _1 formats, plus a
// 32-bit mask of 5th code bits for the Q5 formats) and 16 bytes of nibbles. Byte j holds element j
// in its low nibble and element j+16 in its high nibble, so `w & 0x0F0F0F0F` and `(w >> 4) & ...`
// of the four nibble words are ready v_dot4 operands against activation words 0..3 and 4..7. The
// 5th bits of four consecutive elements are spread from the mask to bit 4 of four bytes with one
// multiply; IQ4_NL's nibbles index a 16-entry signed table through two v_perm_b32 and a select.
// Against the per-32 activation (scale and code sum per block). 64 blocks (2048 weights) per wave
// step. Strides 18 and 22 are 2 mod 4: those blocks are fetched as dwords from the 4-byte boundary
// at or below the block and realigned in registers (realign2); strides 20 and 24 are dword-aligned.
enum class Nib32 { Q4_0, Q4_1, Q5_0, Q5_1, IQ4_NL };

__device__ __forceinline__ uint32_t spread4_to_bit4(uint32_t bits) {
    // bits 0..3 -> bit 4 of bytes 0..3 (the four partial products land on distinct bits)
    return (__umul24(bits & 0xFu, 0x00204081u) & 0x01010101u) << 4;
}

// KVALUES_IQ4NL (crates/infr-gguf/src/dequant.rs:439-441) as four little-endian words of int8.
__device__ __forceinline__ int iq4nl_lookup(uint32_t nib) {
    const uint32_t sel = nib & 0x07070707u;
    const uint32_t lo = __builtin_amdgcn_perm(0xF6EADDCFu, 0xBFAD9881u, sel);  // entries 0..7
    const uint32_t hi = __builtin_amdgcn_perm(0x71594535u, 0x26190D01u, sel);  // entries 8..15
    const uint32_t pick = ((nib >> 3) & 0x01010101u) * 0xFFu;                  // 0xFF where nibble >= 8
    return (int)((hi & pick) | (lo & ~pick));
}

// ───────────────────────────────────── IQ4_XS ─────────────────────────────────────
// 136-byte block, 8-byte aligned: [f16 d][u16 scales_h][u8 scales_l[4]][u8 qs[128]]. Sub-block ib
// (32 weights) is 16 bytes - low nibbles elements 0..15, high nibbles 16..31 - of indices into
// IQ4_NL's signed table, with a 6-bit scale ls (nibble ib of scales_l, two more bits from
// scales_h), entering as ls - 32: isum = sum_ib (ls - 32) * (table[q] . q8), term
// (d * q8.d[b]) * isum (crates/infr-cpu/src/kernels.rs:995-1036), blocks in ascending order.
// Lanes as for Q4_K: block-in-step q = l / 4, lane p = l % 4 owns qs[32 p .. 32 p + 31] - sub-blocks
// 2 p and 2 p + 1 - against 64 consecutive activation bytes.
struct FmtIQ4XS {
    static constexpr int kElemsPerStep = 4096;
    static constexpr bool kPer32 = false;
    static constexpr bool kOrdered = true;
    static constexpr int kBlockBytes = 136, kBlockElems = 256;
    static constexpr int kWide16Steps = 3;
    static constexpr bool kClampedLoads = false;
    static constexpr bool kLaneSums = true;
    static constexpr bool kRowAhead = false;
    struct Row {
        v2i hdr;  // d | scales_h << 16, scales_l
        v4i qa, qb;
    };
    typedef FmtQ4K::Acts Acts;
    __device__ static int units(int in_f) { return in_f / 256; }
    __device__ static bool valid(int t, int lane, int n) { return t * 16 + (lane >> 2) < n; }
    __device__ static void load_row(Row& r, const uint8_t* rowp, int t, int lane, bool ok) {
        if (ok) {
            const uint8_t* blk = rowp + (size_t)(t * 16 + (lane >> 2)) * 136;
            const int p = lane & 3;
            r.hdr = gload<v2i_a4>(blk);
            r.qa = load16_a4(blk + 8 + p * 32);
            r.qb = load16_a4(blk + 24 + p * 32);
        } else {
            r.hdr = v2i{0, 0};
            r.qa = r.qb = v4i{0, 0, 0, 0};
        }
    }
    __device__ static void load_acts(Acts& a, const ActPtrs& s, int t, int lane, bool ok) {
        FmtQ4K::load_acts(a, s, t, lane, ok);
    }
    template <bool STAGES>
    __device__ static float term(const Row& r, const Acts& a, int t, int lane, bool ok,
                                 const StagePtrs& st, size_t row_units) {
        const int p = lane & 3;
        const uint32_t m4 = 0x0F0F0F0Fu;
        const int wa[4] = {r.qa.x, r.qa.y, r.qa.z, r.qa.w}, wb[4] = {r.qb.x, r.qb.y, r.qb.z, r.qb.w};
        int ip_e = 0, ip_o = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            ip_e = dot4(iq4nl_lookup((uint32_t)wa[k] & m4), a.xa[k], ip_e);
            ip_e = dot4(iq4nl_lookup(((uint32_t)wa[k] >> 4) & m4), a.xa[4 + k], ip_e);
            ip_o = dot4(iq4nl_lookup((uint32_t)wb[k] & m4), a.xa[8 + k], ip_o);
            ip_o = dot4(iq4nl_lookup(((uint32_t)wb[k] >> 4) & m4), a.xa[12 + k], ip_o);
        }
        // sub-blocks 2 p, 2 p + 1: nibbles 2 p, 2 p + 1 of scales_l, bits 4 p .. 4 p + 3 of scales_h
        const uint32_t lo = (uint32_t)r.hdr.y >> (8 * p), hi = (uint32_t)r.hdr.x >> (16 + 4 * p);
        const int ls_e = (int)((lo & 15u) | ((hi & 3u) << 4)) - 32;
        const int ls_o = (int)(((lo >> 4) & 15u) | (((hi >> 2) & 3u) << 4)) - 32;
        // |ip| <= 32 * 127 * 127: the 24-bit multiplies are exact
        const int isum = quad_sum(__mul24(ls_e, ip_e) + __mul24(ls_o, ip_o));
        if (STAGES && ok && p == 0) st.a[row_units + t * 16 + (lane >> 2)] = isum;
        // sumf += d * q8.d[b] * isum as f32
        return f16_bits_to_f32((uint32_t)r.hdr.x & 0xFFFFu) * a.dact * (float)isum;
    }
};

template <Nib32 K>
struct FmtNib32 {
    static constexpr bool kAffine = K == Nib32::Q4_1 || K == Nib32::Q5_1;
    static constexpr bool kFive = K == Nib32::Q5_0 || K == Nib32::Q5_1;
    static constexpr int kElemsPerStep = 2048;
    static constexpr bool kPer32 = true;
    static constexpr bool kOrdered = false;
    static constexpr int kBlockBytes = 18 + (kAffine ? 2 : 0) + (kFive ? 4 : 0), kBlockElems = 32;
    static constexpr int kWide16Steps = 4;
    static constexpr bool kClampedLoads = false;
    static constexpr bool kLaneSums = true;
    // long rows load a whole row ahead where that measured faster (Q4_1 +5 %, Q5_1 +1 %; the
    // 18-byte-block kinds and every other format are as fast or faster one step ahead)
    static constexpr bool kRowAhead = K == Nib32::Q4_1 || K == Nib32::Q5_1;
    struct Row {
        v4i qs;
        uint32_t dm;  // f16 d in the low half, f16 m (affine formats) in the high half
        uint32_t qh;
    };
    struct Acts {
        int xa[8];
        float dact, fbs;
    };
    __device__ static int units(int in_f) { return in_f / 32; }
    __device__ static bool valid(int t, int lane, int n) { return t * 64 + lane < n; }
    __device__ static void load_row(Row& r, const uint8_t* rowp, int t, int lane, bool ok) {
        if (!ok) {
            r.qs = v4i{0, 0, 0, 0};
            r.dm = 0;
            r.qh = 0;
            return;
        }
        const uint8_t* blk = rowp + (size_t)(t * 64 + lane) * kBlockBytes;
        if (kAffine) {
            // [d m][qh][qs x4]: every field on a dword
            r.dm = (uint32_t)load_u32(blk);
            r.qh = kFive ? (uint32_t)load_u32(blk + 4) : 0u;
            r.qs = load16_a4(blk + (kFive ? 8 : 4));
        } else {
            // [d][qh?][qs x4] with the payload 2 bytes past the block start: dwords from the
            // boundary at or below the block; an odd block (2 past a boundary) reads the 2 bytes
            // before it, an even one stops at its own last 2 bytes.
            const bool odd = (reinterpret_cast<uintptr_t>(blk) & 2) != 0;
            const uint8_t* a = blk - (odd ? 2 : 0);
            const uint32_t sel = realign2_selector(odd);
            constexpr int kWords = kFive ? 5 : 4;  // payload dwords after the scale
            int w[kWords + 1];
            const v4i lo = load16_a4(a);
            w[0] = lo.x; w[1] = lo.y; w[2] = lo.z; w[3] = lo.w;
            if (kFive) w[4] = load_u32(a + 16);
            uint32_t tail = load_u16(a + 4 * kWords);
            if (odd) tail |= load_u16(a + 4 * kWords + 2) << 16;
            w[kWords] = (int)tail;
            r.dm = odd ? (uint32_t)w[0] >> 16 : (uint32_t)w[0] & 0xFFFFu;
            int pay[kWords];
#pragma unroll
            for (int k = 0; k < kWords; ++k) pay[k] = realign2(w[k], w[k + 1], sel);
            r.qh = kFive ? (uint32_t)pay[0] : 0u;
            r.qs = v4i{pay[kWords - 4], pay[kWords - 3], pay[kWords - 2], pay[kWords - 1]};
        }
    }
    __device__ static void load_acts(Acts& a, const ActPtrs& s, int t, int lane, bool ok) {
        if (ok) {
            const int b = t * 64 + lane;
            const v4i v0 = *reinterpret_cast<const v4i*>(s.qs + (size_t)b * 32);
            const v4i v1 = *reinterpret_cast<const v4i*>(s.qs + (size_t)b * 32 + 16);
            a.xa[0] = v0.x; a.xa[1] = v0.y; a.xa[2] = v0.z; a.xa[3] = v0.w;
            a.xa[4] = v1.x; a.xa[5] = v1.y; a.xa[6] = v1.z; a.xa[7] = v1.w;
            a.dact = s.d[b];
            a.fbs = (float)s.bsums[b];
        } else {
#pragma unroll
            for (int k = 0; k < 8; ++k) a.xa[k] = 0;
            a.dact = 0.0f;
            a.fbs = 0.0f;
        }
    }
    template <bool STAGES>
    __device__ static float term(const Row& r, const Acts& a, int t, int lane, bool ok,
                                 const StagePtrs& st, size_t row_units) {
        const uint32_t m4 = 0x0F0F0F0Fu;
        const int qw[4] = {r.qs.x, r.qs.y, r.qs.z, r.qs.w};
        int ip = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t w = (uint32_t)qw[k];
            uint32_t lo = w & m4, hi = (w >> 4) & m4;
            if (K == Nib32::IQ4_NL) {
                lo = (uint32_t)iq4nl_lookup(lo);
                hi = (uint32_t)iq4nl_lookup(hi);
            }
            if (kFive) {
                lo |= spread4_to_bit4(r.qh >> (4 * k));
                hi |= spread4_to_bit4(r.qh >> (16 + 4 * k));
            }
            ip = dot4((int)lo, a.xa[k], ip);
            ip = dot4((int)hi, a.xa[4 + k], ip);
        }
        if (STAGES && ok) st.a[row_units + t * 64 + lane] = ip;
        const float d = f16_bits_to_f32(r.dm & 0xFFFFu);
        if (kAffine) {
            // sumf += q8.d[b] * (d * iprod as f32 + m * q8.bsum[b] as f32)
            const float mw = f16_bits_to_f32(r.dm >> 16);
            return a.dact * (d * (float)ip + mw * a.fbs);
        }
        if (K == Nib32::IQ4_NL) return d * a.dact * (float)ip;  // d * q8.d[b] * iprod as f32
        // sumf += d * q8.d[b] * (iprod as f32 - OFFSET * q8.bsum[b] as f32), OFFSET = 8 or 16
        return d * a.dact * ((float)ip - (kFive ? 16.0f : 8.0f) * a.fbs);
    }
};
using FmtQ4_0 = FmtNib32<Nib32::Q4_0>;
using FmtQ4_1 = FmtNib32<Nib32::Q4_1>;
using FmtQ5_0 = FmtNib32<Nib32::Q5_0>;
using FmtQ5_1 = FmtNib32<Nib32::Q5_1>;
using FmtIQ4NL = FmtNib32<Nib32::IQ4_NL>;

// ───────────────────────────── MXFP4 / NVFP4: E2M1 codes ─────────────────────────────
// KVALUES_MXFP4 (crates/infr-gguf/src/dequant.rs:405): 0 1 2 3 4 6 8 12 and their negatives - the
// E2M1 values doubled - looked up like IQ4_NL's table.
__device__ __forceinline__ int mxfp4_lookup(uint32_t nib) {
    const uint32_t sel = nib & 0x07070707u;
    const uint32_t lo = __builtin_amdgcn_perm(0x0C080604u, 0x03020100u, sel);  // entries 0..7
    const uint32_t hi = __builtin_amdgcn_perm(0xF4F8FAFCu, 0xFDFEFF00u, sel);  // entries 8..15
    const uint32_t pick = ((nib >> 3) & 0x01010101u) * 0xFFu;                  // 0xFF where nibble >= 8
    return (int)((hi & pick) | (lo & ~pick));
}
// e8m0_to_fp32_half (dequant.rs:411-417): 2^(x - 128), the two lowest codes subnormal.
__device__ __forceinline__ float e8m0_half(uint32_t x) {
    return __builtin_bit_cast(float, x < 2u ? 0x00200000u << x : (x - 1u) << 23);
}
// ue4m3_to_fp32 (dequant.rs:423-435): 4 exponent bits (bias 7), 3 mantissa bits, halved; 0 and 0x7F
// are 0. (8 + man) * 2^(exp - 11) for exp > 0, man * 2^-10 below: both exact.
__device__ __forceinline__ float ue4m3_half(uint32_t x) {
    const uint32_t exp = (x >> 3) & 15u, man = x & 7u;
    const float v = exp ? __builtin_bit_cast(float, ((exp + 119u) << 23) | (man << 20)) : (float)man * 0.0009765625f;
    return (x == 0u || x == 0x7Fu) ? 0.0f : v;
}

// MXFP4 (17-byte block [u8 e][u8 qs[16]], any byte alignment; crates/infr-cpu/src/kernels.rs:6303-6327):
// a lane owns block t * 64 + l against the per-32 activation, sumf += d * q8.d[b] * iprod. The
// block is fetched as the five aligned dwords that hold it - two loads - and shifted into place
// (nothing beyond the dword of the block's last byte is read).
struct FmtMXFP4 {
    static constexpr int kElemsPerStep = 2048;
    static constexpr bool kPer32 = true;
    static constexpr bool kOrdered = false;
    static constexpr int kBlockBytes = 17, kBlockElems = 32;
    static constexpr int kWide16Steps = 4;
    static constexpr bool kClampedLoads = false;
    static constexpr bool kLaneSums = true;
    static constexpr bool kRowAhead = false;
    struct Row {
        v4i qs;
        uint32_t e;
    };
    typedef FmtNib32<Nib32::IQ4_NL>::Acts Acts;
    __device__ static int units(int in_f) { return in_f / 32; }
    __device__ static bool valid(int t, int lane, int n) { return t * 64 + lane < n; }
    __device__ static void load_row(Row& r, const uint8_t* rowp, int t, int lane, bool ok) {
        if (!ok) {
            r.qs = v4i{0, 0, 0, 0};
            r.e = 0;
            return;
        }
        const uint8_t* blk = rowp + (size_t)(t * 64 + lane) * 17;
        // the five aligned words that hold the block: e is byte `off` of the first, the codes start
        // off + 1 bytes in (a whole word further when off == 3)
        const uint32_t off = (uint32_t)(reinterpret_cast<uintptr_t>(blk) & 3);
        const uint8_t* a = blk - off;
        const v4i lo = load16_a4(a);
        const uint32_t w4 = (uint32_t)load_u32(a + 16);
        r.e = ((uint32_t)lo.x >> (8 * off)) & 0xFFu;
        const uint32_t sh = off + 1;  // v_alignbyte_b32 takes the shift modulo 4: 4 selects the next word
        const uint32_t c0 = __builtin_amdgcn_alignbyte((uint32_t)lo.y, (uint32_t)lo.x, sh);
        const uint32_t c1 = __builtin_amdgcn_alignbyte((uint32_t)lo.z, (uint32_t)lo.y, sh);
        const uint32_t c2 = __builtin_amdgcn_alignbyte((uint32_t)lo.w, (uint32_t)lo.z, sh);
        const uint32_t c3 = __builtin_amdgcn_alignbyte(w4, (uint32_t)lo.w, sh);
        const bool whole = off == 3;
        r.qs = v4i{(int)(whole ? (uint32_t)lo.y : c0), (int)(whole ? (uint32_t)lo.z : c1),
                   (int)(whole ? (uint32_t)lo.w : c2), (int)(whole ? w4 : c3)};
    }
    __device__ static void load_acts(Acts& a, const ActPtrs& s, int t, int lane, bool ok) {
        FmtNib32<Nib32::IQ4_NL>::load_acts(a, s, t, lane, ok);
    }
    template <bool STAGES>
    __device__ static float term(const Row& r, const Acts& a, int t, int lane, bool ok,
                                 const StagePtrs& st, size_t row_units) {
        const uint32_t m4 = 0x0F0F0F0Fu;
        const int qw[4] = {r.qs.x, r.qs.y, r.qs.z, r.qs.w};
        int ip = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            ip = dot4(mxfp4_lookup((uint32_t)qw[k] & m4), a.xa[k], ip);
            ip = dot4(mxfp4_lookup(((uint32_t)qw[k] >> 4) & m4), a.xa[4 + k], ip);
        }
        if (STAGES && ok) st.a[row_units + t * 64 + lane] = ip;
        return e8m0_half(r.e) * a.dact * (float)ip;  // d * q8.d[b] * iprod as f32
    }
};

// NVFP4 (36-byte block [u8 d[4]][u8 qs[32]], 64 weights; crates/infr-cpu/src/kernels.rs:6472-6500):
// sub-block s (16 weights, UE4M3 scale d[s]) reads qs[8 s .. 8 s + 7] - low nibbles elements 0..7,
// high nibbles 8..15 - and meets half of activation block 2 b + s / 2:
// sumf += d_s * q8.d[2 b + s / 2] * iprod_s. A lane owns block t * 64 + l (two activation blocks).
struct FmtNVFP4 {
    static constexpr int kElemsPerStep = 4096;
    static constexpr bool kPer32 = true;
    static constexpr bool kOrdered = false;
    static constexpr int kBlockBytes = 36, kBlockElems = 64;
    static constexpr int kWide16Steps = 3;
    static constexpr bool kClampedLoads = false;
    static constexpr bool kLaneSums = true;
    static constexpr bool kRowAhead = false;
    struct Row {
        v4i qa, qb;
        uint32_t d4;
    };
    struct Acts {
        int xa[16];
        float dact0, dact1;
    };
    __device__ static int units(int in_f) { return in_f / 64; }
    __device__ static bool valid(int t, int lane, int n) { return t * 64 + lane < n; }
    __device__ static void load_row(Row& r, const uint8_t* rowp, int t, int lane, bool ok) {
        if (ok) {
            const uint8_t* blk = rowp + (size_t)(t * 64 + lane) * 36;
            r.d4 = (uint32_t)load_u32(blk);
            r.qa = load16_a4(blk + 4);
            r.qb = load16_a4(blk + 20);
        } else {
            r.qa = r.qb = v4i{0, 0, 0, 0};
            r.d4 = 0;
        }
    }
    __device__ static void load_acts(Acts& a, const ActPtrs& s, int t, int lane, bool ok) {
        if (ok) {
            const int b = t * 64 + lane;
            const v4i* xp = reinterpret_cast<const v4i*>(s.qs + (size_t)b * 64);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const v4i v = xp[k];
                a.xa[4 * k + 0] = v.x;
                a.xa[4 * k + 1] = v.y;
                a.xa[4 * k + 2] = v.z;
                a.xa[4 * k + 3] = v.w;
            }
            a.dact0 = s.d[2 * b];
            a.dact1 = s.d[2 * b + 1];
        } else {
#pragma unroll
            for (int k = 0; k < 16; ++k) a.xa[k] = 0;
            a.dact0 = a.dact1 = 0.0f;
        }
    }
    // (no stage outputs: a block has four integers, one per sub-block)
    template <bool STAGES>
    __device__ static float term(const Row& r, const Acts& a, int, int, bool, const StagePtrs&, size_t) {
        const uint32_t m4 = 0x0F0F0F0Fu;
        const int qw[8] = {r.qa.x, r.qa.y, r.qa.z, r.qa.w, r.qb.x, r.qb.y, r.qb.z, r.qb.w};
        float sum = 0.0f;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const uint32_t w0 = (uint32_t)qw[2 * s], w1 = (uint32_t)qw[2 * s + 1];
            int ip = dot4(mxfp4_lookup(w0 & m4), a.xa[4 * s], 0);
            ip = dot4(mxfp4_lookup(w1 & m4), a.xa[4 * s + 1], ip);
            ip = dot4(mxfp4_lookup((w0 >> 4) & m4), a.xa[4 * s + 2], ip);
            ip = dot4(mxfp4_lookup((w1 >> 4) & m4), a.xa[4 * s + 3], ip);
            sum += ue4m3_half((r.d4 >> (8 * s)) & 0xFFu) * (s < 2 ? a.dact0 : a.dact1) * (float)ip;
        }
        return sum;
    }
};

// Pair form of the formats whose block stride is 2 mod 4 (Q4_0 / IQ4_NL 18 B, Q5_0 22 B), for rows
// of whole 64s: two consecutive blocks are 36 / 44 bytes, a whole number of dwords, and every row
// starts on a dword. Lane l owns the pair t*64 + l (64 weights): three dword-aligned loads fetch it
// and only the first block's payload needs realigning (it starts 2 bytes into a dword; the second
// block's starts on one). Fewer, fuller load instructions per byte than the one-block form, whose
// blocks alternate between the two alignments. 64 pairs (4096 weights) per wave step. The two
// blocks' terms are added in block order.
template <Nib32 K>
struct FmtNib32Pair {
    static_assert(K == Nib32::Q4_0 || K == Nib32::IQ4_NL || K == Nib32::Q5_0, "2-mod-4 strides only");
    static constexpr bool kFive = K == Nib32::Q5_0;
    static constexpr int kElemsPerStep = 4096;
    static constexpr bool kPer32 = true;
    static constexpr bool kOrdered = false;
    static constexpr int kOneBlock = kFive ? 22 : 18;
    static constexpr int kBlockBytes = 2 * kOneBlock, kBlockElems = 64;
    static constexpr int kWide16Steps = 3;
    static constexpr bool kClampedLoads = false;
    static constexpr bool kLaneSums = true;
    static constexpr bool kRowAhead = false;
    struct Row {
        v4i q0, q1;
        uint32_t d01;  // f16 d of block 0 in the low half, of block 1 in the high half
        uint32_t qh0, qh1;
    };
    struct Acts {
        int xa[16];
        float da0, da1, fb0, fb1;
    };
    __device__ static int units(int in_f) { return in_f / 64; }
    __device__ static bool valid(int t, int lane, int n) { return t * 64 + lane < n; }
    __device__ static void load_row(Row& r, const uint8_t* rowp, int t, int lane, bool ok) {
        if (!ok) {
            r.q0 = v4i{0, 0, 0, 0};
            r.q1 = v4i{0, 0, 0, 0};
            r.d01 = 0;
            r.qh0 = 0;
            r.qh1 = 0;
            return;
        }
        const uint8_t* p = rowp + (size_t)(t * 64 + lane) * kBlockBytes;
        const uint32_t sel = 0x05040302u;  // bytes 2..5 of a dword pair
        if (!kFive) {
            // dwords 0..8: [d0 | qs0 (16 B, from byte 2)] [.. | d1 (bytes 18,19)] [qs1 (dwords 5..8)]
            const v4i a = load16_a4(p);
            const int w4 = load_u32(p + 16);
            r.q1 = load16_a4(p + 20);
            r.q0 = v4i{realign2(a.x, a.y, sel), realign2(a.y, a.z, sel), realign2(a.z, a.w, sel),
                       realign2(a.w, w4, sel)};
            r.d01 = ((uint32_t)a.x & 0xFFFFu) | ((uint32_t)w4 & 0xFFFF0000u);
            r.qh0 = 0;
            r.qh1 = 0;
        } else {
            // dwords 0..10: d0 | qh0 (bytes 2..5) | qs0 (bytes 6..21) | d1 (22,23) | qh1 (dword 6) |
            // qs1 (dwords 7..10)
            const v4i a = load16_a4(p), b = load16_a4(p + 16);
            const v3i c3 = gload<v3i_a4>(p + 32);
            const int c[3] = {c3.x, c3.y, c3.z};
            r.qh0 = (uint32_t)realign2(a.x, a.y, sel);
            r.q0 = v4i{realign2(a.y, a.z, sel), realign2(a.z, a.w, sel), realign2(a.w, b.x, sel),
                       realign2(b.x, b.y, sel)};
            r.d01 = ((uint32_t)a.x & 0xFFFFu) | ((uint32_t)b.y & 0xFFFF0000u);
            r.qh1 = (uint32_t)b.z;
            r.q1 = v4i{b.w, c[0], c[1], c[2]};
        }
    }
    __device__ static void load_acts(Acts& a, const ActPtrs& s, int t, int lane, bool ok) {
        if (ok) {
            const int u = t * 64 + lane;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const v4i v = *reinterpret_cast<const v4i*>(s.qs + (size_t)u * 64 + 16 * k);
                a.xa[4 * k + 0] = v.x;
                a.xa[4 * k + 1] = v.y;
                a.xa[4 * k + 2] = v.z;
                a.xa[4 * k + 3] = v.w;
            }
            a.da0 = s.d[2 * u];
            a.da1 = s.d[2 * u + 1];
            a.fb0 = (float)s.bsums[2 * u];
            a.fb1 = (float)s.bsums[2 * u + 1];
        } else {
#pragma unroll
            for (int k = 0; k < 16; ++k) a.xa[k] = 0;
            a.da0 = 0.0f;
            a.da1 = 0.0f;
            a.fb0 = 0.0f;
            a.fb1 = 0.0f;
        }
    }
    __device__ static int block_iprod(const v4i& q, uint32_t qh, const int* xa) {
        const uint32_t m4 = 0x0F0F0F0Fu;
        const int qw[4] = {q.x, q.y, q.z, q.w};
        int ip = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t w = (uint32_t)qw[k];
            uint32_t lo = w & m4, hi = (w >> 4) & m4;
            if (K == Nib32::IQ4_NL) {
                lo = (uint32_t)iq4nl_lookup(lo);
                hi = (uint32_t)iq4nl_lookup(hi);
            }
            if (kFive) {
                lo |= spread4_to_bit4(qh >> (4 * k));
                hi |= spread4_to_bit4(qh >> (16 + 4 * k));
            }
            ip = dot4((int)lo, xa[k], ip);
            ip = dot4((int)hi, xa[4 + k], ip);
        }
        return ip;
    }
    template <bool STAGES>
    __device__ static float term(const Row& r, const Acts& a, int t, int lane, bool ok,
                                 const StagePtrs& st, size_t row_units) {
        const int ip0 = block_iprod(r.q0, r.qh0, &a.xa[0]);
        const int ip1 = block_iprod(r.q1, r.qh1, &a.xa[8]);
        if (STAGES && ok) {
            st.a[2 * row_units + 2 * (t * 64 + lane)] = ip0;
            st.a[2 * row_units + 2 * (t * 64 + lane) + 1] = ip1;
        }
        const float d0 = f16_bits_to_f32(r.d01 & 0xFFFFu), d1 = f16_bits_to_f32(r.d01 >> 16);
        if (K == Nib32::IQ4_NL) {
            float s = d0 * a.da0 * (float)ip0;
            s += d1 * a.da1 * (float)ip1;
            return s;
        }
        const float off = kFive ? 16.0f : 8.0f;
        float s = d0 * a.da0 * ((float)ip0 - off * a.fb0);
        s += d1 * a.da1 * ((float)ip1 - off * a.fb1);
        return s;
    }
};
using FmtQ4_0Pair = FmtNib32Pair<Nib32::Q4_0>;
using FmtIQ4NLPair = FmtNib32Pair<Nib32::IQ4_NL>;
using FmtQ5_0Pair = FmtNib32Pair<Nib32::Q5_0>;

}  // namespace infr
