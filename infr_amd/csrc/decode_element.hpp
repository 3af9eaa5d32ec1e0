// One element of a weight row in its GGUF block format, decoded with the host decode's arithmetic
// (crates/infr-gguf/src/dequant.rs:11-51: `sc * code + mn` with sc and mn each rounded to f32 first;
// codebook formats d * value), so the value equals `bytes_to_f32(row)[e]` bit for bit. Used where
// infr-cpu itself decodes to f32: Op::EmbedGather and the `ActsKind::Raw` arm of Op::MoeFfn.
#pragma once

#include "device_common.hpp"

namespace infr {

__device__ __forceinline__ uint32_t ld8(const uint8_t* p) { return gload<uint8_t>(p); }
__device__ __forceinline__ float ldf16(const uint8_t* p) { return f16_bits_to_f32(gload<uint16_t>(p)); }

// get_scale_min_k4 for one sub-block (crates/infr-gguf/src/dequant.rs:73-83)
__device__ __forceinline__ void k4_one(int j, const uint8_t* q, int* sc, int* m) {
    if (j < 4) {
        *sc = (int)(ld8(q + j) & 63);
        *m = (int)(ld8(q + j + 4) & 63);
    } else {
        *sc = (int)((ld8(q + j + 4) & 0xF) | ((ld8(q + j - 4) >> 6) << 4));
        *m = (int)((ld8(q + j + 4) >> 4) | ((ld8(q + j) >> 6) << 4));
    }
}

// Element e of a row stored in `dtype` (ggml type id); rowp is the row's first byte.
__device__ inline float decode_element(int dtype, const uint8_t* rowp, int e) {
    switch (dtype) {
    case 0: return gload<float>(rowp + (size_t)e * 4);
    case 1: return ldf16(rowp + (size_t)e * 2);
    case 30: return __builtin_bit_cast(float, (uint32_t)gload<uint16_t>(rowp + (size_t)e * 2) << 16);
    case 8: {  // Q8_0: (d*1) * (q+128) + d*(-128)
        const uint8_t* blk = rowp + (size_t)(e >> 5) * 34;
        const float d = ldf16(blk);
        const int q = (int)(int8_t)ld8(blk + 2 + (e & 31));
        return (d * 1.0f) * (float)(q + 128) + d * -128.0f;
    }
    case 2: case 3: case 6: case 7: {  // Q4_0, Q4_1, Q5_0, Q5_1
        const bool affine = dtype == 3 || dtype == 7, five = dtype == 6 || dtype == 7;
        const int bytes = 18 + (affine ? 2 : 0) + (five ? 4 : 0);
        const uint8_t* blk = rowp + (size_t)(e >> 5) * bytes;
        const int i = e & 31, j = i & 15;
        const float d = ldf16(blk);
        const uint8_t* p = blk + (affine ? 4 : 2);
        uint32_t code_hi = 0;
        if (five) {
            const uint32_t qh = ld8(p) | (ld8(p + 1) << 8) | (ld8(p + 2) << 16) | (ld8(p + 3) << 24);
            code_hi = ((qh >> i) & 1u) << 4;
            p += 4;
        }
        const uint32_t b = ld8(p + j);
        const uint32_t code = (i < 16 ? (b & 0xF) : (b >> 4)) | code_hi;
        const float mn = affine ? ldf16(blk + 2) * 1.0f : d * (five ? -16.0f : -8.0f);
        return (d * 1.0f) * (float)code + mn;
    }
    case 12: case 13: {  // Q4_K, Q5_K
        const int bytes = dtype == 12 ? 144 : 176;
        const uint8_t* blk = rowp + (size_t)(e >> 8) * bytes;
        const int i = e & 255, s = i >> 5, l = i & 31;
        int sc, m;
        k4_one(s, blk + 4, &sc, &m);
        const uint8_t* qs = blk + (dtype == 12 ? 16 : 48);
        const uint32_t b = ld8(qs + (s >> 1) * 32 + l);
        uint32_t code = (s & 1) ? (b >> 4) : (b & 0xF);
        if (dtype == 13) code += ((ld8(blk + 16 + l) >> s) & 1u) ? 16u : 0u;
        const float fs = ldf16(blk) * (float)sc, fm = ldf16(blk + 2) * (float)(-m);
        return fs * (float)code + fm;
    }
    case 10: {  // Q2_K: (d * scale) * code + dmin * (-min), sub-block i / 16 (dequant.rs:220-247)
        const uint8_t* blk = rowp + (size_t)(e >> 8) * 84;
        const int i = e & 255, n = i >> 7, j = (i >> 5) & 3, half = (i >> 4) & 1, l = i & 15;
        const uint32_t sb = ld8(blk + (i >> 4));
        const uint32_t code = (ld8(blk + 16 + 32 * n + 16 * half + l) >> (2 * j)) & 3u;
        return (ldf16(blk + 80) * (float)(int)(sb & 15u)) * (float)code + ldf16(blk + 82) * (float)(-(int)(sb >> 4));
    }
    case 11: {  // Q3_K: (d * s) * code + d * (-4 s), s = sc6 - 32 (dequant.rs:248-298)
        const uint8_t* blk = rowp + (size_t)(e >> 8) * 110;
        const int i = e & 255, n = i >> 7, j = (i >> 5) & 3, half = (i >> 4) & 1, l = i & 15, is = i >> 4;
        const uint32_t low2 = (ld8(blk + 32 + 32 * n + 16 * half + l) >> (2 * j)) & 3u;
        const uint32_t high = (ld8(blk + 16 * half + l) >> (4 * n + j)) & 1u;
        const uint32_t lo4 = (ld8(blk + 96 + (is & 7)) >> (4 * (is >> 3))) & 15u;
        const uint32_t hi2 = (ld8(blk + 104 + (is & 3)) >> (2 * (is >> 2))) & 3u;
        const int s = (int)(lo4 | (hi2 << 4)) - 32;
        const float d = ldf16(blk + 108);
        return (d * (float)s) * (float)(low2 | (high << 2)) + d * (float)(-4 * s);
    }
    case 23: {  // IQ4_XS: (d * (ls - 32)) * table[nibble] (dequant.rs:517-550)
        const uint8_t* blk = rowp + (size_t)(e >> 8) * 136;
        const int i = e & 255, ib = i >> 5, j = i & 15;
        const uint32_t sh = ld8(blk + 2) | (ld8(blk + 3) << 8);
        const int ls = (int)(((ld8(blk + 4 + (ib >> 1)) >> (4 * (ib & 1))) & 15u) | (((sh >> (2 * ib)) & 3u) << 4)) - 32;
        const uint32_t nib = (ld8(blk + 8 + 16 * ib + j) >> (4 * ((i >> 4) & 1))) & 15u;
        const int kv[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
        return (ldf16(blk) * (float)ls) * (float)kv[nib];
    }
    case 34: {  // TQ1_0: (digit - 1) * d, digit n of a byte = high byte of 3 * (byte * 3^n mod 256) (dequant.rs:922-967)
        const uint8_t* blk = rowp + (size_t)(e >> 8) * 54;
        const int i = e & 255;
        int n, at;
        if (i < 160) { n = i >> 5; at = i & 31; }
        else if (i < 240) { n = (i - 160) >> 4; at = 32 + ((i - 160) & 15); }
        else { n = (i - 240) >> 2; at = 48 + ((i - 240) & 3); }
        uint32_t q = ld8(blk + at);
        for (int k = 0; k < n; ++k) q = (q * 3u) & 0xFFu;
        return (float)((int)((q * 3u) >> 8) - 1) * ldf16(blk + 52);
    }
    case 35: {  // TQ2_0: (q - 1) * d (dequant.rs:968-996)
        const uint8_t* blk = rowp + (size_t)(e >> 8) * 66;
        const int i = e & 255;
        const int q = (int)((ld8(blk + 32 * (i >> 7) + (i & 31)) >> (2 * ((i >> 5) & 3))) & 3u);
        return (float)(q - 1) * ldf16(blk + 64);
    }
    case 39: {  // MXFP4: table[nibble] * 2^(e - 128) (dequant.rs:1024-1042)
        const int kv[16] = {0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12};
        const uint8_t* blk = rowp + (size_t)(e >> 5) * 17;
        const int i = e & 31;
        const uint32_t x = ld8(blk), b = ld8(blk + 1 + (i & 15));
        const float d = __builtin_bit_cast(float, x < 2u ? 0x00200000u << x : (x - 1u) << 23);
        return (float)kv[i < 16 ? (b & 0xF) : (b >> 4)] * d;
    }
    case 40: {  // NVFP4: table[nibble] * ue4m3(d[sub-block]) (dequant.rs:1050-1072, 423-435)
        const int kv[16] = {0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12};
        const uint8_t* blk = rowp + (size_t)(e >> 6) * 36;
        const int i = e & 63, sb = i >> 4, j = i & 7;
        const uint32_t x = ld8(blk + sb), b = ld8(blk + 4 + 8 * sb + j);
        const uint32_t exp = (x >> 3) & 15u, man = x & 7u;
        float d = exp ? __builtin_bit_cast(float, ((exp + 119u) << 23) | (man << 20)) : (float)man * 0.0009765625f;
        if (x == 0u || x == 0x7Fu) d = 0.0f;
        return (float)kv[(i & 8) ? (b >> 4) : (b & 0xF)] * d;
    }
    case 14: {  // Q6_K
        const uint8_t* blk = rowp + (size_t)(e >> 8) * 210;
        const int i = e & 255, half = i >> 7, r = i & 127, col = r >> 5, l = r & 31;
        const uint32_t lb = ld8(blk + half * 64 + (col & 1) * 32 + l);
        const uint32_t lo = col >= 2 ? (lb >> 4) : (lb & 0xF);
        const uint32_t hi = (ld8(blk + 128 + half * 32 + l) >> (2 * col)) & 3u;
        const int s = (int)(int8_t)ld8(blk + 192 + half * 8 + 2 * col + (l >> 4));
        const float d = ldf16(blk + 208);
        return (d * (float)s) * (float)(lo | (hi << 4)) + d * (float)(-32 * s);
    }
    case 20: {  // IQ4_NL
        const int kv[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
        const uint8_t* blk = rowp + (size_t)(e >> 5) * 18;
        const int i = e & 31;
        const uint32_t b = ld8(blk + 2 + (i & 15));
        return ldf16(blk) * (float)kv[i < 16 ? (b & 0xF) : (b >> 4)];
    }
    case 42: {  // Q2_0
        const uint8_t* blk = rowp + (size_t)(e >> 6) * 18;
        const int j = e & 63;
        const int q = (int)((ld8(blk + 2 + (j >> 2)) >> ((j & 3) * 2)) & 3u);
        return (float)(q - 1) * ldf16(blk);
    }
    default: return 0.0f;
    }
}

}  // namespace infr
