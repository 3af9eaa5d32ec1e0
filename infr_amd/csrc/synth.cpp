// Deterministic synthetic inputs (host only). The reference ships no weight quantizer: it only
// reads GGUF, and its tests synthesize valid blocks (crates/infr-testkit/src/lib.rs:106-123).
// These encoders turn N(0, sigma^2) draws into valid blocks of every format the kernels take, so that
// benchmarks and parity tests on any machine see byte-identical weights. Any valid encoder works
// for parity: CPU oracle and GPU consume the same bytes.
//
// Generator: SplitMix64 keyed per weight row (seed, row) -> Box-Muller pairs, so the bytes do not
// depend on how rows are split over threads.
#include "../../include/infr_hip.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <thread>
#include <vector>

namespace {

struct SplitMix64 {
    uint64_t s;
    explicit SplitMix64(uint64_t seed) : s(seed) {}
    uint64_t next() {
        uint64_t z = (s += 0x9E3779B97F4A7C15ull);
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
    }
    // uniform in (0, 1]
    double unit() { return ((double)(next() >> 11) + 1.0) * (1.0 / 9007199254740992.0); }
};

struct Normal {
    SplitMix64 rng;
    bool have = false;
    double spare = 0.0;
    explicit Normal(uint64_t seed) : rng(seed) {}
    double next() {
        if (have) {
            have = false;
            return spare;
        }
        const double u1 = rng.unit(), u2 = rng.unit();
        const double r = std::sqrt(-2.0 * std::log(u1));
        const double t = 6.283185307179586476925 * u2;
        spare = r * std::sin(t);
        have = true;
        return r * std::cos(t);
    }
};

uint64_t row_seed(uint64_t seed, uint64_t row) {
    SplitMix64 m(seed * 0xD1342543DE82EF95ull + row + 1);
    return m.next();
}

// IEEE binary16 <-> binary32, round to nearest even (what half::f16::from_f32 does).
uint16_t f32_to_f16(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t exp = (x >> 23) & 0xFFu;
    uint32_t man = x & 0x7FFFFFu;
    if (exp == 0xFF) return (uint16_t)(sign | 0x7C00u | (man ? 0x200u | (man >> 13) : 0));
    const int e = (int)exp - 127 + 15;
    if (e >= 31) return (uint16_t)(sign | 0x7C00u);
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign;
        man |= 0x800000u;
        const int shift = 14 - e;
        uint32_t hm = man >> shift;
        const uint32_t rem = man & ((1u << shift) - 1), half = 1u << (shift - 1);
        if (rem > half || (rem == half && (hm & 1))) hm++;
        return (uint16_t)(sign | hm);
    }
    uint16_t h = (uint16_t)(sign | ((uint32_t)e << 10) | (man >> 13));
    const uint32_t rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1))) h++;
    return h;
}

float f16_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu, bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {
            int shift = 0;
            while (!(man & 0x400u)) {
                man <<= 1;
                shift++;
            }
            bits = sign | ((uint32_t)(113 - shift) << 23) | ((man & 0x3FFu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112) << 23) | (man << 13);
    }
    float f;
    std::memcpy(&f, &bits, 4);
    return f;
}

void put_f16(uint8_t* p, float v) {
    const uint16_t h = f32_to_f16(v);
    p[0] = (uint8_t)(h & 0xFF);
    p[1] = (uint8_t)(h >> 8);
}

int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

// 256 floats -> one 144-byte Q4_K block. Per 32-weight sub-block an affine 4-bit grid
// [min(0, min x), max x]; sub-block scales and mins quantized to 6 bits against f16 super scales.
void encode_q4k(const float* x, uint8_t* blk) {
    float scale[8], minv[8];
    float max_scale = 0.0f, max_min = 0.0f;
    for (int s = 0; s < 8; ++s) {
        float lo = 0.0f, hi = 0.0f;
        for (int l = 0; l < 32; ++l) {
            lo = std::min(lo, x[s * 32 + l]);
            hi = std::max(hi, x[s * 32 + l]);
        }
        scale[s] = (hi - lo) / 15.0f;
        minv[s] = -lo;
        max_scale = std::max(max_scale, scale[s]);
        max_min = std::max(max_min, minv[s]);
    }
    put_f16(blk, max_scale / 63.0f);
    put_f16(blk + 2, max_min / 63.0f);
    const float d = f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
    const float dmin = f16_to_f32((uint16_t)(blk[2] | (blk[3] << 8)));
    int sc[8], mn[8];
    for (int s = 0; s < 8; ++s) {
        sc[s] = d > 0.0f ? clampi((int)std::lround(scale[s] / d), 0, 63) : 0;
        mn[s] = dmin > 0.0f ? clampi((int)std::lround(minv[s] / dmin), 0, 63) : 0;
    }
    uint8_t* scales = blk + 4;
    std::memset(scales, 0, 12);
    for (int j = 0; j < 8; ++j) {
        if (j < 4) {
            scales[j] |= (uint8_t)sc[j];
            scales[j + 4] |= (uint8_t)mn[j];
        } else {
            scales[j + 4] = (uint8_t)((sc[j] & 0xF) | ((mn[j] & 0xF) << 4));
            scales[j - 4] |= (uint8_t)((sc[j] >> 4) << 6);
            scales[j] |= (uint8_t)((mn[j] >> 4) << 6);
        }
    }
    uint8_t* qs = blk + 16;
    for (int s = 0; s < 8; ++s) {
        const float ws = d * (float)sc[s], wm = dmin * (float)mn[s];
        for (int l = 0; l < 32; ++l) {
            const int q = ws > 0.0f ? clampi((int)std::lround((x[s * 32 + l] + wm) / ws), 0, 15) : 0;
            uint8_t& b = qs[(s / 2) * 32 + l];
            b = (s & 1) ? (uint8_t)((b & 0x0F) | (q << 4)) : (uint8_t)((b & 0xF0) | q);
        }
    }
}

// 256 floats -> one 210-byte Q6_K block: per 16-weight group a symmetric 6-bit grid, int8 group
// scales against one f16 super scale.
void encode_q6k(const float* x, uint8_t* blk) {
    float gscale[16], max_scale = 0.0f;
    for (int g = 0; g < 16; ++g) {
        float amax = 0.0f;
        for (int i = 0; i < 16; ++i) amax = std::max(amax, std::fabs(x[g * 16 + i]));
        gscale[g] = amax / 31.0f;
        max_scale = std::max(max_scale, gscale[g]);
    }
    put_f16(blk + 208, max_scale / 127.0f);
    const float d = f16_to_f32((uint16_t)(blk[208] | (blk[209] << 8)));
    int codes[256];
    int8_t* sc = reinterpret_cast<int8_t*>(blk + 192);
    for (int g = 0; g < 16; ++g) {
        const int s = d > 0.0f ? clampi((int)std::lround(gscale[g] / d), 1, 127) : 0;
        sc[g] = (int8_t)s;
        const float ws = d * (float)s;
        for (int i = 0; i < 16; ++i)
            codes[g * 16 + i] =
                ws > 0.0f ? clampi((int)std::lround(x[g * 16 + i] / ws), -32, 31) + 32 : 32;
    }
    uint8_t* ql = blk;
    uint8_t* qh = blk + 128;
    std::memset(blk, 0, 192);
    for (int half = 0; half < 2; ++half)
        for (int l = 0; l < 32; ++l) {
            const int base = half * 128;
            const int q1 = codes[base + l], q2 = codes[base + l + 32];
            const int q3 = codes[base + l + 64], q4 = codes[base + l + 96];
            ql[half * 64 + l] = (uint8_t)((q1 & 0xF) | ((q3 & 0xF) << 4));
            ql[half * 64 + l + 32] = (uint8_t)((q2 & 0xF) | ((q4 & 0xF) << 4));
            qh[half * 32 + l] =
                (uint8_t)((q1 >> 4) | ((q2 >> 4) << 2) | ((q3 >> 4) << 4) | ((q4 >> 4) << 6));
        }
}

// 32 floats -> one 34-byte Q8_0 block.
void encode_q8_0(const float* x, uint8_t* blk) {
    float amax = 0.0f;
    for (int i = 0; i < 32; ++i) amax = std::max(amax, std::fabs(x[i]));
    put_f16(blk, amax / 127.0f);
    const float d = f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
    for (int i = 0; i < 32; ++i)
        blk[2 + i] = (uint8_t)(int8_t)(d > 0.0f ? clampi((int)std::lround(x[i] / d), -127, 127) : 0);
}

// 256 floats -> one 176-byte Q5_K block: Q4_K's construction on a 5-bit grid; the 5th code bit
// of sub-block s goes to bit s of qh[l].
void encode_q5k(const float* x, uint8_t* blk) {
    float scale[8], minv[8];
    float max_scale = 0.0f, max_min = 0.0f;
    for (int s = 0; s < 8; ++s) {
        float lo = 0.0f, hi = 0.0f;
        for (int l = 0; l < 32; ++l) {
            lo = std::min(lo, x[s * 32 + l]);
            hi = std::max(hi, x[s * 32 + l]);
        }
        scale[s] = (hi - lo) / 31.0f;
        minv[s] = -lo;
        max_scale = std::max(max_scale, scale[s]);
        max_min = std::max(max_min, minv[s]);
    }
    put_f16(blk, max_scale / 63.0f);
    put_f16(blk + 2, max_min / 63.0f);
    const float d = f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
    const float dmin = f16_to_f32((uint16_t)(blk[2] | (blk[3] << 8)));
    int sc[8], mn[8];
    for (int s = 0; s < 8; ++s) {
        sc[s] = d > 0.0f ? clampi((int)std::lround(scale[s] / d), 0, 63) : 0;
        mn[s] = dmin > 0.0f ? clampi((int)std::lround(minv[s] / dmin), 0, 63) : 0;
    }
    uint8_t* scales = blk + 4;
    std::memset(scales, 0, 12);
    for (int j = 0; j < 8; ++j) {
        if (j < 4) {
            scales[j] |= (uint8_t)sc[j];
            scales[j + 4] |= (uint8_t)mn[j];
        } else {
            scales[j + 4] = (uint8_t)((sc[j] & 0xF) | ((mn[j] & 0xF) << 4));
            scales[j - 4] |= (uint8_t)((sc[j] >> 4) << 6);
            scales[j] |= (uint8_t)((mn[j] >> 4) << 6);
        }
    }
    uint8_t* qh = blk + 16;
    uint8_t* qs = blk + 48;
    std::memset(qh, 0, 32 + 128);
    for (int s = 0; s < 8; ++s) {
        const float ws = d * (float)sc[s], wm = dmin * (float)mn[s];
        for (int l = 0; l < 32; ++l) {
            const int q = ws > 0.0f ? clampi((int)std::lround((x[s * 32 + l] + wm) / ws), 0, 31) : 0;
            qs[(s / 2) * 32 + l] |= (uint8_t)((q & 0xF) << ((s & 1) * 4));
            qh[l] |= (uint8_t)((q >> 4) << s);
        }
    }
}

// 256 floats -> one 84-byte Q2_K block (scales[16] | qs[64] | d | dmin): per 16-weight sub-block an
// affine 2-bit grid [min(0, min x), max x]; 4-bit sub-block scales (low nibble) and mins (high
// nibble) against f16 super scales. Sub-block s = 8n + 2j + h holds elements 16s..16s+15; their
// codes sit at bit 2j of qs[32n + 16h ..] (crates/infr-gguf/src/dequant.rs, Q2_K).
void encode_q2k(const float* x, uint8_t* blk) {
    float scale[16], minv[16];
    float max_scale = 0.0f, max_min = 0.0f;
    for (int s = 0; s < 16; ++s) {
        float lo = 0.0f, hi = 0.0f;
        for (int l = 0; l < 16; ++l) {
            lo = std::min(lo, x[s * 16 + l]);
            hi = std::max(hi, x[s * 16 + l]);
        }
        scale[s] = (hi - lo) / 3.0f;
        minv[s] = -lo;
        max_scale = std::max(max_scale, scale[s]);
        max_min = std::max(max_min, minv[s]);
    }
    put_f16(blk + 80, max_scale / 15.0f);
    put_f16(blk + 82, max_min / 15.0f);
    const float d = f16_to_f32((uint16_t)(blk[80] | (blk[81] << 8)));
    const float dmin = f16_to_f32((uint16_t)(blk[82] | (blk[83] << 8)));
    std::memset(blk + 16, 0, 64);
    for (int s = 0; s < 16; ++s) {
        const int sc = d > 0.0f ? clampi((int)std::lround(scale[s] / d), 0, 15) : 0;
        const int mn = dmin > 0.0f ? clampi((int)std::lround(minv[s] / dmin), 0, 15) : 0;
        blk[s] = (uint8_t)(sc | (mn << 4));
        const float ws = d * (float)sc, wm = dmin * (float)mn;
        const int n = s / 8, j = (s % 8) / 2, h = s & 1;
        for (int l = 0; l < 16; ++l) {
            const int q = ws > 0.0f ? clampi((int)std::lround((x[s * 16 + l] + wm) / ws), 0, 3) : 0;
            blk[16 + 32 * n + 16 * h + l] |= (uint8_t)(q << (2 * j));
        }
    }
}

// 256 floats -> one 110-byte Q3_K block (hmask[32] | qs[64] | scales[12] | d): per 16-weight
// sub-block a 3-bit grid (code - 4) whose signed scale puts the element of largest magnitude on
// code 0 (= -4), so sub-block scales take both signs; stored as 6-bit fields with a bias of 32
// against one f16 super scale. Codes: low two bits as in Q2_K, the third in bit 4n + j of
// hmask[16h + l]. Scale field i (group g = i / 4, byte k = i % 4): low nibble in the low (g < 2) or
// high nibble of scales[4 (g & 1) + k], top two bits at bit 2g of scales[8 + k].
void encode_q3k(const float* x, uint8_t* blk) {
    float scale[16], max_scale = 0.0f;
    for (int s = 0; s < 16; ++s) {
        float peak = 0.0f;
        for (int l = 0; l < 16; ++l)
            if (std::fabs(x[s * 16 + l]) > std::fabs(peak)) peak = x[s * 16 + l];
        scale[s] = -peak / 4.0f;
        max_scale = std::max(max_scale, std::fabs(scale[s]));
    }
    put_f16(blk + 108, max_scale / 31.0f);
    const float d = f16_to_f32((uint16_t)(blk[108] | (blk[109] << 8)));
    std::memset(blk, 0, 108);
    for (int s = 0; s < 16; ++s) {
        const int sc = d > 0.0f ? clampi((int)std::lround(scale[s] / d), -31, 31) : 0;
        const int field = sc + 32, g = s / 4, k = s % 4;
        blk[96 + 4 * (g & 1) + k] |= (uint8_t)((field & 0xF) << (g < 2 ? 0 : 4));
        blk[96 + 8 + k] |= (uint8_t)((field >> 4) << (2 * g));
        const float ws = d * (float)sc;
        const int n = s / 8, j = (s % 8) / 2, h = s & 1;
        for (int l = 0; l < 16; ++l) {
            const int c = ws != 0.0f ? clampi((int)std::lround(x[s * 16 + l] / ws) + 4, 0, 7) : 4;
            blk[32 + 32 * n + 16 * h + l] |= (uint8_t)((c & 3) << (2 * j));
            blk[16 * h + l] |= (uint8_t)((c >> 2) << (4 * n + j));
        }
    }
}

// The 16-entry codebook of IQ4_NL (crates/infr-gguf/src/dequant.rs:439-441).
const int kIq4nl[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};

// 256 floats -> one 136-byte IQ4_XS block (d | scales_h | scales_l[4] | qs[128]): per 32-weight
// sub-block the table value nearest to x / (d * (ls - 32)). A sub-block's scale is signed so that
// its element of largest magnitude lands on the table's end value -127; ls - 32 in -31..31 against
// one f16 super scale.
void encode_iq4xs(const float* x, uint8_t* blk) {
    float scale[8], max_scale = 0.0f;
    for (int s = 0; s < 8; ++s) {
        float peak = 0.0f;
        for (int l = 0; l < 32; ++l)
            if (std::fabs(x[s * 32 + l]) > std::fabs(peak)) peak = x[s * 32 + l];
        scale[s] = -peak / 127.0f;
        max_scale = std::max(max_scale, std::fabs(scale[s]));
    }
    put_f16(blk, max_scale / 31.0f);
    const float d = f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
    std::memset(blk + 2, 0, 134);
    uint32_t scales_h = 0;
    for (int s = 0; s < 8; ++s) {
        int sc = d > 0.0f ? clampi((int)std::lround(scale[s] / d), -31, 31) : 0;
        if (sc == 0) sc = scale[s] < 0.0f ? -1 : 1;
        const int ls = sc + 32;
        blk[4 + s / 2] |= (uint8_t)((ls & 0xF) << (4 * (s & 1)));
        scales_h |= (uint32_t)(ls >> 4) << (2 * s);
        const float ws = d * (float)sc;
        for (int l = 0; l < 32; ++l) {
            const float v = ws != 0.0f ? x[s * 32 + l] / ws : 0.0f;
            int best = 0;
            for (int c = 1; c < 16; ++c)
                if (std::fabs(v - (float)kIq4nl[c]) < std::fabs(v - (float)kIq4nl[best])) best = c;
            blk[8 + 16 * s + (l & 15)] |= (uint8_t)(best << (4 * (l >> 4)));
        }
    }
    blk[2] = (uint8_t)(scales_h & 0xFF);
    blk[3] = (uint8_t)(scales_h >> 8);
}

// The E2M1 values, doubled (crates/infr-gguf/src/dequant.rs:405).
const int kFp4[16] = {0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12};
int nearest_fp4(float v) {
    int best = 0;
    for (int c = 1; c < 16; ++c)
        if (c != 8 && std::fabs(v - (float)kFp4[c]) < std::fabs(v - (float)kFp4[best])) best = c;
    return best;
}
// 32 floats -> one 17-byte MXFP4 block [u8 e][u8 qs[16]]: the smallest power of two d = 2^(e - 128)
// with 12 d >= max |x|, codes the nearest table values of x / d.
void encode_mxfp4(const float* x, uint8_t* blk) {
    float amax = 0.0f;
    for (int i = 0; i < 32; ++i) amax = std::max(amax, std::fabs(x[i]));
    int e = amax > 0.0f ? (int)std::ceil(std::log2(amax / 12.0f)) + 128 : 2;
    e = clampi(e, 2, 254);
    const float d = std::ldexp(1.0f, e - 128);
    blk[0] = (uint8_t)e;
    for (int j = 0; j < 16; ++j)
        blk[1 + j] = (uint8_t)(nearest_fp4(x[j] / d) | (nearest_fp4(x[j + 16] / d) << 4));
}
// 64 floats -> one 36-byte NVFP4 block [u8 d[4]][u8 qs[32]]: per 16-weight sub-block the UE4M3 code
// (exponent bias 7, three mantissa bits, decoded halved) whose value is the smallest one with
// 12 d >= max |x|; codes the nearest table values of x / d, low nibbles elements 0..7, high 8..15.
void encode_nvfp4(const float* x, uint8_t* blk) {
    for (int s = 0; s < 4; ++s) {
        float amax = 0.0f;
        for (int i = 0; i < 16; ++i) amax = std::max(amax, std::fabs(x[16 * s + i]));
        int code = 0x7E;
        float d = 0.0f;
        for (int c = 1; c <= 0x7E; ++c) {  // values ascend with the code
            const int ex = c >> 3, man = c & 7;
            const float v = 0.5f * (ex == 0 ? (float)man / 8.0f * std::ldexp(1.0f, -6) : (1.0f + (float)man / 8.0f) * std::ldexp(1.0f, ex - 7));
            if (12.0f * v >= amax) {
                code = c;
                d = v;
                break;
            }
            d = v;
        }
        blk[s] = (uint8_t)code;
        for (int j = 0; j < 8; ++j)
            blk[4 + 8 * s + j] = (uint8_t)(nearest_fp4(x[16 * s + j] / d) | (nearest_fp4(x[16 * s + 8 + j] / d) << 4));
    }
}

// 32 floats -> one block of a 32-weight format. Element j's code goes to the low nibble of qs[j],
// element j+16's to the high nibble; the 5-bit formats put the 5th bit of element e in bit e of qh.
//   Q4_0 [d][qs]: symmetric, code = round(x/d) + 8        Q5_0 [d][qh][qs]: ... + 16
//   Q4_1 [d][m][qs]: affine on [min x, max x]             Q5_1 [d][m][qh][qs]
//   IQ4_NL [d][qs]: nearest codebook value of x/d
void encode_blk32(int dtype, const float* x, uint8_t* blk) {
    const bool affine = dtype == INFR_DTYPE_Q4_1 || dtype == INFR_DTYPE_Q5_1;
    const bool five = dtype == INFR_DTYPE_Q5_0 || dtype == INFR_DTYPE_Q5_1;
    const int levels = five ? 32 : 16;
    float lo = x[0], hi = x[0], amax = 0.0f;
    for (int i = 0; i < 32; ++i) {
        lo = std::min(lo, x[i]);
        hi = std::max(hi, x[i]);
        amax = std::max(amax, std::fabs(x[i]));
    }
    int code[32];
    uint8_t* p = blk + 2;
    if (affine) {
        put_f16(blk, (hi - lo) / (float)(levels - 1));
        put_f16(blk + 2, lo);
        const float d = f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
        const float m = f16_to_f32((uint16_t)(blk[2] | (blk[3] << 8)));
        for (int i = 0; i < 32; ++i)
            code[i] = d > 0.0f ? clampi((int)std::lround((x[i] - m) / d), 0, levels - 1) : 0;
        p = blk + 4;
    } else if (dtype == INFR_DTYPE_IQ4_NL) {
        put_f16(blk, amax / 127.0f);
        const float d = f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
        for (int i = 0; i < 32; ++i) {
            const float v = d > 0.0f ? x[i] / d : 0.0f;
            int best = 0;
            for (int c = 1; c < 16; ++c)
                if (std::fabs(v - (float)kIq4nl[c]) < std::fabs(v - (float)kIq4nl[best])) best = c;
            code[i] = best;
        }
    } else {
        put_f16(blk, amax / (float)(levels / 2 - 1));
        const float d = f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
        for (int i = 0; i < 32; ++i)
            code[i] = (d > 0.0f ? clampi((int)std::lround(x[i] / d), -(levels / 2), levels / 2 - 1) : 0) + levels / 2;
    }
    if (five) {
        uint32_t qh = 0;
        for (int i = 0; i < 32; ++i) qh |= (uint32_t)(code[i] >> 4) << i;
        std::memcpy(p, &qh, 4);
        p += 4;
    }
    for (int j = 0; j < 16; ++j) p[j] = (uint8_t)((code[j] & 0xF) | ((code[j + 16] & 0xF) << 4));
}

template <typename F>
void parallel_rows(size_t rows, F&& fn) {
    unsigned nt = std::thread::hardware_concurrency();
    if (nt == 0) nt = 1;
    nt = (unsigned)std::min<size_t>(nt, std::max<size_t>(1, rows / 8));
    nt = std::min(nt, 16u);
    if (nt <= 1) {
        for (size_t r = 0; r < rows; ++r) fn(r);
        return;
    }
    std::vector<std::thread> th;
    for (unsigned t = 0; t < nt; ++t)
        th.emplace_back([=, &fn] {
            for (size_t r = t; r < rows; r += nt) fn(r);
        });
    for (auto& t : th) t.join();
}

}  // namespace

extern "C" {

int infr_block_layout(int dtype, int* elems, int* bytes) {
    int e, b;
    switch (dtype) {
    case INFR_DTYPE_F32: e = 1; b = 4; break;
    case INFR_DTYPE_F16: e = 1; b = 2; break;
    case INFR_DTYPE_BF16: e = 1; b = 2; break;
    case INFR_DTYPE_Q8_0: e = 32; b = 34; break;
    case INFR_DTYPE_Q4_K: e = 256; b = 144; break;
    case INFR_DTYPE_Q6_K: e = 256; b = 210; break;
    case INFR_DTYPE_Q2_0: e = 64; b = 18; break;
    case INFR_DTYPE_Q4_0: e = 32; b = 18; break;
    case INFR_DTYPE_Q4_1: e = 32; b = 20; break;
    case INFR_DTYPE_Q5_0: e = 32; b = 22; break;
    case INFR_DTYPE_Q5_1: e = 32; b = 24; break;
    case INFR_DTYPE_Q5_K: e = 256; b = 176; break;
    case INFR_DTYPE_Q2_K: e = 256; b = 84; break;
    case INFR_DTYPE_Q3_K: e = 256; b = 110; break;
    case INFR_DTYPE_IQ4_XS: e = 256; b = 136; break;
    case INFR_DTYPE_TQ1_0: e = 256; b = 54; break;
    case INFR_DTYPE_TQ2_0: e = 256; b = 66; break;
    case INFR_DTYPE_MXFP4: e = 32; b = 17; break;
    case INFR_DTYPE_NVFP4: e = 64; b = 36; break;
    case INFR_DTYPE_IQ4_NL: e = 32; b = 18; break;
    default: return 0;
    }
    if (elems) *elems = e;
    if (bytes) *bytes = b;
    return 1;
}

void infr_synth_normal_f32(uint64_t seed, float mean, float sigma, size_t n, float* out) {
    // Keyed per 4096-value chunk so large buffers can be filled in parallel deterministically.
    const size_t chunk = 4096, chunks = (n + chunk - 1) / chunk;
    parallel_rows(chunks, [&](size_t c) {
        Normal g(row_seed(seed, c));
        const size_t end = std::min(n, (c + 1) * chunk);
        for (size_t i = c * chunk; i < end; ++i) out[i] = mean + sigma * (float)g.next();
    });
}

size_t infr_synth_weight(int dtype, uint64_t seed, float sigma, size_t rows, size_t in_f,
                         uint8_t* out) {
    int qpb, bpb;
    if (!out || !infr_block_layout(dtype, &qpb, &bpb) || qpb == 1) return 0;
    if (in_f == 0 || in_f % (size_t)qpb != 0) return 0;
    const size_t bpr = in_f / (size_t)qpb * (size_t)bpb;
    parallel_rows(rows, [&](size_t r) {
        uint8_t* row = out + r * bpr;
        Normal g(row_seed(seed, r));
        if (dtype == INFR_DTYPE_Q2_0) {
            // codes i.i.d. uniform over {0,1,2} (= -1, 0, +1; code 3 unused), scale |N(0, sigma^2)|
            for (size_t b = 0; b < in_f / 64; ++b) {
                uint8_t* blk = row + b * 18;
                put_f16(blk, std::fabs(sigma * (float)g.next()));
                for (int i = 0; i < 16; ++i) {
                    uint8_t byte = 0;
                    for (int k = 0; k < 4; ++k) byte |= (uint8_t)((g.rng.next() % 3) << (2 * k));
                    blk[2 + i] = byte;
                }
            }
            return;
        }
        if (dtype == INFR_DTYPE_TQ1_0) {
            // digits i.i.d. uniform over {0,1,2}, five to a byte as ceil(v * 256 / 243) with the first digit
            // most significant (qh: four digits and a zero), scale |N(0, sigma^2)| per block
            for (size_t b = 0; b < in_f / 256; ++b) {
                uint8_t* blk = row + b * 54;
                put_f16(blk + 52, std::fabs(sigma * (float)g.next()));
                for (int i = 0; i < 52; ++i) {
                    uint32_t v = 0;
                    for (int k = 0; k < 5; ++k) v = v * 3 + (k == 4 && i >= 48 ? 0u : (uint32_t)(g.rng.next() % 3));
                    blk[i] = (uint8_t)((v * 256 + 242) / 243);
                }
            }
            return;
        }
        if (dtype == INFR_DTYPE_TQ2_0) {
            // as Q2_0: codes i.i.d. uniform over {0,1,2} (= -1, 0, +1), scale |N(0, sigma^2)| per block
            for (size_t b = 0; b < in_f / 256; ++b) {
                uint8_t* blk = row + b * 66;
                put_f16(blk + 64, std::fabs(sigma * (float)g.next()));
                for (int i = 0; i < 64; ++i) {
                    uint8_t byte = 0;
                    for (int k = 0; k < 4; ++k) byte |= (uint8_t)((g.rng.next() % 3) << (2 * k));
                    blk[i] = byte;
                }
            }
            return;
        }
        std::vector<float> x((size_t)qpb);
        for (size_t b = 0; b < in_f / (size_t)qpb; ++b) {
            for (int i = 0; i < qpb; ++i) x[(size_t)i] = sigma * (float)g.next();
            uint8_t* blk = row + b * (size_t)bpb;
            if (dtype == INFR_DTYPE_Q4_K) encode_q4k(x.data(), blk);
            else if (dtype == INFR_DTYPE_Q5_K) encode_q5k(x.data(), blk);
            else if (dtype == INFR_DTYPE_Q6_K) encode_q6k(x.data(), blk);
            else if (dtype == INFR_DTYPE_Q2_K) encode_q2k(x.data(), blk);
            else if (dtype == INFR_DTYPE_Q3_K) encode_q3k(x.data(), blk);
            else if (dtype == INFR_DTYPE_IQ4_XS) encode_iq4xs(x.data(), blk);
            else if (dtype == INFR_DTYPE_MXFP4) encode_mxfp4(x.data(), blk);
            else if (dtype == INFR_DTYPE_NVFP4) encode_nvfp4(x.data(), blk);
            else if (dtype == INFR_DTYPE_Q8_0) encode_q8_0(x.data(), blk);
            else encode_blk32(dtype, x.data(), blk);
        }
    });
    return rows * bpr;
}

}  // extern "C"
