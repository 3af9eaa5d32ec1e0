/*
 * CPU oracle: plain-C restatement of infr-cpu's quantized Op::Linear / Op::MoeFfn path.
 * TEST INFRASTRUCTURE ONLY — see infr_cpu_oracle.h for scope, citations and pinning status.
 * Build: gcc -O2 -ffp-contract=off -fno-fast-math -fopenmp (see Makefile).
 */
#include "infr_cpu_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ───────────────────────────── block geometry ───────────────────────────── */

/* crates/infr-core/src/decode_spec.rs:305-358: Q4_0 (32,18), Q4_1 (32,20), Q5_0 (32,22),
 * Q5_1 (32,24), Q8_0 (32,34), Q4K (256,144), Q5K (256,176), Q6K (256,210), IQ4_NL (32,18),
 * Q2_0 (64,18). */
int orc_block_layout(int dtype, int *elems, int *bytes) {
    int e = 0, b = 0;
    switch (dtype) {
    case ORC_F32: e = 1; b = 4; break;
    case ORC_F16: e = 1; b = 2; break;
    case ORC_BF16: e = 1; b = 2; break;
    case ORC_Q4_0: e = 32; b = 18; break;
    case ORC_Q4_1: e = 32; b = 20; break;
    case ORC_Q5_0: e = 32; b = 22; break;
    case ORC_Q5_1: e = 32; b = 24; break;
    case ORC_IQ4_NL: e = 32; b = 18; break;
    case ORC_Q8_0: e = 32; b = 34; break;
    case ORC_Q5_K: e = 256; b = 176; break;
    case ORC_Q2_K: e = 256; b = 84; break;
    case ORC_Q3_K: e = 256; b = 110; break;
    case ORC_IQ4_XS: e = 256; b = 136; break;
    case ORC_TQ1_0: e = 256; b = 54; break;
    case ORC_TQ2_0: e = 256; b = 66; break;
    case ORC_MXFP4: e = 32; b = 17; break;
    case ORC_NVFP4: e = 64; b = 36; break;
    case ORC_Q4_K: e = 256; b = 144; break;
    case ORC_Q6_K: e = 256; b = 210; break;
    case ORC_Q2_0: e = 64; b = 18; break;
    default: return 0;
    }
    if (elems) *elems = e;
    if (bytes) *bytes = b;
    return 1;
}

/* ───────────────────────────── f16 ───────────────────────────── */

/* half::f16::to_f32 — exact widening, subnormals included. */
float orc_f16_bits_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {
            /* subnormal: value = man * 2^-24; normalise */
            int shift = 0;
            while ((man & 0x400u) == 0) {
                man <<= 1;
                shift++;
            }
            man &= 0x3FFu;
            bits = sign | ((uint32_t)(127 - 15 - shift + 1) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + (127 - 15)) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

float orc_rdf16(const uint8_t *b) {
    return orc_f16_bits_to_f32((uint16_t)(b[0] | ((uint16_t)b[1] << 8)));
}

/* half::f16::from_f32 — round to nearest even, overflow to inf, gradual underflow. */
uint16_t orc_f32_to_f16_bits(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t exp = (x >> 23) & 0xFFu;
    uint32_t man = x & 0x7FFFFFu;
    if (exp == 0xFF) { /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | (man ? (0x200u | (man >> 13)) : 0));
    }
    int e = (int)exp - 127 + 15;
    if (e >= 31) return (uint16_t)(sign | 0x7C00u); /* overflow -> inf */
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign; /* underflows to zero even after rounding */
        man |= 0x800000u;                   /* implicit one */
        int shift = 14 - e;                 /* 14..24 */
        uint32_t half_man = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half_man & 1))) half_man++;
        return (uint16_t)(sign | half_man); /* may carry into the exponent: correct */
    }
    uint32_t half_man = man >> 13;
    uint32_t rem = man & 0x1FFFu;
    uint16_t h = (uint16_t)(sign | ((uint32_t)e << 10) | half_man);
    if (rem > 0x1000u || (rem == 0x1000u && (half_man & 1))) h++; /* carry may reach inf: correct */
    return h;
}

/* ───────────────────────────── k4 ───────────────────────────── */

/* crates/infr-gguf/src/dequant.rs:73-83 (llama.cpp get_scale_min_k4). */
void orc_k4(int j, const uint8_t *q, uint32_t *sc, uint32_t *m) {
    if (j < 4) {
        *sc = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *sc = (uint32_t)((q[j + 4] & 0x0F) | ((q[j - 4] >> 6) << 4));
        *m = (uint32_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

/* ───────────────────────────── host decode ───────────────────────────── */

/* crates/infr-gguf/src/dequant.rs:439-441 */
/* crates/infr-gguf/src/dequant.rs:405 (KVALUES_MXFP4: the E2M1 values, doubled). */
const int8_t orc_kvalues_mxfp4[16] = {0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12};

/* crates/infr-gguf/src/dequant.rs:411-417 (e8m0_to_fp32_half): 2^(x - 128); the two lowest codes
 * are f32 subnormals. */
float orc_e8m0_half(uint8_t x) {
    uint32_t bits = x < 2 ? (0x00200000u << x) : (((uint32_t)x - 1u) << 23);
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* crates/infr-gguf/src/dequant.rs:423-435 (ue4m3_to_fp32): unsigned, 4 exponent bits (bias 7), 3
 * mantissa bits, halved; 0 and 0x7F decode to 0. */
float orc_ue4m3_half(uint8_t x) {
    if (x == 0 || x == 0x7F) return 0.0f;
    int exp = (x >> 3) & 0xF;
    float man = (float)(x & 0x7);
    float raw = exp == 0 ? man * ldexpf(1.0f, -9) : (1.0f + man / 8.0f) * ldexpf(1.0f, exp - 7);
    return raw * 0.5f;
}

const int8_t orc_kvalues_iq4nl[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};

/* crates/infr-gguf/src/dequant.rs:11-51: for affine quants the factored form is expanded as
 *   sc = f32(d) * (f32)scm_sc;  mn = f32(dmin) * (f32)scm_m;  out = sc * (f32)code + mn
 * (separate multiply and add). Factored arms: Q8_0 :209-219, Q4K :311-331, Q6K :361-385.
 * Q2_0 is a codebook quant: (q-1) as f32 * d (:998-1018). */
int orc_dequant_block(int dtype, const uint8_t *bytes, size_t nbytes, float *out) {
    int qpb, bpb;
    if (!orc_block_layout(dtype, &qpb, &bpb)) return -1;
    size_t nblk = nbytes / (size_t)bpb;
    switch (dtype) {
    case ORC_F32:
        memcpy(out, bytes, nblk * 4);
        return 0;
    case ORC_F16:
        for (size_t i = 0; i < nblk; i++) out[i] = orc_rdf16(bytes + 2 * i);
        return 0;
    case ORC_BF16: /* dequant.rs:19-22: the 16 bits are the top half of the f32 */
        for (size_t i = 0; i < nblk; i++) {
            uint32_t u = ((uint32_t)bytes[2 * i] | ((uint32_t)bytes[2 * i + 1] << 8)) << 16;
            memcpy(&out[i], &u, 4);
        }
        return 0;
    case ORC_Q8_0:
        for (size_t b = 0; b < nblk; b++) {
            const uint8_t *blk = bytes + b * 34;
            float d = orc_rdf16(blk);
            /* scm = (1, -128) for both 16-groups; code = q + 128 */
            float sc = d * (float)1;
            float mn = d * (float)(-128);
            for (int i = 0; i < 32; i++) {
                uint8_t code = (uint8_t)((int16_t)(int8_t)blk[2 + i] + 128);
                out[b * 32 + i] = sc * (float)code + mn;
            }
        }
        return 0;
    case ORC_Q4_K:
        for (size_t b = 0; b < nblk; b++) {
            const uint8_t *blk = bytes + b * 144;
            float d = orc_rdf16(blk);
            float dmin = orc_rdf16(blk + 2);
            const uint8_t *scales = blk + 4;
            const uint8_t *qs = blk + 16;
            float *o = out + b * 256;
            for (int j = 0; j < 4; j++) {
                uint32_t sc1, m1, sc2, m2;
                orc_k4(2 * j, scales, &sc1, &m1);
                orc_k4(2 * j + 1, scales, &sc2, &m2);
                float fs1 = d * (float)(int16_t)sc1, fm1 = dmin * (float)(int16_t)(-(int16_t)m1);
                float fs2 = d * (float)(int16_t)sc2, fm2 = dmin * (float)(int16_t)(-(int16_t)m2);
                for (int l = 0; l < 32; l++) {
                    uint8_t v = qs[j * 32 + l];
                    o[j * 64 + l] = fs1 * (float)(v & 0xF) + fm1;
                    o[j * 64 + 32 + l] = fs2 * (float)(v >> 4) + fm2;
                }
            }
        }
        return 0;
    case ORC_Q6_K:
        for (size_t b = 0; b < nblk; b++) {
            const uint8_t *blk = bytes + b * 210;
            const uint8_t *ql = blk, *qh = blk + 128, *scales = blk + 192;
            float d = orc_rdf16(blk + 208);
            float *o = out + b * 256;
            for (int half = 0; half < 2; half++) {
                int qlo = half * 64, qho = half * 32, sco = half * 8, base = half * 128;
                for (int l = 0; l < 32; l++) {
                    int is = l / 16;
                    uint8_t c[4];
                    c[0] = (uint8_t)((ql[qlo + l] & 0xF) | ((qh[qho + l] & 3) << 4));
                    c[1] = (uint8_t)((ql[qlo + l + 32] & 0xF) | (((qh[qho + l] >> 2) & 3) << 4));
                    c[2] = (uint8_t)((ql[qlo + l] >> 4) | (((qh[qho + l] >> 4) & 3) << 4));
                    c[3] = (uint8_t)((ql[qlo + l + 32] >> 4) | (((qh[qho + l] >> 6) & 3) << 4));
                    for (int k = 0; k < 4; k++) {
                        int16_t s = (int16_t)(int8_t)scales[sco + is + 2 * k];
                        float sc = d * (float)s;
                        float mn = d * (float)(int16_t)(-32 * s);
                        o[base + l + 32 * k] = sc * (float)c[k] + mn;
                    }
                }
            }
        }
        return 0;
    case ORC_Q4_0:
    case ORC_Q4_1:
    case ORC_Q5_0:
    case ORC_Q5_1:
        /* dequant.rs:141-207: (scale, min) multipliers (1,-8) on (d,d) for Q4_0, (1,1) on (d,m) for
         * Q4_1, (1,-16) on (d,d) for Q5_0, (1,1) on (d,m) for Q5_1; the 5th code bit of element j
         * is qh bit j, of element j+16 qh bit j+16. */
        for (size_t b = 0; b < nblk; b++) {
            const uint8_t *blk = bytes + b * (size_t)bpb;
            int affine = dtype == ORC_Q4_1 || dtype == ORC_Q5_1;
            int five = dtype == ORC_Q5_0 || dtype == ORC_Q5_1;
            float d = orc_rdf16(blk);
            float dm = affine ? orc_rdf16(blk + 2) : d;
            const uint8_t *p = blk + (affine ? 4 : 2);
            uint32_t qh = 0;
            if (five) {
                qh = (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
                p += 4;
            }
            float sc = d * (float)1;
            float mn = dm * (float)(affine ? 1 : (five ? -16 : -8));
            for (int j = 0; j < 16; j++) {
                uint32_t xh0 = five ? ((qh >> j) << 4) & 0x10 : 0;
                uint32_t xh1 = five ? (qh >> (j + 12)) & 0x10 : 0;
                uint8_t c0 = (uint8_t)(((uint32_t)p[j] & 0x0F) | xh0);
                uint8_t c1 = (uint8_t)(((uint32_t)p[j] >> 4) | xh1);
                out[b * 32 + j] = sc * (float)c0 + mn;
                out[b * 32 + j + 16] = sc * (float)c1 + mn;
            }
        }
        return 0;
    case ORC_Q5_K:
        /* dequant.rs:332-358: Q4_K's layout with a 5th code bit from qh[32] (bit 2j for the even
         * sub-block of pair j, bit 2j+1 for the odd one). */
        for (size_t b = 0; b < nblk; b++) {
            const uint8_t *blk = bytes + b * 176;
            float d = orc_rdf16(blk);
            float dmin = orc_rdf16(blk + 2);
            const uint8_t *scales = blk + 4, *qh = blk + 16, *qs = blk + 48;
            float *o = out + b * 256;
            for (int j = 0; j < 4; j++) {
                uint32_t sc1, m1, sc2, m2;
                orc_k4(2 * j, scales, &sc1, &m1);
                orc_k4(2 * j + 1, scales, &sc2, &m2);
                float fs1 = d * (float)(int16_t)sc1, fm1 = dmin * (float)(int16_t)(-(int16_t)m1);
                float fs2 = d * (float)(int16_t)sc2, fm2 = dmin * (float)(int16_t)(-(int16_t)m2);
                for (int l = 0; l < 32; l++) {
                    uint8_t v = qs[j * 32 + l];
                    uint8_t c1 = (uint8_t)((v & 0xF) + ((qh[l] >> (2 * j)) & 1 ? 16 : 0));
                    uint8_t c2 = (uint8_t)((v >> 4) + ((qh[l] >> (2 * j + 1)) & 1 ? 16 : 0));
                    o[j * 64 + l] = fs1 * (float)c1 + fm1;
                    o[j * 64 + 32 + l] = fs2 * (float)c2 + fm2;
                }
            }
        }
        return 0;
    case ORC_Q2_K:
        /* dequant.rs:220-247: [u8 scales[16]][u8 qs[64]][f16 d][f16 dmin]; sub-block `is` (16
         * elements, output order) = 8n + 2j + half reads qs[32n + 16half + l] >> 2j; its scale byte
         * holds the 4-bit scale (low) and the 4-bit min (high). y = (d*scale)*code + dmin*(-min). */
        for (size_t b = 0; b < nblk; b++) {
            const uint8_t *blk = bytes + b * 84;
            const uint8_t *scales = blk, *qs = blk + 16;
            float d = orc_rdf16(blk + 80), dmin = orc_rdf16(blk + 82);
            float *o = out + b * 256;
            int is = 0;
            for (int n = 0; n < 2; n++)
                for (int j = 0; j < 4; j++)
                    for (int half = 0; half < 2; half++, is++) {
                        float fs = d * (float)(int16_t)(scales[is] & 0xF);
                        float fm = dmin * (float)(int16_t)(-(int16_t)(scales[is] >> 4));
                        for (int l = 0; l < 16; l++) {
                            uint8_t c = (uint8_t)((qs[32 * n + 16 * half + l] >> (2 * j)) & 3);
                            o[is * 16 + l] = fs * (float)c + fm;
                        }
                    }
        }
        return 0;
    case ORC_Q3_K:
        /* dequant.rs:248-298: [u8 hmask[32]][u8 qs[64]][u8 scales[12]][f16 d]; the code's low two
         * bits are laid out as Q2_K's, its third bit is bit 4n + j of hmask[16half + l]; scale
         * s = sc6 - 32 per 16 elements, min -4s, both against d: y = (d*s)*code + d*(-4s). */
        for (size_t b = 0; b < nblk; b++) {
            const uint8_t *blk = bytes + b * 110;
            const uint8_t *hmask = blk, *qs = blk + 32;
            int16_t sc[16];
            orc_q3k_scales(blk + 96, sc);
            float d = orc_rdf16(blk + 108);
            float *o = out + b * 256;
            int is = 0;
            for (int n = 0; n < 2; n++)
                for (int j = 0; j < 4; j++)
                    for (int half = 0; half < 2; half++, is++) {
                        float fs = d * (float)sc[is];
                        float fm = d * (float)(int16_t)(-4 * sc[is]);
                        for (int l = 0; l < 16; l++) {
                            uint8_t low2 = (uint8_t)((qs[32 * n + 16 * half + l] >> (2 * j)) & 3);
                            uint8_t high = (uint8_t)((hmask[16 * half + l] >> (4 * n + j)) & 1);
                            o[is * 16 + l] = fs * (float)(uint8_t)(low2 | (high << 2)) + fm;
                        }
                    }
        }
        return 0;
    case ORC_IQ4_NL:
        /* dequant.rs:495-512: pure codebook, d * KVALUES_IQ4NL[nibble]. */
        for (size_t b = 0; b < nblk; b++) {
            const uint8_t *blk = bytes + b * 18;
            float d = orc_rdf16(blk);
            for (int j = 0; j < 16; j++) {
                out[b * 32 + j] = d * (float)orc_kvalues_iq4nl[blk[2 + j] & 0xF];
                out[b * 32 + j + 16] = d * (float)orc_kvalues_iq4nl[blk[2 + j] >> 4];
            }
        }
        return 0;
    case ORC_IQ4_XS:
        /* dequant.rs:517-550: [f16 d][u16 scales_h][u8 scales_l[4]][u8 qs[128]]; eight sub-blocks of
         * 32, ls = nibble ib of scales_l | two bits of scales_h << 4; y = (d * (ls - 32)) * codebook,
         * low nibble of qs[16 ib + j] -> element 32 ib + j, high nibble -> 32 ib + j + 16. */
        for (size_t b = 0; b < nblk; b++) {
            const uint8_t *blk = bytes + b * 136;
            float d = orc_rdf16(blk);
            uint32_t scales_h = (uint32_t)blk[2] | ((uint32_t)blk[3] << 8);
            for (int ib = 0; ib < 8; ib++) {
                float dl = d * (float)orc_iq4xs_scale(scales_h, blk + 4, ib);
                const uint8_t *qs = blk + 8 + 16 * ib;
                for (int j = 0; j < 16; j++) {
                    out[b * 256 + ib * 32 + j] = dl * (float)orc_kvalues_iq4nl[qs[j] & 0xF];
                    out[b * 256 + ib * 32 + j + 16] = dl * (float)orc_kvalues_iq4nl[qs[j] >> 4];
                }
            }
        }
        return 0;
    case ORC_TQ1_0:
        /* dequant.rs:922-967: [u8 qs[48]][u8 qh[4]][f16 d]; y = (digit - 1) * d in three runs:
         * qs[0..32) x 5 digits -> elements 32 n + m, qs[32..48) x 5 -> 160 + 16 n + m,
         * qh[0..4) x 4 -> 240 + 4 n + j. */
        for (size_t b = 0; b < nblk; b++) {
            const uint8_t *blk = bytes + b * 54;
            float d = orc_rdf16(blk + 52);
            for (int i = 0; i < 256; i++) out[b * 256 + i] = (float)(orc_tq1_0_digit(blk, i) - 1) * d;
        }
        return 0;
    case ORC_TQ2_0:
        /* dequant.rs:968-996: [u8 qs[64]][f16 d]; element 128 chunk + 32 l + m reads bit pair l of
         * qs[32 chunk + m]; y = (q - 1) * d. */
        for (size_t b = 0; b < nblk; b++) {
            const uint8_t *blk = bytes + b * 66;
            float d = orc_rdf16(blk + 64);
            for (int chunk = 0; chunk < 2; chunk++)
                for (int l = 0; l < 4; l++)
                    for (int mm = 0; mm < 32; mm++) {
                        int q = (blk[32 * chunk + mm] >> (2 * l)) & 3;
                        out[b * 256 + chunk * 128 + l * 32 + mm] = (float)(q - 1) * d;
                    }
        }
        return 0;
    case ORC_MXFP4:
        /* dequant.rs:1024-1042: [u8 e][u8 qs[16]]; y[j] = table[low nibble] * d, y[j + 16] = table[high] * d. */
        for (size_t b = 0; b < nblk; b++) {
            const uint8_t *blk = bytes + b * 17;
            float d = orc_e8m0_half(blk[0]);
            for (int j = 0; j < 16; j++) {
                out[b * 32 + j] = (float)orc_kvalues_mxfp4[blk[1 + j] & 0xF] * d;
                out[b * 32 + j + 16] = (float)orc_kvalues_mxfp4[blk[1 + j] >> 4] * d;
            }
        }
        return 0;
    case ORC_NVFP4:
        /* dequant.rs:1050-1072: [u8 d[4]][u8 qs[32]]; sub-block s (16 elements) reads qs[8s .. 8s + 7]:
         * low nibbles elements 0..7, high nibbles 8..15, each times the sub-block's UE4M3 scale. */
        for (size_t b = 0; b < nblk; b++) {
            const uint8_t *blk = bytes + b * 36;
            for (int sb = 0; sb < 4; sb++) {
                float d = orc_ue4m3_half(blk[sb]);
                for (int j = 0; j < 8; j++) {
                    out[b * 64 + sb * 16 + j] = (float)orc_kvalues_mxfp4[blk[4 + sb * 8 + j] & 0xF] * d;
                    out[b * 64 + sb * 16 + j + 8] = (float)orc_kvalues_mxfp4[blk[4 + sb * 8 + j] >> 4] * d;
                }
            }
        }
        return 0;
    case ORC_Q2_0:
        for (size_t b = 0; b < nblk; b++) {
            const uint8_t *blk = bytes + b * 18;
            float d = orc_rdf16(blk);
            const uint8_t *qs = blk + 2;
            for (int j = 0; j < 64; j++) {
                int q = (qs[j / 4] >> ((j % 4) * 2)) & 3;
                out[b * 64 + j] = (float)(q - 1) * d;
            }
        }
        return 0;
    default:
        return -1;
    }
}

/* ───────────────────────────── activation quantizers ───────────────────────────── */

static inline int8_t quant_one(float v, float id) {
    /* (v * id).round().clamp(-127.0, 127.0) as i8 — Rust f32::round is half away from zero */
    float r = roundf(v * id);
    if (r < -127.0f) r = -127.0f;
    if (r > 127.0f) r = 127.0f;
    return (int8_t)r;
}

/* crates/infr-cpu/src/quant.rs:27-58 */
void orc_quantize_q8(const float *x, size_t len, int8_t *qs, float *d, int32_t *bsums,
                     int32_t *bsums16) {
    size_t nb = len / 256;
    for (size_t b = 0; b < nb; b++) {
        const float *blk = x + b * 256;
        float amax = 0.0f;
        for (int i = 0; i < 256; i++) {
            float a = fabsf(blk[i]);
            amax = a > amax ? a : amax; /* f32::max fold from 0 */
        }
        float dd = amax / 127.0f;
        float id = dd > 0.0f ? 1.0f / dd : 0.0f;
        d[b] = dd;
        for (int i = 0; i < 256; i++) qs[b * 256 + i] = quant_one(blk[i], id);
    }
    for (size_t b = 0; b < nb; b++) {
        int32_t s16[16];
        for (int s = 0; s < 16; s++) {
            int32_t acc = 0;
            for (int i = 0; i < 16; i++) acc += qs[b * 256 + s * 16 + i];
            s16[s] = acc;
            if (bsums16) bsums16[b * 16 + s] = acc;
        }
        for (int s = 0; s < 8; s++) bsums[b * 8 + s] = s16[2 * s] + s16[2 * s + 1];
    }
}

/* crates/infr-cpu/src/quant.rs:97-117 */
void orc_quantize_q8_32(const float *x, size_t len, int8_t *qs, float *d, int32_t *bsum) {
    size_t nb = len / 32;
    for (size_t b = 0; b < nb; b++) {
        const float *blk = x + b * 32;
        float amax = 0.0f;
        for (int i = 0; i < 32; i++) {
            float a = fabsf(blk[i]);
            amax = a > amax ? a : amax;
        }
        float dd = amax / 127.0f;
        float id = dd > 0.0f ? 1.0f / dd : 0.0f;
        d[b] = dd;
        int32_t s = 0;
        for (int i = 0; i < 32; i++) {
            int8_t q = quant_one(blk[i], id);
            qs[b * 32 + i] = q;
            s += q;
        }
        bsum[b] = s;
    }
}

/* ───────────────────────────── scalar dot kernels ───────────────────────────── */

/* crates/infr-cpu/src/kernels.rs:151-184 (vec_dot_q4k_scalar); the batch scalar (:1458-1509)
 * evaluates the same expression in the same order per activation row. */
float orc_vec_dot_q4k(const uint8_t *row, const int8_t *qs8, const float *d8, const int32_t *bsums,
                      size_t in_f, int32_t *sd_out, int32_t *sm_out) {
    size_t nb = in_f / 256;
    float sumf = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * 144;
        float d = orc_rdf16(blk);
        float dmin = orc_rdf16(blk + 2);
        const uint8_t *scales = blk + 4;
        const uint8_t *qs = blk + 16;
        const int8_t *q8b = qs8 + b * 256;
        int32_t sd = 0, sm = 0;
        for (int s = 0; s < 8; s++) {
            uint32_t sc, m;
            orc_k4(s, scales, &sc, &m);
            int half = s / 2, hi = (s % 2) == 1;
            const uint8_t *qbyte = qs + half * 32;
            const int8_t *q8s = q8b + s * 32;
            int32_t iprod = 0;
            for (int l = 0; l < 32; l++) {
                int32_t q4 = hi ? (qbyte[l] >> 4) : (qbyte[l] & 0xF);
                iprod += q4 * (int32_t)q8s[l];
            }
            int32_t isum = bsums[b * 8 + s];
            sd += (int32_t)sc * iprod;
            sm += (int32_t)m * isum;
        }
        if (sd_out) sd_out[b] = sd;
        if (sm_out) sm_out[b] = sm;
        sumf += d8[b] * (d * (float)sd - dmin * (float)sm);
    }
    return sumf;
}

/* crates/infr-cpu/src/kernels.rs:487-526 (vec_dot_q6k_scalar). */
float orc_vec_dot_q6k(const uint8_t *row, const int8_t *qs8, const float *d8, size_t in_f,
                      int32_t *isum_out) {
    size_t nb = in_f / 256;
    float sumf = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * 210;
        const uint8_t *ql = blk, *qh = blk + 128, *scales = blk + 192;
        float d = orc_rdf16(blk + 208);
        const int8_t *q8b = qs8 + b * 256;
        int32_t sumi[16] = {0}, bsum[16] = {0};
        for (int half = 0; half < 2; half++) {
            int qlo = half * 64, qho = half * 32, sco = half * 8, base = half * 128;
            for (int l = 0; l < 32; l++) {
                int is = l / 16;
                int32_t q[4];
                q[0] = (ql[qlo + l] & 0xF) | ((qh[qho + l] & 3) << 4);
                q[1] = (ql[qlo + l + 32] & 0xF) | (((qh[qho + l] >> 2) & 3) << 4);
                q[2] = (ql[qlo + l] >> 4) | (((qh[qho + l] >> 4) & 3) << 4);
                q[3] = (ql[qlo + l + 32] >> 4) | (((qh[qho + l] >> 6) & 3) << 4);
                for (int k = 0; k < 4; k++) {
                    int sub = sco + is + 2 * k;
                    int32_t v = q8b[base + l + 32 * k];
                    sumi[sub] += q[k] * v;
                    bsum[sub] += v;
                }
            }
        }
        int32_t isum = 0;
        for (int sub = 0; sub < 16; sub++)
            isum += (int32_t)(int8_t)scales[sub] * (sumi[sub] - 32 * bsum[sub]);
        if (isum_out) isum_out[b] = isum;
        sumf += d * d8[b] * (float)isum; /* (d * q8.d[b]) * (isum as f32) */
    }
    return sumf;
}

/* crates/infr-cpu/src/kernels.rs:4972-4991 (vec_dot_q8_0_32_batch_scalar, one activation row):
 * Q8_0 rows whose length is a multiple of 32 but not of 256, against the per-32 activation. */
float orc_vec_dot_q8_0_32(const uint8_t *row, const int8_t *qs, const float *d32, size_t in_f,
                          int32_t *iprod_out) {
    size_t nb = in_f / 32;
    float sumf = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * 34;
        float d_w = orc_rdf16(blk);
        const int8_t *qw = (const int8_t *)(blk + 2);
        int32_t iprod = 0;
        for (int i = 0; i < 32; i++) iprod += (int32_t)qw[i] * (int32_t)qs[b * 32 + i];
        if (iprod_out) iprod_out[b] = iprod;
        sumf += d_w * d32[b] * (float)iprod; /* (d_arr[b] * q8.d[b]) * (iprod as f32) */
    }
    return sumf;
}

/* crates/infr-cpu/src/kernels.rs:1170-1187 (vec_dot_q8_0_scalar): weight blocks of 32 against the
 * per-256 activation scale. */
float orc_vec_dot_q8_0(const uint8_t *row, const int8_t *qs8, const float *d8, size_t in_f,
                       int32_t *iprod_out) {
    size_t nb_super = in_f / 256;
    float sumf = 0.0f;
    for (size_t b = 0; b < nb_super; b++) {
        float dact = d8[b];
        for (int s = 0; s < 8; s++) {
            size_t wb = b * 8 + (size_t)s;
            const uint8_t *blk = row + wb * 34;
            float d_w = orc_rdf16(blk);
            const int8_t *qw = (const int8_t *)(blk + 2);
            const int8_t *qx = qs8 + b * 256 + s * 32;
            int32_t iprod = 0;
            for (int i = 0; i < 32; i++) iprod += (int32_t)qw[i] * (int32_t)qx[i];
            if (iprod_out) iprod_out[wb] = iprod;
            sumf += dact * d_w * (float)iprod; /* (d8 * d_w) * (iprod as f32) */
        }
    }
    return sumf;
}

/* crates/infr-cpu/src/kernels.rs:5641-5668 (vec_dot_q2_0_batch_scalar, one activation row). */
float orc_vec_dot_q2_0(const uint8_t *row, const int8_t *qs8, const float *d8, const int32_t *bsum,
                       size_t in_f, int32_t *iprod_out) {
    size_t nb = in_f / 64;
    float sumf = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * 18;
        const uint8_t *qs = blk + 2;
        float d = orc_rdf16(blk);
        for (int sub = 0; sub < 2; sub++) {
            size_t s = 2 * b + (size_t)sub;
            const int8_t *q8b = qs8 + s * 32;
            int32_t iprod = 0;
            for (int p = 0; p < 32; p++) {
                int j = sub * 32 + p;
                int32_t code = (qs[j / 4] >> ((j % 4) * 2)) & 3;
                iprod += code * (int32_t)q8b[p];
            }
            if (iprod_out) iprod_out[s] = iprod;
            sumf += d * d8[s] * ((float)iprod - (float)bsum[s]);
        }
    }
    return sumf;
}

/* crates/infr-cpu/src/kernels.rs:1286-1327 (vec_dot_q5k_scalar). */
float orc_vec_dot_q5k(const uint8_t *row, const int8_t *qs8, const float *d8, const int32_t *bsums,
                      size_t in_f, int32_t *sd_out, int32_t *sm_out) {
    size_t nb = in_f / 256;
    float sumf = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * 176;
        float d = orc_rdf16(blk);
        float dmin = orc_rdf16(blk + 2);
        const uint8_t *scales = blk + 4, *qh = blk + 16, *ql = blk + 48;
        const int8_t *q8b = qs8 + b * 256;
        int32_t sd = 0, sm = 0;
        uint8_t u1 = 1, u2 = 2;
        for (int j = 0; j < 4; j++) {
            uint32_t sc_e, m_e, sc_o, m_o;
            orc_k4(2 * j, scales, &sc_e, &m_e);
            orc_k4(2 * j + 1, scales, &sc_o, &m_o);
            const int8_t *q8_e = q8b + 2 * j * 32, *q8_o = q8b + (2 * j + 1) * 32;
            int32_t iprod_e = 0, iprod_o = 0;
            for (int l = 0; l < 32; l++) {
                uint8_t v = ql[j * 32 + l];
                int32_t q5_e = (int32_t)(v & 0xF) + ((qh[l] & u1) ? 16 : 0);
                int32_t q5_o = (int32_t)(v >> 4) + ((qh[l] & u2) ? 16 : 0);
                iprod_e += q5_e * (int32_t)q8_e[l];
                iprod_o += q5_o * (int32_t)q8_o[l];
            }
            sd += (int32_t)sc_e * iprod_e + (int32_t)sc_o * iprod_o;
            sm += (int32_t)m_e * bsums[b * 8 + 2 * j] + (int32_t)m_o * bsums[b * 8 + 2 * j + 1];
            u1 = (uint8_t)(u1 << 2);
            u2 = (uint8_t)(u2 << 2);
        }
        if (sd_out) sd_out[b] = sd;
        if (sm_out) sm_out[b] = sm;
        sumf += d8[b] * (d * (float)sd - dmin * (float)sm);
    }
    return sumf;
}

/* crates/infr-cpu/src/kernels.rs:764-783 (q3k_scales): the 12 scale bytes as three little-endian
 * words a0, a1, t; sixteen 6-bit fields = low nibbles of a0, a1, high nibbles of a0, a1, each with
 * two more bits from t (t, t >> 2, t >> 4, t >> 6); minus 32. */
void orc_q3k_scales(const uint8_t *r, int16_t out[16]) {
    uint32_t a0 = (uint32_t)r[0] | ((uint32_t)r[1] << 8) | ((uint32_t)r[2] << 16) | ((uint32_t)r[3] << 24);
    uint32_t a1 = (uint32_t)r[4] | ((uint32_t)r[5] << 8) | ((uint32_t)r[6] << 16) | ((uint32_t)r[7] << 24);
    uint32_t t = (uint32_t)r[8] | ((uint32_t)r[9] << 8) | ((uint32_t)r[10] << 16) | ((uint32_t)r[11] << 24);
    const uint32_t k1 = 0x03030303u, k2 = 0x0f0f0f0fu;
    uint32_t aux[4];
    aux[0] = (a0 & k2) | ((t & k1) << 4);
    aux[1] = (a1 & k2) | (((t >> 2) & k1) << 4);
    aux[2] = ((a0 >> 4) & k2) | (((t >> 4) & k1) << 4);
    aux[3] = ((a1 >> 4) & k2) | (((t >> 6) & k1) << 4);
    for (int i = 0; i < 16; i++)
        out[i] = (int16_t)((int16_t)(int8_t)(uint8_t)((aux[i / 4] >> ((i % 4) * 8)) & 0xFF) - 32);
}

/* crates/infr-cpu/src/kernels.rs:315-361 (vec_dot_q2k_scalar). */
float orc_vec_dot_q2k(const uint8_t *row, const int8_t *qs8, const float *d8, const int32_t *bsums16,
                      size_t in_f, int32_t *sd_out, int32_t *sm_out) {
    size_t nb = in_f / 256;
    float sumf = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * 84;
        const uint8_t *scales = blk, *qs = blk + 16;
        float d = orc_rdf16(blk + 80), dmin = orc_rdf16(blk + 82);
        const int8_t *q8b = qs8 + b * 256;
        int32_t sd = 0, sm = 0;
        int is = 0;
        for (int n = 0; n < 2; n++)
            for (int j = 0; j < 4; j++)
                for (int half = 0; half < 2; half++, is++) {
                    int32_t scale = scales[is] & 0xF, minv = scales[is] >> 4;
                    const uint8_t *qb = qs + 32 * n + 16 * half;
                    int32_t iprod = 0;
                    for (int l = 0; l < 16; l++)
                        iprod += (int32_t)((qb[l] >> (2 * j)) & 3) * (int32_t)q8b[is * 16 + l];
                    sd += scale * iprod;
                    sm += minv * bsums16[b * 16 + is];
                }
        if (sd_out) sd_out[b] = sd;
        if (sm_out) sm_out[b] = sm;
        sumf += d8[b] * (d * (float)sd - dmin * (float)sm);
    }
    return sumf;
}

/* crates/infr-cpu/src/kernels.rs:812-852 (vec_dot_q3k_scalar). */
float orc_vec_dot_q3k(const uint8_t *row, const int8_t *qs8, const float *d8, const int32_t *bsums16,
                      size_t in_f, int32_t *isum_out) {
    size_t nb = in_f / 256;
    float sumf = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * 110;
        const uint8_t *hmask = blk, *qs = blk + 32;
        int16_t sc[16];
        orc_q3k_scales(blk + 96, sc);
        float d = orc_rdf16(blk + 108);
        const int8_t *q8b = qs8 + b * 256;
        int32_t isum = 0;
        int is = 0;
        for (int n = 0; n < 2; n++)
            for (int j = 0; j < 4; j++)
                for (int half = 0; half < 2; half++, is++) {
                    const uint8_t *qb = qs + 32 * n + 16 * half, *hb = hmask + 16 * half;
                    int32_t iprod = 0;
                    for (int l = 0; l < 16; l++) {
                        int32_t low2 = (qb[l] >> (2 * j)) & 3;
                        int32_t high = ((hb[l] >> (4 * n + j)) & 1) ? 4 : 0;
                        iprod += (low2 | high) * (int32_t)q8b[is * 16 + l];
                    }
                    isum += (int32_t)sc[is] * (iprod - 4 * bsums16[b * 16 + is]);
                }
        if (isum_out) isum_out[b] = isum;
        sumf += d * d8[b] * (float)isum;
    }
    return sumf;
}

/* crates/infr-cpu/src/kernels.rs:995-1002 (iq4xs_ls_minus_32): sub-block ib's 6-bit scale, minus 32. */
int orc_iq4xs_scale(uint32_t scales_h, const uint8_t *scales_l, int ib) {
    int lo = (scales_l[ib / 2] >> (4 * (ib % 2))) & 0xF;
    int hi = (int)((scales_h >> (2 * ib)) & 3u);
    return (lo | (hi << 4)) - 32;
}

/* crates/infr-cpu/src/kernels.rs:1008-1036 (vec_dot_iq4xs_scalar): per sub-block of 32 the signed
 * codebook dot with the activation codes, weighted by (ls - 32) in i32; one f32 step per superblock. */
float orc_vec_dot_iq4xs(const uint8_t *row, const int8_t *qs8, const float *d8, size_t in_f, int32_t *isum_out) {
    size_t nb = in_f / 256;
    float sumf = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * 136;
        float d = orc_rdf16(blk);
        uint32_t scales_h = (uint32_t)blk[2] | ((uint32_t)blk[3] << 8);
        const int8_t *q8b = qs8 + b * 256;
        int32_t isum = 0;
        for (int ib = 0; ib < 8; ib++) {
            const uint8_t *qsb = blk + 8 + 16 * ib;
            const int8_t *a = q8b + 32 * ib;
            int32_t dot = 0;
            for (int j = 0; j < 16; j++) {
                dot += (int32_t)orc_kvalues_iq4nl[qsb[j] & 0xF] * (int32_t)a[j];
                dot += (int32_t)orc_kvalues_iq4nl[qsb[j] >> 4] * (int32_t)a[j + 16];
            }
            isum += orc_iq4xs_scale(scales_h, blk + 4, ib) * dot;
        }
        if (isum_out) isum_out[b] = isum;
        sumf += d * d8[b] * (float)isum;
    }
    return sumf;
}

/* Ternary digit (0..2) of element i of a TQ1_0 block: byte * 3^n modulo 256, times three, high byte
 * (crates/infr-cpu/src/kernels.rs:3167-3216, tq1_0_expand_row; dequant.rs:926-962). */
int orc_tq1_0_digit(const uint8_t *blk, int i) {
    static const uint8_t pow3[5] = {1, 3, 9, 27, 81};
    uint8_t byte;
    int n;
    if (i < 160) { n = i / 32; byte = blk[i % 32]; }
    else if (i < 240) { n = (i - 160) / 16; byte = blk[32 + (i - 160) % 16]; }
    else { n = (i - 240) / 4; byte = blk[48 + (i - 240) % 4]; }
    uint8_t q = (uint8_t)(byte * pow3[n]);
    return (int)(((uint16_t)q * 3) >> 8);
}

/* crates/infr-cpu/src/kernels.rs:3218-3240 (vec_dot_tq1_0): the row as digit - 1, one integer dot per
 * superblock, sumf += d * q8.d[b] * iprod. */
float orc_vec_dot_tq1_0(const uint8_t *row, const int8_t *qs8, const float *d8, size_t in_f, int32_t *iprod_out) {
    size_t nb = in_f / 256;
    float sumf = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * 54;
        const int8_t *a = qs8 + b * 256;
        int32_t iprod = 0;
        for (int i = 0; i < 256; i++) iprod += (orc_tq1_0_digit(blk, i) - 1) * (int32_t)a[i];
        if (iprod_out) iprod_out[b] = iprod;
        sumf += orc_rdf16(blk + 52) * d8[b] * (float)iprod;
    }
    return sumf;
}

/* crates/infr-cpu/src/kernels.rs:3066-3126 (tq2_0_expand_row, vec_dot_tq2_0): the ternary row as
 * q - 1 in {-1, 0, 1, 2}, one integer dot per superblock, sumf += d * q8.d[b] * iprod. */
float orc_vec_dot_tq2_0(const uint8_t *row, const int8_t *qs8, const float *d8, size_t in_f, int32_t *iprod_out) {
    size_t nb = in_f / 256;
    float sumf = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * 66;
        const int8_t *a = qs8 + b * 256;
        int32_t iprod = 0;
        for (int chunk = 0; chunk < 2; chunk++)
            for (int l = 0; l < 4; l++)
                for (int mm = 0; mm < 32; mm++)
                    iprod += (((blk[32 * chunk + mm] >> (2 * l)) & 3) - 1) * (int32_t)a[chunk * 128 + l * 32 + mm];
        if (iprod_out) iprod_out[b] = iprod;
        sumf += orc_rdf16(blk + 64) * d8[b] * (float)iprod;
    }
    return sumf;
}

/* crates/infr-cpu/src/kernels.rs:6303-6327 (vec_dot_mxfp4_32_batch_scalar), one activation row:
 * per 32-block the table dot with the per-32 activation codes, sumf += d * q8.d[b] * iprod. */
float orc_vec_dot_mxfp4(const uint8_t *row, const int8_t *qs8, const float *d8, size_t in_f, int32_t *iprod_out) {
    size_t nb = in_f / 32;
    float sumf = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * 17;
        const int8_t *a = qs8 + b * 32;
        int32_t iprod = 0;
        for (int j = 0; j < 16; j++)
            iprod += (int32_t)orc_kvalues_mxfp4[blk[1 + j] & 0xF] * (int32_t)a[j] +
                     (int32_t)orc_kvalues_mxfp4[blk[1 + j] >> 4] * (int32_t)a[j + 16];
        if (iprod_out) iprod_out[b] = iprod;
        sumf += orc_e8m0_half(blk[0]) * d8[b] * (float)iprod;
    }
    return sumf;
}

/* crates/infr-cpu/src/kernels.rs:6472-6500 (vec_dot_nvfp4_batch_scalar), one activation row: the
 * 64-weight block meets activation blocks 2b and 2b + 1; per 16-element sub-block s,
 * sumf += d_s * q8.d[2b + s/2] * iprod_s. iprod_out holds in_f / 16 integers. */
float orc_vec_dot_nvfp4(const uint8_t *row, const int8_t *qs8, const float *d8, size_t in_f, int32_t *iprod_out) {
    size_t nb = in_f / 64;
    float sumf = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * 36;
        for (int sb = 0; sb < 4; sb++) {
            size_t t = 2 * b + (size_t)sb / 2;
            const int8_t *a = qs8 + t * 32 + (sb % 2) * 16;
            const uint8_t *code = blk + 4 + sb * 8;
            int32_t iprod = 0;
            for (int j = 0; j < 8; j++)
                iprod += (int32_t)orc_kvalues_mxfp4[code[j] & 0xF] * (int32_t)a[j] +
                         (int32_t)orc_kvalues_mxfp4[code[j] >> 4] * (int32_t)a[j + 8];
            if (iprod_out) iprod_out[b * 4 + sb] = iprod;
            sumf += orc_ue4m3_half(blk[sb]) * d8[t] * (float)iprod;
        }
    }
    return sumf;
}

/* The 32-weight-block formats against the per-32 activation, one activation row of the batch
 * scalars: Q4_0 kernels.rs:5496-5520, Q4_1 :5793-5822, Q5_0 :5350-5377, Q5_1 :5948-5980,
 * IQ4_NL :6128-6152. Element j of a block takes the low nibble of qs[j], element j+16 the high
 * nibble; Q5_x add qh bit j / j+16 as the 5th code bit. Per-block f32 terms, as written there:
 *   Q4_0   d*d8 * (iprod - 8*bsum)        Q5_0   d*d8 * (iprod - 16*bsum)
 *   Q4_1   d8 * (d*iprod + m*bsum)        Q5_1   d8 * (d*iprod + m*bsum)
 *   IQ4_NL d*d8 * iprod   (iprod over the signed codebook values) */
float orc_vec_dot_blk32(int dtype, const uint8_t *row, const int8_t *qs8, const float *d8,
                        const int32_t *bsum, size_t in_f, int32_t *iprod_out) {
    int qpb, bpb;
    if (!orc_block_layout(dtype, &qpb, &bpb) || qpb != 32) return 0.0f;
    int affine = dtype == ORC_Q4_1 || dtype == ORC_Q5_1;
    int five = dtype == ORC_Q5_0 || dtype == ORC_Q5_1;
    size_t nb = in_f / 32;
    float sumf = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * (size_t)bpb;
        float d = orc_rdf16(blk);
        float mw = affine ? orc_rdf16(blk + 2) : 0.0f;
        const uint8_t *p = blk + (affine ? 4 : 2);
        uint32_t qh = 0;
        if (five) {
            qh = (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
            p += 4;
        }
        const int8_t *q8b = qs8 + b * 32;
        int32_t iprod = 0;
        for (int j = 0; j < 16; j++) {
            int32_t c0, c1;
            if (dtype == ORC_IQ4_NL) {
                c0 = orc_kvalues_iq4nl[p[j] & 0x0F];
                c1 = orc_kvalues_iq4nl[p[j] >> 4];
            } else {
                uint32_t xh0 = five ? ((qh >> j) << 4) & 0x10 : 0;
                uint32_t xh1 = five ? (qh >> (j + 12)) & 0x10 : 0;
                c0 = (int32_t)(((uint32_t)p[j] & 0x0F) | xh0);
                c1 = (int32_t)(((uint32_t)p[j] >> 4) | xh1);
            }
            iprod += c0 * (int32_t)q8b[j] + c1 * (int32_t)q8b[j + 16];
        }
        if (iprod_out) iprod_out[b] = iprod;
        if (affine)
            sumf += d8[b] * (d * (float)iprod + mw * (float)bsum[b]);
        else if (dtype == ORC_IQ4_NL)
            sumf += d * d8[b] * (float)iprod;
        else
            sumf += d * d8[b] * ((float)iprod - (five ? 16.0f : 8.0f) * (float)bsum[b]);
    }
    return sumf;
}

/* crates/infr-cpu/src/kernels.rs:6557-6573 */
float orc_dot(const float *a, const float *b, size_t n) {
    size_t chunks = n / 8;
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (size_t c = 0; c < chunks; c++) {
        size_t base = c * 8;
        for (int j = 0; j < 8; j++) acc[j] = fmaf(a[base + j], b[base + j], acc[j]);
    }
    float s = 0.0f; /* acc.iter().sum() */
    for (int j = 0; j < 8; j++) s += acc[j];
    for (size_t i = chunks * 8; i < n; i++) s = fmaf(a[i], b[i], s);
    return s;
}

/* crates/infr-cpu/src/kernels.rs:6578-6585 (Activation::Silu) */
float orc_silu(float g) { return g / (1.0f + expf(-g)); }

/* crates/infr-cpu/src/kernels.rs:6578-6585 */
float orc_act(int act, float g) {
    switch (act) {
    case ORC_ACT_GELU: return 0.5f * g * (1.0f + tanhf(0.7978846f * (g + 0.044715f * g * g * g)));
    case ORC_ACT_SIGMOID: return 1.0f / (1.0f + expf(-g));
    default: return g / (1.0f + expf(-g));
    }
}

/* crates/infr-cpu/src/kernels.rs:6591-6597 (f32::min / f32::clamp on non-NaN inputs) */
float orc_gated_act(int act, int has_clamp, float l, float gate, float up) {
    if (!has_clamp) return orc_act(act, gate) * up;
    const float g = gate < l ? gate : l;
    const float u = up < -l ? -l : (up > l ? l : up);
    return orc_act(act, g) * u;
}

/* crates/infr-cpu/src/lib.rs:802-850 */
void orc_rms_norm(const float *x, const float *w, float *out, size_t rows, size_t dim, float eps,
                  int accumulate) {
    for (size_t r = 0; r < rows; r++) {
        const float *xr = x + r * dim;
        float sum = 0.0f;
        for (size_t i = 0; i < dim; i++) sum += xr[i] * xr[i];
        const float ss = sum / (float)dim;
        const float s = 1.0f / sqrtf(ss + eps);
        for (size_t i = 0; i < dim; i++) {
            const float v = xr[i] * s * w[i];
            if (accumulate) out[r * dim + i] += v;
            else out[r * dim + i] = v;
        }
    }
}

/* crates/infr-cpu/src/lib.rs:1890-1944 */
void orc_gated_act_op(const float *gate, const float *up, float *out, size_t rows, size_t nff,
                      int act, size_t up_off, size_t up_stride, size_t gate_stride,
                      size_t gate_block_width, int has_clamp, float clamp) {
    for (size_t r = 0; r < rows; r++) {
        const size_t gb = (gate_block_width > 0 || gate_stride > 0) ? r * gate_stride : r * nff;
        const size_t ub = up_stride == 0 ? r * nff + up_off : r * up_stride + up_off;
        for (size_t i = 0; i < nff; i++) {
            size_t gi = gb + i;
            if (gate_block_width > 0) {
                const size_t headw = gate_block_width / 2;
                gi = gb + (i / headw) * gate_block_width + headw + i % headw;
            }
            out[r * nff + i] = orc_gated_act(act, has_clamp, clamp, gate[gi], up[ub + i]);
        }
    }
}

/* crates/infr-cpu/src/lib.rs:1945-1971 */
void orc_gated_act_fused(const float *gu, float *out, size_t rows, size_t nff, int act,
                         int has_clamp, float clamp) {
    for (size_t r = 0; r < rows; r++)
        for (size_t i = 0; i < nff; i++)
            out[r * nff + i] = orc_gated_act(act, has_clamp, clamp, gu[r * 2 * nff + i], gu[r * 2 * nff + nff + i]);
}

/* crates/infr-cpu/src/lib.rs:1972-1988 */
void orc_add(const float *a, const float *b, float *out, size_t n) {
    for (size_t i = 0; i < n; i++) out[i] = a[i] + b[i];
}

/* ───────────────────────────── Op::EmbedGather ───────────────────────────── */

/* crates/infr-cpu/src/lib.rs:2084-2111: total_rows = numel / ne, bpr = bytes / total_rows; per row
 * decode the token's row with the host decode and multiply by `scale`. Returns -2 where the
 * reference would panic (an id past the table), -1 on a dtype the decode does not carry. */
int orc_embed_gather(int dtype, const uint8_t *table, size_t table_bytes, size_t table_numel,
                     const int32_t *ids, size_t rows, size_t ne, float scale, float *out) {
    if (!table || !ids || !out || ne == 0 || table_numel % ne != 0) return -2;
    size_t total_rows = table_numel / ne;
    size_t bpr = table_bytes / total_rows;
    float *row = (float *)malloc(sizeof(float) * ne);
    for (size_t r = 0; r < rows; r++) {
        if (ids[r] < 0 || (size_t)ids[r] >= total_rows) {
            free(row);
            return -2;
        }
        if (orc_dequant_block(dtype, table + (size_t)ids[r] * bpr, bpr, row) != 0) {
            free(row);
            return -1;
        }
        for (size_t e = 0; e < ne; e++) out[r * ne + e] = row[e] * scale;
    }
    free(row);
    return 0;
}

/* ───────────────────────────── Op::Linear ───────────────────────────── */

typedef struct {
    int8_t *qs;
    float *d;
    int32_t *bsums;   /* per 32 */
    int32_t *bsums16; /* per 16 (Q8 only) */
} acts_t;

/* lib.rs:1037-1062: per-256 `Q8` for the 256-block formats and for Q8_0 rows of whole 256s;
 * a Q8_0 row that is a multiple of 32 only takes the per-32 `Q8x32` (q8_0_blk32). */
static int is_q8_super(int dtype, size_t in_f) {
    return dtype == ORC_Q4_K || dtype == ORC_Q5_K || dtype == ORC_Q6_K || dtype == ORC_Q2_K || dtype == ORC_Q3_K ||
           dtype == ORC_IQ4_XS || dtype == ORC_TQ2_0 || dtype == ORC_TQ1_0 || (dtype == ORC_Q8_0 && in_f % 256 == 0);
}

static void acts_free(acts_t *a) {
    free(a->qs);
    free(a->d);
    free(a->bsums);
    free(a->bsums16);
}

/* Quantize m rows with the quantizer the dispatch picks: per-256 `Q8` for Q4K/Q6K/Q8_0
 * (crates/infr-cpu/src/lib.rs:1043-1062,1186-1210), per-32 `Q8x32` for Q2_0 (:1064-1076,1406-1412). */
static int acts_build(int dtype, const float *x, size_t m, size_t in_f, acts_t *a) {
    memset(a, 0, sizeof *a);
    a->qs = (int8_t *)malloc(m * in_f);
    if (is_q8_super(dtype, in_f)) {
        size_t nb = in_f / 256;
        a->d = (float *)malloc(sizeof(float) * m * nb);
        a->bsums = (int32_t *)malloc(sizeof(int32_t) * m * nb * 8);
        a->bsums16 = (int32_t *)malloc(sizeof(int32_t) * m * nb * 16);
#pragma omp parallel for schedule(static)
        for (long r = 0; r < (long)m; r++)
            orc_quantize_q8(x + r * in_f, in_f, a->qs + r * in_f, a->d + r * nb,
                            a->bsums + r * nb * 8, a->bsums16 + r * nb * 16);
    } else {
        size_t nb = in_f / 32;
        a->d = (float *)malloc(sizeof(float) * m * nb);
        a->bsums = (int32_t *)malloc(sizeof(int32_t) * m * nb);
#pragma omp parallel for schedule(static)
        for (long r = 0; r < (long)m; r++)
            orc_quantize_q8_32(x + r * in_f, in_f, a->qs + r * in_f, a->d + r * nb,
                               a->bsums + r * nb);
    }
    return 0;
}

static float row_dot(int dtype, const uint8_t *row, const acts_t *a, size_t r, size_t in_f,
                     int32_t *ia, int32_t *ib) {
    switch (dtype) {
    case ORC_Q4_K: {
        size_t nb = in_f / 256;
        return orc_vec_dot_q4k(row, a->qs + r * in_f, a->d + r * nb, a->bsums + r * nb * 8, in_f,
                               ia, ib);
    }
    case ORC_Q6_K: {
        size_t nb = in_f / 256;
        return orc_vec_dot_q6k(row, a->qs + r * in_f, a->d + r * nb, in_f, ia);
    }
    case ORC_Q8_0: {
        if (in_f % 256 != 0)
            return orc_vec_dot_q8_0_32(row, a->qs + r * in_f, a->d + r * (in_f / 32), in_f, ia);
        size_t nb = in_f / 256;
        return orc_vec_dot_q8_0(row, a->qs + r * in_f, a->d + r * nb, in_f, ia);
    }
    case ORC_Q2_0: {
        size_t nb = in_f / 32;
        return orc_vec_dot_q2_0(row, a->qs + r * in_f, a->d + r * nb, a->bsums + r * nb, in_f, ia);
    }
    case ORC_Q5_K: {
        size_t nb = in_f / 256;
        return orc_vec_dot_q5k(row, a->qs + r * in_f, a->d + r * nb, a->bsums + r * nb * 8, in_f,
                               ia, ib);
    }
    case ORC_Q2_K: {
        size_t nb = in_f / 256;
        return orc_vec_dot_q2k(row, a->qs + r * in_f, a->d + r * nb, a->bsums16 + r * nb * 16, in_f, ia, ib);
    }
    case ORC_Q3_K: {
        size_t nb = in_f / 256;
        return orc_vec_dot_q3k(row, a->qs + r * in_f, a->d + r * nb, a->bsums16 + r * nb * 16, in_f, ia);
    }
    case ORC_IQ4_XS: return orc_vec_dot_iq4xs(row, a->qs + r * in_f, a->d + r * (in_f / 256), in_f, ia);
    case ORC_TQ2_0: return orc_vec_dot_tq2_0(row, a->qs + r * in_f, a->d + r * (in_f / 256), in_f, ia);
    case ORC_TQ1_0: return orc_vec_dot_tq1_0(row, a->qs + r * in_f, a->d + r * (in_f / 256), in_f, ia);
    case ORC_Q4_0:
    case ORC_Q4_1:
    case ORC_Q5_0:
    case ORC_Q5_1:
    case ORC_IQ4_NL: {
        size_t nb = in_f / 32;
        return orc_vec_dot_blk32(dtype, row, a->qs + r * in_f, a->d + r * nb, a->bsums + r * nb, in_f, ia);
    }
    case ORC_MXFP4: return orc_vec_dot_mxfp4(row, a->qs + r * in_f, a->d + r * (in_f / 32), in_f, ia);
    case ORC_NVFP4: return orc_vec_dot_nvfp4(row, a->qs + r * in_f, a->d + r * (in_f / 32), in_f, ia);
    default:
        return 0.0f;
    }
}

static int linear_shape_ok(int dtype, size_t in_f) {
    /* The restatement carries the arms the four formats take when in_f is block-aligned:
     * Q4K/Q6K: 256-element weight blocks; Q8_0: whole 32-blocks, per-256 activations when in_f is
     * a multiple of 256 and the per-32 kernel otherwise (lib.rs:1037-1042); Q2_0 needs
     * in_f % 64 == 0 (lib.rs:1406). */
    switch (dtype) {
    case ORC_Q4_K:
    case ORC_Q5_K:
    case ORC_Q2_K:
    case ORC_Q3_K:
    case ORC_IQ4_XS:
    case ORC_TQ2_0:
    case ORC_TQ1_0:
    case ORC_Q6_K: return in_f % 256 == 0;
    case ORC_Q4_0:
    case ORC_Q4_1:
    case ORC_Q5_0:
    case ORC_Q5_1:
    case ORC_IQ4_NL:
    case ORC_MXFP4:
    case ORC_Q8_0: return in_f % 32 == 0;
    case ORC_NVFP4:
    case ORC_Q2_0: return in_f % 64 == 0;
    case ORC_F32:
    case ORC_F16:
    case ORC_BF16: return 1; /* dot / dot_f16 / dot_bf16, any length (lib.rs:1162-1164, 1443-1462) */
    default: return 0;
    }
}

int orc_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

int orc_linear(int dtype, const uint8_t *w, size_t wbytes, size_t w_numel, size_t w_off,
               const float *x, float *y, size_t m, size_t in_f, size_t out_f, int reference_mode,
               int threads) {
    if (!w || !x || !y || in_f == 0 || w_numel % in_f != 0 || w_off % in_f != 0) return -2;
    if (!linear_shape_ok(dtype, in_f)) return -1;
    /* lib.rs:1003-1008 */
    size_t total_rows = w_numel / in_f;
    size_t bpr = wbytes / total_rows;
    size_t row0 = w_off / in_f;
    if (row0 + out_f > total_rows) return -2;
    const uint8_t *wb = w + row0 * bpr;
#ifdef _OPENMP
    int nt = threads > 0 ? threads : omp_get_max_threads();
#else
    int nt = 1;
    (void)threads;
#endif
    (void)nt;

    if (dtype == ORC_F32 || dtype == ORC_F16 || dtype == ORC_BF16 || reference_mode || (dtype == ORC_Q5_0 && m == 1)) {
        /* lib.rs:1015-1031 (reference mode) / :1162-1164,1443-1462 (F32 / F16 / BF16 weights): decode
         * row, dot(). dot_f16 and dot_bf16 (kernels.rs:6505-6549) widen each weight exactly and run
         * dot's own eight FMA chains, so decoding the row first gives their bits.
         * Q5_0 has no arm in the one-token match (lib.rs:1081-1165), so decode takes its last arm,
         * `dot(&bytes_to_f32(row, dt), xrow)` (:1165): f32 activations, no int8 rounding. With
         * m >= 2 it takes the per-32 int8 kernel (:1322-1329). */
#pragma omp parallel num_threads(nt)
        {
            float *wf = (float *)malloc(sizeof(float) * in_f);
#pragma omp for schedule(dynamic, 8)
            for (long o = 0; o < (long)out_f; o++) {
                orc_dequant_block(dtype, wb + (size_t)o * bpr, bpr, wf);
                for (size_t r = 0; r < m; r++) y[r * out_f + (size_t)o] = orc_dot(wf, x + r * in_f, in_f);
            }
            free(wf);
        }
        return 0;
    }

    acts_t a;
    acts_build(dtype, x, m, in_f, &a);
    if (m == 1) {
        /* lib.rs:1079: 16 output rows per claimed task */
#pragma omp parallel for schedule(dynamic, 16) num_threads(nt)
        for (long o = 0; o < (long)out_f; o++)
            y[o] = row_dot(dtype, wb + (size_t)o * bpr, &a, 0, in_f, NULL, NULL);
    } else {
        /* lib.rs:1211-1489: o-major temp then transpose; per element identical to the single-row
         * kernel (batch kernels are bit-identical, kernels.rs:9297-9405). 8-row groups. */
        float *out_t = (float *)malloc(sizeof(float) * out_f * m);
#pragma omp parallel for schedule(dynamic, 8) num_threads(nt)
        for (long o = 0; o < (long)out_f; o++)
            for (size_t r = 0; r < m; r++)
                out_t[(size_t)o * m + r] = row_dot(dtype, wb + (size_t)o * bpr, &a, r, in_f, NULL, NULL);
#pragma omp parallel for schedule(static) num_threads(nt)
        for (long r = 0; r < (long)m; r++)
            for (size_t o = 0; o < out_f; o++) y[(size_t)r * out_f + o] = out_t[o * m + (size_t)r];
        free(out_t);
    }
    acts_free(&a);
    return 0;
}

int orc_linear_int_stages(int dtype, const uint8_t *w, size_t wbytes, size_t w_numel, size_t w_off,
                          const float *x, size_t m, size_t in_f, size_t out_f, int32_t *ia,
                          int32_t *ib) {
    if (!w || !x || !ia || in_f == 0 || w_numel % in_f != 0 || w_off % in_f != 0) return -2;
    if (!linear_shape_ok(dtype, in_f) || dtype == ORC_F32) return -1;
    size_t total_rows = w_numel / in_f;
    size_t bpr = wbytes / total_rows;
    size_t row0 = w_off / in_f;
    if (row0 + out_f > total_rows) return -2;
    const uint8_t *wb = w + row0 * bpr;
    size_t blocks = (dtype == ORC_Q4_K || dtype == ORC_Q5_K || dtype == ORC_Q6_K || dtype == ORC_Q2_K || dtype == ORC_Q3_K || dtype == ORC_IQ4_XS || dtype == ORC_TQ2_0 || dtype == ORC_TQ1_0) ? in_f / 256 : (dtype == ORC_NVFP4 ? in_f / 16 : in_f / 32);
    acts_t a;
    acts_build(dtype, x, m, in_f, &a);
#pragma omp parallel for schedule(dynamic, 8)
    for (long o = 0; o < (long)out_f; o++)
        for (size_t r = 0; r < m; r++) {
            size_t off = (r * out_f + (size_t)o) * blocks;
            row_dot(dtype, wb + (size_t)o * bpr, &a, r, in_f, ia + off, ib ? ib + off : NULL);
        }
    acts_free(&a);
    return 0;
}

/* crates/infr-testkit/src/lib.rs:150-163 */
void orc_ref_linear_f64(const float *x, const float *w, size_t m, size_t in_f, size_t out_f,
                        float *out) {
#pragma omp parallel for schedule(static)
    for (long o = 0; o < (long)out_f; o++)
        for (size_t r = 0; r < m; r++) {
            double acc = 0.0;
            for (size_t i = 0; i < in_f; i++)
                acc += (double)x[r * in_f + i] * (double)w[(size_t)o * in_f + i];
            out[r * out_f + (size_t)o] = (float)acc;
        }
}

/* ───────────────────────────── Op::MoeFfn ───────────────────────────── */

/* crates/infr-cpu/src/moe.rs:42-53 (restricted to the dtypes this restatement decodes). */
int orc_expert_acts_kind(int dtype, size_t in_f, int int8_ok) {
    if (int8_ok && (dtype == ORC_Q4_K || dtype == ORC_Q6_K || dtype == ORC_Q8_0 || dtype == ORC_Q5_K) && in_f % 256 == 0)
        return ORC_ACTS_SUPER;
    if (int8_ok && (dtype == ORC_Q8_0 || dtype == ORC_Q5_0) && in_f % 32 == 0) return ORC_ACTS_BLK32;
    return ORC_ACTS_RAW;
}

/* One expert bank applied to `count` activation rows: out_t[o*count + i], o-major
 * (crates/infr-cpu/src/moe.rs:66-175). Super: per-256 int8 activations through the batch kernels
 * (bit-identical to the single-row kernels); Blk32: per-32 int8 activations through
 * vec_dot_q8_0_32_batch / vec_dot_q5_0_32_batch (moe.rs:115-141; the 8-row tile computes the same
 * per-row values); Raw: weight row decoded once, f32 dot(). */
static int expert_gemm(const uint8_t *wbytes, size_t wlen, int dt, size_t in_f, size_t out_f,
                       int kind, const float *xin, size_t count, float *out_t) {
    size_t bpr = wlen / out_f;
    if (kind == ORC_ACTS_SUPER || kind == ORC_ACTS_BLK32) {
        acts_t a;
        acts_build(dt, xin, count, in_f, &a); /* per 256 or per 32 by (dt, in_f), as the kind */
        for (size_t o = 0; o < out_f; o++)
            for (size_t i = 0; i < count; i++)
                out_t[o * count + i] = row_dot(dt, wbytes + o * bpr, &a, i, in_f, NULL, NULL);
        acts_free(&a);
        return 0;
    }
    if (kind == ORC_ACTS_RAW) {
        float *wf = (float *)malloc(sizeof(float) * in_f);
        for (size_t o = 0; o < out_f; o++) {
            if (orc_dequant_block(dt, wbytes + o * bpr, bpr, wf) != 0) {
                free(wf);
                return -1;
            }
            for (size_t i = 0; i < count; i++)
                out_t[o * count + i] = orc_dot(wf, xin + i * in_f, in_f);
        }
        free(wf);
        return 0;
    }
    return -1;
}

/* Stable descending order of v[0..n): `idx.sort_by(|a, b| v[b].partial_cmp(&v[a]).unwrap())`
 * (lib.rs:2509, 2528) — ties keep the lower index first. Selection sort over the first `take`. */
static void top_desc_stable(const float *v, size_t n, size_t take, size_t *out, char *taken) {
    memset(taken, 0, n);
    for (size_t k = 0; k < take; k++) {
        size_t best = n;
        for (size_t e = 0; e < n; e++) {
            if (taken[e]) continue;
            if (best == n || v[e] > v[best]) best = e;
        }
        taken[best] = 1;
        out[k] = best;
    }
}

int orc_moe_ffn(const orc_moe_params *p, const float *x, const float *router_x,
                const uint8_t *router, size_t router_bytes, const uint8_t *gate, size_t gate_bytes,
                const uint8_t *up, size_t up_bytes, const uint8_t *down, size_t down_bytes,
                float *y, int32_t *sel_idx, float *sel_w, int threads, const float *down_scale,
                const float *exp_probs_b, const int32_t *expert_ids) {
    size_t ne = p->ne, n_expert = p->n_expert, n_used = p->n_used, nffx = p->n_ff_exp;
    size_t rows = p->rows;
    if (!ne || !n_expert || !n_used || !nffx || !rows || n_used > n_expert) return -2;
    /* the two assertions in front of the arm (lib.rs:2293-2309) */
    if (p->has_clamp && (p->act == ORC_ACT_SIGMOID || p->weight_before)) return -3;
    if (expert_ids && (exp_probs_b || p->n_expert_groups > 1)) return -3;
    if (p->n_expert_groups > 1 && p->n_expert_groups_used > 0 &&
        (n_expert % p->n_expert_groups != 0 || p->n_expert_groups_used > p->n_expert_groups))
        return -2;
#ifdef _OPENMP
    int nt = threads > 0 ? threads : omp_get_max_threads();
#else
    int nt = 1;
    (void)threads;
#endif
    (void)nt;
    /* lib.rs:2340-2348: fused banks hold gate rows then up rows inside each expert's slice */
    size_t gst = gate_bytes / n_expert, dst_ = down_bytes / n_expert;
    size_t ust = p->fused_gate_up ? 0 : up_bytes / n_expert;
    int udt = p->fused_gate_up ? p->gate_dtype : p->up_dtype;
    size_t out_gu = p->fused_gate_up ? 2 * nffx : nffx;
    /* lib.rs:2359 */
    int int8_ok = rows >= 2 && !p->reference_mode;
    int rc = 0;

    /* Router GEMM over all rows (lib.rs:2364-2396). Its activations are router_x. */
    float *lt = (float *)malloc(sizeof(float) * n_expert * rows);
    int r_kind = orc_expert_acts_kind(p->router_dtype, ne, int8_ok);
    if (expert_gemm(router, router_bytes, p->router_dtype, ne, n_expert, r_kind, router_x, rows, lt)) {
        free(lt);
        return -1;
    }

    /* Per-row gating + selection + weights (lib.rs:2421-2543). */
    size_t *idx = (size_t *)malloc(sizeof(size_t) * rows * n_used);
    float *wts = (float *)malloc(sizeof(float) * rows * n_used);
    float *probs = (float *)malloc(sizeof(float) * n_expert);
    float *selp = (float *)malloc(sizeof(float) * n_expert);
    char *taken = (char *)malloc(n_expert);
    for (size_t r = 0; r < rows && rc == 0; r++) {
        if (p->gating == ORC_GATING_SIGMOID) { /* :2437-2439 */
            for (size_t e = 0; e < n_expert; e++) probs[e] = 1.0f / (1.0f + expf(-lt[e * rows + r]));
        } else if (p->gating == ORC_GATING_SQRT_SOFTPLUS) { /* :2440-2454 */
            for (size_t e = 0; e < n_expert; e++) {
                float v = lt[e * rows + r];
                float sp = v > 20.0f ? v : logf(1.0f + expf(v));
                probs[e] = sqrtf(sp);
            }
        } else { /* softmax, :2427-2436 */
            float maxl = -INFINITY;
            for (size_t e = 0; e < n_expert; e++) {
                float v = lt[e * rows + r];
                maxl = v > maxl ? v : maxl;
            }
            float psum = 0.0f;
            for (size_t e = 0; e < n_expert; e++) probs[e] = expf(lt[e * rows + r] - maxl);
            for (size_t e = 0; e < n_expert; e++) psum += probs[e];
            for (size_t e = 0; e < n_expert; e++) probs[e] /= psum;
        }
        if (expert_ids) { /* hash routing: the ids are the selection, in their own order (:2456-2472) */
            for (size_t k = 0; k < n_used; k++) {
                int32_t e = expert_ids[r * n_used + k];
                if (e < 0 || (size_t)e >= n_expert) {
                    rc = -4;
                    break;
                }
                idx[r * n_used + k] = (size_t)e;
            }
            if (rc) break;
        } else {
            /* selection-only copy: bias (:2476-2485), then group masking (:2488-2526) */
            for (size_t e = 0; e < n_expert; e++) selp[e] = exp_probs_b ? probs[e] + exp_probs_b[e] : probs[e];
            if (p->n_expert_groups > 1 && p->n_expert_groups_used > 0) {
                size_t ng = p->n_expert_groups, per = n_expert / ng, ng_used = p->n_expert_groups_used;
                float *gscores = (float *)malloc(sizeof(float) * ng);
                size_t *gidx = (size_t *)malloc(sizeof(size_t) * ng);
                char *gtaken = (char *)malloc(ng);
                for (size_t g = 0; g < ng; g++) {
                    float best0 = -INFINITY, best1 = -INFINITY;
                    for (size_t i = 0; i < per; i++) {
                        float sv = selp[g * per + i];
                        if (sv > best0) {
                            best1 = best0;
                            best0 = sv;
                        } else if (sv > best1) {
                            best1 = sv;
                        }
                    }
                    gscores[g] = best0 + best1;
                }
                top_desc_stable(gscores, ng, ng_used, gidx, gtaken);
                memset(gtaken, 0, ng);
                for (size_t k = 0; k < ng_used; k++) gtaken[gidx[k]] = 1;
                for (size_t g = 0; g < ng; g++)
                    if (!gtaken[g])
                        for (size_t i = 0; i < per; i++) selp[g * per + i] = -INFINITY;
                free(gscores);
                free(gidx);
                free(gtaken);
            }
            top_desc_stable(selp, n_expert, n_used, idx + r * n_used, taken);
        }
        /* weights from the unbiased probs (:2536-2541) */
        float wsum = 0.0f;
        for (size_t k = 0; k < n_used; k++) wsum += probs[idx[r * n_used + k]];
        wsum = wsum > 1e-20f ? wsum : 1e-20f;
        for (size_t k = 0; k < n_used; k++) {
            float pe = probs[idx[r * n_used + k]];
            wts[r * n_used + k] = p->norm_w ? pe / wsum * p->scale : pe * p->scale;
            if (sel_idx) sel_idx[r * n_used + k] = (int32_t)idx[r * n_used + k];
            if (sel_w) sel_w[r * n_used + k] = wts[r * n_used + k];
        }
    }
    free(probs);
    free(selp);
    free(taken);
    free(lt);
    if (rc) {
        free(idx);
        free(wts);
        return rc;
    }

    /* Buckets: (row -> expert) pairs grouped by expert, rows ascending inside a bucket
     * (lib.rs:2554-2587). pair_w = the pair's routing weight (weight_before folds it into stage C). */
    size_t n_pairs = rows * n_used;
    size_t *pair_row = (size_t *)malloc(sizeof(size_t) * n_pairs);
    float *pair_w = (float *)malloc(sizeof(float) * n_pairs);
    size_t *slot_pair = (size_t *)malloc(sizeof(size_t) * n_pairs); /* [r][rank] */
    size_t *bucket_e = (size_t *)malloc(sizeof(size_t) * n_expert);
    size_t *bucket_p0 = (size_t *)malloc(sizeof(size_t) * (n_expert + 1));
    size_t n_buckets = 0, np = 0;
    for (size_t e = 0; e < n_expert; e++) {
        size_t p0 = np;
        for (size_t r = 0; r < rows; r++)
            for (size_t k = 0; k < n_used; k++)
                if (idx[r * n_used + k] == e) {
                    slot_pair[r * n_used + k] = np;
                    pair_w[np] = wts[r * n_used + k];
                    pair_row[np++] = r;
                }
        if (np > p0) {
            bucket_e[n_buckets] = e;
            bucket_p0[n_buckets] = p0;
            n_buckets++;
        }
    }
    bucket_p0[n_buckets] = np;

    int g_kind = orc_expert_acts_kind(p->gate_dtype, ne, int8_ok);
    int u_kind = p->fused_gate_up ? g_kind : orc_expert_acts_kind(udt, ne, int8_ok);
    int d_kind = orc_expert_acts_kind(p->down_dtype, nffx, int8_ok);
    float *y_pairs = (float *)calloc(n_pairs * ne, sizeof(float));

    /* Stages A-D per bucket (lib.rs:2685-2946). The reference quantizes each distinct row once
     * and clones it per pair; quantizing the pair's copy of the same row gives the same bytes. */
#pragma omp parallel for schedule(dynamic, 1) num_threads(nt)
    for (long b = 0; b < (long)n_buckets; b++) {
        size_t e = bucket_e[b], p0 = bucket_p0[b], count = bucket_p0[b + 1] - p0;
        float *xin = (float *)malloc(sizeof(float) * count * ne);
        for (size_t i = 0; i < count; i++)
            memcpy(xin + i * ne, x + pair_row[p0 + i] * ne, sizeof(float) * ne);
        float *gt = (float *)malloc(sizeof(float) * out_gu * count);
        float *ut = p->fused_gate_up ? gt + nffx * count : (float *)malloc(sizeof(float) * nffx * count);
        float *act = (float *)malloc(sizeof(float) * count * nffx);
        float *dt_ = (float *)malloc(sizeof(float) * ne * count);
        int e1 = expert_gemm(gate + e * gst, gst, p->gate_dtype, ne, out_gu, g_kind, xin, count, gt);
        int e2 = p->fused_gate_up ? 0 : expert_gemm(up + e * ust, ust, udt, ne, nffx, u_kind, xin, count, ut);
        /* Stage C (lib.rs:2824-2861): gated_act_fn(act, clamp, wp * g, wp * u), wp = the pair's
         * routing weight under weight_before, else 1.0 */
        for (size_t i = 0; i < count; i++) {
            float wp = p->weight_before ? pair_w[p0 + i] : 1.0f;
            for (size_t f = 0; f < nffx; f++)
                act[i * nffx + f] = orc_gated_act(p->act, p->has_clamp, p->clamp, wp * gt[f * count + i],
                                                  wp * ut[f * count + i]);
        }
        int e3 = expert_gemm(down + e * dst_, dst_, p->down_dtype, nffx, ne, d_kind, act, count, dt_);
        if (e1 || e2 || e3) {
#pragma omp atomic write
            rc = -1;
        }
        /* un-transpose with the per-expert down_scale folded in (lib.rs:2926-2945) */
        for (size_t i = 0; i < count; i++)
            for (size_t d = 0; d < ne; d++)
                y_pairs[(p0 + i) * ne + d] = down_scale ? dt_[d * count + i] * down_scale[e] : dt_[d * count + i];
        free(xin);
        free(gt);
        if (!p->fused_gate_up) free(ut);
        free(act);
        free(dt_);
    }

    /* Stage E (lib.rs:2967-2983): rank order, `*o += w_e * yv` (separate multiply and add);
     * under weight_before the weight is already inside the activation and w_e = 1.0. */
    for (size_t r = 0; r < rows; r++) {
        float *orow = y + r * ne;
        for (size_t d = 0; d < ne; d++) orow[d] = 0.0f;
        for (size_t k = 0; k < n_used; k++) {
            float w_e = p->weight_before ? 1.0f : wts[r * n_used + k];
            const float *yp = y_pairs + slot_pair[r * n_used + k] * ne;
            for (size_t d = 0; d < ne; d++) orow[d] += w_e * yp[d];
        }
    }
    free(y_pairs);
    free(pair_row);
    free(pair_w);
    free(slot_pair);
    free(bucket_e);
    free(bucket_p0);
    free(idx);
    free(wts);
    return rc;
}

/* ───────────────────────────── test-input recipes ───────────────────────────── */

/* crates/infr-testkit/src/lib.rs:49-56 */
void orc_lcg_bytes(uint32_t seed, size_t n, uint8_t *out) {
    for (size_t i = 0; i < n; i++) {
        seed = seed * 1664525u + 1013904223u;
        out[i] = (uint8_t)(seed >> 16);
    }
}

/* crates/infr-testkit/src/lib.rs:60-64 */
void orc_gen_f32(size_t n, size_t salt, float *out) {
    for (size_t i = 0; i < n; i++) out[i] = ((float)((i * 13 + salt) % 29) - 14.0f) * 0.05f;
}

static void put_f16(uint8_t *b, float v) {
    uint16_t h = orc_f32_to_f16_bits(v);
    b[0] = (uint8_t)(h & 0xFF);
    b[1] = (uint8_t)(h >> 8);
}

/* crates/infr-testkit/src/lib.rs:73-93 (synth_scales), :106-123 (synth_weight): LCG payload per
 * block seeded `seed ^ b`, then the f16 scale slots overwritten. Slot offsets from
 * crates/infr-core/src/decode_spec.rs:305-358: Q8_0 d@0; Q4K/Q5K d@0 dmin@2; Q6K d@208; Q2_0 d@0;
 * Q4_0/Q5_0/IQ4_NL d@0; Q4_1/Q5_1 d@0 m@2. Magnitudes from synth_scales (testkit lib.rs:73-93). */
size_t orc_synth_weight(int dtype, size_t n_elem, uint32_t seed, uint8_t *out) {
    int qpb, bpb;
    if (!orc_block_layout(dtype, &qpb, &bpb) || dtype == ORC_F32 || dtype == ORC_F16) return 0;
    if (n_elem % (size_t)qpb != 0) return 0;
    size_t nblk = n_elem / (size_t)qpb;
    for (size_t b = 0; b < nblk; b++) {
        uint8_t *blk = out + b * (size_t)bpb;
        orc_lcg_bytes(seed ^ (uint32_t)b, (size_t)bpb, blk);
        switch (dtype) {
        case ORC_Q8_0: put_f16(blk, 0.01f); break;
        case ORC_Q4_K:
            put_f16(blk, 0.05f);
            put_f16(blk + 2, 0.10f);
            break;
        case ORC_Q6_K: put_f16(blk + 208, 0.03f); break;
        case ORC_Q2_0: put_f16(blk, 0.05f); break;
        case ORC_Q5_K:
            put_f16(blk, 0.05f);
            put_f16(blk + 2, 0.10f);
            break;
        case ORC_Q2_K: /* d@80, dmin@82 (decode_spec.rs:323) */
            put_f16(blk + 80, 0.05f);
            put_f16(blk + 82, 0.10f);
            break;
        case ORC_Q3_K: put_f16(blk + 108, 0.03f); break; /* d@108 (decode_spec.rs:325) */
        case ORC_IQ4_XS: put_f16(blk, 0.06f); break;      /* d@0 (decode_spec.rs:351) */
        case ORC_TQ1_0: put_f16(blk + 52, 0.05f); break;  /* d@52 (decode_spec.rs:354) */
        case ORC_TQ2_0: put_f16(blk + 64, 0.05f); break;  /* d@64 (decode_spec.rs:356) */
        case ORC_MXFP4: blk[0] = 125; break;              /* E8M0 nearest 0.25 in log space: 2^(125 - 127) (decode_spec.rs:191, 216-219) */
        case ORC_NVFP4:                                   /* UE4M3 nearest 0.5 * (0.625 + 0.125 i) (decode_spec.rs:192-198, 223-245) */
            blk[0] = 42, blk[1] = 44, blk[2] = 46, blk[3] = 48;
            break;
        case ORC_Q4_0:
        case ORC_Q5_0: put_f16(blk, 0.04f); break;
        case ORC_Q4_1:
        case ORC_Q5_1:
            put_f16(blk, 0.04f);
            put_f16(blk + 2, -0.30f);
            break;
        case ORC_IQ4_NL: put_f16(blk, 0.004f); break;
        }
    }
    return nblk * (size_t)bpb;
}

/* crates/infr-cpu/src/kernels.rs:6611-6624 */
static uint64_t lcg64(uint64_t *s) {
    *s = *s * 6364136223846793005ull + 1442695040888963407ull;
    return *s;
}
void orc_det_bytes(size_t n, uint64_t seed, uint8_t *out) {
    for (size_t i = 0; i < n; i++) out[i] = (uint8_t)(lcg64(&seed) >> 33);
}
void orc_det_x(size_t n, uint64_t seed, float *out) {
    for (size_t i = 0; i < n; i++)
        out[i] = ((float)(lcg64(&seed) >> 40) / (float)(1ull << 24)) * 2.0f - 1.0f;
}
