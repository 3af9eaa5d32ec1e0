// Prefill GEMM (65 tokens and up) of the 32-weight-block formats Q4_0, Q4_1, Q5_0, Q5_1, IQ4_NL, MXFP4 and
// NVFP4 on the int8 matrix cores, and of Q8_0 rows that are not whole 256s (which infr-cpu multiplies against
// the per-32 activation as well: `q8_0_blk32`, crates/infr-cpu/src/lib.rs:1037-1042, d*d8 * iprod per
// block, kernels.rs:1170-1187). A row may end inside a 256-element step: the quantizer pads the
// activation with zero codes, scales and sums up to the step, and the blocks past the row's end
// are not read (their A and B constants are zero), so the padded blocks add +0.0.
//
// infr-cpu multiplies these against the per-32 activation (scale d8 and code sum bsum per 32
// elements) and adds per block (crates/infr-cpu/src/kernels.rs:5496-5520, :5793-5822, :5350-5377,
// :5948-5980, :6128-6152)
//     Q4_0   d*d8 * (iprod - 8*bsum)        Q5_0   d*d8 * (iprod - 16*bsum)
//     Q4_1   d8 * (d*iprod + m*bsum)        Q5_1   d8 * (d*iprod + m*bsum)
//     IQ4_NL d*d8 * iprod                   (iprod over the signed codebook values)
//     MXFP4  d*d8 * iprod                   (d the E8M0 scale halved, iprod over doubled E2M1 values)
//     NVFP4  d_s*d8 * iprod_s               (per 16 weights: a UE4M3 scale, halved, and a K = 16 MFMA each)
// The codes (0..15, 0..31, or the codebook's int8) are int8 operands, so iprod is one
// v_mfma_i32_32x32x32_i8 per block, exact. Every format's term is d8 * (A * iprod + B * bsum) with
// two per-block constants (A = d; B = -8d, -16d, m or 0), evaluated with one conversion, one
// multiply and two FMAs per output and block: the CPU's terms in another association (these formats'
// one-token kernels already differ from the CPU by their butterfly sums), ~1e-7 relative.
//
// Tiling as the other shared-operand kernels: 128 tokens x 32 weight rows per workgroup, wave w owns
// tokens 32w..32w+31 and unpacks blocks 2w, 2w+1 of every row of a 256-element step into LDS in
// MFMA B order (double-buffered, one barrier per step). Element j of a block is the low nibble of
// qs[j], element j + 16 the high nibble (plus bit j / j + 16 of qh as the fifth code bit), so the
// h = 0 lanes of the B operand take the low nibbles of the block's 16 bytes and the h = 1 lanes the
// high ones.
#include "gemv_formats.hpp"
#include "kernels.hpp"

namespace infr {

typedef int v16i __attribute__((ext_vector_type(16)));

// LDS of one 256-element step: B operands [block][lane] x 16 B | A [row][8] | B [row][8] (f32)
struct Nib32Lds {
    static constexpr int a_off = 8 * 1024;
    static constexpr int b_off = a_off + 32 * 8 * 4;
    static constexpr int bytes = b_off + 32 * 8 * 4;
};

// The formats of this kernel: the five nibble formats and Q8_0 against per-32 activations.
enum class Blk32 { Q4_0, Q4_1, Q5_0, Q5_1, IQ4_NL, Q8_0, MXFP4, NVFP4 };

// nb: 256-element steps (the last one may be partly past the row); nblk: 32-weight blocks of a row
template <Blk32 K, bool STAGES>
__global__ __launch_bounds__(256) void mmq_shared_nib32_kernel(
    const uint8_t* __restrict__ w, size_t bpr, const int8_t* __restrict__ qs, const float* __restrict__ d8,
    const float* __restrict__ bsf, float* __restrict__ y, int m, int out_f, int nb, int nblk,
    int32_t* __restrict__ st_iprod) {
    constexpr bool kAffine = K == Blk32::Q4_1 || K == Blk32::Q5_1;
    constexpr bool kFive = K == Blk32::Q5_0 || K == Blk32::Q5_1;
    constexpr bool kBytes = K == Blk32::Q8_0;  // codes are whole bytes: 32 of them per block
    // MXFP4: [E8M0 scale][16 code bytes], 17 bytes at any byte alignment; the codes index a signed
    // table of doubled E2M1 values and the scale decodes halved (crates/infr-cpu/src/lib.rs:1394-1432)
    constexpr bool kMx = K == Blk32::MXFP4;
    // NVFP4: 36-byte blocks of 64 weights [UE4M3 d[4]][qs[32]]; a 32-element "block" of this kernel is half
    // of one - sub-blocks 2 hf, 2 hf + 1 of 16 weights (qs[8 s .. 8 s + 7]: low nibbles elements 0..7, high
    // nibbles 8..15), each with its own scale against the half's one activation scale
    // (crates/infr-cpu/src/kernels.rs:6472-6500). A sub-block is one K = 16 MFMA; the A constant is the
    // first sub-block's scale and the B constant, which the format does not need, the second's.
    constexpr bool kNv = K == Blk32::NVFP4;
    constexpr int kBlockBytes = kMx ? 17 : (kBytes ? 34 : 18 + (kAffine ? 2 : 0) + (kFive ? 4 : 0));
    constexpr int kQhOff = kAffine ? 4 : 2, kQsOff = kBytes ? 2 : kBlockBytes - 16;
    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * Nib32Lds::bytes];
    __shared__ __attribute__((aligned(16))) float dql[4][8][32], bql[4][8][32];  // per wave: [block][token]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, h = lane >> 5;
    const int tok0 = blockIdx.y * 128 + wave * 32;
    const int wrow = blockIdx.x * 32 + col;
    const bool row_ok = wrow < out_f;
    const uint8_t* wrowp = w + (size_t)(row_ok ? wrow : 0) * bpr;
    const int p = wave;  // this wave unpacks blocks 2p and 2p+1 of the step

    float acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;

    struct Raw {
        v4i q[2];
        uint32_t d[2], mw[2], qh[2];
    };
    auto request_rows = [&](Raw& r, int b) {
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int bi = b * 8 + 2 * p + e;
            const bool in_row = bi < nblk;  // wave-uniform; past the row's end: block 0 again, scale 0
            if (kNv) {
                const uint8_t* nv = wrowp + (size_t)((in_row ? bi : 0) >> 1) * 36;  // 4-byte aligned
                const int hf = (in_row ? bi : 0) & 1;
                r.q[e] = load16_a4(nv + 4 + 16 * hf);
                // the half's two scale bytes; past the row's end both 0 (which decodes to 0)
                r.d[e] = in_row ? ((uint32_t)load_u32(nv) >> (16 * hf)) & 0xFFFFu : 0u;
                r.mw[e] = r.qh[e] = 0u;
                continue;
            }
            const uint8_t* blk = wrowp + (size_t)(in_row ? bi : 0) * kBlockBytes;  // 2-byte aligned
            r.q[e] = kMx ? gload<v4i_a1>(blk + kQsOff) : load16_a2(blk + kQsOff + (kBytes ? 16 * h : 0));
            r.d[e] = in_row ? (kMx ? (uint32_t)gload<uint8_t>(blk) : load_u16(blk)) : (kMx ? 0x100u : 0u);
            r.mw[e] = kAffine && in_row ? load_u16(blk + 2) : 0u;
            r.qh[e] = kFive ? (load_u16(blk + kQhOff) | (load_u16(blk + kQhOff + 2) << 16)) : 0u;
        }
    };
    auto unpack_to = [&](uint8_t* buf, const Raw& r) {
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            v4i out;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                uint32_t c = (uint32_t)r.q[e][k];
                if (!kBytes) c = (c >> (4 * h)) & 0x0F0F0F0Fu;
                if (K == Blk32::IQ4_NL) c = (uint32_t)iq4nl_lookup(c);
                if (kMx || kNv) c = (uint32_t)mxfp4_lookup(c);  // (NVFP4: dwords 0, 1 sub-block 0's K slots 8h .., 2, 3 sub-block 1's)
                if (kFive) c |= spread4_to_bit4(r.qh[e] >> (16 * h + 4 * k));
                out[k] = (int)c;
            }
            *reinterpret_cast<v4i*>(buf + (size_t)(2 * p + e) * 1024 + lane * 16) = out;
            if (h == 0) {
                // (MXFP4: a block past the row's end carries the marker 0x100 instead of a scale byte)
                const float d = kNv ? ue4m3_half(r.d[e] & 0xFFu)
                                    : (kMx ? (r.d[e] < 0x100u ? e8m0_half(r.d[e]) : 0.0f) : f16_bits_to_f32(r.d[e]));
                const float bb = kNv ? ue4m3_half(r.d[e] >> 8)
                                     : (kAffine ? f16_bits_to_f32(r.mw[e])
                                                : (K == Blk32::IQ4_NL || kBytes || kMx ? 0.0f : (kFive ? -16.0f : -8.0f) * d));
                reinterpret_cast<float*>(buf + Nib32Lds::a_off)[col * 8 + 2 * p + e] = d;
                reinterpret_cast<float*>(buf + Nib32Lds::b_off)[col * 8 + 2 * p + e] = bb;
            }
        }
    };
    // activation fragments in the tiled quantizer's order: every load is a contiguous kilobyte
    v4i a[8];
    v4f dt[2], bt[2];  // this lane's token: the step's eight block scales and code sums
    // this wave's group of 32 tokens; a wave wholly past m recomputes the last group (nothing is stored)
    const size_t g = min((size_t)blockIdx.y * 4 + wave, (size_t)(m - 1) / 32);
    auto request_acts = [&](int b) {
        const size_t gb = g * nb + b;
        const int8_t* ap = qs + gb * (8 * 1024) + lane * 16;
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) a[sb] = *reinterpret_cast<const v4i*>(ap + sb * 1024);
        const v4f* dp = reinterpret_cast<const v4f*>(d8 + (gb * 32 + col) * 8);
        const v4f* bp = reinterpret_cast<const v4f*>(bsf + (gb * 32 + col) * 8);
        dt[0] = dp[0];
        dt[1] = dp[1];
        bt[0] = bp[0];
        bt[1] = bp[1];
    };

    Raw raw;
    request_rows(raw, 0);
    unpack_to(lds, raw);
    request_rows(raw, min(1, nb - 1));
    request_acts(0);
    __syncthreads();

    for (int b = 0; b < nb; ++b) {
        const uint8_t* cur = lds + (b & 1) * Nib32Lds::bytes;
        // ---- unpack step b+1 into the other buffer, then ask for step b+2's bytes ----
        unpack_to(lds + ((b + 1) & 1) * Nib32Lds::bytes, raw);
        request_rows(raw, min(b + 2, nb - 1));
        if (h == 0) {
            const float dv[8] = {dt[0].x, dt[0].y, dt[0].z, dt[0].w, dt[1].x, dt[1].y, dt[1].z, dt[1].w};
            const float bv[8] = {bt[0].x, bt[0].y, bt[0].z, bt[0].w, bt[1].x, bt[1].y, bt[1].z, bt[1].w};
#pragma unroll
            for (int sb = 0; sb < 8; ++sb) {
                dql[wave][sb][col] = dv[sb];
                bql[wave][sb][col] = bv[sb];
            }
        }
        const v4f* ap = reinterpret_cast<const v4f*>(cur + Nib32Lds::a_off + col * 32);
        const v4f* bp = reinterpret_cast<const v4f*>(cur + Nib32Lds::b_off + col * 32);
        const v4f a0 = ap[0], a1 = ap[1], b0 = bp[0], b1 = bp[1];
        const float ca[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
        const float cb[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
        const v16i zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) {
            const v4i bf = *reinterpret_cast<const v4i*>(cur + (size_t)sb * 1024 + lane * 16);
            if constexpr (kNv) {
                // lane (token, h) holds sub-block h of the 32 whole; the K = 16 operand wants bytes 8h .. 8h + 7
                // of one sub-block: the swap exchanges lanes 32..63 of its first operand with lanes 0..31 of
                // its second, after which x y are the lane's K slots of sub-block 0 and z w of sub-block 1
                typedef int v2i_ __attribute__((ext_vector_type(2)));
                const auto s0 = __builtin_amdgcn_permlane32_swap(a[sb].x, a[sb].z, false, false);
                const auto s1 = __builtin_amdgcn_permlane32_swap(a[sb].y, a[sb].w, false, false);
                const v2i_ a0 = {(int)s0[0], (int)s1[0]}, a1 = {(int)s0[1], (int)s1[1]}, b0 = {bf.x, bf.y}, b1 = {bf.z, bf.w};
                const v16i r0 = __builtin_amdgcn_mfma_i32_32x32x16_i8(__builtin_bit_cast(long, a0), __builtin_bit_cast(long, b0), zi, 0, 0, 0);
                const v16i r1 = __builtin_amdgcn_mfma_i32_32x32x16_i8(__builtin_bit_cast(long, a1), __builtin_bit_cast(long, b1), zi, 0, 0, 0);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const v4f dq = *reinterpret_cast<const v4f*>(&dql[wave][sb][8 * j + 4 * h]);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int ri = 4 * j + i;
                        // d8 * (d_0 * iprod_0 + d_1 * iprod_1)
                        const float t = __builtin_fmaf(cb[sb], (float)r1[ri], ca[sb] * (float)r0[ri]);
                        acc[ri] = __builtin_fmaf(dq[i], t, acc[ri]);
                    }
                }
                continue;
            }
            const v16i r = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[sb], bf, zi, 0, 0, 0);
            // accumulator i of this lane is token 8*(i/4) + 4*h + i%4 of the wave's 32
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const v4f dq = *reinterpret_cast<const v4f*>(&dql[wave][sb][8 * j + 4 * h]);
                const v4f bq = *reinterpret_cast<const v4f*>(&bql[wave][sb][8 * j + 4 * h]);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int ri = 4 * j + i;
                    if (STAGES) {
                        const int tok = tok0 + 8 * j + 4 * h + i;
                        if (row_ok && tok < m && b * 8 + sb < nblk) st_iprod[((size_t)tok * out_f + wrow) * nblk + b * 8 + sb] = r[ri];
                    }
                    // d8 * (A * iprod + B * bsum)
                    const float t = __builtin_fmaf(cb[sb], bq[i], ca[sb] * (float)r[ri]);
                    acc[ri] = __builtin_fmaf(dq[i], t, acc[ri]);
                }
            }
        }
        // the activation registers are free: fetch step b+1
        request_acts(min(b + 1, nb - 1));
        __syncthreads();
    }

    if (!row_ok) return;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int tok = tok0 + 8 * (r >> 2) + 4 * h + (r & 3);
        if (tok < m) y[(size_t)tok * out_f + wrow] = acc[r];
    }
}

// Q2_0 (64 weights per 18-byte block [f16 d][16 bytes of 2-bit codes], weight = (code - 1) * d, two
// per-32 activation sub-blocks per block; crates/infr-cpu/src/kernels.rs:5641-5668): the same kernel
// with A = d, B = -d for both sub-blocks of a block. Code j of a block sits in bits 2(j % 4) of byte
// j / 4, so one dword of codes is 16 elements and (dword >> 2i) & 0x03030303 is elements i, 4 + i,
// 8 + i, 12 + i: the activations arrive in that order inside every 16 (the transposed16 quantizer).
// Wave w unpacks block w of the step (sub-blocks 2w, 2w+1); lane (row, h) takes dword 2e + h.
template <bool STAGES>
__global__ __launch_bounds__(256) void mmq_shared_q2_0_kernel(
    const uint8_t* __restrict__ w, size_t bpr, const int8_t* __restrict__ qs, const float* __restrict__ d8,
    const float* __restrict__ bsf, float* __restrict__ y, int m, int out_f, int nb, int nblk,
    int32_t* __restrict__ st_iprod) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * Nib32Lds::bytes];
    __shared__ __attribute__((aligned(16))) float dql[4][8][32], bql[4][8][32];  // per wave: [sub-block][token]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, h = lane >> 5;
    const int tok0 = blockIdx.y * 128 + wave * 32;
    const int wrow = blockIdx.x * 32 + col;
    const bool row_ok = wrow < out_f;
    const uint8_t* wrowp = w + (size_t)(row_ok ? wrow : 0) * bpr;
    const int p = wave;

    float acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;

    struct Raw {
        uint32_t c[2], d;
    };
    auto request_rows = [&](Raw& r, int b) {
        const bool in_row = (b * 4 + p) * 2 < nblk;  // nblk counts 32-element sub-blocks
        const uint8_t* blk = wrowp + (size_t)(in_row ? b * 4 + p : 0) * 18;  // 2-byte aligned
        r.d = in_row ? load_u16(blk) : 0u;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const uint8_t* cp = blk + 2 + 8 * e + 4 * h;
            r.c[e] = load_u16(cp) | (load_u16(cp + 2) << 16);
        }
    };
    auto unpack_to = [&](uint8_t* buf, const Raw& r) {
        const float d = f16_bits_to_f32(r.d);
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            v4i out;
#pragma unroll
            for (int i = 0; i < 4; ++i) out[i] = (int)((r.c[e] >> (2 * i)) & 0x03030303u);
            *reinterpret_cast<v4i*>(buf + (size_t)(2 * p + e) * 1024 + lane * 16) = out;
            if (h == 0) {
                reinterpret_cast<float*>(buf + Nib32Lds::a_off)[col * 8 + 2 * p + e] = d;
                reinterpret_cast<float*>(buf + Nib32Lds::b_off)[col * 8 + 2 * p + e] = -d;
            }
        }
    };
    v4i a[8];
    v4f dt[2], bt[2];
    const size_t g = min((size_t)blockIdx.y * 4 + wave, (size_t)(m - 1) / 32);
    auto request_acts = [&](int b) {
        const size_t gb = g * nb + b;
        const int8_t* ap = qs + gb * (8 * 1024) + lane * 16;
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) a[sb] = *reinterpret_cast<const v4i*>(ap + sb * 1024);
        const v4f* dp = reinterpret_cast<const v4f*>(d8 + (gb * 32 + col) * 8);
        const v4f* bp = reinterpret_cast<const v4f*>(bsf + (gb * 32 + col) * 8);
        dt[0] = dp[0];
        dt[1] = dp[1];
        bt[0] = bp[0];
        bt[1] = bp[1];
    };

    Raw raw;
    request_rows(raw, 0);
    unpack_to(lds, raw);
    request_rows(raw, min(1, nb - 1));
    request_acts(0);
    __syncthreads();

    for (int b = 0; b < nb; ++b) {
        const uint8_t* cur = lds + (b & 1) * Nib32Lds::bytes;
        unpack_to(lds + ((b + 1) & 1) * Nib32Lds::bytes, raw);
        request_rows(raw, min(b + 2, nb - 1));
        if (h == 0) {
            const float dv[8] = {dt[0].x, dt[0].y, dt[0].z, dt[0].w, dt[1].x, dt[1].y, dt[1].z, dt[1].w};
            const float bv[8] = {bt[0].x, bt[0].y, bt[0].z, bt[0].w, bt[1].x, bt[1].y, bt[1].z, bt[1].w};
#pragma unroll
            for (int sb = 0; sb < 8; ++sb) {
                dql[wave][sb][col] = dv[sb];
                bql[wave][sb][col] = bv[sb];
            }
        }
        const v4f* ap = reinterpret_cast<const v4f*>(cur + Nib32Lds::a_off + col * 32);
        const v4f* bp = reinterpret_cast<const v4f*>(cur + Nib32Lds::b_off + col * 32);
        const v4f a0 = ap[0], a1 = ap[1], b0 = bp[0], b1 = bp[1];
        const float ca[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
        const float cb[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
        const v16i zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) {
            const v4i bf = *reinterpret_cast<const v4i*>(cur + (size_t)sb * 1024 + lane * 16);
            const v16i r = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[sb], bf, zi, 0, 0, 0);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const v4f dq = *reinterpret_cast<const v4f*>(&dql[wave][sb][8 * j + 4 * h]);
                const v4f bq = *reinterpret_cast<const v4f*>(&bql[wave][sb][8 * j + 4 * h]);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int ri = 4 * j + i;
                    if (STAGES) {
                        const int tok = tok0 + 8 * j + 4 * h + i;
                        if (row_ok && tok < m && b * 8 + sb < nblk) st_iprod[((size_t)tok * out_f + wrow) * nblk + b * 8 + sb] = r[ri];
                    }
                    const float t = __builtin_fmaf(cb[sb], bq[i], ca[sb] * (float)r[ri]);
                    acc[ri] = __builtin_fmaf(dq[i], t, acc[ri]);
                }
            }
        }
        request_acts(min(b + 1, nb - 1));
        __syncthreads();
    }

    if (!row_ok) return;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int tok = tok0 + 8 * (r >> 2) + 4 * h + (r & 3);
        if (tok < m) y[(size_t)tok * out_f + wrow] = acc[r];
    }
}

template <Blk32 K>
static void launch_nib32(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m, size_t in_f,
                         size_t out_f, const IntStages& st, hipStream_t stream) {
    const dim3 grid((unsigned)((out_f + 31) / 32), (unsigned)((m + 127) / 128)), block(256);
    const int nb = (int)((in_f + 255) / 256), nblk = (int)(in_f / 32);
    const float* bsf = reinterpret_cast<const float*>(act.bsums);
    if (st.a)
        hipLaunchKernelGGL((mmq_shared_nib32_kernel<K, true>), grid, block, 0, stream, w, bpr, act.qs, act.d, bsf, y,
                           (int)m, (int)out_f, nb, nblk, st.a);
    else
        hipLaunchKernelGGL((mmq_shared_nib32_kernel<K, false>), grid, block, 0, stream, w, bpr, act.qs, act.d, bsf, y,
                           (int)m, (int)out_f, nb, nblk, (int32_t*)nullptr);
}

bool launch_mmq_shared_nib32(int dtype, const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m,
                             size_t in_f, size_t out_f, const IntStages& st, hipStream_t stream) {
    switch (dtype) {
    case 2: launch_nib32<Blk32::Q4_0>(w, bpr, act, y, m, in_f, out_f, st, stream); return true;
    case 3: launch_nib32<Blk32::Q4_1>(w, bpr, act, y, m, in_f, out_f, st, stream); return true;
    case 6: launch_nib32<Blk32::Q5_0>(w, bpr, act, y, m, in_f, out_f, st, stream); return true;
    case 7: launch_nib32<Blk32::Q5_1>(w, bpr, act, y, m, in_f, out_f, st, stream); return true;
    case 20: launch_nib32<Blk32::IQ4_NL>(w, bpr, act, y, m, in_f, out_f, st, stream); return true;
    case 39: launch_nib32<Blk32::MXFP4>(w, bpr, act, y, m, in_f, out_f, st, stream); return true;
    case 40:
        if (st.a || in_f % 64 != 0) return false;  // (no integer-stage form: four integers per block)
        launch_nib32<Blk32::NVFP4>(w, bpr, act, y, m, in_f, out_f, st, stream);
        return true;
    case 8: launch_nib32<Blk32::Q8_0>(w, bpr, act, y, m, in_f, out_f, st, stream); return true;
    case 42: {
        const dim3 grid((unsigned)((out_f + 31) / 32), (unsigned)((m + 127) / 128)), block(256);
        const float* bsf = reinterpret_cast<const float*>(act.bsums);
        if (st.a)
            hipLaunchKernelGGL((mmq_shared_q2_0_kernel<true>), grid, block, 0, stream, w, bpr, act.qs, act.d, bsf, y,
                               (int)m, (int)out_f, (int)((in_f + 255) / 256), (int)(in_f / 32), st.a);
        else
            hipLaunchKernelGGL((mmq_shared_q2_0_kernel<false>), grid, block, 0, stream, w, bpr, act.qs, act.d, bsf, y,
                               (int)m, (int)out_f, (int)((in_f + 255) / 256), (int)(in_f / 32), (int32_t*)nullptr);
        return true;
    }
    default: return false;
    }
}

}  // namespace infr
