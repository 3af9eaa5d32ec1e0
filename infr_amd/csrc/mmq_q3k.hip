// Prefill GEMM of Q3_K, TQ2_0 and TQ1_0 weights on the int8 matrix cores, 128 tokens x 32 weight rows
// per workgroup. Q3_K and TQ2_0 keep 2-bit fields in the Q2_K arrangement - element 32 sb + 16 h + l of a
// block is bit pair sb % 4 of byte qs[32 (sb / 4) + 16 h + l] - and both reduce a block to ONE
// chain of eight v_mfma_i32_32x32x32_i8 (the accumulators carry from sub-block to sub-block), with
// nothing per group left to do on the outputs:
//
// Q3_K (crates/infr-cpu/src/kernels.rs:812-852; scales :764-783), 16 groups of 16 elements:
//     isum = sum_g (sc6_g - 32) * sum_l (code - 4) * q8        y += d * q8.d[b] * (f32)isum
// with code = the 2-bit field plus 4 where bit sb of hmask[16 h + l] is set. (4 - code) * (sc6 - 32)
// lies in [-128, 124], an int8 operand (code - 4 times the scale would reach +128): the unpack
// looks the product up in an eight-entry byte table built per group from its scale, and the chain
// gives -isum.
//
// TQ2_0 (kernels.rs:3066-3126): the ternary weight q - 1 is the operand as it is;
//     iprod = sum_l (q - 1) * q8                               y += d * q8.d[b] * (f32)iprod
//
// Integers exact, the f32 epilogue the CPU's expression, blocks in ascending order: y equals
// infr-cpu's batch kernels and the one-token GEMV bit for bit. Tiling, LDS double-buffering and
// the tiled activation layout are the other shared-operand kernels' (mmq_q5k.hip).
#include "device_common.hpp"
#include "kernels.hpp"

namespace infr {

typedef int v16i __attribute__((ext_vector_type(16)));

// LDS of one block: B operands [sub-block][lane] x 16 B | d [row]
struct ChainLds {
    static constexpr int d_off = 8 * 1024;
    static constexpr int bytes = d_off + 32 * 4;
};

struct TileQ3K {
    static constexpr int kBlockBytes = 110;
    static constexpr bool kNegate = true;
    struct Raw {
        v4i q, hm;
        uint32_t sc[3];
        uint32_t d;
    };
    __device__ static void load(Raw& r, const uint8_t* blk, int p, int h) {  // 2-byte aligned
        r.hm = load16_a2(blk + 16 * h);
        r.q = load16_a2(blk + 32 + 32 * (p >> 1) + 16 * h);
#pragma unroll
        for (int i = 0; i < 3; ++i) r.sc[i] = (uint32_t)gload<int_a2>(blk + 96 + 4 * i);
        r.d = load_u16(blk + 108);
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
    // The 16 operand bytes of sub-block 2p + e for this lane's elements 16h .. 16h + 15 (group 2 (2p + e) + h).
    __device__ static v4i operand(const Raw& r, int p, int e, int h) {
        const int n = p >> 1, j = 2 * (p & 1) + e;
        // scale field 8 n + 2 j + h: low nibble in nibble n of byte 2 j + h of the first eight, top two
        // bits at bit 4 n + 2 (j / 2) of byte 8 + 2 (j % 2) + h
        const int sh = 8 * h + 4 * n;
        const uint32_t lo4 = ((j < 2 ? r.sc[0] : r.sc[1]) >> (sh + 16 * (j & 1))) & 15u;
        const uint32_t hi2 = (r.sc[2] >> (sh + 16 * (j & 1) + 2 * (j >> 1))) & 3u;
        const uint32_t u = lo4 | (hi2 << 4);
        // table[v] = (4 - v) * (u - 32) as int8, v = 0..3 in t_lo, 4..7 in t_hi
        const uint32_t t_lo = sub_bytes(mul_bytes(0x01020304u, u), 0x20406000u, 0x80808000u);
        const uint32_t t_hi = sub_bytes(mul_bytes(0x03020100u, 64u - u), 0x60402000u, 0x80808080u);
        v4i out;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t low2 = ((uint32_t)r.q[k] >> (2 * j)) & 0x03030303u;
            const uint32_t high = ((uint32_t)r.hm[k] >> (4 * n + j)) & 0x01010101u;
            out[k] = (int)__builtin_amdgcn_perm(t_hi, t_lo, low2 | (high << 2));
        }
        return out;
    }
};

struct TileTQ2_0 {
    static constexpr int kBlockBytes = 66;
    static constexpr bool kNegate = false;
    struct Raw {
        v4i q;
        uint32_t d;
    };
    __device__ static void load(Raw& r, const uint8_t* blk, int p, int h) {  // 2-byte aligned
        r.q = load16_a2(blk + 32 * (p >> 1) + 16 * h);
        r.d = load_u16(blk + 64);
    }
    __device__ static v4i operand(const Raw& r, int p, int e, int) {
        const int sh = 2 * (2 * (p & 1) + e);
        v4i out;
#pragma unroll
        for (int k = 0; k < 4; ++k)  // q - 1 per byte: q + 0x7F stays inside the byte, flipping bit 7 gives q - 1
            out[k] = (int)(((((uint32_t)r.q[k] >> sh) & 0x03030303u) + 0x7F7F7F7Fu) ^ 0x80808080u);
        return out;
    }
};

// TQ1_0 (54-byte block: qs[48], qh[4], d; kernels.rs:3167-3240): base-3 packed ternary digits, weight
// (digit - 1) d. Digit n of a byte is the high byte of three times (byte * 3^n mod 256). Elements
// come in three runs - qs[0..32) x 5 digits -> 32 n + m, qs[32..48) x 5 -> 160 + 16 n + m, qh[0..4) x 4
// -> 240 + 4 n + j - so the 16 elements 32 sb + 16 h .. of lane (row, h) are digit sb of
// qs[16 h .. 16 h + 15] for sb < 5; digit 2 (sb - 5) + h of qs[32..47] for sb = 5, 6; digit 4 of
// qs[32..47] (h = 0) or digits 0..3 of the four qh bytes (h = 1) for sb = 7. The digits are taken
// out once per 128 tokens; digit - 1 is the operand and the block one chain, as for TQ2_0.
struct TileTQ1_0 {
    static constexpr int kBlockBytes = 54;
    static constexpr bool kNegate = false;
    struct Raw {
        v4i qa, qb;
        uint32_t qh, d;
    };
    __device__ static void load(Raw& r, const uint8_t* blk, int, int h) {  // 2-byte aligned
        r.qa = load16_a2(blk + 16 * h);
        r.qb = load16_a2(blk + 32);
        r.qh = (uint32_t)gload<int_a2>(blk + 48);
        r.d = load_u16(blk + 52);
    }
    // The five digits of each of a word's four bytes: out[n] holds digit n of byte k in byte k
    // (even and odd bytes in the two halves of a word: three times a byte fits 16 bits).
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
    __device__ static uint32_t pick(const uint32_t (&dg)[5], int n) {
        return n == 0 ? dg[0] : (n == 1 ? dg[1] : (n == 2 ? dg[2] : (n == 3 ? dg[3] : dg[4])));
    }
    __device__ static v4i operand(const Raw& r, int p, int e, int h) {
        const int sb = 2 * p + e;
        const v4i src = sb < 5 ? r.qa : r.qb;
        const int n = sb < 5 ? sb : (sb == 7 ? 4 : 2 * (sb - 5) + h);
        uint32_t dg[5];
        v4i out;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            digits5((uint32_t)src[k], dg);
            out[k] = (int)pick(dg, n);
        }
        if (sb == 7 && h == 1) {  // the last 16 elements: digit k of the four qh bytes
            digits5(r.qh, dg);
            out = v4i{(int)dg[0], (int)dg[1], (int)dg[2], (int)dg[3]};
        }
#pragma unroll
        for (int k = 0; k < 4; ++k)  // digit - 1 per byte
            out[k] = (int)(((uint32_t)out[k] + 0x7F7F7F7Fu) ^ 0x80808080u);
        return out;
    }
};

template <typename T, bool STAGES>
__global__ __launch_bounds__(256) void mmq_shared_chain_kernel(
    const uint8_t* __restrict__ w, size_t bpr, const int8_t* __restrict__ qs, const float* __restrict__ d8,
    float* __restrict__ y, int m, int out_f, int nb, int32_t* __restrict__ st_isum) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * ChainLds::bytes];
    __shared__ __attribute__((aligned(16))) float dql[4][32];  // per wave: its tokens' activation scales
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, h = lane >> 5;
    const int tok0 = blockIdx.y * 128 + wave * 32;
    const int wrow = blockIdx.x * 32 + col;
    const bool row_ok = wrow < out_f;
    const uint8_t* wrowp = w + (size_t)(row_ok ? wrow : 0) * bpr;
    const int p = wave;  // the sub-block pair (2p, 2p+1) this wave unpacks

    float acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;

    typename T::Raw raw;
    auto unpack_to = [&](uint8_t* buf, const typename T::Raw& r) {
#pragma unroll
        for (int e = 0; e < 2; ++e)
            *reinterpret_cast<v4i*>(buf + (size_t)(2 * p + e) * 1024 + lane * 16) = T::operand(r, p, e, h);
        if (p == 0 && h == 0) reinterpret_cast<float*>(buf + ChainLds::d_off)[col] = f16_bits_to_f32(r.d);
    };
    // activation fragments in the tiled quantizer's order: every load is a contiguous kilobyte
    v4i a[8];
    float dtok;
    // this wave's group of 32 tokens; a wave wholly past m recomputes the last group (nothing is stored)
    const size_t g = min((size_t)blockIdx.y * 4 + wave, (size_t)(m - 1) / 32);
    auto request_acts = [&](int b) {
        const size_t gb = g * nb + b;
        const int8_t* ap = qs + gb * (8 * 1024) + lane * 16;
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) a[sb] = *reinterpret_cast<const v4i*>(ap + sb * 1024);
        dtok = d8[gb * 32 + col];
    };

    T::load(raw, wrowp, p, h);
    unpack_to(lds, raw);
    T::load(raw, wrowp + (size_t)min(1, nb - 1) * T::kBlockBytes, p, h);
    request_acts(0);
    __syncthreads();

    for (int b = 0; b < nb; ++b) {
        const uint8_t* cur = lds + (b & 1) * ChainLds::bytes;
        // ---- unpack block b+1 into the other buffer, then ask for block b+2's bytes ----
        unpack_to(lds + ((b + 1) & 1) * ChainLds::bytes, raw);
        T::load(raw, wrowp + (size_t)min(b + 2, nb - 1) * T::kBlockBytes, p, h);
        if (h == 0) dql[wave][col] = dtok;
        v16i isum = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) {
            const v4i bf = *reinterpret_cast<const v4i*>(cur + (size_t)sb * 1024 + lane * 16);
            isum = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[sb], bf, isum, 0, 0, 0);
        }
        // the activation registers are free: fetch block b+1 while the epilogue runs
        request_acts(min(b + 1, nb - 1));
        const float d = reinterpret_cast<const float*>(cur + ChainLds::d_off)[col];
        // accumulator i of this lane is token 8*(i/4) + 4*h + i%4 of the wave's 32
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const v4f dq = *reinterpret_cast<const v4f*>(&dql[wave][8 * j + 4 * h]);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int r = 4 * j + i;
                const int v = T::kNegate ? -isum[r] : isum[r];
                if (STAGES) {
                    const int tok = tok0 + 8 * j + 4 * h + i;
                    if (row_ok && tok < m) st_isum[((size_t)tok * out_f + wrow) * nb + b] = v;
                }
                acc[r] += (d * dq[i]) * (float)v;  // sumf += d * q8.d[b] * isum as f32
            }
        }
        __syncthreads();
    }

    if (!row_ok) return;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int tok = tok0 + 8 * (r >> 2) + 4 * h + (r & 3);
        if (tok < m) y[(size_t)tok * out_f + wrow] = acc[r];
    }
}

template <typename T>
static void launch_chain(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m, size_t in_f, size_t out_f,
                         const IntStages& st, hipStream_t stream) {
    const dim3 grid((unsigned)((out_f + 31) / 32), (unsigned)((m + 127) / 128)), block(256);
    const int nb = (int)(in_f / 256);
    if (st.a)
        hipLaunchKernelGGL((mmq_shared_chain_kernel<T, true>), grid, block, 0, stream, w, bpr, act.qs, act.d, y, (int)m,
                           (int)out_f, nb, st.a);
    else
        hipLaunchKernelGGL((mmq_shared_chain_kernel<T, false>), grid, block, 0, stream, w, bpr, act.qs, act.d, y, (int)m,
                           (int)out_f, nb, (int32_t*)nullptr);
}

void launch_mmq_shared_q3k(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m, size_t in_f,
                           size_t out_f, const IntStages& st, hipStream_t stream) {
    launch_chain<TileQ3K>(w, bpr, act, y, m, in_f, out_f, st, stream);
}
void launch_mmq_shared_tq2_0(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m, size_t in_f,
                             size_t out_f, const IntStages& st, hipStream_t stream) {
    launch_chain<TileTQ2_0>(w, bpr, act, y, m, in_f, out_f, st, stream);
}

void launch_mmq_shared_tq1_0(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m, size_t in_f,
                             size_t out_f, const IntStages& st, hipStream_t stream) {
    launch_chain<TileTQ1_0>(w, bpr, act, y, m, in_f, out_f, st, stream);
}

}  // namespace infr
