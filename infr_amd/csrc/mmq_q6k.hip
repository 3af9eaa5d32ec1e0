// Prefill GEMM (33 tokens and up) of Q6_K weights on the int8 matrix cores.
//
// Per 256-element block infr-cpu computes, per output (crates/infr-cpu/src/kernels.rs:487-526),
//     isum = sum_g sc_g * (sum_l q * q8 - 32 * bsum16_g)        16 groups g of 16 elements
//     y   += (d * q8.d[b]) * (f32)isum
// with an int8 scale sc_g per group. q - 32 (in -32..31) is an int8 operand as it is, so
// sum_l (q - 32) * q8 comes straight out of the matrix cores; what cannot is the scale: (q - 32) *
// sc_g needs 13 bits. A group is therefore multiplied on its own - one v_mfma_i32_32x32x16_i8 per
// group (the K = 16 form takes half the passes of the K = 32 one, which a group would only half
// fill) - and scaled into the block's isum with one 24-bit multiply-add per output. The tiled
// activation layout gives lane (token, h) elements 16h..16h+15 of a 32-element sub-block, i.e. the
// whole of group h, where the K = 16 operand wants bytes 8h..8h+7 of one group: two
// v_permlane32_swap per sub-block exchange the upper dwords of the h = 0 lanes with the lower
// dwords of the h = 1 lanes, after which a lane's first eight bytes are its share of the even
// group and its last eight of the odd one. isum is the CPU's integer, the f32 epilogue is the CPU's expression
// and the blocks are added in ascending order, so y equals infr-cpu's batch kernel (and this
// library's m == 1 GEMV) bit for bit.
//
// Tiling as the Q4_K shared-operand kernel: a workgroup covers 128 tokens x 32 weight rows, wave w
// owns tokens 32w..32w+31; tokens are the MFMA's M and weight rows its N, so a lane's 16
// accumulators share one weight row and sc_g, d are per lane. Wave w unpacks sub-blocks 2w and 2w+1
// of all 32 rows into LDS in MFMA B order (double-buffered, block b+1 while block b is multiplied,
// one barrier per block); activation fragments come from the tiled quantizer's layout, one
// contiguous kilobyte per load.
#include "device_common.hpp"
#include "kernels.hpp"

namespace infr {

typedef int v16i __attribute__((ext_vector_type(16)));

// LDS of one block: B operands [sub-block][lane] x (8 B of the even group | 8 B of the odd group) |
// group scales [row][16] | d [row]
struct Q6kLds {
    static constexpr int sc_off = 8 * 1024;
    static constexpr int d_off = sc_off + 32 * 16;
    static constexpr int bytes = d_off + 32 * 4;
};

template <bool STAGES>
__global__ __launch_bounds__(256) void mmq_shared_q6k_kernel(
    const uint8_t* __restrict__ w, size_t bpr, const int8_t* __restrict__ qs, const float* __restrict__ d8,
    float* __restrict__ y, int m, int out_f, int nb, int32_t* __restrict__ st_isum) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * Q6kLds::bytes];
    __shared__ __attribute__((aligned(16))) float dql[4][32];  // per wave: its tokens' activation scales
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, h = lane >> 5;
    const int tok0 = blockIdx.y * 128 + wave * 32;
    const int wrow = blockIdx.x * 32 + col;
    const bool row_ok = wrow < out_f;
    const uint8_t* wrowp = w + (size_t)(row_ok ? wrow : 0) * bpr;
    // This wave unpacks sub-blocks s = 2p, 2p+1: half = p / 2 of the block, quarter qd = 2 (p % 2) + e
    // of the half (elements half*128 + 32 qd + l), whose low four bits are a nibble of ql[half*64 +
    // 32 e + l] - the high nibble when p is odd - and whose bits 4, 5 are bits 2qd, 2qd+1 of
    // qh[half*32 + l] (crates/infr-cpu/src/kernels.rs:499-513). This lane takes l = 16h..16h+15.
    const int p = wave, half = p >> 1, nib_shift = 4 * (p & 1);

    v16i isum;
    float acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;

    struct Raw {
        v4i ql[2], qh, sc;
        uint32_t d;
    };
    auto request_rows = [&](Raw& r, int b) {
        const uint8_t* blk = wrowp + (size_t)b * 210;  // 2-byte aligned
        r.ql[0] = load16_a2(blk + half * 64 + 16 * h);
        r.ql[1] = load16_a2(blk + half * 64 + 32 + 16 * h);
        r.qh = load16_a2(blk + 128 + half * 32 + 16 * h);
        r.sc = load16_a2(blk + 192);
        r.d = load_u16(blk + 208);
    };
    auto unpack_to = [&](uint8_t* buf, const Raw& r) {
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int qd_shift = 2 * (2 * (p & 1) + e);
            v4i out;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t nib = ((uint32_t)r.ql[e][k] >> nib_shift) & 0x0F0F0F0Fu;
                const uint32_t hb = ((uint32_t)r.qh[k] >> qd_shift) & 0x03030303u;
                const uint32_t q = (hb << 4) | nib;  // 0..63 per byte
                // q - 32 as a signed byte: q + 0x60 stays inside the byte, flipping bit 7 then gives
                // q - 32 for q >= 32 and 256 + q - 32 below
                out[k] = (int)((q + 0x60606060u) ^ 0x80808080u);
            }
            // this lane holds elements 16h..16h+15 of the sub-block = group 2s + h whole: bytes 0..7
            // are the operand of reader lane (col, 0), bytes 8..15 of reader lane (col, 1), in slot h
            uint8_t* dst = buf + (size_t)(2 * p + e) * 1024 + col * 16 + 8 * h;
            *reinterpret_cast<v2i*>(dst) = v2i{out[0], out[1]};
            *reinterpret_cast<v2i*>(dst + 32 * 16) = v2i{out[2], out[3]};
        }
        if (p == 0 && h == 0) {
            *reinterpret_cast<v4i*>(buf + Q6kLds::sc_off + col * 16) = r.sc;
            reinterpret_cast<float*>(buf + Q6kLds::d_off)[col] = f16_bits_to_f32(r.d);
        }
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

    Raw raw;
    request_rows(raw, 0);
    unpack_to(lds, raw);
    request_rows(raw, min(1, nb - 1));
    request_acts(0);
    __syncthreads();

    for (int b = 0; b < nb; ++b) {
        const uint8_t* cur = lds + (b & 1) * Q6kLds::bytes;
        // ---- unpack block b+1 into the other buffer, then ask for block b+2's bytes ----
        unpack_to(lds + ((b + 1) & 1) * Q6kLds::bytes, raw);
        request_rows(raw, min(b + 2, nb - 1));
        if (h == 0) dql[wave][col] = dtok;
        const v4i scv = *reinterpret_cast<const v4i*>(cur + Q6kLds::sc_off + col * 16);
        const int scw[4] = {scv.x, scv.y, scv.z, scv.w};
        const v16i zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < 16; ++i) isum[i] = 0;
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) {
            // (lane (tok, 0): x y = group 2sb bytes 0..7, z w = bytes 8..15; lane (tok, 1) the same of
            // group 2sb+1) -> x y = the lane's K-slots of group 2sb, z w = of group 2sb+1
            // (the swap exchanges lanes 32..63 of its first operand with lanes 0..31 of its second)
            const auto s0 = __builtin_amdgcn_permlane32_swap(a[sb].x, a[sb].z, false, false);
            const auto s1 = __builtin_amdgcn_permlane32_swap(a[sb].y, a[sb].w, false, false);
            const v2i a0 = {(int)s0[0], (int)s1[0]}, a1 = {(int)s0[1], (int)s1[1]};
            const v4i bf = *reinterpret_cast<const v4i*>(cur + (size_t)sb * 1024 + lane * 16);
            const v2i b0 = {bf.x, bf.y}, b1 = {bf.z, bf.w};
            const v16i r0 = __builtin_amdgcn_mfma_i32_32x32x16_i8(__builtin_bit_cast(long, a0), __builtin_bit_cast(long, b0), zi, 0, 0, 0);
            const v16i r1 = __builtin_amdgcn_mfma_i32_32x32x16_i8(__builtin_bit_cast(long, a1), __builtin_bit_cast(long, b1), zi, 0, 0, 0);
            const int g0 = 2 * sb, g1 = 2 * sb + 1;
            const int sc0 = __builtin_amdgcn_sbfe(scw[g0 >> 2], 8 * (g0 & 3), 8);
            const int sc1 = __builtin_amdgcn_sbfe(scw[g1 >> 2], 8 * (g1 & 3), 8);
#pragma unroll
            for (int i = 0; i < 16; ++i) isum[i] += __mul24(r0[i], sc0) + __mul24(r1[i], sc1);
        }
        // the activation registers are free: fetch block b+1 while the epilogue runs
        request_acts(min(b + 1, nb - 1));
        const float d = reinterpret_cast<const float*>(cur + Q6kLds::d_off)[col];
        // accumulator i of this lane is token 8*(i/4) + 4*h + i%4 of the wave's 32
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const v4f dq = *reinterpret_cast<const v4f*>(&dql[wave][8 * j + 4 * h]);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int r = 4 * j + i;
                if (STAGES) {
                    const int tok = tok0 + 8 * j + 4 * h + i;
                    if (row_ok && tok < m) st_isum[((size_t)tok * out_f + wrow) * nb + b] = isum[r];
                }
                // sumf += d * q8.d[b] * (isum as f32), evaluated (d * q8.d[b]) * isum
                acc[r] += (d * dq[i]) * (float)isum[r];
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

void launch_mmq_shared_q6k(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m, size_t in_f,
                           size_t out_f, const IntStages& st, hipStream_t stream) {
    const dim3 grid((unsigned)((out_f + 31) / 32), (unsigned)((m + 127) / 128)), block(256);
    const int nb = (int)(in_f / 256);
    if (st.a)
        hipLaunchKernelGGL((mmq_shared_q6k_kernel<true>), grid, block, 0, stream, w, bpr, act.qs, act.d, y, (int)m,
                           (int)out_f, nb, st.a);
    else
        hipLaunchKernelGGL((mmq_shared_q6k_kernel<false>), grid, block, 0, stream, w, bpr, act.qs, act.d, y, (int)m,
                           (int)out_f, nb, (int32_t*)nullptr);
}

}  // namespace infr
