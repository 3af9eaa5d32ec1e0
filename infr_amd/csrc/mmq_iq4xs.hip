// Prefill GEMM of IQ4_XS weights on the int8 matrix cores, 128 tokens x 32 weight rows per workgroup.
//
// Per 256-element block infr-cpu computes, per output (crates/infr-cpu/src/kernels.rs:995-1036,
// vec_dot_iq4xs),
//     isum = sum_ib (ls_ib - 32) * (sum_l kvalues_iq4nl[q] * q8)
//     y += d * q8.d[b] * (f32)isum
// with a 6-bit ls per 32-element sub-block and 4-bit indices into IQ4_NL's signed table. The table
// values are int8 operands as they stand; a value times its scale (127 * 32) is not, so every
// sub-block is multiplied on its own - one v_mfma_i32_32x32x32_i8 over its 32 elements - and scaled
// into isum with one 24-bit multiply-add per output (|sub-block product| <= 32 * 127 * 127 < 2^23).
// No mins, so no second product; the epilogue is the CPU expression and the blocks are added in
// ascending order: y equals infr-cpu's batch kernel and the one-token GEMV bit for bit.
//
// Tiling, LDS double-buffering and the tiled activation layout are the other shared-operand
// kernels' (mmq_q5k.hip): wave w owns tokens 32w..32w+31 and unpacks sub-blocks 2w, 2w+1 of all 32
// rows - a sub-block is 16 bytes, low nibbles its elements 0..15 and high nibbles 16..31, which are
// the two halves of a 32x32x32 operand column.
#include "device_common.hpp"
#include "gemv_formats.hpp"
#include "kernels.hpp"

namespace infr {

typedef int v16i __attribute__((ext_vector_type(16)));

// LDS of one block: B operands [sub-block][lane] x 16 B | scales [row][8] i8 | d [row]
struct Iq4xsLds {
    static constexpr int sc_off = 8 * 1024;
    static constexpr int d_off = sc_off + 32 * 8;
    static constexpr int bytes = d_off + 32 * 4;
};

template <bool STAGES>
__global__ __launch_bounds__(256) void mmq_shared_iq4xs_kernel(
    const uint8_t* __restrict__ w, size_t bpr, const int8_t* __restrict__ qs, const float* __restrict__ d8,
    float* __restrict__ y, int m, int out_f, int nb, int32_t* __restrict__ st_isum) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * Iq4xsLds::bytes];
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

    struct Raw {
        v2i hdr;
        v4i q0, q1;
    };
    auto request_rows = [&](Raw& r, int b) {
        const uint8_t* blk = wrowp + (size_t)b * 136;  // 8-byte aligned
        r.hdr = gload<v2i>(blk);
        r.q0 = load16_a4(blk + 8 + p * 32);
        r.q1 = load16_a4(blk + 24 + p * 32);
    };
    auto unpack_to = [&](uint8_t* buf, const Raw& r) {
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const v4i q = e ? r.q1 : r.q0;
            v4i out;
#pragma unroll
            for (int k = 0; k < 4; ++k) out[k] = iq4nl_lookup(((uint32_t)q[k] >> (4 * h)) & 0x0F0F0F0Fu);
            *reinterpret_cast<v4i*>(buf + (size_t)(2 * p + e) * 1024 + lane * 16) = out;
        }
        if (p == 0 && h == 0) {
            const uint32_t sh = (uint32_t)r.hdr.x >> 16, sl = (uint32_t)r.hdr.y;
            uint32_t sc[2] = {0, 0};
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                const int ls = (int)(((sl >> (4 * s)) & 0xFu) | (((sh >> (2 * s)) & 3u) << 4)) - 32;
                sc[s >> 2] |= ((uint32_t)ls & 0xFFu) << (8 * (s & 3));
            }
            uint32_t* scp = reinterpret_cast<uint32_t*>(buf + Iq4xsLds::sc_off + col * 8);
            scp[0] = sc[0];
            scp[1] = sc[1];
            reinterpret_cast<float*>(buf + Iq4xsLds::d_off)[col] = f16_bits_to_f32((uint32_t)r.hdr.x & 0xFFFFu);
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
        const uint8_t* cur = lds + (b & 1) * Iq4xsLds::bytes;
        // ---- unpack block b+1 into the other buffer, then ask for block b+2's bytes ----
        unpack_to(lds + ((b + 1) & 1) * Iq4xsLds::bytes, raw);
        request_rows(raw, min(b + 2, nb - 1));
        if (h == 0) dql[wave][col] = dtok;
        const uint32_t* scp = reinterpret_cast<const uint32_t*>(cur + Iq4xsLds::sc_off + col * 8);
        const uint32_t scw[2] = {scp[0], scp[1]};
        const v16i zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        int isum[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) isum[i] = 0;
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) {
            const v4i bf = *reinterpret_cast<const v4i*>(cur + (size_t)sb * 1024 + lane * 16);
            const v16i r = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[sb], bf, zi, 0, 0, 0);
            const int sc = (int)(scw[sb >> 2] << (24 - 8 * (sb & 3))) >> 24;  // ls - 32, signed
#pragma unroll
            for (int i = 0; i < 16; ++i) isum[i] += __mul24(r[i], sc);
        }
        // the activation registers are free: fetch block b+1 while the epilogue runs
        request_acts(min(b + 1, nb - 1));
        const float d = reinterpret_cast<const float*>(cur + Iq4xsLds::d_off)[col];
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
                acc[r] += (d * dq[i]) * (float)isum[r];  // sumf += d * q8.d[b] * isum as f32
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

void launch_mmq_shared_iq4xs(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m, size_t in_f,
                             size_t out_f, const IntStages& st, hipStream_t stream) {
    const dim3 grid((unsigned)((out_f + 31) / 32), (unsigned)((m + 127) / 128)), block(256);
    const int nb = (int)(in_f / 256);
    if (st.a)
        hipLaunchKernelGGL((mmq_shared_iq4xs_kernel<true>), grid, block, 0, stream, w, bpr, act.qs, act.d, y, (int)m,
                           (int)out_f, nb, st.a);
    else
        hipLaunchKernelGGL((mmq_shared_iq4xs_kernel<false>), grid, block, 0, stream, w, bpr, act.qs, act.d, y, (int)m,
                           (int)out_f, nb, (int32_t*)nullptr);
}

}  // namespace infr
