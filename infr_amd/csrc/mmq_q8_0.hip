// Prefill GEMM (33 tokens and up) of Q8_0 weights on the int8 matrix cores, for rows that are whole
// 256s (the activation then carries one scale per 256, crates/infr-cpu/src/lib.rs:1042-1062).
//
// Per 32-weight block infr-cpu adds (d8 * d_w) * (f32)iprod, iprod = sum_l q_w * q_x, blocks in
// order (crates/infr-cpu/src/kernels.rs:1170-1187). The codes are int8 operands as stored - no
// unpack at all - so iprod is one v_mfma_i32_32x32x32_i8 per block, exact. The f32 side is
// evaluated as d8 * sum_{8 blocks} d_w * (f32)iprod per 256 elements (one conversion and one FMA
// per output and block, one more FMA per 256): the same terms in a different association, as the
// one-token Q8_0 kernel already differs from the CPU by its butterfly sum; results agree with the
// oracle to ~1e-7 relative, far inside the path's 1e-4 gate, and the per-block integers bit for bit.
//
// Tiling as the other shared-operand kernels: 128 tokens x 32 weight rows per workgroup, wave w owns
// tokens 32w..32w+31 and copies blocks 2w, 2w+1 of every row of a 256-element step into LDS in MFMA
// B order (double-buffered, one barrier per step); activation fragments come from the tiled
// quantizer's layout.
#include "device_common.hpp"
#include "kernels.hpp"

namespace infr {

typedef int v16i __attribute__((ext_vector_type(16)));

// LDS of one 256-element step: B operands [block][lane] x 16 B | block scales [row][8] f32
struct Q80Lds {
    static constexpr int d_off = 8 * 1024;
    static constexpr int bytes = d_off + 32 * 8 * 4;
};

template <bool STAGES>
__global__ __launch_bounds__(256) void mmq_shared_q8_0_kernel(
    const uint8_t* __restrict__ w, size_t bpr, const int8_t* __restrict__ qs, const float* __restrict__ d8,
    float* __restrict__ y, int m, int out_f, int nb, int32_t* __restrict__ st_iprod) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * Q80Lds::bytes];
    __shared__ __attribute__((aligned(16))) float dql[4][32];  // per wave: its tokens' activation scales
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, h = lane >> 5;
    const int tok0 = blockIdx.y * 128 + wave * 32;
    const int wrow = blockIdx.x * 32 + col;
    const bool row_ok = wrow < out_f;
    const uint8_t* wrowp = w + (size_t)(row_ok ? wrow : 0) * bpr;
    const int p = wave;  // this wave stages blocks 2p and 2p+1 of the step

    float acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;

    struct Raw {
        v4i q[2];
        uint32_t d[2];
    };
    auto request_rows = [&](Raw& r, int b) {
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const uint8_t* blk = wrowp + ((size_t)b * 8 + 2 * p + e) * 34;  // 2-byte aligned
            r.q[e] = load16_a2(blk + 2 + 16 * h);
            r.d[e] = load_u16(blk);
        }
    };
    auto stage_to = [&](uint8_t* buf, const Raw& r) {
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            *reinterpret_cast<v4i*>(buf + (size_t)(2 * p + e) * 1024 + lane * 16) = r.q[e];
            if (h == 0) reinterpret_cast<float*>(buf + Q80Lds::d_off)[col * 8 + 2 * p + e] = f16_bits_to_f32(r.d[e]);
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
    stage_to(lds, raw);
    request_rows(raw, min(1, nb - 1));
    request_acts(0);
    __syncthreads();

    for (int b = 0; b < nb; ++b) {
        const uint8_t* cur = lds + (b & 1) * Q80Lds::bytes;
        // ---- stage step b+1 into the other buffer, then ask for step b+2's bytes ----
        stage_to(lds + ((b + 1) & 1) * Q80Lds::bytes, raw);
        request_rows(raw, min(b + 2, nb - 1));
        if (h == 0) dql[wave][col] = dtok;
        const v4f dwa = *reinterpret_cast<const v4f*>(cur + Q80Lds::d_off + col * 32);
        const v4f dwb = *reinterpret_cast<const v4f*>(cur + Q80Lds::d_off + col * 32 + 16);
        const float dw[8] = {dwa.x, dwa.y, dwa.z, dwa.w, dwb.x, dwb.y, dwb.z, dwb.w};
        const v16i zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        float part[16];  // sum over the step's eight blocks of d_w * iprod
#pragma unroll
        for (int i = 0; i < 16; ++i) part[i] = 0.0f;
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) {
            const v4i bf = *reinterpret_cast<const v4i*>(cur + (size_t)sb * 1024 + lane * 16);
            const v16i r = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[sb], bf, zi, 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                if (STAGES) {
                    // accumulator i of this lane is token 8*(i/4) + 4*h + i%4 of the wave's 32
                    const int tok = tok0 + 8 * (i >> 2) + 4 * h + (i & 3);
                    if (row_ok && tok < m) st_iprod[((size_t)tok * out_f + wrow) * (nb * 8) + b * 8 + sb] = r[i];
                }
                part[i] = __builtin_fmaf(dw[sb], (float)r[i], part[i]);
            }
        }
        // the activation registers are free: fetch step b+1 while the epilogue runs
        request_acts(min(b + 1, nb - 1));
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const v4f dq = *reinterpret_cast<const v4f*>(&dql[wave][8 * j + 4 * h]);
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[4 * j + i] = __builtin_fmaf(dq[i], part[4 * j + i], acc[4 * j + i]);
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

void launch_mmq_shared_q8_0(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m, size_t in_f,
                            size_t out_f, const IntStages& st, hipStream_t stream) {
    const dim3 grid((unsigned)((out_f + 31) / 32), (unsigned)((m + 127) / 128)), block(256);
    const int nb = (int)(in_f / 256);
    if (st.a)
        hipLaunchKernelGGL((mmq_shared_q8_0_kernel<true>), grid, block, 0, stream, w, bpr, act.qs, act.d, y, (int)m,
                           (int)out_f, nb, st.a);
    else
        hipLaunchKernelGGL((mmq_shared_q8_0_kernel<false>), grid, block, 0, stream, w, bpr, act.qs, act.d, y, (int)m,
                           (int)out_f, nb, (int32_t*)nullptr);
}

}  // namespace infr
