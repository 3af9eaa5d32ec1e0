// Prefill GEMM of Q2_K weights on the int8 matrix cores, 128 tokens x 32 weight rows per workgroup.
//
// Per 256-element block infr-cpu computes, per output (crates/infr-cpu/src/kernels.rs, vec_dot_q2k;
// 16 groups g of 16 elements, a 4-bit scale and a 4-bit min each),
//     sd = sum_g sc_g * (sum_l q2 * q8)     sm = sum_g m_g * bsums16_g
//     y += q8.d[b] * (d * (f32)sd - dmin * (f32)sm)
// A 2-bit code times its group's scale is at most 3 * 15 = 45: an int8 operand. The unpack
// therefore stores scaled codes, and the eight 32-element sub-blocks of a block are eight
// v_mfma_i32_32x32x32_i8 chained into one accumulator set - sd comes out of the matrix cores
// whole, with no per-group arithmetic on the outputs. sm is one K = 16 f16 MFMA of the mins against
// the per-16 sums of the activations, which the lanes form from the fragments they already hold
// (a lane's 16 bytes of a sub-block are exactly one group): all products and sums are integers
// below 2^24, exact in f16 operands and f32 accumulators. The epilogue is the CPU expression and
// the blocks are added in ascending order: y equals infr-cpu's batch kernel and the one-token
// GEMV bit for bit.
//
// Element 32 sb + 16 h + l of a block is bit pair sb % 4 of byte qs[32 (sb / 4) + 16 h + l]; its
// group is 2 sb + h. Tiling, LDS double-buffering and the tiled activation layout are the other
// shared-operand kernels' (mmq_q5k.hip): wave w owns tokens 32w..32w+31 and unpacks sub-blocks
// 2w, 2w+1 of all 32 rows.
#include "device_common.hpp"
#include "kernels.hpp"

namespace infr {

typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

// LDS of one block: B operands [sub-block][lane] x 16 B | mins [row][kh][8] f16 (K slot 8 kh + sb =
// group 2 sb + kh) | (d, dmin) [row]
struct Q2kLds {
    static constexpr int mn_off = 8 * 1024;
    static constexpr int dd_off = mn_off + 32 * 32;
    static constexpr int bytes = dd_off + 32 * 8;
};

template <bool STAGES>
__global__ __launch_bounds__(256) void mmq_shared_q2k_kernel(
    const uint8_t* __restrict__ w, size_t bpr, const int8_t* __restrict__ qs, const float* __restrict__ d8,
    float* __restrict__ y, int m, int out_f, int nb, int32_t* __restrict__ st_sd, int32_t* __restrict__ st_sm) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * Q2kLds::bytes];
    __shared__ __attribute__((aligned(16))) float dql[4][32];  // per wave: its tokens' activation scales
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, h = lane >> 5;
    const int tok0 = blockIdx.y * 128 + wave * 32;
    const int wrow = blockIdx.x * 32 + col;
    const bool row_ok = wrow < out_f;
    const uint8_t* wrowp = w + (size_t)(row_ok ? wrow : 0) * bpr;
    const int p = wave;  // the sub-block pair (2p, 2p+1) this wave unpacks: bytes 32 (p / 2) + 16 h .., bit pairs 2 (p % 2) + e

    float acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;

    struct Raw {
        v4i sc, q;
        int dd;
    };
    auto request_rows = [&](Raw& r, int b) {
        const uint8_t* blk = wrowp + (size_t)b * 84;  // 4-byte aligned
        r.sc = load16_a4(blk);
        r.q = load16_a4(blk + 16 + 32 * (p >> 1) + 16 * h);
        r.dd = load_u32(blk + 80);
    };
    auto unpack_to = [&](uint8_t* buf, const Raw& r) {
        const uint32_t scw = (uint32_t)r.sc[p];  // scales of groups 4p .. 4p+3
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const uint32_t sc = (scw >> (8 * (2 * e + h))) & 0xFu;  // group 2 (2p + e) + h
            const int sh = 2 * (2 * (p & 1) + e);
            v4i out;
#pragma unroll
            for (int k = 0; k < 4; ++k) out[k] = (int)((((uint32_t)r.q[k] >> sh) & 0x03030303u) * sc);  // <= 45 a byte
            *reinterpret_cast<v4i*>(buf + (size_t)(2 * p + e) * 1024 + lane * 16) = out;
        }
        if (p == 0) {
            // this lane: the mins of groups 2 sb + h, sb = 0..7, in K-slot order
            const uint32_t s4[4] = {(uint32_t)r.sc.x, (uint32_t)r.sc.y, (uint32_t)r.sc.z, (uint32_t)r.sc.w};
            v8h mn;
#pragma unroll
            for (int sb = 0; sb < 8; ++sb) {
                const int g = 2 * sb;  // + h
                mn[sb] = (_Float16)(int)((s4[g >> 2] >> (8 * ((g & 3) + h) + 4)) & 0xFu);
            }
            *reinterpret_cast<v8h*>(buf + Q2kLds::mn_off + col * 32 + h * 16) = mn;
            if (h == 0) {
                float* dd = reinterpret_cast<float*>(buf + Q2kLds::dd_off) + col * 2;
                dd[0] = f16_bits_to_f32((uint32_t)r.dd & 0xFFFFu);
                dd[1] = f16_bits_to_f32((uint32_t)r.dd >> 16);
            }
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
        const uint8_t* cur = lds + (b & 1) * Q2kLds::bytes;
        // ---- unpack block b+1 into the other buffer, then ask for block b+2's bytes ----
        unpack_to(lds + ((b + 1) & 1) * Q2kLds::bytes, raw);
        request_rows(raw, min(b + 2, nb - 1));
        if (h == 0) dql[wave][col] = dtok;
        v16i sd = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        const v16f zf = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        v8h bs16;  // this lane's token: the sums of groups 2 sb + h
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) {
            const v4i bf = *reinterpret_cast<const v4i*>(cur + (size_t)sb * 1024 + lane * 16);
            sd = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[sb], bf, sd, 0, 0, 0);
            int s = __builtin_amdgcn_sdot4(a[sb].x, 0x01010101, 0, false);
            s = __builtin_amdgcn_sdot4(a[sb].y, 0x01010101, s, false);
            s = __builtin_amdgcn_sdot4(a[sb].z, 0x01010101, s, false);
            s = __builtin_amdgcn_sdot4(a[sb].w, 0x01010101, s, false);
            bs16[sb] = (_Float16)s;  // |s| <= 2032: exact
        }
        // the activation registers are free: fetch block b+1 while the epilogue runs
        request_acts(min(b + 1, nb - 1));
        const v8h bm = *reinterpret_cast<const v8h*>(cur + Q2kLds::mn_off + col * 32 + h * 16);
        const v16f smf = __builtin_amdgcn_mfma_f32_32x32x16_f16(bs16, bm, zf, 0, 0, 0);
        const float* dd = reinterpret_cast<const float*>(cur + Q2kLds::dd_off) + col * 2;
        const float d = dd[0], dmin = dd[1];
        // accumulator i of this lane is token 8*(i/4) + 4*h + i%4 of the wave's 32
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const v4f dq = *reinterpret_cast<const v4f*>(&dql[wave][8 * j + 4 * h]);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int r = 4 * j + i;
                if (STAGES) {
                    const int tok = tok0 + 8 * j + 4 * h + i;
                    if (row_ok && tok < m) {
                        st_sd[((size_t)tok * out_f + wrow) * nb + b] = sd[r];
                        st_sm[((size_t)tok * out_f + wrow) * nb + b] = (int)smf[r];
                    }
                }
                // sumf += q8.d[b] * (d * sd as f32 - dmin * sm as f32)
                acc[r] += dq[i] * (d * (float)sd[r] - dmin * smf[r]);
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

void launch_mmq_shared_q2k(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m, size_t in_f,
                           size_t out_f, const IntStages& st, hipStream_t stream) {
    const dim3 grid((unsigned)((out_f + 31) / 32), (unsigned)((m + 127) / 128)), block(256);
    const int nb = (int)(in_f / 256);
    if (st.a)
        hipLaunchKernelGGL((mmq_shared_q2k_kernel<true>), grid, block, 0, stream, w, bpr, act.qs, act.d, y, (int)m,
                           (int)out_f, nb, st.a, st.b);
    else
        hipLaunchKernelGGL((mmq_shared_q2k_kernel<false>), grid, block, 0, stream, w, bpr, act.qs, act.d, y, (int)m,
                           (int)out_f, nb, (int32_t*)nullptr, (int32_t*)nullptr);
}

}  // namespace infr
