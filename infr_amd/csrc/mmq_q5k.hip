// Prefill GEMM (33 tokens and up) of Q5_K weights on the int8 matrix cores.
//
// Per 256-element block infr-cpu computes, per output (crates/infr-cpu/src/kernels.rs, the Q5_K
// scalar kernel; same shape as Q4_K's, :151-184),
//     sd = sum_s sc_s * (sum_l q5 * q8)     sm = sum_s m_s * bsums_s
//     y += q8.d[b] * (d * (f32)sd - dmin * (f32)sm)
// with 6-bit sc_s, m_s per 32-element sub-block and 5-bit codes (a nibble of ql plus bit s of qh).
// q5 (0..31) is an int8 operand, q5 * sc_s (up to 1953) is not, and even split scale digits
// overflow a signed byte (31 * 7), so Q4_K's two-plane trick does not carry over: every sub-block is
// multiplied on its own - one v_mfma_i32_32x32x32_i8 over its 32 elements - and scaled into sd with
// one 24-bit multiply-add per output. sm is the K = 16 f16 MFMA of the mins against the split
// per-32 sums, exactly as in the Q4_K kernel, the epilogue is the CPU expression and the blocks are
// added in ascending order: y equals infr-cpu's batch kernel and the one-token GEMV bit for bit.
//
// Tiling, LDS double-buffering and the tiled activation layout are the other shared-operand
// kernels': 128 tokens x 32 weight rows per workgroup, wave w owns tokens 32w..32w+31 and unpacks
// sub-blocks 2w, 2w+1 (nibble pair w) of all 32 rows.
#include "device_common.hpp"
#include "kernels.hpp"

namespace infr {

typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

// LDS of one block: B operands [sub-block][lane] x 16 B | mins [row][8] f16 | scales [row][8] u8 | (d, dmin) [row]
struct Q5kLds {
    static constexpr int mn_off = 8 * 1024;
    static constexpr int sc_off = mn_off + 32 * 16;
    static constexpr int dd_off = sc_off + 32 * 8;
    static constexpr int bytes = dd_off + 32 * 8;
};

template <bool STAGES>
__global__ __launch_bounds__(256) void mmq_shared_q5k_kernel(
    const uint8_t* __restrict__ w, size_t bpr, const int8_t* __restrict__ qs, const float* __restrict__ d8,
    const _Float16* __restrict__ bsh, float* __restrict__ y, int m, int out_f, int nb,
    int32_t* __restrict__ st_sd, int32_t* __restrict__ st_sm) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * Q5kLds::bytes];
    __shared__ __attribute__((aligned(16))) float dql[4][32];  // per wave: its tokens' activation scales
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, h = lane >> 5;
    const int tok0 = blockIdx.y * 128 + wave * 32;
    const int wrow = blockIdx.x * 32 + col;
    const bool row_ok = wrow < out_f;
    const uint8_t* wrowp = w + (size_t)(row_ok ? wrow : 0) * bpr;
    const int p = wave;  // the nibble pair (sub-blocks 2p, 2p+1) this wave unpacks

    float acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;

    struct Raw {
        v4i hdr, qh, ql;
    };
    auto request_rows = [&](Raw& r, int b) {
        const uint8_t* blk = wrowp + (size_t)b * 176;  // 16-byte aligned
        r.hdr = load16(blk);
        r.qh = load16(blk + 16 + 16 * h);
        r.ql = load16(blk + 48 + p * 32 + 16 * h);
    };
    auto unpack_to = [&](uint8_t* buf, const Raw& r) {
#pragma unroll
        for (int e = 0; e < 2; ++e) {  // e = 0: sub-block 2p (low nibbles, qh bit 2p), 1: 2p+1 (high, bit 2p+1)
            v4i out;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t nib = ((uint32_t)r.ql[k] >> (4 * e)) & 0x0F0F0F0Fu;
                const uint32_t hb = ((uint32_t)r.qh[k] >> (2 * p + e)) & 0x01010101u;
                out[k] = (int)((hb << 4) | nib);  // 0..31 per byte
            }
            *reinterpret_cast<v4i*>(buf + (size_t)(2 * p + e) * 1024 + lane * 16) = out;
        }
        if (p == 0 && h == 0) {
            uint32_t sc8[2], mn8[2];
            k4_all((uint32_t)r.hdr.y, (uint32_t)r.hdr.z, (uint32_t)r.hdr.w, sc8, mn8);
            v8h mn;
#pragma unroll
            for (int s = 0; s < 8; ++s) mn[s] = (_Float16)(int)((mn8[s >> 2] >> (8 * (s & 3))) & 0xFFu);
            *reinterpret_cast<v8h*>(buf + Q5kLds::mn_off + col * 16) = mn;
            uint32_t* sc = reinterpret_cast<uint32_t*>(buf + Q5kLds::sc_off + col * 8);
            sc[0] = sc8[0];
            sc[1] = sc8[1];
            float* dd = reinterpret_cast<float*>(buf + Q5kLds::dd_off) + col * 2;
            dd[0] = f16_bits_to_f32((uint32_t)r.hdr.x & 0xFFFFu);
            dd[1] = f16_bits_to_f32((uint32_t)r.hdr.x >> 16);
        }
    };
    // activation fragments in the tiled quantizer's order: every load is a contiguous kilobyte
    v4i a[8];
    v8h abs_;  // split per-32 sums: the h = 0 lanes carry bsum & 63, the h = 1 lanes the rest
    float dtok;
    // this wave's group of 32 tokens; a wave wholly past m recomputes the last group (nothing is stored)
    const size_t g = min((size_t)blockIdx.y * 4 + wave, (size_t)(m - 1) / 32);
    auto request_acts = [&](int b) {
        const size_t gb = g * nb + b;
        const int8_t* ap = qs + gb * (8 * 1024) + lane * 16;
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) a[sb] = *reinterpret_cast<const v4i*>(ap + sb * 1024);
        abs_ = *reinterpret_cast<const v8h*>(bsh + (gb * 64 + lane) * 8);
        dtok = d8[gb * 32 + col];
    };

    Raw raw;
    request_rows(raw, 0);
    unpack_to(lds, raw);
    request_rows(raw, min(1, nb - 1));
    request_acts(0);
    __syncthreads();

    for (int b = 0; b < nb; ++b) {
        const uint8_t* cur = lds + (b & 1) * Q5kLds::bytes;
        // ---- unpack block b+1 into the other buffer, then ask for block b+2's bytes ----
        unpack_to(lds + ((b + 1) & 1) * Q5kLds::bytes, raw);
        request_rows(raw, min(b + 2, nb - 1));
        const v8h abs_b = abs_;
        if (h == 0) dql[wave][col] = dtok;
        const uint32_t* scp = reinterpret_cast<const uint32_t*>(cur + Q5kLds::sc_off + col * 8);
        const uint32_t scw[2] = {scp[0], scp[1]};
        const v16i zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        const v16f zf = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        int sd[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) sd[i] = 0;
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) {
            const v4i bf = *reinterpret_cast<const v4i*>(cur + (size_t)sb * 1024 + lane * 16);
            const v16i r = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[sb], bf, zi, 0, 0, 0);
            const int sc = (int)((scw[sb >> 2] >> (8 * (sb & 3))) & 0xFFu);
#pragma unroll
            for (int i = 0; i < 16; ++i) sd[i] += __mul24(r[i], sc);
        }
        // the activation registers are free: fetch block b+1 while the epilogue runs
        request_acts(min(b + 1, nb - 1));
        const v8h bm = *reinterpret_cast<const v8h*>(cur + Q5kLds::mn_off + col * 16);
        const v16f smf = __builtin_amdgcn_mfma_f32_32x32x16_f16(abs_b, bm, zf, 0, 0, 0);
        const float* dd = reinterpret_cast<const float*>(cur + Q5kLds::dd_off) + col * 2;
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

void launch_mmq_shared_q5k(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m, size_t in_f,
                           size_t out_f, const IntStages& st, hipStream_t stream) {
    const dim3 grid((unsigned)((out_f + 31) / 32), (unsigned)((m + 127) / 128)), block(256);
    const int nb = (int)(in_f / 256);
    const _Float16* bsh = reinterpret_cast<const _Float16*>(act.bsums);
    if (st.a)
        hipLaunchKernelGGL((mmq_shared_q5k_kernel<true>), grid, block, 0, stream, w, bpr, act.qs, act.d, bsh, y,
                           (int)m, (int)out_f, nb, st.a, st.b);
    else
        hipLaunchKernelGGL((mmq_shared_q5k_kernel<false>), grid, block, 0, stream, w, bpr, act.qs, act.d, bsh, y,
                           (int)m, (int)out_f, nb, (int32_t*)nullptr, (int32_t*)nullptr);
}

}  // namespace infr
