// Stand-alone activation quantizer kernels (the arithmetic is in quant_chunk.hpp): used for
// m >= 2 and by the entry points that expose the integer stage.
//
// Layout: one wavefront handles 256 consecutive floats (one float4 per lane). HBM traffic is
// 4 B read + ~1.2 B written per element; the kernel is a pure stream.
#include "elementwise_fn.hpp"
#include "kernels.hpp"
#include "quant_chunk.hpp"

namespace infr {

template <bool PER32>
__global__ __launch_bounds__(256) void quantize_q8_kernel(const float* __restrict__ x,
                                                          int8_t* __restrict__ qs,
                                                          float* __restrict__ d,
                                                          int32_t* __restrict__ bsums,
                                                          int32_t* __restrict__ bsums16,
                                                          size_t n_elems) {
    const int lane = threadIdx.x & 63;
    const size_t chunk = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (chunk * 256 >= n_elems) return;  // wave-uniform
    // Per-32 inputs may end inside a 256-float chunk (n_elems is a multiple of 32, so an 8-lane
    // group is either wholly inside or wholly outside).
    const bool live = chunk * 256 + (size_t)lane * 4 < n_elems;

    v4f v = {0.0f, 0.0f, 0.0f, 0.0f};
    if (live) v = *reinterpret_cast<const v4f*>(x + chunk * 256 + (size_t)lane * 4);
    quantize_chunk<PER32>(v, live, lane, chunk, qs, d, bsums, bsums16);
}

// The per-256 quantizer writing MFMA A-operand order for the shared-operand prefill kernel
// (same codes, scales and sums; only their place in memory differs). Tokens go in groups of 32;
// for group g and block b:
//   qs    [(g*nb + b)*8 + sub-block][lane = h*32 + token%32][16 B]: k = 16h .. 16h+15 of the sub-block
//   d     [(g*nb + b)*32 + token%32]
//   bsums (read as f16) [(g*nb + b)*64 + h*32 + token%32][8]: per-32 sums split bsum = lo + rest,
//         lo = bsum & 63 in the h = 0 half, bsum - lo in the h = 1 half (both exact in f16)
// so that a wave's fragment load is one contiguous kilobyte.
// One workgroup makes the whole 8 KiB code tile of (token group g, block b): each of its sixteen
// waves quantizes two tokens' chunks, the codes cross through LDS, and the tile leaves as 512
// contiguous 16-byte stores - a wave that
// wrote its own token's codes in place would scatter every store over sixteen 128-byte lines.
// Tokens past m quantize zeros (their slots hold d = 0 and zero codes).
template <int kTiledQuantWaves>
__global__ __launch_bounds__(kTiledQuantWaves * 64) void quantize_q8_tiled_kernel(const float* __restrict__ x,
                                                                int8_t* __restrict__ qs,
                                                                float* __restrict__ d,
                                                                _Float16* __restrict__ bsh,
                                                                int m, int nb) {
    // [sub-block][lane = h*32 + token][16 B], each sub-block's KiB followed by 16 B of padding so
    // that the lanes of a wave (eight sub-blocks x two halves x four dwords of one token) spread
    // over the banks
    constexpr int kSbStride = 1024 + 16;
    __shared__ __attribute__((aligned(16))) uint8_t tile[8 * kSbStride];
    __shared__ __attribute__((aligned(16))) _Float16 sums[64 * 8];
    __shared__ float scales[32];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int b = blockIdx.x, g = blockIdx.y;
    const size_t in_f = (size_t)nb * 256;
    constexpr int PW = 32 / kTiledQuantWaves;
    v4f v[PW];
#pragma unroll
    for (int i = 0; i < PW; ++i) {
        const int tok = g * 32 + wave * PW + i;
        v[i] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
        if (tok < m) v[i] = gload<v4f>(x + (size_t)tok * in_f + (size_t)b * 256 + lane * 4);
    }
    const int sb = lane >> 3, h = (lane >> 2) & 1, j4 = lane & 3;
#pragma unroll
    for (int i = 0; i < PW; ++i) {
        const int col = wave * PW + i;
        uint32_t packed;
        float dd;
        int s, s16;
        quantize_chunk_values<false>(v[i], packed, dd, s, s16);
        *reinterpret_cast<uint32_t*>(tile + sb * kSbStride + (h * 32 + col) * 16 + j4 * 4) = packed;
        if (lane == 0) scales[col] = dd;
        if ((lane & 7) == 0) {
            const int lo = s & 63;
            sums[col * 8 + sb] = (_Float16)lo;
            sums[(32 + col) * 8 + sb] = (_Float16)(s - lo);
        }
    }
    __syncthreads();
    const size_t gb = (size_t)g * nb + b;
    for (int piece = tid; piece < 512; piece += kTiledQuantWaves * 64) {  // 16-byte pieces of the tile: [sub-block][lane]
        const v4i c = *reinterpret_cast<const v4i*>(tile + (piece >> 6) * kSbStride + (piece & 63) * 16);
        gstore<v4i>(qs + gb * (8 * 1024) + (size_t)piece * 16, c);
    }
    if (tid < 64) gstore<v4i>(bsh + (gb * 64 + tid) * 8, *reinterpret_cast<const v4i*>(&sums[tid * 8]));
    if (tid < 32) gstore<float>(d + gb * 32 + tid, scales[tid]);
}

void launch_quantize_q8_tiled(const float* x, size_t m, size_t k, const ActQ8& out, hipStream_t stream) {
    if (m == 0 || k < 256) return;
    const dim3 grid((unsigned)(k / 256), (unsigned)((m + 31) / 32));
    // (sixteen waves of two tokens each; eight and four waves a workgroup measured 5-15 % slower)
    hipLaunchKernelGGL(quantize_q8_tiled_kernel<16>, grid, dim3(1024), 0, stream, x, out.qs, out.d,
                       reinterpret_cast<_Float16*>(out.bsums), (int)m, (int)(k / 256));
}

// The per-32 quantizer (quantize_q8_32, crates/infr-cpu/src/quant.rs:97-117) in the same tiled code
// order, for the MFMA prefill kernels of the 32-weight-block formats (k % 256 == 0): scales and code
// sums as f32 [(g*nb + b)*32 + token%32][8 blocks of the 256-element step] (|sum| <= 4064: exact).
// T16: the codes of every 16-element group are stored 4 x 4 transposed (dword i of the group holds
// elements i, 4 + i, 8 + i, 12 + i), the K order in which Q2_0's 2-bit codes unpack with one shift and
// one mask per dword; the matrix product does not care about the order inside a group as long as
// both operands share it.
template <bool T16>
__global__ __launch_bounds__(256) void quantize_q8_32_tiled_kernel(const float* __restrict__ x,
                                                                   int8_t* __restrict__ qs,
                                                                   float* __restrict__ d,
                                                                   float* __restrict__ bsf,
                                                                   size_t n_chunks, int nb, int k) {
    const int lane = threadIdx.x & 63;
    const size_t chunk = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (chunk >= n_chunks) return;  // wave-uniform
    // chunk = 256-element step b of token tok; a row that ends inside its last step is padded with
    // zeros there (whole 32-element groups: codes, scale and sum all zero)
    const size_t tok = chunk / nb, b = chunk % nb;
    v4f v = {0.0f, 0.0f, 0.0f, 0.0f};
    if ((int)b * 256 + lane * 4 < k) v = *reinterpret_cast<const v4f*>(x + tok * k + b * 256 + (size_t)lane * 4);
    uint32_t packed;
    float dd;
    int s, s16;
    quantize_chunk_values<true>(v, packed, dd, s, s16);
    const size_t gb = (tok >> 5) * nb + b;
    const int col = (int)(tok & 31);
    const int sb = lane >> 3, h = (lane >> 2) & 1, j4 = lane & 3;
    if (T16) {
        // lanes 4g..4g+3 hold the group's dwords P0..P3 (elements 4j..4j+3); lane i leaves with byte i
        // of each
        const int base = lane & ~3;
        const uint32_t p0 = (uint32_t)__shfl((int)packed, base, kWave), p1 = (uint32_t)__shfl((int)packed, base + 1, kWave);
        const uint32_t p2 = (uint32_t)__shfl((int)packed, base + 2, kWave), p3 = (uint32_t)__shfl((int)packed, base + 3, kWave);
        const uint32_t sel = (uint32_t)j4 | ((uint32_t)(4 + j4) << 8);       // byte i of src1, byte i of src0
        const uint32_t t01 = __builtin_amdgcn_perm(p1, p0, sel) & 0xFFFFu;   // (P0.b_i, P1.b_i)
        const uint32_t t23 = __builtin_amdgcn_perm(p3, p2, sel) & 0xFFFFu;   // (P2.b_i, P3.b_i)
        packed = t01 | (t23 << 16);
    }
    reinterpret_cast<uint32_t*>(qs)[((gb * 8 + sb) * 64 + h * 32 + col) * 4 + j4] = packed;
    if ((lane & 7) == 0) {
        d[(gb * 32 + col) * 8 + sb] = dd;
        bsf[(gb * 32 + col) * 8 + sb] = (float)s;
    }
}

void launch_quantize_q8_32_tiled(const float* x, size_t m, size_t k, bool transposed16, const ActQ8& out,
                                 hipStream_t stream) {
    const size_t nb = (k + 255) / 256, n_chunks = m * nb;
    if (n_chunks == 0) return;
    const dim3 grid((unsigned)((n_chunks + 3) / 4));
    if (transposed16)
        hipLaunchKernelGGL(quantize_q8_32_tiled_kernel<true>, grid, dim3(256), 0, stream, x, out.qs, out.d,
                           reinterpret_cast<float*>(out.bsums), n_chunks, (int)nb, (int)k);
    else
        hipLaunchKernelGGL(quantize_q8_32_tiled_kernel<false>, grid, dim3(256), 0, stream, x, out.qs, out.d,
                           reinterpret_cast<float*>(out.bsums), n_chunks, (int)nb, (int)k);
}

template <bool PER32>
__global__ __launch_bounds__(256) void quantize_q8_group_kernel(const QuantTile* __restrict__ tiles,
                                                                int8_t* __restrict__ qs,
                                                                float* __restrict__ d,
                                                                int32_t* __restrict__ bsums,
                                                                int32_t* __restrict__ bsums16) {
    __shared__ float part[4];
    const QuantTile t = tiles[blockIdx.x];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int e = wave * 256 + lane * 4;
    const bool live = (uint32_t)e < t.n_elems;
    // the tile's own floats are requested before the row reduction of a folded norm, not behind it
    v4f v = {0.0f, 0.0f, 0.0f, 0.0f}, u = {0.0f, 0.0f, 0.0f, 0.0f};
    if (live) {
        v = *reinterpret_cast<const v4f*>(t.x + e);
        if (t.pre) u = *reinterpret_cast<const v4f*>(t.x2 + e);
    }
    float scale = 0.0f;
    if (t.pre == 2) {
        // rms_norm_kernel's reduction over the whole row (stride-256 partial sums, wave sums,
        // ((p0 + p1) + (p2 + p3))): the same scale, so the same floats and the same codes
        float s = 0.0f;
        for (uint32_t i = threadIdx.x; i < t.dim; i += 256) s += t.row[i] * t.row[i];
        s = wave_sum_f(s);
        if (lane == 0) part[wave] = s;
        __syncthreads();
        const float ss = ((part[0] + part[1]) + (part[2] + part[3])) / (float)t.dim;
        scale = 1.0f / sqrtf(ss + t.eps);
    }
    if ((uint32_t)wave * 256 >= t.n_elems) return;  // wave-uniform
    if (live && t.pre) {
        if (t.pre == 1)
            v = v4f{gated_act_fn(t.act, t.has_clamp != 0, t.clamp, v.x, u.x),
                    gated_act_fn(t.act, t.has_clamp != 0, t.clamp, v.y, u.y),
                    gated_act_fn(t.act, t.has_clamp != 0, t.clamp, v.z, u.z),
                    gated_act_fn(t.act, t.has_clamp != 0, t.clamp, v.w, u.w)};
        else
            v = v4f{v.x * scale * u.x, v.y * scale * u.y, v.z * scale * u.z, v.w * scale * u.w};
        *reinterpret_cast<v4f*>(t.pre_dst + e) = v;
    }
    quantize_chunk<PER32>(v, live, lane, (size_t)t.chunk0 + wave, qs, d, bsums, bsums16);
}

void launch_quantize_q8_group(const QuantTile* tiles_dev, size_t n_tiles, bool per32, const ActQ8& out,
                              hipStream_t stream) {
    if (n_tiles == 0) return;
    if (per32)
        hipLaunchKernelGGL(quantize_q8_group_kernel<true>, dim3((unsigned)n_tiles), dim3(256), 0, stream,
                           tiles_dev, out.qs, out.d, out.bsums, (int32_t*)nullptr);
    else
        hipLaunchKernelGGL(quantize_q8_group_kernel<false>, dim3((unsigned)n_tiles), dim3(256), 0, stream,
                           tiles_dev, out.qs, out.d, out.bsums, out.bsums16);
}

void launch_quantize_q8(const float* x, size_t m, size_t k, bool per32, const ActQ8& out,
                        hipStream_t stream) {
    const size_t n_elems = m * k;
    const size_t n_chunks = (n_elems + 255) / 256;
    if (n_chunks == 0) return;
    const dim3 grid((unsigned)((n_chunks + 3) / 4)), block(256);
    if (per32)
        hipLaunchKernelGGL(quantize_q8_kernel<true>, grid, block, 0, stream, x, out.qs, out.d,
                           out.bsums, (int32_t*)nullptr, n_elems);
    else
        hipLaunchKernelGGL(quantize_q8_kernel<false>, grid, block, 0, stream, x, out.qs, out.d,
                           out.bsums, out.bsums16, n_elems);
}

}  // namespace infr
