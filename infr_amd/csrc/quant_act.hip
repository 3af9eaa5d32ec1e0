// Activation quantizers on the device, bit-exact with infr-cpu:
//   quantize_q8    (crates/infr-cpu/src/quant.rs:27-58)  per 256 elements, f32 scale, i32 sums
//   quantize_q8_32 (crates/infr-cpu/src/quant.rs:97-117) per 32 elements
// amax is an order-independent maximum, `amax / 127` and `1 / d` are IEEE-correct divisions
// (no reciprocal approximation), `round` is half away from zero (roundf), so every output field
// equals the CPU's bit for bit.
//
// Layout: one wavefront handles 256 consecutive floats (one float4 per lane). HBM traffic is
// 4 B read + ~1.2 B written per element; the kernel is a pure stream.
#include "device_common.hpp"
#include "kernels.hpp"

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
    float amax = __builtin_fmaxf(__builtin_fmaxf(__builtin_fabsf(v.x), __builtin_fabsf(v.y)),
                                 __builtin_fmaxf(__builtin_fabsf(v.z), __builtin_fabsf(v.w)));
    // Maximum over the block's lanes: 8 lanes (32 floats) or all 64 (256 floats).
#pragma unroll
    for (int off = 1; off < (PER32 ? 8 : 64); off <<= 1)
        amax = __builtin_fmaxf(amax, __shfl_xor(amax, off, kWave));

    const float dd = amax / 127.0f;
    const float id = dd > 0.0f ? 1.0f / dd : 0.0f;

    auto q1 = [id](float f) -> int {
        float r = roundf(f * id);
        r = r < -127.0f ? -127.0f : r;
        r = r > 127.0f ? 127.0f : r;
        return (int)r;
    };
    const int q0 = q1(v.x), q1_ = q1(v.y), q2 = q1(v.z), q3 = q1(v.w);
    const uint32_t packed = (uint32_t)(q0 & 0xFF) | ((uint32_t)(q1_ & 0xFF) << 8) |
                            ((uint32_t)(q2 & 0xFF) << 16) | ((uint32_t)(q3 & 0xFF) << 24);
    if (live) reinterpret_cast<uint32_t*>(qs)[chunk * 64 + lane] = packed;

    int s = q0 + q1_ + q2 + q3;  // 4 elements
    s += __shfl_xor(s, 1, kWave);
    s += __shfl_xor(s, 2, kWave);  // 16 elements: lanes 4g..4g+3
    const int s16 = s;
    s += __shfl_xor(s, 4, kWave);  // 32 elements: lanes 8g..8g+7

    if (PER32) {
        if (live && (lane & 7) == 0) {
            d[chunk * 8 + (lane >> 3)] = dd;
            bsums[chunk * 8 + (lane >> 3)] = s;
        }
    } else {
        if (lane == 0) d[chunk] = dd;
        if ((lane & 7) == 0) bsums[chunk * 8 + (lane >> 3)] = s;
        if (bsums16 != nullptr && (lane & 3) == 0) bsums16[chunk * 16 + (lane >> 2)] = s16;
    }
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
