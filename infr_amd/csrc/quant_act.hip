// Stand-alone activation quantizer kernels (the arithmetic is in quant_chunk.hpp): used for
// m >= 2 and by the entry points that expose the integer stage.
//
// Layout: one wavefront handles 256 consecutive floats (one float4 per lane). HBM traffic is
// 4 B read + ~1.2 B written per element; the kernel is a pure stream.
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
