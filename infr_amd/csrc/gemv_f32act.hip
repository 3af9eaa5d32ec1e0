// Decode GEMV against f32 activations, for weight formats that infr-cpu's one-token dispatch has
// no int8 kernel for: there a row is decoded to f32 and multiplied with `dot`
// (`_ => dot(&bytes_to_f32(row, dt), xrow)`, crates/infr-cpu/src/lib.rs:1165), so the activation is
// never rounded to int8. Q5_0 is the one such format carried here (with two or more tokens it takes
// the per-32 int8 kernel like its siblings, lib.rs:1322-1329).
//
// One workgroup stages x in LDS once (padded by 4 floats per 32 so that the lanes' 16-byte reads
// spread over all banks) and its four waves walk the tile's rows; lane l owns 32-weight block
// t*64 + l of the row, fetched with the same loader as the int8 kernel. Weights are decoded with
// the host decode's expression, sc * code + mn with sc = d * 1 and mn = d * (-16)
// (crates/infr-gguf/src/dequant.rs:38-44, 173-189), and accumulated with fused multiply-adds as
// `dot` does (kernels.rs:6557-6573); the order of the additions differs from the CPU's eight
// accumulators, within f32 rounding. HBM-bound on the weight bytes (22 B per 32 weights).
#include "gemv_formats.hpp"
#include "kernels.hpp"

namespace infr {

template <typename F>
__global__ __launch_bounds__(256) void gemv_f32act_kernel(const uint8_t* __restrict__ w, size_t bpr,
                                                          const float* __restrict__ x,
                                                          float* __restrict__ y, int in_f, int out_f,
                                                          int rows_per_wg) {
    extern __shared__ __attribute__((aligned(16))) float lx[];
    for (int i = threadIdx.x * 4; i < in_f; i += 1024)
        *reinterpret_cast<v4f*>(lx + i + (i >> 5) * 4) = *reinterpret_cast<const v4f*>(x + i);
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nb = in_f / 32, steps = (nb + 63) / 64;
    const int row_end = min(out_f, ((int)blockIdx.x + 1) * rows_per_wg);
    for (int row = (int)blockIdx.x * rows_per_wg + wave; row < row_end; row += 4) {
        const uint8_t* rowp = w + (size_t)row * bpr;
        float acc = 0.0f;
        for (int t = 0; t < steps; ++t) {
            const bool ok = F::valid(t, lane, nb);
            typename F::Row r;
            F::load_row(r, rowp, t, lane, ok);
            if (!ok) continue;
            const float d = f16_bits_to_f32(r.dm & 0xFFFFu);
            const float sc = d * 1.0f, mn = d * -16.0f;
            const v4f* xb = reinterpret_cast<const v4f*>(lx + (size_t)(t * 64 + lane) * 36);
            const int qw[4] = {r.qs.x, r.qs.y, r.qs.z, r.qs.w};
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t wq = (uint32_t)qw[k];
                const uint32_t lo = (wq & 0x0F0F0F0Fu) | spread4_to_bit4(r.qh >> (4 * k));
                const uint32_t hi = ((wq >> 4) & 0x0F0F0F0Fu) | spread4_to_bit4(r.qh >> (16 + 4 * k));
                const v4f x0 = xb[k], x1 = xb[4 + k];
                const float xl[4] = {x0.x, x0.y, x0.z, x0.w}, xh[4] = {x1.x, x1.y, x1.z, x1.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    acc = __builtin_fmaf(sc * (float)((lo >> (8 * j)) & 0xFFu) + mn, xl[j], acc);
                    acc = __builtin_fmaf(sc * (float)((hi >> (8 * j)) & 0xFFu) + mn, xh[j], acc);
                }
            }
        }
        acc = wave_sum_f(acc);
        if (lane == 0) y[row] = acc;
    }
}

bool gemv_takes_f32_activations(int dtype, size_t m) { return dtype == 6 && m == 1; }

bool launch_gemv_f32act(int dtype, const uint8_t* w, size_t bpr, const float* x, float* y, size_t in_f,
                        size_t out_f, hipStream_t stream) {
    if (dtype != 6 || in_f % 32 != 0) return false;
    const size_t lds = (in_f + in_f / 8) * sizeof(float);
    if (lds > 64 * 1024) return false;  // rows longer than 14,563 elements: no kernel
    if (out_f == 0) return true;
    // enough workgroups to cover the machine a few times, at least 4 rows each (one per wave)
    size_t rows_per_wg = (out_f + 2047) / 2048 * 4;
    rows_per_wg = rows_per_wg < 8 ? 8 : rows_per_wg;
    const dim3 grid((unsigned)((out_f + rows_per_wg - 1) / rows_per_wg));
    hipLaunchKernelGGL((gemv_f32act_kernel<FmtQ5_0>), grid, dim3(256), lds, stream, w, bpr, x, y, (int)in_f,
                       (int)out_f, (int)rows_per_wg);
    return true;
}

}  // namespace infr
