// The ops either side of every Linear in a decoder layer: RmsNorm / RmsNormAdd
// (crates/infr-cpu/src/lib.rs:802-850), GatedAct / GatedActFused (lib.rs:1890-1971, act_fn and
// gated_act_fn kernels.rs:6578-6597) and Add (lib.rs:1972-1988). All are HBM-bound streams of a
// few bytes per element; in plans the decode GEMV absorbs them (see gemv.hip), these stand-alone
// kernels serve every other case.
//
// Numerics. Add and the gated activation are elementwise f32 with the CPU's operation order
// (`act(g) * u`, `x * s * w` left to right, no FMA); expf / tanhf are the device's, so the last
// bit can differ from the host libm. RmsNorm's sum of squares is a tree over the row, not the
// CPU's index-order chain (4096 dependent adds would cost ~15 us): s agrees to ~1e-7 relative.
#include "device_common.hpp"
#include "elementwise_fn.hpp"
#include "kernels.hpp"

namespace infr {

// One workgroup per row. `out` may alias `x` (in-place RmsNorm / RmsNormAdd), so neither carries
// __restrict__.
__global__ __launch_bounds__(256) void rms_norm_kernel(const float* x,
                                                       const float* __restrict__ w, float* out,
                                                       int dim, float eps, int accumulate) {
    __shared__ float part[4];
    const float* xr = x + (size_t)blockIdx.x * dim;
    float* orow = out + (size_t)blockIdx.x * dim;
    float s = 0.0f;
    for (int i = threadIdx.x; i < dim; i += 256) s += xr[i] * xr[i];
    s = wave_sum_f(s);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
    __syncthreads();
    const float ss = ((part[0] + part[1]) + (part[2] + part[3])) / (float)dim;
    const float scale = 1.0f / sqrtf(ss + eps);
    for (int i = threadIdx.x; i < dim; i += 256) {
        const float v = xr[i] * scale * w[i];
        orow[i] = accumulate ? orow[i] + v : v;
    }
}

// The same arithmetic for rows of up to 256 * VPT elements, the thread's elements held in registers:
// `out` may alias `x`, so the loop above has to finish each store before the next load - one memory
// round trip per 256 elements of the row (10.6 us for 16 rows of 4096) - where this form requests all
// of a thread's elements at once.
template <int VPT>
__global__ __launch_bounds__(256) void rms_norm_regs_kernel(const float* x,
                                                            const float* __restrict__ w, float* out,
                                                            int dim, float eps, int accumulate) {
    __shared__ float part[4];
    const float* xr = x + (size_t)blockIdx.x * dim;
    float* orow = out + (size_t)blockIdx.x * dim;
    float v[VPT], wv[VPT], prev[VPT];
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
        const int i = threadIdx.x + 256 * k;
        v[k] = i < dim ? xr[i] : 0.0f;
    }
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
        const int i = threadIdx.x + 256 * k;
        wv[k] = i < dim ? w[i] : 0.0f;
        prev[k] = accumulate && i < dim ? orow[i] : 0.0f;
    }
    float s = 0.0f;
#pragma unroll
    for (int k = 0; k < VPT; ++k)
        if (threadIdx.x + 256 * k < dim) s += v[k] * v[k];
    s = wave_sum_f(s);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
    __syncthreads();
    const float ss = ((part[0] + part[1]) + (part[2] + part[3])) / (float)dim;
    const float scale = 1.0f / sqrtf(ss + eps);
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
        const int i = threadIdx.x + 256 * k;
        if (i < dim) {
            const float r = v[k] * scale * wv[k];
            orow[i] = accumulate ? prev[k] + r : r;
        }
    }
}

__global__ __launch_bounds__(256) void gated_act_kernel(const float* __restrict__ gate,
                                                        const float* __restrict__ up,
                                                        float* __restrict__ out, GatedActShape s) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)s.rows * s.nff) return;
    const size_t r = idx / s.nff, i = idx % s.nff;
    const size_t gb = (s.gate_block_width > 0 || s.gate_stride > 0) ? r * s.gate_stride : r * s.nff;
    const size_t ub = (s.up_stride == 0 ? r * s.nff : r * s.up_stride) + s.up_off;
    size_t gi = gb + i;
    if (s.gate_block_width > 0) {
        const size_t headw = s.gate_block_width / 2;
        gi = gb + (i / headw) * s.gate_block_width + headw + i % headw;
    }
    out[idx] = gated_act_fn(s.act, s.has_clamp != 0, s.clamp, gate[gi], up[ub + i]);
}

__global__ __launch_bounds__(256) void add_kernel(const float* a, const float* b, float* out, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = a[i] + b[i];
}

void launch_rms_norm(const float* x, const float* w, float* out, size_t rows, size_t dim, float eps,
                     bool accumulate, hipStream_t stream) {
    if (rows == 0 || dim == 0) return;
    if (dim <= 256 * 8)
        hipLaunchKernelGGL(rms_norm_regs_kernel<8>, dim3((unsigned)rows), dim3(256), 0, stream, x, w, out, (int)dim, eps,
                           accumulate ? 1 : 0);
    else if (dim <= 256 * 32)
        hipLaunchKernelGGL(rms_norm_regs_kernel<32>, dim3((unsigned)rows), dim3(256), 0, stream, x, w, out, (int)dim, eps,
                           accumulate ? 1 : 0);
    else
        hipLaunchKernelGGL(rms_norm_kernel, dim3((unsigned)rows), dim3(256), 0, stream, x, w, out, (int)dim, eps,
                           accumulate ? 1 : 0);
}

void launch_gated_act(const float* gate, const float* up, float* out, const GatedActShape& s,
                      hipStream_t stream) {
    const size_t n = (size_t)s.rows * s.nff;
    if (n == 0) return;
    hipLaunchKernelGGL(gated_act_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, gate, up, out, s);
}

void launch_add(const float* a, const float* b, float* out, size_t n, hipStream_t stream) {
    if (n == 0) return;
    hipLaunchKernelGGL(add_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, a, b, out, n);
}

// Measurement aid: a read-only streaming pass over `bytes` of device memory with nothing but
// 16-byte loads (plain or non-temporal) and a xor, i.e. what a kernel that only had to fetch the
// weights could reach on this device. Each workgroup walks 16 KB chunks grid-stride; one word per workgroup is written so
// the loads cannot be dropped.
template <bool NT>
__global__ __launch_bounds__(256) void stream_read_kernel(const v4i* __restrict__ src, size_t n_vec,
                                                          int* __restrict__ out) {
    const size_t chunk = 1024;  // v4i per workgroup per iteration: 4 per thread
    v4i acc = v4i{0, 0, 0, 0};
    for (size_t base = (size_t)blockIdx.x * chunk; base < n_vec; base += (size_t)gridDim.x * chunk) {
        v4i v[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const size_t i = base + k * 256 + threadIdx.x;
            v[k] = i < n_vec ? (NT ? gload_stream<v4i>(src + i) : gload<v4i>(src + i)) : v4i{0, 0, 0, 0};
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) acc ^= v[k];
    }
    const int r = acc.x ^ acc.y ^ acc.z ^ acc.w;
    if (threadIdx.x == 0 || r == 0x5EEDF00D) out[blockIdx.x] = r;
}

void launch_stream_read(const void* src, size_t bytes, int* out, int workgroups, bool nontemporal, hipStream_t stream) {
    if (bytes < 16 || workgroups <= 0) return;
    if (nontemporal)
        hipLaunchKernelGGL(stream_read_kernel<true>, dim3((unsigned)workgroups), dim3(256), 0, stream,
                           static_cast<const v4i*>(src), bytes / 16, out);
    else
        hipLaunchKernelGGL(stream_read_kernel<false>, dim3((unsigned)workgroups), dim3(256), 0, stream,
                           static_cast<const v4i*>(src), bytes / 16, out);
}

// Measurement aid: nothing but v_mfma_i32_32x32x32_i8 on four independent accumulator tiles per
// wave, `iters` rounds, operands held in registers - the int8 matrix rate this device sustains with
// no memory traffic at all. random_data = 0 multiplies small constants; 1 fills the operands with
// pseudo-random bytes (weights-times-digit range on one side, full int8 on the other), which is what
// the prefill kernels feed the matrix cores and draws more power per instruction.
__global__ __launch_bounds__(256) void mfma_i8_peak_kernel(int* __restrict__ out, int iters, int random_data) {
    typedef int v16i __attribute__((ext_vector_type(16)));
    v4i a = {1, 2, 3, 4}, b = {5, 6, 7, 8};
    if (random_data) {
        uint32_t hsh = (threadIdx.x + 1) * 2654435761u + blockIdx.x * 40503u;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            hsh = hsh * 1664525u + 1013904223u;
            a[i] = (int)(hsh ^ (hsh >> 13));
            hsh = hsh * 1664525u + 1013904223u;
            b[i] = (int)((hsh ^ (hsh >> 11)) & 0x3F3F3F3Fu);
        }
    }
    v16i c0 = {}, c1 = {}, c2 = {}, c3 = {};
    for (int i = 0; i < iters; ++i) {
        c0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c1, 0, 0, 0);
        c2 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c2, 0, 0, 0);
        c3 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c3, 0, 0, 0);
    }
    int r = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i) r ^= c0[i] ^ c1[i] ^ c2[i] ^ c3[i];
    if (r == 0x5EEDF00D) out[blockIdx.x] = r;  // keeps the chain alive; practically never taken
}

void launch_mfma_i8_peak(int* out, int workgroups, int iters, int random_data, hipStream_t stream) {
    if (workgroups <= 0 || iters <= 0) return;
    hipLaunchKernelGGL(mfma_i8_peak_kernel, dim3((unsigned)workgroups), dim3(256), 0, stream, out, iters, random_data);
}

}  // namespace infr
