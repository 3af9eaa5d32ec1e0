// Decode GEMV against f32 activations, for weight formats that infr-cpu's one-token dispatch has
// no int8 kernel for: there a row is decoded to f32 and multiplied with `dot`
// (`_ => dot(&bytes_to_f32(row, dt), xrow)`, crates/infr-cpu/src/lib.rs:1165), so the activation is
// never rounded to int8. Q5_0 is the one such format carried here (with two or more tokens it takes
// the per-32 int8 kernel like its siblings, lib.rs:1322-1329).
//
// One workgroup stages x in LDS once (padded by 4 floats per 32 so that the lanes' 16-byte reads
// spread over all banks) and its waves walk the tile's rows; lane l owns 32-weight block
// t*64 + l of the row, fetched with the same loader as the int8 kernel. The host decode gives
// w = d * code + d * (-16) (crates/infr-gguf/src/dequant.rs:38-44, 173-189); the kernel takes d out
// of a block's 32 products: d * (sum code * x - 16 * sum x), the code sum as byte-to-float conversions (v_cvt_f32_ubyte) and FMAs
// and the block sums of x computed once per workgroup. Same value in exact arithmetic, f32 rounding
// in a different order than the CPU's `dot` (kernels.rs:6557-6573): about 1e-6 relative. The loop
// is instruction-bound (two VALU operations per weight), not HBM-bound. Inside a plan the ops of a
// level that share a row length run as one launch over a tile table (a launch per op kept a
// 4096 x 4096 matrix at 1.6 TB/s - one short round of workgroups at a time - where the group runs at 4.9).
#include "gemv_formats.hpp"
#include "kernels.hpp"

namespace infr {

template <typename F, int NW>
__global__ __launch_bounds__(NW * 64) void gemv_f32act_kernel(const uint8_t* __restrict__ w, size_t bpr,
                                                          const float* __restrict__ x,
                                                          float* __restrict__ y, int in_f, int out_f,
                                                          int rows_per_wg, const GemvTile* __restrict__ tiles) {
    extern __shared__ __attribute__((aligned(16))) float lx[];
    // A grouped launch (plans): the workgroup's rows are one entry of the tile table - some rows of
    // one of several ops of this row length.
    int first_row = (int)blockIdx.x * rows_per_wg;
    if (tiles) {
        const GemvTile t = tiles[blockIdx.x];
        w = t.w;
        bpr = t.bpr;
        x = t.x;
        y = t.y;
        out_f = t.rows;
        first_row = 0;
        rows_per_wg = t.rows;
    }
    const int nb = in_f / 32;
    float* lsx = lx + (size_t)nb * 36;  // per-block sums of x
    for (int i = threadIdx.x * 4; i < in_f; i += NW * 256)
        *reinterpret_cast<v4f*>(lx + i + (i >> 5) * 4) = gload<v4f>(x + i);
    __syncthreads();
    for (int b = threadIdx.x; b < nb; b += NW * 64) {
        const v4f* xb = reinterpret_cast<const v4f*>(lx + (size_t)b * 36);
        float sx = 0.0f;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const v4f v = xb[k];
            sx += (v.x + v.y) + (v.z + v.w);
        }
        lsx[b] = sx;
    }
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int steps = (nb + 63) / 64;
    const int row_end = min(out_f, first_row + rows_per_wg);
    // The wave's (row, step) sequence is walked with the next step's block already requested.
    int row = first_row + wave, t = 0;
    typename F::Row cur;
    F::load_row(cur, w + (size_t)(row < row_end ? row : 0) * bpr, 0, lane, row < row_end && F::valid(0, lane, nb));
    float acc = 0.0f;
    while (row < row_end) {
        const bool last = t + 1 == steps;
        const int nrow = last ? row + NW : row, nt = last ? 0 : t + 1;
        typename F::Row nxt;
        F::load_row(nxt, w + (size_t)(nrow < row_end ? nrow : 0) * bpr, nt, lane, nrow < row_end && F::valid(nt, lane, nb));
        if (F::valid(t, lane, nb)) {
            const int b = t * 64 + lane;
            const v4f* xb = reinterpret_cast<const v4f*>(lx + (size_t)b * 36);
            const int qw[4] = {cur.qs.x, cur.qs.y, cur.qs.z, cur.qs.w};
            // sum over the block of code * x, then d * (that - 16 * sum x): the host decode's
            // d * code + d * (-16) with the common factor taken out of the 32 products
            // (four partial sums: one chain of 32 dependent FMAs per block left the SIMD idle between them)
            float s1 = 0.0f, s2 = 0.0f, s3 = 0.0f, s4 = 0.0f;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t wq = (uint32_t)qw[k];
                const uint32_t lo = (wq & 0x0F0F0F0Fu) | spread4_to_bit4(cur.qh >> (4 * k));
                const uint32_t hi = ((wq >> 4) & 0x0F0F0F0Fu) | spread4_to_bit4(cur.qh >> (16 + 4 * k));
                const v4f x0 = xb[k], x1 = xb[4 + k];
                s1 = __builtin_fmaf((float)(lo & 0xFFu), x0.x, s1);
                s2 = __builtin_fmaf((float)((lo >> 8) & 0xFFu), x0.y, s2);
                s3 = __builtin_fmaf((float)((lo >> 16) & 0xFFu), x0.z, s3);
                s4 = __builtin_fmaf((float)(lo >> 24), x0.w, s4);
                s1 = __builtin_fmaf((float)(hi & 0xFFu), x1.x, s1);
                s2 = __builtin_fmaf((float)((hi >> 8) & 0xFFu), x1.y, s2);
                s3 = __builtin_fmaf((float)((hi >> 16) & 0xFFu), x1.z, s3);
                s4 = __builtin_fmaf((float)(hi >> 24), x1.w, s4);
            }
            s1 = (s1 + s2) + (s3 + s4);
            const float d = f16_bits_to_f32(cur.dm & 0xFFFFu);
            acc = __builtin_fmaf(d, s1 - 16.0f * lsx[b], acc);
        }
        if (last) {
            const float tot = wave_sum_f(acc);
            if (lane == 0) gstore<float>(y + row, tot);
            acc = 0.0f;
        }
        cur = nxt;
        row = nrow;
        t = nt;
    }
}

bool gemv_takes_f32_activations(int dtype, size_t m) { return dtype == 6 && m == 1; }

static size_t f32act_lds_bytes(size_t in_f) { return (in_f + in_f / 8 + in_f / 32) * sizeof(float); }

// Long rows: their activations fill a third of a compute unit's LDS, so two workgroups share it at
// most - sixteen waves each instead of four (a group of 4096 x 12288 matrices: 2.6 TB/s with four
// waves, 4.1 with eight, 4.9 with sixteen; rows of 4096 columns run the same with any of them).
static int f32act_waves(size_t in_f) { return f32act_lds_bytes(in_f) > 32 * 1024 ? 16 : 4; }

static void f32act_launch(size_t in_f, unsigned wgs, const uint8_t* w, size_t bpr, const float* x, float* y, size_t out_f,
                          int rows_per_wg, const GemvTile* tiles, hipStream_t stream) {
    const size_t lds = f32act_lds_bytes(in_f);
    if (f32act_waves(in_f) == 16)
        hipLaunchKernelGGL((gemv_f32act_kernel<FmtQ5_0, 16>), dim3(wgs), dim3(1024), lds, stream, w, bpr, x, y, (int)in_f,
                           (int)out_f, rows_per_wg, tiles);
    else
        hipLaunchKernelGGL((gemv_f32act_kernel<FmtQ5_0, 4>), dim3(wgs), dim3(256), lds, stream, w, bpr, x, y, (int)in_f,
                           (int)out_f, rows_per_wg, tiles);
}

bool gemv_f32act_groups(int dtype, size_t in_f) {
    return dtype == 6 && in_f % 32 == 0 && f32act_lds_bytes(in_f) <= 64 * 1024;  // (rows up to 14,144 elements)
}

// Rows per workgroup: every workgroup stages x and its block sums first - about what eight rows
// cost - so large groups take taller tiles (a 130-op group of 4096 x 4096 matrices: 4.1 TB/s with 8
// rows, 4.6 with 16, 4.8-4.9 from 32 up); at least a row per wave, and a few workgroups per compute unit.
int gemv_f32act_group_rows(size_t total_rows, size_t in_f) {
    const size_t nw = (size_t)f32act_waves(in_f), lo = nw == 16 ? 16 : 8, hi = nw == 16 ? 128 : 32;
    const size_t r = (total_rows + 2047) / 2048 * 4;
    return (int)(r < lo ? lo : (r > hi ? hi : r));
}

bool launch_gemv_f32act(int dtype, const uint8_t* w, size_t bpr, const float* x, float* y, size_t in_f,
                        size_t out_f, hipStream_t stream) {
    if (!gemv_f32act_groups(dtype, in_f)) return false;
    if (out_f == 0) return true;
    const int rows_per_wg = gemv_f32act_group_rows(out_f, in_f);
    f32act_launch(in_f, (unsigned)((out_f + rows_per_wg - 1) / rows_per_wg), w, bpr, x, y, out_f, rows_per_wg, nullptr, stream);
    return true;
}

bool launch_gemv_f32act_group(int dtype, size_t in_f, const GemvTile* tiles_dev, int n_tiles, hipStream_t stream) {
    if (!gemv_f32act_groups(dtype, in_f) || tiles_dev == nullptr) return false;
    if (n_tiles <= 0) return true;
    f32act_launch(in_f, (unsigned)n_tiles, nullptr, 0, nullptr, nullptr, 0, 0, tiles_dev, stream);
    return true;
}

}  // namespace infr
