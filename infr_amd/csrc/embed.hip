// Op::EmbedGather: dst[r, :] = decode(table[ids[r], :]) * scale (crates/infr-core/src/graph.rs:853-865;
// CPU arm crates/infr-cpu/src/lib.rs:2084-2111). The table stays in its GGUF block format in HBM and
// only the rows asked for are decoded, one thread per element, with the host decode's arithmetic
// (crates/infr-gguf/src/dequant.rs:11-51: `sc * code + mn` with sc and mn each rounded to f32 first;
// codebook formats d * value), so every output equals `bytes_to_f32(row)[e] * scale` bit for bit.
// A token id outside the table yields a row of NaN (the CPU backend panics on the slice); nothing
// is read out of bounds. HBM-bound on rows * (row bytes + 4 * ne), a few MB per prefill.
#include "decode_element.hpp"
#include "kernels.hpp"

namespace infr {

namespace {

__global__ __launch_bounds__(256) void embed_gather_kernel(int dtype, const uint8_t* __restrict__ table,
                                                           size_t bpr, int total_rows,
                                                           const int32_t* __restrict__ ids, int ne,
                                                           float scale, float* __restrict__ dst) {
    const int r = blockIdx.y;
    const int e = (int)blockIdx.x * 256 + (int)threadIdx.x;
    if (e >= ne) return;
    const int tok = ids[r];
    float v;
    if (tok < 0 || tok >= total_rows) v = __builtin_nanf("");
    else v = decode_element(dtype, table + (size_t)tok * bpr, e) * scale;
    dst[(size_t)r * ne + e] = v;
}

}  // namespace

bool embed_gather_supported(int dtype) {
    switch (dtype) {
    case 0: case 1: case 30: case 2: case 3: case 6: case 7: case 8: case 10: case 11: case 12: case 13: case 14: case 20:
    case 23: case 34: case 35: case 39: case 40: case 42:
        return true;
    default: return false;
    }
}

void launch_embed_gather(int dtype, const uint8_t* table, size_t bpr, size_t total_rows, const int32_t* ids,
                         size_t rows, size_t ne, float scale, float* dst, hipStream_t stream) {
    if (rows == 0 || ne == 0) return;
    hipLaunchKernelGGL(embed_gather_kernel, dim3((unsigned)((ne + 255) / 256), (unsigned)rows), dim3(256), 0, stream,
                       dtype, table, bpr, (int)total_rows, ids, (int)ne, scale, dst);
}

}  // namespace infr
