// Host-side launch interface of the device kernels. Every launcher validates nothing: the C-ABI
// layer (backend.hip) checks shapes, alignment and buffer sizes before calling in here.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace infr {

// Device-resident quantized activation of m rows of k elements, laid out row-major per field.
// super == true : per-256 `Q8`   (crates/infr-cpu/src/quant.rs:8-25):  d[m][k/256], bsums[m][k/32],
//                 bsums16[m][k/16]
// super == false: per-32 `Q8x32` (quant.rs:90-95): d[m][k/32], bsums[m][k/32]; bsums16 unused.
struct ActQ8 {
    int8_t* qs = nullptr;
    float* d = nullptr;
    int32_t* bsums = nullptr;
    int32_t* bsums16 = nullptr;
};

// quantize_q8 / quantize_q8_32 over m*k contiguous floats.
void launch_quantize_q8(const float* x, size_t m, size_t k, bool per32, const ActQ8& out,
                        hipStream_t stream);

// Optional per-block integer-stage outputs, i32 [m][out_f][blocks] (nullptr = not wanted).
struct IntStages {
    int32_t* a = nullptr;
    int32_t* b = nullptr;
};

// Decode GEMV, m == 1: y[o] = vec_dot(row o, act) for out_f rows of `bpr` bytes each.
// Returns false when (dtype, in_f) has no kernel.
bool launch_gemv(int dtype, const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t in_f,
                 size_t out_f, const IntStages& st, hipStream_t stream);

// m >= 2: int8 MFMA GEMM over on-device quantized activations. y is [m][out_f] row-major.
bool launch_mmq(int dtype, const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m,
                size_t in_f, size_t out_f, const IntStages& st, hipStream_t stream);

}  // namespace infr
