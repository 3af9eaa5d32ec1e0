// One wavefront quantizes 256 consecutive floats (one float4 per lane), bit-exact with infr-cpu:
//   quantize_q8    (crates/infr-cpu/src/quant.rs:27-58)  per 256 elements, f32 scale, i32 sums
//   quantize_q8_32 (crates/infr-cpu/src/quant.rs:97-117) per 32 elements
// amax is an order-independent maximum, `amax / 127` and `1 / d` are IEEE-correct divisions (no
// reciprocal approximation), `round` is half away from zero (roundf). The outputs may live in
// global memory or in LDS.
#pragma once

#include "device_common.hpp"

namespace infr {

// The arithmetic alone: this lane's four codes (packed little-endian), the block scale, and the
// code sums over the lane's 16- and 32-element groups (valid in every lane of the group).
template <bool PER32>
__device__ __forceinline__ void quantize_chunk_values(v4f v, uint32_t& packed, float& dd, int& s32,
                                                      int& s16) {
    float amax = __builtin_fmaxf(__builtin_fmaxf(__builtin_fabsf(v.x), __builtin_fabsf(v.y)),
                                 __builtin_fmaxf(__builtin_fabsf(v.z), __builtin_fabsf(v.w)));
    // Maximum over the block's lanes: 8 lanes (32 floats) or all 64 (256 floats).
#pragma unroll
    for (int off = 1; off < (PER32 ? 8 : 64); off <<= 1)
        amax = __builtin_fmaxf(amax, __shfl_xor(amax, off, kWave));

    dd = amax / 127.0f;
    const float id = dd > 0.0f ? 1.0f / dd : 0.0f;

    auto q1 = [id](float f) -> int {
        float r = roundf(f * id);
        r = r < -127.0f ? -127.0f : r;
        r = r > 127.0f ? 127.0f : r;
        return (int)r;
    };
    const int q0 = q1(v.x), q1_ = q1(v.y), q2 = q1(v.z), q3 = q1(v.w);
    packed = (uint32_t)(q0 & 0xFF) | ((uint32_t)(q1_ & 0xFF) << 8) | ((uint32_t)(q2 & 0xFF) << 16) |
             ((uint32_t)(q3 & 0xFF) << 24);
    int s = q0 + q1_ + q2 + q3;  // 4 elements
    s += __shfl_xor(s, 1, kWave);
    s += __shfl_xor(s, 2, kWave);  // 16 elements: lanes 4g..4g+3
    s16 = s;
    s += __shfl_xor(s, 4, kWave);  // 32 elements: lanes 8g..8g+7
    s32 = s;
}

// `chunk` indexes 256-float chunks of the output arrays; `live` is false for lanes past the end of
// a per-32 input that stops inside the chunk (whole 8-lane groups at a time).
template <bool PER32>
__device__ __forceinline__ void quantize_chunk(v4f v, bool live, int lane, size_t chunk,
                                               int8_t* qs, float* d, int32_t* bsums,
                                               int32_t* bsums16) {
    uint32_t packed;
    float dd;
    int s, s16;
    quantize_chunk_values<PER32>(v, packed, dd, s, s16);
    if (live) reinterpret_cast<uint32_t*>(qs)[chunk * 64 + lane] = packed;

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

}  // namespace infr
