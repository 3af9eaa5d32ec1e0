// One wavefront quantizes 256 consecutive floats (one float4 per lane), bit-exact with infr-cpu:
//   quantize_q8    (crates/infr-cpu/src/quant.rs:27-58)  per 256 elements, f32 scale, i32 sums
//   quantize_q8_32 (crates/infr-cpu/src/quant.rs:97-117) per 32 elements
// amax is an order-independent maximum, `amax / 127` and `1 / d` are IEEE-correct divisions (no
// reciprocal approximation), `round` is half away from zero (roundf). The outputs may live in
// global memory or in LDS.
#pragma once

#include <type_traits>

#include "device_common.hpp"

namespace infr {

// Maximum over the lanes of a block without touching LDS: DPP exchanges inside the row of 16 lanes
// (quad swaps, then the mirrors: after the quad steps the four lanes of a quad agree, so mirroring
// the 8 and the 16 brings in exactly the other half), and for 64 lanes the four row maxima are read
// out as scalars. A maximum does not depend on the order, so any pairing gives the CPU's amax.
template <int LANES>
__device__ __forceinline__ float lanes_max(float v) {
    static_assert(LANES == 8 || LANES == 64, "a 32-element or a 256-element block");
    auto step = [](float x, auto ctrl) {
        const int o = __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, x), decltype(ctrl)::value, 0xF, 0xF, true);
        return __builtin_fmaxf(x, __builtin_bit_cast(float, o));
    };
    v = step(v, std::integral_constant<int, 0xB1>{});   // quad_perm [1,0,3,2]
    v = step(v, std::integral_constant<int, 0x4E>{});   // quad_perm [2,3,0,1]
    v = step(v, std::integral_constant<int, 0x141>{});  // row_half_mirror
    if constexpr (LANES == 64) {
        v = step(v, std::integral_constant<int, 0x140>{});  // row_mirror
        v = __builtin_fmaxf(__builtin_fmaxf(readlane_f(v, 0), readlane_f(v, 16)),
                            __builtin_fmaxf(readlane_f(v, 32), readlane_f(v, 48)));
    }
    return v;
}

// The arithmetic alone: this lane's four codes (packed little-endian), the block scale, and the
// code sums over the lane's 16- and 32-element groups (valid in every lane of the group).
template <bool PER32>
__device__ __forceinline__ void quantize_chunk_values(v4f v, uint32_t& packed, float& dd, int& s32,
                                                      int& s16) {
    const float amax = lanes_max<PER32 ? 8 : 64>(
        __builtin_fmaxf(__builtin_fmaxf(__builtin_fabsf(v.x), __builtin_fabsf(v.y)),
                        __builtin_fmaxf(__builtin_fabsf(v.z), __builtin_fabsf(v.w))));
    dd = amax / 127.0f;
    const float id = dd > 0.0f ? 1.0f / dd : 0.0f;

    // `(f * id).round().clamp(-127, 127) as i8`. round() is half away from zero: for |x| < 2^23 that
    // is trunc(x + copysign(0.5 - 2^-25, x)) - adding 0.5 itself would carry 0.49999997 up to 1 -
    // and the conversion to integer truncates by itself. |f * id| <= 127 (1 + 2^-22) < 127.5, so the
    // clamp never changes a finite value; NaN converts to 0 here as it does in the CPU's `as i8`.
    auto q1 = [id](float f) -> int {
        const float x = f * id;
        const float half = __builtin_bit_cast(
            float, (__builtin_bit_cast(uint32_t, x) & 0x80000000u) | 0x3EFFFFFFu);  // copysign(0.49999997, x)
        return (int)(x + half);
    };
    const int q0 = q1(v.x), q1_ = q1(v.y), q2 = q1(v.z), q3 = q1(v.w);
    // low bytes of the four codes: two byte permutes and a shift-or
    const uint32_t lo = __builtin_amdgcn_perm((uint32_t)q1_, (uint32_t)q0, 0x0C0C0400u);
    const uint32_t hi = __builtin_amdgcn_perm((uint32_t)q3, (uint32_t)q2, 0x0C0C0400u);
    packed = lo | (hi << 16);
    int s = dot4((int)packed, 0x01010101, 0);  // the lane's 4 codes
    s = quad_sum(s);                           // 16 elements: lanes 4g..4g+3
    s16 = s;
    s += __builtin_amdgcn_mov_dpp(s, 0x141, 0xF, 0xF, true);  // row_half_mirror: the 8's other quad
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
