// Shared device helpers for the gfx950 kernels: wave64 cross-lane primitives, f16 widening,
// packed-int8 unpack helpers. Everything here is compiled with -ffp-contract=off: the f32
// epilogues restate infr-cpu's expressions, which never fuse a multiply with an add unless the
// CPU code calls mul_add (then __builtin_fmaf is written out here).
#pragma once

#include <type_traits>

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace infr {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;

// half::f16::to_f32 (crates/infr-gguf/src/dequant.rs:68-70): exact widening, v_cvt_f32_f16.
__device__ __forceinline__ float f16_bits_to_f32(uint32_t bits16) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)bits16);
}

// Weights, activations and outputs handed to the kernels always live in device memory, but a
// pointer that reaches a kernel through a table in memory (the per-workgroup tile tables) is a
// generic one to the compiler, and loads through it become FLAT loads. Those count against the
// LDS counter as well as the memory counter, so every wait for an LDS access would also wait for
// the weight loads issued just before it - the prefetch of the next row would never overlap the
// arithmetic of the current one. gload / gstore access a pointer as the global-memory pointer it is.
#ifndef INFR_GLOBAL
#define INFR_GLOBAL __attribute__((address_space(1)))
#endif
template <typename T>
__device__ __forceinline__ T gload(const void* p) {
    return *(const INFR_GLOBAL T*)p;
}
template <typename T>
__device__ __forceinline__ void gstore(void* p, T v) {
    *(INFR_GLOBAL T*)p = v;
}

typedef v4i v4i_a4 __attribute__((aligned(4)));
typedef v4i v4i_a2 __attribute__((aligned(2)));
typedef v4i v4i_a1 __attribute__((aligned(1)));
typedef v2i v2i_a2 __attribute__((aligned(2)));
typedef int v3i __attribute__((ext_vector_type(3)));
typedef v3i v3i_a4 __attribute__((aligned(4)));
typedef v3i v3i_a2 __attribute__((aligned(2)));
typedef int int_a2 __attribute__((aligned(2)));
typedef v2i v2i_a4 __attribute__((aligned(4)));

// 16-byte load from an address that is only 2-byte aligned (Q6_K / Q8_0 / Q2_0 block strides
// are 2 mod 4). gfx950 global loads take any alignment in the HSA unaligned-access mode.
__device__ __forceinline__ v4i load16_a2(const uint8_t* p) { return gload<v4i_a2>(p); }
__device__ __forceinline__ v4i load16(const uint8_t* p) { return gload<v4i>(p); }
__device__ __forceinline__ uint32_t load_u16(const uint8_t* p) { return gload<uint16_t>(p); }

// 16-byte load from a 4-byte-aligned address (a dword-aligned multi-dword load runs at full rate;
// one at 2-byte alignment does not).
__device__ __forceinline__ v4i load16_a4(const uint8_t* p) { return gload<v4i_a4>(p); }
__device__ __forceinline__ int load_u32(const uint8_t* p) { return gload<int>(p); }

// Non-temporal load: for bytes that are read exactly once per launch AND that the wave fetches whole
// 128-byte lines at a time (1024 contiguous bytes per instruction). A read-only pass over 1 GiB
// measured 7.0 TB/s so against 6.2-6.3 TB/s with plain loads; instructions that each touch only a
// part of their lines measured 4.9 TB/s non-temporally (the line is gone when the next one asks).
template <typename T>
__device__ __forceinline__ T gload_stream(const void* p) {
    return __builtin_nontemporal_load((const INFR_GLOBAL T*)p);
}

// Q8_0 blocks (34 B stride) start at a 4-byte boundary or 2 bytes past one, and a 16-byte load at
// 2-byte alignment runs far below full rate (measured: +20 % GEMV bandwidth without them; Q6_K and
// Q2_0, with fewer bytes per misaligned load, measured no gain and keep the plain loads). The
// Q8_0 loader fetches dwords from the boundary at or below the block and realigns in registers:
// realign2(lo, hi, odd) = the four bytes that follow byte 2 (block at the boundary) or byte 4
// (block 2 past it, `odd`) of the eight bytes {lo, hi}.
__device__ __forceinline__ int realign2(int lo, int hi, uint32_t sel) {
    return (int)__builtin_amdgcn_perm((uint32_t)hi, (uint32_t)lo, sel);
}
__device__ __forceinline__ uint32_t realign2_selector(bool odd) { return odd ? 0x07060504u : 0x05040302u; }

// signed int8x4 . int8x4 + acc  (v_dot4_i32_i8)
__device__ __forceinline__ int dot4(int a, int b, int acc) {
    return __builtin_amdgcn_sdot4(a, b, acc, false);
}

// DPP quad permutes: exchange with lane^1 / lane^2 inside each group of four lanes.
__device__ __forceinline__ int quad_xor1(int v) {
    return __builtin_amdgcn_mov_dpp(v, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
}
__device__ __forceinline__ int quad_xor2(int v) {
    return __builtin_amdgcn_mov_dpp(v, 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
}
// Sum over each aligned group of four lanes; every lane of the group gets the total.
__device__ __forceinline__ int quad_sum(int v) {
    v += quad_xor1(v);
    v += quad_xor2(v);
    return v;
}

__device__ __forceinline__ float readlane_f(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// Sum over the 64 lanes without touching LDS: DPP adds inside each row of 16 lanes (quad swaps,
// then the two mirrors leave the row total in every lane), then the four row totals are read out
// as scalars and added in row order. The pairing is fixed, so runs are reproducible. The total is
// valid in every lane.
__device__ __forceinline__ float wave_sum_f(float v) {
    auto dpp_add = [](float x, int ctrl_tag) {
        const int xi = __builtin_bit_cast(int, x);
        int o;
        switch (ctrl_tag) {
        case 0: o = __builtin_amdgcn_mov_dpp(xi, 0xB1, 0xF, 0xF, true); break;   // quad_perm [1,0,3,2]
        case 1: o = __builtin_amdgcn_mov_dpp(xi, 0x4E, 0xF, 0xF, true); break;   // quad_perm [2,3,0,1]
        case 2: o = __builtin_amdgcn_mov_dpp(xi, 0x141, 0xF, 0xF, true); break;  // row_half_mirror
        default: o = __builtin_amdgcn_mov_dpp(xi, 0x140, 0xF, 0xF, true); break; // row_mirror
        }
        return x + __builtin_bit_cast(float, o);
    };
    v = dpp_add(v, 0);
    v = dpp_add(v, 1);
    v = dpp_add(v, 2);
    v = dpp_add(v, 3);
    float s = readlane_f(v, 0);
    s += readlane_f(v, 16);
    s += readlane_f(v, 32);
    s += readlane_f(v, 48);
    return s;
}
// MB per-lane values -> one: lane L returns the sum over its row of 16 lanes of value number
// L % MB. Each transposing stage halves the values a lane carries (it keeps the half its own lane
// bit selects and hands the other half to the partner lane), so reducing MB values costs about
// 3 * (MB - 1) instructions plus the rotations, instead of MB whole-wave reductions. MB in {2, 4, 8}.
template <int MB>
__device__ __forceinline__ float row16_transpose_sum(const float (&v)[MB], int lane) {
    static_assert(MB == 2 || MB == 4 || MB == 8, "2, 4 or 8 values");
    auto dpp = [](float x, auto ctrl) {
        return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, x), decltype(ctrl)::value,
                                                                  0xF, 0xF, true));
    };
    using QuadXor1 = std::integral_constant<int, 0xB1>;    // quad_perm [1,0,3,2]
    using QuadXor2 = std::integral_constant<int, 0x4E>;    // quad_perm [2,3,0,1]
    using HalfMirror = std::integral_constant<int, 0x141>; // lane i <-> 7 - i of each 8
    using Ror4 = std::integral_constant<int, 0x124>;       // rotate right by 4 within the row of 16
    using Ror8 = std::integral_constant<int, 0x128>;
    float a[4];
    if constexpr (MB == 8) {
        // partner L ^ 7 sits in the other half of the 8: lanes with bit 2 keep values 4..7
        const bool up = (lane & 4) != 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) a[j] = (up ? v[4 + j] : v[j]) + dpp(up ? v[j] : v[4 + j], HalfMirror{});
    } else {
#pragma unroll
        for (int j = 0; j < MB; ++j) a[j] = v[j];
    }
    float b[2];
    if constexpr (MB >= 4) {
        const bool odd = (lane & 1) != 0;  // partner L ^ 1: odd lanes keep the odd values
#pragma unroll
        for (int j = 0; j < 2; ++j) b[j] = (odd ? a[2 * j + 1] : a[2 * j]) + dpp(odd ? a[2 * j] : a[2 * j + 1], QuadXor1{});
        const bool hi = (lane & 2) != 0;   // partner L ^ 2: lanes with bit 1 keep value pair 1
        float r = (hi ? b[1] : b[0]) + dpp(hi ? b[0] : b[1], QuadXor2{});
        // lane L: value (L % MB) summed over its 8 (MB == 8) or 4 (MB == 4) lanes
        if constexpr (MB == 4) r += dpp(r, Ror4{});
        return r + dpp(r, Ror8{});
    } else {
        const bool odd = (lane & 1) != 0;
        float r = (odd ? a[1] : a[0]) + dpp(odd ? a[0] : a[1], QuadXor1{});
        r += dpp(r, QuadXor2{});
        r += dpp(r, Ror4{});
        return r + dpp(r, Ror8{});
    }
}

__device__ __forceinline__ int wave_sum_i(int v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

// get_scale_min_k4 for all eight sub-blocks at once (crates/infr-gguf/src/dequant.rs:73-83):
// s0,s1,s2 are the three little-endian words of scales[12]; on return sc8[0..1] hold the eight
// 6-bit scales as bytes and mn8[0..1] the eight 6-bit mins.
__device__ __forceinline__ void k4_all(uint32_t s0, uint32_t s1, uint32_t s2, uint32_t sc8[2],
                                       uint32_t mn8[2]) {
    sc8[0] = s0 & 0x3F3F3F3Fu;
    mn8[0] = s1 & 0x3F3F3F3Fu;
    sc8[1] = (s2 & 0x0F0F0F0Fu) | ((s0 >> 2) & 0x30303030u);
    mn8[1] = ((s2 >> 4) & 0x0F0F0F0Fu) | ((s1 >> 2) & 0x30303030u);
}

// Output (token, row) of a small-batch kernel, with the Op::Add a plan folded into the launch: the
// sum goes to `add_dst` (which may be the residual `add_b` itself, or y: then only the sum is
// stored); every output index is written by exactly one thread.
struct BatchAdd {
    const float* b = nullptr;
    float* dst = nullptr;
};
__device__ __forceinline__ void store_batch_out(float* y, const BatchAdd& a, size_t idx, float v) {
    if (y != a.dst) gstore<float>(y + idx, v);
    if (a.dst) gstore<float>(a.dst + idx, v + a.b[idx]);
}

}  // namespace infr
