// Pieces shared by the tiled int8-MFMA kernels (32 or 64 activation rows x 128 weight rows per
// workgroup): the activation tile in LDS, its double-buffered staging, and the tile maps that say
// which rows a workgroup's tile stands for (consecutive tokens, or routed pairs bucketed by expert).
#pragma once

#include "device_common.hpp"

namespace infr {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));

constexpr int kActRowBytes = 256 + 16;  // padded LDS row: conflict-free 16-byte reads and writes

// LDS per workgroup: activation bytes | per-token scale | per-token split bsums (f16 x 16)
template <int BM>
struct MmqLds {
    static constexpr int qs_off = 0;
    static constexpr int d_off = BM * kActRowBytes;
    static constexpr int bs_off = d_off + BM * 4;
    static constexpr int bytes = bs_off + BM * 32;
};

// Activation-tile staging, split in two halves so the global loads of block b+1 are in flight
// while block b is multiplied: fetch() issues the loads into registers, store() writes them to the
// LDS buffer once the previous readers of that buffer are past their barrier.
template <int BM>
struct ActStage {
    static constexpr int kChunks = BM * 16 / 256;       // 16-byte chunks per thread
    static constexpr int kSums = (BM * 8 + 255) / 256;  // per-32 sums per thread
    v4i q[kChunks];
    int bs[kSums];
    float d;

    // Activation rows of this thread's pieces, resolved once per tile: `row_of(t)` maps tile slot
    // t to a row of the quantized activations. Slots past the tile's last row repeat a valid row:
    // their outputs are computed and never stored.
    int q_row[kChunks], bs_row[kSums], d_row;
    template <typename RowOf>
    __device__ __forceinline__ void resolve(int tid, RowOf row_of) {
#pragma unroll
        for (int i = 0; i < kChunks; ++i) q_row[i] = row_of((tid + i * 256) >> 4);
#pragma unroll
        for (int i = 0; i < kSums; ++i) bs_row[i] = row_of(min(tid + i * 256, BM * 8 - 1) >> 3);
        d_row = row_of(min(tid, BM - 1));
    }

    __device__ __forceinline__ void fetch(const int8_t* qs, const float* d8, const int32_t* bsums,
                                          int nb, int b, int tid) {
        const size_t in_f = (size_t)nb * 256;
#pragma unroll
        for (int i = 0; i < kChunks; ++i) {
            const int kc = (tid + i * 256) & 15;
            q[i] = *reinterpret_cast<const v4i*>(qs + (size_t)q_row[i] * in_f + (size_t)b * 256 + kc * 16);
        }
#pragma unroll
        for (int i = 0; i < kSums; ++i) {
            const int s = min(tid + i * 256, BM * 8 - 1) & 7;
            bs[i] = bsums[(size_t)bs_row[i] * (nb * 8) + b * 8 + s];
        }
        d = d8[(size_t)d_row * nb + b];
    }

    __device__ __forceinline__ void store(uint8_t* buf, int tid) const {
#pragma unroll
        for (int i = 0; i < kChunks; ++i) {
            const int c = tid + i * 256, t = c >> 4, kc = c & 15;
            *reinterpret_cast<v4i*>(buf + MmqLds<BM>::qs_off + t * kActRowBytes + kc * 16) = q[i];
        }
#pragma unroll
        for (int i = 0; i < kSums; ++i) {
            const int c = tid + i * 256, t = c >> 3, s = c & 7;
            if (c < BM * 8) {
                const int lo = bs[i] & 63;  // bsum = 64 * hi + lo, 0 <= lo < 64; both exact in f16
                _Float16* p = reinterpret_cast<_Float16*>(buf + MmqLds<BM>::bs_off + t * 32);
                p[s] = (_Float16)lo;
                p[8 + s] = (_Float16)(bs[i] - lo);
            }
        }
        if (tid < BM) reinterpret_cast<float*>(buf + MmqLds<BM>::d_off)[tid] = d;
    }
};

// Which rows a workgroup's tile of BM slots stands for.
// Dense: tile blockIdx.y is tokens [BM * y, BM * y + BM) of an [m, in_f] activation and writes the
// same rows of y.
struct DenseTiles {
    int m;
    __device__ __forceinline__ bool select(int /*tile*/, size_t& /*w_off*/) const { return true; }
    __device__ __forceinline__ int count(int tile, int bm) const { return min(bm, m - tile * bm); }
    __device__ __forceinline__ int act_row(int tile, int bm, int t) const { return min(tile * bm + t, m - 1); }
    __device__ __forceinline__ int out_row(int tile, int bm, int t) const { return tile * bm + t; }
};
// Gathered (routed experts): tile i covers `count[i]` entries of `perm` starting at `slot0[i]`, all
// routed to expert `expert[i]`, whose weights start `expert_stride` bytes apart. An entry p is a
// (token, rank) pair: it reads activation row p / act_div and writes output row p. Tiles at or
// past `*n_tiles` do not exist (the grid is sized for the worst case).
struct GatheredTiles {
    const int32_t* n_tiles;
    const int32_t* expert;
    const int32_t* slot0;
    const int32_t* count_;
    const int32_t* perm;
    size_t expert_stride;
    int act_div;
    __device__ __forceinline__ bool select(int tile, size_t& w_off) const {
        if (tile >= *n_tiles) return false;
        w_off = (size_t)expert[tile] * expert_stride;
        return true;
    }
    __device__ __forceinline__ int count(int tile, int /*bm*/) const { return count_[tile]; }
    __device__ __forceinline__ int act_row(int tile, int /*bm*/, int t) const {
        return perm[slot0[tile] + min(t, count_[tile] - 1)] / act_div;
    }
    __device__ __forceinline__ int out_row(int tile, int /*bm*/, int t) const {
        return perm[slot0[tile] + min(t, count_[tile] - 1)];
    }
};

}  // namespace infr
