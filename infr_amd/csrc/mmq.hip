// Prefill GEMM (m >= 2) of block-quantized weights against on-device int8-quantized activations.
//
// Q4_K runs on the int8 matrix cores. Per 256-element block infr-cpu computes, per output,
//     sd = sum_s sc_s * (sum_l q4 * q8)     sm = sum_s m_s * bsums_s
//     y += q8.d[b] * (d * (f32)sd - dmin * (f32)sm)            (crates/infr-cpu/src/kernels.rs:151-184)
// with 6-bit sc_s, m_s per 32-element sub-block. The MFMA accumulates over K inside the
// instruction, so a per-sub-block scale has to be inside the operand. q4 * sc_s needs 10 bits, so
// the scale is split sc = 8 * sc_hi + sc_lo (3 bits each): q4 * sc_lo and q4 * sc_hi both fit int8,
// two v_mfma_i32_32x32x32_i8 chains run over the whole block, and sd = lo + 8 * hi exactly.
// (The alternative, one K=32 MFMA per sub-block followed by a VALU multiply, runs the legacy
// half-rate instruction and needs eight integer multiply-adds per output per block.)
// sm is a K = 16 product of the mins with the activation's per-32 sums split as bsum = lo + 64*hi
// (both exact in f16): one v_mfma_f32_32x32x16_f16 whose f32 result is the exact integer.
// The f32 epilogue then evaluates the CPU expression with separate multiplies and adds, and each
// output accumulates its blocks in ascending order, so y is bit-identical to infr-cpu's batch
// kernel (and to this library's m == 1 GEMV).
//
// Tiling. Tokens are the MFMA's M (rows of C), weight rows its N (columns): a lane's 16
// accumulators then share one weight row, so d, dmin and the pre-scaled operand are per lane.
// A workgroup (4 waves) covers BM tokens x 128 weight rows; each wave owns 32 weight rows for all
// BM tokens, loads and unpacks its rows' blocks straight from global memory into MFMA B operands
// (no LDS for weights, no redundant unpacking), and reads the activation tile, shared by the four
// waves, from LDS. Per 256-block and 32x32 output tile: 16 int8 MFMAs + 1 f16 MFMA against
// 7 VALU instructions per output for the epilogue.
//
// Small batches (m <= 8) and the other formats take the multi-activation dot4 GEMV (gemv.hip).
#include <cstdlib>

#include "device_common.hpp"
#include "kernels.hpp"

namespace infr {

typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
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

struct Q4kRaw {
    v4i hdr, q[4];
};

__device__ __forceinline__ void q4k_load_raw(Q4kRaw& r, const uint8_t* blk, int h, bool ok) {
    if (ok) {
        r.hdr = load16(blk);
#pragma unroll
        for (int p = 0; p < 4; ++p) r.q[p] = load16(blk + 16 + p * 32 + h * 16);
    } else {
        r.hdr = v4i{0, 0, 0, 0};
#pragma unroll
        for (int p = 0; p < 4; ++p) r.q[p] = v4i{0, 0, 0, 0};
    }
}

// Packed byte-wise multiply of four codes (<= 15) by a scale digit (<= 7): no byte overflows, so
// two 16-bit lane multiplies do it.
__device__ __forceinline__ int scale_codes(uint32_t codes, uint32_t digit) {
    typedef unsigned short us2 __attribute__((ext_vector_type(2)));
    const us2 c = __builtin_bit_cast(us2, codes);
    const us2 s = {(unsigned short)digit, (unsigned short)digit};
    return __builtin_bit_cast(int, (us2)(c * s));
}

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

    __device__ __forceinline__ void fetch(const int8_t* qs, const float* d8, const int32_t* bsums,
                                          int tok0, int m, int nb, int b, int tid) {
        const size_t in_f = (size_t)nb * 256;
#pragma unroll
        for (int i = 0; i < kChunks; ++i) {
            // Tokens past m are clamped to the last row: their outputs are computed and never stored.
            const int c = tid + i * 256, t = c >> 4, kc = c & 15, tok = min(tok0 + t, m - 1);
            q[i] = *reinterpret_cast<const v4i*>(qs + (size_t)tok * in_f + (size_t)b * 256 + kc * 16);
        }
#pragma unroll
        for (int i = 0; i < kSums; ++i) {
            const int c = min(tid + i * 256, BM * 8 - 1), t = c >> 3, s = c & 7, tok = min(tok0 + t, m - 1);
            bs[i] = bsums[(size_t)tok * (nb * 8) + b * 8 + s];
        }
        d = d8[(size_t)min(tok0 + min(tid, BM - 1), m - 1) * nb + b];
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

template <int BM, bool STAGES>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(BM == 32 ? 3 : 2, BM == 32 ? 3 : 2)))
void mmq_q4k_kernel(const uint8_t* __restrict__ w, size_t bpr,
                                                      const int8_t* __restrict__ qs,
                                                      const float* __restrict__ d8,
                                                      const int32_t* __restrict__ bsums,
                                                      float* __restrict__ y, int m, int out_f, int nb,
                                                      int32_t* __restrict__ st_sd,
                                                      int32_t* __restrict__ st_sm) {
    constexpr int TB = BM / 32;  // token blocks of 32
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];  // two MmqLds<BM> buffers
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, h = lane >> 5;
    const int tok0 = blockIdx.y * BM;
    const int wrow = blockIdx.x * 128 + wave * 32 + col;
    const bool row_ok = wrow < out_f;
    const uint8_t* wrowp = w + (size_t)(row_ok ? wrow : 0) * bpr;

    v16f acc[TB];
#pragma unroll
    for (int tb = 0; tb < TB; ++tb)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[tb][i] = 0.0f;

    ActStage<BM> stage;
    stage.fetch(qs, d8, bsums, tok0, m, nb, 0, tid);
    Q4kRaw raw;
    q4k_load_raw(raw, wrowp, h, row_ok);
    stage.store(lds, tid);
    __syncthreads();

    for (int b = 0; b < nb; ++b) {
        const uint8_t* tile = lds + (b & 1) * MmqLds<BM>::bytes;
        // ---- request block b+1: activation tile into registers, this wave's weight rows ----
        const Q4kRaw cur = raw;
        if (b + 1 < nb) {
            stage.fetch(qs, d8, bsums, tok0, m, nb, b + 1, tid);
            q4k_load_raw(raw, wrowp + (size_t)(b + 1) * 144, h, row_ok);
        }

        // ---- this wave's 32 weight rows of block b -> MFMA B operands (registers) ----
        uint32_t sc8[2], mn8[2];
        k4_all((uint32_t)cur.hdr.y, (uint32_t)cur.hdr.z, (uint32_t)cur.hdr.w, sc8, mn8);
        const float d = f16_bits_to_f32((uint32_t)cur.hdr.x & 0xFFFFu);
        const float dmin = f16_bits_to_f32((uint32_t)cur.hdr.x >> 16);
        v4i blo[8], bhi[8];
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const int qw[4] = {cur.q[p].x, cur.q[p].y, cur.q[p].z, cur.q[p].w};
#pragma unroll
            for (int e = 0; e < 2; ++e) {  // e = 0: sub-block 2p (low nibbles), 1: 2p+1 (high)
                const int s = 2 * p + e;
                const uint32_t sc = (sc8[s >> 2] >> (8 * (s & 3))) & 0xFFu;
                const uint32_t lo3 = sc & 7u, hi3 = sc >> 3;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t codes = ((uint32_t)qw[k] >> (4 * e)) & 0x0F0F0F0Fu;
                    blo[s][k] = scale_codes(codes, lo3);
                    bhi[s][k] = scale_codes(codes, hi3);
                }
            }
        }
        // mins as f16 for the K=16 product: k-slots 0..7 pair with bsum lo, 8..15 with 64*hi
        v8h bm;
#pragma unroll
        for (int s = 0; s < 8; ++s) bm[s] = (_Float16)(int)((mn8[s >> 2] >> (8 * (s & 3))) & 0xFFu);

#pragma unroll
        for (int tb = 0; tb < TB; ++tb) {
            const v16i zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            const v16f zf = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            const uint8_t* arow = tile + MmqLds<BM>::qs_off + (tb * 32 + col) * kActRowBytes + h * 16;
            v4i a = *reinterpret_cast<const v4i*>(arow);
            v16i alo = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, blo[0], zi, 0, 0, 0);
            v16i ahi = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, bhi[0], zi, 0, 0, 0);
#pragma unroll
            for (int s = 1; s < 8; ++s) {
                a = *reinterpret_cast<const v4i*>(arow + s * 32);
                alo = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, blo[s], alo, 0, 0, 0);
                ahi = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, bhi[s], ahi, 0, 0, 0);
            }
            const v8h abs_ = *reinterpret_cast<const v8h*>(tile + MmqLds<BM>::bs_off + (tb * 32 + col) * 32 + h * 16);
            const v16f smf = __builtin_amdgcn_mfma_f32_32x32x16_f16(abs_, bm, zf, 0, 0, 0);
            // epilogue: accumulator i of this lane is token 8*(i/4) + 4*h + i%4 of the block
            const float* dtile = reinterpret_cast<const float*>(tile + MmqLds<BM>::d_off) + tb * 32 + 4 * h;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const v4f dq = *reinterpret_cast<const v4f*>(dtile + 8 * j);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int r = 4 * j + i;
                    const int sd = alo[r] + (ahi[r] << 3);
                    if (STAGES) {
                        const int tok = tok0 + tb * 32 + 8 * j + 4 * h + i;
                        if (row_ok && tok < m) {
                            st_sd[((size_t)tok * out_f + wrow) * nb + b] = sd;
                            st_sm[((size_t)tok * out_f + wrow) * nb + b] = (int)smf[r];
                        }
                    }
                    // sumf += q8.d[b] * (d * sd as f32 - dmin * sm as f32)
                    acc[tb][r] += dq[i] * (d * (float)sd - dmin * smf[r]);
                }
            }
        }

        // ---- publish block b+1 in the other buffer (its last readers passed the previous barrier)
        if (b + 1 < nb) stage.store(lds + ((b + 1) & 1) * MmqLds<BM>::bytes, tid);
        __syncthreads();
    }

    if (!row_ok) return;
#pragma unroll
    for (int tb = 0; tb < TB; ++tb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int tok = tok0 + tb * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
            if (tok < m) y[(size_t)tok * out_f + wrow] = acc[tb][r];
        }
}

// ───────────────────────────── skinny form: up to 32 tokens per workgroup ─────────────────────────────
// With few tokens there are too few 32 x 128 output tiles to fill the chip, and a wave that walks
// all of K alone is serial for nb blocks. Here a workgroup owns 32 weight rows x 32 tokens and
// splits K over its NW waves: in every round wave w takes block round*NW + w - loads its weight
// rows and the activation fragments straight from global memory (L2), unpacks, runs the same 17
// MFMAs - and parks the exact per-block integers (sd, sm) in LDS. After a barrier all NW*64
// threads run the f32 epilogue, each for 16/NW of a lane position's outputs, walking the round's
// blocks in ascending order: the same operations in the same order as the CPU, so the result is
// bit-identical to the tiled kernel and the GEMV, at NW-fold K parallelism.
template <int NW, bool STAGES>
__global__ __launch_bounds__(NW * 64) void mmq_skinny_q4k_kernel(
    const uint8_t* __restrict__ w, size_t bpr, const int8_t* __restrict__ qs,
    const float* __restrict__ d8, const int32_t* __restrict__ bsums, float* __restrict__ y, int m,
    int out_f, int nb, int32_t* __restrict__ st_sd, int32_t* __restrict__ st_sm) {
    constexpr int RG = 16 / NW;  // accumulators per epilogue thread
    typedef int vrgi __attribute__((ext_vector_type(RG)));
    typedef float vrgf __attribute__((ext_vector_type(RG)));
    __shared__ __attribute__((aligned(16))) int sd_l[NW][NW][64][RG];    // [writer][reader group][lane]
    __shared__ __attribute__((aligned(16))) float sm_l[NW][NW][64][RG];
    __shared__ float dd_l[NW][32][2];                                    // d, dmin per writer and row
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, h = lane >> 5;
    const int tok0 = blockIdx.y * 32;
    const int wrow = blockIdx.x * 32 + col;
    const bool row_ok = wrow < out_f;
    const uint8_t* wrowp = w + (size_t)(row_ok ? wrow : 0) * bpr;
    const size_t in_f = (size_t)nb * 256;
    const int atok = min(tok0 + col, m - 1);  // this lane's activation row as MFMA A operand
    // tokens of this thread's epilogue outputs: accumulator r = RG*wave + i of lane position `lane`
    int etok[RG];
#pragma unroll
    for (int i = 0; i < RG; ++i) {
        const int r = RG * wave + i;
        etok[i] = tok0 + 8 * (r >> 2) + 4 * h + (r & 3);
    }
    float acc[RG];
#pragma unroll
    for (int i = 0; i < RG; ++i) acc[i] = 0.0f;

    // Everything a round reads from global memory is requested one round ahead: the weight rows
    // (HBM), the activation fragments, per-32 sums and scales (L2).
    struct RoundIn {
        Q4kRaw raw;
        v4i a[8], bs0, bs1;
        float dq[NW][RG];
    };
    auto request = [&](RoundIn& in, int round) {
        const int b = round * NW + wave;
        const bool has = b < nb;
        const int bc = has ? b : 0;
        const int8_t* ap = qs + (size_t)atok * in_f + (size_t)bc * 256 + h * 16;
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) in.a[sb] = *reinterpret_cast<const v4i*>(ap + sb * 32);
        in.bs0 = *reinterpret_cast<const v4i*>(bsums + (size_t)atok * (nb * 8) + bc * 8);
        in.bs1 = *reinterpret_cast<const v4i*>(bsums + (size_t)atok * (nb * 8) + bc * 8 + 4);
#pragma unroll
        for (int j = 0; j < NW; ++j)
#pragma unroll
            for (int i = 0; i < RG; ++i) {
                const int bj = min(round * NW + j, nb - 1);
                in.dq[j][i] = d8[(size_t)min(etok[i], m - 1) * nb + bj];
            }
        q4k_load_raw(in.raw, wrowp + (size_t)bc * 144, h, row_ok && has);
    };
    RoundIn nxt;
    request(nxt, 0);
    const int rounds = (nb + NW - 1) / NW;
    for (int round = 0; round < rounds; ++round) {
        const int b = round * NW + wave;
        const bool has = b < nb;
        const RoundIn in = nxt;
        if (round + 1 < rounds) request(nxt, round + 1);
        const Q4kRaw& cur = in.raw;
        const v4i (&a)[8] = in.a;
        const float (&dq)[NW][RG] = in.dq;
        if (has) {
            const v4i bs0 = in.bs0, bs1 = in.bs1;

            uint32_t sc8[2], mn8[2];
            k4_all((uint32_t)cur.hdr.y, (uint32_t)cur.hdr.z, (uint32_t)cur.hdr.w, sc8, mn8);
            v4i blo[8], bhi[8];
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const int qw[4] = {cur.q[p].x, cur.q[p].y, cur.q[p].z, cur.q[p].w};
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const int sb = 2 * p + e;
                    const uint32_t sc = (sc8[sb >> 2] >> (8 * (sb & 3))) & 0xFFu;
                    const uint32_t lo3 = sc & 7u, hi3 = sc >> 3;
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const uint32_t codes = ((uint32_t)qw[k] >> (4 * e)) & 0x0F0F0F0Fu;
                        blo[sb][k] = scale_codes(codes, lo3);
                        bhi[sb][k] = scale_codes(codes, hi3);
                    }
                }
            }
            v8h bm;
#pragma unroll
            for (int sb = 0; sb < 8; ++sb) bm[sb] = (_Float16)(int)((mn8[sb >> 2] >> (8 * (sb & 3))) & 0xFFu);
            // per-32 sums split bsum = lo + 64*hi': the h = 0 lanes carry lo, the h = 1 lanes bsum - lo
            const int bsv[8] = {bs0.x, bs0.y, bs0.z, bs0.w, bs1.x, bs1.y, bs1.z, bs1.w};
            v8h abs_;
#pragma unroll
            for (int sb = 0; sb < 8; ++sb) {
                const int lo = bsv[sb] & 63;
                abs_[sb] = (_Float16)(h ? bsv[sb] - lo : lo);
            }
            const v16i zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            const v16f zf = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            v16i alo = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[0], blo[0], zi, 0, 0, 0);
            v16i ahi = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[0], bhi[0], zi, 0, 0, 0);
#pragma unroll
            for (int sb = 1; sb < 8; ++sb) {
                alo = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[sb], blo[sb], alo, 0, 0, 0);
                ahi = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[sb], bhi[sb], ahi, 0, 0, 0);
            }
            const v16f smf = __builtin_amdgcn_mfma_f32_32x32x16_f16(abs_, bm, zf, 0, 0, 0);
#pragma unroll
            for (int g = 0; g < NW; ++g) {
                vrgi sdv;
                vrgf smv;
#pragma unroll
                for (int i = 0; i < RG; ++i) {
                    const int r = RG * g + i;
                    sdv[i] = alo[r] + (ahi[r] << 3);
                    smv[i] = smf[r];
                    if (STAGES) {
                        const int tok = tok0 + 8 * (r >> 2) + 4 * h + (r & 3);
                        if (row_ok && tok < m) {
                            st_sd[((size_t)tok * out_f + wrow) * nb + b] = sdv[i];
                            st_sm[((size_t)tok * out_f + wrow) * nb + b] = (int)smv[i];
                        }
                    }
                }
                *reinterpret_cast<vrgi*>(&sd_l[wave][g][lane][0]) = sdv;
                *reinterpret_cast<vrgf*>(&sm_l[wave][g][lane][0]) = smv;
            }
            if (h == 0) {
                dd_l[wave][col][0] = f16_bits_to_f32((uint32_t)cur.hdr.x & 0xFFFFu);
                dd_l[wave][col][1] = f16_bits_to_f32((uint32_t)cur.hdr.x >> 16);
            }
        }
        __syncthreads();
        // f32 epilogue, blocks in ascending order: sumf += q8.d[b] * (d * sd as f32 - dmin * sm as f32)
#pragma unroll
        for (int j = 0; j < NW; ++j) {
            if (round * NW + j < nb) {
                const vrgi sdv = *reinterpret_cast<const vrgi*>(&sd_l[j][wave][lane][0]);
                const vrgf smv = *reinterpret_cast<const vrgf*>(&sm_l[j][wave][lane][0]);
                const float d = dd_l[j][col][0], dmin = dd_l[j][col][1];
#pragma unroll
                for (int i = 0; i < RG; ++i) acc[i] += dq[j][i] * (d * (float)sdv[i] - dmin * smv[i]);
            }
        }
        __syncthreads();
    }
    if (!row_ok) return;
#pragma unroll
    for (int i = 0; i < RG; ++i)
        if (etok[i] < m) y[(size_t)etok[i] * out_f + wrow] = acc[i];
}

template <int NW>
static void launch_mmq_skinny_q4k(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m,
                                  size_t in_f, size_t out_f, const IntStages& st, hipStream_t stream) {
    const dim3 grid((unsigned)((out_f + 31) / 32), (unsigned)((m + 31) / 32)), block(NW * 64);
    const int nb = (int)(in_f / 256);
    if (st.a)
        hipLaunchKernelGGL((mmq_skinny_q4k_kernel<NW, true>), grid, block, 0, stream, w, bpr, act.qs, act.d,
                           act.bsums, y, (int)m, (int)out_f, nb, st.a, st.b);
    else
        hipLaunchKernelGGL((mmq_skinny_q4k_kernel<NW, false>), grid, block, 0, stream, w, bpr, act.qs, act.d,
                           act.bsums, y, (int)m, (int)out_f, nb, (int32_t*)nullptr, (int32_t*)nullptr);
}

template <int BM>
static void launch_mmq_q4k(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m,
                           size_t in_f, size_t out_f, const IntStages& st, hipStream_t stream) {
    const dim3 grid((unsigned)((out_f + 127) / 128), (unsigned)((m + BM - 1) / BM)), block(256);
    const int nb = (int)(in_f / 256);
    if (st.a)
        hipLaunchKernelGGL((mmq_q4k_kernel<BM, true>), grid, block, 2 * MmqLds<BM>::bytes, stream, w, bpr,
                           act.qs, act.d, act.bsums, y, (int)m, (int)out_f, nb, st.a, st.b);
    else
        hipLaunchKernelGGL((mmq_q4k_kernel<BM, false>), grid, block, 2 * MmqLds<BM>::bytes, stream, w, bpr,
                           act.qs, act.d, act.bsums, y, (int)m, (int)out_f, nb, (int32_t*)nullptr,
                           (int32_t*)nullptr);
}

bool launch_mmq(int dtype, const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m,
                size_t in_f, size_t out_f, const IntStages& st, hipStream_t stream) {
    // Small batches and the formats without an MFMA kernel: dot4 GEMV with the activations of up to
    // eight rows in registers (weights re-streamed once per eight rows beyond that).
    static const int env_mfma_min = getenv("INFR_HIP_MMQ_MIN_M") ? atoi(getenv("INFR_HIP_MMQ_MIN_M")) : 2;
    static const int env_skinny_max = getenv("INFR_HIP_MMQ_SKINNY_MAX_M") ? atoi(getenv("INFR_HIP_MMQ_SKINNY_MAX_M")) : 32;
    if (dtype != 12 || (int)m < env_mfma_min)
        return launch_gemv_batch(dtype, w, bpr, act, y, m, in_f, out_f, st, stream);
    if ((int)m <= env_skinny_max) {
        // K split over the waves of a workgroup: four blocks per round; eight for long rows or when
        // four would leave most SIMDs without a wave
        static const int env_nw = getenv("INFR_HIP_MMQ_SKINNY_WAVES") ? atoi(getenv("INFR_HIP_MMQ_SKINNY_WAVES")) : 0;
        const size_t wgs = (out_f + 31) / 32 * ((m + 31) / 32);
        const bool eight = env_nw ? env_nw == 8 : (in_f >= 8192 || (wgs * 4 < 1024 && in_f >= 2048));
        if (eight) launch_mmq_skinny_q4k<8>(w, bpr, act, y, m, in_f, out_f, st, stream);
        else launch_mmq_skinny_q4k<4>(w, bpr, act, y, m, in_f, out_f, st, stream);
        return true;
    }
    if (dtype == 12) {
        static const int env_bm = getenv("INFR_HIP_MMQ_BM") ? atoi(getenv("INFR_HIP_MMQ_BM")) : 0;
        // 64-token tiles amortise the weight unpack over two token blocks at two waves per SIMD and
        // measured ~10-14 % faster than 32-token tiles (three waves per SIMD) from M = 512 up; below
        // that the 32-token grid fills the chip better. 128-token tiles spill.
        const size_t bm = env_bm ? (size_t)env_bm : (m >= 256 ? 64 : 32);
        if (bm <= 32) launch_mmq_q4k<32>(w, bpr, act, y, m, in_f, out_f, st, stream);
        else if (bm <= 64) launch_mmq_q4k<64>(w, bpr, act, y, m, in_f, out_f, st, stream);
        else launch_mmq_q4k<128>(w, bpr, act, y, m, in_f, out_f, st, stream);
        return true;
    }
    return false;
}

}  // namespace infr
