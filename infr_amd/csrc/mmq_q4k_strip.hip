// Q4_K prefill GEMM, strip form: 256 tokens x 32 / 64 / 96 weight rows per workgroup of eight waves.
//
// Arithmetic is that of mmq.hip (crates/infr-cpu/src/kernels.rs:151-184 per block and output):
//     sd = sum_s sc_s * (sum_l q4 * q8)   on the int8 matrix cores, the 6-bit scale split into two
//                                         3-bit digits so that q4 * digit is an int8 operand
//     sm = sum_s m_s * bsum_s             one K = 16 f16 MFMA over the split per-32 sums (exact)
//     y += q8.d[b] * (d * (f32)sd - dmin * (f32)sm)     blocks ascending
// sd and sm are exact in every form. The f32 line has two forms: EXACT evaluates it with separate
// multiplies and adds, as infr-cpu writes it, so y is bit-identical to its batch kernel and to the
// other routes of this library (the integer-stage entry point runs that form); the form Op::Linear
// takes from 128 tokens up contracts it into fused multiply-adds - five vector instructions per output
// and block instead of seven, y within ~1e-7 relative of infr-cpu's.
//
// What differs from the other Q4_K kernels is the shape of the work: every workgroup fills a compute
// unit (or half of one), so the strip height is chosen for the grid to come out at whole rounds of
// the device's compute units.
//  - A workgroup owns a strip of KT 32-row tiles (KT = 1, 2 or 3) and 256 tokens. Wave w owns
//    tokens 32w .. 32w+31 for all the strip's rows: KT accumulator tiles per wave. At 512 tokens x 12288
//    rows and KT = 3 that is 256 workgroups - one per compute unit, two waves per SIMD, no second round;
//    4096 rows take KT = 1 for the same 256 workgroups.
//  - Weights: the 12 (row tile, nibble pair) pieces of a block are unpacked by the waves into MFMA
//    B-operand order in LDS (two digit planes, 48 KB per block, double-buffered), one block ahead of
//    the multiplication, from raw bytes requested two blocks ahead. One barrier per block.
//  - Activations: a wave's fragments come straight from the tiled quantizer's layout (every
//    fragment a contiguous KiB) into registers; each is requested again, for the next block, right
//    after its last use in this one.
//  - Inside a wave every MFMA is followed by the seven f32 instructions of one accumulator of the
//    row tile finished before (the matrix core and the vector ALU then work at the same time),
//    and B fragments are read from LDS three MFMAs ahead of their use.
#include <utility>

#include "device_common.hpp"
#include "kernels.hpp"
#include "mmq_tiles.hpp"

namespace infr {

namespace {

typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kNW = 8;            // waves per workgroup, 32 tokens each
constexpr int kStripTokens = 32 * kNW;

template <int kT>  // 32-row tiles per strip
struct StripLds {
    static constexpr int frag = 1024;                    // one B fragment: 64 lanes x 16 B
    static constexpr int b_bytes = 8 * 2 * kT * frag;    // [sub-block][digit plane][row tile]
    static constexpr int mn_off = b_bytes;               // [row tile][row][8] f16 mins
    static constexpr int dd_off = mn_off + kT * 32 * 16; // [row tile][row] (d, dmin)
    static constexpr int bytes = dd_off + kT * 32 * 8;
    static constexpr int dq_off = 2 * bytes;             // [block parity][wave][32] activation scales
    static constexpr int total = dq_off + 2 * kNW * 32 * 4;
};

// Four codes (<= 15) times a scale digit (<= 7), byte-wise: no byte overflows, so two 16-bit lane
// multiplies do it.
__device__ __forceinline__ int scale_codes4(uint32_t codes, uint32_t digit) {
    typedef unsigned short us2 __attribute__((ext_vector_type(2)));
    const us2 c = __builtin_bit_cast(us2, codes);
    const us2 s = {(unsigned short)digit, (unsigned short)digit};
    return __builtin_bit_cast(int, (us2)(c * s));
}

// B fragments are read from LDS several MFMAs ahead of their use. Left to the compiler, each read is
// sunk to just before the MFMA that takes it and the matrix core waits out the LDS latency 48 times
// a block; so the read and its wait are written out. The compiler does not count these reads in
// its own lgkmcnt bookkeeping: LDS accesses complete in order, so its waits can only cover more than
// they need to, never less, and lds_wait<N> is exact when nothing else was issued in between and
// stricter otherwise. That argument holds for LDS traffic only: scalar memory loads share lgkmcnt
// and return out of order, so a scalar load issued between an ahead-read and its lds_wait<N> could
// let the wait pass with the LDS read still outstanding. The block loop therefore has no scalar
// operand that is not in a register before it starts (kernel arguments, strides and table entries
// are all read in the prologue), and the strip route's bit-identity tests at 512 / 1024 / 2048
// tokens would show a stale fragment.
template <int OFFSET>
__device__ __forceinline__ v4i lds_read16_ahead(uint32_t addr) {
    v4i r;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFFSET));
    return r;
}
// Waits until at most N younger LDS accesses are outstanding; `r` is tied so that its consumer
// cannot be moved in front of the wait.
template <int N>
__device__ __forceinline__ void lds_wait(v4i& r) {
    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(r) : "n"(N));
}

template <int... I, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
    (f(std::integral_constant<int, I>{}), ...);
}
// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>), in order
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(std::make_integer_sequence<int, N>{}, static_cast<F&&>(f));
}

// A wave's activation operands of one 256-block: eight A fragments, the split per-32 sums and the
// lane's token scale.
struct ActFrags {
    v4i a[8];
    v8h bs;
    float d;
};

// EXACT: the f32 epilogue with infr-cpu's separate multiplies and adds (y bit-identical); STAGES (implies
// EXACT) also stores sd / sm per block.
template <int kT, bool STAGES, bool EXACT>
__global__ __launch_bounds__(kNW * 64) void mmq_strip_q4k_kernel(
    const uint8_t* __restrict__ w, size_t bpr, const int8_t* __restrict__ qs, const float* __restrict__ d8,
    const _Float16* __restrict__ bsh, float* __restrict__ y, int m, int out_f, int nb, int nx, int ny,
    int32_t* __restrict__ st_sd, int32_t* __restrict__ st_sm, const StripSeg* __restrict__ segs) {
    static_assert(!STAGES || EXACT, "the integer-stage form is the exact form");
    static_assert(kT >= 1 && kT <= 3, "one to three row tiles");
    typedef StripLds<kT> L;
    constexpr int kStripRows = 32 * kT;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: branches on it are scalar
    const int col = lane & 31, h = lane >> 5;
    // Workgroups go to the eight XCDs round-robin by linear id, and each XCD has its own L2: the
    // workgroups of one strip (same rows, different tokens) get ids that are equal modulo 8 and
    // adjacent within their XCD, so the strip's weights are fetched from HBM once.
    const int xcd = blockIdx.x & 7, chunk = blockIdx.x >> 3;
    const int strip = xcd + 8 * (chunk / ny), ty = chunk % ny;
    if (strip >= nx) return;  // uniform over the workgroup, before any barrier
    int row0 = strip * kStripRows, ldy = out_f;
    const int tok0 = ty * kStripTokens + wave * 32;
    // A grouped launch (several Linears over one activation tensor, plans): the strip is an entry
    // of a table - some rows of one of the ops - and `out_f` below is that entry's.
    if (segs != nullptr) {
        const StripSeg sg = segs[strip];
        w = sg.w;
        y = sg.y;
        out_f = sg.rows;
        row0 = 0;
        ldy = sg.ldy;
    }

    // ---- the unpack pieces of this wave: (row tile, nibble pair) of a block, 4 * kT in all. Waves w
    // and w + 4 share a SIMD. Three tiles: the lower four take (tiles 0 and 1, pair w) and unpack before
    // they multiply, the upper four take (tile 2, pair w - 4) and unpack after, so each SIMD carries
    // three pieces and its two waves are out of phase. Two tiles: one piece each, (tile w / 4, pair
    // w % 4). One tile: the lower four waves one piece each, the upper four none. ----
    constexpr int NU = kT == 3 ? 2 : 1;
    const bool two = wave < 4;                  // the waves that unpack before they multiply
    const int ut[2] = {two ? 0 : kT - 1, 1};
    const int up[2] = {wave & 3, wave & 3};
    // (one tile: waves w and w + 4 share pair w's piece, one sub-block of it each - both read the
    // piece's raw bytes - so that all eight waves carry the same unpack work)
    const int e_first = kT == 1 ? wave >> 2 : 0, e_last = kT == 1 ? wave >> 2 : 1;
    const uint8_t* urow[NU];
#pragma unroll
    for (int u = 0; u < NU; ++u) {
        const int r = row0 + 32 * ut[u] + col;
        urow[u] = w + (size_t)(r < out_f ? r : 0) * bpr + 16 + up[u] * 32 + h * 16;
    }
    v4i hdr[NU], qv[NU];  // raw bytes of the block to unpack next
    auto request_rows = [&](int b) {
#pragma unroll
        for (int u = 0; u < NU; ++u) {
            if (u == 0 || two) {
                const uint8_t* q = urow[u] + (size_t)b * 144;
                hdr[u] = load16(q - 16 - up[u] * 32 - h * 16);
                qv[u] = load16(q);
            }
        }
    };
    auto unpack_to = [&](uint8_t* buf) {
#pragma unroll
        for (int u = 0; u < NU; ++u) {
            if (u == 0 || two) {
                const int t = ut[u], p = up[u];
                uint32_t sc8[2], mn8[2];
                k4_all((uint32_t)hdr[u].y, (uint32_t)hdr[u].z, (uint32_t)hdr[u].w, sc8, mn8);
                const uint32_t scw = (p & 2) ? sc8[1] : sc8[0], mnw = (p & 2) ? mn8[1] : mn8[0];
                const int sh = (p & 1) * 16;
                const int qw[4] = {qv[u].x, qv[u].y, qv[u].z, qv[u].w};
#pragma unroll
                for (int e = 0; e < 2; ++e) {  // e = 0: sub-block 2p (low nibbles), 1: 2p+1 (high)
                    if (e < e_first || e > e_last) continue;
                    const uint32_t sc = (scw >> (sh + 8 * e)) & 0xFFu;
                    const uint32_t lo3 = sc & 7u, hi3 = sc >> 3;
                    v4i blo, bhi;
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const uint32_t codes = ((uint32_t)qw[k] >> (4 * e)) & 0x0F0F0F0Fu;
                        blo[k] = scale_codes4(codes, lo3);
                        bhi[k] = scale_codes4(codes, hi3);
                    }
                    uint8_t* dst = buf + (size_t)(((2 * p + e) * 2) * kT + t) * L::frag + lane * 16;
                    *reinterpret_cast<v4i*>(dst) = blo;
                    *reinterpret_cast<v4i*>(dst + kT * L::frag) = bhi;
                }
                if (h == 0 && e_first == 0) {
                    // the two mins of this pair as f16, k-slots 2p and 2p+1 of the row's eight
                    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
                    const h2 mn = {(_Float16)(int)((mnw >> sh) & 0xFFu), (_Float16)(int)((mnw >> (sh + 8)) & 0xFFu)};
                    *reinterpret_cast<h2*>(buf + L::mn_off + (t * 32 + col) * 16 + p * 4) = mn;
                    if (p == 0) {
                        float* dd = reinterpret_cast<float*>(buf + L::dd_off) + (t * 32 + col) * 2;
                        dd[0] = f16_bits_to_f32((uint32_t)hdr[u].x & 0xFFFFu);
                        dd[1] = f16_bits_to_f32((uint32_t)hdr[u].x >> 16);
                    }
                }
            }
        }
    };

    // ---- this wave's 32 tokens; a wave wholly past m recomputes the last group (nothing is stored) ----
    const size_t g = min((size_t)ty * kNW + wave, (size_t)(m - 1) / 32);
    auto request_acts = [&](ActFrags& f, int b) {
        const size_t gb = g * nb + b;
        const int8_t* ap = qs + gb * (8 * 1024) + lane * 16;
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) f.a[sb] = gload<v4i>(ap + sb * 1024);
        f.bs = gload<v8h>(bsh + (gb * 64 + lane) * 8);
        f.d = gload<float>(d8 + gb * 32 + col);
    };

    v16f acc[kT];
#pragma unroll
    for (int t = 0; t < kT; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[t][i] = 0.0f;
    bool row_ok[kT];
#pragma unroll
    for (int t = 0; t < kT; ++t) row_ok[t] = row0 + 32 * t + col < out_f;

    float* dql = reinterpret_cast<float*>(lds + L::dq_off) + wave * 32;  // + (block & 1) * kNW * 32

    // What a finished row tile leaves for its f32 epilogue: the two digit planes' integer sums, the
    // min term, the rows' (d, dmin) and - in `dq` - the activation scales of the lane's 16 tokens
    // (token 8*(i/4) + 4*h + i%4 for accumulator i).
    v16i hi_prev, lo_prev;
    v16f sm_prev;
    float d_prev = 0.0f, dmin_prev = 0.0f, dq[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) hi_prev[i] = 0, lo_prev[i] = 0, sm_prev[i] = 0.0f, dq[i] = 0.0f;
    // sumf += q8.d[b] * (d * sd as f32 - dmin * sm as f32), sd = lo + 8 * hi, for accumulator r of
    // row tile t in block b
    auto epilogue_one = [&](int t, int r, int b) {
        const int sd = lo_prev[r] + (hi_prev[r] << 3);
        if (STAGES) {
            const int tok = tok0 + 8 * (r >> 2) + 4 * h + (r & 3), wrow = row0 + 32 * t + col;
            if (b >= 0 && row_ok[t] && tok < m) {
                st_sd[((size_t)tok * out_f + wrow) * nb + b] = sd;
                st_sm[((size_t)tok * out_f + wrow) * nb + b] = (int)sm_prev[r];
            }
        }
        if (EXACT) acc[t][r] += dq[r] * (d_prev * (float)sd - dmin_prev * sm_prev[r]);
        else acc[t][r] = __builtin_fmaf(dq[r], __builtin_fmaf(d_prev, (float)sd, -(dmin_prev * sm_prev[r])), acc[t][r]);
    };

    // One block. Between two barriers a wave unpacks the next block's weights into the other
    // buffer (the lower four waves before they multiply, the upper four after, so that the two
    // waves of a SIMD are out of phase) and multiplies this block.
    //
    // The 48 int8 MFMAs of a block form one sequence of slots: slot 16 t + k is row tile t,
    // sub-block k / 2, high digits for even k and low digits for odd k - two independent chains,
    // so an MFMA never waits for the one before it. B fragments are read from LDS three slots
    // ahead. The f32 epilogue of the row tile before (the last tile of the previous block for
    // t = 0) is cut into its 16 accumulators, one behind each MFMA, so that the matrix core and the
    // vector ALU work at the same time inside one wave; each activation fragment is requested
    // again, for the next block, right after its last use.
    //
    // One and two row tiles: a block is too short to cover those requests (an L2 round trip against
    // half a block's MFMAs), so the fragments are double-buffered instead - `fn` receives the next
    // block's at the start of this one - which the three-tile form has no registers for.
    constexpr bool kTwoSets = kT <= 2;
    auto multiply = [&](int b, ActFrags& f, ActFrags& fn) {
        const uint8_t* buf = lds + (b & 1) * L::bytes;
        const size_t gb_next = g * nb + min(b + 1, nb - 1);
        const int8_t* ap_next = qs + gb_next * (8 * 1024) + lane * 16;
        float* dql_b = dql + (b & 1) * (kNW * 32);
        dql_b[col] = f.d;  // both halves of the wave hold the token's scale: same value, same address
        const v8h bs_cur = f.bs;
        // the next block's scales and sums: a whole block ahead
        fn.bs = gload<v8h>(bsh + (gb_next * 64 + lane) * 8);
        fn.d = gload<float>(d8 + gb_next * 32 + col);
        if constexpr (kTwoSets) {
#pragma unroll
            for (int sb = 0; sb < 8; ++sb) fn.a[sb] = gload<v4i>(ap_next + sb * 1024);
        }
        const v16i zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        const v16f zf = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        const uint32_t bl = (uint32_t)(uintptr_t)(buf + lane * 16);  // LDS address of the lane's piece of fragment 0
                constexpr int kAhead = 3, kSlots = 16 * kT;
        v4i ring[kAhead + 1];
        auto read_slot = [&](auto slot_c) {
            constexpr int slot = decltype(slot_c)::value;
            constexpr int t = slot >> 4, k = slot & 15, sb = k >> 1, plane = (k & 1) ? 0 : 1;
            ring[slot % (kAhead + 1)] = lds_read16_ahead<((sb * 2 + plane) * kT + t) * L::frag>(bl);
        };
        static_for<kAhead>([&](auto s) { read_slot(s); });
        v16i hi = zi, lo = zi;
        static_for<kSlots>([&](auto slot_c) {
            constexpr int slot = decltype(slot_c)::value;
            constexpr int t = slot >> 4, k = slot & 15, sb = k >> 1;
            // reads younger than this slot's when its MFMA comes up
            constexpr int kYoung = kSlots - 1 - slot < kAhead ? kSlots - 1 - slot : kAhead;
            if constexpr (slot + kAhead < kSlots) read_slot(std::integral_constant<int, slot + kAhead>{});
            lds_wait<kYoung>(ring[slot % (kAhead + 1)]);
            const v4i bop = ring[slot % (kAhead + 1)];
            if constexpr ((k & 1) == 0)
                hi = __builtin_amdgcn_mfma_i32_32x32x32_i8(f.a[sb], bop, k == 0 ? zi : hi, 0, 0, 0);
            else
                lo = __builtin_amdgcn_mfma_i32_32x32x32_i8(f.a[sb], bop, k == 1 ? zi : lo, 0, 0, 0);
            // the last use of this activation fragment in the block: ask for the next block's
            if constexpr (!kTwoSets && t == kT - 1 && (k & 1)) {
                fn.a[sb] = gload<v4i>(ap_next + sb * 1024);  // (fn is f itself in this form)
            }
            epilogue_one(t == 0 ? kT - 1 : t - 1, k, t == 0 ? b - 1 : b);
            if constexpr (k == 15) {
                if constexpr (t == 0) {
                    // the previous block's last tile is done: from here on the scales are this block's
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const v4f q4 = *reinterpret_cast<const v4f*>(dql_b + 8 * j + 4 * h);
                        dq[4 * j] = q4.x, dq[4 * j + 1] = q4.y, dq[4 * j + 2] = q4.z, dq[4 * j + 3] = q4.w;
                    }
                }
                const v8h bm = *reinterpret_cast<const v8h*>(buf + L::mn_off + (t * 32 + col) * 16);
                const float* dd = reinterpret_cast<const float*>(buf + L::dd_off) + (t * 32 + col) * 2;
                sm_prev = __builtin_amdgcn_mfma_f32_32x32x16_f16(bs_cur, bm, zf, 0, 0, 0);
                hi_prev = hi;
                lo_prev = lo;
                d_prev = dd[0];
                dmin_prev = dd[1];
            }
        });
        // The sums are next read a block later; without a use here the compiler sinks the whole
        // epilogue to that place, behind the barrier, and nothing is left to overlap the MFMAs with.
#pragma unroll
        for (int t = 0; t < kT; ++t) asm volatile("" : "+v"(acc[t]));
        if (!STAGES) {
            // issue order of the block: per slot the MFMA and the vector instructions of one
            // accumulator's epilogue (seven, five in the contracted form)
            constexpr int kMfma = 0x008, kValu = 0x002, kVmemRead = 0x020;
            constexpr int kEpi = EXACT ? 7 : 5;
#pragma unroll
            for (int t = 0; t < kT; ++t) {
#pragma unroll
                for (int k = 0; k < 16; ++k) {
                    __builtin_amdgcn_sched_group_barrier(kMfma, 1, 0);
                    if (!kTwoSets && t == kT - 1 && (k & 1)) __builtin_amdgcn_sched_group_barrier(kVmemRead, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(kValu, kEpi, 0);
                }
                __builtin_amdgcn_sched_group_barrier(kMfma, 1, 0);
            }
        }
    };

    // Requests past the last block are clamped to it (redundant loads, never consumed), so the
    // loop body is straight-line code.
    ActFrags f0, f1;
    request_rows(0);
    request_acts(f0, 0);
    unpack_to(lds);
    request_rows(min(1, nb - 1));
    __syncthreads();
    auto block = [&](int b, ActFrags& f, ActFrags& fn) {
        uint8_t* other = lds + ((b + 1) & 1) * L::bytes;
        if (two) {
            unpack_to(other);
            request_rows(min(b + 2, nb - 1));
        }
        multiply(b, f, fn);
        if (!two) {
            unpack_to(other);
            request_rows(min(b + 2, nb - 1));
        }
        __syncthreads();
    };
    if constexpr (kTwoSets) {
        int b = 0;
        for (; b + 2 <= nb; b += 2) {
            block(b, f0, f1);
            block(b + 1, f1, f0);
        }
        if (b < nb) block(b, f0, f1);
    } else {
        for (int b = 0; b < nb; ++b) block(b, f0, f0);
    }
    // the last block's last row tile
#pragma unroll
    for (int r = 0; r < 16; ++r) epilogue_one(kT - 1, r, nb - 1);

#pragma unroll
    for (int t = 0; t < kT; ++t) {
        if (!row_ok[t]) continue;
        const int wrow = row0 + 32 * t + col;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int tok = tok0 + 8 * (r >> 2) + 4 * h + (r & 3);
            if (tok < m) gstore<float>(y + (size_t)tok * ldy + wrow, acc[t][r]);
        }
    }
}

}  // namespace

// Strip height for `m` tokens x `out_f` rows of `in_f` columns on `cus` compute units: the number of
// 32-row tiles (1..3) whose grid takes the least time, a taller strip winning ties. A workgroup
// walks its whole row; a round of one workgroup per compute unit costs, per 256-block, ~1.6 / 2.3 /
// 3.6 us at one / two / three tiles (measured at 4096 and 12288 columns, 256 to 2048 tokens: two tiles
// have double-buffered activation fragments and an even unpack, three have neither for want of
// registers, one spends most of a block on what does not depend on the height), and the grid runs in
// whole rounds: 512 tokens x 12288 rows are one round at three tiles (58 us) against two at two (74);
// 512 x 4096 one round at one tile (26) against one at two on half the units (37).
int mmq_strip_q4k_tiles(size_t m, size_t out_f, size_t in_f, int cus) {
    if (cus <= 0) cus = 256;
    static const double per_block_us[4] = {0.0, 1.6, 2.3, 3.6};
    const size_t ny = (m + kStripTokens - 1) / kStripTokens, nb = in_f / 256;
    int best = 1;
    double best_cost = 0.0;
    for (int kt = 3; kt >= 1; --kt) {
        const size_t rows = 32 * (size_t)kt;
        const size_t wgs = ((out_f + rows - 1) / rows) * ny;
        const size_t rounds = (wgs + cus - 1) / cus;
        const double cost = (double)rounds * (double)nb * per_block_us[kt];
        if (kt == 3 || cost < best_cost) best = kt, best_cost = cost;
    }
    return best;
}

template <int KT>
static void launch_strip(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m, size_t in_f,
                         size_t out_f, const IntStages& st, bool exact, hipStream_t stream,
                         const StripSeg* segs = nullptr, int n_segs = 0) {
    const int nx = segs ? n_segs : (int)((out_f + 32 * KT - 1) / (32 * KT)), ny = (int)((m + kStripTokens - 1) / kStripTokens);
    const dim3 grid((unsigned)(8 * ((nx + 7) / 8) * ny)), block(kNW * 64);
    const int nb = (int)(in_f / 256);
    const auto* bsh = reinterpret_cast<const _Float16*>(act.bsums);
    constexpr int lds = StripLds<KT>::total;
#define INFR_STRIP(STAGES, EXACT, A, B)                                                                              \
    do {                                                                                                             \
        if (lds > 64 * 1024)                                                                                         \
            (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&mmq_strip_q4k_kernel<KT, STAGES, EXACT>),      \
                                      hipFuncAttributeMaxDynamicSharedMemorySize, lds);                              \
        hipLaunchKernelGGL((mmq_strip_q4k_kernel<KT, STAGES, EXACT>), grid, block, lds, stream, w, bpr, act.qs, act.d, \
                           bsh, y, (int)m, (int)out_f, nb, nx, ny, A, B, segs);                                      \
    } while (0)
    if (st.a) INFR_STRIP(true, true, st.a, st.b);
    else if (exact) INFR_STRIP(false, true, (int32_t*)nullptr, (int32_t*)nullptr);
    else INFR_STRIP(false, false, (int32_t*)nullptr, (int32_t*)nullptr);
#undef INFR_STRIP
}

void launch_mmq_strip_q4k(const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m, size_t in_f,
                          size_t out_f, const IntStages& st, int tiles, bool exact, hipStream_t stream) {
    if (tiles == 3) launch_strip<3>(w, bpr, act, y, m, in_f, out_f, st, exact, stream);
    else if (tiles == 2) launch_strip<2>(w, bpr, act, y, m, in_f, out_f, st, exact, stream);
    else launch_strip<1>(w, bpr, act, y, m, in_f, out_f, st, exact, stream);
}

int mmq_strip_q4k_rows(int tiles) { return 32 * tiles; }

void launch_mmq_strip_q4k_group(size_t bpr, const ActQ8& act, size_t m, size_t in_f, int tiles, const StripSeg* segs_dev,
                                int n_segs, hipStream_t stream) {
    if (n_segs <= 0) return;
    const IntStages none{};
    if (tiles == 3) launch_strip<3>(nullptr, bpr, act, nullptr, m, in_f, 0, none, false, stream, segs_dev, n_segs);
    else if (tiles == 2) launch_strip<2>(nullptr, bpr, act, nullptr, m, in_f, 0, none, false, stream, segs_dev, n_segs);
    else launch_strip<1>(nullptr, bpr, act, nullptr, m, in_f, 0, none, false, stream, segs_dev, n_segs);
}

}  // namespace infr
