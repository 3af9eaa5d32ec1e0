// m >= 2: GEMM of block-quantized weights against on-device int8-quantized activations.
#include "device_common.hpp"
#include "kernels.hpp"

namespace infr {

// Row-at-a-time form: every activation row goes through the decode GEMV, so each output element
// is produced by exactly the code path of m == 1 (the CPU's batch kernels are likewise
// bit-identical to its single-row kernels, crates/infr-cpu/src/kernels.rs:9297-9405). Weights are
// re-streamed once per row, which is only acceptable for very small m.
static bool mmq_by_rows(int dtype, const uint8_t* w, size_t bpr, const ActQ8& act, float* y,
                        size_t m, size_t in_f, size_t out_f, const IntStages& st,
                        hipStream_t stream) {
    const bool per32 = dtype == 42;
    const size_t dper = per32 ? in_f / 32 : in_f / 256;
    const size_t blocks = (dtype == 12 || dtype == 14) ? in_f / 256 : in_f / 32;
    for (size_t r = 0; r < m; ++r) {
        ActQ8 a;
        a.qs = act.qs + r * in_f;
        a.d = act.d + r * dper;
        a.bsums = act.bsums + r * (in_f / 32);
        a.bsums16 = act.bsums16 ? act.bsums16 + r * (in_f / 16) : nullptr;
        IntStages s;
        if (st.a) s.a = st.a + r * out_f * blocks;
        if (st.b) s.b = st.b + r * out_f * blocks;
        if (!launch_gemv(dtype, w, bpr, a, y + r * out_f, in_f, out_f, s, stream)) return false;
    }
    return true;
}

bool launch_mmq(int dtype, const uint8_t* w, size_t bpr, const ActQ8& act, float* y, size_t m,
                size_t in_f, size_t out_f, const IntStages& st, hipStream_t stream) {
    return mmq_by_rows(dtype, w, bpr, act, y, m, in_f, out_f, st, stream);
}

}  // namespace infr
