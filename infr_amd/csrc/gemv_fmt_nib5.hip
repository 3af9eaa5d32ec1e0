// Instantiates the decode GEMV templates for: FmtQ5_1, and the batch (m >= 2) ones for FmtQ5_0
// (a single token of Q5_0 multiplies f32 activations instead, as the CPU backend does).
#include "gemv_impl.hpp"

namespace infr {

const GemvFormatOps& gemv_ops_q5_1() {
    static const GemvFormatOps ops = make_gemv_format_ops<FmtQ5_1>();
    return ops;
}
const GemvFormatOps& gemv_ops_q5_0() {
    static const GemvFormatOps ops = make_gemv_format_ops<FmtQ5_0, false>();
    return ops;
}

}  // namespace infr
