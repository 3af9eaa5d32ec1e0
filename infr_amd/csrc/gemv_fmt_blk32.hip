// Instantiates the decode GEMV templates for: FmtQ8_0A, FmtQ8_0_32, FmtQ8_0_32A, FmtQ2_0, FmtQ2_0A.
#include "gemv_impl.hpp"

namespace infr {

const GemvFormatOps& gemv_ops_q8_0() {
    static const GemvFormatOps ops = make_gemv_format_ops<FmtQ8_0A>();
    return ops;
}
const GemvFormatOps& gemv_ops_q8_0_32() {
    static const GemvFormatOps ops = make_gemv_format_ops<FmtQ8_0_32>();
    return ops;
}
const GemvFormatOps& gemv_ops_q2_0() {
    static const GemvFormatOps ops = make_gemv_format_ops<FmtQ2_0>();
    return ops;
}
const GemvFormatOps& gemv_ops_q8_0_32_aligned() {
    static const GemvFormatOps ops = make_gemv_format_ops<FmtQ8_0_32A>();
    return ops;
}
const GemvFormatOps& gemv_ops_q2_0_aligned() {
    static const GemvFormatOps ops = make_gemv_format_ops<FmtQ2_0A>();
    return ops;
}

}  // namespace infr
