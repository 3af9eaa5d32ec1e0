// Instantiates the decode GEMV templates for: FmtQ4_0, FmtQ4_1, FmtIQ4NL.
#include "gemv_impl.hpp"

namespace infr {

const GemvFormatOps& gemv_ops_q4_0() {
    static const GemvFormatOps ops = make_gemv_format_ops<FmtQ4_0>();
    return ops;
}
const GemvFormatOps& gemv_ops_q4_1() {
    static const GemvFormatOps ops = make_gemv_format_ops<FmtQ4_1>();
    return ops;
}
const GemvFormatOps& gemv_ops_iq4nl() {
    static const GemvFormatOps ops = make_gemv_format_ops<FmtIQ4NL>();
    return ops;
}

}  // namespace infr
