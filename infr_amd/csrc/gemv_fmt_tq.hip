// Instantiates the decode GEMV templates for: FmtTQ1_0, FmtTQ2_0.
#include "gemv_impl.hpp"

namespace infr {

const GemvFormatOps& gemv_ops_tq1_0() {
    static const GemvFormatOps ops = make_gemv_format_ops<FmtTQ1_0>();
    return ops;
}
const GemvFormatOps& gemv_ops_tq2_0() {
    static const GemvFormatOps ops = make_gemv_format_ops<FmtTQ2_0>();
    return ops;
}

}  // namespace infr
