// Instantiates the decode GEMV templates for: FmtQ4K, FmtQ6K.
#include "gemv_impl.hpp"

namespace infr {

const GemvFormatOps& gemv_ops_q4k() {
    static const GemvFormatOps ops = make_gemv_format_ops<FmtQ4K>();
    return ops;
}
const GemvFormatOps& gemv_ops_q6k() {
    static const GemvFormatOps ops = make_gemv_format_ops<FmtQ6K>();
    return ops;
}

}  // namespace infr
