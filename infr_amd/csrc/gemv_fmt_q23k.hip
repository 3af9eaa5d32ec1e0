// Instantiates the decode GEMV templates for: FmtQ2K, FmtQ3K.
#include "gemv_impl.hpp"

namespace infr {

const GemvFormatOps& gemv_ops_q2k() {
    static const GemvFormatOps ops = make_gemv_format_ops<FmtQ2K>();
    return ops;
}
const GemvFormatOps& gemv_ops_q3k() {
    static const GemvFormatOps ops = make_gemv_format_ops<FmtQ3K>();
    return ops;
}

}  // namespace infr
