// Instantiates the decode GEMV templates for: FmtQ5K.
#include "gemv_impl.hpp"

namespace infr {

const GemvFormatOps& gemv_ops_q5k() {
    static const GemvFormatOps ops = make_gemv_format_ops<FmtQ5K>();
    return ops;
}

}  // namespace infr
