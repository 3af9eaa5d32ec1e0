// Instantiates the decode GEMV templates for the pair forms: FmtQ4_0Pair, FmtIQ4NLPair, and the
// batch (m >= 2) ones for FmtQ5_0Pair.
#include "gemv_impl.hpp"

namespace infr {

const GemvFormatOps& gemv_ops_q4_0_pair() {
    static const GemvFormatOps ops = make_gemv_format_ops<FmtQ4_0Pair>();
    return ops;
}
const GemvFormatOps& gemv_ops_iq4nl_pair() {
    static const GemvFormatOps ops = make_gemv_format_ops<FmtIQ4NLPair>();
    return ops;
}
const GemvFormatOps& gemv_ops_q5_0_pair() {
    static const GemvFormatOps ops = make_gemv_format_ops<FmtQ5_0Pair, false>();
    return ops;
}

}  // namespace infr
