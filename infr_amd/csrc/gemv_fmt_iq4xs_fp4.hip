// Instantiates the decode GEMV templates for: FmtIQ4XS, FmtMXFP4, FmtNVFP4.
#include "gemv_impl.hpp"

namespace infr {

const GemvFormatOps& gemv_ops_iq4xs() {
    static const GemvFormatOps ops = make_gemv_format_ops<FmtIQ4XS>();
    return ops;
}
const GemvFormatOps& gemv_ops_mxfp4() {
    static const GemvFormatOps ops = make_gemv_format_ops<FmtMXFP4>();
    return ops;
}
const GemvFormatOps& gemv_ops_nvfp4() {
    static const GemvFormatOps ops = make_gemv_format_ops<FmtNVFP4>();
    return ops;
}

}  // namespace infr
