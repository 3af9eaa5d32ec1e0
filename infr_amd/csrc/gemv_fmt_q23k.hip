// Instantiates the decode GEMV templates for: FmtQ2K, FmtQ3K, FmtTQ1_0, FmtTQ2_0, FmtIQ4XS, FmtMXFP4, FmtNVFP4.
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
const GemvFormatOps& gemv_ops_iq4xs() {
    static const GemvFormatOps ops = make_gemv_format_ops<FmtIQ4XS>();
    return ops;
}
const GemvFormatOps& gemv_ops_tq1_0() {
    static const GemvFormatOps ops = make_gemv_format_ops<FmtTQ1_0>();
    return ops;
}
const GemvFormatOps& gemv_ops_tq2_0() {
    static const GemvFormatOps ops = make_gemv_format_ops<FmtTQ2_0>();
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
