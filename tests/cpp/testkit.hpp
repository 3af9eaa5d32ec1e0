// Shared harness of the C++ seam tests: the bind-run-download sequence and the Linear parity-case
// vocabulary of the reference's infr-testkit (crates/infr-testkit/src/lib.rs:170-201 `run_graph`,
// :205-303 `LinearCase` / `CaseReport` / `case_inputs`, :330-420 `check_linear`,
// `weight_quant_cases`, `SweepReport`), over infr::HipBackend. Expected values come from the CPU
// oracle (oracle/infr_cpu_oracle.h): its restatement of the host decode + f64 GEMM the reference
// scores against, and of infr-cpu's production kernels. Test infrastructure only.
#pragma once

#include <cmath>
#include <cstdio>
#include <string>
#include <utility>
#include <vector>

#include "../../include/infr_hip.hpp"
#include "../../oracle/infr_cpu_oracle.h"

namespace testkit {

using namespace infr;

inline std::vector<uint8_t> f32_bytes(const std::vector<float>& v) {
    std::vector<uint8_t> b(v.size() * 4);
    std::memcpy(b.data(), v.data(), b.size());
    return b;
}

// testkit:60-64
inline std::vector<float> gen_f32(size_t n, size_t salt) {
    std::vector<float> v(n);
    orc_gen_f32(n, salt, v.data());
    return v;
}

// testkit:106-123: valid blocks of `dtype` from an LCG byte stream, scale slots overwritten
inline std::vector<uint8_t> synth_weight(DType dtype, size_t n_elem, uint32_t seed) {
    const auto [e, b] = block_layout(dtype);
    std::vector<uint8_t> w(n_elem / e * b);
    if (orc_synth_weight((int)dtype, n_elem, seed, w.data()) != w.size())
        throw std::runtime_error(std::string("synth_weight: ") + dtype_name(dtype));
    return w;
}

// testkit:133-137: the host decode oracle
inline std::vector<float> dequant_oracle(DType dtype, const std::vector<uint8_t>& bytes) {
    const auto [e, b] = block_layout(dtype);
    std::vector<float> out(bytes.size() / b * e);
    if (orc_dequant_block((int)dtype, bytes.data(), bytes.size(), out.data()) != 0)
        throw std::runtime_error(std::string("host dequant oracle failed for ") + dtype_name(dtype));
    return out;
}

// testkit:142-163: f64-accumulated reference GEMM
inline std::vector<float> ref_linear(const std::vector<float>& x, const std::vector<float>& w, size_t m,
                                     size_t in_f, size_t out_f) {
    std::vector<float> out(m * out_f);
    orc_ref_linear_f64(x.data(), w.data(), m, in_f, out_f, out.data());
    return out;
}

// testkit:170-201: bind raw bytes to graph handles, run `g` once, download `out` as f32.
inline std::vector<float> run_graph(HipBackend& be, const Graph& g,
                                    const std::vector<std::pair<TensorId, std::vector<uint8_t>>>& bound,
                                    TensorId out, size_t out_n) {
    Plan plan = be.compile(g);
    std::vector<std::pair<TensorId, Buffer>> bufs;
    Bindings binds;
    for (const auto& [id, bytes] : bound) {
        const BufferUsage usage = g.kind(id) == TensorKind::Weight ? BufferUsage::Weights : BufferUsage::Activations;
        Buffer b = be.alloc(bytes.size() < 4 ? 4 : bytes.size(), usage);
        be.upload(b, bytes.data(), bytes.size());
        bufs.emplace_back(id, std::move(b));
    }
    Buffer ob = be.alloc(out_n * 4, BufferUsage::Readback);
    for (const auto& [id, b] : bufs) binds.bind(id, b);
    binds.bind(out, ob);
    be.execute(plan, binds);
    std::vector<float> o(out_n);
    be.download(ob, o);
    return o;
}

struct LinearCase {
    DType dtype;
    size_t m, in_f, out_f;
    uint32_t seed = 0x5eed;
    LinearCase with_seed(uint32_t s) const { LinearCase c = *this; c.seed = s; return c; }
};

struct CaseReport {
    DType dtype;
    size_t m, in_f, out_f;
    float abs, rel, ref_mag, tol;
    // A case passes when it is non-vacuous and inside tolerance.
    bool ok() const { return ref_mag > 1e-3f && rel < tol; }
    std::string line() const {
        char buf[256];
        std::snprintf(buf, sizeof buf, "%8s m=%-3zu %zux%zu rel=%.3e abs=%.3e max|ref|=%.3e tol=%.1e%s%s",
                      dtype_name(dtype), m, in_f, out_f, rel, abs, ref_mag, tol, rel < tol ? "" : "  << OVER",
                      ref_mag > 1e-3f ? "" : "  << VACUOUS (oracle is all-zero)");
        return buf;
    }
};

inline std::pair<std::vector<uint8_t>, std::vector<float>> case_inputs(const LinearCase& c) {
    return {synth_weight(c.dtype, c.out_f * c.in_f, c.seed), gen_f32(c.m * c.in_f, (size_t)c.seed ^ 0x9e37)};
}

inline std::vector<float> run_linear(HipBackend& be, const LinearCase& c) {
    auto [w_bytes, x] = case_inputs(c);
    Graph g;
    const TensorId xid = g.input({{c.m, c.in_f}, DType::F32});
    const TensorId wid = g.weight({{c.out_f, c.in_f}, c.dtype});
    const TensorId dst = g.output({{c.m, c.out_f}, DType::F32});
    g.push(op::Linear{xid, wid, dst, (uint32_t)c.m, (uint32_t)c.in_f, (uint32_t)c.out_f, 0});
    return run_graph(be, g, {{xid, f32_bytes(x)}, {wid, w_bytes}}, dst, c.m * c.out_f);
}

inline CaseReport score(const LinearCase& c, const std::vector<float>& got, const std::vector<float>& want, float tol) {
    float abs = 0.0f, mag = 0.0f;
    for (size_t i = 0; i < want.size(); ++i) {
        const float d = std::fabs(want[i] - got[i]);
        abs = (d > abs || d != d) ? d : abs;
        mag = std::fmax(mag, std::fabs(want[i]));
    }
    return {c.dtype, c.m, c.in_f, c.out_f, abs, abs / std::fmax(mag, 1e-3f), mag, tol};
}

// Against the host decode of the same bytes and the f64 GEMM (what the reference's sweeps score).
inline CaseReport check_linear(HipBackend& be, const LinearCase& c, float tol) {
    auto [w_bytes, x] = case_inputs(c);
    const std::vector<float> want = ref_linear(x, dequant_oracle(c.dtype, w_bytes), c.m, c.in_f, c.out_f);
    return score(c, run_linear(be, c), want, tol);
}

// infr-cpu's production arm on the same bytes (crates/infr-cpu/src/lib.rs:985-1492).
inline std::vector<float> cpu_linear(const LinearCase& c, bool reference_mode = false) {
    auto [w_bytes, x] = case_inputs(c);
    std::vector<float> y(c.m * c.out_f);
    if (orc_linear((int)c.dtype, w_bytes.data(), w_bytes.size(), c.out_f * c.in_f, 0, x.data(), y.data(), c.m,
                   c.in_f, c.out_f, reference_mode, 0) != 0)
        throw std::runtime_error(std::string("oracle refuses ") + dtype_name(c.dtype));
    return y;
}

// decode_spec.rs:255-280: the reference's roster, in its order (the index seeds each case); the
// formats this backend takes are marked.
struct RosterEntry { const char* name; int dtype; };
inline const std::vector<RosterEntry>& weight_quants() {
    static const std::vector<RosterEntry> r = {
        {"Q4_0", 2}, {"Q4_1", 3}, {"Q5_0", 6}, {"Q5_1", 7}, {"Q8_0", 8}, {"Q2K", 10}, {"Q3K", 11}, {"Q4K", 12},
        {"Q5K", 13}, {"Q6K", 14}, {"Iq1S", -1}, {"Iq1M", -1}, {"Iq2Xxs", -1}, {"Iq2Xs", -1}, {"Iq2S", -1},
        {"Iq3Xxs", -1}, {"Iq3S", -1}, {"Iq4Nl", 20}, {"Iq4Xs", 23}, {"Tq1_0", 34}, {"Tq2_0", 35}, {"Q2_0", 42},
        {"Mxfp4", 39}, {"Nvfp4", 40}};
    return r;
}

// testkit:392-403, restricted to the formats of this backend; seeds 0x201 + roster index.
inline std::vector<LinearCase> weight_quant_cases(size_t m, size_t in_f, size_t out_f) {
    std::vector<LinearCase> v;
    const auto& r = weight_quants();
    for (size_t i = 0; i < r.size(); ++i)
        if (r[i].dtype >= 0) v.push_back(LinearCase{(DType)r[i].dtype, m, in_f, out_f}.with_seed(0x201 + (uint32_t)i));
    return v;
}

struct SweepReport {
    std::string label;
    std::vector<CaseReport> cases;
    // Print every case, then report how many are outside tolerance.
    int failures() const {
        int bad = 0;
        for (const auto& c : cases) {
            std::printf("[%s] %s\n", label.c_str(), c.line().c_str());
            bad += !c.ok();
        }
        return bad;
    }
};

template <typename TolFn>
SweepReport sweep_linear_on(const std::string& label, HipBackend& be, const std::vector<LinearCase>& cases, TolFn tol) {
    SweepReport r{label, {}};
    for (const auto& c : cases) r.cases.push_back(check_linear(be, c, tol(c)));
    return r;
}

}  // namespace testkit
