// Seam tests in the reference's own shape (crates/infr-cpu/tests/op_parity.rs: the all-quant
// Linear sweeps against the host decode oracle; crates/infr-llama/tests/seam_op_parity.rs: MoeFfn
// against the CPU arm), driven through infr::HipBackend - alloc, upload, compile, bind, execute,
// download - and scored against the CPU oracle. Needs a gfx950 device. Exit status = failed tests.
//
//   op_parity            run every test
//   op_parity NAME...    run the named tests
#include <algorithm>
#include <cstdlib>
#include <functional>

#include "testkit.hpp"

using namespace testkit;

// infr-cpu's own bound for its int8-activation Linear against the f64 host oracle
// (crates/infr-cpu/tests/op_parity.rs:57).
static constexpr float CPU_INT8_ACT_TOL = 2e-2f;

static int g_checks_failed = 0;
#define EXPECT(cond, ...)                                   \
    do {                                                    \
        if (!(cond)) {                                      \
            ++g_checks_failed;                              \
            std::printf("  FAILED %s:%d: ", __FILE__, __LINE__); \
            std::printf(__VA_ARGS__);                       \
            std::printf("\n");                              \
        }                                                   \
    } while (0)

static float rel_l2(const std::vector<float>& got, const std::vector<float>& want) {
    double num = 0.0, den = 0.0;
    for (size_t i = 0; i < want.size(); ++i) {
        const double d = (double)got[i] - (double)want[i];
        num += d * d;
        den += (double)want[i] * (double)want[i];
    }
    return (float)std::sqrt(num / std::max(den, 1e-30));
}
static float max_abs(const std::vector<float>& v) {
    float m = 0.0f;
    for (float f : v) m = std::fmax(m, std::fabs(f));
    return m;
}
static bool same_bits(const std::vector<float>& a, const std::vector<float>& b) {
    return a.size() == b.size() && std::memcmp(a.data(), b.data(), a.size() * 4) == 0;
}
// the path's gate: rel-L2 <= 1e-4 and max-abs <= 1e-3 * max|want|
static void gate(const char* what, const std::vector<float>& got, const std::vector<float>& want) {
    float dmax = 0.0f;
    for (size_t i = 0; i < want.size(); ++i) {
        const float d = std::fabs(got[i] - want[i]);
        dmax = (d > dmax || d != d) ? d : dmax;
    }
    const float rel = rel_l2(got, want), mag = max_abs(want);
    EXPECT(mag > 1e-3f, "%s: oracle output is all-zero", what);
    EXPECT(rel <= 1e-4f && dmax <= 1e-3f * mag, "%s: rel-L2 %.3e max-abs %.3e (max|y| %.3e)", what, rel, dmax, mag);
}

// ── the reference's all-quant sweeps: in_f = 256 is a whole number of blocks of every format ──
static void hip_linear_all_weight_quants_match_the_host_oracle(HipBackend& be) {
    for (size_t m : {1, 2}) {
        const auto cases = weight_quant_cases(m, 256, 8);
        const SweepReport r = sweep_linear_on("hip Linear m=" + std::to_string(m), be, cases,
                                              [](const LinearCase&) { return CPU_INT8_ACT_TOL; });
        EXPECT(r.cases.size() == 17, "expected the seventeen formats of this backend, got %zu", r.cases.size());
        EXPECT(r.failures() == 0, "cases outside %.0e of the host decode oracle", CPU_INT8_ACT_TOL);
    }
}

// Same inputs against infr-cpu's production arm: the activations are quantized the same way on
// both sides, so what is left is f32 summation order (none at all for the ordered K-quants).
static void hip_linear_matches_the_cpu_production_arm(HipBackend& be) {
    const size_t shapes[][2] = {{256, 8}, {1024, 64}, {4096, 48}};
    for (size_t m : {1, 2, 8, 40})
        for (const auto& s : shapes)
            for (const LinearCase& c : weight_quant_cases(m, s[0], s[1])) {
                const std::vector<float> got = run_linear(be, c);
                // one token of Q5_0 multiplies f32 activations on the CPU (no int8 arm there)
                const std::vector<float> want = cpu_linear(c);
                char what[96];
                std::snprintf(what, sizeof what, "%s m=%zu %zux%zu", dtype_name(c.dtype), m, s[0], s[1]);
                gate(what, got, want);
                const bool ordered = c.dtype == DType::Q4K || c.dtype == DType::Q5K || c.dtype == DType::Q6K ||
                                     c.dtype == DType::Q2K || c.dtype == DType::Q3K || c.dtype == DType::IQ4XS ||
                                     c.dtype == DType::TQ2_0 || c.dtype == DType::TQ1_0;
                if (ordered && m <= 8) EXPECT(same_bits(got, want), "%s: not bit-identical to infr-cpu", what);
            }
}

// batch == single, bit for bit (crates/infr-cpu/src/kernels.rs:9297-9405 holds the CPU to the same)
static void hip_linear_batch_rows_equal_single_rows(HipBackend& be) {
    for (DType dt : {DType::Q4K, DType::Q5K, DType::Q6K, DType::Q2K, DType::Q3K, DType::IQ4XS}) {
        const LinearCase c{dt, 6, 1024, 40};
        auto [w, x] = case_inputs(c);
        const std::vector<float> batch = run_linear(be, c);
        for (size_t r = 0; r < c.m; ++r) {
            Graph g;
            const TensorId xid = g.input({{1, c.in_f}, DType::F32});
            const TensorId wid = g.weight({{c.out_f, c.in_f}, dt});
            const TensorId dst = g.output({{1, c.out_f}, DType::F32});
            g.push(op::Linear{xid, wid, dst, 1, (uint32_t)c.in_f, (uint32_t)c.out_f, 0});
            const std::vector<float> xr(x.begin() + r * c.in_f, x.begin() + (r + 1) * c.in_f);
            const std::vector<float> one = run_graph(be, g, {{xid, f32_bytes(xr)}, {wid, w}}, dst, c.out_f);
            EXPECT(std::memcmp(one.data(), batch.data() + r * c.out_f, c.out_f * 4) == 0,
                   "%s: row %zu of the batch differs from the single-row result", dtype_name(dt), r);
        }
    }
}

// w_off addresses rows of a concatenated weight (graph.rs:177-191; lib.rs:1005-1008)
static void hip_linear_w_off_slices_a_concatenated_weight(HipBackend& be) {
    const size_t in_f = 512, rows = 96;
    for (DType dt : {DType::Q4K, DType::Q8_0, DType::Q4_0}) {
        const std::vector<uint8_t> w = synth_weight(dt, rows * in_f, 0x77);
        const std::vector<float> x = gen_f32(in_f, 5);
        for (auto [row0, n] : {std::pair<size_t, size_t>{0, 96}, {32, 24}, {89, 7}}) {
            Graph g;
            const TensorId xid = g.input({{1, in_f}, DType::F32});
            const TensorId wid = g.weight({{rows, in_f}, dt});
            const TensorId dst = g.output({{1, n}, DType::F32});
            g.push(op::Linear{xid, wid, dst, 1, (uint32_t)in_f, (uint32_t)n, row0 * in_f});
            const std::vector<float> got = run_graph(be, g, {{xid, f32_bytes(x)}, {wid, w}}, dst, n);
            std::vector<float> want(n);
            EXPECT(orc_linear((int)dt, w.data(), w.size(), rows * in_f, row0 * in_f, x.data(), want.data(), 1, in_f,
                              n, 0, 0) == 0, "oracle");
            char what[64];
            std::snprintf(what, sizeof what, "%s rows %zu..%zu", dtype_name(dt), row0, row0 + n);
            gate(what, got, want);
        }
    }
}

// RmsNorm -> q/k/v; o -> Add; RmsNorm -> gate/up -> GatedAct -> down -> Add, one token, executed
// three times on one plan with fresh inputs; every stage against the oracle fed with the device's
// own upstream tensor.
static void hip_decoder_layer_graph_matches_the_cpu_arms(HipBackend& be) {
    const uint32_t H = 1024, KV = 256, FF = 2816;
    Graph g;
    Bindings binds;
    std::vector<Buffer> keep;
    auto f32_tensor = [&](TensorKind k, std::vector<size_t> shape, const std::vector<float>* data) {
        TensorDesc d{std::move(shape), DType::F32};
        const size_t n = d.numel();
        const TensorId t = k == TensorKind::Input ? g.input(d) : g.output(d);
        keep.push_back(be.alloc(n * 4, BufferUsage::Activations));
        if (data) be.upload(keep.back(), *data);
        binds.bind(t, keep.back());
        return std::pair<TensorId, size_t>{t, keep.size() - 1};
    };
    std::vector<std::vector<uint8_t>> wbytes;
    auto weight = [&](DType dt, size_t out_f, size_t in_f, uint32_t seed) {
        // zero-mean weights (the LCG recipe's are mostly positive, which drives every gate far
        // negative and the whole activation to zero): nearest-code encodings of N(0, 0.05^2) draws
        wbytes.emplace_back(TensorDesc{{out_f, in_f}, dt}.nbytes());
        if (infr_synth_weight((int)dt, seed, 0.05f, out_f, in_f, wbytes.back().data()) != wbytes.back().size())
            throw std::runtime_error("infr_synth_weight");
        const TensorId t = g.weight({{out_f, in_f}, dt});
        keep.push_back(be.alloc(wbytes.back().size(), BufferUsage::Weights));
        be.upload(keep.back(), wbytes.back());
        binds.bind(t, keep.back());
        return std::pair<TensorId, size_t>{t, wbytes.size() - 1};
    };
    std::vector<float> n1w = gen_f32(H, 3), n2w = gen_f32(H, 4);
    for (auto* v : {&n1w, &n2w})
        for (float& f : *v) f = 1.0f + 0.1f * f;
    auto [x, xb] = f32_tensor(TensorKind::Input, {1, H}, nullptr);
    auto [n1, n1b] = f32_tensor(TensorKind::Input, {H}, &n1w);
    auto [n2, n2b] = f32_tensor(TensorKind::Input, {H}, &n2w);
    (void)n1b; (void)n2b;
    auto [h1, h1b] = f32_tensor(TensorKind::Output, {1, H}, nullptr);
    auto [q, qb] = f32_tensor(TensorKind::Output, {1, H}, nullptr);
    auto [k, kb] = f32_tensor(TensorKind::Output, {1, KV}, nullptr);
    auto [v, vb] = f32_tensor(TensorKind::Output, {1, KV}, nullptr);
    auto [o, ob] = f32_tensor(TensorKind::Output, {1, H}, nullptr);
    auto [h2, h2b] = f32_tensor(TensorKind::Output, {1, H}, nullptr);
    auto [gt, gtb] = f32_tensor(TensorKind::Output, {1, FF}, nullptr);
    auto [up, upb] = f32_tensor(TensorKind::Output, {1, FF}, nullptr);
    auto [act, actb] = f32_tensor(TensorKind::Output, {1, FF}, nullptr);
    auto [down, downb] = f32_tensor(TensorKind::Output, {1, H}, nullptr);
    auto [wq, wqi] = weight(DType::Q4K, H, H, 11);
    auto [wk, wki] = weight(DType::Q4K, KV, H, 12);
    auto [wv, wvi] = weight(DType::Q6K, KV, H, 13);
    auto [wo, woi] = weight(DType::Q4K, H, H, 14);
    auto [wg, wgi] = weight(DType::Q4K, FF, H, 15);
    auto [wu, wui] = weight(DType::Q4K, FF, H, 16);
    auto [wd, wdi] = weight(DType::Q6K, H, FF, 17);
    g.push(op::RmsNorm{x, n1, h1, 1, H, 1e-6f});
    g.push(op::Linear{h1, wq, q, 1, H, H});
    g.push(op::Linear{h1, wk, k, 1, H, KV});
    g.push(op::Linear{h1, wv, v, 1, H, KV});
    g.push(op::Linear{q, wo, o, 1, H, H});
    g.push(op::Add{o, x, x});  // residual in place
    g.push(op::RmsNorm{x, n2, h2, 1, H, 1e-6f});
    g.push(op::Linear{h2, wg, gt, 1, H, FF});
    g.push(op::Linear{h2, wu, up, 1, H, FF});
    g.push(op::GatedAct{gt, up, act, 1, FF});
    g.push(op::Linear{act, wd, down, 1, FF, H});
    g.push(op::Add{down, x, x});
    Plan plan = be.compile(g);

    auto get = [&](size_t buf, size_t n) {
        std::vector<float> out(n);
        be.download(keep[buf], out);
        return out;
    };
    auto lin = [&](DType dt, size_t wi, const std::vector<float>& in, size_t in_f, size_t out_f) {
        std::vector<float> y(out_f);
        orc_linear((int)dt, wbytes[wi].data(), wbytes[wi].size(), out_f * in_f, 0, in.data(), y.data(), 1, in_f, out_f,
                   0, 0);
        return y;
    };
    for (int rep = 0; rep < 3; ++rep) {
        const std::vector<float> x0 = gen_f32(H, 100 + rep);
        be.upload(keep[xb], x0);
        be.execute(plan, binds);
        const auto d_h1 = get(h1b, H), d_q = get(qb, H), d_k = get(kb, KV), d_v = get(vb, KV), d_o = get(ob, H);
        const auto d_h2 = get(h2b, H), d_g = get(gtb, FF), d_u = get(upb, FF), d_act = get(actb, FF);
        const auto d_down = get(downb, H), d_x = get(xb, H);
        std::vector<float> w_h1(H), x1(H), w_h2(H), w_act(FF), x2(H);
        if (getenv("OP_PARITY_DEBUG"))
            std::printf("  max|.|: h1 %.3e q %.3e o %.3e h2 %.3e gate %.3e up %.3e act %.3e down %.3e x %.3e\n", max_abs(d_h1),
                        max_abs(d_q), max_abs(d_o), max_abs(d_h2), max_abs(d_g), max_abs(d_u), max_abs(d_act),
                        max_abs(d_down), max_abs(d_x));
        orc_rms_norm(x0.data(), n1w.data(), w_h1.data(), 1, H, 1e-6f, 0);
        EXPECT(rel_l2(d_h1, w_h1) < 2e-6f, "rep %d: RmsNorm 1", rep);
        gate("q", d_q, lin(DType::Q4K, wqi, d_h1, H, H));
        gate("k", d_k, lin(DType::Q4K, wki, d_h1, H, KV));
        gate("v", d_v, lin(DType::Q6K, wvi, d_h1, H, KV));
        EXPECT(same_bits(d_o, lin(DType::Q4K, woi, d_q, H, H)), "rep %d: o is not bit-identical", rep);
        orc_add(d_o.data(), x0.data(), x1.data(), H);
        orc_rms_norm(x1.data(), n2w.data(), w_h2.data(), 1, H, 1e-6f, 0);
        EXPECT(rel_l2(d_h2, w_h2) < 2e-6f, "rep %d: RmsNorm 2", rep);
        gate("gate", d_g, lin(DType::Q4K, wgi, d_h2, H, FF));
        gate("up", d_u, lin(DType::Q4K, wui, d_h2, H, FF));
        orc_gated_act_op(d_g.data(), d_u.data(), w_act.data(), 1, FF, 0, 0, 0, 0, 0, 0, 0.0f);
        EXPECT(rel_l2(d_act, w_act) < 2e-6f, "rep %d: GatedAct", rep);
        gate("down", d_down, lin(DType::Q6K, wdi, d_act, FF, H));
        orc_add(d_down.data(), x1.data(), x2.data(), H);
        EXPECT(same_bits(d_x, x2), "rep %d: residual stream differs", rep);
    }
    EXPECT(plan.launches() > 0 && plan.launches() < 12, "launch count %zu", plan.launches());
}

// Op::MoeFfn through a plan against the CPU arm (crates/infr-cpu/src/lib.rs:2264-2984): one row
// (decoded f32 weights) and four rows (int8 path).
static void hip_moe_ffn_matches_the_cpu_arm(HipBackend& be) {
    const uint32_t ne = 512, nff = 256, n_expert = 16, n_used = 4;
    const std::vector<uint8_t> gate_w = synth_weight(DType::Q4K, (size_t)n_expert * nff * ne, 21);
    const std::vector<uint8_t> up_w = synth_weight(DType::Q4K, (size_t)n_expert * nff * ne, 22);
    const std::vector<uint8_t> down_w = synth_weight(DType::Q6K, (size_t)n_expert * ne * nff, 23);
    std::vector<float> router = gen_f32((size_t)n_expert * ne, 24);
    for (size_t i = 0; i < router.size(); ++i) router[i] *= 0.25f * (float)(1 + (i / ne) % 5);
    for (uint32_t rows : {1u, 4u}) {
        const std::vector<float> x = gen_f32((size_t)rows * ne, 30 + rows);
        Graph g;
        const TensorId xid = g.input({{rows, ne}, DType::F32});
        const TensorId rid = g.weight({{n_expert, ne}, DType::F32});
        const TensorId gid = g.weight({{n_expert, nff, ne}, DType::Q4K});
        const TensorId uid = g.weight({{n_expert, nff, ne}, DType::Q4K});
        const TensorId did = g.weight({{n_expert, ne, nff}, DType::Q6K});
        const TensorId dst = g.output({{rows, ne}, DType::F32});
        // qwen3moe's setting, then llama4's (sigmoid gating, raw weights, weight on the expert input;
        // graph.rs:956-967) with a GELU expert
        for (int variant = 0; variant < 2; ++variant) {
            op::MoeFfn moe{xid, xid, rid, gid, uid, did, dst, ne, n_expert, n_used, nff, 1.0f};
            orc_moe_params p{};
            p.ne = ne; p.n_expert = n_expert; p.n_used = n_used; p.n_ff_exp = nff; p.rows = rows; p.scale = 1.0f;
            p.router_dtype = 0; p.gate_dtype = 12; p.up_dtype = 12; p.down_dtype = 14; p.norm_w = 1;
            if (variant == 1) {
                moe.gating = MoeGating::Sigmoid; moe.norm_w = false; moe.weight_before = true; moe.act = Activation::Gelu;
                p.gating = ORC_GATING_SIGMOID; p.norm_w = 0; p.weight_before = 1; p.act = ORC_ACT_GELU;
            }
            Graph gv = g;
            gv.push(moe);
            const std::vector<float> got = run_graph(
                be, gv, {{xid, f32_bytes(x)}, {rid, f32_bytes(router)}, {gid, gate_w}, {uid, up_w}, {did, down_w}}, dst,
                (size_t)rows * ne);
            std::vector<float> want((size_t)rows * ne);
            const int rc = orc_moe_ffn(&p, x.data(), x.data(), (const uint8_t*)router.data(), router.size() * 4,
                                       gate_w.data(), gate_w.size(), up_w.data(), up_w.size(), down_w.data(),
                                       down_w.size(), want.data(), nullptr, nullptr, 0, nullptr, nullptr, nullptr);
            EXPECT(rc == 0, "oracle MoeFfn rc %d", rc);
            gate(variant ? (rows == 1 ? "MoeFfn llama4-style rows=1" : "MoeFfn llama4-style rows=4")
                         : (rows == 1 ? "MoeFfn rows=1" : "MoeFfn rows=4"), got, want);
        }
        // an expert-parallel band is another GPU's business: refused, never read as the whole bank
        {
            op::MoeFfn moe{xid, xid, rid, gid, uid, did, dst, ne, n_expert, n_used, nff, 1.0f};
            moe.ep_band = std::make_pair(0u, 8u);
            Graph gv = g;
            gv.push(moe);
            bool refused = false;
            try {
                (void)run_graph(be, gv, {{xid, f32_bytes(x)}, {rid, f32_bytes(router)}, {gid, gate_w}, {uid, up_w}, {did, down_w}},
                                dst, (size_t)rows * ne);
            } catch (const Error& e) {
                refused = e.kind == ErrorKind::Unsupported;
            }
            EXPECT(refused, "MoeFfn with ep_band must be Unsupported");
        }
    }
}

// Op::EmbedGather equals the host decode times scale, bit for bit (lib.rs:2084-2111)
static void hip_embed_gather_equals_the_host_decode(HipBackend& be) {
    const uint32_t ne = 512, vocab = 64, rows = 5;
    const std::vector<int32_t> ids = {3, 63, 0, 17, 3};
    for (DType dt : {DType::Q4K, DType::Q6K, DType::Q8_0, DType::Q5_0}) {
        const std::vector<uint8_t> table = synth_weight(dt, (size_t)vocab * ne, 0x31);
        Graph g;
        const TensorId iid = g.input({{rows}, DType::I32});
        const TensorId tid = g.weight({{vocab, ne}, dt});
        const TensorId dst = g.output({{rows, ne}, DType::F32});
        g.push(op::EmbedGather{iid, tid, dst, rows, ne, 1.5f});
        std::vector<uint8_t> idb(rows * 4);
        std::memcpy(idb.data(), ids.data(), idb.size());
        const std::vector<float> got = run_graph(be, g, {{iid, idb}, {tid, table}}, dst, (size_t)rows * ne);
        std::vector<float> want((size_t)rows * ne);
        EXPECT(orc_embed_gather((int)dt, table.data(), table.size(), (size_t)vocab * ne, ids.data(), rows, ne, 1.5f,
                                want.data()) == 0, "oracle EmbedGather");
        EXPECT(same_bits(got, want), "%s: EmbedGather differs from the host decode", dtype_name(dt));
    }
}

// The parts of the trait's contract a caller relies on (backend.rs:486-662).
static void hip_backend_honours_the_seam_contract(HipBackend& be) {
    EXPECT(!be.name().empty(), "name");
    const Capabilities caps = be.capabilities();
    EXPECT(caps.i8 && caps.i8_dot && caps.decode_replay, "capabilities");
    // both ops are built here, so the runner may emit them (backend.rs:160-164)
    EXPECT(caps.combined_gu == 1 && caps.embed_gather == 1, "combined_gu / embed_gather are advertised");
    EXPECT(caps.gpu_sample == 0 && caps.argmax_rows == 0 && caps.gated_rmsnorm == 0, "host-side ops stay off");
    // alloc is zero-initialised (calloc semantics, backend.rs:491-496)
    Buffer z = be.alloc(4096, BufferUsage::Activations);
    std::vector<uint8_t> host(4096, 0xAB);
    be.download(z, host);
    EXPECT(std::all_of(host.begin(), host.end(), [](uint8_t b) { return b == 0; }), "alloc is not zeroed");
    EXPECT(z.len_bytes() == 4096 && z.device_addr() != 0, "buffer length / address");
    // copy_buffer: an oversize copy is an error, not a fault (backend.rs:23-30)
    Buffer small = be.alloc(64, BufferUsage::Activations);
    bool threw = false;
    try { be.copy_buffer(z, small, 4096); } catch (const Error&) { threw = true; }
    EXPECT(threw, "oversize copy_buffer did not fail");
    std::vector<uint8_t> pat(64);
    for (size_t i = 0; i < 64; ++i) pat[i] = (uint8_t)(i * 7);
    be.upload(small, pat);
    be.copy_buffer(small, z, 64);
    be.download(z, host.data(), 64);
    EXPECT(std::memcmp(host.data(), pat.data(), 64) == 0, "copy_buffer bytes");
    // an unbound tensor is reported (the reference panics), nothing is launched
    Graph g;
    const TensorId xid = g.input({{1, 256}, DType::F32});
    const TensorId wid = g.weight({{8, 256}, DType::Q4K});
    const TensorId dst = g.output({{1, 8}, DType::F32});
    g.push(op::Linear{xid, wid, dst, 1, 256, 8, 0});
    Plan plan = be.compile(g);
    Bindings b;
    Buffer xb = be.alloc(1024, BufferUsage::Activations);
    b.bind(xid, xb);
    threw = false;
    try { be.execute(plan, b); } catch (const Error& e) { threw = e.kind == ErrorKind::Invalid; }
    EXPECT(threw, "execute with an unbound weight did not report Invalid");
    // a format outside this backend is Unsupported at compile, never a wrong answer
    Graph g2;
    const TensorId w2 = g2.weight({{8, 256}, (DType)16 /* IQ2_XXS */});
    const TensorId x2 = g2.input({{1, 256}, DType::F32});
    const TensorId d2 = g2.output({{1, 8}, DType::F32});
    g2.push(op::Linear{x2, w2, d2, 1, 256, 8, 0});
    threw = false;
    try { Plan p2 = be.compile(g2); } catch (const Error& e) { threw = e.kind == ErrorKind::Unsupported; }
    EXPECT(threw, "IQ2_XXS Linear did not report Unsupported");
    // a ragged row is refused, not truncated
    Graph g3;
    const TensorId w3 = g3.weight({{8, 128}, DType::Q4K});
    const TensorId x3 = g3.input({{1, 128}, DType::F32});
    const TensorId d3 = g3.output({{1, 8}, DType::F32});
    g3.push(op::Linear{x3, w3, d3, 1, 128, 8, 0});
    threw = false;
    try { Plan p3 = be.compile(g3); } catch (const Error&) { threw = true; }
    EXPECT(threw, "in_f = 128 for Q4_K was accepted");
}

int main(int argc, char** argv) {
    const std::vector<std::pair<const char*, std::function<void(HipBackend&)>>> tests = {
        {"hip_backend_honours_the_seam_contract", hip_backend_honours_the_seam_contract},
        {"hip_linear_all_weight_quants_match_the_host_oracle", hip_linear_all_weight_quants_match_the_host_oracle},
        {"hip_linear_matches_the_cpu_production_arm", hip_linear_matches_the_cpu_production_arm},
        {"hip_linear_batch_rows_equal_single_rows", hip_linear_batch_rows_equal_single_rows},
        {"hip_linear_w_off_slices_a_concatenated_weight", hip_linear_w_off_slices_a_concatenated_weight},
        {"hip_decoder_layer_graph_matches_the_cpu_arms", hip_decoder_layer_graph_matches_the_cpu_arms},
        {"hip_moe_ffn_matches_the_cpu_arm", hip_moe_ffn_matches_the_cpu_arm},
        {"hip_embed_gather_equals_the_host_decode", hip_embed_gather_equals_the_host_decode},
    };
    if (argc == 2 && std::string(argv[1]) == "--list") {
        for (const auto& t : tests) std::printf("%s\n", t.first);
        return 0;
    }
    int failed = 0, ran = 0;
    try {
        HipBackend be(0);
        for (const auto& [name, fn] : tests) {
            if (argc > 1 && std::find_if(argv + 1, argv + argc, [&](char* a) { return std::string(a) == name; }) == argv + argc)
                continue;
            std::printf("test %s ...\n", name);
            std::fflush(stdout);
            const int before = g_checks_failed;
            try {
                fn(be);
            } catch (const std::exception& e) {
                ++g_checks_failed;
                std::printf("  FAILED: exception: %s\n", e.what());
            }
            ++ran;
            const bool ok = g_checks_failed == before;
            failed += !ok;
            std::printf("test %s ... %s\n", name, ok ? "ok" : "FAILED");
            std::fflush(stdout);
        }
    } catch (const Error& e) {
        std::printf("no usable gfx950 device: %s\n", e.what());
        return 99;
    }
    std::printf("test result: %s. %d passed; %d failed\n", failed ? "FAILED" : "ok", ran - failed, failed);
    return failed ? 1 : (ran ? 0 : 2);
}
