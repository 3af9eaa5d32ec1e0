/*
 * CPU oracle for the quantized-matmul path of kryptic-sh/infr's `infr-cpu` backend.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE. It is a plain-C restatement of the reference's
 * scalar kernels, written from the Rust source text (the reference cannot be compiled where this
 * is built: no Rust toolchain). Only tests, the smoke check and the benchmark's CPU-baseline leg
 * may link or load it; the shipped GPU library never does.
 *
 * Every function names the reference file:line it follows (paths relative to the reference
 * checkout). All float arithmetic must be compiled with -ffp-contract=off: Rust never fuses
 * a*b+c unless `mul_add` is written, and the places that do use `mul_add` call fmaf() here.
 *
 * Pinning status (what independent evidence each function is checked against lives in
 * tests/test_oracle_*.py):
 *   orc_rdf16 / orc_f32_to_f16   exhaustive round trip over all 65,536 f16 values + numpy float16
 *   orc_k4                        hand-derived split-bit vector, independent numpy restatement
 *   orc_dequant_block             reference's q2_0_single_block known answer; hand-derived
 *                                 all-2.0 blocks; independent byte-at-a-time numpy decoders
 *   orc_quantize_q8 / _q8_32      hand-derived tie vector (half away from zero), zero block,
 *                                 one-hot, bsums identities, reconstruction error <= d/2
 *   orc_vec_dot_*                 hand-derived 65024 vectors; brute-force int64 dots;
 *                                 dot(dequant(w), dequant(q8)) at the reference's own 1e-3
 *   Q5_K / Q4_0 / Q4_1 / Q5_0 / Q5_1 / IQ4_NL (dequant, orc_vec_dot_q5k, orc_vec_dot_blk32)
 *                                 the reference's five single-block known answers; hand blocks for
 *                                 the 5th code bit; independent numpy decoders bit for bit; int64
 *                                 brute-force stages; per-block f32 terms re-evaluated in numpy f32
 *   Q2_K / Q3_K (dequant, orc_vec_dot_q2k, orc_vec_dot_q3k, orc_q3k_scales)
 *                                 the reference's q2k_single_block / q3k_single_block known answers;
 *                                 hand blocks (each shift position, the hmask bit, a split scale
 *                                 field); independent numpy decoders bit for bit; int64 brute-force
 *                                 stages; per-superblock f32 terms re-evaluated in numpy f32
 *   TQ1_0 (dequant, orc_tq1_0_digit, orc_vec_dot_tq1_0)
 *                                 the reference's tq1_0_single_block known answer; all 243 five-digit
 *                                 strings packed by the format's rule come back; the element order
 *   TQ2_0 / MXFP4 / NVFP4 (dequant, orc_vec_dot_tq2_0, orc_vec_dot_mxfp4, orc_vec_dot_nvfp4, scale decoders)
 *                                 the reference's three single-block known answers; every E8M0 and
 *                                 UE4M3 byte against its definition; hand blocks; the rest as above
 *   IQ4_XS (dequant, orc_vec_dot_iq4xs, orc_iq4xs_scale)
 *                                 the reference's iq4xs_single_block known answer; a hand block with a
 *                                 scale per sub-block and a code per nibble position; the rest as above
 *   orc_vec_dot_q8_0_32           brute-force int64 dots; hand-derived known answer
 *   orc_rms_norm / orc_gated_act* / orc_add / orc_act
 *                                 closed forms at hand-picked points; layouts against written-out
 *                                 index arithmetic
 *   orc_linear                    batch == single bit-identical; f64 oracle at the reference's 2e-2;
 *                                 reference mode at 1e-5
 *   orc_moe_ffn                   textbook f32 MoE (restated from the reference's moe_ref test helper)
 *                                 at the reference's 1e-4; routing invariants
 *   Not pinnable without the Rust binary (parity unpinned): the exact f32 bit pattern the reference
 *   emits on a given host ISA for Q8_0 (its AVX-512 tier pairs blocks) and libm-dependent expf
 *   bits in the MoE router/SiLU; both are immaterial at the 1e-4 gate.
 */
#ifndef INFR_CPU_ORACLE_H
#define INFR_CPU_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* GGML type ids (crates/infr-gguf/src/lib.rs:330-354). */
enum {
    ORC_F32 = 0,
    ORC_F16 = 1,
    ORC_Q4_0 = 2,
    ORC_Q4_1 = 3,
    ORC_Q5_0 = 6,
    ORC_Q5_1 = 7,
    ORC_Q8_0 = 8,
    ORC_Q2_K = 10,
    ORC_Q3_K = 11,
    ORC_IQ4_XS = 23,
    ORC_TQ1_0 = 34,
    ORC_TQ2_0 = 35,
    ORC_MXFP4 = 39,
    ORC_NVFP4 = 40,
    ORC_Q4_K = 12,
    ORC_Q5_K = 13,
    ORC_Q6_K = 14,
    ORC_IQ4_NL = 20,
    ORC_BF16 = 30,
    ORC_Q2_0 = 42
};

/* Activation kinds chosen by the MoE dispatch (crates/infr-cpu/src/moe.rs:32-53). */
enum { ORC_ACTS_SUPER = 0, ORC_ACTS_BLK32 = 1, ORC_ACTS_RAW = 2 };

/* crates/infr-core/src/decode_spec.rs:319-358 — (elements, bytes) per block; 0 on unknown dtype. */
int orc_block_layout(int dtype, int *elems, int *bytes);

/* crates/infr-gguf/src/dequant.rs:68-70 (half::f16::to_f32, exact widening). */
float orc_rdf16(const uint8_t *b);
float orc_f16_bits_to_f32(uint16_t h);
/* half::f16::from_f32 — IEEE round-to-nearest-even narrowing (used by the test synthesizers,
 * crates/infr-core/src/decode_spec.rs:187-190). */
uint16_t orc_f32_to_f16_bits(float f);

/* crates/infr-gguf/src/dequant.rs:73-83 */
void orc_k4(int j, const uint8_t *q, uint32_t *sc, uint32_t *m);

/* crates/infr-gguf/src/dequant.rs:11-51 (affine: sc*code + mn, two roundings), :998-1018 (Q2_0).
 * `out` holds nbytes/block_bytes*block_elems floats. Returns 0, or -1 on unsupported dtype. */
int orc_dequant_block(int dtype, const uint8_t *bytes, size_t nbytes, float *out);

/* crates/infr-cpu/src/quant.rs:27-58. nb = len/256 blocks (a shorter tail is dropped).
 * qs[nb*256], d[nb], bsums[nb*8], bsums16[nb*16] (bsums16 may be NULL). */
void orc_quantize_q8(const float *x, size_t len, int8_t *qs, float *d, int32_t *bsums,
                     int32_t *bsums16);
/* crates/infr-cpu/src/quant.rs:97-117. nb = len/32. qs[nb*32], d[nb], bsum[nb]. */
void orc_quantize_q8_32(const float *x, size_t len, int8_t *qs, float *d, int32_t *bsum);

/* Scalar single-row dots. The optional int-stage outputs receive the per-block integers the f32
 * epilogue consumes (NULL to skip).
 * Q4_K: crates/infr-cpu/src/kernels.rs:151-184 — sd[nb], sm[nb].
 * Q6_K: kernels.rs:487-526 — isum[nb].
 * Q8_0: kernels.rs:1170-1187 — iprod[in_f/32].
 * Q2_0: kernels.rs:5641-5668 — iprod[in_f/32] (codes 0..3, before the -bsum correction). */
float orc_vec_dot_q4k(const uint8_t *row, const int8_t *qs, const float *d, const int32_t *bsums,
                      size_t in_f, int32_t *sd_out, int32_t *sm_out);
float orc_vec_dot_q6k(const uint8_t *row, const int8_t *qs, const float *d, size_t in_f,
                      int32_t *isum_out);
float orc_vec_dot_q8_0(const uint8_t *row, const int8_t *qs, const float *d, size_t in_f,
                       int32_t *iprod_out);
/* kernels.rs:4972-4991 — Q8_0 against the per-32 activation (in_f % 256 != 0). */
float orc_vec_dot_q8_0_32(const uint8_t *row, const int8_t *qs, const float *d32, size_t in_f,
                          int32_t *iprod_out);
float orc_vec_dot_q2_0(const uint8_t *row, const int8_t *qs, const float *d, const int32_t *bsum,
                       size_t in_f, int32_t *iprod_out);
/* Q5_K: kernels.rs:1286-1327 — sd[nb], sm[nb] like Q4_K. */
float orc_vec_dot_q5k(const uint8_t *row, const int8_t *qs, const float *d, const int32_t *bsums,
                      size_t in_f, int32_t *sd_out, int32_t *sm_out);
/* Q2_K: kernels.rs:315-361 (vec_dot_q2k_scalar) - sd[nb], sm[nb]; the min term reads the per-16 sums. */
float orc_vec_dot_q2k(const uint8_t *row, const int8_t *qs, const float *d, const int32_t *bsums16,
                      size_t in_f, int32_t *sd_out, int32_t *sm_out);
/* Q3_K: kernels.rs:812-852 (vec_dot_q3k_scalar), scales by kernels.rs:764-783 (q3k_scales) - isum[nb]. */
float orc_vec_dot_q3k(const uint8_t *row, const int8_t *qs, const float *d, const int32_t *bsums16,
                      size_t in_f, int32_t *isum_out);
/* IQ4_XS: kernels.rs:1008-1036 (vec_dot_iq4xs_scalar), scale by kernels.rs:995-1002 - isum[nb]. */
float orc_vec_dot_iq4xs(const uint8_t *row, const int8_t *qs, const float *d, size_t in_f, int32_t *isum_out);
int orc_iq4xs_scale(uint32_t scales_h, const uint8_t *scales_l, int ib);
/* TQ1_0: kernels.rs:3167-3240 (tq1_0_expand_row + vec_dot_tq1_0) - iprod[nb]; digit of element i of a block. */
float orc_vec_dot_tq1_0(const uint8_t *row, const int8_t *qs, const float *d, size_t in_f, int32_t *iprod_out);
int orc_tq1_0_digit(const uint8_t *blk, int i);
/* TQ2_0: kernels.rs:3066-3126 (tq2_0_expand_row + vec_dot_tq2_0) - iprod[nb]. */
float orc_vec_dot_tq2_0(const uint8_t *row, const int8_t *qs, const float *d, size_t in_f, int32_t *iprod_out);
/* MXFP4: kernels.rs:6303-6327 - iprod[in_f/32]; NVFP4: kernels.rs:6472-6500 - iprod[in_f/16]. Both
 * against the per-32 activation; scale decoders dequant.rs:411-435. */
float orc_vec_dot_mxfp4(const uint8_t *row, const int8_t *qs, const float *d, size_t in_f, int32_t *iprod_out);
float orc_vec_dot_nvfp4(const uint8_t *row, const int8_t *qs, const float *d, size_t in_f, int32_t *iprod_out);
float orc_e8m0_half(uint8_t x);
float orc_ue4m3_half(uint8_t x);
/* Q3_K's sixteen signed scales (sc6 - 32) of one block from its 12 scale bytes (kernels.rs:764-783). */
void orc_q3k_scales(const uint8_t *scales_raw, int16_t out[16]);
/* Q4_0 / Q4_1 / Q5_0 / Q5_1 / IQ4_NL against the per-32 activation: kernels.rs:5496-5520,
 * 5793-5822, 5350-5377, 5948-5980, 6128-6152 — iprod[in_f/32] (raw codes; IQ4_NL: codebook values). */
float orc_vec_dot_blk32(int dtype, const uint8_t *row, const int8_t *qs, const float *d,
                        const int32_t *bsum, size_t in_f, int32_t *iprod_out);
/* crates/infr-gguf/src/dequant.rs:439-441 */
extern const int8_t orc_kvalues_iq4nl[16];

/* crates/infr-cpu/src/kernels.rs:6557-6573 — 8 FMA accumulators, lanes summed in order, FMA tail. */
float orc_dot(const float *a, const float *b, size_t n);
/* kernels.rs:6578-6597 — act 0 = SiLU; gated_act_fn with clamp None. */
float orc_silu(float g);

/* ---- the ops either side of a Linear ---- */
enum { ORC_ACT_SILU = 0, ORC_ACT_GELU = 1, ORC_ACT_SIGMOID = 2 };
/* act_fn, kernels.rs:6578-6585 (Silu, gelu_pytorch_tanh, Sigmoid). */
float orc_act(int act, float g);
/* gated_act_fn, kernels.rs:6591-6597: act(gate) * up, or with a clamp
 * act(min(gate, l)) * clamp(up, -l, l). */
float orc_gated_act(int act, int has_clamp, float clamp, float gate, float up);
/* Op::RmsNorm / Op::RmsNormAdd arms, crates/infr-cpu/src/lib.rs:802-850: per row
 * ss = (sum_i x_i*x_i, in index order) / dim; s = 1 / sqrt(ss + eps); out_i = x_i * s * w_i
 * (accumulate != 0: out_i += ...). */
void orc_rms_norm(const float *x, const float *w, float *out, size_t rows, size_t dim, float eps,
                  int accumulate);
/* Op::GatedAct arm, lib.rs:1890-1944, with its strides, offset and interleaved-gate layout. */
void orc_gated_act_op(const float *gate, const float *up, float *out, size_t rows, size_t nff,
                      int act, size_t up_off, size_t up_stride, size_t gate_stride,
                      size_t gate_block_width, int has_clamp, float clamp);
/* Op::GatedActFused arm, lib.rs:1945-1971: gu is [rows, 2*nff], gate half first. */
void orc_gated_act_fused(const float *gu, float *out, size_t rows, size_t nff, int act,
                         int has_clamp, float clamp);
/* Op::Add arm, lib.rs:1972-1988. */
void orc_add(const float *a, const float *b, float *out, size_t n);

/* Op::EmbedGather arm, crates/infr-cpu/src/lib.rs:2084-2111: out[r, :] = dequant(table row ids[r]) * scale.
 * Returns 0; -1 unsupported dtype; -2 bad arguments or an id outside the table (the reference panics). */
int orc_embed_gather(int dtype, const uint8_t *table, size_t table_bytes, size_t table_numel,
                     const int32_t *ids, size_t rows, size_t ne, float scale, float *out);

/* crates/infr-cpu/src/lib.rs:985-1492 — the Op::Linear arm for Q4_K/Q6_K/Q8_0/Q2_0/F32 weights.
 *   w/wbytes: the whole bound weight buffer; w_numel: its declared element count;
 *   w_off: element offset of the first row (must be a multiple of in_f);
 *   x[m*in_f] f32; y[m*out_f] f32 row-major.
 *   reference_mode != 0 takes the exact branch (lib.rs:1015-1031): decode row to f32, plain dot.
 *   threads <= 0: all OpenMP threads.
 * Returns 0; -1 unsupported dtype/shape (the reference would take a fallback the restatement
 * does not carry); -2 bad arguments. */
int orc_linear(int dtype, const uint8_t *w, size_t wbytes, size_t w_numel, size_t w_off,
               const float *x, float *y, size_t m, size_t in_f, size_t out_f, int reference_mode,
               int threads);

/* Per-block integer stages of the production path for every (row r, output o), laid out
 * [m][out_f][blocks]: Q4_K -> a=sd, b=sm (blocks=in_f/256); Q6_K -> a=isum; Q8_0/Q2_0 -> a=iprod
 * (blocks=in_f/32). b may be NULL except for Q4_K. */
int orc_linear_int_stages(int dtype, const uint8_t *w, size_t wbytes, size_t w_numel, size_t w_off,
                          const float *x, size_t m, size_t in_f, size_t out_f, int32_t *a,
                          int32_t *b);

/* f64-accumulated reference GEMM over a decoded f32 weight (crates/infr-testkit/src/lib.rs:150-163). */
void orc_ref_linear_f64(const float *x, const float *w, size_t m, size_t in_f, size_t out_f,
                        float *out);

/* crates/infr-cpu/src/moe.rs:42-53 */
int orc_expert_acts_kind(int dtype, size_t in_f, int int8_ok);

/* Op::MoeFfn with every field of the op (crates/infr-core/src/graph.rs:918-1011). qwen3moe builds it
 * with softmax gating, norm_w, weight on the output side, split gate/up banks, SiLU and none of the
 * optional operands (crates/infr-llama/src/seam/runner.rs:3971-3997); a zeroed tail plus norm_w = 1
 * is that setting. ep_band is not restated: the CPU arm ignores it (lib.rs:2283). */
#define ORC_GATING_SOFTMAX 0
#define ORC_GATING_SIGMOID 1
#define ORC_GATING_SQRT_SOFTPLUS 2
typedef struct {
    uint32_t ne, n_expert, n_used, n_ff_exp, rows;
    float scale;
    int router_dtype, gate_dtype, up_dtype, down_dtype;
    int reference_mode;
    int act;            /* ORC_ACT_* */
    int gating;         /* ORC_GATING_* */
    int norm_w;         /* 1: w = p / max(sum_sel p, 1e-20) * scale; 0: w = p * scale */
    int weight_before;  /* 1: the routing weight multiplies gate and up before the activation */
    int fused_gate_up;  /* 1: `gate` holds [gate rows | up rows] per expert; `up` is not read */
    int has_clamp;      /* swiglu_clamp = Some(clamp) */
    float clamp;
    uint32_t n_expert_groups, n_expert_groups_used;
} orc_moe_params;

/* crates/infr-cpu/src/lib.rs:2264-2984. x, router_x: [rows, ne] f32. Banks: expert e is the e-th
 * equal byte slice. y[rows*ne]. sel_idx/sel_w (optional, [rows*n_used]) receive the routing
 * (descending-probability order, or the supplied ids' order). Optional operands, NULL when the op
 * has None: down_scale f32 [n_expert], exp_probs_b f32 [n_expert], expert_ids i32 [rows*n_used].
 * Returns 0, or negative on unsupported input and on the combinations the CPU arm asserts against
 * (a clamp with Sigmoid or weight_before; expert_ids with a bias or groups; an id >= n_expert). */
int orc_moe_ffn(const orc_moe_params *p, const float *x, const float *router_x,
                const uint8_t *router, size_t router_bytes, const uint8_t *gate, size_t gate_bytes,
                const uint8_t *up, size_t up_bytes, const uint8_t *down, size_t down_bytes,
                float *y, int32_t *sel_idx, float *sel_w, int threads, const float *down_scale,
                const float *exp_probs_b, const int32_t *expert_ids);

/* Test-input recipes the reference's own tests use (inputs only; it stores no expected outputs).
 * crates/infr-testkit/src/lib.rs:49-56 */
void orc_lcg_bytes(uint32_t seed, size_t n, uint8_t *out);
/* crates/infr-testkit/src/lib.rs:60-64 */
void orc_gen_f32(size_t n, size_t salt, float *out);
/* crates/infr-testkit/src/lib.rs:73-93,106-123 + decode_spec.rs:173-190 (write_scales, f16 slots).
 * Returns bytes written or 0 on unsupported dtype / ragged n_elem. */
size_t orc_synth_weight(int dtype, size_t n_elem, uint32_t seed, uint8_t *out);
/* crates/infr-cpu/src/kernels.rs:6611-6624 (kernel_tests::det_bytes / det_x). */
void orc_det_bytes(size_t n, uint64_t seed, uint8_t *out);
void orc_det_x(size_t n, uint64_t seed, float *out);

int orc_max_threads(void);

#ifdef __cplusplus
}
#endif
#endif
