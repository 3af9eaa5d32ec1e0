/*
 * infr_hip.h — C ABI of the MI355X (gfx950) backend for infr's quantized-matmul path.
 *
 * The entry points are what an `infr-hip` crate would bind to implement infr-core's `Backend`
 * trait (crates/infr-core/src/backend.rs:486-662) for the two ops on this path, `Op::Linear`
 * (crates/infr-core/src/graph.rs:177-191) and `Op::MoeFfn` (graph.rs:911-1011). Plain pointers,
 * sizes and opaque handles only; every call returns a status code and never throws or aborts
 * across the boundary. One HIP stream per backend; calls on one backend must be externally
 * serialised (the reference runner calls `execute` from one thread at a time,
 * crates/infr-cpu/src/pool.rs:216-240).
 *
 * There is no CPU fallback: every compute entry point fails with INFR_HIP_ERR_BACKEND when no
 * gfx950 device is usable.
 */
#ifndef INFR_HIP_H
#define INFR_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Mirrors infr_core::error::Error (crates/infr-core/src/error.rs:5-25); 0 = Ok. */
typedef enum {
    INFR_HIP_OK = 0,
    INFR_HIP_ERR_BACKEND = 1,     /* Error::Backend: device/runtime failure */
    INFR_HIP_ERR_LOADER = 2,      /* Error::Loader */
    INFR_HIP_ERR_MODEL = 3,       /* Error::Model */
    INFR_HIP_ERR_UNSUPPORTED = 4, /* Error::Unsupported: dtype/shape this backend does not take */
    INFR_HIP_ERR_ABORTED = 5,     /* Error::Aborted: shutdown latch was set */
    INFR_HIP_ERR_IO = 6,          /* Error::Io */
    INFR_HIP_ERR_OTHER = 7,       /* Error::Other */
    INFR_HIP_ERR_INVALID = 8      /* programmer error the reference would panic on (unbound
                                     buffer, size mismatch, misaligned w_off): reported, no abort */
} infr_hip_status;

/* Weight/activation element types, numbered as GGML type ids
 * (crates/infr-gguf/src/lib.rs:330-354; crates/infr-core/src/tensor.rs:7-57). */
typedef enum {
    INFR_DTYPE_F32 = 0,
    INFR_DTYPE_F16 = 1,   /* plain rows: embedding tables, Linear weights, MoE router and banks */
    INFR_DTYPE_Q4_0 = 2,  /* 32 / 18 B:  [f16 d][u8 qs[16]]             w = d*(q-8)        :311-312 */
    INFR_DTYPE_Q4_1 = 3,  /* 32 / 20 B:  [f16 d][f16 m][u8 qs[16]]      w = d*q+m          :313-314 */
    INFR_DTYPE_Q5_0 = 6,  /* 32 / 22 B:  [f16 d][u32 qh][u8 qs[16]]     w = d*(q-16)       :315-316 */
    INFR_DTYPE_Q5_1 = 7,  /* 32 / 24 B:  [f16 d][f16 m][u32 qh][u8 qs[16]]  w = d*q+m      :317-318 */
    INFR_DTYPE_Q8_0 = 8,  /* 32 elems / 34 B:  [f16 d][i8 qs[32]]            decode_spec.rs:319-320 */
    INFR_DTYPE_Q2_K = 10, /* 256 / 84 B:  [u8 scales[16]][u8 qs[64]][f16 d][f16 dmin]     :322-323 */
    INFR_DTYPE_Q3_K = 11, /* 256 / 110 B: [u8 hmask[32]][u8 qs[64]][u8 scales[12]][f16 d] :324-325 */
    INFR_DTYPE_Q4_K = 12, /* 256 / 144 B: [f16 d][f16 dmin][u8 sc[12]][u8 qs[128]]        :326-327 */
    INFR_DTYPE_Q5_K = 13, /* 256 / 176 B: [f16 d][f16 dmin][u8 sc[12]][u8 qh[32]][u8 qs[128]] :328-329 */
    INFR_DTYPE_Q6_K = 14, /* 256 / 210 B: [u8 ql[128]][u8 qh[64]][i8 sc[16]][f16 d]       :330-331 */
    INFR_DTYPE_IQ4_NL = 20, /* 32 / 18 B: [f16 d][u8 qs[16]]  w = d*codebook[q]           :349-350 */
    INFR_DTYPE_IQ4_XS = 23, /* 256 / 136 B: [f16 d][u16 scales_h][u8 scales_l[4]][u8 qs[128]] :351 */
    INFR_DTYPE_TQ1_0 = 34,  /* 256 / 54 B: [u8 qs[48]][u8 qh[4]][f16 d]  w = d*(digit-1), base-3 packed ternary :354 */
    INFR_DTYPE_TQ2_0 = 35,  /* 256 / 66 B: [u8 qs[64]][f16 d]  w = d*(q-1), 2-bit ternary codes         :356 */
    INFR_DTYPE_MXFP4 = 39,  /* 32 / 17 B: [u8 e][u8 qs[16]]  w = table[q] * 2^(e-128)             :361 */
    INFR_DTYPE_NVFP4 = 40,  /* 64 / 36 B: [u8 d[4]][u8 qs[32]]  w = table[q] * ue4m3(d[i/16]) / 2     :363 */
    INFR_DTYPE_BF16 = 30, /* plain rows, as F16 */
    INFR_DTYPE_Q2_0 = 42  /* 64 / 18 B:   [f16 d][u8 qs[16]] ternary-style 2-bit codes    :357-358 */
} infr_dtype;

/* infr_core::backend::BufferUsage (crates/infr-core/src/backend.rs:358-380). Advisory: every
 * class is device-local HBM here; upload/download stage through the copy engine. */
typedef enum {
    INFR_USAGE_WEIGHTS = 0,
    INFR_USAGE_ACTIVATIONS = 1,
    INFR_USAGE_KV_CACHE = 2,
    INFR_USAGE_STAGING = 3,
    INFR_USAGE_READBACK = 4,
    INFR_USAGE_HOST_WEIGHTS = 5
} infr_buffer_usage;

typedef struct infr_hip infr_hip_t;               /* a Backend instance            */
typedef struct infr_hip_buffer infr_hip_buffer_t; /* a Buffer (backend.rs:387-416) */
typedef struct infr_hip_plan infr_hip_plan_t;     /* a Plan   (backend.rs:418-446) */

/* Subset of infr_core::backend::Capabilities (backend.rs:43-213) this backend reports. */
typedef struct {
    int i8;                   /* int8 storage */
    int i8_dot;               /* packed 4x int8 dot (v_dot4) */
    int coopmat_i8_m, coopmat_i8_n, coopmat_i8_k; /* int8 MFMA tile */
    int decode_replay;        /* execute() replays a recorded launch sequence */
    int combined_gu;          /* 1: Linear onto [gate | up] + Op::GatedActFused (backend.rs:160-164) */
    int embed_gather;         /* 1: Op::EmbedGather decodes table rows on the device */
    int gpu_sample, argmax_rows, gated_rmsnorm; /* 0: the runner keeps these on the host */
    int graph_input_inplace;
    int unified_memory;
    uint64_t device_memory_bytes;
    int compute_units;
    char device_name[64];
} infr_hip_caps_t;

/* ---- lifetime (Backend construction; crates/infr-cpu/src/lib.rs:655-701 for the CPU peer) ---- */
int infr_hip_create(int device, infr_hip_t **out);
void infr_hip_destroy(infr_hip_t *be);
/* Backend::name (backend.rs:487) */
const char *infr_hip_name(const infr_hip_t *be);
/* Backend::capabilities (backend.rs:488) */
int infr_hip_capabilities(const infr_hip_t *be, infr_hip_caps_t *out);
/* Message of the last failing call on this backend (Error's payload string). With be == NULL,
 * the message of the last failing infr_hip_create on this thread. */
const char *infr_hip_last_error(const infr_hip_t *be);

/* ---- memory ---- */
/* Backend::alloc (backend.rs:491-496): zero-initialised, calloc semantics. */
int infr_hip_alloc(infr_hip_t *be, size_t bytes, int usage, infr_hip_buffer_t **out);
/* Backend::alloc_uninit (backend.rs:497-503). */
int infr_hip_alloc_uninit(infr_hip_t *be, size_t bytes, int usage, infr_hip_buffer_t **out);
/* Adopt device memory owned by the caller (e.g. a framework tensor) as a Buffer; never freed by
 * the backend. No reference counterpart: the reference's buffers are always backend-allocated. */
int infr_hip_wrap(infr_hip_t *be, void *device_ptr, size_t bytes, infr_hip_buffer_t **out);
/* Drop of Box<dyn Buffer>: the caller owns buffers and frees them. */
void infr_hip_free(infr_hip_t *be, infr_hip_buffer_t *buf);
/* Buffer::len_bytes / Buffer::device_addr (backend.rs:388-415). */
size_t infr_hip_buffer_len(const infr_hip_buffer_t *buf);
uint64_t infr_hip_buffer_device_addr(const infr_hip_buffer_t *buf);
/* Backend::upload / download (backend.rs:504-510). `n` must not exceed the buffer. download
 * observes every previously issued execute/linear on this backend. */
int infr_hip_upload(infr_hip_t *be, infr_hip_buffer_t *dst, const void *src, size_t n);
int infr_hip_download(infr_hip_t *be, const infr_hip_buffer_t *src, void *dst, size_t n);
/* Same with a byte offset into the buffer (the reference slices host-side before uploading). */
int infr_hip_upload_at(infr_hip_t *be, infr_hip_buffer_t *dst, size_t dst_off, const void *src, size_t n);
int infr_hip_download_at(infr_hip_t *be, const infr_hip_buffer_t *src, size_t src_off, void *dst, size_t n);
/* Backend::copy_buffer (backend.rs:547-558): oversize copies return an error, not a fault
 * (check_copy_bytes, backend.rs:23-30). */
int infr_hip_copy_buffer(infr_hip_t *be, const infr_hip_buffer_t *src, infr_hip_buffer_t *dst, size_t bytes);
/* Backend::sync (backend.rs:606). */
int infr_hip_sync(infr_hip_t *be);

/* ---- the hot path, op by op ---- */

/* Op::Linear (graph.rs:177-191; CPU arm crates/infr-cpu/src/lib.rs:985-1492):
 *   dst[m, out_f] = x[m, in_f] . W^T, W row-major [rows, in_f] in raw GGUF blocks of `dtype`.
 *   w        whole bound weight buffer; w_numel its declared element count (rows*in_f);
 *   w_off    element offset of the first row (multiple of in_f) inside a concatenated weight;
 *   x        f32 [m, in_f]; dst f32 [m, out_f], row-major.
 * Activations are quantized on the device exactly as infr-cpu does (per-256 int8 + f32 scale for
 * Q4_K/Q6_K/Q8_0, crates/infr-cpu/src/quant.rs:27-58; per-32 for Q2_0, quant.rs:97-117), the
 * integer dot is exact, and the f32 epilogue follows the CPU kernels' expression per block
 * (Q4_K from 128 tokens up fuses each block's products into its adds: y within 2e-6 relative of
 * infr-cpu instead of equal to it; the integers are exact there too).
 * in_f must be a whole number of weight blocks (256 for the K-quants, 64 for Q2_0, 32 otherwise): a
 * shorter tail is rejected, never truncated. in_f above 32768 (Q8_0, Q4_1, Q5_1: 16384) must be a
 * multiple of 256 (it then runs the prefill kernels at any m), else INFR_HIP_ERR_UNSUPPORTED.
 * Unquantized rows (F32, F16, BF16; in_f a multiple of 32) are multiplied as the CPU arm does
 * (lib.rs:1162-1164, 1443-1462: dot / dot_f16 / dot_bf16 - weights widened exactly, eight FMA
 * chains over the columns i mod 8, added in order): outputs equal infr-cpu's bit for bit. That
 * form is for the odd small matrix a quantized file keeps in floating point, not for speed. */
int infr_hip_linear(infr_hip_t *be, int dtype, const infr_hip_buffer_t *w, size_t w_numel,
                    size_t w_off, const infr_hip_buffer_t *x, infr_hip_buffer_t *dst, size_t m,
                    size_t in_f, size_t out_f);

/* Op::Linear without any device allocation. No counterpart in the reference: it is for callers
 * that cannot allocate device memory around the call - code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc. Arguments, kernels and results are those of
 * infr_hip_linear; the quantized activation of m >= 2 goes into a static device array of the
 * library instead of the backend's grow-on-demand scratch, so ceil32(m) * ceil256(in_f) must not
 * exceed 4,194,304 elements (e.g. 1024 tokens of 4096), else INFR_HIP_ERR_UNSUPPORTED. Each GPU holds one
 * such array (6 MiB) until the process ends and every backend on that GPU shares it: calls that
 * overlap on one GPU, from different backends or streams, race. The array keeps the last call's
 * contents and nothing needs clearing: the quantizer writes every slot the kernels read for the m
 * tokens, and what they compute for the padding tokens (m rounded up to 32) is never stored. */
int infr_hip_linear_noalloc(infr_hip_t *be, int dtype, const infr_hip_buffer_t *w, size_t w_numel,
                            size_t w_off, const infr_hip_buffer_t *x, infr_hip_buffer_t *dst, size_t m,
                            size_t in_f, size_t out_f);

/* quantize_q8 (crates/infr-cpu/src/quant.rs:27-58) for m rows of k floats (k % 256 == 0):
 *   qs i8 [m,k]; d f32 [m,k/256]; bsums i32 [m,k/32]; bsums16 i32 [m,k/16] (may be NULL).
 * Exposes the integer stage so callers can check it bit-for-bit. */
int infr_hip_quantize_q8(infr_hip_t *be, const infr_hip_buffer_t *x, size_t m, size_t k,
                         infr_hip_buffer_t *qs, infr_hip_buffer_t *d, infr_hip_buffer_t *bsums,
                         infr_hip_buffer_t *bsums16);
/* quantize_q8_32 (quant.rs:97-117), k % 32 == 0: qs i8 [m,k]; d f32 [m,k/32]; bsum i32 [m,k/32]. */
int infr_hip_quantize_q8_32(infr_hip_t *be, const infr_hip_buffer_t *x, size_t m, size_t k,
                            infr_hip_buffer_t *qs, infr_hip_buffer_t *d, infr_hip_buffer_t *bsum);

/* Per-block integer stages of Op::Linear for every (row r, output o), i32 [m][out_f][blocks]:
 *   Q4_K: a = sd, b = sm per 256-block (crates/infr-cpu/src/kernels.rs:162-181);
 *   Q6_K: a = isum per 256-block (kernels.rs:519-522);
 *   Q8_0: a = iprod per 32-block (kernels.rs:1182); Q2_0: a = iprod per 32 sub-block (:5657-5662);
 *   Q5_K: a = sd, b = sm; Q2_K: a = sd, b = sm (kernels.rs:315-361); Q3_K, IQ4_XS: a = isum (:812-852,
 *   :1008-1036); TQ1_0, TQ2_0: a = iprod per 256-block (:3218-3240, :3108-3126); the 32-weight-block formats and MXFP4:
 *   a = iprod per block. NVFP4 (four integers per block) and one token of Q5_0 (f32 activations)
 *   return Unsupported.
 * b may be NULL unless dtype is Q4_K, Q5_K or Q2_K. Uses the same device code as infr_hip_linear. */
int infr_hip_linear_int_stages(infr_hip_t *be, int dtype, const infr_hip_buffer_t *w,
                               size_t w_numel, size_t w_off, const infr_hip_buffer_t *x, size_t m,
                               size_t in_f, size_t out_f, infr_hip_buffer_t *a,
                               infr_hip_buffer_t *b);

/* Activation (crates/infr-core/src/graph.rs:47-54; act_fn in crates/infr-cpu/src/kernels.rs:6578-6585) */
typedef enum { INFR_ACT_SILU = 0, INFR_ACT_GELU = 1, INFR_ACT_SIGMOID = 2 } infr_activation;
/* MoeGating (crates/infr-core/src/graph.rs:76-85) */
typedef enum { INFR_GATING_SOFTMAX = 0, INFR_GATING_SIGMOID = 1, INFR_GATING_SQRT_SOFTPLUS = 2 } infr_moe_gating;

/* Op::MoeFfn, every field of the op (graph.rs:918-1011). qwen3moe emits softmax gating, norm_w,
 * weight on the expert output, split gate/up banks, SiLU and none of the optional operands
 * (crates/infr-llama/src/seam/runner.rs:3971-3997): act = gating = 0, norm_w = 1, the rest zero.
 * Expert e of a bank is its e-th equal byte slice. */
typedef struct {
    uint32_t ne, n_expert, n_used, n_ff_exp, rows;
    float scale;
    int router_dtype; /* INFR_DTYPE_F32, _F16 or _BF16 */
    int gate_dtype, up_dtype, down_dtype; /* any INFR_DTYPE_* (quantized, or plain F32 / F16 / BF16 rows), each bank its own */
    int act;            /* infr_activation: act(gate) * up per expert (graph.rs:948) */
    int gating;         /* infr_moe_gating (graph.rs:956-958) */
    int norm_w;         /* 1: w = p / max(sum of the selected p, 1e-20) * scale; 0: w = p * scale (graph.rs:959-962) */
    int weight_before;  /* 1: the routing weight multiplies gate and up before the activation, not the
                           expert output (llama4; graph.rs:963-967, CPU arm lib.rs:2833-2861, 2976) */
    int fused_gate_up;  /* 1: gate_exps holds [gate rows | up rows] per expert, up_exps and up_dtype are
                           not read (graph.rs:936-941) */
    int has_clamp;      /* swiglu_clamp = Some(clamp): act(min(gate, clamp)) * clamp(up, -clamp, clamp)
                           (graph.rs:949-955). As on the CPU (lib.rs:2293-2299) it is refused with
                           INFR_ACT_SIGMOID or weight_before. */
    float clamp;
    uint32_t n_expert_groups, n_expert_groups_used; /* group-limited routing when groups > 1 and used > 0:
                           a group's score is the sum of its two best selection values, the best `used`
                           groups stay, the rest are masked out (graph.rs:983-987, lib.rs:2488-2526);
                           n_expert a multiple of the groups, at most 64 groups */
    /* which optional operands the op carries (infr_hip_moe_optional_t / the op's tensor ids) */
    int has_down_scale;  /* down_scale: Some (graph.rs:932-935) */
    int has_exp_probs_b; /* exp_probs_b: Some (graph.rs:979-982) */
    int has_expert_ids;  /* expert_ids: Some (graph.rs:988-1010); refused together with exp_probs_b or
                            groups > 1, as on the CPU (lib.rs:2303-2309) */
    int has_ep_band;     /* ep_band: Some - an expert-parallel shard of the banks (graph.rs:968-978). This
                            backend runs one GPU and returns INFR_HIP_ERR_UNSUPPORTED for it. */
} infr_hip_moe_params_t;

/* The optional operands of Op::MoeFfn; each must be set exactly when its has_* flag is. */
typedef struct {
    const infr_hip_buffer_t *down_scale;  /* f32 [n_expert]: the selected expert's down output times
                                             down_scale[e] before the weighted sum (lib.rs:2932-2938) */
    const infr_hip_buffer_t *exp_probs_b; /* f32 [n_expert]: added to the probabilities for the SELECTION
                                             only; the weights use the unbiased ones (lib.rs:2476-2485) */
    const infr_hip_buffer_t *expert_ids;  /* i32 [rows, n_used]: the selection, in this order; the weights
                                             are the router's probabilities at these ids (lib.rs:2456-2472).
                                             An id outside [0, n_expert) is a panic on the CPU; here it is
                                             clamped into range and nothing is read out of bounds. */
} infr_hip_moe_optional_t;

/* CPU arm: crates/infr-cpu/src/lib.rs:2264-2984, crates/infr-cpu/src/moe.rs. As there, rows == 1
 * multiplies decoded f32 weights with the unquantized activation; rows >= 2 takes, per bank
 * (expert_acts_kind, moe.rs:42-53), per-256 int8 activations (Q4_K, Q5_K, Q6_K, Q8_0), per-32 int8
 * activations (Q5_0), or the same f32 arm (every other format). ne and n_ff_exp are multiples of 256.
 * Only the selected experts' blocks are read. `opt` may be NULL when the op has no optional operand;
 * up_exps may be NULL with fused_gate_up. sel_idx (i32) / sel_w (f32), [rows, n_used], are
 * optional outputs of the routing in descending-probability order (the supplied order with expert_ids).
 * Every combination of the fields above that the kernels do not implement returns
 * INFR_HIP_ERR_UNSUPPORTED; none is silently read as another. */
int infr_hip_moe_ffn(infr_hip_t *be, const infr_hip_moe_params_t *p, const infr_hip_buffer_t *x,
                     const infr_hip_buffer_t *router_x, const infr_hip_buffer_t *router,
                     const infr_hip_buffer_t *gate_exps, const infr_hip_buffer_t *up_exps,
                     const infr_hip_buffer_t *down_exps, const infr_hip_moe_optional_t *opt,
                     infr_hip_buffer_t *dst, infr_hip_buffer_t *sel_idx, infr_hip_buffer_t *sel_w);

/* Op::EmbedGather (crates/infr-core/src/graph.rs:853-865; CPU arm crates/infr-cpu/src/lib.rs:2084-2111):
 * dst[r, :] = decode(table[ids[r], :]) * scale for `rows` rows of `ne` elements. `table` holds
 * `table_numel / ne` rows of raw `dtype` blocks (every Linear weight format, F32, F16, BF16); `ids`
 * holds `rows` int32 token ids. Outputs equal infr-cpu's host decode times `scale` bit for bit. An id
 * outside the table gives a row of NaN (infr-cpu panics there); nothing is read out of bounds. */
int infr_hip_embed_gather(infr_hip_t *be, int dtype, const infr_hip_buffer_t *table, size_t table_numel,
                          const infr_hip_buffer_t *ids, size_t rows, size_t ne, float scale,
                          infr_hip_buffer_t *dst);

/* ---- graph level: Backend::compile / execute (backend.rs:560-577) over a flat C mirror of
 * infr_core::graph::Graph restricted to the ops of this path ---- */
typedef enum {
    INFR_OP_LINEAR = 1,
    INFR_OP_MOE_FFN = 2,
    /* the ops either side of every Linear in a decoder layer */
    INFR_OP_RMS_NORM = 3,        /* Op::RmsNorm, graph.rs:139-148; CPU arm lib.rs:802-825 */
    INFR_OP_RMS_NORM_ADD = 4,    /* Op::RmsNormAdd, graph.rs:149-158; lib.rs:826-850 */
    INFR_OP_GATED_ACT = 5,       /* Op::GatedAct, graph.rs:697-735; lib.rs:1890-1944 */
    INFR_OP_GATED_ACT_FUSED = 6, /* Op::GatedActFused, graph.rs:736-748; lib.rs:1945-1971 */
    INFR_OP_ADD = 7,             /* Op::Add, graph.rs:749-755; lib.rs:1972-1988 */
    INFR_OP_EMBED_GATHER = 8     /* Op::EmbedGather, graph.rs:853-865; lib.rs:2084-2111 */
} infr_hip_op_kind;

typedef struct {
    int kind;      /* infr_hip_op_kind */
    /* Op::Linear: tensor ids (indices into the bindings array) and shape */
    uint32_t x, weight, dst;
    uint32_t m, in_f, out_f;
    uint64_t w_off;
    uint64_t w_numel;
    int w_dtype;
    /* Op::MoeFfn; down_scale / exp_probs_b / expert_ids are read when moe.has_* says so */
    uint32_t router_x, router, gate_exps, up_exps, down_exps;
    uint32_t down_scale, exp_probs_b, expert_ids;
    infr_hip_moe_params_t moe;
    /* Elementwise ops, all f32. They reuse the fields above:
     *   RmsNorm / RmsNormAdd   x, weight (f32 [dim]), dst, m = rows, in_f = dim, eps
     *   GatedAct               x = gate, aux = up, dst, m = rows, in_f = nff, act, up_off, up_stride,
     *                          gate_stride, gate_block_width, has_clamp / clamp (swiglu_clamp)
     *   GatedActFused          x = gu [rows, 2*nff], dst, m = rows, in_f = nff, act, has_clamp / clamp
     *   Add                    x = a, aux = b, dst, in_f = n (m = 1); in place when dst == x
     * EmbedGather: x = ids (int32 [rows]), weight = table, dst (f32 [rows, ne]), m = rows, in_f = ne,
     *   w_numel = the table's element count, w_dtype, scale */
    uint32_t aux;
    float eps;
    int act; /* infr_activation */
    uint32_t up_off, up_stride, gate_stride, gate_block_width;
    int has_clamp;
    float clamp;
    float scale; /* EmbedGather */
} infr_hip_op_t;

/* Backend::compile: validates and stores the op list (the reference's GraphPlan clones the
 * graph, backend.rs:424-446). */
int infr_hip_compile(infr_hip_t *be, const infr_hip_op_t *ops, size_t n_ops, infr_hip_plan_t **out);
void infr_hip_plan_free(infr_hip_t *be, infr_hip_plan_t *plan);
/* Backend::execute: bindings[i] is the buffer bound to tensor id i (NULL = unbound;
 * Bindings, backend.rs:448-483). With the same bindings as the previous call on this plan the
 * recorded launch sequence is replayed (Capabilities::decode_replay, backend.rs:155-159).
 * Asynchronous: results are visible after infr_hip_sync or a download. */
int infr_hip_execute(infr_hip_t *be, infr_hip_plan_t *plan, infr_hip_buffer_t *const *bindings,
                     size_t n_bindings);
/* Number of kernel launches one execute of this plan issues for the bindings it last ran with
 * (0 before the first execute). Independent decode ops of one dependency level share a launch. */
size_t infr_hip_plan_launches(const infr_hip_plan_t *plan);

/* ---- shutdown latch (crates/infr-core/src/shutdown.rs:30-60): once requested, compute entry
 * points enqueue nothing further and return INFR_HIP_ERR_ABORTED; work already enqueued drains.
 * request_shutdown returns 1 if this call latched it, 0 if it was already set (signo != 0);
 * shutdown_signal returns the latched signal or 0. */
int infr_hip_request_shutdown(int signo);
int infr_hip_shutdown_requested(void);
int infr_hip_shutdown_signal(void);
void infr_hip_reset_shutdown(void); /* tests only: the reference's latch is monotonic */

/* ---- measurement: device-time of the work enqueued between begin and end on the backend's
 * stream (the reference's per-op timing seam, crates/infr-core/src/prof.rs:1-80) ---- */
int infr_hip_timer_begin(infr_hip_t *be);
int infr_hip_timer_end(infr_hip_t *be, float *elapsed_ms); /* synchronises */
/* Measurement aid with no counterpart in the reference: reads the first `bytes` of `src` `reps`
 * times with a plain streaming kernel (16-byte loads, whole lines per instruction, no arithmetic)
 * and reports the device time of those passes - the read bandwidth this device gives a kernel that
 * only fetches, which the HBM-bound GEMVs are compared with. `nontemporal` != 0 issues the loads
 * non-temporally, as the streamed decode GEMV fetches its weights. Synchronises. */
int infr_hip_stream_read(infr_hip_t *be, const infr_hip_buffer_t *src, size_t bytes, int reps, int nontemporal,
                         float *elapsed_ms);
/* Measurement aid with no counterpart in the reference: `iters` rounds of four independent
 * v_mfma_i32_32x32x32_i8 per wave, `waves_per_simd` (1..8) waves on every SIMD, operands in registers
 * (small constants, or pseudo-random bytes when random_data != 0). Reports the device time of one
 * launch and the integer operations it performed: the int8 matrix rate this device sustains with no
 * memory traffic, which the prefill kernels are compared with. Synchronises. */
int infr_hip_mfma_i8_peak(infr_hip_t *be, int waves_per_simd, int iters, int random_data, float *elapsed_ms, double *ops);

/* ---- deterministic synthetic inputs (host side, no device work). The reference has no weight
 * quantizer (it only reads GGUF) and its tests synthesize valid blocks
 * (crates/infr-testkit/src/lib.rs:106-123); these encoders produce valid blocks from
 * N(0, sigma^2) draws of a SplitMix64 + Box-Muller stream so every run sees identical bytes. ---- */
/* f32 N(mean, sigma^2), n values from `seed`. */
void infr_synth_normal_f32(uint64_t seed, float mean, float sigma, size_t n, float *out);
/* Draw rows*in_f weights N(0, sigma^2) from `seed` and encode them in `dtype`
 * (Q4_K/Q6_K/Q8_0: nearest-code encoders; Q2_0: codes uniform over {0,1,2} = {-1,0,+1} with
 * per-64 scale |N(0, sigma^2)|). Returns bytes written (0 on bad arguments). */
size_t infr_synth_weight(int dtype, uint64_t seed, float sigma, size_t rows, size_t in_f, uint8_t *out);
/* Block geometry: elements and bytes per block; returns 0 on unknown dtype. */
int infr_block_layout(int dtype, int *elems, int *bytes);

#ifdef __cplusplus
}
#endif
#endif /* INFR_HIP_H */
