/*
 * dsx_oracle.h -- CPU restatement of the deepstrix MoE feed-forward arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or
 * calls this code: it is the checker the GPU path is compared against and the
 * CPU baseline a benchmark times next to the GPU.  Every function cites the
 * reference file (relative to the reference tree) whose arithmetic it follows.
 *
 * Parity status of each group of functions (what pins it):
 *   formats (f16/bf16/e8m0/e4m3, MXFP4, Q8_0, Q8_K) ... pinned by the
 *       reference's golden vectors and known-answer tests
 *   mxfp4 x q8_k dot, q8_0 dot, swiglu ................ pinned by f64 closed
 *       forms and brute force on small inputs
 *   sqrt-softplus / sigmoid routers ................... pinned by f64 ranking
 *   softmax router, group-limited top-k ............... not in the reference;
 *       pinned by brute-force enumeration and numpy primitives
 *   hc_post (hyper-connection combine) ................ pinned by the f64 closed
 *       form written out with numpy, an asymmetric mixing matrix (a transposed
 *       index fails), and the cases that reduce to a copy / a scale
 *   whole-layer composition ........................... pinned by invariants
 *       (token permutation, pick-set split, per-token == batched); end-to-end
 *       agreement with the external ds4 activation dumps is "parity unpinned"
 *       because those dumps are not available.
 */
#ifndef DSX_ORACLE_H
#define DSX_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Weight format ids = ggml type ids (crates/v4flash-core/src/gguf.rs:569-592). */
#define DSX_REF_FMT_Q8_0 8
#define DSX_REF_FMT_MXFP4 39

/* Router scoring modes. */
#define DSX_REF_ROUTER_SQRT_SOFTPLUS 0 /* kernels/router_topk.hip:32-36,70-74 */
#define DSX_REF_ROUTER_SIGMOID 1       /* kernels/laguna_ops.hip:60-66 */
#define DSX_REF_ROUTER_SOFTMAX 2       /* textbook; not in the reference */

#define DSX_REF_Q8K_BLOCK_BYTES 292
#define DSX_REF_MXFP4_SUPER_BYTES 136

/* ---- scalar format conversions ------------------------------------------ */
float dsx_ref_f16_to_f32(uint16_t bits);   /* core/src/kquants.rs:23-47 */
uint16_t dsx_ref_f32_to_f16(float f);      /* core/src/kquants.rs:51-85 */
float dsx_ref_bf16_to_f32(uint16_t bits);  /* core/src/hf_v41.rs:93-95 */
uint16_t dsx_ref_f32_to_bf16(float f);     /* round-to-nearest-even (input generation) */
float dsx_ref_e8m0_to_f32(uint8_t e);      /* core/src/hf_v41.rs:99-105  : 2^(e-127) */
float dsx_ref_e8m0_half_to_f32(uint8_t e); /* kernels/src/mxfp4_tables.rs:38-45 : 2^(e-128) */
float dsx_ref_e4m3_to_f32(uint8_t b);      /* core/src/hf_v41.rs:109-118 */

/* ---- MXFP4 ---------------------------------------------------------------- */
/* ggml block_mxfp4 = [e][qs16]; n elements, n % 32 == 0 (ds4 patch 0010:393-404). */
void dsx_ref_mxfp4_dequant_ggml(const uint8_t *blocks, float *y, size_t n);
/* engine v2 super-block rows (kernels/src/mxfp4_tables.rs:10-36). cols % 256 == 0. */
void dsx_ref_mxfp4_dequant_v2(const uint8_t *rows, float *y, size_t n_rows, size_t cols);
/* HF [out, in/2] nibbles + [out, in/32] e8m0 -> v2 rows (core/src/hf_v41.rs:1208-1232). */
void dsx_ref_mxfp4_repack_hf_to_v2(const uint8_t *packed, const uint8_t *scale,
                                   uint8_t *dst, size_t out, size_t nb);
void dsx_ref_mxfp4_unpack_v2_to_hf(const uint8_t *src, uint8_t *packed, uint8_t *scale,
                                   size_t out, size_t nb);
/* f32 -> E2M1 x E8M0 per 32 (kernels/kernels/indexer_qat.hip:60-73,
 * kernels/tests/indexer_pipeline.rs:575-636), written as v2 rows. */
void dsx_ref_mxfp4_quantize_v2(const float *x, uint8_t *dst, size_t n_rows, size_t cols);

/* ---- Q8_0 ----------------------------------------------------------------- */
void dsx_ref_q8_0_quantize_block(const float *x32, uint8_t *out34); /* core/src/hf_v41.rs:125-137 */
/* f32 [n_rows, cols] -> engine rows [blocks x f16 d][blocks x 32 i8]
 * (quantize per block, then kernels/src/weights.rs:225-240). cols % 32 == 0. */
void dsx_ref_q8_0_quantize_rows(const float *x, uint8_t *dst, size_t n_rows, size_t cols);
void dsx_ref_q8_0_repack_rows(const uint8_t *ggml, uint8_t *dst, size_t n_rows, size_t blocks);
void dsx_ref_q8_0_dequant_rows(const uint8_t *rows, float *y, size_t n_rows, size_t cols);
/* activation: int8 + f32 scale per 32 (kernels/kernels/q8_0_matvec.hip:150-177). */
void dsx_ref_q8_0_quantize_act(const float *x, int8_t *xq, float *xscale, size_t blocks);
/* one row x one activation (kernels/kernels/q8_0_matvec.hip:64-104; 32 lane-strided
 * partials then the 16/8/4/2/1 shuffle-down tree). */
float dsx_ref_dot_q8_0(size_t blocks, const uint8_t *wrow, const int8_t *xq, const float *xscale);

/* ---- Q8_K ----------------------------------------------------------------- */
/* kernels/tests/q8_k_quantize.rs:37-102 (= kernels/kernels/q8_k_quantize.hip:23-90). */
void dsx_ref_q8k_quantize(const float *x, uint8_t *out, size_t n_blocks);
void dsx_ref_q8k_dequant(const uint8_t *blocks, float *y, size_t n_blocks);
/* kernels/src/mxfp4_tables.rs:49-74 */
float dsx_ref_dot_mxfp4_q8k(size_t n_super, const uint8_t *w, const uint8_t *y);

/* ---- element-wise --------------------------------------------------------- */
/* kernels/kernels/swiglu_clamp_weighted.hip:16-37 */
float dsx_ref_swiglu(float g, float u, float clamp, float ew);
/* kernels/kernels/rms_norm.hip:12-50 (256 f64 strided partials, f32 tree). */
void dsx_ref_rms_norm(float *out, const float *x, const float *weight, size_t n, float eps,
                      size_t rows);
/* kernels/kernels/hc_post.hip:15-34, 40-64, 66-98, 100-141: the hyper-connection combine behind
 * the FFN, out_hc[t, dst, d] = block[t, d] * post[t, dst] + sum_src comb[t, dst + src * n_hc] *
 * residual_hc[t, src, d] with block = block_out (+ add1 (+ add2)); add1 / add2 may be NULL. */
void dsx_ref_hc_post(float *out_hc, const float *block_out, const float *add1, const float *add2,
                     const float *residual_hc, const float *post, const float *comb, size_t n_embd,
                     size_t n_hc, size_t b, size_t post_stride, size_t comb_stride);

/* ---- router ---------------------------------------------------------------
 * selected[T,n_used] (int32), weights[T,n_used].  bias may be NULL.  n_group<=1
 * disables group limiting.  Returns 0, or -1 on bad arguments.
 * Tail (argmax passes, lowest index on ties, weights from unbiased p,
 * w = p / max(sum, eps) * scale): kernels/kernels/router_topk.hip:86-131,
 * kernels/kernels/laguna_ops.hip:70-108.  Group limiting: DeepSeek-V3 rule
 * (group score = sum of the two largest biased scores of the group, keep the
 * topk_group best groups, others masked to -inf). */
int dsx_ref_router_topk(int32_t *selected, float *weights, const float *logits,
                        const float *bias, int n_expert, int n_used, float scale, float eps,
                        int n_tokens, int mode, int n_group, int topk_group);
/* probs[T,E] and biased, group-masked scores[T,E] as the router sees them (for
 * near-tie classification in tests). */
int dsx_ref_router_scores(float *probs, float *scores, const float *logits, const float *bias,
                          int n_expert, int n_tokens, int mode, int n_group, int topk_group);
/* fp32 router matvec logits[t,e] = sum_k W[e,k] x[t,k], sequential in k
 * (kernels/kernels/laguna_ops.hip:57-60). */
void dsx_ref_router_logits(float *logits, const float *w, const float *x, int n_expert,
                           int hidden, int n_tokens);

/* ---- token -> expert inversion --------------------------------------------
 * Deterministic form of kernels/kernels/moe_group_builder.hip:32-51 and
 * moe_work_items_builder.hip:26-44: members of an expert in ascending
 * (token, slot) order, work items in ascending (expert, start) order.
 * offsets[n_expert+1] is the exclusive prefix sum of group_count.
 * members[i] = (token << 16) | slot.  work_items[i] = (expert << 16) | start,
 * start relative to the expert's first member.  Returns the work-item count. */
int dsx_ref_group_build(int32_t *group_count, int32_t *offsets, int32_t *members,
                        int32_t *work_items, const int32_t *selected, int n_tokens, int n_used,
                        int n_expert, int chunk);
/* kernels/src/het/dispatch.rs:450-454 */
uint32_t dsx_ref_wi_upper_bound(size_t members, uint32_t groups, uint32_t chunk, size_t cap);

/* ---- the layer ------------------------------------------------------------ */
typedef struct {
    int hidden;   /* model width (gate/up input, down output) */
    int inter;    /* routed expert intermediate width */
    int n_expert;
    int n_used;
    int gate_fmt, up_fmt, down_fmt; /* DSX_REF_FMT_* */
    const uint8_t *gate, *up, *down; /* [n_expert] experts, contiguous */
    uint64_t gate_bpe, up_bpe, down_bpe;
    float clamp; /* <= 1e-6 disables */
    /* shared expert; sh_inter == 0 means none */
    int sh_inter;
    int sh_gate_fmt, sh_up_fmt, sh_down_fmt;
    const uint8_t *sh_gate, *sh_up, *sh_down;
    float sh_clamp;
} dsx_ref_moe_cfg;

/* out[T,hidden] = sum_slot down_e . Q(swiglu(gate_e . Q(x), up_e . Q(x)) * w) + shared(x).
 * Order of operations: kernels/src/het/forward_layer.rs:456-466 (quantize, gate/up
 * with the expert weight applied before down, quantize mid, down), slot-order sum
 * kernels/kernels/q2_k_accumulate_matvec_par.hip:714-730, shared added last
 * kernels/kernels/vec_add.hip:6-13.  Activations are quantized to Q8_K in front
 * of an MXFP4 matrix and to per-32 Q8_0 in front of a Q8_0 matrix.
 * mid_out (nullable) receives mid[T,n_used,inter]; moe_out (nullable) the routed
 * sum before the shared expert; shared_out (nullable) the shared expert alone.
 * selected < 0 marks an empty slot.  n_threads <= 0 uses all cores. */
int dsx_ref_moe_forward(const dsx_ref_moe_cfg *cfg, const float *x, const int32_t *selected,
                        const float *weights, int n_tokens, float *out, float *mid_out,
                        float *moe_out, float *shared_out, int n_threads);

int dsx_ref_max_threads(void);

#ifdef __cplusplus
}
#endif
#endif
