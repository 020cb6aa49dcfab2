/*
 * dsx_moe.h -- C ABI of libdsx_moe.so: the deepstrix MoE feed-forward path on gfx950.
 *
 * What a host engine binds instead of launching the reference's per-arch code
 * objects.  Every entry point mirrors one launch wrapper / dispatch function of
 * the reference (cited per function, paths relative to the reference tree) and
 * keeps its argument order and meaning; the library owns grid/block selection.
 *
 * Conventions
 *   - all pointers are DEVICE pointers owned by the caller unless stated;
 *   - `stream` is a hipStream_t passed as void*; nothing synchronizes, allocates
 *     or reads back, so every call may sit inside a HIP graph capture
 *     (crates/v4flash-kernels/src/het/dispatch.rs:11-13,622-626);
 *   - return value: 0 = success, > 0 = the hipError_t of the failed launch,
 *     < 0 = argument validation error (DSX_ERR_*), raised BEFORE anything is
 *     launched (crates/v4flash-kernels/src/mxfp4.rs:416-424);
 *     dsx_last_error() returns the thread's last message;
 *   - an empty problem (0 tokens / 0 work items) is success
 *     (crates/v4flash-kernels/src/mxfp4.rs:422-424).
 *
 * Weight layouts are the engine's, unchanged:
 *   MXFP4  rows of 136-byte super-blocks: [8 x 16 B nibbles][8 B E8M0 scales],
 *          256 elements each; experts contiguous, stride = bytes-per-expert
 *          (crates/v4flash-kernels/src/mxfp4_tables.rs:10-36)
 *   Q8_0   rows of [blocks x f16 d][blocks x 32 i8]
 *          (crates/v4flash-kernels/src/weights.rs:225-240)
 * Activations: Q8_K blocks, 292 B per 256 elements
 *          (crates/v4flash-kernels/kernels/q8_k_quantize.hip:9-21).
 */
#ifndef DSX_MOE_H
#define DSX_MOE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DSX_ABI_VERSION 1

/* ggml type ids, as carried by the reference's GgufType
 * (crates/v4flash-core/src/gguf.rs:569-592). */
#define DSX_FMT_Q8_0 8
#define DSX_FMT_MXFP4 39
/* No counterpart in the reference: the same MXFP4 matrix with the bytes of every 16-row tile in
 * another order, made in place by dsx_mxfp4_rows_to_planar.  A tile (16 rows, 16 * cols / 256 * 136
 * bytes, where the engine keeps those rows) holds the rows' 128-byte nibble blocks first, row-major
 * -- each one whole cache line when the matrix is 128-byte aligned -- and then the 8-byte scale
 * groups as [super-block][row in tile].  Same size, same arithmetic, bit-identical results; the
 * grouped GEMMs of dsx_moe_layer_forward fetch such a matrix with about a third of the memory
 * requests (10 % faster at 4096 tokens, 25 % at 96 to 512, where they only stream weights).  Taken by dsx_moe_layer_create (every MXFP4 tensor of a
 * layer in the same form), dsx_dense_ffn and the four dsx_moe_* expert products. */
#define DSX_FMT_MXFP4_PLANAR 1039

#define DSX_ROUTER_SQRT_SOFTPLUS 0
#define DSX_ROUTER_SIGMOID 1
#define DSX_ROUTER_SOFTMAX 2

#define DSX_OK 0
#define DSX_ERR_INVALID_ARG (-1) /* null pointer, zero/oversized dimension */
#define DSX_ERR_SHAPE (-2)       /* divisibility / alignment contract broken */
#define DSX_ERR_UNSUPPORTED (-3) /* format or size this build has no kernel for */
#define DSX_ERR_DEVICE (-4)      /* current device is not gfx950 */

#define DSX_Q8K_BLOCK_BYTES 292
#define DSX_MXFP4_SUPER_BYTES 136
#define DSX_MAX_EXPERTS 512 /* crates/v4flash-kernels/build.rs:93-97 (ROUTER_MAX_EXPERTS) */
#define DSX_MAX_USED 16     /* crates/v4flash-kernels/kernels/laguna_ops.hip:20 */

typedef void *dsx_stream_t;

int dsx_abi_version(void);
const char *dsx_last_error(void);
/* Checks that the current device is gfx950, raises the kernels' LDS limits on it and resolves
 * the device's copy of the built-in scratch array; call once per device, with that device
 * current, before any other entry point (they refuse to run otherwise: doing this lazily would
 * put API calls inside a caller's stream capture). */
int dsx_init(void);

/* ---- router ---------------------------------------------------------------
 * RouterTopk::launch_batched_ex (crates/v4flash-kernels/src/router_topk.rs:245-364;
 * kernels router_topk_par.hip:66-238) and laguna_router_topk_batched
 * (kernels/laguna_ops.hip:395-451).  selected[b,n_used] i32, weights[b,n_used] f32,
 * logits[b,n_expert] f32, bias[n_expert] f32 or NULL.  mode = DSX_ROUTER_*.
 * n_group <= 1 disables group-limited routing; otherwise the n_expert/n_group
 * wide groups are ranked by the sum of their two largest biased scores and only
 * the best topk_group groups stay eligible. */
int dsx_router_topk(dsx_stream_t stream, int32_t *selected, float *weights, const float *logits,
                    const float *bias, uint32_t n_expert, uint32_t n_used, float scale, float eps,
                    uint32_t b, uint32_t mode, uint32_t n_group, uint32_t topk_group);

/* hash_router_select (crates/v4flash-kernels/src/routing.rs:21-44; call sites
 * het/forward_layer.rs:2253, het/forward_prefill.rs:9167): the picks of token t are row
 * token_ids[t] of tid2eid[vocab, n_used]; weights[t,i] = sqrt(softplus(logits[t, pick])) /
 * max(sum over the picks, eps) * scale.  The reference runs this on the host with n_used 6,
 * eps 6.103515625e-5, scale 1.5 after reading the logits back; here everything stays on the
 * device and feeds dsx_moe_layer_forward's selected_in / weights_in.  A token id outside
 * [0, vocab) or an expert id outside [0, n_expert) gives an empty slot (-1, weight 0). */
int dsx_router_hash_select(dsx_stream_t stream, int32_t *selected, float *weights,
                           const float *logits, const int32_t *tid2eid, const int32_t *token_ids,
                           uint32_t n_expert, uint32_t n_used, uint32_t vocab, float scale,
                           float eps, uint32_t b);

/* f32 router matvec: logits[t,e] = sum_k router_w[e,k] * x[t,k]
 * (crates/v4flash-kernels/kernels/laguna_ops.hip:57-60;
 * crates/v4flash-kernels/src/het/forward_prefill.rs:8974-9015). */
int dsx_router_logits(dsx_stream_t stream, float *logits, const float *router_w, const float *x,
                      uint32_t n_expert, uint32_t hidden, uint32_t n_tokens);
/* The same with the router weights in f16, as the engine keeps ffn_gate_inp
 * (F16Matvec::matvec_batched_router, crates/v4flash-kernels/src/f16.rs:37-45; call site
 * crates/v4flash-kernels/src/het/forward_prefill.rs:9008-9016): f32 products and sums. */
int dsx_router_logits_f16(dsx_stream_t stream, float *logits, const uint16_t *router_w,
                          const float *x, uint32_t n_expert, uint32_t hidden, uint32_t n_tokens);

/* ---- activation quantizers ------------------------------------------------
 * Q8KQuantize::launch (crates/v4flash-kernels/src/q8_k.rs:33-104). */
int dsx_q8k_quantize(dsx_stream_t stream, uint8_t *out, const float *x, uint32_t n_blocks);
/* Q8_0 input quantizer (crates/v4flash-kernels/kernels/q8_0_matvec.hip:150-177). */
int dsx_q8_0_quantize(dsx_stream_t stream, int8_t *xq, float *xscale, const float *x,
                      uint32_t blocks);
/* Same quantizer, one activation row per token as the expert entry points take it for
 * a Q8_0 matrix: out[rows] rows of (k + k/8) bytes = [k int8][k/32 f32 scales]. */
int dsx_q8_0_quantize_rows(dsx_stream_t stream, uint8_t *out, const float *x, uint32_t rows,
                           uint32_t k);

/* ---- decode (one token) ---------------------------------------------------
 * dispatch::moe_gate_up_batch (crates/v4flash-kernels/src/het/dispatch.rs:26-66):
 * mid[slot,row] = swiglu(gate_e[row].xq, up_e[row].xq; clamp) * ew[slot],
 * e = selected[slot]; mid is [n_used, n_rows] f32; xq is one token's Q8_K row of
 * n_blocks super-blocks. */
int dsx_moe_gate_up_batch(dsx_stream_t stream, int dtype, float *mid, const uint8_t *gate,
                          const uint8_t *up, const uint8_t *xq, const float *ew,
                          const int32_t *selected, uint64_t gbpe, uint64_t ubpe, uint32_t n_used,
                          float clamp, uint32_t n_rows, uint32_t n_blocks);
/* dispatch::moe_down_batched (crates/v4flash-kernels/src/het/dispatch.rs:121-150):
 * out[row] = sum_slot down_e[row] . midq[slot]; midq slot-major Q8_K with
 * xq_slot_stride bytes between slots. */
int dsx_moe_down_batched(dsx_stream_t stream, int dtype, float *out, const uint8_t *down,
                         const uint8_t *xq, const int32_t *selected, uint64_t dbpe,
                         uint32_t xq_slot_stride, uint32_t n_used, uint32_t n_rows,
                         uint32_t n_blocks_in);

/* ---- by-expert (many tokens) ----------------------------------------------
 * MoeGroupBuilder::launch + launch_work_items
 * (crates/v4flash-kernels/src/moe_group_builder.rs:72-130).  One call builds
 * group_count[n_expert], the exclusive prefix sum group_offset[n_expert+1],
 * expert_members[b*n_used] = (token << 16) | slot in ascending (token, slot)
 * order per expert, work_items = (expert << 16) | start in ascending order and
 * n_work_items[1].  Unlike the reference's atomic builder the order is
 * deterministic and the member table is compacted (no max_per_expert).
 * selected entries outside [0, n_expert) are skipped.  b, n_used, n_expert <
 * 65536; chunk in [1, 64] (the reference executor uses 32,
 * crates/v4flash-kernels/src/het/remote_experts.rs:77). */
int dsx_moe_group_build(dsx_stream_t stream, int32_t *group_count, int32_t *group_offset,
                        int32_t *expert_members, int32_t *work_items, int32_t *n_work_items,
                        const int32_t *selected, uint32_t b, uint32_t n_used, uint32_t n_expert,
                        uint32_t chunk);
/* dispatch::moe_gate_up_chunked_rows (crates/v4flash-kernels/src/het/dispatch.rs:534-570):
 * mid[b, n_used, n_rows]; xq is [b, n_blocks*292]; ew is [b, n_used].
 * max_work_items bounds the grid (dispatch::moe_wi_upper_bound, :450-454); the
 * device-side count is read by the kernel.  chunk (1..64) is the one the work items
 * were built with; an item wider than the columns one workgroup stages is served by
 * several workgroups. */
int dsx_moe_gate_up_chunked_rows(dsx_stream_t stream, int dtype, float *mid, const uint8_t *gate,
                                 const uint8_t *up, const uint8_t *xq, const float *ew,
                                 const int32_t *group_count, const int32_t *group_offset,
                                 const int32_t *expert_members, const int32_t *work_items,
                                 const int32_t *n_work_items, uint32_t max_work_items,
                                 uint64_t gbpe, uint64_t ubpe, uint32_t n_used, uint32_t chunk,
                                 float clamp, uint32_t n_rows, uint32_t n_blocks);
/* dispatch::moe_down_mxfp4 (crates/v4flash-kernels/src/het/dispatch.rs:580-620):
 * partials[(t*n_used+slot)*n_rows + row] = down_e[row] . midq[t,slot];
 * midq is [b*n_used] rows of xq_slot_stride bytes. */
int dsx_moe_down_by_expert(dsx_stream_t stream, int dtype, float *partials, const uint8_t *down,
                           const uint8_t *xq, const int32_t *group_count,
                           const int32_t *group_offset, const int32_t *expert_members,
                           const int32_t *work_items, const int32_t *n_work_items,
                           uint32_t max_work_items, uint64_t dbpe, uint32_t xq_slot_stride,
                           uint32_t n_used, uint32_t chunk, uint32_t n_rows,
                           uint32_t n_blocks_in);
/* The het-split variants (dispatch::moe_gate_up_batch_hetsplit, moe_down_batched_hetsplit,
 * MoeGroupBuilder::launch_hetsplit, launch_reduce_partials_hetsplit;
 * crates/v4flash-kernels/src/het/dispatch.rs:68-119,152-185,
 * kernels/mxfp4_pair_matvec.hip:231-284, kernels/q2_k_accumulate_matvec_par.hip:731-766)
 * share one ownership rule: remap[e] >= 0 is the dense slot of a resident expert on the
 * mode-1 side, -(slot + 1) the packed slot of a cold one; mode 1 takes a token's first `cap`
 * resident picks in slot order, mode 0 everything else.  This entry point applies the rule
 * once: selected_side[b, n_used] = the index this side's weight buffer is addressed with, or
 * -1 where the slot is the other side's (or empty).  Passed as `selected` to
 * dsx_moe_gate_up_batch / dsx_moe_down_batched / dsx_moe_group_build /
 * dsx_moe_reduce_partials / dsx_moe_layer_forward (selected_in), it makes each of them its
 * het-split variant: slots not owned are zero-filled or skipped, so the two sides' results
 * add up to the unsplit one. */
int dsx_moe_hetsplit_select(dsx_stream_t stream, int32_t *selected_side, const int32_t *selected,
                            const int32_t *remap, uint32_t mode, uint32_t cap, uint32_t n_used,
                            uint32_t n_expert, uint32_t b);
/* Q2KAccumulateMatvec::launch_reduce_partials (crates/v4flash-kernels/src/q2_k.rs:454-500;
 * kernels/q2_k_accumulate_matvec_par.hip:714-730): out[t,row] = sum over slots, in
 * slot order.  selected (nullable): slots with selected < 0 are skipped, so the
 * caller does not have to zero rows no pick wrote. */
int dsx_moe_reduce_partials(dsx_stream_t stream, float *out, const float *partials,
                            const int32_t *selected, uint32_t n_used, uint32_t n_rows, uint32_t b);

/* ---- dense SwiGLU expert (the shared expert) -------------------------------
 * issue_shared_expert (crates/v4flash-kernels/src/het/forward_layer.rs:3234-;
 * forward_prefill.rs:3649-3830): out[t,:] (+)= down . Q(swiglu(gate.Q(x), up.Q(x))).
 * x is f32 [b, hidden]; scratch must hold dsx_dense_ffn_scratch_bytes(). */
size_t dsx_dense_ffn_scratch_bytes(uint32_t b, uint32_t hidden, uint32_t inter);
int dsx_dense_ffn(dsx_stream_t stream, int gate_fmt, int up_fmt, int down_fmt, float *out,
                  const uint8_t *gate, const uint8_t *up, const uint8_t *down, const float *x,
                  uint32_t b, uint32_t hidden, uint32_t inter, float clamp, int accumulate,
                  void *scratch);

/* ---- element-wise ----------------------------------------------------------
 * VecAddInplace::launch (crates/v4flash-kernels/src/ffn.rs:135-153). */
int dsx_vec_add_inplace(dsx_stream_t stream, float *out, const float *rhs, uint64_t n);

/* ---- hyper-connection combine behind the FFN ----------------------------------
 * HcPost::launch / launch_batched / launch_from_split* (kernels
 * crates/v4flash-kernels/kernels/hc_post.hip:15-34, 40-64, 66-98, 100-141; call site
 * crates/v4flash-kernels/src/het/forward_layer.rs:3126-3133, right behind the vec_add that adds
 * the shared expert):
 *   out_hc[t, dst, d] = block[t, d] * post[t, dst]
 *                       + sum_src comb[t, dst + src * n_hc] * residual_hc[t, src, d]
 * in f32, src ascending.  post / comb of token t start post_stride / comb_stride floats behind
 * those of token t - 1: separate arrays ([b, n_hc], [b, n_hc, n_hc]: strides n_hc, n_hc * n_hc)
 * and the engine's packed "split" rows (post = split + n_w, comb = split + n_w + n_hc, both
 * strides n_w + n_hc + n_hc * n_hc) are the same descriptor.  out_hc may be residual_hc itself
 * (every element's inputs are read before its outputs are written).  n_hc <= 8. */
typedef struct dsx_hc_post_desc {
    float *out_hc;             /* [b, n_hc, n_embd] */
    const float *residual_hc;  /* [b, n_hc, n_embd] */
    const float *post;         /* n_hc per token */
    const float *comb;         /* n_hc * n_hc per token, addressed [dst + src * n_hc] */
    uint32_t n_hc, post_stride, comb_stride;
} dsx_hc_post_desc;
/* block[t, d] = block_out[t, d] (+ add1[t, d] (+ add2[t, d])): with both addends the block value
 * of hc_post_from_split_batched_add2, (block_out + add1) + add2; add1 / add2 may be NULL (add2
 * only with add1).  block_out is not written. */
int dsx_hc_post(dsx_stream_t stream, const dsx_hc_post_desc *desc, const float *block_out,
                const float *add1, const float *add2, uint32_t n_embd, uint32_t b);
/* RmsNorm batched (crates/v4flash-kernels/src/rms_norm.rs; kernels/rms_norm.hip:52-). */
int dsx_rms_norm(dsx_stream_t stream, float *out, const float *x, const float *weight,
                 uint32_t n, float eps, uint32_t rows);
/* SwiGluKernel::launch_clamped (crates/v4flash-kernels/src/ffn.rs:36-75). */
int dsx_swiglu_clamp_weighted(dsx_stream_t stream, float *mid, const float *gate, const float *up,
                              const float *expert_w, float clamp, uint32_t ff, uint32_t n_experts);

/* ---- weight pipeline ---------------------------------------------------------
 * Mxfp4Repack (crates/v4flash-kernels/src/mxfp4_repack.rs; kernels/mxfp4_repack.hip:35-65):
 * HF packed[out, nb*16] + scale[out, nb] -> v2 rows dst[out, nb*17]. nb % 8 == 0. */
int dsx_mxfp4_repack_hf_to_v2(dsx_stream_t stream, uint8_t *dst, const uint8_t *packed,
                              const uint8_t *scale, uint32_t out, uint32_t nb);
/* No counterpart in the reference: n_matrices MXFP4 matrices of n_rows x cols elements, `stride`
 * bytes apart (at least n_rows * cols / 256 * 136), rewritten in place from the engine's rows
 * into the planar form (DSX_FMT_MXFP4_PLANAR) and back.  n_rows % 16 == 0, cols % 256 == 0
 * (at most 16384), 8-byte alignment; no scratch (a 16-row tile is permuted in LDS).  Meant to
 * run once after the weights are loaded. */
int dsx_mxfp4_rows_to_planar(dsx_stream_t stream, uint8_t *w, uint32_t n_rows, uint32_t cols,
                             uint32_t n_matrices, uint64_t stride);
int dsx_mxfp4_planar_to_rows(dsx_stream_t stream, uint8_t *w, uint32_t n_rows, uint32_t cols,
                             uint32_t n_matrices, uint64_t stride);
/* HfV41Source::read_q8 (crates/v4flash-core/src/hf_v41.rs:728-805): a checkpoint matrix
 * src[out_rows, in_cols] -- f32, bf16, or fp8-e4m3 codes with an E8M0 scale grid
 * scale[scale_rows, scale_cols] that tiles the matrix exactly (scale is ignored for f32 and
 * bf16) -- quantized to Q8_0 with quantize_q8_0_block (hf_v41.rs:125-137).  split_rows = 0
 * writes ggml blocks [f16 d][32 i8] as read_q8 does; split_rows = 1 writes the engine rows
 * [blocks x f16 d][blocks x 32 i8] that repack_q8_0 makes of them, in one pass.  An fp8
 * source without scales, or a grid that does not divide the matrix, is refused. */
#define DSX_SRC_F32 0u
#define DSX_SRC_BF16 1u
#define DSX_SRC_F8E4M3 2u
int dsx_q8_0_weights_from_hf(dsx_stream_t stream, uint8_t *dst, const void *src,
                             const uint8_t *scale, uint32_t src_dtype, uint32_t out_rows,
                             uint32_t in_cols, uint32_t scale_rows, uint32_t scale_cols,
                             uint32_t split_rows);
/* repack_q8_0 (crates/v4flash-kernels/src/weights.rs:225-240): ggml Q8_0 blocks of a row-major
 * matrix -> engine rows.  dst and src may not overlap. */
int dsx_q8_0_repack_rows(dsx_stream_t stream, uint8_t *dst, const uint8_t *src, uint32_t num_rows,
                         uint32_t blocks_per_row);
/* Dequantize engine rows to f32 (checking aid; crates/v4flash-core/src/kquants.rs:105-111 for
 * Q8_0, crates/v4flash-kernels/src/mxfp4_tables.rs:38-45 for MXFP4). */
int dsx_dequant_rows(dsx_stream_t stream, int dtype, float *y, const uint8_t *rows,
                     uint32_t n_rows, uint32_t cols);

/* ---- the whole layer ---------------------------------------------------------
 * Modelled on MoeExecutor::run (crates/v4flash-kernels/src/het/remote_experts.rs:7432-7443)
 * plus the router in front and the shared expert + combine behind it
 * (forward_prefill.rs:9095-9118, 12227-12232).  The descriptor only records
 * pointers and dimensions; no weight is copied. */
typedef struct {
    uint32_t hidden, inter, n_expert, n_used;
    int gate_fmt, up_fmt, down_fmt;
    const uint8_t *gate, *up, *down; /* [n_expert] experts each */
    uint64_t gate_bpe, up_bpe, down_bpe;
    float clamp;
    /* router */
    uint32_t router_mode, n_group, topk_group;
    float route_scale, route_eps;
    const float *bias; /* [n_expert] or NULL */
    /* shared expert, sh_inter == 0 for none */
    uint32_t sh_inter;
    int sh_gate_fmt, sh_up_fmt, sh_down_fmt;
    const uint8_t *sh_gate, *sh_up, *sh_down;
    float sh_clamp;
} dsx_moe_layer_desc;

typedef struct dsx_moe_layer dsx_moe_layer;

int dsx_moe_layer_create(const dsx_moe_layer_desc *desc, dsx_moe_layer **out);
void dsx_moe_layer_destroy(dsx_moe_layer *layer);
/* No counterpart in the reference: rewrites every MXFP4 tensor the layer was created with -- the
 * caller's weight buffers -- in place into the planar form (DSX_FMT_MXFP4_PLANAR above), or back
 * into the engine's rows, and switches the layer over (its default thresholds included: a planar
 * layer leaves the decode path at 12 tokens and starts with the 16-column GEMM tile).  A layer
 * without MXFP4 tensors, or one already in the form asked for, is left as it is.  Shapes are
 * checked before the first byte moves; MXFP4 tensors whose byte ranges overlap are refused.
 * The rewrite is enqueued on `stream` like a kernel launch, while the layer switches over on the
 * host at once: a forward on ANOTHER stream must first be ordered behind `stream` (event or
 * synchronization), or it reads tensors that are still being rewritten.  Thresholds the caller set
 * with dsx_moe_layer_set_tuning are kept.  If the rewrite of one tensor fails, the ones already
 * rewritten are turned back; should that fail too, the layer refuses every later forward
 * (DSX_ERR_UNSUPPORTED).  Nothing else may use the buffers in the other form afterwards (two layers
 * over the same buffers must both be switched, the second one by creating it with the new format
 * ids). */
int dsx_moe_layer_weights_to_planar(dsx_moe_layer *layer, dsx_stream_t stream);
int dsx_moe_layer_weights_to_rows(dsx_moe_layer *layer, dsx_stream_t stream);
/* Measurement aid with no counterpart in the reference: hipEvent_t handles (or NULL) that
 * dsx_moe_layer_forward records on its stream right before and right after the gate/up
 * launch and after the down launch, so a harness can time the dominant kernel in place. */
int dsx_moe_layer_set_profile_events(dsx_moe_layer *layer, void *gate_up_begin, void *gate_up_end,
                                     void *down_end);
/* Tuning knobs with no counterpart in the reference; 0 keeps the current value.  The defaults follow
 * from the layer's shape: which path a token count takes depends on the picks an expert receives,
 * T * n_used / n_expert (in brackets: the DeepSeek-V3 shape, 256 experts, top-8).
 * by_expert_chunk (1..16): token columns per work item of the small-batch by-expert path.
 * gemm_min_tokens (default for an all-MXFP4 layer: 3.5 picks per expert [112 tokens], 7 where
 * n_expert * inter / 256 < 512; MXFP4 gate/up with a Q8_0 down matrix 2 [64], 4 for
 * matrices under 4 M elements; all-Q8_0 layers 1.5; on planar weights right behind the decode path
 * [17]): from this many tokens
 * on, a layer with MXFP4 gate/up runs the grouped-GEMM path (128 token columns per work item,
 * shared expert as an extra group; a Q8_0 down matrix takes the int8 grouped GEMM) and an all-Q8_0
 * layer the int8 grouped GEMMs; an all-MXFP4 layer whose GEMMs use the narrow tile (below)
 * switches at 11/16 of it.
 * decode_max_tokens (default: 0.45 picks per expert -- 0.85 where inter <= 1024 -- and at most 16 [14];
 * 0.375 on planar weights [11]):
 * up to this many tokens, an all-MXFP4 layer runs the decode path (dsx_moe_layer_set_decode: every
 * token on its own picks, no grouping by expert; the one-launch form serves at most 16 tokens,
 * beyond that the decode kernels run once per stage).
 * gemm_narrow_members (default 1 = never; 14 on planar weights): while the picks per expert average
 * less than this, the all-MXFP4 grouped GEMMs use 16 token columns per work item and two
 * workgroups per CU. */
int dsx_moe_layer_set_tuning(dsx_moe_layer *layer, uint32_t by_expert_chunk, uint32_t gemm_min_tokens,
                             uint32_t decode_max_tokens, uint32_t gemm_narrow_members);
/* The current values: out[0] by_expert_chunk, [1] gemm_min_tokens, [2] the same for layers whose
 * GEMMs are int8 (all-Q8_0), [3] decode_max_tokens, [4] gemm_narrow_members, [5] the token count
 * from which the one-launch decode path pairs tokens that name one expert (0: never). */
int dsx_moe_layer_get_tuning(const dsx_moe_layer *layer, uint32_t out[6]);
/* Decode path of an all-MXFP4 layer (up to decode_max_tokens tokens); no counterpart in the
 * reference.  fused: 1 = gate/up, mid quantization, down and the slot-order sum in ONE launch
 * whose workgroups hand results to each other through device memory (the default); from an eighth
 * of a pick per expert on (DeepSeek-V3 shape: 4 tokens), the tokens of a step that name one expert are paired and the expert is streamed
 * once per pair (the reference's drafter groups few picks by distinct expert likewise,
 * crates/v4flash-kernels/kernels/mxfp4_pair_matvec.hip:621-782); results are bitwise the same
 * with and without pairing.  3 = the same launch, never pairing; 4 = the same launch, pairing
 * from 2 tokens on (for steps whose tokens mostly name the same experts, such as the
 * verification of consecutive draft tokens); 2 = one launch per stage; 0 keeps the current
 * value.  spin_limit (0 keeps): bound, in polling rounds of about half a microsecond, of every
 * wait one workgroup does for another; values above 2^20 are taken as 2^20, so that every wait
 * stays bounded. */
int dsx_moe_layer_set_decode(dsx_moe_layer *layer, uint32_t fused, uint32_t spin_limit);
/* Measurement aid with no counterpart in the reference: a device buffer of n_items x 4 uint64
 * that the one-launch decode path fills with clock readings (constant 100 MHz counter) per
 * work item -- start, operands staged / weights requested, wait over, end; items in grid order:
 * gate/up tiles, the relay, down blocks.  Ignored while n_items is smaller than the grid;
 * NULL turns it off. */
int dsx_moe_layer_set_trace(dsx_moe_layer *layer, uint64_t *trace, size_t n_items);
/* Status word of the last dsx_moe_layer_forward / dsx_moe_block_forward that used `workspace`
 * (NULL: the built-in scratch of dsx_moe_layer_forward_noalloc on the current device), copied
 * to *host_out with a synchronous hipMemcpy: call it after synchronizing the stream, never
 * under capture.  0 = every in-kernel hand-off completed; DSX_STATUS_* otherwise, and the
 * output of that forward is then not to be used.  The reference has no such word because its
 * kernels never wait for each other inside a launch. */
#define DSX_STATUS_OK 0u
#define DSX_STATUS_MID_WAIT_EXPIRED 1u  /* a down workgroup gave up waiting for mid values */
#define DSX_STATUS_MIDQ_WAIT_EXPIRED 2u /* the fused mid quantization gave up waiting for a tile */
#define DSX_STATUS_PARTIAL_WAIT_EXPIRED 3u /* the slot-order sum gave up waiting for a partial row */
int dsx_moe_layer_status(const dsx_moe_layer *layer, const void *workspace, uint32_t *host_out);
/* The device address of that status word (no copy, no synchronization: safe under capture), for a
 * caller that wants to test it on the device or copy it with a node of its own graph.  No
 * counterpart in the reference. */
int dsx_moe_layer_status_ptr(const dsx_moe_layer *layer, void *workspace, uint32_t **device_word);
/* Bytes of caller-provided device scratch for up to max_tokens tokens. */
size_t dsx_moe_layer_workspace_bytes(const dsx_moe_layer *layer, uint32_t max_tokens);
/* out[t,:] = sum_slot expert(x[t]) + shared(x[t]);  x f32 [n_tokens, hidden],
 * logits f32 [n_tokens, n_expert].  selected_out / weights_out (nullable) receive
 * the routing.  If selected_in is non-NULL the router is skipped and
 * selected_in / weights_in are used (pinned routing). */
int dsx_moe_layer_forward(dsx_moe_layer *layer, dsx_stream_t stream, float *out, const float *x,
                          const float *logits, uint32_t n_tokens, void *workspace,
                          size_t workspace_bytes, int32_t *selected_out, float *weights_out,
                          const int32_t *selected_in, const float *weights_in);

/* dsx_moe_layer_forward whose result goes straight through the hyper-connection combine
 * (dsx_hc_post above with block = the layer's output, n_embd = hidden) instead of to an output
 * buffer: the kernel that sums a token's slots and the shared expert applies it while it stores
 * -- the reference's vec_add + hc_post pair (crates/v4flash-kernels/src/het/forward_layer.rs:3126-3133)
 * without the launches and without the round trip of the layer output through memory. */
int dsx_moe_layer_forward_hc(dsx_moe_layer *layer, dsx_stream_t stream, const dsx_hc_post_desc *hc,
                             const float *x, const float *logits, uint32_t n_tokens, void *workspace,
                             size_t workspace_bytes, int32_t *selected_out, float *weights_out,
                             const int32_t *selected_in, const float *weights_in);
/* dsx_moe_layer_forward without a workspace argument.  No counterpart in the reference: it is
 * for callers that cannot allocate device memory at all (code under HIP graph capture that owns
 * no buffers, tight serving loops, harnesses that forbid hipMalloc).  The scratch is a fixed
 * DSX_NOALLOC_SCRATCH_BYTES array inside the library's code object; each device holds its own
 * copy from the moment the library is loaded until the process ends, and dsx_init() resolves its
 * address.  Calls whose dsx_moe_layer_workspace_bytes(layer, n_tokens) exceeds the array are
 * refused with DSX_ERR_UNSUPPORTED (at the DeepSeek-V3 shape, 7168 x 2048 with 256 experts and top-8: up to 15 tokens).  Every call on a
 * device shares that device's array: calls that overlap in time on one device (two streams, two
 * layers) race; calls ordered on one stream do not.  Results are those of
 * dsx_moe_layer_forward. */
#define DSX_NOALLOC_SCRATCH_BYTES (8u << 20)
int dsx_moe_layer_forward_noalloc(dsx_moe_layer *layer, dsx_stream_t stream, float *out,
                                  const float *x, const float *logits, uint32_t n_tokens,
                                  int32_t *selected_out, float *weights_out,
                                  const int32_t *selected_in, const float *weights_in);

/* One pre-norm residual MoE block (the unit of BASELINE's chained-layer decode):
 *   h[t,:] += layer(RMSNorm(h[t,:]; norm_w, eps)),  router logits = router_w . RMSNorm(h[t,:])
 * RMSNorm as crates/v4flash-kernels/kernels/rms_norm.hip:12-50, the f32 router matvec as
 * crates/v4flash-kernels/src/het/forward_prefill.rs:8974-9015, the residual add as
 * kernels/vec_add.hip:6-13; sequencing of crates/v4flash-kernels/src/het/forward_layer.rs:424-466.
 * h is f32 [n_tokens, hidden], updated in place; router_w f32 [n_expert, hidden];
 * norm_w f32 [hidden].  Same workspace as dsx_moe_layer_forward. */
int dsx_moe_block_forward(dsx_moe_layer *layer, dsx_stream_t stream, float *h, const float *norm_w,
                          float eps, const float *router_w, uint32_t n_tokens, void *workspace,
                          size_t workspace_bytes);
/* The same block with router_w in f16 [n_expert, hidden] (see dsx_router_logits_f16). */
int dsx_moe_block_forward_f16(dsx_moe_layer *layer, dsx_stream_t stream, float *h,
                              const float *norm_w, float eps, const uint16_t *router_w,
                              uint32_t n_tokens, void *workspace, size_t workspace_bytes);

#ifdef __cplusplus
}
#endif
#endif
