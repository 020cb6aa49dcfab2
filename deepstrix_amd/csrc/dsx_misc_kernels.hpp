// dsx_misc_kernels.hpp -- router, activation quantizers, token->expert inversion,
// reductions and the small element-wise kernels of the MoE path (gfx950, wave64).
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "dsx_device.hpp"
#include "dsx_quant.hpp"

namespace dsx {

#define DSX_MAX_EXPERTS_K 512
#define DSX_MAX_USED_K 16

// ---------------------------------------------------------------------------------------
// Router.  One wave per token; lane l owns experts l, l+64, ...  (n_expert <= 512).
//   p      = sqrt(softplus(logit)) | sigmoid(logit) | softmax(logits)
//   score  = p + bias, then group-limited masking
//   k passes of arg-max over score (ties -> lowest index), winner masked to -inf
//   w_j    = p[sel_j] / max(sum_j p[sel_j], eps) * scale
// crates/v4flash-kernels/kernels/router_topk.hip:32-36,70-131,
// crates/v4flash-kernels/kernels/laguna_ops.hip:395-451.
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ float softplus_stable(float x) {
    if (x > 20.0f) return x;
    if (x < -20.0f) return expf(x);
    return log1pf(expf(x));
}

constexpr int kRouterThreads = 256;

// ---- one-wave router ----------------------------------------------------------------------
// With 64 C experts (C = 1, 2, 4, 8) one wave routes a token without LDS or barriers: lane l
// owns experts C l .. C l + C - 1, the arg-max of each of the k passes is a 64-bit key
// (score, ~index) reduced with DPP moves (wave_max_u64_dpp), the winner is cleared and the
// next pass follows.
// Same picks and weights as the workgroup-wide version below (ties -> lowest index, weights
// summed in pick order).
// Whether the one-wave router takes this shape (softmax keeps the workgroup-wide version).
__device__ __forceinline__ bool route_wave_ok(uint32_t n_expert, uint32_t mode, uint32_t n_group,
                                              uint32_t topk_group) {
    if (mode == 2u || n_expert % 64u != 0u) return false;
    const uint32_t c = n_expert / 64u;
    if (c != 1u && c != 2u && c != 4u && c != 8u) return false;
    if (n_group > 1u && topk_group < n_group) {
        if (n_expert % n_group != 0u) return false;
        const uint32_t gs = n_expert / n_group;
        if (gs % c != 0u) return false;
        const uint32_t lg = gs / c;  // lanes per group
        if ((lg & (lg - 1u)) != 0u) return false;
    }
    return true;
}

template <int C>
__device__ __forceinline__ void route_token_wave(int32_t *__restrict__ selected,
                                                 float *__restrict__ weights,
                                                 const float *__restrict__ lg,
                                                 const float *__restrict__ bias, uint32_t n_expert,
                                                 uint32_t n_used, float scale, float eps, uint32_t mode,
                                                 uint32_t n_group, uint32_t topk_group) {
    const uint32_t lane = threadIdx.x & 63u;
    float p[C], s[C];
#pragma unroll
    for (int i = 0; i < C; i++) p[i] = lg[lane * C + i];
#pragma unroll
    for (int i = 0; i < C; i++) {
        p[i] = (mode == 0u) ? sqrtf(softplus_stable(p[i])) : 1.0f / (1.0f + expf(-p[i]));
        s[i] = (bias != nullptr) ? p[i] + bias[lane * C + i] : p[i];
    }
    if (n_group > 1u && topk_group < n_group) {
        // group score = sum of the two largest biased scores of the group (lanes_per_group
        // consecutive lanes), groups ranked with ties to the lower index
        const uint32_t gs = n_expert / n_group, lanes_per_group = gs / C;
        float a = -INFINITY, b = -INFINITY;
#pragma unroll
        for (int i = 0; i < C; i++) {
            const float v = s[i];
            b = fmaxf(fminf(a, v), b);
            a = fmaxf(a, v);
        }
        // lanes 2^j apart exchange their pairs; up to 16 lanes per group with DPP moves (after
        // the steps before it every lane of a half holds the half's pair, so a mirror of 8 or
        // 16 lanes reaches the other half like an exchange would)
        auto merge = [&](float oa, float ob) {
            const float hi = fmaxf(a, oa), lo = fminf(a, oa);
            b = fmaxf(lo, fmaxf(b, ob));
            a = hi;
        };
        if (lanes_per_group > 1u) merge(dpp_mov_f32<0xb1>(a), dpp_mov_f32<0xb1>(b));    // quad_perm:[1,0,3,2]
        if (lanes_per_group > 2u) merge(dpp_mov_f32<0x4e>(a), dpp_mov_f32<0x4e>(b));    // quad_perm:[2,3,0,1]
        if (lanes_per_group > 4u) merge(dpp_mov_f32<0x141>(a), dpp_mov_f32<0x141>(b));  // row_half_mirror
        if (lanes_per_group > 8u) merge(dpp_mov_f32<0x140>(a), dpp_mov_f32<0x140>(b));  // row_mirror
        for (uint32_t off = 16; off < lanes_per_group; off <<= 1)
            merge(__shfl_xor(a, (int)off, 64), __shfl_xor(b, (int)off, 64));
        const float mine = (gs >= 2u) ? a + b : a;
        const uint32_t my_group = lane / lanes_per_group;
        uint32_t rank = 0;
        for (uint32_t g = 0; g < n_group; g++) {  // g * lanes_per_group is uniform
            const float o = __uint_as_float((uint32_t)__builtin_amdgcn_readlane(
                (int)__float_as_uint(mine), (int)(g * lanes_per_group)));
            rank += (o > mine || (o == mine && g < my_group)) ? 1u : 0u;
        }
        if (rank >= topk_group) {
#pragma unroll
            for (int i = 0; i < C; i++) s[i] = -INFINITY;
        }
    }
    uint64_t key[C];
#pragma unroll
    for (int i = 0; i < C; i++)
        key[i] = (s[i] > -INFINITY) ? (((uint64_t)f32_key(s[i]) << 32) | (uint64_t)(0xFFFFFFFFu - (lane * C + i)))
                                    : 0ull;  // a masked expert is never picked
    int my_sel = -1;
    float my_p = 0.0f;
    for (uint32_t j = 0; j < n_used; j++) {
        uint64_t best = key[0];
#pragma unroll
        for (int i = 1; i < C; i++) best = key[i] > best ? key[i] : best;
        const uint64_t top = wave_max_u64_dpp(best);  // uniform
        if (top == 0ull) break;                       // fewer eligible experts than picks
        const uint32_t e = 0xFFFFFFFFu - (uint32_t)top;
        float pw = 0.0f;
#pragma unroll
        for (int i = 0; i < C; i++) {
            if (key[i] == top) {  // only the winner's lane, only its winning value
                pw = p[i];
                key[i] = 0ull;
            }
        }
        pw = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(pw), (int)(e / C)));
        if (lane == j) {
            my_sel = (int)e;
            my_p = pw;
        }
    }
    float sum = 0.0f;
    for (uint32_t j = 0; j < n_used; j++)  // pick order, as the reference
        sum += __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(my_p), (int)j));
    if (sum < eps) sum = eps;
    if (lane < n_used) {
        selected[lane] = my_sel;
        weights[lane] = my_p / sum * scale;
    }
}

// One workgroup routes one token.  Thread t owns experts t and t + 256.  The top-k is read
// off each expert's rank (how many experts beat it: larger score, or equal score and lower
// index), which every thread counts on its own from 64-bit keys (score, ~index) in LDS.
__device__ __forceinline__ void route_token(int32_t *__restrict__ selected,
                                            float *__restrict__ weights,
                                            const float *__restrict__ lg,
                                            const float *__restrict__ bias, uint32_t n_expert,
                                            uint32_t n_used, float scale, float eps, uint32_t mode,
                                            uint32_t n_group, uint32_t topk_group) {
    __shared__ __attribute__((aligned(16))) uint64_t s_key[512];
    __shared__ float s_score[512];
    __shared__ float s_red[kRouterThreads / 64];
    __shared__ float s_gscore[64];
    __shared__ int s_keep[64];
    __shared__ float s_psel[DSX_MAX_USED_K];
    __shared__ int s_esel[DSX_MAX_USED_K];

    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u;
    if (route_wave_ok(n_expert, mode, n_group, topk_group)) {  // uniform over the workgroup
        if (wave == 0) {
            switch (n_expert / 64u) {
                case 1: route_token_wave<1>(selected, weights, lg, bias, n_expert, n_used, scale, eps, mode, n_group, topk_group); break;
                case 2: route_token_wave<2>(selected, weights, lg, bias, n_expert, n_used, scale, eps, mode, n_group, topk_group); break;
                case 4: route_token_wave<4>(selected, weights, lg, bias, n_expert, n_used, scale, eps, mode, n_group, topk_group); break;
                default: route_token_wave<8>(selected, weights, lg, bias, n_expert, n_used, scale, eps, mode, n_group, topk_group); break;
            }
        }
        return;
    }
    const uint32_t nj = (n_expert + kRouterThreads - 1) / kRouterThreads;  // 1 or 2
    float p[2], s[2];
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const uint32_t e = tid + kRouterThreads * j;
        p[j] = (e < n_expert) ? lg[e] : -INFINITY;
        mx = fmaxf(mx, p[j]);
    }
    if (mode == 2u) {  // softmax
        mx = wave_max_f32(mx);
        if (lane == 0) s_red[wave] = mx;
        __syncthreads();
        mx = fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
        __syncthreads();
        float sum = 0.0f;
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const uint32_t e = tid + kRouterThreads * j;
            p[j] = (e < n_expert) ? expf(p[j] - mx) : 0.0f;
            sum += p[j];
        }
        sum = wave_sum_f32(sum);
        if (lane == 0) s_red[wave] = sum;
        __syncthreads();
        sum = (s_red[0] + s_red[1]) + (s_red[2] + s_red[3]);
#pragma unroll
        for (int j = 0; j < 2; j++) p[j] = p[j] / sum;
    } else {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const uint32_t e = tid + kRouterThreads * j;
            if (e < n_expert)
                p[j] = (mode == 0u) ? sqrtf(softplus_stable(p[j])) : 1.0f / (1.0f + expf(-p[j]));
            else
                p[j] = 0.0f;
        }
    }
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const uint32_t e = tid + kRouterThreads * j;
        s[j] = (e < n_expert) ? ((bias != nullptr) ? p[j] + bias[e] : p[j]) : -INFINITY;
    }
    if (tid < n_used) {
        s_esel[tid] = -1;
        s_psel[tid] = 0.0f;
    }

    if (n_group > 1u && topk_group < n_group) {
        // group score = sum of the two largest biased scores of the group
        const uint32_t gs = n_expert / n_group;
        const bool butterfly = gs <= 64u && (gs & (gs - 1u)) == 0u;
        if (butterfly) {
            // groups are runs of gs consecutive lanes: top-2 by an xor butterfly
            for (uint32_t j = 0; j < nj; j++) {
                float a = s[j], b = -INFINITY;
                for (uint32_t off = 1; off < gs; off <<= 1) {
                    const float oa = __shfl_xor(a, (int)off, 64), ob = __shfl_xor(b, (int)off, 64);
                    const float hi = fmaxf(a, oa), lo = fminf(a, oa);
                    b = fmaxf(lo, fmaxf(b, ob));
                    a = hi;
                }
                const uint32_t e = tid + kRouterThreads * j;
                if (e < n_expert && (e % gs) == 0u) s_gscore[e / gs] = (gs >= 2u) ? a + b : a;
            }
        } else {
#pragma unroll
            for (int j = 0; j < 2; j++) s_score[tid + kRouterThreads * j] = s[j];
            __syncthreads();
            if (tid < n_group) {
                float a = -INFINITY, b = -INFINITY;
                for (uint32_t i = 0; i < gs; i++) {
                    const float v = s_score[tid * gs + i];
                    if (v > a) {
                        b = a;
                        a = v;
                    } else if (v > b) {
                        b = v;
                    }
                }
                s_gscore[tid] = (gs >= 2u) ? a + b : a;
            }
        }
        __syncthreads();
        if (tid < n_group) {
            const float mine = s_gscore[tid];
            uint32_t rank = 0;
            for (uint32_t g = 0; g < n_group; g++) {
                const float o = s_gscore[g];
                rank += (o > mine || (o == mine && g < tid)) ? 1u : 0u;
            }
            s_keep[tid] = rank < topk_group ? 1 : 0;
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const uint32_t e = tid + kRouterThreads * j;
            if (e < n_expert && !s_keep[e / gs]) s[j] = -INFINITY;
        }
    }

    uint64_t key[2];
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const uint32_t e = tid + kRouterThreads * j;
        key[j] = ((uint64_t)f32_key(s[j]) << 32) | (uint64_t)(0xFFFFFFFFu - e);
        s_key[e] = key[j];
    }
    __syncthreads();
    // rank = number of keys above mine (keys are distinct: they carry the index)
    uint32_t rank[2] = {0u, 0u};
    const uint32_t n4 = (n_expert + 3u) / 4u;  // s_key is padded with the keys of -inf
    if (nj == 1u) {
        uint32_t r0 = 0;
        for (uint32_t q = 0; q < n4; q++) {
            const ulonglong2 a = *(const ulonglong2 *)(s_key + 4u * q);
            const ulonglong2 b = *(const ulonglong2 *)(s_key + 4u * q + 2u);
            r0 += (a.x > key[0]) ? 1u : 0u;
            r0 += (a.y > key[0]) ? 1u : 0u;
            r0 += (b.x > key[0]) ? 1u : 0u;
            r0 += (b.y > key[0]) ? 1u : 0u;
        }
        rank[0] = r0;
    } else {
        uint32_t r0 = 0, r1 = 0;
        for (uint32_t q = 0; q < n4; q++) {
            const ulonglong2 a = *(const ulonglong2 *)(s_key + 4u * q);
            const ulonglong2 b = *(const ulonglong2 *)(s_key + 4u * q + 2u);
            r0 += (a.x > key[0]) ? 1u : 0u;
            r0 += (a.y > key[0]) ? 1u : 0u;
            r0 += (b.x > key[0]) ? 1u : 0u;
            r0 += (b.y > key[0]) ? 1u : 0u;
            r1 += (a.x > key[1]) ? 1u : 0u;
            r1 += (a.y > key[1]) ? 1u : 0u;
            r1 += (b.x > key[1]) ? 1u : 0u;
            r1 += (b.y > key[1]) ? 1u : 0u;
        }
        rank[0] = r0;
        rank[1] = r1;
    }
    for (uint32_t j = 0; j < nj; j++) {
        const uint32_t e = tid + kRouterThreads * j;
        // an expert masked to -inf is never picked (a scan with `>` from -inf skips it)
        if (e < n_expert && rank[j] < n_used && s[j] > -INFINITY) {
            s_esel[rank[j]] = (int)e;
            s_psel[rank[j]] = p[j];
        }
    }
    __syncthreads();
    if (tid < n_used) {
        float sum = 0.0f;
        for (uint32_t k = 0; k < n_used; k++) sum += s_psel[k];  // pick order, as the reference
        if (sum < eps) sum = eps;
        selected[tid] = s_esel[tid];
        weights[tid] = s_psel[tid] / sum * scale;
    }
}

__global__ __launch_bounds__(kRouterThreads) void k_router_topk(
    int32_t *__restrict__ selected, float *__restrict__ weights, const float *__restrict__ logits,
    const float *__restrict__ bias, uint32_t n_expert, uint32_t n_used, float scale, float eps,
    uint32_t mode, uint32_t n_group, uint32_t topk_group) {
    const uint32_t t = blockIdx.x;
    route_token(selected + (uint64_t)t * n_used, weights + (uint64_t)t * n_used,
                logits + (uint64_t)t * n_expert, bias, n_expert, n_used, scale, eps, mode, n_group,
                topk_group);
}

// Hash routing of the bootstrap layers: the picks of a token are row `token id` of
// tid2eid[vocab, n_used]; weights = sqrt(softplus(logit)) / max(sum, eps) * scale with the sum
// in slot order.  One thread per token (n_used <= 16).  An id out of range leaves an empty
// slot (-1, weight 0).  crates/v4flash-kernels/src/routing.rs:21-44.
__global__ __launch_bounds__(256) void k_router_hash_select(
    int32_t *__restrict__ selected, float *__restrict__ weights, const float *__restrict__ logits,
    const int32_t *__restrict__ tid2eid, const int32_t *__restrict__ token_ids, uint32_t n_expert,
    uint32_t n_used, uint32_t vocab, float scale, float eps, uint32_t n_tokens) {
    const uint32_t t = blockIdx.x * 256u + threadIdx.x;
    if (t >= n_tokens) return;
    const int tok = token_ids[t];
    const bool tok_ok = tok >= 0 && (uint32_t)tok < vocab;
    const float *lg = logits + (uint64_t)t * n_expert;
    float w[DSX_MAX_USED_K];
    float sum = 0.0f;
#pragma unroll
    for (uint32_t i = 0; i < DSX_MAX_USED_K; i++) {
        if (i < n_used) {
            int e = tok_ok ? tid2eid[(uint64_t)tok * n_used + i] : -1;
            if (e < 0 || (uint32_t)e >= n_expert) e = -1;
            selected[(uint64_t)t * n_used + i] = e;
            w[i] = (e >= 0) ? sqrtf(softplus_stable(lg[e])) : 0.0f;
            sum += w[i];
        }
    }
    if (sum < eps) sum = eps;
#pragma unroll
    for (uint32_t i = 0; i < DSX_MAX_USED_K; i++)
        if (i < n_used) weights[(uint64_t)t * n_used + i] = w[i] / sum * scale;
}

// Het-split ownership (the rule of the reference's *_hetsplit kernels,
// crates/v4flash-kernels/kernels/mxfp4_pair_matvec.hip:231-284,
// kernels/q2_k_accumulate_matvec_par.hip:731-766): remap[e] >= 0 is the dense slot of a
// resident expert on the mode-1 side, -(slot + 1) the packed slot of a cold one; mode 1 takes
// a token's first `cap` resident picks in slot order, mode 0 everything else.  out[b, s] is
// the index this side's weight buffer is addressed with, or -1 (not this side's, or empty):
// with it as `selected`, every entry point computes this side's share and zero-fills the rest.
__global__ __launch_bounds__(256) void k_hetsplit_select(int32_t *__restrict__ out,
                                                         const int32_t *__restrict__ selected,
                                                         const int32_t *__restrict__ remap,
                                                         uint32_t mode, uint32_t cap, uint32_t n_used,
                                                         uint32_t n_expert, uint32_t n_tokens) {
    const uint32_t b = blockIdx.x * 256u + threadIdx.x;
    if (b >= n_tokens) return;
    uint32_t rank = 0;
    for (uint32_t s = 0; s < n_used; s++) {
        const int e = selected[(uint64_t)b * n_used + s];
        int r = -1;
        if (e >= 0 && (uint32_t)e < n_expert) {
            const int dense = remap[e];
            const bool resident = dense >= 0;
            const bool dgpu_takes = resident && rank < cap;
            if (resident) rank++;
            if (mode == 1u) {
                if (dgpu_takes) r = dense;
            } else if (!dgpu_takes) {
                r = resident ? e : -dense - 1;
            }
        }
        out[(uint64_t)b * n_used + s] = r;
    }
}

// Front of the layer in one launch: workgroups [0, n_tokens) route one token each (skipped
// when routing is pinned), the rest quantize the activations into staged rows (one wave per
// 256-element block) and mark the mid buffer of the fused mid quantization as unwritten.
struct FrontParams {
    int32_t *selected;
    float *weights;
    const float *logits;
    const float *bias;
    uint8_t *xp;        // staged rows out, xp_row_bytes apart
    const float *x;     // [n_tokens, k]
    const int32_t *sel_in;  // pinned routing (route == 0): copied to `selected`, picks outside [0, n_expert) as -1
    uint32_t *fill;     // n_fill words to set to fill_value (may be null)
    uint32_t *fill2;    // a second region of n_fill2 words for the same value (may be null)
    uint32_t n_fill2;
    uint32_t *zero;     // n_zero words to clear: status word and hand-off counters (may be null)
    uint32_t n_zero;
    uint32_t n_expert, n_used;
    float scale, eps;
    uint32_t mode, n_group, topk_group;
    uint32_t n_tokens, n_sb, xp_row_bytes, n_fill, fill_value, route;
    uint32_t fp6;   // staged rows in the grouped GEMMs' format (FP6 planes, 384 bytes per super-block)
    uint8_t *xq8;   // also the tokens as Q8_0 activation rows ([k i8][k/32 f32]), or null
    uint32_t xq8_row_bytes;
};

__global__ __launch_bounds__(kRouterThreads) void k_layer_front(const FrontParams p) {
    const uint32_t n_route = p.route ? p.n_tokens : 0u;
    if (blockIdx.x < n_route) {
        const uint32_t t = blockIdx.x;
        route_token(p.selected + (uint64_t)t * p.n_used, p.weights + (uint64_t)t * p.n_used,
                    p.logits + (uint64_t)t * p.n_expert, p.bias, p.n_expert, p.n_used, p.scale,
                    p.eps, p.mode, p.n_group, p.topk_group);
        return;
    }
    const uint32_t qb = blockIdx.x - n_route;
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    // one wave per 256-element block, grid-stride (many tokens: a few thousand workgroups
    // instead of one per four blocks)
    const uint32_t n_q = gridDim.x - n_route;
    // (x rows are contiguous: block blk starts at element 256 blk); the next block's elements are
    // requested before this one is quantized
    const uint32_t n_blk = p.n_tokens * p.n_sb, step = n_q * 4u;
    uint32_t blk = qb * 4u + (tid >> 6);
    float4 v = {0.f, 0.f, 0.f, 0.f};
    if (blk < n_blk) v = *(const float4 *)(p.x + (uint64_t)blk * 256u + lane * 4u);
    for (; blk < n_blk; blk += step) {
        float4 nxt = {0.f, 0.f, 0.f, 0.f};
        if (blk + step < n_blk) nxt = *(const float4 *)(p.x + (uint64_t)(blk + step) * 256u + lane * 4u);
        const uint32_t t = blk / p.n_sb, b = blk - t * p.n_sb;
        uint8_t *row = p.xp + (uint64_t)t * p.xp_row_bytes;
        if (p.fp6)
            quantize_block_to_staged6(v, lane, row + (size_t)b * kStaged6Bytes,
                                      (float *)(row + (size_t)p.n_sb * kStaged6Bytes) + b);
        else
            quantize_block_to_staged(v, lane, row + (size_t)b * 512u, (float *)(row + (size_t)p.n_sb * 512u) + b);
        if (p.xq8 != nullptr) {
            // the same elements as a Q8_0 row, for a shared expert kept in Q8_0
            uint32_t pk;
            float d8;
            q8_0_quantize_lane4(v, pk, d8);
            uint8_t *r8 = p.xq8 + (uint64_t)t * p.xq8_row_bytes;
            *(uint32_t *)(r8 + (size_t)b * 256u + lane * 4u) = pk;
            if ((lane & 7u) == 0u) *(float *)(r8 + (size_t)p.n_sb * 256u + ((size_t)b * 8u + (lane >> 3)) * 4u) = d8;
        }
        v = nxt;
    }
    if (p.sel_in != nullptr)
        for (uint32_t i = qb * kRouterThreads + tid; i < p.n_tokens * p.n_used; i += n_q * kRouterThreads) {
            const int32_t e = p.sel_in[i];
            p.selected[i] = (e < 0 || (uint32_t)e >= p.n_expert) ? -1 : e;
        }
    // the fill goes last: stores count like loads, so in front of the loop its stores would
    // have to drain before the first block's elements count as arrived
    // (n_fill is a multiple of 4 and the buffer 16-byte aligned)
    for (uint32_t i = (qb * kRouterThreads + tid) * 4u; i < p.n_fill; i += n_q * kRouterThreads * 4u)
        *(uint4 *)(p.fill + i) = make_uint4(p.fill_value, p.fill_value, p.fill_value, p.fill_value);
    for (uint32_t i = (qb * kRouterThreads + tid) * 4u; i < p.n_fill2; i += n_q * kRouterThreads * 4u)
        *(uint4 *)(p.fill2 + i) = make_uint4(p.fill_value, p.fill_value, p.fill_value, p.fill_value);
    for (uint32_t i = qb * kRouterThreads + tid; i < p.n_zero; i += n_q * kRouterThreads) p.zero[i] = 0u;
}

__global__ void k_zero_words(uint32_t *p, uint32_t n) {
    for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) p[i] = 0u;
}

// Pinned routing as the layer uses it: picks outside [0, n_expert) become empty slots (-1).
__global__ __launch_bounds__(256) void k_sanitize_picks(int32_t *__restrict__ out,
                                                        const int32_t *__restrict__ in, uint32_t n,
                                                        uint32_t n_expert) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= n) return;
    const int32_t e = in[i];
    out[i] = (e < 0 || (uint32_t)e >= n_expert) ? -1 : e;
}

// Rows of f32 -> staged rows (the mid activations of the by-expert path).
__global__ __launch_bounds__(256) void k_quantize_staged(uint8_t *__restrict__ out,
                                                         const float *__restrict__ x,
                                                         uint32_t n_rows, uint32_t n_sb,
                                                         uint32_t row_bytes) {
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t blk = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (blk >= n_rows * n_sb) return;
    const uint32_t t = blk / n_sb, b = blk - t * n_sb;
    const float4 v = *(const float4 *)(x + (uint64_t)blk * 256u + lane * 4u);
    uint8_t *row = out + (uint64_t)t * row_bytes;
    quantize_block_to_staged(v, lane, row + (size_t)b * 512u, (float *)(row + (size_t)n_sb * 512u) + b);
}

// ---------------------------------------------------------------------------------------
// Q8_K quantizer: one wave per 256-element block, 4 consecutive elements per lane.
// crates/v4flash-kernels/kernels/q8_k_quantize.hip:23-90
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_q8k_quantize(uint8_t *__restrict__ out,
                                                      const float *__restrict__ x,
                                                      uint32_t n_blocks) {
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t b = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (b >= n_blocks) return;
    const float4 v = *(const float4 *)(x + (uint64_t)b * 256u + lane * 4u);
    const Q8kQuant r = q8k_quantize_lane(v, lane);
    uint8_t *blk = out + (uint64_t)b * kQ8kBytes;
    const uint32_t packed = (uint32_t)(r.q[0] & 0xFF) | ((uint32_t)(r.q[1] & 0xFF) << 8) |
                            ((uint32_t)(r.q[2] & 0xFF) << 16) | ((uint32_t)(r.q[3] & 0xFF) << 24);
    *(uint32_t *)(blk + 4u + lane * 4u) = packed;
    int s = r.q[0] + r.q[1] + r.q[2] + r.q[3];
    s += __shfl_xor(s, 1, 64);
    s += __shfl_xor(s, 2, 64);
    if ((lane & 3u) == 0u) *(int16_t *)(blk + 260u + (lane >> 2) * 2u) = (int16_t)s;
    if (lane == 0) *(float *)blk = r.d;
}

// Q8_0 activation quantizer: 8 lanes per 32-element block, 4 elements per lane.
// crates/v4flash-kernels/kernels/q8_0_matvec.hip:150-177
__global__ __launch_bounds__(256) void k_q8_0_quantize(int8_t *__restrict__ xq,
                                                       float *__restrict__ xscale,
                                                       const float *__restrict__ x,
                                                       uint32_t blocks) {
    const uint32_t gid = blockIdx.x * 256u + threadIdx.x;
    const uint32_t b = gid >> 3, sub = gid & 7u;
    const bool live = b < blocks;
    float4 v = {0.f, 0.f, 0.f, 0.f};
    if (live) v = *(const float4 *)(x + (uint64_t)b * 32u + sub * 4u);
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
    amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
    amax = fmaxf(amax, __shfl_xor(amax, 4, 64));
    if (!live) return;
    const float d = amax / 127.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    const float xs[4] = {v.x, v.y, v.z, v.w};
    uint32_t packed = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        int q = (int)rintf(xs[i] * id);
        q = q > 127 ? 127 : q;
        q = q < -128 ? -128 : q;
        packed |= (uint32_t)(q & 0xFF) << (8 * i);
    }
    *(uint32_t *)(xq + (uint64_t)b * 32u + sub * 4u) = packed;
    if (sub == 0) xscale[b] = d;
}

// ---------------------------------------------------------------------------------------
// Token -> expert inversion: histogram, exclusive prefix sum, stable scatter, work items.
// Members of an expert are in ascending (token, slot) order and work items in ascending
// (expert, start) order, so the result is the same on every run.
// Replaces crates/v4flash-kernels/kernels/moe_group_builder.hip:32-51 and
// moe_work_items_builder.hip:26-44 (atomic order, dense [n_expert x max] table).
// ---------------------------------------------------------------------------------------
constexpr int kGbThreads = 1024;

// Exclusive prefix sums of count[0..n) into off[0..n] and of the groups' work items,
// ceil(count / chunk), into wi_off[0..n] (entry n: the totals), by the first wave of the workgroup:
// a lane adds up its share of consecutive groups, the lanes scan their sums with shuffles, and
// every lane writes its groups' offsets (one thread walking 257 groups through LDS took 8 us).
// The caller puts a barrier on either side.
__device__ __forceinline__ void gb_scan(const int *s_count, int *s_off, int *s_wi_off, uint32_t n,
                                        uint32_t chunk, uint32_t tid) {
    if (tid >= 64u) return;
    const uint32_t per = (n + 63u) / 64u;
    const uint32_t b = min(n, tid * per), e = min(n, b + per);
    int sa = 0, sw = 0;
    for (uint32_t i = b; i < e; i++) {
        sa += s_count[i];
        sw += (s_count[i] + (int)chunk - 1) / (int)chunk;
    }
    int ia = sa, iw = sw;   // inclusive scan over the lanes
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const int ta = __shfl_up(ia, o, 64), tw = __shfl_up(iw, o, 64);
        if ((int)tid >= o) {
            ia += ta;
            iw += tw;
        }
    }
    int ea = ia - sa, ew = iw - sw;
    for (uint32_t i = b; i < e; i++) {
        s_off[i] = ea;
        s_wi_off[i] = ew;
        ea += s_count[i];
        ew += (s_count[i] + (int)chunk - 1) / (int)chunk;
    }
    if (tid == 63u) {
        s_off[n] = ia;
        s_wi_off[n] = iw;
    }
}


// ---------------------------------------------------------------------------------------
// The tables in one launch of n_groups + 1 workgroups, with an optional extra group of index
// n_expert that every token belongs to (slot n_used): the dense expert riding along.  Workgroup n_groups makes the histogram, the prefix sums and the work items; workgroup
// e < n_groups places the members of group e.  A placing workgroup reads every pick anyway, so it
// counts the picks of lower groups itself (its group's offset) and waits for nobody.
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ void group_count_body(
    int32_t *__restrict__ group_count, int32_t *__restrict__ group_offset,
    int32_t *__restrict__ work_items, int32_t *__restrict__ n_work_items,
    const int32_t *__restrict__ selected, uint32_t b, uint32_t n_used, uint32_t n_expert,
    uint32_t chunk, uint32_t extra) {
    __shared__ int s_count[DSX_MAX_EXPERTS_K + 1];
    __shared__ int s_off[DSX_MAX_EXPERTS_K + 2];
    __shared__ int s_wi_off[DSX_MAX_EXPERTS_K + 2];
    const uint32_t tid = threadIdx.x;
    const uint32_t total = b * n_used;
    const uint32_t n_groups = n_expert + (extra ? 1u : 0u);
    for (uint32_t e = tid; e < n_groups; e += kGbThreads) s_count[e] = 0;
    __syncthreads();
    auto count = [&](int e) {
        if (e >= 0 && (uint32_t)e < n_expert) atomicAdd(&s_count[e], 1);
    };
    const uint32_t n4 = (((uintptr_t)selected & 15u) == 0u) ? total / 4u : 0u;  // 16-byte loads
    for (uint32_t i = tid; i < n4; i += kGbThreads) {
        const int4 q = *(const int4 *)(selected + 4u * i);
        count(q.x);
        count(q.y);
        count(q.z);
        count(q.w);
    }
    for (uint32_t i = 4u * n4 + tid; i < total; i += kGbThreads) count(selected[i]);
    if (extra && tid == 0) s_count[n_expert] = (int)b;
    __syncthreads();
    gb_scan(s_count, s_off, s_wi_off, n_groups, chunk, tid);
    __syncthreads();
    if (tid == 0) *n_work_items = s_wi_off[n_groups];
    for (uint32_t e = tid; e < n_groups; e += kGbThreads) {
        group_count[e] = s_count[e];
        group_offset[e] = s_off[e];
    }
    if (tid == 0) group_offset[n_groups] = s_off[n_groups];
    // work items: every thread walks the groups whose items it owns
    const uint32_t n_wi = (uint32_t)s_wi_off[n_groups];
    for (uint32_t i = tid; i < n_wi; i += kGbThreads) {
        // largest e with s_wi_off[e] <= i (groups without items share an offset with the next)
        uint32_t lo = 0, hi = n_groups;
        while (hi - lo > 1u) {
            const uint32_t mid = (lo + hi) >> 1;
            if ((uint32_t)s_wi_off[mid] <= i) lo = mid; else hi = mid;
        }
        work_items[i] = (int)((lo << 16) | ((i - (uint32_t)s_wi_off[lo]) * chunk));
    }
}

__global__ __launch_bounds__(kGbThreads) void k_group_tables(
    int32_t *__restrict__ group_count, int32_t *__restrict__ group_offset,
    int32_t *__restrict__ members, int32_t *__restrict__ work_items,
    int32_t *__restrict__ n_work_items, const int32_t *__restrict__ selected, uint32_t b,
    uint32_t n_used, uint32_t n_expert, uint32_t chunk, uint32_t extra) {
    constexpr uint32_t kWaves = kGbThreads / 64;
    __shared__ uint32_t s_mine[kWaves], s_below[kWaves];
    const uint32_t n_groups = n_expert + (extra ? 1u : 0u);
    if (blockIdx.x >= n_groups) {
        group_count_body(group_count, group_offset, work_items, n_work_items, selected, b, n_used,
                         n_expert, chunk, extra);
        return;
    }
    const uint32_t e = blockIdx.x, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u;
    // picks that go in front of this group's members: the valid ones of lower groups (for the extra
    // group e == n_expert: every valid pick)
    // each wave owns a sixteenth of the picks (rounded to 256): count, then place; a lane looks at
    // four consecutive picks per step (one 16-byte load when `selected` is aligned for it)
    const uint32_t total = b * n_used;
    const bool vec = ((uintptr_t)selected & 15u) == 0u;
    const uint32_t share = ((total + 256u * kWaves - 1u) / (256u * kWaves)) * 256u;
    const uint32_t i_begin = min(total, wave * share), i_end = min(total, i_begin + share);
    auto load4 = [&](uint32_t i0) -> int4 {  // picks i0 + 4 lane + j, -1 past the end
        const uint32_t i = i0 + lane * 4u;
        int4 q = {-1, -1, -1, -1};
        if (vec && i + 4u <= i_end) {
            q = *(const int4 *)(selected + i);
        } else {
            if (i < i_end) q.x = selected[i];
            if (i + 1u < i_end) q.y = selected[i + 1u];
            if (i + 2u < i_end) q.z = selected[i + 2u];
            if (i + 3u < i_end) q.w = selected[i + 3u];
        }
        return q;
    };
    auto n_lanes = [](bool c) { return (uint32_t)__popcll(__ballot(c)); };
    // the next step's picks are requested before this step's are counted
    uint32_t mine = 0, below = 0;
    int4 cur = load4(i_begin);
    for (uint32_t i0 = i_begin; i0 < i_end; i0 += 256u) {
        const int4 nxt = load4(i0 + 256u);
        mine += n_lanes(cur.x == (int)e) + n_lanes(cur.y == (int)e) + n_lanes(cur.z == (int)e) +
                n_lanes(cur.w == (int)e);
        // (a negative pick is a large unsigned number: never below)
        below += n_lanes((uint32_t)cur.x < e) + n_lanes((uint32_t)cur.y < e) +
                 n_lanes((uint32_t)cur.z < e) + n_lanes((uint32_t)cur.w < e);
        cur = nxt;
    }
    if (lane == 0) {
        s_mine[wave] = mine;
        s_below[wave] = below;
    }
    __syncthreads();
    uint32_t pos = 0;
    for (uint32_t w = 0; w < kWaves; w++) pos += s_below[w] + (w < wave ? s_mine[w] : 0u);
    if (e >= n_expert) {  // the extra group: every token, slot n_used, behind every valid pick
        uint32_t base = 0;
        for (uint32_t w = 0; w < kWaves; w++) base += s_below[w];
        for (uint32_t t = tid; t < b; t += kGbThreads) members[base + t] = (int)((t << 16) | n_used);
        return;
    }
    if (mine == 0u) return;
    const uint64_t lower = (1ull << lane) - 1ull;
    cur = load4(i_begin);
    for (uint32_t i0 = i_begin; i0 < i_end; i0 += 256u) {
        const int4 nxt = load4(i0 + 256u);
        const bool h[4] = {cur.x == (int)e, cur.y == (int)e, cur.z == (int)e, cur.w == (int)e};
        uint32_t before = 0, all = 0;
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
            const uint64_t mask = __ballot(h[jj]);
            before += (uint32_t)__popcll(mask & lower);
            all += (uint32_t)__popcll(mask);
        }
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
            if (h[jj]) {  // ascending pick index: lower lanes first, then the lane's own earlier picks
                const uint32_t i = i0 + lane * 4u + jj;
                const uint32_t t = i / n_used, slot = i - t * n_used;
                members[pos + before] = (int)((t << 16) | slot);
                before++;
            }
        }
        pos += all;
        cur = nxt;
    }
}

// ---------------------------------------------------------------------------------------
// out[t, row] = sum over slots of partials[(t * n_used + s) * n_rows + row], in slot order.
// crates/v4flash-kernels/kernels/q2_k_accumulate_matvec_par.hip:714-730
// `selected` (nullable): slots with a negative pick are skipped.
// `add` (nullable): added last (the shared expert, crates/v4flash-kernels/kernels/vec_add.hip:6-13).
// ---------------------------------------------------------------------------------------
// `hc` (n_hc != 0): the sum is not stored but goes through the hyper-connection combine.
__global__ __launch_bounds__(256) void k_reduce_partials(float *__restrict__ out,
                                                         const float *__restrict__ partials,
                                                         const int32_t *__restrict__ selected,
                                                         const float *__restrict__ add,
                                                         uint32_t n_used, uint32_t n_rows,
                                                         uint32_t b, const HcPost hc) {
    const uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x;  // float4 index
    const uint64_t per_row = n_rows / 4u;
    if (i >= (uint64_t)b * per_row) return;
    const uint64_t t = i / per_row, c = i - t * per_row;
    float4 acc = {0.f, 0.f, 0.f, 0.f};
    for (uint32_t s = 0; s < n_used; s++) {
        if (selected != nullptr && selected[t * n_used + s] < 0) continue;
        const float4 v = *(const float4 *)(partials + ((t * n_used + s) * n_rows) + c * 4u);
        acc.x += v.x;
        acc.y += v.y;
        acc.z += v.z;
        acc.w += v.w;
    }
    if (add != nullptr) {
        const float4 v = *(const float4 *)(add + t * n_rows + c * 4u);
        acc.x += v.x;
        acc.y += v.y;
        acc.z += v.z;
        acc.w += v.w;
    }
    if (hc.n_hc) hc_post_store4(hc, t, (uint32_t)c * 4u, n_rows, acc);
    else *(float4 *)(out + t * n_rows + c * 4u) = acc;
}

// crates/v4flash-kernels/kernels/vec_add.hip:6-13
__global__ __launch_bounds__(256) void k_vec_add_inplace(float *__restrict__ out,
                                                         const float *__restrict__ rhs,
                                                         uint64_t n) {
    const uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    if (i < n) out[i] += rhs[i];
}

// out = (a + b) + c  (b, c may be null; out may alias any of them): the routed experts' rows, a
// shared expert computed beside them and the residual, in the order the reference adds them
// (crates/v4flash-kernels/src/het/forward_prefill.rs:12227-12232; with both addends the block
// value of hc_post_from_split_batched_add2, crates/v4flash-kernels/kernels/hc_post.hip:100-141).
// `hc` (n_hc != 0): the sum goes through the hyper-connection combine instead of to `out`.
// n_embd is a multiple of 4.
__global__ __launch_bounds__(256) void k_add_rows(float *out, const float *a, const float *b,
                                                  const float *c, uint32_t n_embd, uint32_t n_tokens,
                                                  const HcPost hc) {
    const uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    const uint64_t per_row = n_embd / 4u;
    if (i >= (uint64_t)n_tokens * per_row) return;
    float4 s = ((const float4 *)a)[i];
    if (b) {
        const float4 vb = ((const float4 *)b)[i];
        s.x += vb.x; s.y += vb.y; s.z += vb.z; s.w += vb.w;
    }
    if (c) {
        const float4 vc = ((const float4 *)c)[i];
        s.x += vc.x; s.y += vc.y; s.z += vc.z; s.w += vc.w;
    }
    if (hc.n_hc) {
        const uint64_t t = i / per_row;
        hc_post_store4(hc, t, (uint32_t)(i - t * per_row) * 4u, n_embd, s);
    } else {
        ((float4 *)out)[i] = s;
    }
}

// crates/v4flash-kernels/kernels/swiglu_clamp_weighted.hip:16-37
__global__ __launch_bounds__(256) void k_swiglu_clamp_weighted(float *__restrict__ mid,
                                                               const float *__restrict__ gate,
                                                               const float *__restrict__ up,
                                                               const float *__restrict__ expert_w,
                                                               float clamp, uint32_t ff) {
    const uint32_t r = blockIdx.x * 256u + threadIdx.x;
    if (r >= ff) return;
    const uint32_t e = blockIdx.y;
    const uint64_t idx = (uint64_t)e * ff + r;
    mid[idx] = swiglu_clamp(gate[idx], up[idx], clamp, expert_w[e]);
}

// RMS norm, one workgroup per row: 256 strided f64 partial sums, rounded to f32 and added up in
// the order of the reference's tree (element t takes t + 128, then t + 64, ... t + 1:
// crates/v4flash-kernels/kernels/rms_norm.hip:12-50), then the scale.  The order is the parity
// contract; how it is carried out is not: the 256 values cross the four waves once through LDS
// (strides 128 and 64 are lane-wise sums of whole waves) and the last six steps are shifts
// inside wave 0, so there are two barriers instead of eight.
__global__ __launch_bounds__(256) void k_rms_norm(float *__restrict__ out,
                                                  const float *__restrict__ x,
                                                  const float *__restrict__ weight, uint32_t n,
                                                  float eps) {
    __shared__ float s_part[4][64];
    __shared__ float s_total;
    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u;
    const float *xr = x + (uint64_t)blockIdx.x * n;
    float *orow = out + (uint64_t)blockIdx.x * n;
    double partial = 0.0;
    for (uint32_t i = tid; i < n; i += 256u) {
        const float v = xr[i];
        partial += (double)v * (double)v;
    }
    s_part[wave][lane] = (float)partial;
    __syncthreads();
    if (wave == 0u) {
        const float a = s_part[0][lane] + s_part[2][lane];   // stride 128, elements 0..63
        const float b = s_part[1][lane] + s_part[3][lane];   // stride 128, elements 64..127
        float c = a + b;                                      // stride 64
#pragma unroll
        for (int stride = 32; stride > 0; stride >>= 1) c += __shfl_down(c, stride, 64);
        if (lane == 0u) s_total = c;
    }
    __syncthreads();
    const float mean_sq = s_total / (float)n;
    const float scale = 1.0f / sqrtf(mean_sq + eps);
    for (uint32_t i = tid; i < n; i += 256u) orow[i] = xr[i] * scale * weight[i];
}

// Router logits logits[t, e] = sum_k W[e, k] * x[t, k] in f32, one workgroup per expert, up
// to kRlTokens tokens per pass (crates/v4flash-kernels/kernels/laguna_ops.hip:57-60; the
// engine's f32 router matvec, crates/v4flash-kernels/src/het/forward_prefill.rs:8974-9015).
// NORM: x is first RMS-normalized (same arithmetic as k_rms_norm) and the workgroups with
// e < n_tokens also write the normalized row e to xn, so one launch replaces the norm, the
// router matvec and the copy between them.
constexpr int kRlTokens = 4;

// Sum over the 256 threads of a workgroup; every thread gets the result.  `red` holds 4 floats.
__device__ __forceinline__ float block_sum_256(float v, float *red, uint32_t tid) {
    v = wave_sum_f32(v);
    __syncthreads();  // `red` may still be read from a previous call
    if ((tid & 63u) == 0u) red[tid >> 6] = v;
    __syncthreads();
    return red[0] + red[1] + red[2] + red[3];
}

// Sums of N values over the 256 threads of a workgroup in one pass; every thread gets them.
// `red` holds 4 * N floats.
template <int N>
__device__ __forceinline__ void block_sum_256_multi(float (&v)[N], float *red, uint32_t tid) {
#pragma unroll
    for (int k = 0; k < N; k++) v[k] = wave_sum_f32(v[k]);
    __syncthreads();  // `red` may still be read from a previous call
    if ((tid & 63u) == 0u) {
#pragma unroll
        for (int k = 0; k < N; k++) red[(tid >> 6) * N + k] = v[k];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < N; k++) v[k] = (red[k] + red[N + k]) + (red[2 * N + k] + red[3 * N + k]);
}

// One workgroup per expert, up to kRlTokens tokens per pass.  With NORM the row is normalized
// on the fly: logit = (sum_i w[i] * (x[i] * norm_w[i])) / rms(x) -- the sum of squares and the
// dot product are accumulated in the same sweep and reduced together, so the kernel has one
// round of loads on its critical path; every workgroup then writes its slice of the tokens'
// normalized rows.
// Router weights are f32 or f16 (the engine keeps ffn_gate_inp in f16,
// crates/v4flash-kernels/src/f16.rs:37-45); products and sums are f32 either way.
__device__ __forceinline__ float4 router_w4(const float *p) { return *(const float4 *)p; }
__device__ __forceinline__ float4 router_w4(const __half *p) {
    const uint2 v = *(const uint2 *)p;
    const __half2 a = *(const __half2 *)&v.x, b = *(const __half2 *)&v.y;
    const float2 fa = __half22float2(a), fb = __half22float2(b);
    return make_float4(fa.x, fa.y, fb.x, fb.y);
}
__device__ __forceinline__ float router_w1(const float *p) { return *p; }
__device__ __forceinline__ float router_w1(const __half *p) { return __half2float(*p); }

template <bool NORM, typename WT>
__global__ __launch_bounds__(256) void k_router_logits(float *__restrict__ logits,
                                                       float *__restrict__ xn,
                                                       const WT *__restrict__ w,
                                                       const float *__restrict__ x,
                                                       const float *__restrict__ norm_w, float eps,
                                                       uint32_t n_expert, uint32_t hidden,
                                                       uint32_t n_tokens) {
    __shared__ float s_red[4 * 2 * kRlTokens];
    const uint32_t tid = threadIdx.x;
    const uint32_t e = blockIdx.x;
    const WT *wr = w + (uint64_t)e * hidden;
    // vector loads need aligned rows; otherwise everything goes one element at a time
    const uint32_t n4 = (hidden % 4u == 0u) ? hidden / 4u : 0u;
    for (uint32_t t0 = 0; t0 < n_tokens; t0 += kRlTokens) {
        const uint32_t nt = min((uint32_t)kRlTokens, n_tokens - t0);
        float acc[kRlTokens];
        double sq[kRlTokens];  // sum of squares with f64 partial sums, like k_rms_norm
#pragma unroll
        for (int j = 0; j < kRlTokens; j++) {
            acc[j] = 0.0f;
            sq[j] = 0.0;
        }
#pragma unroll 4
        for (uint32_t i = tid; i < n4; i += 256u) {
            const float4 wv = router_w4(wr + 4u * i);
            float4 nw = {1.f, 1.f, 1.f, 1.f};
            if (NORM) nw = *(const float4 *)(norm_w + 4u * i);
#pragma unroll
            for (int j = 0; j < kRlTokens; j++) {
                if ((uint32_t)j < nt) {
                    float4 xv = *(const float4 *)(x + (uint64_t)(t0 + j) * hidden + 4u * i);
                    if (NORM) {
                        sq[j] += (double)xv.x * xv.x + (double)xv.y * xv.y + (double)xv.z * xv.z +
                                 (double)xv.w * xv.w;
                        xv.x *= nw.x;
                        xv.y *= nw.y;
                        xv.z *= nw.z;
                        xv.w *= nw.w;
                    }
                    acc[j] = fmaf(wv.x, xv.x, acc[j]);
                    acc[j] = fmaf(wv.y, xv.y, acc[j]);
                    acc[j] = fmaf(wv.z, xv.z, acc[j]);
                    acc[j] = fmaf(wv.w, xv.w, acc[j]);
                }
            }
        }
        for (uint32_t i = 4u * n4 + tid; i < hidden; i += 256u) {
            const float wv = router_w1(wr + i);
#pragma unroll
            for (int j = 0; j < kRlTokens; j++) {
                if ((uint32_t)j < nt) {
                    float xv = x[(uint64_t)(t0 + j) * hidden + i];
                    if (NORM) {
                        sq[j] += (double)xv * xv;
                        xv *= norm_w[i];
                    }
                    acc[j] = fmaf(wv, xv, acc[j]);
                }
            }
        }
        float red[2 * kRlTokens];
#pragma unroll
        for (int j = 0; j < kRlTokens; j++) {
            red[j] = acc[j];
            red[kRlTokens + j] = (float)sq[j];
        }
        block_sum_256_multi<2 * kRlTokens>(red, s_red, tid);
#pragma unroll
        for (int j = 0; j < kRlTokens; j++) {
            if ((uint32_t)j < nt) {
                const float scale = NORM ? 1.0f / sqrtf(red[kRlTokens + j] / (float)hidden + eps) : 1.0f;
                if (tid == 0) logits[(uint64_t)(t0 + j) * n_expert + e] = red[j] * scale;
                if (NORM) {
                    // every workgroup holds every token's scale (the same sums in the same order), so
                    // each writes its slice of every normalized row, whatever the number of tokens
                    const uint32_t t = t0 + (uint32_t)j;
                    const uint32_t lo = (uint32_t)((uint64_t)e * hidden / n_expert);
                    const uint32_t hi = (uint32_t)((uint64_t)(e + 1u) * hidden / n_expert);
                    const float *xr = x + (uint64_t)t * hidden;
                    float *xo = xn + (uint64_t)t * hidden;
                    for (uint32_t i = lo + tid; i < hi; i += 256u) xo[i] = xr[i] * scale * norm_w[i];
                }
            }
        }
    }
}

// MXFP4 matrices between the engine's rows (136-byte super-blocks) and the planar form
// (dsx_device.hpp), in place: the permutation stays inside each 16-row tile, so a workgroup
// reads one tile (grid.x) of one matrix (grid.y) into LDS and writes it back in the other
// order, 8 bytes per thread and step.  TO_PLANAR picks the direction.
// LDS (dynamic): 16 n_sb 136 bytes
template <bool TO_PLANAR>
__global__ __launch_bounds__(256) void k_mxfp4_relayout(uint8_t *__restrict__ w, uint32_t n_sb,
                                                        uint64_t stride) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t tile_bytes = 16u * n_sb * kSuperBytes, n_pieces = tile_bytes / 8u;
    uint8_t *tile = w + (uint64_t)blockIdx.y * stride + (uint64_t)blockIdx.x * tile_bytes;
    for (uint32_t i = threadIdx.x; i < n_pieces; i += 256u) *(uint2 *)(smem + i * 8u) = *(const uint2 *)(tile + i * 8u);
    __syncthreads();
    const uint32_t n_nib = 16u * n_sb * 16u;   // 8-byte pieces of nibbles
    for (uint32_t i = threadIdx.x; i < n_pieces; i += 256u) {
        // piece i of the planar order sits at rows_off in the row order
        uint32_t rows_off;
        if (i < n_nib) {
            const uint32_t blk = i >> 4, row = blk / n_sb, sb = blk - row * n_sb;
            rows_off = (row * n_sb + sb) * kSuperBytes + (i & 15u) * 8u;
        } else {
            const uint32_t s = i - n_nib, sb = s >> 4, row = s & 15u;
            rows_off = (row * n_sb + sb) * kSuperBytes + 128u;
        }
        if (TO_PLANAR) *(uint2 *)(tile + i * 8u) = *(const uint2 *)(smem + rows_off);
        else *(uint2 *)(tile + rows_off) = *(const uint2 *)(smem + i * 8u);
    }
}

// HF packed nibbles + E8M0 scales -> v2 super-block rows, one thread per 32-element block.
// crates/v4flash-kernels/kernels/mxfp4_repack.hip:35-65 (same bytes as
// crates/v4flash-core/src/hf_v41.rs:1208-1232).
__global__ __launch_bounds__(256) void k_mxfp4_repack(uint8_t *__restrict__ dst,
                                                      const uint8_t *__restrict__ packed,
                                                      const uint8_t *__restrict__ scale,
                                                      uint32_t out, uint32_t nb) {
    const uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    if (i >= (uint64_t)out * nb) return;
    const uint64_t r = i / nb, j = i - r * nb;
    const uint8_t *pb = packed + (r * nb + j) * 16u;
    uint8_t *sup = dst + r * nb * 17u + (j >> 3) * 136u;
    const uint32_t k = (uint32_t)(j & 7u);
    sup[128u + k] = scale[r * nb + j];
    const uint2 lo = *(const uint2 *)pb, hi = *(const uint2 *)(pb + 8);
    const uint8_t *lob = (const uint8_t *)&lo, *hib = (const uint8_t *)&hi;
    uint32_t w[4];
#pragma unroll
    for (int q = 0; q < 4; q++) {
        uint32_t v = 0;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const uint32_t l8 = lob[2 * q + h], h8 = hib[2 * q + h];
            const uint32_t b0 = (l8 & 0x0Fu) | ((h8 << 4) & 0xF0u);
            const uint32_t b1 = (l8 >> 4) | (h8 & 0xF0u);
            v |= (b0 | (b1 << 8)) << (16 * h);
        }
        w[q] = v;
    }
    uint2 *d2 = (uint2 *)(sup + k * 16u);
    d2[0] = make_uint2(w[0], w[1]);
    d2[1] = make_uint2(w[2], w[3]);
}

// Dequantize engine rows to f32 (checking aid).
__device__ __forceinline__ float e8m0_half(uint32_t e) {
    return __uint_as_float((e < 2u) ? (0x00200000u << e) : ((e - 1u) << 23));
}
__global__ __launch_bounds__(256) void k_mxfp4_dequant(float *__restrict__ y,
                                                       const uint8_t *__restrict__ rows,
                                                       uint64_t n_blocks32) {
    const uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    if (i >= n_blocks32) return;
    const int8_t kv[16] = {0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12};
    const uint8_t *sup = rows + (i >> 3) * 136u;
    const uint32_t k = (uint32_t)(i & 7u);
    const float d = e8m0_half(sup[128u + k]);
    for (int j = 0; j < 16; j++) {
        const uint8_t q = sup[k * 16u + j];
        y[i * 32u + j] = (float)kv[q & 15u] * d;
        y[i * 32u + 16u + j] = (float)kv[q >> 4] * d;
    }
}
__global__ __launch_bounds__(256) void k_q8_0_dequant(float *__restrict__ y,
                                                      const uint8_t *__restrict__ rows,
                                                      uint32_t n_rows, uint32_t blocks) {
    const uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    if (i >= (uint64_t)n_rows * blocks) return;
    const uint64_t r = i / blocks, b = i - r * blocks;
    const uint8_t *wr = rows + r * blocks * 34u;
    const float d = __half2float(*(const __half *)(wr + b * 2u));
    const int8_t *q = (const int8_t *)(wr + (uint64_t)blocks * 2u + b * 32u);
    for (int j = 0; j < 32; j++) y[i * 32u + j] = d * (float)q[j];
}

// ---------------------------------------------------------------------------------------
// Checkpoint matrix -> Q8_0 weights.  Source values are f32, bf16, or fp8-e4m3 codes times an
// E8M0 scale grid whose cells are br x bc elements; eight lanes share a 32-element block
// (four elements each).  d = amax/127 in f32 stored as f16 (round to nearest even),
// q = round-half-away(x * (1/d)), NaN -> 0.
// crates/v4flash-core/src/hf_v41.rs:728-805 (read_q8), :99-118 (E8M0, E4M3), :125-137 (block).
// split != 0 writes engine rows [blocks x f16 d][blocks x 32 i8]
// (crates/v4flash-kernels/src/weights.rs:225-240), else ggml blocks [f16 d][32 i8].
// ---------------------------------------------------------------------------------------
constexpr uint32_t kSrcF32 = 0u, kSrcBF16 = 1u, kSrcF8E4M3 = 2u;

__device__ __forceinline__ float e4m3_value(uint32_t b) {  // torch float8_e4m3fn
    if ((b & 0x7Fu) == 0x7Fu) return __uint_as_float(0x7FC00000u);
    const uint32_t e = (b >> 3) & 15u, m = b & 7u;
    const float v = (e == 0u) ? (float)m * 0x1p-9f
                              : (1.0f + (float)m * 0.125f) * __uint_as_float((e + 120u) << 23);
    return (b & 0x80u) ? -v : v;
}
__device__ __forceinline__ float e8m0_value(uint32_t e) {  // torch float8_e8m0fnu
    if (e == 0xFFu) return __uint_as_float(0x7FC00000u);
    return __uint_as_float(e == 0u ? (1u << 22) : (e << 23));
}

__device__ __forceinline__ void store_q4(uint8_t *p, uint32_t packed) {
    if (((uintptr_t)p & 3u) == 0u) {
        *(uint32_t *)p = packed;
    } else {
        *(uint16_t *)p = (uint16_t)packed;
        *(uint16_t *)(p + 2) = (uint16_t)(packed >> 16);
    }
}

template <uint32_t SRC>
__global__ __launch_bounds__(256) void k_q8_0_weights(uint8_t *__restrict__ dst,
                                                      const void *__restrict__ src,
                                                      const uint8_t *__restrict__ scale,
                                                      uint32_t out_rows, uint32_t in_cols,
                                                      uint32_t br, uint32_t bc, uint32_t sc,
                                                      uint32_t split) {
    const uint64_t gid = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    const uint32_t bpr = in_cols / 32u;
    const uint64_t blk = gid >> 3;
    const uint32_t sub = (uint32_t)(gid & 7u);
    const bool live = blk < (uint64_t)out_rows * bpr;
    const uint64_t r = live ? blk / bpr : 0, b = live ? blk - r * bpr : 0;
    const uint64_t c0 = b * 32u + sub * 4u;
    float xs[4] = {0.f, 0.f, 0.f, 0.f};
    if (live) {
        if (SRC == kSrcF32) {
            const float4 v = *(const float4 *)((const float *)src + r * in_cols + c0);
            xs[0] = v.x, xs[1] = v.y, xs[2] = v.z, xs[3] = v.w;
        } else if (SRC == kSrcBF16) {
            const uint2 v = *(const uint2 *)((const uint16_t *)src + r * in_cols + c0);
            xs[0] = __uint_as_float(v.x << 16), xs[1] = __uint_as_float(v.x & 0xFFFF0000u);
            xs[2] = __uint_as_float(v.y << 16), xs[3] = __uint_as_float(v.y & 0xFFFF0000u);
        } else {
            const uint32_t v = *(const uint32_t *)((const uint8_t *)src + r * in_cols + c0);
            const uint8_t *srow = scale + (r / br) * sc;
#pragma unroll
            for (int i = 0; i < 4; i++)
                xs[i] = e4m3_value((v >> (8 * i)) & 0xFFu) * e8m0_value(srow[(c0 + i) / bc]);
        }
    }
    // fmaxf drops NaN operands, like the reference's fold over f32::max
    float amax = fmaxf(fmaxf(fmaxf(0.0f, fabsf(xs[0])), fabsf(xs[1])),
                       fmaxf(fabsf(xs[2]), fabsf(xs[3])));
    amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
    amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
    amax = fmaxf(amax, __shfl_xor(amax, 4, 64));
    if (!live) return;
    const float d = amax / 127.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    uint32_t packed = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float t = roundf(xs[i] * id);
        int q = (t != t) ? 0 : (t >= 127.0f ? 127 : (t <= -128.0f ? -128 : (int)t));
        packed |= (uint32_t)(q & 0xFF) << (8 * i);
    }
    uint8_t *dp, *qp;
    if (split) {
        uint8_t *row = dst + r * bpr * 34u;
        dp = row + b * 2u;
        qp = row + (uint64_t)bpr * 2u + b * 32u + sub * 4u;
    } else {
        dp = dst + blk * 34u;
        qp = dp + 2u + sub * 4u;
    }
    store_q4(qp, packed);
    if (sub == 0) *(__half *)dp = __float2half_rn(d);
}

// ggml Q8_0 blocks -> engine rows (crates/v4flash-kernels/src/weights.rs:225-240).
__global__ __launch_bounds__(256) void k_q8_0_repack_rows(uint8_t *__restrict__ dst,
                                                          const uint8_t *__restrict__ src,
                                                          uint32_t n_rows, uint32_t bpr) {
    const uint64_t gid = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    const uint64_t blk = gid >> 3;
    const uint32_t sub = (uint32_t)(gid & 7u);
    if (blk >= (uint64_t)n_rows * bpr) return;
    const uint64_t r = blk / bpr, b = blk - r * bpr;
    const uint8_t *s = src + blk * 34u;
    uint8_t *row = dst + r * bpr * 34u;
    const uint32_t lo = *(const uint16_t *)(s + 2u + sub * 4u), hi = *(const uint16_t *)(s + 4u + sub * 4u);
    store_q4(row + (uint64_t)bpr * 2u + b * 32u + sub * 4u, lo | (hi << 16));
    if (sub == 0) *(uint16_t *)(row + b * 2u) = *(const uint16_t *)s;
}

// Identity grouping for a dense expert: every token is a member of expert 0 with weight 1.
// Router logits for many tokens: logits[t, e] = sum_k W[e, k] * x[t, k] with f32 products and
// sums on the f32 matrix instruction (v_mfma_f32_16x16x4_f32).  A workgroup of four waves
// computes 32 experts x 32 tokens, one 16 x 16 fragment per wave; a lane fetches four consecutive
// k of its row of W and of its row of x with one 128-bit load each and feeds them to four
// instructions (k is summed over, so any assignment of k to instructions is the same sum up to
// f32 order).  Every operand row is read once per tile instead of once per expert.
// hidden % 16 == 0, n_expert % 4 == 0.
// (crates/v4flash-kernels/src/het/forward_prefill.rs:8974-9015, the engine's batched router GEMM.)
typedef float v4f_rl __attribute__((ext_vector_type(4)));
template <typename WT>
__global__ __launch_bounds__(256) void k_router_logits_tiled(float *__restrict__ logits,
                                                             const WT *__restrict__ w,
                                                             const float *__restrict__ x,
                                                             uint32_t n_expert, uint32_t hidden,
                                                             uint32_t n_tokens) {
    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u;
    const uint32_t e0 = blockIdx.x * 32u + (wave & 1u) * 16u, t0 = blockIdx.y * 32u + (wave >> 1) * 16u;
    if (e0 >= n_expert || t0 >= n_tokens) return;  // uniform per wave; no barrier below
    const uint32_t r = lane & 15u, kg = lane >> 4;
    // rows past the end repeat the last one (loaded, never stored)
    const WT *wr = w + (uint64_t)min(e0 + r, n_expert - 1u) * hidden + 4u * kg;
    const float *xr = x + (uint64_t)min(t0 + r, n_tokens - 1u) * hidden + 4u * kg;
    v4f_rl acc = {0.f, 0.f, 0.f, 0.f};
    for (uint32_t k = 0; k < hidden; k += 16u) {
        const float4 a = router_w4(wr + k);
        const float4 b = *(const float4 *)(xr + k);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, b.x, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, b.y, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, b.z, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, b.w, acc, 0, 0, 0);
    }
    // the lane holds experts e0 + 4 kg .. + 3 of token t0 + r
    const uint32_t t = t0 + r, e = e0 + 4u * kg;
    if (t < n_tokens && e < n_expert)
        *(float4 *)(logits + (uint64_t)t * n_expert + e) = make_float4(acc.x, acc.y, acc.z, acc.w);
}

__global__ __launch_bounds__(256) void k_dense_groups(int32_t *__restrict__ group_count,
                                                      int32_t *__restrict__ group_offset,
                                                      int32_t *__restrict__ members,
                                                      int32_t *__restrict__ work_items,
                                                      int32_t *__restrict__ n_work_items,
                                                      float *__restrict__ ones, uint32_t b,
                                                      uint32_t chunk) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i < b) {
        members[i] = (int)(i << 16);
        ones[i] = 1.0f;
    }
    const uint32_t nwi = (b + chunk - 1) / chunk;
    if (i < nwi) work_items[i] = (int)(i * chunk);
    if (i == 0) {
        group_count[0] = (int)b;
        group_offset[0] = 0;
        group_offset[1] = (int)b;
        *n_work_items = (int)nwi;
    }
}

// Q8_0 activation rows: [k int8][k/32 f32 scales], one row per token
// (same arithmetic as k_q8_0_quantize; the scales follow the quants so that one pointer
// names a token's activation, like a Q8_K row does).
__global__ __launch_bounds__(256) void k_q8_0_quantize_rows(uint8_t *__restrict__ out,
                                                            const float *__restrict__ x,
                                                            uint32_t rows, uint32_t k) {
    const uint64_t gid = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    const uint32_t bpr = k / 32u;
    const uint64_t blk = gid >> 3;
    const uint32_t sub = (uint32_t)(gid & 7u);
    const bool live = blk < (uint64_t)rows * bpr;
    const uint64_t r = live ? blk / bpr : 0, b = live ? blk - r * bpr : 0;
    float4 v = {0.f, 0.f, 0.f, 0.f};
    if (live) v = *(const float4 *)(x + r * k + b * 32u + sub * 4u);
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
    amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
    amax = fmaxf(amax, __shfl_xor(amax, 4, 64));
    if (!live) return;
    const float d = amax / 127.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    const float xs[4] = {v.x, v.y, v.z, v.w};
    uint32_t packed = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        int q = (int)rintf(xs[i] * id);
        q = q > 127 ? 127 : q;
        q = q < -128 ? -128 : q;
        packed |= (uint32_t)(q & 0xFF) << (8 * i);
    }
    uint8_t *row = out + r * (uint64_t)(k + k / 8u);
    *(uint32_t *)(row + b * 32u + sub * 4u) = packed;
    if (sub == 0) *(float *)(row + k + b * 4u) = d;
}

}  // namespace dsx
