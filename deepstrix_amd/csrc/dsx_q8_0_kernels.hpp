// dsx_q8_0_kernels.hpp -- Q8_0 expert products on gfx950.
//
// Weights: engine rows [blocks x f16 d][blocks x 32 i8] (crates/v4flash-kernels/src/weights.rs:
// 225-240).  Activations: rows [k i8][k/32 f32 scales] made by k_q8_0_quantize_rows
// (crates/v4flash-kernels/kernels/q8_0_matvec.hip:150-177).  The product of one block is
// exact in int32 (v_dot4_i32_i8), scaled by f16(d_w) * xscale in f32
// (crates/v4flash-kernels/kernels/q8_0_matvec.hip:64-104).
//
// A wave reads weight rows front to back: lane l takes blocks l, l + 64, ... (32 int8 =
// 32 contiguous bytes per lane, 2 KiB contiguous per wave load step), multiplies them with
// the matching activation blocks of every token column (LDS), and the 64 partial sums of a
// (row, column) are added by a butterfly.  A workgroup of four waves owns 16 rows, four per
// wave, which the wave streams together.  These are streaming kernels for few columns (decode
// and small batches).
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/dsx_moe.h"
#include "dsx_device.hpp"
#include "dsx_quant.hpp"

namespace dsx {

int q8_0_fail(int code, const char *what, const char *why);

constexpr int kQ8Waves = 4;
constexpr int kQ8RowsPerWg = 16;
constexpr size_t kQ8LdsBudget = 140 * 1024;

__host__ __device__ inline uint32_t q8_0_act_row_bytes(uint32_t n_blocks) { return n_blocks * 36u; }

struct Q8Params {
    float *dst;                       // mid / partials [dest rows, n_rows], or out [n_rows]
    const uint8_t *w0, *w1;           // [n_expert] experts: gate and up, or down in w0
    const uint8_t *sh_w0, *sh_w1;     // decode: the extra slot n_used (weight 1), or null
    uint64_t bpe0, bpe1;
    const uint8_t *xq;                // activation rows, x_stride bytes apart
    const float *ew;
    const int32_t *selected;          // decode
    const int32_t *group_count, *group_offset, *members, *work_items, *n_work_items;
    uint32_t x_stride, n_used, chunk, n_rows, n_blocks;
    float clamp, sh_clamp;
    // by-expert with the extra expert (index n_expert, slot n_used; rows after the routed ones)
    uint32_t n_expert, n_tokens;
    // by-expert: workgroups along grid.y per work item, NT columns each (0 is read as 1)
    uint32_t n_sub;
    // down, by-expert: consecutive 16-row tiles per workgroup (0 is read as 1)
    uint32_t row_tiles;
};

// The lane's share of `rows[r] . x[c]` for R weight rows and NT columns, over all of its blocks.  The
// rows' blocks of a step are all requested before the first is used, so that R times the bytes of a
// single row are in flight: one row at a time is bound by the round trip of each step (a row of 64
// blocks is a single step; a decode step's shared expert went from 69 to 54 us with four rows).
// Per (row, column) the sum runs over the lane's blocks in ascending order, one term
// f16(d_w) * xscale * int32 dot per block.
template <int R, int NT>
__device__ __forceinline__ void q8_0_rows_partial(float (&acc)[R][NT], const uint8_t *const (&rows)[R],
                                                  const uint8_t *lds_x, uint32_t col_stride,
                                                  uint32_t n_blocks, uint32_t lane) {
    for (uint32_t b0 = 0; b0 < n_blocks; b0 += 64u) {
        const uint32_t b = b0 + lane;
        const bool live = b < n_blocks;
        const uint32_t bb = live ? b : n_blocks - 1u;  // clamped: the load stays in the row
        U2A4 w[R][4];
        uint16_t dbits[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            const uint8_t *q = rows[r] + (size_t)n_blocks * 2u + (size_t)bb * 32u;
            w[r][0] = gload8(q);
            w[r][1] = gload8(q + 8u);
            w[r][2] = gload8(q + 16u);
            w[r][3] = gload8(q + 24u);
            dbits[r] = *(const DSX_GLOBAL uint16_t *)(uintptr_t)(rows[r] + (size_t)bb * 2u);
        }
#pragma unroll
        for (int c = 0; c < NT; c++) {
            const uint8_t *xc = lds_x + (size_t)c * col_stride;
            const uint4 x0 = *(const uint4 *)(xc + bb * 32u);
            const uint4 x1 = *(const uint4 *)(xc + bb * 32u + 16u);
            const float xs = *(const float *)(xc + n_blocks * 32u + bb * 4u);
#pragma unroll
            for (int r = 0; r < R; r++) {
                const float dw = live ? __half2float(__ushort_as_half(dbits[r])) : 0.0f;
                int s = 0;
                s = __builtin_amdgcn_sdot4((int)w[r][0].x, (int)x0.x, s, false);
                s = __builtin_amdgcn_sdot4((int)w[r][0].y, (int)x0.y, s, false);
                s = __builtin_amdgcn_sdot4((int)w[r][1].x, (int)x0.z, s, false);
                s = __builtin_amdgcn_sdot4((int)w[r][1].y, (int)x0.w, s, false);
                s = __builtin_amdgcn_sdot4((int)w[r][2].x, (int)x1.x, s, false);
                s = __builtin_amdgcn_sdot4((int)w[r][2].y, (int)x1.y, s, false);
                s = __builtin_amdgcn_sdot4((int)w[r][3].x, (int)x1.z, s, false);
                s = __builtin_amdgcn_sdot4((int)w[r][3].y, (int)x1.w, s, false);
                acc[r][c] += dw * xs * (float)s;
            }
        }
    }
}

// Copies `n_cols` activation rows (row j from src(j)) into LDS, col_stride bytes apart.
template <typename Src>
__device__ __forceinline__ void q8_0_stage(uint8_t *lds_x, uint32_t n_cols, uint32_t row_bytes,
                                           uint32_t tid, const Src src) {
    const uint32_t per = row_bytes / 16u;
    for (uint32_t q = tid; q < n_cols * per; q += kQ8Waves * 64u) {
        const uint32_t j = q / per, c = q - j * per;
        *(uint4 *)(lds_x + (size_t)j * row_bytes + (size_t)c * 16u) =
            *(const uint4 *)(src(j) + (size_t)c * 16u);
    }
}

// ---------------------------------------------------------------------------------------
// gate/up + SwiGLU.  BY_EXPERT = false: one token, grid.y = slot (slot n_used = the extra
// expert).  BY_EXPERT = true: grid.y = work item, columns = its members.
// crates/v4flash-kernels/src/het/dispatch.rs:26-66, 534-570 (Q8_0 arms)
// ---------------------------------------------------------------------------------------
template <int NT, bool BY_EXPERT>
__global__ __launch_bounds__(kQ8Waves * 64) void k_q8_0_gate_up(const Q8Params p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_x[];
    __shared__ uint32_t s_tok[NT];
    __shared__ uint32_t s_dest[NT];
    __shared__ float s_ew[NT];
    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u;
    const uint32_t n_sub = (BY_EXPERT && p.n_sub > 1u) ? p.n_sub : 1u;
    const uint32_t row0 = blockIdx.x * kQ8RowsPerWg, item = blockIdx.y / n_sub;
    const uint32_t col_off = (blockIdx.y - item * n_sub) * (uint32_t)NT;  // first member served here
    const uint32_t row_bytes = q8_0_act_row_bytes(p.n_blocks);
    const uint8_t *g_e, *u_e;
    uint32_t cnt = 1;
    float clamp = p.clamp;
    if (BY_EXPERT) {
        if ((int)item >= *p.n_work_items) return;
        const uint32_t wi = (uint32_t)p.work_items[item];
        const uint32_t e = wi >> 16, start = (wi & 0xFFFFu) + col_off;
        const uint32_t total = (uint32_t)p.group_count[e];
        if (start >= total) return;  // uniform: this sub-chunk of the item has no members
        cnt = min(min(p.chunk - col_off, (uint32_t)NT), total - start);
        const uint32_t mbase = (uint32_t)p.group_offset[e] + start;
        if (tid < cnt) {
            const uint32_t m = (uint32_t)p.members[mbase + tid];
            const uint32_t t = m >> 16, slot = m & 0xFFFFu;
            s_tok[tid] = t;
            s_dest[tid] = slot >= p.n_used ? p.n_tokens * p.n_used + t : t * p.n_used + slot;
            s_ew[tid] = slot >= p.n_used ? 1.0f : p.ew[t * p.n_used + slot];
        }
        const bool extra = p.sh_w0 != nullptr && e >= p.n_expert;
        g_e = extra ? p.sh_w0 : p.w0 + (uint64_t)e * p.bpe0;
        u_e = extra ? p.sh_w1 : p.w1 + (uint64_t)e * p.bpe1;
        if (extra) clamp = p.sh_clamp;
    } else {
        if (item < p.n_used) {
            const int e = p.selected[item];
            if (e < 0) {  // empty slot: defined output
                if (tid < (uint32_t)kQ8RowsPerWg) p.dst[(uint64_t)item * p.n_rows + row0 + tid] = 0.0f;
                return;
            }
            g_e = p.w0 + (uint64_t)e * p.bpe0;
            u_e = p.w1 + (uint64_t)e * p.bpe1;
            if (tid == 0) s_ew[0] = p.ew[item];
        } else {
            g_e = p.sh_w0;
            u_e = p.sh_w1;
            clamp = p.sh_clamp;
            if (tid == 0) s_ew[0] = 1.0f;
        }
        if (tid == 0) {
            s_tok[0] = 0;
            s_dest[0] = item;
        }
    }
    __syncthreads();
    q8_0_stage(lds_x, cnt, row_bytes, tid,
               [&](uint32_t j) { return p.xq + (uint64_t)s_tok[j] * p.x_stride; });
    __syncthreads();

    const uint64_t wstride = (uint64_t)p.n_blocks * 34u;
    // the wave's four rows (wave, wave + 4, ...) two at a time, gate and up together
    static_assert(kQ8RowsPerWg == 4 * kQ8Waves, "four rows per wave");
#pragma unroll
    for (uint32_t half = 0; half < 2u; half++) {
        const uint32_t ra = row0 + wave + half * 2u * kQ8Waves, rb = ra + kQ8Waves;
        const uint8_t *const rows[4] = {g_e + (uint64_t)ra * wstride, u_e + (uint64_t)ra * wstride,
                                        g_e + (uint64_t)rb * wstride, u_e + (uint64_t)rb * wstride};
        float a[4][NT];
#pragma unroll
        for (int r = 0; r < 4; r++)
#pragma unroll
            for (int c = 0; c < NT; c++) a[r][c] = 0.0f;
        q8_0_rows_partial<4, NT>(a, rows, lds_x, row_bytes, p.n_blocks, lane);
#pragma unroll
        for (int c = 0; c < NT; c++) {
            const float g0 = wave_sum_f32(a[0][c]), u0 = wave_sum_f32(a[1][c]);
            const float g1 = wave_sum_f32(a[2][c]), u1 = wave_sum_f32(a[3][c]);
            if (lane == 0 && (uint32_t)c < cnt) {
                p.dst[(uint64_t)s_dest[c] * p.n_rows + ra] = swiglu_clamp(g0, u0, clamp, s_ew[c]);
                p.dst[(uint64_t)s_dest[c] * p.n_rows + rb] = swiglu_clamp(g1, u1, clamp, s_ew[c]);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------
// down, one token: out[row] = sum over slots (slot order) of down_e(slot)[row] . midq[slot].
// crates/v4flash-kernels/src/het/dispatch.rs:121-150 (Q8_0 arm)
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(kQ8Waves * 64) void k_q8_0_down_decode(const Q8Params p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_x[];
    __shared__ int s_sel[DSX_MAX_USED + 1];
    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u;
    const uint32_t row0 = blockIdx.x * kQ8RowsPerWg;
    const uint32_t row_bytes = q8_0_act_row_bytes(p.n_blocks);
    const uint32_t n_slots = p.n_used + (p.sh_w0 ? 1u : 0u);
    if (tid < p.n_used) s_sel[tid] = p.selected[tid];
    q8_0_stage(lds_x, n_slots, row_bytes, tid,
               [&](uint32_t j) { return p.xq + (uint64_t)j * p.x_stride; });
    __syncthreads();
    const uint64_t wstride = (uint64_t)p.n_blocks * 34u;
    // the wave's four rows (wave, wave + 4, ...) at once, slot after slot
    float total[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (uint32_t s = 0; s < n_slots; s++) {
        const uint8_t *w;
        if (s < p.n_used) {
            const int e = s_sel[s];
            if (e < 0) continue;
            w = p.w0 + (uint64_t)e * p.bpe0;
        } else {
            w = p.sh_w0;
        }
        const uint8_t *base = w + (uint64_t)(row0 + wave) * wstride;
        const uint8_t *const rows[4] = {base, base + kQ8Waves * wstride, base + 2u * kQ8Waves * wstride,
                                        base + 3u * kQ8Waves * wstride};
        float a[4][1] = {{0.0f}, {0.0f}, {0.0f}, {0.0f}};
        q8_0_rows_partial<4, 1>(a, rows, lds_x + (size_t)s * row_bytes, row_bytes, p.n_blocks, lane);
#pragma unroll
        for (int r = 0; r < 4; r++) total[r] += wave_sum_f32(a[r][0]);
    }
    if (lane == 0) {
#pragma unroll
        for (int r = 0; r < 4; r++) p.dst[row0 + wave + (uint32_t)r * kQ8Waves] = total[r];
    }
}

// ---------------------------------------------------------------------------------------
// down, by expert: partials[(t * n_used + slot) * n_rows + row] = down_e[row] . midq[t, slot]
// crates/v4flash-kernels/src/het/dispatch.rs:580-620 (Q8_0 arm)
// ---------------------------------------------------------------------------------------
template <int NT>
__global__ __launch_bounds__(kQ8Waves * 64) void k_q8_0_down_by_expert(const Q8Params p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_x[];
    __shared__ uint32_t s_dest[NT];
    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u;
    const uint32_t n_sub = p.n_sub > 1u ? p.n_sub : 1u;
    const uint32_t row_tiles = p.row_tiles > 1u ? p.row_tiles : 1u;
    const uint32_t row00 = blockIdx.x * row_tiles * kQ8RowsPerWg, item = blockIdx.y / n_sub;
    const uint32_t col_off = (blockIdx.y - item * n_sub) * (uint32_t)NT;
    const uint32_t row_bytes = q8_0_act_row_bytes(p.n_blocks);
    if ((int)item >= *p.n_work_items) return;
    const uint32_t wi = (uint32_t)p.work_items[item];
    const uint32_t e = wi >> 16, start = (wi & 0xFFFFu) + col_off;
    const uint32_t total = (uint32_t)p.group_count[e];
    if (start >= total) return;  // uniform: this sub-chunk of the item has no members
    const uint32_t cnt = min(min(p.chunk - col_off, (uint32_t)NT), total - start);
    const uint32_t mbase = (uint32_t)p.group_offset[e] + start;
    if (tid < cnt) {
        const uint32_t m = (uint32_t)p.members[mbase + tid];
        const uint32_t t = m >> 16, slot = m & 0xFFFFu;
        s_dest[tid] = slot >= p.n_used ? p.n_tokens * p.n_used + t : t * p.n_used + slot;
    }
    __syncthreads();
    q8_0_stage(lds_x, cnt, row_bytes, tid,
               [&](uint32_t j) { return p.xq + (uint64_t)s_dest[j] * p.x_stride; });
    __syncthreads();
    const uint8_t *w_e = (p.sh_w0 != nullptr && e >= p.n_expert) ? p.sh_w0 : p.w0 + (uint64_t)e * p.bpe0;
    const uint64_t wstride = (uint64_t)p.n_blocks * 34u;
    // One look-up of the item and one staged copy of its members' rows serve several row tiles (a
    // tile's weights are no more bytes than the staged rows of a few members).
    for (uint32_t rt = 0; rt < row_tiles && row00 + rt * kQ8RowsPerWg < p.n_rows; rt++) {
        const uint32_t row0 = row00 + rt * kQ8RowsPerWg;
        // the wave's four rows (wave, wave + 4, ...) at once
        const uint8_t *base = w_e + (uint64_t)(row0 + wave) * wstride;
        const uint8_t *const rows[4] = {base, base + kQ8Waves * wstride, base + 2u * kQ8Waves * wstride,
                                        base + 3u * kQ8Waves * wstride};
        float a[4][NT];
#pragma unroll
        for (int r = 0; r < 4; r++)
#pragma unroll
            for (int c = 0; c < NT; c++) a[r][c] = 0.0f;
        q8_0_rows_partial<4, NT>(a, rows, lds_x, row_bytes, p.n_blocks, lane);
#pragma unroll
        for (int r = 0; r < 4; r++)
#pragma unroll
            for (int c = 0; c < NT; c++) {
                const float v = wave_sum_f32(a[r][c]);
                if (lane == 0 && (uint32_t)c < cnt)
                    p.dst[(uint64_t)s_dest[c] * p.n_rows + row0 + wave + (uint32_t)r * kQ8Waves] = v;
            }
    }
}

// ---- host side ----------------------------------------------------------------------------
inline void q8_0_raise_lds_limits() {
    const int lim = 160 * 1024 - 16 * 1024;
    (void)hipFuncSetAttribute((const void *)k_q8_0_gate_up<1, false>, hipFuncAttributeMaxDynamicSharedMemorySize, lim);
    (void)hipFuncSetAttribute((const void *)k_q8_0_gate_up<1, true>, hipFuncAttributeMaxDynamicSharedMemorySize, lim);
    (void)hipFuncSetAttribute((const void *)k_q8_0_gate_up<2, true>, hipFuncAttributeMaxDynamicSharedMemorySize, lim);
    (void)hipFuncSetAttribute((const void *)k_q8_0_gate_up<4, true>, hipFuncAttributeMaxDynamicSharedMemorySize, lim);
    (void)hipFuncSetAttribute((const void *)k_q8_0_gate_up<8, true>, hipFuncAttributeMaxDynamicSharedMemorySize, lim);
    (void)hipFuncSetAttribute((const void *)k_q8_0_down_decode, hipFuncAttributeMaxDynamicSharedMemorySize, lim);
    (void)hipFuncSetAttribute((const void *)k_q8_0_down_by_expert<1>, hipFuncAttributeMaxDynamicSharedMemorySize, lim);
    (void)hipFuncSetAttribute((const void *)k_q8_0_down_by_expert<2>, hipFuncAttributeMaxDynamicSharedMemorySize, lim);
    (void)hipFuncSetAttribute((const void *)k_q8_0_down_by_expert<4>, hipFuncAttributeMaxDynamicSharedMemorySize, lim);
    (void)hipFuncSetAttribute((const void *)k_q8_0_down_by_expert<8>, hipFuncAttributeMaxDynamicSharedMemorySize, lim);
}

inline int q8_0_check(const char *what, uint32_t n_rows, uint32_t n_blocks, const void *w0,
                      const void *w1, uint64_t bpe0, uint64_t bpe1, const void *xq, uint32_t x_stride,
                      uint32_t n_cols) {
    if (n_rows == 0 || n_rows % kQ8RowsPerWg != 0)
        return q8_0_fail(DSX_ERR_SHAPE, what, "n_rows must be a multiple of 16");
    if (n_blocks == 0 || n_blocks % 4 != 0)
        return q8_0_fail(DSX_ERR_SHAPE, what, "Q8_0 rows need k % 128 == 0");
    if ((uintptr_t)w0 % 8 || (uintptr_t)w1 % 8 || bpe0 % 8 || bpe1 % 8)
        return q8_0_fail(DSX_ERR_SHAPE, what, "Q8_0 weights must be 8-byte aligned");
    if ((uintptr_t)xq % 16 || x_stride % 16 || x_stride < q8_0_act_row_bytes(n_blocks))
        return q8_0_fail(DSX_ERR_SHAPE, what, "Q8_0 activation rows must be 16-byte aligned, stride >= 36 * blocks");
    if ((size_t)n_cols * q8_0_act_row_bytes(n_blocks) > kQ8LdsBudget)
        return q8_0_fail(DSX_ERR_UNSUPPORTED, what, "activation columns exceed LDS staging");
    return DSX_OK;
}

inline int q8_0_pick_nt(uint32_t chunk) { return chunk <= 1 ? 1 : chunk <= 2 ? 2 : chunk <= 4 ? 4 : 8; }
// Columns per workgroup for a work item of `chunk` members: as many as LDS stages (at most 8);
// a larger chunk is served by several workgroups per item.
inline int q8_0_fit_nt(uint32_t chunk, uint32_t n_blocks) {
    int nt = q8_0_pick_nt(chunk);
    while (nt > 1 && (size_t)nt * q8_0_act_row_bytes(n_blocks) > kQ8LdsBudget) nt /= 2;
    return nt;
}

inline int q8_0_gate_up_decode(hipStream_t st, float *mid, const uint8_t *gate, const uint8_t *up,
                               const uint8_t *xq, const float *ew, const int32_t *selected,
                               const uint8_t *sh_gate, const uint8_t *sh_up, float sh_clamp,
                               uint64_t gbpe, uint64_t ubpe, uint32_t n_used, float clamp,
                               uint32_t n_rows, uint32_t n_blocks) {
    int rc = q8_0_check("moe_gate_up_batch", n_rows, n_blocks, gate, up, gbpe, ubpe, xq,
                        q8_0_act_row_bytes(n_blocks), 1);
    if (rc) return rc;
    Q8Params p{};
    p.dst = mid; p.w0 = gate; p.w1 = up; p.sh_w0 = sh_gate; p.sh_w1 = sh_up; p.bpe0 = gbpe; p.bpe1 = ubpe;
    p.xq = xq; p.ew = ew; p.selected = selected; p.x_stride = q8_0_act_row_bytes(n_blocks);
    p.n_used = n_used; p.chunk = 1; p.n_rows = n_rows; p.n_blocks = n_blocks; p.clamp = clamp;
    p.sh_clamp = sh_clamp;
    const uint32_t n_slots = n_used + (sh_gate ? 1u : 0u);
    hipLaunchKernelGGL((k_q8_0_gate_up<1, false>), dim3(n_rows / kQ8RowsPerWg, n_slots),
                       dim3(kQ8Waves * 64), q8_0_act_row_bytes(n_blocks), st, p);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? DSX_OK : q8_0_fail((int)e, "moe_gate_up_batch", hipGetErrorString(e));
}

inline int q8_0_down_decode(hipStream_t st, float *out, const uint8_t *down, const uint8_t *xq,
                            const int32_t *selected, const uint8_t *sh_down, uint64_t dbpe,
                            uint32_t xq_slot_stride, uint32_t n_used, uint32_t n_rows,
                            uint32_t n_blocks_in) {
    const uint32_t n_slots = n_used + (sh_down ? 1u : 0u);
    int rc = q8_0_check("moe_down_batched", n_rows, n_blocks_in, down, sh_down, dbpe, 0, xq,
                        xq_slot_stride, n_slots);
    if (rc) return rc;
    Q8Params p{};
    p.dst = out; p.w0 = down; p.sh_w0 = sh_down; p.bpe0 = dbpe; p.xq = xq; p.selected = selected;
    p.x_stride = xq_slot_stride; p.n_used = n_used; p.n_rows = n_rows; p.n_blocks = n_blocks_in;
    hipLaunchKernelGGL(k_q8_0_down_decode, dim3(n_rows / kQ8RowsPerWg), dim3(kQ8Waves * 64),
                       (size_t)n_slots * q8_0_act_row_bytes(n_blocks_in), st, p);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? DSX_OK : q8_0_fail((int)e, "moe_down_batched", hipGetErrorString(e));
}

inline int q8_0_gate_up_by_expert(hipStream_t st, float *mid, const uint8_t *gate, const uint8_t *up,
                                  const uint8_t *xq, const float *ew, const int32_t *group_count,
                                  const int32_t *group_offset, const int32_t *members,
                                  const int32_t *work_items, const int32_t *n_work_items,
                                  uint32_t max_wi, uint64_t gbpe, uint64_t ubpe, uint32_t n_used,
                                  uint32_t chunk, float clamp, uint32_t n_rows, uint32_t n_blocks,
                                  const uint8_t *sh_gate = nullptr, const uint8_t *sh_up = nullptr,
                                  float sh_clamp = 0.0f, uint32_t n_expert = 0, uint32_t n_tokens = 0) {
    const int nt = q8_0_fit_nt(chunk, n_blocks);
    const uint32_t n_sub = (chunk + (uint32_t)nt - 1u) / (uint32_t)nt;
    if ((uint64_t)max_wi * n_sub > 65535u)
        return q8_0_fail(DSX_ERR_INVALID_ARG, "moe_gate_up_chunked_rows", "work items x sub-chunks exceed the grid");
    int rc = q8_0_check("moe_gate_up_chunked_rows", n_rows, n_blocks, gate, up, gbpe, ubpe, xq,
                        q8_0_act_row_bytes(n_blocks), (uint32_t)nt);
    if (rc) return rc;
    Q8Params p{};
    p.dst = mid; p.w0 = gate; p.w1 = up; p.bpe0 = gbpe; p.bpe1 = ubpe; p.xq = xq; p.ew = ew;
    p.group_count = group_count; p.group_offset = group_offset; p.members = members;
    p.work_items = work_items; p.n_work_items = n_work_items;
    p.x_stride = q8_0_act_row_bytes(n_blocks); p.n_used = n_used; p.chunk = chunk; p.n_rows = n_rows;
    p.n_blocks = n_blocks; p.clamp = clamp;
    p.sh_w0 = sh_gate; p.sh_w1 = sh_up; p.sh_clamp = sh_clamp; p.n_expert = n_expert; p.n_tokens = n_tokens;
    p.n_sub = n_sub;
    const dim3 grid(n_rows / kQ8RowsPerWg, max_wi * n_sub), block(kQ8Waves * 64);
    const size_t lds = (size_t)nt * q8_0_act_row_bytes(n_blocks);
    switch (nt) {
        case 1: hipLaunchKernelGGL((k_q8_0_gate_up<1, true>), grid, block, lds, st, p); break;
        case 2: hipLaunchKernelGGL((k_q8_0_gate_up<2, true>), grid, block, lds, st, p); break;
        case 4: hipLaunchKernelGGL((k_q8_0_gate_up<4, true>), grid, block, lds, st, p); break;
        default: hipLaunchKernelGGL((k_q8_0_gate_up<8, true>), grid, block, lds, st, p); break;
    }
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? DSX_OK : q8_0_fail((int)e, "moe_gate_up_chunked_rows", hipGetErrorString(e));
}

inline int q8_0_down_by_expert(hipStream_t st, float *partials, const uint8_t *down, const uint8_t *xq,
                               const int32_t *group_count, const int32_t *group_offset,
                               const int32_t *members, const int32_t *work_items,
                               const int32_t *n_work_items, uint32_t max_wi, uint64_t dbpe,
                               uint32_t xq_slot_stride, uint32_t n_used, uint32_t chunk,
                               uint32_t n_rows, uint32_t n_blocks_in, const uint8_t *sh_down = nullptr,
                               uint32_t n_expert = 0, uint32_t n_tokens = 0) {
    const int nt = q8_0_fit_nt(chunk, n_blocks_in);
    const uint32_t n_sub = (chunk + (uint32_t)nt - 1u) / (uint32_t)nt;
    if ((uint64_t)max_wi * n_sub > 65535u)
        return q8_0_fail(DSX_ERR_INVALID_ARG, "moe_down_by_expert", "work items x sub-chunks exceed the grid");
    int rc = q8_0_check("moe_down_by_expert", n_rows, n_blocks_in, down, nullptr, dbpe, 0, xq,
                        xq_slot_stride, (uint32_t)nt);
    if (rc) return rc;
    Q8Params p{};
    p.dst = partials; p.w0 = down; p.bpe0 = dbpe; p.xq = xq;
    p.group_count = group_count; p.group_offset = group_offset; p.members = members;
    p.work_items = work_items; p.n_work_items = n_work_items;
    p.x_stride = xq_slot_stride; p.n_used = n_used; p.chunk = chunk; p.n_rows = n_rows;
    p.n_blocks = n_blocks_in;
    p.sh_w0 = sh_down; p.n_expert = n_expert; p.n_tokens = n_tokens;
    p.n_sub = n_sub;
    // Two row tiles per workgroup where that still leaves thousands of workgroups: the look-up and the
    // staged copy then cost half as much per tile (7168 x 2048 down matrices of 256 experts, 24 / 64
    // tokens: 476 -> 440 / 843 -> 778 us); a small grid needs every workgroup it has (2048 x 1408, 64
    // experts, 4 tokens: 27 -> 30 us with two tiles).
    const uint32_t n_tiles = n_rows / kQ8RowsPerWg;
    p.row_tiles = (uint64_t)n_tiles * max_wi * n_sub >= 16384u ? 2u : 1u;
    const dim3 grid((n_tiles + p.row_tiles - 1u) / p.row_tiles, max_wi * n_sub), block(kQ8Waves * 64);
    const size_t lds = (size_t)nt * q8_0_act_row_bytes(n_blocks_in);
    switch (nt) {
        case 1: hipLaunchKernelGGL(k_q8_0_down_by_expert<1>, grid, block, lds, st, p); break;
        case 2: hipLaunchKernelGGL(k_q8_0_down_by_expert<2>, grid, block, lds, st, p); break;
        case 4: hipLaunchKernelGGL(k_q8_0_down_by_expert<4>, grid, block, lds, st, p); break;
        default: hipLaunchKernelGGL(k_q8_0_down_by_expert<8>, grid, block, lds, st, p); break;
    }
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? DSX_OK : q8_0_fail((int)e, "moe_down_by_expert", hipGetErrorString(e));
}


// ---------------------------------------------------------------------------------------
// Expert products for many tokens per expert: grouped GEMMs on the int8 matrix instruction.
// Work item = (expert, first member), the next up to 128 members are the token columns; a
// workgroup (4 waves) multiplies 64 weight rows with them over all k, wave w owning rows
// 16 w .. 16 w + 15 and all columns.
//   gate/up (PAIR):  the 64 rows of gate and the same 64 rows of up; the epilogue applies the
//                    clamped SwiGLU and the routing weight and stores f32 mid rows;
//   down:            f32 partial rows, one per (token, slot).
// One v_mfma_i32_16x16x32_i8 is exactly one Q8_0 block of a 16 x 16 fragment; its int32 sums
// are folded into the f32 accumulators with f16(d_w) * xscale, as in q8_0_row_partial.
// Operands are fetched in memory order by LDS-direct loads (see lds_dma16) in chunks of 4
// blocks (128 k), double buffered: the weights into a region private to the wave, the
// activations (and their scales) shared; 16-byte units are XOR-swizzled with the row so
// that the 8-byte operand reads spread over the banks.  The extra expert (index n_expert,
// slot n_used) like in the MXFP4 GEMM.
// LDS: B[2][16 KB] | xs[2][2 KB] | A[4 waves][M][2][2 KB] | dw[M][64 rows][n_blocks] f16,
// M = 2 matrices for PAIR, else 1.
// ---------------------------------------------------------------------------------------
constexpr int kQgWaves = 4;
constexpr int kQgCols = 128;
constexpr int kQgRows = 64;
constexpr uint32_t kQgBOff = 0, kQgXsOff = 2 * 16384, kQgAOff = kQgXsOff + 2 * 2048;

struct Q8GemmParams {
    float *out;                    // PAIR: f32 mid [dest rows, n_rows]; else partials [dest rows, n_rows]
    const uint8_t *w0, *w1;        // [n_expert] experts: gate and up, or down in w0
    const uint8_t *sh_w0, *sh_w1;  // the extra expert, or null
    uint64_t bpe0, bpe1;
    const uint8_t *act;            // Q8_0 activation rows, act_row_bytes apart: by token (PAIR) or dest row
    const float *ew;               // [n_tokens, n_used]   (PAIR)
    const int32_t *group_count, *group_offset, *members, *work_items, *n_work_items;
    uint32_t n_tokens, n_used, n_expert, n_rows, n_blocks, act_row_bytes, n_row_tiles;
    float clamp, sh_clamp;
};

// columns (double buffered) | activation scales | the waves' weight chunks (double buffered) | the
// rows' block scales of two chunks at a time (double buffered): 72 KB with both matrices, so that
// two workgroups share a CU
inline size_t q8_0_gemm_lds_bytes(bool pair) {
    const uint32_t m = pair ? 2u : 1u;
    return kQgAOff + (size_t)kQgWaves * m * 4096u + (size_t)2u * m * kQgRows * 16u;
}

typedef int v4i32 __attribute__((ext_vector_type(4)));

template <bool PAIR>
__global__ __launch_bounds__(kQgWaves * 64) void k_q8_0_gemm(const Q8GemmParams p) {
    constexpr uint32_t M = PAIR ? 2u : 1u;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ uint32_t s_dest[kQgCols];
    __shared__ uint32_t s_src[kQgCols];
    __shared__ float s_ew[kQgCols];

    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u;
    const uint32_t g4 = lane >> 4, n16 = lane & 15u;

    // the row tiles of a work item run on one XCD (they share the activations in its L2); the
    // items are dealt to the XCDs like cards, which spreads the wide groups of skewed routing
    const uint32_t xcd = blockIdx.x & 7u, seq = blockIdx.x >> 3;
    const uint32_t n_items = (uint32_t)*p.n_work_items;  // the grid is only an upper bound
    const uint32_t local = seq / p.n_row_tiles;
    // Many column tiles per expert (skewed routing, many tokens): the items are dealt to the XCDs
    // like cards, which spreads the wide groups -- contiguous ranges of the list (it is by expert)
    // left the busiest XCD with 17 % more column groups than the average at Zipf-skewed routing,
    // against 8 % (layer at T=4096: -4.6 %).  About a tile per expert: contiguous ranges, so that
    // an XCD streams one contiguous stretch of the weights (3-5 % faster then).
    const bool deal = n_items > p.n_expert + (p.n_expert >> 1);
    if (!deal && local >= (n_items + 7u) / 8u) return;  // uniform
    const uint32_t item = deal ? local * 8u + xcd : xcd * ((n_items + 7u) / 8u) + local;
    const uint32_t rt = seq % p.n_row_tiles;
    if (item >= n_items) return;

    const uint32_t wi = (uint32_t)p.work_items[item];
    const uint32_t e = wi >> 16, start = wi & 0xFFFFu;
    const uint32_t cnt = min((uint32_t)kQgCols, (uint32_t)p.group_count[e] - start);
    const uint32_t mbase = (uint32_t)p.group_offset[e] + start;
    const bool extra = e >= p.n_expert;
    if (tid < (uint32_t)kQgCols) {
        // columns past the end of the group repeat its last member; they are never stored
        const uint32_t m = (uint32_t)p.members[mbase + min(tid, cnt - 1u)];
        const uint32_t t = m >> 16, slot = m & 0xFFFFu;
        const uint32_t dest = slot >= p.n_used ? p.n_tokens * p.n_used + t : t * p.n_used + slot;
        s_dest[tid] = dest;
        s_src[tid] = PAIR ? t : dest;
        if (PAIR) s_ew[tid] = slot >= p.n_used ? 1.0f : p.ew[dest];
    }
    const uint32_t nb = p.n_blocks, row_bytes = nb * 34u;
    const uint8_t *wbase[M];
    wbase[0] = (extra ? p.sh_w0 : p.w0 + (uint64_t)e * p.bpe0) + (uint64_t)(rt * kQgRows) * row_bytes;
    if (PAIR) wbase[M - 1] = (extra ? p.sh_w1 : p.w1 + (uint64_t)e * p.bpe1) + (uint64_t)(rt * kQgRows) * row_bytes;

    // the rows' block scales travel with the chunks: 16 bytes per row hold the scales of two chunks
    // (8 blocks), fetched by one instruction per matrix every other chunk (wave mm: lane -> row)
    const uint32_t dw_off = kQgAOff + kQgWaves * M * 4096u;
    const uint8_t *s_dw = smem + dw_off;   // [buffer][matrix][row][16 B]
    __syncthreads();  // s_src visible

    const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
    const uint32_t l8 = lane >> 3, c8 = (lane & 7u) ^ l8;
    // A: wave w, matrix mm, rows 16 w + 8 i + l8, 16-byte unit c8 of the chunk's 128 bytes
    const uint32_t a_lds = __builtin_amdgcn_readfirstlane(lds0 + kQgAOff + wave * M * 4096u);
    const uint32_t a_fetch = (wave * 16u + l8) * row_bytes + nb * 2u + c8 * 16u;
    // B: wave w fetches columns 32 w + 8 ii + l8
    const uint32_t b_lds = __builtin_amdgcn_readfirstlane(lds0 + kQgBOff + wave * 4096u);
    uint32_t b_fetch[4];
#pragma unroll
    for (int ii = 0; ii < 4; ii++)
        b_fetch[ii] = s_src[wave * 32u + ii * 8u + l8] * p.act_row_bytes + c8 * 16u;
    // activation scales: waves 0 and 1, lane -> column 64 w + lane, the chunk's 4 floats
    const uint32_t xs_lds = __builtin_amdgcn_readfirstlane(lds0 + kQgXsOff + (wave & 1u) * 1024u);
    const uint32_t dw_lds = __builtin_amdgcn_readfirstlane(lds0 + dw_off);
    const uint32_t wave_u = __builtin_amdgcn_readfirstlane(wave);
    const uint8_t *dw_base = (M == 2u && wave_u == 1u) ? wbase[M - 1] : wbase[0];   // wave mm fetches matrix mm's
    const uint32_t xs_fetch = s_src[(wave & 1u) * 64u + lane] * p.act_row_bytes + nb * 32u;
    const bool b_live = wave * 32u < cnt;
    auto issue = [&](uint32_t c, uint32_t buf) {
#pragma unroll
        for (uint32_t mm = 0; mm < M; mm++)
#pragma unroll
            for (int i = 0; i < 2; i++)
                lds_dma16(a_lds + mm * 4096u + buf * 2048u + (uint32_t)i * 1024u, wbase[mm],
                          a_fetch + (uint32_t)i * 8u * row_bytes + c * 128u);
        if (b_live) {
#pragma unroll
            for (int ii = 0; ii < 4; ii++)
                lds_dma16(b_lds + buf * 16384u + (uint32_t)ii * 1024u, p.act, b_fetch[ii] + c * 128u);
        }
        if (wave < 2u) lds_dma16(xs_lds + buf * 2048u, p.act, xs_fetch + c * 16u);
        // (a last, single chunk reads 8 bytes past the scales, into the row's own quants)
        if ((c & 1u) == 0u && wave_u < M)
            lds_dma16(dw_lds + ((c >> 1) & 1u) * (M * kQgRows * 16u) + wave_u * (kQgRows * 16u), dw_base,
                      lane * row_bytes + (c >> 1) * 16u);
    };

    // read side: lane (row / column n16, 8-byte piece g4 of a block's 32 bytes)
    const uint32_t rd = (n16 >> 3) * 1024u + (n16 & 7u) * 128u + (g4 & 1u) * 8u;
    const uint32_t rd_sw = n16 & 7u, rd_unit = g4 >> 1;
    const uint8_t *a_ptr = smem + kQgAOff + wave * M * 4096u;

    float acc[M][8][4];
#pragma unroll
    for (uint32_t mm = 0; mm < M; mm++)
#pragma unroll
        for (int j = 0; j < 8; j++)
#pragma unroll
            for (int q = 0; q < 4; q++) acc[mm][j][q] = 0.0f;

    const uint32_t n_chunks = nb / 4u;
    const uint32_t nj = (cnt + 15u) / 16u;
    issue(0, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    for (uint32_t c = 0; c < n_chunks; c++) {
        const uint32_t buf = c & 1u;
        if (c + 1u < n_chunks) issue(c + 1u, buf ^ 1u);
        const uint8_t *bb = smem + kQgBOff + buf * 16384u;
        const uint8_t *xb = smem + kQgXsOff + buf * 2048u;
        // the lane's 4 rows' scales of the chunk's 4 blocks, and its A operands
        float dw[M][4][4];
        long av[M][4];
#pragma unroll
        for (uint32_t mm = 0; mm < M; mm++) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const uint2 h = *(const uint2 *)(s_dw + ((size_t)((c >> 1) & 1u) * M + mm) * (kQgRows * 16u) +
                                                 (size_t)(wave * 16u + g4 * 4u + q) * 16u + (c & 1u) * 8u);
                dw[mm][q][0] = __half2float(__ushort_as_half((uint16_t)(h.x & 0xFFFFu)));
                dw[mm][q][1] = __half2float(__ushort_as_half((uint16_t)(h.x >> 16)));
                dw[mm][q][2] = __half2float(__ushort_as_half((uint16_t)(h.y & 0xFFFFu)));
                dw[mm][q][3] = __half2float(__ushort_as_half((uint16_t)(h.y >> 16)));
            }
            const uint8_t *ab = a_ptr + mm * 4096u + buf * 2048u;
#pragma unroll
            for (int b = 0; b < 4; b++)
                av[mm][b] = *(const long *)(ab + rd + (((uint32_t)(2 * b) + rd_unit) ^ rd_sw) * 16u);
        }
#pragma unroll
        for (int j = 0; j < 8; j++) {
            if ((uint32_t)j < nj) {  // uniform
                const float4 xs = *(const float4 *)(xb + (size_t)(j * 16u + n16) * 16u);
                const float xsv[4] = {xs.x, xs.y, xs.z, xs.w};
                const uint8_t *bj = bb + (size_t)j * 2048u + rd;
#pragma unroll
                for (int b = 0; b < 4; b++) {
                    const long bv = *(const long *)(bj + (((uint32_t)(2 * b) + rd_unit) ^ rd_sw) * 16u);
#pragma unroll
                    for (uint32_t mm = 0; mm < M; mm++) {
                        const v4i32 s = __builtin_amdgcn_mfma_i32_16x16x32_i8(av[mm][b], bv, v4i32{0, 0, 0, 0}, 0, 0, 0);
                        // three vector instructions per value: scale product, convert, fused add
                        acc[mm][j][0] = fmaf(dw[mm][0][b] * xsv[b], (float)s.x, acc[mm][j][0]);
                        acc[mm][j][1] = fmaf(dw[mm][1][b] * xsv[b], (float)s.y, acc[mm][j][1]);
                        acc[mm][j][2] = fmaf(dw[mm][2][b] * xsv[b], (float)s.z, acc[mm][j][2]);
                        acc[mm][j][3] = fmaf(dw[mm][3][b] * xsv[b], (float)s.w, acc[mm][j][3]);
                    }
                }
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    }

    // the lane holds rows 16 w + 4 g4 + q of columns 16 j + n16
    const float clamp = extra ? p.sh_clamp : p.clamp;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const uint32_t col = j * 16u + n16;
        if (col >= cnt) continue;
        float *dst = p.out + (uint64_t)s_dest[col] * p.n_rows + rt * kQgRows + wave * 16u + g4 * 4u;
        if (PAIR) {
            const float ew = s_ew[col];
            *(float4 *)dst = make_float4(swiglu_clamp(acc[0][j][0], acc[M - 1][j][0], clamp, ew),
                                         swiglu_clamp(acc[0][j][1], acc[M - 1][j][1], clamp, ew),
                                         swiglu_clamp(acc[0][j][2], acc[M - 1][j][2], clamp, ew),
                                         swiglu_clamp(acc[0][j][3], acc[M - 1][j][3], clamp, ew));
        } else {
            *(float4 *)dst = make_float4(acc[0][j][0], acc[0][j][1], acc[0][j][2], acc[0][j][3]);
        }
    }
}

// Raised once per device by the library's set-up, with the device current.
inline void q8_0_gemm_raise_lds_limits() {
    (void)hipFuncSetAttribute((const void *)k_q8_0_gemm<true>, hipFuncAttributeMaxDynamicSharedMemorySize, 80 * 1024);
    (void)hipFuncSetAttribute((const void *)k_q8_0_gemm<false>, hipFuncAttributeMaxDynamicSharedMemorySize, 80 * 1024);
}

template <bool PAIR>
inline int q8_0_gemm(hipStream_t st, const Q8GemmParams &p, uint32_t max_wi) {
    if (max_wi == 0) return DSX_OK;
    if (p.n_rows % kQgRows || p.n_blocks % 4 || p.n_blocks == 0)
        return q8_0_fail(DSX_ERR_SHAPE, "q8_0 gemm", "n_rows must be a multiple of 64, k of 128");
    const uint64_t act_rows = (uint64_t)p.n_tokens * (p.n_used + 1u);
    if ((uint64_t)p.n_rows * p.n_blocks * 34u > 0xFFFFFFFFull || act_rows * p.act_row_bytes > 0xFFFFFFFFull)
        return q8_0_fail(DSX_ERR_INVALID_ARG, "q8_0 gemm", "a weight matrix or the activation rows exceed 4 GiB");
    const size_t lds = q8_0_gemm_lds_bytes(PAIR);
    const uint32_t per_xcd = (max_wi + 7u) / 8u;
    const uint64_t grid = (uint64_t)8u * per_xcd * p.n_row_tiles;
    if (grid > 0x7FFFFFFFull) return q8_0_fail(DSX_ERR_INVALID_ARG, "q8_0 gemm", "grid too large");
    hipLaunchKernelGGL(k_q8_0_gemm<PAIR>, dim3((uint32_t)grid), dim3(kQgWaves * 64), lds, st, p);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? DSX_OK : q8_0_fail((int)e, "q8_0 gemm", hipGetErrorString(e));
}

}  // namespace dsx
