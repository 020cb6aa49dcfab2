// dsx_expert_kernels.hpp -- MXFP4 expert products on gfx950 (gate/up + SwiGLU, down).
//
// One workgroup computes a 16-row tile of one expert for up to NT token columns.  The
// workgroup's waves split the k dimension by super-block (wave w takes super-blocks
// w, w + W, ...), each accumulating in registers, and the partial sums are added through
// LDS in wave order, so results do not depend on scheduling.
//
// Two ways to name the tokens of a tile:
//   decode    one token; grid.y = slot; expert = selected[slot]
//             (crates/v4flash-kernels/kernels/mxfp4_pair_matvec.hip:200-229,
//              mxfp4_matvec.hip:120-155)
//   by-expert grid.y = work item (expert << 16 | first member); columns = the next
//             `chunk` members (token << 16 | slot) of that expert
//             (crates/v4flash-kernels/kernels/mxfp4_pair_matvec.hip:395-564,
//              mxfp4_matvec.hip:219-427)
#pragma once

#include "dsx_device.hpp"

namespace dsx {

constexpr int kGuWaves = 4;  // waves per gate/up workgroup
#define DSX_MAX_SLOTS 17     // n_used <= 16 picks + the shared expert

struct GateUpParams {
    float *mid;            // decode: [n_slots, n_rows]; by-expert: [b * n_used, n_rows]
    const uint8_t *gate;   // [n_expert] experts, stride gbpe
    const uint8_t *up;
    const uint8_t *xq;     // decode: one Q8_K row; by-expert: [b] rows of xq_row_bytes
    const float *ew;       // decode: [n_used]; by-expert: [b * n_used]
    const int32_t *selected;  // decode only: [n_used]
    const uint8_t *sh_gate;   // decode only: extra slot n_used (weight 1), or null
    const uint8_t *sh_up;
    const int32_t *group_count, *group_offset, *members, *work_items, *n_work_items;
    uint64_t gbpe, ubpe;
    uint32_t n_used, chunk;
    float clamp, sh_clamp;
    uint32_t n_rows, n_blocks, xq_row_bytes;
};

// LDS: [n_blocks] tiles of 512 * NT bytes | yd[n_blocks * NT] floats
template <int NT, bool BY_EXPERT>
__global__ __launch_bounds__(kGuWaves * 64) void k_mxfp4_gate_up(const GateUpParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ float s_red[kGuWaves][2][4][64];
    __shared__ int s_dest[NT];
    __shared__ float s_ew[NT];
    __shared__ uint32_t s_tok[NT];

    uint8_t *tiles = smem;
    float *s_yd = (float *)(smem + (size_t)p.n_blocks * 512u * NT);

    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u;
    const uint32_t row0 = blockIdx.x * 16u;
    const uint32_t item = blockIdx.y;

    // ---- which expert, which columns -------------------------------------------------
    const uint8_t *gate_e, *up_e;
    uint32_t cnt;
    float clamp = p.clamp;
    if (BY_EXPERT) {
        if ((int)item >= *p.n_work_items) return;  // uniform: grid is an upper bound
        const uint32_t wi = (uint32_t)p.work_items[item];
        const uint32_t e = wi >> 16, start = wi & 0xFFFFu;
        const uint32_t total = (uint32_t)p.group_count[e];
        cnt = min(p.chunk, total - start);
        if (cnt > (uint32_t)NT) cnt = NT;
        const uint32_t mbase = (uint32_t)p.group_offset[e] + start;
        if (tid < cnt) {
            const uint32_t m = (uint32_t)p.members[mbase + tid];
            const uint32_t t = m >> 16, slot = m & 0xFFFFu;
            s_tok[tid] = t;
            s_dest[tid] = (int)(t * p.n_used + slot);
            s_ew[tid] = p.ew[t * p.n_used + slot];
        }
        gate_e = p.gate + (uint64_t)e * p.gbpe;
        up_e = p.up + (uint64_t)e * p.ubpe;
    } else {
        cnt = 1;
        if (item < p.n_used) {
            const int e = p.selected[item];
            if (e < 0) {  // empty slot: defined output, nothing to compute
                if (tid < 16) p.mid[(uint64_t)item * p.n_rows + row0 + tid] = 0.0f;
                return;
            }
            gate_e = p.gate + (uint64_t)e * p.gbpe;
            up_e = p.up + (uint64_t)e * p.ubpe;
            if (tid == 0) s_ew[0] = p.ew[item];
        } else {
            gate_e = p.sh_gate;
            up_e = p.sh_up;
            clamp = p.sh_clamp;
            if (tid == 0) s_ew[0] = 1.0f;
        }
        if (tid == 0) {
            s_tok[0] = 0;
            s_dest[0] = (int)item;
        }
    }

    // ---- first weight loads go out before the activations are staged ----------------
    const uint32_t r = lane & 15u, kb = lane >> 4;
    const uint64_t row_stride = (uint64_t)p.n_blocks * kSuperBytes;
    const uint8_t *grow = gate_e + (uint64_t)(row0 + r) * row_stride;
    const uint8_t *urow = up_e + (uint64_t)(row0 + r) * row_stride;
    uint32_t sb = wave;
    WSuper g = {}, u = {};
    if (sb < p.n_blocks) {
        g = load_wsuper(grow + (uint64_t)sb * kSuperBytes, kb);
        u = load_wsuper(urow + (uint64_t)sb * kSuperBytes, kb);
    }

    if (BY_EXPERT) __syncthreads();  // s_tok visible
    for (uint32_t pr = wave; pr < cnt * p.n_blocks; pr += kGuWaves) {
        const uint32_t j = pr / p.n_blocks, b = pr - j * p.n_blocks;
        const uint32_t tok = BY_EXPERT ? s_tok[j] : 0u;
        const uint8_t *blk = p.xq + (uint64_t)tok * p.xq_row_bytes + (uint64_t)b * kQ8kBytes;
        stage_q8k_block<NT>(tiles + (size_t)b * 512u * NT, s_yd + b * NT + j, blk, j, lane);
    }
    __syncthreads();

    // ---- k loop ---------------------------------------------------------------------
    const uint32_t n = lane & 15u;
    const uint32_t col = (n < cnt) ? n : 0u;
    v4f acc_g = {0.f, 0.f, 0.f, 0.f}, acc_u = {0.f, 0.f, 0.f, 0.f};
    for (; sb < p.n_blocks; sb += kGuWaves) {
        WSuper gn = g, un = u;
        const uint32_t nsb = sb + kGuWaves;
        if (nsb < p.n_blocks) {
            gn = load_wsuper(grow + (uint64_t)nsb * kSuperBytes, kb);
            un = load_wsuper(urow + (uint64_t)nsb * kSuperBytes, kb);
        }
        const uint8_t *tile = tiles + (size_t)sb * 512u * NT;
        const BSuper bs = load_bsuper<NT>(tile, kb, col);
        const float yd = s_yd[sb * NT + col];
        mfma_super(acc_g, g, bs, yd, kb);
        mfma_super(acc_u, u, bs, yd, kb);
        g = gn;
        u = un;
    }

    // ---- add the waves' partial sums in wave order, SwiGLU, store --------------------
    s_red[wave][0][0][lane] = acc_g.x;
    s_red[wave][0][1][lane] = acc_g.y;
    s_red[wave][0][2][lane] = acc_g.z;
    s_red[wave][0][3][lane] = acc_g.w;
    s_red[wave][1][0][lane] = acc_u.x;
    s_red[wave][1][1][lane] = acc_u.y;
    s_red[wave][1][2][lane] = acc_u.z;
    s_red[wave][1][3][lane] = acc_u.w;
    __syncthreads();
    if (tid < 16u * cnt) {
        const uint32_t rr = tid & 15u, j = tid >> 4;
        const uint32_t l = (rr >> 2) * 16u + j, i = rr & 3u;  // C layout: row 4*(l/16)+i, col l%16
        float gs = 0.0f, us = 0.0f;
#pragma unroll
        for (int w = 0; w < kGuWaves; w++) {
            gs += s_red[w][0][i][l];
            us += s_red[w][1][i][l];
        }
        p.mid[(uint64_t)s_dest[j] * p.n_rows + row0 + rr] = swiglu_clamp(gs, us, clamp, s_ew[j]);
    }
}

// ---------------------------------------------------------------------------------------
// down, decode: out[row] = sum over slots of down_e[row] . midq[slot].
// The (slot, super-block) pairs of the tile are dealt round-robin to the waves.
// ---------------------------------------------------------------------------------------
constexpr int kDownWaves = 8;

struct DownDecodeParams {
    float *out;             // [n_rows]
    const uint8_t *down;    // [n_expert] experts, stride dbpe
    const uint8_t *xq;      // slot-major Q8_K, xq_slot_stride bytes per slot
    const int32_t *selected;  // [n_used]
    const uint8_t *sh_down;   // extra slot n_used, or null
    uint64_t dbpe;
    uint32_t xq_slot_stride, n_used, n_slots, n_rows, n_blocks_in;
};

// LDS: [n_slots * n_blocks_in] tiles of 512 bytes | yd[n_slots * n_blocks_in]
__global__ __launch_bounds__(kDownWaves * 64) void k_mxfp4_down_decode(const DownDecodeParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ float s_red[kDownWaves][4][64];
    __shared__ int s_sel[DSX_MAX_SLOTS];

    const uint32_t units = p.n_slots * p.n_blocks_in;
    uint8_t *tiles = smem;
    float *s_yd = (float *)(smem + (size_t)units * 512u);

    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u;
    const uint32_t row0 = blockIdx.x * 16u;
    const uint32_t r = lane & 15u, kb = lane >> 4;
    const uint64_t row_off = (uint64_t)(row0 + r) * p.n_blocks_in * kSuperBytes;

    auto unit_ptr = [&](uint32_t un) -> const uint8_t * {
        const uint32_t slot = un / p.n_blocks_in, b = un - slot * p.n_blocks_in;
        const int e = (slot < p.n_used) ? p.selected[slot] : 0;
        const uint8_t *base = (slot < p.n_used) ? p.down + (uint64_t)(e < 0 ? 0 : e) * p.dbpe
                                                : p.sh_down;
        return base + row_off + (uint64_t)b * kSuperBytes;
    };

    uint32_t un = wave;
    WSuper w = {};
    if (un < units) w = load_wsuper(unit_ptr(un), kb);

    if (tid < p.n_slots) s_sel[tid] = (tid < p.n_used) ? p.selected[tid] : 0;
    for (uint32_t pr = wave; pr < units; pr += kDownWaves) {
        const uint32_t slot = pr / p.n_blocks_in, b = pr - slot * p.n_blocks_in;
        const uint8_t *blk = p.xq + (uint64_t)slot * p.xq_slot_stride + (uint64_t)b * kQ8kBytes;
        stage_q8k_block<1>(tiles + (size_t)pr * 512u, s_yd + pr, blk, 0, lane);
    }
    __syncthreads();

    v4f acc = {0.f, 0.f, 0.f, 0.f};
    for (; un < units; un += kDownWaves) {
        WSuper wn = w;
        const uint32_t nun = un + kDownWaves;
        if (nun < units) wn = load_wsuper(unit_ptr(nun), kb);
        const uint32_t slot = un / p.n_blocks_in;
        if (s_sel[slot] >= 0) {  // uniform per wave
            const BSuper bs = load_bsuper<1>(tiles + (size_t)un * 512u, kb, 0);
            mfma_super(acc, w, bs, s_yd[un], kb);
        }
        w = wn;
    }

    s_red[wave][0][lane] = acc.x;
    s_red[wave][1][lane] = acc.y;
    s_red[wave][2][lane] = acc.z;
    s_red[wave][3][lane] = acc.w;
    __syncthreads();
    if (tid < 16u) {
        const uint32_t l = (tid >> 2) * 16u, i = tid & 3u;
        float s = 0.0f;
#pragma unroll
        for (int wv = 0; wv < kDownWaves; wv++) s += s_red[wv][i][l];
        p.out[row0 + tid] = s;
    }
}

// ---------------------------------------------------------------------------------------
// down, by-expert: partials[(t * n_used + slot) * n_rows + row] = down_e[row] . midq[t, slot]
// ---------------------------------------------------------------------------------------
constexpr int kDownBeWaves = 4;

struct DownByExpertParams {
    float *partials;
    const uint8_t *down;
    const uint8_t *xq;  // [b * n_used] rows of xq_slot_stride bytes
    const int32_t *group_count, *group_offset, *members, *work_items, *n_work_items;
    uint64_t dbpe;
    uint32_t xq_slot_stride, n_used, chunk, n_rows, n_blocks_in;
};

// LDS: [n_blocks_in] tiles of 512 * NT bytes | yd[n_blocks_in * NT]
template <int NT>
__global__ __launch_bounds__(kDownBeWaves * 64) void k_mxfp4_down_by_expert(
    const DownByExpertParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ float s_red[kDownBeWaves][4][64];
    __shared__ int s_dest[NT];

    uint8_t *tiles = smem;
    float *s_yd = (float *)(smem + (size_t)p.n_blocks_in * 512u * NT);

    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u;
    const uint32_t row0 = blockIdx.x * 16u;
    const uint32_t item = blockIdx.y;
    if ((int)item >= *p.n_work_items) return;
    const uint32_t wi = (uint32_t)p.work_items[item];
    const uint32_t e = wi >> 16, start = wi & 0xFFFFu;
    uint32_t cnt = min(p.chunk, (uint32_t)p.group_count[e] - start);
    if (cnt > (uint32_t)NT) cnt = NT;
    const uint32_t mbase = (uint32_t)p.group_offset[e] + start;
    if (tid < cnt) {
        const uint32_t m = (uint32_t)p.members[mbase + tid];
        s_dest[tid] = (int)((m >> 16) * p.n_used + (m & 0xFFFFu));
    }

    const uint32_t r = lane & 15u, kb = lane >> 4;
    const uint8_t *wrow = p.down + (uint64_t)e * p.dbpe +
                          (uint64_t)(row0 + r) * p.n_blocks_in * kSuperBytes;
    uint32_t sb = wave;
    WSuper w = {};
    if (sb < p.n_blocks_in) w = load_wsuper(wrow + (uint64_t)sb * kSuperBytes, kb);

    __syncthreads();
    for (uint32_t pr = wave; pr < cnt * p.n_blocks_in; pr += kDownBeWaves) {
        const uint32_t j = pr / p.n_blocks_in, b = pr - j * p.n_blocks_in;
        const uint8_t *blk = p.xq + (uint64_t)s_dest[j] * p.xq_slot_stride + (uint64_t)b * kQ8kBytes;
        stage_q8k_block<NT>(tiles + (size_t)b * 512u * NT, s_yd + b * NT + j, blk, j, lane);
    }
    __syncthreads();

    const uint32_t n = lane & 15u;
    const uint32_t col = (n < cnt) ? n : 0u;
    v4f acc = {0.f, 0.f, 0.f, 0.f};
    for (; sb < p.n_blocks_in; sb += kDownBeWaves) {
        WSuper wn = w;
        const uint32_t nsb = sb + kDownBeWaves;
        if (nsb < p.n_blocks_in) wn = load_wsuper(wrow + (uint64_t)nsb * kSuperBytes, kb);
        const BSuper bs = load_bsuper<NT>(tiles + (size_t)sb * 512u * NT, kb, col);
        mfma_super(acc, w, bs, s_yd[sb * NT + col], kb);
        w = wn;
    }

    s_red[wave][0][lane] = acc.x;
    s_red[wave][1][lane] = acc.y;
    s_red[wave][2][lane] = acc.z;
    s_red[wave][3][lane] = acc.w;
    __syncthreads();
    if (tid < 16u * cnt) {
        const uint32_t rr = tid & 15u, j = tid >> 4;
        const uint32_t l = (rr >> 2) * 16u + j, i = rr & 3u;
        float s = 0.0f;
#pragma unroll
        for (int wv = 0; wv < kDownBeWaves; wv++) s += s_red[wv][i][l];
        p.partials[(uint64_t)s_dest[j] * p.n_rows + row0 + rr] = s;
    }
}

}  // namespace dsx
