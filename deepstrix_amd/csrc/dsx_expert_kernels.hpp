// dsx_expert_kernels.hpp -- MXFP4 expert products on gfx950 (gate/up + SwiGLU, down).
//
// One workgroup computes a 16-row tile of one expert for up to NT token columns.  The
// workgroup's waves split the k dimension by super-block (wave w takes super-blocks
// w, w + W, ...), each accumulating in registers with the next two super-blocks' weights
// already in flight, and the partial sums are added through LDS in wave order, so results
// do not depend on scheduling.
//
// Two ways to name the tokens of a tile:
//   decode    one token; grid.y = slot; expert = selected[slot]
//             (crates/v4flash-kernels/kernels/mxfp4_pair_matvec.hip:200-229,
//              mxfp4_matvec.hip:120-155)
//   by-expert grid.y = work item (expert << 16 | first member); columns = the next
//             `chunk` members (token << 16 | slot) of that expert
//             (crates/v4flash-kernels/kernels/mxfp4_pair_matvec.hip:395-564,
//              mxfp4_matvec.hip:219-427)
//
// Two activation formats:
//   Q8_K rows (the operator ABI)   converted to FP8 planes while they are staged;
//   staged rows (inside the layer) already FP8 planes, produced once by the quantizer:
//             [n_sb][512 B tile][n_sb f32 d], copied to LDS with 128-bit loads.
#pragma once

#include "dsx_device.hpp"
#include "dsx_quant.hpp"

namespace dsx {

constexpr int kGuWaves = 4;  // waves per gate/up workgroup
// mid[] before a result has landed in it (a NaN with every bit set: no sum of products is one)
constexpr uint32_t kMidUnwritten = 0xFFFFFFFFu;
// default bound, in rounds of about a microsecond, of the quantizing wave's wait for the other
// tiles of its block
constexpr uint32_t kMidSpinLimit = 1u << 17;
// codes a kernel leaves in the layer's status word when one of its bounded waits gives up (the
// first one wins; 0 = none did)
constexpr uint32_t kStatusOk = 0u;
constexpr uint32_t kStatusMidWaitExpired = 1u;      // a down item gave up waiting for mid values
constexpr uint32_t kStatusMidqWaitExpired = 2u;     // the fused mid quantization gave up waiting for a tile
constexpr uint32_t kStatusPartialWaitExpired = 3u;  // the slot-order sum gave up waiting for a partial row
#define DSX_MAX_SLOTS 17     // n_used <= 16 picks + the shared expert

// Bytes of one staged activation row of n_sb super-blocks (16-byte aligned).
__host__ __device__ inline uint32_t staged_row_bytes(uint32_t n_sb) {
    return (n_sb * 516u + 15u) & ~15u;
}

// Copies staged tiles into LDS.  The workgroup's tile list is `n_cols` columns of `nb`
// tiles each: column j reads the staged row `row(j)`; its tile b lands in LDS tile
// `lds_base(j) + b`, column `lds_col(j)`.  All threads take part with 128-bit loads, four
// in flight per thread.
struct StageDecode {  // one row, one column (the token of a decode step)
    const uint8_t *base;
    __device__ __forceinline__ const uint8_t *row(uint32_t) const { return base; }
    __device__ __forceinline__ uint32_t lds_base(uint32_t) const { return 0u; }
    __device__ __forceinline__ uint32_t lds_col(uint32_t) const { return 0u; }
};
struct StageSlots {  // down, decode: row j = slot j, its tiles at LDS tiles j*nb.., column 0
    const uint8_t *base;
    uint32_t stride, nb;
    __device__ __forceinline__ const uint8_t *row(uint32_t j) const { return base + (uint64_t)j * stride; }
    __device__ __forceinline__ uint32_t lds_base(uint32_t j) const { return j * nb; }
    __device__ __forceinline__ uint32_t lds_col(uint32_t) const { return 0u; }
};
struct StageMembers {  // by-expert: row j = rows[idx[j]], LDS tiles 0.., column j
    const uint8_t *base;
    uint32_t stride;
    const uint32_t *idx;  // LDS array
    __device__ __forceinline__ const uint8_t *row(uint32_t j) const { return base + (uint64_t)idx[j] * stride; }
    __device__ __forceinline__ uint32_t lds_base(uint32_t) const { return 0u; }
    __device__ __forceinline__ uint32_t lds_col(uint32_t j) const { return j; }
};

template <int NT, int NTHREADS, typename Src>
__device__ __forceinline__ void stage_copy(uint8_t *tiles, float *s_yd, uint32_t n_cols, uint32_t nb,
                                           uint32_t tid, const Src src) {
    const uint32_t per_col = nb * 32u;          // 16-byte chunks of one row
    const uint32_t total = n_cols * per_col;
    auto ld = [&](uint32_t q) -> uint4 {
        const uint32_t j = q / per_col, c = q - j * per_col;
        return *(const uint4 *)(src.row(j) + (size_t)c * 16u);
    };
    auto st = [&](uint32_t q, const uint4 &v) {
        const uint32_t j = q / per_col, c = q - j * per_col;
        const uint32_t t = src.lds_base(j) + (c >> 5);
        *(uint4 *)(tiles + (size_t)t * 512u * NT + ((c & 31u) * NT + src.lds_col(j)) * 16u) = v;
    };
    for (uint32_t q = tid; q < total; q += 4u * NTHREADS) {
        const uint32_t q1 = q + NTHREADS, q2 = q + 2u * NTHREADS, q3 = q + 3u * NTHREADS;
        uint4 v0 = ld(q), v1 = {}, v2 = {}, v3 = {};
        if (q1 < total) v1 = ld(q1);
        if (q2 < total) v2 = ld(q2);
        if (q3 < total) v3 = ld(q3);
        st(q, v0);
        if (q1 < total) st(q1, v1);
        if (q2 < total) st(q2, v2);
        if (q3 < total) st(q3, v3);
    }
    for (uint32_t t = tid; t < n_cols * nb; t += NTHREADS) {
        const uint32_t j = t / nb, b = t - j * nb;
        s_yd[(src.lds_base(j) + b) * NT + src.lds_col(j)] =
            *((const float *)(src.row(j) + (size_t)nb * 512u) + b);
    }
}

struct GateUpParams {
    float *mid;            // decode: [n_slots, n_rows]; by-expert: [b * n_used, n_rows]
    const uint8_t *gate;   // [n_expert] experts, stride gbpe
    const uint8_t *up;
    const uint8_t *xq;     // activation rows (Q8_K or staged), xq_row_bytes apart
    const float *ew;       // decode: [n_used]; by-expert: [b * n_used]
    const int32_t *selected;  // decode only: [n_used]
    const uint8_t *sh_gate;   // decode only: extra slot n_used (weight 1), or null
    const uint8_t *sh_up;
    const int32_t *group_count, *group_offset, *members, *work_items, *n_work_items;
    // fused quantization of mid (FUSE_MIDQ): staged rows out; mid holds kMidUnwritten on entry
    uint8_t *midp;
    uint32_t *status;      // FUSE_MIDQ: where an expired wait leaves its code (may be null)
    uint32_t spin_limit;   // FUSE_MIDQ: bound of the wait in rounds (0 is read as kMidSpinLimit)
    uint64_t gbpe, ubpe;
    uint32_t n_used, chunk;
    float clamp, sh_clamp;
    uint32_t n_rows, n_blocks, xq_row_bytes, midp_row_bytes;
    // by-expert with the extra expert (index n_expert, slot n_used; its rows follow the
    // n_tokens * n_used routed ones): sh_gate / sh_up / sh_clamp above, and
    uint32_t n_expert, n_tokens;
    // by-expert: a work item of `chunk` members is served by n_sub workgroups along grid.y,
    // NT columns each (0 is read as 1)
    uint32_t n_sub;
    uint32_t planar;  // the matrices are in the planar form (dsx_device.hpp)
};

// LDS: [n_blocks] tiles of 512 * NT bytes | yd[n_blocks * NT] floats
template <int NT, bool BY_EXPERT, bool STAGED, bool FUSE_MIDQ>
__global__ __launch_bounds__(kGuWaves * 64) void k_mxfp4_gate_up(const GateUpParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ float s_red[kGuWaves][2][4][64];
    __shared__ int s_dest[NT];
    __shared__ float s_ew[NT];
    __shared__ uint32_t s_tok[NT];

    uint8_t *tiles = smem;
    float *s_yd = (float *)(smem + (size_t)p.n_blocks * 512u * NT);

    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u;
    // Workgroup ids go round the 8 XCDs: each XCD takes one contiguous eighth of the row tiles (a
    // contiguous stretch of every matrix; a fraction of a microsecond per decode step) -- with
    // the fused mid quantization only when an eighth is whole 256-row blocks, so that a block's
    // last row tile still has the largest workgroup id of the block, which it relies on.
    const uint32_t bx = ((gridDim.x & (FUSE_MIDQ ? 127u : 7u)) == 0u)
                            ? (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3)
                            : blockIdx.x;
    const uint32_t row0 = bx * 16u;
    const uint32_t n_sub = (BY_EXPERT && p.n_sub > 1u) ? p.n_sub : 1u;
    const uint32_t item = blockIdx.y / n_sub;
    const uint32_t col_off = (blockIdx.y - item * n_sub) * (uint32_t)NT;  // first member served here
    // decode from a staged row that one pass of the workgroup covers: loaded before the weights
    const bool early = !BY_EXPERT && STAGED && NT == 1 && p.n_blocks * 32u <= 4u * kGuWaves * 64u;
    uint4 ex0 = {}, ex1 = {}, ex2 = {}, ex3 = {};
    float early_yd = 0.0f;

    // ---- which expert, which columns -------------------------------------------------
    const uint8_t *gate_e, *up_e;
    uint32_t cnt;
    float clamp = p.clamp;
    if (BY_EXPERT) {
        if ((int)item >= *p.n_work_items) return;  // uniform: grid is an upper bound
        const uint32_t wi = (uint32_t)p.work_items[item];
        const uint32_t e = wi >> 16, start = (wi & 0xFFFFu) + col_off;
        const uint32_t total = (uint32_t)p.group_count[e];
        if (start >= total) return;  // uniform: this sub-chunk of the item has no members
        cnt = min(min(p.chunk - col_off, (uint32_t)NT), total - start);
        const uint32_t mbase = (uint32_t)p.group_offset[e] + start;
        const bool extra = p.sh_gate != nullptr && e >= p.n_expert;
        if (tid < cnt) {
            const uint32_t m = (uint32_t)p.members[mbase + tid];
            const uint32_t t = m >> 16, slot = m & 0xFFFFu;
            s_tok[tid] = t;
            s_dest[tid] = (int)(slot >= p.n_used ? p.n_tokens * p.n_used + t : t * p.n_used + slot);
            s_ew[tid] = slot >= p.n_used ? 1.0f : p.ew[t * p.n_used + slot];
        }
        gate_e = extra ? p.sh_gate : p.gate + (uint64_t)e * p.gbpe;
        up_e = extra ? p.sh_up : p.up + (uint64_t)e * p.ubpe;
        if (extra) clamp = p.sh_clamp;
    } else {
        // decode: item = token * n_slots + slot; slot n_used is the extra (shared) expert
        cnt = 1;
        const uint32_t n_slots = p.n_used + (p.sh_gate ? 1u : 0u);
        const uint32_t t = item / n_slots, slot = item - t * n_slots;
        if (STAGED && early) {
            // the token's staged row goes out first: it needs nothing but the token index, and
            // (loads of a wave return in order) it must not queue behind the weights
            const uint8_t *xrow = p.xq + (uint64_t)t * p.xq_row_bytes;
            const uint32_t nq = p.n_blocks * 32u, q = tid, step = kGuWaves * 64u;
            if (q < nq) ex0 = *(const uint4 *)(xrow + (size_t)q * 16u);
            if (q + step < nq) ex1 = *(const uint4 *)(xrow + (size_t)(q + step) * 16u);
            if (q + 2u * step < nq) ex2 = *(const uint4 *)(xrow + (size_t)(q + 2u * step) * 16u);
            if (q + 3u * step < nq) ex3 = *(const uint4 *)(xrow + (size_t)(q + 3u * step) * 16u);
            if (tid < p.n_blocks) early_yd = *((const float *)(xrow + (size_t)p.n_blocks * 512u) + tid);
        }
        if (slot < p.n_used) {
            const int e = p.selected[t * p.n_used + slot];
            if (e < 0) {  // empty slot: defined output, nothing to compute
                if (tid < 16) p.mid[(uint64_t)item * p.n_rows + row0 + tid] = 0.0f;
                if (FUSE_MIDQ && row0 % 256u == 0u && wave == 0) {
                    // the slot's staged row must still be defined: zero tile, d = 0
                    uint8_t *row = p.midp + (uint64_t)item * p.midp_row_bytes;
                    const uint32_t blk = row0 / 256u;
                    *(uint2 *)(row + (size_t)blk * 512u + lane * 8u) = make_uint2(0u, 0u);
                    if (lane == 0) *(float *)(row + (size_t)(p.n_rows / 256u) * 512u + blk * 4u) = 0.0f;
                }
                return;
            }
            gate_e = p.gate + (uint64_t)e * p.gbpe;
            up_e = p.up + (uint64_t)e * p.ubpe;
            if (tid == 0) s_ew[0] = p.ew[t * p.n_used + slot];
        } else {
            gate_e = p.sh_gate;
            up_e = p.sh_up;
            clamp = p.sh_clamp;
            if (tid == 0) s_ew[0] = 1.0f;
        }
        if (tid == 0) {
            s_tok[0] = t;
            s_dest[0] = (int)item;
        }
    }

    // ---- the first two super-blocks of weights go out before anything else -----------
    const uint32_t r = lane & 15u, kb = lane >> 4;
    const uint32_t wstep = w_step(p.planar != 0u);
    const WRow grow = w_row(gate_e, row0 + r, p.n_blocks, p.planar != 0u);
    const WRow urow = w_row(up_e, row0 + r, p.n_blocks, p.planar != 0u);
    uint32_t sb = wave;
    // The first two loads are unconditional as well (a wave without a block of its own reads
    // the row's last one and never uses it), so that the k loop starts from a known count of
    // loads in flight.
    WSuper g0, u0, g1, u1;
    {
        const uint32_t last = p.n_blocks - 1u;
        const uint32_t b0 = sb < last ? sb : last, b1 = sb + kGuWaves < last ? sb + kGuWaves : last;
        g0 = load_wsuper(grow, (uint64_t)(b0) * wstep, kb);
        u0 = load_wsuper(urow, (uint64_t)(b0) * wstep, kb);
        g1 = load_wsuper(grow, (uint64_t)(b1) * wstep, kb);
        u1 = load_wsuper(urow, (uint64_t)(b1) * wstep, kb);
    }

    // ---- activations into LDS -----------------------------------------------------------
    __syncthreads();  // s_tok visible
    if (STAGED && early) {
        // (NT == 1: the row's tile bytes are contiguous in LDS as they are in memory)
        const uint32_t nq = p.n_blocks * 32u, q = tid, step = kGuWaves * 64u;
        if (q < nq) *(uint4 *)(tiles + (size_t)q * 16u) = ex0;
        if (q + step < nq) *(uint4 *)(tiles + (size_t)(q + step) * 16u) = ex1;
        if (q + 2u * step < nq) *(uint4 *)(tiles + (size_t)(q + 2u * step) * 16u) = ex2;
        if (q + 3u * step < nq) *(uint4 *)(tiles + (size_t)(q + 3u * step) * 16u) = ex3;
        if (tid < p.n_blocks) s_yd[tid] = early_yd;
    } else if (STAGED) {
        if (BY_EXPERT)
            stage_copy<NT, kGuWaves * 64>(tiles, s_yd, cnt, p.n_blocks, tid,
                                          StageMembers{p.xq, p.xq_row_bytes, s_tok});
        else
            stage_copy<NT, kGuWaves * 64>(tiles, s_yd, 1u, p.n_blocks, tid,
                                          StageDecode{p.xq + (uint64_t)s_tok[0] * p.xq_row_bytes});
    } else {
        for (uint32_t pr = wave; pr < cnt * p.n_blocks; pr += kGuWaves) {
            const uint32_t j = pr / p.n_blocks, b = pr - j * p.n_blocks;
            const uint32_t tok = s_tok[j];
            const uint8_t *blk = p.xq + (uint64_t)tok * p.xq_row_bytes + (uint64_t)b * kQ8kBytes;
            stage_q8k_block<NT>(tiles + (size_t)b * 512u * NT, s_yd + b * NT + j, blk, j, lane);
        }
    }
    __syncthreads();

    // ---- k loop: two super-blocks of weights in flight per matrix ---------------------
    const uint32_t n = lane & 15u;
    const uint32_t col = (n < cnt) ? n : 0u;
    v4f acc_g = {0.f, 0.f, 0.f, 0.f}, acc_u = {0.f, 0.f, 0.f, 0.f};
    auto compute = [&](uint32_t s, const WSuper &g, const WSuper &u) {
        const BSuper bs = load_bsuper<NT>(tiles + (size_t)s * 512u * NT, kb, col);
        const float yd = s_yd[s * NT + col];
        mfma_super(acc_g, g, bs, yd, kb);
        mfma_super(acc_u, u, bs, yd, kb);
    };
    // Steady state: both refills of an iteration happen, unconditionally, so the count of loads
    // in flight is the same on every path and each wait leaves the younger super-block's loads
    // outstanding (behind a condition the compiler waits for everything at the join).  The empty
    // asm statements keep each refill behind the products that read the registers it overwrites:
    // left alone the compiler moves the refill in front of them, into fresh registers, copies
    // those into place at the end of the iteration and waits for them there -- one super-block
    // in flight instead of two.
#define DSX_AFTER_PRODUCTS() asm volatile("" : "+v"(acc_g), "+v"(acc_u) :: "memory")
#define DSX_PIN() asm volatile("" ::: "memory")
    while (sb + 3 * kGuWaves < p.n_blocks) {
        compute(sb, g0, u0);
        DSX_AFTER_PRODUCTS();
        g0 = load_wsuper(grow, (uint64_t)((sb + 2 * kGuWaves)) * wstep, kb);
        u0 = load_wsuper(urow, (uint64_t)((sb + 2 * kGuWaves)) * wstep, kb);
        DSX_PIN();
        // (the scale bytes of the second pair are not touched before this point either)
        asm volatile("" : "+v"(g1.s.x), "+v"(g1.s.y), "+v"(u1.s.x), "+v"(u1.s.y));
        compute(sb + kGuWaves, g1, u1);
        DSX_AFTER_PRODUCTS();
        g1 = load_wsuper(grow, (uint64_t)((sb + 3 * kGuWaves)) * wstep, kb);
        u1 = load_wsuper(urow, (uint64_t)((sb + 3 * kGuWaves)) * wstep, kb);
        DSX_PIN();
        sb += 2 * kGuWaves;
    }
    // Tail: up to three super-blocks are left for this wave (sb in g0/u0, sb + W in g1/u1, and
    // sb + 2 W still to fetch, into a third pair so that it can be requested first).
    if (sb < p.n_blocks) {
        WSuper g2 = {}, u2 = {};
        const bool third = sb + 2 * kGuWaves < p.n_blocks;
        if (third) {
            g2 = load_wsuper(grow, (uint64_t)((sb + 2 * kGuWaves)) * wstep, kb);
            u2 = load_wsuper(urow, (uint64_t)((sb + 2 * kGuWaves)) * wstep, kb);
        }
        DSX_PIN();
        compute(sb, g0, u0);
        if (sb + kGuWaves < p.n_blocks) compute(sb + kGuWaves, g1, u1);
        if (third) compute(sb + 2 * kGuWaves, g2, u2);
    }
#undef DSX_AFTER_PRODUCTS
#undef DSX_PIN

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
        const float v = swiglu_clamp(gs, us, clamp, s_ew[j]);
        float *dst = p.mid + (uint64_t)s_dest[j] * p.n_rows + row0 + rr;
        if (FUSE_MIDQ)  // written through to memory: another XCD's workgroup will read it (a NaN as
                        // the canonical one, so that no result equals the unwritten pattern)
            __hip_atomic_store(dst, v != v ? __uint_as_float(0x7FC00000u) : v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        else
            *dst = v;
    }

    if (FUSE_MIDQ) {
        // The workgroup of a 256-row block's last row tile quantizes the block of mid into the
        // staged format that down reads.  The sixteen tiles finish in any order, on any XCD
        // (whose L2s are not coherent with each other), so: the mid buffer holds a bit pattern
        // that no product can have (kMidUnwritten, written by the front kernel) wherever no
        // result has landed yet; results are stored write-through; and the quantizing wave reads
        // the block with loads that bypass its L2 until no lane sees the pattern any more.  The
        // other fifteen workgroups do not wait for anything (no store acknowledgement, no
        // counter round trip: 3 us per step at one token).  The tiles it waits for have smaller
        // workgroup ids, so they were dispatched before it and depend on nothing; the spin is
        // bounded all the same.
        const uint32_t nblk = p.n_rows / 256u, blk = row0 / 256u;
        if ((row0 & 255u) != 240u) return;  // uniform
        for (uint32_t j = wave; j < cnt; j += kGuWaves) {
            const float *src = p.mid + (uint64_t)s_dest[j] * p.n_rows + (size_t)blk * 256u + lane * 4u;
            float4 v;
            const uint32_t limit = p.spin_limit ? p.spin_limit : kMidSpinLimit;
            bool complete = false;
            for (uint32_t spin = 0; spin < limit; spin++) {
                v.x = __hip_atomic_load(src + 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                v.y = __hip_atomic_load(src + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                v.z = __hip_atomic_load(src + 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                v.w = __hip_atomic_load(src + 3, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                const bool landed = __float_as_uint(v.x) != kMidUnwritten && __float_as_uint(v.y) != kMidUnwritten &&
                                    __float_as_uint(v.z) != kMidUnwritten && __float_as_uint(v.w) != kMidUnwritten;
                complete = __builtin_amdgcn_ballot_w64(!landed) == 0ull;  // wave-uniform
                if (complete) break;
                __builtin_amdgcn_s_sleep(2);
            }
            if (!complete) {
                // gave up: a defined block (all zero, d = 0) instead of whatever was read, and a
                // code in the status word for the host to find
                v = make_float4(0.f, 0.f, 0.f, 0.f);
                if (lane == 0 && p.status) atomicCAS(p.status, kStatusOk, kStatusMidqWaitExpired);
            }
            uint8_t *row = p.midp + (uint64_t)s_dest[j] * p.midp_row_bytes;
            quantize_block_to_staged(v, lane, row + (size_t)blk * 512u,
                                     (float *)(row + (size_t)nblk * 512u) + blk);
        }
    }
}

// ---------------------------------------------------------------------------------------
// down, decode: out[row] = sum over slots of down_e[row] . midq[slot].
// The (slot, super-block) pairs of the tile are dealt round-robin to the waves.
// ---------------------------------------------------------------------------------------
constexpr int kDownWaves = 8;

struct DownDecodeParams {
    float *out;             // [n_tokens, n_rows]; grid.y = token
    const uint8_t *down;    // [n_expert] experts, stride dbpe
    const uint8_t *xq;      // slot-major activation rows (Q8_K or staged), xq_slot_stride apart
    const int32_t *selected;  // [n_tokens, n_used]
    const uint8_t *sh_down;   // extra slot n_used, or null
    const float *residual;    // [n_tokens, n_rows] added to the result (may alias out), or null
    uint64_t dbpe;
    uint32_t xq_slot_stride, n_used, n_slots, n_rows, n_blocks_in;
    uint32_t rows_per_wg;     // output rows of one workgroup, at most 16: the grid is sized to fill the CUs evenly
    uint32_t planar;          // the matrices are in the planar form (dsx_device.hpp)
};

// LDS: [n_slots * n_blocks_in] tiles of 512 bytes | yd[n_slots * n_blocks_in]
// NU > 0: every wave has exactly NU units (n_slots * n_blocks_in == NU * kDownWaves) and the k loop
// is straight-line code; NU == 0: any shape.
template <bool STAGED, int NU = 0>
__global__ __launch_bounds__(kDownWaves * 64) void k_mxfp4_down_decode(const DownDecodeParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ float s_red[kDownWaves][4][64];
    __shared__ int s_sel[DSX_MAX_SLOTS];

    const uint32_t nb = p.n_blocks_in;
    const uint32_t units = p.n_slots * nb;
    uint8_t *tiles = smem;
    float *s_yd = (float *)(smem + (size_t)units * 512u);

    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    // the wave index in a scalar register: the unit a wave works on is then uniform, and the
    // pick that names its expert comes through the scalar cache instead of a vector load whose
    // wait would also wait for every weight load in flight
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // workgroup ids go round the 8 XCDs: each XCD takes one contiguous eighth of the row tiles
    const uint32_t bx = (gridDim.x & 7u) == 0u ? (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3)
                                                : blockIdx.x;
    const uint32_t row0 = bx * p.rows_per_wg;
    const uint32_t r = lane & 15u, kb = lane >> 4;
    // rows of the 16-row fragment past the workgroup's share (or the matrix) repeat its last
    // row: every lane loads, so no load sits behind a condition, and their sums are not stored
    const uint32_t n_live = min(p.rows_per_wg, p.n_rows - row0);
    // the lane's row inside a matrix: offsets of its nibble blocks and of its scales
    const bool planar = p.planar != 0u;
    const uint32_t wstep = w_step(planar);
    const uint32_t wrow_i = row0 + min(r, n_live - 1u);
    uint64_t row_off, sc_off;
    w_row_offsets(wrow_i, nb, planar, row_off, sc_off);
    // blockIdx.y = token: its picks, its n_slots activation rows, its output row
    const int32_t *selected = p.selected + (uint64_t)blockIdx.y * p.n_used;
    const uint8_t *xq = p.xq + (uint64_t)blockIdx.y * p.n_slots * p.xq_slot_stride;
    float *out = p.out + (uint64_t)blockIdx.y * p.n_rows;

    // the part of a unit's address that is the same for every lane
    auto unit_base = [&](uint32_t un) -> const uint8_t * {
        const uint32_t slot = un / nb, b = un - slot * nb;
        const int e = (slot < p.n_used) ? selected[slot] : 0;
        const uint8_t *base = (slot < p.n_used) ? p.down + (uint64_t)(e < 0 ? 0 : e) * p.dbpe
                                                : p.sh_down;
        return base + (uint64_t)b * wstep;
    };
    auto unit_w = [&](const uint8_t *ub) -> WRow { return WRow{ub + row_off, ub + sc_off}; };
    // With a fixed unit count the addresses of the later units are worked out here, while the
    // picks can still be read through the scalar cache (after the first asm statement below the
    // compiler reads them with vector loads, and waiting for one of those waits for every
    // weight load in flight).
    const uint8_t *later[NU > 5 ? NU - 5 : 1];
#pragma unroll
    for (int i = 0; i + 5 < NU; i++) later[i] = unit_base(wave + (uint32_t)(i + 5) * kDownWaves);

    // The activation rows go out first when five loads per thread cover them: they need only
    // the token index, and (a wave's loads return in order) must not queue behind the weights.
    const uint32_t per_slot = nb * 32u;                 // 16-byte pieces of one slot's tiles
    const uint32_t n_pieces = p.n_slots * per_slot;
    constexpr uint32_t kStep = kDownWaves * 64u;
    const bool early = STAGED && n_pieces <= 5u * kStep && units <= kStep;
    uint4 ex0 = {}, ex1 = {}, ex2 = {}, ex3 = {}, ex4 = {};
    float early_yd = 0.0f;
    // this thread's entry of the pick table in LDS (n_used >= 1), requested before the weights:
    // a wave's loads return in order, so waiting for it later would wait for them as well
    const int sel_mine = selected[min(tid, p.n_used - 1u)];
    auto piece_src = [&](uint32_t q) -> const uint8_t * {
        const uint32_t j = q / per_slot, c = q - j * per_slot;
        return xq + (uint64_t)j * p.xq_slot_stride + (size_t)c * 16u;
    };
    if (early) {
        // (indices past the end repeat the last piece: loads without a condition keep the
        // count of loads in flight the same on every path, so later waits can be exact)
        const uint32_t lastq = n_pieces - 1u;
        ex0 = *(const uint4 *)piece_src(min(tid, lastq));
        ex1 = *(const uint4 *)piece_src(min(tid + kStep, lastq));
        ex2 = *(const uint4 *)piece_src(min(tid + 2u * kStep, lastq));
        ex3 = *(const uint4 *)piece_src(min(tid + 3u * kStep, lastq));
        ex4 = *(const uint4 *)piece_src(min(tid + 4u * kStep, lastq));
        {
            const uint32_t t = min(tid, units - 1u);
            const uint32_t j = t / nb, bq = t - j * nb;
            early_yd = *((const float *)(xq + (uint64_t)j * p.xq_slot_stride + (size_t)nb * 512u) + bq);
        }
    }

    // five (slot, super-block) units of weights in flight per wave
    uint32_t un = wave;
    WSuper w0 = {}, w1 = {}, w2 = {}, w3 = {}, w4 = {};
    if (NU > 0) {
        w0 = load_wsuper(unit_w(unit_base(un)), 0u, kb);
        if (NU > 1) w1 = load_wsuper(unit_w(unit_base(un + kDownWaves)), 0u, kb);
        if (NU > 2) w2 = load_wsuper(unit_w(unit_base(un + 2 * kDownWaves)), 0u, kb);
        if (NU > 3) w3 = load_wsuper(unit_w(unit_base(un + 3 * kDownWaves)), 0u, kb);
        if (NU > 4) w4 = load_wsuper(unit_w(unit_base(un + 4 * kDownWaves)), 0u, kb);
    } else {
        if (un < units) w0 = load_wsuper(unit_w(unit_base(un)), 0u, kb);
        if (un + kDownWaves < units) w1 = load_wsuper(unit_w(unit_base(un + kDownWaves)), 0u, kb);
        if (un + 2 * kDownWaves < units) w2 = load_wsuper(unit_w(unit_base(un + 2 * kDownWaves)), 0u, kb);
        if (un + 3 * kDownWaves < units) w3 = load_wsuper(unit_w(unit_base(un + 3 * kDownWaves)), 0u, kb);
        if (un + 4 * kDownWaves < units) w4 = load_wsuper(unit_w(unit_base(un + 4 * kDownWaves)), 0u, kb);
    }

    if (tid < p.n_slots) s_sel[tid] = (tid < p.n_used) ? sel_mine : 0;
    if (early) {
        // (a slot's tiles are contiguous in LDS as they are in its row)
        if (tid < n_pieces) *(uint4 *)(tiles + (size_t)tid * 16u) = ex0;
        if (tid + kStep < n_pieces) *(uint4 *)(tiles + (size_t)(tid + kStep) * 16u) = ex1;
        if (tid + 2u * kStep < n_pieces) *(uint4 *)(tiles + (size_t)(tid + 2u * kStep) * 16u) = ex2;
        if (tid + 3u * kStep < n_pieces) *(uint4 *)(tiles + (size_t)(tid + 3u * kStep) * 16u) = ex3;
        if (tid + 4u * kStep < n_pieces) *(uint4 *)(tiles + (size_t)(tid + 4u * kStep) * 16u) = ex4;
        if (tid < units) s_yd[tid] = early_yd;
    } else if (STAGED) {
        stage_copy<1, kDownWaves * 64>(tiles, s_yd, p.n_slots, nb, tid,
                                       StageSlots{xq, p.xq_slot_stride, nb});
    } else {
        for (uint32_t pr = wave; pr < units; pr += kDownWaves) {
            const uint32_t slot = pr / nb, b = pr - slot * nb;
            const uint8_t *blk = xq + (uint64_t)slot * p.xq_slot_stride + (uint64_t)b * kQ8kBytes;
            stage_q8k_block<1>(tiles + (size_t)pr * 512u, s_yd + pr, blk, 0, lane);
        }
    }
    __syncthreads();

    v4f acc = {0.f, 0.f, 0.f, 0.f};
    auto compute = [&](uint32_t u, const WSuper &w) {
        if (s_sel[u / nb] >= 0) {  // uniform per wave
            const BSuper bs = load_bsuper<1>(tiles + (size_t)u * 512u, kb, 0);
            mfma_super(acc, w, bs, s_yd[u], kb);
        }
    };
    if (NU > 0) {
        // Straight-line: step i multiplies unit i and refills its registers with unit i + 5.
        // No load sits behind a condition, so each wait names exactly the loads that may stay in
        // flight (behind a condition the compiler waits for all of them), and the empty asm
        // statements keep each refill behind the products that read the registers it overwrites
        // (moved in front of them it would need fresh registers, a copy and a wait for it).
#define DSX_DOWN_STEP(I, W)                                                                  \
    if (I < NU) {                                                                            \
        compute(un + I * kDownWaves, W);                                                     \
        asm volatile("" : "+v"(acc) :: "memory");                                            \
        if (I + 5 < NU) W = load_wsuper(unit_w(later[I + 5 < NU ? I : 0]), 0u, kb);            \
        asm volatile("" ::: "memory");                                                       \
    }
        DSX_DOWN_STEP(0, w0)
        DSX_DOWN_STEP(1, w1)
        DSX_DOWN_STEP(2, w2)
        DSX_DOWN_STEP(3, w3)
        DSX_DOWN_STEP(4, w4)
        DSX_DOWN_STEP(5, w0)
        DSX_DOWN_STEP(6, w1)
        DSX_DOWN_STEP(7, w2)
        DSX_DOWN_STEP(8, w3)
        DSX_DOWN_STEP(9, w4)
        DSX_DOWN_STEP(10, w0)
        DSX_DOWN_STEP(11, w1)
        DSX_DOWN_STEP(12, w2)
        DSX_DOWN_STEP(13, w3)
        DSX_DOWN_STEP(14, w4)
        static_assert(NU <= 15, "unrolled for at most 15 units per wave");
#undef DSX_DOWN_STEP
    } else {
#define DSX_DOWN_STEP(W)                                                                     \
    compute(un, W);                                                                          \
    if (un + 5 * kDownWaves < units) W = load_wsuper(unit_w(unit_base(un + 5 * kDownWaves)), 0u, kb);     \
    un += kDownWaves;                                                                        \
    if (un >= units) break;
        while (un < units) {
            DSX_DOWN_STEP(w0)
            DSX_DOWN_STEP(w1)
            DSX_DOWN_STEP(w2)
            DSX_DOWN_STEP(w3)
            DSX_DOWN_STEP(w4)
        }
#undef DSX_DOWN_STEP
    }

    s_red[wave][0][lane] = acc.x;
    s_red[wave][1][lane] = acc.y;
    s_red[wave][2][lane] = acc.z;
    s_red[wave][3][lane] = acc.w;
    __syncthreads();
    if (tid < n_live) {
        const uint32_t l = (tid >> 2) * 16u, i = tid & 3u;
        float s = 0.0f;
#pragma unroll
        for (int wv = 0; wv < kDownWaves; wv++) s += s_red[wv][i][l];
        if (p.residual) s += p.residual[(uint64_t)blockIdx.y * p.n_rows + row0 + tid];
        out[row0 + tid] = s;
    }
}

// ---------------------------------------------------------------------------------------
// down, by-expert: partials[(t * n_used + slot) * n_rows + row] = down_e[row] . midq[t, slot]
// ---------------------------------------------------------------------------------------
constexpr int kDownBeWaves = 4;

struct DownByExpertParams {
    float *partials;
    const uint8_t *down;
    const uint8_t *xq;  // [b * n_used] activation rows (Q8_K or staged), xq_slot_stride apart
    const int32_t *group_count, *group_offset, *members, *work_items, *n_work_items;
    uint64_t dbpe;
    uint32_t xq_slot_stride, n_used, chunk, n_rows, n_blocks_in;
    const uint8_t *sh_down;  // the extra expert (index n_expert, slot n_used), or null
    uint32_t n_expert, n_tokens;
    uint32_t n_sub;  // workgroups along grid.y per work item, NT columns each (0 is read as 1)
    uint32_t planar; // the matrices are in the planar form (dsx_device.hpp)
};

// LDS: [n_blocks_in] tiles of 512 * NT bytes | yd[n_blocks_in * NT]
template <int NT, bool STAGED>
__global__ __launch_bounds__(kDownBeWaves * 64) void k_mxfp4_down_by_expert(
    const DownByExpertParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ float s_red[kDownBeWaves][4][64];
    __shared__ int s_dest[NT];

    const uint32_t nb = p.n_blocks_in;
    uint8_t *tiles = smem;
    float *s_yd = (float *)(smem + (size_t)nb * 512u * NT);

    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u;
    const uint32_t bx = (gridDim.x & 7u) == 0u ? (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3)
                                                : blockIdx.x;  // an XCD's row tiles are contiguous
    const uint32_t row0 = bx * 16u;
    const uint32_t n_sub = p.n_sub > 1u ? p.n_sub : 1u;
    const uint32_t item = blockIdx.y / n_sub;
    const uint32_t col_off = (blockIdx.y - item * n_sub) * (uint32_t)NT;
    if ((int)item >= *p.n_work_items) return;
    const uint32_t wi = (uint32_t)p.work_items[item];
    const uint32_t e = wi >> 16, start = (wi & 0xFFFFu) + col_off;
    const uint32_t total = (uint32_t)p.group_count[e];
    if (start >= total) return;  // uniform: this sub-chunk of the item has no members
    const uint32_t cnt = min(min(p.chunk - col_off, (uint32_t)NT), total - start);
    const uint32_t mbase = (uint32_t)p.group_offset[e] + start;
    const bool extra = p.sh_down != nullptr && e >= p.n_expert;
    if (tid < cnt) {
        const uint32_t m = (uint32_t)p.members[mbase + tid];
        const uint32_t t = m >> 16, slot = m & 0xFFFFu;
        s_dest[tid] = (int)(slot >= p.n_used ? p.n_tokens * p.n_used + t : t * p.n_used + slot);
    }

    const uint32_t r = lane & 15u, kb = lane >> 4;
    const uint32_t wstep = w_step(p.planar != 0u);
    const WRow wrow = w_row(extra ? p.sh_down : p.down + (uint64_t)e * p.dbpe, row0 + r, nb, p.planar != 0u);
    uint32_t sb = wave;
    WSuper w0 = {}, w1 = {};
    if (sb < nb) w0 = load_wsuper(wrow, (uint64_t)(sb) * wstep, kb);
    if (sb + kDownBeWaves < nb) w1 = load_wsuper(wrow, (uint64_t)((sb + kDownBeWaves)) * wstep, kb);

    __syncthreads();
    if (STAGED) {
        stage_copy<NT, kDownBeWaves * 64>(tiles, s_yd, cnt, nb, tid,
                                          StageMembers{p.xq, p.xq_slot_stride, (const uint32_t *)s_dest});
    } else {
        for (uint32_t pr = wave; pr < cnt * nb; pr += kDownBeWaves) {
            const uint32_t j = pr / nb, b = pr - j * nb;
            const uint8_t *blk = p.xq + (uint64_t)s_dest[j] * p.xq_slot_stride + (uint64_t)b * kQ8kBytes;
            stage_q8k_block<NT>(tiles + (size_t)b * 512u * NT, s_yd + b * NT + j, blk, j, lane);
        }
    }
    __syncthreads();

    const uint32_t n = lane & 15u;
    const uint32_t col = (n < cnt) ? n : 0u;
    v4f acc = {0.f, 0.f, 0.f, 0.f};
    auto compute = [&](uint32_t s, const WSuper &w) {
        const BSuper bs = load_bsuper<NT>(tiles + (size_t)s * 512u * NT, kb, col);
        mfma_super(acc, w, bs, s_yd[s * NT + col], kb);
    };
    while (sb < nb) {
        compute(sb, w0);
        if (sb + 2 * kDownBeWaves < nb) w0 = load_wsuper(wrow, (uint64_t)((sb + 2 * kDownBeWaves)) * wstep, kb);
        sb += kDownBeWaves;
        if (sb >= nb) break;
        compute(sb, w1);
        if (sb + 2 * kDownBeWaves < nb) w1 = load_wsuper(wrow, (uint64_t)((sb + 2 * kDownBeWaves)) * wstep, kb);
        sb += kDownBeWaves;
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

// ---------------------------------------------------------------------------------------
// By-expert down and gate/up on staged rows, four row tiles per workgroup.
// The kernels above give a 16-row tile to a workgroup whose four waves split the k range: every
// workgroup looks up its item, stages the members' activation rows -- as many bytes as its
// weights when a few members meet 16 rows of `down` -- and ends in a sum through LDS, for 17 KB
// (down) or 122 KB (gate/up) of weights.  In the down kernel here wave w owns row tile 4 bx + w
// over the whole k range, so that one look-up and one staged copy serve four tiles, nothing is
// exchanged at the end, and four super-blocks of weights are on their way per wave.  The sums keep
// the association of the kernels above -- super-blocks s = w' (mod 4) in ascending order into
// accumulator w', then (((0 + a0) + a1) + a2) + a3 -- and so their bits.
// ---------------------------------------------------------------------------------------
constexpr int kBe4Waves = 8;    // waves = row tiles of a workgroup of the down kernel
constexpr int kGuBeTiles = 8;   // row tiles of a workgroup of the gate/up kernel

template <int NT>
__global__ __launch_bounds__(kBe4Waves * 64) void k_mxfp4_down_be4(const DownByExpertParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ int s_dest[NT];

    const uint32_t nb = p.n_blocks_in;
    uint8_t *tiles = smem;
    float *s_yd = (float *)(smem + (size_t)nb * 512u * NT);

    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u;
    const uint32_t bx = (gridDim.x & 7u) == 0u ? (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3)
                                                : blockIdx.x;  // an XCD's row tiles are contiguous
    const uint32_t row0 = (bx * (uint32_t)kBe4Waves + wave) * 16u;
    const bool live = row0 < p.n_rows;   // (the last workgroup of a matrix of 16 (4 n + r) rows)
    const uint32_t n_sub = p.n_sub > 1u ? p.n_sub : 1u;
    const uint32_t item = blockIdx.y / n_sub;
    const uint32_t col_off = (blockIdx.y - item * n_sub) * (uint32_t)NT;
    if ((int)item >= *p.n_work_items) return;
    const uint32_t wi = (uint32_t)p.work_items[item];
    const uint32_t e = wi >> 16, start = (wi & 0xFFFFu) + col_off;
    const uint32_t total = (uint32_t)p.group_count[e];
    if (start >= total) return;  // uniform: this sub-chunk of the item has no members
    const uint32_t cnt = min(min(p.chunk - col_off, (uint32_t)NT), total - start);
    const uint32_t mbase = (uint32_t)p.group_offset[e] + start;
    const bool extra = p.sh_down != nullptr && e >= p.n_expert;
    if (tid < cnt) {
        const uint32_t m = (uint32_t)p.members[mbase + tid];
        const uint32_t t = m >> 16, slot = m & 0xFFFFu;
        s_dest[tid] = (int)(slot >= p.n_used ? p.n_tokens * p.n_used + t : t * p.n_used + slot);
    }

    // the first four super-blocks of the wave's rows go out before the activations are staged
    // (unconditional: a row shorter than four super-blocks reads its last one again)
    const uint32_t r = lane & 15u, kb = lane >> 4;
    const uint32_t wstep = w_step(p.planar != 0u);
    const WRow wrow = w_row(extra ? p.sh_down : p.down + (uint64_t)e * p.dbpe, (live ? row0 : 0u) + r, nb, p.planar != 0u);
    const uint32_t last = nb - 1u;
    WSuper w[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        w[i] = load_wsuper(wrow, (uint64_t)min((uint32_t)i, last) * wstep, kb);
        // (in this order, as the loop below requests them: the compiler's wait for a super-block
        // is the weaker of what the loop's entry and its back edge allow)
        __builtin_amdgcn_sched_barrier(0);
    }

    __syncthreads();
    stage_copy<NT, kBe4Waves * 64>(tiles, s_yd, cnt, nb, tid,
                                   StageMembers{p.xq, p.xq_slot_stride, (const uint32_t *)s_dest});
    __syncthreads();
    if (!live) return;

    const uint32_t n = lane & 15u;
    const uint32_t col = (n < cnt) ? n : 0u;
    v4f acc[4];
#pragma unroll
    for (int i = 0; i < 4; i++) acc[i] = v4f{0.f, 0.f, 0.f, 0.f};
    auto compute = [&](uint32_t s, const WSuper &ws, v4f &a) {
        const BSuper bs = load_bsuper<NT>(tiles + (size_t)s * 512u * NT, kb, col);
        mfma_super(a, ws, bs, s_yd[s * NT + col], kb);
    };
    uint32_t sb = 0;
    for (; sb + 8u <= nb; sb += 4u) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            compute(sb + (uint32_t)i, w[i], acc[i]);
            w[i] = load_wsuper(wrow, (uint64_t)(sb + 4u + (uint32_t)i) * wstep, kb);
            // (each refill stays right behind the products that free its registers: left alone
            // the compiler multiplies all four super-blocks first and then requests all four)
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // up to seven super-blocks are left: those in the registers, then the rest
#pragma unroll
    for (int i = 0; i < 4; i++)
        if (sb + (uint32_t)i < nb) compute(sb + (uint32_t)i, w[i], acc[i]);
    if (sb + 4u < nb) {
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (sb + 4u + (uint32_t)i < nb) w[i] = load_wsuper(wrow, (uint64_t)(sb + 4u + (uint32_t)i) * wstep, kb);
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (sb + 4u + (uint32_t)i < nb) compute(sb + 4u + (uint32_t)i, w[i], acc[i]);
    }

    // C layout: the lane holds rows 4 kb + i of the tile for column n
    float4 o;
    o.x = ((0.0f + acc[0].x) + acc[1].x + acc[2].x) + acc[3].x;
    o.y = ((0.0f + acc[0].y) + acc[1].y + acc[2].y) + acc[3].y;
    o.z = ((0.0f + acc[0].z) + acc[1].z + acc[2].z) + acc[3].z;
    o.w = ((0.0f + acc[0].w) + acc[1].w + acc[2].w) + acc[3].w;
    if (n < cnt) *(float4 *)(p.partials + (uint64_t)s_dest[n] * p.n_rows + row0 + kb * 4u) = o;
}

// gate/up, by expert on staged rows: the workgroup of k_mxfp4_gate_up<NT, true, true, false> -- four
// waves that split the k range of a 16-row tile and add their sums through LDS -- for kBe4Waves
// consecutive row tiles, one after the other: one look-up of the item and one staged copy of its
// members' rows (half as many bytes as a tile's weights at four members) serve all of them, and a
// tile's first super-blocks are requested before the sums of the tile before it are added up.
// (A wave per row tile over the whole k range, as in k_mxfp4_down_be4, was 10 % slower here: a wave
// that walks along a row alone touches every cache line that two of the 136-byte super-blocks
// share twice, a microsecond apart, where four waves side by side touch it at the same time.)
template <int NT>
__global__ __launch_bounds__(kGuWaves * 64) void k_mxfp4_gate_up_be4(const GateUpParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ float s_red[kGuWaves][2][4][64];
    __shared__ int s_dest[NT];
    __shared__ float s_ew[NT];
    __shared__ uint32_t s_tok[NT];

    const uint32_t nb = p.n_blocks;
    uint8_t *tiles = smem;
    float *s_yd = (float *)(smem + (size_t)nb * 512u * NT);

    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u;
    const uint32_t bx = (gridDim.x & 7u) == 0u ? (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3)
                                                : blockIdx.x;
    const uint32_t tile0 = bx * (uint32_t)kGuBeTiles;
    const uint32_t n_t = min((uint32_t)kGuBeTiles, p.n_rows / 16u - tile0);   // row tiles of this workgroup
    const uint32_t n_sub = p.n_sub > 1u ? p.n_sub : 1u;
    const uint32_t item = blockIdx.y / n_sub;
    const uint32_t col_off = (blockIdx.y - item * n_sub) * (uint32_t)NT;
    if ((int)item >= *p.n_work_items) return;  // uniform: grid is an upper bound
    const uint32_t wi = (uint32_t)p.work_items[item];
    const uint32_t e = wi >> 16, start = (wi & 0xFFFFu) + col_off;
    const uint32_t total = (uint32_t)p.group_count[e];
    if (start >= total) return;  // uniform
    const uint32_t cnt = min(min(p.chunk - col_off, (uint32_t)NT), total - start);
    const uint32_t mbase = (uint32_t)p.group_offset[e] + start;
    const bool extra = p.sh_gate != nullptr && e >= p.n_expert;
    if (tid < cnt) {
        const uint32_t m = (uint32_t)p.members[mbase + tid];
        const uint32_t t = m >> 16, slot = m & 0xFFFFu;
        s_tok[tid] = t;
        s_dest[tid] = (int)(slot >= p.n_used ? p.n_tokens * p.n_used + t : t * p.n_used + slot);
        s_ew[tid] = slot >= p.n_used ? 1.0f : p.ew[t * p.n_used + slot];
    }
    const float clamp = extra ? p.sh_clamp : p.clamp;
    const uint8_t *gate_e = extra ? p.sh_gate : p.gate + (uint64_t)e * p.gbpe;
    const uint8_t *up_e = extra ? p.sh_up : p.up + (uint64_t)e * p.ubpe;

    // the first two super-blocks of a tile (unconditional: a wave without a block of its own reads
    // the row's last one and never uses it, so that the k loop starts from a known count of loads)
    const uint32_t r = lane & 15u, kb = lane >> 4;
    const uint32_t wstep = w_step(p.planar != 0u);
    WRow grow, urow;
    WSuper g0, u0, g1, u1;
    auto first_loads = [&](uint32_t row0) {
        grow = w_row(gate_e, row0 + r, nb, p.planar != 0u);
        urow = w_row(up_e, row0 + r, nb, p.planar != 0u);
        const uint32_t last = nb - 1u;
        const uint32_t b0 = wave < last ? wave : last, b1 = wave + kGuWaves < last ? wave + kGuWaves : last;
        g0 = load_wsuper(grow, (uint64_t)(b0) * wstep, kb);
        u0 = load_wsuper(urow, (uint64_t)(b0) * wstep, kb);
        g1 = load_wsuper(grow, (uint64_t)(b1) * wstep, kb);
        u1 = load_wsuper(urow, (uint64_t)(b1) * wstep, kb);
    };
    first_loads(tile0 * 16u);

    __syncthreads();  // s_tok visible
    stage_copy<NT, kGuWaves * 64>(tiles, s_yd, cnt, nb, tid, StageMembers{p.xq, p.xq_row_bytes, s_tok});
    __syncthreads();

    const uint32_t n = lane & 15u;
    const uint32_t col = (n < cnt) ? n : 0u;
    for (uint32_t rt = 0; rt < n_t; rt++) {
        const uint32_t row0 = (tile0 + rt) * 16u;
        v4f acc_g = {0.f, 0.f, 0.f, 0.f}, acc_u = {0.f, 0.f, 0.f, 0.f};
        auto compute = [&](uint32_t s, const WSuper &g, const WSuper &u) {
            const BSuper bs = load_bsuper<NT>(tiles + (size_t)s * 512u * NT, kb, col);
            const float yd = s_yd[s * NT + col];
            mfma_super(acc_g, g, bs, yd, kb);
            mfma_super(acc_u, u, bs, yd, kb);
        };
        // the k loop of k_mxfp4_gate_up: two super-blocks of weights in flight per matrix, both
        // refills of an iteration unconditional, each behind the products that free its registers
#define DSX_AFTER_PRODUCTS() asm volatile("" : "+v"(acc_g), "+v"(acc_u) :: "memory")
#define DSX_PIN() asm volatile("" ::: "memory")
        uint32_t sb = wave;
        while (sb + 3 * kGuWaves < nb) {
            compute(sb, g0, u0);
            DSX_AFTER_PRODUCTS();
            g0 = load_wsuper(grow, (uint64_t)((sb + 2 * kGuWaves)) * wstep, kb);
            u0 = load_wsuper(urow, (uint64_t)((sb + 2 * kGuWaves)) * wstep, kb);
            DSX_PIN();
            asm volatile("" : "+v"(g1.s.x), "+v"(g1.s.y), "+v"(u1.s.x), "+v"(u1.s.y));
            compute(sb + kGuWaves, g1, u1);
            DSX_AFTER_PRODUCTS();
            g1 = load_wsuper(grow, (uint64_t)((sb + 3 * kGuWaves)) * wstep, kb);
            u1 = load_wsuper(urow, (uint64_t)((sb + 3 * kGuWaves)) * wstep, kb);
            DSX_PIN();
            sb += 2 * kGuWaves;
        }
        if (sb < nb) {
            WSuper g2 = {}, u2 = {};
            const bool third = sb + 2 * kGuWaves < nb;
            if (third) {
                g2 = load_wsuper(grow, (uint64_t)((sb + 2 * kGuWaves)) * wstep, kb);
                u2 = load_wsuper(urow, (uint64_t)((sb + 2 * kGuWaves)) * wstep, kb);
            }
            DSX_PIN();
            compute(sb, g0, u0);
            if (sb + kGuWaves < nb) compute(sb + kGuWaves, g1, u1);
            if (third) compute(sb + 2 * kGuWaves, g2, u2);
        }
        DSX_AFTER_PRODUCTS();
#undef DSX_AFTER_PRODUCTS
#undef DSX_PIN
        // the next tile's first super-blocks are on their way while this one's sums are added up
        if (rt + 1u < n_t) first_loads(row0 + 16u);

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
        __syncthreads();   // s_red is written again by the next tile
    }
}

}  // namespace dsx
