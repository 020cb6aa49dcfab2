// dsx_decode_fused.hpp -- the MXFP4 expert products of a decode step (few tokens) in ONE launch.
//
// The grid is a list of work items that the hardware hands to the CUs in order:
//
//   gate/up items  (token, slot, 16-row tile)   mid[token, slot, rows] = swiglu(gate.x, up.x) * ew
//   down items     (token, slot, 64-row block)  partial[token, slot, rows] = down . Q8_K(mid[token, slot])
//
// All gate/up items come first.  A down item needs the whole mid row of its (token, slot), i.e.
// the 128 gate/up tiles of that slot at the DeepSeek-V3 shape; it requests ALL of its weights
// (a wave holds its 16 rows x 8 super-blocks in registers) and only then waits, so while the last
// gate/up items drain, the slots they free fill with down items whose weights are already on
// their way: the memory pipe sees one stream of gate, up and down weights with no kernel
// boundary in it.  The item of a token's last slot adds the slots' partial rows in slot order
// (crates/v4flash-kernels/kernels/q2_k_accumulate_matvec_par.hip:724-729), then a shared expert's
// rows computed elsewhere and the residual, and writes the output.
//
// Hand-off between workgroups (they may run on different XCDs, whose L2 caches are not coherent
// with each other):
//   * mid is pre-filled with a bit pattern no product can have (kMidUnwritten), results are
//     stored write-through, and a consumer re-reads with loads that bypass its L2 until the
//     pattern is gone.  Producers never wait for anything.
//   * slot_done[token, slot] counts finished gate/up tiles, and ONE relay workgroup (the item
//     between the gate/up and the down items) watches these counters and, when a slot is
//     complete, raises ready[token, slot][0..kDfFan): the same flag in kDfFan separate cache
//     lines.  A waiting down item polls one of them.  (A thousand workgroups polling one word
//     queue up in a single memory channel and slow every load that passes through it; spread
//     over many lines the polls cost nothing measurable.)  Counter and flags are hints that say
//     when looking at mid is worth it; the pattern check stays the guarantee, because a producer
//     does not order its counter update behind its stores.
//   * partial rows are handed over the same way as mid: pre-filled with the pattern, stored
//     write-through, and the item of the token's last slot (in grid order) re-reads the other
//     slots' rows until the pattern is gone, then adds them in slot order to its own sums.
// Waiting is safe because workgroups start in grid order and a gate/up item waits for nothing:
// whatever a down item waits for is already running or finished.  Every wait is bounded all the
// same; a wait that gives up records a code in *status and the kernel still exits.
//
// Decode gate/up: crates/v4flash-kernels/kernels/mxfp4_pair_matvec.hip:200-229;
// decode down:    crates/v4flash-kernels/kernels/mxfp4_matvec.hip:83-155.
#pragma once

#include "dsx_device.hpp"
#include "dsx_expert_kernels.hpp"
#include "dsx_q8_0_kernels.hpp"
#include "dsx_quant.hpp"

namespace dsx {

constexpr int kDfWaves = 4;            // waves per workgroup (both item kinds)
constexpr uint32_t kDfDownRows = 64;   // output rows of a down item: 16 per wave
constexpr uint32_t kDfSpinLimit = 1u << 16;   // rounds of about half a microsecond
constexpr uint32_t kDfSpinLimitMax = 1u << 20;   // the most a caller may ask for (about half a second)
constexpr uint32_t kDfFan = 32;        // copies of a slot's ready flag, one cache line each
constexpr uint32_t kDfFanStride = 32;  // words between the copies (128 bytes)
constexpr uint32_t kDfMaxTokens = 16;  // the flags are laid out for at most this many tokens

struct DecodeFusedParams {
    // gate/up
    const uint8_t *gate, *up;        // [n_expert] experts, gbpe / ubpe apart
    const uint8_t *sh_gate, *sh_up;  // shared expert (slot n_used) or null
    // The shared expert may be kept in Q8_0 (engine rows [blocks x f16 d][blocks x 32 i8]) and be
    // narrower than the routed ones: sh_q8 != 0, sh_inter <= inter, the tokens also as Q8_0 rows
    uint32_t sh_q8, sh_inter;
    const uint8_t *xq8;              // [n_tokens] Q8_0 activation rows, xq8_row_bytes apart
    uint32_t xq8_row_bytes;
    uint64_t gbpe, ubpe;
    const uint8_t *xq;               // [n_tokens] staged rows, xq_row_bytes apart
    const float *ew;                 // [n_tokens, n_used]
    const int32_t *selected;         // [n_tokens, n_used]
    float *mid;                      // [n_tokens, n_slots, inter]; kMidUnwritten on entry
    float clamp, sh_clamp;
    // down
    const uint8_t *down, *sh_down;
    uint64_t dbpe;
    float *partials;                 // [n_tokens, n_slots, hidden]; kMidUnwritten on entry
    float *out;                      // [n_tokens, hidden]
    const float *residual;           // [n_tokens, hidden] or null; may alias out
    const float *shared_rows;        // [n_tokens, hidden] or null: a shared expert computed before the launch
    HcPost hc;                       // n_hc != 0: the result goes through the hyper-connection combine instead of to out
    uint32_t *slot_done;             // [n_tokens, n_slots], zero on entry
    uint32_t *ready;                 // [n_tokens, n_slots, kDfFan] flags kDfFanStride words apart, zero on entry
    uint32_t dn_early;               // super-blocks of a down item's weights requested before its mid row is checked
    uint32_t poll_sleep;             // pause between two polls of a waiting down item, in units of 64 clocks
    uint32_t *status;                // one word, zero on entry
    uint32_t n_expert, n_used, n_slots, n_tokens;
    uint32_t hidden, inter, n_sb, n_sb_in;   // n_sb = hidden / 256, n_sb_in = inter / 256
    uint32_t gu_tiles, dn_blocks;            // inter / 16, hidden / 64
    uint32_t n_gu_items;                     // n_tokens * n_slots * gu_tiles; the relay is item n_gu_items
    uint32_t xq_row_bytes;
    uint32_t spin_limit;
    // measurement aid (null in normal use): 4 clock readings per item -- start, weights
    // requested, wait over, end -- in units of the constant 100 MHz counter
    uint64_t *trace;
};

__device__ __forceinline__ void df_stamp(const DecodeFusedParams &p, uint32_t item, uint32_t which) {
    if (p.trace && threadIdx.x == 0) p.trace[(uint64_t)item * 4u + which] = wall_clock64();
}

// Slot order inside a token: the shared expert first (its weights need no routing result and
// its down items are the first to be wanted), then the picks in slot order.
__device__ __forceinline__ uint32_t df_slot_of(uint32_t order, uint32_t n_used, uint32_t n_slots) {
    return n_slots > n_used ? (order == 0u ? n_used : order - 1u) : order;
}

// Position j of a group of n items -> the group's index space, so that the workgroups one XCD
// receives (every eighth) cover one contiguous eighth of it.
__device__ __forceinline__ uint32_t df_xcd_contiguous(uint32_t j, uint32_t n) {
    return (n & 7u) == 0u ? (j & 7u) * (n >> 3) + (j >> 3) : j;
}

// (A NaN is stored as the canonical quiet NaN: whatever bits an input or a weight produced, no
// stored value can equal the unwritten pattern, itself a NaN, and make its readers wait.)
__device__ __forceinline__ void df_store_f32(float *p, float v) {
    v = v != v ? __uint_as_float(0x7FC00000u) : v;
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// What a reader makes of a value it gave up waiting for: zero.
__device__ __forceinline__ float df_zero_if_unwritten(float v) {
    return __float_as_uint(v) == kMidUnwritten ? 0.0f : v;
}
__device__ __forceinline__ float df_load_f32(const float *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// One word at an address that is the same for the whole wave and was written before the launch.
// SCALAR: through the scalar cache -- a vector load issued by a workgroup that starts on a busy CU
// returns behind everything the CU has in flight, and an item cannot request its weights before
// it knows its expert.  The instantiations that pair tokens (four tokens and more by default)
// read their pick and routing weight this way: 1-3 % off a step at the DeepSeek-V3 shape.  With
// one or two tokens most items start on an idle CU, and the scalar round trip in front of the
// first weight request costs 1-2 % instead, so the other instantiations keep the vector load.
template <bool SCALAR>
__device__ __forceinline__ uint32_t df_uniform_u32(const void *addr) {
    if (!SCALAR) return *(const uint32_t *)addr;
    uint32_t v;
    asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(addr) : "memory");
    return v;
}

// ---- which tokens an item serves ---------------------------------------------------------------
// With sharing on, the tokens that name one expert in a step (the shared expert: all tokens) are
// paired in token order, and the items of the first token of a pair also serve the second one,
// as a second column of the same products; the second token's own items for that expert have
// nothing to compute.  An expert named by 2 n tokens is then streamed n times instead of 2 n.
// (crates/v4flash-kernels/kernels/mxfp4_pair_matvec.hip:621-782 and mxfp4_matvec.hip:568-692
// group the picks of a few tokens by distinct expert in the same spirit.)
struct DfCols {          // the two columns of a pair, in LDS for the staging code
    uint32_t tok[2];
    uint32_t ms[2];      // token * n_slots + slot of each column
    float ew[2];
};
struct DfPair {
    uint32_t cnt;        // 0: second token of a pair (nothing to do), 1: alone, 2: with the token below
    uint32_t t1, ms1;    // the second column
    float ew0, ew1;      // routing weights of the two columns
};

// Every wave works the pairing out for itself, in scalar registers: one vector load covers 64
// (token, slot) picks, a ballot marks those that name expert e, and the tokens before and after
// t that do so follow from the bit positions -- no LDS, no barrier, and the load goes out next
// to the one that fetches e, so an item starts its weights no later than without sharing.
// `e` < 0 names the shared expert (every token has it: tokens 2 i and 2 i + 1 pair up).
template <bool SHARE>
__device__ __forceinline__ DfPair df_pair(const DecodeFusedParams &p, uint32_t t, uint32_t slot, int e) {
    DfPair r{1u, t, t * p.n_slots + slot, 1.0f, 1.0f};
    if (e < 0) {
        if (SHARE) {
            if (t & 1u) {
                r.cnt = 0u;
            } else if (t + 1u < p.n_tokens) {
                r.cnt = 2u;
                r.t1 = t + 1u;
                r.ms1 = (t + 1u) * p.n_slots + slot;
            }
        }
        return r;
    }
    r.ew0 = __uint_as_float(df_uniform_u32<SHARE>(p.ew + t * p.n_used + slot));
    if (!SHARE) return r;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t n = p.n_tokens * p.n_used, mine = t * p.n_used, after = mine + p.n_used;
    uint32_t before = 0u;
    int next = -1;
    for (uint32_t base = 0; base < n; base += 64u) {
        const uint32_t i = base + lane;
        const int v = i < n ? p.selected[i] : -1;
        const uint64_t m = __builtin_amdgcn_ballot_w64(v == e);
        auto below = [&](uint32_t x) -> uint64_t {   // the chunk's entries with index < x
            return x <= base ? 0ull : x >= base + 64u ? ~0ull : (1ull << (x - base)) - 1ull;
        };
        before += (uint32_t)__builtin_popcountll(m & below(mine));
        const uint64_t later = m & ~below(after);
        if (next < 0 && later) next = (int)(base + (uint32_t)__builtin_ctzll(later));
    }
    if (before & 1u) {
        r.cnt = 0u;
    } else if (next >= 0) {
        r.cnt = 2u;
        r.t1 = (uint32_t)next / p.n_used;
        r.ms1 = r.t1 * p.n_slots + ((uint32_t)next - r.t1 * p.n_used);
        r.ew1 = p.ew[next];
    }
    return r;
}

// How an item names its columns: one column held in registers (no sharing: the item's own
// token), or a stretch of the list in LDS.
struct DfOneCol {
    uint32_t t, m;
    float w;
    __device__ __forceinline__ uint32_t tok(uint32_t) const { return t; }
    __device__ __forceinline__ uint32_t ms(uint32_t) const { return m; }
    __device__ __forceinline__ float ew(uint32_t) const { return w; }
    __device__ __forceinline__ const uint32_t *tok_list() const { return nullptr; }
};
struct DfListCols {
    const DfCols *c;
    uint32_t col0;
    __device__ __forceinline__ uint32_t tok(uint32_t j) const { return c->tok[col0 + j]; }
    __device__ __forceinline__ uint32_t ms(uint32_t j) const { return c->ms[col0 + j]; }
    __device__ __forceinline__ float ew(uint32_t j) const { return c->ew[col0 + j]; }
    __device__ __forceinline__ const uint32_t *tok_list() const { return c->tok + col0; }
};

// ---- gate/up item ------------------------------------------------------------------------
// The products of one 16-row tile of gate and of up with NT token columns (col0 .. col0 + n - 1
// of the item's list), SwiGLU, write-through store of the mid values, the slots' counters.
// PRE: the single column's staged row was requested by the caller before the weights (ex0..3,
// early_yd) -- loads of a wave return in order, so the row must not queue behind them.
template <int NT, bool PRE, bool PLANAR, typename Cols>
__device__ __forceinline__ void df_gate_up_core(const DecodeFusedParams &p, const Cols c,
                                                uint32_t n, const uint8_t *gate_e,
                                                const uint8_t *up_e, float clamp, uint32_t row0,
                                                uint8_t *tiles, float *s_yd, float (*s_red)[2][4][64],
                                                uint4 ex0, uint4 ex1, uint4 ex2, uint4 ex3,
                                                float early_yd, uint32_t trace_id) {
    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u;
    constexpr uint32_t kStep = kDfWaves * 64u;
    const uint32_t r = lane & 15u, kb = lane >> 4;
    constexpr uint32_t kStepW = PLANAR ? 128u : (uint32_t)kSuperBytes;
    const WRow grow = w_row(gate_e, row0 + r, p.n_sb, PLANAR);
    const WRow urow = w_row(up_e, row0 + r, p.n_sb, PLANAR);
    uint32_t sb = wave;
    WSuper g0, u0, g1, u1;
    {
        const uint32_t last = p.n_sb - 1u;
        const uint32_t b0 = sb < last ? sb : last, b1 = sb + kDfWaves < last ? sb + kDfWaves : last;
        g0 = load_wsuper(grow, (uint64_t)(b0) * kStepW, kb);
        u0 = load_wsuper(urow, (uint64_t)(b0) * kStepW, kb);
        g1 = load_wsuper(grow, (uint64_t)(b1) * kStepW, kb);
        u1 = load_wsuper(urow, (uint64_t)(b1) * kStepW, kb);
    }

    if (PRE) {
        const uint8_t *xrow = p.xq + (uint64_t)c.tok(0) * p.xq_row_bytes;
        const uint32_t nq = p.n_sb * 32u;   // 16-byte pieces of the row's tiles
        if (tid < nq) *(uint4 *)(tiles + (size_t)tid * 16u) = ex0;
        if (tid + kStep < nq) *(uint4 *)(tiles + (size_t)(tid + kStep) * 16u) = ex1;
        if (tid + 2u * kStep < nq) *(uint4 *)(tiles + (size_t)(tid + 2u * kStep) * 16u) = ex2;
        if (tid + 3u * kStep < nq) *(uint4 *)(tiles + (size_t)(tid + 3u * kStep) * 16u) = ex3;
        // rows longer than four pieces per thread take further passes
        for (uint32_t q = tid + 4u * kStep; q < nq; q += kStep)
            *(uint4 *)(tiles + (size_t)q * 16u) = *(const uint4 *)(xrow + (size_t)q * 16u);
        if (tid < p.n_sb) s_yd[tid] = early_yd;
        for (uint32_t b = tid + kStep; b < p.n_sb; b += kStep)
            s_yd[b] = *((const float *)(xrow + (size_t)p.n_sb * 512u) + b);
    } else {
        stage_copy<NT, kDfWaves * 64>(tiles, s_yd, n, p.n_sb, tid,
                                      StageMembers{p.xq, p.xq_row_bytes, c.tok_list()});
    }
    __syncthreads();
    df_stamp(p, trace_id, 1);

    const uint32_t col = (lane & 15u) < n ? (lane & 15u) : 0u;
    v4f acc_g = {0.f, 0.f, 0.f, 0.f}, acc_u = {0.f, 0.f, 0.f, 0.f};
    auto compute = [&](uint32_t s, const WSuper &g, const WSuper &u) {
        const BSuper bs = load_bsuper<NT>(tiles + (size_t)s * 512u * NT, kb, col);
        const float yd = s_yd[s * NT + col];
        mfma_super(acc_g, g, bs, yd, kb);
        mfma_super(acc_u, u, bs, yd, kb);
    };
    // Two super-blocks of gate and up in flight per wave.  Every load of the steady state is
    // unconditional, so each wait names exactly the loads that may stay outstanding; the empty
    // asm statements keep a refill behind the products that read the registers it overwrites.
#define DSX_AFTER_PRODUCTS() asm volatile("" : "+v"(acc_g), "+v"(acc_u) :: "memory")
#define DSX_PIN() asm volatile("" ::: "memory")
    while (sb + 3 * kDfWaves < p.n_sb) {
        compute(sb, g0, u0);
        DSX_AFTER_PRODUCTS();
        g0 = load_wsuper(grow, (uint64_t)((sb + 2 * kDfWaves)) * kStepW, kb);
        u0 = load_wsuper(urow, (uint64_t)((sb + 2 * kDfWaves)) * kStepW, kb);
        DSX_PIN();
        asm volatile("" : "+v"(g1.s.x), "+v"(g1.s.y), "+v"(u1.s.x), "+v"(u1.s.y));
        compute(sb + kDfWaves, g1, u1);
        DSX_AFTER_PRODUCTS();
        g1 = load_wsuper(grow, (uint64_t)((sb + 3 * kDfWaves)) * kStepW, kb);
        u1 = load_wsuper(urow, (uint64_t)((sb + 3 * kDfWaves)) * kStepW, kb);
        DSX_PIN();
        sb += 2 * kDfWaves;
    }
    if (sb < p.n_sb) {
        WSuper g2 = {}, u2 = {};
        const bool third = sb + 2 * kDfWaves < p.n_sb;
        if (third) {
            g2 = load_wsuper(grow, (uint64_t)((sb + 2 * kDfWaves)) * kStepW, kb);
            u2 = load_wsuper(urow, (uint64_t)((sb + 2 * kDfWaves)) * kStepW, kb);
        }
        DSX_PIN();
        compute(sb, g0, u0);
        if (sb + kDfWaves < p.n_sb) compute(sb + kDfWaves, g1, u1);
        if (third) compute(sb + 2 * kDfWaves, g2, u2);
    }
#undef DSX_AFTER_PRODUCTS
#undef DSX_PIN

    // the waves' partial sums in wave order, SwiGLU, write-through store
    s_red[wave][0][0][lane] = acc_g.x;
    s_red[wave][0][1][lane] = acc_g.y;
    s_red[wave][0][2][lane] = acc_g.z;
    s_red[wave][0][3][lane] = acc_g.w;
    s_red[wave][1][0][lane] = acc_u.x;
    s_red[wave][1][1][lane] = acc_u.y;
    s_red[wave][1][2][lane] = acc_u.z;
    s_red[wave][1][3][lane] = acc_u.w;
    __syncthreads();
    if (tid < 16u * n) {
        const uint32_t rr = tid & 15u, j = tid >> 4;
        const uint32_t l = (rr >> 2) * 16u + j, i = rr & 3u;  // C layout: row 4*(l/16)+i, column l%16
        float gs = 0.0f, us = 0.0f;
#pragma unroll
        for (int w = 0; w < kDfWaves; w++) {
            gs += s_red[w][0][i][l];
            us += s_red[w][1][i][l];
        }
        const uint32_t ms = c.ms(j);
        df_store_f32(p.mid + (uint64_t)ms * p.inter + row0 + rr, swiglu_clamp(gs, us, clamp, c.ew(j)));
        // the hint; not ordered behind the stores on purpose (nobody waits here)
        if (rr == 0)
            __hip_atomic_fetch_add(p.slot_done + ms, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// ---- a shared expert kept in Q8_0 -----------------------------------------------------------------
// Its gate/up and down items sit in the slot the MXFP4 shared expert would take (first in grid
// order) and hand their results over the same way; the arithmetic is that of the Q8_0 streaming
// kernels (dsx_q8_0_kernels.hpp; crates/v4flash-kernels/kernels/shared_expert_fused.hip:69-199
// computes the same products for the same purpose).  Tiles past sh_inter only count as done.
__device__ __forceinline__ void df_q8_gate_up_item(const DecodeFusedParams &p, uint32_t t, uint32_t tile,
                                                   uint8_t *lds) {
    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u;
    const uint32_t ms = t * p.n_slots + p.n_used, row0 = tile * 16u;
    if (row0 < p.sh_inter) {
        const uint32_t nb = p.hidden / 32u, row_bytes = q8_0_act_row_bytes(nb);
        const uint8_t *xrow = p.xq8 + (uint64_t)t * p.xq8_row_bytes;
        q8_0_stage(lds, 1u, row_bytes, tid, [&](uint32_t) { return xrow; });
        __syncthreads();
        const uint64_t wstride = (uint64_t)nb * 34u;
        // the wave's four rows (wave, wave + 4, ...) two at a time, gate and up together
#pragma unroll
        for (uint32_t half = 0; half < 2u; half++) {
            const uint32_t ra = row0 + wave + half * 8u, rb = ra + 4u;
            const uint8_t *const rows[4] = {p.sh_gate + (uint64_t)ra * wstride, p.sh_up + (uint64_t)ra * wstride,
                                            p.sh_gate + (uint64_t)rb * wstride, p.sh_up + (uint64_t)rb * wstride};
            float a[4][1] = {{0.0f}, {0.0f}, {0.0f}, {0.0f}};
            q8_0_rows_partial<4, 1>(a, rows, lds, row_bytes, nb, lane);
            const float g0 = wave_sum_f32(a[0][0]), u0 = wave_sum_f32(a[1][0]);
            const float g1 = wave_sum_f32(a[2][0]), u1 = wave_sum_f32(a[3][0]);
            if (lane == 0) {
                df_store_f32(p.mid + (uint64_t)ms * p.inter + ra, swiglu_clamp(g0, u0, p.sh_clamp, 1.0f));
                df_store_f32(p.mid + (uint64_t)ms * p.inter + rb, swiglu_clamp(g1, u1, p.sh_clamp, 1.0f));
            }
        }
    }
    if (tid == 0) __hip_atomic_fetch_add(p.slot_done + ms, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Waits until the lane's four mid values at `src` are there (lanes with live == false hold
// nothing); the wait is wave-uniform and bounded like every other one.
__device__ __forceinline__ float4 df_wait_mid4(const DecodeFusedParams &p, const float *src, bool live,
                                               uint32_t ms, uint32_t item) {
    const uint32_t lane = threadIdx.x & 63u;
    float4 v = {0.f, 0.f, 0.f, 0.f};
    if (live) v = *(const float4 *)src;
    auto missing = [&]() {
        return live && (__float_as_uint(v.x) == kMidUnwritten || __float_as_uint(v.y) == kMidUnwritten ||
                        __float_as_uint(v.z) == kMidUnwritten || __float_as_uint(v.w) == kMidUnwritten);
    };
    bool flag_seen = false;
    for (uint32_t spin = 0; __builtin_amdgcn_ballot_w64(missing()) != 0ull; spin++) {
        if (spin > p.spin_limit) {
            if (lane == 0) atomicCAS(p.status, kStatusOk, kStatusMidWaitExpired);
            if (missing()) v = float4{0.f, 0.f, 0.f, 0.f};
            break;
        }
        if (!flag_seen) {
            const uint32_t *flag = p.ready + ((uint64_t)ms * kDfFan + (item % kDfFan)) * kDfFanStride;
            uint32_t polls = 0;
            while (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0u &&
                   polls < p.spin_limit) {
                polls++;
                for (uint32_t z = 0; z < p.poll_sleep; z += 8u) __builtin_amdgcn_s_sleep(8);
            }
            flag_seen = true;
        } else {
            __builtin_amdgcn_s_sleep(16);
        }
        if (live) {
            v.x = df_load_f32(src + 0);
            v.y = df_load_f32(src + 1);
            v.z = df_load_f32(src + 2);
            v.w = df_load_f32(src + 3);
        }
    }
    return v;
}

// Rows [row0, row0 + 16) of the wave: the mid row (sh_inter values) is quantized to a Q8_0
// activation row in LDS by every item that needs it, then each row of down is one pass of the wave.
// Returns the lane's row (lane % 16) of the 16 results.
__device__ __forceinline__ float df_q8_down_rows(const DecodeFusedParams &p, uint32_t t, uint32_t row0,
                                                 uint32_t item, uint8_t *lds) {
    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u;
    const uint32_t ms = t * p.n_slots + p.n_used;
    const uint32_t nb = p.sh_inter / 32u, n256 = (p.sh_inter + 255u) / 256u;
    const float *mrow = p.mid + (uint64_t)ms * p.inter;
    for (uint32_t blk = wave; blk < n256; blk += (uint32_t)kDfWaves) {
        const uint32_t idx = blk * 256u + lane * 4u;
        const bool live = idx < p.sh_inter;
        const float4 v = df_wait_mid4(p, mrow + idx, live, ms, item);
        uint32_t pk;
        float d8;
        q8_0_quantize_lane4(v, pk, d8);
        if (live) {
            *(uint32_t *)(lds + idx) = pk;
            if ((lane & 7u) == 0u) *(float *)(lds + p.sh_inter + (idx >> 5) * 4u) = d8;
        }
    }
    __syncthreads();
    const uint64_t wstride = (uint64_t)nb * 34u;
    float own = 0.0f;
    for (uint32_t rr = 0; rr < 16u; rr += 4u) {   // four rows at a time
        const uint8_t *base = p.sh_down + (uint64_t)(row0 + rr) * wstride;
        const uint8_t *const rows[4] = {base, base + wstride, base + 2u * wstride, base + 3u * wstride};
        float a[4][1] = {{0.0f}, {0.0f}, {0.0f}, {0.0f}};
        q8_0_rows_partial<4, 1>(a, rows, lds, 0u, nb, lane);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float v = wave_sum_f32(a[i][0]);
            if ((lane & 15u) == rr + (uint32_t)i) own = v;
        }
    }
    return own;
}

template <bool SHARE, bool PLANAR>
__device__ __forceinline__ void df_gate_up_item(const DecodeFusedParams &p, uint32_t item,
                                                uint8_t *tiles, float *s_yd,
                                                float (*s_red)[2][4][64], DfCols *cols) {
    const uint32_t tid = threadIdx.x;
    const uint32_t per_token = p.n_slots * p.gu_tiles;
    const uint32_t t = item / per_token, rem = item - t * per_token;
    const uint32_t order = rem / p.gu_tiles, j = rem - order * p.gu_tiles;
    const uint32_t slot = df_slot_of(order, p.n_used, p.n_slots);
    const uint32_t row0 = df_xcd_contiguous(j, p.gu_tiles) * 16u;
    df_stamp(p, item, 0);
    if (p.sh_q8 && slot == p.n_used) {   // uniform
        df_q8_gate_up_item(p, t, row0 / 16u, tiles);
        df_stamp(p, item, 3);
        return;
    }

    // the token's staged row goes out first (see df_gate_up_core)
    const uint8_t *xrow = p.xq + (uint64_t)t * p.xq_row_bytes;
    const uint32_t nq = p.n_sb * 32u;
    constexpr uint32_t kStep = kDfWaves * 64u;
    uint4 ex0 = {}, ex1 = {}, ex2 = {}, ex3 = {};
    if (tid < nq) ex0 = *(const uint4 *)(xrow + (size_t)tid * 16u);
    if (tid + kStep < nq) ex1 = *(const uint4 *)(xrow + (size_t)(tid + kStep) * 16u);
    if (tid + 2u * kStep < nq) ex2 = *(const uint4 *)(xrow + (size_t)(tid + 2u * kStep) * 16u);
    if (tid + 3u * kStep < nq) ex3 = *(const uint4 *)(xrow + (size_t)(tid + 3u * kStep) * 16u);
    float early_yd = 0.0f;
    if (tid < p.n_sb) early_yd = *((const float *)(xrow + (size_t)p.n_sb * 512u) + tid);

    const uint8_t *gate_e, *up_e;
    float clamp = p.clamp;
    int e = -1;
    if (slot < p.n_used) {
        e = (int)df_uniform_u32<SHARE>(p.selected + t * p.n_used + slot);
        if (e < 0 || (uint32_t)e >= p.n_expert) return;  // empty slot: its down items skip it too
        gate_e = p.gate + (uint64_t)e * p.gbpe;
        up_e = p.up + (uint64_t)e * p.ubpe;
    } else {
        gate_e = p.sh_gate;
        up_e = p.sh_up;
        clamp = p.sh_clamp;
    }
    const DfPair pr = df_pair<SHARE>(p, t, slot, e);
    if (pr.cnt == 0u) return;   // the token above serves this one
    if (pr.cnt == 1u) {
        df_gate_up_core<1, true, PLANAR>(p, DfOneCol{t, t * p.n_slots + slot, pr.ew0}, 1u, gate_e, up_e, clamp, row0,
                                 tiles, s_yd, s_red, ex0, ex1, ex2, ex3, early_yd, item);
    } else if (SHARE) {
        // the pair's two columns in one pass over the tile's weights
        if (tid == 0) {
            cols->tok[0] = t; cols->ms[0] = t * p.n_slots + slot; cols->ew[0] = pr.ew0;
            cols->tok[1] = pr.t1; cols->ms[1] = pr.ms1; cols->ew[1] = pr.ew1;
        }
        __syncthreads();
        df_gate_up_core<2, false, PLANAR>(p, DfListCols{cols, 0u}, 2u, gate_e, up_e, clamp, row0, tiles, s_yd,
                                  s_red, ex0, ex1, ex2, ex3, early_yd, item);
    }
    df_stamp(p, item, 3);
}

// ---- relay item ----------------------------------------------------------------------------
// One wave: lane l watches the counters of entries l, l + 64, ... (entry = token * n_slots +
// slot) and the wave raises the kDfFan flags of every entry whose gate/up tiles are all done.
__device__ __forceinline__ void df_relay_item(const DecodeFusedParams &p) {
    if (threadIdx.x >= 64u) return;
    const uint32_t lane = threadIdx.x;
    const uint32_t n = p.n_tokens * p.n_slots;
    const uint32_t per_lane = (n + 63u) / 64u;   // at most 32 (host-checked)
    uint32_t pending = 0u;                        // bit i: entry lane + 64 i still to be raised
    for (uint32_t i = 0; i < per_lane; i++) {
        const uint32_t idx = lane + 64u * i;
        if (idx >= n) continue;
        const uint32_t t = idx / p.n_slots, slot = idx - t * p.n_slots;
        bool live = true;
        if (slot < p.n_used) {
            const int e = p.selected[t * p.n_used + slot];
            live = e >= 0 && (uint32_t)e < p.n_expert;   // nobody waits for an empty slot
        }
        if (live) pending |= 1u << i;
    }
    for (uint32_t spin = 0; spin < p.spin_limit; spin++) {
        if (__builtin_amdgcn_ballot_w64(pending != 0u) == 0ull) return;
        for (uint32_t i = 0; i < per_lane; i++) {
            const uint32_t idx = lane + 64u * i;
            bool now = false;
            if ((pending >> i) & 1u)
                now = __hip_atomic_load(p.slot_done + idx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= p.gu_tiles;
            if (now) pending &= ~(1u << i);
            uint64_t m = __builtin_amdgcn_ballot_w64(now);
            while (m) {   // uniform: the whole wave raises the flags of one finished entry
                const uint32_t l = (uint32_t)__builtin_ctzll(m);
                m &= m - 1ull;
                const uint32_t entry = l + 64u * i;
                if (lane < kDfFan)
                    __hip_atomic_store(p.ready + ((uint64_t)entry * kDfFan + lane) * kDfFanStride, 1u,
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        __builtin_amdgcn_s_sleep(4);
    }
}

// ---- down item ---------------------------------------------------------------------------
// Adds up the partial rows of token t for the wave's 16 rows [row0, row0 + 16): picks in slot
// order, then the shared expert, then a shared expert computed before the launch and the residual.  The
// caller is the item of the token's last slot in grid order, so the rows it reads come from
// items that are running or done.  `own` (lane r < 16: row r) stands in for slot `own_slot`;
// own_slot >= n_slots reads every slot from memory.
__device__ __forceinline__ void df_combine(const DecodeFusedParams &p, uint32_t t, uint32_t row0,
                                           float own, uint32_t own_slot) {
    const uint32_t lane = threadIdx.x & 63u;
    const float *col = p.partials + (uint64_t)t * p.n_slots * p.hidden + row0 + (lane & 15u);
    float v[DSX_MAX_SLOTS];
    const uint64_t o = (uint64_t)t * p.hidden + row0 + (lane & 15u);
    for (uint32_t spin = 0;; spin++) {
        bool missing = false;
#pragma unroll
        for (int q = 0; q < DSX_MAX_SLOTS; q++) {
            v[q] = 0.0f;
            if ((uint32_t)q < p.n_slots && (uint32_t)q != own_slot && lane < 16u)
                v[q] = df_load_f32(col + (uint64_t)q * p.hidden);
        }
#pragma unroll
        for (int q = 0; q < DSX_MAX_SLOTS; q++) missing |= __float_as_uint(v[q]) == kMidUnwritten;
        if (__builtin_amdgcn_ballot_w64(missing) == 0ull) break;   // wave-uniform
        if (spin > p.spin_limit) {
            if (lane == 0) atomicCAS(p.status, kStatusOk, kStatusPartialWaitExpired);
#pragma unroll
            for (int q = 0; q < DSX_MAX_SLOTS; q++) v[q] = df_zero_if_unwritten(v[q]);
            break;
        }
        __builtin_amdgcn_s_sleep(8);
    }
    if (lane < 16u) {
        float s = 0.0f;
#pragma unroll
        for (int q = 0; q < DSX_MAX_SLOTS; q++)
            if ((uint32_t)q < p.n_slots) s += (uint32_t)q == own_slot ? own : v[q];
        if (p.shared_rows) s += p.shared_rows[o];
        if (p.residual) s += p.residual[o];
        if (p.hc.n_hc) hc_post_store(p.hc, t, row0 + (lane & 15u), p.hidden, s);
        else p.out[o] = s;
    }
}

// NSB > 0: inter / 256 == NSB, straight-line code with all NSB super-blocks of the wave's rows in
// registers; NSB == 0: any inter, in passes of up to 8 super-blocks.
template <int NSB, bool SHARE, bool PLANAR>
__device__ __forceinline__ void df_down_item(const DecodeFusedParams &p, uint32_t item,
                                             uint8_t *tiles, float *s_yd) {
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t nsb = NSB > 0 ? (uint32_t)NSB : p.n_sb_in;
    const uint32_t per_token = p.n_slots * p.dn_blocks;
    const uint32_t t = item / per_token, rem = item - t * per_token;
    const uint32_t order = rem / p.dn_blocks, j = rem - order * p.dn_blocks;
    const uint32_t slot = df_slot_of(order, p.n_used, p.n_slots);
    const uint32_t row0 = df_xcd_contiguous(j, p.dn_blocks) * kDfDownRows + wave * 16u;
    const uint32_t r = lane & 15u, kb = lane >> 4;
    const uint32_t trace_id = p.n_gu_items + 1u + item;
    const bool last = order + 1u == p.n_slots;   // this item adds up the token's rows
    df_stamp(p, trace_id, 0);

    if (p.sh_q8 && slot == p.n_used) {   // uniform
        const float own = df_q8_down_rows(p, t, row0, item, tiles);
        if (last) df_combine(p, t, row0, own, slot);
        else if (lane < 16u) df_store_f32(p.partials + ((uint64_t)t * p.n_slots + slot) * p.hidden + row0 + lane, own);
        df_stamp(p, trace_id, 3);
        return;
    }
    const uint8_t *down_e = p.sh_down;
    int e = -1;
    if (slot < p.n_used) {
        e = (int)df_uniform_u32<SHARE>(p.selected + t * p.n_used + slot);
        if (e < 0 || (uint32_t)e >= p.n_expert) {
            // empty slot: contributes zeros (the sum must still wait for the others)
            if (last) df_combine(p, t, row0, 0.0f, slot);
            else if (lane < 16u) df_store_f32(p.partials + ((uint64_t)t * p.n_slots + slot) * p.hidden + row0 + lane, 0.0f);
            df_stamp(p, trace_id, 3);
            return;
        }
        down_e = p.down + (uint64_t)e * p.dbpe;
    }
    // column 0's share of the mid row (blocks wave, wave + 4, ...) is requested first, through
    // the caches: when the slot's gate/up tiles finished before this item started -- the usual
    // case, they come earlier in the grid -- the row is complete and nothing below waits for
    // another workgroup.  (Blocks past the row's end repeat its last block, so that no load
    // sits behind a condition.)  A token served by an earlier one loads the same addresses and
    // drops them.
    const uint32_t blk0 = min(wave, nsb - 1u), blk1 = min(wave + kDfWaves, nsb - 1u);
    const float *mrow0 = p.mid + ((uint64_t)t * p.n_slots + slot) * p.inter;
    float4 mv0 = *(const float4 *)(mrow0 + (size_t)blk0 * 256u + lane * 4u);
    float4 mv1 = *(const float4 *)(mrow0 + (size_t)blk1 * 256u + lane * 4u);

    constexpr uint32_t kStepW = PLANAR ? 128u : (uint32_t)kSuperBytes;
    const WRow wrow = w_row(down_e, row0 + r, nsb, PLANAR);
    constexpr int kHold = NSB > 0 ? NSB : 8;
    WSuper w[kHold];
    // the first part of what this wave will read goes out now, the rest once the mid row is
    // known to be there
    const int early = (int)p.dn_early;
#pragma unroll
    for (int b = 0; b < kHold; b++)
        if ((NSB > 0 || (uint32_t)b < nsb) && b < early) w[b] = load_wsuper(wrow, (uint64_t)(b) * kStepW, kb);

    const DfPair pr = df_pair<SHARE>(p, t, slot, e);
    const uint32_t cnt = pr.cnt;
    if (cnt == 0u) {
        // the token above computes this one's rows; what is left here is the sum
        if (last) df_combine(p, t, row0, 0.0f, p.n_slots);
        df_stamp(p, trace_id, 3);
        return;
    }

    auto landed = [](const float4 &v) {
        return __float_as_uint(v.x) != kMidUnwritten && __float_as_uint(v.y) != kMidUnwritten &&
               __float_as_uint(v.z) != kMidUnwritten && __float_as_uint(v.w) != kMidUnwritten;
    };
    // One column's mid row into LDS tiles [c * nsb, (c + 1) * nsb): wait until it is complete,
    // quantize it.  v0 / v1: the wave's first two blocks if already requested (column 0).
    auto stage_column = [&](const uint32_t c, const uint32_t ms, float4 v0, float4 v1, const bool have) {
        const float *mrow = p.mid + (uint64_t)ms * p.inter;
        if (!have) {
            v0 = *(const float4 *)(mrow + (size_t)blk0 * 256u + lane * 4u);
            v1 = *(const float4 *)(mrow + (size_t)blk1 * 256u + lane * 4u);
        }
        auto reload = [&](uint32_t blk) {   // bypassing the caches
            const float *src = mrow + (size_t)blk * 256u + lane * 4u;
            float4 v;
            v.x = df_load_f32(src + 0);
            v.y = df_load_f32(src + 1);
            v.z = df_load_f32(src + 2);
            v.w = df_load_f32(src + 3);
            return v;
        };
        // a block is complete when no lane of the wave sees the pattern (wave-uniform)
        auto wait_block = [&](float4 &v, uint32_t blk) {
            bool flag_seen = false;
            for (uint32_t spin = 0; __builtin_amdgcn_ballot_w64(!landed(v)) != 0ull; spin++) {
                if (spin > p.spin_limit) {
                    if (lane == 0) atomicCAS(p.status, kStatusOk, kStatusMidWaitExpired);
                    v.x = df_zero_if_unwritten(v.x);
                    v.y = df_zero_if_unwritten(v.y);
                    v.z = df_zero_if_unwritten(v.z);
                    v.w = df_zero_if_unwritten(v.w);
                    break;
                }
                if (!flag_seen) {
                    // this item's copy of the slot's ready flag: one word in a line few others poll
                    const uint32_t *flag = p.ready + ((uint64_t)ms * kDfFan + (item % kDfFan)) * kDfFanStride;
                    uint32_t polls = 0;
                    while (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0u &&
                           polls < p.spin_limit) {
                        polls++;
                        for (uint32_t z = 0; z < p.poll_sleep; z += 8u) __builtin_amdgcn_s_sleep(8);
                    }
                    flag_seen = true;
                } else {
                    __builtin_amdgcn_s_sleep(16);
                }
                v = reload(blk);
            }
        };
        wait_block(v0, blk0);
        wait_block(v1, blk1);
        if (c == 0u) {
            // the mid row is there: the rest of the weights goes out
#pragma unroll
            for (int b = 0; b < kHold; b++)
                if ((NSB > 0 || (uint32_t)b < nsb) && b >= early) w[b] = load_wsuper(wrow, (uint64_t)(b) * kStepW, kb);
            df_stamp(p, trace_id, 1);
        }
        uint8_t *tl = tiles + (size_t)c * nsb * 512u;
        float *yd = s_yd + c * nsb;
        if (wave < nsb) quantize_block_to_staged(v0, lane, tl + (size_t)blk0 * 512u, yd + blk0);
        if (wave + kDfWaves < nsb) quantize_block_to_staged(v1, lane, tl + (size_t)blk1 * 512u, yd + blk1);
        for (uint32_t blk = wave + 2u * kDfWaves; blk < nsb; blk += kDfWaves) {   // rows of more than 8 blocks
            float4 v = *(const float4 *)(mrow + (size_t)blk * 256u + lane * 4u);
            wait_block(v, blk);
            quantize_block_to_staged(v, lane, tl + (size_t)blk * 512u, yd + blk);
        }
    };
    const uint32_t ms0 = t * p.n_slots + slot, ms1 = pr.ms1;
    stage_column(0u, ms0, mv0, mv1, true);
    if (SHARE && cnt > 1u) stage_column(1u, ms1, mv0, mv1, false);   // uniform over the workgroup
    __syncthreads();
    df_stamp(p, trace_id, 2);

    // both columns against the weights in one pass (each super-block's registers die as it is used)
    v4f acc = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
    const uint8_t *tl1 = tiles + (size_t)nsb * 512u;
#pragma unroll
    for (int b = 0; b < kHold; b++) {
        if (NSB > 0 || (uint32_t)b < nsb) {
            const BSuper bs = load_bsuper<1>(tiles + (size_t)b * 512u, kb, 0u);
            mfma_super(acc, w[b], bs, s_yd[b], kb);
            if (SHARE && cnt > 1u) {
                const BSuper bt = load_bsuper<1>(tl1 + (size_t)b * 512u, kb, 0u);
                mfma_super(acc1, w[b], bt, s_yd[nsb + b], kb);
            }
            // (keeps the next super-block's LDS reads behind these products: hoisted to the top,
            // the operands of all super-blocks would be live at once)
            if (SHARE) asm volatile("" : "+v"(acc), "+v"(acc1) :: "memory");
        }
    }
    if (NSB == 0) {   // rows longer than 8 super-blocks: the rest in further passes
        for (uint32_t b0 = 8u; b0 < nsb; b0 += 8u) {
            WSuper w2[8];
#pragma unroll
            for (int b = 0; b < 8; b++)
                if (b0 + b < nsb) w2[b] = load_wsuper(wrow, (uint64_t)((b0 + b)) * kStepW, kb);
#pragma unroll
            for (int b = 0; b < 8; b++) {
                if (b0 + b < nsb) {
                    const BSuper bs = load_bsuper<1>(tiles + (size_t)(b0 + b) * 512u, kb, 0u);
                    mfma_super(acc, w2[b], bs, s_yd[b0 + b], kb);
                    if (SHARE && cnt > 1u) {
                        const BSuper bt = load_bsuper<1>(tl1 + (size_t)(b0 + b) * 512u, kb, 0u);
                        mfma_super(acc1, w2[b], bt, s_yd[nsb + b0 + b], kb);
                    }
                }
            }
        }
    }

    // A wave's 16 sums sit in column 0 of the fragment (lanes 0, 16, 32, 48, four rows each);
    // lane r < 16 takes row r.
    auto to_rows = [&](const v4f &a) {
        const int src_lane = (int)(16u * ((lane & 15u) >> 2));
        const float c0 = __shfl(a.x, src_lane, 64), c1 = __shfl(a.y, src_lane, 64);
        const float c2 = __shfl(a.z, src_lane, 64), c3 = __shfl(a.w, src_lane, 64);
        const uint32_t ci = lane & 3u;
        return ci == 0u ? c0 : ci == 1u ? c1 : ci == 2u ? c2 : c3;
    };
    if (SHARE && cnt > 1u) {
        // the second token's rows: always a partial row -- its own item of its last slot adds
        // them up, so that every wait points backwards in the grid
        const float other = to_rows(acc1);
        if (lane < 16u) df_store_f32(p.partials + (uint64_t)ms1 * p.hidden + row0 + lane, other);
    }
    const float own = to_rows(acc);
    if (!last) {
        // not the token's last slot: leave the partial row (write-through, no waiting)
        if (lane < 16u) df_store_f32(p.partials + (uint64_t)ms0 * p.hidden + row0 + lane, own);
    } else {
        df_combine(p, t, row0, own, slot);
    }
    df_stamp(p, trace_id, 3);
}

// LDS (dynamic): max(n_sb (twice that when tokens share experts), n_sb_in) tiles of 512 bytes | as many floats
template <int NSB, bool SHARE, bool PLANAR = false>
__global__ __launch_bounds__(kDfWaves * 64, 1) void k_mxfp4_decode_fused(const DecodeFusedParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ float s_red[kDfWaves][2][4][64];
    __shared__ DfCols s_cols;
    // gate/up stages one or two token columns of n_sb tiles, down one column of n_sb_in tiles
    const uint32_t n_gu = SHARE ? 2u * p.n_sb : p.n_sb, n_dn = SHARE ? 2u * p.n_sb_in : p.n_sb_in;
    const uint32_t n_max = n_gu > n_dn ? n_gu : n_dn;
    uint8_t *tiles = smem;
    float *s_yd = (float *)(smem + (size_t)n_max * 512u);
    if (blockIdx.x < p.n_gu_items)
        df_gate_up_item<SHARE, PLANAR>(p, blockIdx.x, tiles, s_yd, s_red, &s_cols);
    else if (blockIdx.x == p.n_gu_items)
        df_relay_item(p);
    else
        df_down_item<NSB, SHARE, PLANAR>(p, blockIdx.x - p.n_gu_items - 1u, tiles, s_yd);
}

}  // namespace dsx
