// dsx_gemm_kernels.hpp -- MXFP4 expert products for many tokens per expert (prefill): a
// grouped GEMM on the block-scaled matrix instruction.
//
// Work item = (expert, first member), the next up to 128 members of that expert are the
// token columns.  A workgroup (8 waves, two per SIMD, 256 registers each) multiplies 2 x 256
// weight rows with those 128 columns over the whole k range:
//   gate/up (PAIR):  256 rows of gate and the same 256 rows of up; the epilogue applies the
//                    clamped SwiGLU and the routing weight, quantizes the 256 results of
//                    every column as one Q8_K block and writes it as the FP6 row
//                    that `down` reads -- the f32 `mid` never goes to memory;
//   down:            512 rows; the epilogue stores f32 partial rows, one per (token, slot).
// Wave w owns rows [32 w, 32 w + 32) of both row sets and all 128 columns: 2 x 2 x 8 = 32
// accumulator fragments.  Column groups past the end of a short group are skipped.
//
// The activations come as two planes of FP6 (E2M3) codes (dsx_device.hpp): the matrix
// instruction takes a 6-bit operand in half the cycles of an 8-bit one, and the int8 split
// q = 16 (q >> 4) + (q & 15) stays exact in it.
//
// The kernel is bound by the bytes that pass through the CU's L1, which serves requests in
// order: one HBM miss holds back the L2 hits behind it, so every byte moves at about HBM
// speed (19-26 GB/s per CU) whether or not it hits in L2.  Hence the wide tile (weight
// bytes per product halve against 64 columns) and loads in memory order (see below).
//
// The Q8_K block scale d of the activations differs per (column, super-block), so the
// matrix pipe cannot carry a sum across super-blocks.  The wide tile runs a column group's four
// operands of a super-block (half x plane) back to back through one register quad per weight
// fragment and folds it into the accumulator with the column's d once per super-block (one FMA
// per value, placed between the next column group's first matrix instructions); the narrow
// tile, whose operands arrive by half super-blocks, folds once per half.
#pragma once

#include <type_traits>

#include "dsx_device.hpp"
#include "dsx_quant.hpp"

namespace dsx {

constexpr int kGemmWaves = 8;
constexpr int kGemmRF = 2;                  // 16-row fragments per wave and row set
constexpr int kGemmMT = 128;                // token columns per workgroup (the wide tile)
constexpr int kGemmMTNarrow = 16;           // ... of the narrow tile: groups of a few members
constexpr int kGemmAWaveBytes = 2 * kGemmRF * 2048 + 2 * 256;  // a wave's weights of one super-block
// ... of the wide tile on the engine's rows, which fetches every row's 136 bytes as one run of nine
// 16-byte pieces (below): two row sets x 5 loads of 1 KB
constexpr int kGemmARunWaveBytes = 2 * 5 * 1024;
constexpr int gemm_a_wave_bytes(int mt, bool planar) { return mt == kGemmMT && !planar ? kGemmARunWaveBytes : kGemmAWaveBytes; }
// LDS of a workgroup.
// Narrow tile (MT = 16): the operand heads of two half super-blocks of the columns (128 bytes per
// column each) | the operand tails of two super-blocks (128 bytes per column each: both halves,
// one cache line) | two times 4 block scales of every column (the loads that fill them are 64
// lanes wide: 1 KB per 64 columns) | the waves' weight regions.
// Wide tile (MT = 128): two buffers of 64 columns x one whole super-block (384 bytes per column:
// the heads of half 0, the heads of half 1, the tails; 8 KB each) | the block scales | the waves'
// weight regions.
constexpr int kGemmPhaseCols = 64;                       // columns of one buffer of the wide tile
constexpr int kGemmPhaseLine = kGemmPhaseCols * 128;     // one of its three 128-byte lines per column
constexpr int kGemmPhaseBytes = 3 * kGemmPhaseLine;
constexpr int gemm_heads_bytes(int mt) { return mt * 128; }
constexpr int gemm_tails_off(int mt) { return 2 * gemm_heads_bytes(mt); }
constexpr int gemm_tails_bytes(int mt) { return mt * 128; }
constexpr int gemm_yd_off(int mt) { return mt == kGemmMT ? 2 * kGemmPhaseBytes : gemm_tails_off(mt) + 2 * gemm_tails_bytes(mt); }
constexpr int gemm_yd_bytes(int mt) { return mt > 64 ? 2048 : 1024; }
constexpr int gemm_a_off(int mt) { return gemm_yd_off(mt) + 2 * gemm_yd_bytes(mt); }
constexpr size_t gemm_lds_bytes(int mt, bool planar) { return (size_t)gemm_a_off(mt) + kGemmWaves * gemm_a_wave_bytes(mt, planar); }

// f(integral_constant<int, I>) for I = From .. To - 1, unrolled at compile time (the matrix
// instruction wants its format and scale-select arguments as constants)
template <int From, int To, typename F>
__device__ __forceinline__ void gemm_static_for(F &&f) {
    if constexpr (From < To) {
        f(std::integral_constant<int, From>{});
        gemm_static_for<From + 1, To>(f);
    }
}

struct GemmParams {
    const uint8_t *w0, *w1;        // [n_expert] experts (gate, up), or down in w0 (w1 unused)
    const uint8_t *sh_w0, *sh_w1;  // the extra expert with index n_expert, or null
    uint64_t bpe0, bpe1;
    const uint8_t *act;            // staged activation rows, act_row_bytes apart
    const int32_t *group_count, *group_offset, *members, *work_items, *n_work_items;
    const float *ew;               // [n_tokens, n_used]               (gate/up)
    uint8_t *midq;                 // staged rows out, out_row_bytes, or null (gate/up)
    float *mid;                    // f32 [dest rows, n_rows] or null  (gate/up)
    float *partials;               // f32 [dest rows, n_rows]          (down)
    uint32_t n_tokens, n_used, n_expert;
    uint32_t n_rows;               // weight rows of one matrix
    uint32_t n_sb;                 // super-blocks per weight row (k / 256)
    uint32_t act_row_bytes, out_row_bytes;
    uint32_t n_row_tiles;          // n_rows / 256 (gate/up) or n_rows / 512 (down)
    float clamp, sh_clamp;
};

// Row of a per-(token, slot) table for member m = (token << 16) | slot; slot n_used is the
// extra expert, whose rows follow the n_tokens * n_used routed ones.
__device__ __forceinline__ uint32_t gemm_dest_row(uint32_t m, uint32_t n_tokens, uint32_t n_used) {
    const uint32_t t = m >> 16, slot = m & 0xFFFFu;
    return slot >= n_used ? n_tokens * n_used + t : t * n_used + slot;
}

// MT = 128: one workgroup per CU (256 registers per lane).  MT = 16: an eighth of the
// accumulators and of the column LDS, so that two workgroups share a CU (the second template
// argument of the launch bounds asks for four waves per SIMD) -- with few members per group the
// kernel only streams weights, and two workgroups keep twice the weight loads in flight.
template <bool PAIR, int MT, bool PLANAR = false>
__global__ __launch_bounds__(kGemmWaves * 64, MT == kGemmMT ? 2 : 4) void k_mxfp4_gemm(const GemmParams p) {
    constexpr int kGemmCG = MT / 16;                    // column groups
    constexpr int kHeadsBytes = gemm_heads_bytes(MT);    // the heads of half a super-block of all columns
    constexpr int kTailsOff = gemm_tails_off(MT);
    constexpr int kTailsBytes = gemm_tails_bytes(MT);    // the tails of a super-block of all columns
    constexpr int kGemmYdOff = gemm_yd_off(MT);
    constexpr int kYdBytes = gemm_yd_bytes(MT);          // four block scales of all columns
    constexpr int kGemmAOff = gemm_a_off(MT);
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ uint32_t s_dest[MT];
    __shared__ uint32_t s_src[MT];
    __shared__ float s_ew[MT];
    __shared__ uint64_t s_key[kGemmWaves][MT];
    __shared__ float s_iscale[MT];

    uint8_t *tiles = smem;
    float *s_yd = (float *)(smem + kGemmYdOff);

    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u;
    const uint32_t g4 = lane >> 4, n16 = lane & 15u;

    // Workgroups are dealt to the 8 XCDs round-robin by id, and each XCD has its own L2.  The row
    // tiles of a work item run on one XCD (they stream the same activations).  (A list sorted by
    // width and dealt like cards balances better still and was slower: the widest tiles, bound
    // by the matrix pipe, then all run at the same time, and so do the narrow ones, bound by the
    // weight stream.)
    const uint32_t xcd = blockIdx.x & 7u, seq = blockIdx.x >> 3;
    const uint32_t n_items = (uint32_t)*p.n_work_items;   // the grid is only an upper bound
    const uint32_t local = seq / p.n_row_tiles;
    // Many column tiles per expert (skewed routing, many tokens): the items are dealt to the XCDs
    // like cards, which spreads the wide groups -- contiguous ranges of the list (it is by expert)
    // left the busiest XCD with 17 % more column groups than the average at Zipf-skewed routing,
    // against 8 % (layer at T=4096: -4.6 %).  (One list per XCD that keeps every group's column
    // tiles together, balanced to 1 % in items and column groups, fetches a quarter fewer bytes --
    // neighbours share the weights in the XCD's L2 -- and is 6 % slower all the same.)  About a tile per expert: contiguous ranges, so that
    // an XCD streams one contiguous stretch of the weights (3-5 % faster then).
    const bool deal = n_items > p.n_expert + (p.n_expert >> 1);
    if (!deal && local >= (n_items + 7u) / 8u) return;  // uniform
    const uint32_t item = deal ? local * 8u + xcd : xcd * ((n_items + 7u) / 8u) + local;
    if (item >= n_items) return;  // uniform
    const uint32_t rt = seq % p.n_row_tiles;

    const uint32_t wi = (uint32_t)p.work_items[item];
    const uint32_t e = wi >> 16, start = wi & 0xFFFFu;
    const bool extra = e >= p.n_expert;
    // (PLANAR: the matrices in the planar form of dsx_device.hpp -- every 128-byte piece of a
    // row that a lane group fetches is then one whole cache line instead of parts of two)
    constexpr uint32_t kStepW = PLANAR ? 128u : (uint32_t)kSuperBytes;
    const uint32_t row_stride = p.n_sb * kStepW;           // between the rows of a 16-row tile
    const uint32_t tile_row = p.n_sb * kSuperBytes;        // a sixteenth of a tile, in either form
    const uint8_t *wbase[2];
    uint32_t row0[2];
    if (PAIR) {
        wbase[0] = extra ? p.sh_w0 : p.w0 + (uint64_t)e * p.bpe0;
        wbase[1] = extra ? p.sh_w1 : p.w1 + (uint64_t)e * p.bpe1;
        row0[0] = row0[1] = rt * 256u;
    } else {
        wbase[0] = wbase[1] = extra ? p.sh_w0 : p.w0 + (uint64_t)e * p.bpe0;
        row0[0] = rt * 512u;
        row0[1] = rt * 512u + 256u;
    }

    // The first super-block of weights depends on the expert and the row tile alone: it is requested
    // here, so that its trip to memory runs beside the look-ups of the group and its members.
    constexpr uint32_t kRowsPerWave = 16u * kGemmRF;
    static_assert(kGemmRF == 2, "one scale instruction covers the 32 rows of a wave's row set");
    constexpr uint32_t kScaleOff = 2u * kGemmRF * 2048u;
    const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
    // Wide tile on the engine's rows: a row's super-block -- 128 bytes of nibbles and the 8 scale
    // bytes behind them -- is fetched as one run of nine 16-byte pieces (the ninth holds bytes
    // 120..135, so that nothing past the super-block is read), lane slot s = 9 row + piece over the
    // wave's 32 rows of a row set: 288 slots in five loads.  A run lies in two cache lines, where
    // the 128-byte piece and the scales on their own made three requests.
    constexpr bool kRun = MT == kGemmMT && !PLANAR;
    constexpr int kAWaveBytes = gemm_a_wave_bytes(MT, PLANAR);
    const uint32_t a_lds = __builtin_amdgcn_readfirstlane(lds0 + kGemmAOff + wave * kAWaveBytes);
    const uint8_t *a_ptr = smem + kGemmAOff + wave * kAWaveBytes;
    uint32_t run_off[5];   // the lane's byte offset from the first row of the wave's rows, per load of a row set
#pragma unroll
    for (int i = 0; i < 5; i++) {
        const uint32_t slot = min(64u * (uint32_t)i + lane, 287u);   // (the last load's upper half repeats the last piece)
        const uint32_t rw = (slot * 7282u) >> 16, piece = slot - rw * 9u;   // slot / 9, slot % 9
        run_off[i] = rw * (p.n_sb * (uint32_t)kSuperBytes) + (piece < 8u ? piece * 16u : 120u);
    }
    const uint32_t l8 = lane >> 3, c8 = (lane & 7u) ^ l8;
    // fetch side: lane -> row l8 of the 8-row slab, chunk c8
    const uint32_t a_fetch = l8 * row_stride + c8 * 16u;
    uint32_t a_slab[kGemmRF][2];  // first row of fragment (r, m), times the row stride
#pragma unroll
    for (int r = 0; r < kGemmRF; r++)
#pragma unroll
        for (int m = 0; m < 2; m++)
            a_slab[r][m] = __builtin_amdgcn_readfirstlane((row0[m] + wave * kRowsPerWave + r * 16u) * tile_row);
    // scales: one instruction per row set, lane -> (row lane / 2 of the wave's 32, dword lane % 2);
    // planar: the 128 bytes of each of the wave's two 16-row tiles, behind the tile's nibble blocks
    const uint32_t sc_fetch = PLANAR ? (lane >> 5) * 16u * tile_row + p.n_sb * 2048u + (lane & 31u) * 4u
                                     : (lane >> 1) * row_stride + 128u + (lane & 1u) * 4u;
    // The part of an address that all lanes share (row set, fragment, super-block) goes into the
    // scalar base of the load; the lane's own offset is the same register for every weight load.
    auto issue_a = [&](uint32_t sb) {
        if constexpr (kRun) {
#pragma unroll
            for (int m = 0; m < 2; m++)
#pragma unroll
                for (int i = 0; i < 5; i++)
                    lds_dma16(a_lds + (uint32_t)(m * 5120 + i * 1024), wbase[m] + (a_slab[0][m] + sb * kStepW), run_off[i]);
            return;
        }
#pragma unroll
        for (int r = 0; r < kGemmRF; r++)
#pragma unroll
            for (int m = 0; m < 2; m++)
#pragma unroll
                for (int i = 0; i < 2; i++)
                    lds_dma16(a_lds + (uint32_t)((r * 2 + m) * 2048 + i * 1024),
                              wbase[m] + (a_slab[r][m] + (uint32_t)i * 8u * row_stride + sb * kStepW), a_fetch);
#pragma unroll
        for (int m = 0; m < 2; m++)
            lds_dma4(a_lds + kScaleOff + (uint32_t)m * 256u, wbase[m] + (a_slab[0][m] + sb * kStepW), sc_fetch);
    };
    issue_a(0);

    const uint32_t cnt = min((uint32_t)MT, (uint32_t)p.group_count[e] - start);
    const uint32_t mbase = (uint32_t)p.group_offset[e] + start;
    const float clamp = extra ? p.sh_clamp : p.clamp;
    if (tid < (uint32_t)MT) {
        // columns past the end of the group repeat its last member; they are never stored
        const uint32_t m = (uint32_t)p.members[mbase + min(tid, cnt - 1u)];
        const uint32_t dest = gemm_dest_row(m, p.n_tokens, p.n_used);
        s_dest[tid] = dest;
        s_src[tid] = PAIR ? (m >> 16) : dest;
        if (PAIR) s_ew[tid] = (m & 0xFFFFu) >= p.n_used ? 1.0f : p.ew[dest];
    }

    __syncthreads();  // s_src visible

    // ---- data movement: global memory -> LDS without passing through registers ------------
    // A load whose consecutive lanes read consecutive addresses costs the L1 a quarter of what
    // the matrix instruction's own operand layout (lane -> row lane % 16) costs, because the L1
    // looks up one cache line per cycle and a group of four lanes then shares a line.  So both
    // operands are fetched in memory order by LDS-direct loads (lane l of an instruction writes
    // LDS bytes [16 l, 16 l + 16) of the instruction's 1 KB destination) and read back from
    // LDS in operand order.  The 16-byte chunk a lane fetches is XOR-swizzled with its row so
    // that the later reads, 16 rows at a fixed chunk, spread over all banks.
    //
    // A, per wave and super-block: 4 fragments x (16 rows x 128 B of nibbles) + 64 rows x 8 B
    // of scales, private to the wave (no barrier).  B: the 128 columns' 192 B of half a
    // super-block, shared, double buffered; wave w fetches columns 16 w .. 16 w + 15.
    constexpr int kALoads = 4 * kGemmRF + 2;  // per wave and super-block
    // load L of those: 0..7 the halves of the four fragments, 8 and 9 the scales of the row sets
    // (row runs: loads 0..4 the first row set, 5..9 the second)
    auto issue_a_one = [&](int L, uint32_t sb) __attribute__((always_inline)) {
        if constexpr (kRun) {
            const int m = L / 5, i = L - 5 * m;
            lds_dma16(a_lds + (uint32_t)(m * 5120 + i * 1024), wbase[m] + (a_slab[0][m] + sb * kStepW), run_off[i]);
        } else if (L < 4 * kGemmRF) {
            const int f = L >> 1, i = L & 1, r = f >> 1, m = f & 1;
            lds_dma16(a_lds + (uint32_t)(f * 2048 + i * 1024),
                      wbase[m] + (a_slab[r][m] + (uint32_t)i * 8u * row_stride + sb * kStepW), a_fetch);
        } else {
            const int m = L - 4 * kGemmRF;
            lds_dma4(a_lds + kScaleOff + (uint32_t)m * 256u, wbase[m] + (a_slab[0][m] + sb * kStepW), sc_fetch);
        }
    };
    constexpr int kAFirst = 8;  // of them requested during the first half of a super-block
    // read side: lane (row n16, block g4) of fragment f: chunk g4 (first half), 4 + g4 (second)
    const uint32_t sw = ((n16 & 7u) * 8u + (g4 ^ (n16 & 7u))) * 16u;  // within a 1 KB slab
    const uint32_t a_rd = (n16 >> 3) * 1024u + sw;
    // tails: column n16's 128 bytes hold chunk (4 half + 2 plane + g4 / 2) at position
    // chunk ^ (n16 % 8) ^ (n16 / 8): the even columns of a group take eight different positions and
    // so do the odd ones, so that the 16 columns and their two 8-byte halves cover every bank once;
    // half and plane each flip one address bit
    const uint32_t bt_rd = n16 * 128u + (((g4 >> 1) ^ (n16 & 7u) ^ (n16 >> 3)) * 16u) + (g4 & 1u) * 8u;
    // sc: the lane's two scale bytes (block g4 of the first and of the second half), bytes 0 and 1
    struct GemmAFrag { uint4 a0, a1; uint32_t sc; };
    GemmAFrag a_cur[kGemmRF][2];
    auto read_a = [&]() {
#pragma unroll
        for (int r = 0; r < kGemmRF; r++)
#pragma unroll
            for (int m = 0; m < 2; m++) {
                uint2 sv;
                if constexpr (kRun) {
                    // row 16 r + n16 of the row set: pieces g4 and 4 + g4, the scales in the ninth piece's upper half
                    const uint8_t *f = a_ptr + m * 5120 + ((uint32_t)r * 16u + n16) * 144u;
                    a_cur[r][m].a0 = *(const uint4 *)(f + g4 * 16u);
                    a_cur[r][m].a1 = *(const uint4 *)(f + 64u + g4 * 16u);
                    sv = *(const uint2 *)(f + 136u);
                } else {
                    const uint8_t *f = a_ptr + (r * 2 + m) * 2048;
                    a_cur[r][m].a0 = *(const uint4 *)(f + a_rd);
                    a_cur[r][m].a1 = *(const uint4 *)(f + (a_rd ^ 64u));
                    sv = *(const uint2 *)(a_ptr + kScaleOff + m * 256u + r * 128u + n16 * 8u);
                }
                a_cur[r][m].sc = ((sv.x >> (g4 * 8u)) & 0xFFu) | (((sv.y >> (g4 * 8u)) & 0xFFu) << 8);
            }
    };

    // B of super-block sb: of each column's 384 bytes, per half h the 128 at 128 h (the 16-byte
    // heads of the operands of both planes and four blocks), and once per super-block the 128 at
    // 256 (their 8-byte tails, both halves: one cache line).  The heads of the 8 columns 8 g ..
    // 8 g + 7 are slab g of a heads buffer, fetched and swizzled like the weights; the tails of the
    // wave's 16 columns are two slabs of a tails buffer, fetched with the heads' lane offsets (the
    // second slab's with one address bit flipped, see bt_rd).  The columns' block scales d come four
    // super-blocks at a time (16 bytes per column, a wave per 64 columns).
    const uint32_t yd_fetch = s_src[tid & (uint32_t)(MT - 1)] * p.act_row_bytes + p.n_sb * kStaged6Bytes;
    const uint32_t yd_lds = __builtin_amdgcn_readfirstlane(lds0 + kGemmYdOff + (wave & 1u) * 1024u);
    auto issue_yd = [&](uint32_t sb) {  // a wave per 64 columns: d of super-blocks sb .. sb + 3
        if (wave < (uint32_t)(kYdBytes / 1024) && (sb & 3u) == 0u)
            lds_dma16(yd_lds + ((sb >> 2) & 1u) * (uint32_t)kYdBytes, p.act + sb * 4u, yd_fetch);
    };

    v4f acc[kGemmRF][2][kGemmCG];
    if constexpr (MT == kGemmMT) {
        // ---- the wide tile -------------------------------------------------------------------
        // B comes in phases of 64 columns x one whole super-block (each column's three cache lines:
        // heads of half 0, heads of half 1, tails), into two buffers that alternate.  A tile of
        // more than 64 columns runs two phases per super-block (columns 0..63, then 64..127), a
        // narrower one a single phase.  The loads of a phase go out at the start of the phase
        // before it.  Inside a phase a column group's four operands (half x plane) are multiplied
        // back to back against the wave's four weight fragments, so that the matrix pipe carries
        // the sum over the whole super-block -- the reference's order, sum the eight blocks, then
        // scale by the activations' d (crates/v4flash-kernels/src/mxfp4_tables.rs:52-73) -- and the
        // vector ALU folds one quad per fragment and super-block.
        const uint32_t bp_lds = __builtin_amdgcn_readfirstlane(lds0 + wave * 1024u);  // the wave's 8 columns: slab `wave`
        uint32_t bp_fetch[2];   // column 64 ch + 8 w + l8, chunk c8 of a 128-byte line
#pragma unroll
        for (int ch = 0; ch < 2; ch++)
            bp_fetch[ch] = s_src[(uint32_t)ch * kGemmPhaseCols + wave * 8u + l8] * p.act_row_bytes + c8 * 16u;
        // the second slab of a column group keeps its tails with one address bit flipped (bt_rd)
        const uint32_t tflip = (wave & 1u) << 4;
        // a wave whose column group lies past the end of a short group fetches nothing
        const bool ph_live[2] = {(wave >> 1) * 16u < cnt, kGemmPhaseCols + (wave >> 1) * 16u < cnt};
        auto issue_phase = [&](uint32_t sb, int ch, uint32_t buf) __attribute__((always_inline)) {
            if (!ph_live[ch]) return;
            // (uniform values, said so to the compiler: the loads take them in scalar registers)
            const uint8_t *src = p.act + __builtin_amdgcn_readfirstlane(sb * kStaged6Bytes);
            const uint32_t dst = __builtin_amdgcn_readfirstlane(bp_lds + buf * (uint32_t)kGemmPhaseBytes);
            lds_dma16(dst, src, bp_fetch[ch]);
            lds_dma16(dst + (uint32_t)kGemmPhaseLine, src + 128, bp_fetch[ch]);
            lds_dma16(dst + 2u * (uint32_t)kGemmPhaseLine, src + 256, bp_fetch[ch] ^ tflip);
        };
        // read side of a phase buffer: lane (column n16, block g4) of column group jj
        uint32_t head_rd[2], tail_rd[2][2];
#pragma unroll
        for (int q = 0; q < 2; q++) {
            head_rd[q] = ((n16 >> 3) * 1024u + sw) ^ ((uint32_t)q * 64u);
#pragma unroll
            for (int h = 0; h < 2; h++) tail_rd[h][q] = 2u * (uint32_t)kGemmPhaseLine + (bt_rd ^ ((uint32_t)q * 32u) ^ ((uint32_t)h * 64u));
        }
        const uint32_t nj = (cnt + 15u) / 16u;  // column groups that hold a real column
        issue_phase(0, 0, 0);
        issue_yd(0);
#pragma unroll
        for (int r = 0; r < kGemmRF; r++)
#pragma unroll
            for (int m = 0; m < 2; m++)
#pragma unroll
                for (int j = 0; j < kGemmCG; j++) acc[r][m][j] = v4f{0.f, 0.f, 0.f, 0.f};
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();

        // One phase: NJP column groups, the first of them column group J0 of the tile.  ALoads
        // of the next super-block's weight loads, starting with load AFrom, go out one behind each
        // of the first operands' products.
        auto compute_phase = [&](auto njpc, auto j0c, auto afc, auto alc, const uint32_t buf, const uint32_t sb)
                                 __attribute__((always_inline)) {
            constexpr int NJP = decltype(njpc)::value, J0 = decltype(j0c)::value;
            constexpr int AFrom = decltype(afc)::value, ALoads = decltype(alc)::value;
            constexpr int NP = 4 * NJP;
            const uint8_t *pb = tiles + buf * (uint32_t)kGemmPhaseBytes;
            const float *yds = s_yd + ((sb >> 2) & 1u) * (uint32_t)(kYdBytes / 4) + (sb & 3u);
            auto load_piece = [&](int jj, int pp) __attribute__((always_inline)) -> v8i {   // pp = 2 half + plane
                const int h = pp >> 1, q = pp & 1;
                const uint4 hd = *(const uint4 *)(pb + (uint32_t)(h * kGemmPhaseLine + jj * 2048) + head_rd[q]);
                const uint2 tl = *(const uint2 *)(pb + (uint32_t)(jj * 2048) + tail_rd[h][q]);
                return v8i{(int)hd.x, (int)hd.y, (int)hd.z, (int)hd.w, (int)tl.x, (int)tl.y, 0, 0};
            };
            v4f c[kGemmRF][2];
            v8i ring[2];
            ring[0] = load_piece(0, 0);
            float yd_prev = 0.0f, yd = 0.0f;
            gemm_static_for<0, NP>([&](auto gpc) __attribute__((always_inline)) {
                constexpr int gp = decltype(gpc)::value;
                constexpr int jj = gp >> 2, pp = gp & 3, h = pp >> 1, q = pp & 1;
                if (pp == 0) yd = yds[((uint32_t)(J0 + jj) * 16u + n16) * 4u];
                if (gp + 1 < NP) ring[(gp + 1) & 1] = load_piece((gp + 1) >> 2, (gp + 1) & 3);
                const v8i bq = ring[gp & 1];
#pragma unroll
                for (int r = 0; r < kGemmRF; r++)
#pragma unroll
                    for (int m = 0; m < 2; m++) {
                        const GemmAFrag &w = a_cur[r][m];
                        const uint4 &aw = h == 0 ? w.a0 : w.a1;
                        const v8i av = {(int)aw.x, (int)aw.y, (int)aw.z, (int)aw.w, 0, 0, 0, 0};
                        if (pp == 0) {
                            if (jj > 0) {   // the column group before: its sums are complete
                                v4f &a = acc[r][m][J0 + (jj > 0 ? jj - 1 : 0)];
                                a.x = fmaf(yd_prev, c[r][m].x, a.x);
                                a.y = fmaf(yd_prev, c[r][m].y, a.y);
                                a.z = fmaf(yd_prev, c[r][m].z, a.z);
                                a.w = fmaf(yd_prev, c[r][m].w, a.w);
                                // (the sums stay where they are written: without a use here the
                                // compiler moves the products behind the next barrier, all operands live)
                                asm volatile("" : "+v"(a));
                            }
                            c[r][m] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                                av, bq, v4f{0.f, 0.f, 0.f, 0.f}, 4, 2, 0, (int)w.sc, 0, kScaleB6High);
                        } else {
                            c[r][m] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                                av, bq, c[r][m], 4, 2, h, (int)w.sc, 0, q == 0 ? kScaleB6High : kScaleB6Low);
                        }
                    }
                if (pp == 3) yd_prev = yd;
                if constexpr (gp < ALoads) {
                    // literal indices: the load's registers are picked at compile time
                    constexpr int kA = AFrom;
                    if (gp == 0) issue_a_one(kA + 0 < kALoads ? kA + 0 : 0, sb + 1u);
                    if (gp == 1) issue_a_one(kA + 1 < kALoads ? kA + 1 : 0, sb + 1u);
                    if (gp == 2) issue_a_one(kA + 2 < kALoads ? kA + 2 : 0, sb + 1u);
                    if (gp == 3) issue_a_one(kA + 3 < kALoads ? kA + 3 : 0, sb + 1u);
                    if (gp == 4) issue_a_one(kA + 4 < kALoads ? kA + 4 : 0, sb + 1u);
                    if (gp == 5) issue_a_one(kA + 5 < kALoads ? kA + 5 : 0, sb + 1u);
                    if (gp == 6) issue_a_one(kA + 6 < kALoads ? kA + 6 : 0, sb + 1u);
                    if (gp == 7) issue_a_one(kA + 7 < kALoads ? kA + 7 : 0, sb + 1u);
                    if (gp == 8) issue_a_one(kA + 8 < kALoads ? kA + 8 : 0, sb + 1u);
                    if (gp == 9) issue_a_one(kA + 9 < kALoads ? kA + 9 : 0, sb + 1u);
                }
                // Nothing moves across the end of an operand's products: the request of the next
                // operand stays right ahead of them, the folds beside them.  (The empty statement
                // orders the LDS reads, which the compiler otherwise hoists to the top of the loop
                // -- more live operands than there are registers; the barrier holds the scheduler.)
                asm volatile("" ::: "memory");
                if constexpr (pp == 0 && jj > 0) {
                    // a fragment's fold, then its first product: the matrix pipe starts on the new
                    // column group after 4 vector instructions instead of 16
#pragma unroll
                    for (int f = 0; f < 2 * kGemmRF; f++) {
                        __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);   // 4 x vector ALU
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // 1 x matrix
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            });
#pragma unroll
            for (int r = 0; r < kGemmRF; r++)
#pragma unroll
                for (int m = 0; m < 2; m++) {
                    v4f &a = acc[r][m][J0 + NJP - 1];
                    a.x = fmaf(yd_prev, c[r][m].x, a.x);
                    a.y = fmaf(yd_prev, c[r][m].y, a.y);
                    a.z = fmaf(yd_prev, c[r][m].z, a.z);
                    a.w = fmaf(yd_prev, c[r][m].w, a.w);
                    asm volatile("" : "+v"(a));
                }
        };
        using I0 = std::integral_constant<int, 0>;
        // up to 64 columns: one phase per super-block, the buffers alternate by super-block
        // (The last super-block, which requests nothing, is a copy of the loop body: a condition
        // inside the body would split it into basic blocks, and the compiler then moves every
        // matrix instruction into the last of them.)
        using I1 = std::integral_constant<int, 1>;
        auto step_one_phase = [&](auto njc, auto morec, const uint32_t sb) __attribute__((always_inline)) {
            constexpr int NJ = decltype(njc)::value;
            constexpr bool more = decltype(morec)::value != 0;
            read_a();
            // the wave's A region is free again once its reads have returned
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            if constexpr (more) {
                issue_phase(sb + 1u, 0, (sb + 1u) & 1u);
                issue_yd(sb + 1u);
                // fewer operands than weight loads: the rest of the loads in front
                gemm_static_for<4 * NJ, kALoads>([&](auto lc) __attribute__((always_inline)) { issue_a_one(decltype(lc)::value, sb + 1u); });
            }
            constexpr int kBeside = !more ? 0 : 4 * NJ < kALoads ? 4 * NJ : kALoads;
            compute_phase(njc, I0{}, I0{}, std::integral_constant<int, kBeside>{}, sb & 1u, sb);
            // everything this wave fetched for the next super-block has landed before the others
            // may read it
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
        };
        // up to 64 columns: one phase per super-block, the buffers alternate by super-block
        auto loop_one_phase = [&](auto njc) {
            uint32_t sb = 0;
            for (; sb + 1u < p.n_sb; sb++) step_one_phase(njc, I1{}, sb);
            step_one_phase(njc, I0{}, sb);
        };
        auto step_two_phases = [&](auto njc, auto morec, const uint32_t sb) __attribute__((always_inline)) {
            constexpr int NJ2 = decltype(njc)::value - 4;
            constexpr bool more = decltype(morec)::value != 0;
            read_a();
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            issue_phase(sb, 1, 1u);
            compute_phase(std::integral_constant<int, 4>{}, I0{}, I0{}, std::integral_constant<int, more ? kALoads : 0>{}, 0u, sb);
            // the second phase's columns have landed (the younger weight loads may still be on
            // their way)
            if constexpr (more) asm volatile("s_waitcnt vmcnt(%0)" :: "n"(kALoads) : "memory");
            else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if constexpr (more) {
                issue_phase(sb + 1u, 0, 0u);
                issue_yd(sb + 1u);
            }
            compute_phase(std::integral_constant<int, NJ2>{}, std::integral_constant<int, 4>{}, I0{}, I0{}, 1u, sb);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
        };
        // more: columns 0..63 from buffer 0, then 64.. from buffer 1
        auto loop_two_phases = [&](auto njc) {
            uint32_t sb = 0;
            for (; sb + 1u < p.n_sb; sb++) step_two_phases(njc, I1{}, sb);
            step_two_phases(njc, I0{}, sb);
        };
        // (A tile of up to 64 columns on the engine's rows used to run a loop of its own that took the
        // weights through a ring of three super-blocks of registers in operand order instead of LDS:
        // 4 % faster than this loop while it fetched a row's nibbles and scales apart, 5-7 % slower
        // since it fetches them as one run -- 1.44 against 1.53 ms per layer at 256 tokens of the
        // DeepSeek-V3 shape, 3.15 against 3.26 at 4096.)
        switch (nj) {
            case 1: loop_one_phase(std::integral_constant<int, 1>{}); break;
            case 2: loop_one_phase(std::integral_constant<int, 2>{}); break;
            case 3: loop_one_phase(std::integral_constant<int, 3>{}); break;
            case 4: loop_one_phase(std::integral_constant<int, 4>{}); break;
            case 5: loop_two_phases(std::integral_constant<int, 5>{}); break;
            case 6: loop_two_phases(std::integral_constant<int, 6>{}); break;
            case 7: loop_two_phases(std::integral_constant<int, 7>{}); break;
            default: loop_two_phases(std::integral_constant<int, 8>{}); break;
        }
    } else {
        // ---- the narrow tile: B by half super-blocks ------------------------------------
        const uint32_t b_lds = __builtin_amdgcn_readfirstlane(lds0 + wave * 2048u);
        const uint32_t bt_lds = __builtin_amdgcn_readfirstlane(lds0 + kTailsOff + wave * 2048u);
        uint32_t b_fetch[2];   // column 16 w + 8 ii + l8, chunk c8 = lane % 8 ^ l8 of a 128-byte run
    #pragma unroll
        for (int ii = 0; ii < 2; ii++)
            b_fetch[ii] = s_src[(wave * 16u + ii * 8u + l8) & (uint32_t)(MT - 1)] * p.act_row_bytes + c8 * 16u;
        // a wave whose 16 columns lie past the end of a short group fetches nothing (nobody reads
        // them: the column loop stops at the last group that holds a real column)
        const bool b_live = wave * 16u < cnt;
        auto issue_b = [&](uint32_t sb, uint32_t h) {  // the heads of half h, into heads buffer h
            if (!b_live) return;
            const uint8_t *src = p.act + (sb * kStaged6Bytes + h * 128u);
    #pragma unroll
            for (int ii = 0; ii < 2; ii++)
                lds_dma16(b_lds + h * kHeadsBytes + (uint32_t)(ii * 1024), src, b_fetch[ii]);
        };
        auto issue_bt = [&](uint32_t sb) {  // the tails of both halves, into tails buffer sb % 2
            if (!b_live) return;
            const uint8_t *src = p.act + (sb * kStaged6Bytes + 256u);
            lds_dma16(bt_lds + (sb & 1u) * kTailsBytes, src, b_fetch[0]);
            lds_dma16(bt_lds + (sb & 1u) * kTailsBytes + 1024u, src, b_fetch[1] ^ 16u);
        };

        issue_b(0, 0);
        issue_bt(0);
        issue_yd(0);
    #pragma unroll
        for (int r = 0; r < kGemmRF; r++)
    #pragma unroll
            for (int m = 0; m < 2; m++)
    #pragma unroll
                for (int j = 0; j < kGemmCG; j++) acc[r][m][j] = v4f{0.f, 0.f, 0.f, 0.f};

        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();

        const uint32_t nj = (cnt + 15u) / 16u;  // column groups that hold a real column
        // One half super-block with NJ column groups (compile-time, so the code below is one
        // straight line): for every group, the two pieces (high and low plane) against the wave's
        // four fragments, then the fold acc += d * c -- placed right before each fragment's
        // temporary is overwritten by the next group's first piece.  The next piece's B operand is
        // requested from LDS one piece ahead of its use (deeper changes nothing).  Empty asm
        // statements pin that order; they emit no instruction, so the compiler still sees every
        // real one and keeps its hazards.  Left alone it hoists every LDS read of the half to its
        // top, which overflows the registers, pulls each fold up to the instruction that produces
        // its input, where it waits, and with the group count as a run-time condition waits for
        // each operand right after requesting it (layer at T=4096: 4.5 -> 4.0 ms).
    #define DSX_PIN() asm volatile("" ::: "memory")
        auto compute_half = [&](auto hc, auto njc, const uint32_t sb, const bool more) {
            constexpr int h = decltype(hc)::value;
            constexpr int NJ = decltype(njc)::value;
            const uint8_t *half = tiles + h * kHeadsBytes;
            const uint8_t *tails = tiles + kTailsOff + (sb & 1u) * kTailsBytes;
            const float *yds = s_yd + ((sb >> 2) & 1u) * (uint32_t)(kYdBytes / 4) + (sb & 3u);
            // the operand of (column group j, plane q): 16 bytes of head, 8 of tail
            auto load_piece = [&](int j, int q) -> v8i {
                const uint32_t cb = (((uint32_t)(2 * j) + (n16 >> 3)) * 1024u + sw) ^ ((uint32_t)q * 64u);
                const uint4 hd = *(const uint4 *)(half + cb);
                const uint2 tl = *(const uint2 *)(tails + (uint32_t)j * 2048u +
                                                  (bt_rd ^ ((uint32_t)q * 32u) ^ ((uint32_t)h * 64u)));
                return v8i{(int)hd.x, (int)hd.y, (int)hd.z, (int)hd.w, (int)tl.x, (int)tl.y, 0, 0};
            };
            v4f c[kGemmRF][2];
            // piece p = 2 j + q alternates between two operand registers
            constexpr int NP = 2 * NJ;
            v8i ring[2];
            ring[0] = load_piece(0, 0);
            float yd_prev = 0.0f, yd = 0.0f;
            DSX_PIN();
    #pragma unroll
            for (int pc = 0; pc < NP; pc++) {
                const int j = pc >> 1, q = pc & 1;
                if (q == 0) yd = yds[(j * 16u + n16) * 4u];
                if (pc + 1 < NP) ring[(pc + 1) & 1] = load_piece((pc + 1) >> 1, (pc + 1) & 1);
                DSX_PIN();
                v8i &bq = ring[pc & 1];
                asm volatile("" : "+v"(bq));  // the products with this piece stay behind the request above
    #pragma unroll
                for (int r = 0; r < kGemmRF; r++)
    #pragma unroll
                    for (int m = 0; m < 2; m++) {
                        const GemmAFrag &w = a_cur[r][m];
                        const uint4 &aw = h == 0 ? w.a0 : w.a1;
                        const v8i av = {(int)aw.x, (int)aw.y, (int)aw.z, (int)aw.w, 0, 0, 0, 0};
                        if (q == 0) {
                            if (j > 0) {
                                asm volatile("" : "+v"(c[r][m]));
                                v4f &a = acc[r][m][j > 0 ? j - 1 : 0];
                                a.x = fmaf(yd_prev, c[r][m].x, a.x);
                                a.y = fmaf(yd_prev, c[r][m].y, a.y);
                                a.z = fmaf(yd_prev, c[r][m].z, a.z);
                                a.w = fmaf(yd_prev, c[r][m].w, a.w);
                                asm volatile("" : "+v"(a));
                            }
                            c[r][m] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                                av, bq, v4f{0.f, 0.f, 0.f, 0.f}, 4, 2, h, (int)w.sc, 0, kScaleB6High);
                        } else {
                            c[r][m] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                                av, bq, c[r][m], 4, 2, h, (int)w.sc, 0, kScaleB6Low);
                        }
                    }
                if (q == 1) yd_prev = yd;
                // the next super-block's weights, a load or two behind each piece's products: a
                // request that has to wait for room in the memory pipeline then holds back nothing
                // that the matrix pipe does not already have
                {
                    constexpr int kFrom = h == 0 ? 0 : kAFirst, kCnt = h == 0 ? kAFirst : kALoads - kAFirst;
                    // behind the first pieces of a half: 8 of the 10 in the first half, one per piece (a
                    // few per cent faster than 6 + 4 and than all 10 at once, measured at 4096 tokens)
                    constexpr int kSpan = h == 0 ? (NP < 8 ? NP : 8) : (NP + 1) / 2;
                    const int lo = pc * kCnt / kSpan, hi = (pc + 1) * kCnt / kSpan;
                    if (pc < kSpan && more) {
                        // literal indices: the load's registers are picked at compile time
                        if (0 < kCnt && lo <= 0 && 0 < hi) issue_a_one(kFrom + 0, sb + 1u);
                        if (1 < kCnt && lo <= 1 && 1 < hi) issue_a_one(kFrom + 1, sb + 1u);
                        if (2 < kCnt && lo <= 2 && 2 < hi) issue_a_one(kFrom + 2, sb + 1u);
                        if (3 < kCnt && lo <= 3 && 3 < hi) issue_a_one(kFrom + 3, sb + 1u);
                        if (4 < kCnt && lo <= 4 && 4 < hi) issue_a_one(kFrom + 4, sb + 1u);
                        if (5 < kCnt && lo <= 5 && 5 < hi) issue_a_one(kFrom + 5, sb + 1u);
                        if (6 < kCnt && lo <= 6 && 6 < hi) issue_a_one(kFrom + 6, sb + 1u);
                        if (7 < kCnt && lo <= 7 && 7 < hi) issue_a_one(kFrom + 7, sb + 1u);
                        if (8 < kCnt && lo <= 8 && 8 < hi) issue_a_one(kFrom + 8, sb + 1u);
                        if (9 < kCnt && lo <= 9 && 9 < hi) issue_a_one(kFrom + 9, sb + 1u);
                    }
                }
            }
            // fold the last group
    #pragma unroll
            for (int r = 0; r < kGemmRF; r++)
    #pragma unroll
                for (int m = 0; m < 2; m++) {
                    v4f &a = acc[r][m][NJ - 1];
                    a.x = fmaf(yd_prev, c[r][m].x, a.x);
                    a.y = fmaf(yd_prev, c[r][m].y, a.y);
                    a.z = fmaf(yd_prev, c[r][m].z, a.z);
                    a.w = fmaf(yd_prev, c[r][m].w, a.w);
                }
        };
    #undef DSX_PIN

        auto main_loop = [&](auto njc) {
            for (uint32_t sb = 0; sb < p.n_sb; sb++) {
                const bool more = sb + 1u < p.n_sb;
                read_a();
                // the wave's A region is free again once its reads have returned
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                issue_b(sb, 1);
                compute_half(std::integral_constant<int, 0>{}, njc, sb, more);
                // the second half of B has landed (the younger weight loads may still be on their way)
                if (more) asm volatile("s_waitcnt vmcnt(%0)" :: "n"(kAFirst) : "memory");
                else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __syncthreads();
                if (more) {
                    issue_b(sb + 1u, 0);
                    issue_bt(sb + 1u);
                    issue_yd(sb + 1u);
                }
                compute_half(std::integral_constant<int, 1>{}, njc, sb, more);
                // everything this wave fetched for the next super-block has landed before the others
                // may read it
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __syncthreads();
            }
        };
        // the number of column groups that hold a real column picks the instantiation
        if constexpr (kGemmCG == 1) {
            main_loop(std::integral_constant<int, 1>{});
        } else {
            switch (nj) {
                case 1: main_loop(std::integral_constant<int, 1>{}); break;
                case 2: main_loop(std::integral_constant<int, 2>{}); break;
                case 3: main_loop(std::integral_constant<int, 3>{}); break;
                case 4: main_loop(std::integral_constant<int, 4>{}); break;
                case 5: main_loop(std::integral_constant<int, 5>{}); break;
                case 6: main_loop(std::integral_constant<int, 6>{}); break;
                case 7: main_loop(std::integral_constant<int, 7>{}); break;
                default: main_loop(std::integral_constant<int, 8>{}); break;
            }
        }

    }

    // ---- epilogue ---------------------------------------------------------------------
    // The lane holds, for each of its 8 columns j*16 + n16, rows 32w + 16r + 4*g4 + q.
    if (!PAIR) {
#pragma unroll
        for (int j = 0; j < kGemmCG; j++) {
            const uint32_t col = j * 16u + n16;
            if (col >= cnt) continue;
            float *dst = p.partials + (uint64_t)s_dest[col] * p.n_rows;
#pragma unroll
            for (int r = 0; r < kGemmRF; r++)
#pragma unroll
                for (int m = 0; m < 2; m++) {
                    const v4f v = acc[r][m][j];
                    *(float4 *)(dst + row0[m] + wave * kRowsPerWave + r * 16u + g4 * 4u) =
                        make_float4(v.x, v.y, v.z, v.w);
                }
        }
        return;
    }

    // gate/up: SwiGLU in place (the gate accumulator becomes mid), then Q8_K over the 256
    // rows of this tile per column (crates/v4flash-kernels/kernels/q8_k_quantize.hip:23-90:
    // the element of largest |x|, the first one on ties, sets iscale = -127 / x).
#pragma unroll
    for (int j = 0; j < kGemmCG; j++) {
        const float ew = s_ew[j * 16u + n16];
        uint64_t best = 0;
#pragma unroll
        for (int r = 0; r < kGemmRF; r++) {
            v4f &gv = acc[r][0][j];
            const v4f uv = acc[r][1][j];
            gv.x = swiglu_clamp(gv.x, uv.x, clamp, ew);
            gv.y = swiglu_clamp(gv.y, uv.y, clamp, ew);
            gv.z = swiglu_clamp(gv.z, uv.z, clamp, ew);
            gv.w = swiglu_clamp(gv.w, uv.w, clamp, ew);
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float v = q == 0 ? gv.x : q == 1 ? gv.y : q == 2 ? gv.z : gv.w;
                const uint32_t idx = wave * kRowsPerWave + r * 16u + g4 * 4u + q;
                const uint32_t bits = __float_as_uint(v);
                const uint64_t key = ((uint64_t)(bits & 0x7FFFFFFFu) << 32) | ((255u - idx) << 1) | (bits >> 31);
                best = key > best ? key : best;
            }
        }
        // lanes that share the column: n16 equal, g4 = 0..3
        uint64_t o = __shfl_xor(best, 16, 64);
        best = o > best ? o : best;
        o = __shfl_xor(best, 32, 64);
        best = o > best ? o : best;
        if (g4 == 0u) s_key[wave][j * 16u + n16] = best;
    }
    if (p.mid != nullptr) {
#pragma unroll
        for (int j = 0; j < kGemmCG; j++) {
            const uint32_t col = j * 16u + n16;
            if (col >= cnt) continue;
            float *dst = p.mid + (uint64_t)s_dest[col] * p.n_rows + rt * 256u + wave * kRowsPerWave + g4 * 4u;
#pragma unroll
            for (int r = 0; r < kGemmRF; r++) {
                const v4f v = acc[r][0][j];
                *(float4 *)(dst + r * 16u) = make_float4(v.x, v.y, v.z, v.w);
            }
        }
    }
    if (p.midq == nullptr) return;  // f32 mid only (a down matrix of another format follows)
    __syncthreads();
    const uint32_t n_blk_out = p.n_rows / 256u;
    if (tid < (uint32_t)MT) {
        uint64_t k = s_key[0][tid];
#pragma unroll
        for (int w = 1; w < kGemmWaves; w++) k = s_key[w][tid] > k ? s_key[w][tid] : k;
        const uint32_t abits = (uint32_t)(k >> 32);
        float iscale = 0.0f, d = 0.0f;
        if (abits != 0u) {
            const float mx = __uint_as_float(abits | ((uint32_t)(k & 1u) << 31));
            iscale = -127.0f / mx;
            d = 1.0f / iscale;
        }
        s_iscale[tid] = iscale;
        if (tid < cnt)
            *(float *)(p.midq + (uint64_t)s_dest[tid] * p.out_row_bytes + (uint64_t)n_blk_out * kStaged6Bytes +
                       rt * 4u) = d;
    }
    __syncthreads();
    // Rows 16r + 4*g4 + q of fragments r = 2*rho, 2*rho + 1 are the nibble positions
    // 8*g4 .. 8*g4+7 of 32-element block (kGemmRF / 2) * wave + rho (position 4 (q / 2) +
    // 2 (q & 1) + r & 1): 48 bits of each plane's 24-byte operand, at bit 48 g4.  Dwords 0 and 1
    // of the operand come from the lanes g4 = 0 and 1, dword 2 from g4 = 1, dwords 3 and 4 from
    // g4 = 2 and 3, dword 5 from g4 = 3: every lane fetches the low word of the lane 16 above.
#pragma unroll
    for (int j = 0; j < kGemmCG; j++) {
        const uint32_t col = j * 16u + n16;
        const float iscale = s_iscale[col];
#pragma unroll
        for (int rho = 0; rho < kGemmRF / 2; rho++) {
            uint32_t qw[2] = {0u, 0u};
#pragma unroll
            for (int rr = 0; rr < 2; rr++) {
                const v4f v4 = acc[2 * rho + rr][0][j];
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const float v = q == 0 ? v4.x : q == 1 ? v4.y : q == 2 ? v4.z : v4.w;
                    int qi = (int)rintf(iscale * v);
                    qi = qi > 127 ? 127 : qi;
                    qi = qi < -128 ? -128 : qi;
                    qw[q >> 1] |= ((uint32_t)qi & 0xFFu) << ((uint32_t)(2 * (q & 1) + rr) * 8u);
                }
            }
            uint32_t hc[2], lc[2];
            split_q4_fp6(qw[0], hc[0], lc[0]);
            split_q4_fp6(qw[1], hc[1], lc[1]);
            const uint32_t b32 = wave * (kGemmRF / 2) + rho;
            uint8_t *dst = p.midq + (uint64_t)s_dest[col] * p.out_row_bytes + (uint64_t)rt * kStaged6Bytes;
#pragma unroll
            for (int plane = 0; plane < 2; plane++) {
                const uint32_t g0 = pack_codes4(plane == 0 ? hc[0] : lc[0]);
                const uint32_t g1 = pack_codes4(plane == 0 ? hc[1] : lc[1]);
                const uint32_t lo = g0 | (g1 << 24), hi = g1 >> 8;            // the lane's 48 bits
                const uint32_t up = (uint32_t)__shfl((int)lo, (int)((lane + 16u) & 63u), 64);
                if (col >= cnt) continue;
                const uint32_t base = (g4 >> 1) * 3u;   // first operand dword of the lane pair
                if ((g4 & 1u) == 0u) {
                    *(uint32_t *)(dst + staged6_off(b32 >> 2, plane, b32 & 3u, base)) = lo;
                    *(uint32_t *)(dst + staged6_off(b32 >> 2, plane, b32 & 3u, base + 1u)) = hi | (up << 16);
                } else {
                    *(uint32_t *)(dst + staged6_off(b32 >> 2, plane, b32 & 3u, base + 2u)) = (lo >> 16) | (hi << 16);
                }
            }
        }
    }
}

}  // namespace dsx
