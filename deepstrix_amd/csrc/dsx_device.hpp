// dsx_device.hpp -- device-side building blocks shared by the gfx950 MoE kernels.
//
// The expert products run on the CDNA4 block-scaled matrix instruction
// V_MFMA_SCALE_F32_16X16X128_F8F6F4.  One instruction multiplies a 16-row x 128-k tile
// of FP4 (E2M1) weights, each 32-k block carrying its own E8M0 scale, with a 128-k x
// 16-column tile of FP8 (E4M3) activations.  That is exactly the shape of the engine's
// MXFP4 data: a lane's A operand is one 16-byte nibble block of a 136-byte super-block,
// loaded with a single 128-bit global load and never decoded on the vector ALU.
//
// The reference multiplies MXFP4 weights with int8 (Q8_K) activations
// (crates/v4flash-kernels/src/mxfp4_tables.rs:49-74).  int8 is not an MFMA operand type
// next to FP4, so each activation q is split exactly as q + 128 = 16*uh + ul with
// uh, ul in [0, 15]:   q = 16*(uh - 8) + ul.   Both (uh - 8) and ul are small integers
// that E4M3 holds exactly; the "high" plane is multiplied by 2^4 through the B-side
// block scale.  Every product is exact and the block sums are exact in f32, so the
// result is the reference's integer dot product, accumulated in f32.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace dsx {

constexpr int kSuperBytes = 136;   // MXFP4 super-block: 8 x 16 B nibbles + 8 scale bytes
constexpr int kQ8kBytes = 292;     // f32 d | i8 qs[256] | i16 bsums[16]
constexpr int kTileBytes1 = 512;   // staged activation bytes per (super-block, token): 2 planes x 256

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));

struct __attribute__((packed, aligned(8))) U4A8 {
    uint32_t x, y, z, w;
};
struct __attribute__((packed, aligned(4))) U2A4 {
    uint32_t x, y;
};

// Loads that are known to hit global memory.  A pointer that went through LDS or a select is
// "generic" to the compiler, which then emits flat loads; those count against both memory
// counters and force a full wait before every use.  Going through address space 1 keeps
// them global loads whose completion order the compiler can track.
#define DSX_GLOBAL __attribute__((address_space(1)))
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef u32x4_t u32x4_a8_t __attribute__((aligned(8)));
typedef u32x2_t u32x2_a4_t __attribute__((aligned(4)));
__device__ __forceinline__ U4A8 gload16(const uint8_t *p) {
    const u32x4_t v = *(const DSX_GLOBAL u32x4_a8_t *)(uintptr_t)p;
    U4A8 r;
    r.x = v.x; r.y = v.y; r.z = v.z; r.w = v.w;
    return r;
}
__device__ __forceinline__ U2A4 gload8(const uint8_t *p) {
    const u32x2_t v = *(const DSX_GLOBAL u32x2_a4_t *)(uintptr_t)p;
    U2A4 r;
    r.x = v.x; r.y = v.y;
    return r;
}
__device__ __forceinline__ uint32_t gload4(const uint8_t *p) {
    return *(const DSX_GLOBAL uint32_t *)(uintptr_t)p;
}

// int8 q -> (high plane byte, low plane byte):  q + 128 = 16 * uh + ul, the high plane holds
// uh - 8 in [-8, 7], the low plane ul in [0, 15], both as E4M3 (OCP) bytes:
// 0,1,..,7 -> 0x00,0x38,0x40,0x44,0x48,0x4A,0x4C,0x4E ; 8..15 -> 0x50 | (m & 7); sign in bit 7.
// Four int8 values at once (one per byte of `q`, any order) -> the dwords of the high and of the
// low plane with the same byte order.  Bytewise table look-ups (v_perm_b32) instead of four
// scalar splits: u = q + 128 = q ^ 0x80, low nibble and high nibble each index a 16-entry
// table of E4M3 bytes, taken as two 8-entry halves selected by the nibble's bit 3.
__device__ __forceinline__ void split_q4(uint32_t q, uint32_t &hi_word, uint32_t &lo_word) {
    const uint32_t u = q ^ 0x80808080u;
    const uint32_t ul = u & 0x0F0F0F0Fu, uh = (u >> 4) & 0x0F0F0F0Fu;
    // E4M3 of 0..7 and of 8..15; E4M3 of -(8 - m) for m = 0..7
    constexpr uint32_t kPos03 = 0x44403800u, kPos47 = 0x4E4C4A48u;
    constexpr uint32_t kBig03 = 0x53525150u, kBig47 = 0x57565554u;
    constexpr uint32_t kNeg03 = 0xCACCCED0u, kNeg47 = 0xB8C0C4C8u;
    const uint32_t sl = ul & 0x07070707u, sh = uh & 0x07070707u;
    const uint32_t ml = ((ul >> 3) & 0x01010101u) * 0xFFu, mh = ((uh >> 3) & 0x01010101u) * 0xFFu;
    const uint32_t lo_small = __builtin_amdgcn_perm(kPos47, kPos03, sl);
    const uint32_t lo_big = __builtin_amdgcn_perm(kBig47, kBig03, sl);
    lo_word = (lo_big & ml) | (lo_small & ~ml);
    const uint32_t hi_neg = __builtin_amdgcn_perm(kNeg47, kNeg03, sh);   // uh < 8: value uh - 8 < 0
    const uint32_t hi_pos = __builtin_amdgcn_perm(kPos47, kPos03, sh);   // uh >= 8: value uh - 8
    hi_word = (hi_pos & mh) | (hi_neg & ~mh);
}

// ---------------------------------------------------------------------------------------
// The activation format of the grouped GEMMs: two planes of FP6 (E2M3) codes.
//
// The matrix instruction takes a 6-bit operand at twice the rate of an 8-bit one (measured, two
// waves per SIMD: 9.2 against 4.8 PFLOP/s with FP4 weights), and both planes of the int8 split
// fit 6 bits exactly: q = 16 sh + ul with sh = q >> 4 in [-8, 7] and ul = q & 15 in [0, 15]; an
// E2M3 code c < 16 stands for c / 8 (measured with one-hot probes: codes 0..15 are 0, 0.125, ..
// 1.875), so the low plane's code is ul, the high plane's |sh| with the sign in bit 5, and the
// block scales 2^3 (130) and 2^7 (134) restore ul and 16 sh.  The products and sums stay exact.
//
// Operand layout (one-hot probes): lane l holds column l % 16, k = 32 (l / 16) + n for code
// n = 0..31 at bits 6 n of six registers -- one 32-element weight block in nibble order, like
// the FP4 operand.  In memory a row keeps, per super-block, 384 bytes:
//   [half h][plane][block g][16 B]  (2 x 128 B)  then  [half h][plane][block g][8 B]  (2 x 64 B)
// the first 16 and the last 8 bytes of the 24-byte operand of (plane, block 4 h + g); plane 0 =
// high.  Rows are 128 bytes apart in multiples, so the 128-byte runs are whole cache lines.  The
// n_sb block scales d follow the tiles, padded to a multiple of four (readers fetch them four at
// a time).
// ---------------------------------------------------------------------------------------
constexpr uint32_t kStaged6Bytes = 384;
constexpr int kScaleB6High = 134, kScaleB6Low = 130;
__host__ __device__ inline uint32_t staged6_row_bytes(uint32_t n_sb) {
    return (n_sb * kStaged6Bytes + ((n_sb + 3u) & ~3u) * 4u + 127u) & ~127u;
}
// Four int8 values (one per byte of `q`, any order) -> their codes of the high and of the low
// plane, one per byte, same order.
__device__ __forceinline__ void split_q4_fp6(uint32_t q, uint32_t &hi_codes, uint32_t &lo_codes) {
    lo_codes = q & 0x0F0F0F0Fu;
    const uint32_t n = (q >> 4) & 0x0F0F0F0Fu;   // sh as a two's complement nibble
    // n < 8: code n;  n >= 8: sh = n - 16 < 0, code 0x20 | (16 - n)
    constexpr uint32_t kNeg03 = 0x25262728u, kNeg47 = 0x21222324u;
    const uint32_t s = n & 0x07070707u;
    const uint32_t neg = __builtin_amdgcn_perm(kNeg47, kNeg03, s);
    const uint32_t m = ((n >> 3) & 0x01010101u) * 0xFFu;
    hi_codes = (neg & m) | (s & ~m);
}
// Four code bytes -> 24 bits, byte i at bits 6 i.
__device__ __forceinline__ uint32_t pack_codes4(uint32_t c) {
    return (c & 0x3Fu) | ((c >> 2) & 0xFC0u) | ((c >> 4) & 0x3F000u) | ((c >> 6) & 0xFC0000u);
}
// Byte offset, inside a super-block's 384 bytes, of dword i (0..5) of the operand of
// (half h, plane, block g).
__device__ __forceinline__ uint32_t staged6_off(uint32_t h, uint32_t plane, uint32_t g, uint32_t i) {
    return i < 4u ? h * 128u + plane * 64u + g * 16u + i * 4u : 256u + h * 64u + plane * 32u + g * 8u + (i - 4u) * 4u;
}

// ---------------------------------------------------------------------------------------
// Staged activation tile in LDS, for one super-block (256 k) and NT token columns.
//
// Operand layout of the instruction for one 128-k half (measured with one-hot probes):
//   A, FP4, 4 VGPRs:  lane l holds row l % 16, k = 32 * (l / 16) + n for nibble n = 0..31
//                     (low nibble of byte 0 first) -- exactly one 16-byte weight block;
//   B, FP8, 8 VGPRs:  lane l holds column l % 16; bytes 0..15 are k = 16 * (l / 16) + p,
//                     bytes 16..31 are k = 64 + 16 * (l / 16) + (p - 16).
// The weights' nibble byte j holds element j (low) and element 16 + j (high) of its block,
// so nibble n of block b is element n/2 (n even) or 16 + n/2 (n odd) and sits at
// k = 32 * b + n.  The activation for that k goes to B lane group (k % 64) / 16, byte
// 16 * (k / 64) + k % 16:
//
//   tile[half h][plane][chunk c][kb][column][16 B]    c = k / 64, kb = (k % 64) / 16,
//   plane 0 = high (x16), plane 1 = low.
// A lane reads its operand as the two 16-byte chunks c = 0, 1; consecutive lanes read
// consecutive 16-byte words (NT == 16) or broadcast (NT < 16).
// ---------------------------------------------------------------------------------------
template <int NT>
__device__ __forceinline__ uint32_t tile_off(uint32_t h, uint32_t plane, uint32_t c, uint32_t kb,
                                             uint32_t col) {
    return (((((h * 2u + plane) * 2u + c) * 4u + kb) * NT) + col) * 16u;
}

// One wave converts one Q8_K block (292 B in global memory) into the tile of column `col`.
// lane -> (block b32 = lane / 8, dword d = lane % 8); dword d holds nibble positions
// n = 4d..4d+3 = elements (2d, 16+2d, 2d+1, 17+2d) of the block.
template <int NT>
__device__ __forceinline__ void stage_q8k_block(uint8_t *tile, float *yd_slot,
                                                const uint8_t *__restrict__ blk, uint32_t col,
                                                uint32_t lane) {
    const uint32_t b32 = lane >> 3, d = lane & 7u;
    const int8_t *q8 = (const int8_t *)(blk + 4) + b32 * 32u;
    const uint16_t lo2 = *(const uint16_t *)(q8 + 2u * d);
    const uint16_t hi2 = *(const uint16_t *)(q8 + 16u + 2u * d);
    // nibble positions 4d..4d+3 = elements (2d, 16+2d, 2d+1, 17+2d)
    const uint32_t packed = __builtin_amdgcn_perm((uint32_t)hi2, (uint32_t)lo2, 0x05010400u);
    uint32_t hw, lw;
    split_q4(packed, hw, lw);
    const uint32_t h = b32 >> 2, b = b32 & 3u;
    const uint32_t c = b >> 1, kb = 2u * (b & 1u) + (d >> 2), o = (d & 3u) * 4u;
    *(uint32_t *)(tile + tile_off<NT>(h, 0, c, kb, col) + o) = hw;
    *(uint32_t *)(tile + tile_off<NT>(h, 1, c, kb, col) + o) = lw;
    if (lane == 0) *yd_slot = *(const float *)blk;
}

// LDS-direct loads: lane l of the wave fetches `size` bytes from its global address and the
// hardware writes them to LDS at lds_addr + size * l (lds_addr uniform, passed in M0); no
// vector register holds the data.  They count in vmcnt like any load; the compiler does not
// see them, so the caller waits (s_waitcnt vmcnt) before the LDS reads that depend on them.
// `base` must be uniform; `off` is the lane's unsigned byte offset from it.
// Each helper overwrites M0 (the compiler has no clobber name for it); the kernels that use them
// contain nothing else that needs M0 (no LDS-direct builtins, no indirect register indexing).
__device__ __forceinline__ void lds_dma16(uint32_t lds_addr, const void *base, uint32_t off) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(lds_addr), "v"(off), "s"(base) : "memory");
}
__device__ __forceinline__ void lds_dma4(uint32_t lds_addr, const void *base, uint32_t off) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, %2"
                 :: "s"(lds_addr), "v"(off), "s"(base) : "memory");
}
// per-lane 64-bit address form
__device__ __forceinline__ void lds_dma4_v(uint32_t lds_addr, const void *ptr) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, off"
                 :: "s"(lds_addr), "v"(ptr) : "memory");
}

// Weights of one super-block for the lane's row: its two nibble blocks (halves 0 and 1,
// block kb of each) and the 8 scale bytes.
struct WSuper {
    U4A8 a0, a1;
    U2A4 s;
};

__device__ __forceinline__ WSuper load_wsuper(const uint8_t *__restrict__ row_super, uint32_t kb) {
    WSuper w;
    w.a0 = gload16(row_super + kb * 16u);
    w.a1 = gload16(row_super + 64u + kb * 16u);
    w.s = gload8(row_super + 128u);
    return w;
}

// ---- where a matrix keeps a row's super-blocks ------------------------------------------------
// The engine's rows hold each super-block's 128 nibble bytes and 8 scale bytes together (136
// bytes, so a block starts on a cache line only every 16th time).  The planar form permutes the
// bytes of every 16-row tile within the tile: first the 16 rows' nibble blocks, row-major at
// 128 bytes per super-block -- every block is one whole cache line -- then the tile's scales
// as [super-block][row in tile][8 bytes], so that the scales a 16-row fragment needs of one
// super-block are one line too.  A tile keeps its place and size (16 n_sb 136 bytes, a multiple
// of 128), so whoever streams whole tiles reads the same stretch of memory in either form, and
// consecutive super-blocks of a row are `w_step` bytes apart in nibbles and scales alike.
struct WRow {
    const uint8_t *nib, *sc;
};
__device__ __forceinline__ uint32_t w_step(bool planar) { return planar ? 128u : (uint32_t)kSuperBytes; }
// byte offsets, from the start of the matrix, of a row's first nibble block and first scale group
__device__ __forceinline__ void w_row_offsets(uint32_t row, uint32_t n_sb, bool planar, uint64_t &nib,
                                              uint64_t &sc) {
    if (planar) {
        const uint64_t tile = (uint64_t)(row >> 4) * n_sb * (16u * kSuperBytes);
        nib = tile + (row & 15u) * n_sb * 128u;
        sc = tile + n_sb * 2048u + (row & 15u) * 8u;
    } else {
        nib = (uint64_t)row * n_sb * kSuperBytes;
        sc = nib + 128u;
    }
}
__device__ __forceinline__ WRow w_row(const uint8_t *mat, uint32_t row, uint32_t n_sb, bool planar) {
    uint64_t nib, sc;
    w_row_offsets(row, n_sb, planar, nib, sc);
    return WRow{mat + nib, mat + sc};
}
// super-block at byte offset `off` (= index x w_step) of the row
__device__ __forceinline__ WSuper load_wsuper(const WRow &w, uint64_t off, uint32_t kb) {
    WSuper r;
    r.a0 = gload16(w.nib + off + kb * 16u);
    r.a1 = gload16(w.nib + off + 64u + kb * 16u);
    r.s = gload8(w.sc + off);
    return r;
}

__device__ __forceinline__ v8i b_operand(const uint8_t *tile, uint32_t off0, uint32_t off1) {
    const uint4 lo = *(const uint4 *)(tile + off0);
    const uint4 hi = *(const uint4 *)(tile + off1);
    v8i b = {(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
    return b;
}

// The lane's four B operands of one super-block: {high, low} plane x {half 0, half 1}.
struct BSuper {
    v8i h0, l0, h1, l1;
};

template <int NT>
__device__ __forceinline__ BSuper load_bsuper(const uint8_t *tile, uint32_t kb, uint32_t col) {
    BSuper b;
    b.h0 = b_operand(tile, tile_off<NT>(0, 0, 0, kb, col), tile_off<NT>(0, 0, 1, kb, col));
    b.l0 = b_operand(tile, tile_off<NT>(0, 1, 0, kb, col), tile_off<NT>(0, 1, 1, kb, col));
    b.h1 = b_operand(tile, tile_off<NT>(1, 0, 0, kb, col), tile_off<NT>(1, 0, 1, kb, col));
    b.l1 = b_operand(tile, tile_off<NT>(1, 1, 0, kb, col), tile_off<NT>(1, 1, 1, kb, col));
    return b;
}

// acc[i] += yd * sum_k W[row][k] * q[k]   over one super-block, for the lane's 4 rows
// (4 * (lane / 16) + i) and its column (lane % 16).  Scale bytes: the weights' E8M0 as
// stored (2^(e-127) on E2M1 == 2^(e-128) on the doubled kvalues), 131 (2^4) for the
// activation high plane, 127 (2^0) for the low plane.
__device__ __forceinline__ void mfma_super(v4f &acc, const WSuper &w, const BSuper &b, float yd,
                                           uint32_t kb) {
    const v8i a0 = {(int)w.a0.x, (int)w.a0.y, (int)w.a0.z, (int)w.a0.w, 0, 0, 0, 0};
    const v8i a1 = {(int)w.a1.x, (int)w.a1.y, (int)w.a1.z, (int)w.a1.w, 0, 0, 0, 0};
    const int s0 = (int)((w.s.x >> (kb * 8u)) & 0xFFu);
    const int s1 = (int)((w.s.y >> (kb * 8u)) & 0xFFu);
    v4f c = {0.f, 0.f, 0.f, 0.f};
    c = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a0, b.h0, c, 4, 0, 0, s0, 0, 131);
    c = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a0, b.l0, c, 4, 0, 0, s0, 0, 127);
    c = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a1, b.h1, c, 4, 0, 0, s1, 0, 131);
    c = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a1, b.l1, c, 4, 0, 0, s1, 0, 127);
    acc.x = fmaf(yd, c.x, acc.x);
    acc.y = fmaf(yd, c.y, acc.y);
    acc.z = fmaf(yd, c.z, acc.z);
    acc.w = fmaf(yd, c.w, acc.w);
}

// crates/v4flash-kernels/kernels/swiglu_clamp_weighted.hip:27-36
__device__ __forceinline__ float swiglu_clamp(float g, float u, float clamp, float ew) {
    if (clamp > 1.0e-6f) {
        if (g > clamp) g = clamp;
        if (u > clamp) u = clamp;
        if (u < -clamp) u = -clamp;
    }
    const float sig = 1.0f / (1.0f + expf(-g));
    return g * sig * u * ew;
}

// ---- the hyper-connection combine behind a sublayer --------------------------------------------
// out_hc[t, dst, d] = block[t, d] * post[t, dst] + sum_src comb[t, dst + src * n_hc] * residual_hc[t, src, d]
// (crates/v4flash-kernels/kernels/hc_post.hip:15-34, batched :40-64; sums in f32, src ascending,
// products rounded before they are added).  post / comb of token t start post_stride / comb_stride
// floats behind those of token t - 1, so that one descriptor covers separate arrays
// ([b, n_hc] and [b, n_hc, n_hc]) and the reference's packed "split" rows alike
// (hc_post.hip:66-98: post at n_w, comb at n_w + n_hc of a row of n_w + n_hc + n_hc * n_hc).
// n_hc == 0: no combine.
constexpr uint32_t kMaxHc = 8;
struct HcPost {
    float *out_hc;              // [b, n_hc, n_embd]
    const float *residual_hc;   // [b, n_hc, n_embd]
    const float *post, *comb;
    uint32_t n_hc, post_stride, comb_stride;
};
// one value (token t, element d of n_embd)
__device__ __forceinline__ void hc_post_store(const HcPost &h, uint64_t t, uint32_t d, uint32_t n_embd, float block) {
    const float *post = h.post + t * h.post_stride, *comb = h.comb + t * h.comb_stride;
    const float *res = h.residual_hc + t * h.n_hc * n_embd + d;
    float r[kMaxHc];
#pragma unroll
    for (uint32_t s = 0; s < kMaxHc; s++) r[s] = s < h.n_hc ? res[(uint64_t)s * n_embd] : 0.0f;
    for (uint32_t dst = 0; dst < h.n_hc; dst++) {
        float acc = block * post[dst];
#pragma unroll
        for (uint32_t s = 0; s < kMaxHc; s++)
            if (s < h.n_hc) acc += comb[dst + s * h.n_hc] * r[s];
        h.out_hc[(t * h.n_hc + dst) * n_embd + d] = acc;
    }
}
// four consecutive values (d a multiple of 4)
__device__ __forceinline__ void hc_post_store4(const HcPost &h, uint64_t t, uint32_t d, uint32_t n_embd, float4 block) {
    const float *post = h.post + t * h.post_stride, *comb = h.comb + t * h.comb_stride;
    const float *res = h.residual_hc + t * h.n_hc * n_embd + d;
    float4 r[kMaxHc];
#pragma unroll
    for (uint32_t s = 0; s < kMaxHc; s++)
        r[s] = s < h.n_hc ? *(const float4 *)(res + (uint64_t)s * n_embd) : make_float4(0.f, 0.f, 0.f, 0.f);
    for (uint32_t dst = 0; dst < h.n_hc; dst++) {
        const float pd = post[dst];
        float4 acc = make_float4(block.x * pd, block.y * pd, block.z * pd, block.w * pd);
#pragma unroll
        for (uint32_t s = 0; s < kMaxHc; s++)
            if (s < h.n_hc) {
                const float c = comb[dst + s * h.n_hc];
                acc.x += c * r[s].x; acc.y += c * r[s].y; acc.z += c * r[s].z; acc.w += c * r[s].w;
            }
        *(float4 *)(h.out_hc + (t * h.n_hc + dst) * n_embd + d) = acc;
    }
}

}  // namespace dsx
