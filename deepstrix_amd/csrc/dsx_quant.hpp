// dsx_quant.hpp -- wave-level Q8_K quantization (one wave per 256-element block) and the
// "staged" activation format the expert kernels copy straight into LDS.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "dsx_device.hpp"

namespace dsx {

// 64-lane maximum of a 64-bit key with data-parallel-primitive moves: four steps inside each
// row of 16 lanes, two broadcasts across the rows, the result read from lane 63.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint64_t dpp_mov_u64(uint64_t v) {
    const int lo = __builtin_amdgcn_update_dpp((int)(uint32_t)v, (int)(uint32_t)v, CTRL, ROW_MASK, 0xf, false);
    const int hi = __builtin_amdgcn_update_dpp((int)(uint32_t)(v >> 32), (int)(uint32_t)(v >> 32), CTRL,
                                               ROW_MASK, 0xf, false);
    return ((uint64_t)(uint32_t)hi << 32) | (uint64_t)(uint32_t)lo;
}
template <int CTRL>
__device__ __forceinline__ float dpp_mov_f32(float v) {
    const int b = (int)__float_as_uint(v);
    return __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(b, b, CTRL, 0xf, 0xf, false));
}
// Maximum over the 64 lanes, returned to every lane (all lanes must be active).
__device__ __forceinline__ uint64_t wave_max_u64_dpp(uint64_t v) {
    uint64_t o;
    o = dpp_mov_u64<0xb1, 0xf>(v);   // quad_perm:[1,0,3,2]
    v = o > v ? o : v;
    o = dpp_mov_u64<0x4e, 0xf>(v);   // quad_perm:[2,3,0,1]
    v = o > v ? o : v;
    o = dpp_mov_u64<0x124, 0xf>(v);  // row_ror:4
    v = o > v ? o : v;
    o = dpp_mov_u64<0x128, 0xf>(v);  // row_ror:8: every lane holds its row's maximum
    v = o > v ? o : v;
    o = dpp_mov_u64<0x142, 0xa>(v);  // row_bcast:15 into rows 1 and 3
    v = o > v ? o : v;
    o = dpp_mov_u64<0x143, 0xc>(v);  // row_bcast:31 into rows 2 and 3: lane 63 holds the maximum
    v = o > v ? o : v;
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, 63);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), 63);
    return ((uint64_t)hi << 32) | lo;
}

// 64-lane butterfly reductions.  Every lane ends with the full result.
__device__ __forceinline__ uint64_t wave_max_u64(uint64_t v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const uint64_t other = __shfl_xor(v, o, 64);
        v = other > v ? other : v;
    }
    return v;
}
__device__ __forceinline__ float wave_max_f32(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ __forceinline__ float wave_sum_f32(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// Order-preserving map f32 -> u32 (larger float => larger integer).
__device__ __forceinline__ uint32_t f32_key(float f) {
    const uint32_t b = __float_as_uint(f);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

// Q8_K quantizer: one wave per 256-element block, 4 consecutive elements per lane.
// crates/v4flash-kernels/kernels/q8_k_quantize.hip:23-90
struct Q8kQuant {
    float d;       // 1 / iscale (0 for an all-zero block)
    int q[4];      // the lane's four quantized values
};

__device__ __forceinline__ Q8kQuant q8k_quantize_lane(float4 v, uint32_t lane) {
    // key = (|x| bits, 255 - index): the largest |x| wins, the first one on ties
    const float xs[4] = {v.x, v.y, v.z, v.w};
    uint64_t best = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t idx = lane * 4u + i;
        const uint64_t key = ((uint64_t)(__float_as_uint(xs[i]) & 0x7FFFFFFFu) << 32) | (255u - idx);
        best = key > best ? key : best;
    }
    best = wave_max_u64_dpp(best);  // uniform; every lane of the wave is active here
    const uint32_t amax_bits = (uint32_t)(best >> 32);
    const uint32_t idx = 255u - (uint32_t)(best & 0xFFu);
    float cand = xs[0];
    if ((idx & 3u) == 1u) cand = xs[1];
    if ((idx & 3u) == 2u) cand = xs[2];
    if ((idx & 3u) == 3u) cand = xs[3];
    const float mxv = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(cand), (int)(idx >> 2)));
    Q8kQuant r;
    if (amax_bits == 0u) {
        r.d = 0.0f;
        r.q[0] = r.q[1] = r.q[2] = r.q[3] = 0;
        return r;
    }
    const float iscale = -127.0f / mxv;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        int q = (int)rintf(iscale * xs[i]);
        q = q > 127 ? 127 : q;
        q = q < -128 ? -128 : q;
        r.q[i] = q;
    }
    r.d = 1.0f / iscale;
    return r;
}

// Quantizes one 256-element block exactly as Q8_K does and writes it in the staged format:
// a 512-byte tile of FP8 planes (layout of tile_off<1>) and the block scale d.  The int8
// values never reach memory; they are split as described in dsx_device.hpp.
// Lane l holds elements 4l..4l+3 of the block, i.e. elements 4m..4m+3 (m = l % 8) of the
// 32-element block l / 8.  A tile dword holds nibble positions 4d..4d+3 = elements
// (2d, 16+2d, 2d+1, 17+2d): lanes m and m + 4 of a block exchange their values and build
// dwords d = 2(m % 4) and 2(m % 4) + 1.
__device__ __forceinline__ void quantize_block_to_staged(float4 v, uint32_t lane, uint8_t *tile,
                                                         float *d_out) {
    const Q8kQuant r = q8k_quantize_lane(v, lane);
    const uint32_t mine = (uint32_t)(r.q[0] & 0xFF) | ((uint32_t)(r.q[1] & 0xFF) << 8) |
                          ((uint32_t)(r.q[2] & 0xFF) << 16) | ((uint32_t)(r.q[3] & 0xFF) << 24);
    const uint32_t other = (uint32_t)__shfl_xor((int)mine, 4, 64);
    const uint32_t m = lane & 7u;
    const bool low_half = m < 4u;                   // holds elements < 16 of the block
    const uint32_t lo4 = low_half ? mine : other;   // elements 4mm .. 4mm+3
    const uint32_t hi4 = low_half ? other : mine;   // elements 16+4mm .. 16+4mm+3
    // low-half lane: the first two of each group of four; other: the last two.  Packed in the
    // order of the tile dword's nibble positions (a, b, c, d) = (lo4[k], hi4[k], lo4[k+1], hi4[k+1])
    const uint32_t packed = __builtin_amdgcn_perm(hi4, lo4, low_half ? 0x05010400u : 0x07030602u);
    uint32_t hw, lw;
    split_q4(packed, hw, lw);
    const uint32_t b32 = lane >> 3, d = 2u * (m & 3u) + (low_half ? 0u : 1u);
    const uint32_t h = b32 >> 2, b = b32 & 3u;
    const uint32_t c = b >> 1, kb = 2u * (b & 1u) + (d >> 2), o = (d & 3u) * 4u;
    *(uint32_t *)(tile + tile_off<1>(h, 0, c, kb, 0) + o) = hw;
    *(uint32_t *)(tile + tile_off<1>(h, 1, c, kb, 0) + o) = lw;
    if (lane == 0) *d_out = r.d;
}

// The same block in the grouped GEMMs' format (FP6 planes, dsx_device.hpp): `sb` points at the
// super-block's 384 bytes.  The lane that builds nibble positions 4 d .. 4 d + 3 packs their codes
// into 24 bits; dword i of a block's 24-byte operand takes the tail of group i and the head of
// group i + 1 (groups 0..3 make dwords 0..2, groups 4..7 dwords 3..5), so the lanes of groups
// 0, 1, 2 and 4, 5, 6 each fetch their neighbour's group and store one dword per plane.
__device__ __forceinline__ void quantize_block_to_staged6(float4 v, uint32_t lane, uint8_t *sb,
                                                          float *d_out) {
    const Q8kQuant r = q8k_quantize_lane(v, lane);
    const uint32_t mine = (uint32_t)(r.q[0] & 0xFF) | ((uint32_t)(r.q[1] & 0xFF) << 8) |
                          ((uint32_t)(r.q[2] & 0xFF) << 16) | ((uint32_t)(r.q[3] & 0xFF) << 24);
    const uint32_t other = (uint32_t)__shfl_xor((int)mine, 4, 64);
    const uint32_t m = lane & 7u;
    const bool low_half = m < 4u;
    const uint32_t lo4 = low_half ? mine : other;
    const uint32_t hi4 = low_half ? other : mine;
    const uint32_t packed = __builtin_amdgcn_perm(hi4, lo4, low_half ? 0x05010400u : 0x07030602u);
    uint32_t hc, lc;
    split_q4_fp6(packed, hc, lc);
    const uint32_t gh = pack_codes4(hc), gl = pack_codes4(lc);
    const uint32_t d = 2u * (m & 3u) + (low_half ? 0u : 1u);
    // the lane that holds group d + 1 of the same block: d + 1 even -> m' = (d + 1) / 2, odd -> d / 2 + 4
    const uint32_t dn = (d + 1u) & 7u;
    const uint32_t src = (lane & ~7u) + ((dn & 1u) ? (dn >> 1) + 4u : (dn >> 1));
    const uint32_t nh = (uint32_t)__shfl((int)gh, (int)src, 64);
    const uint32_t nl = (uint32_t)__shfl((int)gl, (int)src, 64);
    const uint32_t i = d & 3u;
    if (i < 3u) {
        const uint32_t b32 = lane >> 3, idx = (d >> 2) * 3u + i;
        const uint32_t wh = (gh >> (8u * i)) | (nh << (24u - 8u * i));
        const uint32_t wl = (gl >> (8u * i)) | (nl << (24u - 8u * i));
        *(uint32_t *)(sb + staged6_off(b32 >> 2, 0, b32 & 3u, idx)) = wh;
        *(uint32_t *)(sb + staged6_off(b32 >> 2, 1, b32 & 3u, idx)) = wl;
    }
    if (lane == 0) *d_out = r.d;
}

// Q8_0 activation quantizer, four consecutive elements per lane, eight lanes per 32-element block
// (crates/v4flash-kernels/kernels/q8_0_matvec.hip:150-177): d = max|x| / 127, q = rint(x / d).
// All lanes of the wave take part (lanes without elements pass zeros).
__device__ __forceinline__ void q8_0_quantize_lane4(float4 v, uint32_t &packed, float &d) {
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
    amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
    amax = fmaxf(amax, __shfl_xor(amax, 4, 64));
    d = amax / 127.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    const float xs[4] = {v.x, v.y, v.z, v.w};
    packed = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        int q = (int)rintf(xs[i] * id);
        q = q > 127 ? 127 : q;
        q = q < -128 ? -128 : q;
        packed |= (uint32_t)(q & 0xFF) << (8 * i);
    }
}

}  // namespace dsx
