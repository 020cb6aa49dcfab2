// dsx_synth.hip -- counter-based synthetic tensors for benchmarks and tests (libdsx_synth.so).
//
// Not part of the MoE operator ABI.  Every value is a pure function of
// (seed, tensor id, element index), computed with integer arithmetic only, so the host
// loops and the device kernels below produce the same bytes and any slice of a tensor
// (one expert, one row) can be generated on its own.
//
//   h(c)      = splitmix64(base + c),  base = splitmix64(seed ^ (tensor_id * 0x9E3779B97F4A7C15))
//   normal(i) = (sum of the twelve 16-bit fields of h(3i), h(3i+1), h(3i+2) - 393210) / 65536
//               (Irwin-Hall of order 12: mean 0, variance 1, support +-6)
// Weights: normal * sigma, quantized to MXFP4 (E2M1 x E8M0 per 32, scale =
// 2^ceil(log2(amax/6)), nearest code with ties to the even code) in the engine's
// super-block layout, or to Q8_0 rows ([blocks x f16 d][blocks x 32 i8], d = amax/127,
// q = round-half-away(x / d)).
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <algorithm>
#include <math.h>
#include <stdint.h>
#include <string.h>

#define HD __host__ __device__ __forceinline__

namespace {

HD uint64_t splitmix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

HD uint64_t stream_base(uint64_t seed, uint64_t tensor_id) {
    return splitmix64(seed ^ (tensor_id * 0x9E3779B97F4A7C15ull));
}

HD uint32_t sum16(uint64_t h) {
    return (uint32_t)(h & 0xFFFF) + (uint32_t)((h >> 16) & 0xFFFF) + (uint32_t)((h >> 32) & 0xFFFF) +
           (uint32_t)(h >> 48);
}

HD float normal_at(uint64_t base, uint64_t i) {
    const uint32_t s = sum16(splitmix64(base + 3 * i)) + sum16(splitmix64(base + 3 * i + 1)) +
                       sum16(splitmix64(base + 3 * i + 2));
    return (float)((int32_t)s - 393210) * (1.0f / 65536.0f);
}

HD int e2m1_index(float ax) {
    const float grid[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};
    int best = 0;
    float best_diff = fabsf(ax - grid[0]);
    for (int i = 1; i < 8; i++) {
        const float diff = fabsf(ax - grid[i]);
        if (diff < best_diff || (diff == best_diff && (i & 1) == 0 && (best & 1) != 0)) {
            best = i;
            best_diff = diff;
        }
    }
    return best;
}

// One 32-element block of row-major element index i0 .. i0+31 -> 16 nibble bytes + scale byte.
HD void mxfp4_block(uint64_t base, uint64_t i0, float sigma, uint8_t *nib16, uint8_t *scale_byte) {
    float x[32];
    float amax = 0.0f;
    for (int j = 0; j < 32; j++) {
        x[j] = normal_at(base, i0 + j) * sigma;
        const float a = fabsf(x[j]);
        if (a > amax) amax = a;
    }
    if (amax < 7.052966104933725e-38f) amax = 7.052966104933725e-38f;
    const float t = amax / 6.0f;
    int e;
    const float m = frexpf(t, &e);
    const int cexp = (m == 0.5f) ? e - 1 : e;
    const float scale = ldexpf(1.0f, cexp);
    *scale_byte = (uint8_t)(cexp + 127);
    uint8_t code[32];
    for (int j = 0; j < 32; j++) {
        float q = x[j] / scale;
        if (q > 6.0f) q = 6.0f;
        if (q < -6.0f) q = -6.0f;
        code[j] = (uint8_t)(e2m1_index(fabsf(q)) | ((x[j] < 0.0f) ? 8 : 0));
    }
    for (int j = 0; j < 16; j++) nib16[j] = (uint8_t)(code[j] | (code[j + 16] << 4));
}

HD uint16_t f32_to_f16_bits(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    const uint32_t mant = x & 0x007fffffu;
    const int exp = (int)((x >> 23) & 0xffu);
    if (exp == 0xff) return (uint16_t)(sign | 0x7c00u | (mant ? 0x0200u : 0u));
    const int e = exp - 127 + 15;
    if (e >= 0x1f) return (uint16_t)(sign | 0x7c00u);
    if (e <= 0) {
        if (e < -10) return sign;
        const uint32_t m = mant | 0x00800000u;
        const uint32_t shift = (uint32_t)(14 - e);
        const uint16_t half_mant = (uint16_t)(m >> shift);
        const uint32_t round_bit = 1u << (shift - 1);
        uint16_t result = (uint16_t)(sign | half_mant);
        if ((m & round_bit) && ((m & (round_bit - 1)) || (half_mant & 1))) result++;
        return result;
    }
    const uint16_t half_mant = (uint16_t)(mant >> 13);
    uint16_t result = (uint16_t)(sign | ((uint16_t)e << 10) | half_mant);
    if ((mant & 0x1000u) && ((mant & 0x0fffu) || (half_mant & 1))) result++;
    return result;
}

// One Q8_0 block: f16 scale bits + 32 int8.
HD void q8_0_block(uint64_t base, uint64_t i0, float sigma, uint16_t *d_bits, int8_t *q32) {
    float x[32];
    float amax = 0.0f;
    for (int j = 0; j < 32; j++) {
        x[j] = normal_at(base, i0 + j) * sigma;
        const float a = fabsf(x[j]);
        if (a > amax) amax = a;
    }
    const float d = amax / 127.0f;
    const float id = (d == 0.0f) ? 0.0f : 1.0f / d;
    *d_bits = f32_to_f16_bits(d);
    for (int j = 0; j < 32; j++) q32[j] = (int8_t)roundf(x[j] * id);
}

// Block index b (row-major over [n_rows, cols/32]) of a tensor whose first row has global
// element index elem0.
HD void mxfp4_store(uint8_t *dst, uint64_t base, uint64_t elem0, uint64_t b, uint32_t cols,
                    float sigma) {
    const uint64_t bpr = cols / 32u;
    const uint64_t r = b / bpr, j = b - r * bpr;
    uint8_t *sup = dst + r * bpr * 17u + (j >> 3) * 136u;
    const uint32_t k = (uint32_t)(j & 7u);
    uint8_t nib[16], sc;
    mxfp4_block(base, elem0 + r * cols + j * 32u, sigma, nib, &sc);
    for (int i = 0; i < 16; i++) sup[k * 16u + i] = nib[i];
    sup[128u + k] = sc;
}

HD void q8_0_store(uint8_t *dst, uint64_t base, uint64_t elem0, uint64_t b, uint32_t cols,
                   float sigma) {
    const uint64_t bpr = cols / 32u;
    const uint64_t r = b / bpr, j = b - r * bpr;
    uint8_t *row = dst + r * bpr * 34u;
    uint16_t d;
    int8_t q[32];
    q8_0_block(base, elem0 + r * cols + j * 32u, sigma, &d, q);
    row[j * 2u] = (uint8_t)(d & 0xff);
    row[j * 2u + 1] = (uint8_t)(d >> 8);
    for (int i = 0; i < 32; i++) row[bpr * 2u + j * 32u + i] = (uint8_t)q[i];
}

__global__ void k_normal(float *out, uint64_t base, uint64_t offset, uint64_t n, float sigma,
                         float mean) {
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = normal_at(base, offset + i) * sigma + mean;
}
__global__ void k_mxfp4(uint8_t *dst, uint64_t base, uint64_t elem0, uint64_t n_blocks,
                        uint32_t cols, float sigma) {
    const uint64_t b = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b < n_blocks) mxfp4_store(dst, base, elem0, b, cols, sigma);
}
__global__ void k_q8_0(uint8_t *dst, uint64_t base, uint64_t elem0, uint64_t n_blocks,
                       uint32_t cols, float sigma) {
    const uint64_t b = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b < n_blocks) q8_0_store(dst, base, elem0, b, cols, sigma);
}

// Plain streaming copy, 16 bytes per thread per trip: the known-traffic kernel that hardware
// byte counters are scaled against (reads n16 * 16 bytes, writes n16 * 16 bytes).
__global__ __launch_bounds__(256) void k_copy16(uint4 *__restrict__ dst, const uint4 *__restrict__ src,
                                                uint64_t n16) {
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride)
        dst[i] = src[i];
}

// Plain streaming read: every thread XORs the 16-byte words it reads (four independent loads per
// trip) and every wave stores one word of its own (sink holds 4 words per workgroup), so that next
// to nothing is written back but the loads cannot be dropped.  What a read of a given size reaches on a device: the ceiling a weight-streaming kernel
// is measured against.
__global__ __launch_bounds__(256) void k_read16(uint32_t *__restrict__ sink, const uint4 *__restrict__ src,
                                                uint64_t n16) {
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    uint4 a = {0u, 0u, 0u, 0u}, b = a, c = a, d = a;
    uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    for (; i + 3u * stride < n16; i += 4u * stride) {
        const uint4 v0 = src[i], v1 = src[i + stride], v2 = src[i + 2u * stride], v3 = src[i + 3u * stride];
        a.x ^= v0.x; a.y ^= v0.y; a.z ^= v0.z; a.w ^= v0.w;
        b.x ^= v1.x; b.y ^= v1.y; b.z ^= v1.z; b.w ^= v1.w;
        c.x ^= v2.x; c.y ^= v2.y; c.z ^= v2.z; c.w ^= v2.w;
        d.x ^= v3.x; d.y ^= v3.y; d.z ^= v3.z; d.w ^= v3.w;
    }
    for (; i < n16; i += stride) {
        const uint4 v0 = src[i];
        a.x ^= v0.x; a.y ^= v0.y; a.z ^= v0.z; a.w ^= v0.w;
    }
    uint32_t r = a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w ^ c.x ^ c.y ^ c.z ^ c.w ^ d.x ^ d.y ^ d.z ^ d.w;
    for (int o = 32; o > 0; o >>= 1) r ^= __shfl_xor(r, o, 64);
    if ((threadIdx.x & 63u) == 0u) sink[blockIdx.x * 4u + (threadIdx.x >> 6)] = r;
}


// The same read, shaped like the decode kernels' weight stream: a matrix of MXFP4 rows (n_sb
// super-blocks of 136 bytes each), one workgroup per 16-row tile, its four waves taking every fourth
// super-block, two super-blocks in flight per wave.  OPERAND: every lane loads what the matrix
// instruction wants from it -- row lane % 16, block lane / 16: 16 bytes at 16 (lane / 16), 16 bytes
// 64 further on, the row's 8 scale bytes -- as the decode and by-expert kernels do; otherwise the
// same bytes in memory order (8 rows x 128 bytes per load, the scales by 16 lanes).  What a kernel
// that reads weights tile by tile reaches, whatever it computes.
typedef uint32_t rt_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t rt_u32x2 __attribute__((ext_vector_type(2)));
typedef rt_u32x4 rt_u32x4_a8 __attribute__((aligned(8)));
typedef rt_u32x2 rt_u32x2_a4 __attribute__((aligned(4)));
__device__ __forceinline__ rt_u32x4 rt_ld16(const uint8_t *p) { return *(const rt_u32x4_a8 *)p; }
__device__ __forceinline__ rt_u32x2 rt_ld8(const uint8_t *p) { return *(const rt_u32x2_a4 *)p; }

template <bool OPERAND>
__global__ __launch_bounds__(256) void k_read_tiles(uint32_t *__restrict__ sink, const uint8_t *__restrict__ w,
                                                    uint32_t n_sb) {
    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u;
    const uint32_t gx = gridDim.x;
    // (workgroup ids go round the 8 XCDs: an XCD's tiles are contiguous, as in the decode kernels)
    const uint32_t bx = (gx & 7u) == 0u ? (blockIdx.x & 7u) * (gx >> 3) + (blockIdx.x >> 3) : blockIdx.x;
    const uint64_t row_bytes = (uint64_t)n_sb * 136u;
    const uint8_t *tile = w + (uint64_t)bx * 16u * row_bytes;
    const uint8_t *p0, *p1, *ps;
    bool with_scales = true;
    if (OPERAND) {
        const uint8_t *row = tile + (lane & 15u) * row_bytes;
        p0 = row + (lane >> 4) * 16u;
        p1 = p0 + 64u;
        ps = row + 128u;
    } else {
        p0 = tile + (lane >> 3) * row_bytes + (lane & 7u) * 16u;
        p1 = p0 + 8u * row_bytes;
        ps = tile + (lane & 15u) * row_bytes + 128u;
        with_scales = lane < 16u;
    }
    rt_u32x4 a0[2], a1[2];
    rt_u32x2 s[2] = {};
    uint32_t acc = 0;
    uint32_t sb = wave;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const uint32_t b = min(sb + 4u * (uint32_t)i, n_sb - 1u) * 136u;
        a0[i] = rt_ld16(p0 + b);
        a1[i] = rt_ld16(p1 + b);
        if (with_scales) s[i] = rt_ld8(ps + b);
    }
    for (; sb < n_sb; sb += 8u) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            if (sb + 4u * (uint32_t)i < n_sb)   // (uniform over the wave)
                acc ^= a0[i].x ^ a0[i].y ^ a0[i].z ^ a0[i].w ^ a1[i].x ^ a1[i].y ^ a1[i].z ^ a1[i].w ^ s[i].x ^ s[i].y;
            // (past the end of the row: its last super-block again, never folded in)
            const uint32_t b = min(sb + 8u + 4u * (uint32_t)i, n_sb - 1u) * 136u;
            a0[i] = rt_ld16(p0 + b);
            a1[i] = rt_ld16(p1 + b);
            if (with_scales) s[i] = rt_ld8(ps + b);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // (the last refills are never folded in: every byte of the tile counts once, the scales in
    // operand order once per lane group)
    for (int o = 32; o > 0; o >>= 1) acc ^= __shfl_xor(acc, o, 64);
    if (lane == 0) sink[blockIdx.x * 4u + wave] = acc;
}

}  // namespace

extern "C" {

// out[i] = normal(offset + i) * sigma + mean   (the multiply-add is two rounded f32 ops)
void dsx_synth_normal_host(float *out, uint64_t seed, uint64_t tensor_id, uint64_t offset,
                           uint64_t n, float sigma, float mean) {
    const uint64_t base = stream_base(seed, tensor_id);
    for (uint64_t i = 0; i < n; i++) {
        const float v = normal_at(base, offset + i) * sigma;
        out[i] = v + mean;
    }
}

// n_rows rows of `cols` elements starting at global element index elem0, as MXFP4 rows.
void dsx_synth_mxfp4_host(uint8_t *dst, uint64_t seed, uint64_t tensor_id, uint64_t elem0,
                          uint64_t n_rows, uint32_t cols, float sigma) {
    const uint64_t base = stream_base(seed, tensor_id);
    const uint64_t nb = n_rows * (cols / 32u);
    for (uint64_t b = 0; b < nb; b++) mxfp4_store(dst, base, elem0, b, cols, sigma);
}

void dsx_synth_q8_0_host(uint8_t *dst, uint64_t seed, uint64_t tensor_id, uint64_t elem0,
                         uint64_t n_rows, uint32_t cols, float sigma) {
    const uint64_t base = stream_base(seed, tensor_id);
    const uint64_t nb = n_rows * (cols / 32u);
    for (uint64_t b = 0; b < nb; b++) q8_0_store(dst, base, elem0, b, cols, sigma);
}

int dsx_synth_normal_dev(void *stream, float *out, uint64_t seed, uint64_t tensor_id,
                         uint64_t offset, uint64_t n, float sigma, float mean) {
    if (n == 0) return 0;
    hipLaunchKernelGGL(k_normal, dim3((uint32_t)((n + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, out, stream_base(seed, tensor_id), offset, n, sigma, mean);
    return (int)hipGetLastError();
}

int dsx_synth_mxfp4_dev(void *stream, uint8_t *dst, uint64_t seed, uint64_t tensor_id,
                        uint64_t elem0, uint64_t n_rows, uint32_t cols, float sigma) {
    const uint64_t nb = n_rows * (cols / 32u);
    if (nb == 0) return 0;
    hipLaunchKernelGGL(k_mxfp4, dim3((uint32_t)((nb + 127) / 128)), dim3(128), 0,
                       (hipStream_t)stream, dst, stream_base(seed, tensor_id), elem0, nb, cols, sigma);
    return (int)hipGetLastError();
}

int dsx_synth_q8_0_dev(void *stream, uint8_t *dst, uint64_t seed, uint64_t tensor_id,
                       uint64_t elem0, uint64_t n_rows, uint32_t cols, float sigma) {
    const uint64_t nb = n_rows * (cols / 32u);
    if (nb == 0) return 0;
    hipLaunchKernelGGL(k_q8_0, dim3((uint32_t)((nb + 127) / 128)), dim3(128), 0,
                       (hipStream_t)stream, dst, stream_base(seed, tensor_id), elem0, nb, cols, sigma);
    return (int)hipGetLastError();
}

// dst[0 .. bytes) = src[0 .. bytes); bytes % 16 == 0, both 16-byte aligned.
int dsx_synth_copy_dev(void *stream, void *dst, const void *src, uint64_t bytes) {
    if (bytes == 0) return 0;
    if (bytes % 16u || (uintptr_t)dst % 16u || (uintptr_t)src % 16u) return (int)hipErrorInvalidValue;
    const uint64_t n16 = bytes / 16u;
    const uint32_t grid = (uint32_t)std::min<uint64_t>((n16 + 255) / 256, 256u * 16u);
    hipLaunchKernelGGL(k_copy16, dim3(grid), dim3(256), 0, (hipStream_t)stream, (uint4 *)dst,
                       (const uint4 *)src, n16);
    return (int)hipGetLastError();
}

// Reads `bytes` bytes of src (see k_read16); sink: 4 words per workgroup, i.e. 64 KiB for the
// default of 4096 workgroups (`workgroups` = 0: sixteen per compute unit of a 256-unit device).
int dsx_synth_read_dev(void *stream, void *sink, const void *src, uint64_t bytes, uint32_t workgroups) {
    if (bytes == 0) return 0;
    if (bytes % 16u || (uintptr_t)src % 16u || (uintptr_t)sink % 4u) return (int)hipErrorInvalidValue;
    const uint64_t n16 = bytes / 16u;
    const uint32_t want = workgroups ? workgroups : 256u * 16u;
    const uint32_t grid = (uint32_t)std::min<uint64_t>((n16 + 255) / 256, want);
    hipLaunchKernelGGL(k_read16, dim3(grid), dim3(256), 0, (hipStream_t)stream, (uint32_t *)sink,
                       (const uint4 *)src, n16);
    return (int)hipGetLastError();
}

// Reads n_tiles 16-row tiles of an MXFP4 matrix with n_sb super-blocks per row (n_tiles * 16 * n_sb * 136
// bytes at src) the way the decode kernels stream weights (see k_read_tiles); operand_order = 0: the
// same bytes in memory order.  sink: 4 words per tile.
int dsx_synth_read_tiles_dev(void *stream, void *sink, const void *src, uint32_t n_tiles, uint32_t n_sb,
                             int operand_order) {
    if (n_tiles == 0) return 0;
    if (n_sb == 0 || (uintptr_t)src % 8u || (uintptr_t)sink % 4u) return (int)hipErrorInvalidValue;
    if (operand_order)
        hipLaunchKernelGGL(k_read_tiles<true>, dim3(n_tiles), dim3(256), 0, (hipStream_t)stream, (uint32_t *)sink,
                           (const uint8_t *)src, n_sb);
    else
        hipLaunchKernelGGL(k_read_tiles<false>, dim3(n_tiles), dim3(256), 0, (hipStream_t)stream, (uint32_t *)sink,
                           (const uint8_t *)src, n_sb);
    return (int)hipGetLastError();
}

}  // extern "C"
