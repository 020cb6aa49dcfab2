/*
 * dsx_oracle.c -- CPU restatement of the deepstrix MoE feed-forward arithmetic.
 * TEST INFRASTRUCTURE ONLY; see dsx_oracle.h for scope and parity status.
 * Citations are relative to the reference tree; K/ = crates/v4flash-kernels/,
 * C/ = crates/v4flash-core/.
 */
#include "dsx_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static inline float bits_to_f32(uint32_t b) {
    float f;
    memcpy(&f, &b, 4);
    return f;
}
static inline uint32_t f32_to_bits(float f) {
    uint32_t b;
    memcpy(&b, &f, 4);
    return b;
}

/* ------------------------------------------------------------------------ */
/* scalar formats                                                            */
/* ------------------------------------------------------------------------ */

/* C/src/kquants.rs:23-47 */
float dsx_ref_f16_to_f32(uint16_t bits) {
    uint32_t sign = (bits >> 15) & 1u, exp = (bits >> 10) & 0x1fu, mant = bits & 0x3ffu;
    uint32_t out;
    if (exp == 0) {
        if (mant == 0) {
            out = sign << 31;
        } else {
            int e = -14;
            uint32_t m = mant;
            while ((m & 0x400u) == 0) {
                m <<= 1;
                e -= 1;
            }
            m &= 0x3ffu;
            out = (sign << 31) | ((uint32_t)(e + 127) << 23) | (m << 13);
        }
    } else if (exp == 0x1f) {
        out = (sign << 31) | (0xffu << 23) | (mant << 13);
    } else {
        out = (sign << 31) | ((exp + 112u) << 23) | (mant << 13);
    }
    return bits_to_f32(out);
}

/* C/src/kquants.rs:51-85 */
uint16_t dsx_ref_f32_to_f16(float f) {
    uint32_t x = f32_to_bits(f);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t mant = x & 0x007fffffu;
    int exp = (int)((x >> 23) & 0xffu);
    if (exp == 0xff) return (uint16_t)(sign | 0x7c00u | (mant ? 0x0200u : 0u));
    int e = exp - 127 + 15;
    if (e >= 0x1f) return (uint16_t)(sign | 0x7c00u);
    if (e <= 0) {
        if (e < -10) return sign;
        uint32_t m = mant | 0x00800000u;
        uint32_t shift = (uint32_t)(14 - e);
        uint16_t half_mant = (uint16_t)(m >> shift);
        uint32_t round_bit = 1u << (shift - 1);
        uint16_t result = (uint16_t)(sign | half_mant);
        if ((m & round_bit) && ((m & (round_bit - 1)) || (half_mant & 1))) result++;
        return result;
    }
    uint16_t half_mant = (uint16_t)(mant >> 13);
    uint16_t result = (uint16_t)(sign | ((uint16_t)e << 10) | half_mant);
    if ((mant & 0x1000u) && ((mant & 0x0fffu) || (half_mant & 1))) result++;
    return result;
}

/* C/src/hf_v41.rs:93-95 */
float dsx_ref_bf16_to_f32(uint16_t bits) { return bits_to_f32((uint32_t)bits << 16); }

uint16_t dsx_ref_f32_to_bf16(float f) {
    uint32_t x = f32_to_bits(f);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
    uint32_t lsb = (x >> 16) & 1u;
    x += 0x7fffu + lsb;
    return (uint16_t)(x >> 16);
}

/* C/src/hf_v41.rs:99-105 */
float dsx_ref_e8m0_to_f32(uint8_t e) {
    if (e == 0xff) return NAN;
    if (e == 0) return bits_to_f32(1u << 22);
    return bits_to_f32((uint32_t)e << 23);
}

/* K/src/mxfp4_tables.rs:38-45 */
float dsx_ref_e8m0_half_to_f32(uint8_t e) {
    uint32_t bits = (e < 2) ? (0x00200000u << e) : (((uint32_t)e - 1u) << 23);
    return bits_to_f32(bits);
}

/* C/src/hf_v41.rs:109-118 */
float dsx_ref_e4m3_to_f32(uint8_t b) {
    if ((b & 0x7f) == 0x7f) return NAN;
    float sign = (b & 0x80) ? -1.0f : 1.0f;
    int e = (b >> 3) & 0xf;
    float m = (float)(b & 7);
    float v = (e == 0) ? m * ldexpf(1.0f, -9) : (1.0f + m / 8.0f) * ldexpf(1.0f, e - 7);
    return sign * v;
}

/* ------------------------------------------------------------------------ */
/* MXFP4                                                                     */
/* ------------------------------------------------------------------------ */

/* K/src/mxfp4_tables.rs:8 */
static const int8_t KVALUES[16] = {0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12};

/* One 32-element block: byte j of qs holds element j (low nibble) and element
 * 16+j (high nibble); value = kvalues * 2^(e-128)
 * (external/ds4-patches/0010-iq3xxs-iq2s-mxfp4-cpu-quants.patch:393-404). */
static void mxfp4_dequant_block(uint8_t e, const uint8_t *qs, float *y) {
    const float d = dsx_ref_e8m0_half_to_f32(e);
    for (int j = 0; j < 16; j++) {
        y[j] = (float)KVALUES[qs[j] & 0x0f] * d;
        y[j + 16] = (float)KVALUES[qs[j] >> 4] * d;
    }
}

void dsx_ref_mxfp4_dequant_ggml(const uint8_t *blocks, float *y, size_t n) {
    for (size_t b = 0; b < n / 32; b++)
        mxfp4_dequant_block(blocks[b * 17], blocks + b * 17 + 1, y + b * 32);
}

/* K/src/mxfp4_tables.rs:10-36: block k's nibbles at k*16, its scale at 128+k. */
void dsx_ref_mxfp4_dequant_v2(const uint8_t *rows, float *y, size_t n_rows, size_t cols) {
    const size_t nsb = cols / 256;
    for (size_t r = 0; r < n_rows; r++)
        for (size_t s = 0; s < nsb; s++) {
            const uint8_t *sup = rows + (r * nsb + s) * 136;
            for (int k = 0; k < 8; k++)
                mxfp4_dequant_block(sup[128 + k], sup + k * 16, y + r * cols + s * 256 + k * 32);
        }
}

/* C/src/hf_v41.rs:1208-1232 */
void dsx_ref_mxfp4_repack_hf_to_v2(const uint8_t *packed, const uint8_t *scale, uint8_t *dst,
                                   size_t out, size_t nb) {
    const size_t half = nb * 16;
    for (size_t r = 0; r < out; r++) {
        const uint8_t *prow = packed + r * half;
        const uint8_t *srow = scale + r * nb;
        uint8_t *drow = dst + r * nb * 17;
        for (size_t sb = 0; sb < nb / 8; sb++) {
            uint8_t *sup = drow + sb * 136;
            for (size_t k = 0; k < 8; k++) {
                const size_t j = sb * 8 + k;
                sup[128 + k] = srow[j];
                const uint8_t *pb = prow + j * 16;
                for (size_t i = 0; i < 8; i++) {
                    const uint8_t lo = pb[i], hi = pb[8 + i];
                    sup[k * 16 + 2 * i] = (uint8_t)((lo & 0x0f) | (hi << 4));
                    sup[k * 16 + 1 + 2 * i] = (uint8_t)((lo >> 4) | (hi & 0xf0));
                }
            }
        }
    }
}

/* Inverse of the above (used to check repack . unpack == id). */
void dsx_ref_mxfp4_unpack_v2_to_hf(const uint8_t *src, uint8_t *packed, uint8_t *scale,
                                   size_t out, size_t nb) {
    const size_t half = nb * 16;
    for (size_t r = 0; r < out; r++)
        for (size_t j = 0; j < nb; j++) {
            const uint8_t *sup = src + r * nb * 17 + (j / 8) * 136;
            const size_t k = j % 8;
            scale[r * nb + j] = sup[128 + k];
            uint8_t *pb = packed + r * half + j * 16;
            for (size_t i = 0; i < 8; i++) {
                const uint8_t a = sup[k * 16 + 2 * i], b = sup[k * 16 + 2 * i + 1];
                pb[i] = (uint8_t)((a & 0x0f) | ((b & 0x0f) << 4));
                pb[8 + i] = (uint8_t)((a >> 4) | (b & 0xf0));
            }
        }
}

/* Nearest E2M1 magnitude index, ties to the even index
 * (K/tests/indexer_pipeline.rs:574-588). */
static int e2m1_index(float ax) {
    static const float grid[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};
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

/* K/kernels/indexer_qat.hip:60-73: amax floored at 6*2^-126, scale =
 * 2^ceil(log2(amax/6)) via frexp, q = clamp(x/scale, +-6) -> nearest E2M1. */
void dsx_ref_mxfp4_quantize_v2(const float *x, uint8_t *dst, size_t n_rows, size_t cols) {
    const size_t nsb = cols / 256;
    for (size_t r = 0; r < n_rows; r++)
        for (size_t s = 0; s < nsb; s++) {
            uint8_t *sup = dst + (r * nsb + s) * 136;
            for (int k = 0; k < 8; k++) {
                const float *xb = x + r * cols + s * 256 + (size_t)k * 32;
                float amax = 0.0f;
                for (int j = 0; j < 32; j++) {
                    const float a = fabsf(xb[j]);
                    if (a > amax) amax = a;
                }
                if (amax < 7.052966104933725e-38f) amax = 7.052966104933725e-38f;
                const float t = amax / 6.0f;
                int e;
                const float m = frexpf(t, &e);
                const int cexp = (m == 0.5f) ? e - 1 : e;
                const float scale = ldexpf(1.0f, cexp);
                sup[128 + k] = (uint8_t)(cexp + 127);
                uint8_t code[32];
                for (int j = 0; j < 32; j++) {
                    float q = xb[j] / scale;
                    if (q > 6.0f) q = 6.0f;
                    if (q < -6.0f) q = -6.0f;
                    const int idx = e2m1_index(fabsf(q));
                    code[j] = (uint8_t)(idx | ((xb[j] < 0.0f) ? 8 : 0));
                }
                for (int j = 0; j < 16; j++)
                    sup[k * 16 + j] = (uint8_t)(code[j] | (code[j + 16] << 4));
            }
        }
}

/* ------------------------------------------------------------------------ */
/* Q8_0                                                                      */
/* ------------------------------------------------------------------------ */

/* Rust's `f32 as i8`: NaN -> 0, out of range saturates. */
static int8_t sat_i8(float v) {
    if (v != v) return 0;
    if (v >= 127.0f) return 127;
    if (v <= -128.0f) return -128;
    return (int8_t)v;
}

/* C/src/hf_v41.rs:125-137: d = amax/127 (f32), id = 1/d, q = round-half-away. */
void dsx_ref_q8_0_quantize_block(const float *x, uint8_t *out) {
    float amax = 0.0f;
    for (int i = 0; i < 32; i++) {
        const float a = fabsf(x[i]);
        if (a > amax) amax = a; /* f32::max fold */
    }
    const float d = amax / 127.0f;
    const float id = (d == 0.0f) ? 0.0f : 1.0f / d;
    const uint16_t h = dsx_ref_f32_to_f16(d);
    out[0] = (uint8_t)(h & 0xff);
    out[1] = (uint8_t)(h >> 8);
    for (int i = 0; i < 32; i++) out[2 + i] = (uint8_t)sat_i8(roundf(x[i] * id));
}

/* K/src/weights.rs:225-240 */
void dsx_ref_q8_0_repack_rows(const uint8_t *ggml, uint8_t *dst, size_t n_rows, size_t blocks) {
    const size_t row_bytes = blocks * 34;
    for (size_t r = 0; r < n_rows; r++) {
        const uint8_t *s = ggml + r * row_bytes;
        uint8_t *d = dst + r * row_bytes;
        for (size_t b = 0; b < blocks; b++) {
            memcpy(d + b * 2, s + b * 34, 2);
            memcpy(d + blocks * 2 + b * 32, s + b * 34 + 2, 32);
        }
    }
}

/* C/src/hf_v41.rs:728-805 (read_q8): a checkpoint matrix [out, inn] in f32 (dtype 0), bf16
 * (1) or fp8-e4m3 with an E8M0 scale grid [sr, sc] that tiles it exactly (2) -> ggml Q8_0
 * blocks (34 B each, row-major).  Returns 0, or -1 where the reference returns Err. */
int dsx_ref_q8_0_from_hf(const void *src, const uint8_t *scale, int dtype, size_t out, size_t inn,
                         size_t sr, size_t sc, uint8_t *dst) {
    if (inn % 32) return -1;
    size_t br = 0, bc = 0;
    if (dtype == 2) {
        if (!scale || sr == 0 || sc == 0) return -1;
        br = out / sr;
        bc = inn / sc;
        if (br * sr != out || bc * sc != inn) return -1;
    } else if (dtype != 0 && dtype != 1) {
        return -1;
    }
    float *f = (float *)malloc(inn * sizeof(float));
    for (size_t r = 0; r < out; r++) {
        for (size_t c = 0; c < inn; c++) {
            if (dtype == 0)
                f[c] = ((const float *)src)[r * inn + c];
            else if (dtype == 1)
                f[c] = dsx_ref_bf16_to_f32(((const uint16_t *)src)[r * inn + c]);
            else
                f[c] = dsx_ref_e4m3_to_f32(((const uint8_t *)src)[r * inn + c]) *
                       dsx_ref_e8m0_to_f32(scale[(r / br) * sc + c / bc]);
        }
        for (size_t b = 0; b < inn / 32; b++)
            dsx_ref_q8_0_quantize_block(f + b * 32, dst + (r * (inn / 32) + b) * 34);
    }
    free(f);
    return 0;
}

void dsx_ref_q8_0_quantize_rows(const float *x, uint8_t *dst, size_t n_rows, size_t cols) {
    const size_t blocks = cols / 32;
    uint8_t *tmp = (uint8_t *)malloc(blocks * 34);
    for (size_t r = 0; r < n_rows; r++) {
        for (size_t b = 0; b < blocks; b++)
            dsx_ref_q8_0_quantize_block(x + r * cols + b * 32, tmp + b * 34);
        dsx_ref_q8_0_repack_rows(tmp, dst + r * blocks * 34, 1, blocks);
    }
    free(tmp);
}

/* C/src/kquants.rs:105-111 applied to the engine row layout. */
void dsx_ref_q8_0_dequant_rows(const uint8_t *rows, float *y, size_t n_rows, size_t cols) {
    const size_t blocks = cols / 32;
    for (size_t r = 0; r < n_rows; r++) {
        const uint8_t *wr = rows + r * blocks * 34;
        const int8_t *q = (const int8_t *)(wr + blocks * 2);
        for (size_t b = 0; b < blocks; b++) {
            const float d = dsx_ref_f16_to_f32((uint16_t)(wr[b * 2] | (wr[b * 2 + 1] << 8)));
            for (int i = 0; i < 32; i++) y[r * cols + b * 32 + i] = d * (float)q[b * 32 + i];
        }
    }
}

/* K/kernels/q8_0_matvec.hip:150-177 */
void dsx_ref_q8_0_quantize_act(const float *x, int8_t *xq, float *xscale, size_t blocks) {
    for (size_t b = 0; b < blocks; b++) {
        const float *xb = x + b * 32;
        float amax = 0.0f;
        for (int i = 0; i < 32; i++) amax = fmaxf(amax, fabsf(xb[i]));
        const float d = amax / 127.0f;
        const float id = (d != 0.0f) ? 1.0f / d : 0.0f;
        xscale[b] = d;
        for (int i = 0; i < 32; i++) {
            int q = (int)lrintf(xb[i] * id);
            if (q > 127) q = 127;
            if (q < -128) q = -128;
            xq[b * 32 + i] = (int8_t)q;
        }
    }
}

/* K/kernels/q8_0_matvec.hip:64-104: lane l owns blocks l, l+32, ...;
 * acc += f16(d_w) * xscale * (float)dot; then v += shfl_down(v, 16/8/4/2/1). */
float dsx_ref_dot_q8_0(size_t blocks, const uint8_t *wrow, const int8_t *xq, const float *xscale) {
    const int8_t *quants = (const int8_t *)(wrow + blocks * 2);
    float lane[32];
    for (int l = 0; l < 32; l++) {
        float acc = 0.0f;
        for (size_t b = (size_t)l; b < blocks; b += 32) {
            int32_t dot = 0;
            for (int i = 0; i < 32; i++) dot += (int32_t)quants[b * 32 + i] * (int32_t)xq[b * 32 + i];
            const float dw = dsx_ref_f16_to_f32((uint16_t)(wrow[b * 2] | (wrow[b * 2 + 1] << 8)));
            acc += dw * xscale[b] * (float)dot;
        }
        lane[l] = acc;
    }
    for (int off = 16; off > 0; off >>= 1) {
        float next[32];
        for (int l = 0; l < 32; l++) next[l] = lane[l] + ((l + off < 32) ? lane[l + off] : lane[l]);
        memcpy(lane, next, sizeof lane);
    }
    return lane[0];
}

/* ------------------------------------------------------------------------ */
/* Q8_K                                                                      */
/* ------------------------------------------------------------------------ */

/* K/tests/q8_k_quantize.rs:37-102 */
void dsx_ref_q8k_quantize(const float *x, uint8_t *out, size_t n_blocks) {
    for (size_t b = 0; b < n_blocks; b++) {
        const float *xb = x + b * 256;
        uint8_t *blk = out + b * 292;
        float amax = 0.0f, mxv = 0.0f;
        for (int j = 0; j < 256; j++) {
            const float a = fabsf(xb[j]);
            if (a > amax) {
                amax = a;
                mxv = xb[j];
            }
        }
        if (amax == 0.0f) {
            memset(blk, 0, 292);
            continue;
        }
        const float iscale = -127.0f / mxv;
        const float d = 1.0f / iscale;
        memcpy(blk, &d, 4);
        int8_t *qs = (int8_t *)(blk + 4);
        for (int j = 0; j < 256; j++) {
            int v = (int)rintf(iscale * xb[j]); /* round half to even */
            if (v > 127) v = 127;
            if (v < -128) v = -128;
            qs[j] = (int8_t)v;
        }
        for (int j = 0; j < 16; j++) {
            int s = 0;
            for (int i = 0; i < 16; i++) s += qs[j * 16 + i];
            const int16_t bs = (int16_t)s;
            memcpy(blk + 260 + j * 2, &bs, 2);
        }
    }
}

/* external/ds4-dump/quants_selftest.c:108-118 */
void dsx_ref_q8k_dequant(const uint8_t *blocks, float *y, size_t n_blocks) {
    for (size_t b = 0; b < n_blocks; b++) {
        float d;
        memcpy(&d, blocks + b * 292, 4);
        const int8_t *qs = (const int8_t *)(blocks + b * 292 + 4);
        for (int i = 0; i < 256; i++) y[b * 256 + i] = d * (float)qs[i];
    }
}

/* K/src/mxfp4_tables.rs:49-74 */
float dsx_ref_dot_mxfp4_q8k(size_t n_super, const uint8_t *w_bytes, const uint8_t *y_bytes) {
    float sumf = 0.0f;
    for (size_t s = 0; s < n_super; s++) {
        const uint8_t *w = w_bytes + s * 136;
        const uint8_t *y = y_bytes + s * 292;
        float yd;
        memcpy(&yd, y, 4);
        const int8_t *q8 = (const int8_t *)(y + 4);
        float acc = 0.0f;
        for (int b = 0; b < 8; b++) {
            const float scale = dsx_ref_e8m0_half_to_f32(w[128 + b]);
            const uint8_t *qs = w + b * 16;
            int32_t sumi = 0;
            for (int j = 0; j < 16; j++) {
                sumi += (int32_t)KVALUES[qs[j] & 0x0f] * (int32_t)q8[b * 32 + j];
                sumi += (int32_t)KVALUES[qs[j] >> 4] * (int32_t)q8[b * 32 + 16 + j];
            }
            acc += scale * (float)sumi;
        }
        sumf += yd * acc;
    }
    return sumf;
}

/* ------------------------------------------------------------------------ */
/* element-wise                                                              */
/* ------------------------------------------------------------------------ */

/* K/kernels/swiglu_clamp_weighted.hip:27-36 */
float dsx_ref_swiglu(float g, float u, float clamp, float ew) {
    if (clamp > 1.0e-6f) {
        if (g > clamp) g = clamp;
        if (u > clamp) u = clamp;
        if (u < -clamp) u = -clamp;
    }
    const float sig = 1.0f / (1.0f + expf(-g));
    return g * sig * u * ew;
}

/* K/kernels/rms_norm.hip:12-50 */
void dsx_ref_rms_norm(float *out, const float *x, const float *weight, size_t n, float eps,
                      size_t rows) {
    for (size_t r = 0; r < rows; r++) {
        const float *xr = x + r * n;
        float sdata[256];
        for (size_t t = 0; t < 256; t++) {
            double partial = 0.0;
            for (size_t i = t; i < n; i += 256) partial += (double)xr[i] * (double)xr[i];
            sdata[t] = (float)partial;
        }
        for (size_t stride = 128; stride > 0; stride >>= 1)
            for (size_t t = 0; t < stride; t++) sdata[t] += sdata[t + stride];
        const float mean_sq = sdata[0] / (float)n;
        const float scale = 1.0f / sqrtf(mean_sq + eps);
        for (size_t i = 0; i < n; i++) out[r * n + i] = xr[i] * scale * weight[i];
    }
}

/* K/kernels/hc_post.hip:15-34 (one token), :40-64 (batched), :66-98 (post / comb from the packed
 * split row), :100-141 (block = (block_out + add1) + add2).  f32 throughout, the products rounded
 * before they are added, src ascending. */
void dsx_ref_hc_post(float *out_hc, const float *block_out, const float *add1, const float *add2,
                     const float *residual_hc, const float *post, const float *comb, size_t n_embd,
                     size_t n_hc, size_t b, size_t post_stride, size_t comb_stride) {
    for (size_t t = 0; t < b; t++) {
        const float *pb = post + t * post_stride, *cb = comb + t * comb_stride;
        const float *rh = residual_hc + t * n_hc * n_embd;
        for (size_t dst = 0; dst < n_hc; dst++)
            for (size_t d = 0; d < n_embd; d++) {
                float bv = block_out[t * n_embd + d];
                if (add1) bv = bv + add1[t * n_embd + d];
                if (add2) bv = bv + add2[t * n_embd + d];
                float acc = bv * pb[dst];
                for (size_t src = 0; src < n_hc; src++) {
                    const float prod = cb[dst + src * n_hc] * rh[src * n_embd + d];
                    acc = acc + prod;
                }
                out_hc[(t * n_hc + dst) * n_embd + d] = acc;
            }
    }
}

/* ------------------------------------------------------------------------ */
/* router                                                                    */
/* ------------------------------------------------------------------------ */

/* K/kernels/router_topk.hip:32-36 */
static float softplus_stable(float x) {
    if (x > 20.0f) return x;
    if (x < -20.0f) return expf(x);
    return log1pf(expf(x));
}

static void router_probs(float *p, const float *l, int n, int mode) {
    if (mode == DSX_REF_ROUTER_SQRT_SOFTPLUS) {
        for (int i = 0; i < n; i++) p[i] = sqrtf(softplus_stable(l[i]));
    } else if (mode == DSX_REF_ROUTER_SIGMOID) {
        for (int i = 0; i < n; i++) p[i] = 1.0f / (1.0f + expf(-l[i]));
    } else {
        float m = l[0];
        for (int i = 1; i < n; i++)
            if (l[i] > m) m = l[i];
        float sum = 0.0f;
        for (int i = 0; i < n; i++) {
            p[i] = expf(l[i] - m);
            sum += p[i];
        }
        for (int i = 0; i < n; i++) p[i] = p[i] / sum;
    }
}

/* DeepSeek-V3 group limiting on the biased scores. */
static void group_mask(float *score, int n_expert, int n_group, int topk_group) {
    if (n_group <= 1 || topk_group >= n_group) return;
    const int gs = n_expert / n_group;
    float gscore[512];
    int keep[512];
    for (int g = 0; g < n_group; g++) {
        float a = -INFINITY, b = -INFINITY; /* two largest */
        for (int i = 0; i < gs; i++) {
            const float v = score[g * gs + i];
            if (v > a) {
                b = a;
                a = v;
            } else if (v > b) {
                b = v;
            }
        }
        gscore[g] = (gs >= 2) ? a + b : a;
        keep[g] = 0;
    }
    for (int k = 0; k < topk_group; k++) {
        int best = -1;
        for (int g = 0; g < n_group; g++)
            if (!keep[g] && (best < 0 || gscore[g] > gscore[best])) best = g;
        keep[best] = 1;
    }
    for (int g = 0; g < n_group; g++)
        if (!keep[g])
            for (int i = 0; i < gs; i++) score[g * gs + i] = -INFINITY;
}

int dsx_ref_router_scores(float *probs, float *scores, const float *logits, const float *bias,
                          int n_expert, int n_tokens, int mode, int n_group, int topk_group) {
    if (n_expert <= 0 || n_expert > 512 || mode < 0 || mode > 2) return -1;
    if (n_group > 1 && (n_expert % n_group != 0 || topk_group < 1)) return -1;
    for (int t = 0; t < n_tokens; t++) {
        float *p = probs + (size_t)t * n_expert;
        float *s = scores + (size_t)t * n_expert;
        router_probs(p, logits + (size_t)t * n_expert, n_expert, mode);
        for (int i = 0; i < n_expert; i++) s[i] = bias ? p[i] + bias[i] : p[i];
        group_mask(s, n_expert, n_group, topk_group);
    }
    return 0;
}

int dsx_ref_router_topk(int32_t *selected, float *weights, const float *logits,
                        const float *bias, int n_expert, int n_used, float scale, float eps,
                        int n_tokens, int mode, int n_group, int topk_group) {
    if (n_used <= 0 || n_used > n_expert || n_used > 64) return -1;
    float p[512], s[512];
    for (int t = 0; t < n_tokens; t++) {
        if (dsx_ref_router_scores(p, s, logits + (size_t)t * n_expert, bias, n_expert, 1, mode,
                                  n_group, topk_group) != 0)
            return -1;
        int32_t *sel = selected + (size_t)t * n_used;
        float *w = weights + (size_t)t * n_used;
        /* K/kernels/laguna_ops.hip:70-93: k argmax passes, strict > so the lowest
         * index wins ties, winner masked to -inf. */
        for (int k = 0; k < n_used; k++) {
            int best = -1;
            float bv = -INFINITY;
            for (int i = 0; i < n_expert; i++)
                if (s[i] > bv) {
                    bv = s[i];
                    best = i;
                }
            sel[k] = best;
            if (best >= 0) s[best] = -INFINITY;
        }
        /* K/kernels/laguna_ops.hip:96-112 */
        float sum = 0.0f;
        for (int k = 0; k < n_used; k++) {
            w[k] = (sel[k] >= 0) ? p[sel[k]] : 0.0f;
            sum += w[k];
        }
        if (sum < eps) sum = eps;
        for (int k = 0; k < n_used; k++) w[k] = w[k] / sum * scale;
    }
    return 0;
}

/* K/src/routing.rs:21-44 (hash_router_select): the picks of token id `tok` are row `tok` of
 * tid2eid[vocab, n_used]; weights sqrt(softplus(logit)) / max(sum, eps) * scale, the sum
 * taken in slot order (the reference: n_used 6, eps 6.103515625e-5, scale 1.5).  A token id
 * or an expert id out of range gives an empty slot (-1, weight 0) where the reference would
 * index out of bounds. */
void dsx_ref_router_hash_select(int32_t *selected, float *weights, const float *logits,
                                const int32_t *tid2eid, const int32_t *token_ids, int n_expert,
                                int n_used, int vocab, float scale, float eps, int n_tokens) {
    for (int t = 0; t < n_tokens; t++) {
        const int tok = token_ids[t];
        const float *lg = logits + (size_t)t * n_expert;
        int32_t *sel = selected + (size_t)t * n_used;
        float *w = weights + (size_t)t * n_used;
        float sum = 0.0f;
        for (int i = 0; i < n_used; i++) {
            int e = (tok >= 0 && tok < vocab) ? tid2eid[(size_t)tok * n_used + i] : -1;
            if (e < 0 || e >= n_expert) e = -1;
            sel[i] = e;
            w[i] = (e >= 0) ? sqrtf(softplus_stable(lg[e])) : 0.0f;
            sum += w[i];
        }
        if (sum < eps) sum = eps;
        for (int i = 0; i < n_used; i++) w[i] = w[i] / sum * scale;
    }
}

/* The het-split ownership rule shared by the reference's *_hetsplit kernels
 * (K/kernels/mxfp4_pair_matvec.hip:231-284, K/kernels/q2_k_accumulate_matvec_par.hip:731-766):
 * remap[e] >= 0 is the dense slot of a resident ("hot") expert on the dGPU side, -(slot + 1)
 * the packed slot of a cold one.  The dGPU side (mode 1) takes the first `cap` resident picks
 * of a token in slot order, the other side (mode 0) everything else.  out[b, s] = the expert
 * index this side's weight buffer is addressed with, or -1 where the slot is not this side's
 * (or is empty). */
void dsx_ref_hetsplit_select(int32_t *out, const int32_t *selected, const int32_t *remap, int mode,
                             int cap, int n_used, int n_expert, int n_tokens) {
    for (int b = 0; b < n_tokens; b++) {
        int rank = 0;
        for (int s = 0; s < n_used; s++) {
            const int e = selected[(size_t)b * n_used + s];
            int r = -1;
            if (e >= 0 && e < n_expert) {
                const int dense = remap[e];
                const int resident = dense >= 0;
                const int dgpu_takes = resident && rank < cap;
                if (resident) rank++;
                if (mode == 1) {
                    if (dgpu_takes) r = dense;
                } else if (!dgpu_takes) {
                    r = resident ? e : -dense - 1;
                }
            }
            out[(size_t)b * n_used + s] = r;
        }
    }
}

/* K/kernels/laguna_ops.hip:57-60 */
void dsx_ref_router_logits(float *logits, const float *w, const float *x, int n_expert,
                           int hidden, int n_tokens) {
#pragma omp parallel for collapse(2) schedule(static)
    for (int t = 0; t < n_tokens; t++)
        for (int e = 0; e < n_expert; e++) {
            const float *wr = w + (size_t)e * hidden;
            const float *xr = x + (size_t)t * hidden;
            float acc = 0.0f;
            for (int k = 0; k < hidden; k++) acc += wr[k] * xr[k];
            logits[(size_t)t * n_expert + e] = acc;
        }
}

/* ------------------------------------------------------------------------ */
/* token -> expert inversion                                                 */
/* ------------------------------------------------------------------------ */

int dsx_ref_group_build(int32_t *group_count, int32_t *offsets, int32_t *members,
                        int32_t *work_items, const int32_t *selected, int n_tokens, int n_used,
                        int n_expert, int chunk) {
    memset(group_count, 0, sizeof(int32_t) * (size_t)n_expert);
    const int total = n_tokens * n_used;
    for (int i = 0; i < total; i++) {
        const int e = selected[i];
        if (e >= 0 && e < n_expert) group_count[e]++;
    }
    offsets[0] = 0;
    for (int e = 0; e < n_expert; e++) offsets[e + 1] = offsets[e] + group_count[e];
    int32_t *fill = (int32_t *)calloc((size_t)n_expert, sizeof(int32_t));
    for (int i = 0; i < total; i++) {
        const int e = selected[i];
        if (e < 0 || e >= n_expert) continue;
        const int b = i / n_used, slot = i % n_used;
        members[offsets[e] + fill[e]++] = (int32_t)(((uint32_t)b << 16) | (uint32_t)slot);
    }
    free(fill);
    int n = 0;
    for (int e = 0; e < n_expert; e++)
        for (int start = 0; start < group_count[e]; start += chunk)
            work_items[n++] = (int32_t)(((uint32_t)e << 16) | (uint32_t)start);
    return n;
}

/* K/src/het/dispatch.rs:450-454 */
uint32_t dsx_ref_wi_upper_bound(size_t members, uint32_t groups, uint32_t chunk, size_t cap) {
    const size_t m = members;
    const size_t g = m < groups ? m : groups;
    const size_t c = chunk ? chunk : 1;
    size_t v = g + (m + c - 1) / c;
    if (v > m) v = m;
    if (v > cap) v = cap;
    return (uint32_t)v;
}

/* ------------------------------------------------------------------------ */
/* the layer                                                                 */
/* ------------------------------------------------------------------------ */

int dsx_ref_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* Activation of `n` values quantized for a matrix of format `fmt`. */
typedef struct {
    uint8_t *q8k;  /* MXFP4 consumer */
    int8_t *xq;    /* Q8_0 consumer */
    float *xscale;
} act_q;

static size_t row_bytes(int fmt, int cols) {
    return fmt == DSX_REF_FMT_MXFP4 ? (size_t)(cols / 256) * 136 : (size_t)(cols / 32) * 34;
}

static void act_quantize(act_q *a, int fmt, const float *x, int n) {
    if (fmt == DSX_REF_FMT_MXFP4)
        dsx_ref_q8k_quantize(x, a->q8k, (size_t)n / 256);
    else
        dsx_ref_q8_0_quantize_act(x, a->xq, a->xscale, (size_t)n / 32);
}

static float row_dot(int fmt, const uint8_t *wrow, const act_q *a, int cols) {
    if (fmt == DSX_REF_FMT_MXFP4) return dsx_ref_dot_mxfp4_q8k((size_t)cols / 256, wrow, a->q8k);
    return dsx_ref_dot_q8_0((size_t)cols / 32, wrow, a->xq, a->xscale);
}

static int fmt_ok(int fmt, int cols) {
    if (fmt == DSX_REF_FMT_MXFP4) return cols % 256 == 0;
    if (fmt == DSX_REF_FMT_Q8_0) return cols % 32 == 0;
    return 0;
}

static void act_alloc(act_q *a, int n) {
    a->q8k = (uint8_t *)malloc((size_t)(n / 256 + 1) * 292);
    a->xq = (int8_t *)malloc((size_t)n);
    a->xscale = (float *)malloc(sizeof(float) * (size_t)(n / 32 + 1));
}
static void act_free(act_q *a) {
    free(a->q8k);
    free(a->xq);
    free(a->xscale);
}

/* One SwiGLU expert applied to one token: acc_out[hidden] = down . Q(mid), with
 * mid = swiglu(gate . xg, up . xu) * ew.  xg / xu are the token's activations
 * quantized for the gate / up formats.  mid_buf has `inter` floats. */
static void expert_apply(float *dst, float *mid_buf, act_q *mq, const uint8_t *gate,
                         const uint8_t *up, const uint8_t *down, int gate_fmt, int up_fmt,
                         int down_fmt, const act_q *xg, const act_q *xu, int hidden, int inter,
                         float clamp, float ew) {
    const size_t grb = row_bytes(gate_fmt, hidden), urb = row_bytes(up_fmt, hidden);
    const size_t drb = row_bytes(down_fmt, inter);
#pragma omp parallel for schedule(static)
    for (int r = 0; r < inter; r++) {
        const float g = row_dot(gate_fmt, gate + (size_t)r * grb, xg, hidden);
        const float u = row_dot(up_fmt, up + (size_t)r * urb, xu, hidden);
        mid_buf[r] = dsx_ref_swiglu(g, u, clamp, ew);
    }
    act_quantize(mq, down_fmt, mid_buf, inter);
#pragma omp parallel for schedule(static)
    for (int r = 0; r < hidden; r++) dst[r] = row_dot(down_fmt, down + (size_t)r * drb, mq, inter);
}

int dsx_ref_moe_forward(const dsx_ref_moe_cfg *c, const float *x, const int32_t *selected,
                        const float *weights, int n_tokens, float *out, float *mid_out,
                        float *moe_out, float *shared_out, int n_threads) {
    if (!fmt_ok(c->gate_fmt, c->hidden) || !fmt_ok(c->up_fmt, c->hidden) ||
        !fmt_ok(c->down_fmt, c->inter))
        return -1;
    if (c->sh_inter > 0 && (!fmt_ok(c->sh_gate_fmt, c->hidden) || !fmt_ok(c->sh_up_fmt, c->hidden) ||
                            !fmt_ok(c->sh_down_fmt, c->sh_inter)))
        return -1;
#ifdef _OPENMP
    const int saved = omp_get_max_threads();
    if (n_threads > 0) omp_set_num_threads(n_threads);
#else
    (void)n_threads;
#endif
    const int hidden = c->hidden, inter = c->inter, k = c->n_used;
    const int max_inter = inter > c->sh_inter ? inter : c->sh_inter;
    act_q xa, mq;
    act_alloc(&xa, hidden);
    act_alloc(&mq, max_inter);
    float *mid = (float *)malloc(sizeof(float) * (size_t)max_inter);
    float *part = (float *)malloc(sizeof(float) * (size_t)hidden);
    float *acc = (float *)malloc(sizeof(float) * (size_t)hidden);
    int rc = 0;
    for (int t = 0; t < n_tokens && rc == 0; t++) {
        const float *xt = x + (size_t)t * hidden;
        /* both quantizations of the token (only the ones a format needs are read) */
        act_quantize(&xa, DSX_REF_FMT_MXFP4, xt, hidden);
        act_quantize(&xa, DSX_REF_FMT_Q8_0, xt, hidden);
        for (int r = 0; r < hidden; r++) acc[r] = 0.0f;
        /* slot-order sum: K/kernels/q2_k_accumulate_matvec_par.hip:724-729 */
        for (int s = 0; s < k; s++) {
            const int e = selected[(size_t)t * k + s];
            float *mdst = mid_out ? mid_out + ((size_t)t * k + s) * inter : NULL;
            if (e < 0) {
                if (mdst) memset(mdst, 0, sizeof(float) * (size_t)inter);
                continue;
            }
            if (e >= c->n_expert) {
                rc = -2;
                break;
            }
            expert_apply(part, mid, &mq, c->gate + (uint64_t)e * c->gate_bpe,
                         c->up + (uint64_t)e * c->up_bpe, c->down + (uint64_t)e * c->down_bpe,
                         c->gate_fmt, c->up_fmt, c->down_fmt, &xa, &xa, hidden, inter, c->clamp,
                         weights[(size_t)t * k + s]);
            if (mdst) memcpy(mdst, mid, sizeof(float) * (size_t)inter);
            for (int r = 0; r < hidden; r++) acc[r] += part[r];
        }
        if (moe_out) memcpy(moe_out + (size_t)t * hidden, acc, sizeof(float) * (size_t)hidden);
        if (c->sh_inter > 0) {
            expert_apply(part, mid, &mq, c->sh_gate, c->sh_up, c->sh_down, c->sh_gate_fmt,
                         c->sh_up_fmt, c->sh_down_fmt, &xa, &xa, hidden, c->sh_inter, c->sh_clamp,
                         1.0f);
            if (shared_out)
                memcpy(shared_out + (size_t)t * hidden, part, sizeof(float) * (size_t)hidden);
            /* K/kernels/vec_add.hip:6-13: ffn_moe += ffn_shared */
            for (int r = 0; r < hidden; r++) acc[r] += part[r];
        }
        memcpy(out + (size_t)t * hidden, acc, sizeof(float) * (size_t)hidden);
    }
    act_free(&xa);
    act_free(&mq);
    free(mid);
    free(part);
    free(acc);
#ifdef _OPENMP
    omp_set_num_threads(saved);
#endif
    return rc;
}
