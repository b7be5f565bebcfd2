/*
 * oracle_ops.c — CPU restatement of the arithmetic of ggml's CPU backend for the ops whisper.cpp emits.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the product (the HIP kernels, the ggml backend plugin) includes,
 * links or calls this file; tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg use it as the
 * checker.  Plain scalar C, dense row-major operands (ne0 contiguous, like ggml), no SIMD, no threads.
 *
 * Each function cites the reference code it follows (paths relative to the whisper.cpp tree).  Where the
 * reference's x86 build takes an AVX2 path whose rounding differs from the scalar C path (quantize_row_q8_0
 * rounds half to even; the scalar code uses roundf), the AVX2 behaviour is restated, because that is the build
 * the GPU results are compared with.  Floating-point sums are accumulated in the same precision as the
 * reference but not in its SIMD lane order, so results agree with the reference to rounding, not bitwise —
 * except the (de)quantizers, which are bit-exact.
 *
 * Pinning: every function here is checked in tests/test_oracle.py against the reference's own compiled code
 * (oracle/_ref: libggml-base.so for the quantizers, the ggml CPU backend for the graph ops) and against
 * closed forms that do not share its structure (numpy float64 GEMM / softmax / layer-norm, brute force over
 * all 65536 f16 bit patterns for the conversions, all nibble/high-bit patterns for dequantization).
 * No function here is left without such a check.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define QK 32

/* ---------------------------------------------------------------------------------------------------------
 * f16 <-> f32: GGML_FP16_TO_FP32 / GGML_FP32_TO_FP16 (ggml/src/ggml-impl.h:311-440) are IEEE conversions
 * with round-to-nearest-even (F16C on x86).
 * ------------------------------------------------------------------------------------------------------- */

float oracle_f16_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1F, m = h & 0x3FF;
    uint32_t x;
    if (e == 0) {
        if (m == 0) x = sign;
        else {
            int s = 0; uint32_t mm = m;
            while (!(mm & 0x400)) { mm <<= 1; ++s; }
            x = sign | ((uint32_t)(113 - s) << 23) | ((mm & 0x3FF) << 13);
        }
    } else if (e == 31) x = sign | 0x7F800000u | (m << 13);
    else                x = sign | ((e + 112) << 23) | (m << 13);
    float f; memcpy(&f, &x, 4);
    return f;
}

uint16_t oracle_f32_to_f16(float f) {
    uint32_t x; memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t absx = x & 0x7FFFFFFFu;
    if (absx >= 0x7F800000u) return (uint16_t)(sign | (absx > 0x7F800000u ? 0x7E00u : 0x7C00u));
    if (absx >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);      /* >= 65520 rounds to inf */
    if (absx <  0x33000001u) return (uint16_t) sign;                  /* <= 2^-25 rounds to zero */
    const int32_t e = (int32_t)(absx >> 23) - 127;
    uint32_t m = (absx & 0x7FFFFFu) | 0x800000u;
    int shift; uint32_t base;
    if (e >= -14) { shift = 13; base = (uint32_t)(e + 15) << 10; m &= 0x7FFFFFu; }
    else          { shift = 13 + (-14 - e); base = 0; }
    uint32_t h = m >> shift;
    const uint32_t rem = m & ((1u << shift) - 1), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (h & 1))) ++h;
    return (uint16_t)(sign | (base + h));
}

static inline float rnd16(float f) { return oracle_f16_to_f32(oracle_f32_to_f16(f)); }

void oracle_f32_to_f16_row(const float * x, uint16_t * y, int64_t n) { for (int64_t i = 0; i < n; ++i) y[i] = oracle_f32_to_f16(x[i]); }
void oracle_f16_to_f32_row(const uint16_t * x, float * y, int64_t n) { for (int64_t i = 0; i < n; ++i) y[i] = oracle_f16_to_f32(x[i]); }

/* ---------------------------------------------------------------------------------------------------------
 * block formats: block_q5_0 {f16 d; u8 qh[4]; u8 qs[16]} = 22 B, block_q8_0 {f16 d; i8 qs[32]} = 34 B
 * (ggml/src/ggml-common.h:187-193, 209-214)
 * ------------------------------------------------------------------------------------------------------- */

/* dequantize_row_q5_0 (ggml/src/ggml-quants.c:296-319) */
void oracle_dequantize_row_q5_0(const uint8_t * x, float * y, int64_t k) {
    for (int64_t i = 0; i < k / QK; ++i, x += 22, y += QK) {
        uint16_t dh; memcpy(&dh, x, 2);
        const float d = oracle_f16_to_f32(dh);
        uint32_t qh; memcpy(&qh, x + 2, 4);
        for (int j = 0; j < QK / 2; ++j) {
            const uint8_t xh_0 = ((qh >> (j +  0)) << 4) & 0x10;
            const uint8_t xh_1 = ((qh >> (j + 12))     ) & 0x10;
            const int32_t x0 = ((x[6 + j] & 0x0F) | xh_0) - 16;
            const int32_t x1 = ((x[6 + j] >>   4) | xh_1) - 16;
            y[j]          = x0 * d;
            y[j + QK / 2] = x1 * d;
        }
    }
}

/* dequantize_row_q8_0 (ggml/src/ggml-quants.c:349-363) */
void oracle_dequantize_row_q8_0(const uint8_t * x, float * y, int64_t k) {
    for (int64_t i = 0; i < k / QK; ++i, x += 34, y += QK) {
        uint16_t dh; memcpy(&dh, x, 2);
        const float d = oracle_f16_to_f32(dh);
        for (int j = 0; j < QK; ++j) y[j] = ((const int8_t *) x)[2 + j] * d;
    }
}

/* quantize_row_q5_0_ref (ggml/src/ggml-quants.c:105-143) */
void oracle_quantize_row_q5_0_ref(const float * x, uint8_t * y, int64_t k) {
    for (int64_t i = 0; i < k / QK; ++i, x += QK, y += 22) {
        float amax = 0.0f, max = 0.0f;
        for (int j = 0; j < QK; ++j) { const float v = x[j]; if (amax < fabsf(v)) { amax = fabsf(v); max = v; } }
        const float d  = max / -16;
        const float id = d ? 1.0f / d : 0.0f;
        const uint16_t dh = oracle_f32_to_f16(d);
        memcpy(y, &dh, 2);
        uint32_t qh = 0;
        for (int j = 0; j < QK / 2; ++j) {
            const float x0 = x[j] * id, x1 = x[QK / 2 + j] * id;
            int q0 = (int8_t)(x0 + 16.5f); if (q0 > 31) q0 = 31;
            int q1 = (int8_t)(x1 + 16.5f); if (q1 > 31) q1 = 31;
            const uint8_t xi0 = (uint8_t) q0, xi1 = (uint8_t) q1;
            y[6 + j] = (xi0 & 0x0F) | ((xi1 & 0x0F) << 4);
            qh |= ((xi0 & 0x10u) >> 4) << (j + 0);
            qh |= ((xi1 & 0x10u) >> 4) << (j + QK / 2);
        }
        memcpy(y + 2, &qh, 4);
    }
}

/* quantize_row_q8_0_ref (ggml/src/ggml-quants.c:194-215): model-file quantizer, rounds half away from zero */
void oracle_quantize_row_q8_0_ref(const float * x, uint8_t * y, int64_t k) {
    for (int64_t i = 0; i < k / QK; ++i, x += QK, y += 34) {
        float amax = 0.0f;
        for (int j = 0; j < QK; ++j) { const float v = fabsf(x[j]); if (v > amax) amax = v; }
        const float d  = amax / ((1 << 7) - 1);
        const float id = d ? 1.0f / d : 0.0f;
        const uint16_t dh = oracle_f32_to_f16(d);
        memcpy(y, &dh, 2);
        for (int j = 0; j < QK; ++j) ((int8_t *) y)[2 + j] = (int8_t) roundf(x[j] * id);
    }
}

/* quantize_row_q8_0, AVX2 path (ggml/src/ggml-cpu/ggml-cpu-quants.c:808-865): the activation quantizer used
 * inside MUL_MAT.  id = 127/amax (not 1/d), _mm256_round_ps(_MM_ROUND_NEAREST) = round half to even. */
void oracle_quantize_row_q8_0_act(const float * x, uint8_t * y, int64_t k) {
    for (int64_t i = 0; i < k / QK; ++i, x += QK, y += 34) {
        float amax = 0.0f;
        for (int j = 0; j < QK; ++j) { const float v = fabsf(x[j]); if (v > amax) amax = v; }
        const float d  = amax / 127.f;
        const float id = (amax != 0.0f) ? 127.f / amax : 0.0f;
        const uint16_t dh = oracle_f32_to_f16(d);
        memcpy(y, &dh, 2);
        for (int j = 0; j < QK; ++j) ((int8_t *) y)[2 + j] = (int8_t) nearbyintf(x[j] * id);   /* default rounding mode: half to even */
    }
}

/* ---------------------------------------------------------------------------------------------------------
 * MUL_MAT (ggml_compute_forward_mul_mat, ggml/src/ggml-cpu/ggml-cpu.c:1266-1458)
 *   dst[n*M + m] = sum_k w[m][k] * x[n][k]
 * wtype: 0 f32, 1 f16, 6 q5_0, 8 q8_0 (enum ggml_type).  x is f32 [N][K].
 * ------------------------------------------------------------------------------------------------------- */

/* ggml_vec_dot_q8_0_q8_0 / ggml_vec_dot_q5_0_q8_0 (ggml/src/ggml-cpu/ggml-cpu-quants.c:3597, 2930): per block the
 * integer dot product of the quants, times d_w * d_x, accumulated in f32 */
static float vec_dot_q_q8_0(int wtype, const uint8_t * w, const uint8_t * xq, int64_t k) {
    float sum = 0.0f;
    for (int64_t b = 0; b < k / QK; ++b) {
        const uint8_t * xb = xq + b * 34;
        uint16_t dxh; memcpy(&dxh, xb, 2);
        const int8_t * qx = (const int8_t *) xb + 2;
        int32_t sumi = 0; uint16_t dwh;
        if (wtype == 8) {
            const uint8_t * wb = w + b * 34;
            memcpy(&dwh, wb, 2);
            const int8_t * qw = (const int8_t *) wb + 2;
            for (int j = 0; j < QK; ++j) sumi += (int32_t) qw[j] * qx[j];
        } else {
            const uint8_t * wb = w + b * 22;
            memcpy(&dwh, wb, 2);
            uint32_t qh; memcpy(&qh, wb + 2, 4);
            for (int j = 0; j < QK / 2; ++j) {
                const uint8_t xh_0 = ((qh >> (j +  0)) << 4) & 0x10;
                const uint8_t xh_1 = ((qh >> (j + 12))     ) & 0x10;
                const int32_t x0 = (int8_t)(((wb[6 + j] & 0x0F) | xh_0) - 16);
                const int32_t x1 = (int8_t)(((wb[6 + j] >>   4) | xh_1) - 16);
                sumi += x0 * qx[j] + x1 * qx[j + QK / 2];
            }
        }
        sum += (oracle_f16_to_f32(dwh) * oracle_f16_to_f32(dxh)) * (float) sumi;
    }
    return sum;
}

void oracle_mul_mat(int wtype, const void * w, const float * x, float * dst, int64_t M, int64_t N, int64_t K) {
    if (wtype == 6 || wtype == 8) {
        /* src1 is first converted to the weights' vec_dot_type, Q8_0 (ggml-cpu.c:1328-1363, type traits :211-376) */
        const int64_t row_w = (K / QK) * (wtype == 8 ? 34 : 22), row_x = (K / QK) * 34;
        uint8_t * xq = (uint8_t *) malloc((size_t)(N * row_x));
        for (int64_t n = 0; n < N; ++n) oracle_quantize_row_q8_0_act(x + n * K, xq + n * row_x, K);
        for (int64_t n = 0; n < N; ++n)
            for (int64_t m = 0; m < M; ++m)
                dst[n * M + m] = vec_dot_q_q8_0(wtype, (const uint8_t *) w + m * row_w, xq + n * row_x, K);
        free(xq);
    } else if (wtype == 1) {
        /* f16 weights: src1 is rounded to f16, products accumulate in f32 (ggml_vec_dot_f16, ggml/src/ggml-cpu/vec.cpp) */
        const uint16_t * wh = (const uint16_t *) w;
        float * xr = (float *) malloc((size_t)(N * K) * sizeof(float));
        for (int64_t i = 0; i < N * K; ++i) xr[i] = rnd16(x[i]);
        for (int64_t n = 0; n < N; ++n)
            for (int64_t m = 0; m < M; ++m) {
                float s = 0.0f;
                for (int64_t k = 0; k < K; ++k) s += oracle_f16_to_f32(wh[m * K + k]) * xr[n * K + k];
                dst[n * M + m] = s;
            }
        free(xr);
    } else {
        const float * wf = (const float *) w;
        for (int64_t n = 0; n < N; ++n)
            for (int64_t m = 0; m < M; ++m) {
                float s = 0.0f;
                for (int64_t k = 0; k < K; ++k) s += wf[m * K + k] * x[n * K + k];
                dst[n * M + m] = s;
            }
    }
}

/* f16 x f16 variant used by the conv stem (src0 = im2col patches f16 [M][K], src1 = conv weights f16 [N][K]) */
void oracle_mul_mat_f16_f16(const uint16_t * a, const uint16_t * b, float * dst, int64_t M, int64_t N, int64_t K) {
    for (int64_t n = 0; n < N; ++n)
        for (int64_t m = 0; m < M; ++m) {
            float s = 0.0f;
            for (int64_t k = 0; k < K; ++k) s += oracle_f16_to_f32(a[m * K + k]) * oracle_f16_to_f32(b[n * K + k]);
            dst[n * M + m] = s;
        }
}

/* ---------------------------------------------------------------------------------------------------------
 * FLASH_ATTN_EXT (ggml_compute_forward_flash_attn_ext_f16, ggml/src/ggml-cpu/ops.cpp:6638-6851), f16 K and V,
 * max_bias = 0, logit_softcap = 0.
 *   q f32 [H][N][D], k/v f16 [H][KV][D], mask f16 [N][KV] or NULL, dst f32 [N][H][D]
 * Per (query, head) the keys are visited in order; the running V accumulator VKQ16 is held in f16 and rounded
 * after every key (ops.cpp:6793-6807; the F16C build's ggml_vec_mad_f16 / ggml_vec_scale_f16 compute in f32 and
 * store f16), the softmax sum S and maximum M are f32.
 * ------------------------------------------------------------------------------------------------------- */
void oracle_flash_attn_ext(const float * q, const uint16_t * k, const uint16_t * v, const uint16_t * mask, float * dst,
                           int64_t N, int64_t KV, int64_t H, int64_t D, float scale) {
    uint16_t * vkq = (uint16_t *) malloc((size_t) D * sizeof(uint16_t));
    float * qh = (float *) malloc((size_t) D * sizeof(float));
    for (int64_t h = 0; h < H; ++h) for (int64_t n = 0; n < N; ++n) {
        for (int64_t e = 0; e < D; ++e) { vkq[e] = 0; qh[e] = rnd16(q[(h * N + n) * D + e]); }   /* q -> f16 (ops.cpp:6755) */
        float S = 0.0f, M = -INFINITY;
        for (int64_t ic = 0; ic < KV; ++ic) {
            const float mv = mask ? oracle_f16_to_f32(mask[n * KV + ic]) : 0.0f;
            if (mv == -INFINITY) continue;
            float s = 0.0f;
            for (int64_t e = 0; e < D; ++e) s += oracle_f16_to_f32(k[(h * KV + ic) * D + e]) * qh[e];
            s = s * scale;
            s += mv;
            const float Mold = M;
            float ms = 1.0f, vs = 1.0f;
            if (s > M) {
                M = s; ms = expf(Mold - M);
                for (int64_t e = 0; e < D; ++e) vkq[e] = oracle_f32_to_f16(oracle_f16_to_f32(vkq[e]) * ms);
            } else {
                vs = expf(s - M);
            }
            for (int64_t e = 0; e < D; ++e)    /* VKQ16 += v * vs: fma in f32, stored as f16 */
                vkq[e] = oracle_f32_to_f16(fmaf(oracle_f16_to_f32(v[(h * KV + ic) * D + e]), vs, oracle_f16_to_f32(vkq[e])));
            S = S * ms + vs;
        }
        const float S_inv = 1.0f / S;
        for (int64_t e = 0; e < D; ++e) dst[(n * H + h) * D + e] = oracle_f16_to_f32(vkq[e]) * S_inv;   /* permute(0,2,1,3), ops.cpp:6849 */
    }
    free(vkq); free(qh);
}

/* ---------------------------------------------------------------------------------------------------------
 * NORM (ggml_compute_forward_norm_f32, ggml/src/ggml-cpu/ops.cpp:3109-3158): sums in double
 * ------------------------------------------------------------------------------------------------------- */
void oracle_norm(const float * x, float * y, int64_t ne0, int64_t nrows, float eps) {
    for (int64_t r = 0; r < nrows; ++r, x += ne0, y += ne0) {
        double sum = 0.0;
        for (int64_t i = 0; i < ne0; ++i) sum += (double) x[i];
        const float mean = (float)(sum / ne0);
        double sum2 = 0.0;
        for (int64_t i = 0; i < ne0; ++i) { const float t = x[i] - mean; y[i] = t; sum2 += (double)(t * t); }
        const float variance = (float)(sum2 / ne0);
        const float scale = 1.0f / sqrtf(variance + eps);
        for (int64_t i = 0; i < ne0; ++i) y[i] *= scale;
    }
}

/* ---------------------------------------------------------------------------------------------------------
 * GELU (ggml_vec_gelu_f32 with GGML_GELU_FP16, ggml/src/ggml-cpu/vec.h:428-457; table built at
 * ggml/src/ggml-cpu/ggml-cpu.c:3415-3423): x -> f16 -> table[f16] where table = f16(gelu_f32(f32(f16)))
 * ------------------------------------------------------------------------------------------------------- */
/* The reference's x86 objects are built with FMA contraction: of this expression only 1 + (0.044715 x) x fuses.  Written
 * out like this (the file is compiled with -ffp-contract=off) all finite table entries match the reference bit for bit. */
static float gelu_f32(float x) {
    const float inner = fmaf(0.044715f * x, x, 1.0f);
    return 0.5f * x * (1.0f + tanhf(0.79788456080286535587989211986876f * x * inner));
}
void oracle_gelu(const float * x, float * y, int64_t n) {
    for (int64_t i = 0; i < n; ++i) {
        if (x[i] <= -10.0f) y[i] = 0.0f;
        else if (x[i] >= 10.0f) y[i] = x[i];
        else y[i] = rnd16(gelu_f32(rnd16(x[i])));
    }
}

/* ---------------------------------------------------------------------------------------------------------
 * ADD / MUL with src1 repeated (ggml/src/ggml-cpu/binary-ops.cpp:49-142): dst shape = a's shape [ne3][ne2][ne1][ne0],
 * b's shape divides it.  op 0 add, 1 mul.
 * ------------------------------------------------------------------------------------------------------- */
void oracle_binary(int op, const float * a, const int64_t * ane, const float * b, const int64_t * bne, float * dst) {
    for (int64_t i3 = 0; i3 < ane[3]; ++i3) for (int64_t i2 = 0; i2 < ane[2]; ++i2) for (int64_t i1 = 0; i1 < ane[1]; ++i1)
        for (int64_t i0 = 0; i0 < ane[0]; ++i0) {
            const int64_t ia = ((i3 * ane[2] + i2) * ane[1] + i1) * ane[0] + i0;
            const int64_t ib = (((i3 % bne[3]) * bne[2] + (i2 % bne[2])) * bne[1] + (i1 % bne[1])) * bne[0] + (i0 % bne[0]);
            dst[ia] = op == 0 ? a[ia] + b[ib] : a[ia] * b[ib];
        }
}

/* SCALE (ggml/src/ggml-cpu/ops.cpp:3840-3878) */
void oracle_scale(const float * x, float * y, int64_t n, float s) { for (int64_t i = 0; i < n; ++i) y[i] = x[i] * s; }

/* ---------------------------------------------------------------------------------------------------------
 * IM2COL 1-D, f16 out (ggml_compute_forward_im2col_f16, ggml/src/ggml-cpu/ops.cpp:5784-5855):
 * src f32 [IC][IW] -> dst f16 [OW][IC*KW]
 * ------------------------------------------------------------------------------------------------------- */
void oracle_im2col_1d(const float * src, uint16_t * dst, int64_t IW, int64_t IC, int64_t OW, int KW, int s0, int p0, int d0) {
    for (int64_t iow = 0; iow < OW; ++iow)
        for (int64_t iic = 0; iic < IC; ++iic)
            for (int ikw = 0; ikw < KW; ++ikw) {
                const int64_t iiw = iow * s0 + ikw * d0 - p0;
                dst[iow * (IC * KW) + iic * KW + ikw] = (iiw < 0 || iiw >= IW) ? 0 : oracle_f32_to_f16(src[iic * IW + iiw]);
            }
}

/* ---------------------------------------------------------------------------------------------------------
 * SOFT_MAX (ggml_compute_forward_soft_max_f32, ggml/src/ggml-cpu/ops.cpp:4641-4737), max_bias = 0:
 * x [nrows][ne0], mask f32 [>= rows_per_slice][ne0] shared by all slices of rows_per_slice rows, or NULL
 * ------------------------------------------------------------------------------------------------------- */
void oracle_soft_max(const float * x, const float * mask, float * y, int64_t ne0, int64_t nrows, int64_t rows_per_slice, float scale) {
    for (int64_t r = 0; r < nrows; ++r, x += ne0, y += ne0) {
        const float * mp = mask ? mask + (r % rows_per_slice) * ne0 : NULL;
        float mx = -INFINITY;
        for (int64_t i = 0; i < ne0; ++i) { y[i] = x[i] * scale + (mp ? mp[i] : 0.0f); if (y[i] > mx) mx = y[i]; }
        double sum = 0.0;
        for (int64_t i = 0; i < ne0; ++i) { const float e = (y[i] == -INFINITY) ? 0.0f : expf(y[i] - mx); y[i] = e; sum += (double) e; }
        const float inv = (float)(1.0 / sum);
        for (int64_t i = 0; i < ne0; ++i) y[i] *= inv;
    }
}

/* ---------------------------------------------------------------------------------------------------------
 * GET_ROWS (ggml/src/ggml-cpu/ops.cpp:4146-4188, 4313): dst[i][:] = dequant(table[ids[i]][:])
 * ------------------------------------------------------------------------------------------------------- */
void oracle_get_rows(int type, const void * table, const int32_t * ids, float * dst, int64_t ne0, int64_t nids) {
    for (int64_t i = 0; i < nids; ++i) {
        const int64_t r = ids[i];
        switch (type) {
            case 6: oracle_dequantize_row_q5_0((const uint8_t *) table + r * (ne0 / QK) * 22, dst + i * ne0, ne0); break;
            case 8: oracle_dequantize_row_q8_0((const uint8_t *) table + r * (ne0 / QK) * 34, dst + i * ne0, ne0); break;
            case 1: oracle_f16_to_f32_row((const uint16_t *) table + r * ne0, dst + i * ne0, ne0); break;
            default: memcpy(dst + i * ne0, (const float *) table + r * ne0, (size_t) ne0 * 4); break;
        }
    }
}

/* ---------------------------------------------------------------------------------------------------------
 * Log-mel front end (log_mel_spectrogram and its worker, src/whisper.cpp:3113-3270; tables :3008-3045; the
 * transform :3049-3111): samples f32 [n_samples] at 16 kHz -> mel f32 [n_mel][n_len], n_len = (n_samples +
 * 480000) / 160.  The signal is extended by 200 reflected samples in front and 30 s + 200 samples of zeros
 * behind; frame i is 400 samples from 160 i under a periodic Hann window; its 400-point transform is taken
 * by halving down to 25 points (25-point sums over a 400-entry f32 sine / cosine table, then four rounds of
 * butterflies), all in f32 in the order below; power of bins 0 .. 200; filter bank [n_mel][201] with the
 * products added in fours in f32 and the fours in f64; log10(max(., 1e-10)); finally everything below
 * (global maximum - 8) is raised to it and the result is (x + 4) / 4.
 * Pinned in tests/test_golden.py against vectors written by the reference's compiled function
 * (oracle/ref_mel_shim.cpp) and in tests/test_oracle.py against numpy's float64 rfft.
 * ------------------------------------------------------------------------------------------------------- */
#define MEL_NFFT 400
#define MEL_HOP  160

static float mel_sin[MEL_NFFT], mel_cos[MEL_NFFT], mel_hann[MEL_NFFT];
static int   mel_tables_ready = 0;

static void mel_tables(void) {
    if (mel_tables_ready) return;
    for (int i = 0; i < MEL_NFFT; ++i) {
        const double theta = (2 * M_PI * i) / MEL_NFFT;
        mel_sin[i] = sinf((float) theta);
        mel_cos[i] = cosf((float) theta);
        mel_hann[i] = (float)(0.5 * (1.0 - (double) cosf((float)((2.0 * M_PI * i) / MEL_NFFT))));
    }
    mel_tables_ready = 1;
}

/* transform of x[0], x[stride], ..., n points, into re[0 .. n), im[0 .. n); `tmp` holds 4 n floats */
static void mel_transform(const float * x, int stride, int n, float * re, float * im, float * tmp) {
    const int step = MEL_NFFT / n;
    if (n == 1) { re[0] = x[0]; im[0] = 0.0f; return; }
    if (n % 2 == 1) {
        for (int k = 0; k < n; ++k) {
            float sr = 0.0f, si = 0.0f;
            for (int j = 0; j < n; ++j) {
                const int idx = (k * j * step) % MEL_NFFT;
                sr += x[j * stride] * mel_cos[idx];
                si -= x[j * stride] * mel_sin[idx];
            }
            re[k] = sr; im[k] = si;
        }
        return;
    }
    const int h = n / 2;
    float * er = tmp, * ei = tmp + h, * orr = tmp + 2 * h, * oi = tmp + 3 * h;
    mel_transform(x,          2 * stride, h, er,  ei, tmp + 4 * h);
    mel_transform(x + stride, 2 * stride, h, orr, oi, tmp + 4 * h);
    for (int k = 0; k < h; ++k) {
        const float c = mel_cos[k * step], s = -mel_sin[k * step];
        re[k]     = er[k] + c * orr[k] - s * oi[k];
        im[k]     = ei[k] + c * oi[k]  + s * orr[k];
        re[k + h] = er[k] - c * orr[k] + s * oi[k];
        im[k + h] = ei[k] - c * oi[k]  - s * orr[k];
    }
}

int64_t oracle_log_mel_n_len(int64_t n_samples) { return (n_samples + 480000) / MEL_HOP; }

/* returns n_len; mel must hold n_mel * n_len floats; n_samples > 200 */
int64_t oracle_log_mel_spectrogram(const float * samples, int64_t n_samples, const float * filters, int n_mel, float * mel) {
    mel_tables();
    const int     n_bins = MEL_NFFT / 2 + 1;
    const int64_t n_pad  = n_samples + 480000 + MEL_NFFT, n_len = (n_pad - MEL_NFFT) / MEL_HOP;
    const int64_t n_eff  = n_samples + MEL_NFFT / 2;
    float * padded = (float *) calloc((size_t) n_pad, sizeof(float));
    for (int q = 0; q < MEL_NFFT / 2; ++q) padded[q] = samples[MEL_NFFT / 2 - q];
    memcpy(padded + MEL_NFFT / 2, samples, (size_t) n_samples * sizeof(float));
    int64_t n_frames = n_eff / MEL_HOP + 1;
    if (n_frames > n_len) n_frames = n_len;
    float frame[MEL_NFFT], re[MEL_NFFT], im[MEL_NFFT], tmp[2 * 4 * MEL_NFFT], power[MEL_NFFT / 2 + 1];
    for (int64_t i = 0; i < n_len; ++i) {
        if (i >= n_frames) {
            for (int j = 0; j < n_mel; ++j) mel[(int64_t) j * n_len + i] = (float) log10(1e-10);
            continue;
        }
        const int64_t off = i * MEL_HOP;
        for (int j = 0; j < MEL_NFFT; ++j) frame[j] = off + j < n_eff ? mel_hann[j] * padded[off + j] : 0.0f;
        mel_transform(frame, 1, MEL_NFFT, re, im, tmp);
        for (int k = 0; k < n_bins; ++k) power[k] = re[k] * re[k] + im[k] * im[k];
        for (int j = 0; j < n_mel; ++j) {
            const float * f = filters + (int64_t) j * n_bins;
            double sum = 0.0;
            int k = 0;
            for (; k < n_bins - 3; k += 4) sum += power[k] * f[k] + power[k + 1] * f[k + 1] + power[k + 2] * f[k + 2] + power[k + 3] * f[k + 3];
            for (; k < n_bins; ++k) sum += power[k] * f[k];
            mel[(int64_t) j * n_len + i] = (float) log10(sum > 1e-10 ? sum : 1e-10);
        }
    }
    free(padded);
    double mmax = -1e20;
    for (int64_t i = 0; i < n_mel * n_len; ++i) if (mel[i] > mmax) mmax = mel[i];
    mmax -= 8.0;
    for (int64_t i = 0; i < n_mel * n_len; ++i) {
        if (mel[i] < mmax) mel[i] = (float) mmax;
        mel[i] = (float)((mel[i] + 4.0) / 4.0);
    }
    return n_len;
}
