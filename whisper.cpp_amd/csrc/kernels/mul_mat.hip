// MUL_MAT for gfx950 (ggml_compute_forward_mul_mat, ggml/src/ggml-cpu/ggml-cpu.c:1266-1458):
//   dst[m, n] = sum_k src0[k, m] * src1[k, n]        src0 = "W" (weights, rows m), src1 = "X" (rows n)
//
// Three kernels:
//   * k_gemm_mfma   — N > 8 columns.  128x128x64 tiles, 4 wavefronts in a 2x2 grid, each owning a 64x64
//                     patch as 2x2 v_mfma_f32_32x32x16_f16 accumulators.  W blocks (Q5_0 / Q8_0 / F16 /
//                     F32) are dequantized to f16 on their way into LDS, X (F32 / F16) is converted
//                     likewise; accumulation is f32.  X rows are the MFMA A operand and W rows the B
//                     operand, so that a lane's accumulator column is an m index and every store
//                     instruction writes 32 consecutive floats of dst.
//   * k_gemv_q      — N <= 8 columns, quantized W.  X is quantized to Q8_0 in LDS exactly as the CPU
//                     backend does before its dot products (quantize_row_q8_0, ggml-cpu-quants.c:808-865;
//                     ggml-cpu.c:1328-1363); each lane streams whole weight blocks from HBM and forms the
//                     integer block dot products with v_dot4_i32_i8, scaled by d_w*d_x like
//                     ggml_vec_dot_q8_0_q8_0 / ggml_vec_dot_q5_0_q8_0 (ggml-cpu-quants.c:3597, 2930).
//   * k_mul_mat_generic — any strides / K; one wavefront per output row, f32 FMA.
#include "common.h"

#include <algorithm>
#include <atomic>
#include <mutex>
#include <stdlib.h>
#include <type_traits>

typedef uint32_t __attribute__((aligned(2))) u32a2;
struct __attribute__((packed, aligned(2))) u128a2 { uint32_t x, y, z, w; };

// ------------------------------------------------------------------------------------------------------
// shared: epilogue
// ------------------------------------------------------------------------------------------------------

#include "mul_mat_args.h"
#include "gemv_q8_0_tiles.h"

__device__ __forceinline__ float apply_epilogue(float v, const epi_args & e, int64_t m, int64_t n, int64_t res_off) {
    if (e.flags & MI355X_EPI_BIAS)     v += e.bias[m];
    if (e.flags & MI355X_EPI_BIAS_COL) v += e.bias[n];
    if (e.flags & MI355X_EPI_GELU)     v  = gelu_f32(v, e.gelu);
    if (e.flags & MI355X_EPI_SCALE)    v *= e.scale;
    if (e.flags & MI355X_EPI_RESIDUAL) v += *(const float *)(e.residual + res_off);
    return v;
}

// The same for the 16 registers of one 32x32 accumulator patch (column m, rows n[0..15]) and the stores.  All loads of
// one kind are issued together before their first use; rows beyond N and columns beyond M are computed from clamped
// addresses and not stored.
// The part of the GELU table that the values in front of a GELU fall into, as a workgroup keeps it in LDS: the f16 patterns
// of |x| < 8 — 0x0000 .. 0x47ff and 0x8000 .. 0xc7ff, 2 x 18432 entries, 73728 bytes — positive half first.
#define GELU_LDS_HALF  0x4800
#define GELU_LDS_BYTES (2 * GELU_LDS_HALF * 2)

// FULL: the whole tile lies inside dst (no row or column of the patch is clamped or masked)
template <bool EMIT, bool FULL = false>
__device__ __forceinline__ void patch_epilogue(float16_t v, const epi_args & e, char * db, int64_t batch_off, int64_t d_nb1,
                                               int64_t m, int64_t M, const int64_t (&n)[16], int64_t N, const uint16_t * gelu_lds = nullptr) {
    const bool    m_ok = FULL || m < M;
    const int64_t mc   = m_ok ? m : M - 1;
    int64_t nc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) nc[i] = FULL || n[i] < N ? n[i] : N - 1;
    if (e.flags & MI355X_EPI_BIAS) {
        const float b = e.bias[mc];
#pragma unroll
        for (int i = 0; i < 16; ++i) v[i] += b;
    }
    if (e.flags & MI355X_EPI_BIAS_COL) {
        float b[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) b[i] = e.bias[nc[i]];
#pragma unroll
        for (int i = 0; i < 16; ++i) v[i] += b[i];
    }
    if (e.flags & MI355X_EPI_GELU) {
        if (gelu_lds) {
            // 64 gathers per lane out of the 128 KB table in global memory cost the FFN-up product 10 us of its 45; out of
            // LDS, 8.  A value near 8 or more in magnitude (none in a whisper model's activations) sends the wavefront through
            // the general form: the clamps at +-10 and the table in global memory for what the slice does not hold.
            bool far = false;
#pragma unroll
            for (int i = 0; i < 16; ++i) far = far || !(fabsf(v[i]) < 7.99f);   // (f16 rounds up to 8 from 7.998; NaN is far)
            if (!__any(far)) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const uint32_t hb = f2h_bits(v[i]);
                    v[i] = h2f(gelu_lds[(hb & 0x7FFFu) + (hb >> 15) * GELU_LDS_HALF]);
                }
            } else {
                uint32_t hb[16]; uint16_t t[16];
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    hb[i] = f2h_bits(v[i]);
                    const uint32_t a = hb[i] & 0x7FFFu;
                    t[i] = gelu_lds[(a < GELU_LDS_HALF ? a : 0u) + (hb[i] >> 15) * GELU_LDS_HALF];
                }
#pragma unroll
                for (int i = 0; i < 16; ++i) if ((hb[i] & 0x7FFFu) >= GELU_LDS_HALF) t[i] = e.gelu[hb[i]];
#pragma unroll
                for (int i = 0; i < 16; ++i) v[i] = v[i] <= -10.0f ? 0.0f : v[i] >= 10.0f ? v[i] : h2f(t[i]);
            }
        } else {
            uint16_t t[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) t[i] = e.gelu[f2h_bits(v[i])];
#pragma unroll
            for (int i = 0; i < 16; ++i) v[i] = v[i] <= -10.0f ? 0.0f : v[i] >= 10.0f ? v[i] : h2f(t[i]);
        }
    }
    if (e.flags & MI355X_EPI_SCALE) {
#pragma unroll
        for (int i = 0; i < 16; ++i) v[i] *= e.scale;
    }
    if (e.flags & MI355X_EPI_RESIDUAL) {
        float r[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) r[i] = *(const float *)(e.residual + batch_off + nc[i] * d_nb1 + mc * 4);
#pragma unroll
        for (int i = 0; i < 16; ++i) v[i] += r[i];
    }
    if (e.flags & MI355X_EPI_OUT_F16) {
#pragma unroll
        for (int i = 0; i < 16; ++i) if (m_ok && (FULL || n[i] < N)) *(half_t *)(db + n[i] * d_nb1 + m * 2) = (half_t) v[i];
    } else if (!EMIT || !(e.flags & MI355X_EPI_IMAGE_ONLY)) {
#pragma unroll
        for (int i = 0; i < 16; ++i) if (m_ok && (FULL || n[i] < N)) *(float *)(db + n[i] * d_nb1 + m * 4) = v[i];
    }
    if (EMIT) {
        // The product that reads dst next rounds its rows to Q8_0 first.  The 32 lanes of a half-wavefront hold 32
        // consecutive m of one dst row — exactly one Q8_0 block (M % 32 == 0) — so the block maximum is a 5-step
        // butterfly, and the image f16(q * d) is written here instead of by a pass of its own over dst.
        // The two divisions of a block (127 / amax and amax / 127) would be repeated by all 32 lanes that hold it, for each
        // of the 16 registers: 32 IEEE divisions per lane and patch, most of this epilogue's time.  Instead lane l divides
        // for register l % 16 of its half-wavefront, and the 16 results travel back by lane permutes.
        // Block maxima: v_permlane16_swap of registers i and i + 8 leaves, in the even rows of 16 lanes, both halves of
        // register i's block and, in the odd rows, both halves of register i + 8's — one swap and one maximum take the
        // first butterfly step for two registers and halve what the other four steps (inside a row) have to carry.
        float rmax[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const auto sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(v[i]), __float_as_uint(v[i + 8]), false, false);
            // (the row steps on the bit patterns: non-negative floats order like unsigned integers, and an integer maximum
            // takes its DPP operand in the same instruction)
            rmax[i] = __uint_as_float(lanes_reduce<16>(__float_as_uint(fmaxf(fabsf(__uint_as_float(sw[0])), fabsf(__uint_as_float(sw[1])))),
                                                        [](uint32_t a, uint32_t b) { return a > b ? a : b; }));
        }
        const int lane = threadIdx.x & 63;
        float mine = rmax[0];                               // lane (row, c) of a half-wavefront: register c % 8 + 8 (row % 2)
#pragma unroll
        for (int i = 1; i < 8; ++i) mine = (lane & 7) == i ? rmax[i] : mine;
        const float id_m = mine != 0.0f ? 127.0f / mine : 0.0f;
        const float dq_m = h2f(f2h_bits(div127(mine)));
        const int src = ((lane & 32) << 2);                 // byte address of lane 0 of this half-wavefront for ds_bpermute
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int from = src + 4 * ((i & 7) + (i >= 8 ? 16 : 0));
            const float id = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(from, __builtin_bit_cast(int, id_m)));
            const float dq = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(from, __builtin_bit_cast(int, dq_m)));
            if (m_ok && (FULL || n[i] < N)) e.image[n[i] * M + m] = (half_t)((rintf(v[i] * id) + 0.0f) * dq);
        }
    }
}


// The same for a patch formed the other way round (the weights as the matrix instruction's A operand): the lane owns ONE dst row
// n and 16 of the 32 consecutive m of a patch row — m = mb + 8 q + t, q = e / 4, t = e % 4, with mb = the patch's first m +
// 4 (lane / 32) — and lane + 32 owns the other 16.  That is half a Q8_0 block per lane: the block maximum is 8 three-operand
// maxima and one exchange with lane + 32 instead of five cross-lane steps for each of 16 registers, both divisions are the
// lane's own (no permutes hand them round), bias, residual and stores move four consecutive values at a time.
// M a multiple of 32 (a patch lies inside dst's columns or outside); FULL: the patch is inside and n < N.
template <bool FULL>
__device__ __forceinline__ void patch_epilogue_t(float16_t v, const epi_args & e, char * db, int64_t batch_off, int64_t d_nb1,
                                                 int64_t mb, int64_t M, int64_t n, int64_t N, const uint16_t * gelu_lds) {
    const bool    ok = FULL || (n < N && mb < M);
    const int64_t nc = FULL || n < N ? n : N - 1;
    const int64_t mc = FULL || mb < M ? mb : M - 32 + (mb & 31);
    if (e.flags & MI355X_EPI_BIAS) {
        float4 b[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) b[q] = *(const float4 *)(e.bias + mc + 8 * q);
#pragma unroll
        for (int q = 0; q < 4; ++q) { v[4 * q] += b[q].x; v[4 * q + 1] += b[q].y; v[4 * q + 2] += b[q].z; v[4 * q + 3] += b[q].w; }
    }
    if (e.flags & MI355X_EPI_BIAS_COL) {
        const float b = e.bias[nc];
#pragma unroll
        for (int i = 0; i < 16; ++i) v[i] += b;
    }
    if (e.flags & MI355X_EPI_GELU) {
        if (gelu_lds) {
            // the table slice in LDS holds |x| < 8: the f16 patterns below 0x4800 (infinity and NaN lie above); one integer
            // maximum over the patterns decides for the wavefront, the general form is the one of patch_epilogue
            uint32_t hb[16], top = 0;
#pragma unroll
            for (int i = 0; i < 16; ++i) { hb[i] = f2h_bits(v[i]); top = max(top, hb[i] & 0x7FFFu); }
            if (!__any(top >= GELU_LDS_HALF)) {
#pragma unroll
                for (int i = 0; i < 16; ++i) v[i] = h2f(gelu_lds[(hb[i] & 0x7FFFu) + (hb[i] >> 15) * GELU_LDS_HALF]);
            } else {
                uint16_t t[16];
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const uint32_t a = hb[i] & 0x7FFFu;
                    t[i] = gelu_lds[(a < GELU_LDS_HALF ? a : 0u) + (hb[i] >> 15) * GELU_LDS_HALF];
                }
#pragma unroll
                for (int i = 0; i < 16; ++i) if ((hb[i] & 0x7FFFu) >= GELU_LDS_HALF) t[i] = e.gelu[hb[i]];
#pragma unroll
                for (int i = 0; i < 16; ++i) v[i] = v[i] <= -10.0f ? 0.0f : v[i] >= 10.0f ? v[i] : h2f(t[i]);
            }
        } else {
            uint16_t t[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) t[i] = e.gelu[f2h_bits(v[i])];
#pragma unroll
            for (int i = 0; i < 16; ++i) v[i] = v[i] <= -10.0f ? 0.0f : v[i] >= 10.0f ? v[i] : h2f(t[i]);
        }
    }
    if (e.flags & MI355X_EPI_SCALE) {
#pragma unroll
        for (int i = 0; i < 16; ++i) v[i] *= e.scale;
    }
    if (e.flags & MI355X_EPI_RESIDUAL) {
        float4 r[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) r[q] = *(const float4 *)(e.residual + batch_off + nc * d_nb1 + (mc + 8 * q) * 4);
#pragma unroll
        for (int q = 0; q < 4; ++q) { v[4 * q] += r[q].x; v[4 * q + 1] += r[q].y; v[4 * q + 2] += r[q].z; v[4 * q + 3] += r[q].w; }
    }
    if (e.flags & MI355X_EPI_OUT_F16) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
            if (ok) *(half4_t *)(db + n * d_nb1 + (mb + 8 * q) * 2) = (half4_t){ (half_t) v[4 * q], (half_t) v[4 * q + 1], (half_t) v[4 * q + 2], (half_t) v[4 * q + 3] };
    } else if (!(e.flags & MI355X_EPI_IMAGE_ONLY)) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
            if (ok) *(float4 *)(db + n * d_nb1 + (mb + 8 * q) * 4) = make_float4(v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]);
    }
    // the image: rounded to Q8_0 as the product that reads dst next rounds its rows (see patch_epilogue)
    float amax = fmaxf(fabsf(v[0]), fabsf(v[1]));
#pragma unroll
    for (int i = 2; i < 16; ++i) amax = fmaxf(amax, fabsf(v[i]));
    {   // ... and the half of the block that lane ^ 32 holds (v_permlane32_swap of the value with itself: own half, other half)
        const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(amax), __float_as_uint(amax), false, false);
        amax = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
    }
    const float id = amax != 0.0f ? 127.0f / amax : 0.0f;
    const float dq = h2f(f2h_bits(div127(amax)));
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        // (the addend +0 of the multiply-add turns a product -0 into the +0 that an integer quant of zero gives)
        const half4_t h = { (half_t) __builtin_fmaf(rintf(v[4 * q] * id), dq, 0.0f), (half_t) __builtin_fmaf(rintf(v[4 * q + 1] * id), dq, 0.0f),
                            (half_t) __builtin_fmaf(rintf(v[4 * q + 2] * id), dq, 0.0f), (half_t) __builtin_fmaf(rintf(v[4 * q + 3] * id), dq, 0.0f) };
        if (ok) *(half4_t *)(e.image + n * M + mb + 8 * q) = h;
    }
}


// ------------------------------------------------------------------------------------------------------
// block -> 32 f16 weights
// ------------------------------------------------------------------------------------------------------

// bytes (b0,b1) / (b2,b3) of v, each in [0,255], become the f16 pair (b - bias): 0x6400|b is the f16 1024+b.
__device__ __forceinline__ half2_t bytes_lo_to_half2(uint32_t v, half2_t bias) {
    uint32_t u = (v & 0xFFu) | ((v << 8) & 0xFF0000u) | 0x64006400u;
    half2_t h; __builtin_memcpy(&h, &u, 4);
    return h - bias;
}
__device__ __forceinline__ half2_t bytes_hi_to_half2(uint32_t v, half2_t bias) {
    uint32_t u = ((v >> 16) & 0xFFu) | ((v >> 8) & 0xFF0000u) | 0x64006400u;
    half2_t h; __builtin_memcpy(&h, &u, 4);
    return h - bias;
}
// four bits -> bit 4 of four bytes
__device__ __forceinline__ uint32_t spread4_to_bit4(uint32_t nib) {
    return ((nib * 0x00204081u) & 0x01010101u) << 4;
}

// f16(d * q) equals the f16 rounding of the exact product: q is a small integer, so (q as f16) * (d as f16)
// in one v_pk_mul_f16 rounds once.
__device__ __forceinline__ void q5_0_to_half32(uint32_t d_bits, uint32_t qh, const uint32_t qs[4], half8_t out[4]) {
    half_t d; { uint16_t t = (uint16_t) d_bits; __builtin_memcpy(&d, &t, 2); }
    const half2_t d2 = { d, d };
    const half2_t bias = { (half_t) 1040.0f, (half_t) 1040.0f };   // 1024 + 16
    half2_t * o = (half2_t *) out;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t q  = qs[i];
        const uint32_t lo = (q & 0x0F0F0F0Fu)        | spread4_to_bit4((qh >> (4*i))      & 0xFu);
        const uint32_t hi = ((q >> 4) & 0x0F0F0F0Fu) | spread4_to_bit4((qh >> (16 + 4*i)) & 0xFu);
        o[2*i + 0]     = bytes_lo_to_half2(lo, bias) * d2;   // k = 4i, 4i+1
        o[2*i + 1]     = bytes_hi_to_half2(lo, bias) * d2;   // k = 4i+2, 4i+3
        o[8 + 2*i + 0] = bytes_lo_to_half2(hi, bias) * d2;   // k = 16+4i ..
        o[8 + 2*i + 1] = bytes_hi_to_half2(hi, bias) * d2;
    }
}
__device__ __forceinline__ void q8_0_to_half32(uint32_t d_bits, const uint32_t qs[8], half8_t out[4]) {
    half_t d; { uint16_t t = (uint16_t) d_bits; __builtin_memcpy(&d, &t, 2); }
    const half2_t d2 = { d, d };
    const half2_t bias = { (half_t) 1152.0f, (half_t) 1152.0f };   // 1024 + 128
    half2_t * o = (half2_t *) out;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const uint32_t v = qs[i] ^ 0x80808080u;                    // int8 -> biased uint8
        o[2*i + 0] = bytes_lo_to_half2(v, bias) * d2;
        o[2*i + 1] = bytes_hi_to_half2(v, bias) * d2;
    }
}

// ------------------------------------------------------------------------------------------------------
// MFMA GEMM: operand conversion passes + one f16 x f16 -> f32 kernel
//
// Both operands reach the matrix cores as dense f16 rows [rows][K]:
//   * src1 (F32) is converted by k_x_to_f16.  For quantized weights the CPU backend first rounds src1 to Q8_0
//     (ggml-cpu.c:1328-1363, quantize_row_q8_0 ggml-cpu-quants.c:808-865): the pass reproduces that rounding —
//     block amax, id = 127/amax, round half to even, d stored as f16 — and writes f16(q * d).  For F16 / F32
//     weights (or when the caller asks for un-rounded activations) it is a plain f32 -> f16 conversion, which is
//     what the CPU backend does for F16 weights.
//   * src0 blocks are expanded by k_w_to_f16 to f16(d * q) unless src0 already is F16.  A caller that multiplies by
//     the same weights many times keeps that f16 image itself and passes it as an F16 src0 with MI355X_MM_ACT_Q8_0.
// ------------------------------------------------------------------------------------------------------

static inline size_t round256(size_t n) { return (n + 255) / 256 * 256; }

// one thread per 32 weights
template <int T0>
__global__ void k_w_to_f16(const char * __restrict__ w, half_t * __restrict__ out, int64_t K, int64_t M, int64_t w_nb1, int64_t w_nb2,
                           int64_t ne02, int64_t w_nb3, int64_t slice_halves) {
    const int64_t t   = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t nbk = K / QK;
    if (t >= nbk * M) return;
    const int64_t m = t / nbk, kb = t % nbk, b = blockIdx.y;
    const uint8_t * row = (const uint8_t *) w + m * w_nb1 + (b % ne02) * w_nb2 + (b / ne02) * w_nb3;
    half8_t o[4];
    if constexpr (T0 == MI355X_TYPE_Q5_0) {
        const uint8_t * p = row + kb * 22;
        const u128a2 q = *(const u128a2 *)(p + 6);
        const uint32_t qs[4] = { q.x, q.y, q.z, q.w };
        q5_0_to_half32(*(const uint16_t *) p, *(const u32a2 *)(p + 2), qs, o);
    } else if constexpr (T0 == MI355X_TYPE_Q8_0) {
        const uint8_t * p = row + kb * 34;
        const u128a2 q0 = *(const u128a2 *)(p + 2), q1 = *(const u128a2 *)(p + 18);
        const uint32_t qs[8] = { q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w };
        q8_0_to_half32(*(const uint16_t *) p, qs, o);
    } else {
        const float4 * p = (const float4 *)(row + kb * QK * 4);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float4 u = p[2*i], v = p[2*i + 1];
            o[i] = (half8_t){ (half_t) u.x, (half_t) u.y, (half_t) u.z, (half_t) u.w, (half_t) v.x, (half_t) v.y, (half_t) v.z, (half_t) v.w };
        }
    }
    half8_t * dst = (half8_t *)(out + b * slice_halves + m * K + kb * QK);
#pragma unroll
    for (int i = 0; i < 4; ++i) dst[i] = o[i];
}

// 8 lanes per 32 values, 4 each
template <bool Q8>
__global__ void k_x_to_f16(const char * __restrict__ x, half_t * __restrict__ out, int64_t K, int64_t N,
                           int64_t x_nb1, int64_t x_nb2, int64_t ne12, int64_t x_nb3, int64_t slice_halves) {
    const int64_t t  = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t k4 = K / 4;
    const int64_t b  = blockIdx.y;
    if (t >= k4 * N) return;                                                // whole 8-lane groups leave together (K % 32 == 0 when Q8)
    const int64_t n = t / k4, c = t % k4;
    const float4 v = *(const float4 *)(x + n * x_nb1 + (b % ne12) * x_nb2 + (b / ne12) * x_nb3 + c * 16);
    half4_t h;
    if (Q8) {
        float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
        amax = lanes_max<8>(amax);
        const float id = amax != 0.0f ? 127.0f / amax : 0.0f;
        const float d  = h2f(f2h_bits(div127(amax)));                      // the scale goes through f16, like block_q8_0.d
        // (+ 0.0f: a quant that rounds to -0 is the integer 0, whose product with d is +0)
        h = (half4_t){ (half_t)((rintf(v.x * id) + 0.0f) * d), (half_t)((rintf(v.y * id) + 0.0f) * d), (half_t)((rintf(v.z * id) + 0.0f) * d), (half_t)((rintf(v.w * id) + 0.0f) * d) };
    } else {
        h = (half4_t){ (half_t) v.x, (half_t) v.y, (half_t) v.z, (half_t) v.w };
    }
    *(half4_t *)(out + b * slice_halves + n * K + c * 4) = h;
}

// f16 x f16 -> f32 GEMM.  256 threads = 4 wavefronts in a 2 x 2 grid; a wavefront owns TI x TJ accumulator patches of
// 32 (src1 rows, n) x 32 (weight rows, m), each a v_mfma_f32_32x32x16_f16 chain.  src1 rows are the MFMA A operand and
// weight rows the B operand, so a lane's accumulator column is an m index and every store instruction writes 32
// consecutive values of a dst row.  K advances 64 at a time through two LDS buffers: while the matrix cores work on
// step s, the global loads of step s+2 are in flight and step s+1 moves from registers to the other buffer, with one
// barrier per step.  LDS rows are padded to 144 B so that the 16-byte operand reads of 16 consecutive rows hit
// distinct banks.  What bounds the kernel is the staging, not the K loop: with the operands already in LDS the loop runs
// at 1400 TFLOP/s (8192^3); the LDS stores bring that to 1155 and the global loads to 805 — a 128 x 128 x 64 step
// fetches 32 KB through a vector memory path of 64 B per clock and CU, as many clocks as its matrix instructions take.
#define GB_K  64
#define GB_LD (GB_K + 8)


// What follows the K loop of a tile: GELU reads its table from LDS when the operand buffers, free now (the loop's last barrier
// is behind every wavefront), are large enough to hold the part that matters (TABLE_FITS); then the 32x32 patches.
// (NT: threads of the workgroup; the patches belong to the first 256.  TR: the patches were formed with the weights as the
// matrix instruction's A operand — lanes own dst rows, registers own columns — which the image-emitting epilogue prefers)
template <int TI, int TJ, bool EMIT, bool TABLE_FITS, int NT = 256, bool TR = false>
__device__ __forceinline__ void gemm_tile_epilogue(float16_t (&acc)[TI][TJ], const mm_args & a, const epi_args & epi, char * db, int64_t batch_off, int64_t d_nb1,
                                                   int64_t n0, int64_t m0, int wn, int wmo, char * smem) {
    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
    const uint16_t * gelu_lds = nullptr;
    if constexpr (TABLE_FITS) {
        if (epi.flags & MI355X_EPI_GELU) {
            const u32x4 * pos = (const u32x4 *) epi.gelu, * neg = (const u32x4 *)(epi.gelu + 0x8000);
            u32x4 * dst = (u32x4 *) smem;
            constexpr int pieces = GELU_LDS_HALF * 2 / 16;
            for (int p = tid; p < pieces; p += NT) { dst[p] = pos[p]; dst[pieces + p] = neg[p]; }
            __syncthreads();
            gelu_lds = (const uint16_t *) smem;
        }
    }
    if (NT > 256 && tid >= 256) return;
    if constexpr (TR) {
        static_assert(EMIT, "the transposed patches are the image-emitting kernel's");
        // accumulator register e of a 32x32 patch: column (= n) lane%32, row (= m) 8*(e/4) + 4*g + e%4
        auto patches_t = [&](auto full) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < TI; ++i)
#pragma unroll
                for (int j = 0; j < TJ; ++j)
                    patch_epilogue_t<decltype(full)::value>(acc[i][j], epi, db, batch_off, d_nb1, m0 + wmo + 32 * j + 4 * g, a.M, n0 + wn + 32 * i + l32, a.N, gelu_lds);
        };
        if (n0 + 64 * TI <= a.N && m0 + 64 * TJ <= a.M) patches_t(std::true_type{}); else patches_t(std::false_type{});
        return;
    }
    // accumulator register e of a 32x32 patch: row (= n) 8*(e/4) + 4*g + e%4, column (= m) lane%32
    auto patches = [&](auto full) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < TI; ++i) {
            int64_t n[16];
#pragma unroll
            for (int e = 0; e < 16; ++e) n[e] = n0 + wn + 32 * i + 8 * (e >> 2) + 4 * g + (e & 3);
#pragma unroll
            for (int j = 0; j < TJ; ++j)
                patch_epilogue<EMIT, decltype(full)::value>(acc[i][j], epi, db, batch_off, d_nb1, m0 + wmo + 32 * j + l32, a.M, n, a.N, gelu_lds);
        }
    };
    // tiles inside dst (all but the last row of tiles when N = 1500) store without per-element bounds
    if (n0 + 64 * TI <= a.N && m0 + 64 * TJ <= a.M) patches(std::true_type{}); else patches(std::false_type{});
}

// KTAIL: K is not a multiple of 64 (but of 8); FULL: K / 64 is a multiple of S; EMIT: MI355X_EPI_EMIT_F16 (a kernel of its
// own, because its epilogue needs more registers than two workgroups per CU leave)
template <int TI, int TJ, int S, bool KTAIL, bool FULL, bool EMIT = false>
__device__ __forceinline__ void gemm_f16_tile(const mm_args & a, int tiles_m, int tiles_n, int sw, int tile, const char * wb, const char * xb, char * db,
                                              const epi_args & epi, int64_t batch_off, int64_t d_nb1) {
    constexpr int BN = 64 * TI, BM = 64 * TJ;
    constexpr int XR = BN / 32, WR = BM / 32;          // 16-byte pieces per thread and step
    extern __shared__ __attribute__((aligned(16))) char smem[];
    half_t * xs_base = (half_t *) smem;                // [2][BN * GB_LD]
    half_t * ws_base = xs_base + 2 * BN * GB_LD;       // [2][BM * GB_LD]

    // `tile` counts along a path over the tile grid that walks columns of `sw` m-tiles, each from the first n-panel to the
    // last (m fastest inside the column): a run of consecutive tiles — what one XCD gets, see xcd_run_index — then covers
    // about sqrt(run) tiles in each direction, the shape that touches the fewest X and W rows.
    const int per_col = sw * tiles_n, col = tile / per_col, rem = tile - col * per_col;
    const int cw = min(sw, tiles_m - col * sw);        // (the last column is narrower when sw does not divide tiles_m)
    const int64_t m0 = (int64_t)(col * sw + rem % cw) * BM;
    const int64_t n0 = (int64_t)(rem / cw) * BN;

    const int tid = threadIdx.x;
    const int lc = tid & 7, lr = tid >> 3;             // piece column (8 halves) and first row of this thread
    // rows beyond N / M are read from the last valid row: what they produce is never stored
    const char * xp[XR]; const char * wp[WR];
#pragma unroll
    for (int i = 0; i < XR; ++i) { const int64_t n = n0 + lr + 32 * i; xp[i] = xb + (n < a.N ? n : a.N - 1) * a.x_nb1 + lc * 16; }
#pragma unroll
    for (int i = 0; i < WR; ++i) { const int64_t m = m0 + lr + 32 * i; wp[i] = wb + (m < a.M ? m : a.M - 1) * a.w_nb1 + lc * 16; }

    // S steps of operands are in flight in registers (slot = step % S)
    u32x4 xrs[S][XR], wrs[S][WR];
    auto load = [&](u32x4 (&xr)[XR], u32x4 (&wr)[WR], int64_t k0) __attribute__((always_inline)) {
        if (KTAIL) {                                   // pieces beyond K are read from k = 0 and zeroed
            const bool kok = k0 + 8 * lc < a.K;
            const int64_t ko = kok ? k0 * 2 : -(int64_t) lc * 16;
#pragma unroll
            for (int i = 0; i < XR; ++i) { const u32x4 v = *(const u32x4 *)(xp[i] + ko); xr[i] = kok ? v : (u32x4){0, 0, 0, 0}; }
#pragma unroll
            for (int i = 0; i < WR; ++i) { const u32x4 v = *(const u32x4 *)(wp[i] + ko); wr[i] = kok ? v : (u32x4){0, 0, 0, 0}; }
        } else {
#pragma unroll
            for (int i = 0; i < XR; ++i) xr[i] = *(const u32x4 *)(xp[i] + k0 * 2);
#pragma unroll
            for (int i = 0; i < WR; ++i) wr[i] = *(const u32x4 *)(wp[i] + k0 * 2);
        }
    };
    auto store = [&](const u32x4 (&xr)[XR], const u32x4 (&wr)[WR], int buf) __attribute__((always_inline)) {
        half_t * xs = xs_base + buf * BN * GB_LD, * ws = ws_base + buf * BM * GB_LD;
#pragma unroll
        for (int i = 0; i < XR; ++i) *(u32x4 *)(xs + (lr + 32 * i) * GB_LD + 8 * lc) = xr[i];
#pragma unroll
        for (int i = 0; i < WR; ++i) *(u32x4 *)(ws + (lr + 32 * i) * GB_LD + 8 * lc) = wr[i];
    };

    const int lane = tid & 63, wave = tid >> 6;
    const int wn = (wave >> 1) * 32 * TI, wmo = (wave & 1) * 32 * TJ;   // wave patch origin inside the tile
    const int l32 = lane & 31, g = lane >> 5;

    float16_t acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    const int KT = (int)((a.K + GB_K - 1) / GB_K);
    // one K step: the operand fragments of sub-step kk + 1 are read from LDS while the matrix cores work on kk
    auto mma = [&](int buf) __attribute__((always_inline)) {
        const half_t * xs = xs_base + buf * BN * GB_LD + (wn  + l32) * GB_LD + 8 * g;
        const half_t * ws = ws_base + buf * BM * GB_LD + (wmo + l32) * GB_LD + 8 * g;
        half8_t av[2][TI], bv[2][TJ];
#pragma unroll
        for (int i = 0; i < TI; ++i) av[0][i] = *(const half8_t *)(xs + 32 * i * GB_LD);
#pragma unroll
        for (int j = 0; j < TJ; ++j) bv[0][j] = *(const half8_t *)(ws + 32 * j * GB_LD);
#pragma unroll
        for (int kk = 0; kk < GB_K / 16; ++kk) {
            const int c = kk & 1, nx = c ^ 1;
            if (kk + 1 < GB_K / 16) {
#pragma unroll
                for (int i = 0; i < TI; ++i) av[nx][i] = *(const half8_t *)(xs + 32 * i * GB_LD + (kk + 1) * 16);
#pragma unroll
                for (int j = 0; j < TJ; ++j) bv[nx][j] = *(const half8_t *)(ws + 32 * j * GB_LD + (kk + 1) * 16);
            }
#pragma unroll
            for (int i = 0; i < TI; ++i)
#pragma unroll
                for (int j = 0; j < TJ; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av[c][i], bv[c][j], acc[i][j], 0, 0, 0);
            if (kk + 1 < GB_K / 16) {
                // issue order: one LDS read after each of the first matrix instructions of this sub-step
#pragma unroll
                for (int r = 0; r < TI + TJ; ++r) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // 1 MFMA
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // 1 DS read
                }
            }
        }
    };
    if constexpr (FULL) {
        // The number of steps is a multiple of S: every step stores and loads unconditionally (beyond the end it re-reads
        // the last step's operands, which nobody consumes).  With no load behind a branch the compiler knows how many
        // are outstanding at every point and waits for exactly the oldest slot — with conditional loads it has to assume
        // the younger ones were never issued, waits for all of them, and the ring degenerates to one step in flight.
        const int last = KT - 1;
#pragma unroll
        for (int st = 0; st < S; ++st) load(xrs[st], wrs[st], (int64_t) st * GB_K);
        store(xrs[0], wrs[0], 0);
        load(xrs[0], wrs[0], (int64_t) min(S, last) * GB_K);
        __syncthreads();
        auto step = [&](int kt, int buf, u32x4 (&xr)[XR], u32x4 (&wr)[WR]) __attribute__((always_inline)) {   // xr / wr: slot of step kt + 1
            mma(buf);
            store(xr, wr, buf ^ 1);                     // the last readers of that buffer passed the previous barrier
            load(xr, wr, (int64_t) min(kt + 1 + S, last) * GB_K);
            __syncthreads();
        };
        for (int kt0 = 0; kt0 < KT; kt0 += S) {         // S is even: the LDS buffer of a step is the parity of its slot
            step(kt0 + 0, 0, xrs[1 % S], wrs[1 % S]);
            step(kt0 + 1, 1, xrs[2 % S], wrs[2 % S]);
            if (S > 2) { step(kt0 + 2, 0, xrs[3 % S], wrs[3 % S]); step(kt0 + 3, 1, xrs[4 % S], wrs[4 % S]); }
            if (S > 4) { step(kt0 + 4, 0, xrs[5 % S], wrs[5 % S]); step(kt0 + 5, 1, xrs[6 % S], wrs[6 % S]); }
        }
    } else {
        load(xrs[0], wrs[0], 0);
        if (1 < KT) load(xrs[1], wrs[1], GB_K);
        if (S > 2) { if (2 < KT) load(xrs[2 % S], wrs[2 % S], 2 * GB_K); if (3 < KT) load(xrs[3 % S], wrs[3 % S], 3 * GB_K); }
        if (S > 4) { if (4 < KT) load(xrs[4 % S], wrs[4 % S], 4 * GB_K); if (5 < KT) load(xrs[5 % S], wrs[5 % S], 5 * GB_K); }
        store(xrs[0], wrs[0], 0);
        if (S < KT) load(xrs[0], wrs[0], (int64_t) S * GB_K);
        __syncthreads();
        auto step = [&](int kt, int buf, u32x4 (&xr)[XR], u32x4 (&wr)[WR]) __attribute__((always_inline)) {
            mma(buf);
            if (kt + 1 < KT) {
                store(xr, wr, buf ^ 1);
                if (kt + 1 + S < KT) load(xr, wr, (int64_t)(kt + 1 + S) * GB_K);
            }
            __syncthreads();
        };
        for (int kt0 = 0; kt0 < KT; kt0 += S) {
            if (kt0 + 0 < KT) step(kt0 + 0, 0, xrs[1 % S], wrs[1 % S]);
            if (kt0 + 1 < KT) step(kt0 + 1, 1, xrs[2 % S], wrs[2 % S]);
            if (S > 2) {
                if (kt0 + 2 < KT) step(kt0 + 2, 0, xrs[3 % S], wrs[3 % S]);
                if (kt0 + 3 < KT) step(kt0 + 3, 1, xrs[4 % S], wrs[4 % S]);
            }
            if (S > 4) {
                if (kt0 + 4 < KT) step(kt0 + 4, 0, xrs[5 % S], wrs[5 % S]);
                if (kt0 + 5 < KT) step(kt0 + 5, 1, xrs[6 % S], wrs[6 % S]);
            }
        }
    }

    gemm_tile_epilogue<TI, TJ, EMIT, ((size_t) 2 * (BN + BM) * GB_LD * sizeof(half_t) >= GELU_LDS_BYTES)>(acc, a, epi, db, batch_off, d_nb1, n0, m0, wn, wmo, smem);
}

// The same tile by a workgroup of eight wavefronts in two roles: wavefronts 4 .. 7 move the operands (global loads into a
// register ring, LDS stores of the step after next), wavefronts 0 .. 3 issue the matrix instructions of the current step,
// one barrier per step between them.  In the one-role loop above a wavefront spends two thirds of a step issuing loads and
// stores, during which it issues no matrix instruction; here the matrix wavefronts do nothing else, and a SIMD holds
// one of each role per workgroup.  K a multiple of 64 S.
// NP: threads that move operands (256 or 512), behind the 256 that multiply
template <int TI, int TJ, int S, bool EMIT, int NP>
__device__ __forceinline__ void gemm_f16_tile_rs(const mm_args & a, int tiles_m, int tiles_n, int sw, int tile, const char * wb, const char * xb, char * db,
                                                 const epi_args & epi, int64_t batch_off, int64_t d_nb1) {
    constexpr int BN = 64 * TI, BM = 64 * TJ;
    constexpr int RP = NP / 8;                         // rows that the operand threads cover in one pass (8 threads to a row)
    constexpr int XR = BN / RP, WR = BM / RP;          // 16-byte pieces per operand thread and step
    static_assert(BN % RP == 0 && BM % RP == 0, "");
    extern __shared__ __attribute__((aligned(16))) char smem[];
    half_t * xs_base = (half_t *) smem;                // [2][BN * GB_LD]
    half_t * ws_base = xs_base + 2 * BN * GB_LD;       // [2][BM * GB_LD]

    const int per_col = sw * tiles_n, col = tile / per_col, rem = tile - col * per_col;
    const int cw = min(sw, tiles_m - col * sw);
    const int64_t m0 = (int64_t)(col * sw + rem % cw) * BM;
    const int64_t n0 = (int64_t)(rem / cw) * BN;

    const int tid = threadIdx.x;
    const int KT = (int)(a.K / GB_K), last = KT - 1;
    const int lane = tid & 63, wave = (tid >> 6) & 3;
    const int wn = (wave >> 1) * 32 * TI, wmo = (wave & 1) * 32 * TJ;   // (matrix wavefronts) patch origin inside the tile

    float16_t acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    if (tid >= 256) {
        // ---- operand wavefronts
        const int pt = tid - 256, lc = pt & 7, lr = pt >> 3;
        const char * xp[XR]; const char * wp[WR];
#pragma unroll
        for (int i = 0; i < XR; ++i) { const int64_t n = n0 + lr + RP * i; xp[i] = xb + (n < a.N ? n : a.N - 1) * a.x_nb1 + lc * 16; }
#pragma unroll
        for (int i = 0; i < WR; ++i) { const int64_t m = m0 + lr + RP * i; wp[i] = wb + (m < a.M ? m : a.M - 1) * a.w_nb1 + lc * 16; }
        u32x4 xrs[S][XR], wrs[S][WR];
        auto load = [&](u32x4 (&xr)[XR], u32x4 (&wr)[WR], int64_t k0) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < XR; ++i) xr[i] = *(const u32x4 *)(xp[i] + k0 * 2);
#pragma unroll
            for (int i = 0; i < WR; ++i) wr[i] = *(const u32x4 *)(wp[i] + k0 * 2);
        };
        auto store = [&](const u32x4 (&xr)[XR], const u32x4 (&wr)[WR], int buf) __attribute__((always_inline)) {
            half_t * xs = xs_base + buf * BN * GB_LD, * ws = ws_base + buf * BM * GB_LD;
#pragma unroll
            for (int i = 0; i < XR; ++i) *(u32x4 *)(xs + (lr + RP * i) * GB_LD + 8 * lc) = xr[i];
#pragma unroll
            for (int i = 0; i < WR; ++i) *(u32x4 *)(ws + (lr + RP * i) * GB_LD + 8 * lc) = wr[i];
        };
        // every step loads unconditionally (beyond the end: the last step again), so the waits are counts, not vmcnt(0)
#pragma unroll
        for (int st = 0; st < S; ++st) load(xrs[st], wrs[st], (int64_t) min(st, last) * GB_K);
        store(xrs[0], wrs[0], 0);
        load(xrs[0], wrs[0], (int64_t) min(S, last) * GB_K);
        __syncthreads();                               // step 0 is in LDS
        auto step = [&](int kt, int buf, u32x4 (&xr)[XR], u32x4 (&wr)[WR]) __attribute__((always_inline)) {   // xr / wr: slot of step kt + 1
            store(xr, wr, buf ^ 1);                     // the matrix wavefronts read `buf`; the readers of buf ^ 1 passed the last barrier
            load(xr, wr, (int64_t) min(kt + 1 + S, last) * GB_K);
            __syncthreads();
        };
        for (int kt0 = 0; kt0 < KT; kt0 += S) {
            step(kt0 + 0, 0, xrs[1 % S], wrs[1 % S]);
            step(kt0 + 1, 1, xrs[2 % S], wrs[2 % S]);
            if (S > 2) { step(kt0 + 2, 0, xrs[3 % S], wrs[3 % S]); step(kt0 + 3, 1, xrs[4 % S], wrs[4 % S]); }
        }
    } else {
        // ---- matrix wavefronts
        const int l32 = lane & 31, g = lane >> 5;
        auto mma = [&](int buf) __attribute__((always_inline)) {
            const half_t * xs = xs_base + buf * BN * GB_LD + (wn  + l32) * GB_LD + 8 * g;
            const half_t * ws = ws_base + buf * BM * GB_LD + (wmo + l32) * GB_LD + 8 * g;
            // fragments of sub-step kk + 1 are read while the matrix cores work on kk (two sets of registers: with two
            // workgroups to a CU a wavefront has 128)
            half8_t av[2][TI], bv[2][TJ];
#pragma unroll
            for (int i = 0; i < TI; ++i) av[0][i] = *(const half8_t *)(xs + 32 * i * GB_LD);
#pragma unroll
            for (int j = 0; j < TJ; ++j) bv[0][j] = *(const half8_t *)(ws + 32 * j * GB_LD);
#pragma unroll
            for (int kk = 0; kk < GB_K / 16; ++kk) {
                const int c = kk & 1, nx = c ^ 1;
                if (kk + 1 < GB_K / 16) {
#pragma unroll
                    for (int i = 0; i < TI; ++i) av[nx][i] = *(const half8_t *)(xs + 32 * i * GB_LD + (kk + 1) * 16);
#pragma unroll
                    for (int j = 0; j < TJ; ++j) bv[nx][j] = *(const half8_t *)(ws + 32 * j * GB_LD + (kk + 1) * 16);
                }
#pragma unroll
                for (int i = 0; i < TI; ++i)
#pragma unroll
                    for (int j = 0; j < TJ; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av[c][i], bv[c][j], acc[i][j], 0, 0, 0);
                if (kk + 1 < GB_K / 16) {
#pragma unroll
                    for (int r = 0; r < TI + TJ; ++r) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // 1 MFMA
                        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // 1 DS read
                    }
                }
            }
        };
        __syncthreads();                               // step 0 is in LDS
        for (int kt = 0; kt < KT; kt += 2) {            // (KT is even)
            mma(0); __syncthreads();
            mma(1); __syncthreads();
        }
    }
    // all eight wavefronts are behind the last barrier: the operand buffers are free
    gemm_tile_epilogue<TI, TJ, EMIT, ((size_t) 2 * (BN + BM) * GB_LD * sizeof(half_t) >= GELU_LDS_BYTES), 256 + NP>(acc, a, epi, db, batch_off, d_nb1, n0, m0, wn, wmo, smem);
}

// The same tile with the operands going from global memory straight into LDS (global_load_lds_dwordx4: lane l's 16 bytes
// land at the wave's LDS base + 16 l, no register and no LDS store instruction in between).  Measured on the register-staged
// loop above, a wavefront spends two thirds of a K step outside its matrix phase — issuing the global loads, whose return
// path into the registers is busy, and the LDS stores — and here both phases are gone: a step is a wait, a barrier,
// the issue of the loads NBUF - 1 steps ahead and the matrix phase.
// LDS tile of an operand: row pairs form 256-byte lines, the 16-byte chunk c of row r sits in slot (r & 1) * 8 +
// (c ^ ((r >> 1) & 7)) of line r >> 1 — the 16 lanes of a b128 fragment read (16 consecutive rows, one chunk) then cover 256
// consecutive bytes' worth of banks, and a wave's load (1 KB: 8 rows) writes whole lines from whole 128-byte row pieces.
// K a multiple of 64; operands as f16 rows (16-byte aligned).
#define DL_STEP_ROW 128     // bytes of a row in one K step

template <int N>
__device__ __forceinline__ void wait_vmcnt() {                // s_waitcnt vmcnt(N) only (gfx9 encoding: expcnt and lgkmcnt at their maxima)
    static_assert(N >= 0 && N < 64, "vmcnt has six bits");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

template <int TI, int TJ, int NBUF, bool EMIT>
__device__ __forceinline__ void gemm_f16_tile_dl(const mm_args & a, int tiles_m, int tiles_n, int sw, int tile, const char * wb, const char * xb, char * db,
                                                 const epi_args & epi, int64_t batch_off, int64_t d_nb1) {
    constexpr int BN = 64 * TI, BM = 64 * TJ;
    constexpr int XL = BN / 32, WL = BM / 32;          // 1 KB loads per wavefront and step (8 rows each)
    constexpr int STEP_BYTES = (BN + BM) * DL_STEP_ROW;
    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int per_col = sw * tiles_n, col = tile / per_col, rem = tile - col * per_col;
    const int cw = min(sw, tiles_m - col * sw);
    const int64_t m0 = (int64_t)(col * sw + rem % cw) * BM;
    const int64_t n0 = (int64_t)(rem / cw) * BN;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // load i of this wavefront covers rows 32 i + 8 wave .. + 7 of the tile; this lane: row lrow of the 8, chunk lchunk
    const int lrow = 2 * (lane >> 4) + ((lane & 15) >> 3);
    const int lchunk = (lane & 7) ^ ((4 * (wave & 1) + (lane >> 4)) & 7);
    const char * xp[XL]; const char * wp[WL];
#pragma unroll
    for (int i = 0; i < XL; ++i) { const int64_t n = n0 + 32 * i + 8 * wave + lrow; xp[i] = xb + (n < a.N ? n : a.N - 1) * a.x_nb1 + lchunk * 16; }
#pragma unroll
    for (int i = 0; i < WL; ++i) { const int64_t m = m0 + 32 * i + 8 * wave + lrow; wp[i] = wb + (m < a.M ? m : a.M - 1) * a.w_nb1 + lchunk * 16; }
    auto load = [&](int step, int buf) __attribute__((always_inline)) {
        const int64_t ko = (int64_t) step * DL_STEP_ROW;
        char * xs = smem + buf * STEP_BYTES + wave * 1024, * ws = xs + BN * DL_STEP_ROW;
#pragma unroll
        for (int i = 0; i < XL; ++i)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(xp[i] + ko), (__attribute__((address_space(3))) void *)(xs + i * 4096), 16, 0, 0);
#pragma unroll
        for (int i = 0; i < WL; ++i)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(wp[i] + ko), (__attribute__((address_space(3))) void *)(ws + i * 4096), 16, 0, 0);
    };

    const int wn = (wave >> 1) * 32 * TI, wmo = (wave & 1) * 32 * TJ;   // wave patch origin inside the tile
    const int l32 = lane & 31, g = lane >> 5;
    // fragment reads: row wn + 32 i + l32 (its line and half of the line), chunk 2 kk + g swizzled by the row
    const int rsw = (l32 >> 1) & 7;
    const int xrow = ((wn + l32) >> 1) * 256 + (l32 & 1) * 128, wrow = BN * DL_STEP_ROW + ((wmo + l32) >> 1) * 256 + (l32 & 1) * 128;
    int koff[GB_K / 16];
#pragma unroll
    for (int kk = 0; kk < GB_K / 16; ++kk) koff[kk] = ((2 * kk + g) ^ rsw) * 16;

    float16_t acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    // One K step: all fragment reads of the step go out first (they return in order, so the matrix instructions start when
    // the first sub-step's have arrived and never wait for a read issued behind them); then the loads of a later step, one
    // behind each of the first matrix instructions — a load can sit in the issue stage while the CU's vector-memory path is
    // backed up, and everything behind it waits with it: spread out, a matrix instruction is already running each time
    // (1480 clocks per step instead of 1730 with the eight loads in front); then the rest of the 4 TI TJ matrix instructions.
    auto mma = [&](int buf, int load_step, int load_buf) __attribute__((always_inline)) {
        const char * xs = smem + buf * STEP_BYTES + xrow, * ws = smem + buf * STEP_BYTES + wrow;
        half8_t av[GB_K / 16][TI], bv[GB_K / 16][TJ];
#pragma unroll
        for (int kk = 0; kk < GB_K / 16; ++kk) {
#pragma unroll
            for (int i = 0; i < TI; ++i) av[kk][i] = *(const half8_t *)(xs + i * 4096 + koff[kk]);
#pragma unroll
            for (int j = 0; j < TJ; ++j) bv[kk][j] = *(const half8_t *)(ws + j * 4096 + koff[kk]);
        }
        load(load_step, load_buf);
#pragma unroll
        for (int kk = 0; kk < GB_K / 16; ++kk)
#pragma unroll
            for (int i = 0; i < TI; ++i)
#pragma unroll
                for (int j = 0; j < TJ; ++j)
                    // (EMIT: the patch transposed — rows are m, columns n — for the epilogue that writes the Q8_0-rounded image)
                    acc[i][j] = EMIT ? __builtin_amdgcn_mfma_f32_32x32x16_f16(bv[kk][j], av[kk][i], acc[i][j], 0, 0, 0)
                                     : __builtin_amdgcn_mfma_f32_32x32x16_f16(av[kk][i], bv[kk][j], acc[i][j], 0, 0, 0);
        constexpr int n_mma = (GB_K / 16) * TI * TJ, n_ld = XL + WL;
        static_assert(n_mma >= n_ld, "a matrix instruction in front of every load");
        __builtin_amdgcn_sched_group_barrier(0x100, (GB_K / 16) * (TI + TJ), 0);     // the DS reads
#pragma unroll
        for (int q = 0; q < n_ld; ++q) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                       // one matrix instruction,
            __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);                       // one load
        }
        __builtin_amdgcn_sched_group_barrier(0x008, n_mma - n_ld, 0);                // the remaining matrix instructions
    };

    const int KT = (int)(a.K / GB_K), last = KT - 1;
    // Every step issues its XL + WL loads unconditionally (beyond the end it re-reads the last step into a buffer nobody reads
    // again), so "all but the (NBUF - 2) (XL + WL) youngest have landed" is a constant wait.
#pragma unroll
    for (int st = 0; st < NBUF - 1; ++st) load(min(st, last), st);
    int buf = 0, fill = NBUF - 1;                      // buffer of step kt; buffer that step kt + NBUF - 1 goes into
    for (int kt = 0; kt < KT; ++kt) {
        wait_vmcnt<(NBUF - 2) * (XL + WL)>();             // this wavefront's pieces of step kt are in LDS
        __syncthreads();                                // ... everybody's are, and everybody is done reading step kt - 1
        mma(buf, min(kt + NBUF - 1, last), fill);       // ... whose buffer the loads of step kt + NBUF - 1 go into
        buf = buf + 1 == NBUF ? 0 : buf + 1; fill = fill + 1 == NBUF ? 0 : fill + 1;
    }
    wait_vmcnt<0>();                                    // the surplus loads still write LDS, which the epilogue reuses
    __syncthreads();
    gemm_tile_epilogue<TI, TJ, EMIT, true, 256, EMIT>(acc, a, epi, db, batch_off, d_nb1, n0, m0, wn, wmo, smem);
}

// Workgroups are dealt round-robin to the 8 XCDs, each with its own L2: workgroup `lin` of `total` runs on XCD lin % 8.
// Give every XCD one run of consecutive work items, so that what its workgroups read is shared inside that L2: the index
// of this workgroup's item when XCD x takes items [x q + min(x, r), ...) with q = total / 8, r = total % 8.
__device__ __forceinline__ int xcd_run_index(int lin, int total) {
    const int xcd = lin % 8, q = total / 8, r = total % 8;
    return xcd * q + (xcd < r ? xcd : r) + lin / 8;
}

// width (in m-tiles) of the columns of the tile path: a run of `run` tiles should be as square as the tiles allow
static int tile_path_width(int64_t tiles_m, int64_t tiles_n, int64_t run, int bn, int bm) {
    if (run >= tiles_m * tiles_n || tiles_n == 1) return (int) tiles_m;
    int best = (int) tiles_m; int64_t best_cost = INT64_MAX;
    for (int64_t sw = 1; sw <= tiles_m; ++sw) {
        // rows of X and of W that a run touches (one more panel for a run that starts mid-way), more when the columns are uneven
        const int64_t cost = (std::min(tiles_n, (run + sw - 1) / sw + 1)) * bn + sw * bm + (tiles_m % sw ? bm : 0);
        if (cost < best_cost) { best_cost = cost; best = (int) sw; }
    }
    return best;
}

template <int TI, int TJ, int S, bool KTAIL, bool FULL, bool EMIT>
__global__ void __launch_bounds__(256, 2) k_gemm_f16(mm_args a, int tiles_m, int tiles_n, int sw) {
    const int64_t b2 = blockIdx.y % a.ne12, b3 = blockIdx.y / a.ne12;
    gemm_f16_tile<TI, TJ, S, KTAIL, FULL, EMIT>(a, tiles_m, tiles_n, sw, xcd_run_index(blockIdx.x, tiles_m * tiles_n),
                                          a.w + (b2 / a.r2) * a.w_nb2 + (b3 / a.r3) * a.w_nb3, a.x + b2 * a.x_nb2 + b3 * a.x_nb3,
                                          a.d + b2 * a.d_nb2 + b3 * a.d_nb3, a.e, b2 * a.d_nb2 + b3 * a.d_nb3, a.d_nb1);
}

// Several products over the same src1 in one launch (the Q, K and V projections of a layer; the cross-attention K and V
// of all decoder layers): blockIdx.y picks the weights, the destination and the epilogue.  One launch of 3 x 120 or
// 64 x 120 tiles fills 256 CUs where 120 tiles at a time leave half of them idle.
#define MM_GROUP_MAX 64
struct mm_group_entry { const char * w; char * d; const float * bias; const char * residual; int64_t d_nb1; int flags; float scale; };
struct mm_group { mm_group_entry e[MM_GROUP_MAX]; };

template <int TI, int TJ, int S>
__global__ void __launch_bounds__(256, 2) k_gemm_f16_group(mm_args a, int tiles_m, int tiles_n, int sw, mm_group grp) {
    // the products' tiles form one pool, product after product, and an XCD's run may cross from one product into the next
    const int nblk = tiles_m * tiles_n;
    const int item = xcd_run_index((int)(blockIdx.x + gridDim.x * blockIdx.y), nblk * (int) gridDim.y);
    const mm_group_entry & ge = grp.e[item / nblk];
    epi_args e;
    e.flags = ge.flags; e.scale = ge.scale; e.bias = ge.bias; e.residual = ge.residual; e.gelu = a.e.gelu; e.image = nullptr;
    gemm_f16_tile<TI, TJ, S, false, true>(a, tiles_m, tiles_n, sw, item % nblk, ge.w, a.x, ge.d, e, 0, ge.d_nb1);
}

// the direct-to-LDS form of the two kernels above (K a multiple of 64)
template <int TI, int TJ, int NBUF, bool EMIT>
__global__ void __launch_bounds__(256, 2) k_gemm_f16_dl(mm_args a, int tiles_m, int tiles_n, int sw) {
    const int64_t b2 = blockIdx.y % a.ne12, b3 = blockIdx.y / a.ne12;
    gemm_f16_tile_dl<TI, TJ, NBUF, EMIT>(a, tiles_m, tiles_n, sw, xcd_run_index(blockIdx.x, tiles_m * tiles_n),
                                         a.w + (b2 / a.r2) * a.w_nb2 + (b3 / a.r3) * a.w_nb3, a.x + b2 * a.x_nb2 + b3 * a.x_nb3,
                                         a.d + b2 * a.d_nb2 + b3 * a.d_nb3, a.e, b2 * a.d_nb2 + b3 * a.d_nb3, a.d_nb1);
}
template <int TI, int TJ, int NBUF>
__global__ void __launch_bounds__(256, 2) k_gemm_f16_dl_group(mm_args a, int tiles_m, int tiles_n, int sw, mm_group grp) {
    const int nblk = tiles_m * tiles_n;
    const int item = xcd_run_index((int)(blockIdx.x + gridDim.x * blockIdx.y), nblk * (int) gridDim.y);
    const mm_group_entry & ge = grp.e[item / nblk];
    epi_args e;
    e.flags = ge.flags; e.scale = ge.scale; e.bias = ge.bias; e.residual = ge.residual; e.gelu = a.e.gelu; e.image = nullptr;
    gemm_f16_tile_dl<TI, TJ, NBUF, false>(a, tiles_m, tiles_n, sw, item % nblk, ge.w, a.x, ge.d, e, 0, ge.d_nb1);
}
// LDS buffers of K steps in flight by tile shape: 128 x 128 tiles keep two workgroups per CU (2 x 32 KB each)
template <int TI, int TJ> constexpr int dl_buffers() { return TI * TJ == 4 ? 2 : 3; }
template <int TI, int TJ> constexpr size_t dl_lds_bytes() {
    constexpr size_t ring = (size_t) dl_buffers<TI, TJ>() * 64 * (TI + TJ) * DL_STEP_ROW;
    return ring > GELU_LDS_BYTES ? ring : GELU_LDS_BYTES;        // the epilogue keeps the GELU table slice there
}

template <int TI, int TJ, bool EMIT>
static int launch_gemm_f16_dl(const mm_args & a, hipStream_t st) {
    constexpr int BN = 64 * TI, BM = 64 * TJ, NBUF = dl_buffers<TI, TJ>();
    constexpr size_t lds = dl_lds_bytes<TI, TJ>();
    static std::atomic<bool> configured[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return MI355X_ERR_HIP;
    if (!configured[dev].load(std::memory_order_acquire)) {
        if (hipFuncSetAttribute((const void *) k_gemm_f16_dl<TI, TJ, NBUF, EMIT>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds) != hipSuccess) return MI355X_ERR_HIP;
        configured[dev].store(true, std::memory_order_release);
    }
    const int64_t tm = (a.M + BM - 1) / BM, tn = (a.N + BN - 1) / BN;
    if (tm * tn > 0x7fffffff) return MI355X_ERR_UNSUPPORTED;
    dim3 grid((unsigned)(tm * tn), (unsigned)(a.ne12 * a.ne13));
    const int sw = tile_path_width(tm, tn, (tm * tn + 7) / 8, BN, BM);
    k_gemm_f16_dl<TI, TJ, NBUF, EMIT><<<grid, 256, lds, st>>>(a, (int) tm, (int) tn, sw);
    return launch_status();
}

// the two-role form (K a multiple of 64 S)
template <int TI, int TJ, int S, bool EMIT, int NP>
__global__ void __launch_bounds__(256 + NP) k_gemm_f16_rs(mm_args a, int tiles_m, int tiles_n, int sw) {
    const int64_t b2 = blockIdx.y % a.ne12, b3 = blockIdx.y / a.ne12;
    gemm_f16_tile_rs<TI, TJ, S, EMIT, NP>(a, tiles_m, tiles_n, sw, xcd_run_index(blockIdx.x, tiles_m * tiles_n),
                                      a.w + (b2 / a.r2) * a.w_nb2 + (b3 / a.r3) * a.w_nb3, a.x + b2 * a.x_nb2 + b3 * a.x_nb3,
                                      a.d + b2 * a.d_nb2 + b3 * a.d_nb3, a.e, b2 * a.d_nb2 + b3 * a.d_nb3, a.d_nb1);
}
template <int TI, int TJ> constexpr int rs_ring() { return 4; }
#define RS_NP 512       // operand threads: 512 (three 16-byte pieces each per step of a 128 x 64 tile) beat 256 by 7 %

template <int TI, int TJ, bool EMIT>
static int launch_gemm_f16_rs(const mm_args & a, hipStream_t st) {
    constexpr int BN = 64 * TI, BM = 64 * TJ, S = rs_ring<TI, TJ>();
    constexpr size_t lds = (size_t) 2 * (BN + BM) * GB_LD * sizeof(half_t);
    static std::atomic<bool> configured[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return MI355X_ERR_HIP;
    if (!configured[dev].load(std::memory_order_acquire)) {
        if (hipFuncSetAttribute((const void *) k_gemm_f16_rs<TI, TJ, S, EMIT, RS_NP>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds) != hipSuccess) return MI355X_ERR_HIP;
        configured[dev].store(true, std::memory_order_release);
    }
    const int64_t tm = (a.M + BM - 1) / BM, tn = (a.N + BN - 1) / BN;
    if (tm * tn > 0x7fffffff) return MI355X_ERR_UNSUPPORTED;
    dim3 grid((unsigned)(tm * tn), (unsigned)(a.ne12 * a.ne13));
    const int sw = tile_path_width(tm, tn, (tm * tn + 7) / 8, BN, BM);
    k_gemm_f16_rs<TI, TJ, S, EMIT, RS_NP><<<grid, 256 + RS_NP, lds, st>>>(a, (int) tm, (int) tn, sw);
    return launch_status();
}

template <int TI, int TJ, int S, bool KTAIL, bool FULL, bool EMIT = false>
static int launch_gemm_f16_k(const mm_args & a, hipStream_t st) {
    static_assert(S % 2 == 0, "the LDS buffer index is the parity of the register slot");
    constexpr int BN = 64 * TI, BM = 64 * TJ;
    constexpr size_t lds = (size_t) 2 * (BN + BM) * GB_LD * sizeof(half_t);
    static std::atomic<bool> configured[64];                         // per device: kernels may use more than the default 64 KB of LDS
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return MI355X_ERR_HIP;
    if (!configured[dev].load(std::memory_order_acquire)) {
        if (hipFuncSetAttribute((const void *) k_gemm_f16<TI, TJ, S, KTAIL, FULL, EMIT>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds) != hipSuccess) return MI355X_ERR_HIP;
        configured[dev].store(true, std::memory_order_release);
    }
    const int64_t tm = (a.M + BM - 1) / BM, tn = (a.N + BN - 1) / BN;
    if (tm * tn > 0x7fffffff) return MI355X_ERR_UNSUPPORTED;
    dim3 grid((unsigned)(tm * tn), (unsigned)(a.ne12 * a.ne13));
    const int sw = tile_path_width(tm, tn, (tm * tn + 7) / 8, BN, BM);
    k_gemm_f16<TI, TJ, S, KTAIL, FULL, EMIT><<<grid, 256, lds, st>>>(a, (int) tm, (int) tn, sw);
    return launch_status();
}
template <int TI, int TJ>
static int launch_gemm_f16(const mm_args & a, hipStream_t st) {
    static const bool staged = getenv("MI355X_GEMM_STAGED") != nullptr;        // the register-staged loop, for comparison
    // 128 x 64 tiles (one workgroup to a CU when M = 1280): two roles, 13.0 vs 14.9 us at K = 1280, 33.5 vs 39.9 us at K = 5120
    if constexpr (TI * TJ == 2) {
        if (!staged && a.K % (GB_K * rs_ring<TI, TJ>()) == 0)
            return (a.e.flags & MI355X_EPI_EMIT_F16) ? launch_gemm_f16_rs<TI, TJ, true>(a, st) : launch_gemm_f16_rs<TI, TJ, false>(a, st);
    }
    // 128 x 128 tiles only: the direct loads move about half the bytes per clock of the register path, which pays where two
    // workgroups share a CU (10 - 13 % faster) and loses on the 128 x 64 tiles that run one to a CU
    if constexpr (TI * TJ == 4) {
        if (a.K % GB_K == 0 && !staged) return (a.e.flags & MI355X_EPI_EMIT_F16) ? launch_gemm_f16_dl<TI, TJ, true>(a, st) : launch_gemm_f16_dl<TI, TJ, false>(a, st);
    }
    if (a.e.flags & MI355X_EPI_EMIT_F16) {
        if (a.K % (2 * GB_K)) return MI355X_ERR_UNSUPPORTED;
        return a.K % (4 * GB_K) == 0 ? launch_gemm_f16_k<TI, TJ, 4, false, true, true>(a, st) : launch_gemm_f16_k<TI, TJ, 2, false, true, true>(a, st);
    }
    if (a.K % GB_K) return launch_gemm_f16_k<TI, TJ, 2, true, false>(a, st);
    const int64_t kt = a.K / GB_K;
    if (kt % 4 == 0) return launch_gemm_f16_k<TI, TJ, 4, false, true>(a, st);
    if (kt % 2 == 0) return launch_gemm_f16_k<TI, TJ, 2, false, true>(a, st);
    return launch_gemm_f16_k<TI, TJ, 4, false, false>(a, st);
}

template <int TI, int TJ>
static int launch_gemm_f16_group(const mm_args & a, const mm_group & grp, int count, hipStream_t st) {
    constexpr int BN = 64 * TI, BM = 64 * TJ;
    constexpr size_t lds = (size_t) 2 * (BN + BM) * GB_LD * sizeof(half_t);
    static std::atomic<bool> configured[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return MI355X_ERR_HIP;
    if (!configured[dev].load(std::memory_order_acquire)) {
        if (hipFuncSetAttribute((const void *) k_gemm_f16_group<TI, TJ, 4>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds) != hipSuccess) return MI355X_ERR_HIP;
        configured[dev].store(true, std::memory_order_release);
    }
    const int64_t tm = (a.M + BM - 1) / BM, tn = (a.N + BN - 1) / BN;
    if (tm * tn > 0x7fffffff) return MI355X_ERR_UNSUPPORTED;
    dim3 grid((unsigned)(tm * tn), (unsigned) count);
    const int sw = tile_path_width(tm, tn, (tm * tn * count + 7) / 8, BN, BM);
    static const bool staged = getenv("MI355X_GEMM_STAGED") != nullptr;
    if constexpr (TI * TJ == 4) {
    if (!staged) {
        static std::atomic<bool> dl_configured[64];
        constexpr size_t dl_lds = dl_lds_bytes<TI, TJ>();
        if (!dl_configured[dev].load(std::memory_order_acquire)) {
            if (hipFuncSetAttribute((const void *) k_gemm_f16_dl_group<TI, TJ, dl_buffers<TI, TJ>()>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) dl_lds) != hipSuccess) return MI355X_ERR_HIP;
            dl_configured[dev].store(true, std::memory_order_release);
        }
        k_gemm_f16_dl_group<TI, TJ, dl_buffers<TI, TJ>()><<<grid, 256, dl_lds, st>>>(a, (int) tm, (int) tn, sw, grp);
        return launch_status();
    }
    }
    k_gemm_f16_group<TI, TJ, 4><<<grid, 256, lds, st>>>(a, (int) tm, (int) tn, sw, grp);
    return launch_status();
}

// tile shape: the largest whose grid still covers the 256 CUs about twice
static int launch_gemm_f16_auto(const mm_args & a, hipStream_t st) {
    const int64_t nb = a.ne12 * a.ne13;
    auto blocks = [&](int bn, int bm) { return ((a.N + bn - 1) / bn) * ((a.M + bm - 1) / bm) * nb; };
    if (blocks(128, 128) >= 384) return launch_gemm_f16<2, 2>(a, st);
    if (blocks(128, 64)  >= 192 || a.N > 64) return launch_gemm_f16<2, 1>(a, st);
    return launch_gemm_f16<1, 1>(a, st);
}

// ------------------------------------------------------------------------------------------------------
// quantized GEMV (N <= 8)
// ------------------------------------------------------------------------------------------------------

// one weight block as loaded: scale bits, (Q5_0: high bits,) quants
template <int T0> struct wraw { uint32_t d, qh, q[T0 == MI355X_TYPE_Q8_0 ? 8 : 4]; };
template <int T0>
__device__ __forceinline__ wraw<T0> load_wraw(const uint8_t * wrow, int kb) {
    wraw<T0> r;
    if constexpr (T0 == MI355X_TYPE_Q8_0) {
        const uint8_t * b = wrow + (int64_t) kb * 34;
        r.d = *(const uint16_t *) b; r.qh = 0;
        const u128a2 q0 = *(const u128a2 *)(b + 2), q1 = *(const u128a2 *)(b + 18);
        r.q[0] = q0.x; r.q[1] = q0.y; r.q[2] = q0.z; r.q[3] = q0.w; r.q[4] = q1.x; r.q[5] = q1.y; r.q[6] = q1.z; r.q[7] = q1.w;
    } else {
        const uint8_t * b = wrow + (int64_t) kb * 22;
        r.d = *(const uint16_t *) b; r.qh = *(const u32a2 *)(b + 2);
        const u128a2 qs = *(const u128a2 *)(b + 6);
        r.q[0] = qs.x; r.q[1] = qs.y; r.q[2] = qs.z; r.q[3] = qs.w;
    }
    return r;
}

// X -> Q8_0 in LDS (int32 xq[NC][K/4] | float xd[NC][K/32] | int32 xsum[NC][K/32]) by the 256 threads of a workgroup
template <int NC>
__device__ __forceinline__ void quantize_x_to_lds(const mm_args & a, int32_t * xq, float * xd, int32_t * xsum, int nbk) {
    const int64_t K = a.K;
    // --- quantize X: 8 lanes per 32-value block, round-to-nearest-even like _mm256_round_ps(_MM_ROUND_NEAREST).
    // Eight independent loads per thread are in flight before the first is consumed.
    {
        const int total = NC * nbk * 8;                         // float4 pieces
        const int k8 = nbk * 8;
        for (int base = 0; base < total; base += 256 * 8) {
            float4 v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int idx = base + u * 256 + (int) threadIdx.x;
                v[u] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (idx < total) v[u] = *(const float4 *)(a.x + (int64_t)(idx / k8) * a.x_nb1 + (int64_t)(idx % k8) * 16);
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int idx = base + u * 256 + (int) threadIdx.x;      // lanes 8i .. 8i+7 share a block
                float amax = fmaxf(fmaxf(fabsf(v[u].x), fabsf(v[u].y)), fmaxf(fabsf(v[u].z), fabsf(v[u].w)));
                amax = lanes_max<8>(amax);
                const float d  = div127(amax);
                const float id = amax != 0.0f ? 127.0f / amax : 0.0f;
                const int q0 = (int) rintf(v[u].x * id), q1 = (int) rintf(v[u].y * id), q2 = (int) rintf(v[u].z * id), q3 = (int) rintf(v[u].w * id);
                int sum = q0 + q1 + q2 + q3;
                sum = lanes_sum<8>(sum);
                if (idx < total) {
                    const int n = idx / k8, c = idx % k8;       // c: float4 piece within the row
                    xq[(int64_t) n * (K / 4) + c] = (q0 & 0xFF) | ((q1 & 0xFF) << 8) | ((q2 & 0xFF) << 16) | ((q3 & 0xFF) << 24);
                    if ((c & 7) == 0) {
                        xd[n * nbk + c / 8]   = h2f(f2h_bits(d));     // the CPU backend stores d as f16 and reads it back
                        xsum[n * nbk + c / 8] = sum;
                    }
                }
            }
        }
    }
}

// LDS: int32 xq[NC][K/4] | float xd[NC][K/32] | int32 xsum[NC][K/32]
template <int T0, int NC, int LPR>
__global__ void __launch_bounds__(256) k_gemv_q(mm_args a) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int64_t K = a.K;
    const int nbk = (int)(K / QK);
    int32_t * xq   = (int32_t *) smem;
    float *   xd   = (float *)(smem + (size_t) NC * K);
    int32_t * xsum = (int32_t *)(smem + (size_t) NC * K + (size_t) NC * nbk * 4);

    // A workgroup takes every gridDim.x-th group of 4 * (64 / LPR) rows; the activations are quantized once for all of them.
    constexpr int RPW = WAVE / LPR;                 // rows per wavefront
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = lane % LPR, r = lane / LPR;
    const int64_t n_groups = (a.M + 4 * RPW - 1) / (4 * RPW);
    int64_t group = blockIdx.x;
    int64_t row = group * (4 * RPW) + wave * RPW + r;
    bool row_ok = row < a.M;
    const uint8_t * wrow = (const uint8_t *) a.w + (row_ok ? row : 0) * a.w_nb1;

    // the epilogue operands of the lane that will store are fetched early, under the weight stream
    float e_bias = 0.0f, e_bcol[NC], e_res[NC];
#pragma unroll
    for (int n = 0; n < NC; ++n) { e_bcol[n] = 0.0f; e_res[n] = 0.0f; }
    auto fetch_epilogue = [&]() __attribute__((always_inline)) {
        if (row_ok && j == 0) {
            if (a.e.flags & MI355X_EPI_BIAS) e_bias = a.e.bias[row];
            if (a.e.flags & MI355X_EPI_BIAS_COL) {
#pragma unroll
                for (int n = 0; n < NC; ++n) e_bcol[n] = a.e.bias[n];
            }
            if (a.e.flags & MI355X_EPI_RESIDUAL) {
#pragma unroll
                for (int n = 0; n < NC; ++n) e_res[n] = *(const float *)(a.e.residual + n * a.d_nb1 + row * 4);
            }
        }
    };
    fetch_epilogue();

    // this lane's first weight block is requested before the activations are touched: the two HBM round trips of the
    // kernel (activations, weights) overlap instead of following each other
    wraw<T0> blk;
    if (row_ok && j < nbk) blk = load_wraw<T0>(wrow, j);

    quantize_x_to_lds<NC>(a, xq, xd, xsum, nbk);
    __syncthreads();

    for (;;) {
        float acc[NC];
#pragma unroll
        for (int n = 0; n < NC; ++n) acc[n] = 0.0f;
        if (row_ok) {
            for (int kb = j; kb < nbk; kb += LPR) {
                const wraw<T0> cur = blk;
                if (kb + LPR < nbk) blk = load_wraw<T0>(wrow, kb + LPR);      // next block in flight under this one's dot products
                uint32_t q[8];
                const float dw = h2f((uint16_t) cur.d);
                if constexpr (T0 == MI355X_TYPE_Q8_0) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) q[i] = cur.q[i];
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {     // unsigned 5-bit values; the -16 is applied through xsum
                        q[i]     = (cur.q[i] & 0x0F0F0F0Fu)        | spread4_to_bit4((cur.qh >> (4*i))      & 0xFu);
                        q[4 + i] = ((cur.q[i] >> 4) & 0x0F0F0F0Fu) | spread4_to_bit4((cur.qh >> (16 + 4*i)) & 0xFu);
                    }
                }
#pragma unroll
                for (int n = 0; n < NC; ++n) {
                    const int4 x0 = *(const int4 *)(xq + (int64_t) n * (K / 4) + kb * 8);
                    const int4 x1 = *(const int4 *)(xq + (int64_t) n * (K / 4) + kb * 8 + 4);
                    int s = 0;
                    s = __builtin_amdgcn_sdot4((int) q[0], x0.x, s, false);
                    s = __builtin_amdgcn_sdot4((int) q[1], x0.y, s, false);
                    s = __builtin_amdgcn_sdot4((int) q[2], x0.z, s, false);
                    s = __builtin_amdgcn_sdot4((int) q[3], x0.w, s, false);
                    s = __builtin_amdgcn_sdot4((int) q[4], x1.x, s, false);
                    s = __builtin_amdgcn_sdot4((int) q[5], x1.y, s, false);
                    s = __builtin_amdgcn_sdot4((int) q[6], x1.z, s, false);
                    s = __builtin_amdgcn_sdot4((int) q[7], x1.w, s, false);
                    if constexpr (T0 == MI355X_TYPE_Q5_0) s -= 16 * xsum[n * nbk + kb];
                    acc[n] += (float) s * (dw * xd[n * nbk + kb]);
                }
            }
        }
        // this group's results are complete in registers; request the next group's first block before reducing and storing
        const int64_t done_row = row;
        const bool done_writer = row_ok && j == 0;
        const float o_bias = e_bias;
        float o_bcol[NC], o_res[NC];
#pragma unroll
        for (int n = 0; n < NC; ++n) { o_bcol[n] = e_bcol[n]; o_res[n] = e_res[n]; }
        group += gridDim.x;
        const bool more = group < n_groups;                 // uniform
        if (more) {
            row = group * (4 * RPW) + wave * RPW + r;
            row_ok = row < a.M;
            wrow = (const uint8_t *) a.w + (row_ok ? row : 0) * a.w_nb1;
            if (row_ok && j < nbk) blk = load_wraw<T0>(wrow, j);
            fetch_epilogue();
        }
#pragma unroll
        for (int n = 0; n < NC; ++n) {
#pragma unroll
            for (int o = LPR / 2; o > 0; o >>= 1) acc[n] += __shfl_xor(acc[n], o, LPR);
        }
        if (done_writer) {
            const bool out_f16 = a.e.flags & MI355X_EPI_OUT_F16;
#pragma unroll
            for (int n = 0; n < NC; ++n) {
                float v = acc[n] + o_bias + o_bcol[n];          // at most one of the two biases is set
                if (a.e.flags & MI355X_EPI_GELU)     v  = gelu_f32(v, a.e.gelu);
                if (a.e.flags & MI355X_EPI_SCALE)    v *= a.e.scale;
                if (a.e.flags & MI355X_EPI_RESIDUAL) v += o_res[n];
                if (out_f16) *(half_t *)(a.d + n * a.d_nb1 + done_row * 2) = (half_t) v;
                else         *(float  *)(a.d + n * a.d_nb1 + done_row * 4) = v;
            }
        }
        if (!more) break;
    }
}

// Activations quantized ahead of the product, once for every product that reads them:
//   int8 xq[N][K] | float xd[N][K/32] (the f16-rounded block scales) | int32 xsum[N][K/32] (sum of a block's quants)
// One thread per four values, eight lanes per block; rounding as quantize_row_q8_0 (ggml-cpu-quants.c:808-865).
__global__ void __launch_bounds__(256) k_quantize_x_q8(const char * __restrict__ x, int64_t x_nb1, int64_t K, int64_t N, char * __restrict__ ws) {
    const int64_t k4 = K / 4, nbk = K / QK;
    const int64_t idx = (int64_t) blockIdx.x * 256 + threadIdx.x;          // K % 32 == 0: the 8 lanes of a block are in or out together
    if (idx >= N * k4) return;
    const int64_t n = idx / k4, c = idx % k4;
    const float4 v = *(const float4 *)(x + n * x_nb1 + c * 16);
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = lanes_max<8>(amax);
    const float d  = div127(amax);
    const float id = amax != 0.0f ? 127.0f / amax : 0.0f;
    const int q0 = (int) rintf(v.x * id), q1 = (int) rintf(v.y * id), q2 = (int) rintf(v.z * id), q3 = (int) rintf(v.w * id);
    int sum = q0 + q1 + q2 + q3;
    sum = lanes_sum<8>(sum);
    int32_t * xq   = (int32_t *) ws;
    float *   xd   = (float *)(ws + N * K);
    int32_t * xsum = (int32_t *)(ws + N * K + N * nbk * 4);
    xq[n * k4 + c] = (q0 & 0xFF) | ((q1 & 0xFF) << 8) | ((q2 & 0xFF) << 16) | ((q3 & 0xFF) << 24);
    if ((c & 7) == 0) {
        xd[n * nbk + c / 8]   = h2f(f2h_bits(d));          // the CPU backend stores d as f16 and reads it back
        xsum[n * nbk + c / 8] = sum;
    }
}

// The product over activations quantized ahead (a.x: the layout above, NC rows).  Lane j of a row's LPR lanes owns blocks
// j, j + LPR, ... (NB of them) of EVERY row it visits, so its slices of the activations are read once and stay in
// registers while the workgroup walks its row groups: the loop is weight loads and integer dot products only.  With
// the activations in LDS, their reads (NC x 32 bytes per 34-byte block) are what bounds the kernel, and quantizing them
// in every workgroup costs more than the product itself once K is large.
struct gemv_no_prologue {
    static constexpr bool LATE = false;
    __device__ __forceinline__ void request() {}
    __device__ __forceinline__ void request_late() {}
    __device__ __forceinline__ const char * finish(const char * x) { return x; }
};

// `prologue` has two halves: request() issues its own loads BEFORE the first weight blocks are requested (request_late(),
// if it has one, the loads that depend on those, after the first weight blocks), finish() runs
// after them and returns where the quantized activations are (the plain product: the workspace as passed; the fused
// LayerNorm first produces them in LDS).  Loads are waited for in the order they were issued, so in this order the
// LayerNorm's reductions run while the weight blocks are still on their way from HBM (vmcnt(3) in front of them, where
// the other order had vmcnt(0)); every load up to finish() is unconditional (clamped address, value masked where it is
// used), because behind a branch the compiler waits for all loads, not for a count.  Measured, the launch takes the
// same 10.3 us either way: what the LayerNorm adds to the bare product is its own dependent chain (two reductions, the
// block maxima, a barrier, the LDS round trip of the quantized rows), not a wait it shares with the weights.
template <int T0, int NC, int LPR, int NB, typename PRO = gemv_no_prologue>
__device__ __forceinline__ void gemv_qr_rows(const mm_args & a, PRO prologue = PRO()) {
    const int64_t K = a.K;
    const int nbk = (int)(K / QK);

    constexpr int RPW = WAVE / LPR;                 // rows per wavefront
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = lane % LPR, r = lane / LPR;
    const int64_t n_groups = (a.M + 4 * RPW - 1) / (4 * RPW);
    // MI355X_EPI_EMIT_Q8_0: the results are also left quantized to Q8_0 for the product that reads them next.  A Q8_0 block is
    // 32 consecutive rows, GPB groups of this kernel, so the groups are then dealt in runs (workgroup b: groups b T .. b T + T - 1,
    // T a multiple of GPB) instead of round-robin, the results of a block meet in LDS and the workgroup rounds them.
    constexpr int GPB = QK / (4 * RPW);
    const bool emit_q8 = (a.e.flags & MI355X_EPI_EMIT_Q8_0) != 0;                          // uniform
    const int64_t run = emit_q8 ? GPB * ((n_groups + (int64_t) GPB * gridDim.x - 1) / ((int64_t) GPB * gridDim.x)) : 0;
    const int64_t group_end = emit_q8 ? (n_groups < (blockIdx.x + 1) * run ? n_groups : (blockIdx.x + 1) * run) : n_groups;
    const int64_t group_step = emit_q8 ? 1 : gridDim.x;
    __shared__ float q8_rows[MI355X_GEMV_MAX_COLS][QK];
    int64_t group = emit_q8 ? blockIdx.x * run : blockIdx.x;
    const bool idle = emit_q8 && group >= group_end;    // (a grid larger than the runs need: such a workgroup walks one group without storing)
    int64_t row = group * (4 * RPW) + wave * RPW + r;
    bool row_ok = row < a.M && !idle;
    const uint8_t * wrow = (const uint8_t *) a.w + (row_ok ? row : 0) * a.w_nb1;

    // a lane whose block index lies beyond the row reads the row's last block again and counts it with a zero scale
    prologue.request();
    __builtin_amdgcn_sched_barrier(0);                  // (the scheduler would hoist the weight loads above them again)
    wraw<T0> blk[NB];
    bool blk_ok[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) blk_ok[b] = j + b * LPR < nbk;
    auto load_blocks = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int b = 0; b < NB; ++b) blk[b] = load_wraw<T0>(wrow, blk_ok[b] ? j + b * LPR : nbk - 1);
    };
    load_blocks();
    if constexpr (PRO::LATE) {                          // loads whose addresses request() fetched: behind the first weight blocks
        __builtin_amdgcn_sched_barrier(0);
        prologue.request_late();
    }

    const char * xbase = prologue.finish(a.x);
    const int32_t * xq   = (const int32_t *) xbase;
    const float *   xd   = (const float *)(xbase + (size_t) NC * K);
    const int32_t * xsum = (const int32_t *)(xbase + (size_t) NC * K + (size_t) NC * nbk * 4);
    int32_t xr[NC][NB][8];
    float   xs[NC][NB];          // scale of the block
    int32_t xo[NC][NB];          // 16 x sum of its quants (Q5_0 weights are stored with an offset of 16)
#pragma unroll
    for (int n = 0; n < NC; ++n) {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const int kb = j + b * LPR < nbk ? j + b * LPR : 0;
            const int4 x0 = *(const int4 *)(xq + (int64_t) n * (K / 4) + kb * 8), x1 = *(const int4 *)(xq + (int64_t) n * (K / 4) + kb * 8 + 4);
            xr[n][b][0] = x0.x; xr[n][b][1] = x0.y; xr[n][b][2] = x0.z; xr[n][b][3] = x0.w;
            xr[n][b][4] = x1.x; xr[n][b][5] = x1.y; xr[n][b][6] = x1.z; xr[n][b][7] = x1.w;
            xs[n][b] = xd[n * nbk + kb];
            xo[n][b] = T0 == MI355X_TYPE_Q5_0 ? 16 * xsum[n * nbk + kb] : 0;
        }
    }

    // the epilogue operands of the lane that will store are fetched early, under the weight stream
    float e_bias = 0.0f, e_bcol[NC], e_res[NC];
#pragma unroll
    for (int n = 0; n < NC; ++n) { e_bcol[n] = 0.0f; e_res[n] = 0.0f; }
    auto fetch_epilogue = [&]() __attribute__((always_inline)) {
        if (row_ok && j == 0) {
            if (a.e.flags & MI355X_EPI_BIAS) e_bias = a.e.bias[row];
            if (a.e.flags & MI355X_EPI_BIAS_COL) {
#pragma unroll
                for (int n = 0; n < NC; ++n) e_bcol[n] = a.e.bias[n];
            }
            if (a.e.flags & MI355X_EPI_RESIDUAL) {
#pragma unroll
                for (int n = 0; n < NC; ++n) e_res[n] = *(const float *)(a.e.residual + n * a.d_nb1 + row * 4);
            }
        }
    };
    fetch_epilogue();

    for (;;) {
        wraw<T0> cur[NB];
#pragma unroll
        for (int b = 0; b < NB; ++b) cur[b] = blk[b];
        const int64_t done_row = row;
        const bool done_writer = row_ok && j == 0;
        const float o_bias = e_bias;
        float o_bcol[NC], o_res[NC];
#pragma unroll
        for (int n = 0; n < NC; ++n) { o_bcol[n] = e_bcol[n]; o_res[n] = e_res[n]; }
        // the next row's blocks and epilogue operands travel while this row is worked on
        const int64_t done_group = group;
        group += group_step;
        const bool more = group < group_end;                // uniform
        if (more) {
            row = group * (4 * RPW) + wave * RPW + r;
            row_ok = row < a.M;
            wrow = (const uint8_t *) a.w + (row_ok ? row : 0) * a.w_nb1;
            load_blocks();
            fetch_epilogue();
        }

        float acc[NC];
#pragma unroll
        for (int n = 0; n < NC; ++n) acc[n] = 0.0f;
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            uint32_t q[8];
            const float dw = blk_ok[b] ? h2f((uint16_t) cur[b].d) : 0.0f;
            if constexpr (T0 == MI355X_TYPE_Q8_0) {
#pragma unroll
                for (int i = 0; i < 8; ++i) q[i] = cur[b].q[i];
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    q[i]     = (cur[b].q[i] & 0x0F0F0F0Fu)        | spread4_to_bit4((cur[b].qh >> (4*i))      & 0xFu);
                    q[4 + i] = ((cur[b].q[i] >> 4) & 0x0F0F0F0Fu) | spread4_to_bit4((cur[b].qh >> (16 + 4*i)) & 0xFu);
                }
            }
#pragma unroll
            for (int n = 0; n < NC; ++n) {
                int s = 0;
#pragma unroll
                for (int i = 0; i < 8; ++i) s = __builtin_amdgcn_sdot4((int) q[i], xr[n][b][i], s, false);
                if constexpr (T0 == MI355X_TYPE_Q5_0) s -= xo[n][b];
                acc[n] += (float) s * (dw * xs[n][b]);
            }
        }
#pragma unroll
        for (int n = 0; n < NC; ++n) acc[n] = lanes_sum<LPR>(acc[n]);
        if (done_writer) {
            const bool out_f16 = a.e.flags & MI355X_EPI_OUT_F16;
#pragma unroll
            for (int n = 0; n < NC; ++n) {
                float v = acc[n] + o_bias + o_bcol[n];          // at most one of the two biases is set
                if (a.e.flags & MI355X_EPI_GELU)     v  = gelu_f32(v, a.e.gelu);
                if (a.e.flags & MI355X_EPI_SCALE)    v *= a.e.scale;
                if (a.e.flags & MI355X_EPI_RESIDUAL) v += o_res[n];
                if (out_f16) *(half_t *)(a.d + n * a.d_nb1 + done_row * 2) = (half_t) v;
                else         *(float  *)(a.d + n * a.d_nb1 + done_row * 4) = v;
                if (emit_q8) q8_rows[n][(int)(done_group % GPB) * (4 * RPW) + wave * RPW + r] = v;
            }
        }
        if (emit_q8 && ((done_group % GPB) == GPB - 1 || !more)) {          // uniform: a block of 32 rows is complete (M % 32 == 0)
            // thread (column n, row rr of the block): rounding as quantize_row_q8_0 (ggml-cpu-quants.c:808-865), into the layout of
            // k_quantize_x_q8 for NC rows of M values
            __syncthreads();
            const int n = threadIdx.x >> 5, rr = threadIdx.x & 31;
            const float v = n < NC ? q8_rows[n][rr] : 0.0f;
            const float amax = lanes_max<32>(fabsf(v));
            const float id = amax != 0.0f ? 127.0f / amax : 0.0f;
            const int q = (int) rintf(v * id);
            const int qsum = lanes_sum<32>(q);
            if (n < NC && !idle) {
                char * img = (char *) a.e.image;
                const int64_t bi = done_group / GPB, nb2 = a.M / QK;
                ((int8_t *) img)[n * a.M + bi * QK + rr] = (int8_t) q;
                if (rr == 0) {
                    ((float *)(img + (size_t) NC * a.M))[n * nb2 + bi] = h2f(f2h_bits(div127(amax)));
                    ((int32_t *)(img + (size_t) NC * a.M + (size_t) NC * nb2 * 4))[n * nb2 + bi] = qsum;
                }
            }
            __syncthreads();
        }
        if (!more) break;
    }
}

template <int T0, int NC, int LPR, int NB>
__global__ void __launch_bounds__(256) k_gemv_qr(mm_args a) { gemv_qr_rows<T0, NC, LPR, NB>(a); }

// ------------------------------------------------------------------------------------------------------
// Q8_0 weights as tiles for the matrix cores: the product over a matrix long enough to be a stream (the vocabulary
// projection: 70 MB a decode step)
// ------------------------------------------------------------------------------------------------------
// What holds the register kernel back on that matrix is its vector work — 40 v_dot4 per block for five columns — which
// adds to the stream instead of hiding under it.  One v_mfma_i32_16x16x64_i8 takes 16 weight rows x two blocks (the B
// operand: lane (r, g) holds 16 quants of row r — block g / 2 of the pair, half g % 2) against the activations of up
// to eight columns (the A operand, in registers for the whole kernel).  The two blocks of a pair have scales of their
// own, so their sums must not mix: column n sits in A row n with the first block's quants and zeros where the second's
// would be, and in A row 8 + n the other way round.  Result row 4 g' + i then reaches lane (r, g') for the block whose
// scale that lane loads (g' / 2), and what is left per lane and pair of blocks is four conversions, four scale
// products and four f32 fused multiply-adds.  A row's blocks are therefore summed as two interleaved f32 sequences
// (even blocks, odd blocks) that are added at the end.
// Read from the block rows as ggml lays them out, that operand costs more than it saves: every load takes 16 bytes
// from each of 16 rows, at 2-byte alignment, plus a 2-byte load per lane for the scale.  So the matrix is repacked once
// into the order the instruction wants — per 16 rows and pair of blocks, 1024 bytes of quants in lane order followed by
// the 32 scales (68 bytes a row, as before) — and every load of the stream is one aligned, contiguous run of a kilobyte.

__global__ void k_q8_0_tiles_pack(const char * __restrict__ w, int64_t w_nb1, int64_t M, int ksteps, int64_t n_tiles, char * __restrict__ tiles) {
    const int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;     // (tile, step, lane)
    if (i >= n_tiles * ksteps * 64) return;
    const int lane = (int)(i & 63), r = lane & 15, g = lane >> 4;
    const int64_t ts = i >> 6, tile = ts / ksteps;
    const int step = (int)(ts % ksteps);
    const int64_t row = tile * 16 + r;
    u32x4 q = { 0, 0, 0, 0 };
    uint16_t d = 0;
    if (row < M) {                                     // rows beyond the matrix: zero quants, zero scale
        const char * b = w + row * w_nb1 + (int64_t)(2 * step + (g >> 1)) * 34;
        const u128a2 t = *(const u128a2 *)(b + 2 + 16 * (g & 1));
        q = (u32x4){ t.x, t.y, t.z, t.w };
        d = *(const uint16_t *) b;
    }
    char * o = tiles + ts * Q8T_STEP;
    *(u32x4 *)(o + lane * 16) = q;
    if ((g & 1) == 0) *(uint16_t *)(o + 1024 + ((g >> 1) * 16 + r) * 2) = d;
}

template <int KSTEPS>
static int launch_gemv_q8_0_tiles_k(const mm_args & a, hipStream_t st) {
    const int64_t n_tiles = (a.M + 15) / 16;
    const int64_t resident = 256 * 2 * 4;                 // wavefronts: two workgroups of four per CU
    const int64_t rounds = (n_tiles + resident - 1) / resident;
    const int64_t waves = (n_tiles + rounds - 1) / rounds;
    k_gemv_q8_0_tiles<KSTEPS, false><<<(unsigned)(waves / 4 > 0 ? waves / 4 : 1), 256, 0, st>>>(a, nullptr);
    return launch_status();
}
static bool q8_0_tiles_k_ok(int64_t K) { return K == 384 || K == 512 || K == 768 || K == 1024 || K == 1280; }

// several products over the same activations in one launch (a decode step's Q, K and V): blockIdx.y picks the matrix
struct gemv_group_entry { const char * w; char * d; const float * bias; const char * residual; int64_t d_nb1; int flags; float scale; };
#define GEMV_GROUP_MAX 8
struct gemv_group { gemv_group_entry e[GEMV_GROUP_MAX]; };

template <int T0, int NC, int LPR, int NB>
__global__ void __launch_bounds__(256) k_gemv_qr_group(mm_args a, gemv_group grp) {
    const gemv_group_entry & ge = grp.e[blockIdx.y];
    a.w = ge.w; a.d = ge.d; a.d_nb1 = ge.d_nb1;
    a.e.flags = ge.flags; a.e.scale = ge.scale; a.e.bias = ge.bias; a.e.residual = ge.residual;
    gemv_qr_rows<T0, NC, LPR, NB>(a);
}

// LayerNorm in front of the products, in the same launch.  A decode step's LayerNorm has five rows to work on and is
// over in the latency of a launch (7 us); here every workgroup normalizes the rows for itself while its first weight
// blocks travel — the rows in registers between the passes as in k_norm — and leaves them quantized in LDS, where the
// lanes pick up their slices.  The first workgroup also writes what a separate
// LayerNorm would have left behind: the f32 rows and the Q8_0 form in the workspace, for whatever reads them later.
struct gemv_norm_args {
    const char * src; int64_t src_nb1;
    const float * w; const float * b; float eps;
    char * dst; int64_t dst_nb1;       // f32 rows of the normalized activations
    char * ws;                         // their Q8_0 form (layout of k_quantize_x_q8)
    // EMB instances: row n of the source is not read but made here, token row tok_ids[n] (Q8_0, Q5_0 or F16) plus position row
    // pos_ids[n] (F32) as in k_get_rows_add, and the first workgroup writes it to x0
    const char * tok; int tok_type; int64_t tok_nb1, tok_ne1; const int32_t * tok_ids;
    const char * pos; int64_t pos_nb1, pos_ne1; const int32_t * pos_ids;
    char * x0;
};

// NJ > 0: the rows are exactly 256 NJ values long and both affine vectors are there (whisper's LayerNorms at 512 ... 1280):
// NJ float4s per lane instead of eight, no guard around a term, no clamped address
template <int NC, int NJ = 0, bool EMB = false>
struct gemv_norm_prologue {
    const gemv_norm_args & nm; int64_t K; char * lds;
    // wavefront w takes rows w and w + 4; both rows and the affine vectors are requested before anything is reduced, so
    // the prologue is one memory round trip long
    static constexpr int RW = (NC + 3) / 4;                 // rows per wavefront
    static constexpr int JN = NJ ? NJ : 8;                  // float4s per lane and row
    float4 v[RW][JN], ww[JN], bb[JN];
    // EMB: four values of the token row as they lie in the table (Q8_0: four quants and the block's scale; Q5_0: four bytes
    // of nibbles, the scale and the block's fifth bits; F16: two words) next to the position row's four in v, and whether
    // the row's two indices are inside their tables
    uint32_t tq[EMB ? RW : 1][EMB ? JN : 1], td[EMB ? RW : 1][EMB ? JN : 1], th[EMB ? RW : 1][EMB ? JN : 1];
    int32_t r0[RW], r1[RW];
    bool ok[RW];
    static constexpr bool LATE = EMB;

    __device__ __forceinline__ void request() {
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
        const int n4 = (int)(K / 4);
        if constexpr (EMB) {                                // the rows' indices now, the rows themselves in request_late()
#pragma unroll
            for (int rr = 0; rr < RW; ++rr) {
                const int row = wave + 4 * rr < NC ? wave + 4 * rr : NC - 1;
                r0[rr] = nm.tok_ids[row]; r1[rr] = nm.pos_ids[row];
            }
        }
        // no branch around a load: addresses are clamped into the rows, and a missing affine vector reads the source instead
        const float4 * wp = (const float4 *)(NJ || nm.w ? (const char *) nm.w : nm.src), * bp = (const float4 *)(NJ || nm.b ? (const char *) nm.b : nm.src);
#pragma unroll
        for (int jj = 0; jj < JN; ++jj) {
            const int c = NJ || lane + jj * WAVE < n4 ? lane + jj * WAVE : n4 - 1;
            ww[jj] = wp[c]; bb[jj] = bp[c];
            if constexpr (!EMB) {
#pragma unroll
                for (int rr = 0; rr < RW; ++rr) {
                    const int row = wave + 4 * rr < NC ? wave + 4 * rr : NC - 1;
                    v[rr][jj] = ((const float4 *)(nm.src + row * nm.src_nb1))[c];
                }
            }
        }
    }

    __device__ __forceinline__ void request_late() {
        if constexpr (EMB) {
            const int lane = threadIdx.x & 63;
            const int n4 = (int)(K / 4);
#pragma unroll
            for (int rr = 0; rr < RW; ++rr) {
                ok[rr] = r0[rr] >= 0 && r0[rr] < nm.tok_ne1 && r1[rr] >= 0 && r1[rr] < nm.pos_ne1;
                const uint8_t * tp = (const uint8_t *) nm.tok + (int64_t)(ok[rr] ? r0[rr] : 0) * nm.tok_nb1;
                const float4 *  pp = (const float4 *)(nm.pos + (int64_t)(ok[rr] ? r1[rr] : 0) * nm.pos_nb1);
#pragma unroll
                for (int jj = 0; jj < JN; ++jj) {
                    const int c = NJ || lane + jj * WAVE < n4 ? lane + jj * WAVE : n4 - 1;
                    v[rr][jj] = pp[c];
                    if (nm.tok_type == MI355X_TYPE_Q8_0) {          // uniform
                        const uint8_t * blk = tp + (c >> 3) * 34;
                        td[rr][jj] = ld_u16(blk); tq[rr][jj] = *(const u32a2 *)(blk + 2 + 4 * (c & 7));
                    } else if (nm.tok_type == MI355X_TYPE_Q5_0) {   // (weights j and j + 16 of a block share a byte)
                        const uint8_t * blk = tp + (c >> 3) * 22;
                        td[rr][jj] = ld_u16(blk); th[rr][jj] = *(const u32a2 *)(blk + 2); tq[rr][jj] = *(const u32a2 *)(blk + 6 + 4 * (c & 3));
                    } else {
                        const uint2 h = ((const uint2 *) tp)[c];
                        tq[rr][jj] = h.x; td[rr][jj] = h.y;
                    }
                }
            }
        }
    }

    __device__ __forceinline__ const char * finish(const char *) {
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
        const int n4 = (int)(K / 4), nbk = (int)(K / QK);
        const bool writer = blockIdx.x == 0 && blockIdx.y == 0;
        int32_t * xq   = (int32_t *) lds;
        float *   xd   = (float *)(lds + (size_t) NC * K);
        int32_t * xsum = (int32_t *)(lds + (size_t) NC * nbk * 4 + (size_t) NC * K);
#pragma unroll
        for (int rr = 0; rr < RW; ++rr) {
            const int row = wave + 4 * rr;
            if (row >= NC) break;                           // uniform
            if constexpr (EMB) {                            // the source row: dequantized token values plus position values
#pragma unroll
                for (int jj = 0; jj < JN; ++jj) {
                    float4 e;
                    const uint32_t q = tq[rr][jj], d = td[rr][jj];
                    if (nm.tok_type == MI355X_TYPE_Q8_0) {
                        const float sc = h2f((uint16_t) d);
                        e.x = (float)(int8_t) q * sc;         e.y = (float)(int8_t)(q >> 8) * sc;
                        e.z = (float)(int8_t)(q >> 16) * sc;  e.w = (float)(int8_t)(q >> 24) * sc;
                    } else if (nm.tok_type == MI355X_TYPE_Q5_0) {
                        const float sc = h2f((uint16_t) d);
                        const int c = NJ || lane + jj * WAVE < n4 ? lane + jj * WAVE : n4 - 1;
                        const int j0 = 4 * (c & 7);                                     // first of the lane's four weights in the block
                        const uint32_t nib = (j0 < 16 ? q : q >> 4) & 0x0F0F0F0Fu, hb = th[rr][jj] >> j0;
                        e.x = (float)((int)((nib & 15)         | ((hb & 1) << 4))        - 16) * sc;
                        e.y = (float)((int)(((nib >> 8) & 15)  | (((hb >> 1) & 1) << 4)) - 16) * sc;
                        e.z = (float)((int)(((nib >> 16) & 15) | (((hb >> 2) & 1) << 4)) - 16) * sc;
                        e.w = (float)((int)(((nib >> 24) & 15) | (((hb >> 3) & 1) << 4)) - 16) * sc;
                    } else {
                        e.x = h2f((uint16_t) q); e.y = h2f((uint16_t)(q >> 16)); e.z = h2f((uint16_t) d); e.w = h2f((uint16_t)(d >> 16));
                    }
                    float4 & t = v[rr][jj];
                    const float nan = __builtin_nanf("");
                    t.x = ok[rr] ? e.x + t.x : nan; t.y = ok[rr] ? e.y + t.y : nan; t.z = ok[rr] ? e.z + t.z : nan; t.w = ok[rr] ? e.w + t.w : nan;
                    if (writer && (NJ || lane + jj * WAVE < n4)) ((float4 *)(nm.x0 + row * nm.src_nb1))[lane + jj * WAVE] = t;
                }
            }
            float sum = 0.0f;
#pragma unroll
            for (int jj = 0; jj < JN; ++jj) if (NJ || lane + jj * WAVE < n4) sum += (v[rr][jj].x + v[rr][jj].y) + (v[rr][jj].z + v[rr][jj].w);
            const float mean = wave_sum(sum) / (float) K;
            float sum2 = 0.0f;
#pragma unroll
            for (int jj = 0; jj < JN; ++jj) {
                if (NJ || lane + jj * WAVE < n4) {
                    float4 & t = v[rr][jj];
                    t.x -= mean; t.y -= mean; t.z -= mean; t.w -= mean;
                    sum2 += (t.x*t.x + t.y*t.y) + (t.z*t.z + t.w*t.w);
                }
            }
            const float scale = 1.0f / sqrtf(wave_sum(sum2) / (float) K + nm.eps);
            // The JN pieces of the row go through each step together — normalize, block maximum, scale, round, block sum, store —
            // and nothing between the steps branches: every piece is a chain of dependent instructions (three cross-lane steps
            // for the maximum, a division, three more for the sum), and side by side the chains fill each other's waits.  (All
            // eight lanes of a block store its scale and its sum: the same value to the same address, instead of a branch
            // around one lane's store.)
            float4 r[JN];
            float amax[JN], id[JN];
            int q[JN][4], qsum[JN];
#pragma unroll
            for (int jj = 0; jj < JN; ++jj) {
                r[jj] = make_float4(v[rr][jj].x * scale, v[rr][jj].y * scale, v[rr][jj].z * scale, v[rr][jj].w * scale);
                {   // (MUL then ADD, two graph nodes: two roundings — without guards around them the two would be contracted)
#pragma clang fp contract(off)
                    if (NJ || nm.w) { r[jj].x *= ww[jj].x; r[jj].y *= ww[jj].y; r[jj].z *= ww[jj].z; r[jj].w *= ww[jj].w; }
                    if (NJ || nm.b) { r[jj].x += bb[jj].x; r[jj].y += bb[jj].y; r[jj].z += bb[jj].z; r[jj].w += bb[jj].w; }
                }
            }
#pragma unroll
            for (int jj = 0; jj < JN; ++jj)     // (lanes beyond the row hold the clamped last piece: their groups are whole, K % 32 == 0)
                amax[jj] = lanes_max<8>(fmaxf(fmaxf(fabsf(r[jj].x), fabsf(r[jj].y)), fmaxf(fabsf(r[jj].z), fabsf(r[jj].w))));
#pragma unroll
            for (int jj = 0; jj < JN; ++jj) id[jj] = amax[jj] != 0.0f ? 127.0f / amax[jj] : 0.0f;
#pragma unroll
            for (int jj = 0; jj < JN; ++jj) {
                q[jj][0] = (int) rintf(r[jj].x * id[jj]); q[jj][1] = (int) rintf(r[jj].y * id[jj]);
                q[jj][2] = (int) rintf(r[jj].z * id[jj]); q[jj][3] = (int) rintf(r[jj].w * id[jj]);
            }
#pragma unroll
            for (int jj = 0; jj < JN; ++jj) qsum[jj] = lanes_sum<8>((q[jj][0] + q[jj][1]) + (q[jj][2] + q[jj][3]));
#pragma unroll
            for (int jj = 0; jj < JN; ++jj) {
                const int c = lane + jj * WAVE;
                if (NJ || c < n4) {
                    xq[row * n4 + c] = (q[jj][0] & 0xFF) | ((q[jj][1] & 0xFF) << 8) | ((q[jj][2] & 0xFF) << 16) | ((q[jj][3] & 0xFF) << 24);
                    xd[row * nbk + c / 8] = h2f(f2h_bits(div127(amax[jj])));
                    xsum[row * nbk + c / 8] = qsum[jj];
                }
            }
            if (writer) {
#pragma unroll
                for (int jj = 0; jj < JN; ++jj) if (NJ || lane + jj * WAVE < n4) ((float4 *)(nm.dst + row * nm.dst_nb1))[lane + jj * WAVE] = r[jj];
            }
        }
        __syncthreads();
        if (writer) {                                       // the workspace copy, 16 bytes per thread and step
            const int pieces = (int)(((size_t) NC * K + (size_t) NC * nbk * 8) / 16);
            for (int i = threadIdx.x; i < pieces; i += 256) ((u32x4 *) nm.ws)[i] = ((const u32x4 *) lds)[i];
        }
        return lds;
    }
};

template <int T0, int NC, int LPR, int NB, int NJ = 0, bool EMB = false>
__global__ void __launch_bounds__(256) k_gemv_qr_norm_group(mm_args a, gemv_group grp, gemv_norm_args nm) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const gemv_group_entry & ge = grp.e[blockIdx.y];
    a.w = ge.w; a.d = ge.d; a.d_nb1 = ge.d_nb1;
    a.e.flags = ge.flags; a.e.scale = ge.scale; a.e.bias = ge.bias; a.e.residual = ge.residual;
    gemv_qr_rows<T0, NC, LPR, NB>(a, gemv_norm_prologue<NC, NJ, EMB>{ nm, a.K, smem });
}

// the product over the tile-ordered vocabulary matrix with the decoder's last LayerNorm in front, the same way: the
// LayerNorm of the step's rows runs in every workgroup while its first tile row is on the way
template <int KSTEPS, int NC, int NJ>
__global__ void __launch_bounds__(256, 2) k_gemv_q8_0_tiles_norm(mm_args a, gemv_norm_args nm) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    gemv_q8_0_tiles_body<KSTEPS, false>(a, nullptr, gemv_norm_prologue<NC, NJ>{ nm, a.K, smem });
}

template <int KSTEPS, int NC>
static int launch_gemv_q8_0_tiles_norm_kn(const mm_args & a, const gemv_norm_args & nm, hipStream_t st) {
    const int64_t n_tiles = (a.M + 15) / 16;
    const int64_t resident = 256 * 2 * 4;                 // wavefronts: two workgroups of four per CU
    const int64_t rounds = (n_tiles + resident - 1) / resident;
    const int64_t waves = (n_tiles + rounds - 1) / rounds;
    const unsigned grid = (unsigned)(waves / 4 > 0 ? waves / 4 : 1);
    const size_t lds = (size_t) NC * a.K + (size_t) NC * (a.K / QK) * 8;
    if (KSTEPS == 20 && nm.w && nm.b) k_gemv_q8_0_tiles_norm<KSTEPS, NC, KSTEPS == 20 ? 5 : 0><<<grid, 256, lds, st>>>(a, nm);
    else                              k_gemv_q8_0_tiles_norm<KSTEPS, NC, 0><<<grid, 256, lds, st>>>(a, nm);
    return launch_status();
}
template <int KSTEPS>
static int launch_gemv_q8_0_tiles_norm_k(const mm_args & a, const gemv_norm_args & nm, hipStream_t st) {
    switch (a.N) {
        case 1: return launch_gemv_q8_0_tiles_norm_kn<KSTEPS, 1>(a, nm, st);
        case 2: return launch_gemv_q8_0_tiles_norm_kn<KSTEPS, 2>(a, nm, st);
        case 3: return launch_gemv_q8_0_tiles_norm_kn<KSTEPS, 3>(a, nm, st);
        case 4: return launch_gemv_q8_0_tiles_norm_kn<KSTEPS, 4>(a, nm, st);
        case 5: return launch_gemv_q8_0_tiles_norm_kn<KSTEPS, 5>(a, nm, st);
        case 6: return launch_gemv_q8_0_tiles_norm_kn<KSTEPS, 6>(a, nm, st);
        case 7: return launch_gemv_q8_0_tiles_norm_kn<KSTEPS, 7>(a, nm, st);
        case 8: return launch_gemv_q8_0_tiles_norm_kn<KSTEPS, 8>(a, nm, st);
    }
    return MI355X_ERR_INVALID;
}

// ------------------------------------------------------------------------------------------------------
// generic fallback: one wavefront per (m, group of up to 8 columns, batch); element-wise dequant, f32 FMA
// ------------------------------------------------------------------------------------------------------

__device__ __forceinline__ float w_elem(int type, const uint8_t * row, int64_t k) {
    switch (type) {
        case MI355X_TYPE_Q5_0: {
            const uint8_t * b = row + (k / QK) * 22; const int jj = (int)(k % QK);
            const float d = h2f(*(const uint16_t *) b);
            const uint32_t qh = *(const u32a2 *)(b + 2);
            const uint32_t qs = b[6 + (jj & 15)];
            const int nib = jj < 16 ? (qs & 0xF) : (qs >> 4);
            return (float)((nib | (((qh >> jj) & 1) << 4)) - 16) * d;
        }
        case MI355X_TYPE_Q8_0: {
            const uint8_t * b = row + (k / QK) * 34;
            return (float)((const int8_t *) b)[2 + k % QK] * h2f(*(const uint16_t *) b);
        }
        case MI355X_TYPE_F16: return (float)((const half_t *) row)[k];
        default:              return ((const float *) row)[k];
    }
}

__global__ void k_mul_mat_generic(mm_args a, int t0, int t1) {
    const int lane = threadIdx.x;
    const int64_t m  = blockIdx.x;
    const int64_t nb = (int64_t) blockIdx.y * 8;
    const int64_t b2 = blockIdx.z % a.ne12, b3 = blockIdx.z / a.ne12;
    const uint8_t * wrow = (const uint8_t *) a.w + m * a.w_nb1 + (b2 / a.r2) * a.w_nb2 + (b3 / a.r3) * a.w_nb3;
    const char * xb = a.x + b2 * a.x_nb2 + b3 * a.x_nb3;
    char * db = a.d + b2 * a.d_nb2 + b3 * a.d_nb3;
    float acc[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) acc[c] = 0.0f;
    for (int64_t k = lane; k < a.K; k += WAVE) {
        const float w = w_elem(t0, wrow, k);
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const int64_t n = nb + c;
            if (n < a.N) {
                const char * xr = xb + n * a.x_nb1;
                const float x = t1 == MI355X_TYPE_F32 ? ((const float *) xr)[k] : (float)((const half_t *) xr)[k];
                acc[c] += w * x;
            }
        }
    }
    const bool out_f16 = a.e.flags & MI355X_EPI_OUT_F16;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        const float s = wave_sum(acc[c]);
        const int64_t n = nb + c;
        if (lane == 0 && n < a.N) {
            const float v = apply_epilogue(s, a.e, m, n, (b2 * a.d_nb2 + b3 * a.d_nb3) + n * a.d_nb1 + m * 4);
            if (out_f16) *(half_t *)(db + n * a.d_nb1 + m * 2) = (half_t) v;
            else         *(float  *)(db + n * a.d_nb1 + m * 4) = v;
        }
    }
}

// ------------------------------------------------------------------------------------------------------
// host dispatch
// ------------------------------------------------------------------------------------------------------

static bool aligned16(const mi355x_tensor * t) {
    return (uintptr_t) t->data % 16 == 0 && t->nb[1] % 16 == 0 && t->nb[2] % 16 == 0 && t->nb[3] % 16 == 0;
}

// Register-resident variant: LPR = 16, 32 or 64 lanes per row with NB <= 3 blocks per lane and N * NB <= 15 block slices of
// activations (120 registers).  The fewest lanes per row that still give 512 workgroups (few lanes per row = few idle
// lanes when the blocks of a row do not divide evenly), else the most.  Returns LPR, 0 when the shape does not fit.
static int gemv_r_lanes(int64_t M, int64_t N, int64_t K) {
    const int64_t nbk = K / QK;
    int best = 0;
    for (int lpr = 64; lpr >= 16; lpr /= 2) {
        const int64_t nb = (nbk + lpr - 1) / lpr;
        if (nb > 3 || nb * N > 15) break;
        if (best == 0 || M * lpr / 256 >= 512) best = lpr;
    }
    return best;
}
// bytes of the quantized activations the register variant reads (0: the shape runs with in-kernel quantization)
static size_t gemv_ws_bytes(const mi355x_tensor * src0, const mi355x_tensor * src1) {
    const int64_t K = src0->ne[0], N = src1->ne[1];
    if (!gemv_r_lanes(src0->ne[1], N, K)) return 0;
    return round256((size_t)(N * K + N * (K / QK) * 8));
}

template <int T0, int NC, int LPR, int NB>
static int launch_gemv_r_k(const mm_args & a, unsigned grid, const gemv_group * grp, int count, const gemv_norm_args * nm, hipStream_t st) {
    if (nm) {
        const size_t lds = (size_t) NC * a.K + (size_t) NC * (a.K / QK) * 8;
        // (the widest model's rows, 1280 values, have an instance without guards)
        const bool full = a.K == 1280 && nm->w && nm->b;
        if (nm->tok) {                                      // (made for one block per lane, the shape of a layer's Q, K and V)
            if constexpr (NB == 1) {
                if (full) k_gemv_qr_norm_group<T0, NC, LPR, NB, 5, true><<<dim3(grid, (unsigned) count), 256, lds, st>>>(a, *grp, *nm);
                else      k_gemv_qr_norm_group<T0, NC, LPR, NB, 0, true><<<dim3(grid, (unsigned) count), 256, lds, st>>>(a, *grp, *nm);
            }
            else return MI355X_ERR_UNSUPPORTED;
        }
        else if (full) k_gemv_qr_norm_group<T0, NC, LPR, NB, 5><<<dim3(grid, (unsigned) count), 256, lds, st>>>(a, *grp, *nm);
        else           k_gemv_qr_norm_group<T0, NC, LPR, NB><<<dim3(grid, (unsigned) count), 256, lds, st>>>(a, *grp, *nm);
    }
    else if (grp) k_gemv_qr_group<T0, NC, LPR, NB><<<dim3(grid, (unsigned) count), 256, 0, st>>>(a, *grp);
    else          k_gemv_qr<T0, NC, LPR, NB><<<grid, 256, 0, st>>>(a);
    return launch_status();
}
template <int T0, int NC, int LPR>
static int launch_gemv_r_nb(const mm_args & a, int nb, unsigned grid, const gemv_group * grp, int count, const gemv_norm_args * nm, hipStream_t st) {
    switch (nb) {
        case 1: return launch_gemv_r_k<T0, NC, LPR, 1>(a, grid, grp, count, nm, st);
        case 2: if constexpr (NC * 2 <= 15) return launch_gemv_r_k<T0, NC, LPR, 2>(a, grid, grp, count, nm, st); break;
        case 3: if constexpr (NC * 3 <= 15) return launch_gemv_r_k<T0, NC, LPR, 3>(a, grid, grp, count, nm, st); break;
    }
    return MI355X_ERR_UNSUPPORTED;
}
template <int T0, int NC>
static int launch_gemv_r(const mm_args & a, hipStream_t st, const gemv_group * grp = nullptr, int count = 1, const gemv_norm_args * nm = nullptr) {
    int lpr = gemv_r_lanes(a.M * count, NC, a.K);
    if (!lpr) return MI355X_ERR_UNSUPPORTED;
    // with the Q8_0 emission a workgroup owns whole blocks of 32 rows, so there are M / 32 workgroups at most: the fewer lanes a
    // row takes, the fewer groups each of them walks one after the other
    const bool emit_q8 = ((grp ? grp->e[0].flags : a.e.flags) & MI355X_EPI_EMIT_Q8_0) != 0;
    if (emit_q8 && (a.K / QK + 15) / 16 <= 3 && (a.K / QK + 15) / 16 * NC <= 15) lpr = 16;
    const int nb = (int)((a.K / QK + lpr - 1) / lpr);
    const int rows_per_wg = 4 * (WAVE / lpr);
    const int64_t n_groups = (a.M + rows_per_wg - 1) / rows_per_wg;
    // one resident set of workgroups (the registers allow 4 per CU with one block per lane, else 2), each walking its
    // share of the row groups: a second, partly filled set would double the time
    const int per_cu = nb > 1 ? 2 : nm ? 3 : 4;           // (the LayerNorm prologue costs the one-block kernels 50 registers)
    const int64_t resident = 256 * per_cu / count > 0 ? 256 * per_cu / count : 1;
    const int64_t rounds   = (n_groups + resident - 1) / resident;
    const unsigned grid    = (unsigned)((n_groups + rounds - 1) / rounds);
    switch (lpr) {
        case 16: return launch_gemv_r_nb<T0, NC, 16>(a, nb, grid, grp, count, nm, st);
        case 32: return launch_gemv_r_nb<T0, NC, 32>(a, nb, grid, grp, count, nm, st);
        default: return launch_gemv_r_nb<T0, NC, 64>(a, nb, grid, grp, count, nm, st);
    }
}
template <int T0>
static int launch_gemv_r_n(const mm_args & a, hipStream_t st, const gemv_group * grp = nullptr, int count = 1, const gemv_norm_args * nm = nullptr) {
    switch (a.N) {
        case 1: return launch_gemv_r<T0, 1>(a, st, grp, count, nm);
        case 2: return launch_gemv_r<T0, 2>(a, st, grp, count, nm);
        case 3: return launch_gemv_r<T0, 3>(a, st, grp, count, nm);
        case 4: return launch_gemv_r<T0, 4>(a, st, grp, count, nm);
        case 5: return launch_gemv_r<T0, 5>(a, st, grp, count, nm);
        case 6: return launch_gemv_r<T0, 6>(a, st, grp, count, nm);
        case 7: return launch_gemv_r<T0, 7>(a, st, grp, count, nm);
        case 8: return launch_gemv_r<T0, 8>(a, st, grp, count, nm);
    }
    return MI355X_ERR_INVALID;
}

template <int T0, int NC>
static int launch_gemv(const mm_args & a, hipStream_t st) {
    const size_t lds = (size_t) NC * a.K + (size_t) NC * (a.K / QK) * 8;
    // lanes per row: the smallest split of a row's blocks that still yields enough workgroups to fill 256 CUs
    int lpr = 8;
    while (lpr < 64 && a.M * lpr / 256 < 512) lpr *= 2;
    const int rows_per_wg = 4 * (WAVE / lpr);
    // a workgroup walks several row groups when there are more than three per CU, so that the activations are quantized
    // fewer times; the groups are dealt out evenly
    const int64_t n_groups = (a.M + rows_per_wg - 1) / rows_per_wg;
    const int64_t rounds   = (n_groups + 767) / 768;
    const unsigned grid    = (unsigned)((n_groups + rounds - 1) / rounds);
    switch (lpr) {
        case 8:  k_gemv_q<T0, NC, 8 ><<<grid, 256, lds, st>>>(a); break;
        case 16: k_gemv_q<T0, NC, 16><<<grid, 256, lds, st>>>(a); break;
        case 32: k_gemv_q<T0, NC, 32><<<grid, 256, lds, st>>>(a); break;
        default: k_gemv_q<T0, NC, 64><<<grid, 256, lds, st>>>(a); break;
    }
    return launch_status();
}

template <int T0>
static int launch_gemv_n(const mm_args & a, hipStream_t st) {
    switch (a.N) {
        case 1: return launch_gemv<T0, 1>(a, st);
        case 2: return launch_gemv<T0, 2>(a, st);
        case 3: return launch_gemv<T0, 3>(a, st);
        case 4: return launch_gemv<T0, 4>(a, st);
        case 5: return launch_gemv<T0, 5>(a, st);
        case 6: return launch_gemv<T0, 6>(a, st);
        case 7: return launch_gemv<T0, 7>(a, st);
        case 8: return launch_gemv<T0, 8>(a, st);
    }
    return MI355X_ERR_INVALID;
}

enum { MM_GENERIC = 0, MM_GEMV = 1, MM_GEMM = 2 };

// which kernel a (src0, src1) pair runs on; depends on types, column count and alignment only
static int mm_path(const mi355x_tensor * src0, const mi355x_tensor * src1) {
    const int t0 = src0->type, t1 = src1->type;
    const int64_t K = src0->ne[0], N = src1->ne[1];
    const int64_t nbatch = src1->ne[2] * src1->ne[3];
    const bool quant = blck_size(t0) > 1;
    const bool w_al2 = (uintptr_t) src0->data % 2 == 0 && src0->nb[1] % 2 == 0 && src0->nb[2] % 2 == 0 && src0->nb[3] % 2 == 0;

    // GEMV: few columns, quantized weights, plain 2-d problem, activations fit the LDS staging area
    if (quant && N <= MI355X_GEMV_MAX_COLS && nbatch == 1 && t1 == MI355X_TYPE_F32 && aligned16(src1) && w_al2 &&
        (size_t) N * K + (size_t) N * (K / QK) * 8 <= 64 * 1024) {
        return MM_GEMV;
    }
    bool fast = N > MI355X_GEMV_MAX_COLS || !quant;
    if (N <= 2) fast = false;                         // a 64-wide tile for one or two columns is mostly padding
    fast = fast && aligned16(src1) && K % 8 == 0;
    if (quant)                 fast = fast && w_al2;
    else if (t0 == MI355X_TYPE_F16) fast = fast && aligned16(src0);
    else                       fast = fast && aligned16(src0) && K % QK == 0;
    return fast ? MM_GEMM : MM_GENERIC;
}

extern "C" const char * mi355x_mul_mat_kernel_name(const mi355x_tensor * src0, const mi355x_tensor * src1) {
    if (!src0 || !src1) return "mul_mat.invalid";
    const int path = mm_path(src0, src1);
    switch (src0->type) {
        case MI355X_TYPE_Q5_0: return path == MM_GEMV ? "mul_mat.gemv_q5_0" : path == MM_GEMM ? "mul_mat.gemm_q5_0" : "mul_mat.generic_q5_0";
        case MI355X_TYPE_Q8_0: return path == MM_GEMV ? "mul_mat.gemv_q8_0" : path == MM_GEMM ? "mul_mat.gemm_q8_0" : "mul_mat.generic_q8_0";
        case MI355X_TYPE_F16:  return path == MM_GEMM ? "mul_mat.gemm_f16" : "mul_mat.generic_f16";
        default:               return path == MM_GEMM ? "mul_mat.gemm_f32" : "mul_mat.generic_f32";
    }
}

// workspace of the GEMM path: f16 image of src1 (when src1 is F32), then f16 image of src0 (when src0 is not F16), each
// batch slice rounded up to 256 bytes
static size_t x16_bytes(const mi355x_tensor * src1) {
    return src1->type == MI355X_TYPE_F32 ? round256((size_t) src1->ne[0] * src1->ne[1] * 2) * (size_t)(src1->ne[2] * src1->ne[3]) : 0;
}
static size_t w16_bytes(const mi355x_tensor * src0) {
    return src0->type != MI355X_TYPE_F16 ? round256((size_t) src0->ne[0] * src0->ne[1] * 2) * (size_t)(src0->ne[2] * src0->ne[3]) : 0;
}
extern "C" size_t mi355x_mul_mat_workspace_size(const mi355x_tensor * src0, const mi355x_tensor * src1) {
    if (!src0 || !src1) return 0;
    const int path = mm_path(src0, src1);
    if (path == MM_GEMV) return gemv_ws_bytes(src0, src1);
    if (path != MM_GEMM) return 0;
    return x16_bytes(src1) + w16_bytes(src0);
}

// the few-column form of mi355x_mul_mat_group: quantized weights of one type and shape, activations quantized once
static int mul_mat_group_gemv(const mi355x_mul_mat_item * items, int count, const mi355x_tensor * src1, int flags,
                              void * workspace, size_t workspace_size, void * stream, gemv_norm_args * nm = nullptr) {
    const mi355x_tensor * w0 = items[0].src0;
    if (count > GEMV_GROUP_MAX || src1->type != MI355X_TYPE_F32 || mm_path(w0, src1) != MM_GEMV) return MI355X_ERR_UNSUPPORTED;
    if (w0->type != MI355X_TYPE_Q8_0 && w0->type != MI355X_TYPE_Q5_0) return MI355X_ERR_UNSUPPORTED;
    mm_args a;
    a.K = w0->ne[0]; a.M = w0->ne[1]; a.N = src1->ne[1];
    if (src1->ne[0] != a.K || a.K % QK != 0) return MI355X_ERR_INVALID;
    if (a.M == 0 || a.N == 0) return MI355X_OK;
    const size_t need = gemv_ws_bytes(w0, src1);
    if (!need || !gemv_r_lanes(a.M * count, a.N, a.K)) return MI355X_ERR_UNSUPPORTED;
    if (!workspace || workspace_size < need || (uintptr_t) workspace % 16 != 0) return MI355X_ERR_WORKSPACE;
    gemv_group grp;
    bool any_gelu = false;
    for (int i = 0; i < count; ++i) {
        const mi355x_tensor * w = items[i].src0, * d = items[i].dst;
        const mi355x_epilogue * e = items[i].epi;
        if (!w || !d) return MI355X_ERR_INVALID;
        if (w->type != w0->type || w->ne[0] != a.K || w->ne[1] != a.M || w->ne[2] != 1 || w->ne[3] != 1 || w->nb[1] != w0->nb[1] || (uintptr_t) w->data % 2 != 0) return MI355X_ERR_UNSUPPORTED;
        if (e && (e->flags & MI355X_EPI_EMIT_F16)) return MI355X_ERR_UNSUPPORTED;
        int ef = e ? (e->flags & 63) : 0;
        const int td = (ef & MI355X_EPI_OUT_F16) ? MI355X_TYPE_F16 : MI355X_TYPE_F32;
        if (d->type != td || d->ne[0] != a.M || d->ne[1] != a.N || d->ne[2] != 1 || d->ne[3] != 1 || d->nb[0] != type_size(td)) return MI355X_ERR_UNSUPPORTED;
        if ((ef & (MI355X_EPI_BIAS | MI355X_EPI_BIAS_COL)) && !e->bias) return MI355X_ERR_INVALID;
        if ((ef & MI355X_EPI_BIAS) && (ef & MI355X_EPI_BIAS_COL)) return MI355X_ERR_INVALID;
        if ((ef & MI355X_EPI_RESIDUAL) && (!e->residual || (ef & MI355X_EPI_OUT_F16))) return MI355X_ERR_INVALID;
        if (e && (e->flags & MI355X_EPI_EMIT_Q8_0)) {           // the result also as Q8_0: one product per launch, whole blocks
            if (count != 1 || (ef & MI355X_EPI_OUT_F16) || a.M % QK != 0) return MI355X_ERR_UNSUPPORTED;
            if (!e->image || (uintptr_t) e->image % 16 != 0) return MI355X_ERR_INVALID;
            ef |= MI355X_EPI_EMIT_Q8_0;
        }
        any_gelu = any_gelu || (ef & MI355X_EPI_GELU);
        grp.e[i] = { (const char *) w->data, (char *) d->data, e ? (const float *) e->bias : nullptr, e ? (const char *) e->residual : nullptr, (int64_t) d->nb[1], ef, e ? e->scale : 1.0f };
    }
    a.w = (const char *) w0->data; a.x = (const char *) src1->data; a.d = (char *) items[0].dst->data;
    a.w_nb1 = w0->nb[1]; a.w_nb2 = a.w_nb3 = 0;
    a.x_nb1 = src1->nb[1]; a.x_nb2 = a.x_nb3 = 0;
    a.d_nb1 = items[0].dst->nb[1]; a.d_nb2 = a.d_nb3 = 0;
    a.ne12 = a.ne13 = a.r2 = a.r3 = 1;
    a.e.flags = 0; a.e.scale = 1.0f; a.e.bias = nullptr; a.e.residual = nullptr; a.e.gelu = nullptr;
    a.e.image = (grp.e[0].flags & MI355X_EPI_EMIT_Q8_0) ? (half_t *) items[0].epi->image : nullptr;
    if (any_gelu && !(a.e.gelu = gelu_table_device())) return MI355X_ERR_HIP;
    hipStream_t st = (hipStream_t) stream;
    if (nm) {                                               // the LayerNorm in front, in the same launch: it writes src1 and the workspace
        nm->ws = (char *) workspace;
        return w0->type == MI355X_TYPE_Q8_0 ? launch_gemv_r_n<MI355X_TYPE_Q8_0>(a, st, &grp, count, nm) : launch_gemv_r_n<MI355X_TYPE_Q5_0>(a, st, &grp, count, nm);
    }
    if (!(flags & MI355X_MM_WS_READY)) {
        k_quantize_x_q8<<<(unsigned)((a.N * (a.K / 4) + 255) / 256), 256, 0, st>>>(a.x, a.x_nb1, a.K, a.N, (char *) workspace);
        if (const int rc = launch_status()) return rc;
    }
    if (flags & MI355X_MM_PREPARE_ONLY) return MI355X_OK;
    a.x = (const char *) workspace;
    return w0->type == MI355X_TYPE_Q8_0 ? launch_gemv_r_n<MI355X_TYPE_Q8_0>(a, st, &grp, count) : launch_gemv_r_n<MI355X_TYPE_Q5_0>(a, st, &grp, count);
}

// the checks common to the LayerNorm-and-products entries; `nm` arrives with the gather fields set or zero
static int norm_mul_mat_group(const mi355x_tensor * src, const mi355x_tensor * normed, float eps, const float * w, const float * b,
                              const mi355x_mul_mat_item * items, int count, void * workspace, size_t workspace_size, void * stream, gemv_norm_args nm) {
    if (!src || !normed || !items || count < 1 || !(eps >= 0.0f)) return MI355X_ERR_INVALID;
    if (!items[0].src0 || !items[0].dst) return MI355X_ERR_INVALID;
    if (src->type != MI355X_TYPE_F32 || normed->type != MI355X_TYPE_F32 || src->nb[0] != 4 || normed->nb[0] != 4) return MI355X_ERR_UNSUPPORTED;
    for (int i = 0; i < 4; ++i) if (src->ne[i] != normed->ne[i]) return MI355X_ERR_INVALID;
    const int64_t K = src->ne[0], N = src->ne[1];
    if (src->ne[2] != 1 || src->ne[3] != 1 || N < 1 || N > MI355X_GEMV_MAX_COLS || K % QK != 0 || K > 2048) return MI355X_ERR_UNSUPPORTED;
    if (!aligned16(src) || !aligned16(normed) || (uintptr_t) w % 16 != 0 || (uintptr_t) b % 16 != 0) return MI355X_ERR_UNSUPPORTED;
    if (blck_size(items[0].src0->type) <= 1) return MI355X_ERR_UNSUPPORTED;
    nm.src = (const char *) src->data; nm.src_nb1 = (int64_t) src->nb[1]; nm.w = w; nm.b = b; nm.eps = eps;
    nm.dst = (char *) normed->data; nm.dst_nb1 = (int64_t) normed->nb[1]; nm.ws = nullptr;
    return mul_mat_group_gemv(items, count, normed, 0, workspace, workspace_size, stream, &nm);
}

extern "C" int mi355x_norm_mul_mat_group(const mi355x_tensor * src, const mi355x_tensor * normed, float eps, const float * w, const float * b,
                                         const mi355x_mul_mat_item * items, int count, void * workspace, size_t workspace_size, void * stream) {
    return norm_mul_mat_group(src, normed, eps, w, b, items, count, workspace, workspace_size, stream, gemv_norm_args{});
}

extern "C" int mi355x_embed_norm_mul_mat_group(const mi355x_tensor * tok, const mi355x_tensor * tok_ids, const mi355x_tensor * pos, const mi355x_tensor * pos_ids,
                                               const mi355x_tensor * x0, const mi355x_tensor * normed, float eps, const float * w, const float * b,
                                               const mi355x_mul_mat_item * items, int count, void * workspace, size_t workspace_size, void * stream) {
    if (!tok || !tok_ids || !pos || !pos_ids || !x0) return MI355X_ERR_INVALID;
    if (tok_ids->type != MI355X_TYPE_I32 || pos_ids->type != MI355X_TYPE_I32 || pos->type != MI355X_TYPE_F32) return MI355X_ERR_UNSUPPORTED;
    if (tok->type != MI355X_TYPE_Q8_0 && tok->type != MI355X_TYPE_Q5_0 && tok->type != MI355X_TYPE_F16) return MI355X_ERR_UNSUPPORTED;
    const int64_t K = x0->ne[0], N = x0->ne[1];
    for (int i = 1; i < 4; ++i) if (tok_ids->ne[i] != 1 || pos_ids->ne[i] != 1) return MI355X_ERR_UNSUPPORTED;
    if (tok_ids->ne[0] != N || pos_ids->ne[0] != N || tok_ids->nb[0] != 4 || pos_ids->nb[0] != 4) return MI355X_ERR_UNSUPPORTED;
    if (tok->ne[2] != 1 || tok->ne[3] != 1 || pos->ne[2] != 1 || pos->ne[3] != 1) return MI355X_ERR_UNSUPPORTED;
    if (tok->ne[0] != K || pos->ne[0] != K || pos->nb[0] != 4 || tok->nb[0] != type_size(tok->type)) return MI355X_ERR_INVALID;
    // (a lane reads four values of a row at a time: 8 bytes of an F16 row, 16 of a position row; quantized blocks sit at even addresses)
    const uintptr_t ta = tok->type == MI355X_TYPE_F16 ? 8 : 2;
    if ((uintptr_t) tok->data % ta != 0 || tok->nb[1] % ta != 0 || (uintptr_t) pos->data % 16 != 0 || pos->nb[1] % 16 != 0 ||
        (uintptr_t) tok_ids->data % 4 != 0 || (uintptr_t) pos_ids->data % 4 != 0) return MI355X_ERR_UNSUPPORTED;
    gemv_norm_args nm{};
    nm.tok = (const char *) tok->data; nm.tok_type = tok->type; nm.tok_nb1 = (int64_t) tok->nb[1]; nm.tok_ne1 = tok->ne[1]; nm.tok_ids = (const int32_t *) tok_ids->data;
    nm.pos = (const char *) pos->data; nm.pos_nb1 = (int64_t) pos->nb[1]; nm.pos_ne1 = pos->ne[1]; nm.pos_ids = (const int32_t *) pos_ids->data;
    nm.x0 = (char *) x0->data;
    return norm_mul_mat_group(x0, normed, eps, w, b, items, count, workspace, workspace_size, stream, nm);
}

extern "C" int mi355x_mul_mat_group(const mi355x_mul_mat_item * items, int count, const mi355x_tensor * src1, int flags,
                                    void * workspace, size_t workspace_size, void * stream) {
    if (!items || !src1 || count < 1) return MI355X_ERR_INVALID;
    if (count > MM_GROUP_MAX) return MI355X_ERR_UNSUPPORTED;
    const mi355x_tensor * w0 = items[0].src0;
    if (!w0 || !items[0].dst) return MI355X_ERR_INVALID;
    if (blck_size(w0->type) > 1) return mul_mat_group_gemv(items, count, src1, flags, workspace, workspace_size, stream);
    // one shape of problem only: dense f16 weights (or weight images), 2-d, K a multiple of 256, the MFMA GEMM path
    if (w0->type != MI355X_TYPE_F16 || (src1->type != MI355X_TYPE_F32 && src1->type != MI355X_TYPE_F16)) return MI355X_ERR_UNSUPPORTED;
    if (src1->ne[2] != 1 || src1->ne[3] != 1 || w0->ne[2] != 1 || w0->ne[3] != 1) return MI355X_ERR_UNSUPPORTED;
    if (mm_path(w0, src1) != MM_GEMM || w0->ne[0] % (4 * GB_K) != 0) return MI355X_ERR_UNSUPPORTED;
    mm_args a;
    a.K = w0->ne[0]; a.M = w0->ne[1]; a.N = src1->ne[1];
    if (src1->ne[0] != a.K || w0->nb[0] != 2 || src1->nb[0] != type_size(src1->type)) return MI355X_ERR_INVALID;
    if (a.M == 0 || a.N == 0) return MI355X_OK;
    mm_group grp;
    bool any_gelu = false;
    for (int i = 0; i < count; ++i) {
        const mi355x_tensor * w = items[i].src0, * d = items[i].dst;
        const mi355x_epilogue * e = items[i].epi;
        if (!w || !d) return MI355X_ERR_INVALID;
        if (w->type != MI355X_TYPE_F16 || w->ne[0] != a.K || w->ne[1] != a.M || w->ne[2] != 1 || w->ne[3] != 1 || w->nb[0] != 2 || w->nb[1] != w0->nb[1] || !aligned16(w)) return MI355X_ERR_UNSUPPORTED;
        if (e && (e->flags & MI355X_EPI_EMIT_F16)) return MI355X_ERR_UNSUPPORTED;
        const int ef = e ? (e->flags & 63) : 0;
        const int td = (ef & MI355X_EPI_OUT_F16) ? MI355X_TYPE_F16 : MI355X_TYPE_F32;
        if (d->type != td || d->ne[0] != a.M || d->ne[1] != a.N || d->ne[2] != 1 || d->ne[3] != 1 || d->nb[0] != type_size(td) || d->nb[1] % 4 != 0) return MI355X_ERR_UNSUPPORTED;
        if ((ef & (MI355X_EPI_BIAS | MI355X_EPI_BIAS_COL)) && !e->bias) return MI355X_ERR_INVALID;
        if ((ef & MI355X_EPI_BIAS) && (ef & MI355X_EPI_BIAS_COL)) return MI355X_ERR_INVALID;
        if ((ef & MI355X_EPI_RESIDUAL) && (!e->residual || (ef & MI355X_EPI_OUT_F16))) return MI355X_ERR_INVALID;
        any_gelu = any_gelu || (ef & MI355X_EPI_GELU);
        grp.e[i] = { (const char *) w->data, (char *) d->data, e ? (const float *) e->bias : nullptr, e ? (const char *) e->residual : nullptr, (int64_t) d->nb[1], ef, e ? e->scale : 1.0f };
    }
    a.w = (const char *) w0->data; a.x = (const char *) src1->data; a.d = (char *) items[0].dst->data;
    a.w_nb1 = w0->nb[1]; a.w_nb2 = a.w_nb3 = 0;
    a.x_nb1 = src1->nb[1]; a.x_nb2 = a.x_nb3 = 0;
    a.d_nb1 = items[0].dst->nb[1]; a.d_nb2 = a.d_nb3 = 0;
    a.ne12 = a.ne13 = a.r2 = a.r3 = 1;
    a.e.flags = 0; a.e.scale = 1.0f; a.e.bias = nullptr; a.e.residual = nullptr; a.e.gelu = nullptr; a.e.image = nullptr;
    if (any_gelu && !(a.e.gelu = gelu_table_device())) return MI355X_ERR_HIP;
    hipStream_t st = (hipStream_t) stream;

    const size_t xbytes = x16_bytes(src1);
    if (xbytes) {
        if (!workspace || workspace_size < xbytes || (uintptr_t) workspace % 256 != 0) return MI355X_ERR_WORKSPACE;
        if (!(flags & MI355X_MM_WS_READY)) {
            dim3 qgrid((unsigned)((a.K / 4 * a.N + 255) / 256), 1);
            const bool q8 = (flags & MI355X_MM_ACT_Q8_0) && !(flags & MI355X_MM_EXACT_ACT);
            if (q8) k_x_to_f16<true ><<<qgrid, 256, 0, st>>>(a.x, (half_t *) workspace, a.K, a.N, a.x_nb1, 0, 1, 0, 0);
            else    k_x_to_f16<false><<<qgrid, 256, 0, st>>>(a.x, (half_t *) workspace, a.K, a.N, a.x_nb1, 0, 1, 0, 0);
        }
        a.x = (const char *) workspace; a.x_nb1 = a.K * 2;
    }
    if (flags & MI355X_MM_PREPARE_ONLY) return launch_status();
    const int64_t blocks22 = ((a.N + 127) / 128) * ((a.M + 127) / 128) * count;
    return blocks22 >= 300 ? launch_gemm_f16_group<2, 2>(a, grp, count, st) : launch_gemm_f16_group<2, 1>(a, grp, count, st);
}

extern "C" size_t mi355x_q8_0_tiles_size(int64_t K, int64_t M) {
    if (K <= 0 || M <= 0 || K % 64 != 0) return 0;
    return (size_t)((M + 15) / 16) * (size_t)(K / 64) * Q8T_STEP;
}

extern "C" int mi355x_q8_0_tiles_pack(const mi355x_tensor * src0, void * tiles, void * stream) {
    if (!src0 || !tiles) return MI355X_ERR_INVALID;
    if (src0->type != MI355X_TYPE_Q8_0 || src0->ne[2] != 1 || src0->ne[3] != 1 || src0->nb[0] != 34) return MI355X_ERR_UNSUPPORTED;
    const int64_t K = src0->ne[0], M = src0->ne[1];
    if (K <= 0 || M <= 0 || K % 64 != 0 || (uintptr_t) src0->data % 2 != 0 || src0->nb[1] % 2 != 0 || (uintptr_t) tiles % 16 != 0) return MI355X_ERR_UNSUPPORTED;
    const int64_t n_tiles = (M + 15) / 16, threads = n_tiles * (K / 64) * 64;
    if ((threads + 255) / 256 > 0x7fffffff) return MI355X_ERR_UNSUPPORTED;
    k_q8_0_tiles_pack<<<(unsigned)((threads + 255) / 256), 256, 0, (hipStream_t) stream>>>((const char *) src0->data, (int64_t) src0->nb[1], M, (int)(K / 64), n_tiles, (char *) tiles);
    return launch_status();
}

extern "C" int mi355x_mul_mat_q8_0_tiles(const void * tiles, int64_t K, int64_t M, const mi355x_tensor * src1, const mi355x_tensor * dst,
                                         int flags, void * workspace, size_t workspace_size, void * stream) {
    if (!tiles || !src1 || !dst) return MI355X_ERR_INVALID;
    if (!q8_0_tiles_k_ok(K) || M <= 0 || (uintptr_t) tiles % 16 != 0) return MI355X_ERR_UNSUPPORTED;
    if (flags & ~(MI355X_EPI_OUT_F16 | MI355X_MM_WS_READY | MI355X_MM_PREPARE_ONLY)) return MI355X_ERR_UNSUPPORTED;
    const int td = (flags & MI355X_EPI_OUT_F16) ? MI355X_TYPE_F16 : MI355X_TYPE_F32;
    const int64_t N = src1->ne[1];
    if (src1->type != MI355X_TYPE_F32 || dst->type != td || src1->nb[0] != 4 || dst->nb[0] != type_size(td)) return MI355X_ERR_UNSUPPORTED;
    if (src1->ne[0] != K || dst->ne[0] != M || dst->ne[1] != N) return MI355X_ERR_INVALID;
    if (N < 1 || N > MI355X_GEMV_MAX_COLS || src1->ne[2] != 1 || src1->ne[3] != 1 || dst->ne[2] != 1 || dst->ne[3] != 1 || !aligned16(src1)) return MI355X_ERR_UNSUPPORTED;
    const size_t need = round256((size_t)(N * K + N * (K / QK) * 8));
    if (!workspace || workspace_size < need || (uintptr_t) workspace % 16 != 0) return MI355X_ERR_WORKSPACE;
    hipStream_t st = (hipStream_t) stream;
    if (!(flags & MI355X_MM_WS_READY)) {
        k_quantize_x_q8<<<(unsigned)((N * (K / 4) + 255) / 256), 256, 0, st>>>((const char *) src1->data, (int64_t) src1->nb[1], K, N, (char *) workspace);
        if (const int rc = launch_status()) return rc;
    }
    if (flags & MI355X_MM_PREPARE_ONLY) return MI355X_OK;
    mm_args a;
    a.K = K; a.M = M; a.N = N;
    a.w = (const char *) tiles; a.x = (const char *) workspace; a.d = (char *) dst->data;
    a.w_nb1 = a.w_nb2 = a.w_nb3 = 0; a.x_nb1 = a.x_nb2 = a.x_nb3 = 0;
    a.d_nb1 = dst->nb[1]; a.d_nb2 = a.d_nb3 = 0;
    a.ne12 = a.ne13 = a.r2 = a.r3 = 1;
    a.e.flags = flags & MI355X_EPI_OUT_F16; a.e.scale = 1.0f; a.e.bias = nullptr; a.e.residual = nullptr; a.e.gelu = nullptr; a.e.image = nullptr;
    switch (K) {
        case 384:  return launch_gemv_q8_0_tiles_k<6>(a, st);
        case 512:  return launch_gemv_q8_0_tiles_k<8>(a, st);
        case 768:  return launch_gemv_q8_0_tiles_k<12>(a, st);
        case 1024: return launch_gemv_q8_0_tiles_k<16>(a, st);
        default:   return launch_gemv_q8_0_tiles_k<20>(a, st);
    }
}

extern "C" int mi355x_norm_mul_mat_q8_0_tiles(const void * tiles, int64_t K, int64_t M, const mi355x_tensor * src, const mi355x_tensor * normed,
                                              float eps, const float * w, const float * b, const mi355x_tensor * dst, int flags,
                                              void * workspace, size_t workspace_size, void * stream) {
    if (!tiles || !src || !normed || !dst || !(eps >= 0.0f)) return MI355X_ERR_INVALID;
    if (!q8_0_tiles_k_ok(K) || M <= 0 || (uintptr_t) tiles % 16 != 0) return MI355X_ERR_UNSUPPORTED;
    if (flags & ~MI355X_EPI_OUT_F16) return MI355X_ERR_UNSUPPORTED;
    const int td = (flags & MI355X_EPI_OUT_F16) ? MI355X_TYPE_F16 : MI355X_TYPE_F32;
    const int64_t N = src->ne[1];
    if (src->type != MI355X_TYPE_F32 || normed->type != MI355X_TYPE_F32 || dst->type != td || src->nb[0] != 4 || normed->nb[0] != 4 || dst->nb[0] != type_size(td)) return MI355X_ERR_UNSUPPORTED;
    for (int i = 0; i < 4; ++i) if (src->ne[i] != normed->ne[i]) return MI355X_ERR_INVALID;
    if (src->ne[0] != K || dst->ne[0] != M || dst->ne[1] != N) return MI355X_ERR_INVALID;
    if (N < 1 || N > MI355X_GEMV_MAX_COLS || src->ne[2] != 1 || src->ne[3] != 1 || dst->ne[2] != 1 || dst->ne[3] != 1) return MI355X_ERR_UNSUPPORTED;
    if (!aligned16(src) || !aligned16(normed) || (uintptr_t) w % 16 != 0 || (uintptr_t) b % 16 != 0) return MI355X_ERR_UNSUPPORTED;
    const size_t need = round256((size_t)(N * K + N * (K / QK) * 8));
    if (!workspace || workspace_size < need || (uintptr_t) workspace % 16 != 0) return MI355X_ERR_WORKSPACE;
    gemv_norm_args nm{};
    nm.src = (const char *) src->data; nm.src_nb1 = (int64_t) src->nb[1]; nm.w = w; nm.b = b; nm.eps = eps;
    nm.dst = (char *) normed->data; nm.dst_nb1 = (int64_t) normed->nb[1]; nm.ws = (char *) workspace;
    mm_args a;
    a.K = K; a.M = M; a.N = N;
    a.w = (const char *) tiles; a.x = (const char *) workspace; a.d = (char *) dst->data;
    a.w_nb1 = a.w_nb2 = a.w_nb3 = 0; a.x_nb1 = a.x_nb2 = a.x_nb3 = 0;
    a.d_nb1 = dst->nb[1]; a.d_nb2 = a.d_nb3 = 0;
    a.ne12 = a.ne13 = a.r2 = a.r3 = 1;
    a.e.flags = flags & MI355X_EPI_OUT_F16; a.e.scale = 1.0f; a.e.bias = nullptr; a.e.residual = nullptr; a.e.gelu = nullptr; a.e.image = nullptr;
    hipStream_t st = (hipStream_t) stream;
    switch (K) {
        case 384:  return launch_gemv_q8_0_tiles_norm_k<6>(a, nm, st);
        case 512:  return launch_gemv_q8_0_tiles_norm_k<8>(a, nm, st);
        case 768:  return launch_gemv_q8_0_tiles_norm_k<12>(a, nm, st);
        case 1024: return launch_gemv_q8_0_tiles_norm_k<16>(a, nm, st);
        default:   return launch_gemv_q8_0_tiles_norm_k<20>(a, nm, st);
    }
}

extern "C" int mi355x_dequantize_row_f16(int type, const void * src, void * dst, int64_t k, void * stream) {
    if (!src || !dst || k < 0 || k % QK != 0 || (uintptr_t) src % 2 != 0 || (uintptr_t) dst % 16 != 0) return MI355X_ERR_INVALID;
    if (k == 0) return MI355X_OK;
    if (k / QK > 0x7fffffff * (int64_t) 256) return MI355X_ERR_UNSUPPORTED;
    hipStream_t st = (hipStream_t) stream;
    const unsigned grid = (unsigned)((k / QK + 255) / 256);
    if      (type == MI355X_TYPE_Q5_0) k_w_to_f16<MI355X_TYPE_Q5_0><<<grid, 256, 0, st>>>((const char *) src, (half_t *) dst, k, 1, 0, 0, 1, 0, 0);
    else if (type == MI355X_TYPE_Q8_0) k_w_to_f16<MI355X_TYPE_Q8_0><<<grid, 256, 0, st>>>((const char *) src, (half_t *) dst, k, 1, 0, 0, 1, 0, 0);
    else return MI355X_ERR_UNSUPPORTED;
    return launch_status();
}

extern "C" int mi355x_mul_mat(const mi355x_tensor * src0, const mi355x_tensor * src1, const mi355x_tensor * dst,
                              const mi355x_epilogue * epi, void * workspace, size_t workspace_size, void * stream) {
    if (!src0 || !src1 || !dst) return MI355X_ERR_INVALID;
    const int t0 = src0->type, t1 = src1->type;
    if (t0 != MI355X_TYPE_Q5_0 && t0 != MI355X_TYPE_Q8_0 && t0 != MI355X_TYPE_F16 && t0 != MI355X_TYPE_F32) return MI355X_ERR_UNSUPPORTED;
    if (t1 != MI355X_TYPE_F32 && t1 != MI355X_TYPE_F16) return MI355X_ERR_UNSUPPORTED;
    const int flags = epi ? epi->flags : 0;
    const int td = (flags & MI355X_EPI_OUT_F16) ? MI355X_TYPE_F16 : MI355X_TYPE_F32;
    if (dst->type != td) return MI355X_ERR_INVALID;

    mm_args a;
    a.K = src0->ne[0]; a.M = src0->ne[1]; a.N = src1->ne[1];
    if (src1->ne[0] != a.K || dst->ne[0] != a.M || dst->ne[1] != a.N) return MI355X_ERR_INVALID;
    if (dst->ne[2] != src1->ne[2] || dst->ne[3] != src1->ne[3]) return MI355X_ERR_INVALID;
    if (src0->ne[2] <= 0 || src0->ne[3] <= 0 || src1->ne[2] % src0->ne[2] != 0 || src1->ne[3] % src0->ne[3] != 0) return MI355X_ERR_INVALID;
    if (src0->nb[0] != type_size(t0) || src1->nb[0] != type_size(t1) || dst->nb[0] != type_size(td)) return MI355X_ERR_UNSUPPORTED;
    if (blck_size(t0) > 1 && a.K % QK != 0) return MI355X_ERR_INVALID;
    if ((flags & (MI355X_EPI_BIAS | MI355X_EPI_BIAS_COL)) && !epi->bias) return MI355X_ERR_INVALID;
    if ((flags & MI355X_EPI_BIAS) && (flags & MI355X_EPI_BIAS_COL)) return MI355X_ERR_INVALID;      // there is one bias pointer
    if ((flags & MI355X_EPI_RESIDUAL) && !epi->residual) return MI355X_ERR_INVALID;
    if ((flags & MI355X_EPI_RESIDUAL) && (flags & MI355X_EPI_OUT_F16)) return MI355X_ERR_UNSUPPORTED;
    if (a.M == 0 || a.N == 0 || dst->ne[2] * dst->ne[3] == 0) return MI355X_OK;
    if ((flags & MI355X_MM_PREPARE_ONLY) && mm_path(src0, src1) == MM_GENERIC) return MI355X_OK;   // nothing to prepare

    a.w = (const char *) src0->data; a.x = (const char *) src1->data; a.d = (char *) dst->data;
    a.w_nb1 = src0->nb[1]; a.w_nb2 = src0->nb[2]; a.w_nb3 = src0->nb[3];
    a.x_nb1 = src1->nb[1]; a.x_nb2 = src1->nb[2]; a.x_nb3 = src1->nb[3];
    a.d_nb1 = dst->nb[1];  a.d_nb2 = dst->nb[2];  a.d_nb3 = dst->nb[3];
    a.ne12 = src1->ne[2]; a.ne13 = src1->ne[3];
    a.r2 = src1->ne[2] / src0->ne[2]; a.r3 = src1->ne[3] / src0->ne[3];
    a.e.flags = flags; a.e.scale = epi ? epi->scale : 1.0f;
    a.e.bias = epi ? (const float *) epi->bias : nullptr;
    a.e.residual = epi ? (const char *) epi->residual : nullptr;
    a.e.gelu = nullptr;
    if ((flags & MI355X_EPI_GELU) && !(a.e.gelu = gelu_table_device())) return MI355X_ERR_HIP;
    a.e.image = epi ? (half_t *) epi->image : nullptr;
    if (flags & MI355X_EPI_EMIT_F16) {
        if (!a.e.image || (flags & MI355X_EPI_OUT_F16)) return MI355X_ERR_INVALID;
    }
    if ((flags & MI355X_EPI_IMAGE_ONLY) && !(flags & MI355X_EPI_EMIT_F16)) return MI355X_ERR_INVALID;
    if (flags & MI355X_EPI_EMIT_Q8_0) {                       // the register kernel of the few-column path only
        if (!a.e.image || (uintptr_t) a.e.image % 16 != 0 || (flags & (MI355X_EPI_OUT_F16 | MI355X_EPI_EMIT_F16))) return MI355X_ERR_INVALID;
        const size_t ws_need = gemv_ws_bytes(src0, src1);
        if (a.M % QK != 0 || mm_path(src0, src1) != MM_GEMV || !ws_need || !workspace || workspace_size < ws_need || (uintptr_t) workspace % 16 != 0) return MI355X_ERR_UNSUPPORTED;
    }
    if (flags & MI355X_EPI_EMIT_F16) {
        if (a.M % QK != 0 || dst->ne[2] * dst->ne[3] != 1 || mm_path(src0, src1) != MM_GEMM) return MI355X_ERR_UNSUPPORTED;
    }

    hipStream_t st = (hipStream_t) stream;
    const int64_t nbatch = a.ne12 * a.ne13;
    if (nbatch > 65535) return MI355X_ERR_UNSUPPORTED;

    const int path = mm_path(src0, src1);
    const bool quant = blck_size(t0) > 1;
    if (path == MM_GEMV) {
        // with a workspace: activations quantized once (skipped when the caller says they are there), then the product
        // with them in registers; without: every workgroup quantizes them into LDS for itself
        const size_t need = gemv_ws_bytes(src0, src1);
        if (need && workspace && workspace_size >= need && (uintptr_t) workspace % 16 == 0) {
            if (!(flags & MI355X_MM_WS_READY)) {
                k_quantize_x_q8<<<(unsigned)((a.N * (a.K / 4) + 255) / 256), 256, 0, st>>>(a.x, a.x_nb1, a.K, a.N, (char *) workspace);
                if (const int rc = launch_status()) return rc;
            }
            if (flags & MI355X_MM_PREPARE_ONLY) return MI355X_OK;
            mm_args g = a;
            g.x = (const char *) workspace;
            return t0 == MI355X_TYPE_Q8_0 ? launch_gemv_r_n<MI355X_TYPE_Q8_0>(g, st) : launch_gemv_r_n<MI355X_TYPE_Q5_0>(g, st);
        }
        if (flags & MI355X_MM_PREPARE_ONLY) return MI355X_OK;
        return t0 == MI355X_TYPE_Q8_0 ? launch_gemv_n<MI355X_TYPE_Q8_0>(a, st) : launch_gemv_n<MI355X_TYPE_Q5_0>(a, st);
    }
    if (path == MM_GEMM) {
        const size_t xbytes = x16_bytes(src1), wbytes = w16_bytes(src0);
        if (xbytes + wbytes > 0 && (!workspace || workspace_size < xbytes + wbytes || (uintptr_t) workspace % 256 != 0)) return MI355X_ERR_WORKSPACE;
        mm_args g = a;
        if (xbytes) {
            const int64_t slice = (int64_t) round256((size_t)(a.N * a.K * 2));
            if (!(flags & MI355X_MM_WS_READY)) {
                dim3 qgrid((unsigned)((a.K / 4 * a.N + 255) / 256), (unsigned) nbatch);
                const bool q8 = (quant || (flags & MI355X_MM_ACT_Q8_0)) && !(flags & MI355X_MM_EXACT_ACT);
                if (q8 && a.K % QK != 0) return MI355X_ERR_INVALID;
                if (q8) k_x_to_f16<true ><<<qgrid, 256, 0, st>>>(a.x, (half_t *) workspace, a.K, a.N, a.x_nb1, a.x_nb2, a.ne12, a.x_nb3, slice / 2);
                else    k_x_to_f16<false><<<qgrid, 256, 0, st>>>(a.x, (half_t *) workspace, a.K, a.N, a.x_nb1, a.x_nb2, a.ne12, a.x_nb3, slice / 2);
            }
            g.x = (const char *) workspace; g.x_nb1 = a.K * 2; g.x_nb2 = slice; g.x_nb3 = slice * a.ne12;
        }
        if (flags & MI355X_MM_PREPARE_ONLY) return launch_status();
        if (wbytes) {
            const int64_t slice = (int64_t) round256((size_t)(a.M * a.K * 2));
            half_t * w16 = (half_t *)((char *) workspace + xbytes);
            dim3 wgrid((unsigned)((a.K / QK * a.M + 255) / 256), (unsigned)(src0->ne[2] * src0->ne[3]));
            switch (t0) {
                case MI355X_TYPE_Q5_0: k_w_to_f16<MI355X_TYPE_Q5_0><<<wgrid, 256, 0, st>>>(a.w, w16, a.K, a.M, a.w_nb1, a.w_nb2, src0->ne[2], a.w_nb3, slice / 2); break;
                case MI355X_TYPE_Q8_0: k_w_to_f16<MI355X_TYPE_Q8_0><<<wgrid, 256, 0, st>>>(a.w, w16, a.K, a.M, a.w_nb1, a.w_nb2, src0->ne[2], a.w_nb3, slice / 2); break;
                default:               k_w_to_f16<MI355X_TYPE_F32 ><<<wgrid, 256, 0, st>>>(a.w, w16, a.K, a.M, a.w_nb1, a.w_nb2, src0->ne[2], a.w_nb3, slice / 2); break;
            }
            g.w = (const char *) w16; g.w_nb1 = a.K * 2; g.w_nb2 = slice; g.w_nb3 = slice * src0->ne[2];
        }
        return launch_gemm_f16_auto(g, st);
    }

    if (a.M > 0x7fffffff || (a.N + 7) / 8 > 65535) return MI355X_ERR_UNSUPPORTED;
    dim3 grid((unsigned) a.M, (unsigned)((a.N + 7) / 8), (unsigned) nbatch);
    k_mul_mat_generic<<<grid, WAVE, 0, st>>>(a, t0, t1);
    return launch_status();
}

// ------------------------------------------------------------------------------------------------------
// mi355x_mul_mat for callers that cannot allocate (code under HIP graph capture, serving loops, harnesses that forbid
// hipMalloc): the workspace is a fixed array in device memory that belongs to the library, one copy per GPU.
// ------------------------------------------------------------------------------------------------------

#define MM_SCRATCH_BYTES (32u << 20)

static __device__ __align__(256) unsigned char scratch[MM_SCRATCH_BYTES];

// The array's device address on the current device (each GPU holds its own copy at its own address), looked up once per
// device with that device current.  `scratch` itself is only a host-side handle: host code never passes it to a kernel
// or a copy, always this pointer.
static void * scratch_on_current_device() {
    static std::mutex mu;
    static void * ptr[64] = {};
    static bool   failed[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) { (void) hipGetLastError(); return nullptr; }
    std::lock_guard<std::mutex> lock(mu);
    if (ptr[dev] || failed[dev]) return ptr[dev];
    void * p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) { (void) hipGetLastError(); failed[dev] = true; return nullptr; }
    ptr[dev] = p;
    return p;
}

extern "C" int mi355x_mul_mat_noalloc(const mi355x_tensor * src0, const mi355x_tensor * src1, const mi355x_tensor * dst,
                                      const mi355x_epilogue * epi, void * stream) {
    if (!src0 || !src1 || !dst) return MI355X_ERR_INVALID;
    // the array keeps whatever the call before left in it: nothing may claim that it already holds this call's activations
    if (epi && (epi->flags & (MI355X_MM_WS_READY | MI355X_MM_PREPARE_ONLY))) return MI355X_ERR_INVALID;
    const size_t need = mi355x_mul_mat_workspace_size(src0, src1);
    if (need > MM_SCRATCH_BYTES) return MI355X_ERR_WORKSPACE;         // beyond the array: use mi355x_mul_mat with a workspace of the caller's
    void * ws = scratch_on_current_device();
    if (!ws) return MI355X_ERR_HIP;
    // every byte a kernel of this call reads from the array is written by this call's own conversion pass first, so
    // nothing needs clearing
    return mi355x_mul_mat(src0, src1, dst, epi, ws, MM_SCRATCH_BYTES, stream);
}

