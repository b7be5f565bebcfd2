// FLASH_ATTN_EXT for gfx950 (ggml_compute_forward_flash_attn_ext_f16, ggml/src/ggml-cpu/ops.cpp:6638-6851)
//   dst[:, h, n] = softmax_keys(scale * q[:, n, h] . k[:, key, h] + mask[key, n]) @ v[:, key, h]
// head size 64, q f32 (rounded to f16 first, as the CPU backend does before its f16 dot), k/v f16.
//
// The CPU backend keeps its running V accumulator in f16 and rounds it after every key (ops.cpp:6793-6807).  With
// flat attention over ~1500 keys that rounding, not the mathematics, decides the low bits of the result, so two
// accumulation orders are offered:
//
//   MI355X_FA_F16_SEQ (default)  the keys are visited in order per (query, head, d) with an f16 accumulator, exactly
//                                the reference's sequence.  The running maximum is turned into a prefix maximum, so
//                                all exp() factors (vs = exp(s - M_k), ms = exp(M_{k-1} - M_k)) are computed in
//                                parallel up front and only the one-instruction f16 fma chain stays sequential.
//       k_fattn_seq_tile   N > 8:  64 queries x 64 keys per tile, two roles: four wavefronts make the next tile's
//                                  factors (QK^T on v_mfma_f32_32x32x16_f16 from LDS-staged K) while four walk this
//                                  tile's 64 keys, 16 queries each, with v_fma_mix_f32 + v_cvt_pk_f16_f32 chains
//                                  against the LDS-staged V tile.
//       k_fattn_seq_row    N <= 8: one block per (query, head): one wavefront (lane = d) runs the chain while the
//                                  other three score, scan and stage the next 192 keys.
//   MI355X_FA_F16_PK             the same sequence with the step of the reference's builds that have f16 vector units: the
//                                factor rounded to f16, one fused f16 multiply-add per element (k_fattn_pk_tile for N > 8,
//                                k_fattn_pk_row for N <= 8).
//   MI355X_FA_F32          f32 accumulators: closer to exact arithmetic, not to the reference (whose f16 accumulator
//                          loses about 1e-4 NMSE per attention, which whole-model logits then show as several 1e-3).
//       k_fattn_mfma       N > 8:  both products on the matrix cores, online softmax, probabilities as f16 operands
//       k_fattn_vec        N <= 8: one wavefront per (query, head), keys split across lanes
#include "common.h"
#include <atomic>

#define FA_D 64
#define LOG2E_F 1.44269504088896340736f

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

struct fa_args {
    const char * q; const char * k; const char * v; const char * mask; char * d;
    int64_t N, KV, H;
    int64_t q_nb1, q_nb2, q_nb3;
    int64_t k_nb1, k_nb2, k_nb3;
    int64_t v_nb1, v_nb2, v_nb3;
    int64_t m_nb1;
    int     mask_f32;                // the mask is F32 and is rounded to f16 as it is read (k_fattn_seq_row only)
    half_t * mask_copy;              // when set (with mask_f32): head 0 also stores the rounded values here, rows of mc_nb1 bytes
    int64_t mc_nb1;
    int64_t hk_ratio, hv_ratio;      // q heads per k head / v head (broadcast)
    int64_t ne3, k_ne3_ratio, v_ne3_ratio;
    float scale;
    half_t * x16;                    // when set: also the Q8_0-rounded f16 image of dst ([N][H * 64] rows), for the product that follows
};

// ------------------------------------------------------------------------------------------------------
// f32-accumulator kernel
// ------------------------------------------------------------------------------------------------------

__global__ void __launch_bounds__(256) k_fattn_vec(fa_args a) {
    const int lane = threadIdx.x & 63;
    const int64_t wid = (int64_t) blockIdx.x * 4 + (threadIdx.x >> 6);   // (n, h, i3) flattened, n fastest
    const int64_t total = a.N * a.H * a.ne3;
    if (wid >= total) return;
    const int64_t n = wid % a.N, h = (wid / a.N) % a.H, i3 = wid / (a.N * a.H);

    const float * qp = (const float *)(a.q + n * a.q_nb1 + h * a.q_nb2 + i3 * a.q_nb3);
    const char *  kb = a.k + (h / a.hk_ratio) * a.k_nb2 + (i3 / a.k_ne3_ratio) * a.k_nb3;
    const char *  vb = a.v + (h / a.hv_ratio) * a.v_nb2 + (i3 / a.v_ne3_ratio) * a.v_nb3;
    const half_t * mp = a.mask ? (const half_t *)(a.mask + n * a.m_nb1) : nullptr;

    float q[FA_D];
#pragma unroll
    for (int d = 0; d < FA_D; d += 4) {
        const float4 t = *(const float4 *)(qp + d);
        q[d] = (float)(half_t) t.x; q[d+1] = (float)(half_t) t.y; q[d+2] = (float)(half_t) t.z; q[d+3] = (float)(half_t) t.w;
    }

    float M = -INFINITY, S = 0.0f;
    float acc[FA_D];
#pragma unroll
    for (int d = 0; d < FA_D; ++d) acc[d] = 0.0f;

    for (int64_t key = lane; key < a.KV; key += WAVE) {
        const float mv = mp ? (float) mp[key] : 0.0f;
        if (mv == -INFINITY) continue;
        const half8_t * kr = (const half8_t *)(kb + key * a.k_nb1);
        float s = 0.0f;
#pragma unroll
        for (int c = 0; c < FA_D / 8; ++c) {
            const half8_t kk = kr[c];
#pragma unroll
            for (int e = 0; e < 8; ++e) s += q[8*c + e] * (float) kk[e];
        }
        s = s * a.scale + mv;
        float ms = 1.0f, vs = 1.0f;
        if (s > M) { ms = __expf(M - s); M = s; } else { vs = __expf(s - M); }
        const half8_t * vr = (const half8_t *)(vb + key * a.v_nb1);
#pragma unroll
        for (int c = 0; c < FA_D / 8; ++c) {
            const half8_t vv = vr[c];
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[8*c + e] = acc[8*c + e] * ms + vs * (float) vv[e];
        }
        S = S * ms + vs;
    }

    // merge the 64 per-lane states
    const float Mw = wave_max(M);
    const float f  = (M == -INFINITY) ? 0.0f : __expf(M - Mw);
    const float Sw = wave_sum(S * f);
    const float inv = 1.0f / Sw;
    float out = 0.0f;
#pragma unroll
    for (int d = 0; d < FA_D; ++d) {
        const float t = wave_sum(acc[d] * f);
        if (lane == d) out = t;
    }
    float * dp = (float *) a.d + ((i3 * a.N + n) * a.H + h) * FA_D;   // dst [D, H, N, ne3] dense
    dp[lane] = out * inv;
}

// ------------------------------------------------------------------------------------------------------
// shared pieces of the f16-sequential kernels
// ------------------------------------------------------------------------------------------------------

// one key of the reference's inner loop for one accumulator element:
//   VKQ16 = f16(f32(VKQ16) * ms)            only when a new maximum arrived (ggml_vec_scale_f16)
//   VKQ16 = f16(fma(f32(v), vs, f32(VKQ16)))  (ggml_vec_mad_f16: fma in f32, stored as f16)
__device__ __forceinline__ half_t seq_scale(half_t acc, float ms) { return (half_t)((float) acc * ms); }
__device__ __forceinline__ half_t seq_mad(half_t acc, half_t v, float vs) { return (half_t) __builtin_fmaf((float) v, vs, (float) acc); }

// The same two steps on a pair of accumulators: two full-rate v_fma_mix_f32 (f16 and f32 sources, fma rounded to f32)
// and one v_cvt_pk_f16_f32 (round to nearest even) per pair — the reference's f32 fma followed by GGML_FP32_TO_FP16,
// both roundings included.  Spelled out as instructions because the compiler otherwise mixes in v_fma_mixlo/hi_f16,
// which issue at half rate on gfx950 and round the exact fma once (a last-bit difference from the reference's two steps).
__device__ __forceinline__ half2_t seq_mad2(half2_t acc, half2_t v, float vs) {
    float lo, hi;
    half2_t r;
    asm("v_fma_mix_f32 %0, %2, %3, %4 op_sel_hi:[1,0,1]\n\t"
        "v_fma_mix_f32 %1, %2, %3, %4 op_sel:[1,0,1] op_sel_hi:[1,0,1]" : "=&v"(lo), "=&v"(hi) : "v"(v), "v"(vs), "v"(acc));
    asm("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(r) : "v"(lo), "v"(hi));
    return r;
}
// One key for the 16 accumulators of a lane (eight pairs): the 16 fma first, then the 8 packs — in that order no
// instruction reads what the one or two before it wrote.  Written pair by pair (fma, fma, pack) every pack waited for the
// fma in front of it, and the compiler, which does not move instructions out of asm statements, also had to put a wait state
// between them: the chains ran at three quarters of the vector issue rate.
// va / vb: the key's V values d0 .. d0 + 7 and d0 + 8 .. d0 + 15 (two f16 per register).
__device__ __forceinline__ void seq_mad16(half2_t (&acc)[8], const u32x4 va, const u32x4 vb, float vs) {
    float t0, t1, t2, t3, t4, t5, t6, t7, t8, t9, t10, t11, t12, t13, t14, t15;
    asm("v_fma_mix_f32 %0, %8, %12, %13 op_sel_hi:[1,0,1]\n\t"
        "v_fma_mix_f32 %1, %8, %12, %13 op_sel:[1,0,1] op_sel_hi:[1,0,1]\n\t"
        "v_fma_mix_f32 %2, %9, %12, %14 op_sel_hi:[1,0,1]\n\t"
        "v_fma_mix_f32 %3, %9, %12, %14 op_sel:[1,0,1] op_sel_hi:[1,0,1]\n\t"
        "v_fma_mix_f32 %4, %10, %12, %15 op_sel_hi:[1,0,1]\n\t"
        "v_fma_mix_f32 %5, %10, %12, %15 op_sel:[1,0,1] op_sel_hi:[1,0,1]\n\t"
        "v_fma_mix_f32 %6, %11, %12, %16 op_sel_hi:[1,0,1]\n\t"
        "v_fma_mix_f32 %7, %11, %12, %16 op_sel:[1,0,1] op_sel_hi:[1,0,1]"
        : "=&v"(t0), "=&v"(t1), "=&v"(t2), "=&v"(t3), "=&v"(t4), "=&v"(t5), "=&v"(t6), "=&v"(t7)
        : "v"(va.x), "v"(va.y), "v"(va.z), "v"(va.w), "v"(vs), "v"(acc[0]), "v"(acc[1]), "v"(acc[2]), "v"(acc[3]));
    asm("v_fma_mix_f32 %0, %8, %12, %13 op_sel_hi:[1,0,1]\n\t"
        "v_fma_mix_f32 %1, %8, %12, %13 op_sel:[1,0,1] op_sel_hi:[1,0,1]\n\t"
        "v_fma_mix_f32 %2, %9, %12, %14 op_sel_hi:[1,0,1]\n\t"
        "v_fma_mix_f32 %3, %9, %12, %14 op_sel:[1,0,1] op_sel_hi:[1,0,1]\n\t"
        "v_fma_mix_f32 %4, %10, %12, %15 op_sel_hi:[1,0,1]\n\t"
        "v_fma_mix_f32 %5, %10, %12, %15 op_sel:[1,0,1] op_sel_hi:[1,0,1]\n\t"
        "v_fma_mix_f32 %6, %11, %12, %16 op_sel_hi:[1,0,1]\n\t"
        "v_fma_mix_f32 %7, %11, %12, %16 op_sel:[1,0,1] op_sel_hi:[1,0,1]"
        : "=&v"(t8), "=&v"(t9), "=&v"(t10), "=&v"(t11), "=&v"(t12), "=&v"(t13), "=&v"(t14), "=&v"(t15)
        : "v"(vb.x), "v"(vb.y), "v"(vb.z), "v"(vb.w), "v"(vs), "v"(acc[4]), "v"(acc[5]), "v"(acc[6]), "v"(acc[7]));
    asm("v_cvt_pk_f16_f32 %0, %8, %9\n\t"
        "v_cvt_pk_f16_f32 %1, %10, %11\n\t"
        "v_cvt_pk_f16_f32 %2, %12, %13\n\t"
        "v_cvt_pk_f16_f32 %3, %14, %15\n\t"
        "v_cvt_pk_f16_f32 %4, %16, %17\n\t"
        "v_cvt_pk_f16_f32 %5, %18, %19\n\t"
        "v_cvt_pk_f16_f32 %6, %20, %21\n\t"
        "v_cvt_pk_f16_f32 %7, %22, %23"
        : "=&v"(acc[0]), "=&v"(acc[1]), "=&v"(acc[2]), "=&v"(acc[3]), "=&v"(acc[4]), "=&v"(acc[5]), "=&v"(acc[6]), "=&v"(acc[7])
        : "v"(t0), "v"(t1), "v"(t2), "v"(t3), "v"(t4), "v"(t5), "v"(t6), "v"(t7), "v"(t8), "v"(t9), "v"(t10), "v"(t11), "v"(t12), "v"(t13), "v"(t14), "v"(t15));
}
// the rescale of the 16 accumulators by ms (f32 product, rounded to f16), instructions ordered like seq_mad16
__device__ __forceinline__ void seq_scale16(half2_t (&acc)[8], float ms) {
    float t0, t1, t2, t3, t4, t5, t6, t7, t8, t9, t10, t11, t12, t13, t14, t15;
    asm("v_fma_mix_f32 %0, %8, %12, 0 op_sel_hi:[1,0,0]\n\t"
        "v_fma_mix_f32 %1, %8, %12, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]\n\t"
        "v_fma_mix_f32 %2, %9, %12, 0 op_sel_hi:[1,0,0]\n\t"
        "v_fma_mix_f32 %3, %9, %12, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]\n\t"
        "v_fma_mix_f32 %4, %10, %12, 0 op_sel_hi:[1,0,0]\n\t"
        "v_fma_mix_f32 %5, %10, %12, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]\n\t"
        "v_fma_mix_f32 %6, %11, %12, 0 op_sel_hi:[1,0,0]\n\t"
        "v_fma_mix_f32 %7, %11, %12, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]"
        : "=&v"(t0), "=&v"(t1), "=&v"(t2), "=&v"(t3), "=&v"(t4), "=&v"(t5), "=&v"(t6), "=&v"(t7)
        : "v"(acc[0]), "v"(acc[1]), "v"(acc[2]), "v"(acc[3]), "v"(ms));
    asm("v_fma_mix_f32 %0, %8, %12, 0 op_sel_hi:[1,0,0]\n\t"
        "v_fma_mix_f32 %1, %8, %12, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]\n\t"
        "v_fma_mix_f32 %2, %9, %12, 0 op_sel_hi:[1,0,0]\n\t"
        "v_fma_mix_f32 %3, %9, %12, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]\n\t"
        "v_fma_mix_f32 %4, %10, %12, 0 op_sel_hi:[1,0,0]\n\t"
        "v_fma_mix_f32 %5, %10, %12, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]\n\t"
        "v_fma_mix_f32 %6, %11, %12, 0 op_sel_hi:[1,0,0]\n\t"
        "v_fma_mix_f32 %7, %11, %12, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]"
        : "=&v"(t8), "=&v"(t9), "=&v"(t10), "=&v"(t11), "=&v"(t12), "=&v"(t13), "=&v"(t14), "=&v"(t15)
        : "v"(acc[4]), "v"(acc[5]), "v"(acc[6]), "v"(acc[7]), "v"(ms));
    asm("v_cvt_pk_f16_f32 %0, %8, %9\n\t"
        "v_cvt_pk_f16_f32 %1, %10, %11\n\t"
        "v_cvt_pk_f16_f32 %2, %12, %13\n\t"
        "v_cvt_pk_f16_f32 %3, %14, %15\n\t"
        "v_cvt_pk_f16_f32 %4, %16, %17\n\t"
        "v_cvt_pk_f16_f32 %5, %18, %19\n\t"
        "v_cvt_pk_f16_f32 %6, %20, %21\n\t"
        "v_cvt_pk_f16_f32 %7, %22, %23"
        : "=&v"(acc[0]), "=&v"(acc[1]), "=&v"(acc[2]), "=&v"(acc[3]), "=&v"(acc[4]), "=&v"(acc[5]), "=&v"(acc[6]), "=&v"(acc[7])
        : "v"(t0), "v"(t1), "v"(t2), "v"(t3), "v"(t4), "v"(t5), "v"(t6), "v"(t7), "v"(t8), "v"(t9), "v"(t10), "v"(t11), "v"(t12), "v"(t13), "v"(t14), "v"(t15));
}
__device__ __forceinline__ half2_t seq_scale2(half2_t acc, float ms) {
    float lo, hi;
    half2_t r;
    asm("v_fma_mix_f32 %0, %2, %3, 0 op_sel_hi:[1,0,0]\n\t"
        "v_fma_mix_f32 %1, %2, %3, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=&v"(lo), "=&v"(hi) : "v"(acc), "v"(ms));
    asm("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(r) : "v"(lo), "v"(hi));
    return r;
}

// ---- the packed-f16 form of the same chain (MI355X_FA_F16_PK) ----
// The reference's builds with f16 vector arithmetic (Arm: GGML_F16_VEC_FMA = vfmaq_f16, GGML_F16_VEC_SET1 = vdupq_n_f16,
// ggml/src/ggml-cpu/simd-mappings.h:68-105 under vec.h:180-203 and :295-311) round the factor to f16 once per key and do
// the step as one fused f16 multiply-add per element: acc = f16(acc + v * f16(vs)), a rescale as acc = f16(acc * f16(ms)).
// The accumulator is rounded to f16 after every key as in the f32-fma form; a step differs from that form by the factor's
// rounding (2^-12 of an increment that is itself a small part of the sum) and by one rounding instead of two.  On gfx950
// that is v_pk_fma_f16, two elements per instruction.
//
// One key for a lane that owns 4 queries x 4 d: acc[2 q + j] holds d pair j of query q, v the key's two d pairs, f[q] the
// factors of two consecutive keys for query q as two f16; SEL picks the first or the second of them for both elements.
template <int SEL>
__device__ __forceinline__ void pk_mad8(half2_t (&acc)[8], const uint32_t v0, const uint32_t v1, const u32x4 f) {
    if (SEL == 0) {
        asm("v_pk_fma_f16 %0, %8, %10, %0 op_sel_hi:[1,0,1]\n\t"
            "v_pk_fma_f16 %2, %8, %11, %2 op_sel_hi:[1,0,1]\n\t"
            "v_pk_fma_f16 %4, %8, %12, %4 op_sel_hi:[1,0,1]\n\t"
            "v_pk_fma_f16 %6, %8, %13, %6 op_sel_hi:[1,0,1]\n\t"
            "v_pk_fma_f16 %1, %9, %10, %1 op_sel_hi:[1,0,1]\n\t"
            "v_pk_fma_f16 %3, %9, %11, %3 op_sel_hi:[1,0,1]\n\t"
            "v_pk_fma_f16 %5, %9, %12, %5 op_sel_hi:[1,0,1]\n\t"
            "v_pk_fma_f16 %7, %9, %13, %7 op_sel_hi:[1,0,1]"
            : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3]), "+v"(acc[4]), "+v"(acc[5]), "+v"(acc[6]), "+v"(acc[7])
            : "v"(v0), "v"(v1), "v"(f.x), "v"(f.y), "v"(f.z), "v"(f.w));
    } else {
        asm("v_pk_fma_f16 %0, %8, %10, %0 op_sel:[0,1,0] op_sel_hi:[1,1,1]\n\t"
            "v_pk_fma_f16 %2, %8, %11, %2 op_sel:[0,1,0] op_sel_hi:[1,1,1]\n\t"
            "v_pk_fma_f16 %4, %8, %12, %4 op_sel:[0,1,0] op_sel_hi:[1,1,1]\n\t"
            "v_pk_fma_f16 %6, %8, %13, %6 op_sel:[0,1,0] op_sel_hi:[1,1,1]\n\t"
            "v_pk_fma_f16 %1, %9, %10, %1 op_sel:[0,1,0] op_sel_hi:[1,1,1]\n\t"
            "v_pk_fma_f16 %3, %9, %11, %3 op_sel:[0,1,0] op_sel_hi:[1,1,1]\n\t"
            "v_pk_fma_f16 %5, %9, %12, %5 op_sel:[0,1,0] op_sel_hi:[1,1,1]\n\t"
            "v_pk_fma_f16 %7, %9, %13, %7 op_sel:[0,1,0] op_sel_hi:[1,1,1]"
            : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3]), "+v"(acc[4]), "+v"(acc[5]), "+v"(acc[6]), "+v"(acc[7])
            : "v"(v0), "v"(v1), "v"(f.x), "v"(f.y), "v"(f.z), "v"(f.w));
    }
}
// acc = f16(acc * ms): m[q] holds -ms of query q in the half SEL picks (the sign is taken off by the instruction)
template <int SEL>
__device__ __forceinline__ void pk_scale8(half2_t (&acc)[8], const u32x4 m) {
    if (SEL == 0) {
        asm("v_pk_mul_f16 %0, %0, %8 op_sel_hi:[1,0] neg_lo:[0,1] neg_hi:[0,1]\n\t"
            "v_pk_mul_f16 %2, %2, %9 op_sel_hi:[1,0] neg_lo:[0,1] neg_hi:[0,1]\n\t"
            "v_pk_mul_f16 %4, %4, %10 op_sel_hi:[1,0] neg_lo:[0,1] neg_hi:[0,1]\n\t"
            "v_pk_mul_f16 %6, %6, %11 op_sel_hi:[1,0] neg_lo:[0,1] neg_hi:[0,1]\n\t"
            "v_pk_mul_f16 %1, %1, %8 op_sel_hi:[1,0] neg_lo:[0,1] neg_hi:[0,1]\n\t"
            "v_pk_mul_f16 %3, %3, %9 op_sel_hi:[1,0] neg_lo:[0,1] neg_hi:[0,1]\n\t"
            "v_pk_mul_f16 %5, %5, %10 op_sel_hi:[1,0] neg_lo:[0,1] neg_hi:[0,1]\n\t"
            "v_pk_mul_f16 %7, %7, %11 op_sel_hi:[1,0] neg_lo:[0,1] neg_hi:[0,1]"
            : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3]), "+v"(acc[4]), "+v"(acc[5]), "+v"(acc[6]), "+v"(acc[7])
            : "v"(m.x), "v"(m.y), "v"(m.z), "v"(m.w));
    } else {
        asm("v_pk_mul_f16 %0, %0, %8 op_sel:[0,1] op_sel_hi:[1,1] neg_lo:[0,1] neg_hi:[0,1]\n\t"
            "v_pk_mul_f16 %2, %2, %9 op_sel:[0,1] op_sel_hi:[1,1] neg_lo:[0,1] neg_hi:[0,1]\n\t"
            "v_pk_mul_f16 %4, %4, %10 op_sel:[0,1] op_sel_hi:[1,1] neg_lo:[0,1] neg_hi:[0,1]\n\t"
            "v_pk_mul_f16 %6, %6, %11 op_sel:[0,1] op_sel_hi:[1,1] neg_lo:[0,1] neg_hi:[0,1]\n\t"
            "v_pk_mul_f16 %1, %1, %8 op_sel:[0,1] op_sel_hi:[1,1] neg_lo:[0,1] neg_hi:[0,1]\n\t"
            "v_pk_mul_f16 %3, %3, %9 op_sel:[0,1] op_sel_hi:[1,1] neg_lo:[0,1] neg_hi:[0,1]\n\t"
            "v_pk_mul_f16 %5, %5, %10 op_sel:[0,1] op_sel_hi:[1,1] neg_lo:[0,1] neg_hi:[0,1]\n\t"
            "v_pk_mul_f16 %7, %7, %11 op_sel:[0,1] op_sel_hi:[1,1] neg_lo:[0,1] neg_hi:[0,1]"
            : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3]), "+v"(acc[4]), "+v"(acc[5]), "+v"(acc[6]), "+v"(acc[7])
            : "v"(m.x), "v"(m.y), "v"(m.z), "v"(m.w));
    }
}
// A key at which some query of the wavefront has a new maximum.  The factor tile marks such a (query, key) by its sign:
// -ms in place of vs (then vs is exactly 1).  Rescales the accumulators — the queries that stay as they are multiply by 1,
// which leaves the value — and puts 1 in place of -ms in the factor registers, so that the multiply-add that follows is the
// same instruction sequence with or without a rescale.  Everything happens in the registers it finds (tied asm operands):
// written as C++ selects, the compiler gives the changed factors or accumulators new registers and copies them back on the
// path without a rescale, eight or four v_mov per key on the path that matters.
template <int SEL>
__device__ __forceinline__ void pk_rescale(half2_t (&acc)[8], u32x4 & f) {
    const uint32_t keep = SEL ? 0x0000ffffu : 0xffff0000u, one = SEL ? 0x3c000000u : 0x00003c00u, neg_one = 0xbc00bc00u;
    u32x4 msn;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        uint32_t fq = f[q], m, t;
        if (SEL == 0)
            asm("v_and_b32 %1, 0x8000, %0\n\t"
                "v_cmp_ne_u32 vcc, 0, %1\n\t"
                "v_and_or_b32 %2, %0, %3, %5\n\t"
                "s_nop 0\n\t"
                "v_cndmask_b32 %1, %4, %0, vcc\n\t"           // -ms, or -1
                "v_cndmask_b32 %0, %0, %2, vcc"                 // 1 in place of -ms
                : "+v"(fq), "=&v"(m), "=&v"(t) : "v"(keep), "v"(neg_one), "v"(one) : "vcc");
        else
            asm("v_cmp_gt_i32 vcc, 0, %0\n\t"
                "v_and_or_b32 %2, %0, %3, %5\n\t"
                "s_nop 0\n\t"
                "v_cndmask_b32 %1, %4, %0, vcc\n\t"
                "v_cndmask_b32 %0, %0, %2, vcc"
                : "+v"(fq), "=&v"(m), "=&v"(t) : "v"(keep), "v"(neg_one), "v"(one) : "vcc");
        f[q] = fq; msn[q] = m;
    }
    pk_scale8<SEL>(acc, msn);
}
// two f32 factors -> one register of two f16 (round to nearest even, as the conversion in front of vdupq_n_f16)
__device__ __forceinline__ uint32_t pk_factors(float f0, float f1) {
    uint32_t r;
    asm("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(r) : "v"(f0), "v"(f1));
    return r;
}

// softmax factors of a run of scores that continues a running maximum M:  s[i] -> vs[i], ms[i]; also the run's
// contribution to the softmax denominator as (P, A): S_after = S_before * P + A
__device__ __forceinline__ void seq_factors(float s, float & M, float & vs, float & ms, float & P, float & A) {
    if (s == -INFINITY) { vs = 0.0f; ms = 1.0f; return; }       // masked key: the reference skips it
    const float Mn = fmaxf(M, s);
    ms = M == Mn ? 1.0f : expf(M - Mn);                          // 1 when the maximum stands, 0 for the first key
    vs = expf(s - Mn);                                           // 1 when s is the new maximum (libm-grade exp: the factors
                                                                 // feed f16 roundings that amplify last-bit differences)
    M = Mn;
    P *= ms;
    A = A * ms + vs;
}

// ------------------------------------------------------------------------------------------------------
// k_fattn_seq_row: one block per (query, head)
// ------------------------------------------------------------------------------------------------------

#define ROW_CHUNK 64
#define ROW_STAGE 192     // keys per stage: one per thread of the three wavefronts that do not walk the chain
#define ROW_VT    (ROW_STAGE + 8)   // f16 pitch of a d-row of the transposed V stage

// x of lane - N of the same row of 16 lanes (FILL where there is none), and lane 15 / lane 31 handed to the rows after it:
// the steps of a scan over the wavefront that stays out of LDS
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ float dpp_fill(float v, float fill) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, fill), __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xf, false));
}
__device__ __forceinline__ float readlane_f(float v, int l) { return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), l)); }
__device__ __forceinline__ float wave_scan_max(float v) {                      // inclusive
    v = fmaxf(v, dpp_fill<0x111>(v, -INFINITY));                               // row_shr:1
    v = fmaxf(v, dpp_fill<0x112>(v, -INFINITY));                               // row_shr:2
    v = fmaxf(v, dpp_fill<0x114>(v, -INFINITY));                               // row_shr:4
    v = fmaxf(v, dpp_fill<0x118>(v, -INFINITY));                               // row_shr:8
    v = fmaxf(v, dpp_fill<0x142, 0xa>(v, -INFINITY));                          // row_bcast:15 into rows 1 and 3
    v = fmaxf(v, dpp_fill<0x143, 0xc>(v, -INFINITY));                          // row_bcast:31 into rows 2 and 3
    return v;
}

// A pipeline of two roles with a stage of 192 keys between them.  Wavefront 0 (lane = d) walks the chain over stage s
// while wavefronts 1 .. 3 (one key per thread) work on the two stages after it, one barrier per stage:
//   factors of stage s + 1   exclusive prefix maximum (running maximum of the stages before, the wavefronts before, the
//                            thread's own scan value from the round before), the key's factor (vs, or -ms where it raises
//                            the maximum: then vs is exactly 1) -> LDS, the stage's share (P, A) of the denominator
//                            S <- S * P + A, the key's V row -> LDS transposed; request the V row of the stage after
//   scores of stage s + 2    dot product of the key's row (requested a round earlier) with q, the score, the maximum of
//                            the wavefront's 64 scores as an inclusive scan -> LDS; request the K row of the stage after
// so what a query costs is the chain (192 keys x two dependent instructions per stage) plus two rounds of lead-in: the
// scores, the exponentials and the staging run beside it on the other three SIMDs, and no array grows with the number
// of keys.
__global__ void __launch_bounds__(256) k_fattn_seq_row(fa_args a, int kv_pad) {
    // V stage, transposed: [d][key], in 16-byte pieces of eight keys.  Inside each run of 64 keys, piece p of row d sits at
    // p ^ 2 (d / 16): the producers' 16-byte writes (lanes: 8 pieces of d x 2 pieces of keys) then cover all banks once, as
    // the walker's reads do (16 consecutive d, one piece; the pitch is an odd number of pieces).
    __shared__ __attribute__((aligned(16))) half_t v_lds[2][FA_D * ROW_VT];
    __shared__ __attribute__((aligned(16))) float f_lds[2][ROW_STAGE];       // one factor per key
    __shared__ float red_m[2][3], red_p[2][3], red_a[2][3];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // Workgroup w runs on XCD w % 8, and each XCD has an L2 of its own: the queries of a head are dealt to one XCD (head h to
    // XCD h % 8), so that a head's K and V rows are fetched into one L2, once, instead of into as many as it has queries.
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int64_t n = slot % (int) a.N, h = xcd + 8 * (slot / (int) a.N), i3 = blockIdx.z;
    if (h >= a.H) return;                                  // (the grid is 8 x ceil(H / 8) x N wide)
    const int KV = (int) a.KV;
    const int n_stages = (kv_pad + ROW_STAGE - 1) / ROW_STAGE;

    if (wave != 0) {
        // ---- producers ----------------------------------------------------------------------------------------------
        const float * qp = (const float *)(a.q + n * a.q_nb1 + h * a.q_nb2 + i3 * a.q_nb3);
        const char *  kb = a.k + (h / a.hk_ratio) * a.k_nb2 + (i3 / a.k_ne3_ratio) * a.k_nb3;
        const char *  vb = a.v + (h / a.hv_ratio) * a.v_nb2 + (i3 / a.v_ne3_ratio) * a.v_nb3;
        const char * mp = a.mask ? a.mask + n * a.m_nb1 : nullptr;
        const int stid = tid - WAVE, pw = wave - 1;

        // Rows are read eight lanes to a row (16 bytes each): lane (r = lane / 8, c = lane % 8) takes piece c of the rows
        // 8 r + i, i = 0 .. 7, of its wavefront's 64 keys, so that every load instruction covers eight whole 128-byte
        // rows — with a row per lane it touches 64 of them and the stage's loads alone take longer than the chain.
        const int r8 = lane >> 3, c8 = lane & 7;
        float q[8];                                        // this lane's piece of q
        {
            const float4 t0 = *(const float4 *)(qp + 8 * c8), t1 = *(const float4 *)(qp + 8 * c8 + 4);
            q[0] = (float)(half_t) t0.x; q[1] = (float)(half_t) t0.y; q[2] = (float)(half_t) t0.z; q[3] = (float)(half_t) t0.w;
            q[4] = (float)(half_t) t1.x; q[5] = (float)(half_t) t1.y; q[6] = (float)(half_t) t1.z; q[7] = (float)(half_t) t1.w;
        }
        // Every load is unconditional and nothing in the loop is: a key beyond the end reads the last one (its score is
        // -inf and its V row zero), and after the last stage one more is scored that nobody walks.  With a load behind
        // a condition the registers it fills are copied where the paths join, and the copy waits for the load — the next
        // stage's rows would be waited for in the round that requests them.
        half8_t krow[8];
        u32x4 vrow[8];
        uint16_t mbits = 0;                                // the mask value of key `stid` of the stage as loaded (f16)
        // The mask comes as f16, or as the f32 tensor an f16 copy would have been made of (then each value is rounded here
        // as that copy rounds it).  Both forms are read, from an address that is readable either way, and one is kept.
        const uint16_t * mrow  = mp && !a.mask_f32 ? (const uint16_t *) mp : (const uint16_t *) kb;   // without such a mask: any readable address
        const float *    mrowf = mp && a.mask_f32 ? (const float *) mp : (const float *) kb;
        const int64_t m_step = mp && !a.mask_f32 ? 1 : 0, m_stepf = mp && a.mask_f32 ? 1 : 0;
        auto load_k = [&](int s) __attribute__((always_inline)) {
            const int key0 = s * ROW_STAGE + pw * WAVE + 8 * r8;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int kc = key0 + i < KV ? key0 + i : KV - 1;
                krow[i] = *(const half8_t *)(kb + (int64_t) kc * a.k_nb1 + 16 * c8);
            }
            const int key = s * ROW_STAGE + stid;
            const uint16_t m16 = mrow[(key < KV ? key : KV - 1) * m_step];
            const float    m32 = mrowf[(key < KV ? key : KV - 1) * m_stepf];
            mbits = a.mask_f32 ? f2h_bits(m32) : m16;
            if (a.mask_copy && h == 0 && key < KV) *(uint16_t *)((char *) a.mask_copy + n * a.mc_nb1 + (int64_t) key * 2) = mbits;
        };
        auto load_v = [&](int s) __attribute__((always_inline)) {
            const int key0 = s * ROW_STAGE + pw * WAVE + 8 * r8;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int kc = key0 + i < KV ? key0 + i : KV - 1;
                vrow[i] = *(const u32x4 *)(vb + (int64_t) kc * a.v_nb1 + 16 * c8);
            }
        };

        float score, inc, exc;                             // of the stage scored last: the score, the scan and the scan of the lane before
        auto score_phase = [&](int s) __attribute__((always_inline)) {
            const int key = s * ROW_STAGE + stid;
            // the piece's share of the eight rows' dot products, summed over the eight lanes of a row; lane c keeps row 8 r + c:
            // its own key
            float dot = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                float part = 0.0f;
#pragma unroll
                for (int e = 0; e < 8; ++e) part += q[e] * (float) krow[i][e];
                part = lanes_sum<8>(part);
                dot = c8 == i ? part : dot;
            }
            const float mval = mp ? h2f(mbits) : 0.0f;
            score = key < KV && mval != -INFINITY ? __fadd_rn(__fmul_rn(dot, a.scale), mval) : -INFINITY;
            load_k(s + 1);
            inc = wave_scan_max(score);
            if (lane == WAVE - 1) red_m[s & 1][pw] = inc;
            exc = dpp_fill<0x138>(inc, -INFINITY);         // wave_shr:1
        };

        // V rows first, then K rows, as in the loop: the wait in front of a use then leaves the younger loads in flight
        // on every path into it
        load_v(0);
        __builtin_amdgcn_sched_barrier(0);
        load_k(0);
        __builtin_amdgcn_sched_barrier(0);
        score_phase(0);
        __syncthreads();

        float M = -INFINITY;                               // running maximum over the stages whose factors are made
        for (int s = 1; s <= n_stages; ++s) {
            // ---- factors of stage s - 1
            {
                const int f = (s - 1) & 1;
                const int key = (s - 1) * ROW_STAGE + stid;
                float Mk = fmaxf(exc, M);
                if (pw > 0) Mk = fmaxf(Mk, red_m[f][0]);
                if (pw > 1) Mk = fmaxf(Mk, red_m[f][1]);
                M = fmaxf(fmaxf(M, red_m[f][0]), fmaxf(red_m[f][1], red_m[f][2]));
                float vs, ms, P = 1.0f, A = 0.0f;
                seq_factors(score, Mk, vs, ms, P, A);
                f_lds[f][stid] = ms != 1.0f ? -ms : vs;
                // ordered reduction of (P, A): (P1, A1) then (P2, A2) -> (P1*P2, A1*P2 + A2), as a binary tree over the
                // 64 keys: inside each row of 16 lanes with the lane 1, 2, 4, 8 further on (row_shl; beyond the row the
                // identity), then the four row totals
#define ROW_PA_STEP(CTRL) { const float Pn = dpp_fill<CTRL>(P, 1.0f), An = dpp_fill<CTRL>(A, 0.0f); A = A * Pn + An; P = P * Pn; }
                ROW_PA_STEP(0x101) ROW_PA_STEP(0x102) ROW_PA_STEP(0x104) ROW_PA_STEP(0x108)
#undef ROW_PA_STEP
                {
                    const float P0 = readlane_f(P, 0), P1 = readlane_f(P, 16), P2 = readlane_f(P, 32), P3 = readlane_f(P, 48);
                    const float A0 = readlane_f(A, 0), A1 = readlane_f(A, 16), A2 = readlane_f(A, 32), A3 = readlane_f(A, 48);
                    const float A01 = A0 * P1 + A1, P01 = P0 * P1, A23 = A2 * P3 + A3, P23 = P2 * P3;
                    if (lane == 0) { red_p[f][pw] = P01 * P23; red_a[f][pw] = A01 * P23 + A23; }
                }
                // V rows -> [d][key]: the lane holds d = 8 c .. 8 c + 7 of the keys 8 r .. 8 r + 7, which are 16 contiguous bytes
                // of each of its eight d-rows once the 8 x 8 block of halves is transposed in registers
                {
                    const int key0 = (s - 1) * ROW_STAGE + pw * WAVE + 8 * r8;
                    half_t * dst = v_lds[f] + (8 * c8) * ROW_VT + pw * WAVE + 8 * (r8 ^ (2 * (c8 >> 1)));   // (swizzled, see v_lds)
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        u32x4 o;
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const uint32_t lo = key0 + 2 * j     < KV ? vrow[2 * j    ][e >> 1] : 0u;
                            const uint32_t hi = key0 + 2 * j + 1 < KV ? vrow[2 * j + 1][e >> 1] : 0u;
                            o[j] = __builtin_amdgcn_perm(hi, lo, (e & 1) ? 0x07060302u : 0x05040100u);
                        }
                        *(u32x4 *)(dst + e * ROW_VT) = o;
                    }
                }
                load_v(s);
                __builtin_amdgcn_sched_barrier(0);         // requested here, a round before the rows are stored: not after the dot product
            }
            // ---- scores of stage s
            score_phase(s);
            __syncthreads();
        }
        return;
    }

    // ---- the walker: the sequential f16 chain, lane = d -------------------------------------------------------------------
    // With nothing else running on its SIMD the time of a key is the latency of its dependent instructions, so the common
    // case is straight-line code of two per key: v_fma_mix_f32 (f16 V, f32 factor, f16 accumulator -> f32) and
    // v_cvt_f16_f32 — the reference's f32 fma and its f16 store — and nothing between them: a v_readlane per key for the
    // factor would add a quarter to the time of a key.  So a unit of 32 keys is read from LDS a unit ahead as registers
    // only: the lane's V values, eight keys per 16-byte read (V sits in LDS transposed, pitch ROW_VT: such reads of 16
    // lanes cover all banks once), the 32 factors as eight reads of one address for all lanes, and factor k0 + lane % 32
    // once more for the vote on which keys raise the maximum.
    uint32_t acc = 0;                                      // f16 accumulator in the low half
    // one key: acc = f16(fma(v, vs, acc)); v is the low or the high half of `pair`
    auto mad = [&](uint32_t pair, bool high, float vs) __attribute__((always_inline)) {
        float t;
        if (high) asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel:[1,0,0] op_sel_hi:[1,0,1]" : "=v"(t) : "v"(pair), "v"(vs), "v"(acc));
        else      asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel_hi:[1,0,1]" : "=v"(t) : "v"(pair), "v"(vs), "v"(acc));
        asm("v_cvt_f16_f32 %0, %1" : "=v"(acc) : "v"(t));
    };
    constexpr int UNIT = 32;
    struct unit { u32x4 v[UNIT / 8]; float4 f[UNIT / 4]; float fl; };
    const int swz = 2 * (lane >> 4);                       // of this lane's row of the V stage
    auto read_unit = [&](unit & u, int buf, int k0) __attribute__((always_inline)) {      // k0: a multiple of 32
        const half_t * row = v_lds[buf] + lane * ROW_VT + (k0 & ~63);
#pragma unroll
        for (int i = 0; i < UNIT / 8; ++i) u.v[i] = *(const u32x4 *)(row + 8 * ((((k0 & 32) >> 3) + i) ^ swz));
        const float4 * fs = (const float4 *)(f_lds[buf] + k0);
#pragma unroll
        for (int i = 0; i < UNIT / 4; ++i) u.f[i] = fs[i];
        u.fl = f_lds[buf][k0 + (lane & (UNIT - 1))];
    };
    auto factor_of = [&](const unit & u, int j) __attribute__((always_inline)) {
        const float4 & f4 = u.f[j >> 2];
        return (j & 3) == 0 ? f4.x : (j & 3) == 1 ? f4.y : (j & 3) == 2 ? f4.z : f4.w;
    };
    auto run_unit = [&](const unit & u) __attribute__((always_inline)) {
        const uint32_t raised = (uint32_t) __ballot((int32_t) __float_as_uint(u.fl) < 0);   // uniform: keys with -ms (down to -0)
        if (raised == 0) {
#pragma unroll
            for (int j = 0; j < UNIT; ++j) mad(u.v[j >> 3][(j >> 1) & 3], j & 1, factor_of(u, j));   // masked keys: vs = 0 leaves acc as it is
        } else {
            // rare after the first keys of a row: eight keys at a time, key by key only where one of the eight raises
#pragma unroll
            for (int g = 0; g < UNIT / 8; ++g) {
                if (((raised >> (8 * g)) & 0xff) == 0) {
#pragma unroll
                    for (int j = 8 * g; j < 8 * g + 8; ++j) mad(u.v[g][(j >> 1) & 3], j & 1, factor_of(u, j));
                } else {
#pragma unroll
                    for (int j = 8 * g; j < 8 * g + 8; ++j) {
                        float fj = factor_of(u, j);
                        if ((raised >> j) & 1) {           // scalar condition
                            float t;
                            asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel_hi:[1,0,0]" : "=v"(t) : "v"(acc), "v"(-fj));
                            asm("v_cvt_f16_f32 %0, %1" : "=v"(acc) : "v"(t));
                            fj = 1.0f;                     // vs = 1
                        }
                        mad(u.v[g][(j >> 1) & 3], j & 1, fj);
                    }
                }
            }
        }
    };

    // Three sets of registers go round the six units of a stage.  The last unit of a stage is walked after the barrier that
    // opens the next one, under that stage's first LDS reads: its values are in registers by then, and the producers get
    // the buffer a unit earlier.
    float S = 0.0f;
    unit ua, ub, uc;
    bool pending = false;                                  // uc holds the sixth unit of the stage before
    __syncthreads();                                       // stage 0 is scored
    for (int s = 0; s < n_stages; ++s) {
        __syncthreads();                                   // stage s has its factors and its V rows
        const int buf = s & 1;
        const int nk = min(ROW_STAGE, kv_pad - s * ROW_STAGE);                  // 64, 128 or 192
        read_unit(ua, buf, 0);
#pragma unroll
        for (int w = 0; w < 3; ++w) S = S * red_p[buf][w] + red_a[buf][w];
        if (pending) run_unit(uc);
        read_unit(ub, buf, UNIT);
        run_unit(ua);
        if (nk > 2 * UNIT) read_unit(uc, buf, 2 * UNIT);
        run_unit(ub);
        pending = false;
        if (nk > 2 * UNIT) {
            read_unit(ua, buf, 3 * UNIT);
            run_unit(uc);
            if (nk > 4 * UNIT) read_unit(ub, buf, 4 * UNIT);
            run_unit(ua);
            if (nk > 4 * UNIT) {
                read_unit(uc, buf, 5 * UNIT);
                run_unit(ub);
                pending = true;
            }
        }
    }
    if (pending) run_unit(uc);

    half_t acc_h; { const uint16_t t16 = (uint16_t) acc; __builtin_memcpy(&acc_h, &t16, 2); }
    float * dp = (float *) a.d + ((i3 * a.N + n) * a.H + h) * FA_D;
    const float o = (float) acc_h * (1.0f / S);
    dp[lane] = o;
    if (a.x16) {
        // MI355X_FA_EMIT_Q8_0: the projection that follows reads its activations as Q8_0 (rows [N][H * 64]: int8 quants |
        // f32 scales | int32 block sums); this wavefront holds two blocks of one row, one per 32 lanes
        float amax = fabsf(o);
        amax = lanes_max<32>(amax);
        const float id = amax != 0.0f ? 127.0f / amax : 0.0f;
        const int q = (int) rintf(o * id);
        int qsum = q;
        qsum = lanes_sum<32>(qsum);
        char * q8 = (char *) a.x16;
        const int64_t K = a.H * FA_D, nbk = K / 32, rows = a.N * a.ne3, rowi = i3 * a.N + n;
        ((int8_t *) q8)[rowi * K + h * FA_D + lane] = (int8_t) q;
        if ((lane & 31) == 0) {
            const int64_t blk = rowi * nbk + h * 2 + (lane >> 5);
            ((float *)(q8 + rows * K))[blk] = h2f(f2h_bits(div127(amax)));
            ((int32_t *)(q8 + rows * K + rows * nbk * 4))[blk] = qsum;
        }
    }
}

// ------------------------------------------------------------------------------------------------------
// k_fattn_pk_row: one block per (query, head), the packed-f16 form of the step (MI355X_FA_F16_PK with at most 8 queries)
//
// The same pipeline as k_fattn_seq_row — wavefront 0 walks the chain over stage s while wavefronts 1 .. 3 make the factors
// of stage s + 1 and the scores of stage s + 2, one barrier per stage — with the step the reference's Arm build takes
// (vec.h:180-203, 295-311: the factor rounded to f16, one f16 fused multiply-add per element).  A key is then ONE dependent
// instruction for the walker, v_pk_fma_f16 on a lane's pair of d (3.7 ns against the 5.3 ns of v_fma_mix_f32 +
// v_cvt_f16_f32), and what stood beside the chain had to shrink with it (a stage of 192 keys: 1.9 us -> 1.05 us):
//   walker     lane l holds d = 2 (l % 32), 2 (l % 32) + 1 (the upper half of the wavefront mirrors the lower).  Per unit of
//              32 keys: eight 16-byte reads of V (the stage holds V as [d pair][key], a dword per key), four 16-byte reads
//              of factors (f16, eight keys each, one address for all lanes), and the unit's raise bits as a scalar: no
//              vote, no selects.  A unit without a raise is 32 instructions in a row; a unit with one multiplies the
//              accumulator by a second factor in front of every key (1 where the key raises nothing) — no branch per key
//              and no copy of the code per raise pattern, which for a lone wavefront cost more than the arithmetic.
//   producers  the factors of a key come from one v_exp_f32: with scores in log2 units, exp2(-|s - M|) against the
//              exclusive prefix maximum M is vs where the maximum stands and ms where the key raises it (then vs is
//              exactly 1).  The denominator's share of a stage is a plain sum of exp2(s - M_end) over its keys and
//              P = exp2(M_before - M_end): S <- S P + A (f32, as the reference keeps it).  V rows go to the stage as
//              they are loaded, dword by dword — pairs of d stay together, so there is nothing to transpose inside a
//              register.  Rows come through buffer descriptors with the stage's offset as a scalar operand: no address
//              arithmetic in the loop (it was a quarter of a round's instructions, the slow integer multiplies among them).
//   placement  the queries of a head run on one XCD, so a head's K and V reach one L2, once (with a query per XCD, as
//              the plain grid deals them, every XCD fetches every head: more than its L2 holds).
// ------------------------------------------------------------------------------------------------------

#define PROW_PITCH (ROW_STAGE + 4)     // dwords per d-pair row of the V stage: 784 bytes, 16 mod 256

__global__ void __launch_bounds__(256) k_fattn_pk_row(fa_args a, int kv_pad) {
    // V stage: [d pair][key], a dword per key.  The 16-byte piece g (keys 4 g .. 4 g + 3) of row p sits at piece g ^ (p / 16):
    // 16 lanes of a producer's write (eight rows four apart, pieces 2 r and 2 r + 1) and 16 lanes of the walker's read (16
    // consecutive rows, one piece: the pitch is 16 bytes past a multiple of 256) each cover all 64 banks once.
    __shared__ __attribute__((aligned(16))) uint32_t v_lds[2][32 * PROW_PITCH];
    // two f16 factors per key: the accumulator is multiplied by fm (ms where the key raises the maximum, else 1) and takes
    // v * fv (1 where it raises, else vs); a unit of 32 keys without a raise — almost all of them — needs fv only
    __shared__ __attribute__((aligned(16))) uint16_t fv_lds[2][ROW_STAGE], fm_lds[2][ROW_STAGE];
    __shared__ uint32_t raise_lds[2][8];                                      // does the key raise the maximum?  32 keys to a dword
    __shared__ float red_m[2][3], red_a[2][3], red_p[2];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // Workgroup w runs on XCD w % 8, and each XCD has an L2 of its own: the queries of a head are dealt to one XCD (head h to
    // XCD h % 8), so that a head's K and V rows are fetched into one L2, once, instead of into as many as it has queries.
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int64_t n = slot % (int) a.N, h = xcd + 8 * (slot / (int) a.N), i3 = blockIdx.z;
    if (h >= a.H) return;                                  // (the grid is 8 x ceil(H / 8) x N wide)
    const int KV = (int) a.KV;
    const int n_stages = (kv_pad + ROW_STAGE - 1) / ROW_STAGE;

    if (wave != 0) {
        // ---- producers ----------------------------------------------------------------------------------------------
        const float * qp = (const float *)(a.q + n * a.q_nb1 + h * a.q_nb2 + i3 * a.q_nb3);
        const char *  kb = a.k + (h / a.hk_ratio) * a.k_nb2 + (i3 / a.k_ne3_ratio) * a.k_nb3;
        const char *  vb = a.v + (h / a.hv_ratio) * a.v_nb2 + (i3 / a.v_ne3_ratio) * a.v_nb3;
        const char * mp = a.mask ? a.mask + n * a.m_nb1 : nullptr;
        const int stid = tid - WAVE, pw = wave - 1;
        const float scale2 = a.scale * LOG2E_F;

        // Rows are read eight lanes to a row (16 bytes each), as in k_fattn_seq_row, through buffer descriptors: the offset of a
        // lane's eight rows inside a stage is computed once, the stage's own offset is a scalar operand of the load, and a key
        // beyond the end reads zeros (its score is -inf, its factor 0) — no address arithmetic and no clamps inside the loop.
        const int r8 = lane >> 3, c8 = lane & 7;
        float q[8];                                        // this lane's piece of q
        {
            const float4 t0 = *(const float4 *)(qp + 8 * c8), t1 = *(const float4 *)(qp + 8 * c8 + 4);
            q[0] = (float)(half_t) t0.x; q[1] = (float)(half_t) t0.y; q[2] = (float)(half_t) t0.z; q[3] = (float)(half_t) t0.w;
            q[4] = (float)(half_t) t1.x; q[5] = (float)(half_t) t1.y; q[6] = (float)(half_t) t1.z; q[7] = (float)(half_t) t1.w;
        }
        const uint32_t k_nb1 = (uint32_t) a.k_nb1, v_nb1 = (uint32_t) a.v_nb1;
        const __amdgpu_buffer_rsrc_t k_rs = __builtin_amdgcn_make_buffer_rsrc((void *) kb, 0, (uint32_t)(KV - 1) * k_nb1 + FA_D * 2, 0x00020000);
        const __amdgpu_buffer_rsrc_t v_rs = __builtin_amdgcn_make_buffer_rsrc((void *) vb, 0, (uint32_t)(KV - 1) * v_nb1 + FA_D * 2, 0x00020000);
        // the mask as f16, or as the f32 tensor an f16 copy would have been made of (then each value is rounded here as that copy
        // rounds it): both forms are read, one of them from a descriptor without records (zeros)
        const __amdgpu_buffer_rsrc_t m16_rs = __builtin_amdgcn_make_buffer_rsrc((void *)(mp ? mp : a.k), 0, mp && !a.mask_f32 ? (uint32_t) KV * 2 : 0u, 0x00020000);
        const __amdgpu_buffer_rsrc_t m32_rs = __builtin_amdgcn_make_buffer_rsrc((void *)(mp ? mp : a.k), 0, mp && a.mask_f32 ? (uint32_t) KV * 4 : 0u, 0x00020000);
        uint32_t k_off[8], v_off[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) { k_off[i] = (uint32_t)(pw * WAVE + 8 * r8 + i) * k_nb1 + 16 * c8; v_off[i] = (uint32_t)(pw * WAVE + 8 * r8 + i) * v_nb1 + 16 * c8; }
        u32x4 krow[8];
        u32x4 vrow[8];
        uint16_t mbits = 0;                                // the mask value of key `stid` of the stage as loaded (f16)
        auto load_k = [&](int s) __attribute__((always_inline)) {
            const uint32_t so = (uint32_t) __builtin_amdgcn_readfirstlane(s * ROW_STAGE) * k_nb1;
#pragma unroll
            for (int i = 0; i < 8; ++i) krow[i] = __builtin_amdgcn_raw_buffer_load_b128(k_rs, k_off[i], so, 0);
            const uint32_t ko = (uint32_t) __builtin_amdgcn_readfirstlane(s * ROW_STAGE);
            const uint16_t m16 = __builtin_amdgcn_raw_buffer_load_b16(m16_rs, stid * 2, ko * 2, 0);
            const float    m32 = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(m32_rs, stid * 4, ko * 4, 0));
            mbits = a.mask_f32 ? f2h_bits(m32) : m16;
            const int key = s * ROW_STAGE + stid;
            if (a.mask_copy && h == 0 && key < KV) *(uint16_t *)((char *) a.mask_copy + n * a.mc_nb1 + (int64_t) key * 2) = mbits;
        };
        auto load_v = [&](int s) __attribute__((always_inline)) {
            const uint32_t so = (uint32_t) __builtin_amdgcn_readfirstlane(s * ROW_STAGE) * v_nb1;
#pragma unroll
            for (int i = 0; i < 8; ++i) vrow[i] = __builtin_amdgcn_raw_buffer_load_b128(v_rs, v_off[i], so, 0);
        };

        float score, inc, exc;                             // of the stage scored last, in log2 units: the score, its scan, the scan of the lane before
        auto score_phase = [&](int s) __attribute__((always_inline)) {
            const int key = s * ROW_STAGE + stid;
            // the piece's share of the eight rows' dot products (f32 multiply-adds on the converted halves: v_dot2_f32_f16 would
            // halve them, and moves flat attention over 1500 keys from 2e-7 to 2e-5 of the pinned sequence), summed over the
            // eight lanes of a row; lane c keeps row 8 r + c: its own key
            // (the eight rows side by side, element by element and step by step: a lone wavefront pays the full latency of
            // every instruction that depends on the one before it)
            float part[8] = { 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f };
#pragma unroll
            for (int e = 0; e < 8; ++e) {
#pragma unroll
                for (int i = 0; i < 8; ++i) part[i] = __builtin_fmaf(q[e], (float) __builtin_bit_cast(half8_t, krow[i])[e], part[i]);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) part[i] += dpp_move<float, 0xB1>(part[i]);      // quad_perm [1,0,3,2]
#pragma unroll
            for (int i = 0; i < 8; ++i) part[i] += dpp_move<float, 0x4E>(part[i]);      // quad_perm [2,3,0,1]
#pragma unroll
            for (int i = 0; i < 8; ++i) part[i] += dpp_move<float, 0x141>(part[i]);     // row_half_mirror
            float dot = part[0];
#pragma unroll
            for (int i = 1; i < 8; ++i) dot = c8 == i ? part[i] : dot;
            const float mval = mp ? h2f(mbits) : 0.0f;
            score = key < KV && mval != -INFINITY ? __builtin_fmaf(dot, scale2, mval * LOG2E_F) : -INFINITY;
            load_k(s + 1);
            inc = wave_scan_max(score);
            if (lane == WAVE - 1) red_m[s & 1][pw] = inc;
            exc = dpp_fill<0x138>(inc, -INFINITY);         // wave_shr:1
        };
        load_v(0);
        __builtin_amdgcn_sched_barrier(0);
        load_k(0);
        __builtin_amdgcn_sched_barrier(0);
        score_phase(0);
        __syncthreads();

        float M = -INFINITY;                               // running maximum over the stages whose factors are made
        for (int s = 1; s <= n_stages; ++s) {
            // ---- factors of stage s - 1
            {
                const int f = (s - 1) & 1;
                const float m0 = red_m[f][0], m1 = red_m[f][1], m2 = red_m[f][2];
                float Mk = fmaxf(exc, M);                  // the maximum over every key before this one
                if (pw > 0) Mk = fmaxf(Mk, m0);
                if (pw > 1) Mk = fmaxf(Mk, m1);
                const float Mend = fmaxf(fmaxf(M, m0), fmaxf(m1, m2));
                // (-inf - -inf, a masked key before any other: NaN, which the maximum with 0 turns into 0)
                const float e  = fmaxf(__builtin_amdgcn_exp2f(-fabsf(score - Mk)), 0.0f);
                const float ak = fmaxf(__builtin_amdgcn_exp2f(score - Mend), 0.0f);
                const bool raise = score > Mk;
                const uint16_t eh = f2h_bits(e);
                fv_lds[f][stid] = raise ? (uint16_t) 0x3c00 : eh;
                fm_lds[f][stid] = raise ? eh : (uint16_t) 0x3c00;
                const uint64_t rb = __ballot(raise);
                float A = lanes_sum<16>(ak);                 // (the four rows' sums joined in a fixed order, without the LDS trip of a swizzle)
                A = (readlane_f(A, 0) + readlane_f(A, 16)) + (readlane_f(A, 32) + readlane_f(A, 48));
                if (lane == 0) {
                    raise_lds[f][2 * pw] = (uint32_t) rb; raise_lds[f][2 * pw + 1] = (uint32_t)(rb >> 32);
                    red_a[f][pw] = A;
                    if (pw == 0) red_p[f] = fmaxf(__builtin_amdgcn_exp2f(M - Mend), 0.0f);
                }
                M = Mend;
                // V rows -> [d pair][key]: dword j of the lane's eight rows is d pair 4 c + j of the keys 8 r .. 8 r + 7
                {
                    uint32_t * dst = v_lds[f] + (4 * c8) * PROW_PITCH;
                    const int g = 16 * pw + 2 * r8, sw = c8 >> 2;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const u32x4 lo = { vrow[0][j], vrow[1][j], vrow[2][j], vrow[3][j] }, hi = { vrow[4][j], vrow[5][j], vrow[6][j], vrow[7][j] };
                        *(u32x4 *)(dst + j * PROW_PITCH + 4 * (g ^ sw))       = lo;
                        *(u32x4 *)(dst + j * PROW_PITCH + 4 * ((g + 1) ^ sw)) = hi;
                    }
                }
                load_v(s);
                __builtin_amdgcn_sched_barrier(0);
            }
            // ---- scores of stage s (there is none behind the last)
            if (s < n_stages) score_phase(s);
            __syncthreads();
        }
        return;
    }

    // ---- the walker ---------------------------------------------------------------------------------------------------
    const int p = lane & 31;                               // d pair
    uint32_t acc = 0;
    constexpr int UNIT = 32;
    struct unit { u32x4 v[UNIT / 4]; u32x4 f[UNIT / 8]; };
    const int swz = p >> 4;
    auto read_unit = [&](unit & u, int buf, int k0) __attribute__((always_inline)) {      // k0: a multiple of 32
        const uint32_t * row = v_lds[buf] + p * PROW_PITCH;
#pragma unroll
        for (int i = 0; i < UNIT / 4; ++i) u.v[i] = *(const u32x4 *)(row + 4 * ((k0 / 4 + i) ^ swz));
        const u32x4 * fs = (const u32x4 *)(fv_lds[buf] + k0);
#pragma unroll
        for (int i = 0; i < UNIT / 8; ++i) u.f[i] = fs[i];
    };
    // eight keys without a raise: one asm statement, so that nothing is placed between the dependent instructions
    auto eight = [&](const u32x4 & v0, const u32x4 & v1, const u32x4 & f) __attribute__((always_inline)) {
        asm("v_pk_fma_f16 %0, %1, %9, %0 op_sel_hi:[1,0,1]\n\t"
            "v_pk_fma_f16 %0, %2, %9, %0 op_sel:[0,1,0] op_sel_hi:[1,1,1]\n\t"
            "v_pk_fma_f16 %0, %3, %10, %0 op_sel_hi:[1,0,1]\n\t"
            "v_pk_fma_f16 %0, %4, %10, %0 op_sel:[0,1,0] op_sel_hi:[1,1,1]\n\t"
            "v_pk_fma_f16 %0, %5, %11, %0 op_sel_hi:[1,0,1]\n\t"
            "v_pk_fma_f16 %0, %6, %11, %0 op_sel:[0,1,0] op_sel_hi:[1,1,1]\n\t"
            "v_pk_fma_f16 %0, %7, %12, %0 op_sel_hi:[1,0,1]\n\t"
            "v_pk_fma_f16 %0, %8, %12, %0 op_sel:[0,1,0] op_sel_hi:[1,1,1]"
            : "+v"(acc)
            : "v"(v0.x), "v"(v0.y), "v"(v0.z), "v"(v0.w), "v"(v1.x), "v"(v1.y), "v"(v1.z), "v"(v1.w), "v"(f.x), "v"(f.y), "v"(f.z), "v"(f.w));
    };
    // ... and eight keys of a unit in which some key raises the maximum: the scale by fm in front of every step.  No branch
    // per key and no second copy of the code per raise pattern: a taken branch costs a lone wavefront as much as four keys,
    // and code that is rarely run comes from beyond the instruction cache.
    auto eight_scaled = [&](const u32x4 & v0, const u32x4 & v1, const u32x4 & f, const u32x4 & m) __attribute__((always_inline)) {
        asm("v_pk_mul_f16 %0, %0, %13 op_sel_hi:[1,0]\n\t"            "v_pk_fma_f16 %0, %1, %9, %0 op_sel_hi:[1,0,1]\n\t"
            "v_pk_mul_f16 %0, %0, %13 op_sel:[0,1] op_sel_hi:[1,1]\n\t" "v_pk_fma_f16 %0, %2, %9, %0 op_sel:[0,1,0] op_sel_hi:[1,1,1]\n\t"
            "v_pk_mul_f16 %0, %0, %14 op_sel_hi:[1,0]\n\t"            "v_pk_fma_f16 %0, %3, %10, %0 op_sel_hi:[1,0,1]\n\t"
            "v_pk_mul_f16 %0, %0, %14 op_sel:[0,1] op_sel_hi:[1,1]\n\t" "v_pk_fma_f16 %0, %4, %10, %0 op_sel:[0,1,0] op_sel_hi:[1,1,1]\n\t"
            "v_pk_mul_f16 %0, %0, %15 op_sel_hi:[1,0]\n\t"            "v_pk_fma_f16 %0, %5, %11, %0 op_sel_hi:[1,0,1]\n\t"
            "v_pk_mul_f16 %0, %0, %15 op_sel:[0,1] op_sel_hi:[1,1]\n\t" "v_pk_fma_f16 %0, %6, %11, %0 op_sel:[0,1,0] op_sel_hi:[1,1,1]\n\t"
            "v_pk_mul_f16 %0, %0, %16 op_sel_hi:[1,0]\n\t"            "v_pk_fma_f16 %0, %7, %12, %0 op_sel_hi:[1,0,1]\n\t"
            "v_pk_mul_f16 %0, %0, %16 op_sel:[0,1] op_sel_hi:[1,1]\n\t" "v_pk_fma_f16 %0, %8, %12, %0 op_sel:[0,1,0] op_sel_hi:[1,1,1]"
            : "+v"(acc)
            : "v"(v0.x), "v"(v0.y), "v"(v0.z), "v"(v0.w), "v"(v1.x), "v"(v1.y), "v"(v1.z), "v"(v1.w), "v"(f.x), "v"(f.y), "v"(f.z), "v"(f.w),
              "v"(m.x), "v"(m.y), "v"(m.z), "v"(m.w));
    };
    struct scales { u32x4 m[UNIT / 8]; };
    auto read_scales = [&](scales & t, int buf, int k0) __attribute__((always_inline)) {
        const u32x4 * ms = (const u32x4 *)(fm_lds[buf] + k0);
#pragma unroll
        for (int i = 0; i < UNIT / 8; ++i) t.m[i] = ms[i];
    };
    auto run_unit_with = [&](const unit & u, uint32_t raised, const scales & t) __attribute__((always_inline)) {   // raised: uniform
        if (raised == 0) {
#pragma unroll
            for (int g = 0; g < UNIT / 8; ++g) eight(u.v[2 * g], u.v[2 * g + 1], u.f[g]);
        } else {                                           // rare after the first keys of a row
#pragma unroll
            for (int g = 0; g < UNIT / 8; ++g) eight_scaled(u.v[2 * g], u.v[2 * g + 1], u.f[g], t.m[g]);
        }
    };
    auto run_unit = [&](const unit & u, uint32_t raised, int buf, int k0) __attribute__((always_inline)) {
        scales t = {};
        if (raised != 0) read_scales(t, buf, k0);
        run_unit_with(u, raised, t);
    };
    auto raise_bits = [&](int buf, int u) __attribute__((always_inline)) { return (uint32_t) __builtin_amdgcn_readfirstlane((int) raise_lds[buf][u]); };

    float S = 0.0f;
    unit ua, ub, uc;
    scales sc = {};                                        // of the unit held in uc, when it has a raise
    uint32_t rc = 0;                                       // raise bits of the unit held in uc
    bool pending = false;                                  // uc holds the sixth unit of the stage before
    __syncthreads();                                       // stage 0 is scored
    for (int s = 0; s < n_stages; ++s) {
        __syncthreads();                                   // stage s has its factors and its V rows
        const int buf = s & 1;
        const int nk = min(ROW_STAGE, kv_pad - s * ROW_STAGE);                  // 64, 128 or 192
        read_unit(ua, buf, 0);
        const uint32_t r0 = raise_bits(buf, 0), r1 = raise_bits(buf, 1), r2 = raise_bits(buf, 2), r3 = raise_bits(buf, 3), r4 = raise_bits(buf, 4), r5 = raise_bits(buf, 5);
        S = S * red_p[buf] + ((red_a[buf][0] + red_a[buf][1]) + red_a[buf][2]);
        if (pending) run_unit_with(uc, rc, sc);           // (its scales were read before the barrier: the producers have the buffer now)
        read_unit(ub, buf, UNIT);
        run_unit(ua, r0, buf, 0);
        if (nk > 2 * UNIT) read_unit(uc, buf, 2 * UNIT);
        run_unit(ub, r1, buf, UNIT);
        pending = false;
        if (nk > 2 * UNIT) {
            read_unit(ua, buf, 3 * UNIT);
            run_unit(uc, r2, buf, 2 * UNIT);
            if (nk > 4 * UNIT) read_unit(ub, buf, 4 * UNIT);
            run_unit(ua, r3, buf, 3 * UNIT);
            if (nk > 4 * UNIT) {
                read_unit(uc, buf, 5 * UNIT);
                if (r5 != 0) read_scales(sc, buf, 5 * UNIT);
                run_unit(ub, r4, buf, 4 * UNIT);
                rc = r5;
                pending = true;
            }
        }
    }
    if (pending) run_unit_with(uc, rc, sc);

    const float inv = 1.0f / S;
    half2_t acc_h; __builtin_memcpy(&acc_h, &acc, 4);
    const float o0 = (float) acc_h[0] * inv, o1 = (float) acc_h[1] * inv;
    float * dp = (float *) a.d + ((i3 * a.N + n) * a.H + h) * FA_D;
    if (lane < 32) *(float2 *)(dp + 2 * p) = make_float2(o0, o1);
    if (a.x16) {
        // MI355X_FA_EMIT_Q8_0 (rows [N][H * 64]: int8 quants | f32 scales | int32 block sums): 16 lanes hold a block
        float amax = fmaxf(fabsf(o0), fabsf(o1));
        amax = lanes_max<16>(amax);
        const float id = amax != 0.0f ? 127.0f / amax : 0.0f;
        const int q0 = (int) rintf(o0 * id), q1 = (int) rintf(o1 * id);
        int qsum = q0 + q1;
        qsum = lanes_sum<16>(qsum);
        char * q8 = (char *) a.x16;
        const int64_t K = a.H * FA_D, nbk = K / 32, rows = a.N * a.ne3, rowi = i3 * a.N + n;
        if (lane < 32) {
            *(uint16_t *)(q8 + rowi * K + h * FA_D + 2 * p) = (uint16_t)((q0 & 0xff) | ((q1 & 0xff) << 8));
            if ((p & 15) == 0) {
                const int64_t blk = rowi * nbk + h * 2 + (p >> 4);
                ((float *)(q8 + rows * K))[blk] = h2f(f2h_bits(div127(amax)));
                ((int32_t *)(q8 + rows * K + rows * nbk * 4))[blk] = qsum;
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------------
// k_fattn_seq_tile: 64 queries per block, 64 keys per step
//
// Per step: (1) K tile -> LDS, S = Q K^T on the matrix cores, scores -> LDS; (2) thread (query, 16-key run) turns the
// scores into one factor per (query, key): f = vs = exp(s - M_k) when the running maximum stands, f = -ms =
// -exp(M_{k-1} - M_k) when key k raises it (then vs is exactly 1); (3) the chains: lane = query, wavefront = 16 of the
// 64 d.  All lanes of a wavefront then want the same 16 V values per key: two broadcast LDS reads; the factors come
// four keys per LDS read.  Per key and lane that leaves the 16 fma + 8 pack instructions the reference's rounding
// sequence dictates; a rescale is only looked for once per four keys.
// ------------------------------------------------------------------------------------------------------

#define T_Q   64
#define T_KV  64
#define T_LDH (FA_D + 8)      // f16 pitch of the Q and K tiles (144 B rows: conflict-free b128 reads for the MFMA operands)
#define T_LDF (T_KV + 4)      // f32 pitch of the factor tile (272 B rows: conflict-free b128 reads with lane = row)

// exp(x) for x <= 0 to about 1 ulp: 2^(x log2 e) with the rounding error of the product fed back in.  Without a branch:
// below the smallest denormal, at x = -inf (first key of a row) and for NaN (-inf - -inf: a masked key before any other)
// the result is selected to 0 afterwards.
__device__ __forceinline__ float exp_neg(float x) {
    const float l2e_hi = 1.44269502e+0f, l2e_lo = 1.92596299e-8f;
    const float t = x * l2e_hi;
    float e = __builtin_fmaf(x, l2e_hi, -t);
    e = __builtin_fmaf(x, l2e_lo, e);
    const float r = __builtin_amdgcn_exp2f(t);
    const float y = __builtin_fmaf(r, e * 0.693147182f, r);
    return x >= -104.0f ? y : 0.0f;
}

typedef const uint32_t __attribute__((address_space(4))) * const_u32_ptr;   // read-only data: uniform loads become scalar loads

// Eight wavefronts in two roles, a tile of 64 keys between them:
//   wavefronts 4 .. 7 (producers) prepare tile t + 1: K / V rows -> LDS, S = Q K^T on the matrix cores, the factors;
//   wavefronts 0 .. 3 (chains) walk tile t: 16 queries x all 64 d each (lane = query 16 w + l % 16, d slice l / 16).
// The factor tile and the V tile are double buffered, so the two roles meet at two barriers per tile — the tile boundary
// and the point inside a tile where the producers' factor step needs all of their score writes — and otherwise run side
// by side: a SIMD holds one chain and one producer wavefront of each workgroup,
// and the chains' vector work, which is what bounds the kernel, no longer waits for the score and factor steps.
#define T_LDS_BYTES ((T_Q * T_LDH + T_KV * T_LDH + 2 * T_KV * FA_D) * 2 + (2 * T_Q * T_LDF + 2 * T_Q) * 4)     // 70144: beyond the 64 KB a launch gets unasked

__global__ void __launch_bounds__(512, 2) k_fattn_seq_tile(fa_args a) {
    extern __shared__ __attribute__((aligned(16))) char t_smem[];
    half_t * q_s = (half_t *) t_smem;                      // [T_Q * T_LDH]
    half_t * k_s = q_s + T_Q * T_LDH;                      // [T_KV * T_LDH]
    half_t * v_s2 = k_s + T_KV * T_LDH;                    // [2][T_KV * FA_D]
    float *  f_s2 = (float *)(v_s2 + 2 * T_KV * FA_D);     // [2][T_Q * T_LDF]
    float *  m_run = f_s2 + 2 * T_Q * T_LDF, * s_run = m_run + T_Q;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // Workgroups go round-robin to the 8 XCDs, each with an L2 of its own.  The query tiles of one head all read that head's K
    // and V (384 KB for 1500 keys), so every XCD gets one run of consecutive (head, query tile) pairs, head-major: a head's
    // K and V are then fetched into one or two L2s instead of all eight.
    const uint32_t lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z), total = gridDim.x * gridDim.y * gridDim.z;
    const uint32_t xcd = lin % 8, per = total / 8, extra = total % 8;
    const uint32_t item = xcd * per + (xcd < extra ? xcd : extra) + lin / 8;
    const int64_t n0 = (int64_t)(item % gridDim.x) * T_Q, h = (item / gridDim.x) % gridDim.y, i3 = item / (gridDim.x * gridDim.y);
    const int n_tiles = (int)((a.KV + T_KV - 1) / T_KV);

    if (wave >= 4) {
        // ---- producers ---------------------------------------------------------------------------------------------------------------
        const int tid = threadIdx.x - 256, pw = wave - 4;
        const char * qb = a.q + h * a.q_nb2 + i3 * a.q_nb3;
        const char * kb = a.k + (h / a.hk_ratio) * a.k_nb2 + (i3 / a.k_ne3_ratio) * a.k_nb3;
        const char * vb = a.v + (h / a.hv_ratio) * a.v_nb2 + (i3 / a.v_ne3_ratio) * a.v_nb3;

        // Q tile -> f16 in LDS; thread t: row t/4, 16 values
        {
            const int r = tid >> 2, c = (tid & 3) * 16;
            const int64_t n = n0 + r;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
                if (n < a.N) t = *(const float4 *)(qb + n * a.q_nb1 + (c + 4 * i) * 4);
                half4_t hq = { (half_t) t.x, (half_t) t.y, (half_t) t.z, (half_t) t.w };
                *(half4_t *)(q_s + r * T_LDH + c + 4 * i) = hq;
            }
        }
        if (tid < T_Q) { m_run[tid] = -INFINITY; s_run[tid] = 0.0f; }

        // score role: wavefront w computes the 32x32 patch (queries 32*(w/2).., keys 32*(w%2)..)
        const int sq = (pw >> 1) * 32, sk = (pw & 1) * 32, l32 = lane & 31, g = lane >> 5;
        // K / V tile staging: thread t: row t/4, 32 bytes of each; the tile after the next is in flight while one is worked on
        const int kr = tid >> 2, kc = (tid & 3) * 16;
        u32x4 kreg0, kreg1, vreg0, vreg1;
        auto load_kv = [&](int64_t key0) __attribute__((always_inline)) {
            const int64_t key = key0 + kr < a.KV ? key0 + kr : a.KV - 1;      // rows past the end repeat the last key; their scores are masked
            const u32x4 * kp = (const u32x4 *)(kb + key * a.k_nb1 + kc * 2);
            const u32x4 * vp = (const u32x4 *)(vb + key * a.v_nb1 + kc * 2);
            kreg0 = kp[0]; kreg1 = kp[1]; vreg0 = vp[0]; vreg1 = vp[1];
        };
        load_kv(0);
        *(u32x4 *)(k_s + kr * T_LDH + kc) = kreg0; *(u32x4 *)(k_s + kr * T_LDH + kc + 8) = kreg1;

        for (int it = 0; it <= n_tiles; ++it) {
            // tile boundary: buffer it & 1 is free (its chains ended with the previous iteration); the K tile staged at the end
            // of that iteration (and, first time, the Q tile) is visible
            __syncthreads();
            if (it == n_tiles) { __syncthreads(); break; }
            const int64_t key0 = (int64_t) it * T_KV;
            half_t * vs_buf = v_s2 + (it & 1) * T_KV * FA_D;
            float *  fs_buf = f_s2 + (it & 1) * T_Q * T_LDF;
            *(u32x4 *)(vs_buf + kr * FA_D + kc) = vreg0; *(u32x4 *)(vs_buf + kr * FA_D + kc + 8) = vreg1;
            if (it + 1 < n_tiles) load_kv(key0 + T_KV);    // a whole iteration ahead of its use

            // ---- scores: S = Q K^T on the matrix cores
            {
                float16_t c16;
#pragma unroll
                for (int r = 0; r < 16; ++r) c16[r] = 0.0f;
#pragma unroll
                for (int kk = 0; kk < FA_D / 16; ++kk) {
                    const half8_t av = *(const half8_t *)(q_s + (sq + l32) * T_LDH + kk * 16 + 8 * g);
                    const half8_t bv = *(const half8_t *)(k_s + (sk + l32) * T_LDH + kk * 16 + 8 * g);
                    c16 = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, bv, c16, 0, 0, 0);
                }
                const int64_t key = key0 + sk + l32;                  // accumulator column = key, rows = queries
                const bool key_ok = key < a.KV;
                if (!a.mask && key0 + T_KV <= a.KV) {
                    // no mask and every key of the tile exists (all but the last tile of an encoder layer): the score is the product
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int qi = sq + 8 * (r >> 2) + 4 * g + (r & 3);
                        fs_buf[qi * T_LDF + sk + l32] = __fmul_rn(c16[r], a.scale);
                    }
                } else {
                float mv[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int qi = sq + 8 * (r >> 2) + 4 * g + (r & 3);
                    mv[r] = 0.0f;
                    if (a.mask) {
                        const int64_t n = n0 + qi < a.N ? n0 + qi : a.N - 1;
                        mv[r] = (float) *(const half_t *)(a.mask + n * a.m_nb1 + (key_ok ? key : a.KV - 1) * 2);
                    }
                }
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int qi = sq + 8 * (r >> 2) + 4 * g + (r & 3);
                    fs_buf[qi * T_LDF + sk + l32] = key_ok ? __fadd_rn(__fmul_rn(c16[r], a.scale), mv[r]) : -INFINITY;
                }
                }
            }
            __syncthreads();                               // scores visible

            // ---- factors: thread t: query t/4, keys 16*(t%4) .. +15
            {
                const int qi = tid >> 2, sgm = tid & 3;
                float4 * fp = (float4 *)(fs_buf + qi * T_LDF + sgm * 16);
                float sv[16], lmax = -INFINITY;
#pragma unroll
                for (int i = 0; i < 4; ++i) { const float4 t = fp[i]; sv[4*i] = t.x; sv[4*i+1] = t.y; sv[4*i+2] = t.z; sv[4*i+3] = t.w; }
#pragma unroll
                for (int i = 0; i < 16; ++i) lmax = fmaxf(lmax, sv[i]);
                float M = m_run[qi];
                const float S0 = s_run[qi];
                // (the four runs of a query sit in one quad of lanes: broadcasts inside it are DPP moves, not LDS permutes)
                const float m0 = dpp_move<float, 0x00>(lmax), m1 = dpp_move<float, 0x55>(lmax), m2 = dpp_move<float, 0xAA>(lmax);
                if (sgm > 0) M = fmaxf(M, m0);
                if (sgm > 1) M = fmaxf(M, m1);
                if (sgm > 2) M = fmaxf(M, m2);
                // this run's effect on the softmax denominator: S_after = S_before * P + A
                float P = 1.0f, A = 0.0f;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    // one exp serves both cases: a new maximum (ms = exp(M - s), 0 for the first key; vs = 1) and a standing
                    // one (vs = exp(s - M); masked keys, s = -inf, get vs = 0, a no-op on the accumulator)
                    const float s = sv[i];
                    const bool  raised = s > M;
                    const float ex = exp_neg(-fabsf(s - M));   // M - s when raised, s - M otherwise: both <= 0 (or NaN / -inf: 0)
                    if (__any(raised)) {
                        const float ms = raised ? ex : 1.0f, vs = raised ? 1.0f : ex;
                        M = raised ? s : M;
                        P *= ms; A = A * ms + vs;
                        sv[i] = raised ? -ex : ex;             // -0.0 keeps the sign
                    } else {
                        // no query of this wavefront has a new maximum at this key (nine keys in ten, past the first tiles):
                        // ms = 1 leaves M and P as they are and A * 1 + vs is A + vs, bit for bit
                        A = A + ex;
                        sv[i] = ex;
                    }
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) fp[i] = make_float4(sv[4*i], sv[4*i+1], sv[4*i+2], sv[4*i+3]);
                // fold the four runs of this query in key order
                const float P1 = dpp_move<float, 0x55>(P), A1 = dpp_move<float, 0x55>(A);
                const float P2 = dpp_move<float, 0xAA>(P), A2 = dpp_move<float, 0xAA>(A);
                const float P3 = dpp_move<float, 0xFF>(P), A3 = dpp_move<float, 0xFF>(A);
                const float M3 = dpp_move<float, 0xFF>(M);
                if (sgm == 0) {
                    float S = S0 * P + A;
                    S = S * P1 + A1; S = S * P2 + A2; S = S * P3 + A3;
                    s_run[qi] = S; m_run[qi] = M3;
                }
            }
            // the next tile's K rows: every wavefront's matrix instructions over this tile's are behind the barrier above
            if (it + 1 < n_tiles) { *(u32x4 *)(k_s + kr * T_LDH + kc) = kreg0; *(u32x4 *)(k_s + kr * T_LDH + kc + 8) = kreg1; }
        }
        return;
    }

    // ---- chains: the sequential f16 accumulation, tile by tile ------------------------------------------------------------------------
    // A lane owns 16 of the 64 d of one query.  A wavefront takes 16 queries x all four d slices: a key that raises the running
    // maximum of any query of the wavefront costs the whole wavefront a rescale of its accumulators, and with 16 queries
    // instead of 64 that happens for 6 % of the keys instead of 18 % (records of an i.i.d. sequence: about
    // min(1, queries / k) at key k).
    // The chains are what the kernel's time consists of; the producers only have to be done a tile ahead.  With the four
    // wavefronts of a SIMD at equal priority the arbiter hands the producers a quarter of the issue slots whenever they
    // are ready, and the chains arrive late at the tile boundary: 197 us per launch; chains first, 190.  (Producers first: 214.)
    __builtin_amdgcn_s_setprio(1);
    const int cq = 16 * wave + (lane & 15);
    const int d0 = (lane >> 4) * 16;
    half2_t acc2[8];                                       // 16 f16 accumulators, two per register
#pragma unroll
    for (int e = 0; e < 8; ++e) acc2[e] = (half2_t){ (half_t) 0.0f, (half_t) 0.0f };

    for (int it = 0; it <= n_tiles; ++it) {
        __syncthreads();                                   // tile boundary: tile it - 1 has its factors and its V rows
        int barriers = 0;                                  // the meeting point inside an iteration, wherever the keys end
        if (it > 0) {
            const int64_t key0 = (int64_t)(it - 1) * T_KV;
            const int nk = (int)(a.KV - key0 < T_KV ? a.KV - key0 : T_KV);       // uniform
            const float4 * fp = (const float4 *)(f_s2 + ((it - 1) & 1) * T_Q * T_LDF + cq * T_LDF);
            const u32x4 * vp = (const u32x4 *)(v_s2 + ((it - 1) & 1) * T_KV * FA_D + d0);      // + key * FA_D halves = 8 of these
            // one group = four keys: their factors (one b128 read) and their V values (two broadcast b128 reads per key);
            // the next group is read while this one is consumed
            // (Keys of the tile past the last one carry a factor of exactly 0 — their scores are -inf — and finite V values,
            // the last key's: walking them leaves every accumulator as it is, so groups are walked whole and the code has no
            // per-key bounds.)
            struct group { float4 f; u32x4 v[4][2]; };
            auto gload = [&](group & gr, int k4) __attribute__((always_inline)) {
                gr.f = fp[k4 >> 2];
#pragma unroll
                for (int j = 0; j < 4; ++j) { gr.v[j][0] = vp[(k4 + j) * 8]; gr.v[j][1] = vp[(k4 + j) * 8 + 1]; }
            };
            auto chain4 = [&](const group & gr) __attribute__((always_inline)) {
                const float fk[4] = { gr.f.x, gr.f.y, gr.f.z, gr.f.w };
                const uint32_t sign = (__float_as_uint(fk[0]) | __float_as_uint(fk[1]) | __float_as_uint(fk[2]) | __float_as_uint(fk[3])) >> 31;
                if (__any(sign)) {                         // some query's maximum moved within these keys: rescale its accumulators
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const bool raised = __float_as_uint(fk[j]) >> 31;
                        const float ms = raised ? -fk[j] : 1.0f, vs = raised ? 1.0f : fk[j];
                        if (__any(raised)) seq_scale16(acc2, ms);          // ms == 1 leaves the value as it is
                        seq_mad16(acc2, gr.v[j][0], gr.v[j][1], vs);
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j) seq_mad16(acc2, gr.v[j][0], gr.v[j][1], fk[j]);
                }
            };
            // arrived(): first use of a group, placed before the next group's reads are issued, so that the wait it
            // implies only covers reads that have had four keys' worth of time
            auto arrived = [&](const group & gr) __attribute__((always_inline)) {
                asm volatile("" :: "v"(gr.f.x), "v"(gr.v[3][1]));
                __builtin_amdgcn_sched_barrier(0);
            };
            group ga, gb;
            gload(ga, 0);
            const int nk8 = (nk + 7) & ~7;                 // whole pairs of groups (a tile holds 64 keys' worth of factors and rows)
            for (int k4 = 0; k4 < nk8; k4 += 8) {
                arrived(ga);
                gload(gb, k4 + 4);
                __builtin_amdgcn_sched_barrier(0);
                chain4(ga);
                arrived(gb);
                gload(ga, k4 + 8 < T_KV ? k4 + 8 : 0);     // (behind the last group: any readable group, nobody walks it)
                __builtin_amdgcn_sched_barrier(0);
                chain4(gb);
                // the producers' meeting point: after 16 keys their scores are written; the other 48 keys are the time their
                // factor step has
                if (k4 == 8) { __syncthreads(); ++barriers; }
            }
        }
        for (; barriers < 1; ++barriers) __syncthreads();
    }

    const int64_t n = n0 + cq;
    float o[16];
    {
        const float inv = 1.0f / s_run[cq];
#pragma unroll
        for (int i = 0; i < 8; ++i) { o[2*i] = (float) acc2[i][0] * inv; o[2*i + 1] = (float) acc2[i][1] * inv; }
    }
    if (a.d && n < a.N) {                                  // (no dst: the caller reads the image below and nothing else)
        float * dp = (float *) a.d + ((i3 * a.N + n) * a.H + h) * FA_D + d0;
#pragma unroll
        for (int i = 0; i < 4; ++i) *(float4 *)(dp + 4 * i) = make_float4(o[4*i], o[4*i + 1], o[4*i + 2], o[4*i + 3]);
    }
    if (a.x16) {
        // The projection that follows rounds these rows to Q8_0 (blocks of 32 along d: two wavefronts' slices of a query)
        // before multiplying; write that image — f16(q * d), as quantize_row_q8_0 would produce q and d — here, so that it
        // needs no pass of its own over the attention output.
        float amax = 0.0f;
#pragma unroll
        for (int e = 0; e < 16; ++e) amax = fmaxf(amax, fabsf(o[e]));
        // (the other half of the block is in lane ^ 16)
        amax = fmaxf(amax, __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, amax), 0x401F)));
        if (n < a.N) {
            const float id = amax != 0.0f ? 127.0f / amax : 0.0f;
            const float dq = h2f(f2h_bits(div127(amax)));
            half8_t h0, h1;
#pragma unroll
            for (int e = 0; e < 8; ++e) { h0[e] = (half_t)((rintf(o[e] * id) + 0.0f) * dq); h1[e] = (half_t)((rintf(o[8 + e] * id) + 0.0f) * dq); }
            half8_t * xp = (half8_t *)(a.x16 + ((i3 * a.N + n) * a.H + h) * FA_D + d0);
            xp[0] = h0; xp[1] = h1;
        }
    }
}

// ------------------------------------------------------------------------------------------------------
// k_fattn_pk_tile: the tile kernel for the packed-f16 form of the step (MI355X_FA_F16_PK).
//
// Same roles, tiles and barriers as k_fattn_seq_tile.  With 8 instead of 24 vector instructions per key the chains of
// that kernel's layout (a lane = one query x 16 d, every lane reading the key's 32 bytes of V) are bound by the LDS
// reads, not by the vector units: a V register that arrives serves one instruction.  Here a lane owns 4 queries x 4 d
// (lane = query quad l / 16 of the wavefront's 16 queries, d slice l % 16), so a key costs it one 8-byte read of V for
// 8 instructions, and the factors arrive as f16, two keys to a register and the four queries of the quad side by side:
// one 16-byte read per pair of keys.  Per key and lane 12 bytes from LDS instead of 36.
//   factor tile  fp[key pair][query ^ swizzle]: 32 rows of 64 registers, each register the factors of keys 2 p, 2 p + 1
//                for one query (vs, or -ms where the key raises that query's maximum); the producers' thread (query,
//                16-key run) writes a column piece of 8, and the swizzle (bit 4 of the query index flipped in the rows
//                of odd runs) spreads a wavefront's 64 writes over all banks twice instead of 16 banks four times
//   raise masks  per chain wavefront and tile 64 bits: does key k raise the maximum of any of its 16 queries?  Built
//                by the producer wavefront that has the same 16 queries; the chain tests them with scalar
//                instructions, so a pair of keys without a raise costs its 16 multiply-adds and nothing else.
// ------------------------------------------------------------------------------------------------------

#define P_FP_ROW   T_Q                                    // registers per key-pair row of the factor tile
#define P_FP_TILE  ((T_KV / 2) * P_FP_ROW)
#define P_LDS_BYTES ((T_Q * T_LDH + T_KV * T_LDH + 2 * T_KV * FA_D) * 2 + T_Q * T_LDF * 4 + 2 * P_FP_TILE * 4 + 2 * 4 * 2 * 4 + 2 * T_Q * 4)   // 69184

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// The factor step of a run of 16 scores, written out: s[i] becomes its factor (negated where key i raises the row's maximum),
// M the running maximum, (P, A) the run's part of the denominator (S_after = S_before * P + A), bit i of `bits` the raise.
// The common key raises no maximum in the whole wavefront (85 % of the keys of the encoder's launches) and takes the
// straight path — test, difference, exponential, sum and a branch not taken; a raise anywhere in the wavefront sends it
// through the general form at the end of the block and back.  As C++ the same loop met after every key in a join
// for which the compiler copied three to five registers, on the straight path too: nine vector instructions and two taken
// branches per key.  (The s_nop behind v_exp_f32 is the wait state its result needs in front of a vector instruction.)
// The factor is 2^-|s - M|: 2^(s - M), or 2^(M - s) where s raises the maximum.  M starts at PKT_M_START, a finite number
// below every score, so that the difference is never (-inf) - (-inf): a masked key (s = -inf) gives -inf and the factor 0
// whatever was seen before it, the first real key of a row raises the maximum with the factor 2^-huge = 0, as with -inf.
#define PKT_M_START (-3.0e38f)
#define PKT_KEY(i) \
    "v_cmp_gt_f32 vcc, %[s" #i "], %[M]\n" \
    "v_sub_f32 %[t], %[s" #i "], %[M]\n" \
    "s_cbranch_vccnz 1" #i "f\n" \
    "v_exp_f32_e64 %[s" #i "], -|%[t]|\n" \
    "s_nop 0\n" \
    "v_add_f32 %[A], %[A], %[s" #i "]\n" \
    "2" #i ":\n"
#define PKT_RAISE(i) \
    "1" #i ":\n" \
    "v_max_f32 %[M], %[M], %[s" #i "]\n" \
    "v_exp_f32_e64 %[ex], -|%[t]|\n" \
    "s_nop 0\n" \
    "v_cndmask_b32_e64 %[ms], 1.0, %[ex], vcc\n" \
    "v_cndmask_b32_e64 %[vs], %[ex], 1.0, vcc\n" \
    "v_mul_f32 %[P], %[P], %[ms]\n" \
    "v_fma_f32 %[A], %[A], %[ms], %[vs]\n" \
    "v_cndmask_b32_e64 %[s" #i "], %[ex], -%[ex], vcc\n" \
    "v_cndmask_b32_e64 %[ms], 0, 1, vcc\n" \
    "v_lshl_or_b32 %[bits], %[ms], " #i ", %[bits]\n" \
    "s_branch 2" #i "b\n"
__device__ __forceinline__ void pkt_factor_run(float (&sv)[16], float & M, float & P, float & A, uint32_t & bits) {
    float t, ex, ms, vs;
    asm volatile(
        PKT_KEY(0) PKT_KEY(1) PKT_KEY(2) PKT_KEY(3) PKT_KEY(4) PKT_KEY(5) PKT_KEY(6) PKT_KEY(7)
        PKT_KEY(8) PKT_KEY(9) PKT_KEY(10) PKT_KEY(11) PKT_KEY(12) PKT_KEY(13) PKT_KEY(14) PKT_KEY(15)
        "s_branch 3f\n"
        PKT_RAISE(0) PKT_RAISE(1) PKT_RAISE(2) PKT_RAISE(3) PKT_RAISE(4) PKT_RAISE(5) PKT_RAISE(6) PKT_RAISE(7)
        PKT_RAISE(8) PKT_RAISE(9) PKT_RAISE(10) PKT_RAISE(11) PKT_RAISE(12) PKT_RAISE(13) PKT_RAISE(14) PKT_RAISE(15)
        "3:\n"
        : [s0] "+v"(sv[0]), [s1] "+v"(sv[1]), [s2] "+v"(sv[2]), [s3] "+v"(sv[3]), [s4] "+v"(sv[4]), [s5] "+v"(sv[5]), [s6] "+v"(sv[6]), [s7] "+v"(sv[7]),
          [s8] "+v"(sv[8]), [s9] "+v"(sv[9]), [s10] "+v"(sv[10]), [s11] "+v"(sv[11]), [s12] "+v"(sv[12]), [s13] "+v"(sv[13]), [s14] "+v"(sv[14]), [s15] "+v"(sv[15]),
          [M] "+v"(M), [P] "+v"(P), [A] "+v"(A), [bits] "+v"(bits), [t] "=&v"(t), [ex] "=&v"(ex), [ms] "=&v"(ms), [vs] "=&v"(vs)
        : : "vcc");
}

__global__ void __launch_bounds__(512, 2) k_fattn_pk_tile(fa_args a) {
    extern __shared__ __attribute__((aligned(16))) char t_smem[];
    half_t *   q_s  = (half_t *) t_smem;                      // [T_Q * T_LDH]
    half_t *   k_s  = q_s + T_Q * T_LDH;                      // [T_KV * T_LDH]
    half_t *   v_s2 = k_s + T_KV * T_LDH;                     // [2][T_KV * FA_D]
    float *    sc_s = (float *)(v_s2 + 2 * T_KV * FA_D);      // [T_Q * T_LDF]   scores of the tile in work (producers only)
    uint32_t * fp_s = (uint32_t *)(sc_s + T_Q * T_LDF);       // [2][P_FP_TILE]
    uint32_t * rm_s = fp_s + 2 * P_FP_TILE;                   // [2][4][2]
    float *    m_run = (float *)(rm_s + 16), * s_run = m_run + T_Q;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // an XCD gets one run of consecutive (head, query tile) pairs, head-major, so that a head's K and V stay in one or two L2s
    const uint32_t lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z), total = gridDim.x * gridDim.y * gridDim.z;
    const uint32_t xcd = lin % 8, per = total / 8, extra = total % 8;
    const uint32_t item = xcd * per + (xcd < extra ? xcd : extra) + lin / 8;
    const int64_t n0 = (int64_t)(item % gridDim.x) * T_Q, h = (item / gridDim.x) % gridDim.y, i3 = item / (gridDim.x * gridDim.y);
    const int n_tiles = (int)((a.KV + T_KV - 1) / T_KV);

    if (wave >= 4) {
        // ---- producers ---------------------------------------------------------------------------------------------------------------
        const int tid = threadIdx.x - 256, pw = wave - 4;
        const char * qb = a.q + h * a.q_nb2 + i3 * a.q_nb3;
        const char * kb = a.k + (h / a.hk_ratio) * a.k_nb2 + (i3 / a.k_ne3_ratio) * a.k_nb3;
        const char * vb = a.v + (h / a.hv_ratio) * a.v_nb2 + (i3 / a.v_ne3_ratio) * a.v_nb3;
        {   // Q tile -> f16 in LDS; thread t: row t/4, 16 values
            const int r = tid >> 2, c = (tid & 3) * 16;
            const int64_t n = n0 + r;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
                if (n < a.N) t = *(const float4 *)(qb + n * a.q_nb1 + (c + 4 * i) * 4);
                half4_t hq = { (half_t) t.x, (half_t) t.y, (half_t) t.z, (half_t) t.w };
                *(half4_t *)(q_s + r * T_LDH + c + 4 * i) = hq;
            }
        }
        if (tid < T_Q) { m_run[tid] = PKT_M_START; s_run[tid] = 0.0f; }

        const int sq = (pw >> 1) * 32, sk = (pw & 1) * 32, l32 = lane & 31, g = lane >> 5;
        const int kr = tid >> 2, kc = (tid & 3) * 16;
        const float scale2 = a.scale * LOG2E_F;
        u32x4 kreg0, kreg1, vreg0, vreg1;
        auto load_kv = [&](int64_t key0) __attribute__((always_inline)) {
            const int64_t key = key0 + kr < a.KV ? key0 + kr : a.KV - 1;      // rows past the end repeat the last key; their scores are masked
            const u32x4 * kp = (const u32x4 *)(kb + key * a.k_nb1 + kc * 2);
            const u32x4 * vp = (const u32x4 *)(vb + key * a.v_nb1 + kc * 2);
            kreg0 = kp[0]; kreg1 = kp[1]; vreg0 = vp[0]; vreg1 = vp[1];
        };
        load_kv(0);
        *(u32x4 *)(k_s + kr * T_LDH + kc) = kreg0; *(u32x4 *)(k_s + kr * T_LDH + kc + 8) = kreg1;

        for (int it = 0; it <= n_tiles; ++it) {
            __syncthreads();                               // tile boundary
            if (it == n_tiles) { __syncthreads(); break; }
            const int64_t key0 = (int64_t) it * T_KV;
            half_t * vs_buf = v_s2 + (it & 1) * T_KV * FA_D;
            *(u32x4 *)(vs_buf + kr * FA_D + kc) = vreg0; *(u32x4 *)(vs_buf + kr * FA_D + kc + 8) = vreg1;
            if (it + 1 < n_tiles) load_kv(key0 + T_KV);

            {   // ---- scores: S = Q K^T on the matrix cores
                float16_t c16;
#pragma unroll
                for (int r = 0; r < 16; ++r) c16[r] = 0.0f;
#pragma unroll
                for (int kk = 0; kk < FA_D / 16; ++kk) {
                    const half8_t av = *(const half8_t *)(q_s + (sq + l32) * T_LDH + kk * 16 + 8 * g);
                    const half8_t bv = *(const half8_t *)(k_s + (sk + l32) * T_LDH + kk * 16 + 8 * g);
                    c16 = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, bv, c16, 0, 0, 0);
                }
                const int64_t key = key0 + sk + l32;
                const bool key_ok = key < a.KV;
                // (scores are kept in units of log2 e: the factors are then one v_exp_f32 each)
                if (!a.mask && key0 + T_KV <= a.KV) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int qi = sq + 8 * (r >> 2) + 4 * g + (r & 3);
                        sc_s[qi * T_LDF + sk + l32] = __fmul_rn(c16[r], scale2);
                    }
                } else {
                    float mv[16];
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int qi = sq + 8 * (r >> 2) + 4 * g + (r & 3);
                        mv[r] = 0.0f;
                        if (a.mask) {
                            const int64_t n = n0 + qi < a.N ? n0 + qi : a.N - 1;
                            mv[r] = (float) *(const half_t *)(a.mask + n * a.m_nb1 + (key_ok ? key : a.KV - 1) * 2);
                        }
                    }
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int qi = sq + 8 * (r >> 2) + 4 * g + (r & 3);
                        sc_s[qi * T_LDF + sk + l32] = key_ok ? __builtin_fmaf(c16[r], scale2, mv[r] * LOG2E_F) : -INFINITY;
                    }
                }
            }
            __syncthreads();                               // scores visible

            {   // ---- factors: thread t: query t/4, keys 16*(t%4) .. +15
                const int qi = tid >> 2, sgm = tid & 3;
                const float4 * sp = (const float4 *)(sc_s + qi * T_LDF + sgm * 16);
                float sv[16], lmax = -INFINITY;
#pragma unroll
                for (int i = 0; i < 4; ++i) { const float4 t = sp[i]; sv[4*i] = t.x; sv[4*i+1] = t.y; sv[4*i+2] = t.z; sv[4*i+3] = t.w; }
#pragma unroll
                for (int i = 0; i < 16; ++i) lmax = fmaxf(lmax, sv[i]);
                float M = m_run[qi];
                const float S0 = s_run[qi];
                const float m0 = dpp_move<float, 0x00>(lmax), m1 = dpp_move<float, 0x55>(lmax), m2 = dpp_move<float, 0xAA>(lmax);
                if (sgm > 0) M = fmaxf(M, m0);
                if (sgm > 1) M = fmaxf(M, m1);
                if (sgm > 2) M = fmaxf(M, m2);
                float P = 1.0f, A = 0.0f;
                uint32_t rbits = 0;                        // bit i: key i of this run raises this query's maximum
                // sv[i] -> 2^(s - M), or -2^(M - s) where key i raises the maximum (-0.0 keeps the sign)
                pkt_factor_run(sv, M, P, A, rbits);
                // f16 factors, two keys to a register, into column (query ^ swizzle) of this run's eight key-pair rows
                uint32_t * fpw = fp_s + (it & 1) * P_FP_TILE + (8 * sgm) * P_FP_ROW + (qi ^ ((sgm & 1) << 4));
#pragma unroll
                for (int j = 0; j < 8; ++j) fpw[j * P_FP_ROW] = pk_factors(sv[2*j], sv[2*j + 1]);
                // the raise mask of the wavefront's 16 queries: OR over the lanes of a run (lane = 4 * query + run)
                rbits |= dpp_move<uint32_t, 0x124>(rbits);     // row_ror:4
                rbits |= dpp_move<uint32_t, 0x128>(rbits);     // row_ror:8
                rbits |= (uint32_t) __builtin_amdgcn_ds_swizzle((int) rbits, 0x401F);       // lane ^ 16
                rbits |= (uint32_t) __shfl_xor((int) rbits, 32, WAVE);
                const uint32_t r1 = dpp_move<uint32_t, 0x55>(rbits), r2 = dpp_move<uint32_t, 0xAA>(rbits), r3 = dpp_move<uint32_t, 0xFF>(rbits);
                if (lane == 0) *(u32x2 *)(rm_s + ((it & 1) * 4 + pw) * 2) = (u32x2){ rbits | (r1 << 16), r2 | (r3 << 16) };
                // fold the four runs of this query in key order
                const float P1 = dpp_move<float, 0x55>(P), A1 = dpp_move<float, 0x55>(A);
                const float P2 = dpp_move<float, 0xAA>(P), A2 = dpp_move<float, 0xAA>(A);
                const float P3 = dpp_move<float, 0xFF>(P), A3 = dpp_move<float, 0xFF>(A);
                const float M3 = dpp_move<float, 0xFF>(M);
                if (sgm == 0) {
                    float S = S0 * P + A;
                    S = S * P1 + A1; S = S * P2 + A2; S = S * P3 + A3;
                    s_run[qi] = S; m_run[qi] = M3;
                }
            }
            if (it + 1 < n_tiles) { *(u32x4 *)(k_s + kr * T_LDH + kc) = kreg0; *(u32x4 *)(k_s + kr * T_LDH + kc + 8) = kreg1; }
        }
        return;
    }

    // ---- chains: lane = (query quad qd, d slice ds) of the wavefront's 16 queries ----------------------------------------------------
    __builtin_amdgcn_s_setprio(1);
    const int qd = lane >> 4, ds = lane & 15;
    half2_t acc[8];                                        // acc[2 q + j]: d pair j of the quad's query q
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = (half2_t){ (half_t) 0.0f, (half_t) 0.0f };
    const int fcol = 16 * wave + 4 * qd;

    for (int it = 0; it <= n_tiles; ++it) {
        __syncthreads();                                   // tile boundary: tile it - 1 has its factors, its masks and its V rows
        int barriers = 0;
        if (it > 0) {
            const int64_t key0 = (int64_t)(it - 1) * T_KV;
            const int nk = (int)(a.KV - key0 < T_KV ? a.KV - key0 : T_KV);       // uniform
            const int buf = (it - 1) & 1;
            const uint32_t * fpb = fp_s + buf * P_FP_TILE;
            const char * vbase = (const char *)(v_s2 + buf * T_KV * FA_D) + 8 * ds;     // + key * 128
            const u32x2 mv = *(const u32x2 *)(rm_s + (buf * 4 + wave) * 2);
            const uint32_t mlo = __builtin_amdgcn_readfirstlane(mv.x), mhi = __builtin_amdgcn_readfirstlane(mv.y);
            // one group = four pairs of keys: their factors (a 16-byte read per pair) and their V values (an 8-byte read per key);
            // the next group is read while this one is walked.  (Keys past the end carry factors of exactly 0 and the last
            // key's finite V values: walking them changes nothing, so groups are walked whole.)
            struct pgroup { u32x4 f[4]; u32x2 v[8]; };
            auto gload = [&](pgroup & gr, int kp0, int swz) __attribute__((always_inline)) {
#pragma unroll
                for (int j = 0; j < 4; ++j) gr.f[j] = *(const u32x4 *)(fpb + (kp0 + j) * P_FP_ROW + (fcol ^ swz));
#pragma unroll
                for (int j = 0; j < 8; ++j) gr.v[j] = *(const u32x2 *)(vbase + (2 * kp0 + j) * (FA_D * 2));
            };
            // bits: two per pair of keys, lowest first: does the first / the second key of the pair raise a maximum in this wavefront.
            // Only the rescale sits behind the (scalar) test; the multiply-adds are the same instructions on either path.
            auto walk = [&](pgroup & gr, uint32_t bits) __attribute__((always_inline)) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (bits & (1u << (2*j))) pk_rescale<0>(acc, gr.f[j]);
                    pk_mad8<0>(acc, gr.v[2*j].x, gr.v[2*j].y, gr.f[j]);
                    if (bits & (2u << (2*j))) pk_rescale<1>(acc, gr.f[j]);
                    pk_mad8<1>(acc, gr.v[2*j + 1].x, gr.v[2*j + 1].y, gr.f[j]);
                }
            };
            auto arrived = [&](const pgroup & gr) __attribute__((always_inline)) {
                asm volatile("" :: "v"(gr.f[3].w), "v"(gr.v[7].y));
                __builtin_amdgcn_sched_barrier(0);
            };
            pgroup ga, gb;
            gload(ga, 0, 0);
            const int n_runs = (nk + 15) >> 4;             // runs of 16 keys = 8 pairs = two groups
            for (int u = 0; u < n_runs; ++u) {
                const uint32_t fld = ((u & 2) ? mhi : mlo) >> (16 * (u & 1));
                const int swz = (u & 1) << 4;
                arrived(ga);
                gload(gb, 8 * u + 4, swz);
                __builtin_amdgcn_sched_barrier(0);
                walk(ga, fld & 0xffu);
                arrived(gb);
                gload(ga, u < 3 ? 8 * u + 8 : 0, u < 3 ? swz ^ 16 : 0);     // (behind the last group: any readable group, nobody walks it)
                __builtin_amdgcn_sched_barrier(0);
                walk(gb, (fld >> 8) & 0xffu);
                // the producers' meeting point: after 16 keys their scores are written; the other 48 keys are the time their
                // factor step has
                if (u == 0) { __syncthreads(); ++barriers; }
            }
        }
        for (; barriers < 1; ++barriers) __syncthreads();
    }

    // ---- results: a lane holds 4 d of 4 queries
    const int64_t nq0 = n0 + 16 * wave + 4 * qd;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int64_t n = nq0 + q;
        const float inv = 1.0f / s_run[16 * wave + 4 * qd + q];
        const float o[4] = { (float) acc[2*q][0] * inv, (float) acc[2*q][1] * inv, (float) acc[2*q + 1][0] * inv, (float) acc[2*q + 1][1] * inv };
        if (a.d && n < a.N) *(float4 *)((float *) a.d + ((i3 * a.N + n) * a.H + h) * FA_D + 4 * ds) = make_float4(o[0], o[1], o[2], o[3]);
        if (a.x16) {
            // the Q8_0-rounded f16 image of the row for the projection that follows: a block is 32 d, eight lanes of a row
            float amax = fmaxf(fmaxf(fabsf(o[0]), fabsf(o[1])), fmaxf(fabsf(o[2]), fabsf(o[3])));
            amax = lanes_max<8>(amax);
            if (n < a.N) {
                const float id = amax != 0.0f ? 127.0f / amax : 0.0f;
                const float dq = h2f(f2h_bits(div127(amax)));
                half4_t hx;
#pragma unroll
                for (int e = 0; e < 4; ++e) hx[e] = (half_t)((rintf(o[e] * id) + 0.0f) * dq);
                *(half4_t *)(a.x16 + ((i3 * a.N + n) * a.H + h) * FA_D + 4 * ds) = hx;
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------------
// N > 8, f32 accumulators on the matrix cores (MI355X_FA_F32).
//
// Both products run on v_mfma_f32_32x32x16_f16, transposed so that a lane owns one query throughout:
//   S^T = K Q^T     (32 keys x 32 queries per wavefront; Q^T is the B operand and stays in registers for the whole kernel)
//   O^T += V^T P^T  (64 d x 32 queries; P^T = exp2(S^T - m) leaves the accumulator registers of the first product in the
//                    very lanes that need it as the B operand of the second, once the keys of a block are visited in the
//                    order those registers hold them — the V^T operand is read from LDS in the same order)
// so the running maximum and sum are per-lane scalars (one exchange with lane ^ 32 per tile) and the rescale of O is a
// per-lane multiply.  A workgroup is 64 queries of one head; wavefront w takes queries 32 * (w / 2) and the keys
// 32 * (w % 2) .. + 31 of each 64-key tile with a softmax state of its own, and the two states of a query are merged at
// the end.  K tiles go to LDS as they are; V tiles are transposed on the way in (two keys packed per 32-bit store), both
// double buffered with the next tile's global loads in flight.
// ------------------------------------------------------------------------------------------------------

#define M_Q   64
#define M_KV  64
#define M_LDK (FA_D + 8)      // f16 pitch of a K row
#define M_LDV (M_KV + 4)      // f16 pitch of a V^T row (136 B: the b64 operand reads of 32 d-rows cover all banks once)
#define LOG2E 1.44269504088896340736f

__global__ void __launch_bounds__(256) k_fattn_mfma(fa_args a) {
    __shared__ __attribute__((aligned(16))) half_t k_s[2][M_KV * M_LDK];
    __shared__ __attribute__((aligned(16))) half_t vt_s[2][FA_D * M_LDV];

    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wq = (wave >> 1) * 32, wk = (wave & 1) * 32;
    const int64_t n0 = (int64_t) blockIdx.x * M_Q, h = blockIdx.y, i3 = blockIdx.z;
    const char * qb = a.q + h * a.q_nb2 + i3 * a.q_nb3;
    const char * kb = a.k + (h / a.hk_ratio) * a.k_nb2 + (i3 / a.k_ne3_ratio) * a.k_nb3;
    const char * vb = a.v + (h / a.hv_ratio) * a.v_nb2 + (i3 / a.v_ne3_ratio) * a.v_nb3;

    // B operand of the first product: lane (query l32, half g) holds q[16 kk + 8 g .. + 7], rounded to f16 as the CPU backend does
    const int64_t n  = n0 + wq + l32;
    const int64_t nc = n < a.N ? n : a.N - 1;
    half8_t qf[FA_D / 16];
    {
        const float * qp = (const float *)(qb + nc * a.q_nb1);
#pragma unroll
        for (int kk = 0; kk < FA_D / 16; ++kk) {
            const float4 t0 = *(const float4 *)(qp + 16 * kk + 8 * g), t1 = *(const float4 *)(qp + 16 * kk + 8 * g + 4);
            qf[kk] = (half8_t){ (half_t) t0.x, (half_t) t0.y, (half_t) t0.z, (half_t) t0.w, (half_t) t1.x, (half_t) t1.y, (half_t) t1.z, (half_t) t1.w };
        }
    }
    const half_t * mrow = a.mask ? (const half_t *)(a.mask + nc * a.m_nb1) : nullptr;
    const bool mask_al8 = (((uintptr_t) a.mask | (uintptr_t) a.m_nb1) & 7) == 0;      // rows of the mask can be read four keys at a time

    // staging roles: K: thread t -> key t / 4, 32 bytes; V: thread t -> keys 2 (t / 8) and + 1, d 8 (t % 8) .. + 7
    const int kr = tid >> 2, kc = (tid & 3) * 16;
    const int vp = tid >> 3, vc = (tid & 7) * 8;
    u32x4 kreg0, kreg1, vreg0, vreg1;
    auto load_kv = [&](int64_t key0) __attribute__((always_inline)) {
        const int64_t last = a.KV - 1;                    // rows past the end repeat the last key; their scores are masked
        const int64_t kk = key0 + kr < last ? key0 + kr : last;
        const int64_t v0 = key0 + 2 * vp < last ? key0 + 2 * vp : last, v1 = key0 + 2 * vp + 1 < last ? key0 + 2 * vp + 1 : last;
        const u32x4 * kp = (const u32x4 *)(kb + kk * a.k_nb1 + kc * 2);
        kreg0 = kp[0]; kreg1 = kp[1];
        vreg0 = *(const u32x4 *)(vb + v0 * a.v_nb1 + vc * 2);
        vreg1 = *(const u32x4 *)(vb + v1 * a.v_nb1 + vc * 2);
    };
    auto store_kv = [&](int b) __attribute__((always_inline)) {
        *(u32x4 *)(k_s[b] + kr * M_LDK + kc) = kreg0; *(u32x4 *)(k_s[b] + kr * M_LDK + kc + 8) = kreg1;
        uint32_t * vt = (uint32_t *)(vt_s[b] + vc * M_LDV) + vp;          // V^T[d = vc + j][keys 2 vp, 2 vp + 1]
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            vt[(2 * i    ) * (M_LDV / 2)] = (vreg0[i] & 0xffffu) | (vreg1[i] << 16);
            vt[(2 * i + 1) * (M_LDV / 2)] = (vreg0[i] >> 16) | (vreg1[i] & 0xffff0000u);
        }
    };

    float16_t o[2];
#pragma unroll
    for (int r = 0; r < 16; ++r) { o[0][r] = 0.0f; o[1][r] = 0.0f; }
    float m = -1.0e30f, l = 0.0f;                          // log2 domain; finite so that a fully masked tile gives factors of 0, not NaN
    const float c = a.scale * LOG2E;

    const int nt = (int)((a.KV + M_KV - 1) / M_KV);
    load_kv(0);
    for (int t = 0; t < nt; ++t) {
        const int b = t & 1;
        const int64_t key0 = (int64_t) t * M_KV;
        store_kv(b);
        __syncthreads();                                   // tile t visible; everyone is done with tile t - 1, whose buffer the next store reuses
        if (t + 1 < nt) load_kv(key0 + M_KV);

        float16_t sc;
#pragma unroll
        for (int r = 0; r < 16; ++r) sc[r] = 0.0f;
#pragma unroll
        for (int kk = 0; kk < FA_D / 16; ++kk) {
            const half8_t av = *(const half8_t *)(k_s[b] + (wk + l32) * M_LDK + 16 * kk + 8 * g);
            sc = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, qf[kk], sc, 0, 0, 0);
        }
        // register r: key key0 + wk + 8 (r / 4) + 4 g + r % 4, query l32
        float tv[16];
        if (mrow) {
            half4_t mk[4];
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                const int64_t key = key0 + wk + 8 * q4 + 4 * g;
                if (mask_al8 && key + 3 < a.KV) mk[q4] = *(const half4_t *)(mrow + key);
                else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) mk[q4][e] = mrow[key + e < a.KV ? key + e : a.KV - 1];   // past the end: masked below
                }
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) tv[r] = __builtin_fmaf(sc[r], c, (float) mk[r >> 2][r & 3] * LOG2E);
        } else {
#pragma unroll
            for (int r = 0; r < 16; ++r) tv[r] = sc[r] * c;
        }
        if (key0 + M_KV > a.KV) {
#pragma unroll
            for (int r = 0; r < 16; ++r) if (key0 + wk + 8 * (r >> 2) + 4 * g + (r & 3) >= a.KV) tv[r] = -INFINITY;
        }
        float tmax = tv[0];
#pragma unroll
        for (int r = 1; r < 16; ++r) tmax = fmaxf(tmax, tv[r]);
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, WAVE));
        const float m_new = fmaxf(m, tmax);
        if (__any(m_new > m)) {
            const float alpha = __builtin_amdgcn_exp2f(m - m_new);
            l *= alpha;
#pragma unroll
            for (int r = 0; r < 16; ++r) { o[0][r] *= alpha; o[1][r] *= alpha; }
            m = m_new;
        }
        half8_t ph[2];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const float p = __builtin_amdgcn_exp2f(tv[r] - m);
            l += p;
            ph[r >> 3][r & 7] = (half_t) p;
        }
#pragma unroll
        for (int db = 0; db < 2; ++db) {
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                const half_t * vr = vt_s[b] + (32 * db + l32) * M_LDV + wk + 16 * ks + 4 * g;
                const half4_t lo = *(const half4_t *) vr, hi = *(const half4_t *)(vr + 8);
                const half8_t av = { lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3] };
                o[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, ph[ks], o[db], 0, 0, 0);
            }
        }
    }
    l += __shfl_xor(l, 32, WAVE);

    // merge the two key halves of each query: this wavefront finishes d block (wave & 1) and hands the other block over
    __syncthreads();                                       // the tiles are no longer needed
    float * xch = (float *) k_s;                           // [wave][16][64] f32 = 16 KB of the 18 KB
    float * ml  = (float *) vt_s;                          // [wave][2][64]
    const bool odd = wave & 1;
    const float16_t mine = odd ? o[1] : o[0], send = odd ? o[0] : o[1];
#pragma unroll
    for (int r = 0; r < 16; ++r) xch[(wave * 16 + r) * 64 + lane] = send[r];
    ml[(wave * 2 + 0) * 64 + lane] = m; ml[(wave * 2 + 1) * 64 + lane] = l;
    __syncthreads();
    const int pw = wave ^ 1;
    const float pm = ml[(pw * 2 + 0) * 64 + lane], pl = ml[(pw * 2 + 1) * 64 + lane];
    const float mm = fmaxf(m, pm);
    const float fa = __builtin_amdgcn_exp2f(m - mm), fb = __builtin_amdgcn_exp2f(pm - mm);
    const float inv = 1.0f / (l * fa + pl * fb);
    float out[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) out[r] = (mine[r] * fa + xch[(pw * 16 + r) * 64 + lane] * fb) * inv;

    // out[r]: d = 32 (wave & 1) + 8 (r / 4) + 4 g + r % 4 of query n
    const int64_t row = ((i3 * a.N + n) * a.H + h) * FA_D + 32 * (wave & 1) + 4 * g;
    if (n < a.N) {
        float * dp = (float *) a.d + row;
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) *(float4 *)(dp + 8 * q4) = make_float4(out[4*q4], out[4*q4 + 1], out[4*q4 + 2], out[4*q4 + 3]);
    }
    if (a.x16) {
        // the Q8_0-rounded image for the projection that follows: one block = the 32 d of this wavefront's block of a query,
        // half of them here and half in lane ^ 32
        float amax = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; ++r) amax = fmaxf(amax, fabsf(out[r]));
        amax = fmaxf(amax, __shfl_xor(amax, 32, WAVE));
        if (n < a.N) {
            const float id = amax != 0.0f ? 127.0f / amax : 0.0f;
            const float dq = h2f(f2h_bits(div127(amax)));
            half_t * xp = a.x16 + row;
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                half4_t hv;
#pragma unroll
                for (int e = 0; e < 4; ++e) hv[e] = (half_t)((rintf(out[4*q4 + e] * id) + 0.0f) * dq);
                *(half4_t *)(xp + 8 * q4) = hv;
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------------
// host dispatch
// ------------------------------------------------------------------------------------------------------

#define SEQ_ROW_MAX_N   8

enum { FA_K_VEC = 0, FA_K_SEQ_ROW = 1, FA_K_SEQ_TILE = 2, FA_K_MFMA = 3, FA_K_PK_ROW = 4 };
static inline bool fa_is_row(int kernel) { return kernel == FA_K_SEQ_ROW || kernel == FA_K_PK_ROW; }

// k_fattn_pk_row addresses the rows of a head's K and V with 32-bit offsets
static bool fits_32bit_offsets(const mi355x_tensor * t) { return t->ne[1] > 0 && t->nb[1] > 0 && (uint64_t) t->ne[1] * (uint64_t) t->nb[1] < ((uint64_t) 1 << 31); }

static int fa_kernel(const mi355x_tensor * q, const mi355x_tensor * k, int mode, const mi355x_tensor * v = nullptr) {
    if (mode == MI355X_FA_F32) return q->ne[1] > SEQ_ROW_MAX_N ? FA_K_MFMA : FA_K_VEC;
    if (q->ne[1] <= SEQ_ROW_MAX_N) return mode == MI355X_FA_F16_PK && fits_32bit_offsets(k) && (!v || fits_32bit_offsets(v)) ? FA_K_PK_ROW : FA_K_SEQ_ROW;
    return FA_K_SEQ_TILE;
}

extern "C" const char * mi355x_flash_attn_ext_kernel_name(const mi355x_tensor * q, const mi355x_tensor * k, int mode) {
    if (!q || !k) return "flash_attn.invalid";
    switch (fa_kernel(q, k, mode)) {
        case FA_K_SEQ_ROW:  return "flash_attn.seq_row";
        case FA_K_PK_ROW:   return "flash_attn.seq_row_pk";
        case FA_K_SEQ_TILE: return mode == MI355X_FA_F16_PK ? "flash_attn.seq_tile_pk" : "flash_attn.seq_tile";
        case FA_K_MFMA:     return "flash_attn.mfma_f32";
        default:            return "flash_attn.vec_f32";
    }
}

extern "C" size_t mi355x_flash_attn_ext_workspace_size(const mi355x_tensor * q, const mi355x_tensor * k) {
    (void) q; (void) k;
    return 0;
}

static int flash_attn_ext(const mi355x_tensor * q, const mi355x_tensor * k, const mi355x_tensor * v,
                          const mi355x_tensor * mask, const mi355x_tensor * mask_f16, const mi355x_tensor * dst, float scale, int mode,
                          void * workspace, size_t workspace_size, void * stream) {
    if (!q || !k || !v || !dst) return MI355X_ERR_INVALID;
    const bool emit = mode & MI355X_FA_EMIT_F16, emit_q8 = mode & MI355X_FA_EMIT_Q8_0;
    mode &= ~(MI355X_FA_EMIT_F16 | MI355X_FA_EMIT_Q8_0);
    if (emit && emit_q8) return MI355X_ERR_INVALID;
    if (mode != MI355X_FA_F16_SEQ && mode != MI355X_FA_F32 && mode != MI355X_FA_F16_PK) return MI355X_ERR_INVALID;
    // dst without memory: only the image is wanted (the key-by-key tile kernel with MI355X_FA_EMIT_F16)
    if (!dst->data && !(emit && fa_kernel(q, k, mode, v) == FA_K_SEQ_TILE)) return MI355X_ERR_INVALID;
    if (q->type != MI355X_TYPE_F32 || k->type != MI355X_TYPE_F16 || v->type != MI355X_TYPE_F16 || dst->type != MI355X_TYPE_F32) return MI355X_ERR_UNSUPPORTED;
    if (q->ne[0] != FA_D || k->ne[0] != FA_D || v->ne[0] != FA_D) return MI355X_ERR_UNSUPPORTED;
    if (q->nb[0] != 4 || k->nb[0] != 2 || v->nb[0] != 2) return MI355X_ERR_UNSUPPORTED;
    const int64_t N = q->ne[1], H = q->ne[2], KV = k->ne[1];
    if (v->ne[1] != KV || k->ne[2] <= 0 || v->ne[2] <= 0 || H % k->ne[2] != 0 || H % v->ne[2] != 0) return MI355X_ERR_INVALID;
    if (k->ne[3] <= 0 || v->ne[3] <= 0 || q->ne[3] % k->ne[3] != 0 || q->ne[3] % v->ne[3] != 0) return MI355X_ERR_INVALID;
    if (dst->ne[0] != FA_D || dst->ne[1] != H || dst->ne[2] != N || dst->ne[3] != q->ne[3] || !is_contiguous(dst)) return MI355X_ERR_INVALID;
    if (mask) {
        // an F32 mask is what the few-query kernel takes in place of its f16 copy (same values after its own rounding)
        if (mask->type == MI355X_TYPE_F32) { if (!fa_is_row(fa_kernel(q, k, mode, v))) return MI355X_ERR_UNSUPPORTED; }
        else if (mask->type != MI355X_TYPE_F16) return MI355X_ERR_UNSUPPORTED;
        if (mask->ne[0] != KV || mask->ne[1] < N || mask->nb[0] != type_size(mask->type)) return MI355X_ERR_INVALID;
    }
    if (mask_f16) {                                        // the f16 copy of an F32 mask, written on the way
        if (!mask || mask->type != MI355X_TYPE_F32 || mask_f16->type != MI355X_TYPE_F16) return MI355X_ERR_UNSUPPORTED;
        if (mask_f16->ne[0] != KV || mask_f16->ne[1] < N || mask_f16->nb[0] != 2 || !mask_f16->data) return MI355X_ERR_INVALID;
        // dst is written by workgroups that finish while others still read the mask, and the copy is written while the f32
        // form is read: the three may not share memory
        auto overlap = [](const void * a, size_t an, const void * b, size_t bn) { return (const char *) a < (const char *) b + bn && (const char *) b < (const char *) a + an; };
        const size_t dst_bytes = (size_t)(N * H * q->ne[3]) * FA_D * 4, m32_bytes = (size_t) mask->nb[1] * (size_t) N, m16_bytes = (size_t) mask_f16->nb[1] * (size_t) N;
        if (overlap(dst->data, dst_bytes, mask->data, m32_bytes) || overlap(dst->data, dst_bytes, mask_f16->data, m16_bytes) ||
            overlap(mask->data, m32_bytes, mask_f16->data, m16_bytes)) return MI355X_ERR_INVALID;
    }
    auto al16 = [](const mi355x_tensor * t) {
        return (uintptr_t) t->data % 16 == 0 && t->nb[1] % 16 == 0 && t->nb[2] % 16 == 0 && t->nb[3] % 16 == 0;
    };
    if (!al16(q) || !al16(k) || !al16(v) || (uintptr_t) dst->data % 16 != 0) return MI355X_ERR_UNSUPPORTED;
    if (N == 0 || H == 0 || q->ne[3] == 0) return MI355X_OK;
    if (KV == 0 || KV > (1 << 30)) return MI355X_ERR_UNSUPPORTED;        // every kernel reads key 0 and counts keys in 32 bits
    if (H > 65535 || q->ne[3] > 65535) return MI355X_ERR_UNSUPPORTED;

    fa_args a;
    a.q = (const char *) q->data; a.k = (const char *) k->data; a.v = (const char *) v->data;
    a.mask = mask ? (const char *) mask->data : nullptr; a.d = (char *) dst->data;
    a.N = N; a.KV = KV; a.H = H;
    a.q_nb1 = q->nb[1]; a.q_nb2 = q->nb[2]; a.q_nb3 = q->nb[3];
    a.k_nb1 = k->nb[1]; a.k_nb2 = k->nb[2]; a.k_nb3 = k->nb[3];
    a.v_nb1 = v->nb[1]; a.v_nb2 = v->nb[2]; a.v_nb3 = v->nb[3];
    a.m_nb1 = mask ? mask->nb[1] : 0;
    a.mask_f32 = mask && mask->type == MI355X_TYPE_F32;
    a.mask_copy = mask_f16 ? (half_t *) mask_f16->data : nullptr; a.mc_nb1 = mask_f16 ? (int64_t) mask_f16->nb[1] : 0;
    a.hk_ratio = H / k->ne[2]; a.hv_ratio = H / v->ne[2];
    a.ne3 = q->ne[3]; a.k_ne3_ratio = q->ne[3] / k->ne[3]; a.v_ne3_ratio = q->ne[3] / v->ne[3];
    a.scale = scale;
    a.x16 = nullptr;
    if (emit) {
        // only the tile kernels write the image; say so rather than silently skip it
        if (fa_kernel(q, k, mode, v) != FA_K_SEQ_TILE && fa_kernel(q, k, mode, v) != FA_K_MFMA) return MI355X_ERR_UNSUPPORTED;
        if (!workspace || (uintptr_t) workspace % 16 != 0 || workspace_size < (size_t)(N * H * q->ne[3]) * FA_D * sizeof(half_t)) return MI355X_ERR_WORKSPACE;
        a.x16 = (half_t *) workspace;
    }
    if (emit_q8) {
        // the few-query kernel writes the Q8_0 form
        if (!fa_is_row(fa_kernel(q, k, mode, v))) return MI355X_ERR_UNSUPPORTED;
        const size_t rows = (size_t)(N * q->ne[3]), K = (size_t) H * FA_D;
        if (!workspace || (uintptr_t) workspace % 16 != 0 || workspace_size < rows * K + rows * (K / 32) * 8) return MI355X_ERR_WORKSPACE;
        a.x16 = (half_t *) workspace;
    }
    hipStream_t st = (hipStream_t) stream;

    switch (fa_kernel(q, k, mode, v)) {
        case FA_K_SEQ_ROW: {
            const int kv_pad = (int)((KV + ROW_CHUNK - 1) / ROW_CHUNK * ROW_CHUNK);
            dim3 grid((unsigned)(8 * ((H + 7) / 8) * N), 1, (unsigned) q->ne[3]);
            k_fattn_seq_row<<<grid, 256, 0, st>>>(a, kv_pad);
        } break;
        case FA_K_PK_ROW: {
            const int kv_pad = (int)((KV + ROW_CHUNK - 1) / ROW_CHUNK * ROW_CHUNK);
            dim3 grid((unsigned)(8 * ((H + 7) / 8) * N), 1, (unsigned) q->ne[3]);
            k_fattn_pk_row<<<grid, 256, 0, st>>>(a, kv_pad);
        } break;
        case FA_K_SEQ_TILE: {
            const int64_t gx = (N + T_Q - 1) / T_Q;
            if (gx > 0x7fffffff) return MI355X_ERR_UNSUPPORTED;
            dim3 grid((unsigned) gx, (unsigned) H, (unsigned) q->ne[3]);
            // per device and kernel: they ask for more LDS than a launch gets by default
            static std::atomic<bool> configured[64][2];
            int dev = 0;
            if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) { (void) hipGetLastError(); return MI355X_ERR_HIP; }
            const int pk = mode == MI355X_FA_F16_PK;
            if (!configured[dev][pk].load(std::memory_order_acquire)) {
                const void * fn = pk ? (const void *) k_fattn_pk_tile : (const void *) k_fattn_seq_tile;
                if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, pk ? (int) P_LDS_BYTES : (int) T_LDS_BYTES) != hipSuccess) { (void) hipGetLastError(); return MI355X_ERR_HIP; }
                configured[dev][pk].store(true, std::memory_order_release);
            }
            if (pk) k_fattn_pk_tile<<<grid, 512, P_LDS_BYTES, st>>>(a);
            else    k_fattn_seq_tile<<<grid, 512, T_LDS_BYTES, st>>>(a);
        } break;
        case FA_K_MFMA: {
            const int64_t gx = (N + M_Q - 1) / M_Q;
            if (gx > 0x7fffffff) return MI355X_ERR_UNSUPPORTED;
            k_fattn_mfma<<<dim3((unsigned) gx, (unsigned) H, (unsigned) q->ne[3]), 256, 0, st>>>(a);
        } break;
        default: {
            const int64_t waves = N * H * q->ne[3];
            const int64_t grid = (waves + 3) / 4;
            if (grid > 0x7fffffff) return MI355X_ERR_UNSUPPORTED;
            k_fattn_vec<<<(unsigned) grid, 256, 0, st>>>(a);
        }
    }
    return launch_status();
}

extern "C" int mi355x_flash_attn_ext(const mi355x_tensor * q, const mi355x_tensor * k, const mi355x_tensor * v,
                                     const mi355x_tensor * mask, const mi355x_tensor * dst, float scale, int mode,
                                     void * workspace, size_t workspace_size, void * stream) {
    return flash_attn_ext(q, k, v, mask, nullptr, dst, scale, mode, workspace, workspace_size, stream);
}

extern "C" int mi355x_flash_attn_ext_cast_mask(const mi355x_tensor * q, const mi355x_tensor * k, const mi355x_tensor * v,
                                               const mi355x_tensor * mask_f32, const mi355x_tensor * mask_f16, const mi355x_tensor * dst, float scale, int mode,
                                               void * workspace, size_t workspace_size, void * stream) {
    if (!mask_f32 || !mask_f16) return MI355X_ERR_INVALID;
    return flash_attn_ext(q, k, v, mask_f32, mask_f16, dst, scale, mode, workspace, workspace_size, stream);
}
