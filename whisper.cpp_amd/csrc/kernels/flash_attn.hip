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
//       k_fattn_seq_tile   N > 8:  64 queries x 64 keys per step; QK^T on v_mfma_f32_32x32x16_f16 from LDS-staged K,
//                                  softmax factors in LDS, then 16 queries per wavefront walk the 64 keys with
//                                  v_fma_mixlo/hi_f16 chains against the LDS-staged V tile.
//       k_fattn_seq_row    N <= 8: one block per (query, head): 256 threads score all keys and scan the maximum,
//                                  one wavefront (lane = d) runs the chain with V streamed from global memory.
//   MI355X_FA_F32          f32 accumulators, keys split across lanes (k_fattn_vec): closer to exact arithmetic,
//                          not to the reference.
#include "common.h"

#define FA_D 64

struct fa_args {
    const char * q; const char * k; const char * v; const char * mask; char * d;
    int64_t N, KV, H;
    int64_t q_nb1, q_nb2, q_nb3;
    int64_t k_nb1, k_nb2, k_nb3;
    int64_t v_nb1, v_nb2, v_nb3;
    int64_t m_nb1;
    int64_t hk_ratio, hv_ratio;      // q heads per k head / v head (broadcast)
    int64_t ne3, k_ne3_ratio, v_ne3_ratio;
    float scale;
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

__global__ void __launch_bounds__(256) k_fattn_seq_row(fa_args a, int kv_pad) {
    extern __shared__ __attribute__((aligned(16))) float sm[];
    float * vs_s = sm;                 // [kv_pad] scores, then vs
    float * ms_s = sm + kv_pad;        // [kv_pad]
    __shared__ float red_m[4], red_p[4], red_a[4];
    __shared__ float s_total;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t n = blockIdx.x, h = blockIdx.y, i3 = blockIdx.z;
    const int KV = (int) a.KV;

    const float * qp = (const float *)(a.q + n * a.q_nb1 + h * a.q_nb2 + i3 * a.q_nb3);
    const char *  kb = a.k + (h / a.hk_ratio) * a.k_nb2 + (i3 / a.k_ne3_ratio) * a.k_nb3;
    const char *  vb = a.v + (h / a.hv_ratio) * a.v_nb2 + (i3 / a.v_ne3_ratio) * a.v_nb3;
    const half_t * mp = a.mask ? (const half_t *)(a.mask + n * a.m_nb1) : nullptr;

    // ---- scores -------------------------------------------------------------------------------------
    float q[FA_D];
#pragma unroll
    for (int d = 0; d < FA_D; d += 4) {
        const float4 t = *(const float4 *)(qp + d);
        q[d] = (float)(half_t) t.x; q[d+1] = (float)(half_t) t.y; q[d+2] = (float)(half_t) t.z; q[d+3] = (float)(half_t) t.w;
    }
    for (int key = tid; key < kv_pad; key += 256) {
        float s = -INFINITY;
        if (key < KV) {
            const float mv = mp ? (float) mp[key] : 0.0f;
            if (mv != -INFINITY) {
                const half8_t * kr = (const half8_t *)(kb + (int64_t) key * a.k_nb1);
                float dot = 0.0f;
#pragma unroll
                for (int c = 0; c < FA_D / 8; ++c) {
                    const half8_t kk = kr[c];
#pragma unroll
                    for (int e = 0; e < 8; ++e) dot += q[8*c + e] * (float) kk[e];
                }
                s = __fadd_rn(__fmul_rn(dot, a.scale), mv);
            }
        }
        vs_s[key] = s;
    }
    __syncthreads();

    // ---- prefix maximum and softmax factors: thread t owns keys [t*seg, (t+1)*seg) ---------------------------------
    const int seg = (kv_pad + 255) / 256;
    const int k0 = tid * seg, k1 = min(kv_pad, k0 + seg);
    float lmax = -INFINITY;
    for (int key = k0; key < k1; ++key) lmax = fmaxf(lmax, vs_s[key]);
    // exclusive prefix maximum across the block: inclusive scan inside the wavefront, then the wavefront totals
    float inc = lmax;
#pragma unroll
    for (int o = 1; o < WAVE; o <<= 1) { const float t = __shfl_up(inc, o, WAVE); if (lane >= o) inc = fmaxf(inc, t); }
    if (lane == WAVE - 1) red_m[wave] = inc;
    float exc = __shfl_up(inc, 1, WAVE);
    if (lane == 0) exc = -INFINITY;
    __syncthreads();
    for (int w = 0; w < wave; ++w) exc = fmaxf(exc, red_m[w]);

    float M = exc, P = 1.0f, A = 0.0f;
    for (int key = k0; key < k1; ++key) {
        float vs, ms;
        seq_factors(vs_s[key], M, vs, ms, P, A);
        vs_s[key] = vs; ms_s[key] = ms;
    }
    // ordered reduction of (P, A): (P1, A1) then (P2, A2) -> (P1*P2, A1*P2 + A2)
#pragma unroll
    for (int o = 1; o < WAVE; o <<= 1) {
        const float Pn = __shfl_down(P, o, WAVE), An = __shfl_down(A, o, WAVE);
        if ((lane & (2 * o - 1)) == 0) { A = A * Pn + An; P = P * Pn; }
    }
    if (lane == 0) { red_p[wave] = P; red_a[wave] = A; }
    __syncthreads();
    if (tid == 0) {
        float S = 0.0f;
        for (int w = 0; w < 4; ++w) S = S * red_p[w] + red_a[w];
        s_total = S;
    }
    __syncthreads();
    if (wave != 0) return;

    // ---- the sequential f16 chain: lane = d -----------------------------------------------------------------------------------
    // 64 keys at a time: their V values sit in registers (the next 64 are in flight while these are consumed), their
    // factors are read once, one per lane, and handed to the chain through v_readlane, so that the dependent part of
    // every step is a single v_fma_mixlo_f16.
    half_t acc = (half_t) 0.0f;
    const char * vcol = vb + lane * 2;
    half_t va[ROW_CHUNK], vn[ROW_CHUNK];
    auto load_chunk = [&](half_t * dst, int key0) {
#pragma unroll
        for (int j = 0; j < ROW_CHUNK; ++j) {
            const int key = key0 + j;
            dst[j] = key < KV ? *(const half_t *)(vcol + (int64_t) key * a.v_nb1) : (half_t) 0.0f;
        }
    };
    auto run_chunk = [&](const half_t * v, int key0) {
        const int vs_l = __float_as_int(vs_s[key0 + lane]), ms_l = __float_as_int(ms_s[key0 + lane]);
#pragma unroll
        for (int j = 0; j < ROW_CHUNK; ++j) {
            const float vs = __int_as_float(__builtin_amdgcn_readlane(vs_l, j));
            const float ms = __int_as_float(__builtin_amdgcn_readlane(ms_l, j));
            if (ms != 1.0f) acc = seq_scale(acc, ms);      // scalar condition: uniform across the wavefront
            if (vs != 0.0f) acc = seq_mad(acc, v[j], vs);
        }
    };
    load_chunk(va, 0);
    for (int key0 = 0; key0 < kv_pad; key0 += 2 * ROW_CHUNK) {
        const bool more = key0 + ROW_CHUNK < kv_pad;
        if (more) load_chunk(vn, key0 + ROW_CHUNK);
        run_chunk(va, key0);
        if (more) {
            if (key0 + 2 * ROW_CHUNK < kv_pad) load_chunk(va, key0 + 2 * ROW_CHUNK);
            run_chunk(vn, key0 + ROW_CHUNK);
        }
    }
    float * dp = (float *) a.d + ((i3 * a.N + n) * a.H + h) * FA_D;
    dp[lane] = (float) acc * (1.0f / s_total);
}

// ------------------------------------------------------------------------------------------------------
// k_fattn_seq_tile: 64 queries per block, 64 keys per step
// ------------------------------------------------------------------------------------------------------

#define T_Q   64
#define T_KV  64
#define T_LDH (FA_D + 8)      // f16 pitch of the Q and K tiles (144 B rows: conflict-free b128 reads for the MFMA operands)
#define T_LDS (T_KV + 1)      // f32 pitch of the factor tiles

__global__ void __launch_bounds__(256) k_fattn_seq_tile(fa_args a) {
    __shared__ __attribute__((aligned(16))) half_t q_s[T_Q * T_LDH];
    __shared__ __attribute__((aligned(16))) half_t k_s[T_KV * T_LDH];
    __shared__ __attribute__((aligned(16))) half_t v_s[T_KV * FA_D];
    __shared__ float vs_s[T_Q * T_LDS];
    __shared__ float ms_s[T_Q * T_LDS];
    __shared__ float m_run[T_Q], s_run[T_Q];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t n0 = (int64_t) blockIdx.x * T_Q, h = blockIdx.y, i3 = blockIdx.z;
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
    __syncthreads();

    // accumulation role: wavefront w owns queries 16w .. 16w+15, 4 lanes per query, 16 d each
    const int aq = wave * 16 + (lane >> 2), ad = (lane & 3) * 16;
    half_t acc[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = (half_t) 0.0f;

    // score role: wavefront w computes the 32x32 patch (queries 32*(w/2).., keys 32*(w%2)..)
    const int sq = (wave >> 1) * 32, sk = (wave & 1) * 32, l32 = lane & 31, g = lane >> 5;

    for (int64_t key0 = 0; key0 < a.KV; key0 += T_KV) {
        // ---- stage K and V: thread t: row t/4, 32 bytes -----------------------------------------------------------------
        {
            const int r = tid >> 2, c = (tid & 3) * 16;
            const int64_t key = key0 + r;
            uint4 k0 = make_uint4(0, 0, 0, 0), k1 = k0, v0 = k0, v1 = k0;
            if (key < a.KV) {
                const uint4 * kp = (const uint4 *)(kb + key * a.k_nb1 + c * 2);
                const uint4 * vp = (const uint4 *)(vb + key * a.v_nb1 + c * 2);
                k0 = kp[0]; k1 = kp[1]; v0 = vp[0]; v1 = vp[1];
            }
            *(uint4 *)(k_s + r * T_LDH + c) = k0; *(uint4 *)(k_s + r * T_LDH + c + 8) = k1;
            *(uint4 *)(v_s + r * FA_D + c)  = v0; *(uint4 *)(v_s + r * FA_D + c + 8)  = v1;
        }
        __syncthreads();

        // ---- scores: S = Q K^T on the matrix cores ------------------------------------------------------------------------------
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
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int qi = sq + 8 * (r >> 2) + 4 * g + (r & 3);
                float s = -INFINITY;
                if (key < a.KV) {
                    float mv = 0.0f;
                    if (a.mask && n0 + qi < a.N) mv = (float) *(const half_t *)(a.mask + (n0 + qi) * a.m_nb1 + key * 2);
                    s = __fadd_rn(__fmul_rn(c16[r], a.scale), mv);
                }
                vs_s[qi * T_LDS + sk + l32] = s;
            }
        }
        __syncthreads();

        // ---- softmax factors: thread t: query t/4, keys 16*(t%4) .. +15 ------------------------------------------------------------
        {
            const int qi = tid >> 2, sgm = tid & 3;
            float * sp = vs_s + qi * T_LDS + sgm * 16;
            float * mp = ms_s + qi * T_LDS + sgm * 16;
            float sv[16], lmax = -INFINITY;
#pragma unroll
            for (int i = 0; i < 16; ++i) { sv[i] = sp[i]; lmax = fmaxf(lmax, sv[i]); }
            float M = m_run[qi];
            const float S0 = s_run[qi];
            const int base = lane & ~3;
            const float m0 = __shfl(lmax, base + 0, WAVE), m1 = __shfl(lmax, base + 1, WAVE), m2 = __shfl(lmax, base + 2, WAVE);
            if (sgm > 0) M = fmaxf(M, m0);
            if (sgm > 1) M = fmaxf(M, m1);
            if (sgm > 2) M = fmaxf(M, m2);
            float P = 1.0f, A = 0.0f;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                float vs, ms;
                seq_factors(sv[i], M, vs, ms, P, A);
                sp[i] = vs; mp[i] = ms;
            }
            // fold the four runs of this query in key order
            const float P1 = __shfl(P, base + 1, WAVE), A1 = __shfl(A, base + 1, WAVE);
            const float P2 = __shfl(P, base + 2, WAVE), A2 = __shfl(A, base + 2, WAVE);
            const float P3 = __shfl(P, base + 3, WAVE), A3 = __shfl(A, base + 3, WAVE);
            const float M3 = __shfl(M, base + 3, WAVE);
            if (sgm == 0) {
                float S = S0 * P + A;
                S = S * P1 + A1; S = S * P2 + A2; S = S * P3 + A3;
                s_run[qi] = S; m_run[qi] = M3;
            }
        }
        __syncthreads();

        // ---- the sequential f16 chains over this tile's keys -----------------------------------------------------------------------------
        {
            const float * vsp = vs_s + aq * T_LDS;
            const float * msp = ms_s + aq * T_LDS;
#pragma unroll 4
            for (int key = 0; key < T_KV; ++key) {
                const float vs = vsp[key], ms = msp[key];
                const half8_t va = *(const half8_t *)(v_s + key * FA_D + ad);
                const half8_t vb8 = *(const half8_t *)(v_s + key * FA_D + ad + 8);
                if (__any(ms != 1.0f)) {
#pragma unroll
                    for (int e = 0; e < 16; ++e) acc[e] = seq_scale(acc[e], ms);     // lanes with ms == 1 keep their value exactly
                }
#pragma unroll
                for (int e = 0; e < 8; ++e) { acc[e] = seq_mad(acc[e], va[e], vs); acc[8 + e] = seq_mad(acc[8 + e], vb8[e], vs); }
            }
        }
        __syncthreads();
    }

    const int64_t n = n0 + aq;
    if (n < a.N) {
        const float inv = 1.0f / s_run[aq];
        float * dp = (float *) a.d + ((i3 * a.N + n) * a.H + h) * FA_D + ad;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float4 o = { (float) acc[4*i] * inv, (float) acc[4*i + 1] * inv, (float) acc[4*i + 2] * inv, (float) acc[4*i + 3] * inv };
            *(float4 *)(dp + 4 * i) = o;
        }
    }
}

// ------------------------------------------------------------------------------------------------------
// host dispatch
// ------------------------------------------------------------------------------------------------------

#define SEQ_ROW_MAX_N   8
#define SEQ_ROW_MAX_KV  7168      // two f32 arrays of that many keys stay under 64 KB of LDS

enum { FA_K_VEC = 0, FA_K_SEQ_ROW = 1, FA_K_SEQ_TILE = 2 };

static int fa_kernel(const mi355x_tensor * q, const mi355x_tensor * k, int mode) {
    if (mode == MI355X_FA_F32) return FA_K_VEC;
    if (q->ne[1] <= SEQ_ROW_MAX_N && k->ne[1] <= SEQ_ROW_MAX_KV) return FA_K_SEQ_ROW;
    return FA_K_SEQ_TILE;
}

extern "C" const char * mi355x_flash_attn_ext_kernel_name(const mi355x_tensor * q, const mi355x_tensor * k, int mode) {
    if (!q || !k) return "flash_attn.invalid";
    switch (fa_kernel(q, k, mode)) {
        case FA_K_SEQ_ROW:  return "flash_attn.seq_row";
        case FA_K_SEQ_TILE: return "flash_attn.seq_tile";
        default:            return "flash_attn.vec_f32";
    }
}

extern "C" size_t mi355x_flash_attn_ext_workspace_size(const mi355x_tensor * q, const mi355x_tensor * k) {
    (void) q; (void) k;
    return 0;
}

extern "C" int mi355x_flash_attn_ext(const mi355x_tensor * q, const mi355x_tensor * k, const mi355x_tensor * v,
                                     const mi355x_tensor * mask, const mi355x_tensor * dst, float scale, int mode,
                                     void * workspace, size_t workspace_size, void * stream) {
    (void) workspace; (void) workspace_size;
    if (!q || !k || !v || !dst) return MI355X_ERR_INVALID;
    if (mode != MI355X_FA_F16_SEQ && mode != MI355X_FA_F32) return MI355X_ERR_INVALID;
    if (q->type != MI355X_TYPE_F32 || k->type != MI355X_TYPE_F16 || v->type != MI355X_TYPE_F16 || dst->type != MI355X_TYPE_F32) return MI355X_ERR_UNSUPPORTED;
    if (q->ne[0] != FA_D || k->ne[0] != FA_D || v->ne[0] != FA_D) return MI355X_ERR_UNSUPPORTED;
    if (q->nb[0] != 4 || k->nb[0] != 2 || v->nb[0] != 2) return MI355X_ERR_UNSUPPORTED;
    const int64_t N = q->ne[1], H = q->ne[2], KV = k->ne[1];
    if (v->ne[1] != KV || k->ne[2] <= 0 || v->ne[2] <= 0 || H % k->ne[2] != 0 || H % v->ne[2] != 0) return MI355X_ERR_INVALID;
    if (k->ne[3] <= 0 || v->ne[3] <= 0 || q->ne[3] % k->ne[3] != 0 || q->ne[3] % v->ne[3] != 0) return MI355X_ERR_INVALID;
    if (dst->ne[0] != FA_D || dst->ne[1] != H || dst->ne[2] != N || dst->ne[3] != q->ne[3] || !is_contiguous(dst)) return MI355X_ERR_INVALID;
    if (mask) {
        if (mask->type != MI355X_TYPE_F16) return MI355X_ERR_UNSUPPORTED;
        if (mask->ne[0] != KV || mask->ne[1] < N || mask->nb[0] != 2) return MI355X_ERR_INVALID;
    }
    auto al16 = [](const mi355x_tensor * t) {
        return (uintptr_t) t->data % 16 == 0 && t->nb[1] % 16 == 0 && t->nb[2] % 16 == 0 && t->nb[3] % 16 == 0;
    };
    if (!al16(q) || !al16(k) || !al16(v) || (uintptr_t) dst->data % 16 != 0) return MI355X_ERR_UNSUPPORTED;
    if (N == 0 || H == 0 || q->ne[3] == 0) return MI355X_OK;
    if (H > 65535 || q->ne[3] > 65535) return MI355X_ERR_UNSUPPORTED;

    fa_args a;
    a.q = (const char *) q->data; a.k = (const char *) k->data; a.v = (const char *) v->data;
    a.mask = mask ? (const char *) mask->data : nullptr; a.d = (char *) dst->data;
    a.N = N; a.KV = KV; a.H = H;
    a.q_nb1 = q->nb[1]; a.q_nb2 = q->nb[2]; a.q_nb3 = q->nb[3];
    a.k_nb1 = k->nb[1]; a.k_nb2 = k->nb[2]; a.k_nb3 = k->nb[3];
    a.v_nb1 = v->nb[1]; a.v_nb2 = v->nb[2]; a.v_nb3 = v->nb[3];
    a.m_nb1 = mask ? mask->nb[1] : 0;
    a.hk_ratio = H / k->ne[2]; a.hv_ratio = H / v->ne[2];
    a.ne3 = q->ne[3]; a.k_ne3_ratio = q->ne[3] / k->ne[3]; a.v_ne3_ratio = q->ne[3] / v->ne[3];
    a.scale = scale;
    hipStream_t st = (hipStream_t) stream;

    switch (fa_kernel(q, k, mode)) {
        case FA_K_SEQ_ROW: {
            const int kv_pad = (int)((KV + ROW_CHUNK - 1) / ROW_CHUNK * ROW_CHUNK);
            dim3 grid((unsigned) N, (unsigned) H, (unsigned) q->ne[3]);
            k_fattn_seq_row<<<grid, 256, (size_t) kv_pad * 8, st>>>(a, kv_pad);
        } break;
        case FA_K_SEQ_TILE: {
            const int64_t gx = (N + T_Q - 1) / T_Q;
            if (gx > 0x7fffffff) return MI355X_ERR_UNSUPPORTED;
            dim3 grid((unsigned) gx, (unsigned) H, (unsigned) q->ne[3]);
            k_fattn_seq_tile<<<grid, 256, 0, st>>>(a);
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
