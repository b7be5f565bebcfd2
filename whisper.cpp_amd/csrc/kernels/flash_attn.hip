// FLASH_ATTN_EXT for gfx950 (ggml_compute_forward_flash_attn_ext_f16, ggml/src/ggml-cpu/ops.cpp:6638-6851)
//   dst[:, h, n] = softmax_keys(scale * q[:, n, h] . k[:, key, h] + mask[key, n]) @ v[:, key, h]
// head size 64, q f32 (rounded to f16 first, as the CPU backend does before its f16 dot), k/v f16, f32 softmax state.
//
//   * k_fattn_vec  — any N / KV / mask.  One wavefront per (query, head); the 64 lanes take keys
//                    lane, lane+64, ... each with its own running (max, sum, 64-wide accumulator), merged
//                    across lanes at the end.  Used for the decoder's few-query steps.
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
    // dst [D, H, N, ne3] contiguous
    float * dp = (float *) a.d + ((i3 * a.N + n) * a.H + h) * FA_D;
    dp[lane] = out * inv;
}

extern "C" const char * mi355x_flash_attn_ext_kernel_name(const mi355x_tensor * q, const mi355x_tensor * k) {
    (void) q; (void) k;
    return "flash_attn.vec";
}

extern "C" size_t mi355x_flash_attn_ext_workspace_size(const mi355x_tensor * q, const mi355x_tensor * k) {
    (void) q; (void) k;
    return 0;
}

extern "C" int mi355x_flash_attn_ext(const mi355x_tensor * q, const mi355x_tensor * k, const mi355x_tensor * v,
                                     const mi355x_tensor * mask, const mi355x_tensor * dst, float scale,
                                     void * workspace, size_t workspace_size, void * stream) {
    (void) workspace; (void) workspace_size;
    if (!q || !k || !v || !dst) return MI355X_ERR_INVALID;
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
    if (!al16(q) || !al16(k) || !al16(v)) return MI355X_ERR_UNSUPPORTED;
    if (N == 0 || H == 0 || q->ne[3] == 0) return MI355X_OK;

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

    const int64_t waves = N * H * q->ne[3];
    const int64_t grid = (waves + 3) / 4;
    if (grid > 0x7fffffff) return MI355X_ERR_UNSUPPORTED;
    k_fattn_vec<<<(unsigned) grid, 256, 0, (hipStream_t) stream>>>(a);
    return launch_status();
}
