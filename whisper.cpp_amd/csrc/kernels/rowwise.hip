// Row reductions: NORM (+ fused LayerNorm affine) and SOFT_MAX.  One 64-lane wavefront owns one row, so
// the reductions are pure cross-lane shuffles with no LDS traffic and no block barrier; four rows share
// a 256-thread block.  Both are HBM-bound: one read and one write of the row.
#include "common.h"

#define ROWS_PER_BLOCK 4
#define NORM_MAX_V4    8      // rows up to 64*4*8 = 2048 floats are held in registers between the passes (NV = float4s per lane)

// ------------------------------------------------------------------------------------------------------
// NORM (ggml/src/ggml-cpu/ops.cpp:3109-3158): mean, then variance of the centred values, then scale.
// ------------------------------------------------------------------------------------------------------

// EMIT: also write the row as the MFMA GEMM wants its activations — rounded to Q8_0 like quantize_row_q8_0
// (ggml-cpu-quants.c:808-865: block amax, id = 127/amax, round half to even, d through f16) and stored as f16(q * d),
// dense [nrows][ne0] — so that the products that follow need no conversion pass of their own.
// EMIT == 2: the row quantized to Q8_0 itself, in the layout the few-column product reads its activations from
// (int8 q[nrows][ne0] | float d[nrows][ne0/32] | int32 sum of a block's quants).
// FULL: the row fills every lane's NV float4s (ne0 = 256 NV) and both affine vectors are there — whisper's LayerNorms over 256,
// 512, ... 1280 values: no guard around any load, reduction term or store (34 exec-mask branches less in a kernel whose time
// is its chain of dependent instructions)
template <int NV, int EMIT, bool FULL = false>
__global__ void __launch_bounds__(ROWS_PER_BLOCK * WAVE) k_norm(tview s, tview d, int64_t nrows, float eps, const float * __restrict__ w, const float * __restrict__ b, half_t * __restrict__ x16) {
    const int     lane = threadIdx.x % WAVE;
    const int64_t row  = (int64_t) blockIdx.x * ROWS_PER_BLOCK + threadIdx.x / WAVE;
    if (row >= nrows) return;
    const int64_t i1 = row % s.ne1, i2 = (row / s.ne1) % s.ne2, i3 = row / (s.ne1 * s.ne2);
    const float * x = (const float *)(s.p + i1*s.nb1 + i2*s.nb2 + i3*s.nb3);
    float *       y = (float *)(d.p + i1*d.nb1 + i2*d.nb2 + i3*d.nb3);
    const int64_t ne0 = s.ne0;

    if (NV > 0) {
        const int n4 = (int)(ne0 / 4);
        float4 v[NV ? NV : 1], ww[NV ? NV : 1], bb[NV ? NV : 1];
        // the affine vectors are fetched together with the row, not after the two reductions
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int c = lane + j * WAVE;
            ww[j] = make_float4(1.f, 1.f, 1.f, 1.f); bb[j] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (FULL || c < n4) { if (FULL || w) ww[j] = ((const float4 *) w)[c]; if (FULL || b) bb[j] = ((const float4 *) b)[c]; }
        }
        float sum = 0.0f;
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int c = lane + j * WAVE;
            if (FULL || c < n4) { v[j] = ((const float4 *) x)[c]; sum += (v[j].x + v[j].y) + (v[j].z + v[j].w); }
        }
        const float mean = wave_sum(sum) / (float) ne0;
        float sum2 = 0.0f;
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int c = lane + j * WAVE;
            if (FULL || c < n4) {
                v[j].x -= mean; v[j].y -= mean; v[j].z -= mean; v[j].w -= mean;
                sum2 += (v[j].x*v[j].x + v[j].y*v[j].y) + (v[j].z*v[j].z + v[j].w*v[j].w);
            }
        }
        const float scale = 1.0f / sqrtf(wave_sum(sum2) / (float) ne0 + eps);
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int c = lane + j * WAVE;
            if (FULL || c < n4) {
                float4 r = { v[j].x * scale, v[j].y * scale, v[j].z * scale, v[j].w * scale };
                // (the affine is two graph nodes, MUL then ADD: two roundings, never one fused multiply-add — without the guards
                // around them the two would be contracted)
                {
#pragma clang fp contract(off)
                    if (FULL || w) { r.x *= ww[j].x; r.y *= ww[j].y; r.z *= ww[j].z; r.w *= ww[j].w; }
                    if (FULL || b) { r.x += bb[j].x; r.y += bb[j].y; r.z += bb[j].z; r.w += bb[j].w; }
                }
                if (EMIT != 1 || d.p) ((float4 *) y)[c] = r;     // (EMIT == 1 without a destination: the image is all the caller wants)
                if (EMIT) {                                // a 32-value block = 8 consecutive lanes (ne0 % 32 == 0: they are all here)
                    float amax = fmaxf(fmaxf(fabsf(r.x), fabsf(r.y)), fmaxf(fabsf(r.z), fabsf(r.w)));
                    amax = lanes_max<8>(amax);
                    const float id = amax != 0.0f ? 127.0f / amax : 0.0f;
                    const float dq = h2f(f2h_bits(div127(amax)));
                    if (EMIT == 1) {
                        const half4_t h = { (half_t)((rintf(r.x * id) + 0.0f) * dq), (half_t)((rintf(r.y * id) + 0.0f) * dq), (half_t)((rintf(r.z * id) + 0.0f) * dq), (half_t)((rintf(r.w * id) + 0.0f) * dq) };
                        *(half4_t *)(x16 + row * ne0 + 4 * (int64_t) c) = h;
                    } else {
                        const int q0 = (int) rintf(r.x * id), q1 = (int) rintf(r.y * id), q2 = (int) rintf(r.z * id), q3 = (int) rintf(r.w * id);
                        int qsum = q0 + q1 + q2 + q3;
                        qsum = lanes_sum<8>(qsum);
                        char * q8 = (char *) x16;
                        const int64_t nbk = ne0 / 32;
                        ((int32_t *) q8)[row * (ne0 / 4) + c] = (q0 & 0xFF) | ((q1 & 0xFF) << 8) | ((q2 & 0xFF) << 16) | ((q3 & 0xFF) << 24);
                        if ((c & 7) == 0) {
                            ((float *)(q8 + nrows * ne0))[row * nbk + c / 8] = dq;
                            ((int32_t *)(q8 + nrows * ne0 + nrows * nbk * 4))[row * nbk + c / 8] = qsum;
                        }
                    }
                }
            }
        }
    } else {
        float sum = 0.0f;
        for (int64_t c = lane; c < ne0; c += WAVE) sum += x[c];
        const float mean = wave_sum(sum) / (float) ne0;
        float sum2 = 0.0f;
        for (int64_t c = lane; c < ne0; c += WAVE) { const float t = x[c] - mean; sum2 += t * t; }
        const float scale = 1.0f / sqrtf(wave_sum(sum2) / (float) ne0 + eps);
        for (int64_t c = lane; c < ne0; c += WAVE) {
            float r = (x[c] - mean) * scale;
            if (w) r *= w[c];
            if (b) r += b[c];
            y[c] = r;
        }
    }
}

static int norm_impl(const mi355x_tensor * src, const mi355x_tensor * dst, float eps, const float * w, const float * b, void * x16, int emit, void * stream);

extern "C" int mi355x_norm(const mi355x_tensor * src, const mi355x_tensor * dst, float eps, const float * w, const float * b, void * stream) {
    return norm_impl(src, dst, eps, w, b, nullptr, 0, stream);
}

extern "C" int mi355x_norm_emit_f16(const mi355x_tensor * src, const mi355x_tensor * dst, float eps, const float * w, const float * b, void * x16, void * stream) {
    if (!x16 || (uintptr_t) x16 % 8 != 0) return MI355X_ERR_INVALID;
    return norm_impl(src, dst, eps, w, b, x16, 1, stream);
}
extern "C" int mi355x_norm_emit_q8_0(const mi355x_tensor * src, const mi355x_tensor * dst, float eps, const float * w, const float * b, void * q8, void * stream) {
    if (!q8 || (uintptr_t) q8 % 16 != 0) return MI355X_ERR_INVALID;
    if (src && (src->ne[2] != 1 || src->ne[3] != 1)) return MI355X_ERR_UNSUPPORTED;
    return norm_impl(src, dst, eps, w, b, q8, 2, stream);
}

static int norm_impl(const mi355x_tensor * src, const mi355x_tensor * dst, float eps, const float * w, const float * b, void * x16, int emit, void * stream) {
    if (!src || !dst || !(eps >= 0.0f)) return MI355X_ERR_INVALID;
    if (src->type != MI355X_TYPE_F32 || dst->type != MI355X_TYPE_F32) return MI355X_ERR_UNSUPPORTED;
    if (!same_shape(src, dst) || src->nb[0] != 4 || dst->nb[0] != 4) return MI355X_ERR_INVALID;
    const int64_t nrows = src->ne[1] * src->ne[2] * src->ne[3];
    if (nrows == 0 || src->ne[0] == 0) return MI355X_OK;
    // a destination without memory is an argument of the f16-image form alone (the caller wants the image and nothing else)
    if (!src->data || (!dst->data && emit != 1)) return MI355X_ERR_INVALID;
    const int64_t grid = (nrows + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK;
    if (grid > 0x7fffffff) return MI355X_ERR_UNSUPPORTED;
    hipStream_t st = (hipStream_t) stream;
    auto al16 = [](const void * p, const size_t * nb) {
        return (uintptr_t) p % 16 == 0 && nb[1] % 16 == 0 && nb[2] % 16 == 0 && nb[3] % 16 == 0;
    };
    const bool in_regs = src->ne[0] % 4 == 0 && src->ne[0] <= 4 * WAVE * NORM_MAX_V4 &&
                         al16(src->data, src->nb) && al16(dst->data, dst->nb) &&
                         (uintptr_t) w % 16 == 0 && (uintptr_t) b % 16 == 0;
    // the register-resident form is compiled per row length (float4s per lane), so that a 1280-wide row runs five
    // iterations' worth of code, not eight guarded ones: these kernels are latency, not bandwidth, when the rows are few
    const int nv = in_regs ? (int)((src->ne[0] / 4 + WAVE - 1) / WAVE) : 0;
    if (x16 && (!in_regs || src->ne[0] % QK != 0)) return MI355X_ERR_UNSUPPORTED;      // only that form emits, and only whole blocks
    const tview vs = make_view(src), vd = make_view(dst);
    const unsigned g = (unsigned) grid, t = ROWS_PER_BLOCK * WAVE;
    const bool full = nv > 0 && src->ne[0] == (int64_t) 4 * WAVE * nv && w && b;
#define NORM_LAUNCH(NV) \
    do { \
        if (full) { \
            if (!x16)           k_norm<NV, 0, true><<<g, t, 0, st>>>(vs, vd, nrows, eps, w, b, nullptr); \
            else if (emit == 2) k_norm<NV, 2, true><<<g, t, 0, st>>>(vs, vd, nrows, eps, w, b, (half_t *) x16); \
            else                k_norm<NV, 1, true><<<g, t, 0, st>>>(vs, vd, nrows, eps, w, b, (half_t *) x16); \
        } else { \
            if (!x16)           k_norm<NV, 0><<<g, t, 0, st>>>(vs, vd, nrows, eps, w, b, nullptr); \
            else if (emit == 2) k_norm<NV, 2><<<g, t, 0, st>>>(vs, vd, nrows, eps, w, b, (half_t *) x16); \
            else                k_norm<NV, 1><<<g, t, 0, st>>>(vs, vd, nrows, eps, w, b, (half_t *) x16); \
        } \
    } while (0)
    switch (nv) {
        case 0:  k_norm<0, 0><<<g, t, 0, st>>>(vs, vd, nrows, eps, w, b, nullptr); break;
        case 1:  NORM_LAUNCH(1); break;
        case 2:  NORM_LAUNCH(2); break;
        case 3:  NORM_LAUNCH(3); break;
        case 4:  NORM_LAUNCH(4); break;
        case 5:  NORM_LAUNCH(5); break;
        case 6:  NORM_LAUNCH(6); break;
        default: NORM_LAUNCH(8); break;
    }
#undef NORM_LAUNCH
    return launch_status();
}

// ------------------------------------------------------------------------------------------------------
// SOFT_MAX (ggml/src/ggml-cpu/ops.cpp:4641-4737), max_bias = 0
// ------------------------------------------------------------------------------------------------------

template <typename TM>
__global__ void k_soft_max(tview s, tview d, const char * __restrict__ mask, int64_t mask_nb1, int64_t nrows, float scale) {
    const int     lane = threadIdx.x % WAVE;
    const int64_t row  = (int64_t) blockIdx.x * ROWS_PER_BLOCK + threadIdx.x / WAVE;
    if (row >= nrows) return;
    const int64_t i1 = row % s.ne1, i2 = (row / s.ne1) % s.ne2, i3 = row / (s.ne1 * s.ne2);
    const float * x = (const float *)(s.p + i1*s.nb1 + i2*s.nb2 + i3*s.nb3);
    float *       y = (float *)(d.p + i1*d.nb1 + i2*d.nb2 + i3*d.nb3);
    const TM *    m = mask ? (const TM *)(mask + i1 * mask_nb1) : nullptr;   // the mask is shared by all heads
    const int64_t ne0 = s.ne0;

    float mx = -INFINITY;
    for (int64_t c = lane; c < ne0; c += WAVE) {
        const float v = x[c] * scale + (m ? (float) m[c] : 0.0f);
        mx = fmaxf(mx, v);
    }
    mx = wave_max(mx);
    float sum = 0.0f;
    for (int64_t c = lane; c < ne0; c += WAVE) {
        const float v = x[c] * scale + (m ? (float) m[c] : 0.0f);
        const float e = (v == -INFINITY) ? 0.0f : __expf(v - mx);
        y[c] = e;                                  // in-place safe: each lane rereads only what it wrote
        sum += e;
    }
    const float inv = 1.0f / wave_sum(sum);
    for (int64_t c = lane; c < ne0; c += WAVE) y[c] *= inv;
}

extern "C" int mi355x_soft_max(const mi355x_tensor * src, const mi355x_tensor * mask, const mi355x_tensor * dst, float scale, void * stream) {
    if (!src || !dst) return MI355X_ERR_INVALID;
    if (src->type != MI355X_TYPE_F32 || dst->type != MI355X_TYPE_F32) return MI355X_ERR_UNSUPPORTED;
    if (!same_shape(src, dst) || src->nb[0] != 4 || dst->nb[0] != 4) return MI355X_ERR_INVALID;
    if (mask) {
        if (mask->type != MI355X_TYPE_F32 && mask->type != MI355X_TYPE_F16) return MI355X_ERR_UNSUPPORTED;
        if (mask->ne[0] != src->ne[0] || mask->ne[1] < src->ne[1] || mask->nb[0] != type_size(mask->type)) return MI355X_ERR_INVALID;
    }
    const int64_t nrows = src->ne[1] * src->ne[2] * src->ne[3];
    if (nrows == 0 || src->ne[0] == 0) return MI355X_OK;
    const int64_t grid = (nrows + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK;
    if (grid > 0x7fffffff) return MI355X_ERR_UNSUPPORTED;
    hipStream_t st = (hipStream_t) stream;
    // when src aliases dst the first pass must not be overwritten before the second reads it: the kernel
    // recomputes v from x in pass 2 and only then stores, lane-locally, so aliasing is safe.
    if (mask && mask->type == MI355X_TYPE_F16)
        k_soft_max<half_t><<<(unsigned) grid, ROWS_PER_BLOCK * WAVE, 0, st>>>(make_view(src), make_view(dst), (const char *) mask->data, (int64_t) mask->nb[1], nrows, scale);
    else
        k_soft_max<float ><<<(unsigned) grid, ROWS_PER_BLOCK * WAVE, 0, st>>>(make_view(src), make_view(dst), mask ? (const char *) mask->data : nullptr, mask ? (int64_t) mask->nb[1] : 0, nrows, scale);
    return launch_status();
}
