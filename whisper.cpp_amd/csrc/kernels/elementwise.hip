// Elementwise, gather and layout kernels: ADD/MUL (broadcast), SCALE, GELU, CPY/CONT, GET_ROWS, IM2COL,
// CONCAT, byte fill, and the standalone (de)quantizers.  All of them are HBM-bound: the fast paths move
// 16 bytes per lane with consecutive lanes on consecutive addresses; the generic paths take any strides.
#include "common.h"

#define EW_BLOCK 256

static inline int ew_grid(int64_t n, int per_block = EW_BLOCK) {
    int64_t g = (n + per_block - 1) / per_block;
    return (int) (g < 1 ? 1 : g);
}

// ------------------------------------------------------------------------------------------------------
// ADD / MUL  (ggml/src/ggml-cpu/binary-ops.cpp:49-142)
// ------------------------------------------------------------------------------------------------------

template <int OP> __device__ __forceinline__ float bin_op(float a, float b) { return OP == 0 ? a + b : a * b; }

// src0, dst contiguous with identical layout; src1 contiguous and either the same shape (n1 == n) or a
// shorter contiguous array that repeats every n1 elements (row vector, or whole lower-dimensional slab).
template <int OP>
__global__ void k_bin_contig4(const float4 * __restrict__ a, const float4 * __restrict__ b, float4 * __restrict__ d,
                              int64_t n4, int64_t n1_4) {
    int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n4) return;
    float4 x = a[i];
    float4 y = b[n1_4 == n4 ? i : i % n1_4];
    float4 r;
    r.x = bin_op<OP>(x.x, y.x); r.y = bin_op<OP>(x.y, y.y); r.z = bin_op<OP>(x.z, y.z); r.w = bin_op<OP>(x.w, y.w);
    d[i] = r;
}

template <int OP>
__global__ void k_bin_generic(tview a, tview b, tview d, int64_t n) {
    int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    int64_t i0 = i % d.ne0; int64_t t = i / d.ne0;
    int64_t i1 = t % d.ne1; t /= d.ne1;
    int64_t i2 = t % d.ne2; int64_t i3 = t / d.ne2;
    const float x = *(const float *)(a.p + i0*a.nb0 + i1*a.nb1 + i2*a.nb2 + i3*a.nb3);
    const float y = *(const float *)(b.p + (i0 % b.ne0)*b.nb0 + (i1 % b.ne1)*b.nb1 + (i2 % b.ne2)*b.nb2 + (i3 % b.ne3)*b.nb3);
    *(float *)(d.p + i0*d.nb0 + i1*d.nb1 + i2*d.nb2 + i3*d.nb3) = bin_op<OP>(x, y);
}

extern "C" int mi355x_binary(int op, const mi355x_tensor * src0, const mi355x_tensor * src1, const mi355x_tensor * dst, void * stream) {
    if (!src0 || !src1 || !dst || (op != 0 && op != 1)) return MI355X_ERR_INVALID;
    if (src0->type != MI355X_TYPE_F32 || src1->type != MI355X_TYPE_F32 || dst->type != MI355X_TYPE_F32) return MI355X_ERR_UNSUPPORTED;
    if (!same_shape(src0, dst)) return MI355X_ERR_INVALID;
    for (int i = 0; i < 4; ++i) if (src1->ne[i] <= 0 || dst->ne[i] % src1->ne[i] != 0) return MI355X_ERR_INVALID;
    const int64_t n = nelements(dst);
    if (n == 0) return MI355X_OK;
    hipStream_t st = (hipStream_t) stream;

    // src1 repeats as a contiguous prefix slab: every dim is either full or (from some dim upward) 1
    bool slab = is_contiguous(src0) && is_contiguous(src1) && is_contiguous(dst);
    if (slab) {
        bool ones = false;
        for (int i = 0; i < 4; ++i) {
            if (src1->ne[i] == dst->ne[i] && !ones) continue;
            if (src1->ne[i] == 1) { ones = true; continue; }
            slab = false;
        }
    }
    const int64_t n1 = nelements(src1);
    if (slab && n % 4 == 0 && n1 % 4 == 0 &&
        ((uintptr_t) src0->data % 16 == 0) && ((uintptr_t) src1->data % 16 == 0) && ((uintptr_t) dst->data % 16 == 0)) {
        const int64_t n4 = n / 4;
        if (op == 0) k_bin_contig4<0><<<ew_grid(n4), EW_BLOCK, 0, st>>>((const float4 *) src0->data, (const float4 *) src1->data, (float4 *) dst->data, n4, n1 / 4);
        else         k_bin_contig4<1><<<ew_grid(n4), EW_BLOCK, 0, st>>>((const float4 *) src0->data, (const float4 *) src1->data, (float4 *) dst->data, n4, n1 / 4);
        return launch_status();
    }
    if (op == 0) k_bin_generic<0><<<ew_grid(n), EW_BLOCK, 0, st>>>(make_view(src0), make_view(src1), make_view(dst), n);
    else         k_bin_generic<1><<<ew_grid(n), EW_BLOCK, 0, st>>>(make_view(src0), make_view(src1), make_view(dst), n);
    return launch_status();
}

// ------------------------------------------------------------------------------------------------------
// SCALE, GELU  (ggml/src/ggml-cpu/ops.cpp:3840-3878, 2606-2643)
// ------------------------------------------------------------------------------------------------------

template <int OP> __device__ __forceinline__ float un_op(float x, float s, const uint16_t * tab) { return OP == 0 ? x * s : gelu_f32(x, tab); }

template <int OP>
__global__ void k_unary_contig4(const float4 * __restrict__ a, float4 * __restrict__ d, int64_t n4, float s, const uint16_t * __restrict__ tab) {
    int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n4) return;
    float4 x = a[i];
    x.x = un_op<OP>(x.x, s, tab); x.y = un_op<OP>(x.y, s, tab); x.z = un_op<OP>(x.z, s, tab); x.w = un_op<OP>(x.w, s, tab);
    d[i] = x;
}

template <int OP>
__global__ void k_unary_generic(tview a, tview d, int64_t n, float s, const uint16_t * __restrict__ tab) {
    int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    int64_t i0 = i % d.ne0; int64_t t = i / d.ne0;
    int64_t i1 = t % d.ne1; t /= d.ne1;
    int64_t i2 = t % d.ne2; int64_t i3 = t / d.ne2;
    const float x = *(const float *)(a.p + i0*a.nb0 + i1*a.nb1 + i2*a.nb2 + i3*a.nb3);
    *(float *)(d.p + i0*d.nb0 + i1*d.nb1 + i2*d.nb2 + i3*d.nb3) = un_op<OP>(x, s, tab);
}

template <int OP>
static int unary_launch(const mi355x_tensor * src, const mi355x_tensor * dst, float s, void * stream) {
    if (!src || !dst) return MI355X_ERR_INVALID;
    if (src->type != MI355X_TYPE_F32 || dst->type != MI355X_TYPE_F32) return MI355X_ERR_UNSUPPORTED;
    if (!same_shape(src, dst)) return MI355X_ERR_INVALID;
    const int64_t n = nelements(dst);
    if (n == 0) return MI355X_OK;
    hipStream_t st = (hipStream_t) stream;
    const uint16_t * tab = nullptr;
    if (OP == 1 && !(tab = gelu_table_device())) return MI355X_ERR_HIP;
    if (is_contiguous(src) && is_contiguous(dst) && n % 4 == 0 &&
        ((uintptr_t) src->data % 16 == 0) && ((uintptr_t) dst->data % 16 == 0)) {
        k_unary_contig4<OP><<<ew_grid(n / 4), EW_BLOCK, 0, st>>>((const float4 *) src->data, (float4 *) dst->data, n / 4, s, tab);
    } else {
        k_unary_generic<OP><<<ew_grid(n), EW_BLOCK, 0, st>>>(make_view(src), make_view(dst), n, s, tab);
    }
    return launch_status();
}

extern "C" int mi355x_scale(const mi355x_tensor * src, const mi355x_tensor * dst, float s, void * stream) {
    return unary_launch<0>(src, dst, s, stream);
}
extern "C" int mi355x_gelu(const mi355x_tensor * src, const mi355x_tensor * dst, void * stream) {
    return unary_launch<1>(src, dst, 0.0f, stream);
}

// ------------------------------------------------------------------------------------------------------
// CPY / CONT / DUP  (ggml/src/ggml-cpu/ops.cpp:670-1183)
// ------------------------------------------------------------------------------------------------------

template <typename T> __device__ __forceinline__ float ld_as_f32(const char * p);
template <> __device__ __forceinline__ float ld_as_f32<float>(const char * p)  { return *(const float *) p; }
template <> __device__ __forceinline__ float ld_as_f32<half_t>(const char * p) { return (float) *(const half_t *) p; }
template <typename T> __device__ __forceinline__ void st_from_f32(char * p, float v);
template <> __device__ __forceinline__ void st_from_f32<float>(char * p, float v)  { *(float *) p = v; }
template <> __device__ __forceinline__ void st_from_f32<half_t>(char * p, float v) { *(half_t *) p = (half_t) v; }

// The i-th element of src in its own index order goes to the i-th element of dst in its index order.
template <typename TS, typename TD>
__global__ void k_cpy_generic(tview s, tview d, int64_t n) {
    int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    int64_t s0 = i % s.ne0; int64_t t = i / s.ne0;
    int64_t s1 = t % s.ne1; t /= s.ne1;
    int64_t s2 = t % s.ne2; int64_t s3 = t / s.ne2;
    int64_t d0 = i % d.ne0; t = i / d.ne0;
    int64_t d1 = t % d.ne1; t /= d.ne1;
    int64_t d2 = t % d.ne2; int64_t d3 = t / d.ne2;
    const float v = ld_as_f32<TS>(s.p + s0*s.nb0 + s1*s.nb1 + s2*s.nb2 + s3*s.nb3);
    st_from_f32<TD>(d.p + d0*d.nb0 + d1*d.nb1 + d2*d.nb2 + d3*d.nb3, v);
}

// both sides dense: 4 elements per lane
__global__ void k_cpy_f32_f16_contig4(const float4 * __restrict__ s, half4_t * __restrict__ d, int64_t n4) {
    int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n4) return;
    float4 x = s[i];
    half4_t h = { (half_t) x.x, (half_t) x.y, (half_t) x.z, (half_t) x.w };
    d[i] = h;
}
__global__ void k_cpy_bytes16(const uint4 * __restrict__ s, uint4 * __restrict__ d, int64_t n16) {
    int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n16) d[i] = s[i];
}

// 2-d transpose through LDS: src element (i0, i1) at i0*nb0 + i1*4 bytes (ne1 is the dense direction of
// src), dst dense [ne0, ne1] f32.  32x32 tiles, one 256-thread block per tile and batch slice.
__global__ void k_transpose_f32(const char * __restrict__ s, float * __restrict__ d, int64_t ne0, int64_t ne1,
                                int64_t s_nb0, int64_t s_nb2, int64_t d_nb2_elems) {
    __shared__ float tile[32][33];
    const int64_t b0 = (int64_t) blockIdx.x * 32, b1 = (int64_t) blockIdx.y * 32;
    const char * sp = s + (int64_t) blockIdx.z * s_nb2;
    float *      dp = d + (int64_t) blockIdx.z * d_nb2_elems;
    const int tx = threadIdx.x % 32, ty = threadIdx.x / 32;   // 8 rows per pass
    for (int r = ty; r < 32; r += 8) {
        int64_t i0 = b0 + r, i1 = b1 + tx;                     // lanes run along i1: dense in src
        tile[r][tx] = (i0 < ne0 && i1 < ne1) ? *(const float *)(sp + i0*s_nb0 + i1*4) : 0.0f;
    }
    __syncthreads();
    for (int r = ty; r < 32; r += 8) {
        int64_t i1 = b1 + r, i0 = b0 + tx;                     // lanes run along i0: dense in dst
        if (i0 < ne0 && i1 < ne1) dp[i1*ne0 + i0] = tile[tx][r];
    }
}

extern "C" int mi355x_cpy(const mi355x_tensor * src, const mi355x_tensor * dst, void * stream) {
    if (!src || !dst) return MI355X_ERR_INVALID;
    const int64_t n = nelements(src);
    if (n != nelements(dst)) return MI355X_ERR_INVALID;
    if (n == 0) return MI355X_OK;
    const int ts = src->type, td = dst->type;
    const bool fs = ts == MI355X_TYPE_F32 || ts == MI355X_TYPE_F16;
    const bool fd = td == MI355X_TYPE_F32 || td == MI355X_TYPE_F16;
    hipStream_t st = (hipStream_t) stream;
    const bool dense = is_contiguous(src) && is_contiguous(dst);

    if (ts == td && dense) {   // same type, both dense: byte copy (also covers I32 and block types)
        const size_t bytes = (size_t)(n / blck_size(ts)) * type_size(ts);
        if (type_size(ts) == 0) return MI355X_ERR_UNSUPPORTED;
        if (bytes % 16 == 0 && (uintptr_t) src->data % 16 == 0 && (uintptr_t) dst->data % 16 == 0) {
            k_cpy_bytes16<<<ew_grid(bytes / 16), EW_BLOCK, 0, st>>>((const uint4 *) src->data, (uint4 *) dst->data, bytes / 16);
            return launch_status();
        }
        if (hipMemcpyAsync(dst->data, src->data, bytes, hipMemcpyDeviceToDevice, st) != hipSuccess) return MI355X_ERR_HIP;
        return MI355X_OK;
    }
    if (!fs || !fd) return MI355X_ERR_UNSUPPORTED;

    if (ts == MI355X_TYPE_F32 && td == MI355X_TYPE_F16 && dense && n % 4 == 0 &&
        (uintptr_t) src->data % 16 == 0 && (uintptr_t) dst->data % 8 == 0) {
        k_cpy_f32_f16_contig4<<<ew_grid(n / 4), EW_BLOCK, 0, st>>>((const float4 *) src->data, (half4_t *) dst->data, n / 4);
        return launch_status();
    }
    // f32 transposed view -> dense f32 (whisper's CONT of the conv output, src/whisper.cpp:2102)
    if (ts == MI355X_TYPE_F32 && td == MI355X_TYPE_F32 && is_contiguous(dst) && same_shape(src, dst) &&
        src->nb[1] == 4 && src->nb[0] >= 4 * (size_t) src->ne[1] && src->ne[3] == 1 && src->ne[2] < 65536) {
        dim3 grid((unsigned)((src->ne[0] + 31) / 32), (unsigned)((src->ne[1] + 31) / 32), (unsigned) src->ne[2]);
        k_transpose_f32<<<grid, 256, 0, st>>>((const char *) src->data, (float *) dst->data, src->ne[0], src->ne[1],
                                              (int64_t) src->nb[0], (int64_t) src->nb[2], src->ne[0] * src->ne[1]);
        return launch_status();
    }
    tview s = make_view(src), d = make_view(dst);
    if      (ts == MI355X_TYPE_F32 && td == MI355X_TYPE_F32) k_cpy_generic<float,  float ><<<ew_grid(n), EW_BLOCK, 0, st>>>(s, d, n);
    else if (ts == MI355X_TYPE_F32 && td == MI355X_TYPE_F16) k_cpy_generic<float,  half_t><<<ew_grid(n), EW_BLOCK, 0, st>>>(s, d, n);
    else if (ts == MI355X_TYPE_F16 && td == MI355X_TYPE_F16) k_cpy_generic<half_t, half_t><<<ew_grid(n), EW_BLOCK, 0, st>>>(s, d, n);
    else                                                     k_cpy_generic<half_t, float ><<<ew_grid(n), EW_BLOCK, 0, st>>>(s, d, n);
    return launch_status();
}

// ------------------------------------------------------------------------------------------------------
// dequantization (ggml/src/ggml-quants.c:296-319, 349-363): y = q * d with q an integer and d the f16
// block scale widened to f32 — one f32 multiply per weight, so the result is bit-exact.
// ------------------------------------------------------------------------------------------------------

// weight `j` (0..31) of a block
__device__ __forceinline__ float dq_q5_0(const uint8_t * blk, int j) {
    const float    d  = h2f(ld_u16(blk));
    const uint32_t qh = ld_u32_2(blk + 2);
    const int      jj = j & 15;
    const uint32_t qs = blk[6 + jj];
    const int nib = (j < 16) ? (qs & 0x0F) : (qs >> 4);
    const int hb  = (qh >> j) & 1;
    return (float) ((nib | (hb << 4)) - 16) * d;
}
__device__ __forceinline__ float dq_q8_0(const uint8_t * blk, int j) {
    const float d = h2f(ld_u16(blk));
    return (float) ((const int8_t *) blk)[2 + j] * d;
}

template <int TYPE>
__device__ __forceinline__ float dq_elem(const uint8_t * row, int64_t k) {
    if (TYPE == MI355X_TYPE_Q5_0) return dq_q5_0(row + (k / QK) * 22, (int)(k % QK));
    if (TYPE == MI355X_TYPE_Q8_0) return dq_q8_0(row + (k / QK) * 34, (int)(k % QK));
    if (TYPE == MI355X_TYPE_F16)  return (float) ((const half_t *) row)[k];
    return ((const float *) row)[k];
}

template <int TYPE>
__global__ void k_dequantize_row(const uint8_t * __restrict__ src, float * __restrict__ dst, int64_t k) {
    int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i < k) dst[i] = dq_elem<TYPE>(src, i);
}

extern "C" int mi355x_dequantize_row(int type, const void * src, float * dst, int64_t k, void * stream) {
    if (!src || !dst || k < 0 || k % QK != 0) return MI355X_ERR_INVALID;
    if (k == 0) return MI355X_OK;
    hipStream_t st = (hipStream_t) stream;
    if      (type == MI355X_TYPE_Q5_0) k_dequantize_row<MI355X_TYPE_Q5_0><<<ew_grid(k), EW_BLOCK, 0, st>>>((const uint8_t *) src, dst, k);
    else if (type == MI355X_TYPE_Q8_0) k_dequantize_row<MI355X_TYPE_Q8_0><<<ew_grid(k), EW_BLOCK, 0, st>>>((const uint8_t *) src, dst, k);
    else return MI355X_ERR_UNSUPPORTED;
    return launch_status();
}

// ------------------------------------------------------------------------------------------------------
// GET_ROWS (ggml/src/ggml-cpu/ops.cpp:4146-4188, 4313)
// ------------------------------------------------------------------------------------------------------

template <int TYPE>
__global__ void k_get_rows(tview s, tview ids, tview d) {
    // grid: x over chunks of ne0, y over ids (flattened ne10*ne11*ne12)
    const int64_t r   = blockIdx.y;
    const int64_t i10 = r % ids.ne0, i11 = (r / ids.ne0) % ids.ne1, i12 = r / (ids.ne0 * ids.ne1);
    const int32_t row = *(const int32_t *)(ids.p + i10*ids.nb0 + i11*ids.nb1 + i12*ids.nb2);
    // The reference stops the process on an index outside the matrix (GGML_ASSERT(i01 >= 0 && i01 < ne01), ops.cpp:4174).
    // Here such a row is not read — the address would be outside the tensor — and the gathered row is NaN throughout, so
    // that the mistake shows in everything computed from it.
    const bool ok = row >= 0 && row < s.ne1;
    const uint8_t * sp = (const uint8_t *) s.p + (int64_t)(ok ? row : 0)*s.nb1 + i11*s.nb2 + i12*s.nb3;
    float * dp = (float *)(d.p + i10*d.nb1 + i11*d.nb2 + i12*d.nb3);
    for (int64_t k = (int64_t) blockIdx.x * blockDim.x + threadIdx.x; k < d.ne0; k += (int64_t) gridDim.x * blockDim.x) {
        dp[k] = ok ? dq_elem<TYPE>(sp, k) : __builtin_nanf("");
    }
}

extern "C" int mi355x_get_rows(const mi355x_tensor * src0, const mi355x_tensor * ids, const mi355x_tensor * dst, void * stream) {
    if (!src0 || !ids || !dst) return MI355X_ERR_INVALID;
    if (ids->type != MI355X_TYPE_I32 || dst->type != MI355X_TYPE_F32) return MI355X_ERR_UNSUPPORTED;
    if (dst->ne[0] != src0->ne[0] || dst->nb[0] != 4 || src0->nb[0] != type_size(src0->type)) return MI355X_ERR_INVALID;
    const int64_t nr = ids->ne[0] * ids->ne[1] * ids->ne[2];
    if (nr == 0 || dst->ne[0] == 0) return MI355X_OK;
    if (nr > 65535) return MI355X_ERR_UNSUPPORTED;
    hipStream_t st = (hipStream_t) stream;
    int gx = (int) ((dst->ne[0] + EW_BLOCK - 1) / EW_BLOCK); if (gx > 64) gx = 64;
    dim3 grid(gx, (unsigned) nr);
    tview s = make_view(src0), i = make_view(ids), d = make_view(dst);
    switch (src0->type) {
        case MI355X_TYPE_Q5_0: k_get_rows<MI355X_TYPE_Q5_0><<<grid, EW_BLOCK, 0, st>>>(s, i, d); break;
        case MI355X_TYPE_Q8_0: k_get_rows<MI355X_TYPE_Q8_0><<<grid, EW_BLOCK, 0, st>>>(s, i, d); break;
        case MI355X_TYPE_F16:  k_get_rows<MI355X_TYPE_F16 ><<<grid, EW_BLOCK, 0, st>>>(s, i, d); break;
        case MI355X_TYPE_F32:  k_get_rows<MI355X_TYPE_F32 ><<<grid, EW_BLOCK, 0, st>>>(s, i, d); break;
        default: return MI355X_ERR_UNSUPPORTED;
    }
    return launch_status();
}

// dst[:, i] = dequant(src0 row ids0[i]) + src1 row ids1[i]: a decode step's token embedding plus positional embedding
// (GET_ROWS, GET_ROWS, ADD of src/whisper.cpp:2526-2529) as one launch; the same f32 values and the same f32 sum
template <int TYPE>
__global__ void k_get_rows_add(tview s0, tview ids0, tview s1, tview ids1, tview d) {
    const int64_t i = blockIdx.y;
    const int32_t r0 = *(const int32_t *)(ids0.p + i * ids0.nb0), r1 = *(const int32_t *)(ids1.p + i * ids1.nb0);
    const bool ok = r0 >= 0 && r0 < s0.ne1 && r1 >= 0 && r1 < s1.ne1;      // as in k_get_rows: an index outside either matrix gives a NaN row
    const uint8_t * sp = (const uint8_t *) s0.p + (int64_t)(ok ? r0 : 0) * s0.nb1;
    const float *   pp = (const float *)(s1.p + (int64_t)(ok ? r1 : 0) * s1.nb1);
    float * dp = (float *)(d.p + i * d.nb1);
    for (int64_t k = (int64_t) blockIdx.x * blockDim.x + threadIdx.x; k < d.ne0; k += (int64_t) gridDim.x * blockDim.x) {
        dp[k] = ok ? dq_elem<TYPE>(sp, k) + pp[k] : __builtin_nanf("");
    }
}

extern "C" int mi355x_get_rows_add(const mi355x_tensor * src0, const mi355x_tensor * ids0, const mi355x_tensor * src1, const mi355x_tensor * ids1,
                                   const mi355x_tensor * dst, void * stream) {
    if (!src0 || !ids0 || !src1 || !ids1 || !dst) return MI355X_ERR_INVALID;
    if (ids0->type != MI355X_TYPE_I32 || ids1->type != MI355X_TYPE_I32 || dst->type != MI355X_TYPE_F32 || src1->type != MI355X_TYPE_F32) return MI355X_ERR_UNSUPPORTED;
    const int64_t nr = ids0->ne[0];
    if (ids0->ne[1] != 1 || ids0->ne[2] != 1 || ids0->ne[3] != 1 || ids1->ne[0] != nr || ids1->ne[1] != 1 || ids1->ne[2] != 1 || ids1->ne[3] != 1 ||
        dst->ne[1] != nr || dst->ne[2] != 1 || dst->ne[3] != 1 || src0->ne[2] != 1 || src0->ne[3] != 1 || src1->ne[2] != 1 || src1->ne[3] != 1) return MI355X_ERR_UNSUPPORTED;
    if (dst->ne[0] != src0->ne[0] || dst->ne[0] != src1->ne[0] || dst->nb[0] != 4 || src1->nb[0] != 4 || src0->nb[0] != type_size(src0->type)) return MI355X_ERR_INVALID;
    if (nr == 0 || dst->ne[0] == 0) return MI355X_OK;
    if (nr > 65535) return MI355X_ERR_UNSUPPORTED;
    hipStream_t st = (hipStream_t) stream;
    int gx = (int) ((dst->ne[0] + EW_BLOCK - 1) / EW_BLOCK); if (gx > 64) gx = 64;
    dim3 grid(gx, (unsigned) nr);
    tview a = make_view(src0), ia = make_view(ids0), b = make_view(src1), ib = make_view(ids1), d = make_view(dst);
    switch (src0->type) {
        case MI355X_TYPE_Q5_0: k_get_rows_add<MI355X_TYPE_Q5_0><<<grid, EW_BLOCK, 0, st>>>(a, ia, b, ib, d); break;
        case MI355X_TYPE_Q8_0: k_get_rows_add<MI355X_TYPE_Q8_0><<<grid, EW_BLOCK, 0, st>>>(a, ia, b, ib, d); break;
        case MI355X_TYPE_F16:  k_get_rows_add<MI355X_TYPE_F16 ><<<grid, EW_BLOCK, 0, st>>>(a, ia, b, ib, d); break;
        case MI355X_TYPE_F32:  k_get_rows_add<MI355X_TYPE_F32 ><<<grid, EW_BLOCK, 0, st>>>(a, ia, b, ib, d); break;
        default: return MI355X_ERR_UNSUPPORTED;
    }
    return launch_status();
}

// ------------------------------------------------------------------------------------------------------
// quantize_row_q8_0, AVX2 flavour (ggml/src/ggml-cpu/ggml-cpu-quants.c:808-865): one 32-lane half-wave per block
// ------------------------------------------------------------------------------------------------------

__global__ void k_quantize_q8_0(const float * __restrict__ x, uint8_t * __restrict__ y, int64_t nblk) {
    const int64_t t   = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t blk = t / QK;
    const int     j   = (int)(t % QK);
    if (blk >= nblk) return;                       // whole half-waves leave together (blockDim is a multiple of 32)
    const float v = x[blk * QK + j];
    float amax = fabsf(v);
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 32));
    const float d  = div127(amax);
    const float id = amax != 0.0f ? 127.0f / amax : 0.0f;
    uint8_t * b = y + blk * 34;
    if (j == 0) *(uint16_t *) b = f2h_bits(d);
    ((int8_t *) b)[2 + j] = (int8_t) (int) rintf(v * id);
}

extern "C" int mi355x_quantize_row_q8_0(const float * src, void * dst, int64_t k, void * stream) {
    if (!src || !dst || k < 0 || k % QK != 0) return MI355X_ERR_INVALID;
    if (k == 0) return MI355X_OK;
    k_quantize_q8_0<<<ew_grid(k), EW_BLOCK, 0, (hipStream_t) stream>>>(src, (uint8_t *) dst, k / QK);
    return launch_status();
}

// ------------------------------------------------------------------------------------------------------
// IM2COL 1-D, f16 out (ggml/src/ggml-cpu/ops.cpp:5784-5855)
// ------------------------------------------------------------------------------------------------------

// dst[(n*OW + ow)*IC*KW + ic*KW + kw].  A block stages a [32 ow+halo] x [32 ic] patch of src through LDS
// so that both the reads (along iw) and the writes (along ic*KW+kw) are coalesced.
#define I2C_OW 32
#define I2C_IC 32
__global__ void k_im2col_1d(const char * __restrict__ src, half_t * __restrict__ dst, int64_t IW, int64_t IC, int64_t OW,
                            int64_t nb11, int64_t nb12, int KW, int s0, int p0, int d0, int span) {
    extern __shared__ float patch[];              // [I2C_IC][span + 1]
    const int64_t ow0 = (int64_t) blockIdx.x * I2C_OW;
    const int64_t ic0 = (int64_t) blockIdx.y * I2C_IC;
    const int64_t n   = blockIdx.z;
    const int64_t iw0 = ow0 * s0 - p0;
    const int ld = span + 1;
    for (int e = threadIdx.x; e < I2C_IC * span; e += blockDim.x) {
        const int c = e / span, w = e % span;
        const int64_t iw = iw0 + w, ic = ic0 + c;
        float v = 0.0f;
        if (ic < IC && iw >= 0 && iw < IW) v = *(const float *)(src + n*nb12 + ic*nb11 + iw*4);
        patch[c * ld + w] = v;
    }
    __syncthreads();
    const int cols = I2C_IC * KW;                 // dst elements per ow for this ic range
    for (int e = threadIdx.x; e < I2C_OW * cols; e += blockDim.x) {
        const int o = e / cols, r = e % cols;
        const int c = r / KW, kw = r % KW;
        const int64_t ow = ow0 + o, ic = ic0 + c;
        if (ow < OW && ic < IC) {
            dst[(n*OW + ow) * (IC*KW) + ic0*KW + r] = (half_t) patch[c * ld + o*s0 + kw*d0];
        }
    }
}

extern "C" int mi355x_im2col_1d(const mi355x_tensor * src, const mi355x_tensor * dst, int kw, int s0, int p0, int d0, void * stream) {
    if (!src || !dst || kw <= 0 || s0 <= 0 || d0 <= 0) return MI355X_ERR_INVALID;
    if (src->type != MI355X_TYPE_F32 || dst->type != MI355X_TYPE_F16) return MI355X_ERR_UNSUPPORTED;
    if (src->nb[0] != 4 || !is_contiguous(dst) || src->ne[3] != 1) return MI355X_ERR_UNSUPPORTED;
    const int64_t IW = src->ne[0], IC = src->ne[1], N = src->ne[2], OW = dst->ne[1];
    if (dst->ne[0] != IC * kw || dst->ne[2] != N) return MI355X_ERR_INVALID;
    if (OW == 0 || IC == 0 || N == 0) return MI355X_OK;
    if (N > 65535 || (IC + I2C_IC - 1) / I2C_IC > 65535) return MI355X_ERR_UNSUPPORTED;
    const int span = (I2C_OW - 1) * s0 + (kw - 1) * d0 + 1;
    const size_t lds = (size_t) I2C_IC * (span + 1) * sizeof(float);
    if (lds > 64 * 1024) return MI355X_ERR_UNSUPPORTED;
    dim3 grid((unsigned)((OW + I2C_OW - 1) / I2C_OW), (unsigned)((IC + I2C_IC - 1) / I2C_IC), (unsigned) N);
    k_im2col_1d<<<grid, 256, lds, (hipStream_t) stream>>>((const char *) src->data, (half_t *) dst->data, IW, IC, OW,
                                                          (int64_t) src->nb[1], (int64_t) src->nb[2], kw, s0, p0, d0, span);
    return launch_status();
}

// ------------------------------------------------------------------------------------------------------
// CONCAT (ggml/src/ggml-cpu/ops.cpp:2575)
// ------------------------------------------------------------------------------------------------------

__global__ void k_concat(tview a, tview b, tview d, int64_t n, int dim) {
    int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    int64_t idx[4];
    idx[0] = i % d.ne0; int64_t t = i / d.ne0;
    idx[1] = t % d.ne1; t /= d.ne1;
    idx[2] = t % d.ne2; idx[3] = t / d.ne2;
    const int64_t split = dim == 0 ? a.ne0 : dim == 1 ? a.ne1 : dim == 2 ? a.ne2 : a.ne3;
    float v;
    if (idx[dim] < split) {
        v = *(const float *)(a.p + idx[0]*a.nb0 + idx[1]*a.nb1 + idx[2]*a.nb2 + idx[3]*a.nb3);
    } else {
        int64_t j[4] = { idx[0], idx[1], idx[2], idx[3] };
        j[dim] -= split;
        v = *(const float *)(b.p + j[0]*b.nb0 + j[1]*b.nb1 + j[2]*b.nb2 + j[3]*b.nb3);
    }
    *(float *)(d.p + idx[0]*d.nb0 + idx[1]*d.nb1 + idx[2]*d.nb2 + idx[3]*d.nb3) = v;
}

extern "C" int mi355x_concat(const mi355x_tensor * src0, const mi355x_tensor * src1, const mi355x_tensor * dst, int dim, void * stream) {
    if (!src0 || !src1 || !dst || dim < 0 || dim > 3) return MI355X_ERR_INVALID;
    if (src0->type != MI355X_TYPE_F32 || src1->type != MI355X_TYPE_F32 || dst->type != MI355X_TYPE_F32) return MI355X_ERR_UNSUPPORTED;
    for (int i = 0; i < 4; ++i) {
        const int64_t want = i == dim ? src0->ne[i] + src1->ne[i] : src0->ne[i];
        if (dst->ne[i] != want || (i != dim && src1->ne[i] != src0->ne[i])) return MI355X_ERR_INVALID;
    }
    const int64_t n = nelements(dst);
    if (n == 0) return MI355X_OK;
    k_concat<<<ew_grid(n), EW_BLOCK, 0, (hipStream_t) stream>>>(make_view(src0), make_view(src1), make_view(dst), n, dim);
    return launch_status();
}

// ------------------------------------------------------------------------------------------------------
// byte fill
// ------------------------------------------------------------------------------------------------------

__global__ void k_fill16(uint4 * __restrict__ d, uint32_t w, int64_t n16) {
    int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n16) d[i] = make_uint4(w, w, w, w);
}
__global__ void k_fill1(uint8_t * __restrict__ d, uint8_t v, int64_t n) {
    int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) d[i] = v;
}

extern "C" int mi355x_fill_bytes(void * dst, uint8_t value, size_t n, void * stream) {
    if (n == 0) return MI355X_OK;
    if (!dst) return MI355X_ERR_INVALID;
    hipStream_t st = (hipStream_t) stream;
    uint8_t * p = (uint8_t *) dst;
    const size_t head = ((uintptr_t) p % 16) ? 16 - ((uintptr_t) p % 16) : 0;
    const size_t h = head < n ? head : n;
    if (h) k_fill1<<<1, 64, 0, st>>>(p, value, (int64_t) h);
    const size_t body = (n - h) / 16 * 16;
    if (body) {
        const uint32_t w = 0x01010101u * value;
        k_fill16<<<ew_grid((int64_t)(body / 16)), EW_BLOCK, 0, st>>>((uint4 *)(p + h), w, (int64_t)(body / 16));
    }
    const size_t tail = n - h - body;
    if (tail) k_fill1<<<1, 64, 0, st>>>(p + h + body, value, (int64_t) tail);
    return launch_status();
}
