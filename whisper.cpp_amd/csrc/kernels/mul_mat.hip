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

typedef uint32_t __attribute__((aligned(2))) u32a2;
struct __attribute__((packed, aligned(2))) u128a2 { uint32_t x, y, z, w; };

// ------------------------------------------------------------------------------------------------------
// shared: epilogue
// ------------------------------------------------------------------------------------------------------

struct epi_args {
    int          flags;
    float        scale;
    const float *bias;
    const char * residual;   // same strides as dst, f32
    const uint16_t * gelu;   // GELU table (device), set when MI355X_EPI_GELU is
};

__device__ __forceinline__ float apply_epilogue(float v, const epi_args & e, int64_t m, int64_t n, int64_t res_off) {
    if (e.flags & MI355X_EPI_BIAS)     v += e.bias[m];
    if (e.flags & MI355X_EPI_BIAS_COL) v += e.bias[n];
    if (e.flags & MI355X_EPI_GELU)     v  = gelu_f32(v, e.gelu);
    if (e.flags & MI355X_EPI_SCALE)    v *= e.scale;
    if (e.flags & MI355X_EPI_RESIDUAL) v += *(const float *)(e.residual + res_off);
    return v;
}

struct mm_args {
    const char * w; const char * x; char * d;
    int64_t M, N, K;
    int64_t w_nb1, w_nb2, w_nb3;
    int64_t x_nb1, x_nb2, x_nb3;
    int64_t d_nb1, d_nb2, d_nb3;
    int64_t ne12, ne13, r2, r3;      // batch dims of src1/dst and broadcast ratios of src0
    epi_args e;
};

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
// MFMA GEMM
// ------------------------------------------------------------------------------------------------------

#define GB_M 128      // W rows per block
#define GB_N 128      // X rows per block
#define GB_K 64
#define GB_LD (GB_K + 8)   // LDS row pitch in halves: 144 B, so 8 consecutive rows start 4 banks apart

// per-thread staging registers for one K step
template <int T0> struct w_frag;
template <> struct w_frag<MI355X_TYPE_Q5_0> { uint32_t d, qh, qs[4]; };
template <> struct w_frag<MI355X_TYPE_Q8_0> { uint32_t d, qs[8]; };
template <> struct w_frag<MI355X_TYPE_F16>  { uint4 h[4]; };
template <> struct w_frag<MI355X_TYPE_F32>  { float4 f[8]; };
template <int T1> struct x_frag;
template <> struct x_frag<MI355X_TYPE_F32>  { float4 f[8]; };
template <> struct x_frag<MI355X_TYPE_F16>  { uint4 h[4]; };

// thread t stages W row t/2, k-half t%2 (32 weights)
template <int T0>
__device__ __forceinline__ void load_w(w_frag<T0> & f, const char * wrow, bool row_ok, int64_t k0, int64_t K) {
    const int kh = threadIdx.x & 1;
    const int64_t k = k0 + kh * 32;
    if constexpr (T0 == MI355X_TYPE_Q5_0) {
        if (row_ok && k < K) {
            const uint8_t * b = (const uint8_t *) wrow + (k / QK) * 22;
            f.d  = *(const uint16_t *) b;
            f.qh = *(const u32a2 *)(b + 2);
            const u128a2 q = *(const u128a2 *)(b + 6);
            f.qs[0] = q.x; f.qs[1] = q.y; f.qs[2] = q.z; f.qs[3] = q.w;
        } else {
            f.d = 0; f.qh = 0; f.qs[0] = f.qs[1] = f.qs[2] = f.qs[3] = 0;
        }
    } else if constexpr (T0 == MI355X_TYPE_Q8_0) {
        if (row_ok && k < K) {
            const uint8_t * b = (const uint8_t *) wrow + (k / QK) * 34;
            f.d = *(const uint16_t *) b;
            const u128a2 q0 = *(const u128a2 *)(b + 2);
            const u128a2 q1 = *(const u128a2 *)(b + 18);
            f.qs[0] = q0.x; f.qs[1] = q0.y; f.qs[2] = q0.z; f.qs[3] = q0.w;
            f.qs[4] = q1.x; f.qs[5] = q1.y; f.qs[6] = q1.z; f.qs[7] = q1.w;
        } else {
            f.d = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i) f.qs[i] = 0;
        }
    } else if constexpr (T0 == MI355X_TYPE_F16) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int64_t kk = k + 8 * i;
            f.h[i] = (row_ok && kk < K) ? *(const uint4 *)(wrow + kk * 2) : make_uint4(0, 0, 0, 0);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int64_t kk = k + 4 * i;
            f.f[i] = (row_ok && kk < K) ? *(const float4 *)(wrow + kk * 4) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
}

__device__ __forceinline__ half4_t f4_to_h4(float4 v) {
    half4_t h = { (half_t) v.x, (half_t) v.y, (half_t) v.z, (half_t) v.w };
    return h;
}

template <int T0>
__device__ __forceinline__ void store_w(const w_frag<T0> & f, half_t * ws) {
    half_t * p = ws + (threadIdx.x >> 1) * GB_LD + (threadIdx.x & 1) * 32;
    half8_t o[4];
    if constexpr (T0 == MI355X_TYPE_Q5_0) {
        q5_0_to_half32(f.d, f.qh, f.qs, o);
    } else if constexpr (T0 == MI355X_TYPE_Q8_0) {
        q8_0_to_half32(f.d, f.qs, o);
    } else if constexpr (T0 == MI355X_TYPE_F16) {
#pragma unroll
        for (int i = 0; i < 4; ++i) __builtin_memcpy(&o[i], &f.h[i], 16);
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const half4_t a = f4_to_h4(f.f[2*i]), b = f4_to_h4(f.f[2*i + 1]);
            o[i] = (half8_t){ a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3] };
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) *(half8_t *)(p + 8 * i) = o[i];
}

// X tile, F32: thread t covers float4 column t%16 of rows t/16 + 16 i (i < 8)
// X tile, F16: thread t covers 8-half column t%8 of rows t/8 + 32 i (i < 4)
template <int T1>
__device__ __forceinline__ void load_x(x_frag<T1> & f, const char * xb, int64_t x_nb1, int64_t n0, int64_t N, int64_t k0, int64_t K) {
    if constexpr (T1 == MI355X_TYPE_F32) {
        const int c = threadIdx.x & 15, r = threadIdx.x >> 4;
        const int64_t k = k0 + 4 * c;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int64_t n = n0 + r + 16 * i;
            f.f[i] = (n < N && k < K) ? *(const float4 *)(xb + n * x_nb1 + k * 4) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    } else {
        const int c = threadIdx.x & 7, r = threadIdx.x >> 3;
        const int64_t k = k0 + 8 * c;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int64_t n = n0 + r + 32 * i;
            f.h[i] = (n < N && k < K) ? *(const uint4 *)(xb + n * x_nb1 + k * 2) : make_uint4(0, 0, 0, 0);
        }
    }
}
template <int T1>
__device__ __forceinline__ void store_x(const x_frag<T1> & f, half_t * xs) {
    if constexpr (T1 == MI355X_TYPE_F32) {
        const int c = threadIdx.x & 15, r = threadIdx.x >> 4;
#pragma unroll
        for (int i = 0; i < 8; ++i) *(half4_t *)(xs + (r + 16 * i) * GB_LD + 4 * c) = f4_to_h4(f.f[i]);
    } else {
        const int c = threadIdx.x & 7, r = threadIdx.x >> 3;
#pragma unroll
        for (int i = 0; i < 4; ++i) *(uint4 *)(xs + (r + 32 * i) * GB_LD + 8 * c) = f.h[i];
    }
}

template <int T0, int T1>
__global__ void __launch_bounds__(256, 2) k_gemm_mfma(mm_args a) {
    __shared__ __attribute__((aligned(16))) half_t xs[GB_N * GB_LD];
    __shared__ __attribute__((aligned(16))) half_t ws[GB_M * GB_LD];

    const int64_t m0 = (int64_t) blockIdx.x * GB_M;
    const int64_t n0 = (int64_t) blockIdx.y * GB_N;
    const int64_t b2 = blockIdx.z % a.ne12, b3 = blockIdx.z / a.ne12;

    const char * wb = a.w + (b2 / a.r2) * a.w_nb2 + (b3 / a.r3) * a.w_nb3;
    const char * xb = a.x + b2 * a.x_nb2 + b3 * a.x_nb3;
    char *       db = a.d + b2 * a.d_nb2 + b3 * a.d_nb3;

    const int64_t wm     = m0 + (threadIdx.x >> 1);
    const bool    w_ok   = wm < a.M;
    const char *  wrow   = wb + (w_ok ? wm : 0) * a.w_nb1;

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wn = (wave >> 1) * 64, wmo = (wave & 1) * 64;   // wave patch origin inside the tile
    const int l32 = lane & 31, g = lane >> 5;

    float16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    w_frag<T0> wf;
    x_frag<T1> xf;
    load_w<T0>(wf, wrow, w_ok, 0, a.K);
    load_x<T1>(xf, xb, a.x_nb1, n0, a.N, 0, a.K);

    for (int64_t k0 = 0; k0 < a.K; k0 += GB_K) {
        store_w<T0>(wf, ws);
        store_x<T1>(xf, xs);
        __syncthreads();
        if (k0 + GB_K < a.K) {
            load_w<T0>(wf, wrow, w_ok, k0 + GB_K, a.K);
            load_x<T1>(xf, xb, a.x_nb1, n0, a.N, k0 + GB_K, a.K);
        }
#pragma unroll
        for (int kk = 0; kk < GB_K / 16; ++kk) {
            half8_t av[2], bv[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) av[i] = *(const half8_t *)(xs + (wn  + 32 * i + l32) * GB_LD + kk * 16 + 8 * g);
#pragma unroll
            for (int j = 0; j < 2; ++j) bv[j] = *(const half8_t *)(ws + (wmo + 32 * j + l32) * GB_LD + kk * 16 + 8 * g);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av[i], bv[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

    // accumulator register r of a 32x32 patch: row (= n) 8*(r/4) + 4*g + r%4, column (= m) lane%32
    const bool out_f16 = a.e.flags & MI355X_EPI_OUT_F16;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int64_t m = m0 + wmo + 32 * j + l32;
            if (m >= a.M) continue;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int64_t n = n0 + wn + 32 * i + 8 * (r >> 2) + 4 * g + (r & 3);
                if (n >= a.N) continue;
                const int64_t res_off = (b2 * a.d_nb2 + b3 * a.d_nb3) + n * a.d_nb1 + m * 4;
                const float v = apply_epilogue(acc[i][j][r], a.e, m, n, res_off);
                if (out_f16) *(half_t *)(db + n * a.d_nb1 + m * 2) = (half_t) v;
                else         *(float  *)(db + n * a.d_nb1 + m * 4) = v;
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------------
// Quantized-weight GEMM on the int8 matrix cores.
//
// ggml's MUL_MAT with Q5_0 / Q8_0 weights is, by definition of the CPU backend, an integer computation
// (ggml-cpu.c:1328-1363 converts src1 to Q8_0 with quantize_row_q8_0; ggml_vec_dot_q5_0_q8_0 / ggml_vec_dot_q8_0_q8_0,
// ggml-cpu-quants.c:2930, 3597, then form per 32-value block the exact integer dot product of the quants and add
// it, times d_w * d_x, to an f32 sum).  The kernel does exactly that: one pass quantizes src1 (k_quantize_act), then
// each 32x32 accumulator patch takes one v_mfma_i32_32x32x32_i8 per block — K = 32 is one quant block — and the
// exact i32 block sums are folded into f32 accumulators with the outer product of the block scales.
//
// Tile 128 (src1 rows) x 128 (weight rows) x 64 (two blocks), 4 wavefronts as 2 x 2, LDS double-buffered: the
// global loads of step s+2 and the nibble unpacking / LDS stores of step s+1 are issued in the same basic block as
// the MFMAs and scale FMAs of step s.
// ------------------------------------------------------------------------------------------------------

typedef int v4i_t  __attribute__((ext_vector_type(4)));
typedef int v16i_t __attribute__((ext_vector_type(16)));

static inline size_t round256(size_t n) { return (n + 255) / 256 * 256; }

// workspace of one batch slice: int8 quants [N][K], then f32 block scales [K/32][N]
__global__ void k_quantize_act(const char * __restrict__ x, char * __restrict__ ws, int64_t K, int64_t N,
                               int64_t x_nb1, int64_t x_nb2, int64_t ne12, int64_t x_nb3, int64_t slice_bytes, int64_t xd_off) {
    const int64_t t  = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;     // 8 lanes per block of 32 values, 4 values each
    const int64_t k4 = K / 4;
    const int64_t b  = blockIdx.y;
    if (t >= k4 * N) return;                                                // whole 8-lane groups leave together
    const int64_t n = t / k4, c = t % k4;
    const float4 v = *(const float4 *)(x + n * x_nb1 + (b % ne12) * x_nb2 + (b / ne12) * x_nb3 + c * 16);
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = fmaxf(amax, __shfl_xor(amax, 1, 8));
    amax = fmaxf(amax, __shfl_xor(amax, 2, 8));
    amax = fmaxf(amax, __shfl_xor(amax, 4, 8));
    const float id = amax != 0.0f ? 127.0f / amax : 0.0f;
    const int q0 = (int) rintf(v.x * id), q1 = (int) rintf(v.y * id), q2 = (int) rintf(v.z * id), q3 = (int) rintf(v.w * id);
    char * slice = ws + b * slice_bytes;
    *(int32_t *)(slice + n * K + c * 4) = (q0 & 0xFF) | ((q1 & 0xFF) << 8) | ((q2 & 0xFF) << 16) | ((q3 & 0xFF) << 24);
    if ((c & 7) == 0) ((float *)(slice + xd_off))[(c / 8) * N + n] = h2f(f2h_bits(amax / 127.0f));   // the scale goes through f16, like block_q8_0.d
}

#define I8_N   128
#define I8_M   128
#define I8_K   64            // two quant blocks per step
#define I8_LD  80            // byte pitch of the quant tiles: 64 + 16, so that 8 consecutive rows start 4 banks apart

struct i8_args {
    mm_args m;               // x = workspace quants of this launch, x_nb* describe them; w / d as usual
    const char * xd;         // block scales [K/32][N] of batch slice 0
    int64_t xd_slice;        // bytes between batch slices
};

template <int T0> struct wq_frag;
template <> struct wq_frag<MI355X_TYPE_Q5_0> { uint32_t d, qh, qs[4]; };
template <> struct wq_frag<MI355X_TYPE_Q8_0> { uint32_t d, qs[8]; };

template <int T0>
__device__ __forceinline__ void i8_load_w(wq_frag<T0> & f, const char * wrow, bool row_ok, int64_t k0, int64_t K) {
    const int64_t k = k0 + (threadIdx.x & 1) * 32;
    if constexpr (T0 == MI355X_TYPE_Q5_0) {
        if (row_ok && k < K) {
            const uint8_t * b = (const uint8_t *) wrow + (k / QK) * 22;
            f.d  = *(const uint16_t *) b;
            f.qh = *(const u32a2 *)(b + 2);
            const u128a2 q = *(const u128a2 *)(b + 6);
            f.qs[0] = q.x; f.qs[1] = q.y; f.qs[2] = q.z; f.qs[3] = q.w;
        } else { f.d = 0; f.qh = 0; f.qs[0] = f.qs[1] = f.qs[2] = f.qs[3] = 0; }
    } else {
        if (row_ok && k < K) {
            const uint8_t * b = (const uint8_t *) wrow + (k / QK) * 34;
            f.d = *(const uint16_t *) b;
            const u128a2 q0 = *(const u128a2 *)(b + 2), q1 = *(const u128a2 *)(b + 18);
            f.qs[0] = q0.x; f.qs[1] = q0.y; f.qs[2] = q0.z; f.qs[3] = q0.w;
            f.qs[4] = q1.x; f.qs[5] = q1.y; f.qs[6] = q1.z; f.qs[7] = q1.w;
        } else {
            f.d = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i) f.qs[i] = 0;
        }
    }
}

// block -> 32 signed bytes in weight order, plus the f32 scale
template <int T0>
__device__ __forceinline__ void i8_store_w(const wq_frag<T0> & f, char * wq_s, float * wd_s) {
    const int row = threadIdx.x >> 1, blk = threadIdx.x & 1;
    uint32_t o[8];
    if constexpr (T0 == MI355X_TYPE_Q5_0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            // q - 16 as a signed byte: the nibble, with 0xF0 on top where the fifth bit is clear
            const uint32_t lo_h = ((~(f.qh >> (4*i))      & 0xFu) * 0x00204081u) & 0x01010101u;
            const uint32_t hi_h = ((~(f.qh >> (16 + 4*i)) & 0xFu) * 0x00204081u) & 0x01010101u;
            o[i]     = (f.qs[i] & 0x0F0F0F0Fu)        | (lo_h * 0xF0u);
            o[4 + i] = ((f.qs[i] >> 4) & 0x0F0F0F0Fu) | (hi_h * 0xF0u);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = f.qs[i];
    }
    uint4 * p = (uint4 *)(wq_s + row * I8_LD + blk * 32);
    p[0] = make_uint4(o[0], o[1], o[2], o[3]);
    p[1] = make_uint4(o[4], o[5], o[6], o[7]);
    wd_s[blk * I8_M + row] = h2f((uint16_t) f.d);
}

struct xq_frag { uint32_t q[8]; float d; };

__device__ __forceinline__ void i8_load_x(xq_frag & f, const char * xq, const float * xd, int64_t n0, int64_t N, int64_t k0, int64_t K) {
    const int row = threadIdx.x >> 1, half = threadIdx.x & 1;
    const int64_t n = n0 + row, k = k0 + half * 32;
    if (n < N && k < K) {
        const uint4 * p = (const uint4 *)(xq + n * K + k);
        const uint4 v0 = p[0], v1 = p[1];
        f.q[0] = v0.x; f.q[1] = v0.y; f.q[2] = v0.z; f.q[3] = v0.w; f.q[4] = v1.x; f.q[5] = v1.y; f.q[6] = v1.z; f.q[7] = v1.w;
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) f.q[i] = 0;
    }
    // scales: thread t -> block t / 128 of this step, row t % 128
    const int64_t sn = n0 + (threadIdx.x & 127), sk = k0 + (threadIdx.x >> 7) * 32;
    f.d = (sn < N && sk < K) ? xd[(sk / QK) * N + sn] : 0.0f;
}
__device__ __forceinline__ void i8_store_x(const xq_frag & f, char * xq_s, float * xd_s) {
    uint4 * p = (uint4 *)(xq_s + (threadIdx.x >> 1) * I8_LD + (threadIdx.x & 1) * 32);
    p[0] = make_uint4(f.q[0], f.q[1], f.q[2], f.q[3]);
    p[1] = make_uint4(f.q[4], f.q[5], f.q[6], f.q[7]);
    xd_s[threadIdx.x] = f.d;               // [blk][row]
}

template <int T0>
__global__ void __launch_bounds__(256, 2) k_gemm_i8(i8_args ia) {
    const mm_args & a = ia.m;
    __shared__ __attribute__((aligned(16))) char  xq_s[2][I8_N * I8_LD];
    __shared__ __attribute__((aligned(16))) char  wq_s[2][I8_M * I8_LD];
    __shared__ __attribute__((aligned(16))) float xd_s[2][2 * I8_N];
    __shared__ __attribute__((aligned(16))) float wd_s[2][2 * I8_M];

    const int64_t m0 = (int64_t) blockIdx.x * I8_M, n0 = (int64_t) blockIdx.y * I8_N;
    const int64_t bz = blockIdx.z, b2 = bz % a.ne12, b3 = bz / a.ne12;
    const char *  wb = a.w + (b2 / a.r2) * a.w_nb2 + (b3 / a.r3) * a.w_nb3;
    const char *  xq = a.x + bz * a.x_nb2;
    const float * xd = (const float *)(ia.xd + bz * ia.xd_slice);
    char *        db = a.d + b2 * a.d_nb2 + b3 * a.d_nb3;

    const int64_t wm   = m0 + (threadIdx.x >> 1);
    const bool    w_ok = wm < a.M;
    const char *  wrow = wb + (w_ok ? wm : 0) * a.w_nb1;

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wn = (wave >> 1) * 64, wmo = (wave & 1) * 64, l32 = lane & 31, g = lane >> 5;

    float16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    wq_frag<T0> wf;
    xq_frag     xf;
    i8_load_w<T0>(wf, wrow, w_ok, 0, a.K);
    i8_load_x(xf, xq, xd, n0, a.N, 0, a.K);
    i8_store_w<T0>(wf, wq_s[0], wd_s[0]);
    i8_store_x(xf, xq_s[0], xd_s[0]);
    if (I8_K < a.K) { i8_load_w<T0>(wf, wrow, w_ok, I8_K, a.K); i8_load_x(xf, xq, xd, n0, a.N, I8_K, a.K); }
    __syncthreads();

    int buf = 0;
    for (int64_t k0 = 0; k0 < a.K; k0 += I8_K, buf ^= 1) {
        if (k0 + I8_K < a.K) {                      // stage s+1 goes to the other buffer (its last readers passed the barrier)
            i8_store_w<T0>(wf, wq_s[buf ^ 1], wd_s[buf ^ 1]);
            i8_store_x(xf, xq_s[buf ^ 1], xd_s[buf ^ 1]);
        }
        if (k0 + 2 * I8_K < a.K) { i8_load_w<T0>(wf, wrow, w_ok, k0 + 2 * I8_K, a.K); i8_load_x(xf, xq, xd, n0, a.N, k0 + 2 * I8_K, a.K); }

        const char *  xs = xq_s[buf]; const char * ws = wq_s[buf];
        const float * xds = xd_s[buf]; const float * wds = wd_s[buf];
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
            v4i_t av[2], bv[2];
            float dw[2];
            float4 dx[2][4];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                av[i] = *(const v4i_t *)(xs + (wn + 32 * i + l32) * I8_LD + blk * 32 + 16 * g);
#pragma unroll
                for (int q = 0; q < 4; ++q) dx[i][q] = *(const float4 *)(xds + blk * I8_N + wn + 32 * i + 8 * q + 4 * g);
            }
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                bv[j] = *(const v4i_t *)(ws + (wmo + 32 * j + l32) * I8_LD + blk * 32 + 16 * g);
                dw[j] = wds[blk * I8_M + wmo + 32 * j + l32];
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    v16i_t c;
#pragma unroll
                    for (int r = 0; r < 16; ++r) c[r] = 0;
                    c = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[i], bv[j], c, 0, 0, 0);
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        acc[i][j][4*q + 0] += (float) c[4*q + 0] * (dx[i][q].x * dw[j]);
                        acc[i][j][4*q + 1] += (float) c[4*q + 1] * (dx[i][q].y * dw[j]);
                        acc[i][j][4*q + 2] += (float) c[4*q + 2] * (dx[i][q].z * dw[j]);
                        acc[i][j][4*q + 3] += (float) c[4*q + 3] * (dx[i][q].w * dw[j]);
                    }
                }
        }
        __syncthreads();
    }

    const bool out_f16 = a.e.flags & MI355X_EPI_OUT_F16;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int64_t m = m0 + wmo + 32 * j + l32;
            if (m >= a.M) continue;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int64_t n = n0 + wn + 32 * i + 8 * (r >> 2) + 4 * g + (r & 3);
                if (n >= a.N) continue;
                const int64_t res_off = (b2 * a.d_nb2 + b3 * a.d_nb3) + n * a.d_nb1 + m * 4;
                const float v = apply_epilogue(acc[i][j][r], a.e, m, n, res_off);
                if (out_f16) *(half_t *)(db + n * a.d_nb1 + m * 2) = (half_t) v;
                else         *(float  *)(db + n * a.d_nb1 + m * 4) = v;
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------------
// quantized GEMV (N <= 8)
// ------------------------------------------------------------------------------------------------------

// LDS: int32 xq[NC][K/4] | float xd[NC][K/32] | int32 xsum[NC][K/32]
template <int T0, int NC, int LPR>
__global__ void __launch_bounds__(256) k_gemv_q(mm_args a) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int64_t K = a.K;
    const int nbk = (int)(K / QK);
    int32_t * xq   = (int32_t *) smem;
    float *   xd   = (float *)(smem + (size_t) NC * K);
    int32_t * xsum = (int32_t *)(smem + (size_t) NC * K + (size_t) NC * nbk * 4);

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
                amax = fmaxf(amax, __shfl_xor(amax, 1, 8));
                amax = fmaxf(amax, __shfl_xor(amax, 2, 8));
                amax = fmaxf(amax, __shfl_xor(amax, 4, 8));
                const float d  = amax / 127.0f;
                const float id = amax != 0.0f ? 127.0f / amax : 0.0f;
                const int q0 = (int) rintf(v[u].x * id), q1 = (int) rintf(v[u].y * id), q2 = (int) rintf(v[u].z * id), q3 = (int) rintf(v[u].w * id);
                int sum = q0 + q1 + q2 + q3;
                sum += __shfl_xor(sum, 1, 8);
                sum += __shfl_xor(sum, 2, 8);
                sum += __shfl_xor(sum, 4, 8);
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
    __syncthreads();

    constexpr int RPW = WAVE / LPR;                 // rows per wavefront
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = lane % LPR, r = lane / LPR;
    const int64_t row = (int64_t) blockIdx.x * (4 * RPW) + wave * RPW + r;
    const bool row_ok = row < a.M;
    const uint8_t * wrow = (const uint8_t *) a.w + (row_ok ? row : 0) * a.w_nb1;

    float acc[NC];
#pragma unroll
    for (int n = 0; n < NC; ++n) acc[n] = 0.0f;

    if (row_ok) {
        for (int kb = j; kb < nbk; kb += LPR) {
            uint32_t q[8];
            float dw;
            if constexpr (T0 == MI355X_TYPE_Q8_0) {
                const uint8_t * b = wrow + (int64_t) kb * 34;
                dw = h2f(*(const uint16_t *) b);
                const u128a2 q0 = *(const u128a2 *)(b + 2);
                const u128a2 q1 = *(const u128a2 *)(b + 18);
                q[0] = q0.x; q[1] = q0.y; q[2] = q0.z; q[3] = q0.w;
                q[4] = q1.x; q[5] = q1.y; q[6] = q1.z; q[7] = q1.w;
            } else {
                const uint8_t * b = wrow + (int64_t) kb * 22;
                dw = h2f(*(const uint16_t *) b);
                const uint32_t qh = *(const u32a2 *)(b + 2);
                const u128a2 qs = *(const u128a2 *)(b + 6);
                const uint32_t s[4] = { qs.x, qs.y, qs.z, qs.w };
#pragma unroll
                for (int i = 0; i < 4; ++i) {     // unsigned 5-bit values; the -16 is applied through xsum
                    q[i]     = (s[i] & 0x0F0F0F0Fu)        | spread4_to_bit4((qh >> (4*i))      & 0xFu);
                    q[4 + i] = ((s[i] >> 4) & 0x0F0F0F0Fu) | spread4_to_bit4((qh >> (16 + 4*i)) & 0xFu);
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
#pragma unroll
    for (int n = 0; n < NC; ++n) {
#pragma unroll
        for (int o = LPR / 2; o > 0; o >>= 1) acc[n] += __shfl_xor(acc[n], o, LPR);
    }
    if (row_ok && j == 0) {
        const bool out_f16 = a.e.flags & MI355X_EPI_OUT_F16;
#pragma unroll
        for (int n = 0; n < NC; ++n) {
            const float v = apply_epilogue(acc[n], a.e, row, n, n * a.d_nb1 + row * 4);
            if (out_f16) *(half_t *)(a.d + n * a.d_nb1 + row * 2) = (half_t) v;
            else         *(float  *)(a.d + n * a.d_nb1 + row * 4) = v;
        }
    }
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

template <int T0, int NC>
static int launch_gemv(const mm_args & a, hipStream_t st) {
    const size_t lds = (size_t) NC * a.K + (size_t) NC * (a.K / QK) * 8;
    // lanes per row: the smallest split of a row's blocks that still yields enough workgroups to fill 256 CUs
    int lpr = 8;
    while (lpr < 64 && a.M * lpr / 256 < 512) lpr *= 2;
    const int rows_per_wg = 4 * (WAVE / lpr);
    const unsigned grid = (unsigned)((a.M + rows_per_wg - 1) / rows_per_wg);
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
    if (N <= 2) fast = false;                         // a 128-wide tile for one or two columns is mostly padding
    if (t1 == MI355X_TYPE_F32) fast = fast && aligned16(src1) && K % 4 == 0;
    else                       fast = fast && aligned16(src1) && K % 8 == 0 && t0 == MI355X_TYPE_F16;
    if (t0 == MI355X_TYPE_F16) fast = fast && aligned16(src0) && K % 8 == 0;
    if (t0 == MI355X_TYPE_F32) fast = fast && aligned16(src0) && K % 4 == 0;
    if (quant)                 fast = fast && w_al2;
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

// the GEMM with quantized weights quantizes src1 into `workspace`: per batch slice int8 [N][K], then f32 scales [K/32][N]
extern "C" size_t mi355x_mul_mat_workspace_size(const mi355x_tensor * src0, const mi355x_tensor * src1) {
    if (!src0 || !src1) return 0;
    if (blck_size(src0->type) == 1 || src1->type != MI355X_TYPE_F32 || mm_path(src0, src1) != MM_GEMM) return 0;
    const size_t K = (size_t) src1->ne[0], N = (size_t) src1->ne[1];
    return (round256(N * K) + round256(K / QK * N * 4)) * (size_t)(src1->ne[2] * src1->ne[3]);
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
    if ((flags & MI355X_EPI_RESIDUAL) && !epi->residual) return MI355X_ERR_INVALID;
    if ((flags & MI355X_EPI_RESIDUAL) && (flags & MI355X_EPI_OUT_F16)) return MI355X_ERR_UNSUPPORTED;
    if (a.M == 0 || a.N == 0 || dst->ne[2] * dst->ne[3] == 0) return MI355X_OK;

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

    hipStream_t st = (hipStream_t) stream;
    const int64_t nbatch = a.ne12 * a.ne13;
    if (nbatch > 65535) return MI355X_ERR_UNSUPPORTED;

    const int path = mm_path(src0, src1);
    const bool quant = blck_size(t0) > 1;
    if (path == MM_GEMV) {
        return t0 == MI355X_TYPE_Q8_0 ? launch_gemv_n<MI355X_TYPE_Q8_0>(a, st) : launch_gemv_n<MI355X_TYPE_Q5_0>(a, st);
    }
    if (path == MM_GEMM) {
        dim3 grid((unsigned)((a.M + GB_M - 1) / GB_M), (unsigned)((a.N + GB_N - 1) / GB_N), (unsigned) nbatch);
        if (grid.y > 65535) return MI355X_ERR_UNSUPPORTED;
        if (quant && t1 == MI355X_TYPE_F32 && !(flags & MI355X_MM_EXACT_ACT)) {
            const size_t need = mi355x_mul_mat_workspace_size(src0, src1);
            if (!workspace || workspace_size < need || (uintptr_t) workspace % 256 != 0) return MI355X_ERR_WORKSPACE;
            const int64_t xd_off = (int64_t) round256((size_t)(a.N * a.K));
            const int64_t slice  = xd_off + (int64_t) round256((size_t)(a.K / QK * a.N * 4));
            if (!(flags & MI355X_MM_WS_READY)) {
                const int64_t threads = a.K / 4 * a.N;
                dim3 qgrid((unsigned)((threads + 255) / 256), (unsigned) nbatch);
                k_quantize_act<<<qgrid, 256, 0, st>>>(a.x, (char *) workspace, a.K, a.N, a.x_nb1, a.x_nb2, a.ne12, a.x_nb3, slice, xd_off);
            }
            i8_args ia;
            ia.m = a;
            ia.m.x = (const char *) workspace; ia.m.x_nb1 = a.K; ia.m.x_nb2 = slice; ia.m.x_nb3 = slice * a.ne12;
            ia.xd = (const char *) workspace + xd_off; ia.xd_slice = slice;
            if (t0 == MI355X_TYPE_Q5_0) k_gemm_i8<MI355X_TYPE_Q5_0><<<grid, 256, 0, st>>>(ia);
            else                        k_gemm_i8<MI355X_TYPE_Q8_0><<<grid, 256, 0, st>>>(ia);
            return launch_status();
        }
        if (t1 == MI355X_TYPE_F16) {
            k_gemm_mfma<MI355X_TYPE_F16, MI355X_TYPE_F16><<<grid, 256, 0, st>>>(a);
        } else switch (t0) {
            case MI355X_TYPE_Q5_0: k_gemm_mfma<MI355X_TYPE_Q5_0, MI355X_TYPE_F32><<<grid, 256, 0, st>>>(a); break;
            case MI355X_TYPE_Q8_0: k_gemm_mfma<MI355X_TYPE_Q8_0, MI355X_TYPE_F32><<<grid, 256, 0, st>>>(a); break;
            case MI355X_TYPE_F16:  k_gemm_mfma<MI355X_TYPE_F16,  MI355X_TYPE_F32><<<grid, 256, 0, st>>>(a); break;
            default:               k_gemm_mfma<MI355X_TYPE_F32,  MI355X_TYPE_F32><<<grid, 256, 0, st>>>(a); break;
        }
        return launch_status();
    }

    if (a.M > 0x7fffffff || (a.N + 7) / 8 > 65535) return MI355X_ERR_UNSUPPORTED;
    dim3 grid((unsigned) a.M, (unsigned)((a.N + 7) / 8), (unsigned) nbatch);
    k_mul_mat_generic<<<grid, WAVE, 0, st>>>(a, t0, t1);
    return launch_status();
}
