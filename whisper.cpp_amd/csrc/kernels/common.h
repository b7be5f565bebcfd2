// Shared device/host helpers for the gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

#include "mi355x_kernels.h"

#define WAVE 64

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float    float4_t  __attribute__((ext_vector_type(4)));
typedef float    float16_t __attribute__((ext_vector_type(16)));

// block formats (ggml/src/ggml-common.h:187-193, 209-214)
#define QK 32
struct __attribute__((packed)) blk_q5_0 { uint16_t d; uint8_t qh[4]; uint8_t qs[16]; };
struct __attribute__((packed)) blk_q8_0 { uint16_t d; int8_t  qs[32]; };
static_assert(sizeof(blk_q5_0) == 22, "q5_0 block is 22 bytes");
static_assert(sizeof(blk_q8_0) == 34, "q8_0 block is 34 bytes");

// 4-d tensor view passed to kernels by value
struct tview {
    char *  p;
    int64_t ne0, ne1, ne2, ne3;
    int64_t nb0, nb1, nb2, nb3;
};

static inline tview make_view(const mi355x_tensor * t) {
    tview v;
    v.p = (char *) t->data;
    v.ne0 = t->ne[0]; v.ne1 = t->ne[1]; v.ne2 = t->ne[2]; v.ne3 = t->ne[3];
    v.nb0 = (int64_t) t->nb[0]; v.nb1 = (int64_t) t->nb[1]; v.nb2 = (int64_t) t->nb[2]; v.nb3 = (int64_t) t->nb[3];
    return v;
}

static inline int64_t nelements(const mi355x_tensor * t) { return t->ne[0]*t->ne[1]*t->ne[2]*t->ne[3]; }

static inline size_t type_size(int type) {
    switch (type) {
        case MI355X_TYPE_F32:  return 4;
        case MI355X_TYPE_F16:  return 2;
        case MI355X_TYPE_I32:  return 4;
        case MI355X_TYPE_Q5_0: return 22;
        case MI355X_TYPE_Q8_0: return 34;
        default: return 0;
    }
}
static inline int blck_size(int type) { return (type == MI355X_TYPE_Q5_0 || type == MI355X_TYPE_Q8_0) ? QK : 1; }

// dims 1..3 of `t` are laid out densely after dim 0 (rows may still be padded: nb1 is free)
static inline bool is_contiguous(const mi355x_tensor * t) {
    size_t ts = type_size(t->type);
    int    bs = blck_size(t->type);
    if (t->nb[0] != ts) return false;
    size_t nb1 = ts * (size_t)(t->ne[0] / bs);
    if (t->ne[1] > 1 && t->nb[1] != nb1) return false;
    if (t->ne[2] > 1 && t->nb[2] != nb1 * (size_t) t->ne[1]) return false;
    if (t->ne[3] > 1 && t->nb[3] != nb1 * (size_t) t->ne[1] * (size_t) t->ne[2]) return false;
    return true;
}

static inline bool same_shape(const mi355x_tensor * a, const mi355x_tensor * b) {
    return a->ne[0] == b->ne[0] && a->ne[1] == b->ne[1] && a->ne[2] == b->ne[2] && a->ne[3] == b->ne[3];
}

static inline int launch_status() {
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? MI355X_OK : MI355X_ERR_HIP;
}

// Device address of the GELU table for the current device; built on the host on first use with the reference's own
// formula and libm (ggml/src/ggml-cpu/ggml-cpu.c:3415-3423, vec.h:432-434) and copied into a __device__ array.
// NULL on failure.
const uint16_t * gelu_table_device();

#ifdef __HIPCC__

__device__ __forceinline__ float h2f(uint16_t h) {
    half_t x;
    __builtin_memcpy(&x, &h, 2);
    return (float) x;
}
__device__ __forceinline__ uint16_t f2h_bits(float f) {
    half_t x = (half_t) f;   // v_cvt_f16_f32: round-to-nearest-even, like the F16C conversion the CPU backend uses
    uint16_t h;
    __builtin_memcpy(&h, &x, 2);
    return h;
}

// Reductions over aligned groups of W = 4 .. 64 lanes, the result in every lane of the group: DPP steps inside the rows
// of 16 lanes (a mirror pairs the lanes as well as an exchange does, for a commutative reduction), a swizzle across two
// rows, a permute across the halves of the wavefront.  A DPP step costs one vector instruction; the ds_bpermute behind
// __shfl_xor costs an LDS round trip, which is what kernels over a handful of rows spend their time waiting for.
template <typename T, int CTRL>
__device__ __forceinline__ T dpp_move(T v) {
    static_assert(sizeof(T) == 4, "one 32-bit register");
    return __builtin_bit_cast(T, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
template <int W, typename T, typename OP>
__device__ __forceinline__ T lanes_reduce(T x, OP op) {
    static_assert(W == 4 || W == 8 || W == 16 || W == 32 || W == 64, "aligned power-of-two groups");
    x = op(x, dpp_move<T, 0xB1>(x));                        // quad_perm [1,0,3,2]
    x = op(x, dpp_move<T, 0x4E>(x));                        // quad_perm [2,3,0,1]
    if (W >= 8)  x = op(x, dpp_move<T, 0x141>(x));          // row_half_mirror
    if (W >= 16) x = op(x, dpp_move<T, 0x140>(x));          // row_mirror
    if (W >= 32) x = op(x, __builtin_bit_cast(T, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, x), 0x401F)));   // lane ^ 16
    if (W >= 64) x = op(x, __shfl_xor(x, 32, WAVE));
    return x;
}
template <int W> __device__ __forceinline__ float lanes_sum(float x) { return lanes_reduce<W>(x, [](float a, float b) { return a + b; }); }
template <int W> __device__ __forceinline__ int   lanes_sum(int x)   { return lanes_reduce<W>(x, [](int a, int b) { return a + b; }); }
template <int W> __device__ __forceinline__ float lanes_max(float x) { return lanes_reduce<W>(x, [](float a, float b) { return fmaxf(a, b); }); }
__device__ __forceinline__ float wave_sum(float v) { return lanes_sum<WAVE>(v); }
__device__ __forceinline__ float wave_max(float v) { return lanes_max<WAVE>(v); }

// a / 127.0f, bit for bit — the scale of a Q8_0 block, amax / 127 (quantize_row_q8_0, ggml-cpu-quants.c:808-865): the product
// with the rounded reciprocal, corrected once by the exact residual.  Three multiply-adds where the division takes twelve
// instructions, and the same result for every finite non-negative float (checked over all 2^31 of them on the host and on
// the device; the harness library's mi355x_probe_div127 repeats the device check).  Infinity and NaN, whose residual is
// NaN, keep the plain product, which is what the division gives for them.
__device__ __forceinline__ float div127(float a) {
    const float r = 1.0f / 127.0f;
    const float q = a * r;
    const float e = __builtin_fmaf(-q, 127.0f, a);
    return e == e ? __builtin_fmaf(e, r, q) : q;
}

// GELU as ggml_vec_gelu_f32 evaluates it (ggml/src/ggml-cpu/vec.h:443-457): outside (-10, 10) the clamps, inside a
// lookup in a 65536-entry table indexed by the f16 bits of x that holds f16(gelu(f32(f16 x))).  `table` is the device
// copy of that table (gelu_table_device below).
__device__ __forceinline__ float gelu_f32(float x, const uint16_t * __restrict__ table) {
    if (x <= -10.0f) return 0.0f;
    if (x >=  10.0f) return x;
    return h2f(table[f2h_bits(x)]);
}

// unaligned little-endian loads from byte-addressed block data
__device__ __forceinline__ uint32_t ld_u16(const uint8_t * p) { return *(const uint16_t *) p; }
__device__ __forceinline__ uint32_t ld_u32_2(const uint8_t * p) {   // 2-byte aligned 32-bit load
    return (uint32_t) *(const uint16_t *) p | ((uint32_t) *(const uint16_t *)(p + 2) << 16);
}

#endif // __HIPCC__
