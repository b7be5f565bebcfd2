// The few-column product over a Q8_0 matrix repacked into matrix-core operand order (mi355x_q8_0_tiles_pack): the kernel
// behind mi355x_mul_mat_q8_0_tiles.  In a header because the measurement harness compiles an instance of the same code that
// also leaves time stamps; the product's instance (mul_mat.hip) has STAMPS = false.
#pragma once

#include "mul_mat_args.h"

#include <type_traits>

#define Q8T_STEP 1088      // bytes of 16 rows x one pair of blocks

// the activations as they come: quantized ahead, in global memory
struct q8t_no_prologue {
    __device__ __forceinline__ void request() {}
    __device__ __forceinline__ const char * finish(const char * x) { return x; }
};

// a.w: the tiles; a.x: the activations quantized ahead (layout of k_quantize_x_q8); K = 64 KSTEPS
// STAMPS (measurement instances only, never the product's): every wavefront leaves the device's 100 MHz clock at its start and
// after each of its tiles in `stamps` ([wavefront][1 + tiles per wavefront]; 0 = no such tile), from which the rate of the
// stream between its ramp and its tail can be read.
// `pro`: where the quantized activations come from.  request() issues its loads in front of the first tile's, finish() runs
// behind them and returns the activations' address (the plain product: a.x as passed; with a LayerNorm in front, the rows
// it has just normalized and rounded, in LDS) — the first tile takes 7 us to arrive, which is the time such a prologue has.
template <int KSTEPS, bool STAMPS, typename PRO>
__device__ __forceinline__ void gemv_q8_0_tiles_body(const mm_args & a, uint64_t * stamps, PRO pro) {
    __shared__ __attribute__((aligned(16))) float xs_lds[KSTEPS * 2 * 8];       // activation scales, [block][column 0 .. 7]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, g = lane >> 4;
    const int nbk = KSTEPS * 2;
    const int64_t n_tiles = (a.M + 15) / 16;
    const int64_t stride = (int64_t) gridDim.x * 4;
    int64_t tile = (int64_t) blockIdx.x * 4 + wave;
    constexpr int H = KSTEPS / 2;
    u32x4 wq[2][H]; uint32_t wd[2][H];
    const int q_ofs = lane * 16, d_ofs = 1024 + ((g >> 1) * 16 + r) * 2;
    auto request = [&](int half, int64_t t) __attribute__((always_inline)) {
        const char * p = a.w + (t * KSTEPS + half * H) * Q8T_STEP;
#pragma unroll
        for (int s = 0; s < H; ++s) {
            wq[half][s] = *(const u32x4 *)(p + s * Q8T_STEP + q_ofs);
            wd[half][s] = *(const uint16_t *)(p + s * Q8T_STEP + d_ofs);
        }
    };
    const int64_t tiles_per_wave = (n_tiles + stride - 1) / stride;
    uint64_t * my_stamps = nullptr;
    if (STAMPS) {
        my_stamps = stamps + tile * (1 + tiles_per_wave);
        if (lane == 0) my_stamps[0] = __builtin_amdgcn_s_memrealtime();
    }
    const bool live = tile < n_tiles;                   // (a matrix of fewer than 64 rows)
    if constexpr (!std::is_same<PRO, q8t_no_prologue>::value) {
        pro.request();
        __builtin_amdgcn_sched_barrier(0);
    }
    request(0, live ? tile : n_tiles - 1);
    __builtin_amdgcn_sched_barrier(0);
    request(1, live ? tile : n_tiles - 1);
    __builtin_amdgcn_sched_barrier(0);

    // activations: quants as the A operand (lane = A row r, 16 k of group g), scales through LDS
    const char *  xq = pro.finish(a.x);
    const float * xd = (const float *)(xq + (size_t) a.N * a.K);
    const int col = r & 7;
    const bool mine = ((r < 8) == (g < 2)) && col < a.N;
    v4i_t xa[KSTEPS];
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
        xa[s] = (v4i_t){ 0, 0, 0, 0 };
        if (mine) xa[s] = *(const v4i_t *)(xq + (int64_t) col * a.K + 64 * s + 16 * g);
    }
    for (int i = threadIdx.x; i < nbk * 8; i += 256) xs_lds[i] = (i & 7) < a.N ? xd[(i & 7) * nbk + (i >> 3)] : 0.0f;
    __syncthreads();
    if (!live) return;
    const float * xsl = xs_lds + (g >> 1) * 8 + (g & 1) * 4;      // + 16 per pair of blocks
    const bool out_f16 = a.e.flags & MI355X_EPI_OUT_F16;

    auto do_tile = [&](auto again) __attribute__((always_inline)) {
        float acc[4] = { 0.0f, 0.0f, 0.0f, 0.0f };
#pragma unroll
        for (int half = 0; half < 2; ++half) {
#pragma unroll
            for (int s = 0; s < H; ++s) {
                const u32x4 w = wq[half][s];
                const v4i_t d = __builtin_amdgcn_mfma_i32_16x16x64_i8(xa[half * H + s], (v4i_t){ (int) w.x, (int) w.y, (int) w.z, (int) w.w }, (v4i_t){ 0, 0, 0, 0 }, 0, 0, 0);
                const float dw = h2f((uint16_t) wd[half][s]);
                const float4 x4 = *(const float4 *)(xsl + (half * H + s) * 16);
                acc[0] += (float) d[0] * (dw * x4.x); acc[1] += (float) d[1] * (dw * x4.y);
                acc[2] += (float) d[2] * (dw * x4.z); acc[3] += (float) d[3] * (dw * x4.w);
            }
            if constexpr (decltype(again)::value) {
                request(half, tile + stride);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] += __shfl_xor(acc[i], 32, WAVE);     // even blocks + odd blocks
        const int64_t row = tile * 16 + r;
        if (g < 2 && row < a.M) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int n = 4 * g + i;
                if (n < a.N) {
                    if (out_f16) *(half_t *)(a.d + n * a.d_nb1 + row * 2) = (half_t) acc[i];
                    else         *(float  *)(a.d + n * a.d_nb1 + row * 4) = acc[i];
                }
            }
        }
        if (STAMPS && lane == 0) *++my_stamps = __builtin_amdgcn_s_memrealtime();
    };
    // every tile but the wavefront's last requests the next one's halves as its own are used up
    for (; tile + stride < n_tiles; tile += stride) do_tile(std::true_type{});
    do_tile(std::false_type{});
}

template <int KSTEPS, bool STAMPS>
__global__ void __launch_bounds__(256, 2) k_gemv_q8_0_tiles(mm_args a, uint64_t * stamps) {
    gemv_q8_0_tiles_body<KSTEPS, STAMPS>(a, stamps, q8t_no_prologue{});
}

