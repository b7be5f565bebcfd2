// Measurement yardsticks for bench.py — a library of its own (libmi355x_probes.so), loaded by the benchmark and by nothing
// else: no product path links or calls it.
//
//   mi355x_probe_read              a kernel that only streams bytes out of HBM
//   mi355x_probe_mfma              v_mfma_f32_32x32x16_f16 from registers, no memory in the loop
//   mi355x_probe_read_stamped      the read stream with a time stamp per workgroup and chunk
//   mi355x_probe_gemv_tiles_stamped  an instance of the product's own logits kernel (k_gemv_q8_0_tiles, same source) that
//                                  also leaves a time stamp per wavefront and tile
//   mi355x_probe_div127            every finite non-negative float through the kernels' three-instruction a / 127.0f beside the
//                                  division itself: the number of results that differ (the claim is none)
// The stamped forms answer what a stream sustains between its ramp and its tail: the stamps are the device's 100 MHz
// clock (s_memrealtime), one after each unit of work; the caller sorts the completions and divides the bytes finished
// between the 10th and the 90th percentile by the time between them.
#include "../kernels/gemv_q8_0_tiles.h"

#include <stdint.h>

#define PROBE_API extern "C" __attribute__((visibility("default")))

// every lane has eight 16-byte loads in flight; the words are folded so that the loads stay
__global__ void __launch_bounds__(256) k_probe_read(const u32x4 * __restrict__ p, int64_t n16, uint32_t * __restrict__ out) {
    const int64_t stride = (int64_t) gridDim.x * 256;
    int64_t i = (int64_t) blockIdx.x * 256 + threadIdx.x;
    u32x4 acc = { 0, 0, 0, 0 };
    for (; i + 7 * stride < n16; i += 8 * stride) {
        u32x4 v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = p[i + j * stride];
#pragma unroll
        for (int j = 0; j < 8; ++j) acc ^= v[j];
    }
    for (; i < n16; i += stride) acc ^= p[i];
    const uint32_t f = acc.x ^ acc.y ^ acc.z ^ acc.w;
    if (f == 0x9E3779B9u) out[0] = f;                      // (practically never: the loads are kept without a store per thread)
}

// n: bytes at src (16-byte aligned); out: 4 bytes of device memory
PROBE_API int mi355x_probe_read(const void * src, size_t n, void * out, int workgroups, void * stream) {
    if (!src || !out || (uintptr_t) src % 16 != 0 || (uintptr_t) out % 4 != 0 || workgroups < 1 || workgroups > 65535) return MI355X_ERR_INVALID;
    if (n < 16) return MI355X_OK;
    k_probe_read<<<(unsigned) workgroups, 256, 0, (hipStream_t) stream>>>((const u32x4 *) src, (int64_t)(n / 16), (uint32_t *) out);
    return launch_status();
}

// The same stream in chunks of 32 KB per workgroup (eight 16-byte loads per lane), workgroup w taking chunks w, w + grid, ...:
// after each chunk the workgroup's first lane writes the clock into stamps[chunk]; stamps[n_chunks + w] is the workgroup's start.
__global__ void __launch_bounds__(256) k_probe_read_stamped(const u32x4 * __restrict__ p, int64_t n_chunks, uint32_t * __restrict__ out, uint64_t * __restrict__ stamps) {
    if (threadIdx.x == 0) stamps[n_chunks + blockIdx.x] = __builtin_amdgcn_s_memrealtime();
    u32x4 acc = { 0, 0, 0, 0 };
    for (int64_t c = blockIdx.x; c < n_chunks; c += gridDim.x) {
        const u32x4 * q = p + c * 2048 + threadIdx.x;
        u32x4 v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = q[j * 256];
#pragma unroll
        for (int j = 0; j < 8; ++j) acc ^= v[j];
        __syncthreads();                                   // all of the chunk's loads have arrived
        if (threadIdx.x == 0) stamps[c] = __builtin_amdgcn_s_memrealtime();
    }
    const uint32_t f = acc.x ^ acc.y ^ acc.z ^ acc.w;
    if (f == 0x9E3779B9u) out[0] = f;
}

// stamps: (n / 32768 + workgroups) x 8 bytes of device memory; returns the number of 32 KB chunks, or a negative status
PROBE_API int64_t mi355x_probe_read_stamped(const void * src, size_t n, void * out, int workgroups, void * stamps, void * stream) {
    if (!src || !out || !stamps || (uintptr_t) src % 16 != 0 || (uintptr_t) stamps % 8 != 0 || workgroups < 1 || workgroups > 65535) return MI355X_ERR_INVALID;
    const int64_t n_chunks = (int64_t)(n / 32768);
    if (n_chunks < 1) return MI355X_ERR_INVALID;
    k_probe_read_stamped<<<(unsigned) workgroups, 256, 0, (hipStream_t) stream>>>((const u32x4 *) src, n_chunks, (uint32_t *) out, (uint64_t *) stamps);
    const int rc = launch_status();
    return rc ? rc : n_chunks;
}

// four independent accumulators per wavefront: 2 * 32 * 32 * 16 flops per instruction, 4 * iters instructions per wavefront
__global__ void __launch_bounds__(256) k_probe_mfma(int iters, float * __restrict__ out) {
    const half8_t a = { (_Float16)(threadIdx.x & 7), 1, 2, 3, 4, 5, 6, 7 }, b = { 1, 1, 1, 1, 1, 1, 1, (_Float16)(blockIdx.x & 3) };
    float16_t c0 = {}, c1 = {}, c2 = {}, c3 = {};
    for (int i = 0; i < iters; ++i) {
        c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c1, 0, 0, 0);
        c2 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c2, 0, 0, 0);
        c3 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c3, 0, 0, 0);
    }
    const float f = c0[0] + c1[1] + c2[2] + c3[3];
    if (f == -1.0f) out[0] = f;                            // (never: the sums are >= 0; keeps the instructions)
}

PROBE_API int mi355x_probe_mfma(int iters, int workgroups, void * out, void * stream) {
    if (!out || (uintptr_t) out % 4 != 0 || iters < 1 || iters > (1 << 20) || workgroups < 1 || workgroups > 65535) return MI355X_ERR_INVALID;
    k_probe_mfma<<<(unsigned) workgroups, 256, 0, (hipStream_t) stream>>>(iters, (float *) out);
    return launch_status();
}

// The logits product with stamps: `tiles` as mi355x_q8_0_tiles_pack wrote them (K = 1280), `x_q8` the quantized activations as
// mi355x_mul_mat_q8_0_tiles leaves them in its workspace (call it with MI355X_MM_PREPARE_ONLY first), dst f32 [M, N] dense.
// stamps: wavefronts x (1 + tiles per wavefront) x 8 bytes, zeroed by the caller; *wavefronts and *tiles_per_wavefront describe
// the launch, which is the one mi355x_mul_mat_q8_0_tiles makes.  A tile is 16 rows: 16 * K / 32 * 34 bytes of the stream.
PROBE_API int mi355x_probe_gemv_tiles_stamped(const void * tiles, int64_t K, int64_t M, const void * x_q8, int64_t N, void * dst, void * stamps,
                                              int64_t * wavefronts, int64_t * tiles_per_wavefront, void * stream) {
    if (!tiles || !x_q8 || !dst || !wavefronts || !tiles_per_wavefront || K != 1280 || M < 1 || N < 1 || N > 8) return MI355X_ERR_INVALID;
    mm_args a;
    a.K = K; a.M = M; a.N = N;
    a.w = (const char *) tiles; a.x = (const char *) x_q8; a.d = (char *) dst;
    a.w_nb1 = a.w_nb2 = a.w_nb3 = 0; a.x_nb1 = a.x_nb2 = a.x_nb3 = 0;
    a.d_nb1 = M * 4; a.d_nb2 = a.d_nb3 = 0;
    a.ne12 = a.ne13 = a.r2 = a.r3 = 1;
    a.e.flags = 0; a.e.scale = 1.0f; a.e.bias = nullptr; a.e.residual = nullptr; a.e.gelu = nullptr; a.e.image = nullptr;
    const int64_t n_tiles = (M + 15) / 16, resident = 256 * 2 * 4;
    const int64_t rounds = (n_tiles + resident - 1) / resident;
    const int64_t waves = (n_tiles + rounds - 1) / rounds;
    const unsigned grid = (unsigned)(waves / 4 > 0 ? waves / 4 : 1);
    *wavefronts = (int64_t) grid * 4;
    *tiles_per_wavefront = (n_tiles + *wavefronts - 1) / *wavefronts;
    if (!stamps) return MI355X_OK;                         // (sizes only)
    k_gemv_q8_0_tiles<20, true><<<grid, 256, 0, (hipStream_t) stream>>>(a, (uint64_t *) stamps);
    return launch_status();
}


// ---- div127 (kernels/common.h) against the division, over every finite non-negative float
__global__ void __launch_bounds__(256) k_probe_div127(unsigned long long * __restrict__ differing) {
    const uint64_t stride = (uint64_t) gridDim.x * blockDim.x;
    unsigned long long n = 0;
    for (uint64_t i = (uint64_t) blockIdx.x * blockDim.x + threadIdx.x; i <= 0x7f800000u; i += stride) {      // (up to and with infinity)
        const float a = __builtin_bit_cast(float, (uint32_t) i);
        const float want = a / 127.0f, got = div127(a);
        n += __builtin_bit_cast(uint32_t, want) != __builtin_bit_cast(uint32_t, got);
    }
    if (n) atomicAdd(differing, n);
}
// differing: 8 bytes of device memory, zeroed by the call; the count is there when the stream has finished
PROBE_API int mi355x_probe_div127(void * differing, void * stream) {
    if (!differing || (uintptr_t) differing % 8 != 0) return MI355X_ERR_INVALID;
    if (hipMemsetAsync(differing, 0, 8, (hipStream_t) stream) != hipSuccess) return MI355X_ERR_HIP;
    k_probe_div127<<<2048, 256, 0, (hipStream_t) stream>>>((unsigned long long *) differing);
    return launch_status();
}

// The path from global memory into a CU that the GEMM operands take.  Every wavefront issues rounds of eight 1 KB loads (a
// lane's 16 bytes of a 128-byte row piece, rows 2560 bytes apart as in an f16 operand with K = 1280), either straight into LDS
// (global_load_lds_dwordx4, one round in flight behind the one being issued) or into registers (all eight awaited).
// span = 0: every wavefront reads the same 8 KB, which stay in the L1; span > 0: the workgroups start at scattered rows of
// [src, src + span) and walk 20 K steps of 128 bytes, round and round — 2 MB stay in every L2, the 17 MB of an FFN-up
// product's operands do not.  clocks[2 w], clocks[2 w + 1]: s_memtime and s_memrealtime (100 MHz) ticks of workgroup w's loop.
// Bytes moved: workgroups * 4 wavefronts * iters * 8 KB.  `src` must hold span + 1 MB.
template <bool TO_LDS>
__global__ void __launch_bounds__(256, 2) k_probe_load_path(const char * __restrict__ src, size_t span, int iters, unsigned long long * __restrict__ clocks, u32x4 * __restrict__ sink) {
    extern __shared__ __attribute__((aligned(16))) char probe_lds[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const size_t row0 = ((size_t) blockIdx.x * 37 % 1024) * 128 + wave * 8 + (lane >> 3);
    const char * p = span == 0 ? src + lane * 16 : src + (row0 * 2560 + (lane & 7) * 16) % span;
    const size_t istep = span == 0 ? 1024 : (size_t) 32 * 2560, kstep = span == 0 ? 0 : 128;
    u32x4 acc = { 0, 0, 0, 0 };
    const unsigned long long c0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
    for (int it = 0; it < iters; ++it) {
        const size_t ko = (size_t)(it % 20) * kstep;
        char * dst = probe_lds + ((it & 1) * 32 + wave * 8) * 1024;
        if (TO_LDS) {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(p + ko + (size_t) i * istep),
                                                 (__attribute__((address_space(3))) void *)(dst + i * 1024), 16, 0, 0);
            __builtin_amdgcn_s_waitcnt((8 & 15) | ((8 >> 4) << 14) | (7 << 4) | (15 << 8));      // vmcnt(8): the round before has landed
        } else {
            u32x4 v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = __builtin_nontemporal_load((const u32x4 *)(p + ko + (size_t) i * istep));
#pragma unroll
            for (int i = 0; i < 8; ++i) acc ^= v[i];
        }
    }
    __builtin_amdgcn_s_waitcnt(0);
    if (threadIdx.x == 0) { clocks[2 * blockIdx.x] = __builtin_amdgcn_s_memtime() - c0; clocks[2 * blockIdx.x + 1] = __builtin_amdgcn_s_memrealtime() - r0; }
    if (!TO_LDS && acc.x == 0x12345678u) sink[0] = acc;
}

PROBE_API int mi355x_probe_load_path(const void * src, size_t span, int to_lds, int iters, int workgroups, void * clocks, void * stream) {
    if (!src || !clocks || (uintptr_t) src % 16 != 0 || (uintptr_t) clocks % 16 != 0 || iters < 1 || iters > (1 << 20) || workgroups < 1 || workgroups > 4096) return MI355X_ERR_INVALID;
    if (span != 0 && span < ((size_t) 1 << 20)) return MI355X_ERR_INVALID;
    // (the last 16 bytes of `clocks`, behind the 2 * workgroups counters, take the register variant's sink)
    u32x4 * sink = (u32x4 *)((unsigned long long *) clocks + 2 * (size_t) workgroups);
    if (to_lds) k_probe_load_path<true ><<<(unsigned) workgroups, 256, 65536, (hipStream_t) stream>>>((const char *) src, span, iters, (unsigned long long *) clocks, sink);
    else        k_probe_load_path<false><<<(unsigned) workgroups, 256, 65536, (hipStream_t) stream>>>((const char *) src, span, iters, (unsigned long long *) clocks, sink);
    return launch_status();
}
