// Log-mel front end on the device: 16 kHz samples -> the [n_mel, n_len] input of the encoder's conv stem
// (log_mel_spectrogram, src/whisper.cpp:3181-3270, and its worker :3113-3179).
//
// The reference extends the signal by 200 reflected samples in front and 30 s + 200 samples of zeros behind, takes
// 400-sample frames every 160 samples under a periodic Hann window, a 400-point transform per frame (f32, halved down
// to 25-point sums), the power of bins 0 .. 200, a [n_mel, 201] filter bank, log10(max(., 1e-10)), and finally raises
// everything below (global maximum - 8) to it and maps x to (x + 4) / 4.
//
// Here a frame's transform is the direct sum over its 400 samples — 0.48 G multiply-adds for a 30 s window, little for this
// part, where the halving scheme would be 25 x less arithmetic but a dependent chain of small passes — in f64: with
// f64 sums the result does not depend on the order of the terms, so it is the mathematical value to 1e-12 where the
// reference's f32 transform is within about 1e-6 of it (v_fma_f64 issues at half the f32 rate, 4.2 ns per wavefront,
// which is what the kernel's time comes to).
// One workgroup takes 12 consecutive frames: thread k < 201 owns bin k of all 12 (24 f64 accumulators), the windowed
// samples sit in LDS sample-major (the 12 frames' values of one sample index are one 96-byte broadcast read), the
// twiddles cos, sin(2 pi i / 400) are a 400-entry LDS table walked by (k n) mod 400.  Then thread (band j, half of
// the frames) applies the filter bank from a transposed copy ([208][n_mel], zero rows past bin 200: lanes = bands read
// consecutive floats, 16 rows per request and the next request in flight) to the powers, which have replaced the
// samples in LDS.  Frames past the end of the signal are not computed: they hold log10(1e-10) by definition, and the
// last pass writes that.  Three launches: filters transposed + maximum cleared; frames; clamp and scale.
#include "common.h"

#define MEL_NFFT   400
#define MEL_HOP    160
#define MEL_BINS   201
#define MEL_FRAMES 12           // frames per workgroup: the 3002 frames of a 30 s window make 251 workgroups for 256 CUs
#define MEL_CHUNK  16           // filter-bank rows a thread requests at a time
#define MEL_ROWS   208          // rows of the transposed filter bank: 201 bins padded with zero rows to whole chunks
#define MEL_MAX_BANDS 128

typedef double double2_t __attribute__((ext_vector_type(2)));

// order-preserving map of f32 onto signed integers, for atomicMax
__device__ __forceinline__ int   mel_key(float x)  { const int i = __float_as_int(x); return i ^ ((i >> 31) & 0x7fffffff); }
__device__ __forceinline__ float mel_unkey(int k)  { return __int_as_float(k ^ ((k >> 31) & 0x7fffffff)); }

__global__ void k_log_mel_setup(const float * __restrict__ filters, int n_mel, float * __restrict__ filters_t, int * __restrict__ max_key) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;          // element of the transposed copy: (k, j)
    if (i < MEL_ROWS * n_mel) { const int k = i / n_mel, j = i % n_mel; filters_t[i] = k < MEL_BINS ? filters[j * MEL_BINS + k] : 0.0f; }
    if (i == 0) *max_key = mel_key(-INFINITY);
}

__global__ void __launch_bounds__(256) k_log_mel_frames(const float * __restrict__ samples, int64_t n_samples, const float * __restrict__ filters_t,
                                                       int n_mel, int64_t n_frames, int64_t n_len, float * __restrict__ mel, int * __restrict__ max_key) {
    __shared__ __attribute__((aligned(16))) double    fr[MEL_NFFT * MEL_FRAMES];   // windowed samples [n][frame]; later powers [bin][frame]
    __shared__ __attribute__((aligned(16))) double2_t cs[MEL_NFFT];                // (cos, sin)(2 pi i / 400)
    const int tid = threadIdx.x;
    const int64_t i0 = (int64_t) blockIdx.x * MEL_FRAMES;

    for (int i = tid; i < MEL_NFFT; i += 256) {
        double s, c;
        sincospi(2.0 * i / MEL_NFFT, &s, &c);
        cs[i] = (double2_t){ c, s };
    }
    __syncthreads();
    // sample p of the extended signal: reflected head, the samples, zeros.  Every load is unconditional (index clamped,
    // value selected afterwards) and all of a thread's loads are requested before the first is used: behind a condition
    // each of the 19 rounds would wait for its own trip to memory.
    {
        constexpr int ROUNDS = (MEL_NFFT * MEL_FRAMES + 255) / 256;
        float xs[ROUNDS];
#pragma unroll
        for (int r = 0; r < ROUNDS; ++r) {
            const int e = tid + r * 256, n = e / MEL_FRAMES, f = e % MEL_FRAMES;
            const int64_t p = (i0 + f) * MEL_HOP + n;
            int64_t at = p < MEL_NFFT / 2 ? MEL_NFFT / 2 - p : p - MEL_NFFT / 2;
            at = at < n_samples ? at : n_samples - 1;
            const float x = samples[at];
            xs[r] = p < n_samples + MEL_NFFT / 2 ? x : 0.0f;
        }
#pragma unroll
        for (int r = 0; r < ROUNDS; ++r) {
            const int e = tid + r * 256;
            if (e < MEL_NFFT * MEL_FRAMES) fr[e] = (0.5 * (1.0 - cs[e / MEL_FRAMES].x)) * (double) xs[r];
        }
    }
    __syncthreads();

    // filter bank role: thread = (band j, half of the frames).  Its filter column comes MEL_CHUNK rows per request through a
    // ring of four chunks, so that a request has three chunks' worth of arithmetic to arrive in.
    const int j = tid & (MEL_MAX_BANDS - 1), fh = tid >> 7;
    const float * fcol = filters_t + (j < n_mel ? j : 0);
    constexpr int CHUNKS = MEL_ROWS / MEL_CHUNK;
    static_assert(CHUNKS % 4 == 1, "rounds of four plus one");
    float wr[4][MEL_CHUNK];
    auto request = [&](float (&w)[MEL_CHUNK], int c) __attribute__((always_inline)) {
        c = c < CHUNKS ? c : CHUNKS - 1;
#pragma unroll
        for (int i = 0; i < MEL_CHUNK; ++i) w[i] = fcol[(c * MEL_CHUNK + i) * n_mel];
    };

    double pw[MEL_FRAMES];
    if (tid < MEL_BINS) {
        double re[MEL_FRAMES], im[MEL_FRAMES];
#pragma unroll
        for (int f = 0; f < MEL_FRAMES; ++f) { re[f] = 0.0; im[f] = 0.0; }
        // one sample index per step: its twiddle and the frames' values are read from LDS a step ahead of their use
        struct step { double2_t w; double2_t x[MEL_FRAMES / 2]; };
        int idx = 0;                                                  // (tid * n) mod 400
        auto fetch = [&](step & s, int n) __attribute__((always_inline)) {
            s.w = cs[idx];
            const double2_t * x2 = (const double2_t *)(fr + n * MEL_FRAMES);
#pragma unroll
            for (int f = 0; f < MEL_FRAMES / 2; ++f) s.x[f] = x2[f];
            idx += tid; if (idx >= MEL_NFFT) idx -= MEL_NFFT;
        };
        auto mad = [&](const step & s) __attribute__((always_inline)) {
#pragma unroll
            for (int f = 0; f < MEL_FRAMES / 2; ++f) {
                re[2 * f]     = __builtin_fma(s.x[f].x, s.w.x, re[2 * f]);     im[2 * f]     = __builtin_fma(s.x[f].x, s.w.y, im[2 * f]);
                re[2 * f + 1] = __builtin_fma(s.x[f].y, s.w.x, re[2 * f + 1]); im[2 * f + 1] = __builtin_fma(s.x[f].y, s.w.y, im[2 * f + 1]);
            }
        };
        step sa, sb;
        fetch(sa, 0);
#pragma unroll 1
        for (int n = 0; n < MEL_NFFT; n += 2) {
            fetch(sb, n + 1);
            __builtin_amdgcn_sched_barrier(0);
            mad(sa);
            __builtin_amdgcn_sched_barrier(0);
            fetch(sa, n + 2 < MEL_NFFT ? n + 2 : MEL_NFFT - 1);      // (the last one is not used)
            __builtin_amdgcn_sched_barrier(0);
            mad(sb);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int f = 0; f < MEL_FRAMES; ++f) pw[f] = re[f] * re[f] + im[f] * im[f];
    } else {
#pragma unroll
        for (int f = 0; f < MEL_FRAMES; ++f) pw[f] = 0.0;            // rows 201 .. 207 of the power tile meet zero filter rows
    }
    request(wr[0], 0); request(wr[1], 1); request(wr[2], 2); request(wr[3], 3);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();                                                  // every bin is done with the samples
    if (tid < MEL_ROWS) {
#pragma unroll
        for (int f = 0; f < MEL_FRAMES; ++f) fr[tid * MEL_FRAMES + f] = pw[f];
    }
    __syncthreads();

    float vmax = -INFINITY;
    {
        double sum[MEL_FRAMES / 2];
#pragma unroll
        for (int f = 0; f < MEL_FRAMES / 2; ++f) sum[f] = 0.0;
        auto use = [&](const float (&w)[MEL_CHUNK], int c) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < MEL_CHUNK; ++i) {
                const double wk = (double) w[i];
                const double2_t * p2 = (const double2_t *)(fr + (c * MEL_CHUNK + i) * MEL_FRAMES + fh * (MEL_FRAMES / 2));
#pragma unroll
                for (int f = 0; f < MEL_FRAMES / 4; ++f) {
                    const double2_t p = p2[f];
                    sum[2 * f] = __builtin_fma(p.x, wk, sum[2 * f]); sum[2 * f + 1] = __builtin_fma(p.y, wk, sum[2 * f + 1]);
                }
            }
        };
        // rounds of four chunks in a loop that is not unrolled (unrolled, every request moves to the top and the registers
        // run out); a chunk's buffer is requested again as soon as it is used up
#pragma unroll 1
        for (int c = 0; c < CHUNKS - 1; c += 4) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                use(wr[q], c + q);
                __builtin_amdgcn_sched_barrier(0);
                request(wr[q], c + q + 4);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        use(wr[0], CHUNKS - 1);
        if (j < n_mel) {
#pragma unroll
            for (int f = 0; f < MEL_FRAMES / 2; ++f) {
                const int64_t i = i0 + fh * (MEL_FRAMES / 2) + f;
                if (i < n_frames) {
                    const float v = (float) log10(sum[f] > 1e-10 ? sum[f] : 1e-10);
                    mel[(int64_t) j * n_len + i] = v;
                    vmax = fmaxf(vmax, v);
                }
            }
        }
    }
    vmax = wave_max(vmax);
    if ((tid & 63) == 0 && vmax > -INFINITY) atomicMax(max_key, mel_key(vmax));
}

// frames past the signal hold log10(1e-10); everything below (maximum - 8) is raised to it; (x + 4) / 4 (in f64, as the
// reference's expressions are)
__global__ void k_log_mel_finish(float * __restrict__ mel, int n_mel, int64_t n_frames, int64_t n_len, const int * __restrict__ max_key) {
    const int64_t e = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= (int64_t) n_mel * n_len) return;
    const int64_t i = e % n_len;
    float top = mel_unkey(*max_key);
    if (n_frames < n_len) top = fmaxf(top, -10.0f);
    const double floor_ = (double) top - 8.0;
    float x = i < n_frames ? mel[e] : -10.0f;
    if ((double) x < floor_) x = (float) floor_;
    mel[e] = (float)(((double) x + 4.0) / 4.0);
}

extern "C" int64_t mi355x_log_mel_n_len(int64_t n_samples) { return n_samples > 0 ? (n_samples + 30 * 16000) / MEL_HOP : 0; }

extern "C" size_t mi355x_log_mel_workspace_size(int n_mel) {
    if (n_mel < 1 || n_mel > MEL_MAX_BANDS) return 0;
    return ((size_t) MEL_ROWS * n_mel * 4 + 256 + 255) / 256 * 256;
}

extern "C" int mi355x_log_mel_spectrogram(const float * samples, int64_t n_samples, const float * filters, int n_mel, float * mel,
                                          void * workspace, size_t workspace_size, void * stream) {
    if (!samples || !filters || !mel) return MI355X_ERR_INVALID;
    if (n_mel < 1 || n_mel > MEL_MAX_BANDS) return MI355X_ERR_UNSUPPORTED;
    if (n_samples <= MEL_NFFT / 2 || n_samples > (int64_t) 1 << 40) return MI355X_ERR_INVALID;      // the reflected head reads samples 1 .. 200
    if (!workspace || workspace_size < mi355x_log_mel_workspace_size(n_mel) || (uintptr_t) workspace % 16 != 0) return MI355X_ERR_WORKSPACE;
    hipStream_t st = (hipStream_t) stream;
    const int64_t n_len = mi355x_log_mel_n_len(n_samples);
    int64_t n_frames = (n_samples + MEL_NFFT / 2) / MEL_HOP + 1;
    if (n_frames > n_len) n_frames = n_len;
    float * filters_t = (float *) workspace;
    int *   max_key   = (int *)((char *) workspace + (size_t) MEL_ROWS * n_mel * 4);
    const int64_t groups = (n_frames + MEL_FRAMES - 1) / MEL_FRAMES, elems = (int64_t) n_mel * n_len;
    if (groups > 0x7fffffff || (elems + 255) / 256 > 0x7fffffff) return MI355X_ERR_UNSUPPORTED;
    k_log_mel_setup<<<(MEL_ROWS * n_mel + 255) / 256, 256, 0, st>>>(filters, n_mel, filters_t, max_key);
    if (const int rc = launch_status()) return rc;
    k_log_mel_frames<<<(unsigned) groups, 256, 0, st>>>(samples, n_samples, filters_t, n_mel, n_frames, n_len, mel, max_key);
    if (const int rc = launch_status()) return rc;
    k_log_mel_finish<<<(unsigned)((elems + 255) / 256), 256, 0, st>>>(mel, n_mel, n_frames, n_len, max_key);
    return launch_status();
}
