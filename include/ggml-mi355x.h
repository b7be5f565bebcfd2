/*
 * ggml-mi355x.h — public entry points of the MI355X (gfx950) ggml compute backend.
 *
 * The backend is a plugin for ggml's backend interface (ggml/src/ggml-backend-impl.h:17-207 of the
 * whisper.cpp tree): it implements the buffer-type, buffer, backend(stream), device and reg vtables
 * and is found by a ggml host in either of two ways:
 *
 *   - dynamically: ggml_backend_load("libggml-mi355x.so") (ggml/include/ggml-backend.h:228) resolves
 *     ggml_backend_score() and ggml_backend_init() (ggml/src/ggml-backend-impl.h:215-218,
 *     ggml/src/ggml-backend-reg.cpp:227-271) and registers the returned reg;
 *   - statically: the host calls ggml_backend_register(ggml_backend_mi355x_reg())
 *     (ggml/src/ggml-backend-impl.h:210), the same pattern as ggml_backend_cuda_reg()
 *     (ggml/include/ggml-cuda.h:45).
 *
 * This header is compiled against the host tree's ggml.h / ggml-backend.h, like every other backend's
 * public header (ggml/include/ggml-cuda.h:3-4).
 */
#pragma once

#include "ggml.h"
#include "ggml-backend.h"

#ifdef __cplusplus
extern "C" {
#endif

#define GGML_MI355X_NAME "MI355X"

/* counterpart of ggml_backend_cuda_reg (ggml/include/ggml-cuda.h:45) */
GGML_BACKEND_API ggml_backend_reg_t         ggml_backend_mi355x_reg(void);
/* counterpart of ggml_backend_cuda_init (ggml/include/ggml-cuda.h:23); NULL if `device` is not a gfx950 GPU */
GGML_BACKEND_API ggml_backend_t             ggml_backend_mi355x_init(int device);
/* counterpart of ggml_backend_is_cuda (ggml/include/ggml-cuda.h:25) */
GGML_BACKEND_API bool                       ggml_backend_is_mi355x(ggml_backend_t backend);
/* counterpart of ggml_backend_cuda_buffer_type (ggml/include/ggml-cuda.h:28) */
GGML_BACKEND_API ggml_backend_buffer_type_t ggml_backend_mi355x_buffer_type(int device);
/* counterpart of ggml_backend_cuda_get_device_count (ggml/include/ggml-cuda.h:36): number of gfx950 devices */
GGML_BACKEND_API int                        ggml_backend_mi355x_get_device_count(void);

/* dynamic-loading entry points (ggml/src/ggml-backend-impl.h:215-218) */
GGML_BACKEND_API ggml_backend_reg_t ggml_backend_init(void);
GGML_BACKEND_API int                ggml_backend_score(void);

/*
 * Extras reachable through ggml_backend_reg_get_proc_address(reg, name) (ggml/include/ggml-backend.h:185-200):
 *
 *   "ggml_backend_get_features"        ggml_backend_get_features_t
 *   "ggml_backend_mi355x_set_option"   ggml_backend_mi355x_set_option_t
 *   "ggml_backend_mi355x_get_stats"    ggml_backend_mi355x_get_stats_t
 *   "ggml_backend_mi355x_get_counters" ggml_backend_mi355x_get_counters_t
 *   "ggml_backend_mi355x_log_mel"      ggml_backend_mi355x_log_mel_t
 */

/* Options: "fuse" (0/1: fold bias/activation/residual/LayerNorm-affine neighbours into one kernel, default 1),
 * "profile" (0/1: bracket every kernel with HIP events on the backend's stream, default 0),
 * "exact" (0/1, default 0: 0 reproduces the two roundings that the reference's CPU backend applies — Q8_0-rounded
 * activations in front of quantized MUL_MAT, f16 key-by-key V accumulation in FLASH_ATTN_EXT; 1 keeps f16 activations
 * and f32 accumulators, which is closer to exact arithmetic and further from the reference),
 * "fa_accum" (0..3, default 0: how FLASH_ATTN_EXT accumulates V.  0: key by key with an f16 accumulator that is rounded
 * after every key — the reference's sequence (ops.cpp:6793-6807), and the only setting that keeps whole-model logits
 * within 1e-3 NMSE of the CPU backend.  Bit 0: f32 accumulators with both products on the matrix cores for more than 8 queries —
 * five times faster, within the per-op bound, but the reference's f16 rounding is then missing and whole-model logits sit
 * several 1e-3 away.  Bit 1: f32 accumulators for a decode step's few queries; the decoder's layers alone move the
 * logits to 6e-3 … 8e-3 NMSE).
 * "fa_chain" (0..2, default 2: the arithmetic of one step of that key-by-key sequence.  2: the factor rounded to f16 and
 * one fused f16 multiply-add per element, the reference's ggml_vec_mad_f16 on hardware with f16 vector arithmetic
 * (vec.h:180-203 with GGML_F16_VEC_FMA = vfmaq_f16, simd-mappings.h:68-105) — a third of the vector instructions where a
 * launch has more than 8 queries, one dependent instruction per key instead of two in a decode step.  1: that form only
 * where a launch has more than 8 queries.  0: f32 fma followed by an f16 store everywhere, the same function in the
 * reference's x86 build.  Whole-model logits stay within the same 1e-3 of the x86 CPU backend with all three.)
 * The environment variables GGML_MI355X_FUSE, GGML_MI355X_PROFILE, GGML_MI355X_EXACT, GGML_MI355X_FA_ACCUM and
 * GGML_MI355X_FA_CHAIN give the initial values.
 * backend == NULL addresses every live MI355X backend of the process (a host such as whisper.cpp keeps its
 * backends private). */
typedef int (*ggml_backend_mi355x_set_option_t)(ggml_backend_t backend, const char * name, int value);

/* Per-kernel statistics gathered while "profile" is on: writes a JSON array
 * [{"kernel": name, "calls": n, "ms": total, "bytes": algorithmic bytes, "flops": algorithmic flops}, ...]
 * into buf (at most size bytes, NUL-terminated), resets the counters when `reset` is non-zero and returns the
 * length needed. */
typedef size_t (*ggml_backend_mi355x_get_stats_t)(ggml_backend_t backend, char * buf, size_t size, int reset);

/* What graph_compute was handed and did since the last reset (always counted, whatever "profile" says):
 * out[0] graph_compute calls, out[1] nodes of the graphs as received, out[2] those of them that are not view ops or empty
 * tensors (every one of them is carried out by a launch of this backend: there is no other path), out[3] kernel
 * launches, out[4] get_tensor calls served from the pinned host mirror of a graph output, out[5] get_tensor calls that
 * were a blocking device-to-host copy, out[6] nanoseconds of host time inside graph_compute (planning and queueing the
 * launches), out[7] nanoseconds the host waited inside synchronize, out[8] graphs that held a FLASH_ATTN_EXT node with at
 * most 8 queries (decode steps), out[9] the largest number of keys such a node with a mask saw (n_kv: the extent of the
 * self-attention cache a step walked; a maximum, not a sum).  A host that sees one call per graph it computes, with the graph's
 * full node count, knows that the scheduler (ggml_backend_sched_split_graph, ggml/src/ggml-backend.cpp:863-1317) left
 * no node to another backend. */
#define GGML_MI355X_N_COUNTERS 10
typedef void (*ggml_backend_mi355x_get_counters_t)(ggml_backend_t backend, int64_t out[GGML_MI355X_N_COUNTERS], int reset);

/* The log-mel front end (log_mel_spectrogram, src/whisper.cpp:3181-3270 — what whisper_pcm_to_mel, :3881, runs on
 * host threads) on device `device`, for a host that holds its samples in host memory: uploads the 16 kHz f32 samples
 * and the model's filter bank [n_mel][201], runs mi355x_log_mel_spectrogram and downloads mel [n_mel][n_len] into
 * `mel` (capacity in floats).  Returns n_len = (n_samples + 480000) / 160, which is what whisper_set_mel takes next to
 * `mel`, or a negative mi355x status; with mel == NULL it only returns n_len.  whisper_full(ctx, params, NULL, 0) then
 * transcribes from that mel without computing its own (src/whisper.cpp:5492).  `device_ms`, when not NULL, receives
 * the time of the device work alone (HIP events around the kernels; the rest of the call is the allocation and the
 * three copies). */
typedef int64_t (*ggml_backend_mi355x_log_mel_t)(int device, const float * samples, int64_t n_samples, const float * filters, int n_mel,
                                                 float * mel, int64_t mel_capacity, float * device_ms);

#ifdef __cplusplus
}
#endif
