// Synthetic whisper models in the legacy "ggml" container (loader: src/whisper.cpp:1498-1969 of the
// whisper.cpp tree): random-init tensors of a named architecture, matmul weights quantized the way
// examples/quantize does (examples/common-ggml.cpp:138-192), so that the unmodified loader accepts them.
#pragma once

#include <stdint.h>
#include <string>
#include <vector>

namespace synth {

struct arch {
    const char * name;
    int n_vocab, n_audio_ctx, n_audio_state, n_audio_head, n_audio_layer;
    int n_text_ctx, n_text_state, n_text_head, n_text_layer, n_mels;
};

// "tiny", "base", "large-v3", "large-v3-turbo"; plus "micro" (2+2 layers, d=128) for fast CPU tests
const arch * find_arch(const std::string & name);

// ggml_type numbers (ggml/include/ggml.h:351-392)
enum { T_F32 = 0, T_F16 = 1, T_Q5_0 = 6, T_Q8_0 = 8 };
// ggml_ftype numbers (ggml/include/ggml.h:396-417)
enum { FT_F16 = 1, FT_Q8_0 = 7, FT_Q5_0 = 8 };

int ftype_from_name(const std::string & s);      // "f16" | "q8_0" | "q5_0" -> FT_*, -1 if unknown
int wtype_of_ftype(int ftype);

// deterministic N(0,1) from (seed, index): the same value on any thread count
float normal_at(uint64_t seed, uint64_t index);

// quantize_row_q5_0_ref / quantize_row_q8_0_ref (ggml/src/ggml-quants.c:105-143, 194-215); k multiple of 32
void quantize_q5_0(const float * x, void * y, int64_t k);
void quantize_q8_0(const float * x, void * y, int64_t k);
uint16_t f32_to_f16(float f);                    // round-to-nearest-even, like GGML_FP32_TO_FP16 with F16C
float    f16_to_f32(uint16_t h);

// bytes of n values of `type` generated as scale * N(0,1) + offset from (seed, index)
std::vector<uint8_t> random_tensor(int type, int64_t n, uint64_t seed, float scale, float offset = 0.0f);

// writes the model file; returns false on I/O error
bool write_model(const std::string & path, const arch & a, int ftype, uint64_t seed);

// synthetic log-mel window [n_mels x n_len], row-major by mel bin, built as
// (max(x, max(x) - 8) + 4) / 4 with x = log10 of Exp(1)-distributed power (src/whisper.cpp:3246-3259)
std::vector<float> synthetic_mel(int n_mels, int n_len, uint64_t seed);

} // namespace synth
