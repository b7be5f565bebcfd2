// Single-op (and small fused-chain) graphs at the shapes whisper emits, run on two ggml backends with the
// same inputs.
#pragma once

#include <functional>
#include <string>
#include <vector>

#include "ggml.h"
#include "ggml-backend.h"

namespace ops {

enum fill_kind {
    FILL_NORMAL,     // scale * N(0,1) + offset, converted / quantized to the tensor's type
    FILL_IDS,        // int32 uniform in [0, range)
    FILL_MASK,       // attention mask of 0 / -inf, f32 or f16: range = 1 beam-style (every row sees the first half of the
                     // keys; of the rest row r sees key k iff k % rows == r), range = 2 causal; rows >= `rows` are all -inf
    FILL_ZERO_TAIL,  // FILL_NORMAL for the first `range` rows of `rows` values each, zeros after: the never-written pad
                     // rows of whisper's kv_pad / kv_cross
};

struct input {
    ggml_tensor * t;
    fill_kind     kind;
    float         scale  = 1.0f;
    float         offset = 0.0f;
    int64_t       range  = 0;     // see fill_kind
    int64_t       rows   = 0;
};

struct built {
    std::vector<input>         inputs;
    std::vector<ggml_tensor *> roots;    // nodes to expand into the graph, in order
    ggml_tensor *              result;   // tensor to read back and compare
};

struct op_case {
    std::string name;
    std::string op;
    std::function<built(ggml_context *)> build;
    double nmse_tol;        // north-star per-op bound is 5e-4
    bool   bit_exact;       // demand identical bytes (dequantization, copies, gathers)
    double flops;           // algorithmic work of one run, for the report
    double bytes;
    bool   heavy;           // skipped by --quick (CPU reference takes seconds)
};

std::vector<op_case> all_cases();

} // namespace ops
