// Argument blocks of the MUL_MAT kernels (shared by mul_mat.hip and the harness-only instances of its kernels).
#pragma once

#include "common.h"

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef int      v4i_t __attribute__((ext_vector_type(4)));

struct epi_args {
    int          flags;
    float        scale;
    const float *bias;
    const char * residual;   // same strides as dst, f32
    const uint16_t * gelu;   // GELU table (device), set when MI355X_EPI_GELU is
    half_t * image;          // MI355X_EPI_EMIT_F16: where the Q8_0-rounded f16 image of dst goes ([N][M] dense)
};

struct mm_args {
    const char * w; const char * x; char * d;
    int64_t M, N, K;
    int64_t w_nb1, w_nb2, w_nb3;
    int64_t x_nb1, x_nb2, x_nb3;
    int64_t d_nb1, d_nb2, d_nb3;
    int64_t ne12, ne13, r2, r3;      // batch dims of src1/dst and broadcast ratios of src0
    epi_args e;
};
