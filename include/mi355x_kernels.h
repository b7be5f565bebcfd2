/*
 * mi355x_kernels.h — C ABI of the hand-written gfx950 (MI355X) kernels behind the ggml-mi355x backend.
 *
 * Every entry point takes plain device pointers, element counts and byte strides (the same
 * ne[]/nb[] convention as ggml: ne[0] is the contiguous dimension, nb[i] is the byte stride of
 * dimension i), launches asynchronously on the HIP stream handed in as `stream` (a hipStream_t passed
 * as void*, NULL = default stream) and returns MI355X_OK or a negative error code.  Nothing here
 * allocates device memory; ops that need scratch take a caller-provided workspace.  (The one piece of
 * library-owned device state is the 128 KiB GELU table in a __device__ array, filled by a synchronous
 * copy the first time GELU is used on a device.)
 *
 * Each declaration cites the function of the reference's CPU backend whose results it reproduces
 * (paths relative to the whisper.cpp tree).
 */
#ifndef MI355X_KERNELS_H
#define MI355X_KERNELS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355X_API __attribute__((visibility("default")))

/* element types; numeric values equal the reference's enum ggml_type (ggml/include/ggml.h:351-392) */
enum mi355x_type {
    MI355X_TYPE_F32  = 0,
    MI355X_TYPE_F16  = 1,
    MI355X_TYPE_Q5_0 = 6,  /* block_q5_0, 22 bytes per 32 weights (ggml/src/ggml-common.h:187-193) */
    MI355X_TYPE_Q8_0 = 8,  /* block_q8_0, 34 bytes per 32 weights (ggml/src/ggml-common.h:209-214) */
    MI355X_TYPE_I32  = 26,
};

enum mi355x_status {
    MI355X_OK               =  0,
    MI355X_ERR_UNSUPPORTED  = -1,  /* type / layout combination has no kernel */
    MI355X_ERR_INVALID      = -2,  /* inconsistent shapes, NULL pointer, misaligned operand */
    MI355X_ERR_WORKSPACE    = -3,  /* workspace missing or too small */
    MI355X_ERR_HIP          = -4,  /* the HIP runtime reported an error at launch */
};

/* A strided view of device memory.  For block-quantized types ne[0] counts weights (a multiple of 32)
 * and nb[0] is the block size in bytes. */
typedef struct mi355x_tensor {
    void *  data;
    int32_t type;       /* enum mi355x_type */
    int32_t _pad;
    int64_t ne[4];
    size_t  nb[4];
} mi355x_tensor;

/* epilogue fused into MUL_MAT: dst = act((src0^T src1) + bias) * scale + residual, each part optional */
enum mi355x_epilogue_flags {
    MI355X_EPI_NONE     = 0,
    MI355X_EPI_BIAS     = 1,   /* + bias[m]      (f32, ne0 = dst ne0)            : ggml ADD with a row vector  */
    MI355X_EPI_GELU     = 2,   /* tanh-GELU       (ggml/src/ggml-cpu/vec.h:432-457)                            */
    MI355X_EPI_SCALE    = 4,   /* * scale         (ggml/src/ggml-cpu/ops.cpp:3840-3878)                        */
    MI355X_EPI_RESIDUAL = 8,   /* + residual[m,n] (f32, same shape and strides as dst)                         */
    MI355X_EPI_BIAS_COL = 16,  /* + bias[n]       (f32, one value per dst row n: conv bias [1,d], broadcast along ne0) */
    MI355X_EPI_OUT_F16  = 32,  /* dst is f16 instead of f32 (ggml CPY f32->f16 folded in)                      */
    /* not epilogue parts, but options of the same call: */
    MI355X_MM_EXACT_ACT = 64,  /* GEMM path: keep src1 at f16 precision instead of rounding it to Q8_0 first   */
    MI355X_MM_WS_READY  = 128, /* GEMM path: `workspace` already holds the f16 image of this call's src1 (left
                                  there by the previous call with the same src1): skip the conversion pass     */
    MI355X_MM_ACT_Q8_0  = 256, /* GEMM path, F16 src0 that is the f16 image (mi355x_dequantize_row_f16) of a
                                  quantized weight: round src1 to Q8_0 as for the quantized weight itself      */
    MI355X_EPI_EMIT_F16 = 1024, /* GEMM path, f32 dst with ne0 a multiple of 32: also write to `image` the rows of dst
                                  rounded to Q8_0 like quantize_row_q8_0 and stored as f16(q * d), dense [N][M] — what
                                  the src1 conversion pass of the MUL_MAT that reads dst next would produce            */
    MI355X_EPI_IMAGE_ONLY = 2048, /* with MI355X_EPI_EMIT_F16: write the image only, not dst (whose data pointer may then be
                                  NULL) — for a result whose only readers are products that take the image              */
    MI355X_EPI_EMIT_Q8_0 = 4096, /* few-column path with a workspace, f32 dst with ne0 a multiple of 32, one product per call: also
                                  write to `image` (16-byte aligned) dst quantized to Q8_0 as quantize_row_q8_0 does, in the
                                  layout of mi355x_norm_emit_q8_0 for N rows of ne0 values — what the quantization pass of the
                                  few-column MUL_MAT that reads dst next would write into its workspace                    */
    MI355X_MM_PREPARE_ONLY = 512, /* GEMM path: run only the src1 conversion pass into `workspace` and return; the
                                  product itself then follows in a second call with MI355X_MM_WS_READY (lets a
                                  caller time or overlap the two separately); a no-op on the other paths       */
};

typedef struct mi355x_epilogue {
    int32_t      flags;
    float        scale;
    const void * bias;
    const void * residual;
    void *       image;      /* MI355X_EPI_EMIT_F16 */
} mi355x_epilogue;

/* library / device ---------------------------------------------------------------------------------- */

/* Version of this ABI (bumped on any incompatible change). */
MI355X_API int          mi355x_abi_version(void);
/* 1 if HIP device `device` is a gfx950 part, 0 otherwise, negative on HIP error. */
MI355X_API int          mi355x_device_is_gfx950(int device);
MI355X_API const char * mi355x_status_string(int status);

/* quantization formats -------------------------------------------------------------------------------
 * dequantize_row_q5_0 / dequantize_row_q8_0 (ggml/src/ggml-quants.c:296-319, 349-363): y[i] = d * q,
 * bit-exact.  `k` weights (multiple of 32) from `src` (device) to f32 `dst` (device). */
MI355X_API int mi355x_dequantize_row(int type, const void * src, float * dst, int64_t k, void * stream);
/* the same rows as f16: y[i] = f16(d * q), the exact product rounded once to nearest even */
MI355X_API int mi355x_dequantize_row_f16(int type, const void * src, void * dst, int64_t k, void * stream);

/* quantize_row_q8_0 of the CPU backend's AVX2 build (ggml/src/ggml-cpu/ggml-cpu-quants.c:738,808-865):
 * per 32 values d = amax/127 stored as f16, q = round-to-nearest-even(x * (127/amax)).  `k` multiple of 32. */
MI355X_API int mi355x_quantize_row_q8_0(const float * src, void * dst, int64_t k, void * stream);

/* MUL_MAT ---------------------------------------------------------------------------------------------
 * ggml_compute_forward_mul_mat (ggml/src/ggml-cpu/ggml-cpu.c:1266-1458):
 *   dst[m, n, b2, b3] = sum_k src0[k, m, b2/r2, b3/r3] * src1[k, n, b2, b3]
 * src0: Q5_0 | Q8_0 | F16 | F32, ne0 = K contiguous.  src1: F32 | F16, ne0 = K contiguous.  dst: F32
 * (F16 with MI355X_EPI_OUT_F16), ne0 = M contiguous.  `epi` may be NULL.
 * Columns n <= MI355X_GEMV_MAX_COLS with a quantized src0 take the HBM-streaming GEMV path, which
 * quantizes src1 to Q8_0 (in LDS) exactly like the CPU backend does (ggml-cpu.c:1328-1363) and
 * accumulates integer block dot products like ggml_vec_dot_q5_0_q8_0 / ggml_vec_dot_q8_0_q8_0
 * (ggml-cpu-quants.c:2930, 3597).  Everything else runs the MFMA GEMM: f16 operands, f32 accumulation.
 * Its operands are brought to dense f16 rows in `workspace` (256-byte aligned, size from
 * mi355x_mul_mat_workspace_size) by one pass each: an F32 src1 first, then a src0 that is not F16 (blocks
 * expanded to f16(d*q)).  With quantized weights the src1 pass also rounds to Q8_0 — it writes f16(d*q) of
 * the Q8_0 blocks — because that rounding is part of what the reference computes; MI355X_MM_EXACT_ACT turns
 * it off.  A caller that reuses a quantized weight keeps its f16 image (mi355x_dequantize_row_f16) and
 * passes that as an F16 src0 with MI355X_MM_ACT_Q8_0, which skips the src0 pass. */
#define MI355X_GEMV_MAX_COLS 8
/* name of the kernel mi355x_mul_mat would launch for these operands ("mul_mat.gemm_q5_0", "mul_mat.gemv_q8_0", ...);
 * a static string, used to label profiles */
MI355X_API const char * mi355x_mul_mat_kernel_name(const mi355x_tensor * src0, const mi355x_tensor * src1);
MI355X_API size_t mi355x_mul_mat_workspace_size(const mi355x_tensor * src0, const mi355x_tensor * src1);
MI355X_API int    mi355x_mul_mat(const mi355x_tensor * src0, const mi355x_tensor * src1, const mi355x_tensor * dst,
                                 const mi355x_epilogue * epi, void * workspace, size_t workspace_size, void * stream);

/* mi355x_mul_mat without a workspace argument and without any allocation: the scratch memory (the f16 / Q8_0 forms of the
 * operands that mi355x_mul_mat keeps in `workspace`) is a fixed array of MI355X_MUL_MAT_NOALLOC_MAX bytes in device
 * memory that the library owns, one copy per GPU, held until the process ends.  No counterpart in the reference; it is
 * for callers that cannot allocate device memory: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  Same arguments, kernels and results as mi355x_mul_mat.  MI355X_ERR_WORKSPACE when the operands need
 * more scratch than the array holds (mi355x_mul_mat_workspace_size > MI355X_MUL_MAT_NOALLOC_MAX);
 * MI355X_ERR_INVALID with MI355X_MM_WS_READY or MI355X_MM_PREPARE_ONLY (the array is shared by every call on a GPU and keeps
 * the last call's contents, so no call may rely on them).  Calls that overlap on one GPU (two streams, two threads) race
 * on the array: serialize them.  The first call on a device looks up the array's address, the first call with
 * MI355X_EPI_GELU fills the GELU table with a synchronous copy, and the first launch of each kernel instance on a device
 * sets its LDS size attribute (the instance follows from the operand types, the size class of M, N and K, and the epilogue
 * flags): before a capture starts, make one call with the same types, shapes and flags as every call that will be
 * captured. */
#define MI355X_MUL_MAT_NOALLOC_MAX ((size_t) 32 << 20)
MI355X_API int    mi355x_mul_mat_noalloc(const mi355x_tensor * src0, const mi355x_tensor * src1, const mi355x_tensor * dst,
                                         const mi355x_epilogue * epi, void * stream);

/* Several MUL_MATs over the same src1 in one launch (a layer's Q, K and V projections; the cross-attention K and V of all
 * decoder layers): the same arithmetic as `count` calls of mi355x_mul_mat, item by item, but one grid that fills the
 * device where a single 1280-row product covers half of it.  No counterpart in the reference, whose graphs issue these
 * products one node at a time.  Only the shape this exists for: every src0 a dense 2-d F16 matrix of the same size (e.g.
 * the f16 images of quantized weights, with MI355X_MM_ACT_Q8_0 in `flags`), K a multiple of 256, more than 8 columns,
 * count <= 64 — or, for at most 8 columns, every src0 a Q5_0 / Q8_0 matrix of one type and size that takes the
 * workspace form of the few-column product (mi355x_mul_mat_workspace_size > 0), count <= 8: a decode step's Q, K and V;
 * anything else returns MI355X_ERR_UNSUPPORTED and the caller issues single calls.
 * `flags`: MI355X_MM_* options common to all items; the items' epilogues carry MI355X_EPI_* only. */
typedef struct mi355x_mul_mat_item {
    const mi355x_tensor *   src0;
    const mi355x_tensor *   dst;
    const mi355x_epilogue * epi;     /* may be NULL */
} mi355x_mul_mat_item;
MI355X_API int    mi355x_mul_mat_group(const mi355x_mul_mat_item * items, int count, const mi355x_tensor * src1, int flags,
                                       void * workspace, size_t workspace_size, void * stream);
/* LayerNorm (mi355x_norm: eps, optional affine w / b) of the rows of `src`, written to `normed`, and in the same launch the
 * few-column products of mi355x_mul_mat_group over `normed` (count 1 .. 8; one product is the common case).  For a decode
 * step, where a LayerNorm of five rows costs a launch of its own and nothing else: every workgroup normalizes the rows
 * for itself while its first weight blocks travel.  Also leaves the Q8_0 form of `normed` in `workspace`, as the products'
 * quantization pass would.  src / normed: F32 [K, N] with N <= 8, K a multiple of 32 and at most 2048, 16-byte aligned
 * rows; items as for the few-column form of mi355x_mul_mat_group; MI355X_ERR_UNSUPPORTED otherwise (then call
 * mi355x_norm_emit_q8_0 and the products).  No counterpart in the reference, whose graphs hold these as separate nodes. */
MI355X_API int    mi355x_norm_mul_mat_group(const mi355x_tensor * src, const mi355x_tensor * normed, float eps, const float * w, const float * b,
                                            const mi355x_mul_mat_item * items, int count, void * workspace, size_t workspace_size, void * stream);
/* mi355x_norm_mul_mat_group over rows that no launch has written yet: row n of `x0` is the token embedding tok[:, tok_ids[n]]
 * plus the positional embedding pos[:, pos_ids[n]] — what mi355x_get_rows_add would leave there (GET_ROWS, GET_ROWS and ADD of
 * src/whisper.cpp:2526-2529) — made by every workgroup for itself from the two tables, and written to `x0` by the first for
 * the residual connections that read it later; an index outside its table gives a NaN row, as there.  The same values bit for
 * bit as mi355x_get_rows_add followed by mi355x_norm_mul_mat_group.  tok: Q8_0, Q5_0 or F16 [K, n_vocab]; pos: F32 [K, n_ctx],
 * 16-byte aligned rows; tok_ids, pos_ids: dense I32 vectors of x0's row count; everything else as for
 * mi355x_norm_mul_mat_group, and only where the products take one weight block per lane (K <= 2048 with 64 lanes per row:
 * a layer's Q, K and V); MI355X_ERR_UNSUPPORTED otherwise (then call mi355x_get_rows_add and mi355x_norm_mul_mat_group).
 * No counterpart in the reference, whose graphs hold these as separate nodes. */
MI355X_API int    mi355x_embed_norm_mul_mat_group(const mi355x_tensor * tok, const mi355x_tensor * tok_ids, const mi355x_tensor * pos, const mi355x_tensor * pos_ids,
                                                  const mi355x_tensor * x0, const mi355x_tensor * normed, float eps, const float * w, const float * b,
                                                  const mi355x_mul_mat_item * items, int count, void * workspace, size_t workspace_size, void * stream);

/* The few-column product (ggml_compute_forward_mul_mat with ggml_vec_dot_q8_0_q8_0, ggml-cpu.c:1266-1458,
 * ggml-cpu-quants.c:3597) over a Q8_0 matrix long enough to be a stream — the vocabulary projection — with the integer
 * dot products on the matrix cores, from a copy of the matrix in the order those want: per 16 rows and pair of blocks,
 * 1024 bytes of quants (lane l of v_mfma_i32_16x16x64_i8's B operand: row l % 16, block (l / 16) / 2 of the pair, half
 * (l / 16) % 2) followed by the 32 f16 scales ([block of the pair][row]); rows padded to a multiple of 16 with zero
 * blocks.  The same bytes as the block rows (68 per row and pair), the same integer sums and scales as the reference;
 * a row's blocks are added up as two f32 sequences (even blocks, odd blocks) that are joined at the end.  No
 * counterpart in the reference, which keeps one layout per type.
 *   mi355x_q8_0_tiles_size    bytes of the copy for a [K, M] matrix (0: K is not a multiple of 64)
 *   mi355x_q8_0_tiles_pack    src0: Q8_0 [K, M], 2-d, rows at 2-byte alignment -> `tiles` (16-byte aligned)
 *   mi355x_mul_mat_q8_0_tiles dst[m, n] over `tiles`; src1: F32 [K, N <= 8], dst: F32 [M, N] (F16 with
 *                             MI355X_EPI_OUT_F16); K one of 384, 512, 768, 1024, 1280 (else MI355X_ERR_UNSUPPORTED).
 *                             `workspace` (16-byte aligned, N * K * 1.25 bytes rounded up to 256) receives the Q8_0 form of
 *                             src1 unless MI355X_MM_WS_READY says it is there; MI355X_MM_PREPARE_ONLY stops after that. */
MI355X_API size_t mi355x_q8_0_tiles_size(int64_t K, int64_t M);
MI355X_API int    mi355x_q8_0_tiles_pack(const mi355x_tensor * src0, void * tiles, void * stream);
MI355X_API int    mi355x_mul_mat_q8_0_tiles(const void * tiles, int64_t K, int64_t M, const mi355x_tensor * src1, const mi355x_tensor * dst,
                                            int flags, void * workspace, size_t workspace_size, void * stream);
/* mi355x_mul_mat_q8_0_tiles over LayerNorm(src) (mi355x_norm: eps, optional affine w / b) in one launch — the decoder's last
 * LayerNorm and the logits of a decode step: every workgroup normalizes the step's rows while its first tile row is on the
 * way; the first also writes the rows to `normed` and their Q8_0 form to `workspace`, as mi355x_norm_emit_q8_0 would.  The
 * same values bit for bit as that call followed by mi355x_mul_mat_q8_0_tiles with MI355X_MM_WS_READY.  src / normed: F32
 * [K, N <= 8], 16-byte aligned rows; `flags`: MI355X_EPI_OUT_F16 or 0; K as for mi355x_mul_mat_q8_0_tiles.  No counterpart in
 * the reference, whose graphs hold these as separate nodes. */
MI355X_API int    mi355x_norm_mul_mat_q8_0_tiles(const void * tiles, int64_t K, int64_t M, const mi355x_tensor * src, const mi355x_tensor * normed,
                                                 float eps, const float * w, const float * b, const mi355x_tensor * dst, int flags,
                                                 void * workspace, size_t workspace_size, void * stream);

/* FLASH_ATTN_EXT --------------------------------------------------------------------------------------
 * ggml_compute_forward_flash_attn_ext_f16 (ggml/src/ggml-cpu/ops.cpp:6638-6851), max_bias = 0 and
 * logit_softcap = 0 (the only values whisper uses):
 *   dst[:, h, n] = softmax_over_keys(scale * q[:, n, h] . k[:, key, h] + mask[key, n]) @ v[:, key, h]
 * q: F32 [D, N, H], k/v: F16 [D, KV, H] (D = 64), mask: F16 [KV, >=N] or NULL (-inf entries skip the
 * key), dst: F32 [D, H, N] contiguous.  With at most 8 queries the mask may also be the F32 tensor that the graph
 * casts to F16 (ggml_cast in src/whisper.cpp:2523): each value is rounded to f16 as it is read, which is what the
 * cast does, so a caller can leave the cast out; MI355X_ERR_UNSUPPORTED with more queries.
 * mode: MI355X_FA_F16_SEQ accumulates V in f16, key by key in order, as the reference does (ops.cpp:6793-6807) —
 * with near-uniform attention over ~1500 keys that rounding sequence dominates the low bits of the result;
 * MI355X_FA_F32 accumulates in f32 (closer to exact arithmetic, further from the reference); with more than 8 queries
 * both products run on the matrix cores with the softmax probabilities as f16 operands.
 * MI355X_FA_F16_PK keeps the f16 accumulator and the key order and does the step in f16 arithmetic — the factor rounded
 * to f16, one fused f16 multiply-add per element, a rescale as one f16 multiply — which is the arithmetic of the
 * reference's builds with f16 vector units (GGML_F16_VEC_FMA = vfmaq_f16, ggml/src/ggml-cpu/simd-mappings.h:68-105, under
 * ggml_vec_mad_f16 / ggml_vec_scale_f16, vec.h:180-203, 295-311), a third of the vector instructions of the x86 form
 * and, for the at most 8 queries of a decode step, one dependent instruction per key instead of two (that kernel
 * addresses the rows of a head's K and V with 32-bit offsets; a head slice of 2 GiB or more takes the x86 form). */
enum mi355x_fa_mode { MI355X_FA_F16_SEQ = 0, MI355X_FA_F32 = 1, MI355X_FA_F16_PK = 2,
    /* or-ed into the mode: also write into `workspace` (16-byte aligned, N * H * ne3 * 64 halves) the image of dst that
     * a following MUL_MAT with quantized weights wants — rows [N][H * 64] rounded to Q8_0 as quantize_row_q8_0 does and
     * stored as f16(q * d) (then pass MI355X_MM_WS_READY there).  More than 8 queries; MI355X_ERR_UNSUPPORTED otherwise.
     * With MI355X_FA_F16_SEQ, dst->data may then be NULL: only the image is written (a caller whose only reader of dst is
     * that product); MI355X_ERR_INVALID for a NULL dst->data in any other case. */
    MI355X_FA_EMIT_F16 = 0x100,
    /* or-ed into the mode, at most 8 queries (the f16-sequential kernels of a decode step, either form): also write into `workspace`
     * (16-byte aligned) the rows [N * ne3][H * 64] of dst quantized to Q8_0, in the layout the few-column mi355x_mul_mat
     * reads its activations from (see mi355x_norm_emit_q8_0); MI355X_ERR_UNSUPPORTED for other kernels. */
    MI355X_FA_EMIT_Q8_0 = 0x200 };
MI355X_API const char * mi355x_flash_attn_ext_kernel_name(const mi355x_tensor * q, const mi355x_tensor * k, int mode);
MI355X_API size_t mi355x_flash_attn_ext_workspace_size(const mi355x_tensor * q, const mi355x_tensor * k);
MI355X_API int    mi355x_flash_attn_ext(const mi355x_tensor * q, const mi355x_tensor * k, const mi355x_tensor * v,
                                        const mi355x_tensor * mask, const mi355x_tensor * dst, float scale, int mode,
                                        void * workspace, size_t workspace_size, void * stream);

/* The same with an F32 mask (at most 8 queries, see above) whose f16 form — the result of the ggml_cast that precedes the
 * first attention node of a decode step, src/whisper.cpp:2523 — is also written to `mask_f16` (F16 [KV, >=N]; rows < N),
 * for the attention nodes of the later layers: the cast needs no launch of its own. */
MI355X_API int    mi355x_flash_attn_ext_cast_mask(const mi355x_tensor * q, const mi355x_tensor * k, const mi355x_tensor * v,
                                                  const mi355x_tensor * mask_f32, const mi355x_tensor * mask_f16, const mi355x_tensor * dst,
                                                  float scale, int mode, void * workspace, size_t workspace_size, void * stream);

/* elementwise / row ops ------------------------------------------------------------------------------ */

/* ADD / MUL with src1 repeated over any dimension, including ne0 (ggml/src/ggml-cpu/binary-ops.cpp:49-142).
 * All F32; dst may alias src0 or src1.  op: 0 = add, 1 = mul. */
MI355X_API int mi355x_binary(int op, const mi355x_tensor * src0, const mi355x_tensor * src1, const mi355x_tensor * dst, void * stream);

/* SCALE: dst = src * s (ggml/src/ggml-cpu/ops.cpp:3840-3878).  F32, may run in place. */
MI355X_API int mi355x_scale(const mi355x_tensor * src, const mi355x_tensor * dst, float s, void * stream);

/* UNARY GELU (ggml/src/ggml-cpu/ops.cpp:2606-2643, vec.h:432-457): 0.5x(1+tanh(sqrt(2/pi) x (1+0.044715x^2))),
 * read for |x| < 10 from a 65536-entry table indexed by f16(x), exactly like the CPU backend (table built at
 * ggml/src/ggml-cpu/ggml-cpu.c:3415-3423).  The library builds the same table on the host on first use (same
 * formula, same libm) and keeps a copy in a __device__ array. */
MI355X_API int mi355x_gelu(const mi355x_tensor * src, const mi355x_tensor * dst, void * stream);

/* NORM (ggml/src/ggml-cpu/ops.cpp:3109-3158): y = (x - mean) / sqrt(var + eps) over ne0.  With w and/or b
 * non-NULL also applies the following MUL by w[ne0] and ADD of b[ne0] (whisper's LayerNorm affine,
 * src/whisper.cpp:2116-2121).  All F32. */
MI355X_API int mi355x_norm(const mi355x_tensor * src, const mi355x_tensor * dst, float eps,
                           const float * w, const float * b, void * stream);
/* The same, and in the same pass the result's image for the MFMA GEMM: rounded to Q8_0 as quantize_row_q8_0 does
 * (ggml-cpu-quants.c:808-865) and stored as f16(q * d), dense [rows][ne0], at `x16` — what mi355x_mul_mat's src1
 * conversion pass would write into its workspace (then pass MI355X_MM_WS_READY).  ne0 multiple of 32 and at most 2048,
 * 16-byte aligned rows; MI355X_ERR_UNSUPPORTED otherwise.  With dst->data == NULL (shape and strides still describe the
 * result) only the image is written: for a result whose only readers are products that take the image. */
MI355X_API int mi355x_norm_emit_f16(const mi355x_tensor * src, const mi355x_tensor * dst, float eps, const float * w, const float * b,
                                    void * x16, void * stream);
/* The same for the few-column product (N <= 8) over quantized weights: the result quantized to Q8_0 itself, in the layout
 * mi355x_mul_mat's quantization pass writes into its workspace for that path —
 *   int8 q[rows][ne0] | float d[rows][ne0/32] (the f16-rounded scales) | int32 s[rows][ne0/32] (sum of a block's quants)
 * — at `q8` (16-byte aligned, mi355x_mul_mat_workspace_size bytes of the product that follows).  2-d src; otherwise the
 * conditions of mi355x_norm_emit_f16. */
MI355X_API int mi355x_norm_emit_q8_0(const mi355x_tensor * src, const mi355x_tensor * dst, float eps, const float * w, const float * b,
                                     void * q8, void * stream);

/* SOFT_MAX (ggml/src/ggml-cpu/ops.cpp:4641-4737), max_bias = 0: softmax(scale * x + mask) over ne0.
 * mask F32 or F16 [ne0, >= ne1], broadcast over ne2/ne3, or NULL. */
MI355X_API int mi355x_soft_max(const mi355x_tensor * src, const mi355x_tensor * mask, const mi355x_tensor * dst,
                               float scale, void * stream);

/* CPY / CONT / DUP (ggml/src/ggml-cpu/ops.cpp:670-1183): strided element copy with conversion between
 * F32 and F16 (round-to-nearest-even).  src and dst hold the same number of elements; either may be
 * a strided / permuted view. */
MI355X_API int mi355x_cpy(const mi355x_tensor * src, const mi355x_tensor * dst, void * stream);

/* GET_ROWS (ggml/src/ggml-cpu/ops.cpp:4146-4188, 4313): dst[:, i] = dequant(src0[:, ids[i]]).
 * src0: Q5_0 | Q8_0 | F16 | F32, ids: I32, dst: F32.  An index outside [0, src0 ne1) — on which the reference aborts the
 * process (GGML_ASSERT, ops.cpp:4174) — reads nothing and yields a row of NaN. */
MI355X_API int mi355x_get_rows(const mi355x_tensor * src0, const mi355x_tensor * ids, const mi355x_tensor * dst, void * stream);
/* dst[:, i] = dequant(src0 row ids0[i]) + src1 row ids1[i]: the token embedding plus the positional embedding of a
 * decoder input (GET_ROWS, GET_ROWS and ADD of src/whisper.cpp:2526-2529, ops.cpp:4313 and binary-ops.cpp:49-142) in one
 * launch; the same f32 values and the same f32 sum.  src1 F32; ids0, ids1 I32 vectors of one length; dst F32 [ne0, n]. */
MI355X_API int mi355x_get_rows_add(const mi355x_tensor * src0, const mi355x_tensor * ids0, const mi355x_tensor * src1, const mi355x_tensor * ids1,
                                   const mi355x_tensor * dst, void * stream);

/* IM2COL, 1-D, F16 output (ggml/src/ggml-cpu/ops.cpp:5784-5855; ggml/src/ggml.c:3818-3858):
 * dst[ic*KW + kw, ow, n] = f16(src[ow*s0 + kw*d0 - p0, ic, n]) or 0 outside.  src F32 [IW, IC, N]. */
MI355X_API int mi355x_im2col_1d(const mi355x_tensor * src, const mi355x_tensor * dst, int kw, int s0, int p0, int d0, void * stream);

/* CONCAT along `dim` (ggml/src/ggml-cpu/ops.cpp:2575).  F32. */
MI355X_API int mi355x_concat(const mi355x_tensor * src0, const mi355x_tensor * src1, const mi355x_tensor * dst, int dim, void * stream);

/* Log-mel front end -----------------------------------------------------------------------------------
 * log_mel_spectrogram (src/whisper.cpp:3181-3270; worker :3113-3179; tables and transform :3008-3111), the step
 * whisper_pcm_to_mel (:3881) runs on host threads before the encoder: 16 kHz f32 samples -> mel f32 [n_mel][n_len],
 * n_len = (n_samples + 480000) / 160, ready for whisper_set_mel.  The signal is extended by 200 reflected samples in
 * front and 30 s + 200 samples of zeros behind; 400-sample frames every 160 samples under the periodic Hann window;
 * power of bins 0 .. 200 of each frame's transform; filter bank `filters` [n_mel][201] (the model file's);
 * log10(max(., 1e-10)); values below (global maximum - 8) raised to it; (x + 4) / 4.  The transform is evaluated as
 * direct sums in f64 where the reference runs an f32 halving scheme: results agree with it to its own rounding
 * (about 1e-5 absolute on the output's range of roughly [-1, 1.5]), not bitwise.
 * All pointers are device memory; n_samples > 200; n_mel <= 128; workspace 16-byte aligned. */
MI355X_API int64_t mi355x_log_mel_n_len(int64_t n_samples);
MI355X_API size_t  mi355x_log_mel_workspace_size(int n_mel);          /* 0: n_mel out of range */
MI355X_API int     mi355x_log_mel_spectrogram(const float * samples, int64_t n_samples, const float * filters, int n_mel, float * mel,
                                              void * workspace, size_t workspace_size, void * stream);


/* Fill `n` bytes at `dst` with `value` through a kernel (safe inside HIP graph capture). */
MI355X_API int mi355x_fill_bytes(void * dst, uint8_t value, size_t n, void * stream);

#ifdef __cplusplus
}
#endif
#endif /* MI355X_KERNELS_H */
