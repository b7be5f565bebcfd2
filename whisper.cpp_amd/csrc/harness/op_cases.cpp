#include "op_cases.h"

#include <math.h>

namespace ops {

namespace {

const double TOL = 5e-4;   // per-op NMSE bound

double wbytes(ggml_type t, double n) { return n / ggml_blck_size(t) * ggml_type_size(t); }

// ---- MUL_MAT ---------------------------------------------------------------------------------------------

op_case mm(const std::string & name, ggml_type wt, int64_t K, int64_t M, int64_t N, bool heavy = false, ggml_type xt = GGML_TYPE_F32) {
    op_case c;
    c.name = name; c.op = "MUL_MAT"; c.nmse_tol = TOL; c.bit_exact = false; c.heavy = heavy;
    c.flops = 2.0 * M * N * K;
    c.bytes = wbytes(wt, (double) M * K) + wbytes(xt, (double) K * N) + 4.0 * M * N;
    c.build = [=](ggml_context * ctx) {
        built b;
        ggml_tensor * w = ggml_new_tensor_2d(ctx, wt, K, M); ggml_set_name(w, "w");
        ggml_tensor * x = ggml_new_tensor_2d(ctx, xt, K, N); ggml_set_name(x, "x");
        b.inputs.push_back({ w, FILL_NORMAL, 0.02f });
        b.inputs.push_back({ x, FILL_NORMAL, 1.0f });
        b.result = ggml_mul_mat(ctx, w, x);
        b.roots = { b.result };
        return b;
    };
    return c;
}

// MUL_MAT followed by the neighbours whisper attaches to it; the MI355X backend folds them into the GEMM
// epilogue, the CPU backend runs them one by one.
enum chain_kind { CH_BIAS_GELU, CH_BIAS_RESID, CH_BIAS_SCALE, CH_SCALE_CPY16, CH_BIAS_CPY16 };

op_case mm_chain(const std::string & name, chain_kind kind, ggml_type wt, int64_t K, int64_t M, int64_t N) {
    op_case c;
    c.name = name; c.op = "MUL_MAT+"; c.nmse_tol = TOL; c.bit_exact = false; c.heavy = false;
    c.flops = 2.0 * M * N * K;
    c.bytes = wbytes(wt, (double) M * K) + 4.0 * K * N + 4.0 * M * N;
    c.build = [=](ggml_context * ctx) {
        built b;
        ggml_tensor * w    = ggml_new_tensor_2d(ctx, wt, K, M);            ggml_set_name(w, "w");
        ggml_tensor * x    = ggml_new_tensor_2d(ctx, GGML_TYPE_F32, K, N); ggml_set_name(x, "x");
        ggml_tensor * bias = ggml_new_tensor_1d(ctx, GGML_TYPE_F32, M);    ggml_set_name(bias, "bias");
        b.inputs.push_back({ w, FILL_NORMAL, 0.02f });
        b.inputs.push_back({ x, FILL_NORMAL, 1.0f });
        b.inputs.push_back({ bias, FILL_NORMAL, 0.5f });
        ggml_tensor * cur = ggml_mul_mat(ctx, w, x);
        switch (kind) {
            case CH_BIAS_GELU:  cur = ggml_gelu(ctx, ggml_add(ctx, cur, bias)); break;
            case CH_BIAS_SCALE: cur = ggml_scale(ctx, ggml_add(ctx, cur, bias), 0.35355339f); break;
            case CH_BIAS_RESID: {
                ggml_tensor * r = ggml_new_tensor_2d(ctx, GGML_TYPE_F32, M, N); ggml_set_name(r, "resid");
                b.inputs.push_back({ r, FILL_NORMAL, 1.0f });
                cur = ggml_add(ctx, ggml_add(ctx, cur, bias), r);
            } break;
            case CH_SCALE_CPY16: case CH_BIAS_CPY16: {
                // the K / V store of whisper_build_graph_cross (src/whisper.cpp:2316-2351): f16 cache slab at a layer offset
                ggml_tensor * cache = ggml_new_tensor_1d(ctx, GGML_TYPE_F16, 3 * M * N); ggml_set_name(cache, "cache");
                b.inputs.push_back({ cache, FILL_NORMAL, 1.0f });
                cur = kind == CH_SCALE_CPY16 ? ggml_scale(ctx, cur, 0.35355339f) : ggml_add(ctx, cur, bias);
                ggml_tensor * dst = ggml_view_1d(ctx, cache, M * N, (size_t)(M * N) * 2);
                b.roots = { ggml_cpy(ctx, cur, dst) };
                b.result = cache;
                return b;
            }
        }
        b.result = cur;
        b.roots = { cur };
        return b;
    };
    return c;
}

// ggml_conv_1d_ph + bias + GELU, the conv stem (src/whisper.cpp:2019-2027): IM2COL, F16 x F16 MUL_MAT, RESHAPE, ADD [1,d], GELU
op_case conv_stem(const std::string & name, int64_t IW, int64_t IC, int64_t OC, int stride, bool heavy) {
    op_case c;
    c.name = name; c.op = "IM2COL+MUL_MAT+ADD+GELU"; c.nmse_tol = TOL; c.bit_exact = false; c.heavy = heavy;
    const int64_t OW = (IW + 2 - 3) / stride + 1;
    c.flops = 2.0 * OW * OC * IC * 3;
    c.bytes = 4.0 * IW * IC + 2.0 * 3 * IC * OC + 4.0 * OW * OC;
    c.build = [=](ggml_context * ctx) {
        built b;
        ggml_tensor * w    = ggml_new_tensor_3d(ctx, GGML_TYPE_F16, 3, IC, OC); ggml_set_name(w, "conv_w");
        ggml_tensor * x    = ggml_new_tensor_2d(ctx, GGML_TYPE_F32, IW, IC);    ggml_set_name(x, "x");
        ggml_tensor * bias = ggml_new_tensor_2d(ctx, GGML_TYPE_F32, 1, OC);     ggml_set_name(bias, "bias");
        b.inputs.push_back({ w, FILL_NORMAL, 0.02f });
        b.inputs.push_back({ x, FILL_NORMAL, 0.5f, 0.5f });
        b.inputs.push_back({ bias, FILL_NORMAL, 0.1f });
        ggml_tensor * cur = ggml_conv_1d_ph(ctx, w, x, stride, 1);
        cur = ggml_gelu(ctx, ggml_add(ctx, cur, bias));
        b.result = cur; b.roots = { cur };
        return b;
    };
    return c;
}

// non-flash attention products (src/whisper.cpp:2631-2646): strided f16 K view x permuted f32 Q, batched over heads
op_case mm_kq(const std::string & name, int64_t n_kv, int64_t n_tok, int64_t H, int64_t n_ctx) {
    op_case c;
    c.name = name; c.op = "MUL_MAT"; c.nmse_tol = TOL; c.bit_exact = false; c.heavy = false;
    c.flops = 2.0 * n_kv * n_tok * 64 * H; c.bytes = 2.0 * n_kv * 64 * H + 4.0 * n_tok * 64 * H + 4.0 * n_kv * n_tok * H;
    c.build = [=](ggml_context * ctx) {
        built b;
        const int64_t d = 64 * H;
        ggml_tensor * cache = ggml_new_tensor_1d(ctx, GGML_TYPE_F16, d * n_ctx); ggml_set_name(cache, "k_cache");
        ggml_tensor * qcur  = ggml_new_tensor_2d(ctx, GGML_TYPE_F32, d, n_tok);  ggml_set_name(qcur, "q");
        b.inputs.push_back({ cache, FILL_NORMAL, 1.0f });
        b.inputs.push_back({ qcur, FILL_NORMAL, 1.0f });
        ggml_tensor * Q = ggml_permute(ctx, ggml_reshape_3d(ctx, qcur, 64, H, n_tok), 0, 2, 1, 3);
        ggml_tensor * K = ggml_view_3d(ctx, cache, 64, n_kv, H, 2 * d, 2 * 64, 0);
        b.result = ggml_mul_mat(ctx, K, Q);
        b.roots = { b.result };
        return b;
    };
    return c;
}

op_case mm_kqv(const std::string & name, int64_t n_kv, int64_t n_tok, int64_t H, int64_t n_ctx) {
    op_case c;
    c.name = name; c.op = "MUL_MAT"; c.nmse_tol = TOL; c.bit_exact = false; c.heavy = false;
    c.flops = 2.0 * n_kv * n_tok * 64 * H; c.bytes = 2.0 * n_kv * 64 * H + 4.0 * n_tok * n_kv * H + 4.0 * 64 * n_tok * H;
    c.build = [=](ggml_context * ctx) {
        built b;
        const int64_t d = 64 * H;
        ggml_tensor * cache = ggml_new_tensor_1d(ctx, GGML_TYPE_F16, d * n_ctx);          ggml_set_name(cache, "vT_cache");
        ggml_tensor * p     = ggml_new_tensor_3d(ctx, GGML_TYPE_F32, n_kv, n_tok, H);    ggml_set_name(p, "softmax");
        b.inputs.push_back({ cache, FILL_NORMAL, 1.0f });
        b.inputs.push_back({ p, FILL_NORMAL, 0.1f, 0.1f });
        ggml_tensor * V = ggml_view_3d(ctx, cache, n_kv, 64, H, n_ctx * 2, n_ctx * 2 * 64, 0);
        b.result = ggml_mul_mat(ctx, V, p);
        b.roots = { b.result };
        return b;
    };
    return c;
}

// ---- FLASH_ATTN_EXT ----------------------------------------------------------------------------------------

// Q is the permuted view of a [d, N] projection, K / V are strided views of 1-d f16 caches with kv_alloc rows of
// which the first kv_valid hold data (src/whisper.cpp:2149-2172, 2606-2626, 2686-2706).  mask_mode: 0 none,
// 1 = beam-style (all rows see the first half of the keys, of the rest row r sees key k iff k % N == r), 2 = causal.
op_case fa(const std::string & name, int64_t N, int64_t KV, int64_t kv_valid, int64_t H, int mask_mode, float scale, bool heavy = false) {
    op_case c;
    c.name = name; c.op = "FLASH_ATTN_EXT"; c.nmse_tol = TOL; c.bit_exact = false; c.heavy = heavy;
    c.flops = 4.0 * N * KV * 64 * H;
    c.bytes = 4.0 * N * 64 * H + 2.0 * 2 * KV * 64 * H + 4.0 * N * 64 * H;
    c.build = [=](ggml_context * ctx) {
        built b;
        const int64_t d = 64 * H;
        ggml_tensor * qcur = ggml_new_tensor_2d(ctx, GGML_TYPE_F32, d, N);    ggml_set_name(qcur, "q");
        ggml_tensor * kc   = ggml_new_tensor_1d(ctx, GGML_TYPE_F16, d * KV);  ggml_set_name(kc, "k_cache");
        ggml_tensor * vc   = ggml_new_tensor_1d(ctx, GGML_TYPE_F16, d * KV);  ggml_set_name(vc, "v_cache");
        b.inputs.push_back({ qcur, FILL_NORMAL, 1.0f });
        input ik{ kc, FILL_ZERO_TAIL, 1.0f }; ik.range = kv_valid; ik.rows = d;   // rows of d values, zero after kv_valid rows
        input iv{ vc, FILL_ZERO_TAIL, 1.0f }; iv.range = kv_valid; iv.rows = d;
        b.inputs.push_back(ik);
        b.inputs.push_back(iv);
        ggml_tensor * Q = ggml_permute(ctx, ggml_reshape_3d(ctx, qcur, 64, H, N), 0, 2, 1, 3);
        ggml_tensor * K = ggml_view_3d(ctx, kc, 64, KV, H, 2 * d, 2 * 64, 0);
        ggml_tensor * V = ggml_view_3d(ctx, vc, 64, KV, H, 2 * d, 2 * 64, 0);
        ggml_tensor * mask = nullptr;
        if (mask_mode) {
            mask = ggml_new_tensor_2d(ctx, GGML_TYPE_F16, KV, GGML_PAD(N, GGML_KQ_MASK_PAD)); ggml_set_name(mask, "mask");
            input im{ mask, FILL_MASK }; im.range = mask_mode; im.rows = N;
            b.inputs.push_back(im);
        }
        b.result = ggml_flash_attn_ext(ctx, Q, K, V, mask, scale, 0.0f, 0.0f);
        b.roots = { b.result };
        return b;
    };
    return c;
}

// ---- everything else --------------------------------------------------------------------------------------------

op_case simple(const std::string & name, const std::string & op, bool bit_exact, double bytes, bool heavy,
               std::function<built(ggml_context *)> build) {
    op_case c;
    c.name = name; c.op = op; c.nmse_tol = TOL; c.bit_exact = bit_exact; c.flops = 0; c.bytes = bytes; c.heavy = heavy;
    c.build = std::move(build);
    return c;
}

ggml_tensor * in2(ggml_context * ctx, built & b, const char * name, ggml_type t, int64_t ne0, int64_t ne1, float scale = 1.0f, float offset = 0.0f) {
    ggml_tensor * x = ggml_new_tensor_2d(ctx, t, ne0, ne1); ggml_set_name(x, name);
    b.inputs.push_back({ x, FILL_NORMAL, scale, offset });
    return x;
}

} // namespace

std::vector<op_case> all_cases() {
    std::vector<op_case> v;

    // the Whisper-base FFN-up product over a 30 s window (the smallest benchmarked case) and the encoder GEMMs of Whisper-base and large-v3
    v.push_back(mm("mul_mat.q8_0.cfg0_512x2048_n1500",  GGML_TYPE_Q8_0, 512, 2048, 1500));
    v.push_back(mm("mul_mat.q5_0.base_512x512_n1500",   GGML_TYPE_Q5_0, 512, 512, 1500));
    v.push_back(mm("mul_mat.q5_0.base_2048x512_n1500",  GGML_TYPE_Q5_0, 2048, 512, 1500));
    v.push_back(mm("mul_mat.q5_0.l3_1280x1280_n1500",   GGML_TYPE_Q5_0, 1280, 1280, 1500));
    v.push_back(mm("mul_mat.q5_0.l3_1280x5120_n1500",   GGML_TYPE_Q5_0, 1280, 5120, 1500, true));
    v.push_back(mm("mul_mat.q5_0.l3_5120x1280_n1500",   GGML_TYPE_Q5_0, 5120, 1280, 1500, true));
    v.push_back(mm("mul_mat.q8_0.l3_1280x1280_n1500",   GGML_TYPE_Q8_0, 1280, 1280, 1500));
    v.push_back(mm("mul_mat.f16.l3_1280x1280_n1500",    GGML_TYPE_F16,  1280, 1280, 1500));
    v.push_back(mm("mul_mat.f32.512x512_n100",          GGML_TYPE_F32,  512, 512, 100));
    // ragged tiles: N and M just around the 128-wide tile, N just above the GEMV limit, prompt-sized N
    v.push_back(mm("mul_mat.q8_0.ragged_n9",            GGML_TYPE_Q8_0, 1280, 1280, 9));
    v.push_back(mm("mul_mat.q5_0.ragged_n127_m1000",    GGML_TYPE_Q5_0, 512, 1000, 127));
    v.push_back(mm("mul_mat.q5_0.ragged_n129_m130",     GGML_TYPE_Q5_0, 512, 130, 129));
    v.push_back(mm("mul_mat.q8_0.prompt_n448",          GGML_TYPE_Q8_0, 1280, 1280, 448));
    v.push_back(mm("mul_mat.q5_0.k32_single_block",     GGML_TYPE_Q5_0, 32, 64, 200));
    // decoder GEMV (1..8 columns), incl. the 1280x51866 logits projection of a large-v3-turbo decode step
    v.push_back(mm("mul_mat.q8_0.logits_51866_n5",      GGML_TYPE_Q8_0, 1280, 51866, 5));
    v.push_back(mm("mul_mat.q8_0.logits_51866_n1",      GGML_TYPE_Q8_0, 1280, 51866, 1));
    v.push_back(mm("mul_mat.q5_0.logits_51866_n5",      GGML_TYPE_Q5_0, 1280, 51866, 5));
    v.push_back(mm("mul_mat.q8_0.gemv_1280x1280_n5",    GGML_TYPE_Q8_0, 1280, 1280, 5));
    v.push_back(mm("mul_mat.q8_0.gemv_1280x5120_n5",    GGML_TYPE_Q8_0, 1280, 5120, 5));
    v.push_back(mm("mul_mat.q8_0.gemv_5120x1280_n5",    GGML_TYPE_Q8_0, 5120, 1280, 5));
    v.push_back(mm("mul_mat.q5_0.gemv_1280x1280_n1",    GGML_TYPE_Q5_0, 1280, 1280, 1));
    v.push_back(mm("mul_mat.q5_0.gemv_5120x1280_n8",    GGML_TYPE_Q5_0, 5120, 1280, 8));
    v.push_back(mm("mul_mat.q5_0.gemv_m1001_n3",        GGML_TYPE_Q5_0, 512, 1001, 3));
    v.push_back(mm("mul_mat.f16.gemv_1280x1280_n1",     GGML_TYPE_F16,  1280, 1280, 1));
    v.push_back(mm("mul_mat.f16.gemv_1280x1280_n5",     GGML_TYPE_F16,  1280, 1280, 5));
    v.push_back(mm("mul_mat.f32.odd_k37",               GGML_TYPE_F32,  37, 50, 11));
    // conv-as-GEMM operands (f16 x f16): im2col patches times conv weights, K = 3*n_mels or 3*d
    v.push_back(mm("mul_mat.f16xf16.conv1_l3_k384",     GGML_TYPE_F16, 384, 3000, 1280, false, GGML_TYPE_F16));
    v.push_back(mm("mul_mat.f16xf16.conv1_base_k240",   GGML_TYPE_F16, 240, 3000, 512,  false, GGML_TYPE_F16));
    v.push_back(mm("mul_mat.f16xf16.conv2_base_k1536",  GGML_TYPE_F16, 1536, 1500, 512, false, GGML_TYPE_F16));
    // non-flash attention products
    v.push_back(mm_kq ("mul_mat.f16.kq_kv37_n5_h20",    37, 5, 20, 448));
    v.push_back(mm_kq ("mul_mat.f16.kq_kv1500_n1500_h8", 1500, 1500, 8, 1500));
    v.push_back(mm_kqv("mul_mat.f16.kqv_kv37_n5_h20",   37, 5, 20, 448));
    v.push_back(mm_kqv("mul_mat.f16.kqv_kv40_n5_h20",   40, 5, 20, 448));
    // fused neighbours
    v.push_back(mm_chain("mul_mat+bias+gelu.q5_0_512x2048_n1500",  CH_BIAS_GELU,   GGML_TYPE_Q5_0, 512, 2048, 1500));
    v.push_back(mm_chain("mul_mat+bias+resid.q5_0_2048x512_n1500", CH_BIAS_RESID,  GGML_TYPE_Q5_0, 2048, 512, 1500));
    v.push_back(mm_chain("mul_mat+bias+scale.q8_0_1280x1280_n5",   CH_BIAS_SCALE,  GGML_TYPE_Q8_0, 1280, 1280, 5));
    v.push_back(mm_chain("mul_mat+scale+cpy16.q5_0_512x512_n1500", CH_SCALE_CPY16, GGML_TYPE_Q5_0, 512, 512, 1500));
    v.push_back(mm_chain("mul_mat+bias+cpy16.q8_0_1280x1280_n5",   CH_BIAS_CPY16,  GGML_TYPE_Q8_0, 1280, 1280, 5));
    v.push_back(conv_stem("conv_stem.base_conv1_80x3000",  3000, 80, 512, 1, false));
    v.push_back(conv_stem("conv_stem.base_conv2_512x3000", 3000, 512, 512, 2, false));
    v.push_back(conv_stem("conv_stem.l3_conv1_128x3000",   3000, 128, 1280, 1, false));
    v.push_back(conv_stem("conv_stem.l3_conv2_1280x3000",  3000, 1280, 1280, 2, true));

    // the large-v3 encoder's self-attention (1500 x 1500, 20 heads) and whisper's three attention kinds
    v.push_back(fa("flash_attn.cfg2_enc_n1500_kv1500_h20", 1500, 1500, 1500, 20, 0, 0.125f, true));
    v.push_back(fa("flash_attn.enc_base_n1500_kv1536pad_h8", 1500, 1536, 1500, 8, 0, 0.125f, true));
    v.push_back(fa("flash_attn.cfg2_cross_n5_kv1500_h20",  5, 1500, 1500, 20, 0, 0.125f));
    v.push_back(fa("flash_attn.cross_n5_kv1536pad_h20",    5, 1536, 1500, 20, 0, 0.35355339f));
    v.push_back(fa("flash_attn.cross_n1_kv1536pad_h8",     1, 1536, 1500, 8, 0, 0.35355339f));
    v.push_back(fa("flash_attn.self_n5_kv37_mask_h20",     5, 37, 37, 20, 1, 1.0f));
    v.push_back(fa("flash_attn.self_n1_kv1_mask_h20",      1, 1, 1, 20, 1, 1.0f));
    v.push_back(fa("flash_attn.self_n5_kv448_mask_h20",    5, 448, 448, 20, 1, 1.0f));
    v.push_back(fa("flash_attn.self_n3_kv200_causal_h8",   3, 200, 200, 8, 2, 1.0f));
    v.push_back(fa("flash_attn.prompt_n256_kv256_causal_h20", 256, 256, 256, 20, 2, 1.0f));
    v.push_back(fa("flash_attn.enc_small_n70_kv100_h2",    70, 100, 100, 2, 0, 0.125f));

    // IM2COL (src/whisper.cpp:2019, 2024 via ggml_conv_1d_ph)
    auto im2col_case = [](const std::string & name, int64_t IW, int64_t IC, int stride, bool heavy) {
        const int64_t OW = (IW + 2 - 3) / stride + 1;
        return simple(name, "IM2COL", true, 4.0 * IW * IC + 2.0 * 3 * IC * OW, heavy, [=](ggml_context * ctx) {
            built b;
            ggml_tensor * w = ggml_new_tensor_3d(ctx, GGML_TYPE_F16, 3, IC, 8); ggml_set_name(w, "w");
            b.inputs.push_back({ w, FILL_NORMAL, 0.02f });
            ggml_tensor * x = in2(ctx, b, "x", GGML_TYPE_F32, IW, IC);
            b.result = ggml_im2col(ctx, w, x, stride, 0, 1, 0, 1, 0, false, GGML_TYPE_F16);
            b.roots = { b.result };
            return b;
        });
    };
    v.push_back(im2col_case("im2col.l3_conv1_128x3000_s1", 3000, 128, 1, false));
    v.push_back(im2col_case("im2col.l3_conv2_1280x3000_s2", 3000, 1280, 2, false));
    v.push_back(im2col_case("im2col.base_conv1_80x3000_s1", 3000, 80, 1, false));
    v.push_back(im2col_case("im2col.odd_33x77_s2", 77, 33, 2, false));

    // NORM, alone and with the LayerNorm affine behind it
    auto norm_case = [](const std::string & name, int64_t ne0, int64_t ne1, bool affine) {
        return simple(name, affine ? "NORM+MUL+ADD" : "NORM", false, 8.0 * ne0 * ne1, false, [=](ggml_context * ctx) {
            built b;
            ggml_tensor * x = in2(ctx, b, "x", GGML_TYPE_F32, ne0, ne1, 2.0f, 0.3f);
            ggml_tensor * cur = ggml_norm(ctx, x, 1e-5f);
            if (affine) {
                ggml_tensor * w = ggml_new_tensor_1d(ctx, GGML_TYPE_F32, ne0); ggml_set_name(w, "ln_w");
                ggml_tensor * bb = ggml_new_tensor_1d(ctx, GGML_TYPE_F32, ne0); ggml_set_name(bb, "ln_b");
                b.inputs.push_back({ w, FILL_NORMAL, 0.02f, 1.0f });
                b.inputs.push_back({ bb, FILL_NORMAL, 0.02f });
                cur = ggml_add(ctx, ggml_mul(ctx, cur, w), bb);
            }
            b.result = cur; b.roots = { cur };
            return b;
        });
    };
    v.push_back(norm_case("norm.l3_1280x1500", 1280, 1500, false));
    v.push_back(norm_case("norm.base_512x1500", 512, 1500, false));
    v.push_back(norm_case("norm.odd_100x7", 100, 7, false));
    v.push_back(norm_case("norm.long_5000x3", 5000, 3, false));
    v.push_back(norm_case("norm+affine.l3_1280x1500", 1280, 1500, true));
    v.push_back(norm_case("norm+affine.dec_1280x5", 1280, 5, true));

    // GELU, SCALE
    v.push_back(simple("gelu.l3_5120x1500", "UNARY(GELU)", false, 8.0 * 5120 * 1500, false, [](ggml_context * ctx) {
        built b; ggml_tensor * x = in2(ctx, b, "x", GGML_TYPE_F32, 5120, 1500, 3.0f);
        b.result = ggml_gelu(ctx, x); b.roots = { b.result }; return b; }));
    v.push_back(simple("gelu.wide_range_1000x13", "UNARY(GELU)", false, 8.0 * 13000, false, [](ggml_context * ctx) {
        built b; ggml_tensor * x = in2(ctx, b, "x", GGML_TYPE_F32, 1000, 13, 8.0f);
        b.result = ggml_gelu(ctx, x); b.roots = { b.result }; return b; }));
    v.push_back(simple("scale.1280x1500", "SCALE", true, 8.0 * 1280 * 1500, false, [](ggml_context * ctx) {
        built b; ggml_tensor * x = in2(ctx, b, "x", GGML_TYPE_F32, 1280, 1500);
        b.result = ggml_scale(ctx, x, 0.35355339f); b.roots = { b.result }; return b; }));

    // ADD / MUL broadcasts (src/whisper.cpp:2020, 2102, 2119-2121, 2215)
    v.push_back(simple("add.bias_row_1280x1500", "ADD", true, 8.0 * 1280 * 1500, false, [](ggml_context * ctx) {
        built b; ggml_tensor * x = in2(ctx, b, "x", GGML_TYPE_F32, 1280, 1500);
        ggml_tensor * bias = ggml_new_tensor_1d(ctx, GGML_TYPE_F32, 1280); ggml_set_name(bias, "bias"); b.inputs.push_back({ bias, FILL_NORMAL, 1.0f });
        b.result = ggml_add(ctx, x, bias); b.roots = { b.result }; return b; }));
    v.push_back(simple("add.residual_1280x1500", "ADD", true, 12.0 * 1280 * 1500, false, [](ggml_context * ctx) {
        built b; ggml_tensor * x = in2(ctx, b, "x", GGML_TYPE_F32, 1280, 1500); ggml_tensor * y = in2(ctx, b, "y", GGML_TYPE_F32, 1280, 1500);
        b.result = ggml_add(ctx, x, y); b.roots = { b.result }; return b; }));
    v.push_back(simple("add.conv_bias_bcast_ne0_3000x512", "ADD", true, 8.0 * 3000 * 512, false, [](ggml_context * ctx) {
        built b; ggml_tensor * x = ggml_new_tensor_3d(ctx, GGML_TYPE_F32, 3000, 512, 1); ggml_set_name(x, "x"); b.inputs.push_back({ x, FILL_NORMAL, 1.0f });
        ggml_tensor * bias = in2(ctx, b, "bias", GGML_TYPE_F32, 1, 512);
        b.result = ggml_add(ctx, x, bias); b.roots = { b.result }; return b; }));
    v.push_back(simple("add.pos_embd_view_plus_cont_transpose", "CONT+ADD", true, 16.0 * 512 * 1500, false, [](ggml_context * ctx) {
        built b; ggml_tensor * conv = in2(ctx, b, "conv_out", GGML_TYPE_F32, 1500, 512);
        ggml_tensor * pe = in2(ctx, b, "e_pe", GGML_TYPE_F32, 512, 1500);
        ggml_tensor * pev = ggml_view_2d(ctx, pe, 512, 1500, 512 * 4, 0);
        b.result = ggml_add(ctx, pev, ggml_cont(ctx, ggml_transpose(ctx, conv))); b.roots = { b.result }; return b; }));
    v.push_back(simple("mul.ln_weight_512x1500", "MUL", true, 8.0 * 512 * 1500, false, [](ggml_context * ctx) {
        built b; ggml_tensor * x = in2(ctx, b, "x", GGML_TYPE_F32, 512, 1500);
        ggml_tensor * w = ggml_new_tensor_1d(ctx, GGML_TYPE_F32, 512); ggml_set_name(w, "w"); b.inputs.push_back({ w, FILL_NORMAL, 0.02f, 1.0f });
        b.result = ggml_mul(ctx, x, w); b.roots = { b.result }; return b; }));
    v.push_back(simple("add.odd_shapes_bcast_dim1_dim2", "ADD", true, 0, false, [](ggml_context * ctx) {
        built b; ggml_tensor * x = ggml_new_tensor_3d(ctx, GGML_TYPE_F32, 7, 5, 6); ggml_set_name(x, "x"); b.inputs.push_back({ x, FILL_NORMAL, 1.0f });
        ggml_tensor * y = ggml_new_tensor_3d(ctx, GGML_TYPE_F32, 7, 1, 3); ggml_set_name(y, "y"); b.inputs.push_back({ y, FILL_NORMAL, 1.0f });
        b.result = ggml_add(ctx, x, y); b.roots = { b.result }; return b; }));

    // CPY / CONT (src/whisper.cpp:2155-2156, 2102, 2590-2601, 2523)
    v.push_back(simple("cpy.f32_to_f16_kv_store_1280x1500", "CPY", true, 6.0 * 1280 * 1500, false, [](ggml_context * ctx) {
        built b; ggml_tensor * x = in2(ctx, b, "kcur", GGML_TYPE_F32, 1280, 1500);
        ggml_tensor * cache = ggml_new_tensor_1d(ctx, GGML_TYPE_F16, 1280 * 1536); ggml_set_name(cache, "kv_pad"); b.inputs.push_back({ cache, FILL_NORMAL, 1.0f });
        b.roots = { ggml_cpy(ctx, x, ggml_view_1d(ctx, cache, 1280 * 1500, 0)) }; b.result = cache; return b; }));
    v.push_back(simple("cpy.f32_to_f16_self_kv_offset_n5", "CPY", true, 6.0 * 1280 * 5, false, [](ggml_context * ctx) {
        built b; ggml_tensor * x = in2(ctx, b, "kcur", GGML_TYPE_F32, 1280, 5);
        ggml_tensor * cache = ggml_new_tensor_1d(ctx, GGML_TYPE_F16, 1280 * 448 * 2); ggml_set_name(cache, "kv_self"); b.inputs.push_back({ cache, FILL_NORMAL, 1.0f });
        b.roots = { ggml_cpy(ctx, x, ggml_view_1d(ctx, cache, 5 * 1280, (size_t) 2 * 1280 * (448 + 37))) }; b.result = cache; return b; }));
    v.push_back(simple("cpy.f32_to_f16_strided_vT_store", "CPY", true, 6.0 * 1280 * 5, false, [](ggml_context * ctx) {
        built b; ggml_tensor * x = in2(ctx, b, "vcur", GGML_TYPE_F32, 1280, 5);
        ggml_tensor * cache = ggml_new_tensor_1d(ctx, GGML_TYPE_F16, 1280 * 448); ggml_set_name(cache, "kv_self_vT"); b.inputs.push_back({ cache, FILL_NORMAL, 1.0f });
        ggml_tensor * vT = ggml_transpose(ctx, ggml_reshape_2d(ctx, x, 1280, 5));
        ggml_tensor * dst = ggml_view_2d(ctx, cache, 5, 1280, 448 * 2, 37 * 2);
        b.roots = { ggml_cpy(ctx, vT, dst) }; b.result = cache; return b; }));
    v.push_back(simple("cont.transpose_1500x1280", "CONT", true, 8.0 * 1280 * 1500, false, [](ggml_context * ctx) {
        built b; ggml_tensor * x = in2(ctx, b, "x", GGML_TYPE_F32, 1500, 1280);
        b.result = ggml_cont(ctx, ggml_transpose(ctx, x)); b.roots = { b.result }; return b; }));
    v.push_back(simple("cont.permute_heads_64x5x20", "CONT", true, 0, false, [](ggml_context * ctx) {
        built b; ggml_tensor * x = ggml_new_tensor_3d(ctx, GGML_TYPE_F32, 64, 5, 20); ggml_set_name(x, "kqv"); b.inputs.push_back({ x, FILL_NORMAL, 1.0f });
        b.result = ggml_cont_2d(ctx, ggml_permute(ctx, x, 0, 2, 1, 3), 1280, 5); b.roots = { b.result }; return b; }));
    v.push_back(simple("cpy.mask_cast_f32_to_f16_448x64", "CPY", true, 6.0 * 448 * 64, false, [](ggml_context * ctx) {
        built b; ggml_tensor * m = ggml_new_tensor_3d(ctx, GGML_TYPE_F32, 448, 64, 1); ggml_set_name(m, "KQ_mask");
        input im{ m, FILL_MASK }; im.range = 1; im.rows = 5; b.inputs.push_back(im);
        b.result = ggml_cast(ctx, m, GGML_TYPE_F16); b.roots = { b.result }; return b; }));

    // GET_ROWS: the dequantization contract (bit-exact with dequantize_row_q5_0 / q8_0)
    auto get_rows_case = [](const std::string & name, ggml_type t, int64_t ne0, int64_t rows, int64_t nids) {
        return simple(name, "GET_ROWS", true, 8.0 * ne0 * nids, false, [=](ggml_context * ctx) {
            built b; ggml_tensor * tab = ggml_new_tensor_2d(ctx, t, ne0, rows); ggml_set_name(tab, "table"); b.inputs.push_back({ tab, FILL_NORMAL, 0.02f });
            ggml_tensor * ids = ggml_new_tensor_1d(ctx, GGML_TYPE_I32, nids); ggml_set_name(ids, "ids");
            input ii{ ids, FILL_IDS }; ii.range = rows; b.inputs.push_back(ii);
            b.result = ggml_get_rows(ctx, tab, ids); b.roots = { b.result }; return b; });
    };
    v.push_back(get_rows_case("get_rows.q5_0_dequant_1280x4096_all", GGML_TYPE_Q5_0, 1280, 4096, 4096));
    v.push_back(get_rows_case("get_rows.q8_0_dequant_1280x4096_all", GGML_TYPE_Q8_0, 1280, 4096, 4096));
    v.push_back(get_rows_case("get_rows.q8_0_token_embd_n5", GGML_TYPE_Q8_0, 1280, 51866, 5));
    v.push_back(get_rows_case("get_rows.f32_pos_embd_n5", GGML_TYPE_F32, 1280, 448, 5));
    v.push_back(get_rows_case("get_rows.f16_n7", GGML_TYPE_F16, 512, 100, 7));

    // SOFT_MAX (non-flash path, src/whisper.cpp:2186, 2633)
    auto soft_max_case = [](const std::string & name, int64_t ne0, int64_t ne1, int64_t ne2, int mask_type /*0 none, 1 f32, 2 f16*/, float scale) {
        return simple(name, "SOFT_MAX", false, 8.0 * ne0 * ne1 * ne2, false, [=](ggml_context * ctx) {
            built b; ggml_tensor * x = ggml_new_tensor_3d(ctx, GGML_TYPE_F32, ne0, ne1, ne2); ggml_set_name(x, "kq"); b.inputs.push_back({ x, FILL_NORMAL, 3.0f });
            ggml_tensor * m = nullptr;
            if (mask_type) {
                m = ggml_new_tensor_2d(ctx, mask_type == 1 ? GGML_TYPE_F32 : GGML_TYPE_F16, ne0, GGML_PAD(ne1, GGML_KQ_MASK_PAD)); ggml_set_name(m, "mask");
                input im{ m, FILL_MASK }; im.range = 1; im.rows = ne1; b.inputs.push_back(im);
            }
            b.result = ggml_soft_max_ext(ctx, x, m, scale, 0.0f); b.roots = { b.result }; return b; });
    };
    v.push_back(soft_max_case("soft_max.enc_1500x64x8_nomask", 1500, 64, 8, 0, 0.125f));
    v.push_back(soft_max_case("soft_max.self_37x5x20_f32mask", 37, 5, 20, 1, 1.0f));
    v.push_back(soft_max_case("soft_max.self_448x5x20_f16mask", 448, 5, 20, 2, 1.0f));

    // CONCAT (DTW path, src/whisper.cpp:2744)
    v.push_back(simple("concat.dim2_1500x5", "CONCAT", true, 0, false, [](ggml_context * ctx) {
        built b; ggml_tensor * x = ggml_new_tensor_3d(ctx, GGML_TYPE_F32, 1500, 5, 2); ggml_set_name(x, "a"); b.inputs.push_back({ x, FILL_NORMAL, 1.0f });
        ggml_tensor * y = ggml_new_tensor_3d(ctx, GGML_TYPE_F32, 1500, 5, 3); ggml_set_name(y, "b"); b.inputs.push_back({ y, FILL_NORMAL, 1.0f });
        b.result = ggml_concat(ctx, x, y, 2); b.roots = { b.result }; return b; }));

    return v;
}

} // namespace ops
