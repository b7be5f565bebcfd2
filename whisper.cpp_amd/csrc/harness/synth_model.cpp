#include "synth_model.h"

#include <math.h>
#include <stdio.h>
#include <string.h>

#include <algorithm>

namespace synth {

static const arch k_archs[] = {
    //  name              n_vocab  a_ctx a_state a_head a_layer t_ctx t_state t_head t_layer n_mels
    { "micro",            51865,   1500,  128,    2,     2,     448,  128,    2,     2,      80  },
    { "tiny",             51865,   1500,  384,    6,     4,     448,  384,    6,     4,      80  },
    { "base",             51865,   1500,  512,    8,     6,     448,  512,    8,     6,      80  },
    { "small",            51865,   1500,  768,    12,    12,    448,  768,    12,    12,     80  },
    { "medium",           51865,   1500,  1024,   16,    24,    448,  1024,   16,    24,     80  },
    { "large-v3",         51866,   1500,  1280,   20,    32,    448,  1280,   20,    32,     128 },
    { "large-v3-turbo",   51866,   1500,  1280,   20,    32,    448,  1280,   20,    4,      128 },
};

const arch * find_arch(const std::string & name) {
    for (const arch & a : k_archs) if (name == a.name) return &a;
    return nullptr;
}

int ftype_from_name(const std::string & s) {
    if (s == "f16")  return FT_F16;
    if (s == "q8_0") return FT_Q8_0;
    if (s == "q5_0") return FT_Q5_0;
    return -1;
}

int wtype_of_ftype(int ftype) {
    switch (ftype) {
        case FT_F16:  return T_F16;
        case FT_Q8_0: return T_Q8_0;
        case FT_Q5_0: return T_Q5_0;
        default:      return -1;
    }
}

// ---- numbers -------------------------------------------------------------------------------------------

static inline uint64_t splitmix64(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

static inline double uniform01(uint64_t bits) {   // (0, 1]
    return ((double)(bits >> 11) + 1.0) * (1.0 / 9007199254740992.0);
}

float normal_at(uint64_t seed, uint64_t index) {
    const uint64_t h  = splitmix64(seed * 0xD6E8FEB86659FD93ull + (index >> 1));
    const double   u1 = uniform01(splitmix64(h));
    const double   u2 = uniform01(splitmix64(h ^ 0xA5A5A5A5A5A5A5A5ull));
    const double   r  = sqrt(-2.0 * log(u1));
    const double   t  = 6.283185307179586476925 * u2;
    return (float)((index & 1) ? r * sin(t) : r * cos(t));
}

uint16_t f32_to_f16(float f) {
    uint32_t x; memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t absx = x & 0x7FFFFFFFu;
    if (absx >= 0x7F800000u) return (uint16_t)(sign | (absx > 0x7F800000u ? 0x7E00u : 0x7C00u));   // nan / inf
    if (absx >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);                                     // rounds to inf (>= 65520)
    if (absx < 0x33000001u)  return (uint16_t) sign;                                                // rounds to zero (<= 2^-25)
    int32_t  e = (int32_t)(absx >> 23) - 127;
    uint32_t m = (absx & 0x7FFFFFu) | 0x800000u;
    int shift;
    uint32_t base;
    if (e >= -14) { shift = 13; base = (uint32_t)(e + 15) << 10; m &= 0x7FFFFFu; }   // normal: drop the hidden bit
    else          { shift = 13 + (-14 - e); base = 0; }                               // subnormal: keep it
    uint32_t h = m >> shift;
    const uint32_t rem = m & ((1u << shift) - 1), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (h & 1))) ++h;                                  // nearest, ties to even
    return (uint16_t)(sign | (base + h));                                             // a carry out of the mantissa bumps the exponent
}

float f16_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1F, m = h & 0x3FF;
    uint32_t x;
    if (e == 0) {
        if (m == 0) x = sign;
        else {
            int s = 0; uint32_t mm = m;
            while (!(mm & 0x400)) { mm <<= 1; ++s; }
            x = sign | ((uint32_t)(127 - 15 - s + 1) << 23) | ((mm & 0x3FF) << 13);
        }
    } else if (e == 31) x = sign | 0x7F800000u | (m << 13);
    else                x = sign | ((e + 112) << 23) | (m << 13);
    float f; memcpy(&f, &x, 4);
    return f;
}

// ---- quantizers (ggml/src/ggml-quants.c:105-143, 194-215) ---------------------------------------------

void quantize_q5_0(const float * x, void * vy, int64_t k) {
    uint8_t * y = (uint8_t *) vy;
    for (int64_t i = 0; i < k / 32; ++i, x += 32, y += 22) {
        float amax = 0.0f, vmax = 0.0f;                      // value of largest magnitude, sign kept
        for (int j = 0; j < 32; ++j) if (amax < fabsf(x[j])) { amax = fabsf(x[j]); vmax = x[j]; }
        const float d  = vmax / -16;
        const float id = d ? 1.0f / d : 0.0f;
        const uint16_t dh = f32_to_f16(d);
        memcpy(y, &dh, 2);
        uint32_t qh = 0;
        for (int j = 0; j < 16; ++j) {
            const float x0 = x[j] * id, x1 = x[16 + j] * id;
            const uint8_t q0 = (uint8_t) std::min(31, (int)(int8_t)(x0 + 16.5f));   // truncation toward zero, then clamp
            const uint8_t q1 = (uint8_t) std::min(31, (int)(int8_t)(x1 + 16.5f));
            y[6 + j] = (uint8_t)((q0 & 0x0F) | ((q1 & 0x0F) << 4));
            qh |= (uint32_t)((q0 & 0x10u) >> 4) << j;
            qh |= (uint32_t)((q1 & 0x10u) >> 4) << (j + 16);
        }
        memcpy(y + 2, &qh, 4);
    }
}

void quantize_q8_0(const float * x, void * vy, int64_t k) {
    uint8_t * y = (uint8_t *) vy;
    for (int64_t i = 0; i < k / 32; ++i, x += 32, y += 34) {
        float amax = 0.0f;
        for (int j = 0; j < 32; ++j) amax = std::max(amax, fabsf(x[j]));
        const float d  = amax / 127;
        const float id = d ? 1.0f / d : 0.0f;
        const uint16_t dh = f32_to_f16(d);
        memcpy(y, &dh, 2);
        for (int j = 0; j < 32; ++j) ((int8_t *) y)[2 + j] = (int8_t) roundf(x[j] * id);
    }
}

static size_t tensor_bytes(int type, int64_t n) {
    switch (type) {
        case T_F32:  return (size_t) n * 4;
        case T_F16:  return (size_t) n * 2;
        case T_Q5_0: return (size_t)(n / 32) * 22;
        case T_Q8_0: return (size_t)(n / 32) * 34;
    }
    return 0;
}

std::vector<uint8_t> random_tensor(int type, int64_t n, uint64_t seed, float scale, float offset) {
    std::vector<uint8_t> out(tensor_bytes(type, n));
    const int64_t chunk = 32 * 1024;                       // multiple of the block size
    const int64_t nchunks = (n + chunk - 1) / chunk;
#pragma omp parallel for schedule(dynamic, 4)
    for (int64_t c = 0; c < nchunks; ++c) {
        const int64_t i0 = c * chunk, i1 = std::min(n, i0 + chunk);
        std::vector<float> tmp((size_t)(i1 - i0));
        for (int64_t i = i0; i < i1; ++i) tmp[(size_t)(i - i0)] = scale * normal_at(seed, (uint64_t) i) + offset;
        switch (type) {
            case T_F32:  memcpy(out.data() + i0 * 4, tmp.data(), tmp.size() * 4); break;
            case T_F16:  for (int64_t i = i0; i < i1; ++i) { uint16_t h = f32_to_f16(tmp[(size_t)(i - i0)]); memcpy(out.data() + i * 2, &h, 2); } break;
            case T_Q5_0: quantize_q5_0(tmp.data(), out.data() + (i0 / 32) * 22, i1 - i0); break;
            case T_Q8_0: quantize_q8_0(tmp.data(), out.data() + (i0 / 32) * 34, i1 - i0); break;
        }
    }
    return out;
}

// ---- file writer ------------------------------------------------------------------------------------------

namespace {

struct writer {
    FILE * f;
    bool   ok = true;
    uint64_t seed;
    int    n_written = 0;
    template <typename T> void put(T v) { ok = ok && fwrite(&v, sizeof(T), 1, f) == 1; }
    void put_bytes(const void * p, size_t n) { ok = ok && (n == 0 || fwrite(p, 1, n, f) == n); }

    // tensor record: n_dims, name length, type, dims (innermost first), name, data (src/whisper.cpp:1882-1950)
    void tensor(const std::string & name, int type, std::vector<int32_t> ne, float scale, float offset = 0.0f) {
        int64_t n = 1;
        for (int32_t d : ne) n *= d;
        put<int32_t>((int32_t) ne.size());
        put<int32_t>((int32_t) name.size());
        put<int32_t>(type);
        for (int32_t d : ne) put<int32_t>(d);
        put_bytes(name.data(), name.size());
        uint64_t h = seed;
        for (char c : name) h = splitmix64(h ^ (uint8_t) c);   // per-tensor stream
        std::vector<uint8_t> data = random_tensor(type, n, h, scale, offset);
        put_bytes(data.data(), data.size());
        ++n_written;
    }
};

} // namespace

bool write_model(const std::string & path, const arch & a, int ftype, uint64_t seed) {
    const int wtype = wtype_of_ftype(ftype);
    if (wtype < 0) return false;
    FILE * f = fopen(path.c_str(), "wb");
    if (!f) return false;
    writer w{ f, true, seed };

    w.put<uint32_t>(0x67676d6c);                         // GGML_FILE_MAGIC (ggml/include/ggml.h:212)
    w.put<int32_t>(a.n_vocab);
    w.put<int32_t>(a.n_audio_ctx);
    w.put<int32_t>(a.n_audio_state);
    w.put<int32_t>(a.n_audio_head);
    w.put<int32_t>(a.n_audio_layer);
    w.put<int32_t>(a.n_text_ctx);
    w.put<int32_t>(a.n_text_state);
    w.put<int32_t>(a.n_text_head);
    w.put<int32_t>(a.n_text_layer);
    w.put<int32_t>(a.n_mels);
    w.put<int32_t>(ftype == FT_F16 ? ftype : 2 * 1000 + ftype);   // GGML_QNT_VERSION 2 * GGML_QNT_VERSION_FACTOR 1000

    // mel filter bank: only consumed by the PCM front end, which synthetic runs bypass with whisper_set_mel
    const int n_fft = 201;
    w.put<int32_t>(a.n_mels);
    w.put<int32_t>(n_fft);
    {
        std::vector<float> filters((size_t) a.n_mels * n_fft, 0.0f);
        for (int m = 0; m < a.n_mels; ++m) filters[(size_t) m * n_fft + (m * n_fft) / a.n_mels] = 1.0f;
        w.put_bytes(filters.data(), filters.size() * 4);
    }

    // vocabulary: 50257 placeholder byte strings; id 220 is " " because whisper_process_logits looks it up
    // (src/whisper.cpp:5057).  The loader synthesises the special tokens above 50257 itself (:1654-1685).
    const int n_tok = 50257;
    w.put<int32_t>(n_tok);
    for (int i = 0; i < n_tok; ++i) {
        std::string s = i == 220 ? std::string(" ") : "t" + std::to_string(i);
        w.put<uint32_t>((uint32_t) s.size());
        w.put_bytes(s.data(), s.size());
    }

    const int   d = a.n_audio_state, dt = a.n_text_state;
    const float sw = 0.02f;                               // weights ~ N(0, 0.02)
    const int vtype = T_F16;                              // conv weights stay f16 (examples/common-ggml.cpp:138-139)

    // encoder (tensor set: src/whisper.cpp:1778-1811; names: src/whisper-arch.h:42-68)
    w.tensor("encoder.positional_embedding", T_F32, { d, a.n_audio_ctx }, sw);
    w.tensor("encoder.conv1.weight", vtype, { 3, a.n_mels, d }, sw);
    w.tensor("encoder.conv1.bias",   T_F32, { 1, d }, sw);
    w.tensor("encoder.conv2.weight", vtype, { 3, d, d }, sw);
    w.tensor("encoder.conv2.bias",   T_F32, { 1, d }, sw);
    w.tensor("encoder.ln_post.weight", T_F32, { d }, sw, 1.0f);
    w.tensor("encoder.ln_post.bias",   T_F32, { d }, sw);
    for (int i = 0; i < a.n_audio_layer; ++i) {
        const std::string p = "encoder.blocks." + std::to_string(i) + ".";
        w.tensor(p + "mlp_ln.weight", T_F32, { d }, sw, 1.0f);
        w.tensor(p + "mlp_ln.bias",   T_F32, { d }, sw);
        w.tensor(p + "mlp.0.weight",  wtype, { d, 4 * d }, sw);
        w.tensor(p + "mlp.0.bias",    T_F32, { 4 * d }, sw);
        w.tensor(p + "mlp.2.weight",  wtype, { 4 * d, d }, sw);
        w.tensor(p + "mlp.2.bias",    T_F32, { d }, sw);
        w.tensor(p + "attn_ln.weight", T_F32, { d }, sw, 1.0f);
        w.tensor(p + "attn_ln.bias",   T_F32, { d }, sw);
        w.tensor(p + "attn.query.weight", wtype, { d, d }, sw);
        w.tensor(p + "attn.query.bias",   T_F32, { d }, sw);
        w.tensor(p + "attn.key.weight",   wtype, { d, d }, sw);
        w.tensor(p + "attn.value.weight", wtype, { d, d }, sw);
        w.tensor(p + "attn.value.bias",   T_F32, { d }, sw);
        w.tensor(p + "attn.out.weight",   wtype, { d, d }, sw);
        w.tensor(p + "attn.out.bias",     T_F32, { d }, sw);
    }
    // decoder (src/whisper.cpp:1814-1856; names: src/whisper-arch.h:70-109)
    w.tensor("decoder.positional_embedding", T_F32, { dt, a.n_text_ctx }, sw);
    w.tensor("decoder.token_embedding.weight", wtype, { dt, a.n_vocab }, sw);
    w.tensor("decoder.ln.weight", T_F32, { dt }, sw, 1.0f);
    w.tensor("decoder.ln.bias",   T_F32, { dt }, sw);
    for (int i = 0; i < a.n_text_layer; ++i) {
        const std::string p = "decoder.blocks." + std::to_string(i) + ".";
        w.tensor(p + "mlp_ln.weight", T_F32, { dt }, sw, 1.0f);
        w.tensor(p + "mlp_ln.bias",   T_F32, { dt }, sw);
        w.tensor(p + "mlp.0.weight",  wtype, { dt, 4 * dt }, sw);
        w.tensor(p + "mlp.0.bias",    T_F32, { 4 * dt }, sw);
        w.tensor(p + "mlp.2.weight",  wtype, { 4 * dt, dt }, sw);
        w.tensor(p + "mlp.2.bias",    T_F32, { dt }, sw);
        w.tensor(p + "attn_ln.weight", T_F32, { dt }, sw, 1.0f);
        w.tensor(p + "attn_ln.bias",   T_F32, { dt }, sw);
        w.tensor(p + "attn.query.weight", wtype, { dt, dt }, sw);
        w.tensor(p + "attn.query.bias",   T_F32, { dt }, sw);
        w.tensor(p + "attn.key.weight",   wtype, { dt, dt }, sw);
        w.tensor(p + "attn.value.weight", wtype, { dt, dt }, sw);
        w.tensor(p + "attn.value.bias",   T_F32, { dt }, sw);
        w.tensor(p + "attn.out.weight",   wtype, { dt, dt }, sw);
        w.tensor(p + "attn.out.bias",     T_F32, { dt }, sw);
        w.tensor(p + "cross_attn_ln.weight", T_F32, { dt }, sw, 1.0f);
        w.tensor(p + "cross_attn_ln.bias",   T_F32, { dt }, sw);
        w.tensor(p + "cross_attn.query.weight", wtype, { dt, dt }, sw);
        w.tensor(p + "cross_attn.query.bias",   T_F32, { dt }, sw);
        w.tensor(p + "cross_attn.key.weight",   wtype, { dt, dt }, sw);
        w.tensor(p + "cross_attn.value.weight", wtype, { dt, dt }, sw);
        w.tensor(p + "cross_attn.value.bias",   T_F32, { dt }, sw);
        w.tensor(p + "cross_attn.out.weight",   wtype, { dt, dt }, sw);
        w.tensor(p + "cross_attn.out.bias",     T_F32, { dt }, sw);
    }
    const bool ok = w.ok && fclose(f) == 0;
    return ok;
}

std::vector<float> synthetic_mel(int n_mels, int n_len, uint64_t seed) {
    const size_t n = (size_t) n_mels * n_len;
    std::vector<float> x(n);
    float mmax = -1e20f;
    for (size_t i = 0; i < n; ++i) {
        const double u = uniform01(splitmix64(seed * 0x9E3779B97F4A7C15ull + i));
        const double power = std::max(-log(u), 1e-10);   // Exp(1), clamped like the 1e-10 floor of the front end
        x[i] = (float) log10(power);
        mmax = std::max(mmax, x[i]);
    }
    mmax -= 8.0f;
    for (size_t i = 0; i < n; ++i) x[i] = (std::max(x[i], mmax) + 4.0f) / 4.0f;
    return x;
}

} // namespace synth
