// Library identity and device probing.
#include "common.h"
#include <math.h>
#include <string.h>

#include <mutex>

extern "C" int mi355x_abi_version(void) { return 1; }

extern "C" int mi355x_device_is_gfx950(int device) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) != hipSuccess) { (void) hipGetLastError(); return -1; }
    return strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : 0;
}

extern "C" const char * mi355x_status_string(int status) {
    switch (status) {
        case MI355X_OK:              return "ok";
        case MI355X_ERR_UNSUPPORTED: return "unsupported type or layout";
        case MI355X_ERR_INVALID:     return "invalid argument";
        case MI355X_ERR_WORKSPACE:   return "workspace missing or too small";
        case MI355X_ERR_HIP:         return "HIP launch error";
        default:                     return "unknown status";
    }
}

// ------------------------------------------------------------------------------------------------------
// GELU table
// ------------------------------------------------------------------------------------------------------

static __device__ uint16_t g_gelu_table[1 << 16];

static uint16_t host_f32_to_f16(float f) {     // round-to-nearest-even, like GGML_FP32_TO_FP16
    uint32_t x; memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u, absx = x & 0x7FFFFFFFu;
    if (absx >= 0x7F800000u) return (uint16_t)(sign | (absx > 0x7F800000u ? 0x7E00u : 0x7C00u));
    if (absx >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);
    if (absx <  0x33000001u) return (uint16_t) sign;
    const int32_t e = (int32_t)(absx >> 23) - 127;
    uint32_t m = (absx & 0x7FFFFFu) | 0x800000u, base; int shift;
    if (e >= -14) { shift = 13; base = (uint32_t)(e + 15) << 10; m &= 0x7FFFFFu; } else { shift = 13 + (-14 - e); base = 0; }
    uint32_t h = m >> shift;
    const uint32_t rem = m & ((1u << shift) - 1), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (h & 1))) ++h;
    return (uint16_t)(sign | (base + h));
}
static float host_f16_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1F, m = h & 0x3FF;
    uint32_t x;
    if (e == 0) {
        if (m == 0) x = sign;
        else { int s = 0; uint32_t mm = m; while (!(mm & 0x400)) { mm <<= 1; ++s; } x = sign | ((uint32_t)(113 - s) << 23) | ((mm & 0x3FF) << 13); }
    } else if (e == 31) x = sign | 0x7F800000u | (m << 13);
    else x = sign | ((e + 112) << 23) | (m << 13);
    float f; memcpy(&f, &x, 4);
    return f;
}

// 0.5x(1 + tanh(sqrt(2/pi) x (1 + 0.044715 x^2))) with the roundings of the reference's x86 build: the inner
// 1 + (0.044715 x) x is one fused multiply-add, every other product and sum rounds on its own.  With glibc's tanhf this
// reproduces all finite entries of ggml_table_gelu_f16 bit for bit.
#pragma clang fp contract(off)
static float host_gelu(float x) {
    const float inner = fmaf(0.044715f * x, x, 1.0f);
    const float u = 0.79788456080286535587989211986876f * x;
    const float t = tanhf(u * inner);
    const float hx = 0.5f * x;
    return hx * (1.0f + t);
}

const uint16_t * gelu_table_device() {
    static std::mutex mu;
    static const uint16_t * dev_ptr[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) { (void) hipGetLastError(); return nullptr; }
    std::lock_guard<std::mutex> lock(mu);
    if (dev_ptr[dev]) return dev_ptr[dev];
    static uint16_t host[1 << 16];
    static bool built = false;
    if (!built) {
        for (uint32_t i = 0; i < (1u << 16); ++i) host[i] = host_f32_to_f16(host_gelu(host_f16_to_f32((uint16_t) i)));
        built = true;
    }
    void * p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_gelu_table)) != hipSuccess || !p) { (void) hipGetLastError(); return nullptr; }
    if (hipMemcpy(p, host, sizeof(host), hipMemcpyHostToDevice) != hipSuccess) { (void) hipGetLastError(); return nullptr; }
    dev_ptr[dev] = (const uint16_t *) p;
    return dev_ptr[dev];
}
