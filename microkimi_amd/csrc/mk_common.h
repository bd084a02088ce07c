// Shared device helpers for the gfx950 kernels (wave64, CDNA4).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mk_hip.h"

#define MK_WAVE 64

typedef _Float16 mk_h2 __attribute__((ext_vector_type(2)));
typedef float mk_f2 __attribute__((ext_vector_type(2)));
typedef int mk_i4 __attribute__((ext_vector_type(4)));
typedef int mk_i8v __attribute__((ext_vector_type(8)));
typedef float mk_f4 __attribute__((ext_vector_type(4)));
typedef float mk_f16v __attribute__((ext_vector_type(16)));

// 2^(sb-127) from an e8m0 byte as an exact bit pattern; byte 0 is the
// subnormal 2^-127 (mxfp4::scale_from_byte, src/mxfp4.rs:340-346).
__device__ __forceinline__ float mk_scale_from_byte(uint32_t sb) {
    return __uint_as_float(sb == 0 ? 0x00400000u : (sb << 23));
}

// 2^(sb-128) (mxfp4::exp2_i(sb - 128), src/mxfp4.rs:10-16,415): bytes 0 and 1
// are the subnormals 2^-128 and 2^-127.
__device__ __forceinline__ float mk_half_scale_from_byte(uint32_t sb) {
    return __uint_as_float(sb >= 2 ? ((sb - 1) << 23) : (sb == 1 ? 0x00400000u : 0x00200000u));
}

// E2M1 value of a nibble (src/mxfp4.rs:5-7), sign kept on zero.
__device__ __forceinline__ float mk_e2m1(uint32_t nib) {
    // magnitudes 0, .5, 1, 1.5, 2, 3, 4, 6 as f32 bit patterns
    const uint32_t mag = nib & 7u;
    uint32_t bits;
    switch (mag) {
        case 0: bits = 0x00000000u; break;
        case 1: bits = 0x3F000000u; break;
        case 2: bits = 0x3F800000u; break;
        case 3: bits = 0x3FC00000u; break;
        case 4: bits = 0x40000000u; break;
        case 5: bits = 0x40400000u; break;
        case 6: bits = 0x40800000u; break;
        default: bits = 0x40C00000u; break;
    }
    return __uint_as_float(bits | ((nib & 8u) << 28));
}

__device__ __forceinline__ float mk_wave_sum(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, MK_WAVE);
    return v;
}

__device__ __forceinline__ float mk_wave_max(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, MK_WAVE));
    return v;
}

// sum / max over aligned groups of 32 lanes
__device__ __forceinline__ float mk_half_wave_max(float v) {
#pragma unroll
    for (int off = 16; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, MK_WAVE));
    return v;
}

// q8 rounding of one value against its block scale (src/q8.rs:66): round half
// away from zero, clamp to +-127.  dx > 0.
__device__ __forceinline__ int mk_q8_round(float v, float dx) {
    float r = roundf(v / dx);
    r = fminf(fmaxf(r, -127.0f), 127.0f);
    return (int)r;
}

// f16 scale stored as raw bits -> f32
__device__ __forceinline__ float mk_f16_bits_to_f32(uint16_t b) {
    union {
        uint16_t u;
        _Float16 h;
    } c;
    c.u = b;
    return (float)c.h;
}
__device__ __forceinline__ uint16_t mk_f32_to_f16_bits(float f) {
    union {
        uint16_t u;
        _Float16 h;
    } c;
    c.h = (_Float16)f;  // round to nearest even
    return c.u;
}

// silu(x) = x / (1 + exp(-x)) (src/deepseek.rs:97-100)
__device__ __forceinline__ float mk_silu(float x) { return x / (1.0f + expf(-x)); }
// situ (src/model.rs:619-621)
__device__ __forceinline__ float mk_situ(float g, float u) {
    return 4.0f * tanhf(g / 4.0f) * (1.0f / (1.0f + expf(-g))) * (25.0f * tanhf(u / 25.0f));
}
__device__ __forceinline__ float mk_act(int kind, float g, float u, float limit, float wgt) {
    if (kind == MK_ACT_SITU) return mk_situ(g, u);
    if (kind == MK_ACT_DS) {
        g = fminf(g, limit);
        u = fminf(fmaxf(u, -limit), limit);
        return wgt * (g / (1.0f + expf(-g))) * u;
    }
    return (g / (1.0f + expf(-g))) * u;
}

// host side ---------------------------------------------------------------
void mk_set_error(const char *fmt, ...);
int mk_check_hip(hipError_t e, const char *what);
#define MK_HIP_TRY(expr)                                \
    do {                                                \
        int _s = mk_check_hip((expr), #expr);           \
        if (_s != MK_OK) return _s;                     \
    } while (0)
#define MK_REQUIRE(cond, msg)                           \
    do {                                                \
        if (!(cond)) {                                  \
            mk_set_error("invalid argument: %s", msg);  \
            return MK_ERR_INVALID;                      \
        }                                               \
    } while (0)
int mk_launch_status(const char *kernel);
