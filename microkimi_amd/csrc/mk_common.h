// Shared device helpers for the gfx950 kernels (wave64, CDNA4).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mk_hip.h"

#define MK_WAVE 64

// The reference is Rust, which never fuses a multiplication with the addition that follows it.  Device code is
// compiled with contraction on by default, so it is switched off for everything that includes this header
// (a fused multiply-add is written fmaf / __builtin_elementwise_fma where one is wanted).  mk_add / mk_mul mark
// the places where the separate roundings are part of the parity contract; HIP's __fadd_rn / __fmul_rn are plain
// operators inside header functions compiled with contraction on, and do get fused after inlining.
#pragma clang fp contract(off)
__device__ __forceinline__ float mk_add(float a, float b) { return a + b; }
__device__ __forceinline__ float mk_mul(float a, float b) { return a * b; }

typedef _Float16 mk_h2 __attribute__((ext_vector_type(2)));
typedef float mk_f2 __attribute__((ext_vector_type(2)));
typedef int mk_i4 __attribute__((ext_vector_type(4)));
typedef int mk_i8v __attribute__((ext_vector_type(8)));
typedef float mk_f4 __attribute__((ext_vector_type(4)));
typedef unsigned int mk_u2 __attribute__((ext_vector_type(2)));
typedef unsigned int mk_v4u __attribute__((ext_vector_type(4)));
typedef float mk_f16v __attribute__((ext_vector_type(16)));

// Loads that tell the compiler the pointer is global memory.  A pointer that was
// itself loaded from memory (an expert table entry) is a generic pointer to the
// compiler and would be read with flat_load, which also ties up the LDS counter.
#define MK_GLOBAL __attribute__((address_space(1)))
__device__ __forceinline__ mk_i4 mk_ldg128(const void *p) { return *(const MK_GLOBAL mk_i4 *)(const MK_GLOBAL void *)p; }
// base + 32-bit byte offset, with the address arithmetic done in the global address space: a uniform base
// and a lane offset then become the scalar-base form of the load (no 64-bit address per lane)
__device__ __forceinline__ mk_i4 mk_ldg128_off(const void *base, uint32_t off) {
    const MK_GLOBAL uint8_t *b = (const MK_GLOBAL uint8_t *)base;
    return *(const MK_GLOBAL mk_i4 *)(b + off);
}
// the same, marked non-temporal: for data that is streamed once and should not displace what the caches hold
__device__ __forceinline__ mk_i4 mk_ldg128_off_nt(const void *base, uint32_t off) {
    const MK_GLOBAL uint8_t *b = (const MK_GLOBAL uint8_t *)base;
    return __builtin_nontemporal_load((const MK_GLOBAL mk_i4 *)(b + off));
}
__device__ __forceinline__ uint32_t mk_ldg_u8_off(const void *base, uint32_t off) {
    const MK_GLOBAL uint8_t *b = (const MK_GLOBAL uint8_t *)base;
    return b[off];
}
__device__ __forceinline__ uint16_t mk_ldg_u16_off(const void *base, uint32_t off) {
    const MK_GLOBAL uint8_t *b = (const MK_GLOBAL uint8_t *)base;
    return *(const MK_GLOBAL uint16_t *)(b + off);
}
__device__ __forceinline__ float mk_ldg_f32_off(const void *base, uint32_t off) {
    const MK_GLOBAL uint8_t *b = (const MK_GLOBAL uint8_t *)base;
    return *(const MK_GLOBAL float *)(b + off);
}
__device__ __forceinline__ mk_u2 mk_ldg64(const void *p) { return *(const MK_GLOBAL mk_u2 *)(const MK_GLOBAL void *)p; }
__device__ __forceinline__ uint32_t mk_ldg_u32(const void *p) { return *(const MK_GLOBAL uint32_t *)(const MK_GLOBAL void *)p; }
__device__ __forceinline__ mk_i4 mk_ldg128_nt(const void *p) { return __builtin_nontemporal_load((const MK_GLOBAL mk_i4 *)(const MK_GLOBAL void *)p); }
__device__ __forceinline__ uint32_t mk_ldg_u8(const void *p) { return *(const MK_GLOBAL uint8_t *)(const MK_GLOBAL void *)p; }
__device__ __forceinline__ uint16_t mk_ldg_u16(const void *p) { return *(const MK_GLOBAL uint16_t *)(const MK_GLOBAL void *)p; }
__device__ __forceinline__ float mk_ldg_f32(const void *p) { return *(const MK_GLOBAL float *)(const MK_GLOBAL void *)p; }

// A pointer that is the same in every lane but was loaded with a vector load (an
// expert table entry): moving it to scalar registers lets the loads that use it
// take the "scalar base + 32-bit lane offset" form instead of a 64-bit address per lane.
__device__ __forceinline__ const uint8_t *mk_uniform_ptr(const uint8_t *p) {
    const uint64_t v = (uint64_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (const uint8_t *)(((uint64_t)hi << 32) | lo);
}

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

// Wave-wide reductions without LDS traffic: four DPP steps fold each row of 16
// lanes (quad swaps, half-row mirror, row mirror), then the four row results are
// read with v_readlane and combined.  All 64 lanes must be active.  The result
// is the same value in every lane; the association is fixed (deterministic).
template <int CTRL>
__device__ __forceinline__ float mk_dpp(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
template <int CTRL>
__device__ __forceinline__ int mk_dpp_i(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}
__device__ __forceinline__ float mk_readlane(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}
__device__ __forceinline__ float mk_wave_sum(float v) {
    v += mk_dpp<0xB1>(v);   // quad_perm [1,0,3,2]
    v += mk_dpp<0x4E>(v);   // quad_perm [2,3,0,1]
    v += mk_dpp<0x141>(v);  // row_half_mirror
    v += mk_dpp<0x140>(v);  // row_mirror
    return (mk_readlane(v, 0) + mk_readlane(v, 16)) + (mk_readlane(v, 32) + mk_readlane(v, 48));
}

__device__ __forceinline__ float mk_wave_max(float v) {
    v = fmaxf(v, mk_dpp<0xB1>(v));
    v = fmaxf(v, mk_dpp<0x4E>(v));
    v = fmaxf(v, mk_dpp<0x141>(v));
    v = fmaxf(v, mk_dpp<0x140>(v));
    return fmaxf(fmaxf(mk_readlane(v, 0), mk_readlane(v, 16)), fmaxf(mk_readlane(v, 32), mk_readlane(v, 48)));
}

// sum / max over the four lanes {c, c+16, c+32, c+48} without LDS traffic
// (gfx950 lane-swap instructions: halves of the wave, then odd/even rows of 16).
// All 64 lanes must be active; every lane gets the result.
__device__ __forceinline__ float mk_rows_max(float v) {
    const unsigned u = __builtin_bit_cast(unsigned, v);
    mk_u2 r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    const unsigned w = __builtin_bit_cast(unsigned, fmaxf(__builtin_bit_cast(float, (unsigned)r[0]), __builtin_bit_cast(float, (unsigned)r[1])));
    r = __builtin_amdgcn_permlane16_swap(w, w, false, false);
    return fmaxf(__builtin_bit_cast(float, (unsigned)r[0]), __builtin_bit_cast(float, (unsigned)r[1]));
}
__device__ __forceinline__ float mk_rows_sum(float v) {
    const unsigned u = __builtin_bit_cast(unsigned, v);
    mk_u2 r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    const unsigned w = __builtin_bit_cast(unsigned, __builtin_bit_cast(float, (unsigned)r[0]) + __builtin_bit_cast(float, (unsigned)r[1]));
    r = __builtin_amdgcn_permlane16_swap(w, w, false, false);
    return __builtin_bit_cast(float, (unsigned)r[0]) + __builtin_bit_cast(float, (unsigned)r[1]);
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
    if (r != r) return 0;  // a NaN value, or inf / inf: the reference's `as i8` of NaN is 0 (fmaxf would drop the NaN and give -127)
    r = fminf(fmaxf(r, -127.0f), 127.0f);
    return (int)r;
}

// Four values of a q8 block at once: the same integers as mk_q8_round on each (returned as floats), at a third of the
// instructions.  q = v * rcp(dx) is within 2.3e-5 of the real quotient (|v/dx| <= 127, rcp and the product each within an
// ulp), and so is the correctly rounded v / dx of the reference; unless q's fraction is within 1e-4 of one half, all of
// them round to the same integer.  Lanes that are that close to a tie, or whose scale is too small for rcp, take the
// division.  dx > 0.
__device__ __forceinline__ void mk_q8_round4(const mk_f4 v, float dx, float *q) {
    const float r = __builtin_amdgcn_rcpf(dx);
    q[0] = v.x * r;
    q[1] = v.y * r;
    q[2] = v.z * r;
    q[3] = v.w * r;
    bool risky = dx < 1e-30f;
#pragma unroll
    for (int k = 0; k < 4; k++) risky |= !(fabsf(__builtin_amdgcn_fractf(fabsf(q[k])) - 0.5f) >= 1e-4f);
    if (risky) {
        q[0] = (float)mk_q8_round(v.x, dx);
        q[1] = (float)mk_q8_round(v.y, dx);
        q[2] = (float)mk_q8_round(v.z, dx);
        q[3] = (float)mk_q8_round(v.w, dx);
    } else {
#pragma unroll
        for (int k = 0; k < 4; k++) q[k] = __builtin_copysignf(fminf(__builtin_floorf(fabsf(q[k]) + 0.5f), 127.0f), q[k]);
    }
}
// the same as f16 integers (the form the dot kernels consume)
__device__ __forceinline__ void mk_q8_round4_f16(const mk_f4 v, float dx, mk_h2 &lo, mk_h2 &hi) {
    float q[4];
    mk_q8_round4(v, dx, q);
    lo.x = (_Float16)q[0];
    lo.y = (_Float16)q[1];
    hi.x = (_Float16)q[2];
    hi.y = (_Float16)q[3];
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

// f32 -> e4m3fn, round to nearest even, saturating at 448 (src/dequant.rs:92-120).
__device__ __forceinline__ uint32_t mk_f32_to_e4m3(float v) {
    if (v != v) return 0x7Fu;
    uint32_t sign = (__float_as_uint(v) >> 24) & 0x80u;
    float a = fminf(fabsf(v), 448.0f);
    if (a < 0.015625f) {  // below the smallest normal 2^-6: m = rne(a * 2^9), 8 carries into e=1
        return sign | (uint32_t)rintf(a * 512.0f);
    }
    uint32_t bits = __float_as_uint(a);
    uint32_t r = (bits + 0x7FFFFu + ((bits >> 20) & 1u)) >> 20;  // exponent and 3 mantissa bits, RNE with carry
    return sign | (r - (120u << 3));
}

// ceil(log2f(r)) for a normal positive r, where log2f is the correctly rounded float logarithm the reference calls
// (f32::log2; (float)log2((double)r) is that value).  With r = m * 2^k, 1 <= m < 2: the result is k when m == 1 and
// k + 1 as soon as log2(m) survives the rounding of k + log2(m) to float.  For |k| <= 127 half an ulp is at most
// 3.9e-6 and log2(m) >= 1.1e-5 once the mantissa field is 64 or more, so only mantissa fields 1..63 (one value in
// 131072) need the real logarithm; that branch is divergent and almost never taken.
__device__ __forceinline__ int mk_ceil_log2f(float r) {
    const uint32_t bits = __float_as_uint(r);
    const int k = (int)(bits >> 23) - 127;
    const uint32_t mf = bits & 0x7FFFFFu;
    if (mf == 0) return k;
    if (mf >= 64) return k + 1;
    return (int)ceilf((float)log2((double)r));
}

// MXFP8 of one value of a 32-block held by an aligned group of 32 lanes (all active): scale exponent
// e = ceil(log2(max(amax, 1e-4) / 448)) clamped to [-127, 8], code = e4m3(clamp(x / 2^e)) (deepseek::fp8_roundtrip,
// src/deepseek.rs:312-322).  Returns the code; exp_byte = e + 127.
__device__ __forceinline__ uint32_t mk_mxfp8_quantize(float v, uint32_t &exp_byte) {
    const float amax = fmaxf(mk_half_wave_max(fabsf(v)), 1e-4f);
    int e = mk_ceil_log2f(amax / 448.0f);
    e = max(-127, min(8, e));
    exp_byte = (uint32_t)(e + 127);
    const float s = mk_scale_from_byte(exp_byte);
    return mk_f32_to_e4m3(fminf(fmaxf(v / s, -448.0f), 448.0f));
}

// The same for a 32-block held as 8 consecutive values in each lane of an aligned quad of lanes: the block maximum
// needs two DPP steps, the division by the power-of-two scale is an exact multiplication, and the e4m3 codes come
// from v_cvt_pk_fp8_f32 (round to nearest even on the OCP e4m3 grid; the inputs are clamped to +-448 before).
// c0 holds the codes of v[0..3], c1 of v[4..7], lowest byte first.  EMAX: upper clamp of the scale exponent, 8 in the
// reference's rule; 127 uses the whole e8m0 range, so that no block saturates.
template <int EMAX = 8>
__device__ __forceinline__ void mk_mxfp8_quantize8(const float (&v)[8], uint32_t &exp_byte, uint32_t &c0, uint32_t &c1) {
    float a = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; i++) a = fmaxf(a, fabsf(v[i]));
    a = fmaxf(a, mk_dpp<0xB1>(a));
    a = fmaxf(a, mk_dpp<0x4E>(a));
    int e = mk_ceil_log2f(fmaxf(a, 1e-4f) / 448.0f);
    e = max(-127, min(EMAX, e));
    exp_byte = (uint32_t)(e + 127);
    // 2^-e, exact: byte 254 - (e + 127) for e < 127; for e = 127 the power 2^-127 is the subnormal that byte 0 decodes to
    const float inv = mk_scale_from_byte(254u - exp_byte);
    float q[8];
#pragma unroll
    for (int i = 0; i < 8; i++) q[i] = fminf(fmaxf(v[i] * inv, -448.0f), 448.0f);
    int w0 = 0, w1 = 0;
    w0 = __builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], w0, false);
    w0 = __builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], w0, true);
    w1 = __builtin_amdgcn_cvt_pk_fp8_f32(q[4], q[5], w1, false);
    w1 = __builtin_amdgcn_cvt_pk_fp8_f32(q[6], q[7], w1, true);
    c0 = (uint32_t)w0;
    c1 = (uint32_t)w1;
}

// bfloat16 (round to nearest even) of 8 consecutive values of a 32-block as TWO e4m3 terms per value with a block
// exponent each: x = hi + lo, hi = the leading four significant bits of the bfloat16 value (sign, exponent, three
// mantissa bits) and lo the other four -- both exact on the e4m3 grid of their block unless the value lies more than
// 2^13 below the block's largest (then its last bits round off: below 2^-17 of that largest value).  A dot product over
// hi and lo against exact weights with f32 sums is the bfloat16 dot product.  ROWS: the block's other values sit in the
// lanes c + 16, + 32, + 48 (matrix-instruction results); otherwise in the aligned quad of lanes.  Codes: lowest byte
// first, [0] = v[0..3], [1] = v[4..7].  A value that is not finite gets the e4m3 NaN code.
template <bool ROWS>
__device__ __forceinline__ void mk_bf16_split8(const float (&v)[8], uint32_t (&hi)[2], uint32_t (&lo)[2], uint32_t &exp_hi, uint32_t &exp_lo) {
    float h[8], l[8], ah = 0.0f, al = 0.0f;
    uint32_t bad[2] = {0u, 0u};
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const float b = (float)(__bf16)v[i];
        const uint32_t bits = __float_as_uint(b);
        const bool fin = (bits & 0x7F800000u) != 0x7F800000u;
        h[i] = __uint_as_float(bits & 0xFFF00000u);
        l[i] = fin ? b - h[i] : 0.0f;
        if (!fin) bad[i >> 2] |= 0x7Fu << (8 * (i & 3));
        ah = fmaxf(ah, fabsf(h[i]));
        al = fmaxf(al, fabsf(l[i]));
    }
    if constexpr (ROWS) {
        ah = mk_rows_max(ah);
        al = mk_rows_max(al);
    } else {
        ah = fmaxf(ah, mk_dpp<0xB1>(ah));
        ah = fmaxf(ah, mk_dpp<0x4E>(ah));
        al = fmaxf(al, mk_dpp<0xB1>(al));
        al = fmaxf(al, mk_dpp<0x4E>(al));
    }
    auto encode = [](const float (&x)[8], float amax, uint32_t (&codes)[2], uint32_t &exp_byte) {
        // the smallest e with amax <= 448 * 2^e, from the bits of amax = m * 2^k: k - 8, one more when m > 1.75
        const uint32_t ab = __float_as_uint(amax);
        int e = (int)(ab >> 23) - 127 - 8 + ((ab & 0x7FFFFFu) > 0x600000u ? 1 : 0);
        e = max(-127, min(127, e));
        exp_byte = (uint32_t)(e + 127);
        const float inv = mk_scale_from_byte(254u - exp_byte);  // 2^-e, exact
        float q[8];
#pragma unroll
        for (int i = 0; i < 8; i++) q[i] = fminf(fmaxf(x[i] * inv, -448.0f), 448.0f);
        int w0 = 0, w1 = 0;
        w0 = __builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], w0, false);
        w0 = __builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], w0, true);
        w1 = __builtin_amdgcn_cvt_pk_fp8_f32(q[4], q[5], w1, false);
        w1 = __builtin_amdgcn_cvt_pk_fp8_f32(q[6], q[7], w1, true);
        codes[0] = (uint32_t)w0;
        codes[1] = (uint32_t)w1;
    };
    encode(h, ah, hi, exp_hi);
    encode(l, al, lo, exp_lo);
#pragma unroll
    for (int k = 0; k < 2; k++) {
        const uint32_t m = ((bad[k] >> 6) & 0x01010101u) * 0xFFu;  // bytes of the values that are not finite
        hi[k] = (hi[k] & ~m) | (bad[k] & m);
    }
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
// The process-wide off switch (mk_set_enabled, MK_HIP=0 in the environment): 1 on, 0 off, -1 not yet read from the
// environment.  Every entry point that returns a status checks its arguments through MK_REQUIRE first, so the switch is
// tested there: a disabled library returns MK_ERR_NO_DEVICE before any HIP call.
extern int mk_enabled_state;
int mk_enabled_slow();
static inline bool mk_enabled() {
    const int v = __atomic_load_n(&mk_enabled_state, __ATOMIC_RELAXED);
    return v > 0 || (v < 0 && mk_enabled_slow());
}
#define MK_REQUIRE_ENABLED()                                                                          \
    do {                                                                                              \
        if (!mk_enabled()) {                                                                          \
            mk_set_error("the library is switched off (mk_set_enabled(0) or MK_HIP=0)");              \
            return MK_ERR_NO_DEVICE;                                                                  \
        }                                                                                             \
    } while (0)
#define MK_REQUIRE(cond, msg)                           \
    do {                                                \
        MK_REQUIRE_ENABLED();                           \
        if (!(cond)) {                                  \
            mk_set_error("invalid argument: %s", msg);  \
            return MK_ERR_INVALID;                      \
        }                                               \
    } while (0)
int mk_launch_status(const char *kernel);
// Raises a kernel's dynamic LDS limit (hipFuncAttributeMaxDynamicSharedMemorySize) once per kernel and device; checked,
// safe to call from several threads.  Launch sites call it before every launch: after the first it is a set lookup.
int mk_lds_opt_in(const void *kernel, int bytes);
// integer value of an environment variable, dflt when unset or empty
int mk_env_int(const char *name, int dflt);
// A tuning or A/B switch of a launcher: the environment is read once per process, at the first launch that asks; after
// that the value is a constant (no getenv on the launch path).
#define MK_TUNE(name, dflt) ([]() -> int { static const int v = mk_env_int(name, dflt); return v; }())

// mla.hip: resolves the device address of the static scratch of mk_dev_mla_q8_decode_static on the current device
// (once per device); out_ptr may be null.
int mk_mla_static_init(void **out_ptr);

// mk_dev_mxfp4_grouped_gemm for n_mats (1 or 2) weight matrices per group that multiply the same token rows, in one launch
// (gemm_mxfp4.hip): matrix k of group e is packed_ptrs[k][e] / scales_ptrs[k][e], its [m x rows] result goes to out[k].
// scales_t_ptrs (may be null, and so may its entries): the matrices' scale bytes in K-tile order
// (mk_dev_mxfp4_scales_by_tile), read instead of scales_ptrs by the kernels that walk K in tiles of 512.
// two: the token rows are bfloat16 values as two e4m3 terms each (mk_bf16_split8): codes [m][cols / 512][2][512], exps
// [m][cols / 512][2][16]; cols % 512 == 0.  (The gate/up call then writes the activation in that form too; rows % 512 == 0.)
int mk_mxfp4_grouped_gemm_n(int n_mats, const uint8_t *const *const *packed_ptrs, const uint8_t *const *const *scales_ptrs, size_t n_groups,
                            size_t rows, size_t cols, const uint8_t *codes, const uint8_t *exps, const int32_t *offsets, size_t m,
                            float *const *out, void *stream, const uint8_t *const *const *scales_t_ptrs = nullptr, bool two = false);
// matvec_packed_nt (f32 products and sums, gemv_mxfp4.hip) for groups of rows that each meet their own n_mats (1 or 2)
// matrices: group e owns the grouped rows offsets[e] .. offsets[e+1]; grouped row p multiplies activation row
// xrow[p] / xdiv of x (xrow null: row p itself); matrix k's [. x rows] result goes to out[k] at the grouped row.  m: the
// number of grouped rows in all (only the choice of the pass size looks at it).  vq_codebook (may be null): with it, a
// group whose scale pointer is null has a VQ1 matrix (index bytes where the packed nibbles would be) and is multiplied
// with the codebook's entries (quant::matvec_vq_nt's terms).
int mk_mxfp4_grouped_gemm_nt(int n_mats, const uint8_t *const *const *packed_ptrs, const uint8_t *const *const *scales_ptrs, size_t n_groups,
                             size_t rows, size_t cols, const float *x, const int32_t *xrow, int xdiv, const int32_t *offsets, size_t m,
                             const float *vq_codebook, float *const *out, void *stream);
// The grouped product with bfloat16 activation rows x [grouped rows][cols] (gemv_mxfp4.hip): exact bf16 weights, f32
// products and sums on the bf16 matrix instruction.  MK_ERR_UNSUPPORTED unless cols % 512 == 0 and rows % 4 == 0.
// scales_t_ptrs: as for mk_mxfp4_grouped_gemm_n.
int mk_mxfp4_grouped_gemm_bf16(int n_mats, const uint8_t *const *const *packed_ptrs, const uint8_t *const *const *scales_ptrs, size_t n_groups,
                               size_t rows, size_t cols, const uint16_t *x, const int32_t *offsets, float *const *out, void *stream,
                               const uint8_t *const *const *scales_t_ptrs = nullptr);
// The gate and up matrices of every group against the same token rows, the activation ACT(gate, up) and its MXFP8 form
// (e4m3 codes [m][rows], e8m0 bytes [m][rows / 32], whole exponent range) in one launch; the f32 gate / up rows are
// written too when keep_g and keep_u are given.  MK_ERR_UNSUPPORTED (nothing launched) for shapes it does not take.
int mk_mxfp4_grouped_gemm_gate_up_act(const uint8_t *const *w1p, const uint8_t *const *w1s, const uint8_t *const *w3p, const uint8_t *const *w3s,
                                      size_t n_groups, size_t rows, size_t cols, const uint8_t *codes, const uint8_t *exps,
                                      const int32_t *offsets, size_t m, int act_kind, uint8_t *act_codes, uint8_t *act_exps, float *keep_g,
                                      float *keep_u, void *stream, const uint8_t *const *w1st = nullptr, const uint8_t *const *w3st = nullptr,
                                      bool two = false);
