/*
 * mk_oracle.c -- CPU restatement of microkimi's quantized-weight hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the parity checker for the HIP
 * kernels and the timed CPU baseline of the benchmark.  Nothing in the product
 * path (the microkimi_amd package, libmk_hip.so) may link, load or call it.
 *
 * Every function restates one function of the reference (a Rust program that
 * cannot be compiled in this environment) and cites the file:line it follows.
 * Loop orders, rounding functions and the "multiply, then add, never fused"
 * rule of the reference are kept, so results are meant to be bit-identical to
 * what the reference's CPU path produces.  Build with -ffp-contract=off and
 * without -ffast-math (see Makefile): Rust never contracts a*b+c.
 *
 * What pins each function (tests/test_oracle_*.py):
 *   codec (e2m1, e8m0, e4m3)     golden vectors ref/ds_golden.json (fp4, fp8),
 *                                exhaustive closed forms
 *   quantize_q8                  constants of src/q8.rs:321-334, dx/2 bound
 *   block_dot, block_dot_i8      brute force on the reference's RNG streams
 *   matvec_packed (f32 / q8)     f64 closed forms, 1e-3 bound between modes
 *   matvec_packed_nt             bit-identity with matvec_packed (f32 mode)
 *   q8head                       src/model.rs:3866-3881 restated, f64 closed form
 *   mla_*                        bit-identity MQA vs per-head, f64 closed form,
 *                                round-trip bound, len-1 special case
 *   gate / expert                golden vectors ref/ds_golden2.json
 * No function here is "parity unpinned".
 */
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#if defined(__x86_64__)
#include <immintrin.h>
#endif

#define ORC_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------ codec */

/* src/mxfp4.rs:5-7 */
static const float E2M1[16] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f,
                               -0.0f, -0.5f, -1.0f, -1.5f, -2.0f, -3.0f, -4.0f, -6.0f};
/* src/q8.rs:22 */
static const int8_t E2M1_X2[16] = {0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12};

static inline float f32_from_bits(uint32_t b) {
    float f;
    memcpy(&f, &b, 4);
    return f;
}

/* src/mxfp4.rs:10-16: exact 2^e; e < -126 is the subnormal powi fallback */
ORC_API float orc_exp2_i(int e) {
    if (e < -126) return ldexpf(1.0f, e);
    return f32_from_bits((uint32_t)(e + 127) << 23);
}

/* src/mxfp4.rs:340-346 */
ORC_API float orc_scale_from_byte(uint8_t sb) {
    return sb == 0 ? f32_from_bits(0x00400000u) : f32_from_bits((uint32_t)sb << 23);
}

/* src/mxfp4.rs:19-31 (= src/dequant.rs:43-45 dequant_fp4) */
ORC_API void orc_mxfp4_dequant(const uint8_t *packed, const uint8_t *scales, size_t rows, size_t cols, float *out) {
    for (size_t r = 0; r < rows; r++) {
        const uint8_t *prow = packed + r * cols / 2;
        const uint8_t *srow = scales + r * cols / 32;
        for (size_t c = 0; c < cols; c++) {
            uint8_t byte = prow[c / 2];
            uint8_t nib = (c % 2 == 0) ? (byte & 0x0F) : (byte >> 4);
            out[r * cols + c] = E2M1[nib] * orc_exp2_i((int)srow[c / 32] - 127);
        }
    }
}

static const float MX_BOUNDS[7] = {0.25f, 0.75f, 1.25f, 1.75f, 2.5f, 3.5f, 5.0f};

static inline float clampf(float v, float lo, float hi) {
    /* Rust f32::clamp: NaN stays NaN; callers never pass NaN */
    return v < lo ? lo : (v > hi ? hi : v);
}

/* src/mxfp4.rs:51-69 */
static double group_sse(const float *group, int e) {
    float inv = 1.0f / orc_exp2_i(e);
    double s = (double)orc_exp2_i(e);
    double sse = 0.0;
    for (int i = 0; i < 32; i++) {
        float v = group[i];
        float q = clampf(v * inv, -6.0f, 6.0f);
        float mag = fabsf(q);
        int idx = 0;
        while (idx < 7 && mag >= MX_BOUNDS[idx]) idx++;
        double lvl = (double)E2M1[idx];
        double dq = (signbit(q) ? -lvl : lvl) * s;
        double d = (double)v - dq;
        sse += d * d;
    }
    return sse;
}

/* src/mxfp4.rs:77-92 */
ORC_API int orc_search_mx_scale(const float *group, int e) {
    int best = e;
    double best_sse = group_sse(group, e);
    int cands[2] = {e - 1, e + 1};
    for (int i = 0; i < 2; i++) {
        int cand = cands[i];
        if (cand < -127 || cand > 128) continue;
        double sse = group_sse(group, cand);
        if (sse < best_sse) {
            best_sse = sse;
            best = cand;
        }
    }
    return best;
}

/* src/mxfp4.rs:94-138; search = 1 is mxfp4::quantize, 0 is quantize_naive.
 * packed and scales must be zero-initialised by the caller (the reference
 * allocates zeroed vectors and ORs nibbles in). */
ORC_API void orc_mxfp4_quantize(const float *w, size_t rows, size_t cols, int search, uint8_t *packed, uint8_t *scales) {
    memset(packed, 0, rows * cols / 2);
    memset(scales, 0, rows * cols / 32);
    for (size_t r = 0; r < rows; r++) {
        const float *row = w + r * cols;
        for (size_t g = 0; g < cols / 32; g++) {
            const float *group = row + g * 32;
            float maxabs = 0.0f;
            for (int i = 0; i < 32; i++) maxabs = fmaxf(maxabs, fabsf(group[i]));
            int e;
            if (maxabs == 0.0f) {
                e = -127;
            } else {
                e = (int)ceilf(log2f(maxabs / 6.0f));
            }
            if (e < -127) e = -127;
            if (e > 128) e = 128;
            if (search && maxabs != 0.0f) e = orc_search_mx_scale(group, e);
            int sb = e + 127;
            if (sb < 0) sb = 0;
            if (sb > 255) sb = 255;
            scales[r * cols / 32 + g] = (uint8_t)sb;
            float inv = 1.0f / orc_exp2_i(e);
            for (int j = 0; j < 32; j++) {
                float q = clampf(group[j] * inv, -6.0f, 6.0f);
                float mag = fabsf(q);
                int idx = 0;
                while (idx < 7 && mag >= MX_BOUNDS[idx]) idx++;
                if (signbit(q)) idx += 8;
                size_t c = g * 32 + j;
                uint8_t *byte = &packed[r * cols / 2 + c / 2];
                if (c % 2 == 0)
                    *byte |= (uint8_t)idx;
                else
                    *byte |= (uint8_t)(idx << 4);
            }
        }
    }
}

/* ---- MXFP4SQ: quadratic scale byte against a per-tensor smax (src/mxfp4.rs:140-240) */

/* src/mxfp4.rs:154-158 */
ORC_API float orc_scale_sq(uint8_t q, float smax) {
    float t = ((float)q + 1.0f) * (1.0f / 256.0f);
    return t * t * smax;
}

/* src/mxfp4.rs:160-214: returns smax; packed [rows][cols/2], scales [rows][cols/32] */
ORC_API float orc_mxfp4sq_quantize(const float *w, size_t rows, size_t cols, uint8_t *packed, uint8_t *scales) {
    size_t ng = rows * cols / 32;
    float *ideal = (float *)malloc(sizeof(float) * (ng ? ng : 1));
    float smax = 0.0f;
    for (size_t gi = 0; gi < ng; gi++) {
        float maxabs = 0.0f;
        for (int i = 0; i < 32; i++) maxabs = fmaxf(maxabs, fabsf(w[gi * 32 + i]));
        ideal[gi] = maxabs / 6.0f;
        smax = fmaxf(smax, ideal[gi]);
    }
    memset(packed, 0, rows * cols / 2);
    for (size_t gi = 0; gi < ng; gi++) {
        int q = 0;
        if (!(smax == 0.0f || ideal[gi] == 0.0f)) {
            q = (int)ceilf(256.0f * sqrtf(ideal[gi] / smax)) - 1;
            if (q < 0) q = 0;
            if (q > 255) q = 255;
        }
        scales[gi] = (uint8_t)q;
        float inv = 1.0f / orc_scale_sq((uint8_t)q, smax);
        for (int j = 0; j < 32; j++) {
            float qv = clampf(w[gi * 32 + j] * inv, -6.0f, 6.0f);
            float mag = fabsf(qv);
            int idx = 0;
            while (idx < 7 && mag >= MX_BOUNDS[idx]) idx++;
            if (signbit(qv)) idx += 8;
            size_t c = gi * 32 + j; /* rows are whole groups: the element's index in the matrix */
            uint8_t *byte = &packed[c / 2];
            if (c % 2 == 0)
                *byte |= (uint8_t)idx;
            else
                *byte |= (uint8_t)(idx << 4);
        }
    }
    free(ideal);
    return smax;
}

/* src/mxfp4.rs:216-229 */
ORC_API void orc_mxfp4sq_dequant(const uint8_t *packed, const uint8_t *scales, float smax, size_t rows, size_t cols, float *out) {
    for (size_t r = 0; r < rows; r++)
        for (size_t c = 0; c < cols; c++) {
            uint8_t byte = packed[r * cols / 2 + c / 2];
            uint8_t nib = (c % 2 == 0) ? (byte & 0x0F) : (byte >> 4);
            out[r * cols + c] = E2M1[nib] * orc_scale_sq(scales[r * cols / 32 + c / 32], smax);
        }
}

/* src/dequant.rs:12-23 */
ORC_API float orc_e4m3_to_f32(uint8_t b) {
    float sign = (b & 0x80) ? -1.0f : 1.0f;
    int e = (b >> 3) & 0x0F;
    float m = (float)(b & 0x07);
    if (e == 15 && (b & 0x07) == 7) return NAN;
    if (e == 0) return sign * (m / 8.0f) * ldexpf(1.0f, -6);
    return sign * (1.0f + m / 8.0f) * orc_exp2_i(e - 7);
}

/* src/dequant.rs:77-89 */
static int rne_i(float x) {
    float f = floorf(x);
    float frac = x - f;
    int i = (int)f;
    if (frac > 0.5f) return i + 1;
    if (frac < 0.5f) return i;
    return (i % 2 == 0) ? i : i + 1;
}

/* src/dequant.rs:92-120 */
ORC_API uint8_t orc_f32_to_e4m3(float v) {
    if (isnan(v)) return 0x7F;
    uint8_t sign = signbit(v) ? 0x80 : 0;
    float a = fminf(fabsf(v), 448.0f);
    if (a < ldexpf(1.0f, -10)) return sign;
    if (a < ldexpf(1.0f, -6)) {
        int m = rne_i(a / ldexpf(1.0f, -6) * 8.0f);
        return m >= 8 ? (uint8_t)(sign | 0x08) : (uint8_t)(sign | (uint8_t)m);
    }
    int e = 1;
    while (e < 15 && a >= ldexpf(1.0f, e - 6)) e++;
    float base = ldexpf(1.0f, e - 7);
    int m = rne_i((a / base - 1.0f) * 8.0f);
    int e2 = e, m2 = m;
    if (m == 8) {
        e2 = e + 1;
        m2 = 0;
    }
    if (e2 >= 15 && m2 > 6) return (uint8_t)(sign | 0x7E);
    return (uint8_t)(sign | (uint8_t)(e2 << 3) | (uint8_t)m2);
}

/* src/dequant.rs:27-39 */
ORC_API void orc_dequant_fp8(const uint8_t *w, const uint8_t *scales, size_t rows, size_t cols, float *out) {
    size_t scols = (cols + 127) / 128;
    for (size_t r = 0; r < rows; r++)
        for (size_t c = 0; c < cols; c++) {
            float s = orc_exp2_i((int)scales[(r / 128) * scols + c / 128] - 127);
            out[r * cols + c] = orc_e4m3_to_f32(w[r * cols + c]) * s;
        }
}

/* src/dequant.rs:50-74; rows and cols must be multiples of 128 */
ORC_API void orc_quantize_fp8(const float *w, size_t rows, size_t cols, uint8_t *qw, uint8_t *scales) {
    for (size_t br = 0; br < rows / 128; br++)
        for (size_t bc = 0; bc < cols / 128; bc++) {
            float maxabs = 0.0f;
            for (size_t r = br * 128; r < (br + 1) * 128; r++)
                for (size_t c = bc * 128; c < (bc + 1) * 128; c++) maxabs = fmaxf(maxabs, fabsf(w[r * cols + c]));
            int e = (maxabs == 0.0f) ? -127 : (int)ceilf(log2f(maxabs / 448.0f));
            if (e < -127) e = -127;
            if (e > 8) e = 8;
            scales[br * (cols / 128) + bc] = (uint8_t)(e + 127);
            float inv = 1.0f / orc_exp2_i(e);
            for (size_t r = br * 128; r < (br + 1) * 128; r++)
                for (size_t c = bc * 128; c < (bc + 1) * 128; c++) qw[r * cols + c] = orc_f32_to_e4m3(w[r * cols + c] * inv);
        }
}

/* src/deepseek.rs:312-322: act_quant round trip, pow2 scale per `block`.
 * Also returns the scale exponent bytes (e + 127) when exps != NULL: that is
 * the MXFP8 (e4m3 + e8m0) activation encoding the block-scaled GEMM consumes. */
/* The same round trip with the upper clamp of the scale exponent as a parameter.  The reference clamps at 8
 * (its rule for DeepSeek's activations); with emax = 127 the whole e8m0 range is used and no block saturates,
 * which is how the prefill expert section of this build encodes its MXFP8 activations (a SwiGLU value of the
 * benchmark's random experts reaches 4e5 > 448 * 2^8). */
ORC_API void orc_fp8_roundtrip_emax(float *x, size_t n, size_t block, int emax, uint8_t *codes, uint8_t *exps) {
    for (size_t b0 = 0; b0 < n; b0 += block) {
        size_t len = (b0 + block <= n) ? block : n - b0;
        float amax = 0.0f;
        for (size_t i = 0; i < len; i++) amax = fmaxf(amax, fabsf(x[b0 + i]));
        amax = fmaxf(amax, 1e-4f);
        int e = (int)ceilf(log2f(amax / 448.0f));
        if (e < -127) e = -127;
        if (e > emax) e = emax;
        float s = orc_exp2_i(e);
        if (exps) exps[b0 / block] = (uint8_t)(e + 127);
        for (size_t i = 0; i < len; i++) {
            uint8_t c = orc_f32_to_e4m3(clampf(x[b0 + i] / s, -448.0f, 448.0f));
            if (codes) codes[b0 + i] = c;
            x[b0 + i] = orc_e4m3_to_f32(c) * s;
        }
    }
}

ORC_API void orc_fp8_roundtrip(float *x, size_t n, size_t block, uint8_t *codes, uint8_t *exps) {
    orc_fp8_roundtrip_emax(x, n, block, 8, codes, exps);
}

/* ------------------------------------------------------- q8 activations */

/* src/q8.rs:49-69.  q: n int8, scales: n/32 f32.  n % 32 == 0. */
ORC_API void orc_quantize_q8(const float *x, size_t n, int8_t *q, float *scales) {
    size_t nb = n / 32;
    memset(q, 0, n);
    for (size_t g = 0; g < nb; g++) {
        const float *b = x + g * 32;
        float max = 0.0f;
        for (int j = 0; j < 32; j++) max = fmaxf(max, fabsf(b[j]));
        float dx = max / 127.0f;
        scales[g] = dx;
        if (dx == 0.0f) continue;
        for (int j = 0; j < 32; j++) {
            float v = roundf(b[j] / dx); /* Rust f32::round: half away from zero */
            v = clampf(v, -127.0f, 127.0f);
            q[g * 32 + j] = v != v ? 0 : (int8_t)v; /* Rust's `as i8` of NaN (a NaN value, or inf / inf) is 0 */
        }
    }
}

/* src/q8.rs:194-202 */
static int32_t dot_block_scalar(const uint8_t *packed16, const int8_t *x32) {
    int32_t s = 0;
    for (int j = 0; j < 16; j++) {
        uint8_t b = packed16[j];
        s += (int32_t)E2M1_X2[b & 0x0F] * (int32_t)x32[2 * j];
        s += (int32_t)E2M1_X2[b >> 4] * (int32_t)x32[2 * j + 1];
    }
    return s;
}

/* src/q8.rs:119-125 */
static int32_t dot_i8_scalar(const int8_t *w32, const int8_t *x32) {
    int32_t s = 0;
    for (int j = 0; j < 32; j++) s += (int32_t)w32[j] * (int32_t)x32[j];
    return s;
}

#if defined(__x86_64__)
/* src/q8.rs:153-168 */
__attribute__((target("avx2"))) static int32_t dot_i8_avx2(const int8_t *w32, const int8_t *x32) {
    __m256i w = _mm256_loadu_si256((const __m256i *)w32);
    __m256i x = _mm256_loadu_si256((const __m256i *)x32);
    __m256i ax = _mm256_sign_epi8(x, x);
    __m256i aw = _mm256_sign_epi8(w, x);
    __m256i pairs = _mm256_maddubs_epi16(ax, aw);
    __m256i quads = _mm256_madd_epi16(pairs, _mm256_set1_epi16(1));
    __m128i s128 = _mm_add_epi32(_mm256_castsi256_si128(quads), _mm256_extracti128_si256(quads, 1));
    __m128i s64 = _mm_add_epi32(s128, _mm_shuffle_epi32(s128, 0x4E));
    __m128i s32 = _mm_add_epi32(s64, _mm_shuffle_epi32(s64, 0xB1));
    return _mm_cvtsi128_si32(s32);
}

/* src/q8.rs:238-263 */
__attribute__((target("avx2"))) static int32_t dot_block_avx2(const uint8_t *packed16, const int8_t *x32) {
    __m256i lut = _mm256_broadcastsi128_si256(_mm_loadu_si128((const __m128i *)E2M1_X2));
    __m256i b = _mm256_broadcastsi128_si256(_mm_loadu_si128((const __m128i *)packed16));
    __m256i msk = _mm256_set1_epi8(0x0F);
    __m256i andlo = _mm256_and_si256(b, msk);
    __m256i andhi = _mm256_and_si256(_mm256_srli_epi16(b, 4), msk);
    __m256i lo = _mm256_shuffle_epi8(lut, andlo);
    __m256i hi = _mm256_shuffle_epi8(lut, andhi);
    __m256i ilo = _mm256_unpacklo_epi8(lo, hi);
    __m256i ihi = _mm256_unpackhi_epi8(lo, hi);
    __m256i w = _mm256_permute2x128_si256(ilo, ihi, 0x20);
    __m256i x = _mm256_loadu_si256((const __m256i *)x32);
    __m256i ax = _mm256_sign_epi8(x, x);
    __m256i aw = _mm256_sign_epi8(w, x);
    __m256i pairs = _mm256_maddubs_epi16(ax, aw);
    __m256i quads = _mm256_madd_epi16(pairs, _mm256_set1_epi16(1));
    __m128i s128 = _mm_add_epi32(_mm256_castsi256_si128(quads), _mm256_extracti128_si256(quads, 1));
    __m128i s64 = _mm_add_epi32(s128, _mm_shuffle_epi32(s128, 0x4E));
    __m128i s32 = _mm_add_epi32(s64, _mm_shuffle_epi32(s64, 0xB1));
    return _mm_cvtsi128_si32(s32);
}
#endif

/* 0 = follow the CPU (AVX2 when present, as the reference does), 1 = force scalar */
static int g_force_scalar = 0;
ORC_API void orc_force_scalar(int on) { g_force_scalar = on; }

static int have_avx2(void) {
#if defined(__x86_64__)
    static int cached = -1;
    if (cached < 0) cached = __builtin_cpu_supports("avx2") ? 1 : 0;
    return cached && !g_force_scalar;
#else
    return 0;
#endif
}

/* src/q8.rs:177-191 */
ORC_API int32_t orc_block_dot(const uint8_t *packed16, const int8_t *x32) {
#if defined(__x86_64__)
    if (have_avx2()) return dot_block_avx2(packed16, x32);
#endif
    return dot_block_scalar(packed16, x32);
}

/* src/q8.rs:102-116 */
ORC_API int32_t orc_block_dot_i8(const int8_t *w32, const int8_t *x32) {
#if defined(__x86_64__)
    if (have_avx2()) return dot_i8_avx2(w32, x32);
#endif
    return dot_i8_scalar(w32, x32);
}

/* ---------------------------------------------------- f32 dot (8 lanes) */

/* src/model.rs:63-82: 8 accumulators, mul then add, ((p01+p23)+p45)+p67, tail sequential */
ORC_API float orc_dot(const float *a, const float *b, size_t n) {
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    size_t i = 0;
    for (; i + 8 <= n; i += 8)
        for (int j = 0; j < 8; j++) acc[j] += a[i + j] * b[i + j];
    float s = (acc[0] + acc[1]) + (acc[2] + acc[3]) + (acc[4] + acc[5]) + (acc[6] + acc[7]);
    for (; i < n; i++) s += a[i] * b[i];
    return s;
}

/* src/model.rs:214-222 (single job; the pool split does not change any row) */
ORC_API void orc_matvec_f32(const float *w, size_t rows, size_t cols, const float *x, float *out) {
    for (size_t r = 0; r < rows; r++) out[r] = orc_dot(w + r * cols, x, cols);
}

/* src/model.rs:599-605 and src/deepseek.rs:241-248: ss = dot(x, x) / n; inv = 1 / sqrt(ss + eps);
 * out[i] = x[i] * inv * w[i] (two multiplications, left to right) */
ORC_API void orc_rmsnorm(const float *x, size_t n, const float *w, float eps, float *out) {
    float ss = orc_dot(x, x, n) / (float)n;
    float inv = 1.0f / sqrtf(ss + eps);
    for (size_t i = 0; i < n; i++) out[i] = x[i] * inv * w[i];
}

/* ------------------------------------------------ VQ1 matvec / LUT GEMV */

/* src/quant.rs:313-331 (matvec_vq_gather): codebook [256][16] f32, one index byte per vector of 16 consecutive
 * row-major weights; per row the 16-wide dots in order, each accumulated from 0 in ascending j, summed in ascending
 * vector order */
ORC_API void orc_vq1_matvec_gather(const float *codebook, const uint8_t *indices, size_t rows, size_t cols, const float *x, float *out) {
    const size_t vpr = cols / 16;
    for (size_t r = 0; r < rows; r++) {
        const uint8_t *irow = indices + r * vpr;
        float sum = 0.0f;
        for (size_t v = 0; v < vpr; v++) {
            const float *cb = codebook + (size_t)irow[v] * 16, *xs = x + v * 16;
            float s = 0.0f;
            for (int j = 0; j < 16; j++) s += cb[j] * xs[j];
            sum += s;
        }
        out[r] = sum;
    }
}

/* src/lutgemv.rs:208-240 (matvec_vq_lut) with build_vq_lut_scalar (:175-185) and sweep (:67-98): tables of 256
 * entry-activation dots per 16-wide group, built and swept 16 groups at a time, rows inner; additions only in the sweep */
ORC_API void orc_vq1_matvec_lut(const float *codebook, const uint8_t *indices, size_t rows, size_t cols, const float *x, float *out) {
    enum { TILE = 16 };
    const size_t vpr = cols / 16;
    float *lut = (float *)malloc(sizeof(float) * TILE * 256);
    for (size_t r = 0; r < rows; r++) out[r] = 0.0f;
    for (size_t g0 = 0; g0 < vpr; g0 += TILE) {
        const size_t groups = vpr - g0 < TILE ? vpr - g0 : TILE;
        for (size_t g = 0; g < groups; g++) {
            const float *xs = x + (g0 + g) * 16;
            for (int k = 0; k < 256; k++) {
                const float *cb = codebook + (size_t)k * 16;
                float s = 0.0f;
                for (int j = 0; j < 16; j++) s += cb[j] * xs[j];
                lut[g * 256 + k] = s;
            }
        }
        for (size_t r = 0; r < rows; r++) {
            float a = out[r];
            const uint8_t *ir = indices + r * vpr;
            for (size_t g = 0; g < groups; g++) a += lut[g * 256 + ir[g0 + g]];
            out[r] = a;
        }
    }
    free(lut);
}

/* src/quant.rs:353-376 (matvec_vq_nt): m inputs transposed in xt [cols][m], blocks of 8 positions, rows inner; every
 * product goes straight into its position's sum, in (vector, j) order; out [m][rows] */
ORC_API void orc_vq1_matvec_nt(const float *codebook, const uint8_t *indices, size_t rows, size_t cols, const float *xt, size_t m, float *out) {
    const size_t vpr = cols / 16;
    for (size_t t0 = 0; t0 < m; t0 += 8) {
        for (size_t r = 0; r < rows; r++) {
            const uint8_t *irow = indices + r * vpr;
            float sum[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            for (size_t v = 0; v < vpr; v++) {
                const float *cb = codebook + (size_t)irow[v] * 16;
                for (int j = 0; j < 16; j++) {
                    const float wv = cb[j];
                    const float *xc = xt + (v * 16 + j) * m + t0;
                    for (int p = 0; p < 8; p++) sum[p] += wv * xc[p];
                }
            }
            for (int p = 0; p < 8; p++) out[(t0 + p) * rows + r] = sum[p];
        }
    }
}

/* ------------------------------------------------------- mxfp4 matvecs */

/* src/mxfp4.rs:409-418: one row of the q8-integer path */
static float q8_row(const uint8_t *prow, const uint8_t *srow, size_t cols, const int8_t *xq, const float *xs) {
    float sum = 0.0f;
    for (size_t g = 0; g < cols / 32; g++) {
        int32_t idot = orc_block_dot(prow + g * 16, xq + g * 32);
        sum += (float)idot * (orc_exp2_i((int)srow[g] - 128) * xs[g]);
    }
    return sum;
}

/* src/mxfp4.rs:405-443 (row chunks over threads give the same rows) */
ORC_API void orc_matvec_packed_q8(const uint8_t *packed, const uint8_t *scales, size_t rows, size_t cols, const int8_t *xq,
                                  const float *xs, float *out) {
    for (size_t r = 0; r < rows; r++) out[r] = q8_row(packed + r * cols / 2, scales + r * cols / 32, cols, xq, xs);
}

/* src/mxfp4.rs:494-505: one row of the exact f32 path */
static float f32_row(const uint8_t *prow, const uint8_t *srow, size_t cols, const float *x) {
    float sum = 0.0f;
    for (size_t g = 0; g < cols / 32; g++) {
        float gsum = 0.0f;
        for (int j = 0; j < 32; j++) {
            size_t c = g * 32 + j;
            uint8_t byte = prow[c / 2];
            uint8_t nib = (c % 2 == 0) ? (byte & 0x0F) : (byte >> 4);
            gsum += E2M1[nib] * x[c];
        }
        sum += gsum * orc_exp2_i((int)srow[g] - 127);
    }
    return sum;
}

/* src/mxfp4.rs:458-539.  mode 1 = q8 integer path (the reference default),
 * mode 0 = exact f32 path (MICROKIMI_NO_Q8=1 / force_q8(0)). */
ORC_API void orc_matvec_packed(const uint8_t *packed, const uint8_t *scales, size_t rows, size_t cols, const float *x, float *out,
                               int mode) {
    if (mode == 1) {
        int8_t *xq = (int8_t *)malloc(cols);
        float *xs = (float *)malloc(sizeof(float) * (cols / 32));
        orc_quantize_q8(x, cols, xq, xs);
        orc_matvec_packed_q8(packed, scales, rows, cols, xq, xs, out);
        free(xq);
        free(xs);
        return;
    }
    for (size_t r = 0; r < rows; r++) out[r] = f32_row(packed + r * cols / 2, scales + r * cols / 32, cols, x);
}

/* src/mxfp4.rs:357-393: emulation of a one-group-per-row GPU kernel's order */
static float tree_sum(float *v, size_t n) {
    while (n > 1) {
        for (size_t i = 0; i < n / 2; i++) v[i] += v[n / 2 + i];
        n /= 2;
    }
    return v[0];
}
ORC_API void orc_matvec_packed_shader_emul(const uint8_t *packed, const uint8_t *scales, size_t rows, size_t cols, const float *x,
                                           float *out, size_t lanes) {
    float *part = (float *)malloc(sizeof(float) * lanes);
    float *sg = (float *)malloc(sizeof(float) * (lanes / 32));
    for (size_t r = 0; r < rows; r++) {
        const uint8_t *prow = packed + r * cols / 2;
        const uint8_t *srow = scales + r * cols / 32;
        for (size_t lane = 0; lane < lanes; lane++) {
            float acc = 0.0f;
            for (size_t c = lane; c < cols; c += lanes) {
                uint8_t byte = prow[c / 2];
                uint8_t nib = (c % 2 == 0) ? (byte & 0x0F) : (byte >> 4);
                acc += E2M1[nib] * orc_scale_from_byte(srow[c / 32]) * x[c];
            }
            part[lane] = acc;
        }
        for (size_t s = 0; s < lanes / 32; s++) sg[s] = tree_sum(part + s * 32, 32);
        out[r] = tree_sum(sg, lanes / 32);
    }
    free(part);
    free(sg);
}

/* src/model.rs:2412-2447.  xt = inputs transposed [cols][m], m % 8 == 0;
 * out position-major [m][rows]. */
ORC_API void orc_matvec_packed_nt(const uint8_t *packed, const uint8_t *scales, size_t rows, size_t cols, const float *xt, size_t m,
                                  float *out) {
    float *wrow = (float *)malloc(sizeof(float) * cols);
    for (size_t r = 0; r < rows; r++) {
        const uint8_t *prow = packed + r * cols / 2;
        const uint8_t *srow = scales + r * cols / 32;
        for (size_t c = 0; c < cols; c++) {
            uint8_t byte = prow[c / 2];
            uint8_t nib = (c % 2 == 0) ? (byte & 0x0F) : (byte >> 4);
            wrow[c] = E2M1[nib];
        }
        for (size_t t0 = 0; t0 < m; t0 += 8) {
            float sum[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            for (size_t g = 0; g < cols / 32; g++) {
                float gsum[8] = {0, 0, 0, 0, 0, 0, 0, 0};
                for (int j = 0; j < 32; j++) {
                    size_t c = g * 32 + j;
                    float wv = wrow[c];
                    const float *xc = xt + c * m + t0;
                    for (int p = 0; p < 8; p++) gsum[p] += wv * xc[p];
                }
                float sc = orc_exp2_i((int)srow[g] - 127);
                for (int p = 0; p < 8; p++) sum[p] += gsum[p] * sc;
            }
            for (int p = 0; p < 8; p++) out[(t0 + p) * rows + r] = sum[p];
        }
    }
    free(wrow);
}

/* ------------------------------------------------------------- q8 head */

/* ------------------------------------------- summation order of the device kernels
 * What matvec_packed_shader_emul (src/mxfp4.rs:348-393) is for the reference's Metal kernel: the order in which the
 * device kernels of this library add a row's terms, restated on the CPU.  The terms themselves are the reference's
 * (exact integer block dots times the f32 scale product); only the association of the f32 sum differs.  With it the gap
 * between the device's and the reference's order is bounded without a device, and on a device the kernels must give
 * these values bit for bit. */

/* The wave-wide sum of the kernels: four exchange steps inside each row of 16 lanes (lane ^ 1, lane ^ 2, mirror of the
 * half row, mirror of the row), then (v[0] + v[16]) + (v[32] + v[48]). */
static float wave_sum_order(const float *in) {
    float v[64], n[64];
    memcpy(v, in, sizeof(v));
    for (int l = 0; l < 64; l++) n[l] = v[l] + v[l ^ 1];
    memcpy(v, n, sizeof(v));
    for (int l = 0; l < 64; l++) n[l] = v[l] + v[l ^ 2];
    memcpy(v, n, sizeof(v));
    for (int l = 0; l < 64; l++) n[l] = v[l] + v[(l & ~7) + 7 - (l & 7)];
    memcpy(v, n, sizeof(v));
    for (int l = 0; l < 64; l++) n[l] = v[l] + v[(l & ~15) + 15 - (l & 15)];
    return (n[0] + n[16]) + (n[32] + n[48]);
}

static size_t gcd_sz(size_t a, size_t b) { return b == 0 ? a : gcd_sz(b, a % b); }

/* matvec_packed_q8 in the order of the single-row MXFP4 GEMV kernel: a tile is lcm(nb, 64) blocks = RT whole rows; lane l
 * takes the blocks l, l + 64, ... of the tile in turn and adds a block's term to the sum of the row the block belongs
 * to (zero to the other row's); the lanes' sums of a row then meet in the wave-wide sum.  nb = cols / 32. */
ORC_API void orc_matvec_packed_q8_device_order(const uint8_t *packed, const uint8_t *scales, size_t rows, size_t cols, const int8_t *xq,
                                               const float *xs, float *out) {
    size_t nb = cols / 32, tile = nb / gcd_sz(nb, 64) * 64, T = tile / 64, RT = tile / nb;
    for (size_t row = 0; row < rows; row++) {
        size_t r = row % RT;
        float lanes[64];
        for (size_t l = 0; l < 64; l++) {
            float acc = 0.0f;
            for (size_t t = 0; t < T; t++) {
                size_t b = t * 64 + l;
                float term = 0.0f;
                if (b / nb == r) {
                    size_t g = b % nb;
                    int32_t idot = orc_block_dot(packed + row * cols / 2 + g * 16, xq + g * 32);
                    term = (float)idot * (orc_exp2_i((int)scales[row * nb + g] - 128) * xs[g]);
                }
                acc += term;
            }
            lanes[l] = acc;
        }
        out[row] = wave_sum_order(lanes);
    }
}

/* Q8Head::matvec in the order of the batch-1 q8 GEMV kernel: lane l takes the half blocks (16 values) l, l + 64, ... of
 * the row; a half block's term is (ws * xs) * (its integer dot); then the wave-wide sum.  cols a multiple of 1024. */
ORC_API void orc_q8head_matvec_device_order(const int8_t *q, const float *ws, size_t rows, size_t cols, const int8_t *xq, const float *xs,
                                            float *out) {
    size_t nb = cols / 32, T = nb * 2 / 64;
    for (size_t row = 0; row < rows; row++) {
        float lanes[64];
        for (size_t l = 0; l < 64; l++) {
            float acc = 0.0f;
            for (size_t t = 0; t < T; t++) {
                size_t hb = t * 64 + l;
                int32_t d = 0;
                for (int i = 0; i < 16; i++) d += (int32_t)q[row * cols + hb * 16 + i] * (int32_t)xq[hb * 16 + i];
                acc += (ws[row * nb + hb / 2] * xs[hb / 2]) * (float)d;
            }
            lanes[l] = acc;
        }
        out[row] = wave_sum_order(lanes);
    }
}

/* src/model.rs:274-286: row-wise q8_0 copy of an f32 matrix */
ORC_API void orc_q8head_from_f32(const float *w, size_t rows, size_t cols, int8_t *q, float *scales) {
    size_t nb = cols / 32;
    for (size_t r = 0; r < rows; r++) orc_quantize_q8(w + r * cols, cols, q + r * cols, scales + r * nb);
}

/* src/model.rs:323-330 / 337-347: rows r0..r1 against a q8 activation */
static void q8head_rows(const int8_t *q, const float *ws, size_t cols, const int8_t *xq, const float *xs, float *out, size_t r0,
                        size_t r1) {
    size_t nb = cols / 32;
    for (size_t r = r0; r < r1; r++) {
        float acc = 0.0f;
        for (size_t g = 0; g < nb; g++) {
            int32_t idot = orc_block_dot_i8(q + r * cols + g * 32, xq + g * 32);
            acc += ws[r * nb + g] * xs[g] * (float)idot;
        }
        out[r] = acc;
    }
}

typedef struct {
    const int8_t *q;
    const float *ws;
    size_t cols;
    const int8_t *xq;
    const float *xs;
    float *out;
    size_t r0, r1;
} head_job_t;

static void *head_job(void *p) {
    head_job_t *j = (head_job_t *)p;
    q8head_rows(j->q, j->ws, j->cols, j->xq, j->xs, j->out, j->r0, j->r1);
    return NULL;
}

/* src/model.rs:290-335: quantize x, split rows into
 * njobs = clamp(rows*cols/60000, 1, workers) chunks, one thread per chunk. */
ORC_API void orc_q8head_matvec(const int8_t *q, const float *ws, size_t rows, size_t cols, const float *x, float *out, size_t workers) {
    int8_t *xq = (int8_t *)malloc(cols);
    float *xs = (float *)malloc(sizeof(float) * (cols / 32));
    orc_quantize_q8(x, cols, xq, xs);
    size_t njobs = rows * cols / 60000;
    if (njobs < 1) njobs = 1;
    if (njobs > workers) njobs = workers;
    if (njobs > rows) njobs = rows;
    if (njobs <= 1) {
        q8head_rows(q, ws, cols, xq, xs, out, 0, rows);
    } else {
        size_t chunk = (rows + njobs - 1) / njobs;
        pthread_t *th = (pthread_t *)malloc(sizeof(pthread_t) * njobs);
        head_job_t *jobs = (head_job_t *)malloc(sizeof(head_job_t) * njobs);
        size_t started = 0;
        for (size_t j = 0; j < njobs; j++) {
            size_t r0 = j * chunk, r1 = (j + 1) * chunk < rows ? (j + 1) * chunk : rows;
            if (r0 >= r1) break;
            head_job_t jb = {q, ws, cols, xq, xs, out, r0, r1};
            jobs[j] = jb;
            pthread_create(&th[j], NULL, head_job, &jobs[j]);
            started++;
        }
        for (size_t j = 0; j < started; j++) pthread_join(th[j], NULL);
        free(th);
        free(jobs);
    }
    free(xq);
    free(xs);
}

/* src/model.rs:3271-3291 with k = 1: the greedy token.  Ties resolve to the
 * lowest index (strict '>' insertion, stable sort). */
ORC_API size_t orc_argmax(const float *logits, size_t n) {
    size_t best = 0;
    for (size_t i = 1; i < n; i++)
        if (logits[i] > logits[best]) best = i;
    return best;
}

/* ------------------------------------------------------------ MLA cache */

typedef struct {
    size_t nh, nope, rope, vd;
} orc_mla_cfg;

/* src/model.rs:1540-1554 */
ORC_API void orc_hadamard64(float *x) {
    for (size_t h = 1; h < 64; h *= 2)
        for (size_t i = 0; i < 64; i += 2 * h)
            for (size_t j = i; j < i + h; j++) {
                float a = x[j], b = x[j + h];
                x[j] = a + b;
                x[j + h] = a - b;
            }
}

/* src/model.rs:1583-1618 (q8 mode): quantize one position.  Outputs are the
 * slices of that position: kq [nh*nope], ks [nh*nope/32], kr [rope],
 * vq [nh*vd], vs [nh*vd/32].  k_row is [nh][nope+rope], v_row is [nh][vd]. */
ORC_API void orc_mla_cache_push(const orc_mla_cfg *cfg, int had_on, const float *k_row, const float *v_row, int8_t *kq, float *ks,
                                float *kr, int8_t *vq, float *vs) {
    size_t nh = cfg->nh, nope = cfg->nope, rope = cfg->rope, vd = cfg->vd;
    int had = had_on && nope % 64 == 0 && vd % 64 == 0;
    size_t qh = nope + rope;
    memcpy(kr, k_row + nope, sizeof(float) * rope);
    size_t smax = nope > vd ? nope : vd;
    float *scratch = (float *)malloc(sizeof(float) * smax);
    for (size_t h = 0; h < nh; h++) {
        memcpy(scratch, k_row + h * qh, sizeof(float) * nope);
        if (had)
            for (size_t b = 0; b < nope; b += 64) orc_hadamard64(scratch + b);
        orc_quantize_q8(scratch, nope, kq + h * nope, ks + h * (nope / 32));
        memcpy(scratch, v_row + h * vd, sizeof(float) * vd);
        if (had)
            for (size_t b = 0; b < vd; b += 64) orc_hadamard64(scratch + b);
        orc_quantize_q8(scratch, vd, vq + h * vd, vs + h * (vd / 32));
    }
    free(scratch);
}

/* src/model.rs:1623-1676: dequantize n positions back to f32 rows */
ORC_API void orc_mla_cache_to_f32(const orc_mla_cfg *cfg, int had_on, size_t n, const int8_t *kq, const float *ks, const float *kr,
                                  const int8_t *vq, const float *vs, float *k, float *v) {
    size_t nh = cfg->nh, nope = cfg->nope, rope = cfg->rope, vd = cfg->vd;
    int had = had_on && nope % 64 == 0 && vd % 64 == 0;
    size_t qh = nope + rope, nb_n = nope / 32, nb_v = vd / 32;
    for (size_t j = 0; j < n; j++)
        for (size_t h = 0; h < nh; h++) {
            size_t base_q = (j * nh + h) * nope, base_s = (j * nh + h) * nb_n;
            float *out = k + (j * nh + h) * qh;
            for (size_t g = 0; g < nb_n; g++) {
                float s = ks[base_s + g];
                for (int i = 0; i < 32; i++) out[g * 32 + i] = (float)kq[base_q + g * 32 + i] * s;
            }
            if (had)
                for (size_t b = 0; b < nope; b += 64) {
                    orc_hadamard64(out + b);
                    for (int i = 0; i < 64; i++) out[b + i] /= 64.0f;
                }
            memcpy(out + nope, kr + j * rope, sizeof(float) * rope);
            base_q = (j * nh + h) * vd;
            base_s = (j * nh + h) * nb_v;
            out = v + (j * nh + h) * vd;
            for (size_t g = 0; g < nb_v; g++) {
                float s = vs[base_s + g];
                for (int i = 0; i < 32; i++) out[g * 32 + i] = (float)vq[base_q + g * 32 + i] * s;
            }
            if (had)
                for (size_t b = 0; b < vd; b += 64) {
                    orc_hadamard64(out + b);
                    for (int i = 0; i < 64; i++) out[b + i] /= 64.0f;
                }
        }
}

#define FLASH_KV 64 /* src/model.rs:1348 */

/* src/model.rs:1353-1375 */
ORC_API void orc_mla_attn_ref(const orc_mla_cfg *cfg, const float *k, const float *v, const float *qh, size_t h, size_t pos,
                              float scale, float *oh) {
    size_t nh = cfg->nh, hd = cfg->nope + cfg->rope, vd = cfg->vd;
    float *scores = (float *)malloc(sizeof(float) * (pos + 1));
    for (size_t j = 0; j <= pos; j++) scores[j] = orc_dot(qh, k + (j * nh + h) * hd, hd) * scale;
    float m = -INFINITY;
    for (size_t j = 0; j <= pos; j++) m = fmaxf(m, scores[j]);
    float z = 0.0f;
    for (size_t j = 0; j <= pos; j++) {
        scores[j] = expf(scores[j] - m);
        z += scores[j];
    }
    for (size_t j = 0; j <= pos; j++) scores[j] /= z;
    for (size_t j = 0; j <= pos; j++) {
        const float *vj = v + (j * nh + h) * vd;
        float p = scores[j];
        for (size_t d = 0; d < vd; d++) oh[d] += p * vj[d];
    }
    free(scores);
}

/* src/model.rs:1385-1425 */
ORC_API void orc_mla_attn_flash(const orc_mla_cfg *cfg, const float *k, const float *v, const float *qh, size_t h, size_t pos,
                                float scale, float *oh) {
    size_t nh = cfg->nh, hd = cfg->nope + cfg->rope, vd = cfg->vd;
    float m = -INFINITY, l = 0.0f;
    float scores[FLASH_KV];
    size_t t = 0;
    while (t <= pos) {
        size_t end = t + FLASH_KV - 1 < pos ? t + FLASH_KV - 1 : pos;
        float tm = -INFINITY;
        for (size_t j = t, i = 0; j <= end; j++, i++) {
            float s = orc_dot(qh, k + (j * nh + h) * hd, hd) * scale;
            scores[i] = s;
            tm = fmaxf(tm, s);
        }
        float m_new = fmaxf(m, tm);
        float corr = expf(m - m_new);
        float tile_l = 0.0f;
        for (size_t i = 0; i < end - t + 1; i++) {
            scores[i] = expf(scores[i] - m_new);
            tile_l += scores[i];
        }
        for (size_t d = 0; d < vd; d++) oh[d] *= corr;
        l = l * corr + tile_l;
        for (size_t j = t, i = 0; j <= end; j++, i++) {
            const float *vj = v + (j * nh + h) * vd;
            float p = scores[i];
            for (size_t d = 0; d < vd; d++) oh[d] += p * vj[d];
        }
        m = m_new;
        t = end + 1;
    }
    for (size_t d = 0; d < vd; d++) oh[d] /= l;
}

/* src/model.rs:1706-1786: one (query, head) over the q8 cache */
ORC_API void orc_mla_attn_flash_q8(const orc_mla_cfg *cfg, int had_on, const int8_t *kq, const float *ks, const float *kr,
                                   const int8_t *vq, const float *vs, const float *qh, size_t h, size_t pos, float scale, float *oh) {
    size_t nh = cfg->nh, nope = cfg->nope, rope = cfg->rope, vd = cfg->vd;
    int had = had_on && nope % 64 == 0 && vd % 64 == 0;
    size_t nb = nope / 32;
    float *qnope = (float *)malloc(sizeof(float) * nope);
    memcpy(qnope, qh, sizeof(float) * nope);
    if (had)
        for (size_t b = 0; b < nope; b += 64) orc_hadamard64(qnope + b);
    int8_t *qq = (int8_t *)malloc(nope);
    float *qs = (float *)malloc(sizeof(float) * nb);
    orc_quantize_q8(qnope, nope, qq, qs);
    const float *q_rope = qh + nope;
    float had_k = had ? 1.0f / 64.0f : 1.0f;
    float m = -INFINITY, l = 0.0f;
    float scores[FLASH_KV];
    float *vtile = (float *)malloc(sizeof(float) * FLASH_KV * vd);
    size_t t = 0;
    while (t <= pos) {
        size_t end = t + FLASH_KV - 1 < pos ? t + FLASH_KV - 1 : pos;
        size_t tn = end - t + 1;
        float tm = -INFINITY;
        for (size_t j = t, i = 0; j <= end; j++, i++) {
            float s = orc_dot(q_rope, kr + j * rope, rope);
            float acc = 0.0f;
            size_t bq = (j * nh + h) * nope, bs = (j * nh + h) * nb;
            for (size_t g = 0; g < nb; g++) {
                int32_t d = orc_block_dot_i8(kq + bq + g * 32, qq + g * 32);
                acc += qs[g] * ks[bs + g] * (float)d;
            }
            s += had_k * acc;
            s = s * scale;
            scores[i] = s;
            tm = fmaxf(tm, s);
        }
        float m_new = fmaxf(m, tm);
        float corr = expf(m - m_new);
        float tile_l = 0.0f;
        for (size_t i = 0; i < tn; i++) {
            scores[i] = expf(scores[i] - m_new);
            tile_l += scores[i];
        }
        for (size_t d = 0; d < vd; d++) oh[d] *= corr;
        l = l * corr + tile_l;
        for (size_t j = t, i = 0; j <= end; j++, i++) {
            size_t bq = (j * nh + h) * vd, bs = (j * nh + h) * (vd / 32);
            float *out = vtile + i * vd;
            for (size_t g = 0; g < vd / 32; g++) {
                float sc = vs[bs + g];
                for (int d2 = 0; d2 < 32; d2++) out[g * 32 + d2] = (float)vq[bq + g * 32 + d2] * sc;
            }
            float p = scores[i];
            for (size_t d = 0; d < vd; d++) oh[d] += p * out[d];
        }
        m = m_new;
        t = end + 1;
    }
    if (had)
        for (size_t b = 0; b < vd; b += 64) {
            orc_hadamard64(oh + b);
            for (int i = 0; i < 64; i++) oh[b + i] /= 64.0f;
        }
    for (size_t d = 0; d < vd; d++) oh[d] /= l;
    free(qnope);
    free(qq);
    free(qs);
    free(vtile);
}

/* src/model.rs:1804-1908: all heads at once, tile-outer / head-inner.
 *
 * kv_heads selects the cache indexing: kv_heads == nh is the reference layout
 * (one K-nope row and one V row per head and position).  kv_heads == 1 is the
 * weight-absorbed MLA form: ONE latent row per position serves every head,
 * as K (with the shared rope row) and as V; pass vq == kq, vs == ks and
 * vd == nope for it.  The operation sequence per head is the same in both
 * cases -- only `h` is replaced by `h % kv_heads` in the cache offsets -- so
 * the absorbed form equals the reference function run on a cache whose per-head
 * rows are copies of the shared row (tested bit for bit). */
ORC_API void orc_mla_attn_flash_q8_mqa(const orc_mla_cfg *cfg, int had_on, size_t kv_heads, const int8_t *kq, const float *ks,
                                       const float *kr, const int8_t *vq, const float *vs, const float *q, size_t pos, float scale,
                                       float *attn) {
    size_t nh = cfg->nh, nope = cfg->nope, rope = cfg->rope, vd = cfg->vd;
    int had = had_on && nope % 64 == 0 && vd % 64 == 0;
    size_t hd = nope + rope, nb = nope / 32, nbv = vd / 32;
    int8_t *qq = (int8_t *)malloc(nh * nope);
    float *qs = (float *)malloc(sizeof(float) * nh * nb);
    float *qnope = (float *)malloc(sizeof(float) * nope);
    for (size_t h = 0; h < nh; h++) {
        memcpy(qnope, q + h * hd, sizeof(float) * nope);
        if (had)
            for (size_t b = 0; b < nope; b += 64) orc_hadamard64(qnope + b);
        orc_quantize_q8(qnope, nope, qq + h * nope, qs + h * nb);
    }
    float had_k = had ? 1.0f / 64.0f : 1.0f;
    float *m = (float *)malloc(sizeof(float) * nh);
    float *l = (float *)malloc(sizeof(float) * nh);
    float *scores = (float *)malloc(sizeof(float) * nh * FLASH_KV);
    float *vtile = (float *)malloc(sizeof(float) * vd);
    for (size_t h = 0; h < nh; h++) {
        m[h] = -INFINITY;
        l[h] = 0.0f;
    }
    size_t t = 0;
    while (t <= pos) {
        size_t end = t + FLASH_KV - 1 < pos ? t + FLASH_KV - 1 : pos;
        size_t tn = end - t + 1;
        for (size_t j = t, i = 0; j <= end; j++, i++) {
            const float *krj = kr + j * rope;
            const int8_t *kqj = kq + j * kv_heads * nope;
            const float *ksj = ks + j * kv_heads * nb;
            for (size_t h = 0; h < nh; h++) {
                size_t hk = h % kv_heads;
                float s = orc_dot(q + h * hd + nope, krj, rope);
                float acc = 0.0f;
                for (size_t g = 0; g < nb; g++) {
                    int32_t d = orc_block_dot_i8(kqj + hk * nope + g * 32, qq + h * nope + g * 32);
                    acc += qs[h * nb + g] * ksj[hk * nb + g] * (float)d;
                }
                s += had_k * acc;
                scores[h * FLASH_KV + i] = s * scale;
            }
        }
        for (size_t h = 0; h < nh; h++) {
            float *sh = scores + h * FLASH_KV;
            float tm = -INFINITY;
            for (size_t i = 0; i < tn; i++) tm = fmaxf(tm, sh[i]);
            float m_new = fmaxf(m[h], tm);
            float corr = expf(m[h] - m_new);
            float tile_l = 0.0f;
            for (size_t i = 0; i < tn; i++) {
                sh[i] = expf(sh[i] - m_new);
                tile_l += sh[i];
            }
            float *oh = attn + h * vd;
            for (size_t d = 0; d < vd; d++) oh[d] *= corr;
            l[h] = l[h] * corr + tile_l;
            m[h] = m_new;
        }
        for (size_t j = t, i = 0; j <= end; j++, i++) {
            const int8_t *vqj = vq + j * kv_heads * vd;
            const float *vsj = vs + j * kv_heads * nbv;
            for (size_t h = 0; h < nh; h++) {
                size_t hk = h % kv_heads;
                for (size_t g = 0; g < nbv; g++) {
                    float sc = vsj[hk * nbv + g];
                    for (int d2 = 0; d2 < 32; d2++) vtile[g * 32 + d2] = (float)vqj[hk * vd + g * 32 + d2] * sc;
                }
                float p = scores[h * FLASH_KV + i];
                float *oh = attn + h * vd;
                for (size_t d = 0; d < vd; d++) oh[d] += p * vtile[d];
            }
        }
        t = end + 1;
    }
    if (had)
        for (size_t h = 0; h < nh; h++)
            for (size_t b = 0; b < vd; b += 64) {
                orc_hadamard64(attn + h * vd + b);
                for (int i = 0; i < 64; i++) attn[h * vd + b + i] /= 64.0f;
            }
    for (size_t h = 0; h < nh; h++)
        for (size_t d = 0; d < vd; d++) attn[h * vd + d] /= l[h];
    free(qq);
    free(qs);
    free(qnope);
    free(m);
    free(l);
    free(scores);
    free(vtile);
}

/* src/model.rs:1914-1937: materialised-softmax reference over the dequantized
 * cache (k, v = orc_mla_cache_to_f32 output) */
ORC_API void orc_mla_attn_ref_q8(const orc_mla_cfg *cfg, const float *k, const float *v, const float *qh, size_t h, size_t pos,
                                 float scale, float *oh) {
    orc_mla_attn_ref(cfg, k, v, qh, h, pos, scale, oh);
}

/* ------------------------------------------------------------------ MoE */

/* src/model.rs:607-621 */
static inline float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }
ORC_API float orc_situ(float g, float u) { return 4.0f * tanhf(g / 4.0f) * sigmoidf_(g) * (25.0f * tanhf(u / 25.0f)); }
/* src/deepseek.rs:97-100 and :1086 */
ORC_API float orc_silu(float x) { return x / (1.0f + expf(-x)); }
/* src/deepseek.rs:61-68 */
static inline float softplusf_(float x) { return x > 20.0f ? x : logf(1.0f + expf(x)); }

typedef struct {
    uint32_t id;
    float score;
    float key;
} sel_t;

/* Rust's sort_by is a stable merge sort: a stable insertion sort on the
 * descending key gives the same order (src/model.rs:2165). */
static void sort_desc_stable(sel_t *s, size_t n) {
    for (size_t i = 1; i < n; i++) {
        sel_t v = s[i];
        size_t j = i;
        while (j > 0 && s[j - 1].key < v.key) {
            s[j] = s[j - 1];
            j--;
        }
        s[j] = v;
    }
}

/* The selection loop shared by src/model.rs:2157-2171 and src/deepseek.rs:36-48:
 * keep the k best keys, strict '>' against the current worst, stable re-sort. */
static size_t topk_select(const float *score, const float *key, size_t n, size_t k, sel_t *sel) {
    size_t len = 0;
    for (size_t i = 0; i < n; i++) {
        sel_t item = {(uint32_t)i, score[i], key[i]};
        if (len < k) {
            sel[len++] = item;
            if (len == k) sort_desc_stable(sel, k);
        } else if (item.key > sel[k - 1].key) {
            sel[k - 1] = item;
            sort_desc_stable(sel, k);
        }
    }
    return len;
}

/* src/deepseek.rs:16-58 (no hash routing): sqrtsoftplus scores, bias only for
 * selection, weights from the bias-free scores, renormalised, x route_scale. */
ORC_API void orc_gate_forward(const float *x, size_t d, const float *gate_w, const float *bias, size_t n_experts, size_t topk,
                              float route_scale, uint32_t *ids, float *weights) {
    float *orig = (float *)malloc(sizeof(float) * n_experts);
    float *key = (float *)malloc(sizeof(float) * n_experts);
    sel_t *sel = (sel_t *)malloc(sizeof(sel_t) * topk);
    for (size_t i = 0; i < n_experts; i++) {
        float logit = orc_dot(gate_w + i * d, x, d);
        orig[i] = sqrtf(softplusf_(logit));
        key[i] = orig[i] + (bias ? bias[i] : 0.0f);
    }
    size_t len = topk_select(orig, key, n_experts, topk, sel);
    float sum = 0.0f;
    for (size_t i = 0; i < len; i++) sum += orig[sel[i].id];
    for (size_t i = 0; i < len; i++) {
        ids[i] = sel[i].id;
        weights[i] = orig[sel[i].id] / sum * route_scale;
    }
    free(orig);
    free(key);
    free(sel);
}

/* src/model.rs:2157-2173: K3 router on given logits: sigmoid scores, bias for
 * the key, weights = score / (sum + 1e-20). */
ORC_API void orc_router_sigmoid(const float *logits, const float *bias, size_t n_experts, size_t topk, uint32_t *ids, float *weights) {
    float *sc = (float *)malloc(sizeof(float) * n_experts);
    float *key = (float *)malloc(sizeof(float) * n_experts);
    sel_t *sel = (sel_t *)malloc(sizeof(sel_t) * topk);
    for (size_t i = 0; i < n_experts; i++) {
        sc[i] = sigmoidf_(logits[i]);
        key[i] = sc[i] + (bias ? bias[i] : 0.0f);
    }
    size_t len = topk_select(sc, key, n_experts, topk, sel);
    float sumw = 0.0f;
    for (size_t i = 0; i < len; i++) sumw += sel[i].score;
    sumw += 1e-20f;
    for (size_t i = 0; i < len; i++) {
        ids[i] = sel[i].id;
        weights[i] = sel[i].score / sumw;
    }
    free(sc);
    free(key);
    free(sel);
}

/* Router of the benchmark's MoE layer: softmax over the logits (max-subtracted,
 * as src/model.rs:3271-3277 computes probabilities), top-k by probability with
 * the reference's selection rule (topk_select above: ties go to the lowest
 * index), weights renormalised to sum 1. */
ORC_API void orc_router_softmax(const float *logits, size_t n_experts, size_t topk, uint32_t *ids, float *weights) {
    float *p = (float *)malloc(sizeof(float) * n_experts);
    sel_t *sel = (sel_t *)malloc(sizeof(sel_t) * topk);
    float m = -INFINITY;
    for (size_t i = 0; i < n_experts; i++) m = fmaxf(m, logits[i]);
    float z = 0.0f;
    for (size_t i = 0; i < n_experts; i++) z += expf(logits[i] - m);
    for (size_t i = 0; i < n_experts; i++) p[i] = expf(logits[i] - m) / z;
    size_t len = topk_select(p, p, n_experts, topk, sel);
    float sum = 0.0f;
    for (size_t i = 0; i < len; i++) sum += sel[i].score;
    for (size_t i = 0; i < len; i++) {
        ids[i] = sel[i].id;
        weights[i] = sel[i].score / sum;
    }
    free(p);
    free(sel);
}

/* src/deepseek.rs:74-95: f32 expert with the SwiGLU clamp */
ORC_API void orc_expert_forward_f32(const float *w1, const float *w2, const float *w3, const float *x, size_t d, size_t inter,
                                    float limit, float *out) {
    float *gate = (float *)malloc(sizeof(float) * inter);
    float *up = (float *)malloc(sizeof(float) * inter);
    float *act = (float *)malloc(sizeof(float) * inter);
    orc_matvec_f32(w1, inter, d, x, gate);
    orc_matvec_f32(w3, inter, d, x, up);
    for (size_t i = 0; i < inter; i++) {
        float g = fminf(gate[i], limit);
        float u = clampf(up[i], -limit, limit);
        act[i] = orc_silu(g) * u;
    }
    orc_matvec_f32(w2, d, inter, act, out);
    free(gate);
    free(up);
    free(act);
}

/* Activation rules of the packed experts.
 *   ORC_ACT_SWIGLU  act = silu(g) * u                       (benchmark MoE layer; silu as src/deepseek.rs:1086)
 *   ORC_ACT_SITU    act = situ(g, u)                        (src/model.rs:2250-2252)
 *   ORC_ACT_DS      act = wgt * silu(min(g,L)) * clamp(u,L) (src/deepseek.rs:1083-1087; weight applied before W2) */
enum { ORC_ACT_SWIGLU = 0, ORC_ACT_SITU = 1, ORC_ACT_DS = 2 };

/* The first two matvec_packed calls of a packed expert and its activation
 * (src/model.rs:2246-2252 / src/deepseek.rs:1080-1087): act[j] = ACT(W1 x, W3 x)[j],
 * the f32 vector that the third call (W2) takes as its input. */
ORC_API void orc_expert_act(const uint8_t *w1p, const uint8_t *w1s, const uint8_t *w3p, const uint8_t *w3s, size_t d, size_t inter,
                            const float *x, int mode, int act_kind, float limit, float wgt, float *act) {
    float *a = (float *)malloc(sizeof(float) * inter);
    float *u = (float *)malloc(sizeof(float) * inter);
    orc_matvec_packed(w1p, w1s, inter, d, x, a, mode);
    orc_matvec_packed(w3p, w3s, inter, d, x, u, mode);
    for (size_t j = 0; j < inter; j++) {
        if (act_kind == ORC_ACT_SITU) {
            act[j] = orc_situ(a[j], u[j]);
        } else if (act_kind == ORC_ACT_DS) {
            float g = fminf(a[j], limit);
            float uu = clampf(u[j], -limit, limit);
            act[j] = wgt * (g / (1.0f + expf(-g))) * uu;
        } else {
            act[j] = (a[j] / (1.0f + expf(-a[j]))) * u[j];
        }
    }
    free(a);
    free(u);
}

/* A VQ1 ("cold") expert on one input (src/model.rs:2243-2259, vq branch): quant::matvec_vq for W1 and W3 on the f32
 * row, the activation, quant::matvec_vq for W2 on the f32 activation.  i1, i3: index bytes [inter][d/16]; i2: [d][inter/16]. */
ORC_API void orc_expert_vq(const float *codebook, const uint8_t *i1, const uint8_t *i3, const uint8_t *i2, size_t d, size_t inter,
                           const float *x, int act_kind, float limit, float wgt, float *out) {
    float *a = (float *)malloc(sizeof(float) * inter);
    float *u = (float *)malloc(sizeof(float) * inter);
    float *act = (float *)malloc(sizeof(float) * inter);
    orc_vq1_matvec_lut(codebook, i1, inter, d, x, a);
    orc_vq1_matvec_lut(codebook, i3, inter, d, x, u);
    for (size_t j = 0; j < inter; j++) {
        if (act_kind == ORC_ACT_SITU) {
            act[j] = orc_situ(a[j], u[j]);
        } else if (act_kind == ORC_ACT_DS) {
            float g = fminf(a[j], limit);
            float uu = clampf(u[j], -limit, limit);
            act[j] = wgt * (g / (1.0f + expf(-g))) * uu;
        } else {
            act[j] = (a[j] / (1.0f + expf(-a[j]))) * u[j];
        }
    }
    orc_vq1_matvec_lut(codebook, i2, d, inter, act, out);
    free(a);
    free(u);
    free(act);
}

/* One packed expert on one input: the three matvec_packed calls of
 * src/model.rs:2246-2259 / src/deepseek.rs:1080-1089.  w1,w3: [inter][d],
 * w2: [d][inter]; each as (packed, scales).  mode as orc_matvec_packed. */
ORC_API void orc_expert_packed(const uint8_t *w1p, const uint8_t *w1s, const uint8_t *w3p, const uint8_t *w3s, const uint8_t *w2p,
                               const uint8_t *w2s, size_t d, size_t inter, const float *x, int mode, int act_kind, float limit,
                               float wgt, float *out) {
    float *act = (float *)malloc(sizeof(float) * inter);
    orc_expert_act(w1p, w1s, w3p, w3s, d, inter, x, mode, act_kind, limit, wgt, act);
    orc_matvec_packed(w2p, w2s, d, inter, act, out, mode);
    free(act);
}

typedef struct {
    const uint8_t *const *w1p, *const *w1s, *const *w3p, *const *w3s, *const *w2p, *const *w2s;
    size_t d, inter;
    const float *x;
    int mode, act_kind;
    float limit, wgt;
    uint32_t eid;
    float *out;
} expert_job_t;

static void *expert_job(void *p) {
    expert_job_t *j = (expert_job_t *)p;
    uint32_t e = j->eid;
    orc_expert_packed(j->w1p[e], j->w1s[e], j->w3p[e], j->w3s[e], j->w2p[e], j->w2s[e], j->d, j->inter, j->x, j->mode, j->act_kind,
                      j->limit, j->wgt, j->out);
    return NULL;
}

/* Decode MoE layer for B tokens: per token, one job per selected expert
 * (src/model.rs:2227-2264, src/deepseek.rs:1069-1093; run on `threads` threads,
 * 1 = sequential), then the combination in slot order:
 *   ORC_ACT_DS:    out = sum_slot o_slot            (src/deepseek.rs:1095-1100)
 *   otherwise:     out = sum_slot w_slot * o_slot   (src/model.rs:2346-2351)
 * plus, when shared >= 0, the unweighted output of expert table entry `shared`
 * on the same input (src/deepseek.rs:1101-1106 adds an unweighted shared
 * expert; here it is a packed expert like the others, as the benchmark's layer
 * has it).  Expert tables are arrays of pointers indexed by expert id.
 * ids, weights: [B][topk]; x: [B][d]; out: [B][d]. */
ORC_API void orc_moe_decode(const uint8_t *const *w1p, const uint8_t *const *w1s, const uint8_t *const *w3p, const uint8_t *const *w3s,
                            const uint8_t *const *w2p, const uint8_t *const *w2s, size_t d, size_t inter, size_t B, size_t topk,
                            const uint32_t *ids, const float *weights, int shared, const float *x, int mode, int act_kind, float limit,
                            size_t threads, float *out) {
    size_t nj = topk + (shared >= 0 ? 1 : 0);
    float *outs = (float *)malloc(sizeof(float) * nj * d);
    expert_job_t *jobs = (expert_job_t *)malloc(sizeof(expert_job_t) * nj);
    pthread_t *th = (pthread_t *)malloc(sizeof(pthread_t) * nj);
    for (size_t t = 0; t < B; t++) {
        for (size_t s = 0; s < nj; s++) {
            expert_job_t jb = {w1p, w1s, w3p, w3s, w2p, w2s, d, inter, x + t * d, mode, act_kind, limit, 1.0f, 0, outs + s * d};
            if (s < topk) {
                jb.eid = ids[t * topk + s];
                jb.wgt = weights[t * topk + s];
            } else {
                jb.eid = (uint32_t)shared;
                jb.wgt = 1.0f;
            }
            jobs[s] = jb;
        }
        if (threads <= 1) {
            for (size_t s = 0; s < nj; s++) expert_job(&jobs[s]);
        } else {
            /* one job per expert; at most `threads` in flight */
            for (size_t s0 = 0; s0 < nj; s0 += threads) {
                size_t s1 = s0 + threads < nj ? s0 + threads : nj;
                for (size_t s = s0; s < s1; s++) pthread_create(&th[s], NULL, expert_job, &jobs[s]);
                for (size_t s = s0; s < s1; s++) pthread_join(th[s], NULL);
            }
        }
        float *y = out + t * d;
        for (size_t j = 0; j < d; j++) y[j] = 0.0f;
        for (size_t s = 0; s < topk; s++) {
            float wi = (act_kind == ORC_ACT_DS) ? 1.0f : weights[t * topk + s];
            if (act_kind == ORC_ACT_DS) {
                for (size_t j = 0; j < d; j++) y[j] += outs[s * d + j];
            } else {
                for (size_t j = 0; j < d; j++) y[j] += wi * outs[s * d + j];
            }
        }
        if (shared >= 0)
            for (size_t j = 0; j < d; j++) y[j] += outs[topk * d + j];
    }
    free(outs);
    free(jobs);
    free(th);
}

/* Prefill MoE (src/model.rs:2539-2602, 2690-2700): (token, slot) pairs grouped
 * by expert; per used expert the inputs are gathered transposed [d][m8], three
 * matvec_packed_nt calls with the activation between, outputs scattered to
 * (token, slot), then per token the weighted sum in slot order.  Always the
 * f32 arithmetic of matvec_packed_nt.  act_kind SWIGLU or SITU.
 * When round_mxfp8 != 0 the gathered inputs and the activation are first
 * passed through the e4m3 + e8m0/32 round trip (block 32 along K): that is the
 * input precision of the block-scaled MFMA GEMM, and the oracle it is compared
 * against tightly.  1: the reference's orc_fp8_roundtrip (scale exponent
 * clamped at 8); 2: the full e8m0 range (orc_fp8_roundtrip_emax with 127), the
 * encoding of the device's prefill section; 3: hidden rows and activation
 * rounded to bfloat16 (round to nearest even), the inputs of the device's
 * bf16 prefill section. */
ORC_API void orc_round_bf16(float *x, size_t n) {
    for (size_t i = 0; i < n; i++) {
        uint32_t b;
        memcpy(&b, &x[i], 4);
        if ((b & 0x7F800000u) == 0x7F800000u) continue; /* inf / NaN stay */
        b += 0x7FFFu + ((b >> 16) & 1u);
        b &= 0xFFFF0000u;
        memcpy(&x[i], &b, 4);
    }
}
static void orc_round_inputs(float *x, size_t n, int mode) {
    if (mode == 3) orc_round_bf16(x, n);
    else if (mode) orc_fp8_roundtrip_emax(x, n, 32, mode == 2 ? 127 : 8, NULL, NULL);
}
ORC_API void orc_moe_prefill(const uint8_t *const *w1p, const uint8_t *const *w1s, const uint8_t *const *w3p, const uint8_t *const *w3s,
                             const uint8_t *const *w2p, const uint8_t *const *w2s, size_t n_experts, size_t d, size_t inter, size_t n,
                             size_t topk, const uint32_t *ids, const float *weights, const float *x, int act_kind, int round_mxfp8,
                             float *out) {
    float *outs = (float *)malloc(sizeof(float) * n * topk * d);
    size_t *cnt = (size_t *)calloc(n_experts, sizeof(size_t));
    for (size_t i = 0; i < n * topk; i++) cnt[ids[i]]++;
    size_t *pairs = (size_t *)malloc(sizeof(size_t) * n * topk);
    for (uint32_t e = 0; e < n_experts; e++) {
        size_t m = cnt[e];
        if (m == 0) continue;
        size_t k = 0;
        for (size_t t = 0; t < n; t++)
            for (size_t s = 0; s < topk; s++)
                if (ids[t * topk + s] == e) pairs[k++] = t * topk + s;
        size_t m8 = (m + 7) / 8 * 8;
        float *ht = (float *)calloc(m8 * d, sizeof(float));
        float *tmp = (float *)malloc(sizeof(float) * (d > inter ? d : inter));
        for (size_t i = 0; i < m; i++) {
            size_t t = pairs[i] / topk;
            memcpy(tmp, x + t * d, sizeof(float) * d);
            orc_round_inputs(tmp, d, round_mxfp8);
            for (size_t c = 0; c < d; c++) ht[c * m8 + i] = tmp[c];
        }
        float *a = (float *)malloc(sizeof(float) * m8 * inter);
        float *u = (float *)malloc(sizeof(float) * m8 * inter);
        orc_matvec_packed_nt(w1p[e], w1s[e], inter, d, ht, m8, a);
        orc_matvec_packed_nt(w3p[e], w3s[e], inter, d, ht, m8, u);
        float *act_t = (float *)calloc(m8 * inter, sizeof(float));
        for (size_t i = 0; i < m; i++) {
            for (size_t j = 0; j < inter; j++) {
                float g = a[i * inter + j], uu = u[i * inter + j];
                tmp[j] = (act_kind == ORC_ACT_SITU) ? orc_situ(g, uu) : (g / (1.0f + expf(-g))) * uu;
            }
            orc_round_inputs(tmp, inter, round_mxfp8);
            for (size_t j = 0; j < inter; j++) act_t[j * m8 + i] = tmp[j];
        }
        float *o = (float *)malloc(sizeof(float) * m8 * d);
        orc_matvec_packed_nt(w2p[e], w2s[e], d, inter, act_t, m8, o);
        for (size_t i = 0; i < m; i++) memcpy(outs + pairs[i] * d, o + i * d, sizeof(float) * d);
        free(ht);
        free(tmp);
        free(a);
        free(u);
        free(act_t);
        free(o);
    }
    for (size_t t = 0; t < n; t++) {
        float *y = out + t * d;
        for (size_t j = 0; j < d; j++) y[j] = 0.0f;
        for (size_t s = 0; s < topk; s++) {
            float wi = weights[t * topk + s];
            for (size_t j = 0; j < d; j++) y[j] += wi * outs[(t * topk + s) * d + j];
        }
    }
    free(outs);
    free(cnt);
    free(pairs);
}

/* ------------------------------------------------------- test utilities */

/* splitmix64 byte stream of src/q8.rs:269-278 */
ORC_API void orc_rng_u8(uint64_t *state, uint8_t *out, size_t n) {
    for (size_t i = 0; i < n; i++) {
        *state += 0x9E3779B97F4A7C15ull;
        uint64_t z = *state;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        out[i] = (uint8_t)(z ^ (z >> 31));
    }
}

/* splitmix64 float stream of src/model.rs:3683-3692: uniform in [-0.5, 0.5] */
ORC_API void orc_rng_f32(uint64_t *state, float *out, size_t n) {
    for (size_t i = 0; i < n; i++) {
        *state += 0x9E3779B97F4A7C15ull;
        uint64_t z = *state;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        out[i] = (float)((double)(z ^ (z >> 31)) / (double)UINT64_MAX - 0.5);
    }
}

/* the integer-hash pattern of src/selftest.rs:540-543 (values in [-1, 1]) */
ORC_API void orc_pattern(size_t start, float *out, size_t n) {
    for (size_t i = 0; i < n; i++) {
        uint64_t h = (uint64_t)(start + i) * 2654435761ull + 0x9E3779B9ull;
        out[i] = (float)((h >> 13) % 2000) / 1000.0f - 1.0f;
    }
}
