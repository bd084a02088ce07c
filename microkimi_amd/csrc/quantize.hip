// Weight quantizers of the offline path, on the device: mxfp4::quantize / quantize_naive (src/mxfp4.rs:38-138),
// dequant::quantize_fp8 (src/dequant.rs:50-74) and the MXFP4SQ storage variant (quantize_sq / dequant_sq,
// src/mxfp4.rs:140-229).  Neither is on a decode or prefill path (weights arrive quantized); they
// are here so that a caller that quantizes on load need not leave the device, and they give the reference's bytes.
#include "mk_common.h"

namespace {

// ceil(log2f(r)) for any positive finite r (subnormal too), log2f being the correctly rounded float logarithm
__device__ __forceinline__ int ceil_log2f_any(float r) {
    if (__float_as_uint(r) >= 0x00800000u) return mk_ceil_log2f(r);
    return (int)ceilf((float)log2((double)r));
}

// 2^e for e in [-127, 128] (mxfp4::exp2_i, src/mxfp4.rs:332-338): -127 is the subnormal, 128 is infinity
__device__ __forceinline__ float exp2_i(int e) {
    if (e <= -127) return __uint_as_float(0x00400000u);
    if (e >= 128) return __uint_as_float(0x7F800000u);
    return __uint_as_float((uint32_t)(e + 127) << 23);
}

// index of the nearest E2M1 level by the midpoints {.25, .75, 1.25, 1.75, 2.5, 3.5, 5} (src/mxfp4.rs:41-49)
__device__ __forceinline__ int e2m1_index(float mag) {
    return (mag >= 0.25f) + (mag >= 0.75f) + (mag >= 1.25f) + (mag >= 1.75f) + (mag >= 2.5f) + (mag >= 3.5f) + (mag >= 5.0f);
}
__device__ __forceinline__ float clamp6(float v) { return v < -6.0f ? -6.0f : (v > 6.0f ? 6.0f : v); }

// squared error of a group quantized with scale 2^e, in f64 (group_sse, src/mxfp4.rs:51-69)
__device__ __forceinline__ double group_sse(const float (&g)[32], int e) {
    const float inv = 1.0f / exp2_i(e);
    const double s = (double)exp2_i(e);
    double sse = 0.0;
#pragma unroll 4
    for (int i = 0; i < 32; i++) {
        const float q = clamp6(g[i] * inv);
        const int idx = e2m1_index(fabsf(q));
        const double lvl = idx < 5 ? 0.5 * idx : (idx == 5 ? 3.0 : (idx == 6 ? 4.0 : 6.0));
        const double dq = (__float_as_uint(q) >> 31 ? -lvl : lvl) * s;
        const double d = (double)g[i] - dq;
        sse += d * d;
    }
    return sse;
}

// one thread per 32-group
__global__ __launch_bounds__(256) void mxfp4_quantize_kernel(const float *__restrict__ w, size_t n_groups, int search, uint8_t *__restrict__ packed,
                                                             uint8_t *__restrict__ scales) {
    const size_t gi = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gi >= n_groups) return;
    float g[32];
    const mk_f4 *src = reinterpret_cast<const mk_f4 *>(w + gi * 32);
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const mk_f4 v = src[i];
        g[4 * i] = v.x;
        g[4 * i + 1] = v.y;
        g[4 * i + 2] = v.z;
        g[4 * i + 3] = v.w;
    }
    float maxabs = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; i++) maxabs = fmaxf(maxabs, fabsf(g[i]));
    int e = maxabs == 0.0f ? -127 : ceil_log2f_any(maxabs / 6.0f);
    e = max(-127, min(128, e));
    if (search && maxabs != 0.0f) {  // search_mx_scale (src/mxfp4.rs:77-92): e - 1, e + 1 against e, strictly better only
        int best = e;
        double best_sse = group_sse(g, e);
        for (int c = 0; c < 2; c++) {
            const int cand = c == 0 ? e - 1 : e + 1;
            if (cand < -127 || cand > 128) continue;
            const double sse = group_sse(g, cand);
            if (sse < best_sse) {
                best_sse = sse;
                best = cand;
            }
        }
        e = best;
    }
    scales[gi] = (uint8_t)max(0, min(255, e + 127));
    const float inv = 1.0f / exp2_i(e);
    uint32_t out[4] = {0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < 32; j++) {
        const float q = clamp6(g[j] * inv);
        const uint32_t idx = (uint32_t)e2m1_index(fabsf(q)) + ((__float_as_uint(q) >> 31) ? 8u : 0u);
        out[j >> 3] |= idx << (4 * (j & 7));  // element 2 c in the low nibble of byte c, 2 c + 1 in the high one
    }
    *reinterpret_cast<mk_v4u *>(packed + gi * 16) = mk_v4u{out[0], out[1], out[2], out[3]};
}

// one workgroup per 128 x 128 block
__global__ __launch_bounds__(256) void quantize_fp8_kernel(const float *__restrict__ w, int cols, uint8_t *__restrict__ qw,
                                                           uint8_t *__restrict__ scales) {
    __shared__ float red[4];
    __shared__ int e_l;
    const int bc = blockIdx.x, br = blockIdx.y, tid = threadIdx.x;
    const size_t base = (size_t)br * 128 * cols + (size_t)bc * 128;
    // thread: column quad tid % 32, rows tid / 32, + 8, ...
    const int c4 = (tid & 31) * 4, r0 = tid >> 5;
    float mx = 0.0f;
    for (int r = r0; r < 128; r += 8) {
        const mk_f4 v = *reinterpret_cast<const mk_f4 *>(w + base + (size_t)r * cols + c4);
        mx = fmaxf(mx, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
    }
    mx = mk_wave_max(mx);
    if ((tid & 63) == 0) red[tid >> 6] = mx;
    __syncthreads();
    if (tid == 0) {
        const float maxabs = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        int e = maxabs == 0.0f ? -127 : ceil_log2f_any(maxabs / 448.0f);
        e = max(-127, min(8, e));
        e_l = e;
        scales[(size_t)br * gridDim.x + bc] = (uint8_t)(e + 127);
    }
    __syncthreads();
    const float inv = 1.0f / exp2_i(e_l);
    for (int r = r0; r < 128; r += 8) {
        const mk_f4 v = *reinterpret_cast<const mk_f4 *>(w + base + (size_t)r * cols + c4);
        const uint32_t c = mk_f32_to_e4m3(v.x * inv) | (mk_f32_to_e4m3(v.y * inv) << 8) | (mk_f32_to_e4m3(v.z * inv) << 16) |
                           (mk_f32_to_e4m3(v.w * inv) << 24);
        *reinterpret_cast<uint32_t *>(qw + base + (size_t)r * cols + c4) = c;
    }
}

// ---- MXFP4SQ (src/mxfp4.rs:140-229): e2m1 nibbles as MXFP4, scale byte q -> ((q + 1) / 256)^2 * smax, smax the largest
// maxabs / 6 over the tensor's groups.
__device__ __forceinline__ float scale_sq(uint32_t q, float smax) {
    const float t = ((float)q + 1.0f) * (1.0f / 256.0f);
    return t * t * smax;
}

__global__ void sq_clear_kernel(float *smax) { *smax = 0.0f; }

// pass 1: smax = max over groups of maxabs / 6 (non-negative floats order like their bit patterns)
__global__ __launch_bounds__(256) void sq_smax_kernel(const float *__restrict__ w, size_t n_groups, float *__restrict__ smax) {
    const size_t gi = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    float ideal = 0.0f;
    if (gi < n_groups) {
        const mk_f4 *src = reinterpret_cast<const mk_f4 *>(w + gi * 32);
        float maxabs = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const mk_f4 v = src[i];
            maxabs = fmaxf(maxabs, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
        }
        ideal = maxabs / 6.0f;
    }
    ideal = mk_wave_max(ideal);
    if ((threadIdx.x & 63) == 0 && ideal > 0.0f) atomicMax(reinterpret_cast<unsigned int *>(smax), __float_as_uint(ideal));
}

// pass 2: one thread per group
__global__ __launch_bounds__(256) void sq_quantize_kernel(const float *__restrict__ w, size_t n_groups, const float *__restrict__ smax_p,
                                                          uint8_t *__restrict__ packed, uint8_t *__restrict__ scales) {
    const size_t gi = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gi >= n_groups) return;
    const float smax = *smax_p;
    float g[32];
    const mk_f4 *src = reinterpret_cast<const mk_f4 *>(w + gi * 32);
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const mk_f4 v = src[i];
        g[4 * i] = v.x;
        g[4 * i + 1] = v.y;
        g[4 * i + 2] = v.z;
        g[4 * i + 3] = v.w;
    }
    float maxabs = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; i++) maxabs = fmaxf(maxabs, fabsf(g[i]));
    const float ideal = maxabs / 6.0f;
    int q = 0;
    if (!(smax == 0.0f || ideal == 0.0f)) q = max(0, min(255, (int)ceilf(256.0f * sqrtf(ideal / smax)) - 1));  // rounded up: no value clips
    scales[gi] = (uint8_t)q;
    const float inv = 1.0f / scale_sq((uint32_t)q, smax);
    uint32_t out[4] = {0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < 32; j++) {
        const float qv = clamp6(g[j] * inv);
        const uint32_t idx = (uint32_t)e2m1_index(fabsf(qv)) + ((__float_as_uint(qv) >> 31) ? 8u : 0u);
        out[j >> 3] |= idx << (4 * (j & 7));
    }
    *reinterpret_cast<mk_v4u *>(packed + gi * 16) = mk_v4u{out[0], out[1], out[2], out[3]};
}

// a thread per packed word (8 values)
__global__ __launch_bounds__(256) void sq_dequant_kernel(const uint32_t *__restrict__ packed, const uint8_t *__restrict__ scales, const float *smax_p,
                                                         float smax_v, size_t n_words, float *__restrict__ out) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_words) return;
    const float smax = smax_p ? *smax_p : smax_v;
    const uint32_t w = packed[i];
    const float s = scale_sq(scales[i >> 2], smax);
    mk_f4 lo, hi;
    lo.x = mk_e2m1(w & 15u) * s;
    lo.y = mk_e2m1((w >> 4) & 15u) * s;
    lo.z = mk_e2m1((w >> 8) & 15u) * s;
    lo.w = mk_e2m1((w >> 12) & 15u) * s;
    hi.x = mk_e2m1((w >> 16) & 15u) * s;
    hi.y = mk_e2m1((w >> 20) & 15u) * s;
    hi.z = mk_e2m1((w >> 24) & 15u) * s;
    hi.w = mk_e2m1(w >> 28) * s;
    reinterpret_cast<mk_f4 *>(out)[2 * i] = lo;
    reinterpret_cast<mk_f4 *>(out)[2 * i + 1] = hi;
}

}  // namespace

extern "C" int mk_dev_mxfp4sq_quantize(const float *w, size_t rows, size_t cols, uint8_t *packed, uint8_t *scales, float *smax, void *stream) {
    MK_REQUIRE(w && packed && scales && smax, "null pointer");
    MK_REQUIRE(cols % 32 == 0, "cols must be a multiple of 32");
    MK_REQUIRE(((uintptr_t)w & 15) == 0 && ((uintptr_t)packed & 15) == 0 && ((uintptr_t)smax & 3) == 0, "w and packed must be 16-byte aligned");
    const size_t n_groups = rows * (cols / 32);
    MK_REQUIRE((n_groups + 255) / 256 <= 0x7FFFFFFFull, "matrix too large for one launch");
    hipStream_t st = (hipStream_t)stream;
    hipLaunchKernelGGL(sq_clear_kernel, dim3(1), dim3(1), 0, st, smax);
    int s = mk_launch_status("sq_clear");
    if (s != MK_OK || n_groups == 0) return s;
    const unsigned grid = (unsigned)((n_groups + 255) / 256);
    hipLaunchKernelGGL(sq_smax_kernel, dim3(grid), dim3(256), 0, st, w, n_groups, smax);
    if ((s = mk_launch_status("sq_smax")) != MK_OK) return s;
    hipLaunchKernelGGL(sq_quantize_kernel, dim3(grid), dim3(256), 0, st, w, n_groups, smax, packed, scales);
    return mk_launch_status("sq_quantize");
}

extern "C" int mk_dev_mxfp4sq_dequant(const uint8_t *packed, const uint8_t *scales, const float *smax_dev, float smax, size_t rows, size_t cols,
                                      float *out, void *stream) {
    MK_REQUIRE(packed && scales && out, "null pointer");
    MK_REQUIRE(cols % 32 == 0, "cols must be a multiple of 32");
    MK_REQUIRE(((uintptr_t)packed & 3) == 0 && ((uintptr_t)out & 15) == 0, "packed must be 4-byte and out 16-byte aligned");
    const size_t n_words = rows * cols / 8;
    if (n_words == 0) return MK_OK;
    MK_REQUIRE((n_words + 255) / 256 <= 0x7FFFFFFFull, "matrix too large for one launch");
    hipLaunchKernelGGL(sq_dequant_kernel, dim3((unsigned)((n_words + 255) / 256)), dim3(256), 0, (hipStream_t)stream, (const uint32_t *)packed, scales,
                       smax_dev, smax, n_words, out);
    return mk_launch_status("sq_dequant");
}

extern "C" int mk_dev_mxfp4_quantize(const float *w, size_t rows, size_t cols, int search, uint8_t *packed, uint8_t *scales, void *stream) {
    MK_REQUIRE(w && packed && scales, "null pointer");
    MK_REQUIRE(cols % 32 == 0, "cols must be a multiple of 32");
    MK_REQUIRE(((uintptr_t)w & 15) == 0 && ((uintptr_t)packed & 15) == 0, "w and packed must be 16-byte aligned");
    const size_t n_groups = rows * (cols / 32);
    if (n_groups == 0) return MK_OK;
    MK_REQUIRE((n_groups + 255) / 256 <= 0x7FFFFFFFull, "matrix too large for one launch");
    hipLaunchKernelGGL(mxfp4_quantize_kernel, dim3((unsigned)((n_groups + 255) / 256)), dim3(256), 0, (hipStream_t)stream, w, n_groups, search ? 1 : 0,
                       packed, scales);
    return mk_launch_status("mxfp4_quantize");
}

extern "C" int mk_dev_quantize_fp8(const float *w, size_t rows, size_t cols, uint8_t *qw, uint8_t *scales, void *stream) {
    MK_REQUIRE(w && qw && scales, "null pointer");
    MK_REQUIRE(rows % 128 == 0 && cols % 128 == 0, "rows and cols must be multiples of 128");
    MK_REQUIRE(((uintptr_t)w & 15) == 0 && ((uintptr_t)qw & 3) == 0, "w must be 16-byte and the codes 4-byte aligned");
    MK_REQUIRE(cols <= 0x7FFFFF80ull && rows / 128 <= 65535, "matrix too large for one launch");
    if (rows == 0 || cols == 0) return MK_OK;
    hipLaunchKernelGGL(quantize_fp8_kernel, dim3((unsigned)(cols / 128), (unsigned)(rows / 128)), dim3(256), 0, (hipStream_t)stream, w, (int)cols, qw,
                       scales);
    return mk_launch_status("quantize_fp8");
}
