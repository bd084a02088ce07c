// Codec kernels: MXFP4 / FP8 dequantization (bit-exact), q8_0 and MXFP8
// activation quantization.  All HBM-bound elementwise work: 128-bit accesses,
// one pass over the data.
#include "mk_common.h"

// ---------------------------------------------------------------- mxfp4::dequant
// One thread decodes 8 nibbles (one dword of packed bytes) into two float4
// stores.  W[r,c] = E2M1[nibble] * 2^(sb-127), low nibble = even column
// (src/mxfp4.rs:19-31).  The product is one IEEE multiply, as in the reference.
__global__ __launch_bounds__(256) void mk_mxfp4_dequant_kernel(const uint32_t *__restrict__ packed, const uint8_t *__restrict__ scales,
                                                               size_t n_words, float *__restrict__ out) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_words) return;
    uint32_t w = packed[i];
    // word i holds elements 8i .. 8i+7; 4 words per 32-block
    float s = mk_scale_from_byte(scales[i >> 2]);
    mk_f4 lo, hi;
    lo.x = mk_e2m1(w & 15u) * s;
    lo.y = mk_e2m1((w >> 4) & 15u) * s;
    lo.z = mk_e2m1((w >> 8) & 15u) * s;
    lo.w = mk_e2m1((w >> 12) & 15u) * s;
    hi.x = mk_e2m1((w >> 16) & 15u) * s;
    hi.y = mk_e2m1((w >> 20) & 15u) * s;
    hi.z = mk_e2m1((w >> 24) & 15u) * s;
    hi.w = mk_e2m1((w >> 28) & 15u) * s;
    mk_f4 *o = reinterpret_cast<mk_f4 *>(out + i * 8);
    o[0] = lo;
    o[1] = hi;
}

// ---------------------------------------------------------------- dequant::dequant_fp8
// e4m3fn byte -> f32 by bit construction (src/dequant.rs:12-23): normal
// (-1)^s 2^(e-7) (1+m/8), subnormal (-1)^s (m/8) 2^-6, 0x7F/0xFF NaN.
__device__ __forceinline__ float mk_e4m3_to_f32(uint32_t b) {
    uint32_t sign = (b & 0x80u) << 24;
    uint32_t e = (b >> 3) & 15u, m = b & 7u;
    if (e == 15u && m == 7u) return __uint_as_float(0x7FC00000u);
    if (e == 0u) {
        float v = (float)m * 0.001953125f;  // m * 2^-9, exact
        return __uint_as_float(__float_as_uint(v) | sign);
    }
    return __uint_as_float(sign | ((e + 120u) << 23) | (m << 20));
}

__global__ __launch_bounds__(256) void mk_fp8_dequant_kernel(const uint8_t *__restrict__ w, const uint8_t *__restrict__ scales, size_t rows,
                                                             size_t cols, float *__restrict__ out) {
    // one thread = 4 consecutive columns of one row (cols % 4 == 0)
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t per_row = cols / 4;
    if (i >= rows * per_row) return;
    size_t r = i / per_row, c = (i % per_row) * 4;
    size_t scols = (cols + 127) / 128;
    float s = mk_scale_from_byte(scales[(r / 128) * scols + c / 128]);
    // byte 0 must mean 2^-127 here as well (exp2_i(-127)); mk_scale_from_byte gives that
    uint32_t v = *reinterpret_cast<const uint32_t *>(w + r * cols + c);
    mk_f4 o;
    o.x = mk_e4m3_to_f32(v & 255u) * s;
    o.y = mk_e4m3_to_f32((v >> 8) & 255u) * s;
    o.z = mk_e4m3_to_f32((v >> 16) & 255u) * s;
    o.w = mk_e4m3_to_f32(v >> 24) * s;
    *reinterpret_cast<mk_f4 *>(out + r * cols + c) = o;
}

// ---------------------------------------------------------------- q8::quantize_q8_into
// One half-wave (32 lanes) per block of 32 values: lane j holds x[32 g + j],
// the block maximum comes from 5 cross-lane steps, every lane rounds its own
// value (src/q8.rs:57-68).  SCALE_F16: the scale is stored as f16 (q8_0 storage
// form) after the quantization used the f32 value.
template <bool SCALE_F16>
__global__ __launch_bounds__(256) void mk_quantize_q8_kernel(const float *__restrict__ x, size_t n_blocks, int8_t *__restrict__ q,
                                                             void *__restrict__ scales) {
    // 8 lanes per 32-block, four values each
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_blocks * 8) return;  // whole groups of 8 lanes leave together
    const mk_f4 v = reinterpret_cast<const mk_f4 *>(x)[i];
    float mx = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    mx = fmaxf(mx, mk_dpp<0xB1>(mx));
    mx = fmaxf(mx, mk_dpp<0x4E>(mx));
    mx = fmaxf(mx, mk_dpp<0x141>(mx));
    const float dx = fmaxf(mx, 0.0f) / 127.0f;  // (a block of NaN only: the reference's maximum, folded from 0, is 0)
    uint32_t packed = 0;
    if (dx != 0.0f) {
        float qf[4];
        mk_q8_round4(v, dx, qf);
        packed = ((uint32_t)(int)qf[0] & 255u) | (((uint32_t)(int)qf[1] & 255u) << 8) | (((uint32_t)(int)qf[2] & 255u) << 16) |
                 ((uint32_t)(int)qf[3] << 24);
    }
    reinterpret_cast<uint32_t *>(q)[i] = packed;
    if ((i & 7) == 0) {
        if (SCALE_F16)
            reinterpret_cast<uint16_t *>(scales)[i >> 3] = mk_f32_to_f16_bits(dx);
        else
            reinterpret_cast<float *>(scales)[i >> 3] = dx;
    }
}

// ---------------------------------------------------------------- MXFP8 activations
// The e4m3 encoder and the per-32 MXFP8 quantizer live in mk_common.h (the prefill
// pipeline uses them too).
// a lane takes 8 consecutive values, four lanes a 32-block
__global__ __launch_bounds__(256) void mk_quantize_mxfp8_kernel(const float *__restrict__ x, size_t n_blocks, uint8_t *__restrict__ codes,
                                                                uint8_t *__restrict__ exps) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;  // group of 8 values
    if (i >= n_blocks * 4) return;
    const mk_f4 a = reinterpret_cast<const mk_f4 *>(x)[2 * i], b = reinterpret_cast<const mk_f4 *>(x)[2 * i + 1];
    const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    uint32_t eb, c0, c1;
    mk_mxfp8_quantize8(v, eb, c0, c1);
    reinterpret_cast<mk_u2 *>(codes)[i] = mk_u2{c0, c1};
    if ((i & 3) == 0) exps[i >> 2] = (uint8_t)eb;
}

// The scale bytes of an MXFP4 matrix, [rows][cols / 32], once more as [cols / 512][rows][16]: the 16 bytes that a row has
// per 512 columns, rows of one K tile together.  One thread per 16 bytes.
__global__ __launch_bounds__(256) void mk_scales_by_tile_kernel(const uint4 *__restrict__ scales, uint4 *__restrict__ out, size_t rows, size_t kt) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * kt) return;
    const size_t t = i / rows, r = i - t * rows;
    out[i] = scales[r * kt + t];
}

// bfloat16 of every value as two e4m3 terms (mk_bf16_split8), rows of n values, in the K-tile layout of the two-term GEMM
__global__ __launch_bounds__(256) void mk_quantize_bf16_split_kernel(const float *__restrict__ x, size_t n_groups8, int n, uint8_t *__restrict__ codes,
                                                                     uint8_t *__restrict__ exps) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;  // group of 8 values
    if (i >= n_groups8) return;                               // (n % 32 == 0: whole quads leave together)
    const int per_row = n / 8;
    const size_t r = i / per_row, c = i % per_row;
    const mk_f4 a = reinterpret_cast<const mk_f4 *>(x)[2 * i], b = reinterpret_cast<const mk_f4 *>(x)[2 * i + 1];
    const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    uint32_t hi[2], lo[2], eh, el;
    mk_bf16_split8<false>(v, hi, lo, eh, el);
    const size_t kt = c >> 6, within = (c & 63) * 8;
    uint8_t *dst = codes + r * (2 * (size_t)n) + kt * 1024 + within;
    *reinterpret_cast<mk_u2 *>(dst) = mk_u2{hi[0], hi[1]};
    *reinterpret_cast<mk_u2 *>(dst + 512) = mk_u2{lo[0], lo[1]};
    if ((c & 3) == 0) {
        uint8_t *ed = exps + r * (size_t)(n / 16) + kt * 32 + ((c & 63) >> 2);
        ed[0] = (uint8_t)eh;
        ed[16] = (uint8_t)el;
    }
}

// ------------------------------------------------------------------ C ABI
extern "C" int mk_dev_quantize_bf16_split(const float *x, size_t nvec, size_t n, uint8_t *codes, uint8_t *exps, void *stream) {
    MK_REQUIRE(x && codes && exps, "null pointer");
    MK_REQUIRE(n % 512 == 0 && n <= 0x7FFFFFFFull, "n must be a multiple of 512");
    MK_REQUIRE(((uintptr_t)x & 15) == 0 && ((uintptr_t)codes & 7) == 0, "x must be 16-byte and codes 8-byte aligned");
    const size_t n8 = nvec * (n / 8);
    if (n8 == 0) return MK_OK;
    MK_REQUIRE(n8 <= 0x7fffffffull * 256, "too many values");
    hipLaunchKernelGGL(mk_quantize_bf16_split_kernel, dim3((unsigned)((n8 + 255) / 256)), dim3(256), 0, (hipStream_t)stream, x, n8, (int)n, codes, exps);
    return mk_launch_status("quantize_bf16_split");
}

extern "C" int mk_dev_mxfp4_scales_by_tile(const uint8_t *scales, size_t rows, size_t cols, uint8_t *out, void *stream) {
    MK_REQUIRE(scales && out, "null pointer");
    MK_REQUIRE(cols % 512 == 0, "cols must be a multiple of 512");
    MK_REQUIRE(((uintptr_t)scales & 15) == 0 && ((uintptr_t)out & 15) == 0, "scales and out must be 16-byte aligned");
    const size_t n = rows * (cols / 512);
    if (n == 0) return MK_OK;
    MK_REQUIRE(n <= 0x7fffffffull * 256, "matrix too large");
    hipLaunchKernelGGL(mk_scales_by_tile_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, (const uint4 *)scales,
                       (uint4 *)out, rows, cols / 512);
    return mk_launch_status("mxfp4_scales_by_tile");
}

extern "C" int mk_dev_mxfp4_dequant(const uint8_t *packed, const uint8_t *scales, size_t rows, size_t cols, float *out, void *stream) {
    MK_REQUIRE(packed && scales && out, "null pointer");
    MK_REQUIRE(cols % 32 == 0, "cols must be a multiple of 32");
    MK_REQUIRE(((uintptr_t)packed & 3) == 0 && ((uintptr_t)out & 15) == 0, "packed must be 4-byte and out 16-byte aligned");
    size_t n_words = rows * cols / 8;
    if (n_words == 0) return MK_OK;
    unsigned grid = (unsigned)((n_words + 255) / 256);
    hipLaunchKernelGGL(mk_mxfp4_dequant_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, (const uint32_t *)packed, scales, n_words,
                       out);
    return mk_launch_status("mxfp4_dequant");
}

extern "C" int mk_dev_fp8_dequant(const uint8_t *w, const uint8_t *scales, size_t rows, size_t cols, float *out, void *stream) {
    MK_REQUIRE(w && scales && out, "null pointer");
    MK_REQUIRE(cols % 4 == 0, "cols must be a multiple of 4");
    MK_REQUIRE(((uintptr_t)w & 3) == 0 && ((uintptr_t)out & 15) == 0, "w must be 4-byte and out 16-byte aligned");
    size_t n = rows * cols / 4;
    if (n == 0) return MK_OK;
    unsigned grid = (unsigned)((n + 255) / 256);
    hipLaunchKernelGGL(mk_fp8_dequant_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, w, scales, rows, cols, out);
    return mk_launch_status("fp8_dequant");
}

extern "C" int mk_dev_quantize_q8(const float *x, size_t nvec, size_t n, int8_t *q, float *scales, void *stream) {
    MK_REQUIRE(x && q && scales, "null pointer");
    MK_REQUIRE(n % 32 == 0, "q8 blocks are 32 wide");
    MK_REQUIRE(((uintptr_t)x & 15) == 0 && ((uintptr_t)q & 3) == 0, "x must be 16-byte and q 4-byte aligned");
    size_t n_blocks = nvec * n / 32;
    if (n_blocks == 0) return MK_OK;
    unsigned grid = (unsigned)((n_blocks + 31) / 32);
    hipLaunchKernelGGL(mk_quantize_q8_kernel<false>, dim3(grid), dim3(256), 0, (hipStream_t)stream, x, n_blocks, q, (void *)scales);
    return mk_launch_status("quantize_q8");
}

extern "C" int mk_dev_q8head_from_f32(const float *w, size_t rows, size_t cols, int8_t *q, void *scales, int scales_f16, void *stream) {
    MK_REQUIRE(w && q && scales, "null pointer");
    MK_REQUIRE(cols % 32 == 0, "q8 blocks are 32 wide");
    MK_REQUIRE(((uintptr_t)w & 15) == 0 && ((uintptr_t)q & 3) == 0, "w must be 16-byte and q 4-byte aligned");
    size_t n_blocks = rows * cols / 32;
    if (n_blocks == 0) return MK_OK;
    unsigned grid = (unsigned)((n_blocks + 31) / 32);
    if (scales_f16)
        hipLaunchKernelGGL(mk_quantize_q8_kernel<true>, dim3(grid), dim3(256), 0, (hipStream_t)stream, w, n_blocks, q, scales);
    else
        hipLaunchKernelGGL(mk_quantize_q8_kernel<false>, dim3(grid), dim3(256), 0, (hipStream_t)stream, w, n_blocks, q, scales);
    return mk_launch_status("q8head_from_f32");
}

extern "C" int mk_dev_quantize_mxfp8(const float *x, size_t nvec, size_t n, uint8_t *codes, uint8_t *exps, void *stream) {
    MK_REQUIRE(x && codes && exps, "null pointer");
    MK_REQUIRE(n % 32 == 0, "MXFP8 blocks are 32 wide");
    MK_REQUIRE(((uintptr_t)x & 15) == 0 && ((uintptr_t)codes & 7) == 0, "x must be 16-byte and codes 8-byte aligned");
    size_t n_blocks = nvec * n / 32;
    if (n_blocks == 0) return MK_OK;
    unsigned grid = (unsigned)((n_blocks * 4 + 255) / 256);
    hipLaunchKernelGGL(mk_quantize_mxfp8_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, x, n_blocks, codes, exps);
    return mk_launch_status("quantize_mxfp8");
}

extern "C" int mk_dev_mla_cache_append(const float *latent, const float *rope, size_t L, size_t R, size_t pos, int8_t *lat_q, void *lat_s,
                                       int8_t *rope_q, void *rope_s, void *stream) {
    MK_REQUIRE(latent && rope && lat_q && lat_s && rope_q && rope_s, "null pointer");
    MK_REQUIRE(L % 32 == 0 && R % 32 == 0, "q8 blocks are 32 wide");
    MK_REQUIRE(((uintptr_t)latent & 15) == 0 && ((uintptr_t)rope & 15) == 0 && ((uintptr_t)lat_q & 3) == 0 && ((uintptr_t)rope_q & 3) == 0,
               "latent and rope must be 16-byte, the cache rows 4-byte aligned");
    unsigned g1 = (unsigned)((L / 32 + 31) / 32), g2 = (unsigned)((R / 32 + 31) / 32);
    hipLaunchKernelGGL(mk_quantize_q8_kernel<true>, dim3(g1), dim3(256), 0, (hipStream_t)stream, latent, L / 32, lat_q + pos * L,
                       (void *)((uint16_t *)lat_s + pos * (L / 32)));
    hipLaunchKernelGGL(mk_quantize_q8_kernel<true>, dim3(g2), dim3(256), 0, (hipStream_t)stream, rope, R / 32, rope_q + pos * R,
                       (void *)((uint16_t *)rope_s + pos * (R / 32)));
    return mk_launch_status("mla_cache_append");
}
