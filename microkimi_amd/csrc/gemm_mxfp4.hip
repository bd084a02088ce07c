// Prefill expert GEMM: the per-expert batched evaluation of moe_prefill
// (src/model.rs:2539-2602) on the gfx950 block-scaled matrix cores.
//
//   y[i][r] = sum_k W_e[r][k] * x[i][k]      for the token rows i of group e
//
// v_mfma_scale_f32_16x16x128_f8f6f4 multiplies a 16x128 by a 128x16 tile with
// one e8m0 scale per 32 K-elements on each side -- the MXFP4 weight format as
// it is stored: a lane's B operand is the 16 bytes (32 nibbles) of ONE block of
// one weight row and its scale byte, loaded straight from the reference layout.
// The A operand is the activation in MXFP8 (e4m3 codes + e8m0 per 32), 32 bytes
// per lane.  Accumulation is f32 in the matrix core.
//
// Operand layout of the instruction (measured on the device with one-hot
// operands, both formats):
//   scales        lane i + 16 b supplies the e8m0 byte of row/column i, K block b (k in [32 b, 32 b + 32))
//   4-bit operand lane i + 16 b holds k = 32 b + j in registers 0-3, nibble j (low nibble first): one MXFP4 block
//   8-bit operand lane i + 16 g holds k = 16 g + j in registers 0-3 (bytes 0-15) and k = 64 + 16 g + j in
//                 registers 4-7 (bytes 16-31): the K = 128 step is two K = 64 halves
//   result        lane l holds column l % 16, rows 4 (l / 16) + r
//
// Tiling: workgroup = 4 waves = 64 weight rows of one expert; each wave owns 16
// rows and up to 64 token rows (4 accumulator tiles), so an expert's weights are
// streamed from HBM once for up to 64 tokens.  At the prefill shapes (about 16
// tokens per expert) the kernel is bound by that weight stream, not by the MFMA.
#include "mk_common.h"

namespace {

constexpr int MC = 4;  // 16-token accumulator tiles per wave

__global__ __launch_bounds__(256) void mxfp4_grouped_gemm_kernel(const uint8_t *const *__restrict__ packed_ptrs,
                                                                 const uint8_t *const *__restrict__ scales_ptrs, int rows, int cols,
                                                                 const uint8_t *__restrict__ codes, const uint8_t *__restrict__ exps,
                                                                 const int32_t *__restrict__ offsets, float *__restrict__ out) {
    const int e = blockIdx.y;
    const int tok0 = offsets[e], tok1 = offsets[e + 1];
    if (tok1 <= tok0) return;
    const uint8_t *packed = packed_ptrs[e];
    const uint8_t *scales = scales_ptrs[e];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = lane & 15, kb = lane >> 4;
    const int nb = cols / 32, steps = cols / 128;
    const int row = blockIdx.x * 64 + wave * 16 + n;
    const bool row_ok = row < rows;
    const uint8_t *wrow = packed + (size_t)(row_ok ? row : 0) * (cols / 2) + kb * 16;
    const uint8_t *srow = scales + (size_t)(row_ok ? row : 0) * nb + kb;

    for (int base = tok0; base < tok1; base += 16 * MC) {
        const int ntok = min(16 * MC, tok1 - base);
        const int nchunk = (ntok + 15) / 16;
        mk_f4 acc[MC];
#pragma unroll
        for (int c = 0; c < MC; c++) acc[c] = mk_f4{0.0f, 0.0f, 0.0f, 0.0f};
        // A rows of this lane: token base + c*16 + n (clamped; rows past the group are discarded at the store)
        const uint8_t *arow[MC];
        const uint8_t *aexp[MC];
#pragma unroll
        for (int c = 0; c < MC; c++) {
            const int t = min(base + c * 16 + n, tok1 - 1);
            arow[c] = codes + (size_t)t * cols + kb * 16;
            aexp[c] = exps + (size_t)t * nb + kb;
        }
        for (int s = 0; s < steps; s++) {
            const mk_i4 wv = *reinterpret_cast<const mk_i4 *>(wrow + s * 64);
            const int wsb = srow[s * 4];
            mk_i8v b = {wv[0], wv[1], wv[2], wv[3], 0, 0, 0, 0};
#pragma unroll
            for (int c = 0; c < MC; c++) {
                if (c < nchunk) {
                    const mk_i4 a0 = *reinterpret_cast<const mk_i4 *>(arow[c] + s * 128);
                    const mk_i4 a1 = *reinterpret_cast<const mk_i4 *>(arow[c] + s * 128 + 64);
                    const int asb = aexp[c][s * 4];
                    mk_i8v a = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
                    acc[c] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, acc[c], 0 /*A: fp8 e4m3*/, 4 /*B: fp4 e2m1*/, 0, asb, 0, wsb);
                }
            }
        }
        if (row_ok) {
#pragma unroll
            for (int c = 0; c < MC; c++) {
                if (c < nchunk) {
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const int t = base + c * 16 + kb * 4 + i;
                        if (t < tok1) out[(size_t)t * rows + row] = acc[c][i];
                    }
                }
            }
        }
    }
}

}  // namespace

extern "C" int mk_dev_mxfp4_grouped_gemm(const uint8_t *const *packed_ptrs, const uint8_t *const *scales_ptrs, size_t n_groups, size_t rows,
                                         size_t cols, const uint8_t *codes, const uint8_t *exps, const int32_t *offsets, size_t m, float *out,
                                         void *stream) {
    MK_REQUIRE(packed_ptrs && scales_ptrs && codes && exps && offsets && out, "null pointer");
    MK_REQUIRE(cols % 128 == 0 && cols > 0, "cols must be a positive multiple of 128");
    MK_REQUIRE(n_groups >= 1 && n_groups <= 65535 && rows >= 1 && rows <= 0x7FFFFF00u, "bad shape");
    MK_REQUIRE(((uintptr_t)codes & 15) == 0, "codes must be 16-byte aligned");
    if (m == 0) return MK_OK;
    hipLaunchKernelGGL(mxfp4_grouped_gemm_kernel, dim3((unsigned)((rows + 63) / 64), (unsigned)n_groups), dim3(256), 0, (hipStream_t)stream,
                       packed_ptrs, scales_ptrs, (int)rows, (int)cols, codes, exps, offsets, out);
    return mk_launch_status("mxfp4_grouped_gemm");
}
