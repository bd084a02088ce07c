// VQ1 matvec (quant::matvec_vq, src/quant.rs:313-346) as the LUT GEMV of src/lutgemv.rs:208-240 on gfx950.
//
// Weights are vectors of 16 consecutive row-major values, each replaced by one index byte into a 256 x 16 f32
// codebook shared by all VQ1 tensors: a 2048 x 7168 matrix is 917 504 index bytes.  The products that can occur
// are computed once per activation: lut[g][k] = dot(codebook[k], x[16g .. 16g+16]), 256 entries per group of 16
// columns; a row is then the sum over its groups of lut[g][index].
//
//   table   one workgroup per group, thread k forms entry k with the reference's sequential chain (multiply, then
//           add, ascending j, from 0): every entry is bit-identical to build_vq_lut_scalar (src/lutgemv.rs:175-185).
//   sweep   fast: a wave per row, lane l adds the groups l, l + 64, ... in ascending order and the 64 partial sums
//           are reduced across the wave (the order of the sum over groups differs from the reference);
//           exact: a lane per row adds its groups in ascending order from 0, as sweep (src/lutgemv.rs:67-98) does:
//           bit-identical to the reference, which is itself bit-identical to matvec_vq_gather.
//
// The table (cols/16 KiB) and the index rows stay in the L2; the kernels are latency- and launch-bound, not HBM-bound.
// The batched form for prefill, matvec_vq_nt, is the last kernel of this file.
#include "mk_common.h"

namespace {

__global__ __launch_bounds__(256) void vq1_table_kernel(const float *__restrict__ codebook, const float *__restrict__ x, float *__restrict__ lut) {
    __shared__ float xs[16];
    const int g = blockIdx.x, k = threadIdx.x;
    if (k < 16) xs[k] = x[g * 16 + k];
    __syncthreads();
    const mk_f4 *cb = reinterpret_cast<const mk_f4 *>(codebook + k * 16);
    float s = 0.0f;
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const mk_f4 c = cb[q];
        s = mk_add(s, mk_mul(c.x, xs[q * 4 + 0]));
        s = mk_add(s, mk_mul(c.y, xs[q * 4 + 1]));
        s = mk_add(s, mk_mul(c.z, xs[q * 4 + 2]));
        s = mk_add(s, mk_mul(c.w, xs[q * 4 + 3]));
    }
    lut[g * 256 + k] = s;
}

__global__ __launch_bounds__(256) void vq1_sweep_fast_kernel(const float *__restrict__ lut, const uint8_t *__restrict__ indices, int rows, int vpr,
                                                             float *__restrict__ out) {
    const int lane = threadIdx.x & 63;
    const int r = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= rows) return;  // whole waves leave together
    const uint8_t *ir = indices + (size_t)r * vpr;
    float a = 0.0f;
    for (int g0 = 0; g0 < vpr; g0 += 256) {  // four gathers in flight per lane
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int g = g0 + i * 64 + lane;
            v[i] = g < vpr ? lut[g * 256 + ir[g]] : 0.0f;
        }
#pragma unroll
        for (int i = 0; i < 4; i++) a += v[i];
    }
    a = mk_wave_sum(a);
    if (lane == 0) out[r] = a;
}

__global__ __launch_bounds__(64) void vq1_sweep_exact_kernel(const float *__restrict__ lut, const uint8_t *__restrict__ indices, int rows, int vpr,
                                                             float *__restrict__ out) {
    const int r = blockIdx.x * 64 + threadIdx.x;
    if (r >= rows) return;
    const uint8_t *ir = indices + (size_t)r * vpr;
    float a = 0.0f;
    for (int g0 = 0; g0 < vpr; g0 += 16) {  // sixteen gathers in flight, then the additions in order
        float v[16];
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int g = min(g0 + i, vpr - 1);
            v[i] = lut[g * 256 + ir[g]];
        }
#pragma unroll
        for (int i = 0; i < 16; i++)
            if (g0 + i < vpr) a = mk_add(a, v[i]);
    }
    out[r] = a;
}

// Grouped forms for a MoE layer with VQ1 experts (src/model.rs:2243-2257): matrix p of a launch is the index bytes
// idx_ptrs[p]; it belongs to this path when marker_ptrs[p] is null (an MXFP4 matrix has its scale bytes there).
// tables: vector v of `x` (n_vec x cols) -> lut + v * (cols / 16) * 256; sweep: matrix p reads the table of vector
// vec_index[p] (p itself when vec_index is null).
__global__ __launch_bounds__(256) void vq1_table_grouped_kernel(const float *__restrict__ codebook, const float *__restrict__ x, int cols,
                                                                const uint8_t *const *__restrict__ marker_ptrs, float *__restrict__ lut) {
    __shared__ float xs[16];
    const int g = blockIdx.x, v = blockIdx.y, k = threadIdx.x;
    if (marker_ptrs && marker_ptrs[v]) return;
    if (k < 16) xs[k] = x[(size_t)v * cols + g * 16 + k];
    __syncthreads();
    const mk_f4 *cb = reinterpret_cast<const mk_f4 *>(codebook + k * 16);
    float s = 0.0f;
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const mk_f4 c = cb[q];
        s = mk_add(s, mk_mul(c.x, xs[q * 4 + 0]));
        s = mk_add(s, mk_mul(c.y, xs[q * 4 + 1]));
        s = mk_add(s, mk_mul(c.z, xs[q * 4 + 2]));
        s = mk_add(s, mk_mul(c.w, xs[q * 4 + 3]));
    }
    lut[((size_t)v * (cols / 16) + g) * 256 + k] = s;
}

__global__ __launch_bounds__(256) void vq1_sweep_grouped_kernel(const float *__restrict__ lut, const int32_t *__restrict__ vec_index,
                                                                const uint8_t *const *__restrict__ idx_ptrs,
                                                                const uint8_t *const *__restrict__ marker_ptrs, int rows, int vpr,
                                                                float *const *__restrict__ out_ptrs) {
    const int p = blockIdx.y;
    if (marker_ptrs[p]) return;
    const int lane = threadIdx.x & 63;
    const int r = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= rows) return;  // whole waves leave together
    const float *tab = lut + (size_t)(vec_index ? vec_index[p] : p) * vpr * 256;
    const uint8_t *ir = idx_ptrs[p] + (size_t)r * vpr;
    float a = 0.0f;
    for (int g0 = 0; g0 < vpr; g0 += 256) {  // four gathers in flight per lane
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int g = g0 + i * 64 + lane;
            v[i] = g < vpr ? tab[g * 256 + ir[g]] : 0.0f;
        }
#pragma unroll
        for (int i = 0; i < 4; i++) a += v[i];
    }
    a = mk_wave_sum(a);
    if (lane == 0) out_ptrs[p][r] = a;
}

// quant::matvec_vq_nt (src/quant.rs:353-376): m positions at once, every product added to its position's running sum in
// (vector, j) order -- one sequential chain of cols multiply-adds per (row, position), not the per-vector partial sums of
// matvec_vq.  A lane owns a row and 8 positions (the reference's block of 8): the codebook entry is gathered from LDS
// (entries 20 floats apart, so that the 16-byte reads of different entries spread over the banks), the 8 activations of
// a (vector, j) are the same for every lane (uniform loads).  Multiply, then add, never fused: bit-identical.
constexpr int CB_STRIDE = 20;
template <bool QUAD>  // QUAD: cols / 16 is a multiple of 4 and the index rows are 4-byte aligned: four index bytes per load
__global__ __launch_bounds__(256) void vq1_nt_kernel(const float *__restrict__ codebook, const uint8_t *__restrict__ indices, int rows, int vpr,
                                                     const float *__restrict__ xt, int m, float *__restrict__ out) {
    __shared__ __attribute__((aligned(16))) float cb[256 * CB_STRIDE];
    for (int i = threadIdx.x; i < 256 * 4; i += 256)
        *reinterpret_cast<mk_f4 *>(cb + (i >> 2) * CB_STRIDE + (i & 3) * 4) = reinterpret_cast<const mk_f4 *>(codebook)[i];
    __syncthreads();
    const int r = blockIdx.x * 256 + threadIdx.x, t0 = blockIdx.y * 8;
    const uint8_t *ir = indices + (size_t)min(r, rows - 1) * vpr;
    float sum[8];
#pragma unroll
    for (int p = 0; p < 8; p++) sum[p] = 0.0f;
    auto vec = [&](int v, int idx) {
        const float *e = cb + idx * CB_STRIDE;
        const mk_f4 c0 = *reinterpret_cast<const mk_f4 *>(e), c1 = *reinterpret_cast<const mk_f4 *>(e + 4);
        const mk_f4 c2 = *reinterpret_cast<const mk_f4 *>(e + 8), c3 = *reinterpret_cast<const mk_f4 *>(e + 12);
        const float c[16] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w, c2.x, c2.y, c2.z, c2.w, c3.x, c3.y, c3.z, c3.w};
        const float *xv = xt + (size_t)v * 16 * m + t0;  // the same address in every lane
#pragma unroll
        for (int j = 0; j < 16; j++) {
            const mk_f4 xa = *reinterpret_cast<const mk_f4 *>(xv + (size_t)j * m), xb = *reinterpret_cast<const mk_f4 *>(xv + (size_t)j * m + 4);
            sum[0] = mk_add(sum[0], mk_mul(c[j], xa.x));
            sum[1] = mk_add(sum[1], mk_mul(c[j], xa.y));
            sum[2] = mk_add(sum[2], mk_mul(c[j], xa.z));
            sum[3] = mk_add(sum[3], mk_mul(c[j], xa.w));
            sum[4] = mk_add(sum[4], mk_mul(c[j], xb.x));
            sum[5] = mk_add(sum[5], mk_mul(c[j], xb.y));
            sum[6] = mk_add(sum[6], mk_mul(c[j], xb.z));
            sum[7] = mk_add(sum[7], mk_mul(c[j], xb.w));
        }
    };
    if constexpr (QUAD) {
        uint32_t nxt = *reinterpret_cast<const uint32_t *>(ir);
        for (int v = 0; v < vpr; v += 4) {
            const uint32_t cur = nxt;
            nxt = *reinterpret_cast<const uint32_t *>(ir + min(v + 4, vpr - 4));  // one load ahead
#pragma unroll
            for (int k = 0; k < 4; k++) vec(v + k, (int)((cur >> (8 * k)) & 0xFF));
        }
    } else {
        for (int v = 0; v < vpr; v++) vec(v, (int)ir[v]);
    }
    if (r < rows) {
#pragma unroll
        for (int p = 0; p < 8; p++) out[(size_t)(t0 + p) * rows + r] = sum[p];
    }
}

}  // namespace

extern "C" int mk_dev_vq1_matvec_nt(const float *codebook, const uint8_t *indices, size_t rows, size_t cols, const float *xt, size_t m, float *out,
                                    void *stream) {
    MK_REQUIRE(codebook && indices && xt && out, "null pointer");
    MK_REQUIRE(cols % 16 == 0 && cols > 0, "cols must be a positive multiple of 16");
    MK_REQUIRE(m % 8 == 0, "m must be a multiple of 8 (the reference's position blocks)");
    MK_REQUIRE(rows <= 0x7FFFFF00u && cols <= (1u << 24) && m / 8 <= 65535, "shape too large");
    MK_REQUIRE(((uintptr_t)codebook & 15) == 0 && ((uintptr_t)xt & 15) == 0, "codebook and xt must be 16-byte aligned");
    if (rows == 0 || m == 0) return MK_OK;
    const dim3 grid((unsigned)((rows + 255) / 256), (unsigned)(m / 8));
    if ((cols / 16) % 4 == 0 && ((uintptr_t)indices & 3) == 0)
        hipLaunchKernelGGL(vq1_nt_kernel<true>, grid, dim3(256), 0, (hipStream_t)stream, codebook, indices, (int)rows, (int)(cols / 16), xt, (int)m, out);
    else
        hipLaunchKernelGGL(vq1_nt_kernel<false>, grid, dim3(256), 0, (hipStream_t)stream, codebook, indices, (int)rows, (int)(cols / 16), xt, (int)m, out);
    return mk_launch_status("vq1_nt");
}

int mk_vq1_grouped_tables(const float *codebook, const float *x, size_t n_vec, size_t cols, const uint8_t *const *marker_ptrs, float *lut,
                          hipStream_t st) {
    if (n_vec == 0) return MK_OK;
    hipLaunchKernelGGL(vq1_table_grouped_kernel, dim3((unsigned)(cols / 16), (unsigned)n_vec), dim3(256), 0, st, codebook, x, (int)cols, marker_ptrs,
                       lut);
    return mk_launch_status("vq1_table_grouped");
}

int mk_vq1_grouped_sweep(const float *lut, const int32_t *vec_index, const uint8_t *const *idx_ptrs, const uint8_t *const *marker_ptrs,
                         size_t n_mat, size_t rows, size_t cols, float *const *out_ptrs, hipStream_t st) {
    if (n_mat == 0 || rows == 0) return MK_OK;
    hipLaunchKernelGGL(vq1_sweep_grouped_kernel, dim3((unsigned)((rows + 3) / 4), (unsigned)n_mat), dim3(256), 0, st, lut, vec_index, idx_ptrs,
                       marker_ptrs, (int)rows, (int)(cols / 16), out_ptrs);
    return mk_launch_status("vq1_sweep_grouped");
}

extern "C" size_t mk_vq1_workspace_bytes(size_t cols) { return cols / 16 * 256 * sizeof(float); }

extern "C" int mk_dev_vq1_matvec(const float *codebook, const uint8_t *indices, size_t rows, size_t cols, const float *x, int exact,
                                 void *workspace, float *out, void *stream) {
    MK_REQUIRE(codebook && indices && x && workspace && out, "null pointer");
    MK_REQUIRE(cols % 16 == 0 && cols > 0, "cols must be a positive multiple of 16");
    MK_REQUIRE(rows <= 0x7FFFFF00u && cols <= (1u << 24), "shape too large");
    MK_REQUIRE(((uintptr_t)codebook & 15) == 0 && ((uintptr_t)workspace & 15) == 0, "codebook and workspace must be 16-byte aligned");
    if (rows == 0) return MK_OK;
    hipStream_t st = (hipStream_t)stream;
    const int vpr = (int)(cols / 16);
    float *lut = reinterpret_cast<float *>(workspace);
    hipLaunchKernelGGL(vq1_table_kernel, dim3(vpr), dim3(256), 0, st, codebook, x, lut);
    int s = mk_launch_status("vq1_table");
    if (s != MK_OK) return s;
    if (exact)
        hipLaunchKernelGGL(vq1_sweep_exact_kernel, dim3((unsigned)((rows + 63) / 64)), dim3(64), 0, st, lut, indices, (int)rows, vpr, out);
    else
        hipLaunchKernelGGL(vq1_sweep_fast_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, st, lut, indices, (int)rows, vpr, out);
    return mk_launch_status("vq1_sweep");
}
