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

}  // namespace

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
