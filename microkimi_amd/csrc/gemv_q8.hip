// q8_0 GEMV (Q8Head::matvec, src/model.rs:290-347) for gfx950: int8 weights
// [rows][cols] + one scale per 32 (f16 storage form or f32), q8 activations.
//
// out[b][r] = sum_g (ws[r][g] * xs[b][g]) * idot(r, b, g), idot exact int32.
//
// batch 1   VALU path.  Lane l of wave iteration t owns the 16-byte half block
//           t*64+l of the row (perfectly coalesced 1 KiB wave loads, no repack)
//           and keeps the matching 16 activation bytes and block scale in
//           registers for the whole kernel; 4 x v_dot4_i32_i8 per load.
// batch 2-3 at 7168 columns: the batch-1 streaming pattern with the activation in
//           LDS and two rows per LDS read (see q8_gemv_bn_kernel).
// batch 2-8 matrix-core path (batch 4-8 at 7168 columns, 2-8 elsewhere; 219 -> 197 us at batch 8 since the loads take
//           whole lines).  One v_mfma_i32_16x16x64_i8 per 16 rows x 64
//           columns.  The MFMA sums over K = 64 = two q8 blocks, whose scales
//           differ, so the activation operand is laid out as 16 "columns" =
//           8 batch rows x 2 block parities, each holding the activation bytes of
//           one block and zeros for the other: the 16x16 result then holds the
//           per-block integer dots, and the per-block scale product is applied in
//           f32 exactly as the reference does.  Weights are read once for the
//           whole batch.
// generic   one wave per row, any cols % 32 == 0, any batch <= 8.
#include <stdlib.h>

#include "mk_common.h"

namespace {

template <bool F16>
__device__ __forceinline__ float load_scale(const void *scales, size_t idx) {
    if (F16) return mk_f16_bits_to_f32(mk_ldg_u16(reinterpret_cast<const uint16_t *>(scales) + idx));
    return mk_ldg_f32(reinterpret_cast<const float *>(scales) + idx);
}

// ------------------------------------------------------------- batch 1
// Rows are dealt round-robin to a fixed number of resident waves: wave w takes
// rows w, w + W, w + 2W, ...  Every wave has the same amount of work (no tail)
// and at any moment the chip reads one compact window of W consecutive rows.
template <int NB, bool F16>
__global__ __launch_bounds__(256) void q8_gemv_b1_kernel(const int8_t *__restrict__ q, const void *__restrict__ scales, int rows,
                                                         const int8_t *__restrict__ xq, const float *__restrict__ xs,
                                                         float *__restrict__ out) {
    constexpr int T = NB * 2 / 64;  // half blocks per row / 64 lanes
    static_assert(NB % 32 == 0 && T >= 1 && T <= 8, "row shape not covered by the fast path");
    const int lane = threadIdx.x & 63;
    const int wave = blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n_waves = gridDim.x * 4;
    mk_i4 xr[T];
    float cf[T];
#pragma unroll
    for (int t = 0; t < T; t++) {
        const int hb = t * 64 + lane;
        xr[t] = *reinterpret_cast<const mk_i4 *>(xq + hb * 16);
        cf[t] = xs[hb >> 1];
    }
    mk_i4 w[T];
    float ws[T];
    // two rows in flight (ping, pong); prefetches are unconditional, past the
    // end they re-read the last row (a load under a branch forces a full wait)
    mk_i4 wa[T], wb[T];
    float sa[T], sb[T];
    // uniform base + 32-bit lane offsets (the host checks rows * cols < 2^32): scalar-base loads; the row
    // index is uniform per wave and goes through readfirstlane so that it stays on the scalar unit
    auto load_row = [&](mk_i4 *w, float *ws, int r) {
        const uint32_t ru = (uint32_t)__builtin_amdgcn_readfirstlane(min(r, rows - 1));
        const uint32_t qoff = ru * (NB * 32) + lane * 16, soff = ru * NB + (lane >> 1);
#pragma unroll
        for (int t = 0; t < T; t++) {
            w[t] = mk_ldg128_off_nt(q, qoff + t * 1024);  // streamed once: non-temporal (measured 207 -> 179 us on the lm_head)
            if (F16) ws[t] = mk_f16_bits_to_f32(mk_ldg_u16_off(scales, (soff + t * 32) * 2));
            else ws[t] = mk_ldg_f32_off(scales, (soff + t * 32) * 4);
        }
    };
    auto compute_row = [&](const mk_i4 *w, const float *ws, int r) {
        float acc = 0.0f;
#pragma unroll
        for (int t = 0; t < T; t++) {
            int d = 0;
#pragma unroll
            for (int k = 0; k < 4; k++) d = __builtin_amdgcn_sdot4(w[t][k], xr[t][k], d, false);
            acc += (ws[t] * cf[t]) * (float)d;
        }
        acc = mk_wave_sum(acc);
        if (lane == 0 && r < rows) out[r] = acc;
    };
    load_row(wa, sa, wave);
    for (int r = wave; r < rows; r += 2 * n_waves) {
        load_row(wb, sb, r + n_waves);
        compute_row(wa, sa, r);
        load_row(wa, sa, r + 2 * n_waves);
        compute_row(wb, sb, r + n_waves);
    }
}

// -------------------------------------------------- batch 2..3, long rows
// The batch-1 streaming pattern (a wave reads whole rows, 1 KiB per load, non-
// temporal, rows dealt round-robin to a resident grid) with the batch's
// activation bytes and block scales in LDS: two rows are in the registers at a
// time, so that every 16 activation bytes read from LDS meet two weight rows.
// 4 x v_dot4_i32_i8 per (half block, batch column), the per-block term in f32 as
// the reference writes it.  At 7168 columns this reads the matrix at the batch-1
// rate; the matrix-core kernel below, whose lanes take 64 bytes of a row per
// load, stays for the other row lengths.
template <int NB, bool F16, int BATCH>
__global__ __launch_bounds__(256, 2) void q8_gemv_bn_kernel(const int8_t *__restrict__ q, const void *__restrict__ scales, int rows,
                                                         const int8_t *__restrict__ xq, const float *__restrict__ xs,
                                                         float *__restrict__ out) {
    constexpr int T = NB * 2 / 64;
    static_assert(NB % 32 == 0 && T >= 1 && T <= 8, "row shape not covered");
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    mk_i4 *xl = reinterpret_cast<mk_i4 *>(lds);                            // [BATCH][NB * 2] half blocks
    float *xsl = reinterpret_cast<float *>(lds + (size_t)BATCH * NB * 32);  // [BATCH][NB]
    for (int i = threadIdx.x; i < BATCH * NB * 2; i += 256) xl[i] = reinterpret_cast<const mk_i4 *>(xq)[i];
    for (int i = threadIdx.x; i < BATCH * NB; i += 256) xsl[i] = xs[i];

    const int lane = threadIdx.x & 63;
    const int wave = blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n_waves = gridDim.x * 4;
    struct Row {
        mk_i4 w[T];
        float s[T];
    };
    auto load_row = [&](Row &R, int r) {
        const uint32_t ru = (uint32_t)__builtin_amdgcn_readfirstlane(min(r, rows - 1));  // past the end: the last row again
        const uint32_t qoff = ru * (NB * 32) + lane * 16, soff = ru * NB + (lane >> 1);
#pragma unroll
        for (int t = 0; t < T; t++) {
            R.w[t] = mk_ldg128_off_nt(q, qoff + t * 1024);
            if (F16) R.s[t] = mk_f16_bits_to_f32(mk_ldg_u16_off(scales, (soff + t * 32) * 2));
            else R.s[t] = mk_ldg_f32_off(scales, (soff + t * 32) * 4);
        }
    };
    auto compute_rows = [&](const Row &A, const Row &Bq, int r0, int r1) {
        float acc0[BATCH], acc1[BATCH];
#pragma unroll
        for (int b = 0; b < BATCH; b++) acc0[b] = acc1[b] = 0.0f;
        // (t, b) steps with the next step's LDS operands requested one step ahead
        // the activation does not change from row to row: without an opaque index the compiler keeps all of it in
        // registers (408 at batch 8) instead of reading LDS
        int z = lane;
        asm volatile("" : "+v"(z));
        mk_i4 xv = xl[z];
        float cf = xsl[z >> 1];
#pragma unroll
        for (int i = 0; i < T * BATCH; i++) {
            const int t = i / BATCH, b = i % BATCH;
            const int tn = (i + 1) / BATCH, bn = (i + 1) % BATCH;
            mk_i4 xn = xv;
            float cn = cf;
            if (i + 1 < T * BATCH) {
                xn = xl[bn * NB * 2 + tn * 64 + z];
                cn = xsl[bn * NB + ((tn * 64 + z) >> 1)];
            }
            int d0 = 0, d1 = 0;
#pragma unroll
            for (int k = 0; k < 4; k++) {
                d0 = __builtin_amdgcn_sdot4(A.w[t][k], xv[k], d0, false);
                d1 = __builtin_amdgcn_sdot4(Bq.w[t][k], xv[k], d1, false);
            }
            acc0[b] += (A.s[t] * cf) * (float)d0;
            acc1[b] += (Bq.s[t] * cf) * (float)d1;
            xv = xn;
            cf = cn;
            // the index of the following reads is made to depend on this step's dots: one step of operands in flight
            asm volatile("" : "+v"(z) : "v"(d0), "v"(d1));
        }
#pragma unroll
        for (int b = 0; b < BATCH; b++) {
            const float v0 = mk_wave_sum(acc0[b]), v1 = mk_wave_sum(acc1[b]);
            if (lane == 0) {
                if (r0 < rows) out[(size_t)b * rows + r0] = v0;
                if (r1 < rows) out[(size_t)b * rows + r1] = v1;
            }
        }
    };
    Row a0, a1, b0, b1;
    load_row(a0, wave);
    load_row(a1, wave + n_waves);
    __syncthreads();
    for (int r = wave; r < rows; r += 4 * n_waves) {
        load_row(b0, r + 2 * n_waves);
        load_row(b1, r + 3 * n_waves);
        compute_rows(a0, a1, r, r + n_waves);
        load_row(a0, r + 4 * n_waves);
        load_row(a1, r + 5 * n_waves);
        if (r + 2 * n_waves < rows) compute_rows(b0, b1, r + 2 * n_waves, r + 3 * n_waves);
    }
}

// ------------------------------------------------------- batch 2..8 (MFMA)
// Workgroup of WAVES waves; LDS holds the batch's activation bytes in operand
// order ([K/16 chunks][8 batch rows][16 bytes]), the activation block scales
// ([NB][8]) and, per wave, the weight scales of the 16-row group the wave is
// working on.  The scales of 16 consecutive rows are one contiguous range:
// they are fetched with seven fully coalesced 1 KiB loads, one group ahead,
// and read back from LDS per step -- scattered 2-byte global loads per step cost
// a cache line each and halved the bandwidth.
template <bool F16, int WAVES, bool FULL>
__global__ __launch_bounds__(WAVES * 64) void q8_gemv_mfma_kernel(const int8_t *__restrict__ q, const void *__restrict__ scales, int rows,
                                                                  int nb, const int8_t *__restrict__ xq, const float *__restrict__ xs,
                                                                  int batch, float *__restrict__ out) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    constexpr int SB = F16 ? 2 : 4;  // bytes per weight scale
    constexpr int NIT = F16 ? 8 : 16;  // 1 KiB wave loads covering the scales of one group (nb <= 256)
    const int cols = nb * 32;
    mk_i4 *xl = reinterpret_cast<mk_i4 *>(lds);                      // [cols/16][8]
    float *xsl = reinterpret_cast<float *>(lds + (size_t)cols * 8);  // [nb][8]
    const int group_bytes = 16 * nb * SB;
    // A row of the wave's scale tile takes row_bytes + 4 in LDS when the row is a whole number of 16-byte chunks: the
    // 16 rows a step's 2-byte reads touch then start in different banks (at 448 bytes a row they fell on four).
    const int row_bytes = nb * SB, cpr = row_bytes / 16;
    const bool padded = (row_bytes & 15) == 0;
    const int row_stride = padded ? row_bytes + 4 : row_bytes;
    uint8_t *sl = lds + (size_t)cols * 8 + (size_t)nb * 32 + (size_t)(threadIdx.x >> 6) * (group_bytes + 64);  // this wave's scale tile
    for (int i = threadIdx.x; i < (cols / 16) * 8; i += WAVES * 64) {
        const int c = i >> 3, b = i & 7;
        mk_i4 v = {0, 0, 0, 0};
        if (b < batch) v = *reinterpret_cast<const mk_i4 *>(xq + (size_t)b * cols + c * 16);
        xl[i] = v;
    }
    for (int i = threadIdx.x; i < nb * 8; i += WAVES * 64) {
        const int g = i >> 3, b = i & 7;
        xsl[i] = b < batch ? xs[(size_t)b * nb + g] : 0.0f;
    }
    __syncthreads();

    const int lane = threadIdx.x & 63;
    const int n = lane & 15;   // weight row inside the group (B operand column / result column)
    const int kb = lane >> 4;  // 16-byte K chunk inside the 64-wide step; also the result row group
    const int par = kb >> 1;   // which of the step's two q8 blocks this lane's result rows belong to
    const int a_batch = n & 7, a_par = n >> 3;  // A operand row m = n: batch row and block parity
    const bool a_live = (kb >> 1) == a_par;
    const int steps = nb / 2;
    const int wave = blockIdx.x * WAVES + (threadIdx.x >> 6);
    const int n_waves = gridDim.x * WAVES;
    const int n_groups = (rows + 15) / 16;
    const size_t scale_bytes = (size_t)rows * nb * SB;
    constexpr int S = 8;  // K steps per register block; two blocks (ping, pong) are in flight per lane

    mk_i4 spre[NIT];  // scales of the next group, in flight while the current group is computed
    auto prefetch_scales = [&](int grp) {
        const size_t base = (size_t)grp * group_bytes;
#pragma unroll
        for (int it = 0; it < NIT; it++) {
            const size_t off = (size_t)(it * 64 + lane) * 16;
            spre[it] = (off < (size_t)group_bytes && base + off + 16 <= scale_bytes)
                           ? *reinterpret_cast<const mk_i4 *>(reinterpret_cast<const uint8_t *>(scales) + base + off)
                           : mk_i4{0, 0, 0, 0};
        }
    };
    int soff[NIT];  // where chunk it * 64 + lane of a group's scales goes in the tile
#pragma unroll
    for (int it = 0; it < NIT; it++) {
        const int c = it * 64 + lane;
        soff[it] = padded ? (c / cpr) * row_stride + (c % cpr) * 16 : c * 16;
    }
    if (wave < n_groups) prefetch_scales(wave);
    // 16-row groups are dealt round-robin to the resident waves
    for (int grp = wave; grp < n_groups; grp += n_waves) {
#pragma unroll
        for (int it = 0; it < NIT; it++) {
            const int off = (it * 64 + lane) * 16;
            if (off < group_bytes) {
                // (a padded row starts 4 bytes later than the one before: the chunk is stored as four words)
                uint32_t *dst = reinterpret_cast<uint32_t *>(sl + soff[it]);
                dst[0] = (uint32_t)spre[it][0], dst[1] = (uint32_t)spre[it][1], dst[2] = (uint32_t)spre[it][2], dst[3] = (uint32_t)spre[it][3];
            }
        }
        if (grp + n_waves < n_groups) prefetch_scales(grp + n_waves);
        const int row = grp * 16 + n;
        const bool row_ok = row < rows;
        const int8_t *wrow = q + (size_t)(row_ok ? row : 0) * cols + kb * 16;
        // FULL (cols % 128 == 0): a load takes whole 128-byte lines, 8 rows x 128 bytes (lane (r3 = lane / 8, c = lane % 8)
        // reads bytes 16c .. of row 8h + r3; loads 2i and 2i + 1 of a block cover line i of rows 0-7 and 8-15), and the
        // operand form (16 rows x 64 bytes per step, lane (kb, n)) is restored in registers: a rotation of the lane
        // index by three bits, then the two registers exchange the 8-lane halves of every 16-lane row.  With the
        // operand's own mapping every line is requested by two loads.
        const int8_t *wline[2];
#pragma unroll
        for (int h = 0; h < 2; h++) wline[h] = q + (size_t)min(grp * 16 + 8 * h + (lane >> 3), rows - 1) * cols + (lane & 7) * 16;
        const int rot_idx = (((lane & 7) << 3) | (((lane >> 3) & 1) << 2) | (lane >> 4)) * 4;
        const uint8_t *srow = sl + (size_t)n * row_stride + (size_t)par * SB;
        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        mk_i4 wa[S], wb[S];
        auto load_block = [&](mk_i4 *wv, int s0) {
#pragma unroll
            for (int j = 0; j < S; j++) {
                if constexpr (FULL) {
                    const int line = min(s0 / 2 + (j >> 1), steps / 2 - 1);  // past the end: a repeated, unused load
                    wv[j] = mk_ldg128_nt(wline[j & 1] + line * 128);
                } else {
                    const int s = min(s0 + j, steps - 1);
                    wv[j] = mk_ldg128(wrow + s * 64);  // not non-temporal: the second half of the line must stay cached
                }
            }
        };
        auto compute_block = [&](const mk_i4 *wl, int s0) {
            mk_i4 wv[S];
#pragma unroll
            for (int i = 0; i < S / 2; i++) {
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    if constexpr (FULL) {
                        const int ra = __builtin_amdgcn_ds_bpermute(rot_idx, wl[2 * i][k]), rb = __builtin_amdgcn_ds_bpermute(rot_idx, wl[2 * i + 1][k]);
                        wv[2 * i][k] = __builtin_amdgcn_update_dpp(ra, rb, 0x128 /* row_ror:8 */, 0xF, 0xC, false);
                        wv[2 * i + 1][k] = __builtin_amdgcn_update_dpp(rb, ra, 0x128 /* row_ror:8 */, 0xF, 0x3, false);
                    } else {
                        wv[2 * i][k] = wl[2 * i][k];
                        wv[2 * i + 1][k] = wl[2 * i + 1][k];
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < S; j++) {
                const int s = s0 + j;
                if (s < steps) {
                    mk_i4 xa = xl[(s * 4 + kb) * 8 + a_batch];
                    if (!a_live) xa = mk_i4{0, 0, 0, 0};
                    mk_i4 c = {0, 0, 0, 0};
                    c = __builtin_amdgcn_mfma_i32_16x16x64_i8(xa, wv[j], c, 0, 0, 0);
                    const mk_f4 x4 = *reinterpret_cast<const mk_f4 *>(xsl + (2 * s + par) * 8 + 4 * (kb & 1));
                    const float wsf = F16 ? mk_f16_bits_to_f32(*reinterpret_cast<const uint16_t *>(srow + 2 * s * SB))
                                          : *reinterpret_cast<const float *>(srow + 2 * s * SB);
#pragma unroll
                    for (int i = 0; i < 4; i++) acc[i] += (wsf * x4[i]) * (float)c[i];
                }
            }
        };
        load_block(wa, 0);
        for (int s0 = 0; s0 < steps; s0 += 2 * S) {
            load_block(wb, s0 + S);  // unconditional: past the end it repeats the last step
            compute_block(wa, s0);
            load_block(wa, s0 + 2 * S);
            compute_block(wb, s0 + S);
        }
#pragma unroll
        for (int i = 0; i < 4; i++) acc[i] += __shfl_xor(acc[i], 32, MK_WAVE);  // the two block parities
        if (lane < 32 && row_ok) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int b = 4 * (kb & 1) + i;
                if (b < batch) out[(size_t)b * rows + row] = acc[i];
            }
        }
    }
}

// ---------------------------------------------------------------- generic
template <bool F16>
__global__ __launch_bounds__(256) void q8_gemv_generic_kernel(const int8_t *__restrict__ q, const void *__restrict__ scales, int rows, int nb,
                                                              const int8_t *__restrict__ xq, const float *__restrict__ xs, int batch,
                                                              float *__restrict__ out) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const size_t cols = (size_t)nb * 32;
    float acc[8];
#pragma unroll
    for (int b = 0; b < 8; b++) acc[b] = 0.0f;
    for (int hb = lane; hb < nb * 2; hb += 64) {
        mk_i4 w = *reinterpret_cast<const mk_i4 *>(q + (size_t)row * cols + hb * 16);
        float wsf = load_scale<F16>(scales, (size_t)row * nb + (hb >> 1));
#pragma unroll
        for (int b = 0; b < 8; b++) {
            if (b < batch) {
                mk_i4 x = *reinterpret_cast<const mk_i4 *>(xq + (size_t)b * cols + hb * 16);
                int d = 0;
#pragma unroll
                for (int k = 0; k < 4; k++) d = __builtin_amdgcn_sdot4(w[k], x[k], d, false);
                acc[b] += (wsf * xs[(size_t)b * nb + (hb >> 1)]) * (float)d;
            }
        }
    }
#pragma unroll
    for (int b = 0; b < 8; b++) {
        if (b < batch) {
            float v = mk_wave_sum(acc[b]);
            if (lane == 0) out[(size_t)b * rows + row] = v;
        }
    }
}

// ----------------------------------------------------------------- argmax
// Greedy token: largest value, ties to the lowest index (the strict '>' of
// top_k_probs, src/model.rs:3283-3287).  Stage 1: up to 1024 blocks per row
// write (value, index) partials; stage 2: one block per row folds them.
__device__ __forceinline__ void argmax_fold(float &bv, int &bi, float v, int i) {
    if (v > bv || (v == bv && i < bi)) {
        bv = v;
        bi = i;
    }
}

__device__ void argmax_block_reduce(float &bv, int &bi) {
    __shared__ float sv[4];
    __shared__ int si[4];
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        float ov = __shfl_xor(bv, off, MK_WAVE);
        int oi = __shfl_xor(bi, off, MK_WAVE);
        argmax_fold(bv, bi, ov, oi);
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) {
        sv[wave] = bv;
        si[wave] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; w++) argmax_fold(bv, bi, sv[w], si[w]);
    }
}

__global__ __launch_bounds__(256) void argmax_stage1_kernel(const float *__restrict__ logits, int n, int chunk, float *__restrict__ pv,
                                                            int *__restrict__ pi) {
    const int b = blockIdx.y;
    const float *row = logits + (size_t)b * n;
    const int i0 = blockIdx.x * chunk, i1 = min(i0 + chunk, n);
    float bv = -INFINITY;
    int bi = 0x7FFFFFFF;
    for (int i = i0 + threadIdx.x; i < i1; i += 256) argmax_fold(bv, bi, row[i], i);
    argmax_block_reduce(bv, bi);
    if (threadIdx.x == 0) {
        pv[b * gridDim.x + blockIdx.x] = bv;
        pi[b * gridDim.x + blockIdx.x] = bi;
    }
}

__global__ __launch_bounds__(256) void argmax_stage2_kernel(const float *__restrict__ pv, const int *__restrict__ pi, int parts,
                                                            int32_t *__restrict__ out) {
    const int b = blockIdx.x;
    float bv = -INFINITY;
    int bi = 0x7FFFFFFF;
    for (int i = threadIdx.x; i < parts; i += 256) argmax_fold(bv, bi, pv[b * parts + i], pi[b * parts + i]);
    argmax_block_reduce(bv, bi);
    if (threadIdx.x == 0) out[b] = bi == 0x7FFFFFFF ? 0 : bi;
}


template <int NB, bool F16>
void launch_b1(const int8_t *q, const void *scales, int rows, const int8_t *xq, const float *xs, float *out, hipStream_t st) {
    // a fixed, fully resident grid: blocks-per-CU x 256 CUs x 4 waves
    int blocks = MK_TUNE("MK_Q8_B1_BLOCKS", 512);
    if (blocks * 4 > rows) blocks = (rows + 3) / 4;
    hipLaunchKernelGGL((q8_gemv_b1_kernel<NB, F16>), dim3(blocks), dim3(256), 0, st, q, scales, rows, xq, xs, out);
}

template <bool F16, int BATCH>
int launch_bn(const int8_t *q, const void *scales, int rows, const int8_t *xq, const float *xs, float *out, hipStream_t st) {
    constexpr int NB = 224;
    int blocks = MK_TUNE("MK_Q8_BN_BLOCKS", 512);
    if (blocks * 4 > rows) blocks = (rows + 3) / 4;
    const size_t lds = (size_t)BATCH * NB * 36;
    const int s = mk_lds_opt_in(reinterpret_cast<const void *>(q8_gemv_bn_kernel<NB, F16, BATCH>), 80 * 1024);
    if (s != MK_OK) return s;
    hipLaunchKernelGGL((q8_gemv_bn_kernel<NB, F16, BATCH>), dim3(blocks), dim3(256), lds, st, q, scales, rows, xq, xs, out);
    return mk_launch_status("q8_gemv_bn");
}

template <bool F16>
int launch_q8(const int8_t *q, const void *scales, size_t rows, size_t cols, const int8_t *xq, const float *xs, size_t batch, float *out,
              hipStream_t st) {
    const int nb = (int)(cols / 32);
    // measured on the 163840 x 7168 head: streaming kernel 188 / 198 / 203 us at batch 2 / 3 / 4 against 204 / 206 / 195 us
    // for the matrix-core kernel, whose time (195-198 us) does not grow with the batch
    if (batch >= 2 && batch <= 3 && nb == 224 && rows * cols < 0xFFFFFFFFull && !MK_TUNE("MK_Q8_NO_BN", 0)) {
        if (batch == 2) return launch_bn<F16, 2>(q, scales, (int)rows, xq, xs, out, st);
        return launch_bn<F16, 3>(q, scales, (int)rows, xq, xs, out, st);
    }
    if (batch == 1 && rows * cols < 0xFFFFFFFFull) {  // the batch-1 kernel addresses the matrix with 32-bit byte offsets
        switch (nb) {
            case 32: launch_b1<32, F16>(q, scales, (int)rows, xq, xs, out, st); return mk_launch_status("q8_gemv_b1");
            case 64: launch_b1<64, F16>(q, scales, (int)rows, xq, xs, out, st); return mk_launch_status("q8_gemv_b1");
            case 128: launch_b1<128, F16>(q, scales, (int)rows, xq, xs, out, st); return mk_launch_status("q8_gemv_b1");
            case 224: launch_b1<224, F16>(q, scales, (int)rows, xq, xs, out, st); return mk_launch_status("q8_gemv_b1");
            default: break;
        }
    } else if (nb % 2 == 0 && nb <= 256) {
        // LDS: activations (cols * 8) + their scales (nb * 32) + one scale tile per wave (16 * nb * 2 or 4 bytes)
        constexpr int WAVES = F16 ? 8 : 4;
        const int n_groups = (int)((rows + 15) / 16);
        int blocks = MK_TUNE("MK_Q8_MFMA_BLOCKS", 256);  // one per CU
        if (blocks * WAVES > n_groups) blocks = (n_groups + WAVES - 1) / WAVES;
        const size_t lds = cols * 8 + (size_t)nb * 32 + (size_t)WAVES * (16 * nb * (F16 ? 2 : 4) + 64);
        if (nb % 4 == 0 && !MK_TUNE("MK_Q8_MFMA_HALF_LINES", 0))  // rows are whole 128-byte lines
            hipLaunchKernelGGL((q8_gemv_mfma_kernel<F16, WAVES, true>), dim3(blocks), dim3(WAVES * 64), lds, st, q, scales, (int)rows, nb, xq,
                               xs, (int)batch, out);
        else
            hipLaunchKernelGGL((q8_gemv_mfma_kernel<F16, WAVES, false>), dim3(blocks), dim3(WAVES * 64), lds, st, q, scales, (int)rows, nb, xq,
                               xs, (int)batch, out);
        return mk_launch_status("q8_gemv_mfma");
    }
    hipLaunchKernelGGL(q8_gemv_generic_kernel<F16>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, st, q, scales, (int)rows, nb, xq, xs,
                       (int)batch, out);
    return mk_launch_status("q8_gemv_generic");
}

}  // namespace

extern "C" int mk_dev_q8_matvec(const int8_t *q, const void *scales, int scales_f16, size_t rows, size_t cols, const int8_t *xq,
                                const float *xs, size_t batch, float *out, void *stream) {
    MK_REQUIRE(q && scales && xq && xs && out, "null pointer");
    MK_REQUIRE(cols % 32 == 0 && cols > 0, "cols must be a positive multiple of 32");
    MK_REQUIRE(batch >= 1 && batch <= 8, "batch must be 1..8");
    MK_REQUIRE(rows <= 0x7FFFFFF0u && cols <= (1u << 24), "shape too large");
    MK_REQUIRE(((uintptr_t)q & 15) == 0 && ((uintptr_t)xq & 15) == 0, "q and xq must be 16-byte aligned");
    if (rows == 0) return MK_OK;
    // the batch kernel uses up to 136 KiB of the 160 KiB LDS
    const void *batch_kernels[4] = {reinterpret_cast<const void *>(q8_gemv_mfma_kernel<true, 8, true>),
                                    reinterpret_cast<const void *>(q8_gemv_mfma_kernel<false, 4, true>),
                                    reinterpret_cast<const void *>(q8_gemv_mfma_kernel<true, 8, false>),
                                    reinterpret_cast<const void *>(q8_gemv_mfma_kernel<false, 4, false>)};
    for (const void *k : batch_kernels) {
        const int s = mk_lds_opt_in(k, 160 * 1024);
        if (s != MK_OK) return s;
    }
    if (scales_f16) return launch_q8<true>(q, scales, rows, cols, xq, xs, batch, out, (hipStream_t)stream);
    return launch_q8<false>(q, scales, rows, cols, xq, xs, batch, out, (hipStream_t)stream);
}

extern "C" int mk_dev_argmax(const float *logits, size_t batch, size_t n, void *ws, int32_t *out_idx, void *stream) {
    MK_REQUIRE(logits && ws && out_idx, "null pointer");
    MK_REQUIRE(batch >= 1 && batch <= 65535 && n >= 1 && n <= 0x7FFFFFF0u, "bad shape");
    int parts = (int)((n + 4095) / 4096);
    if (parts > 1024) parts = 1024;
    const int chunk = (int)((n + parts - 1) / parts);
    float *pv = reinterpret_cast<float *>(ws);
    int *pi = reinterpret_cast<int *>(pv + batch * 1024);
    hipLaunchKernelGGL(argmax_stage1_kernel, dim3(parts, (unsigned)batch), dim3(256), 0, (hipStream_t)stream, logits, (int)n, chunk, pv, pi);
    hipLaunchKernelGGL(argmax_stage2_kernel, dim3((unsigned)batch), dim3(256), 0, (hipStream_t)stream, pv, pi, parts, out_idx);
    return mk_launch_status("argmax");
}
