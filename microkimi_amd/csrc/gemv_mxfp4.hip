// MXFP4 decode GEMV (mxfp4::matvec_packed and friends) for gfx950.
//
// HBM-bound: every weight byte is read exactly once with 128-bit loads, in the
// reference's own layout (packed [rows][cols/2], scales [rows][cols/32]; rows are
// contiguous, so a tile of rows is one contiguous byte range).  No repacking.
//
// Fast path (template on NB = cols/32):
//   * a tile is lcm(NB,64) blocks = RT rows; T = tile/64 wave iterations.
//     Lane l of iteration t owns block t*64+l of the tile: one 16-byte load of
//     32 nibbles plus one scale byte; the wave's T loads cover RT rows with
//     perfectly coalesced 1 KiB requests.
//   * the block index a lane owns repeats from tile to tile, so the lane keeps
//     "its" 32 activations (as f16 pairs) and block scale in registers for the
//     whole kernel; they are loaded straight from global memory (no LDS, no
//     barrier) behind the first two blocks of weight loads.
//   * q8 mode: nibbles -> f16 by v_cvt_scalef32_pk_f16_fp4, activation bytes as
//     f16 integers, v_dot2_f32_f16 accumulation.  Every term is a multiple of 0.5
//     below 2^15, so the f32 accumulation is exact: h = idot/2 and the block
//     contribution is (h+h) * (2^(sb-128) * dx), the reference's expression.
//   * one butterfly reduction per row, fixed order (deterministic).
// Generic path: one wave per row, any cols % 32 == 0.
#include <stdlib.h>

#include "mk_common.h"

namespace {

constexpr int gcd_c(int a, int b) { return b == 0 ? a : gcd_c(b, a % b); }
constexpr int lcm_c(int a, int b) { return a / gcd_c(a, b) * b; }

struct GemvArgs {
    // single-matrix form
    const uint8_t *packed;
    const uint8_t *scales;
    float *out;
    // grouped form (device arrays), used when packed == nullptr
    const uint8_t *const *packed_ptrs;
    const uint8_t *const *scales_ptrs;
    float *const *out_ptrs;
    const int32_t *x_index;
    // activation(s)
    const int8_t *xq;  // [nx][cols]
    const float *xs;   // [nx][cols/32]
    const float *xf;   // f32 mode: [nx][cols]
    int rows;
    int tiles_per_wave;
    int mat_xcd;  // q8 kernel: a matrix's workgroups on one XCD (grouped launches over a multiple of 8 matrices)
};

__device__ __forceinline__ float dot32_fp4_f16(const mk_i4 w, const mk_h2 *xr) {
    float h = 0.0f;
#pragma unroll
    for (int d = 0; d < 4; d++) {
        uint32_t wd = (uint32_t)w[d];
        h = __builtin_amdgcn_fdot2(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(wd, 1.0f, 0), xr[d * 4 + 0], h, false);
        h = __builtin_amdgcn_fdot2(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(wd, 1.0f, 1), xr[d * 4 + 1], h, false);
        h = __builtin_amdgcn_fdot2(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(wd, 1.0f, 2), xr[d * 4 + 2], h, false);
        h = __builtin_amdgcn_fdot2(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(wd, 1.0f, 3), xr[d * 4 + 3], h, false);
    }
    return h;
}

// ------------------------------------------------------------ q8 fast path
template <int NB>
__global__ __launch_bounds__(256) void mxfp4_gemv_q8_kernel(GemvArgs a) {
    constexpr int TILE = lcm_c(NB, 64);
    constexpr int T = TILE / 64;
    constexpr int RT = TILE / NB;
    static_assert(RT <= 2 && T <= 8, "tile shape not covered by the fast path");
    // Consecutive workgroup ids go round the 8 XCDs.  With the plain order every matrix of a grouped launch is read by all
    // eight of them; when the matrix count allows it, XCD c takes the matrices c, c + 8, ... whole (its L2 then holds
    // the windows of 1/8 of the matrices): 80 against 81-84 us on 64 matrices in the same run.
    int mat = blockIdx.y, bx = blockIdx.x;
    if (a.mat_xcd) {
        const int lin = blockIdx.y * gridDim.x + blockIdx.x, r = lin >> 3;
        mat = (lin & 7) + 8 * (r / (int)gridDim.x);
        bx = r % (int)gridDim.x;
    }
    // uniform pointers in scalar registers + 32-bit lane offsets: the loads take the scalar-base form
    const uint8_t *packed = mk_uniform_ptr(a.packed ? a.packed : a.packed_ptrs[mat]);
    const uint8_t *scales = mk_uniform_ptr(a.packed ? a.scales : a.scales_ptrs[mat]);
    if (!scales) return;  // a matrix without scale bytes is not MXFP4 (a VQ1 expert of a mixed layer): not this kernel's
    float *out = a.packed ? a.out : a.out_ptrs[mat];
    const int xi = (a.packed || !a.x_index) ? 0 : a.x_index[mat];
    const int8_t *xq = a.xq + (size_t)xi * NB * 32;
    const float *xs = a.xs + (size_t)xi * NB;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // tile arithmetic stays on the scalar unit
    // Tiles of this matrix are dealt round-robin to the matrix's resident waves
    // (wave w takes tiles w, w + W, ...): equal work, one compact read window
    // per matrix.  (One sequence of tiles over all matrices of a grouped launch --
    // a single window for the whole chip, as the lm_head kernel has -- measured
    // slower: 91.5 against 83.8 us on 64 matrices.)
    // U tiles form a register block; two blocks (ping, pong) are in flight.
    constexpr int U = (T >= 4) ? 1 : 8 / T;  // about 8 KiB per register block: T=1 -> 8 tiles, T=2 -> 4, T=3 -> 2
    const int n_tiles = (a.rows + RT - 1) / RT;
    const int wv = bx * 4 + wave;
    const int wpm = gridDim.x * 4;
    const int my_tiles = wv < n_tiles ? (n_tiles - wv + wpm - 1) / wpm : 0;

    mk_i4 wa[U][T], wb[U][T];
    uint32_t sa[U][T], sb[U][T];
    // Loads are unconditional (a predicated load becomes a branch and a full
    // wait): a tile past the end re-reads the wave's first tile and a lane past
    // the last row re-reads the last block; neither result is stored.  Block
    // indices are 32-bit (the host checks rows * NB < 2^28).
    const uint32_t last_blk = (uint32_t)a.rows * NB - 1;
    auto load_block = [&](mk_i4(*w)[T], uint32_t(*sc)[T], int k0) {
        k0 = __builtin_amdgcn_readfirstlane(k0);
#pragma unroll
        for (int u = 0; u < U; u++) {
            const uint32_t tile = (uint32_t)wv + ((k0 + u < my_tiles) ? (uint32_t)(k0 + u) * (uint32_t)wpm : 0u);
            const uint32_t blk0 = tile * TILE + lane;
#pragma unroll
            for (int t = 0; t < T; t++) {
                const uint32_t blk = min(blk0 + t * 64, last_blk);
                // long contiguous tiles (7 KB at K = 7168) are streamed non-temporally: 96 -> 84 us on 64 matrices;
                // the 1 KB tiles of short rows measured slower with it (47.6 -> 51.3 us)
                w[u][t] = T >= 4 ? mk_ldg128_off_nt(packed, blk * 16) : mk_ldg128_off(packed, blk * 16);
                sc[u][t] = mk_ldg_u8_off(scales, blk);
            }
        }
    };
    // both register blocks are requested before the activation is fetched: the
    // weight stream does not wait for the prologue
    load_block(wa, sa, 0);
    load_block(wb, sb, U);

    // The lane's activation blocks go straight from global memory (7 KiB, cache
    // resident) to registers, no LDS and no barrier: int8 -> f16 exactly, two
    // values per v_perm: byte b ^ 0x80 in the mantissa of 1024.0 is 1152 + b.
    mk_h2 xr[T][16];
    float cf[T];
    {
        mk_h2 bias;
        bias.x = bias.y = (_Float16)1152.0f;
#pragma unroll
        for (int t = 0; t < T; t++) {
            const int g = (t * 64 + lane) % NB;
            const mk_i4 v0 = mk_ldg128(xq + g * 32), v1 = mk_ldg128(xq + g * 32 + 16);
            cf[t] = xs[g];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const uint32_t u = (uint32_t)(j < 4 ? v0[j] : v1[j - 4]) ^ 0x80808080u;
                xr[t][2 * j] = __builtin_bit_cast(mk_h2, __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u)) - bias;
                xr[t][2 * j + 1] = __builtin_bit_cast(mk_h2, __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u)) - bias;
            }
        }
    }

    auto compute_block = [&](const mk_i4(*w)[T], const uint32_t(*sc)[T], int k0) {
        float acc[U][RT];
#pragma unroll
        for (int u = 0; u < U; u++) {
#pragma unroll
            for (int r = 0; r < RT; r++) acc[u][r] = 0.0f;
#pragma unroll
            for (int t = 0; t < T; t++) {
                float h = dot32_fp4_f16(w[u][t], xr[t]);
                float term = (h + h) * (mk_half_scale_from_byte(sc[u][t]) * cf[t]);
                const int rit = (t * 64 + lane) / NB;
#pragma unroll
                for (int r = 0; r < RT; r++) acc[u][r] += (rit == r) ? term : 0.0f;
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++)
#pragma unroll
            for (int r = 0; r < RT; r++) acc[u][r] = mk_wave_sum(acc[u][r]);
#pragma unroll
        for (int u = 0; u < U; u++) {
            if (k0 + u < my_tiles && lane < RT) {
                const int row = (wv + (k0 + u) * wpm) * RT + lane;
                if (row < a.rows) out[row] = (RT == 2 && lane == 1) ? acc[u][RT - 1] : acc[u][0];
            }
        }
    };
    // the prefetches are unconditional (past the end they re-read a valid tile):
    // a load under a branch forces a full wait at the join
    for (int k0 = 0; k0 < my_tiles; k0 += 2 * U) {
        compute_block(wa, sa, k0);
        load_block(wa, sa, k0 + 2 * U);
        compute_block(wb, sb, k0 + U);
        load_block(wb, sb, k0 + 3 * U);
    }
}

// ----------------------------------------------------------- f32 fast path
// Same tiling; the f32 activation stays in LDS (28 KiB at cols 7168) and each
// lane walks its block in column order with separate multiply and add, so the
// per-block sum gsum and the term gsum * 2^(sb-127) are the reference's values
// bit for bit (src/mxfp4.rs:494-505); only the order of the sum over blocks differs.
template <int NB>
__global__ __launch_bounds__(256) void mxfp4_gemv_f32_kernel(GemvArgs a) {
    constexpr int TILE = lcm_c(NB, 64);
    constexpr int T = TILE / 64;
    constexpr int RT = TILE / NB;
    static_assert(RT <= 2 && T <= 8, "tile shape not covered by the fast path");
    __shared__ __attribute__((aligned(16))) float xl[NB * 32];
    const int mat = blockIdx.y;
    const uint8_t *packed = a.packed ? a.packed : a.packed_ptrs[mat];
    const uint8_t *scales = a.packed ? a.scales : a.scales_ptrs[mat];
    if (!scales) return;  // (see the q8 kernel)
    float *out = a.packed ? a.out : a.out_ptrs[mat];
    const int xi = (a.packed || !a.x_index) ? 0 : a.x_index[mat];
    const float *xf = a.xf + (size_t)xi * NB * 32;
    for (int i = threadIdx.x; i < NB * 8; i += 256) reinterpret_cast<mk_f4 *>(xl)[i] = reinterpret_cast<const mk_f4 *>(xf)[i];
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n_tiles = (a.rows + RT - 1) / RT;
    const int tile0 = (blockIdx.x * 4 + wave) * a.tiles_per_wave;
    const int tile1 = min(tile0 + a.tiles_per_wave, n_tiles);
    for (int tile = tile0; tile < tile1; tile++) {
        const size_t blk0 = (size_t)tile * TILE;
        mk_i4 w[T];
        uint32_t sb[T];
#pragma unroll
        for (int t = 0; t < T; t++) {
            const int bi = t * 64 + lane;
            const bool ok = tile * RT + bi / NB < a.rows;
            w[t] = ok ? *reinterpret_cast<const mk_i4 *>(packed + (blk0 + bi) * 16) : mk_i4{0, 0, 0, 0};
            sb[t] = ok ? (uint32_t)scales[blk0 + bi] : 0u;
        }
        float acc[RT];
#pragma unroll
        for (int r = 0; r < RT; r++) acc[r] = 0.0f;
#pragma unroll
        for (int t = 0; t < T; t++) {
            const int bi = t * 64 + lane;
            const int g = bi % NB;
            const mk_f4 *xv = reinterpret_cast<const mk_f4 *>(xl + g * 32);
            float gsum = 0.0f;
#pragma unroll
            for (int d = 0; d < 4; d++) {
                uint32_t wd = (uint32_t)w[t][d];
                mk_f4 x0 = xv[d * 2], x1 = xv[d * 2 + 1];
                mk_f2 p0 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(wd, 1.0f, 0);
                mk_f2 p1 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(wd, 1.0f, 1);
                mk_f2 p2 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(wd, 1.0f, 2);
                mk_f2 p3 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(wd, 1.0f, 3);
                gsum = mk_add(gsum, mk_mul(p0.x, x0.x));
                gsum = mk_add(gsum, mk_mul(p0.y, x0.y));
                gsum = mk_add(gsum, mk_mul(p1.x, x0.z));
                gsum = mk_add(gsum, mk_mul(p1.y, x0.w));
                gsum = mk_add(gsum, mk_mul(p2.x, x1.x));
                gsum = mk_add(gsum, mk_mul(p2.y, x1.y));
                gsum = mk_add(gsum, mk_mul(p3.x, x1.z));
                gsum = mk_add(gsum, mk_mul(p3.y, x1.w));
            }
            float term = mk_mul(gsum, mk_scale_from_byte(sb[t]));
            const int rit = bi / NB;
#pragma unroll
            for (int r = 0; r < RT; r++) acc[r] += (rit == r) ? term : 0.0f;
        }
#pragma unroll
        for (int r = 0; r < RT; r++) acc[r] = mk_wave_sum(acc[r]);
        if (lane < RT) {
            const int row = tile * RT + lane;
            if (row < a.rows) out[row] = (RT == 2 && lane == 1) ? acc[RT - 1] : acc[0];
        }
    }
}

// ------------------------------------------------------------ generic path
// One wave per row, lanes stride over the row's blocks; activations come from
// global memory (L2-resident).  Any cols % 32 == 0.
template <bool Q8>
__global__ __launch_bounds__(256) void mxfp4_gemv_generic_kernel(GemvArgs a, int nb) {
    const int mat = blockIdx.y;
    const uint8_t *packed = a.packed ? a.packed : a.packed_ptrs[mat];
    const uint8_t *scales = a.packed ? a.scales : a.scales_ptrs[mat];
    if (!scales) return;  // (see the q8 kernel)
    float *out = a.packed ? a.out : a.out_ptrs[mat];
    const int xi = (a.packed || !a.x_index) ? 0 : a.x_index[mat];
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= a.rows) return;
    float acc = 0.0f;
    for (int g = lane; g < nb; g += 64) {
        const size_t blk = (size_t)row * nb + g;
        mk_i4 w = *reinterpret_cast<const mk_i4 *>(packed + blk * 16);
        uint32_t sb = scales[blk];
        if (Q8) {
            const int8_t *xq = a.xq + ((size_t)xi * nb + g) * 32;
            mk_h2 xr[16];
#pragma unroll
            for (int k = 0; k < 16; k++) {
                xr[k].x = (_Float16)(float)xq[2 * k];
                xr[k].y = (_Float16)(float)xq[2 * k + 1];
            }
            float h = dot32_fp4_f16(w, xr);
            acc += (h + h) * (mk_half_scale_from_byte(sb) * a.xs[(size_t)xi * nb + g]);
        } else {
            const float *x = a.xf + ((size_t)xi * nb + g) * 32;
            float gsum = 0.0f;
#pragma unroll
            for (int d = 0; d < 4; d++) {
                uint32_t wd = (uint32_t)w[d];
#pragma unroll
                for (int k = 0; k < 8; k++) gsum = mk_add(gsum, mk_mul(mk_e2m1((wd >> (4 * k)) & 15u), x[d * 8 + k]));
            }
            acc += mk_mul(gsum, mk_scale_from_byte(sb));
        }
    }
    acc = mk_wave_sum(acc);
    if (lane == 0) out[row] = acc;
}

// ---------------------------------------------------------- batched f32 (nt)
// model::matvec_packed_nt (src/model.rs:2412-2447): exact-f32 arithmetic for m
// positions against one packed matrix.  One wave per row; the row's nibbles are
// decoded once per 8-position group from registers, the activations stream from
// L2.  Per position and block the sum runs in column order with separate
// multiply and add (the reference's gsum), then gsum * scale; blocks are summed
// across lanes.  This is the exact-arithmetic twin of the MFMA GEMM, not the
// fast prefill path.
__global__ __launch_bounds__(256) void mxfp4_gemv_nt_kernel(const uint8_t *__restrict__ packed, const uint8_t *__restrict__ scales, int rows,
                                                            int nb, const float *__restrict__ x, int m, float *__restrict__ out) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const size_t cols = (size_t)nb * 32;
    for (int p0 = 0; p0 < m; p0 += 4) {
        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int g = lane; g < nb; g += 64) {
            const size_t blk = (size_t)row * nb + g;
            mk_i4 w = *reinterpret_cast<const mk_i4 *>(packed + blk * 16);
            float s = mk_scale_from_byte(scales[blk]);
#pragma unroll
            for (int p = 0; p < 4; p++) {
                if (p0 + p < m) {
                    const mk_f4 *xv = reinterpret_cast<const mk_f4 *>(x + (size_t)(p0 + p) * cols + (size_t)g * 32);
                    float gsum = 0.0f;
#pragma unroll
                    for (int d = 0; d < 4; d++) {
                        uint32_t wd = (uint32_t)w[d];
                        mk_f4 x0 = xv[d * 2], x1 = xv[d * 2 + 1];
                        gsum = mk_add(gsum, mk_mul(mk_e2m1(wd & 15u), x0.x));
                        gsum = mk_add(gsum, mk_mul(mk_e2m1((wd >> 4) & 15u), x0.y));
                        gsum = mk_add(gsum, mk_mul(mk_e2m1((wd >> 8) & 15u), x0.z));
                        gsum = mk_add(gsum, mk_mul(mk_e2m1((wd >> 12) & 15u), x0.w));
                        gsum = mk_add(gsum, mk_mul(mk_e2m1((wd >> 16) & 15u), x1.x));
                        gsum = mk_add(gsum, mk_mul(mk_e2m1((wd >> 20) & 15u), x1.y));
                        gsum = mk_add(gsum, mk_mul(mk_e2m1((wd >> 24) & 15u), x1.z));
                        gsum = mk_add(gsum, mk_mul(mk_e2m1((wd >> 28) & 15u), x1.w));
                    }
                    acc[p] += mk_mul(gsum, s);
                }
            }
        }
#pragma unroll
        for (int p = 0; p < 4; p++) {
            float v = mk_wave_sum(acc[p]);
            if (lane == 0 && p0 + p < m) out[(size_t)(p0 + p) * rows + row] = v;
        }
    }
}


// matvec_packed_nt for four and more positions on the f32 matrix instruction (v_mfma_f32_16x16x4_f32: f32 products, f32
// sums), cols % 128 == 0.  A wave works on 16 weight rows and a step of 128 columns at a time.  Lane (i = lane % 16,
// g = lane / 16) loads the 16 packed bytes of block 4 T + g of row i; a 4 x 4 exchange between the lanes i, i + 16,
// i + 32, i + 48 then leaves it dword g of each of the four blocks, i.e. the columns 32 b + 8 g .. + 7 (b = 0..3) of the
// step, dequantized exactly (e2m1 value times 2^(sb - 127): the scale rides on every weight because one instruction
// sums over columns of four blocks).  The activations of position j = lane % 16 for the same columns are 32 contiguous
// bytes per block, and the four lanes of a position read whole 128-byte lines between them (a lane that read its own
// block instead would touch 64 lines with every load instruction, and the address unit of the CU becomes the limit).
// Up to 16 NTT positions a pass (NTT accumulator tiles) against the same weight registers.  The terms are the
// reference's (src/model.rs:2412-2447); the order of the sums is not.
//
// The 4 x 4 exchange and the dequantization of one step: wq = the lane's 16 packed bytes of block g, sb = the scale
// bytes of the step's four blocks; wf[8 b + c] = weight of column 32 b + 8 g + c.  All 64 lanes must be active.
__device__ __forceinline__ void nt_dequant(mk_i4 wq, uint32_t sb, float (&wf)[32]) {
    // dword d of lane row g <-> dword g of lane row d (rows of 16 lanes): two swaps between the halves of the wave,
    // two between neighbouring rows
    const mk_u2 a = __builtin_amdgcn_permlane32_swap((unsigned)wq[0], (unsigned)wq[2], false, false);
    const mk_u2 b = __builtin_amdgcn_permlane32_swap((unsigned)wq[1], (unsigned)wq[3], false, false);
    const mk_u2 c = __builtin_amdgcn_permlane16_swap((unsigned)a[0], (unsigned)b[0], false, false);
    const mk_u2 e = __builtin_amdgcn_permlane16_swap((unsigned)a[1], (unsigned)b[1], false, false);
    const uint32_t w[4] = {c[0], c[1], e[0], e[1]};
    // (the hardware conversion gives the e2m1 values; the power of two is applied in f32: exact)
#pragma unroll
    for (int d = 0; d < 4; d++) {
        const uint32_t wd = w[d];
        const float sc = mk_scale_from_byte((sb >> (8 * d)) & 255u);
        const mk_f2 p0 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(wd, 1.0f, 0), p1 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(wd, 1.0f, 1);
        const mk_f2 p2 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(wd, 1.0f, 2), p3 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(wd, 1.0f, 3);
        wf[8 * d + 0] = p0.x * sc, wf[8 * d + 1] = p0.y * sc, wf[8 * d + 2] = p1.x * sc, wf[8 * d + 3] = p1.y * sc;
        wf[8 * d + 4] = p2.x * sc, wf[8 * d + 5] = p2.y * sc, wf[8 * d + 6] = p3.x * sc, wf[8 * d + 7] = p3.y * sc;
    }
}
// 16 weight rows x 16 positions x the step's 128 columns: xa[2 b + h] = the position's columns 32 b + 8 g + 4 h .. + 3.
// Two chains of dependent matrix instructions, added at the end.
__device__ __forceinline__ void nt_mfma_tile(const float (&wf)[32], const mk_f4 (&xa)[8], mk_f4 &acc) {
    mk_f4 c1 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int k = 0; k < 8; k += 2) {
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(wf[4 * k], xa[k].x, acc, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_16x16x4f32(wf[4 * k + 4], xa[k + 1].x, c1, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(wf[4 * k + 1], xa[k].y, acc, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_16x16x4f32(wf[4 * k + 5], xa[k + 1].y, c1, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(wf[4 * k + 2], xa[k].z, acc, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_16x16x4f32(wf[4 * k + 6], xa[k + 1].z, c1, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(wf[4 * k + 3], xa[k].w, acc, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_16x16x4f32(wf[4 * k + 7], xa[k + 1].w, c1, 0, 0, 0);
    }
    acc += c1;
}

// nt_mfma_pass: this wave's share (steps wave, wave + WAVES, ..) of one pass.  xp[tt] is the lane's activation row of
// tile tt, already moved to column 8 g; ntl (uniform, 1 .. NTT) tiles are in use.  All 64 lanes must be active.
template <int WAVES, int NTT>
__device__ __forceinline__ void nt_mfma_pass(const uint8_t *__restrict__ packed, const uint8_t *__restrict__ scales, int row, int nb, int wave,
                                             int g, const float *const (&xp)[NTT], int ntl, mk_f4 (&acc)[NTT]) {
    const int steps = nb / 4;
    // Everything is requested one item ahead: the next step's weights and scale byte before this step is worked on, the
    // next tile's activations (from L2) before this tile's matrix instructions.  Past the end: the last one again.
    const bool sc_al4 = ((uintptr_t)scales & 3) == 0;  // (nb % 4 == 0: every row's scale bytes then start on a dword)
    auto load_w = [&](int T, mk_i4 &wq, uint32_t &sb) {
        const size_t blk = (size_t)row * nb + 4 * min(T, steps - 1);
        wq = mk_ldg128_nt(packed + (blk + g) * 16);
        if (sc_al4) sb = mk_ldg_u32(scales + blk);  // the scale bytes of the step's four blocks
        else sb = mk_ldg_u8(scales + blk) | (mk_ldg_u8(scales + blk + 1) << 8) | (mk_ldg_u8(scales + blk + 2) << 16) | (mk_ldg_u8(scales + blk + 3) << 24);
    };
    auto load_x = [&](mk_f4 *xr, const float *xrow, int T) {
        const mk_f4 *xv = reinterpret_cast<const mk_f4 *>(xrow + (size_t)min(T, steps - 1) * 128);
#pragma unroll
        for (int k = 0; k < 8; k++) xr[k] = xv[8 * (k >> 1) + (k & 1)];  // columns 32 b + 8 g + 4 h of the step, k = 2 b + h
    };
    mk_i4 wq, wq_n;
    uint32_t sb, sb_n;
    mk_f4 xa[8], xb[8];
    load_w(wave, wq, sb);
    load_x(xa, xp[0], wave);
    for (int T = wave; T < steps; T += WAVES) {
        load_w(T + WAVES, wq_n, sb_n);
        __builtin_amdgcn_sched_barrier(0);
        float wf[32];
        nt_dequant(wq, sb, wf);
#pragma unroll
        for (int tt = 0; tt < NTT; tt++) {
            if (tt >= ntl) continue;
            if (tt + 1 < NTT && tt + 1 < ntl) load_x(xb, xp[tt + 1 < NTT ? tt + 1 : 0], T);
            else load_x(xb, xp[0], T + WAVES);
            __builtin_amdgcn_sched_barrier(0);  // (the requests stay in front of the matrix instructions that cover them)
            nt_mfma_tile(wf, xa, acc[tt]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int k = 0; k < 8; k++) xa[k] = xb[k];
        }
        wq = wq_n;
        sb = sb_n;
    }
}

// The waves' partial sums of one pass meet in wave 0, which stores tile tt's rows 4 g + r of position tok0 + 16 tt + i
// (result tile: column = position = lane % 16) for positions below tok_end.  Every wave of the workgroup calls it.
template <int WAVES, int NTT>
__device__ __forceinline__ void nt_mfma_store(mk_f4 (*red_l)[NTT][64], int wave, int lane, const mk_f4 (&acc)[NTT], int ntl, int row0, int rows,
                                              int tok0, int tok_end, float *__restrict__ out) {
    const int i = lane & 15, g = lane >> 4;
    if (wave > 0) {
#pragma unroll
        for (int tt = 0; tt < NTT; tt++) red_l[wave - 1][tt][lane] = acc[tt];
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
        for (int tt = 0; tt < NTT; tt++) {
            if (tt >= ntl) continue;
            mk_f4 v = acc[tt];
#pragma unroll
            for (int w = 0; w < WAVES - 1; w++) v += red_l[w][tt][lane];
            const int tok = tok0 + 16 * tt + i;
            const int r0 = row0 + 4 * g;
            if (tok < tok_end) {
                float *dst = out + (size_t)tok * rows + r0;
                if (r0 + 0 < rows) dst[0] = v.x;
                if (r0 + 1 < rows) dst[1] = v.y;
                if (r0 + 2 < rows) dst[2] = v.z;
                if (r0 + 3 < rows) dst[3] = v.w;
            }
        }
    }
}

template <int WAVES, int NTT>
__global__ __launch_bounds__(64 * WAVES) void mxfp4_gemm_nt_mfma_kernel(const uint8_t *__restrict__ packed, const uint8_t *__restrict__ scales,
                                                                        int rows, int nb, const float *__restrict__ x, int m,
                                                                        float *__restrict__ out) {
    __shared__ mk_f4 red_l[WAVES - 1][NTT][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, i = lane & 15, g = lane >> 4;
    const int row = min((int)blockIdx.x * 16 + i, rows - 1);
    const int tok0 = blockIdx.y * 16 * NTT;  // NTT tiles of 16 positions a pass (positions past the end: the last one, not stored)
    const size_t cols = (size_t)nb * 32;
    mk_f4 acc[NTT];
    const float *xp[NTT];
#pragma unroll
    for (int tt = 0; tt < NTT; tt++) {
        acc[tt] = mk_f4{0.0f, 0.0f, 0.0f, 0.0f};
        xp[tt] = x + (size_t)min(tok0 + 16 * tt + i, m - 1) * cols + (size_t)g * 8;
    }
    nt_mfma_pass<WAVES, NTT>(packed, scales, row, nb, wave, g, xp, NTT, acc);
    nt_mfma_store<WAVES, NTT>(red_l, wave, lane, acc, NTT, (int)blockIdx.x * 16, rows, tok0, m, out);
}

// The same product for groups of positions that each meet their own matrices (the experts of a prompt section): group e
// owns the grouped rows offsets[e] .. offsets[e+1] of out ([.][rows]); grouped row p reads activation row xrow[p] / xdiv
// of x (xrow null: row p).  Grid (tiles of 16 RW weight rows, groups, matrices per group).  The waves of a workgroup take
// 16 weight rows each and all the column steps of them, against the same activations: the workgroup stages each step's
// 16 NTT x 128 activations in LDS once (two buffers, one barrier a step; loaded a step ahead), so that the L1 sees them
// once per 16 RW weight rows instead of once per 16.  A workgroup walks its group in passes of 16 NTT rows.
struct NtGroupedArgs {
    const uint8_t *const *packed[2];
    const uint8_t *const *scales[2];
    float *out[2];
    const float *x;
    const int32_t *xrow;
    const int32_t *offsets;
    int rows, nb, xdiv;
    // offsets null: one matrix (packed1, scales1) for all m1 rows of x; blockIdx.y then counts passes of 16 NTT rows
    const uint8_t *packed1, *scales1;
    int m1;
    // VQ instantiation: the file's 256 x 16 f32 codebook; a group's "packed" pointer then holds index bytes [rows][cols / 16]
    const float *codebook;
};
// VQ = false takes the groups whose matrix has scale bytes (MXFP4) and leaves the others alone; VQ = true takes the groups
// with a null scale pointer, whose matrix is VQ1 (W[r][16 v .. 16 v + 16] = codebook[index[r][v]], src/quant.rs:353-376):
// the codebook sits in LDS and a lane fetches the halves of the four vectors that hold its columns.
template <int RW, int NTT, bool VQ = false>
__global__ __launch_bounds__(64 * RW) void mxfp4_gemm_nt_grouped_kernel(NtGroupedArgs a) {
    constexpr int XS = 136;                            // floats a staged row takes (128 + 8: neighbouring rows start 8 banks apart)
    constexpr int PER = NTT * 16 * 32 / (64 * RW);     // 16-byte pieces of a step's activations per thread
    static_assert(PER >= 1 && PER * 64 * RW == NTT * 16 * 32, "threads must divide the staged activations");
    __shared__ float xs_l[2][NTT * 16][XS];
    __shared__ __attribute__((aligned(16))) float cb_l[VQ ? 256 * 16 : 4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, i = lane & 15, g = lane >> 4;
    const bool one = a.offsets == nullptr;
    // (groups in a multiple of 8: a group's workgroups on one XCD, see the bf16 kernel below)
    int grp = blockIdx.y, mat = blockIdx.z, rblk = blockIdx.x;
    if (!one && (gridDim.y & 7) == 0) {
        const int per = gridDim.x * gridDim.z;
        const int lin = (int)blockIdx.x + (int)gridDim.x * ((int)blockIdx.y + (int)gridDim.y * (int)blockIdx.z);
        const int xcd = lin & 7, slot = lin >> 3;
        grp = (slot / per) * 8 + xcd;
        const int inner = slot % per;
        mat = inner / (int)gridDim.x;
        rblk = inner % (int)gridDim.x;
    }
    const int p_begin = one ? grp * 16 * NTT : a.offsets[grp], p_end = one ? min(a.m1, p_begin + 16 * NTT) : a.offsets[grp + 1];
    if (p_end <= p_begin) return;  // (the whole workgroup)
    const uint8_t *__restrict__ packed = one ? a.packed1 : a.packed[mat][grp];
    const uint8_t *__restrict__ scales = one ? a.scales1 : a.scales[mat][grp];
    if ((scales == nullptr) != VQ) return;  // (the other instantiation's group)
    float *__restrict__ out = a.out[mat];
    const int nb = a.nb, steps = nb / 4;
    if (VQ) {
        for (int k = threadIdx.x; k < 256 * 4; k += 64 * RW) reinterpret_cast<mk_f4 *>(cb_l)[k] = reinterpret_cast<const mk_f4 *>(a.codebook)[k];
        // (the barrier in front of the first step also covers the codebook)
    }
    const int row0 = (rblk * RW + wave) * 16;   // (a wave past the last row works on the last row and stores nothing)
    const int row = min(row0 + i, a.rows - 1);
    const size_t cols = (size_t)nb * 32;
    const bool sc_al4 = ((uintptr_t)scales & 3) == 0;
    auto load_w = [&](int T, mk_i4 &wq, uint32_t &sb) {
        if (VQ) {
            // the index bytes of the vectors 2 b + g / 2 (b = 0..3) of the step's eight
            const uint8_t *ip = packed + (size_t)row * (nb * 2) + 8 * min(T, steps - 1) + (g >> 1);
#pragma unroll
            for (int b = 0; b < 4; b++) wq[b] = (int)mk_ldg_u8(ip + 2 * b);
            sb = 0;
            return;
        }
        const size_t blk = (size_t)row * nb + 4 * min(T, steps - 1);
        wq = mk_ldg128_nt(packed + (blk + g) * 16);
        if (sc_al4) sb = mk_ldg_u32(scales + blk);
        else sb = mk_ldg_u8(scales + blk) | (mk_ldg_u8(scales + blk + 1) << 8) | (mk_ldg_u8(scales + blk + 2) << 16) | (mk_ldg_u8(scales + blk + 3) << 24);
    };
    for (int p0 = p_begin; p0 < p_end; p0 += 16 * NTT) {
        const int ntl = min(NTT, (p_end - p0 + 15) >> 4);
        // staging: piece q of this thread is 4 columns (sc) of staged row sr; rows of unused tiles are not touched
        const float *sp[PER];
        int so[PER];
#pragma unroll
        for (int q = 0; q < PER; q++) {
            const int idx = (int)threadIdx.x + q * 64 * RW, sr = idx >> 5, sc = (idx & 31) * 4;
            const int p = min(p0 + sr, p_end - 1);
            const int xr = a.xrow ? a.xrow[p] / a.xdiv : p;
            sp[q] = sr < 16 * ntl ? a.x + (size_t)xr * cols + sc : nullptr;
            so[q] = sr * XS + sc;
        }
        mk_f4 st[PER];
#pragma unroll
        for (int q = 0; q < PER; q++)
            if (sp[q]) *reinterpret_cast<mk_f4 *>(&xs_l[0][0][0] + so[q]) = *reinterpret_cast<const mk_f4 *>(sp[q]);
        mk_f4 acc[NTT];
#pragma unroll
        for (int tt = 0; tt < NTT; tt++) acc[tt] = mk_f4{0.0f, 0.0f, 0.0f, 0.0f};
        mk_i4 wq, wq_n;
        uint32_t sb, sb_n;
        load_w(0, wq, sb);
        __syncthreads();
        for (int T = 0; T < steps; T++) {
            const bool more = T + 1 < steps;
#pragma unroll
            for (int q = 0; q < PER; q++)
                if (more && sp[q]) st[q] = *reinterpret_cast<const mk_f4 *>(sp[q] + (size_t)(T + 1) * 128);
            load_w(T + 1, wq_n, sb_n);
            float wf[32];
            if (VQ) {
#pragma unroll
                for (int b = 0; b < 4; b++) {
                    const mk_f4 *e = reinterpret_cast<const mk_f4 *>(cb_l + wq[b] * 16 + 8 * (g & 1));
                    const mk_f4 lo = e[0], hi = e[1];
                    wf[8 * b + 0] = lo.x, wf[8 * b + 1] = lo.y, wf[8 * b + 2] = lo.z, wf[8 * b + 3] = lo.w;
                    wf[8 * b + 4] = hi.x, wf[8 * b + 5] = hi.y, wf[8 * b + 6] = hi.z, wf[8 * b + 7] = hi.w;
                }
            } else {
                nt_dequant(wq, sb, wf);
            }
            const float *xb = &xs_l[T & 1][0][0] + i * XS + 8 * g;
#pragma unroll
            for (int tt = 0; tt < NTT; tt++) {
                if (tt >= ntl) continue;
                mk_f4 xa[8];
#pragma unroll
                for (int k = 0; k < 8; k++) xa[k] = *reinterpret_cast<const mk_f4 *>(xb + tt * 16 * XS + 32 * (k >> 1) + 4 * (k & 1));
                nt_mfma_tile(wf, xa, acc[tt]);
            }
#pragma unroll
            for (int q = 0; q < PER; q++)
                if (more && sp[q]) *reinterpret_cast<mk_f4 *>(&xs_l[(T + 1) & 1][0][0] + so[q]) = st[q];
            wq = wq_n;
            sb = sb_n;
            __syncthreads();  // (the next step reads what was just written; the step after it overwrites what was just read)
        }
        // result tile: column = grouped row p0 + 16 tt + i, rows row0 + 4 g + r
#pragma unroll
        for (int tt = 0; tt < NTT; tt++) {
            if (tt >= ntl) continue;
            const int p = p0 + 16 * tt + i, r0 = row0 + 4 * g;
            if (p < p_end && r0 < a.rows) {
                float *dst = out + (size_t)p * a.rows + r0;
                if (r0 + 3 < a.rows) *reinterpret_cast<mk_f4 *>(dst) = acc[tt];
                else {
                    dst[0] = acc[tt].x;
                    if (r0 + 1 < a.rows) dst[1] = acc[tt].y;
                    if (r0 + 2 < a.rows) dst[2] = acc[tt].z;
                }
            }
        }
    }
}

// The grouped product with bfloat16 activations on v_mfma_f32_16x16x32_bf16: the weights are exact in bf16 (an e2m1
// value times a power of two), the products exact in f32 and summed in f32, so the one rounding is that of the
// activations (done by the caller, once per row).  cols % 512 == 0.  Same split of the work as the f32 kernel above: a
// wave owns 16 weight rows and all their columns, the workgroup stages the group's activation rows in LDS, here a K
// tile of 512 columns at a time (two buffers, one barrier a K tile).
//
// Weight side: the 256 bytes a row has in a K tile are fetched as whole 128-byte lines (a load takes 8 rows x 128 bytes:
// lane (r3 = lane / 8, c = lane % 8) reads bytes 16 c .. of row 8 h + r3; loads 2 i and 2 i + 1 cover line i of rows 0-7
// and 8-15), non-temporally, a K tile ahead; a rotation of the lane index by three bits (ds_bpermute) and an exchange
// of the 8-lane halves of every 16-lane row between two registers (DPP row_ror:8 under a bank mask) then give lane
// (i = lane % 16, g = lane / 16) the 16 bytes of block 4 u + g of row i for the four steps u of the K tile.  Dword s2 of
// such a block and the block's scale become the eight bf16 values lane group g feeds to matrix instruction (u, s2)
// through v_cvt_scalef32_pk_bf16_fp4.  The activations of those columns, 128 u + 32 g + 8 s2 .. + 7, are one 16-byte
// LDS read; the staging stores piece 4 g + s2 of a step at place 4 s2 + g, so that the four lanes of a position read
// 64 contiguous bytes (with the pieces in column order the same reads ran into bank conflicts: 2.1-2.2 ms for the
// 512-token section against 1.7), and rows are 32 bytes of padding apart (16: 2.7 times the conflict cycles).
// Measured on the way: loads of 16 rows x 64 bytes in the operand's own form streamed at 4.1 TB/s with everything
// else compiled out, the whole-line loads at 5.0; held to 128 registers (two workgroups a CU) 1.68 ms, at 138
// registers (one workgroup) 1.96-2.1 ms; ordinary instead of non-temporal loads 1.77 ms.
typedef __bf16 mk_bf8 __attribute__((ext_vector_type(8)));
typedef __bf16 mk_bf2 __attribute__((ext_vector_type(2)));
struct Bf16GroupedArgs {
    const uint8_t *const *packed[2];
    const uint8_t *const *scales[2];
    const uint8_t *const *scales_t[2];  // optional: the scale bytes in [K tile][row][16] order (16-byte aligned), read instead
    float *out[2];
    const uint16_t *x;       // [grouped rows][cols] bf16
    const int32_t *offsets;  // [groups + 1]
    int rows, nb;
};
template <int RW, int NTT>
__global__ __launch_bounds__(64 * RW) __attribute__((amdgpu_waves_per_eu(4))) void mxfp4_gemm_bf16_grouped_kernel(Bf16GroupedArgs a) {
    constexpr int XSB = 512 * 2 + 32;                   // bytes a staged row takes (32 of padding: neighbouring rows 8 banks apart)
    constexpr int PER = NTT * 16 * 64 / (64 * RW);      // 16-byte pieces of a K tile per thread
    static_assert(PER >= 1 && PER * 64 * RW == NTT * 16 * 64, "threads must divide the staged activations");
    __shared__ __attribute__((aligned(16))) uint8_t xs_l[2][NTT * 16 * XSB];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, i = lane & 15, g = lane >> 4;
    // Workgroup ids go round the eight XCDs in turn, each with its own L2: with a multiple of 8 groups, id -> (XCD,
    // slot) and a group's workgroups (row blocks x matrices) take consecutive slots of one XCD, so that the group's
    // activation rows are fetched into one L2 instead of eight.
    int grp = blockIdx.y, mat = blockIdx.z, rblk = blockIdx.x;
    if ((gridDim.y & 7) == 0) {
        const int per = gridDim.x * gridDim.z;
        const int lin = (int)blockIdx.x + (int)gridDim.x * ((int)blockIdx.y + (int)gridDim.y * (int)blockIdx.z);
        const int xcd = lin & 7, slot = lin >> 3;
        grp = (slot / per) * 8 + xcd;
        const int inner = slot % per;
        mat = inner / (int)gridDim.x;
        rblk = inner % (int)gridDim.x;
    }
    const int p_begin = a.offsets[grp], p_end = a.offsets[grp + 1];
    if (p_end <= p_begin) return;  // (the whole workgroup)
    const uint8_t *__restrict__ packed = a.packed[mat][grp];
    const uint8_t *__restrict__ scales = a.scales[mat][grp];
    float *__restrict__ out = a.out[mat];
    const int nb = a.nb, ktiles = nb / 16;
    const int row0 = (rblk * RW + wave) * 16;  // (a wave past the last row works on the last row and stores nothing)
    const size_t cols = (size_t)nb * 32;
    const uint8_t *wline[2];
#pragma unroll
    for (int h = 0; h < 2; h++) wline[h] = packed + (size_t)min(row0 + 8 * h + (lane >> 3), a.rows - 1) * (cols / 2) + (lane & 7) * 16;
    const int rot_idx = (((lane & 7) << 3) | (((lane >> 3) & 1) << 2) | (lane >> 4)) * 4;
    // a wave's 16 rows x 16 scale bytes of a K tile: 16 eighths of lines in the reference layout, two whole lines in K-tile order
    const uint8_t *scales_t = a.scales_t[mat] ? a.scales_t[mat][grp] : nullptr;
    const uint8_t *srow = scales_t ? scales_t + (size_t)min(row0 + i, a.rows - 1) * 16 : scales + (size_t)min(row0 + i, a.rows - 1) * nb;
    const size_t sstep = scales_t ? (size_t)a.rows * 16 : 16;
    const int sc_al = scales_t || ((uintptr_t)scales & 15) == 0 ? 16 : ((uintptr_t)scales & 3) == 0 ? 4 : 1;  // (nb % 16 == 0)
    auto load_w = [&](int kt, mk_i4 (&wl)[4], mk_i4 &sc) {
        const size_t ku = (size_t)min(kt, ktiles - 1);
#pragma unroll
        for (int j = 0; j < 4; j++) wl[j] = mk_ldg128_nt(wline[j & 1] + ku * 256 + (j >> 1) * 128);
        const uint8_t *sp = srow + ku * sstep;  // the scale bytes of the row's 16 blocks in the K tile
        if (sc_al == 16) sc = *reinterpret_cast<const mk_i4 *>(sp);
        else if (sc_al == 4) sc = mk_i4{(int)mk_ldg_u32(sp), (int)mk_ldg_u32(sp + 4), (int)mk_ldg_u32(sp + 8), (int)mk_ldg_u32(sp + 12)};
        else {
#pragma unroll
            for (int k = 0; k < 4; k++)
                sc[k] = (int)(mk_ldg_u8(sp + 4 * k) | (mk_ldg_u8(sp + 4 * k + 1) << 8) | (mk_ldg_u8(sp + 4 * k + 2) << 16) | (mk_ldg_u8(sp + 4 * k + 3) << 24));
        }
    };
    for (int p0 = p_begin; p0 < p_end; p0 += 16 * NTT) {
        const int ntl = min(NTT, (p_end - p0 + 15) >> 4);
        // staging: piece q of this thread is 8 columns (16 bytes) of staged row sr; rows of unused tiles are not touched
        const uint8_t *sp[PER];
        int so[PER];
#pragma unroll
        for (int q = 0; q < PER; q++) {
            const int idx = (int)threadIdx.x + q * 64 * RW, sr = idx >> 6, pc = idx & 63;
            const int p = min(p0 + sr, p_end - 1);
            sp[q] = sr < 16 * ntl ? reinterpret_cast<const uint8_t *>(a.x) + ((size_t)p * cols) * 2 + pc * 16 : nullptr;
            // inside a step's 16 pieces, piece 4 g + s2 (block g, dword s2) goes to place 4 s2 + g: the four lanes of a
            // position then read 64 contiguous bytes for a matrix instruction
            so[q] = sr * XSB + ((pc & 48) | ((pc & 3) << 2) | ((pc >> 2) & 3)) * 16;
        }
        mk_i4 st[PER];
#pragma unroll
        for (int q = 0; q < PER; q++)
            if (sp[q]) *reinterpret_cast<mk_i4 *>(&xs_l[0][so[q]]) = *reinterpret_cast<const mk_i4 *>(sp[q]);
        mk_f4 acc[NTT][2];
#pragma unroll
        for (int tt = 0; tt < NTT; tt++) acc[tt][0] = acc[tt][1] = mk_f4{0.0f, 0.0f, 0.0f, 0.0f};
        mk_i4 wl[4], wl_n[4], sc, sc_n;
        load_w(0, wl, sc);
        __syncthreads();
        for (int kt = 0; kt < ktiles; kt++) {
            const bool more = kt + 1 < ktiles;
#pragma unroll
            for (int q = 0; q < PER; q++)
                if (more && sp[q]) st[q] = *reinterpret_cast<const mk_i4 *>(sp[q] + (size_t)(kt + 1) * 1024);
            load_w(kt + 1, wl_n, sc_n);
            // operand form of the K tile's two lines: lane (i, g) gets the 16 bytes of block 4 u + g of row i
            mk_i4 w[4];
#pragma unroll
            for (int l2 = 0; l2 < 2; l2++)
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const int ra = __builtin_amdgcn_ds_bpermute(rot_idx, wl[2 * l2][k]), rb = __builtin_amdgcn_ds_bpermute(rot_idx, wl[2 * l2 + 1][k]);
                    w[2 * l2][k] = __builtin_amdgcn_update_dpp(ra, rb, 0x128 /* row_ror:8 */, 0xF, 0xC, false);
                    w[2 * l2 + 1][k] = __builtin_amdgcn_update_dpp(rb, ra, 0x128 /* row_ror:8 */, 0xF, 0x3, false);
                }
            const uint8_t *xb = &xs_l[kt & 1][0] + i * XSB + 16 * g;
#pragma unroll
            for (int u = 0; u < 4; u++) {
                mk_bf8 wa[4];
                const float scf = mk_scale_from_byte(((uint32_t)sc[u] >> (8 * g)) & 255u);  // block 4 u + g
#pragma unroll
                for (int s2 = 0; s2 < 4; s2++) {
                    const uint32_t wd = (uint32_t)w[u][s2];
                    const mk_bf2 c0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(wd, scf, 0), c1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(wd, scf, 1);
                    const mk_bf2 c2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(wd, scf, 2), c3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(wd, scf, 3);
                    wa[s2] = mk_bf8{c0[0], c0[1], c1[0], c1[1], c2[0], c2[1], c3[0], c3[1]};
                }
#pragma unroll
                for (int tt = 0; tt < NTT; tt++) {
                    if (tt >= ntl) continue;
#pragma unroll
                    for (int s2 = 0; s2 < 4; s2++) {
                        const mk_bf8 xv = *reinterpret_cast<const mk_bf8 *>(xb + tt * 16 * XSB + u * 256 + 64 * s2);
                        acc[tt][s2 & 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[s2], xv, acc[tt][s2 & 1], 0, 0, 0);
                    }
                }
            }
#pragma unroll
            for (int q = 0; q < PER; q++)
                if (more && sp[q]) *reinterpret_cast<mk_i4 *>(&xs_l[(kt + 1) & 1][so[q]]) = st[q];
#pragma unroll
            for (int u = 0; u < 4; u++) wl[u] = wl_n[u];
            sc = sc_n;
            __syncthreads();  // (the next K tile reads what was just written; the one after it overwrites what was just read)
        }
        // result tile: column = grouped row p0 + 16 tt + i, rows row0 + 4 g + r
#pragma unroll
        for (int tt = 0; tt < NTT; tt++) {
            if (tt >= ntl) continue;
            const mk_f4 v = acc[tt][0] + acc[tt][1];
            const int p = p0 + 16 * tt + i, r0 = row0 + 4 * g;
            if (p < p_end && r0 < a.rows) {
                float *dst = out + (size_t)p * a.rows + r0;
                if (r0 + 3 < a.rows) *reinterpret_cast<mk_f4 *>(dst) = v;
                else {
                    dst[0] = v.x;
                    if (r0 + 1 < a.rows) dst[1] = v.y;
                    if (r0 + 2 < a.rows) dst[2] = v.z;
                }
            }
        }
    }
}

template <int WAVES, int NTT>
int launch_nt_mfma(const uint8_t *packed, const uint8_t *scales, size_t rows, size_t cols, const float *x, size_t m, float *out, hipStream_t st) {
    const dim3 grid((unsigned)((rows + 15) / 16), (unsigned)((m + 16 * NTT - 1) / (16 * NTT)));
    hipLaunchKernelGGL((mxfp4_gemm_nt_mfma_kernel<WAVES, NTT>), grid, dim3(64 * WAVES), 0, st, packed, scales, (int)rows, (int)(cols / 32), x, (int)m, out);
    return mk_launch_status("mxfp4_gemm_nt_mfma");
}
template <int WAVES>
int launch_nt_mfma_w(const uint8_t *packed, const uint8_t *scales, size_t rows, size_t cols, const float *x, size_t m, float *out, hipStream_t st) {
    // tiles of 16 positions a workgroup takes against its weight registers: as many as leaves the chip 512 workgroups
    const size_t row_tiles = (rows + 15) / 16, tiles = (m + 15) / 16;
    size_t ntt = std::min<size_t>(4, tiles);
    while (ntt > 1 && row_tiles * ((tiles + ntt - 1) / ntt) < 512) ntt--;
    switch (ntt) {
        case 1: return launch_nt_mfma<WAVES, 1>(packed, scales, rows, cols, x, m, out, st);
        case 2: return launch_nt_mfma<WAVES, 2>(packed, scales, rows, cols, x, m, out, st);
        case 3: return launch_nt_mfma<WAVES, 3>(packed, scales, rows, cols, x, m, out, st);
        default: return launch_nt_mfma<WAVES, 4>(packed, scales, rows, cols, x, m, out, st);
    }
}

template <int RW, int NTT = 2>
int launch_nt_grouped(const NtGroupedArgs &a, size_t n_groups, int n_mats, hipStream_t st) {
    const dim3 grid((unsigned)((a.rows + 16 * RW - 1) / (16 * RW)), (unsigned)n_groups, (unsigned)n_mats);
    hipLaunchKernelGGL((mxfp4_gemm_nt_grouped_kernel<RW, NTT>), grid, dim3(64 * RW), 0, st, a);
    int s = mk_launch_status("mxfp4_gemm_nt_grouped");
    if (s != MK_OK || !a.codebook) return s;
    // a layer with VQ1 experts: their groups in a second launch (which groups they are is known on the device only)
    hipLaunchKernelGGL((mxfp4_gemm_nt_grouped_kernel<RW, 2, true>), grid, dim3(64 * RW), 0, st, a);
    return mk_launch_status("vq1_gemm_nt_grouped");
}

template <int NB>
int launch_fast(const GemvArgs &a0, bool q8, size_t nmat, hipStream_t st) {
    constexpr int RT = lcm_c(NB, 64) / NB;
    GemvArgs a = a0;
    const int n_tiles = (a.rows + RT - 1) / RT;
    if (q8) {
        // a fixed, fully resident grid shared by the matrices of the launch
        // (2 workgroups per CU measured best for every block count per row)
        int per_mat = MK_TUNE("MK_MXFP4_BLOCKS", 512) / (int)nmat;
        if (per_mat < 1) per_mat = 1;
        if (per_mat * 4 > n_tiles) per_mat = (n_tiles + 3) / 4;
        a.mat_xcd = nmat % 8 == 0 && nmat >= 8 && MK_TUNE("MK_MXFP4_MAT_XCD", 1);
        hipLaunchKernelGGL(mxfp4_gemv_q8_kernel<NB>, dim3(per_mat, (unsigned)nmat), dim3(256), 0, st, a);
        return mk_launch_status("mxfp4_gemv_q8");
    }
    int tpw = 1;
    while (tpw < 16 && (size_t)n_tiles * nmat / (tpw * 2) >= 256 * 4 * 4) tpw *= 2;
    a.tiles_per_wave = tpw;
    const unsigned gx = (unsigned)((n_tiles + 4 * tpw - 1) / (4 * tpw));
    hipLaunchKernelGGL(mxfp4_gemv_f32_kernel<NB>, dim3(gx, (unsigned)nmat), dim3(256), 0, st, a);
    return mk_launch_status("mxfp4_gemv_f32");
}

int launch_gemv(const GemvArgs &a, bool q8, size_t nmat, size_t cols, hipStream_t st) {
    const int nb = (int)(cols / 32);
    if (a.rows == 0 || nmat == 0) return MK_OK;
    if ((size_t)a.rows * nb < (1u << 28)) {  // the fast kernels index blocks in 32 bits (16 bytes each)
        switch (nb) {
            case 32: return launch_fast<32>(a, q8, nmat, st);
            case 64: return launch_fast<64>(a, q8, nmat, st);
            case 128: return launch_fast<128>(a, q8, nmat, st);
            case 224: return launch_fast<224>(a, q8, nmat, st);
            default: break;
        }
    }
    const unsigned gx = (unsigned)((a.rows + 3) / 4);
    if (q8)
        hipLaunchKernelGGL(mxfp4_gemv_generic_kernel<true>, dim3(gx, (unsigned)nmat), dim3(256), 0, st, a, nb);
    else
        hipLaunchKernelGGL(mxfp4_gemv_generic_kernel<false>, dim3(gx, (unsigned)nmat), dim3(256), 0, st, a, nb);
    return mk_launch_status("mxfp4_gemv_generic");
}

bool shape_ok(size_t rows, size_t cols) { return cols % 32 == 0 && cols > 0 && rows <= 0x7FFFFFFF / 64 && cols <= (1u << 24); }

}  // namespace

extern "C" int mk_dev_mxfp4_matvec_q8(const uint8_t *packed, const uint8_t *scales, size_t rows, size_t cols, const int8_t *xq,
                                      const float *xs, float *out, void *stream) {
    MK_REQUIRE(packed && scales && xq && xs && out, "null pointer");
    MK_REQUIRE(shape_ok(rows, cols), "cols must be a positive multiple of 32");
    MK_REQUIRE(((uintptr_t)packed & 15) == 0 && ((uintptr_t)xq & 3) == 0, "packed must be 16-byte and xq 4-byte aligned");
    GemvArgs a = {};
    a.packed = packed;
    a.scales = scales;
    a.out = out;
    a.xq = xq;
    a.xs = xs;
    a.rows = (int)rows;
    return launch_gemv(a, true, 1, cols, (hipStream_t)stream);
}

extern "C" int mk_dev_mxfp4_matvec_f32(const uint8_t *packed, const uint8_t *scales, size_t rows, size_t cols, const float *x, float *out,
                                       void *stream) {
    MK_REQUIRE(packed && scales && x && out, "null pointer");
    MK_REQUIRE(shape_ok(rows, cols), "cols must be a positive multiple of 32");
    MK_REQUIRE(((uintptr_t)packed & 15) == 0 && ((uintptr_t)x & 15) == 0, "packed and x must be 16-byte aligned");
    GemvArgs a = {};
    a.packed = packed;
    a.scales = scales;
    a.out = out;
    a.xf = x;
    a.rows = (int)rows;
    return launch_gemv(a, false, 1, cols, (hipStream_t)stream);
}

extern "C" int mk_dev_mxfp4_matvec(const uint8_t *packed, const uint8_t *scales, size_t rows, size_t cols, const float *x, float *out,
                                   int mode, int8_t *xq_ws, float *xs_ws, void *stream) {
    if (mode == MK_MODE_F32) return mk_dev_mxfp4_matvec_f32(packed, scales, rows, cols, x, out, stream);
    MK_REQUIRE(mode == MK_MODE_Q8, "mode must be MK_MODE_F32 or MK_MODE_Q8");
    MK_REQUIRE(xq_ws && xs_ws, "q8 mode needs the xq/xs scratch");
    int s = mk_dev_quantize_q8(x, 1, cols, xq_ws, xs_ws, stream);
    if (s != MK_OK) return s;
    return mk_dev_mxfp4_matvec_q8(packed, scales, rows, cols, xq_ws, xs_ws, out, stream);
}

extern "C" int mk_dev_mxfp4_matvec_q8_grouped(const uint8_t *const *packed_ptrs, const uint8_t *const *scales_ptrs, size_t nmat,
                                              size_t rows, size_t cols, const int8_t *xq, const float *xs, const int32_t *x_index,
                                              float *const *out_ptrs, void *stream) {
    MK_REQUIRE(packed_ptrs && scales_ptrs && xq && xs && out_ptrs, "null pointer");
    MK_REQUIRE(shape_ok(rows, cols), "cols must be a positive multiple of 32");
    MK_REQUIRE(nmat <= 65535, "at most 65535 matrices per launch");
    GemvArgs a = {};
    a.packed_ptrs = packed_ptrs;
    a.scales_ptrs = scales_ptrs;
    a.out_ptrs = out_ptrs;
    a.x_index = x_index;
    a.xq = xq;
    a.xs = xs;
    a.rows = (int)rows;
    return launch_gemv(a, true, nmat, cols, (hipStream_t)stream);
}

int mk_gemv_grouped_internal(bool q8, const uint8_t *const *packed_ptrs, const uint8_t *const *scales_ptrs, size_t nmat, size_t rows,
                             size_t cols, const int8_t *xq, const float *xs, const float *xf, const int32_t *x_index, float *const *out_ptrs,
                             hipStream_t st) {
    GemvArgs a = {};
    a.packed_ptrs = packed_ptrs;
    a.scales_ptrs = scales_ptrs;
    a.out_ptrs = out_ptrs;
    a.x_index = x_index;
    a.xq = xq;
    a.xs = xs;
    a.xf = xf;
    a.rows = (int)rows;
    return launch_gemv(a, q8, nmat, cols, st);
}

int mk_mxfp4_grouped_gemm_nt(int n_mats, const uint8_t *const *const *packed_ptrs, const uint8_t *const *const *scales_ptrs, size_t n_groups,
                             size_t rows, size_t cols, const float *x, const int32_t *xrow, int xdiv, const int32_t *offsets, size_t m,
                             const float *vq_codebook, float *const *out, void *stream) {
    MK_REQUIRE((n_mats == 1 || n_mats == 2) && packed_ptrs && scales_ptrs && x && offsets && out, "bad argument");
    MK_REQUIRE(rows > 0 && cols > 0 && cols % 128 == 0 && n_groups >= 1 && n_groups <= 65535, "cols must be a multiple of 128, at most 65535 groups");
    MK_REQUIRE(rows <= (size_t)INT32_MAX && ((uintptr_t)x & 15) == 0 && (!xrow || xdiv >= 1), "bad shape or alignment");
    NtGroupedArgs a{};
    for (int k = 0; k < n_mats; k++) {
        MK_REQUIRE(packed_ptrs[k] && scales_ptrs[k] && out[k], "null pointer");
        a.packed[k] = packed_ptrs[k], a.scales[k] = scales_ptrs[k], a.out[k] = out[k];
    }
    a.x = x, a.xrow = xrow, a.offsets = offsets, a.rows = (int)rows, a.nb = (int)(cols / 32), a.xdiv = xdiv;
    MK_REQUIRE(!vq_codebook || ((uintptr_t)vq_codebook & 15) == 0, "the codebook must be 16-byte aligned");
    a.codebook = vq_codebook;
    MK_REQUIRE(rows % 4 == 0 && ((uintptr_t)out[0] & 15) == 0 && (n_mats == 1 || ((uintptr_t)out[1] & 15) == 0), "rows % 4 and 16-byte aligned results");
    // passes of 64 grouped rows (twice the LDS, half the workgroups a CU holds) pay from about 48 rows a group
    const int tiles = MK_TUNE("MK_MXFP4_NT_GROUPED_TILES", 0);
    if (tiles == 4 || (tiles == 0 && m >= 48 * n_groups)) return launch_nt_grouped<8, 4>(a, n_groups, n_mats, (hipStream_t)stream);
    if (MK_TUNE("MK_MXFP4_NT_GROUPED_WAVES", 8) == 8) return launch_nt_grouped<8>(a, n_groups, n_mats, (hipStream_t)stream);
    return launch_nt_grouped<4>(a, n_groups, n_mats, (hipStream_t)stream);
}

int mk_mxfp4_grouped_gemm_bf16(int n_mats, const uint8_t *const *const *packed_ptrs, const uint8_t *const *const *scales_ptrs, size_t n_groups,
                               size_t rows, size_t cols, const uint16_t *x, const int32_t *offsets, float *const *out, void *stream,
                               const uint8_t *const *const *scales_t_ptrs) {
    MK_REQUIRE((n_mats == 1 || n_mats == 2) && packed_ptrs && scales_ptrs && x && offsets && out, "bad argument");
    if (cols == 0 || cols % 512 != 0 || rows % 4 != 0) {
        mk_set_error("the bf16 grouped product takes cols % 512 == 0 and rows % 4 == 0");
        return MK_ERR_UNSUPPORTED;
    }
    MK_REQUIRE(rows > 0 && n_groups >= 1 && n_groups <= 65535 && rows <= (size_t)INT32_MAX && ((uintptr_t)x & 15) == 0, "bad shape or alignment");
    Bf16GroupedArgs a{};
    for (int k = 0; k < n_mats; k++) {
        MK_REQUIRE(packed_ptrs[k] && scales_ptrs[k] && out[k] && ((uintptr_t)out[k] & 15) == 0, "null or unaligned pointer");
        a.packed[k] = packed_ptrs[k], a.scales[k] = scales_ptrs[k], a.out[k] = out[k];
        a.scales_t[k] = scales_t_ptrs ? scales_t_ptrs[k] : nullptr;
    }
    a.x = x, a.offsets = offsets, a.rows = (int)rows, a.nb = (int)(cols / 32);
    constexpr int RW = 8;
    const dim3 grid((unsigned)((rows + 16 * RW - 1) / (16 * RW)), (unsigned)n_groups, (unsigned)n_mats);
    hipLaunchKernelGGL((mxfp4_gemm_bf16_grouped_kernel<RW, 2>), grid, dim3(64 * RW), 0, (hipStream_t)stream, a);
    return mk_launch_status("mxfp4_gemm_bf16_grouped");
}

extern "C" int mk_dev_mxfp4_grouped_gemm_f32(const uint8_t *const *packed_ptrs, const uint8_t *const *scales_ptrs, size_t n_groups, size_t rows,
                                             size_t cols, const float *x, const int32_t *offsets, size_t m, float *out, void *stream) {
    MK_REQUIRE(packed_ptrs && scales_ptrs && x && offsets && out, "null pointer");
    return mk_mxfp4_grouped_gemm_nt(1, &packed_ptrs, &scales_ptrs, n_groups, rows, cols, x, nullptr, 1, offsets, m, nullptr, &out, stream);
}

extern "C" int mk_dev_mxfp4_grouped_gemm_bf16(const uint8_t *const *packed_ptrs, const uint8_t *const *scales_ptrs, size_t n_groups, size_t rows,
                                              size_t cols, const uint16_t *x, const int32_t *offsets, size_t m, float *out, void *stream) {
    MK_REQUIRE(packed_ptrs && scales_ptrs && x && offsets && out, "null pointer");
    (void)m;
    return mk_mxfp4_grouped_gemm_bf16(1, &packed_ptrs, &scales_ptrs, n_groups, rows, cols, x, offsets, &out, stream, nullptr);
}

extern "C" int mk_dev_mxfp4_matvec_nt(const uint8_t *packed, const uint8_t *scales, size_t rows, size_t cols, const float *x, size_t m,
                                      float *out, void *stream) {
    MK_REQUIRE(packed && scales && x && out, "null pointer");
    MK_REQUIRE(shape_ok(rows, cols), "cols must be a positive multiple of 32");
    MK_REQUIRE(((uintptr_t)packed & 15) == 0 && ((uintptr_t)x & 15) == 0, "packed and x must be 16-byte aligned");
    if (rows == 0 || m == 0) return MK_OK;
    if (m >= (size_t)MK_TUNE("MK_MXFP4_NT_MFMA_MIN", 4) && cols % 128 == 0 && m <= 65535 * 64) {
        // many positions: 64 weight rows a workgroup, each step's activations staged in LDS once for all of them
        if (m >= (size_t)MK_TUNE("MK_MXFP4_NT_STAGED_MIN", 512) && m <= 65535 * 32 && rows % 4 == 0 && ((uintptr_t)out & 15) == 0 && rows <= (size_t)INT32_MAX) {
            NtGroupedArgs a{};
            a.out[0] = out, a.x = x, a.rows = (int)rows, a.nb = (int)(cols / 32), a.xdiv = 1;
            a.packed1 = packed, a.scales1 = scales, a.m1 = (int)m;
            if (MK_TUNE("MK_MXFP4_NT_STAGED_TILES", 4) == 4) return launch_nt_grouped<4, 4>(a, (m + 63) / 64, 1, (hipStream_t)stream);
            return launch_nt_grouped<4, 2>(a, (m + 31) / 32, 1, (hipStream_t)stream);
        }
        // waves of a workgroup = shares of the 128-column steps: eight for long rows while the grid is small
        if (cols / 128 >= 16 && (rows + 15) / 16 * ((m + 63) / 64) < 2048)
            return launch_nt_mfma_w<8>(packed, scales, rows, cols, x, m, out, (hipStream_t)stream);
        return launch_nt_mfma_w<4>(packed, scales, rows, cols, x, m, out, (hipStream_t)stream);
    }
    hipLaunchKernelGGL(mxfp4_gemv_nt_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, (hipStream_t)stream, packed, scales, (int)rows,
                       (int)(cols / 32), x, (int)m, out);
    return mk_launch_status("mxfp4_gemv_nt");
}
