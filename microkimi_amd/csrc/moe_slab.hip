// MoE decode layer in ONE streaming launch (plus a small reduction): the expert section of moe_forward / ds_moe
// (src/model.rs:2227-2264,2346-2351; src/deepseek.rs:1069-1106) for a few decode tokens, q8 mode.
//
// The two-launch form (moe.hip) has a grid-wide dependency between gate/up and down: every row of W2 needs the whole
// activation row.  matvec_packed re-quantizes its input per 32 (src/mxfp4.rs:476-487, src/q8.rs:49-69), so ONE q8 block
// of the activation row is self-contained: it is made of 32 consecutive rows of W1 and W3, and it meets W2 in 32
// consecutive columns only.  A workgroup therefore owns (pair, K blocks of 32 rows): it streams those rows of W1 and W3,
// forms the activation values and their q8 blocks, and multiplies them straight into the matching 32-column slabs of W2,
//     part[pair][group][r] = sum over the group's blocks b of  idot(W2[r][32b..32b+31], q_b) * (2^(sb-128) * dx_b),
// the reference's block terms (src/mxfp4.rs:405-443) added in ascending block order.  A second, small kernel adds the
// groups of a pair in ascending order (so o = W2 act is a fixed-order sum of the reference's terms) and then the
// token's pairs in slot order, y += w * o (src/model.rs:2346-2351).  No atomics, no flags: the result is deterministic.
//
// A 32-column slab of the row-major W2 is 16 bytes out of every row (a 1 KiB stride at inter = 2048), so W2 is kept a
// second time in slab-major tiles (mk_dev_mxfp4_to_slab, tab.w2t): tile (b, i) holds the block b of the rows 256 i ..
// 256 i + 255 as 4 x 64 x 16 nibble bytes (row 256 i + 64 j + lane at j * 1024 + lane * 16) followed by 64 x 4 scale bytes
// (lane * 4 + j): 4352 bytes = 34 whole lines, one contiguous 119 KiB stream per slab, a lane owns whole rows (no
// cross-lane reduction) and the q8 block is wave-uniform (scalar registers).
#include "mk_moe.h"

namespace {

constexpr int SLAB_TILE_BYTES = 4352;

__device__ __forceinline__ void mk_lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// ------------------------------------------------------------------ layout
// thread = (row r, block b), b fastest: 16-byte reads along a row are coalesced
__global__ __launch_bounds__(256) void mxfp4_to_slab_kernel(const uint8_t *__restrict__ packed, const uint8_t *__restrict__ scales, int rows,
                                                            int nb, uint8_t *__restrict__ slab) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)rows * nb) return;
    const int r = (int)(i / nb), b = (int)(i % nb);
    const int tile = r >> 8, j = (r >> 6) & 3, lane = r & 63;
    uint8_t *dst = slab + ((size_t)b * (rows >> 8) + tile) * SLAB_TILE_BYTES;
    *reinterpret_cast<mk_i4 *>(dst + j * 1024 + lane * 16) = *reinterpret_cast<const mk_i4 *>(packed + ((size_t)r * nb + b) * 16);
    dst[4096 + lane * 4 + j] = scales[(size_t)r * nb + b];
}

// mxfp4::dequant (src/mxfp4.rs:19-31) read from the slab-major copy: thread = 8 consecutive columns of a row
__global__ __launch_bounds__(256) void mxfp4_slab_dequant_kernel(const uint8_t *__restrict__ slab, int rows, int nb, float *__restrict__ out) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)rows * nb * 4) return;
    const int r = (int)(i / (nb * 4)), wi = (int)(i % (nb * 4)), b = wi >> 2, dd = wi & 3;
    const int tile = r >> 8, j = (r >> 6) & 3, lane = r & 63;
    const uint8_t *src = slab + ((size_t)b * (rows >> 8) + tile) * SLAB_TILE_BYTES;
    const uint32_t w = *reinterpret_cast<const uint32_t *>(src + j * 1024 + lane * 16 + dd * 4);
    const float s = mk_scale_from_byte(src[4096 + lane * 4 + j]);
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

// ------------------------------------------------------------------ the streaming kernel
// Workgroup (pair q, group g) of four waves.  NB = d / 32, K = activation blocks per workgroup, UP = (gate row, up row)
// units a wave keeps in flight.
//   phase 1  wave w streams the rows 32 K g + 8 K w .. + 8 K - 1 of W1 and W3 (a row: LW lanes x T loads of 16 bytes,
//            one scale byte each) against the token's hidden row, whose q8 form (f16 integers + block scales) the
//            workgroup makes itself in LDS while its first weight loads are in flight.
//   phase 2  every wave forms the K q8 blocks of the 32 K activation values (8 lanes a block; the same bytes in every
//            wave) and takes them into scalar registers; wave w owns the 256-row tiles w, w + 4, ... of the K slabs.
//            The first slab items are requested before phase 1's last units are worked on.
template <int NB>
struct SlabRowUnit {
    static constexpr int T = (NB + 63) / 64;
    mk_i4 w1[T], w3[T];
    uint32_t s1[T], s3[T];
};
struct SlabItem {
    mk_i4 w[4];
    uint32_t sc;
};

template <int NB, int K, int UP>
__global__ __launch_bounds__(256) void moe_slab_kernel(FusedArgs a, int stage, float *__restrict__ part) {
    constexpr int T = (NB + 63) / 64, LW = NB / T;
    constexpr int TPW = NB / 32;  // 256-row tiles per wave: d = 32 NB = 4 waves x TPW x 256 rows
    constexpr int NT = NB / 8;    // tiles per slab
    constexpr int NU = 8 * K;     // units per wave
    constexpr int NI = TPW * K;   // slab items per wave
    constexpr int R2 = NI < 4 ? NI : 4;
    constexpr int NX = NB * 8;    // 16-byte pieces of a hidden row
    constexpr int SB = NX / 256;
    static_assert(NB % 32 == 0 && NB % T == 0 && T <= 4 && NU % UP == 0 && NX % 256 == 0, "shape not covered");
    __shared__ __attribute__((aligned(16))) uint32_t xh[NB * 16];  // q8 of the hidden row as f16 pairs, [4 chunks][NB][4 words]
    __shared__ float xsc[NB];
    __shared__ __attribute__((aligned(16))) float act_l[32 * K];

    const int lane = threadIdx.x & 63, lane_c = lane < LW ? lane : LW - 1;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int G = a.inter / (32 * K);
    const int q = blockIdx.x / G, g = blockIdx.x - q * G;
    const int tok = q / a.per, slot = q - tok * a.per;
    bool ok = true;
    const int e = __builtin_amdgcn_readfirstlane(slot < a.topk ? mk_checked_expert(a.ids[tok * a.topk + slot], a.tab.n_experts, ok) : a.shared);
    const uint8_t *w2t = mk_uniform_ptr(a.tab.w2t[e]);

    SlabItem it[R2];
    auto load_item = [&](SlabItem &I, int n) {
        const int i = n / K, blk = n - i * K;
        const uint32_t off = (uint32_t)(((K * g + blk) * NT + wave + 4 * i) * SLAB_TILE_BYTES);
#pragma unroll
        for (int j = 0; j < 4; j++) I.w[j] = mk_ldg128_off_nt(w2t, off + j * 1024 + lane * 16);
        I.sc = __builtin_nontemporal_load((const MK_GLOBAL uint32_t *)((const MK_GLOBAL uint8_t *)w2t + off + 4096 + lane * 4));
    };

    if (stage != MK_MOE_STAGE_FROM_ACT) {
        // q8 of the hidden row (src/q8.rs:57-68): 8 lanes per 32-block, one 16-byte load each, requested first
        const mk_f4 *xsrc = reinterpret_cast<const mk_f4 *>(a.x + (size_t)tok * NB * 32);
        mk_f4 xv[SB];
#pragma unroll
        for (int b = 0; b < SB; b++) xv[b] = xsrc[threadIdx.x + b * 256];
        const float wgt = slot < a.topk ? (ok ? a.weights[tok * a.topk + slot] : 0.0f) : 1.0f;
        const uint8_t *p1 = mk_uniform_ptr(a.tab.w1p[e]), *p3 = mk_uniform_ptr(a.tab.w3p[e]);
        const uint8_t *c1 = mk_uniform_ptr(a.tab.w1s[e]), *c3 = mk_uniform_ptr(a.tab.w3s[e]);
        const int row0 = 32 * K * g + NU * wave;
        SlabRowUnit<NB> ring[UP];
        auto load_unit = [&](SlabRowUnit<NB> &U, int u) {
            const uint32_t boff = (uint32_t)(row0 + u) * NB + lane_c;
#pragma unroll
            for (int t = 0; t < T; t++) {
                U.w1[t] = mk_ldg128_off_nt(p1, (boff + t * LW) * 16);
                U.w3[t] = mk_ldg128_off_nt(p3, (boff + t * LW) * 16);
                U.s1[t] = mk_ldg_u8_off(c1, boff + t * LW);
                U.s3[t] = mk_ldg_u8_off(c3, boff + t * LW);
            }
        };
#pragma unroll
        for (int k = 0; k < UP; k++) load_unit(ring[k], k);
#pragma unroll
        for (int b = 0; b < SB; b++) {
            const int i = threadIdx.x + b * 256;
            const mk_f4 v = xv[b];
            float mx = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
            mx = fmaxf(mx, mk_dpp<0xB1>(mx));
            mx = fmaxf(mx, mk_dpp<0x4E>(mx));
            mx = fmaxf(mx, mk_dpp<0x141>(mx));
            const float dx = fmaxf(mx, 0.0f) / 127.0f;  // (a block of NaN only: the reference's maximum, folded from 0, is 0)
            mk_h2 lo = {(_Float16)0.0f, (_Float16)0.0f}, hi = lo;
            if (dx != 0.0f) mk_q8_round4_f16(v, dx, lo, hi);
            const int gb = i >> 3, j = i & 7;
            uint32_t *dst = xh + ((j >> 1) * NB + gb) * 4 + 2 * (j & 1);
            dst[0] = __builtin_bit_cast(uint32_t, lo);
            dst[1] = __builtin_bit_cast(uint32_t, hi);
            if (j == 0) xsc[gb] = dx;
        }
        mk_lds_barrier();

        auto compute_unit = [&](const SlabRowUnit<NB> &U, int u) {
            float s1 = 0.0f, s3 = 0.0f;
#pragma unroll
            for (int t = 0; t < T; t++) {
                const int gb = t * LW + lane_c;
                mk_h2 xr[16];
#pragma unroll
                for (int kk = 0; kk < 4; kk++) {
                    // (read word by word: a bit cast of an element of an ext-vector reads element 0 for every index)
                    const uint32_t *xp = xh + (kk * NB + gb) * 4;
#pragma unroll
                    for (int c = 0; c < 4; c++) xr[kk * 4 + c] = __builtin_bit_cast(mk_h2, xp[c]);
                }
                const float cf = xsc[gb];
                const float h1 = mk_dot32_fp4_f16(U.w1[t], xr), h3 = mk_dot32_fp4_f16(U.w3[t], xr);
                s1 += (h1 + h1) * (mk_half_scale_from_byte(U.s1[t]) * cf);
                s3 += (h3 + h3) * (mk_half_scale_from_byte(U.s3[t]) * cf);
            }
            if (lane >= LW) s1 = s3 = 0.0f;
            const float gsum = mk_wave_sum(s1), usum = mk_wave_sum(s3);
            const float act = mk_act(a.act_kind, gsum, usum, a.limit, wgt);
            if (lane == 0) {
                act_l[NU * wave + u] = act;
                if (stage == MK_MOE_STAGE_ACT) a.af[(size_t)q * a.inter + row0 + u] = act;
            }
        };
#pragma unroll 1
        for (int u0 = 0; u0 < NU - UP; u0 += UP) {
#pragma unroll
            for (int k = 0; k < UP; k++) {
                compute_unit(ring[k], u0 + k);
                load_unit(ring[k], u0 + k + UP);
            }
        }
#pragma unroll
        for (int k = 0; k < UP; k++) {
            if (k < R2) load_item(it[k], k);
            compute_unit(ring[k], NU - UP + k);
        }
#pragma unroll
        for (int k = UP; k < R2; k++) load_item(it[k], k);
        if (stage == MK_MOE_STAGE_ACT) return;
    } else {
#pragma unroll
        for (int k = 0; k < R2; k++) load_item(it[k], k);
        if (threadIdx.x < 32 * K) act_l[threadIdx.x] = a.af[(size_t)q * a.inter + 32 * K * g + threadIdx.x];
    }
    mk_lds_barrier();

    // q8 of the K activation blocks (what matvec_packed does to its input): lanes 8 b .. 8 b + 7 hold block b
    mk_h2 xa[K][16];
    float dxs[K];
    {
        const mk_f4 v = *reinterpret_cast<const mk_f4 *>(act_l + 4 * (lane & (8 * K - 1)));
        float mx = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
        mx = fmaxf(mx, mk_dpp<0xB1>(mx));
        mx = fmaxf(mx, mk_dpp<0x4E>(mx));
        mx = fmaxf(mx, mk_dpp<0x141>(mx));
        const float dx = fmaxf(mx, 0.0f) / 127.0f;
        mk_h2 lo = {(_Float16)0.0f, (_Float16)0.0f}, hi = lo;
        if (dx != 0.0f) mk_q8_round4_f16(v, dx, lo, hi);
        const int lo_i = __builtin_bit_cast(int, lo), hi_i = __builtin_bit_cast(int, hi);
#pragma unroll
        for (int b = 0; b < K; b++) {
            dxs[b] = mk_readlane(dx, 8 * b);
#pragma unroll
            for (int j = 0; j < 8; j++) {
                xa[b][2 * j] = __builtin_bit_cast(mk_h2, __builtin_amdgcn_readlane(lo_i, 8 * b + j));
                xa[b][2 * j + 1] = __builtin_bit_cast(mk_h2, __builtin_amdgcn_readlane(hi_i, 8 * b + j));
            }
        }
    }

    float y[TPW][4];
#pragma unroll
    for (int i = 0; i < TPW; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) y[i][j] = 0.0f;
#pragma unroll
    for (int n = 0; n < NI; n++) {
        const SlabItem &I = it[n % R2];
        const int i = n / K, blk = n - i * K;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float h = mk_dot32_fp4_f16(I.w[j], xa[blk]);
            y[i][j] = mk_add(y[i][j], (h + h) * (mk_half_scale_from_byte((I.sc >> (8 * j)) & 255u) * dxs[blk]));
        }
        if (n + R2 < NI) load_item(it[n % R2], n + R2);
    }
    float *dst = part + (size_t)blockIdx.x * (NB * 32);
#pragma unroll
    for (int i = 0; i < TPW; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) dst[(wave + 4 * i) * 256 + j * 64 + lane] = y[i][j];
}

// out[t][r] = sum over the token's pairs in slot order of w * o, o = the pair's groups added in ascending order.
// grid (d / 64, B), block (64, per): thread (rl, s) adds the groups of pair (t, s) at row 64 blockIdx.x + rl.
__global__ __launch_bounds__(1024) void moe_slab_reduce_kernel(FusedArgs a, const float *__restrict__ part, int G) {
    __shared__ float o_l[16][64];
    const int rl = threadIdx.x, s = threadIdx.y, t = blockIdx.y, per = a.per;
    const int row = blockIdx.x * 64 + rl;
    const float *src = part + ((size_t)(t * per + s) * G) * a.d + row;
    float o = 0.0f;
    int g = 0;
    for (; g + 8 <= G; g += 8) {
        float v[8];
#pragma unroll
        for (int k = 0; k < 8; k++) v[k] = src[(size_t)(g + k) * a.d];
#pragma unroll
        for (int k = 0; k < 8; k++) o = mk_add(o, v[k]);
    }
    for (; g < G; g++) o = mk_add(o, src[(size_t)g * a.d]);
    o_l[s][rl] = o;
    __syncthreads();
    if (s != 0) return;
    float y = 0.0f;
    for (int k = 0; k < per; k++) {
        float pw = 1.0f;
        if (k < a.topk) {
            bool ok = true;
            mk_checked_expert(a.ids[t * a.topk + k], a.tab.n_experts, ok);
            pw = !ok ? 0.0f : a.ds_rule ? 1.0f : a.weights[t * a.topk + k];
        }
        y = mk_add(y, mk_mul(pw, o_l[k][rl]));
    }
    a.out[(size_t)t * a.d + row] = y;
}

template <int NB, int K, int UP>
int launch_slab(const FusedArgs &a, size_t P, int stage, float *part, hipStream_t st) {
    const int G = a.inter / (32 * K);
    hipLaunchKernelGGL((moe_slab_kernel<NB, K, UP>), dim3((unsigned)(P * G)), dim3(256), 0, st, a, stage, part);
    return mk_launch_status("moe_slab");
}

template <int NB>
int launch_slab_nb(const FusedArgs &a, size_t P, int stage, float *part, int k, hipStream_t st) {
    const int up = MK_TUNE("MK_MOE_SLAB_UP", 4);
    if (k == 1) return up == 2 ? launch_slab<NB, 1, 2>(a, P, stage, part, st) : launch_slab<NB, 1, 4>(a, P, stage, part, st);
    return up == 2 ? launch_slab<NB, 2, 2>(a, P, stage, part, st) : launch_slab<NB, 2, 4>(a, P, stage, part, st);
}

int slab_k(size_t inter) {
    const int k = MK_TUNE("MK_MOE_SLAB_K", 2);
    return (k == 2 && inter % 64 == 0) ? 2 : 1;
}

}  // namespace

bool mk_moe_slab_takes(size_t d, size_t inter, int per) {
    const size_t nb = d / 32;
    return (nb == 32 || nb == 64 || nb == 128 || nb == 224) && d % 1024 == 0 && inter % 32 == 0 && per <= 16 && inter * (d / 2) < 0x7FFFFFFFull;
}

size_t mk_moe_slab_part_bytes(size_t P, size_t d, size_t inter) { return P * (inter / 32) * d * sizeof(float); }

int mk_moe_slab_launch(const FusedArgs &a, size_t B, int stage, float *part, hipStream_t st) {
    const size_t P = B * a.per;
    const int k = slab_k(a.inter);
    int s;
    switch (a.d / 32) {
        case 32: s = launch_slab_nb<32>(a, P, stage, part, k, st); break;
        case 64: s = launch_slab_nb<64>(a, P, stage, part, k, st); break;
        case 128: s = launch_slab_nb<128>(a, P, stage, part, k, st); break;
        case 224: s = launch_slab_nb<224>(a, P, stage, part, k, st); break;
        default: mk_set_error("moe_slab: d = %d not covered", a.d); return MK_ERR_UNSUPPORTED;
    }
    if (s != MK_OK || stage == MK_MOE_STAGE_ACT) return s;
    hipLaunchKernelGGL(moe_slab_reduce_kernel, dim3((unsigned)(a.d / 64), (unsigned)B), dim3(64, a.per), 0, st, a, part, a.inter / (32 * k));
    return mk_launch_status("moe_slab_reduce");
}

extern "C" size_t mk_mxfp4_slab_bytes(size_t rows, size_t cols) { return rows * (cols / 32) * 17; }

extern "C" int mk_dev_mxfp4_to_slab(const uint8_t *packed, const uint8_t *scales, size_t rows, size_t cols, uint8_t *slab, void *stream) {
    MK_REQUIRE(packed && scales && slab, "null pointer");
    MK_REQUIRE(rows > 0 && rows % 256 == 0 && cols > 0 && cols % 32 == 0, "rows must be a multiple of 256 and cols of 32");
    MK_REQUIRE(rows * (cols / 32) * 17 < 0x7FFFFFFFull, "matrix too large for the slab form");
    MK_REQUIRE((((uintptr_t)packed | (uintptr_t)slab) & 15) == 0, "packed and slab must be 16-byte aligned");
    const size_t n = rows * (cols / 32);
    hipLaunchKernelGGL(mxfp4_to_slab_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, packed, scales, (int)rows,
                       (int)(cols / 32), slab);
    return mk_launch_status("mxfp4_to_slab");
}

extern "C" int mk_dev_mxfp4_slab_dequant(const uint8_t *slab, size_t rows, size_t cols, float *out, void *stream) {
    MK_REQUIRE(slab && out, "null pointer");
    MK_REQUIRE(rows > 0 && rows % 256 == 0 && cols > 0 && cols % 32 == 0, "rows must be a multiple of 256 and cols of 32");
    MK_REQUIRE((((uintptr_t)slab | (uintptr_t)out) & 15) == 0, "slab and out must be 16-byte aligned");
    const size_t n = rows * (cols / 32) * 4;
    hipLaunchKernelGGL(mxfp4_slab_dequant_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, slab, (int)rows,
                       (int)(cols / 32), out);
    return mk_launch_status("mxfp4_slab_dequant");
}
