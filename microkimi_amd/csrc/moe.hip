// MoE decode layer: the expert section of moe_forward / ds_moe
// (src/model.rs:2227-2264,2346-2351; src/deepseek.rs:1069-1106) for B tokens as
// one grouped pass over the (token, slot) pairs.
//
// Fast path (q8 mode, benchmark-like shapes): two fused launches, see below.
// Composed path (any shape, both modes):
//   setup     pair tables (expert pointers per pair) from the router's ids
//   quantize  x -> q8 (once per token; gate and up quantize the same input to
//             the same bytes in the reference)
//   gate, up  grouped MXFP4 GEMVs over all pairs, elementwise activation,
//             q8 quantization of the activation
//   down      o = W2 act: the grouped MXFP4 GEMV over all pairs
//   combine   out_t = sum_slot w * o in slot order (+ shared expert)
//
// HBM traffic: every selected expert's 23.4 MB is read once per pair; the
// intermediates (act: 2 KiB + 256 B per pair, o: 28 KiB per pair) are noise.
#include <stdlib.h>

#include "mk_moe.h"

// grouped MXFP4 GEMV of gemv_mxfp4.hip: q8 (xq, xs) or f32 (xf) activations, one launch over nmat matrices
int mk_gemv_grouped_internal(bool q8, const uint8_t *const *packed_ptrs, const uint8_t *const *scales_ptrs, size_t nmat, size_t rows,
                             size_t cols, const int8_t *xq, const float *xs, const float *xf, const int32_t *x_index, float *const *out_ptrs,
                             hipStream_t st);

// grouped VQ1 LUT GEMV of vq1.hip: tables for n_vec activation vectors, then the sweep over the matrices whose marker
// pointer is null
int mk_vq1_grouped_tables(const float *codebook, const float *x, size_t n_vec, size_t cols, const uint8_t *const *marker_ptrs, float *lut,
                          hipStream_t st);
int mk_vq1_grouped_sweep(const float *lut, const int32_t *vec_index, const uint8_t *const *idx_ptrs, const uint8_t *const *marker_ptrs,
                         size_t n_mat, size_t rows, size_t cols, float *const *out_ptrs, hipStream_t st);

int mk_q8x_grouped(int n_mats, const uint8_t *const *const *packed_ptrs, const uint8_t *const *const *scales_ptrs, size_t rows, size_t cols,
                   const int8_t *xq, const float *xs, const int32_t *arow, const int32_t *goff, const int32_t *gexp, const int32_t *ngroups,
                   const int32_t *gbig, size_t max_groups, size_t max_group_rows, float *const *out, void *stream,
                   const uint8_t *const *const *scales_t_ptrs);

namespace {

constexpr int gcd_c(int a, int b) { return b == 0 ? a : gcd_c(b, a % b); }
constexpr int lcm_c(int a, int b) { return a / gcd_c(a, b) * b; }

struct PairTables {
    const uint8_t **w1p, **w1s, **w3p, **w3s, **w2p, **w2s;  // [P]
    float **optr;                                            // [P] -> o [P][d]
    float **gptr, **uptr;                                    // [P] -> g, u [P][inter] (composed path)
    int32_t *xidx;                                           // [P] token of the pair (activation row)
    int32_t *aidx;                                           // [P] = p (act row of the pair)
    float *pw;                                               // [P] routing weight of the pair (1 for shared)
};

struct Workspace {
    PairTables pt;
    int8_t *xq;   // [B][d]
    float *xs;    // [B][d/32]
    int8_t *aq;   // [P][inter]
    float *as;    // [P][inter/32]
    float *af;    // [P][inter]   (f32 mode)
    float *g;     // [P][inter]   (composed path)
    float *u;     // [P][inter]
    float *o;     // [P][d]
    // batched path: the pairs grouped by expert
    int32_t *order;    // [P] grouped row -> pair
    int32_t *pos;      // [P] pair -> grouped row
    int32_t *rtok;     // [P] grouped row -> token
    int32_t *goff;     // [P + 1] first grouped row of every group
    int32_t *gexp;     // [P] expert of every group
    int32_t *ngroups;  // [2]: number of groups, index of the largest group
    void *lines;       // one-launch path: [P][inter] 8-byte units (activation value, launch tag)
    size_t bytes;
};

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }


Workspace carve(void *base, size_t B, size_t topk, int has_shared, size_t d, size_t inter) {
    const size_t P = B * (topk + (has_shared ? 1 : 0));
    uint8_t *p = (uint8_t *)base;
    size_t off = 0;
    auto take = [&](size_t bytes) {
        uint8_t *r = p ? p + off : nullptr;
        off += align_up(bytes, 256);
        return r;
    };
    Workspace w;
    w.pt.w1p = (const uint8_t **)take(P * 8);
    w.pt.w1s = (const uint8_t **)take(P * 8);
    w.pt.w3p = (const uint8_t **)take(P * 8);
    w.pt.w3s = (const uint8_t **)take(P * 8);
    w.pt.w2p = (const uint8_t **)take(P * 8);
    w.pt.w2s = (const uint8_t **)take(P * 8);
    w.pt.optr = (float **)take(P * 8);
    w.pt.gptr = (float **)take(P * 8);
    w.pt.uptr = (float **)take(P * 8);
    w.pt.xidx = (int32_t *)take(P * 4);
    w.pt.aidx = (int32_t *)take(P * 4);
    w.pt.pw = (float *)take(P * 4);
    w.xq = (int8_t *)take(B * d);
    w.xs = (float *)take(B * (d / 32) * 4);
    w.aq = (int8_t *)take(P * inter);
    w.as = (float *)take(P * (inter / 32) * 4);
    w.af = (float *)take(P * inter * 4);
    w.g = (float *)take(P * inter * 4);
    w.u = (float *)take(P * inter * 4);
    w.o = (float *)take(P * d * 4);
    w.order = (int32_t *)take(P * 4);
    w.pos = (int32_t *)take(P * 4);
    w.rtok = (int32_t *)take(P * 4);
    w.goff = (int32_t *)take((P + 1) * 4);
    w.gexp = (int32_t *)take(P * 4);
    w.ngroups = (int32_t *)take(8);
    w.lines = (void *)take(B <= 3 ? mk_moe_persist_lines_bytes(P, inter) : 0);
    w.bytes = off;
    return w;
}

__global__ void moe_setup_kernel(mk_expert_table tab, int B, int topk, int shared, const int32_t *__restrict__ ids,
                                 const float *__restrict__ weights, PairTables pt, float *o, float *g, float *u, int d, int inter) {
    const int per = topk + (shared >= 0 ? 1 : 0);
    const int p = blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= B * per) return;
    const int t = p / per, s = p % per;
    bool ok = true;
    const int e = s < topk ? mk_checked_expert(ids[t * topk + s], tab.n_experts, ok) : shared;
    pt.w1p[p] = tab.w1p[e];
    pt.w1s[p] = tab.w1s[e];
    pt.w3p[p] = tab.w3p[e];
    pt.w3s[p] = tab.w3s[e];
    pt.w2p[p] = tab.w2p[e];
    pt.w2s[p] = tab.w2s[e];
    pt.optr[p] = o + (size_t)p * d;
    pt.gptr[p] = g + (size_t)p * inter;
    pt.uptr[p] = u + (size_t)p * inter;
    pt.xidx[p] = t;
    pt.aidx[p] = p;
    pt.pw[p] = s < topk ? (ok ? weights[t * topk + s] : 0.0f) : 1.0f;
}

// ------------------------------------------------------------ fused fast path
// Two launches per layer, no setup / quantize / combine kernels:
//
//   gate_up  one resident workgroup of 8 waves per CU.  Wave w owns the rows w,
//            w + W, ... of W1 and W3 in every (token, slot) pair and streams them
//            pair after pair; the workgroup quantizes the hidden rows to q8
//            itself (src/q8.rs:57-68) while its first weight loads are in
//            flight, and a lane keeps the activation blocks it owns in registers.
//            Every wave has the same number of rows: no tail.  The activation
//            value ACT(W1 x, W3 x) goes out in f32.
//   down     grid (tokens, blocks).  The workgroup forms the q8 blocks of the
//            token's activation rows in LDS (the block matvec_packed forms when
//            it re-quantizes its input for W2).  The rows of W2 are dealt
//            round-robin to the token's waves; a wave walks its rows pair by
//            pair in slot order and accumulates y += w * (W2_e act) in registers,
//            so the weighted sum of src/model.rs:2346-2351 needs no intermediate
//            buffer.
// Row-owner gate/up: wave w owns the rows w, w + W, ... of W1 and W3 in every pair
// (three units = 3 x 2 rows in flight per wave).  Tokens are taken in groups
// that fit LDS (q8 of the hidden rows as f16 pairs); a lane keeps the activation
// blocks it owns in registers and re-reads them from LDS only when the token
// changes.  Walking the pairs in expert order instead, so that a repeated expert
// finds its rows in the XCD's L2, was measured and gave nothing (B = 16: 577 us
// against 569 us in token order): at 8 tokens and more the kernel is bound by the
// vector unit's work per pair, not by where the bytes come from.  The stronger
// form was measured too: pairs sorted by expert inside the token group and one
// pass over an expert's rows for all pairs of its run (72 pairs of a group meet
// about 59 distinct experts; the shared expert is then read once per group, not
// once per token).  The fetched bytes went down, the time did not (B = 4: 150 ->
// 154 us, B = 16: 535 -> 532 us, B = 1 unchanged), so the kernel keeps the
// simpler (token, slot) order.
struct RowUnit4 {
    mk_i4 w1[4], w3[4];
    uint32_t s1[4], s3[4];
};

template <int NB>
__global__ __launch_bounds__(512) void moe_gate_up_rows_kernel(FusedArgs a, int B, int tg) {
    constexpr int T = (NB + 63) / 64;  // loads per row
    constexpr int LW = NB / T;         // lanes that carry a row (56 at NB = 224)
    static_assert(NB % T == 0 && T <= 4, "row shape not covered");
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
    const int per = a.per, gp_max = tg * per;
    uint32_t *xh = lds;                                                   // [tg][NB * 16] f16 pairs, [4 chunks][NB][4 words]
    float *xsc = reinterpret_cast<float *>(xh + (size_t)tg * NB * 16);   // [tg][NB]
    const uint8_t **wp1 = reinterpret_cast<const uint8_t **>(xsc + (size_t)tg * NB);
    const uint8_t **wp3 = wp1 + gp_max, **ws1 = wp3 + gp_max, **ws3 = ws1 + gp_max;
    float *wgt_l = reinterpret_cast<float *>(ws3 + gp_max);
    int *next_l = reinterpret_cast<int *>(wgt_l + gp_max);  // the workgroup's unit counter (units are taken, not owned)

    const int lane = threadIdx.x & 63, lane_c = lane < LW ? lane : LW - 1;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nw = gridDim.x * 8, w = blockIdx.x * 8 + wave;
    // rows of this workgroup: 8 b + i + j nw for i < 8, j < J (the same J for all its waves); a row beyond the last one
    // is read as row inter - 1 and stored nowhere: loads under a condition would make every later wait a full one
    const int wg_row0 = (int)blockIdx.x * 8;
    const int J = wg_row0 < a.inter ? (a.inter - wg_row0 + nw - 1) / nw : 1;
    for (int t0 = 0; t0 < B; t0 += tg) {
        const int nt = min(tg, B - t0), gp = nt * per;
        // q8 of the group's hidden rows (src/q8.rs:57-68): 8 lanes per 32-block, one 16-byte load each.  The first batch
        // of loads is issued before anything else, so that it returns ahead of the first weight loads.
        constexpr int SB = 4;
        const mk_f4 *xsrc = reinterpret_cast<const mk_f4 *>(a.x + (size_t)t0 * NB * 32);
        const int n_x = nt * NB * 8;
        mk_f4 xv[SB];
        auto stage_load = [&](mk_f4 *v, int i0) {
#pragma unroll
            for (int b = 0; b < SB; b++) v[b] = xsrc[min(i0 + b * 512, n_x - 1)];
        };
        auto stage_store = [&](const mk_f4 *v, int i0) {
#pragma unroll
            for (int b = 0; b < SB; b++) {
                const int i = i0 + b * 512;
                float mx = fmaxf(fmaxf(fabsf(v[b].x), fabsf(v[b].y)), fmaxf(fabsf(v[b].z), fabsf(v[b].w)));
                mx = fmaxf(mx, mk_dpp<0xB1>(mx));
                mx = fmaxf(mx, mk_dpp<0x4E>(mx));
                mx = fmaxf(mx, mk_dpp<0x141>(mx));
                const float dx = fmaxf(mx, 0.0f) / 127.0f;  // (a block of NaN only: the reference's maximum, folded from 0, is 0)
                mk_h2 lo = {(_Float16)0.0f, (_Float16)0.0f}, hi = lo;
                if (dx != 0.0f) mk_q8_round4_f16(v[b], dx, lo, hi);
                if (i < n_x) {
                    const int tl = i / (NB * 8), g = (i / 8) % NB, j = i % 8;
                    uint32_t *dst = xh + (size_t)tl * NB * 16 + ((j >> 1) * NB + g) * 4 + 2 * (j & 1);
                    dst[0] = __builtin_bit_cast(uint32_t, lo);
                    dst[1] = __builtin_bit_cast(uint32_t, hi);
                    if (j == 0) xsc[tl * NB + g] = dx;
                }
            }
        };
        stage_load(xv, threadIdx.x);
        if (t0) __syncthreads();  // the previous group's LDS is still being read
        if (threadIdx.x < gp) {
            const int q = threadIdx.x, tok = t0 + q / per, slot = q % per;
            bool ok = true;
            const int e = slot < a.topk ? mk_checked_expert(a.ids[tok * a.topk + slot], a.tab.n_experts, ok) : a.shared;
            wp1[q] = a.tab.w1p[e];
            wp3[q] = a.tab.w3p[e];
            ws1[q] = a.tab.w1s[e];
            ws3[q] = a.tab.w3s[e];
            wgt_l[q] = slot < a.topk ? (ok ? a.weights[tok * a.topk + slot] : 0.0f) : 1.0f;
        }
        __syncthreads();

        // The workgroup's units -- (pair, one of its 8 J rows) -- are taken by its waves from a counter in LDS instead of
        // being dealt in advance: the waves of a workgroup are served unevenly by the memory system (with equal shares
        // they finished up to 5 us apart), so the faster ones take more.  The first three units of a wave are fixed.
        const int upw = 8 * J, n_units = gp * upw;
        RowUnit4 ua, ub, uc;
        auto load_unit = [&](RowUnit4 &U, int u) {
            // past the end (the loads stay unconditional): every lane reads the first block of the last pair's matrices,
            // one line per load instead of a row (the streaming loads would fetch a repeated row again)
            const bool past = u >= n_units;
            u = __builtin_amdgcn_readfirstlane(min(u, n_units - 1));
            const int q = u / upw, r = u - q * upw;  // pairs in (token, slot) order
            const uint8_t *p1 = mk_uniform_ptr(wp1[q]), *p3 = mk_uniform_ptr(wp3[q]);
            const uint8_t *c1 = mk_uniform_ptr(ws1[q]), *c3 = mk_uniform_ptr(ws3[q]);
            const uint32_t boff = past ? 0u : (uint32_t)min((int)blockIdx.x * 8 + (r & 7) + (r >> 3) * nw, a.inter - 1) * NB + lane_c;
#pragma unroll
            for (int t = 0; t < T; t++) {
                U.w1[t] = mk_ldg128_off_nt(p1, (boff + t * LW) * 16);
                U.w3[t] = mk_ldg128_off_nt(p3, (boff + t * LW) * 16);
                U.s1[t] = mk_ldg_u8_off(c1, boff + t * LW);
                U.s3[t] = mk_ldg_u8_off(c3, boff + t * LW);
            }
        };
        int ia = wave, ib = wave + 8, ic = wave + 16;
        if (threadIdx.x == 0) *next_l = 24;
        load_unit(ua, ia);  // in flight while the hidden rows are quantized (a third unit here spills registers)
        load_unit(ub, ib);

        stage_store(xv, threadIdx.x);
        for (int i0 = threadIdx.x + 512 * SB; i0 < n_x; i0 += 512 * SB) {
            stage_load(xv, i0);
            stage_store(xv, i0);
        }
        __syncthreads();

        {
            mk_h2 xr[T][16];
            float cf[T];
            int cur_tok = -1;
            auto compute_unit = [&](const RowUnit4 &U, int u) {
                // The waves that share a SIMD (w and w + 4) take turns at the higher issue priority, unit by unit: left
                // alone the older wave of each pair is served first all the time and finishes a quarter earlier (waves
                // 0-3 done at 19 us, waves 4-7 at 25 us at B = 1).  With the rotation they end within 3 us of each other;
                // the kernel itself gains little (B = 4: 172 -> 166 us), the younger waves end when they did before.
                if ((u + (wave >> 2)) & 1) __builtin_amdgcn_s_setprio(1);
                else __builtin_amdgcn_s_setprio(0);
                const int q = u / upw, r = u - q * upw;  // pairs in (token, slot) order
                const int row = (int)blockIdx.x * 8 + (r & 7) + (r >> 3) * nw;
                const int tl = q / per;
                if (tl != cur_tok) {
                    cur_tok = tl;
                    const uint32_t *src = xh + (size_t)tl * NB * 16;
#pragma unroll
                    for (int t = 0; t < T; t++) {
                        const int g = t * LW + lane_c;
#pragma unroll
                        for (int kk = 0; kk < 16; kk++) xr[t][kk] = __builtin_bit_cast(mk_h2, src[((kk >> 2) * NB + g) * 4 + (kk & 3)]);
                        cf[t] = xsc[tl * NB + g];
                    }
                }
                float s1 = 0.0f, s3 = 0.0f;
#pragma unroll
                for (int t = 0; t < T; t++) {
                    const float h1 = mk_dot32_fp4_f16(U.w1[t], xr[t]), h3 = mk_dot32_fp4_f16(U.w3[t], xr[t]);
                    s1 += (h1 + h1) * (mk_half_scale_from_byte(U.s1[t]) * cf[t]);
                    s3 += (h3 + h3) * (mk_half_scale_from_byte(U.s3[t]) * cf[t]);
                }
                if (lane >= LW) s1 = s3 = 0.0f;
                const float gsum = mk_wave_sum(s1), usum = mk_wave_sum(s3);
                const float act = mk_act(a.act_kind, gsum, usum, a.limit, wgt_l[q]);
                if (lane == 0 && row < a.inter) a.af[(size_t)(t0 * per + q) * a.inter + row] = act;
            };
            auto take = [&]() {
                int v = 0;
                if (lane == 0) v = atomicAdd(next_l, 1);
                return __builtin_amdgcn_readfirstlane(v);
            };
            // unit ids grow along a wave's sequence: once one is past the end, so are the later ones
            while (ia < n_units) {
                load_unit(uc, ic);
                const int na = take();
                compute_unit(ua, ia);
                ia = na;
                load_unit(ua, ia);
                const int nb2 = take();
                if (ib < n_units) compute_unit(ub, ib);
                ib = nb2;
                load_unit(ub, ib);
                const int nc = take();
                if (ic < n_units) compute_unit(uc, ic);
                ic = nc;
            }
        }
    }
}

constexpr int MAX_PER = 32;  // pairs per token the fused down kernel keeps in LDS

template <int NB, int U, int WAVES>  // U = tiles per register block
__global__ __launch_bounds__(WAVES * 64) void moe_down_fused_kernel(FusedArgs a) {
    constexpr int TILE = lcm_c(NB, 64);
    constexpr int T = TILE / 64;
    constexpr int RT = TILE / NB;
    static_assert(RT <= 2 && T <= 2 && U * T <= 8, "tile shape not covered by the fused down kernel");
    // per pair: the activation as f16 pairs, [4 chunks][NB blocks][4 words] (see
    // the gate/up kernel); after all pairs, their block scales [per][NB]
    extern __shared__ __attribute__((aligned(16))) uint32_t ah[];
    __shared__ const uint8_t *wp_l[MAX_PER];
    __shared__ const uint8_t *ws_l[MAX_PER];
    __shared__ float pw_l[MAX_PER];
    const int tok = blockIdx.x, per = a.per;  // tokens fastest: they walk the rows in step
    float *asc = reinterpret_cast<float *>(ah + (size_t)per * NB * 16);
    // q8 of the activation rows (what matvec_packed does to its input, src/q8.rs:49-69): 8 lanes per 32-block, one
    // 16-byte load each; the first batch of loads is issued before anything else
    constexpr int SB = 6;
    const mk_f4 *af = reinterpret_cast<const mk_f4 *>(a.af + (size_t)tok * per * NB * 32);
    const int n_a = per * NB * 8;
    mk_f4 av[SB];
    auto stage_load = [&](mk_f4 *v, int i0) {
#pragma unroll
        for (int b = 0; b < SB; b++) v[b] = af[min(i0 + b * WAVES * 64, n_a - 1)];
    };
    auto stage_store = [&](const mk_f4 *v, int i0) {
#pragma unroll
        for (int b = 0; b < SB; b++) {
            const int i = i0 + b * WAVES * 64;
            float mx = fmaxf(fmaxf(fabsf(v[b].x), fabsf(v[b].y)), fmaxf(fabsf(v[b].z), fabsf(v[b].w)));
            mx = fmaxf(mx, mk_dpp<0xB1>(mx));
            mx = fmaxf(mx, mk_dpp<0x4E>(mx));
            mx = fmaxf(mx, mk_dpp<0x141>(mx));
            const float dx = fmaxf(mx, 0.0f) / 127.0f;  // (a block of NaN only: the reference's maximum, folded from 0, is 0)
            mk_h2 lo = {(_Float16)0.0f, (_Float16)0.0f}, hi = lo;
            if (dx != 0.0f) mk_q8_round4_f16(v[b], dx, lo, hi);
            if (i < n_a) {
                const int s = i / (NB * 8), g = (i / 8) % NB, j = i % 8;
                uint32_t *dst = ah + (size_t)s * NB * 16 + ((j >> 1) * NB + g) * 4 + 2 * (j & 1);
                dst[0] = __builtin_bit_cast(uint32_t, lo);
                dst[1] = __builtin_bit_cast(uint32_t, hi);
                if (j == 0) asc[s * NB + g] = dx;
            }
        }
    };
    stage_load(av, threadIdx.x);
    if (threadIdx.x < per) {
        const int s = threadIdx.x;
        bool ok = true;
        const int e = s < a.topk ? mk_checked_expert(a.ids[tok * a.topk + s], a.tab.n_experts, ok) : a.shared;
        wp_l[s] = a.tab.w2p[e];
        ws_l[s] = a.tab.w2s[e];
        pw_l[s] = !ok ? 0.0f : (s < a.topk && !a.ds_rule) ? a.weights[tok * a.topk + s] : 1.0f;
    }
    __syncthreads();  // the pair tables: the first weight loads need them

    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n_tiles = a.d / RT;
    const int wv = blockIdx.y * WAVES + wave, wpt = gridDim.y * WAVES;
    const int my_tiles = wv < n_tiles ? (n_tiles - wv + wpt - 1) / wpt : 0;
    const int groups = (my_tiles + U - 1) / U;
    const int n_items = groups * per;  // (tile group, pair), pair fastest: slot order per row

    mk_i4 wa[U][T], wb[U][T];
    uint32_t sa[U][T], sb[U][T];
    auto load_item = [&](mk_i4(*w)[T], uint32_t(*sc)[T], int i) {
        const bool past = i >= n_items;  // unconditional loads: past the end, one line of item 0 per load
        i = __builtin_amdgcn_readfirstlane(past ? 0 : i);
        const int grp = i / per, s = i - grp * per;
        // uniform pointers in scalar registers + 32-bit block indices: the loads take the scalar-base form
        const uint8_t *wp = mk_uniform_ptr(wp_l[s]), *ws = mk_uniform_ptr(ws_l[s]);
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int k = grp * U + u;
            const uint32_t tile = min((uint32_t)(wv + (k < my_tiles ? k : 0) * wpt), (uint32_t)(n_tiles - 1));  // idle waves re-read the last tile
            const uint32_t blk0 = past ? 0u : tile * TILE + lane;
#pragma unroll
            for (int t = 0; t < T; t++) {
                w[u][t] = mk_ldg128_off_nt(wp, (blk0 + t * 64) * 16);
                sc[u][t] = mk_ldg_u8_off(ws, blk0 + t * 64);
            }
        }
    };
    float y[U][RT];
#pragma unroll
    for (int u = 0; u < U; u++)
#pragma unroll
        for (int r = 0; r < RT; r++) y[u][r] = 0.0f;
    auto compute_item = [&](const mk_i4(*w)[T], const uint32_t(*sc)[T], int i) {
        // the waves that share a SIMD (w, w + 4, w + 8, ...) rotate through the issue priorities item by item, so that
        // none of them is served first all the time (see the gate/up kernel)
        if constexpr (WAVES > 4) {
            switch ((i + (wave >> 2)) & 3) {
                case 0: __builtin_amdgcn_s_setprio(0); break;
                case 1: __builtin_amdgcn_s_setprio(1); break;
                case 2: __builtin_amdgcn_s_setprio(2); break;
                default: __builtin_amdgcn_s_setprio(3); break;
            }
        }
        const int grp = i / per, s = i - grp * per;
        mk_h2 xr[T][16];
        float cf[T];
#pragma unroll
        for (int t = 0; t < T; t++) {
            const int g = (t * 64 + lane) % NB;
#pragma unroll
            for (int k = 0; k < 16; k++) xr[t][k] = __builtin_bit_cast(mk_h2, ah[(size_t)s * NB * 16 + ((k >> 2) * NB + g) * 4 + (k & 3)]);
            cf[t] = asc[s * NB + g];
        }
        const float pw = pw_l[s];
#pragma unroll
        for (int u = 0; u < U; u++) {
            float acc[RT];
#pragma unroll
            for (int r = 0; r < RT; r++) acc[r] = 0.0f;
#pragma unroll
            for (int t = 0; t < T; t++) {
                float h = mk_dot32_fp4_f16(w[u][t], xr[t]);
                float term = (h + h) * (mk_half_scale_from_byte(sc[u][t]) * cf[t]);
                const int rit = (t * 64 + lane) / NB;
#pragma unroll
                for (int r = 0; r < RT; r++) acc[r] += (rit == r) ? term : 0.0f;
            }
#pragma unroll
            for (int r = 0; r < RT; r++) y[u][r] = mk_add(y[u][r], mk_mul(pw, mk_wave_sum(acc[r])));
        }
        if (s == per - 1) {  // the row's last pair: store and start the next rows
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int k = grp * U + u;
                if (k < my_tiles && lane < RT) {
                    const int row = (wv + k * wpt) * RT + lane;
                    a.out[(size_t)tok * a.d + row] = (RT == 2 && lane == 1) ? y[u][RT - 1] : y[u][0];
                }
#pragma unroll
                for (int r = 0; r < RT; r++) y[u][r] = 0.0f;
            }
        }
    };
    constexpr bool PRE2 = U * T <= 4;  // small register blocks: both in flight while the activation is staged
    load_item(wa, sa, 0);
    if constexpr (PRE2) load_item(wb, sb, 1);

    stage_store(av, threadIdx.x);
    for (int i0 = threadIdx.x + WAVES * 64 * SB; i0 < n_a; i0 += WAVES * 64 * SB) {
        stage_load(av, i0);
        stage_store(av, i0);
    }
    __syncthreads();

    for (int i = 0; i < n_items; i += 2) {
        if constexpr (!PRE2) load_item(wb, sb, i + 1);
        compute_item(wa, sa, i);
        load_item(wa, sa, i + 2);
        if (i + 1 < n_items) compute_item(wb, sb, i + 1);
        if constexpr (PRE2) load_item(wb, sb, i + 3);
    }
}

// elementwise activation for the composed path: act[p][j] = ACT(g, u)
__global__ __launch_bounds__(256) void moe_act_kernel(const float *__restrict__ g, const float *__restrict__ u, const float *__restrict__ pw,
                                                      int inter, int n, int act_kind, float limit, float *__restrict__ act) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    act[i] = mk_act(act_kind, g[i], u[i], limit, pw[i / inter]);
}

// out[t][j] = sum_s w * o[p(t,s)][j] in slot order (+ shared, unweighted)
__global__ __launch_bounds__(256) void moe_combine_kernel(const float *__restrict__ o, const float *__restrict__ pw, int per, int topk, int d,
                                                          int ds_rule, float *__restrict__ out) {
    const int t = blockIdx.y;
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= d) return;
    float y = 0.0f;
    for (int s = 0; s < topk; s++) {
        const float v = o[((size_t)t * per + s) * d + j];
        y = ds_rule ? mk_add(y, v) : mk_add(y, mk_mul(pw[t * per + s], v));
    }
    if (per > topk) y = mk_add(y, o[((size_t)t * per + topk) * d + j]);
    out[(size_t)t * d + j] = y;
}

// ------------------------------------------------------------ batched path
// From 4 tokens (the measured crossover: batch 3 140 / 154 us, batch 4 148 / 142 us, batch 5 229 / 216 us, two-kernel
// path / this one) the layer is taken expert by expert: the (token, slot) pairs are grouped by expert (stable: inside a
// group in (token, slot) order), every group's rows go through the expert's matrices together on the matrix cores
// with the exact q8 arithmetic (gemm_q8x.hip), so an expert that several tokens selected -- the shared expert: all of
// them -- is read once.  Kernels: this grouping, quantize_q8 of the hidden rows, gate + up, activation with the q8 form
// of the activation rows (matvec_packed's own step), down, and the weighted sum per token in slot order.
constexpr int BATCHED_MAX_P = 1024;

// Workgroup 0 groups the pairs; the others form the q8 blocks of the hidden rows (src/q8.rs:57-68, 8 lanes per
// 32-block as mk_quantize_q8_kernel) -- one launch for the two steps in front of the gate/up GEMM.
__global__ __launch_bounds__(1024) void moe_group_pairs_kernel(int B, int topk, int shared, size_t n_experts, const int32_t *__restrict__ ids,
                                                               const float *__restrict__ weights, int32_t *order, int32_t *pos, int32_t *rtok,
                                                               int32_t *goff, int32_t *gexp, int32_t *ngroups, float *pw,
                                                               const float *__restrict__ x, size_t n_blocks, int8_t *__restrict__ xq,
                                                               float *__restrict__ xs) {
    if (blockIdx.x > 0) {
        const size_t i = (size_t)(blockIdx.x - 1) * blockDim.x + threadIdx.x;
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
        reinterpret_cast<uint32_t *>(xq)[i] = packed;
        if ((i & 7) == 0) xs[i >> 3] = dx;
        return;
    }
    __shared__ __attribute__((aligned(16))) int e_l[BATCHED_MAX_P], start_l[BATCHED_MAX_P];
    __shared__ int se_l[BATCHED_MAX_P], goff_l[BATCHED_MAX_P + 1], cnt_l[BATCHED_MAX_P];
    __shared__ int ng_l, best_l;
    const int per = topk + (shared >= 0 ? 1 : 0), P = B * per, tid = threadIdx.x;
    {
        int e = 0x7FFFFFFF;  // behind every pair: the loops below read whole 16-byte groups
        if (tid < P) {
            const int t = tid / per, s = tid % per;
            bool ok = true;
            e = s < topk ? mk_checked_expert(ids[t * topk + s], n_experts, ok) : shared;
            pw[tid] = s < topk ? (ok ? weights[t * topk + s] : 0.0f) : 1.0f;
        }
        e_l[tid] = e;
        start_l[tid] = 0;
        cnt_l[tid] = 0;
    }
    if (tid == 0) best_l = 0;
    __syncthreads();
    // The P x P comparisons are spread over all 1024 threads: thread (p, part) counts over a slice of q.
    const int parts = max(1, 1024 / P), p = tid % P, part = tid / P;
    const int slice = ((P + parts - 1) / parts + 3) & ~3;  // a multiple of 4
    const bool worker = part < parts;
    const int q0 = part * slice, q1 = min(P, q0 + slice);
    if (worker) {
        // stable rank of the pair among all pairs by expert id
        const int e = e_l[p];
        int rank = 0;
        for (int q = q0; q < q1; q += 4) {
            const mk_i4 v = *reinterpret_cast<const mk_i4 *>(e_l + q);
#pragma unroll
            for (int k = 0; k < 4; k++) rank += (v[k] < e || (v[k] == e && q + k < p)) ? 1 : 0;
        }
        if (rank) atomicAdd(&cnt_l[p], rank);
    }
    __syncthreads();
    if (tid < P) {
        const int rank = cnt_l[tid];
        order[rank] = tid;
        pos[tid] = rank;
        rtok[rank] = tid / per;
        se_l[rank] = e_l[tid];
    }
    __syncthreads();
    if (tid < P) {
        start_l[tid] = (tid == 0 || se_l[tid] != se_l[tid - 1]) ? 1 : 0;
        cnt_l[tid] = 0;
    }
    __syncthreads();
    if (worker) {
        int g = 0;  // groups that start at or before grouped row p, this thread's slice of them
        for (int q = q0; q < q1 && q <= p; q += 4) {
            const mk_i4 v = *reinterpret_cast<const mk_i4 *>(start_l + q);
#pragma unroll
            for (int k = 0; k < 4; k++) g += (q + k <= p) ? v[k] : 0;
        }
        if (g) atomicAdd(&cnt_l[p], g);
    }
    __syncthreads();
    if (tid < P) {
        const int g = cnt_l[tid];
        if (start_l[tid]) {
            goff[g - 1] = tid;
            goff_l[g - 1] = tid;
            gexp[g - 1] = se_l[tid];
        }
        if (tid == P - 1) {
            goff[g] = P;
            goff_l[g] = P;
            ngroups[0] = g;
            ng_l = g;
        }
    }
    __syncthreads();
    // the largest group (ties: the first)
    if (tid < ng_l) atomicMax(&best_l, ((goff_l[tid + 1] - goff_l[tid]) << 12) | (4095 - tid));
    __syncthreads();
    if (tid == 0) ngroups[1] = 4095 - (best_l & 4095);
}

// The activation of the grouped rows and its q8 form in one kernel (the block matvec_packed forms when it re-quantizes
// its input for W2, src/q8.rs:57-68): 8 lanes per 32-block, four values each.  act_in (optional): the activation rows
// are given, [pair][inter] in (token, slot) order, instead of being formed from g and u; act_out (optional): the f32
// activation rows are also written there in that order.
__global__ __launch_bounds__(256) void moe_act_q8_grouped_kernel(const float *__restrict__ g, const float *__restrict__ u,
                                                                 const float *__restrict__ pw, const int32_t *__restrict__ order, int inter,
                                                                 size_t n_blocks, int act_kind, float limit, const float *__restrict__ act_in,
                                                                 float *__restrict__ act_out, int8_t *__restrict__ q,
                                                                 float *__restrict__ scales) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_blocks * 8) return;  // whole groups of 8 lanes leave together
    const size_t row = (i * 4) / (size_t)inter, col4 = i - row * (size_t)(inter / 4);
    const int pair = order[row];
    mk_f4 v;
    if (act_in) {
        v = reinterpret_cast<const mk_f4 *>(act_in + (size_t)pair * inter)[col4];
    } else {
        const mk_f4 gv = reinterpret_cast<const mk_f4 *>(g)[i], uv = reinterpret_cast<const mk_f4 *>(u)[i];
        const float wgt = pw[pair];
        v = mk_f4{mk_act(act_kind, gv.x, uv.x, limit, wgt), mk_act(act_kind, gv.y, uv.y, limit, wgt), mk_act(act_kind, gv.z, uv.z, limit, wgt),
                  mk_act(act_kind, gv.w, uv.w, limit, wgt)};
    }
    if (act_out) reinterpret_cast<mk_f4 *>(act_out + (size_t)pair * inter)[col4] = v;
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
    if ((i & 7) == 0) scales[i >> 3] = dx;
}

// out[t][j] = sum_s w * o[pos(t, s)][j] in slot order (+ shared, unweighted)
__global__ __launch_bounds__(256) void moe_combine_grouped_kernel(const float *__restrict__ o, const float *__restrict__ pw,
                                                                  const int32_t *__restrict__ pos, int per, int topk, int d, int ds_rule,
                                                                  float *__restrict__ out) {
    const int t = blockIdx.y;
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= d) return;
    float y = 0.0f;
    for (int s = 0; s < topk; s++) {
        const float v = o[(size_t)pos[t * per + s] * d + j];
        y = ds_rule ? mk_add(y, v) : mk_add(y, mk_mul(pw[t * per + s], v));
    }
    if (per > topk) y = mk_add(y, o[(size_t)pos[t * per + topk] * d + j]);
    out[(size_t)t * d + j] = y;
}

}  // namespace

extern "C" size_t mk_moe_decode_workspace_bytes(size_t B, size_t topk, int has_shared, size_t d, size_t inter) {
    return carve(nullptr, B, topk, has_shared, d, inter).bytes;
}

// behind it when the table holds VQ1 experts: the tables of the hidden rows, then those of the activation rows
extern "C" size_t mk_moe_decode_vq_workspace_bytes(size_t B, size_t topk, int has_shared, size_t d, size_t inter) {
    const size_t P = B * (topk + (has_shared ? 1 : 0));
    return align_up(B * (d / 16) * 256 * sizeof(float), 256) + align_up(P * (inter / 16) * 256 * sizeof(float), 256);
}

namespace {

template <int NB>
int launch_gate_up_rows(const FusedArgs &a, size_t B, hipStream_t st) {
    // token group: as many hidden rows (f16 pairs + scales) and pair tables as fit 150 KiB of LDS, at most 8
    const size_t per_tok = (size_t)NB * 68 + (size_t)a.per * 48;
    int tg = (int)((150 * 1024) / per_tok);
    if (tg > 8) tg = 8;
    if (tg > (int)B) tg = (int)B;
    const size_t lds = (size_t)tg * per_tok;
    const int s = mk_lds_opt_in(reinterpret_cast<const void *>(moe_gate_up_rows_kernel<NB>), 160 * 1024);
    if (s != MK_OK) return s;
    int blocks = MK_TUNE("MK_MOE_ROWS_BLOCKS", 256);  // one resident workgroup per CU
    if (blocks * 8 > a.inter) blocks = (a.inter + 7) / 8;
    hipLaunchKernelGGL(moe_gate_up_rows_kernel<NB>, dim3(blocks), dim3(512), lds, st, a, (int)B, tg);
    return mk_launch_status("moe_gate_up_rows");
}

template <int NB, int U, int WAVES = 4>
int launch_down_u(const FusedArgs &a, size_t B, int blocks, hipStream_t st) {
    const size_t lds = (size_t)a.per * NB * 64 + (size_t)a.per * NB * 4;
    const int s = mk_lds_opt_in(reinterpret_cast<const void *>(moe_down_fused_kernel<NB, U, WAVES>), 150 * 1024);
    if (s != MK_OK) return s;
    hipLaunchKernelGGL((moe_down_fused_kernel<NB, U, WAVES>), dim3((unsigned)B, blocks), dim3(WAVES * 64), lds, st, a);
    return mk_launch_status("moe_down_fused");
}

// The tokens share one resident grid.  A wave streams register blocks of U tiles;
// U is the largest of 8/T, 4/T ... 1 for which the rows still spread over at
// least two workgroups per CU, and the block count is then set so that the tiles
// divide evenly among the waves (a register block that is only partly filled
// would re-read and re-compute the wave's first tile).
template <int NB>
int launch_down_fused(const FusedArgs &a, size_t B, hipStream_t st) {
    constexpr int TILE = lcm_c(NB, 64), T = TILE / 64, RT = TILE / NB;
    const int n_tiles = a.d / RT;
    if constexpr (T == 1) {
        // One workgroup of 14 waves per CU when the rows then divide evenly (7168 = 2^10 x 7): the activation is
        // quantized once per CU instead of once per small workgroup, and every wave has the same number of tiles.
        const int bpt = 256 / (int)B;  // workgroups per token
        if (bpt >= 1 && !MK_TUNE("MK_MOE_DOWN_SMALL", 0) && n_tiles % (bpt * 14) == 0) {
            const int tiles = n_tiles / (bpt * 14);  // per wave
            if (tiles % 8 == 0) return launch_down_u<NB, 8, 14>(a, B, bpt, st);
            if (tiles % 4 == 0) return launch_down_u<NB, 4, 14>(a, B, bpt, st);
            if (tiles % 2 == 0) return launch_down_u<NB, 2, 14>(a, B, bpt, st);
        }
    }
    const int target = MK_TUNE("MK_MOE_DOWN_BLOCKS", 768) / (int)B;  // blocks per token
    int u = 8 / T;
    int forced = MK_TUNE("MK_MOE_DOWN_U", 0);
    auto blocks_for = [&](int uu) {
        int groups = (int)((double)n_tiles / ((double)(target > 0 ? target : 1) * 4 * uu) + 0.5);
        if (groups < 1) groups = 1;
        return (n_tiles + 4 * uu * groups - 1) / (4 * uu * groups);
    };
    if (forced > 0) u = forced;
    else
        while (u > 1 && (size_t)blocks_for(u) * B < 512) u >>= 1;
    const int blocks = blocks_for(u);
    switch (u) {
        case 8: if constexpr (8 * T <= 8) return launch_down_u<NB, 8>(a, B, blocks, st);
        case 4: if constexpr (4 * T <= 8) return launch_down_u<NB, 4>(a, B, blocks, st);
        case 2: return launch_down_u<NB, 2>(a, B, blocks, st);
        default: return launch_down_u<NB, 1>(a, B, blocks, st);
    }
}
}  // namespace

namespace {
enum { STAGE_ALL = MK_MOE_STAGE_ALL, STAGE_ACT = MK_MOE_STAGE_ACT, STAGE_FROM_ACT = MK_MOE_STAGE_FROM_ACT };

// The layer, or one of its two stages: STAGE_ACT stops after the activation rows (act_io [B * per][inter], out),
// STAGE_FROM_ACT starts from given activation rows (act_io, in).  Both run the kernels the whole layer runs.
int moe_decode_impl(const mk_expert_table *table, size_t B, size_t topk, const int32_t *ids, const float *weights, int shared, const float *x,
                    int mode, int act_kind, float limit, void *workspace, float *out, void *stream, int stage, float *act_io) {
    MK_REQUIRE(table && ids && weights && workspace, "null pointer");
    MK_REQUIRE(stage == STAGE_FROM_ACT || x, "null pointer");
    MK_REQUIRE(stage == STAGE_ACT || out, "null pointer");
    MK_REQUIRE(stage == STAGE_ALL || act_io, "null pointer");
    MK_REQUIRE(mode == MK_MODE_Q8 || mode == MK_MODE_F32, "mode must be MK_MODE_F32 or MK_MODE_Q8");
    MK_REQUIRE(act_kind >= MK_ACT_SWIGLU && act_kind <= MK_ACT_DS, "unknown activation");
    const size_t d = table->d, inter = table->inter;
    MK_REQUIRE(d % 32 == 0 && inter % 32 == 0 && d > 0 && inter > 0, "d and inter must be positive multiples of 32");
    MK_REQUIRE(B >= 1 && topk >= 1 && B * (topk + 1) <= 65535, "bad batch / top-k");
    MK_REQUIRE(table->n_experts == 0 || shared < (long long)table->n_experts, "shared expert id beyond the table");
    MK_REQUIRE(((uintptr_t)workspace & 255) == 0, "workspace must be 256-byte aligned");
    MK_REQUIRE(!act_io || ((uintptr_t)act_io & 15) == 0, "activation rows must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    const int per = (int)topk + (shared >= 0 ? 1 : 0);
    const size_t P = B * per;
    Workspace w = carve(workspace, B, topk, shared >= 0, d, inter);
    const int nb = (int)(d / 32), nbi = (int)(inter / 32);
    const bool fast = mode == MK_MODE_Q8 && (nb == 32 || nb == 64 || nb == 128 || nb == 224) && (nbi == 32 || nbi == 64 || nbi == 128) &&
                      per <= MAX_PER && d % 2 == 0 && (size_t)per * nbi * 68 <= 150 * 1024;
    int s;
    // A layer with VQ1 experts (src/model.rs:2243-2257) takes the composed kernels: which pairs are VQ1 is known on the
    // device only, so both kinds of launch run over all pairs and each skips the other kind's.
    const bool has_vq = table->vq_codebook != nullptr;
    float *lut_x = reinterpret_cast<float *>((uint8_t *)workspace + w.bytes);
    float *lut_a = reinterpret_cast<float *>((uint8_t *)lut_x + align_up(B * (d / 16) * 256 * sizeof(float), 256));
    // batched path: q8 mode, both projections in K tiles of 512, enough tokens for experts to repeat
    const bool batched = !has_vq && mode == MK_MODE_Q8 && d % 512 == 0 && inter % 512 == 0 && P <= (size_t)BATCHED_MAX_P &&
                         (int)B >= MK_TUNE("MK_MOE_BATCHED_MIN", 4) && inter * (d / 2) < 0xFFFFFFFFull && P * d < 0xFFFFFFFFull;
    if (batched) {
        {
            // the grouping is needed by both stages; with given activation rows there is no hidden row to quantize
            MK_REQUIRE(stage == STAGE_FROM_ACT || ((uintptr_t)x & 15) == 0, "x must be 16-byte aligned");
            const size_t n_blocks = stage == STAGE_FROM_ACT ? 0 : B * d / 32;
            hipLaunchKernelGGL(moe_group_pairs_kernel, dim3(1 + (unsigned)((n_blocks * 8 + 1023) / 1024)), dim3(1024), 0, st, (int)B, (int)topk,
                               shared, table->n_experts, ids, weights, w.order, w.pos, w.rtok, w.goff, w.gexp, w.ngroups, w.pt.pw, x, n_blocks, w.xq, w.xs);
            if ((s = mk_launch_status("moe_group_pairs")) != MK_OK) return s;
        }
        if (stage != STAGE_FROM_ACT) {
            const uint8_t *const *pp[2] = {table->w1p, table->w3p};
            const uint8_t *const *sp[2] = {table->w1s, table->w3s};
            float *gu[2] = {w.g, w.u};
            const uint8_t *const *tp[2] = {table->w1st, table->w3st};
            if ((s = mk_q8x_grouped(2, pp, sp, inter, d, w.xq, w.xs, w.rtok, w.goff, w.gexp, w.ngroups, w.ngroups + 1, P, B, gu, stream,
                                    table->w1st && table->w3st ? tp : nullptr)) != MK_OK)
                return s;
        }
        {
            const size_t n_blocks = P * inter / 32;
            hipLaunchKernelGGL(moe_act_q8_grouped_kernel, dim3((unsigned)((n_blocks + 31) / 32)), dim3(256), 0, st, w.g, w.u, w.pt.pw, w.order,
                               (int)inter, n_blocks, act_kind, limit, stage == STAGE_FROM_ACT ? act_io : nullptr,
                               stage == STAGE_ACT ? act_io : nullptr, w.aq, w.as);
            if ((s = mk_launch_status("moe_act_q8_grouped")) != MK_OK) return s;
        }
        if (stage == STAGE_ACT) return MK_OK;
        {
            const uint8_t *const *pp[1] = {table->w2p};
            const uint8_t *const *sp[1] = {table->w2s};
            float *oo[1] = {w.o};
            const uint8_t *const *tp[1] = {table->w2st};
            if ((s = mk_q8x_grouped(1, pp, sp, d, inter, w.aq, w.as, nullptr, w.goff, w.gexp, w.ngroups, w.ngroups + 1, P, B, oo, stream,
                                    table->w2st ? tp : nullptr)) != MK_OK)
                return s;
        }
        hipLaunchKernelGGL(moe_combine_grouped_kernel, dim3((unsigned)((d + 255) / 256), (unsigned)B), dim3(256), 0, st, w.o, w.pt.pw, w.pos, per,
                           (int)topk, (int)d, act_kind == MK_ACT_DS ? 1 : 0, out);
        return mk_launch_status("moe_combine_grouped");
    }
    float *af = stage == STAGE_ALL ? w.af : act_io;  // [P][inter] activation rows in (token, slot) order
    // one launch of one resident workgroup per CU when the table carries the packed copies of its matrices
    const bool persist = !has_vq && mode == MK_MODE_Q8 && table->w13t && table->w2t && mk_moe_persist_takes(B, d, inter, per) &&
                         ((uintptr_t)x & 15) == 0 && !MK_TUNE("MK_MOE_NO_PERSIST", 0);
    if ((fast || persist) && !has_vq) {
        FusedArgs fa;
        fa.tab = *table;
        fa.ids = ids;
        fa.weights = weights;
        fa.x = x;
        fa.topk = (int)topk;
        fa.shared = shared;
        fa.per = per;
        fa.d = (int)d;
        fa.inter = (int)inter;
        fa.act_kind = act_kind;
        fa.ds_rule = act_kind == MK_ACT_DS ? 1 : 0;
        fa.limit = limit;
        fa.af = af;
        fa.out = out;
        if (persist) return mk_moe_persist_launch(fa, B, stage, w.lines, st);
        if (stage != STAGE_FROM_ACT) {
            switch (nb) {
                case 32: s = launch_gate_up_rows<32>(fa, B, st); break;
                case 64: s = launch_gate_up_rows<64>(fa, B, st); break;
                case 128: s = launch_gate_up_rows<128>(fa, B, st); break;
                default: s = launch_gate_up_rows<224>(fa, B, st); break;
            }
            if (s != MK_OK || stage == STAGE_ACT) return s;
        }
        switch (nbi) {
            case 32: return launch_down_fused<32>(fa, B, st);
            case 64: return launch_down_fused<64>(fa, B, st);
            default: return launch_down_fused<128>(fa, B, st);
        }
    }
    hipLaunchKernelGGL(moe_setup_kernel, dim3((unsigned)((P + 63) / 64)), dim3(64), 0, st, *table, (int)B, (int)topk, shared, ids, weights,
                       w.pt, w.o, w.g, w.u, (int)d, (int)inter);
    s = mk_launch_status("moe_setup");
    if (s != MK_OK) return s;
    const bool q8 = mode == MK_MODE_Q8;
    if (stage != STAGE_FROM_ACT) {
        // composed path (any shape, both modes): gate and up as grouped GEMVs,
        // elementwise activation, then (q8) the activation's own quantization
        if (q8 && (s = mk_dev_quantize_q8(x, B, d, w.xq, w.xs, stream)) != MK_OK) return s;
        if ((s = mk_gemv_grouped_internal(q8, w.pt.w1p, w.pt.w1s, P, inter, d, w.xq, w.xs, x, w.pt.xidx, w.pt.gptr, st)) != MK_OK) return s;
        if ((s = mk_gemv_grouped_internal(q8, w.pt.w3p, w.pt.w3s, P, inter, d, w.xq, w.xs, x, w.pt.xidx, w.pt.uptr, st)) != MK_OK) return s;
        if (has_vq) {  // quant::matvec_vq on the f32 hidden row (no q8 step for VQ1 experts)
            if ((s = mk_vq1_grouped_tables(table->vq_codebook, x, B, d, nullptr, lut_x, st)) != MK_OK) return s;
            if ((s = mk_vq1_grouped_sweep(lut_x, w.pt.xidx, w.pt.w1p, w.pt.w1s, P, inter, d, w.pt.gptr, st)) != MK_OK) return s;
            if ((s = mk_vq1_grouped_sweep(lut_x, w.pt.xidx, w.pt.w3p, w.pt.w3s, P, inter, d, w.pt.uptr, st)) != MK_OK) return s;
        }
        const int n = (int)(P * inter);
        hipLaunchKernelGGL(moe_act_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, w.g, w.u, w.pt.pw, (int)inter, n, act_kind, limit,
                           af);
        if ((s = mk_launch_status("moe_act")) != MK_OK || stage == STAGE_ACT) return s;
    }
    if (q8 && (s = mk_dev_quantize_q8(af, P, inter, w.aq, w.as, stream)) != MK_OK) return s;
    if ((s = mk_gemv_grouped_internal(q8, w.pt.w2p, w.pt.w2s, P, d, inter, w.aq, w.as, af, w.pt.aidx, w.pt.optr, st)) != MK_OK) return s;
    if (has_vq) {
        if ((s = mk_vq1_grouped_tables(table->vq_codebook, af, P, inter, w.pt.w2s, lut_a, st)) != MK_OK) return s;
        if ((s = mk_vq1_grouped_sweep(lut_a, nullptr, w.pt.w2p, w.pt.w2s, P, d, inter, w.pt.optr, st)) != MK_OK) return s;
    }
    hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)((d + 255) / 256), (unsigned)B), dim3(256), 0, st, w.o, w.pt.pw, per, (int)topk, (int)d,
                       act_kind == MK_ACT_DS ? 1 : 0, out);
    return mk_launch_status("moe_combine");
}
}  // namespace

namespace {
// one workgroup: count[0] = number of ids outside [0, n_experts)
__global__ __launch_bounds__(256) void count_bad_ids_kernel(const int32_t *__restrict__ ids, size_t n, unsigned n_experts, int32_t *__restrict__ count) {
    __shared__ int part[4];
    int c = 0;
    for (size_t i = threadIdx.x; i < n; i += 256) c += (unsigned)ids[i] >= n_experts ? 1 : 0;
    for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = c;
    __syncthreads();
    if (threadIdx.x == 0) count[0] = part[0] + part[1] + part[2] + part[3];
}
}  // namespace

extern "C" int mk_dev_moe_count_bad_ids(const int32_t *ids, size_t n, size_t n_experts, int32_t *count, void *stream) {
    MK_REQUIRE(ids && count, "null pointer");
    MK_REQUIRE(n >= 1 && n_experts >= 1 && n_experts < (1u << 31), "n and n_experts must be at least 1");
    hipLaunchKernelGGL(count_bad_ids_kernel, dim3(1), dim3(256), 0, (hipStream_t)stream, ids, n, (unsigned)n_experts, count);
    return mk_launch_status("count_bad_ids");
}

extern "C" int mk_dev_moe_decode(const mk_expert_table *table, size_t B, size_t topk, const int32_t *ids, const float *weights, int shared,
                                 const float *x, int mode, int act_kind, float limit, void *workspace, float *out, void *stream) {
    return moe_decode_impl(table, B, topk, ids, weights, shared, x, mode, act_kind, limit, workspace, out, stream, STAGE_ALL, nullptr);
}

extern "C" int mk_dev_moe_decode_act(const mk_expert_table *table, size_t B, size_t topk, const int32_t *ids, const float *weights, int shared,
                                     const float *x, int mode, int act_kind, float limit, void *workspace, float *act, void *stream) {
    return moe_decode_impl(table, B, topk, ids, weights, shared, x, mode, act_kind, limit, workspace, nullptr, stream, STAGE_ACT, act);
}

extern "C" int mk_dev_moe_decode_from_act(const mk_expert_table *table, size_t B, size_t topk, const int32_t *ids, const float *weights,
                                          int shared, const float *act, int mode, int act_kind, void *workspace, float *out, void *stream) {
    return moe_decode_impl(table, B, topk, ids, weights, shared, nullptr, mode, act_kind, 0.0f, workspace, out, stream, STAGE_FROM_ACT,
                           const_cast<float *>(act));
}
