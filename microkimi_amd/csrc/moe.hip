// MoE decode layer: the expert section of moe_forward / ds_moe
// (src/model.rs:2227-2264,2346-2351; src/deepseek.rs:1069-1106) for B tokens as
// one grouped pass over the (token, slot) pairs.
//
//   setup     pair tables (expert pointers per pair) from the router's ids
//   quantize  x -> q8 (once per token; gate and up quantize the same input to
//             the same bytes in the reference)
//   gate_up   per pair and 32-row block: a = W1 x, u = W3 x with the GEMV tiling
//             of gemv_mxfp4.hip, act = ACT(a, u) kept in lanes 0..31, then the
//             q8 quantization of that 32-block of `act` in-wave -- exactly the
//             block matvec_packed would form when it re-quantizes its input for W2
//   down      o = W2 act: the grouped MXFP4 GEMV over all pairs
//   combine   out_t = sum_slot w * o in slot order (+ shared expert)
//
// HBM traffic: every selected expert's 23.4 MB is read once per pair; the
// intermediates (act: 2 KiB + 256 B per pair, o: 28 KiB per pair) are noise.
#include "mk_common.h"

// grouped MXFP4 GEMV of gemv_mxfp4.hip: q8 (xq, xs) or f32 (xf) activations, one launch over nmat matrices
int mk_gemv_grouped_internal(bool q8, const uint8_t *const *packed_ptrs, const uint8_t *const *scales_ptrs, size_t nmat, size_t rows,
                             size_t cols, const int8_t *xq, const float *xs, const float *xf, const int32_t *x_index, float *const *out_ptrs,
                             hipStream_t st);

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
    w.bytes = off;
    return w;
}

__global__ void moe_setup_kernel(mk_expert_table tab, int B, int topk, int shared, const int32_t *__restrict__ ids,
                                 const float *__restrict__ weights, PairTables pt, float *o, float *g, float *u, int d, int inter) {
    const int per = topk + (shared >= 0 ? 1 : 0);
    const int p = blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= B * per) return;
    const int t = p / per, s = p % per;
    const int e = s < topk ? ids[t * topk + s] : shared;
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
    pt.pw[p] = s < topk ? weights[t * topk + s] : 1.0f;
}

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

// gate + up + activation + q8 of the activation block.  One wave = 32 rows of
// one pair.  NB = d / 32.
template <int NB>
__global__ __launch_bounds__(256) void moe_gate_up_q8_kernel(PairTables pt, const int8_t *__restrict__ xq, const float *__restrict__ xs,
                                                             int inter, int act_kind, float limit, int8_t *__restrict__ aq,
                                                             float *__restrict__ as) {
    constexpr int TILE = lcm_c(NB, 64);
    constexpr int T = TILE / 64;
    constexpr int RT = TILE / NB;
    static_assert(RT <= 2 && T <= 8, "tile shape not covered by the fast path");
    // f16 pairs kept as 32-bit words: written and read through the same type
    __shared__ __attribute__((aligned(16))) uint32_t xh[NB * 16];
    __shared__ float xsc[NB];
    const int p = blockIdx.y;
    const uint8_t *w1p = pt.w1p[p], *w1s = pt.w1s[p], *w3p = pt.w3p[p], *w3s = pt.w3s[p];
    const int tok = pt.xidx[p];
    const float wgt = pt.pw[p];
    const int8_t *xqv = xq + (size_t)tok * NB * 32;
    const float *xsv = xs + (size_t)tok * NB;
    for (int i = threadIdx.x; i < NB * 8; i += 256) {
        uint32_t v = reinterpret_cast<const uint32_t *>(xqv)[i];
        mk_h2 lo, hi;
        lo.x = (_Float16)(float)(int8_t)(v & 255u);
        lo.y = (_Float16)(float)(int8_t)((v >> 8) & 255u);
        hi.x = (_Float16)(float)(int8_t)((v >> 16) & 255u);
        hi.y = (_Float16)(float)(int8_t)(v >> 24);
        xh[i * 2] = __builtin_bit_cast(uint32_t, lo);
        xh[i * 2 + 1] = __builtin_bit_cast(uint32_t, hi);
    }
    for (int i = threadIdx.x; i < NB; i += 256) xsc[i] = xsv[i];
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const int rb = blockIdx.x * 4 + (threadIdx.x >> 6);  // 32-row block of the pair
    if (rb * 32 >= inter) return;
    mk_h2 xr[T][16];
    float cf[T];
#pragma unroll
    for (int t = 0; t < T; t++) {
        const int g = (t * 64 + lane) % NB;
#pragma unroll
        for (int k = 0; k < 16; k++) xr[t][k] = __builtin_bit_cast(mk_h2, xh[g * 16 + k]);
        cf[t] = xsc[g];
    }
    float myact = 0.0f;
    for (int i = 0; i < 32 / RT; i++) {
        const size_t blk0 = ((size_t)rb * 32 + (size_t)i * RT) * NB;  // first block of the tile (rows are contiguous)
        mk_i4 wa[T], wu[T];
        uint32_t sa[T], su[T];
#pragma unroll
        for (int t = 0; t < T; t++) {
            const size_t b = blk0 + t * 64 + lane;
            wa[t] = *reinterpret_cast<const mk_i4 *>(w1p + b * 16);
            wu[t] = *reinterpret_cast<const mk_i4 *>(w3p + b * 16);
            sa[t] = w1s[b];
            su[t] = w3s[b];
        }
        float ga[RT], gu[RT];
#pragma unroll
        for (int r = 0; r < RT; r++) ga[r] = gu[r] = 0.0f;
#pragma unroll
        for (int t = 0; t < T; t++) {
            float ha = dot32_fp4_f16(wa[t], xr[t]);
            float hu = dot32_fp4_f16(wu[t], xr[t]);
            float ta = (ha + ha) * (mk_half_scale_from_byte(sa[t]) * cf[t]);
            float tu = (hu + hu) * (mk_half_scale_from_byte(su[t]) * cf[t]);
            const int rit = (t * 64 + lane) / NB;
#pragma unroll
            for (int r = 0; r < RT; r++) {
                ga[r] += (rit == r) ? ta : 0.0f;
                gu[r] += (rit == r) ? tu : 0.0f;
            }
        }
#pragma unroll
        for (int r = 0; r < RT; r++) {
            float a = mk_wave_sum(ga[r]);
            float u = mk_wave_sum(gu[r]);
            float act = mk_act(act_kind, a, u, limit, wgt);
            if (lane == i * RT + r) myact = act;
        }
    }
    // lanes 0..31 hold act[rb*32 + lane]: q8 of this block (src/q8.rs:57-68)
    float mx = mk_half_wave_max(fabsf(myact));
    float dx = mx / 127.0f;
    if (lane < 32) {
        int qi = dx != 0.0f ? mk_q8_round(myact, dx) : 0;
        aq[(size_t)p * inter + rb * 32 + lane] = (int8_t)qi;
        if (lane == 0) as[(size_t)p * (inter / 32) + rb] = dx;
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
        y = ds_rule ? __fadd_rn(y, v) : __fadd_rn(y, __fmul_rn(pw[t * per + s], v));
    }
    if (per > topk) y = __fadd_rn(y, o[((size_t)t * per + topk) * d + j]);
    out[(size_t)t * d + j] = y;
}

}  // namespace

extern "C" size_t mk_moe_decode_workspace_bytes(size_t B, size_t topk, int has_shared, size_t d, size_t inter) {
    return carve(nullptr, B, topk, has_shared, d, inter).bytes;
}

namespace {
template <int NB>
void launch_gate_up(const Workspace &w, size_t P, size_t inter, int act_kind, float limit, hipStream_t st) {
    const unsigned gx = (unsigned)((inter / 32 + 3) / 4);
    hipLaunchKernelGGL(moe_gate_up_q8_kernel<NB>, dim3(gx, (unsigned)P), dim3(256), 0, st, w.pt, w.xq, w.xs, (int)inter, act_kind, limit, w.aq,
                       w.as);
}
}  // namespace

extern "C" int mk_dev_moe_decode(const mk_expert_table *table, size_t B, size_t topk, const int32_t *ids, const float *weights, int shared,
                                 const float *x, int mode, int act_kind, float limit, void *workspace, float *out, void *stream) {
    MK_REQUIRE(table && ids && weights && x && workspace && out, "null pointer");
    MK_REQUIRE(mode == MK_MODE_Q8 || mode == MK_MODE_F32, "mode must be MK_MODE_F32 or MK_MODE_Q8");
    MK_REQUIRE(act_kind >= MK_ACT_SWIGLU && act_kind <= MK_ACT_DS, "unknown activation");
    const size_t d = table->d, inter = table->inter;
    MK_REQUIRE(d % 32 == 0 && inter % 32 == 0 && d > 0 && inter > 0, "d and inter must be positive multiples of 32");
    MK_REQUIRE(B >= 1 && topk >= 1 && B * (topk + 1) <= 65535, "bad batch / top-k");
    MK_REQUIRE(((uintptr_t)workspace & 255) == 0, "workspace must be 256-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    const int per = (int)topk + (shared >= 0 ? 1 : 0);
    const size_t P = B * per;
    Workspace w = carve(workspace, B, topk, shared >= 0, d, inter);
    hipLaunchKernelGGL(moe_setup_kernel, dim3((unsigned)((P + 63) / 64)), dim3(64), 0, st, *table, (int)B, (int)topk, shared, ids, weights,
                       w.pt, w.o, w.g, w.u, (int)d, (int)inter);
    int s = mk_launch_status("moe_setup");
    if (s != MK_OK) return s;
    const int nb = (int)(d / 32);
    const bool fast = mode == MK_MODE_Q8 && (nb == 32 || nb == 64 || nb == 128 || nb == 224);
    if (mode == MK_MODE_Q8) {
        if ((s = mk_dev_quantize_q8(x, B, d, w.xq, w.xs, stream)) != MK_OK) return s;
    }
    if (fast) {
        switch (nb) {
            case 32: launch_gate_up<32>(w, P, inter, act_kind, limit, st); break;
            case 64: launch_gate_up<64>(w, P, inter, act_kind, limit, st); break;
            case 128: launch_gate_up<128>(w, P, inter, act_kind, limit, st); break;
            default: launch_gate_up<224>(w, P, inter, act_kind, limit, st); break;
        }
        if ((s = mk_launch_status("moe_gate_up")) != MK_OK) return s;
    } else {
        // composed path (any shape, both modes): gate and up as grouped GEMVs,
        // elementwise activation, then (q8) the activation's own quantization
        const bool q8 = mode == MK_MODE_Q8;
        if ((s = mk_gemv_grouped_internal(q8, w.pt.w1p, w.pt.w1s, P, inter, d, w.xq, w.xs, x, w.pt.xidx, w.pt.gptr, st)) != MK_OK) return s;
        if ((s = mk_gemv_grouped_internal(q8, w.pt.w3p, w.pt.w3s, P, inter, d, w.xq, w.xs, x, w.pt.xidx, w.pt.uptr, st)) != MK_OK) return s;
        const int n = (int)(P * inter);
        hipLaunchKernelGGL(moe_act_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, w.g, w.u, w.pt.pw, (int)inter, n, act_kind, limit,
                           w.af);
        if ((s = mk_launch_status("moe_act")) != MK_OK) return s;
        if (q8 && (s = mk_dev_quantize_q8(w.af, P, inter, w.aq, w.as, stream)) != MK_OK) return s;
    }
    if ((s = mk_gemv_grouped_internal(mode == MK_MODE_Q8, w.pt.w2p, w.pt.w2s, P, d, inter, w.aq, w.as, w.af, w.pt.aidx, w.pt.optr, st)) != MK_OK)
        return s;
    hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)((d + 255) / 256), (unsigned)B), dim3(256), 0, st, w.o, w.pt.pw, per, (int)topk, (int)d,
                       act_kind == MK_ACT_DS ? 1 : 0, out);
    return mk_launch_status("moe_combine");
}

// ---------------------------------------------------------------- router
// softmax over n logits, top-k by probability with strict '>' replacement of
// the current worst and a stable order (ties to the lowest index), weights
// renormalised (src/model.rs:2157-2173 selection rule on softmax scores).
// One wave per token; n <= 4096, k <= 64.
__global__ __launch_bounds__(64) void router_softmax_topk_kernel(const float *__restrict__ logits, int n, int k, int32_t *__restrict__ ids,
                                                                 float *__restrict__ weights) {
    extern __shared__ float prob[];  // [n]
    const int t = blockIdx.x, lane = threadIdx.x;
    const float *row = logits + (size_t)t * n;
    float m = -INFINITY;
    for (int i = lane; i < n; i += 64) m = fmaxf(m, row[i]);
    m = mk_wave_max(m);
    // the reference sums exp(l - m) sequentially; the sum is only a common
    // normaliser, so its association does not change the selection order
    float z = 0.0f;
    for (int i = lane; i < n; i += 64) {
        float e = expf(row[i] - m);
        prob[i] = e;
        z += e;
    }
    z = mk_wave_sum(z);
    __syncthreads();
    for (int i = lane; i < n; i += 64) prob[i] = prob[i] / z;
    __syncthreads();
    // k rounds of (max value, lowest index) extraction == the stable descending order
    float sum = 0.0f;
    float myw = 0.0f;
    int myid = 0;
    for (int r = 0; r < k; r++) {
        float bv = -1.0f;
        int bi = 0x7FFFFFFF;
        for (int i = lane; i < n; i += 64) {
            float v = prob[i];
            if (v > bv || (v == bv && i < bi)) {
                bv = v;
                bi = i;
            }
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            float ov = __shfl_xor(bv, off, MK_WAVE);
            int oi = __shfl_xor(bi, off, MK_WAVE);
            if (ov > bv || (ov == bv && oi < bi)) {
                bv = ov;
                bi = oi;
            }
        }
        if (lane == r) {
            myw = bv;
            myid = bi;
        }
        sum += bv;  // slot order, as the reference sums the selected scores
        if (lane == 0) prob[bi] = -2.0f;
        __syncthreads();
    }
    if (lane < k) {
        ids[t * k + lane] = myid;
        weights[t * k + lane] = myw / sum;
    }
}

extern "C" int mk_dev_router_softmax_topk(const float *logits, size_t B, size_t n, size_t k, int32_t *ids, float *weights, void *stream) {
    MK_REQUIRE(logits && ids && weights, "null pointer");
    MK_REQUIRE(n >= 1 && n <= 4096 && k >= 1 && k <= 64 && k <= n && B >= 1 && B <= 65535, "bad router shape");
    hipLaunchKernelGGL(router_softmax_topk_kernel, dim3((unsigned)B), dim3(64), n * sizeof(float), (hipStream_t)stream, logits, (int)n, (int)k,
                       ids, weights);
    return mk_launch_status("router_softmax_topk");
}
