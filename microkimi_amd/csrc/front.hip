// What a decode layer runs in front of its quantized matvecs, so that
// norm -> route -> experts needs no host round trip:
//
//   rmsnorm (+ q8)  model::rmsnorm / ds_rmsnorm (src/model.rs:599-605,
//                   src/deepseek.rs:241-248), optionally followed by
//                   q8::quantize_q8_into of the normed row (src/q8.rs:49-69)
//   f32 matvec      model::matvec_cpu (src/model.rs:214-222): the router gate,
//                   latent projections and other small f32 matrices
//   router          the three selection rules (src/model.rs:2157-2173,
//                   src/deepseek.rs:16-58, and softmax for the benchmark layer)
//
// The f32 dot is the reference's contract (src/model.rs:46-82): 8 accumulators,
// element j of every 8-wide chunk goes to accumulator j with a multiply, then an
// add (never fused), reduction ((p01 + p23) + p45) + p67, remainder sequential.
// It is replayed here operation for operation -- lane j of a group of 8 lanes
// owns accumulator j -- so rmsnorm outputs and router logits are the reference's
// values bit for bit; the price is a sequential chain of cols/8 additions per
// lane, which is fine for the small matrices this is meant for.
#include "mk_common.h"

namespace {

// the reduction of the 8 accumulators held by lanes g*8 .. g*8+7; the result is valid in lane g*8
__device__ __forceinline__ float dot8_reduce(float acc) {
    const float pair = mk_add(acc, __shfl_xor(acc, 1, MK_WAVE));  // lanes 0,2,4,6 of the group: p01, p23, p45, p67
    const int base = (threadIdx.x & 63) & ~7;
    float s = mk_add(pair, __shfl(pair, base + 2, MK_WAVE));
    s = mk_add(s, __shfl(pair, base + 4, MK_WAVE));
    s = mk_add(s, __shfl(pair, base + 6, MK_WAVE));
    return s;
}

// One workgroup per row.  The row is staged in LDS; lanes 0..7 of wave 0 replay dot(x, x); then every
// thread scales 8 consecutive values (x * inv * w, two multiplications in that order) and, when asked,
// a quad of lanes quantizes its 32-block to q8.
__global__ __launch_bounds__(256) void rmsnorm_q8_kernel(const float *__restrict__ x, int d, const float *__restrict__ w, float eps,
                                                         float *__restrict__ out, int8_t *__restrict__ q, float *__restrict__ scales) {
    extern __shared__ __attribute__((aligned(16))) float xl[];  // [d], then inv
    const int t = blockIdx.x, tid = threadIdx.x;
    const float *row = x + (size_t)t * d;
    for (int i = tid; i < d / 4; i += 256) reinterpret_cast<mk_f4 *>(xl)[i] = reinterpret_cast<const mk_f4 *>(row)[i];
    for (int i = (d & ~3) + tid; i < d; i += 256) xl[i] = row[i];
    __syncthreads();
    if (tid < 64) {
        float acc = 0.0f;
        const int j = tid & 7, chunks = d / 8;
        if (tid < 8) {
#pragma unroll 8
            for (int i = 0; i < chunks; i++) {
                const float v = xl[i * 8 + j];
                acc = mk_add(acc, mk_mul(v, v));
            }
        }
        float s = dot8_reduce(acc);
        if (tid == 0) {
            for (int i = chunks * 8; i < d; i++) s = mk_add(s, mk_mul(xl[i], xl[i]));
            // Correctly rounded float division and square root, as the host computes them: done in double and
            // rounded once (53 bits are enough for the double rounding to be harmless for both operations).
            const float ss = (float)((double)s / (double)d);
            const float rt = (float)sqrt((double)mk_add(ss, eps));
            xl[d] = (float)(1.0 / (double)rt);
        }
    }
    __syncthreads();
    const float inv = xl[d];
    for (int g = tid; g < (d + 7) / 8; g += 256) {  // 8 values per lane; a q8 block is a quad of lanes
        float v[8];
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const int i = g * 8 + k;
            v[k] = i < d ? mk_mul(mk_mul(xl[i], inv), w[i]) : 0.0f;
        }
        if (out) {
#pragma unroll
            for (int k = 0; k < 8; k++)
                if (g * 8 + k < d) out[(size_t)t * d + g * 8 + k] = v[k];
        }
        if (q) {  // d % 32 == 0 is checked by the host in this case
            float a = 0.0f;
#pragma unroll
            for (int k = 0; k < 8; k++) a = fmaxf(a, fabsf(v[k]));
            a = fmaxf(a, mk_dpp<0xB1>(a));
            a = fmaxf(a, mk_dpp<0x4E>(a));
            const float dx = a / 127.0f;
            uint32_t w0 = 0, w1 = 0;
            if (dx != 0.0f) {
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    w0 |= (uint32_t)(mk_q8_round(v[k], dx) & 255) << (8 * k);
                    w1 |= (uint32_t)(mk_q8_round(v[4 + k], dx) & 255) << (8 * k);
                }
            }
            reinterpret_cast<mk_u2 *>(q + (size_t)t * d)[g] = mk_u2{w0, w1};
            if ((g & 3) == 0) scales[(size_t)t * (d / 32) + (g >> 2)] = dx;
        }
    }
}

// out[b][r] = dot(w[r], x[b]) with the reference's dot contract: 8 lanes per row, 8 rows per wave
__global__ __launch_bounds__(256) void matvec_f32_kernel(const float *__restrict__ w, int rows, int cols, const float *__restrict__ x,
                                                         float *__restrict__ out) {
    const int b = blockIdx.y;
    const int r = (blockIdx.x * 256 + threadIdx.x) >> 3, j = threadIdx.x & 7;
    const int rr = min(r, rows - 1);  // every lane takes part in the shuffles
    const float *wr = w + (size_t)rr * cols, *xb = x + (size_t)b * cols;
    const int chunks = cols / 8;
    float acc = 0.0f;
#pragma unroll 8
    for (int i = 0; i < chunks; i++) acc = mk_add(acc, mk_mul(wr[i * 8 + j], xb[i * 8 + j]));
    float s = dot8_reduce(acc);
    if (j == 0 && r < rows) {
        for (int i = chunks * 8; i < cols; i++) s = mk_add(s, mk_mul(wr[i], xb[i]));
        out[(size_t)b * rows + r] = s;
    }
}

// ---------------------------------------------------------------- router
// Scores and selection keys per rule, then the top k keys with strict '>'
// replacement of the current worst and a stable order (ties to the lowest
// index: src/model.rs:2160-2171, src/deepseek.rs:36-48), which is k rounds of
// (largest key, lowest index) extraction.  Weights: the bias-free scores of the
// selected experts, summed in that order.
//   MK_ROUTER_SOFTMAX       score = key = softmax(logits);  w = score / sum
//   MK_ROUTER_SIGMOID       score = sigmoid(l), key = score + bias;  w = score / (sum + 1e-20)   (K3, noaux_tc)
//   MK_ROUTER_SQRTSOFTPLUS  score = sqrt(softplus(l)), key = score + bias;  w = score / sum * route_scale   (DeepSeek-V4)
// One wave per token; n <= 4096, k <= 64.
__global__ __launch_bounds__(64) void router_topk_kernel(const float *__restrict__ logits, int n, int k, int kind,
                                                         const float *__restrict__ bias, float route_scale, int32_t *__restrict__ ids,
                                                         float *__restrict__ weights) {
    extern __shared__ float lds_f[];  // score [n], key [n]
    float *score = lds_f, *key = lds_f + n;
    const int t = blockIdx.x, lane = threadIdx.x;
    const float *row = logits + (size_t)t * n;
    if (kind == MK_ROUTER_SOFTMAX) {
        float m = -INFINITY;
        for (int i = lane; i < n; i += 64) m = fmaxf(m, row[i]);
        m = mk_wave_max(m);
        // the reference sums exp(l - m) sequentially; the sum is only a common
        // normaliser, so its association does not change the selection order
        float z = 0.0f;
        for (int i = lane; i < n; i += 64) {
            float e = expf(row[i] - m);
            score[i] = e;
            z += e;
        }
        z = mk_wave_sum(z);
        __syncthreads();
        for (int i = lane; i < n; i += 64) {
            const float p = score[i] / z;
            score[i] = p;
            key[i] = p;
        }
    } else {
        for (int i = lane; i < n; i += 64) {
            const float l = row[i];
            float sc;
            if (kind == MK_ROUTER_SIGMOID) {
                sc = 1.0f / (1.0f + expf(-l));
            } else {
                const float sp = l > 20.0f ? l : logf(1.0f + expf(l));  // src/deepseek.rs:61-68
                sc = sqrtf(sp);
            }
            score[i] = sc;
            key[i] = sc + (bias ? bias[i] : 0.0f);
        }
    }
    __syncthreads();
    float sum = 0.0f, myw = 0.0f;
    int myid = 0;
    for (int r = 0; r < k; r++) {
        float bv = -INFINITY;
        int bi = 0x7FFFFFFF;
        for (int i = lane; i < n; i += 64) {
            float v = key[i];
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
        const float sc = score[bi];
        if (lane == r) {
            myw = sc;
            myid = bi;
        }
        sum += sc;  // slot order, as the reference sums the selected scores
        __syncthreads();
        if (lane == 0) key[bi] = -INFINITY;
        __syncthreads();
    }
    if (lane < k) {
        ids[t * k + lane] = myid;
        float wv;
        if (kind == MK_ROUTER_SIGMOID) wv = myw / (sum + 1e-20f);
        else if (kind == MK_ROUTER_SQRTSOFTPLUS) wv = myw / sum * route_scale;
        else wv = myw / sum;
        weights[t * k + lane] = wv;
    }
}

}  // namespace

extern "C" int mk_dev_rmsnorm(const float *x, size_t B, size_t d, const float *w, float eps, float *out, int8_t *q, float *scales,
                              void *stream) {
    MK_REQUIRE(x && w && (out || q), "null pointer");
    MK_REQUIRE((q == nullptr) == (scales == nullptr), "q and scales go together");
    MK_REQUIRE(d >= 1 && d <= 32768 && B >= 1 && B <= 65535, "bad shape");
    MK_REQUIRE(!q || d % 32 == 0, "q8 blocks are 32 wide");
    MK_REQUIRE(((uintptr_t)x & 15) == 0 && (d % 4 == 0 || B == 1) && (!q || ((uintptr_t)q & 7) == 0), "x must be 16-byte aligned rows");
    const size_t lds = (d + 4) * sizeof(float);
    int st = mk_lds_opt_in(reinterpret_cast<const void *>(rmsnorm_q8_kernel), 132 * 1024);
    if (st != MK_OK) return st;
    hipLaunchKernelGGL(rmsnorm_q8_kernel, dim3((unsigned)B), dim3(256), lds, (hipStream_t)stream, x, (int)d, w, eps, out, q, scales);
    return mk_launch_status("rmsnorm_q8");
}

extern "C" int mk_dev_matvec_f32(const float *w, size_t rows, size_t cols, const float *x, size_t B, float *out, void *stream) {
    MK_REQUIRE(w && x && out, "null pointer");
    MK_REQUIRE(rows >= 1 && rows <= (1u << 24) && cols >= 1 && cols <= (1u << 24) && B >= 1 && B <= 65535, "bad shape");
    hipLaunchKernelGGL(matvec_f32_kernel, dim3((unsigned)((rows * 8 + 255) / 256), (unsigned)B), dim3(256), 0, (hipStream_t)stream, w, (int)rows,
                       (int)cols, x, out);
    return mk_launch_status("matvec_f32");
}

extern "C" int mk_dev_router_topk(const float *logits, size_t B, size_t n, size_t k, int kind, const float *bias, float route_scale,
                                  int32_t *ids, float *weights, void *stream) {
    MK_REQUIRE(logits && ids && weights, "null pointer");
    MK_REQUIRE(kind >= MK_ROUTER_SOFTMAX && kind <= MK_ROUTER_SQRTSOFTPLUS, "unknown router rule");
    MK_REQUIRE(n >= 1 && n <= 4096 && k >= 1 && k <= 64 && k <= n && B >= 1 && B <= 65535, "bad router shape");
    hipLaunchKernelGGL(router_topk_kernel, dim3((unsigned)B), dim3(64), 2 * n * sizeof(float), (hipStream_t)stream, logits, (int)n, (int)k, kind,
                       bias, route_scale, ids, weights);
    return mk_launch_status("router_topk");
}

extern "C" int mk_dev_router_softmax_topk(const float *logits, size_t B, size_t n, size_t k, int32_t *ids, float *weights, void *stream) {
    return mk_dev_router_topk(logits, B, n, k, MK_ROUTER_SOFTMAX, nullptr, 1.0f, ids, weights, stream);
}
