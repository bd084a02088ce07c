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
// values bit for bit.  The price is a sequential chain of cols/8 additions per
// lane; only the additions are sequential, so the other threads of the workgroup
// form the products and lay them out in LDS in the order a chain consumes them
// (chain-major, 16 bytes a read): a chain then runs at the latency of an add.
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

// acc + p[0] + p[1] + ... + p[n-1], one addition after the other.  p: LDS, 16-byte aligned.  Batches of 32 values: the
// next batch is requested before the current one is added (the scheduling barriers keep that order; left alone, the
// compiler moves the requests down to their first use and every batch then waits for the whole LDS latency).
struct ChainBatch {
    mk_f4 v[8];
};
__device__ __forceinline__ void chain_load(ChainBatch &c, const mk_f4 *p4) {
#pragma unroll
    for (int k = 0; k < 8; k++) c.v[k] = p4[k];
}
__device__ __forceinline__ float chain_sum32(float acc, const ChainBatch &c) {
#pragma unroll
    for (int k = 0; k < 8; k++) acc = mk_add(mk_add(mk_add(mk_add(acc, c.v[k].x), c.v[k].y), c.v[k].z), c.v[k].w);
    return acc;
}
__device__ __forceinline__ float chain_add(float acc, const float *p, int n) {
    const mk_f4 *p4 = reinterpret_cast<const mk_f4 *>(p);
    const int n32 = n >> 5;
    if (n32 > 0) {
        ChainBatch a, b;
        chain_load(a, p4);
        for (int i = 0; i < n32; i += 2) {
            chain_load(b, p4 + 8 * min(i + 1, n32 - 1));  // (past the end: the last batch once more, unused)
            __builtin_amdgcn_sched_barrier(0);
            acc = chain_sum32(acc, a);
            __builtin_amdgcn_sched_barrier(0);
            chain_load(a, p4 + 8 * min(i + 2, n32 - 1));
            __builtin_amdgcn_sched_barrier(0);
            if (i + 1 < n32) acc = chain_sum32(acc, b);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    int i = n32 * 32;
    for (; i + 4 <= n; i += 4) {
        const mk_f4 v = p4[i >> 2];
        acc = mk_add(mk_add(mk_add(mk_add(acc, v.x), v.y), v.z), v.w);
    }
    for (; i < n; i++) acc = mk_add(acc, p[i]);
    return acc;
}
// floats between two chains' rows in LDS for `steps` values a chain: a multiple of 4 that is 4 modulo 64, so that the 16
// lanes of one pass of a 16-byte read fall into 16 different groups of four banks
__host__ __device__ constexpr int chain_stride(int steps) { return ((steps + 63) & ~63) + 4; }

// One workgroup per row.  The row is staged in LDS; lanes 0..7 of wave 0 replay dot(x, x); then every
// thread scales 8 consecutive values (x * inv * w, two multiplications in that order) and, when asked,
// a quad of lanes quantizes its 32-block to q8.
// prod_off: float offset of the chain-major squares inside the LDS block (8 rows of chain_stride(d / 8)), or 0 when the
// block has no room for them (then the chain lanes square the staged values themselves).  w_off: float offset of a copy
// of w that the waves without a chain fetch while the chain runs, or 0 (then the last loop reads w from memory).
// Loads go out eight at a time per thread: a loop of one load and one store per trip pays a memory latency per trip.
__global__ __launch_bounds__(256) void rmsnorm_q8_kernel(const float *__restrict__ x, int d, const float *__restrict__ w, float eps,
                                                         float *__restrict__ out, int8_t *__restrict__ q, float *__restrict__ scales, int prod_off,
                                                         int w_off) {
    extern __shared__ __attribute__((aligned(16))) float xl[];  // [d], then inv
    const int t = blockIdx.x, tid = threadIdx.x;
    const float *row = x + (size_t)t * d;
    const int chunks = d / 8, stride = chain_stride(chunks), n4 = d / 4;
    float *prod = xl + prod_off;
    for (int base = 0; base < n4; base += 256 * 8) {
        mk_f4 v[8];
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const int i = base + 256 * k + tid;
            v[k] = reinterpret_cast<const mk_f4 *>(row)[min(i, n4 - 1)];
        }
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const int i = base + 256 * k + tid;
            if (i < n4) {
                reinterpret_cast<mk_f4 *>(xl)[i] = v[k];
                if (prod_off && (i >> 1) < chunks) {  // values 4 i .. 4 i + 3: accumulators 4 (i % 2) .. + 3 of chunk i / 2
                    float *dst = prod + (4 * (i & 1)) * stride + (i >> 1);
                    dst[0] = mk_mul(v[k].x, v[k].x);
                    dst[stride] = mk_mul(v[k].y, v[k].y);
                    dst[2 * stride] = mk_mul(v[k].z, v[k].z);
                    dst[3 * stride] = mk_mul(v[k].w, v[k].w);
                }
            }
        }
    }
    for (int i = (d & ~3) + tid; i < d; i += 256) xl[i] = row[i];
    __syncthreads();
    if (tid < 64) {
        float acc = 0.0f;
        const int j = tid & 7;
        if (tid < 8) {
            if (prod_off) {
                acc = chain_add(acc, prod + j * stride, chunks);
            } else {
#pragma unroll 8
                for (int i = 0; i < chunks; i++) {
                    const float v = xl[i * 8 + j];
                    acc = mk_add(acc, mk_mul(v, v));
                }
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
    } else if (w_off) {  // d % 4 == 0 here
        float *wl = xl + w_off;
        for (int base = 0; base < n4; base += 192 * 8) {
            mk_f4 v[8];
#pragma unroll
            for (int k = 0; k < 8; k++) v[k] = reinterpret_cast<const mk_f4 *>(w)[min(base + 192 * k + tid - 64, n4 - 1)];
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const int i = base + 192 * k + tid - 64;
                if (i < n4) reinterpret_cast<mk_f4 *>(wl)[i] = v[k];
            }
        }
    }
    __syncthreads();
    const float inv = xl[d];
    // 16-byte pieces when the row is whole groups of 8 and the output rows are aligned (w_off implies an aligned w)
    const bool vec = d % 8 == 0 && w_off != 0 && (!out || ((uintptr_t)out & 15) == 0);
    for (int g = tid; g < (d + 7) / 8; g += 256) {  // 8 values per lane; a q8 block is a quad of lanes
        float v[8];
        if (vec) {
            const mk_f4 a0 = reinterpret_cast<const mk_f4 *>(xl)[2 * g], a1 = reinterpret_cast<const mk_f4 *>(xl)[2 * g + 1];
            const mk_f4 w0 = reinterpret_cast<const mk_f4 *>(xl + w_off)[2 * g], w1 = reinterpret_cast<const mk_f4 *>(xl + w_off)[2 * g + 1];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                v[k] = mk_mul(mk_mul(a0[k], inv), w0[k]);
                v[4 + k] = mk_mul(mk_mul(a1[k], inv), w1[k]);
            }
            if (out) {
                mk_f4 *dst = reinterpret_cast<mk_f4 *>(out + (size_t)t * d) + 2 * g;
                dst[0] = mk_f4{v[0], v[1], v[2], v[3]};
                dst[1] = mk_f4{v[4], v[5], v[6], v[7]};
            }
        } else {
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const int i = g * 8 + k;
                v[k] = i < d ? mk_mul(mk_mul(xl[i], inv), w_off ? xl[w_off + i] : w[i]) : 0.0f;
            }
            if (out) {
#pragma unroll
                for (int k = 0; k < 8; k++)
                    if (g * 8 + k < d) out[(size_t)t * d + g * 8 + k] = v[k];
            }
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

// The same product with the chains fed from LDS: a workgroup per weight row and group of up to 4 tokens.  Waves 1-3 form
// the products w[r][c] * x[t][c] of a segment of 2048 columns and store them chain-major (chain = (token, accumulator),
// chain_stride(256) floats a chain); wave 0's lane 8 t + j adds chain (t, j) of the segment before, one addition after
// the other.  Two segment buffers, one barrier a segment; a producer has all its loads of a segment in flight at once.
// Needs cols % 4 == 0 and 16-byte aligned w and x.
constexpr int MV_SEG = 2048, MV_STEPS = MV_SEG / 8, MV_STRIDE = chain_stride(MV_STEPS), MV_TB = 4, MV_NG = (MV_SEG / 4 + 191) / 192;
__global__ __launch_bounds__(256) void matvec_f32_chain_kernel(const float *__restrict__ w, int rows, int cols, const float *__restrict__ x, int B,
                                                               float *__restrict__ out, int tb_max) {
    extern __shared__ __attribute__((aligned(16))) float mv_lds[];  // [2][8 tb_max][MV_STRIDE]
    const int r = blockIdx.x, b0 = blockIdx.y * MV_TB, tb = min(MV_TB, B - b0);
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int chunks = cols / 8, chain_cols = chunks * 8, nseg = (chain_cols + MV_SEG - 1) / MV_SEG;
    const int buf_floats = 8 * tb_max * MV_STRIDE;
    const float *wr = w + (size_t)r * cols, *xb = x + (size_t)b0 * cols;

    auto produce = [&](int seg) {  // waves 1-3: 192 threads, four columns at a time, up to MV_NG column groups a thread
        float *buf = mv_lds + (seg & 1) * buf_floats;
        const int c0 = seg * MV_SEG, c1 = min(c0 + MV_SEG, chain_cols);
        mk_f4 wv[MV_NG], xv[MV_TB][MV_NG];
#pragma unroll
        for (int k = 0; k < MV_NG; k++) {
            const int c = min(c0 + 4 * (tid - 64 + 192 * k), cols - 4);
            wv[k] = *reinterpret_cast<const mk_f4 *>(wr + c);
#pragma unroll
            for (int t = 0; t < MV_TB; t++) xv[t][k] = *reinterpret_cast<const mk_f4 *>(xb + (size_t)min(t, tb - 1) * cols + c);
        }
#pragma unroll
        for (int k = 0; k < MV_NG; k++) {
            const int c = c0 + 4 * (tid - 64 + 192 * k);
            if (c < c1) {
                float *dst = buf + (4 * ((c >> 2) & 1)) * MV_STRIDE + ((c - c0) >> 3);
#pragma unroll
                for (int t = 0; t < MV_TB; t++) {
                    if (t < tb) {
                        float *dt = dst + 8 * t * MV_STRIDE;
                        dt[0] = mk_mul(wv[k].x, xv[t][k].x);
                        dt[MV_STRIDE] = mk_mul(wv[k].y, xv[t][k].y);
                        dt[2 * MV_STRIDE] = mk_mul(wv[k].z, xv[t][k].z);
                        dt[3 * MV_STRIDE] = mk_mul(wv[k].w, xv[t][k].w);
                    }
                }
            }
        }
    };
    float acc = 0.0f;
    if (wave != 0 && nseg > 0) produce(0);
    __syncthreads();
    for (int seg = 0; seg < nseg; seg++) {
        if (wave != 0) {
            if (seg + 1 < nseg) produce(seg + 1);
        } else if (lane < 8 * tb) {
            const int steps = (min((seg + 1) * MV_SEG, chain_cols) - seg * MV_SEG) >> 3;
            acc = chain_add(acc, mv_lds + (seg & 1) * buf_floats + lane * MV_STRIDE, steps);
        }
        __syncthreads();
    }
    if (wave == 0) {
        float s = dot8_reduce(acc);
        const int t = lane >> 3;
        if ((lane & 7) == 0 && t < tb) {
            const float *xt = xb + (size_t)t * cols;
            for (int i = chain_cols; i < cols; i++) s = mk_add(s, mk_mul(wr[i], xt[i]));
            out[(size_t)(b0 + t) * rows + r] = s;
        }
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
// One wave routes one token.  score / key: LDS, n floats each, this wave's own; no workgroup barrier is needed (a wave's
// LDS operations stay in program order), so several waves of a workgroup can each route a token.  COHERENT: the logits were
// written by other workgroups of the same launch (read with agent-scope loads).
template <bool COHERENT>
__device__ __forceinline__ void router_wave(const float *row, int n, int k, int kind, const float *__restrict__ bias, float route_scale,
                                            int32_t *ids_t, float *weights_t, float *score, float *key, int lane) {
    auto logit = [&](int i) -> float {
        if (COHERENT) return __hip_atomic_load(row + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return row[i];
    };
    if (kind == MK_ROUTER_SOFTMAX) {
        float m = -INFINITY;
        for (int i = lane; i < n; i += 64) m = fmaxf(m, logit(i));
        m = mk_wave_max(m);
        // the reference sums exp(l - m) sequentially; the sum is only a common
        // normaliser, so its association does not change the selection order
        float z = 0.0f;
        for (int i = lane; i < n; i += 64) {
            float e = expf(logit(i) - m);
            score[i] = e;
            z += e;
        }
        z = mk_wave_sum(z);
        for (int i = lane; i < n; i += 64) {
            const float p = score[i] / z;
            score[i] = p;
            key[i] = p;
        }
    } else {
        for (int i = lane; i < n; i += 64) {
            const float l = logit(i);
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
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");  // the lanes' LDS writes above are read by other lanes below
    __builtin_amdgcn_wave_barrier();
    float sum = 0.0f, myw = 0.0f;
    int myid = 0;
    // A lane keeps the best of its own keys (i = lane, lane + 64, ...: the lowest index among equals); a round takes the
    // wave's largest key, the lowest index among the lanes that hold it, and only the owner of that key looks through its
    // keys again.  Keys that are NaN are never larger than anything and are never selected.
    float bv = -INFINITY;
    int bi = 0x7FFFFFFF;
    auto rescan = [&]() {
        bv = -INFINITY;
        bi = 0x7FFFFFFF;
        for (int i = lane; i < n; i += 64) {
            const float v = key[i];
            if (v > bv) {
                bv = v;
                bi = i;
            }
        }
        if (bi == 0x7FFFFFFF && lane < n) bi = lane;  // all of them -inf (or NaN): still a valid index, never out of range
    };
    rescan();
    for (int r = 0; r < k; r++) {
        const float top = mk_wave_max(bv);
        int cand = bv == top ? bi : 0x7FFFFFFF;
        cand = min(cand, mk_dpp_i<0xB1>(cand));
        cand = min(cand, mk_dpp_i<0x4E>(cand));
        cand = min(cand, mk_dpp_i<0x141>(cand));
        cand = min(cand, mk_dpp_i<0x140>(cand));
        const int best = min(min(__builtin_amdgcn_readlane(cand, 0), __builtin_amdgcn_readlane(cand, 16)),
                             min(__builtin_amdgcn_readlane(cand, 32), __builtin_amdgcn_readlane(cand, 48)));
        const float sc = score[best];
        if (lane == r) {
            myw = sc;
            myid = best;
        }
        sum += sc;  // slot order, as the reference sums the selected scores
        if ((best & 63) == lane) {  // the owner
            key[best] = -INFINITY;
            rescan();
        }
    }
    if (lane < k) {
        ids_t[lane] = myid;
        float wv;
        if (kind == MK_ROUTER_SIGMOID) wv = myw / (sum + 1e-20f);
        else if (kind == MK_ROUTER_SQRTSOFTPLUS) wv = myw / sum * route_scale;
        else wv = myw / sum;
        weights_t[lane] = wv;
    }
}

// One wave per token; n <= 4096, k <= 64.
__global__ __launch_bounds__(64) void router_topk_kernel(const float *__restrict__ logits, int n, int k, int kind,
                                                         const float *__restrict__ bias, float route_scale, int32_t *__restrict__ ids,
                                                         float *__restrict__ weights) {
    extern __shared__ float lds_f[];  // score [n], key [n]
    const int t = blockIdx.x;
    router_wave<false>(logits + (size_t)t * n, n, k, kind, bias, route_scale, ids + (size_t)t * k, weights + (size_t)t * k, lds_f, lds_f + n,
                       (int)threadIdx.x);
}

// rmsnorm -> gate matvec of a decode step in one launch, every value the one the two separate kernels give.
// Grid (n experts, groups of up to 4 tokens).  Workgroup (r, tg):
//   1  dot(x, x) of its tokens through the chain pipeline of matvec_f32_chain_kernel (the products are the squares); every
//      workgroup does this for itself -- a chain of d / 8 additions costs less than a launch;
//   2  the same pipeline with the products gate[r][c] * xn[t][c], xn = (x * inv) * w as rmsnorm forms it; on the way the
//      workgroup stores its share of the xn rows (column groups r, r + n, ...);
//   3  stores its logit.
// The routing stays a launch of its own: having the last workgroup of a token group route it (a counter per group) was
// built and measured 36.8 us against 19.3 for the two launches at 256 experts x 7168 -- the release fence in front of the
// count writes the XCD's L2 back (16 us over the launch), and 256 increments of one counter from 8 XCDs take 8 us more.
__global__ __launch_bounds__(256) void norm_gate_kernel(const float *__restrict__ x, int B, int d, const float *__restrict__ norm_w, float eps,
                                                              const float *__restrict__ gate, int n, float *__restrict__ xn_out,
                                                              float *__restrict__ logits, int tb_max) {
    extern __shared__ __attribute__((aligned(16))) float mv_lds[];  // [2][8 tb_max][MV_STRIDE]
    __shared__ float inv_l[MV_TB];
    const int r = blockIdx.x, tg = blockIdx.y, b0 = tg * MV_TB, tb = min(MV_TB, B - b0);
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int nseg = (d + MV_SEG - 1) / MV_SEG;  // d % 8 == 0: every column is in a chain
    const int buf_floats = 8 * tb_max * MV_STRIDE;
    const float *gr = gate + (size_t)r * d, *xb = x + (size_t)b0 * d;

    // products of one segment, by the 192 threads of waves 1-3; PASS 1: squares, PASS 2: gate * normed value
    auto produce = [&](int seg, int pass, const float *inv) __attribute__((always_inline)) {
        float *buf = mv_lds + (seg & 1) * buf_floats;
        const int c0 = seg * MV_SEG, c1 = min(c0 + MV_SEG, d);
        mk_f4 gv[MV_NG], nv[MV_NG], xv[MV_TB][MV_NG];
#pragma unroll
        for (int kk = 0; kk < MV_NG; kk++) {
            const int c = min(c0 + 4 * (tid - 64 + 192 * kk), d - 4);
            if (pass == 2) {
                gv[kk] = *reinterpret_cast<const mk_f4 *>(gr + c);
                nv[kk] = *reinterpret_cast<const mk_f4 *>(norm_w + c);
            }
#pragma unroll
            for (int t = 0; t < MV_TB; t++) xv[t][kk] = *reinterpret_cast<const mk_f4 *>(xb + (size_t)min(t, tb - 1) * d + c);
        }
#pragma unroll
        for (int kk = 0; kk < MV_NG; kk++) {
            const int c = c0 + 4 * (tid - 64 + 192 * kk);
            if (c < c1) {
                float *dst = buf + (4 * ((c >> 2) & 1)) * MV_STRIDE + ((c - c0) >> 3);
                const bool mine = pass == 2 && xn_out && ((c >> 2) % n) == r;
#pragma unroll
                for (int t = 0; t < MV_TB; t++) {
                    if (t < tb) {
                        float *dt = dst + 8 * t * MV_STRIDE;
                        mk_f4 p;
                        if (pass == 1) {
#pragma unroll
                            for (int e = 0; e < 4; e++) p[e] = mk_mul(xv[t][kk][e], xv[t][kk][e]);
                        } else {
                            mk_f4 y;
#pragma unroll
                            for (int e = 0; e < 4; e++) {
                                y[e] = mk_mul(mk_mul(xv[t][kk][e], inv[t]), nv[kk][e]);
                                p[e] = mk_mul(gv[kk][e], y[e]);
                            }
                            if (mine) *reinterpret_cast<mk_f4 *>(xn_out + (size_t)(b0 + t) * d + c) = y;
                        }
                        dt[0] = p.x;
                        dt[MV_STRIDE] = p.y;
                        dt[2 * MV_STRIDE] = p.z;
                        dt[3 * MV_STRIDE] = p.w;
                    }
                }
            }
        }
    };
    float result = 0.0f;  // lane 8 t of wave 0: the dot of token t
    auto run = [&](int pass) __attribute__((always_inline)) {
        float inv[MV_TB] = {0.0f, 0.0f, 0.0f, 0.0f};
        if (pass == 2) {
#pragma unroll
            for (int t = 0; t < MV_TB; t++) inv[t] = inv_l[t];
        }
        float acc = 0.0f;
        if (wave != 0) produce(0, pass, inv);
        __syncthreads();
        for (int seg = 0; seg < nseg; seg++) {
            if (wave != 0) {
                if (seg + 1 < nseg) produce(seg + 1, pass, inv);
            } else if (lane < 8 * tb) {
                const int steps = (min((seg + 1) * MV_SEG, d) - seg * MV_SEG) >> 3;
                acc = chain_add(acc, mv_lds + (seg & 1) * buf_floats + lane * MV_STRIDE, steps);
            }
            __syncthreads();
        }
        if (wave == 0) result = dot8_reduce(acc);
    };
    run(1);
    if (wave == 0 && (lane & 7) == 0 && (lane >> 3) < tb) {
        // as rmsnorm_q8_kernel: correctly rounded division and square root through double
        const float ss = (float)((double)result / (double)d);
        const float rt = (float)sqrt((double)mk_add(ss, eps));
        inv_l[lane >> 3] = (float)(1.0 / (double)rt);
    }
    __syncthreads();
    run(2);
    if (wave == 0 && (lane & 7) == 0 && (lane >> 3) < tb) logits[(size_t)(b0 + (lane >> 3)) * n + r] = result;
}

}  // namespace

extern "C" int mk_dev_rmsnorm(const float *x, size_t B, size_t d, const float *w, float eps, float *out, int8_t *q, float *scales,
                              void *stream) {
    MK_REQUIRE(x && w && (out || q), "null pointer");
    MK_REQUIRE((q == nullptr) == (scales == nullptr), "q and scales go together");
    MK_REQUIRE(d >= 1 && d <= 32768 && B >= 1 && B <= 65535, "bad shape");
    MK_REQUIRE(!q || d % 32 == 0, "q8 blocks are 32 wide");
    MK_REQUIRE(((uintptr_t)x & 15) == 0 && (d % 4 == 0 || B == 1) && (!q || ((uintptr_t)q & 7) == 0), "x must be 16-byte aligned rows");
    size_t lds = (d + 4) * sizeof(float);
    // the chain-major squares behind the row when both fit (the staging loop forms them from 16-byte pieces: d % 4 == 0)
    const size_t with_prod = lds + 8 * (size_t)chain_stride((int)(d / 8)) * sizeof(float);
    int prod_off = 0, w_off = 0;
    if (d % 4 == 0 && d >= 128 && with_prod <= 150 * 1024) {
        prod_off = (int)(d + 4);
        lds = with_prod;
    }
    if (d % 4 == 0 && ((uintptr_t)w & 15) == 0 && lds + d * sizeof(float) <= 150 * 1024) {
        w_off = (int)(lds / sizeof(float));
        lds += d * sizeof(float);
    }
    int st = mk_lds_opt_in(reinterpret_cast<const void *>(rmsnorm_q8_kernel), 150 * 1024);
    if (st != MK_OK) return st;
    hipLaunchKernelGGL(rmsnorm_q8_kernel, dim3((unsigned)B), dim3(256), lds, (hipStream_t)stream, x, (int)d, w, eps, out, q, scales, prod_off, w_off);
    return mk_launch_status("rmsnorm_q8");
}

extern "C" int mk_dev_matvec_f32(const float *w, size_t rows, size_t cols, const float *x, size_t B, float *out, void *stream) {
    MK_REQUIRE(w && x && out, "null pointer");
    MK_REQUIRE(rows >= 1 && rows <= (1u << 24) && cols >= 1 && cols <= (1u << 24) && B >= 1 && B <= 65535, "bad shape");
    // rows long enough for the chains to matter, 16-byte pieces: the workgroup-per-row form
    if (cols >= 512 && cols % 4 == 0 && (((uintptr_t)w | (uintptr_t)x) & 15) == 0 && !MK_TUNE("MK_MATVEC_F32_PLAIN", 0)) {
        const int tb_max = (int)(B < (size_t)MV_TB ? B : (size_t)MV_TB);
        const int nbuf = cols / 8 * 8 > (size_t)MV_SEG ? 2 : 1;
        const size_t lds = (size_t)nbuf * 8 * tb_max * MV_STRIDE * sizeof(float);
        int st = mk_lds_opt_in(reinterpret_cast<const void *>(matvec_f32_chain_kernel), 140 * 1024);
        if (st != MK_OK) return st;
        hipLaunchKernelGGL(matvec_f32_chain_kernel, dim3((unsigned)rows, (unsigned)((B + MV_TB - 1) / MV_TB)), dim3(256), lds, (hipStream_t)stream, w, (int)rows,
                           (int)cols, x, (int)B, out, tb_max);
        return mk_launch_status("matvec_f32_chain");
    }
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

extern "C" int mk_dev_norm_gate_route(const float *x, size_t B, size_t d, const float *norm_w, float eps, const float *gate, size_t n_experts,
                                      size_t k, int kind, const float *bias, float route_scale, float *xn, float *logits, int32_t *ids,
                                      float *weights, void *stream) {
    MK_REQUIRE(x && norm_w && gate && logits && ids && weights, "null pointer");
    MK_REQUIRE(kind >= MK_ROUTER_SOFTMAX && kind <= MK_ROUTER_SQRTSOFTPLUS, "unknown router rule");
    MK_REQUIRE(B >= 1 && B <= 65535 && k >= 1 && k <= 64 && k <= n_experts && n_experts <= 4096, "bad batch, k or expert count");
    MK_REQUIRE(((((uintptr_t)x | (uintptr_t)norm_w | (uintptr_t)gate | (uintptr_t)xn)) & 15) == 0, "x, norm_w, gate and xn must be 16-byte aligned");
    if (d % 8 != 0 || d < 512 || d > 32768) {
        mk_set_error("this call takes d %% 8 == 0 and 512 <= d <= 32768: use mk_dev_rmsnorm, mk_dev_matvec_f32, mk_dev_router_topk");
        return MK_ERR_UNSUPPORTED;
    }
    if (B > (size_t)MV_TB) {
        // from 5 tokens the rows are normed once, by a launch of their own: in the fused kernel every workgroup norms its
        // group's rows itself, which pays for one launch but not for the second group of tokens (16 tokens: 38.7 us
        // fused, 31.6 us as three launches, at 256 experts x 7168)
        MK_REQUIRE(xn, "more than 4 tokens take the normed rows as a buffer (xn)");
        int s3 = mk_dev_rmsnorm(x, B, d, norm_w, eps, xn, nullptr, nullptr, stream);
        if (s3 != MK_OK) return s3;
        if ((s3 = mk_dev_matvec_f32(gate, n_experts, d, xn, B, logits, stream)) != MK_OK) return s3;
        return mk_dev_router_topk(logits, B, n_experts, k, kind, bias, route_scale, ids, weights, stream);
    }
    const int tb_max = (int)(B < (size_t)MV_TB ? B : (size_t)MV_TB);
    const int nbuf = d > (size_t)MV_SEG ? 2 : 1;
    const size_t lds = (size_t)nbuf * 8 * tb_max * MV_STRIDE * sizeof(float);
    int st = mk_lds_opt_in(reinterpret_cast<const void *>(norm_gate_kernel), 140 * 1024);
    if (st != MK_OK) return st;
    hipLaunchKernelGGL(norm_gate_kernel, dim3((unsigned)n_experts, (unsigned)((B + MV_TB - 1) / MV_TB)), dim3(256), lds, (hipStream_t)stream, x, (int)B,
                       (int)d, norm_w, eps, gate, (int)n_experts, xn, logits, tb_max);
    if ((st = mk_launch_status("norm_gate")) != MK_OK) return st;
    return mk_dev_router_topk(logits, B, n_experts, k, kind, bias, route_scale, ids, weights, stream);
}
