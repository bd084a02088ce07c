// The expert section of moe_prefill (src/model.rs:2528-2602, 2690-2700) on the
// device: (token, slot) pairs grouped by expert, the three projections as
// grouped GEMMs on the block-scaled matrix cores, scatter, and the per-token
// weighted sum in slot order.
//
//   group     counting sort of the pairs by expert id, stable in (token, slot)
//             order inside a group as the reference fills its groups
//   gather    MXFP8 (e4m3 + e8m0 per 32) of each pair's hidden row, in grouped order
//   gate, up  the grouped GEMM over the expert table, both matrices in one launch
//   act       ACT(gate, up) and its MXFP8 form (the input of the down projection)
//   down      mk_dev_mxfp4_grouped_gemm
//   combine   out_t = sum_s w[t][s] * o[pair (t, s)], multiply then add, in slot order
//
// The activations enter the matrix cores as MXFP8: that is the arithmetic of
// deepseek::fp8_roundtrip (src/deepseek.rs:312-322) applied to the gathered rows
// and to the activation, not the pure f32 of matvec_packed_nt.  One departure
// from that function: its clamp of the block exponent at 8 is dropped (the full
// e8m0 range is used).  With the clamp a block whose largest value passes
// 448 * 2^8 = 114688 saturates, and SwiGLU of hidden rows ~ N(0, 1) against
// random experts of this size reaches 4e5: the layer output then misses the f32
// path by 85 % instead of the 2-3 % that the e4m3 rounding costs.
#include "mk_common.h"

namespace {

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

struct PrefillWs {
    int32_t *order;    // [P] grouped row -> pair index t * topk + s
    int32_t *pos;      // [P] pair index -> grouped row (-1: expert id out of range)
    int32_t *offsets;  // [n_experts + 1]
    uint8_t *codes, *exps;    // [P][d], [P][d/32]
    float *g, *u;             // [P][inter]
    uint8_t *codes2, *exps2;  // [P][inter], [P][inter/32]
    float *o;                 // [P][d]
    uint16_t *xb;             // [P][max(d, inter)] bf16: the hidden rows, then the activation rows, of the bf16 section (matrix-instruction form)
    // bf16 section, two-term form (mk_bf16_split8): [P][d / 512][2][512] codes and [P][d / 512][2][16] exponents of the
    // hidden rows, the same for the activation rows
    uint8_t *split_codes, *split_exps, *split_codes2, *split_exps2;
    size_t bytes;
};

PrefillWs carve(void *base, size_t P, size_t n_experts, size_t d, size_t inter) {
    PrefillWs w;
    uint8_t *p = (uint8_t *)base;
    size_t off = 0;
    auto take = [&](size_t n) {
        uint8_t *r = p ? p + off : nullptr;
        off += align_up(n, 256);
        return r;
    };
    w.order = (int32_t *)take(P * 4);
    w.pos = (int32_t *)take(P * 4);
    w.offsets = (int32_t *)take((n_experts + 1) * 4);
    w.codes = take(P * d);
    w.exps = take(P * (d / 32));
    w.g = (float *)take(P * inter * 4);
    w.u = (float *)take(P * inter * 4);
    w.codes2 = take(P * inter);
    w.exps2 = take(P * (inter / 32));
    w.o = (float *)take(P * d * 4);
    w.xb = (uint16_t *)take(P * (d > inter ? d : inter) * 2);
    w.split_codes = take(P * d * 2);
    w.split_exps = take(P * (d / 32) * 2);
    w.split_codes2 = take(P * inter * 2);
    w.split_exps2 = take(P * (inter / 32) * 2);
    w.bytes = off;
    return w;
}

// One workgroup of 16 waves: a stable counting sort of the pairs by expert id.  Wave w owns the pairs
// [w C, (w + 1) C).  Per-wave histograms (LDS integer atomics: counts do not depend on their order), the expert
// offsets by an exclusive scan, each wave's start inside each expert, then every wave places its pairs in order,
// 64 at a time: the lanes that hold the same expert id are found with a ballot and ranked by lane number.
constexpr int GROUP_MAX_P = 16384;
constexpr int GROUP_WAVES = 16;
__global__ __launch_bounds__(GROUP_WAVES * 64) void prefill_group_kernel(const int32_t *__restrict__ ids, int P, int n_experts,
                                                                         int32_t *__restrict__ order, int32_t *__restrict__ pos,
                                                                         int32_t *__restrict__ offsets) {
    extern __shared__ int hist[];  // [GROUP_WAVES][n_experts], then [n_experts + 1] expert offsets
    int *eoff = hist + GROUP_WAVES * n_experts;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int C = ((P + GROUP_WAVES * 64 - 1) / (GROUP_WAVES * 64)) * 64;  // pairs per wave, a multiple of 64
    for (int i = threadIdx.x; i < GROUP_WAVES * n_experts + n_experts + 1; i += blockDim.x) hist[i] = 0;
    __syncthreads();
    int *mine = hist + wave * n_experts;
    for (int i = wave * C + lane; i < min((wave + 1) * C, P); i += 64) {
        const int e = ids[i];
        if (e >= 0 && e < n_experts) atomicAdd(&mine[e], 1);
    }
    __syncthreads();
    // per expert: total and each wave's start relative to the expert's first row
    for (int e = threadIdx.x; e < n_experts; e += blockDim.x) {
        int run = 0;
        for (int w = 0; w < GROUP_WAVES; w++) {
            const int c = hist[w * n_experts + e];
            hist[w * n_experts + e] = run;
            run += c;
        }
        eoff[e + 1] = run;  // counts, scanned below
    }
    __syncthreads();
    if (wave == 0) {
        // exclusive scan of the counts (held at eoff[e + 1]) by one wave: a lane takes `per` consecutive experts
        constexpr int MAX_PER_LANE = 15;  // 960 experts
        const int per = (n_experts + 63) / 64;
        int cnt[MAX_PER_LANE];
        int local = 0;
#pragma unroll
        for (int k = 0; k < MAX_PER_LANE; k++) {
            const int e = lane * per + k;
            cnt[k] = (k < per && e < n_experts) ? eoff[e + 1] : 0;
            local += cnt[k];
        }
        int incl = local;
#pragma unroll
        for (int dlt = 1; dlt < 64; dlt <<= 1) {
            const int t = __shfl_up(incl, dlt, MK_WAVE);
            if (lane >= dlt) incl += t;
        }
        int run = incl - local;
#pragma unroll
        for (int k = 0; k < MAX_PER_LANE; k++) {
            const int e = lane * per + k;
            if (k < per && e < n_experts) eoff[e] = run;
            run += cnt[k];
        }
        if (lane == 63) eoff[n_experts] = incl;
    }
    __syncthreads();
    for (int e = threadIdx.x; e <= n_experts; e += blockDim.x) offsets[e] = eoff[e];
    // bits an expert id takes: the lanes of a chunk that hold the same id are found with one ballot per bit
    int nbits = 1;
    while ((1 << nbits) < n_experts) nbits++;
    const int i_end = min((wave + 1) * C, P);
    int e_next = wave * C + lane < P ? ids[wave * C + lane] : -1;  // (the next chunk's ids are asked for a chunk ahead)
    for (int i0 = wave * C; i0 < i_end; i0 += 64) {
        const int i = i0 + lane;
        const int e = e_next;
        e_next = (i0 + 64 < i_end && i + 64 < P) ? ids[i + 64] : -1;
        const bool valid = i < P && e >= 0 && e < n_experts;
        if (i < P && !valid) pos[i] = -1;
        // rank of the lane among the lanes of this chunk that hold the same expert, and the size of that group
        unsigned long long same_mask = __ballot(valid);
        for (int b = 0; b < nbits; b++) {
            const bool bit = (e >> b) & 1;
            const unsigned long long m = __ballot(valid && bit);
            same_mask &= bit ? m : ~m;
        }
        const int same = __popcll(same_mask), rank = __popcll(same_mask & ((1ull << lane) - 1ull));
        int start = 0;
        if (valid) start = eoff[e] + mine[e];  // every lane reads before any lane of this wave advances the counter
        __builtin_amdgcn_wave_barrier();       // ... also in the compiler's schedule: the reads above stay above the update
        if (valid) {
            const int r = start + rank;
            order[r] = i;
            pos[i] = r;
            if (rank == 0) mine[e] = start - eoff[e] + same;  // one lane per distinct key
        }
        __builtin_amdgcn_wave_barrier();  // the next chunk's reads come after this update
    }
}

// MXFP8 of the hidden row of each grouped pair: a lane takes 8 consecutive values, four lanes a 32-block
__global__ __launch_bounds__(256) void prefill_gather_mxfp8_kernel(const float *__restrict__ x, const int32_t *__restrict__ order,
                                                                   const int32_t *__restrict__ offsets, int n_experts, int topk, int d,
                                                                   uint8_t *__restrict__ codes, uint8_t *__restrict__ exps) {
    const int per_row = d / 8;
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;  // group of 8 values
    const size_t rows = (size_t)offsets[n_experts];                  // pairs with a valid expert id
    if (i >= rows * per_row) return;
    const size_t r = i / per_row, c = i % per_row;
    const int t = order[r] / topk;
    const mk_f4 *src = reinterpret_cast<const mk_f4 *>(x + (size_t)t * d) + 2 * c;
    const mk_f4 a = src[0], b = src[1];
    const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    uint32_t eb, c0, c1;
    mk_mxfp8_quantize8<127>(v, eb, c0, c1);  // full e8m0 range: a SwiGLU value of large experts passes 448 * 2^8
    reinterpret_cast<mk_u2 *>(codes)[i] = mk_u2{c0, c1};
    if ((c & 3) == 0) exps[r * (d / 32) + (c >> 2)] = (uint8_t)eb;
}

// act = ACT(gate, up) and its MXFP8 form
__global__ __launch_bounds__(256) void prefill_act_mxfp8_kernel(const float *__restrict__ g, const float *__restrict__ u,
                                                                const int32_t *__restrict__ offsets, int n_experts, int inter, int act_kind,
                                                                uint8_t *__restrict__ codes, uint8_t *__restrict__ exps) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;  // group of 8 values
    const size_t n = (size_t)offsets[n_experts] * (inter / 8);
    if (i >= n) return;
    const mk_f4 g0 = reinterpret_cast<const mk_f4 *>(g)[2 * i], g1 = reinterpret_cast<const mk_f4 *>(g)[2 * i + 1];
    const mk_f4 u0 = reinterpret_cast<const mk_f4 *>(u)[2 * i], u1 = reinterpret_cast<const mk_f4 *>(u)[2 * i + 1];
    const float gv[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w}, uv[8] = {u0.x, u0.y, u0.z, u0.w, u1.x, u1.y, u1.z, u1.w};
    float v[8];
#pragma unroll
    for (int k = 0; k < 8; k++) v[k] = mk_act(act_kind, gv[k], uv[k], 0.0f, 1.0f);
    uint32_t eb, c0, c1;
    mk_mxfp8_quantize8<127>(v, eb, c0, c1);  // full e8m0 range: a SwiGLU value of large experts passes 448 * 2^8
    reinterpret_cast<mk_u2 *>(codes)[i] = mk_u2{c0, c1};
    if ((i & 3) == 0) exps[i >> 2] = (uint8_t)eb;
}

// ACT(gate, up) in f32, written over the gate rows (src/model.rs:2589-2595)
__global__ __launch_bounds__(256) void prefill_act_f32_kernel(float *__restrict__ g, const float *__restrict__ u, const int32_t *__restrict__ offsets,
                                                              int n_experts, int inter, int act_kind) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;  // group of 4 values
    const size_t n = (size_t)offsets[n_experts] * (inter / 4);
    if (i >= n) return;
    const mk_f4 gv = reinterpret_cast<const mk_f4 *>(g)[i], uv = reinterpret_cast<const mk_f4 *>(u)[i];
    reinterpret_cast<mk_f4 *>(g)[i] = mk_f4{mk_act(act_kind, gv.x, uv.x, 0.0f, 1.0f), mk_act(act_kind, gv.y, uv.y, 0.0f, 1.0f),
                                           mk_act(act_kind, gv.z, uv.z, 0.0f, 1.0f), mk_act(act_kind, gv.w, uv.w, 0.0f, 1.0f)};
}

// bfloat16 (round to nearest even) of the hidden row of each grouped pair: a lane takes 8 consecutive values
__global__ __launch_bounds__(256) void prefill_gather_bf16_kernel(const float *__restrict__ x, const int32_t *__restrict__ order,
                                                                  const int32_t *__restrict__ offsets, int n_experts, int topk, int d,
                                                                  uint16_t *__restrict__ xb) {
    const int per_row = d / 8;
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t rows = (size_t)offsets[n_experts];
    if (i >= rows * per_row) return;
    const size_t r = i / per_row, c = i % per_row;
    const int t = order[r] / topk;
    const mk_f4 *src = reinterpret_cast<const mk_f4 *>(x + (size_t)t * d) + 2 * c;
    const mk_f4 a = src[0], b = src[1];
    typedef __bf16 bf8 __attribute__((ext_vector_type(8)));
    const bf8 v = {(__bf16)a.x, (__bf16)a.y, (__bf16)a.z, (__bf16)a.w, (__bf16)b.x, (__bf16)b.y, (__bf16)b.z, (__bf16)b.w};
    reinterpret_cast<bf8 *>(xb)[i] = v;
}

// bfloat16 of the hidden row of each grouped pair as two e4m3 terms per value (mk_bf16_split8), in the K-tile layout the
// two-term GEMM stages: a lane takes 8 consecutive values, four lanes a 32-block
__global__ __launch_bounds__(256) void prefill_gather_split_kernel(const float *__restrict__ x, const int32_t *__restrict__ order,
                                                                   const int32_t *__restrict__ offsets, int n_experts, int topk, int d,
                                                                   uint8_t *__restrict__ codes, uint8_t *__restrict__ exps) {
    const int per_row = d / 8;
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;  // group of 8 values
    const size_t rows = (size_t)offsets[n_experts];                  // pairs with a valid expert id
    if (i >= rows * per_row) return;  // (d % 32 == 0: whole quads leave together)
    const size_t r = i / per_row, c = i % per_row;
    const int t = order[r] / topk;
    const mk_f4 *src = reinterpret_cast<const mk_f4 *>(x + (size_t)t * d) + 2 * c;
    const mk_f4 a = src[0], b = src[1];
    const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    uint32_t hi[2], lo[2], eh, el;
    mk_bf16_split8<false>(v, hi, lo, eh, el);
    const size_t kt = c >> 6, within = (c & 63) * 8;  // K tile of 512 columns, byte inside it
    uint8_t *dst = codes + r * (2 * (size_t)d) + kt * 1024 + within;
    *reinterpret_cast<mk_u2 *>(dst) = mk_u2{hi[0], hi[1]};
    *reinterpret_cast<mk_u2 *>(dst + 512) = mk_u2{lo[0], lo[1]};
    if ((c & 3) == 0) {
        uint8_t *ed = exps + r * (size_t)(d / 16) + kt * 32 + ((c & 63) >> 2);
        ed[0] = (uint8_t)eh;
        ed[16] = (uint8_t)el;
    }
}

// act = ACT(gate, up) in f32, stored as bfloat16 (round to nearest even)
__global__ __launch_bounds__(256) void prefill_act_bf16_kernel(const float *__restrict__ g, const float *__restrict__ u,
                                                               const int32_t *__restrict__ offsets, int n_experts, int inter, int act_kind,
                                                               uint16_t *__restrict__ ab) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;  // group of 8 values
    const size_t n = (size_t)offsets[n_experts] * (inter / 8);
    if (i >= n) return;
    const mk_f4 g0 = reinterpret_cast<const mk_f4 *>(g)[2 * i], g1 = reinterpret_cast<const mk_f4 *>(g)[2 * i + 1];
    const mk_f4 u0 = reinterpret_cast<const mk_f4 *>(u)[2 * i], u1 = reinterpret_cast<const mk_f4 *>(u)[2 * i + 1];
    const float gv[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w}, uv[8] = {u0.x, u0.y, u0.z, u0.w, u1.x, u1.y, u1.z, u1.w};
    typedef __bf16 bf8 __attribute__((ext_vector_type(8)));
    bf8 v;
#pragma unroll
    for (int k = 0; k < 8; k++) v[k] = (__bf16)mk_act(act_kind, gv[k], uv[k], 0.0f, 1.0f);
    reinterpret_cast<bf8 *>(ab)[i] = v;
}

// out_t = sum_s w[t][s] * o[pos(t, s)] in slot order, multiply then add (src/model.rs:2690-2700)
__global__ __launch_bounds__(256) void prefill_combine_kernel(const float *__restrict__ o, const int32_t *__restrict__ pos,
                                                              const float *__restrict__ weights, int topk, int d, float *__restrict__ out) {
    const int t = blockIdx.y;
    const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (c >= d) return;
    mk_f4 y = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int s = 0; s < topk; s++) {
        const int r = pos[t * topk + s];
        if (r < 0) continue;
        const float w = weights[t * topk + s];
        const mk_f4 v = *reinterpret_cast<const mk_f4 *>(o + (size_t)r * d + c);
        y.x = mk_add(y.x, mk_mul(w, v.x));
        y.y = mk_add(y.y, mk_mul(w, v.y));
        y.z = mk_add(y.z, mk_mul(w, v.z));
        y.w = mk_add(y.w, mk_mul(w, v.w));
    }
    *reinterpret_cast<mk_f4 *>(out + (size_t)t * d + c) = y;
}

}  // namespace

extern "C" size_t mk_moe_prefill_workspace_bytes(size_t T, size_t topk, size_t n_experts, size_t d, size_t inter) {
    return carve(nullptr, T * topk, n_experts, d, inter).bytes;
}

extern "C" int mk_moe_prefill_workspace_layout(size_t T, size_t topk, size_t n_experts, size_t d, size_t inter, mk_prefill_layout *out) {
    MK_REQUIRE(out, "null pointer");
    // carve() from a non-null dummy base: the differences are the offsets
    uint8_t *base = reinterpret_cast<uint8_t *>((uintptr_t)4096);
    const PrefillWs w = carve(base, T * topk, n_experts, d, inter);
    auto off = [&](const void *p) { return (size_t)((const uint8_t *)p - base); };
    out->order = off(w.order);
    out->pos = off(w.pos);
    out->offsets = off(w.offsets);
    out->g = off(w.g);
    out->u = off(w.u);
    out->o = off(w.o);
    return MK_OK;
}

namespace {
int moe_prefill_impl(const mk_expert_table *table, size_t n_experts, size_t T, size_t topk, const int32_t *ids, const float *weights,
                     const float *x, int act_kind, void *workspace, float *out, void *stream, bool keep) {
    MK_REQUIRE(table && ids && weights && x && workspace && out, "null pointer");
    MK_REQUIRE(act_kind == MK_ACT_SWIGLU || act_kind == MK_ACT_SITU, "moe_prefill knows the SwiGLU and SiTU activations");
    if (table->vq_codebook) {  // quant::matvec_vq_nt experts (src/model.rs:2556-2566): mk_dev_vq1_matvec_nt per expert, not this call
        mk_set_error("mk_dev_moe_prefill reads MXFP4 experts only; this layer holds VQ1 experts");
        return MK_ERR_UNSUPPORTED;
    }
    const size_t d = table->d, inter = table->inter;
    MK_REQUIRE(d % 128 == 0 && inter % 128 == 0 && d > 0 && inter > 0, "d and inter must be positive multiples of 128");
    MK_REQUIRE(n_experts >= 1 && n_experts <= 960 && T >= 1 && topk >= 1 && T <= 65535, "bad token / expert count");
    MK_REQUIRE(T * topk <= (size_t)GROUP_MAX_P, "at most 16384 (token, slot) pairs per call: split the prompt");
    MK_REQUIRE(((uintptr_t)workspace & 255) == 0 && ((uintptr_t)out & 15) == 0, "workspace must be 256-byte and out 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    const size_t P = T * topk;
    PrefillWs w = carve(workspace, P, n_experts, d, inter);
    const size_t group_lds = ((size_t)GROUP_WAVES * n_experts + n_experts + 1) * sizeof(int);
    MK_REQUIRE(group_lds <= 64 * 1024, "too many experts for the grouping kernel (17 counters per expert in 64 KiB of LDS)");
    hipLaunchKernelGGL(prefill_group_kernel, dim3(1), dim3(GROUP_WAVES * 64), group_lds, st, ids, (int)P, (int)n_experts, w.order, w.pos,
                       w.offsets);
    int s = mk_launch_status("prefill_group");
    if (s != MK_OK) return s;
    MK_REQUIRE(((uintptr_t)x & 15) == 0, "x must be 16-byte aligned");
    hipLaunchKernelGGL(prefill_gather_mxfp8_kernel, dim3((unsigned)((P * (d / 8) + 255) / 256)), dim3(256), 0, st, x, w.order, w.offsets,
                       (int)n_experts, (int)topk, (int)d, w.codes, w.exps);
    if ((s = mk_launch_status("prefill_gather_mxfp8")) != MK_OK) return s;
    // gate, up, activation and its MXFP8 form in one launch; shapes that launch does not take run the three steps
    s = MK_TUNE("MK_PREFILL_SEPARATE", 0) ? MK_ERR_UNSUPPORTED
                                         : mk_mxfp4_grouped_gemm_gate_up_act(table->w1p, table->w1s, table->w3p, table->w3s, n_experts, inter, d, w.codes,
                                                                             w.exps, w.offsets, P, act_kind, w.codes2, w.exps2, keep ? w.g : nullptr,
                                                                             keep ? w.u : nullptr, stream, table->w1st, table->w3st);
    if (s == MK_ERR_UNSUPPORTED) {
        const uint8_t *const *pp[2] = {table->w1p, table->w3p};
        const uint8_t *const *sp[2] = {table->w1s, table->w3s};
        float *gu[2] = {w.g, w.u};
        const uint8_t *const *tp[2] = {table->w1st, table->w3st};
        if ((s = mk_mxfp4_grouped_gemm_n(2, pp, sp, n_experts, inter, d, w.codes, w.exps, w.offsets, P, gu, stream,
                                         table->w1st && table->w3st ? tp : nullptr)) != MK_OK)
            return s;
        hipLaunchKernelGGL(prefill_act_mxfp8_kernel, dim3((unsigned)((P * (inter / 8) + 255) / 256)), dim3(256), 0, st, w.g, w.u, w.offsets,
                           (int)n_experts, (int)inter, act_kind, w.codes2, w.exps2);
        s = mk_launch_status("prefill_act_mxfp8");
    }
    if (s != MK_OK) return s;
    {
        const uint8_t *const *pd[1] = {table->w2p};
        const uint8_t *const *sd[1] = {table->w2s};
        const uint8_t *const *td[1] = {table->w2st};
        float *od[1] = {w.o};
        if ((s = mk_mxfp4_grouped_gemm_n(1, pd, sd, n_experts, d, inter, w.codes2, w.exps2, w.offsets, P, od, stream, table->w2st ? td : nullptr)) != MK_OK)
            return s;
    }
    hipLaunchKernelGGL(prefill_combine_kernel, dim3((unsigned)((d / 4 + 255) / 256), (unsigned)T), dim3(256), 0, st, w.o, w.pos, weights, (int)topk,
                       (int)d, out);
    return mk_launch_status("prefill_combine");
}
}  // namespace

// The section in the reference's own arithmetic: f32 hidden rows and f32 activation against the dequantized weights.
extern "C" int mk_dev_moe_prefill_f32(const mk_expert_table *table, size_t n_experts, size_t T, size_t topk, const int32_t *ids,
                                      const float *weights, const float *x, int act_kind, void *workspace, float *out, void *stream) {
    MK_REQUIRE(table && ids && weights && x && workspace && out, "null pointer");
    MK_REQUIRE(act_kind == MK_ACT_SWIGLU || act_kind == MK_ACT_SITU, "moe_prefill knows the SwiGLU and SiTU activations");
    const size_t d = table->d, inter = table->inter;
    MK_REQUIRE(d % 128 == 0 && inter % 128 == 0 && d > 0 && inter > 0, "d and inter must be positive multiples of 128");
    MK_REQUIRE(n_experts >= 1 && n_experts <= 960 && T >= 1 && topk >= 1 && T <= 65535, "bad token / expert count");
    MK_REQUIRE(T * topk <= (size_t)GROUP_MAX_P, "at most 16384 (token, slot) pairs per call: split the prompt");
    MK_REQUIRE(((uintptr_t)workspace & 255) == 0 && ((uintptr_t)out & 15) == 0 && ((uintptr_t)x & 15) == 0,
               "workspace must be 256-byte, x and out 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    const size_t P = T * topk;
    PrefillWs w = carve(workspace, P, n_experts, d, inter);
    const size_t group_lds = ((size_t)GROUP_WAVES * n_experts + n_experts + 1) * sizeof(int);
    MK_REQUIRE(group_lds <= 64 * 1024, "too many experts for the grouping kernel (17 counters per expert in 64 KiB of LDS)");
    hipLaunchKernelGGL(prefill_group_kernel, dim3(1), dim3(GROUP_WAVES * 64), group_lds, st, ids, (int)P, (int)n_experts, w.order, w.pos,
                       w.offsets);
    int s = mk_launch_status("prefill_group");
    if (s != MK_OK) return s;
    // gate and up read the hidden row of their pair through the grouping (pair index / topk), no gathered copy
    const uint8_t *const *pp[2] = {table->w1p, table->w3p};
    const uint8_t *const *sp[2] = {table->w1s, table->w3s};
    float *gu[2] = {w.g, w.u};
    if ((s = mk_mxfp4_grouped_gemm_nt(2, pp, sp, n_experts, inter, d, x, w.order, (int)topk, w.offsets, P, table->vq_codebook, gu, stream)) != MK_OK) return s;
    hipLaunchKernelGGL(prefill_act_f32_kernel, dim3((unsigned)((P * (inter / 4) + 255) / 256)), dim3(256), 0, st, w.g, w.u, w.offsets,
                       (int)n_experts, (int)inter, act_kind);
    if ((s = mk_launch_status("prefill_act_f32")) != MK_OK) return s;
    const uint8_t *const *pd[1] = {table->w2p};
    const uint8_t *const *sd[1] = {table->w2s};
    float *od[1] = {w.o};
    if ((s = mk_mxfp4_grouped_gemm_nt(1, pd, sd, n_experts, d, inter, w.g, nullptr, 1, w.offsets, P, table->vq_codebook, od, stream)) != MK_OK) return s;
    hipLaunchKernelGGL(prefill_combine_kernel, dim3((unsigned)((d / 4 + 255) / 256), (unsigned)T), dim3(256), 0, st, w.o, w.pos, weights, (int)topk,
                       (int)d, out);
    return mk_launch_status("prefill_combine");
}

// The section with bfloat16 hidden rows and activation rows against the exact weights (bf16 matrix instruction).
namespace {
int moe_prefill_bf16_impl(const mk_expert_table *table, size_t n_experts, size_t T, size_t topk, const int32_t *ids, const float *weights,
                          const float *x, int act_kind, void *workspace, float *out, void *stream, bool keep) {
    MK_REQUIRE(table && ids && weights && x && workspace && out, "null pointer");
    MK_REQUIRE(act_kind == MK_ACT_SWIGLU || act_kind == MK_ACT_SITU, "moe_prefill knows the SwiGLU and SiTU activations");
    if (table->vq_codebook) {
        mk_set_error("mk_dev_moe_prefill_bf16 reads MXFP4 experts only; this layer holds VQ1 experts (mk_dev_moe_prefill_f32 takes them)");
        return MK_ERR_UNSUPPORTED;
    }
    const size_t d = table->d, inter = table->inter;
    if (d == 0 || inter == 0 || d % 512 != 0 || inter % 512 != 0) {
        mk_set_error("mk_dev_moe_prefill_bf16 takes d and inter in multiples of 512");
        return MK_ERR_UNSUPPORTED;
    }
    MK_REQUIRE(n_experts >= 1 && n_experts <= 960 && T >= 1 && topk >= 1 && T <= 65535, "bad token / expert count");
    MK_REQUIRE(T * topk <= (size_t)GROUP_MAX_P, "at most 16384 (token, slot) pairs per call: split the prompt");
    MK_REQUIRE(((uintptr_t)workspace & 255) == 0 && ((uintptr_t)out & 15) == 0 && ((uintptr_t)x & 15) == 0,
               "workspace must be 256-byte, x and out 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    const size_t P = T * topk;
    PrefillWs w = carve(workspace, P, n_experts, d, inter);
    const size_t group_lds = ((size_t)GROUP_WAVES * n_experts + n_experts + 1) * sizeof(int);
    MK_REQUIRE(group_lds <= 64 * 1024, "too many experts for the grouping kernel (17 counters per expert in 64 KiB of LDS)");
    hipLaunchKernelGGL(prefill_group_kernel, dim3(1), dim3(GROUP_WAVES * 64), group_lds, st, ids, (int)P, (int)n_experts, w.order, w.pos,
                       w.offsets);
    int s = mk_launch_status("prefill_group");
    if (s != MK_OK) return s;
    // Two forms.  The two-term form (every bfloat16 value as two e4m3 terms on the block-scaled matrix instruction, the
    // streaming kernels of the MXFP8 section) is the default; MK_PREFILL_BF16_MFMA=1 selects the bfloat16 matrix instruction.
    if (!MK_TUNE("MK_PREFILL_BF16_MFMA", 0) && P * d * 2 < 0xFFFFFFFFull && P * inter * 2 < 0xFFFFFFFFull) {
        hipLaunchKernelGGL(prefill_gather_split_kernel, dim3((unsigned)((P * (d / 8) + 255) / 256)), dim3(256), 0, st, x, w.order, w.offsets,
                           (int)n_experts, (int)topk, (int)d, w.split_codes, w.split_exps);
        if ((s = mk_launch_status("prefill_gather_split")) != MK_OK) return s;
        s = mk_mxfp4_grouped_gemm_gate_up_act(table->w1p, table->w1s, table->w3p, table->w3s, n_experts, inter, d, w.split_codes, w.split_exps,
                                              w.offsets, P, act_kind, w.split_codes2, w.split_exps2, keep ? w.g : nullptr, keep ? w.u : nullptr, stream,
                                              table->w1st, table->w3st, true);
        if (s != MK_OK) return s;  // (d and inter in multiples of 512: the launch takes every such shape)
        const uint8_t *const *pd[1] = {table->w2p};
        const uint8_t *const *sd[1] = {table->w2s};
        const uint8_t *const *td[1] = {table->w2st};
        float *od[1] = {w.o};
        if ((s = mk_mxfp4_grouped_gemm_n(1, pd, sd, n_experts, d, inter, w.split_codes2, w.split_exps2, w.offsets, P, od, stream,
                                         table->w2st ? td : nullptr, true)) != MK_OK)
            return s;
        hipLaunchKernelGGL(prefill_combine_kernel, dim3((unsigned)((d / 4 + 255) / 256), (unsigned)T), dim3(256), 0, st, w.o, w.pos, weights,
                           (int)topk, (int)d, out);
        return mk_launch_status("prefill_combine");
    }
    hipLaunchKernelGGL(prefill_gather_bf16_kernel, dim3((unsigned)((P * (d / 8) + 255) / 256)), dim3(256), 0, st, x, w.order, w.offsets,
                       (int)n_experts, (int)topk, (int)d, w.xb);
    if ((s = mk_launch_status("prefill_gather_bf16")) != MK_OK) return s;
    const uint8_t *const *pp[2] = {table->w1p, table->w3p};
    const uint8_t *const *sp[2] = {table->w1s, table->w3s};
    float *gu[2] = {w.g, w.u};
    const uint8_t *const *tp[2] = {table->w1st, table->w3st};
    if ((s = mk_mxfp4_grouped_gemm_bf16(2, pp, sp, n_experts, inter, d, w.xb, w.offsets, gu, stream, table->w1st && table->w3st ? tp : nullptr)) != MK_OK)
        return s;
    // (the hidden rows are used up: the activation rows take their place)
    hipLaunchKernelGGL(prefill_act_bf16_kernel, dim3((unsigned)((P * (inter / 8) + 255) / 256)), dim3(256), 0, st, w.g, w.u, w.offsets,
                       (int)n_experts, (int)inter, act_kind, w.xb);
    if ((s = mk_launch_status("prefill_act_bf16")) != MK_OK) return s;
    const uint8_t *const *pd[1] = {table->w2p};
    const uint8_t *const *sd[1] = {table->w2s};
    float *od[1] = {w.o};
    const uint8_t *const *td[1] = {table->w2st};
    if ((s = mk_mxfp4_grouped_gemm_bf16(1, pd, sd, n_experts, d, inter, w.xb, w.offsets, od, stream, table->w2st ? td : nullptr)) != MK_OK) return s;
    hipLaunchKernelGGL(prefill_combine_kernel, dim3((unsigned)((d / 4 + 255) / 256), (unsigned)T), dim3(256), 0, st, w.o, w.pos, weights, (int)topk,
                       (int)d, out);
    return mk_launch_status("prefill_combine");
}

}  // namespace

extern "C" int mk_dev_moe_prefill_bf16(const mk_expert_table *table, size_t n_experts, size_t T, size_t topk, const int32_t *ids,
                                       const float *weights, const float *x, int act_kind, void *workspace, float *out, void *stream) {
    // (the f32 gate and up rows are stored too: the launch is bound by its loads and the stores cost nothing measurable)
    return moe_prefill_bf16_impl(table, n_experts, T, topk, ids, weights, x, act_kind, workspace, out, stream, true);
}

extern "C" int mk_dev_moe_prefill(const mk_expert_table *table, size_t n_experts, size_t T, size_t topk, const int32_t *ids,
                                  const float *weights, const float *x, int act_kind, void *workspace, float *out, void *stream) {
    return moe_prefill_impl(table, n_experts, T, topk, ids, weights, x, act_kind, workspace, out, stream, false);
}

extern "C" int mk_dev_moe_prefill_keep(const mk_expert_table *table, size_t n_experts, size_t T, size_t topk, const int32_t *ids,
                                       const float *weights, const float *x, int act_kind, void *workspace, float *out, void *stream) {
    return moe_prefill_impl(table, n_experts, T, topk, ids, weights, x, act_kind, workspace, out, stream, true);
}
