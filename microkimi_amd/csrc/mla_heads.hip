// q8_0 MLA attention over the cache layout the reference keeps (src/model.rs:765-781): per position and head a
// latent K row (nope int8 + nope/32 f32 scales) and a V row (vd int8 + vd/32 f32 scales), plus ONE f32 rope row per
// position shared by the heads.
//
//   append   MlaCache::push (src/model.rs:1583-1618) for one or many positions (many = assign_f32,
//            src/model.rs:1680-1692): rope row from head 0, q8::quantize_q8_into per head for K-nope and V
//   to_f32   MlaCache::to_f32 (src/model.rs:1623-1676)
//   decode   mla_attn_flash_q8_mqa (src/model.rs:1804-1908) for one query per head: every head owns its K and V
//            rows, so each cache byte is used once -- a streaming kernel, HBM-bound by construction.  Grid (split,
//            head, query): four waves walk 64-position tiles; scores with v_dot4_i32_i8 on the raw bytes and the
//            reference's per-block scale product, f32 rope dot, online softmax, V rows dequantized as q * s.
//            Splits are merged by log-sum-exp.  With several queries (prefill, src/model.rs:2080-2102) query i
//            attends positions 0 ..= pos0 + i.
//
// The Hadamard option (kv_hadamard / hadamard64, src/model.rs:1529-1554; MICROKIMI_KV_HADAMARD=1, off by default): every
// 64-chunk of a K-nope row, a V row and a query's nope part goes through the unnormalized Walsh-Hadamard butterfly
// before it is quantized; the latent score carries the factor 1/64 and the attention output is rotated back.  As in the
// reference it applies only when nope and v are multiples of 64.  The butterfly is the reference's: the same six stages
// of one addition or subtraction per element, so the rotated values (and the cache bytes) are identical.
#include "mk_common.h"

namespace {

constexpr int TJ = 64;          // positions per tile (FLASH_KV, src/model.rs:1348)
constexpr int MAX_SPLITS = 64;
constexpr int MAX_NB = 8;       // latent blocks per head the decode kernel holds in registers (nope <= 256)
constexpr int MAX_VD = 512;

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// hadamard64 (src/model.rs:1540-1554) on a 64-chunk held one element per lane by a whole wave: stage h pairs lane j
// (bit h clear) with lane j + h: x[j] = a + b, x[j + h] = a - b.
__device__ __forceinline__ float hadamard64_lane(float v, int lane) {
#pragma unroll
    for (int h = 1; h < 64; h <<= 1) {
        const float o = __shfl_xor(v, h, MK_WAVE);
        v = (lane & h) ? o - v : v + o;
    }
    return v;
}

// One 32-block per aligned group of 32 lanes: q8::quantize_q8_into (src/q8.rs:57-68).
__device__ __forceinline__ void quantize_block32(float v, int8_t *q_out, float *s_out, int j) {
    const float mx = mk_half_wave_max(fabsf(v));
    const float dx = fmaxf(mx, 0.0f) / 127.0f;  // (a block of NaN only: the reference's maximum, folded from 0, is 0)
    q_out[j] = (int8_t)(dx != 0.0f ? mk_q8_round(v, dx) : 0);
    if (j == 0) *s_out = dx;
}

// grid: (blocks of the position's rows, position).  Blocks 0 .. nh*nope/32-1: K-nope of head h; then nh*vd/32 V blocks;
// the last workgroups copy the rope row of head 0.
__global__ __launch_bounds__(256) void heads_append_kernel(const float *__restrict__ k_rows, const float *__restrict__ v_rows, int nh, int nope,
                                                           int rope, int vd, size_t pos0, int had, int8_t *__restrict__ kq,
                                                           float *__restrict__ ks, float *__restrict__ kr, int8_t *__restrict__ vq,
                                                           float *__restrict__ vs) {
    // (with the Hadamard option nope and vd are multiples of 64: a wave then holds one 64-chunk, two blocks of one row)
    const int nbk = nh * nope / 32, nbv = nh * vd / 32;
    const size_t jn = blockIdx.y, pos = pos0 + jn;
    const int blk = (blockIdx.x * blockDim.x + threadIdx.x) >> 5, j = threadIdx.x & 31;
    const int qh = nope + rope;
    if (blk < nbk) {
        const int h = blk / (nope / 32), g = blk % (nope / 32);
        float v = k_rows[(jn * nh + h) * qh + g * 32 + j];
        if (had) v = hadamard64_lane(v, threadIdx.x & 63);
        quantize_block32(v, kq + (pos * nh + h) * nope + g * 32, ks + pos * nbk + blk, j);
    } else if (blk < nbk + nbv) {
        const int b = blk - nbk, h = b / (vd / 32), g = b % (vd / 32);
        float v = v_rows[(jn * nh + h) * vd + g * 32 + j];
        if (had) v = hadamard64_lane(v, threadIdx.x & 63);
        quantize_block32(v, vq + (pos * nh + h) * vd + g * 32, vs + pos * nbv + b, j);
    } else {
        const int d = (blk - nbk - nbv) * 32 + j;
        if (d < rope) kr[pos * rope + d] = k_rows[jn * nh * qh + nope + d];  // rope is shared: stored once, from head 0
    }
}

__global__ __launch_bounds__(256) void heads_to_f32_kernel(const int8_t *__restrict__ kq, const float *__restrict__ ks,
                                                           const float *__restrict__ kr, const int8_t *__restrict__ vq,
                                                           const float *__restrict__ vs, int nh, int nope, int rope, int vd,
                                                           float *__restrict__ k, float *__restrict__ v) {
    const size_t j = blockIdx.y;
    const int qh = nope + rope;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < nh * qh; i += gridDim.x * blockDim.x) {
        const int h = i / qh, d = i % qh;
        k[(j * nh + h) * qh + d] = d < nope ? (float)kq[(j * nh + h) * nope + d] * ks[(j * nh + h) * (nope / 32) + d / 32] : kr[j * rope + d - nope];
    }
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < nh * vd; i += gridDim.x * blockDim.x) {
        const int h = i / vd, d = i % vd;
        v[(j * nh + h) * vd + d] = (float)vq[(j * nh + h) * vd + d] * vs[(j * nh + h) * (vd / 32) + d / 32];
    }
}

// The same with the Hadamard option: a wave per 64-chunk, dequantized, rotated back (butterfly, then / 64).
__global__ __launch_bounds__(256) void heads_to_f32_had_kernel(const int8_t *__restrict__ kq, const float *__restrict__ ks,
                                                               const float *__restrict__ kr, const int8_t *__restrict__ vq,
                                                               const float *__restrict__ vs, int nh, int nope, int rope, int vd,
                                                               float *__restrict__ k, float *__restrict__ v) {
    const size_t j = blockIdx.y;
    const int qh = nope + rope, lane = threadIdx.x & 63;
    const int ck = nh * nope / 64, cv = nh * vd / 64;
    for (int c = (blockIdx.x * blockDim.x + threadIdx.x) >> 6; c < ck + cv; c += (gridDim.x * blockDim.x) >> 6) {
        if (c < ck) {
            const int h = c / (nope / 64), d = (c % (nope / 64)) * 64 + lane;
            const float x = (float)kq[(j * nh + h) * nope + d] * ks[(j * nh + h) * (nope / 32) + d / 32];
            k[(j * nh + h) * qh + d] = hadamard64_lane(x, lane) / 64.0f;
        } else {
            const int cc = c - ck, h = cc / (vd / 64), d = (cc % (vd / 64)) * 64 + lane;
            const float x = (float)vq[(j * nh + h) * vd + d] * vs[(j * nh + h) * (vd / 32) + d / 32];
            v[(j * nh + h) * vd + d] = hadamard64_lane(x, lane) / 64.0f;
        }
    }
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < nh * rope; i += gridDim.x * blockDim.x) {
        const int h = i / rope, d = i % rope;
        k[(j * nh + h) * qh + nope + d] = kr[j * rope + d];
    }
}

// The attention rows rotated back (src/model.rs:1896-1903): butterfly, then / 64, per 64-chunk.
__global__ __launch_bounds__(256) void heads_out_had_kernel(float *__restrict__ out, size_t chunks) {
    const size_t c = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int lane = threadIdx.x & 63;
    if (c >= chunks) return;
    out[c * 64 + lane] = hadamard64_lane(out[c * 64 + lane], lane) / 64.0f;
}

// q8 of the latent part of every (query, head): (src/model.rs:1812-1821)
__global__ __launch_bounds__(256) void heads_q_prep_kernel(const float *__restrict__ q, int rows, int nope, int rope, int had,
                                                           int8_t *__restrict__ qq, float *__restrict__ qs) {
    const int nb = nope / 32;
    const int blk = (blockIdx.x * blockDim.x + threadIdx.x) >> 5, j = threadIdx.x & 31;
    if (blk >= rows * nb) return;  // (with the Hadamard option nb is even: both halves of a wave stay or leave together)
    const int r = blk / nb, g = blk % nb;
    float v = q[(size_t)r * (nope + rope) + g * 32 + j];
    if (had) v = hadamard64_lane(v, threadIdx.x & 63);
    quantize_block32(v, qq + (size_t)r * nope + g * 32, qs + blk, j);
}

// The same without the rotation, 8 lanes a block and four values a lane (quantize_q8_into, src/q8.rs:57-68).
__global__ __launch_bounds__(256) void heads_q_prep4_kernel(const float *__restrict__ q, size_t n_blocks, int nope, int rope,
                                                            int8_t *__restrict__ qq, float *__restrict__ qs) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_blocks * 8) return;  // whole groups of 8 lanes leave together
    const int nb = nope / 32;
    const size_t blk = i >> 3, r = blk / nb;
    const int g = (int)(blk - r * nb), c = (int)(i & 7);
    const mk_f4 v = *reinterpret_cast<const mk_f4 *>(q + r * (nope + rope) + g * 32 + c * 4);
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
    reinterpret_cast<uint32_t *>(qq)[i] = packed;  // qq is [rows][nope]: block blk starts at byte 32 blk
    if (c == 0) qs[blk] = dx;
}

struct HeadsArgs {
    const int8_t *kq;
    const float *ks;
    const float *kr;
    const int8_t *vq;
    const float *vs;
    const float *q;    // [m][nh][nope+rope]
    const int8_t *qq;  // [m][nh][nope]
    const float *qs;   // [m][nh][nope/32]
    int nh, nope, rope, vd, n_pos0, split_len, n_splits;
    float scale;
    float had_k;          // factor of the latent part of a score: 1/64 with the Hadamard option (src/model.rs:1823), else 1
    float *po, *pm, *pl;  // split partials (one query only)
    float *out;           // [m][nh][vd]
};

// Workgroup = (split, head, query), 256 threads.  Per 64-position tile:
//   scores   thread (i = tid / 4, part = tid % 4): position i of the tile, blocks part, part + 4, ... of the head's latent
//            row and every 4th rope dim; the four parts meet through two lane shuffles
//   softmax  every wave reduces the 64 scores itself (no second barrier for the statistics)
//   out      thread (slot = tid / 32, dq = tid % 32): positions slot, slot + 8, ... of the tile, dims 4 dq .. 4 dq + 3
//            (+128, +256, +384 for wider V rows); the eight slots meet in LDS at the end
__global__ __launch_bounds__(256) void heads_decode_kernel(HeadsArgs a) {
    __shared__ float sc_l[TJ];
    __shared__ float red_l[8][MAX_VD];
    const int tid = threadIdx.x, lane = tid & 63;
    const int split = blockIdx.x, h = blockIdx.y, qi = blockIdx.z;
    const int nh = a.nh, nope = a.nope, rope = a.rope, vd = a.vd, nb = nope / 32, nbv = vd / 32;
    const int n_pos = a.n_pos0 + qi;
    const int p_begin = split * a.split_len;
    const int p_end = min(p_begin + a.split_len, n_pos);
    const size_t qrow = (size_t)qi * nh + h;
    // this thread's share of the query: latent blocks part, part + 4, ... and rope dims part, part + 4, ...
    const int part = tid & 3, ip = tid >> 2;
    mk_i4 qreg[MAX_NB / 4][2];
    float qsc[MAX_NB / 4];
#pragma unroll
    for (int k = 0; k < MAX_NB / 4; k++) {
        const int g = part + 4 * k;
        if (g < nb) {
            const mk_i4 *src = reinterpret_cast<const mk_i4 *>(a.qq + qrow * nope + g * 32);
            qreg[k][0] = src[0];
            qreg[k][1] = src[1];
            qsc[k] = a.qs[qrow * nb + g] * a.had_k;  // (a power of two: the product with 1/64 is exact)
        } else {
            qreg[k][0] = qreg[k][1] = mk_i4{0, 0, 0, 0};
            qsc[k] = 0.0f;
        }
    }
    const float *qr = a.q + qrow * (nope + rope) + nope;
    const int slot = tid >> 5, dq = tid & 31;
    float o[MAX_VD / 128][4];
#pragma unroll
    for (int c = 0; c < MAX_VD / 128; c++)
#pragma unroll
        for (int e = 0; e < 4; e++) o[c][e] = 0.0f;
    float m = -INFINITY, l = 0.0f;

    for (int t0 = p_begin; t0 < p_end; t0 += TJ) {
        const int tn = min(TJ, p_end - t0);
        // ---- scores
        float s = 0.0f;
        if (ip < tn) {
            const size_t j = (size_t)(t0 + ip);
            const int8_t *krow = a.kq + (j * nh + h) * nope;
            const float *ksr = a.ks + (j * nh + h) * nb;
#pragma unroll
            for (int k = 0; k < MAX_NB / 4; k++) {
                const int g = part + 4 * k;
                if (g < nb) {
                    const mk_i4 *src = reinterpret_cast<const mk_i4 *>(krow + g * 32);
                    const mk_i4 k0 = src[0], k1 = src[1];
                    int idot = 0;
#pragma unroll
                    for (int e = 0; e < 4; e++) idot = __builtin_amdgcn_sdot4(k0[e], qreg[k][0][e], idot, false);
#pragma unroll
                    for (int e = 0; e < 4; e++) idot = __builtin_amdgcn_sdot4(k1[e], qreg[k][1][e], idot, false);
                    s += (qsc[k] * ksr[g]) * (float)idot;
                }
            }
            const float *krr = a.kr + j * rope;
            for (int d = part; d < rope; d += 4) s += qr[d] * krr[d];
        }
        s += __shfl_xor(s, 1, MK_WAVE);
        s += __shfl_xor(s, 2, MK_WAVE);
        __syncthreads();  // the previous tile's scores have been consumed
        if (part == 0) sc_l[ip] = ip < tn ? s * a.scale : -INFINITY;
        __syncthreads();
        // ---- online softmax (every wave computes the tile's statistics for itself)
        const float sv = sc_l[lane];
        const float tm = mk_wave_max(sv);
        const float m_new = fmaxf(m, tm);
        const float corr = expf(m - m_new);
        const float pv = expf(sv - m_new);  // -inf score (position past the end) gives 0
        l = l * corr + mk_wave_sum(pv);
        m = m_new;
#pragma unroll
        for (int c = 0; c < MAX_VD / 128; c++)
#pragma unroll
            for (int e = 0; e < 4; e++) o[c][e] *= corr;
        // ---- out += p V: this thread's positions slot, slot + 8, ...
        for (int i = slot; i < tn; i += 8) {
            const float p = expf(sc_l[i] - m_new);
            const size_t j = (size_t)(t0 + i);
            const int8_t *vrow = a.vq + (j * nh + h) * vd;
            const float *vsr = a.vs + (j * nh + h) * nbv;
#pragma unroll
            for (int c = 0; c < MAX_VD / 128; c++) {
                const int d0 = 128 * c + 4 * dq;
                if (d0 < vd) {
                    const uint32_t w = *reinterpret_cast<const uint32_t *>(vrow + d0);
                    const float ps = p * vsr[d0 >> 5];
#pragma unroll
                    for (int e = 0; e < 4; e++) o[c][e] += ps * (float)(int8_t)(w >> (8 * e));
                }
            }
        }
    }
    // ---- the eight position slots meet in LDS
    __syncthreads();
#pragma unroll
    for (int c = 0; c < MAX_VD / 128; c++) {
        const int d0 = 128 * c + 4 * dq;
        if (d0 < vd)
#pragma unroll
            for (int e = 0; e < 4; e++) red_l[slot][d0 + e] = o[c][e];
    }
    __syncthreads();
    for (int d = tid; d < vd; d += 256) {
        float v = red_l[0][d];
#pragma unroll
        for (int k = 1; k < 8; k++) v += red_l[k][d];
        if (a.n_splits == 1) {
            a.out[qrow * vd + d] = v / l;
        } else {
            a.po[((size_t)split * nh + h) * vd + d] = v;
        }
    }
    if (a.n_splits > 1 && tid == 0) {
        a.pm[split * nh + h] = m;
        a.pl[split * nh + h] = l;
    }
}

// The all-heads form for the reference's own head shape, nope 128 + rope 64 / v 128 (its mla_attn_flash_q8_mqa streams the
// cache once, tile outer / head inner, src/model.rs:1804-1908): a workgroup takes 8 neighbouring heads over a split of the positions, a wave
// every 4th position, 8 lanes a head.  One load instruction of a wave is then 1 KB of consecutive bytes (the K rows, or
// the V rows, of the 8 heads at one position), the 8 heads' block scales are exactly one 128-byte line, the rope row is
// read once for the 8 heads.  Every wave runs its own online softmax over its positions (no barrier and no LDS in the
// loop); the four states of a head meet once at the end.
struct G8Pos {
    mk_i4 k;
    float ks;
    mk_f4 r0, r1;
    mk_i4 v;
    float vs;
};

constexpr int G8_U = 2;  // positions a wave takes per step (4 measured the same with twice the registers)
__global__ __launch_bounds__(256) void heads_decode_g8_kernel(HeadsArgs a) {
        constexpr int NOPE = 128, ROPE = 64, VD = 128, U = G8_U;
    __shared__ float o_l[4][8][VD + 4];
    __shared__ float m_l[4][8], l_l[4][8];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int hgroups = (a.nh + 7) >> 3;  // a last group with fewer than 8 heads re-reads the last head in its idle lanes
    // consecutive workgroup ids go round the 8 XCDs (each with its own L2): XCD x takes the splits x, x + 8, ... with all
    // their head groups, so a position's rope row is fetched by one of them only
    int split, hg;
    if ((a.n_splits & 7) == 0) {
        const int r = blockIdx.x >> 3;
        split = (blockIdx.x & 7) + 8 * (r / hgroups);
        hg = r % hgroups;
    } else {
        split = blockIdx.x / hgroups;
        hg = blockIdx.x - split * hgroups;
    }
    const int qi = blockIdx.y;
    const int hl = lane >> 3, c = lane & 7, h = min(hg * 8 + hl, a.nh - 1);
    const uint32_t nh = (uint32_t)a.nh;
    const int n_pos = a.n_pos0 + qi;
    // Split s takes the steps (4 U positions) s, s + n_splits, ...: at any time the launch reads one compact window of the
    // cache (n_splits x 4 U positions), not n_splits distant ranges.  (The softmax partials do not care which positions a
    // split holds.)
    const int p_end = n_pos;
    const uint32_t last = (uint32_t)n_pos - 1u;
    const size_t qrow = (size_t)qi * nh + h;
    // lane c of a head: bytes 16 c .. of a K row (half of block c / 2), rope values 4 c .. and 32 + 4 c .., V dims 16 c ..
    mk_i4 qk;
    float qsc;
    if (a.qq) {  // quantized by the launch before this one (the Hadamard option rotates the query first)
        qk = mk_ldg128(a.qq + qrow * NOPE + c * 16);
        qsc = a.qs[qrow * (NOPE / 32) + (c >> 1)] * a.had_k;
    } else {  // quantize_q8 of the query's latent part here (src/model.rs:1812-1821): lanes c and c ^ 1 share a block
        const mk_f4 *src = reinterpret_cast<const mk_f4 *>(a.q + qrow * (NOPE + ROPE) + c * 16);
        mk_f4 v[4];
        float mx = 0.0f;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            v[k] = src[k];
            mx = fmaxf(mx, fmaxf(fmaxf(fabsf(v[k].x), fabsf(v[k].y)), fmaxf(fabsf(v[k].z), fabsf(v[k].w))));
        }
        mx = fmaxf(mx, mk_dpp<0xB1>(mx));
        const float dx = mx / 127.0f;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            uint32_t w = 0;
            if (dx != 0.0f) {
                float qf[4];
                mk_q8_round4(v[k], dx, qf);
                w = ((uint32_t)(int)qf[0] & 255u) | (((uint32_t)(int)qf[1] & 255u) << 8) | (((uint32_t)(int)qf[2] & 255u) << 16) |
                    ((uint32_t)(int)qf[3] << 24);
            }
            qk[k] = (int)w;
        }
        qsc = dx;
    }
    const mk_f4 qr0 = *reinterpret_cast<const mk_f4 *>(a.q + qrow * (NOPE + ROPE) + NOPE + c * 4);
    const mk_f4 qr1 = *reinterpret_cast<const mk_f4 *>(a.q + qrow * (NOPE + ROPE) + NOPE + 32 + c * 4);
    float o[16];
#pragma unroll
    for (int e = 0; e < 16; e++) o[e] = 0.0f;
    float m = -INFINITY, l = 0.0f;
    // byte offsets are 32-bit (the host checks positions * heads * 128 < 2^32); a position past the end re-reads the last one
    auto load_step = [&](G8Pos *t, int t0) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const uint32_t j = min((uint32_t)(t0 + 4 * u), last);
            const uint32_t row = j * nh + (uint32_t)h;
            t[u].k = mk_ldg128_off_nt(a.kq, row * NOPE + c * 16);  // streamed once: non-temporal
            t[u].ks = mk_ldg_f32_off(a.ks, (row * (NOPE / 32) + (c >> 1)) * 4);
            t[u].r0 = __builtin_bit_cast(mk_f4, mk_ldg128_off(a.kr, (j * ROPE + c * 4) * 4));
            t[u].r1 = __builtin_bit_cast(mk_f4, mk_ldg128_off(a.kr, (j * ROPE + 32 + c * 4) * 4));
            t[u].v = mk_ldg128_off_nt(a.vq, row * VD + c * 16);
            t[u].vs = mk_ldg_f32_off(a.vs, (row * (VD / 32) + (c >> 1)) * 4);
        }
    };
    const int stride = 4 * U * a.n_splits;
    G8Pos t[U], nx[U];
    load_step(t, split * 4 * U + wave);
    for (int t0 = split * 4 * U + wave; t0 < p_end; t0 += stride) {
        load_step(nx, t0 + stride);  // the next step's values are requested before this step is worked on
        // ---- scores (src/model.rs:1833-1851): integer block dot, the block's scale product, the f32 rope part
        float s[U];
        float m_new = m;
#pragma unroll
        for (int u = 0; u < U; u++) {
            int idot = 0;
#pragma unroll
            for (int e = 0; e < 4; e++) idot = __builtin_amdgcn_sdot4(t[u].k[e], qk[e], idot, false);
            idot += __builtin_amdgcn_update_dpp(0, idot, 0xB1, 0xF, 0xF, true);  // the other half of the block (lane ^ 1)
            float x = (c & 1) ? 0.0f : (qsc * t[u].ks) * (float)idot;
            x += qr0.x * t[u].r0.x + qr0.y * t[u].r0.y + qr0.z * t[u].r0.z + qr0.w * t[u].r0.w;
            x += qr1.x * t[u].r1.x + qr1.y * t[u].r1.y + qr1.z * t[u].r1.z + qr1.w * t[u].r1.w;
            x += mk_dpp<0xB1>(x);
            x += mk_dpp<0x4E>(x);
            x += mk_dpp<0x141>(x);
            s[u] = (t0 + 4 * u < p_end) ? x * a.scale : -INFINITY;
            m_new = fmaxf(m_new, s[u]);
        }
        // ---- online softmax of this wave's positions (the first position of the step is inside the split: m_new is finite)
        const float corr = expf(m - m_new);
        l *= corr;
#pragma unroll
        for (int e = 0; e < 16; e++) o[e] *= corr;
        m = m_new;
#pragma unroll
        for (int u = 0; u < U; u++) {
            const float p = expf(s[u] - m_new);  // a position past the end has score -inf: 0
            l += p;
            const float ps = p * t[u].vs;
#pragma unroll
            for (int d = 0; d < 4; d++) {
                const int w = t[u].v[d];
                o[4 * d + 0] += ps * (float)(int8_t)w;
                o[4 * d + 1] += ps * (float)(int8_t)(w >> 8);
                o[4 * d + 2] += ps * (float)(int8_t)(w >> 16);
                o[4 * d + 3] += ps * (float)(w >> 24);
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) t[u] = nx[u];
    }
    // ---- the four waves' states of a head meet (a wave without a position has m = -inf, l = 0, o = 0: weight 0)
#pragma unroll
    for (int e = 0; e < 16; e++) o_l[wave][hl][c * 16 + e] = o[e];
    if (c == 0) {
        m_l[wave][hl] = m;
        l_l[wave][hl] = l;
    }
    __syncthreads();
    for (int idx = tid; idx < 8 * VD; idx += 256) {
        const int hh = idx / VD, d = idx - hh * VD;
        const float ms = fmaxf(fmaxf(m_l[0][hh], m_l[1][hh]), fmaxf(m_l[2][hh], m_l[3][hh]));
        float num = 0.0f, den = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const float wt = expf(m_l[w][hh] - ms);
            num += wt * o_l[w][hh][d];
            den += wt * l_l[w][hh];
        }
        const size_t hrow = (size_t)hg * 8 + hh;
        if (hrow >= nh) continue;
        if (a.n_splits == 1) {
            a.out[((size_t)qi * nh + hrow) * VD + d] = num / den;
        } else {
            a.po[((size_t)split * nh + hrow) * VD + d] = num;
            if (d == 0) {
                a.pm[split * nh + hrow] = ms;
                a.pl[split * nh + hrow] = den;
            }
        }
    }
}

// The attention loop of mla_prefill (src/model.rs:2080-2102) for the same head shape: 16 queries of one head share every
// K / V tile on the matrix cores -- a wave per (head, 16 queries), tiles of 16 positions -- instead of one pass over the
// cache per query.  The arithmetic keeps the reference's terms: integer block dots (v_mfma_i32_16x16x64_i8, issued once
// with the second block's query bytes zeroed and once whole: the second block's dot is the difference), the per-block
// scale product in f32, the f32 rope dot and P V on the f32 matrix instruction (v_mfma_f32_16x16x4_f32: f32 products,
// f32 sums; V = scale * byte is formed exactly as the decode kernel forms it).  Only the order of the sums differs.
// Operands (lane = j + 16 g): the scores are computed transposed, positions as rows and queries as columns, so that the
// probabilities a lane holds -- query j, positions 4 g + r -- are already the B operand of P V (k = g at step r); the A
// operand of P V is V transposed with output row i of tile t standing for dim 8 i + t, so a lane reads 8 consecutive V
// bytes per position and ends with 8 consecutive output values per accumulator row.
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(3))) void heads_prefill_mfma_kernel(HeadsArgs a, int m) {
    constexpr int NOPE = 128, ROPE = 64, VD = 128;
    const int lane = threadIdx.x, j = lane & 15, g = lane >> 4;
    const int qg = (int)gridDim.x - 1 - (int)blockIdx.x;  // the groups with the longest contexts start first
    const int h = blockIdx.y;
    const uint32_t nh = (uint32_t)a.nh;
    const int qi = min(qg * 16 + j, m - 1);            // this lane's query (a column of the score tile)
    const size_t qrow = (size_t)qi * nh + h;
    const int lim = a.n_pos0 - 1 + qi;                 // its last position
    const int t_end = a.n_pos0 + min(qg * 16 + 15, m - 1);  // positions the group's last query sees
    const uint32_t last = (uint32_t)(a.n_pos0 + m - 2);      // last cached position the call may read
    // query side
    mk_i4 bq[2], bq0[2];
    float qsv[4], qr[16];
#pragma unroll
    for (int s2 = 0; s2 < 2; s2++) {
        bq[s2] = mk_ldg128(a.qq + qrow * NOPE + 64 * s2 + 16 * g);
        bq0[s2] = g < 2 ? bq[s2] : mk_i4{0, 0, 0, 0};
    }
    {
        const mk_f4 v = *reinterpret_cast<const mk_f4 *>(a.qs + qrow * (NOPE / 32));
        qsv[0] = v.x * a.had_k, qsv[1] = v.y * a.had_k, qsv[2] = v.z * a.had_k, qsv[3] = v.w * a.had_k;
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const mk_f4 v = *reinterpret_cast<const mk_f4 *>(a.q + qrow * (NOPE + ROPE) + NOPE + 16 * g + 4 * i);
        qr[4 * i] = v.x, qr[4 * i + 1] = v.y, qr[4 * i + 2] = v.z, qr[4 * i + 3] = v.w;
    }
    mk_f4 o[8];
#pragma unroll
    for (int t = 0; t < 8; t++) o[t] = mk_f4{0.0f, 0.0f, 0.0f, 0.0f};
    float mrun = -INFINITY, lrun = 0.0f;
    const mk_i4 zero4 = {0, 0, 0, 0};
    // a tile's values as this lane needs them: as row j of the tile (position t0 + j) and as the rows 4 g + r of the results
    struct Tile {
        mk_i4 ak[2];
        mk_f4 ar[4];
        mk_f4 ksv[4];
        mk_u2 vb[4];
        float vsv[4];
    };
    auto load_tile = [&](Tile &T, int t0) {
        const uint32_t pa = min((uint32_t)(t0 + j), last);
        const uint32_t rowa = pa * nh + (uint32_t)h;
#pragma unroll
        for (int s2 = 0; s2 < 2; s2++) T.ak[s2] = mk_ldg128_off(a.kq, rowa * NOPE + 64 * s2 + 16 * g);
#pragma unroll
        for (int i = 0; i < 4; i++) T.ar[i] = __builtin_bit_cast(mk_f4, mk_ldg128_off(a.kr, (pa * ROPE + 16 * g + 4 * i) * 4));
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const uint32_t pr = min((uint32_t)(t0 + 4 * g + r), last);
            const uint32_t rowr = pr * nh + (uint32_t)h;
            T.ksv[r] = __builtin_bit_cast(mk_f4, mk_ldg128_off(a.ks, rowr * (NOPE / 32) * 4));
            T.vb[r] = mk_ldg64(reinterpret_cast<const uint8_t *>(a.vq) + (size_t)rowr * VD + 8 * j);
            T.vsv[r] = mk_ldg_f32_off(a.vs, (rowr * (VD / 32) + (j >> 2)) * 4);
        }
    };
    // (requesting the next tile a tile ahead was measured: the same time with 50 more registers -- the kernel is bound by
    // the issue of its matrix and vector instructions, 41 % and 48 % of the cycles, not by the loads)
    for (int t0 = 0; t0 < t_end; t0 += 16) {
        Tile cur;
        load_tile(cur, t0);
        const mk_i4 *ak = cur.ak;
        const mk_f4 *ar = cur.ar, *ksv = cur.ksv;
        const mk_u2 *vb = cur.vb;
        const float *vsv = cur.vsv;
        // ---- scores, transposed: rows = positions, columns = queries
        mk_f4 sc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int s2 = 0; s2 < 2; s2++) {
            const mk_i4 c0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(ak[s2], bq0[s2], zero4, 0, 0, 0);
            const mk_i4 cf = __builtin_amdgcn_mfma_i32_16x16x64_i8(ak[s2], bq[s2], zero4, 0, 0, 0);
            sc.x = fmaf(qsv[2 * s2 + 1] * ksv[0][2 * s2 + 1], (float)(cf[0] - c0[0]), fmaf(qsv[2 * s2] * ksv[0][2 * s2], (float)c0[0], sc.x));
            sc.y = fmaf(qsv[2 * s2 + 1] * ksv[1][2 * s2 + 1], (float)(cf[1] - c0[1]), fmaf(qsv[2 * s2] * ksv[1][2 * s2], (float)c0[1], sc.y));
            sc.z = fmaf(qsv[2 * s2 + 1] * ksv[2][2 * s2 + 1], (float)(cf[2] - c0[2]), fmaf(qsv[2 * s2] * ksv[2][2 * s2], (float)c0[2], sc.z));
            sc.w = fmaf(qsv[2 * s2 + 1] * ksv[3][2 * s2 + 1], (float)(cf[3] - c0[3]), fmaf(qsv[2 * s2] * ksv[3][2 * s2], (float)c0[3], sc.w));
        }
        // (four chains of four dependent matrix instructions, not one of sixteen)
        mk_f4 c4[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            c4[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(ar[i].x, qr[4 * i], mk_f4{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
            c4[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(ar[i].y, qr[4 * i + 1], c4[i], 0, 0, 0);
            c4[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(ar[i].z, qr[4 * i + 2], c4[i], 0, 0, 0);
            c4[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(ar[i].w, qr[4 * i + 3], c4[i], 0, 0, 0);
        }
        const mk_f4 cr = (c4[0] + c4[1]) + (c4[2] + c4[3]);
        float sv[4];
        sv[0] = (t0 + 4 * g + 0) <= lim ? (sc.x + cr.x) * a.scale : -INFINITY;
        sv[1] = (t0 + 4 * g + 1) <= lim ? (sc.y + cr.y) * a.scale : -INFINITY;
        sv[2] = (t0 + 4 * g + 2) <= lim ? (sc.z + cr.z) * a.scale : -INFINITY;
        sv[3] = (t0 + 4 * g + 3) <= lim ? (sc.w + cr.w) * a.scale : -INFINITY;
        // ---- online softmax of query j: its 16 scores of the tile sit in the lanes j, j + 16, j + 32, j + 48
        // (position 0 is inside every query's range, so the running maximum is finite from the first tile on)
        const float tm = mk_rows_max(fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3])));
        const float m_new = fmaxf(mrun, tm);
        const float corr = expf(mrun - m_new);
        float p[4];
#pragma unroll
        for (int r = 0; r < 4; r++) p[r] = expf(sv[r] - m_new);  // a position past the query's range: 0
        lrun = lrun * corr + mk_rows_sum((p[0] + p[1]) + (p[2] + p[3]));
        mrun = m_new;
        if (__builtin_amdgcn_ballot_w64(corr != 1.0f)) {  // (after the first tiles a new maximum is rare)
#pragma unroll
            for (int t = 0; t < 8; t++) o[t] *= corr;
        }
        // ---- out^T += V^T P^T: step r takes the positions t0 + 4 g + r (k = g)
#pragma unroll
        for (int r = 0; r < 4; r++) {
#pragma unroll
            for (int t = 0; t < 8; t++) {
                const int byte = (int)(int8_t)((t < 4 ? vb[r][0] : vb[r][1]) >> (8 * (t & 3)));
                o[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(vsv[r] * (float)byte, p[r], o[t], 0, 0, 0);
            }
        }
    }
    // accumulator row i = 4 g + r of tile t is dim 8 i + t of query j
    if (qg * 16 + j < m) {
        const float inv = 1.0f / lrun;
        float *dst = a.out + qrow * VD;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int d0 = 8 * (4 * g + r);
            *reinterpret_cast<mk_f4 *>(dst + d0) = mk_f4{o[0][r] * inv, o[1][r] * inv, o[2][r] * inv, o[3][r] * inv};
            *reinterpret_cast<mk_f4 *>(dst + d0 + 4) = mk_f4{o[4][r] * inv, o[5][r] * inv, o[6][r] * inv, o[7][r] * inv};
        }
    }
}

// log-sum-exp merge of the splits of one query: a workgroup per head
// GROUPS: thread groups that share out the splits of a dim; a workgroup takes 256 / GROUPS consecutive dims of a row
// (blockIdx.y-th such chunk).  GROUPS = 0: the group count follows vd (256 / vd for vd <= 128, else a plain loop).
template <int GROUPS>
__global__ __launch_bounds__(256) void heads_merge_kernel(const float *__restrict__ po, const float *__restrict__ pm, const float *__restrict__ pl,
                                                          int nh, int vd, int n_splits, float *__restrict__ out) {
    __shared__ float w_l[MAX_SPLITS];
    __shared__ float den_l;
    __shared__ float part_l[256];
    const int h = blockIdx.x, tid = threadIdx.x;
    // The partials come from other compute dies: every dependent round of loads costs a trip to memory.  Narrow rows
    // (vd <= 128) take ONE round: the splits are shared out over 256 / vd groups of threads and a thread requests all
    // its partial values before the weights exist (a split past the end re-reads the last one with weight 0).
    const int groups = GROUPS ? GROUPS : (vd <= 128 ? 256 / vd : 1);
    constexpr int PER = MAX_SPLITS / (GROUPS ? GROUPS : 2);
    const int vdc = GROUPS ? 256 / GROUPS : vd, d0 = GROUPS ? (int)blockIdx.y * vdc : 0;  // this workgroup's dims d0 .. d0 + vdc - 1
    const int sg = tid / vdc, d = d0 + tid - sg * vdc;
    float pv[PER];
    if (groups > 1 && sg < groups) {
#pragma unroll
        for (int i = 0; i < PER; i++) {
            const int s = min(sg + groups * i, n_splits - 1);
            pv[i] = po[((size_t)s * nh + h) * vd + d];
        }
    }
    if (tid < 64) {
        static_assert(MAX_SPLITS <= 64, "one lane per split");
        const float ms = tid < n_splits ? pm[tid * nh + h] : -INFINITY;
        const float ls = tid < n_splits ? pl[tid * nh + h] : 0.0f;
        const float mx = mk_wave_max(ms);
        const float w = expf(ms - mx);  // (a lane past the last split: 0)
        w_l[tid] = w;
        const float den = mk_wave_sum(ls * w);
        if (tid == 0) den_l = den;
    }
    __syncthreads();
    if (groups > 1) {
        float num = 0.0f;
        if (sg < groups) {
#pragma unroll
            for (int i = 0; i < PER; i++) {
                const int s = sg + groups * i;
                num += pv[i] * (s < n_splits ? w_l[s] : 0.0f);
            }
            part_l[tid] = num;
        }
        __syncthreads();
        if (tid < vdc) {
            for (int g = 1; g < groups; g++) num += part_l[g * vdc + tid];
            out[(size_t)h * vd + d0 + tid] = num / den_l;
        }
        return;
    }
    for (int dd = tid; dd < vd; dd += 256) {
        float num = 0.0f;
        for (int s = 0; s < n_splits; s++) num += po[((size_t)s * nh + h) * vd + dd] * w_l[s];
        out[(size_t)h * vd + dd] = num / den_l;
    }
}

int check_shape(size_t nh, size_t nope, size_t rope, size_t vd) {
    MK_REQUIRE(nh >= 1 && nh <= 65535, "bad head count");
    MK_REQUIRE(nope % 32 == 0 && nope >= 32 && nope <= 32 * MAX_NB, "latent K width must be a multiple of 32 up to 256");
    MK_REQUIRE(vd % 32 == 0 && vd >= 32 && vd <= MAX_VD, "V width must be a multiple of 32 up to 512");
    MK_REQUIRE(rope <= 4096, "rope width out of range");
    return MK_OK;
}

}  // namespace

// the option applies only when both widths are whole 64-chunks (src/model.rs:1590, 1631, 1811)
static int had_applies(int hadamard, size_t nope, size_t vd) { return hadamard && nope % 64 == 0 && vd % 64 == 0; }

extern "C" int mk_dev_mla_heads_append(const float *k_rows, const float *v_rows, size_t n_new, size_t nh, size_t nope, size_t rope, size_t vd,
                                       size_t pos0, int hadamard, int8_t *kq, float *ks, float *kr, int8_t *vq, float *vs, void *stream) {
    MK_REQUIRE(k_rows && v_rows && kq && ks && vq && vs && (kr || rope == 0), "null pointer");
    int s = check_shape(nh, nope, rope, vd);
    if (s != MK_OK) return s;
    if (n_new == 0) return MK_OK;
    MK_REQUIRE(n_new <= 65535, "at most 65535 positions per call");
    const size_t blocks32 = nh * nope / 32 + nh * vd / 32 + (rope + 31) / 32;
    hipLaunchKernelGGL(heads_append_kernel, dim3((unsigned)((blocks32 + 7) / 8), (unsigned)n_new), dim3(256), 0, (hipStream_t)stream, k_rows, v_rows,
                       (int)nh, (int)nope, (int)rope, (int)vd, pos0, had_applies(hadamard, nope, vd), kq, ks, kr, vq, vs);
    return mk_launch_status("heads_append");
}

extern "C" int mk_dev_mla_heads_to_f32(const int8_t *kq, const float *ks, const float *kr, const int8_t *vq, const float *vs, size_t n,
                                       size_t nh, size_t nope, size_t rope, size_t vd, int hadamard, float *k, float *v, void *stream) {
    MK_REQUIRE(kq && ks && vq && vs && k && v && (kr || rope == 0), "null pointer");
    int s = check_shape(nh, nope, rope, vd);
    if (s != MK_OK) return s;
    if (n == 0) return MK_OK;
    MK_REQUIRE(n <= 65535 * 64, "too many positions");
    for (size_t j0 = 0; j0 < n; j0 += 65535) {
        const size_t nj = n - j0 < 65535 ? n - j0 : 65535;
        if (had_applies(hadamard, nope, vd))
            hipLaunchKernelGGL(heads_to_f32_had_kernel, dim3(8, (unsigned)nj), dim3(256), 0, (hipStream_t)stream, kq + j0 * nh * nope,
                               ks + j0 * nh * (nope / 32), kr + j0 * rope, vq + j0 * nh * vd, vs + j0 * nh * (vd / 32), (int)nh, (int)nope,
                               (int)rope, (int)vd, k + j0 * nh * (nope + rope), v + j0 * nh * vd);
        else
            hipLaunchKernelGGL(heads_to_f32_kernel, dim3(8, (unsigned)nj), dim3(256), 0, (hipStream_t)stream, kq + j0 * nh * nope,
                               ks + j0 * nh * (nope / 32), kr + j0 * rope, vq + j0 * nh * vd, vs + j0 * nh * (vd / 32), (int)nh, (int)nope,
                               (int)rope, (int)vd, k + j0 * nh * (nope + rope), v + j0 * nh * vd);
        if ((s = mk_launch_status("heads_to_f32")) != MK_OK) return s;
    }
    return MK_OK;
}

extern "C" size_t mk_mla_heads_workspace_bytes(size_t m, size_t nh, size_t nope, size_t vd) {
    return align_up(m * nh * nope, 256) + align_up(m * nh * (nope / 32) * 4, 256) + align_up(MAX_SPLITS * nh * vd * 4, 256) +
           2 * align_up(MAX_SPLITS * nh * 4, 256);
}

extern "C" int mk_dev_mla_heads_q8_attn(const int8_t *kq, const float *ks, const float *kr, const int8_t *vq, const float *vs, size_t pos0,
                                        const float *q, size_t m, size_t nh, size_t nope, size_t rope, size_t vd, float scale, int hadamard,
                                        void *workspace, float *out, void *stream) {
    MK_REQUIRE(kq && ks && vq && vs && q && workspace && out && (kr || rope == 0), "null pointer");
    int s = check_shape(nh, nope, rope, vd);
    if (s != MK_OK) return s;
    MK_REQUIRE(m >= 1 && m <= 65535, "bad query count");
    MK_REQUIRE(pos0 + m < 0x7FFFFF00u, "position out of range");
    MK_REQUIRE(((uintptr_t)kq & 15) == 0 && ((uintptr_t)vq & 3) == 0 && ((uintptr_t)workspace & 255) == 0,
               "K bytes must be 16-byte, V bytes 4-byte and the workspace 256-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    uint8_t *w = (uint8_t *)workspace;
    HeadsArgs a;
    a.kq = kq;
    a.ks = ks;
    a.kr = kr;
    a.vq = vq;
    a.vs = vs;
    a.q = q;
    int8_t *qq = (int8_t *)w;
    w += align_up(m * nh * nope, 256);
    float *qs = (float *)w;
    w += align_up(m * nh * (nope / 32) * 4, 256);
    a.po = (float *)w;
    w += align_up(MAX_SPLITS * nh * vd * 4, 256);
    a.pm = (float *)w;
    w += align_up(MAX_SPLITS * nh * 4, 256);
    a.pl = (float *)w;
    a.qq = qq;
    a.qs = qs;
    a.nh = (int)nh;
    a.nope = (int)nope;
    a.rope = (int)rope;
    a.vd = (int)vd;
    a.n_pos0 = (int)pos0 + 1;
    a.scale = scale;
    a.out = out;
    const int had = had_applies(hadamard, nope, vd);
    a.had_k = had ? 1.0f / 64.0f : 1.0f;
    // the reference's own head shape takes the all-heads kernel
    const bool g8 = nope == 128 && rope == 64 && vd == 128 && (pos0 + m) * nh * 128 < 0xFFFFFFFFull &&
                      (pos0 + m) * nh * rope * 4 < 0xFFFFFFFFull &&  // the kernel's 32-bit byte offsets: q8 rows and f32 rope rows
                      ((uintptr_t)vq & 15) == 0 && ((uintptr_t)kr & 15) == 0 && ((uintptr_t)q & 15) == 0 && !MK_TUNE("MK_MLA_HEADS_GENERIC", 0);
    const bool many = g8 && m >= (size_t)MK_TUNE("MK_MLA_HEADS_PREFILL_MIN", 16);
    if (g8 && !had && !many) {
        a.qq = nullptr;  // the all-heads kernel quantizes the query itself
    } else {
        const int rows = (int)(m * nh);
        if (!had && ((uintptr_t)q & 15) == 0 && (nope + rope) % 4 == 0) {
            const size_t n_blocks = (size_t)rows * (nope / 32);
            hipLaunchKernelGGL(heads_q_prep4_kernel, dim3((unsigned)((n_blocks * 8 + 255) / 256)), dim3(256), 0, st, q, n_blocks, (int)nope, (int)rope,
                               qq, qs);
        } else {
            hipLaunchKernelGGL(heads_q_prep_kernel, dim3((unsigned)((rows * (nope / 32) + 7) / 8)), dim3(256), 0, st, q, rows, (int)nope, (int)rope, had,
                               qq, qs);
        }
        if ((s = mk_launch_status("heads_q_prep")) != MK_OK) return s;
    }
    // one query: split the context so that about 1024 workgroups stream the cache; several queries (prefill): the
    // (query, head) grid is parallel enough, one split each
    const int hgroups = (int)((nh + 7) / 8);
    int n_splits = 1, split_len = (int)((pos0 + m + TJ - 1) / TJ) * TJ;
    if (m == 1) {
        const int tiles = (int)((pos0 + 1 + TJ - 1) / TJ);
        int want = (int)((1024 + nh - 1) / nh);
        if (want > MAX_SPLITS) want = MAX_SPLITS;
        if (want > tiles) want = tiles;
        const int tps = (tiles + want - 1) / want;
        split_len = tps * TJ;
        n_splits = (tiles + tps - 1) / tps;
        if (g8) {  // interleaved steps of 4 U positions: any count up to the number of steps
            const int steps = (int)((pos0 + 4 * G8_U) / (4 * G8_U));
            n_splits = (int)((MK_TUNE("MK_MLA_HEADS_WGS", 768) + hgroups - 1) / hgroups);
            if (n_splits > MAX_SPLITS) n_splits = MAX_SPLITS;
            if (n_splits > steps) n_splits = steps;
        }
    }
    a.split_len = split_len;
    a.n_splits = n_splits;
    if (g8 && m >= (size_t)MK_TUNE("MK_MLA_HEADS_PREFILL_MIN", 16) && ((uintptr_t)out & 15) == 0 && ((uintptr_t)ks & 15) == 0 &&
        ((uintptr_t)vq & 7) == 0) {
        // several queries: 16 of them share every K / V tile on the matrix cores
        hipLaunchKernelGGL(heads_prefill_mfma_kernel, dim3((unsigned)((m + 15) / 16), (unsigned)nh), dim3(64), 0, st, a, (int)m);
    } else if (g8) {
        hipLaunchKernelGGL(heads_decode_g8_kernel, dim3((unsigned)(n_splits * hgroups), (unsigned)m), dim3(256), 0, st, a);
    } else {
        hipLaunchKernelGGL(heads_decode_kernel, dim3((unsigned)n_splits, (unsigned)nh, (unsigned)m), dim3(256), 0, st, a);
    }
    if ((s = mk_launch_status("heads_decode")) != MK_OK) return s;
    if (n_splits > 1) {
        if (vd % 64 == 0 && vd <= 512 && n_splits > 16 && MK_TUNE("MK_MLA_HEADS_MERGE4", 1))  // 64 dims a workgroup, four split groups
            hipLaunchKernelGGL(heads_merge_kernel<4>, dim3((unsigned)nh, (unsigned)(vd / 64)), dim3(256), 0, st, a.po, a.pm, a.pl, (int)nh, (int)vd, n_splits, out);
        else
            hipLaunchKernelGGL(heads_merge_kernel<0>, dim3((unsigned)nh), dim3(256), 0, st, a.po, a.pm, a.pl, (int)nh, (int)vd, n_splits, out);
        if ((s = mk_launch_status("heads_merge")) != MK_OK) return s;
    }
    if (had) {
        const size_t chunks = m * nh * vd / 64;
        hipLaunchKernelGGL(heads_out_had_kernel, dim3((unsigned)((chunks + 3) / 4)), dim3(256), 0, st, out, chunks);
        return mk_launch_status("heads_out_had");
    }
    return MK_OK;
}
