// q8_0 MLA decode attention over the shared-latent cache: the all-heads kernel
// mla_attn_flash_q8_mqa (src/model.rs:1804-1908) in the weight-absorbed form,
// split over the context (split-KV) so the whole chip works on one token.
//
//   prep     q8-quantize the latent part of every head's query (src/model.rs:1812-1821)
//   partial  grid (split, head group): a workgroup stages 64-position tiles of
//            the cache in LDS once and serves 16 heads from them.  Per tile and
//            head, exactly the reference's tile body: integer latent dot with the
//            per-block scale product, f32 rope dot, running max / normaliser,
//            V rows (= the latent rows) dequantized as q * s and accumulated.
//   merge    log-sum-exp merge of the splits' (m, l, acc).
//
// Differences from the reference's order of operations: sums over blocks / rope
// dims / positions are tree-shaped across lanes, and the splits are merged at
// the end instead of one running rescale -- the same reassociation the
// reference accepts between its flash and materialised kernels
// (src/selftest.rs:648-704, 1e-5).
#include <stdlib.h>

#include <mutex>

#include "mk_common.h"

namespace {

constexpr int TJ = 64;    // positions per tile (FLASH_KV, src/model.rs:1348)
constexpr int HPW = 4;    // heads per wave
constexpr int HPG = 16;   // heads per workgroup (4 waves)
constexpr int MAX_SPLITS = 64;

__global__ __launch_bounds__(256) void mla_q_prep_kernel(const float *__restrict__ q, int nh, int L, int R, int8_t *__restrict__ qq,
                                                         float *__restrict__ qs) {
    const int nb = L / 32;
    const int blk = (blockIdx.x * blockDim.x + threadIdx.x) >> 5;  // (head, block)
    const int j = threadIdx.x & 31;
    if (blk >= nh * nb) return;
    const int h = blk / nb, g = blk % nb;
    float v = q[(size_t)h * (L + R) + g * 32 + j];
    float mx = mk_half_wave_max(fabsf(v));
    float dx = mx / 127.0f;
    int qi = dx != 0.0f ? mk_q8_round(v, dx) : 0;
    qq[(size_t)h * L + g * 32 + j] = (int8_t)qi;
    if (j == 0) qs[blk] = dx;
}

struct MlaArgs {
    const int8_t *lat_q;
    const uint16_t *lat_s;
    const int8_t *rope_q;
    const uint16_t *rope_s;
    const float *q;    // [nh][L+R]
    const int8_t *qq;  // [nh][L]
    const float *qs;   // [nh][L/32]
    int nh, L, R, n_pos, split_len, n_splits;
    float scale;
    float *po;  // [n_splits][nh][L]
    float *pm;  // [n_splits][nh]
    float *pl;  // [n_splits][nh]
};

__global__ __launch_bounds__(256) void mla_partial_kernel(MlaArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int L = a.L, R = a.R, nb = L / 32, nbr = R / 32;
    int8_t *kq_l = reinterpret_cast<int8_t *>(lds);                       // [TJ][L]
    float *ks_l = reinterpret_cast<float *>(lds + (size_t)TJ * L);       // [TJ][nb]
    float *kr_l = ks_l + TJ * nb;                                        // [TJ][R]
    float *sc_l = kr_l + TJ * R;                                         // [HPG][TJ]

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int split = blockIdx.x;
    const int h0 = blockIdx.y * HPG + wave * HPW;  // first head of this wave
    const int p_begin = split * a.split_len;
    const int p_end = min(p_begin + a.split_len, a.n_pos);  // exclusive

    // this lane's share of the wave's queries
    const int g = lane & 15, jl = lane >> 4;
    mk_i4 qreg[HPW][2];
    float qsc[HPW];
    float qrope[HPW][4];
#pragma unroll
    for (int hh = 0; hh < HPW; hh++) {
        const int h = min(h0 + hh, a.nh - 1);
        if (g < nb) {
            const mk_i4 *src = reinterpret_cast<const mk_i4 *>(a.qq + (size_t)h * L + g * 32);
            qreg[hh][0] = src[0];
            qreg[hh][1] = src[1];
            qsc[hh] = a.qs[h * nb + g];
        } else {
            qreg[hh][0] = qreg[hh][1] = mk_i4{0, 0, 0, 0};
            qsc[hh] = 0.0f;
        }
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int d = g + 16 * k;
            qrope[hh][k] = d < R ? a.q[(size_t)h * (L + R) + L + d] : 0.0f;
        }
    }
    const int dpl = L / 64;  // output dims per lane
    float o[HPW][8];
    float m[HPW], l[HPW];
#pragma unroll
    for (int hh = 0; hh < HPW; hh++) {
        m[hh] = -INFINITY;
        l[hh] = 0.0f;
#pragma unroll
        for (int k = 0; k < 8; k++) o[hh][k] = 0.0f;
    }

    for (int t0 = p_begin; t0 < p_end; t0 += TJ) {
        const int tn = min(TJ, p_end - t0);
        __syncthreads();  // previous tile fully consumed
        // stage the tile: latent bytes (16 B per thread per step), scales and rope rows as f32
        for (int i = threadIdx.x; i < tn * L / 16; i += 256)
            reinterpret_cast<mk_i4 *>(kq_l)[i] = reinterpret_cast<const mk_i4 *>(a.lat_q + (size_t)t0 * L)[i];
        for (int i = threadIdx.x; i < tn * nb; i += 256) ks_l[i] = mk_f16_bits_to_f32(a.lat_s[(size_t)t0 * nb + i]);
        for (int i = threadIdx.x; i < tn * R; i += 256) {
            const int j = i / R, d = i % R;
            // MlaCache::to_f32 dequantization q * s (src/model.rs:1641-1646)
            kr_l[i] = (float)a.rope_q[(size_t)(t0 + j) * R + d] * mk_f16_bits_to_f32(a.rope_s[(size_t)(t0 + j) * nbr + d / 32]);
        }
        __syncthreads();

        // scores: 4 positions per pass, 16 lanes per position (one latent block and up to 4 rope dims each)
        for (int pp = 0; pp < TJ / 4; pp++) {
            const int j = pp * 4 + jl;
            const bool live = j < tn;
            mk_i4 k0 = {0, 0, 0, 0}, k1 = {0, 0, 0, 0};
            float ksc = 0.0f;
            float kr[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            if (live) {
                if (g < nb) {
                    const mk_i4 *src = reinterpret_cast<const mk_i4 *>(kq_l + j * L + g * 32);
                    k0 = src[0];
                    k1 = src[1];
                    ksc = ks_l[j * nb + g];
                }
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const int d = g + 16 * k;
                    if (d < R) kr[k] = kr_l[j * R + d];
                }
            }
#pragma unroll
            for (int hh = 0; hh < HPW; hh++) {
                int idot = 0;
#pragma unroll
                for (int k = 0; k < 4; k++) idot = __builtin_amdgcn_sdot4(k0[k], qreg[hh][0][k], idot, false);
#pragma unroll
                for (int k = 0; k < 4; k++) idot = __builtin_amdgcn_sdot4(k1[k], qreg[hh][1][k], idot, false);
                float part = (qsc[hh] * ksc) * (float)idot;
#pragma unroll
                for (int k = 0; k < 4; k++) part += qrope[hh][k] * kr[k];
                part += __shfl_xor(part, 1, MK_WAVE);
                part += __shfl_xor(part, 2, MK_WAVE);
                part += __shfl_xor(part, 4, MK_WAVE);
                part += __shfl_xor(part, 8, MK_WAVE);
                if (g == 0) sc_l[(wave * HPW + hh) * TJ + j] = live ? part * a.scale : -INFINITY;
            }
        }
        __syncthreads();  // score rows complete (each row is written and read by one wave only)

        float corr[HPW];
#pragma unroll
        for (int hh = 0; hh < HPW; hh++) {
            float *row = sc_l + (wave * HPW + hh) * TJ;
            float s = row[lane];
            float tm = mk_wave_max(s);
            float m_new = fmaxf(m[hh], tm);
            corr[hh] = expf(m[hh] - m_new);
            float p = expf(s - m_new);  // -inf score (position past the end) gives 0
            float tile_l = mk_wave_sum(p);
            l[hh] = l[hh] * corr[hh] + tile_l;
            m[hh] = m_new;
            row[lane] = p;
        }
        __syncthreads();  // probabilities in place

#pragma unroll
        for (int hh = 0; hh < HPW; hh++)
#pragma unroll
            for (int k = 0; k < 8; k++) o[hh][k] *= corr[hh];
        const int d0 = lane * dpl;
        for (int j = 0; j < tn; j++) {
            const float sc = ks_l[j * nb + d0 / 32];
            float v[8];
#pragma unroll
            for (int k = 0; k < 8; k++) v[k] = k < dpl ? (float)kq_l[j * L + d0 + k] * sc : 0.0f;
#pragma unroll
            for (int hh = 0; hh < HPW; hh++) {
                const float p = sc_l[(wave * HPW + hh) * TJ + j];
#pragma unroll
                for (int k = 0; k < 8; k++) o[hh][k] += p * v[k];
            }
        }
    }
#pragma unroll
    for (int hh = 0; hh < HPW; hh++) {
        const int h = h0 + hh;
        if (h < a.nh) {
            float *dst = a.po + ((size_t)split * a.nh + h) * L + lane * dpl;
#pragma unroll
            for (int k = 0; k < 8; k++)
                if (k < dpl) dst[k] = o[hh][k];
            if (lane == 0) {
                a.pm[split * a.nh + h] = m[hh];
                a.pl[split * a.nh + h] = l[hh];
            }
        }
    }
}

// ---------------------------------------------------------------- MFMA kernel
// Latent 512 + rope 64 (the shape of the production models).  A workgroup serves
// 16 heads over one split of the context; its 4 waves share each 64-position
// tile in LDS and take 16 positions each, every wave with its own running
// (max, normaliser, output) that are merged through LDS at the end -- so a
// split costs one partial result per 16 heads, not one per wave.  Per tile and
// wave:
//
//   scores^T [pos][head]  latent part: v_mfma_i32_16x16x64_i8, cache bytes as the
//            A operand (lane l: row l%16, bytes 16*(l/16).. of the 64-byte step),
//            q8 query as B.  One instruction spans two scale blocks: it is
//            issued once with the query masked to the first block and once
//            whole, the second block's dot is the difference.  The integer block
//            dots are scaled by (query block scale * cache block scale) in f32,
//            the reference's per-block term (src/model.rs:1858-1871).  Rope part:
//            f16 MFMA in split precision (see "out"): the rope bytes times
//            their scale as exact f16 pairs, the f32 query as hi + lo.
//   softmax  a lane holds head l%16 and positions 4*(l/16)+r, which is the A
//            operand layout of the next product: probabilities stay in registers.
//   out      v_mfma_f32_16x16x32_f16 in split precision.  The cache value
//            v = q * s (int8 times f16 scale, src/model.rs:1641-1646) is formed
//            as an exact f16 pair: hi = rn(q*s), lo = fma(q, s, -hi) (the product
//            has 19 significant bits and the residual is a multiple of the
//            scale's ulp, so hi + lo == v).  The probability is split the same
//            way (hi = rn(p), lo = rn(p - hi), relative error below 2^-21).  K = 32
//            holds the 16 positions twice: (p_hi | p_hi) and (p_lo | 0) against
//            (v_hi | v_lo); accumulation is f32.  A lane reads 4 rows x
//            16 dims and transposes 4x4 byte blocks in registers, because the
//            operand wants positions contiguous in a lane and the cache has dims
//            contiguous.  Lane l keeps dims 16c..16c+15 and 256+16c.. (c = l%16)
//            of heads 4*(l/16)+r.
//
// The query's latent part is quantized in the prologue, in registers
// (src/model.rs:1812-1821).  The next tile is fetched into registers while the
// current one is computed and written to the other LDS buffer afterwards (one
// barrier per tile).  With a single split the workgroup writes the normalised
// output itself.
constexpr int ML = 512, MR = 64;
constexpr float MLA_TAU = 8.0f;
constexpr int KROW = 592;      // LDS row stride in bytes: 16 rows at 16-byte granularity fall in distinct banks
constexpr int KS_STRIDE = 68;  // f32 scale row [block][position]
constexpr int KH_STRIDE = 72;  // f16 scale row [block][position]
constexpr int KS_OFF = TJ * KROW;
constexpr int KH_OFF = KS_OFF + 18 * KS_STRIDE * 4;
constexpr int MLA_TILE_BYTES = KH_OFF + 16 * KH_STRIDE * 2;
constexpr int MLA_Q_OFF = 2 * MLA_TILE_BYTES;              // the quantized query, exchanged between the waves in the prologue
constexpr int MLA_Q_BYTES = 8 * 64 * 16 + 8 * 64 * 8;
constexpr int MLA_O_OFF = 1024;                            // epilogue: after the waves' (m, l), four [16 heads][512] f32 outputs
constexpr int MLA_LDS_BYTES = MLA_O_OFF + 4 * 16 * ML * 4;
static_assert(MLA_Q_OFF + MLA_Q_BYTES <= MLA_LDS_BYTES, "LDS layout");

typedef _Float16 mk_h4 __attribute__((ext_vector_type(4)));
typedef _Float16 mk_h8 __attribute__((ext_vector_type(8)));

struct MlaStage {
    mk_i4 lat[8];
    mk_i4 rope;
    mk_u2 ls;
    uint32_t rs;
};

__device__ __forceinline__ float mk_byte_f32(int w, int k) { return (float)(int8_t)((uint32_t)w >> (8 * k)); }
__device__ __forceinline__ uint32_t mk_perm(uint32_t hi, uint32_t lo, uint32_t sel) { return __builtin_amdgcn_perm(hi, lo, sel); }

__global__ __launch_bounds__(256) void mla_mfma_kernel(MlaArgs a, float *__restrict__ out) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int q4 = lane >> 4, c = lane & 15;
    const int split = blockIdx.x;
    const int hbase = blockIdx.y * 16;
    const int p_begin = split * a.split_len;
    const int p_end = min(p_begin + a.split_len, a.n_pos);
    const int ntiles = (p_end - p_begin + TJ - 1) / TJ;
    const int last_pos = a.n_pos - 1;

    // byte offsets stay below 2^31: the host checks the position count
    auto stage_load = [&](MlaStage &st, int t0) {
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const uint32_t pr = (uint32_t)min(t0 + (tid >> 5) + 8 * k, last_pos);
            st.lat[k] = mk_ldg128(a.lat_q + (pr * ML + (tid & 31) * 16));
        }
        const uint32_t pr = (uint32_t)min(t0 + (tid >> 2), last_pos);
        st.rope = mk_ldg128(a.rope_q + (pr * MR + (tid & 3) * 16));
        st.ls = mk_ldg64(a.lat_s + (pr * (ML / 32) + 4 * (tid & 3)));
        const uint32_t pr2 = (uint32_t)min(t0 + (tid & 63), last_pos);
        st.rs = mk_ldg_u32(a.rope_s + pr2 * (MR / 32));
    };
    auto stage_store = [&](const MlaStage &st, uint8_t *buf) {
        float *ks = reinterpret_cast<float *>(buf + KS_OFF);
        uint16_t *kh = reinterpret_cast<uint16_t *>(buf + KH_OFF);
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const int i = tid + 256 * k;
            *reinterpret_cast<mk_i4 *>(buf + (i >> 5) * KROW + (i & 31) * 16) = st.lat[k];  // row (tid >> 5) + 8k
        }
        *reinterpret_cast<mk_i4 *>(buf + (tid >> 2) * KROW + ML + (tid & 3) * 16) = st.rope;
        const int pos = tid >> 2, g0 = 4 * (tid & 3);
        const uint16_t h0 = (uint16_t)(st.ls.x & 0xFFFFu), h1 = (uint16_t)(st.ls.x >> 16);
        const uint16_t h2 = (uint16_t)(st.ls.y & 0xFFFFu), h3 = (uint16_t)(st.ls.y >> 16);
        ks[(g0 + 0) * KS_STRIDE + pos] = mk_f16_bits_to_f32(h0);
        ks[(g0 + 1) * KS_STRIDE + pos] = mk_f16_bits_to_f32(h1);
        ks[(g0 + 2) * KS_STRIDE + pos] = mk_f16_bits_to_f32(h2);
        ks[(g0 + 3) * KS_STRIDE + pos] = mk_f16_bits_to_f32(h3);
        kh[(g0 + 0) * KH_STRIDE + pos] = h0;
        kh[(g0 + 1) * KH_STRIDE + pos] = h1;
        kh[(g0 + 2) * KH_STRIDE + pos] = h2;
        kh[(g0 + 3) * KH_STRIDE + pos] = h3;
        if (tid < 64) {
            ks[16 * KS_STRIDE + tid] = mk_f16_bits_to_f32((uint16_t)(st.rs & 0xFFFFu));
            ks[17 * KS_STRIDE + tid] = mk_f16_bits_to_f32((uint16_t)(st.rs >> 16));
        }
    };
    MlaStage st;
    stage_load(st, p_begin);

    // The query of head hbase + c.  Lane (c, q4) owns bytes 16*(4S+q4).. of each
    // 64-value step S, half of scale block 2S + q4/2; its partner for the block
    // maximum is lane ^ 16.  Each wave quantizes two of the eight steps and
    // passes them to the others through LDS.
    const int head = min(hbase + c, a.nh - 1);
    const float *qrow = a.q + (size_t)head * (ML + MR);
    mk_i4 *qb_l = reinterpret_cast<mk_i4 *>(lds + MLA_Q_OFF);            // [S][lane]
    mk_f2 *qs_l = reinterpret_cast<mk_f2 *>(lds + MLA_Q_OFF + 8 * 64 * 16);  // [S][lane]: scales of blocks 2S, 2S+1
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int S = 2 * wave + i;
        const mk_f4 *src = reinterpret_cast<const mk_f4 *>(qrow + (4 * S + q4) * 16);
        mk_f4 v[4];
        float mx = 0.0f;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            v[k] = src[k];
            mx = fmaxf(mx, fmaxf(fmaxf(fabsf(v[k].x), fabsf(v[k].y)), fmaxf(fabsf(v[k].z), fabsf(v[k].w))));
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, MK_WAVE));
        const float dx = mx / 127.0f;
        mk_i4 packed;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            uint32_t w = 0;
            if (dx != 0.0f) {
                float qf[4];
                mk_q8_round4(v[k], dx, qf);  // the same integers as mk_q8_round, a third of the instructions
                w = ((uint32_t)(int)qf[0] & 255u) | (((uint32_t)(int)qf[1] & 255u) << 8) | (((uint32_t)(int)qf[2] & 255u) << 16) |
                    ((uint32_t)(int)qf[3] << 24);
            }
            packed[k] = (int)w;
        }
        const float other = __shfl_xor(dx, 32, MK_WAVE);
        qb_l[S * 64 + lane] = packed;
        qs_l[S * 64 + lane] = q4 < 2 ? mk_f2{dx, other} : mk_f2{other, dx};
    }
    const int blk0_mask = q4 < 2 ? -1 : 0;
    // rope part of the query (f32 in the reference), dims 16*q4.. of head c, as an f16 pair hi + lo
    mk_h8 qrh[2], qrl[2];
#pragma unroll
    for (int k = 0; k < 16; k++) {
        const float v = qrow[ML + 16 * q4 + k];
        const _Float16 hi = (_Float16)v;
        qrh[k >> 3][k & 7] = hi;
        qrl[k >> 3][k & 7] = (_Float16)(v - (float)hi);
    }

    mk_f4 o[32];
#pragma unroll
    for (int n = 0; n < 32; n++) o[n] = mk_f4{0.0f, 0.0f, 0.0f, 0.0f};
    float m = -INFINITY, l = 0.0f;
    const mk_i4 zero4 = {0, 0, 0, 0};
    stage_store(st, lds);
    __syncthreads();

    auto compute_tile = [&](const uint8_t *buf, int t0) {
        const float *ks = reinterpret_cast<const float *>(buf + KS_OFF);
        // ---- scores of this wave's 16 positions
        const int prow = 16 * wave;
        const uint8_t *krow = buf + (prow + c) * KROW + q4 * 16;
        float sc[4];
        {
            // all integer block dots first (16 independent MFMAs), the rope product while
            // they drain, then the per-block scaling: no MFMA result is waited for early
            mk_i4 ka[8], c0[8], cf[8];
#pragma unroll
            for (int S = 0; S < 8; S++) ka[S] = *reinterpret_cast<const mk_i4 *>(krow + S * 64);
            const mk_i4 kr = *reinterpret_cast<const mk_i4 *>(buf + (prow + c) * KROW + ML + q4 * 16);
            const float rsc = ks[(16 + (q4 >> 1)) * KS_STRIDE + prow + c];
#pragma unroll
            for (int S = 0; S < 8; S++) {
                const mk_i4 qv = qb_l[S * 64 + lane];  // the query stays in LDS: registers are the scarce resource here
                const mk_i4 qm = {qv[0] & blk0_mask, qv[1] & blk0_mask, qv[2] & blk0_mask, qv[3] & blk0_mask};
                c0[S] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ka[S], qm, zero4, 0, 0, 0);
                cf[S] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ka[S], qv, zero4, 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            // rope: bytes -> exact f16 pairs (see the output product below), 64 dims = two K=32 steps
            mk_f4 cr0 = {0.0f, 0.0f, 0.0f, 0.0f}, cr1 = cr0;
            {
                const _Float16 rs = (_Float16)rsc;  // exact: the scale is stored as f16
                const mk_h2 s2 = {rs, rs};
                const mk_h2 bias = {(_Float16)1152.0f, (_Float16)1152.0f};
                mk_h8 kh8[2], kl8[2];
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const uint32_t d = (uint32_t)kr[k] ^ 0x80808080u;
                    const mk_h2 v0 = __builtin_bit_cast(mk_h2, mk_perm(0x64646464u, d, 0x04010400u)) - bias;
                    const mk_h2 v1 = __builtin_bit_cast(mk_h2, mk_perm(0x64646464u, d, 0x04030402u)) - bias;
                    const mk_h2 h0 = v0 * s2, h1 = v1 * s2;
                    const mk_h2 l0 = __builtin_elementwise_fma(v0, s2, -h0), l1 = __builtin_elementwise_fma(v1, s2, -h1);
                    kh8[k >> 1][4 * (k & 1) + 0] = h0.x;
                    kh8[k >> 1][4 * (k & 1) + 1] = h0.y;
                    kh8[k >> 1][4 * (k & 1) + 2] = h1.x;
                    kh8[k >> 1][4 * (k & 1) + 3] = h1.y;
                    kl8[k >> 1][4 * (k & 1) + 0] = l0.x;
                    kl8[k >> 1][4 * (k & 1) + 1] = l0.y;
                    kl8[k >> 1][4 * (k & 1) + 2] = l1.x;
                    kl8[k >> 1][4 * (k & 1) + 3] = l1.y;
                }
                cr0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kh8[0], qrh[0], cr0, 0, 0, 0);
                cr1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kh8[1], qrh[1], cr1, 0, 0, 0);
                cr0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kl8[0], qrh[0], cr0, 0, 0, 0);
                cr1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kl8[1], qrh[1], cr1, 0, 0, 0);
                cr0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kh8[0], qrl[0], cr0, 0, 0, 0);
                cr1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kh8[1], qrl[1], cr1, 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            mk_f4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int S = 0; S < 8; S++) {
                const mk_f2 qsc = qs_l[S * 64 + lane];
                const mk_f4 k0 = *reinterpret_cast<const mk_f4 *>(ks + (2 * S) * KS_STRIDE + prow + 4 * q4);
                const mk_f4 k1 = *reinterpret_cast<const mk_f4 *>(ks + (2 * S + 1) * KS_STRIDE + prow + 4 * q4);
#pragma unroll
                for (int r = 0; r < 4; r++) acc[r] += (qsc.x * k0[r]) * (float)c0[S][r] + (qsc.y * k1[r]) * (float)(cf[S][r] - c0[S][r]);
            }
#pragma unroll
            for (int r = 0; r < 4; r++) sc[r] = (t0 + prow + 4 * q4 + r) < p_end ? (acc[r] + (cr0[r] + cr1[r])) * a.scale : -INFINITY;
        }
        __builtin_amdgcn_sched_barrier(0);
        // ---- online softmax for head c over the 16 positions
        float tm = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
        tm = mk_rows_max(tm);
        // The reference point of the exponentials moves only when the maximum has
        // grown by more than MLA_TAU: weights stay below e^TAU and the 128
        // accumulators are rescaled a few times per split instead of every tile.
        const bool move = tm > m + MLA_TAU;  // false for a wave that still has no valid position (tm = -inf)
        const float m_new = move ? tm : m;
        const float m_ref = m_new == -INFINITY ? 0.0f : m_new;  // no position seen yet: all weights 0
        const float corr = move ? expf(m - m_ref) : 1.0f;
        float ts = 0.0f;
        mk_h8 pa1, pa2;  // (p_hi | p_hi) and (p_lo | 0) over this lane's 4 positions
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const float pv = expf(sc[r] - m_ref);
            ts += pv;
            const _Float16 hi = (_Float16)pv;
            pa1[r] = hi;
            pa1[4 + r] = hi;
            pa2[r] = (_Float16)(pv - (float)hi);
            pa2[4 + r] = (_Float16)0.0f;
        }
        ts = mk_rows_sum(ts);
        l = l * corr + ts;
        m = m_new;
        if (__any(move)) {
            // the accumulators hold heads 4*q4+r: fetch their corrections from the lanes that own those heads
            float oc[4];
#pragma unroll
            for (int r = 0; r < 4; r++) oc[r] = __shfl(corr, 4 * q4 + r, MK_WAVE);
            // The accumulators live in the MFMA accumulation registers.  The empty asm statements pin each
            // one there on entry and exit of this rare block, so the copies through the vector registers
            // that the multiplication needs stay inside it instead of being paid on every tile.
#pragma unroll
            for (int n = 0; n < 32; n++) {
                mk_f4 t = o[n];
                asm volatile("" : "+a"(t));
#pragma unroll
                for (int r = 0; r < 4; r++) t[r] *= oc[r];
                asm volatile("" : "+a"(t));
                o[n] = t;
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        // ---- out += P V over rows prow + 4*q4 + e
        const uint8_t *vbase = buf + (prow + 4 * q4) * KROW + 16 * c;
        const uint16_t *kh = reinterpret_cast<const uint16_t *>(buf + KH_OFF);
#pragma unroll
        for (int half = 0; half < 2; half++) {
            // scales of the 4 rows for this lane's block, as f16 pairs (rows 0,1) and (rows 2,3)
            const mk_u2 sraw = *reinterpret_cast<const mk_u2 *>(kh + (8 * half + (c >> 1)) * KH_STRIDE + prow + 4 * q4);
            const uint32_t sw0 = sraw[0], sw1 = sraw[1];  // scalars first: a bit cast straight from a vector element reads element 0
            const mk_h2 s01 = __builtin_bit_cast(mk_h2, sw0), s23 = __builtin_bit_cast(mk_h2, sw1);
            mk_i4 w[4];
#pragma unroll
            for (int e = 0; e < 4; e++) w[e] = *reinterpret_cast<const mk_i4 *>(vbase + e * KROW + 256 * half);
#pragma unroll
            for (int k = 0; k < 4; k++) {
                // 4 rows x 4 dims of bytes, sign bit flipped (b ^ 0x80 = b + 128 as unsigned), transposed
                const uint32_t d0 = (uint32_t)w[0][k] ^ 0x80808080u, d1 = (uint32_t)w[1][k] ^ 0x80808080u;
                const uint32_t d2 = (uint32_t)w[2][k] ^ 0x80808080u, d3 = (uint32_t)w[3][k] ^ 0x80808080u;
                const uint32_t t01l = mk_perm(d1, d0, 0x05010400u), t01h = mk_perm(d1, d0, 0x07030602u);  // (r0 r1) pairs of dims 0,1 / 2,3
                const uint32_t t23l = mk_perm(d3, d2, 0x05010400u), t23h = mk_perm(d3, d2, 0x07030602u);
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const uint32_t p01 = j < 2 ? t01l : t01h, p23 = j < 2 ? t23l : t23h;
                    // two bytes -> two f16: 0x6400 | u is 1024 + u exactly (the 0x64 bytes come out of the same v_perm);
                    // minus 1152 gives the signed byte
                    const uint32_t sel = (j & 1) ? 0x04030402u : 0x04010400u;
                    const uint32_t f01 = mk_perm(0x64646464u, p01, sel), f23 = mk_perm(0x64646464u, p23, sel);
                    const mk_h2 bias = {(_Float16)1152.0f, (_Float16)1152.0f};
                    const mk_h2 v01 = __builtin_bit_cast(mk_h2, f01) - bias, v23 = __builtin_bit_cast(mk_h2, f23) - bias;
                    const mk_h2 hi01 = v01 * s01, hi23 = v23 * s23;
                    const mk_h2 lo01 = __builtin_elementwise_fma(v01, s01, -hi01), lo23 = __builtin_elementwise_fma(v23, s23, -hi23);
                    const mk_h8 b = {hi01.x, hi01.y, hi23.x, hi23.y, lo01.x, lo01.y, lo23.x, lo23.y};  // (v_hi | v_lo)
                    const int n = 16 * half + 4 * k + j;
                    o[n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa1, b, o[n], 0, 0, 0);  // p_hi v_hi + p_hi v_lo
                    o[n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa2, b, o[n], 0, 0, 0);  // p_lo v_hi
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };

    for (int tile = 0; tile < ntiles; tile++) {
        const int t0 = p_begin + tile * TJ;
        stage_load(st, min(t0 + TJ, last_pos));  // next tile (clamped: the last iteration's fetch is not used)
        compute_tile(lds + (tile & 1) * MLA_TILE_BYTES, t0);
        stage_store(st, lds + ((tile + 1) & 1) * MLA_TILE_BYTES);
        __syncthreads();
    }

    // ---- merge the four waves (log-sum-exp), then store
    float *ml = reinterpret_cast<float *>(lds);              // [wave][head][m, l]
    float *ob = reinterpret_cast<float *>(lds + MLA_O_OFF);  // [wave][head][dim]
    if (q4 == 0) {
        ml[(wave * 16 + c) * 2] = m;
        ml[(wave * 16 + c) * 2 + 1] = l;
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const int h = 4 * q4 + r;
        float mm = -INFINITY;
#pragma unroll
        for (int w2 = 0; w2 < 4; w2++) mm = fmaxf(mm, ml[(w2 * 16 + h) * 2]);
        const float wself = expf(ml[(wave * 16 + h) * 2] - mm);
        float *dst = ob + ((size_t)(wave * 16 + h)) * ML + 16 * c;
#pragma unroll
        for (int half = 0; half < 2; half++)
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const mk_f4 v = {o[16 * half + 4 * k][r] * wself, o[16 * half + 4 * k + 1][r] * wself, o[16 * half + 4 * k + 2][r] * wself,
                                 o[16 * half + 4 * k + 3][r] * wself};
                // 16-byte chunks are swizzled within groups of four so that the 16 lanes of a row hit 16 bank groups
                *reinterpret_cast<mk_f4 *>(dst + 256 * half + 4 * (k ^ ((c >> 2) & 3))) = v;
            }
    }
    __syncthreads();
    {
        // thread: head tid/16, dims 4*(tid%16 + 16*i)
        const int hl = tid >> 4, h = hbase + hl;
        float mm = -INFINITY;
#pragma unroll
        for (int w2 = 0; w2 < 4; w2++) mm = fmaxf(mm, ml[(w2 * 16 + hl) * 2]);
        float lt = 0.0f;
#pragma unroll
        for (int w2 = 0; w2 < 4; w2++) lt += ml[(w2 * 16 + hl) * 2 + 1] * expf(ml[(w2 * 16 + hl) * 2] - mm);
        if (h < a.nh) {
            const bool single = a.n_splits == 1;
            float *dst = single ? out + (size_t)h * ML : a.po + ((size_t)split * a.nh + h) * ML;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int ch = (tid & 15) + 16 * i;  // logical chunk: dims 4*ch..; written by lane c = (ch >> 2) & 15
                const int d = 4 * ch, dp = 4 * (ch ^ ((ch >> 4) & 3));
                mk_f4 v = *reinterpret_cast<const mk_f4 *>(ob + (size_t)hl * ML + dp);
#pragma unroll
                for (int w2 = 1; w2 < 4; w2++) v += *reinterpret_cast<const mk_f4 *>(ob + (size_t)(w2 * 16 + hl) * ML + dp);
                if (single) v = mk_f4{v.x / lt, v.y / lt, v.z / lt, v.w / lt};
                *reinterpret_cast<mk_f4 *>(dst + d) = v;
            }
            if (!single && (tid & 15) == 0) {
                a.pm[split * a.nh + h] = mm;
                a.pl[split * a.nh + h] = lt;
            }
        }
    }
}

// log-sum-exp merge of the splits.  A workgroup per head: thread (d4, part)
// sums every 4th split for 4 output dims with all its loads in flight at once,
// the four parts meet in LDS.
__global__ __launch_bounds__(512) void mla_merge_kernel(const float *__restrict__ po, const float *__restrict__ pm, const float *__restrict__ pl,
                                                        int nh, int L, int n_splits, float *__restrict__ out) {
    __shared__ float w_l[MAX_SPLITS];
    __shared__ float den_l;
    __shared__ mk_f4 part_l[3][128];
    const int h = blockIdx.x, tid = threadIdx.x;
    if (tid < 64) {
        float mx = -INFINITY;
        for (int s = tid; s < n_splits; s += 64) mx = fmaxf(mx, pm[s * nh + h]);
        mx = mk_wave_max(mx);
        float den = 0.0f;
        for (int s = tid; s < n_splits; s += 64) {
            const float w = expf(pm[s * nh + h] - mx);
            w_l[s] = w;
            den += pl[s * nh + h] * w;
        }
        den = mk_wave_sum(den);
        if (tid == 0) den_l = den;
    }
    __syncthreads();
    const int d4 = tid & 127, part = tid >> 7;
    const bool live = d4 * 4 < L;
    mk_f4 num = {0.0f, 0.0f, 0.0f, 0.0f};
    if (live) {
#pragma unroll 4
        for (int s = part; s < n_splits; s += 4) num += *reinterpret_cast<const mk_f4 *>(po + ((size_t)s * nh + h) * L + d4 * 4) * w_l[s];
    }
    if (part > 0) part_l[part - 1][d4] = num;
    __syncthreads();
    if (part == 0 && live) {
        num += part_l[0][d4] + part_l[1][d4] + part_l[2][d4];
        const float den = den_l;
        *reinterpret_cast<mk_f4 *>(out + (size_t)h * L + d4 * 4) = mk_f4{num.x / den, num.y / den, num.z / den, num.w / den};
    }
}

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

}  // namespace

extern "C" size_t mk_mla_decode_workspace_bytes(size_t nh, size_t L, size_t n_pos) {
    (void)n_pos;
    return align_up(nh * L, 256) + align_up(nh * (L / 32) * 4, 256) + align_up(MAX_SPLITS * nh * L * 4, 256) +
           2 * align_up(MAX_SPLITS * nh * 4, 256);
}

namespace {
int mla_decode_impl(const int8_t *lat_q, const void *lat_s, const int8_t *rope_q, const void *rope_s, size_t pos, const float *q, size_t nh,
                    size_t L, size_t R, float scale, void *workspace, float *out, void *stream) {
    MK_REQUIRE(lat_q && lat_s && q && workspace && out && (R == 0 || (rope_q && rope_s)), "null pointer");
    MK_REQUIRE(L % 64 == 0 && L >= 64 && L <= 512, "latent width must be a multiple of 64 up to 512");
    MK_REQUIRE(R % 32 == 0 && R <= 64, "rope width must be 0, 32 or 64");
    MK_REQUIRE(nh >= 1 && nh <= 65535 && pos < 0x7FFFFF00u, "bad head count or position");
    MK_REQUIRE(((uintptr_t)lat_q & 15) == 0 && ((uintptr_t)workspace & 255) == 0, "cache must be 16-byte and workspace 256-byte aligned");
    MK_REQUIRE(((uintptr_t)rope_q & 15) == 0 && ((uintptr_t)lat_s & 7) == 0 && ((uintptr_t)rope_s & 3) == 0,
               "rope bytes must be 16-byte, latent scales 8-byte, rope scales 4-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    const int n_pos = (int)pos + 1;
    uint8_t *w = (uint8_t *)workspace;
    MlaArgs a;
    a.lat_q = lat_q;
    a.lat_s = (const uint16_t *)lat_s;
    a.rope_q = rope_q;
    a.rope_s = (const uint16_t *)rope_s;
    a.q = q;
    int8_t *qq = (int8_t *)w;
    w += align_up(nh * L, 256);
    float *qs = (float *)w;
    w += align_up(nh * (L / 32) * 4, 256);
    a.po = (float *)w;
    w += align_up(MAX_SPLITS * nh * L * 4, 256);
    a.pm = (float *)w;
    w += align_up(MAX_SPLITS * nh * 4, 256);
    a.pl = (float *)w;
    a.qq = qq;
    a.qs = qs;
    a.nh = (int)nh;
    a.L = (int)L;
    a.R = (int)R;
    a.n_pos = n_pos;
    a.scale = scale;
    const int tiles = (n_pos + TJ - 1) / TJ;
    const bool mfma = L == ML && R == MR && !MK_TUNE("MK_MLA_VALU", 0);
    // split the context in whole tiles: one workgroup per CU for the MFMA kernel
    // (its register and LDS budget allows one), about 512 for the VALU kernel
    const int head_groups = (int)((nh + HPG - 1) / HPG);
    int want = ((mfma ? 256 : 512) + head_groups - 1) / head_groups;
    if (want > MAX_SPLITS) want = MAX_SPLITS;
    if (want > tiles) want = tiles;
    const int tiles_per_split = (tiles + want - 1) / want;
    a.split_len = tiles_per_split * TJ;
    a.n_splits = (tiles + tiles_per_split - 1) / tiles_per_split;
    int s;
    if (mfma) {
        MK_REQUIRE(n_pos <= (1 << 22), "the MFMA kernel addresses the cache with 32-bit byte offsets: at most 4 Mi positions");
        if ((s = mk_lds_opt_in(reinterpret_cast<const void *>(mla_mfma_kernel), MLA_LDS_BYTES)) != MK_OK) return s;
        hipLaunchKernelGGL(mla_mfma_kernel, dim3(a.n_splits, head_groups), dim3(256), MLA_LDS_BYTES, st, a, out);
        if ((s = mk_launch_status("mla_mfma")) != MK_OK) return s;
        if (a.n_splits == 1) return MK_OK;
    } else {
        const int nblk = (int)(nh * (L / 32));
        hipLaunchKernelGGL(mla_q_prep_kernel, dim3((nblk + 7) / 8), dim3(256), 0, st, q, (int)nh, (int)L, (int)R, qq, qs);
        if ((s = mk_launch_status("mla_q_prep")) != MK_OK) return s;
        const size_t lds = (size_t)TJ * L + (size_t)TJ * (L / 32) * 4 + (size_t)TJ * R * 4 + (size_t)HPG * TJ * 4;
        if ((s = mk_lds_opt_in(reinterpret_cast<const void *>(mla_partial_kernel), 96 * 1024)) != MK_OK) return s;
        hipLaunchKernelGGL(mla_partial_kernel, dim3(a.n_splits, head_groups), dim3(256), lds, st, a);
        if ((s = mk_launch_status("mla_partial")) != MK_OK) return s;
    }
    hipLaunchKernelGGL(mla_merge_kernel, dim3((unsigned)nh), dim3(512), 0, st, a.po, a.pm, a.pl, (int)nh, (int)L, a.n_splits, out);
    return mk_launch_status("mla_merge");
}
}  // namespace

extern "C" int mk_dev_mla_q8_decode(const int8_t *lat_q, const void *lat_s, const int8_t *rope_q, const void *rope_s, size_t pos,
                                    const float *q, size_t nh, size_t L, size_t R, float scale, void *workspace, float *out, void *stream) {
    return mla_decode_impl(lat_q, lat_s, rope_q, rope_s, pos, q, nh, L, R, scale, workspace, out, stream);
}

// ------------------------------------------------ the entry point that allocates nothing
// mk_dev_mla_q8_decode_static: the same kernels with their scratch (the quantized query, the splits' partial outputs
// and their (max, normaliser) pairs) in a file-scope device array instead of a caller's workspace.  Sized for the
// largest supported call: 128 heads, latent 512, MAX_SPLITS splits.
constexpr size_t MLA_STATIC_MAX_NH = 128, MLA_STATIC_MAX_L = 512;
constexpr size_t MLA_STATIC_BYTES = 128 * 512 + 128 * 16 * 4 + (size_t)MAX_SPLITS * 128 * 512 * 4 + 2 * (size_t)MAX_SPLITS * 128 * 4;
static __device__ __align__(256) uint8_t mla_static_scratch[MLA_STATIC_BYTES];

namespace {
constexpr int MLA_STATIC_MAX_DEVICES = 64;
std::mutex g_static_mu;
void *g_static_ptr[MLA_STATIC_MAX_DEVICES] = {};  // device address of mla_static_scratch on each device (every GPU holds its own copy)
}  // namespace

// Resolves the scratch array's address on the current device, once per device.  mk_init calls it, so a caller that
// initialises the library before it starts a graph capture never reaches the runtime query from inside the capture.
int mk_mla_static_init(void **out_ptr) {
    int dev = 0;
    MK_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= MLA_STATIC_MAX_DEVICES) {
        mk_set_error("device index %d beyond the %d this entry point keeps scratch addresses for", dev, MLA_STATIC_MAX_DEVICES);
        return MK_ERR_UNSUPPORTED;
    }
    std::lock_guard<std::mutex> lk(g_static_mu);
    if (!g_static_ptr[dev]) {
        void *p = nullptr;
        MK_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(mla_static_scratch)));
        if (!p || ((uintptr_t)p & 255) != 0) {
            mk_set_error("hipGetSymbolAddress(mla_static_scratch) gave %p", p);
            return MK_ERR_HIP;
        }
        g_static_ptr[dev] = p;
    }
    if (out_ptr) *out_ptr = g_static_ptr[dev];
    return MK_OK;
}

extern "C" size_t mk_mla_decode_static_max_heads(void) { return MLA_STATIC_MAX_NH; }

extern "C" int mk_dev_mla_q8_decode_static(const int8_t *lat_q, const void *lat_s, const int8_t *rope_q, const void *rope_s, size_t pos,
                                           const float *q, size_t nh, size_t L, size_t R, float scale, float *out, void *stream) {
    if (nh > MLA_STATIC_MAX_NH || L > MLA_STATIC_MAX_L || mk_mla_decode_workspace_bytes(nh, L, pos + 1) > MLA_STATIC_BYTES) {
        mk_set_error("mk_dev_mla_q8_decode_static holds scratch for at most %zu heads of latent width %zu (%zu bytes); got %zu heads, width %zu: "
                     "use mk_dev_mla_q8_decode with a workspace",
                     MLA_STATIC_MAX_NH, MLA_STATIC_MAX_L, MLA_STATIC_BYTES, nh, L);
        return MK_ERR_UNSUPPORTED;
    }
    void *scratch = nullptr;  // the array's device address: never the array's name, which is a host-side stand-in here
    const int s = mk_mla_static_init(&scratch);
    if (s != MK_OK) return s;
    return mla_decode_impl(lat_q, lat_s, rope_q, rope_s, pos, q, nh, L, R, scale, scratch, out, stream);
}
