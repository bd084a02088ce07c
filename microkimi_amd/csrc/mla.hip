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
    float dx = fmaxf(mx, 0.0f) / 127.0f;  // (a block of NaN only: the reference's maximum, folded from 0, is 0)
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
// Latent 512 + rope 64 (the shape of the production models).
constexpr int ML = 512, MR = 64;
constexpr int KROW = 592;      // LDS row stride in bytes: 16 rows at 16-byte granularity fall in distinct banks
constexpr int KS_STRIDE = 68;  // f32 scale row [block][position]
constexpr int KH_STRIDE = 72;  // f16 scale row [block][position]
constexpr int KS_OFF = TJ * KROW;
constexpr int KH_OFF = KS_OFF + 18 * KS_STRIDE * 4;
constexpr int MLA_TILE_BYTES = KH_OFF + 16 * KH_STRIDE * 2;
constexpr int P_STRIDE = 72;   // f16 per probability row: 64 positions + 8 of padding

typedef _Float16 mk_h4 __attribute__((ext_vector_type(4)));
typedef _Float16 mk_h8 __attribute__((ext_vector_type(8)));
typedef int mk_i2 __attribute__((ext_vector_type(2)));

struct MlaStage {
    mk_i4 lat[8];
    mk_i4 rope;
    mk_u2 ls;
    uint32_t rs;
};

__device__ __forceinline__ uint32_t mk_perm(uint32_t hi, uint32_t lo, uint32_t sel) { return __builtin_amdgcn_perm(hi, lo, sel); }

// Workgroup barrier that waits for this wave's LDS traffic only.  __syncthreads() also waits for every global load
// in flight (s_waitcnt vmcnt(0)), which would put the latency of the next tile's prefetch into each barrier.
__device__ __forceinline__ void mk_lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// e^x for x <= 0 through the hardware 2^x (v_exp_f32, about 1 ulp): the rounding of x * log2(e) adds |x| * 2^-24
// relative, 2e-6 at x = -30, where the weight itself is 1e-13.  exp(-inf) = 0.
__device__ __forceinline__ float mk_exp_neg(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896340736f); }

// A workgroup of four waves serves 16 heads over one split of the context, 64 positions (a tile) at a time, from ONE
// tile buffer: 180 registers and 62 KiB of LDS, so two workgroups share a compute unit.
//
//   scores   wave w: positions 16 w .. 16 w + 15 against the 16 heads.  Latent part: v_mfma_i32_16x16x64_i8, cache bytes
//            as the A operand (lane l: row l%16, bytes 16*(l/16).. of the 64-byte step), q8 query as B.  One
//            instruction spans two scale blocks: it is issued with the second block's query bytes zeroed and whole,
//            the second block's dot is the difference.  The integer block dots are scaled by (query block scale *
//            cache block scale) in f32, the reference's per-block term (src/model.rs:1858-1871).  Rope part:
//            v_mfma_f32_16x16x32_f16 in split precision: the rope bytes times their scale as exact f16 pairs (see
//            "out"), the f32 query as hi + lo.
//   softmax  one reference point per head and tile: the four waves exchange maxima and sums through LDS and write the
//            probabilities as f16 pairs into a [head][position] tile
//   out      wave w owns the output dims 128 w .. 128 w + 127 of all heads over all 64 positions: each cache byte is
//            converted once per workgroup.  v_mfma_f32_16x16x32_f16 in split precision: the cache value v = q * s (int8
//            times f16 scale, src/model.rs:1641-1646) is formed as an exact f16 pair, hi = rn(q*s), lo = fma(q, s, -hi)
//            (the product has 19 significant bits and the residual is a multiple of the scale's ulp, so hi + lo == v);
//            the probability is split the same way (hi = rn(p), lo = rn(p - hi), relative error below 2^-21); the
//            products p_hi v_hi, p_hi v_lo, p_lo v_hi are accumulated in f32.  The B operand (K = 32 positions x N = 16
//            dims) wants the 8 positions of a lane contiguous while the cache has dims contiguous:
//            ds_read_b64_tr_b8 delivers that transpose (a group of 16 lanes reads 8 rows x 16 bytes, lanes 2k and 2k+1
//            giving the two halves of row k, and lane i receives byte i of every row; measured with byte-valued LDS
//            contents).  Bytes -> f16 with v_perm: 0x6400 | (b ^ 0x80) is 1152 + b.  Two operand tiles are converted
//            and multiplied at a time.
//   refill   barrier, the prefetched next tile goes from registers into the one buffer, barrier
//
// A split's partial result is one [16][512] block per workgroup; with a single split the workgroup writes the
// normalised output itself.  Where the time goes at 16k context (64 splits x 8 head groups, 31 us; measured by
// compiling parts out): launch, first tile and exit 5 us, query quantization 2 us, the partial results' stores 5.5 us,
// rope scores + softmax + refill 1.5 us per tile, latent scores 1.35 us per tile, output product 1.85 us per tile; the
// barriers cost 1.2 us in all and the prefetch loads nothing.  Two other forms were built, passed the parity tests and
// measured the same 30-31 us: eight waves serving 32 heads (half the byte conversions per head, but lock-stepped
// phases and one workgroup per CU), and four waves serving 32 heads with one wave per SIMD.
constexpr int NHG = 1;  // 16-head groups per workgroup
struct M4 {
    static constexpr int HEADS = 16 * NHG;
    static constexpr int Q_OFF = MLA_TILE_BYTES;                // [NHG][8 S][64 lanes] 16-byte query operands
    static constexpr int Z_OFF = Q_OFF + NHG * 8 * 64 * 16;     // 64 zero bytes: the "masked" query operand of lanes 32-63
    static constexpr int QS_OFF = Z_OFF + 64;                   // [NHG][8][64] scale pairs
    static constexpr int P_OFF = QS_OFF + NHG * 8 * 64 * 8;     // P hi [HEADS][P_STRIDE] f16, then P lo
    static constexpr int ST_OFF = P_OFF + 2 * HEADS * P_STRIDE * 2;
    static constexpr int LDS_BYTES = ST_OFF + (4 * HEADS + 4 * HEADS + 3 * HEADS) * 4;  // wmax, wsum, corr, final m, final l
};

// -DMK_MLA_TRACE: wave 0 of every workgroup leaves time stamps (100 MHz) of the last launch, read with mk_debug_mla_ts:
// 0 start, 1 queries and first tile staged, 2 first tile's scores, 3 its probabilities, 4 its output product, 5 all tiles
// done, 6 end
#ifdef MK_MLA_TRACE
__device__ unsigned long long g_mla_ts[1024 * 8];
#define MLA_TS(i) ts[i] = __builtin_amdgcn_s_memrealtime()
#else
#define MLA_TS(i)
#endif

__global__ __launch_bounds__(256, 2) void mla_mfma_kernel(MlaArgs a, float *__restrict__ out) {
    using C4 = M4;
#ifdef MK_MLA_TRACE
    unsigned long long ts[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#endif
    MLA_TS(0);
    constexpr int HEADS = C4::HEADS;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int split = blockIdx.x;
    const int hbase = blockIdx.y * HEADS;
    const int p_begin = split * a.split_len;
    const int p_end = min(p_begin + a.split_len, a.n_pos);
    const int ntiles = (p_end - p_begin + TJ - 1) / TJ;
    const int last_pos = a.n_pos - 1;

    float *wmax_l = reinterpret_cast<float *>(lds + C4::ST_OFF);  // [4 waves][HEADS]
    float *wsum_l = wmax_l + 4 * HEADS;
    float *corr_l = wsum_l + 4 * HEADS;
    float *finm_l = corr_l + HEADS, *finl_l = finm_l + HEADS;
    _Float16 *ph_l = reinterpret_cast<_Float16 *>(lds + C4::P_OFF);
    _Float16 *pl_l = ph_l + HEADS * P_STRIDE;
    mk_i4 *qb_l = reinterpret_cast<mk_i4 *>(lds + C4::Q_OFF);   // [hg][S][lane]
    mk_f2 *qs_l = reinterpret_cast<mk_f2 *>(lds + C4::QS_OFF);  // [hg][S][lane]: scales of blocks 2S, 2S+1

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
        const uint32_t pr2 = (uint32_t)min(t0 + lane, last_pos);
        st.rs = mk_ldg_u32(a.rope_s + pr2 * (MR / 32));
    };
    auto stage_store = [&](const MlaStage &st) {
        float *ks = reinterpret_cast<float *>(lds + KS_OFF);
        uint16_t *kh = reinterpret_cast<uint16_t *>(lds + KH_OFF);
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const int i = tid + 256 * k;
            *reinterpret_cast<mk_i4 *>(lds + (i >> 5) * KROW + (i & 31) * 16) = st.lat[k];  // row (tid >> 5) + 8k
        }
        *reinterpret_cast<mk_i4 *>(lds + (tid >> 2) * KROW + ML + (tid & 3) * 16) = st.rope;
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
        if (wave == 0) {
            ks[16 * KS_STRIDE + lane] = mk_f16_bits_to_f32((uint16_t)(st.rs & 0xFFFFu));
            ks[17 * KS_STRIDE + lane] = mk_f16_bits_to_f32((uint16_t)(st.rs >> 16));
        }
    };
    MlaStage st;
    stage_load(st, p_begin);

    // The queries.  Lane (c, q4) owns bytes 16*(4S+q4).. of each 64-value step S of head c of a 16-head group, half of
    // scale block 2S + q4/2; its partner for the block maximum is lane ^ 16.  Each wave quantizes two of the eight
    // steps of every head group and passes them to the others through LDS (src/model.rs:1812-1821).
    mk_h8 qrh[NHG][2], qrl[NHG][2];  // rope part of the query (f32 in the reference), dims 16*q4.. of head c, as f16 pairs hi + lo
    {
        const int q4 = lane >> 4, c = lane & 15;
#pragma unroll
        for (int hg = 0; hg < NHG; hg++) {
            const float *qrow = a.q + (size_t)min(hbase + 16 * hg + c, a.nh - 1) * (ML + MR);
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
                const float dx = fmaxf(mx, 0.0f) / 127.0f;  // (a block of NaN only: the reference's maximum, folded from 0, is 0)
                mk_i4 packed;
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    uint32_t w = 0;
                    if (dx != 0.0f) {
                        float qf[4];
                        mk_q8_round4(v[k], dx, qf);
                        w = ((uint32_t)(int)qf[0] & 255u) | (((uint32_t)(int)qf[1] & 255u) << 8) | (((uint32_t)(int)qf[2] & 255u) << 16) |
                            ((uint32_t)(int)qf[3] << 24);
                    }
                    packed[k] = (int)w;
                }
                const float other = __shfl_xor(dx, 32, MK_WAVE);
                qb_l[(hg * 8 + S) * 64 + lane] = packed;
                qs_l[(hg * 8 + S) * 64 + lane] = q4 < 2 ? mk_f2{dx, other} : mk_f2{other, dx};
            }
#pragma unroll
            for (int k = 0; k < 16; k++) {
                const float v = qrow[ML + 16 * q4 + k];
                const _Float16 hi = (_Float16)v;
                qrh[hg][k >> 3][k & 7] = hi;
                qrl[hg][k >> 3][k & 7] = (_Float16)(v - (float)hi);
            }
        }
        if (tid < 16) reinterpret_cast<uint32_t *>(lds + C4::Z_OFF)[tid] = 0u;
    }

    mk_f4 o[NHG][8];  // heads 16 hg + 4 q4 + r, dim 128 wave + 16 n + c
#pragma unroll
    for (int hg = 0; hg < NHG; hg++)
#pragma unroll
        for (int n = 0; n < 8; n++) o[hg][n] = mk_f4{0.0f, 0.0f, 0.0f, 0.0f};
    float m[NHG], l[NHG];  // of head 16 hg + c; the four waves keep equal copies
#pragma unroll
    for (int hg = 0; hg < NHG; hg++) {
        m[hg] = -INFINITY;
        l[hg] = 0.0f;
    }
    const mk_i4 zero4 = {0, 0, 0, 0};
    stage_store(st);
    __syncthreads();
    MLA_TS(1);

    for (int tile = 0; tile < ntiles; tile++) {
        const int t0 = p_begin + tile * TJ;
        const int t_next = min(t0 + TJ, last_pos);
        // The lane index is made opaque once per tile: every LDS address below is then recomputed from it inside the
        // loop (a few instructions each) instead of being kept in a register of its own across the whole kernel.
        int lane_v = lane;
        asm volatile("" : "+v"(lane_v));
        const int q4 = lane_v >> 4, c = lane_v & 15;
        const float *ks = reinterpret_cast<const float *>(lds + KS_OFF);
        // ---- scores of this wave's 16 positions x 16 NHG heads
        const int prow = 16 * wave;
        const uint8_t *krow = lds + (prow + c) * KROW + q4 * 16;
        float sc[NHG][4];
        {
            // rope: bytes -> exact f16 pairs (see the output product below), 64 dims = two K = 32 steps
            const mk_i4 kr = *reinterpret_cast<const mk_i4 *>(lds + (prow + c) * KROW + ML + q4 * 16);
            const float rsc = ks[(16 + (q4 >> 1)) * KS_STRIDE + prow + c];
            mk_f4 cr[NHG];
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
#pragma unroll
                for (int hg = 0; hg < NHG; hg++) {
                    mk_f4 cr0 = {0.0f, 0.0f, 0.0f, 0.0f}, cr1 = cr0;
                    cr0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kh8[0], qrh[hg][0], cr0, 0, 0, 0);
                    cr1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kh8[1], qrh[hg][1], cr1, 0, 0, 0);
                    cr0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kl8[0], qrh[hg][0], cr0, 0, 0, 0);
                    cr1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kl8[1], qrh[hg][1], cr1, 0, 0, 0);
                    cr0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kh8[0], qrl[hg][0], cr0, 0, 0, 0);
                    cr1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kh8[1], qrl[hg][1], cr1, 0, 0, 0);
                    cr[hg] = cr0 + cr1;
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            // latent part in two halves of four 64-value steps.  A step spans two scale blocks: the instruction is issued
            // with the query of lanes 32-63 (the second block) replaced by zeros, and whole; the second block's dot is
            // the difference.  The zeroed operand is read from a zero region of LDS, one address select per step.
            mk_f4 acc[NHG];
#pragma unroll
            for (int hg = 0; hg < NHG; hg++) acc[hg] = mk_f4{0.0f, 0.0f, 0.0f, 0.0f};
            const uint32_t q_addr = (uint32_t)(C4::Q_OFF + lane_v * 16), qm_addr = q4 < 2 ? q_addr : (uint32_t)C4::Z_OFF;
            const uint32_t qm_step = q4 < 2 ? 1024u : 0u;
#pragma unroll
            for (int half = 0; half < 2; half++) {
                mk_i4 ka[4];
#pragma unroll
                for (int S = 0; S < 4; S++) ka[S] = *reinterpret_cast<const mk_i4 *>(krow + (4 * half + S) * 64);
                mk_f4 k0[4], k1[4];  // the cache's block scales of this lane's 4 positions: shared by the head groups
#pragma unroll
                for (int S = 0; S < 4; S++) {
                    const int SS = 4 * half + S;
                    k0[S] = *reinterpret_cast<const mk_f4 *>(ks + (2 * SS) * KS_STRIDE + prow + 4 * q4);
                    k1[S] = *reinterpret_cast<const mk_f4 *>(ks + (2 * SS + 1) * KS_STRIDE + prow + 4 * q4);
                }
#pragma unroll
                for (int hg = 0; hg < NHG; hg++) {
                    mk_i4 c0[4], cf[4];
#pragma unroll
                    for (int S = 0; S < 4; S++) {
                        const int SS = hg * 8 + 4 * half + S;
                        const mk_i4 qv = *reinterpret_cast<const mk_i4 *>(lds + q_addr + SS * 1024);
                        const mk_i4 qm = *reinterpret_cast<const mk_i4 *>(lds + qm_addr + SS * qm_step);
                        c0[S] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ka[S], qm, zero4, 0, 0, 0);
                        cf[S] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ka[S], qv, zero4, 0, 0, 0);
                    }
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int S = 0; S < 4; S++) {
                        const mk_f2 qsc = qs_l[(hg * 8 + 4 * half + S) * 64 + lane_v];
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            acc[hg][r] = fmaf(qsc.y * k1[S][r], (float)(cf[S][r] - c0[S][r]), fmaf(qsc.x * k0[S][r], (float)c0[S][r], acc[hg][r]));
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
#pragma unroll
            for (int hg = 0; hg < NHG; hg++)
#pragma unroll
                for (int r = 0; r < 4; r++) sc[hg][r] = (t0 + prow + 4 * q4 + r) < p_end ? (acc[hg][r] + cr[hg][r]) * a.scale : -INFINITY;
        }
        __builtin_amdgcn_sched_barrier(0);
        // the next tile's loads go out behind the score stage (whose registers they would otherwise share); the softmax
        // exchange and the output product cover their latency
#ifdef MK_MLA_TRACE
        if (tile == 0) MLA_TS(2);
#endif
        const bool more = tile + 1 < ntiles;  // the last tile fetches nothing and leaves the buffer as it is
        stage_load(st, t_next);  // (clamped to the last position; the last tile's fetch is never waited for)
        __builtin_amdgcn_sched_barrier(0);
        // ---- online softmax: one reference point per head and tile for all four waves
#pragma unroll
        for (int hg = 0; hg < NHG; hg++) {
            float tm = fmaxf(fmaxf(sc[hg][0], sc[hg][1]), fmaxf(sc[hg][2], sc[hg][3]));
            tm = mk_rows_max(tm);
            if (q4 == 0) wmax_l[wave * HEADS + 16 * hg + c] = tm;
        }
        mk_lds_barrier();
#pragma unroll
        for (int hg = 0; hg < NHG; hg++) {
            const int hl = 16 * hg + c;
            const float mt4 = fmaxf(fmaxf(wmax_l[hl], wmax_l[HEADS + hl]), fmaxf(wmax_l[2 * HEADS + hl], wmax_l[3 * HEADS + hl]));  // finite
            const float m_new = fmaxf(m[hg], mt4);
            const float corr = mk_exp_neg(m[hg] - m_new);  // first tile: exp(-inf) = 0
            float ts = 0.0f;
            mk_h4 phi, plo;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const float pv = mk_exp_neg(sc[hg][r] - m_new);
                ts += pv;
                const _Float16 hi = (_Float16)pv;
                phi[r] = hi;
                plo[r] = (_Float16)(pv - (float)hi);
            }
            ts = mk_rows_sum(ts);
            if (q4 == 0) wsum_l[wave * HEADS + hl] = ts;
            if (wave == 0 && q4 == 0) corr_l[hl] = corr;
            *reinterpret_cast<mk_h4 *>(ph_l + hl * P_STRIDE + prow + 4 * q4) = phi;
            *reinterpret_cast<mk_h4 *>(pl_l + hl * P_STRIDE + prow + 4 * q4) = plo;
            l[hg] *= corr;
            m[hg] = m_new;
        }
        mk_lds_barrier();
#pragma unroll
        for (int hg = 0; hg < NHG; hg++) {
            const int hl = 16 * hg + c;
            l[hg] += (wsum_l[hl] + wsum_l[HEADS + hl]) + (wsum_l[2 * HEADS + hl] + wsum_l[3 * HEADS + hl]);
        }
        __builtin_amdgcn_sched_barrier(0);
#ifdef MK_MLA_TRACE
        if (tile == 0) MLA_TS(3);
#endif
        // ---- out[heads][dims 128 wave ..] += P V over the tile's 64 positions
#pragma unroll
        for (int hg = 0; hg < NHG; hg++) {
            const mk_f4 cA = *reinterpret_cast<const mk_f4 *>(corr_l + 16 * hg + 4 * q4);
#pragma unroll
            for (int n = 0; n < 8; n++)
#pragma unroll
                for (int r = 0; r < 4; r++) o[hg][n][r] *= cA[r];
        }
        const uint16_t *kh = reinterpret_cast<const uint16_t *>(lds + KH_OFF);
        const mk_h2 bias = {(_Float16)1152.0f, (_Float16)1152.0f};
        // operand tile (kstep, n): positions 32 kstep + 8 q4 .. + 7, dims 128 wave + 16 n + c.  Transposed read: lanes
        // 2k, 2k+1 of each 16-lane group address the two halves of row p0 + k, dims d0..d0+15; lane c receives dim
        // d0 + c of rows p0 .. p0 + 7.  Two tiles (n, n + 1) go through conversion and the matrix cores together, so
        // that consecutive matrix instructions accumulate into different registers; the next pair's bytes and scales
        // are requested before the current pair is converted.
        mk_i2 raw[2][2];
        mk_i4 sraw[2];
        auto fetch = [&](int j, int slot) {  // pair j = (kstep, n / 2): both tiles lie in one 32-dim block
            const int p0 = 32 * (j >> 2) + 8 * q4;
            const int d0 = 128 * wave + 32 * (j & 3);
#pragma unroll
            for (int e = 0; e < 2; e++) {
                const uint8_t *src = lds + (p0 + (c >> 1)) * KROW + d0 + 16 * e + 8 * (c & 1);
                raw[slot][e] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) mk_i2 *)src);
            }
            sraw[slot] = *reinterpret_cast<const mk_i4 *>(kh + (d0 >> 5) * KH_STRIDE + p0);
        };
        fetch(0, 0);
        mk_h8 pah[NHG], pal[NHG];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int kstep = j >> 2, n0 = 2 * (j & 3);
            if ((j & 3) == 0) {
                const int p0 = 32 * kstep + 8 * q4;  // this lane's 8 positions of the K = 32 step
#pragma unroll
                for (int hg = 0; hg < NHG; hg++) {
                    pah[hg] = *reinterpret_cast<const mk_h8 *>(ph_l + (16 * hg + c) * P_STRIDE + p0);
                    pal[hg] = *reinterpret_cast<const mk_h8 *>(pl_l + (16 * hg + c) * P_STRIDE + p0);
                }
            }
            if (j + 1 < 8) fetch(j + 1, (j + 1) & 1);
            const int sl = j & 1;
            const uint32_t s0 = (uint32_t)sraw[sl][0], s1 = (uint32_t)sraw[sl][1], s2 = (uint32_t)sraw[sl][2], s3 = (uint32_t)sraw[sl][3];
            const mk_h2 s01 = __builtin_bit_cast(mk_h2, s0), s23 = __builtin_bit_cast(mk_h2, s1);
            const mk_h2 s45 = __builtin_bit_cast(mk_h2, s2), s67 = __builtin_bit_cast(mk_h2, s3);
            mk_h8 bh[2], bl[2];
#pragma unroll
            for (int e = 0; e < 2; e++) {
                const uint32_t w0 = (uint32_t)raw[sl][e][0] ^ 0x80808080u, w1 = (uint32_t)raw[sl][e][1] ^ 0x80808080u;
                const mk_h2 v01 = __builtin_bit_cast(mk_h2, mk_perm(0x64646464u, w0, 0x04010400u)) - bias;
                const mk_h2 v23 = __builtin_bit_cast(mk_h2, mk_perm(0x64646464u, w0, 0x04030402u)) - bias;
                const mk_h2 v45 = __builtin_bit_cast(mk_h2, mk_perm(0x64646464u, w1, 0x04010400u)) - bias;
                const mk_h2 v67 = __builtin_bit_cast(mk_h2, mk_perm(0x64646464u, w1, 0x04030402u)) - bias;
                const mk_h2 h01 = v01 * s01, h23 = v23 * s23, h45 = v45 * s45, h67 = v67 * s67;
                const mk_h2 l01 = __builtin_elementwise_fma(v01, s01, -h01), l23 = __builtin_elementwise_fma(v23, s23, -h23);
                const mk_h2 l45 = __builtin_elementwise_fma(v45, s45, -h45), l67 = __builtin_elementwise_fma(v67, s67, -h67);
                bh[e] = mk_h8{h01.x, h01.y, h23.x, h23.y, h45.x, h45.y, h67.x, h67.y};
                bl[e] = mk_h8{l01.x, l01.y, l23.x, l23.y, l45.x, l45.y, l67.x, l67.y};
            }
#pragma unroll
            for (int hg = 0; hg < NHG; hg++) {
                o[hg][n0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pah[hg], bh[0], o[hg][n0], 0, 0, 0);
                o[hg][n0 + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pah[hg], bh[1], o[hg][n0 + 1], 0, 0, 0);
            }
#pragma unroll
            for (int hg = 0; hg < NHG; hg++) {
                o[hg][n0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pah[hg], bl[0], o[hg][n0], 0, 0, 0);
                o[hg][n0 + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pah[hg], bl[1], o[hg][n0 + 1], 0, 0, 0);
            }
#pragma unroll
            for (int hg = 0; hg < NHG; hg++) {
                o[hg][n0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pal[hg], bh[0], o[hg][n0], 0, 0, 0);
                o[hg][n0 + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pal[hg], bh[1], o[hg][n0 + 1], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // ---- refill the tile buffer: everybody is done reading it, then the prefetched rows go in
#ifdef MK_MLA_TRACE
        if (tile == 0) MLA_TS(4);
#endif
        if (more) {
            mk_lds_barrier();
            stage_store(st);
            mk_lds_barrier();
        }
    }
    MLA_TS(5);

    // ---- store: the split's partial [HEADS][512] block, or the normalised rows when there is one split
    {
        const int q4 = lane >> 4, c = lane & 15;
        if (wave == 0 && q4 == 0) {
#pragma unroll
            for (int hg = 0; hg < NHG; hg++) {
                finm_l[16 * hg + c] = m[hg];
                finl_l[16 * hg + c] = l[hg];
            }
        }
        __syncthreads();
        const bool single = a.n_splits == 1;
#pragma unroll
        for (int hg = 0; hg < NHG; hg++) {
            const mk_f4 lt = *reinterpret_cast<const mk_f4 *>(finl_l + 16 * hg + 4 * q4);
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int h = hbase + 16 * hg + 4 * q4 + r;
                if (h < a.nh) {
                    float *dst = (single ? out + (size_t)h * ML : a.po + ((size_t)split * a.nh + h) * ML) + 128 * wave + c;
                    if (single) {
#pragma unroll
                        for (int n = 0; n < 8; n++) dst[16 * n] = o[hg][n][r] / lt[r];
                    } else {
#pragma unroll
                        for (int n = 0; n < 8; n++) dst[16 * n] = o[hg][n][r];
                    }
                }
            }
        }
        if (!single && tid < HEADS && hbase + tid < a.nh) {
            a.pm[split * a.nh + hbase + tid] = finm_l[tid];
            a.pl[split * a.nh + hbase + tid] = finl_l[tid];
        }
    }
#ifdef MK_MLA_TRACE
    MLA_TS(6);
    if (tid == 0 && blockIdx.y * gridDim.x + blockIdx.x < 1024)
        for (int i = 0; i < 8; i++) g_mla_ts[(blockIdx.y * gridDim.x + blockIdx.x) * 8 + i] = ts[i];
#endif
}

#ifdef MK_MLA_TRACE
}  // namespace
extern "C" int mk_debug_mla_ts(unsigned long long *out) {
    MK_HIP_TRY(hipMemcpyFromSymbol(out, HIP_SYMBOL(g_mla_ts), sizeof(unsigned long long) * 1024 * 8));
    return MK_OK;
}
namespace {
#endif

// log-sum-exp merge of the splits.  A workgroup per (head, quarter of the output dims): thread (d4, part) sums
// every 8th split for 4 output dims with all its loads in flight at once, the eight parts meet in LDS.
__global__ __launch_bounds__(256) void mla_merge_kernel(const float *__restrict__ po, const float *__restrict__ pm, const float *__restrict__ pl,
                                                        int nh, int L, int n_splits, float *__restrict__ out) {
    __shared__ float w_l[MAX_SPLITS];
    __shared__ float den_l;
    __shared__ mk_f4 part_l[7][32];
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
    const int d4 = blockIdx.y * 32 + (tid & 31), part = tid >> 5;
    const bool live = d4 * 4 < L;
    mk_f4 num = {0.0f, 0.0f, 0.0f, 0.0f};
    if (live) {
#pragma unroll 8
        for (int s = part; s < n_splits; s += 8) num += *reinterpret_cast<const mk_f4 *>(po + ((size_t)s * nh + h) * L + d4 * 4) * w_l[s];
    }
    if (part > 0) part_l[part - 1][tid & 31] = num;
    __syncthreads();
    if (part == 0 && live) {
#pragma unroll
        for (int k = 0; k < 7; k++) num += part_l[k][tid & 31];
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
    // Split the context in whole tiles.  Every split costs a partial result per head (2 KiB each way: stored here,
    // read by the merge), every workgroup a launch slot: two workgroups per CU (512) pay from about 8k positions,
    // below that one per CU (256).  About 512 workgroups for the VALU kernel.
    const int head_groups = (int)((nh + HPG - 1) / HPG);
    const int wgs_tune = MK_TUNE("MK_MLA_WGS", 0);
    int want = ((wgs_tune ? wgs_tune : (mfma && n_pos < 8192 ? 256 : 512)) + head_groups - 1) / head_groups;
    if (want > MAX_SPLITS) want = MAX_SPLITS;
    if (want > tiles) want = tiles;
    const int tiles_per_split = (tiles + want - 1) / want;
    a.split_len = tiles_per_split * TJ;
    a.n_splits = (tiles + tiles_per_split - 1) / tiles_per_split;
    int s;
    if (mfma) {
        MK_REQUIRE(n_pos <= (1 << 22), "the MFMA kernel addresses the cache with 32-bit byte offsets: at most 4 Mi positions");
        if ((s = mk_lds_opt_in(reinterpret_cast<const void *>(mla_mfma_kernel), M4::LDS_BYTES)) != MK_OK) return s;
        hipLaunchKernelGGL(mla_mfma_kernel, dim3(a.n_splits, head_groups), dim3(256), M4::LDS_BYTES, st, a, out);
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
    hipLaunchKernelGGL(mla_merge_kernel, dim3((unsigned)nh, (unsigned)((L / 4 + 31) / 32)), dim3(256), 0, st, a.po, a.pm, a.pl, (int)nh, (int)L, a.n_splits, out);
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
