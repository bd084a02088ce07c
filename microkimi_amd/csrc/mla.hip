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

__global__ __launch_bounds__(256) void mla_merge_kernel(const float *__restrict__ po, const float *__restrict__ pm, const float *__restrict__ pl,
                                                        int nh, int L, int n_splits, float *__restrict__ out) {
    const int h = blockIdx.y;
    const int d = blockIdx.x * blockDim.x + threadIdx.x;
    if (d >= L) return;
    float M = -INFINITY;
    for (int s = 0; s < n_splits; s++) M = fmaxf(M, pm[s * nh + h]);
    float num = 0.0f, den = 0.0f;
    for (int s = 0; s < n_splits; s++) {
        const float w = expf(pm[s * nh + h] - M);
        num += po[((size_t)s * nh + h) * L + d] * w;
        den += pl[s * nh + h] * w;
    }
    out[(size_t)h * L + d] = num / den;
}

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

}  // namespace

extern "C" size_t mk_mla_decode_workspace_bytes(size_t nh, size_t L, size_t n_pos) {
    (void)n_pos;
    return align_up(nh * L, 256) + align_up(nh * (L / 32) * 4, 256) + align_up(MAX_SPLITS * nh * L * 4, 256) +
           2 * align_up(MAX_SPLITS * nh * 4, 256);
}

extern "C" int mk_dev_mla_q8_decode(const int8_t *lat_q, const void *lat_s, const int8_t *rope_q, const void *rope_s, size_t pos,
                                    const float *q, size_t nh, size_t L, size_t R, float scale, void *workspace, float *out, void *stream) {
    MK_REQUIRE(lat_q && lat_s && q && workspace && out && (R == 0 || (rope_q && rope_s)), "null pointer");
    MK_REQUIRE(L % 64 == 0 && L >= 64 && L <= 512, "latent width must be a multiple of 64 up to 512");
    MK_REQUIRE(R % 32 == 0 && R <= 64, "rope width must be 0, 32 or 64");
    MK_REQUIRE(nh >= 1 && nh <= 65535 && pos < 0x7FFFFF00u, "bad head count or position");
    MK_REQUIRE(((uintptr_t)lat_q & 15) == 0 && ((uintptr_t)workspace & 255) == 0, "cache must be 16-byte and workspace 256-byte aligned");
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
    // split the context in whole tiles so that about 512 workgroups exist
    const int head_groups = (int)((nh + HPG - 1) / HPG);
    const int tiles = (n_pos + TJ - 1) / TJ;
    int want = (512 + head_groups - 1) / head_groups;
    if (want > MAX_SPLITS) want = MAX_SPLITS;
    if (want > tiles) want = tiles;
    const int tiles_per_split = (tiles + want - 1) / want;
    a.split_len = tiles_per_split * TJ;
    a.n_splits = (tiles + tiles_per_split - 1) / tiles_per_split;

    const int nblk = (int)(nh * (L / 32));
    hipLaunchKernelGGL(mla_q_prep_kernel, dim3((nblk + 7) / 8), dim3(256), 0, st, q, (int)nh, (int)L, (int)R, qq, qs);
    int s = mk_launch_status("mla_q_prep");
    if (s != MK_OK) return s;
    const size_t lds = (size_t)TJ * L + (size_t)TJ * (L / 32) * 4 + (size_t)TJ * R * 4 + (size_t)HPG * TJ * 4;
    static bool lds_opt_in = false;
    if (!lds_opt_in) {
        hipFuncSetAttribute(reinterpret_cast<const void *>(mla_partial_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
        lds_opt_in = true;
    }
    hipLaunchKernelGGL(mla_partial_kernel, dim3(a.n_splits, head_groups), dim3(256), lds, st, a);
    if ((s = mk_launch_status("mla_partial")) != MK_OK) return s;
    hipLaunchKernelGGL(mla_merge_kernel, dim3((unsigned)((L + 255) / 256), (unsigned)nh), dim3(256), 0, st, a.po, a.pm, a.pl, (int)nh, (int)L,
                       a.n_splits, out);
    return mk_launch_status("mla_merge");
}
