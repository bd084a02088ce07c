// Batched MoE decode: matvec_packed_q8 (src/mxfp4.rs:405-443) for all tokens that share an expert, with the expert's
// weights streamed once per group of tokens, on the gfx950 block-scaled matrix cores -- and still the reference's q8
// arithmetic, block term for block term:
//
//   out[i][r] = sum_g (idot_g as f32) * (2^(sb_g - 128) * dx_g[i]),   idot_g = sum_j LUT2[nib_j] * q_j[i]  (exact)
//
// An int8 activation is q = 16 a + b with a in [-8, 7] and b in [0, 15]: both exact in e4m3.  v_mfma_scale_f32_16x16x128_
// f8f6f4 multiplies 16 weight rows x 128 K-elements (four 32-blocks of MXFP4, as stored, with their e8m0 bytes) by 16
// columns.  A column here is (token t2 of a pair, phase p, part): it holds the a codes (part 0, block scale 2^4) or
// the b codes (part 1, scale 2^0) of ONE block -- block 4 s + p of the step s -- and zeros in the other three, so the
// result column is w_scale * 16 sum w a  or  w_scale * sum w b  of that single block: exact (multiples of a power of two
// below 2^24 of it).  The two parts are added (exact), the sum is multiplied by the token's f32 block scale dx (the
// one rounding of the reference's term, same value) and accumulated in f32; only the order of the sum over blocks
// differs from the CPU loop.  One matrix instruction serves two tokens; a group with more tokens issues more of them
// against the same weight registers, so an expert that several tokens of a decode batch selected (the shared expert:
// all of them) is read from HBM once.
//
// Weight side as in the prefill GEMM (gemm_mxfp4.hip): a workgroup owns 256 rows of one expert matrix, walks K in tiles
// of 512, loads whole 128-byte lines non-temporally one unit (16 rows x 256 bytes) ahead and restores the operand form
// in registers; the scale bytes of its rows go through LDS with the activation tile.
#include "mk_common.h"

namespace {

constexpr int QX_STEPS = 4;          // matrix instructions per K tile and row tile (K tile = 512 columns)
constexpr int QX_TOK = 4;            // tokens per pass: two pairs (one pair per pass ran batch 16 at 508 us against 467: groups of three
                                     // and four tokens then take a second pass over the weights)
constexpr int QX_ROW = 528;          // LDS bytes of one code row (512 + 16: the a and b rows of a token 4 banks apart)
constexpr int QX_TOK_STRIDE = 1152;  // LDS bytes between tokens (32 banks apart)
constexpr int QX_DX_OFF = QX_TOK * QX_TOK_STRIDE;  // then 16 f32 block scales per token
constexpr int QX_WSC_OFF = QX_DX_OFF + QX_TOK * 64;  // then 16 weight scale bytes for each of the 256 rows
constexpr int QX_BUF = QX_WSC_OFF + 256 * 16;
// behind the two buffers: zeros, as far as the largest constant offset of an operand read reaches (see q8x_pass)
constexpr int QX_ZERO_OFF = 2 * QX_BUF;
constexpr int QX_ZERO_BYTES = (QX_TOK / 2 - 1) * 2 * QX_TOK_STRIDE + (QX_STEPS - 1) * 128 + 16;
constexpr int QX_LDS = QX_ZERO_OFF + ((QX_ZERO_BYTES + 255) / 256) * 256;

struct Q8xArgs {
    const uint8_t *const *packed_ptrs[2];  // by expert id
    const uint8_t *const *scales_ptrs[2];
    const uint8_t *const *scales_t_ptrs[2];  // optional: the scale bytes in K-tile order (see gemm_mxfp4.hip)
    int rows, cols;
    const int8_t *xq;       // [activation rows][cols]
    const float *xs;        // [activation rows][cols / 32]
    const int32_t *arow;    // grouped row -> activation row (nullptr: the grouped row itself)
    const int32_t *goff;    // [groups + 1] first grouped row of every group
    const int32_t *gexp;    // [groups] expert id
    const int32_t *ngroups; // number of groups (device)
    const int32_t *gbig;    // the group with the most rows (device): every one of its passes gets workgroups of its own
    int regular;            // workgroups of the regular part of the grid (groups x matrices x row blocks)
    int extra_sets;         // passes of the largest group beyond the first (0: it is a regular group like the others)
    float *out[2];          // [grouped rows][rows]
    int n_mats, row_blocks;
};

// e4m3 codes of the two parts of four int8 values: q = 16 a + b.  Table look-up with v_perm: entries 0-7 and 8-15 of
// a 16-entry byte table, selected by bit 3 of the index.
__device__ __forceinline__ uint32_t qx_lut16(uint32_t idx, uint32_t t0, uint32_t t1, uint32_t t2, uint32_t t3) {
    const uint32_t sel = idx & 0x07070707u;
    const uint32_t lo = __builtin_amdgcn_perm(t1, t0, sel), hi = __builtin_amdgcn_perm(t3, t2, sel);
    const uint32_t m = ((idx >> 3) & 0x01010101u) * 0xFFu;
    return (hi & m) | (lo & ~m);
}
__device__ __forceinline__ void qx_split(uint32_t q4, uint32_t &a_codes, uint32_t &b_codes) {
    // b = q & 15: 0 .. 15 -> 0, 1, 2, 3, 4, 5, 6, 7 | 8 .. 15
    b_codes = qx_lut16(q4 & 0x0F0F0F0Fu, 0x44403800u, 0x4E4C4A48u, 0x53525150u, 0x57565554u);
    // a = q >> 4 (arithmetic) as a 4-bit two's complement index: 0 .. 7 | -8 .. -1
    a_codes = qx_lut16((q4 >> 4) & 0x0F0F0F0Fu, 0x44403800u, 0x4E4C4A48u, 0xCACCCED0u, 0xB8C0C4C8u);
}

// One pass: up to QX_TOK tokens (NP pairs) of a group against the workgroup's 256 rows.
template <int NP, int WAVES>
__device__ __forceinline__ void q8x_pass(const Q8xArgs &a, const uint8_t *packed, const uint8_t *scales, const uint8_t *scales_t, float *out, int rb,
                                         int base, int tok1, uint8_t *lds) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, kb = lane >> 4;
    const int cols = a.cols, nb = cols / 32, ktiles = cols / 512;
    const int row0 = rb * (64 * WAVES) + wave * 64;
    // weight loads: whole 128-byte lines (8 rows x 128 bytes per load), see gemm_mxfp4.hip
    const int r3 = lane >> 3, c8 = lane & 7;
    uint32_t woff[4][2];
#pragma unroll
    for (int rt = 0; rt < 4; rt++)
#pragma unroll
        for (int h = 0; h < 2; h++) woff[rt][h] = (uint32_t)min(row0 + rt * 16 + 8 * h + r3, a.rows - 1) * (uint32_t)(cols / 2) + c8 * 16;
    const int rot_idx = (((lane & 7) << 3) | (((lane >> 3) & 1) << 2) | (lane >> 4)) * 4;
    const bool ws_tiles = scales_t != nullptr;  // (uniform)
    const uint8_t *ws_base = ws_tiles ? scales_t : scales;
    const uint32_t ws_r = (uint32_t)min(rb * (64 * WAVES) + tid, a.rows - 1);
    const uint32_t wsoff = ws_tiles ? ws_r * 16u : ws_r * (uint32_t)nb, ws_step = ws_tiles ? (uint32_t)a.rows * 16u : 16u;

    // this lane as a column of the instruction: token t2 of the pair, phase p, part (0: a codes, 1: b codes)
    const int t2 = n >> 3, ph = (n >> 1) & 3, part = n & 1;
    // 8-bit operand layout: lane group kb holds K bytes 16 kb .. (registers 0-3) and 64 + 16 kb .. (registers 4-7), so
    // K block ph lives in registers (ph >> 1) of the lane groups 2 (ph & 1), 2 (ph & 1) + 1
    // A lane whose register half holds none of its column's block reads that half from a region of zeros instead
    // (all such lanes the same address: a broadcast), which saves masking the operand: 8 instructions per matrix
    // instruction.
    const bool active = (ph & 1) == (kb >> 1);
    const bool has_lo = active && ph < 2, has_hi = active && ph >= 2;
    const int bscale = part ? 127 : 131;  // e8m0 of the column's blocks: 2^0 for the b codes, 2^4 for the a codes
    const uint32_t a_lane_off = (uint32_t)(t2 * QX_TOK_STRIDE + part * QX_ROW + ph * 32 + (kb & 1) * 16);
    const uint32_t dx_lane_off = (uint32_t)(QX_DX_OFF + t2 * 64 + ph * 4);

    const int ntok = min(2 * NP, tok1 - base);
    const int npair = (ntok + 1) >> 1;
    // staging: thread -> token tid / 32, 16-byte chunk tid % 32 of the K tile's 512 int8 values
    const int stok = min(tid >> 5, 2 * NP - 1), sch = tid & 31;
    const bool stager = tid < 2 * NP * 32;
    const int srow_i = base + min(stok, ntok - 1);
    const uint32_t srow = (uint32_t)(a.arow ? a.arow[srow_i] : srow_i);
    const uint32_t qoff = srow * (uint32_t)cols + sch * 16, dxoff = srow * (uint32_t)nb;
    mk_i4 stq, stw;
    float stdx;
    auto stage_load = [&](int kt) __attribute__((always_inline)) {
        const uint32_t ku = (uint32_t)__builtin_amdgcn_readfirstlane(min(kt, ktiles - 1));
        stq = mk_ldg128_off(a.xq, qoff + ku * 512);
        stw = mk_ldg128_off(ws_base, wsoff + ku * ws_step);
        stdx = mk_ldg_f32_off(a.xs, (dxoff + ku * 16 + (sch & 15)) * 4);  // unconditional: a load under a branch forces a full wait
    };
    auto stage_store = [&](uint8_t *buf) __attribute__((always_inline)) {
        mk_i4 ca, cb;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            uint32_t ac, bc;
            qx_split((uint32_t)stq[k], ac, bc);
            ca[k] = (int)ac;
            cb[k] = (int)bc;
        }
        if (stok >= ntok) ca = cb = mk_i4{0, 0, 0, 0};
        if (stager) {
            *reinterpret_cast<mk_i4 *>(buf + stok * QX_TOK_STRIDE + sch * 16) = ca;
            *reinterpret_cast<mk_i4 *>(buf + stok * QX_TOK_STRIDE + QX_ROW + sch * 16) = cb;
            if (sch < 16) *reinterpret_cast<float *>(buf + QX_DX_OFF + stok * 64 + sch * 4) = stok < ntok ? stdx : 0.0f;
        }
        *reinterpret_cast<mk_i4 *>(buf + QX_WSC_OFF + tid * 16) = stw;
    };

    mk_i4 wa[QX_STEPS], wb[QX_STEPS];
    auto load_unit = [&](mk_i4 *w, int kt, int rt) __attribute__((always_inline)) {
        const uint32_t ku = (uint32_t)__builtin_amdgcn_readfirstlane(min(kt, ktiles - 1));
#pragma unroll
        for (int j = 0; j < QX_STEPS; j++) w[j] = mk_ldg128_off_nt(packed, woff[rt][j & 1] + ku * (QX_STEPS * 64) + (j >> 1) * 128);
    };
    mk_f4 acc[4][NP];
#pragma unroll
    for (int rt = 0; rt < 4; rt++)
#pragma unroll
        for (int c = 0; c < NP; c++) acc[rt][c] = mk_f4{0.0f, 0.0f, 0.0f, 0.0f};

    auto compute_unit = [&](const mk_i4 *wl, int rt, const uint8_t *buf, const uint8_t *plo, const uint8_t *phi) __attribute__((always_inline)) {
        // operand form of the unit's two lines (see gemm_mxfp4.hip): lane rotation, then the half-row exchange
        mk_i4 w[QX_STEPS];
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int ra = __builtin_amdgcn_ds_bpermute(rot_idx, wl[2 * i][k]), rb2 = __builtin_amdgcn_ds_bpermute(rot_idx, wl[2 * i + 1][k]);
                w[2 * i][k] = __builtin_amdgcn_update_dpp(ra, rb2, 0x128 /* row_ror:8 */, 0xF, 0xC, false);
                w[2 * i + 1][k] = __builtin_amdgcn_update_dpp(rb2, ra, 0x128 /* row_ror:8 */, 0xF, 0x3, false);
            }
        const mk_i4 sc = *reinterpret_cast<const mk_i4 *>(buf + QX_WSC_OFF + (wave * 64 + rt * 16 + n) * 16);
        // A matrix instruction's result is taken out after the next one has been issued, so that its latency is covered.
        mk_f4 tp[NP];
        float dp[NP];
#pragma unroll
        for (int s = 0; s <= QX_STEPS; s++) {
#pragma unroll
            for (int c = 0; c < NP; c++) {
                if (c < npair) {
                    mk_f4 tc = {0.0f, 0.0f, 0.0f, 0.0f};
                    float dc = 0.0f;
                    if (s < QX_STEPS) {
                        const mk_i8v wv = {w[s & 3][0], w[s & 3][1], w[s & 3][2], w[s & 3][3], 0, 0, 0, 0};
                        const int wsb = (int)((uint32_t)sc[s & 3] >> (8 * kb));
                        const mk_i4 dl = *reinterpret_cast<const mk_i4 *>(plo + c * 2 * QX_TOK_STRIDE + (s & 3) * 128);
                        const mk_i4 dh = *reinterpret_cast<const mk_i4 *>(phi + c * 2 * QX_TOK_STRIDE + (s & 3) * 128);
                        dc = *reinterpret_cast<const float *>(buf + dx_lane_off + c * 128 + (s & 3) * 16);
                        const mk_i8v av = {dl[0], dl[1], dl[2], dl[3], dh[0], dh[1], dh[2], dh[3]};
                        tc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wv, av, mk_f4{0.0f, 0.0f, 0.0f, 0.0f}, 4 /*M: fp4 weights*/,
                                                                              0 /*N: e4m3 codes*/, 0, wsb, 0, bscale);
                    }
                    if (s > 0) {
#pragma unroll
                        for (int r = 0; r < 4; r++) {
                            // the a and the b part of the block sit in neighbouring lanes: exact sum, then the block term
                            const float both = tp[c][r] + mk_dpp<0xB1>(tp[c][r]);  // quad_perm [1, 0, 3, 2]
                            acc[rt][c][r] += both * dp[c];
                        }
                    }
                    tp[c] = tc;
                    dp[c] = dc;
                }
            }
        }
    };

    load_unit(wa, 0, 0);
    stage_load(0);
    __syncthreads();  // the previous pass (if any) has finished with the LDS buffers
    stage_store(lds);
    __syncthreads();
#pragma unroll 1
    for (int kt = 0; kt < ktiles; kt++) {
        const uint8_t *buf = lds + (kt & 1) * QX_BUF;
        const uint8_t *plo = has_lo ? buf + a_lane_off : lds + QX_ZERO_OFF, *phi = has_hi ? buf + a_lane_off : lds + QX_ZERO_OFF;
        stage_load(kt + 1);
        load_unit(wb, kt, 1);
        compute_unit(wa, 0, buf, plo, phi);
        load_unit(wa, kt, 2);
        compute_unit(wb, 1, buf, plo, phi);
        load_unit(wb, kt, 3);
        compute_unit(wa, 2, buf, plo, phi);
        load_unit(wa, kt + 1, 0);
        compute_unit(wb, 3, buf, plo, phi);
        stage_store(lds + ((kt + 1) & 1) * QX_BUF);
        __syncthreads();
    }
    // the four phases of a token are the lanes n ^ 2, n ^ 4 (and n ^ 6): sum them, then the lane of phase 0, part 0 stores
    // four consecutive weight rows of its token
#pragma unroll
    for (int rt = 0; rt < 4; rt++)
#pragma unroll
        for (int c = 0; c < NP; c++) {
            if (c >= npair) continue;
            mk_f4 v = acc[rt][c];
#pragma unroll
            for (int r = 0; r < 4; r++) {
                v[r] += mk_dpp<0x4E>(v[r]);  // quad_perm [2, 3, 0, 1]: lane ^ 2
                v[r] += __shfl_xor(v[r], 4, MK_WAVE);
            }
            const int tok = base + 2 * c + t2, row = row0 + rt * 16 + kb * 4;
            if ((n & 7) == 0 && tok < tok1) {
                float *dst = out + (size_t)tok * a.rows + row;
                if (row + 3 < a.rows && ((reinterpret_cast<uintptr_t>(dst) & 15) == 0)) {
                    *reinterpret_cast<mk_f4 *>(dst) = v;
                } else {
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        if (row + r < a.rows) dst[r] = v[r];
                }
            }
        }
}

// WAVES: 4 (a workgroup owns 256 rows) or 2 (128 rows: twice as many, shorter workgroups).
template <int WAVES>
__global__ __launch_bounds__(64 * WAVES) __attribute__((amdgpu_waves_per_eu(3))) void q8x_grouped_kernel(Q8xArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int per_group = a.n_mats * a.row_blocks;
    // The group with the most rows (in a decode batch the shared expert, which has every token) comes first and has one
    // workgroup per (matrix, row block, pass): workgroup ids go round the eight XCDs in turn, so the passes of a row block
    // get ids 8 apart -- same XCD, dispatched together -- and walk the same weight lines at the same time: one of them
    // fetches a line from HBM, the others find it in their XCD's L2.  Behind them the regular workgroups: (group, matrix,
    // row block), all passes of the group one after the other.
    int gi, r0, first_pass, pass_step;
    const int big = *a.gbig;
    const int passes = a.extra_sets + 1, nbig = a.extra_sets > 0 ? passes * ((per_group + 7) / 8 * 8) : 0;
    if ((int)blockIdx.x < nbig) {
        // (row blocks padded to whole sets of eight: the workgroups of the padding leave at once)
        const int x = blockIdx.x, blk = x / (8 * passes), in = x % (8 * passes);
        r0 = blk * 8 + (in & 7);
        if (r0 >= per_group) return;
        first_pass = in >> 3;
        gi = big;
        pass_step = 0x10000;  // whatever the group's size, every pass is taken by exactly one workgroup
    } else {
        const int x = blockIdx.x - nbig;
        gi = x / per_group;
        r0 = x % per_group;
        if (gi >= *a.ngroups || (gi == big && nbig > 0)) return;
        first_pass = 0;
        pass_step = 1;
    }
    const int m = r0 / a.row_blocks, rb = r0 % a.row_blocks;
    const int tok0 = a.goff[gi], tok1 = a.goff[gi + 1];
    const int e = a.gexp[gi];
    const uint8_t *packed = mk_uniform_ptr(a.packed_ptrs[m][e]);
    const uint8_t *scales = mk_uniform_ptr(a.scales_ptrs[m][e]);
    const uint8_t *scales_t = a.scales_t_ptrs[m] ? mk_uniform_ptr(a.scales_t_ptrs[m][e]) : nullptr;
    float *out = a.out[m];
    for (int i = threadIdx.x * 16; i < QX_LDS - QX_ZERO_OFF; i += 64 * WAVES * 16) *reinterpret_cast<mk_i4 *>(lds + QX_ZERO_OFF + i) = mk_i4{0, 0, 0, 0};
#pragma unroll 1
    for (int pass = first_pass; tok0 + QX_TOK * pass < tok1; pass += pass_step)
        q8x_pass<QX_TOK / 2, WAVES>(a, packed, scales, scales_t, out, rb, tok0 + QX_TOK * pass, tok1, lds);
}

}  // namespace

// All groups' rows against one (n_mats = 1) or two matrices per expert; see mk_common.h.
int mk_q8x_grouped(int n_mats, const uint8_t *const *const *packed_ptrs, const uint8_t *const *const *scales_ptrs, size_t rows, size_t cols,
                   const int8_t *xq, const float *xs, const int32_t *arow, const int32_t *goff, const int32_t *gexp, const int32_t *ngroups,
                   const int32_t *gbig, size_t max_groups, size_t max_group_rows, float *const *out, void *stream,
                   const uint8_t *const *const *scales_t_ptrs) {
    MK_REQUIRE(n_mats == 1 || n_mats == 2, "one or two matrices per group");
    MK_REQUIRE(cols % 512 == 0 && cols > 0 && rows >= 1, "cols must be a positive multiple of 512");
    MK_REQUIRE(rows * (cols / 2) < 0xFFFFFFFFull, "matrix too large for 32-bit byte offsets");
    Q8xArgs a{};
    for (int k = 0; k < n_mats; k++) {
        a.packed_ptrs[k] = packed_ptrs[k];
        a.scales_ptrs[k] = scales_ptrs[k];
        a.scales_t_ptrs[k] = scales_t_ptrs ? scales_t_ptrs[k] : nullptr;
        a.out[k] = out[k];
    }
    a.rows = (int)rows;
    a.cols = (int)cols;
    a.xq = xq;
    a.xs = xs;
    a.arow = arow;
    a.goff = goff;
    a.gexp = gexp;
    a.ngroups = ngroups;
    a.gbig = gbig;
    a.n_mats = n_mats;
    // 128-row workgroups (twice as many, shorter) measured the same as 256-row ones on the benchmark layer (472 / 466 us)
    const int waves = MK_TUNE("MK_Q8X_WAVES", 4);
    const size_t wg_rows = 64 * (size_t)waves;
    a.row_blocks = (int)((rows + wg_rows - 1) / wg_rows);
    const size_t passes = (max_group_rows + QX_TOK - 1) / QX_TOK;
    const size_t per_group = (size_t)n_mats * a.row_blocks;
    const size_t regular = max_groups * per_group, grid = regular + (passes > 1 ? passes : 0) * ((per_group + 7) / 8 * 8);
    MK_REQUIRE(passes >= 1 && grid < 0x7FFFFFFFull, "too many workgroups");
    a.regular = (int)regular;
    a.extra_sets = (int)(passes - 1);
    if (waves == 2) {
        const int s = mk_lds_opt_in(reinterpret_cast<const void *>(q8x_grouped_kernel<2>), QX_LDS);
        if (s != MK_OK) return s;
        hipLaunchKernelGGL(q8x_grouped_kernel<2>, dim3((unsigned)grid), dim3(128), QX_LDS, (hipStream_t)stream, a);
    } else {
        const int s = mk_lds_opt_in(reinterpret_cast<const void *>(q8x_grouped_kernel<4>), QX_LDS);
        if (s != MK_OK) return s;
        hipLaunchKernelGGL(q8x_grouped_kernel<4>, dim3((unsigned)grid), dim3(256), QX_LDS, (hipStream_t)stream, a);
    }
    return mk_launch_status("q8x_grouped");
}

namespace {
// the description of one group of m rows on expert 0, written where the grouped kernel expects device arrays
__global__ void q8x_one_group_kernel(const uint8_t *packed, const uint8_t *scales, int m, uint8_t *ws) {
    if (threadIdx.x != 0) return;
    *reinterpret_cast<const uint8_t **>(ws) = packed;
    *reinterpret_cast<const uint8_t **>(ws + 8) = scales;
    int32_t *w = reinterpret_cast<int32_t *>(ws + 16);
    w[0] = 0;  // goff[0]
    w[1] = m;  // goff[1]
    w[2] = 0;  // gexp[0]
    w[3] = 1;  // ngroups
    w[4] = 0;  // the largest group
}
}  // namespace

extern "C" int mk_dev_mxfp4_matvec_q8_batched(const uint8_t *packed, const uint8_t *scales, size_t rows, size_t cols, const int8_t *xq,
                                              const float *xs, size_t m, void *workspace, float *out, void *stream) {
    MK_REQUIRE(packed && scales && xq && xs && workspace && out, "null pointer");
    MK_REQUIRE(cols % 512 == 0 && cols > 0 && rows >= 1 && rows <= 0x7FFFFF00u, "cols must be a positive multiple of 512");
    MK_REQUIRE(m <= 65535 && m * cols < 0xFFFFFFFFull, "too many activation rows");
    MK_REQUIRE(((uintptr_t)packed & 15) == 0 && ((uintptr_t)xq & 15) == 0 && ((uintptr_t)scales & 15) == 0 && ((uintptr_t)workspace & 255) == 0,
               "packed, scales and xq must be 16-byte aligned, the workspace 256-byte aligned");
    if (m == 0) return MK_OK;
    uint8_t *ws = (uint8_t *)workspace;
    hipLaunchKernelGGL(q8x_one_group_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, packed, scales, (int)m, ws);
    const int s = mk_launch_status("q8x_one_group");
    if (s != MK_OK) return s;
    const uint8_t *const *pp = reinterpret_cast<const uint8_t *const *>(ws);
    const uint8_t *const *sp = reinterpret_cast<const uint8_t *const *>(ws + 8);
    const int32_t *w = reinterpret_cast<const int32_t *>(ws + 16);
    return mk_q8x_grouped(1, &pp, &sp, rows, cols, xq, xs, nullptr, w, w + 2, w + 3, w + 4, 1, m, &out, stream, nullptr);
}
