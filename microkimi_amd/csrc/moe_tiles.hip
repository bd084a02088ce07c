// MoE decode layer in ONE streaming launch (plus a small reduction): the expert section of moe_forward / ds_moe
// (src/model.rs:2227-2264,2346-2351; src/deepseek.rs:1069-1106) for a few decode tokens, q8 mode.
//
// The two-launch form (moe.hip) has a grid-wide dependency between gate/up and down: every row of W2 needs the whole
// activation row.  matvec_packed re-quantizes its input per 32 (src/mxfp4.rs:476-487, src/q8.rs:49-69), so a q8 block of
// the activation row is self-contained: it is made of 32 consecutive rows of W1 and W3, and it meets W2 in 32
// consecutive columns only.  A workgroup therefore owns (pair, 64 rows = two blocks): it streams those rows of W1 and
// W3, forms the 64 activation values and their two q8 blocks, and multiplies them straight into the matching 64 columns
// of W2,
//     part[pair][g][r] = idot(W2[r][64g .. 64g+31], q_2g) * (2^(sb-128) * dx_2g) + idot(W2[r][64g+32 ..], q_2g+1) * (...),
// the reference's block terms (src/mxfp4.rs:405-443).  A second, small kernel adds the 64-column groups of a pair in
// ascending order (o = W2 act as a fixed-order sum of the reference's terms) and then the token's pairs in slot order,
// y += w * o (src/model.rs:2346-2351).  No atomics, no flags: the result is deterministic.
//
// Arithmetic.  v_mfma_scale_f32_16x16x128_f8f6f4 with the MXFP4 weights as stored (16 rows x four 32-blocks, e8m0 byte a
// lane) and the q8 activation as exact e4m3 codes, q = 16 a + b with a in [-8, 7] and b in [0, 15] (gemm_q8x.hip): a
// column is (block phase, part) and holds the a codes (block scale 2^4) or the b codes of ONE block and zeros in the
// other three, so a result is w_scale * sum w (16 a) or w_scale * sum w b of that single block, exact; the two parts
// are added (exact), multiplied by the f32 block scale dx (the one rounding of the reference's term) and accumulated
// in f32.  On the vector unit the same work is one conversion and one dot instruction per two weights, which made
// this kernel issue-bound at one or two waves a SIMD (measured: 51 us with the vector unit 42 % busy and the
// workgroups that share a CU taking twice as long).
//
// Layout.  The row-major matrices would be read as 64-byte pieces of 16 rows (the operand's form), and 64 columns of
// W2 are 32 bytes out of every row.  The three matrices are therefore kept a second time in the operand's own order
// (mk_dev_mxfp4_to_tiles): a CHUNK is what one matrix instruction takes, 64 lanes x 16 bytes (lane l = n + 16 kb holds
// one 32-block of row n) with one scale byte a lane; two chunks and their scale bytes make a 2176-byte container (17
// whole lines: chunk k at k * 1024, the scale byte of lane l at 2048 + 2 l + k).
//   W1, W3 (col_major = 0): chunk (rt, s) = rows 16 rt .. + 15, columns 128 s .. + 127 (lane (n, kb): row 16 rt + n, block
//     4 s + kb), chunks of a row tile contiguous along K.
//   W2 (col_major = 1): chunk (g, rt) = rows 32 rt .. + 31, columns 64 g .. + 63 (lane (n, kb): row 32 rt + 16 (kb >> 1) + n,
//     block 2 g + (kb & 1)), chunks of a 64-column group contiguous along the rows: one instruction multiplies 32 rows
//     by the two activation blocks of the group.
#include "mk_moe.h"

namespace {

constexpr int TC_BYTES = 2176;  // a container: two chunks of 1 KiB and 64 x 2 scale bytes

__device__ __forceinline__ void mk_lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// chunk index and lane of (row r, block b)
__device__ __forceinline__ void tile_place(int r, int b, int rows, int nb, int col_major, size_t &chunk, int &lane) {
    if (col_major) {
        chunk = (size_t)(b >> 1) * (rows >> 5) + (r >> 5);
        lane = (r & 15) + 16 * (2 * ((r >> 4) & 1) + (b & 1));
    } else {
        chunk = (size_t)(r >> 4) * (nb >> 2) + (b >> 2);
        lane = (r & 15) + 16 * (b & 3);
    }
}

// ------------------------------------------------------------------ layout
// thread = (row r, block b), b fastest: 16-byte reads along a row are coalesced
__global__ __launch_bounds__(256) void mxfp4_to_tiles_kernel(const uint8_t *__restrict__ packed, const uint8_t *__restrict__ scales, int rows,
                                                             int nb, int col_major, uint8_t *__restrict__ tiles) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)rows * nb) return;
    const int r = (int)(i / nb), b = (int)(i % nb);
    size_t chunk;
    int lane;
    tile_place(r, b, rows, nb, col_major, chunk, lane);
    uint8_t *dst = tiles + (chunk >> 1) * TC_BYTES;
    const int k = (int)(chunk & 1);
    *reinterpret_cast<mk_i4 *>(dst + k * 1024 + lane * 16) = *reinterpret_cast<const mk_i4 *>(packed + ((size_t)r * nb + b) * 16);
    dst[2048 + lane * 2 + k] = scales[(size_t)r * nb + b];
}

// mxfp4::dequant (src/mxfp4.rs:19-31) read from the tiled copy: thread = 8 consecutive columns of a row
__global__ __launch_bounds__(256) void mxfp4_tiles_dequant_kernel(const uint8_t *__restrict__ tiles, int rows, int nb, int col_major,
                                                                  float *__restrict__ out) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)rows * nb * 4) return;
    const int r = (int)(i / (nb * 4)), wi = (int)(i % (nb * 4)), b = wi >> 2, dd = wi & 3;
    size_t chunk;
    int lane;
    tile_place(r, b, rows, nb, col_major, chunk, lane);
    const uint8_t *src = tiles + (chunk >> 1) * TC_BYTES;
    const int k = (int)(chunk & 1);
    const uint32_t w = *reinterpret_cast<const uint32_t *>(src + k * 1024 + lane * 16 + dd * 4);
    const float s = mk_scale_from_byte(src[2048 + lane * 2 + k]);
    mk_f4 lo, hi;
    lo.x = mk_e2m1(w & 15u) * s;
    lo.y = mk_e2m1((w >> 4) & 15u) * s;
    lo.z = mk_e2m1((w >> 8) & 15u) * s;
    lo.w = mk_e2m1((w >> 12) & 15u) * s;
    hi.x = mk_e2m1((w >> 16) & 15u) * s;
    hi.y = mk_e2m1((w >> 20) & 15u) * s;
    hi.z = mk_e2m1((w >> 24) & 15u) * s;
    hi.w = mk_e2m1((w >> 28) & 15u) * s;
    mk_f4 *o = reinterpret_cast<mk_f4 *>(out + i * 8);
    o[0] = lo;
    o[1] = hi;
}

// e4m3 codes of the two parts of four int8 values, q = 16 a + b (as gemm_q8x.hip): a 16-entry byte table through v_perm
__device__ __forceinline__ uint32_t tl_lut16(uint32_t idx, uint32_t t0, uint32_t t1, uint32_t t2, uint32_t t3) {
    const uint32_t sel = idx & 0x07070707u;
    const uint32_t lo = __builtin_amdgcn_perm(t1, t0, sel), hi = __builtin_amdgcn_perm(t3, t2, sel);
    const uint32_t m = ((idx >> 3) & 0x01010101u) * 0xFFu;
    return (hi & m) | (lo & ~m);
}
__device__ __forceinline__ void tl_split(uint32_t q4, uint32_t &a_codes, uint32_t &b_codes) {
    b_codes = tl_lut16(q4 & 0x0F0F0F0Fu, 0x44403800u, 0x4E4C4A48u, 0x53525150u, 0x57565554u);         // b = q & 15: 0 .. 15
    a_codes = tl_lut16((q4 >> 4) & 0x0F0F0F0Fu, 0x44403800u, 0x4E4C4A48u, 0xCACCCED0u, 0xB8C0C4C8u);  // a = q >> 4: 0 .. 7 | -8 .. -1
}
// q8 of four values of a block held by 8 lanes (src/q8.rs:57-68): the block scale and the packed int8 values
__device__ __forceinline__ uint32_t tl_q8_pack4(const mk_f4 v, float &dx) {
    float mx = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    mx = fmaxf(mx, mk_dpp<0xB1>(mx));
    mx = fmaxf(mx, mk_dpp<0x4E>(mx));
    mx = fmaxf(mx, mk_dpp<0x141>(mx));
    dx = fmaxf(mx, 0.0f) / 127.0f;  // (a block of NaN only: the reference's maximum, folded from 0, is 0)
    if (dx == 0.0f) return 0u;
    float qf[4];
    mk_q8_round4(v, dx, qf);
    return ((uint32_t)(int)qf[0] & 255u) | (((uint32_t)(int)qf[1] & 255u) << 8) | (((uint32_t)(int)qf[2] & 255u) << 16) | ((uint32_t)(int)qf[3] << 24);
}

// ------------------------------------------------------------------ the streaming kernel
// Workgroup (pair q, 64-row group g) of four waves; NB = d / 32.
//   phase 1  wave w owns the rows 64 g + 16 w .. + 15 of W1 and of W3 over all of K: NB / 4 steps of one matrix instruction
//            each, against the token's hidden row, whose q8 codes the workgroup makes itself in LDS while its first
//            weight loads are in flight.  A lane is the column (block phase, part) of the instruction and reads its 16
//            code bytes of the step (or zeros) from LDS; its four results are rows 4 kb .. 4 kb + 3.
//   phase 2  every wave forms the two q8 blocks of the 64 activation values (the same bytes in every wave) and holds its
//            operand of them in registers; wave w walks NB / 4 chunks of the column group g of W2 (32 rows an
//            instruction) and stores the partial values.  The first of these chunks are requested while phase 1's last
//            steps are worked on.
struct Cont {  // a lane's share of a container: two chunks and their scale bytes
    mk_i4 w[2];
    uint32_t sc;
};
struct Unit {
    Cont a, u;  // the same container (two K steps) of W1 and of W3
};

constexpr int X_ROWB_PAD = 16;  // the b-code row starts 4 banks behind the a-code row

template <int NB, int R1, int R2>
__global__ __launch_bounds__(256) void moe_tiles_kernel(FusedArgs a, int stage, float *__restrict__ part) {
    constexpr int D = NB * 32;
    constexpr int NS = NB / 4;  // K steps of phase 1 per wave = chunks of phase 2 per wave
    constexpr int NU = NS / 2;  // containers per wave and matrix
    constexpr int NX = NB * 8;  // 16-byte pieces of a hidden row
    constexpr int SB = NX / 256;
    constexpr int ROWB = D + X_ROWB_PAD;
    static_assert(NB % 32 == 0 && NU % R1 == 0 && NU % R2 == 0 && R2 <= 2 * R1, "shape not covered");
    // codes of the hidden row: the a row, the b row; then zeros (what an idle half of the operand reads)
    __shared__ __attribute__((aligned(16))) uint8_t xc[2 * ROWB + 32];
    __shared__ float xsc[NB];
    __shared__ __attribute__((aligned(16))) float act_l[64];
    __shared__ __attribute__((aligned(16))) uint8_t ac[4][160];  // per wave: a codes [64], b codes [64], zeros [32]

    const int lane = threadIdx.x & 63, n = lane & 15, kb = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int G = a.inter >> 6;
    const int q = blockIdx.x / G, g = blockIdx.x - q * G;
    const int tok = q / a.per, slot = q - tok * a.per;
    bool ok = true;
    const int e = __builtin_amdgcn_readfirstlane(slot < a.topk ? mk_checked_expert(a.ids[tok * a.topk + slot], a.tab.n_experts, ok) : a.shared);
    const uint8_t *w2t = mk_uniform_ptr(a.tab.w2t[e]);

    // this lane as a column of the instruction: phase ph (the K block of the step), part (0: a codes, 1: b codes); the
    // columns 8 .. 15 stay empty (one token).  8-bit operand: lane group kb holds the K bytes 16 kb .. (registers 0-3)
    // and 64 + 16 kb .. (registers 4-7), so block ph lives in registers 4 (ph >> 1) .. of the lane groups 2 (ph & 1), + 1.
    const int ph = (n >> 1) & 3, pt = n & 1;
    const bool active = n < 8 && (ph & 1) == (kb >> 1);
    const bool has_lo = active && ph < 2, has_hi = active && ph >= 2;
    const int bscale = pt ? 127 : 131;  // e8m0 of the column: 2^0 for the b codes, 2^4 for the a codes

    auto load_cont = [&](Cont &c, const uint8_t *base, uint32_t off) {
        c.w[0] = mk_ldg128_off_nt(base, off + lane * 16);
        c.w[1] = mk_ldg128_off_nt(base, off + 1024 + lane * 16);
        c.sc = __builtin_nontemporal_load((const MK_GLOBAL uint16_t *)((const MK_GLOBAL uint8_t *)base + off + 2048 + lane * 2));
    };
    auto mfma = [&](const mk_i4 w, uint32_t wsb, const mk_i4 lo, const mk_i4 hi) {
        const mk_i8v wv = {w[0], w[1], w[2], w[3], 0, 0, 0, 0};
        const mk_i8v av = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wv, av, mk_f4{0.0f, 0.0f, 0.0f, 0.0f}, 4 /* fp4 weights */, 0 /* e4m3 codes */, 0,
                                                                (int)wsb, 0, bscale);
    };
    Cont it[R2];
    const uint32_t off2 = (uint32_t)((g * (NB / 2) + wave * NU) * TC_BYTES);  // W2: column group g, this wave's chunks
    float *dst = part + (size_t)blockIdx.x * D + (size_t)(wave * NS) * 32;

    if (stage != MK_MOE_STAGE_FROM_ACT) {
        // q8 of the hidden row (src/q8.rs:57-68): 8 lanes per 32-block, one 16-byte load each, requested first
        const mk_f4 *xsrc = reinterpret_cast<const mk_f4 *>(a.x + (size_t)tok * D);
        mk_f4 xv[SB];
#pragma unroll
        for (int b = 0; b < SB; b++) xv[b] = xsrc[threadIdx.x + b * 256];
        const float wgt = slot < a.topk ? (ok ? a.weights[tok * a.topk + slot] : 0.0f) : 1.0f;
        const uint8_t *p1 = mk_uniform_ptr(a.tab.w1t[e]), *p3 = mk_uniform_ptr(a.tab.w3t[e]);
        const uint32_t off1 = (uint32_t)(((4 * g + wave) * NU) * TC_BYTES);  // W1 / W3: row tile 4 g + wave
        Unit ring[R1];
        auto load_unit = [&](Unit &U, int u) {
            load_cont(U.a, p1, off1 + u * TC_BYTES);
            load_cont(U.u, p3, off1 + u * TC_BYTES);
        };
#pragma unroll
        for (int k = 0; k < R1; k++) load_unit(ring[k], k);
        if (threadIdx.x < 8) reinterpret_cast<uint32_t *>(xc + 2 * ROWB)[threadIdx.x] = 0u;
#pragma unroll
        for (int b = 0; b < SB; b++) {
            const int i = threadIdx.x + b * 256;  // piece i = values 4 (i & 7) .. + 3 of block i >> 3
            float dx;
            const uint32_t q4 = tl_q8_pack4(xv[b], dx);
            uint32_t ca, cb;
            tl_split(q4, ca, cb);
            *reinterpret_cast<uint32_t *>(xc + 4 * i) = ca;
            *reinterpret_cast<uint32_t *>(xc + ROWB + 4 * i) = cb;
            if ((i & 7) == 0) xsc[i >> 3] = dx;
        }
        mk_lds_barrier();

        const uint8_t *zero = xc + 2 * ROWB;
        const uint8_t *plo = has_lo ? xc + pt * ROWB + ph * 32 + (kb & 1) * 16 : zero, *phi = has_hi ? xc + pt * ROWB + ph * 32 + (kb & 1) * 16 : zero;
        const uint32_t klo = has_lo ? 128u : 0u, khi = has_hi ? 128u : 0u;  // an idle half keeps reading the zeros
        const float *pdx = xsc + (n < 8 ? ph : 0);
        mk_f4 accg = {0.0f, 0.0f, 0.0f, 0.0f}, accu = accg;
        mk_f4 tg = accg, tu = accg;  // the previous step's results, taken out after the next instructions are issued
        float dprev = 0.0f;
        auto step = [&](const Cont &ca, const Cont &cu, int k, int s) {
            const mk_i4 lo = *reinterpret_cast<const mk_i4 *>(plo + s * klo), hi = *reinterpret_cast<const mk_i4 *>(phi + s * khi);
            const float dcur = pdx[4 * s];
            const mk_f4 ng = mfma(ca.w[k], ca.sc >> (8 * k), lo, hi), nu = mfma(cu.w[k], cu.sc >> (8 * k), lo, hi);
#pragma unroll
            for (int r = 0; r < 4; r++) {
                // the a and the b part of the block sit in neighbouring lanes: exact sum, then the block term
                accg[r] = mk_add(accg[r], mk_mul(tg[r] + mk_dpp<0xB1>(tg[r]), dprev));
                accu[r] = mk_add(accu[r], mk_mul(tu[r] + mk_dpp<0xB1>(tu[r]), dprev));
            }
            tg = ng;
            tu = nu;
            dprev = dcur;
        };
#pragma unroll 1
        for (int u0 = 0; u0 < NU - R1; u0 += R1) {
#pragma unroll
            for (int k = 0; k < R1; k++) {
                step(ring[k].a, ring[k].u, 0, 2 * (u0 + k));
                step(ring[k].a, ring[k].u, 1, 2 * (u0 + k) + 1);
                load_unit(ring[k], u0 + k + R1);
            }
        }
#pragma unroll
        for (int k = 0; k < R1; k++) {
            step(ring[k].a, ring[k].u, 0, 2 * (NU - R1 + k));
            step(ring[k].a, ring[k].u, 1, 2 * (NU - R1 + k) + 1);
            if (2 * k < R2) load_cont(it[2 * k], w2t, off2 + 2 * k * TC_BYTES);
            if (2 * k + 1 < R2) load_cont(it[2 * k + 1], w2t, off2 + (2 * k + 1) * TC_BYTES);
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
            accg[r] = mk_add(accg[r], mk_mul(tg[r] + mk_dpp<0xB1>(tg[r]), dprev));
            accu[r] = mk_add(accu[r], mk_mul(tu[r] + mk_dpp<0xB1>(tu[r]), dprev));
            // the four phases are the lanes n ^ 2, n ^ 4 (and n ^ 6)
            accg[r] += mk_dpp<0x4E>(accg[r]);
            accu[r] += mk_dpp<0x4E>(accu[r]);
            accg[r] += __shfl_xor(accg[r], 4, MK_WAVE);
            accu[r] += __shfl_xor(accu[r], 4, MK_WAVE);
        }
        mk_f4 av;
#pragma unroll
        for (int r = 0; r < 4; r++) av[r] = mk_act(a.act_kind, accg[r], accu[r], a.limit, wgt);
        if (n == 0) {
            *reinterpret_cast<mk_f4 *>(act_l + 16 * wave + 4 * kb) = av;
            if (stage == MK_MOE_STAGE_ACT) *reinterpret_cast<mk_f4 *>(a.af + (size_t)q * a.inter + 64 * g + 16 * wave + 4 * kb) = av;
        }
        if (stage == MK_MOE_STAGE_ACT) return;
    } else {
#pragma unroll
        for (int k = 0; k < R2; k++) load_cont(it[k], w2t, off2 + k * TC_BYTES);
        if (threadIdx.x < 64) act_l[threadIdx.x] = a.af[(size_t)q * a.inter + 64 * g + threadIdx.x];
    }
    mk_lds_barrier();

    // q8 of the two activation blocks (what matvec_packed does to its input, src/q8.rs:57-68), in every wave: lanes
    // 8 b .. 8 b + 7 hold block b, four values each; the codes go through the wave's own piece of LDS into the operand
    mk_i4 blo, bhi;
    float dxl;
    {
        float dx;
        const uint32_t q4 = tl_q8_pack4(*reinterpret_cast<const mk_f4 *>(act_l + 4 * (lane & 15)), dx);
        uint32_t ca, cb;
        tl_split(q4, ca, cb);
        uint8_t *mine = ac[wave];
        if (lane < 16) {
            *reinterpret_cast<uint32_t *>(mine + 4 * lane) = ca;
            *reinterpret_cast<uint32_t *>(mine + 64 + 4 * lane) = cb;
        } else if (lane < 24) {
            *reinterpret_cast<uint32_t *>(mine + 128 + 4 * (lane - 16)) = 0u;
        }
        // a column here is (half of the 32 rows, block, part): the K block ph of the instruction is block ph & 1 of the
        // rows 16 (ph >> 1) ..
        dxl = mk_readlane(dx, 0);
        const float dx1 = mk_readlane(dx, 8);
        if (ph & 1) dxl = dx1;
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        const uint8_t *src = mine + pt * 64 + (ph & 1) * 32 + (kb & 1) * 16, *zero = mine + 128;
        blo = *reinterpret_cast<const mk_i4 *>(has_lo ? src : zero);
        bhi = *reinterpret_cast<const mk_i4 *>(has_hi ? src : zero);
    }

    mk_f4 tp = {0.0f, 0.0f, 0.0f, 0.0f};
    auto finish = [&](const mk_f4 t, int c) {  // chunk c of this wave: rows 32 c + 16 (ph >> 1) + 4 kb .. + 3
        mk_f4 y;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const float term = mk_mul(t[r] + mk_dpp<0xB1>(t[r]), dxl);  // the block term
            y[r] = term + mk_dpp<0x4E>(term);                            // block 2 g + block 2 g + 1 (lanes n ^ 2)
        }
        if ((n & 11) == 0) *reinterpret_cast<mk_f4 *>(dst + 32 * c + 16 * (ph >> 1) + 4 * kb) = y;
    };
    auto chunk2 = [&](const Cont &c, int u) {
        const mk_f4 t0 = mfma(c.w[0], c.sc, blo, bhi);
        if (u > 0) finish(tp, 2 * u - 1);
        const mk_f4 t1 = mfma(c.w[1], c.sc >> 8, blo, bhi);
        finish(t0, 2 * u);
        tp = t1;
    };
#pragma unroll 1
    for (int u0 = 0; u0 < NU - R2; u0 += R2) {
#pragma unroll
        for (int k = 0; k < R2; k++) {
            chunk2(it[k], u0 + k);
            load_cont(it[k], w2t, off2 + (u0 + k + R2) * TC_BYTES);
        }
    }
#pragma unroll
    for (int k = 0; k < R2; k++) chunk2(it[k], NU - R2 + k);
    finish(tp, 2 * NU - 1);
}

// out[t][r] = sum over the token's pairs in slot order of w * o, o = the pair's groups added in ascending order.
// grid (d / 64, B), block (64, per): thread (rl, s) adds the groups of pair (t, s) at row 64 blockIdx.x + rl.
__global__ __launch_bounds__(1024) void moe_tiles_reduce_kernel(FusedArgs a, const float *__restrict__ part, int G) {
    __shared__ float o_l[16][64];
    const int rl = threadIdx.x, s = threadIdx.y, t = blockIdx.y, per = a.per;
    const int row = blockIdx.x * 64 + rl;
    const float *src = part + ((size_t)(t * per + s) * G) * a.d + row;
    float o = 0.0f;
    int g = 0;
    for (; g + 8 <= G; g += 8) {
        float v[8];
#pragma unroll
        for (int k = 0; k < 8; k++) v[k] = src[(size_t)(g + k) * a.d];
#pragma unroll
        for (int k = 0; k < 8; k++) o = mk_add(o, v[k]);
    }
    for (; g < G; g++) o = mk_add(o, src[(size_t)g * a.d]);
    o_l[s][rl] = o;
    __syncthreads();
    if (s != 0) return;
    float y = 0.0f;
    for (int k = 0; k < per; k++) {
        float pw = 1.0f;
        if (k < a.topk) {
            bool ok = true;
            mk_checked_expert(a.ids[t * a.topk + k], a.tab.n_experts, ok);
            pw = !ok ? 0.0f : a.ds_rule ? 1.0f : a.weights[t * a.topk + k];
        }
        y = mk_add(y, mk_mul(pw, o_l[k][rl]));
    }
    a.out[(size_t)t * a.d + row] = y;
}

template <int NB, int R1, int R2>
int launch_tiles(const FusedArgs &a, size_t P, int stage, float *part, hipStream_t st) {
    const int extra_lds = MK_TUNE("MK_MOE_TILES_LDS", 0);  // (experiment: dynamic LDS that only limits the workgroups a CU takes)
    if (extra_lds > 0 && mk_lds_opt_in(reinterpret_cast<const void *>(moe_tiles_kernel<NB, R1, R2>), 140 * 1024) != MK_OK) return MK_ERR_HIP;
    hipLaunchKernelGGL((moe_tiles_kernel<NB, R1, R2>), dim3((unsigned)(P * (a.inter / 64))), dim3(256), (size_t)extra_lds, st, a, stage, part);
    return mk_launch_status("moe_tiles");
}

}  // namespace

bool mk_moe_tiles_takes(size_t d, size_t inter, int per) {
    const size_t nb = d / 32;
    return (nb == 32 || nb == 64 || nb == 128 || nb == 224) && inter % 64 == 0 && per <= 16 && inter * (d / 32) * 17 < 0x7FFFFFFFull;
}

size_t mk_moe_tiles_part_bytes(size_t P, size_t d, size_t inter) { return P * (inter / 64) * d * sizeof(float); }

int mk_moe_tiles_launch(const FusedArgs &a, size_t B, int stage, float *part, hipStream_t st) {
    const size_t P = B * a.per;
    int s;
    switch (a.d / 32) {
        case 32: s = launch_tiles<32, 4, 4>(a, P, stage, part, st); break;
        case 64: s = launch_tiles<64, 8, 8>(a, P, stage, part, st); break;
        case 128: s = launch_tiles<128, 8, 16>(a, P, stage, part, st); break;
        case 224: s = MK_TUNE("MK_MOE_TILES_R", 0) == 1 ? launch_tiles<224, 4, 7>(a, P, stage, part, st) : launch_tiles<224, 7, 14>(a, P, stage, part, st); break;
        default: mk_set_error("moe_tiles: d = %d not covered", a.d); return MK_ERR_UNSUPPORTED;
    }
    if (s != MK_OK || stage == MK_MOE_STAGE_ACT) return s;
    hipLaunchKernelGGL(moe_tiles_reduce_kernel, dim3((unsigned)(a.d / 64), (unsigned)B), dim3(64, a.per), 0, st, a, part, a.inter / 64);
    return mk_launch_status("moe_tiles_reduce");
}

extern "C" size_t mk_mxfp4_tiles_bytes(size_t rows, size_t cols) { return rows * (cols / 32) * 17; }

extern "C" int mk_dev_mxfp4_to_tiles(const uint8_t *packed, const uint8_t *scales, size_t rows, size_t cols, int col_major, uint8_t *tiles,
                                     void *stream) {
    MK_REQUIRE(packed && scales && tiles, "null pointer");
    MK_REQUIRE(rows > 0 && cols > 0 && (col_major ? rows % 64 == 0 && cols % 64 == 0 : rows % 16 == 0 && cols % 256 == 0),
               "rows % 16 == 0 and cols % 256 == 0 (col_major: both multiples of 64)");
    MK_REQUIRE(rows * (cols / 32) * 17 < 0x7FFFFFFFull, "matrix too large for the tiled form");
    MK_REQUIRE((((uintptr_t)packed | (uintptr_t)tiles) & 15) == 0, "packed and tiles must be 16-byte aligned");
    const size_t n = rows * (cols / 32);
    hipLaunchKernelGGL(mxfp4_to_tiles_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, packed, scales, (int)rows,
                       (int)(cols / 32), col_major ? 1 : 0, tiles);
    return mk_launch_status("mxfp4_to_tiles");
}

extern "C" int mk_dev_mxfp4_tiles_dequant(const uint8_t *tiles, size_t rows, size_t cols, int col_major, float *out, void *stream) {
    MK_REQUIRE(tiles && out, "null pointer");
    MK_REQUIRE(rows > 0 && cols > 0 && (col_major ? rows % 64 == 0 && cols % 64 == 0 : rows % 16 == 0 && cols % 256 == 0),
               "rows % 16 == 0 and cols % 256 == 0 (col_major: both multiples of 64)");
    MK_REQUIRE((((uintptr_t)tiles | (uintptr_t)out) & 15) == 0, "tiles and out must be 16-byte aligned");
    const size_t n = rows * (cols / 32) * 4;
    hipLaunchKernelGGL(mxfp4_tiles_dequant_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, tiles, (int)rows,
                       (int)(cols / 32), col_major ? 1 : 0, out);
    return mk_launch_status("mxfp4_tiles_dequant");
}
