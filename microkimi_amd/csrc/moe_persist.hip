// MoE decode layer in ONE launch: the expert section of moe_forward / ds_moe (src/model.rs:2227-2264,2346-2351;
// src/deepseek.rs:1069-1106) for up to three decode tokens, q8 mode, as one resident workgroup per CU that does an equal
// share of the gate/up rows and then an equal share of the down rows.
//
// Why this shape.  Measured on this part: a CU streams at most about 30 B/ns whatever its waves keep in flight, so the
// chip reaches its HBM rate only while every CU is busy, and a launch that touches HBM at all costs about 8 us of ramp
// and tail.  The layer at one token is 141 MB of gate/up weights and 70 MB of down weights with a dependency between
// them: two launches pay the ramp and tail twice (27 + 18 us), and one launch of self-contained (pair, 64 rows)
// workgroups has 288 or 576 unequal shares for 256 CUs (52 us).  Here the 256 workgroups stay for the whole layer:
//
//   phase 1  workgroup c owns the rows 8 c .. 8 c + 7 of W1 AND of W3 of every (token, slot) pair: one 16-row operand
//            of v_mfma_scale_f32_16x16x128_f8f6f4 holds the eight W1 rows and the eight W3 rows, so a workgroup has
//            the gate and the up value of its rows and forms ACT(g, u) itself.  Its four waves split K; the last
//            wave to finish a pair adds the four partial sums in wave order and PUBLISHES the eight activation
//            values: 8-byte units (value, launch tag), agent-scope stores into the caller's workspace.
//   phase 2  workgroup c owns the rows RW c .. RW c + RW - 1 of W2 (RW = d / 256) of every pair.  It reads a pair's 2048
//            units with agent-scope loads until every unit carries this launch's tag -- the data says when it is
//            there: no flag, no fence, no atomic read-modify-write between workgroups -- forms the q8 blocks of the
//            activation row exactly as matvec_packed does for its input (src/q8.rs:49-69), and multiplies.  Its waves
//            split K; the partial sums meet in LDS in wave order and a thread per row adds the pairs in slot order,
//            y += w * o (src/model.rs:2346-2351).  The units of the next pair are requested before the current pair is
//            worked on, and the first weights of phase 2 before the first units are awaited.
//
// Every wait is bounded (a workgroup that gives up raises a device flag and writes NaN to its rows), and the grid is
// the CU count with more than half a CU's LDS per workgroup: all workgroups are resident at once, so none waits for
// one that cannot start.  Calls that take this path must not overlap on one device (two such grids would hold each
// other's CUs); they are meant to be issued on one stream, layer after layer.
//
// Arithmetic: the reference's block terms (src/mxfp4.rs:405-443) on the matrix cores as in gemm_q8x.hip -- an int8
// activation is q = 16 a + b, a in [-8, 7], b in [0, 15], both exact in e4m3; a column of the instruction is (block
// phase, part) with the codes of ONE block, so a result is the exact integer dot of that block times the weight scale;
// the two parts are added (exact), multiplied by the f32 block scale (the reference's one rounding) and accumulated in
// f32.  Only the order of the sum over blocks differs from the CPU loop.
//
// Layout: the experts are kept a second time in the operand's order (mk_dev_moe_pack_gate_up / _down, table->w13t /
// w2t), so that every load instruction of a wave is one contiguous KiB and a workgroup's share is one stream.
#include "mk_moe.h"

namespace {

constexpr int PK_CONT = 2176;   // gate/up pack: two 1-KiB chunks and 64 x 2 scale bytes
constexpr int PK_GRID = 256;    // workgroups = CUs
constexpr int PK_MAX_P = 32;    // pairs per call

__device__ __forceinline__ void mk_lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// bytes of one K step (128 columns) of a row group of the down pack: tile A (16 rows), tile B (rb rows), their scale bytes
__host__ __device__ constexpr int pk_step_bytes(int rb) { return (1024 + 64 * rb + 64 + 4 * rb + 127) / 128 * 128; }

// launch counter of this device (the tag of a launch is its value + 1) and the give-up flag
__device__ unsigned g_moe_launch_ctr;
__device__ int g_moe_fail;
// -DMK_MOE_TRACE: every multiplying wave leaves time stamps (100 MHz) of the last launch, read with mk_debug_moe_ts:
// 0 start, 1 hidden rows staged, 2 phase 1 done, 3 first pair of phase 2 done, 4 time spent waiting for codes in phase 2,
// 5 end
#ifdef MK_MOE_TRACE
__device__ unsigned long long g_moe_ts[PK_GRID * 4 * 8];
#define TS(i) ts[i] = __builtin_amdgcn_s_memrealtime()
#else
#define TS(i)
#endif

// ------------------------------------------------------------------ layout kernels
// gate/up pack: chunk (t, s) = rows 8 t .. 8 t + 7 of W1 and of W3, columns 128 s .. + 127; lane = (row % 8 + 8 m) + 16 kb
// (m = 0: W1, 1: W3; kb = block % 4).  chunk index ci = t * (d / 128) + s; container ci >> 1, half ci & 1.
__device__ __forceinline__ size_t pk13_place(int m, int r, int b, int nb, int &lane, int &half) {
    const size_t ci = (size_t)(r >> 3) * (nb >> 2) + (b >> 2);
    lane = (r & 7) + 8 * m + 16 * (b & 3);
    half = (int)(ci & 1);
    return (ci >> 1) * PK_CONT;
}
// thread = (matrix m, row r, block b), b fastest
__global__ __launch_bounds__(256) void pack13_kernel(const uint8_t *p1, const uint8_t *s1, const uint8_t *p3, const uint8_t *s3, int inter, int nb,
                                                     uint8_t *pack, int unpack, uint8_t *o1, uint8_t *os1, uint8_t *o3, uint8_t *os3) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x, per = (size_t)inter * nb;
    if (i >= 2 * per) return;
    const int m = (int)(i / per), r = (int)((i % per) / nb), b = (int)(i % nb);
    int lane, half;
    uint8_t *at = pack + pk13_place(m, r, b, nb, lane, half);
    const size_t src = ((size_t)r * nb + b);
    if (!unpack) {
        *reinterpret_cast<mk_i4 *>(at + half * 1024 + lane * 16) = *reinterpret_cast<const mk_i4 *>((m ? p3 : p1) + src * 16);
        at[2048 + lane * 2 + half] = (m ? s3 : s1)[src];
    } else {
        *reinterpret_cast<mk_i4 *>((m ? o3 : o1) + src * 16) = *reinterpret_cast<const mk_i4 *>(at + half * 1024 + lane * 16);
        (m ? os3 : os1)[src] = at[2048 + lane * 2 + half];
    }
}
// down pack: group c = row / rw, i = row % rw, step s = block / 4, kb = block % 4; step (c, s) at (c * (inter / 128) + s) * STEP:
//   i < 16 : nibbles at 16 (i + 16 kb), scale byte at 1024 + 64 rb + (i + 16 kb)
//   i >= 16: nibbles at 1024 + 16 (kb rb + i - 16), scale byte at 1024 + 64 rb + 64 + kb rb + i - 16       (rb = rw - 16)
__global__ __launch_bounds__(256) void pack2_kernel(const uint8_t *p2, const uint8_t *s2, int d, int nbi, int rw, uint8_t *pack, int unpack,
                                                    uint8_t *o2, uint8_t *os2) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)d * nbi) return;
    const int r = (int)(i / nbi), b = (int)(i % nbi);
    const int rb = rw - 16, c = r / rw, ri = r - c * rw, s = b >> 2, kb = b & 3;
    uint8_t *at = pack + ((size_t)c * (nbi >> 2) + s) * pk_step_bytes(rb);
    const int noff = ri < 16 ? 16 * (ri + 16 * kb) : 1024 + 16 * (kb * rb + ri - 16);
    const int soff = 1024 + 64 * rb + (ri < 16 ? ri + 16 * kb : 64 + kb * rb + ri - 16);
    if (!unpack) {
        *reinterpret_cast<mk_i4 *>(at + noff) = *reinterpret_cast<const mk_i4 *>(p2 + i * 16);
        at[soff] = s2[i];
    } else {
        *reinterpret_cast<mk_i4 *>(o2 + i * 16) = *reinterpret_cast<const mk_i4 *>(at + noff);
        os2[i] = at[soff];
    }
}

// e4m3 codes of the two parts of four int8 values, q = 16 a + b (as gemm_q8x.hip): a 16-entry byte table through v_perm
__device__ __forceinline__ uint32_t pk_lut16(uint32_t idx, uint32_t t0, uint32_t t1, uint32_t t2, uint32_t t3) {
    const uint32_t sel = idx & 0x07070707u;
    const uint32_t lo = __builtin_amdgcn_perm(t1, t0, sel), hi = __builtin_amdgcn_perm(t3, t2, sel);
    const uint32_t m = ((idx >> 3) & 0x01010101u) * 0xFFu;
    return (hi & m) | (lo & ~m);
}
__device__ __forceinline__ void pk_split(uint32_t q4, uint32_t &a_codes, uint32_t &b_codes) {
    b_codes = pk_lut16(q4 & 0x0F0F0F0Fu, 0x44403800u, 0x4E4C4A48u, 0x53525150u, 0x57565554u);         // b = q & 15: 0 .. 15
    a_codes = pk_lut16((q4 >> 4) & 0x0F0F0F0Fu, 0x44403800u, 0x4E4C4A48u, 0xCACCCED0u, 0xB8C0C4C8u);  // a = q >> 4: 0 .. 7 | -8 .. -1
}
// q8 of four values of a block held by 8 lanes (src/q8.rs:57-68): the block scale and the packed int8 values
__device__ __forceinline__ uint32_t pk_q8_pack4(const mk_f4 v, float &dx) {
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

struct Cont13 {  // a lane's share of a gate/up container: two chunks and their scale bytes
    mk_i4 w[2];
    uint32_t sc;
};
struct Step2 {  // a lane's share of one K step of its row group of W2: tile A, tile B, their scale bytes
    mk_i4 wa, wb;
    uint32_t sa, sb;
};

struct PersistArgs {
    FusedArgs f;
    int B, stage, spin_limit;
    unsigned long long *lines;  // [P][inter] units (value bits | tag << 32)
};

// LDS map (bytes), D = hidden width
template <int D>
struct PLds {
    static constexpr int ROWB = D + 16;                 // the b-code row of a token starts 4 banks behind its a-code row
    static constexpr int XTOK = 2 * ROWB;               // codes of one token's hidden row
    static constexpr int ZERO_OFF = 0;                  // 32 bytes of zeros
    static constexpr int FLAG_OFF = 32;                 // ints: fail, -, -, -, ready[4], prog[4]
    static constexpr int PTR_OFF = FLAG_OFF + 64;       // p13 [32], p2 [32] pointers
    static constexpr int PW_OFF = PTR_OFF + 2 * PK_MAX_P * 8;    // pw [32] f32 (weight of the pair in the sum), wg [32] (weight inside ACT)
    static constexpr int CNT_OFF = PW_OFF + 2 * PK_MAX_P * 4;    // waves that finished the item, [32]
    static constexpr int PGU_OFF = CNT_OFF + PK_MAX_P * 4;       // [32 items][4 waves][16] f32 (the waves of a workgroup may be items apart)
    static constexpr int PO_OFF = PGU_OFF + PK_MAX_P * 4 * 16 * 4;   // [32 pairs][4 waves][32] f32
    static constexpr int XSC_OFF = PO_OFF + PK_MAX_P * 4 * 32 * 4;   // [B][D / 32] f32
    static constexpr int x_off(int B) { return XSC_OFF + B * (D / 32) * 4; }  // [B][XTOK]
    static constexpr int act_bytes(int inter) { return 2 * (inter + 16) + (inter / 32) * 4; }  // a codes, b codes, block scales of a pair
    static constexpr int act_off(int B) { return x_off(B) + B * XTOK; }                     // [RC][act_bytes]
    static constexpr int total(int B, int inter, int rc) { return act_off(B) + rc * act_bytes(inter); }
};

__device__ __forceinline__ int pk_lds_int(const int *p) { return __builtin_amdgcn_readfirstlane(*(const volatile int *)p); }
// the smallest of four counters in LDS (16-byte aligned), one read
__device__ __forceinline__ int pk_lds_min4(const int *p) {
    mk_i4 v;
    asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"((uint32_t)(uintptr_t)p) : "memory");
    return __builtin_amdgcn_readfirstlane(min(min(v[0], v[1]), min(v[2], v[3])));
}

// 512 threads: the waves 0-3 multiply (phase 1, then phase 2), the waves 4-7 carry the exchange between the workgroups
// (units -> q8 codes in LDS, ahead of the multiplying waves) and wave 4 then adds the pairs of the workgroup's rows.  The
// roles talk through counters in LDS (the LDS operations of a CU are performed in order: data first, then the counter);
// after the hidden rows are staged there is no workgroup barrier.  The exchange has waves of its own because a wave's
// loads return in order: a unit requested behind three pairs of prefetched weights would arrive behind them.
template <int D, int INTER, int STAGE>
__global__ __launch_bounds__(512) void moe_persist_kernel(PersistArgs pa, int RC) {
    using L = PLds<D>;
    constexpr int NB = D / 32;
    constexpr int RW = D / 256, RB = RW - 16;    // rows of W2 per workgroup; rows of its second tile
    constexpr int STEP = pk_step_bytes(RB);
    constexpr int NC = D / 256;                  // gate/up containers per 8-row tile
    constexpr int CW = NC / 4;                   // per wave
    constexpr int NX = NB * 8;                   // 16-byte pieces of a hidden row
    constexpr int SB = (NX + 511) / 512;         // per thread
    static_assert(D % 1024 == 0 && RB >= 1 && RB <= 16, "hidden width not covered");
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const FusedArgs &a = pa.f;
    const int lane = threadIdx.x & 63, n = lane & 15, kb = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = blockIdx.x, per = a.per, P = pa.B * per;
    constexpr int inter = INTER;
    constexpr int KI = INTER / (8 * PK_GRID);  // 8-row tiles of a pair per workgroup
    constexpr int NSI = INTER / 128;           // K steps of W2
    constexpr int SW = NSI / 4;                // per wave
    static_assert(INTER % (8 * PK_GRID) == 0 && INTER % 1024 == 0 && INTER <= 2048 && PK_MAX_P * KI <= 32, "intermediate width not covered");
    constexpr int stage = STAGE;  // (a run-time stage would put a branch around every unit load, and every wait behind a join is a full one)
    const uint32_t tag = __hip_atomic_load(&g_moe_launch_ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u;
#ifdef MK_MOE_TRACE
    unsigned long long ts[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#endif
    TS(0);

    const uint8_t *zero = lds + L::ZERO_OFF;
    int *fail_l = reinterpret_cast<int *>(lds + L::FLAG_OFF), *ready_l = fail_l + 4, *prog_l = fail_l + 8;  // both 16-byte aligned
    const uint8_t **p13 = reinterpret_cast<const uint8_t **>(lds + L::PTR_OFF), **p2 = p13 + PK_MAX_P;
    float *pw_l = reinterpret_cast<float *>(lds + L::PW_OFF), *wg_l = pw_l + PK_MAX_P;
    int *cnt_l = reinterpret_cast<int *>(lds + L::CNT_OFF);
    float *pgu = reinterpret_cast<float *>(lds + L::PGU_OFF);
    float *po = reinterpret_cast<float *>(lds + L::PO_OFF);
    float *xsc = reinterpret_cast<float *>(lds + L::XSC_OFF);
    uint8_t *xc = lds + L::x_off(pa.B);
    uint8_t *actb = lds + L::act_off(pa.B);
    constexpr int AROWB = inter + 16, ACTB = L::act_bytes(inter);

    // the first token's hidden row is requested before anything else (phase 1 turns it into codes)
    mk_f4 xv0[SB];
    if constexpr (stage != MK_MOE_STAGE_FROM_ACT) {
#pragma unroll
        for (int b = 0; b < SB; b++) xv0[b] = reinterpret_cast<const mk_f4 *>(a.x)[min((int)threadIdx.x + b * 512, NX - 1)];
    }
    // the pair tables: a pair's expert id and its two pointers would be two memory round trips one after the other before
    // the first weight can be asked for; the pointer tables (when the table states its size and it fits) are read beside
    // the ids and looked up in LDS
    const bool tabs_in_lds = a.tab.n_experts > 0 && a.tab.n_experts <= 512;
    const uint8_t **t13 = reinterpret_cast<const uint8_t **>(lds + L::PGU_OFF), **t2 = t13 + 512;  // (the partial sums' place, before they exist)
    int my_e = 0;
    bool my_ok = true;
    if ((int)threadIdx.x < P) {
        const int q = threadIdx.x, tok = q / per, sl = q - tok * per;
        my_e = sl < a.topk ? mk_checked_expert(a.ids[tok * a.topk + sl], a.tab.n_experts, my_ok) : a.shared;
    }
    if (tabs_in_lds) {
        if (threadIdx.x < a.tab.n_experts) {
            t13[threadIdx.x] = a.tab.w13t[threadIdx.x];
            t2[threadIdx.x] = a.tab.w2t[threadIdx.x];
        }
        __syncthreads();
    }
    if ((int)threadIdx.x < P) {
        const int q = threadIdx.x, tok = q / per, sl = q - tok * per;
        const int e = my_e;
        const bool ok = my_ok;
        p13[q] = tabs_in_lds ? t13[e] : a.tab.w13t[e];
        p2[q] = tabs_in_lds ? t2[e] : a.tab.w2t[e];
        const float w = sl < a.topk ? (ok ? a.weights[tok * a.topk + sl] : 0.0f) : 1.0f;
        wg_l[q] = w;                                                     // inside the activation (DeepSeek rule)
        pw_l[q] = !ok ? 0.0f : (sl < a.topk && !a.ds_rule) ? w : 1.0f;  // in the sum over the pairs
    }
    if (threadIdx.x < PK_MAX_P) cnt_l[threadIdx.x] = 0;
    if (threadIdx.x < 24) reinterpret_cast<uint32_t *>(lds)[threadIdx.x] = 0u;  // the zeros and the flags

    // this lane as a column of the instruction: phase ph (the K block of the step), part (0: a codes, 1: b codes); the
    // columns 8 .. 15 stay empty.  8-bit operand: lane group kb holds the K bytes 16 kb .. (registers 0-3) and 64 + 16 kb ..
    // (registers 4-7), so block ph lives in registers 4 (ph >> 1) .. of the lane groups 2 (ph & 1), + 1.
    const int ph = (n >> 1) & 3, pt = n & 1;
    const bool active = n < 8 && (ph & 1) == (kb >> 1);
    const bool has_lo = active && ph < 2, has_hi = active && ph >= 2;
    const int bscale = pt ? 127 : 131;  // e8m0 of the column: 2^0 for the b codes, 2^4 for the a codes
    const uint32_t code_off = (uint32_t)(ph * 32 + (kb & 1) * 16);
    const uint32_t klo = has_lo ? 128u : 0u, khi = has_hi ? 128u : 0u;  // an idle half keeps reading the zeros
    auto mfma = [&](const mk_i4 w, uint32_t wsb, const mk_i4 lo, const mk_i4 hi) {
        const mk_i8v wv = {w[0], w[1], w[2], w[3], 0, 0, 0, 0};
        const mk_i8v av = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wv, av, mk_f4{0.0f, 0.0f, 0.0f, 0.0f}, 4 /* fp4 weights */, 0 /* e4m3 codes */, 0,
                                                                (int)wsb, 0, bscale);
    };
    __syncthreads();  // the pair tables, the flags

    const int nitems = P * KI;
    Cont13 ring[CW];
    auto load_item = [&](int it) {
        it = __builtin_amdgcn_readfirstlane(min(it, nitems - 1));  // past the end: the last item once more (unconditional loads)
        const int q = it / KI, m = it - q * KI;
        const uint8_t *base = mk_uniform_ptr(p13[q]);
        const uint32_t off = (uint32_t)(((c + PK_GRID * m) * NC + CW * wave) * PK_CONT);
#pragma unroll
        for (int i = 0; i < CW; i++) {
            ring[i].w[0] = mk_ldg128_off_nt(base, off + i * PK_CONT + lane * 16);
            ring[i].w[1] = mk_ldg128_off_nt(base, off + i * PK_CONT + 1024 + lane * 16);
            ring[i].sc = __builtin_nontemporal_load((const MK_GLOBAL uint16_t *)((const MK_GLOBAL uint8_t *)base + off + i * PK_CONT + 2048 + lane * 2));
        }
    };
    if constexpr (stage != MK_MOE_STAGE_FROM_ACT) {
        if (wave < 4) load_item(0);
        // q8 codes of the hidden rows (src/q8.rs:57-68): 8 lanes per 32-block, one 16-byte load each
        for (int t = 0; t < pa.B; t++) {
            const mk_f4 *xsrc = reinterpret_cast<const mk_f4 *>(a.x + (size_t)t * D);
            mk_f4 xv[SB];
#pragma unroll
            for (int b = 0; b < SB; b++) xv[b] = t == 0 ? xv0[b] : xsrc[min((int)threadIdx.x + b * 512, NX - 1)];
#pragma unroll
            for (int b = 0; b < SB; b++) {
                const int i = threadIdx.x + b * 512;  // piece i = values 4 (i & 7) .. + 3 of block i >> 3
                float dx;
                const uint32_t q4 = pk_q8_pack4(xv[b], dx);
                uint32_t ca, cb;
                pk_split(q4, ca, cb);
                if (i < NX) {
                    *reinterpret_cast<uint32_t *>(xc + t * L::XTOK + 4 * i) = ca;
                    *reinterpret_cast<uint32_t *>(xc + t * L::XTOK + L::ROWB + 4 * i) = cb;
                    if ((i & 7) == 0) xsc[t * NB + (i >> 3)] = dx;
                }
            }
        }
        mk_lds_barrier();
    }
    TS(1);

    if (wave < 4) {
        // (phase 2's weights: declared here because the first of them are requested before phase 1's last item is worked on)
        constexpr int R2 = 2;  // pairs of this wave's K steps of W2 in flight (three measured slower: 41.9 against 40.5 us)
        Step2 w2r[R2][SW];
        const int nb_c = min(n, RB - 1);
        auto load_pair = [&](Step2 *S, int q) {
            q = __builtin_amdgcn_readfirstlane(min(q, P - 1));  // past the end: the last pair once more (unconditional loads)
            const uint8_t *base = mk_uniform_ptr(p2[q]);
#pragma unroll
            for (int s = 0; s < SW; s++) {
                const uint32_t off = (uint32_t)((c * NSI + wave * SW + s) * STEP);
                S[s].wa = mk_ldg128_off_nt(base, off + lane * 16);
                S[s].wb = mk_ldg128_off_nt(base, off + 1024 + (kb * RB + nb_c) * 16);
                S[s].sa = mk_ldg_u8_off(base, off + 1024 + 64 * RB + lane);
                S[s].sb = mk_ldg_u8_off(base, off + 1024 + 64 * RB + 64 + kb * RB + nb_c);
            }
        };
        // ------------------------------------------------------------ the multiplying waves, phase 1
        if constexpr (stage != MK_MOE_STAGE_FROM_ACT) {
            mk_f4 acc = {0.0f, 0.0f, 0.0f, 0.0f}, tp = acc;  // tp: the previous step's result, taken out after the next instruction is issued
            float dprev = 0.0f;
            // The item's sums of this wave are complete: the four phases are the lanes n ^ 2, n ^ 4 (and n ^ 6).  The last wave
            // to get here adds the waves' partial sums in wave order and publishes the eight activation values.
            auto finish_item = [&](int it) {
                const int q = it / KI, m = it - q * KI;
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    acc[r] += mk_dpp<0x4E>(acc[r]);
                    acc[r] += __shfl_xor(acc[r], 4, MK_WAVE);
                }
                float *mine = pgu + (it * 4 + wave) * 16;
                if (n == 0) *reinterpret_cast<mk_f4 *>(mine + 4 * kb) = acc;
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                int old = 0;
                if (lane == 0) old = atomicAdd(&cnt_l[it], 1);  // the LDS operations of a CU are performed in order
                old = __builtin_amdgcn_readfirstlane(old);
                if (old == 3 && lane < 8) {
                    const float *pp = pgu + it * 64;
                    const float g = mk_add(mk_add(mk_add(pp[lane], pp[16 + lane]), pp[32 + lane]), pp[48 + lane]);
                    const float u = mk_add(mk_add(mk_add(pp[8 + lane], pp[24 + lane]), pp[40 + lane]), pp[56 + lane]);
                    const float act = mk_act(a.act_kind, g, u, a.limit, wg_l[q]);
                    const size_t at = (size_t)q * inter + 8 * (c + PK_GRID * m) + lane;
                    if constexpr (stage == MK_MOE_STAGE_ACT) a.af[at] = act;
                    else __hip_atomic_store(pa.lines + at, ((unsigned long long)tag << 32) | __float_as_uint(act), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            };
            auto do_item = [&](const Cont13 *cur, int it) {
                const int q = it / KI, tok = q / per;
                const uint8_t *xt = xc + tok * L::XTOK + pt * L::ROWB + code_off + (CW * wave) * 256;
                const uint8_t *plo = has_lo ? xt : zero, *phi = has_hi ? xt : zero;
                const float *pdx = xsc + tok * NB + (n < 8 ? ph : 0) + (CW * wave) * 8;
#pragma unroll
                for (int i = 0; i < CW; i++) {
#pragma unroll
                    for (int k = 0; k < 2; k++) {
                        const int s = 2 * i + k;
                        const mk_i4 lo = *reinterpret_cast<const mk_i4 *>(plo + s * klo), hi = *reinterpret_cast<const mk_i4 *>(phi + s * khi);
                        const float dcur = pdx[4 * s];
                        const mk_f4 nw = mfma(cur[i].w[k], cur[i].sc >> (8 * k), lo, hi);
#pragma unroll
                        for (int r = 0; r < 4; r++) acc[r] = mk_add(acc[r], mk_mul(tp[r] + mk_dpp<0xB1>(tp[r]), dprev));  // a + b part: exact; the block term
                        if (s == 0 && it > 0) {  // the previous item's last result is in: its sums are complete
                            finish_item(it - 1);
                            acc = mk_f4{0.0f, 0.0f, 0.0f, 0.0f};
                        }
                        tp = nw;
                        dprev = dcur;
                    }
                }
            };
            // an item's containers are in the ring; they are taken out and the ring is refilled with the next item's
            Cont13 cur[CW];
            for (int it = 0; it < nitems - 1; it++) {
#pragma unroll
                for (int i = 0; i < CW; i++) cur[i] = ring[i];
                load_item(it + 1);
                do_item(cur, it);
            }
            // the last item: phase 2's first weights are requested in its place
#pragma unroll
            for (int i = 0; i < CW; i++) cur[i] = ring[i];
            if constexpr (stage == MK_MOE_STAGE_ALL) {
#pragma unroll
                for (int k = 0; k < R2; k++) load_pair(w2r[k], k);
            }
            do_item(cur, nitems - 1);
#pragma unroll
            for (int r = 0; r < 4; r++) acc[r] = mk_add(acc[r], mk_mul(tp[r] + mk_dpp<0xB1>(tp[r]), dprev));
            finish_item(nitems - 1);
            TS(2);
            if constexpr (stage == MK_MOE_STAGE_ACT) return;
        } else {
#pragma unroll
            for (int k = 0; k < R2; k++) load_pair(w2r[k], k);
        }

        // ------------------------------------------------------------ the multiplying waves, phase 2
        // W2_e act of pair q for this wave's K steps: partial sums of the workgroup's rows into po[q][wave]
        auto multiply = [&](const Step2 *S, int q) {
            // the pair's codes are in LDS when both exchange waves have counted it (they always count on, also after giving up)
#ifdef MK_MOE_TRACE
            const unsigned long long tw0 = __builtin_amdgcn_s_memrealtime();
#endif
            for (int spin = 0; pk_lds_min4(ready_l) <= q && spin < (1 << 26); spin++) __builtin_amdgcn_s_sleep(1);
#ifdef MK_MOE_TRACE
            ts[4] += __builtin_amdgcn_s_memrealtime() - tw0;
#endif
            const uint8_t *buf = actb + (q % RC) * ACTB;
            const float *adx = reinterpret_cast<const float *>(buf + 2 * AROWB);
            const uint8_t *xt = buf + pt * AROWB + code_off + (SW * wave) * 128;
            const uint8_t *plo = has_lo ? xt : zero, *phi = has_hi ? xt : zero;
            const float *pdx = adx + (n < 8 ? ph : 0) + (SW * wave) * 4;
            mk_f4 oa = {0.0f, 0.0f, 0.0f, 0.0f}, ob = oa, ta = oa, tb2 = oa;
            float dprev = 0.0f;
#pragma unroll
            for (int s = 0; s < SW; s++) {
                const mk_i4 lo = *reinterpret_cast<const mk_i4 *>(plo + s * klo), hi = *reinterpret_cast<const mk_i4 *>(phi + s * khi);
                const float dcur = pdx[4 * s];
                const mk_f4 na = mfma(S[s].wa, S[s].sa, lo, hi), nb2 = mfma(S[s].wb, S[s].sb, lo, hi);
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    oa[r] = mk_add(oa[r], mk_mul(ta[r] + mk_dpp<0xB1>(ta[r]), dprev));
                    ob[r] = mk_add(ob[r], mk_mul(tb2[r] + mk_dpp<0xB1>(tb2[r]), dprev));
                }
                ta = na;
                tb2 = nb2;
                dprev = dcur;
            }
#pragma unroll
            for (int r = 0; r < 4; r++) {
                oa[r] = mk_add(oa[r], mk_mul(ta[r] + mk_dpp<0xB1>(ta[r]), dprev));
                ob[r] = mk_add(ob[r], mk_mul(tb2[r] + mk_dpp<0xB1>(tb2[r]), dprev));
                oa[r] += mk_dpp<0x4E>(oa[r]);
                ob[r] += mk_dpp<0x4E>(ob[r]);
                oa[r] += __shfl_xor(oa[r], 4, MK_WAVE);
                ob[r] += __shfl_xor(ob[r], 4, MK_WAVE);
            }
            if (n == 0) {
                float *mine = po + (q * 4 + wave) * 32;
                *reinterpret_cast<mk_f4 *>(mine + 4 * kb) = oa;
                *reinterpret_cast<mk_f4 *>(mine + 16 + 4 * kb) = ob;
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            if (lane == 0) *(volatile int *)(prog_l + wave) = q + 1;
            if (q == 0) TS(3);
        };
        for (int q0 = 0; q0 < P; q0 += R2) {
#pragma unroll
            for (int k = 0; k < R2; k++) {
                const int q = q0 + k;
                if (q < P) {
                    multiply(w2r[k], q);
                    load_pair(w2r[k], q + R2);
                }
            }
        }
        TS(5);
    } else {
        // ------------------------------------------------------------ the exchange waves
        if constexpr (stage == MK_MOE_STAGE_ACT) return;
        const int xw = wave - 4;
        // a pair's units: lane l of exchange wave xw holds the values 4 i .. 4 i + 3 for i = 64 xw + l + 256 b, eight lanes a 32-block
        constexpr int NPC = inter / 1024;  // pieces of four values per lane
        constexpr int NUN = 4;            // pairs whose units are on their way
        unsigned long long un[NUN][NPC][4];
        auto load_units = [&](unsigned long long (*U)[4], int q) {
            q = min(q, P - 1);
#pragma unroll
            for (int b = 0; b < NPC; b++)
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    const size_t at = (size_t)q * inter + 4 * (64 * xw + lane + 256 * b) + u;
                    if constexpr (stage == MK_MOE_STAGE_FROM_ACT) U[b][u] = ((unsigned long long)tag << 32) | __float_as_uint(a.af[at]);
                    else U[b][u] = __hip_atomic_load(pa.lines + at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
        };
        auto units_complete = [&](unsigned long long (*U)[4]) {
            bool bad = false;
#pragma unroll
            for (int b = 0; b < NPC; b++)
#pragma unroll
                for (int u = 0; u < 4; u++) bad |= (uint32_t)(U[b][u] >> 32) != tag;
            return __builtin_amdgcn_ballot_w64(bad) == 0;
        };
        // The exchange runs beside phase 1, LAG pairs behind this workgroup's own multiplying waves (the other workgroups are
        // about as far: a pair that far back is complete nearly everywhere, so a read seldom has to be repeated); the last
        // LAG pairs wait for this workgroup's phase 1 to end.
        constexpr int LAG = 2;
        int own_done = 0;  // items this workgroup has published
        auto eligible = [&](int q) {
            if constexpr (stage != MK_MOE_STAGE_ALL) return true;
            while (own_done < nitems && pk_lds_int(cnt_l + own_done) == 4) own_done++;
            return own_done >= min((q + LAG + 1) * KI, nitems);
        };
        bool failed = false;
        // the pair's activation row: wait (bounded) until every unit carries the tag, then its q8 blocks (what matvec_packed
        // does to its input, src/q8.rs:49-69) as codes in the pair's slot of LDS
        auto form_codes = [&](unsigned long long (*U)[4], int q) {
            // the slot was pair q - RC's: every multiplying wave must be through with it
            for (int spin = 0; q >= RC && pk_lds_min4(prog_l) < q - RC + 1 && spin < (1 << 26); spin++) __builtin_amdgcn_s_sleep(1);
            for (int tries = 0; !units_complete(U); tries++) {
                if (tries >= pa.spin_limit) {
                    failed = true;
                    break;
                }
                __builtin_amdgcn_s_sleep(4);
                load_units(U, q);
            }
            uint8_t *buf = actb + (q % RC) * ACTB;
            float *adx = reinterpret_cast<float *>(buf + 2 * AROWB);
#pragma unroll
            for (int b = 0; b < NPC; b++) {
                const int i = 64 * xw + lane + 256 * b;  // piece i = values 4 (i & 7) .. + 3 of block i >> 3
                const mk_f4 v = {__uint_as_float((uint32_t)U[b][0]), __uint_as_float((uint32_t)U[b][1]), __uint_as_float((uint32_t)U[b][2]),
                                 __uint_as_float((uint32_t)U[b][3])};
                float dx;
                const uint32_t q4 = pk_q8_pack4(v, dx);
                uint32_t ca, cb;
                pk_split(q4, ca, cb);
                *reinterpret_cast<uint32_t *>(buf + 4 * i) = ca;
                *reinterpret_cast<uint32_t *>(buf + AROWB + 4 * i) = cb;
                if ((i & 7) == 0) adx[i >> 3] = dx;
            }
            if (failed && lane == 0) *(volatile int *)fail_l = 1;
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            if (lane == 0) *(volatile int *)(ready_l + xw) = q + 1;
        };
        // wave 4 also owns the workgroup's rows: o of pair q from the four waves' partial sums in wave order, y += w * o in
        // slot order -- whenever the multiplying waves are through with a pair
        float y = 0.0f;
        int next_add = 0;
        auto add_pairs = [&](bool wait) {
            while (next_add < P) {
                if (pk_lds_min4(prog_l) <= next_add) {
                    if (!wait) return;
                    for (int spin = 0; pk_lds_min4(prog_l) <= next_add && spin < (1 << 26); spin++) __builtin_amdgcn_s_sleep(1);
                }
                const int q = next_add++;
                if (lane < RW) {
                    const float *pp = po + q * 128;
                    const float o = mk_add(mk_add(mk_add(pp[lane], pp[32 + lane]), pp[64 + lane]), pp[96 + lane]);
                    y = mk_add(y, mk_mul(pw_l[q], o));
                    const int tok = q / per;
                    if (q - tok * per == per - 1) {  // the token's last pair
                        a.out[(size_t)tok * D + RW * c + lane] = *(volatile int *)fail_l ? __uint_as_float(0x7FC00000u) : y;
                        y = 0.0f;
                    }
                }
            }
        };
        int issued = 0;  // the units of the pairs [0, issued) have been requested
        for (int q0 = 0; q0 < P; q0 += NUN) {
#pragma unroll
            for (int k = 0; k < NUN; k++) {
                const int q = q0 + k;
                if (q < P) {
                    if (issued <= q) {  // not requested ahead: wait (bounded) until the pair is worth asking for
                        for (int spin = 0; !eligible(q) && spin < (1 << 26); spin++) __builtin_amdgcn_s_sleep(8);
                        load_units(un[k], q);
                        issued = q + 1;
                    }
                    // ask ahead for the pairs that are worth it, as far as the buffers go
#pragma unroll
                    for (int j = 1; j < NUN; j++)
                        if (issued == q + j && q + j < P && eligible(q + j)) {
                            load_units(un[(k + j) % NUN], q + j);
                            issued = q + j + 1;
                        }
                    form_codes(un[k], q);
                    if (xw == 0) add_pairs(false);
                }
            }
        }
        if (xw != 0) return;
        add_pairs(true);
        if (*(volatile int *)fail_l && lane == 0) g_moe_fail = 1;
        // the next launch's tag: only after this workgroup has seen every unit of this launch, i.e. after every workgroup has
        // read the counter
        if (stage == MK_MOE_STAGE_ALL && c == 0 && lane == 0) atomicAdd(&g_moe_launch_ctr, 1u);
    }
#ifdef MK_MOE_TRACE
    if (lane == 0 && wave < 4)
        for (int i = 0; i < 8; i++) g_moe_ts[(c * 4 + wave) * 8 + i] = ts[i];
#endif
}

template <int D>
int launch_persist(const PersistArgs &pa, hipStream_t st) {
    // slots for the codes of the pairs: all of them when they fit
    const int P = pa.B * pa.f.per, budget = 150 * 1024;
    int rc = (budget - PLds<D>::act_off(pa.B)) / PLds<D>::act_bytes(2048);
    if (rc > P) rc = P;
    if (rc < 4) {
        mk_set_error("moe_persist: the codes of the hidden rows leave no room in LDS");
        return MK_ERR_UNSUPPORTED;
    }
    int lds = PLds<D>::total(pa.B, 2048, rc);
    if (lds < 84 * 1024) lds = 84 * 1024;  // more than half a CU's LDS: one workgroup per CU, the whole grid resident
    int s;
    switch (pa.stage) {
        case MK_MOE_STAGE_ACT:
            if ((s = mk_lds_opt_in(reinterpret_cast<const void *>(moe_persist_kernel<D, 2048, MK_MOE_STAGE_ACT>), 152 * 1024)) != MK_OK) return s;
            hipLaunchKernelGGL((moe_persist_kernel<D, 2048, MK_MOE_STAGE_ACT>), dim3(PK_GRID), dim3(512), (size_t)lds, st, pa, rc);
            break;
        case MK_MOE_STAGE_FROM_ACT:
            if ((s = mk_lds_opt_in(reinterpret_cast<const void *>(moe_persist_kernel<D, 2048, MK_MOE_STAGE_FROM_ACT>), 152 * 1024)) != MK_OK) return s;
            hipLaunchKernelGGL((moe_persist_kernel<D, 2048, MK_MOE_STAGE_FROM_ACT>), dim3(PK_GRID), dim3(512), (size_t)lds, st, pa, rc);
            break;
        default:
            if ((s = mk_lds_opt_in(reinterpret_cast<const void *>(moe_persist_kernel<D, 2048, MK_MOE_STAGE_ALL>), 152 * 1024)) != MK_OK) return s;
            hipLaunchKernelGGL((moe_persist_kernel<D, 2048, MK_MOE_STAGE_ALL>), dim3(PK_GRID), dim3(512), (size_t)lds, st, pa, rc);
    }
    return mk_launch_status("moe_persist");
}

int device_cus() {
    static int cus = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
            (void)hipGetLastError();
            return 0;
        }
        return n;
    }();
    return cus;
}

}  // namespace

bool mk_moe_persist_takes(size_t B, size_t d, size_t inter, int per) {
    return (d == 7168 || d == 5120) && inter == 2048 && B >= 1 && B <= 3 && B * per <= (size_t)PK_MAX_P && device_cus() == PK_GRID;
}

size_t mk_moe_persist_lines_bytes(size_t P, size_t inter) { return P * inter * sizeof(unsigned long long); }

int mk_moe_persist_launch(const FusedArgs &a, size_t B, int stage, void *lines, hipStream_t st) {
    PersistArgs pa;
    pa.f = a;
    pa.B = (int)B;
    pa.stage = stage;
    pa.spin_limit = MK_TUNE("MK_MOE_SPIN_LIMIT", 1 << 16);
    pa.lines = reinterpret_cast<unsigned long long *>(lines);
    switch (a.d) {
        case 7168: return launch_persist<7168>(pa, st);
        case 5120: return launch_persist<5120>(pa, st);
        default: mk_set_error("moe_persist: d = %d not covered", a.d); return MK_ERR_UNSUPPORTED;
    }
}

#ifdef MK_MOE_TRACE
extern "C" int mk_debug_moe_ts(unsigned long long *out) {
    MK_HIP_TRY(hipMemcpyFromSymbol(out, HIP_SYMBOL(g_moe_ts), sizeof(unsigned long long) * PK_GRID * 4 * 8));
    return MK_OK;
}
#endif

extern "C" int mk_dev_moe_decode_gave_up(int *flag) {
    MK_REQUIRE(flag, "null pointer");
    int v = 0;
    MK_HIP_TRY(hipMemcpyFromSymbol(&v, HIP_SYMBOL(g_moe_fail), sizeof(int)));
    *flag = v;
    return MK_OK;
}

extern "C" size_t mk_moe_pack_bytes(size_t d, size_t inter, int down) {
    if (!down) return 2 * inter * (d / 32) * 17;
    if (d % 256 != 0 || d / 256 <= 16 || d / 256 > 32) return 0;
    return (size_t)PK_GRID * (inter / 128) * pk_step_bytes((int)(d / 256) - 16);
}

extern "C" int mk_dev_moe_pack_gate_up(const uint8_t *w1p, const uint8_t *w1s, const uint8_t *w3p, const uint8_t *w3s, size_t d, size_t inter,
                                       uint8_t *pack, void *stream) {
    MK_REQUIRE(w1p && w1s && w3p && w3s && pack, "null pointer");
    MK_REQUIRE(d > 0 && d % 256 == 0 && inter > 0 && inter % 8 == 0, "d % 256 == 0 and inter % 8 == 0");
    MK_REQUIRE(2 * inter * (d / 32) * 17 < 0x7FFFFFFFull, "matrices too large for the packed form");
    MK_REQUIRE((((uintptr_t)w1p | (uintptr_t)w3p | (uintptr_t)pack) & 15) == 0, "the nibble arrays and the pack must be 16-byte aligned");
    const size_t nthr = 2 * inter * (d / 32);
    hipLaunchKernelGGL(pack13_kernel, dim3((unsigned)((nthr + 255) / 256)), dim3(256), 0, (hipStream_t)stream, w1p, w1s, w3p, w3s, (int)inter,
                       (int)(d / 32), pack, 0, nullptr, nullptr, nullptr, nullptr);
    return mk_launch_status("moe_pack_gate_up");
}

extern "C" int mk_dev_moe_unpack_gate_up(const uint8_t *pack, size_t d, size_t inter, uint8_t *w1p, uint8_t *w1s, uint8_t *w3p, uint8_t *w3s,
                                         void *stream) {
    MK_REQUIRE(w1p && w1s && w3p && w3s && pack, "null pointer");
    MK_REQUIRE(d > 0 && d % 256 == 0 && inter > 0 && inter % 8 == 0, "d % 256 == 0 and inter % 8 == 0");
    MK_REQUIRE((((uintptr_t)w1p | (uintptr_t)w3p | (uintptr_t)pack) & 15) == 0, "the nibble arrays and the pack must be 16-byte aligned");
    const size_t nthr = 2 * inter * (d / 32);
    hipLaunchKernelGGL(pack13_kernel, dim3((unsigned)((nthr + 255) / 256)), dim3(256), 0, (hipStream_t)stream, nullptr, nullptr, nullptr, nullptr,
                       (int)inter, (int)(d / 32), const_cast<uint8_t *>(pack), 1, w1p, w1s, w3p, w3s);
    return mk_launch_status("moe_unpack_gate_up");
}

extern "C" int mk_dev_moe_pack_down(const uint8_t *w2p, const uint8_t *w2s, size_t d, size_t inter, uint8_t *pack, void *stream) {
    MK_REQUIRE(w2p && w2s && pack, "null pointer");
    MK_REQUIRE(d % 256 == 0 && d / 256 > 16 && d / 256 <= 32 && inter > 0 && inter % 128 == 0, "d / 256 in 17 .. 32 and inter % 128 == 0");
    MK_REQUIRE((((uintptr_t)w2p | (uintptr_t)pack) & 15) == 0, "the nibble array and the pack must be 16-byte aligned");
    MK_HIP_TRY(hipMemsetAsync(pack, 0, mk_moe_pack_bytes(d, inter, 1), (hipStream_t)stream));  // the padding of every step
    const size_t nthr = d * (inter / 32);
    hipLaunchKernelGGL(pack2_kernel, dim3((unsigned)((nthr + 255) / 256)), dim3(256), 0, (hipStream_t)stream, w2p, w2s, (int)d, (int)(inter / 32),
                       (int)(d / 256), pack, 0, nullptr, nullptr);
    return mk_launch_status("moe_pack_down");
}

extern "C" int mk_dev_moe_unpack_down(const uint8_t *pack, size_t d, size_t inter, uint8_t *w2p, uint8_t *w2s, void *stream) {
    MK_REQUIRE(w2p && w2s && pack, "null pointer");
    MK_REQUIRE(d % 256 == 0 && d / 256 > 16 && d / 256 <= 32 && inter > 0 && inter % 128 == 0, "d / 256 in 17 .. 32 and inter % 128 == 0");
    MK_REQUIRE((((uintptr_t)w2p | (uintptr_t)pack) & 15) == 0, "the nibble array and the pack must be 16-byte aligned");
    const size_t nthr = d * (inter / 32);
    hipLaunchKernelGGL(pack2_kernel, dim3((unsigned)((nthr + 255) / 256)), dim3(256), 0, (hipStream_t)stream, nullptr, nullptr, (int)d,
                       (int)(inter / 32), (int)(d / 256), const_cast<uint8_t *>(pack), 1, w2p, w2s);
    return mk_launch_status("moe_unpack_down");
}
