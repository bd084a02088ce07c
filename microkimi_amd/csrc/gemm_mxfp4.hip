// Prefill expert GEMM: the per-expert batched evaluation of moe_prefill
// (src/model.rs:2539-2602) on the gfx950 block-scaled matrix cores.
//
//   y[i][r] = sum_k W_e[r][k] * x[i][k]      for the token rows i of group e
//
// v_mfma_scale_f32_16x16x128_f8f6f4 multiplies a 16x128 by a 128x16 tile with
// one e8m0 scale per 32 K-elements on each side -- the MXFP4 weight format as
// it is stored: a lane's B operand is the 16 bytes (32 nibbles) of ONE block of
// one weight row and its scale byte, loaded straight from the reference layout.
// The A operand is the activation in MXFP8 (e4m3 codes + e8m0 per 32), 32 bytes
// per lane.  Accumulation is f32 in the matrix core.
//
// Operand layout of the instruction (measured on the device with one-hot
// operands, both formats):
//   scales        lane i + 16 b supplies the e8m0 byte of row/column i, K block b (k in [32 b, 32 b + 32))
//   4-bit operand lane i + 16 b holds k = 32 b + j in registers 0-3, nibble j (low nibble first): one MXFP4 block
//   8-bit operand lane i + 16 g holds k = 16 g + j in registers 0-3 (bytes 0-15) and k = 64 + 16 g + j in
//                 registers 4-7 (bytes 16-31): the K = 128 step is two K = 64 halves
//   result        lane l holds column l % 16, rows 4 (l / 16) + r
//
// Two kernels.  The general one (cols % 128 == 0): workgroup = 4 waves = 64
// weight rows of one expert; each wave owns 16 rows and up to 64 token rows (4
// accumulator tiles), so an expert's weights are streamed from HBM once for up
// to 64 tokens.  The streaming one (cols % 512 == 0, below) is the one the
// model shapes take.  At the prefill shapes (about 16 tokens per expert) the
// work is bound by the weight stream, not by the MFMA.
#include <algorithm>

#include "mk_common.h"
#include <type_traits>

namespace {

constexpr int MC = 4;  // 16-token accumulator tiles per wave

__global__ __launch_bounds__(256) void mxfp4_grouped_gemm_kernel(const uint8_t *const *__restrict__ packed_ptrs,
                                                                 const uint8_t *const *__restrict__ scales_ptrs, int rows, int cols,
                                                                 const uint8_t *__restrict__ codes, const uint8_t *__restrict__ exps,
                                                                 const int32_t *__restrict__ offsets, float *__restrict__ out) {
    const int e = blockIdx.y;
    const int tok0 = offsets[e], tok1 = offsets[e + 1];
    if (tok1 <= tok0) return;
    const uint8_t *packed = packed_ptrs[e];
    const uint8_t *scales = scales_ptrs[e];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = lane & 15, kb = lane >> 4;
    const int nb = cols / 32, steps = cols / 128;
    const int row = blockIdx.x * 64 + wave * 16 + n;
    const bool row_ok = row < rows;
    const uint8_t *wrow = packed + (size_t)(row_ok ? row : 0) * (cols / 2) + kb * 16;
    const uint8_t *srow = scales + (size_t)(row_ok ? row : 0) * nb + kb;

    for (int base = tok0; base < tok1; base += 16 * MC) {
        const int ntok = min(16 * MC, tok1 - base);
        const int nchunk = (ntok + 15) / 16;
        mk_f4 acc[MC];
#pragma unroll
        for (int c = 0; c < MC; c++) acc[c] = mk_f4{0.0f, 0.0f, 0.0f, 0.0f};
        // A rows of this lane: token base + c*16 + n (clamped; rows past the group are discarded at the store)
        const uint8_t *arow[MC];
        const uint8_t *aexp[MC];
#pragma unroll
        for (int c = 0; c < MC; c++) {
            const int t = min(base + c * 16 + n, tok1 - 1);
            arow[c] = codes + (size_t)t * cols + kb * 16;
            aexp[c] = exps + (size_t)t * nb + kb;
        }
        for (int s = 0; s < steps; s++) {
            const mk_i4 wv = *reinterpret_cast<const mk_i4 *>(wrow + s * 64);
            const int wsb = srow[s * 4];
            mk_i8v b = {wv[0], wv[1], wv[2], wv[3], 0, 0, 0, 0};
#pragma unroll
            for (int c = 0; c < MC; c++) {
                if (c < nchunk) {
                    const mk_i4 a0 = *reinterpret_cast<const mk_i4 *>(arow[c] + s * 128);
                    const mk_i4 a1 = *reinterpret_cast<const mk_i4 *>(arow[c] + s * 128 + 64);
                    const int asb = aexp[c][s * 4];
                    mk_i8v a = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
                    acc[c] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, acc[c], 0 /*A: fp8 e4m3*/, 4 /*B: fp4 e2m1*/, 0, asb, 0, wsb);
                }
            }
        }
        if (row_ok) {
#pragma unroll
            for (int c = 0; c < MC; c++) {
                if (c < nchunk) {
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const int t = base + c * 16 + kb * 4 + i;
                        if (t < tok1) out[(size_t)t * rows + row] = acc[c][i];
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------- streaming kernel
// cols % 512 == 0.  A workgroup owns 256 weight rows of one expert (a wave 64 =
// four 16-row tiles) and walks K in tiles of 512 (four MFMA steps):
//
//   * the group's activation tile (up to 16*MC tokens x 512 codes + 16 scale
//     bytes each) is staged in LDS once per K tile and serves all 16 row tiles
//     of the workgroup; the next tile is fetched into registers meanwhile;
//   * weights go straight from global memory to registers, one unit = one row
//     tile x four steps (256 contiguous bytes per row, 4 KB per wave) ahead, in
//     two alternating register blocks, with unconditional (clamped) addresses so
//     that no wait is forced.  Units that gave a row shorter runs (64 or 128
//     bytes, more row tiles per unit) were measured slower, whatever their
//     bytes in flight;
//   * the 16 scale bytes per weight row and K tile are fetched once per
//     workgroup (thread i: row i, one 16-byte load) and staged in LDS with the
//     activation tile, transposed to [K block][step]; a lane reads the dword of
//     its row and K block from there and shifts out the byte of its step.
//
// Loads take the form "uniform base + 32-bit lane offset".  The K offset goes
// through readfirstlane, which hides the loop counter from the induction
// variable widening that would otherwise rebuild 64-bit pointers per lane.
constexpr int KT_STEPS = 4;
// LDS row stride of the activation tile: rows 8 banks apart (with 4 or 16 banks the 16-byte operand reads counted 2.5
// times the bank-conflict cycles).  TWO (see gemm_pass): a token row has two code rows and two exponent rows per K tile.
constexpr int a_stride(bool two = false) { return (two ? 1024 : 512) + 32; }
constexpr int a_codes_bytes(int mc, bool two = false) { return 16 * mc * a_stride(two); }
constexpr int a_wsc_off(int mc, bool two = false) { return a_codes_bytes(mc, two) + 16 * mc * (two ? 32 : 16); }  // codes, then the scale bytes per token,
constexpr int a_buf_bytes(int mc, bool two = false, int wg_rows = 256) { return a_wsc_off(mc, two) + wg_rows * 16; }  // then the K tile's 16 scale bytes of the workgroup's weight rows

// One launch covers n_mats (1 or 2) weight matrices per group that share the activation rows (gate and up): matrix m
// of group e is packed_ptrs[m][e], its result goes to out[m].
struct GemmArgs {
    const uint8_t *const *packed_ptrs[2];
    const uint8_t *const *scales_ptrs[2];
    // optional: the same scale bytes in [K tile of 512 columns][row][16] order (mk_dev_mxfp4_scales_by_tile).  A row's 16
    // bytes per K tile are an eighth of a 128-byte line of the plain array, and that line is asked for in eight K tiles:
    // the scale lines of the workgroups resident on an XCD outgrow its L2 and were fetched 2.9 times; in this order a
    // workgroup's 4 KB per K tile are whole lines that are used once
    const uint8_t *const *scales_t_ptrs[2];
    int rows, cols;
    const uint8_t *codes;
    const uint8_t *exps;
    const int32_t *offsets;
    float *out[2];
    int n_groups, n_mats, row_blocks;
    // gate/up form (GU passes): a workgroup owns 128 rows of BOTH matrices of a group, and the epilogue applies the
    // activation and writes its MXFP8 form (the input of the down projection); out[] is written only when `keep` is set
    int act_kind, keep;
    uint8_t *act_codes;  // [token rows][rows] e4m3
    uint8_t *act_exps;   // [token rows][rows / 32] e8m0
};

// PIN: the weights are the instruction's M operand and the token rows its N operand, so a lane of the 16 x 16 result
// holds four consecutive weight rows of one token row: one 16-byte store.  (With the roles the other way round a lane
// holds one weight row of four tokens and every value is a store of its own; on the down projection of the prefill
// shape those stores took 100 of the kernel's 400 us.)
template <bool NT>
__device__ __forceinline__ void store_tile(float *out, int rows, int t, int tok1, int row, const mk_f4 &v) {
    if (t >= tok1) return;
    float *dst = out + (size_t)t * rows + row;
    if (row + 3 < rows && ((reinterpret_cast<uintptr_t>(dst) & 15) == 0)) {
        if constexpr (NT) __builtin_nontemporal_store(v, reinterpret_cast<mk_f4 *>(dst));
        else *reinterpret_cast<mk_f4 *>(dst) = v;
    } else {
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (row + i < rows) dst[i] = v[i];
    }
}

// Two neighbouring 16-row tiles of 16 tokens as full 128-byte lines: the lanes of tokens 8-15 hand their half of the
// second tile to the lanes of tokens 0-7 and take those lanes' half of the first (a rotation by 8 inside every 16-lane row),
// so that one store instruction writes the whole line (32 rows) of 8 tokens instead of half a line of 16.
// x: rows row .. row + 15, y: rows row + 16 .. row + 31 (this lane: token t0 + n, rows + 4 kb .. + 4 kb + 3 of each).
template <bool NT>
__device__ __forceinline__ void store_tile_pair(float *out, int rows, int t0, int tok1, int row, int n, int kb, const mk_f4 &x, const mk_f4 &y) {
    const bool up = n >= 8;
    // tokens 0-7: own first tile | second tile of the lane 8 below;  tokens 8-15: first tile of the lane 8 above | own second tile
    // (written component by component: the same exchange in a loop over a vector index gave all four lanes' values of
    // component 0 on the device)
    const mk_i4 xi = __builtin_bit_cast(mk_i4, x), yi = __builtin_bit_cast(mk_i4, y);
    mk_i4 fi, si;
    fi.x = __builtin_amdgcn_update_dpp(xi.x, yi.x, 0x128 /* row_ror:8 */, 0xF, 0xC, false);
    fi.y = __builtin_amdgcn_update_dpp(xi.y, yi.y, 0x128, 0xF, 0xC, false);
    fi.z = __builtin_amdgcn_update_dpp(xi.z, yi.z, 0x128, 0xF, 0xC, false);
    fi.w = __builtin_amdgcn_update_dpp(xi.w, yi.w, 0x128, 0xF, 0xC, false);
    si.x = __builtin_amdgcn_update_dpp(yi.x, xi.x, 0x128, 0xF, 0x3, false);
    si.y = __builtin_amdgcn_update_dpp(yi.y, xi.y, 0x128, 0xF, 0x3, false);
    si.z = __builtin_amdgcn_update_dpp(yi.z, xi.z, 0x128, 0xF, 0x3, false);
    si.w = __builtin_amdgcn_update_dpp(yi.w, xi.w, 0x128, 0xF, 0x3, false);
    const mk_f4 first = __builtin_bit_cast(mk_f4, fi), second = __builtin_bit_cast(mk_f4, si);
    store_tile<NT>(out, rows, t0 + (n & 7), tok1, row + (up ? 16 : 0) + kb * 4, first);
    store_tile<NT>(out, rows, t0 + 8 + (n & 7), tok1, row + (up ? 16 : 0) + kb * 4, second);
}

// The 16 scale bytes a row has in a K tile, [step][K block of the step], as [K block][step]: a lane (K block kb) then finds
// the bytes of its four steps in ONE dword of LDS, and the byte of a step is a shift by a constant.
__device__ __forceinline__ mk_i4 mk_scale_bytes_by_kb(const mk_i4 v) {
    const uint32_t d0 = (uint32_t)v[0], d1 = (uint32_t)v[1], d2 = (uint32_t)v[2], d3 = (uint32_t)v[3];
    // v_perm_b32(hi, lo, sel): selector bytes 0-3 pick from lo, 4-7 from hi
    const uint32_t a01 = __builtin_amdgcn_perm(d1, d0, 0x05010400u);  // d0.b0 d1.b0 d0.b1 d1.b1
    const uint32_t b01 = __builtin_amdgcn_perm(d1, d0, 0x07030602u);  // d0.b2 d1.b2 d0.b3 d1.b3
    const uint32_t a23 = __builtin_amdgcn_perm(d3, d2, 0x05010400u);
    const uint32_t b23 = __builtin_amdgcn_perm(d3, d2, 0x07030602u);
    mk_i4 o;
    o[0] = (int)__builtin_amdgcn_perm(a23, a01, 0x05040100u);  // kb 0: d0.b0 d1.b0 d2.b0 d3.b0
    o[1] = (int)__builtin_amdgcn_perm(a23, a01, 0x07060302u);  // kb 1
    o[2] = (int)__builtin_amdgcn_perm(b23, b01, 0x05040100u);  // kb 2
    o[3] = (int)__builtin_amdgcn_perm(b23, b01, 0x07060302u);  // kb 3
    return o;
}

// PIN: the loads and the matrix instructions stay where the source puts them.  Left alone, instruction selection places
// all of a K tile's matrix instructions at its end (nothing orders them against the loads), every unit's operands stay
// live until then, and the scheduler, out of registers, moves loads down to their first use -- one of them to the end
// of the K tile, behind a wait for every load in flight.  An empty volatile statement that takes a unit's accumulators
// keeps its matrix instructions in front of the next unit's loads; scheduling barriers keep the loads in place.  Prefill
// shape: 256 -> 167 registers (three workgroups per CU), gate GEMM 450 -> 409 us, down GEMM 463 -> 403 us.  The kernel for
// larger groups lost by it while a group's passes ran one after the other on 64 workgroups (403 -> 474 us); with the
// passes dealt to the whole chip it runs pinned too (DEEP below).
// FULL: the weight loads take whole 128-byte lines (see below).  NT: they are non-temporal.  Measured: 8 experts x 512
// tokens (eight passes over each expert's weights) 495 -> 403 us with FULL, 459 us with FULL + NT; prefill shape (one pass,
// at most 32 tokens per expert) 488 -> 504 us with FULL alone, 451 us with FULL + NT.
// DEEP: four register blocks of weights, one per row tile, each re-requested for the next K tile as soon as it has
// been used (three units of matrix work between issue and use) instead of two alternating blocks.
// Large groups (8 experts x 512 tokens, 120 GFLOP): 403 us while the eight 64-token passes of a group ran one after the
// other on 64 workgroups; 93 us (1.29 PFLOP/s) with the passes dealt to 512 workgroups, pinned order, DEEP and two
// workgroups per CU.  Counters on that shape: the matrix cores are busy 27 us of the 93; waves spend half of their time
// waiting for loads although the L2 hit rate is 83 % and it answers in 270 cycles on average; the vector cache handles
// 94k accesses per CU.  Per K tile a workgroup moves 64 KB of weights and 33 KB of activations through it for 16.8
// MFLOP.  Measured since, each passing the tests and none changing the time by more than the run-to-run spread: a
// step-major pass (the K tile walked step by step with all four row tiles' weights in registers, activation operands
// read from LDS once per step for all of them, exchange of the whole-line loads under the matrix instructions, the
// barrier passed before the last step) 84-100 us; the operand's own load mapping (a lane per row: 53 cache accesses per
// load instruction instead of 26); the scale bytes fetched once per row and K tile through LDS (a third fewer cache
// accesses; kept).  What did help: two row tiles sharing one read of the activation operands (half the LDS reads) with
// the line exchange done in place, so that it still fits two waves per SIMD: 93-109 -> 82-95 us (1.3-1.5 PFLOP/s; the
// same form with a second copy of the units in registers ran at one wave per SIMD and 101-111 us).  All four row tiles
// per read (step-major, in place) needs 43 registers more than two waves per SIMD allow.  The next thing to measure is a larger tile
// per workgroup (256 x 128 tokens: half the bytes through the cache per FLOP) with a per-step timeline of one wave.
// GU: the gate/up form.  The wave's row tiles 0, 1 are rows row0 .. row0 + 31 of the first matrix (gate) and its row tiles
// 2, 3 the same rows of the second (up: packed3 / scales3), so a lane ends up with g and u of the same (row, token); the
// epilogue forms ACT(g, u), quantizes each token's 32 values to MXFP8 (mk_mxfp8_quantize8's arithmetic with the whole
// e8m0 range; the block's maximum crosses the four lanes of a token) and stores codes and exponent bytes: 1.03 bytes
// per value instead of 8 written and 8 read back by a kernel of its own.
// TWO: every activation value is the sum of two e4m3 terms with block exponents of their own -- the exact split of a
// bfloat16 value x = hi + lo, hi its leading four significant bits and lo the other four (mk_bf16_split8) -- kept per
// K tile as [hi codes 512][lo codes 512] and [hi exponents 16][lo exponents 16].  The K tile then is 1024 products deep:
// two matrix instructions per step against the same weight registers into the same accumulators, nothing else changes.
// The products are exact and the sums f32, so this is the bfloat16 GEMM (apart from values more than 2^13 below their
// block's largest, whose last bits fall off the e4m3 grid) at the streaming rate of the MXFP8 one.
// NW: waves of the workgroup (4, or 8 for large groups: 512 weight rows share one staged activation tile, which halves the
// activation bytes a CU fetches per FLOP -- the pass for large groups is bound by what a CU can load, about 30 B/ns).
// RT: 16-row tiles a wave owns (4; 2 with eight token tiles for large groups: 32 rows x 128 tokens a wave keeps the same 64
// accumulator registers and moves 0.8 x the bytes per FLOP of 64 rows x 64 tokens).
template <int MC, bool FULL, bool NT, bool PIN, bool DEEP = false, bool GU = false, bool TWO = false, int NW = 4, int RT = 4>
__device__ __forceinline__ void gemm_pass(const GemmArgs &a, const uint8_t *packed, const uint8_t *scales, float *out, int rb, int base, int tok1,
                                          uint8_t *lds, const uint8_t *scales_t, const uint8_t *packed3 = nullptr, const uint8_t *scales3 = nullptr,
                                          const uint8_t *scales3_t = nullptr) {
    static_assert(!GU || (FULL && PIN && !DEEP && MC <= 2), "the gate/up form exists for the small-group pass");
    static_assert(!TWO || (FULL && PIN && !DEEP && MC <= 2), "the two-term form exists for the small-group pass");
    static_assert(NW == 4 || (NW == 8 && !GU && !TWO), "eight waves: the plain pass only");
    static_assert(RT == 4 || (RT == 2 && DEEP && PIN && FULL && !GU && !TWO), "two row tiles a wave: the deep pass only");
    constexpr int WG_ROWS = 16 * RT * NW;
    constexpr int AW = TWO ? 2 : 1, AS = a_stride(TWO);
    constexpr int NTH = 64 * NW, STG_N = 2 * MC * AW * 4 / NW;  // threads; 16-byte chunks of the activation tile per thread
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, kb = lane >> 4;
    const int cols = a.cols, nb = cols / 32, ktiles = cols / 512;
    const int row0 = GU ? rb * 128 + wave * 32 : rb * WG_ROWS + wave * (16 * RT);
    // first row of the wave's row tile rt
    auto tile_row = [&](int rt) { return GU ? row0 + (rt & 1) * 16 : row0 + rt * 16; };
    // this lane's weight row in each of the wave's four row tiles (clamped; stores are guarded)
    // FULL: weight loads take whole 128-byte lines: load j = 2i + h of a unit covers line i (of the K tile's two) of the
    // rows 8h .. 8h+7 of the row tile, lane (r3 = lane / 8, c = lane % 8) reading bytes 16c .. of row 8h + r3, and the
    // operand form is restored in registers (compute_unit).  Otherwise the operand's own mapping: load s covers 64 bytes
    // of all 16 rows, lane (kb, n) reading bytes 16 kb .. of row n (every line is then requested by two loads).
    static_assert(KT_STEPS == 4, "two lines of 128 bytes per row and K tile");
    const int r3 = lane >> 3, c8 = lane & 7;
    uint32_t woff[RT][FULL ? 2 : 1];
#pragma unroll
    for (int rt = 0; rt < RT; rt++) {
        if constexpr (FULL) {
#pragma unroll
            for (int h = 0; h < 2; h++) woff[rt][h] = (uint32_t)min(tile_row(rt) + 8 * h + r3, a.rows - 1) * (uint32_t)(cols / 2) + c8 * 16;
        } else {
            woff[rt][0] = (uint32_t)min(tile_row(rt) + n, a.rows - 1) * (uint32_t)(cols / 2) + kb * 16;
        }
    }
    // after the lane rotation below, lane (kg, x, r3) holds what lane (r3, x, kg) loaded
    const int rot_idx = (((lane & 7) << 3) | (((lane >> 3) & 1) << 2) | (lane >> 4)) * 4;
    mk_i4 wa[KT_STEPS], wb[KT_STEPS];
    auto load_unit = [&](mk_i4 *w, int kt, int rt) {
        const uint32_t ku = (uint32_t)__builtin_amdgcn_readfirstlane(min(kt, ktiles - 1));
        const uint8_t *pk = (GU && rt >= 2) ? packed3 : packed;
#pragma unroll
        for (int j = 0; j < KT_STEPS; j++)
            if constexpr (GU) w[j] = mk_ldg128_off_nt(pk, woff[rt][j & 1] + ku * (KT_STEPS * 64) + (j >> 1) * 128);
            else if constexpr (FULL && NT) w[j] = mk_ldg128_off_nt(packed, woff[rt][j & 1] + ku * (KT_STEPS * 64) + (j >> 1) * 128);
            else if constexpr (FULL) w[j] = mk_ldg128_off(packed, woff[rt][j & 1] + ku * (KT_STEPS * 64) + (j >> 1) * 128);
            else w[j] = mk_ldg128_off(packed, woff[rt][0] + ku * (KT_STEPS * 64) + j * 64);
    };
    // activation tile staging: chunk i = tid + 256 k -> token i / 32, 16-byte chunk i % 32
    // The K tile's scale bytes of the workgroup's 256 weight rows (16 per row) go through LDS with the activation
    // tile: thread i fetches row i's once.  Fetched by the lanes that use them (a lane per row, four lanes of a
    // row the same 16 bytes) they were 4 of a wave's 29 loads per K tile and about half of its vector-cache
    // accesses: a 16-byte load whose lanes sit in 16 different lines is looked up once per lane and pass.
    mk_i4 st[STG_N], ste, stw;
    // (gate/up form: thread i is row slot (wave i / 64, row tile (i / 16) % 4, row i % 16) of the workgroup)
    // (two row tiles a wave: the workgroup has fewer rows than threads, the upper threads fetch a row again and store nothing)
    const int ws_row = GU ? rb * 128 + (tid >> 6) * 32 + ((tid >> 4) & 1) * 16 + (tid & 15) : rb * WG_ROWS + min(tid, WG_ROWS - 1);
    const bool ws_tiles = scales_t != nullptr;  // (uniform)
    const uint8_t *ws_base = (GU && ((tid >> 5) & 1)) ? (ws_tiles ? scales3_t : scales3) : (ws_tiles ? scales_t : scales);
    const uint32_t ws_r = (uint32_t)min(ws_row, a.rows - 1);
    const uint32_t wsoff = ws_tiles ? ws_r * 16u : ws_r * (uint32_t)nb, ws_step = ws_tiles ? (uint32_t)a.rows * 16u : 16u;
    uint32_t coff[STG_N];  // the host checks that tokens x cols (x 2) stays below 2^32
#pragma unroll
    for (int k = 0; k < STG_N; k++) {
        const int i = tid + NTH * k;
        coff[k] = (uint32_t)min(base + i / (32 * AW), tok1 - 1) * (uint32_t)(cols * AW) + (i % (32 * AW)) * 16;
    }
    // (thread i: token i / AW, exponent row i % AW)
    const uint32_t eoff = (uint32_t)min(base + (tid & (16 * MC * AW - 1)) / AW, tok1 - 1) * (uint32_t)(nb * AW) + (tid % AW) * 16;
    auto stage_load = [&](int kt) {
        const uint32_t ku = (uint32_t)__builtin_amdgcn_readfirstlane(min(kt, ktiles - 1));
#ifdef MK_GEMM_FP4_PROBE
        constexpr int STG = MC >= 4 ? STG_N / 2 : STG_N;  // (half the bytes a token row has in a K tile)
#else
        constexpr int STG = STG_N;
#endif
#pragma unroll
        for (int k = 0; k < STG; k++) st[k] = mk_ldg128_off(a.codes, coff[k] + ku * (512 * AW));
        ste = mk_ldg128_off(a.exps, eoff + ku * (16 * AW));
        stw = mk_ldg128_off(ws_base, wsoff + ku * ws_step);
    };
    auto stage_store = [&](uint8_t *buf) {
#pragma unroll
        for (int k = 0; k < STG_N; k++) {
#ifdef MK_GEMM_FP4_PROBE
            if (MC >= 4 && k >= STG_N / 2) break;
#endif
            const int i = tid + NTH * k;
            *reinterpret_cast<mk_i4 *>(buf + (i / (32 * AW)) * AS + (i % (32 * AW)) * 16) = st[k];
        }
        if (tid < 16 * MC * AW) *reinterpret_cast<mk_i4 *>(buf + a_codes_bytes(MC, TWO) + tid * 16) = mk_scale_bytes_by_kb(ste);
        if (WG_ROWS >= NTH || tid < WG_ROWS) *reinterpret_cast<mk_i4 *>(buf + a_wsc_off(MC, TWO) + tid * 16) = mk_scale_bytes_by_kb(stw);
    };
    mk_f4 acc[RT][MC];
#pragma unroll
    for (int rt = 0; rt < RT; rt++)
#pragma unroll
        for (int c = 0; c < MC; c++) acc[rt][c] = mk_f4{0.0f, 0.0f, 0.0f, 0.0f};

    auto mma_unit = [&](const mk_i4 *w, int rt, const uint8_t *buf) {
        const uint32_t sc = *reinterpret_cast<const uint32_t *>(buf + a_wsc_off(MC, TWO) + (wave * (16 * RT) + rt * 16 + n) * 16 + kb * 4);
#pragma unroll
        for (int c = 0; c < MC; c++) {
            const uint32_t ae = *reinterpret_cast<const uint32_t *>(buf + a_codes_bytes(MC, TWO) + (c * 16 + n) * (16 * AW) + kb * 4);
            const uint8_t *arow = buf + (c * 16 + n) * AS + kb * 16;
#pragma unroll
            for (int s = 0; s < KT_STEPS; s++) {
                const mk_i4 a0 = *reinterpret_cast<const mk_i4 *>(arow + s * 128);
                const mk_i4 a1 = *reinterpret_cast<const mk_i4 *>(arow + s * 128 + 64);
                const mk_i8v av = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
                const mk_i8v bv = {w[s][0], w[s][1], w[s][2], w[s][3], 0, 0, 0, 0};
                const int asb = (int)(ae >> (8 * s));  // the instruction reads byte 0
                const int wsb = (int)(sc >> (8 * s));
                if constexpr (PIN)
                    acc[rt][c] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bv, av, acc[rt][c], 4 /*M: fp4 weights*/, 0 /*N: fp8 rows*/, 0, wsb, 0, asb);
                else
                    acc[rt][c] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, bv, acc[rt][c], 0 /*M: fp8 rows*/, 4 /*N: fp4 weights*/, 0, asb, 0, wsb);
            }
            if constexpr (TWO) {  // the second term of every value against the same weight registers
                const uint32_t ael = *reinterpret_cast<const uint32_t *>(buf + a_codes_bytes(MC, TWO) + (c * 16 + n) * 32 + 16 + kb * 4);
#pragma unroll
                for (int s = 0; s < KT_STEPS; s++) {
                    const mk_i4 a0 = *reinterpret_cast<const mk_i4 *>(arow + 512 + s * 128);
                    const mk_i4 a1 = *reinterpret_cast<const mk_i4 *>(arow + 512 + s * 128 + 64);
                    const mk_i8v av = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
                    const mk_i8v bv = {w[s][0], w[s][1], w[s][2], w[s][3], 0, 0, 0, 0};
                    acc[rt][c] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bv, av, acc[rt][c], 4, 0, 0, (int)(sc >> (8 * s)), 0, (int)(ael >> (8 * s)));
                }
            }
        }
    };
    // Two row tiles against one read of the activation operands (large groups: with four token tiles the LDS reads of a
    // unit, 32 KB per wave, take longer than its 16 matrix instructions; shared by two units they take half)
    auto mma_unit2 = [&](const mk_i4 *w0, const mk_i4 *w1, int rt, const uint8_t *buf, auto c_begin, auto c_end) {
        constexpr int C0 = decltype(c_begin)::value, C1 = decltype(c_end)::value;  // token tiles [C0, C1)
        // (a lane's scale bytes of the K tile are one dword each: staged as [K block][step], see mk_scale_bytes_by_kb)
        const uint32_t sc0 = *reinterpret_cast<const uint32_t *>(buf + a_wsc_off(MC, TWO) + (wave * (16 * RT) + rt * 16 + n) * 16 + kb * 4);
        const uint32_t sc1 = *reinterpret_cast<const uint32_t *>(buf + a_wsc_off(MC, TWO) + (wave * (16 * RT) + rt * 16 + n) * 16 + kb * 4 + 256);
#pragma unroll
        for (int c = C0; c < C1; c++) {
            const uint32_t ae = *reinterpret_cast<const uint32_t *>(buf + a_codes_bytes(MC, TWO) + (c * 16 + n) * 16 + kb * 4);
            const uint8_t *arow = buf + (c * 16 + n) * AS + kb * 16;
#pragma unroll
            for (int s = 0; s < KT_STEPS; s++) {
                const mk_i4 a0 = *reinterpret_cast<const mk_i4 *>(arow + s * 128);
#ifdef MK_GEMM_FP4_PROBE
                // timing only (the results mean nothing): the activation operand taken as e2m1 -- 16 bytes a lane instead of
                // 32, both operands fp4, the instruction at its fp4 rate -- to see what MXFP4 activations would buy
                const mk_i8v av = {a0[0], a0[1], a0[2], a0[3], 0, 0, 0, 0};
                constexpr int AFMT = 4;
#else
                const mk_i4 a1 = *reinterpret_cast<const mk_i4 *>(arow + s * 128 + 64);
                const mk_i8v av = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
                constexpr int AFMT = 0;
#endif
                const int asb = (int)(ae >> (8 * s));
                const mk_i8v b0 = {w0[s][0], w0[s][1], w0[s][2], w0[s][3], 0, 0, 0, 0}, b1 = {w1[s][0], w1[s][1], w1[s][2], w1[s][3], 0, 0, 0, 0};
                acc[rt][c] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(b0, av, acc[rt][c], 4, AFMT, 0, (int)(sc0 >> (8 * s)), 0, asb);
                acc[rt + 1][c] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(b1, av, acc[rt + 1][c], 4, AFMT, 0, (int)(sc1 >> (8 * s)), 0, asb);
            }
        }
    };
    // the line exchange of compute_unit, in place (no second copy of the unit in registers)
    auto exchange_in_place = [&](mk_i4 *w) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int ra = __builtin_amdgcn_ds_bpermute(rot_idx, w[2 * i][k]), rb2 = __builtin_amdgcn_ds_bpermute(rot_idx, w[2 * i + 1][k]);
                w[2 * i][k] = __builtin_amdgcn_update_dpp(ra, rb2, 0x128 /* row_ror:8 */, 0xF, 0xC, false);
                w[2 * i + 1][k] = __builtin_amdgcn_update_dpp(rb2, ra, 0x128 /* row_ror:8 */, 0xF, 0x3, false);
            }
        }
    };
    auto pin_acc = [&](int rt) {
        if constexpr (PIN) {
#pragma unroll
            for (int c = 0; c < MC; c++) asm volatile("" : "+v"(acc[rt][c]));
        }
    };
    // One unit: 4 steps x MC token tiles.  The LDS reads of the activation operands do not depend on the
    // row tile, so after inlining the four calls of a K tile share them.
    auto compute_unit = [&](const mk_i4 *wl, int rt, const uint8_t *buf) {
        if constexpr (!FULL) {
            mma_unit(wl, rt, buf);
            pin_acc(rt);
            return;
        }
        // Loaded: for line i, wl[2i] = rows 0-7 and wl[2i+1] = rows 8-15, lane (r3, s', kg) holding the 16 bytes of K
        // group kg of step 2i + s'.  Wanted: step s in w[s], lane (kg, row).  A rotation of the lane index by three
        // bits (ds_bpermute) brings (kg, s', r3); then the two registers exchange their 8-lane halves inside every
        // 16-lane row (DPP row rotate by 8 with a bank mask), which trades the lane bit s' for the row-half bit.
        mk_i4 w[KT_STEPS];
#pragma unroll
        for (int i = 0; i < 2; i++) {
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int ra = __builtin_amdgcn_ds_bpermute(rot_idx, wl[2 * i][k]), rb = __builtin_amdgcn_ds_bpermute(rot_idx, wl[2 * i + 1][k]);
                w[2 * i][k] = __builtin_amdgcn_update_dpp(ra, rb, 0x128 /* row_ror:8 */, 0xF, 0xC, false);      // lanes 8-15 of a row <- rb
                w[2 * i + 1][k] = __builtin_amdgcn_update_dpp(rb, ra, 0x128 /* row_ror:8 */, 0xF, 0x3, false);  // lanes 0-7 of a row <- ra
            }
        }
        mma_unit(w, rt, buf);
        pin_acc(rt);
    };

    if constexpr (DEEP) {
        // Four register blocks, one per row tile: the unit of row tile rt for K tile kt + 1 is requested as soon as the
        // unit of K tile kt has been used, three units of matrix work ahead of its use.
        mk_i4 w4[RT][KT_STEPS];
#pragma unroll
        for (int rt = 0; rt < RT; rt++) load_unit(w4[rt], 0, rt);
        stage_load(0);
        __syncthreads();  // the previous pass (if any) has finished with the LDS buffers
        stage_store(lds);
        __syncthreads();
#pragma unroll 1
        for (int kt = 0; kt < ktiles; kt++) {
            const uint8_t *buf = lds + (kt & 1) * a_buf_bytes(MC, TWO, WG_ROWS);
            stage_load(kt + 1);
            if constexpr (PIN && FULL && RT == 2) {
                // One pair of row tiles: its weights are in use until the K tile's last matrix instruction, so the next K
                // tile's are asked for half way, into the registers the staged activation chunks leave when they are
                // stored (the other LDS buffer is free since the last barrier); left to the end of the K tile the loads
                // had nothing but the barrier in front of their first use.
                mk_i4 wn[2][KT_STEPS];
                __builtin_amdgcn_sched_barrier(0);
                exchange_in_place(w4[0]);
                exchange_in_place(w4[1]);
                mma_unit2(w4[0], w4[1], 0, buf, std::integral_constant<int, 0>{}, std::integral_constant<int, MC / 2>{});
                pin_acc(0);
                pin_acc(1);
                __builtin_amdgcn_sched_barrier(0);
                stage_store(lds + ((kt + 1) & 1) * a_buf_bytes(MC, TWO, WG_ROWS));
                __builtin_amdgcn_sched_barrier(0);
                load_unit(wn[0], kt + 1, 0);
                load_unit(wn[1], kt + 1, 1);
                __builtin_amdgcn_sched_barrier(0);
                mma_unit2(w4[0], w4[1], 0, buf, std::integral_constant<int, MC / 2>{}, std::integral_constant<int, MC>{});
                pin_acc(0);
                pin_acc(1);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int j = 0; j < KT_STEPS; j++) w4[0][j] = wn[0][j], w4[1][j] = wn[1][j];
                __syncthreads();
                continue;
            } else if constexpr (PIN && FULL && MC >= 4) {
                // large groups: two row tiles per read of the activation operands (93-109 -> 82-95 us on 8 experts x 512 tokens)
#pragma unroll
                for (int rt = 0; rt < RT; rt += 2) {
                    __builtin_amdgcn_sched_barrier(0);
                    exchange_in_place(w4[rt]);
                    exchange_in_place(w4[rt + 1]);
                    mma_unit2(w4[rt], w4[rt + 1], rt, buf, std::integral_constant<int, 0>{}, std::integral_constant<int, MC>{});
                    pin_acc(rt);
                    pin_acc(rt + 1);
                    __builtin_amdgcn_sched_barrier(0);
                    load_unit(w4[rt], kt + 1, rt);
                    load_unit(w4[rt + 1], kt + 1, rt + 1);
                }
            } else {
#pragma unroll
                for (int rt = 0; rt < RT; rt++) {
                    if constexpr (PIN) __builtin_amdgcn_sched_barrier(0);
                    compute_unit(w4[rt], rt, buf);
                    if constexpr (PIN) __builtin_amdgcn_sched_barrier(0);
                    load_unit(w4[rt], kt + 1, rt);
                }
            }
            if constexpr (PIN) __builtin_amdgcn_sched_barrier(0);
            stage_store(lds + ((kt + 1) & 1) * a_buf_bytes(MC, TWO, WG_ROWS));
            __syncthreads();
        }
    } else {
        load_unit(wa, 0, 0);
        stage_load(0);
        __syncthreads();  // the previous pass (if any) has finished with the LDS buffers
        stage_store(lds);
        __syncthreads();
#pragma unroll 1
        for (int kt = 0; kt < ktiles; kt++) {
            const uint8_t *buf = lds + (kt & 1) * a_buf_bytes(MC, TWO, WG_ROWS);
            stage_load(kt + 1);
            load_unit(wb, kt, 1);
            if constexpr (PIN) __builtin_amdgcn_sched_barrier(0);
            compute_unit(wa, 0, buf);
            if constexpr (PIN) __builtin_amdgcn_sched_barrier(0);
            load_unit(wa, kt, 2);
            if constexpr (PIN) __builtin_amdgcn_sched_barrier(0);
            compute_unit(wb, 1, buf);
            if constexpr (PIN) __builtin_amdgcn_sched_barrier(0);
            load_unit(wb, kt, 3);
            if constexpr (PIN) __builtin_amdgcn_sched_barrier(0);
            compute_unit(wa, 2, buf);
            if constexpr (PIN) __builtin_amdgcn_sched_barrier(0);
            load_unit(wa, kt + 1, 0);
            if constexpr (PIN) __builtin_amdgcn_sched_barrier(0);
            compute_unit(wb, 3, buf);
            if constexpr (PIN) __builtin_amdgcn_sched_barrier(0);
            stage_store(lds + ((kt + 1) & 1) * a_buf_bytes(MC, TWO, WG_ROWS));
            __syncthreads();
        }
    }
    if constexpr (GU) {
        // lane (n, kb): token base + 16 c + n, rows row0 + 4 kb .. + 3 (tiles 0 / 2) and row0 + 16 + 4 kb .. (tiles 1 / 3)
#pragma unroll
        for (int c = 0; c < MC; c++) {
            float v[8];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                v[i] = mk_act(a.act_kind, acc[0][c][i], acc[2][c][i], 0.0f, 1.0f);
                v[4 + i] = mk_act(a.act_kind, acc[1][c][i], acc[3][c][i], 0.0f, 1.0f);
            }
            if constexpr (TWO) {
                // bfloat16 of the activation as two e4m3 terms, in the K-tile layout the down projection stages
                uint32_t hi[2], lo[2], eh, el;
                mk_bf16_split8<true>(v, hi, lo, eh, el);
                const int t = base + c * 16 + n;
                if (t < tok1 && row0 + 31 < a.rows) {
                    const int r = row0 + kb * 4;
                    uint8_t *dst = a.act_codes + (size_t)t * (2 * (size_t)a.rows) + (r >> 9) * 1024 + (r & 511);
                    *reinterpret_cast<uint32_t *>(dst) = hi[0];
                    *reinterpret_cast<uint32_t *>(dst + 16) = hi[1];
                    *reinterpret_cast<uint32_t *>(dst + 512) = lo[0];
                    *reinterpret_cast<uint32_t *>(dst + 528) = lo[1];
                    if (kb == 0) {
                        uint8_t *ed = a.act_exps + (size_t)t * (a.rows / 16) + (r >> 9) * 32 + ((r & 511) >> 5);
                        ed[0] = (uint8_t)eh;
                        ed[16] = (uint8_t)el;
                    }
                }
                continue;
            }
            float amax = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; i++) amax = fmaxf(amax, fabsf(v[i]));
            amax = mk_rows_max(amax);  // the token's 32 rows: this lane's eight and those of the lanes n + 16, + 32, + 48
            int e = mk_ceil_log2f(fmaxf(amax, 1e-4f) / 448.0f);
            e = max(-127, min(127, e));
            const uint32_t eb = (uint32_t)(e + 127);
            const float inv = mk_scale_from_byte(254u - eb);
            float q[8];
#pragma unroll
            for (int i = 0; i < 8; i++) q[i] = fminf(fmaxf(v[i] * inv, -448.0f), 448.0f);
            int w0 = 0, w1 = 0;
            w0 = __builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], w0, false);
            w0 = __builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], w0, true);
            w1 = __builtin_amdgcn_cvt_pk_fp8_f32(q[4], q[5], w1, false);
            w1 = __builtin_amdgcn_cvt_pk_fp8_f32(q[6], q[7], w1, true);
            const int t = base + c * 16 + n;
            if (t < tok1 && row0 + 31 < a.rows) {
                uint8_t *dst = a.act_codes + (size_t)t * a.rows + row0 + kb * 4;
                *reinterpret_cast<uint32_t *>(dst) = (uint32_t)w0;
                *reinterpret_cast<uint32_t *>(dst + 16) = (uint32_t)w1;
                if (kb == 0) a.act_exps[(size_t)t * (a.rows / 32) + row0 / 32] = (uint8_t)eb;
            }
        }
        if (a.keep) {  // the f32 gate and up rows as well (tests read them)
#pragma unroll
            for (int c = 0; c < MC; c++) {
                store_tile_pair<NT>(a.out[0], a.rows, base + c * 16, tok1, row0, n, kb, acc[0][c], acc[1][c]);
                store_tile_pair<NT>(a.out[1], a.rows, base + c * 16, tok1, row0, n, kb, acc[2][c], acc[3][c]);
            }
        }
        return;
    }
#pragma unroll
    for (int rt = 0; rt < RT; rt += 2) {
        if constexpr (PIN) {
#pragma unroll
            for (int c = 0; c < MC; c++) store_tile_pair<NT>(out, a.rows, base + c * 16, tok1, row0 + rt * 16, n, kb, acc[rt][c], acc[rt + 1][c]);
        } else {
            // token rows as the M operand: a lane holds one weight row of four tokens
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int row = row0 + (rt + h) * 16 + n;
                if (row < a.rows) {
#pragma unroll
                    for (int c = 0; c < MC; c++)
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            const int t = base + c * 16 + kb * 4 + i;
                            if (t < tok1) out[(size_t)t * a.rows + row] = acc[rt + h][c][i];
                        }
                }
            }
        }
    }
}

// Two instantiations share the grid: groups of up to 32 tokens (the prefill
// case; one or two token tiles) and larger ones, in passes of 64 tokens.  A
// workgroup whose group belongs to the other one exits.
template <int MC, bool TWO = false, int NW = 4, int RT = 4>
__global__ __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(2))) void mxfp4_grouped_gemm_stream_kernel(GemmArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    // Workgroup -> (group, matrix, row block).  Consecutive workgroup ids go round the 8 XCDs, each with its own L2: with
    // the plain order the workgroups of one group land on all of them and each fetches the group's activation rows for
    // itself (prefill gate GEMM: 235 MB of 2.45 GB).  When the group count allows it, XCD x takes the groups x, x + 8, ...
    // and runs all workgroups of a group itself.
    const int per_group = a.n_mats * a.row_blocks, n_items = a.n_groups * per_group;
    if constexpr (!TWO && MC >= 4) {
        // The launch for large groups follows every launch for small ones, because the group sizes live on the device.
        // When no group has more than 32 rows (the prefill shape) it has nothing to do: found here, once per workgroup,
        // and the grid is a few hundred workgroups that walk the items -- workgroups of this size go one to a CU, and
        // one per item, each leaving at its own count, took 12-20 us to drain.
        int big = 0;
        for (int g = threadIdx.x; g < a.n_groups; g += blockDim.x) big |= (a.offsets[g + 1] - a.offsets[g] > 32) ? 1 : 0;
        if (!__syncthreads_or(big)) return;
    }
#pragma unroll 1
    for (int item = blockIdx.x; item < n_items; item += gridDim.x) {
    int e, r;
    if (a.n_groups % 8 == 0) {
        const int x = item & 7, j = item >> 3;
        e = x + 8 * (j / per_group);
        r = j % per_group;
    } else {
        e = item / per_group;
        r = item % per_group;
    }
    const int m = r / a.row_blocks, rb = r % a.row_blocks;
    const int tok0 = a.offsets[e], tok1 = a.offsets[e + 1];
    const int count = tok1 - tok0;
    if (count <= 0 || (!TWO && (count <= 32) != (MC == 2))) continue;
    const uint8_t *packed = mk_uniform_ptr(a.packed_ptrs[m][e]);
    const uint8_t *scales = mk_uniform_ptr(a.scales_ptrs[m][e]);
    const uint8_t *scales_t = a.scales_t_ptrs[m] ? mk_uniform_ptr(a.scales_t_ptrs[m][e]) : nullptr;
    float *out = a.out[m];
    if constexpr (TWO) {
        // any group size: passes of 32 token rows, one after the other
        if (count <= 16) {
            gemm_pass<1, true, true, true, false, false, true>(a, packed, scales, out, rb, tok0, tok1, lds, scales_t);
        } else {
#pragma unroll 1
            for (int base = tok0; base < tok1; base += 32) gemm_pass<2, true, true, true, false, false, true>(a, packed, scales, out, rb, base, tok1, lds, scales_t);
        }
    } else if (MC == 2) {
        if (count <= 16) gemm_pass<1, true, true, true>(a, packed, scales, out, rb, tok0, tok1, lds, scales_t);
        else gemm_pass<2, true, true, true>(a, packed, scales, out, rb, tok0, tok1, lds, scales_t);
    } else {
        // the 64-token passes of a group are dealt to gridDim.y workgroups: a few large groups still fill the chip
#pragma unroll 1
        for (int base = tok0 + 16 * MC * (int)blockIdx.y; base < tok1; base += 16 * MC * (int)gridDim.y)
            gemm_pass<MC, true, false, true, true, false, false, NW, RT>(a, packed, scales, out, rb, base, tok1, lds, scales_t);
    }
    }  // items
}

// The gate/up form: workgroup -> (group, block of 128 rows), both matrices.  Groups of up to 16 tokens take one token
// tile, larger ones passes of 32 tokens (a group beyond 32 passes over its weights again: the prefill shape has none).
template <bool TWO = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void mxfp4_grouped_gemm_gu_kernel(GemmArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int per_group = a.row_blocks;  // blocks of 128 rows
    int e, rb;
    if (a.n_groups % 8 == 0) {  // a group's workgroups on one XCD (see the kernel above)
        const int x = blockIdx.x & 7, j = blockIdx.x >> 3;
        e = x + 8 * (j / per_group);
        rb = j % per_group;
    } else {
        e = blockIdx.x / per_group;
        rb = blockIdx.x % per_group;
    }
    const int tok0 = a.offsets[e], tok1 = a.offsets[e + 1];
    const int count = tok1 - tok0;
    if (count <= 0) return;
    const uint8_t *p1 = mk_uniform_ptr(a.packed_ptrs[0][e]), *s1 = mk_uniform_ptr(a.scales_ptrs[0][e]);
    const uint8_t *p3 = mk_uniform_ptr(a.packed_ptrs[1][e]), *s3 = mk_uniform_ptr(a.scales_ptrs[1][e]);
    const bool tiles = a.scales_t_ptrs[0] && a.scales_t_ptrs[1];
    const uint8_t *t1 = tiles ? mk_uniform_ptr(a.scales_t_ptrs[0][e]) : nullptr, *t3 = tiles ? mk_uniform_ptr(a.scales_t_ptrs[1][e]) : nullptr;
    if (count <= 16) {
        gemm_pass<1, true, true, true, false, true, TWO>(a, p1, s1, nullptr, rb, tok0, tok1, lds, t1, p3, s3, t3);
    } else {
#pragma unroll 1
        for (int base = tok0; base < tok1; base += 32)
            gemm_pass<2, true, true, true, false, true, TWO>(a, p1, s1, nullptr, rb, base, tok1, lds, t1, p3, s3, t3);
    }
}

template <int MC, bool TWO = false, int NW = 4, int RT = 4>
int launch_stream(GemmArgs a, size_t m, hipStream_t st) {
    // Large groups: the group sizes live on the device, so the number of workgroups per (group, row block) follows the
    // average group size (one per 64 tokens, at most 16); a workgroup without a pass exits at once.
    unsigned passes = 1;
    if (MC >= 4) passes = (unsigned)std::min<size_t>(16, std::max<size_t>(1, (m / a.n_groups + 16 * MC - 1) / (16 * MC)));
    constexpr int WG_ROWS = 16 * RT * NW;
    a.row_blocks = (a.rows + WG_ROWS - 1) / WG_ROWS;
    const size_t n_items = (size_t)a.n_groups * a.n_mats * a.row_blocks;
    const dim3 grid((unsigned)(MC >= 4 ? std::min<size_t>(n_items, 512) : n_items), passes);  // (512: a multiple of the 8 XCDs)
    const int s = mk_lds_opt_in(reinterpret_cast<const void *>(mxfp4_grouped_gemm_stream_kernel<MC, TWO, NW, RT>), 2 * a_buf_bytes(MC, TWO, WG_ROWS));
    if (s != MK_OK) return s;
    hipLaunchKernelGGL((mxfp4_grouped_gemm_stream_kernel<MC, TWO, NW, RT>), grid, dim3(64 * NW), 2 * a_buf_bytes(MC, TWO, WG_ROWS), st, a);
    return mk_launch_status("mxfp4_grouped_gemm_stream");
}

}  // namespace

// gate and up of the prefill section in one launch (the matrices share the token rows); see mk_common.h
int mk_mxfp4_grouped_gemm_n(int n_mats, const uint8_t *const *const *packed_ptrs, const uint8_t *const *const *scales_ptrs, size_t n_groups,
                            size_t rows, size_t cols, const uint8_t *codes, const uint8_t *exps, const int32_t *offsets, size_t m,
                            float *const *out, void *stream, const uint8_t *const *const *scales_t_ptrs, bool two) {
    MK_REQUIRE(n_mats == 1 || n_mats == 2, "one or two matrices per group");
    MK_REQUIRE(!two || (cols % 512 == 0 && m * cols * 2 < 0xFFFFFFFFull), "the two-term form takes cols in multiples of 512");
    for (int k = 0; k < n_mats; k++) MK_REQUIRE(packed_ptrs[k] && scales_ptrs[k] && out[k], "null pointer");
    MK_REQUIRE(codes && exps && offsets, "null pointer");
    MK_REQUIRE(cols % 128 == 0 && cols > 0, "cols must be a positive multiple of 128");
    MK_REQUIRE(n_groups >= 1 && n_groups <= 65535 && rows >= 1 && rows <= 0x7FFFFF00u, "bad shape");
    MK_REQUIRE(((uintptr_t)codes & 15) == 0, "codes must be 16-byte aligned");
    if (m == 0) return MK_OK;
    const size_t row_blocks = (rows + 255) / 256;
    if (cols % 512 == 0 && rows * (cols / 2) < 0xFFFFFFFFull && m * cols < 0xFFFFFFFFull && ((uintptr_t)exps & 15) == 0 &&
        n_groups * n_mats * row_blocks < 0x7FFFFFFFull) {
        GemmArgs a{};
        for (int k = 0; k < n_mats; k++) {
            a.packed_ptrs[k] = packed_ptrs[k];
            a.scales_ptrs[k] = scales_ptrs[k];
            a.scales_t_ptrs[k] = scales_t_ptrs ? scales_t_ptrs[k] : nullptr;
            a.out[k] = out[k];
        }
        a.rows = (int)rows;
        a.cols = (int)cols;
        a.codes = codes;
        a.exps = exps;
        a.offsets = offsets;
        a.n_groups = (int)n_groups;
        a.n_mats = n_mats;
        a.row_blocks = (int)row_blocks;
        if (two) return launch_stream<2, true>(a, m, (hipStream_t)stream);
        int st = launch_stream<2>(a, m, (hipStream_t)stream);
        if (st == MK_OK && m > 32) {
            const int form = MK_TUNE("MK_GEMM_LARGE_FORM", 2);  // 0: 4 waves x 64 rows x 64 tokens; 1: 8 waves x 64 x 64; 2: 8 waves x 32 rows x 128 tokens
            st = form == 2 ? launch_stream<8, false, 8, 2>(a, m, (hipStream_t)stream)
                 : form == 1 ? launch_stream<4, false, 8>(a, m, (hipStream_t)stream) : launch_stream<4>(a, m, (hipStream_t)stream);
        }
        return st;
    }
    MK_REQUIRE(!two, "the two-term form needs the streaming kernel's shapes");
    for (int k = 0; k < n_mats; k++) {
        hipLaunchKernelGGL(mxfp4_grouped_gemm_kernel, dim3((unsigned)((rows + 63) / 64), (unsigned)n_groups), dim3(256), 0, (hipStream_t)stream,
                           packed_ptrs[k], scales_ptrs[k], (int)rows, (int)cols, codes, exps, offsets, out[k]);
        const int st = mk_launch_status("mxfp4_grouped_gemm");
        if (st != MK_OK) return st;
    }
    return MK_OK;
}

// Gate and up of the prefill section with the activation and its MXFP8 form in the epilogue (see mk_common.h).
// MK_ERR_UNSUPPORTED for shapes the streaming kernel does not take: the caller then runs the separate steps.
int mk_mxfp4_grouped_gemm_gate_up_act(const uint8_t *const *w1p, const uint8_t *const *w1s, const uint8_t *const *w3p, const uint8_t *const *w3s,
                                      size_t n_groups, size_t rows, size_t cols, const uint8_t *codes, const uint8_t *exps,
                                      const int32_t *offsets, size_t m, int act_kind, uint8_t *act_codes, uint8_t *act_exps, float *keep_g,
                                      float *keep_u, void *stream, const uint8_t *const *w1st, const uint8_t *const *w3st, bool two) {
    MK_REQUIRE(w1p && w1s && w3p && w3s && codes && exps && offsets && act_codes && act_exps, "null pointer");
    if (two && (rows % 512 != 0 || m * cols * 2 >= 0xFFFFFFFFull)) return MK_ERR_UNSUPPORTED;
    if (!(cols % 512 == 0 && rows % 128 == 0 && rows * (cols / 2) < 0xFFFFFFFFull && m * cols < 0xFFFFFFFFull && ((uintptr_t)exps & 15) == 0 &&
          ((uintptr_t)codes & 15) == 0 && ((uintptr_t)act_codes & 3) == 0 && n_groups * (rows / 128) < 0x7FFFFFFFull))
        return MK_ERR_UNSUPPORTED;
    if (m == 0) return MK_OK;
    GemmArgs a{};
    a.packed_ptrs[0] = w1p;
    a.scales_ptrs[0] = w1s;
    a.packed_ptrs[1] = w3p;
    a.scales_ptrs[1] = w3s;
    a.scales_t_ptrs[0] = w1st;
    a.scales_t_ptrs[1] = w3st;
    a.out[0] = keep_g;
    a.out[1] = keep_u;
    a.keep = keep_g && keep_u;
    a.rows = (int)rows;
    a.cols = (int)cols;
    a.codes = codes;
    a.exps = exps;
    a.offsets = offsets;
    a.n_groups = (int)n_groups;
    a.n_mats = 2;
    a.row_blocks = (int)(rows / 128);
    a.act_kind = act_kind;
    a.act_codes = act_codes;
    a.act_exps = act_exps;
    if (two) {
        const int s = mk_lds_opt_in(reinterpret_cast<const void *>(mxfp4_grouped_gemm_gu_kernel<true>), 2 * a_buf_bytes(2, true));
        if (s != MK_OK) return s;
        hipLaunchKernelGGL(mxfp4_grouped_gemm_gu_kernel<true>, dim3((unsigned)(n_groups * (rows / 128))), dim3(256), 2 * a_buf_bytes(2, true),
                           (hipStream_t)stream, a);
        return mk_launch_status("mxfp4_grouped_gemm_gu");
    }
    const int s = mk_lds_opt_in(reinterpret_cast<const void *>(mxfp4_grouped_gemm_gu_kernel<false>), 2 * a_buf_bytes(2));
    if (s != MK_OK) return s;
    hipLaunchKernelGGL(mxfp4_grouped_gemm_gu_kernel<false>, dim3((unsigned)(n_groups * (rows / 128))), dim3(256), 2 * a_buf_bytes(2), (hipStream_t)stream, a);
    return mk_launch_status("mxfp4_grouped_gemm_gu");
}

extern "C" int mk_dev_mxfp4_grouped_gemm(const uint8_t *const *packed_ptrs, const uint8_t *const *scales_ptrs, size_t n_groups, size_t rows,
                                         size_t cols, const uint8_t *codes, const uint8_t *exps, const int32_t *offsets, size_t m, float *out,
                                         void *stream) {
    MK_REQUIRE(packed_ptrs && scales_ptrs && codes && exps && offsets && out, "null pointer");
    return mk_mxfp4_grouped_gemm_n(1, &packed_ptrs, &scales_ptrs, n_groups, rows, cols, codes, exps, offsets, m, &out, stream, nullptr, false);
}

extern "C" int mk_dev_mxfp4_grouped_gemm_split(const uint8_t *const *packed_ptrs, const uint8_t *const *scales_ptrs, size_t n_groups, size_t rows,
                                               size_t cols, const uint8_t *codes, const uint8_t *exps, const int32_t *offsets, size_t m,
                                               float *out, void *stream) {
    MK_REQUIRE(packed_ptrs && scales_ptrs && codes && exps && offsets && out, "null pointer");
    if (cols == 0 || cols % 512 != 0 || rows * (cols / 2) >= 0xFFFFFFFFull || m * cols * 2 >= 0xFFFFFFFFull) {
        mk_set_error("the two-term grouped product takes cols in multiples of 512 and operands below 4 GiB");
        return MK_ERR_UNSUPPORTED;
    }
    MK_REQUIRE(((uintptr_t)exps & 15) == 0, "exps must be 16-byte aligned");
    return mk_mxfp4_grouped_gemm_n(1, &packed_ptrs, &scales_ptrs, n_groups, rows, cols, codes, exps, offsets, m, &out, stream, nullptr, true);
}
