/*
 * mk_hip.h -- C ABI of libmk_hip.so: microkimi's quantized-weight hot path on
 * one AMD MI355X (gfx950).  Plain pointers and sizes only; no C++ or torch types.
 *
 * Two levels:
 *
 *   mk_dev_*   device level.  Every pointer is DEVICE memory, `stream` is a
 *              hipStream_t passed as void* (NULL = the default stream).  The call
 *              enqueues kernels and returns; nothing is allocated or synchronised.
 *              This is the level a resident engine (weights and activations kept
 *              in HBM) binds, and the level the benchmark measures.
 *
 *   mk_*       host level: the drop-in for the reference's operator entry points.
 *              Pointers are HOST memory, as the Rust slices are; weights are
 *              uploaded once into a device cache keyed by (pointer, rows, cols)
 *              exactly like the reference's Metal weight cache
 *              (src/metal.rs:874-936), inputs and outputs are staged per call and
 *              the call returns after the result is in `out`.
 *
 * There is NO CPU fallback in this library: when no device is present or a HIP
 * call fails the function returns a negative status, leaves `out` untouched and
 * mk_last_error() says why.  (The reference's Metal path falls back to its CPU
 * kernels, src/metal.rs:949-960; a caller that wants that keeps its own CPU path
 * and takes it on a negative status.)
 *
 * Status: 0 = done on the GPU, < 0 = error, nothing written.
 * All entry points are thread-safe; host-level calls serialise on one lock, as
 * the reference's Metal path does (src/metal.rs:432-439).
 */
#ifndef MK_HIP_H
#define MK_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MK_OK 0
#define MK_ERR_INVALID (-1)     /* bad argument (shape, alignment, null pointer) */
#define MK_ERR_NO_DEVICE (-2)   /* no gfx950 device / mk_init not possible */
#define MK_ERR_HIP (-3)         /* a HIP runtime call failed */
#define MK_ERR_UNSUPPORTED (-4) /* valid request the kernels do not cover */
#define MK_ERR_NOMEM (-5)       /* device cache budget or allocation exhausted */

/* Arithmetic of the MXFP4 matvec, the reference's q8 toggle (src/q8.rs:71-89):
 * MK_MODE_Q8  activation quantized to q8 per 32, exact integer block dots (reference default)
 * MK_MODE_F32 exact f32 path (MICROKIMI_NO_Q8=1 / force_q8(0)) */
#define MK_MODE_F32 0
#define MK_MODE_Q8 1

/* Activation rule of a packed expert (see mk_dev_moe_decode). */
#define MK_ACT_SWIGLU 0 /* silu(g) * u, silu(x) = x / (1 + exp(-x))            (src/deepseek.rs:1086) */
#define MK_ACT_SITU 1   /* 4 tanh(g/4) sigmoid(g) * 25 tanh(u/25)                (src/model.rs:619-621)  */
#define MK_ACT_DS 2     /* w * silu(min(g,L)) * clamp(u,-L,L), weight before W2  (src/deepseek.rs:1083-1087) */

/* ------------------------------------------------------------- lifecycle */

/* Replaces metal::gpu_available / init_ctx (src/metal.rs:445-593): binds the
 * library to HIP device `device` (first call wins; later calls return the same
 * status).  mk_available() = 1 once a gfx950 device is bound. */
int mk_init(int device);
int mk_available(void);
void mk_shutdown(void);
const char *mk_last_error(void);
/* The process-wide off switch, the counterpart of the reference's A/B override (mxfp4::no_packed_gpu,
 * src/mxfp4.rs:327-333, MICROKIMI_NO_PACKED_GPU=1): after mk_set_enabled(0), or with MK_HIP=0 in the
 * environment at the first call, every entry point that returns a status returns MK_ERR_NO_DEVICE before it makes any HIP
 * call, and mk_available() is 0, so a caller's existing CPU path takes over.  mk_set_enabled(1) switches back on (it also
 * overrides MK_HIP=0).  mk_enabled_now() reads the switch.  Work already queued on a stream is not affected. */
void mk_set_enabled(int on);
int mk_enabled_now(void);
/* Device-cache budget in MiB for the host-level weight cache (MICROKIMI_GPU_CACHE_MB,
 * src/metal.rs:554-558).  0 = unlimited (default). */
void mk_set_cache_mb(size_t mb);
/* q8::force_q8 / q8::q8_enabled (src/q8.rs:77-89): -1 follows the environment
 * (MICROKIMI_NO_Q8=1 selects the f32 path), 0 forces f32, 1 forces q8. */
void mk_force_q8(int v);
int mk_q8_enabled(void);

/* ---------------------------------------------------- device level: codec */

/* mxfp4::dequant (src/mxfp4.rs:19-31) = dequant::dequant_fp4 (src/dequant.rs:43-45).
 * packed [rows][cols/2] u8 (low nibble = even column), scales [rows][cols/32] e8m0,
 * out [rows][cols] f32, bit-exact (nibble 8 gives -0.0, byte 0 gives 2^-127). */
int mk_dev_mxfp4_dequant(const uint8_t *packed, const uint8_t *scales, size_t rows, size_t cols, float *out, void *stream);

/* dequant::dequant_fp8 (src/dequant.rs:27-39): e4m3fn bytes [rows][cols] with e8m0
 * scales per 128x128 block -> f32, bit-exact. */
int mk_dev_fp8_dequant(const uint8_t *w, const uint8_t *scales, size_t rows, size_t cols, float *out, void *stream);

/* q8::quantize_q8_into (src/q8.rs:49-69) for `nvec` vectors of `n` floats each
 * (n % 32 == 0): q [nvec][n] i8, scales [nvec][n/32] f32.  dx = max|x|/127,
 * q = round-half-away(x/dx) clamped to +-127, zero block -> scale 0.
 * x must be 16-byte aligned, q 4-byte aligned. */
int mk_dev_quantize_q8(const float *x, size_t nvec, size_t n, int8_t *q, float *scales, void *stream);

/* deepseek::fp8_roundtrip with block 32 (src/deepseek.rs:312-322) kept in coded
 * form: codes [nvec][n] e4m3 bytes, exps [nvec][n/32] e8m0 bytes (MXFP8).  This
 * is the activation format of mk_dev_mxfp4_grouped_gemm. */
int mk_dev_quantize_mxfp8(const float *x, size_t nvec, size_t n, uint8_t *codes, uint8_t *exps, void *stream);

/* bfloat16 (round to nearest even) of `nvec` rows of `n` floats, every value as the sum of TWO e4m3 terms with an e8m0
 * block exponent each per 32 values: hi = the leading four significant bits of the bfloat16 value, lo = the other four;
 * hi * 2^(eh - 127) + lo * 2^(el - 127) is the bfloat16 value exactly unless it lies more than 2^13 below the largest of
 * its block (then its last bits round off, an error below 2^-17 of that largest value); a value that is not finite
 * becomes the e4m3 NaN.  Layout per row and K tile of 512 values: codes [n / 512][2][512] (hi row, lo row), exps
 * [n / 512][2][16].  This is the activation format of mk_dev_mxfp4_grouped_gemm_split and, inside, of
 * mk_dev_moe_prefill_bf16: bfloat16 activations on the block-scaled matrix instruction (no counterpart in the
 * reference, whose prefill is f32: src/model.rs:2412-2447).  n % 512 == 0; x 16-byte, codes 8-byte aligned. */
int mk_dev_quantize_bf16_split(const float *x, size_t nvec, size_t n, uint8_t *codes, uint8_t *exps, void *stream);

/* mxfp4::quantize (search != 0) / quantize_naive (search == 0) (src/mxfp4.rs:38-138): per 32-group
 * e = ceil(log2(maxabs / 6)) clamped to [-127, 128], with `search` the better of e - 1, e, e + 1 by squared error in f64
 * (e wins ties), nearest E2M1 level by the midpoints, sign from the sign bit.  w [rows][cols] f32 ->
 * packed [rows][cols/2], scales [rows][cols/32]: the reference's bytes.  An offline path (weights arrive quantized).
 * w and packed 16-byte aligned. */
int mk_dev_mxfp4_quantize(const float *w, size_t rows, size_t cols, int search, uint8_t *packed, uint8_t *scales, void *stream);

/* MXFP4SQ, the quadratic-scale storage variant (src/mxfp4.rs:140-229; dtype 4 of the weight file): e2m1 nibbles and
 * groups of 32 as MXFP4, the scale byte q decodes to ((q + 1) / 256)^2 * smax with smax = max over the tensor's groups
 * of maxabs / 6 (the trailing f32 of a dtype-4 blob).
 *   _quantize  mxfp4::quantize_sq: q = ceil(256 sqrt(ideal / smax)) - 1 clamped to 0..255 (rounded up: nothing clips);
 *              smax is written to a device float.  The reference's bytes.
 *   _dequant   mxfp4::dequant_sq, bit-exact; smax from the device float smax_dev, or, when that is NULL, the value
 *              `smax`.  With a dtype-4 blob (packed || scales || smax) this is mxfp4::dequant_any's second branch.
 * The runtime matvecs read MXFP4 only, as in the reference (src/mxfp4.rs:150-151). */
int mk_dev_mxfp4sq_quantize(const float *w, size_t rows, size_t cols, uint8_t *packed, uint8_t *scales, float *smax, void *stream);
int mk_dev_mxfp4sq_dequant(const uint8_t *packed, const uint8_t *scales, const float *smax_dev, float smax, size_t rows, size_t cols,
                           float *out, void *stream);

/* dequant::quantize_fp8 (src/dequant.rs:50-74): e4m3fn codes with one e8m0 scale per 128x128 block,
 * e = ceil(log2(maxabs / 448)) clamped to [-127, 8].  rows and cols multiples of 128; qw [rows][cols],
 * scales [rows/128][cols/128]: the reference's bytes. */
int mk_dev_quantize_fp8(const float *w, size_t rows, size_t cols, uint8_t *qw, uint8_t *scales, void *stream);

/* ------------------------------------------- device level: MXFP4 matvecs */

/* mxfp4::matvec_packed_q8 (src/mxfp4.rs:405-443): out[r] = sum_g idot_g * (2^(sb_g-128) * xs_g).
 * cols % 32 == 0; packed, xq 16-byte aligned. */
int mk_dev_mxfp4_matvec_q8(const uint8_t *packed, const uint8_t *scales, size_t rows, size_t cols, const int8_t *xq, const float *xs,
                           float *out, void *stream);

/* mxfp4::matvec_packed, exact f32 path (src/mxfp4.rs:488-538): out[r] = sum_g (sum_j E2M1[nib]*x) * 2^(sb_g-127). */
int mk_dev_mxfp4_matvec_f32(const uint8_t *packed, const uint8_t *scales, size_t rows, size_t cols, const float *x, float *out,
                            void *stream);

/* mxfp4::matvec_packed (src/mxfp4.rs:458-539), the operator entry point: mode
 * MK_MODE_Q8 quantizes x (into `xq_ws`, `xs_ws`: device scratch of cols bytes and
 * cols/32 floats supplied by the caller) and runs the integer path; MK_MODE_F32
 * ignores the scratch. */
int mk_dev_mxfp4_matvec(const uint8_t *packed, const uint8_t *scales, size_t rows, size_t cols, const float *x, float *out, int mode,
                        int8_t *xq_ws, float *xs_ws, void *stream);

/* matvec_packed_q8 (src/mxfp4.rs:405-443) for m activation rows against ONE matrix, the weights read once for all of
 * them, on the block-scaled matrix cores with the reference's block terms bit for bit:
 *   out[i][r] = sum_g (idot_g as f32) * (2^(sb_g - 128) * xs[i][g])      (only the order of the sum over g differs)
 * xq [m][cols] int8 and xs [m][cols/32] f32 as quantize_q8 gives them, out [m][rows]; cols % 512 == 0.
 * workspace: 256 bytes of device memory, 256-byte aligned (the one-group description the grouped kernel reads).
 * The MoE decode layer uses the same kernel for the tokens that share an expert (from 4 tokens per call). */
int mk_dev_mxfp4_matvec_q8_batched(const uint8_t *packed, const uint8_t *scales, size_t rows, size_t cols, const int8_t *xq,
                                   const float *xs, size_t m, void *workspace, float *out, void *stream);

/* The same q8 matvec over `nmat` matrices of one shape in ONE launch: the
 * grouped-expert form.  packed_ptrs / scales_ptrs / out_ptrs: device arrays of
 * nmat device pointers; xq [nx][cols], xs [nx][cols/32]; x_index[nmat] (device,
 * may be NULL = all use vector 0) picks the activation of each matrix. */
int mk_dev_mxfp4_matvec_q8_grouped(const uint8_t *const *packed_ptrs, const uint8_t *const *scales_ptrs, size_t nmat, size_t rows,
                                   size_t cols, const int8_t *xq, const float *xs, const int32_t *x_index, float *const *out_ptrs,
                                   void *stream);

/* model::matvec_packed_nt (src/model.rs:2412-2447): exact-f32 batched matvec.
 * x [m][cols] position-major (the kernel needs no transposed copy and no
 * padding to 8), out [m][rows]. */
int mk_dev_mxfp4_matvec_nt(const uint8_t *packed, const uint8_t *scales, size_t rows, size_t cols, const float *x, size_t m, float *out,
                           void *stream);

/* ------------------------------------------------- device level: q8 head */

/* Q8Head::matvec / row_dot (src/model.rs:290-347) on `batch` already-quantized
 * activations: out[b][r] = sum_g (ws[r][g] * xs[b][g]) * idot.
 * q [rows][cols] i8; scales [rows][cols/32], f16 when scales_f16 != 0 (the q8_0
 * storage form) else f32 (the reference's in-memory form); xq [batch][cols],
 * xs [batch][cols/32]; out [batch][rows].  batch <= 8. */
int mk_dev_q8_matvec(const int8_t *q, const void *scales, int scales_f16, size_t rows, size_t cols, const int8_t *xq, const float *xs,
                     size_t batch, float *out, void *stream);

/* The greedy token of model::top_k_probs (src/model.rs:3271-3291): index of the
 * largest logit per row, ties to the lowest index.  logits [batch][n];
 * ws: device scratch of 2 * batch * 1024 * 4 bytes; out_idx [batch] int32. */
int mk_dev_argmax(const float *logits, size_t batch, size_t n, void *ws, int32_t *out_idx, void *stream);

/* Q8Head::from_f32 (src/model.rs:274-286) on device: row-wise q8_0 of w [rows][cols];
 * scales written as f16 (scales_f16 != 0; the rounded value is what the matvec
 * then uses) or f32.  w must be 16-byte aligned, q 4-byte aligned. */
int mk_dev_q8head_from_f32(const float *w, size_t rows, size_t cols, int8_t *q, void *scales, int scales_f16, void *stream);

/* ------------------------------------------------ device level: MoE layer */

/* Expert table: device arrays of per-expert device pointers, indexed by expert
 * id.  w1, w3: [inter][d] (gate, up); w2: [d][inter] (down); each MXFP4 as
 * (packed, scales) in the reference layout.  n_experts: entries per array; when
 * it is not 0 a routed id outside [0, n_experts) selects nothing (the pair adds
 * nothing to its token's row), with 0 the ids are trusted. */
typedef struct {
    const uint8_t *const *w1p, *const *w1s;
    const uint8_t *const *w3p, *const *w3s;
    const uint8_t *const *w2p, *const *w2s;
    size_t d, inter;
    size_t n_experts;
    /* A layer with VQ1 ("cold") experts (src/model.rs:729-730, 2243-2257): the file's global 256 x 16 f32 codebook on the
     * device, or NULL when every expert is MXFP4.  A VQ1 expert has its index bytes ([rows][cols/16]) where the packed
     * nibbles would be (w1p, w3p, w2p) and NULL scale pointers (w1s, w3s, w2s). */
    const float *vq_codebook;
    /* Optional (NULL: not there; both or none): per expert, the matrices once more in the order the one-launch decode
     * kernel streams them (mk_dev_moe_pack_gate_up -> w13t, mk_dev_moe_pack_down -> w2t).  With them, up to 3 decode tokens in
     * q8 mode at d = 7168 or 5120, inter = 2048 on a 256-CU device take the one-launch form of the layer (see
     * mk_dev_moe_decode); such calls must not overlap on one device. */
    const uint8_t *const *w13t, *const *w2t;
    /* Optional (NULL: not there; each on its own): per expert, the scale bytes of W1, W3, W2 once more in K-tile order
     * (mk_dev_mxfp4_scales_by_tile; d % 512 == 0 for W1 and W3, inter % 512 == 0 for W2; 1/16 of the experts' bytes again).
     * The matrix-core kernels of mk_dev_moe_decode (from 4 tokens) and of mk_dev_moe_prefill then read these instead of
     * w1s, w3s, w2s: same bytes, same results, whole 128-byte lines per K tile instead of an eighth of eight lines. */
    const uint8_t *const *w1st, *const *w3st, *const *w2st;
} mk_expert_table;

/* out[(t * rows + r) * 16 + j] = scales[r * (cols / 32) + 16 t + j]: the scale bytes ([rows][cols / 32], src/mxfp4.rs:1-3) with the 16
 * bytes a row has per 512 columns kept together and the rows of one such K tile adjacent.  cols % 512 == 0; both 16-byte
 * aligned; rows * cols / 32 bytes. */
int mk_dev_mxfp4_scales_by_tile(const uint8_t *scales, size_t rows, size_t cols, uint8_t *out, void *stream);

/* The experts of a layer in the operand order of v_mfma_scale_f32_16x16x128_f8f6f4, for the one-launch decode kernel: the
 * same bytes as (packed, scales) in another order -- mk_dev_moe_unpack_* restores the reference layout byte for byte
 * (src/mxfp4.rs:1-3), so mxfp4::dequant of the restored matrices is the reference's bit for bit.
 *   gate/up pack (W1 and W3 [inter][d] together): chunk (t, s) = rows 8 t .. 8 t + 7 of W1 and of W3, columns 128 s .. + 127, 64 lanes
 *     x 16 bytes: the 32-block b of row r of matrix m (0: W1, 1: W3) sits at lane (r % 8 + 8 m) + 16 (b % 4) of chunk
 *     ci = (r / 8) * (d / 128) + b / 4.  Two chunks share a 2176-byte container: chunk ci at (ci >> 1) * 2176 + (ci & 1) * 1024,
 *     lane l at + 16 l, its scale byte at (ci >> 1) * 2176 + 2048 + 2 l + (ci & 1).  d % 256 == 0, inter % 8 == 0;
 *     2 * inter * d / 32 * 17 bytes.
 *   down pack (W2 [d][inter]): the rows in 256 groups of rw = d / 256 (17 .. 32); one K step of a group (128 columns) is
 *     STEP = (1024 + 64 rb + 64 + 4 rb) rounded up to 128 bytes, rb = rw - 16, at (group * (inter / 128) + b / 4) * STEP: row
 *     i < 16 of the group has its block at 16 (i + 16 (b % 4)) and its scale byte at 1024 + 64 rb + i + 16 (b % 4); row
 *     i >= 16 at 1024 + 16 ((b % 4) rb + i - 16) and 1024 + 64 rb + 64 + (b % 4) rb + i - 16; the padding is zero.
 *     256 * (inter / 128) * STEP bytes.
 * mk_moe_pack_bytes(d, inter, down): the size of the gate/up pack (down == 0) or of the down pack (0: d not covered). */
size_t mk_moe_pack_bytes(size_t d, size_t inter, int down);
int mk_dev_moe_pack_gate_up(const uint8_t *w1p, const uint8_t *w1s, const uint8_t *w3p, const uint8_t *w3s, size_t d, size_t inter,
                            uint8_t *pack, void *stream);
int mk_dev_moe_unpack_gate_up(const uint8_t *pack, size_t d, size_t inter, uint8_t *w1p, uint8_t *w1s, uint8_t *w3p, uint8_t *w3s,
                              void *stream);
int mk_dev_moe_pack_down(const uint8_t *w2p, const uint8_t *w2s, size_t d, size_t inter, uint8_t *pack, void *stream);
int mk_dev_moe_unpack_down(const uint8_t *pack, size_t d, size_t inter, uint8_t *w2p, uint8_t *w2s, void *stream);

/* Bytes of device scratch mk_dev_moe_decode needs for B tokens of topk(+shared) experts. */
size_t mk_moe_decode_workspace_bytes(size_t B, size_t topk, int has_shared, size_t d, size_t inter);
/* Further bytes, directly behind those, when the table has a vq_codebook (the LUT GEMV's tables). */
size_t mk_moe_decode_vq_workspace_bytes(size_t B, size_t topk, int has_shared, size_t d, size_t inter);

/* The expert section of moe_forward / ds_moe for B decode tokens in one grouped
 * pass (src/model.rs:2227-2264,2346-2351; src/deepseek.rs:1069-1106):
 *   per token t and slot s: e = ids[t][s];
 *     a = W1_e x_t ; u = W3_e x_t ; act = ACT(a, u) ; o = W2_e act     (matvec_packed, `mode`)
 *   out_t = sum_s w[t][s] * o   in slot order   (MK_ACT_DS: plain sum, weight inside act)
 *         + o(shared expert)    when shared >= 0, unweighted.
 * ids [B][topk] int32, weights [B][topk] f32, x [B][d], out [B][d]; all device.
 * mode MK_MODE_Q8 re-quantizes x and act per 32 exactly as matvec_packed does on
 * each call.  A selected expert that is VQ1 (table->vq_codebook set, NULL scale pointers) takes quant::matvec_vq
 * (src/quant.rs:333-346) for its three products, on the f32 hidden and activation rows, whatever `mode` says
 * (src/model.rs:2243-2257); the workspace then also holds mk_moe_decode_vq_workspace_bytes.
 * Kernels by batch (q8 mode, MXFP4 experts, model-like shapes): 1-3 tokens with the table's packed copies (w13t, w2t):
 * ONE launch of one resident workgroup per CU -- every workgroup takes 8 rows of W1 and W3 of every pair, publishes their
 * activation values through the workspace (8-byte units that carry the launch's tag), then takes d / 256 rows of W2 of
 * every pair; every wait is bounded, a workgroup that gives up writes NaN to its rows and raises the flag that
 * mk_dev_moe_decode_gave_up reads.  Without the copies: a gate/up launch and a down launch.  From 4 tokens: the pairs
 * grouped by expert on the matrix cores.
 * Every form adds the reference's block terms (src/mxfp4.rs:405-443); only the order of the sum over blocks differs. */
int mk_dev_moe_decode(const mk_expert_table *table, size_t B, size_t topk, const int32_t *ids, const float *weights, int shared,
                      const float *x, int mode, int act_kind, float limit, void *workspace, float *out, void *stream);
/* *flag = 1 if a workgroup of the one-launch form ever gave up waiting on this device (its rows are NaN), else 0.
 * Synchronous (a device-to-host copy).  A give-up means that the launch did not have the device to itself (calls that
 * overlapped, or a bound set too low with MK_MOE_SPIN_LIMIT); the call that follows a give-up on the same workspace is
 * not to be trusted either (a late workgroup of the failed launch may have tagged its values for the next one): check
 * the flag, then drop both results.  Has no counterpart in the reference. */
int mk_dev_moe_decode_gave_up(int *flag);
/* count[0] (device int32) = how many of the n routed ids lie outside [0, n_experts): the pairs that the decode and prefill
 * calls skip when the table states its size.  The reference would panic on such an index (a slice index out of range,
 * src/model.rs:2243); a caller that wants to know asks here, on the same stream.  Asynchronous. */
int mk_dev_moe_count_bad_ids(const int32_t *ids, size_t n, size_t n_experts, int32_t *count, void *stream);

/* The two halves of mk_dev_moe_decode on their own, for callers that keep the reference's call structure (two
 * matvec_packed calls, the activation, then the third matvec_packed: src/model.rs:2246-2259, src/deepseek.rs:1080-1089)
 * and for stage-wise checks.  Arguments as mk_dev_moe_decode; the same kernels run.
 *   _act       act[(t * per + s)][inter] = ACT(W1_e x_t, W3_e x_t) for slot s of token t, per = topk (+ 1: the shared
 *              expert is the last slot); f32, before matvec_packed's own q8 step.
 *   _from_act  out_t from given activation rows in that layout (the q8 mode re-quantizes them per 32 exactly as
 *              matvec_packed does for W2), weighted sum in slot order. */
int mk_dev_moe_decode_act(const mk_expert_table *table, size_t B, size_t topk, const int32_t *ids, const float *weights, int shared,
                          const float *x, int mode, int act_kind, float limit, void *workspace, float *act, void *stream);
int mk_dev_moe_decode_from_act(const mk_expert_table *table, size_t B, size_t topk, const int32_t *ids, const float *weights, int shared,
                               const float *act, int mode, int act_kind, void *workspace, float *out, void *stream);

/* Router of the benchmark MoE layer on device: softmax over logits [B][n], top-k
 * with the reference's rule (strict '>' insertion: ties to the lowest index;
 * src/model.rs:2157-2173), weights renormalised.  ids [B][k] int32, weights [B][k]. */
int mk_dev_router_softmax_topk(const float *logits, size_t B, size_t n, size_t k, int32_t *ids, float *weights, void *stream);

/* The reference's three routing rules on given logits [B][n] (one call, B tokens):
 *   MK_ROUTER_SOFTMAX       score = key = softmax(l);               w = score / sum         (benchmark MoE layer)
 *   MK_ROUTER_SIGMOID       score = sigmoid(l), key = score + bias; w = score / (sum+1e-20) (src/model.rs:2151-2173)
 *   MK_ROUTER_SQRTSOFTPLUS  score = sqrt(softplus(l)), key = score + bias;
 *                           w = score / sum * route_scale                                   (src/deepseek.rs:16-58)
 * Selection: the k largest keys, strict '>' against the current worst, stable
 * (ties to the lowest index), in descending key order; sums run in that order.
 * bias [n] may be NULL.  ids [B][k] int32, weights [B][k]. */
#define MK_ROUTER_SOFTMAX 0
#define MK_ROUTER_SIGMOID 1
#define MK_ROUTER_SQRTSOFTPLUS 2
int mk_dev_router_topk(const float *logits, size_t B, size_t n, size_t k, int kind, const float *bias, float route_scale, int32_t *ids,
                       float *weights, void *stream);

/* model::rmsnorm / deepseek::ds_rmsnorm (src/model.rs:599-605, src/deepseek.rs:241-248) for B rows of d floats:
 *   ss = dot(x, x) / d;  inv = 1 / sqrt(ss + eps);  y[i] = x[i] * inv * w[i]
 * with the reference's dot contract (src/model.rs:46-82) replayed operation for operation: y is bit-identical.
 * out [B][d] may be NULL.  When q and scales are given (both or neither), y is also quantized as
 * q8::quantize_q8_into does (src/q8.rs:49-69): q [B][d] i8, scales [B][d/32] f32, d % 32 == 0 -- the input the
 * q8-mode matvecs take, so norm -> quantize -> matvec needs no pass over y in between. */
int mk_dev_rmsnorm(const float *x, size_t B, size_t d, const float *w, float eps, float *out, int8_t *q, float *scales, void *stream);

/* model::matvec_cpu (src/model.rs:214-222): out[b][r] = dot(w[r], x[b]) for a row-major f32 matrix [rows][cols]
 * and B vectors, with the reference's dot contract replayed operation for operation (bit-identical; each lane
 * walks a sequential chain of cols/8 additions, so this is meant for the small matrices of a layer: router
 * gate, latent projections). */
int mk_dev_matvec_f32(const float *w, size_t rows, size_t cols, const float *x, size_t B, float *out, void *stream);

/* The three calls above as a decode step runs them in front of its expert section (src/model.rs:2151-2173 after the
 * layer's rmsnorm: norm, router gate matvec, routing) as ONE call of two launches: xn = rmsnorm(x) and logits = gate xn in
 * the first (every workgroup norms the rows itself: that costs less than a launch), (ids, weights) = route(logits) in the
 * second.  Every value is the one the separate calls give, bit for bit (the same operations in the same order).
 * x [B][d], norm_w [d], gate [n_experts][d] f32 row-major, bias [n_experts] or NULL; xn [B][d] (may be NULL), logits
 * [B][n_experts] (always written), ids / weights [B][k].  d % 8 == 0 and 512 <= d <= 32768, else MK_ERR_UNSUPPORTED
 * (use the three calls).  From 5 tokens the call runs the three kernels one after the other (norming the rows once is
 * then cheaper) and needs xn.  Has no single counterpart in the reference. */
int mk_dev_norm_gate_route(const float *x, size_t B, size_t d, const float *norm_w, float eps, const float *gate, size_t n_experts, size_t k,
                           int kind, const float *bias, float route_scale, float *xn, float *logits, int32_t *ids, float *weights,
                           void *stream);

/* ------------------------------------------- device level: MLA attention */

/* mla_attn_flash_q8_mqa (src/model.rs:1804-1908) in the weight-absorbed form:
 * one shared q8_0 latent row per position is K (with the rope row) and V of
 * every head.
 *   lat_q [n][L] i8, lat_s [n][L/32] f16; rope_q [n][R] i8, rope_s [n][R/32] f16
 *   q [nh][L+R] f32 (latent part first), out [nh][L] f32
 * score = (dot(q_rope, dequant(rope)) + sum_g (qs_g*ks_g)*idot_g) * scale over the
 * q8-quantized latent query; online softmax; out = sum p * dequant(latent) / l.
 * Positions 0..=pos are attended (pos < n).  L a multiple of 64 up to 512; R 0, 32 or 64.
 * workspace: mk_mla_decode_workspace_bytes(nh, L, pos + 1). */
size_t mk_mla_decode_workspace_bytes(size_t nh, size_t L, size_t n_pos);
int mk_dev_mla_q8_decode(const int8_t *lat_q, const void *lat_s, const int8_t *rope_q, const void *rope_s, size_t pos, const float *q,
                         size_t nh, size_t L, size_t R, float scale, void *workspace, float *out, void *stream);

/* mk_dev_mla_q8_decode for callers that cannot allocate or carry a workspace: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same arguments without
 * the workspace: the kernels' scratch (quantized query, the context splits' partial outputs and their softmax
 * statistics) lives in a device array inside the library, 16 916 480 bytes that every GPU the library runs on holds
 * until the process ends.  Limits: nh <= 128 (mk_mla_decode_static_max_heads) and L <= 512; beyond them the call
 * returns MK_ERR_UNSUPPORTED and writes nothing.  It calls no hipMalloc / hipFree and no allocating library routine.
 * All calls on one GPU share the one array: calls that overlap on a GPU (two streams, two threads) race -- issue them
 * on one stream or order them with events.  Nothing in the array needs clearing between calls (every word a call
 * reads was written by that call).  mk_init resolves the array's device address; without mk_init the first call on a
 * device does, so make that first call outside a graph capture. */
size_t mk_mla_decode_static_max_heads(void);
int mk_dev_mla_q8_decode_static(const int8_t *lat_q, const void *lat_s, const int8_t *rope_q, const void *rope_s, size_t pos, const float *q,
                                size_t nh, size_t L, size_t R, float scale, float *out, void *stream);

/* MlaCache::push (src/model.rs:1583-1618) for the shared-latent cache: quantize
 * one position (latent [L] f32, rope [R] f32) into row `pos` of the cache arrays.
 * latent and rope must be 16-byte aligned. */
int mk_dev_mla_cache_append(const float *latent, const float *rope, size_t L, size_t R, size_t pos, int8_t *lat_q, void *lat_s,
                            int8_t *rope_q, void *rope_s, void *stream);

/* The cache layout the reference keeps (MlaCache, src/model.rs:765-781): per position
 *   kq [nh][nope] i8, ks [nh][nope/32] f32   latent part of K per head
 *   kr [rope] f32                             rope part of K, shared by the heads, never quantized
 *   vq [nh][vd] i8, vs [nh][vd/32] f32        V per head
 * positions contiguous in each array.  nope a multiple of 32 up to 256, vd a multiple of 32 up to 512.  The Hadamard
 * option (MICROKIMI_KV_HADAMARD, off by default) is not built.
 *
 * _append   MlaCache::push (src/model.rs:1583-1618) for n_new positions into rows pos0 .. pos0 + n_new - 1 (n_new > 1
 *           is MlaCache::assign_f32, src/model.rs:1680-1692): k_rows [n_new][nh][nope+rope] (latent part first per
 *           head; the rope row is taken from head 0), v_rows [n_new][nh][vd].
 * _to_f32   MlaCache::to_f32 (src/model.rs:1623-1676): k [n][nh][nope+rope], v [n][nh][vd].
 * _q8_attn  mla_attn_flash_q8_mqa (src/model.rs:1804-1908) for m queries q [m][nh][nope+rope]: query i attends the
 *           positions 0 ..= pos0 + i (m = 1: the decode step of mla_forward, src/model.rs:1980-1985; m > 1: the
 *           per-position loop of mla_prefill, src/model.rs:2080-2102).  out [m][nh][vd].
 *           workspace: mk_mla_heads_workspace_bytes(m, nh, nope, vd).  At the reference's own head shape (nope 128, rope 64,
 *           vd 128) one query streams the cache once for all heads and 16 or more queries share every K / V tile on the
 *           matrix cores; other shapes take a per-head kernel.  The results do not depend on which one runs beyond the
 *           order of the sums.
 * hadamard  nonzero: the cache is kept in the rotated form of kv_hadamard (src/model.rs:1529-1554, MICROKIMI_KV_HADAMARD=1):
 *           hadamard64 on every 64-chunk of a K-nope row, a V row and the query's nope part before quantization, the
 *           factor 1/64 on the latent score, the output rotated back.  As in the reference it takes effect only when
 *           nope and vd are multiples of 64.  All three calls of a cache must agree on it. */
int mk_dev_mla_heads_append(const float *k_rows, const float *v_rows, size_t n_new, size_t nh, size_t nope, size_t rope, size_t vd,
                            size_t pos0, int hadamard, int8_t *kq, float *ks, float *kr, int8_t *vq, float *vs, void *stream);
int mk_dev_mla_heads_to_f32(const int8_t *kq, const float *ks, const float *kr, const int8_t *vq, const float *vs, size_t n, size_t nh,
                            size_t nope, size_t rope, size_t vd, int hadamard, float *k, float *v, void *stream);
size_t mk_mla_heads_workspace_bytes(size_t m, size_t nh, size_t nope, size_t vd);
int mk_dev_mla_heads_q8_attn(const int8_t *kq, const float *ks, const float *kr, const int8_t *vq, const float *vs, size_t pos0,
                             const float *q, size_t m, size_t nh, size_t nope, size_t rope, size_t vd, float scale, int hadamard,
                             void *workspace, float *out, void *stream);

/* ---------------------------------- device level: prefill expert GEMM */

/* The per-expert batched evaluation of moe_prefill (src/model.rs:2539-2602) as a
 * grouped GEMM on the block-scaled FP8/FP4 matrix cores.
 *   y[i][r] = sum_k dequant(W_e)[r][k] * dequant(xa)[i][k]  for the rows i of group e
 * xa: MXFP8 activations from mk_dev_quantize_mxfp8: codes [m][cols], exps [m][cols/32];
 * rows of one expert are contiguous: group e covers rows offsets[e] .. offsets[e+1].
 * packed_ptrs/scales_ptrs [n_groups]: the weight of each group; out [m][rows] f32. */
int mk_dev_mxfp4_grouped_gemm(const uint8_t *const *packed_ptrs, const uint8_t *const *scales_ptrs, size_t n_groups, size_t rows,
                              size_t cols, const uint8_t *codes, const uint8_t *exps, const int32_t *offsets, size_t m, float *out,
                              void *stream);

/* The same grouped product in the reference's own arithmetic, matvec_packed_nt per group (src/model.rs:2412-2447,
 * called per expert at src/model.rs:2580-2599): x [m][cols] f32, exactly dequantized weights, f32 products and sums on
 * the f32 matrix instruction (order of the sums apart: relative L2 below 1e-5).  cols % 128 == 0, rows % 4 == 0,
 * x and out 16-byte aligned; same offsets and out as above. */
int mk_dev_mxfp4_grouped_gemm_f32(const uint8_t *const *packed_ptrs, const uint8_t *const *scales_ptrs, size_t n_groups, size_t rows,
                                  size_t cols, const float *x, const int32_t *offsets, size_t m, float *out, void *stream);
/* And with bfloat16 activations x [m][cols] (the caller rounds them once): the weights are exact in bfloat16, the
 * products exact in f32 and summed in f32 on v_mfma_f32_16x16x32_bf16.  MK_ERR_UNSUPPORTED unless cols % 512 == 0 and
 * rows % 4 == 0. */
int mk_dev_mxfp4_grouped_gemm_bf16(const uint8_t *const *packed_ptrs, const uint8_t *const *scales_ptrs, size_t n_groups, size_t rows,
                                   size_t cols, const uint16_t *x, const int32_t *offsets, size_t m, float *out, void *stream);

/* mk_dev_mxfp4_grouped_gemm with bfloat16 token rows in the two-term form of mk_dev_quantize_bf16_split (codes
 * [m][cols / 512][2][512], exps [m][cols / 512][2][16], 16-byte aligned): both terms of a value meet the same weight
 * registers on v_mfma_scale_f32_16x16x128_f8f6f4 and are summed in f32, so y[i][r] = sum_k dequant(W_e)[r][k] * bf16(x)[i][k]
 * (matvec_packed_nt of src/model.rs:2412-2447 on bfloat16-rounded rows) up to the arithmetic of the instruction, which
 * keeps fewer bits of a step's 128 products than a chain of f32 additions would: relative L2 about 1e-5 over a group,
 * up to 3e-5 measured on single rows with a wide range of magnitudes (the bfloat16 rounding of the rows themselves is
 * 2e-3).  Groups of any size (passes of 32 rows).  MK_ERR_UNSUPPORTED unless cols % 512 == 0. */
int mk_dev_mxfp4_grouped_gemm_split(const uint8_t *const *packed_ptrs, const uint8_t *const *scales_ptrs, size_t n_groups, size_t rows,
                                    size_t cols, const uint8_t *codes, const uint8_t *exps, const int32_t *offsets, size_t m, float *out,
                                    void *stream);

/* Bytes of device scratch mk_dev_moe_prefill needs. */
size_t mk_moe_prefill_workspace_bytes(size_t T, size_t topk, size_t n_experts, size_t d, size_t inter);

/* Where mk_dev_moe_prefill keeps its intermediates inside the workspace (byte offsets from its start; valid after the
 * call has run, until the next one on that workspace).  P = T * topk pairs, "grouped row" = position of a pair after the
 * grouping by expert (src/model.rs:2539-2544).
 *   order   [P] int32      grouped row -> pair index t * topk + s
 *   pos     [P] int32      pair index -> grouped row, -1 for an expert id out of range
 *   offsets [n_experts+1]  int32: expert e owns the grouped rows offsets[e] .. offsets[e+1]
 *   g, u    [P][inter] f32 the gate and up projections per grouped row (before the activation): written by
 *                          mk_dev_moe_prefill_keep only (mk_dev_moe_prefill goes from the accumulators straight to the
 *                          activation's MXFP8 form and leaves these rows untouched)
 *   o       [P][d] f32     the down projection per grouped row, before the weighted sum */
typedef struct {
    size_t order, pos, offsets, g, u, o;
} mk_prefill_layout;
int mk_moe_prefill_workspace_layout(size_t T, size_t topk, size_t n_experts, size_t d, size_t inter, mk_prefill_layout *out);

/* The expert section of moe_prefill (src/model.rs:2528-2602, 2690-2700) for T
 * prompt positions: the (token, slot) pairs are grouped by expert (stable in
 * (token, slot) order), each used expert evaluates gate, up, activation and
 * down for its rows with mk_dev_mxfp4_grouped_gemm, and per token
 *   out_t = sum_s w[t][s] * o[t][s]   in slot order, multiply then add.
 * The gathered hidden rows and the activation enter the matrix cores as MXFP8
 * (deepseek::fp8_roundtrip per 32, src/deepseek.rs:312-322, with the block
 * exponent free to use the whole e8m0 range instead of that function's clamp at
 * 8, so that large activations do not saturate); the reference's own prefill is
 * the f32 arithmetic of matvec_packed_nt (mk_dev_mxfp4_matvec_nt), from which
 * this differs by the e4m3 rounding of the two inputs (2-3 % of a row's norm).
 * table entries 0..n_experts-1 are used; ids [T][topk] int32 (a pair whose id is
 * out of range contributes nothing), weights [T][topk], x [T][d], out [T][d].
 * act_kind MK_ACT_SWIGLU or MK_ACT_SITU.  d, inter multiples of 128; T * topk <= 16384
 * per call (a longer prompt is split by the caller).  MK_ERR_UNSUPPORTED for a table with VQ1 experts
 * (mk_dev_moe_prefill_f32 takes those). */
int mk_dev_moe_prefill(const mk_expert_table *table, size_t n_experts, size_t T, size_t topk, const int32_t *ids, const float *weights,
                       const float *x, int act_kind, void *workspace, float *out, void *stream);
/* The same call, the same kernels and the same result bit for bit, with the f32 gate and up rows stored as well (for
 * callers that inspect the intermediates, see mk_moe_prefill_workspace_layout). */
int mk_dev_moe_prefill_keep(const mk_expert_table *table, size_t n_experts, size_t T, size_t topk, const int32_t *ids, const float *weights,
                       const float *x, int act_kind, void *workspace, float *out, void *stream);

/* The same section in the reference's own arithmetic (matvec_packed_nt, src/model.rs:2412-2447, as moe_prefill calls
 * it at src/model.rs:2580-2599): f32 hidden rows and f32 activation against the exactly dequantized weights on the f32
 * matrix instruction, f32 products and sums.  Only the order of the sums inside a dot product differs from the
 * reference (relative L2 below 1e-5).  Same arguments, same workspace and same layout of the intermediates as
 * mk_dev_moe_prefill; afterwards g holds ACT(gate, up), u the up rows, o the down rows.  About four times the time of
 * the MXFP8 path at 512 tokens over 256 experts.  A table with a vq_codebook is taken too: the three products of a VQ1
 * expert (NULL scale pointers) are quant::matvec_vq_nt's (src/quant.rs:353-376, src/model.rs:2576-2593) with the
 * codebook entries as the weights, again with the order of the sums as the only difference. */
int mk_dev_moe_prefill_f32(const mk_expert_table *table, size_t n_experts, size_t T, size_t topk, const int32_t *ids, const float *weights,
                           const float *x, int act_kind, void *workspace, float *out, void *stream);

/* The same section with bfloat16 activations: the hidden rows and the activation rows are rounded to bfloat16 (nearest
 * even) once, the MXFP4 weights are exact, products exact and sums f32: the results are those of moe_prefill
 * (src/model.rs:2528-2602) on bfloat16-rounded inputs, about 2e-3 of a row's norm from the reference's f32 arithmetic
 * (the MXFP8 call differs by 2-5 %).  Two forms compute it.  The default keeps every bfloat16 value as two e4m3 terms
 * (mk_dev_quantize_bf16_split) and runs the block-scaled matrix instruction, v_mfma_scale_f32_16x16x128_f8f6f4, twice
 * per step against the same weight registers (the kernels of mk_dev_moe_prefill; gate, up, activation and its two-term
 * form in one launch): exact inputs, and the instruction's own arithmetic, which stays about 1e-5 (relative L2 of a row)
 * from f32 sums.  MK_PREFILL_BF16_MFMA=1 selects v_mfma_f32_16x16x32_bf16 with the weights converted exactly
 * (3e-7 from f32 sums, 1.2 times the time).  A hidden or activation value that is not finite makes the rows it enters
 * NaN.  Same arguments, workspace and intermediates as mk_dev_moe_prefill_f32 (g holds the gate rows here and u the
 * up rows: the activation is kept in its matrix-instruction form elsewhere in the workspace).  MK_ERR_UNSUPPORTED unless
 * d and inter are multiples of 512, and for a table with VQ1 experts.  Weights whose value lies below 2^-126 may be
 * flushed to zero by the hardware conversion (bf16 instruction form). */
int mk_dev_moe_prefill_bf16(const mk_expert_table *table, size_t n_experts, size_t T, size_t topk, const int32_t *ids, const float *weights,
                            const float *x, int act_kind, void *workspace, float *out, void *stream);

/* ---------------------------------------- device level: VQ1 / LUT GEMV */

/* Bytes of device scratch for the lookup tables of one activation: cols/16 tables of 256 f32. */
size_t mk_vq1_workspace_bytes(size_t cols);

/* quant::matvec_vq (src/quant.rs:333-346), i.e. lutgemv::matvec_vq_lut (src/lutgemv.rs:208-240):
 * out[r] = sum_c W[r][c] x[c] with W[r][16v .. 16v+16] = codebook[indices[r][v]].
 * codebook [256][16] f32 (the file's global "vq_codebook"), indices [rows][cols/16] u8, x [cols], out [rows].
 * Table entries are bit-identical to the reference's (sequential multiply-add chain).  exact != 0: each row adds its
 * table entries in ascending group order from 0 like the reference's sweep, and the result is bit-identical to
 * matvec_vq_lut / matvec_vq_gather; exact == 0: the sum over groups is split across the 64 lanes of a wave
 * (relative L2 error against the reference below 1e-5). */
int mk_dev_vq1_matvec(const float *codebook, const uint8_t *indices, size_t rows, size_t cols, const float *x, int exact,
                      void *workspace, float *out, void *stream);

/* quant::matvec_vq_nt (src/quant.rs:353-376), the batched form for prefill: xt [cols][m] (m inputs, transposed, m a
 * multiple of 8), out [m][rows] position-major.  Every product is added to its position's running sum in (vector, j)
 * order, multiply then add: bit-identical to the reference.  xt must be 16-byte aligned. */
int mk_dev_vq1_matvec_nt(const float *codebook, const uint8_t *indices, size_t rows, size_t cols, const float *xt, size_t m, float *out,
                         void *stream);

/* ------------------------------------------- MKIM weight files -> device */

/* Tensor dtypes of the file format (src/weights.rs:25-29). */
#define MK_DTYPE_F32 0
#define MK_DTYPE_MXFP4 1
#define MK_DTYPE_I32 2
#define MK_DTYPE_VQ1 3
#define MK_DTYPE_MXFP4SQ 4
#define MK_BIN_MAX_DIMS 8

/* weights::Entry (src/weights.rs:31-37): one directory entry. */
typedef struct mk_bin_entry {
    uint8_t dtype, n_dims;
    uint32_t dims[MK_BIN_MAX_DIMS];
    uint64_t offset, size; /* bytes from the start of the file */
} mk_bin_entry;

typedef struct mk_binfile mk_binfile;

/* BinFile::open / read_directory (src/weights.rs:424-500): parses "MKIM0001" or "MKIM0002"
 * (+ JSON config block) and the tensor directory, and maps the whole file read-only.  Every
 * entry is checked against blob_size (src/weights.rs:40-66) and the file length; a malformed
 * file gives MK_ERR_INVALID where the reference panics.  No GPU is touched. */
int mk_bin_open(const char *path, mk_binfile **out);
void mk_bin_close(mk_binfile *f);
size_t mk_bin_n_tensors(const mk_binfile *f);
/* Entry i in directory order; `name` points into the handle. */
int mk_bin_entry_at(const mk_binfile *f, size_t i, const char **name, mk_bin_entry *e);
/* entries.get(name) (src/weights.rs:601): MK_ERR_INVALID "missing tensor" when absent. */
int mk_bin_find(const mk_binfile *f, const char *name, mk_bin_entry *e);
/* BinFile::blob: pointer to the tensor's bytes inside the mapping (valid until mk_bin_close), or NULL. */
const void *mk_bin_blob(const mk_binfile *f, const char *name, size_t *size);
/* The MKIM0002 config block (not NUL-terminated inside the file; the returned copy is), or NULL for MKIM0001. */
const char *mk_bin_config_json(const mk_binfile *f, size_t *len);
/* BinFile::mxfp4_parts (src/weights.rs:619-627): packed [R][C/2] then scales [R][C/32] of one blob. */
int mk_bin_mxfp4_parts(const mk_binfile *f, const char *name, const uint8_t **packed, const uint8_t **scales, size_t *rows, size_t *cols);

typedef struct mk_expert_set mk_expert_set;

/* The routed experts of one MoE layer made resident on the current device: the tensors
 * "<layer_prefix>block_sparse_moe.experts.<e>.w1|w2|w3" for e < n_experts (the names resolved in
 * src/model.rs:979-989), each MXFP4 blob copied as stored (256-byte aligned; scales = packed +
 * R*C/2), plus the device pointer arrays of an mk_expert_table.  w1 of expert 0 fixes
 * [inter, d]; every other tensor is checked against it.  An expert stored as VQ1 (dtype 3, `slice --cold-vq`; its kind
 * is taken from w1 as in src/model.rs:988-990, w2 and w3 must agree) keeps its index bytes and a NULL scale pointer, and
 * the file's global "vq_codebook" (256 x 16 f32, src/model.rs:995-999) is uploaded with the set: table->vq_codebook.
 * MXFP4SQ experts (dtype 4) give MK_ERR_UNSUPPORTED: a storage format the runtime matvec does not read
 * (src/mxfp4.rs:150-151); such a layer stays on the caller's CPU path.  This replaces the pointer-keyed upload cache
 * of src/metal.rs:874-936 for callers that load whole layers. */
int mk_bin_load_experts(const mk_binfile *f, const char *layer_prefix, size_t n_experts, mk_expert_set **out);
const mk_expert_table *mk_expert_set_table(const mk_expert_set *s);
size_t mk_expert_set_count(const mk_expert_set *s);
size_t mk_expert_set_bytes(const mk_expert_set *s); /* device bytes held */
void mk_expert_set_free(mk_expert_set *s);

/* ------------------------------------------------------------ host level */

/* metal::gpu_matvec_fp4 (src/metal.rs:943-1017), i.e. the GPU branch of
 * mxfp4::matvec_packed (src/mxfp4.rs:467-473).  Host slices; the weight is
 * cached on device by (packed pointer, rows, cols) and re-validated against the
 * first 16 host bytes on every hit.  Arithmetic follows mk_q8_enabled(). */
int mk_mxfp4_matvec(const uint8_t *packed, const uint8_t *scales, size_t rows, size_t cols, const float *x, float *out);

/* metal::gpu_matvec (src/metal.rs:750-870), the GPU branch of model::matvec (src/model.rs:199-208): y = W x for a
 * row-major f32 matrix on host slices, the weight cached on the device like the packed ones.  The dot contract of
 * src/model.rs:46-82 is replayed: the result is bit-identical to matvec_cpu. */
int mk_matvec_f32(const float *w, size_t rows, size_t cols, const float *x, float *out);

/* GpuProf / gpu_prof_print (src/metal.rs:667-716): accumulated over the host-level matvecs while profiling is on
 * (MK_GPU_DEBUG=1 at mk_init, or mk_prof_enable(1)).  With profiling on the phases are separated by extra
 * synchronisations: cache = weight lookup / upload, io = input upload, launch = kernel enqueue, wait = until the
 * kernels are done, readback = result copy. */
typedef struct {
    uint64_t calls, hits, misses;
    double t_cache_ms, t_io_ms, t_launch_ms, t_wait_ms, t_readback_ms;
    size_t cache_tensors, cache_bytes;
} mk_prof;
void mk_prof_enable(int on);
void mk_prof_reset(void);
void mk_prof_get(mk_prof *out);
void mk_prof_print(void);

/* mxfp4::dequant on host slices (upload, kernel, download). */
int mk_mxfp4_dequant(const uint8_t *packed, const uint8_t *scales, size_t rows, size_t cols, float *out);

/* q8::quantize_q8_into on host slices. */
int mk_quantize_q8(const float *x, size_t n, int8_t *q, float *scales);

/* Q8Head (src/model.rs:261-348): built once, kept on device. */
typedef struct mk_q8head mk_q8head;
int mk_q8head_from_f32(const float *w, size_t rows, size_t cols, int scales_f16, mk_q8head **out);
int mk_q8head_from_q8(const int8_t *q, const float *scales, size_t rows, size_t cols, int scales_f16, mk_q8head **out);
/* logits for `batch` host rows x [batch][cols] -> out [batch][rows]; argmax_out (may be NULL) [batch] */
int mk_q8head_matvec(mk_q8head *h, const float *x, size_t batch, float *out, int32_t *argmax_out);
void mk_q8head_free(mk_q8head *h);

/* MlaCache (src/model.rs:765-781,1556-1692) kept on the device, in one of two layouts:
 *   mk_mla_cache_new        shared latent: per position one q8_0 latent row (L int8, f16 scales) that is K and V of every
 *                           head, and one q8_0 rope row (R int8, f16 scales) -- the weight-absorbed form.  L a multiple of
 *                           64 up to 512, R 32 or 64.  A position is given as (latent [L], rope [R]).
 *   mk_mla_cache_new_heads  the reference's own layout: per position and head a K-nope row and a V row (int8 + f32
 *                           scales) and one shared f32 rope row.  A position is given as the reference gives it to
 *                           MlaCache::push: (k_row [nh][nope+rope], v_row [nh][vd]).  The Hadamard option is read
 *                           from MICROKIMI_KV_HADAMARD when the cache is made, like kv_hadamard() (src/model.rs:1532-1535),
 *                           or set with mk_mla_cache_set_hadamard while the cache is empty.
 * row0 / row1 below are those two rows; rows0 / rows1 are n of them, position-major. */
typedef struct mk_mla_cache mk_mla_cache;
int mk_mla_cache_new(size_t nh, size_t L, size_t R, size_t capacity, mk_mla_cache **out);
int mk_mla_cache_new_heads(size_t nh, size_t nope, size_t rope, size_t vd, size_t capacity, mk_mla_cache **out);
/* MlaCache.had (src/model.rs:1567) of a cache in the reference's layout; MK_ERR_INVALID once positions are held */
int mk_mla_cache_set_hadamard(mk_mla_cache *c, int on);
/* MlaCache::push (src/model.rs:1583-1618) */
int mk_mla_cache_push(mk_mla_cache *c, const float *row0, const float *row1);
/* MlaCache::assign_f32 (src/model.rs:1680-1692): the cache is emptied and refilled from n f32 positions (snapshot restore) */
int mk_mla_cache_assign_f32(mk_mla_cache *c, const float *rows0, const float *rows1, size_t n);
size_t mk_mla_cache_positions(const mk_mla_cache *c);
/* MlaCache::to_f32 (src/model.rs:1623-1676): the dequantized rows q * s of all positions, in the shapes push takes */
int mk_mla_cache_to_f32(const mk_mla_cache *c, float *rows0, float *rows1);
/* mla_attn_flash_q8_mqa (src/model.rs:1804-1908) over positions 0 ..= positions-1: q [nh][L+R] (heads layout:
 * [nh][nope+rope]) host, out [nh][L] (heads layout: [nh][vd]) host */
int mk_mla_attn(mk_mla_cache *c, const float *q, float scale, float *out);
/* the attention loop of mla_prefill (src/model.rs:2080-2102) after the prompt's m positions have been pushed: query i
 * of q [m][nh][...] attends the positions 0 ..= positions - m + i; out [m][nh][...] */
int mk_mla_attn_prefill(mk_mla_cache *c, const float *q, size_t m, float scale, float *out);
void mk_mla_cache_free(mk_mla_cache *c);

#ifdef __cplusplus
}
#endif
#endif /* MK_HIP_H */
