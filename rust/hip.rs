//! hip.rs -- binding of libmk_hip.so (include/mk_hip.h) for the reference crate: the counterpart of src/metal.rs.
//!
//! Drop this file into `src/`, add `mod hip;` next to `mod metal;` in src/main.rs, a `hip` feature to Cargo.toml
//! (`[features] hip = []`) and `rust/build.rs` as the crate's build script.  The three entry points the reference
//! already calls on macOS keep their shapes, so the `cfg` branches at the top of `mxfp4::matvec_packed`
//! (src/mxfp4.rs:467-473) and `model::matvec` (src/model.rs:199-208) become
//!
//! ```ignore
//! #[cfg(feature = "hip")]
//! if model::gpu_on() && !no_packed_gpu() && rows * cols >= model::GPU_MIN_ELEMS && hip::gpu_available()
//!     && hip::gpu_matvec_fp4(packed, scales, rows, cols, x, out) { return; }
//! ```
//!
//! This file was written against the header and has not been compiled: the build image has no Rust toolchain.
#![allow(dead_code)]
use std::ffi::CStr;
use std::os::raw::{c_char, c_int, c_void};

pub const MK_OK: c_int = 0;
pub const MK_ERR_INVALID: c_int = -1;
pub const MK_ERR_NO_DEVICE: c_int = -2;
pub const MK_ERR_HIP: c_int = -3;
pub const MK_ERR_UNSUPPORTED: c_int = -4;
pub const MK_ERR_NOMEM: c_int = -5;
pub const MK_MODE_F32: c_int = 0;
pub const MK_MODE_Q8: c_int = 1;
pub const MK_ACT_SWIGLU: c_int = 0;
pub const MK_ACT_SITU: c_int = 1;
pub const MK_ACT_DS: c_int = 2;
pub const MK_ROUTER_SOFTMAX: c_int = 0;
pub const MK_ROUTER_SIGMOID: c_int = 1;
pub const MK_ROUTER_SQRTSOFTPLUS: c_int = 2;
pub const MK_BIN_MAX_DIMS: usize = 8;

/// mk_expert_table: device arrays of per-expert device pointers, indexed by expert id.
#[repr(C)]
#[derive(Clone, Copy)]
pub struct MkExpertTable {
    pub w1p: *const *const u8,
    pub w1s: *const *const u8,
    pub w3p: *const *const u8,
    pub w3s: *const *const u8,
    pub w2p: *const *const u8,
    pub w2s: *const *const u8,
    pub d: usize,
    pub inter: usize,
    pub n_experts: usize,
    /// the file's 256 x 16 f32 VQ codebook on the device, or null when every expert is MXFP4
    pub vq_codebook: *const f32,
    /// optional (both or none): per expert, the matrices once more in the one-launch decode kernel's order
    /// (mk_dev_moe_pack_gate_up, mk_dev_moe_pack_down)
    pub w13t: *const *const u8,
    pub w2t: *const *const u8,
    /// optional (each on its own): per expert, the scale bytes of W1, W3, W2 in K-tile order (mk_dev_mxfp4_scales_by_tile)
    pub w1st: *const *const u8,
    pub w3st: *const *const u8,
    pub w2st: *const *const u8,
}

/// mk_bin_entry: one directory entry of an MKIM file (weights::Entry, src/weights.rs:31-37).
#[repr(C)]
#[derive(Clone, Copy)]
pub struct MkBinEntry {
    pub dtype: u8,
    pub n_dims: u8,
    pub dims: [u32; MK_BIN_MAX_DIMS],
    pub offset: u64,
    pub size: u64,
}

/// mk_prefill_layout: byte offsets of mk_dev_moe_prefill's intermediates inside its workspace.
#[repr(C)]
#[derive(Clone, Copy, Default)]
pub struct MkPrefillLayout {
    pub order: usize,
    pub pos: usize,
    pub offsets: usize,
    pub g: usize,
    pub u: usize,
    pub o: usize,
}

/// mk_prof: GpuProf (src/metal.rs:667-680).
#[repr(C)]
#[derive(Clone, Copy, Default)]
pub struct MkProf {
    pub calls: u64,
    pub hits: u64,
    pub misses: u64,
    pub t_cache_ms: f64,
    pub t_io_ms: f64,
    pub t_launch_ms: f64,
    pub t_wait_ms: f64,
    pub t_readback_ms: f64,
    pub cache_tensors: usize,
    pub cache_bytes: usize,
}

#[repr(C)]
pub struct MkBinfile {
    _private: [u8; 0],
}
#[repr(C)]
pub struct MkExpertSet {
    _private: [u8; 0],
}
#[repr(C)]
pub struct MkQ8Head {
    _private: [u8; 0],
}
#[repr(C)]
pub struct MkMlaCache {
    _private: [u8; 0],
}

#[link(name = "mk_hip")]
extern "C" {
    pub fn mk_init(device: c_int) -> c_int;
    pub fn mk_available() -> c_int;
    pub fn mk_shutdown();
    pub fn mk_set_enabled(on: c_int);
    pub fn mk_enabled_now() -> c_int;
    pub fn mk_last_error() -> *const c_char;
    pub fn mk_set_cache_mb(mb: usize);
    pub fn mk_force_q8(v: c_int);
    pub fn mk_q8_enabled() -> c_int;
    pub fn mk_dev_mxfp4_dequant(packed: *const u8, scales: *const u8, rows: usize, cols: usize, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_quantize_bf16_split(x: *const f32, nvec: usize, n: usize, codes: *mut u8, exps: *mut u8, stream: *mut c_void) -> c_int;
    pub fn mk_dev_mxfp4_grouped_gemm_split(packed_ptrs: *const *const u8, scales_ptrs: *const *const u8, n_groups: usize, rows: usize, cols: usize, codes: *const u8, exps: *const u8, offsets: *const i32, m: usize, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_mxfp4_scales_by_tile(scales: *const u8, rows: usize, cols: usize, out: *mut u8, stream: *mut c_void) -> c_int;
    pub fn mk_moe_pack_bytes(d: usize, inter: usize, down: c_int) -> usize;
    pub fn mk_dev_moe_pack_gate_up(w1p: *const u8, w1s: *const u8, w3p: *const u8, w3s: *const u8, d: usize, inter: usize, pack: *mut u8, stream: *mut c_void) -> c_int;
    pub fn mk_dev_moe_unpack_gate_up(pack: *const u8, d: usize, inter: usize, w1p: *mut u8, w1s: *mut u8, w3p: *mut u8, w3s: *mut u8, stream: *mut c_void) -> c_int;
    pub fn mk_dev_moe_pack_down(w2p: *const u8, w2s: *const u8, d: usize, inter: usize, pack: *mut u8, stream: *mut c_void) -> c_int;
    pub fn mk_dev_moe_unpack_down(pack: *const u8, d: usize, inter: usize, w2p: *mut u8, w2s: *mut u8, stream: *mut c_void) -> c_int;
    pub fn mk_dev_moe_decode_gave_up(flag: *mut c_int) -> c_int;
    pub fn mk_dev_moe_count_bad_ids(ids: *const i32, n: usize, n_experts: usize, count: *mut i32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_fp8_dequant(w: *const u8, scales: *const u8, rows: usize, cols: usize, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_quantize_q8(x: *const f32, nvec: usize, n: usize, q: *mut i8, scales: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_mxfp4_quantize(w: *const f32, rows: usize, cols: usize, search: c_int, packed: *mut u8, scales: *mut u8, stream: *mut c_void) -> c_int;
    pub fn mk_dev_mxfp4sq_quantize(w: *const f32, rows: usize, cols: usize, packed: *mut u8, scales: *mut u8, smax: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_mxfp4sq_dequant(packed: *const u8, scales: *const u8, smax_dev: *const f32, smax: f32, rows: usize, cols: usize, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_quantize_fp8(w: *const f32, rows: usize, cols: usize, qw: *mut u8, scales: *mut u8, stream: *mut c_void) -> c_int;
    pub fn mk_dev_quantize_mxfp8(x: *const f32, nvec: usize, n: usize, codes: *mut u8, exps: *mut u8, stream: *mut c_void) -> c_int;
    pub fn mk_dev_mxfp4_matvec_q8(packed: *const u8, scales: *const u8, rows: usize, cols: usize, xq: *const i8, xs: *const f32, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_mxfp4_matvec_f32(packed: *const u8, scales: *const u8, rows: usize, cols: usize, x: *const f32, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_mxfp4_matvec(packed: *const u8, scales: *const u8, rows: usize, cols: usize, x: *const f32, out: *mut f32, mode: c_int, xq_ws: *mut i8, xs_ws: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_mxfp4_matvec_q8_batched(packed: *const u8, scales: *const u8, rows: usize, cols: usize, xq: *const i8, xs: *const f32, m: usize, workspace: *mut c_void, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_mxfp4_matvec_q8_grouped(packed_ptrs: *const *const u8, scales_ptrs: *const *const u8, nmat: usize, rows: usize, cols: usize, xq: *const i8, xs: *const f32, x_index: *const i32, out_ptrs: *const *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_mxfp4_matvec_nt(packed: *const u8, scales: *const u8, rows: usize, cols: usize, x: *const f32, m: usize, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_q8_matvec(q: *const i8, scales: *const c_void, scales_f16: c_int, rows: usize, cols: usize, xq: *const i8, xs: *const f32, batch: usize, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_argmax(logits: *const f32, batch: usize, n: usize, ws: *mut c_void, out_idx: *mut i32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_q8head_from_f32(w: *const f32, rows: usize, cols: usize, q: *mut i8, scales: *mut c_void, scales_f16: c_int, stream: *mut c_void) -> c_int;
    pub fn mk_moe_decode_vq_workspace_bytes(B: usize, topk: usize, has_shared: c_int, d: usize, inter: usize) -> usize;
    pub fn mk_moe_decode_workspace_bytes(B: usize, topk: usize, has_shared: c_int, d: usize, inter: usize) -> usize;
    pub fn mk_dev_moe_decode(table: *const MkExpertTable, B: usize, topk: usize, ids: *const i32, weights: *const f32, shared: c_int, x: *const f32, mode: c_int, act_kind: c_int, limit: f32, workspace: *mut c_void, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_moe_decode_act(table: *const MkExpertTable, B: usize, topk: usize, ids: *const i32, weights: *const f32, shared: c_int, x: *const f32, mode: c_int, act_kind: c_int, limit: f32, workspace: *mut c_void, act: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_moe_decode_from_act(table: *const MkExpertTable, B: usize, topk: usize, ids: *const i32, weights: *const f32, shared: c_int, act: *const f32, mode: c_int, act_kind: c_int, workspace: *mut c_void, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_router_softmax_topk(logits: *const f32, B: usize, n: usize, k: usize, ids: *mut i32, weights: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_router_topk(logits: *const f32, B: usize, n: usize, k: usize, kind: c_int, bias: *const f32, route_scale: f32, ids: *mut i32, weights: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_rmsnorm(x: *const f32, B: usize, d: usize, w: *const f32, eps: f32, out: *mut f32, q: *mut i8, scales: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_matvec_f32(w: *const f32, rows: usize, cols: usize, x: *const f32, B: usize, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_norm_gate_route(x: *const f32, b: usize, d: usize, norm_w: *const f32, eps: f32, gate: *const f32, n_experts: usize, k: usize,
                                  kind: c_int, bias: *const f32, route_scale: f32, xn: *mut f32, logits: *mut f32,
                                  ids: *mut i32, weights: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_mla_decode_workspace_bytes(nh: usize, L: usize, n_pos: usize) -> usize;
    pub fn mk_dev_mla_q8_decode(lat_q: *const i8, lat_s: *const c_void, rope_q: *const i8, rope_s: *const c_void, pos: usize, q: *const f32, nh: usize, L: usize, R: usize, scale: f32, workspace: *mut c_void, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_mla_decode_static_max_heads() -> usize;
    pub fn mk_dev_mla_q8_decode_static(lat_q: *const i8, lat_s: *const c_void, rope_q: *const i8, rope_s: *const c_void, pos: usize, q: *const f32, nh: usize, L: usize, R: usize, scale: f32, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_mla_cache_append(latent: *const f32, rope: *const f32, L: usize, R: usize, pos: usize, lat_q: *mut i8, lat_s: *mut c_void, rope_q: *mut i8, rope_s: *mut c_void, stream: *mut c_void) -> c_int;
    pub fn mk_dev_mla_heads_append(k_rows: *const f32, v_rows: *const f32, n_new: usize, nh: usize, nope: usize, rope: usize, vd: usize, pos0: usize, hadamard: c_int, kq: *mut i8, ks: *mut f32, kr: *mut f32, vq: *mut i8, vs: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_mla_heads_to_f32(kq: *const i8, ks: *const f32, kr: *const f32, vq: *const i8, vs: *const f32, n: usize, nh: usize, nope: usize, rope: usize, vd: usize, hadamard: c_int, k: *mut f32, v: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_mla_heads_workspace_bytes(m: usize, nh: usize, nope: usize, vd: usize) -> usize;
    pub fn mk_dev_mla_heads_q8_attn(kq: *const i8, ks: *const f32, kr: *const f32, vq: *const i8, vs: *const f32, pos0: usize, q: *const f32, m: usize, nh: usize, nope: usize, rope: usize, vd: usize, scale: f32, hadamard: c_int, workspace: *mut c_void, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_mxfp4_grouped_gemm(packed_ptrs: *const *const u8, scales_ptrs: *const *const u8, n_groups: usize, rows: usize, cols: usize, codes: *const u8, exps: *const u8, offsets: *const i32, m: usize, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_mxfp4_grouped_gemm_f32(packed_ptrs: *const *const u8, scales_ptrs: *const *const u8, n_groups: usize, rows: usize, cols: usize, x: *const f32, offsets: *const i32, m: usize, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_mxfp4_grouped_gemm_bf16(packed_ptrs: *const *const u8, scales_ptrs: *const *const u8, n_groups: usize, rows: usize, cols: usize, x: *const u16, offsets: *const i32, m: usize, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_moe_prefill_workspace_bytes(T: usize, topk: usize, n_experts: usize, d: usize, inter: usize) -> usize;
    pub fn mk_moe_prefill_workspace_layout(T: usize, topk: usize, n_experts: usize, d: usize, inter: usize, out: *mut MkPrefillLayout) -> c_int;
    pub fn mk_dev_moe_prefill(table: *const MkExpertTable, n_experts: usize, T: usize, topk: usize, ids: *const i32, weights: *const f32, x: *const f32, act_kind: c_int, workspace: *mut c_void, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_moe_prefill_keep(table: *const MkExpertTable, n_experts: usize, T: usize, topk: usize, ids: *const i32, weights: *const f32, x: *const f32, act_kind: c_int, workspace: *mut c_void, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_moe_prefill_f32(table: *const MkExpertTable, n_experts: usize, T: usize, topk: usize, ids: *const i32, weights: *const f32, x: *const f32, act_kind: c_int, workspace: *mut c_void, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_moe_prefill_bf16(table: *const MkExpertTable, n_experts: usize, T: usize, topk: usize, ids: *const i32, weights: *const f32, x: *const f32, act_kind: c_int, workspace: *mut c_void, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_vq1_workspace_bytes(cols: usize) -> usize;
    pub fn mk_dev_vq1_matvec(codebook: *const f32, indices: *const u8, rows: usize, cols: usize, x: *const f32, exact: c_int, workspace: *mut c_void, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_dev_vq1_matvec_nt(codebook: *const f32, indices: *const u8, rows: usize, cols: usize, xt: *const f32, m: usize, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn mk_bin_open(path: *const c_char, out: *mut *mut MkBinfile) -> c_int;
    pub fn mk_bin_close(f: *mut MkBinfile);
    pub fn mk_bin_n_tensors(f: *const MkBinfile) -> usize;
    pub fn mk_bin_entry_at(f: *const MkBinfile, i: usize, name: *mut *const c_char, e: *mut MkBinEntry) -> c_int;
    pub fn mk_bin_find(f: *const MkBinfile, name: *const c_char, e: *mut MkBinEntry) -> c_int;
    pub fn mk_bin_blob(f: *const MkBinfile, name: *const c_char, size: *mut usize) -> *const c_void;
    pub fn mk_bin_config_json(f: *const MkBinfile, len: *mut usize) -> *const c_char;
    pub fn mk_bin_mxfp4_parts(f: *const MkBinfile, name: *const c_char, packed: *mut *const u8, scales: *mut *const u8, rows: *mut usize, cols: *mut usize) -> c_int;
    pub fn mk_bin_load_experts(f: *const MkBinfile, layer_prefix: *const c_char, n_experts: usize, out: *mut *mut MkExpertSet) -> c_int;
    pub fn mk_expert_set_table(s: *const MkExpertSet) -> *const MkExpertTable;
    pub fn mk_expert_set_count(s: *const MkExpertSet) -> usize;
    pub fn mk_expert_set_bytes(s: *const MkExpertSet) -> usize;
    pub fn mk_expert_set_free(s: *mut MkExpertSet);
    pub fn mk_mxfp4_matvec(packed: *const u8, scales: *const u8, rows: usize, cols: usize, x: *const f32, out: *mut f32) -> c_int;
    pub fn mk_matvec_f32(w: *const f32, rows: usize, cols: usize, x: *const f32, out: *mut f32) -> c_int;
    pub fn mk_prof_enable(on: c_int);
    pub fn mk_prof_reset();
    pub fn mk_prof_get(out: *mut MkProf);
    pub fn mk_prof_print();
    pub fn mk_mxfp4_dequant(packed: *const u8, scales: *const u8, rows: usize, cols: usize, out: *mut f32) -> c_int;
    pub fn mk_quantize_q8(x: *const f32, n: usize, q: *mut i8, scales: *mut f32) -> c_int;
    pub fn mk_q8head_from_f32(w: *const f32, rows: usize, cols: usize, scales_f16: c_int, out: *mut *mut MkQ8Head) -> c_int;
    pub fn mk_q8head_from_q8(q: *const i8, scales: *const f32, rows: usize, cols: usize, scales_f16: c_int, out: *mut *mut MkQ8Head) -> c_int;
    pub fn mk_q8head_matvec(h: *mut MkQ8Head, x: *const f32, batch: usize, out: *mut f32, argmax_out: *mut i32) -> c_int;
    pub fn mk_q8head_free(h: *mut MkQ8Head);
    pub fn mk_mla_cache_new(nh: usize, L: usize, R: usize, capacity: usize, out: *mut *mut MkMlaCache) -> c_int;
    pub fn mk_mla_cache_new_heads(nh: usize, nope: usize, rope: usize, vd: usize, capacity: usize, out: *mut *mut MkMlaCache) -> c_int;
    pub fn mk_mla_cache_set_hadamard(c: *mut MkMlaCache, on: c_int) -> c_int;
    pub fn mk_mla_cache_push(c: *mut MkMlaCache, row0: *const f32, row1: *const f32) -> c_int;
    pub fn mk_mla_cache_assign_f32(c: *mut MkMlaCache, rows0: *const f32, rows1: *const f32, n: usize) -> c_int;
    pub fn mk_mla_cache_positions(c: *const MkMlaCache) -> usize;
    pub fn mk_mla_cache_to_f32(c: *const MkMlaCache, rows0: *mut f32, rows1: *mut f32) -> c_int;
    pub fn mk_mla_attn(c: *mut MkMlaCache, q: *const f32, scale: f32, out: *mut f32) -> c_int;
    pub fn mk_mla_attn_prefill(c: *mut MkMlaCache, q: *const f32, m: usize, scale: f32, out: *mut f32) -> c_int;
    pub fn mk_mla_cache_free(c: *mut MkMlaCache);
}

fn last_error() -> String {
    unsafe { CStr::from_ptr(mk_last_error()) }.to_string_lossy().into_owned()
}

/// Same shape as metal::gpu_available (src/metal.rs:445): true once a gfx950 device is bound.  Never fatal.
pub fn gpu_available() -> bool {
    unsafe { mk_available() == 1 || mk_init(0) == MK_OK }
}

/// Same signature as metal::gpu_matvec_fp4 (src/metal.rs:943) plus a result: false when the device path did not run.
/// `y` is untouched in that case and the caller takes its CPU path (the library itself never falls back).
pub fn gpu_matvec_fp4(packed: &[u8], scales: &[u8], rows: usize, cols: usize, x: &[f32], y: &mut [f32]) -> bool {
    assert_eq!(cols % 32, 0);
    assert_eq!(packed.len(), rows * cols / 2);
    assert_eq!(scales.len(), rows * cols / 32);
    assert_eq!(x.len(), cols);
    assert_eq!(y.len(), rows);
    // the arithmetic follows the reference's toggle (src/q8.rs:77-83)
    unsafe { mk_force_q8(if crate::q8::q8_enabled() { 1 } else { 0 }) };
    let st = unsafe { mk_mxfp4_matvec(packed.as_ptr(), scales.as_ptr(), rows, cols, x.as_ptr(), y.as_mut_ptr()) };
    if st != MK_OK {
        println!("gpu: hip matvec_fp4 failed ({}): {} - falling back to CPU for this matvec", st, last_error());
    }
    st == MK_OK
}

/// Same signature as metal::gpu_matvec (src/metal.rs:750) plus a result; bit-identical to model::matvec_cpu.
pub fn gpu_matvec(w: &[f32], rows: usize, cols: usize, x: &[f32], y: &mut [f32]) -> bool {
    assert_eq!(w.len(), rows * cols);
    assert_eq!(x.len(), cols);
    assert_eq!(y.len(), rows);
    let st = unsafe { mk_matvec_f32(w.as_ptr(), rows, cols, x.as_ptr(), y.as_mut_ptr()) };
    if st != MK_OK {
        println!("gpu: hip matvec failed ({}): {} - falling back to CPU for this matvec", st, last_error());
    }
    st == MK_OK
}

/// metal::gpu_prof_print (src/metal.rs:695): the accumulated profile, printed at the end of a run under --gpu.
pub fn gpu_prof_print() {
    unsafe { mk_prof_print() }
}

/// model::Q8Head (src/model.rs:261-348) resident on the device.
pub struct HipQ8Head {
    h: *mut MkQ8Head,
    pub rows: usize,
    pub cols: usize,
}

unsafe impl Send for HipQ8Head {}

impl HipQ8Head {
    /// Q8Head::from_f32 (src/model.rs:274-286); `None` when the device path is unavailable.
    pub fn from_f32(w: &[f32], rows: usize, cols: usize) -> Option<HipQ8Head> {
        assert_eq!(w.len(), rows * cols);
        let mut h: *mut MkQ8Head = std::ptr::null_mut();
        // f32 scales: the reference's in-memory form (src/model.rs:261-266)
        let st = unsafe { mk_q8head_from_f32(w.as_ptr(), rows, cols, 0, &mut h) };
        if st != MK_OK {
            println!("gpu: hip q8 head unavailable ({}): {}", st, last_error());
            return None;
        }
        Some(HipQ8Head { h, rows, cols })
    }

    /// Q8Head::matvec (src/model.rs:290-335) for one position; `greedy` receives the arg-max token when given.
    pub fn matvec(&self, x: &[f32], out: &mut [f32], greedy: Option<&mut i32>) -> bool {
        assert_eq!(x.len(), self.cols);
        assert_eq!(out.len(), self.rows);
        let idx = greedy.map_or(std::ptr::null_mut(), |g| g as *mut i32);
        unsafe { mk_q8head_matvec(self.h, x.as_ptr(), 1, out.as_mut_ptr(), idx) == MK_OK }
    }
}

impl Drop for HipQ8Head {
    fn drop(&mut self) {
        unsafe { mk_q8head_free(self.h) }
    }
}

/// MlaCache (src/model.rs:765-781) resident on the device, in the reference's own layout.
pub struct HipMlaCache {
    c: *mut MkMlaCache,
    nh: usize,
    qh: usize,
    vd: usize,
}

unsafe impl Send for HipMlaCache {}

impl HipMlaCache {
    pub fn new(nh: usize, nope: usize, rope: usize, vd: usize, capacity: usize) -> Option<HipMlaCache> {
        let mut c: *mut MkMlaCache = std::ptr::null_mut();
        let st = unsafe { mk_mla_cache_new_heads(nh, nope, rope, vd, capacity, &mut c) };
        if st != MK_OK {
            println!("gpu: hip mla cache unavailable ({}): {}", st, last_error());
            return None;
        }
        Some(HipMlaCache { c, nh, qh: nope + rope, vd })
    }

    /// MlaCache::positions (src/model.rs:1571-1578)
    pub fn positions(&self) -> usize {
        unsafe { mk_mla_cache_positions(self.c) }
    }

    /// MlaCache::push (src/model.rs:1583-1618): k_row H x (nope + rope), v_row H x v.
    pub fn push(&mut self, k_row: &[f32], v_row: &[f32]) -> bool {
        assert_eq!(k_row.len(), self.nh * self.qh);
        assert_eq!(v_row.len(), self.nh * self.vd);
        unsafe { mk_mla_cache_push(self.c, k_row.as_ptr(), v_row.as_ptr()) == MK_OK }
    }

    /// MlaCache::assign_f32 (src/model.rs:1680-1692)
    pub fn assign_f32(&mut self, k: &[f32], v: &[f32]) -> bool {
        let n = k.len() / (self.nh * self.qh);
        assert_eq!(v.len(), n * self.nh * self.vd);
        unsafe { mk_mla_cache_assign_f32(self.c, k.as_ptr(), v.as_ptr(), n) == MK_OK }
    }

    /// MlaCache::to_f32 (src/model.rs:1623-1676)
    pub fn to_f32(&self) -> Option<(Vec<f32>, Vec<f32>)> {
        let n = self.positions();
        let mut k = vec![0f32; n * self.nh * self.qh];
        let mut v = vec![0f32; n * self.nh * self.vd];
        let st = unsafe { mk_mla_cache_to_f32(self.c, k.as_mut_ptr(), v.as_mut_ptr()) };
        if st == MK_OK { Some((k, v)) } else { None }
    }

    /// mla_attn_flash_q8_mqa (src/model.rs:1804-1908) over all cached positions: q H x (nope + rope), attn H x v.
    pub fn attn(&mut self, q: &[f32], scale: f32, attn: &mut [f32]) -> bool {
        assert_eq!(q.len(), self.nh * self.qh);
        assert_eq!(attn.len(), self.nh * self.vd);
        unsafe { mk_mla_attn(self.c, q.as_ptr(), scale, attn.as_mut_ptr()) == MK_OK }
    }

    /// The attention loop of mla_prefill (src/model.rs:2080-2102) after the prompt's m positions have been pushed.
    pub fn attn_prefill(&mut self, q: &[f32], m: usize, scale: f32, attn: &mut [f32]) -> bool {
        assert_eq!(q.len(), m * self.nh * self.qh);
        assert_eq!(attn.len(), m * self.nh * self.vd);
        unsafe { mk_mla_attn_prefill(self.c, q.as_ptr(), m, scale, attn.as_mut_ptr()) == MK_OK }
    }
}

impl Drop for HipMlaCache {
    fn drop(&mut self) {
        unsafe { mk_mla_cache_free(self.c) }
    }
}
