"""ctypes binding of libmk_hip.so (the C ABI declared in include/mk_hip.h).

The library is the product: there is no Python or CPU stand-in for it.  If it
has not been built (python microkimi_amd/build.py) loading fails with an error.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmk_hip.so")

MK_OK = 0
MODE_F32, MODE_Q8 = 0, 1
ACT_SWIGLU, ACT_SITU, ACT_DS = 0, 1, 2


class MkError(RuntimeError):
    def __init__(self, status, msg):
        super().__init__(f"libmk_hip status {status}: {msg}")
        self.status = status


class BinEntry(C.Structure):
    _fields_ = [("dtype", C.c_uint8), ("n_dims", C.c_uint8), ("dims", C.c_uint32 * 8), ("offset", C.c_uint64), ("size", C.c_uint64)]


class ExpertTable(C.Structure):
    _fields_ = [("w1p", C.c_void_p), ("w1s", C.c_void_p), ("w3p", C.c_void_p), ("w3s", C.c_void_p), ("w2p", C.c_void_p),
                ("w2s", C.c_void_p), ("d", C.c_size_t), ("inter", C.c_size_t), ("n_experts", C.c_size_t), ("vq_codebook", C.c_void_p),
                ("w13t", C.c_void_p), ("w2t", C.c_void_p), ("w1st", C.c_void_p), ("w3st", C.c_void_p), ("w2st", C.c_void_p)]


class Prof(C.Structure):
    _fields_ = [("calls", C.c_uint64), ("hits", C.c_uint64), ("misses", C.c_uint64), ("t_cache_ms", C.c_double), ("t_io_ms", C.c_double),
                ("t_launch_ms", C.c_double), ("t_wait_ms", C.c_double), ("t_readback_ms", C.c_double), ("cache_tensors", C.c_size_t),
                ("cache_bytes", C.c_size_t)]


class PrefillLayout(C.Structure):
    _fields_ = [("order", C.c_size_t), ("pos", C.c_size_t), ("offsets", C.c_size_t), ("g", C.c_size_t), ("u", C.c_size_t), ("o", C.c_size_t)]


def _load():
    # torch ships its own HIP runtime (same soname as the system one).  Loading torch first makes the dynamic
    # loader bind libmk_hip.so to that already-loaded copy; the other order leaves two runtimes in the process
    # and the second one finds no device.
    import torch  # noqa: F401
    if not os.path.exists(LIB_PATH):
        raise ImportError(f"{LIB_PATH} is missing: build it with `python microkimi_amd/build.py` (needs hipcc); "
                          "there is no fallback implementation")
    lib = C.CDLL(LIB_PATH)
    vp, sz, i32, f32 = C.c_void_p, C.c_size_t, C.c_int, C.c_float
    sig = {
        "mk_init": (i32, [i32]),
        "mk_available": (i32, []),
        "mk_shutdown": (None, []),
        "mk_set_enabled": (None, [i32]),
        "mk_enabled_now": (i32, []),
        "mk_last_error": (C.c_char_p, []),
        "mk_set_cache_mb": (None, [sz]),
        "mk_force_q8": (None, [i32]),
        "mk_q8_enabled": (i32, []),
        "mk_dev_mxfp4_dequant": (i32, [vp, vp, sz, sz, vp, vp]),
        "mk_dev_mxfp4_scales_by_tile": (i32, [vp, sz, sz, vp, vp]),
        "mk_dev_quantize_bf16_split": (i32, [vp, sz, sz, vp, vp, vp]),
        "mk_dev_mxfp4_grouped_gemm_split": (i32, [vp, vp, sz, sz, sz, vp, vp, vp, sz, vp, vp]),
        "mk_dev_fp8_dequant": (i32, [vp, vp, sz, sz, vp, vp]),
        "mk_dev_quantize_q8": (i32, [vp, sz, sz, vp, vp, vp]),
        "mk_dev_quantize_mxfp8": (i32, [vp, sz, sz, vp, vp, vp]),
        "mk_dev_mxfp4_quantize": (i32, [vp, sz, sz, i32, vp, vp, vp]),
        "mk_dev_quantize_fp8": (i32, [vp, sz, sz, vp, vp, vp]),
        "mk_dev_mxfp4sq_quantize": (i32, [vp, sz, sz, vp, vp, vp, vp]),
        "mk_dev_mxfp4sq_dequant": (i32, [vp, vp, vp, f32, sz, sz, vp, vp]),
        "mk_dev_mxfp4_matvec_q8": (i32, [vp, vp, sz, sz, vp, vp, vp, vp]),
        "mk_dev_mxfp4_matvec_f32": (i32, [vp, vp, sz, sz, vp, vp, vp]),
        "mk_dev_mxfp4_matvec": (i32, [vp, vp, sz, sz, vp, vp, i32, vp, vp, vp]),
        "mk_dev_mxfp4_matvec_q8_grouped": (i32, [vp, vp, sz, sz, sz, vp, vp, vp, vp, vp]),
        "mk_dev_mxfp4_matvec_q8_batched": (i32, [vp, vp, sz, sz, vp, vp, sz, vp, vp, vp]),
        "mk_dev_mxfp4_matvec_nt": (i32, [vp, vp, sz, sz, vp, sz, vp, vp]),
        "mk_dev_q8_matvec": (i32, [vp, vp, i32, sz, sz, vp, vp, sz, vp, vp]),
        "mk_dev_argmax": (i32, [vp, sz, sz, vp, vp, vp]),
        "mk_dev_q8head_from_f32": (i32, [vp, sz, sz, vp, vp, i32, vp]),
        "mk_moe_pack_bytes": (sz, [sz, sz, i32]),
        "mk_dev_moe_pack_gate_up": (i32, [vp, vp, vp, vp, sz, sz, vp, vp]),
        "mk_dev_moe_unpack_gate_up": (i32, [vp, sz, sz, vp, vp, vp, vp, vp]),
        "mk_dev_moe_pack_down": (i32, [vp, vp, sz, sz, vp, vp]),
        "mk_dev_moe_unpack_down": (i32, [vp, sz, sz, vp, vp, vp]),
        "mk_dev_moe_decode_gave_up": (i32, [C.POINTER(C.c_int)]),
        "mk_dev_moe_count_bad_ids": (i32, [vp, sz, sz, vp, vp]),
        "mk_moe_decode_workspace_bytes": (sz, [sz, sz, i32, sz, sz]),
        "mk_moe_decode_vq_workspace_bytes": (sz, [sz, sz, i32, sz, sz]),
        "mk_dev_moe_decode": (i32, [C.POINTER(ExpertTable), sz, sz, vp, vp, i32, vp, i32, i32, f32, vp, vp, vp]),
        "mk_dev_moe_decode_act": (i32, [C.POINTER(ExpertTable), sz, sz, vp, vp, i32, vp, i32, i32, f32, vp, vp, vp]),
        "mk_dev_moe_decode_from_act": (i32, [C.POINTER(ExpertTable), sz, sz, vp, vp, i32, vp, i32, i32, vp, vp, vp]),
        "mk_dev_router_softmax_topk": (i32, [vp, sz, sz, sz, vp, vp, vp]),
        "mk_dev_router_topk": (i32, [vp, sz, sz, sz, i32, vp, f32, vp, vp, vp]),
        "mk_dev_rmsnorm": (i32, [vp, sz, sz, vp, f32, vp, vp, vp, vp]),
        "mk_dev_matvec_f32": (i32, [vp, sz, sz, vp, sz, vp, vp]),
        "mk_dev_norm_gate_route": (i32, [vp, sz, sz, vp, f32, vp, sz, sz, i32, vp, f32, vp, vp, vp, vp, vp]),
        "mk_mla_decode_workspace_bytes": (sz, [sz, sz, sz]),
        "mk_dev_mla_q8_decode": (i32, [vp, vp, vp, vp, sz, vp, sz, sz, sz, f32, vp, vp, vp]),
        "mk_mla_decode_static_max_heads": (sz, []),
        "mk_dev_mla_q8_decode_static": (i32, [vp, vp, vp, vp, sz, vp, sz, sz, sz, f32, vp, vp]),
        "mk_dev_mla_cache_append": (i32, [vp, vp, sz, sz, sz, vp, vp, vp, vp, vp]),
        "mk_dev_mla_heads_append": (i32, [vp, vp, sz, sz, sz, sz, sz, sz, i32, vp, vp, vp, vp, vp, vp]),
        "mk_dev_mla_heads_to_f32": (i32, [vp, vp, vp, vp, vp, sz, sz, sz, sz, sz, i32, vp, vp, vp]),
        "mk_mla_heads_workspace_bytes": (sz, [sz, sz, sz, sz]),
        "mk_dev_mla_heads_q8_attn": (i32, [vp, vp, vp, vp, vp, sz, vp, sz, sz, sz, sz, sz, f32, i32, vp, vp, vp]),
        "mk_dev_mxfp4_grouped_gemm": (i32, [vp, vp, sz, sz, sz, vp, vp, vp, sz, vp, vp]),
        "mk_dev_mxfp4_grouped_gemm_f32": (i32, [vp, vp, sz, sz, sz, vp, vp, sz, vp, vp]),
        "mk_dev_mxfp4_grouped_gemm_bf16": (i32, [vp, vp, sz, sz, sz, vp, vp, sz, vp, vp]),
        "mk_moe_prefill_workspace_bytes": (sz, [sz, sz, sz, sz, sz]),
        "mk_moe_prefill_workspace_layout": (i32, [sz, sz, sz, sz, sz, C.POINTER(PrefillLayout)]),
        "mk_dev_moe_prefill": (i32, [C.POINTER(ExpertTable), sz, sz, sz, vp, vp, vp, i32, vp, vp, vp]),
        "mk_dev_moe_prefill_keep": (i32, [C.POINTER(ExpertTable), sz, sz, sz, vp, vp, vp, i32, vp, vp, vp]),
        "mk_dev_moe_prefill_f32": (i32, [C.POINTER(ExpertTable), sz, sz, sz, vp, vp, vp, i32, vp, vp, vp]),
        "mk_dev_moe_prefill_bf16": (i32, [C.POINTER(ExpertTable), sz, sz, sz, vp, vp, vp, i32, vp, vp, vp]),
        "mk_mxfp4_matvec": (i32, [vp, vp, sz, sz, vp, vp]),
        "mk_mxfp4_dequant": (i32, [vp, vp, sz, sz, vp]),
        "mk_matvec_f32": (i32, [vp, sz, sz, vp, vp]),
        "mk_prof_enable": (None, [i32]),
        "mk_prof_reset": (None, []),
        "mk_prof_get": (None, [C.POINTER(Prof)]),
        "mk_prof_print": (None, []),
        "mk_quantize_q8": (i32, [vp, sz, vp, vp]),
        "mk_q8head_from_f32": (i32, [vp, sz, sz, i32, C.POINTER(vp)]),
        "mk_q8head_from_q8": (i32, [vp, vp, sz, sz, i32, C.POINTER(vp)]),
        "mk_q8head_matvec": (i32, [vp, vp, sz, vp, vp]),
        "mk_q8head_free": (None, [vp]),
        "mk_mla_cache_new": (i32, [sz, sz, sz, sz, C.POINTER(vp)]),
        "mk_mla_cache_new_heads": (i32, [sz, sz, sz, sz, sz, C.POINTER(vp)]),
        "mk_mla_cache_set_hadamard": (i32, [vp, i32]),
        "mk_mla_cache_push": (i32, [vp, vp, vp]),
        "mk_mla_cache_assign_f32": (i32, [vp, vp, vp, sz]),
        "mk_mla_attn_prefill": (i32, [vp, vp, sz, f32, vp]),
        "mk_mla_cache_positions": (sz, [vp]),
        "mk_mla_cache_to_f32": (i32, [vp, vp, vp]),
        "mk_mla_attn": (i32, [vp, vp, f32, vp]),
        "mk_mla_cache_free": (None, [vp]),
        "mk_vq1_workspace_bytes": (sz, [sz]),
        "mk_dev_vq1_matvec": (i32, [vp, vp, sz, sz, vp, i32, vp, vp, vp]),
        "mk_dev_vq1_matvec_nt": (i32, [vp, vp, sz, sz, vp, sz, vp, vp]),
        "mk_bin_open": (i32, [C.c_char_p, C.POINTER(vp)]),
        "mk_bin_close": (None, [vp]),
        "mk_bin_n_tensors": (sz, [vp]),
        "mk_bin_entry_at": (i32, [vp, sz, C.POINTER(C.c_char_p), C.POINTER(BinEntry)]),
        "mk_bin_find": (i32, [vp, C.c_char_p, C.POINTER(BinEntry)]),
        "mk_bin_blob": (vp, [vp, C.c_char_p, C.POINTER(sz)]),
        "mk_bin_config_json": (vp, [vp, C.POINTER(sz)]),
        "mk_bin_mxfp4_parts": (i32, [vp, C.c_char_p, C.POINTER(vp), C.POINTER(vp), C.POINTER(sz), C.POINTER(sz)]),
        "mk_bin_load_experts": (i32, [vp, C.c_char_p, sz, C.POINTER(vp)]),
        "mk_expert_set_table": (C.POINTER(ExpertTable), [vp]),
        "mk_expert_set_count": (sz, [vp]),
        "mk_expert_set_bytes": (sz, [vp]),
        "mk_expert_set_free": (None, [vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)  # AttributeError here = the library does not export a declared symbol
        fn.restype = res
        fn.argtypes = args
    return lib, sorted(sig)


lib, SYMBOLS = _load()


def check(status):
    if status != MK_OK:
        raise MkError(status, lib.mk_last_error().decode("utf-8", "replace"))


def require_device():
    """Binds device 0; raises if no gfx950 device is usable (no fallback)."""
    check(lib.mk_init(0))


def ptr(t):
    """Device pointer of a torch tensor (must be contiguous) or None."""
    if t is None:
        return None
    assert t.is_contiguous(), "tensor must be contiguous"
    return C.c_void_p(t.data_ptr())


def hptr(a):
    """Host pointer of a contiguous numpy array."""
    assert a.flags["C_CONTIGUOUS"]
    return C.c_void_p(a.ctypes.data)


def cur_stream():
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)
