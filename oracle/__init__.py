"""ctypes front end of the CPU oracle (oracle/mk_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
the cpu_baseline leg of bench.py.  The product package never imports it.

Each function takes and returns numpy arrays and forwards to the C function of
the same name (orc_*), which cites the reference lines it restates.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libmk_oracle.so")

ACT_SWIGLU, ACT_SITU, ACT_DS = 0, 1, 2


def build(force=False):
    """Compile libmk_oracle.so with the committed Makefile."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.run(["make", "-s", "-C", _HERE, "libmk_oracle.so"], check=True)


def _load():
    src = os.path.join(_HERE, "mk_oracle.c")
    if not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        build()
    return C.CDLL(_SO)


_lib = _load()

_u8p = C.POINTER(C.c_uint8)
_i8p = C.POINTER(C.c_int8)
_f32p = C.POINTER(C.c_float)
_u32p = C.POINTER(C.c_uint32)
_sz = C.c_size_t


class MlaCfg(C.Structure):
    _fields_ = [("nh", _sz), ("nope", _sz), ("rope", _sz), ("vd", _sz)]


def _p(a, ty):
    return a.ctypes.data_as(ty)


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


_lib.orc_exp2_i.restype = C.c_float
_lib.orc_exp2_i.argtypes = [C.c_int]
_lib.orc_scale_from_byte.restype = C.c_float
_lib.orc_scale_from_byte.argtypes = [C.c_uint8]
_lib.orc_e4m3_to_f32.restype = C.c_float
_lib.orc_e4m3_to_f32.argtypes = [C.c_uint8]
_lib.orc_f32_to_e4m3.restype = C.c_uint8
_lib.orc_f32_to_e4m3.argtypes = [C.c_float]
_lib.orc_block_dot.restype = C.c_int32
_lib.orc_block_dot.argtypes = [_u8p, _i8p]
_lib.orc_block_dot_i8.restype = C.c_int32
_lib.orc_block_dot_i8.argtypes = [_i8p, _i8p]
_lib.orc_dot.restype = C.c_float
_lib.orc_dot.argtypes = [_f32p, _f32p, _sz]
_lib.orc_situ.restype = C.c_float
_lib.orc_situ.argtypes = [C.c_float, C.c_float]
_lib.orc_silu.restype = C.c_float
_lib.orc_silu.argtypes = [C.c_float]
_lib.orc_search_mx_scale.restype = C.c_int
_lib.orc_search_mx_scale.argtypes = [_f32p, C.c_int]
_lib.orc_argmax.restype = _sz
_lib.orc_argmax.argtypes = [_f32p, _sz]
_lib.orc_force_scalar.argtypes = [C.c_int]
_lib.orc_mxfp4_dequant.argtypes = [_u8p, _u8p, _sz, _sz, _f32p]
_lib.orc_mxfp4_quantize.argtypes = [_f32p, _sz, _sz, C.c_int, _u8p, _u8p]
_lib.orc_dequant_fp8.argtypes = [_u8p, _u8p, _sz, _sz, _f32p]
_lib.orc_quantize_fp8.argtypes = [_f32p, _sz, _sz, _u8p, _u8p]
_lib.orc_fp8_roundtrip.argtypes = [_f32p, _sz, _sz, _u8p, _u8p]
_lib.orc_fp8_roundtrip_emax.argtypes = [_f32p, _sz, _sz, C.c_int, _u8p, _u8p]
_lib.orc_round_bf16.argtypes = [_f32p, _sz]
_lib.orc_quantize_q8.argtypes = [_f32p, _sz, _i8p, _f32p]
_lib.orc_matvec_f32.argtypes = [_f32p, _sz, _sz, _f32p, _f32p]
_lib.orc_matvec_packed_q8.argtypes = [_u8p, _u8p, _sz, _sz, _i8p, _f32p, _f32p]
_lib.orc_matvec_packed.argtypes = [_u8p, _u8p, _sz, _sz, _f32p, _f32p, C.c_int]
_lib.orc_matvec_packed_shader_emul.argtypes = [_u8p, _u8p, _sz, _sz, _f32p, _f32p, _sz]
_lib.orc_matvec_packed_nt.argtypes = [_u8p, _u8p, _sz, _sz, _f32p, _sz, _f32p]
_lib.orc_q8head_from_f32.argtypes = [_f32p, _sz, _sz, _i8p, _f32p]
_lib.orc_q8head_matvec.argtypes = [_i8p, _f32p, _sz, _sz, _f32p, _f32p, _sz]
_lib.orc_hadamard64.argtypes = [_f32p]
_lib.orc_mla_cache_push.argtypes = [C.POINTER(MlaCfg), C.c_int, _f32p, _f32p, _i8p, _f32p, _f32p, _i8p, _f32p]
_lib.orc_mla_cache_to_f32.argtypes = [C.POINTER(MlaCfg), C.c_int, _sz, _i8p, _f32p, _f32p, _i8p, _f32p, _f32p, _f32p]
_lib.orc_mla_attn_ref.argtypes = [C.POINTER(MlaCfg), _f32p, _f32p, _f32p, _sz, _sz, C.c_float, _f32p]
_lib.orc_mla_attn_flash.argtypes = [C.POINTER(MlaCfg), _f32p, _f32p, _f32p, _sz, _sz, C.c_float, _f32p]
_lib.orc_mla_attn_flash_q8.argtypes = [C.POINTER(MlaCfg), C.c_int, _i8p, _f32p, _f32p, _i8p, _f32p, _f32p, _sz, _sz, C.c_float, _f32p]
_lib.orc_mla_attn_flash_q8_mqa.argtypes = [C.POINTER(MlaCfg), C.c_int, _sz, _i8p, _f32p, _f32p, _i8p, _f32p, _f32p, _sz, C.c_float, _f32p]
_lib.orc_gate_forward.argtypes = [_f32p, _sz, _f32p, _f32p, _sz, _sz, C.c_float, _u32p, _f32p]
_lib.orc_router_sigmoid.argtypes = [_f32p, _f32p, _sz, _sz, _u32p, _f32p]
_lib.orc_router_softmax.argtypes = [_f32p, _sz, _sz, _u32p, _f32p]
_lib.orc_expert_forward_f32.argtypes = [_f32p, _f32p, _f32p, _f32p, _sz, _sz, C.c_float, _f32p]
_PP = C.POINTER(_u8p)
_lib.orc_expert_packed.argtypes = [_u8p, _u8p, _u8p, _u8p, _u8p, _u8p, _sz, _sz, _f32p, C.c_int, C.c_int, C.c_float, C.c_float, _f32p]
_lib.orc_matvec_packed_q8_device_order.argtypes = [_u8p, _u8p, _sz, _sz, _i8p, _f32p, _f32p]
_lib.orc_q8head_matvec_device_order.argtypes = [_i8p, _f32p, _sz, _sz, _i8p, _f32p, _f32p]
_lib.orc_scale_sq.argtypes = [C.c_uint8, C.c_float]
_lib.orc_scale_sq.restype = C.c_float
_lib.orc_mxfp4sq_quantize.argtypes = [_f32p, _sz, _sz, _u8p, _u8p]
_lib.orc_mxfp4sq_quantize.restype = C.c_float
_lib.orc_mxfp4sq_dequant.argtypes = [_u8p, _u8p, C.c_float, _sz, _sz, _f32p]
_lib.orc_expert_vq.argtypes = [_f32p, _u8p, _u8p, _u8p, _sz, _sz, _f32p, C.c_int, C.c_float, C.c_float, _f32p]
_lib.orc_expert_act.argtypes = [_u8p, _u8p, _u8p, _u8p, _sz, _sz, _f32p, C.c_int, C.c_int, C.c_float, C.c_float, _f32p]
_lib.orc_moe_decode.argtypes = [_PP, _PP, _PP, _PP, _PP, _PP, _sz, _sz, _sz, _sz, _u32p, _f32p, C.c_int, _f32p, C.c_int, C.c_int,
                                C.c_float, _sz, _f32p]
_lib.orc_moe_prefill.argtypes = [_PP, _PP, _PP, _PP, _PP, _PP, _sz, _sz, _sz, _sz, _sz, _u32p, _f32p, _f32p, C.c_int, C.c_int, _f32p]
_lib.orc_rng_u8.argtypes = [C.POINTER(C.c_uint64), _u8p, _sz]
_lib.orc_rng_f32.argtypes = [C.POINTER(C.c_uint64), _f32p, _sz]
_lib.orc_pattern.argtypes = [_sz, _f32p, _sz]
_lib.orc_vq1_matvec_gather.argtypes = [_f32p, _u8p, _sz, _sz, _f32p, _f32p]
_lib.orc_vq1_matvec_lut.argtypes = [_f32p, _u8p, _sz, _sz, _f32p, _f32p]
_lib.orc_vq1_matvec_nt.argtypes = [_f32p, _u8p, _sz, _sz, _f32p, _sz, _f32p]

# ---------------------------------------------------------------- scalars
exp2_i = _lib.orc_exp2_i
scale_from_byte = _lib.orc_scale_from_byte
e4m3_to_f32 = _lib.orc_e4m3_to_f32
f32_to_e4m3 = _lib.orc_f32_to_e4m3
situ = _lib.orc_situ
silu = _lib.orc_silu
force_scalar = _lib.orc_force_scalar


class Rng:
    """splitmix64 streams of the reference's tests (src/q8.rs:269-278, src/model.rs:3683-3692)."""

    def __init__(self, seed):
        self.state = C.c_uint64(seed)

    def u8(self, n):
        out = np.empty(n, np.uint8)
        _lib.orc_rng_u8(C.byref(self.state), _p(out, _u8p), n)
        return out

    def f32(self, n):
        out = np.empty(n, np.float32)
        _lib.orc_rng_f32(C.byref(self.state), _p(out, _f32p), n)
        return out


def pattern(start, n):
    out = np.empty(n, np.float32)
    _lib.orc_pattern(start, _p(out, _f32p), n)
    return out


# ------------------------------------------------------------------ codec
def mxfp4_dequant(packed, scales, rows, cols):
    packed, scales = _c(packed, np.uint8), _c(scales, np.uint8)
    assert packed.size == rows * cols // 2 and scales.size == rows * cols // 32
    out = np.empty((rows, cols), np.float32)
    _lib.orc_mxfp4_dequant(_p(packed, _u8p), _p(scales, _u8p), rows, cols, _p(out, _f32p))
    return out


def mxfp4_quantize(w, rows, cols, search=True):
    w = _c(w, np.float32)
    assert cols % 32 == 0 and w.size == rows * cols
    packed = np.zeros((rows, cols // 2), np.uint8)
    scales = np.zeros((rows, cols // 32), np.uint8)
    _lib.orc_mxfp4_quantize(_p(w, _f32p), rows, cols, int(search), _p(packed, _u8p), _p(scales, _u8p))
    return packed, scales


def scale_sq(q, smax):
    """mxfp4::scale_sq (src/mxfp4.rs:154-158)."""
    return float(_lib.orc_scale_sq(int(q), float(smax)))


def mxfp4sq_quantize(w, rows, cols):
    """mxfp4::quantize_sq (src/mxfp4.rs:160-214): (packed, scale bytes, smax)."""
    w = _c(w, np.float32)
    assert cols % 32 == 0 and w.size == rows * cols
    packed = np.zeros((rows, cols // 2), np.uint8)
    scales = np.zeros((rows, cols // 32), np.uint8)
    smax = _lib.orc_mxfp4sq_quantize(_p(w, _f32p), rows, cols, _p(packed, _u8p), _p(scales, _u8p))
    return packed, scales, np.float32(smax)


def mxfp4sq_dequant(packed, scales, smax, rows, cols):
    """mxfp4::dequant_sq (src/mxfp4.rs:216-229)."""
    packed, scales = _c(packed, np.uint8), _c(scales, np.uint8)
    assert packed.size == rows * cols // 2 and scales.size == rows * cols // 32
    out = np.empty((rows, cols), np.float32)
    _lib.orc_mxfp4sq_dequant(_p(packed, _u8p), _p(scales, _u8p), float(smax), rows, cols, _p(out, _f32p))
    return out


def search_mx_scale(group, e):
    group = _c(group, np.float32)
    assert group.size == 32
    return _lib.orc_search_mx_scale(_p(group, _f32p), e)


def dequant_fp8(w, scales, rows, cols):
    w, scales = _c(w, np.uint8), _c(scales, np.uint8)
    out = np.empty((rows, cols), np.float32)
    _lib.orc_dequant_fp8(_p(w, _u8p), _p(scales, _u8p), rows, cols, _p(out, _f32p))
    return out


def quantize_fp8(w, rows, cols):
    w = _c(w, np.float32)
    assert rows % 128 == 0 and cols % 128 == 0
    qw = np.empty((rows, cols), np.uint8)
    scales = np.empty((rows // 128, cols // 128), np.uint8)
    _lib.orc_quantize_fp8(_p(w, _f32p), rows, cols, _p(qw, _u8p), _p(scales, _u8p))
    return qw, scales


def fp8_roundtrip(x, block, emax=8):
    """Returns (rounded x, e4m3 codes, e8m0 exponent bytes).  emax = 8 is the reference's clamp of the scale exponent,
    127 the full e8m0 range."""
    x = _c(x, np.float32).copy().reshape(-1)
    codes = np.empty(x.size, np.uint8)
    exps = np.empty((x.size + block - 1) // block, np.uint8)
    _lib.orc_fp8_roundtrip_emax(_p(x, _f32p), x.size, block, emax, _p(codes, _u8p), _p(exps, _u8p))
    return x, codes, exps


def round_bf16(x):
    """x rounded to bfloat16 (nearest, ties to even; inf and NaN unchanged), returned as f32: the input rounding of the
    bf16 prefill section (moe_prefill with round_mxfp8=3)."""
    y = _c(x, np.float32).copy().reshape(-1)
    _lib.orc_round_bf16(_p(y, _f32p), y.size)
    return y.reshape(np.shape(x))


# --------------------------------------------------------------------- q8
def quantize_q8(x):
    x = _c(x, np.float32).reshape(-1)
    assert x.size % 32 == 0
    q = np.empty(x.size, np.int8)
    s = np.empty(x.size // 32, np.float32)
    _lib.orc_quantize_q8(_p(x, _f32p), x.size, _p(q, _i8p), _p(s, _f32p))
    return q, s


def q8_0_rows(x):
    """quantize_q8 of every row of x [n][w]; the f32 block scales are also returned rounded to f16 (the q8_0 storage
    form of the device caches).  Returns (q [n][w] int8, scales f32 [n][w/32], scales f16 [n][w/32])."""
    x = _c(x, np.float32)
    n, w = x.shape
    q = np.empty((n, w), np.int8)
    s = np.empty((n, w // 32), np.float32)
    for i in range(n):
        q[i], s[i] = quantize_q8(x[i])
    return q, s, s.astype(np.float16)


def block_dot(packed16, x32):
    packed16, x32 = _c(packed16, np.uint8), _c(x32, np.int8)
    assert packed16.size == 16 and x32.size == 32
    return _lib.orc_block_dot(_p(packed16, _u8p), _p(x32, _i8p))


def block_dot_i8(w32, x32):
    w32, x32 = _c(w32, np.int8), _c(x32, np.int8)
    assert w32.size == 32 and x32.size == 32
    return _lib.orc_block_dot_i8(_p(w32, _i8p), _p(x32, _i8p))


def dot(a, b):
    a, b = _c(a, np.float32), _c(b, np.float32)
    n = min(a.size, b.size)
    return _lib.orc_dot(_p(a, _f32p), _p(b, _f32p), n)


def rmsnorm(x, w, eps):
    x, w = _c(x, np.float32), _c(w, np.float32)
    out = np.empty(x.size, np.float32)
    _lib.orc_rmsnorm(_p(x, _f32p), x.size, _p(w, _f32p), C.c_float(eps), _p(out, _f32p))
    return out


def matvec_f32(w, rows, cols, x):
    w, x = _c(w, np.float32), _c(x, np.float32)
    out = np.empty(rows, np.float32)
    _lib.orc_matvec_f32(_p(w, _f32p), rows, cols, _p(x, _f32p), _p(out, _f32p))
    return out


# ------------------------------------------------------- VQ1 / LUT GEMV
def vq1_matvec(codebook, indices, rows, cols, x, lut=True):
    """quant::matvec_vq_gather (lut=False, src/quant.rs:313-331) or lutgemv::matvec_vq_lut (src/lutgemv.rs:208-240)."""
    codebook, indices, x = _c(codebook, np.float32), _c(indices, np.uint8), _c(x, np.float32)
    assert codebook.size == 256 * 16 and cols % 16 == 0 and indices.size == rows * cols // 16 and x.size == cols
    out = np.empty(rows, np.float32)
    fn = _lib.orc_vq1_matvec_lut if lut else _lib.orc_vq1_matvec_gather
    fn(_p(codebook, _f32p), _p(indices, _u8p), rows, cols, _p(x, _f32p), _p(out, _f32p))
    return out


def vq1_matvec_nt(codebook, indices, rows, cols, xt, m):
    """quant::matvec_vq_nt (src/quant.rs:353-376): xt [cols, m] -> out [m, rows]."""
    codebook, indices, xt = _c(codebook, np.float32), _c(indices, np.uint8), _c(xt, np.float32)
    assert codebook.size == 256 * 16 and cols % 16 == 0 and m % 8 == 0 and indices.size == rows * cols // 16 and xt.size == cols * m
    out = np.empty((m, rows), np.float32)
    _lib.orc_vq1_matvec_nt(_p(codebook, _f32p), _p(indices, _u8p), rows, cols, _p(xt, _f32p), m, _p(out, _f32p))
    return out


# ---------------------------------------------------------- mxfp4 matvecs
def _chk_packed(packed, scales, rows, cols):
    packed, scales = _c(packed, np.uint8), _c(scales, np.uint8)
    assert cols % 32 == 0
    assert packed.size == rows * cols // 2 and scales.size == rows * cols // 32
    return packed, scales


def matvec_packed(packed, scales, rows, cols, x, mode=1):
    """mode 1: q8 integer path (reference default); mode 0: exact f32 path."""
    packed, scales = _chk_packed(packed, scales, rows, cols)
    x = _c(x, np.float32)
    assert x.size == cols
    out = np.empty(rows, np.float32)
    _lib.orc_matvec_packed(_p(packed, _u8p), _p(scales, _u8p), rows, cols, _p(x, _f32p), _p(out, _f32p), mode)
    return out


def matvec_packed_q8(packed, scales, rows, cols, xq, xs):
    packed, scales = _chk_packed(packed, scales, rows, cols)
    xq, xs = _c(xq, np.int8), _c(xs, np.float32)
    assert xq.size == cols and xs.size == cols // 32
    out = np.empty(rows, np.float32)
    _lib.orc_matvec_packed_q8(_p(packed, _u8p), _p(scales, _u8p), rows, cols, _p(xq, _i8p), _p(xs, _f32p), _p(out, _f32p))
    return out


def matvec_packed_shader_emul(packed, scales, rows, cols, x, lanes=256):
    packed, scales = _chk_packed(packed, scales, rows, cols)
    x = _c(x, np.float32)
    out = np.empty(rows, np.float32)
    _lib.orc_matvec_packed_shader_emul(_p(packed, _u8p), _p(scales, _u8p), rows, cols, _p(x, _f32p), _p(out, _f32p), lanes)
    return out


def matvec_packed_q8_device_order(packed, scales, rows, cols, xq, xs):
    """matvec_packed_q8 with the row sums associated as the single-row MXFP4 GEMV kernel of the library associates them
    (the counterpart of matvec_packed_shader_emul for this device)."""
    packed, scales = _chk_packed(packed, scales, rows, cols)
    xq, xs = _c(xq, np.int8), _c(xs, np.float32)
    out = np.empty(rows, np.float32)
    _lib.orc_matvec_packed_q8_device_order(_p(packed, _u8p), _p(scales, _u8p), rows, cols, _p(xq, _i8p), _p(xs, _f32p), _p(out, _f32p))
    return out


def q8head_matvec_device_order(q, ws, rows, cols, xq, xs):
    """Q8Head::matvec with the row sums associated as the batch-1 q8 GEMV kernel associates them; cols % 1024 == 0."""
    q, ws, xq, xs = _c(q, np.int8), _c(ws, np.float32), _c(xq, np.int8), _c(xs, np.float32)
    assert cols % 1024 == 0 and q.size == rows * cols and ws.size == rows * cols // 32
    out = np.empty(rows, np.float32)
    _lib.orc_q8head_matvec_device_order(_p(q, _i8p), _p(ws, _f32p), rows, cols, _p(xq, _i8p), _p(xs, _f32p), _p(out, _f32p))
    return out


def matvec_packed_nt(packed, scales, rows, cols, xt, m):
    """xt: [cols][m] (m % 8 == 0); returns [m][rows]."""
    packed, scales = _chk_packed(packed, scales, rows, cols)
    xt = _c(xt, np.float32)
    assert m % 8 == 0 and xt.size == cols * m
    out = np.empty((m, rows), np.float32)
    _lib.orc_matvec_packed_nt(_p(packed, _u8p), _p(scales, _u8p), rows, cols, _p(xt, _f32p), m, _p(out, _f32p))
    return out


# ---------------------------------------------------------------- q8 head
def q8head_from_f32(w, rows, cols):
    w = _c(w, np.float32)
    q = np.empty((rows, cols), np.int8)
    s = np.empty((rows, cols // 32), np.float32)
    _lib.orc_q8head_from_f32(_p(w, _f32p), rows, cols, _p(q, _i8p), _p(s, _f32p))
    return q, s


def q8head_matvec(q, ws, rows, cols, x, workers=1):
    q, ws, x = _c(q, np.int8), _c(ws, np.float32), _c(x, np.float32)
    assert q.size == rows * cols and ws.size == rows * cols // 32 and x.size == cols
    out = np.empty(rows, np.float32)
    _lib.orc_q8head_matvec(_p(q, _i8p), _p(ws, _f32p), rows, cols, _p(x, _f32p), _p(out, _f32p), workers)
    return out


def argmax(logits):
    logits = _c(logits, np.float32)
    return _lib.orc_argmax(_p(logits, _f32p), logits.size)


# -------------------------------------------------------------------- MLA
def hadamard64(x):
    x = _c(x, np.float32).copy()
    assert x.size == 64
    _lib.orc_hadamard64(_p(x, _f32p))
    return x


class MlaCache:
    """q8 MLA cache in the reference layout (src/model.rs:765-781): per position
    kq [nh*nope] i8, ks [nh*nope/32] f32, kr [rope] f32, vq [nh*vd] i8, vs [nh*vd/32] f32."""

    def __init__(self, nh, nope, rope, vd, had=False, capacity=1024):
        self.cfg = MlaCfg(nh, nope, rope, vd)
        self.nh, self.nope, self.rope, self.vd, self.had = nh, nope, rope, vd, had
        self.n = 0
        self._alloc(capacity)

    def _alloc(self, cap):
        nh, nope, rope, vd = self.nh, self.nope, self.rope, self.vd
        new = dict(kq=np.zeros((cap, nh * nope), np.int8), ks=np.zeros((cap, nh * nope // 32), np.float32),
                   kr=np.zeros((cap, rope), np.float32), vq=np.zeros((cap, nh * vd), np.int8),
                   vs=np.zeros((cap, nh * vd // 32), np.float32))
        for k, a in new.items():
            if self.n:
                a[:self.n] = getattr(self, k)[:self.n]
            setattr(self, k, a)
        self.cap = cap

    def push(self, k_row, v_row):
        if self.n == self.cap:
            self._alloc(self.cap * 2)
        k_row, v_row = _c(k_row, np.float32), _c(v_row, np.float32)
        assert k_row.size == self.nh * (self.nope + self.rope) and v_row.size == self.nh * self.vd
        j = self.n
        _lib.orc_mla_cache_push(C.byref(self.cfg), int(self.had), _p(k_row, _f32p), _p(v_row, _f32p), _p(self.kq[j], _i8p),
                                _p(self.ks[j], _f32p), _p(self.kr[j], _f32p), _p(self.vq[j], _i8p), _p(self.vs[j], _f32p))
        self.n += 1

    def to_f32(self):
        n = self.n
        k = np.empty((n, self.nh * (self.nope + self.rope)), np.float32)
        v = np.empty((n, self.nh * self.vd), np.float32)
        _lib.orc_mla_cache_to_f32(C.byref(self.cfg), int(self.had), n, _p(self.kq, _i8p), _p(self.ks, _f32p), _p(self.kr, _f32p),
                                  _p(self.vq, _i8p), _p(self.vs, _f32p), _p(k, _f32p), _p(v, _f32p))
        return k, v


def mla_attn_ref(nh, nope, rope, vd, k, v, qh, h, pos, scale):
    cfg = MlaCfg(nh, nope, rope, vd)
    k, v, qh = _c(k, np.float32), _c(v, np.float32), _c(qh, np.float32)
    oh = np.zeros(vd, np.float32)
    _lib.orc_mla_attn_ref(C.byref(cfg), _p(k, _f32p), _p(v, _f32p), _p(qh, _f32p), h, pos, scale, _p(oh, _f32p))
    return oh


def mla_attn_flash(nh, nope, rope, vd, k, v, qh, h, pos, scale):
    cfg = MlaCfg(nh, nope, rope, vd)
    k, v, qh = _c(k, np.float32), _c(v, np.float32), _c(qh, np.float32)
    oh = np.zeros(vd, np.float32)
    _lib.orc_mla_attn_flash(C.byref(cfg), _p(k, _f32p), _p(v, _f32p), _p(qh, _f32p), h, pos, scale, _p(oh, _f32p))
    return oh


def mla_attn_flash_q8(cache, qh, h, pos, scale):
    qh = _c(qh, np.float32)
    oh = np.zeros(cache.vd, np.float32)
    _lib.orc_mla_attn_flash_q8(C.byref(cache.cfg), int(cache.had), _p(cache.kq, _i8p), _p(cache.ks, _f32p), _p(cache.kr, _f32p),
                               _p(cache.vq, _i8p), _p(cache.vs, _f32p), _p(qh, _f32p), h, pos, scale, _p(oh, _f32p))
    return oh


def mla_attn_flash_q8_mqa(cache, q, pos, scale):
    q = _c(q, np.float32)
    attn = np.zeros(cache.nh * cache.vd, np.float32)
    _lib.orc_mla_attn_flash_q8_mqa(C.byref(cache.cfg), int(cache.had), cache.nh, _p(cache.kq, _i8p), _p(cache.ks, _f32p),
                                   _p(cache.kr, _f32p), _p(cache.vq, _i8p), _p(cache.vs, _f32p), _p(q, _f32p), pos, scale,
                                   _p(attn, _f32p))
    return attn


def mla_absorbed_decode(lat_q, lat_s, rope_q, rope_s, q, nh, scale, pos=None):
    """Weight-absorbed MLA decode over a shared q8 latent cache.

    lat_q [n][L] i8, lat_s [n][L/32] f32 (the f16-rounded scales widened),
    rope_q [n][R] i8, rope_s [n][R/32] f32, q [nh][L+R] f32.  The latent row is K
    and V of every head; the rope row is dequantized (q * s, as MlaCache::to_f32
    dequantizes) and enters the score through the f32 rope dot of the reference.
    Returns [nh][L]."""
    lat_q, lat_s = _c(lat_q, np.int8), _c(lat_s, np.float32)
    rope_q, rope_s = _c(rope_q, np.int8), _c(rope_s, np.float32)
    n, L = lat_q.shape
    R = rope_q.shape[1]
    if pos is None:
        pos = n - 1
    kr = (rope_q.astype(np.float32).reshape(n, R // 32, 32) * rope_s.reshape(n, R // 32, 1)).reshape(n, R)
    kr = _c(kr, np.float32)
    cfg = MlaCfg(nh, L, R, L)
    q = _c(q, np.float32)
    assert q.size == nh * (L + R)
    attn = np.zeros(nh * L, np.float32)
    _lib.orc_mla_attn_flash_q8_mqa(C.byref(cfg), 0, 1, _p(lat_q, _i8p), _p(lat_s, _f32p), _p(kr, _f32p), _p(lat_q, _i8p),
                                   _p(lat_s, _f32p), _p(q, _f32p), pos, scale, _p(attn, _f32p))
    return attn.reshape(nh, L)


# -------------------------------------------------------------------- MoE
def gate_forward(x, gate_w, bias, n_experts, topk, route_scale):
    x, gate_w = _c(x, np.float32), _c(gate_w, np.float32)
    b = None if bias is None else _c(bias, np.float32)
    ids = np.empty(topk, np.uint32)
    w = np.empty(topk, np.float32)
    _lib.orc_gate_forward(_p(x, _f32p), x.size, _p(gate_w, _f32p), None if b is None else _p(b, _f32p), n_experts, topk,
                          route_scale, _p(ids, _u32p), _p(w, _f32p))
    return ids, w


def router_sigmoid(logits, bias, topk):
    logits = _c(logits, np.float32)
    b = None if bias is None else _c(bias, np.float32)
    ids = np.empty(topk, np.uint32)
    w = np.empty(topk, np.float32)
    _lib.orc_router_sigmoid(_p(logits, _f32p), None if b is None else _p(b, _f32p), logits.size, topk, _p(ids, _u32p), _p(w, _f32p))
    return ids, w


def router_softmax(logits, topk):
    logits = _c(logits, np.float32)
    ids = np.empty(topk, np.uint32)
    w = np.empty(topk, np.float32)
    _lib.orc_router_softmax(_p(logits, _f32p), logits.size, topk, _p(ids, _u32p), _p(w, _f32p))
    return ids, w


def expert_forward_f32(w1, w2, w3, x, inter, limit):
    w1, w2, w3, x = (_c(a, np.float32) for a in (w1, w2, w3, x))
    d = x.size
    out = np.empty(d, np.float32)
    _lib.orc_expert_forward_f32(_p(w1, _f32p), _p(w2, _f32p), _p(w3, _f32p), _p(x, _f32p), d, inter, limit, _p(out, _f32p))
    return out


class ExpertTable:
    """Arrays of pointers to per-expert (packed, scales) blobs: w1, w3 [inter][d], w2 [d][inter]."""

    def __init__(self, w1, w3, w2, d, inter):
        # w1, w3, w2: lists of (packed uint8 array, scales uint8 array)
        self.d, self.inter, self.n = d, inter, len(w1)
        self._keep = []
        self.ptrs = []
        for lst, (r, c) in ((w1, (inter, d)), (w3, (inter, d)), (w2, (d, inter))):
            pp = (_u8p * self.n)()
            ps = (_u8p * self.n)()
            for i, (pk, sc) in enumerate(lst):
                pk, sc = _chk_packed(pk, sc, r, c)
                self._keep += [pk, sc]
                pp[i] = _p(pk, _u8p)
                ps[i] = _p(sc, _u8p)
            self.ptrs += [pp, ps]  # order: w1p w1s w3p w3s w2p w2s


def expert_packed(w1, w3, w2, d, inter, x, mode=1, act_kind=ACT_SWIGLU, limit=0.0, wgt=1.0):
    (w1p, w1s), (w3p, w3s), (w2p, w2s) = (_chk_packed(p, s, r, c) for (p, s), (r, c) in
                                          ((w1, (inter, d)), (w3, (inter, d)), (w2, (d, inter))))
    x = _c(x, np.float32)
    out = np.empty(d, np.float32)
    _lib.orc_expert_packed(_p(w1p, _u8p), _p(w1s, _u8p), _p(w3p, _u8p), _p(w3s, _u8p), _p(w2p, _u8p), _p(w2s, _u8p), d, inter,
                           _p(x, _f32p), mode, act_kind, limit, wgt, _p(out, _f32p))
    return out


def expert_act(w1, w3, d, inter, x, mode=1, act_kind=ACT_SWIGLU, limit=0.0, wgt=1.0):
    """ACT(W1 x, W3 x): the f32 vector a packed expert hands to its W2 matvec."""
    (w1p, w1s), (w3p, w3s) = (_chk_packed(p, s, inter, d) for (p, s) in (w1, w3))
    x = _c(x, np.float32)
    act = np.empty(inter, np.float32)
    _lib.orc_expert_act(_p(w1p, _u8p), _p(w1s, _u8p), _p(w3p, _u8p), _p(w3s, _u8p), d, inter, _p(x, _f32p), mode, act_kind, limit, wgt,
                        _p(act, _f32p))
    return act


def expert_vq(codebook, i1, i3, i2, d, inter, x, act_kind=ACT_SWIGLU, limit=0.0, wgt=1.0):
    """A VQ1 expert (src/model.rs:2243-2259, vq branch): three quant::matvec_vq calls with the activation between."""
    codebook, x = _c(codebook, np.float32), _c(x, np.float32)
    i1, i3, i2 = _c(i1, np.uint8), _c(i3, np.uint8), _c(i2, np.uint8)
    assert codebook.size == 256 * 16 and i1.size == inter * d // 16 == i3.size == i2.size and x.size == d
    out = np.empty(d, np.float32)
    _lib.orc_expert_vq(_p(codebook, _f32p), _p(i1, _u8p), _p(i3, _u8p), _p(i2, _u8p), d, inter, _p(x, _f32p), act_kind, limit, wgt,
                       _p(out, _f32p))
    return out


def moe_decode_mixed(experts, codebook, d, inter, ids, weights, x, shared=-1, mode=1, act_kind=ACT_SWIGLU, limit=0.0):
    """moe_forward's expert section for a layer that mixes MXFP4 and VQ1 experts (src/model.rs:2227-2264, 2346-2351):
    experts[e] = ("mxfp4", w1, w3, w2) with (packed, scales) pairs or ("vq1", i1, i3, i2) index bytes.  Per token the
    outputs are added in slot order, weight times output (ACT_DS: the weight sits inside the activation), then the
    shared expert unweighted."""
    ids, weights, x = _c(ids, np.uint32), _c(weights, np.float32), _c(x, np.float32)
    B, topk = ids.shape
    out = np.empty((B, d), np.float32)

    def run(e, xt, wgt):
        ex = experts[e]
        if ex[0] == "vq1":
            return expert_vq(codebook, ex[1], ex[2], ex[3], d, inter, xt, act_kind, limit, wgt)
        return expert_packed(ex[1], ex[2], ex[3], d, inter, xt, mode, act_kind, limit, wgt)

    for t in range(B):
        y = np.zeros(d, np.float32)
        for s in range(topk):
            w = np.float32(weights[t, s])
            if act_kind == ACT_DS:
                y = y + run(int(ids[t, s]), x[t], float(w))
            else:
                y = y + w * run(int(ids[t, s]), x[t], 1.0)
        if shared >= 0:
            y = y + run(shared, x[t], 1.0)
        out[t] = y
    return out


def moe_decode(table, ids, weights, x, shared=-1, mode=1, act_kind=ACT_SWIGLU, limit=0.0, threads=1):
    ids, weights, x = _c(ids, np.uint32), _c(weights, np.float32), _c(x, np.float32)
    B, topk = ids.shape
    assert x.shape == (B, table.d)
    out = np.empty((B, table.d), np.float32)
    w1p, w1s, w3p, w3s, w2p, w2s = table.ptrs
    _lib.orc_moe_decode(w1p, w1s, w3p, w3s, w2p, w2s, table.d, table.inter, B, topk, _p(ids, _u32p), _p(weights, _f32p), shared,
                        _p(x, _f32p), mode, act_kind, limit, threads, _p(out, _f32p))
    return out


def moe_prefill(table, ids, weights, x, act_kind=ACT_SWIGLU, round_mxfp8=False):
    """round_mxfp8: False/0 the reference's f32 arithmetic; True/1 inputs and activation through the reference's
    fp8_roundtrip per 32; 2 the same with the full e8m0 scale range (no saturation); 3 inputs and activation rounded
    to bfloat16 (nearest even)."""
    ids, weights, x = _c(ids, np.uint32), _c(weights, np.float32), _c(x, np.float32)
    n, topk = ids.shape
    out = np.empty((n, table.d), np.float32)
    w1p, w1s, w3p, w3s, w2p, w2s = table.ptrs
    _lib.orc_moe_prefill(w1p, w1s, w3p, w3s, w2p, w2s, table.n, table.d, table.inter, n, topk, _p(ids, _u32p), _p(weights, _f32p),
                         _p(x, _f32p), act_kind, int(round_mxfp8), _p(out, _f32p))
    return out
