"""Host mirror of src/mxfp4.rs: MXFP4 dequantization and the packed matvec entry points."""
import numpy as np

from . import _lib, q8 as _q8
from ._lib import MODE_F32, MODE_Q8, check, cur_stream, hptr, lib, ptr

E2M1 = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0)  # src/mxfp4.rs:5-7


def _check_shapes(packed, scales, rows, cols):
    if cols % 32 != 0:
        raise ValueError("cols must be a multiple of 32")  # the reference asserts (src/mxfp4.rs:95, src/metal.rs:944)
    n = packed.size if isinstance(packed, np.ndarray) else packed.numel()
    m = scales.size if isinstance(scales, np.ndarray) else scales.numel()
    if n != rows * cols // 2 or m != rows * cols // 32:
        raise ValueError("packed/scales length does not match rows x cols")


def dequant(packed, scales, rows, cols):
    """mxfp4::dequant (src/mxfp4.rs:19-31): f32 [rows, cols], bit-exact."""
    _check_shapes(packed, scales, rows, cols)
    if isinstance(packed, np.ndarray):
        packed, scales = np.ascontiguousarray(packed, np.uint8), np.ascontiguousarray(scales, np.uint8)
        out = np.empty((rows, cols), np.float32)
        check(lib.mk_mxfp4_dequant(hptr(packed), hptr(scales), rows, cols, hptr(out)))
        return out
    import torch
    _lib.require_device()
    out = torch.empty((rows, cols), dtype=torch.float32, device=packed.device)
    check(lib.mk_dev_mxfp4_dequant(ptr(packed), ptr(scales), rows, cols, ptr(out), cur_stream()))
    return out


def quantize(w, search=True):
    """mxfp4::quantize (search) / quantize_naive (src/mxfp4.rs:38-138) of a device tensor [rows, cols] f32: the
    reference's (packed [rows, cols/2], scales [rows, cols/32]) bytes."""
    import torch
    _lib.require_device()
    w = w.contiguous()
    rows, cols = w.shape
    if cols % 32:
        raise ValueError("cols must be a multiple of 32")
    packed = torch.empty((rows, cols // 2), dtype=torch.uint8, device=w.device)
    scales = torch.empty((rows, cols // 32), dtype=torch.uint8, device=w.device)
    check(lib.mk_dev_mxfp4_quantize(ptr(w), rows, cols, int(bool(search)), ptr(packed), ptr(scales), cur_stream()))
    return packed, scales


def quantize_sq(w):
    """mxfp4::quantize_sq (src/mxfp4.rs:160-214) of a device tensor [rows, cols] f32: (packed, scale bytes, smax as a
    one-element device tensor)."""
    import torch
    _lib.require_device()
    w = w.contiguous()
    rows, cols = w.shape
    if cols % 32:
        raise ValueError("cols must be a multiple of 32")
    packed = torch.empty((rows, cols // 2), dtype=torch.uint8, device=w.device)
    scales = torch.empty((rows, cols // 32), dtype=torch.uint8, device=w.device)
    smax = torch.empty(1, dtype=torch.float32, device=w.device)
    check(lib.mk_dev_mxfp4sq_quantize(ptr(w), rows, cols, ptr(packed), ptr(scales), ptr(smax), cur_stream()))
    return packed, scales, smax


def dequant_sq(packed, scales, smax, rows, cols):
    """mxfp4::dequant_sq (src/mxfp4.rs:216-229) on device tensors; smax a float or a one-element device tensor."""
    import torch
    _lib.require_device()
    _check_shapes(packed, scales, rows, cols)
    out = torch.empty((rows, cols), dtype=torch.float32, device=packed.device)
    on_dev = isinstance(smax, torch.Tensor)
    check(lib.mk_dev_mxfp4sq_dequant(ptr(packed), ptr(scales), ptr(smax) if on_dev else None, 0.0 if on_dev else float(smax), rows, cols,
                                     ptr(out), cur_stream()))
    return out


def dequant_any(dtype, blob, rows, cols):
    """mxfp4::dequant_any (src/mxfp4.rs:231-240) on a raw blob of either flavour (a uint8 device tensor): packed || scales
    for dtype 1, packed || scales || smax (f32) for dtype 4."""
    n_p, n_s = rows * cols // 2, rows * cols // 32
    if dtype == 1:
        return dequant(blob[:n_p].contiguous(), blob[n_p:n_p + n_s].contiguous(), rows, cols)
    if dtype == 4:
        smax = float(blob[n_p + n_s:n_p + n_s + 4].cpu().numpy().view(np.float32)[0])
        return dequant_sq(blob[:n_p].contiguous(), blob[n_p:n_p + n_s].contiguous(), smax, rows, cols)
    raise ValueError(f"dequant_any: dtype {dtype} is not an mxfp4 flavor")


def quantize_naive(w):
    """mxfp4::quantize_naive (src/mxfp4.rs:94-100)."""
    return quantize(w, search=False)


def matvec_packed_q8(packed, scales, rows, cols, xq, out):
    """mxfp4::matvec_packed_q8 (src/mxfp4.rs:405-443) on device tensors; xq is a q8.Q8Vec."""
    _check_shapes(packed, scales, rows, cols)
    if xq.q.numel() != cols or xq.scales.numel() != cols // 32 or out.numel() != rows:
        raise ValueError("activation / output length does not match the matrix")
    _lib.require_device()
    check(lib.mk_dev_mxfp4_matvec_q8(ptr(packed), ptr(scales), rows, cols, ptr(xq.q), ptr(xq.scales), ptr(out), cur_stream()))


def matvec_packed(packed, scales, rows, cols, x, out, n_threads=1):
    """mxfp4::matvec_packed (src/mxfp4.rs:458-539): out[r] = sum_c W[r,c] x[c].

    The arithmetic follows q8.q8_enabled(): the q8 integer path by default, the exact f32 path under
    MICROKIMI_NO_Q8=1 / force_q8(0).  n_threads is accepted for signature parity and ignored.
    numpy arguments take the host-level drop-in (weights cached on the device by pointer); torch CUDA
    tensors stay on the device and the call only enqueues work on the current stream."""
    _check_shapes(packed, scales, rows, cols)
    if isinstance(packed, np.ndarray):
        if x.size != cols or out.size != rows:
            raise ValueError("activation / output length does not match the matrix")
        assert out.dtype == np.float32 and out.flags["C_CONTIGUOUS"]
        x = np.ascontiguousarray(x, np.float32)
        check(lib.mk_mxfp4_matvec(hptr(packed), hptr(scales), rows, cols, hptr(x), hptr(out)))
        return
    import torch
    if x.numel() != cols or out.numel() != rows:
        raise ValueError("activation / output length does not match the matrix")
    _lib.require_device()
    if _q8.q8_enabled():
        xq = torch.empty(cols, dtype=torch.int8, device=x.device)
        xs = torch.empty(cols // 32, dtype=torch.float32, device=x.device)
        check(lib.mk_dev_mxfp4_matvec(ptr(packed), ptr(scales), rows, cols, ptr(x), ptr(out), MODE_Q8, ptr(xq), ptr(xs), cur_stream()))
    else:
        check(lib.mk_dev_mxfp4_matvec(ptr(packed), ptr(scales), rows, cols, ptr(x), ptr(out), MODE_F32, None, None, cur_stream()))


def matvec_packed_q8_batched(packed, scales, rows, cols, xq, out=None):
    """matvec_packed_q8 (src/mxfp4.rs:405-443) for the m rows of the Q8Vec xq ([m, cols] int8 + [m, cols/32] scales)
    against one matrix on the matrix cores, with the reference's block terms bit for bit; returns [m, rows]."""
    import torch
    _lib.require_device()
    m = xq.q.shape[0] if xq.q.dim() == 2 else 1
    if out is None:
        out = torch.empty((m, rows), dtype=torch.float32, device=packed.device)
    ws = torch.empty(256, dtype=torch.uint8, device=packed.device)
    check(lib.mk_dev_mxfp4_matvec_q8_batched(ptr(packed), ptr(scales), rows, cols, ptr(xq.q), ptr(xq.scales), m, ptr(ws), ptr(out), cur_stream()))
    return out


def matvec_packed_grouped_q8(packed_list, scales_list, rows, cols, xq, x_index, outs):
    """One launch over many matrices of one shape (the grouped-expert form): packed_list / scales_list / outs are
    lists of device tensors, xq a Q8Vec holding [nx, cols] activations, x_index an int32 device tensor or None."""
    import torch
    _lib.require_device()
    dev = packed_list[0].device
    mk = lambda ts: torch.tensor([t.data_ptr() for t in ts], dtype=torch.int64, device=dev)
    pp, sp, op = mk(packed_list), mk(scales_list), mk(outs)
    check(lib.mk_dev_mxfp4_matvec_q8_grouped(ptr(pp), ptr(sp), len(packed_list), rows, cols, ptr(xq.q), ptr(xq.scales), ptr(x_index), ptr(op),
                                             cur_stream()))
    return pp, sp, op  # keep alive until the stream has run
