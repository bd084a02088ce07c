"""VQ1 tensors (src/quant.rs): the matvec over codebook-quantized weights, on the device."""
from . import _lib
from ._lib import check, cur_stream, lib, ptr

VQ_DIM, VQ_K = 16, 256  # src/quant.rs:17-18


def matvec_vq(codebook, indices, rows, cols, x, out=None, exact=False):
    """quant::matvec_vq (src/quant.rs:333-346) through the LUT GEMV (src/lutgemv.rs:208-240).

    codebook [256, 16] f32, indices [rows, cols/16] u8, x [cols] f32: device tensors; returns out [rows] f32.
    exact=True reproduces the reference bit for bit (one lane per row, groups added in order); the default splits a
    row's sum across a wave."""
    import torch
    _lib.require_device()
    if cols % VQ_DIM or codebook.numel() != VQ_K * VQ_DIM or indices.numel() != rows * cols // VQ_DIM or x.numel() != cols:
        raise ValueError("vq1 shapes: codebook [256,16], indices [rows, cols/16], x [cols]")
    if out is None:
        out = torch.empty(rows, dtype=torch.float32, device=x.device)
    ws = torch.empty(lib.mk_vq1_workspace_bytes(cols), dtype=torch.uint8, device=x.device)
    check(lib.mk_dev_vq1_matvec(ptr(codebook.contiguous()), ptr(indices.contiguous()), rows, cols, ptr(x.contiguous()), int(exact),
                                ptr(ws), ptr(out), cur_stream()))
    return out


def matvec_vq_nt(codebook, indices, rows, cols, xt, m, out=None):
    """quant::matvec_vq_nt (src/quant.rs:353-376): xt [cols, m] f32 (m inputs transposed, m % 8 == 0) -> out [m, rows],
    bit-identical to the reference (one sequential multiply-add chain per row and position)."""
    import torch
    _lib.require_device()
    if cols % VQ_DIM or m % 8 or codebook.numel() != VQ_K * VQ_DIM or indices.numel() != rows * cols // VQ_DIM or xt.numel() != cols * m:
        raise ValueError("vq1 shapes: codebook [256,16], indices [rows, cols/16], xt [cols, m] with m a multiple of 8")
    if out is None:
        out = torch.empty((m, rows), dtype=torch.float32, device=xt.device)
    check(lib.mk_dev_vq1_matvec_nt(ptr(codebook.contiguous()), ptr(indices.contiguous()), rows, cols, ptr(xt.contiguous()), m, ptr(out),
                                   cur_stream()))
    return out
