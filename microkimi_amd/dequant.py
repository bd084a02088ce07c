"""Host mirror of src/dequant.rs: DeepSeek-V4 checkpoint formats."""
from . import _lib, mxfp4
from ._lib import check, cur_stream, lib, ptr


def dequant_fp4(packed, scales, rows, cols):
    """dequant::dequant_fp4 (src/dequant.rs:43-45): the MXFP4 layout under its V4 name."""
    return mxfp4.dequant(packed, scales, rows, cols)


def dequant_fp8(w, scales, rows, cols):
    """dequant::dequant_fp8 (src/dequant.rs:27-39): e4m3fn bytes + e8m0 per 128x128 block -> f32, device tensors."""
    import torch
    if w.numel() != rows * cols or scales.numel() != ((rows + 127) // 128) * ((cols + 127) // 128):
        raise ValueError("fp8: bad weight or scale length")
    _lib.require_device()
    out = torch.empty((rows, cols), dtype=torch.float32, device=w.device)
    check(lib.mk_dev_fp8_dequant(ptr(w), ptr(scales), rows, cols, ptr(out), cur_stream()))
    return out


def quantize_fp8(w):
    """dequant::quantize_fp8 (src/dequant.rs:50-74) of a device tensor [rows, cols] f32, both multiples of 128:
    (e4m3fn codes [rows, cols], e8m0 scales [rows/128, cols/128])."""
    import torch
    _lib.require_device()
    w = w.contiguous()
    rows, cols = w.shape
    if rows % 128 or cols % 128:
        raise ValueError("fp8: rows and cols must be multiples of 128")
    qw = torch.empty((rows, cols), dtype=torch.uint8, device=w.device)
    scales = torch.empty((rows // 128, cols // 128), dtype=torch.uint8, device=w.device)
    check(lib.mk_dev_quantize_fp8(ptr(w), rows, cols, ptr(qw), ptr(scales), cur_stream()))
    return qw, scales


def quantize_mxfp8(x):
    """deepseek::fp8_roundtrip with block 32 (src/deepseek.rs:312-322) in coded form: (e4m3 codes, e8m0 exponents)."""
    import torch
    _lib.require_device()
    x = x.contiguous()
    n = x.shape[-1]
    nvec = x.numel() // n
    codes = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    exps = torch.empty(x.shape[:-1] + (n // 32,), dtype=torch.uint8, device=x.device)
    check(lib.mk_dev_quantize_mxfp8(ptr(x), nvec, n, ptr(codes), ptr(exps), cur_stream()))
    return codes, exps


def quantize_bf16_split(x):
    """bfloat16 of x [..., n] (n % 512 == 0) as two e4m3 terms per value (mk_dev_quantize_bf16_split): codes
    [..., n / 512, 2, 512] and exps [..., n / 512, 2, 16], the activation format of model.grouped_gemm_split."""
    import torch
    _lib.require_device()
    x = x.contiguous()
    n = x.shape[-1]
    nvec = x.numel() // n
    codes = torch.empty(x.shape[:-1] + (n // 512, 2, 512), dtype=torch.uint8, device=x.device)
    exps = torch.empty(x.shape[:-1] + (n // 512, 2, 16), dtype=torch.uint8, device=x.device)
    check(lib.mk_dev_quantize_bf16_split(ptr(x), nvec, n, ptr(codes), ptr(exps), cur_stream()))
    return codes, exps
