"""Host mirror of src/q8.rs: q8_0 activation quantization and the q8 toggle."""
import numpy as np

from . import _lib
from ._lib import check, cur_stream, hptr, lib, ptr


class Q8Vec:
    """q8::Q8Vec (src/q8.rs:26-29): int8 values + one f32 scale per block of 32."""

    def __init__(self, q, scales):
        self.q, self.scales = q, scales


def q8_enabled():
    """q8::q8_enabled (src/q8.rs:77-83)."""
    return bool(lib.mk_q8_enabled())


def force_q8(v):
    """q8::force_q8 (src/q8.rs:87-89): -1 follows MICROKIMI_NO_Q8, 0 / 1 force the f32 / q8 path."""
    lib.mk_force_q8(int(v))


def quantize_q8(x):
    """q8::quantize_q8 (src/q8.rs:40-44).

    torch CUDA tensor [..., n] (n % 32 == 0) -> Q8Vec of device tensors, enqueued on the current stream;
    numpy array -> Q8Vec of numpy arrays through the host-level entry point."""
    if isinstance(x, np.ndarray):
        x = np.ascontiguousarray(x, np.float32).reshape(-1)
        assert x.size % 32 == 0, "q8 blocks are 32 wide"
        q = np.empty(x.size, np.int8)
        s = np.empty(x.size // 32, np.float32)
        check(lib.mk_quantize_q8(hptr(x), x.size, hptr(q), hptr(s)))
        return Q8Vec(q, s)
    import torch
    assert x.is_cuda and x.dtype == torch.float32
    _lib.require_device()
    x = x.contiguous()
    n = x.shape[-1]
    assert n % 32 == 0, "q8 blocks are 32 wide"
    nvec = x.numel() // n if n else 0
    q = torch.empty(x.shape, dtype=torch.int8, device=x.device)
    s = torch.empty(x.shape[:-1] + (n // 32,), dtype=torch.float32, device=x.device)
    check(lib.mk_dev_quantize_q8(ptr(x), nvec, n, ptr(q), ptr(s), cur_stream()))
    return Q8Vec(q, s)
