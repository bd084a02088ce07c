"""microkimi_amd: microkimi's quantized-weight hot path on one MI355X.

The package is a thin host mirror of the reference's operator modules
(mxfp4.rs, q8.rs, dequant.rs and the operators inside model.rs / deepseek.rs)
over the C ABI of libmk_hip.so.  Device memory and streams come from torch.
"""
from . import _lib  # noqa: F401  (fails loudly when libmk_hip.so is not built)
from . import dequant, model, mxfp4, q8  # noqa: F401

__all__ = ["mxfp4", "q8", "dequant", "model"]
