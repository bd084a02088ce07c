"""MKIM weight files (src/weights.rs): the reader's interface, over the C ABI's mk_bin_* entry points.

    f = BinFile.open(path)            # BinFile::open: header + directory, whole file mapped read-only
    f.entries[name]                   # Entry(dtype, dims, offset, size)
    f.config                          # dict from the MKIM0002 JSON block, None for MKIM0001
    f.blob(name) / f.f32_vec(name) / f.i32_vec(name) / f.mxfp4_parts(name)
    experts = f.load_experts("layers.3.", n_experts)    # one layer's routed experts, resident on the device

`load_experts` returns an object that model.moe_decode / model.moe_prefill accept in place of PackedExperts.
"""
import collections
import ctypes as C
import json

import numpy as np

from . import _lib
from ._lib import BinEntry, check, lib

DTYPE_F32, DTYPE_MXFP4, DTYPE_I32, DTYPE_VQ1, DTYPE_MXFP4SQ = 0, 1, 2, 3, 4  # src/weights.rs:25-29

Entry = collections.namedtuple("Entry", "dtype dims offset size")  # src/weights.rs:31-37


class DeviceExperts:
    """The routed experts of one layer on the device (mk_bin_load_experts); owns the device memory."""

    def __init__(self, handle):
        self._h = handle
        t = lib.mk_expert_set_table(handle).contents
        self.table = t
        self.d, self.inter = int(t.d), int(t.inter)
        self.has_vq = bool(t.vq_codebook)  # VQ1 experts among them (dtype 3): the file's codebook came along
        self.n = int(lib.mk_expert_set_count(handle))
        self.bytes = int(lib.mk_expert_set_bytes(handle))
        self._ws = None

    def close(self):
        if self._h:
            lib.mk_expert_set_free(self._h)
            self._h = None

    def __del__(self):
        self.close()


class BinFile:
    def __init__(self, handle):
        self._h = handle
        self.entries = {}
        self.names = []
        name, e = C.c_char_p(), BinEntry()
        for i in range(lib.mk_bin_n_tensors(handle)):
            check(lib.mk_bin_entry_at(handle, i, C.byref(name), C.byref(e)))
            n = name.value.decode("utf-8")
            self.names.append(n)
            self.entries[n] = Entry(int(e.dtype), tuple(int(e.dims[k]) for k in range(e.n_dims)), int(e.offset), int(e.size))
        ln = C.c_size_t()
        p = lib.mk_bin_config_json(handle, C.byref(ln))
        self.config = json.loads(C.string_at(p, ln.value).decode("utf-8")) if p else None

    @classmethod
    def open(cls, path):
        h = C.c_void_p()
        check(lib.mk_bin_open(str(path).encode("utf-8"), C.byref(h)))
        return cls(h)

    def close(self):
        if self._h:
            lib.mk_bin_close(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def _entry(self, name):
        e = self.entries.get(name)
        if e is None:
            raise KeyError(f"missing tensor: {name}")
        return e

    def blob(self, name):
        """The tensor's bytes (a copy of the mapped range: the mapping goes away with close())."""
        self._entry(name)
        ln = C.c_size_t()
        p = lib.mk_bin_blob(self._h, name.encode("utf-8"), C.byref(ln))
        return np.frombuffer(C.string_at(p, ln.value), dtype=np.uint8)

    def f32_vec(self, name):
        e = self._entry(name)
        if e.dtype != DTYPE_F32:
            raise TypeError(f"{name} is not f32")
        return self.blob(name).view("<f4").reshape(e.dims)

    def i32_vec(self, name):
        e = self._entry(name)
        if e.dtype != DTYPE_I32:
            raise TypeError(f"{name} is not i32")
        return self.blob(name).view("<i4").reshape(e.dims)

    def mxfp4_parts(self, name):
        """(packed [R, C/2] u8, scales [R, C/32] u8, R, C) of an mxfp4 tensor (src/weights.rs:619-627)."""
        e = self._entry(name)
        if e.dtype != DTYPE_MXFP4:
            raise TypeError(f"{name} is not mxfp4")
        r, c = e.dims
        b = self.blob(name)
        return b[: r * c // 2].reshape(r, c // 2), b[r * c // 2:].reshape(r, c // 32), r, c

    def load_experts(self, layer_prefix, n_experts):
        """Uploads "<layer_prefix>block_sparse_moe.experts.<e>.w1|w2|w3", e < n_experts, as stored."""
        _lib.require_device()
        h = C.c_void_p()
        check(lib.mk_bin_load_experts(self._h, layer_prefix.encode("utf-8"), n_experts, C.byref(h)))
        return DeviceExperts(h)
