"""The C ABI without a GPU: the library loads, exports every symbol include/mk_hip.h declares, and fails loudly
(negative status, message, nothing written) when no device is present."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "mk_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mk_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from microkimi_amd import _lib
    names = declared_symbols()
    assert len(names) >= 35
    raw = ctypes.CDLL(_lib.LIB_PATH)
    missing = [n for n in names if not hasattr(raw, n)]
    assert not missing, missing
    assert set(names) == set(_lib.SYMBOLS)  # the Python binding covers the whole header


def test_no_oracle_in_product_path():
    # the product package must not import, load or name the CPU oracle
    pkg = os.path.join(ROOT, "microkimi_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "import oracle" not in text and "libmk_oracle" not in text and "from oracle" not in text, f


def test_fails_loudly_without_device():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a device is present")
    from microkimi_amd import _lib, mxfp4
    assert _lib.lib.mk_available() == 0
    packed = np.zeros((4, 16), np.uint8)
    scales = np.full((4, 1), 127, np.uint8)
    out = np.full(4, 7.0, np.float32)
    with pytest.raises(_lib.MkError) as e:
        mxfp4.matvec_packed(packed, scales, 4, 32, np.ones(32, np.float32), out)
    assert e.value.status == -2 and "device" in str(e.value)
    assert np.all(out == 7.0)  # untouched: there is no CPU fallback


def test_argument_checks_need_no_device():
    from microkimi_amd import _lib, mxfp4
    with pytest.raises(ValueError):
        mxfp4.matvec_packed(np.zeros(8, np.uint8), np.zeros(1, np.uint8), 1, 16, np.zeros(16, np.float32), np.zeros(1, np.float32))
    # the C ABI itself rejects a cols that is not a multiple of 32 before touching the device
    st = _lib.lib.mk_dev_mxfp4_dequant(ctypes.c_void_p(16), ctypes.c_void_p(16), 1, 48, ctypes.c_void_p(16), None)
    assert st == -1 and b"multiple of 32" in _lib.lib.mk_last_error()
    st = _lib.lib.mk_dev_q8_matvec(ctypes.c_void_p(16), ctypes.c_void_p(16), 1, 4, 64, ctypes.c_void_p(16), ctypes.c_void_p(16), 9,
                                   ctypes.c_void_p(16), None)
    assert st == -1 and b"batch" in _lib.lib.mk_last_error()


def test_argument_checks_of_the_two_term_and_scale_layout_entry_points():
    # shapes these entry points do not take are refused before anything is launched
    from microkimi_amd import _lib
    lib, p16 = _lib.lib, ctypes.c_void_p(16)
    assert lib.mk_dev_mxfp4_scales_by_tile(p16, 8, 768, p16, None) == -1 and b"512" in lib.mk_last_error()
    assert lib.mk_dev_mxfp4_scales_by_tile(p16, 8, 1024, ctypes.c_void_p(8), None) == -1 and b"aligned" in lib.mk_last_error()
    assert lib.mk_dev_quantize_bf16_split(p16, 2, 256, p16, p16, None) == -1 and b"512" in lib.mk_last_error()
    assert lib.mk_dev_quantize_bf16_split(None, 2, 512, p16, p16, None) == -1
    st = lib.mk_dev_mxfp4_grouped_gemm_split(p16, p16, 1, 64, 256, p16, p16, p16, 4, p16, None)
    assert st == -4 and b"512" in lib.mk_last_error()   # MK_ERR_UNSUPPORTED


def test_off_switch_returns_no_device_before_anything_else():
    # mk_set_enabled(0): every status-returning entry point answers MK_ERR_NO_DEVICE, also for arguments that it would
    # otherwise reject (the switch is tested first) and for device-level calls (whose launch would otherwise be tried)
    from microkimi_amd import _lib
    lib = _lib.lib
    assert lib.mk_enabled_now() == 1
    lib.mk_set_enabled(0)
    try:
        assert lib.mk_enabled_now() == 0 and lib.mk_available() == 0
        assert lib.mk_init(0) == -2 and b"switched off" in lib.mk_last_error()
        st = lib.mk_dev_mxfp4_dequant(ctypes.c_void_p(16), ctypes.c_void_p(16), 1, 48, ctypes.c_void_p(16), None)
        assert st == -2
        st = lib.mk_dev_mxfp4_dequant(ctypes.c_void_p(16), ctypes.c_void_p(16), 1, 64, ctypes.c_void_p(16), None)
        assert st == -2
        out = np.full(4, 7.0, np.float32)
        st = lib.mk_mxfp4_matvec(_lib.hptr(np.zeros((4, 16), np.uint8)), _lib.hptr(np.full((4, 1), 127, np.uint8)), 4, 32,
                                 _lib.hptr(np.ones(32, np.float32)), _lib.hptr(out))
        assert st == -2 and np.all(out == 7.0)
        assert lib.mk_dev_moe_count_bad_ids(ctypes.c_void_p(16), 8, 4, ctypes.c_void_p(16), None) == -2
    finally:
        lib.mk_set_enabled(1)
    assert lib.mk_enabled_now() == 1
    st = lib.mk_dev_mxfp4_dequant(ctypes.c_void_p(16), ctypes.c_void_p(16), 1, 48, ctypes.c_void_p(16), None)
    assert st == -1   # back on: the argument check answers again


def test_off_switch_from_the_environment():
    import subprocess
    import sys
    code = ("import ctypes; from microkimi_amd import _lib; l = _lib.lib; "
            "print(l.mk_enabled_now(), l.mk_init(0), l.mk_available()); l.mk_set_enabled(1); print(l.mk_enabled_now())")
    env = dict(os.environ, MK_HIP="0")
    out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, cwd=ROOT, timeout=300)
    assert out.returncode == 0, out.stderr
    assert out.stdout.split() == ["0", "-2", "0", "1"]


def test_workloads_are_reproducible():
    from microkimi_amd import workloads as w
    p, s, x = w.config0(rows=8, cols=64)
    p2, s2, x2 = w.config0(rows=8, cols=64)
    assert np.array_equal(p, p2) and np.array_equal(s, s2) and np.array_equal(x, x2)
    assert s.min() >= 118 and s.max() <= 130
    q, sc, xx = w.config1(rows=64, cols=64, batch=2)
    assert q.min() >= -127 and sc.dtype == np.float16 and xx.shape == (2, 64)
