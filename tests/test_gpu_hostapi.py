"""GPU tests of the host-level drop-in entry points (host slices in, host slices out) and their error behaviour."""
import ctypes

import numpy as np
import pytest

import oracle
from gpu_util import rel_l2, torch_cuda

pytestmark = pytest.mark.gpu


def test_matvec_packed_host_slices_and_weight_cache():
    torch_cuda()
    from microkimi_amd import mxfp4, q8, workloads
    p, s, x = workloads.config0(rows=512, cols=7168)
    out = np.zeros(512, np.float32)
    for mode in (1, 0, -1):
        q8.force_q8(mode)
        mxfp4.matvec_packed(p, s, 512, 7168, x, out)
        want = oracle.matvec_packed(p, s, 512, 7168, x, mode=0 if mode == 0 else 1)
        assert rel_l2(out, want) <= 1e-5
    q8.force_q8(-1)
    # second call hits the pointer-keyed cache; changing the host bytes behind the same pointer must be noticed
    p[0, :16] ^= 0x5A
    mxfp4.matvec_packed(p, s, 512, 7168, x, out)
    assert rel_l2(out, oracle.matvec_packed(p, s, 512, 7168, x, mode=1)) <= 1e-5


def test_q8head_host_api():
    torch_cuda()
    from microkimi_amd import _lib
    rows, cols, batch = 2000, 1024, 11
    rng = np.random.default_rng(3)
    w = (rng.standard_normal((rows, cols)) * 0.02).astype(np.float32)
    x = rng.standard_normal((batch, cols)).astype(np.float32)
    h = ctypes.c_void_p()
    _lib.check(_lib.lib.mk_q8head_from_f32(_lib.hptr(w), rows, cols, 0, ctypes.byref(h)))
    out = np.zeros((batch, rows), np.float32)
    am = np.zeros(batch, np.int32)
    _lib.check(_lib.lib.mk_q8head_matvec(h, _lib.hptr(x), batch, _lib.hptr(out), _lib.hptr(am)))
    q, s = oracle.q8head_from_f32(w, rows, cols)
    for b in range(batch):
        want = oracle.q8head_matvec(q, s, rows, cols, x[b])
        assert rel_l2(out[b], want) <= 1e-5
        assert am[b] == oracle.argmax(want)
    _lib.lib.mk_q8head_free(h)
    # from_q8 with f16 storage
    s16 = s.astype(np.float16)
    s16_as_f32 = s16.astype(np.float32)  # must outlive the call: hptr() only takes the address
    _lib.check(_lib.lib.mk_q8head_from_q8(_lib.hptr(q), _lib.hptr(s16_as_f32), rows, cols, 1, ctypes.byref(h)))
    _lib.check(_lib.lib.mk_q8head_matvec(h, _lib.hptr(x), 1, _lib.hptr(out), None))
    assert rel_l2(out[0], oracle.q8head_matvec(q, s16.astype(np.float32), rows, cols, x[0])) <= 1e-5
    _lib.lib.mk_q8head_free(h)


def test_mla_cache_host_api():
    torch_cuda()
    from microkimi_amd import _lib, workloads
    nh, L, R, n = 8, 512, 64, 130
    rng = np.random.default_rng(8)
    lat = rng.standard_normal((n, L)).astype(np.float32)
    rope = rng.standard_normal((n, R)).astype(np.float32)
    q = rng.standard_normal((nh, L + R)).astype(np.float32)
    c = ctypes.c_void_p()
    _lib.check(_lib.lib.mk_mla_cache_new(nh, L, R, n, ctypes.byref(c)))
    for j in range(n):
        _lib.check(_lib.lib.mk_mla_cache_push(c, _lib.hptr(lat[j]), _lib.hptr(rope[j])))
    assert _lib.lib.mk_mla_cache_positions(c) == n
    assert _lib.lib.mk_mla_cache_push(c, _lib.hptr(lat[0]), _lib.hptr(rope[0])) == -5  # full
    out = np.zeros((nh, L), np.float32)
    _lib.check(_lib.lib.mk_mla_attn(c, _lib.hptr(q), workloads.MLA_SCALE, _lib.hptr(out)))
    lq, ls = workloads.q8_0_rows(lat)
    rq, rs = workloads.q8_0_rows(rope)
    want = oracle.mla_absorbed_decode(lq, ls.astype(np.float32), rq, rs.astype(np.float32), q, nh, workloads.MLA_SCALE)
    assert rel_l2(out, want) <= 1e-5
    lat2, rope2 = np.zeros_like(lat), np.zeros_like(rope)
    _lib.check(_lib.lib.mk_mla_cache_to_f32(c, _lib.hptr(lat2), _lib.hptr(rope2)))
    assert np.array_equal(lat2, lq.astype(np.float32) * np.repeat(ls.astype(np.float32), 32, axis=1))
    _lib.lib.mk_mla_cache_free(c)


def test_invalid_arguments_write_nothing():
    torch_cuda()
    from microkimi_amd import _lib
    out = np.full(4, 3.0, np.float32)
    st = _lib.lib.mk_mxfp4_matvec(_lib.hptr(np.zeros(40, np.uint8)), _lib.hptr(np.zeros(4, np.uint8)), 4, 20, _lib.hptr(np.zeros(20, np.float32)),
                                  _lib.hptr(out))
    assert st == -1 and np.all(out == 3.0)
    assert _lib.lib.mk_available() == 1
