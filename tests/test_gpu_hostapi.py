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


def test_weight_cache_budget_is_an_error_not_an_eviction():
    # MICROKIMI_GPU_CACHE_MB (src/metal.rs:554-558): a weight that does not fit the budget is not uploaded; the call fails
    # with MK_ERR_NOMEM and a message, leaves `out` alone, and works once the budget is raised
    torch_cuda()
    from microkimi_amd import workloads
    from microkimi_amd._lib import check, hptr, lib
    rows, cols = 2048, 2048                       # 2 MiB of nibbles + 128 KiB of scale bytes
    p, s, x = workloads.config0(rows=rows, cols=cols)
    out = np.full(rows, 7.0, np.float32)
    lib.mk_set_cache_mb(1)
    try:
        st = lib.mk_mxfp4_matvec(hptr(p), hptr(s), rows, cols, hptr(x), hptr(out))
        assert st == -5 and b"budget exhausted" in lib.mk_last_error()
        assert np.all(out == 7.0)
        lib.mk_set_cache_mb(1 << 20)
        check(lib.mk_mxfp4_matvec(hptr(p), hptr(s), rows, cols, hptr(x), hptr(out)))
        assert rel_l2(out, oracle.matvec_packed(p, s, rows, cols, x, mode=1)) <= 1e-5
        lib.mk_set_cache_mb(1)                    # a cached weight stays usable under a budget that is lowered afterwards
        out2 = np.zeros(rows, np.float32)
        check(lib.mk_mxfp4_matvec(hptr(p), hptr(s), rows, cols, hptr(x), hptr(out2)))
        assert np.array_equal(out, out2)
    finally:
        lib.mk_set_cache_mb(0)


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


def test_matvec_f32_host_level_is_bit_identical_and_cached():
    # metal::gpu_matvec (src/metal.rs:750): host slices, the weight cached by (pointer, rows, cols)
    import ctypes as C
    from microkimi_amd._lib import Prof, check, hptr, lib
    rng = np.random.default_rng(3)
    rows, cols = 300, 1000
    w = rng.standard_normal((rows, cols)).astype(np.float32)
    x = rng.standard_normal(cols).astype(np.float32)
    y = np.empty(rows, np.float32)
    lib.mk_prof_reset()
    lib.mk_prof_enable(1)
    try:
        for _ in range(3):
            check(lib.mk_matvec_f32(hptr(w), rows, cols, hptr(x), hptr(y)))
        want = oracle.matvec_f32(w, rows, cols, x)
        assert np.array_equal(y.view(np.uint32), want.view(np.uint32))
        w[0, 0] += 1.0   # same pointer, other contents: the first 16 bytes differ, the copy is replaced
        check(lib.mk_matvec_f32(hptr(w), rows, cols, hptr(x), hptr(y)))
        assert np.array_equal(y.view(np.uint32), oracle.matvec_f32(w, rows, cols, x).view(np.uint32))
        p = Prof()
        lib.mk_prof_get(C.byref(p))
        # GpuProf (src/metal.rs:667-716): 4 calls, 2 uploads (first use, changed contents), 2 hits, phases timed
        assert (p.calls, p.misses, p.hits) == (4, 2, 2)
        assert p.t_wait_ms > 0 and p.t_readback_ms > 0 and p.t_io_ms > 0 and p.cache_tensors >= 1
        lib.mk_prof_print()
    finally:
        lib.mk_prof_enable(0)


def test_host_level_matvec_from_several_threads():
    # the reference calls matvec_packed from its pool workers, one job per selected expert (src/model.rs:2227-2264):
    # eight threads, each with its own weight, activation and output, 20 calls each
    import threading
    from microkimi_amd._lib import hptr, lib
    from microkimi_amd import workloads
    rows, cols, nthreads = 256, 2048, 8
    mats = [workloads.mxfp4_matrix(0, "tw", rows, cols, t) for t in range(nthreads)]
    xs = [np.random.default_rng(t).standard_normal(cols).astype(np.float32) for t in range(nthreads)]
    want = [oracle.matvec_packed(mats[t][0], mats[t][1], rows, cols, xs[t], mode=1) for t in range(nthreads)]
    outs = [np.zeros(rows, np.float32) for _ in range(nthreads)]
    errs = []

    def work(t):
        for _ in range(20):
            st = lib.mk_mxfp4_matvec(hptr(mats[t][0]), hptr(mats[t][1]), rows, cols, hptr(xs[t]), hptr(outs[t]))
            if st != 0:
                errs.append((t, st))
                return
            if rel_l2(outs[t], want[t]) > 1e-5:
                errs.append((t, "wrong result"))
                return

    lib.mk_force_q8(1)
    try:
        th = [threading.Thread(target=work, args=(t,)) for t in range(nthreads)]
        for t in th:
            t.start()
        for t in th:
            t.join()
    finally:
        lib.mk_force_q8(-1)
    assert not errs, errs


def test_shared_latent_handle_assign_f32_and_prefill():
    # MlaCache::assign_f32 (src/model.rs:1680-1692) and the mla_prefill loop on the shared-latent handle
    torch_cuda()
    from microkimi_amd import _lib, workloads
    nh, L, R, n = 8, 512, 64, 70
    lat, rope, q = workloads.config3_raw(n, nh=nh)
    c = ctypes.c_void_p()
    _lib.check(_lib.lib.mk_mla_cache_new(nh, L, R, n, ctypes.byref(c)))
    try:
        _lib.check(_lib.lib.mk_mla_cache_push(c, _lib.hptr(lat[5]), _lib.hptr(rope[5])))   # stale: assign starts empty
        _lib.check(_lib.lib.mk_mla_cache_assign_f32(c, _lib.hptr(lat), _lib.hptr(rope), n))
        assert _lib.lib.mk_mla_cache_positions(c) == n
        lq, _, ls = oracle.q8_0_rows(lat)
        rq, _, rs = oracle.q8_0_rows(rope)
        qs = np.stack([q, q * 0.5, -q]).astype(np.float32)
        outs = np.zeros((3, nh, L), np.float32)
        _lib.check(_lib.lib.mk_mla_attn_prefill(c, _lib.hptr(qs), 3, workloads.MLA_SCALE, _lib.hptr(outs)))
        for i in range(3):
            want = oracle.mla_absorbed_decode(lq, ls.astype(np.float32), rq, rs.astype(np.float32), qs[i], nh, workloads.MLA_SCALE, pos=n - 3 + i)
            assert rel_l2(outs[i], want) <= 1e-5
    finally:
        _lib.lib.mk_mla_cache_free(c)
