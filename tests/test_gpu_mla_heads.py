"""GPU parity, q8_0 MLA attention over the cache layout the reference keeps (per-head K-nope and V rows, one f32 rope
row per position): append / assign_f32 / to_f32 bit for bit, decode and the prefill loop against the oracle's
MlaCache and mla_attn_flash_q8_mqa.  Tolerance for attention: relative L2 <= 1e-5."""
import ctypes as C

import numpy as np
import pytest

import oracle
from gpu_util import dev, rel_l2, torch_cuda

pytestmark = pytest.mark.gpu
TOL = 1e-5


def rows(n, nh, nope, rope, vd, seed):
    rng = np.random.default_rng(seed)
    k = rng.standard_normal((n, nh * (nope + rope))).astype(np.float32)
    v = rng.standard_normal((n, nh * vd)).astype(np.float32)
    return k, v


def oracle_cache(k, v, nh, nope, rope, vd):
    c = oracle.MlaCache(nh, nope, rope, vd, capacity=max(1, k.shape[0]))
    for j in range(k.shape[0]):
        c.push(k[j], v[j])
    return c


@pytest.mark.parametrize("n,nh,nope,rope,vd", [(1, 4, 128, 64, 128), (37, 6, 128, 64, 128), (70, 3, 64, 32, 96), (5, 2, 256, 64, 512)])
def test_push_assign_and_to_f32_are_the_reference_bytes(n, nh, nope, rope, vd):
    from microkimi_amd import model
    k, v = rows(n, nh, nope, rope, vd, n)
    k[0, :32] = 0.0                                       # a zero block
    if n > 2:
        k[2, :32] = 0.0
        k[2, 0], k[2, 1], k[2, 2], k[2, 3] = 127.0, 0.5, -2.5, np.float32(0.49999997)  # exact ties, just below a tie
    want = oracle_cache(k, v, nh, nope, rope, vd)
    one = model.MlaHeadsCache(nh, nope, rope, vd, n)
    for j in range(n):                                    # MlaCache::push, position by position
        one.push(dev(k[j]), dev(v[j]))
    bulk = model.MlaHeadsCache(nh, nope, rope, vd, n + 3)
    bulk.push(dev(k[:1] * 3.0), dev(v[:1]))               # stale contents: assign_f32 starts from an empty cache
    bulk.assign_f32(dev(k), dev(v))
    for c in (one, bulk):
        assert c.positions() == n
        assert np.array_equal(c.kq[:n].cpu().numpy(), want.kq[:n]) and np.array_equal(c.vq[:n].cpu().numpy(), want.vq[:n])
        assert np.array_equal(c.ks[:n].cpu().numpy().view(np.uint32), want.ks[:n].view(np.uint32))
        assert np.array_equal(c.vs[:n].cpu().numpy().view(np.uint32), want.vs[:n].view(np.uint32))
        assert np.array_equal(c.kr[:n].cpu().numpy().view(np.uint32), want.kr[:n].view(np.uint32))   # rope from head 0, f32, untouched
    kf, vf = one.to_f32()
    wk, wv = want.to_f32()
    assert np.array_equal(kf.cpu().numpy().view(np.uint32), wk.view(np.uint32))
    assert np.array_equal(vf.cpu().numpy().view(np.uint32), wv.view(np.uint32))


@pytest.mark.parametrize("n,nh,nope,rope,vd,qscale", [(1, 4, 128, 64, 128, 1.0), (7, 4, 128, 64, 128, 1.0), (64, 6, 128, 64, 128, 1.0),
                                                     (65, 6, 128, 64, 128, 1.0), (512, 6, 128, 64, 128, 1.0), (300, 5, 64, 32, 96, 3.0),
                                                     (4200, 24, 128, 64, 128, 1.0), (130, 2, 256, 64, 512, 0.0),
                                                     # the reference's head shape (128 + 64 / 128) takes the all-heads kernel, 8 heads a
                                                     # workgroup (the cases above with 4, 6 and 24 heads too; other shapes the
                                                     # per-head one): whole groups, a context split over the chip, zero query
                                                     (1, 8, 128, 64, 128, 1.0), (7, 8, 128, 64, 128, 1.0), (64, 16, 128, 64, 128, 1.0),
                                                     (65, 8, 128, 64, 128, 3.0), (512, 8, 128, 64, 128, 1.0), (2100, 96, 128, 64, 128, 1.0),
                                                     (200, 8, 128, 64, 128, 0.0)])
def test_decode_matches_mla_attn_flash_q8_mqa(n, nh, nope, rope, vd, qscale):
    # the lengths of src/selftest.rs:871-876 (1, 7, 64, 65, 512), a long context (split over the chip), odd shapes,
    # an all-zero query (uniform weights)
    from microkimi_amd import model
    k, v = rows(n, nh, nope, rope, vd, 100 + n)
    rng = np.random.default_rng(n)
    q = (rng.standard_normal(nh * (nope + rope)) * qscale).astype(np.float32)
    scale = float(np.float32(nope + rope) ** np.float32(-0.5))
    want_c = oracle_cache(k, v, nh, nope, rope, vd)
    c = model.MlaHeadsCache(nh, nope, rope, vd, n)
    c.push(dev(k), dev(v))
    for pos in sorted({n - 1, n // 2, 0}):
        got = c.attn(dev(q), pos, scale).cpu().numpy()[0]
        want = oracle.mla_attn_flash_q8_mqa(want_c, q, pos, scale)
        assert np.isfinite(got).all()
        assert rel_l2(got, want) <= TOL, (pos, rel_l2(got, want))


def test_decode_at_the_published_shape_16384_positions_96_heads():
    # the shape the reference's own figure is quoted on (96 heads, 128 + 64 / 128, 16k positions), at full size against the
    # oracle: the cache is filled in chunks of 2048 positions on both sides
    from microkimi_amd import model
    n, nh, nope, rope, vd = 16384, 96, 128, 64, 128
    rng = np.random.default_rng(16384)
    want_c = oracle.MlaCache(nh, nope, rope, vd, capacity=n)
    c = model.MlaHeadsCache(nh, nope, rope, vd, n)
    for j0 in range(0, n, 2048):
        k = rng.standard_normal((2048, nh * (nope + rope)), dtype=np.float32)
        v = rng.standard_normal((2048, nh * vd), dtype=np.float32)
        c.push(dev(k), dev(v))
        for j in range(2048):
            want_c.push(k[j], v[j])
    assert c.positions() == n == want_c.n
    assert np.array_equal(c.kq[n - 3:n].cpu().numpy(), want_c.kq[n - 3:n]) and np.array_equal(c.vq[n - 3:n].cpu().numpy(), want_c.vq[n - 3:n])
    q = rng.standard_normal(nh * (nope + rope), dtype=np.float32) * np.float32(2.0)   # scores a few units apart: not a flat softmax
    scale = float(np.float32(nope + rope) ** np.float32(-0.5))
    for pos in (n - 1, 9001):
        got = c.attn(dev(q), pos, scale).cpu().numpy()[0]
        want = oracle.mla_attn_flash_q8_mqa(want_c, q, pos, scale)
        assert np.isfinite(got).all()
        assert rel_l2(got, want) <= TOL, (pos, rel_l2(got, want))
        per_head = [rel_l2(got[h * vd:(h + 1) * vd], want[h * vd:(h + 1) * vd]) for h in range(nh)]
        assert max(per_head) <= TOL, (pos, int(np.argmax(per_head)), max(per_head))


@pytest.mark.parametrize("nh,n0,m,had", [(8, 300, 70, False), (3, 0, 40, False), (16, 1000, 16, True), (4, 17, 130, False)])
def test_prefill_on_the_matrix_cores(nh, n0, m, had):
    # 16 and more queries at the reference's head shape share the K / V tiles on the matrix cores: every query against
    # its own decode in the oracle (a prompt from position 0, a chunk behind a long context, a last group of queries
    # that is not full, the Hadamard option)
    from microkimi_amd import model
    nope, rope, vd = 128, 64, 128
    k, v = rows(n0 + m, nh, nope, rope, vd, 50 + m)
    rng = np.random.default_rng(m)
    q = rng.standard_normal((m, nh * (nope + rope))).astype(np.float32)
    scale = float(np.float32(nope + rope) ** np.float32(-0.5))
    want_c = oracle.MlaCache(nh, nope, rope, vd, had=had, capacity=n0 + m)
    for i in range(n0 + m):
        want_c.push(k[i], v[i])
    c = model.MlaHeadsCache(nh, nope, rope, vd, n0 + m, hadamard=had)
    c.push(dev(k), dev(v))
    got = c.attn(dev(q), n0, scale).cpu().numpy()
    assert np.isfinite(got).all()
    worst = max(rel_l2(got[i], oracle.mla_attn_flash_q8_mqa(want_c, q[i], n0 + i, scale)) for i in range(m))
    assert worst <= TOL, worst


@pytest.mark.parametrize("nh", [6, 8])
def test_prefill_loop_equals_one_decode_per_position(nh):
    # mla_prefill (src/model.rs:2080-2102): query i over the positions 0 ..= pos0 + i (6 heads: a partial group of the
    # all-heads kernel, 8: a whole one)
    from microkimi_amd import model
    nope, rope, vd, n0, m = 128, 64, 128, 40, 33
    k, v = rows(n0 + m, nh, nope, rope, vd, 5)
    rng = np.random.default_rng(6)
    q = rng.standard_normal((m, nh * (nope + rope))).astype(np.float32)
    scale = float(np.float32(nope + rope) ** np.float32(-0.5))
    want_c = oracle_cache(k, v, nh, nope, rope, vd)
    c = model.MlaHeadsCache(nh, nope, rope, vd, n0 + m)
    c.push(dev(k), dev(v))
    got = c.attn(dev(q), n0, scale).cpu().numpy()
    for i in range(m):
        want = oracle.mla_attn_flash_q8_mqa(want_c, q[i], n0 + i, scale)
        assert rel_l2(got[i], want) <= TOL, i


def test_host_level_handle_in_the_reference_layout():
    # mk_mla_cache_new_heads / push / assign_f32 / to_f32 / attn / attn_prefill on host slices
    torch_cuda()
    from microkimi_amd._lib import check, hptr, lib
    nh, nope, rope, vd, n = 5, 128, 64, 128, 90
    k, v = rows(n, nh, nope, rope, vd, 9)
    rng = np.random.default_rng(10)
    q = rng.standard_normal((4, nh * (nope + rope))).astype(np.float32)
    scale = float(np.float32(nope + rope) ** np.float32(-0.5))
    want_c = oracle_cache(k, v, nh, nope, rope, vd)
    h = C.c_void_p()
    check(lib.mk_mla_cache_new_heads(nh, nope, rope, vd, n, C.byref(h)))
    try:
        for j in range(10):
            check(lib.mk_mla_cache_push(h, hptr(k[j]), hptr(v[j])))
        assert lib.mk_mla_cache_positions(h) == 10
        out = np.empty(nh * vd, np.float32)
        check(lib.mk_mla_attn(h, hptr(q[0]), scale, hptr(out)))
        assert rel_l2(out, oracle.mla_attn_flash_q8_mqa(want_c, q[0], 9, scale)) <= TOL
        check(lib.mk_mla_cache_assign_f32(h, hptr(k), hptr(v), n))       # snapshot restore: all n positions
        assert lib.mk_mla_cache_positions(h) == n
        kf, vf = np.empty_like(k), np.empty_like(v)
        check(lib.mk_mla_cache_to_f32(h, hptr(kf), hptr(vf)))
        wk, wv = want_c.to_f32()
        assert np.array_equal(kf.view(np.uint32), wk.view(np.uint32)) and np.array_equal(vf.view(np.uint32), wv.view(np.uint32))
        outs = np.empty((4, nh * vd), np.float32)
        check(lib.mk_mla_attn_prefill(h, hptr(q), 4, scale, hptr(outs)))  # the last 4 positions as a prompt
        for i in range(4):
            assert rel_l2(outs[i], oracle.mla_attn_flash_q8_mqa(want_c, q[i], n - 4 + i, scale)) <= TOL
        q20 = rng.standard_normal((20, nh * (nope + rope))).astype(np.float32)
        outs = np.empty((20, nh * vd), np.float32)
        check(lib.mk_mla_attn_prefill(h, hptr(q20), 20, scale, hptr(outs)))  # 16 and more queries: the matrix-core kernel
        for i in range(20):
            assert rel_l2(outs[i], oracle.mla_attn_flash_q8_mqa(want_c, q20[i], n - 20 + i, scale)) <= TOL
        assert lib.mk_mla_cache_push(h, hptr(k[0]), hptr(v[0])) == -5   # full: MK_ERR_NOMEM
    finally:
        lib.mk_mla_cache_free(h)


def test_shapes_the_kernels_do_not_cover_are_refused():
    torch_cuda()
    from microkimi_amd._lib import lib
    h = C.c_void_p()
    assert lib.mk_mla_cache_new_heads(4, 100, 64, 128, 8, C.byref(h)) == -1    # nope not a multiple of 32
    assert lib.mk_mla_cache_new_heads(4, 128, 64, 1024, 8, C.byref(h)) == -1   # V rows wider than the kernel holds
    assert lib.mk_mla_cache_new(4, 512, 0, 8, C.byref(h)) == -1                # the shared-latent cache needs a rope row
    assert lib.mk_mla_cache_new(4, 96, 64, 8, C.byref(h)) == -1                # latent width the decode kernel rejects


@pytest.mark.parametrize("n,nh,nope,rope,vd,applies", [(37, 4, 128, 64, 128, True), (70, 3, 64, 32, 192, True), (300, 6, 128, 64, 128, True),
                                                     (20, 3, 96, 32, 128, False), (300, 8, 128, 64, 128, True)])
def test_hadamard_option(n, nh, nope, rope, vd, applies):
    # kv_hadamard (src/model.rs:1529-1554): rotated cache bytes, to_f32 and attention against the oracle in the same
    # mode; widths that are not whole 64-chunks leave the option without effect, as in the reference
    from microkimi_amd import model
    k, v = rows(n, nh, nope, rope, vd, 300 + n)
    k[0, :64] = 0.0
    rng = np.random.default_rng(n)
    q = rng.standard_normal(nh * (nope + rope)).astype(np.float32)
    scale = float(np.float32(nope + rope) ** np.float32(-0.5))
    want = oracle.MlaCache(nh, nope, rope, vd, had=True, capacity=n)
    for j in range(n):
        want.push(k[j], v[j])
    c = model.MlaHeadsCache(nh, nope, rope, vd, n, hadamard=True)
    c.push(dev(k), dev(v))
    assert np.array_equal(c.kq[:n].cpu().numpy(), want.kq[:n]) and np.array_equal(c.vq[:n].cpu().numpy(), want.vq[:n])
    assert np.array_equal(c.ks[:n].cpu().numpy().view(np.uint32), want.ks[:n].view(np.uint32))
    assert np.array_equal(c.vs[:n].cpu().numpy().view(np.uint32), want.vs[:n].view(np.uint32))
    plain = oracle_cache(k, v, nh, nope, rope, vd)
    assert np.array_equal(want.kq[:n], plain.kq[:n]) != applies      # the rotation changes the bytes exactly when it applies
    kf, vf = c.to_f32()
    wk, wv = want.to_f32()
    assert np.array_equal(kf.cpu().numpy().view(np.uint32), wk.view(np.uint32))
    assert np.array_equal(vf.cpu().numpy().view(np.uint32), wv.view(np.uint32))
    for pos in sorted({n - 1, n // 2}):
        got = c.attn(dev(q), pos, scale).cpu().numpy()[0]
        assert rel_l2(got, oracle.mla_attn_flash_q8_mqa(want, q, pos, scale)) <= TOL
    m = min(5, n)
    qs = rng.standard_normal((m, nh * (nope + rope))).astype(np.float32)
    got = c.attn(dev(qs), n - m, scale).cpu().numpy()
    for i in range(m):
        assert rel_l2(got[i], oracle.mla_attn_flash_q8_mqa(want, qs[i], n - m + i, scale)) <= TOL


def test_host_level_hadamard_switch():
    torch_cuda()
    from microkimi_amd._lib import check, hptr, lib
    nh, nope, rope, vd, n = 4, 128, 64, 128, 12
    k, v = rows(n, nh, nope, rope, vd, 11)
    want = oracle.MlaCache(nh, nope, rope, vd, had=True, capacity=n)
    for j in range(n):
        want.push(k[j], v[j])
    q = np.random.default_rng(12).standard_normal(nh * (nope + rope)).astype(np.float32)
    scale = float(np.float32(nope + rope) ** np.float32(-0.5))
    h = C.c_void_p()
    check(lib.mk_mla_cache_new_heads(nh, nope, rope, vd, n, C.byref(h)))
    try:
        check(lib.mk_mla_cache_set_hadamard(h, 1))
        check(lib.mk_mla_cache_assign_f32(h, hptr(k), hptr(v), n))
        assert lib.mk_mla_cache_set_hadamard(h, 0) == -1              # not while positions are held
        kf, vf = np.empty_like(k), np.empty_like(v)
        check(lib.mk_mla_cache_to_f32(h, hptr(kf), hptr(vf)))
        wk, wv = want.to_f32()
        assert np.array_equal(kf.view(np.uint32), wk.view(np.uint32)) and np.array_equal(vf.view(np.uint32), wv.view(np.uint32))
        out = np.empty(nh * vd, np.float32)
        check(lib.mk_mla_attn(h, hptr(q), scale, hptr(out)))
        assert rel_l2(out, oracle.mla_attn_flash_q8_mqa(want, q, n - 1, scale)) <= TOL
    finally:
        lib.mk_mla_cache_free(h)
