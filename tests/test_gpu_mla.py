"""GPU parity, q8_0 MLA decode attention over the shared-latent cache against the oracle's
mla_attn_flash_q8_mqa.  Tolerance: relative L2 <= 1e-5."""
import numpy as np
import pytest

import oracle
from gpu_util import dev, rel_l2, torch_cuda

pytestmark = pytest.mark.gpu
TOL = 1e-5


def make_cache(ctx, L, R, nh, seed):
    from microkimi_amd import workloads
    rng = np.random.default_rng(seed)
    lat = rng.standard_normal((ctx, L)).astype(np.float32)
    rope = rng.standard_normal((ctx, R)).astype(np.float32)
    q = rng.standard_normal((nh, L + R)).astype(np.float32)
    lq, ls = workloads.q8_0_rows(lat)
    rq, rs = workloads.q8_0_rows(rope)
    return lat, rope, q, lq, ls, rq, rs


@pytest.mark.parametrize("ctx,L,R,nh", [(1, 128, 64, 6), (7, 128, 64, 6), (64, 128, 64, 6), (65, 128, 64, 6), (512, 128, 64, 6),
                                        (300, 512, 64, 20), (1000, 256, 32, 16)])
def test_small_shapes(ctx, L, R, nh):
    from microkimi_amd import model
    lat, rope, q, lq, ls, rq, rs = make_cache(ctx, L, R, nh, ctx)
    cache = model.MlaCache(L, R, ctx)
    cache.assign_q8(dev(lq), dev(ls), dev(rq), dev(rs))
    scale = float(np.float32(L // 4 + R) ** np.float32(-0.5))
    got = model.mla_attn_flash_q8_mqa(cache, dev(q), ctx - 1, scale).cpu().numpy()
    want = oracle.mla_absorbed_decode(lq, ls.astype(np.float32), rq, rs.astype(np.float32), q, nh, scale)
    assert rel_l2(got, want) <= TOL
    if ctx > 10:  # a shorter window over the same cache
        got = model.mla_attn_flash_q8_mqa(cache, dev(q), ctx // 2, scale).cpu().numpy()
        want = oracle.mla_absorbed_decode(lq, ls.astype(np.float32), rq, rs.astype(np.float32), q, nh, scale, pos=ctx // 2)
        assert rel_l2(got, want) <= TOL


@pytest.mark.parametrize("ctx,nh,qscale", [(1, 16, 1.0), (3, 5, 1.0), (17, 20, 1.0), (64, 16, 1.0), (65, 33, 1.0), (130, 128, 1.0),
                                            (700, 16, 6.0), (2048, 48, 6.0), (4100, 7, 0.0)])
def test_production_shape_matrix_core_kernel(ctx, nh, qscale):
    # latent 512 + rope 64 takes the MFMA kernel: single split and several, partial tiles and head groups,
    # queries scaled up so that scores spread over far more than the lazy-rescale threshold, and an all-zero
    # query (uniform weights)
    from microkimi_amd import model
    L, R = 512, 64
    lat, rope, q, lq, ls, rq, rs = make_cache(ctx, L, R, nh, 1000 + ctx)
    q = (q * qscale).astype(np.float32)
    cache = model.MlaCache(L, R, ctx)
    cache.assign_q8(dev(lq), dev(ls), dev(rq), dev(rs))
    scale = float(np.float32(L // 4 + R) ** np.float32(-0.5))
    for pos in sorted({ctx - 1, ctx // 2, 0}):
        got = model.mla_attn_flash_q8_mqa(cache, dev(q), pos, scale).cpu().numpy()
        want = oracle.mla_absorbed_decode(lq, ls.astype(np.float32), rq, rs.astype(np.float32), q, nh, scale, pos=pos)
        assert np.all(np.isfinite(got))
        assert rel_l2(got, want) <= TOL


def test_append_quantizes_like_the_reference():
    # MlaCache::push (src/model.rs:1583-1618) against the oracle's quantize_q8 (src/q8.rs:49-69), the f32 block scale
    # then stored as f16; with a zero block, exact ties (round half away), a value just below a tie and tiny values
    torch = torch_cuda()
    from microkimi_amd import model
    L, R, n = 512, 64, 40
    lat, rope, q, _, _, _, _ = make_cache(n, L, R, 4, 77)
    lat[3, :32] = 0.0
    lat[5, :32] = 0.0
    lat[5, 0], lat[5, 1], lat[5, 2], lat[5, 3], lat[5, 4], lat[5, 5] = 127.0, 0.5, -0.5, 2.5, np.float32(0.49999997), -126.5
    rope[6, :32] = 0.0
    rope[6, 0], rope[6, 1], rope[6, 2] = -127.0, 1.5, np.float32(-0.49999997)
    lat[7, 32:64] *= np.float32(1e-30)
    lq, _, ls = oracle.q8_0_rows(lat)
    rq, _, rs = oracle.q8_0_rows(rope)
    assert list(lq[5, :6]) == [127, 1, -1, 3, 0, -127] and list(rq[6, :3]) == [-127, 2, 0]
    cache = model.MlaCache(L, R, n)
    for j in range(n):
        cache.push(dev(lat[j]), dev(rope[j]))
    assert cache.positions() == n
    assert np.array_equal(cache.lat_q.cpu().numpy(), lq) and np.array_equal(cache.rope_q.cpu().numpy(), rq)
    assert np.array_equal(cache.lat_s.cpu().numpy().view(np.uint16), ls.view(np.uint16))
    assert np.array_equal(cache.rope_s.cpu().numpy().view(np.uint16), rs.view(np.uint16))
    # round trip within the q8_0 bound dx/2 (+ the f16 rounding of the scale: relative 2^-11, and absolute half a
    # subnormal step 2^-25 per unit of q for the block whose scale lies below the f16 range), src/selftest.rs:790-841
    lat2, rope2 = cache.to_f32()
    bound = np.abs(lat.reshape(n, L // 32, 32)).max(axis=2, keepdims=True) / 254.0
    err = np.abs(lat2.cpu().numpy().reshape(n, L // 32, 32) - lat.reshape(n, L // 32, 32))
    assert np.all(err <= bound * 1.02 + np.abs(lat.reshape(n, L // 32, 32)) * 2.0 ** -11 + 127 * 2.0 ** -25)


@pytest.mark.parametrize("ctx", [1024, 4096, 16384])
def test_benchmark_shapes(ctx):
    # configuration 3: 128 heads, latent 512 + rope 64, scale 1/sqrt(192)
    from microkimi_amd import model, workloads
    lat, rope, q = workloads.config3_raw(ctx)
    lq, ls = workloads.q8_0_rows(lat)
    rq, rs = workloads.q8_0_rows(rope)
    cache = model.MlaCache(workloads.MLA_LATENT, workloads.MLA_ROPE, ctx)
    cache.assign_q8(dev(lq), dev(ls), dev(rq), dev(rs))
    got = model.mla_attn_flash_q8_mqa(cache, dev(q), ctx - 1, workloads.MLA_SCALE).cpu().numpy()
    want = oracle.mla_absorbed_decode(lq, ls.astype(np.float32), rq, rs.astype(np.float32), q, workloads.MLA_HEADS, workloads.MLA_SCALE)
    assert rel_l2(got, want) <= TOL
    # softmax-weighted averages of the cache rows stay inside the rows' range (size-independent property)
    v = lq.astype(np.float32) * np.repeat(ls.astype(np.float32), 32, axis=1)
    assert np.all(got <= v.max(axis=0) + 1e-4) and np.all(got >= v.min(axis=0) - 1e-4)
