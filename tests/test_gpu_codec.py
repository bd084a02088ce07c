"""GPU parity, codec kernels: bit-exact against the oracle."""
import json
import os

import numpy as np
import pytest

import oracle
from gpu_util import dev, torch_cuda

pytestmark = pytest.mark.gpu
G = os.path.join(os.path.dirname(__file__), "golden")


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def test_mxfp4_dequant_golden_and_exhaustive():
    from microkimi_amd import mxfp4
    g = json.load(open(os.path.join(G, "ds_golden_fp4.json")))
    p, s = np.asarray(g["packed"], np.uint8), np.asarray(g["scales"], np.uint8)
    w = mxfp4.dequant(dev(p), dev(s), g["rows"], g["cols"]).cpu().numpy()
    assert np.array_equal(bits(w), bits(oracle.mxfp4_dequant(p, s, g["rows"], g["cols"])))
    # every nibble x every scale byte 0..254 (255 is NaN in e8m0 and unused), sign of -0.0 included
    rows = 255
    p = np.tile(np.array([n | (n << 4) for n in range(16)], np.uint8), (rows, 1))
    s = np.arange(rows, dtype=np.uint8).reshape(rows, 1)
    w = mxfp4.dequant(dev(p), dev(s), rows, 32).cpu().numpy()
    assert np.array_equal(bits(w), bits(oracle.mxfp4_dequant(p, s, rows, 32)))
    # host-level entry point (numpy in, numpy out)
    w2 = mxfp4.dequant(p, s, rows, 32)
    assert np.array_equal(bits(w2), bits(w))


def test_mxfp4_dequant_config_shape():
    from microkimi_amd import mxfp4, workloads
    p, s, _ = workloads.config0()
    w = mxfp4.dequant(dev(p), dev(s), 2048, 7168).cpu().numpy()
    assert np.array_equal(bits(w), bits(oracle.mxfp4_dequant(p, s, 2048, 7168)))


def test_fp8_dequant_golden():
    from microkimi_amd import dequant
    g = np.load(os.path.join(G, "ds_golden_fp8.npz"))
    rows, cols = int(g["rows"]), int(g["cols"])
    w = dequant.dequant_fp8(dev(g["w_packed"]), dev(g["scales"]), rows, cols).cpu().numpy()
    assert np.array_equal(bits(w.reshape(-1)), bits(g["dequant"]))
    # all 256 codes, NaN codes included (compare as bits of the oracle's value, NaN == NaN)
    codes = np.tile(np.arange(256, dtype=np.uint8), (128, 1))
    sc = np.array([[120, 131]], np.uint8)
    w = dequant.dequant_fp8(dev(codes), dev(sc), 128, 256).cpu().numpy()
    want = oracle.dequant_fp8(codes, sc, 128, 256)
    assert np.array_equal(np.isnan(w), np.isnan(want))
    assert np.array_equal(bits(w)[~np.isnan(want)], bits(want)[~np.isnan(want)])


def test_quantize_q8_bit_exact():
    from microkimi_amd import q8
    rng = np.random.default_rng(0)
    x = rng.standard_normal((16, 7168)).astype(np.float32)
    x[1, :64] = 0.0                      # zero blocks
    x[2, :32] = np.float32(1e-30)        # tiny block
    x[3, 0:5] = [127.0, 0.5, -0.5, 1.5, 2.5]
    x[3, 5:32] = 0.25                    # scale exactly 1: ties round away from zero
    x[4] *= 1e4
    v = q8.quantize_q8(dev(x))
    q, s = v.q.cpu().numpy(), v.scales.cpu().numpy()
    for r in range(16):
        qo, so = oracle.quantize_q8(x[r])
        assert np.array_equal(q[r], qo), r
        assert np.array_equal(bits(s[r]), bits(so)), r
    # values on and next to rounding ties: block maximum 127 makes the scale exactly 1, so k + 0.5 is a tie and its
    # float neighbours are not; other maxima put quotients within an ulp of a tie
    n = 4096
    y = np.zeros((n, 32), dtype=np.float32)
    k = rng.integers(0, 126, size=(n, 31)).astype(np.float32) + 0.5
    step = rng.integers(-2, 3, size=(n, 31))
    near = k.copy()
    for _ in range(2):
        near = np.where(step > 0, np.nextafter(near, np.float32(200)), np.where(step < 0, np.nextafter(near, np.float32(-200)), near))
        step = step - np.sign(step)
    y[:, 1:] = near * rng.choice([-1.0, 1.0], size=(n, 31)).astype(np.float32)
    y[:, 0] = 127.0
    y[n // 2:] *= rng.uniform(0.01, 100.0, size=(n - n // 2, 1)).astype(np.float32)   # scales that are not a power of two
    vt = q8.quantize_q8(dev(y.reshape(1, -1)))
    qo, so = oracle.quantize_q8(y.reshape(-1))
    assert np.array_equal(vt.q.cpu().numpy().reshape(-1), qo)
    assert np.array_equal(bits(vt.scales.cpu().numpy().reshape(-1)), bits(so))
    # NaN and inf: the maximum skips a NaN, a NaN quotient (a NaN value, inf / inf) gives 0 as the reference's cast does
    z = rng.standard_normal((4, 64)).astype(np.float32)
    z[0, 3] = np.nan
    z[1, 7] = np.inf
    z[1, 9] = -np.inf
    z[2, :32] = np.nan
    z[3, 33] = np.nan
    z[3, 40] = np.inf
    vz = q8.quantize_q8(dev(z))
    for r in range(4):
        qo, so = oracle.quantize_q8(z[r])
        assert np.array_equal(vz.q.cpu().numpy()[r], qo), r
        assert np.array_equal(bits(vz.scales.cpu().numpy()[r]), bits(so)), r
    # host-level entry point
    hv = q8.quantize_q8(x[0])
    assert np.array_equal(hv.q, q[0]) and np.array_equal(hv.scales, s[0])


def test_quantize_mxfp8_bit_exact():
    from microkimi_amd import dequant
    rng = np.random.default_rng(1)
    x = (rng.standard_normal((8, 2048)) * np.array([1e-3, 0.1, 1, 3, 30, 300, 1e4, 1])[:, None]).astype(np.float32)
    x[7, :64] = 0.0
    x[7, 64:96] = np.float32(448.0)  # amax / 448 is an exact power of two
    x[7, 96:128] = np.float32(0.875)
    # mk_dev_quantize_mxfp8 keeps the reference's clamp of the scale exponent at 8 (src/deepseek.rs:316): a block above
    # 448 * 2^8 gets byte 8 + 127 and its large values saturate at code 0x7E / 0xFE
    x[7, 128:160] = np.linspace(-4.0e5, 4.0e5, 32, dtype=np.float32)
    x[7, 160:192] = np.float32(448.0 * 256.0)   # exactly at the limit: exponent 8, no saturation
    x[7, 192:224] = np.float32(448.0 * 256.0 * 1.001)
    # every e4m3 value, every midpoint between neighbours (ties) and their float neighbours, in blocks whose scale
    # is 1 (a 448 in each block) and in blocks scaled by 2^-3
    grid = np.array([oracle.e4m3_to_f32(c) for c in range(0x7F)], np.float32)  # 0 .. 448 ascending
    mids = ((grid[:-1].astype(np.float64) + grid[1:].astype(np.float64)) / 2).astype(np.float32)
    pts = np.concatenate([grid, mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(1e9))]).astype(np.float32)
    pts = np.concatenate([pts, -pts])
    rows = []
    for k in range(0, len(pts), 31):
        blk = np.zeros(32, np.float32)
        blk[0] = 448.0
        blk[1:1 + len(pts[k:k + 31])] = pts[k:k + 31]
        rows.append(blk)
    ties = np.concatenate(rows)
    ties = np.concatenate([ties, ties * np.float32(0.125)])
    pad = (-len(ties)) % 2048
    ties = np.concatenate([ties, np.zeros(pad, np.float32)]).reshape(-1, 2048)
    x = np.concatenate([x, ties]).astype(np.float32)
    codes, exps = dequant.quantize_mxfp8(dev(x))
    codes, exps = codes.cpu().numpy(), exps.cpu().numpy()
    for r in range(x.shape[0]):
        _, c, e = oracle.fp8_roundtrip(x[r], 32)
        assert np.array_equal(exps[r], e), r
        assert np.array_equal(codes[r], c), r
    assert exps[7, 4] == exps[7, 5] == exps[7, 6] == 8 + 127
    assert (codes[7, 128:138] == 0xFE).all() and (codes[7, 150:160] == 0x7E).all() and (codes[7, 160:224] == 0x7E).all()


def _quantizer_inputs(rows, cols, seed):
    rng = np.random.default_rng(seed)
    w = rng.standard_normal((rows, cols)).astype(np.float32)
    w *= np.exp2(rng.integers(-20, 20, size=(rows, cols // 32)).astype(np.float32)).repeat(32, axis=1)  # group scales all over
    w[0, :32] = 0.0                                              # a zero group: scale byte 0, all nibbles 0
    w[0, 32:64] = -0.0
    w[1, :32] = 0.0
    w[1, 0] = 6.0                                                # maxabs / 6 an exact power of two
    w[1, 1:8] = [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0]          # every midpoint: the upper level
    w[1, 8:15] = [-0.25, -0.75, -1.25, -1.75, -2.5, -3.5, -5.0]
    w[1, 15] = np.float32(0.24999999)
    w[2, :32] = np.float32(6.0000005)                            # just above a power of two: the logarithm rounds down
    w[2, 32:64] = np.float32(1e-41)                              # maxabs / 6 subnormal
    w[3, :32] = np.float32(3e38)                                 # the largest exponents
    w[3, 32:64] = np.float32(2.0 ** -126)
    w[4, :32] = np.linspace(-7, 7, 32, dtype=np.float32)         # clamps at +-6
    return w


@pytest.mark.parametrize("search", [True, False])
def test_mxfp4_quantize_gives_the_reference_bytes(search):
    # mxfp4::quantize / quantize_naive (src/mxfp4.rs:38-138)
    from microkimi_amd import mxfp4
    rows, cols = 48, 256
    w = _quantizer_inputs(rows, cols, 21)
    wp, ws = oracle.mxfp4_quantize(w, rows, cols, search=search)
    gp, gs = mxfp4.quantize(dev(w), search=search)
    assert np.array_equal(gs.cpu().numpy(), ws)
    assert np.array_equal(gp.cpu().numpy(), wp)
    if search:  # the search moves some scales (else this case tests nothing beyond the naive one)
        assert (ws != oracle.mxfp4_quantize(w, rows, cols, search=False)[1]).any()
    # round trip through the device decoder (the rows of random values): inside the clamp the error is at most half the
    # widest level step, 2^e
    back = mxfp4.dequant(gp, gs, rows, cols).cpu().numpy()[5:]
    step = np.exp2(gs.cpu().numpy()[5:].astype(np.float64) - 127.0).repeat(32, axis=1)
    inside = np.abs(w[5:]) <= 6.0 * step
    assert inside.mean() > 0.9 and np.all(np.abs(back.astype(np.float64) - w[5:])[inside] <= step[inside])


def test_quantize_fp8_gives_the_reference_bytes():
    # dequant::quantize_fp8 (src/dequant.rs:50-74)
    from microkimi_amd import dequant
    rows, cols = 256, 384
    rng = np.random.default_rng(22)
    w = rng.standard_normal((rows, cols)).astype(np.float32)
    w[:128, :128] = 0.0                                          # a zero block: exponent byte 0
    w[:128, 128:256] *= np.float32(1e6)                          # clamp of the exponent at 8: codes saturate at 448
    w[128:, :128] *= np.float32(1e-30)
    w[128, 128] = 448.0                                          # block maximum / 448 an exact power of two
    w[128:, 128:256] = np.clip(w[128:, 128:256], -400, 400)
    w[128, 128] = 448.0
    wq, wsc = oracle.quantize_fp8(w, rows, cols)
    gq, gsc = dequant.quantize_fp8(dev(w))
    assert np.array_equal(gsc.cpu().numpy(), wsc)
    assert np.array_equal(gq.cpu().numpy(), wq)
    assert wsc[0, 0] == 0 and wsc[0, 1] == 135 and wsc[1, 1] == 127


def test_mxfp4sq_quantize_and_dequant_give_the_reference_bytes():
    # mxfp4::quantize_sq / dequant_sq / dequant_any (src/mxfp4.rs:140-240)
    from microkimi_amd import mxfp4
    rows, cols = 48, 256
    w = _quantizer_inputs(rows, cols, 23)
    w[3, :32] = np.float32(3e30)   # (keeps smax finite enough for the small groups to be distinct)
    wp, ws, wsmax = oracle.mxfp4sq_quantize(w, rows, cols)
    gp, gs, gsmax = mxfp4.quantize_sq(dev(w))
    assert np.float32(gsmax.cpu().numpy()[0]) == wsmax
    assert np.array_equal(gs.cpu().numpy(), ws) and np.array_equal(gp.cpu().numpy(), wp)
    want = oracle.mxfp4sq_dequant(wp, ws, wsmax, rows, cols)
    got = mxfp4.dequant_sq(gp, gs, gsmax, rows, cols).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    blob = np.concatenate([wp.reshape(-1), ws.reshape(-1), np.array([wsmax], np.float32).view(np.uint8)])   # a dtype-4 blob
    got2 = mxfp4.dequant_any(4, dev(blob), rows, cols).cpu().numpy()
    assert np.array_equal(got2.view(np.uint32), want.view(np.uint32))
    # moderate magnitudes too (the case above is dominated by one huge group)
    w2 = _quantizer_inputs(rows, cols, 24)[5:]
    p2, s2, m2 = oracle.mxfp4sq_quantize(w2, rows - 5, cols)
    g2 = mxfp4.quantize_sq(dev(w2))
    assert np.array_equal(g2[0].cpu().numpy(), p2) and np.array_equal(g2[1].cpu().numpy(), s2) and np.float32(g2[2].cpu().numpy()[0]) == m2
    # an all-zero tensor: smax 0, scale 0, and 0 * (1 / 0) is a NaN whose sign bit decides the nibble (8 where the
    # default NaN is negative, as on x86 and here; 0 elsewhere): bytes and smax as the oracle on this host has them
    z = mxfp4.quantize_sq(dev(np.zeros((2, 64), np.float32)))
    zp, zs, zm = oracle.mxfp4sq_quantize(np.zeros((2, 64), np.float32), 2, 64)
    assert not z[1].any() and float(z[2]) == 0.0 and zm == 0.0
    assert set(np.unique(z[0].cpu().numpy())) <= {0x00, 0x88}
