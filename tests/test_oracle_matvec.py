"""Pins matvec_packed (both modes), matvec_packed_nt and Q8Head (src/mxfp4.rs, src/model.rs)."""
import numpy as np
import pytest

import oracle
from test_oracle_codec import np_dequant
from test_oracle_q8 import brute_block_dot

SHAPES = [(128, 512), (512, 128), (64, 128), (3, 64), (1, 32), (256, 1024), (2048, 4096), (333, 1024)]  # src/selftest.rs:610-619


def make_case(rows, cols):
    w = oracle.pattern(0, rows * cols)
    p, s = oracle.mxfp4_quantize(w, rows, cols)
    x = oracle.pattern(4242, cols)
    return p, s, x


@pytest.mark.parametrize("rows,cols", SHAPES)
def test_f32_mode_matches_f64_closed_form(rows, cols):
    p, s, x = make_case(rows, cols)
    y = oracle.matvec_packed(p, s, rows, cols, x, mode=0)
    w = np_dequant(p, s, rows, cols).astype(np.float64)
    want = w @ x.astype(np.float64)
    scale = np.abs(w).dot(np.abs(x.astype(np.float64))).max()
    assert np.abs(y - want).max() <= 1e-6 * scale


def test_f32_mode_tiny_brute_force_in_reference_order():
    # 1x32 and 3x64 evaluated with explicit f32 steps: gsum over 32 in order, then sum += gsum * scale
    for rows, cols in [(1, 32), (3, 64)]:
        p, s, x = make_case(rows, cols)
        y = oracle.matvec_packed(p, s, rows, cols, x, mode=0)
        lut = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0], np.float32)
        for r in range(rows):
            tot = np.float32(0)
            for g in range(cols // 32):
                gs = np.float32(0)
                for j in range(32):
                    c = g * 32 + j
                    b = p[r, c // 2]
                    nib = (b & 15) if c % 2 == 0 else (b >> 4)
                    gs = np.float32(gs + np.float32(lut[nib] * x[c]))
                tot = np.float32(tot + np.float32(gs * np.float32(2.0 ** (int(s[r, g]) - 127))))
            assert tot.view(np.uint32) == np.float32(y[r]).view(np.uint32)


@pytest.mark.parametrize("rows,cols", SHAPES)
def test_q8_mode_formula_and_bound(rows, cols):
    p, s, x = make_case(rows, cols)
    xq, xs = oracle.quantize_q8(x)
    y = oracle.matvec_packed_q8(p, s, rows, cols, xq, xs)
    assert np.array_equal(y, oracle.matvec_packed(p, s, rows, cols, x, mode=1))
    # closed form in f64 of the same quantities: sum_g idot_g * 2^(sb-128) * dx_g
    lo, hi = (p & 0x0F).astype(np.int64), (p >> 4).astype(np.int64)
    lut2 = np.array([0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12], np.int64)
    w2 = np.empty((rows, cols), np.int64)
    w2[:, 0::2], w2[:, 1::2] = lut2[lo], lut2[hi]
    idot = (w2.reshape(rows, cols // 32, 32) * xq.astype(np.int64).reshape(1, cols // 32, 32)).sum(axis=2)
    coef = np.exp2(s.astype(np.float64) - 128.0) * xs.astype(np.float64)[None, :]
    want = (idot * coef).sum(axis=1)
    scale = (np.abs(idot) * coef).sum(axis=1).max()
    assert np.abs(y - want).max() <= 2e-6 * scale
    # src/selftest.rs:597-646: within 1e-3 of the exact f32 path, relative to the output scale
    yf = oracle.matvec_packed(p, s, rows, cols, x, mode=0)
    assert np.abs(y - yf).max() / max(np.abs(yf).max(), 1e-12) <= 1e-3


def test_q8_row_brute_force_small():
    rows, cols = 3, 64
    p, s, x = make_case(rows, cols)
    xq, xs = oracle.quantize_q8(x)
    y = oracle.matvec_packed_q8(p, s, rows, cols, xq, xs)
    for r in range(rows):
        tot = np.float32(0)
        for g in range(2):
            idot = brute_block_dot(p[r, g * 16:(g + 1) * 16], xq[g * 32:(g + 1) * 32])
            tot = np.float32(tot + np.float32(np.float32(idot) * np.float32(np.float32(2.0 ** (int(s[r, g]) - 128)) * xs[g])))
        assert tot.view(np.uint32) == np.float32(y[r]).view(np.uint32)


def test_zero_block_scale_byte_zero():
    # src/selftest.rs:561-569: an all-zero block gets scale byte 0 and contributes exactly 0
    rows, cols = 64, 128
    w = oracle.pattern(0, rows * cols)
    w[2 * cols:4 * cols] = 0
    p, s = oracle.mxfp4_quantize(w, rows, cols)
    assert np.all(s[2:4] == 0)
    x = oracle.pattern(4242, cols)
    for mode in (0, 1):
        y = oracle.matvec_packed(p, s, rows, cols, x, mode=mode)
        assert np.all(y[2:4] == 0)


@pytest.mark.parametrize("rows,cols", [(128, 512), (64, 128), (3, 64), (256, 1024)])
def test_shader_emul_within_1e3(rows, cols):
    # src/selftest.rs:534-595
    p, s, x = make_case(rows, cols)
    y = oracle.matvec_packed(p, s, rows, cols, x, mode=0)
    ye = oracle.matvec_packed_shader_emul(p, s, rows, cols, x, 256)
    assert np.abs(y - ye).max() / max(np.abs(y).max(), 1e-12) <= 1e-3


@pytest.mark.parametrize("rows,cols,m", [(64, 128, 8), (33, 64, 16), (128, 512, 24)])
def test_nt_bit_identical_to_f32_matvec(rows, cols, m):
    # src/model.rs:2403-2406
    p, s, _ = make_case(rows, cols)
    xs = oracle.pattern(99, cols * m).reshape(m, cols)
    xs[m - 3:] = 0  # zero-padded lanes
    out = oracle.matvec_packed_nt(p, s, rows, cols, np.ascontiguousarray(xs.T), m)
    for t in range(m):
        y = oracle.matvec_packed(p, s, rows, cols, xs[t], mode=0)
        assert np.array_equal(out[t].view(np.uint32), y.view(np.uint32))
    assert not out[m - 3:].any()


def test_q8head_matches_f32_reference_test():
    # src/model.rs:3866-3881 restated: 512x1024, seed 0xC0FFEE, err/span < 1e-2, same argmax
    rows, cols = 512, 1024
    rng = oracle.Rng(0xC0FFEE)
    w = rng.f32(rows * cols) * np.float32(0.02)
    x = rng.f32(cols)
    q, s = oracle.q8head_from_f32(w, rows, cols)
    got = oracle.q8head_matvec(q, s, rows, cols, x, workers=8)
    want = oracle.matvec_f32(w, rows, cols, x)
    span = np.abs(want).max()
    assert np.abs(got.astype(np.float64) - want).max() / span < 1e-2
    assert oracle.argmax(got) == oracle.argmax(want) == int(np.argmax(want))
    # any row partition gives identical rows
    for workers in (1, 2, 3, 7):
        assert np.array_equal(got, oracle.q8head_matvec(q, s, rows, cols, x, workers=workers))
    # f64 closed form of sum_g ws*xs*idot
    xq, xs = oracle.quantize_q8(x)
    idot = (q.astype(np.int64).reshape(rows, cols // 32, 32) * xq.astype(np.int64).reshape(1, -1, 32)).sum(axis=2)
    coef = s.astype(np.float64) * xs.astype(np.float64)[None, :]
    ref = (idot * coef).sum(axis=1)
    assert np.abs(got - ref).max() <= 2e-6 * (np.abs(idot) * coef).sum(axis=1).max()


def test_argmax_ties_lowest_index():
    assert oracle.argmax(np.array([1, 3, 3, 2], np.float32)) == 1


@pytest.mark.parametrize("rows,cols", [(64, 128), (9, 1024), (5, 2048), (6, 4096), (7, 7168), (3, 96)])
def test_device_order_emulation_bounds_the_gap_without_a_device(rows, cols):
    # the association of a row's f32 sum as the library's MXFP4 GEMV kernel has it (the role matvec_packed_shader_emul,
    # src/selftest.rs:534-595, plays for the Metal kernel): the same terms, another order -- a few ulp of the row's norm
    p, s, x = make_case(rows, cols)
    xq, xs = oracle.quantize_q8(x)
    ref = oracle.matvec_packed_q8(p, s, rows, cols, xq, xs)
    emu = oracle.matvec_packed_q8_device_order(p, s, rows, cols, xq, xs)
    assert np.linalg.norm(ref.astype(np.float64) - emu) <= 2e-6 * np.linalg.norm(ref)
    # one block per row: a single term, no association to differ in -> the same bits
    if cols >= 64:
        x1 = x.copy()
        x1[32:] = 0.0
        xq1, xs1 = oracle.quantize_q8(x1)
        a = oracle.matvec_packed_q8(p, s, rows, cols, xq1, xs1)
        b = oracle.matvec_packed_q8_device_order(p, s, rows, cols, xq1, xs1)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_q8head_device_order_emulation():
    rng = np.random.default_rng(3)
    rows, cols = 12, 7168
    q = rng.integers(-127, 128, (rows, cols), dtype=np.int8)
    ws = (np.abs(rng.standard_normal((rows, cols // 32))) * 0.02 / 127).astype(np.float32)
    x = rng.standard_normal(cols).astype(np.float32)
    xq, xs = oracle.quantize_q8(x)
    ref = oracle.q8head_matvec(q, ws, rows, cols, x)
    emu = oracle.q8head_matvec_device_order(q, ws, rows, cols, xq, xs)
    assert np.linalg.norm(ref.astype(np.float64) - emu) <= 2e-6 * np.linalg.norm(ref)
    # the first 16 values of the activation only: one half block per row, one term -> the same bits as the reference order
    x1 = np.zeros(cols, np.float32)
    x1[:16] = x[:16]
    xq1, xs1 = oracle.quantize_q8(x1)
    a = oracle.q8head_matvec(q, ws, rows, cols, x1)
    b = oracle.q8head_matvec_device_order(q, ws, rows, cols, xq1, xs1)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
