"""Oracle pins for the VQ1 matvec (src/quant.rs:313-346) and the LUT GEMV (src/lutgemv.rs:208-240).

The reference's own test (src/lutgemv.rs:351-370) requires the two paths to agree bit for bit on six shapes; codebook
training and index assignment (train_codebook, quantize) are offline steps outside the path, so the codebook and the
indices are drawn directly (the reference's splitmix filler for values, uniform bytes for indices).
"""
import numpy as np
import pytest

import oracle

M64 = (1 << 64) - 1


class Rng:  # src/lutgemv.rs:246-256
    def __init__(self, seed):
        self.s = seed

    def f32(self):
        self.s = (self.s + 0x9E3779B97F4A7C15) & M64
        z = self.s
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M64
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M64
        return np.float32((z ^ (z >> 31)) / float(M64) - 0.5)


def case(rows, cols, rng):
    cb = np.array([rng.f32() * np.float32(0.05) for _ in range(256 * 16)], np.float32).reshape(256, 16)
    x = np.array([rng.f32() for _ in range(cols)], np.float32)
    idx = np.random.default_rng(rows * 7 + cols).integers(0, 256, (rows, cols // 16), dtype=np.uint8)
    return cb, idx, x


SHAPES = [(1, 16), (7, 64), (64, 128), (128, 64), (512, 1408), (1408, 512)]   # src/lutgemv.rs:354


def test_lut_path_is_bit_identical_to_gather():
    rng = Rng(0xC01D00155EED0001)
    for rows, cols in SHAPES:
        cb, idx, x = case(rows, cols, rng)
        a = oracle.vq1_matvec(cb, idx, rows, cols, x, lut=False)
        b = oracle.vq1_matvec(cb, idx, rows, cols, x, lut=True)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (rows, cols)


def test_closed_form_and_explicit_replay():
    rng = Rng(5)
    cb, idx, x = case(64, 256, rng)
    got = oracle.vq1_matvec(cb, idx, 64, 256, x)
    w = cb[idx].reshape(64, 256)                      # dequantized rows
    want = w.astype(np.float64) @ x.astype(np.float64)
    assert np.max(np.abs(got - want)) <= 1e-5 * np.max(np.abs(want))
    # explicit f32 replay of one row: per-vector dot from 0 in ascending j, vectors added in order
    r = 13
    s = np.float32(0)
    for v in range(16):
        t = np.float32(0)
        for j in range(16):
            t = np.float32(t + np.float32(w[r, v * 16 + j] * x[v * 16 + j]))
        s = np.float32(s + t)
    assert got[r].view(np.uint32) == s.view(np.uint32)
    # a one-hot activation picks single codebook values: out[r] = codebook[idx[r][v]][j] * x[c] exactly
    x1 = np.zeros(256, np.float32)
    x1[37] = 2.0
    one = oracle.vq1_matvec(cb, idx, 64, 256, x1)
    assert np.array_equal(one, cb[idx[:, 2], 5] * np.float32(2.0))


def nt_case(rows, cols, m, seed):
    cb, idx, _ = case(rows, cols, Rng(seed))
    xt = np.random.default_rng(seed).standard_normal((cols, m)).astype(np.float32)
    return cb, idx, xt


def test_batched_form_closed_form_and_explicit_replay():
    """matvec_vq_nt (src/quant.rs:353-376): one running sum per (row, position) over all cols products, in (vector, j) order."""
    rows, cols, m = 24, 96, 16
    cb, idx, xt = nt_case(rows, cols, m, 11)
    got = oracle.vq1_matvec_nt(cb, idx, rows, cols, xt, m)
    assert got.shape == (m, rows)
    w = cb[idx].reshape(rows, cols)
    want = (w.astype(np.float64) @ xt.astype(np.float64)).T
    assert np.max(np.abs(got - want)) <= 1e-5 * np.max(np.abs(want))
    # explicit f32 replay of a few (row, position) pairs: a single chain over the columns, multiply then add
    for r, p in ((0, 0), (5, 9), (23, 15)):
        s = np.float32(0)
        for c in range(cols):
            s = np.float32(s + np.float32(w[r, c] * xt[c, p]))
        assert got[p, r].view(np.uint32) == s.view(np.uint32)
    # the chain is not the per-vector sum of matvec_vq: same value to rounding, position by position
    for p in (0, 7, 8):
        one = oracle.vq1_matvec(cb, idx, rows, cols, np.ascontiguousarray(xt[:, p]))
        assert np.max(np.abs(one - got[p])) <= 1e-5 * np.max(np.abs(one))
    # a one-hot column of xt picks single codebook values, for its position only
    x1 = np.zeros((cols, 8), np.float32)
    x1[37, 3] = 2.0
    o = oracle.vq1_matvec_nt(cb, idx, rows, cols, x1, 8)
    assert np.array_equal(o[3], cb[idx[:, 2], 5] * np.float32(2.0))
    assert not o[[0, 1, 2, 4, 5, 6, 7]].any()
