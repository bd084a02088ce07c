"""Pins quantize_q8, block_dot and block_dot_i8 (src/q8.rs)."""
import numpy as np

import oracle

LUT2 = np.array([0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12], np.int64)


def brute_block_dot(packed16, x32):
    lo, hi = packed16 & 0x0F, packed16 >> 4
    w = np.empty(32, np.int64)
    w[0::2], w[1::2] = LUT2[lo], LUT2[hi]
    return int((w * x32.astype(np.int64)).sum())


def test_quantize_conventions():
    # src/q8.rs:321-334
    x = np.zeros(64, np.float32)
    x[3], x[40] = 12.7, -3.3
    q, s = oracle.quantize_q8(x)
    assert s[0] == np.float32(12.7) / np.float32(127.0)
    assert s[1] == np.float32(3.3) / np.float32(127.0)
    assert q[3] == 127 and q[40] == -127
    assert q.min() >= -127
    q, s = oracle.quantize_q8(np.zeros(32, np.float32))
    assert s[0] == 0.0 and not q.any()


def test_quantize_bound_and_ties():
    rng = np.random.default_rng(3)
    x = rng.standard_normal(4096).astype(np.float32)
    q, s = oracle.quantize_q8(x)
    assert np.abs(q.astype(np.int32)).max() <= 127
    dx = np.repeat(s, 32)
    assert np.all(np.abs(x - q * dx) <= dx * 0.5 * (1 + 1e-6))
    # each block's largest magnitude maps to +-127
    assert np.all(np.abs(q.reshape(-1, 32)).max(axis=1) == 127)
    # round half away from zero: with max 127 the step is exactly 1
    x = np.zeros(32, np.float32)
    x[0], x[1], x[2], x[3], x[4] = 127.0, 0.5, -0.5, 1.5, 2.5
    q, s = oracle.quantize_q8(x)
    assert s[0] == 1.0 and list(q[:5]) == [127, 1, -1, 2, 3]


def test_quantize_just_below_a_tie_rounds_down():
    # roundf, not floor(|r| + 0.5) in f32: 0.49999997 + 0.5 rounds to 1.0 in f32, roundf(0.49999997) is 0
    x = np.zeros(32, np.float32)
    x[0], x[1], x[2] = 127.0, np.float32(0.49999997), np.float32(-0.49999997)
    q, s = oracle.quantize_q8(x)
    assert s[0] == 1.0 and list(q[:3]) == [127, 0, 0]


def test_workloads_q8_0_rows_equals_the_oracle():
    # the benchmark's cache builder (numpy) against quantize_q8, including ties and the case above
    from microkimi_amd import workloads
    rng = np.random.default_rng(11)
    x = rng.standard_normal((50, 576)).astype(np.float32)
    x[0, :32] = 0.0
    x[1, :32] = 0.0
    x[1, 0], x[1, 1], x[1, 2], x[1, 3], x[1, 4] = 127.0, 0.5, -1.5, np.float32(0.49999997), 126.5
    x[2, 32:64] = np.float32(1e-30)
    q, s16 = workloads.q8_0_rows(x)
    oq, os32, os16 = oracle.q8_0_rows(x)
    assert np.array_equal(q, oq)
    assert np.array_equal(s16.view(np.uint16), os16.view(np.uint16))
    assert list(q[1, :5]) == [127, 1, -2, 0, 127]


def test_block_dot_matches_brute_force_on_reference_stream():
    # src/q8.rs:283-296: seed 0xDEADBEEF, 2000 cases, x = (u8 % 255) as i8
    for scalar in (0, 1):
        oracle.force_scalar(scalar)
        rng = oracle.Rng(0xDEADBEEF)
        for _ in range(2000):
            packed = rng.u8(16)
            x = (rng.u8(32) % 255).astype(np.uint8).view(np.int8)
            assert oracle.block_dot(packed, x) == brute_block_dot(packed, x)
        x = np.full(32, 127, np.int8)
        assert oracle.block_dot(np.full(16, 0x77, np.uint8), x) == 32 * 12 * 127
        assert oracle.block_dot(np.full(16, 0xFF, np.uint8), x) == -32 * 12 * 127
        assert oracle.block_dot(np.full(16, 0x88, np.uint8), x) == 0  # negative zero nibble counts 0
    oracle.force_scalar(0)


def test_block_dot_i8_matches_brute_force_on_reference_stream():
    # src/q8.rs:301-316: seed 0x12345678
    for scalar in (0, 1):
        oracle.force_scalar(scalar)
        rng = oracle.Rng(0x12345678)
        for _ in range(2000):
            w = (rng.u8(32) % 255).astype(np.uint8).view(np.int8)
            x = (rng.u8(32) % 255).astype(np.uint8).view(np.int8)
            if not scalar:
                # the stream holds -128 (128 as i8); the AVX2 kernel is only exact for |q| <= 127
                # (src/q8.rs:147-150), which quantize_q8 guarantees: keep the SIMD cases in that domain
                w, x = np.maximum(w, -127), np.maximum(x, -127)
            assert oracle.block_dot_i8(w, x) == int((w.astype(np.int64) * x.astype(np.int64)).sum())
        p, n = np.full(32, 127, np.int8), np.full(32, -127, np.int8)
        assert oracle.block_dot_i8(p, p) == 32 * 127 * 127
        assert oracle.block_dot_i8(n, p) == -32 * 127 * 127
        assert oracle.block_dot_i8(n, n) == 32 * 127 * 127
    oracle.force_scalar(0)


def test_dot_order():
    # src/model.rs:63-82: 8 accumulators, ((p01+p23)+p45)+p67, sequential tail
    rng = oracle.Rng(0xABCDEF)
    for n in [0, 1, 7, 8, 9, 15, 16, 17, 64, 100, 1024, 1027]:
        a, b = rng.f32(n), rng.f32(n)
        acc = np.zeros(8, np.float32)
        i = 0
        while i + 8 <= n:
            acc = (acc + a[i:i + 8] * b[i:i + 8]).astype(np.float32)
            i += 8
        s = np.float32(np.float32(np.float32(acc[0] + acc[1]) + np.float32(acc[2] + acc[3])) + np.float32(acc[4] + acc[5]))
        s = np.float32(s + np.float32(acc[6] + acc[7]))
        for j in range(i, n):
            s = np.float32(s + np.float32(a[j] * b[j]))
        assert np.float32(oracle.dot(a, b)).view(np.uint32) == s.view(np.uint32), n


def test_rmsnorm_closed_forms():
    # model::rmsnorm (src/model.rs:599-605).  Pins: (1) a constant vector of a power of two, where every operation of
    # the chain is exact except the final 1/sqrt, which is checked against the float64 value rounded once;
    # (2) random vectors against the float64 formula; (3) the mean square goes through dot()'s accumulation order
    # (a permutation that changes the 8-lane sums changes the last bits, a plain sequential sum would not match).
    n = 64
    x = np.full(n, 0.5, np.float32)
    w = np.arange(1, n + 1, dtype=np.float32)
    eps = np.float32(1e-5)
    inv = np.float32(1.0) / np.sqrt(np.float32(0.25) + eps, dtype=np.float32)
    want = (x * inv) * w
    got = oracle.rmsnorm(x, w, float(eps))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    rng = np.random.default_rng(3)
    for n in (8, 33, 512, 7168):
        x = rng.standard_normal(n).astype(np.float32)
        w = rng.standard_normal(n).astype(np.float32)
        got = oracle.rmsnorm(x, w, 1e-6)
        ref = x.astype(np.float64) / np.sqrt((x.astype(np.float64) ** 2).mean() + 1e-6) * w
        assert np.abs(got - ref).max() <= 4e-7 * np.abs(ref).max() + 1e-12
        ss = np.float32(oracle.dot(x, x)) / np.float32(n)
        inv = np.float32(1.0) / np.sqrt(ss + np.float32(1e-6), dtype=np.float32)
        assert np.array_equal(got.view(np.uint32), ((x * inv) * w).view(np.uint32))
    # scale invariance up to eps: rmsnorm(2x) == rmsnorm(x) when eps = 0 (powers of two commute with every rounding)
    x = rng.standard_normal(256).astype(np.float32)
    w = np.ones(256, np.float32)
    assert np.array_equal(oracle.rmsnorm(x, w, 0.0).view(np.uint32), oracle.rmsnorm(2 * x, w, 0.0).view(np.uint32))
