"""Pins the oracle's codec functions (e2m1 / e8m0 / e4m3) against the
reference's golden vectors and against closed forms."""
import json
import os

import numpy as np

import oracle

G = os.path.join(os.path.dirname(__file__), "golden")
E2M1 = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0], np.float64)


def np_dequant(packed, scales, rows, cols):
    """Independent closed form: LUT[nibble] * 2^(byte-127), low nibble = even column (ref/mxfp4_numpy.py:16-27)."""
    packed = np.asarray(packed, np.uint8).reshape(rows, cols // 2)
    idx = np.empty((rows, cols), np.uint8)
    idx[:, 0::2] = packed & 0x0F
    idx[:, 1::2] = packed >> 4
    sc = np.exp2(np.asarray(scales, np.float64).reshape(rows, cols // 32) - 127.0)
    return (E2M1[idx] * np.repeat(sc, 32, axis=1)).astype(np.float32)


def test_fp4_golden_vector_bit_exact():
    # src/selftest.rs:226-234 consumes the same vector (torch-generated)
    g = json.load(open(os.path.join(G, "ds_golden_fp4.json")))
    w = oracle.mxfp4_dequant(g["packed"], g["scales"], g["rows"], g["cols"])
    want = np.asarray(g["dequant"], np.float64).astype(np.float32).reshape(g["rows"], g["cols"])
    assert np.array_equal(np.abs(w).view(np.uint32), np.abs(want).view(np.uint32))  # the JSON renders -0.0 as "-0.0" or "0.0"
    assert np.array_equal(w, want)


def test_dequant_exhaustive_nibble_x_scale():
    # all 16 nibbles x all 256 scale bytes; byte 0 is the subnormal 2^-127
    for sb in range(256):
        packed = np.array([n | (n << 4) for n in range(16)], np.uint8)
        row = np.zeros(16, np.uint8)
        row[:16] = packed
        w = oracle.mxfp4_dequant(row, [sb], 1, 32)[0]
        want = np_dequant(row, [min(sb, 254)], 1, 32)[0]
        if sb == 255:  # 2^128 overflows f32: exp2_i builds the bit pattern of +inf
            assert np.isinf(oracle.exp2_i(128))
            continue
        assert np.array_equal(w.view(np.uint32), want.view(np.uint32)), sb
    assert np.float32(oracle.exp2_i(-127)).view(np.uint32) == 0x00400000
    assert np.float32(oracle.scale_from_byte(0)).view(np.uint32) == 0x00400000
    for sb in range(1, 255):
        assert oracle.scale_from_byte(sb) == oracle.exp2_i(sb - 127) == 2.0 ** (sb - 127)
    # nibble 8 is negative zero: the sign bit survives the scale
    w = oracle.mxfp4_dequant(np.full(16, 0x88, np.uint8), [127], 1, 32)
    assert np.all(w.view(np.uint32) == 0x80000000)


def test_e4m3_decode_closed_form_and_roundtrip():
    for b in range(256):
        v = oracle.e4m3_to_f32(b)
        s, e, m = b >> 7, (b >> 3) & 15, b & 7
        if e == 15 and m == 7:
            assert np.isnan(v)
            continue
        want = (-1.0) ** s * ((m / 8.0) * 2.0 ** -6 if e == 0 else (1 + m / 8.0) * 2.0 ** (e - 7))
        assert v == want, b
        # encode(decode(b)) == b for every finite code (negative zero keeps its sign)
        assert oracle.f32_to_e4m3(v) == b, b
    assert oracle.f32_to_e4m3(1e9) == 0x7E and oracle.f32_to_e4m3(-1e9) == 0xFE
    assert oracle.f32_to_e4m3(float("nan")) == 0x7F
    # ties to even mantissa: 1 + 1/16 is halfway between m=0 and m=1 -> m=0; 1 + 3/16 -> m=2
    assert oracle.f32_to_e4m3(1.0625) == 0x38 and oracle.f32_to_e4m3(1.1875) == 0x3A
    # subnormal carry into the smallest normal
    assert oracle.f32_to_e4m3(2.0 ** -6 * (7.6 / 8)) == 0x08


def test_fp8_golden_vector_byte_exact():
    # src/selftest.rs:204-225: dequant matches torch, quantize reproduces torch's bytes with zero diffs
    g = np.load(os.path.join(G, "ds_golden_fp8.npz"))
    rows, cols = int(g["rows"]), int(g["cols"])
    w = oracle.dequant_fp8(g["w_packed"], g["scales"], rows, cols)
    assert np.array_equal(w.reshape(-1), g["dequant"])
    qw, qs = oracle.quantize_fp8(g["w_orig"], rows, cols)
    assert np.array_equal(qw.reshape(-1), g["w_packed"])
    assert np.array_equal(qs.reshape(-1), g["scales"])


def test_fp8_roundtrip_block32():
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(256) * 3).astype(np.float32)
    y, codes, exps = oracle.fp8_roundtrip(x, 32)
    for b in range(8):
        blk = x[b * 32:(b + 1) * 32]
        e = int(np.ceil(np.log2(max(np.abs(blk).max(), 1e-4) / 448.0)))
        assert exps[b] == e + 127
        dec = np.array([oracle.e4m3_to_f32(int(c)) for c in codes[b * 32:(b + 1) * 32]], np.float32) * np.float32(2.0 ** e)
        assert np.array_equal(dec, y[b * 32:(b + 1) * 32])
        assert np.abs(y[b * 32:(b + 1) * 32] - blk).max() <= np.abs(blk).max() * 2.0 ** -4 + 1e-6


def test_fp8_roundtrip_scale_clamp():
    # a block whose largest value exceeds 448 * 2^8: with the reference's clamp (src/deepseek.rs:316) the scale stops at
    # 2^8 and the values saturate at +-448 * 2^8; with the full e8m0 range the block keeps its relative precision
    x = np.zeros(64, np.float32)
    x[:32] = np.linspace(-4.0e5, 4.0e5, 32, dtype=np.float32)      # 4e5 > 448 * 256 = 114688
    x[32:] = np.linspace(-1.0e5, 1.0e5, 32, dtype=np.float32)      # below the limit: both forms agree
    y8, c8, e8 = oracle.fp8_roundtrip(x, 32, emax=8)
    yf, cf, ef = oracle.fp8_roundtrip(x, 32, emax=127)
    assert e8[0] == 8 + 127 and ef[0] == int(np.ceil(np.log2(4.0e5 / 448.0))) + 127 == 10 + 127
    assert np.abs(y8[:32]).max() == 448.0 * 256.0
    sat = np.abs(x[:32]) >= 448.0 * 256.0
    assert sat.sum() >= 10 and np.array_equal(y8[:32][sat], np.sign(x[:32][sat]) * np.float32(448.0 * 256.0))
    assert np.abs(yf[:32] - x[:32]).max() <= 4.0e5 * 2.0 ** -4
    assert e8[1] == ef[1] and np.array_equal(y8[32:], yf[32:]) and np.array_equal(c8[32:], cf[32:])
    # the lower clamp is the same in both: an all-zero block takes amax = 1e-4
    z8, _, ez8 = oracle.fp8_roundtrip(np.zeros(32, np.float32), 32, emax=8)
    zf, _, ezf = oracle.fp8_roundtrip(np.zeros(32, np.float32), 32, emax=127)
    assert ez8[0] == ezf[0] == int(np.ceil(np.log2(1e-4 / 448.0))) + 127 and not z8.any() and not zf.any()


def test_round_bf16_is_torch_bfloat16():
    import torch
    rng = np.random.default_rng(11)
    bits = rng.integers(0, 2 ** 32, 200000, dtype=np.uint64).astype(np.uint32)
    # ties (low half exactly 0x8000) with even and odd upper halves, values next to them, the largest finite
    # numbers (which round up to infinity), subnormals, zeros, infinities
    special = np.array([0x3F808000, 0x3F818000, 0x3F807FFF, 0x3F808001, 0xBF808000, 0xBF818000, 0x7F7FFFFF, 0x7F7F8000, 0x7F7F7FFF,
                        0xFF7FFFFF, 0x00008000, 0x00018000, 0x00007FFF, 0x80008000, 0, 0x80000000, 0x7F800000, 0xFF800000], np.uint32)
    x = np.concatenate([bits, special]).view(np.float32)
    x = x[~np.isnan(x)]
    got = oracle.round_bf16(x)
    want = torch.from_numpy(x.copy()).to(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    nan = oracle.round_bf16(np.array([np.nan], np.float32))
    assert np.isnan(nan[0])


def _block_errors(w, rows, cols, p, s):
    wq = oracle.mxfp4_dequant(p, s, rows, cols).astype(np.float64).reshape(-1, 32)
    return ((w.astype(np.float64).reshape(-1, 32) - wq) ** 2).sum(axis=1)


def _never_worse(w, rows, cols):
    p0, s0 = oracle.mxfp4_quantize(w, rows, cols, search=False)
    p1, s1 = oracle.mxfp4_quantize(w, rows, cols, search=True)
    e0, e1 = _block_errors(w, rows, cols, p0, s0), _block_errors(w, rows, cols, p1, s1)
    assert np.all(e1 <= e0 * (1 + 1e-9) + 1e-20)


def test_quantize_search_never_worse():
    # src/mxfp4.rs:575-598 restated
    for rows, cols in [(64, 128), (128, 64), (3, 64), (1, 32), (256, 1024)]:
        _never_worse(oracle.pattern(0, rows * cols), rows, cols)
    rows, cols = 16, 64
    w = np.full(rows * cols, 0.01, np.float32)
    for g in range(rows * cols // 32):
        w[g * 32] = 3.7 if g % 2 == 0 else -5.9
    _never_worse(w, rows, cols)
    _never_worse(np.zeros(64, np.float32), 2, 32)
    _never_worse((E2M1[np.arange(64) % 16] * 0.125).astype(np.float32), 2, 32)


def test_quantize_roundtrip_exact_levels_and_zero_group():
    # src/mxfp4.rs:600-611
    rows, cols = 4, 64
    w = (E2M1[np.arange(rows * cols) % 16] * 0.25).astype(np.float32)
    p, s = oracle.mxfp4_quantize(w, rows, cols)
    assert np.array_equal(oracle.mxfp4_dequant(p, s, rows, cols).reshape(-1), w)
    # an all-zero group gets scale byte 0 (src/metal.rs:1332) and zero nibbles
    p, s = oracle.mxfp4_quantize(np.zeros(64, np.float32), 2, 32)
    assert np.all(s == 0) and np.all(p == 0)
    # quantize(dequant(.)) is the identity on grids that use the top level (naive scale is then exact)
    rng = np.random.default_rng(1)
    packed = rng.integers(0, 256, (8, 32), dtype=np.uint8)
    packed[:, 0] = 0x77
    scales = rng.integers(110, 140, (8, 2), dtype=np.uint8)
    w = oracle.mxfp4_dequant(packed, scales, 8, 64)
    p2, s2 = oracle.mxfp4_quantize(w, 8, 64, search=False)
    assert np.array_equal(s2, scales)
    assert np.array_equal(oracle.mxfp4_dequant(p2, s2, 8, 64), w)


def test_naive_scale_rule_matches_numpy_restatement():
    # nano/export.py:23-41 states the same rule in numpy: e = ceil(log2(maxabs/6)), nearest level
    rng = np.random.default_rng(7)
    w = (rng.standard_normal((16, 64)) * 2).astype(np.float32)
    p, s = oracle.mxfp4_quantize(w, 16, 64, search=False)
    grp = w.reshape(16, 2, 32)
    e = np.ceil(np.log2(np.abs(grp).max(axis=2) / np.float32(6.0))).astype(np.int32)
    assert np.array_equal(s.astype(np.int32) - 127, e)
    q = np.clip(grp / np.exp2(e)[..., None].astype(np.float32), -6, 6)
    lv = np.abs(E2M1[:8])
    idx = np.abs(np.abs(q)[..., None] - lv).argmin(-1)
    # midpoints go up in the reference (mag >= bound): argmin picks the lower one, so compare off midpoints only
    off_mid = ~np.isin(np.abs(q), [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0])
    idx = np.where(np.signbit(q), idx + 8, idx).reshape(16, 64)
    got = np.empty((16, 64), np.uint8)
    got[:, 0::2] = p & 0x0F
    got[:, 1::2] = p >> 4
    assert np.array_equal(got[off_mid.reshape(16, 64)], idx[off_mid.reshape(16, 64)])


def test_mxfp4sq_properties():
    # MXFP4SQ (src/mxfp4.rs:140-229), pinned by what the format promises: smax is the largest maxabs / 6; the decoded
    # scale of every group is at least its ideal scale (nothing clips) and the byte is the smallest with that property;
    # the group that sets smax gets byte 255 and scale smax exactly; values that sit on the grid come back exactly
    rng = np.random.default_rng(8)
    rows, cols = 16, 128
    w = (rng.standard_normal((rows, cols)) * np.exp2(rng.integers(-8, 3, (rows, cols // 32)).astype(np.float32)).repeat(32, axis=1)).astype(np.float32)
    w[3, 32:64] = 0.0
    p, s, smax = oracle.mxfp4sq_quantize(w, rows, cols)
    ideal = np.abs(w).reshape(rows, cols // 32, 32).max(axis=2) / np.float32(6.0)
    assert smax == ideal.max()
    dec = np.array([[oracle.scale_sq(q, smax) for q in r] for r in s], np.float32)
    assert np.all(dec >= ideal) and s[3, 1] == 0
    lower = np.array([[oracle.scale_sq(q - 1, smax) if q > 0 else 0.0 for q in r] for r in s], np.float32)
    assert np.all((lower < ideal) | (s == 0))
    gi = np.unravel_index(ideal.argmax(), ideal.shape)
    assert s[gi] == 255 and oracle.scale_sq(255, smax) == smax
    assert oracle.scale_sq(0, 1.0) == 2.0 ** -16 and oracle.scale_sq(127, 4.0) == 1.0
    back = oracle.mxfp4sq_dequant(p, s, smax, rows, cols)
    assert np.all(np.abs(back) <= 6.0 * dec.repeat(32, axis=1)) and np.all(np.abs(back - w) <= dec.repeat(32, axis=1))   # half the widest level step
    # a matrix built on the grid: levels times decoded scales of chosen bytes round-trips bit for bit
    levels = np.array([0, 0.5, 1, 1.5, 2, 3, 4, 6], np.float32)
    q = rng.integers(0, 256, (4, 2)).astype(np.uint8)
    q[0, 0] = 255
    sc = np.array([[oracle.scale_sq(v, 3.0) for v in r] for r in q], np.float32)
    nib = rng.integers(0, 8, (4, 64))
    nib[:, 0] = 7
    nib[:, 32] = 7                                   # every group reaches level 6: its ideal scale is its decoded scale
    grid = (levels[nib] * sc.repeat(32, axis=1) * rng.choice([-1.0, 1.0], (4, 64))).astype(np.float32)
    p2, s2, smax2 = oracle.mxfp4sq_quantize(grid, 4, 64)
    assert smax2 == np.float32(3.0)
    b2 = oracle.mxfp4sq_dequant(p2, s2, smax2, 4, 64)
    assert np.array_equal(np.abs(b2), np.abs(grid))


def test_quantize_q8_non_finite_values():
    """src/q8.rs:49-69 on blocks with NaN or inf, fixed by the language rules the reference's expression runs under:
    f32::max skips a NaN (the block maximum comes from the other values), f32::clamp keeps a NaN, and `NaN as i8` is 0;
    a block with an inf has scale inf, finite / inf = 0 and inf / inf = NaN -> 0."""
    x = np.zeros(96, dtype=np.float32)
    x[:32] = np.linspace(-2.0, 2.0, 32, dtype=np.float32)
    x[5] = np.nan
    x[32:64] = 1.5
    x[40] = np.inf
    x[41] = -np.inf
    x[64:96] = np.nan
    q, s = oracle.quantize_q8(x)
    clean = x[:32].copy()
    clean[5] = 0.0
    qc, sc = oracle.quantize_q8(clean)
    assert s[0] == sc[0] and np.array_equal(q[:32], qc[:32]) and q[5] == 0
    assert np.isinf(s[1]) and not q[32:64].any()
    assert s[2] == 0.0 and not q[64:].any()   # every value skipped: maximum 0, the all-zero rule
