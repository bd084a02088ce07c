"""Pins the MLA q8 cache and the flash attention kernels (src/model.rs:1322-1937)."""
import numpy as np
import pytest

import oracle

NH, NOPE, ROPE, VD = 4, 128, 64, 128  # micro MLA dims (head count reduced to keep the test fast)
HD = NOPE + ROPE
SCALE = float(np.float32(HD) ** np.float32(-0.5))


def fill(length, had=False, spike=False, nh=NH):
    """src/selftest.rs:729-771: same patterns, shared rope across heads."""
    c = oracle.MlaCache(nh, NOPE, ROPE, VD, had=had)
    kf = np.zeros((length, nh * HD), np.float32)
    vf = np.zeros((length, nh * VD), np.float32)
    for j in range(length):
        k = oracle.pattern(j * 7919, nh * HD)
        v = oracle.pattern(j * 5449 + 313, nh * VD)
        for h in range(1, nh):
            k[h * HD + NOPE:(h + 1) * HD] = k[NOPE:HD]
        if spike and j % 3 == 0:
            for h in range(nh):
                k[h * HD + 5] = 30.0 * oracle.pattern(j + 17, 1)[0]
                v[h * VD + 9] = 30.0 * oracle.pattern(j + 23, 1)[0]
        kf[j], vf[j] = k, v
        c.push(k, v)
    q = oracle.pattern(4242, nh * HD)
    return c, kf, vf, q


@pytest.mark.parametrize("length", [1, 7, 64, 65, 512])
def test_flash_vs_materialised_f32(length):
    # src/selftest.rs:656-704: tol 1e-5 abs
    _, kf, vf, q = fill(length)
    for h in range(NH):
        qh = q[h * HD:(h + 1) * HD]
        a = oracle.mla_attn_ref(NH, NOPE, ROPE, VD, kf, vf, qh, h, length - 1, SCALE)
        b = oracle.mla_attn_flash(NH, NOPE, ROPE, VD, kf, vf, qh, h, length - 1, SCALE)
        assert np.abs(a - b).max() <= 1e-5


@pytest.mark.parametrize("length,had,spike", [(1, False, False), (7, False, False), (64, False, False), (65, False, False),
                                              (512, False, False), (65, True, False), (512, True, True), (512, False, True)])
def test_q8_mqa_bit_identical_and_bounds(length, had, spike):
    c, kf, vf, q = fill(length, had=had, spike=spike)
    pos = length - 1
    per_head = np.concatenate([oracle.mla_attn_flash_q8(c, q[h * HD:(h + 1) * HD], h, pos, SCALE) for h in range(NH)])
    mqa = oracle.mla_attn_flash_q8_mqa(c, q, pos, SCALE)
    assert np.array_equal(mqa.view(np.uint32), per_head.view(np.uint32))  # src/selftest.rs:774-789
    # round trip within the q8_0 bound (src/selftest.rs:790-841), rope exact
    k2, v2 = c.to_f32()
    kk, k2k = kf.reshape(length, NH, HD), k2.reshape(length, NH, HD)
    assert np.array_equal(kk[:, :, NOPE:], k2k[:, :, NOPE:])
    rot = kk[:, :, :NOPE].copy()
    rotv = vf.reshape(length, NH, VD).copy()
    if had:
        for arr in (rot, rotv):
            flat = arr.reshape(-1, 64)
            for i in range(flat.shape[0]):
                flat[i] = oracle.hadamard64(flat[i])
    bound = max(np.abs(rot.reshape(-1, 32)).max(axis=1).max(), np.abs(rotv.reshape(-1, 32)).max(axis=1).max()) / 254.0
    err = max(np.abs(kk[:, :, :NOPE] - k2k[:, :, :NOPE]).max(), np.abs(vf - v2).max())
    assert err <= bound * 1.02
    # attention vs the f32 cache (src/selftest.rs:871-879)
    worst = 0.0
    for h in range(NH):
        a = oracle.mla_attn_flash(NH, NOPE, ROPE, VD, kf, vf, q[h * HD:(h + 1) * HD], h, pos, SCALE)
        b = per_head[h * VD:(h + 1) * VD]
        worst = max(worst, np.abs(a - b).max() / max(np.abs(a).max(), 1e-12))
    assert worst <= (5e-2 if had else (3e-2 if spike else 1e-2))


def test_q8_flash_closed_form_f64():
    # softmax(scale * (q_rope.kr + dequant(q8 q).dequant(K))) . dequant(V) in f64 reproduces the kernel
    length = 200
    c, kf, vf, q = fill(length)
    k2, v2 = c.to_f32()
    k2 = k2.reshape(length, NH, HD).astype(np.float64)
    v2 = v2.reshape(length, NH, VD).astype(np.float64)
    mqa = oracle.mla_attn_flash_q8_mqa(c, q, length - 1, SCALE).reshape(NH, VD)
    for h in range(NH):
        qh = q[h * HD:(h + 1) * HD]
        qq, qs = oracle.quantize_q8(qh[:NOPE])
        qd = np.concatenate([qq.astype(np.float64) * np.repeat(qs.astype(np.float64), 32), qh[NOPE:].astype(np.float64)])
        s = (k2[:, h, :] @ qd) * SCALE
        p = np.exp(s - s.max())
        p /= p.sum()
        want = p @ v2[:, h, :]
        assert np.abs(mqa[h] - want).max() <= 2e-6 * np.abs(want).max() + 1e-7


def test_len1_output_is_dequantized_v_row():
    c, kf, vf, q = fill(1)
    _, v2 = c.to_f32()
    out = oracle.mla_attn_flash_q8_mqa(c, q, 0, SCALE)
    assert np.array_equal(out, v2[0])  # p = exp(0)/1 = 1 exactly


def test_pos_limits_the_window():
    c, kf, vf, q = fill(130)
    c2, _, _, _ = fill(70)
    a = oracle.mla_attn_flash_q8_mqa(c, q, 69, SCALE)
    b = oracle.mla_attn_flash_q8_mqa(c2, q, 69, SCALE)
    assert np.array_equal(a, b)


def test_absorbed_form_equals_reference_on_replicated_cache():
    """One shared latent row per position (K and V of every head) == the reference kernel run on a
    cache whose per-head rows are copies of that row."""
    nh, L, R, n = 6, 128, 64, 150
    rng = np.random.default_rng(11)
    lat = rng.standard_normal((n, L)).astype(np.float32)
    rope = rng.standard_normal((n, R)).astype(np.float32)
    lq, ls = oracle.quantize_q8(lat)
    rq, rs = oracle.quantize_q8(rope)
    lq, ls, rq, rs = lq.reshape(n, L), ls.reshape(n, L // 32), rq.reshape(n, R), rs.reshape(n, R // 32)
    ls = ls.astype(np.float16).astype(np.float32)  # device scales are f16
    rs = rs.astype(np.float16).astype(np.float32)
    q = rng.standard_normal((nh, L + R)).astype(np.float32)
    scale = float(np.float32(1.0) / np.sqrt(np.float32(192.0)))
    out = oracle.mla_absorbed_decode(lq, ls, rq, rs, q, nh, scale)
    # replicated reference-layout cache
    c = oracle.MlaCache(nh, L, R, L, capacity=n)
    c.n = n
    c.kq[:n] = np.tile(lq, (1, nh))
    c.ks[:n] = np.tile(ls, (1, nh))
    c.vq[:n] = np.tile(lq, (1, nh))
    c.vs[:n] = np.tile(ls, (1, nh))
    c.kr[:n] = (rq.astype(np.float32).reshape(n, R // 32, 32) * rs.reshape(n, R // 32, 1)).reshape(n, R)
    ref = oracle.mla_attn_flash_q8_mqa(c, q.reshape(-1), n - 1, scale).reshape(nh, L)
    assert np.array_equal(out.view(np.uint32), ref.view(np.uint32))
    per_head = oracle.mla_attn_flash_q8(c, q[3], 3, n - 1, scale)
    assert np.array_equal(out[3].view(np.uint32), per_head.view(np.uint32))


def test_hadamard_involution():
    x = oracle.pattern(5, 64)
    y = oracle.hadamard64(oracle.hadamard64(x)) / 64.0
    assert np.abs(x - y).max() <= 1e-6


def test_hadamard_is_the_sylvester_matrix():
    # the butterfly of src/model.rs:1540-1554 is the natural-order Walsh-Hadamard transform: on integer vectors (exact
    # arithmetic) it equals the product with scipy's Sylvester matrix, so a wrong stage, stride or sign shows
    from scipy.linalg import hadamard
    H = hadamard(64).astype(np.float64)
    rng = np.random.default_rng(64)
    for _ in range(4):
        x = rng.integers(-50, 51, 64).astype(np.float32)
        assert np.array_equal(oracle.hadamard64(x).astype(np.float64), H @ x.astype(np.float64))
    e = np.zeros(64, np.float32)
    e[37] = 1.0
    assert np.array_equal(oracle.hadamard64(e).astype(np.float64), H[:, 37])


def test_hadamard_cache_attends_like_the_plain_one():
    # the rotation is orthogonal up to the factor the kernel takes out again: attention over a Hadamard-mode cache agrees
    # with the plain q8 cache to the quantization noise of both (and both with the f32 attention)
    rng = np.random.default_rng(9)
    nh, nope, rope, vd, n = 3, 128, 64, 128, 40
    k = rng.standard_normal((n, nh * (nope + rope))).astype(np.float32)
    v = rng.standard_normal((n, nh * vd)).astype(np.float32)
    q = rng.standard_normal(nh * (nope + rope)).astype(np.float32)
    scale = float(np.float32(nope + rope) ** np.float32(-0.5))
    plain, had = oracle.MlaCache(nh, nope, rope, vd, capacity=n), oracle.MlaCache(nh, nope, rope, vd, had=True, capacity=n)
    for j in range(n):
        plain.push(k[j], v[j])
        had.push(k[j], v[j])
    assert not np.array_equal(plain.kq[:n], had.kq[:n])
    a = oracle.mla_attn_flash_q8_mqa(plain, q, n - 1, scale)
    b = oracle.mla_attn_flash_q8_mqa(had, q, n - 1, scale)
    assert np.linalg.norm(a - b) <= 2e-2 * np.linalg.norm(a)
    kf, vf = had.to_f32()   # de-rotated rows: the q8 round trip (the rope part of a K row is head 0's for every head)
    nope_cols = (np.arange(nh * (nope + rope)) % (nope + rope)) < nope
    assert np.abs(kf - k)[:, nope_cols].max() <= 0.05 and np.abs(vf - v).max() <= 0.05
