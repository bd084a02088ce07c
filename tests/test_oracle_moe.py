"""Pins the routers, the expert FFN and the MoE layer structure (src/model.rs:2150-2729, src/deepseek.rs:16-100,1038-1108)."""
import json
import os

import numpy as np

import oracle

G = os.path.join(os.path.dirname(__file__), "golden")
GOLD = json.load(open(os.path.join(G, "ds_golden2_gate_expert.json")))


def test_gate_golden_vector():
    # src/selftest.rs:258-311: 3 tokens x 32 experts, top-6, route_scale 1.5
    g = GOLD["gate"]
    x = np.asarray(g["x"], np.float32).reshape(3, 16)
    want_idx = np.asarray(g["indices"]).reshape(3, 6)
    want_w = np.asarray(g["weights"], np.float64).reshape(3, 6)
    scale = np.abs(want_w).max()
    for t in range(3):
        ids, w = oracle.gate_forward(x[t], g["gate_w"], g["bias"], 32, 6, 1.5)
        assert sorted(ids.tolist()) == sorted(want_idx[t].tolist())
        got = dict(zip(ids.tolist(), w.tolist()))
        for i, ww in zip(want_idx[t], want_w[t]):
            assert abs(got[int(i)] - ww) <= 1e-5 + 1e-3 * scale


def test_expert_golden_vector():
    # src/selftest.rs:313-323: swiglu_limit 10, inter 16, d 8
    g = GOLD["expert"]
    out = oracle.expert_forward_f32(g["w1"], g["w2"], g["w3"], g["x"], 16, 10.0)
    want = np.asarray(g["out"], np.float64)
    assert np.abs(out - want).max() <= 1e-4 * max(np.abs(want).max(), 1.0)


def test_router_softmax_brute_force_and_ties():
    rng = np.random.default_rng(2)
    for _ in range(50):
        logits = rng.standard_normal(256).astype(np.float32)
        ids, w = oracle.router_softmax(logits, 8)
        p = np.exp(logits.astype(np.float64) - logits.max())
        p /= p.sum()
        order = np.argsort(-p, kind="stable")[:8]
        assert ids.tolist() == order.tolist()
        assert np.abs(w - p[order] / p[order].sum()).max() <= 1e-6
        assert abs(w.sum() - 1) <= 1e-6
    # ties resolve to the lowest index, in ascending index order inside the selection
    logits = np.zeros(16, np.float32)
    logits[[3, 9]] = 1.0
    ids, w = oracle.router_softmax(logits, 4)
    assert ids.tolist() == [3, 9, 0, 1]
    ids, _ = oracle.router_sigmoid(np.zeros(10, np.float32), None, 3)
    assert ids.tolist() == [0, 1, 2]


def test_router_sigmoid_bias_only_for_selection():
    logits = np.array([0.0, 2.0, 1.0, -1.0], np.float32)
    bias = np.array([10.0, 0.0, 0.0, 0.0], np.float32)
    ids, w = oracle.router_sigmoid(logits, bias, 2)
    assert ids.tolist() == [0, 1]
    sc = 1 / (1 + np.exp(-logits[[0, 1]].astype(np.float64)))
    assert np.abs(w - sc / sc.sum()).max() <= 1e-6


def make_experts(n, d, inter, seed):
    rng = np.random.default_rng(seed)

    def blob(r, c):
        return rng.integers(0, 256, (r, c // 2), dtype=np.uint8), rng.integers(118, 131, (r, c // 32), dtype=np.uint8)

    w1 = [blob(inter, d) for _ in range(n)]
    w3 = [blob(inter, d) for _ in range(n)]
    w2 = [blob(d, inter) for _ in range(n)]
    return oracle.ExpertTable(w1, w3, w2, d, inter), (w1, w3, w2)


def test_moe_decode_is_the_sum_of_expert_calls():
    d, inter, n, B, topk = 128, 64, 6, 3, 2
    table, (w1, w3, w2) = make_experts(n, d, inter, 4)
    rng = np.random.default_rng(9)
    x = rng.standard_normal((B, d)).astype(np.float32) * np.float32(0.05)
    ids = np.array([[1, 4], [0, 2], [4, 3]], np.uint32)
    wts = rng.random((B, topk)).astype(np.float32)
    for mode in (0, 1):
        out = oracle.moe_decode(table, ids, wts, x, shared=5, mode=mode, threads=3)
        assert np.array_equal(out, oracle.moe_decode(table, ids, wts, x, shared=5, mode=mode, threads=1))
        for t in range(B):
            y = np.zeros(d, np.float32)
            for s in range(topk):
                e = int(ids[t, s])
                o = oracle.expert_packed(w1[e], w3[e], w2[e], d, inter, x[t], mode=mode)
                y = (y + wts[t, s] * o).astype(np.float32)
            y = (y + oracle.expert_packed(w1[5], w3[5], w2[5], d, inter, x[t], mode=mode)).astype(np.float32)
            assert np.array_equal(out[t].view(np.uint32), y.view(np.uint32))
    # DeepSeek rule: weight folded into the activation before W2, plain sum (src/deepseek.rs:1083-1100)
    out = oracle.moe_decode(table, ids, wts, x, shared=-1, mode=1, act_kind=oracle.ACT_DS, limit=10.0)
    y = np.zeros(d, np.float32)
    for s in range(topk):
        e = int(ids[0, s])
        y = (y + oracle.expert_packed(w1[e], w3[e], w2[e], d, inter, x[0], mode=1, act_kind=oracle.ACT_DS, limit=10.0,
                                      wgt=float(wts[0, s]))).astype(np.float32)
    assert np.array_equal(out[0], y)


def test_expert_packed_swiglu_closed_form():
    d, inter = 64, 32
    table, (w1, w3, w2) = make_experts(1, d, inter, 6)
    x = (np.random.default_rng(3).standard_normal(d) * 0.05).astype(np.float32)
    out = oracle.expert_packed(w1[0], w3[0], w2[0], d, inter, x, mode=0)
    W1 = oracle.mxfp4_dequant(*w1[0], inter, d).astype(np.float64)
    W3 = oracle.mxfp4_dequant(*w3[0], inter, d).astype(np.float64)
    W2 = oracle.mxfp4_dequant(*w2[0], d, inter).astype(np.float64)
    g, u = W1 @ x, W3 @ x
    want = W2 @ (g / (1 + np.exp(-g)) * u)
    assert np.abs(out - want).max() <= 1e-5 * np.abs(want).max()


def test_prefill_grouping_bit_identical_to_decode_f32():
    # src/model.rs:2449-2456: grouped-by-expert batched evaluation == per-token evaluation (f32 arithmetic)
    d, inter, n, T, topk = 64, 64, 8, 21, 3
    table, _ = make_experts(n, d, inter, 8)
    rng = np.random.default_rng(10)
    x = (rng.standard_normal((T, d)) * 0.05).astype(np.float32)
    ids = np.stack([rng.permutation(n)[:topk] for _ in range(T)]).astype(np.uint32)
    wts = rng.random((T, topk)).astype(np.float32)
    a = oracle.moe_prefill(table, ids, wts, x)
    b = oracle.moe_decode(table, ids, wts, x, shared=-1, mode=0)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    # the MXFP8 input rounding changes the result by the e4m3 step (2^-4 relative per element)
    c = oracle.moe_prefill(table, ids, wts, x, round_mxfp8=True)
    rel = np.linalg.norm(c - a) / np.linalg.norm(a)
    assert 0 < rel < 0.1


def test_situ_values():
    for g, u in [(0.3, -1.2), (5.0, 40.0), (-3.0, 0.1)]:
        want = 4 * np.tanh(g / 4) / (1 + np.exp(-g)) * 25 * np.tanh(u / 25)
        assert abs(oracle.situ(g, u) - want) <= 1e-6 * max(1.0, abs(want))


def test_mixed_layer_composition_is_the_layer_and_the_vq_expert_is_three_matvec_vq():
    # oracle.moe_decode_mixed restates the combine of orc_moe_decode in numpy: on a layer without VQ1 experts the two
    # must give the same bits; oracle.expert_vq is matvec_vq, the activation, matvec_vq (src/model.rs:2243-2259)
    rng = np.random.default_rng(0)
    d, inter, ne = 64, 64, 5
    mat = lambda r, c: (rng.integers(0, 256, (r, c // 2), dtype=np.uint8), rng.integers(120, 130, (r, c // 32), dtype=np.uint8))
    w1, w3, w2 = [mat(inter, d) for _ in range(ne)], [mat(inter, d) for _ in range(ne)], [mat(d, inter) for _ in range(ne)]
    tab = oracle.ExpertTable(w1, w3, w2, d, inter)
    ids = np.array([[0, 2], [3, 1], [2, 0]], np.uint32)
    wts = rng.random((3, 2)).astype(np.float32)
    x = rng.standard_normal((3, d)).astype(np.float32)
    ex = [("mxfp4", w1[e], w3[e], w2[e]) for e in range(ne)]
    for act, limit in ((0, 0.0), (1, 0.0), (2, 7.0)):
        a = oracle.moe_decode(tab, ids, wts, x, shared=4, act_kind=act, limit=limit)
        b = oracle.moe_decode_mixed(ex, None, d, inter, ids, wts, x, shared=4, act_kind=act, limit=limit)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    cb = (rng.standard_normal((256, 16)) * 0.1).astype(np.float32)
    i1, i3 = rng.integers(0, 256, (inter, d // 16), dtype=np.uint8), rng.integers(0, 256, (inter, d // 16), dtype=np.uint8)
    i2 = rng.integers(0, 256, (d, inter // 16), dtype=np.uint8)
    g = oracle.vq1_matvec(cb, i1, inter, d, x[0], lut=False)
    u = oracle.vq1_matvec(cb, i3, inter, d, x[0], lut=False)
    act = (g / (np.float32(1.0) + np.exp(-g.astype(np.float64)).astype(np.float32))) * u   # silu(g) * u
    want = oracle.vq1_matvec(cb, i2, d, inter, act.astype(np.float32), lut=False)
    got = oracle.expert_vq(cb, i1, i3, i2, d, inter, x[0])
    assert np.linalg.norm(got - want) <= 1e-6 * np.linalg.norm(want)
