"""GPU parity, MoE decode layer and router (mk_dev_moe_decode, mk_dev_router_softmax_topk) against the oracle."""
import numpy as np
import pytest

import oracle
from gpu_util import dev, rel_l2, torch_cuda

pytestmark = pytest.mark.gpu
TOL = 1e-5


def build(n_experts, d, inter, cfg=2):
    from microkimi_amd import model, workloads
    host = [(workloads.mxfp4_matrix(cfg, "w1", inter, d, e), workloads.mxfp4_matrix(cfg, "w3", inter, d, e),
             workloads.mxfp4_matrix(cfg, "w2", d, inter, e)) for e in range(n_experts)]
    w1 = [h[0] for h in host]
    w3 = [h[1] for h in host]
    w2 = [h[2] for h in host]
    table = oracle.ExpertTable(w1, w3, w2, d, inter)
    todev = lambda lst: [(dev(p), dev(s)) for p, s in lst]
    experts = model.PackedExperts(todev(w1), todev(w3), todev(w2), d, inter)
    return table, experts


@pytest.mark.parametrize("d,inter,n_experts,B,topk,shared,act", [
    (7168, 2048, 12, 1, 8, 11, 0),    # benchmark layer shapes, batch 1, shared expert
    (7168, 2048, 12, 4, 8, 11, 0),    # batch 4
    (2048, 1024, 6, 3, 2, -1, 1),     # SiTU (K3 rule), no shared expert
    (4096, 2048, 5, 2, 3, 4, 2),      # DeepSeek rule: clamp, weight before W2, plain sum
    (1024, 512, 4, 16, 2, 3, 0),      # batch 16
    (7168, 2048, 12, 9, 8, 11, 0),    # benchmark shapes, two token groups in the gate/up kernel (8 + 1)
    (1024, 4096, 4, 5, 2, 3, 0),      # two rows of W1/W3 per wave
    (96, 64, 4, 2, 2, -1, 0),         # shape off the fast path (composed kernels)
])
def test_moe_decode_q8(d, inter, n_experts, B, topk, shared, act):
    torch = torch_cuda()
    from microkimi_amd import model
    table, experts = build(n_experts, d, inter)
    rng = np.random.default_rng(B * 100 + d)
    n_routed = n_experts - (1 if shared >= 0 else 0)
    ids = np.stack([rng.permutation(n_routed)[:topk] for _ in range(B)]).astype(np.int32)
    wts = rng.random((B, topk)).astype(np.float32)
    wts /= wts.sum(axis=1, keepdims=True)
    # expert outputs grow with d * inter: keep the hidden state small so SwiGLU stays in range
    x = (rng.standard_normal((B, d)) * 0.02).astype(np.float32)
    limit = 10.0 if act == 2 else 0.0
    got = model.moe_decode(experts, dev(ids), dev(wts), dev(x), shared=shared, mode=1, act_kind=act, limit=limit).cpu().numpy()
    want = oracle.moe_decode(table, ids.astype(np.uint32), wts, x, shared=shared, mode=1, act_kind=act, limit=limit, threads=8)
    assert np.isfinite(want).all()
    assert rel_l2(got, want) <= TOL


def test_moe_decode_f32_mode():
    from microkimi_amd import model
    d, inter, n_experts, B, topk = 2048, 1024, 6, 2, 3
    table, experts = build(n_experts, d, inter)
    rng = np.random.default_rng(5)
    ids = np.stack([rng.permutation(n_experts - 1)[:topk] for _ in range(B)]).astype(np.int32)
    wts = rng.random((B, topk)).astype(np.float32)
    x = (rng.standard_normal((B, d)) * 0.02).astype(np.float32)
    got = model.moe_decode(experts, dev(ids), dev(wts), dev(x), shared=5, mode=0).cpu().numpy()
    want = oracle.moe_decode(table, ids.astype(np.uint32), wts, x, shared=5, mode=0, threads=8)
    assert rel_l2(got, want) <= TOL


def test_router_softmax_topk():
    from microkimi_amd import model, workloads
    logits, _ = workloads.config2_tokens(16)
    logits[3, [7, 100]] = logits[3].max() + 1.0   # exact tie for the first place
    logits[4, :] = 0.0                            # all equal: the first k indices in order
    ids, w = model.router_softmax_topk(dev(logits), 8)
    ids, w = ids.cpu().numpy(), w.cpu().numpy()
    for t in range(16):
        oi, ow = oracle.router_softmax(logits[t], 8)
        assert ids[t].tolist() == oi.tolist(), t
        assert np.abs(w[t] - ow).max() <= 1e-6
    assert ids[3, :2].tolist() == [7, 100] and ids[4].tolist() == list(range(8))
