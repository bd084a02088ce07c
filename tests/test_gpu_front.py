"""GPU parity of the steps in front of the quantized matvecs: rmsnorm (+ q8), the f32 matvec with the reference's
dot contract, and the three routing rules, against the oracle.  rmsnorm, its q8 form and the f32 matvec are
bit-exact; router ids are exact and weights within 1e-6 (device expf / logf differ from the host libm by ulps)."""
import numpy as np
import pytest

import oracle
from gpu_util import dev, torch_cuda

pytestmark = pytest.mark.gpu


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


@pytest.mark.parametrize("B,d", [(1, 7168), (3, 512), (2, 64), (5, 2048), (1, 100)])
def test_rmsnorm_bit_exact(B, d):
    from microkimi_amd import model
    rng = np.random.default_rng(B * 1000 + d)
    x = (rng.standard_normal((B, d)) * rng.choice([1e-3, 1.0, 50.0])).astype(np.float32)
    w = rng.standard_normal(d).astype(np.float32)
    for eps in (1e-5, 1e-6):
        got = model.rmsnorm(dev(x), dev(w), eps).cpu().numpy()
        for b in range(B):
            assert np.array_equal(bits(got[b]), bits(oracle.rmsnorm(x[b], w, eps))), (b, eps)
    if d % 32 == 0:
        y, q, s = model.rmsnorm(dev(x), dev(w), 1e-5, quantize=True)
        q, s = q.cpu().numpy(), s.cpu().numpy()
        for b in range(B):
            qo, so = oracle.quantize_q8(oracle.rmsnorm(x[b], w, 1e-5))
            assert np.array_equal(q[b], qo) and np.array_equal(bits(s[b]), bits(so)), b


def test_rmsnorm_zero_row_and_ties():
    from microkimi_amd import model
    d = 64
    x = np.zeros((2, d), np.float32)
    x[1, :32] = np.arange(32) - 15.5  # q8 ties after scaling
    w = np.ones(d, np.float32)
    y, q, s = model.rmsnorm(dev(x), dev(w), 1e-5, quantize=True)
    for b in range(2):
        ref = oracle.rmsnorm(x[b], w, 1e-5)
        assert np.array_equal(bits(y.cpu().numpy()[b]), bits(ref))
        qo, so = oracle.quantize_q8(ref)
        assert np.array_equal(q.cpu().numpy()[b], qo) and np.array_equal(bits(s.cpu().numpy()[b]), bits(so))


@pytest.mark.parametrize("rows,cols,B", [(256, 7168, 1), (256, 7168, 4), (7, 40, 2), (33, 8, 1), (64, 1027, 3)])
def test_matvec_f32_bit_exact(rows, cols, B):
    from microkimi_amd import model
    rng = np.random.default_rng(rows + cols)
    w = rng.standard_normal((rows, cols)).astype(np.float32)
    x = rng.standard_normal((B, cols)).astype(np.float32)
    got = model.matvec(dev(w), dev(x)).cpu().numpy()
    for b in range(B):
        assert np.array_equal(bits(got[b]), bits(oracle.matvec_f32(w, rows, cols, x[b]))), b


@pytest.mark.parametrize("n,k", [(256, 8), (384, 6), (16, 4), (5, 5)])
def test_router_rules(n, k):
    from microkimi_amd import model
    rng = np.random.default_rng(n * 10 + k)
    B = 6
    logits = (rng.standard_normal((B, n)) * 2).astype(np.float32)
    logits[1, 3] = logits[1, min(7, n - 1)]  # a tie on the logits: the lowest index wins
    bias = (rng.standard_normal(n) * 0.1).astype(np.float32)
    for kind, name in ((model.ROUTER_SOFTMAX, "softmax"), (model.ROUTER_SIGMOID, "sigmoid"), (model.ROUTER_SQRTSOFTPLUS, "sqrtsoftplus")):
        for use_bias in (False, True):
            if kind == model.ROUTER_SOFTMAX and use_bias:
                continue
            b = bias if use_bias else None
            ids, wts = model.router_topk(dev(logits), k, kind, None if b is None else dev(b), route_scale=2.5)
            ids, wts = ids.cpu().numpy(), wts.cpu().numpy()
            for t in range(B):
                if kind == model.ROUTER_SOFTMAX:
                    io, wo = oracle.router_softmax(logits[t], k)
                elif kind == model.ROUTER_SIGMOID:
                    io, wo = oracle.router_sigmoid(logits[t], b, k)
                else:
                    # the oracle's gate takes x and a gate matrix: the identity reproduces the given logits exactly
                    io, wo = oracle.gate_forward(logits[t], np.eye(n, dtype=np.float32), b, n, k, 2.5)
                assert np.array_equal(ids[t], io.astype(np.int32)), (name, use_bias, t)
                assert np.abs(wts[t] - wo).max() <= 1e-6 * max(1.0, np.abs(wo).max()), (name, use_bias, t)


def test_norm_route_experts_without_host_round_trip():
    # one decode token through norm -> gate matvec -> router -> expert section, every step on the device,
    # against the same chain on the oracle
    torch = torch_cuda()
    from microkimi_amd import model, workloads
    d, inter, n_experts, topk = 256, 128, 12, 4
    rng = np.random.default_rng(5)
    host = [(workloads.mxfp4_matrix(2, "w1", inter, d, e), workloads.mxfp4_matrix(2, "w3", inter, d, e),
             workloads.mxfp4_matrix(2, "w2", d, inter, e)) for e in range(n_experts)]
    hidden = rng.standard_normal(d).astype(np.float32)
    nw = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32)
    gate = (rng.standard_normal((n_experts, d)) * 0.2).astype(np.float32)
    bias = (rng.standard_normal(n_experts) * 0.01).astype(np.float32)
    xo = oracle.rmsnorm(hidden, nw, 1e-5)
    lo = oracle.matvec_f32(gate, n_experts, d, xo)
    io, wo = oracle.router_sigmoid(lo, bias, topk)
    table = oracle.ExpertTable([h[0] for h in host], [h[1] for h in host], [h[2] for h in host], d, inter)
    want = oracle.moe_decode(table, io[None, :], wo[None, :], xo[None, :], act_kind=oracle.ACT_SITU)
    pk = lambda k: [(dev(h[k][0]), dev(h[k][1])) for h in host]
    experts = model.PackedExperts(pk(0), pk(1), pk(2), d, inter)
    x = model.rmsnorm(dev(hidden[None, :]), dev(nw), 1e-5)
    logits = model.matvec(dev(gate), x)
    ids, wts = model.router_topk(logits, topk, model.ROUTER_SIGMOID, dev(bias))
    got = model.moe_decode(experts, ids, wts, x, act_kind=model.ACT_SITU).cpu().numpy()
    assert np.array_equal(ids.cpu().numpy()[0], io.astype(np.int32))
    assert np.linalg.norm(got - want) / np.linalg.norm(want) <= 1e-5


@pytest.mark.parametrize("B,d,n,k,kind", [(1, 7168, 256, 8, 0), (3, 7168, 384, 6, 1), (4, 512, 16, 4, 2), (5, 2048, 64, 8, 0), (9, 4096, 4096, 64, 1),
                                          (16, 7168, 256, 8, 0)])
def test_norm_gate_route_gives_the_three_calls_bits(B, d, n, k, kind):
    # mk_dev_norm_gate_route against mk_dev_rmsnorm -> mk_dev_matvec_f32 -> mk_dev_router_topk (each held to the oracle by the
    # tests above): normed rows, logits and routing weights bit for bit, ids equal; and the rows against the oracle too
    torch = torch_cuda()
    from microkimi_amd import model
    rng = np.random.default_rng(B * 1000 + n)
    x = rng.standard_normal((B, d)).astype(np.float32)
    nw = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32)
    gate = (rng.standard_normal((n, d)) * d ** -0.5).astype(np.float32)
    bias = (rng.standard_normal(n) * 0.05).astype(np.float32) if kind else None
    xd, nwd, gd, bd = dev(x), dev(nw), dev(gate), None if bias is None else dev(bias)
    xn0 = model.rmsnorm(xd, nwd, 1e-6)
    lg0 = model.matvec(gd, xn0)
    ids0, w0 = model.router_topk(lg0, k, kind, bd, route_scale=1.5)
    for rep in range(2):
        xn, lg, ids, w = model.norm_gate_route(xd, nwd, 1e-6, gd, k, kind, bd, route_scale=1.5)
        torch.cuda.synchronize()
        assert np.array_equal(bits(xn.cpu().numpy()), bits(xn0.cpu().numpy())), rep
        assert np.array_equal(bits(lg.cpu().numpy()), bits(lg0.cpu().numpy())), rep
        assert np.array_equal(ids.cpu().numpy(), ids0.cpu().numpy()), rep
        assert np.array_equal(bits(w.cpu().numpy()), bits(w0.cpu().numpy())), rep
    assert np.array_equal(bits(xn.cpu().numpy()[0]), bits(oracle.rmsnorm(x[0], nw, 1e-6)))
    assert np.array_equal(bits(lg.cpu().numpy()[0]), bits(oracle.matvec_f32(gate, n, d, oracle.rmsnorm(x[0], nw, 1e-6))))


def test_norm_gate_route_refuses_what_it_does_not_take():
    torch = torch_cuda()
    from microkimi_amd import model
    from microkimi_amd._lib import MkError
    x = torch.zeros((1, 100), device="cuda")
    with pytest.raises(MkError) as e:
        model.norm_gate_route(x, torch.ones(100, device="cuda"), 1e-6, torch.zeros((8, 100), device="cuda"), 2)
    assert e.value.status == -4
