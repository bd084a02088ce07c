"""GPU parity, MXFP4 grouped expert GEMM on the block-scaled matrix cores.

Tight check: against the f64 product of the dequantized weights and the MXFP8-rounded activations (the oracle's
fp8_roundtrip with block 32), i.e. the same inputs the kernel sees.  Informational: the distance to the pure-f32
CPU path, which is the e4m3 rounding of the activations (about 2-3 %)."""
import numpy as np
import pytest

import oracle
from gpu_util import dev, rel_l2, torch_cuda

pytestmark = pytest.mark.gpu


def run_case(rows, cols, counts, seed):
    torch = torch_cuda()
    from microkimi_amd import dequant, model, workloads
    rng = np.random.default_rng(seed)
    n_groups = len(counts)
    mats = [workloads.mxfp4_matrix(4, "w", rows, cols, seed * 100 + e) for e in range(n_groups)]
    m = int(sum(counts))
    x = rng.standard_normal((m, cols)).astype(np.float32)
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    codes, exps = dequant.quantize_mxfp8(dev(x))
    out = model.grouped_gemm_mxfp8([dev(p) for p, _ in mats], [dev(s) for _, s in mats], rows, cols, codes, exps, dev(offsets))
    got = out.cpu().numpy()
    want = np.zeros((m, rows))
    plain = np.zeros((m, rows))
    for e in range(n_groups):
        W = oracle.mxfp4_dequant(mats[e][0], mats[e][1], rows, cols).astype(np.float64)
        for i in range(offsets[e], offsets[e + 1]):
            xr, _, _ = oracle.fp8_roundtrip(x[i], 32)
            want[i] = W @ xr.astype(np.float64)
            plain[i] = W @ x[i].astype(np.float64)
    return got, want, plain


@pytest.mark.parametrize("rows,cols,counts", [(64, 128, [16]), (128, 256, [3, 0, 17, 1]), (200, 1024, [70, 5]), (2048, 7168, [9, 24]),
                                              (7168, 2048, [16, 1, 40]), (300, 512, [0, 33, 32, 17, 64, 65]),
                                              # large groups: their 64-token passes are dealt to several workgroups
                                              (512, 1024, [300, 2, 130, 64]), (256, 512, [700])])
def test_grouped_gemm(rows, cols, counts):
    got, want, plain = run_case(rows, cols, counts, len(counts) + rows)
    assert rel_l2(got, want) <= 1e-5
    info = rel_l2(got, plain)
    assert info < 0.06  # the MXFP8 rounding of the activations, reported, not a parity claim


def test_matches_oracle_prefill_expert_section():
    # gate -> SwiGLU -> down for grouped tokens equals the oracle's moe_prefill with the MXFP8 rounding switched on
    torch = torch_cuda()
    from microkimi_amd import dequant, model, workloads
    d, inter, n_experts, T, topk = 256, 128, 4, 24, 2
    rng = np.random.default_rng(12)
    host = [(workloads.mxfp4_matrix(4, "w1", inter, d, e), workloads.mxfp4_matrix(4, "w3", inter, d, e),
             workloads.mxfp4_matrix(4, "w2", d, inter, e)) for e in range(n_experts)]
    table = oracle.ExpertTable([h[0] for h in host], [h[1] for h in host], [h[2] for h in host], d, inter)
    x = (rng.standard_normal((T, d)) * 0.05).astype(np.float32)
    ids = np.stack([rng.permutation(n_experts)[:topk] for _ in range(T)]).astype(np.uint32)
    wts = rng.random((T, topk)).astype(np.float32)
    want = oracle.moe_prefill(table, ids, wts, x, round_mxfp8=True)
    # group (token, slot) pairs by expert, in (token, slot) order inside a group, as the reference does
    flat = ids.reshape(-1)
    order = np.argsort(flat, kind="stable")
    counts = np.bincount(flat, minlength=n_experts)
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    xg = dev(x[order // topk])
    codes, exps = dequant.quantize_mxfp8(xg)
    dv = lambda k, j: [dev(h[k][j]) for h in host]
    g = model.grouped_gemm_mxfp8(dv(0, 0), dv(0, 1), inter, d, codes, exps, dev(offsets))
    u = model.grouped_gemm_mxfp8(dv(1, 0), dv(1, 1), inter, d, codes, exps, dev(offsets))
    act = (g / (1.0 + torch.exp(-g))) * u
    ac, ae = dequant.quantize_mxfp8(act)
    o = model.grouped_gemm_mxfp8(dv(2, 0), dv(2, 1), d, inter, ac, ae, dev(offsets)).cpu().numpy()
    outs = np.zeros((T * topk, d), np.float32)
    outs[order] = o
    got = (outs.reshape(T, topk, d) * wts[:, :, None]).sum(axis=1)
    # the activation is re-rounded to e4m3 after a device expf: a last-bit difference in exp can move a value across
    # a rounding boundary, so this end-to-end check is looser than the single-GEMM one
    assert rel_l2(got, want) <= 2e-3


@pytest.mark.parametrize("T,topk,n_experts,d,inter,act", [(24, 2, 4, 256, 128, "swiglu"), (40, 3, 7, 512, 256, "situ"), (5, 1, 3, 1024, 512, "swiglu")])
def test_moe_prefill_on_device(T, topk, n_experts, d, inter, act):
    # grouping, gather, the three grouped GEMMs, activation and combine all on the device (mk_dev_moe_prefill) against
    # the oracle's moe_prefill with the MXFP8 rounding switched on; the looser bound is the device expf in front of an
    # e4m3 rounding (see the test above)
    from microkimi_amd import model, workloads
    rng = np.random.default_rng(T * 7 + n_experts)
    host = [(workloads.mxfp4_matrix(4, "w1", inter, d, e), workloads.mxfp4_matrix(4, "w3", inter, d, e),
             workloads.mxfp4_matrix(4, "w2", d, inter, e)) for e in range(n_experts)]
    table = oracle.ExpertTable([h[0] for h in host], [h[1] for h in host], [h[2] for h in host], d, inter)
    x = (rng.standard_normal((T, d)) * 0.05).astype(np.float32)
    ids = np.stack([rng.permutation(n_experts)[:topk] for _ in range(T)]).astype(np.uint32)
    if n_experts > 4:
        ids[ids == 2] = 5  # an expert nobody selects
    wts = rng.random((T, topk)).astype(np.float32)
    kind = oracle.ACT_SITU if act == "situ" else oracle.ACT_SWIGLU
    want = oracle.moe_prefill(table, ids, wts, x, act_kind=kind, round_mxfp8=True)
    pk = lambda k: [(dev(h[k][0]), dev(h[k][1])) for h in host]
    experts = model.PackedExperts(pk(0), pk(1), pk(2), d, inter)
    got = model.moe_prefill(experts, dev(ids.astype(np.int32)), dev(wts), dev(x),
                            act_kind=model.ACT_SITU if act == "situ" else model.ACT_SWIGLU).cpu().numpy()
    assert np.all(np.isfinite(got))
    assert rel_l2(got, want) <= 2e-3
