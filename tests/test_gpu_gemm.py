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
    want = oracle.moe_prefill(table, ids, wts, x, round_mxfp8=2)
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


@pytest.mark.parametrize("T,topk,n_experts,d,inter,act", [(24, 2, 4, 256, 128, "swiglu"), (40, 3, 7, 512, 256, "situ"), (5, 1, 3, 1024, 512, "swiglu"),
                                                          # groups of about 50 and 75 tokens: several 32-token passes of the gate/up launch
                                                          (100, 2, 4, 512, 256, "swiglu"), (150, 2, 4, 1024, 384, "situ")])
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
    want = oracle.moe_prefill(table, ids, wts, x, act_kind=kind, round_mxfp8=2)
    pk = lambda k: [(dev(h[k][0]), dev(h[k][1])) for h in host]
    experts = model.PackedExperts(pk(0), pk(1), pk(2), d, inter)
    got = model.moe_prefill(experts, dev(ids.astype(np.int32)), dev(wts), dev(x), mxfp8=True,
                            act_kind=model.ACT_SITU if act == "situ" else model.ACT_SWIGLU).cpu().numpy()
    assert np.all(np.isfinite(got))
    assert rel_l2(got, want) <= 2e-3


@pytest.mark.parametrize("T,topk,n_experts,d,inter,act", [(24, 2, 4, 256, 128, "swiglu"), (40, 3, 7, 512, 256, "situ"), (5, 1, 3, 1024, 512, "swiglu"),
                                                          # groups of about 50 and 75 tokens: several 32-row passes per workgroup
                                                          (100, 2, 4, 512, 256, "swiglu"), (150, 2, 4, 1024, 384, "situ"),
                                                          # one group of exactly 16, 17, 32 and 33 rows (tile and pass boundaries)
                                                          (16, 1, 1, 256, 128, "swiglu"), (17, 1, 1, 256, 128, "swiglu"),
                                                          (32, 1, 1, 128, 256, "situ"), (33, 1, 1, 128, 256, "situ"),
                                                          # 48 and more rows a group: passes of 64 rows
                                                          (64, 1, 1, 256, 128, "swiglu"), (65, 1, 1, 256, 128, "swiglu"), (49, 1, 1, 128, 128, "situ")])
def test_moe_prefill_f32_on_device(T, topk, n_experts, d, inter, act):
    # the section in the reference's own arithmetic (mk_dev_moe_prefill_f32: f32 rows against the dequantized weights on
    # the f32 matrix instruction) against oracle.moe_prefill without any rounding; the order of the sums is the only
    # difference, hence 1e-5.  The stored intermediates are checked stage by stage as well.
    from microkimi_amd import model, workloads
    rng = np.random.default_rng(T * 11 + n_experts)
    host = [(workloads.mxfp4_matrix(4, "w1", inter, d, e), workloads.mxfp4_matrix(4, "w3", inter, d, e),
             workloads.mxfp4_matrix(4, "w2", d, inter, e)) for e in range(n_experts)]
    table = oracle.ExpertTable([h[0] for h in host], [h[1] for h in host], [h[2] for h in host], d, inter)
    x = (rng.standard_normal((T, d)) * 0.05).astype(np.float32)
    ids = np.stack([rng.permutation(n_experts)[:topk] for _ in range(T)]).astype(np.uint32)
    if n_experts > 4:
        ids[ids == 2] = 5  # an expert nobody selects
    wts = rng.random((T, topk)).astype(np.float32)
    kind = oracle.ACT_SITU if act == "situ" else oracle.ACT_SWIGLU
    want = oracle.moe_prefill(table, ids, wts, x, act_kind=kind, round_mxfp8=False)
    pk = lambda k: [(dev(h[k][0]), dev(h[k][1])) for h in host]
    experts = model.PackedExperts(pk(0), pk(1), pk(2), d, inter)
    got = model.moe_prefill(experts, dev(ids.astype(np.int32)), dev(wts), dev(x), act_kind=model.ACT_SITU if act == "situ" else model.ACT_SWIGLU,
                            exact=True).cpu().numpy()
    assert np.all(np.isfinite(got))
    assert rel_l2(got, want) <= 1e-5
    # stages: up rows and down rows per grouped row, in f64 from the dequantized weights
    mid = {k: v.cpu().numpy() for k, v in model.moe_prefill_intermediates(experts, T, topk).items()}
    order = np.argsort(ids.reshape(-1), kind="stable")
    assert np.array_equal(mid["order"], order.astype(np.int32))
    for r in range(0, T * topk, max(1, T * topk // 7)):
        e, t = int(ids.reshape(-1)[order[r]]), int(order[r]) // topk
        W3 = oracle.mxfp4_dequant(host[e][1][0], host[e][1][1], inter, d).astype(np.float64)
        W2 = oracle.mxfp4_dequant(host[e][2][0], host[e][2][1], d, inter).astype(np.float64)
        assert rel_l2(mid["u"][r], W3 @ x[t].astype(np.float64)) <= 1e-5
        assert rel_l2(mid["o"][r], W2 @ mid["g"][r].astype(np.float64)) <= 1e-5  # "g" holds ACT(gate, up) after this call


@pytest.mark.parametrize("rows,cols,counts,bf16", [(128, 512, [5, 0, 20, 33], False), (100, 256, [16, 17], False), (64, 1024, [3, 70], True),
                                                  (256, 512, [0, 0, 16, 1, 32, 0, 7, 9], True)])
def test_grouped_gemm_f32_and_bf16(rows, cols, counts, bf16):
    # the grouped products on their own (a caller that keeps its own grouping): every group's rows against the f64
    # product of its dequantized matrix and the rows (bf16: the rows as the kernel gets them), empty groups included
    torch = torch_cuda()
    from microkimi_amd import model, workloads
    rng = np.random.default_rng(rows + cols)
    mats = [workloads.mxfp4_matrix(4, "w1", rows, cols, e) for e in range(len(counts))]
    m = int(sum(counts))
    x = (rng.standard_normal((m, cols)) * 0.1).astype(np.float32)
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    xd = dev(x).to(torch.bfloat16).contiguous() if bf16 else dev(x)
    got = model.grouped_gemm_f32([dev(p) for p, _ in mats], [dev(s) for _, s in mats], rows, cols, xd, dev(offsets), bf16=bf16).cpu().numpy()
    xin = xd.to(torch.float32).cpu().numpy().astype(np.float64) if bf16 else x.astype(np.float64)
    for e, (p, s) in enumerate(mats):
        r0, r1 = int(offsets[e]), int(offsets[e + 1])
        if r1 > r0:
            Wd = oracle.mxfp4_dequant(p, s, rows, cols).astype(np.float64)
            assert rel_l2(got[r0:r1], xin[r0:r1] @ Wd.T) <= 1e-5, e


def decode_split(codes, exps):
    """The values a two-term row stands for: codes [m, kt, 2, 512] e4m3, exps [m, kt, 2, 16] e8m0 -> (hi + lo) [m, kt * 512] f64."""
    c = codes.astype(np.int32)
    e, mant = (c >> 3) & 15, c & 7
    v = np.where(e == 0, mant / 8.0 * 2.0 ** -6, (1 + mant / 8.0) * 2.0 ** (e - 7.0))
    v = np.where((c & 127) == 127, np.nan, v) * np.where(c & 128, -1.0, 1.0)
    m, kt = codes.shape[:2]
    v = v.reshape(m, kt, 2, 16, 32) * (2.0 ** (exps.astype(np.float64) - 127))[..., None]
    return (v[:, :, 0] + v[:, :, 1]).reshape(m, kt * 512)


def test_bf16_split_is_the_bfloat16_value():
    # mk_dev_quantize_bf16_split: hi + lo is bfloat16(x) exactly for every value within 2^13 of its block's largest,
    # and within 2^-17 of that largest value otherwise; zeros, a zero block, huge and tiny blocks; NaN / inf -> NaN
    torch = torch_cuda()
    from microkimi_amd import dequant
    rng = np.random.default_rng(11)
    n = 1024
    x = rng.standard_normal((40, n)).astype(np.float32)
    x[1] *= 1e-3
    x[2] *= 3e5
    x[3] = (x[3] * np.exp(rng.uniform(-30, 12, n))).astype(np.float32)       # 60 binades inside the blocks
    x[4, :32] = 0.0
    x[5] = np.float32(2.0) ** rng.integers(-20, 20, n).astype(np.float32)    # powers of two: lo is zero everywhere
    x[6] = (x[6] * 1e-30).astype(np.float32)
    x[7] = (x[7] * 1e30).astype(np.float32)
    x[8, ::7] = 0.0
    codes, exps = dequant.quantize_bf16_split(dev(x))
    got = decode_split(codes.cpu().numpy(), exps.cpu().numpy())
    want = bf16_round(x).astype(np.float64)
    blockmax = np.abs(want).reshape(40, n // 32, 32).max(axis=2, keepdims=True)
    near = (np.abs(want).reshape(40, n // 32, 32) >= blockmax * 2.0 ** -13).reshape(40, n)
    assert np.array_equal(got[near], want[near])
    slack = np.broadcast_to(blockmax * 2.0 ** -17, (40, n // 32, 32)).reshape(40, n)
    assert np.all(np.abs(got - want)[~near] <= slack[~near])
    assert near.mean() > 0.9 and (~near).sum() > 100   # both kinds of value were there
    y = x[:2].copy()
    y[0, 5], y[0, 40], y[1, 100] = np.inf, -np.inf, np.nan
    codes, exps = dequant.quantize_bf16_split(dev(y))
    got = decode_split(codes.cpu().numpy(), exps.cpu().numpy())
    assert np.isnan(got[0, 5]) and np.isnan(got[0, 40]) and np.isnan(got[1, 100])
    ok = near[:2].copy()
    ok[0, :64] = False   # (the blocks that hold an infinity: their other values underflow against it)
    ok[1, 100] = False
    assert np.array_equal(got[ok], bf16_round(y).astype(np.float64)[ok])


@pytest.mark.parametrize("rows,cols,counts", [(128, 512, [5, 0, 20, 33]), (64, 1024, [3, 70]), (256, 512, [0, 0, 16, 1, 32, 0, 7, 9]),
                                              (2048, 7168, [9, 24]), (7168, 2048, [16, 1, 40]), (300, 512, [1, 17, 65])])
def test_grouped_gemm_split(rows, cols, counts):
    # the two-term grouped product: every group's rows against the f64 product of its dequantized matrix and the
    # bfloat16-rounded rows; group sizes around the 16-row tile and the 32-row pass, empty groups, ragged weight rows
    torch_cuda()
    from microkimi_amd import dequant, model, workloads
    rng = np.random.default_rng(rows + cols)
    mats = [workloads.mxfp4_matrix(4, "w1", rows, cols, e) for e in range(len(counts))]
    m = int(sum(counts))
    x = rng.standard_normal((m, cols)).astype(np.float32)
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    codes, exps = dequant.quantize_bf16_split(dev(x))
    got = model.grouped_gemm_split([dev(p) for p, _ in mats], [dev(s) for _, s in mats], rows, cols, codes, exps, dev(offsets)).cpu().numpy()
    xin = bf16_round(x).astype(np.float64)
    for e, (p, s) in enumerate(mats):
        r0, r1 = int(offsets[e]), int(offsets[e + 1])
        if r1 > r0:
            Wd = oracle.mxfp4_dequant(p, s, rows, cols).astype(np.float64)
            want = xin[r0:r1] @ Wd.T
            # the block-scaled instruction keeps fewer bits of a step's 128 products than a chain of f32 additions would:
            # 1e-5 over a group, single rows up to a few times that
            assert rel_l2(got[r0:r1], want) <= 1.5e-5, e
            assert max(rel_l2(got[i], want[i - r0]) for i in range(r0, r1)) <= 4e-5, e
    with pytest.raises(Exception, match="512"):
        model.grouped_gemm_split([dev(mats[0][0])], [dev(mats[0][1])], rows, 256, codes, exps, dev(offsets[:2]))


_BF16_MFMA_SCRIPT = r"""
import sys
sys.path.insert(0, sys.argv[1]); sys.path.insert(0, sys.argv[1] + "/tests")
import numpy as np, oracle
from gpu_util import dev, rel_l2
from microkimi_amd import model, workloads
T, topk, ne, d, inter = 70, 2, 3, 1024, 512
rng = np.random.default_rng(5)
host = [(workloads.mxfp4_matrix(4, "w1", inter, d, e), workloads.mxfp4_matrix(4, "w3", inter, d, e), workloads.mxfp4_matrix(4, "w2", d, inter, e)) for e in range(ne)]
table = oracle.ExpertTable([h[0] for h in host], [h[1] for h in host], [h[2] for h in host], d, inter)
x = (rng.standard_normal((T, d)) * 0.05).astype(np.float32)
ids = np.stack([rng.permutation(ne)[:topk] for _ in range(T)]).astype(np.uint32)
wts = rng.random((T, topk)).astype(np.float32)
pk = lambda k: [(dev(h[k][0]), dev(h[k][1])) for h in host]
experts = model.PackedExperts(pk(0), pk(1), pk(2), d, inter)
got = model.moe_prefill(experts, dev(ids.astype(np.int32)), dev(wts), dev(x), bf16=True).cpu().numpy()
want = oracle.moe_prefill(table, ids, wts, x, round_mxfp8=3)
print("RESULT", rel_l2(got, want), int(np.isfinite(got).all()))
"""


def test_moe_prefill_bf16_on_the_bf16_matrix_instruction():
    # MK_PREFILL_BF16_MFMA=1 (read once per process, hence a process of its own): the same section on
    # v_mfma_f32_16x16x32_bf16 instead of the two-term form, against the same oracle
    import os
    import subprocess
    import sys
    torch_cuda()
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, MK_PREFILL_BF16_MFMA="1")
    r = subprocess.run([sys.executable, "-c", _BF16_MFMA_SCRIPT, root], env=env, capture_output=True, text=True, timeout=240)
    assert r.returncode == 0, r.stderr[-2000:]
    line = [l for l in r.stdout.splitlines() if l.startswith("RESULT")][-1].split()
    assert float(line[1]) <= 3e-4 and int(line[2]) == 1, line


def bf16_round(a):
    """bfloat16, round to nearest even, of an f32 array (as f32 values)."""
    b = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    b = ((b + 0x7FFF + ((b >> 16) & 1)) & 0xFFFF0000).astype(np.uint32)
    return b.view(np.float32).reshape(np.shape(a))


@pytest.mark.parametrize("T,topk,n_experts,d,inter,act", [(24, 2, 4, 512, 512, "swiglu"), (100, 2, 4, 1024, 512, "situ"), (5, 1, 3, 512, 1024, "swiglu"),
                                                          # one group of 16, 17, 32, 33 rows: tile and pass boundaries
                                                          (16, 1, 1, 512, 512, "swiglu"), (17, 1, 1, 512, 512, "situ"),
                                                          (32, 1, 1, 1024, 512, "swiglu"), (33, 1, 1, 512, 512, "swiglu")])
def test_moe_prefill_bf16_on_device(T, topk, n_experts, d, inter, act):
    # mk_dev_moe_prefill_bf16: hidden rows and activation rows rounded to bfloat16 once, exact weights, f32 products and
    # sums on the bf16 matrix instruction.
    #   gate / up rows  against the f64 product of the dequantized weights and the bf16-rounded hidden rows: 1e-5
    #   token rows      against oracle.moe_prefill(round_mxfp8=3) (the reference's loops on bf16-rounded inputs): 3e-4 --
    #                   the device's expf and the CPU's can differ in the last bit in front of a bfloat16 rounding
    #                   boundary of an activation value; one such step is 2^-8 of that value, about 1e-4 of a row of
    #                   2048 activations (config 4 measures 6e-5 on its worst token row)
    #   and the distance to the reference's own f32 arithmetic, which is the bfloat16 rounding of the two inputs
    from microkimi_amd import model, workloads
    rng = np.random.default_rng(T * 13 + n_experts)
    host = [(workloads.mxfp4_matrix(4, "w1", inter, d, e), workloads.mxfp4_matrix(4, "w3", inter, d, e),
             workloads.mxfp4_matrix(4, "w2", d, inter, e)) for e in range(n_experts)]
    table = oracle.ExpertTable([h[0] for h in host], [h[1] for h in host], [h[2] for h in host], d, inter)
    x = (rng.standard_normal((T, d)) * 0.05).astype(np.float32)
    ids = np.stack([rng.permutation(n_experts)[:topk] for _ in range(T)]).astype(np.uint32)
    wts = rng.random((T, topk)).astype(np.float32)
    kind = oracle.ACT_SITU if act == "situ" else oracle.ACT_SWIGLU
    want = oracle.moe_prefill(table, ids, wts, x, act_kind=kind, round_mxfp8=3)
    plain = oracle.moe_prefill(table, ids, wts, x, act_kind=kind, round_mxfp8=False)
    pk = lambda k: [(dev(h[k][0]), dev(h[k][1])) for h in host]
    experts = model.PackedExperts(pk(0), pk(1), pk(2), d, inter)
    got = model.moe_prefill(experts, dev(ids.astype(np.int32)), dev(wts), dev(x), act_kind=model.ACT_SITU if act == "situ" else model.ACT_SWIGLU,
                            bf16=True).cpu().numpy()
    assert np.all(np.isfinite(got))
    assert rel_l2(got, want) <= 3e-4
    assert rel_l2(got, plain) <= 6e-3
    mid = {k: v.cpu().numpy() for k, v in model.moe_prefill_intermediates(experts, T, topk).items()}
    order = np.argsort(ids.reshape(-1), kind="stable")
    for r in range(0, T * topk, max(1, T * topk // 7)):
        e, t = int(ids.reshape(-1)[order[r]]), int(order[r]) // topk
        xb = bf16_round(x[t]).astype(np.float64)
        for name, k in (("g", 0), ("u", 1)):
            Wd = oracle.mxfp4_dequant(host[e][k][0], host[e][k][1], inter, d).astype(np.float64)
            assert rel_l2(mid[name][r], Wd @ xb) <= 1e-5, (name, r)


@pytest.mark.parametrize("T,topk,n_experts,d,inter", [(40, 2, 4, 1024, 512), (300, 3, 5, 512, 1024)])
def test_moe_prefill_with_and_without_the_tile_ordered_scale_bytes(T, topk, n_experts, d, inter):
    # the MXFP8 and bf16 sections' kernels read the same scale bytes from either place: the same bits, intermediates included
    from microkimi_amd import model, workloads
    rng = np.random.default_rng(T + d)
    host = [(workloads.mxfp4_matrix(4, "w1", inter, d, e), workloads.mxfp4_matrix(4, "w3", inter, d, e),
             workloads.mxfp4_matrix(4, "w2", d, inter, e)) for e in range(n_experts)]
    pk = lambda k: [(dev(h[k][0]), dev(h[k][1])) for h in host]
    w1, w3, w2 = pk(0), pk(1), pk(2)
    x = dev((rng.standard_normal((T, d)) * 0.05).astype(np.float32))
    ids = dev(np.stack([rng.permutation(n_experts)[:topk] for _ in range(T)]).astype(np.int32))
    wts = dev(rng.random((T, topk)).astype(np.float32))
    res = []
    for tiles in (True, False):
        experts = model.PackedExperts(w1, w3, w2, d, inter, scales_by_tile=tiles)
        assert bool(experts.table.w1st) == tiles
        for keep in (False, True):
            out = model.moe_prefill(experts, ids, wts, x, mxfp8=True, keep=keep).cpu().numpy()
            mid = {k: v.cpu().numpy() for k, v in model.moe_prefill_intermediates(experts, T, topk).items()} if keep else {}
            res.append((out, mid))
        out = model.moe_prefill(experts, ids, wts, x, bf16=True).cpu().numpy()
        res.append((out, {k: v.cpu().numpy() for k, v in model.moe_prefill_intermediates(experts, T, topk).items()}))
    for (a, ma), (b, mb) in zip(res[:3], res[3:]):
        assert np.isfinite(a).all() and np.array_equal(a.view(np.uint32), b.view(np.uint32))
        for k in ma:
            assert np.array_equal(ma[k].view(np.uint32), mb[k].view(np.uint32)), k


def test_moe_prefill_bf16_non_finite_hidden_value_gives_nan_rows():
    # a hidden value that is not finite makes the token's row NaN (its e4m3 code is the NaN), the other tokens' rows stay as they were
    from microkimi_amd import model, workloads
    T, topk, n_experts, d, inter = 20, 2, 3, 512, 512
    rng = np.random.default_rng(9)
    host = [(workloads.mxfp4_matrix(4, "w1", inter, d, e), workloads.mxfp4_matrix(4, "w3", inter, d, e),
             workloads.mxfp4_matrix(4, "w2", d, inter, e)) for e in range(n_experts)]
    pk = lambda k: [(dev(h[k][0]), dev(h[k][1])) for h in host]
    experts = model.PackedExperts(pk(0), pk(1), pk(2), d, inter)
    x = (rng.standard_normal((T, d)) * 0.05).astype(np.float32)
    ids = dev(np.stack([rng.permutation(n_experts)[:topk] for _ in range(T)]).astype(np.int32))
    wts = dev(rng.random((T, topk)).astype(np.float32))
    clean = model.moe_prefill(experts, ids, wts, dev(x), bf16=True).cpu().numpy()
    x[3, 17], x[11, 400] = np.inf, np.nan
    got = model.moe_prefill(experts, ids, wts, dev(x), bf16=True).cpu().numpy()
    assert np.isnan(got[3]).all() and np.isnan(got[11]).all()
    others = [t for t in range(T) if t not in (3, 11)]
    assert np.array_equal(got[others].view(np.uint32), clean[others].view(np.uint32))


def test_moe_prefill_bf16_refuses_other_shapes():
    # d or inter not in multiples of 512, or a layer with VQ1 experts: MK_ERR_UNSUPPORTED, nothing computed
    from microkimi_amd import model, workloads
    d, inter = 256, 512
    host = [(workloads.mxfp4_matrix(4, "w1", inter, d, 0), workloads.mxfp4_matrix(4, "w3", inter, d, 0), workloads.mxfp4_matrix(4, "w2", d, inter, 0))]
    pk = lambda k: [(dev(h[k][0]), dev(h[k][1])) for h in host]
    experts = model.PackedExperts(pk(0), pk(1), pk(2), d, inter)
    x = np.zeros((4, d), np.float32)
    with pytest.raises(Exception, match="512"):
        model.moe_prefill(experts, dev(np.zeros((4, 1), np.int32)), dev(np.ones((4, 1), np.float32)), dev(x), bf16=True)


def test_moe_prefill_f32_random_shapes():
    # a dozen seeded random shapes (token counts, top-k, expert counts, d and inter in multiples of 128, both
    # activations; routing with repeats allowed across tokens only) against the oracle without rounding
    from microkimi_amd import model, workloads
    rng = np.random.default_rng(2024)
    for case in range(12):
        n_experts = int(rng.integers(1, 9))
        topk = int(rng.integers(1, min(n_experts, 4) + 1))
        T = int(rng.integers(1, 130))
        d, inter = 128 * int(rng.integers(1, 5)), 128 * int(rng.integers(1, 4))
        act = int(rng.integers(0, 2))
        host = [(workloads.mxfp4_matrix(4, "w1", inter, d, e), workloads.mxfp4_matrix(4, "w3", inter, d, e),
                 workloads.mxfp4_matrix(4, "w2", d, inter, e)) for e in range(n_experts)]
        table = oracle.ExpertTable([h[0] for h in host], [h[1] for h in host], [h[2] for h in host], d, inter)
        x = (rng.standard_normal((T, d)) * 0.05).astype(np.float32)
        ids = np.stack([rng.permutation(n_experts)[:topk] for _ in range(T)]).astype(np.uint32)
        wts = rng.random((T, topk)).astype(np.float32)
        want = oracle.moe_prefill(table, ids, wts, x, act_kind=act, round_mxfp8=False)
        pk = lambda k: [(dev(h[k][0]), dev(h[k][1])) for h in host]
        experts = model.PackedExperts(pk(0), pk(1), pk(2), d, inter)
        got = model.moe_prefill(experts, dev(ids.astype(np.int32)), dev(wts), dev(x), act_kind=act, exact=True).cpu().numpy()
        err = rel_l2(got, want)
        assert np.isfinite(got).all() and err <= 1e-5, (case, T, topk, n_experts, d, inter, act, err)


def test_moe_prefill_wrapper_splits_a_prompt_of_more_than_16384_pairs():
    # one C call takes at most 16384 (token, slot) pairs; the wrapper cuts a longer prompt into calls of whole tokens.
    # Tokens are independent, so the pieces are the rows of the separate calls, and a sample of rows is held to the oracle.
    from microkimi_amd import model, workloads
    from microkimi_amd._lib import MkError
    rng = np.random.default_rng(77)
    n_experts, topk, T, d, inter = 8, 8, 2100, 128, 128     # 16800 pairs: calls of 2048 and 52 tokens
    host = [(workloads.mxfp4_matrix(4, "w1", inter, d, e), workloads.mxfp4_matrix(4, "w3", inter, d, e),
             workloads.mxfp4_matrix(4, "w2", d, inter, e)) for e in range(n_experts)]
    x = (rng.standard_normal((T, d)) * 0.05).astype(np.float32)
    ids = np.stack([rng.permutation(n_experts)[:topk] for _ in range(T)]).astype(np.int32)
    wts = rng.random((T, topk)).astype(np.float32)
    pk = lambda k: [(dev(h[k][0]), dev(h[k][1])) for h in host]
    experts = model.PackedExperts(pk(0), pk(1), pk(2), d, inter)
    from microkimi_amd._lib import cur_stream, lib, ptr
    import ctypes as C
    import torch
    ws = torch.empty(lib.mk_moe_prefill_workspace_bytes(T, topk, n_experts, d, inter), dtype=torch.uint8, device="cuda")
    out = torch.empty((T, d), device="cuda")
    st = lib.mk_dev_moe_prefill_f32(C.byref(experts.table), n_experts, T, topk, ptr(dev(ids)), ptr(dev(wts)), ptr(dev(x)), 0, ptr(ws), ptr(out),
                                    cur_stream())
    assert st == -1 and b"16384" in lib.mk_last_error()      # the C call itself refuses
    got = model.moe_prefill(experts, dev(ids), dev(wts), dev(x)).cpu().numpy()
    a = model.moe_prefill(experts, dev(ids[:2048]), dev(wts[:2048]), dev(x[:2048])).cpu().numpy()
    b = model.moe_prefill(experts, dev(ids[2048:]), dev(wts[2048:]), dev(x[2048:])).cpu().numpy()
    assert np.array_equal(got[:2048], a) and np.array_equal(got[2048:], b)
    table = oracle.ExpertTable([h[0] for h in host], [h[1] for h in host], [h[2] for h in host], d, inter)
    rows = np.array([0, 1, 2047, 2048, 2049, 2099])
    want = oracle.moe_prefill(table, ids[rows].astype(np.uint32), wts[rows], x[rows], round_mxfp8=False)
    assert rel_l2(got[rows], want) <= 1e-5


@pytest.mark.parametrize("arith", ["mxfp8", "f32", "bf16"])
def test_moe_prefill_skips_ids_out_of_range(arith):
    # a pair whose expert id lies outside the table adds nothing to its token (include/mk_hip.h): the result equals the
    # oracle's with that pair pointed at a valid expert with routing weight 0; a token whose pairs are all out of range
    # comes out as zeros
    from microkimi_amd import model, workloads
    T, topk, n_experts, d, inter = 37, 3, 5, 512, 512
    exact = arith == "f32"
    rng = np.random.default_rng(5)
    host = [(workloads.mxfp4_matrix(4, "w1", inter, d, e), workloads.mxfp4_matrix(4, "w3", inter, d, e),
             workloads.mxfp4_matrix(4, "w2", d, inter, e)) for e in range(n_experts)]
    table = oracle.ExpertTable([h[0] for h in host], [h[1] for h in host], [h[2] for h in host], d, inter)
    x = (rng.standard_normal((T, d)) * 0.05).astype(np.float32)
    ids = np.stack([rng.permutation(n_experts)[:topk] for _ in range(T)]).astype(np.int32)
    wts = (rng.random((T, topk)) + 0.1).astype(np.float32)
    bad = rng.random((T, topk)) < 0.25
    bad[7, :] = True
    dev_ids = ids.copy()
    dev_ids[bad] = np.where(rng.random(int(bad.sum())) < 0.5, -1, n_experts + 2)
    ref_ids, ref_wts = ids.copy(), wts.copy()
    ref_wts[bad] = 0.0
    want = oracle.moe_prefill(table, ref_ids.astype(np.uint32), ref_wts, x, round_mxfp8={"f32": False, "mxfp8": 2, "bf16": 3}[arith])
    pk = lambda k: [(dev(h[k][0]), dev(h[k][1])) for h in host]
    experts = model.PackedExperts(pk(0), pk(1), pk(2), d, inter)
    got = model.moe_prefill(experts, dev(dev_ids), dev(wts), dev(x), exact=exact, bf16=arith == "bf16", mxfp8=arith == "mxfp8").cpu().numpy()
    assert np.all(np.isfinite(got)) and not got[7].any()
    assert rel_l2(got, want) <= {"f32": 1e-5, "mxfp8": 2e-3, "bf16": 3e-4}[arith]


@pytest.mark.parametrize("T,topk,d,inter,act", [(40, 3, 256, 128, 0), (90, 2, 512, 256, 1), (7, 1, 128, 384, 0)])
def test_moe_prefill_f32_with_vq1_experts(T, topk, d, inter, act):
    # moe_prefill over a layer that mixes MXFP4 and VQ1 ("cold") experts (src/model.rs:2556-2599: matvec_vq_nt for the
    # three products of a VQ1 expert, matvec_packed_nt for the others): experts 1, 3, 5 are VQ1.  The oracle is the
    # per-token form of the same layer in f32 (both nt functions keep their per-position terms; the order of the sums
    # is what differs on the device).  mk_dev_moe_prefill (MXFP8) still refuses such a layer.
    from microkimi_amd import model, workloads
    n_experts = 6
    rng = np.random.default_rng(T + d)
    codebook = (rng.standard_normal((256, 16)) * 0.05).astype(np.float32)
    host, devs = [], ([], [], [])
    for e in range(n_experts):
        if e % 2:
            idx = [rng.integers(0, 256, (inter, d // 16), dtype=np.uint8), rng.integers(0, 256, (inter, d // 16), dtype=np.uint8),
                   rng.integers(0, 256, (d, inter // 16), dtype=np.uint8)]
            host.append(("vq1", idx[0], idx[1], idx[2]))
            for k in range(3):
                devs[k].append((dev(idx[k]), None))
        else:
            m = [workloads.mxfp4_matrix(2, "w1", inter, d, e), workloads.mxfp4_matrix(2, "w3", inter, d, e),
                 workloads.mxfp4_matrix(2, "w2", d, inter, e)]
            host.append(("mxfp4", m[0], m[1], m[2]))
            for k in range(3):
                devs[k].append((dev(m[k][0]), dev(m[k][1])))
    experts = model.PackedExperts(devs[0], devs[1], devs[2], d, inter, vq_codebook=dev(codebook))
    ids = np.stack([rng.permutation(n_experts)[:topk] for _ in range(T)]).astype(np.int32)
    wts = rng.random((T, topk)).astype(np.float32)
    x = (rng.standard_normal((T, d)) * 0.05).astype(np.float32)
    want = oracle.moe_decode_mixed(host, codebook, d, inter, ids.astype(np.uint32), wts, x, shared=-1, mode=0, act_kind=act, limit=0.0)
    got = model.moe_prefill(experts, dev(ids), dev(wts), dev(x), act_kind=act, exact=True).cpu().numpy()
    assert np.isfinite(got).all() and np.isfinite(want).all()
    for t in range(T):
        assert rel_l2(got[t], want[t]) <= 1e-5, (t, rel_l2(got[t], want[t]))
    # the batched VQ1 product of the oracle on one expert's group: the up rows
    mid = {k: v.cpu().numpy() for k, v in model.moe_prefill_intermediates(experts, T, topk).items()}
    e = 3
    r0, r1 = int(mid["offsets"][e]), int(mid["offsets"][e + 1])
    toks = mid["order"][r0:r1] // topk
    m8 = (len(toks) + 7) // 8 * 8
    xt = np.zeros((d, m8), np.float32)
    xt[:, :len(toks)] = x[toks].T
    want_u = oracle.vq1_matvec_nt(codebook, host[e][2], inter, d, xt, m8)[:len(toks)]
    assert len(toks) > 0 and rel_l2(mid["u"][r0:r1], want_u) <= 1e-5
    with pytest.raises(Exception):
        model.moe_prefill(experts, dev(ids), dev(wts), dev(x), act_kind=act, mxfp8=True)


def test_config4_full_size_expert_section():
    """Configuration 4 at its full size: 512 prompt tokens routed top-8 (seeded logits, uneven groups) over 256
    experts of 2048 x 7168 / 7168 x 2048 (6 GB of MXFP4 drawn on the device), mk_dev_moe_prefill end to end.

      grouping   order / pos / offsets of the device's counting sort equal a host stable sort by expert id exactly
                 (the reference fills its groups in (token, slot) order, src/model.rs:2539-2544)
      gate, up   every row of three sampled experts against the f64 product of the dequantized weights and the
                 MXFP8-rounded hidden rows (the inputs the matrix cores see): relative L2 <= 1e-5
      down rows  every row of the same experts against oracle.moe_prefill(round_mxfp8=2: MXFP8 inputs, full scale range) run on that expert alone
      tokens     the output rows of ten sampled tokens against oracle.moe_prefill(round_mxfp8=2: MXFP8 inputs, full scale range), which gets the
                 eight experts of that token; the distance to the reference's own arithmetic (pure f32
                 matvec_packed_nt) is reported beside it
      bf16 mode  mk_dev_moe_prefill_bf16 on the same weights: gate rows of two experts against the f64 product with the
                 bf16-rounded hidden rows (1e-5), the ten token rows against the oracle on bf16-rounded inputs (3e-4)
      f32 mode   mk_dev_moe_prefill_f32 on the same weights: the up and down rows of two experts and the same ten
                 token rows against the oracle without rounding (the reference's arithmetic): relative L2 <= 1e-5
    The looser bound on the last two is one e4m3 rounding step of the activation (2^-4 relative) where the device's
    expf and the CPU's differ in the last bit in front of a rounding boundary: see test_moe_prefill_on_device."""
    torch = torch_cuda()
    from microkimi_amd import model, workloads as W
    d, inter, ne, topk = W.D_MODEL, W.D_INTER, W.N_EXPERTS, W.TOP_K
    g = torch.Generator(device="cuda").manual_seed(44)

    def draw(rows, cols):
        return (torch.randint(0, 256, (rows, cols // 2), dtype=torch.uint8, device="cuda", generator=g),
                torch.randint(118, 131, (rows, cols // 32), dtype=torch.uint8, device="cuda", generator=g))

    w1 = [draw(inter, d) for _ in range(ne)]
    w3 = [draw(inter, d) for _ in range(ne)]
    w2 = [draw(d, inter) for _ in range(ne)]
    experts = model.PackedExperts(w1, w3, w2, d, inter)
    logits, x = W.config4_tokens()
    T = x.shape[0]
    ids, wts = model.router_softmax_topk(dev(logits), topk)
    plain = model.moe_prefill(experts, ids, wts, dev(x), mxfp8=True).cpu().numpy()
    got = model.moe_prefill(experts, ids, wts, dev(x), mxfp8=True, keep=True).cpu().numpy()   # the same kernels, gate / up rows stored as well
    assert np.isfinite(got).all() and np.array_equal(plain.view(np.uint32), got.view(np.uint32))
    mid = {k: v.cpu().numpy() for k, v in model.moe_prefill_intermediates(experts, T, topk).items()}
    ids_h, wts_h = ids.cpu().numpy(), wts.cpu().numpy()

    # ---- grouping, exactly
    flat = ids_h.reshape(-1)
    order = np.argsort(flat, kind="stable").astype(np.int32)
    counts = np.bincount(flat, minlength=ne)
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    assert counts.max() > 16 and counts.min() < 16, "the seeded routing is meant to be uneven"
    assert np.array_equal(mid["offsets"], offsets)
    assert np.array_equal(mid["order"], order)
    pos = np.empty(T * topk, np.int32)
    pos[order] = np.arange(T * topk, dtype=np.int32)
    assert np.array_equal(mid["pos"], pos)

    host = lambda pair: (pair[0].cpu().numpy(), pair[1].cpu().numpy())
    # ---- three experts, all their rows: the largest group, the smallest non-empty one and one in between
    by_size = np.argsort(counts, kind="stable")
    nonempty = [int(e) for e in by_size if counts[e] > 0]
    for e in (nonempty[-1], nonempty[0], nonempty[len(nonempty) // 2]):
        r0, r1 = int(offsets[e]), int(offsets[e + 1])
        toks = order[r0:r1] // topk
        h1, h3, h2 = host(w1[e]), host(w3[e]), host(w2[e])
        xr = np.stack([oracle.fp8_roundtrip(x[t], 32)[0] for t in toks]).astype(np.float64)
        for name, hw in (("g", h1), ("u", h3)):
            Wd = oracle.mxfp4_dequant(hw[0], hw[1], inter, d).astype(np.float64)
            want = xr @ Wd.T
            err = rel_l2(mid[name][r0:r1], want)
            assert err <= 1e-5, f"expert {e} ({r1 - r0} rows) {name}: {err:.2e}"
        table = oracle.ExpertTable([h1], [h3], [h2], d, inter)
        m = r1 - r0
        want_o = oracle.moe_prefill(table, np.zeros((m, 1), np.uint32), np.ones((m, 1), np.float32), x[toks], round_mxfp8=2)
        err = rel_l2(mid["o"][r0:r1], want_o)
        assert err <= 2e-3, f"expert {e}: down rows {err:.2e}"

    # ---- the same section in the reference's own arithmetic (mk_dev_moe_prefill_f32), against the oracle without rounding
    got_f32 = model.moe_prefill(experts, ids, wts, dev(x), exact=True).cpu().numpy()
    assert np.isfinite(got_f32).all()
    mid32 = {k: v.cpu().numpy() for k, v in model.moe_prefill_intermediates(experts, T, topk).items()}
    assert np.array_equal(mid32["order"], order) and np.array_equal(mid32["offsets"], offsets)
    for e in (nonempty[-1], nonempty[0]):
        r0, r1 = int(offsets[e]), int(offsets[e + 1])
        toks = order[r0:r1] // topk
        table = oracle.ExpertTable([host(w1[e])], [host(w3[e])], [host(w2[e])], d, inter)
        m = r1 - r0
        want_o = oracle.moe_prefill(table, np.zeros((m, 1), np.uint32), np.ones((m, 1), np.float32), x[toks], round_mxfp8=False)
        err = rel_l2(mid32["o"][r0:r1], want_o)
        assert err <= 1e-5, f"expert {e}: f32 down rows {err:.2e}"
        Wd = oracle.mxfp4_dequant(*host(w3[e]), inter, d).astype(np.float64)
        err = rel_l2(mid32["u"][r0:r1], x[toks].astype(np.float64) @ Wd.T)
        assert err <= 1e-5, f"expert {e}: f32 up rows {err:.2e}"

    # ---- the bf16 section (mk_dev_moe_prefill_bf16) on the same weights
    got_bf16 = model.moe_prefill(experts, ids, wts, dev(x), bf16=True).cpu().numpy()
    assert np.isfinite(got_bf16).all()
    mid16 = {k: v.cpu().numpy() for k, v in model.moe_prefill_intermediates(experts, T, topk).items()}
    for e in (nonempty[-1], nonempty[0]):
        r0, r1 = int(offsets[e]), int(offsets[e + 1])
        toks = order[r0:r1] // topk
        Wd = oracle.mxfp4_dequant(*host(w1[e]), inter, d).astype(np.float64)
        err = rel_l2(mid16["g"][r0:r1], bf16_round(x[toks]).astype(np.float64) @ Wd.T)
        assert err <= 1e-5, f"expert {e}: bf16 gate rows {err:.2e}"

    # ---- ten tokens end to end
    worst, worst_f32, worst_exact, worst_bf16, worst_bf16_f32 = 0.0, 0.0, 0.0, 0.0, 0.0
    for tok in (0, 1, 63, 64, 127, 200, 255, 256, 400, 511):
        used = [int(e) for e in ids_h[tok]]
        table = oracle.ExpertTable([host(w1[e]) for e in used], [host(w3[e]) for e in used], [host(w2[e]) for e in used], d, inter)
        lid = np.arange(topk, dtype=np.uint32)[None, :]
        want = oracle.moe_prefill(table, lid, wts_h[tok:tok + 1], x[tok:tok + 1], round_mxfp8=2)
        plain = oracle.moe_prefill(table, lid, wts_h[tok:tok + 1], x[tok:tok + 1], round_mxfp8=False)
        worst = max(worst, rel_l2(got[tok], want[0]))
        worst_f32 = max(worst_f32, rel_l2(got[tok], plain[0]))
        worst_exact = max(worst_exact, rel_l2(got_f32[tok], plain[0]))
        want16 = oracle.moe_prefill(table, lid, wts_h[tok:tok + 1], x[tok:tok + 1], round_mxfp8=3)
        worst_bf16 = max(worst_bf16, rel_l2(got_bf16[tok], want16[0]))
        worst_bf16_f32 = max(worst_bf16_f32, rel_l2(got_bf16[tok], plain[0]))
    print(f"config 4 full size: worst token row vs MXFP8 oracle {worst:.2e}, vs the pure-f32 reference path {worst_f32:.2e}")
    print(f"config 4 full size, f32 mode: worst token row vs the pure-f32 reference path {worst_exact:.2e}")
    print(f"config 4 full size, bf16 mode: worst token row vs the bf16-input oracle {worst_bf16:.2e}, vs the pure-f32 reference path {worst_bf16_f32:.2e}")
    assert worst <= 2e-3
    # bf16 mode against the oracle on bf16-rounded rows: what is left is activation values whose bfloat16 rounding falls
    # the other way (one such value moves its row by 2^-9 of that value).  The gate and up rows carry 5e-6 of arithmetic
    # noise here (the block-scaled matrix instruction adds into its accumulator by truncation) where the bfloat16 matrix
    # instruction (MK_PREFILL_BF16_MFMA=1) carries 3e-7, so more values fall the other way: 4.3e-4 against 6.3e-5
    # measured.  The distance to the f32 reference, which is the rounding to bfloat16 itself, is the same for both: 1.7e-3.
    assert worst_bf16 <= 8e-4 and worst_bf16_f32 <= 3e-3
    assert worst_exact <= 1e-5
    assert worst_f32 < 0.06  # the e4m3 rounding of the activations: reported, not a parity claim
