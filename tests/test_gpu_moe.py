"""GPU parity, MoE decode layer and router (mk_dev_moe_decode, mk_dev_router_softmax_topk) against the oracle."""
import numpy as np
import pytest

import oracle
from gpu_util import dev, rel_l2, torch_cuda

pytestmark = pytest.mark.gpu
TOL = 1e-5


def rows_match_up_to_q8_flips(got, want, w2_of_token, d, inter, max_flips=2):
    """The layer re-quantizes the f32 activation to q8 before W2 (matvec_packed's own step, src/mxfp4.rs:476-479), a
    step function of its input: the gate/up sums here differ from the CPU's in their last bits (the order of the sum
    over blocks, expf), so an activation that lies within a few ulp of a rounding boundary takes the other int8 value
    (about one activation in 60 000).  Such a flip changes the token's row by exactly one column of that expert's W2
    times one quantization step (4e-5 .. 4e-4 of the row).  Returns the number of such single-column differences
    removed; asserts that a row needs at most max_flips of them and agrees to TOL otherwise."""
    torch = torch_cuda()
    from microkimi_amd import mxfp4
    flips = 0
    for t in range(got.shape[0]):
        diff = torch.from_numpy(got[t].astype(np.float64) - want[t].astype(np.float64)).cuda()
        wn = float(np.linalg.norm(want[t]))
        raw = float(diff.norm()) / wn  # before any column is removed
        for _ in range(max_flips):
            if float(diff.norm()) / wn <= TOL:
                break
            best = None
            for p, sc in w2_of_token(t):
                Wd = mxfp4.dequant(p, sc, d, inter).double()
                c = (Wd.T @ diff) / (Wd.norm(dim=0) * diff.norm())
                j = int(c.abs().argmax())
                if best is None or abs(float(c[j])) > abs(best[0]):
                    best = (float(c[j]), Wd[:, j].clone())
            assert abs(best[0]) > 0.7, f"token {t}: raw rel-L2 {raw:.2e}; a difference of {float(diff.norm()) / wn:.2e} that is not a q8 step of one activation"
            diff = diff - best[1] * (best[1] @ diff) / (best[1] @ best[1])
            flips += 1
        assert float(diff.norm()) / wn <= TOL, f"token {t}: raw rel-L2 {raw:.2e}, {float(diff.norm()) / wn:.2e} after {flips} single-column steps"
    return flips


def build(n_experts, d, inter, cfg=2, pack=None):
    from microkimi_amd import model, workloads
    host = [(workloads.mxfp4_matrix(cfg, "w1", inter, d, e), workloads.mxfp4_matrix(cfg, "w3", inter, d, e),
             workloads.mxfp4_matrix(cfg, "w2", d, inter, e)) for e in range(n_experts)]
    w1 = [h[0] for h in host]
    w3 = [h[1] for h in host]
    w2 = [h[2] for h in host]
    table = oracle.ExpertTable(w1, w3, w2, d, inter)
    todev = lambda lst: [(dev(p), dev(s)) for p, s in lst]
    experts = model.PackedExperts(todev(w1), todev(w3), todev(w2), d, inter, pack=pack)
    return table, experts


def table_host(table, k):
    """The (packed, scales) host arrays of matrix k (0 = w1, 1 = w3, 2 = w2) of every expert of an oracle table."""
    n = table.n
    return [(table._keep[(k * n + e) * 2], table._keep[(k * n + e) * 2 + 1]) for e in range(n)]


@pytest.mark.parametrize("d,inter,n_experts,B,topk,shared,act", [
    (7168, 2048, 12, 1, 8, 11, 0),    # benchmark layer shapes, batch 1, shared expert
    (7168, 2048, 12, 4, 8, 11, 0),    # batch 4 (the smallest batch on the batched path)
    (7168, 2048, 12, 3, 8, 11, 0),    # batch 3 (one-launch path)
    (2048, 1024, 6, 3, 2, -1, 1),     # SiTU (K3 rule), no shared expert
    (4096, 2048, 5, 2, 3, 4, 2),      # DeepSeek rule: clamp, weight before W2, plain sum
    (1024, 512, 4, 16, 2, 3, 0),      # batch 16
    (7168, 2048, 12, 9, 8, 11, 0),    # benchmark shapes, two token groups in the gate/up kernel (8 + 1)
    (1024, 4096, 4, 5, 2, 3, 0),      # two rows of W1/W3 per wave
    (96, 64, 4, 2, 2, -1, 0),         # shape off the fast path (composed kernels)
    (2048, 1024, 6, 8, 2, -1, 1),     # batched path (4 tokens and more: pairs grouped by expert), SiTU, no shared expert
    (4096, 2048, 5, 11, 3, 4, 2),     # batched path, DeepSeek rule, groups of more than four tokens (several passes)
    (7168, 2048, 12, 16, 8, 11, 0),   # batched path at the benchmark layer's shapes, batch 16
    (1024, 512, 4, 5, 3, -1, 0),      # batched path, an odd number of pairs
    (7168, 2048, 12, 2, 8, 11, 100),  # hidden ~ N(0, 1) as the benchmark configuration states (saturated silu), one-launch path
    (7168, 2048, 12, 8, 8, 11, 100),  # the same on the batched path
])
def test_moe_decode_q8(d, inter, n_experts, B, topk, shared, act):
    hs = 0.02
    if act >= 100:  # marker: full-scale hidden state, SwiGLU
        act, hs = act - 100, 1.0
    torch = torch_cuda()
    from microkimi_amd import model
    table, experts = build(n_experts, d, inter)
    rng = np.random.default_rng(B * 100 + d)
    n_routed = n_experts - (1 if shared >= 0 else 0)
    ids = np.stack([rng.permutation(n_routed)[:topk] for _ in range(B)]).astype(np.int32)
    wts = rng.random((B, topk)).astype(np.float32)
    wts /= wts.sum(axis=1, keepdims=True)
    # most cases use a small hidden state (|g| of a few units: the curved part of the activation); the last two use
    # N(0, 1) as the benchmark configuration states, where |g| reaches hundreds and silu saturates
    x = (rng.standard_normal((B, d)) * hs).astype(np.float32)
    limit = 10.0 if act == 2 else 0.0
    got = model.moe_decode(experts, dev(ids), dev(wts), dev(x), shared=shared, mode=1, act_kind=act, limit=limit).cpu().numpy()
    want = oracle.moe_decode(table, ids.astype(np.uint32), wts, x, shared=shared, mode=1, act_kind=act, limit=limit, threads=8)
    assert np.isfinite(want).all()
    w2_dev = experts._keep[2]
    used = lambda t: [w2_dev[int(e)] for e in ids[t]] + ([w2_dev[shared]] if shared >= 0 else [])
    flips = rows_match_up_to_q8_flips(got, want, used, d, inter)
    assert flips <= max(1, B // 3)


STAGE_CASES = [
    # d, inter, n_experts, B, topk, shared, act, hidden scale
    (7168, 2048, 12, 1, 8, 11, 0, 1.0),    # benchmark layer shapes, batch 1 (one-launch path), hidden ~ N(0, 1)
    (7168, 2048, 12, 3, 8, 11, 0, 1.0),    # batch 3
    (7168, 2048, 12, 4, 8, 11, 0, 1.0),    # batch 4: batched path (pairs grouped by expert, matrix cores)
    (7168, 2048, 12, 16, 8, 11, 0, 1.0),   # batch 16
    (2048, 1024, 6, 3, 2, -1, 1, 0.05),    # SiTU, no shared expert
    (4096, 2048, 5, 11, 3, 4, 2, 0.05),    # DeepSeek rule on the batched path (weight inside the activation)
    (4096, 2048, 5, 2, 3, 4, 2, 1.0),      # DeepSeek rule, clamp active at hidden ~ N(0, 1)
    (96, 64, 4, 2, 2, -1, 0, 1.0),         # composed path
    (5120, 2048, 6, 2, 3, 5, 1, 0.05),     # the one-launch kernel's other hidden width (20 rows of W2 a workgroup), SiTU
    (5120, 2048, 6, 3, 4, -1, 2, 1.0),     # the same, DeepSeek rule, no shared expert
]


def stage_inputs(d, inter, n_experts, B, topk, shared, hs):
    rng = np.random.default_rng(B * 1000 + d + inter)
    n_routed = n_experts - (1 if shared >= 0 else 0)
    ids = np.stack([rng.permutation(n_routed)[:topk] for _ in range(B)]).astype(np.int32)
    wts = rng.random((B, topk)).astype(np.float32)
    wts /= wts.sum(axis=1, keepdims=True)
    x = (rng.standard_normal((B, d)) * hs).astype(np.float32)
    return ids, wts, x


def oracle_act_rows(host, ids, wts, x, shared, d, inter, mode, act, limit):
    """ACT(W1 x, W3 x) of every (token, slot) pair from the oracle (two matvec_packed calls and the activation)."""
    B, topk = ids.shape
    per = topk + (1 if shared >= 0 else 0)
    want = np.empty((B, per, inter), np.float32)
    for t in range(B):
        for s in range(per):
            e = int(ids[t, s]) if s < topk else shared
            wgt = float(wts[t, s]) if s < topk else 1.0
            want[t, s] = oracle.expert_act(host[0][e], host[1][e], d, inter, x[t], mode=mode, act_kind=act, limit=limit, wgt=wgt)
    return want


@pytest.mark.parametrize("d,inter,n_experts,B,topk,shared,act,hs", STAGE_CASES)
def test_stage_gate_up_activation_without_exemption(d, inter, n_experts, B, topk, shared, act, hs):
    """First half of the layer alone: the f32 activation rows ACT(W1 x, W3 x) (two matvec_packed calls per pair in q8
    mode, src/model.rs:2246-2252) against the oracle, every row to TOL -- nothing is removed or exempted here."""
    from microkimi_amd import model
    table, experts = build(n_experts, d, inter)
    host = (table_host(table, 0), table_host(table, 1))
    ids, wts, x = stage_inputs(d, inter, n_experts, B, topk, shared, hs)
    limit = 10.0 if act == 2 else 0.0
    got = model.moe_decode_act(experts, dev(ids), dev(wts), dev(x), shared=shared, mode=1, act_kind=act, limit=limit).cpu().numpy()
    want = oracle_act_rows(host, ids, wts, x, shared, d, inter, 1, act, limit)
    assert np.isfinite(want).all() and np.isfinite(got).all()
    worst = max(rel_l2(got[t, s], want[t, s]) for t in range(B) for s in range(got.shape[1]))
    assert worst <= TOL, f"worst activation row rel-L2 {worst:.2e}"


@pytest.mark.parametrize("d,inter,n_experts,B,topk,shared,act,hs", STAGE_CASES)
def test_stage_down_from_oracle_activation_without_exemption(d, inter, n_experts, B, topk, shared, act, hs):
    """Second half alone: the device gets the ORACLE's f32 activation rows, re-quantizes them per 32 as matvec_packed
    does for W2 (bit-exact, so both sides multiply the same int8 blocks), and its rows must equal the oracle's layer
    output to TOL with nothing removed."""
    from microkimi_amd import model
    table, experts = build(n_experts, d, inter)
    host = (table_host(table, 0), table_host(table, 1))
    ids, wts, x = stage_inputs(d, inter, n_experts, B, topk, shared, hs)
    limit = 10.0 if act == 2 else 0.0
    act_rows = oracle_act_rows(host, ids, wts, x, shared, d, inter, 1, act, limit)
    got = model.moe_decode_from_act(experts, dev(ids), dev(wts), dev(act_rows), shared=shared, mode=1, act_kind=act).cpu().numpy()
    want = oracle.moe_decode(table, ids.astype(np.uint32), wts, x, shared=shared, mode=1, act_kind=act, limit=limit, threads=8)
    worst = max(rel_l2(got[t], want[t]) for t in range(B))
    assert worst <= TOL, f"worst row rel-L2 {worst:.2e}"


def test_stages_compose_to_the_layer():
    # act -> from_act on the device's own activation rows is the layer bit for bit (same kernels, same order)
    from microkimi_amd import model
    for d, inter, n_experts, B, topk, shared, act, hs in STAGE_CASES[:4]:
        table, experts = build(n_experts, d, inter)
        ids, wts, x = stage_inputs(d, inter, n_experts, B, topk, shared, hs)
        a = model.moe_decode_act(experts, dev(ids), dev(wts), dev(x), shared=shared, mode=1, act_kind=act)
        two = model.moe_decode_from_act(experts, dev(ids), dev(wts), a, shared=shared, mode=1, act_kind=act).cpu().numpy()
        one = model.moe_decode(experts, dev(ids), dev(wts), dev(x), shared=shared, mode=1, act_kind=act).cpu().numpy()
        assert np.array_equal(one.view(np.uint32), two.view(np.uint32)), (d, inter, B)


def pack_gate_up_np(p1, s1, p3, s3, d, inter):
    """The gate/up pack as include/mk_hip.h states it, element by element."""
    nb = d // 32
    out = np.zeros(2 * inter * nb * 17, np.uint8)
    r, b = np.meshgrid(np.arange(inter), np.arange(nb), indexing="ij")
    ci = (r >> 3) * (nb >> 2) + (b >> 2)
    base = (ci >> 1) * 2176
    for m, (p, s) in enumerate(((p1, s1), (p3, s3))):
        lane = (r & 7) + 8 * m + 16 * (b & 3)
        at = (base + (ci & 1) * 1024 + 16 * lane)[..., None] + np.arange(16)
        out[at.reshape(-1)] = p.reshape(inter, nb, 16).reshape(-1)
        out[(base + 2048 + 2 * lane + (ci & 1)).reshape(-1)] = s.reshape(-1)
    return out


def pack_down_np(p2, s2, d, inter):
    """The down pack as include/mk_hip.h states it, element by element (padding zero)."""
    nbi, rw = inter // 32, d // 256
    rb = rw - 16
    step = (1024 + 64 * rb + 64 + 4 * rb + 127) // 128 * 128
    out = np.zeros(256 * (inter // 128) * step, np.uint8)
    r, b = np.meshgrid(np.arange(d), np.arange(nbi), indexing="ij")
    c, i, kb = r // rw, r % rw, b & 3
    base = (c * (nbi >> 2) + (b >> 2)) * step
    noff = np.where(i < 16, 16 * (i + 16 * kb), 1024 + 16 * (kb * rb + i - 16))
    soff = 1024 + 64 * rb + np.where(i < 16, i + 16 * kb, 64 + kb * rb + i - 16)
    at = (base + noff)[..., None] + np.arange(16)
    out[at.reshape(-1)] = p2.reshape(d, nbi, 16).reshape(-1)
    out[(base + soff).reshape(-1)] = s2.reshape(-1)
    return out


@pytest.mark.parametrize("d,inter", [(7168, 2048), (5120, 2048), (4608, 256)])
def test_packed_copies_are_the_same_matrices_byte_for_byte(d, inter):
    # the experts in the one-launch kernel's order: the bytes sit where the header says, unpacking restores the reference
    # layout byte for byte, and dequant of the restored matrices is mxfp4::dequant bit for bit
    torch = torch_cuda()
    from microkimi_amd import mxfp4
    from microkimi_amd._lib import check, lib, ptr
    rng = np.random.default_rng(d + inter)
    draw = lambda rows, cols: (rng.integers(0, 256, (rows, cols // 2), dtype=np.uint8), rng.integers(0, 256, (rows, cols // 32), dtype=np.uint8))
    (p1, s1), (p3, s3), (p2, s2) = draw(inter, d), draw(inter, d), draw(d, inter)  # every nibble and every scale byte
    dv = [dev(x) for x in (p1, s1, p3, s3, p2, s2)]
    pk13 = torch.empty(lib.mk_moe_pack_bytes(d, inter, 0), dtype=torch.uint8, device="cuda")
    pk2 = torch.full((lib.mk_moe_pack_bytes(d, inter, 1),), 0xAB, dtype=torch.uint8, device="cuda")
    check(lib.mk_dev_moe_pack_gate_up(ptr(dv[0]), ptr(dv[1]), ptr(dv[2]), ptr(dv[3]), d, inter, ptr(pk13), None))
    check(lib.mk_dev_moe_pack_down(ptr(dv[4]), ptr(dv[5]), d, inter, ptr(pk2), None))
    assert np.array_equal(pk13.cpu().numpy(), pack_gate_up_np(p1, s1, p3, s3, d, inter))
    assert np.array_equal(pk2.cpu().numpy(), pack_down_np(p2, s2, d, inter))
    back = [torch.zeros_like(t) for t in dv]
    check(lib.mk_dev_moe_unpack_gate_up(ptr(pk13), d, inter, ptr(back[0]), ptr(back[1]), ptr(back[2]), ptr(back[3]), None))
    check(lib.mk_dev_moe_unpack_down(ptr(pk2), d, inter, ptr(back[4]), ptr(back[5]), None))
    for t, h in zip(back, (p1, s1, p3, s3, p2, s2)):
        assert np.array_equal(t.cpu().numpy(), h)
    got = mxfp4.dequant(back[4], back[5], d, inter).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), oracle.mxfp4_dequant(p2, s2, d, inter).view(np.uint32))


TWO_LAUNCH_CASES = [
    (7168, 2048, 12, 1, 8, 11, 0, 1.0),   # benchmark layer shapes, batch 1
    (7168, 2048, 12, 3, 8, 11, 0, 1.0),   # batch 3
    (2048, 1024, 6, 3, 2, -1, 1, 0.05),   # SiTU, no shared expert
    (4096, 2048, 5, 2, 3, 4, 2, 1.0),     # DeepSeek rule, clamp active
    (1024, 4096, 4, 3, 2, 3, 0, 0.02),    # two rows of W1/W3 per wave
]


@pytest.mark.parametrize("d,inter,n_experts,B,topk,shared,act,hs", TWO_LAUNCH_CASES)
def test_two_launch_path_without_the_packed_copies(d, inter, n_experts, B, topk, shared, act, hs):
    """A table without the packed copies takes the gate/up launch and the down launch (up to 3 tokens): both stages
    against the oracle to TOL with nothing removed, the stages compose to the layer bit for bit, and (where the one-launch
    kernel takes the shape) that kernel fed the same activation rows adds the same block terms in another order."""
    from microkimi_amd import model
    table, experts = build(n_experts, d, inter, pack=False)
    assert experts.table.w2t is None
    host = (table_host(table, 0), table_host(table, 1))
    ids, wts, x = stage_inputs(d, inter, n_experts, B, topk, shared, hs)
    limit = 10.0 if act == 2 else 0.0
    a = model.moe_decode_act(experts, dev(ids), dev(wts), dev(x), shared=shared, mode=1, act_kind=act, limit=limit)
    want_a = oracle_act_rows(host, ids, wts, x, shared, d, inter, 1, act, limit)
    got_a = a.cpu().numpy()
    worst = max(rel_l2(got_a[t, s], want_a[t, s]) for t in range(B) for s in range(got_a.shape[1]))
    assert worst <= TOL, f"worst activation row rel-L2 {worst:.2e}"
    want = oracle.moe_decode(table, ids.astype(np.uint32), wts, x, shared=shared, mode=1, act_kind=act, limit=limit, threads=8)
    got = model.moe_decode_from_act(experts, dev(ids), dev(wts), dev(want_a), shared=shared, mode=1, act_kind=act).cpu().numpy()
    worst = max(rel_l2(got[t], want[t]) for t in range(B))
    assert worst <= TOL, f"worst row rel-L2 {worst:.2e}"
    two = model.moe_decode_from_act(experts, dev(ids), dev(wts), a, shared=shared, mode=1, act_kind=act).cpu().numpy()
    one = model.moe_decode(experts, dev(ids), dev(wts), dev(x), shared=shared, mode=1, act_kind=act, limit=limit).cpu().numpy()
    assert np.array_equal(one.view(np.uint32), two.view(np.uint32))
    if d == 7168 and inter == 2048:
        # the one-launch kernel on the same inputs: the same block terms, added in another order
        _, packed = build(n_experts, d, inter, pack=True)
        assert packed.table.w2t is not None and packed.table.w13t is not None
        a_one = model.moe_decode_act(packed, dev(ids), dev(wts), dev(x), shared=shared, mode=1, act_kind=act, limit=limit).cpu().numpy()
        assert max(rel_l2(a_one[t, s], got_a[t, s]) for t in range(B) for s in range(got_a.shape[1])) <= 2e-6
        rows = model.moe_decode_from_act(packed, dev(ids), dev(wts), a, shared=shared, mode=1, act_kind=act).cpu().numpy()
        assert max(rel_l2(rows[t], two[t]) for t in range(B)) <= 2e-6


def test_one_launch_kernel_repeated_and_captured():
    """The one-launch kernel carries a launch tag in its exchanged values: repeated calls on one workspace, calls with
    fewer pairs after calls with more, and replays of a captured graph all give the first call's rows bit for bit, and no
    workgroup ever gave up waiting."""
    torch = torch_cuda()
    import ctypes
    from microkimi_amd import model
    from microkimi_amd._lib import check, lib
    d, inter, n_experts, topk, shared = 7168, 2048, 12, 8, 11
    table, experts = build(n_experts, d, inter)
    assert experts.table.w13t is not None
    res = {}
    for B in (3, 1, 2, 3, 1):
        ids, wts, x = stage_inputs(d, inter, n_experts, B, topk, shared, 1.0)
        got = model.moe_decode(experts, dev(ids), dev(wts), dev(x), shared=shared, mode=1).cpu().numpy()
        assert np.isfinite(got).all()
        if B in res:
            assert np.array_equal(got.view(np.uint32), res[B].view(np.uint32)), B
        res[B] = got
    ids, wts, x = stage_inputs(d, inter, n_experts, 2, topk, shared, 1.0)
    di, dw, dx = dev(ids), dev(wts), dev(x)
    out = torch.empty((2, d), device="cuda")
    model.moe_decode(experts, di, dw, dx, shared=shared, mode=1, out=out)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            model.moe_decode(experts, di, dw, dx, shared=shared, mode=1, out=out)
            model.moe_decode(experts, di, dw, dx, shared=shared, mode=1, out=out)
    torch.cuda.synchronize()
    for _ in range(3):
        out.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy().view(np.uint32), res[2].view(np.uint32))
    flag = ctypes.c_int(-1)
    check(lib.mk_dev_moe_decode_gave_up(ctypes.byref(flag)))
    assert flag.value == 0


def test_out_of_range_expert_id_adds_nothing():
    # a table that states its size: a routed id outside it contributes nothing (and no pointer is read out of bounds)
    from microkimi_amd import model
    d, inter, n_experts, topk, shared = 2048, 1024, 6, 3, 5
    table, experts = build(n_experts, d, inter)
    for B in (2, 6):
        ids, wts, x = stage_inputs(d, inter, n_experts, B, topk, shared, 0.05)
        bad = ids.copy()
        bad[0, 1] = 1000
        bad[B - 1, 2] = -7
        got = model.moe_decode(experts, dev(bad), dev(wts), dev(x), shared=shared, mode=1).cpu().numpy()
        w0 = wts.copy()
        w0[0, 1] = 0.0
        w0[B - 1, 2] = 0.0
        ref = model.moe_decode(experts, dev(ids), dev(w0), dev(x), shared=shared, mode=1).cpu().numpy()
        assert np.isfinite(got).all()
        assert rel_l2(got, ref) <= 1e-6


def test_batched_path_all_tokens_on_the_same_experts():
    """Every token selects the same two experts (and the shared one): three groups of 13 rows, each several passes of
    four tokens -- the largest group's later passes run on workgroups of their own, the others' one after the other."""
    from microkimi_amd import model
    d, inter, n_experts, B, topk, shared = 1024, 512, 4, 13, 2, 3
    table, experts = build(n_experts, d, inter)
    rng = np.random.default_rng(77)
    ids = np.tile(np.array([[2, 0]], dtype=np.int32), (B, 1))
    wts = rng.random((B, topk)).astype(np.float32)
    x = (rng.standard_normal((B, d)) * 0.02).astype(np.float32)
    got = model.moe_decode(experts, dev(ids), dev(wts), dev(x), shared=shared, mode=1).cpu().numpy()
    want = oracle.moe_decode(table, ids.astype(np.uint32), wts, x, shared=shared, mode=1, threads=8)
    w2_dev = experts._keep[2]
    rows_match_up_to_q8_flips(got, want, lambda t: [w2_dev[2], w2_dev[0], w2_dev[shared]], d, inter)


def test_scale_bytes_by_tile_are_the_same_bytes():
    # out[(t * rows + r) * 16 + j] = scales[r * (cols / 32) + 16 t + j]; a cols that is not a multiple of 512 is refused
    from microkimi_amd import _lib
    import torch
    rng = np.random.default_rng(5)
    for rows, cols in ((1, 512), (37, 1024), (256, 7168), (300, 2048)):
        sc = rng.integers(0, 256, size=(rows, cols // 32), dtype=np.uint8)
        out = torch.zeros(rows * cols // 32, dtype=torch.uint8, device="cuda")
        _lib.check(_lib.lib.mk_dev_mxfp4_scales_by_tile(_lib.ptr(dev(sc)), rows, cols, _lib.ptr(out), None))
        torch.cuda.synchronize()
        want = sc.reshape(rows, cols // 512, 16).transpose(1, 0, 2)
        assert np.array_equal(out.cpu().numpy().reshape(cols // 512, rows, 16), want)
    st = _lib.lib.mk_dev_mxfp4_scales_by_tile(_lib.ptr(out), 4, 768, _lib.ptr(out), None)
    assert st == -1 and b"512" in _lib.lib.mk_last_error()


@pytest.mark.parametrize("B,topk,shared", [(4, 2, -1), (16, 3, 5), (13, 2, 3)])
def test_batched_path_with_and_without_the_tile_ordered_scale_bytes(B, topk, shared):
    """The matrix-core path reads the scale bytes from the K-tile ordered copies when the table has them and from the
    reference layout when it has not: the same bytes, so the same bits."""
    from microkimi_amd import model
    d, inter, n_experts = 1024, 512, 6
    host = build(n_experts, d, inter)[1]._keep
    with_st = model.PackedExperts(host[0], host[1], host[2], d, inter, scales_by_tile=True)
    without = model.PackedExperts(host[0], host[1], host[2], d, inter, scales_by_tile=False)
    assert with_st.table.w1st and with_st.table.w3st and with_st.table.w2st
    assert not (without.table.w1st or without.table.w3st or without.table.w2st)
    rng = np.random.default_rng(B * 7 + topk)
    ids = np.stack([rng.permutation(5)[:topk] for _ in range(B)]).astype(np.int32)
    wts = rng.random((B, topk)).astype(np.float32)
    x = (rng.standard_normal((B, d)) * 0.02).astype(np.float32)
    a = model.moe_decode(with_st, dev(ids), dev(wts), dev(x), shared=shared, mode=1).cpu().numpy()
    b = model.moe_decode(without, dev(ids), dev(wts), dev(x), shared=shared, mode=1).cpu().numpy()
    assert np.isfinite(a).all() and np.array_equal(a.view(np.uint32), b.view(np.uint32))


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


def test_full_layer_257_experts_sampled_tokens():
    """Configuration 2 at its full size (256 routed + 1 shared expert at 2048 x 7168, 6 GB of MXFP4 drawn on the
    device, batch 16 routed by the seeded logits): the rows of sampled tokens against the oracle, which gets only the
    nine experts of that token copied to the host, at batch 16 (batched path) and at batch 1 (one-launch path).

    The layer re-quantizes the f32 activation to q8 before W2 (matvec_packed's own step, src/mxfp4.rs:476-479), which
    is a step function of its input: the gate/up sums here differ from the CPU's in their last bits (the order of
    the sum over blocks, expf), so an activation that lies within a few ulp of a rounding boundary takes the other
    int8 value.  Such a flip changes the layer's row by exactly one column of that expert's W2 times one
    quantization step (relative 4e-5 .. 4e-4 of the row; seen for about one activation in 60 000).  The check
    therefore allows at most two such single-column differences per token and requires the rest to agree to TOL."""
    torch = torch_cuda()
    from microkimi_amd import model, mxfp4, workloads as W
    d, inter, ne, topk = W.D_MODEL, W.D_INTER, W.N_EXPERTS, W.TOP_K
    g = torch.Generator(device="cuda").manual_seed(22)

    def draw(rows, cols):
        return (torch.randint(0, 256, (rows, cols // 2), dtype=torch.uint8, device="cuda", generator=g),
                torch.randint(118, 131, (rows, cols // 32), dtype=torch.uint8, device="cuda", generator=g))

    w1 = [draw(inter, d) for _ in range(ne + 1)]
    w3 = [draw(inter, d) for _ in range(ne + 1)]
    w2 = [draw(d, inter) for _ in range(ne + 1)]
    experts = model.PackedExperts(w1, w3, w2, d, inter)
    B = 16
    logits, hidden = W.config2_tokens(B)
    ids, wts = model.router_softmax_topk(dev(logits), topk)
    x = dev(hidden)  # hidden ~ N(0, 1) as the configuration states: |g| reaches hundreds, silu saturates
    got16 = model.moe_decode(experts, ids, wts, x, shared=ne, mode=1).cpu().numpy()
    assert np.isfinite(got16).all()
    ids_h, wts_h = ids.cpu().numpy(), wts.cpu().numpy()
    host = lambda pair: (pair[0].cpu().numpy(), pair[1].cpu().numpy())
    flips = 0
    for tok in (0, 3, 7, 8, 15):
        used = [int(e) for e in ids_h[tok]] + [ne]
        table = oracle.ExpertTable([host(w1[e]) for e in used], [host(w3[e]) for e in used], [host(w2[e]) for e in used], d, inter)
        local_ids = np.arange(topk, dtype=np.uint32)[None, :]
        want = oracle.moe_decode(table, local_ids, wts_h[tok:tok + 1], hidden[tok:tok + 1], shared=topk, mode=1, threads=8)
        flips += rows_match_up_to_q8_flips(got16[tok:tok + 1], want, lambda t: [w2[e] for e in used], d, inter)
        # batch 1 takes the one-launch path, batch 16 the batched one: the same arithmetic per block, another order of the sum
        got1 = model.moe_decode(experts, ids[tok:tok + 1].contiguous(), wts[tok:tok + 1].contiguous(), x[tok:tok + 1].contiguous(), shared=ne, mode=1).cpu().numpy()
        flips += rows_match_up_to_q8_flips(got1, want, lambda t: [w2[e] for e in used], d, inter)
    assert flips <= 8


@pytest.mark.parametrize("d,inter,B,topk,shared,act,mode", [
    (1024, 512, 1, 3, 5, 1, 0),      # SiTU (the rule of the model that stores cold experts as VQ1), shared expert VQ1, f32 mode
    (1024, 512, 5, 3, 4, 1, 0),      # shared expert MXFP4
    (2048, 1024, 3, 2, -1, 0, 0),    # SwiGLU, no shared expert
    (1024, 512, 4, 3, 5, 2, 0),      # DeepSeek rule (weight inside the activation)
    (1024, 512, 6, 3, 5, 1, 1),      # q8 mode: the MXFP4 experts quantize their inputs, the VQ1 experts do not
])
def test_layer_with_vq1_experts(d, inter, B, topk, shared, act, mode):
    # moe_forward over a layer that mixes MXFP4 and VQ1 ("cold") experts (src/model.rs:2227-2264): experts 1, 3, 5 are VQ1
    torch_cuda()
    from microkimi_amd import model, workloads
    n_experts = 6
    rng = np.random.default_rng(d + B)
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
    n_routed = n_experts - (1 if shared >= 0 else 0)
    ids = np.stack([rng.permutation(n_routed)[:topk] for _ in range(B)]).astype(np.int32)
    wts = rng.random((B, topk)).astype(np.float32)
    wts /= wts.sum(axis=1, keepdims=True)
    x = (rng.standard_normal((B, d)) * 0.05).astype(np.float32)
    limit = 10.0 if act == 2 else 0.0
    got = model.moe_decode(experts, dev(ids), dev(wts), dev(x), shared=shared, mode=mode, act_kind=act, limit=limit).cpu().numpy()
    want = oracle.moe_decode_mixed(host, codebook, d, inter, ids.astype(np.uint32), wts, x, shared=shared, mode=mode, act_kind=act, limit=limit)
    assert np.isfinite(got).all() and np.isfinite(want).all()
    if mode == 0:
        for t in range(B):
            assert rel_l2(got[t], want[t]) <= TOL, (t, rel_l2(got[t], want[t]))
    else:
        w2_dev = devs[2]
        used = lambda t: [w2_dev[int(e)] for e in list(ids[t]) + ([shared] if shared >= 0 else []) if int(e) % 2 == 0]
        rows_match_up_to_q8_flips(got, want, used, d, inter)
    # the two stages compose to the same rows
    act_rows = model.moe_decode_act(experts, dev(ids), dev(wts), dev(x), shared=shared, mode=mode, act_kind=act, limit=limit)
    again = model.moe_decode_from_act(experts, dev(ids), dev(wts), act_rows, shared=shared, mode=mode, act_kind=act).cpu().numpy()
    assert np.array_equal(again.view(np.uint32), got.view(np.uint32))


def test_count_of_routed_ids_outside_the_table():
    torch = torch_cuda()
    from microkimi_amd._lib import check, cur_stream, lib, ptr
    rng = np.random.default_rng(5)
    for n, n_experts in [(1, 1), (8, 384), (700, 64), (16384, 384)]:
        ids = rng.integers(0, n_experts, n).astype(np.int32)
        bad = rng.random(n) < 0.1
        ids[bad] = np.where(rng.random(int(bad.sum())) < 0.5, -1 - rng.integers(0, 5, int(bad.sum())), n_experts + rng.integers(0, 5, int(bad.sum())))
        count = torch.full((1,), -7, dtype=torch.int32, device="cuda")
        check(lib.mk_dev_moe_count_bad_ids(ptr(dev(ids)), n, n_experts, ptr(count), cur_stream()))
        assert int(count.item()) == int(bad.sum())


_GIVE_UP_SCRIPT = r"""
import ctypes, sys, numpy as np, torch
sys.path.insert(0, sys.argv[1]); sys.path.insert(0, sys.argv[1] + "/tests")
from microkimi_amd import model, workloads
from microkimi_amd._lib import check, lib
d, inter, n, topk = 7168, 2048, 10, 8
dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
host = [(workloads.mxfp4_matrix(2, "w1", inter, d, e), workloads.mxfp4_matrix(2, "w3", inter, d, e), workloads.mxfp4_matrix(2, "w2", d, inter, e))
        for e in range(n)]
pk = lambda k: [(dev(h[k][0]), dev(h[k][1])) for h in host]
experts = model.PackedExperts(pk(0), pk(1), pk(2), d, inter)
assert experts.table.w13t is not None
rng = np.random.default_rng(0)
x = dev(rng.standard_normal((1, d)).astype(np.float32))
ids = dev(rng.permutation(n - 1)[:topk].astype(np.int32)[None, :])
wts = dev(np.full((1, topk), 0.125, np.float32))
for _ in range(3):
    out = model.moe_decode(experts, ids, wts, x, shared=n - 1)
    torch.cuda.synchronize()
flag = ctypes.c_int(-1)
check(lib.mk_dev_moe_decode_gave_up(ctypes.byref(flag)))
o = out.cpu().numpy()
print("RESULT", flag.value, int(np.isnan(o).sum()), int(np.isfinite(o).all()))
"""


def test_one_launch_kernel_gives_up_instead_of_waiting_forever():
    # the waits of the one-launch kernel are bounded: with a bound of zero polls (MK_MOE_SPIN_LIMIT=0, read once per process,
    # hence a process of its own) a workgroup that does not find another's values at its first look gives up, its rows
    # become NaN, the flag goes up -- and every launch still ends.  (With luck all values are there at the first look: then
    # the rows are finite and the flag is down.  Both are the contract; a hang or a finite wrong row is not.)
    import os
    import subprocess
    import sys
    torch_cuda()
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, MK_MOE_SPIN_LIMIT="0")
    r = subprocess.run([sys.executable, "-c", _GIVE_UP_SCRIPT, root], env=env, capture_output=True, text=True, timeout=240)
    assert r.returncode == 0, r.stderr[-2000:]
    line = [l for l in r.stdout.splitlines() if l.startswith("RESULT")][-1].split()
    flag, n_nan, finite = int(line[1]), int(line[2]), int(line[3])
    assert (flag == 1 and n_nan > 0) or (flag == 0 and finite == 1), line
