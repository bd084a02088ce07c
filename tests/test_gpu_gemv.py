"""GPU parity, MXFP4 GEMV (mxfp4::matvec_packed, both modes) and the q8_0 head, against the oracle.
Tolerance (north star): relative L2 <= 1e-5 with f32 accumulation; identical argmax on logits."""
import numpy as np
import pytest

import oracle
from gpu_util import dev, rel_l2, torch_cuda

pytestmark = pytest.mark.gpu
TOL = 1e-5
SHAPES = [(128, 512), (512, 128), (64, 128), (3, 64), (1, 32), (256, 1024), (2048, 4096), (333, 1024), (4096, 2048), (77, 7168),
          (5, 96), (130, 2048)]


def quantized_case(rows, cols):
    w = oracle.pattern(0, rows * cols)
    p, s = oracle.mxfp4_quantize(w, rows, cols)
    return p, s, oracle.pattern(4242, cols)


@pytest.mark.parametrize("rows,cols", SHAPES)
@pytest.mark.parametrize("mode", [1, 0])
def test_matvec_packed_selftest_shapes(rows, cols, mode):
    torch = torch_cuda()
    from microkimi_amd import mxfp4, q8
    p, s, x = quantized_case(rows, cols)
    want = oracle.matvec_packed(p, s, rows, cols, x, mode=mode)
    out = torch.full((rows,), 7.0, device="cuda")
    q8.force_q8(mode)
    try:
        mxfp4.matvec_packed(dev(p), dev(s), rows, cols, dev(x), out)
    finally:
        q8.force_q8(-1)
    assert rel_l2(out.cpu().numpy(), want) <= TOL


def test_q8_block_terms_are_exact():
    # one block per row: out = idot * (2^(sb-128) * dx) has no summation at all, so the result must be bit-identical
    from microkimi_amd import mxfp4, q8
    torch = torch_cuda()
    rng = np.random.default_rng(4)
    rows = 4096
    p = rng.integers(0, 256, (rows, 16), dtype=np.uint8)
    s = rng.integers(0, 255, (rows, 1), dtype=np.uint8)
    x = rng.standard_normal(32).astype(np.float32)
    xq, xs = oracle.quantize_q8(x)
    want = oracle.matvec_packed_q8(p, s, rows, 32, xq, xs)
    out = torch.empty(rows, device="cuda")
    mxfp4.matvec_packed_q8(dev(p), dev(s), rows, 32, q8.Q8Vec(dev(xq), dev(xs)), out)
    got = out.cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_zero_block_and_config0():
    torch = torch_cuda()
    from microkimi_amd import mxfp4, q8, workloads
    rows, cols = 64, 128
    w = oracle.pattern(0, rows * cols)
    w[2 * cols:4 * cols] = 0
    p, s = oracle.mxfp4_quantize(w, rows, cols)
    x = oracle.pattern(4242, cols)
    for mode in (1, 0):
        out = torch.empty(rows, device="cuda")
        q8.force_q8(mode)
        mxfp4.matvec_packed(dev(p), dev(s), rows, cols, dev(x), out)
        q8.force_q8(-1)
        got = out.cpu().numpy()
        assert np.all(got[2:4] == 0) and rel_l2(got, oracle.matvec_packed(p, s, rows, cols, x, mode=mode)) <= TOL
    # benchmark configuration 0 at full size, both modes
    p, s, x = workloads.config0()
    for mode in (1, 0):
        out = torch.empty(2048, device="cuda")
        q8.force_q8(mode)
        mxfp4.matvec_packed(dev(p), dev(s), 2048, 7168, dev(x), out)
        q8.force_q8(-1)
        assert rel_l2(out.cpu().numpy(), oracle.matvec_packed(p, s, 2048, 7168, x, mode=mode)) <= TOL


def test_grouped_launch_matches_per_matrix():
    torch = torch_cuda()
    from microkimi_amd import mxfp4, q8, workloads
    rows, cols, nmat = 256, 7168, 5
    mats = [workloads.mxfp4_matrix(9, "g", rows, cols, i) for i in range(nmat)]
    xs = workloads.normal(9, "x", (3, cols))
    idx = np.array([0, 2, 1, 1, 0], np.int32)
    pd, sd = [dev(m[0]) for m in mats], [dev(m[1]) for m in mats]
    outs = [torch.empty(rows, device="cuda") for _ in range(nmat)]
    xq = q8.quantize_q8(dev(xs))
    keep = mxfp4.matvec_packed_grouped_q8(pd, sd, rows, cols, xq, dev(idx), outs)
    torch.cuda.synchronize()
    for i in range(nmat):
        want = oracle.matvec_packed(mats[i][0], mats[i][1], rows, cols, xs[idx[i]], mode=1)
        assert rel_l2(outs[i].cpu().numpy(), want) <= TOL
    del keep
    # all matrices against one activation (no index); the results are bit-identical to the per-matrix launches (same
    # tiles, same per-tile arithmetic, whatever the number of workgroups per matrix)
    for r2, n2 in ((256, 5), (301, 3), (2048, 7)):
        mats2 = [workloads.mxfp4_matrix(9, "h", r2, cols, i) for i in range(n2)]
        pd2, sd2 = [dev(m[0]) for m in mats2], [dev(m[1]) for m in mats2]
        outs2 = [torch.empty(r2, device="cuda") for _ in range(n2)]
        x1 = q8.quantize_q8(dev(xs[:1]))
        keep = mxfp4.matvec_packed_grouped_q8(pd2, sd2, r2, cols, x1, None, outs2)
        torch.cuda.synchronize()
        for i in range(n2):
            want = oracle.matvec_packed(mats2[i][0], mats2[i][1], r2, cols, xs[0], mode=1)
            assert rel_l2(outs2[i].cpu().numpy(), want) <= TOL
            single = torch.empty(r2, device="cuda")
            mxfp4.matvec_packed(pd2[i], sd2[i], r2, cols, dev(xs[0]), single)
            assert torch.equal(single, outs2[i])
        del keep


@pytest.mark.parametrize("rows,cols,m", [(64, 128, 8), (33, 64, 5), (128, 512, 24), (40, 7168, 3),
                                         # four and more positions at cols % 128 == 0 run on the f32 matrix instruction: ragged rows,
                                         # position counts around the tiles of 16 and the passes of 64, the model shapes
                                         (37, 7168, 4), (2048, 7168, 17), (100, 2048, 70), (7168, 2048, 16), (16, 128, 130),
                                         (100, 2048, 129), (2048, 7168, 160),
                                         # from 512 positions the activations of a step are staged in LDS for 64 weight rows: ragged
                                         # rows and positions, and a row count the staged stores do not take
                                         (100, 2048, 515), (260, 128, 513), (38, 256, 520), (512, 7168, 512)])
def test_matvec_packed_nt(rows, cols, m):
    from microkimi_amd import model
    p, s, _ = quantized_case(rows, cols)
    x = oracle.pattern(99, cols * m).reshape(m, cols)
    got = model.matvec_packed_nt(dev(p), dev(s), rows, cols, dev(x), m).cpu().numpy()
    m8 = (m + 7) // 8 * 8
    xt = np.zeros((cols, m8), np.float32)
    xt[:, :m] = x.T
    want = oracle.matvec_packed_nt(p, s, rows, cols, xt, m8)[:m]
    assert rel_l2(got, want) <= TOL


@pytest.mark.parametrize("rows,cols,m", [(64, 512, 1), (40, 7168, 3), (33, 64, 2)])
def test_nt_vector_path_and_f32_matvec_give_the_same_bits(rows, cols, m):
    # matvec_packed_nt (src/model.rs:2412-2447) and the f32 branch of matvec_packed (src/mxfp4.rs:475-539) are the same
    # sum in the reference (the oracle's two restatements agree bit for bit, checked here too); on the device the
    # up-to-3-positions path of mk_dev_mxfp4_matvec_nt and mk_dev_mxfp4_matvec_f32 are two kernels: same bits
    torch = torch_cuda()
    from microkimi_amd import model
    from microkimi_amd._lib import check, cur_stream, lib, ptr
    p, s, _ = quantized_case(rows, cols)
    x = oracle.pattern(7, cols * m).reshape(m, cols)
    got = model.matvec_packed_nt(dev(p), dev(s), rows, cols, dev(x), m).cpu().numpy()
    dp, ds = dev(p), dev(s)
    xt = np.zeros((cols, 8), np.float32)
    xt[:, :m] = x.T
    want_nt = oracle.matvec_packed_nt(p, s, rows, cols, xt, 8)[:m]
    for j in range(m):
        out = torch.empty(rows, device="cuda")
        check(lib.mk_dev_mxfp4_matvec_f32(ptr(dp), ptr(ds), rows, cols, ptr(dev(x[j])), ptr(out), cur_stream()))
        assert np.array_equal(out.cpu().numpy().view(np.uint32), got[j].view(np.uint32)), j
        assert np.array_equal(oracle.matvec_packed(p, s, rows, cols, x[j], mode=0).view(np.uint32), want_nt[j].view(np.uint32)), j


@pytest.mark.parametrize("sb,m", [(0, 16), (1, 16), (2, 16), (1, 3), (250, 16), (1, 600)])
def test_matvec_packed_nt_extreme_scale_bytes(sb, m):
    # scale bytes 0..2 make every weight a subnormal or the smallest normals (byte 0 is 2^-127, src/mxfp4.rs:340-346),
    # byte 250 the largest that keeps the sums finite: the matrix-instruction paths (m >= 4, m >= 512) and the vector
    # path (m = 3) keep subnormal weights and products as the reference's f32 loop does
    from microkimi_amd import model
    rows, cols = 64, 256
    rng = np.random.default_rng(sb + m)
    packed = rng.integers(0, 256, (rows, cols // 2), dtype=np.uint8)
    scales = np.full((rows, cols // 32), sb, np.uint8)
    x = (rng.standard_normal((m, cols)) * (1.0 if sb < 100 else 1e-30)).astype(np.float32)
    got = model.matvec_packed_nt(dev(packed), dev(scales), rows, cols, dev(x), m).cpu().numpy()
    m8 = (m + 7) // 8 * 8
    xt = np.zeros((cols, m8), np.float32)
    xt[:, :m] = x.T
    want = oracle.matvec_packed_nt(packed, scales, rows, cols, xt, m8)[:m]
    assert np.isfinite(want).all() and np.abs(want).max() > 0
    err = np.linalg.norm(got.astype(np.float64) - want) / np.linalg.norm(want.astype(np.float64))
    assert err <= TOL


@pytest.mark.parametrize("rows,cols,batch,f16", [(512, 1024, 1, True), (512, 1024, 8, True), (512, 1024, 3, False), (100, 7168, 1, True),
                                                  (100, 7168, 8, True), (37, 96, 2, True), (37, 96, 1, False), (64, 2048, 5, True),
                                                  (1000, 4096, 1, False),
                                                  # streaming batch kernel (7168 columns, batch 2-4): ragged row counts
                                                  (4099, 7168, 2, True), (2050, 7168, 3, False), (3, 7168, 4, True),
                                                  (5000, 7168, 4, True)])
def test_q8head_shapes(rows, cols, batch, f16):
    torch = torch_cuda()
    from microkimi_amd import model
    rng = np.random.default_rng(rows + cols + batch)
    q = rng.integers(-127, 128, (rows, cols), dtype=np.int8)
    s = (np.abs(rng.standard_normal((rows, cols // 32))) * 0.02 / 127).astype(np.float32)
    if f16:
        s16 = s.astype(np.float16)
        s = s16.astype(np.float32)
        head = model.Q8Head.from_q8(dev(q), dev(s16), rows, cols)
    else:
        head = model.Q8Head.from_q8(dev(q), dev(s), rows, cols)
    x = rng.standard_normal((batch, cols)).astype(np.float32)
    got = head.matvec(dev(x)).cpu().numpy()
    for b in range(batch):
        want = oracle.q8head_matvec(q, s, rows, cols, x[b], workers=8)
        assert rel_l2(got[b], want) <= TOL, b
        assert int(np.argmax(got[b])) == oracle.argmax(want)


def test_q8head_reference_unit_test():
    # src/model.rs:3866-3881 through the device path: from_f32 on the device, err/span < 1e-2, same argmax as f32
    from microkimi_amd import model
    rows, cols = 512, 1024
    rng = oracle.Rng(0xC0FFEE)
    w = rng.f32(rows * cols) * np.float32(0.02)
    x = rng.f32(cols)
    head = model.Q8Head.from_f32(dev(w.reshape(rows, cols)), rows, cols, scales_f16=False)
    qo, so = oracle.q8head_from_f32(w, rows, cols)
    assert np.array_equal(head.q.cpu().numpy(), qo) and np.array_equal(head.scales.cpu().numpy(), so)  # bit-exact quantization
    got = head.matvec(dev(x)).cpu().numpy()[0]
    want = oracle.matvec_f32(w, rows, cols, x)
    assert np.abs(got - want).max() / np.abs(want).max() < 1e-2
    assert int(np.argmax(got)) == int(np.argmax(want))
    assert rel_l2(got, oracle.q8head_matvec(qo, so, rows, cols, x)) <= TOL
    assert int(head.argmax(head.matvec(dev(x)))[0]) == oracle.argmax(want)


def test_argmax_ties_lowest_index():
    torch = torch_cuda()
    from microkimi_amd import model
    logits = np.zeros((3, 163840), np.float32)
    logits[0, [70000, 5, 163839]] = 3.0
    logits[1, 163839] = 1.0
    logits[2] = -1.0
    head = model.Q8Head(torch.empty(0), torch.empty(0, dtype=torch.float16), 0, 0)
    idx = head.argmax(dev(logits)).cpu().numpy()
    assert idx.tolist() == [5, 163839, 0]


def test_lm_head_full_size_argmax_and_parity():
    # benchmark configuration 1: 163840 x 7168, batch 1 and 8; top-1 must match the CPU path
    from microkimi_amd import model, workloads
    q, s16, x = workloads.config1()
    head = model.Q8Head.from_q8(dev(q), dev(s16), workloads.VOCAB, workloads.D_MODEL)
    s = s16.astype(np.float32)
    got8 = head.matvec(dev(x)).cpu().numpy()
    got1 = head.matvec(dev(x[:1])).cpu().numpy()
    am = head.argmax(dev(got8)).cpu().numpy()
    for b in range(8):
        want = oracle.q8head_matvec(q, s, workloads.VOCAB, workloads.D_MODEL, x[b], workers=16)
        assert rel_l2(got8[b], want) <= TOL, b
        assert int(am[b]) == oracle.argmax(want), b
        if b == 0:
            assert rel_l2(got1[0], want) <= TOL


def test_matrices_beyond_32_bit_offsets():
    # maximum sizes: matrices whose byte size passes 2^32 leave the kernels that address them with 32-bit offsets; the
    # rows are independent, so a sample of rows (first, last, around the 4 GiB boundary) is checked against the oracle
    torch = torch_cuda()
    from microkimi_amd import mxfp4, q8
    from microkimi_amd._lib import check, cur_stream, lib, ptr
    cols = 7168
    g = torch.Generator(device="cuda").manual_seed(11)
    x = torch.randn((8, cols), device="cuda", generator=g)
    # q8_0 head, 600 000 rows: 4.3e9 weight bytes
    rows = 600_000
    q = torch.randint(-127, 128, (rows, cols), dtype=torch.int8, device="cuda", generator=g)
    s = (torch.rand((rows, cols // 32), device="cuda", generator=g) * 1e-3 + 1e-4).to(torch.float16)
    edge = (1 << 32) // cols
    sample = np.unique(np.clip(np.concatenate([np.arange(0, 40), np.arange(edge - 20, edge + 20), np.arange(rows - 40, rows)]), 0, rows - 1))
    sq, ss = q[sample].cpu().numpy(), s[sample].cpu().numpy().astype(np.float32)
    for batch in (1, 3, 8):
        xq = q8.quantize_q8(x[:batch].contiguous())
        out = torch.empty((batch, rows), device="cuda")
        check(lib.mk_dev_q8_matvec(ptr(q), ptr(s), 1, rows, cols, ptr(xq.q), ptr(xq.scales), batch, ptr(out), cur_stream()))
        got = out[:, sample].cpu().numpy()
        for b in range(batch):
            want = oracle.q8head_matvec(sq, ss, len(sample), cols, x[b].cpu().numpy())
            assert rel_l2(got[b], want) <= TOL, (batch, b)
    del q, s, out
    torch.cuda.empty_cache()
    # MXFP4, 1 250 000 rows: 4.5e9 packed bytes, 2.8e8 blocks
    rows = 1_250_000
    packed = torch.randint(0, 256, (rows, cols // 2), dtype=torch.uint8, device="cuda", generator=g)
    scales = torch.randint(118, 131, (rows, cols // 32), dtype=torch.uint8, device="cuda", generator=g)
    edge = (1 << 32) // (cols // 2)
    sample = np.unique(np.clip(np.concatenate([np.arange(0, 40), np.arange(edge - 20, edge + 20), np.arange(rows - 40, rows)]), 0, rows - 1))
    sp, sc = packed[sample].cpu().numpy(), scales[sample].cpu().numpy()
    x0 = x[0].contiguous()
    for mode in (1, 0):
        out = torch.empty(rows, device="cuda")
        if mode == 1:
            xq = q8.quantize_q8(x0)
            check(lib.mk_dev_mxfp4_matvec_q8(ptr(packed), ptr(scales), rows, cols, ptr(xq.q), ptr(xq.scales), ptr(out), cur_stream()))
        else:
            check(lib.mk_dev_mxfp4_matvec_f32(ptr(packed), ptr(scales), rows, cols, ptr(x0), ptr(out), cur_stream()))
        want = oracle.matvec_packed(sp, sc, len(sample), cols, x0.cpu().numpy(), mode=mode)
        assert rel_l2(out[sample].cpu().numpy(), want) <= TOL, mode


def test_batched_q8_matvec_on_the_matrix_cores():
    """mk_dev_mxfp4_matvec_q8_batched (the kernel of the batched MoE decode): m activation rows against one matrix.
    (1) With a single non-zero block per weight row the output IS one block term: bit-identical to the oracle's
    matvec_packed_q8 -- the int8 = 16 a + b split on the FP8 matrix cores is exact and the term is rounded once, as the
    reference's.  (2) Dense weights: the sum over blocks in another order, rel. L2 <= 1e-5, for 1 to 9 rows (one pass
    with one or two token pairs, several passes)."""
    torch = torch_cuda()
    from microkimi_amd import mxfp4, q8
    rng = np.random.default_rng(11)
    rows, cols = 300, 1024
    nb = cols // 32
    for m in (1, 2, 3, 4, 9):
        x = rng.standard_normal((m, cols)).astype(np.float32) * rng.uniform(0.01, 30.0, (m, 1)).astype(np.float32)
        xq = q8.quantize_q8(dev(x))
        xq_h, xs_h = xq.q.cpu().numpy(), xq.scales.cpu().numpy()
        # (1) one block per row
        packed = np.zeros((rows, cols // 2), np.uint8)
        scales = rng.integers(100, 150, (rows, nb)).astype(np.uint8)
        blk = rng.integers(0, nb, rows)
        for r in range(rows):
            packed[r, blk[r] * 16:(blk[r] + 1) * 16] = rng.integers(0, 256, 16)
        got = mxfp4.matvec_packed_q8_batched(dev(packed), dev(scales), rows, cols, xq).cpu().numpy()
        for i in range(m):
            want = oracle.matvec_packed_q8(packed, scales, rows, cols, xq_h[i], xs_h[i])
            assert np.array_equal(got[i].view(np.uint32), want.view(np.uint32)), (m, i)
        # (2) dense
        packed = rng.integers(0, 256, (rows, cols // 2)).astype(np.uint8)
        scales = rng.integers(118, 131, (rows, nb)).astype(np.uint8)
        got = mxfp4.matvec_packed_q8_batched(dev(packed), dev(scales), rows, cols, xq).cpu().numpy()
        for i in range(m):
            want = oracle.matvec_packed_q8(packed, scales, rows, cols, xq_h[i], xs_h[i])
            assert rel_l2(got[i], want) <= 1e-5


@pytest.mark.parametrize("rows,cols", [(77, 7168), (2048, 7168), (130, 2048), (333, 1024), (2048, 4096)])
def test_mxfp4_gemv_equals_its_order_emulation_bit_for_bit(rows, cols):
    # the kernel's terms are the reference's (exact block dots, the same scale product); the oracle restates the order in
    # which the kernel adds them (matvec_packed_q8_device_order): the device must give exactly those floats
    torch = torch_cuda()
    from microkimi_amd import mxfp4, q8
    rng = np.random.default_rng(rows + cols)
    p = rng.integers(0, 256, (rows, cols // 2), dtype=np.uint8)
    s = rng.integers(118, 131, (rows, cols // 32), dtype=np.uint8)
    x = rng.standard_normal(cols).astype(np.float32)
    xq, xs = oracle.quantize_q8(x)
    want = oracle.matvec_packed_q8_device_order(p, s, rows, cols, xq, xs)
    out = torch.empty(rows, device="cuda")
    mxfp4.matvec_packed_q8(dev(p), dev(s), rows, cols, q8.quantize_q8(dev(x)), out)
    got = out.cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), float(np.abs(got - want).max())


@pytest.mark.parametrize("f16", [True, False])
def test_lm_head_gemv_equals_its_order_emulation_bit_for_bit(f16):
    # the batch-1 q8 head kernel at the benchmark's row length, against q8head_matvec_device_order
    torch_cuda()
    from microkimi_amd import model
    rng = np.random.default_rng(44)
    rows, cols = 3000, 7168
    q = rng.integers(-127, 128, (rows, cols), dtype=np.int8)
    s = (np.abs(rng.standard_normal((rows, cols // 32))) * 0.02 / 127).astype(np.float32)
    if f16:
        s16 = s.astype(np.float16)
        s = s16.astype(np.float32)
    head = model.Q8Head.from_q8(dev(q), dev(s16 if f16 else s), rows, cols)
    x = rng.standard_normal((1, cols)).astype(np.float32)
    xq, xs = oracle.quantize_q8(x[0])
    want = oracle.q8head_matvec_device_order(q, s, rows, cols, xq, xs)
    got = head.matvec(dev(x)).cpu().numpy()[0]
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), float(np.abs(got - want).max())
