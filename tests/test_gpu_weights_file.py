"""GPU: experts loaded from an MKIM file (mk_bin_load_experts) drive the MoE kernels like tables built from tensors."""
import numpy as np
import pytest

import mkim_writer as W
import oracle
from gpu_util import dev, rel_l2, torch_cuda

pytestmark = pytest.mark.gpu


def make_file(path, n_experts, d, inter, bad_dtype_at=None, bad_shape_at=None, vq_experts=(), codebook=None):
    from microkimi_amd import workloads
    rng = np.random.default_rng(7)
    tensors = [("model.embed_tokens.weight", W.F32, (16, d), rng.standard_normal((16, d)).astype(np.float32))]
    if codebook is not None:
        tensors.append(("vq_codebook", W.F32, (256, 16), codebook))
    host = []
    for e in range(n_experts):
        if e in vq_experts:   # a cold expert: one index byte per 16 weights (src/weights.rs:49-55)
            idx = {"w1": rng.integers(0, 256, (inter, d // 16), dtype=np.uint8), "w3": rng.integers(0, 256, (inter, d // 16), dtype=np.uint8),
                   "w2": rng.integers(0, 256, (d, inter // 16), dtype=np.uint8)}
            host.append(("vq1", idx["w1"], idx["w3"], idx["w2"]))
            for k, dims in (("w1", (inter, d)), ("w2", (d, inter)), ("w3", (inter, d))):
                tensors.append((f"layers.2.block_sparse_moe.experts.{e}.{k}", W.VQ1, dims, idx[k].tobytes()))
            continue
        w1 = workloads.mxfp4_matrix(2, "w1", inter, d, e)
        w3 = workloads.mxfp4_matrix(2, "w3", inter, d, e)
        w2 = workloads.mxfp4_matrix(2, "w2", d, inter, e)
        host.append((w1, w3, w2))
        for k, m, dims in (("w1", w1, (inter, d)), ("w2", w2, (d, inter)), ("w3", w3, (inter, d))):   # file order of the reference
            name = f"layers.2.block_sparse_moe.experts.{e}.{k}"
            if bad_dtype_at == (e, k):
                tensors.append((name, W.VQ1, dims, bytes(dims[0] * dims[1] // 16)))
            elif bad_shape_at == (e, k):
                tensors.append((name, W.MXFP4, (dims[0], dims[1] // 2), (m[0][:, : dims[1] // 4], m[1][:, : dims[1] // 64])))
            else:
                tensors.append((name, W.MXFP4, dims, m))
        tensors.append((f"layers.2.note.{e}", W.I32, (3,), np.array([e, 1, 2], np.int32)))   # unaligned filler between experts
    W.write(path, tensors, config={"d_model": d})
    return host


def test_loaded_experts_match_tables_built_from_tensors(tmp_path):
    torch = torch_cuda()
    from microkimi_amd import model, weights
    n, d, inter, B, topk = 6, 1024, 512, 5, 2
    host = make_file(tmp_path / "m.bin", n, d, inter)
    f = weights.BinFile.open(tmp_path / "m.bin")
    ex = f.load_experts("layers.2.", n)
    assert (ex.n, ex.d, ex.inter) == (n, d, inter)
    assert ex.bytes >= sum(m[0].size + m[1].size for h in host for m in h)
    todev = lambda lst: [(dev(p), dev(s)) for p, s in lst]
    ref = model.PackedExperts(todev([h[0] for h in host]), todev([h[1] for h in host]), todev([h[2] for h in host]), d, inter)
    rng = np.random.default_rng(3)
    ids = np.stack([rng.permutation(n - 1)[:topk] for _ in range(B)]).astype(np.int32)
    wts = rng.random((B, topk)).astype(np.float32)
    x = (rng.standard_normal((B, d)) * 0.05).astype(np.float32)
    got = model.moe_decode(ex, dev(ids), dev(wts), dev(x), shared=n - 1).cpu().numpy()
    same = model.moe_decode(ref, dev(ids), dev(wts), dev(x), shared=n - 1).cpu().numpy()
    assert np.array_equal(got, same)   # same kernels, same bytes: identical
    table = oracle.ExpertTable([h[0] for h in host], [h[1] for h in host], [h[2] for h in host], d, inter)
    want = oracle.moe_decode(table, ids.astype(np.uint32), wts, x, shared=n - 1, mode=1, threads=8)
    assert rel_l2(got, want) <= 1e-5
    # the prefill path reads the same table
    T = 24
    idp = np.stack([rng.permutation(n)[:topk] for _ in range(T)]).astype(np.int32)
    wp = rng.random((T, topk)).astype(np.float32)
    xp = (rng.standard_normal((T, d)) * 0.05).astype(np.float32)
    a = model.moe_prefill(ex, dev(idp), dev(wp), dev(xp)).cpu().numpy()
    b = model.moe_prefill(ref, dev(idp), dev(wp), dev(xp)).cpu().numpy()
    assert np.array_equal(a, b)
    ex.close()
    f.close()


def test_layer_with_vq1_experts_from_a_file(tmp_path):
    # experts 1 and 4 stored as VQ1 (dtype 3) with the file's global vq_codebook (src/model.rs:979-999): the loaded table
    # drives the layer like one built from tensors, and the oracle's mixed layer agrees
    torch_cuda()
    from microkimi_amd import model, weights
    n, d, inter, B, topk = 6, 1024, 512, 4, 3
    codebook = (np.random.default_rng(11).standard_normal((256, 16)) * 0.05).astype(np.float32)
    host = make_file(tmp_path / "cold.bin", n, d, inter, vq_experts=(1, 4), codebook=codebook)
    f = weights.BinFile.open(tmp_path / "cold.bin")
    ex = f.load_experts("layers.2.", n)
    assert ex.has_vq and (ex.n, ex.d, ex.inter) == (n, d, inter)
    oracle_experts = [h if h[0] == "vq1" else ("mxfp4", h[0], h[1], h[2]) for h in host]
    rng = np.random.default_rng(5)
    ids = np.stack([rng.permutation(n - 1)[:topk] for _ in range(B)]).astype(np.int32)
    wts = rng.random((B, topk)).astype(np.float32)
    x = (rng.standard_normal((B, d)) * 0.05).astype(np.float32)
    got = model.moe_decode(ex, dev(ids), dev(wts), dev(x), shared=n - 1, mode=0, act_kind=1).cpu().numpy()
    want = oracle.moe_decode_mixed(oracle_experts, codebook, d, inter, ids.astype(np.uint32), wts, x, shared=n - 1, mode=0, act_kind=1)
    for t in range(B):
        assert rel_l2(got[t], want[t]) <= 1e-5
    from microkimi_amd._lib import MkError
    with pytest.raises(MkError) as e:   # the prefill call reads MXFP4 experts only
        model.moe_prefill(ex, dev(ids), dev(wts), dev(x), mxfp8=True)
    assert e.value.status == -4
    ex.close()
    f.close()


def test_unsupported_dtype_and_shape_mismatch(tmp_path):
    torch_cuda()
    from microkimi_amd import weights
    from microkimi_amd._lib import MkError
    make_file(tmp_path / "vq.bin", 3, 256, 128, bad_dtype_at=(1, "w3"))   # one tensor of an MXFP4 expert stored as VQ1
    with pytest.raises(MkError) as e:
        weights.BinFile.open(tmp_path / "vq.bin").load_experts("layers.2.", 3)
    assert e.value.status == -1 and "differs from the expert's w1" in str(e.value)
    make_file(tmp_path / "nocb.bin", 3, 256, 128, vq_experts=(1,))        # VQ1 expert, but the file has no codebook
    with pytest.raises(MkError) as e:
        weights.BinFile.open(tmp_path / "nocb.bin").load_experts("layers.2.", 3)
    assert "missing tensor" in str(e.value) and "vq_codebook" in str(e.value)
    make_file(tmp_path / "shape.bin", 3, 256, 128, bad_shape_at=(2, "w2"))
    with pytest.raises(MkError) as e:
        weights.BinFile.open(tmp_path / "shape.bin").load_experts("layers.2.", 3)
    assert e.value.status == -1 and "expected [256, 128]" in str(e.value)
    with pytest.raises(MkError) as e:
        weights.BinFile.open(tmp_path / "shape.bin").load_experts("layers.9.", 3)
    assert "missing tensor" in str(e.value)


def test_file_written_by_the_reference_writer_dequantizes_like_the_reference_reader():
    """The fixture of tests/golden/make_mkim_fixture.py: a file from the reference's exporter (nano/export.py), with the
    values the reference's reader (nano/bin2pt.py dequant_mxfp4) gives for its expert tensors.  mk_bin_* blobs through
    mk_dev_mxfp4_dequant, and the resident expert table of mk_bin_load_experts, must give those values bit for bit."""
    import os
    torch = torch_cuda()
    from microkimi_amd import mxfp4, weights
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    exp = np.load(os.path.join(here, "mkim_ref_expected.npz"))
    f = weights.BinFile.open(os.path.join(here, "mkim_ref.bin"))
    d, inter, n = 64, 32, 3
    for e in range(n):
        for k, (r, c) in (("w1", (inter, d)), ("w2", (d, inter)), ("w3", (inter, d))):
            name = f"layers.0.block_sparse_moe.experts.{e}.{k}"
            pk, sc, rr, cc = f.mxfp4_parts(name)
            assert (rr, cc) == (r, c)
            got = mxfp4.dequant(dev(np.ascontiguousarray(pk)), dev(np.ascontiguousarray(sc)), r, c).cpu().numpy()
            want = exp["dequant:" + name]
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), name
            # the oracle agrees too (its dequant is pinned by ref/ds_golden.json)
            assert np.array_equal(oracle.mxfp4_dequant(pk, sc, r, c).view(np.uint32), want.view(np.uint32))
    ex = f.load_experts("layers.0.", n)
    assert (ex.n, ex.d, ex.inter) == (n, d, inter)
    # the resident copies give the same layer output as a table built from the file's tensors, and the oracle's
    from microkimi_amd import model
    parts = {k: [f.mxfp4_parts(f"layers.0.block_sparse_moe.experts.{e}.{k}")[:2] for e in range(n)] for k in ("w1", "w3", "w2")}
    todev = lambda lst: [(dev(np.ascontiguousarray(p)), dev(np.ascontiguousarray(s))) for p, s in lst]
    ref = model.PackedExperts(todev(parts["w1"]), todev(parts["w3"]), todev(parts["w2"]), d, inter)
    rng = np.random.default_rng(4)
    ids = np.stack([rng.permutation(n)[:2] for _ in range(3)]).astype(np.int32)
    wts = rng.random((3, 2)).astype(np.float32)
    x = rng.standard_normal((3, d)).astype(np.float32)
    got = model.moe_decode(ex, dev(ids), dev(wts), dev(x)).cpu().numpy()
    same = model.moe_decode(ref, dev(ids), dev(wts), dev(x)).cpu().numpy()
    assert np.array_equal(got, same)
    hostp = lambda k: [(np.ascontiguousarray(p), np.ascontiguousarray(s)) for p, s in parts[k]]
    table = oracle.ExpertTable(hostp("w1"), hostp("w3"), hostp("w2"), d, inter)
    want = oracle.moe_decode(table, ids.astype(np.uint32), wts, x, mode=1)
    assert rel_l2(got, want) <= 1e-5
    ex.close()
    f.close()


def test_mxfp4sq_expert_blobs_are_refused(tmp_path):
    # dtype 4 (MXFP4SQ, src/mxfp4.rs:140-240) is off the runtime path in the reference too ("the runtime packed matvec
    # still reads DTYPE_MXFP4 only", src/mxfp4.rs:150-151): such a layer stays on the caller's CPU path
    torch_cuda()
    from microkimi_amd import weights
    from microkimi_amd._lib import MkError
    d, inter = 64, 32
    rng = np.random.default_rng(1)
    tensors = []
    for e in range(2):
        for k, (r, c) in (("w1", (inter, d)), ("w2", (d, inter)), ("w3", (inter, d))):
            name = f"layers.0.block_sparse_moe.experts.{e}.{k}"
            if (e, k) == (1, "w2"):
                tensors.append((name, 4, (r, c), bytes(r * c // 2 + r * c // 32 + 4)))   # packed + quadratic scale bytes + f32 smax
            else:
                tensors.append((name, W.MXFP4, (r, c), (rng.integers(0, 256, (r, c // 2), dtype=np.uint8), rng.integers(118, 131, (r, c // 32), dtype=np.uint8))))
    W.write(tmp_path / "sq.bin", tensors, config={"d_model": d})
    f = weights.BinFile.open(tmp_path / "sq.bin")
    assert f.entries["layers.0.block_sparse_moe.experts.1.w2"].dtype == 4
    with pytest.raises(MkError) as e:
        f.load_experts("layers.0.", 2)
    assert e.value.status == -4 and "dtype 4" in str(e.value)
    f.close()
