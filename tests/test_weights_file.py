"""MKIM weight files (src/weights.rs:1-18, 424-470, 601-640) through mk_bin_*: no GPU needed.

The reference ships no file of this format and its reader is Rust, so the parser is pinned by a file assembled byte by
byte below from the format comment at the top of src/weights.rs, by files from tests/mkim_writer.py (BinWriter's layout
rules restated), and by the malformed inputs a reader must refuse.
"""
import struct

import numpy as np
import pytest

import mkim_writer as W
from microkimi_amd import weights
from microkimi_amd._lib import MkError

EXP = "layers.0.block_sparse_moe.experts.0.w1"


def hand_made(tmp_path):
    # MKIM0001 | n = 2 | ("norm.weight", f32, [4]) | (EXP, mxfp4, [2, 32]) | data
    e1 = struct.pack("<H", 11) + b"norm.weight" + bytes([0, 1]) + struct.pack("<I", 4) + struct.pack("<QQ", 128, 16)
    e2 = struct.pack("<H", len(EXP)) + EXP.encode() + bytes([1, 2]) + struct.pack("<II", 2, 32) + struct.pack("<QQ", 4096, 34)
    head = b"MKIM0001" + struct.pack("<I", 2) + e1 + e2
    assert len(head) <= 128
    f32 = np.array([1.0, -2.5, 3.25, 0.0], "<f4").tobytes()
    packed = bytes(range(32))              # 2 rows x 16 bytes
    scales = bytes([127, 120])             # 2 rows x 1 block
    data = head + b"\0" * (128 - len(head)) + f32
    data += b"\0" * (4096 - len(data)) + packed + scales
    p = tmp_path / "hand.bin"
    p.write_bytes(data)
    return p, packed, scales


def test_hand_assembled_file(tmp_path):
    p, packed, scales = hand_made(tmp_path)
    f = weights.BinFile.open(p)
    assert f.config is None and f.names == ["norm.weight", EXP]
    assert f.entries["norm.weight"] == weights.Entry(0, (4,), 128, 16)
    assert f.entries[EXP] == weights.Entry(1, (2, 32), 4096, 34)
    assert np.array_equal(f.f32_vec("norm.weight"), np.array([1.0, -2.5, 3.25, 0.0], np.float32))
    pk, sc, r, c = f.mxfp4_parts(EXP)
    assert (r, c) == (2, 32) and pk.tobytes() == packed and sc.tobytes() == scales
    with pytest.raises(TypeError):
        f.f32_vec(EXP)
    with pytest.raises(KeyError):
        f.blob("nope")
    f.close()


def test_writer_layout_and_config(tmp_path):
    rng = np.random.default_rng(0)
    cfg = {"d_model": 64, "n_experts": 2, "name": "tiny"}
    tensors = [("tok_embeddings.weight", W.F32, (8, 64), rng.standard_normal((8, 64)).astype(np.float32)),
               ("ids", W.I32, (5,), np.arange(5, dtype=np.int32) - 2)]
    for e in range(2):
        for k, (r, c) in (("w1", (32, 64)), ("w2", (64, 32)), ("w3", (32, 64))):
            tensors.append((f"layers.1.block_sparse_moe.experts.{e}.{k}", W.MXFP4, (r, c),
                            (rng.integers(0, 256, (r, c // 2), dtype=np.uint8), rng.integers(118, 131, (r, c // 32), dtype=np.uint8))))
    tensors.append(("layers.1.block_sparse_moe.gate.weight", W.F32, (2, 64), rng.standard_normal((2, 64)).astype(np.float32)))
    p = tmp_path / "v2.bin"
    offs = W.write(p, tensors, config=cfg)
    f = weights.BinFile.open(p)
    assert f.config == cfg
    assert f.names == [t[0] for t in tensors]
    for name, dt, dims, val in tensors:
        e = f.entries[name]
        assert (e.dtype, e.dims, e.offset) == (dt, tuple(dims), offs[name])
        # routed-expert blobs on 4096, everything else on 64 (src/weights.rs:96-124)
        assert e.offset % (4096 if W.is_expert_tensor(name) else 64) == 0
        assert f.blob(name).tobytes() == W.blob_bytes(dt, val)
    assert np.array_equal(f.i32_vec("ids"), np.arange(5) - 2)
    # the dense layout of slice --expert-order (set_expert_align(64))
    offs64 = W.write(tmp_path / "dense.bin", tensors, config=cfg, expert_align=64)
    g = weights.BinFile.open(tmp_path / "dense.bin")
    assert all(g.blob(t[0]).tobytes() == W.blob_bytes(t[1], t[3]) for t in tensors)
    assert any(o % 4096 for n, o in offs64.items() if W.is_expert_tensor(n))


@pytest.mark.parametrize("damage,msg", [
    (lambda b: b"MKIMxxxx" + b[8:], "bad magic"),
    (lambda b: b[:100], "beyond the end"),
    (lambda b: b[:40], "tensor count"),
    (lambda b: b[:8] + struct.pack("<I", 1 << 30) + b[12:], "tensor count"),
    (lambda b: b[:4000], "beyond the end"),
])
def test_malformed_files_are_refused(tmp_path, damage, msg):
    p, _, _ = hand_made(tmp_path)
    q = tmp_path / "bad.bin"
    q.write_bytes(damage(p.read_bytes()))
    with pytest.raises(MkError) as e:
        weights.BinFile.open(q)
    assert e.value.status == -1 and msg in str(e.value)


def test_directory_size_must_match_dims(tmp_path):
    p, _, _ = hand_made(tmp_path)
    b = bytearray(p.read_bytes())
    i = b.index(b"norm.weight") + 11 + 2 + 4 + 8   # the size field of the first entry
    b[i:i + 8] = struct.pack("<Q", 20)
    q = tmp_path / "bad2.bin"
    q.write_bytes(bytes(b))
    with pytest.raises(MkError) as e:
        weights.BinFile.open(q)
    assert "does not match" in str(e.value)
    with pytest.raises(MkError):
        weights.BinFile.open(tmp_path / "absent.bin")


def test_file_written_by_the_reference_writer():
    """tests/golden/mkim_ref.bin was written by the reference's own exporter (nano/export.py write_bin, experts
    quantized by its quantize_mxfp4) and read back by the reference's own reader (nano/bin2pt.py read_bin):
    mk_bin_* must see the same config, directory and bytes.  (tests/golden/make_mkim_fixture.py made both files.)"""
    import json
    import os
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    exp = np.load(os.path.join(here, "mkim_ref_expected.npz"))
    raw = open(os.path.join(here, "mkim_ref.bin"), "rb").read()
    f = weights.BinFile.open(os.path.join(here, "mkim_ref.bin"))
    assert f.config == json.loads(exp["config_json"].tobytes().decode())
    names = [str(n) for n in exp["names"]]
    assert f.names == names
    for i, name in enumerate(names):
        e = f.entries[name]
        nd = int(exp["n_dims"][i])
        assert e.dtype == int(exp["dtypes"][i]) and e.dims == tuple(int(v) for v in exp["dims"][i][:nd])
        assert (e.offset, e.size) == (int(exp["offsets"][i]), int(exp["sizes"][i]))
        assert f.blob(name).tobytes() == raw[e.offset:e.offset + e.size]
    # an expert blob splits into nibbles then scales (weights::BinFile::mxfp4_parts); the all-zero block has scale byte 0
    pk, sc, r, c = f.mxfp4_parts("layers.0.block_sparse_moe.experts.1.w1")
    assert (r, c) == (32, 64) and sc[3, 0] == 0 and not pk[3, :16].any()
    assert np.array_equal(f.i32_vec("mla_layers"), np.array([0, 3, 7]))
    f.close()
