"""Writes a small MKIM0002 weight file with the reference's own writer, and what the reference's own reader makes of
it, as fixtures for the MKIM loader (mk_bin_*), which no held file of the reference pins.

Imported from the reference (in the build container only; nothing of it travels): nano/export.py `write_bin` and
`quantize_mxfp4` (the exporter of the .bin format, nano/export.py:23-75), nano/bin2pt.py `read_bin`, `dequant_mxfp4`
and `dequant_vq1` (its inverse, nano/bin2pt.py:52-99).  Outputs, both data:

    tests/golden/mkim_ref.bin           the file write_bin produced (f32, i32, MXFP4 expert and VQ1 tensors)
    tests/golden/mkim_ref_expected.npz  read_bin's directory and config, and the dequantized expert tensors

    python tests/golden/make_mkim_fixture.py /root/reference
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
DTYPE_F32, DTYPE_MXFP4, DTYPE_I32, DTYPE_VQ1 = 0, 1, 2, 3


def main(ref_root):
    sys.path.insert(0, os.path.join(ref_root, "nano"))
    import bin2pt   # noqa: E402  (the reference's reader)
    import export   # noqa: E402  (the reference's writer)

    rng = np.random.default_rng(20260)
    d, inter, n_experts = 64, 32, 3
    config = {"n_layers": 1, "hidden": d, "vocab": 48, "n_experts": n_experts, "top_k": 2, "moe_inter": inter, "rms_eps": 1e-5}
    tensors = []
    embed = rng.standard_normal((48, d)).astype(np.float32)
    tensors.append(("embed_tokens.weight", DTYPE_F32, [48, d], embed.tobytes()))
    tensors.append(("layers.0.block_sparse_moe.gate.weight", DTYPE_F32, [n_experts, d], rng.standard_normal((n_experts, d)).astype(np.float32).tobytes()))
    tensors.append(("mla_layers", DTYPE_I32, [3], np.array([0, 3, 7], np.int32).tobytes()))
    weights = {}
    for e in range(n_experts):
        for nm, (r, c) in (("w1", (inter, d)), ("w2", (d, inter)), ("w3", (inter, d))):
            w = (rng.standard_normal((r, c)) * (0.02 * (e + 1))).astype(np.float32)
            if e == 1 and nm == "w1":
                w[3, :32] = 0.0          # an all-zero block: scale byte 0
            packed, scales = export.quantize_mxfp4(w)
            name = f"layers.0.block_sparse_moe.experts.{e}.{nm}"
            tensors.append((name, DTYPE_MXFP4, [r, c], packed.tobytes() + scales.tobytes()))
            weights[name] = (r, c)
    codebook = rng.standard_normal((256, 16)).astype(np.float32)
    tensors.append(("vq_codebook", DTYPE_F32, [256, 16], codebook.tobytes()))
    vq_idx = rng.integers(0, 256, (8, 64 // 16), dtype=np.uint8)
    tensors.append(("layers.0.cold.w1", DTYPE_VQ1, [8, 64], vq_idx.tobytes()))
    tensors.append(("norm.weight", DTYPE_F32, [d], np.ones(d, np.float32).tobytes()))

    path = os.path.join(HERE, "mkim_ref.bin")
    export.write_bin(path, config, tensors)

    cfg, entries, f = bin2pt.read_bin(path)
    out = {"config_json": np.frombuffer(json.dumps(cfg).encode(), np.uint8),
           "names": np.array([e[0] for e in entries]),
           "dtypes": np.array([e[1] for e in entries], np.int64),
           "n_dims": np.array([len(e[2]) for e in entries], np.int64),
           "dims": np.array([e[2] + [0] * (8 - len(e[2])) for e in entries], np.int64),
           "offsets": np.array([e[3] for e in entries], np.int64),
           "sizes": np.array([e[4] for e in entries], np.int64)}
    for name, dtype, dims, offset, size in entries:
        f.seek(offset)
        blob = f.read(size)
        if dtype == DTYPE_MXFP4:
            out["dequant:" + name] = bin2pt.dequant_mxfp4(blob, dims)
        elif dtype == DTYPE_VQ1:
            out["dequant:" + name] = bin2pt.dequant_vq1(blob, dims, codebook)
    f.close()
    np.savez_compressed(os.path.join(HERE, "mkim_ref_expected.npz"), **out)
    print("wrote", path, os.path.getsize(path), "bytes and mkim_ref_expected.npz;", len(entries), "tensors")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
