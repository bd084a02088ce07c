"""Writes the golden fixtures under tests/golden/ from the data files the
reference's own selftest consumes (ref/ds_golden.json, ref/ds_golden2.json,
read by src/selftest.rs:193-243 and :247-323).  Only data is read (JSON); no
reference code is imported or run.  Run once in the build container:

    python tests/golden/make_fixtures.py /root/reference
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def main(ref_root):
    g = json.load(open(os.path.join(ref_root, "ref", "ds_golden.json")))
    fp4 = g["fp4"]
    json.dump({k: fp4[k] for k in ("rows", "cols", "packed", "scales", "dequant")},
              open(os.path.join(HERE, "ds_golden_fp4.json"), "w"))
    fp8 = g["fp8"]
    np.savez_compressed(
        os.path.join(HERE, "ds_golden_fp8.npz"),
        rows=np.int64(fp8["rows"]), cols=np.int64(fp8["cols"]),
        w_packed=np.asarray(fp8["w_packed"], np.uint8), scales=np.asarray(fp8["scales"], np.uint8),
        # the JSON holds decimal renderings of f32 values: float32() restores the exact bits
        dequant=np.asarray(fp8["dequant"], np.float64).astype(np.float32),
        w_orig=np.asarray(fp8["w_orig"], np.float64).astype(np.float32))
    g2 = json.load(open(os.path.join(ref_root, "ref", "ds_golden2.json")))
    json.dump({"gate": g2["gate"], "expert": g2["expert"]}, open(os.path.join(HERE, "ds_golden2_gate_expert.json"), "w"))


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
