"""Writes tests/golden/int8_networks.json: per-tensor activation scales of the two int8 benchmark networks, fixed by
a calibration pass of the CPU oracle on a seeded batch, plus the oracle's output for two seeded images (the golden
vectors the GPU path must reproduce bit for bit).  Run from the repository root:

    python tests/golden/make_int8_networks.py
"""
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import __graft_entry__ as ge  # noqa: E402

import int8_ref  # noqa: E402


def main():
    ge.load_package()  # architecture tables and the seeded parameter generator live in the package; no GPU is touched
    from zant_amd import networks as nets
    out = {}
    for arch in (nets.tiny_yolo_arch(), nets.mobilenet_v2_035_arch()):
        params = nets.int8_params(arch, seed=0)
        g = np.random.default_rng(1234)
        calib = g.integers(0, 256, (4,) + tuple(arch["input"]), dtype=np.uint8)
        quant = int8_ref.calibrate(arch, params, calib)
        x = np.random.default_rng(99).integers(0, 256, (2,) + tuple(arch["input"]), dtype=np.uint8)
        y = int8_ref.forward(arch, params, quant, x)
        out[arch["name"]] = {
            "param_seed": 0, "input_seed": 99, "quant": quant,
            "macs_per_inference": int(nets.int8_macs_per_inference(arch)),
            "expected_shape": list(y.shape), "expected_u8": y.ravel().tolist(),
        }
        print(arch["name"], "macs/inference", out[arch["name"]]["macs_per_inference"], "output", y.shape,
              "distinct values", len(np.unique(y)))
    with open(os.path.join(ROOT, "tests", "golden", "int8_networks.json"), "w") as f:
        json.dump(out, f)


if __name__ == "__main__":
    main()
