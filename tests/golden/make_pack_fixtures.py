#!/usr/bin/env python3
"""Writes pack_seed42.json and pack_seed123.json: what the reference's own producer gives.

Run from the repository root, in a container that holds the reference tree:

    python tests/golden/make_pack_fixtures.py [/root/reference]

Route: imports ternarize/pack.py of the reference (torch on the CPU) and calls ternarize_tensor and
pack_ternary_to_bitmasks on the two seeded weight tensors of the reference's packing test
(tests/test_packing.py:92-111: seed 42, 256 x 128; tests/test_packing.py:141-173: seed 123, 64 x 100
padded to 128 columns). The fixture keeps the INPUT (fp32 bit patterns) beside the outputs, so the
tests that read it need neither torch's random stream nor the reference. Nothing of the reference
travels: the files hold numbers only.
"""
import importlib.util
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def load_pack(ref_root):
    spec = importlib.util.spec_from_file_location("ref_pack", os.path.join(ref_root, "ternarize", "pack.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def make(pack, name, seed, rows, cols, pad):
    torch.manual_seed(seed)
    w = torch.randn(rows, cols)
    if pad:
        w = pack.pad_to_multiple(w, 32)
    ternary, scales = pack.ternarize_tensor(w, group_size=128, threshold_factor=0.7)
    nz, sg = pack.pack_ternary_to_bitmasks(ternary)
    fx = {
        "name": name, "seed": seed, "rows": int(w.shape[0]), "cols": int(w.shape[1]), "group": 128,
        "threshold_factor": 0.7, "torch": torch.__version__,
        "weight_f32": [f"{v:08x}" for v in w.numpy().astype(np.float32).view(np.uint32).reshape(-1)],
        "ternary": "".join("-0+"[int(v) + 1] for v in ternary.numpy().reshape(-1)),
        "nz": [f"{v:08x}" for v in nz.reshape(-1)],
        "sign": [f"{v:08x}" for v in sg.reshape(-1)],
        "scales": [f"{v:04x}" for v in scales.numpy().view(np.uint16).reshape(-1)],
    }
    with open(os.path.join(HERE, name + ".json"), "w") as f:
        json.dump(fx, f, separators=(",", ":"))
        f.write("\n")
    print(name, w.shape, "groups", scales.numel())


if __name__ == "__main__":
    pack = load_pack(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
    make(pack, "pack_seed42", 42, 256, 128, False)
    make(pack, "pack_seed123", 123, 64, 100, True)
