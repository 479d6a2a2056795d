#!/usr/bin/env python3
"""Write tests/golden/dynamic_maps.json: bit patterns of the two 8-bit dynamic maps.

Nothing under the reference tree holds these tables (the reference's 8-bit Adam is per-tensor
linear), so the fixture restates the published bitsandbytes construction
(functional.py: create_dynamic_map, max_exponent_bits=7, total_bits=8) with float32 torch.linspace,
exactly as that package evaluates it.  The tests compare the product's table and the oracle's
inputs with these bits, and pin the bits themselves against a float64 closed form.
"""
import json
import os
import struct

import torch


def build(signed):
    vals = []
    for decade in range(7):
        k = 2 ** decade if signed else 2 ** (decade + 1)
        edges = torch.linspace(0.1, 1, k + 1)
        mids = (edges[:-1] + edges[1:]) / 2.0
        scaled = (10 ** (decade - 6)) * mids
        vals += scaled.tolist()
        if signed:
            vals += (-(10 ** (decade - 6)) * mids).tolist()
    vals += [0, 1.0]
    vals.sort()
    t = torch.tensor(vals, dtype=torch.float32)
    return ["%08x" % struct.unpack("<I", struct.pack("<f", float(x)))[0] for x in t.tolist()]


if __name__ == "__main__":
    out = {"format": "hex of IEEE-754 binary32, index = 8-bit code",
           "signed": build(True), "unsigned": build(False)}
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "dynamic_maps.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=0)
        f.write("\n")
