#!/usr/bin/env python3
"""Writes tests/golden/convblock_init.json: what the REFERENCE's ConvBlock constructor produces under a fixed seed.

Run in the build container only (CPU; it needs /root/reference and launches no kernel):

    python tests/golden/make_init_fixture.py

It imports the reference's ``pyramid_dwconv.conv_block.ConvBlock`` (pyramid_dwconv/conv_block.py:25-34), constructs it
under ``torch.manual_seed(0)`` for a few argument sets and records, per state_dict entry, the shape, the dtype and
order-sensitive checksums of the values.  tests/test_init_fixture.py compares this repository's module with the file,
which pins the constructor's draw order (conv_up, one depthwise weight per gate, conv_out, conv_pool) and the
initialisers against the reference itself.  The reference's sources stay where they are: only the numbers travel.
"""
import json
import os
import sys

import torch

REF = "/root/reference"
CASES = [
    dict(dim=64, kernel_size=7),
    dict(dim=128, kernel_size=13),
    dict(dim=48, kernel_size=5, bias=True, out_bias=False, scales=(1.0, 0.5, 0.25), inter_ratio=0.25),
]


def checksums(t):
    v = t.detach().double().flatten()
    idx = torch.arange(1, v.numel() + 1, dtype=torch.float64)
    return {"shape": list(t.shape), "dtype": str(t.dtype), "sum": float(v.sum()), "abs_sum": float(v.abs().sum()),
            "weighted_sum": float((v * idx).sum() / v.numel()), "head": [float(x) for x in v[:4]]}


def main():
    sys.path[:] = [p for p in sys.path if os.path.abspath(p or ".") != os.path.abspath(os.path.join(os.path.dirname(__file__), "..", ".."))]
    sys.path.insert(0, REF)
    from pyramid_dwconv.conv_block import ConvBlock  # the reference's

    assert os.path.abspath(sys.modules["pyramid_dwconv"].__file__).startswith(REF)
    out = []
    for kw in CASES:
        torch.manual_seed(0)
        m = ConvBlock(**kw)
        out.append({"kwargs": {k: (list(v) if isinstance(v, tuple) else v) for k, v in kw.items()},
                    "state_dict": {k: checksums(v) for k, v in m.state_dict().items()}})
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "convblock_init.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1)
    print("wrote", path)


if __name__ == "__main__":
    main()
