#!/usr/bin/env python3
"""Extract the TQ4 codebook literals from the reference header into a JSON data fixture.

The reference keeps the Lloyd-Max centroids, the encode boundaries and the seed-42
Rademacher sign diagonal only as numeric literals
(crates/warp34-kernels/csrc/tq/tq4_codebook.cuh:46-101); their generator is not in the
tree.  This script reads the header as text, pulls out the numbers and writes them to
tests/golden/tq4_tables.json so that the tables compiled into the oracle and into the
HIP library can be compared with the reference's values on machines that do not have
the reference checked out.  Nothing from the reference is executed.

Usage: python tests/golden/make_table_fixture.py [/root/reference]
"""
import json
import os
import re
import sys


def _array(text, name):
    m = re.search(name + r"\[\d+\]\s*=\s*\{(.*?)\};", text, re.S)
    if m is None:
        raise SystemExit("array %s not found" % name)
    return re.findall(r"-?\d+\.\d+(?:e-?\d+)?(?=f)", m.group(1))


def main():
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    path = os.path.join(root, "crates/warp34-kernels/csrc/tq/tq4_codebook.cuh")
    text = open(path).read()
    signs = [float(s) for s in _array(text, "kTq4Signs256")]
    mask = 0
    for i, s in enumerate(signs):
        if s < 0:
            mask |= 1 << i
    out = {
        "source": "crates/warp34-kernels/csrc/tq/tq4_codebook.cuh:46-101",
        # decimal literals exactly as written in the header (they round to fp32 on use)
        "d256_centroids": _array(text, "kTq4D256Centroids"),
        "d256_boundaries": _array(text, "kTq4D256Boundaries"),
        "d128_centroids": _array(text, "kTq4D128Centroids"),
        "d128_boundaries": _array(text, "kTq4D128Boundaries"),
        "signs256": [int(s) for s in signs],
        # bit i set <=> signs256[i] == -1, little-endian bit order
        "signs256_negative_mask_hex": "%064x" % mask,
        "signs256_negative_count": sum(1 for s in signs if s < 0),
    }
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tq4_tables.json")
    with open(dst, "w") as f:
        json.dump(out, f, indent=1)
    print("wrote", dst)


if __name__ == "__main__":
    main()
