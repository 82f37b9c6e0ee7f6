"""Regenerates the fixtures in this folder from the build's own CPU oracle.

    python tests/golden/make_golden.py

dequant_table.sha256 -- SHA-256 of the exhaustive u8 -> fp16 dequantisation table
    (256 quantised values x 65536 fp16 scale bit patterns, row-major uint16, NaN results
    canonicalised to 0x7E00).  The table itself is pinned against an independent float64
    evaluation in tests/test_oracle_quant.py; the digest only lets other tests compare a
    full table cheaply.
"""
import hashlib
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import oracle  # noqa: E402


def main():
    table = oracle.dequant_table().copy()
    table[np.isnan(table.view(np.float16))] = 0x7E00
    digest = hashlib.sha256(table.tobytes()).hexdigest()
    with open(os.path.join(HERE, "dequant_table.sha256"), "w") as f:
        f.write(digest + "  dequant_table[256][65536] uint16, NaN -> 0x7E00\n")
    print(digest)


if __name__ == "__main__":
    main()
