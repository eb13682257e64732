"""Writes the small golden fixtures of tests/golden/ (run from the repo root):

    python tests/golden/make_fixtures.py

 * c3_slice_offsets.json -- the 64 seeded, non-overlapping, non-aligned 32-wide
   column offsets of benchmark config 3 (so that every run, CPU or GPU, moves
   exactly the same columns).
 * fp8_e4m3fn_kat.json   -- a 16-value known-answer vector for the
   float32 -> OCP e4m3fn quantiser (round-to-nearest-even including subnormals,
   largest finite value 448), stored as the byte codes torch produces.
Nothing here reads or runs the reference.
"""
import json
import os
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", ".."))
from oracle.inputs import make_slice_offsets  # noqa: E402


def main():
    starts = make_slice_offsets(64, 32, 8192, seed=0)
    with open(os.path.join(HERE, "c3_slice_offsets.json"), "w") as f:
        json.dump({"width": 32, "src_cols": 8192, "starts": starts}, f)
    vals = [0.0, 1.0, 1.0625, 1.1875, 2.0**-10, 1.5 * 2.0**-9, 2.0**-9, 3.0, 17.0, 100.0, 240.0, 448.0, 464.0, -1.1875, -448.0, 0.3]
    q = torch.tensor(vals, dtype=torch.float32).to(torch.float8_e4m3fn)
    with open(os.path.join(HERE, "fp8_e4m3fn_kat.json"), "w") as f:
        json.dump({"inputs": vals, "codes": q.view(torch.uint8).tolist(), "decoded": q.float().tolist()}, f)


if __name__ == "__main__":
    main()
