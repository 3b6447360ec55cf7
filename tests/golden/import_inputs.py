"""Converts the reference's communication-pattern matrices (inputs/<P>proc/global_comm_pattern_<P>proc.txt,
P x P byte counts, row = sender; read by examples/MLinputs_example.cpp:119-145) into compressed int32 fixtures
under tests/golden/inputs/.  Data only: same numbers, binary instead of text.  Runs in the build container.

    python tests/golden/import_inputs.py
"""
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = "/root/reference/inputs"

for P in (4, 8, 16, 32, 64, 128, 256, 512, 1024):
    m = np.loadtxt(os.path.join(SRC, f"{P}proc", f"global_comm_pattern_{P}proc.txt"), dtype=np.int64)
    assert m.shape == (P, P) and m.min() >= 0 and m.max() < 2**31
    out = os.path.join(HERE, "inputs", f"global_comm_pattern_{P}proc.npz")
    np.savez_compressed(out, counts=m.astype(np.int32))
    print(P, m.sum(), os.path.getsize(out))
