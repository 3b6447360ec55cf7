"""Writes tests/golden/golden.json (+ c1_recv.bin) by running the REAL reference functions.

Runs only in the build container: it needs oracle/_ref/ref_driver (`make -C oracle ref`, which
compiles the reference's sources from /root/reference with the image's MPICH) and mpiexec.
Each case regenerates its inputs from a seed through rbruck_alltoallv_amd.workloads, hands the
count matrix to `mpiexec -n P ref_driver ...` and records the per-rank FNV-1a digests of the
receive blocks the reference produced (and, for the P=8 plumbing case, every byte of every
rank's recvbuf).  The fixtures are data only; the tests rebuild the same inputs from the same
seeds and never need the reference again.

    python tests/golden/make_golden.py
"""
from __future__ import annotations

import json
import os
import subprocess
import sys
import tempfile

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from rbruck_alltoallv_amd import workloads as W  # noqa: E402

DRIVER = os.path.join(ROOT, "oracle", "_ref", "ref_driver")
MPIEXEC = "/opt/conda/bin/mpiexec"
HERE = os.path.dirname(os.path.abspath(__file__))
INPUTS_DIR = os.path.join(HERE, "inputs")


def counts_for(spec: dict) -> np.ndarray:
    kind = spec["kind"]
    if kind == "uniform_random":
        c = W.counts_uniform_random(spec["P"], spec["hi"], spec["seed"])
    elif kind == "zipf":
        c = W.counts_zipf(spec["P"], spec["max"], 1.2, 5, spec["seed"])
    elif kind == "normal":
        c = W.counts_normal(spec["P"], spec["mean"], spec["sd"], 0, spec["hi"], spec["seed"])
    elif kind == "fft":
        c = W.counts_fft_rows(spec["P"], spec["row_len"], spec["count"])
    elif kind == "zeros":
        c = np.zeros((spec["P"], spec["P"]), dtype=np.int32)
    elif kind == "ml":
        # the reference's own communication-pattern matrices (inputs/<P>proc), scaled down
        c = W.counts_from_npz(os.path.join(INPUTS_DIR, f"global_comm_pattern_{spec['P']}proc.npz"), spec["divide"])
    else:
        raise ValueError(kind)
    if spec.get("sparsify"):
        c = c.copy()
        c[c % spec["sparsify"] == 0] = 0
    return c


def cases() -> list[dict]:
    out = []

    def add(cid, func, counts, esz, r=2, b=0, n=0, bblock=0, layout=0, payload=W.PAYLOAD_HASH, seed=1, count=0):
        out.append(dict(id=cid, func=func, counts=counts, esz=esz, r=r, b=b, n=n, bblock=bblock, layout=layout,
                        payload=payload, seed=seed, count=count))

    c1 = dict(kind="uniform_random", P=8, hi=64, seed=0)
    for f in ("twophase", "om", "tuna"):
        add(f"C1-{f}", f, c1, 4, r=2, b=1, payload=W.PAYLOAD_SELFDESC32)
    for f in ("ttpl", "ttpl_s1"):
        add(f"C1-{f}", f, c1, 4, r=2, n=4, payload=W.PAYLOAD_SELFDESC32)
    c2 = dict(kind="uniform_random", P=64, hi=256, seed=0)
    for r in (2, 4, 8):
        for f in ("twophase", "om", "tuna"):
            add(f"C2s-{f}-r{r}", f, c2, 1, r=r, b=2)
    c3 = dict(kind="zipf", P=64, max=2048, seed=0)
    for f in ("twophase", "om", "tuna"):
        add(f"C3s-{f}-r16", f, c3, 4, r=16, b=0)
    c4 = dict(kind="normal", P=128, mean=64.0, sd=16.0, hi=256, seed=0)
    add("C4s-ttpl", "ttpl", c4, 1, r=32, n=32, bblock=0)
    add("C4s-ttpl-b3", "ttpl", c4, 1, r=32, n=32, bblock=3)
    add("C4s-ttpl_s1", "ttpl_s1", c4, 1, r=32, n=32, bblock=0)
    add("C4s-ttpl_s1-r4", "ttpl_s1", c4, 1, r=4, n=32, bblock=40)
    add("C4s-ttpl-r2", "ttpl", c4, 1, r=2, n=32, bblock=0)
    c5 = dict(kind="fft", P=64, row_len=8, count=96)
    for r in (2, 8, 32, 64):
        add(f"C5s-tuna-r{r}", "tuna", c5, 8, r=r, b=0)
    add("C5s-tuna-r8-b1", "tuna", c5, 8, r=8, b=1)
    # odd sizes, gaps, zeros
    for P, r in ((12, 3), (17, 5), (27, 3), (7, 7), (49, 7), (5, 99)):
        cg = dict(kind="uniform_random", P=P, hi=9, seed=P, sparsify=4)
        for f in ("twophase", "om", "tuna"):
            add(f"odd-P{P}-{f}-r{r}", f, cg, 2, r=r, b=3, layout=1)
    for P, n, r in ((12, 4, 2), (12, 3, 3), (27, 9, 3), (16, 8, 3), (16, 16, 4)):
        cg = dict(kind="uniform_random", P=P, hi=9, seed=P, sparsify=5)
        add(f"odd-P{P}-n{n}-ttpl-r{r}", "ttpl", cg, 2, r=r, n=n, bblock=2, layout=1)
        add(f"odd-P{P}-n{n}-ttpl_s1-r{r}", "ttpl_s1", cg, 2, r=r, n=n, bblock=5, layout=1)
    zz = dict(kind="zeros", P=8)
    for f in ("twophase", "om", "tuna"):
        add(f"zeros-{f}", f, zz, 4, r=2, b=1)
    add("zeros-ttpl", "ttpl", zz, 4, r=2, n=4)
    add("zeros-ttpl_s1", "ttpl_s1", zz, 4, r=2, n=4)
    # the reference's own input matrices (examples/MLinputs_example.cpp: MPI_CHAR, packed displacements), scaled down
    for P, div, r in ((4, 65536, 2), (8, 65536, 2), (16, 32768, 4), (32, 16384, 2), (64, 16384, 8), (128, 16384, 12)):
        ml = dict(kind="ml", P=P, divide=div)
        add(f"ml-P{P}-twophase-r{r}", "twophase", ml, 1, r=r)
        add(f"ml-P{P}-tuna-r{r}", "tuna", ml, 1, r=r, b=0)
    add("ml-P64-ttpl-n8", "ttpl", dict(kind="ml", P=64, divide=16384), 1, r=4, n=8)
    add("ml-P128-ttpl_s1-n32", "ttpl_s1", dict(kind="ml", P=128, divide=16384), 1, r=32, n=32)
    # TuNA2 with b = 1 (the reference reuses its send buffer under in-flight sends for b > 1, src/tuna2.cpp:175-185)
    for P, r in ((8, 2), (12, 3), (27, 3), (32, 4), (64, 8)):
        add(f"tuna2-P{P}-r{r}", "tuna2", dict(kind="uniform_random", P=P, hi=40, seed=P + 9, sparsify=4), 2, r=r, b=1, layout=1)
    # linear comparators
    for P in (8, 12, 32):
        cg = dict(kind="uniform_random", P=P, hi=30, seed=P + 5, sparsify=4)
        for f in ("scattered", "ompi_linear", "ompi_pairwise", "spreadout") + (("xor",) if P & (P - 1) == 0 else ()):
            add(f"cmp-P{P}-{f}", f, cg, 4, bblock=3, layout=1)
    # linear two-layer comparators
    for P, n in ((8, 4), (12, 3), (32, 8)):
        cg = dict(kind="uniform_random", P=P, hi=30, seed=P + 7, sparsify=4)
        add(f"tl-linear-P{P}-n{n}", "tl_linear", cg, 4, n=n, layout=1)
        add(f"tl-linear-s2-P{P}-n{n}", "tl_linear_s2", cg, 4, n=n, b=2, bblock=5, layout=1)
    # TTPL_rbruck_alltoallv: the reference delivers only the blocks that stay inside a node ("scope": "node")
    for P, n, r in ((8, 4, 2), (12, 4, 2), (12, 3, 3), (27, 9, 3), (32, 4, 2), (64, 8, 4)):
        cg = dict(kind="uniform_random", P=P, hi=30, seed=P + 11, sparsify=4)
        add(f"ttpl-rbruck-P{P}-n{n}-r{r}", "ttpl_rbruck", cg, 2, r=r, n=n, layout=1)
    # the benchmark configurations at their REAL rank counts, with small blocks (minutes of mpiexec each)
    add("C3p-twophase-r16", "twophase", dict(kind="zipf", P=256, max=512, seed=0), 4, r=16)
    add("C3p-tuna-r16", "tuna", dict(kind="zipf", P=256, max=512, seed=0), 4, r=16, b=0)
    c4p = dict(kind="normal", P=1024, mean=64.0, sd=16.0, hi=256, seed=0)
    add("C4p-ttpl", "ttpl", c4p, 1, r=32, n=32, bblock=0)
    add("C4p-ttpl_s1", "ttpl_s1", c4p, 1, r=32, n=32, bblock=0)
    add("C5p-tuna-r32", "tuna", dict(kind="fft", P=512, row_len=32, count=8), 8, r=32, b=0)
    # uniform two-layer functions
    for P, n, r in ((16, 4, 2), (16, 4, 3), (16, 4, 4), (12, 3, 2), (64, 8, 4), (64, 16, 3)):
        add(f"uni-spread-P{P}-n{n}-r{r}", "uniform_spreadout", None, 4, r=r, n=n, count=5)
        add(f"uni-isplit-P{P}-n{n}-r{r}", "uniform_isplit", None, 4, r=r, n=n, count=5)
    return out


def run_case(case: dict, tmp: str) -> dict:
    uniform = case["func"].startswith("uniform")
    if uniform:
        P = int(case["id"].split("-P")[1].split("-")[0])
        counts_arg = str(case["count"])
    else:
        counts = counts_for(case["counts"])
        P = counts.shape[0]
        counts_arg = os.path.join(tmp, "counts.bin")
        counts.astype("<i4").tofile(counts_arg)
    outp = os.path.join(tmp, "out")
    cmd = [MPIEXEC, "-n", str(P), DRIVER, case["func"], counts_arg, str(case["esz"]), str(case["r"]), str(case["b"]),
           str(case["n"]), str(case["bblock"]), str(case["layout"]), str(case["payload"]), str(case["seed"]), "1", outp]
    res = subprocess.run(cmd, capture_output=True, text=True, timeout=1800)
    line = res.stdout.strip().splitlines()[-1] if res.stdout.strip() else ""
    if res.returncode != 0:
        raise RuntimeError(f"{case['id']}: reference run failed ({res.returncode}): {line} {res.stderr[-400:]}")
    digests = open(outp + ".digests").read().split()
    rec = dict(case)
    rec["P"] = P
    rec["digests"] = digests
    if case["func"] == "ttpl_rbruck":
        rec["scope"] = "node"
    rec["reference_says"] = line
    if case["id"] == "C1-twophase":
        os.replace(outp + ".recv.bin", os.path.join(HERE, "c1_recv.bin"))
    return rec


def main() -> None:
    """Without arguments every case is run again; `--only TEXT` runs the cases whose id contains TEXT and replaces just
    those in the existing golden.json."""
    if not os.path.exists(DRIVER):
        raise SystemExit("build the reference driver first: make -C oracle ref")
    only = sys.argv[sys.argv.index("--only") + 1] if "--only" in sys.argv else None
    path = os.path.join(HERE, "golden.json")
    todo = [c for c in cases() if only is None or only in c["id"]]
    recs = []
    with tempfile.TemporaryDirectory() as tmp:
        for case in todo:
            rec = run_case(case, tmp)
            print(rec["id"], rec["reference_says"], flush=True)
            recs.append(rec)
    if only is not None:
        new = {r["id"]: r for r in recs}
        old = json.load(open(path))["cases"]
        order = [c["id"] for c in cases()]
        merged = {r["id"]: r for r in old}
        merged.update(new)
        recs = [merged[i] for i in order if i in merged]
    with open(path, "w") as f:
        json.dump({"made_by": "tests/golden/make_golden.py", "mpi": "MPICH 3.3.2 (/opt/conda), mpiexec -n P, oversubscribed on 8 cores",
                   "cases": recs}, f, indent=1)
    print(f"{len(recs)} cases written")


if __name__ == "__main__":
    main()
