"""Shared by the CPU and GPU tests: rebuild a golden case's inputs and run one function on the oracle."""
from __future__ import annotations

import dataclasses
import json
import os

import numpy as np

from rbruck_alltoallv_amd import workloads as W

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN_DIR = os.path.join(ROOT, "tests", "golden")
INPUTS_DIR = os.path.join(GOLDEN_DIR, "inputs")


def load_golden() -> list[dict]:
    with open(os.path.join(GOLDEN_DIR, "golden.json")) as f:
        return json.load(f)["cases"]


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


def problem_for_case(case: dict) -> W.Problem:
    """The inputs tests/golden/make_golden.py gave the reference for this case."""
    if case["func"].startswith("uniform"):
        return W.make_uniform_problem(case["P"], case["count"], case["esz"])
    counts = counts_for(case["counts"])
    recv_layout = 0 if case["func"] == "ttpl" else case["layout"]
    return W.make_problem(counts, case["esz"], case["layout"], recv_layout)


def digest_problem(case: dict, prob: W.Problem) -> W.Problem:
    """The blocks a case's digests cover: all of them, or ("scope": "node") only those whose source is on the
    receiver's node — what the reference's TTPL_rbruck_alltoallv delivers."""
    if case.get("scope") != "node":
        return prob
    node = np.arange(prob.P) // case["n"]
    keep = node[:, None] == node[None, :]
    return dataclasses.replace(prob, recvcounts=np.ascontiguousarray(np.where(keep, prob.recvcounts, 0).astype(np.int32)))


def run_on(backend, case: dict, prob: W.Problem, send, recv) -> int:
    """Dispatch one golden case to a backend exposing the reference's function names
    (oracle.oracle_py on numpy arenas, or the GPU package on device arenas)."""
    f = case["func"]
    if f == "twophase":
        return backend.twophase_rbruck_alltoallv(case["r"], prob, send, recv)
    if f == "om":
        return backend.twophase_rbruck_alltoallv_om(case["r"], prob, send, recv)
    if f == "tuna":
        return backend.tuna_algorithm(case["r"], case["b"], prob, send, recv)
    if f == "tuna2":
        return backend.tuna2_algorithm(case["r"], case["b"], prob, send, recv)
    if f == "ttpl":
        return backend.TTPL_BT_alltoallv(case["n"], case["r"], case["bblock"], prob, send, recv)
    if f == "ttpl_s1":
        return backend.TTPL_BT_alltoallv_s1(case["n"], case["r"], case["bblock"], prob, send, recv)
    if f == "uniform_spreadout":
        return backend.uniform_spreadout_twolayer(case["n"], case["r"], prob, case["count"], send, recv)
    if f == "uniform_isplit":
        return backend.uniform_inverse_isplit_r_bruck(case["n"], case["r"], case["b"], prob, case["count"], send, recv)
    if f == "scattered":
        return backend.MPICH_intra_scattered(case["bblock"], prob, send, recv)
    if f == "ompi_linear":
        return backend.ompi_alltoallv_intra_basic_linear(prob, send, recv)
    if f == "ompi_pairwise":
        return backend.ompi_alltoallv_intra_pairwise(prob, send, recv)
    if f == "xor":
        return backend.exclisive_or_alltoallv(prob, send, recv)
    if f == "ttpl_rbruck":
        return backend.TTPL_rbruck_alltoallv(case["n"], case["r"], prob, send, recv)
    if f == "tl_linear":
        return backend.twolayer_communicator_linear(case["n"], prob, send, recv)
    if f == "tl_linear_s2":
        return backend.twolayer_communicator_linear_s2(case["n"], case["b"], case["bblock"], prob, send, recv)
    if f == "spreadout":
        return backend.spreadout_alltoallv(prob, send, recv)
    raise ValueError(f)


def fnv1a64_blocks(prob: W.Problem, recv: np.ndarray) -> list[str]:
    """Per-rank FNV-1a 64 over the receive blocks in source order (numpy restatement of the digest the
    MPI driver around the reference wrote)."""
    out = []
    for t in range(prob.P):
        h = 0xCBF29CE484222325
        for s in range(prob.P):
            nb = int(prob.recvcounts[t, s]) * prob.esz
            at = int(prob.rbase[t]) + int(prob.rdispls[t, s]) * prob.esz
            for byte in recv[at:at + nb].tolist():
                h = ((h ^ byte) * 0x100000001B3) & 0xFFFFFFFFFFFFFFFF
        out.append(f"{h:016x}")
    return out


COLLECTIVES = ("twophase_rbruck_alltoallv", "twophase_rbruck_alltoallv_om", "tuna_algorithm", "tuna2_algorithm", "TTPL_BT_alltoallv",
               "TTPL_BT_alltoallv_s1", "TTPL_rbruck_alltoallv", "uniform_spreadout_twolayer", "uniform_inverse_isplit_r_bruck",
               "MPICH_intra_scattered", "ompi_alltoallv_intra_basic_linear", "ompi_alltoallv_intra_pairwise", "exclisive_or_alltoallv",
               "spreadout_alltoallv", "twolayer_communicator_linear", "twolayer_communicator_linear_s2")


class CalledTwice:
    """The package's API with every collective called twice.  In the library's default mode (vc_comm_set_forwarding 1) the
    first call on a communicator goes through the work-item list and leaves the hint by which the next one picks its
    kernel (listless, batched, fixed-stride staging): a test that makes one call per communicator would never reach those.
    The receive arena is put back to what it held before the first call, the second call runs on the hint of the first,
    and both must leave the same bytes; the test's own checks then see the second call's result."""

    def __init__(self, module):
        self._module = module

    def __getattr__(self, name):
        fn = getattr(self._module, name)
        if name not in COLLECTIVES:
            return fn

        def twice(*args):
            import torch
            recv = args[-1]
            small = recv.numel() <= (1 << 28)
            before = recv.clone() if small else None
            rc = fn(*args)
            if rc != 0:
                return rc
            first = recv.clone() if small else None
            if small:
                recv.copy_(before)
            rc = fn(*args)
            assert rc == 0, "the second call failed where the first one passed"
            if small:
                assert torch.equal(first, recv), "the second call on a communicator left other bytes than the first"
            return rc
        return twice
