"""Pins the CPU oracle against what the REAL reference produced (tests/golden/golden.json, written by
tests/golden/make_golden.py from `mpiexec -n P` runs of the reference's own functions)."""
import os

import numpy as np
import pytest

from oracle import oracle_py as O
from rbruck_alltoallv_amd import workloads as W
from tests.helpers import GOLDEN_DIR, digest_problem, fnv1a64_blocks, load_golden, problem_for_case, run_on

CASES = load_golden()


@pytest.mark.parametrize("case", CASES, ids=[c["id"] for c in CASES])
def test_oracle_matches_reference_digests(case):
    prob = problem_for_case(case)
    send = W.fill_send_arena(prob, case["payload"], case["seed"])
    recv = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
    assert run_on(O, case, prob, send.copy(), recv) == 0
    got = [f"{int(h):016x}" for h in O.digest_recv(digest_problem(case, prob), recv)]
    assert got == case["digests"]


def test_digest_restatement_agrees():
    """The C digest and its numpy restatement agree, so a digest mismatch can only mean different bytes."""
    case = next(c for c in CASES if c["id"] == "odd-P12-tuna-r3")
    prob = problem_for_case(case)
    send = W.fill_send_arena(prob, case["payload"], case["seed"])
    recv = W.expected_recv_arena(prob, send)
    assert fnv1a64_blocks(prob, recv) == [f"{int(h):016x}" for h in O.digest_recv(prob, recv)] == case["digests"]


def test_c1_every_byte_of_every_recvbuf():
    """Benchmark configuration 1 (P=8, r=2, int32, counts U{0..64} from seed 0, word = src*2^20 + dst*2^10 + idx):
    the reference's complete receive buffers, byte for byte."""
    case = next(c for c in CASES if c["id"] == "C1-twophase")
    prob = problem_for_case(case)
    ref = np.fromfile(os.path.join(GOLDEN_DIR, "c1_recv.bin"), dtype=np.uint8)
    send = W.fill_send_arena(prob, W.PAYLOAD_SELFDESC32, case["seed"])
    recv = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
    assert O.twophase_rbruck_alltoallv(2, prob, send, recv) == 0
    # the driver dumped each rank's extent back to back (no alignment padding between ranks)
    ext = (prob.recvcounts.astype(np.int64).sum(axis=1)) * prob.esz
    off = 0
    for t in range(prob.P):
        mine = recv[int(prob.rbase[t]):int(prob.rbase[t]) + int(ext[t])]
        assert np.array_equal(mine, ref[off:off + int(ext[t])]), f"rank {t}"
        words = mine.view("<u4")
        # self-describing payload: destination field says t everywhere, sources ascend
        assert np.all((words >> 10) & 0x3FF == t)
        assert np.all(np.diff((words >> 20).astype(np.int64)) >= 0)
        off += int(ext[t])
    assert off == ref.size
