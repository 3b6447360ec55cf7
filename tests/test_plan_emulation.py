"""Host logic of the product without a GPU: the schedule builder (csrc/vc_sched.h) and the per-entry plan
arithmetic (csrc/vc_plan_math.h) compiled for the CPU (tests/plan_emulator.cpp), checked against the reference's
golden digests, the textbook alltoallv and the oracle's message trace (the route)."""
import numpy as np
import pytest

from oracle import oracle_py as O
from rbruck_alltoallv_amd import workloads as W
from tests import emulator as E
from tests.helpers import digest_problem, load_golden, problem_for_case, run_on

CASES = load_golden()


@pytest.mark.parametrize("case", CASES, ids=[c["id"] for c in CASES])
def test_plan_reproduces_reference_digests(case):
    prob = problem_for_case(case)
    send = W.fill_send_arena(prob, case["payload"], case["seed"])
    recv = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
    keep = send.copy()
    assert run_on(E, case, prob, send, recv) == 0
    assert E.last.errors == 0
    assert [f"{int(h):016x}" for h in O.digest_recv(digest_problem(case, prob), recv)] == case["digests"]
    assert np.array_equal(recv, W.expected_recv_arena(prob, send))       # gaps between blocks stay untouched
    assert np.array_equal(send, keep)


def _prob(P, layout, esz, seed, recv_layout=None):
    counts = W.counts_uniform_random(P, 9, seed=seed)
    counts[counts % 4 == 0] = 0
    return W.make_problem(counts, esz, layout, layout if recv_layout is None else recv_layout)


@pytest.mark.parametrize("P", [1, 2, 3, 4, 5, 6, 7, 8, 9, 12, 16, 17, 27, 32, 50])
def test_flat_plans_all_radices(P):
    for layout in (0, 1):
        for esz in (1, 4):
            prob = _prob(P, layout, esz, seed=P)
            send = W.fill_send_arena(prob, 0, 5)
            want = W.expected_recv_arena(prob, send)
            for r in sorted({2, 3, 4, 5, 8, P, P + 3, max(2, P - 1)} - {1}):
                for name, fn in (("twophase", lambda d: E.twophase_rbruck_alltoallv(r, prob, send, d)),
                                 ("om", lambda d: E.twophase_rbruck_alltoallv_om(r, prob, send, d)),
                                 ("tuna1", lambda d: E.tuna_algorithm(r, 1, prob, send, d)),
                                 ("tuna3", lambda d: E.tuna_algorithm(r, 3, prob, send, d)),
                                 ("tunaP", lambda d: E.tuna_algorithm(r, 0, prob, send, d)),
                                 ("tuna2", lambda d: E.tuna2_algorithm(r, 2, prob, send, d))):
                    recv = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
                    rc = fn(recv)
                    if name.startswith("tuna") and P < 3:
                        assert rc == -3
                        continue
                    assert rc == 0 and E.last.errors == 0, (name, P, layout, esz, r, rc)
                    assert np.array_equal(recv, want), (name, P, layout, esz, r)


@pytest.mark.parametrize("P,n", [(4, 2), (6, 2), (6, 3), (8, 2), (8, 4), (9, 3), (12, 4), (16, 8), (32, 8), (8, 8), (8, 1), (27, 9)])
def test_twolayer_plans(P, n):
    for layout in (0, 1):
        for esz in (1, 8):
            for r in sorted({2, 3, 4, n, n + 1} - {1}):
                for bblock in (0, 1, 3):
                    for name, fn in (("ttpl", E.TTPL_BT_alltoallv), ("s1", E.TTPL_BT_alltoallv_s1)):
                        prob = _prob(P, layout, esz, seed=P + 100, recv_layout=0 if name == "ttpl" else layout)
                        send = W.fill_send_arena(prob, 0, 5)
                        recv = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
                        assert fn(n, r, bblock, prob, send, recv) == 0, (name, layout, esz, r, bblock)
                        assert np.array_equal(recv, W.expected_recv_arena(prob, send)), (name, layout, esz, r, bblock)


def test_error_codes_match_the_oracle():
    prob = _prob(8, 0, 4, seed=3)
    send = W.fill_send_arena(prob, 0, 1)
    recv = np.zeros(prob.recv_bytes, dtype=np.uint8)
    for backend in (E, O):
        for r in (0, 1, -5):
            assert backend.twophase_rbruck_alltoallv(r, prob, send, recv) == -1
            assert backend.twophase_rbruck_alltoallv_om(r, prob, send, recv) == -1
            assert backend.TTPL_BT_alltoallv(4, r, 0, prob, send, recv) == -1
            assert backend.TTPL_BT_alltoallv_s1(4, r, 0, prob, send, recv) == -1
            assert backend.tuna_algorithm(r, 1, prob, send, recv) == 0
        assert backend.TTPL_BT_alltoallv(3, 2, 0, prob, send, recv) == -2
        assert backend.TTPL_BT_alltoallv_s1(5, 2, 0, prob, send, recv) == -2
        up = W.make_uniform_problem(8, 2, 4)
        us = W.fill_send_arena(up, 0, 1)
        ur = np.zeros(up.recv_bytes, dtype=np.uint8)
        assert backend.uniform_spreadout_twolayer(4, 1, up, 2, us.copy(), ur) == -1
        assert backend.uniform_spreadout_twolayer(8, 2, up, 2, us.copy(), ur) == -2
        assert backend.uniform_spreadout_twolayer(3, 2, up, 2, us.copy(), ur) == -2
        assert backend.uniform_inverse_isplit_r_bruck(8, 2, 2, up, 2, us.copy(), ur) == -2
    p2 = _prob(2, 0, 1, seed=1)
    s2 = W.fill_send_arena(p2, 0, 1)
    r2 = np.zeros(p2.recv_bytes, dtype=np.uint8)
    assert E.tuna_algorithm(2, 1, p2, s2, r2) == O.tuna_algorithm(2, 1, p2, s2, r2) == -3


def _oracle_traffic(rec, P, select):
    m = np.zeros((P, P), dtype=np.int64)
    for t in rec[select]:
        m[int(t["src"]), int(t["dst"])] += int(t["bytes"])
    return m


@pytest.mark.parametrize("P,r", [(8, 2), (12, 3), (17, 5), (27, 3), (64, 4), (49, 7), (30, 29)])
@pytest.mark.parametrize("func", ["twophase", "om", "tuna"])
def test_route_equals_the_oracles_message_trace(P, r, func):
    """Per digit phase, the bytes every rank sends to every other rank are those of the reference's rounds of
    that digit — the plan really walks the Bruck route instead of gathering in one pass."""
    counts = W.counts_uniform_random(P, 20, seed=P * 7 + r)
    counts[counts % 3 == 0] = 0
    prob = W.make_problem(counts, 2, 0, 0)
    send = W.fill_send_arena(prob, 0, 2)
    recv = np.zeros(prob.recv_bytes, dtype=np.uint8)
    ofn = {"twophase": lambda: O.twophase_rbruck_alltoallv(r, prob, send, recv),
           "om": lambda: O.twophase_rbruck_alltoallv_om(r, prob, send, recv),
           "tuna": lambda: O.tuna_algorithm(r, 0, prob, send, recv)}[func]
    with O.trace() as t:
        assert ofn() == 0
    rec = t.records
    efn = {"twophase": lambda: E.twophase_rbruck_alltoallv(r, prob, send, recv),
           "om": lambda: E.twophase_rbruck_alltoallv_om(r, prob, send, recv),
           "tuna": lambda: E.tuna_algorithm(r, 0, prob, send, recv)}[func]
    assert efn() == 0
    res = E.last
    digits = list(dict.fromkeys(rec[rec["kind"] != 4]["digit"].tolist()))      # order the oracle visited them
    assert res.nlaunch == len(digits)
    for k, x in enumerate(digits):
        want = _oracle_traffic(rec, P, (rec["digit"] == x) & (rec["kind"] != 4))
        if k == 0:
            want += _oracle_traffic(rec, P, rec["kind"] == 4)                  # self copies ride in the first launch
        assert np.array_equal(res.traffic[k], want), (func, x)
    assert res.moved * 2 == W.algorithmic_bytes(prob.sendcounts, prob.esz, W.hops_flat(P, min(r, P - 1) if func == "tuna" else min(r, P)))


@pytest.mark.parametrize("P,n,r", [(8, 4, 2), (12, 4, 2), (27, 9, 3), (64, 16, 4), (64, 32, 32), (16, 8, 3)])
def test_twolayer_route_equals_the_oracles_trace(P, n, r):
    counts = W.counts_uniform_random(P, 20, seed=P + n + r)
    counts[counts % 3 == 0] = 0
    prob = W.make_problem(counts, 1, 0, 0)
    send = W.fill_send_arena(prob, 0, 2)
    recv = np.zeros(prob.recv_bytes, dtype=np.uint8)
    with O.trace() as t:
        assert O.TTPL_BT_alltoallv_s1(n, r, 0, prob, send, recv) == 0
    rec = t.records
    assert E.TTPL_BT_alltoallv_s1(n, r, 0, prob, send, recv) == 0
    res = E.last
    digits = list(dict.fromkeys(rec[rec["kind"] == 0]["digit"].tolist()))
    assert res.nlaunch == len(digits) + (1 if P > n else 0)
    for k, x in enumerate(digits):
        got = res.traffic[k].copy()
        if k == 0:
            got[np.arange(P), np.arange(P)] = 0                                  # self copies
        # the staggered reference sends own-node finals inside the intra rounds too: identical matrices
        assert np.array_equal(got, _oracle_traffic(rec, P, (rec["digit"] == x) & (rec["kind"] == 0))), x
    if P > n:
        assert np.array_equal(res.traffic[len(digits)], _oracle_traffic(rec, P, rec["kind"] == 3))
    assert res.moved * 2 == W.algorithmic_bytes(prob.sendcounts, prob.esz, W.hops_twolayer(P, n, r))


def _digits(v, r):
    out = []
    while v:
        out.append(v % r)
        v //= r
    return out


@pytest.mark.parametrize("P,n,r", [(8, 4, 2), (12, 4, 2), (12, 3, 3), (27, 3, 3), (64, 4, 2), (64, 16, 4), (60, 3, 3), (16, 1, 2),
                                   (8, 8, 2), (40, 4, 5), (49, 7, 2)])
def test_twolayer_bruck_route_equals_the_oracles_trace(P, n, r):
    """TTPL_rbruck_alltoallv: the intra-node launches carry the reference's intra-node rounds
    (src/twophase_twolayer_rbruck.cpp:88-168); every launch of the inter-node Bruck carries the messages of the
    rounds of one digit of the group offset (:179-227: same rank pairs; bytes = the blocks of the group slots the
    reference packs), and a block rides in as many inter-node launches as its group offset has non-zero digits."""
    counts = W.counts_uniform_random(P, 20, seed=P + n + r)
    counts[counts % 3 == 0] = 0
    for layout in (0, 1):
        prob = W.make_problem(counts, 1, layout, layout)
        send = W.fill_send_arena(prob, 0, 2)
        want = W.expected_recv_arena(prob, send)
        recv = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
        with O.trace() as t:
            assert O.TTPL_rbruck_alltoallv(n, r, prob, send, recv) == 0
        assert np.array_equal(recv, want)
        rec = t.records
        recv[:] = 0xEE
        assert E.TTPL_rbruck_alltoallv(n, r, prob, send, recv) == 0
        res = E.last
        assert res.errors == 0 and np.array_equal(recv, want)
        intra = list(dict.fromkeys(rec[rec["kind"] == 0]["digit"].tolist()))
        inter = list(dict.fromkeys(rec[rec["kind"] == 6]["digit"].tolist()))
        assert res.nlaunch == max(len(intra), 1) + len(inter)
        for k, x in enumerate(intra):
            got = res.traffic[k].copy()
            if k == 0:
                got[np.arange(P), np.arange(P)] = 0                              # self copies
            assert np.array_equal(got, _oracle_traffic(rec, P, (rec["digit"] == x) & (rec["kind"] == 0))), x
        G, reff = P // n, max(min(r, n), 2)
        for k, x in enumerate(inter):
            got = res.traffic[max(len(intra), 1) + k]
            assert np.array_equal(got, _oracle_traffic(rec, P, (rec["digit"] == x) & (rec["kind"] == 6))), x
            src, dst = np.nonzero(got)
            assert np.all(src % n == dst % n)                                    # equal local index (:210-211)
            hop = (src // n - dst // n) % G
            assert np.all((hop % reff ** x == 0) & (hop // reff ** x < reff) & (hop > 0))
        # hops per block: one per non-zero digit of the local offset and of the group offset
        s_idx, t_idx = np.meshgrid(np.arange(P), np.arange(P), indexing="ij")
        nnz = np.vectorize(lambda v: sum(1 for dgt in _digits(int(v), reff) if dgt))
        hops = nnz((s_idx % n - t_idx % n) % n) + nnz((s_idx // n - t_idx // n) % G)
        hops[np.arange(P), np.arange(P)] = 1
        assert res.moved == int((prob.sendcounts.astype(np.int64) * hops).sum()) * prob.esz


@pytest.mark.parametrize("esz", [3, 5, 12, 24])
def test_element_sizes_that_are_no_power_of_two(esz):
    """The reference multiplies counts and displacements by MPI_Type_size (src/twophase_tunable_rbruckv.cpp:28, 63); any
    contiguous type size must work."""
    counts = W.counts_uniform_random(12, 700, seed=esz)
    counts[counts % 3 == 0] = 0
    prob = W.make_problem(counts, esz, 1, 1)
    send = W.fill_send_arena(prob, 0, 3)
    want = W.expected_recv_arena(prob, send)
    for forward in (False, True):
        for func, kw in ((E.F_TWOPHASE, dict(r=3)), (E.F_TUNA, dict(r=2)), (E.F_TTPL_S1, dict(n=4, r=2)), (E.F_TTPL_RBRUCK, dict(n=3, r=2))):
            recv = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
            res = E.emulate(func, prob, send, recv, forward=forward, **kw)
            assert res.rc == 0 and res.errors == 0, (esz, func, forward)
            assert np.array_equal(recv, want)
            ref = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
            assert O.twophase_rbruck_alltoallv(3, prob, send, ref) == 0 and np.array_equal(ref, want)


def test_twolayer_bruck_error_codes():
    prob = W.make_problem(W.counts_uniform_random(12, 5, seed=1), 1, 0, 0)
    send = W.fill_send_arena(prob, 0, 2)
    recv = np.zeros(prob.recv_bytes, dtype=np.uint8)
    for backend in (O, E):
        assert backend.TTPL_rbruck_alltoallv(4, 1, prob, send, recv) == -1         # src/twophase_twolayer_rbruck.cpp:20
        assert backend.TTPL_rbruck_alltoallv(5, 2, prob, send, recv) == -2
        assert backend.TTPL_rbruck_alltoallv(0, 2, prob, send, recv) == -2


def test_large_blocks_split_into_pieces():
    P = 12
    counts = (W.counts_uniform_random(P, 70000, seed=11) * (W.counts_uniform_random(P, 3, seed=12) > 0)).astype(np.int32)
    for layout in (0, 1):
        prob = W.make_problem(counts, 1, layout, layout)
        send = W.fill_send_arena(prob, 0, 9)
        want = W.expected_recv_arena(prob, send)
        for fn in (lambda d: E.twophase_rbruck_alltoallv(3, prob, send, d), lambda d: E.tuna_algorithm(4, 2, prob, send, d),
                   lambda d: E.TTPL_BT_alltoallv_s1(4, 2, 3, prob, send, d)):
            recv = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
            assert fn(recv) == 0 and E.last.errors == 0
            assert np.array_equal(recv, want)
            assert E.last.items > P * P          # pieces, not blocks


@pytest.mark.parametrize("P", [1, 2, 5, 8, 12, 32])
def test_linear_comparator_plans(P):
    for layout in (0, 1):
        counts = W.counts_uniform_random(P, 30, seed=P + 40)
        counts[counts % 4 == 0] = 0
        prob = W.make_problem(counts, 2, layout, layout)
        send = W.fill_send_arena(prob, 0, 3)
        want = W.expected_recv_arena(prob, send)
        for name, fn, launches in (("spreadout", lambda d: E.spreadout_alltoallv(prob, send, d), 1),
                                   ("linear", lambda d: E.ompi_alltoallv_intra_basic_linear(prob, send, d), 1),
                                   ("pairwise", lambda d: E.ompi_alltoallv_intra_pairwise(prob, send, d), 1),
                                   ("xor", lambda d: E.exclisive_or_alltoallv(prob, send, d), 1),
                                   ("scattered3", lambda d: E.MPICH_intra_scattered(3, prob, send, d), -(-P // 3)),
                                   ("scattered0", lambda d: E.MPICH_intra_scattered(0, prob, send, d), 1)):
            recv = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
            rc = fn(recv)
            if name == "xor" and P & (P - 1):
                assert rc == -1
                continue
            assert rc == 0 and E.last.errors == 0, (name, P)
            assert np.array_equal(recv, want), (name, P, layout)
            assert E.last.nlaunch == launches
            assert E.last.moved == prob.payload_bytes            # one hop per block
            if name == "scattered3":
                # launch k carries the rank distances 3k .. 3k+2, like the reference's batches (MPICH_scattered.cpp:38-45)
                for k in range(E.last.nlaunch):
                    src, dst = np.nonzero(E.last.traffic[k])
                    assert np.all(((src - dst) % P >= 3 * k) & ((src - dst) % P < 3 * k + 3))


@pytest.mark.parametrize("P,n", [(4, 2), (8, 4), (12, 3), (12, 4), (32, 8), (16, 1), (27, 9)])
def test_linear_twolayer_comparator_plans(P, n):
    """twolayer_communicator_linear / _s2 (src/twolayer_communicator_linear.cpp:13-88, 92-192): launches inside the
    nodes first, then between them; each launch carries the messages of one of the reference's Waitall batches."""
    G = P // n
    node = np.arange(P) // n
    same = node[:, None] == node[None, :]
    for layout in (0, 1):
        counts = W.counts_uniform_random(P, 30, seed=P + n)
        counts[counts % 4 == 0] = 0
        prob = W.make_problem(counts, 2, layout, layout)
        send = W.fill_send_arena(prob, 0, 3)
        want = W.expected_recv_arena(prob, send)
        for b1, b2 in ((None, None), (0, 0), (1, 1), (2, 5), (3, P + 4)):
            recv = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
            if b1 is None:
                rc = E.twolayer_communicator_linear(n, prob, send, recv)
                e1, e2 = n, P
            else:
                rc = E.twolayer_communicator_linear_s2(n, b1, b2, prob, send, recv)
                e1 = n if b1 <= 0 or b1 > n else b1
                e2 = P if b2 <= 0 or b2 > P else b2
            assert rc == 0 and E.last.errors == 0, (P, n, b1, b2)
            assert np.array_equal(recv, want), (P, n, layout, b1, b2)
            assert E.last.moved == prob.payload_bytes and E.last.stage_bytes == 0
            n_intra = -(-n // e1)
            first = n if b1 is None else 1
            n_inter = -(-(P - first) // e2)
            assert E.last.nlaunch == n_intra + n_inter
            for k in range(E.last.nlaunch):
                src, dst = np.nonzero(E.last.traffic[k])
                if k < n_intra:
                    assert np.all(same[src, dst])
                    d = (src % n - dst % n) % n
                    assert np.all((d >= k * e1) & (d < (k + 1) * e1))
                else:
                    assert not np.any(same[src, dst])
                    q = ((dst // n - src // n) % G) * n + src % n          # ii of the receiver's loop (:150-156)
                    lo = first + (k - n_intra) * e2
                    assert np.all((q >= lo) & (q < lo + e2))
    # group size that is no proper divisor of P
    recv = np.zeros(prob.recv_bytes, dtype=np.uint8)
    for bad in (0, P, P + 1, 5 if P % 5 else 7):
        assert E.twolayer_communicator_linear(bad, prob, send, recv) == -2
        assert E.twolayer_communicator_linear_s2(bad, 1, 1, prob, send, recv) == -2
        assert O.twolayer_communicator_linear(bad, prob, send, recv) == -2
        assert O.twolayer_communicator_linear_s2(bad, 1, 1, prob, send, recv) == -2


@pytest.mark.parametrize("P,n,r,bblock", [(8, 4, 4, 0), (12, 4, 2, 2), (27, 9, 3, 0), (64, 16, 16, 3), (64, 32, 32, 0), (16, 2, 2, 0)])
def test_coalesced_twolayer_route(P, n, r, bblock):
    """TTPL_BT_alltoallv: intra-node launches as in the staggered variant; every inter-node message is the coalesced
    one of the reference (src/twophase_twolayer_rbruck.cpp:430-453) — same rank pairs, same bytes — and is copied in
    at most three contiguous parts instead of n blocks."""
    counts = W.counts_uniform_random(P, 300, seed=P + n + r)
    counts[counts % 3 == 0] = 0
    prob = W.make_problem(counts, 1, 1, 0)
    send = W.fill_send_arena(prob, 0, 2)
    recv = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
    with O.trace() as t:
        assert O.TTPL_BT_alltoallv(n, r, bblock, prob, send, recv) == 0
    rec = t.records
    want = recv.copy()
    recv[:] = 0xEE
    assert E.TTPL_BT_alltoallv(n, r, bblock, prob, send, recv) == 0 and E.last.errors == 0
    assert np.array_equal(recv, want)
    res = E.last
    G = P // n
    digits = list(dict.fromkeys(rec[rec["kind"] == 0]["digit"].tolist()))
    groups = G if bblock <= 0 or bblock > G else bblock
    n_inter = -(-G // groups)
    assert res.nlaunch == len(digits) + n_inter
    inter = rec[rec["kind"] == 2]
    cross = inter[inter["src"] // n != inter["dst"] // n]          # the reference also sends a message to itself
    got = sum(res.traffic[len(digits) + k] for k in range(n_inter))
    assert np.array_equal(got, _oracle_traffic(cross, P, np.ones(len(cross), dtype=bool)))
    # batches follow the group distance (src/twophase_twolayer_rbruck.cpp:425-447)
    for k in range(n_inter):
        src, dst = np.nonzero(res.traffic[len(digits) + k])
        dist = (src // n - dst // n) % G
        assert np.all((dist >= k * groups) & (dist < (k + 1) * groups))
    assert res.moved * 2 == W.algorithmic_bytes(prob.sendcounts, prob.esz, W.hops_twolayer(P, n, r))


def test_unaligned_recvbuf_pointer_keeps_the_phase_rule():
    """The low bits of the recvbuf pointer enter every staging phase; pieces after the first still start on a
    cache-line boundary of the real destination address."""
    counts = (W.counts_uniform_random(12, 30000, seed=5) * (W.counts_uniform_random(12, 3, seed=6) > 0)).astype(np.int32)
    prob = W.make_problem(counts, 1, 1, 0)
    send = W.fill_send_arena(prob, 0, 9)
    want = W.expected_recv_arena(prob, send)
    for recv_lo in (0, 5, 15, 100, 2048 + 7, 4095):
        for func, kw in ((E.F_TWOPHASE, dict(r=3)), (E.F_TUNA, dict(r=2, batch=1)), (E.F_TTPL, dict(n=4, r=4)),
                         (E.F_TTPL_S1, dict(n=6, r=2, batch=5)), (E.F_SPREADOUT, {})):
            recv = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
            res = E.emulate(func, prob, send, recv, recv_lo=recv_lo, **kw)
            assert res.rc == 0 and res.errors == 0, (func, recv_lo, res.errors)
            assert np.array_equal(recv, want)


# ---- forwarded execution: one work item carries a block piece through all its hops ----

@pytest.fixture
def forwarded():
    E.FORWARD = True
    yield
    E.FORWARD = False


@pytest.mark.parametrize("case", CASES, ids=[c["id"] for c in CASES])
def test_forwarded_plan_reproduces_reference_digests(case, forwarded):
    """The chain items write the same bytes to the same staging slots and receive buffers as the launch-per-digit
    execution (the emulator runs both and compares the arenas), and the result has the reference's digests."""
    prob = problem_for_case(case)
    send = W.fill_send_arena(prob, case["payload"], case["seed"])
    recv = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
    keep = send.copy()
    assert run_on(E, case, prob, send, recv) == 0
    assert E.last.errors == 0
    assert [f"{int(h):016x}" for h in O.digest_recv(digest_problem(case, prob), recv)] == case["digests"]
    assert np.array_equal(recv, W.expected_recv_arena(prob, send))
    assert np.array_equal(send, keep)


@pytest.mark.parametrize("P", [1, 2, 3, 5, 8, 12, 17, 27, 32, 50])
def test_forwarded_flat_plans_all_radices(P, forwarded):
    for layout in (0, 1):
        prob = _prob(P, layout, 2, seed=P + 60)
        send = W.fill_send_arena(prob, 0, 3)
        want = W.expected_recv_arena(prob, send)
        for r in sorted({2, 3, 4, 5, 8, P, P + 3} - {1}):
            calls = [lambda d: E.twophase_rbruck_alltoallv(r, prob, send, d), lambda d: E.twophase_rbruck_alltoallv_om(r, prob, send, d)]
            if P >= 3:
                calls += [lambda d: E.tuna_algorithm(r, 2, prob, send, d), lambda d: E.tuna2_algorithm(r, 0, prob, send, d)]
            for fn in calls:
                recv = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
                assert fn(recv) == 0 and E.last.errors == 0, (P, r)
                assert np.array_equal(recv, want)
                # hops: the chain writes every block once per non-zero digit
                assert E.last.moved * 2 == W.algorithmic_bytes(prob.sendcounts, prob.esz, W.hops_flat(P, min(r, P - 1) if fn in calls[2:] else min(r, P)))


@pytest.mark.parametrize("P,n", [(4, 2), (6, 3), (8, 4), (12, 4), (16, 8), (32, 8), (8, 8), (8, 1), (27, 9), (64, 4)])
def test_forwarded_twolayer_plans(P, n, forwarded):
    for layout in (0, 1):
        prob = _prob(P, layout, 1, seed=P + n, recv_layout=0)
        send = W.fill_send_arena(prob, 0, 3)
        want = W.expected_recv_arena(prob, send)
        for r in sorted({2, 3, max(n, 2)}):
            for fn in (lambda d: E.TTPL_BT_alltoallv(n, r, 3, prob, send, d), lambda d: E.TTPL_BT_alltoallv_s1(n, r, 5, prob, send, d),
                       lambda d: E.TTPL_rbruck_alltoallv(n, r, prob, send, d)):
                recv = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
                assert fn(recv) == 0 and E.last.errors == 0, (P, n, r)
                assert np.array_equal(recv, want)
    if 2 <= n < P:
        up = W.make_uniform_problem(P, 7, 4)
        us = W.fill_send_arena(up, 0, 1)
        uw = W.expected_recv_arena(up, us)
        for fn in (lambda d: E.uniform_spreadout_twolayer(n, 2, up, 7, us.copy(), d), lambda d: E.uniform_inverse_isplit_r_bruck(n, 3, 2, up, 7, us.copy(), d),
                   lambda d: E.twolayer_communicator_linear_s2(n, 2, 5, up, us, d)):
            ur = np.full(up.recv_bytes, 0xEE, dtype=np.uint8)
            assert fn(ur) == 0 and E.last.errors == 0
            assert np.array_equal(ur, uw)


def test_forwarded_large_blocks_and_unaligned_recvbuf(forwarded):
    counts = (W.counts_uniform_random(12, 30000, seed=5) * (W.counts_uniform_random(12, 3, seed=6) > 0)).astype(np.int32)
    prob = W.make_problem(counts, 1, 1, 0)
    send = W.fill_send_arena(prob, 0, 9)
    want = W.expected_recv_arena(prob, send)
    for recv_lo in (0, 5, 100, 2048 + 7, 4095):
        for func, kw in ((E.F_TWOPHASE, dict(r=3)), (E.F_TUNA, dict(r=2, batch=1)), (E.F_TTPL, dict(n=4, r=4)),
                         (E.F_TTPL_S1, dict(n=6, r=2, batch=5)), (E.F_TTPL_RBRUCK, dict(n=2, r=2)), (E.F_SPREADOUT, {})):
            recv = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
            res = E.emulate(func, prob, send, recv, recv_lo=recv_lo, **kw)
            assert res.rc == 0 and res.errors == 0, (func, recv_lo, res.errors)
            assert np.array_equal(recv, want)
            assert res.items > 12 * 12


@pytest.mark.parametrize("name,counts", [
    ("truncated normal", lambda: W.counts_truncated_normal_rows(24, 300.0, 120.0, 700, seed=1)),
    ("power law", lambda: W.counts_power_law_rows(24, 0.8, 900, seed=2)),
    ("sparse blocks", lambda: W.counts_sparse_blocks(24, 0.4, 0.25, 37)),
    ("last block differs", lambda: W.counts_sparse_blocks(24, 0.0, 0.0, 5, last=401))])
def test_distributions_of_the_reference_drivers(name, counts):
    """The count distributions of examples/other_distributions.cpp and examples/FFT_distribution.cpp, 8-byte elements as
    there, through the functions those drivers call — in both execution modes, against the oracle and the definition."""
    c = counts()
    assert c.shape == (24, 24) and c.min() >= 0
    prob = W.make_problem(c, 8, 0, 0)
    send = W.fill_send_arena(prob, 0, 3)
    want = W.expected_recv_arena(prob, send)
    for forward in (False, True):
        for func, kw, ofn in ((E.F_TWOPHASE, dict(r=4), lambda d: O.twophase_rbruck_alltoallv(4, prob, send, d)),
                              (E.F_TTPL_S1, dict(n=6, r=3, batch=4), lambda d: O.TTPL_BT_alltoallv_s1(6, 3, 4, prob, send, d)),
                              (E.F_TTPL, dict(n=4, r=2, batch=0), lambda d: O.TTPL_BT_alltoallv(4, 2, 0, prob, send, d))):
            recv = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
            res = E.emulate(func, prob, send, recv, forward=forward, **kw)
            assert res.rc == 0 and res.errors == 0, (name, func, forward)
            assert np.array_equal(recv, want)
            ref = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
            assert ofn(ref) == 0 and np.array_equal(ref, want)


# ---- fixed-stride staging (the layout calls of short blocks get in the library's default mode) ----

@pytest.fixture
def strided():
    E.FORWARD = True
    E.STRIDED = True
    yield
    E.FORWARD = False
    E.STRIDED = False


@pytest.mark.parametrize("case", [c for c in CASES if c["P"] <= 128], ids=[c["id"] for c in CASES if c["P"] <= 128])
def test_strided_plan_reproduces_reference_digests(case, strided):
    """Slots at the closed-form addresses ((region P + holder) P + slot) x stride: every copy stays inside the arena, no
    two slots overlap, forwarded and launch-per-digit execution agree, and the result has the reference's digests."""
    prob = problem_for_case(case)
    send = W.fill_send_arena(prob, case["payload"], case["seed"])
    recv = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
    assert run_on(E, case, prob, send, recv) == 0
    assert E.last.errors == 0
    assert [f"{int(h):016x}" for h in O.digest_recv(digest_problem(case, prob), recv)] == case["digests"]
    assert np.array_equal(recv, W.expected_recv_arena(prob, send))


@pytest.mark.parametrize("P", [1, 2, 3, 5, 8, 12, 17, 27, 32, 50])
def test_strided_plans_all_radices(P, strided):
    for layout in (0, 1):
        prob = _prob(P, layout, 3, seed=P + 90)
        send = W.fill_send_arena(prob, 0, 3)
        want = W.expected_recv_arena(prob, send)
        for r in sorted({2, 3, 5, P, P + 3} - {1}):
            calls = [lambda d: E.twophase_rbruck_alltoallv(r, prob, send, d), lambda d: E.twophase_rbruck_alltoallv_om(r, prob, send, d)]
            if P >= 3:
                calls += [lambda d: E.tuna_algorithm(r, 2, prob, send, d)]
            for n in [d for d in (1, 2, 3, 4, 8) if P % d == 0]:
                calls += [lambda d, n=n: E.TTPL_BT_alltoallv_s1(n, r, 0, prob, send, d), lambda d, n=n: E.TTPL_rbruck_alltoallv(n, r, prob, send, d)]
            for fn in calls:
                recv = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
                assert fn(recv) == 0 and E.last.errors == 0, (P, r)
                assert np.array_equal(recv, want)


# ---- reused staging (launch-per-digit execution with at least three staging regions) ----

@pytest.mark.parametrize("P,r,func", [(64, 2, "tuna"), (64, 2, "twophase"), (81, 3, "om"), (100, 2, "twophase"), (50, 3, "tuna"),
                                      (64, 4, "om"), (128, 2, "tuna")])
def test_reused_staging_is_smaller_and_stays_below_one_and_a_half_payloads(P, r, func):
    """A sub-region of staging takes the memory of sub-regions whose blocks have all left before it is written.  The
    emulator checks every launch (nothing lands on bytes that still wait for their next hop, every staged byte is read
    exactly once, all have left at the end); here: the arena shrinks and stays below 1.5 x the payload, on all-pairs
    traffic and on the pencil pattern of configuration 5 (rows of a grid)."""
    fn = {"tuna": lambda rec, p, s, d: E.emulate(E.F_TUNA, p, s, d, r=r, recycle=rec),
          "twophase": lambda rec, p, s, d: E.emulate(E.F_TWOPHASE, p, s, d, r=r, recycle=rec),
          "om": lambda rec, p, s, d: E.emulate(E.F_OM, p, s, d, r=r, recycle=rec)}[func]
    for counts in (W.counts_uniform_random(P, 300, seed=P + r), W.counts_fft_rows(P, 8 if P % 8 == 0 else 10 if P % 10 == 0 else 9, 64)):
        prob = W.make_problem(counts, 2, 0, 0)
        send = W.fill_send_arena(prob, 0, 2)
        want = W.expected_recv_arena(prob, send)
        sizes = []
        for rec in (False, True):
            recv = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
            res = fn(rec, prob, send, recv)
            assert res.rc == 0 and res.errors == 0, (P, r, func, rec, res.errors)
            assert np.array_equal(recv, want)
            sizes.append(res.stage_bytes)
        assert sizes[1] <= sizes[0] and (r > 2 or sizes[1] < 0.8 * sizes[0]), sizes
        # sub-regions are placed in pieces (a hole need not hold a whole one): close to what is alive at the worst moment
        assert sizes[1] <= 1.5 * prob.payload_bytes + 128 * P * P, (sizes, prob.payload_bytes)


@pytest.mark.parametrize("P,n,r", [(64, 8, 2), (64, 16, 2), (81, 27, 3), (128, 32, 2), (64, 8, 3)])
def test_reused_staging_twolayer(P, n, r):
    prob = _prob(P, 0, 3, seed=P + n + r, recv_layout=0)
    send = W.fill_send_arena(prob, 0, 3)
    want = W.expected_recv_arena(prob, send)
    for func, kw in ((E.F_TTPL, dict(n=n, r=r, batch=2)), (E.F_TTPL_S1, dict(n=n, r=r, batch=7)), (E.F_TTPL_RBRUCK, dict(n=n, r=r)),
                     (E.F_TUNA, dict(r=r, batch=1))):
        sizes = []
        for rec in (False, True):
            recv = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
            res = E.emulate(func, prob, send, recv, recycle=rec, **kw)
            assert res.rc == 0 and res.errors == 0, (func, rec, res.errors)
            assert np.array_equal(recv, want)
            sizes.append(res.stage_bytes)
        assert sizes[1] <= sizes[0], (func, sizes)
    up = W.make_uniform_problem(P, 5, 4)
    us = W.fill_send_arena(up, 0, 1)
    for func, kw in ((E.F_UNIFORM_SPREADOUT, dict(n=n, r=r, uniform_count=5)), (E.F_UNIFORM_ISPLIT, dict(n=n, r=r, uniform_count=5))):
        ur = np.full(up.recv_bytes, 0xEE, dtype=np.uint8)
        res = E.emulate(func, up, us, ur, recycle=True, **kw)
        assert res.rc == 0 and res.errors == 0, func
        assert np.array_equal(ur, W.expected_recv_arena(up, us))


@pytest.mark.parametrize("msd", [0, 1])
def test_staging_allocator_never_overlaps_live_sub_regions(msd):
    """vc_allocate_staging on random sizes: the pieces of two sub-regions whose lifetimes (arrival slot .. departure slot, in
    the call's order) touch never share memory, nor do two pieces of one sub-region; the arena is no larger than separate
    regions and no smaller than the most bytes alive during any digit's launches."""
    import ctypes as C
    lib = C.CDLL(E.build())
    lib.staging_allocate.restype = C.c_int64
    nseg = lib.recycle_segments()
    rng = np.random.default_rng(7 + msd)
    excess = []
    for trial in range(300):
        w = int(rng.integers(1, 9))
        w2 = int(rng.integers(0, 11 - w)) if not msd else 0
        ns = w + w2 + 1
        time = lambda k: (w - 1 - k) if (k < w and msd) else k
        size = np.zeros((ns * ns + 1, nseg), dtype=np.int64)
        fams = [(ka, kd) for ka in range(ns - 1) for kd in range(ns) if time(kd) > time(ka)]
        for ka, kd in fams:
            if rng.random() < 0.8:
                size[ka * ns + kd] = 128 * rng.integers(0, 300, size=nseg) * (rng.random(nseg) < 0.9)
        if rng.random() < 0.3:
            size[ns * ns] = 128 * rng.integers(1, 70, size=nseg)
        base = np.zeros_like(size)
        peak = lib.staging_allocate(w, w2, msd, int(size[ns * ns].sum() > 0), size.ctypes.data_as(C.c_void_p), base.ctypes.data_as(C.c_void_p))
        live = [(time(ka), time(kd), int(base[ka * ns + kd, g]), int(size[ka * ns + kd, g])) for ka, kd in fams for g in range(nseg)
                if size[ka * ns + kd, g]]
        live += [(0, ns - 1, int(base[ns * ns, g]), int(size[ns * ns, g])) for g in range(nseg) if size[ns * ns, g]]
        for i, (a0, d0, b0, s0) in enumerate(live):
            assert 0 <= b0 and b0 + s0 <= peak
            for a1, d1, b1, s1 in live[i + 1:]:
                if a0 <= d1 and a1 <= d0:                      # alive during the launches of a common slot
                    assert b0 + s0 <= b1 or b1 + s1 <= b0, (trial, (a0, d0, b0, s0), (a1, d1, b1, s1))
        assert peak <= int(size.sum())
        need = max(sum(s for a, d, _, s in live if a <= t <= d) for t in range(ns)) if live else 0
        assert peak >= need
        if need:
            excess.append(peak / need)
    # placing sub-regions in pieces keeps the arena close to what is alive at the worst moment
    assert np.median(excess) < 1.1 and max(excess) < 1.6, (np.median(excess), max(excess))


def test_multiply_and_shift_division_is_exact():
    """The route arithmetic divides by the call's constants (ranks per node, nodes, radix and its powers, ranks) with a
    multiplication and a shift (vc_div, csrc/vc_common.h).  Exact for every divisor a call can have — 1 .. 32768, and the
    stand-in for a power of the radix beyond every span — and, as a property of the construction, for any other divisor
    below 2^31: around every multiple of the divisor, at the ends of the numerators' range and on random numerators."""
    assert E.division_mismatches(1, 32768) == 0
    assert E.division_mismatches(1 << 30, 1 << 30) == 0
    for d in (32769, 65535, 65536, 65537, 1000003, (1 << 24) - 1, (1 << 30) - 1, (1 << 30) + 1, (1 << 31) - 1):
        assert E.division_mismatches(d, d, 4096) == 0, d
