"""Pins the oracle against what the mathematics fixes: the textbook MPI_Alltoallv definition on brute-force
inputs, the closed forms for the round structure, and the residency (route) invariants of each variant."""
import numpy as np
import pytest

from oracle import oracle_py as O
from rbruck_alltoallv_amd import workloads as W


def _prob(P, layout, esz, seed, hi=9, sparsify=4, recv_layout=None):
    counts = W.counts_uniform_random(P, hi, seed=seed)
    counts[counts % sparsify == 0] = 0
    return W.make_problem(counts, esz, layout, layout if recv_layout is None else recv_layout)


FLAT = {
    "twophase": lambda r, b, prob, s, d: O.twophase_rbruck_alltoallv(r, prob, s, d),
    "om": lambda r, b, prob, s, d: O.twophase_rbruck_alltoallv_om(r, prob, s, d),
    "tuna": lambda r, b, prob, s, d: O.tuna_algorithm(r, b, prob, s, d),
}


@pytest.mark.parametrize("P", [2, 3, 4, 5, 6, 7, 8, 9, 12, 16, 17, 27, 32])
@pytest.mark.parametrize("func", sorted(FLAT))
def test_flat_variants_equal_textbook_alltoallv(P, func):
    for layout in (0, 1):
        for esz in (1, 4):
            prob = _prob(P, layout, esz, seed=P)
            send = W.fill_send_arena(prob, W.PAYLOAD_HASH, 5)
            want = W.expected_recv_arena(prob, send)
            for r in sorted({2, 3, 4, 5, 8, P, P + 3, max(2, P - 1)}):
                for b in ((1, 2, 0) if func == "tuna" else (0,)):
                    recv = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
                    keep = send.copy()
                    rc = FLAT[func](r, b, prob, send, recv)
                    if func == "tuna" and P < 3:
                        assert rc == -3
                        continue
                    assert rc == 0
                    assert np.array_equal(recv, want), (P, layout, esz, r, b)
                    assert np.array_equal(send, keep), "sendbuf must be read-only"


@pytest.mark.parametrize("P,n", [(4, 2), (6, 2), (6, 3), (8, 2), (8, 4), (9, 3), (12, 4), (12, 3), (16, 4), (16, 8),
                                 (32, 8), (8, 8), (27, 9)])
def test_twolayer_variants_equal_textbook_alltoallv(P, n):
    for layout in (0, 1):
        for esz in (1, 8):
            for r in sorted({2, 3, 4, n, n + 1}):
                for bblock in (0, 1, 3):
                    for name, fn in (("ttpl", O.TTPL_BT_alltoallv), ("s1", O.TTPL_BT_alltoallv_s1)):
                        # the coalesced variant ignores rdispls: its contract is the packed receive layout
                        prob = _prob(P, layout, esz, seed=P + 100, sparsify=5, recv_layout=0 if name == "ttpl" else layout)
                        send = W.fill_send_arena(prob, W.PAYLOAD_HASH, 5)
                        want = W.expected_recv_arena(prob, send)
                        recv = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
                        assert fn(n, r, bblock, prob, send, recv) == 0
                        assert np.array_equal(recv, want), (name, layout, esz, r, bblock)


@pytest.mark.parametrize("P,n", [(4, 2), (6, 2), (6, 3), (8, 4), (9, 3), (12, 4), (16, 4), (16, 8), (32, 8), (27, 9), (64, 16)])
def test_uniform_twolayer_equal_textbook_alltoall(P, n):
    for cnt in (1, 3):
        for esz in (1, 4):
            prob = W.make_uniform_problem(P, cnt, esz)
            send = W.fill_send_arena(prob, W.PAYLOAD_HASH, 5)
            want = W.expected_recv_arena(prob, send, fill=0)
            for r in sorted({2, 3, 4, n, n + 1}):
                for fn in (lambda s, d: O.uniform_spreadout_twolayer(n, r, prob, cnt, s, d),
                           lambda s, d: O.uniform_inverse_isplit_r_bruck(n, r, 2, prob, cnt, s, d)):
                    recv = np.zeros(prob.recv_bytes, dtype=np.uint8)
                    assert fn(send.copy(), recv) == 0
                    assert np.array_equal(recv, want), (cnt, esz, r)


def test_error_codes():
    prob = _prob(8, 0, 4, seed=3)
    send = W.fill_send_arena(prob, 0, 1)
    recv = np.zeros(prob.recv_bytes, dtype=np.uint8)
    for r in (0, 1, -5):
        assert O.twophase_rbruck_alltoallv(r, prob, send, recv) == -1       # twophase_tunable_rbruckv.cpp:16
        assert O.twophase_rbruck_alltoallv_om(r, prob, send, recv) == -1
        assert O.TTPL_BT_alltoallv(4, r, 0, prob, send, recv) == -1
        assert O.TTPL_BT_alltoallv_s1(4, r, 0, prob, send, recv) == -1
        assert O.tuna_algorithm(r, 1, prob, send, recv) == 0                # tuna.cpp:13 clamps instead
    assert O.TTPL_BT_alltoallv(3, 2, 0, prob, send, recv) == -2             # n does not divide P
    assert O.TTPL_BT_alltoallv_s1(5, 2, 0, prob, send, recv) == -2


# ---------------------------------------------------------------- closed forms

def _digits(j, r, w):
    return [(j // r ** x) % r for x in range(w)]


@pytest.mark.parametrize("P", list(range(3, 70)) + [100, 127, 128, 129, 243, 256, 343, 512, 1000, 1024])
def test_radix_params_and_round_count(P):
    for r in sorted({2, 3, 4, 5, 7, 8, 16, 32, P - 1, P}):
        if r < 2 or r > P:
            continue
        w, nlpow, d, K = O.radix_params_int(P, r)
        assert (w, nlpow, d, K) == W.radix_params(P, r)
        # w = digits of P-1; K = offsets with exactly one non-zero digit
        assert r ** (w - 1) <= P - 1 < r ** w and nlpow == r ** (w - 1)
        single = sum(1 for j in range(1, P) if sum(1 for dg in _digits(j, r, w) if dg) == 1)
        assert K == single
        # the float-log form is either the same or one digit too many with an empty top digit
        wf, nlf, df = O.radix_params_float(P, r)
        assert (wf, nlf, df) == (w, nlpow, d) or (wf == w + 1 and df == r - 1)


def _trace(fn):
    with O.trace() as t:
        assert fn() == 0
    return t.records


@pytest.mark.parametrize("P,r", [(8, 2), (12, 3), (17, 5), (27, 3), (64, 4), (49, 7), (30, 29), (64, 8)])
@pytest.mark.parametrize("func", ["twophase", "om", "tuna"])
def test_route_of_flat_variants(P, r, func):
    """Every round (x, z) moves exactly the offsets whose digit x is z, from p + z*r^x to p; the bytes a rank
    receives in a round are the blocks predicted by the residency invariant (LSD: source s = holder +
    (j mod r^x); MSD: source s = holder + (j div r^(x+1)) * r^(x+1)); MSD visits digits top-down."""
    prob = _prob(P, 0, 2, seed=P * 7 + r, hi=20, sparsify=3)
    send = W.fill_send_arena(prob, 0, 2)
    recv = np.zeros(prob.recv_bytes, dtype=np.uint8)
    rec = _trace(lambda: FLAT[func](r, 1, prob, send, recv))
    rr = min(r, P - 1) if func == "tuna" else min(r, P)
    w, nlpow, d, K = W.radix_params(P, rr)
    rounds = rec[rec["kind"] != 4]
    assert len(rec[rec["kind"] == 4]) == P
    seen = []
    for (x, z) in dict.fromkeys(zip(rounds["digit"].tolist(), rounds["z"].tolist())):
        sel = rounds[(rounds["digit"] == x) & (rounds["z"] == z)]
        assert len(sel) == P
        dist = rr ** x
        offs = [j for j in range(1, P) if (j // dist) % rr == z]
        # closed form for the number of blocks in the round (tuna.cpp:75-77)
        nc, rem = P // (dist * rr) * dist, max(0, P % (dist * rr) - z * dist)
        assert len(offs) == nc + min(rem, dist)
        for m in sel:
            p = int(m["dst"])
            assert int(m["src"]) == (p + z * dist) % P
            assert int(m["nblocks"]) == len(offs)
            want = 0
            for j in offs:
                low = j % dist if func != "twophase" else j // (dist * rr) * (dist * rr)
                s = (p + z * dist + low) % P          # source rank of the block the sender held in slot j
                t = (s - j) % P
                want += int(prob.sendcounts[s, t]) * prob.esz
            assert int(m["bytes"]) == want
            assert int(m["kind"]) == (1 if (len(offs) == 1 and func != "twophase") else 0)
        seen.append((x, z))
    assert len(seen) == K
    xs = [x for x, _ in seen]
    assert xs == sorted(xs, reverse=(func == "twophase"))
    # total hop-weighted traffic = the model used for the roofline
    hops = W.hops_flat(P, rr)
    assert int(rec["bytes"].sum()) * 2 == W.algorithmic_bytes(prob.sendcounts, prob.esz, hops)


@pytest.mark.parametrize("P,n,r", [(8, 4, 2), (12, 4, 2), (27, 9, 3), (64, 16, 4), (64, 32, 32), (16, 8, 3)])
@pytest.mark.parametrize("func", ["ttpl", "s1"])
def test_route_of_twolayer_variants(P, n, r, func):
    """Intra-node rounds stay inside a node and carry, for every destination group, the blocks whose local offset
    digit matches; the inter-node phase connects equal local indices only."""
    prob = _prob(P, 0, 1, seed=P + n + r, hi=20, sparsify=3)
    send = W.fill_send_arena(prob, 0, 2)
    recv = np.zeros(prob.recv_bytes, dtype=np.uint8)
    fn = O.TTPL_BT_alltoallv if func == "ttpl" else O.TTPL_BT_alltoallv_s1
    rec = _trace(lambda: fn(n, r, 0, prob, send, recv))
    ngroup = P // n
    intra = rec[rec["kind"] == 0]
    inter = rec[(rec["kind"] == 2) | (rec["kind"] == 3)]
    assert np.all(intra["src"] // n == intra["dst"] // n)
    assert np.all(inter["src"] % n == inter["dst"] % n)
    for m in intra:
        x, z, p = int(m["digit"]), int(m["z"]), int(m["dst"])
        dist = r ** x
        offs = [j for j in range(1, n) if (j // dist) % r == z]
        assert int(m["nblocks"]) == len(offs) * ngroup
        assert int(m["src"]) == p // n * n + (p % n + z * dist) % n
        want = 0
        for g in range(ngroup):
            for j in offs:
                ls = (p % n + z * dist + j % dist) % n        # local rank of the source inside the sender's node
                s = p // n * n + ls
                t = g * n + (ls - j) % n
                want += int(prob.sendcounts[s, t]) * prob.esz
        assert int(m["bytes"]) == want
    if func == "ttpl":
        # coalesced: one message per (rank, destination group), n blocks each, own group included
        assert len(inter) == P * ngroup
        for m in inter:
            p, q = int(m["src"]), int(m["dst"])
            want = sum(int(prob.sendcounts[p // n * n + mloc, q]) for mloc in range(n)) * prob.esz
            assert int(m["bytes"]) == want
    else:
        # staggered: one message per block, own group skipped
        assert len(inter) == P * (ngroup - 1) * n
    # blocks that change node cross exactly once
    s, t = np.meshgrid(np.arange(P), np.arange(P), indexing="ij")
    cross = int(prob.sendcounts[(s // n) != (t // n)].astype(np.int64).sum()) * prob.esz
    own = int(prob.sendcounts[(s // n) == (t // n)].astype(np.int64).sum()) * prob.esz
    assert int(inter["bytes"].sum()) == cross + (own if func == "ttpl" else 0)


@pytest.mark.parametrize("P", [1, 2, 3, 4, 5, 8, 12, 16, 27, 32])
def test_linear_comparators_equal_textbook_alltoallv(P):
    """src/MPICH_scattered.cpp, OpenMPI_basic_linear.cpp, OpenMPI_pairwise.cpp, exclusive_or_alltoallv.cpp,
    benchmarks/common.cpp: one direct message per pair."""
    for layout in (0, 1):
        prob = _prob(P, layout, 2, seed=P + 40)
        send = W.fill_send_arena(prob, W.PAYLOAD_HASH, 3)
        want = W.expected_recv_arena(prob, send)
        fns = {"spreadout": lambda d: O.spreadout_alltoallv(prob, send, d),
               "linear": lambda d: O.ompi_alltoallv_intra_basic_linear(prob, send, d),
               "pairwise": lambda d: O.ompi_alltoallv_intra_pairwise(prob, send, d),
               "xor": lambda d: O.exclisive_or_alltoallv(prob, send, d)}
        for bb in (0, 1, 3, P + 5):
            fns[f"scattered{bb}"] = lambda d, bb=bb: O.MPICH_intra_scattered(bb, prob, send, d)
        for name, fn in fns.items():
            recv = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
            with O.trace() as t:
                rc = fn(recv)
            if name == "xor" and P & (P - 1):
                assert rc == -1                     # exclusive_or_alltoallv.cpp:31
                continue
            assert rc == 0
            assert np.array_equal(recv, want), (name, P, layout)
            rec = t.records
            direct = rec[rec["kind"] == 5]
            # every non-empty pair exactly once, one hop: total traffic = payload
            assert int(rec["bytes"].sum()) == prob.payload_bytes
            pairs = set(zip(direct["src"].tolist(), direct["dst"].tolist()))
            assert len(pairs) == len(direct)


@pytest.mark.parametrize("P,n", [(2, 1), (4, 2), (6, 3), (8, 4), (12, 3), (12, 4), (32, 8), (27, 9)])
def test_linear_twolayer_comparators_equal_textbook_alltoallv(P, n):
    """src/twolayer_communicator_linear.cpp:13-88, 92-192: every pair once, inside the node before between nodes."""
    for layout in (0, 1):
        prob = _prob(P, layout, 2, seed=P + n)
        send = W.fill_send_arena(prob, W.PAYLOAD_HASH, 3)
        want = W.expected_recv_arena(prob, send)
        fns = {"plain": lambda d: O.twolayer_communicator_linear(n, prob, send, d)}
        for b1, b2 in ((0, 0), (1, 1), (2, 5), (n + 3, P + 3)):
            fns[f"s2-{b1}-{b2}"] = lambda d, b1=b1, b2=b2: O.twolayer_communicator_linear_s2(n, b1, b2, prob, send, d)
        for name, fn in fns.items():
            recv = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
            with O.trace() as t:
                assert fn(recv) == 0
            assert np.array_equal(recv, want), (name, P, n, layout)
            rec = t.records
            assert np.all(rec["kind"] == 5)
            assert int(rec["bytes"].sum()) == prob.payload_bytes
            pairs = list(zip(rec["src"].tolist(), rec["dst"].tolist()))
            assert len(set(pairs)) == len(pairs)
            inside = rec["src"] // n == rec["dst"] // n
            # all messages inside the nodes come before the first one between nodes (:34 before :55 / :147)
            if inside.any() and (~inside).any():
                assert np.nonzero(inside)[0].max() < np.nonzero(~inside)[0].min()


@pytest.mark.parametrize("P", [1, 2, 4, 6, 8, 9, 12, 16, 24, 27, 32, 36, 64])
def test_twolayer_bruck_equals_textbook_alltoallv(P):
    """TTPL_rbruck_alltoallv with the inter-node Bruck completed (src/twophase_twolayer_rbruck.cpp:15-235): for every
    divisor n of P and every radix, the definition of alltoallv — the only pin the blocks that change node have,
    since the reference drops them."""
    for layout in (0, 1):
        prob = _prob(P, layout, 2, seed=P + 3)
        send = W.fill_send_arena(prob, W.PAYLOAD_HASH, 7)
        keep = send.copy()
        want = W.expected_recv_arena(prob, send)
        for n in [d for d in range(1, P + 1) if P % d == 0]:
            for r in sorted({2, 3, 4, 7, max(n, 2), P + 2}):
                recv = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
                with O.trace() as t:
                    assert O.TTPL_rbruck_alltoallv(n, r, prob, send, recv) == 0
                assert np.array_equal(recv, want), (P, layout, n, r)
                assert np.array_equal(send, keep)
                rec = t.records
                inter = rec[rec["kind"] == 6]
                assert np.all(inter["src"] % n == inter["dst"] % n)
                assert np.all(inter["src"] // n != inter["dst"] // n)
                intra = rec[rec["kind"] == 0]
                assert np.all(intra["src"] // n == intra["dst"] // n)


@pytest.mark.parametrize("P", [3, 4, 5, 8, 12, 17, 27, 32, 50])
def test_tuna2_equals_definition_and_walks_tunas_route(P):
    """src/tuna2.cpp: same rounds as TuNA (same messages between the same ranks), unpack deferred per digit."""
    for layout in (0, 1):
        prob = _prob(P, layout, 2, seed=P)
        send = W.fill_send_arena(prob, W.PAYLOAD_HASH, 5)
        want = W.expected_recv_arena(prob, send)
        for r in sorted({2, 3, 4, 5, 8, P, P - 1}):
            for b in (1, 2, 0):
                recv = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
                with O.trace() as t2:
                    assert O.tuna2_algorithm(r, b, prob, send, recv) == 0
                assert np.array_equal(recv, want), (P, layout, r, b)
                with O.trace() as t1:
                    assert O.tuna_algorithm(r, b, prob, send, np.empty_like(recv)) == 0
                key = ["kind", "digit", "z", "src", "dst"]
                assert np.array_equal(np.sort(t1.records, order=key), np.sort(t2.records, order=key))


def test_compact_staging_index_closed_form():
    """extra_id(j) = rank of j among the offsets with at least two non-zero digits (tuna2.cpp:63-73 builds that table;
    tuna.cpp:93-97 evaluates j - r - (dx-1)(r-1) - dz through float logs)."""
    lib = O.lib()
    for P in list(range(3, 70)) + [100, 128, 243, 256, 343, 512, 1000, 1024]:
        for r in sorted({2, 3, 4, 5, 7, 8, 16, 32, P - 1}):
            if r < 2 or r > P - 1:
                continue
            w, _, _, K = W.radix_params(P, r)
            rank = 0
            for j in range(1, P):
                nz = sum(1 for x in range(w) if (j // r ** x) % r)
                if nz >= 2:
                    assert lib.ora_compact_slot_float(j, r) == rank, (P, r, j)
                    rank += 1
            assert rank == P - K - 1
