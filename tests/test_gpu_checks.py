"""Checks of the checkers and of the library's default execution mode, through the C ABI on a real MI355X.

* vc_verify_alltoallv (the on-device definition check the full-size tests and the benchmark lean on) must count exactly
  the bytes that are wrong, not merely return 0 on a correct arena;
* the library's default mode (vc_comm_set_forwarding 1: the last call on the communicator decides between the work-item
  list and the listless kernels, which may refuse a call on the device and have it redone) against the oracle's bytes;
* table validation beyond negative entries; the staging arena under live plans."""
import collections

import numpy as np
import pytest

from oracle import oracle_py as O
from rbruck_alltoallv_amd import _lib
from rbruck_alltoallv_amd import workloads as W
from tests.helpers import digest_problem, load_golden, problem_for_case, run_on

pytestmark = pytest.mark.gpu

CASES = load_golden()


@pytest.fixture(scope="module")
def api():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU"
    from rbruck_alltoallv_amd import api as A
    A.DEFAULT_FORWARDING = None
    return A


def _host_mismatch(prob, send, recv, rdispls=None, packed=False):
    """Bytes of recv that differ from the definition, counted block by block on the host (numpy)."""
    rd = prob.rdispls if rdispls is None else rdispls
    bad = 0
    for t in range(prob.P):
        at_packed = 0
        for s in range(prob.P):
            nb = int(prob.sendcounts[s, t]) * prob.esz
            a = int(prob.sbase[s]) + int(prob.sdispls[s, t]) * prob.esz
            b = int(prob.rbase[t]) + (at_packed if packed else int(rd[t, s]) * prob.esz)
            bad += int(np.count_nonzero(send[a:a + nb] != recv[b:b + nb]))
            at_packed += int(prob.recvcounts[t, s]) * prob.esz
    return bad


@pytest.mark.parametrize("packed", [False, True])
def test_verify_counts_exactly_the_wrong_bytes(api, packed):
    import torch
    P, esz = 24, 2
    counts = W.counts_uniform_random(P, 900, seed=31)
    counts[counts % 7 == 0] = 0
    prob = W.make_problem(counts, esz, 0, 0)
    send = W.fill_send_arena(prob, 0, 17)
    dp = api.DeviceProblem(prob)
    ds = torch.from_numpy(send).to("cuda:0")
    dr = dp.new_recv_arena(0xEE)
    fn = (lambda: api.TTPL_BT_alltoallv(6, 3, 0, dp, ds, dr)) if packed else (lambda: api.twophase_rbruck_alltoallv(3, dp, ds, dr))
    assert fn() == 0, dp.comm.error()
    assert dp.verify(ds, dr, packed_recv=packed) == 0
    good = dr.clone()

    # one flipped byte inside a block
    t, s = 5, 9
    assert counts[s, t] > 0
    at = int(prob.rbase[t]) + int(prob.rdispls[t, s]) * esz + 3
    dr[at] ^= 0x40
    assert dp.verify(ds, dr, packed_recv=packed) == 1
    dr.copy_(good)

    # a byte between the ranks' buffers or in a gap is nobody's: not counted (the arena comparison of the parity tests covers those)
    # two blocks of one receiver swapped (the first min(len) bytes of each)
    s1, s2 = 2, 11
    n1, n2 = int(counts[s1, t]) * esz, int(counts[s2, t]) * esz
    assert n1 > 0 and n2 > 0
    a1 = int(prob.rbase[t]) + int(prob.rdispls[t, s1]) * esz
    a2 = int(prob.rbase[t]) + int(prob.rdispls[t, s2]) * esz
    m = min(n1, n2)
    tmp = dr[a1:a1 + m].clone()
    dr[a1:a1 + m] = dr[a2:a2 + m]
    dr[a2:a2 + m] = tmp
    want = _host_mismatch(prob, send, dr.cpu().numpy(), packed=packed)
    assert want > m                                           # random payload: nearly all 2 m bytes differ
    assert dp.verify(ds, dr, packed_recv=packed) == want
    dr.copy_(good)

    # a whole rank's buffer wiped
    t2 = 13
    lo, hi = int(prob.rbase[t2]), int(prob.rbase[t2]) + int(counts[:, t2].sum()) * esz
    dr[lo:hi] = 0
    want = _host_mismatch(prob, send, dr.cpu().numpy(), packed=packed)
    assert dp.verify(ds, dr, packed_recv=packed) == want > 0
    dr.copy_(good)

    if not packed:
        # one receive displacement shifted by one element: the check reads the block one element further on
        rd = prob.rdispls.copy()
        rd[t, s] += 1
        drd = torch.from_numpy(rd).to("cuda:0")
        keep = dp.rdispls
        dp.rdispls = drd
        want = _host_mismatch(prob, send, good.cpu().numpy(), rdispls=rd)
        assert want > 0
        assert dp.verify(ds, good) == want
        dp.rdispls = keep
    # a receive count that disagrees with the send count is one mismatch of its own
    rc = prob.recvcounts.copy()
    rc[t, s] += 1
    keep = dp.recvcounts
    dp.recvcounts = torch.from_numpy(rc).to("cuda:0")
    got = dp.verify(ds, good, packed_recv=packed)
    dp.recvcounts = keep
    if packed:                                                # the packed layout follows the receive counts: later blocks shift too
        assert got >= 1
    else:
        assert got == 1
    dp.comm.free()


def test_default_mode_on_the_golden_cases(api):
    """vc_comm_set_forwarding 1, the library's default: one long-lived communicator per rank count, the golden cases in
    file order, two calls each.  The first call of a case runs on whatever the previous case left as a hint (the listless
    kernels refuse what they were not made for and the call is redone through the list, or redone behind a larger
    staging arena); the second on the hint of the first.  Every call must leave the oracle's bytes."""
    import torch
    comms = {}
    ran = collections.Counter()
    for case in CASES:
        print("case", case["id"], flush=True)
        prob = problem_for_case(case)
        send = W.fill_send_arena(prob, case["payload"], case["seed"])
        want = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
        assert run_on(O, case, prob, send.copy(), want) == 0
        if prob.P not in comms:
            comms[prob.P] = api.VirtualComm(prob.P)
            comms[prob.P].set_forwarding(1)
        dp = api.DeviceProblem(prob, comm=comms[prob.P])
        dsend = torch.from_numpy(send).to("cuda:0")
        for call in range(2):
            drecv = dp.new_recv_arena(0xEE)
            rc = run_on(api, case, dp, dsend, drecv)
            assert rc == 0, (case["id"], call, dp.comm.error())
            got = drecv.cpu().numpy()
            assert np.array_equal(got, want), (case["id"], call)
            st = dp.comm.last_stats()
            assert st.n_launches == 1 and st.payload_bytes == prob.payload_bytes
            ran[(int(st.execution), int(st.lanes_per_item))] += 1
        assert [f"{int(h):016x}" for h in O.digest_recv(digest_problem(case, prob), got)] == case["digests"]
    for c in comms.values():
        c.free()
    print("executions (mode, lanes):", dict(ran), flush=True)
    assert any(k[0] == 1 for k in ran) and any(k[0] in (2, 3) for k in ran)      # with the list and without


def test_refused_listless_call_is_redone(api):
    """The ways a listless attempt ends without having moved anything, each compared with the oracle's bytes: the staging
    arena was too small (the call is enqueued again behind a larger one), the blocks are longer than the fixed stride the
    last call suggested, and the call was not of the kind the hint promised (it continues through the work-item list)."""
    import torch
    P = 48
    comm = api.VirtualComm(P)
    tiny = W.make_problem(W.counts_uniform_random(P, 8, seed=1), 1, 0, 0)
    short = W.make_problem(W.counts_uniform_random(P, 700, seed=2), 1, 1, 1)
    long_counts = W.counts_uniform_random(P, 700, seed=3)
    long_counts[7, 30] = 500000                                                       # one block of 123 pieces
    long = W.make_problem(long_counts, 1, 0, 0)
    seen = []
    # vc_comm_set_forwarding 4: always a quarter of a wavefront per pair, compact staging; 1: the library's choice
    for mode, prob in ((4, tiny), (4, short), (1, tiny), (1, tiny), (1, short), (1, short), (1, long), (1, short)):
        comm.set_forwarding(mode)
        send = W.fill_send_arena(prob, 0, 5)
        want = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
        assert O.twophase_rbruck_alltoallv(3, prob, send, want) == 0
        dp = api.DeviceProblem(prob, comm=comm)
        comm.set_forwarding(mode)
        ds = torch.from_numpy(send).to("cuda:0")
        dr = dp.new_recv_arena(0xEE)
        assert api.twophase_rbruck_alltoallv(3, dp, ds, dr) == 0, comm.error()
        assert np.array_equal(dr.cpu().numpy(), want)
        st = comm.last_stats()
        seen.append((int(st.execution), int(st.staging_bytes)))
    # listless; listless again behind a grown arena; (hint of short blocks) fixed stride twice; stride too short -> compact
    # listless; fixed stride; a block of 123 pieces: refused twice on the device -> list; hint of long blocks -> list
    assert [e for e, _ in seen] == [2, 2, 3, 3, 2, 3, 1, 1], seen
    assert seen[1][1] > 2 * seen[0][1]                       # the second call needed a larger arena than there was
    comm.free()


def test_tables_that_disagree_are_refused(api):
    """recvcounts must be the transpose of sendcounts (the reference fails with an MPI truncation error); a packed receive
    layout past INT_MAX elements is an overflow, as in vc_displs_from_counts.  Nothing moves before the tables have been
    checked, in any execution mode."""
    import torch
    counts = W.counts_uniform_random(12, 40, seed=5)
    prob = W.make_problem(counts, 4, 0, 0)
    dp = api.DeviceProblem(prob)
    s, d = dp.new_send_arena(), dp.new_recv_arena()
    dp.fill_payload(0, 1, s)
    keep = int(dp.recvcounts[7, 3].item())
    for mode in (0, 1, 2, 3, 4, 5):
        dp.comm.set_forwarding(mode)
        for delta in (1, -1):
            dp.recvcounts[7, 3] = keep + delta
            for call in (lambda: api.twophase_rbruck_alltoallv(3, dp, s, d), lambda: api.TTPL_BT_alltoallv(4, 2, 0, dp, s, d),
                         lambda: api.spreadout_alltoallv(dp, s, d)):
                assert call() == _lib.VC_ERR_TABLES and "recvcounts" in dp.comm.error(), mode
            assert bool((d == 0xEE).all()), mode
        dp.recvcounts[7, 3] = keep
        assert api.twophase_rbruck_alltoallv(3, dp, s, d) == 0 and dp.verify(s, d) == 0
        d.fill_(0xEE)
    dp.comm.free()
    # 2 ranks that each receive 2^31 one-byte elements: found by the planner, nothing is touched
    comm = api.VirtualComm(2)
    z = torch.zeros(2, dtype=torch.int64, device="cuda:0")
    comm.set_bases(z, z)
    big = torch.full((2, 2), 2 ** 30, dtype=torch.int32, device="cuda:0")
    displs = torch.tensor([[0, 2 ** 30], [0, 2 ** 30]], dtype=torch.int32, device="cuda:0")
    buf = torch.full((256,), 0xEE, dtype=torch.uint8, device="cuda:0")
    for mode in (0, 2, 3):
        comm.set_forwarding(mode)
        rc = comm.lib.TTPL_BT_alltoallv(1, 2, 0, buf.data_ptr(), big.data_ptr(), displs.data_ptr(), 1, buf.data_ptr(), big.data_ptr(),
                                        None, 1, comm.handle)
        assert rc == _lib.VC_ERR_OVERFLOW, (mode, rc, comm.error())
        assert bool((buf == 0xEE).all())
    comm.free()


@pytest.mark.parametrize("P", [33, 64, 150, 192])
def test_single_launch_totals_equal_the_planner_header(api, P):
    """A small call in the default mode is one launch that plans nothing: its first wavefronts add up (one atomic per
    wavefront and word) what the planner kernels otherwise put into the plan header — payload, block pieces, the most pieces
    and the longest block, hop-weighted bytes, and the table entries no set of ranks could have passed (src/utils.cpp:31-46
    is the reference's check of a result; here the tables are checked before).  Same tables, same words, whoever adds
    them up — also when the tables are bad."""
    rng = np.random.default_rng(P)
    counts = rng.integers(0, 600, size=(P, P)).astype(np.int32)
    counts[rng.random((P, P)) < 0.1] = 0
    prob = W.make_problem(counts, 1, 1, 1)
    dp = api.DeviceProblem(prob)
    ds, dr = dp.new_send_arena(), dp.new_recv_arena(0xEE)
    dp.fill_payload(0, 9, ds)

    def words(mode, calls):
        dp.comm.set_forwarding(mode)
        for _ in range(calls):
            rc = api.twophase_rbruck_alltoallv(3, dp, ds, dr)
        st = dp.comm.last_stats()
        return rc, int(st.execution), (int(st.payload_bytes), int(st.moved_bytes), int(st.block_pieces), int(st.max_block_pieces),
                                       int(st.max_block_bytes), int(st.bad_table_entries))

    rc, execution, planner = words(2, 1)
    assert rc == 0 and execution == 1, dp.comm.error()
    rc, execution, single = words(1, 2)
    assert rc == 0 and execution == 3, (execution, dp.comm.error())             # one launch, fixed-stride staging
    assert planner == single and single[0] == prob.payload_bytes and single[5] == 0
    assert dp.verify(ds, dr) == 0
    # bad tables: negative entries in all four tables and receivers that expect something else than is sent
    picks = rng.choice(P * P, size=9, replace=False)
    for k, at in enumerate(picks):
        t, s_ = int(at // P), int(at % P)
        if k < 2:
            dp.sendcounts[t, s_] = -5
        elif k < 4:
            dp.sdispls[t, s_] = -1
        elif k < 6:
            dp.rdispls[t, s_] = -7
        else:
            dp.recvcounts[t, s_] += 3 if k < 8 else -600
    rc, _, planner_bad = words(2, 1)
    assert rc == _lib.VC_ERR_TABLES
    rc, _, single_bad = words(1, 1)                                               # on the hint of the good calls: one launch again
    assert rc == _lib.VC_ERR_TABLES
    assert planner_bad[5] == single_bad[5] and planner_bad[5] >= 9, (planner_bad, single_bad)
    dp.comm.free()


def test_bad_tables_after_a_good_call_in_the_default_mode(api):
    """The default mode chooses its kernel from what the last call looked like.  After good calls of short blocks (which
    leave the hint for the single launch that checks the tables beside the copying: its copying wavefronts hold their
    stores back until the checking ones have reported), a call with tables that disagree returns VC_ERR_TABLES and has
    written nothing; the communicator stays usable."""
    import torch
    counts = W.counts_uniform_random(40, 500, seed=8)
    prob = W.make_problem(counts, 2, 1, 1)
    send = W.fill_send_arena(prob, 0, 3)
    want = W.expected_recv_arena(prob, send)
    dp = api.DeviceProblem(prob)
    ds = torch.from_numpy(send).to("cuda:0")
    dr = dp.new_recv_arena(0xEE)
    dp.comm.set_forwarding(1)
    for _ in range(2):
        assert api.twophase_rbruck_alltoallv(2, dp, ds, dr) == 0, dp.comm.error()
    assert dp.comm.last_stats().execution == 3 and np.array_equal(dr.cpu().numpy(), want)
    keep = int(dp.recvcounts[9, 4].item()), int(dp.sdispls[21, 30].item())
    dp.recvcounts[9, 4] = keep[0] + 2
    dp.sdispls[21, 30] = -3
    dr.fill_(0xEE)
    assert api.twophase_rbruck_alltoallv(2, dp, ds, dr) == _lib.VC_ERR_TABLES
    assert bool((dr == 0xEE).all()), "a refused call wrote into recvbuf"
    dp.recvcounts[9, 4], dp.sdispls[21, 30] = keep
    assert api.twophase_rbruck_alltoallv(2, dp, ds, dr) == 0 and np.array_equal(dr.cpu().numpy(), want)
    dp.comm.free()


def test_staging_arena_stays_put_while_a_plan_lives(api):
    """A HIP graph captured from vc_plan_execute_async holds the staging arena's address.  A later call on the same
    communicator that needs a larger arena must not free the one the graph writes to: the replay after it is still exact."""
    import torch
    P = 32
    small = W.make_problem(W.counts_uniform_random(P, 900, seed=8), 1, 0, 0)
    large = W.make_problem(W.counts_uniform_random(P, 60000, seed=9), 1, 0, 0)
    comm = api.VirtualComm(P)
    comm.set_forwarding(2)
    dp = api.DeviceProblem(small, comm=comm)
    send = W.fill_send_arena(small, 0, 3)
    want = W.expected_recv_arena(small, send, fill=0)
    ds = torch.from_numpy(send).to("cuda:0")
    dr = dp.new_recv_arena(0)
    plan = api.Plan("twophase_rbruck_alltoallv", dp, dr, r=2)
    assert plan.rc == 0, comm.error()
    assert plan.execute(ds, dr) == 0 and np.array_equal(dr.cpu().numpy(), want)
    before = comm.staging()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        comm.use_current_stream()
        assert plan.execute_async(ds, dr) == 0, comm.error()
    comm.use_current_stream()
    # a larger call on the same communicator: its bases are another problem's
    dpl = api.DeviceProblem(large, comm=comm)
    dsl, drl = dpl.new_send_arena(), dpl.new_recv_arena()
    dpl.fill_payload(0, 4, dsl)
    assert api.twophase_rbruck_alltoallv(2, dpl, dsl, drl) == 0 and dpl.verify(dsl, drl) == 0
    after = comm.staging()
    assert after[1] > before[1] and after[0] != before[0]    # a second arena; the first one is still allocated
    for rep in range(3):
        dr.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert np.array_equal(dr.cpu().numpy(), want), rep
    plan.free()
    comm.free()


def suggestion_against_measured(api, name, mode):
    """vc_suggest_tunables replaces the sweep over bases of the reference's drivers (examples/rbruckv_example.cpp:33-35,
    98-103).  Times every candidate radix on the shape of configuration 3 or 5 or on one of the reference's input matrices
    (reduced sizes) and returns (time of the suggested radix) / (time of the fastest candidate), by wall clock."""
    import os
    import time
    import torch
    from tests.helpers import INPUTS_DIR
    if name == "C3":
        counts, esz = W.counts_zipf(256, 16384, 1.2, 5, 0), 4
        fn = lambda r, dp, s, d: api.twophase_rbruck_alltoallv(r, dp, s, d)
    elif name == "C5":
        counts, esz = W.counts_fft_rows(512, 32, 8192), 8
        fn = lambda r, dp, s, d: api.tuna_algorithm(r, 0, dp, s, d)
    else:
        counts, esz = W.counts_from_npz(os.path.join(INPUTS_DIR, "global_comm_pattern_256proc.npz"), 32), 1
        fn = lambda r, dp, s, d: api.twophase_rbruck_alltoallv(r, dp, s, d)
    prob = W.make_problem(counts, esz, 0, 0)
    dp = api.DeviceProblem(prob)
    dp.comm.set_forwarding(mode)
    ds, dr = dp.new_send_arena(), dp.new_recv_arena()
    dp.fill_payload(0, 3, ds)
    cands = [2, 4, 8, 16, 32, prob.P]
    best, b, modelled = api.suggest_tunables(dp, cands)
    assert best in cands and b == min(best, prob.P) - 1
    measured = {}
    for r in cands:
        for _ in range(2):
            assert fn(r, dp, ds, dr) == 0, dp.comm.error()
        times = []
        for _ in range(7):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            fn(r, dp, ds, dr)
            times.append(time.perf_counter() - t0)
        measured[r] = sorted(times)[len(times) // 2]
        assert dp.verify(ds, dr) == 0
    print(name, "mode", mode, "suggested", best, {r: (round(measured[r] * 1e3, 3), round(m * 1e3, 3)) for r, m in zip(cands, modelled)}, flush=True)
    # without a candidate list: the whole range 2 .. min(P, 63) and P
    free_choice, _, _ = api.suggest_tunables(dp)
    assert 2 <= free_choice <= prob.P
    rate, launch = api.calibration(dp.comm)
    assert 1e12 < rate < 8e12 and 2e-7 < launch < 1e-4, (rate, launch)
    dp.comm.free()
    return measured[best] / min(measured.values())


@pytest.mark.parametrize("mode", [2, 0], ids=["forwarded", "launch-per-digit"])
@pytest.mark.parametrize("name", ["C3", "C5", "ML256"])
def test_suggested_radix_is_a_sane_choice(api, name, mode):
    """The radix the model picks is among the good ones when all candidates are timed: within 1.5 x of the fastest.  (The
    bad candidates are 2 - 4 x slower, so a broken model fails this; the 10 % bar is a wall-clock assertion and lives under
    its own marker, tests/test_perf_tuner.py, where a noisy box cannot stop the correctness suite.)"""
    ratio = suggestion_against_measured(api, name, mode)
    assert ratio <= 1.5, ratio


def test_async_twins_overlap_two_communicators(api):
    """The _async entry points only enqueue: two communicators on two streams run their collectives side by side, each is
    completed by vc_comm_wait, and both leave the oracle's bytes.  All seven twins, errors reported at the wait, the arena
    grown at the wait, and the communicator busy in between."""
    import torch
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    pa = W.make_problem(W.counts_uniform_random(48, 2500, seed=41), 2, 1, 1)
    pb = W.make_problem(W.counts_normal(64, 700.0, 300.0, 0, 3000, 5), 1, 0, 0)
    senda, sendb = W.fill_send_arena(pa, 0, 6), W.fill_send_arena(pb, 0, 7)
    dpa, dpb = api.DeviceProblem(pa), api.DeviceProblem(pb)
    dsa, dsb = torch.from_numpy(senda).to("cuda:0"), torch.from_numpy(sendb).to("cuda:0")
    twins = [("twophase_rbruck_alltoallv", (3,), lambda p, s, r: O.twophase_rbruck_alltoallv(3, p, s, r), False),
             ("twophase_rbruck_alltoallv_om", (4,), lambda p, s, r: O.twophase_rbruck_alltoallv_om(4, p, s, r), False),
             ("tuna_algorithm", (2, 1), lambda p, s, r: O.tuna_algorithm(2, 1, p, s, r), False),
             ("TTPL_BT_alltoallv_s1", (8, 2, 3), lambda p, s, r: O.TTPL_BT_alltoallv_s1(8, 2, 3, p, s, r), False),
             ("TTPL_BT_alltoallv", (8, 8, 0), lambda p, s, r: O.TTPL_BT_alltoallv(8, 8, 0, p, s, r), True)]
    torch.cuda.synchronize()
    for k, (name, tun, ofn, packed) in enumerate(twins):
        print("  async", name, flush=True)
        other = twins[(k + 1) % 4]                            # another function on the second communicator, at the same time
        if packed:                                            # the packed layout needs packed receive displacements: pb has them
            wa = None
        else:
            wa = np.full(pa.recv_bytes, 0xEE, dtype=np.uint8)
            assert ofn(pa, senda, wa) == 0
        wb = np.full(pb.recv_bytes, 0xEE, dtype=np.uint8)
        assert (ofn if packed else other[2])(pb, sendb, wb) == 0
        dra, drb = dpa.new_recv_arena(0xEE), dpb.new_recv_arena(0xEE)
        torch.cuda.synchronize()
        if not packed:
            assert api.call_async(name, tun, dpa, dsa, dra, s1) == 0, dpa.comm.error()
        bname, btun = (name, tun) if packed else (other[0], other[1])
        assert api.call_async(bname, btun, dpb, dsb, drb, s2) == 0, dpb.comm.error()
        # busy until collected
        assert api.twophase_rbruck_alltoallv(2, dpb, dsb, drb) == _lib.VC_ERR_BUSY
        assert dpb.comm.wait() == 0, dpb.comm.error()
        assert np.array_equal(drb.cpu().numpy(), wb), (bname, "second communicator")
        assert dpb.comm.last_stats().execution == 2 and dpb.comm.last_stats().payload_bytes == pb.payload_bytes
        if not packed:
            assert dpa.comm.wait() == 0, dpa.comm.error()
            assert np.array_equal(dra.cpu().numpy(), wa), (name, "first communicator")
        assert dpa.comm.wait() == 0                           # nothing pending: just a synchronisation
    # a table error is found on the device and reported by the wait; recvbuf stays untouched
    keep = int(dpa.sdispls[5, 6].item())
    dpa.sdispls[5, 6] = -3
    dra = dpa.new_recv_arena(0xEE)
    assert api.call_async("tuna_algorithm", (3, 0), dpa, dsa, dra, s1) == 0
    assert dpa.comm.wait() == _lib.VC_ERR_TABLES
    assert bool((dra == 0xEE).all())
    dpa.sdispls[5, 6] = keep
    assert api.call_async("twophase_rbruck_alltoallv", (1,), dpa, dsa, dra, s1) == -1 and dpa.comm.wait() == 0
    dpa.comm.free()
    dpb.comm.free()
    # a fresh communicator has no staging arena: the copy kernel refuses on the device and the wait redoes it
    pc = W.make_problem(W.counts_uniform_random(40, 5000, seed=43), 1, 0, 0)
    sendc = W.fill_send_arena(pc, 0, 8)
    dpc = api.DeviceProblem(pc)
    dsc, drc = torch.from_numpy(sendc).to("cuda:0"), dpc.new_recv_arena(0xEE)
    assert api.call_async("twophase_rbruck_alltoallv", (2,), dpc, dsc, drc, s1) == 0
    assert dpc.comm.wait() == 0, dpc.comm.error()
    assert dpc.comm.last_stats().staging_bytes > 0
    assert np.array_equal(drc.cpu().numpy(), W.expected_recv_arena(pc, sendc))
    dpc.comm.free()
    # the equal-block twins
    up = W.make_uniform_problem(48, 333, 2)
    dpu = api.DeviceProblem(up)
    dsu = dpu.new_send_arena()
    dpu.fill_payload(0, 9, dsu)
    for name, tun in (("uniform_spreadout_twolayer", (8, 3)), ("uniform_inverse_isplit_r_bruck", (6, 2, 2))):
        dru = dpu.new_recv_arena(0xEE)
        assert api.uniform_async(name, tun, dpu, 333, dsu, dru, s2) == 0, dpu.comm.error()
        assert dpu.comm.wait() == 0, dpu.comm.error()
        assert dpu.verify(dsu, dru) == 0, name
    dpu.comm.free()


def test_staging_bound(api):
    """A radix-2 Bruck on the pencil pattern of configuration 5 (512 ranks, rows of 32, here 64 KiB blocks: 1 GiB of
    payload, 4.5 hops per block) would keep 3.5 x the payload in separate staging regions.  A communicator that bounds its
    staging (the default) runs the call one launch per digit on reused staging, below twice the payload; unbounded it stays
    forwarded.  Both exact."""
    counts = W.counts_fft_rows(512, 32, 8192)
    prob = W.make_problem(counts, 8, 0, 0)
    S = prob.payload_bytes
    assert S == 1 << 30
    dp = api.DeviceProblem(prob)
    ds = dp.new_send_arena()
    dp.fill_payload(0, 21, ds)
    seen = {}
    for bound in (True, False):
        dp.comm.set_staging_bound(1024 if bound else 0)      # an allowance of 1 GiB (the default is an eighth of the device's memory)
        for mode in (2, 0):
            dp.comm.set_forwarding(mode)
            dr = dp.new_recv_arena(0xEE)
            assert api.tuna_algorithm(2, 0, dp, ds, dr) == 0, dp.comm.error()
            assert dp.verify(ds, dr) == 0
            st = dp.comm.last_stats()
            seen[(bound, mode)] = (int(st.execution), int(st.staging_bytes), int(st.n_launches))
            assert st.moved_bytes * 2 == W.algorithmic_bytes(counts, 8, W.hops_flat(512, 2))
    print(seen, flush=True)
    # a persistent plan made in forwarded mode for a call beyond the bound is a launch-per-digit plan too
    dp.comm.set_staging_bound(1024)
    dp.comm.set_forwarding(2)
    dr = dp.new_recv_arena(0xEE)
    plan = api.Plan("tuna_algorithm", dp, dr, r=2, batch=0)
    assert plan.rc == 0, dp.comm.error()
    for _ in range(2):
        dr.fill_(0xEE)
        assert plan.execute(ds, dr) == 0, dp.comm.error()
        assert dp.verify(ds, dr) == 0
        assert (dp.comm.last_stats().execution, dp.comm.last_stats().staging_bytes) == seen[(True, 0)][:2]
    plan.free()
    assert seen[(False, 2)][0] == 1 and seen[(False, 2)][1] > 3.4 * S            # forwarded, every region of its own
    assert seen[(False, 0)][0] == 0 and seen[(False, 0)][1] == seen[(False, 2)][1]
    assert seen[(True, 0)][0] == 0 and seen[(True, 0)][1] < 1.25 * S               # reused, sub-regions placed in pieces
    assert seen[(True, 2)] == seen[(True, 0)]                                      # asked for forwarded, run per digit
    # a radix with few hops stays forwarded under the bound
    dp.comm.set_staging_bound(1024)
    dp.comm.set_forwarding(2)
    dr = dp.new_recv_arena(0xEE)
    assert api.tuna_algorithm(32, 0, dp, ds, dr) == 0 and dp.verify(ds, dr) == 0
    assert dp.comm.last_stats().execution == 1 and dp.comm.last_stats().staging_bytes < S
    # ... and so does the radix-2 call under the default allowance, which 3.5 GiB do not reach
    dp.comm.set_staging_bound(True)
    assert api.tuna_algorithm(2, 0, dp, ds, dr) == 0 and dp.verify(ds, dr) == 0
    assert dp.comm.last_stats().execution == 1 and dp.comm.last_stats().staging_bytes > 3.4 * S
    dp.comm.free()
    # the _async twin on a fresh communicator (no staging arena yet): enqueued forwarded, refused on the device for want of
    # staging, found out of bound at the wait and run one launch per digit there, like the blocking call
    import torch
    dp2 = api.DeviceProblem(prob)
    dp2.comm.set_staging_bound(1024)
    dr2 = dp2.new_recv_arena(0xEE)
    assert api.call_async("tuna_algorithm", (2, 0), dp2, ds, dr2, torch.cuda.Stream()) == 0, dp2.comm.error()
    assert dp2.comm.wait() == 0, dp2.comm.error()
    assert dp2.verify(ds, dr2) == 0
    assert (int(dp2.comm.last_stats().execution), int(dp2.comm.last_stats().staging_bytes)) == seen[(True, 0)][:2]
    assert api.tuna_algorithm(32, 0, dp2, ds, dr2) == 0 and dp2.verify(ds, dr2) == 0      # the communicator is free and on its own stream again
    dp2.comm.free()


def test_list_and_copy_enqueued_behind_the_sizing_kernels(api):
    """A forwarded call through the work-item list normally waits for the sizing kernels in mid-call (vc_stats_t.host_waits
    2).  Once two calls of a kind have been seen on a communicator, the list and the copy go out right behind the sizing
    kernels, sized from the last call, and check the plan on the device (host_waits 1).  Every way that can end, against
    the definition's bytes: the guess fits; the call needs a longer list and a larger arena than there are (nothing moves,
    the call goes the general way); the call is shorter than guessed; its tables disagree (refused, recvbuf untouched);
    it is longer than guessed (a second launch takes the rest); its staging is out of the communicator's bound (one
    launch per digit instead)."""
    import torch
    P = 96
    comm = api.VirtualComm(P)
    base = W.counts_uniform_random(P, 3000, seed=11)
    more = W.counts_uniform_random(P, 5000, seed=12)
    more[::5, ::6] = 40000                                                            # + 320 blocks of 10 pieces
    less = W.counts_uniform_random(P, 900, seed=13)
    less[less % 5 != 0] = 0                                                           # four blocks in five are empty
    probs = {"base": W.make_problem(base, 1, 0, 0), "more": W.make_problem(more, 1, 1, 1), "less": W.make_problem(less, 1, 0, 0)}

    def call(name, func=None, expect=0, spoil=False):
        prob = probs[name]
        send = W.fill_send_arena(prob, 0, 21)
        want = W.expected_recv_arena(prob, send)
        dp = api.DeviceProblem(prob, comm=comm)
        comm.set_forwarding(2)                                                        # forwarded, through the list
        ds = torch.from_numpy(send).to("cuda:0")
        dr = dp.new_recv_arena(0xEE)
        if spoil:
            dp.recvcounts[9, 4] += 2
        rc = api.twophase_rbruck_alltoallv(4, dp, ds, dr) if func is None else func(dp, ds, dr)
        assert rc == expect, (name, rc, comm.error())
        got = dr.cpu().numpy()
        if expect == 0:
            assert np.array_equal(got, want), name
        else:
            assert bool((got == 0xEE).all()), "a refused call wrote into recvbuf"
        st = comm.last_stats()
        return int(st.host_waits), int(st.execution), int(st.block_pieces), int(st.staging_bytes)

    seen = [call("base"), call("base"), call("base")]
    assert [w for w, _, _, _ in seen] == [2, 2, 1] and all(e == 1 for _, e, _, _ in seen), seen
    grown = call("more")                               # longer list, larger arena: refused on the device, redone the general way
    assert grown[:2] == (2, 1) and seen[0][2] < grown[2] <= 2 * seen[0][2] and grown[3] > seen[0][3], (seen, grown)
    assert call("more")[0] == 1                        # now the guess fits again
    shorter = call("less")                             # fewer pieces than guessed: the surplus workgroups find nothing
    assert shorter[0] == 1 and 2 * shorter[2] < grown[2], (shorter, grown)
    call("base", expect=_lib.VC_ERR_TABLES, spoil=True)        # enqueued like the others: the device-side check refuses it
    longer = call("more")                              # more pieces than guessed (the last good call was the short one): a second launch
    assert longer[0] == 2 and longer[2] == grown[2], (longer, grown)
    assert call("base")[0] == 2                        # after a short and a long call: not of a kind, the host looks first
    assert call("base")[0] == 1
    # the packed receive layout of the two-layer function
    two_layer = [call("base", func=lambda dp, ds, dr: api.TTPL_BT_alltoallv(8, 4, 0, dp, ds, dr)) for _ in range(3)]
    assert two_layer[-1][:2] == (1, 1), two_layer
    comm.free()

    # out of the staging bound: 512 ranks, radix 2 (4.5 hops per block: staging 3.5 x the payload), an allowance of 2 MiB
    P = 512
    comm = api.VirtualComm(P)
    prob = W.make_problem(W.counts_uniform_random(P, 64, seed=14), 1, 0, 0)
    send = W.fill_send_arena(prob, 0, 22)
    want = W.expected_recv_arena(prob, send)
    dp = api.DeviceProblem(prob, comm=comm)
    ds = torch.from_numpy(send).to("cuda:0")
    comm.set_forwarding(2)
    comm.set_staging_bound(0)
    for expected_waits in (2, 2, 1):
        dr = dp.new_recv_arena(0xEE)
        assert api.tuna_algorithm(2, 0, dp, ds, dr) == 0, comm.error()
        st = comm.last_stats()
        assert int(st.host_waits) == expected_waits and st.execution == 1 and np.array_equal(dr.cpu().numpy(), want)
    comm.set_staging_bound(2)
    dr = dp.new_recv_arena(0xEE)
    assert api.tuna_algorithm(2, 0, dp, ds, dr) == 0, comm.error()
    st = comm.last_stats()
    assert st.execution == 0 and np.array_equal(dr.cpu().numpy(), want)      # refused on the device, run one launch per digit
    comm.free()
