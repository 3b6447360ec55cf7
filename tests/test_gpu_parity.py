"""Parity of the HIP path with the oracle, through the C ABI, on a real MI355X (pytest -m gpu).

Bit-exact bar: every byte of every virtual rank's receive arena — blocks and the untouched gaps between
them — equals what the CPU oracle produced from the same seeded inputs; the per-rank digests equal the ones
the real reference produced under mpiexec (tests/golden/golden.json)."""
import numpy as np
import pytest

from oracle import oracle_py as O
from rbruck_alltoallv_amd import workloads as W
from tests.helpers import CalledTwice, digest_problem, load_golden, problem_for_case, run_on

pytestmark = pytest.mark.gpu

CASES = load_golden()


# vc_comm_set_forwarding: 2 forwarded through a work-item list, 3 / 4 / 5 forwarded without one (a workgroup / a quarter of a
# wavefront per pair of ranks / a batch of pairs per wavefront), 0 one launch per digit phase
# "default": 1, the mode callers get: the library picks per call from what the last call on the communicator looked like, so
# every collective is called twice there (tests.helpers.CalledTwice)
MODES = {"forwarded": 2, "forwarded-listless": 3, "forwarded-listless-quarter": 4, "forwarded-listless-batch": 5, "launch-per-digit": 0,
         "default": 1}


@pytest.fixture(scope="module", params=list(MODES))
def api(request):
    """The package's API with one of the execution modes set on every communicator the tests create."""
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU"
    from rbruck_alltoallv_amd import api as A
    A.DEFAULT_FORWARDING = MODES[request.param]
    yield CalledTwice(A) if request.param == "default" else A
    A.DEFAULT_FORWARDING = None


def _to_dev(api, arr):
    import torch
    return torch.from_numpy(arr).to("cuda:0")


@pytest.mark.parametrize("case", CASES, ids=[c["id"] for c in CASES])
def test_golden_case(api, case):
    print("case", case["id"], flush=True)
    prob = problem_for_case(case)
    send = W.fill_send_arena(prob, case["payload"], case["seed"])
    want = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
    assert run_on(O, case, prob, send.copy(), want) == 0
    dp = api.DeviceProblem(prob)
    dsend = dp.new_send_arena()
    dp.fill_payload(case["payload"], case["seed"], dsend)            # the GPU fill must equal the host fill
    assert np.array_equal(dsend.cpu().numpy(), send)
    drecv = dp.new_recv_arena(0xEE)
    rc = run_on(api, case, dp, dsend, drecv)
    assert rc == 0, dp.comm.error()
    got = drecv.cpu().numpy()
    assert np.array_equal(got, want)
    assert [f"{int(h):016x}" for h in O.digest_recv(digest_problem(case, prob), got)] == case["digests"]
    assert np.array_equal(dsend.cpu().numpy(), send), "sendbuf must stay intact"
    assert dp.verify(dsend, drecv, packed_recv=(case["func"] == "ttpl")) == 0
    dp.comm.free()


@pytest.mark.parametrize("P", [1, 2, 3, 5, 8, 12, 17, 27, 50])
def test_flat_variants_odd_sizes(api, P):
    print("flat P", P, flush=True)
    for layout in (0, 1):
        for esz in (1, 4) if layout else (3, 12):            # element sizes as MPI_Type_contiguous would make them
            counts = W.counts_uniform_random(P, 40, seed=P)
            counts[counts % 4 == 0] = 0
            prob = W.make_problem(counts, esz, layout, layout)
            send = W.fill_send_arena(prob, 0, 5)
            want = W.expected_recv_arena(prob, send)
            dp = api.DeviceProblem(prob)
            dsend = _to_dev(api, send)
            for r in sorted({2, 3, 5, P, P + 3} - {1}):
                for name, fn in (("twophase", lambda d: api.twophase_rbruck_alltoallv(r, dp, dsend, d)),
                                 ("om", lambda d: api.twophase_rbruck_alltoallv_om(r, dp, dsend, d)),
                                 ("tuna2", lambda d: api.tuna_algorithm(r, 2, dp, dsend, d)),
                                 ("tunaP", lambda d: api.tuna_algorithm(r, 0, dp, dsend, d)),
                                 ("tuna2", lambda d: api.tuna2_algorithm(r, 3, dp, dsend, d))):
                    drecv = dp.new_recv_arena(0xEE)
                    rc = fn(drecv)
                    if name.startswith("tuna") and P < 3:
                        assert rc == -3
                        continue
                    assert rc == 0, (name, P, r, dp.comm.error())
                    assert np.array_equal(drecv.cpu().numpy(), want), (name, P, layout, esz, r)
            dp.comm.free()


def test_error_codes(api):
    counts = W.counts_uniform_random(8, 9, seed=3)
    prob = W.make_problem(counts, 4, 0, 0)
    dp = api.DeviceProblem(prob)
    s, d = dp.new_send_arena(), dp.new_recv_arena()
    for r in (0, 1, -5):
        assert api.twophase_rbruck_alltoallv(r, dp, s, d) == -1
        assert api.twophase_rbruck_alltoallv_om(r, dp, s, d) == -1
        assert api.TTPL_BT_alltoallv(4, r, 0, dp, s, d) == -1
        assert api.TTPL_BT_alltoallv_s1(4, r, 0, dp, s, d) == -1
        assert api.tuna_algorithm(r, 1, dp, s, d) == 0
    assert api.TTPL_BT_alltoallv(3, 2, 0, dp, s, d) == -2
    assert api.TTPL_BT_alltoallv_s1(5, 2, 0, dp, s, d) == -2
    assert api.uniform_spreadout_twolayer(8, 2, dp, 1, s, d) == -2
    assert api.uniform_spreadout_twolayer(4, 1, dp, 1, s, d) == -1
    # without bases: a clear error instead of a wild access
    c2 = api.VirtualComm(8)
    rc = c2.lib.twophase_rbruck_alltoallv(2, s.data_ptr(), dp.sendcounts.data_ptr(), dp.sdispls.data_ptr(), 4, d.data_ptr(),
                                          dp.recvcounts.data_ptr(), dp.rdispls.data_ptr(), 4, c2.handle)
    assert rc == -5 and "bases" in c2.error()
    c2.free()
    dp.comm.free()


def test_tables_are_validated_before_anything_moves(api):
    """A negative count or displacement would send the copy kernels outside the arenas: the planner finds it on the
    device and the call returns VC_ERR_TABLES (-7) with recvbuf untouched; the communicator stays usable."""
    import torch
    counts = W.counts_uniform_random(12, 40, seed=5)
    prob = W.make_problem(counts, 4, 0, 0)
    dp = api.DeviceProblem(prob)
    s, d = dp.new_send_arena(), dp.new_recv_arena()
    dp.fill_payload(0, 1, s)
    for name in ("sendcounts", "sdispls", "recvcounts", "rdispls"):
        table = getattr(dp, name)
        keep = int(table[7, 3].item())
        table[7, 3] = -1
        for call in (lambda: api.twophase_rbruck_alltoallv(3, dp, s, d), lambda: api.tuna_algorithm(2, 1, dp, s, d),
                     lambda: api.TTPL_BT_alltoallv_s1(4, 2, 0, dp, s, d), lambda: api.spreadout_alltoallv(dp, s, d)):
            assert call() == -7 and "negative" in dp.comm.error()
        assert bool((d == 0xEE).all())
        table[7, 3] = keep
    assert api.twophase_rbruck_alltoallv(3, dp, s, d) == 0 and dp.verify(s, d) == 0
    # the displacement scan reports what the reference's int arithmetic would silently wrap
    big = torch.full((2, 2), 2 ** 30, dtype=torch.int32, device="cuda:0")
    displs = torch.zeros_like(big)
    ext = torch.zeros(2, dtype=torch.int64, device="cuda:0")
    c2 = api.VirtualComm(2)
    assert c2.lib.vc_displs_from_counts(big.data_ptr(), displs.data_ptr(), ext.data_ptr(), c2.handle) == -8
    assert ext.tolist() == [2 ** 31, 2 ** 31]
    big[1, 0] = -4
    assert c2.lib.vc_displs_from_counts(big.data_ptr(), displs.data_ptr(), ext.data_ptr(), c2.handle) == -7
    c2.free()
    dp.comm.free()


def _oracle_traffic(rec, P, select):
    m = np.zeros((P, P), dtype=np.int64)
    for t in rec[select]:
        m[int(t["src"]), int(t["dst"])] += int(t["bytes"])
    return m


@pytest.mark.parametrize("func,P,r", [("twophase", 27, 3), ("om", 64, 4), ("tuna", 30, 29), ("tuna", 17, 5)])
def test_route_on_gpu_equals_oracle_trace(api, func, P, r):
    """The launches of the GPU call carry, rank to rank, the bytes of the reference's rounds digit by digit."""
    if api.DEFAULT_FORWARDING:
        pytest.skip("launches can be inspected one by one only in the launch-per-digit mode")
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
    dp = api.DeviceProblem(prob)
    ds, dr = _to_dev(api, send), dp.new_recv_arena()
    gfn = {"twophase": lambda: api.twophase_rbruck_alltoallv(r, dp, ds, dr),
           "om": lambda: api.twophase_rbruck_alltoallv_om(r, dp, ds, dr),
           "tuna": lambda: api.tuna_algorithm(r, 0, dp, ds, dr)}[func]
    assert gfn() == 0
    st = dp.comm.last_stats()
    digits = list(dict.fromkeys(rec[rec["kind"] != 4]["digit"].tolist()))
    assert st.n_launches == len(digits)
    for k, x in enumerate(digits):
        want = _oracle_traffic(rec, P, (rec["digit"] == x) & (rec["kind"] != 4))
        if k == 0:
            want += _oracle_traffic(rec, P, rec["kind"] == 4)
        assert np.array_equal(dp.comm.last_traffic(k), want)
        assert st.launch_bytes[k] == int(want.sum())
    assert st.payload_bytes == prob.payload_bytes
    assert st.moved_bytes * 2 == W.algorithmic_bytes(prob.sendcounts, prob.esz, W.hops_flat(P, min(r, P - 1) if func == "tuna" else r))
    dp.comm.free()


def test_caller_side_metadata_kernels(api):
    """Count-matrix exchange (transpose), displacement prefix sums, bases and global maximum against numpy."""
    import ctypes as C
    import torch
    for P in (1, 5, 32, 33, 100, 257, 1024):
        counts = W.counts_uniform_random(P, 5000, seed=P)
        comm = api.VirtualComm(P)
        dc = _to_dev(api, counts)
        out = torch.zeros_like(dc)
        assert comm.lib.vc_alltoall_counts(dc.data_ptr(), out.data_ptr(), comm.handle) == 0
        assert np.array_equal(out.cpu().numpy(), counts.T)
        displs = torch.zeros_like(dc)
        ext = torch.zeros(P, dtype=torch.int64, device="cuda:0")
        assert comm.lib.vc_displs_from_counts(dc.data_ptr(), displs.data_ptr(), ext.data_ptr(), comm.handle) == 0
        want_d, want_e = W.layout_displs(counts, 0)
        assert np.array_equal(displs.cpu().numpy(), want_d) and np.array_equal(ext.cpu().numpy(), want_e)
        base = torch.zeros(P, dtype=torch.int64, device="cuda:0")
        tot = torch.zeros(1, dtype=torch.int64, device="cuda:0")
        assert comm.lib.vc_bases_from_extents(ext.data_ptr(), 4, 256, base.data_ptr(), tot.data_ptr(), comm.handle) == 0
        wb, wt = W.aligned_bases(want_e * 4, 256)
        assert np.array_equal(base.cpu().numpy(), wb) and int(tot.item()) == wt
        mx = torch.zeros(1, dtype=torch.int32, device="cuda:0")
        assert comm.lib.vc_allreduce_max_count(dc.data_ptr(), mx.data_ptr(), comm.handle) == 0
        assert int(mx.item()) == int(counts.max())
        comm.free()


@pytest.mark.parametrize("layout", [0, 1])
def test_large_blocks_split_into_pieces(api, layout):
    """Blocks far above the 8 KiB work-item size, odd lengths and alignments, zeros in between."""
    P = 12
    counts = (W.counts_uniform_random(P, 70000, seed=11) * (W.counts_uniform_random(P, 3, seed=12) > 0)).astype(np.int32)
    prob = W.make_problem(counts, 1, layout, layout)
    send = W.fill_send_arena(prob, 0, 9)
    want = W.expected_recv_arena(prob, send)
    dp = api.DeviceProblem(prob)
    ds = _to_dev(api, send)
    for name, fn in (("twophase r=3", lambda d: api.twophase_rbruck_alltoallv(3, dp, ds, d)),
                     ("om r=2", lambda d: api.twophase_rbruck_alltoallv_om(2, dp, ds, d)),
                     ("tuna r=4 b=2", lambda d: api.tuna_algorithm(4, 2, dp, ds, d)),
                     ("s1 n=4 r=2", lambda d: api.TTPL_BT_alltoallv_s1(4, 2, 3, dp, ds, d))):
        dr = dp.new_recv_arena(0xEE)
        assert fn(dr) == 0, (name, dp.comm.error())
        assert np.array_equal(dr.cpu().numpy(), want), name
    prob2 = W.make_problem(counts, 1, layout, 0)
    dp2 = api.DeviceProblem(prob2)
    send2 = W.fill_send_arena(prob2, 0, 9)
    dr = dp2.new_recv_arena(0xEE)
    assert api.TTPL_BT_alltoallv(6, 3, 1, dp2, _to_dev(api, send2), dr) == 0
    assert np.array_equal(dr.cpu().numpy(), W.expected_recv_arena(prob2, send2))
    dp.comm.free()
    dp2.comm.free()


@pytest.mark.parametrize("P", [1, 5, 8, 32])
def test_linear_comparators(api, P):
    for layout in (0, 1):
        counts = W.counts_uniform_random(P, 3000, seed=P + 40)
        counts[counts % 4 == 0] = 0
        prob = W.make_problem(counts, 2, layout, layout)
        send = W.fill_send_arena(prob, 0, 3)
        want = W.expected_recv_arena(prob, send)
        dp = api.DeviceProblem(prob)
        ds = _to_dev(api, send)
        for name, fn in (("spreadout", lambda d: api.spreadout_alltoallv(dp, ds, d)),
                         ("linear", lambda d: api.ompi_alltoallv_intra_basic_linear(dp, ds, d)),
                         ("pairwise", lambda d: api.ompi_alltoallv_intra_pairwise(dp, ds, d)),
                         ("xor", lambda d: api.exclisive_or_alltoallv(dp, ds, d)),
                         ("scattered3", lambda d: api.MPICH_intra_scattered(3, dp, ds, d)),
                         ("scattered0", lambda d: api.MPICH_intra_scattered(0, dp, ds, d))):
            dr = dp.new_recv_arena(0xEE)
            rc = fn(dr)
            if name == "xor" and P & (P - 1):
                assert rc == -1
                continue
            assert rc == 0, (name, dp.comm.error())
            assert np.array_equal(dr.cpu().numpy(), want), (name, P, layout)
            st = dp.comm.last_stats()
            assert st.moved_bytes == prob.payload_bytes
        dp.comm.free()


@pytest.mark.parametrize("P,n", [(8, 4), (12, 3), (32, 8), (16, 1), (256, 32)])
def test_linear_twolayer_comparators(api, P, n):
    """twolayer_communicator_linear / _s2 (src/twolayer_communicator_linear.cpp:13-88, 92-192)."""
    for layout in (0, 1):
        counts = W.counts_uniform_random(P, 3000, seed=P + n)
        counts[counts % 4 == 0] = 0
        prob = W.make_problem(counts, 2, layout, layout)
        send = W.fill_send_arena(prob, 0, 3)
        want = W.expected_recv_arena(prob, send)
        dp = api.DeviceProblem(prob)
        ds = _to_dev(api, send)
        for name, fn, launches in (
                ("plain", lambda d: api.twolayer_communicator_linear(n, dp, ds, d), 2),
                ("s2 0 0", lambda d: api.twolayer_communicator_linear_s2(n, 0, 0, dp, ds, d), 2),
                ("s2 2 5", lambda d: api.twolayer_communicator_linear_s2(n, 2, 5, dp, ds, d), -(-n // min(2, n)) + -(-(P - 1) // 5))):
            dr = dp.new_recv_arena(0xEE)
            assert fn(dr) == 0, (name, dp.comm.error())
            assert np.array_equal(dr.cpu().numpy(), want), (name, P, n, layout)
            st = dp.comm.last_stats()
            assert st.moved_bytes == prob.payload_bytes and st.n_launches == (1 if api.DEFAULT_FORWARDING else launches)
        dr = dp.new_recv_arena(0xEE)
        assert api.twolayer_communicator_linear(P, dp, ds, dr) == -2
        assert api.twolayer_communicator_linear_s2(0, 1, 1, dp, ds, dr) == -2
        dp.comm.free()


@pytest.mark.parametrize("P,n,r", [(8, 4, 2), (12, 3, 3), (64, 4, 2), (64, 16, 4), (16, 1, 2), (8, 8, 2), (256, 16, 4), (243, 9, 3)])
def test_twolayer_bruck(api, P, n, r):
    """TTPL_rbruck_alltoallv (src/twophase_twolayer_rbruck.cpp:15-235, inter-node Bruck completed) against the oracle,
    the definition and the oracle's per-digit traffic."""
    for layout in (0, 1):
        counts = W.counts_uniform_random(P, 3000 if P <= 64 else 300, seed=P + n + r)
        counts[counts % 4 == 0] = 0
        prob = W.make_problem(counts, 2, layout, layout)
        send = W.fill_send_arena(prob, 0, 3)
        want = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
        with O.trace() as t:
            assert O.TTPL_rbruck_alltoallv(n, r, prob, send, want) == 0
        assert np.array_equal(want, W.expected_recv_arena(prob, send))
        dp = api.DeviceProblem(prob)
        ds = _to_dev(api, send)
        dr = dp.new_recv_arena(0xEE)
        assert api.TTPL_rbruck_alltoallv(n, r, dp, ds, dr) == 0, dp.comm.error()
        assert np.array_equal(dr.cpu().numpy(), want), (P, n, r, layout)
        assert dp.verify(ds, dr) == 0
        rec = t.records
        st = dp.comm.last_stats()
        assert st.moved_bytes == int(rec["bytes"].sum())
        inter = list(dict.fromkeys(rec[rec["kind"] == 6]["digit"].tolist()))
        if inter and P <= 64 and not api.DEFAULT_FORWARDING:
            m = np.zeros((P, P), dtype=np.int64)
            sel = rec[(rec["kind"] == 6) & (rec["digit"] == inter[-1])]
            np.add.at(m, (sel["src"], sel["dst"]), sel["bytes"])
            assert np.array_equal(dp.comm.last_traffic(st.n_launches - 1), m)
        assert api.TTPL_rbruck_alltoallv(n, 1, dp, ds, dr) == -1
        assert api.TTPL_rbruck_alltoallv(P + 1, 2, dp, ds, dr) == -2
        dp.comm.free()


@pytest.mark.parametrize("shift", [(0, 0), (5, 0), (0, 7), (3, 13)])
def test_arena_pointers_of_any_alignment(api, shift):
    """sendbuf / recvbuf need not be 16-byte aligned."""
    import torch
    s_shift, r_shift = shift
    counts = (W.counts_uniform_random(12, 30000, seed=5) * (W.counts_uniform_random(12, 3, seed=6) > 0)).astype(np.int32)
    prob = W.make_problem(counts, 1, 1, 0)
    send = W.fill_send_arena(prob, 0, 9)
    want = W.expected_recv_arena(prob, send)
    dp = api.DeviceProblem(prob)
    sbig = torch.zeros(prob.send_bytes + 64, dtype=torch.uint8, device="cuda:0")
    ds = sbig[s_shift:s_shift + prob.send_bytes]
    ds.copy_(torch.from_numpy(send))
    for name, fn in (("twophase r=3", lambda d: api.twophase_rbruck_alltoallv(3, dp, ds, d)),
                     ("tuna r=2 b=1", lambda d: api.tuna_algorithm(2, 1, dp, ds, d)),
                     ("ttpl n=4 r=4", lambda d: api.TTPL_BT_alltoallv(4, 4, 0, dp, ds, d)),
                     ("s1 n=6 r=2", lambda d: api.TTPL_BT_alltoallv_s1(6, 2, 5, dp, ds, d)),
                     ("spreadout", lambda d: api.spreadout_alltoallv(dp, ds, d))):
        rbig = torch.full((prob.recv_bytes + 64,), 0xEE, dtype=torch.uint8, device="cuda:0")
        dr = rbig[r_shift:r_shift + prob.recv_bytes]
        assert fn(dr) == 0, (name, dp.comm.error())
        assert np.array_equal(dr.cpu().numpy(), want), (name, shift)
        assert bool((rbig[:r_shift] == 0xEE).all()) and bool((rbig[r_shift + prob.recv_bytes:] == 0xEE).all())
    dp.comm.free()


def test_persistent_plans(api):
    """A plan executes the same copies as the call it was made from, any number of times, on any arenas."""
    import torch
    counts = W.counts_uniform_random(24, 5000, seed=21)
    counts[counts % 5 == 0] = 0
    prob = W.make_problem(counts, 2, 1, 0)
    send = W.fill_send_arena(prob, 0, 4)
    want = W.expected_recv_arena(prob, send)
    dp = api.DeviceProblem(prob)
    ds = _to_dev(api, send)
    for function, kw, direct in (
        ("twophase_rbruck_alltoallv", dict(r=3), lambda d: api.twophase_rbruck_alltoallv(3, dp, ds, d)),
        ("tuna_algorithm", dict(r=4, batch=2), lambda d: api.tuna_algorithm(4, 2, dp, ds, d)),
        ("TTPL_BT_alltoallv", dict(n=6, r=6, batch=0), lambda d: api.TTPL_BT_alltoallv(6, 6, 0, dp, ds, d)),
        ("TTPL_BT_alltoallv_s1", dict(n=4, r=2, batch=7), lambda d: api.TTPL_BT_alltoallv_s1(4, 2, 7, dp, ds, d)),
        ("MPICH_intra_scattered", dict(batch=5), lambda d: api.MPICH_intra_scattered(5, dp, ds, d)),
    ):
        dr = dp.new_recv_arena(0xEE)
        plan = api.Plan(function, dp, dr, **kw)
        assert plan.rc == 0, dp.comm.error()
        assert direct(dr) == 0
        per_digit = not api.DEFAULT_FORWARDING
        traffic_direct = [dp.comm.last_traffic(k) for k in range(dp.comm.last_stats().n_launches)] if per_digit else [None]
        for rep in range(3):
            dr2 = dp.new_recv_arena(0xEE)
            ds2 = ds.clone()
            assert plan.execute(ds2, dr2) == 0, dp.comm.error()
            assert np.array_equal(dr2.cpu().numpy(), want), (function, rep)
        st = dp.comm.last_stats()
        assert st.n_launches == len(traffic_direct) and st.payload_bytes == prob.payload_bytes
        for k, m in enumerate(traffic_direct if per_digit else []):
            assert np.array_equal(dp.comm.last_traffic(k), m)
        # a receive arena with other low address bits is refused, not mis-copied
        rbig = torch.full((prob.recv_bytes + 16,), 0xEE, dtype=torch.uint8, device="cuda:0")
        assert plan.execute(ds, rbig[3:]) == -5
        plan.free()
    bad = api.Plan("no_such_function", dp, dp.new_recv_arena())
    assert bad.rc == -5
    assert api.Plan("twophase_rbruck_alltoallv", dp, dp.new_recv_arena(), r=1).rc == -1
    dp.comm.free()


def _device_check(api, prob, seed, calls):
    """Runs calls on device-filled payload and checks each with the exact on-device definition check."""
    dp = api.DeviceProblem(prob)
    ds = dp.new_send_arena()
    dp.fill_payload(0, seed, ds)
    for name, fn, packed in calls(dp, ds):
        print("  ", name, flush=True)
        dr = dp.new_recv_arena(0xEE)
        assert fn(dr) == 0, (name, dp.comm.error())
        assert dp.verify(ds, dr, packed_recv=packed) == 0, name
        st = dp.comm.last_stats()
        assert st.payload_bytes == prob.payload_bytes
    dp.comm.free()


def test_benchmark_shapes_at_reduced_size(api):
    """The five benchmark shapes at their full rank counts with smaller blocks: many digits, many launches."""
    c3 = W.counts_zipf(256, 4096, 1.2, 5, 0)
    _device_check(api, W.make_problem(c3, 4, 0, 0), 1, lambda dp, ds: [
        ("C3 twophase r=16", lambda d: api.twophase_rbruck_alltoallv(16, dp, ds, d), False),
        ("C3 om r=2", lambda d: api.twophase_rbruck_alltoallv_om(2, dp, ds, d), False),
        ("C3 tuna r=255 b=1 (255 launches)", lambda d: api.tuna_algorithm(255, 1, dp, ds, d), False)])
    c4 = W.counts_normal(1024, 256.0, 64.0, 0, 1024, 0)
    _device_check(api, W.make_problem(c4, 1, 0, 0), 2, lambda dp, ds: [
        ("C4 ttpl n=32 r=32", lambda d: api.TTPL_BT_alltoallv(32, 32, 0, dp, ds, d), True),
        ("C4 ttpl n=32 r=2 bblock=5", lambda d: api.TTPL_BT_alltoallv(32, 2, 5, dp, ds, d), True),
        ("C4 s1 n=32 r=32 bblock=100", lambda d: api.TTPL_BT_alltoallv_s1(32, 32, 100, dp, ds, d), False),
        ("C4 s1 n=64 r=8", lambda d: api.TTPL_BT_alltoallv_s1(64, 8, 0, dp, ds, d), False),
        ("C4 twophase r=2 (10 digits)", lambda d: api.twophase_rbruck_alltoallv(2, dp, ds, d), False)])
    c5 = W.counts_fft_rows(512, 32, 4096)
    _device_check(api, W.make_problem(c5, 8, 0, 0), 3, lambda dp, ds: [
        (f"C5 tuna r={r} b={b}", (lambda d, r=r, b=b: api.tuna_algorithm(r, b, dp, ds, d)), False)
        for r, b in ((2, 0), (8, 0), (32, 0), (512, 0), (32, 7))])
    up = W.make_uniform_problem(256, 300, 4)
    _device_check(api, up, 4, lambda dp, ds: [
        ("uniform spreadout n=16 r=4", lambda d: api.uniform_spreadout_twolayer(16, 4, dp, 300, ds, d), False),
        ("uniform isplit n=32 r=3", lambda d: api.uniform_inverse_isplit_r_bruck(32, 3, 2, dp, 300, ds, d), False)])


def test_persistent_plans_of_the_uniform_functions(api):
    """vc_plan_create for the equal-block functions: the block length travels as `batch`, the tables are implied."""
    up = W.make_uniform_problem(96, 700, 2)
    dp = api.DeviceProblem(up)
    ds = dp.new_send_arena()
    dp.fill_payload(0, 8, ds)
    for function, n, r, direct in (("uniform_spreadout_twolayer", 8, 3, lambda d: api.uniform_spreadout_twolayer(8, 3, dp, 700, ds, d)),
                                   ("uniform_inverse_isplit_r_bruck", 12, 2, lambda d: api.uniform_inverse_isplit_r_bruck(12, 2, 2, dp, 700, ds, d))):
        want = dp.new_recv_arena(0xEE)
        assert direct(want) == 0, dp.comm.error()
        assert dp.verify(ds, want) == 0
        got = dp.new_recv_arena(0xEE)
        plan = api.Plan(function, dp, got, n=n, r=r, batch=700)
        assert plan.rc == 0, dp.comm.error()
        for _ in range(2):
            got.fill_(0xEE)
            assert plan.execute(ds, got) == 0, dp.comm.error()
            assert bool((got == want).all()), function
        plan.free()
    assert api.Plan("uniform_spreadout_twolayer", dp, want, n=7, r=2, batch=700).rc == -2       # 7 does not divide 96
    dp.comm.free()


def _byte_sum(t):
    """Sum of all bytes of a uint8 tensor, in slices (a one-shot sum would widen the whole tensor to int64 first)."""
    import torch
    step = 1 << 28
    return sum(int(t[i:i + step].sum(dtype=torch.int64)) for i in range(0, t.numel(), step))


def _transposed(prob):
    """The alltoallv that undoes `prob`: every rank sends back what it received, from where it landed."""
    import dataclasses
    return dataclasses.replace(prob, sendcounts=prob.recvcounts, sdispls=prob.rdispls, sbase=prob.rbase, send_bytes=prob.recv_bytes,
                               recvcounts=prob.sendcounts, rdispls=prob.sdispls, rbase=prob.sbase, recv_bytes=prob.send_bytes)


@pytest.mark.parametrize("name", ["C2", "C3", "C4", "C5"])
def test_benchmark_configurations_at_full_size(api, name):
    """The benchmark configurations at their real sizes (up to 17 GB of payload), where no host oracle can follow:
    the on-device definition check, a checksum over all bytes, and the round trip — the transposed alltoallv, run by
    a different function, must give back the send arena bit for bit."""
    import torch
    counts, esz, tun = W.config_counts(name, 0)
    prob = W.make_problem(counts, esz, 0, 0)
    P = prob.P
    fwd = {"C2": [("twophase r=2", lambda dp, s, d: api.twophase_rbruck_alltoallv(2, dp, s, d), False),
                  ("tuna r=8", lambda dp, s, d: api.tuna_algorithm(8, 0, dp, s, d), False)],
           "C3": [("twophase r=16", lambda dp, s, d: api.twophase_rbruck_alltoallv(16, dp, s, d), False)],
           "C4": [("ttpl n=32 r=32", lambda dp, s, d: api.TTPL_BT_alltoallv(32, 32, 0, dp, s, d), True),
                  ("ttpl_rbruck n=32 r=4", lambda dp, s, d: api.TTPL_rbruck_alltoallv(32, 4, dp, s, d), False)],
           "C5": [("tuna r=32", lambda dp, s, d: api.tuna_algorithm(32, 0, dp, s, d), False)]}[name]
    if api.DEFAULT_FORWARDING in (0, 1, 2):
        # the other radices the configuration names, through the work-item list and one launch per digit (the listless
        # kernels give a 1 MiB block to 16 or 256 lanes: exact, shown above for one radix, but slow)
        fwd += {"C2": [("twophase r=4", lambda dp, s, d: api.twophase_rbruck_alltoallv(4, dp, s, d), False),
                       ("twophase r=8", lambda dp, s, d: api.twophase_rbruck_alltoallv(8, dp, s, d), False)],
                "C5": [("tuna r=2", lambda dp, s, d: api.tuna_algorithm(2, 0, dp, s, d), False),
                       ("tuna r=8", lambda dp, s, d: api.tuna_algorithm(8, 0, dp, s, d), False),
                       ("tuna r=512", lambda dp, s, d: api.tuna_algorithm(512, 0, dp, s, d), False)]}.get(name, [])
    back = {"C2": lambda dp, s, d: api.twophase_rbruck_alltoallv_om(4, dp, s, d),
            "C3": lambda dp, s, d: api.tuna_algorithm(2, 0, dp, s, d),
            "C4": lambda dp, s, d: api.TTPL_BT_alltoallv_s1(32, 32, 0, dp, s, d),
            "C5": lambda dp, s, d: api.spreadout_alltoallv(dp, s, d)}[name]
    dp = api.DeviceProblem(prob)
    ds = dp.new_send_arena()
    ds.zero_()
    dp.fill_payload(0, 11, ds)
    checksum = _byte_sum(ds)
    for label, fn, packed in fwd:
        print("  ", name, label, flush=True)
        dr = dp.new_recv_arena(0)
        assert fn(dp, ds, dr) == 0, (label, dp.comm.error())
        assert dp.verify(ds, dr, packed_recv=packed) == 0, label
        assert _byte_sum(dr) == checksum, label
        assert dp.comm.last_stats().payload_bytes == prob.payload_bytes
    dp.comm.free()
    tp = api.DeviceProblem(_transposed(prob))
    dback = tp.new_recv_arena(0)
    assert back(tp, dr, dback) == 0, tp.comm.error()
    assert torch.equal(dback, ds), name
    tp.comm.free()


def test_blocks_beyond_two_gib(api):
    """Counts and displacements are int32 elements, byte offsets 64-bit: a 2.4 GB block (300 M elements of 8 bytes; the
    reference's int byte arithmetic, src/twophase_tunable_rbruckv.cpp:98, would overflow) next to empty and tiny ones."""
    if api.DEFAULT_FORWARDING in (4, 5):
        pytest.skip("one 2.4 GB block moved by the 16 lanes of its pair: exact, but half a minute")
    import torch
    counts = np.array([[3, 300_000_000, 0], [1, 0, 7], [200_000_000, 5, 2]], dtype=np.int32)
    prob = W.make_problem(counts, 8, 0, 0)
    assert prob.payload_bytes > 2 ** 31
    dp = api.DeviceProblem(prob)
    ds = dp.new_send_arena()
    dp.fill_payload(0, 5, ds)
    checksum = _byte_sum(ds)
    for name, fn in (("twophase r=2", lambda d: api.twophase_rbruck_alltoallv(2, dp, ds, d)),
                     ("tuna r=2", lambda d: api.tuna_algorithm(2, 0, dp, ds, d)),
                     ("ttpl n=1", lambda d: api.TTPL_BT_alltoallv_s1(1, 2, 0, dp, ds, d)),
                     ("ttpl_rbruck n=1 r=2", lambda d: api.TTPL_rbruck_alltoallv(1, 2, dp, ds, d)),
                     ("spreadout", lambda d: api.spreadout_alltoallv(dp, ds, d))):
        print("  ", name, flush=True)
        dr = dp.new_recv_arena(0)
        assert fn(dr) == 0, (name, dp.comm.error())
        assert dp.verify(ds, dr) == 0, name
        assert _byte_sum(dr) == checksum, name
        del dr
    dp.comm.free()


def test_more_than_4096_ranks(api):
    """Tables of 4100 x 4100 entries, mostly empty pairs."""
    P = 4100
    rng = np.random.default_rng(3)
    counts = np.where(rng.random((P, P)) < 0.01, rng.integers(1, 400, (P, P)), 0).astype(np.int32)
    prob = W.make_problem(counts, 2, 0, 0)
    dp = api.DeviceProblem(prob)
    ds = dp.new_send_arena()
    dp.fill_payload(0, 2, ds)
    dr = dp.new_recv_arena(0xEE)
    assert api.twophase_rbruck_alltoallv(65, dp, ds, dr) == 0, dp.comm.error()
    assert dp.verify(ds, dr) == 0
    st = dp.comm.last_stats()
    assert st.n_launches == (1 if api.DEFAULT_FORWARDING else 2) and st.payload_bytes == prob.payload_bytes
    dp.comm.free()


def test_more_work_items_than_one_launch_holds(api):
    """4100 x 4100 non-empty pairs are 16.81 M work items; one dispatch holds 2^32 / 256 - 8 workgroups (its grid is
    counted in work-items, in 32 bits), so the list goes out in two launches."""
    P = 4100
    rng = np.random.default_rng(8)
    counts = rng.integers(1, 4, (P, P)).astype(np.int32)
    prob = W.make_problem(counts, 1, 0, 0)
    dp = api.DeviceProblem(prob)
    ds = dp.new_send_arena()
    dp.fill_payload(0, 6, ds)
    for name, fn in (("spreadout", lambda dr: api.spreadout_alltoallv(dp, ds, dr)),
                     ("twophase r=65", lambda dr: api.twophase_rbruck_alltoallv(65, dp, ds, dr))):
        print("  ", name, flush=True)
        dr = dp.new_recv_arena(0xEE)
        assert fn(dr) == 0, (name, dp.comm.error())
        assert dp.verify(ds, dr) == 0, name
        assert dp.comm.last_stats().payload_bytes == prob.payload_bytes
    dp.comm.free()


def test_distributions_of_the_reference_drivers(api):
    """examples/other_distributions.cpp (truncated normal, power law) and examples/FFT_distribution.cpp (sparse blocks) at
    256 ranks, 8-byte elements, through the functions those drivers call."""
    for name, counts in (("truncated normal", W.counts_truncated_normal_rows(256, 600.0, 250.0, 1500, seed=1)),
                         ("power law", W.counts_power_law_rows(256, 0.98, 4000, seed=2)),
                         ("sparse blocks", W.counts_sparse_blocks(256, 0.4, 0.25, 777)),
                         ("last block differs", W.counts_sparse_blocks(256, 0.0, 0.0, 50, last=90001))):
        _device_check(api, W.make_problem(counts, 8, 0, 0), 6, lambda dp, ds: [
            (f"{name}: twophase r=16", lambda d: api.twophase_rbruck_alltoallv(16, dp, ds, d), False),
            (f"{name}: s1 n=16 r=4", lambda d: api.TTPL_BT_alltoallv_s1(16, 4, 0, dp, ds, d), False),
            (f"{name}: ttpl n=32 r=32", lambda d: api.TTPL_BT_alltoallv(32, 32, 0, dp, ds, d), True)])


def test_reference_input_matrices(api):
    """The reference's own communication patterns (inputs/<P>proc), scaled down, through the function its driver uses."""
    import os
    from tests.helpers import INPUTS_DIR
    for P, div in ((256, 4096), (512, 2048), (1024, 1024)):
        counts = W.counts_from_npz(os.path.join(INPUTS_DIR, f"global_comm_pattern_{P}proc.npz"), div)
        _device_check(api, W.make_problem(counts, 1, 0, 0), 5, lambda dp, ds: [
            (f"ML{P} twophase r=32", lambda d: api.twophase_rbruck_alltoallv(32, dp, ds, d), False),
            (f"ML{P} tuna r=8", lambda d: api.tuna_algorithm(8, 0, dp, ds, d), False)])


@pytest.mark.parametrize("P", [64, 1024])
def test_reference_input_matrices_at_full_size(api, P):
    """The smallest and the largest of the reference's communication patterns at their real sizes (5.2 and 12.8 GB of
    payload, examples/MLinputs_example.cpp:96: twophase_rbruck_alltoallv on 1-byte elements), checked as the benchmark
    configurations are: definition check on the device, byte sum, and the transposed alltoallv by another function."""
    if api.DEFAULT_FORWARDING not in (0, 1, 2):
        pytest.skip("blocks of megabytes belong to the work-item list and to launch-per-digit execution")
    import os
    import torch
    from tests.helpers import INPUTS_DIR
    counts = W.counts_from_npz(os.path.join(INPUTS_DIR, f"global_comm_pattern_{P}proc.npz"))
    prob = W.make_problem(counts, 1, 0, 0)
    dp = api.DeviceProblem(prob)
    ds = dp.new_send_arena()
    ds.zero_()
    dp.fill_payload(0, 13, ds)
    checksum = _byte_sum(ds)
    dr = dp.new_recv_arena(0)
    print("  ML", P, "payload", prob.payload_bytes, flush=True)
    assert api.twophase_rbruck_alltoallv(32, dp, ds, dr) == 0, dp.comm.error()
    assert dp.verify(ds, dr) == 0
    assert _byte_sum(dr) == checksum
    assert dp.comm.last_stats().payload_bytes == prob.payload_bytes
    dp.comm.free()
    tp = api.DeviceProblem(_transposed(prob))
    dback = tp.new_recv_arena(0)
    assert api.tuna_algorithm(8, 0, tp, dr, dback) == 0, tp.comm.error()
    assert torch.equal(dback, ds)
    tp.comm.free()


def test_suggest_radix_matches_the_traffic_model(api):
    for P, n in ((64, 0), (100, 0), (256, 0), (128, 32), (64, 8)):
        counts = W.counts_zipf(P, 4096, 1.2, 5, P)
        prob = W.make_problem(counts, 4, 0, 0)
        dp = api.DeviceProblem(prob)
        cands = [2, 3, 4, 8, 16, 32, P]
        best, moved = api.suggest_radix(dp, cands, n)
        for r, m in zip(cands, moved):
            hops = W.hops_twolayer(P, n, r) if n else W.hops_flat(P, r)
            assert 2 * m == W.algorithmic_bytes(counts, 4, hops), (P, n, r)
        assert best in cands
        # the model prefers fewer bytes when launch counts are equal
        assert moved[cands.index(best)] <= moved[0]
        dp.comm.free()


def test_plan_in_a_hip_graph(api):
    """vc_plan_execute_async only enqueues kernels, so a plan can be captured into a graph and replayed; every replay,
    with other work and synchronisations in between, gives the eager result."""
    import torch
    counts = W.counts_uniform_random(64, 4096, seed=0)
    prob = W.make_problem(counts, 1, 0, 0)
    send = W.fill_send_arena(prob, 0, 4)
    want = W.expected_recv_arena(prob, send, fill=0)
    dp = api.DeviceProblem(prob)
    ds = _to_dev(api, send)
    dr = dp.new_recv_arena(0)
    plan = api.Plan("twophase_rbruck_alltoallv", dp, dr, r=2)
    assert plan.rc == 0
    assert plan.execute(ds, dr) == 0 and np.array_equal(dr.cpu().numpy(), want)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        dp.comm.use_current_stream()
        assert plan.execute_async(ds, dr) == 0, dp.comm.error()
    dp.comm.use_current_stream()
    for rep in range(4):
        dr.fill_(rep + 1)                                  # eager work between replays: the stale result is wiped
        dr.zero_()                                         # (bytes between the ranks' buffers are not written by the call)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert np.array_equal(dr.cpu().numpy(), want), rep
        ds2 = ds.clone()
        assert plan.execute(ds2, dr) == 0                 # and eager calls of the library in between
    plan.free()
    dp.comm.free()


# ---- forwarded execution (vc_comm_set_forwarding): one launch, every block piece carried through all its hops ----

@pytest.mark.parametrize("case", CASES, ids=[c["id"] for c in CASES])
def test_golden_case_forwarded(api, case):
    print("case", case["id"], flush=True)
    prob = problem_for_case(case)
    send = W.fill_send_arena(prob, case["payload"], case["seed"])
    want = np.full(prob.recv_bytes, 0xEE, dtype=np.uint8)
    assert run_on(O, case, prob, send.copy(), want) == 0
    dp = api.DeviceProblem(prob)
    dp.comm.set_forwarding(api.DEFAULT_FORWARDING or 2)
    dsend = _to_dev(api, send)
    drecv = dp.new_recv_arena(0xEE)
    rc = run_on(api, case, dp, dsend, drecv)
    assert rc == 0, dp.comm.error()
    got = drecv.cpu().numpy()
    assert np.array_equal(got, want)
    assert [f"{int(h):016x}" for h in O.digest_recv(digest_problem(case, prob), got)] == case["digests"]
    assert np.array_equal(dsend.cpu().numpy(), send), "sendbuf must stay intact"
    st = dp.comm.last_stats()
    assert st.n_launches == 1
    # same hops as the launch-per-digit execution: every hop of every block is written once
    dp.comm.set_forwarding(False)
    drecv2 = dp.new_recv_arena(0xEE)
    assert run_on(api, case, dp, dsend, drecv2) == 0
    if case["func"] != "ttpl":                       # (the coalesced variant also counts nothing more: same hops per block)
        assert dp.comm.last_stats().moved_bytes == st.moved_bytes
    assert st.payload_bytes == prob.payload_bytes
    dp.comm.free()


def test_seeded_random_sweep(api):
    """Random rank counts, radices, node sizes, batches, element sizes, count ranges (with zeros and a few huge blocks),
    displacement layouts and recvbuf alignments; three of the entry points per case, checked against the definition
    on the device, and the bytes around recvbuf must stay untouched."""
    import random
    import torch
    rnd = random.Random(2024)
    for it in range(60):
        P = rnd.choice([2, 3, 4, 6, 7, 8, 12, 16, 24, 27, 30, 36, 48, 64, 81, 96, 100, 128])
        esz = rnd.choice([1, 1, 2, 3, 4, 8, 12])
        hi = rnd.choice([0, 1, 5, 60, 700, 5000, 20000])
        layout = rnd.choice([0, 1])
        counts = W.counts_uniform_random(P, hi, seed=it)
        if rnd.random() < 0.5:
            counts[counts % rnd.choice([2, 3, 5]) == 0] = 0
        if rnd.random() < 0.2 and P >= 4:
            counts[rnd.randrange(P), rnd.randrange(P)] = rnd.choice([100000, 300000])
        n = rnd.choice([d for d in range(1, P + 1) if P % d == 0])
        r = rnd.choice([2, 3, 4, 5, 8, 16, 31, P, P + 1])
        b = rnd.choice([0, 1, 2, 7])
        prob = W.make_problem(counts, esz, layout, layout)
        dp = api.DeviceProblem(prob)
        ds = dp.new_send_arena()
        dp.fill_payload(0, it, ds)
        shift = rnd.choice([0, 0, 1, 7, 64, 100])
        rbig = torch.full((prob.recv_bytes + 256,), 0xEE, dtype=torch.uint8, device="cuda:0")
        dr = rbig[shift:shift + prob.recv_bytes]
        calls = [("twophase", lambda: api.twophase_rbruck_alltoallv(r, dp, ds, dr), False),
                 ("om", lambda: api.twophase_rbruck_alltoallv_om(r, dp, ds, dr), False),
                 ("s1", lambda: api.TTPL_BT_alltoallv_s1(n, r, b, dp, ds, dr), False),
                 ("rbruck", lambda: api.TTPL_rbruck_alltoallv(n, r, dp, ds, dr), False),
                 ("scattered", lambda: api.MPICH_intra_scattered(b, dp, ds, dr), False)]
        if P >= 3:
            calls += [("tuna", lambda: api.tuna_algorithm(r, b, dp, ds, dr), False),
                      ("tuna2", lambda: api.tuna2_algorithm(r, b, dp, ds, dr), False)]
        if layout == 0:
            calls.append(("ttpl", lambda: api.TTPL_BT_alltoallv(n, r, b, dp, ds, dr), True))
        if 1 <= n < P:
            calls.append(("tl_s2", lambda: api.twolayer_communicator_linear_s2(n, b, b + 1, dp, ds, dr), False))
        for name, fn, packed in rnd.sample(calls, 3):
            what = f"case {it} {name}: P={P} n={n} r={r} b={b} esz={esz} hi={hi} layout={layout} shift={shift}"
            rbig.fill_(0xEE)
            assert fn() == 0, (what, dp.comm.error())
            assert dp.verify(ds, dr, packed_recv=packed) == 0, what
            assert bool((rbig[:shift] == 0xEE).all()) and bool((rbig[shift + prob.recv_bytes:] == 0xEE).all()), what
        dp.comm.free()


@pytest.mark.parametrize("P", [24, 100])
def test_seeded_sweep_on_one_communicator(api, P):
    """One long-lived communicator, every call with other sizes, another function and another execution mode: buffers
    grow, the hints of the default mode go stale, the listless kernels refuse calls and the list takes over."""
    import random
    rnd = random.Random(P)
    comm = api.VirtualComm(P)
    divs = [d for d in range(1, P + 1) if P % d == 0]
    for it in range(60):
        hi = rnd.choice([0, 3, 40, 300, 2000, 9000, 30000])
        esz = rnd.choice([1, 2, 4, 8])
        counts = W.counts_uniform_random(P, hi, seed=it * 7 + P)
        if rnd.random() < 0.3:
            counts[counts % 3 == 0] = 0
        if rnd.random() < 0.15:
            counts[rnd.randrange(P), rnd.randrange(P)] = rnd.choice([60000, 250000])
        layout = rnd.choice([0, 1])
        prob = W.make_problem(counts, esz, layout, layout)
        dp = api.DeviceProblem(prob, comm=comm)
        mode = rnd.choice([0, 1, 1, 1, 1, 2, 3, 4])
        comm.set_forwarding(mode)
        ds = dp.new_send_arena()
        dp.fill_payload(0, it, ds)
        dr = dp.new_recv_arena(0xEE)
        n, r, b = rnd.choice(divs), rnd.choice([2, 3, 4, 8, 16, P]), rnd.choice([0, 1, 5])
        calls = [("twophase", lambda: api.twophase_rbruck_alltoallv(r, dp, ds, dr), False),
                 ("om", lambda: api.twophase_rbruck_alltoallv_om(r, dp, ds, dr), False),
                 ("s1", lambda: api.TTPL_BT_alltoallv_s1(n, r, b, dp, ds, dr), False),
                 ("rbruck", lambda: api.TTPL_rbruck_alltoallv(n, r, dp, ds, dr), False),
                 ("tuna", lambda: api.tuna_algorithm(r, b, dp, ds, dr), False),
                 ("spreadout", lambda: api.spreadout_alltoallv(dp, ds, dr), False)]
        if layout == 0:
            calls.append(("ttpl", lambda: api.TTPL_BT_alltoallv(n, r, b, dp, ds, dr), True))
        name, fn, packed = rnd.choice(calls)
        what = f"call {it} {name}: mode={mode} n={n} r={r} b={b} esz={esz} hi={hi} layout={layout}"
        assert fn() == 0, (what, comm.error())
        assert dp.verify(ds, dr, packed_recv=packed) == 0, what
    comm.free()


def test_default_mode_picks_the_listless_kernel_for_small_calls(api):
    """Mode 1 (the library's default): forwarded, and after a call of few short blocks the next one goes without the
    work-item list; a call with long blocks is refused by the listless kernel's own check of the plan and goes through
    the list.  Every call is exact whichever way it went."""
    if isinstance(api, CalledTwice):
        pytest.skip("this test lays out the sequence of calls itself")
    small = W.make_problem(W.counts_uniform_random(64, 4096, seed=0), 1, 0, 0)
    big_counts = W.counts_uniform_random(64, 4096, seed=1)
    big_counts[5, 9] = 200000                          # 49 pieces
    big = W.make_problem(big_counts, 1, 0, 0)
    comm = api.VirtualComm(64)
    comm.set_forwarding(1)
    seen = []
    for prob in (small, small, small, big, big, small, small):
        dp = api.DeviceProblem(prob, comm=comm)
        comm.set_forwarding(1)
        ds, dr = dp.new_send_arena(), dp.new_recv_arena()
        dp.fill_payload(0, 4, ds)
        assert api.twophase_rbruck_alltoallv(2, dp, ds, dr) == 0, comm.error()
        assert dp.verify(ds, dr) == 0
        st = comm.last_stats()
        assert st.n_launches == 1 and st.payload_bytes == prob.payload_bytes
        seen.append(st.execution)
    # 3: without the list, on fixed-stride staging sized from the call before; the 4th call was tried that way, refused on the
    # device (longer blocks than the stride holds), and redone through the list
    assert seen == [1, 3, 3, 1, 1, 1, 3]
    comm.free()
    # blocks of a few hundred bytes go without the list on any number of ranks: a quarter of a wavefront per pair, or (average
    # block below 384 bytes on more than 128 ranks) a batch of pairs per wavefront, reported as 1 lane per pair
    for top, lanes in ((900, 16), (600, 1)):
        prob = W.make_problem(W.counts_uniform_random(300, top, seed=2), 1, 0, 0)
        dp = api.DeviceProblem(prob)
        dp.comm.set_forwarding(1)
        ds, dr = dp.new_send_arena(), dp.new_recv_arena()
        dp.fill_payload(0, 5, ds)
        seen = []
        for _ in range(3):
            assert api.TTPL_BT_alltoallv_s1(10, 3, 0, dp, ds, dr) == 0 and dp.verify(ds, dr) == 0
            st = dp.comm.last_stats()
            seen.append((st.execution, st.lanes_per_item))
        assert seen[0][0] == 1 and seen[1:] == [(2, lanes), (2, lanes)], (top, seen)      # (fixed-stride staging only on at most 128 ranks)
        dp.comm.free()


@pytest.mark.parametrize("hi,lanes", [(200, 16), (3000, 64), (12000, 256)])
def test_three_shapes_of_the_copy_kernel(api, hi, lanes):
    """The copy kernels give a work item a quarter of a wavefront, a wavefront or a workgroup, by the average piece of
    the list; the listless kernel always a workgroup."""
    counts = W.counts_uniform_random(96, hi, seed=hi)
    counts[3, 7] = 40000                                   # one long block among them, cut into pieces
    prob = W.make_problem(counts, 1, 1, 1)
    dp = api.DeviceProblem(prob)
    ds = dp.new_send_arena()
    dp.fill_payload(0, 12, ds)
    for name, fn, packed in (("twophase r=3", lambda d: api.twophase_rbruck_alltoallv(3, dp, ds, d), False),
                             ("s1 n=8 r=2", lambda d: api.TTPL_BT_alltoallv_s1(8, 2, 5, dp, ds, d), False),
                             ("scattered", lambda d: api.MPICH_intra_scattered(7, dp, ds, d), False)):
        dr = dp.new_recv_arena(0xEE)
        assert fn(dr) == 0, (name, dp.comm.error())
        assert dp.verify(ds, dr) == 0, name
        st = dp.comm.last_stats()
        if api.DEFAULT_FORWARDING == 1 and st.execution in (2, 3):       # the default mode went without the list: by its own rule
            assert st.lanes_per_item in (1, 16, 64, 256), (name, st.lanes_per_item)
        else:
            assert st.lanes_per_item == ({3: 256, 4: 16, 5: 1}[api.DEFAULT_FORWARDING] if st.execution == 2 else lanes), (name, st.lanes_per_item)
    dp.comm.free()


def test_phase_times(api):
    """With timing on, the statistics split the launches as the reference's phase timers do (src/rbruckv.h:13-18):
    inside the nodes and between them."""
    prob = W.make_problem(W.counts_normal(64, 300.0, 100.0, 0, 1000, 0), 1, 0, 0)
    dp = api.DeviceProblem(prob)
    ds, dr = dp.new_send_arena(), dp.new_recv_arena()
    dp.fill_payload(0, 2, ds)
    dp.comm.set_timing(True)
    for forward in (False, True):
        dp.comm.set_forwarding(forward)
        for name, fn, two_layer in (("ttpl", lambda: api.TTPL_BT_alltoallv_s1(8, 2, 0, dp, ds, dr), True),
                                    ("twophase", lambda: api.twophase_rbruck_alltoallv(4, dp, ds, dr), False)):
            assert fn() == 0
            st = dp.comm.last_stats()
            launches = sum(st.launch_ms[k] for k in range(st.n_launches))
            assert st.intra_ms > 0 and abs(st.intra_ms + st.inter_ms - launches) < 1e-3 * max(launches, 1e-3), name
            assert (st.inter_ms > 0) == (two_layer and not forward), name
            assert st.total_ms >= launches and st.plan_ms > 0, name
    dp.comm.set_timing(False)
    assert api.twophase_rbruck_alltoallv(4, dp, ds, dr) == 0
    st = dp.comm.last_stats()
    assert st.total_ms == 0 and st.intra_ms == 0 and st.inter_ms == 0
    dp.comm.free()


def test_both_execution_modes_leave_the_same_staging(api):
    """The route on the GPU, forwarded execution included: after a call the staging arena holds every block in every
    slot it waited in on the way, byte for byte what the launch-per-digit execution (whose launches are pinned against
    the oracle's message trace) leaves there; bytes between the slots are not touched by either."""
    import torch
    c4 = W.counts_normal(256, 300.0, 120.0, 0, 1500, 0)
    c3 = W.counts_zipf(60, 9000, 1.2, 5, 0)
    for prob, calls in (
            (W.make_problem(c4, 1, 0, 0), [("s1 r=2", lambda dp, s, d: api.TTPL_BT_alltoallv_s1(16, 2, 0, dp, s, d)),
                                          ("s1 r=16", lambda dp, s, d: api.TTPL_BT_alltoallv_s1(16, 16, 0, dp, s, d)),
                                          ("ttpl_rbruck r=3", lambda dp, s, d: api.TTPL_rbruck_alltoallv(16, 3, dp, s, d)),
                                          ("om r=4", lambda dp, s, d: api.twophase_rbruck_alltoallv_om(4, dp, s, d))]),
            (W.make_problem(c3, 4, 1, 1), [("twophase r=2", lambda dp, s, d: api.twophase_rbruck_alltoallv(2, dp, s, d)),
                                          ("twophase r=7", lambda dp, s, d: api.twophase_rbruck_alltoallv(7, dp, s, d)),
                                          ("tuna r=3", lambda dp, s, d: api.tuna_algorithm(3, 2, dp, s, d))])):
        dp = api.DeviceProblem(prob)
        dp.comm.set_staging_bound(False)             # every digit phase its own region: the layout all four modes share
        ds = dp.new_send_arena()
        dp.fill_payload(0, 11, ds)
        lib, h = dp.comm.lib, dp.comm.handle
        for name, fn in calls:
            print("  ", name, flush=True)
            snaps, sizes = [], []
            for mode in (0, 2, 3, 4, 5):
                dp.comm.set_forwarding(mode)
                dr = dp.new_recv_arena(0xEE)
                assert fn(dp, ds, dr) == 0, (name, dp.comm.error())          # sizes the arena
                ptr, size = dp.comm.staging()
                n = (size + 15) // 16 * 16
                assert size > 0 and ptr
                pattern = torch.full((n,), 0xAB, dtype=torch.uint8, device="cuda:0")
                assert lib.vc_calibration_copy(ptr, pattern.data_ptr(), n, h) == 0
                assert fn(dp, ds, dr) == 0 and dp.verify(ds, dr) == 0
                assert dp.comm.staging() == (ptr, size)
                snap = torch.empty(n, dtype=torch.uint8, device="cuda:0")
                assert lib.vc_calibration_copy(snap.data_ptr(), ptr, n, h) == 0
                assert dp.comm.last_stats().execution == {0: 0, 2: 1, 3: 2, 4: 2, 5: 2}[mode]
                snaps.append(snap.cpu().numpy())
                sizes.append(size)
            assert sizes[0] == sizes[1] == sizes[2] == sizes[3], name
            assert all(np.array_equal(snaps[0], other) for other in snaps[1:]), name
            assert np.count_nonzero(snaps[0] != 0xAB) > sizes[0] // 4, name        # the slots were written
            # with the staging bound on (the default), launch-per-digit execution reuses staging memory: never more, and
            # the same result
            dp.comm.set_staging_bound(2)             # (an allowance of 2 MiB: calls as small as these are planned for reuse)
            dp.comm.set_forwarding(0)
            dr = dp.new_recv_arena(0xEE)
            assert fn(dp, ds, dr) == 0 and dp.verify(ds, dr) == 0, name
            assert dp.comm.last_stats().staging_bytes <= sizes[0], name
            if name == "twophase r=2":               # (two-layer calls keep most staged blocks until the inter-node phase)
                assert dp.comm.last_stats().staging_bytes < 0.85 * sizes[0], name
            dp.comm.set_staging_bound(False)
        dp.comm.free()


def test_forwarded_shapes_plans_and_graphs(api):
    """Forwarded execution on the benchmark shapes (reduced), unaligned arenas, as a persistent plan and inside a HIP graph."""
    import torch
    c4 = W.counts_normal(1024, 256.0, 64.0, 0, 1024, 0)
    c3 = W.counts_zipf(256, 4096, 1.2, 5, 0)
    c5 = W.counts_fft_rows(512, 32, 4096)
    for prob, calls in (
            (W.make_problem(c4, 1, 0, 0), [("ttpl", lambda dp, s, d: api.TTPL_BT_alltoallv(32, 32, 0, dp, s, d), True),
                                          ("s1 r=2", lambda dp, s, d: api.TTPL_BT_alltoallv_s1(32, 2, 7, dp, s, d), False),
                                          ("ttpl_rbruck r=4", lambda dp, s, d: api.TTPL_rbruck_alltoallv(32, 4, dp, s, d), False),
                                          ("twophase r=2", lambda dp, s, d: api.twophase_rbruck_alltoallv(2, dp, s, d), False)]),
            (W.make_problem(c3, 4, 1, 1), [("twophase r=16", lambda dp, s, d: api.twophase_rbruck_alltoallv(16, dp, s, d), False),
                                          ("tuna r=3 b=1", lambda dp, s, d: api.tuna_algorithm(3, 1, dp, s, d), False)]),
            (W.make_problem(c5, 8, 0, 0), [("tuna r=32", lambda dp, s, d: api.tuna_algorithm(32, 0, dp, s, d), False),
                                          ("spreadout", lambda dp, s, d: api.spreadout_alltoallv(dp, s, d), False)])):
        dp = api.DeviceProblem(prob)
        dp.comm.set_forwarding(api.DEFAULT_FORWARDING or 2)
        dp.comm.set_staging_bound(False)             # (the radix-4 two-layer Bruck on 256-byte blocks stages 4 x its payload)
        ds = dp.new_send_arena()
        dp.fill_payload(0, 3, ds)
        for name, fn, packed in calls:
            print("  ", name, flush=True)
            dr = dp.new_recv_arena(0xEE)
            assert fn(dp, ds, dr) == 0, (name, dp.comm.error())
            assert dp.verify(ds, dr, packed_recv=packed) == 0, name
            assert dp.comm.last_stats().n_launches == 1
        dp.comm.free()
    # unaligned arenas, a plan, a graph
    counts = (W.counts_uniform_random(12, 30000, seed=5) * (W.counts_uniform_random(12, 3, seed=6) > 0)).astype(np.int32)
    prob = W.make_problem(counts, 1, 1, 0)
    send = W.fill_send_arena(prob, 0, 9)
    want = W.expected_recv_arena(prob, send)
    dp = api.DeviceProblem(prob)
    dp.comm.set_forwarding(api.DEFAULT_FORWARDING or 2)
    sbig = torch.zeros(prob.send_bytes + 64, dtype=torch.uint8, device="cuda:0")
    ds = sbig[5:5 + prob.send_bytes]
    ds.copy_(torch.from_numpy(send))
    rbig = torch.full((prob.recv_bytes + 256,), 0xEE, dtype=torch.uint8, device="cuda:0")
    dr = rbig[77:77 + prob.recv_bytes]
    assert api.twophase_rbruck_alltoallv(3, dp, ds, dr) == 0, dp.comm.error()
    assert np.array_equal(dr.cpu().numpy(), want)
    assert bool((rbig[:77] == 0xEE).all()) and bool((rbig[77 + prob.recv_bytes:] == 0xEE).all())
    plan = api.Plan("tuna_algorithm", dp, dr, r=2, batch=0)
    assert plan.rc == 0, dp.comm.error()
    for _ in range(3):
        dr.fill_(0xEE)
        assert plan.execute(ds, dr) == 0, dp.comm.error()
        assert np.array_equal(dr.cpu().numpy(), want)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        dp.comm.use_current_stream()
        assert plan.execute_async(ds, dr) == 0, dp.comm.error()
    dp.comm.use_current_stream()
    for _ in range(3):
        dr.fill_(0xEE)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert np.array_equal(dr.cpu().numpy(), want)
    plan.free()
    dp.comm.free()
