"""The entry point that allocates nothing (twophase_rbruck_alltoallv_noalloc), through the C ABI on a real MI355X.

Its plan tables and staging arena live in the library's static device array; its result must equal, byte for byte
(blocks and the untouched gaps between them), what twophase_rbruck_alltoallv leaves for the same inputs.  Two calls in
a row share the array, the second with a smaller input: nothing of the first call may leak into the second."""
import numpy as np
import pytest

from rbruck_alltoallv_amd import _lib
from rbruck_alltoallv_amd import workloads as W

pytestmark = pytest.mark.gpu


def _both(api, P, hi, esz, r, seed, layout=0):
    """Runs the existing entry point and the one that allocates nothing on the same inputs; returns both receive arenas."""
    import torch
    counts = W.counts_uniform_random(P, hi, seed=seed)
    counts[counts % 5 == 0] = 0
    prob = W.make_problem(counts, esz, layout, layout)
    send = W.fill_send_arena(prob, 0, seed)
    dp = api.DeviceProblem(prob)
    dp.comm.set_forwarding(2)
    dsend = torch.from_numpy(send).to("cuda:0")
    want = dp.new_recv_arena(0xEE)
    assert api.twophase_rbruck_alltoallv(r, dp, dsend, want) == 0, dp.comm.error()
    assert np.array_equal(want.cpu().numpy(), W.expected_recv_arena(prob, send))
    got = dp.new_recv_arena(0xEE)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]                 # the driver's figure: sees hipMalloc by anyone in the process
    rc = api.twophase_rbruck_alltoallv_noalloc(r, dp, dsend, got)
    assert rc == 0, dp.comm.error()
    assert torch.cuda.mem_get_info()[0] == free_before, "the call allocated or freed device memory"
    st = dp.comm.last_stats()
    assert st.execution == 2 and st.payload_bytes == prob.payload_bytes
    assert np.array_equal(dsend.cpu().numpy(), send), "sendbuf must stay intact"
    out = got.cpu().numpy(), want.cpu().numpy()
    dp.comm.free()
    return out


def test_two_calls_in_a_row_the_second_smaller():
    import torch
    assert torch.cuda.is_available(), "this test needs the GPU"
    from rbruck_alltoallv_amd import api
    print("no-alloc: P=40 blocks 0..3000 x 4 B r=3, then P=20 blocks 0..40 x 1 B r=2", flush=True)
    got, want = _both(api, 40, 3000, 4, 3, seed=11)            # several pieces per block, 4 digits, ~15 MB of staging
    assert np.array_equal(got, want)
    got, want = _both(api, 20, 40, 1, 2, seed=12, layout=1)    # short blocks, gapped reversed displacements
    assert np.array_equal(got, want)
    got, want = _both(api, 40, 3000, 4, 3, seed=11)            # and the first one once more, after the small one
    assert np.array_equal(got, want)


def test_same_communicator_twice_and_radices():
    import torch
    from rbruck_alltoallv_amd import api
    print("no-alloc: one communicator, radices 2..P, two rounds", flush=True)
    P = 33
    counts = W.counts_uniform_random(P, 700, seed=4)
    prob = W.make_problem(counts, 2, 1, 1)
    send = W.fill_send_arena(prob, 0, 9)
    want = W.expected_recv_arena(prob, send)
    dp = api.DeviceProblem(prob)
    dsend = torch.from_numpy(send).to("cuda:0")
    for _ in range(2):                                         # the second round runs on the hint of the first
        for r in (2, 3, 6, 33, 40):
            drecv = dp.new_recv_arena(0xEE)
            assert api.twophase_rbruck_alltoallv_noalloc(r, dp, dsend, drecv) == 0, dp.comm.error()
            assert np.array_equal(drecv.cpu().numpy(), want), r
    assert api.twophase_rbruck_alltoallv_noalloc(1, dp, dsend, drecv) == -1
    dp.comm.free()


def test_sizes_beyond_the_static_array_are_refused():
    import torch
    from rbruck_alltoallv_amd import api
    print("no-alloc: refusals", flush=True)
    # staging: 64 ranks, radix 2, blocks of 64 KiB: ~2/3 of 268 MB make more than one hop
    counts = np.full((64, 64), 65536, dtype=np.int32)
    prob = W.make_problem(counts, 1, 0, 0)
    dp = api.DeviceProblem(prob)
    dsend, drecv = dp.new_send_arena(), dp.new_recv_arena(0xEE)
    rc = api.twophase_rbruck_alltoallv_noalloc(2, dp, dsend, drecv)
    assert rc == _lib.VC_ERR_SCRATCH and "staging" in dp.comm.error(), (rc, dp.comm.error())
    assert bool((drecv == 0xEE).all()), "a refused call must leave recvbuf untouched"
    # the same blocks in one hop each need no staging at all
    assert api.twophase_rbruck_alltoallv_noalloc(64, dp, dsend, drecv) == 0, dp.comm.error()
    assert dp.verify(dsend, drecv) == 0
    dp.comm.free()
    # plan tables: 2048 ranks with radix 2 need 8 * P * P * 12 bytes
    c = api.VirtualComm(2048)
    z = torch.zeros(2048, dtype=torch.int64, device="cuda:0")
    c.set_bases(z, z)
    t = torch.zeros(16, dtype=torch.int32, device="cuda:0")            # never read: the call is refused before any kernel
    rc = c.lib.twophase_rbruck_alltoallv_noalloc(2, t.data_ptr(), t.data_ptr(), t.data_ptr(), 1, t.data_ptr(), t.data_ptr(),
                                                 t.data_ptr(), 1, c.handle)
    assert rc == _lib.VC_ERR_SCRATCH and "plan tables" in c.error(), (rc, c.error())
    c.free()
