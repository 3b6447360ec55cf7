"""Host-side mirror of the reference's function interface (src/rbruckv.h) over the C ABI.

Same names, same argument meaning, same return codes as the reference functions; one call
serves all P virtual ranks.  PyTorch is used only to own device memory and to hand out
pointers and the current stream; all work happens in librbruck_vc.so.
"""
from __future__ import annotations

import ctypes as C

import numpy as np
import torch

from . import _lib
from .workloads import Problem


class VcError(RuntimeError):
    pass


class VirtualComm:
    """vc_comm_t: the stand-in for MPI_Comm — P virtual ranks on one GPU."""

    def __init__(self, nranks: int, device: str = "cuda:0"):
        self.lib = _lib.load()
        self.device = torch.device(device)
        torch.cuda.set_device(self.device)
        h = C.c_void_p()
        rc = self.lib.vc_comm_create(nranks, C.byref(h))
        if rc != 0:
            raise VcError(f"vc_comm_create: {rc} {self.lib.vc_last_error_string().decode()}")
        self.handle = h
        self.P = nranks
        self._keep = []
        self.lib.vc_comm_set_stream(self.handle, C.c_void_p(torch.cuda.current_stream(self.device).cuda_stream))

    def set_bases(self, sbase: torch.Tensor, rbase: torch.Tensor) -> None:
        assert sbase.dtype == torch.int64 and rbase.dtype == torch.int64 and sbase.is_cuda and rbase.is_cuda
        self._keep = [sbase, rbase]
        self._check(self.lib.vc_comm_set_bases(self.handle, sbase.data_ptr(), rbase.data_ptr()))

    def use_current_stream(self) -> None:
        """Launch on whatever stream torch has current now (e.g. the capture stream of torch.cuda.graph)."""
        self._check(self.lib.vc_comm_set_stream(self.handle, C.c_void_p(torch.cuda.current_stream(self.device).cuda_stream)))

    def set_timing(self, on: bool) -> None:
        self._check(self.lib.vc_comm_set_timing(self.handle, int(on)))

    def set_forwarding(self, enable: bool | int) -> None:
        """vc_comm_set_forwarding: 0 / False one launch per digit phase; 1 / True forwarded (one launch per call, every
        block piece carried through all its hops in registers; the library picks list or listless); 2 forwarded through
        a work-item list; 3 / 4 / 5 forwarded without one, a workgroup / a quarter of a wavefront per pair of ranks / a
        batch of pairs per wavefront."""
        self._check(self.lib.vc_comm_set_forwarding(self.handle, int(enable)))

    def set_staging_bound(self, on: bool | int) -> None:
        """vc_comm_set_staging_bound: reuse staging memory in launch-per-digit execution and run forwarded calls that would
        need more than three times their payload (and an eighth of the device's memory; an int > 1: that many MiB) that
        way (default), or give every digit phase its own region."""
        self._check(self.lib.vc_comm_set_staging_bound(self.handle, int(on)))

    def last_stats(self) -> _lib.VcStats:
        s = _lib.VcStats()
        self._check(self.lib.vc_comm_last_stats(self.handle, C.byref(s)))
        return s

    def last_traffic(self, launch: int) -> np.ndarray:
        m = np.zeros((self.P, self.P), dtype=np.int64)
        self._check(self.lib.vc_comm_last_traffic(self.handle, launch, m.ctypes.data_as(C.c_void_p)))
        return m

    def staging(self) -> tuple[int, int]:
        """(device address, bytes used by the last call) of the staging arena."""
        ptr, size = C.c_void_p(), C.c_int64()
        self._check(self.lib.vc_comm_staging(self.handle, C.byref(ptr), C.byref(size)))
        return ptr.value or 0, size.value

    def wait(self) -> int:
        """vc_comm_wait: completes the call an _async entry point enqueued; returns its code."""
        return self.lib.vc_comm_wait(self.handle)

    def error(self) -> str:
        return self.lib.vc_last_error_string().decode()

    def _check(self, rc: int) -> None:
        if rc != 0:
            raise VcError(f"librbruck_vc returned {rc}: {self.error()}")

    def free(self) -> None:
        if self.handle:
            self.lib.vc_comm_free(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


# None: the library's default execution mode (forwarded); True / False: every new DeviceProblem sets this mode on its
# communicator (the tests run both)
DEFAULT_FORWARDING = None


class DeviceProblem:
    """Rank-major tables and arena bases of a Problem, resident in HBM, plus its communicator."""

    def __init__(self, prob: Problem, device: str = "cuda:0", comm: VirtualComm | None = None):
        self.host = prob
        self.P, self.esz = prob.P, prob.esz
        dev = torch.device(device)
        self.sendcounts = torch.from_numpy(prob.sendcounts).to(dev)
        self.sdispls = torch.from_numpy(prob.sdispls).to(dev)
        self.recvcounts = torch.from_numpy(prob.recvcounts).to(dev)
        self.rdispls = torch.from_numpy(prob.rdispls).to(dev)
        self.sbase = torch.from_numpy(prob.sbase).to(dev)
        self.rbase = torch.from_numpy(prob.rbase).to(dev)
        self.comm = comm or VirtualComm(prob.P, device)
        self.comm.set_bases(self.sbase, self.rbase)
        if DEFAULT_FORWARDING is not None:
            self.comm.set_forwarding(DEFAULT_FORWARDING)

    def new_send_arena(self) -> torch.Tensor:
        return torch.zeros(self.host.send_bytes, dtype=torch.uint8, device=self.sbase.device)

    def new_recv_arena(self, fill: int = 0xEE) -> torch.Tensor:
        return torch.full((self.host.recv_bytes,), fill, dtype=torch.uint8, device=self.sbase.device)

    def fill_payload(self, mode: int, seed: int, send: torch.Tensor) -> None:
        c = self.comm
        c._check(c.lib.vc_fill_payload(mode, seed, send.data_ptr(), self.sendcounts.data_ptr(), self.sdispls.data_ptr(),
                                       self.esz, c.handle))

    def verify(self, send: torch.Tensor, recv: torch.Tensor, packed_recv: bool = False) -> int:
        c = self.comm
        bad = C.c_int64(-1)
        c._check(c.lib.vc_verify_alltoallv(send.data_ptr(), self.sendcounts.data_ptr(), self.sdispls.data_ptr(), self.esz,
                                           recv.data_ptr(), self.recvcounts.data_ptr(), self.rdispls.data_ptr(),
                                           int(packed_recv), C.byref(bad), c.handle))
        return bad.value


def _tail(p: DeviceProblem, send: torch.Tensor, recv: torch.Tensor):
    return (send.data_ptr(), p.sendcounts.data_ptr(), p.sdispls.data_ptr(), p.esz, recv.data_ptr(),
            p.recvcounts.data_ptr(), p.rdispls.data_ptr(), p.esz, p.comm.handle)


def twophase_rbruck_alltoallv(r: int, p: DeviceProblem, send: torch.Tensor, recv: torch.Tensor) -> int:
    """src/twophase_tunable_rbruckv.cpp:13-152"""
    return p.comm.lib.twophase_rbruck_alltoallv(r, *_tail(p, send, recv))


def twophase_rbruck_alltoallv_noalloc(r: int, p: DeviceProblem, send: torch.Tensor, recv: torch.Tensor) -> int:
    """twophase_rbruck_alltoallv out of the library's static device scratch array: allocates nothing."""
    return p.comm.lib.twophase_rbruck_alltoallv_noalloc(r, *_tail(p, send, recv))


def twophase_rbruck_alltoallv_om(r: int, p: DeviceProblem, send: torch.Tensor, recv: torch.Tensor) -> int:
    """src/twophase_tunable_rbruckv-om.cpp:10-157"""
    return p.comm.lib.twophase_rbruck_alltoallv_om(r, *_tail(p, send, recv))


def tuna_algorithm(r: int, b: int, p: DeviceProblem, send: torch.Tensor, recv: torch.Tensor) -> int:
    """src/tuna.cpp:10-177"""
    return p.comm.lib.tuna_algorithm(r, b, *_tail(p, send, recv))


def tuna2_algorithm(r: int, b: int, p: DeviceProblem, send: torch.Tensor, recv: torch.Tensor) -> int:
    """src/tuna2.cpp:10-239"""
    return p.comm.lib.tuna2_algorithm(r, b, *_tail(p, send, recv))


def TTPL_BT_alltoallv(n: int, r: int, bblock: int, p: DeviceProblem, send: torch.Tensor, recv: torch.Tensor) -> int:
    """src/twophase_twolayer_rbruck.cpp:237-463"""
    return p.comm.lib.TTPL_BT_alltoallv(n, r, bblock, *_tail(p, send, recv))


def TTPL_BT_alltoallv_s1(n: int, r: int, bblock: int, p: DeviceProblem, send: torch.Tensor, recv: torch.Tensor) -> int:
    """src/twophase_twolayer_rbruck.cpp:467-681"""
    return p.comm.lib.TTPL_BT_alltoallv_s1(n, r, bblock, *_tail(p, send, recv))


def TTPL_rbruck_alltoallv(n: int, r: int, p: DeviceProblem, send: torch.Tensor, recv: torch.Tensor) -> int:
    """src/twophase_twolayer_rbruck.cpp:15-235, with the inter-node Bruck completed"""
    return p.comm.lib.TTPL_rbruck_alltoallv(n, r, *_tail(p, send, recv))


def uniform_spreadout_twolayer(n: int, r: int, p: DeviceProblem, count: int, send: torch.Tensor, recv: torch.Tensor) -> int:
    """src/twolayer_rbruck.cpp:10-134"""
    return p.comm.lib.uniform_spreadout_twolayer(n, r, send.data_ptr(), count, p.esz, recv.data_ptr(), count, p.esz, p.comm.handle)


def uniform_inverse_isplit_r_bruck(n: int, r1: int, r2: int, p: DeviceProblem, count: int, send: torch.Tensor,
                                   recv: torch.Tensor) -> int:
    """src/twolayer_rbruck.cpp:137-277"""
    return p.comm.lib.uniform_inverse_isplit_r_bruck(n, r1, r2, send.data_ptr(), count, p.esz, recv.data_ptr(), count,
                                                     p.esz, p.comm.handle)


def MPICH_intra_scattered(bblock: int, p: DeviceProblem, send: torch.Tensor, recv: torch.Tensor) -> int:
    """src/MPICH_scattered.cpp:11-76"""
    return p.comm.lib.MPICH_intra_scattered(bblock, *_tail(p, send, recv))


def ompi_alltoallv_intra_basic_linear(p: DeviceProblem, send: torch.Tensor, recv: torch.Tensor) -> int:
    """src/OpenMPI_basic_linear.cpp:10-77"""
    return p.comm.lib.ompi_alltoallv_intra_basic_linear(*_tail(p, send, recv))


def ompi_alltoallv_intra_pairwise(p: DeviceProblem, send: torch.Tensor, recv: torch.Tensor) -> int:
    """src/OpenMPI_pairwise.cpp:14-64"""
    return p.comm.lib.ompi_alltoallv_intra_pairwise(*_tail(p, send, recv))


def exclisive_or_alltoallv(p: DeviceProblem, send: torch.Tensor, recv: torch.Tensor) -> int:
    """src/exclusive_or_alltoallv.cpp:12-51"""
    return p.comm.lib.exclisive_or_alltoallv(*_tail(p, send, recv))


def spreadout_alltoallv(p: DeviceProblem, send: torch.Tensor, recv: torch.Tensor) -> int:
    """benchmarks/common.cpp:10-37"""
    return p.comm.lib.spreadout_alltoallv(*_tail(p, send, recv))


def call_async(name: str, tunables: tuple, p: DeviceProblem, send: torch.Tensor, recv: torch.Tensor, stream: torch.cuda.Stream) -> int:
    """The _async twin of the alltoallv-shaped entry point `name` (e.g. "tuna_algorithm" with tunables (r, b)): enqueues on
    `stream` and returns; VirtualComm.wait() completes the call."""
    return getattr(p.comm.lib, name + "_async")(*tunables, *_tail(p, send, recv), C.c_void_p(stream.cuda_stream))


def uniform_async(name: str, tunables: tuple, p: DeviceProblem, count: int, send: torch.Tensor, recv: torch.Tensor,
                  stream: torch.cuda.Stream) -> int:
    """The _async twin of uniform_spreadout_twolayer (tunables (n, r)) or uniform_inverse_isplit_r_bruck ((n, r1, r2))."""
    return getattr(p.comm.lib, name + "_async")(*tunables, send.data_ptr(), count, p.esz, recv.data_ptr(), count, p.esz, p.comm.handle,
                                                C.c_void_p(stream.cuda_stream))


class Plan:
    """vc_plan_t: a planned (persistent) collective for one set of tables."""

    def __init__(self, function: str, p: DeviceProblem, recv: torch.Tensor, n: int = 0, r: int = 2, batch: int = 0):
        """For the uniform_* functions `batch` is the block length in elements and the tables are implied."""
        self.problem = p
        h = C.c_void_p()
        tables = [None] * 4 if function.startswith("uniform_") else [t.data_ptr() for t in (p.sendcounts, p.sdispls, p.recvcounts, p.rdispls)]
        rc = p.comm.lib.vc_plan_create(function.encode(), n, r, batch, tables[0], tables[1], p.esz, tables[2], tables[3],
                                       recv.data_ptr() & 4095, p.comm.handle, C.byref(h))
        self.rc = rc
        self.handle = h if rc == 0 else None

    def execute(self, send: torch.Tensor, recv: torch.Tensor) -> int:
        return self.problem.comm.lib.vc_plan_execute(self.handle, send.data_ptr(), recv.data_ptr())

    def execute_async(self, send: torch.Tensor, recv: torch.Tensor) -> int:
        return self.problem.comm.lib.vc_plan_execute_async(self.handle, send.data_ptr(), recv.data_ptr())

    def free(self) -> None:
        if self.handle:
            self.problem.comm.lib.vc_plan_free(self.handle)
            self.handle = None


def suggest_radix(p: DeviceProblem, candidates: list[int], n: int = 0) -> tuple[int, list[int]]:
    """vc_suggest_radix: (best radix, bytes moved per candidate)."""
    cand = (C.c_int * len(candidates))(*candidates)
    moved = (C.c_int64 * len(candidates))()
    best = C.c_int(0)
    p.comm._check(p.comm.lib.vc_suggest_radix(p.sendcounts.data_ptr(), p.esz, n, cand, len(candidates), C.byref(best), moved,
                                              p.comm.handle))
    return best.value, list(moved)


def suggest_tunables(p: DeviceProblem, candidates: list[int] | None = None, n: int = 0) -> tuple[int, int, list[float]]:
    """vc_suggest_tunables: (radix, rounds per launch, modelled seconds per candidate); no candidates = search 2..min(n, 63), n."""
    ncand = len(candidates) if candidates else 0
    cand = (C.c_int * max(ncand, 1))(*(candidates or [0]))
    secs = (C.c_double * max(ncand, 1))()
    r, b = C.c_int(0), C.c_int(0)
    p.comm._check(p.comm.lib.vc_suggest_tunables(p.sendcounts.data_ptr(), p.esz, n, cand if ncand else None, ncand, C.byref(r),
                                                 C.byref(b), secs if ncand else None, None, p.comm.handle))
    return r.value, b.value, list(secs)[:ncand]


def calibration(comm: VirtualComm) -> tuple[float, float]:
    """vc_comm_calibration: (bytes per second of a plain copy, seconds per kernel launch)."""
    rate, launch = C.c_double(0), C.c_double(0)
    comm._check(comm.lib.vc_comm_calibration(comm.handle, C.byref(rate), C.byref(launch)))
    return rate.value, launch.value


def twolayer_communicator_linear(n: int, p: DeviceProblem, send: torch.Tensor, recv: torch.Tensor) -> int:
    """src/twolayer_communicator_linear.cpp:13-88"""
    return p.comm.lib.twolayer_communicator_linear(n, *_tail(p, send, recv))


def twolayer_communicator_linear_s2(n: int, bblock1: int, bblock2: int, p: DeviceProblem, send: torch.Tensor, recv: torch.Tensor) -> int:
    """src/twolayer_communicator_linear.cpp:92-192"""
    return p.comm.lib.twolayer_communicator_linear_s2(n, bblock1, bblock2, *_tail(p, send, recv))
