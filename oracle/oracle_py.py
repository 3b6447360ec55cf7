"""ctypes binding of the CPU oracle (oracle/bruck_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the
benchmark's cpu_baseline leg as the checker / reported baseline — never by the product
package, whose only compute path is the HIP library.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libbruck_oracle.so")
REF_DRIVER = os.path.join(_HERE, "_ref", "ref_driver")
MPIEXEC = "/opt/conda/bin/mpiexec"


class TraceRec(C.Structure):
    _fields_ = [("kind", C.c_int32), ("digit", C.c_int32), ("z", C.c_int32), ("src", C.c_int32),
                ("dst", C.c_int32), ("nblocks", C.c_int32), ("bytes", C.c_int64)]


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (seconds)."""
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "bruck_oracle.c")):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s", "all"], check=True, capture_output=True)
    return _LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        _lib = C.CDLL(build())
        _lib.ora_trace_count.restype = C.c_int64
        _lib.ora_trace_data.restype = C.POINTER(TraceRec)
    return _lib


def _p(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def _v_args(prob, send, recv):
    assert send.dtype == np.uint8 and recv.dtype == np.uint8 and send.flags.c_contiguous and recv.flags.c_contiguous
    return (_p(send), _p(prob.sbase), _p(prob.sendcounts), _p(prob.sdispls), C.c_int(prob.esz),
            _p(recv), _p(prob.rbase), _p(prob.recvcounts), _p(prob.rdispls), C.c_int(prob.P))


def twophase_rbruck_alltoallv(r, prob, send, recv):
    return lib().ora_twophase_rbruck_alltoallv(C.c_int(r), *_v_args(prob, send, recv))


def twophase_rbruck_alltoallv_om(r, prob, send, recv):
    return lib().ora_twophase_rbruck_alltoallv_om(C.c_int(r), *_v_args(prob, send, recv))


def tuna_algorithm(r, b, prob, send, recv):
    return lib().ora_tuna_algorithm(C.c_int(r), C.c_int(b), *_v_args(prob, send, recv))


def tuna2_algorithm(r, b, prob, send, recv):
    return lib().ora_tuna2_algorithm(C.c_int(r), C.c_int(b), *_v_args(prob, send, recv))


def TTPL_BT_alltoallv(n, r, bblock, prob, send, recv):
    return lib().ora_TTPL_BT_alltoallv(C.c_int(n), C.c_int(r), C.c_int(bblock), *_v_args(prob, send, recv))


def TTPL_BT_alltoallv_s1(n, r, bblock, prob, send, recv):
    return lib().ora_TTPL_BT_alltoallv_s1(C.c_int(n), C.c_int(r), C.c_int(bblock), *_v_args(prob, send, recv))


def TTPL_rbruck_alltoallv(n, r, prob, send, recv):
    return lib().ora_TTPL_rbruck_alltoallv(C.c_int(n), C.c_int(r), *_v_args(prob, send, recv))


def uniform_spreadout_twolayer(n, r, prob, count, send, recv):
    """`send` is used as scratch, as in the reference."""
    return lib().ora_uniform_spreadout_twolayer(C.c_int(n), C.c_int(r), _p(send), _p(prob.sbase), C.c_int(count),
                                                C.c_int(prob.esz), _p(recv), _p(prob.rbase), C.c_int(prob.P))


def uniform_inverse_isplit_r_bruck(n, r1, r2, prob, count, send, recv):
    return lib().ora_uniform_inverse_isplit_r_bruck(C.c_int(n), C.c_int(r1), C.c_int(r2), _p(send), _p(prob.sbase),
                                                    C.c_int(count), C.c_int(prob.esz), _p(recv), _p(prob.rbase),
                                                    C.c_int(prob.P))


def MPICH_intra_scattered(bblock, prob, send, recv):
    return lib().ora_MPICH_intra_scattered(C.c_int(bblock), *_v_args(prob, send, recv))


def ompi_alltoallv_intra_basic_linear(prob, send, recv):
    return lib().ora_ompi_alltoallv_intra_basic_linear(*_v_args(prob, send, recv))


def ompi_alltoallv_intra_pairwise(prob, send, recv):
    return lib().ora_ompi_alltoallv_intra_pairwise(*_v_args(prob, send, recv))


def exclisive_or_alltoallv(prob, send, recv):
    return lib().ora_exclisive_or_alltoallv(*_v_args(prob, send, recv))


def spreadout_alltoallv(prob, send, recv):
    return lib().ora_spreadout_alltoallv(*_v_args(prob, send, recv))


def twolayer_communicator_linear(n, prob, send, recv):
    return lib().ora_twolayer_communicator_linear(C.c_int(n), *_v_args(prob, send, recv))


def twolayer_communicator_linear_s2(n, bblock1, bblock2, prob, send, recv):
    return lib().ora_twolayer_communicator_linear_s2(C.c_int(n), C.c_int(bblock1), C.c_int(bblock2), *_v_args(prob, send, recv))


def fill_payload(mode, seed, prob, send):
    lib().ora_fill_payload(C.c_int(mode), C.c_uint64(seed), _p(send), _p(prob.sbase), _p(prob.sendcounts),
                           _p(prob.sdispls), C.c_int(prob.esz), C.c_int(prob.P))


def digest_recv(prob, recv) -> np.ndarray:
    out = np.zeros(prob.P, dtype=np.uint64)
    lib().ora_digest_recv(_p(recv), _p(prob.rbase), _p(prob.recvcounts), _p(prob.rdispls), C.c_int(prob.esz),
                          C.c_int(prob.P), _p(out))
    return out


def radix_params_float(P, r):
    w, nl, d = C.c_int(), C.c_int(), C.c_int()
    lib().ora_radix_params_float(C.c_int(P), C.c_int(r), C.byref(w), C.byref(nl), C.byref(d))
    return w.value, nl.value, d.value


def radix_params_int(P, r):
    w, nl, d, k = C.c_int(), C.c_int(), C.c_int(), C.c_int()
    lib().ora_radix_params_int(C.c_int(P), C.c_int(r), C.byref(w), C.byref(nl), C.byref(d), C.byref(k))
    return w.value, nl.value, d.value, k.value


class trace:
    """with trace() as t: <oracle call>; t.records -> structured numpy array of the simulated messages."""

    def __enter__(self):
        lib().ora_trace_begin()
        return self

    def __exit__(self, *exc):
        n = lib().ora_trace_count()
        lib().ora_trace_end()
        dt = np.dtype([("kind", "<i4"), ("digit", "<i4"), ("z", "<i4"), ("src", "<i4"), ("dst", "<i4"),
                       ("nblocks", "<i4"), ("bytes", "<i8")])
        if n:
            buf = C.string_at(lib().ora_trace_data(), n * C.sizeof(TraceRec))
            self.records = np.frombuffer(buf, dtype=dt).copy()
        else:
            self.records = np.zeros(0, dtype=dt)
        return False
