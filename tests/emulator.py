"""Loads tests/plan_emulator.cpp (CPU build of the library's schedule + plan arithmetic) and exposes the
reference's function names on numpy arenas, like oracle.oracle_py does for the oracle."""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "plan_emulator.cpp")
LIB = os.path.join(HERE, "_build", "libplan_emulator.so")
CSRC = os.path.join(os.path.dirname(HERE), "rbruck_alltoallv_amd", "csrc")

F_TWOPHASE, F_OM, F_TUNA, F_TTPL, F_TTPL_S1, F_UNIFORM_SPREADOUT, F_UNIFORM_ISPLIT, F_SPREADOUT, F_MPICH_SCATTERED, \
    F_OMPI_LINEAR, F_OMPI_PAIRWISE, F_XOR, F_TUNA2, F_TWOLAYER_LINEAR, F_TWOLAYER_LINEAR_S2, F_TTPL_RBRUCK = range(16)
MAX_LAUNCHES = 64


def build() -> str:
    deps = [SRC] + [os.path.join(CSRC, f) for f in ("vc_plan_math.h", "vc_sched.h", "vc_common.h", "vc_dispatch.h", "vc_scan.h")]
    if not os.path.exists(LIB) or os.path.getmtime(LIB) < max(os.path.getmtime(d) for d in deps):
        os.makedirs(os.path.dirname(LIB), exist_ok=True)
        tmp = f"{LIB}.{os.getpid()}.tmp"                      # parallel test workers may build at the same time
        subprocess.run(["/opt/rocm/bin/hipcc", "-O1", "-g", "-std=c++17", "-fPIC", "-shared", "-o", tmp, SRC],
                       check=True, capture_output=True)
        os.replace(tmp, LIB)
    return LIB


_lib = None


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


class Result:
    def __init__(self, rc, stats, traffic):
        self.rc, self.nlaunch, self.stage_bytes, self.moved, self.errors = rc, int(stats[0]), int(stats[1]), int(stats[2]), int(stats[3])
        self.items = int(stats[4])
        self.traffic = traffic[: self.nlaunch] if rc == 0 else None


def emulate(func, prob, send, recv, n=0, r=2, batch=0, uniform_count=0, recv_lo=0, batch2=0, forward=None, stride=0, recycle=None) -> Result:
    global _lib
    if _lib is None:
        _lib = C.CDLL(build())
    P = prob.P
    stats = np.zeros(5, dtype=np.int64)
    traffic = np.zeros((MAX_LAUNCHES, P, P), dtype=np.int64)
    rc = _lib.plan_emulate(C.c_int(func), C.c_int(P), C.c_int(n), C.c_int(r), C.c_int(batch), C.c_int(prob.esz),
                           C.c_int(uniform_count), _p(send), C.c_int64(send.size), _p(recv), C.c_int64(recv.size),
                           _p(prob.sbase), _p(prob.rbase), _p(prob.sendcounts), _p(prob.sdispls), _p(prob.recvcounts),
                           _p(prob.rdispls), C.c_int(recv_lo), _p(stats), _p(traffic), C.c_int(MAX_LAUNCHES), C.c_int(batch2),
                           C.c_int(int(FORWARD if forward is None else forward)), C.c_int(stride),
                           C.c_int(int(RECYCLE if recycle is None else recycle)))
    return Result(rc, stats, traffic)


# the reference's names, returning the return code and remembering the last Result
last = None
# module-wide switch: emulate forwarded execution (and check it against the launch-per-digit execution)
FORWARD = False
# module-wide switch: launch-per-digit execution reuses staging memory where the library would (its default)
RECYCLE = True
# module-wide switch: fixed-stride staging, every slot as long as the call's longest block at any cache-line phase
STRIDED = False


def stride_for(prob, uniform_count=0) -> int:
    longest = (uniform_count if uniform_count else int(prob.sendcounts.max(initial=0))) * prob.esz
    return (longest + 255) // 128 * 128


def _run(func, prob, *a, **k):
    global last
    if STRIDED:
        k["stride"] = stride_for(prob, k.get("uniform_count", 0))
    last = emulate(func, prob, *a, **k)
    if last.rc == 0 and last.errors:
        return 1000 + last.errors
    return last.rc


def twophase_rbruck_alltoallv(r, prob, send, recv):
    return _run(F_TWOPHASE, prob, send, recv, r=r)


def twophase_rbruck_alltoallv_om(r, prob, send, recv):
    return _run(F_OM, prob, send, recv, r=r)


def tuna_algorithm(r, b, prob, send, recv):
    return _run(F_TUNA, prob, send, recv, r=r, batch=b)


def TTPL_BT_alltoallv(n, r, bblock, prob, send, recv):
    return _run(F_TTPL, prob, send, recv, n=n, r=r, batch=bblock)


def TTPL_BT_alltoallv_s1(n, r, bblock, prob, send, recv):
    return _run(F_TTPL_S1, prob, send, recv, n=n, r=r, batch=bblock)


def TTPL_rbruck_alltoallv(n, r, prob, send, recv):
    return _run(F_TTPL_RBRUCK, prob, send, recv, n=n, r=r)


def uniform_spreadout_twolayer(n, r, prob, count, send, recv):
    return _run(F_UNIFORM_SPREADOUT, prob, send, recv, n=n, r=r, uniform_count=count)


def uniform_inverse_isplit_r_bruck(n, r1, r2, prob, count, send, recv):
    return _run(F_UNIFORM_ISPLIT, prob, send, recv, n=n, r=r1, uniform_count=count)


def MPICH_intra_scattered(bblock, prob, send, recv):
    return _run(F_MPICH_SCATTERED, prob, send, recv, batch=bblock)


def ompi_alltoallv_intra_basic_linear(prob, send, recv):
    return _run(F_OMPI_LINEAR, prob, send, recv)


def ompi_alltoallv_intra_pairwise(prob, send, recv):
    return _run(F_OMPI_PAIRWISE, prob, send, recv)


def exclisive_or_alltoallv(prob, send, recv):
    return _run(F_XOR, prob, send, recv)


def spreadout_alltoallv(prob, send, recv):
    return _run(F_SPREADOUT, prob, send, recv)


def tuna2_algorithm(r, b, prob, send, recv):
    return _run(F_TUNA2, prob, send, recv, r=r, batch=b)


def twolayer_communicator_linear(n, prob, send, recv):
    return _run(F_TWOLAYER_LINEAR, prob, send, recv, n=n)


def twolayer_communicator_linear_s2(n, bblock1, bblock2, prob, send, recv):
    return _run(F_TWOLAYER_LINEAR_S2, prob, send, recv, n=n, batch=bblock1, batch2=bblock2)


def dispatch(func, P, hint, mode=1, call_kind=0, n=0, r=2):
    """csrc/vc_dispatch.h on the CPU: hint = (valid, block pieces, payload bytes, most pieces of a block, longest block).
    Returns dict(lanes, stride, stride_lanes, max_pieces, max_items, max_average, max_len)."""
    global _lib
    if _lib is None:
        _lib = C.CDLL(build())
    out = np.zeros(7, dtype=np.int64)
    valid, items, payload, max_pieces, max_len = hint
    rc = _lib.dispatch_decision(C.c_int(func), C.c_int(P), C.c_int(n), C.c_int(r), C.c_int(mode), C.c_int(call_kind), C.c_int(int(valid)),
                                C.c_int64(items), C.c_int64(payload), C.c_int64(max_pieces), C.c_int64(max_len), _p(out))
    assert rc == 0, rc
    return dict(zip(("lanes", "stride", "stride_lanes", "max_pieces", "max_items", "max_average", "max_len"), (int(v) for v in out)))


def lanes_for_items(nbytes, items):
    global _lib
    if _lib is None:
        _lib = C.CDLL(build())
    return _lib.lanes_for_items(C.c_int64(nbytes), C.c_int64(items))


def division_mismatches(d_lo, d_hi, samples=64):
    """Numerators below 2^31 for which vc_div / vc_mod (csrc/vc_common.h) differ from the hardware division, over the divisors
    d_lo .. d_hi."""
    global _lib
    if _lib is None:
        _lib = C.CDLL(build())
    _lib.division_mismatches.restype = C.c_int64
    return int(_lib.division_mismatches(C.c_int(d_lo), C.c_int(d_hi), C.c_int(samples)))
