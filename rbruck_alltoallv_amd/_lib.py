"""ctypes binding of librbruck_vc.so (include/rbruck_vc.h).  There is no fallback: if the
library is missing, loading fails loudly."""
from __future__ import annotations

import ctypes as C
import os

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, "librbruck_vc.so")
VC_MAX_LAUNCHES = 1024

VC_OK, VC_ERR_RADIX, VC_ERR_GROUP, VC_ERR_TOO_FEW_RANKS, VC_ERR_HIP, VC_ERR_ARG, VC_ERR_NO_DEVICE = 0, -1, -2, -3, -4, -5, -6
VC_ERR_TABLES, VC_ERR_OVERFLOW, VC_ERR_SCRATCH, VC_ERR_BUSY = -7, -8, -9, -10
VC_NOALLOC_SCRATCH_BYTES = 64 << 20


class VcStats(C.Structure):
    _fields_ = [("n_launches", C.c_int32), ("n_digits", C.c_int32), ("payload_bytes", C.c_int64),
                ("moved_bytes", C.c_int64), ("staging_bytes", C.c_int64), ("plan_ms", C.c_float),
                ("total_ms", C.c_float), ("intra_ms", C.c_float), ("inter_ms", C.c_float),
                ("launch_bytes", C.c_int64 * VC_MAX_LAUNCHES),
                ("launch_ms", C.c_float * VC_MAX_LAUNCHES), ("execution", C.c_int32), ("lanes_per_item", C.c_int32),
                ("block_pieces", C.c_int64), ("max_block_pieces", C.c_int64), ("max_block_bytes", C.c_int64),
                ("bad_table_entries", C.c_int64), ("host_waits", C.c_int64)]


# every symbol include/rbruck_vc.h declares: name -> (restype, argtypes)
_P, _I, _I64, _U64 = C.c_void_p, C.c_int, C.c_int64, C.c_uint64
_V_TAIL = [_P, _P, _P, _I, _P, _P, _P, _I, _P]      # sendbuf, sendcounts, sdispls, size, recvbuf, recvcounts, rdispls, size, comm
SYMBOLS = {
    "vc_comm_create": (_I, [_I, C.POINTER(_P)]),
    "vc_comm_free": (_I, [_P]),
    "vc_comm_size": (_I, [_P]),
    "vc_comm_set_stream": (_I, [_P, _P]),
    "vc_comm_set_forwarding": (_I, [_P, _I]),
    "vc_comm_set_bases": (_I, [_P, _P, _P]),
    "vc_comm_set_staging_bound": (_I, [_P, _I]),
    "vc_last_error_string": (C.c_char_p, []),
    "vc_alltoall_counts": (_I, [_P, _P, _P]),
    "vc_displs_from_counts": (_I, [_P, _P, _P, _P]),
    "vc_bases_from_extents": (_I, [_P, _I, _I64, _P, _P, _P]),
    "vc_allreduce_max_count": (_I, [_P, _P, _P]),
    "twophase_rbruck_alltoallv": (_I, [_I] + _V_TAIL),
    "twophase_rbruck_alltoallv_om": (_I, [_I] + _V_TAIL),
    "twophase_rbruck_alltoallv_noalloc": (_I, [_I] + _V_TAIL),
    "tuna_algorithm": (_I, [_I, _I] + _V_TAIL),
    "tuna2_algorithm": (_I, [_I, _I] + _V_TAIL),
    "TTPL_BT_alltoallv": (_I, [_I, _I, _I] + _V_TAIL),
    "TTPL_BT_alltoallv_s1": (_I, [_I, _I, _I] + _V_TAIL),
    "TTPL_rbruck_alltoallv": (_I, [_I, _I] + _V_TAIL),
    "twophase_rbruck_alltoallv_async": (_I, [_I] + _V_TAIL + [_P]),
    "twophase_rbruck_alltoallv_om_async": (_I, [_I] + _V_TAIL + [_P]),
    "tuna_algorithm_async": (_I, [_I, _I] + _V_TAIL + [_P]),
    "TTPL_BT_alltoallv_async": (_I, [_I, _I, _I] + _V_TAIL + [_P]),
    "TTPL_BT_alltoallv_s1_async": (_I, [_I, _I, _I] + _V_TAIL + [_P]),
    "uniform_spreadout_twolayer_async": (_I, [_I, _I, _P, _I, _I, _P, _I, _I, _P, _P]),
    "uniform_inverse_isplit_r_bruck_async": (_I, [_I, _I, _I, _P, _I, _I, _P, _I, _I, _P, _P]),
    "vc_comm_wait": (_I, [_P]),
    "uniform_spreadout_twolayer": (_I, [_I, _I, _P, _I, _I, _P, _I, _I, _P]),
    "uniform_inverse_isplit_r_bruck": (_I, [_I, _I, _I, _P, _I, _I, _P, _I, _I, _P]),
    "MPICH_intra_scattered": (_I, [_I] + _V_TAIL),
    "ompi_alltoallv_intra_basic_linear": (_I, _V_TAIL),
    "ompi_alltoallv_intra_pairwise": (_I, _V_TAIL),
    "exclisive_or_alltoallv": (_I, _V_TAIL),
    "spreadout_alltoallv": (_I, _V_TAIL),
    "twolayer_communicator_linear": (_I, [_I] + _V_TAIL),
    "twolayer_communicator_linear_s2": (_I, [_I, _I, _I] + _V_TAIL),
    "vc_plan_create": (_I, [C.c_char_p, _I, _I, _I, _P, _P, _I, _P, _P, _I, _P, C.POINTER(_P)]),
    "vc_plan_execute": (_I, [_P, _P, _P]),
    "vc_plan_execute_async": (_I, [_P, _P, _P]),
    "vc_plan_free": (_I, [_P]),
    "vc_suggest_radix": (_I, [_P, _I, _I, _P, _I, C.POINTER(_I), _P, _P]),
    "vc_suggest_tunables": (_I, [_P, _I, _I, _P, _I, C.POINTER(_I), C.POINTER(_I), _P, _P, _P]),
    "vc_comm_calibration": (_I, [_P, C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "vc_comm_set_timing": (_I, [_P, _I]),
    "vc_comm_last_stats": (_I, [_P, C.POINTER(VcStats)]),
    "vc_comm_last_traffic": (_I, [_P, _I, _P]),
    "vc_comm_staging": (_I, [_P, C.POINTER(_P), C.POINTER(_I64)]),
    "vc_fill_payload": (_I, [_I, _U64, _P, _P, _P, _I, _P]),
    "vc_verify_alltoallv": (_I, [_P, _P, _P, _I, _P, _P, _P, _I, C.POINTER(_I64), _P]),
    "vc_calibration_copy": (_I, [_P, _P, _I64, _P]),
    "vc_calibration_copy2": (_I, [_P, _P, _P, _I64, _P]),
}

_lib = None


def load() -> C.CDLL:
    """Loads the built library; raises if it has not been built (python -m rbruck_alltoallv_amd.build)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `python -m rbruck_alltoallv_amd.build` "
                               "(there is no CPU fallback)")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(lib, name)          # AttributeError if the library does not export it
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib
