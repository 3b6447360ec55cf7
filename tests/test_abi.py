"""The C-ABI library loads and exports every function include/rbruck_vc.h declares (no GPU needed)."""
import ctypes
import os
import re

from rbruck_alltoallv_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "rbruck_vc.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"^\s*#.*$", "", text, flags=re.M)
    names = re.findall(r"\b([A-Za-z_][A-Za-z0-9_]*)\s*\([^;{}]*\)\s*;", text)
    return sorted(set(names))


def test_header_declares_the_reference_entry_points():
    names = declared_functions()
    for ref in ("twophase_rbruck_alltoallv", "twophase_rbruck_alltoallv_om", "tuna_algorithm", "TTPL_BT_alltoallv",
                "TTPL_BT_alltoallv_s1", "uniform_spreadout_twolayer", "uniform_inverse_isplit_r_bruck"):
        assert ref in names


def test_library_exports_every_declared_symbol():
    assert os.path.exists(_lib.LIB_PATH), "build first: python -m rbruck_alltoallv_amd.build"
    lib = ctypes.CDLL(_lib.LIB_PATH)
    names = declared_functions()
    assert len(names) >= 22
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/rbruck_vc.h but not exported"
    # and the Python binding knows all of them
    assert sorted(_lib.SYMBOLS) == names


def test_stats_struct_layout_matches_header():
    text = open(os.path.join(ROOT, "include", "rbruck_vc.h")).read()
    assert f"#define VC_MAX_LAUNCHES {_lib.VC_MAX_LAUNCHES}" in text
    # two int32, three int64, four float, the two per-launch arrays, two int32, five int64
    fields = 2 * 4 + 3 * 8 + 4 * 4 + _lib.VC_MAX_LAUNCHES * (8 + 4) + 2 * 4 + 5 * 8
    assert ctypes.sizeof(_lib.VcStats) == fields and fields % 8 == 0
    assert _lib.VcStats.launch_bytes.offset == 48 and _lib.VcStats.execution.offset == fields - 8 - 5 * 8
    assert _lib.VcStats.bad_table_entries.offset == fields - 16 and _lib.VcStats.host_waits.offset == fields - 8


def test_argument_errors_need_no_gpu():
    """Entry points reject bad arguments before touching the device; without a HIP device vc_comm_create says so."""
    lib = _lib.load()
    handle = ctypes.c_void_p()
    assert lib.vc_comm_create(0, ctypes.byref(handle)) == -5                 # VC_ERR_ARG: nranks < 1
    assert b"nranks" in lib.vc_last_error_string()
    rc = lib.vc_comm_create(4, ctypes.byref(handle))
    assert rc in (0, -6)                                                      # VC_OK on a GPU box, VC_ERR_NO_DEVICE here
    if rc == 0:
        assert lib.vc_comm_size(handle) == 4
        assert lib.vc_comm_free(handle) == 0
    else:
        assert b"no HIP device" in lib.vc_last_error_string()
    assert lib.vc_comm_size(None) == -5
    assert lib.vc_comm_set_forwarding(None, 1) == -5
    assert lib.twophase_rbruck_alltoallv(2, None, None, None, 1, None, None, None, 1, None) == -5
    assert lib.vc_plan_execute(None, None, None) == -5
