"""The C++ driver above the C ABI (rbruck_alltoallv_amd/examples/vc_example.cpp): the reference's example loops
(examples/rbruckv_example.cpp, examples/twophaseLayer_example.cpp) with every element of every receive buffer checked
on the host."""
import os
import subprocess

import pytest

from rbruck_alltoallv_amd.build import EXAMPLE_BIN, MLINPUTS_EXAMPLE_BIN

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("P,ncores,bases", [(64, 8, [2, 4, 8]), (12, 3, [3, 12])])
def test_example_driver_reports_no_errors(P, ncores, bases):
    assert os.path.exists(EXAMPLE_BIN), "build it with python -m rbruck_alltoallv_amd.build"
    res = subprocess.run([EXAMPLE_BIN, str(P), "1", str(ncores)] + [str(b) for b in bases], capture_output=True, text=True,
                         timeout=300)
    assert res.returncode == 0, res.stdout[-2000:] + res.stderr[-2000:]
    lines = res.stdout.splitlines()
    assert lines[-1] == "errors: 0"
    assert not any("has errors" in l or "fail!" in l for l in lines)
    sizes = 11                                               # n = 2 .. 2048
    assert sum(l.startswith("[Rbruckv]") for l in lines) == sizes * len(bases)
    assert sum(l.startswith("[TTPL]") for l in lines) == sizes * len(bases)
    assert sum(l.startswith("[TTPL_S1]") for l in lines) == sizes * len(bases)
    assert sum(l.startswith("[Spreadout]") for l in lines) == sizes
    assert sum(l.startswith("[ExcOr]") for l in lines) == (sizes if P & (P - 1) == 0 else 0)
    assert sum(l.startswith("[SOR_alltoall]") for l in lines) == sizes * len(bases)      # the equal-block functions
    assert sum(l.startswith("[BR_alltoall]") for l in lines) == sizes * len(bases)


def test_mlinputs_driver_reads_the_reference_text_format(tmp_path):
    """examples/MLinputs_example.cpp on the virtual communicator: a matrix in the reference's text format (one of its own
    input matrices, scaled down and written back as text), the one-pass exchange and twophase_rbruck_alltoallv per base."""
    import numpy as np

    from rbruck_alltoallv_amd import workloads as W
    from tests.helpers import INPUTS_DIR
    assert os.path.exists(MLINPUTS_EXAMPLE_BIN), "build it with python -m rbruck_alltoallv_amd.build"
    counts = W.counts_from_npz(os.path.join(INPUTS_DIR, "global_comm_pattern_64proc.npz"), 64)
    path = tmp_path / "global_comm_pattern_64proc.txt"
    np.savetxt(path, counts, fmt="%d")
    res = subprocess.run([MLINPUTS_EXAMPLE_BIN, str(path), "64", "2", "2", "8", "64"], capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stdout[-2000:] + res.stderr[-2000:]
    lines = res.stdout.splitlines()
    assert lines[-1] == "errors: 0"
    total = int(counts.astype(np.int64).sum())
    assert sum(l.startswith("MPI_Alltoallv, 64 ") and l.endswith(f" {total} {total}") for l in lines) == 2
    for base in (2, 8, 64):
        assert sum(l.startswith(f"TUNA, 64 {base} ") for l in lines) == 2
