"""Wall-clock assertions about the tuner, on a real MI355X: `pytest -m perf`.  They are kept out of `-m gpu` (the
correctness suite, run with -x) because a timing taken on a busy box says nothing about the library's results."""
import pytest

pytestmark = pytest.mark.perf


def _gpu():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


@pytest.mark.skipif(not _gpu(), reason="needs the GPU")
@pytest.mark.parametrize("mode", [2, 0], ids=["forwarded", "launch-per-digit"])
@pytest.mark.parametrize("name", ["C3", "C5", "ML256"])
def test_suggested_radix_is_within_ten_percent_of_the_best_measured(name, mode):
    """The radix vc_suggest_tunables picks from its model runs within 10 % of the fastest candidate when all are timed
    (medians of 7 blocking calls each), on the shapes of configurations 3 and 5 and on the reference's 256-rank input matrix."""
    from rbruck_alltoallv_amd import api as A
    from tests.test_gpu_checks import suggestion_against_measured
    A.DEFAULT_FORWARDING = None
    ratio = suggestion_against_measured(A, name, mode)
    assert ratio <= 1.10, ratio
