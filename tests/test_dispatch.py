"""The library's choice of kernel for a call, pinned as a table (csrc/vc_dispatch.h compiled for the CPU): from the rank
count and what the last forwarded call on the communicator looked like to lanes per pair of ranks (0 = through the
work-item list, 256 / 64 / 16 = a workgroup / a wavefront / a quarter of one per pair, 1 = a batch of pairs per wavefront)
and whether the call is first tried as one launch on fixed-stride staging.  Every entry point decides through this one
function; a changed threshold shows here."""
import pytest

from tests import emulator as E

LIST, BATCH, QUARTER, WAVE, GROUP = 0, 1, 16, 64, 256
# the last call: (average piece, most pieces of a block, longest block), one piece per pair of ranks
HINTS = {"100 B": (100, 1, 300), "500 B": (500, 1, 1500), "1 KB": (1000, 2, 5000), "2 KB": (2000, 3, 9000),
         "4 KB": (4000, 4, 16000), "4 KB, a block of 20 pieces": (4000, 20, 100000)}
# rank count -> per hint (lanes, fixed stride tried first), radix-2 Bruck
TABLE = {
    16: [(WAVE, True), (WAVE, True), (WAVE, True), (WAVE, True), (GROUP, True), (LIST, False)],       # up to 32 ranks never a quarter
    32: [(WAVE, True), (WAVE, True), (WAVE, True), (WAVE, True), (GROUP, True), (LIST, False)],
    64: [(QUARTER, True), (QUARTER, True), (QUARTER, True), (WAVE, True), (GROUP, False), (LIST, False)],   # a quarter below 1.75 KiB
    128: [(QUARTER, True), (QUARTER, True), (QUARTER, False), (QUARTER, False), (GROUP, False), (LIST, False)],   # ... below 3 KiB; 256 MiB of slots at most
    160: [(BATCH, True), (QUARTER, False), (LIST, False), (LIST, False), (LIST, False), (LIST, False)],     # above 128 ranks: short blocks only
    192: [(BATCH, True), (QUARTER, False), (LIST, False), (LIST, False), (LIST, False), (LIST, False)],
    256: [(BATCH, False), (QUARTER, False), (LIST, False), (LIST, False), (LIST, False), (LIST, False)],    # above 192 ranks no fixed stride
    1024: [(BATCH, False), (QUARTER, False), (LIST, False), (LIST, False), (LIST, False), (LIST, False)],
}


def _hint(P, average, max_pieces, max_len):
    return (1, P * P, average * P * P, max_pieces, max_len)


@pytest.mark.parametrize("P", sorted(TABLE))
def test_default_mode_decision_table(P):
    for (name, h), (lanes, strided) in zip(HINTS.items(), TABLE[P]):
        d = E.dispatch(E.F_TWOPHASE, P, _hint(P, *h), mode=1, r=2)
        assert (d["lanes"], d["stride"] > 0) == (lanes, strided), (P, name, d)
        if strided:
            # slots hold the last call's longest block at any cache-line phase; the batches become quarters there
            assert d["stride"] % 128 == 0 and d["stride"] >= h[2] + 127 and d["max_len"] == d["stride"] - 127
            assert d["stride_lanes"] == (QUARTER if lanes == BATCH else lanes)
        if lanes:
            # the hint is a guess: what the kernel checks on the device before it moves anything
            short = lanes in (BATCH, QUARTER)
            assert (d["max_pieces"], d["max_items"], d["max_average"]) == ((8, 0, 4096) if short else (16, 32768, 0)), (P, name, d)


def test_without_a_hint_and_in_the_forced_modes():
    for P in (8, 64, 1024):
        assert E.dispatch(E.F_TWOPHASE, P, (0, 0, 0, 0, 0), mode=1)["lanes"] == LIST            # the first call on a communicator
        short = _hint(P, 100, 1, 300)
        assert E.dispatch(E.F_TWOPHASE, P, short, mode=0)["lanes"] == LIST                        # launch per digit
        assert E.dispatch(E.F_TWOPHASE, P, short, mode=2)["lanes"] == LIST                        # the list was asked for
        for mode, lanes in ((3, GROUP), (4, QUARTER), (5, BATCH)):
            d = E.dispatch(E.F_TWOPHASE, P, (0, 0, 0, 0, 0), mode=mode)
            assert d == dict(lanes=lanes, stride=0, stride_lanes=0, max_pieces=0, max_items=0, max_average=0, max_len=0)


def test_calls_that_cannot_wait_for_a_list():
    """The _async twins and the entry point that allocates nothing never go through the list and never guard: short blocks by
    the same rule as the blocking calls, everything else a workgroup per pair."""
    for P, expect in ((64, [QUARTER, QUARTER, QUARTER, GROUP, GROUP, GROUP]), (1024, [BATCH, QUARTER, GROUP, GROUP, GROUP, GROUP])):
        for h, lanes in zip(HINTS.values(), expect):
            for mode in (0, 1, 2):
                d = E.dispatch(E.F_TWOPHASE, P, _hint(P, *h), mode=mode, call_kind=1)
                assert d == dict(lanes=lanes, stride=0, stride_lanes=0, max_pieces=0, max_items=0, max_average=0, max_len=0), (P, h, d)
        assert E.dispatch(E.F_TWOPHASE, P, (0, 0, 0, 0, 0), mode=1, call_kind=1)["lanes"] == GROUP


def test_many_digits_and_two_layers():
    # a staging region per digit: 7 regions of 128 x 128 slots of 1.6 KB are 184 MiB, of 5.1 KB more than the 256 MiB allowed
    assert E.dispatch(E.F_TWOPHASE, 128, _hint(128, 500, 1, 1500), r=2)["stride"] == 1664
    assert E.dispatch(E.F_TWOPHASE, 128, _hint(128, 1000, 2, 5000), r=2)["stride"] == 0
    assert E.dispatch(E.F_TWOPHASE, 128, _hint(128, 1000, 2, 5000), r=16)["stride"] == 5248       # two regions
    # the two-layer functions, forwarded, carry every block on its own (no organized region): same rule
    for f in (E.F_TTPL, E.F_TTPL_S1):
        d = E.dispatch(f, 64, _hint(64, 100, 1, 300), n=8, r=2)
        assert (d["lanes"], d["stride"]) == (QUARTER, 512)


def test_lanes_per_work_item_of_the_list_kernels():
    for average, lanes in ((16, QUARTER), (447, QUARTER), (448, WAVE), (3071, WAVE), (3072, GROUP), (4096, GROUP)):
        assert E.lanes_for_items(average * 1000, 1000) == lanes
    assert E.lanes_for_items(0, 0) == GROUP
