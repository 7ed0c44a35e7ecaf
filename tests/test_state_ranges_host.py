"""Selections of a state snapshot: canonical form and payload size (host logic, no GPU).  Mirrors the reference's
own checks of `selected_buffer_ranges` (crates/inference-executor-metal/src/model/state_snapshot.rs:743-776)."""
import importlib

import pytest

psi = importlib.import_module("psi-dec_amd")
snap = importlib.import_module("psi-dec_amd.state_snapshot")


def test_payload_is_the_sum_of_the_ranges():
    assert snap.selected_payload_bytes([(0, 1)], 64, 64) == 64
    assert snap.selected_payload_bytes([(1, 3), (5, 6), (9, 16)], 32768, 16 * 32768) == 10 * 32768
    assert snap.selected_payload_bytes([], 64, 64) == 0
    assert snap.selected_payload_bytes([(0, 0xFFFFFFFF)], 3, 3 * 0xFFFFFFFF) == 3 * 0xFFFFFFFF  # u64 arithmetic


@pytest.mark.parametrize("ranges", [
    [(2, 2)],            # empty
    [(3, 2)],            # reversed
    [(4, 6), (1, 2)],    # unsorted
    [(1, 4), (3, 6)],    # overlapping
    [(1, 3), (3, 6)],    # adjacent: must have been merged
])
def test_non_canonical_ranges_are_rejected(ranges):
    with pytest.raises(psi.PsiHipError, match="nonempty, sorted, disjoint, and nonadjacent"):
        snap.selected_payload_bytes(ranges, 16, 1 << 20)


def test_out_of_bounds_and_zero_entry_size():
    with pytest.raises(psi.PsiHipError, match="entry range is out of bounds: entry_range=2..5 entry_bytes=16"):
        snap.selected_payload_bytes([(0, 1), (2, 5)], 16, 79)
    assert snap.selected_payload_bytes([(0, 1), (2, 5)], 16, 80) == 64
    with pytest.raises(psi.PsiHipError, match="entry size must be positive"):
        snap.selected_payload_bytes([(0, 1)], 0, 64)
    with pytest.raises(ValueError):
        snap.selected_payload_bytes([(0, 1, 2)], 16, 64)
