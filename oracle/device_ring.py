"""The device-ring rules the reference states for its GPU session, restated for the oracle
(crates/wgpu-compute/src/session.rs:235-346): ring capacity, the snapshot-visible range of a
layer, and the split of a stored range into runs of consecutive ring slots. Test
infrastructure only.

Pinned by the reference's own cases (tests/test_oracle_device_ring.py): ring capacities
2111 / 2079 / 2048 / 67 (session.rs:6091-6120), the visible ranges of session.rs:6183-6202,
and the slot runs of session.rs:6204-6268 including its sweep over caps 1/4/32/64 and
positions 0..300 (at most two runs, exact coverage, slots == position % ring).
"""
from __future__ import annotations

from typing import List, Optional, Tuple


def ring_capacity(sliding_window: int, chunk_cap: int) -> int:  # session.rs:247-249
    return sliding_window + chunk_cap - 1


def prefix_visible_range(window: Optional[int], position: int) -> Tuple[int, int]:  # session.rs:284-292
    """(first_position, rows) a snapshot holds of one layer at `position`; window None = global."""
    if window is None:
        return 0, position
    rows = min(position, window)
    return position - rows, rows


def prefix_slot_runs(windowed: bool, first_position: int, rows: int, ring: int) -> List[Tuple[int, int, int]]:
    """session.rs:320-346: (row, slot, count) runs; a global layer slots a position at itself,
    a windowed one at position % ring."""
    runs: List[List[int]] = []
    for r in range(rows):
        position = first_position + r
        slot = position % ring if windowed else position
        if runs and runs[-1][1] + runs[-1][2] == slot:
            runs[-1][2] += 1
            continue
        runs.append([r, slot, 1])
    return [tuple(run) for run in runs]
