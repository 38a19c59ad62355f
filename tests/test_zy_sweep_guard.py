"""The planner's choices, guarded by what they achieve: the 1.2 GB column of the table of achieved bandwidth
(``python bench.py --sweep``, kept as ``profiles/sweep.json``) is measured again and compared row by row with the
fraction of the HBM peak recorded there.

The table is recorded with every row settled (0.3 s of its own launches before it is timed: under sustained load
the device lowers its clocks, and a burst on a device that has just been idle has not brought them up yet), and the
test settles every row for 0.15 s; measured like that a box reads 0.97-1.02 of the table row by row. Boxes still
differ by some 5 % as a whole, and the float64 kernels can run in one of two states a tenth apart from process to
process with the same code, so a row is not judged against the recorded number alone: the test fails when the rows
as a whole have fallen a tenth (the median of measured / recorded below 0.9), or when a single row has fallen more
than 15 % below what that median makes of its recorded value. A slow row is measured up to three times, with fresh
buffers, before it counts (another process's burst on the box).

Collected next to last, so that a timing that fails hides no parity test.
"""

import os

import pytest

from gpu_utils import announce
from sphericart_amd import sweep

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_no_shape_has_fallen_a_tenth_below_the_recorded_table(library):
    recorded = {sweep.key_of(row): row for row in sweep.load(os.path.join(ROOT, "profiles", "sweep.json"))}
    shapes = {}
    for shape in sweep.shapes(sizes=("1.2GB",)):
        key = sweep.key_of(dict(zip(("derivatives", "dtype", "harmonics", "l_max", "size"), shape[:5])))
        if key in recorded:
            shapes[key] = shape
    assert len(shapes) >= 150, "profiles/sweep.json holds too few rows of the 1.2 GB column"
    rows = {}
    for key, shape in shapes.items():
        announce("sweep guard", key)
        rows[key] = sweep.measure_row(library, *shape, launches=20, series=3, settle=0.15)
    ratio = lambda key: rows[key]["frac"] / recorded[key]["frac"]
    median = sorted(ratio(key) for key in rows)[len(rows) // 2]
    print(f"median of measured / recorded over {len(rows)} rows: {median:.3f}")
    floor = 0.85 * min(median, 1.0)
    for key in [key for key in rows if ratio(key) < floor]:
        for _ in range(2):
            if ratio(key) >= floor:
                break
            announce("sweep guard, again", key)
            rows[key] = sweep.measure_row(library, *shapes[key], launches=40, series=4, settle=0.3)
    fallen = [(key, rows[key]["kernel"], rows[key]["frac"], "recorded", recorded[key]["kernel"], recorded[key]["frac"])
              for key in rows if ratio(key) < floor]
    worst = sorted(rows, key=ratio)[:8]
    print("lowest:", [(key, round(ratio(key), 3)) for key in worst])
    assert median >= 0.9, f"the rows as a whole run at {median:.3f} of the recorded table"
    assert not fallen, (f"median {median:.3f}", fallen)


def test_recorded_table_meets_the_bars_it_was_made_for():
    """What the table says of itself, no GPU involved in the check: the rows at 1.2 GB that the kernels were
    tuned for."""
    rows = [r for r in sweep.load(os.path.join(ROOT, "profiles", "sweep.json")) if r["size"] == "1.2GB"]
    assert len(rows) >= 150
    for r in rows:
        assert 0.3 < r["frac"] < 1.0, r
