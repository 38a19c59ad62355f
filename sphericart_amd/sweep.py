"""The table of achieved HBM bandwidth over the shapes of a call: l_max x derivatives x precision x kind of
harmonics, each at three sizes (20 000 points, as many points as give 1.2 GB of output, 2 000 000 points where
those stay below 6 GB).

`python bench.py --sweep` prints it as one JSON document; `profiles/sweep.json` is that output, and
tests/test_zy_sweep_guard.py measures the 1.2 GB column again and fails where a shape has fallen more than a
tenth below it. A row is

    ["gradients", "f32", "spherical", 20, "1.2GB", 169779, 274.1, 0.547, "pairs_kernel"]

(derivatives, dtype, harmonics, l_max, size, n_samples, us, frac, kernel; `load` gives the rows as dictionaries).

`us` is the best of three series of launches enqueued back to back after a warm-up (`bench.py --sweep`: after 0.3 s
of the same launches, so that the clocks have settled as they do under sustained load), between two events on the
launch stream; `frac` the algorithmic bytes of a launch, sizeof(T) * (3 + (l_max + 1)^2 * {1, 4, 13}) per point,
over `us` and the 8 TB/s peak. The points are uniform in a cube: no kernel here branches on the coordinates
except for points on the z axis, which the five benchmark clouds cover.
"""

import ctypes
import time

PEAK_HBM_GBPS = 8000.0
L_MAX = (1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 14, 16, 18, 20, 24, 28, 32)
DERIVATIVES = ("values", "gradients", "hessians")
SIZES = ("20k", "1.2GB", "2M")
_COMPONENTS = {"values": 1, "gradients": 4, "hessians": 13}


def bytes_per_point(l_max, derivatives, dtype):
    return (4 if dtype == "f32" else 8) * (3 + (l_max + 1) ** 2 * _COMPONENTS[derivatives])


def samples_for(size, l_max, derivatives, dtype):
    """Points of a row; None where the size is not measured for this shape."""
    per_point = bytes_per_point(l_max, derivatives, dtype)
    if size == "20k":
        return 20_000
    if size == "1.2GB":
        return int(min(2_000_000, max(20_000, 1.2e9 // per_point)))
    if size == "2M":
        return 2_000_000 if 1.2e9 < 2_000_000 * per_point <= 6e9 else None
    raise ValueError(size)


def shapes(sizes=SIZES, l_values=L_MAX):
    """Every row of the table as (derivatives, dtype, harmonics, l_max, size, n_samples)."""
    for derivatives in DERIVATIVES:
        for l_max in l_values:
            if derivatives == "hessians" and l_max > 24:
                continue
            for dtype in ("f32", "f64"):
                for harmonics in ("spherical", "solid"):
                    for size in sizes:
                        n = samples_for(size, l_max, derivatives, dtype)
                        if n is not None:
                            yield derivatives, dtype, harmonics, l_max, size, n


def measure_row(lib, derivatives, dtype, harmonics, l_max, size, n, launches=30, series=3, settle=0.0):
    """One row, measured on the current device: the best of `series` runs of `launches` launches back to back,
    after `settle` seconds of the same launches (under sustained load the device lowers its clocks, and some shapes
    rank differently in a short burst and after it has done so)."""
    import numpy as np
    import torch

    mode = DERIVATIVES.index(derivatives)
    normalized = int(harmonics == "spherical")
    ny = (l_max + 1) ** 2
    tdtype = torch.float32 if dtype == "f32" else torch.float64
    rng = np.random.default_rng(1)
    xyz = torch.from_numpy(rng.uniform(-3.0, 3.0, size=(n, 3))).to(tdtype).cuda()
    sph = torch.empty((n, ny), dtype=tdtype, device="cuda")
    dsph = torch.empty((n, 3, ny), dtype=tdtype, device="cuda") if mode >= 1 else None
    ddsph = torch.empty((n, 9, ny), dtype=tdtype, device="cuda") if mode >= 2 else None
    forward = lib.sphx_forward_f32 if dtype == "f32" else lib.sphx_forward_f64
    stream = torch.cuda.current_stream()
    args = (xyz.data_ptr(), n, l_max, normalized, mode, sph.data_ptr(),
            dsph.data_ptr() if dsph is not None else None, ddsph.data_ptr() if ddsph is not None else None,
            stream.cuda_stream)

    def launch():
        if forward(*args) != 0:
            raise RuntimeError(lib.sphx_last_error().decode())

    for _ in range(max(8, launches // 2)):
        launch()
    torch.cuda.synchronize()
    began = time.monotonic()
    while time.monotonic() - began < settle:
        for _ in range(50):
            launch()
        torch.cuda.synchronize()
    best = None
    for _ in range(series):
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        begin.record(stream)
        for _ in range(launches):
            launch()
        end.record(stream)
        torch.cuda.synchronize()
        us = begin.elapsed_time(end) / launches * 1e3
        best = us if best is None else min(best, us)
    text = ctypes.create_string_buffer(1024)
    lib.sphx_describe_plan(n, l_max, mode, int(dtype == "f64"), normalized, text, len(text))
    plan = text.value.decode()
    kernel = "+".join(part.split("<")[0].strip() for part in plan.split(" + "))
    nbytes = bytes_per_point(l_max, derivatives, dtype) * n
    del sph, dsph, ddsph, xyz
    torch.cuda.empty_cache()
    return {"derivatives": derivatives, "dtype": dtype, "harmonics": harmonics, "l_max": l_max, "size": size,
            "n_samples": n, "us": round(best, 2), "frac": round(nbytes / best / 1e3 / PEAK_HBM_GBPS, 4),
            "kernel": kernel}


COLUMNS = ("derivatives", "dtype", "harmonics", "l_max", "size", "n_samples", "us", "frac", "kernel")


def dump(rows, **header):
    """The table as JSON text: the header's fields, the column names once, one row per line."""
    import json

    head = json.dumps(dict(header, columns=list(COLUMNS)))[:-1]
    lines = ",\n".join(json.dumps([row[c] for c in COLUMNS]) for row in rows)
    return head + ', "rows": [\n' + lines + "\n]}"


def load(path):
    """The rows of a table written by dump, as dictionaries."""
    import json

    with open(path) as fd:
        table = json.load(fd)
    return [dict(zip(table["columns"], row)) for row in table["rows"]]


def key_of(row):
    return f"{row['derivatives']}/{row['dtype']}/{row['harmonics']}/l{row['l_max']}/{row['size']}"


def run(lib, sizes=SIZES, l_values=L_MAX, progress=None, settle=0.0):
    rows = []
    for shape in shapes(sizes, l_values):
        row = measure_row(lib, *shape, launches=60 if shape[4] == "20k" else 30, settle=settle)
        rows.append(row)
        if progress is not None:
            progress(row)
    return rows


def as_markdown(rows, size="1.2GB"):
    """The rows of one size as a table: l_max down, derivatives x precision x kind of harmonics across, percent
    of the HBM peak."""
    columns = [(d, t, h) for d in DERIVATIVES for t in ("f32", "f64") for h in ("spherical", "solid")]
    by_key = {(r["derivatives"], r["dtype"], r["harmonics"], r["l_max"]): r for r in rows if r["size"] == size}
    lines = ["| l_max | " + " | ".join(f"{d[:4]} {t} {h[:3]}" for d, t, h in columns) + " |",
             "|---|" + "---|" * len(columns)]
    for l_max in sorted({r["l_max"] for r in rows}):
        cells = []
        for d, t, h in columns:
            r = by_key.get((d, t, h, l_max))
            cells.append(f"{100 * r['frac']:.0f}" if r else "")
        lines.append(f"| {l_max} | " + " | ".join(cells) + " |")
    return "\n".join(lines)
