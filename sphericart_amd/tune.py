"""Settled timings of planner settings, the measurement behind the tables of `csrc/sphx_plan_shapes.hpp` and the
thresholds of `csrc/sphx_plan.cpp`.

    python -m sphericart_amd.tune --switch SPHX_WAVE_PRIORITIES,SPHX_SEQUENCE_WAVES \\
        --values "-1,-1 1,-1 1,3 0,2" --shapes "f32:10:gradients:solid f64:19:gradients:solid:300000"

For every shape (dtype : l_max : values | gradients | hessians : spherical | solid [: points], 1.2 GB of output
where no number of points is given) every setting of the switches (one value per switch, -1 = leave it to the
planner) runs `--settle` seconds of its own launches before `--launches` launches are timed between two events, in
`--turns` turns over all settings; the median of a setting's turns is printed in us per launch.

Why every setting settles on its own: under sustained load the device lowers its clocks within some tens of
milliseconds, a burst on a cool device runs 2-10 % faster than the same launches after that, settings that take
turns in short bursts are timed at the clocks the one before them left behind, and a few shapes rank differently
in the two states. Measured like this, three turns of a setting agree to about 1 us in 200.
"""

import argparse
import ctypes
import statistics
import sys
import time

from . import _c_lib, sweep

HARMONICS = ("solid", "spherical")


def parse_shape(text):
    parts = text.split(":")
    if len(parts) not in (4, 5) or parts[0] not in ("f32", "f64") or parts[2] not in sweep.DERIVATIVES or \
            parts[3] not in HARMONICS:
        raise ValueError(f"not dtype:l_max:derivatives:harmonics[:points]: {text!r}")
    l_max = int(parts[1])
    points = int(parts[4]) if len(parts) == 5 else sweep.samples_for("1.2GB", l_max, parts[2], parts[0])
    return parts[0], l_max, parts[2], parts[3], points


def parse_values(text, count):
    settings = [tuple(int(v) for v in setting.split(",")) for setting in text.split()]
    for setting in settings:
        if len(setting) != count:
            raise ValueError(f"{count} switches, but the setting {setting} has {len(setting)} values")
    return settings


def measure(lib, shape, names, settings, settle, launches, turns):
    """us per launch of every setting: the median over `turns` turns."""
    import numpy as np
    import torch

    dtype, l_max, derivatives, harmonics, n = shape
    mode = sweep.DERIVATIVES.index(derivatives)
    tdtype = torch.float32 if dtype == "f32" else torch.float64
    ny = (l_max + 1) ** 2
    xyz = torch.from_numpy(np.random.default_rng(1).uniform(-3.0, 3.0, size=(n, 3))).to(tdtype).cuda()
    outs = [torch.empty((n, c, ny), dtype=tdtype, device="cuda") for c in (1, 3, 9)[: mode + 1]]
    pointers = [o.data_ptr() for o in outs] + [None] * (2 - mode)
    forward = lib.sphx_forward_f32 if dtype == "f32" else lib.sphx_forward_f64
    stream = torch.cuda.current_stream()
    args = (xyz.data_ptr(), n, l_max, int(harmonics == "spherical"), mode, *pointers, stream.cuda_stream)

    def launch():
        if forward(*args) != 0:
            raise RuntimeError(lib.sphx_last_error().decode())

    times = [[] for _ in settings]
    for _ in range(turns):
        for which, setting in enumerate(settings):
            lib.sphx_reset_switches()
            for name, value in zip(names, setting):
                if value >= 0 and lib.sphx_set_switch(name.encode(), value) != 0:
                    raise ValueError(lib.sphx_last_error().decode())
            began = time.monotonic()
            launch()
            while time.monotonic() - began < settle:
                for _ in range(50):
                    launch()
                torch.cuda.synchronize()
            begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            begin.record(stream)
            for _ in range(launches):
                launch()
            end.record(stream)
            torch.cuda.synchronize()
            times[which].append(begin.elapsed_time(end) / launches * 1e3)
    lib.sphx_reset_switches()
    return [statistics.median(t) for t in times]


def main(argv=None):
    p = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    p.add_argument("--switch", required=True, help="names of planner switches (csrc/sphx_plan.hpp), comma-separated")
    p.add_argument("--values", required=True, help='settings, space-separated, one value per switch: "-1,-1 1,3"')
    p.add_argument("--shapes", required=True, help="dtype:l_max:derivatives:harmonics[:points], space-separated")
    p.add_argument("--settle", type=float, default=0.4, help="seconds of a setting's own launches before it is timed")
    p.add_argument("--launches", type=int, default=100)
    p.add_argument("--turns", type=int, default=3)
    args = p.parse_args(argv)
    names = args.switch.split(",")
    settings = parse_values(args.values, len(names))
    shapes = [parse_shape(text) for text in args.shapes.split()]
    lib = _c_lib.get_library()
    lib.sphx_set_switch.argtypes = [ctypes.c_char_p, ctypes.c_int]
    for shape in shapes:
        us = measure(lib, shape, names, settings, args.settle, args.launches, args.turns)
        best = min(range(len(us)), key=us.__getitem__)
        cells = "  ".join(f"{','.join(map(str, s))}: {t:7.1f}" for s, t in zip(settings, us))
        print(f"{':'.join(map(str, shape))}  {cells}   best {','.join(map(str, settings[best]))} "
              f"({us[0] / us[best]:.3f} x the first)", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
