#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg3]

A step is one evaluation of one batch of synthetic points that already sit in
HBM: one kernel launch through the C launch layer (sphx_forward_*) writing
preallocated outputs. The default workload is the configuration the headline
metric is quoted on: real spherical harmonics, l_max = 6, float32, values and
gradients, 1,000,000 points.

The K timed steps are enqueued back to back between one pair of host clock
readings (`value`, `ms_per_step`) and one pair of events on the launch stream,
whose distance over K is the average launch duration that `roofline` is
computed from. A second pass of K steps with an event pair around every launch
records the spread; such a pair adds 2-4 us to the launch it brackets, which
matters for the configurations whose launch takes 12 us.

One JSON line is printed. Next to the contract fields it carries

  roofline      achieved HBM bandwidth of the kernel: algorithmic bytes per
                launch (sizeof(T) * (3 + (l_max+1)^2 * components) per point)
                divided by the average launch duration, measured with events
                on the launch stream around the timed region, against the
                8 TB/s peak of MI355X;
  roofline_by_config
                (default workload only) the same figure for the other four
                configurations of the reference's benchmark set, each with the
                kernel it launches, and for cfg1-cfg3 a second figure with the
                outputs rotating through 1 GB of buffers, so that no launch
                finds its lines in the 256 MB Infinity Cache;
  cpu_baseline  the reference CPU implementation (oracle/_ref, built from the
                reference's own sources; the repository's restatement when that
                is absent) timed on the host cores on a bounded number of
                passes over the same points.
"""

import argparse
import ctypes
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_HBM_GBPS = 8000.0

def measured_traffic(key, kernels):
    """HBM bytes per launch of a workload from profiles/traffic.json: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs
    of this script (the summaries under profiles/ that each entry names), each counter scaled by what it reads
    for a plain device-to-device copy of known size (`--calibrate-copy`: WRITE_SIZE reads the copied bytes
    exactly, FETCH_SIZE half of them, so fetches are doubled), fetch + write, all kernels of one call added up.
    None when the entry was measured on another kernel than the one the library now launches for the shape."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as fd:
            entry = json.load(fd)["workloads"].get(key)
    except (OSError, ValueError, KeyError):
        return None
    if entry is None:
        return None
    if kernels is not None:
        launched = "+".join(part.split("<")[0].strip() for part in kernels.split(" + "))
        if launched != entry["kernel"]:
            return None
    return entry["bytes"]


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=200)
    p.add_argument("--warmup", type=int, default=20)
    p.add_argument("--workload", default="cfg3")
    p.add_argument(
        "--settle-seconds",
        type=float,
        default=0.5,
        help="untimed launches before the warm-up steps until the GPU has been busy this long: the "
        "memory and fabric clocks of an idle MI355X take tens of milliseconds of load to ramp up "
        "(the same launch takes 160 us right after idle and 136 us once settled)",
    )
    p.add_argument(
        "--op",
        choices=("forward", "backward", "vjp"),
        default="forward",
        help="backward: time the vector-Jacobian product xyz_grad = sum_k dsph * sph_grad "
        "(sphx_backward_*) on the gradients of the workload instead of the forward pass; "
        "vjp: the same product fused with the evaluation of the gradients (sphx_vjp_*)",
    )
    p.add_argument(
        "--rotate-mb",
        type=int,
        default=0,
        help="forward pass only: write to a rotating set of output buffers of at least this many MB "
        "in total, so that a workload whose outputs fit into the 256 MB Infinity Cache (cfg1, cfg2) "
        "is also measured with every launch going to memory that is not cached",
    )
    p.add_argument("--no-cpu-baseline", action="store_true")
    p.add_argument("--no-by-config", action="store_true",
                   help="default workload only: leave out the measurements of the other four configurations")
    p.add_argument(
        "--calibrate-copy",
        action="store_true",
        help="instead of the hot path, launch plain device-to-device copies of as many bytes as "
        "the workload writes per launch: the yardstick for the FETCH_SIZE / WRITE_SIZE counters",
    )
    p.add_argument(
        "--sweep",
        action="store_true",
        help="instead of one workload, the table of achieved bandwidth over l_max x derivatives x precision x "
        "kind of harmonics at 20 000 points, at 1.2 GB of output and at 2 000 000 points (sphericart_amd/sweep.py), "
        "as one JSON document on stdout; progress goes to stderr",
    )
    p.add_argument("--sweep-sizes", default="20k,1.2GB,2M", help="with --sweep: which of the three sizes")
    p.add_argument("--sweep-markdown", action="store_true", help="with --sweep: print the tables as Markdown instead")
    p.add_argument("--sweep-settle-seconds", type=float, default=0.3,
                   help="with --sweep: seconds of launches of a row before it is timed (the clocks settle)")
    return p.parse_args()


def sweep(lib, args):
    import subprocess

    from sphericart_amd import sweep as table

    sizes = tuple(s for s in args.sweep_sizes.split(",") if s)

    def progress(row):
        print(f"{table.key_of(row):48s} {row['us']:9.1f} us {100 * row['frac']:5.1f} %  {row['kernel']}",
              file=sys.stderr, flush=True)

    rows = table.run(lib, sizes=sizes, progress=progress, settle=args.sweep_settle_seconds)
    if args.sweep_markdown:
        for size in sizes:
            print(f"\n{size}\n\n{table.as_markdown(rows, size)}")
        return 0
    try:
        commit = subprocess.run(["git", "-C", ROOT, "rev-parse", "--short", "HEAD"], capture_output=True, text=True,
                                timeout=10).stdout.strip() or None
    except (OSError, subprocess.SubprocessError):
        commit = None
    print(table.dump(rows, command="python bench.py --sweep --sweep-sizes " + ",".join(sizes), commit=commit,
                     peak_GBps=table.PEAK_HBM_GBPS))
    return 0


def cpu_baseline(workload, xyz):
    """Reference CPU path on the host cores: best-of timing over a bounded number of passes."""
    import numpy as np

    import oracle  # the CPU checker: used here only as the baseline being reported

    if oracle.available("ref_fma"):
        flavour, kind = "ref_fma", "reference"
    else:
        flavour, kind = "oracle", "port"
    n = workload.n_samples
    ny = (workload.l_max + 1) ** 2
    mode = workload.derivatives
    out = (
        np.empty((n, ny), dtype=xyz.dtype),
        np.empty((n, 3, ny), dtype=xyz.dtype) if mode != "values" else None,
        np.empty((n, 3, 3, ny), dtype=xyz.dtype) if mode == "hessians" else None,
    )
    for o in out:
        if o is not None:
            o.fill(0)  # touch the pages once
    times = []
    started = time.perf_counter()
    passes = 0
    while passes < 3 or (time.perf_counter() - started < 2.0 and passes < 40):
        t0 = time.perf_counter()
        oracle.compute(xyz, workload.l_max, workload.normalized, mode, flavour, out=out)
        times.append(time.perf_counter() - t0)
        passes += 1
    timed = times[2:] if len(times) > 4 else times
    best = min(timed)
    cores = oracle.max_threads(flavour)
    model = "unknown CPU"
    try:
        with open("/proc/cpuinfo") as fd:
            for line in fd:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {
        "value": n / best,
        "unit": "points/s",
        "cores": cores,
        "kind": kind,
        "sample": f"{passes} passes over all {n} points of the workload, best pass "
        f"{best * 1e3:.2f} ms, median {statistics.median(timed) * 1e3:.2f} ms; "
        f"{'compiled reference sources (g++ -O3 -march=x86-64-v3 -ffp-contract=fast)' if kind == 'reference' else 'restatement (g++ -O2 -ffp-contract=off)'}, "
        f"OpenMP over {cores} threads of {model}",
        "GBps": workload.bytes_per_point * n / best / 1e9,
    }


def cpu_backward_baseline(dsph, sph_grad):
    """The checker's contraction loop, one thread, timed on a bounded slice of the points."""
    import oracle  # reported baseline only

    n = min(dsph.shape[0], 200_000)
    best = None
    for _ in range(5):
        t0 = time.perf_counter()
        oracle.backward(dsph[:n], sph_grad[:n])
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    return {
        "value": n / best,
        "unit": "points/s",
        "cores": 1,
        "kind": "port",
        "sample": f"5 passes over the first {n} points, best pass {best * 1e3:.2f} ms; plain C loop, one thread",
    }


def cpu_vjp_baseline(workload, xyz, sph_grad):
    """Gradients by the CPU evaluator (all cores), contracted by the checker's loop (one thread)."""
    import oracle  # reported baseline only

    flavour, kind = ("ref_fma", "reference") if oracle.available("ref_fma") else ("oracle", "port")
    n = min(xyz.shape[0], 200_000)
    best = None
    for _ in range(5):
        t0 = time.perf_counter()
        _, dsph, _ = oracle.compute(xyz[:n], workload.l_max, workload.normalized, "gradients", flavour)
        oracle.backward(dsph, sph_grad[:n])
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    return {
        "value": n / best,
        "unit": "points/s",
        "cores": oracle.max_threads(flavour),
        "kind": kind,
        "sample": f"5 passes over the first {n} points, best pass {best * 1e3:.2f} ms; gradients by the CPU "
        "evaluator (OpenMP), then the contraction loop on one thread",
    }


class Prepared:
    """A workload's points and preallocated outputs on the GPU and the call that evaluates them."""

    def __init__(self, lib, w, rotate_mb=0):
        import torch

        self.lib, self.w = lib, w
        self.xyz_host = w.points()
        self.xyz = torch.from_numpy(self.xyz_host).cuda()
        self.n, self.ny = w.n_samples, (w.l_max + 1) ** 2
        self.opts = dict(dtype=self.xyz.dtype, device=self.xyz.device)
        self.mode = {"values": 0, "gradients": 1, "hessians": 2}[w.derivatives]
        self.forward = lib.sphx_forward_f32 if w.dtype == "f32" else lib.sphx_forward_f64
        self.stream = torch.cuda.current_stream()
        self.bytes_per_launch = w.bytes_per_point * self.n
        copies = 1
        if rotate_mb > 0:
            copies = max(2, -(-rotate_mb * 1_000_000 // self.bytes_per_launch))
        self.outputs = [self._allocate() for _ in range(copies)]
        self.calls = [self._pointers(o) for o in self.outputs]
        self.turn = 0

    def _allocate(self):
        import torch

        n, ny, mode = self.n, self.ny, self.mode
        return (torch.empty((n, ny), **self.opts),
                torch.empty((n, 3, ny), **self.opts) if mode >= 1 else None,
                torch.empty((n, 3, 3, ny), **self.opts) if mode >= 2 else None)

    def _pointers(self, o):
        return (self.xyz.data_ptr(), self.n, self.w.l_max, int(self.w.normalized), self.mode, o[0].data_ptr(),
                o[1].data_ptr() if o[1] is not None else None,
                o[2].data_ptr() if o[2] is not None else None, self.stream.cuda_stream)

    def step(self):
        status = self.forward(*self.calls[self.turn % len(self.calls)])
        self.turn += 1
        if status != 0:
            raise RuntimeError(self.lib.sphx_last_error().decode())

    def kernels(self):
        text = ctypes.create_string_buffer(1024)
        status = self.lib.sphx_describe_plan(self.n, self.w.l_max, self.mode, int(self.w.dtype == "f64"),
                                             int(self.w.normalized), text, len(text))
        return text.value.decode() if status == 0 else None


def settle(step, seconds, warmup):
    import torch

    until = time.perf_counter() + seconds
    while time.perf_counter() < until:
        for _ in range(50):
            step()
        torch.cuda.synchronize()
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()


def time_back_to_back(step, steps, stream):
    """K steps enqueued one after the other: host seconds between two synchronisations, and
    device milliseconds between one event before the first and one after the last launch."""
    import torch

    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    begin.record(stream)
    for _ in range(steps):
        step()
    end.record(stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall, begin.elapsed_time(end)


def time_each_launch(step, steps, stream):
    """Milliseconds of every one of K launches, an event pair around each."""
    import torch

    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    torch.cuda.synchronize()
    for begin, end in events:
        begin.record(stream)
        step()
        end.record(stream)
    torch.cuda.synchronize()
    return [b.elapsed_time(e) for b, e in events]


def roofline_of(device_ms, steps, launch_ms, bytes_per_launch):
    """`device_ms`: between one event before the first and one after the last of `steps` launches
    enqueued back to back; the average launch duration is that over `steps` (it agrees with the
    profiler's kernel durations to a few percent at every size). `launch_ms`: every launch between
    an event pair of its own, which adds 2-4 us to each (kept for the spread: median, minimum)."""
    avg_s = device_ms / steps / 1e3
    achieved = bytes_per_launch / avg_s / 1e9
    return {
        "bound": "hbm",
        "achieved": achieved,
        "peak": PEAK_HBM_GBPS,
        "unit": "GB/s",
        "frac": achieved / PEAK_HBM_GBPS,
        "algorithmic_bytes_per_launch": bytes_per_launch,
        "avg_launch_us": avg_s * 1e6,
        "back_to_back_us_per_launch": avg_s * 1e6,
        "per_launch_events": {
            "avg_us": sum(launch_ms) / len(launch_ms) * 1e3,
            "median_us": statistics.median(launch_ms) * 1e3,
            "min_us": min(launch_ms) * 1e3,
        },
    }


def measure_yardsticks(lib, stream):
    """What bounds a launch from below on this device, measured here: the duration of a kernel that does nothing,
    enqueued back to back (what the GPU needs to start and retire any kernel), and the rate at which plain
    streaming stores fill 1 GB of HBM (the evaluator's store pattern with nothing to compute)."""
    import torch

    def timed(step, steps):
        for _ in range(steps // 4):
            step()
        best = None
        for _ in range(3):
            _, ms = time_back_to_back(step, steps, stream)
            best = ms if best is None else min(best, ms)
        return best / steps * 1e-3

    def empty():
        if lib.sphx_probe_empty_launch(stream.cuda_stream) != 0:
            raise RuntimeError(lib.sphx_last_error().decode())

    nbytes = 1 << 30
    buffer = torch.empty(nbytes, dtype=torch.uint8, device="cuda")

    def fill():
        if lib.sphx_probe_fill(buffer.data_ptr(), nbytes, stream.cuda_stream) != 0:
            raise RuntimeError(lib.sphx_last_error().decode())

    empty_s = timed(empty, 2000)
    fill_s = timed(fill, 40)
    del buffer
    torch.cuda.empty_cache()
    return {"empty_launch_us": empty_s * 1e6, "fill_GBps": nbytes / fill_s / 1e9}


def with_floor(entry, yardsticks, nbytes):
    """latency_floor_us: an empty launch plus the algorithmic bytes at the measured fill rate; frac_of_floor: that
    over the measured launch (1 = nothing left to gain for a kernel that computes nothing)."""
    floor_us = yardsticks["empty_launch_us"] + nbytes / (yardsticks["fill_GBps"] * 1e9) * 1e6
    entry["latency_floor_us"] = floor_us
    entry["frac_of_floor"] = floor_us / entry["avg_launch_us"]
    return entry


def host_cost(lib, stream):
    """Host microseconds per call of calls in a row that nobody waits for, the shape of cfg1 (10 000 points,
    l_max = 8, float64, values and gradients): through sphx_forward_f64 and through the sphericart_cuda_* C API
    from a loop in C (sphx_probe_host_cost_f64), through sphx_forward_f64 from Python (ctypes), and through the
    torch operator. The host enqueues faster than the GPU evaluates, and once some 1 500 launches wait in the
    queue a further call blocks until one has run: `burst` is ten bursts of 1 000 calls, each started with the
    queue empty (what a call costs the host), `sustained` 10 000 calls in one go (what it costs once the queue is
    full: the kernel's time), `gpu` the same with the wait at the end included."""
    import torch

    import sphericart_amd.torch as sphericart_torch
    from sphericart_amd.workloads import WORKLOADS

    w = WORKLOADS["cfg1"]
    prepared = Prepared(lib, w)
    sph, dsph, _ = prepared.outputs[0]
    result = {"shape": "cfg1", "burst_calls": 1000, "sustained_calls": 10_000}
    seconds = ctypes.c_double()

    def in_c(through, calls):
        status = lib.sphx_probe_host_cost_f64(through, prepared.xyz.data_ptr(), prepared.n, w.l_max, sph.data_ptr(),
                                              dsph.data_ptr(), stream.cuda_stream, calls, ctypes.byref(seconds))
        if status != 0:
            raise RuntimeError(lib.sphx_last_error().decode())
        return seconds.value

    def from_python(step, calls):
        t0 = time.perf_counter()
        for _ in range(calls):
            step()
        return (time.perf_counter() - t0) / calls

    calculator = sphericart_torch.SphericalHarmonics(w.l_max)
    routes = {
        "sphx_forward_f64": lambda calls: in_c(0, calls),
        "sphericart_cuda_c_api": lambda calls: in_c(1, calls),
        "sphx_forward_f64_from_python": lambda calls: from_python(prepared.step, calls),
        "torch_op": lambda calls: from_python(lambda: calculator.compute_with_gradients(prepared.xyz), calls),
    }
    with torch.no_grad():
        for name, route in routes.items():
            route(200)
            bursts = []
            for _ in range(10):
                torch.cuda.synchronize()
                bursts.append(route(1000))
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            sustained = route(10_000)
            torch.cuda.synchronize()
            with_wait = (time.perf_counter() - t0) / 10_000
            result[name] = {"burst": statistics.median(bursts) * 1e6, "sustained": sustained * 1e6,
                            "gpu": with_wait * 1e6}
    del prepared
    torch.cuda.empty_cache()
    return result


def measure(prepared, steps, settle_seconds, warmup):
    settle(prepared.step, settle_seconds, warmup)
    wall, device_ms = time_back_to_back(prepared.step, steps, prepared.stream)
    launch_ms = time_each_launch(prepared.step, steps, prepared.stream)
    return wall, roofline_of(device_ms, steps, launch_ms, prepared.bytes_per_launch)


def measure_config(lib, name, steps, settle_seconds, with_cold, yardsticks):
    """One of the benchmark configurations next to the headline: per-launch event times with the
    outputs in place and, for the small ones, rotating through 1 GB of output buffers."""
    import torch

    from sphericart_amd.workloads import WORKLOADS

    w = WORKLOADS[name]
    steps = max(steps, 50)
    prepared = Prepared(lib, w)
    wall, entry = measure(prepared, steps, settle_seconds, 10)
    entry.update({
        "workload": f"{w.name}: {w.description}",
        "dtype": w.dtype,
        "kernels": prepared.kernels(),
        "launches_timed": steps,
        "points_per_s": w.n_samples * steps / wall,
        "traffic": measured_traffic(name, prepared.kernels()),
    })
    with_floor(entry, yardsticks, prepared.bytes_per_launch)
    del prepared
    torch.cuda.empty_cache()
    if with_cold:
        cold = Prepared(lib, w, rotate_mb=1024)
        _, r = measure(cold, steps, settle_seconds, 10)
        entry["cold"] = {"rotate_mb": 1024, "output_buffers": len(cold.outputs), "avg_launch_us": r["avg_launch_us"],
                         "achieved": r["achieved"], "frac": r["frac"], "per_launch_events": r["per_launch_events"]}
        del cold
        torch.cuda.empty_cache()
    return entry


def main():
    args = parse()
    if args.gpus != 1:
        print(
            "bench.py measures one GPU: the evaluator shards by giving each GPU its own slice of "
            "points and needs no exchange, so there is no multi-GPU figure to report (--gpus 1 only).",
            file=sys.stderr,
        )
        return 2

    import torch

    import sphericart_amd
    from sphericart_amd.workloads import WORKLOADS

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    w = WORKLOADS[args.workload]
    lib = sphericart_amd.get_library()
    torch.cuda.set_device(0)
    if args.sweep:
        return sweep(lib, args)

    prepared = Prepared(lib, w, args.rotate_mb if args.op == "forward" else 0)
    xyz_host, xyz = prepared.xyz_host, prepared.xyz
    n, ny, mode, opts, stream = prepared.n, prepared.ny, prepared.mode, prepared.opts, prepared.stream
    sph, dsph, ddsph = prepared.outputs[0]
    step = prepared.step
    bytes_per_launch = prepared.bytes_per_launch

    if args.op == "backward":
        if mode < 1:
            print("--op backward needs a workload with gradients", file=sys.stderr)
            return 2
        step()  # fill dsph
        torch.manual_seed(w.seed)
        sph_grad = torch.randn((n, ny), **opts)
        xyz_grad = torch.empty((n, 3), **opts)
        backward = lib.sphx_backward_f32 if w.dtype == "f32" else lib.sphx_backward_f64
        backward_args = (dsph.data_ptr(), sph_grad.data_ptr(), n, ny, xyz_grad.data_ptr(), 0, stream.cuda_stream)

        def step():  # noqa: F811
            status = backward(*backward_args)
            if status != 0:
                raise RuntimeError(lib.sphx_last_error().decode())

        # reads dsph and sph_grad once, writes three numbers per point
        bytes_per_launch = xyz.element_size() * n * (4 * ny + 3)

    if args.op == "vjp":
        if mode != 1:
            print("--op vjp needs a workload with gradients and no Hessians", file=sys.stderr)
            return 2
        torch.manual_seed(w.seed)
        sph_grad = torch.randn((n, ny), **opts)
        xyz_grad = torch.empty((n, 3), **opts)
        fused = lib.sphx_vjp_f32 if w.dtype == "f32" else lib.sphx_vjp_f64
        fused_args = (xyz.data_ptr(), sph_grad.data_ptr(), n, w.l_max, int(w.normalized),
                      xyz_grad.data_ptr(), 0, stream.cuda_stream)

        def step():  # noqa: F811
            status = fused(*fused_args)
            if status != 0:
                raise RuntimeError(lib.sphx_last_error().decode())

        # reads xyz and sph_grad, writes xyz_grad
        bytes_per_launch = xyz.element_size() * n * (3 + ny + 3)

    if args.calibrate_copy:
        nbytes = w.bytes_per_point * n
        src = torch.zeros(nbytes // 4, dtype=torch.float32, device=xyz.device)
        dst = torch.empty_like(src)
        for _ in range(args.warmup):
            dst.copy_(src)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            dst.copy_(src)
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        print(json.dumps({
            "calibration": "device-to-device copy", "bytes_read_per_launch": src.numel() * 4,
            "bytes_written_per_launch": src.numel() * 4, "steps": args.steps,
            "us_per_launch": wall / args.steps * 1e6,
        }))
        return 0

    settle(step, args.settle_seconds, args.warmup)
    # the timed region: K steps back to back
    wall, device_ms = time_back_to_back(step, args.steps, stream)
    # the single launch: K more steps, an event pair around each
    roofline = roofline_of(device_ms, args.steps, time_each_launch(step, args.steps, stream), bytes_per_launch)
    roofline["traffic"] = measured_traffic(args.workload if args.op == "forward" else f"{args.workload}:{args.op}",
                                           prepared.kernels() if args.op == "forward" else None)
    headline = args.workload == "cfg3" and args.op == "forward" and args.rotate_mb == 0

    result = {
        "metric": "points/sec + achieved HBM GB/s (% peak), l_max=6 fp32 w/ gradients, 1M pts"
        if args.workload == "cfg3" and args.op == "forward"
        else f"points/sec + achieved HBM GB/s (% peak), {args.op} pass, {w.description}",
        "value": n * args.steps / wall,
        "unit": "points/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": wall / args.steps * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": w.dtype,
        "data": "synthetic",
        "config": {
            "workload": f"{w.name}: {w.description}",
            "op": args.op,
            "rotate_mb": args.rotate_mb,
            "settle_seconds": args.settle_seconds,
            "l_max": w.l_max,
            "n_samples": n,
            "derivatives": w.derivatives,
            "harmonics": "spherical" if w.normalized else "solid",
            "seed": w.seed,
            "kernels": prepared.kernels() if args.op == "forward" else None,
        },
        "roofline": roofline,
    }
    if not args.no_cpu_baseline:
        if args.op == "forward":
            result["cpu_baseline"] = cpu_baseline(w, xyz_host)
        elif args.op == "vjp":
            result["cpu_baseline"] = cpu_vjp_baseline(w, xyz_host, sph_grad.cpu().numpy())
        else:
            result["cpu_baseline"] = cpu_backward_baseline(dsph.cpu().numpy(), sph_grad.cpu().numpy())
    if headline and not args.no_by_config:
        cold = Prepared(lib, w, rotate_mb=1024)
        _, r = measure(cold, max(args.steps, 50), args.settle_seconds, 10)
        result["roofline"]["cold"] = {
            "rotate_mb": 1024, "output_buffers": len(cold.outputs), "avg_launch_us": r["avg_launch_us"],
            "achieved": r["achieved"], "frac": r["frac"], "per_launch_events": r["per_launch_events"],
        }
        del cold, prepared, sph, dsph, ddsph
        torch.cuda.empty_cache()
        yardsticks = measure_yardsticks(lib, stream)
        result["yardsticks"] = yardsticks
        with_floor(result["roofline"], yardsticks, bytes_per_launch)
        result["roofline_by_config"] = {
            name: measure_config(lib, name, args.steps, args.settle_seconds, name in ("cfg1", "cfg2"), yardsticks)
            for name in ("cfg1", "cfg2", "cfg4", "cfg5")
        }
        result["host_us_per_call"] = host_cost(lib, stream)
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
