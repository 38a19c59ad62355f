"""What a user of the reference sees when switching: the deviation of the GPU results from the
reference CPU library *as its own build system compiles it* (-O3 with FMA contraction,
``oracle/_ref/libsphx_ref_fma.so``), for the five benchmark configurations at full size, next to
the same figures for the reference against itself built with and without contraction (the
control). The GPU library follows the reference's operation order without contraction, so its
deviation from the contracted build must not exceed what the reference's two builds differ by.

Per array: max |a - b| / max(1, |b|); entries outside the literal rule (|a - b| <= tol |b| or
<= tol, tol = 1e-5 float32 / 1e-12 float64, python/tests/test_cupy.py:22-49); entries outside
the block-scale rule (|a - b| <= tol max(|b|, S), S the largest magnitude in the entry's
(point, component, l) block); entries that are non-finite in exactly one of the two.
"""

import json

import numpy as np
import pytest
import torch

from gpu_utils import announce, run_launch_layer
from sphericart_amd.workloads import WORKLOADS

pytestmark = pytest.mark.gpu

TOL = {"f32": 1e-5, "f64": 1e-12}


class Deviation:
    def __init__(self):
        self.entries = self.literal = self.block = self.nonfinite_mismatch = self.nonfinite = 0
        self.max_err = 0.0

    def add(self, a, b, l_max, tol):
        """a against b; arrays [..., (l_max+1)^2]."""
        fa, fb = np.isfinite(a), np.isfinite(b)
        both = fa & fb
        self.entries += a.size
        self.nonfinite += int((~fb).sum())
        self.nonfinite_mismatch += int((fa != fb).sum())
        with np.errstate(invalid="ignore", over="ignore"):
            diff = np.where(both, np.abs(a - b), 0.0)
            mag = np.where(both, np.abs(b), 0.0)
        self.max_err = max(self.max_err, float((diff / np.maximum(1.0, mag)).max()))
        self.literal += int(((diff > tol * mag) & (diff > tol)).sum())
        for l in range(l_max + 1):
            block = slice(l * l, (l + 1) * (l + 1))
            scale = mag[..., block].max(axis=-1, keepdims=True)
            self.block += int((diff[..., block] > tol * np.maximum(mag[..., block], scale)).sum())

    def row(self):
        return {"entries": self.entries, "max_err": self.max_err, "outside_literal": self.literal,
                "outside_block_scale": self.block, "nonfinite_in_reference": self.nonfinite,
                "nonfinite_in_one_only": self.nonfinite_mismatch}


@pytest.mark.parametrize("name", ["cfg1", "cfg2", "cfg3", "cfg4", "cfg5"])
def test_deviation_from_the_reference_as_built(oracle, library, name):
    if not (oracle.available("ref") and oracle.available("ref_fma")):
        pytest.skip("oracle/_ref was not built (needs the reference checkout at build time)")
    w = WORKLOADS[name]
    announce("parity report", name, w.description)
    xyz = w.points()
    status, out = run_launch_layer(library, torch.from_numpy(xyz).cuda(), w.l_max, w.normalized, w.derivatives)
    assert status == 0, library.sphx_last_error()
    torch.cuda.synchronize()
    gpu_dev, control = Deviation(), Deviation()
    labels = ("sph", "dsph", "ddsph")
    per_array = {label: (Deviation(), Deviation()) for label in labels}
    slab = max(1, min(w.n_samples, (128 << 20) // w.bytes_per_point))
    for first in range(0, w.n_samples, slab):
        last = min(w.n_samples, first + slab)
        with np.errstate(all="ignore"):
            built = oracle.compute(xyz[first:last], w.l_max, w.normalized, w.derivatives, flavour="ref_fma")
            strict = oracle.compute(xyz[first:last], w.l_max, w.normalized, w.derivatives, flavour="ref")
        for label, g, b, s in zip(labels, out, built, strict):
            if b is None:
                continue
            g = g[first:last].cpu().numpy()
            for dev, a in ((gpu_dev, g), (per_array[label][0], g), (control, s), (per_array[label][1], s)):
                dev.add(a, b, w.l_max, TOL[w.dtype])
    report = {"config": name, "tolerance": TOL[w.dtype], "gpu_vs_reference_as_built": gpu_dev.row(),
              "reference_strict_vs_as_built": control.row(),
              "by_array": {label: {"gpu": g.row(), "control": c.row()}
                           for label, (g, c) in per_array.items() if g.entries}}
    print("[parity report]", json.dumps(report), flush=True)
    g, c = gpu_dev.row(), control.row()
    assert g["nonfinite_in_one_only"] <= c["nonfinite_in_one_only"]
    assert g["max_err"] <= c["max_err"]
    assert g["outside_literal"] <= c["outside_literal"]
    assert g["outside_block_scale"] <= c["outside_block_scale"]
    # the block-scale rule is the one a comparison at this dynamic range can meet; the literal
    # rule fails for the reference against itself on cfg4 (values up to 1e12 next to nodes)
    if name in ("cfg1", "cfg2"):
        assert g["outside_literal"] == 0
