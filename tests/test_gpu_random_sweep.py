"""Seeded random configurations of the extended dispatch + combine calls: shape, payload, capacity limit, tile size and
schedule are drawn per seed, two layers run through the same buffers, and every output is compared bit for bit with the
CPU oracle (the comparison itself is `run_and_check` of the full-size flag tests).  The draws reach kernel geometries
the fixed shapes leave out: quantised rows of 8192 and 16384 columns (two and four 16-byte vectors per lane in the
quantised reduce), rows that are not a multiple of 16 bytes (the element-granular kernels) and tiles larger than the
whole dispatch.
"""
import numpy as np
import pytest

from test_gpu_flags_full_size import Layers, run_and_check
from tilexr_amd import workloads

pytestmark = pytest.mark.gpu

WIDTHS_ANY = [8, 40, 64, 136, 1000, 1024, 2048, 4096, 7168, 8192, 12288, 16384]
WIDTHS_QUANT = [64, 128, 1024, 2048, 4096, 7168, 8192, 16384]


def draw(seed):
    rng = np.random.default_rng(1000 + seed)
    quant = ["none", "int8", "fp8_block128"][seed % 3]
    h = int(rng.choice(WIDTHS_QUANT if quant != "none" else WIDTHS_ANY))
    top_k = int(rng.integers(1, 9))
    experts = int(rng.integers(top_k, 257))
    # enough routes for the count + scatter kernels (the single-launch dispatch is for 2048 routes and fewer, without
    # flags); wide rows get fewer tokens so that the oracle stays quick
    bs = int(rng.integers(1, 64)) if seed % 7 == 0 else int(rng.integers(300, 1400 if h <= 4096 else 500))
    routing = ["uniform", "zipf", "gating"][int(rng.integers(0, 3))]
    capacity_factor = float(rng.choice([0.0, 0.0, 0.6, 1.25]))
    x_dist = ["normal", "normal2", "student_t3"][int(rng.integers(0, 3))]
    w = workloads.Workload(f"sweep{seed}", 1, bs, h, top_k, experts, x_dist=x_dist, routing=routing, zipf_s=1.1,
                           quant=quant, capacity_factor=capacity_factor, seed=5000 + seed)
    tile_rows = int(rng.choice([1, 7, 16, 64, 100, 1 << 20]))
    two_streams = bool(rng.integers(0, 2))
    return w, tile_rows, two_streams


@pytest.mark.parametrize("seed", range(24))
def test_random_configuration(seed):
    w, tile_rows, two_streams = draw(seed)
    print(f"sweep seed={seed}: bs={w.bs} h={w.h} top_k={w.top_k} experts={w.experts} quant={w.quant} "
          f"capacity={w.capacity} routing={w.routing} tile_rows={tile_rows} two_streams={two_streams}", flush=True)
    run_and_check(Layers(w), tile_rows, two_streams)
