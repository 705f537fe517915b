"""Tile readiness flags at the sizes of the measured configurations: the headline workload (4096 tokens x 7168 bf16,
256 experts, top-8, Zipf) with dispatch publishing tiles and combine consuming them, one after the other on one
stream and side by side on two, and wide quantised rows.

These shapes select kernels the small flag tests do not reach: the per-route scatter with write-through stores and a
row cut into column slices (every slice reports its part of the row, so a row counts `slices` times towards its tile),
the whole-workgroup-per-token reduce with flag waits, and the quantised reduce with flag waits on rows wider than a
wave.  Every output is compared bit for bit with the CPU oracle, every readiness word with (epoch << 32) | rows in its
tile, and the same buffers carry two different layers in a row.
"""
import numpy as np
import pytest
import torch

from gpu_harness import DEV, Session, bits16
from oracle import ep as O
from tilexr_amd import ep, workloads

pytestmark = pytest.mark.gpu

QUANT = {"none": ep.Q_NONE, "int8": ep.Q_TOKEN_INT8, "fp8_block128": ep.Q_FP8_BLOCK128}
OQUANT = {"none": O.Q_NONE, "int8": O.Q_TOKEN_INT8, "fp8_block128": O.Q_FP8_BLOCK128}


def oracle_layer(w, x, ids, weights):
    quant = OQUANT[w.quant]
    case = O.Case(1, w.bs, w.h, w.top_k, w.experts, dtype=O.DT_BF16, quant_mode=quant, capacity=w.capacity,
                  token_nums_type=1)
    want = O.mem_dispatch(case, 0, bits16(x)[None], ids.numpy()[None])
    eo = want["expand_x"][None] if quant else want["expand_x"].view(np.uint16)[None]
    want["y"] = O.mem_combine(O.Case(1, w.bs, w.h, w.top_k, w.experts, dtype=O.DT_BF16), 0, eo, want["assist"][None],
                              want["send_counts"][None], expert_scales=weights.numpy(), in_quant=quant,
                              in_scales=want["dyn_scales"] if quant else None)
    return want


class Layers:
    """Two layers of one workload (the second with its token rows in reverse order and other routing) + their oracle
    results, computed once per workload."""

    def __init__(self, w):
        self.w = w
        x = workloads.make_x(w)
        ids, weights = workloads.make_routing(w)
        w2 = workloads.Workload(w.name, w.ranks, w.bs, w.h, w.top_k, w.experts, w.x_dist, w.routing, w.zipf_s, w.quant,
                                w.capacity_factor, w.seed + 1)
        ids2, weights2 = workloads.make_routing(w2)
        self.inputs = [(x, ids, weights), (x.flip(0).contiguous(), ids2, weights2)]
        self.want = [oracle_layer(w, *layer) for layer in self.inputs]


_layers = {}


def layers_of(w):
    if w.name not in _layers:
        _layers[w.name] = Layers(w)
    return _layers[w.name]


def run_and_check(L, tile_rows, two_streams, expect_scatter=None, expect_reduce=None):
    w = L.w
    bs, h, K, E = w.bs, w.h, w.top_k, w.experts
    quant = QUANT[w.quant]
    n = bs * K
    row_bytes = h * 2 if quant == ep.Q_NONE else h
    tiles = (n + tile_rows - 1) // tile_rows
    with Session() as s:
        side = torch.cuda.Stream()
        expand_x = torch.full((n, row_bytes), 0x5a, dtype=torch.uint8, device=DEV)
        assist = torch.full((n, 4), -77, dtype=torch.int32, device=DEV)
        token_nums = torch.zeros((E,), dtype=torch.int64, device=DEV)
        send_counts = torch.zeros((E,), dtype=torch.int32, device=DEV)
        row_map = torch.full((bs, K), -9, dtype=torch.int32, device=DEV)
        y = torch.full((bs, h), 5.0, dtype=torch.bfloat16, device=DEV)
        scales = None
        if quant == ep.Q_TOKEN_INT8:
            scales = torch.full((n, 1), -3.0, dtype=torch.float32, device=DEV)
        elif quant == ep.Q_FP8_BLOCK128:
            scales = torch.full((n, (h + 127) // 128), -3.0, dtype=torch.float32, device=DEV)
        flags = torch.zeros((tiles,), dtype=torch.int64, device=DEV)          # never cleared between the layers
        status = torch.zeros((1,), dtype=torch.int32, device=DEV)
        meta_ready, consumed = ep.HipEvent(), ep.HipEvent()
        epochs = []
        for layer, ((x, ids, weights), want) in enumerate(zip(L.inputs, L.want)):
            d_x, d_ids, d_w = x.to(DEV), ids.to(DEV), weights.to(DEV)
            torch.cuda.synchronize()
            print(f"flags full size: {w.name} tile_rows={tile_rows} two_streams={two_streams} layer={layer}", flush=True)
            st, epoch = ep.dispatch_memory_ex(d_x, d_ids, s.comm, bs, h, K, E, expand_x, assist, token_nums,
                                              send_counts, ep.DT_BF16, s.stream, quant_mode=quant,
                                              expert_capacity=w.capacity, dynamic_scales=scales, row_index_map=row_map,
                                              tile_flags=flags, tile_rows=tile_rows,
                                              meta_ready_event=meta_ready.value if two_streams else None)
            assert st == 0 and epoch > 0
            epochs.append(epoch)
            consumer = side if two_streams else s.stream
            if two_streams:
                meta_ready.wait_on(side)
            st = ep.combine_memory_ex(expand_x, assist, send_counts, s.comm, bs, h, K, E, y, ep.DT_BF16, consumer,
                                      expert_out_quant_mode=quant, expert_out_scales=scales, expert_scales=d_w,
                                      row_index_map=row_map, tile_flags=flags, tile_rows=tile_rows, flag_epoch=epoch,
                                      wait_timeout_us=5_000_000, device_status=status)
            assert st == 0
            if two_streams:
                consumed.record(side)
                consumed.wait_on(s.stream)
            s.sync()
            side.synchronize()
            assert status.item() == 0, "a flag wait expired"
            if expect_scatter:
                assert ep.last_kernel_name(s.comm, ep.K_SCATTER) == expect_scatter
            if expect_reduce:
                assert ep.last_kernel_name(s.comm, ep.K_REDUCE) == expect_reduce
            rows = want["rows"]
            assert np.array_equal(send_counts.cpu().numpy(), want["send_counts"]), f"layer {layer}"
            assert np.array_equal(token_nums.cpu().numpy(), want["expert_token_nums"]), f"layer {layer}"
            assert np.array_equal(assist.cpu().numpy()[:rows], want["assist"][:rows]), f"layer {layer}"
            assert np.array_equal(expand_x.cpu().numpy()[:rows], want["expand_x"][:rows]), f"layer {layer}"
            if quant:
                got_s = scales.cpu().numpy()[:rows]
                assert np.array_equal(got_s.reshape(rows, -1), want["dyn_scales"][:rows].reshape(rows, -1))
            assert np.array_equal(bits16(y), want["y"]), f"layer {layer}"
            # every tile that holds rows ends at (epoch << 32) | rows in the tile; tiles past the kept rows keep
            # whatever they held before
            f = flags.cpu().numpy().astype(np.uint64)
            live = (rows + tile_rows - 1) // tile_rows
            rows_in_tile = np.minimum(tile_rows, rows - np.arange(live) * tile_rows)
            assert np.array_equal(f[:live] >> np.uint64(32), np.full(live, epoch, np.uint64)), f"layer {layer}"
            assert np.array_equal(f[:live] & np.uint64(0xffffffff), rows_in_tile.astype(np.uint64)), f"layer {layer}"
        assert epochs[1] > epochs[0]
        meta_ready.destroy()
        consumed.destroy()


@pytest.mark.parametrize("two_streams", [False, True], ids=["one_stream", "two_streams"])
@pytest.mark.parametrize("tile_rows", [8, 64, 1024])
def test_headline_workload_with_tile_flags(tile_rows, two_streams):
    run_and_check(layers_of(workloads.CONFIGS["C3"]), tile_rows, two_streams,
                  expect_scatter="ep_scatter_route_kernel", expect_reduce="ep_reduce_vec_kernel")


@pytest.mark.parametrize("two_streams", [False, True], ids=["one_stream", "two_streams"])
def test_wide_quantised_rows_with_tile_flags(two_streams):
    # int8 rows of 4096 columns (the quantised reduce with a whole workgroup per token) ...
    c4 = workloads.scaled(workloads.CONFIGS["C4"], 2048, name="C4@2048")
    run_and_check(layers_of(c4), 64, two_streams, expect_scatter="ep_scatter_vec_kernel",
                  expect_reduce="ep_reduce_quant_kernel")
    # ... and fp8 rows of 7168 columns with 56 block scales per row, a capacity limit, tiles of 100 rows
    wide = workloads.Workload("fp8@7168", 1, 1536, 7168, 8, 64, x_dist="student_t3", routing="zipf", zipf_s=1.2,
                              quant="fp8_block128", capacity_factor=1.25, seed=99)
    run_and_check(layers_of(wide), 100, two_streams, expect_scatter="ep_scatter_vec_kernel",
                  expect_reduce="ep_reduce_quant_kernel")


@pytest.mark.parametrize("two_streams", [False, True], ids=["one_stream", "two_streams"])
def test_rows_wider_than_one_publishing_workgroup(two_streams):
    """Rows of 1536 vectors: the publishing per-route scatter cuts them into two workgroups of 512 lanes, each of which
    reports its part of the row, so a row counts twice towards its tile (the headline rows fit one such workgroup)."""
    wide = workloads.Workload("bf16@12288", 1, 1024, 12288, 4, 32, x_dist="normal", routing="zipf", zipf_s=1.0, seed=77)
    run_and_check(layers_of(wide), 100, two_streams, expect_scatter="ep_scatter_route_kernel",
                  expect_reduce="ep_reduce_vec_kernel")


@pytest.mark.parametrize("tile_rows", [1, 7, 64, 1 << 20])
@pytest.mark.parametrize("capacity_factor", [0.0, 0.8], ids=["no_limit", "capacity"])
def test_decode_sized_dispatch_publishes_tiles_from_its_single_launch(capacity_factor, tile_rows):
    """At most 2048 routes: dispatch is one launch (a workgroup per route, or per token when a capacity limit needs the
    per-expert histogram), and with flags on one stream it stays one launch: the rows are written through and reported
    landed by the same kernel.  Outputs, combine result and every readiness word against the oracle, two layers through
    the same buffers."""
    w = workloads.Workload(f"decode@{capacity_factor}", 1, 128, 7168, 8, 256, x_dist="normal", routing="gating",
                           capacity_factor=capacity_factor, seed=11)
    run_and_check(layers_of(w), tile_rows, False,
                  expect_scatter="ep_dispatch_small_kernel" if capacity_factor else "ep_dispatch_small_route_kernel",
                  expect_reduce="ep_reduce_vec_kernel")


def test_two_communicators_share_one_flag_array():
    """Flag epochs come from one counter for the whole process: two communicators that are handed the same flag array
    one after the other can never tag it with the same value, so words left by the first read as not ready to a
    consumer of the second."""
    bs, h, K, E, tile_rows = 512, 1024, 4, 32, 32
    rng = np.random.default_rng(3)
    n = bs * K
    tiles = n // tile_rows
    flags = torch.zeros((tiles,), dtype=torch.int64, device=DEV)
    seen = []
    for round_ in range(3):                       # a fresh communicator every round: its own magic restarts at 1
        with Session() as s:
            ids = np.stack([rng.permutation(E)[:K] for _ in range(bs)]).astype(np.int32)
            x = torch.from_numpy(rng.standard_normal((bs, h)).astype(np.float32)).to(torch.bfloat16)
            d_x, d_ids = x.to(DEV), torch.from_numpy(ids).to(DEV)
            expand_x = torch.zeros((n, h * 2), dtype=torch.uint8, device=DEV)
            assist = torch.zeros((n, 4), dtype=torch.int32, device=DEV)
            token_nums = torch.zeros((E,), dtype=torch.int64, device=DEV)
            counts = torch.zeros((E,), dtype=torch.int32, device=DEV)
            torch.cuda.synchronize()
            before = flags.cpu().numpy().astype(np.uint64) >> np.uint64(32)
            st, epoch = ep.dispatch_memory_ex(d_x, d_ids, s.comm, bs, h, K, E, expand_x, assist, token_nums, counts,
                                              ep.DT_BF16, s.stream, tile_flags=flags, tile_rows=tile_rows)
            assert st == 0
            s.sync()
            assert epoch not in seen and epoch != 0 and not np.any(before == epoch)
            seen.append(epoch)
            after = flags.cpu().numpy().astype(np.uint64) >> np.uint64(32)
            assert np.all(after == epoch)
    assert seen == sorted(seen)
