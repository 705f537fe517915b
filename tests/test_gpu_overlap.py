"""Tile readiness flags: combine on one stream consuming rows while dispatch on another stream is still writing them,
and the bounded wait that ends a combine whose producer never shows up.

No kernel here is allowed to wait forever: the flag wait has a wall-clock bound and reports through a device word.
"""
import numpy as np
import pytest
import torch

from gpu_harness import DEV, Session, alloc_dispatch_outputs, bits16, to_dev
from oracle import ep as O
from tilexr_amd import ep

pytestmark = pytest.mark.gpu


def routing(rng, bs, K, E):
    ids = np.stack([rng.permutation(E)[:K] for _ in range(bs)]).astype(np.int32)
    w = rng.random((bs, K)).astype(np.float32)
    return ids, w


@pytest.mark.parametrize("shape,tile_rows", [((64, 256, 4, 16), 8), ((2048, 2048, 8, 64), 128), ((777, 1024, 6, 32), 100)])
def test_combine_overlapped_with_dispatch_through_tile_flags(shape, tile_rows):
    bs, h, K, E = shape
    rng = np.random.default_rng(sum(shape))
    n = bs * K
    tiles = (n + tile_rows - 1) // tile_rows
    with Session() as s:
        side = torch.cuda.Stream()
        flags = torch.zeros((tiles,), dtype=torch.int64, device=DEV)     # never cleared between rounds
        status = torch.zeros((1,), dtype=torch.int32, device=DEV)
        meta_ready = ep.HipEvent()
        epochs = []
        for round_ in range(4):
            ids, w = routing(rng, bs, K, E)
            x = torch.from_numpy(rng.standard_normal((bs, h)).astype(np.float32)).to(torch.bfloat16)
            xb = bits16(x)
            d_x, d_ids, d_w = x.to(DEV), to_dev(ids), to_dev(w)
            out = alloc_dispatch_outputs(bs, h, K, E)
            counts = torch.zeros((E,), dtype=torch.int32, device=DEV)
            y = torch.full((bs, h), 3.0, dtype=torch.bfloat16, device=DEV)
            torch.cuda.synchronize()
            st, epoch = ep.dispatch_memory_ex(d_x, d_ids, s.comm, bs, h, K, E, out["expand_x"], out["assist"],
                                              out["token_nums"], counts, ep.DT_BF16, s.stream,
                                              row_index_map=out["row_map"], tile_flags=flags, tile_rows=tile_rows,
                                              meta_ready_event=meta_ready.value)
            assert st == 0 and epoch > 0
            epochs.append(epoch)
            # the consumer may start once counts, row map and the re-armed flag words are enqueued
            meta_ready.wait_on(side)
            st = ep.combine_memory_ex(out["expand_x"], out["assist"], counts, s.comm, bs, h, K, E, y, ep.DT_BF16, side,
                                      expert_scales=d_w, row_index_map=out["row_map"], tile_flags=flags,
                                      tile_rows=tile_rows, flag_epoch=epoch, wait_timeout_us=5_000_000,
                                      device_status=status)
            assert st == 0
            s.sync()
            side.synchronize()
            assert status.item() == 0
            case = O.Case(1, bs, h, K, E, token_nums_type=1)
            want = O.mem_dispatch(case, 0, xb[None], ids[None])
            assert np.array_equal(out["expand_x"].cpu().numpy(), want["expand_x"])
            wy = O.mem_combine(case, 0, want["expand_x"].view(np.uint16)[None], want["assist"][None],
                               want["send_counts"][None], expert_scales=w)
            assert np.array_equal(bits16(y), wy)
            # every tile ends at (epoch << 32) | rows in the tile
            f = flags.cpu().numpy().astype(np.uint64)
            rows_in_tile = np.minimum(tile_rows, n - np.arange(tiles) * tile_rows)
            assert np.array_equal(f >> np.uint64(32), np.full(tiles, epoch, np.uint64))
            assert np.array_equal(f & np.uint64(0xffffffff), rows_in_tile.astype(np.uint64))
        assert epochs == sorted(set(epochs))
        meta_ready.destroy()


@pytest.mark.parametrize("quant", ["none", "int8", "fp8_block128"])
def test_overlap_on_reused_buffers_never_reads_a_previous_round(quant):
    """The same output buffers carry five different layers in a row, the consumer starts as early as it can and the
    tiles are small, so rows are read a moment after another compute unit wrote them: a row served from a cache that
    still holds the previous layer, or read before its stores have landed, shows up as a bit difference."""
    bs, h, K, E, tile_rows = 4096, 2048, 8, 64, 8
    qmode = {"none": ep.Q_NONE, "int8": ep.Q_TOKEN_INT8, "fp8_block128": ep.Q_FP8_BLOCK128}[quant]
    oq = {"none": O.Q_NONE, "int8": O.Q_TOKEN_INT8, "fp8_block128": O.Q_FP8_BLOCK128}[quant]
    rng = np.random.default_rng(4242 + qmode)
    n = bs * K
    tiles = (n + tile_rows - 1) // tile_rows
    with Session() as s:
        side = torch.cuda.Stream()
        flags = torch.zeros((tiles,), dtype=torch.int64, device=DEV)
        status = torch.zeros((1,), dtype=torch.int32, device=DEV)
        meta_ready, consumed = ep.HipEvent(), ep.HipEvent()
        out = alloc_dispatch_outputs(bs, h, K, E, quant=qmode)
        counts = torch.zeros((E,), dtype=torch.int32, device=DEV)
        y = torch.zeros((bs, h), dtype=torch.bfloat16, device=DEV)
        for round_ in range(5):
            ids, w = routing(rng, bs, K, E)
            x = torch.from_numpy((rng.standard_normal((bs, h)) * (1 + round_)).astype(np.float32)).to(torch.bfloat16)
            xb = bits16(x)
            d_x, d_ids, d_w = x.to(DEV), to_dev(ids), to_dev(w)
            torch.cuda.synchronize()
            st, epoch = ep.dispatch_memory_ex(d_x, d_ids, s.comm, bs, h, K, E, out["expand_x"], out["assist"],
                                              out["token_nums"], counts, ep.DT_BF16, s.stream, quant_mode=qmode,
                                              dynamic_scales=out["scales"], row_index_map=out["row_map"],
                                              tile_flags=flags, tile_rows=tile_rows, meta_ready_event=meta_ready.value)
            assert st == 0
            meta_ready.wait_on(side)
            st = ep.combine_memory_ex(out["expand_x"], out["assist"], counts, s.comm, bs, h, K, E, y, ep.DT_BF16, side,
                                      expert_out_quant_mode=qmode, expert_out_scales=out["scales"], expert_scales=d_w,
                                      row_index_map=out["row_map"], tile_flags=flags, tile_rows=tile_rows,
                                      flag_epoch=epoch, wait_timeout_us=5_000_000, device_status=status)
            assert st == 0
            consumed.record(side)
            consumed.wait_on(s.stream)
            s.sync()
            side.synchronize()
            assert status.item() == 0
            case = O.Case(1, bs, h, K, E, dtype=O.DT_BF16, quant_mode=oq, token_nums_type=1)
            want = O.mem_dispatch(case, 0, xb[None], ids[None])
            assert np.array_equal(out["expand_x"].cpu().numpy(), want["expand_x"]), f"round {round_}"
            eo = want["expand_x"][None] if oq else want["expand_x"].view(np.uint16)[None]
            wy = O.mem_combine(O.Case(1, bs, h, K, E, dtype=O.DT_BF16), 0, eo, want["assist"][None],
                               want["send_counts"][None], expert_scales=w, in_quant=oq,
                               in_scales=want["dyn_scales"] if oq else None)
            assert np.array_equal(bits16(y), wy), f"round {round_}"
        meta_ready.destroy()
        consumed.destroy()


def test_flag_wait_expires_instead_of_hanging():
    bs, h, K, E = 256, 512, 4, 16
    rng = np.random.default_rng(9)
    ids, w = routing(rng, bs, K, E)
    x = torch.from_numpy(rng.standard_normal((bs, h)).astype(np.float32)).to(torch.bfloat16)
    with Session() as s:
        d_x, d_ids = x.to(DEV), to_dev(ids)
        out = alloc_dispatch_outputs(bs, h, K, E)
        counts = torch.zeros((E,), dtype=torch.int32, device=DEV)
        st, _ = ep.dispatch_memory_ex(d_x, d_ids, s.comm, bs, h, K, E, out["expand_x"], out["assist"],
                                      out["token_nums"], counts, ep.DT_BF16, s.stream, row_index_map=out["row_map"])
        assert st == 0
        s.sync()
        tile_rows = 32
        flags = torch.zeros(((bs * K + tile_rows - 1) // tile_rows,), dtype=torch.int64, device=DEV)   # nobody sets them
        status = torch.zeros((1,), dtype=torch.int32, device=DEV)
        y = torch.full((bs, h), 3.0, dtype=torch.bfloat16, device=DEV)
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        with torch.cuda.stream(s.stream):
            start.record()
            st = ep.combine_memory_ex(out["expand_x"], out["assist"], counts, s.comm, bs, h, K, E, y, ep.DT_BF16,
                                      s.stream, row_index_map=out["row_map"], tile_flags=flags, tile_rows=tile_rows,
                                      flag_epoch=4242, wait_timeout_us=2000, device_status=status)
            stop.record()
        assert st == 0
        s.sync()
        assert status.item() == 1                       # reported, not hung
        assert start.elapsed_time(stop) < 500.0          # milliseconds: about one timeout, not one per tile
        # rows whose tile never became ready contribute nothing
        assert np.all(bits16(y) == 0)
    # a bad timeout is rejected on the host
    with Session() as s:
        st = ep.combine_memory_ex(out["expand_x"], out["assist"], counts, s.comm, bs, h, K, E, y, ep.DT_BF16, s.stream,
                                  tile_flags=flags, tile_rows=0)
        assert st == ep.ERR_PARA_CHECK_FAIL


@pytest.mark.parametrize("h", [1024, 1020])
@pytest.mark.parametrize("quant", ["none", "int8"])
def test_missing_word_after_a_same_stream_dispatch_gives_zero_tokens_at_once(quant, h):
    """Combine on the stream of the dispatch that published the flags does not wait (the producer is done before it
    starts); a word that is not there then (here: wiped between the two calls) can never come, so the tokens that need
    that tile get rows of zeros and the status word is set, without the wait bound being sat out, and every other token
    still equals the oracle.  1020 columns take the element-granular reduce, whose waits are blocking ones."""
    bs, K, E, tile_rows = 512, 4, 32, 32
    rng = np.random.default_rng(21)
    ids, w = routing(rng, bs, K, E)
    x = torch.from_numpy(rng.standard_normal((bs, h)).astype(np.float32)).to(torch.bfloat16)
    q = ep.Q_TOKEN_INT8 if quant == "int8" else ep.Q_NONE
    oq = O.Q_TOKEN_INT8 if quant == "int8" else O.Q_NONE
    case = O.Case(1, bs, h, K, E, dtype=O.DT_BF16, quant_mode=oq, token_nums_type=1)
    want = O.mem_dispatch(case, 0, bits16(x)[None], ids[None])
    eo = want["expand_x"][None] if oq else want["expand_x"].view(np.uint16)[None]
    want_y = O.mem_combine(O.Case(1, bs, h, K, E, dtype=O.DT_BF16), 0, eo, want["assist"][None],
                           want["send_counts"][None], expert_scales=w, in_quant=oq,
                           in_scales=want["dyn_scales"] if oq else None)
    n = bs * K
    wiped = [3, 17]
    with Session() as s:
        d_x, d_ids, d_w = x.to(DEV), to_dev(ids), to_dev(w)
        out = alloc_dispatch_outputs(bs, h, K, E, quant=q)
        counts = torch.zeros((E,), dtype=torch.int32, device=DEV)
        flags = torch.zeros((n // tile_rows,), dtype=torch.int64, device=DEV)
        status = torch.zeros((1,), dtype=torch.int32, device=DEV)
        y = torch.full((bs, h), 3.0, dtype=torch.bfloat16, device=DEV)
        st, epoch = ep.dispatch_memory_ex(d_x, d_ids, s.comm, bs, h, K, E, out["expand_x"], out["assist"],
                                          out["token_nums"], counts, ep.DT_BF16, s.stream, quant_mode=q,
                                          dynamic_scales=out.get("scales"), row_index_map=out["row_map"],
                                          tile_flags=flags, tile_rows=tile_rows)
        assert st == 0
        flags[wiped] = 0                                   # on the session's stream, between the two calls
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        st = ep.combine_memory_ex(out["expand_x"], out["assist"], counts, s.comm, bs, h, K, E, y, ep.DT_BF16, s.stream,
                                  expert_out_quant_mode=q, expert_out_scales=out.get("scales"), expert_scales=d_w,
                                  row_index_map=out["row_map"], tile_flags=flags, tile_rows=tile_rows, flag_epoch=epoch,
                                  wait_timeout_us=30_000_000, device_status=status)
        stop.record()
        assert st == 0
        s.sync()
        assert status.item() == 1
        assert start.elapsed_time(stop) < 1000.0           # milliseconds: nowhere near the 30 s bound
        row_map = out["row_map"].cpu().numpy()
        hit = np.isin(row_map // tile_rows, wiped).any(axis=1) & (row_map >= 0).any(axis=1)
        assert 0 < hit.sum() < bs
        got = bits16(y)
        assert np.all(got[hit] == 0)
        assert np.array_equal(got[~hit], want_y[~hit])


def test_combine_follows_an_expert_stage_that_publishes_tiles_in_random_order():
    """The producer here is not the dispatch but an "expert stage" written with torch ops on a second stream: it
    rewrites the rows tile by tile in a random order and stores a tile's readiness word after the tile's rows (a
    kernel boundary on one stream is a release at device scope).  The producer's stream starts with a few milliseconds
    of other work, so a combine that runs beside it really waits; it must return the weighted sum of the rewritten
    rows, never of the rows the buffer held before.  The producer is enqueued first: two streams of a process can share
    a hardware queue, and a waiting kernel at the head of that queue would keep the kernels it waits for behind it."""
    bs, h, K, E, tile_rows = 2048, 1024, 4, 32, 128
    rng = np.random.default_rng(31)
    n = bs * K
    tiles = (n + tile_rows - 1) // tile_rows
    with Session() as s:
        producer = torch.cuda.Stream()
        ids, w = routing(rng, bs, K, E)
        x = torch.from_numpy(rng.standard_normal((bs, h)).astype(np.float32)).to(torch.bfloat16)
        d_x, d_ids, d_w = x.to(DEV), to_dev(ids), to_dev(w)
        out = alloc_dispatch_outputs(bs, h, K, E)
        counts = torch.zeros((E,), dtype=torch.int32, device=DEV)
        st, _ = ep.dispatch_memory_ex(d_x, d_ids, s.comm, bs, h, K, E, out["expand_x"], out["assist"],
                                      out["token_nums"], counts, ep.DT_BF16, s.stream, row_index_map=out["row_map"])
        assert st == 0
        s.sync()
        rows = out["expand_x"].view(torch.bfloat16).view(n, h)
        expert_out = torch.full((n, h), 99.0, dtype=torch.bfloat16, device=DEV)      # what a stale read would return
        flags = torch.zeros((tiles,), dtype=torch.int64, device=DEV)
        status = torch.zeros((1,), dtype=torch.int32, device=DEV)
        y = torch.full((bs, h), 3.0, dtype=torch.bfloat16, device=DEV)
        busy = torch.zeros((64 << 20,), dtype=torch.int32, device=DEV)      # 40 passes over 256 MiB: a few milliseconds
        for epoch in (5, 6, 7):
            scale = float(epoch)
            torch.cuda.synchronize()
            with torch.cuda.stream(producer):
                for _ in range(40):
                    busy.add_(1)
                for tile in rng.permutation(tiles):
                    lo, hi = int(tile) * tile_rows, min(int(tile + 1) * tile_rows, n)
                    expert_out[lo:hi] = (rows[lo:hi].float() * scale).to(torch.bfloat16)
                    flags[int(tile)] = (epoch << 32) | (hi - lo)
            st = ep.combine_memory_ex(expert_out, out["assist"], counts, s.comm, bs, h, K, E, y, ep.DT_BF16, s.stream,
                                      expert_scales=d_w, row_index_map=out["row_map"], tile_flags=flags,
                                      tile_rows=tile_rows, flag_epoch=epoch, wait_timeout_us=10_000_000,
                                      device_status=status)
            assert st == 0
            producer.synchronize()
            s.sync()
            assert status.item() == 0
            xb = bits16((x.float() * scale).to(torch.bfloat16))
            case = O.Case(1, bs, h, K, E, token_nums_type=1)
            want = O.mem_dispatch(case, 0, xb[None], ids[None])
            wy = O.mem_combine(case, 0, want["expand_x"].view(np.uint16)[None], want["assist"][None],
                               want["send_counts"][None], expert_scales=w)
            assert np.array_equal(bits16(y), wy), f"epoch {epoch}"


@pytest.mark.parametrize("shape,tile_rows,workgroups,tile_ns", [((1024, 7168, 8, 64), 64, 48, 20000),
                                                                ((2048, 2048, 6, 32), 100, 16, 5000),
                                                                ((512, 1024, 4, 16), 8, 200, 0)])
def test_combine_beside_a_slow_producer_that_publishes_tiles_as_it_goes(shape, tile_rows, workgroups, tile_ns):
    """An expert-stage stand-in of the library (a HIP kernel: a few workgroups copy the dispatched rows into the expert
    output tile by tile at a set pace, ordinary stores, one release at agent scope per tile, then the tile's word) runs
    on one stream; combine runs beside it on another, waits per token for the tiles it needs and reads them from memory.
    The expert output starts as garbage and is garbage again before every round, so a row that is read early, or from a
    stale cache line, changes the result.  Three rounds on the same buffers with growing epochs."""
    bs, h, K, E = shape
    rng = np.random.default_rng(sum(shape) + tile_rows)
    n = bs * K
    tiles = (n + tile_rows - 1) // tile_rows
    ids, w = routing(rng, bs, K, E)
    x = torch.from_numpy(rng.standard_normal((bs, h)).astype(np.float32)).to(torch.bfloat16)
    xb = bits16(x)
    case = O.Case(1, bs, h, K, E, token_nums_type=1)
    want = O.mem_dispatch(case, 0, xb[None], ids[None])
    wy = O.mem_combine(case, 0, want["expand_x"].view(np.uint16)[None], want["assist"][None],
                       want["send_counts"][None], expert_scales=w)
    with Session() as s:
        side = torch.cuda.Stream()
        d_x, d_ids, d_w = x.to(DEV), to_dev(ids), to_dev(w)
        out = alloc_dispatch_outputs(bs, h, K, E)
        counts = torch.zeros((E,), dtype=torch.int32, device=DEV)
        st, _ = ep.dispatch_memory_ex(d_x, d_ids, s.comm, bs, h, K, E, out["expand_x"], out["assist"],
                                      out["token_nums"], counts, ep.DT_BF16, s.stream, row_index_map=out["row_map"])
        assert st == 0
        s.sync()
        rows = int(counts[-1].item())
        assert rows == n
        expert_out = torch.empty((n, h * 2), dtype=torch.uint8, device=DEV)
        flags = torch.zeros((tiles,), dtype=torch.int64, device=DEV)
        status = torch.zeros((1,), dtype=torch.int32, device=DEV)
        y = torch.empty((bs, h), dtype=torch.bfloat16, device=DEV)
        for epoch in (11, 12, 4_000_000_000):
            expert_out.fill_(0x7f)                 # bf16 0x7f7f = 3.4e38: an early read cannot go unnoticed
            y.fill_(-1.0)
            torch.cuda.synchronize()
            print(f"slow producer: shape {shape} tile_rows {tile_rows} epoch {epoch}", flush=True)
            # producer first: a waiting kernel enqueued ahead of it on a shared hardware queue would keep it out
            # (the second run with workgroups that do not move in step: tiles complete at a steady rate)
            assert ep.tile_producer_probe(out["expand_x"], expert_out, rows, h * 2, flags, tile_rows, epoch, workgroups,
                                          tile_ns, s.stream, stagger_ns=tile_ns if epoch == 12 else 0) == 0
            st = ep.combine_memory_ex(expert_out, out["assist"], counts, s.comm, bs, h, K, E, y, ep.DT_BF16, side,
                                      expert_scales=d_w, row_index_map=out["row_map"], tile_flags=flags,
                                      tile_rows=tile_rows, flag_epoch=epoch, wait_timeout_us=10_000_000,
                                      device_status=status)
            assert st == 0
            s.sync()
            side.synchronize()
            assert status.item() == 0
            assert np.array_equal(expert_out.cpu().numpy(), want["expand_x"])
            assert np.array_equal(bits16(y), wy), f"epoch {epoch}"
            f = flags.cpu().numpy().astype(np.uint64)
            rows_in_tile = np.minimum(tile_rows, n - np.arange(tiles) * tile_rows)
            assert np.array_equal(f, (np.uint64(epoch) << np.uint64(32)) | rows_in_tile.astype(np.uint64))
    # argument checks of the stand-in
    with Session() as s:
        assert ep.tile_producer_probe(expert_out, expert_out, 0, 64, flags, 8, 1, 4, 0, s.stream) == ep.ERR_PARA_CHECK_FAIL
        assert ep.tile_producer_probe(expert_out, expert_out, 8, 24, flags, 8, 1, 4, 0, s.stream) == ep.ERR_PARA_CHECK_FAIL
        assert ep.tile_producer_probe(expert_out, expert_out, 8, 64, flags, 8, 0, 4, 0, s.stream) == ep.ERR_PARA_CHECK_FAIL
        assert ep.tile_producer_probe(expert_out, expert_out, 8, 64, flags, 8, 1, 4, 0, s.stream,
                                      stagger_ns=-1) == ep.ERR_PARA_CHECK_FAIL


def test_flag_protocol_on_randomised_rounds():
    """A bounded randomised run of the whole flag protocol on buffers that are reused from round to round: random shapes,
    tile sizes, payload formats and schedules (combine after dispatch on one stream, beside it on a second stream, or
    beside an expert-stage stand-in that rewrites the rows).  Every round is compared bit for bit with the CPU oracle
    and must report no expired wait; the run ends at the first round that fails, after 48 rounds or after 60 seconds,
    whichever comes first.  Seeded: the same rounds every time."""
    import time
    rng = np.random.default_rng(20240607)
    max_rows, max_h = 4096 * 8, 7168
    with Session() as s:
        side = torch.cuda.Stream()
        pool_rows = torch.empty((max_rows * max_h * 2,), dtype=torch.uint8, device=DEV)
        pool_stage = torch.empty((max_rows * max_h * 2,), dtype=torch.uint8, device=DEV)
        pool_scales = torch.empty((max_rows * (max_h // 128),), dtype=torch.float32, device=DEV)
        pool_y = torch.empty((4096 * max_h,), dtype=torch.bfloat16, device=DEV)
        flags = torch.zeros((max_rows,), dtype=torch.int64, device=DEV)          # one array for every tile size
        stage_flags = torch.zeros((max_rows,), dtype=torch.int64, device=DEV)
        status = torch.zeros((1,), dtype=torch.int32, device=DEV)
        meta_ready, consumed = ep.HipEvent(), ep.HipEvent()
        started = time.monotonic()
        rounds = 0
        for round_ in range(48):
            if time.monotonic() - started > 60.0:
                break
            bs = int(rng.choice([64, 200, 777, 1024, 2048, 4096]))
            h = int(rng.choice([256, 1024, 2048, 4096, 7168]))
            K = int(rng.choice([2, 4, 8]))
            E = int(rng.choice([16, 64, 256]))
            tile_rows = int(rng.choice([1, 8, 16, 64, 100, 1024]))
            quant = str(rng.choice(["none", "none", "int8", "fp8_block128"]))
            schedule = str(rng.choice(["one_stream", "two_streams", "expert_stage"]))
            if quant != "none" and schedule == "expert_stage":
                schedule = "two_streams"
            qmode = {"none": ep.Q_NONE, "int8": ep.Q_TOKEN_INT8, "fp8_block128": ep.Q_FP8_BLOCK128}[quant]
            oq = {"none": O.Q_NONE, "int8": O.Q_TOKEN_INT8, "fp8_block128": O.Q_FP8_BLOCK128}[quant]
            n = bs * K
            row_bytes = h * 2 if qmode == ep.Q_NONE else h
            ids, w = routing(rng, bs, K, E)
            x = torch.from_numpy((rng.standard_normal((bs, h)) * (1 + round_ % 5)).astype(np.float32)).to(torch.bfloat16)
            xb = bits16(x)
            d_x, d_ids, d_w = x.to(DEV), to_dev(ids), to_dev(w)
            expand_x = pool_rows[:n * row_bytes].view(n, row_bytes)
            expert_out = pool_stage[:n * row_bytes].view(n, row_bytes)
            scales = None
            if qmode == ep.Q_TOKEN_INT8:
                scales = pool_scales[:n].view(n, 1)
            elif qmode == ep.Q_FP8_BLOCK128:
                scales = pool_scales[:n * ((h + 127) // 128)].view(n, (h + 127) // 128)
            y = pool_y[:bs * h].view(bs, h)
            y.fill_(-1234.0)                 # tells a token that was never written from one that was summed wrongly
            assist = torch.empty((n, 4), dtype=torch.int32, device=DEV)
            token_nums = torch.empty((E,), dtype=torch.int64, device=DEV)
            counts = torch.empty((E,), dtype=torch.int32, device=DEV)
            row_map = torch.empty((bs, K), dtype=torch.int32, device=DEV)
            torch.cuda.synchronize()
            print(f"flag rounds: {round_} bs={bs} h={h} K={K} E={E} tile_rows={tile_rows} {quant} {schedule}", flush=True)
            two = schedule == "two_streams"
            st, epoch = ep.dispatch_memory_ex(d_x, d_ids, s.comm, bs, h, K, E, expand_x, assist, token_nums, counts,
                                              ep.DT_BF16, s.stream, quant_mode=qmode, dynamic_scales=scales,
                                              row_index_map=row_map, tile_flags=flags, tile_rows=tile_rows,
                                              meta_ready_event=meta_ready.value if two else None)
            assert st == 0
            rows_in, use_flags, use_epoch, consumer = expand_x, flags, epoch, s.stream
            if two:
                meta_ready.wait_on(side)
                consumer = side
            elif schedule == "expert_stage":
                # the stand-in follows the dispatch on its stream and republishes the rows under an epoch of its own;
                # combine runs beside it on the second stream (the row map is complete: dispatch was enqueued first and
                # the stand-in's stream order puts every flag of it after the dispatch)
                s.sync()
                assert ep.tile_producer_probe(expand_x, expert_out, n, row_bytes, stage_flags, tile_rows, 1000 + round_,
                                              int(rng.choice([8, 64, 200])), int(rng.choice([0, 3000])), s.stream,
                                              stagger_ns=int(rng.choice([0, 3000]))) == 0
                rows_in, use_flags, use_epoch, consumer = expert_out, stage_flags, 1000 + round_, side
            st = ep.combine_memory_ex(rows_in, assist, counts, s.comm, bs, h, K, E, y, ep.DT_BF16, consumer,
                                      expert_out_quant_mode=qmode, expert_out_scales=scales, expert_scales=d_w,
                                      row_index_map=row_map, tile_flags=use_flags, tile_rows=tile_rows,
                                      flag_epoch=use_epoch, wait_timeout_us=5_000_000, device_status=status)
            assert st == 0
            if consumer is side:
                consumed.record(side)
                consumed.wait_on(s.stream)
            s.sync()
            side.synchronize()
            assert status.item() == 0, f"round {round_}: a flag wait expired"
            case = O.Case(1, bs, h, K, E, dtype=O.DT_BF16, quant_mode=oq, token_nums_type=1)
            want = O.mem_dispatch(case, 0, xb[None], ids[None])
            assert np.array_equal(expand_x.cpu().numpy(), want["expand_x"]), f"round {round_}: rows"
            # the row map the combine was given: row of (token, k) as the oracle's tuples have it
            want_map = np.full((bs, K), -1, np.int32)
            live = want["assist"][:want["rows"]]
            want_map[live[:, 1], live[:, 2]] = np.arange(want["rows"], dtype=np.int32)
            assert np.array_equal(row_map.cpu().numpy(), want_map), f"round {round_}: row map"
            assert np.array_equal(assist.cpu().numpy()[:want["rows"]], live), f"round {round_}: assist tuples"
            if schedule == "expert_stage":
                assert torch.equal(expert_out, expand_x), f"round {round_}: the stand-in's copy of the rows"
                f = stage_flags[:(n + tile_rows - 1) // tile_rows].cpu().numpy().astype(np.uint64)
                assert np.all(f >> np.uint64(32) == np.uint64(1000 + round_)), f"round {round_}: the stand-in's words"
            eo = want["expand_x"][None] if oq else want["expand_x"].view(np.uint16)[None]
            wy = O.mem_combine(O.Case(1, bs, h, K, E, dtype=O.DT_BF16), 0, eo, want["assist"][None],
                               want["send_counts"][None], expert_scales=w, in_quant=oq,
                               in_scales=want["dyn_scales"] if oq else None)
            got_y = bits16(y)
            bad = np.flatnonzero((got_y != wy).any(axis=1))
            untouched = int((got_y[bad] == bits16(torch.tensor([-1234.0], dtype=torch.bfloat16))[0]).all(axis=1).sum())
            detail = ""
            if bad.size:
                t = int(bad[0])
                cols = np.flatnonzero(got_y[t] != wy[t])
                rows_t = row_map.cpu().numpy()[t]
                src = (expert_out if schedule == "expert_stage" else expand_x).cpu().numpy()
                detail = (f"; token {t}: {cols.size} columns differ, first {cols[:6].tolist()} last {cols[-3:].tolist()}, "
                          f"got {got_y[t][cols[:4]].tolist()} want {wy[t][cols[:4]].tolist()}, weights {w[t].tolist()}")
                if qmode == ep.Q_NONE:
                    f32 = lambda bits: (bits.astype(np.uint32) << 16).view(np.float32)
                    parts = [f32(src[r].view(np.uint16)) * np.float32(w[t, k]) for k, r in enumerate(rows_t) if r >= 0]
                    for k, part in enumerate(parts):
                        alone = ((part.view(np.uint32) + 0x7fff + ((part.view(np.uint32) >> 16) & 1)) >> 16).astype(np.uint16)
                        detail += f", equals slot {k} alone on {int((got_y[t][cols] == alone[cols]).sum())} of them"
            assert bad.size == 0, (f"round {round_}: y differs for {bad.size} tokens ({untouched} of them never written), "
                                   f"first {bad[:8].tolist()}, rows {row_map.cpu().numpy()[bad[:4]].tolist()}" + detail)
            rounds += 1
        assert rounds >= 8
        meta_ready.destroy()
        consumed.destroy()
