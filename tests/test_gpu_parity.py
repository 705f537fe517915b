"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle on the same seeded inputs.

Integer / byte outputs (row order, counts, source-index map, int8 / fp8 payloads, scales) must be bit-exact.
Combine outputs are compared bit-exactly too, because the kernels reproduce the reference's order of roundings;
the looser bound the workload definition allows (1e-2 relative) is only used for the full-size property checks.
"""
import numpy as np
import pytest
import torch

from gpu_harness import DEV, Session, alloc_dispatch_outputs, bits16, fetch, to_dev
from oracle import ep as O
from tilexr_amd import ep, workloads

pytestmark = pytest.mark.gpu


def ids_for(rng, bs, K, E, invalid=0.0):
    ids = np.stack([rng.permutation(E)[:K] if E >= K else rng.integers(0, E, K) for _ in range(bs)]).astype(np.int32)
    if invalid:
        bad = rng.random(ids.shape) < invalid
        ids[bad] = rng.choice([-1, -9, E, E + 3], size=int(bad.sum()))
    return ids


def x_for(rng, bs, h, dtype, scale=1.0):
    f = (rng.standard_normal((bs, h)) * scale).astype(np.float32)
    t = torch.from_numpy(f).to(torch.bfloat16 if dtype == ep.DT_BF16 else torch.float16)
    return t.to(DEV), bits16(t)      # the device copy stays alive in the caller's scope while kernels read it


def check_dispatch(got, want, rows_key="rows"):
    n = want[rows_key]
    assert np.array_equal(got["assist"][:n], want["assist"][:n])
    assert np.array_equal(got["expand_x"][:n], want["expand_x"][:n])
    assert np.array_equal(got["token_nums"], want["expert_token_nums"])
    # rows beyond the last valid one are never written
    assert np.all(got["assist"][n:] == -77)


SHAPES = [(7, 8, 2, 5), (64, 64, 4, 16), (33, 40, 3, 7), (16, 33, 2, 4), (300, 1024, 8, 64), (2100, 256, 8, 256),
          (128, 7168, 8, 256), (5, 16400, 2, 4), (19, 2048, 12, 32)]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("dtype", [ep.DT_BF16, ep.DT_FP16])
@pytest.mark.parametrize("legacy_routing", [False, True])
def test_memory_dispatch_matches_oracle(shape, dtype, legacy_routing):
    bs, h, K, E = shape
    if legacy_routing and bs * K <= 2048:
        pytest.skip("batches this small take the single-launch dispatch under either setting")
    rng = np.random.default_rng(sum(shape) + dtype)
    ids = ids_for(rng, bs, K, E, invalid=0.1)
    xt, xb = x_for(rng, bs, h, dtype)
    with Session(legacy_routing=legacy_routing) as s:
        for mask_type in (ep.MASK_NONE, ep.MASK_TOKEN, ep.MASK_EXPERT):
            mask = None
            if mask_type == ep.MASK_TOKEN:
                mask = (rng.random(bs) < 0.7).astype(np.uint8)
            elif mask_type == ep.MASK_EXPERT:
                mask = (rng.random((bs, K)) < 0.7).astype(np.uint8)
            for nums_type in (0, 1):
                out = alloc_dispatch_outputs(bs, h, K, E)
                counts = torch.full((E,), -1, dtype=torch.int32, device=DEV)
                st = ep.dispatch_memory_v2(xt, to_dev(ids), s.comm, bs, h, K, E, out["expand_x"], out["assist"],
                                           out["token_nums"], counts, dtype, s.stream, active_mask=to_dev(mask),
                                           active_mask_type=mask_type, token_nums_type=nums_type)
                assert st == 0
                s.sync()
                got = fetch(out, "send_counts", counts)
                case = O.Case(1, bs, h, K, E, dtype=dtype, mask_type=mask_type, token_nums_type=nums_type)
                want = O.mem_dispatch(case, 0, xb[None], ids[None], None if mask is None else mask[None])
                check_dispatch(got, want)
                assert np.array_equal(got["send_counts"], want["send_counts"])


ROUTING_SHAPES = [
    # bs, h, K, E, invalid share, what the shape is there for
    (1024, 16, 3, 5, 0.1),          # 3072 routes: not a multiple of 256 per wave, slots 1
    (2049, 16, 1, 1, 0.0),          # one expert, topK 1
    (683, 16, 3, 2048, 0.05),       # as many experts as the tables hold, most of them without a route
    (4096, 16, 8, 256, 0.0),        # 32 768 routes: eight slots per wave, one batch of loads
    (4097, 16, 8, 256, 0.02),       # just beyond it: nine slots, the last waves hold nothing but padding
    (8192, 16, 8, 64, 0.0),         # 65 536 routes, 64 experts: four workgroups per expert
    (8193, 16, 8, 64, 0.0),         # seventeen slots: two parts at least, the second nearly empty
    (16384, 16, 8, 128, 0.01),      # 131 072 routes: 32 slots per wave in two parts of sixteen
    (32768, 8, 8, 512, 0.0),        # 262 144 routes: the largest table the one-launch routing takes
    (32769, 8, 8, 512, 0.0),        # one token more: count + place
    (3000, 16, 7, 37, 1.0),         # no route names an expert
    (3000, 16, 6, 9, 0.0),          # few experts: thousands of routes per key, several per lane and slot
    (4096, 16, 8, 8, 0.0),          # eight experts, eight workgroups each: one slot of every wave's eight per workgroup
]


@pytest.mark.parametrize("case", ROUTING_SHAPES)
def test_one_launch_routing_matches_oracle(case):
    """The routing kernel that resolves every route's row in one launch (memory route, no mask, no capacity limit, up
    to 262 144 routes), at the edges of what it takes; ids drawn with repeats within a token too.  Compared with the
    oracle and, bit for bit, with the count + place routing on the same inputs."""
    bs, h, K, E, invalid = case
    rng = np.random.default_rng(bs * 31 + K * 7 + E)
    ids = rng.integers(0, E, (bs, K)).astype(np.int32)          # repeats within a token allowed
    if E == 9:
        ids[:, 0] = 4                                           # one expert takes a route of every token
    bad = rng.random(ids.shape) < invalid
    ids[bad] = rng.choice([-1, -9, E, E + 3, 2 ** 31 - 1, -2 ** 31], size=int(bad.sum()))
    xt, xb = x_for(rng, bs, h, ep.DT_BF16)
    results = []
    for legacy in (False, True):
        with Session(legacy_routing=legacy) as s:
            for nums_type in (0, 1):
                out = alloc_dispatch_outputs(bs, h, K, E)
                counts = torch.full((E,), -1, dtype=torch.int32, device=DEV)
                st, _ = ep.dispatch_memory_ex(xt, to_dev(ids), s.comm, bs, h, K, E, out["expand_x"], out["assist"],
                                              out["token_nums"], counts, ep.DT_BF16, s.stream,
                                              token_nums_type=nums_type, row_index_map=out["row_map"])
                assert st == 0
                s.sync()
                expect = "ep_route_count_kernel" if legacy or bs * K > 262144 else "ep_route_rows_kernel"
                assert ep.last_kernel_name(s.comm, ep.K_COUNT) == expect
                got = fetch(out, "send_counts", counts)
                want = O.mem_dispatch(O.Case(1, bs, h, K, E, token_nums_type=nums_type), 0, xb[None], ids[None])
                check_dispatch(got, want)
                assert np.array_equal(got["send_counts"], want["send_counts"])
                # the row map is the inverse of the tuples, -1 where a route has no row
                rm = np.full(bs * K, -1, np.int32)
                n = want["rows"]
                rm[want["assist"][:n, 1] * K + want["assist"][:n, 2]] = np.arange(n, dtype=np.int32)
                assert np.array_equal(got["row_map"].reshape(-1), rm)
                results.append(got)
    for name in ("assist", "expand_x", "token_nums", "send_counts", "row_map"):
        assert np.array_equal(results[0][name], results[2][name]), name


@pytest.mark.parametrize("seed", range(40))
def test_one_launch_routing_on_random_tables(seed):
    """Tables of random size (up to 120 000 routes: one to thirty slots per wave, one to sixteen workgroups per key),
    random topK and expert count, ids with repeats and a random share of ids that name no expert: rows, tuples, counts
    and row map against the oracle."""
    rng = np.random.default_rng(9000 + seed)
    K = int(rng.integers(1, 10))
    bs = int(rng.integers(1, 120000 // K + 1)) if seed % 4 else int(rng.integers(1, 3000))
    E = int(rng.choice([1, 2, 3, 7, 8, 16, 33, 64, 100, 256, 257, 700, 2048]))
    h = 8
    ids = rng.integers(0, E, (bs, K)).astype(np.int32)
    bad = rng.random(ids.shape) < float(rng.choice([0.0, 0.01, 0.3]))
    ids[bad] = rng.choice([-1, -9, E, E + 3, 2 ** 31 - 1, -2 ** 31], size=int(bad.sum()))
    xt, xb = x_for(rng, bs, h, ep.DT_BF16)
    nums_type = seed % 2
    with Session(legacy_routing=False) as s:
        out = alloc_dispatch_outputs(bs, h, K, E)
        counts = torch.full((E,), -1, dtype=torch.int32, device=DEV)
        st, _ = ep.dispatch_memory_ex(xt, to_dev(ids), s.comm, bs, h, K, E, out["expand_x"], out["assist"],
                                      out["token_nums"], counts, ep.DT_BF16, s.stream, token_nums_type=nums_type,
                                      row_index_map=out["row_map"])
        assert st == 0
        s.sync()
        small = bs * K <= 2048       # decode-sized calls take the single-launch dispatch whatever the switch says
        assert small or ep.last_kernel_name(s.comm, ep.K_COUNT) == "ep_route_rows_kernel"
        got = fetch(out, "send_counts", counts)
        want = O.mem_dispatch(O.Case(1, bs, h, K, E, token_nums_type=nums_type), 0, xb[None], ids[None])
        check_dispatch(got, want)
        assert np.array_equal(got["send_counts"], want["send_counts"])
        rm = np.full(bs * K, -1, np.int32)
        n = want["rows"]
        rm[want["assist"][:n, 1] * K + want["assist"][:n, 2]] = np.arange(n, dtype=np.int32)
        assert np.array_equal(got["row_map"].reshape(-1), rm)


def test_routing_kernels_are_picked_by_the_size_of_the_call():
    """Left to itself the library takes the one-launch routing where it was measured to be the faster one: small
    tables always; larger ones while routes x experts stays small, less far when the same launch also reads token rows
    ahead of a scatter that copies per route (rows wider than 4 KiB, plain payload) and then only against count + place
    (readiness flags ask for the rows ahead of the scatter)."""
    cases = [  # bs, K, E, h, flags, kernel
        (1024, 8, 256, 16, False, "ep_route_rows_kernel"), (2048, 8, 2048, 16, False, "ep_route_count_kernel"),
        (2048, 8, 2048, 16, True, "ep_route_rows_kernel"), (4096, 8, 256, 16, False, "ep_route_rows_kernel"),
        (4096, 8, 1024, 16, True, "ep_route_count_kernel"), (8192, 6, 64, 16, True, "ep_route_rows_kernel"),
        (8192, 8, 256, 16, True, "ep_route_count_kernel"), (16384, 8, 64, 16, False, "ep_route_count_kernel"),
        (4096, 8, 256, 2056, False, "ep_route_count_kernel"), (4096, 8, 256, 2056, True, "ep_route_rows_kernel"),
        (4096, 8, 512, 2056, True, "ep_route_count_kernel"), (6144, 8, 64, 2056, True, "ep_route_count_kernel"),
    ]
    with Session() as s:
        for bs, K, E, h, with_flags, kernel in cases:
            rng = np.random.default_rng(bs + E)
            ids = rng.integers(0, E, (bs, K)).astype(np.int32)
            xt, xb = x_for(rng, bs, h, ep.DT_BF16)
            out = alloc_dispatch_outputs(bs, h, K, E)
            counts = torch.full((E,), -1, dtype=torch.int32, device=DEV)
            flags = torch.zeros(((bs * K + 63) // 64,), dtype=torch.int64, device=DEV) if with_flags else None
            torch.cuda.synchronize()
            st, _ = ep.dispatch_memory_ex(xt, to_dev(ids), s.comm, bs, h, K, E, out["expand_x"], out["assist"],
                                          out["token_nums"], counts, ep.DT_BF16, s.stream, row_index_map=out["row_map"],
                                          tile_flags=flags, tile_rows=64 if with_flags else 0)
            assert st == 0
            s.sync()
            assert ep.last_kernel_name(s.comm, ep.K_COUNT) == kernel, (bs, K, E, h, with_flags)
            if h == 16:
                want = O.mem_dispatch(O.Case(1, bs, h, K, E), 0, xb[None], ids[None])
                check_dispatch(fetch(out, "send_counts", counts), want)
            del out


def test_one_launch_routing_with_unaligned_tables():
    """An id table that is not 16-byte aligned takes the count + place routing; an unaligned tuple array takes the
    one-launch routing with four-byte stores."""
    bs, h, K, E = 1500, 32, 4, 24
    rng = np.random.default_rng(77)
    ids = ids_for(rng, bs, K, E, invalid=0.05)
    xt, xb = x_for(rng, bs, h, ep.DT_BF16)
    want = O.mem_dispatch(O.Case(1, bs, h, K, E, token_nums_type=1), 0, xb[None], ids[None])
    n = want["rows"]
    with Session(legacy_routing=False) as s:
        for shift_ids, shift_assist in ((1, 0), (0, 1)):
            out = alloc_dispatch_outputs(bs, h, K, E)
            counts = torch.full((E,), -1, dtype=torch.int32, device=DEV)
            d_ids = torch.zeros((bs * K + 4,), dtype=torch.int32, device=DEV)
            d_ids[shift_ids:shift_ids + bs * K] = torch.from_numpy(ids.reshape(-1)).to(DEV)
            assist = torch.full((bs * K * 4 + 4,), -77, dtype=torch.int32, device=DEV)
            torch.cuda.synchronize()
            st = ep.dispatch_memory(xt, d_ids[shift_ids:], s.comm, bs, h, K, E, out["expand_x"], out["token_nums"], counts,
                                    assist[shift_assist:], ep.DT_BF16, s.stream)
            assert st == 0
            s.sync()
            assert ep.last_kernel_name(s.comm, ep.K_COUNT) == ("ep_route_count_kernel" if shift_ids else "ep_route_rows_kernel")
            got = assist.cpu().numpy()[shift_assist:shift_assist + bs * K * 4].reshape(-1, 4)
            assert np.array_equal(got[:n], want["assist"][:n])
            assert np.all(got[n:] == -77)
            assert np.array_equal(out["expand_x"].cpu().numpy()[:n], want["expand_x"][:n])
            assert np.array_equal(counts.cpu().numpy(), want["send_counts"])


@pytest.mark.parametrize("shape", SHAPES[:6])
def test_mvp_dispatch_matches_oracle(shape):
    bs, h, K, E = shape
    rng = np.random.default_rng(sum(shape) + 99)
    ids = ids_for(rng, bs, K, E, invalid=0.1)
    xt, xb = x_for(rng, bs, h, ep.DT_FP16, scale=3.0)
    mask = (rng.random(bs) < 0.7).astype(np.uint8)
    static = np.array([1.75], np.float32)
    with Session() as s:
        for quant in (ep.Q_NONE, ep.Q_STATIC_INT8, ep.Q_TOKEN_INT8):
            for use_mask in (False, True):
                for nums_type in (1, 0):
                    out = alloc_dispatch_outputs(bs, h, K, E, quant=quant)
                    counts = torch.full((1,), -1, dtype=torch.int32, device=DEV)
                    tp_counts = torch.full((1,), -1, dtype=torch.int32, device=DEV)
                    st = ep.dispatch_v2(
                        xt, to_dev(ids), s.comm, bs, h, K, E, out["expand_x"], out["assist"], out["token_nums"],
                        counts, ep.DT_FP16 if quant == ep.Q_NONE else ep.DT_INT8, s.stream,
                        scales=to_dev(static) if quant == ep.Q_STATIC_INT8 else None,
                        active_mask=to_dev(mask) if use_mask else None, quant_mode=quant, token_nums_type=nums_type,
                        dynamic_scales=out["scales"] if quant == ep.Q_TOKEN_INT8 else None, tp_recv_counts=tp_counts)
                    assert st == 0
                    s.sync()
                    got = fetch(out, "recv_counts", counts)
                    case = O.Case(1, bs, h, K, E, dtype=O.DT_FP16, quant_mode=quant, token_nums_type=nums_type)
                    want = O.mvp_dispatch(case, 0, xb[None], ids[None], mask[None] if use_mask else None, static)
                    check_dispatch(got, want)
                    assert np.array_equal(got["recv_counts"], want["recv_counts"])
                    assert tp_counts.item() == want["recv_counts"][0]
                    if quant == ep.Q_TOKEN_INT8:
                        n = want["rows"]
                        assert np.array_equal(got["scales"][:n, 0], want["dyn_scales"][:n])


def test_simple_entry_points():
    bs, h, K, E = 50, 128, 4, 32
    rng = np.random.default_rng(5)
    ids = ids_for(rng, bs, K, E)
    xt, xb = x_for(rng, bs, h, ep.DT_BF16)
    w = np.ones((bs, K), np.float32)
    with Session() as s:
        for memory in (True, False):
            out = alloc_dispatch_outputs(bs, h, K, E)
            counts = torch.zeros((E if memory else 1,), dtype=torch.int32, device=DEV)
            fn = ep.dispatch_memory if memory else ep.dispatch
            assert fn(xt, to_dev(ids), s.comm, bs, h, K, E, out["expand_x"], out["token_nums"], counts,
                      out["assist"], ep.DT_BF16, s.stream) == 0
            y = torch.zeros((bs, h), dtype=torch.bfloat16, device=DEV)
            fnc = ep.combine_memory if memory else ep.combine
            assert fnc(out["expand_x"], out["assist"], counts, s.comm, bs, h, K, E, y, ep.DT_BF16, s.stream) == 0
            s.sync()
            case = O.Case(1, bs, h, K, E, token_nums_type=1)
            want = (O.mem_dispatch if memory else O.mvp_dispatch)(case, 0, xb[None], ids[None])
            got = fetch(out, "counts", counts)
            check_dispatch(got, want)
            eo = want["expand_x"].view(np.uint16)[None]
            if memory:
                wy = O.mem_combine(case, 0, eo, want["assist"][None], want["send_counts"][None])
            else:
                wy = O.mvp_combine(case, 0, eo, want["assist"][None], want["recv_counts"][None])
            assert np.array_equal(bits16(y), wy)
    del w


QUANT_SHAPES = [(40, 256, 4, 8), (17, 40, 2, 4), (9, 33, 2, 4), (130, 4096, 6, 64), (64, 2048, 8, 128),
                (20, 7168, 8, 256)]


@pytest.mark.parametrize("shape", QUANT_SHAPES)
@pytest.mark.parametrize("dtype", [ep.DT_BF16, ep.DT_FP16])
@pytest.mark.parametrize("quant,fp8", [(ep.Q_TOKEN_INT8, None), (ep.Q_MXFP8, ep.DT_FP8E4M3), (ep.Q_MXFP8, ep.DT_FP8E5M2),
                                       (ep.Q_FP8_BLOCK128, None)])
def test_quantised_dispatch_matches_oracle(shape, dtype, quant, fp8):
    bs, h, K, E = shape
    rng = np.random.default_rng(sum(shape) + dtype + quant)
    ids = ids_for(rng, bs, K, E, invalid=0.05)
    xt, xb = x_for(rng, bs, h, dtype, scale=2.0)
    xb[0, :] = 0                       # an all-zero row
    if h >= 64:
        xb[1, 32:64] = 0               # an all-zero block
    xt = torch.from_numpy(xb.view(np.int16)).view(torch.bfloat16 if dtype == ep.DT_BF16 else torch.float16).to(DEV)
    with Session() as s:
        out = alloc_dispatch_outputs(bs, h, K, E, quant=quant)
        counts = torch.zeros((E,), dtype=torch.int32, device=DEV)
        st, _ = ep.dispatch_memory_ex(xt, to_dev(ids), s.comm, bs, h, K, E, out["expand_x"], out["assist"],
                                      out["token_nums"], counts, dtype, s.stream, quant_mode=quant,
                                      dynamic_scales=out["scales"], expand_x_dtype=fp8, row_index_map=out["row_map"])
        assert st == 0
        s.sync()
        got = fetch(out, "send_counts", counts)
        case = O.Case(1, bs, h, K, E, dtype=dtype, quant_mode=quant, out_dtype=fp8 or O.DT_FP8E4M3)
        want = O.mem_dispatch(case, 0, xb[None], ids[None])
        check_dispatch(got, want)
        n = want["rows"]
        assert np.array_equal(got["scales"][:n], want["dyn_scales"][:n])
        # the row map is the inverse of the assist tuples
        rm = got["row_map"]
        for row in range(n):
            _, t, k, _ = want["assist"][row]
            assert rm[t, k] == row
        assert (rm >= 0).sum() == n
        if quant == ep.Q_MXFP8:
            # the reference API takes the same mode through DispatchMemoryV2
            out2 = alloc_dispatch_outputs(bs, h, K, E, quant=quant)
            st = ep.dispatch_memory_v2(xt, to_dev(ids), s.comm, bs, h, K, E, out2["expand_x"], out2["assist"],
                                       out2["token_nums"], counts, dtype, s.stream, quant_mode=4,
                                       dynamic_scales=out2["scales"], expand_x_dtype=fp8)
            assert st == 0
            s.sync()
            assert torch.equal(out2["expand_x"][:n], out["expand_x"][:n])
            assert torch.equal(out2["scales"][:n], out["scales"][:n])


def test_capacity_drop_matches_oracle():
    rng = np.random.default_rng(77)
    bs, h, K, E, cap = 700, 64, 8, 16, 300
    w = workloads.Workload("t", 1, bs, h, K, E, routing="zipf", zipf_s=1.2, seed=3)
    ids = workloads.make_routing(w)[0].numpy()
    xt, xb = x_for(rng, bs, h, ep.DT_BF16)
    with Session() as s:
        out = alloc_dispatch_outputs(bs, h, K, E)
        counts = torch.zeros((E,), dtype=torch.int32, device=DEV)
        st, _ = ep.dispatch_memory_ex(xt, to_dev(ids), s.comm, bs, h, K, E, out["expand_x"], out["assist"],
                                      out["token_nums"], counts, ep.DT_BF16, s.stream, expert_capacity=cap,
                                      row_index_map=out["row_map"])
        assert st == 0
        s.sync()
        got = fetch(out, "send_counts", counts)
        want = O.mem_dispatch(O.Case(1, bs, h, K, E, capacity=cap), 0, xb[None], ids[None])
        assert want["rows"] < bs * K                     # something was dropped
        assert want["expert_token_nums"].max() == cap
        check_dispatch(got, want)
        assert np.array_equal(got["send_counts"], want["send_counts"])
        assert (got["row_map"] >= 0).sum() == want["rows"]


COMBINE_SHAPES = [(7, 8, 2, 5), (64, 64, 4, 16), (33, 40, 3, 7), (16, 33, 2, 4), (100, 1024, 8, 64),
                  (40, 7168, 8, 256), (3, 16400, 2, 4)]


@pytest.mark.parametrize("shape", COMBINE_SHAPES)
@pytest.mark.parametrize("dtype", [ep.DT_BF16, ep.DT_FP16])
def test_memory_combine_matches_oracle(shape, dtype):
    bs, h, K, E = shape
    rng = np.random.default_rng(sum(shape) + 3 * dtype)
    ids = ids_for(rng, bs, K, E, invalid=0.1)
    xt, xb = x_for(rng, bs, h, dtype, scale=3.0)
    case = O.Case(1, bs, h, K, E, dtype=dtype)
    d = O.mem_dispatch(case, 0, xb[None], ids[None])
    rows = d["rows"]
    eo = d["expand_x"].view(np.uint16).copy()
    for r in range(rows):
        eo[r] = np.roll(eo[r], r % 5)          # make every route's row different
    w = (0.25 + rng.random((bs, K))).astype(np.float32)
    w[0, 0] = 1.0
    tmask = (rng.random(bs) < 0.8).astype(np.uint8)
    _, sxb = x_for(rng, bs, h, dtype)
    with Session() as s:
        d_eo, d_assist, d_counts = to_dev(eo), to_dev(d["assist"]), to_dev(d["send_counts"])
        for use_w, use_mask, use_shared in ((False, False, False), (True, False, False), (True, True, True)):
            y = torch.full((bs, h), 7.0, dtype=torch.bfloat16 if dtype == ep.DT_BF16 else torch.float16, device=DEV)
            st = ep.combine_memory_v2(d_eo, d_assist, d_counts, s.comm, bs, h, K, E, y, dtype, s.stream,
                                      expert_scales=to_dev(w) if use_w else None,
                                      active_mask=to_dev(tmask) if use_mask else None,
                                      active_mask_type=ep.MASK_TOKEN if use_mask else ep.MASK_NONE,
                                      shared_expert_x=to_dev(sxb) if use_shared else None)
            assert st == 0
            s.sync()
            want = O.mem_combine(case, 0, eo[None], d["assist"][None], d["send_counts"][None],
                                 expert_scales=w if use_w else None, token_mask=tmask if use_mask else None,
                                 shared_expert_x=sxb if use_shared else None)
            assert np.array_equal(bits16(y), want)


@pytest.mark.parametrize("route", ["memory", "mvp"])
def test_small_combine_reads_the_assist_table_itself(route):
    """Through the reference's entry points combine gets no row map.  Up to 2048 routes (and a million tokens x tuples)
    the reduce finds a token's rows in the assist table itself (one launch); beyond that, or with rows the kernel's
    waves cannot cover, a first launch inverts the table.  Both give the oracle's result; the cases sit on either side of every limit."""
    cases = [  # bs, h, K, E, kernel
        (256, 64, 8, 32, "ep_reduce_small_kernel"),        # 2048 routes: the most one workgroup scans
        (257, 64, 8, 32, "ep_reduce_vec_kernel"),
        (1024, 8, 1, 4, "ep_reduce_small_kernel"),         # one slot per token, rows of one vector
        (2048, 8, 1, 4, "ep_reduce_vec_kernel"),           # more tokens than it pays to let every one read the table
        (512, 64, 4, 32, "ep_reduce_small_kernel"),        # tokens x tuples at its limit
        (5, 16384, 3, 9, "ep_reduce_small_kernel"),        # sixteen waves per row
        (5, 16392, 3, 9, "ep_reduce_generic_kernel"),
        (128, 7168, 8, 256, "ep_reduce_small_kernel"),     # decode
        (64, 36, 15, 40, "ep_reduce_generic_kernel"),      # rows that are no multiple of 16 bytes
        (40, 1024, 15, 40, "ep_reduce_small_kernel"),
        (32, 256, 64, 80, "ep_reduce_small_kernel"),       # as many slots as a wave has lanes
    ]
    dtype = ep.DT_BF16 if route == "memory" else ep.DT_FP16
    tdt = torch.bfloat16 if dtype == ep.DT_BF16 else torch.float16
    with Session() as s:
        for bs, h, K, E, kernel in cases:
            rng = np.random.default_rng(bs + h + K)
            ids = ids_for(rng, bs, K, E, invalid=0.1)
            _, xb = x_for(rng, bs, h, dtype, scale=3.0)
            case = O.Case(1, bs, h, K, E, dtype=dtype)
            d = (O.mem_dispatch if route == "memory" else O.mvp_dispatch)(case, 0, xb[None], ids[None])
            rows = d["rows"]
            eo = d["expand_x"].view(np.uint16).copy()
            for r in range(rows):
                eo[r] = np.roll(eo[r], r % 5)
            counts = d["send_counts" if route == "memory" else "recv_counts"]
            w = (0.25 + rng.random((bs, K))).astype(np.float32)
            y = torch.full((bs, h), 7.0, dtype=tdt, device=DEV)
            d_eo = torch.zeros((bs * K, h), dtype=torch.int16, device=DEV)
            d_eo[:eo.shape[0]] = torch.from_numpy(eo.view(np.int16)).to(DEV)
            d_assist = torch.full((bs * K, 4), -1, dtype=torch.int32, device=DEV)
            d_assist[:d["assist"].shape[0]] = torch.from_numpy(d["assist"]).to(DEV)
            torch.cuda.synchronize()
            print(f"small combine: {route} bs={bs} h={h} K={K} E={E}", flush=True)
            if route == "memory":
                st = ep.combine_memory_v2(d_eo, d_assist, to_dev(counts), s.comm, bs, h, K, E, y, dtype, s.stream,
                                          expert_scales=to_dev(w))
            else:
                st = ep.combine_v2(d_eo, d_assist, to_dev(counts), s.comm, bs, h, K, E, y, dtype, s.stream)
            assert st == 0
            s.sync()
            assert ep.last_kernel_name(s.comm, ep.K_REDUCE) == kernel, (bs, h, K, E)
            host_eo = d_eo.cpu().numpy().view(np.uint16)[None]
            host_assist = d_assist.cpu().numpy()[None]
            if route == "memory":
                want = O.mem_combine(case, 0, host_eo, host_assist, counts[None], expert_scales=w)
            else:
                want = O.mvp_combine(case, 0, host_eo, host_assist, counts[None])
            assert np.array_equal(bits16(y), want), (bs, h, K, E)


@pytest.mark.parametrize("seed", range(32))
def test_small_combine_on_random_calls(seed):
    """Seeded draws around the single-launch combine: shape (on both sides of its 2048 routes), route, element type,
    gate weights, token mask, shared-expert row, and now and then a table with corrupted tuples, a duplicate claim on
    a slot and a count that points past the buffer.  Every result is the oracle's, bit for bit."""
    from test_oracle_routes import corrupt_tuples
    rng = np.random.default_rng(4200 + seed)
    route = "memory" if seed % 3 else "mvp"
    dtype = ep.DT_BF16 if rng.integers(0, 2) else ep.DT_FP16
    tdt = torch.bfloat16 if dtype == ep.DT_BF16 else torch.float16
    K = int(rng.integers(1, 17))
    bs = int(rng.integers(1, 2500 // K + 1))
    E = int(rng.integers(K, 300))
    h = int(rng.choice([8, 64, 136, 1000, 1024, 2048, 4096, 7168, 16384]))
    ids = ids_for(rng, bs, K, E, invalid=float(rng.choice([0.0, 0.1, 0.6])))
    _, xb = x_for(rng, bs, h, dtype, scale=3.0)
    case = O.Case(1, bs, h, K, E, dtype=dtype)
    d = (O.mem_dispatch if route == "memory" else O.mvp_dispatch)(case, 0, xb[None], ids[None])
    rows = d["rows"]
    eo = d["expand_x"].view(np.uint16).copy()
    for r in range(rows):
        eo[r] = np.roll(eo[r], r % 5)
    assist = d["assist"].copy()
    counts = d["send_counts" if route == "memory" else "recv_counts"].copy()
    spoiled = seed % 4 == 1 and rows > 8
    if spoiled:
        corrupt_tuples(rng, assist[None], [rows], bs, K, 1, max(3, rows // 10))
        if route == "memory":
            intact = [r for r in range(rows) if np.array_equal(assist[r], d["assist"][r])]
            assist[intact[-1], :3] = assist[intact[0], :3]
            counts[-1] = bs * K + 999
    use_w, use_mask, use_shared = (bool(v) for v in rng.integers(0, 2, 3))
    w = (0.25 + rng.random((bs, K))).astype(np.float32)
    tmask = (rng.random(bs) < 0.7).astype(np.uint8)
    _, sxb = x_for(rng, bs, h, dtype)
    print(f"small combine seed={seed}: {route} bs={bs} h={h} K={K} E={E} dtype={dtype} spoiled={spoiled} "
          f"weights={use_w} mask={use_mask} shared={use_shared}", flush=True)
    with Session() as s:
        y = torch.full((bs, h), 7.0, dtype=tdt, device=DEV)
        d_eo = torch.full((bs * K, h), 0x7f7f, dtype=torch.int16, device=DEV)
        d_eo[:eo.shape[0]] = torch.from_numpy(eo.view(np.int16)).to(DEV)
        d_assist = torch.full((bs * K, 4), -77, dtype=torch.int32, device=DEV)
        d_assist[:assist.shape[0]] = torch.from_numpy(assist).to(DEV)
        torch.cuda.synchronize()
        if route == "memory":
            st = ep.combine_memory_v2(d_eo, d_assist, to_dev(counts), s.comm, bs, h, K, E, y, dtype, s.stream,
                                      expert_scales=to_dev(w) if use_w else None,
                                      active_mask=to_dev(tmask) if use_mask else None,
                                      active_mask_type=ep.MASK_TOKEN if use_mask else ep.MASK_NONE,
                                      shared_expert_x=to_dev(sxb) if use_shared else None)
        else:
            st = ep.combine_v2(d_eo, d_assist, to_dev(counts), s.comm, bs, h, K, E, y, dtype, s.stream)
        assert st == 0
        s.sync()
        small = bs * K <= 2048 and bs * bs * K <= 1 << 20 and h % 8 == 0
        assert (ep.last_kernel_name(s.comm, ep.K_REDUCE) == "ep_reduce_small_kernel") == small
        host_eo = d_eo.cpu().numpy().view(np.uint16)[None]
        host_assist = d_assist.cpu().numpy()[None]
        if route == "memory":
            want = O.mem_combine(case, 0, host_eo, host_assist, counts[None], expert_scales=w if use_w else None,
                                 token_mask=tmask if use_mask else None, shared_expert_x=sxb if use_shared else None)
        else:
            want = O.mvp_combine(case, 0, host_eo, host_assist, counts[None])
        assert np.array_equal(bits16(y), want)


@pytest.mark.parametrize("shape", [(24, 64, 4, 16), (33, 96, 3, 7), (12, 1024, 8, 64), (6, 7168, 8, 256), (9, 40, 2, 4)])
@pytest.mark.parametrize("dtype", [ep.DT_BF16, ep.DT_FP16])
@pytest.mark.parametrize("mode", [3, 4])
def test_memory_combine_mxfp8_exchange_matches_oracle(shape, dtype, mode):
    bs, h, K, E = shape
    rng = np.random.default_rng(sum(shape) + dtype + mode)
    ids = ids_for(rng, bs, K, E)
    xt, xb = x_for(rng, bs, h, dtype, scale=4.0)
    case = O.Case(1, bs, h, K, E, dtype=dtype)
    d = O.mem_dispatch(case, 0, xb[None], ids[None])
    eo = d["expand_x"].view(np.uint16)
    w = (0.5 + rng.random((bs, K))).astype(np.float32)
    with Session() as s:
        y = torch.zeros((bs, h), dtype=torch.bfloat16 if dtype == ep.DT_BF16 else torch.float16, device=DEV)
        st = ep.combine_memory_v2(to_dev(eo), to_dev(d["assist"]), to_dev(d["send_counts"]), s.comm, bs, h, K, E, y,
                                  dtype, s.stream, expert_scales=to_dev(w), quant_mode=mode)
        assert st == 0
        s.sync()
        want = O.mem_combine(case, 0, eo[None], d["assist"][None], d["send_counts"][None], expert_scales=w,
                             comm_quant=mode)
        assert np.array_equal(bits16(y), want)


@pytest.mark.parametrize("shape", [(24, 64, 4, 16), (12, 1024, 6, 64), (10, 2048, 8, 128), (9, 40, 2, 4), (5, 33, 2, 4)])
@pytest.mark.parametrize("dtype", [ep.DT_BF16, ep.DT_FP16])
@pytest.mark.parametrize("quant", [ep.Q_TOKEN_INT8, ep.Q_FP8_BLOCK128])
def test_quantised_combine_matches_oracle(shape, dtype, quant):
    bs, h, K, E = shape
    rng = np.random.default_rng(sum(shape) + dtype + quant)
    ids = ids_for(rng, bs, K, E)
    xt, xb = x_for(rng, bs, h, dtype, scale=2.0)
    d = O.mem_dispatch(O.Case(1, bs, h, K, E, dtype=dtype, quant_mode=quant), 0, xb[None], ids[None])
    w = (0.5 + rng.random((bs, K))).astype(np.float32)
    with Session() as s:
        y = torch.zeros((bs, h), dtype=torch.bfloat16 if dtype == ep.DT_BF16 else torch.float16, device=DEV)
        st = ep.combine_memory_ex(to_dev(d["expand_x"]), to_dev(d["assist"]), to_dev(d["send_counts"]), s.comm, bs, h,
                                  K, E, y, dtype, s.stream, expert_out_quant_mode=quant,
                                  expert_out_scales=to_dev(d["dyn_scales"]), expert_scales=to_dev(w))
        assert st == 0
        s.sync()
        want = O.mem_combine(O.Case(1, bs, h, K, E, dtype=dtype), 0, d["expand_x"][None], d["assist"][None],
                             d["send_counts"][None], expert_scales=w, in_quant=quant, in_scales=d["dyn_scales"])
        assert np.array_equal(bits16(y), want)


@pytest.mark.parametrize("shape", [(7, 8, 2, 5), (64, 64, 4, 16), (16, 33, 2, 4), (60, 1024, 8, 64), (20, 7168, 8, 256)])
@pytest.mark.parametrize("dtype", [ep.DT_FP16, ep.DT_BF16])
def test_mvp_combine_matches_oracle(shape, dtype):
    bs, h, K, E = shape
    rng = np.random.default_rng(sum(shape) + 11 * dtype)
    ids = ids_for(rng, bs, K, E, invalid=0.1)
    xt, xb = x_for(rng, bs, h, dtype, scale=20.0)
    case = O.Case(1, bs, h, K, E, dtype=dtype)
    d = O.mvp_dispatch(case, 0, xb[None], ids[None])
    eo = d["expand_x"].view(np.uint16).copy()
    for r in range(d["rows"]):
        eo[r] = np.roll(eo[r], r % 3)
    with Session() as s:
        y = torch.full((bs, h), 3.0, dtype=torch.bfloat16 if dtype == ep.DT_BF16 else torch.float16, device=DEV)
        st = ep.combine_v2(to_dev(eo), to_dev(d["assist"]), to_dev(d["recv_counts"]), s.comm, bs, h, K, E, y, dtype,
                           s.stream)
        assert st == 0
        s.sync()
        want = O.mvp_combine(case, 0, eo[None], d["assist"][None], d["recv_counts"][None])
        assert np.array_equal(bits16(y), want)


def test_unsupported_requests_are_reported():
    bs, h, K, E = 8, 64, 2, 4
    with Session() as s:
        x = torch.zeros((bs, h), dtype=torch.bfloat16, device=DEV)
        ids = torch.zeros((bs, K), dtype=torch.int32, device=DEV)
        out = alloc_dispatch_outputs(bs, h, K, E)
        counts = torch.zeros((E,), dtype=torch.int32, device=DEV)
        base = (x, ids, s.comm, bs, h, K, E, out["expand_x"], out["assist"], out["token_nums"], counts, ep.DT_BF16)
        assert ep.dispatch_memory_v2(*base, None) == ep.ERR_PARA_CHECK_FAIL                 # null stream
        assert ep.dispatch_memory_v2(*base, s.stream, quant_mode=2) == ep.ERR_NOT_SUPPORT
        assert ep.dispatch_memory_v2(*base, s.stream, tp_world_size=2) == ep.ERR_NOT_SUPPORT
        assert ep.dispatch_memory_v2(*base, s.stream, global_bs=bs + 1) == ep.ERR_PARA_CHECK_FAIL
        assert ep.dispatch_memory_v2(*base, s.stream, ep_world_size=2) == ep.ERR_PARA_CHECK_FAIL
        assert ep.dispatch_memory_v2(*base, s.stream, active_mask_type=ep.MASK_TOKEN) == ep.ERR_PARA_CHECK_FAIL
        assert ep.dispatch_v2(*base, s.stream, quant_mode=3) == ep.ERR_NOT_SUPPORT
        assert ep.dispatch_v2(*base, s.stream, quant_mode=2) == ep.ERR_PARA_CHECK_FAIL      # needs int8 + scales out
        st, _ = ep.dispatch_memory_ex(*base, s.stream, quant_mode=1)
        assert st == ep.ERR_NOT_SUPPORT
        st, _ = ep.dispatch_memory_ex(*base, s.stream, quant_mode=5)                         # no scales buffer
        assert st == ep.ERR_PARA_CHECK_FAIL
        y = torch.zeros((bs, h), dtype=torch.bfloat16, device=DEV)
        cb = (out["expand_x"], out["assist"], counts, s.comm, bs, h, K, E, y, ep.DT_BF16, s.stream)
        assert ep.combine_memory_v2(*cb, quant_mode=2) == ep.ERR_NOT_SUPPORT
        assert ep.combine_memory_v2(*cb, quant_mode=4) == ep.ERR_PARA_CHECK_FAIL            # needs expertScales
        assert ep.combine_memory_v2(*cb, active_mask_type=ep.MASK_EXPERT, active_mask=y) == ep.ERR_NOT_SUPPORT
        assert ep.combine_v2(out["expand_x"], out["assist"], counts, s.comm, bs, h, K, E, y, ep.DT_INT8, s.stream) == \
            ep.ERR_NOT_SUPPORT
        # nothing above consumed a magic or launched anything
        assert s.comm.next_magic() == 1


# ---------------------------------------------------------------------------------------------
# Degenerate and extreme routing tables (both dispatch paths: one launch for small batches, count + scatter above)
# ---------------------------------------------------------------------------------------------
def _edge_ids(kind, rng, bs, K, E):
    if kind == "all_invalid":
        return rng.choice([-1, -5, E, E + 9], size=(bs, K)).astype(np.int32)
    if kind == "one_expert":
        return np.full((bs, K), E - 1, np.int32)                       # every route, duplicates within a token too
    if kind == "duplicates":
        ids = rng.integers(0, E, size=(bs, K)).astype(np.int32)
        ids[:, 1:] = ids[:, :1]                                         # a token names the same expert K times
        return ids
    if kind == "last_token_only":
        ids = np.full((bs, K), -1, np.int32)
        ids[-1] = rng.permutation(E)[:K]
        return ids
    raise ValueError(kind)


@pytest.mark.parametrize("kind", ["all_invalid", "one_expert", "duplicates", "last_token_only"])
@pytest.mark.parametrize("shape", [(1, 8, 1, 1), (3, 64, 64, 64), (200, 40, 8, 2048), (300, 1024, 8, 2048), (1500, 256, 2, 7)])
def test_degenerate_routing_tables(kind, shape):
    bs, h, K, E = shape
    rng = np.random.default_rng(sum(shape))
    ids = _edge_ids(kind, rng, bs, K, E)
    xt, xb = x_for(rng, bs, h, ep.DT_BF16)
    w = rng.random((bs, K)).astype(np.float32)
    with Session() as s:
        for capacity in (0, 3):
            out = alloc_dispatch_outputs(bs, h, K, E)
            counts = torch.full((E,), -1, dtype=torch.int32, device=DEV)
            st, _ = ep.dispatch_memory_ex(xt, to_dev(ids), s.comm, bs, h, K, E, out["expand_x"], out["assist"],
                                          out["token_nums"], counts, ep.DT_BF16, s.stream, expert_capacity=capacity,
                                          row_index_map=out["row_map"])
            assert st == 0
            y = torch.full((bs, h), 9.0, dtype=torch.bfloat16, device=DEV)
            assert ep.combine_memory_ex(out["expand_x"], out["assist"], counts, s.comm, bs, h, K, E, y, ep.DT_BF16,
                                        s.stream, expert_scales=to_dev(w), row_index_map=out["row_map"]) == 0
            s.sync()
            case = O.Case(1, bs, h, K, E, dtype=O.DT_BF16, capacity=capacity, token_nums_type=1)
            want = O.mem_dispatch(case, 0, xb[None], ids[None])
            got = fetch(out, "send_counts", counts)
            check_dispatch(got, want)
            assert np.array_equal(got["send_counts"], want["send_counts"])
            # the row map is the inverse of the tuples, -1 where a route has no row
            rm = np.full(bs * K, -1, np.int32)
            n = want["rows"]
            rm[want["assist"][:n, 1] * K + want["assist"][:n, 2]] = np.arange(n, dtype=np.int32)
            assert np.array_equal(got["row_map"].reshape(-1), rm)
            wy = O.mem_combine(O.Case(1, bs, h, K, E, dtype=O.DT_BF16), 0, want["expand_x"].view(np.uint16)[None],
                               want["assist"][None], want["send_counts"][None], expert_scales=w)
            assert np.array_equal(bits16(y), wy)
            if kind == "all_invalid":
                assert n == 0 and not bits16(y).any()


# ---------------------------------------------------------------------------------------------
# Every finite 16-bit input pattern through the device quantisers and the device reduce
# ---------------------------------------------------------------------------------------------
def _all_finite_patterns(dtype, seed):
    """[128, 512] uint16 holding every finite bf16 / fp16 bit pattern once (non-finite ones replaced by zero), shuffled
    so that every pattern meets different row and block maxima under different seeds."""
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    exp_all_ones = (bits & 0x7f80) == 0x7f80 if dtype == ep.DT_BF16 else (bits & 0x7c00) == 0x7c00
    bits[exp_all_ones] = 0
    np.random.default_rng(seed).shuffle(bits)
    return bits.reshape(128, 512)


@pytest.mark.parametrize("dtype", [ep.DT_BF16, ep.DT_FP16])
@pytest.mark.parametrize("quant,fp8", [(ep.Q_TOKEN_INT8, None), (ep.Q_MXFP8, ep.DT_FP8E4M3), (ep.Q_MXFP8, ep.DT_FP8E5M2),
                                       (ep.Q_FP8_BLOCK128, None)])
def test_device_quantisers_on_every_finite_input_pattern(dtype, quant, fp8):
    bs, h, K, E = 128, 512, 1, 4
    for seed in (1, 2, 3):
        xb = _all_finite_patterns(dtype, seed)
        if seed == 3:
            # moderate magnitudes only: the first two seeds put a huge element into nearly every block, which sends
            # almost everything else to zero; here the small values get quantised for real
            big = (xb & 0x7fff) > (0x4300 if dtype == ep.DT_BF16 else 0x5800)
            xb = np.where(big, xb & 0x80ff, xb).astype(np.uint16)
        xt = torch.from_numpy(xb.view(np.int16)).view(torch.bfloat16 if dtype == ep.DT_BF16 else torch.float16).to(DEV)
        ids = (np.arange(bs, dtype=np.int32) % E).reshape(bs, K)
        with Session() as s:
            out = alloc_dispatch_outputs(bs, h, K, E, quant=quant)
            counts = torch.zeros((E,), dtype=torch.int32, device=DEV)
            st, _ = ep.dispatch_memory_ex(xt, to_dev(ids), s.comm, bs, h, K, E, out["expand_x"], out["assist"],
                                          out["token_nums"], counts, dtype, s.stream, quant_mode=quant,
                                          dynamic_scales=out["scales"], expand_x_dtype=fp8)
            assert st == 0
            s.sync()
            got = fetch(out, "send_counts", counts)
            case = O.Case(1, bs, h, K, E, dtype=dtype, quant_mode=quant, out_dtype=fp8 or O.DT_FP8E4M3)
            want = O.mem_dispatch(case, 0, xb[None], ids[None])
            assert want["rows"] == bs
            assert np.array_equal(got["expand_x"], want["expand_x"]), f"seed {seed}"
            assert np.array_equal(got["scales"].reshape(bs, -1), want["dyn_scales"].reshape(bs, -1)), f"seed {seed}"


@pytest.mark.parametrize("dtype", [ep.DT_BF16, ep.DT_FP16])
@pytest.mark.parametrize("comm_quant", [0, 3, 4])
def test_device_reduce_on_every_finite_input_pattern(dtype, comm_quant):
    """Rows holding every finite pattern, weights that are not powers of two, three rows per token: the fp32 multiply,
    the adds in k order, the MXFP8 exchange round trip and the final rounding all see every input once."""
    bs, h, K, E = 128, 512, 3, 8
    rng = np.random.default_rng(17 + dtype + comm_quant)
    rows = np.concatenate([_all_finite_patterns(dtype, seed) for seed in (5, 6, 7)])          # [384, 512]
    if dtype == ep.DT_FP16:
        rows = np.where((rows & 0x7fff) > 0x7000, rows & 0x8fff, rows).astype(np.uint16)     # keep sums finite
    ids = np.stack([rng.permutation(E)[:K] for _ in range(bs)]).astype(np.int32)
    w = (rng.random((bs, K)) * 1.7 + 0.05).astype(np.float32)
    # a layout to combine over: dispatch a dummy x, then put the pattern rows in place of the expert outputs
    tdt = torch.bfloat16 if dtype == ep.DT_BF16 else torch.float16
    with Session() as s:
        out = alloc_dispatch_outputs(bs, h, K, E)
        counts = torch.zeros((E,), dtype=torch.int32, device=DEV)
        xt = torch.zeros((bs, h), dtype=tdt, device=DEV)
        st, _ = ep.dispatch_memory_ex(xt, to_dev(ids), s.comm, bs, h, K, E, out["expand_x"], out["assist"],
                                      out["token_nums"], counts, dtype, s.stream, row_index_map=out["row_map"])
        assert st == 0
        expert_out = torch.from_numpy(rows.view(np.int16)).view(tdt).to(DEV)
        y = torch.zeros((bs, h), dtype=tdt, device=DEV)
        assert ep.combine_memory_v2(expert_out, out["assist"], counts, s.comm, bs, h, K, E, y, dtype, s.stream,
                                    expert_scales=to_dev(w), quant_mode=comm_quant) == 0
        s.sync()
        case = O.Case(1, bs, h, K, E, dtype=dtype)
        wy = O.mem_combine(case, 0, rows[None], out["assist"].cpu().numpy()[None], counts.cpu().numpy()[None],
                           expert_scales=w, comm_quant=comm_quant)
        assert np.array_equal(bits16(y), wy)


@pytest.mark.parametrize("dtype", [ep.DT_BF16, ep.DT_FP16])
@pytest.mark.parametrize("quant", [ep.Q_TOKEN_INT8, ep.Q_FP8_BLOCK128])
def test_quantised_combine_input_on_every_code(dtype, quant):
    """Every int8 value / every e4m3 code that is a number, under scales spread over the fp32 range that keep the
    dequantised values finite in the output type: dequantise, round to the element type, weight, sum."""
    bs, h, K, E = 64, 512, 2, 4
    rng = np.random.default_rng(23 + dtype + quant)
    n = bs * K
    ids = np.stack([rng.permutation(E)[:K] for _ in range(bs)]).astype(np.int32)
    codes = np.arange(256, dtype=np.uint8)
    if quant == ep.Q_FP8_BLOCK128:
        codes = codes[(codes & 0x7f) != 0x7f]                       # 0x7f / 0xff are NaN codes
    payload = rng.choice(codes, size=(n, h)).astype(np.uint8)
    payload[:, :codes.size] = codes                                 # every code in every row
    top = 200.0 if dtype == ep.DT_FP16 else 1e30                    # code 448 * scale stays finite in fp16
    if quant == ep.Q_TOKEN_INT8:
        scales = np.exp(rng.uniform(np.log(1e-30), np.log(top), size=(n, 1))).astype(np.float32)
    else:
        scales = np.exp(rng.uniform(np.log(1e-30), np.log(top / 4), size=(n, h // 128))).astype(np.float32)
    w = (0.3 + rng.random((bs, K))).astype(np.float32)
    tdt = torch.bfloat16 if dtype == ep.DT_BF16 else torch.float16
    with Session() as s:
        out = alloc_dispatch_outputs(bs, h, K, E)
        counts = torch.zeros((E,), dtype=torch.int32, device=DEV)
        xt = torch.zeros((bs, h), dtype=tdt, device=DEV)
        st, _ = ep.dispatch_memory_ex(xt, to_dev(ids), s.comm, bs, h, K, E, out["expand_x"], out["assist"],
                                      out["token_nums"], counts, dtype, s.stream, row_index_map=out["row_map"])
        assert st == 0
        y = torch.zeros((bs, h), dtype=tdt, device=DEV)
        assert ep.combine_memory_ex(to_dev(payload), out["assist"], counts, s.comm, bs, h, K, E, y, dtype, s.stream,
                                    expert_out_quant_mode=quant, expert_out_scales=to_dev(scales),
                                    expert_scales=to_dev(w)) == 0
        s.sync()
        want = O.mem_combine(O.Case(1, bs, h, K, E, dtype=dtype), 0, payload[None], out["assist"].cpu().numpy()[None],
                             counts.cpu().numpy()[None], expert_scales=w, in_quant=quant, in_scales=scales)
        assert np.array_equal(bits16(y), want)


# ---------------------------------------------------------------------------------------------------------------
# corrupted assist tuples, counts and row maps: skipped, never followed
# (reference: src/ep/kernels/tilexr_ep_combine_memory_kernel.h:256-266, 340-342; tilexr_ep_combine_kernel.cpp:94-97)
# ---------------------------------------------------------------------------------------------------------------
def _guarded(bs, h, dtype, fill):
    """y as the middle of a larger buffer whose edges must stay as they are."""
    tdt = torch.bfloat16 if dtype == ep.DT_BF16 else torch.float16
    whole = torch.full((bs + 64, h), fill, dtype=tdt, device=DEV)
    return whole, whole[32:32 + bs]


@pytest.mark.parametrize("shape", [(64, 64, 4, 16), (300, 1024, 8, 64), (2100, 256, 8, 256), (40, 7168, 8, 256)])
@pytest.mark.parametrize("route", ["memory", "mvp"])
def test_combine_skips_corrupted_tuples(shape, route):
    from test_oracle_routes import corrupt_tuples
    bs, h, K, E = shape
    dtype = ep.DT_BF16 if route == "memory" else ep.DT_FP16
    rng = np.random.default_rng(sum(shape) + len(route))
    ids = ids_for(rng, bs, K, E, invalid=0.05)
    _, xb = x_for(rng, bs, h, dtype, scale=3.0)
    case = O.Case(1, bs, h, K, E, dtype=dtype)
    d = (O.mem_dispatch if route == "memory" else O.mvp_dispatch)(case, 0, xb[None], ids[None])
    rows = d["rows"]
    counts_key = "send_counts" if route == "memory" else "recv_counts"
    eo = d["expand_x"].view(np.uint16).copy()
    for r in range(rows):
        eo[r] = np.roll(eo[r], r % 5)
    assist = d["assist"].copy()
    corrupt_tuples(rng, assist[None], [rows], bs, K, 1, max(6, rows // 10))
    if route == "memory":
        # a duplicate: a later row that claims the slot of an intact earlier one (the later row wins)
        intact = [r for r in range(rows) if np.array_equal(assist[r], d["assist"][r])]
        assist[intact[-1], :3] = assist[intact[0], :3]
    w = (0.25 + rng.random((bs, K))).astype(np.float32)
    for count_case in ("as dispatched", "past the buffer", "negative"):
        counts = d[counts_key].copy()
        if count_case == "past the buffer":
            counts[-1] = bs * K + 12345 if route == "memory" else bs * K + 1       # MVP: outside [0, bs*K] reads as 0
        elif count_case == "negative":
            counts[-1] = -7
        with Session() as s:
            whole, y = _guarded(bs, h, dtype, 9.0)
            d_eo = torch.full((bs * K, h), 0x7f7f, dtype=torch.int16, device=DEV)      # rows past `rows` hold 3.4e38
            d_eo[:eo.shape[0]] = torch.from_numpy(eo.view(np.int16)).to(DEV)
            d_assist = torch.full((bs * K, 4), -77, dtype=torch.int32, device=DEV)
            d_assist[:assist.shape[0]] = torch.from_numpy(assist).to(DEV)
            torch.cuda.synchronize()
            print(f"corrupted tuples: {route} {shape} counts {count_case}", flush=True)
            if route == "memory":
                st = ep.combine_memory_v2(d_eo, d_assist, to_dev(counts), s.comm, bs, h, K, E, y, dtype, s.stream,
                                          expert_scales=to_dev(w))
            else:
                st = ep.combine_v2(d_eo, d_assist, to_dev(counts), s.comm, bs, h, K, E, y, dtype, s.stream)
            assert st == 0
            s.sync()
            host_eo = d_eo.cpu().numpy().view(np.uint16)[None]
            host_assist = d_assist.cpu().numpy()[None]
            if route == "memory":
                want = O.mem_combine(case, 0, host_eo, host_assist, counts[None], expert_scales=w)
            else:
                want = O.mvp_combine(case, 0, host_eo, host_assist, counts[None])
            assert np.array_equal(bits16(y), want), count_case
            edges = torch.cat([whole[:32], whole[32 + bs:]])
            assert torch.all(edges == 9.0)                  # nothing was stored outside y


@pytest.mark.parametrize("h", [1024, 7168])
@pytest.mark.parametrize("quant", [ep.Q_NONE, ep.Q_TOKEN_INT8, ep.Q_FP8_BLOCK128])
def test_combine_with_rows_missing_in_any_pattern_of_slots(quant, h):
    """The reduce takes the slots of a token that have a row first, in k order, a few at a time; the sum must be the
    one the oracle forms by walking all slots.  Every token here loses a random subset of its eight rows (a tuple whose
    token is -1 stands for no row): none, all, the leading ones, more than one batch's worth left, exactly one left."""
    bs, K, E = 96, 8, 32
    rng = np.random.default_rng(h + quant)
    ids = ids_for(rng, bs, K, E)
    xt, xb = x_for(rng, bs, h, ep.DT_BF16, scale=2.0)
    d = O.mem_dispatch(O.Case(1, bs, h, K, E, dtype=ep.DT_BF16, quant_mode=quant), 0, xb[None], ids[None])
    w = (0.5 + rng.random((bs, K))).astype(np.float32)
    keep = rng.random((bs, K)) < rng.random((bs, 1))          # a different share of rows kept for every token
    keep[0], keep[1], keep[2, :5], keep[2, 5:] = True, False, False, True
    keep[3], keep[3, 6] = False, True
    assist = d["assist"].copy()
    lost = ~keep[assist[:, 1], assist[:, 2]]
    assist[lost, 1] = -1
    assert 0 < lost.sum() < bs * K
    with Session() as s:
        y = torch.full((bs, h), 7.0, dtype=torch.bfloat16, device=DEV)
        eo = to_dev(d["expand_x"]) if quant else to_dev(d["expand_x"].view(np.uint16))
        st = ep.combine_memory_ex(eo, to_dev(assist), to_dev(d["send_counts"]), s.comm, bs, h, K, E, y, ep.DT_BF16,
                                  s.stream, expert_out_quant_mode=quant,
                                  expert_out_scales=to_dev(d["dyn_scales"]) if quant else None, expert_scales=to_dev(w))
        assert st == 0
        s.sync()
        host_eo = d["expand_x"][None] if quant else d["expand_x"].view(np.uint16)[None]
        want = O.mem_combine(O.Case(1, bs, h, K, E, dtype=ep.DT_BF16), 0, host_eo, assist[None], d["send_counts"][None],
                             expert_scales=w, in_quant=quant, in_scales=d["dyn_scales"] if quant else None)
        assert np.array_equal(bits16(y), want)
        assert np.all(bits16(y)[1] == 0)


def test_combine_ignores_row_map_entries_outside_the_buffer():
    """The row map dispatch hands to combine is trusted input, but an entry at or beyond bs * topK (or below -1) must
    read as "no row": the kernels never touch memory outside the rows the caller's buffer holds."""
    bs, h, K, E = 200, 1024, 4, 32
    rng = np.random.default_rng(5)
    ids = ids_for(rng, bs, K, E)
    xt, xb = x_for(rng, bs, h, ep.DT_BF16)
    case = O.Case(1, bs, h, K, E, dtype=O.DT_BF16)
    d = O.mem_dispatch(case, 0, xb[None], ids[None])
    w = (0.25 + rng.random((bs, K))).astype(np.float32)
    with Session() as s:
        out = alloc_dispatch_outputs(bs, h, K, E)
        counts = torch.zeros((E,), dtype=torch.int32, device=DEV)
        st, _ = ep.dispatch_memory_ex(xt, to_dev(ids), s.comm, bs, h, K, E, out["expand_x"], out["assist"],
                                      out["token_nums"], counts, ep.DT_BF16, s.stream, row_index_map=out["row_map"])
        assert st == 0
        s.sync()
        row_map = out["row_map"].cpu().numpy().copy()
        assist = d["assist"].copy()
        for j, (t, k) in enumerate([(0, 0), (5, 3), (77, 1), (199, 3), (100, 2)]):
            row = row_map[t, k]
            row_map[t, k] = [bs * K, 0x7fffffff, -5, bs * K + 7, -2147483648][j]
            assist[row, 1] = -1                     # the oracle learns of the same loss through the tuple
        whole, y = _guarded(bs, h, ep.DT_BF16, 9.0)
        torch.cuda.synchronize()
        st = ep.combine_memory_ex(out["expand_x"], out["assist"], counts, s.comm, bs, h, K, E, y, ep.DT_BF16, s.stream,
                                  expert_scales=to_dev(w), row_index_map=to_dev(row_map))
        assert st == 0
        s.sync()
        want = O.mem_combine(case, 0, d["expand_x"].view(np.uint16)[None], assist[None], d["send_counts"][None],
                             expert_scales=w)
        assert np.array_equal(bits16(y), want)
        assert torch.all(torch.cat([whole[:32], whole[32 + bs:]]) == 9.0)
