"""Pins the CPU oracle's dispatch / combine data movement: row order, counts, source-index map and reductions.

Pins used: the reference checker's known answers (tests/checker/unit/test_checker_oracles.cpp:279-323,
test_checker_executor.cpp:389-401), the reference checker compiled in place (oracle/_ref: ExpectedEpDispatchRoutes
and the executor's output blobs), numpy stable sorts / bincount / cumsum as an independent model of the
memory-route order (design: local expert -> source rank -> route order), brute force for the capacity rule and
numpy sequential float16 / float32 sums for the two combine contracts.
"""
import numpy as np
import pytest
import torch

from oracle import ep as O


def rand_ids(rng, R, bs, K, E, invalid_frac=0.0):
    ids = np.stack([np.stack([rng.permutation(E)[:K] for _ in range(bs)]) for _ in range(R)]).astype(np.int32)
    if invalid_frac:
        bad = rng.random(ids.shape) < invalid_frac
        ids[bad] = rng.choice([-1, -7, E, E + 5], size=int(bad.sum()))
    return ids


def rand_x(rng, R, bs, h):
    return rng.integers(0, 0x7bff, size=(R, bs, h), dtype=np.uint16)


# ---------------------------------------------------------------------------------------------
# MVP route vs the reference checker
# ---------------------------------------------------------------------------------------------
def test_mvp_checker_known_answers(known, orc):
    k = known["checker_case"]
    s = k["shape"]
    case = O.Case(s["rank_size"], s["bs"], s["h"], s["top_k"], s["moe_expert_num"], dtype=s["dtype"])
    # DefaultEpDispatchExpertIds (tools/checker/src/oracle.cpp:422-445), restated for the known answers
    ids = np.zeros((s["bs"], s["top_k"]), np.int32)
    le = case.local_experts
    for t in range(s["bs"]):
        for kk in range(s["top_k"]):
            grp = t % s["rank_size"] if kk % 2 == 0 else s["rank_size"] - 1 - (t % s["rank_size"])
            loc = ((0 if kk % 2 == 0 else le - 1) + kk // 2) % le
            ids[t, kk] = (grp * le + loc) % s["moe_expert_num"]
    assert ids.size == k["default_ids_len"] and ids.reshape(-1)[:2].tolist() == k["default_ids_first"]
    iv = k["input_value"]
    assert (0x1000 + iv["rank"] * 0x100 + iv["token"] * 0x10 + iv["h"]) & 0xffff == iv["value"]
    x = np.zeros((s["rank_size"], s["bs"], s["h"]), np.uint16)
    for r in range(s["rank_size"]):
        for t in range(s["bs"]):
            for hh in range(s["h"]):
                x[r, t, hh] = (0x1000 + r * 0x100 + t * 0x10 + hh) & 0xffff
    all_ids = np.broadcast_to(ids, (s["rank_size"],) + ids.shape).copy()
    out = orc.mvp_dispatch(case, 1, x, all_ids)
    assert out["rows"] == k["rank1_route_count"]
    assert out["assist"][0].tolist() == k["rank1_first_route"]
    assert out["recv_counts"][0] == k["rank1_recv_count_src0"]
    assert out["expert_token_nums"][0] == k["rank1_local_expert0_count"]
    # payload rows are byte copies of the source rows
    for row in range(out["rows"]):
        src, tok = out["assist"][row][:2]
        assert np.array_equal(out["expand_x"][row].view(np.uint16), x[src, tok])


@pytest.mark.parametrize("shape", [(2, 3, 4, 2, 4), (4, 16, 8, 2, 16), (4, 9, 8, 3, 8), (8, 5, 8, 4, 32), (1, 7, 8, 2, 5)])
def test_mvp_routes_match_compiled_checker(ref, orc, shape):
    R, bs, h, K, E = shape
    rng = np.random.default_rng(sum(shape))
    ids = rand_ids(rng, 1, bs, K, E, invalid_frac=0.15)[0]
    x = rand_x(rng, R, bs, h)
    case = O.Case(R, bs, h, K, E, dtype=O.DT_FP16)
    all_ids = np.broadcast_to(ids, (R,) + ids.shape).copy()
    for dst in range(R):
        want = ref.checker_routes(R, bs, K, E, ids, dst)
        got = orc.mvp_dispatch(case, dst, x, all_ids)
        assert got["rows"] == len(want)
        assert np.array_equal(got["assist"][: len(want)], want)
        assert np.array_equal(got["recv_counts"], np.bincount(want[:, 0], minlength=R))
        le = case.local_experts
        assert np.array_equal(got["expert_token_nums"], np.bincount(want[:, 3] % le, minlength=le))


@pytest.mark.parametrize("shape,dtype", [((2, 3, 4, 2, 4), 3), ((4, 8, 16, 2, 8), 11), ((4, 128, 1024, 2, 16), 11)])
def test_mvp_dispatch_and_restore_match_checker_blobs(ref, orc, shape, dtype):
    """The checker's executor output blob: [R*bs*K*h payload | bs*K assist | R int32 | localE int64]
    (tools/checker/src/oracle.cpp:661-708); ep_combine restores rows to [bs, K, h] (executor.cpp:471-541)."""
    R, bs, h, K, E = shape
    st, blobs, events = ref.checker_run(0, R, bs, h, K, E, dtype)
    assert st == 0
    ids = ref.checker_default_ids(R, bs, K, E)
    x = np.zeros((R, bs, h), np.uint16)
    tt, hh = np.meshgrid(np.arange(bs), np.arange(h), indexing="ij")
    for r in range(R):
        x[r] = (0x1000 + r * 0x100 + tt * 0x10 + hh) & 0xffff
    case = O.Case(R, bs, h, K, E, dtype=dtype)
    all_ids = np.broadcast_to(ids, (R,) + ids.shape).copy()
    payload_bytes = R * bs * K * h * 2
    assist_bytes = bs * K * 16
    le = case.local_experts
    for dst in range(R):
        got = orc.mvp_dispatch(case, dst, x, all_ids)
        n = got["rows"]
        assert n == bs * K          # the checker's default ids are balanced (oracle.cpp:432-441)
        blob = blobs[dst]
        assert np.array_equal(blob[: n * h * 2], got["expand_x"][:n].reshape(-1))
        assert np.array_equal(blob[payload_bytes: payload_bytes + assist_bytes].view(np.int32).reshape(-1, 4),
                              got["assist"][:n])
        off = payload_bytes + assist_bytes
        assert np.array_equal(blob[off: off + 4 * R].view(np.int32), got["recv_counts"])
        assert np.array_equal(blob[off + 4 * R: off + 4 * R + 8 * le].view(np.int64), got["expert_token_nums"])
    if shape == (4, 128, 1024, 2, 16):
        assert events == 4148       # event count the reference CLI reports for this configuration
    # inverse route: every source rank gets its rows back at [token, k]
    st, cblobs, cevents = ref.checker_run(1, R, bs, h, K, E, dtype)
    assert st == 0
    for r in range(R):
        restored = cblobs[r].view(np.uint16).reshape(bs, K, h)
        assert np.array_equal(restored, np.broadcast_to(x[r][:, None, :], (bs, K, h)))
    if shape == (4, 128, 1024, 2, 16):
        assert cevents == 6164


def test_mvp_token_mask_and_prefix_type(orc):
    rng = np.random.default_rng(4)
    R, bs, h, K, E = 2, 10, 8, 3, 8
    ids = rand_ids(rng, R, bs, K, E, 0.1)
    x = rand_x(rng, R, bs, h)
    mask = (rng.random((R, bs)) < 0.6).astype(np.uint8)
    base = orc.mvp_dispatch(O.Case(R, bs, h, K, E, token_nums_type=1), 0, x, ids, mask)
    pref = orc.mvp_dispatch(O.Case(R, bs, h, K, E, token_nums_type=0), 0, x, ids, mask)
    assert np.array_equal(np.cumsum(base["expert_token_nums"]), pref["expert_token_nums"])
    # every emitted route comes from an active token and nothing else is emitted
    a = base["assist"][: base["rows"]]
    assert all(mask[s, t] for s, t in a[:, :2])
    expected = sum(int(mask[s, t]) and 0 <= ids[s, t, k] < E and ids[s, t, k] // (E // R) == 0
                   for s in range(R) for t in range(bs) for k in range(K))
    assert base["rows"] == expected


# ---------------------------------------------------------------------------------------------
# memory route
# ---------------------------------------------------------------------------------------------
def np_memory_order(case, dst, ids, live):
    """Independent model: stable sort of live routes by (local expert, source rank), keeping flat order."""
    R, bs, K = ids.shape
    le = case.local_experts
    src, tok, k = np.meshgrid(np.arange(R), np.arange(bs), np.arange(K), indexing="ij")
    flat = np.stack([src.ravel(), tok.ravel(), k.ravel(), ids.ravel()], axis=1)
    ok = live.ravel() & (flat[:, 3] >= 0) & (flat[:, 3] < case.moe_expert_num)
    ok &= np.where(ok, flat[:, 3] // le == dst, False)
    sel = flat[ok]
    key = (sel[:, 3] % le) * R + sel[:, 0]
    order = np.argsort(key, kind="stable")
    return sel[order], np.cumsum(np.bincount(key, minlength=le * R))


@pytest.mark.parametrize("shape", [(1, 16, 8, 2, 4), (1, 64, 16, 8, 32), (2, 12, 8, 2, 8), (4, 20, 8, 3, 16)])
@pytest.mark.parametrize("mask_type", [O.MASK_NONE, O.MASK_TOKEN, O.MASK_EXPERT])
def test_memory_order_and_counts(orc, shape, mask_type):
    R, bs, h, K, E = shape
    rng = np.random.default_rng(sum(shape) + mask_type)
    ids = rand_ids(rng, R, bs, K, E, 0.1)
    x = rand_x(rng, R, bs, h)
    mask = None
    live = np.ones((R, bs, K), bool)
    if mask_type == O.MASK_TOKEN:
        mask = (rng.random((R, bs)) < 0.7).astype(np.uint8)
        # prefix semantics (tilexr_ep_dispatch_memory_kernel.h:1387-1410,1538-1544): the first sum(mask) tokens
        for r in range(R):
            live[r] = (np.arange(bs) < mask[r].sum())[:, None]
    elif mask_type == O.MASK_EXPERT:
        mask = (rng.random((R, bs, K)) < 0.7).astype(np.uint8)
        live = mask.astype(bool)
    for nums_type in (0, 1):
        case = O.Case(R, bs, h, K, E, dtype=O.DT_BF16, mask_type=mask_type, token_nums_type=nums_type)
        for dst in range(R):
            got = orc.mem_dispatch(case, dst, x, ids, mask)
            want, send = np_memory_order(case, dst, ids, live)
            assert got["rows"] == len(want)
            assert np.array_equal(got["assist"][: len(want)], want)
            assert np.array_equal(got["send_counts"], send)
            per_expert = send[R - 1:: R]
            want_nums = per_expert if nums_type == 0 else np.diff(np.concatenate([[0], per_expert]))
            assert np.array_equal(got["expert_token_nums"], want_nums)
            for row in range(got["rows"]):
                s, t = got["assist"][row][:2]
                assert np.array_equal(got["expand_x"][row].view(np.uint16), x[s, t])


def test_memory_route_is_a_permutation_of_the_mvp_route(orc):
    rng = np.random.default_rng(8)
    R, bs, h, K, E = 4, 24, 8, 3, 16
    ids = rand_ids(rng, R, bs, K, E, 0.05)
    x = rand_x(rng, R, bs, h)
    case = O.Case(R, bs, h, K, E)
    for dst in range(R):
        a = orc.mvp_dispatch(case, dst, x, ids)
        b = orc.mem_dispatch(case, dst, x, ids)
        assert a["rows"] == b["rows"]
        sa = {tuple(t) for t in a["assist"][: a["rows"]]}
        sb = {tuple(t) for t in b["assist"][: b["rows"]]}
        assert sa == sb and len(sa) == a["rows"]
        # expert counts agree between the two routes
        assert np.array_equal(a["expert_token_nums"], b["expert_token_nums"])


def test_capacity_drops_highest_route_indices(orc):
    """ext rule: per (source rank, expert) keep the `capacity` lowest flat route indices."""
    rng = np.random.default_rng(13)
    R, bs, h, K, E, cap = 2, 40, 8, 4, 8, 5
    ids = rand_ids(rng, R, bs, K, E)
    x = rand_x(rng, R, bs, h)
    case = O.Case(R, bs, h, K, E, capacity=cap)
    le = case.local_experts
    for dst in range(R):
        got = orc.mem_dispatch(case, dst, x, ids)
        want = []
        for e in range(dst * le, (dst + 1) * le):
            for s in range(R):
                flat = [i for i in range(bs * K) if ids[s].reshape(-1)[i] == e][:cap]
                want += [(s, i // K, i % K, e) for i in flat]
        assert got["rows"] == len(want)
        assert [tuple(t) for t in got["assist"][: got["rows"]]] == want
    # a capacity at least as large as the biggest bucket changes nothing
    big = orc.mem_dispatch(O.Case(R, bs, h, K, E, capacity=bs * K), 0, x, ids)
    none = orc.mem_dispatch(O.Case(R, bs, h, K, E), 0, x, ids)
    assert big["rows"] == none["rows"] and np.array_equal(big["assist"], none["assist"])


def test_memory_dispatch_quantised_payloads(orc):
    rng = np.random.default_rng(17)
    R, bs, h, K, E = 1, 12, 160, 2, 4
    ids = rand_ids(rng, R, bs, K, E)
    xf = torch.from_numpy((rng.standard_normal((R, bs, h)) * 2).astype(np.float32)).to(torch.bfloat16)
    x = xf.view(torch.int16).numpy().view(np.uint16)
    plain = orc.mem_dispatch(O.Case(R, bs, h, K, E), 0, x, ids)
    for mode in (O.Q_TOKEN_INT8, O.Q_MXFP8, O.Q_FP8_BLOCK128):
        case = O.Case(R, bs, h, K, E, quant_mode=mode)
        got = orc.mem_dispatch(case, 0, x, ids)
        assert got["rows"] == plain["rows"] and np.array_equal(got["assist"], plain["assist"])
        for row in range(got["rows"]):
            tok = got["assist"][row][1]
            if mode == O.Q_TOKEN_INT8:
                q, s = orc.quant_row_token_int8(x[0, tok], O.DT_BF16)
                assert np.array_equal(got["expand_x"][row].view(np.int8), q) and got["dyn_scales"][row, 0] == s
            elif mode == O.Q_MXFP8:
                q, s = orc.quant_row_mxfp8(x[0, tok], O.DT_BF16, O.DT_FP8E4M3)
                assert np.array_equal(got["expand_x"][row], q) and np.array_equal(got["dyn_scales"][row], s)
            else:
                q, s = orc.quant_row_fp8_block128(x[0, tok], O.DT_BF16)
                assert np.array_equal(got["expand_x"][row], q) and np.array_equal(got["dyn_scales"][row], s)


# ---------------------------------------------------------------------------------------------
# combine
# ---------------------------------------------------------------------------------------------
def _dispatch_all(orc, case, x, ids, memory):
    R = case.rank_size
    outs = [(orc.mem_dispatch if memory else orc.mvp_dispatch)(case, d, x, ids) for d in range(R)]
    expert_out = np.stack([o["expand_x"].view(np.uint16) for o in outs])
    assist = np.stack([o["assist"] for o in outs])
    counts = np.stack([o["send_counts" if memory else "recv_counts"] for o in outs])
    return expert_out, assist, counts


def test_mvp_combine_is_a_sequential_float16_sum(orc):
    rng = np.random.default_rng(23)
    R, bs, h, K, E = 2, 6, 32, 4, 8
    ids = rand_ids(rng, R, bs, K, E, 0.1)
    xf = (rng.standard_normal((R, bs, h)) * 30).astype(np.float16)
    x = xf.view(np.uint16)
    case = O.Case(R, bs, h, K, E, dtype=O.DT_FP16)
    expert_out, assist, counts = _dispatch_all(orc, case, x, ids, memory=False)
    # make the rows differ per route so the order of additions matters
    scale = (1 + 0.37 * np.arange(expert_out.shape[1]) % 5).astype(np.float16)
    eo = (expert_out.view(np.float16) * scale[None, :, None]).astype(np.float16)
    for rank in range(R):
        y = orc.mvp_combine(case, rank, eo.view(np.uint16), assist, counts)
        want = np.zeros((bs, h), np.float16)
        for er in range(R):                     # expert-rank major, then row order
            start = int(counts[er][:rank].sum())
            for row in range(start, start + int(counts[er][rank])):
                tok = assist[er, row, 1]
                want[tok] = (want[tok].astype(np.float32) + eo[er, row].astype(np.float32)).astype(np.float16)
        assert np.array_equal(y, want.view(np.uint16))
    # per-add rounding is observable: a single fp32 accumulation gives a different answer somewhere
    acc = np.zeros((bs, h), np.float32)
    for er in range(R):
        for row in range(int(counts[er][0])):
            acc[assist[er, row, 1]] += eo[er, row].astype(np.float32)
    y0 = orc.mvp_combine(case, 0, eo.view(np.uint16), assist, counts)
    assert not np.array_equal(y0, acc.astype(np.float16).view(np.uint16))


@pytest.mark.parametrize("dtype", [O.DT_BF16, O.DT_FP16])
def test_memory_combine_is_fp32_k_ordered(orc, dtype):
    rng = np.random.default_rng(29)
    R, bs, h, K, E = 2, 9, 64, 4, 8
    ids = rand_ids(rng, R, bs, K, E)
    f = (rng.standard_normal((R, bs, h)) * 3).astype(np.float32)
    if dtype == O.DT_BF16:
        x = torch.from_numpy(f).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    else:
        x = f.astype(np.float16).view(np.uint16)
    case = O.Case(R, bs, h, K, E, dtype=dtype)
    expert_out, assist, counts = _dispatch_all(orc, case, x, ids, memory=True)
    # perturb rows per route so each k contributes a different vector
    rows = expert_out.shape[1]
    for er in range(R):
        for row in range(rows):
            expert_out[er, row] = np.roll(expert_out[er, row], row % 7)
    w = (0.5 + rng.random((R, bs, K))).astype(np.float32)
    shared = rand_x(rng, R, bs, h) if dtype == O.DT_FP16 else None
    tmask = (rng.random((R, bs)) < 0.8).astype(np.uint8)

    def dec(u):
        if dtype == O.DT_BF16:
            return (u.astype(np.uint32) << 16).view(np.float32)
        return u.view(np.float16).astype(np.float32)

    for rank in range(R):
        sh = None if shared is None else (shared[rank] & 0x3fff)
        y = orc.mem_combine(case, rank, expert_out, assist, counts, expert_scales=w[rank], token_mask=tmask[rank],
                            shared_expert_x=sh)
        slot = -np.ones((bs, K, 2), np.int64)
        for er in range(R):
            for row in range(int(counts[er][-1])):
                s, t, k, _ = assist[er, row]
                if s == rank:
                    slot[t, k] = (er, row)
        want = np.zeros((bs, h), np.float32)
        for t in range(bs):
            if not tmask[rank, t]:
                continue
            acc = np.zeros(h, np.float32)
            for k in range(K):
                er, row = slot[t, k]
                if er < 0:
                    continue
                acc = (acc + (dec(expert_out[er, row]) * w[rank, t, k]).astype(np.float32)).astype(np.float32)
            if sh is not None:
                acc = (acc + dec(sh[t])).astype(np.float32)
            want[t] = acc
        if dtype == O.DT_BF16:
            wb = torch.from_numpy(want).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
        else:
            wb = np.clip(want, -65504, 65504).astype(np.float16).view(np.uint16)
        assert np.array_equal(y, wb)
        assert not y[tmask[rank] == 0].any()


def test_memory_combine_k_order_is_observable(orc):
    """Summing the same rows in reverse k order changes some bf16 results: the order is part of the contract."""
    rng = np.random.default_rng(31)
    bs, h, K, E = 64, 128, 8, 16
    ids = rand_ids(rng, 1, bs, K, E)
    f = (rng.standard_normal((1, bs, h)) * 100).astype(np.float32)
    x = torch.from_numpy(f).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    case = O.Case(1, bs, h, K, E)
    d = orc.mem_dispatch(case, 0, x, ids)
    eo = d["expand_x"].view(np.uint16)[None]
    for row in range(d["rows"]):
        eo[0, row] = np.roll(eo[0, row], row % 11)
    w = (rng.random((bs, K)) * 4).astype(np.float32)
    a = orc.mem_combine(case, 0, eo, d["assist"][None], d["send_counts"][None], expert_scales=w)
    rev_assist = d["assist"].copy()
    rev_assist[:, 2] = K - 1 - rev_assist[:, 2]
    b = orc.mem_combine(case, 0, eo, rev_assist[None], d["send_counts"][None], expert_scales=w[:, ::-1].copy())
    assert not np.array_equal(a, b)
    assert np.mean(a != b) < 0.2     # ...but only by final-rounding effects


def test_memory_combine_mxfp8_comm_quant(orc):
    """comm quant 3/4: each row goes through the MXFP8 round trip, then (fp8*2^(s-127))*w is accumulated
    (tilexr_ep_mxfp8_quant.h:286-352).  Checked against the quantiser + numpy."""
    rng = np.random.default_rng(37)
    bs, h, K, E = 5, 96, 2, 4
    ids = rand_ids(rng, 1, bs, K, E)
    f = (rng.standard_normal((1, bs, h)) * 4).astype(np.float16)
    x = f.view(np.uint16)
    w = (0.5 + rng.random((bs, K))).astype(np.float32)
    case = O.Case(1, bs, h, K, E, dtype=O.DT_FP16)
    d = orc.mem_dispatch(case, 0, x, ids)
    eo = d["expand_x"].view(np.uint16)[None]
    for mode, fp8 in ((3, O.DT_FP8E5M2), (4, O.DT_FP8E4M3)):
        y = orc.mem_combine(case, 0, eo, d["assist"][None], d["send_counts"][None], expert_scales=w, comm_quant=mode)
        want = np.zeros((bs, h), np.float32)
        inv = {(int(t), int(k)): r for r, (_, t, k, _) in enumerate(d["assist"][: d["rows"]])}
        for t in range(bs):
            acc = np.zeros(h, np.float32)
            for k in range(K):
                row = inv[(t, k)]
                q, s = orc.quant_row_mxfp8(eo[0, row], O.DT_FP16, fp8)
                dq = np.array([orc.fp8_decode(int(b), fp8) for b in q], np.float32) * \
                    np.exp2(s[np.arange(h) // 32].astype(np.float32) - 127).astype(np.float32)
                acc = (acc + (dq * w[t, k]).astype(np.float32)).astype(np.float32)
            want[t] = acc
        assert np.array_equal(y, np.clip(want, -65504, 65504).astype(np.float16).view(np.uint16))
        # and it stays within the demo's tolerance of the unquantised combine (tilexr_ep_dispatch_demo.cpp:1039-1040)
        exact = orc.mem_combine(case, 0, eo, d["assist"][None], d["send_counts"][None], expert_scales=w)
        ya, yb = y.view(np.float16).astype(np.float32), exact.view(np.float16).astype(np.float32)
        tol = np.maximum(1e-3, np.abs(yb) * (0.30 if mode == 3 else 0.15))
        assert np.all(np.abs(ya - yb) <= tol)


def test_memory_combine_quantised_input_equals_combine_of_dequantised_rows(orc):
    """ext: combine(q, scales) == combine(round_to_dtype(dequant(q, scales)))."""
    rng = np.random.default_rng(41)
    bs, h, K, E = 10, 256, 3, 8
    ids = rand_ids(rng, 1, bs, K, E)
    xf = torch.from_numpy((rng.standard_normal((1, bs, h)) * 2).astype(np.float32)).to(torch.bfloat16)
    x = xf.view(torch.int16).numpy().view(np.uint16)
    w = (rng.random((bs, K)) + 0.1).astype(np.float32)
    for mode in (O.Q_TOKEN_INT8, O.Q_FP8_BLOCK128):
        case = O.Case(1, bs, h, K, E, quant_mode=mode)
        d = orc.mem_dispatch(case, 0, x, ids)
        rows = d["rows"]
        if mode == O.Q_TOKEN_INT8:
            deq = d["expand_x"].view(np.int8).astype(np.float32) * d["dyn_scales"][:, :1]
        else:
            dec = np.array([orc.fp8_decode(c) for c in range(256)], np.float32)
            deq = dec[d["expand_x"]] * np.repeat(d["dyn_scales"], 128, axis=1)[:, :h]
        deq_bits = torch.from_numpy(np.ascontiguousarray(deq, np.float32)).to(torch.bfloat16).view(torch.int16) \
            .numpy().view(np.uint16)
        plain_case = O.Case(1, bs, h, K, E)
        want = orc.mem_combine(plain_case, 0, deq_bits[None], d["assist"][None], d["send_counts"][None],
                               expert_scales=w)
        got = orc.mem_combine(plain_case, 0, d["expand_x"][None], d["assist"][None], d["send_counts"][None],
                              expert_scales=w, in_quant=mode, in_scales=d["dyn_scales"])
        assert np.array_equal(got, want)
        assert rows > 0


# ---------------------------------------------------------------------------------------------
# committed checker fixtures (usable where the reference sources are absent)
# ---------------------------------------------------------------------------------------------
def test_oracle_matches_committed_checker_fixtures(orc):
    """tests/golden/checker_fixtures.npz holds the reference checker's ep_dispatch / ep_combine blobs
    (made by tests/golden/make_checker_fixtures.py); the oracle must reproduce them byte for byte."""
    import hashlib
    import os
    fx = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "checker_fixtures.npz"))
    assert int(fx["num_cases"][0]) >= 4
    for i in range(int(fx["num_cases"][0])):
        R, bs, h, K, E, dtype = (int(v) for v in fx[f"case{i}_shape"])
        ids = np.broadcast_to(fx[f"case{i}_ids"], (R, bs, K)).copy()
        tt, hh = np.meshgrid(np.arange(bs), np.arange(h), indexing="ij")
        x = np.stack([((0x1000 + r * 0x100 + tt * 0x10 + hh) & 0xffff).astype(np.uint16) for r in range(R)])
        case = O.Case(R, bs, h, K, E, dtype=dtype)
        for r in range(R):
            got = orc.mvp_dispatch(case, r, x, ids)
            n = got["rows"]
            assert n == bs * K
            blob = np.concatenate([got["expand_x"][:n].reshape(-1), np.zeros((R - 1) * n * h * 2, np.uint8),
                                   got["assist"][:n].reshape(-1).view(np.uint8), got["recv_counts"].view(np.uint8),
                                   got["expert_token_nums"].view(np.uint8)])
            if f"case{i}_dispatch_blobs" in fx:
                assert np.array_equal(blob, fx[f"case{i}_dispatch_blobs"][r])
                restored = fx[f"case{i}_combine_blobs"][r].view(np.uint16).reshape(bs, K, h)
                assert np.array_equal(restored, np.broadcast_to(x[r][:, None, :], (bs, K, h)))
            else:
                digest = np.frombuffer(hashlib.sha256(blob.tobytes()).digest(), np.uint8)
                assert np.array_equal(digest, fx[f"case{i}_dispatch_sha256"][r])
                want = np.broadcast_to(x[r][:, None, :], (bs, K, h))
                digest = np.frombuffer(hashlib.sha256(np.ascontiguousarray(want).tobytes()).digest(), np.uint8)
                assert np.array_equal(digest, fx[f"case{i}_combine_sha256"][r])
    assert int(fx["case3_dispatch_events"][0]) == 4148 and int(fx["case3_combine_events"][0]) == 6164


# ---------------------------------------------------------------------------------------------
# Shared experts: the reference demo's golden route model, restated as a brute-force walk
# (tests/ep/demo/tilexr_ep_dispatch_demo.cpp:622-792: LocalExpertNum, DstRankForExpert, LocalExpertForExpert,
# BuildExpectedRoutes, BuildExpectedMemoryRoutes, BuildExpectedRecvCounts)
# ---------------------------------------------------------------------------------------------
def demo_routes(case, dst, ids, token_live):
    """Source-major routes of destination rank `dst`: [(src, token, topKId, expertId)]."""
    R, S, SR, K = case.rank_size, case.shared_expert_num, case.shared_expert_rank_num, case.top_k
    le = case.moe_expert_num // (R - SR)
    per = SR // S if S else 1
    out = []
    for src in range(R):
        for t in range(case.bs):
            if not token_live[src][t]:
                continue
            for s in range(S):
                if src % per + s * per == dst:
                    out.append((src, t, K + s, s))
            for k in range(K):
                e = int(ids[src, t, k])
                if 0 <= e < case.moe_expert_num and SR + e // le == dst:
                    out.append((src, t, k, S + e))
    return out


def demo_local_expert(case, expert_id):
    le = case.moe_expert_num // (case.rank_size - case.shared_expert_rank_num)
    return 0 if expert_id < case.shared_expert_num else (expert_id - case.shared_expert_num) % le


SHARED_SHAPES = [  # R, bs, h, K, E, S, SR
    (4, 6, 8, 2, 6, 1, 1), (4, 9, 8, 3, 8, 2, 2), (8, 5, 8, 2, 12, 2, 4), (3, 7, 8, 2, 4, 1, 1), (6, 4, 8, 4, 16, 1, 2)]


@pytest.mark.parametrize("shape", SHARED_SHAPES)
@pytest.mark.parametrize("masked", [False, True, "expert"])
def test_shared_experts_memory_route_matches_demo_golden(orc, shape, masked):
    R, bs, h, K, E, S, SR = shape
    rng = np.random.default_rng(sum(shape) + bool(masked) + 2 * (masked == "expert"))
    mask_type = {False: O.MASK_NONE, True: O.MASK_TOKEN, "expert": O.MASK_EXPERT}[masked]
    case = O.Case(R, bs, h, K, E, dtype=O.DT_BF16, shared_expert_num=S, shared_expert_rank_num=SR,
                  mask_type=mask_type, token_nums_type=1)
    ids = rand_ids(rng, R, bs, K, E, invalid_frac=0.1)
    x = rand_x(rng, R, bs, h)
    mask = None
    if masked == "expert":
        # demo :599-620: a route is live when its mask byte is set, a token when one of its routes is
        mask = (rng.random((R, bs, K)) < 0.5).astype(np.uint8)
        live = [[bool(mask[s, t].any()) for t in range(bs)] for s in range(R)]
        ids = np.where(mask != 0, ids, -1).astype(np.int32)          # what the golden walk sees of a masked route
    elif masked:
        mask = (rng.random((R, bs)) < 0.7).astype(np.uint8)
        # the memory route dispatches the first sum(mask) tokens of a source rank (prefix rule)
        live = [[t < int(mask[s].sum()) for t in range(bs)] for s in range(R)]
    else:
        live = [[True] * bs] * R
    total = 0
    for dst in range(R):
        got = orc.mem_dispatch(case, dst, x, ids, mask)
        source_major = demo_routes(case, dst, ids, live)
        out_local = 1 if dst < SR else case.local_experts
        want = [r for loc in range(out_local) for src in range(R) for r in source_major
                if r[0] == src and demo_local_expert(case, r[3]) == loc]
        assert got["rows"] == len(want)
        assert got["assist"][:len(want)].tolist() == [list(r) for r in want]
        running, counts = 0, []
        for loc in range(out_local):
            for src in range(R):
                running += sum(1 for r in source_major if r[0] == src and demo_local_expert(case, r[3]) == loc)
                counts.append(running)
        assert got["send_counts"].tolist() == counts
        per_expert = [sum(1 for r in want if demo_local_expert(case, r[3]) == loc) for loc in range(out_local)]
        assert got["expert_token_nums"].tolist() == per_expert
        for row, (src, t, _, _) in enumerate(want):
            assert np.array_equal(got["expand_x"][row].view(np.uint16), x[src, t])
        total += len(want)
    # closed form: every live token reaches each shared expert once, every valid routed id once
    live_tokens = sum(sum(l) for l in live)
    valid = sum(1 for s in range(R) for t in range(bs) for k in range(K) if live[s][t] and 0 <= ids[s, t, k] < E)
    assert total == live_tokens * S + valid


@pytest.mark.parametrize("shape", [s for s in SHARED_SHAPES if s[5] == s[6]])     # the MVP route needs S == SR
@pytest.mark.parametrize("masked", [False, True])
def test_shared_experts_mvp_route_matches_demo_golden(orc, shape, masked):
    R, bs, h, K, E, S, SR = shape
    rng = np.random.default_rng(sum(shape) * 3 + masked)
    case = O.Case(R, bs, h, K, E, dtype=O.DT_FP16, shared_expert_num=S, shared_expert_rank_num=SR, token_nums_type=1)
    ids = rand_ids(rng, R, bs, K, E, invalid_frac=0.1)
    x = rand_x(rng, R, bs, h)
    mask = (rng.random((R, bs)) < 0.7).astype(np.uint8) if masked else None
    live = [[bool(mask[s][t]) for t in range(bs)] for s in range(R)] if masked else [[True] * bs] * R
    le = case.local_experts
    for dst in range(R):
        got = orc.mvp_dispatch(case, dst, x, ids, mask)
        want = demo_routes(case, dst, ids, live)
        assert got["rows"] == len(want)
        assert got["assist"][:len(want)].tolist() == [list(r) for r in want]
        assert got["recv_counts"].tolist() == [sum(1 for r in want if r[0] == src) for src in range(R)]
        # per-expert counts follow the kernel, which files a shared row under its expert id
        # (src/ep/kernels/tilexr_ep_dispatch_helpers.h:99-101, tilexr_ep_combine_helpers.h:124-128), not the demo's
        # "local expert 0"; the two agree for shared expert 0
        counts = [0] * le
        for r in want:
            loc = r[3] if r[3] < S else (r[3] - S) % le
            if loc < le:
                counts[loc] += 1
        assert got["expert_token_nums"].tolist() == counts
        if dst == 0 and S >= 1:
            assert counts[0] >= sum(1 for r in want if r[3] == 0)


def test_shared_slots_enter_the_memory_combine_after_the_routed_ones(orc):
    R, bs, h, K, E, S, SR = 4, 5, 16, 2, 6, 2, 2
    rng = np.random.default_rng(77)
    case = O.Case(R, bs, h, K, E, dtype=O.DT_BF16, shared_expert_num=S, shared_expert_rank_num=SR, token_nums_type=1)
    ids = rand_ids(rng, R, bs, K, E)
    x = torch.from_numpy(rng.standard_normal((R, bs, h)).astype(np.float32)).to(torch.bfloat16)
    xb = x.view(torch.int16).numpy().view(np.uint16)
    w = rng.random((R, bs, K)).astype(np.float32)
    outs = [orc.mem_dispatch(case, d, xb, ids) for d in range(R)]
    mr = case.max_rows
    eo = np.zeros((R, mr, h), np.uint16)
    asst = np.zeros((R, mr, 4), np.int32)
    sc = np.zeros((R, case.local_experts * R), np.int32)
    for d, o in enumerate(outs):
        eo[d], asst[d] = o["expand_x"].view(np.uint16), o["assist"]
        sc[d, :o["send_counts"].size] = o["send_counts"]
    for r in range(R):
        y = orc.mem_combine(case, r, eo, asst, sc, expert_scales=w[r])
        xf = x[r].to(torch.float32).numpy()
        for t in range(bs):
            acc = np.zeros(h, np.float32)
            for k in range(K):
                acc = acc + xf[t] * np.float32(w[r, t, k])        # identity experts: every slot returns x[t]
            for _ in range(S):
                acc = acc + xf[t]
            want = torch.from_numpy(acc).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
            assert np.array_equal(y[t], want)


# ---------------------------------------------------------------------------------------------
# Tensor-parallel groups on the MVP route: the demo's BuildExpectedRoutes / BuildExpectedTpRoutes restated
# (tests/ep/demo/tilexr_ep_dispatch_demo.cpp:687-743), counts per the kernel
# (src/ep/kernels/tilexr_ep_dispatch_kernel.cpp:809-827, tilexr_ep_combine_helpers.h:92-95)
# ---------------------------------------------------------------------------------------------
def demo_tp_own_routes(case, rank, ids, token_live):
    R, S, SR, K, tp = case.rank_size, case.shared_expert_num, case.shared_expert_rank_num, case.top_k, case.tp_world_size
    er_size = R // tp
    le = case.moe_expert_num // (er_size - SR)
    per = SR // S if S else 1
    out = []
    for src in range(R):
        if src % tp != rank % tp:
            continue
        for t in range(case.bs):
            if not token_live[src][t]:
                continue
            for s in range(S):
                if (src // tp) % per + s * per == rank // tp:
                    out.append((src, t, K + s, s))
            for k in range(K):
                e = int(ids[src, t, k])
                if 0 <= e < case.moe_expert_num and SR + e // le == rank // tp:
                    out.append((src, t, k, S + e))
    return out


TP_SHAPES = [  # R, bs, h, K, E, S, SR, tp
    (4, 6, 8, 2, 4, 0, 0, 2), (8, 9, 8, 3, 8, 0, 0, 2), (8, 5, 8, 2, 6, 1, 1, 2), (8, 7, 8, 2, 8, 0, 0, 4),
    (6, 4, 8, 2, 6, 0, 0, 3)]


@pytest.mark.parametrize("shape", TP_SHAPES)
@pytest.mark.parametrize("masked", [False, True])
def test_tensor_parallel_groups_match_demo_golden(orc, shape, masked):
    R, bs, h, K, E, S, SR, tp = shape
    rng = np.random.default_rng(sum(shape) * 5 + masked)
    case = O.Case(R, bs, h, K, E, dtype=O.DT_FP16, shared_expert_num=S, shared_expert_rank_num=SR, tp_world_size=tp,
                  token_nums_type=1)
    ids = rand_ids(rng, R, bs, K, E, invalid_frac=0.1)
    x = rand_x(rng, R, bs, h)
    mask = (rng.random((R, bs)) < 0.7).astype(np.uint8) if masked else None
    live = [[bool(mask[s][t]) for t in range(bs)] for s in range(R)] if masked else [[True] * bs] * R
    le = case.local_experts
    for rank in range(R):
        got = orc.mvp_dispatch(case, rank, x, ids, mask, count_fill=-1)
        own = demo_tp_own_routes(case, rank, ids, live)
        group = (rank // tp) * tp
        want = list(own)
        for lane in range(tp):
            if group + lane != rank:
                want += demo_tp_own_routes(case, group + lane, ids, live)
        assert got["rows"] == len(want)
        assert got["assist"][:len(want)].tolist() == [list(r) for r in want]
        for row, (src, t, _, _) in enumerate(want):
            assert np.array_equal(got["expand_x"][row].view(np.uint16), x[src, t])
        # recvCounts: own-lane sources only, the rest is left alone
        recv = [-1] * R
        for src in range(rank % tp, R, tp):
            recv[src] = sum(1 for r in own if r[0] == src)
        assert got["recv_counts"].tolist() == recv
        # tpRecvCounts: the same per-source entries, then rows per lane in the first tp entries
        tp_recv = list(recv)
        for lane in range(tp):
            tp_recv[lane] = len(own) if group + lane == rank else len(demo_tp_own_routes(case, group + lane, ids, live))
        assert got["tp_recv_counts"].tolist() == tp_recv
        counts = [0] * le
        for r in want:
            loc = r[3] if r[3] < S else (r[3] - S) % le
            if loc < le:
                counts[loc] += 1
        assert got["expert_token_nums"].tolist() == counts
    # every rank of a group ends up with the same multiset of rows
    for g in range(0, R, tp):
        sets = []
        for lane in range(tp):
            o = orc.mvp_dispatch(case, g + lane, x, ids, mask)
            sets.append(sorted(map(tuple, o["assist"][:o["rows"]].tolist())))
        assert all(s == sets[0] for s in sets)


# ---------------------------------------------------------------------------------------------------------------
# corrupted assist tuples and counts: skipped, never followed
# (src/ep/kernels/tilexr_ep_combine_memory_kernel.h:256-266, 340-342; tilexr_ep_combine_kernel.cpp:28-52, 94-97)
# ---------------------------------------------------------------------------------------------------------------
def corrupt_tuples(rng, assist, rows, bs, K, rank_size, how_many):
    """Plants the mistakes the kernels must survive into `how_many` random rows of each rank's table; returns the
    rows that were touched.  A later test with the same seed reproduces the same table."""
    bad = {}
    for er in range(assist.shape[0]):
        picks = rng.choice(rows[er], size=min(how_many, rows[er]), replace=False)
        for j, row in enumerate(picks):
            kind = j % 6
            if kind == 0:
                assist[er, row, 1] = -1
            elif kind == 1:
                assist[er, row, 1] = bs
            elif kind == 2:
                assist[er, row, 2] = K
            elif kind == 3:
                assist[er, row, 2] = -3
            elif kind == 4:
                assist[er, row, 0] = rank_size + 5            # a rank that does not exist
            else:
                assist[er, row, 1] = 0x7fffffff
        bad[er] = set(int(r) for r in picks)
    return bad


def np_bf16(f):
    return torch.from_numpy(np.ascontiguousarray(f, np.float32)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


def np_memory_combine_walk(rank, bs, h, K, expert_out, assist, send_counts, w):
    """Plain walk over the rows, written without reference to the oracle's code: rows [0, min(count, buffer)) of every
    expert rank; a row whose tuple names this rank, a token in [0, bs) and a slot in [0, K) fills that slot (a later
    row replaces an earlier one); y[t] = bf16(sum over k in order of fp32(w * row))."""
    R, max_rows = assist.shape[0], assist.shape[1]
    slot = {}
    for er in range(R):
        rows = min(max(int(send_counts[er][-1]), 0), max_rows)
        for row in range(rows):
            s, t, k, _ = (int(v) for v in assist[er, row])
            if s != rank or not 0 <= t < bs or not 0 <= k < K:
                continue
            slot[(t, k)] = (er, row)
    y = np.zeros((bs, h), np.float32)
    for t in range(bs):
        acc = np.zeros(h, np.float32)
        for k in range(K):
            if (t, k) in slot:
                er, row = slot[(t, k)]
                r = (expert_out[er, row].astype(np.uint32) << 16).view(np.float32)
                acc = (acc + (r * np.float32(w[t, k])).astype(np.float32)).astype(np.float32)
        y[t] = acc
    return np_bf16(y)


def test_memory_combine_skips_corrupted_tuples_like_a_plain_walk(orc):
    rng = np.random.default_rng(71)
    R, bs, h, K, E = 2, 24, 32, 4, 8
    ids = rand_ids(rng, R, bs, K, E, 0.05)
    x = np_bf16(rng.standard_normal((R, bs, h)) * 3)
    case = O.Case(R, bs, h, K, E, dtype=O.DT_BF16)
    expert_out, assist, counts = _dispatch_all(orc, case, x, ids, memory=True)
    rows = [int(counts[er][-1]) for er in range(R)]
    w = (0.5 + rng.random((R, bs, K))).astype(np.float32)
    clean = [orc.mem_combine(case, r, expert_out, assist, counts, expert_scales=w[r]) for r in range(R)]
    bad = corrupt_tuples(rng, assist, rows, bs, K, R, 12)
    # one duplicate as well: a second row that claims the slot of an intact one (the later row wins)
    er, victim = 0, next(r for r in range(rows[0]) if r not in bad[0])
    thief = next(r for r in range(victim + 1, rows[0]) if r not in bad[0])
    assist[er, thief, :3] = assist[er, victim, :3]
    # and a count that runs past the buffer: the walk stops at the buffer's end
    counts = counts.copy()
    counts[1][-1] = assist.shape[1] + 1000
    for rank in range(R):
        y = orc.mem_combine(case, rank, expert_out, assist, counts, expert_scales=w[rank])
        assert np.array_equal(y, np_memory_combine_walk(rank, bs, h, K, expert_out, assist, counts, w[rank]))
        assert not np.array_equal(y, clean[rank])        # the planted rows really mattered


def test_mvp_combine_skips_corrupted_tuples_like_a_plain_walk(orc):
    rng = np.random.default_rng(73)
    R, bs, h, K, E = 2, 16, 16, 3, 6
    ids = rand_ids(rng, R, bs, K, E)
    xf = (rng.standard_normal((R, bs, h)) * 5).astype(np.float16)
    case = O.Case(R, bs, h, K, E, dtype=O.DT_FP16)
    expert_out, assist, counts = _dispatch_all(orc, case, xf.view(np.uint16), ids, memory=False)
    rows = [int(counts[er].sum()) for er in range(R)]
    corrupt_tuples(rng, assist, rows, bs, K, R, 9)
    counts = counts.copy()
    counts[1][0] = -4                      # a count outside [0, bs * K] reads as 0: rank 0 gets nothing from rank 1,
    for rank in range(R):                  # and rank 1's own rows start at row 0 of that table
        y = orc.mvp_combine(case, rank, expert_out, assist, counts)
        want = np.zeros((bs, h), np.float16)
        for er in range(R):
            c = [int(v) if 0 <= int(v) <= bs * K else 0 for v in counts[er]]
            start = sum(c[:rank])
            for row in range(start, start + c[rank]):
                _, t, k, _ = (int(v) for v in assist[er, row])
                if not 0 <= t < bs or not 0 <= k < K:
                    continue               # the rank field is overwritten on the way (combine_kernel.cpp:28-52)
                want[t] = (want[t].astype(np.float32) + expert_out[er, row].view(np.float16).astype(np.float32)).astype(np.float16)
        assert np.array_equal(y, want.view(np.uint16))
