"""The measured configurations at their full sizes: bit-exact against the CPU oracle (it finishes each of them in
well under a minute) plus size-independent properties computed on the device: counts are the clipped histogram,
rows are a stable sort of the kept routes by expert, every kept route has exactly one row, payload rows are their
source rows (or within the quantiser's error bound of them), and combine is the gate-weighted sum of the kept rows
within 1e-2 relative.
"""
import numpy as np
import pytest
import torch

from gpu_harness import DEV, Session, bits16
from oracle import ep as O
from tilexr_amd import ep, workloads

pytestmark = pytest.mark.gpu

QUANT = {"none": ep.Q_NONE, "int8": ep.Q_TOKEN_INT8, "fp8_block128": ep.Q_FP8_BLOCK128}


def run_layer(s, w, x, ids, weights):
    bs, h, K, E = w.bs, w.h, w.top_k, w.experts
    quant = QUANT[w.quant]
    n = bs * K
    row_bytes = h * 2 if quant == ep.Q_NONE else h
    t = dict(
        x=x.to(DEV), ids=ids.to(DEV), w=weights.to(DEV),
        expand_x=torch.full((n, row_bytes), 0x5a, dtype=torch.uint8, device=DEV),
        assist=torch.full((n, 4), -77, dtype=torch.int32, device=DEV),
        token_nums=torch.zeros((E,), dtype=torch.int64, device=DEV),
        send_counts=torch.zeros((E,), dtype=torch.int32, device=DEV),
        row_map=torch.full((bs, K), -9, dtype=torch.int32, device=DEV),
        y=torch.full((bs, h), 5.0, dtype=torch.bfloat16, device=DEV), scales=None)
    if quant == ep.Q_TOKEN_INT8:
        t["scales"] = torch.full((n, 1), -3.0, dtype=torch.float32, device=DEV)
    elif quant == ep.Q_FP8_BLOCK128:
        t["scales"] = torch.full((n, (h + 127) // 128), -3.0, dtype=torch.float32, device=DEV)
    # the fills above run on torch's default stream, the library on the session's own (non-blocking) stream: without
    # this wait a 4.7 GB fill can still be writing when the first rows land
    torch.cuda.synchronize()
    st, _ = ep.dispatch_memory_ex(t["x"], t["ids"], s.comm, bs, h, K, E, t["expand_x"], t["assist"], t["token_nums"],
                                  t["send_counts"], ep.DT_BF16, s.stream, quant_mode=quant,
                                  expert_capacity=w.capacity, dynamic_scales=t["scales"], row_index_map=t["row_map"])
    assert st == 0
    st = ep.combine_memory_ex(t["expand_x"], t["assist"], t["send_counts"], s.comm, bs, h, K, E, t["y"], ep.DT_BF16,
                              s.stream, expert_out_quant_mode=quant, expert_out_scales=t["scales"],
                              expert_scales=t["w"], row_index_map=t["row_map"])
    assert st == 0
    s.sync()
    return t


def dequantised_rows(w, t, rows):
    """fp32 [rows, h] of what the payload rows stand for."""
    h = w.h
    if w.quant == "none":
        return t["expand_x"][:rows].view(torch.bfloat16).float()
    if w.quant == "int8":
        return t["expand_x"][:rows].view(torch.int8).float() * t["scales"][:rows]
    q = t["expand_x"][:rows].view(torch.float8_e4m3fn).float().view(rows, h // 128, 128)
    return (q * t["scales"][:rows, :, None]).view(rows, h)


@pytest.mark.parametrize("name", ["C2", "C3", "C4", "C5"])
def test_full_size_layer(name):
    w = workloads.CONFIGS[name]
    bs, h, K, E = w.bs, w.h, w.top_k, w.experts
    x = workloads.make_x(w)
    ids, weights = workloads.make_routing(w)
    with Session() as s:
        t = run_layer(s, w, x, ids, weights)

        # ---- properties on the device ----
        flat_ids = t["ids"].view(-1).long()
        hist = torch.bincount(flat_ids, minlength=E)
        kept = hist.clamp(max=w.capacity) if w.capacity else hist
        assert torch.equal(t["send_counts"].long(), torch.cumsum(kept, 0))
        assert torch.equal(t["token_nums"], kept)
        rows = int(kept.sum().item())
        if name == "C5":
            assert rows < bs * K                      # the Zipf(1.2) head overflows the capacity
        a = t["assist"][:rows].long()
        assert torch.all(t["assist"][rows:] == -77)
        assert torch.all(a[:, 0] == 0)
        expert, flat = a[:, 3], a[:, 1] * K + a[:, 2]
        assert torch.equal(flat_ids[flat], expert)                        # the tuple names a real route
        order_key = expert * (bs * K) + flat
        assert torch.all(order_key[1:] > order_key[:-1])                  # expert-major, stable, no duplicates
        rm = t["row_map"].view(-1).long()
        assert int((rm >= 0).sum().item()) == rows
        assert torch.equal(rm[flat], torch.arange(rows, device=DEV))      # row map is the inverse of the tuples
        if w.capacity:
            # within an expert the kept routes are the lowest flat indices: every dropped route of an expert lies
            # after the last kept one
            last_kept = torch.full((E,), -1, dtype=torch.long, device=DEV).scatter_reduce(0, expert, flat, "amax")
            dropped = rm < 0
            assert torch.all(torch.arange(bs * K, device=DEV)[dropped] > last_kept[flat_ids[dropped]])
        src = t["x"].float()[a[:, 1]]
        deq = dequantised_rows(w, t, rows)
        if w.quant == "none":
            assert torch.equal(t["expand_x"][:rows].view(torch.int16), t["x"].view(torch.int16)[a[:, 1]])
        elif w.quant == "int8":
            assert torch.all((deq - src).abs() <= t["scales"][:rows] * 0.5001)
        else:
            # e4m3 keeps 3 mantissa bits: the error is at most 2^-4 of the value or half the smallest subnormal step
            bound = torch.maximum(src.abs() * 2.0 ** -4, t["scales"][:rows].repeat_interleave(128, dim=1) * 2.0 ** -10)
            assert torch.all((deq - src).abs() <= bound * 1.0001)
        # combine = weighted sum over kept routes of the (dequantised, rounded to bf16) rows
        rows_bf16 = deq.to(torch.bfloat16).float()
        contrib = torch.zeros((bs * K, h), dtype=torch.float32, device=DEV)
        contrib[flat] = rows_bf16 * t["w"].view(-1)[flat][:, None]
        want_y = contrib.view(bs, K, h).sum(1)
        got_y = t["y"].float()
        err = (got_y - want_y).abs()
        assert torch.all(err <= 1e-2 * want_y.abs() + 1e-2 * want_y.abs().mean())   # 1e-2 relative
        del contrib, want_y, got_y, err, deq, src, rows_bf16

        # ---- bit-exact against the oracle at full size ----
        xb = bits16(x)
        quant = {"none": O.Q_NONE, "int8": O.Q_TOKEN_INT8, "fp8_block128": O.Q_FP8_BLOCK128}[w.quant]
        case = O.Case(1, bs, h, K, E, dtype=O.DT_BF16, quant_mode=quant, capacity=w.capacity, token_nums_type=1)
        want = O.mem_dispatch(case, 0, xb[None], ids.numpy()[None])
        assert want["rows"] == rows
        assert np.array_equal(t["assist"].cpu().numpy()[:rows], want["assist"][:rows])
        assert np.array_equal(t["expand_x"].cpu().numpy()[:rows], want["expand_x"][:rows])
        assert np.array_equal(t["send_counts"].cpu().numpy(), want["send_counts"])
        if quant:
            got_s = t["scales"].cpu().numpy()[:rows]
            assert np.array_equal(got_s.reshape(rows, -1), want["dyn_scales"][:rows].reshape(rows, -1))
        eo = want["expand_x"][None] if quant else want["expand_x"].view(np.uint16)[None]
        wy = O.mem_combine(O.Case(1, bs, h, K, E, dtype=O.DT_BF16), 0, eo, want["assist"][None],
                           want["send_counts"][None], expert_scales=weights.numpy(), in_quant=quant,
                           in_scales=want["dyn_scales"] if quant else None)
        assert np.array_equal(bits16(t["y"]), wy)


def test_c1_checker_configuration_round_trip():
    """C1: 4 logical ranks x 128 tokens x 1024 bf16, 16 experts, top-2, MVP route, softmax gate weights are applied by
    the caller in that route, so the round trip with an identity expert returns K * x per token."""
    w = workloads.CONFIGS["C1"]
    R, bs, h, K, E = w.ranks, w.bs, w.h, w.top_k, w.experts
    from test_gpu_multi_rank import World, run_dispatch
    xs = [workloads.make_x(w, r) for r in range(R)]
    ids = np.stack([workloads.make_routing(w, r)[0].numpy() for r in range(R)])
    xt = torch.stack(xs).to(DEV)
    xb = np.stack([bits16(x) for x in xs])
    with World(R) as world:
        outs = run_dispatch(world, False, xt, ids, bs, h, K, E, ep.DT_BF16)
        case = O.Case(R, bs, h, K, E, dtype=O.DT_BF16)
        ys = [torch.zeros((bs, h), dtype=torch.bfloat16, device=DEV) for _ in range(R)]
        for r in range(R):
            want = O.mvp_dispatch(case, r, xb, ids)
            n = want["rows"]
            assert np.array_equal(outs[r]["expand_x"].cpu().numpy()[:n], want["expand_x"][:n])
            assert np.array_equal(outs[r]["assist"].cpu().numpy()[:n], want["assist"][:n])
            assert np.array_equal(outs[r]["counts"].cpu().numpy(), want["recv_counts"])
        for r in range(R):
            assert ep.combine(outs[r]["expand_x"], outs[r]["assist"], outs[r]["counts"], world.comms[r], bs, h, K, E,
                              ys[r], ep.DT_BF16, world.streams[r]) == 0
        world.sync()
        for r in range(R):
            # two bf16 additions of the same value: 0 + x = x, x + x = 2x, both exact
            assert torch.equal(ys[r].float(), xt[r].float() * K)


def test_rows_beyond_four_gib_keep_their_addresses():
    """40960 tokens x 7168 x top-8: 327 680 rows of 14 336 bytes = 4.7 GB, so row offsets do not fit 32 bits.
    Checked through properties on the device (the oracle would take minutes here): the payload rows are their source
    rows, and combine with all weights 1/8 returns every token unchanged up to one rounding."""
    w = workloads.Workload("wide", 1, 40960, 7168, 8, 256, routing="zipf", zipf_s=1.0, seed=77)
    bs, h, K, E = w.bs, w.h, w.top_k, w.experts
    x = workloads.make_x(w)
    ids, _ = workloads.make_routing(w)
    weights = torch.full((bs, K), 0.125, dtype=torch.float32)
    with Session() as s:
        t = run_layer(s, w, x, ids, weights)
        rows = bs * K
        assert int(t["send_counts"][-1].item()) == rows
        a = t["assist"].long()
        flat = a[:, 1] * K + a[:, 2]
        assert torch.equal(t["ids"].view(-1).long()[flat], a[:, 3])
        assert torch.equal(t["row_map"].view(-1).long()[flat], torch.arange(rows, device=DEV))
        got = t["expand_x"].view(torch.int16).view(rows, h)
        src = t["x"].view(torch.int16)
        for begin in range(0, rows, 65536):                                  # in pieces: the gather is 4.7 GB
            end = min(begin + 65536, rows)
            assert torch.equal(got[begin:end], src[a[begin:end, 1]]), f"rows {begin}..{end}"
        # 8 x (x / 8) summed in fp32 is x exactly (power-of-two weights), so y == x bit for bit
        assert torch.equal(t["y"].view(torch.int16), src)
