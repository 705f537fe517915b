"""The torch-facing layer (tilexr_amd/layer.py) against a plain PyTorch fp32 reference of the same two ops, on torch's
default stream like ordinary torch code.

Reference dispatch: stable sort of the valid routes by expert; reference combine: fp32 sum over k of w * row.
Layout, indices and counts must be identical; the combined rows are bit-identical to the k-ordered fp32 loop and
within 1e-2 relative of torch's own reduction order (the tolerance the workload definition states for the combine).
"""
import numpy as np
import pytest
import torch

from tilexr_amd import layer, workloads

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def torch_dispatch(x, ids, experts):
    bs, K = ids.shape
    flat = torch.arange(bs * K, device=x.device)
    e = ids.reshape(-1).long()
    valid = (e >= 0) & (e < experts)
    key = torch.where(valid, e * (bs * K) + flat, torch.full_like(flat, experts * bs * K))
    order = torch.argsort(key, stable=True)[: int(valid.sum().item())]
    rows = x[order // K]
    assist = torch.stack([torch.zeros_like(order), order // K, order % K, e[order]], 1).int()
    counts = torch.bincount(e[valid], minlength=experts)
    row_map = torch.full((bs * K,), -1, dtype=torch.int32, device=x.device)
    row_map[order] = torch.arange(order.numel(), device=x.device, dtype=torch.int32)
    return rows, assist, counts, row_map.view(bs, K)


def torch_combine_k_ordered(expert_out, row_map, weights):
    bs, K = row_map.shape
    acc = torch.zeros((bs, expert_out.shape[1]), dtype=torch.float32, device=expert_out.device)
    for k in range(K):
        r = row_map[:, k].long()
        row = expert_out[r.clamp(min=0)].float() * weights[:, k:k + 1]
        acc = acc + torch.where((r >= 0)[:, None], row, torch.zeros_like(row))
    return acc


@pytest.mark.parametrize("name,bs", [("C2", 128), ("C3", 1536), ("C3", 4096)])
def test_layer_matches_torch_reference(name, bs):
    w = workloads.scaled(workloads.CONFIGS[name], bs)
    x = workloads.make_x(w).to(DEV)
    ids, weights = workloads.make_routing(w)
    ids[::7, 0] = -1                                      # some invalid routes
    ids, weights = ids.to(DEV), weights.to(DEV)
    with layer.MoeEpLayer(w.experts, w.top_k, w.h) as moe:
        d = moe.dispatch(x, ids)
        want_rows, want_assist, want_counts, want_map = torch_dispatch(x, ids, w.experts)
        n = d.rows()
        assert n == want_rows.shape[0]
        assert torch.equal(d.expand_x[:n].view(torch.int16), want_rows.view(torch.int16))
        assert torch.equal(d.assist[:n], want_assist)
        assert torch.equal(d.token_nums, want_counts)
        assert torch.equal(d.send_counts.long(), torch.cumsum(want_counts, 0))
        assert torch.equal(d.row_map, want_map)
        # an "expert stage" written in torch on the current stream, then combine
        expert_out = (d.expand_x.float() * 0.5 + 1.0).to(torch.bfloat16)
        y = moe.combine(expert_out, d, weights)
        ref = torch_combine_k_ordered(expert_out, d.row_map, weights)
        assert torch.equal(y.view(torch.int16), ref.to(torch.bfloat16).view(torch.int16))
        # torch's own reduction order: within 1e-2 relative
        gathered = expert_out[d.row_map.long().clamp(min=0)].float() * (d.row_map >= 0)[..., None]
        other = (gathered * weights[..., None]).sum(1)
        err = (y.float() - other).abs()
        assert torch.all(err <= 1e-2 * other.abs() + 1e-2 * other.abs().mean())


@pytest.mark.parametrize("quant", ["int8", "fp8_block128"])
def test_layer_quantised_round_trip(quant):
    w = workloads.scaled(workloads.CONFIGS["C4" if quant == "int8" else "C5"], 512)
    x = workloads.make_x(w).to(DEV)
    ids, weights = workloads.make_routing(w)
    ids, weights = ids.to(DEV), weights.to(DEV)
    with layer.MoeEpLayer(w.experts, w.top_k, w.h) as moe:
        d = moe.dispatch(x, ids, quant=quant, capacity=w.capacity)
        n = d.rows()
        if quant == "int8":
            deq = d.expand_x[:n].view(torch.int8).float() * d.scales[:n]
        else:
            deq = (d.expand_x[:n].view(torch.float8_e4m3fn).float().view(n, w.h // 128, 128) *
                   d.scales[:n, :, None]).view(n, w.h)
        src = x.float()[d.assist[:n, 1].long()]
        bound = d.scales[:n] * 0.5001 if quant == "int8" else torch.maximum(
            src.abs() * 2.0 ** -4, d.scales[:n].repeat_interleave(128, dim=1) * 2.0 ** -10) * 1.0001
        assert torch.all((deq - src).abs() <= bound)
        # identity expert on the quantised payload: combine dequantises, rounds to bf16 and reduces
        y = moe.combine(d.expand_x, d, weights, expert_out_scales=d.scales, expert_out_quant=quant)
        padded = torch.zeros((w.bs * w.top_k, w.h), dtype=torch.bfloat16, device=DEV)
        padded[:n] = deq.to(torch.bfloat16)
        ref = torch_combine_k_ordered(padded, d.row_map, weights)
        assert torch.equal(y.view(torch.int16), ref.to(torch.bfloat16).view(torch.int16))


def test_plan_driven_layer_round_trip():
    """The torch-facing wrapper of the plan-driven stages on a one-rank world: dispatch builds the duplicate plan on the
    first call and follows it on the second; with an identity expert combine returns bf16(K * x); weights come back."""
    from tilexr_amd.layer import PlanDrivenLayer
    s, k, h = 300, 4, 1024
    g = torch.Generator().manual_seed(11)
    x = torch.randn(s, h, generator=g).to(torch.bfloat16).to(DEV)
    w = torch.rand(s, k, generator=g).to(DEV)
    nvs = s * k + 17
    rows_of = torch.randperm(nvs, generator=g)[:s * k].to(torch.int32)
    dst = rows_of.clone().reshape(s, k)
    dst[:, 1:] = -dst[:, 1:] - 1                       # one rank: every route after a token's first is a duplicate
    dst = dst.reshape(-1).to(DEV)
    with PlanDrivenLayer(s, k, h, nvs=nvs) as layer:
        layer.set_plan(dst)
        for call in range(2):
            rows, rw = layer.dispatch(x, w)
            torch.cuda.synchronize()
            assert int(layer.status[0].item()) == 2000
            raw = rows_of.to(torch.int64).to(DEV)
            assert torch.equal(rows[raw].view(torch.int16), x.repeat_interleave(k, dim=0).view(torch.int16)), f"call {call}"
            assert torch.equal(rw[raw], w.reshape(-1))
            unused = torch.ones(nvs, dtype=torch.bool, device=DEV)
            unused[raw] = False
            assert not rows[unused].view(torch.int16).any() and not rw[unused].any()
        y, wy = layer.combine(rows, rw)
        torch.cuda.synchronize()
        assert int(layer.status[0].item()) == 0
        assert torch.equal(y.view(torch.int16), (x.float() * k).to(torch.bfloat16).view(torch.int16))
        assert torch.equal(wy, w)


@pytest.mark.gpu
def test_memory_probe_patterns_move_what_they_say():
    """The yardstick kernels of the benchmark: every pattern writes exactly the bytes it is specified to write."""
    import torch
    from tilexr_amd import ep

    dev = "cuda:0"
    n = 1 << 20
    stream = torch.cuda.Stream()
    src = torch.arange(n, dtype=torch.int32, device=dev)
    dst = torch.full((n + 64,), -1, dtype=torch.int32, device=dev)
    torch.cuda.synchronize()
    nbytes = n * 4
    assert ep.memory_probe(ep.PROBE_COPY, src, dst, nbytes, stream) == 0
    stream.synchronize()
    assert torch.equal(dst[:n], src) and bool((dst[n:] == -1).all())
    dst.fill_(-1)
    torch.cuda.synchronize()
    assert ep.memory_probe(ep.PROBE_FAN_OUT, src, dst, nbytes, stream) == 0
    stream.synchronize()
    assert torch.equal(dst[:n].view(8, n // 8), src[:n // 8].expand(8, n // 8)) and bool((dst[n:] == -1).all())
    dst.fill_(-1)
    torch.cuda.synchronize()
    assert ep.memory_probe(ep.PROBE_FAN_IN, src, dst, nbytes, stream) == 0
    stream.synchronize()
    want = src.view(8, n // 8)[0].clone()
    for k in range(1, 8):
        want ^= src.view(8, n // 8)[k]
    assert torch.equal(dst[:n // 8], want) and bool((dst[n // 8:] == -1).all())
    dst.fill_(-1)
    torch.cuda.synchronize()
    assert ep.memory_probe(ep.PROBE_WRITE, None, dst, nbytes, stream) == 0
    assert ep.memory_probe(ep.PROBE_READ, src, dst[n:], nbytes, stream) == 0
    stream.synchronize()
    assert torch.equal(dst[:n].view(-1, 4), torch.tensor([1, 2, 3, 4], dtype=torch.int32, device=dev).expand(n // 4, 4))
    assert bool((dst[n:] == -1).all())
    # argument rules
    assert ep.memory_probe(8, src, dst, nbytes, stream) == -3
    assert ep.memory_probe(-1, src, dst, nbytes, stream) == -3
    assert ep.memory_probe(ep.PROBE_COPY, src, dst, nbytes + 4, stream) == -3
    assert ep.memory_probe(ep.PROBE_COPY, None, dst, nbytes, stream) == -3


@pytest.mark.gpu
def test_memory_probe_row_gather_reads_rows_whole():
    """The row-gather yardstick: every output row is the xor of eight source rows, taken whole."""
    import torch
    from tilexr_amd import ep

    dev = "cuda:0"
    rows, row_ints = 64, 14336 // 4
    stream = torch.cuda.Stream()
    g = torch.Generator().manual_seed(5)
    src = torch.randint(-2**31, 2**31 - 1, (rows, row_ints), generator=g, dtype=torch.int64).to(torch.int32).to(dev)
    dst = torch.full((rows // 8 + 1, row_ints), -1, dtype=torch.int32, device=dev)
    torch.cuda.synchronize()
    assert ep.memory_probe(ep.PROBE_GATHER_ROWS, src, dst, rows * 14336, stream) == 0
    stream.synchronize()
    strides = [1, 7919, 10007, 12289, 15013, 17389, 20011, 22291]
    for t in range(rows // 8):
        want = torch.zeros(row_ints, dtype=torch.int32, device=dev)
        for k in range(8):
            want ^= src[(t * strides[k] + k * 977) % rows]
        assert torch.equal(dst[t], want), f"row {t}"
    assert bool((dst[rows // 8] == -1).all())
    assert ep.memory_probe(ep.PROBE_GATHER_ROWS, src, dst, rows * 14336 + 128, stream) == -3


@pytest.mark.gpu
@pytest.mark.parametrize("pattern,row_bytes,k", [("PROBE_GATHER_ROWS_2K_X8", 2048, 8), ("PROBE_GATHER_ROWS_4K_X6", 4096, 6)])
def test_memory_probe_narrow_row_gathers(pattern, row_bytes, k):
    """The yardsticks of the quantised reduce: every output row, twice as wide as a source row, interleaves 16-byte
    pieces of the xor of k source rows with pieces of the same xor without its last row."""
    import torch
    from tilexr_amd import ep

    dev = "cuda:0"
    groups = 11
    rows, row_ints = groups * k, row_bytes // 4
    stream = torch.cuda.Stream()
    g = torch.Generator().manual_seed(6)
    src = torch.randint(-2**31, 2**31 - 1, (rows, row_ints), generator=g, dtype=torch.int64).to(torch.int32).to(dev)
    dst = torch.full((groups + 1, 2 * row_ints), -1, dtype=torch.int32, device=dev)
    torch.cuda.synchronize()
    assert ep.memory_probe(getattr(ep, pattern), src, dst, rows * row_bytes, stream) == 0
    stream.synchronize()
    strides = [1, 7919, 10007, 12289, 15013, 17389, 20011, 22291]
    for t in range(groups):
        picked = [src[(t * strides[j] + j * 977) % rows] for j in range(k)]
        all_k = picked[0].clone()
        for r in picked[1:]:
            all_k ^= r
        want = torch.stack([all_k.view(-1, 4), (all_k ^ picked[-1]).view(-1, 4)], dim=1).reshape(-1)
        assert torch.equal(dst[t], want), f"row {t}"
    assert bool((dst[groups] == -1).all())
    assert ep.memory_probe(getattr(ep, pattern), src, dst, rows * row_bytes + row_bytes, stream) == -3
