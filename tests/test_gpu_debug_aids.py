"""Debug aids of the dispatch / combine calls: the phase-stamp ring and the poison fill.

The stamps are breadcrumbs (which kernel of which call was reached, on the device's own clock); the poison fill makes a
row that was counted but never written stand out.  Neither may change what the calls compute: every run here is also
compared with the CPU oracle.
"""
import numpy as np
import pytest
import torch

from gpu_harness import DEV, Session, bits16
from oracle import ep as O
from tilexr_amd import ep

pytestmark = pytest.mark.gpu

POISON = 0x7f7f7f7f


def make_case(bs, h, K, E, seed):
    rng = np.random.default_rng(seed)
    ids = np.stack([rng.permutation(E)[:K] for _ in range(bs)]).astype(np.int32)
    x = torch.from_numpy(rng.standard_normal((bs, h)).astype(np.float32)).to(torch.bfloat16)
    w = torch.from_numpy(rng.random((bs, K)).astype(np.float32))
    return x, ids, w


def oracle(bs, h, K, E, x, ids, w, quant=O.Q_NONE, capacity=0):
    case = O.Case(1, bs, h, K, E, dtype=O.DT_BF16, quant_mode=quant, capacity=capacity, token_nums_type=1)
    want = O.mem_dispatch(case, 0, bits16(x)[None], ids[None])
    eo = want["expand_x"][None] if quant else want["expand_x"].view(np.uint16)[None]
    want["y"] = O.mem_combine(O.Case(1, bs, h, K, E, dtype=O.DT_BF16), 0, eo, want["assist"][None],
                              want["send_counts"][None], expert_scales=w.numpy(), in_quant=quant,
                              in_scales=want["dyn_scales"] if quant else None)
    return want


def records(ring, count):
    r = ring.cpu().numpy().astype(np.uint64)
    return [tuple(int(v) for v in r[i % len(r)]) for i in range(count)]


@pytest.mark.parametrize("bs,h,K,E,kernels_d,kernels_c", [
    # two launches per dispatch (count + scatter), invert + reduce without a row map
    (1024, 1024, 4, 32, [ep.K_COUNT, ep.K_SCATTER], [ep.K_INVERT, ep.K_REDUCE]),
])
def test_phase_stamps_follow_the_kernels_of_each_call(bs, h, K, E, kernels_d, kernels_c):
    x, ids, w = make_case(bs, h, K, E, 1)
    want = oracle(bs, h, K, E, x, ids, w)
    n = bs * K
    with Session() as s:
        ring = torch.zeros((64, 4), dtype=torch.int64, device=DEV)
        assert ep.set_debug_options(s.comm, phase_stamps=ring) == 0
        expand_x = torch.zeros((n, h * 2), dtype=torch.uint8, device=DEV)
        assist = torch.zeros((n, 4), dtype=torch.int32, device=DEV)
        token_nums = torch.zeros((E,), dtype=torch.int64, device=DEV)
        counts = torch.zeros((E,), dtype=torch.int32, device=DEV)
        y = torch.zeros((bs, h), dtype=torch.bfloat16, device=DEV)
        d_x, d_ids, d_w = x.to(DEV), torch.from_numpy(ids).to(DEV), w.to(DEV)
        magics = []
        for _ in range(2):
            st, magic = ep.dispatch_memory_ex(d_x, d_ids, s.comm, bs, h, K, E, expand_x, assist, token_nums, counts,
                                              ep.DT_BF16, s.stream)
            assert st == 0
            magics.append(magic)
            assert ep.combine_memory_ex(expand_x, assist, counts, s.comm, bs, h, K, E, y, ep.DT_BF16, s.stream,
                                        expert_scales=d_w) == 0
        s.sync()
        assert np.array_equal(bits16(y), want["y"])
        per_layer = 2 * (len(kernels_d) + len(kernels_c))
        got = records(ring, 2 * per_layer)
        # kernel ids and edges in launch order, before / after pairs
        expect = [(k, e) for k in kernels_d + kernels_c for e in (0, 1)] * 2
        assert [(r[1], r[2]) for r in got] == expect
        # the dispatch's records carry its magic; the combine's carry the combine's own, which is later
        d_records = len(kernels_d) * 2
        for layer in range(2):
            base = layer * per_layer
            assert all(r[0] == magics[layer] for r in got[base:base + d_records])
            assert all(r[0] > magics[layer] for r in got[base + d_records:base + per_layer])
        # one device clock, read in stream order
        clocks = [r[3] for r in got]
        assert clocks == sorted(clocks) and clocks[0] > 0
        # untouched records stay zero
        assert not ring.cpu().numpy()[2 * per_layer:].any()

        # the ring wraps: a capacity of 3 keeps the last three records
        small = torch.zeros((3, 4), dtype=torch.int64, device=DEV)
        assert ep.set_debug_options(s.comm, phase_stamps=small) == 0
        st, magic = ep.dispatch_memory_ex(d_x, d_ids, s.comm, bs, h, K, E, expand_x, assist, token_nums, counts,
                                          ep.DT_BF16, s.stream)
        assert st == 0
        s.sync()
        r = small.cpu().numpy()
        # four records went in at 0, 1, 2, 0
        assert [(int(v[1]), int(v[2])) for v in r] == [(kernels_d[1], 1), (kernels_d[0], 1), (kernels_d[1], 0)]
        assert all(int(v[0]) == magic for v in r)

        # switched off: nothing more is written
        assert ep.set_debug_options(s.comm) == 0
        before = small.clone()
        st, _ = ep.dispatch_memory_ex(d_x, d_ids, s.comm, bs, h, K, E, expand_x, assist, token_nums, counts,
                                      ep.DT_BF16, s.stream)
        assert st == 0
        s.sync()
        assert torch.equal(before, small)


def test_phase_stamps_name_the_single_launch_of_a_decode_sized_call():
    bs, h, K, E = 16, 1024, 4, 32
    x, ids, w = make_case(bs, h, K, E, 2)
    n = bs * K
    with Session() as s:
        ring = torch.zeros((8, 4), dtype=torch.int64, device=DEV)
        assert ep.set_debug_options(s.comm, phase_stamps=ring) == 0
        expand_x = torch.zeros((n, h * 2), dtype=torch.uint8, device=DEV)
        assist = torch.zeros((n, 4), dtype=torch.int32, device=DEV)
        token_nums = torch.zeros((E,), dtype=torch.int64, device=DEV)
        counts = torch.zeros((E,), dtype=torch.int32, device=DEV)
        st, magic = ep.dispatch_memory_ex(x.to(DEV), torch.from_numpy(ids).to(DEV), s.comm, bs, h, K, E, expand_x,
                                          assist, token_nums, counts, ep.DT_BF16, s.stream)
        assert st == 0
        s.sync()
        got = records(ring, 8)
        used = [r for r in got if r[0] != 0]
        assert len(used) % 2 == 0 and len(used) >= 2
        assert all(r[0] == magic for r in used)
        assert [r[2] for r in used] == [0, 1] * (len(used) // 2)


def test_debug_options_argument_rules():
    with Session() as s:
        ring = torch.zeros((4, 4), dtype=torch.int64, device=DEV)
        fn = ep.lib().TileXREpSetDebugOptions
        import ctypes as C
        fn.argtypes = [C.c_void_p, C.POINTER(ep.DebugOptions)]
        bad = [ep.DebugOptions(ring.data_ptr(), 0, 0), ep.DebugOptions(None, 4, 0), ep.DebugOptions(ring.data_ptr(), -1, 0),
               ep.DebugOptions(ring.data_ptr(), (1 << 24) + 1, 0)]
        for opt in bad:
            assert fn(s.comm.handle, C.byref(opt)) == -3
        assert fn(None, None) != 0
        assert fn(s.comm.handle, None) == 0


@pytest.mark.parametrize("quant,oquant", [(ep.Q_NONE, O.Q_NONE), (ep.Q_TOKEN_INT8, O.Q_TOKEN_INT8),
                                          (ep.Q_FP8_BLOCK128, O.Q_FP8_BLOCK128)], ids=["bf16", "int8", "fp8_block128"])
def test_poison_marks_rows_the_dispatch_did_not_write(quant, oquant):
    """With a capacity limit the dispatch keeps fewer rows than experts * capacity: the kept rows hold data, the rest
    of what the call may write holds the poison pattern, memory behind that is not touched, and combine is unaffected."""
    bs, h, K, E, capacity = 256, 512, 4, 16, 40
    rng = np.random.default_rng(7)
    # skewed routing: some experts overflow the capacity, others stay under it
    p = np.arange(1, E + 1, dtype=np.float64) ** -1.3
    p /= p.sum()
    ids = np.stack([rng.choice(E, size=K, replace=False, p=p) for _ in range(bs)]).astype(np.int32)
    x = torch.from_numpy(rng.standard_normal((bs, h)).astype(np.float32)).to(torch.bfloat16)
    w = torch.from_numpy(rng.random((bs, K)).astype(np.float32))
    want = oracle(bs, h, K, E, x, ids, w, quant=oquant, capacity=capacity)
    rows = want["rows"]
    n = bs * K
    may_write = min(n, E * capacity)
    assert 0 < rows < may_write < n
    row_bytes = h * 2 if quant == ep.Q_NONE else h
    with Session() as s:
        assert ep.set_debug_options(s.comm, poison=True) == 0
        expand_x = torch.full((n, row_bytes), 0x5a, dtype=torch.uint8, device=DEV)
        assist = torch.full((n, 4), -77, dtype=torch.int32, device=DEV)
        token_nums = torch.zeros((E,), dtype=torch.int64, device=DEV)
        counts = torch.zeros((E,), dtype=torch.int32, device=DEV)
        y = torch.zeros((bs, h), dtype=torch.bfloat16, device=DEV)
        scales = None
        if quant == ep.Q_TOKEN_INT8:
            scales = torch.full((n, 1), -3.0, dtype=torch.float32, device=DEV)
        elif quant == ep.Q_FP8_BLOCK128:
            scales = torch.full((n, (h + 127) // 128), -3.0, dtype=torch.float32, device=DEV)
        d_w = w.to(DEV)
        for _ in range(2):
            st, _ = ep.dispatch_memory_ex(x.to(DEV), torch.from_numpy(ids).to(DEV), s.comm, bs, h, K, E, expand_x, assist,
                                          token_nums, counts, ep.DT_BF16, s.stream, quant_mode=quant,
                                          expert_capacity=capacity, dynamic_scales=scales)
            assert st == 0
            assert ep.combine_memory_ex(expand_x, assist, counts, s.comm, bs, h, K, E, y, ep.DT_BF16, s.stream,
                                        expert_out_quant_mode=quant, expert_out_scales=scales, expert_scales=d_w) == 0
            s.sync()
            ex = expand_x.cpu().numpy()
            assert np.array_equal(ex[:rows], want["expand_x"].view(np.uint8).reshape(-1, row_bytes)[:rows])
            assert (ex[rows:may_write] == 0x7f).all()
            assert (ex[may_write:] == 0x5a).all()
            a = assist.cpu().numpy()
            assert np.array_equal(a[:rows], want["assist"][:rows])
            assert (a[rows:may_write] == POISON).all() and (a[may_write:] == -77).all()
            if scales is not None:
                sc = scales.cpu().numpy()
                assert np.array_equal(sc[:rows].reshape(rows, -1), want["dyn_scales"][:rows].reshape(rows, -1))
                assert (sc[rows:may_write].view(np.uint32) == POISON).all()
                assert (sc[may_write:] == -3.0).all()
            assert np.array_equal(counts.cpu().numpy(), want["send_counts"])
            assert np.array_equal(bits16(y), want["y"])
