"""The entry point that allocates nothing (TileXRMoeEpDispatchMemoryNoAlloc): its kernels' scratch is one static device
array per GPU instead of a buffer from hipMalloc.  Called through the C ABI and compared, bit for bit, with
TileXRMoeEpDispatchMemory on the same inputs, on two calls in a row of which the second is smaller (the array keeps
the first call's contents), then once more with the first size.  Sizes beyond the array are rejected before anything
is enqueued."""
import numpy as np
import pytest
import torch

from gpu_harness import DEV, Session
from tilexr_amd import ep

pytestmark = pytest.mark.gpu


def _outputs(bs, h, K, E, fill):
    n = bs * K
    return dict(expand_x=torch.full((n, h), fill, dtype=torch.bfloat16, device=DEV),
                assist=torch.full((n, 4), -77, dtype=torch.int32, device=DEV),
                token_nums=torch.full((E,), -5, dtype=torch.int64, device=DEV),
                counts=torch.full((E,), -6, dtype=torch.int32, device=DEV))


def _call(fn, s, x, ids, bs, h, K, E, out):
    return fn(x, ids, s.comm, bs, h, K, E, out["expand_x"], out["token_nums"], out["counts"], out["assist"],
              ep.DT_BF16, s.stream)


@pytest.mark.parametrize("legacy_routing", [False, True])
def test_no_alloc_dispatch_matches_the_allocating_entry_point(legacy_routing):
    # every shape has more than 2048 routes: routing launch(es) + scatter, the path that needs scratch (the row of every
    # route and the kept-row count with the one-launch routing; ranks, histograms, offsets and the ticket word, which the
    # call has to clear, with the count + place routing)
    shapes = [(4096, 1024, 8, 256), (700, 512, 6, 48), (4096, 1024, 8, 256), (1031, 264, 4, 7)]
    rng = np.random.default_rng(20)
    with Session(legacy_routing=legacy_routing) as s:
        free_before = None
        for call, (bs, h, K, E) in enumerate(shapes):
            ids = np.stack([rng.permutation(E)[:K] for _ in range(bs)]).astype(np.int32)
            ids[rng.random((bs, K)) < 0.03] = -1                       # a few routes without an expert
            x = torch.from_numpy(rng.standard_normal((bs, h)).astype(np.float32)).to(torch.bfloat16).to(DEV)
            d_ids = torch.from_numpy(ids).to(DEV)
            want, got = _outputs(bs, h, K, E, 3.0), _outputs(bs, h, K, E, 3.0)
            torch.cuda.synchronize()
            print(f"no-alloc dispatch: call {call} shape {(bs, h, K, E)}", flush=True)
            assert _call(ep.dispatch_memory, s, x, d_ids, bs, h, K, E, want) == 0
            s.sync()
            if call == 1:
                free_before = torch.cuda.mem_get_info()[0]
            assert _call(ep.dispatch_memory_no_alloc, s, x, d_ids, bs, h, K, E, got) == 0
            s.sync()
            if call >= 1:
                # the device's free memory did not shrink across the call (the first call may still load code)
                assert torch.cuda.mem_get_info()[0] >= free_before
            for name in want:
                assert torch.equal(want[name].view(torch.int16) if name == "expand_x" else want[name],
                                   got[name].view(torch.int16) if name == "expand_x" else got[name]), (call, name)
            rows = int(want["counts"][-1].item())
            assert 0 < rows <= bs * K


def test_no_alloc_dispatch_at_the_largest_size_it_documents():
    """131 072 routes over 2048 experts: the count scratch of the largest call the header promises fits the array."""
    bs, h, K, E = 16384, 8, 8, 2048
    rng = np.random.default_rng(21)
    ids = rng.integers(0, E, (bs, K)).astype(np.int32)
    x = torch.from_numpy(rng.standard_normal((bs, h)).astype(np.float32)).to(torch.bfloat16).to(DEV)
    d_ids = torch.from_numpy(ids).to(DEV)
    with Session() as s:
        want, got = _outputs(bs, h, K, E, 3.0), _outputs(bs, h, K, E, 3.0)
        torch.cuda.synchronize()
        assert _call(ep.dispatch_memory, s, x, d_ids, bs, h, K, E, want) == 0
        assert _call(ep.dispatch_memory_no_alloc, s, x, d_ids, bs, h, K, E, got) == 0
        s.sync()
        assert ep.last_kernel_name(s.comm, ep.K_COUNT) == "ep_route_count_kernel"
        for name in want:
            assert torch.equal(want[name].view(torch.int16) if name == "expand_x" else want[name],
                               got[name].view(torch.int16) if name == "expand_x" else got[name]), name
        assert int(got["counts"][-1].item()) == bs * K


def test_no_alloc_dispatch_rejects_what_does_not_fit():
    with Session() as s:
        fake = torch.zeros((16,), dtype=torch.int32, device=DEV)
        magic = s.comm.next_magic()
        # 262 144 routes need more count scratch than the 2 MiB array holds: rejected on the host, nothing is launched
        args = (fake, fake, s.comm, 32768, 64, 8, 256, fake, fake, fake, fake, ep.DT_BF16, s.stream)
        assert ep.dispatch_memory_no_alloc(*args) == ep.ERR_NOT_SUPPORT
        assert ep.dispatch_memory_no_alloc(None, *args[1:]) == ep.ERR_PARA_CHECK_FAIL
        assert s.comm.next_magic() == magic + 1                       # rejected calls drew no magic
    # worlds of several logical ranks stage rows in allocated buffers
    a, b = ep.Comm(2, 0), ep.Comm(2, 1)
    stream = torch.cuda.Stream()
    assert ep.dispatch_memory_no_alloc(fake, fake, a, 64, 64, 2, 8, fake, fake, fake, fake, ep.DT_BF16,
                                       stream) == ep.ERR_NOT_SUPPORT
    a.destroy()
    b.destroy()
