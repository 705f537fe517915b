"""Drives libtilexr-ep through its C ABI with torch tensors as device memory, and fetches results as numpy arrays
shaped like the oracle's outputs (tests/ and the smoke check use it).

Stream discipline of the tests: inside a Session torch's own work (fills, host copies, comparisons) runs on the
session's stream, the one the library calls use.  Multi-rank worlds and side streams use torch's default stream for
that work and wait for it (`torch.cuda.synchronize()`) before a library call is issued on another stream.  Library
results are read after the stream of the call has been synchronised."""
import os

import numpy as np
import torch

from tilexr_amd import ep

DEV = "cuda:0"


_KEEP = []      # device copies made by to_dev(): kernels on side streams may still read them after the call returns


def to_dev(a):
    if a is None:
        return None
    t = torch.from_numpy(np.ascontiguousarray(a)).to(DEV)
    _KEEP.append(t)
    return t


def release_device_copies():
    torch.cuda.synchronize()
    _KEEP.clear()


def bits16(t):
    """bf16/fp16 torch tensor -> uint16 numpy."""
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


class Session:
    """One communicator (single rank) + a non-default stream."""

    def __init__(self, rank_size=1, rank=0, legacy_routing=None):
        """legacy_routing: True = the communicator's dispatches route with the count + place launches everywhere,
        False = with the one-launch routing wherever it can take the call, None = the library picks by the size of the
        call (it reads TILEXR_EP_ROUTING when a communicator is created)."""
        torch.cuda.set_device(0)
        previous = os.environ.get("TILEXR_EP_ROUTING")
        if legacy_routing is None:
            os.environ.pop("TILEXR_EP_ROUTING", None)
        else:
            os.environ["TILEXR_EP_ROUTING"] = "legacy" if legacy_routing else "one-launch"
        try:
            self.comm = ep.Comm(rank_size, rank)
        finally:
            if previous is None:
                os.environ.pop("TILEXR_EP_ROUTING", None)
            else:
                os.environ["TILEXR_EP_ROUTING"] = previous
        self.stream = torch.cuda.Stream()
        # torch's own work (fills, host copies, comparisons) goes on the same stream as the library calls, as a
        # caller that keeps a whole layer on one stream would have it
        self._previous = torch.cuda.current_stream()
        torch.cuda.synchronize()
        torch.cuda.set_stream(self.stream)

    def close(self):
        torch.cuda.synchronize()
        torch.cuda.set_stream(self._previous)
        release_device_copies()
        self.comm.destroy()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def sync(self):
        self.stream.synchronize()


def alloc_dispatch_outputs(bs, h, top_k, experts, ranks=1, quant=ep.Q_NONE, fill=0x5a):
    rows = ranks * bs * top_k
    row_bytes = h * 2 if quant == ep.Q_NONE else h
    out = dict(
        expand_x=torch.full((rows, row_bytes), fill, dtype=torch.uint8, device=DEV),
        assist=torch.full((rows, 4), -77, dtype=torch.int32, device=DEV),
        token_nums=torch.full((experts // ranks,), -5, dtype=torch.int64, device=DEV),
        row_map=torch.full((bs, top_k), -9, dtype=torch.int32, device=DEV),
    )
    if quant == ep.Q_MXFP8:
        out["scales"] = torch.full((rows, ((h + 31) // 32 + 1) // 2 * 2), 0xee, dtype=torch.uint8, device=DEV)
    elif quant == ep.Q_FP8_BLOCK128:
        out["scales"] = torch.full((rows, (h + 127) // 128), -3.0, dtype=torch.float32, device=DEV)
    elif quant in (ep.Q_TOKEN_INT8,):
        out["scales"] = torch.full((rows, 1), -3.0, dtype=torch.float32, device=DEV)
    else:
        out["scales"] = None
    # the fills run on torch's default stream, the library on the caller's own (non-blocking) stream
    torch.cuda.synchronize()
    return out


def fetch(out, counts_name, counts):
    res = {k: (None if v is None else v.cpu().numpy()) for k, v in out.items()}
    res[counts_name] = counts.cpu().numpy()
    return res
