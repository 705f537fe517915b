"""A torch-facing convenience layer over the C ABI for one rank per device: allocate the outputs, call dispatch,
hand the expert-contiguous rows to the caller's expert stage, call combine.

It adds nothing to the data path: every call below is one call of `TileXRMoeEpDispatchMemoryEx` /
`TileXRMoeEpCombineMemoryEx` (include/tilexr_ep.h).  torch only provides the tensors and the stream.  The library's
calls run on a stream owned by the layer (the C ABI, like the reference, rejects the null stream) that is ordered
after torch's current stream on entry and before it on return, so callers can treat the methods like ordinary
torch ops.
"""
from dataclasses import dataclass
from typing import Optional

import torch

from . import ep

_TORCH_DTYPE = {torch.bfloat16: ep.DT_BF16, torch.float16: ep.DT_FP16}
_QUANT = {None: ep.Q_NONE, "none": ep.Q_NONE, "int8": ep.Q_TOKEN_INT8, "mxfp8": ep.Q_MXFP8,
          "fp8_block128": ep.Q_FP8_BLOCK128}


@dataclass
class Dispatched:
    """What dispatch produced.  Rows [0, rows) of `expand_x` are valid, grouped by expert in expert order;
    `send_counts` is the inclusive prefix sum of rows per expert (device tensor), `token_nums` rows per expert."""
    expand_x: torch.Tensor            # [bs * top_k, h] in the input type, or uint8 payload rows when quantised
    scales: Optional[torch.Tensor]    # per-row / per-block scales of a quantised payload
    assist: torch.Tensor              # [bs * top_k, 4] int32 {srcRank, token, k, expert}
    send_counts: torch.Tensor         # [experts] int32
    token_nums: torch.Tensor          # [experts] int64
    row_map: torch.Tensor             # [bs, top_k] int32, row of every route, -1 = dropped / invalid
    quant: int
    bs: int

    def rows(self) -> int:
        """Number of valid rows (synchronises with the device)."""
        return int(self.send_counts[-1].item())


class MoeEpLayer:
    def __init__(self, experts: int, top_k: int, hidden: int, device="cuda:0"):
        self.experts, self.top_k, self.hidden = experts, top_k, hidden
        self.device = torch.device(device)
        torch.cuda.set_device(self.device)
        self.comm = ep.Comm(1, 0)
        self.stream = torch.cuda.Stream(device=self.device)

    def close(self):
        if self.comm is not None:
            torch.cuda.synchronize(self.device)
            self.comm.destroy()
            self.comm = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    # ---- stream hand-over -------------------------------------------------------------------------------
    def _enter(self):
        self.stream.wait_stream(torch.cuda.current_stream(self.device))

    def _leave(self, *tensors):
        cur = torch.cuda.current_stream(self.device)
        cur.wait_stream(self.stream)
        for t in tensors:
            if t is not None:
                t.record_stream(self.stream)

    # ---- dispatch ---------------------------------------------------------------------------------------
    def dispatch(self, x: torch.Tensor, expert_ids: torch.Tensor, quant: Optional[str] = None, capacity: int = 0,
                 prefix_token_nums: bool = False) -> Dispatched:
        """x [bs, hidden] bf16/fp16, expert_ids [bs, top_k] int32 (ids outside [0, experts) are skipped)."""
        bs, h = x.shape
        if h != self.hidden or tuple(expert_ids.shape) != (bs, self.top_k):
            raise ValueError("shape mismatch")
        if x.dtype not in _TORCH_DTYPE or expert_ids.dtype != torch.int32:
            raise TypeError("x must be bfloat16 / float16 and expert_ids int32")
        x, expert_ids = x.contiguous(), expert_ids.contiguous()
        q = _QUANT[quant]
        n = bs * self.top_k
        dev = self.device
        if q == ep.Q_NONE:
            expand_x, scales = torch.empty((n, h), dtype=x.dtype, device=dev), None
        else:
            expand_x = torch.empty((n, h), dtype=torch.uint8, device=dev)
            if q == ep.Q_TOKEN_INT8:
                scales = torch.empty((n, 1), dtype=torch.float32, device=dev)
            elif q == ep.Q_MXFP8:
                scales = torch.empty((n, ((h + 31) // 32 + 1) // 2 * 2), dtype=torch.uint8, device=dev)
            else:
                scales = torch.empty((n, (h + 127) // 128), dtype=torch.float32, device=dev)
        assist = torch.empty((n, 4), dtype=torch.int32, device=dev)
        send_counts = torch.empty((self.experts,), dtype=torch.int32, device=dev)
        token_nums = torch.empty((self.experts,), dtype=torch.int64, device=dev)
        row_map = torch.empty((bs, self.top_k), dtype=torch.int32, device=dev)
        self._enter()
        st, _ = ep.dispatch_memory_ex(x, expert_ids, self.comm, bs, h, self.top_k, self.experts, expand_x, assist,
                                      token_nums, send_counts, _TORCH_DTYPE[x.dtype], self.stream, quant_mode=q,
                                      expert_capacity=capacity, token_nums_type=0 if prefix_token_nums else 1,
                                      dynamic_scales=scales, row_index_map=row_map)
        ep.check(st, "TileXRMoeEpDispatchMemoryEx")
        self._leave(x, expert_ids, expand_x, scales, assist, send_counts, token_nums, row_map)
        return Dispatched(expand_x, scales, assist, send_counts, token_nums, row_map, q, bs)

    # ---- combine ----------------------------------------------------------------------------------------
    def combine(self, expert_out: torch.Tensor, d: Dispatched, weights: Optional[torch.Tensor] = None,
                dtype: torch.dtype = torch.bfloat16, expert_out_scales: Optional[torch.Tensor] = None,
                expert_out_quant: Optional[str] = None, shared_expert_x: Optional[torch.Tensor] = None,
                token_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
        """y[t] = sum_k weights[t, k] * expert_out[row of route (t, k)] (+ shared_expert_x[t]), fp32 accumulation in k
        order, one rounding to `dtype`.  expert_out has the row layout of `d.expand_x`."""
        q = _QUANT[expert_out_quant]
        bs, h = d.bs, self.hidden
        expert_out = expert_out.contiguous()
        if weights is not None:
            weights = weights.to(torch.float32).contiguous()
        y = torch.empty((bs, h), dtype=dtype, device=self.device)
        mask = None if token_mask is None else token_mask.to(torch.uint8).contiguous()
        self._enter()
        st = ep.combine_memory_ex(expert_out, d.assist, d.send_counts, self.comm, bs, h, self.top_k, self.experts, y,
                                  _TORCH_DTYPE[dtype], self.stream, expert_out_quant_mode=q,
                                  expert_out_scales=expert_out_scales, expert_scales=weights,
                                  active_mask=mask, active_mask_type=ep.MASK_TOKEN if mask is not None else ep.MASK_NONE,
                                  shared_expert_x=shared_expert_x, row_index_map=d.row_map)
        ep.check(st, "TileXRMoeEpCombineMemoryEx")
        self._leave(expert_out, weights, y, mask, shared_expert_x, expert_out_scales)
        return y
