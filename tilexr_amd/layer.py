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
        # the library reads raw bytes: a tensor of another element type would be reinterpreted, not converted
        want = {ep.Q_NONE: (dtype,), ep.Q_TOKEN_INT8: (torch.int8, torch.uint8),
                ep.Q_FP8_BLOCK128: (torch.float8_e4m3fn, torch.uint8)}[q]
        if expert_out.dtype not in want:
            raise ValueError(f"expert_out is {expert_out.dtype}, expected one of {want} for this payload")
        if expert_out.shape[-1] != h:
            raise ValueError(f"expert_out rows have {expert_out.shape[-1]} columns, expected {h}")
        expert_out = expert_out.contiguous()
        if q != ep.Q_NONE:
            if expert_out_scales is None or expert_out_scales.dtype != torch.float32:
                raise ValueError("a quantised expert_out needs float32 expert_out_scales")
            expert_out_scales = expert_out_scales.contiguous()
        if shared_expert_x is not None:
            if shared_expert_x.dtype != dtype or tuple(shared_expert_x.shape) != (bs, h):
                raise ValueError("shared_expert_x must be [bs, hidden] of the output type")
            shared_expert_x = shared_expert_x.contiguous()
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


class PlanDrivenLayer:
    """The plan-driven Dispatch / Combine stages (include/tilexr_moonep.h) for a world of one rank, as torch-style
    methods: every route of the plan stays on this device.

    A plan is the int32 tensor `dst [S * K]` of signed route words (row of the receive tensor, negated as `-row - 1` for
    a duplicate: a later route of a token that already has one).  `dispatch` builds the duplicate plan on the first call
    for a plan and follows the saved one afterwards; `combine` is its inverse with an fp32 sum per token."""

    def __init__(self, tokens: int, top_k: int, hidden: int, nvs: int = 0, device="cuda:0"):
        from . import moonep as mp
        self._mp = mp
        self.s, self.k, self.h = tokens, top_k, hidden
        self.nvs = nvs if nvs > 0 else tokens * top_k
        self.device = torch.device(device)
        torch.cuda.set_device(self.device)
        self.comm = ep.Comm(1, 0)
        self.stream = torch.cuda.Stream(device=self.device)
        dev = self.device
        self._groups = torch.zeros((self.nvs, 3), dtype=torch.int32, device=dev)
        self._loffs = torch.zeros((self.nvs,), dtype=torch.int32, device=dev)
        self._counts = torch.zeros((2,), dtype=torch.int32, device=dev)
        self.status = torch.zeros((4,), dtype=torch.int32, device=dev)
        self._dst = None
        self._dst_local = None
        self._plan = None
        self._built = False

    def close(self):
        if self.comm is not None:
            torch.cuda.synchronize(self.device)
            self.comm.destroy()
            self.comm = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def set_plan(self, dst: torch.Tensor):
        """dst int32 [S * K] on the device; rows must lie in [0, nvs)."""
        if dst.dtype != torch.int32 or dst.numel() != self.s * self.k:
            raise ValueError("dst must be int32 with S * K entries")
        mp = self._mp
        self._dst = dst.contiguous()
        raw = torch.where(self._dst >= 0, self._dst, -self._dst - 1).to(torch.int64)
        # reverse routes: receive row -> rank * nvs + route (rank 0 here), -1 where no route lands.  A row outside
        # [0, nvs) is left out here (an index past the end would abort the device context); the library reports it
        # through the plan's status word when the plan is used
        ok = raw < self.nvs
        self._dst_local = torch.full((self.nvs,), -1, dtype=torch.int32, device=self.device)
        self._dst_local[raw[ok]] = torch.arange(self.s * self.k, dtype=torch.int32, device=self.device)[ok]
        self._plan = mp.plan(self.s * self.k, 1, self.k, 1, self.nvs, self.k, self._dst, self._groups, self._loffs,
                             self._counts, self.status)
        self._built = False

    def _enter(self):
        self.stream.wait_stream(torch.cuda.current_stream(self.device))

    def _leave(self, *tensors):
        torch.cuda.current_stream(self.device).wait_stream(self.stream)
        for t in tensors:
            if t is not None:
                t.record_stream(self.stream)

    def dispatch(self, x: torch.Tensor, weights: Optional[torch.Tensor] = None):
        """x [S, hidden] bf16, weights [S, K] fp32 or None -> (rows [nvs, hidden] bf16, row_weights [nvs] fp32 or None)."""
        mp = self._mp
        if self._plan is None:
            raise RuntimeError("set_plan() first")
        if x.dtype != torch.bfloat16 or tuple(x.shape) != (self.s, self.h):
            raise ValueError("x must be bfloat16 [S, hidden]")
        x = x.contiguous()
        rows = torch.empty((self.nvs, self.h), dtype=torch.bfloat16, device=self.device)
        wsk = wnv = None
        kwargs = {}
        if weights is not None:
            wsk = weights.to(torch.float32).contiguous()
            wnv = torch.empty((self.nvs,), dtype=torch.float32, device=self.device)
            kwargs = dict(weights_sk=mp.tensor(wsk, mp.DT_FP32, (self.s, self.k)), weights_nvs=mp.tensor(wnv, mp.DT_FP32, (self.nvs,)))
        self._enter()
        ep.check(mp.dispatch_v1(self.comm, self._plan, mp.tensor(x, mp.DT_BF16, (self.s, self.h)),
                                mp.tensor(rows, mp.DT_BF16, (self.nvs, self.h)), self.stream,
                                flags=0 if self._built else mp.FLAG_BUILD_DEDUP, **kwargs), "TileXRMoonEpDispatchV1")
        self._built = True
        self._leave(x, rows, wsk, wnv)
        return rows, wnv

    def combine(self, rows: torch.Tensor, row_weights: Optional[torch.Tensor] = None):
        """rows [nvs, hidden] bf16 (expert outputs in the receive layout) -> (y [S, hidden] bf16, weights [S, K] or None)."""
        mp = self._mp
        if not self._built:
            raise RuntimeError("dispatch() builds the duplicate plan combine needs")
        rows = rows.contiguous()
        y = torch.empty((self.s, self.h), dtype=torch.bfloat16, device=self.device)
        wy = None
        kwargs = {}
        if row_weights is not None:
            row_weights = row_weights.to(torch.float32).contiguous()
            wy = torch.empty((self.s, self.k), dtype=torch.float32, device=self.device)
            kwargs = dict(weights_nvs=mp.tensor(row_weights, mp.DT_FP32, (self.nvs,)), weights_sk=mp.tensor(wy, mp.DT_FP32, (self.s, self.k)))
        self._enter()
        ep.check(mp.combine_v1(self.comm, self._plan, self._dst_local, mp.tensor(rows, mp.DT_BF16, (self.nvs, self.h)),
                               mp.tensor(y, mp.DT_BF16, (self.s, self.h)), self.stream, **kwargs), "TileXRMoonEpCombineV1")
        self._leave(rows, row_weights, y, wy)
        return y, wy
