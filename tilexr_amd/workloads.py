"""Seeded synthetic inputs for the five dispatch/combine configurations this library is measured and tested on.

Everything is generated on the CPU with torch generators so the same seed gives the same bytes everywhere;
`describe()` reports a sha256 of the expert-id table so two runs can be compared.

  C1  128 x 1024 bf16 N(0,1); 16 experts as 4 logical ranks x 4; top-2 distinct uniform; softmax weights
  C2  128 x 7168 bf16 N(0,1); 256 experts; top-8 of N(0,1) gating logits, softmax renormalised over the 8
  C3  4096 x 7168 bf16 N(0,1); 256 experts; 8 distinct experts per token sampled without replacement from a
      Zipf(s=1.0) popularity laid over a seeded permutation of the experts; softmax weights of N(0,1) logits
  C4  8192 x 4096 bf16 N(0, sigma=2); 64 experts; top-6 distinct uniform; per-token int8 payload
  C5  16384 x 2048 bf16 Student-t(df=3); 128 experts; top-8 Zipf(s=1.2); fp8 e4m3 with fp32 scale per 128 columns;
      capacity ceil(1.25 * bs * K / E) rows per expert
"""
import hashlib
import math
from dataclasses import dataclass, field

import torch


@dataclass
class Workload:
    name: str
    ranks: int
    bs: int
    h: int
    top_k: int
    experts: int
    x_dist: str = "normal"          # normal | normal2 | student_t3
    routing: str = "uniform"        # uniform | gating | zipf
    zipf_s: float = 1.0
    quant: str = "none"             # none | int8 | fp8_block128
    capacity_factor: float = 0.0
    seed: int = 1234
    extra: dict = field(default_factory=dict)

    @property
    def capacity(self):
        if self.capacity_factor <= 0:
            return 0
        return int(math.ceil(self.capacity_factor * self.bs * self.top_k / self.experts))


CONFIGS = {
    "C1": Workload("C1", 4, 128, 1024, 2, 16, routing="uniform"),
    "C2": Workload("C2", 1, 128, 7168, 8, 256, routing="gating"),
    "C3": Workload("C3", 1, 4096, 7168, 8, 256, routing="zipf", zipf_s=1.0),
    "C4": Workload("C4", 1, 8192, 4096, 6, 64, x_dist="normal2", routing="uniform", quant="int8"),
    "C5": Workload("C5", 1, 16384, 2048, 8, 128, x_dist="student_t3", routing="zipf", zipf_s=1.2,
                   quant="fp8_block128", capacity_factor=1.25),
}


def scaled(w: Workload, bs: int, name=None) -> Workload:
    """Same shape per token, fewer tokens (used where a CPU check has to finish in seconds)."""
    return Workload(name or f"{w.name}@{bs}", w.ranks, bs, w.h, w.top_k, w.experts, w.x_dist, w.routing, w.zipf_s,
                    w.quant, w.capacity_factor, w.seed)


def _gen(seed):
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def make_x(w: Workload, rank=0):
    """[bs, h] bfloat16 on the CPU."""
    g = _gen(w.seed * 1000 + 17 + rank)
    if w.x_dist == "normal":
        x = torch.randn(w.bs, w.h, generator=g)
    elif w.x_dist == "normal2":
        x = torch.randn(w.bs, w.h, generator=g) * 2.0          # standard deviation 2
    elif w.x_dist == "student_t3":
        # t(3) = Z / sqrt(chi2_3 / 3)
        z = torch.randn(w.bs, w.h, generator=g)
        chi = torch.randn(3, w.bs, w.h, generator=g).pow(2).sum(0)
        x = z / torch.sqrt(chi / 3.0)
    else:
        raise ValueError(w.x_dist)
    return x.to(torch.bfloat16)


def make_routing(w: Workload, rank=0):
    """(expert_ids int32 [bs, K], weights fp32 [bs, K]) on the CPU."""
    g = _gen(w.seed * 1000 + 101 + rank)
    E, K = w.experts, w.top_k
    if w.routing == "gating":
        logits = torch.randn(w.bs, E, generator=g)
        top, ids = torch.topk(logits, K, dim=1)
        weights = torch.softmax(top, dim=1)
    else:
        if w.routing == "uniform":
            logp = torch.zeros(E)
        elif w.routing == "zipf":
            perm = torch.randperm(E, generator=_gen(w.seed * 1000 + 7))
            p = 1.0 / torch.arange(1, E + 1, dtype=torch.float64).pow(w.zipf_s)
            p = p / p.sum()
            logp = torch.empty(E, dtype=torch.float64)
            logp[perm] = p.log()
            logp = logp.float()
        else:
            raise ValueError(w.routing)
        # Gumbel top-K = sampling K distinct experts without replacement, proportionally to p
        u = torch.rand(w.bs, E, generator=g).clamp_(1e-12, 1.0 - 1e-7)
        keys = logp[None, :] - torch.log(-torch.log(u))
        ids = torch.topk(keys, K, dim=1).indices
        weights = torch.softmax(torch.randn(w.bs, K, generator=g), dim=1)
    return ids.to(torch.int32).contiguous(), weights.float().contiguous()


def describe(w: Workload, ids):
    return {
        "workload": w.name, "tokens": w.bs, "hidden": w.h, "top_k": w.top_k, "experts": w.experts,
        "logical_ranks": w.ranks, "routing": w.routing, "payload": w.quant, "capacity": w.capacity, "seed": w.seed,
        "ids_sha256": hashlib.sha256(ids.numpy().tobytes()).hexdigest()[:16],
    }


def algorithmic_bytes(w: Workload, kept_rows: int, inverse_index: bool = False):
    """Bytes one dispatch and one combine must move (flags and scratch excluded):
       dispatch = T*H*2 (read x once) + T*K*4 (ids) + rows*(H*b + s) (write rows) + rows*16 (assist) + E*12 (counts)
       combine  = rows*(H*b + s) (read rows) + rows*16 (read map) + T*K*4 (weights) + T*H*2 (write y)
    With `inverse_index` the combine reads the [T, K] row map dispatch produced (T*K*4) instead of the tuples."""
    T, H, K, E = w.bs, w.h, w.top_k, w.experts
    if w.quant == "none":
        b, s = 2, 0
    elif w.quant == "int8":
        b, s = 1, 4
    else:
        b, s = 1, 4 * ((H + 127) // 128)
    row = H * b + s
    dispatch = T * H * 2 + T * K * 4 + kept_rows * row + kept_rows * 16 + E * 12
    combine = kept_rows * row + (T * K * 4 if inverse_index else kept_rows * 16) + T * K * 4 + T * H * 2
    return dispatch, combine


# ---- plan-driven (MoonEP) stages ---------------------------------------------------------------------------------
# M1  8 logical ranks x (4096 x 7168 bf16 N(0,1)); 32 experts (4 per rank); top-8 distinct uniform; fp32 route weights.
#     The shape the reference publishes its MoonEP stage timings for (S=4096, K=8, H=7168, E=32, EP8).
MOONEP_CONFIGS = {
    "M1": Workload("M1", 8, 4096, 7168, 8, 32, routing="uniform"),
}


def moonep_home_plan(topk_experts, experts, token_padding=1, prefetch_slots=1, slack_rows=0):
    """Plan of a world in which every expert is served by its home rank (no expert is replicated).

    topk_experts: int32 tensor [R, S, K].  Returns a dict with
      dst         int32 [R, S*K]  signed route words: rank * nvS + row, negated (-raw - 1) when an earlier route of the
                                  same token already goes to that rank
      cu_seqlens  int32 [R, E+B]  cumulative padded group ends of every rank's receive tensor (groups = the E experts,
                                  then the B prefetch slots, all empty here)
      nvs         rows of every rank's receive tensor
    It follows the reference planner's layout and route numbering for the case without expert moves
    (src/moonep/planner_v2/reference/ep_plan_reference.cpp:436-459 segments, :461-538 layouts, :540-595 route words):
    on its home rank an expert's rows are ordered by source rank, then by the order its routes appear in the source's
    [S, K] table; groups are padded to `token_padding` rows.  The reference sizes nvS for a balanced world
    (S*K + (padding-1) * 2 * E/R, moonep_stage_reference.cpp:86-107); here it is the larger of that and what the busiest
    rank receives, plus `slack_rows`, because nothing rebalances this plan."""
    R, S, K = topk_experts.shape
    E, B = experts, prefetch_slots
    per_rank = E // R
    ids = topk_experts.to(torch.int64).reshape(R, S * K)
    home = ids // per_rank                                              # [R, N]
    counts = torch.zeros(R, E, dtype=torch.int64)
    counts.scatter_add_(1, ids, torch.ones_like(ids))                   # [src, expert]
    seg_begin = torch.cumsum(counts, dim=0) - counts                     # rows of earlier sources within the expert
    total = counts.sum(0)                                                # [E] rows of each expert on its home rank
    padded = torch.where(total > 0, (total + token_padding - 1) // token_padding * token_padding, total)
    cu = torch.zeros(R, E + B, dtype=torch.int64)
    base = torch.zeros(E, dtype=torch.int64)
    for d in range(R):
        sizes = torch.zeros(E + B, dtype=torch.int64)
        sizes[d * per_rank:(d + 1) * per_rank] = padded[d * per_rank:(d + 1) * per_rank]
        ends = torch.cumsum(sizes, 0)
        cu[d] = ends
        base[d * per_rank:(d + 1) * per_rank] = (ends - sizes)[d * per_rank:(d + 1) * per_rank]
    nvs = max(S * K + (token_padding - 1) * 2 * per_rank, int(cu[:, -1].max())) + slack_rows
    # ordinal of a route among its source's routes to the same expert, in table order
    order = torch.argsort(ids, dim=1, stable=True)
    sorted_ids = torch.gather(ids, 1, order)
    first = torch.searchsorted(sorted_ids, sorted_ids, right=False)      # start of each expert's run per source
    ordinal = torch.empty_like(ids)
    ordinal.scatter_(1, order, torch.arange(S * K).expand(R, -1) - first)
    src_index = torch.arange(R).unsqueeze(1).expand(R, S * K)
    row = base[ids] + seg_begin[src_index, ids] + ordinal
    raw = home * nvs + row
    # a route is a duplicate when an earlier route of its token goes to the same rank
    hk = home.reshape(R, S, K)
    same = hk.unsqueeze(3) == hk.unsqueeze(2)                            # [R, S, k, j]
    earlier = torch.tril(torch.ones(K, K, dtype=torch.bool), diagonal=-1)
    dup = (same & earlier).any(dim=3).reshape(R, S * K)
    dst = torch.where(dup, -raw - 1, raw)
    assert int(raw.max()) < 2 ** 31
    return {"dst": dst.to(torch.int32).contiguous(), "cu_seqlens": cu.to(torch.int32), "nvs": int(nvs)}


def moonep_dst_local(dst, nvs):
    """Reverse routes of a world for Combine: int32 [R, nvs], entry [rank][row] = source rank * nvs + route index of
    the route that lands on that row, -1 where none does (reference: the dstLocal input of
    src/moonep/combine/kernels/tilexr_moonep_combine_kernel.cpp:117-177).  `dst` int32 [R, S*K] as moonep_home_plan
    returns it; raises ValueError for a route word outside the world."""
    R, n = dst.shape
    raw = torch.where(dst >= 0, dst, -dst - 1).to(torch.int64)
    if int(raw.max()) >= R * nvs:
        raise ValueError("a route word names a row outside the world")
    out = torch.full((R * nvs,), -1, dtype=torch.int32)
    src = torch.arange(R, dtype=torch.int64).unsqueeze(1) * nvs + torch.arange(n, dtype=torch.int64).unsqueeze(0)
    out[raw.reshape(-1)] = src.reshape(-1).to(torch.int32)
    return out.reshape(R, nvs)


def moonep_algorithmic_bytes(s: int, k: int, h: int, with_weights: bool = True):
    """Bytes one rank's dispatch and combine must move when every route names its own row:
       dispatch = S*H*2 (read tokens once) + S*K*4 (route words) + S*K*H*2 (write rows) [+ S*K*8 weights in and out]
       combine  = S*K*H*2 (read rows) + S*K*4 (reverse routes) + S*H*2 (write tokens) [+ S*K*8 weights]"""
    w = s * k * 8 if with_weights else 0
    dispatch = s * h * 2 + s * k * 4 + s * k * h * 2 + w
    combine = s * k * h * 2 + s * k * 4 + s * h * 2 + w
    return dispatch, combine
