"""Plans and inputs shared by the CPU and GPU tests of the plan-driven (MoonEP) stages."""
import numpy as np
import torch

from oracle import moonep as M
from tilexr_amd import workloads as W


def balanced_dst(sh: M.Shape):
    """Route g = src * n + route goes to rank g % world, row g // world (the reference unit test's balanced plan,
    tests/moonep/unit/test_tilexr_moonep_stage_reference.cpp:35-51, with nvS rows per rank)."""
    n = sh.n
    g = np.arange(sh.world * n).reshape(sh.world, n)
    return ((g % sh.world) * sh.nvs + g // sh.world).astype(np.int32)


def random_dst(sh: M.Shape, rng, duplicates=True):
    """A random consistent plan: every route gets a row of its own somewhere in the world; with `duplicates` a route is
    marked as a duplicate when an earlier route of its token goes to the same rank, otherwise the rows are dealt so that
    no token visits a rank twice (which needs k <= world) or, when k > world, all routes stay non-negative."""
    world, n, nvs, k = sh.world, sh.n, sh.nvs, sh.k
    rows = rng.permutation(world * nvs)[:world * n].reshape(world, n)
    if not duplicates and k <= world:
        # give each token k distinct ranks, then rows on those ranks
        free = [list(rng.permutation(nvs)) for _ in range(world)]
        rows = np.zeros((world, n), np.int64)
        load = np.zeros(world, np.int64)
        for src in range(world):
            for t in range(sh.s):
                # prefer the emptiest ranks so no rank runs out of rows
                order = np.argsort(load + rng.random(world))[:k]
                for j, peer in enumerate(rng.permutation(order)):
                    rows[src, t * k + j] = peer * nvs + free[peer].pop()
                    load[peer] += 1
    dst = rows.astype(np.int64)
    if duplicates:
        peer = (dst // nvs).reshape(world, sh.s, k)
        same = peer[:, :, :, None] == peer[:, :, None, :]
        earlier = np.tril(np.ones((k, k), bool), -1)
        dup = (same & earlier).any(axis=3).reshape(world, n)
        dst = np.where(dup, -dst - 1, dst)
    return dst.astype(np.int32)


def status_with_invalid_plans(world, invalid, stage):
    """Device status of every rank when the ranks in `invalid` hold an invalid plan, written out from the rule in
    include/tilexr_moonep.h without the oracle: an invalid rank reports its own code; a valid one names the first invalid
    rank after itself going upwards with wrap-around (dispatch), or the lowest invalid rank (combine)."""
    own, base, ok = {"dispatch": (2001, 2100, 2000), "combine": (3001, 3100, 0)}[stage]
    invalid = sorted(set(invalid))
    out = []
    for r in range(world):
        if not invalid:
            out.append(ok)
        elif r in invalid:
            out.append(own)
        elif stage == "dispatch":
            out.append(base + min(invalid, key=lambda p: (p - r) % world))
        else:
            out.append(base + invalid[0])
    return out


def groups_as_sets(plan: M.DupPlan, rank):
    out = {}
    for g in range(int(plan.counts[rank, 0])):
        primary, start, count = (int(v) for v in plan.groups[rank, g])
        out[primary] = frozenset(int(v) for v in plan.loffs[rank, start:start + count])
    return out


def uniform_experts(world, s, k, experts, seed):
    g = torch.Generator().manual_seed(seed)
    keys = torch.rand(world, s, experts, generator=g)
    return torch.topk(keys, k, dim=2).indices.to(torch.int32)


def home_plan(world, s, k, experts, padding=1, seed=0, slack=0):
    ids = uniform_experts(world, s, k, experts, seed)
    return W.moonep_home_plan(ids, experts, token_padding=padding, slack_rows=slack), ids
