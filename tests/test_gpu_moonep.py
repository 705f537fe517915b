"""GPU parity tests of the plan-driven (MoonEP) Dispatch / Combine stages: every call goes through the C ABI
(include/tilexr_moonep.h) and every output byte is compared with the CPU oracle on the same inputs."""
import numpy as np
import pytest
import torch

import moonep_cases as MC
from gpu_harness import DEV
from oracle import moonep as M
from tilexr_amd import ep, moonep as mp, workloads as W

pytestmark = pytest.mark.gpu

SENTINEL16 = 0x5a5a


def dev_bits16(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).to(DEV).view(torch.bfloat16)


def host_bits16(t):
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


class World:
    """All logical ranks of one world, one stream per rank.  torch's own work stays on the default stream and is waited
    for before the library is called on the ranks' streams."""

    def __init__(self, world):
        torch.cuda.set_device(0)
        self.world = world
        self.comms = [ep.Comm(world, r) for r in range(world)]
        self.streams = [torch.cuda.Stream() for _ in range(world)]
        self.keep = []

    def close(self):
        torch.cuda.synchronize()
        for c in self.comms:
            c.destroy()
        self.keep.clear()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def sync(self):
        for s in self.streams:
            s.synchronize()

    def plan_tensors(self, sh, dst, dup=None, experts=None):
        """Per-rank device tensors of a plan; a saved duplicate plan is uploaded, otherwise the arrays hold sentinels."""
        out = []
        for r in range(sh.world):
            t = dict(
                dst=torch.from_numpy(np.ascontiguousarray(dst[r])).to(DEV),
                groups=torch.full((sh.nvs, 3), -7, dtype=torch.int32, device=DEV),
                loffs=torch.full((sh.nvs,), -7, dtype=torch.int32, device=DEV),
                counts=torch.full((2,), -7, dtype=torch.int32, device=DEV),
                status=torch.full((8,), -1, dtype=torch.int32, device=DEV),
            )
            if dup is not None:
                t["groups"].copy_(torch.from_numpy(dup.groups[r]))
                t["loffs"].copy_(torch.from_numpy(dup.loffs[r]))
                t["counts"].copy_(torch.from_numpy(dup.counts[r]))
            e = experts if experts is not None else sh.world
            t["desc"] = mp.plan(sh.n, sh.world, e, 1, sh.nvs, sh.k, t["dst"], t["groups"], t["loffs"], t["counts"], t["status"])
            out.append(t)
        self.keep.append(out)
        return out

    def dispatch(self, sh, plans, hidden, weights=None, flags=0, order=None, expect=mp.SUCCESS):
        """hidden uint16 [world, s, h], weights fp32 [world, s*k] or None.  Returns device tensors per rank."""
        res = []
        for r in range(sh.world):
            t = dict(
                hidden=dev_bits16(hidden[r]),
                out=torch.full((sh.nvs, sh.h), 0, dtype=torch.int16, device=DEV).fill_(SENTINEL16).view(torch.bfloat16),
                w=None if weights is None else torch.from_numpy(np.ascontiguousarray(weights[r])).to(DEV).reshape(sh.s, sh.k),
                wout=None if weights is None else torch.full((sh.nvs,), -3.0, dtype=torch.float32, device=DEV),
            )
            res.append(t)
        self.keep.append(res)
        torch.cuda.synchronize()
        for r in (order if order is not None else range(sh.world)):
            t = res[r]
            ret = mp.dispatch_v1(
                self.comms[r], plans[r]["desc"], mp.tensor(t["hidden"], mp.DT_BF16, (sh.s, sh.h)),
                mp.tensor(t["out"], mp.DT_BF16, (sh.nvs, sh.h)), self.streams[r],
                weights_sk=None if weights is None else mp.tensor(t["w"], mp.DT_FP32, (sh.s, sh.k)),
                weights_nvs=None if weights is None else mp.tensor(t["wout"], mp.DT_FP32, (sh.nvs,)), flags=flags)
            assert ret == expect, f"rank {r}: dispatch returned {ret}"
        return res

    def combine(self, sh, plans, dst_local, rows, weights_nvs=None, order=None, expect=mp.SUCCESS):
        """rows: per-rank device tensors [nvs, h] bf16; weights_nvs: per-rank device tensors [nvs] or None."""
        res = []
        for r in range(sh.world):
            t = dict(
                dst_local=torch.from_numpy(np.ascontiguousarray(dst_local[r])).to(DEV),
                y=torch.full((sh.s, sh.h), 0, dtype=torch.int16, device=DEV).fill_(SENTINEL16).view(torch.bfloat16),
                wy=None if weights_nvs is None else torch.full((sh.s, sh.k), -3.0, dtype=torch.float32, device=DEV),
            )
            res.append(t)
        self.keep.append(res)
        torch.cuda.synchronize()
        for r in (order if order is not None else range(sh.world)):
            t = res[r]
            ret = mp.combine_v1(
                self.comms[r], plans[r]["desc"], t["dst_local"], mp.tensor(rows[r], mp.DT_BF16, (sh.nvs, sh.h)),
                mp.tensor(t["y"], mp.DT_BF16, (sh.s, sh.h)), self.streams[r],
                weights_nvs=None if weights_nvs is None else mp.tensor(weights_nvs[r], mp.DT_FP32, (sh.nvs,)),
                weights_sk=None if weights_nvs is None else mp.tensor(t["wy"], mp.DT_FP32, (sh.s, sh.k)))
            assert ret == expect, f"rank {r}: combine returned {ret}"
        return res


def check_dispatch(sh, res, plans, want, fresh):
    out, wout, status, dup = want
    for r in range(sh.world):
        assert int(plans[r]["status"][0].item()) == int(status[r]), f"rank {r} status"
        np.testing.assert_array_equal(host_bits16(res[r]["out"]), out[r], err_msg=f"rank {r} hiddenNvsh")
        if wout is not None:
            np.testing.assert_array_equal(res[r]["wout"].cpu().numpy(), wout[r], err_msg=f"rank {r} routeWeightsNvs")
        if fresh:
            counts = plans[r]["counts"].cpu().numpy()
            np.testing.assert_array_equal(counts, dup.counts[r], err_msg=f"rank {r} dupCounts")
            gc, dc = int(counts[0]), int(counts[1])
            np.testing.assert_array_equal(plans[r]["groups"].cpu().numpy()[:gc], dup.groups[r, :gc], err_msg=f"rank {r} dupGroups")
            np.testing.assert_array_equal(plans[r]["loffs"].cpu().numpy()[:dc], dup.loffs[r, :dc], err_msg=f"rank {r} dupLoffs")
            # nothing beyond the plan's extent is written
            assert (plans[r]["groups"].cpu().numpy()[gc:] == -7).all() and (plans[r]["loffs"].cpu().numpy()[dc:] == -7).all()


def random_rows(rng, shape):
    """bf16 bit patterns of finite values up to 2^97, both signs, subnormals included (sums of 32 stay finite)."""
    bits = rng.integers(0, 0x7000, size=shape, dtype=np.uint16)
    return bits | (rng.integers(0, 2, size=shape, dtype=np.uint16) << 15)


CASES = [
    # world, s, k, h, slack rows, weights, duplicates
    (1, 5, 1, 8, 0, False, False),
    (1, 33, 8, 64, 3, True, True),
    (2, 40, 2, 128, 0, True, False),
    (2, 17, 4, 7168, 9, True, True),
    (4, 64, 4, 1024, 5, False, True),
    (8, 21, 8, 512, 0, True, True),
    (3, 9, 32, 256, 11, True, True),
    (16, 4, 4, 64, 2, True, True),
    (2, 300, 8, 2048, 700, True, True),      # more than one 2048-row pass of the plan build, many unused rows
    (1, 2100, 8, 64, 700, True, True),       # nine passes: the plan's workgroups in the scatter launch read chunk totals
    (2, 13, 3, 17, 4, True, True),           # odd hidden size: element-wise kernels
    (4, 6, 5, 24, 0, False, True),           # rows of three 16-byte vectors
]


@pytest.fixture(params=["rows_cached", "rows_uncached"])
def row_cache(request):
    """Both scatter kernels: the library picks by the bytes of token rows against this setting."""
    previous = mp.set_cached_row_bytes(0 if request.param == "rows_uncached" else 1 << 40)
    yield "moon_scatter_token_kernel" if request.param == "rows_uncached" else "moon_scatter_kernel"
    mp.set_cached_row_bytes(previous)


@pytest.mark.parametrize("world,s,k,h,slack,with_weights,dups", CASES)
def test_dispatch_and_combine_match_oracle(world, s, k, h, slack, with_weights, dups, row_cache):
    rng = np.random.default_rng(world * 1000 + s * 10 + k)
    sh = M.Shape(world, s, k, h, s * k + slack)
    dst = MC.random_dst(sh, rng, duplicates=dups)
    hidden = random_rows(rng, (world, s, h))
    weights = rng.standard_normal((world, s * k)).astype(np.float32) if with_weights else None
    want = M.dispatch_world(sh, dst, hidden, weights, flags=M.FLAG_BUILD_DEDUP)
    with World(world) as w:
        plans = w.plan_tensors(sh, dst)
        res = w.dispatch(sh, plans, hidden, weights, flags=mp.FLAG_BUILD_DEDUP, order=list(rng.permutation(world)))
        w.sync()
        check_dispatch(sh, res, plans, want, fresh=True)
        if h % 8 == 0:
            assert ep.last_kernel_name(w.comms[0], ep.K_SCATTER) == row_cache
        # saved plan on the same world: same rows, the plan's arrays are left as they are
        before = [(p["groups"].clone(), p["loffs"].clone(), p["counts"].clone()) for p in plans]
        res2 = w.dispatch(sh, plans, hidden, weights, flags=0)
        w.sync()
        check_dispatch(sh, res2, plans, want, fresh=False)
        for p, (g, l, c) in zip(plans, before):
            assert torch.equal(p["groups"], g) and torch.equal(p["loffs"], l) and torch.equal(p["counts"], c)
        # combine over an "expert" that changes the rows, so that duplicate rows differ from their primaries
        out, wout, _, dup = want
        expert = random_rows(rng, (world, sh.nvs, h))
        rows = [dev_bits16(expert[r]) for r in range(world)]
        wn = None if weights is None else [res[r]["wout"] for r in range(world)]
        dst_local = M.build_dst_local(sh, dst)
        cres = w.combine(sh, plans, dst_local, rows, wn, order=list(rng.permutation(world)))
        w.sync()
        y, wy, cstatus = M.combine_world(sh, dst_local, dup, expert, wout)
        for r in range(world):
            assert int(plans[r]["status"][0].item()) == int(cstatus[r])
            np.testing.assert_array_equal(host_bits16(cres[r]["y"]), y[r], err_msg=f"rank {r} hiddenSh")
            if wy is not None:
                np.testing.assert_array_equal(cres[r]["wy"].cpu().numpy(), wy[r], err_msg=f"rank {r} routeWeightsSk")


@pytest.mark.parametrize("seed", range(24))
def test_random_shapes(seed, row_cache):
    """Small random worlds, hidden sizes on both sides of the vector / element-wise split, fresh and saved plans."""
    rng = np.random.default_rng(1000 + seed)
    world = int(rng.choice([1, 2, 3, 5, 8]))
    s = int(rng.integers(1, 70))
    k = int(rng.integers(1, 13))
    h = int(rng.choice([8, 16, 24, 40, 64, 136, 17, 33, 1]))
    slack = int(rng.integers(0, 20))
    with_weights = bool(rng.integers(0, 2))
    sh = M.Shape(world, s, k, h, s * k + slack)
    dst = MC.random_dst(sh, rng, duplicates=bool(rng.integers(0, 4)))
    hidden = random_rows(rng, (world, s, h))
    weights = rng.standard_normal((world, s * k)).astype(np.float32) if with_weights else None
    want = M.dispatch_world(sh, dst, hidden, weights, flags=M.FLAG_BUILD_DEDUP)
    with World(world) as w:
        plans = w.plan_tensors(sh, dst)
        res = w.dispatch(sh, plans, hidden, weights, flags=mp.FLAG_BUILD_DEDUP, order=list(rng.permutation(world)))
        w.sync()
        check_dispatch(sh, res, plans, want, fresh=True)
        res2 = w.dispatch(sh, plans, hidden, weights, flags=0, order=list(rng.permutation(world)))
        w.sync()
        check_dispatch(sh, res2, plans, want, fresh=False)
        out, wout, _, dup = want
        expert = random_rows(rng, (world, sh.nvs, h))
        dst_local = M.build_dst_local(sh, dst)
        cres = w.combine(sh, plans, dst_local, [dev_bits16(expert[r]) for r in range(world)],
                         None if weights is None else [res[r]["wout"] for r in range(world)])
        w.sync()
        y, wy, cstatus = M.combine_world(sh, dst_local, dup, expert, wout)
        for r in range(world):
            assert int(plans[r]["status"][0].item()) == int(cstatus[r])
            np.testing.assert_array_equal(host_bits16(cres[r]["y"]), y[r], err_msg=f"rank {r} hiddenSh")
            if wy is not None:
                np.testing.assert_array_equal(cres[r]["wy"].cpu().numpy(), wy[r], err_msg=f"rank {r} routeWeightsSk")


def test_home_plans_with_padding():
    """Plans as the reference's planner lays them out (expert groups padded to 8 rows, duplicates marked), fresh and
    saved, three exchanges back to back on one world without waiting in between."""
    world, s, k, experts, h = 4, 96, 8, 16, 256
    with World(world) as w:
        for it in range(3):
            plan, _ = MC.home_plan(world, s, k, experts, padding=8, seed=40 + it, slack=3)
            sh = M.Shape(world, s, k, h, plan["nvs"])
            dst = plan["dst"].numpy()
            rng = np.random.default_rng(it)
            hidden = random_rows(rng, (world, s, h))
            weights = rng.standard_normal((world, s * k)).astype(np.float32)
            want = M.dispatch_world(sh, dst, hidden, weights, flags=M.FLAG_BUILD_DEDUP)
            plans = w.plan_tensors(sh, dst, experts=experts)
            res = w.dispatch(sh, plans, hidden, weights, flags=mp.FLAG_BUILD_DEDUP)
            # identity expert: combine straight away on the same streams
            dst_local = M.build_dst_local(sh, dst)
            cres = w.combine(sh, plans, dst_local, [r["out"] for r in res], [r["wout"] for r in res])
            w.sync()
            out, wout, _, dup = want
            for r in range(world):
                np.testing.assert_array_equal(host_bits16(res[r]["out"]), out[r])
                np.testing.assert_array_equal(plans[r]["counts"].cpu().numpy(), dup.counts[r])
            y, wy, cstatus = M.combine_world(sh, dst_local, dup, out, wout)
            for r in range(world):
                assert int(plans[r]["status"][0].item()) == 0
                np.testing.assert_array_equal(host_bits16(cres[r]["y"]), y[r])
                np.testing.assert_array_equal(cres[r]["wy"].cpu().numpy().reshape(-1), weights[r])


def test_saved_plan_is_followed_as_given(row_cache):
    """A saved plan is data: an empty one leaves duplicate rows zero, and a plan in the CPU model's group order gives
    the same rows as the one the kernels build."""
    world, s, k, h = 2, 12, 4, 64
    rng = np.random.default_rng(3)
    sh = M.Shape(world, s, k, h, s * k + 2)
    dst = MC.random_dst(sh, rng, duplicates=True)
    hidden = random_rows(rng, (world, s, h))
    with World(world) as w:
        empty = M.DupPlan.empty(sh)
        plans = w.plan_tensors(sh, dst, dup=empty)
        res = w.dispatch(sh, plans, hidden, flags=0)
        w.sync()
        check_dispatch(sh, res, plans, M.dispatch_world(sh, dst, hidden, flags=0, dup=empty), fresh=False)
        built = M.dispatch_world(sh, dst, hidden, flags=M.FLAG_BUILD_DEDUP)[3]
        shuffled = built.copy()
        for q in range(world):                       # reverse the order of the groups, keep their slices
            gc = int(built.counts[q, 0])
            shuffled.groups[q, :gc] = built.groups[q, :gc][::-1]
        plans = w.plan_tensors(sh, dst, dup=shuffled)
        res = w.dispatch(sh, plans, hidden, flags=0)
        w.sync()
        check_dispatch(sh, res, plans, M.dispatch_world(sh, dst, hidden, flags=0, dup=shuffled), fresh=False)


def test_combine_with_groups_longer_than_a_wave():
    """A saved plan may list any number of duplicates under one primary: groups of 66 and 70 rows (the reduce kernel deals
    a token's rows to the 64 lanes of a wave, so these span two rounds) next to a short one.  Checked against the
    oracle on random rows and, on rows of small integers whose sums are exact in bf16 whatever the order, against the
    sum written out: the primary's slot returns the whole group, the duplicates' slots nothing."""
    world, s, k, h = 2, 50, 2, 136
    rng = np.random.default_rng(66)
    sh = M.Shape(world, s, k, h, s * k)
    dst = MC.random_dst(sh, rng, duplicates=False)
    dl = M.build_dst_local(sh, dst)
    dup = M.DupPlan.empty(sh)
    members = {}
    for q, sizes in ((0, (66,)), (1, (70, 3))):
        used = rng.permutation(np.flatnonzero(dl[q] >= 0))
        at = fill = 0
        for g, size in enumerate(sizes):
            rows = used[at:at + size + 1]
            at += size + 1
            dup.groups[q, g] = [rows[0], fill, size]
            dup.loffs[q, fill:fill + size] = rows[1:]
            fill += size
            members[(q, int(rows[0]))] = [int(r) for r in rows]
        dup.counts[q] = [len(sizes), fill]
    ints = rng.integers(-3, 4, (world, sh.nvs, h)).astype(np.float32)
    int_rows = (ints.view(np.uint32) >> 16).astype(np.uint16)
    with World(world) as w:
        for rows in (random_rows(rng, (world, sh.nvs, h)), int_rows):
            plans = w.plan_tensors(sh, dst, dup=dup)
            res = w.combine(sh, plans, dl, [dev_bits16(rows[r]) for r in range(world)])
            w.sync()
            want, _, status = M.combine_world(sh, dl, dup, rows)
            assert status.tolist() == [0, 0] == [int(p["status"][0].item()) for p in plans]
            for r in range(world):
                np.testing.assert_array_equal(host_bits16(res[r]["y"]), want[r], err_msg=f"rank {r}")
        # the integer rows once more, summed by hand
        total = np.zeros((world, s * k, h), np.float32)
        in_group = {(q, r) for (q, _), rows in members.items() for r in rows[1:]}
        for q in range(world):
            for row in np.flatnonzero(dl[q] >= 0):
                if (q, int(row)) in in_group:
                    continue
                origin, slot = divmod(int(dl[q, row]), sh.nvs)
                total[origin, slot] = sum(ints[q, r] for r in members.get((q, int(row)), [int(row)]))
        by_hand = total.reshape(world, s, k, h).sum(axis=2)
        for r in range(world):
            got = (host_bits16(res[r]["y"]).astype(np.uint32) << 16).view(np.float32)
            np.testing.assert_array_equal(got, by_hand[r])


def test_rows_that_are_not_finite():
    """Infinities, the largest finite values, NaNs and zeros of both signs among the rows, with and without duplicate
    groups: dispatch copies bits; combine's sums equal the oracle's element for element, NaNs up to sign and payload
    (which of two NaN operands an addition returns differs between the host's adder and the device's)."""
    world, s, k, h = 2, 24, 4, 72
    rng = np.random.default_rng(405)
    special = np.array([0x7f80, 0xff80, 0x7f7f, 0xff7f, 0x7fc0, 0xffc1, 0x7f81, 0x0000, 0x8000, 0x0001, 0x3f80, 0xbf80], np.uint16)
    for dups in (False, True):
        sh = M.Shape(world, s, k, h, s * k + 5)
        dst = MC.random_dst(sh, rng, duplicates=dups)
        hidden = special[rng.integers(0, len(special), size=(world, s, h))]
        want_out, _, _, want_dup = M.dispatch_world(sh, dst, hidden, flags=M.FLAG_BUILD_DEDUP)
        with World(world) as w:
            plans = w.plan_tensors(sh, dst)
            res = w.dispatch(sh, plans, hidden, flags=mp.FLAG_BUILD_DEDUP)
            w.sync()
            for r in range(world):
                assert int(plans[r]["status"][0].item()) == mp.DISPATCH_STATUS_SUCCESS
                np.testing.assert_array_equal(host_bits16(res[r]["out"]), want_out[r])
            dl = M.build_dst_local(sh, dst)
            got = w.combine(sh, plans, dl, [res[r]["out"] for r in range(world)])
            w.sync()
            want_y, _, _ = M.combine_world(sh, dl, want_dup, want_out)
            for r in range(world):
                a, b = host_bits16(got[r]["y"]), want_y[r]
                nan_a, nan_b = (a & 0x7fff) > 0x7f80, (b & 0x7fff) > 0x7f80
                np.testing.assert_array_equal(nan_a, nan_b)
                np.testing.assert_array_equal(a[~nan_a], b[~nan_b])
                assert nan_a.any() and ((a & 0x7fff) == 0x7f80).any()


def test_device_status_of_bad_plans(row_cache):
    world, s, k, h = 3, 8, 2, 64
    rng = np.random.default_rng(9)
    sh = M.Shape(world, s, k, h, s * k)
    dst = MC.random_dst(sh, rng, duplicates=False)
    hidden = random_rows(rng, (world, s, h))
    with World(world) as w:
        bad = dst.copy()
        bad[1, 5] = world * sh.nvs                    # a rank that does not exist
        plans = w.plan_tensors(sh, bad)
        w.dispatch(sh, plans, hidden, flags=mp.FLAG_BUILD_DEDUP)
        w.sync()
        want = M.dispatch_world(sh, bad, hidden, flags=M.FLAG_BUILD_DEDUP)[2]
        assert [int(p["status"][0].item()) for p in plans] == want.tolist() == [2101, 2001, 2101]
        orphan = dst.copy()
        orphan[2, 0] = -int(orphan[2, 0]) - 1         # a duplicate with no earlier route of its token to that rank
        plans = w.plan_tensors(sh, orphan)
        w.dispatch(sh, plans, hidden, flags=mp.FLAG_BUILD_DEDUP)
        w.sync()
        assert [int(p["status"][0].item()) for p in plans] == [2102, 2102, 2001]
        # combine: a reverse route to a rank that does not exist; a group whose duplicate is its own primary
        rows = [dev_bits16(random_rows(rng, (sh.nvs, h))) for r in range(world)]
        good = M.DupPlan.empty(sh)
        dl = M.build_dst_local(sh, dst)
        bad_dl = dl.copy()
        bad_dl[0, 3] = world * sh.nvs
        plans = w.plan_tensors(sh, dst, dup=good)
        w.combine(sh, plans, bad_dl, rows)
        w.sync()
        assert [int(p["status"][0].item()) for p in plans] == [3001, 3100, 3100]
        self_dup = M.DupPlan.empty(sh)
        self_dup.groups[1, 0] = [2, 0, 1]
        self_dup.loffs[1, 0] = 2
        self_dup.counts[1] = [1, 1]
        plans = w.plan_tensors(sh, dst, dup=self_dup)
        w.combine(sh, plans, dl, rows)
        w.sync()
        assert [int(p["status"][0].item()) for p in plans] == [3101, 3001, 3101]
        # the world is still usable afterwards
        plans = w.plan_tensors(sh, dst)
        res = w.dispatch(sh, plans, hidden, flags=mp.FLAG_BUILD_DEDUP)
        w.sync()
        check_dispatch(sh, res, plans, M.dispatch_world(sh, dst, hidden, flags=M.FLAG_BUILD_DEDUP), fresh=True)


@pytest.mark.parametrize("world,invalid", [(5, (1, 3)), (6, (0, 2, 5)), (4, (3,))])
def test_device_status_with_several_invalid_plans(world, invalid):
    """Several invalid plans in one exchange: every rank's status is the closed form stated in include/tilexr_moonep.h
    (dispatch names the first invalid rank upwards from one's own, combine the lowest), and the world works afterwards."""
    s, k, h = 8, 2, 64
    rng = np.random.default_rng(31 + world)
    sh = M.Shape(world, s, k, h, s * k)
    dst = MC.random_dst(sh, rng, duplicates=False)
    hidden = random_rows(rng, (world, s, h))
    with World(world) as w:
        bad = dst.copy()
        for r in invalid:
            bad[r, int(rng.integers(sh.n))] = world * sh.nvs
        plans = w.plan_tensors(sh, bad)
        w.dispatch(sh, plans, hidden, flags=mp.FLAG_BUILD_DEDUP)
        w.sync()
        got = [int(p["status"][0].item()) for p in plans]
        assert got == MC.status_with_invalid_plans(world, invalid, "dispatch")
        assert got == M.dispatch_world(sh, bad, hidden, flags=M.FLAG_BUILD_DEDUP)[2].tolist()
        rows = [dev_bits16(random_rows(rng, (sh.nvs, h))) for r in range(world)]
        dl = M.build_dst_local(sh, dst)
        bad_dl = dl.copy()
        for r in invalid:
            bad_dl[r, int(rng.choice(np.flatnonzero(dl[r] >= 0)))] = world * sh.nvs
        plans = w.plan_tensors(sh, dst, dup=M.DupPlan.empty(sh))
        w.combine(sh, plans, bad_dl, rows)
        w.sync()
        assert [int(p["status"][0].item()) for p in plans] == MC.status_with_invalid_plans(world, invalid, "combine")
        plans = w.plan_tensors(sh, dst)
        res = w.dispatch(sh, plans, hidden, flags=mp.FLAG_BUILD_DEDUP)
        w.sync()
        check_dispatch(sh, res, plans, M.dispatch_world(sh, dst, hidden, flags=M.FLAG_BUILD_DEDUP), fresh=True)


def test_argument_rules_on_the_device():
    """What needs a live device to be told apart: a call that is valid except for the registered workspace, and
    disagreeing ranks."""
    world, s, k, h = 2, 4, 2, 64
    rng = np.random.default_rng(1)
    sh = M.Shape(world, s, k, h, s * k)
    dst = MC.random_dst(sh, rng, duplicates=False)
    hidden = random_rows(rng, (world, s, h))
    with World(world) as w:
        plans = w.plan_tensors(sh, dst)
        x = dev_bits16(hidden[0])
        out = torch.zeros((sh.nvs, h), dtype=torch.bfloat16, device=DEV)
        torch.cuda.synchronize()
        args = (w.comms[0], plans[0]["desc"], mp.tensor(x, mp.DT_BF16, (s, h)), mp.tensor(out, mp.DT_BF16, (sh.nvs, h)),
                w.streams[0])
        assert mp.dispatch_v1(*args, registered_workspace=out.data_ptr(), registered_workspace_bytes=64) == mp.ERR_NOT_SUPPORTED
        assert mp.dispatch_v1(*args, flags=mp.FLAG_ZERO_COPY) == mp.ERR_NOT_SUPPORTED
        assert mp.dispatch_v1(*args, flags=1 << 20) == mp.ERR_INVALID_ARGUMENT
        assert mp.dispatch_v1(*args[:4], None) == mp.ERR_INVALID_ARGUMENT
        # rank 0 files a call and may not file another while it waits; rank 1 disagrees about the flags: it is refused
        # and rank 0's call is cancelled with rank 1 named as the failed peer; then both call again and the exchange runs
        assert mp.dispatch_v1(*args, flags=mp.FLAG_BUILD_DEDUP) == mp.SUCCESS
        assert mp.dispatch_v1(*args, flags=mp.FLAG_BUILD_DEDUP) == mp.ERR_INTERNAL
        x1 = dev_bits16(hidden[1])
        out1 = torch.zeros((sh.nvs, h), dtype=torch.bfloat16, device=DEV)
        torch.cuda.synchronize()
        args1 = (w.comms[1], plans[1]["desc"], mp.tensor(x1, mp.DT_BF16, (s, h)), mp.tensor(out1, mp.DT_BF16, (sh.nvs, h)),
                 w.streams[1])
        assert mp.dispatch_v1(*args1, flags=0) == mp.ERR_INVALID_ARGUMENT
        w.sync()
        assert int(plans[0]["status"][0].item()) == mp.DISPATCH_STATUS_REMOTE_FAILURE_BASE + 1
        assert int(plans[1]["status"][0].item()) == -1          # the refused call left nothing behind
        assert not out.view(torch.int16).any().item()           # and the cancelled one wrote no row
        assert mp.dispatch_v1(*args1, flags=mp.FLAG_BUILD_DEDUP) == mp.SUCCESS
        assert mp.dispatch_v1(*args, flags=mp.FLAG_BUILD_DEDUP) == mp.SUCCESS
        w.sync()
        assert int(plans[0]["status"][0].item()) == int(plans[1]["status"][0].item()) == mp.DISPATCH_STATUS_SUCCESS
        want = M.dispatch_world(sh, dst, hidden, flags=M.FLAG_BUILD_DEDUP)
        np.testing.assert_array_equal(host_bits16(out), want[0][0])
        np.testing.assert_array_equal(host_bits16(out1), want[0][1])


def test_published_shape_round_trip():
    """One rank's share at the shape the reference publishes stage timings for (S=4096, K=8, H=7168, 32 experts over 8
    ranks), on a one-rank world so that it fits a test: every route stays on the rank, seven of a token's eight rows
    are duplicates.  Checked through properties that need no oracle run at this size: every receive row equals its
    token's row, and with an identity expert combine returns bf16(8 * x)."""
    s, k, h, experts = 4096, 8, 7168, 8
    plan, ids = MC.home_plan(1, s, k, experts, padding=1, seed=77)
    sh = M.Shape(1, s, k, h, plan["nvs"])
    dst = plan["dst"].numpy()
    g = torch.Generator().manual_seed(5)
    x = torch.randn(s, h, generator=g).to(torch.bfloat16)
    weights = torch.rand(s, k, generator=g)
    with World(1) as w:
        plans = w.plan_tensors(sh, dst, experts=experts)
        xd, wd = x.to(DEV), weights.to(DEV)
        out = torch.empty((sh.nvs, h), dtype=torch.bfloat16, device=DEV)
        wout = torch.empty((sh.nvs,), dtype=torch.float32, device=DEV)
        torch.cuda.synchronize()
        assert mp.dispatch_v1(w.comms[0], plans[0]["desc"], mp.tensor(xd, mp.DT_BF16, (s, h)),
                              mp.tensor(out, mp.DT_BF16, (sh.nvs, h)), w.streams[0],
                              weights_sk=mp.tensor(wd, mp.DT_FP32, (s, k)), weights_nvs=mp.tensor(wout, mp.DT_FP32, (sh.nvs,)),
                              flags=mp.FLAG_BUILD_DEDUP) == mp.SUCCESS
        w.sync()
        assert int(plans[0]["status"][0].item()) == 2000
        raw = torch.from_numpy(np.where(dst[0] >= 0, dst[0], -dst[0].astype(np.int64) - 1)).to(DEV)
        token = torch.arange(s * k, device=DEV) // k
        assert torch.equal(out[raw].view(torch.int16), xd[token].view(torch.int16))
        assert torch.equal(wout[raw], wd.reshape(-1))
        counts = plans[0]["counts"].cpu().numpy()
        assert counts.tolist() == [s, s * (k - 1)]
        y = torch.empty((s, h), dtype=torch.bfloat16, device=DEV)
        wy = torch.empty((s, k), dtype=torch.float32, device=DEV)
        dl = torch.from_numpy(M.build_dst_local(sh, dst)[0]).to(DEV)
        torch.cuda.synchronize()
        assert mp.combine_v1(w.comms[0], plans[0]["desc"], dl, mp.tensor(out, mp.DT_BF16, (sh.nvs, h)),
                             mp.tensor(y, mp.DT_BF16, (s, h)), w.streams[0], weights_nvs=mp.tensor(wout, mp.DT_FP32, (sh.nvs,)),
                             weights_sk=mp.tensor(wy, mp.DT_FP32, (s, k))) == mp.SUCCESS
        w.sync()
        assert int(plans[0]["status"][0].item()) == 0
        want = (xd.float() * 8.0).to(torch.bfloat16)
        assert torch.equal(y.view(torch.int16), want.view(torch.int16))
        assert torch.equal(wy, wd)
