"""CPU tests that pin the oracle of the plan-driven (MoonEP) stages.

Pins, in order: the known answers the reference's own unit test holds for its CPU model
(tests/moonep/unit/test_tilexr_moonep_stage_reference.cpp:115-128, 130-163, 165-225, 271-310), restated here as data;
a build of that CPU model (oracle/_ref, where the reference checkout was present) on random plans; and closed forms
for the two places where the device kernels -- which the oracle follows -- differ from the CPU model."""
import numpy as np
import pytest

from oracle import moonep as M
import moonep_cases as MC


def bf16(values):
    """float32 array -> bf16 bits, round to nearest even (no NaNs in these tests)."""
    u = np.asarray(values, np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7fff + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def f32(bits):
    return (np.asarray(bits, np.uint16).astype(np.uint32) << 16).view(np.float32)


@pytest.fixture(scope="module")
def mref():
    if not M.ref_available():
        pytest.skip("oracle/_ref not built (reference checkout absent)")
    M.ref()
    return M


# ---- known answers held by the reference's unit test ---------------------------------------------------------------
def test_decode_known_answers():
    assert M.decode_route(0, 8, 2) == (0, 0, 0, False)
    assert M.decode_route(10, 8, 2) == (0, 1, 2, False)
    assert M.decode_route(-11, 8, 2) == (0, 1, 2, True)
    assert M.decode_route(-2 ** 31, 268435456, 8) == (0, 7, 268435455, True)
    assert M.decode_route(16, 8, 2)[0] != 0


def test_nvs_and_padded_layout_known_answers():
    assert M.compute_nvs(4, 2, 8, 2, 4) == (0, 32)
    assert M.compute_nvs(4, 2, 7, 2, 4)[0] != 0
    ret, cu, ranges = M.padded_layout([3, 0, 5, 1], 4, 16)
    assert ret == 0 and cu.tolist() == [4, 4, 12, 16]
    assert ranges.tolist() == [[3, 1], [0, 0], [9, 3], [13, 3]]
    ret, cu, ranges = M.padded_layout([3, 0, 5, 1], 4, 20)
    assert ret == 0 and cu.tolist() == [4, 4, 12, 16] and ranges[3].tolist() == [13, 7]
    assert M.padded_layout([3, 5], 4, 8)[0] != 0


def test_duplicate_plan_known_answer():
    sh = M.Shape(2, 2, 3, 4, 8)
    dst = np.array([[0, -2, -3, 3, 12, -14], [4, -6, 7, 8, -10, -11]], np.int32)
    hidden = np.arange(2 * 2 * 4, dtype=np.uint16).reshape(2, 2, 4) + 1
    _, _, status, dup = M.dispatch_world(sh, dst, hidden, flags=M.FLAG_BUILD_DEDUP)
    assert status.tolist() == [M.DISPATCH_OK] * 2
    assert dup.counts[0].tolist() == [2, 3]
    assert dup.groups[0, 0].tolist() == [0, 0, 2]
    assert dup.loffs[0, :2].tolist() == [1, 2]
    # the rest of rank 0's plan and rank 1's follow from the same rule
    assert dup.groups[0, 1].tolist() == [4, 2, 1] and dup.loffs[0, 2] == 5
    assert dup.counts[1].tolist() == [2, 3]
    assert dup.groups[1, :2].tolist() == [[0, 0, 2], [4, 2, 1]] and dup.loffs[1, :3].tolist() == [1, 2, 5]


def test_balanced_round_trip_is_k_times_input():
    """reference unit test :130-163: without duplicates combine(dispatch(x)) = bf16(k * x), weights come back unchanged"""
    sh = M.Shape(2, 3, 2, 4, 6)
    dst = MC.balanced_dst(sh)
    hidden = bf16(np.arange(2 * 3 * 4, dtype=np.float32).reshape(2, 3, 4) + np.array([1, 101])[:, None, None])
    weights = (np.arange(12, dtype=np.float32).reshape(2, 6) + 0.25 + np.array([0, 1000])[:, None]).astype(np.float32)
    out, wout, status, dup = M.dispatch_world(sh, dst, hidden, weights, flags=M.FLAG_BUILD_DEDUP)
    assert status.tolist() == [M.DISPATCH_OK] * 2 and dup.counts.tolist() == [[0, 0], [0, 0]]
    y, wy, cstatus = M.combine_world(sh, M.build_dst_local(sh, dst), dup, out, wout)
    assert cstatus.tolist() == [M.COMBINE_OK] * 2
    np.testing.assert_array_equal(y, bf16(f32(hidden) * 2.0))
    np.testing.assert_array_equal(wy.reshape(2, 6), weights)


def test_unused_rows_are_zero():
    """reference unit test :194-224: rows no route names stay zero (also the weights)"""
    sh = M.Shape(2, 2, 2, 3, 4)
    dst = np.array([[0, 1, 2, 3], [0 + 4, 1 + 4, 2 + 4, -(2 + 4) - 1]], np.int32)     # rank 1 row 3 is never named
    hidden = np.full((2, 2, 3), 0x4000, np.uint16)
    weights = np.ones((2, 4), np.float32)
    out, wout, status, _ = M.dispatch_world(sh, dst, hidden, weights)
    assert status.tolist() == [M.DISPATCH_OK] * 2
    assert not out[1, 3].any() and wout[1, 3] == 0.0
    assert out[0].all() and out[1, :3].all()


# ---- against a build of the reference's CPU model -------------------------------------------------------------------
@pytest.mark.parametrize("world,s,k,h,slack", [(1, 5, 1, 8, 0), (2, 7, 2, 16, 3), (4, 9, 4, 8, 5), (8, 3, 8, 24, 0),
                                               (2, 2, 32, 8, 7)])
def test_without_duplicates_oracle_equals_reference_model(mref, world, s, k, h, slack):
    rng = np.random.default_rng(world * 100 + k)
    sh = M.Shape(world, s, k, h, s * k + slack)
    dst = MC.random_dst(sh, rng, duplicates=False)
    hidden = rng.integers(0, 0x7000, size=(world, s, h), dtype=np.uint16) | (rng.integers(0, 2, size=(world, s, h),
                                                                                          dtype=np.uint16) << 15)
    weights = rng.standard_normal((world, s * k)).astype(np.float32)
    out, wout, status, dup = M.dispatch_world(sh, dst, hidden, weights, flags=M.FLAG_BUILD_DEDUP)
    rout, rwout = mref.ref_dispatch(sh, dst, hidden, weights)
    np.testing.assert_array_equal(out, rout)
    np.testing.assert_array_equal(wout, rwout)
    assert dup.counts.tolist() == [[0, 0]] * world
    # an "expert": any deterministic change of the rows
    expert = bf16(f32(out) * np.float32(0.5) + np.float32(1.0))
    y, wy, cstatus = M.combine_world(sh, M.build_dst_local(sh, dst), dup, expert, wout)
    ry, rwy = mref.ref_combine(sh, dst, expert, wout)
    assert cstatus.tolist() == [M.COMBINE_OK] * world
    np.testing.assert_array_equal(y, ry)
    np.testing.assert_array_equal(wy, rwy)


def same_up_to_nan_payload(a, b):
    """Equal bit for bit, except that two NaNs may differ in sign and payload (which of two NaN operands an addition
    returns is the adder's business: the CPU's and the GPU's differ)."""
    a, b = np.asarray(a, np.uint16), np.asarray(b, np.uint16)
    nan_a, nan_b = (a & 0x7fff) > 0x7f80, (b & 0x7fff) > 0x7f80
    return np.array_equal(nan_a, nan_b) and np.array_equal(a[~nan_a], b[~nan_b])


def test_rows_that_are_not_finite_against_reference_model(mref):
    """Infinities, the largest finite values (sums that overflow), NaNs and zeros of both signs among the rows: dispatch
    copies bits; combine's sums agree with the reference's CPU model element for element, NaNs up to their payload."""
    world, s, k, h = 2, 12, 4, 16
    rng = np.random.default_rng(404)
    sh = M.Shape(world, s, k, h, s * k + 3)
    dst = MC.random_dst(sh, rng, duplicates=False)
    special = np.array([0x7f80, 0xff80, 0x7f7f, 0xff7f, 0x7fc0, 0xffc1, 0x7f81, 0x0000, 0x8000, 0x0001, 0x3f80, 0xbf80], np.uint16)
    hidden = special[rng.integers(0, len(special), size=(world, s, h))]
    out, _, status, dup = M.dispatch_world(sh, dst, hidden, flags=M.FLAG_BUILD_DEDUP)
    rout, _ = mref.ref_dispatch(sh, dst, hidden)
    assert status.tolist() == [M.DISPATCH_OK] * world
    np.testing.assert_array_equal(out, rout)
    y, _, cstatus = M.combine_world(sh, M.build_dst_local(sh, dst), dup, out)
    ry, _ = mref.ref_combine(sh, dst, out)
    assert cstatus.tolist() == [M.COMBINE_OK] * world
    assert same_up_to_nan_payload(y, ry)
    kinds = ((y & 0x7fff) > 0x7f80).sum(), ((y & 0x7fff) == 0x7f80).sum()
    assert kinds[0] > 0 and kinds[1] > 0          # the draw does produce NaN sums (inf - inf) and infinite ones


@pytest.mark.parametrize("world,s,k,h", [(1, 6, 4, 8), (2, 5, 4, 8), (4, 4, 8, 16), (8, 2, 32, 8)])
def test_with_duplicates_against_reference_model(mref, world, s, k, h):
    rng = np.random.default_rng(world * 7 + k)
    sh = M.Shape(world, s, k, h, s * k + 4)
    dst = MC.random_dst(sh, rng, duplicates=True)
    assert (dst < 0).any()
    # small integers: every sum below is exact in bf16, so the order and place of the roundings cannot matter
    hidden = bf16(rng.integers(-3, 4, size=(world, s, h)).astype(np.float32))
    weights = rng.standard_normal((world, s * k)).astype(np.float32)
    out, wout, status, dup = M.dispatch_world(sh, dst, hidden, weights, flags=M.FLAG_BUILD_DEDUP)
    rout, rwout = mref.ref_dispatch(sh, dst, hidden, weights)
    assert status.tolist() == [M.DISPATCH_OK] * world
    np.testing.assert_array_equal(out, rout)           # the model copies a duplicate's row itself: same bytes
    np.testing.assert_array_equal(wout, rwout)
    # the same groups as the model's, whatever their order
    rplan = mref.ref_duplicate_plans(sh, dst)
    np.testing.assert_array_equal(dup.counts, rplan.counts)
    for q in range(world):
        assert MC.groups_as_sets(dup, q) == MC.groups_as_sets(rplan, q)
    y, wy, cstatus = M.combine_world(sh, M.build_dst_local(sh, dst), dup, out, wout)
    ry, rwy = mref.ref_combine(sh, dst, out, wout)
    assert cstatus.tolist() == [M.COMBINE_OK] * world
    np.testing.assert_array_equal(y, ry)
    np.testing.assert_array_equal(wy, rwy)
    # saved plan: the same rows without rebuilding; without any plan the duplicates' rows stay zero
    out2, _, _, dup2 = M.dispatch_world(sh, dst, hidden, weights, flags=0, dup=dup)
    np.testing.assert_array_equal(out2, out)
    np.testing.assert_array_equal(dup2.groups, dup.groups)
    out3, _, _, _ = M.dispatch_world(sh, dst, hidden, weights, flags=0, dup=M.DupPlan.empty(sh))
    for src in range(world):
        for route in np.nonzero(dst[src] < 0)[0]:
            _, peer, row, _ = M.decode_route(dst[src, route], sh.nvs, world)
            assert not out3[peer, row].any()


# ---- where the device kernels differ from the CPU model --------------------------------------------------------------
def test_duplicate_group_is_rounded_before_the_token_sum(mref):
    """1 + 2^-8 (+ 2^-8): the kernels round the group {1, 2^-8} to bf16 first (a tie, to even: 1), then add the third
    row and round again (a tie again: 1).  One fp32 sum with a single rounding gives 1 + 2^-7."""
    sh = M.Shape(2, 1, 3, 1, 3)
    dst = np.array([[0, -2, 3], [5, 4, 2]], np.int32)       # rank 0: rows (0,0), duplicate (0,1), (1,0)
    dup = M.DupPlan.empty(sh)
    dup.groups[0, 0] = [0, 0, 1]
    dup.loffs[0, 0] = 1
    dup.counts[0] = [1, 1]
    rows = np.zeros((2, 3, 1), np.uint16)
    rows[0, 0, 0] = bf16([1.0])[0]
    rows[0, 1, 0] = bf16([2.0 ** -8])[0]
    rows[1, 0, 0] = bf16([2.0 ** -8])[0]
    y, _, status = M.combine_world(sh, M.build_dst_local(sh, dst), dup, rows)
    assert status.tolist() == [0, 0]
    assert y[0, 0, 0] == 0x3f80
    ry, _ = mref.ref_combine(sh, dst, rows)
    assert ry[0, 0, 0] == 0x3f81


def test_plan_lists_groups_by_first_duplicate_row():
    """Two tokens of one source, both with a duplicate on rank 0; the second token's duplicate has the smaller row, so
    its group comes first (the CPU model would list the first token's group first)."""
    sh = M.Shape(1, 2, 2, 2, 4)
    dst = np.array([[0, -(3) - 1, 1, -(2) - 1]], np.int32)   # token 0: row 0 + duplicate row 3; token 1: row 1 + duplicate row 2
    hidden = np.array([[[0x3f80, 0x4000], [0x4040, 0x4080]]], np.uint16)
    out, _, status, dup = M.dispatch_world(sh, dst, hidden, flags=M.FLAG_BUILD_DEDUP)
    assert status.tolist() == [M.DISPATCH_OK]
    assert dup.counts[0].tolist() == [2, 2]
    assert dup.groups[0, :2].tolist() == [[1, 0, 1], [0, 1, 1]]
    assert dup.loffs[0, :2].tolist() == [2, 3]
    np.testing.assert_array_equal(out[0, 3], hidden[0, 0])
    np.testing.assert_array_equal(out[0, 2], hidden[0, 1])


# ---- failures -------------------------------------------------------------------------------------------------------
def test_invalid_routes_are_reported_per_rank():
    sh = M.Shape(3, 2, 2, 2, 4)
    rng = np.random.default_rng(5)
    dst = MC.random_dst(sh, rng, duplicates=False)
    hidden = np.ones((3, 2, 2), np.uint16)
    bad = dst.copy()
    bad[1, 2] = 3 * 4                                        # one past the last rank
    _, _, status, _ = M.dispatch_world(sh, bad, hidden, flags=M.FLAG_BUILD_DEDUP)
    assert status.tolist() == [M.DISPATCH_REMOTE_FAILURE_BASE + 1, M.DISPATCH_INVALID_ROUTE, M.DISPATCH_REMOTE_FAILURE_BASE + 1]
    orphan = dst.copy()
    orphan[2, 0] = -int(orphan[2, 0]) - 1                    # a duplicate with no earlier route to its rank
    _, _, status, _ = M.dispatch_world(sh, orphan, hidden, flags=M.FLAG_BUILD_DEDUP)
    assert status[2] == M.DISPATCH_INVALID_ROUTE and status[0] == M.DISPATCH_REMOTE_FAILURE_BASE + 2
    # combine: a reverse route that names a slot beyond the origin's S*K, and a duplicate equal to its primary
    dl = M.build_dst_local(sh, dst)
    good = M.DupPlan.empty(sh)
    rows = np.ones((3, 4, 2), np.uint16)
    bad_dl = dl.copy()
    bad_dl[0, 0] = 3 * 4                                     # a rank that does not exist
    _, _, status = M.combine_world(sh, bad_dl, good, rows)
    assert status[0] == M.COMBINE_INVALID_ROUTE and status[1] == M.COMBINE_REMOTE_FAILURE_BASE + 0
    self_dup = M.DupPlan.empty(sh)
    self_dup.groups[1, 0] = [2, 0, 1]
    self_dup.loffs[1, 0] = 2
    self_dup.counts[1] = [1, 1]
    _, _, status = M.combine_world(sh, dl, self_dup, rows)
    assert status[1] == M.COMBINE_INVALID_ROUTE and status[0] == M.COMBINE_REMOTE_FAILURE_BASE + 1


@pytest.mark.parametrize("world,invalid", [(5, (1, 3)), (5, (0, 4)), (4, (2,)), (6, (1, 2, 5)), (3, (0, 1, 2)), (4, ())])
def test_status_with_several_invalid_plans_follows_the_stated_rule(world, invalid):
    """Several ranks with an invalid plan at once: who is named follows the closed form of include/tilexr_moonep.h
    (dispatch: the first invalid rank upwards from one's own with wrap-around; combine: the lowest invalid rank), worked
    out in moonep_cases.status_with_invalid_plans without the oracle."""
    sh = M.Shape(world, 4, 2, 2, 8)
    rng = np.random.default_rng(world * 10 + len(invalid))
    dst = MC.random_dst(sh, rng, duplicates=False)
    hidden = np.ones((world, 4, 2), np.uint16)
    bad = dst.copy()
    for r in invalid:
        bad[r, int(rng.integers(sh.n))] = world * sh.nvs     # a rank that does not exist
    status = M.dispatch_world(sh, bad, hidden, flags=M.FLAG_BUILD_DEDUP)[2]
    assert status.tolist() == MC.status_with_invalid_plans(world, invalid, "dispatch")
    dl = M.build_dst_local(sh, dst)
    bad_dl = dl.copy()
    for r in invalid:
        used = np.flatnonzero(dl[r] >= 0)
        bad_dl[r, int(rng.choice(used))] = world * sh.nvs
    status = M.combine_world(sh, bad_dl, M.DupPlan.empty(sh), np.ones((world, sh.nvs, 2), np.uint16))[2]
    assert status.tolist() == MC.status_with_invalid_plans(world, invalid, "combine")


def test_the_stated_rule_on_hand_worked_cases():
    """The helper itself against cases worked by hand."""
    assert MC.status_with_invalid_plans(5, (1, 3), "dispatch") == [2101, 2001, 2103, 2001, 2101]
    assert MC.status_with_invalid_plans(5, (1, 3), "combine") == [3101, 3001, 3101, 3001, 3101]
    assert MC.status_with_invalid_plans(4, (0,), "dispatch") == [2001, 2100, 2100, 2100]
    assert MC.status_with_invalid_plans(3, (), "dispatch") == [2000] * 3 and MC.status_with_invalid_plans(3, (), "combine") == [0] * 3


# ---- the plan generator used by the GPU tests and the benchmark -----------------------------------------------------
@pytest.mark.parametrize("world,s,k,experts,padding", [(1, 8, 4, 8, 1), (2, 16, 2, 8, 4), (4, 12, 4, 16, 1), (8, 6, 8, 32, 8)])
def test_home_plan_is_a_consistent_plan(world, s, k, experts, padding):
    plan, ids = MC.home_plan(world, s, k, experts, padding, seed=world + k)
    nvs = plan["nvs"]
    sh = M.Shape(world, s, k, 8, nvs)
    dst = plan["dst"].numpy()
    raw = np.where(dst >= 0, dst, -dst.astype(np.int64) - 1)
    assert len(np.unique(raw)) == raw.size                                          # every route has its own row
    per_rank = experts // world
    cu = plan["cu_seqlens"].numpy()
    for src in range(world):
        for route in range(s * k):
            e = int(ids[src].reshape(-1)[route])
            peer, row = raw[src, route] // nvs, raw[src, route] % nvs
            assert peer == e // per_rank
            lo = 0 if e == 0 else int(cu[peer, e - 1])
            assert lo <= row < int(cu[peer, e])                                     # inside its expert's group
    assert (cu[:, -1] <= nvs).all() and (cu % padding == 0).all()
    # duplicates are exactly the later routes of a token to a rank it already goes to
    hidden = np.ones((world, s, 8), np.uint16)
    _, _, status, dup = M.dispatch_world(sh, dst, hidden, flags=M.FLAG_BUILD_DEDUP)
    assert status.tolist() == [M.DISPATCH_OK] * world
    assert int(dup.counts[:, 1].sum()) == int((dst < 0).sum())
