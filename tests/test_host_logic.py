"""Host side of libtilexr-ep on the CPU: exported symbols, window arithmetic, argument rules, status codes.

The expected numbers and codes are the ones the reference's own host tests hold
(tests/ep/unit/test_tilexr_ep_layout.cpp, tests/ep/unit/test_tilexr_ep_host_validation.cpp), kept as data in
tests/golden/reference_known_answers.json or in the tables below; where oracle/_ref is built, the arithmetic is also
compared with the reference's compiled functions on random shapes.  Nothing here launches a kernel.
"""
import ctypes as C
import os
import re

import numpy as np
import pytest
import torch

import hostlib as H
from tilexr_amd import ep

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    lib = ep.lib()
    declared = set()
    for header in ("tilexr_ep.h", "tilexr_api.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        declared |= set(re.findall(r"^(?:int|const char \*)\s*\*?(TileXR\w+)\(", text, flags=re.M))
    assert len(declared) == 20, sorted(declared)
    assert declared == set(ep.EXPORTS)
    for name in declared:
        assert getattr(lib, name) is not None
    assert ep.version().startswith("tilexr-ep gfx950")


def test_library_exports_nothing_but_the_declared_entry_points():
    """The dynamic symbol table of libtilexr-ep.so is exactly the functions that include/*.h declare: no C++ internals,
    no test seams (those live in the companion hooks library)."""
    import subprocess
    declared = set()
    for header in ("tilexr_ep.h", "tilexr_api.h", "tilexr_moonep.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        declared |= set(re.findall(r"^(?:int|uint32_t|int64_t|const char \*)\s*\*?(TileXR\w+)\(", text, flags=re.M))
    out = subprocess.run(["nm", "-D", "--defined-only", ep.LIB_PATH], check=True, capture_output=True, text=True).stdout
    exported = {line.split()[-1] for line in out.splitlines() if line.strip()}
    assert exported == declared, sorted(exported ^ declared)
    hooks = subprocess.run(["nm", "-D", "--defined-only", H.HOOKS_PATH], check=True, capture_output=True, text=True).stdout
    names = {line.split()[-1] for line in hooks.splitlines() if line.strip()}
    assert names and all(n.startswith(("TileXREpHook", "TileXREpTrace")) for n in names), sorted(names)
    probes = subprocess.run(["nm", "-D", "--defined-only", ep.PROBES_PATH], check=True, capture_output=True, text=True).stdout
    assert {line.split()[-1] for line in probes.splitlines() if line.strip()} == \
        {"TileXREpMemoryProbe", "TileXREpTileProducerProbe"}


# ---------------------------------------------------------------------------------------------
# arithmetic: reference known answers
# ---------------------------------------------------------------------------------------------
def _window(args, extra=0, shared=(0, 0), expert_ranks=None):
    rank_size, bs, h, top_k, experts, dtype = args
    out = (C.c_int64 * 9)()
    ret = H.lib().TileXREpHookWindowConfig(rank_size, expert_ranks or rank_size, bs, h, top_k, experts, shared[0],
                                           shared[1], dtype, extra, out)
    names = ("localExpertNum", "dtypeBytes", "maxRoutesPerSrc", "rowBytes", "payloadRowBytes",
             "payloadBytesPerSlot", "assistBytesPerSlot", "slotBytes", "totalBytes")
    return ret, dict(zip(names, out))


def _mem_dispatch(args):
    out = (C.c_int64 * 19)()
    ret = H.lib().TileXREpHookMemoryDispatchConfig(*args, out)
    from oracle.ref import MEM_DISPATCH_FIELDS
    return ret, dict(zip(MEM_DISPATCH_FIELDS, out))


def _mem_combine(args):
    out = (C.c_int64 * 10)()
    ret = H.lib().TileXREpHookMemoryCombineConfig(*args, out)
    from oracle.ref import MEM_COMBINE_FIELDS
    return ret, dict(zip(MEM_COMBINE_FIELDS, out))


def test_expert_mapping_and_dtype_sizes(known):
    lib = H.lib()
    for c in known["expert_mapping"]["cases"]:
        assert lib.TileXREpHookDstRank(c["expert"], c["local_experts"]) == c["dst"]
        assert lib.TileXREpHookLocalExpert(c["expert"], c["local_experts"]) == c["local"]
    for c in known["dtype_sizes"]["cases"]:
        assert lib.TileXREpHookDataTypeSize(c["dtype"]) == c["bytes"]


def test_window_config_known_answers(known):
    for case in known["window_config"]["ok"]:
        ret, got = _window(case["args"])
        assert ret == 0
        for k, v in case["expect"].items():
            assert got[k] == v, (case["args"], k)
    for case in known["window_config"]["rejected"]:
        ret, _ = _window(case["args"])
        assert ret == case["ret"], case["why"]
    assert H.lib().TileXREpHookWindowConfig(2, 2, 4, 8, 2, 8, 0, 0, 3, 0, None) == -3      # null out


def test_memory_config_known_answers(known):
    for c in known["memory_count_core_num"]["cases"]:
        assert H.lib().TileXREpHookMemoryCountCoreNum(*c["args"]) == c["expect"]
    for case in known["memory_dispatch_config"]["ok"]:
        ret, got = _mem_dispatch(case["args"])
        assert ret == 0, case["args"]
        for k, v in case["expect"].items():
            assert got[k] == v, (case["args"], k)
        if "expect_sum" in case:
            total = got["combineReserveBytes"] + got["rscvStatusNum"] * got["expertPerSizeOnWin"]
            assert total == case["expect_sum"]["value"]
    for case in known["memory_dispatch_config"]["rejected"]:
        assert _mem_dispatch(case["args"])[0] == case["ret"], case["why"]
    for case in known["memory_combine_config"]["ok"]:
        ret, got = _mem_combine(case["args"])
        assert ret == 0, case["args"]
        for k, v in case["expect"].items():
            assert got[k] == v, (case["args"], k)
    for case in known["memory_combine_config"]["rejected"]:
        assert _mem_combine(case["args"])[0] == case["ret"], case["why"]


def test_baseline_config_windows():
    """Window sizes of the five measured configurations under the reference's arithmetic (its 512 MiB staged window
    would reject every single-rank configuration except C2 on the MVP route; the entry points do not apply it)."""
    ret, c1 = _window((4, 128, 1024, 2, 16, 11))
    assert ret == 0 and (c1["maxRoutesPerSrc"], c1["rowBytes"], c1["slotBytes"], c1["totalBytes"]) == \
        (256, 2048, 528448, 2113856)
    ret, c2 = _window((1, 128, 7168, 8, 256, 11))
    assert ret == 0 and c2["totalBytes"] == 64 + 64 + 1024 * 14336 + 1024 * 16
    assert _window((1, 4096, 7168, 8, 256, 11))[0] == 0            # 470 MB, just under the limit
    assert _window((8, 4096, 7168, 8, 256, 11))[0] == -3
    assert _window((1, 16384, 2048, 8, 128, 11))[0] == -3
    # memory route at R = 1: only the 128-token shapes fit the reference's window halves
    assert _mem_dispatch((1, 0, 128, 7168, 8, 256, 0, 0, 128, 11, 11, 0, 48))[0] == -3
    ret, got = _mem_dispatch((4, 0, 128, 1024, 2, 16, 0, 0, 512, 11, 11, 0, 48))
    assert ret == 0 and got["hCommuSize"] == 2560
    ret, got = _mem_combine((1, 0, 4096, 7168, 8, 256, 0, 0, 4096, 11, 0, 48))
    assert ret == -3                                               # 32768 rows x 15360 B > 255 MiB half


def _rand_shapes(seed, n):
    rng = np.random.default_rng(seed)
    for _ in range(n):
        rank_size = int(rng.choice([1, 2, 4, 8, 16]))
        shared = int(rng.choice([0, 0, 0, 1, 2]))
        shared_ranks = 0 if shared == 0 else shared * int(rng.choice([1, 2]))
        moe_ranks = rank_size - shared_ranks
        if moe_ranks <= 0:
            shared, shared_ranks, moe_ranks = 0, 0, rank_size
        experts = moe_ranks * int(rng.choice([1, 2, 4, 8, 16]))
        if rng.random() < 0.1:
            experts += 1
        yield dict(rank_size=rank_size, rank=int(rng.integers(0, rank_size)), bs=int(rng.choice([1, 4, 32, 256, 4096])),
                   h=int(rng.choice([8, 33, 1024, 2048, 3584, 7168, 60000])), top_k=int(rng.choice([1, 2, 6, 8, 16])),
                   experts=experts, shared=shared, shared_ranks=shared_ranks,
                   dtype=int(rng.choice([3, 11, 11, 3, 0, 4])), block_dim=int(rng.choice([1, 2, 24, 48, 200, 201])))


def test_arithmetic_matches_compiled_reference_on_random_shapes(ref):
    n_ok = 0
    for s in _rand_shapes(7, 600):
        gbs = s["bs"] * s["rank_size"]
        for extra in (0, 4):
            a = (s["rank_size"], s["rank_size"], s["bs"], s["h"], s["top_k"], s["experts"], s["shared"],
                 s["shared_ranks"], s["dtype"], extra)
            r_ret, r_cfg = ref.window_config(*a)
            out = (C.c_int64 * 9)()
            ret = H.lib().TileXREpHookWindowConfig(*a, out)
            assert ret == r_ret, a
            if ret == 0:
                assert list(out) == list(r_cfg.values()), a
                n_ok += 1
                assert H.lib().TileXREpHookUdmaOperationBytes(r_cfg["totalBytes"], s["rank_size"], r_cfg["slotBytes"]) \
                    == ref.lib().ref_udma_operation_bytes(r_cfg["totalBytes"], s["rank_size"], r_cfg["slotBytes"])
                assert H.lib().TileXREpHookUdmaWorkspaceBytes(r_cfg["totalBytes"], s["rank_size"], r_cfg["slotBytes"]) \
                    == ref.lib().ref_udma_workspace_bytes(r_cfg["totalBytes"], s["rank_size"], r_cfg["slotBytes"])
        for quant, out_dtype in ((0, s["dtype"]), (4, 15), (4, 16), (2, 0)):
            a = (s["rank_size"], s["rank"], s["bs"], s["h"], s["top_k"], s["experts"], s["shared"], s["shared_ranks"],
                 gbs, s["dtype"], out_dtype, quant, s["block_dim"])
            r_ret, r_cfg = ref.memory_dispatch_config(*a)
            ret, cfg = _mem_dispatch(a)
            assert ret == r_ret, a
            if ret == 0:
                assert cfg == r_cfg, a
                n_ok += 1
        for quant in (0, 3, 4, 2):
            a = (s["rank_size"], s["rank"], s["bs"], s["h"], s["top_k"], s["experts"], s["shared"], s["shared_ranks"],
                 gbs, s["dtype"], quant, s["block_dim"])
            r_ret, r_cfg = ref.memory_combine_config(*a)
            ret, cfg = _mem_combine(a)
            assert ret == r_ret, a
            if ret == 0:
                assert cfg == r_cfg, a
                n_ok += 1
        assert H.lib().TileXREpHookMemoryCountCoreNum(s["experts"], s["rank_size"] * 3, s["block_dim"]) == \
            ref.lib().ref_memory_count_core_num(s["experts"], s["rank_size"] * 3, s["block_dim"])
    assert n_ok > 300


# ---------------------------------------------------------------------------------------------
# argument rules (reference: tests/ep/unit/test_tilexr_ep_host_validation.cpp:186-562)
# ---------------------------------------------------------------------------------------------
OK, NOINIT, BAD, UNSUP = 0, -1, -3, -6


def vd(rule, params, comm=None):
    return H.lib().TileXREpHookValidateDispatch(rule, C.byref(params), None if comm is None else C.byref(comm))


def vc(rule, params, comm=None):
    return H.lib().TileXREpHookValidateCombine(rule, C.byref(params), None if comm is None else C.byref(comm))


def test_basic_dispatch_rules():
    assert vd(H.RULE_BASIC, H.dispatch_params()) == OK
    for missing in (H.X, H.COMM, H.EXPERT_IDS, H.EXPAND_X, H.TOKEN_NUMS, H.COUNTS, H.ASSIST, H.STREAM):
        assert vd(H.RULE_BASIC, H.dispatch_params(drop=missing)) == BAD
    for field in ("bs", "h", "topK", "moeExpertNum"):
        assert vd(H.RULE_BASIC, H.dispatch_params(**{field: 0})) == BAD
    assert vd(H.RULE_BASIC, H.dispatch_params(dtype=ep.DT_FP32)) == BAD
    assert vd(H.RULE_BASIC, H.dispatch_params(dtype=ep.DT_BF16)) == OK


def test_dispatch_comm_rules():
    assert vd(H.RULE_MVP, H.dispatch_params(), H.comm()) == OK
    assert vd(H.RULE_MVP, H.dispatch_params(), H.comm(rank_size=0)) == BAD
    assert vd(H.RULE_MVP, H.dispatch_params(), H.comm(null_peer=1)) == NOINIT
    assert vd(H.RULE_MVP, H.dispatch_params(), H.cross_node_comm()) == NOINIT
    assert vd(H.RULE_MEMORY, H.dispatch_params(), H.cross_node_comm()) == OK
    c = H.cross_node_comm()
    c.nullPeer = 1
    assert vd(H.RULE_MEMORY, H.dispatch_params(), c) == NOINIT
    assert vd(H.RULE_MEMORY, H.dispatch_v2_params(tpWorldSize=2, epWorldSize=1, add=H.TP_COUNTS), H.comm()) == UNSUP
    assert vd(H.RULE_MEMORY, H.static_quant_params(), H.comm()) == UNSUP
    assert vd(H.RULE_MEMORY, H.memory_mxfp8_params(), H.comm()) == OK
    assert vd(H.RULE_MEMORY, H.memory_mxfp8_params(expandXOutDtype=ep.DT_FP8E5M2), H.comm()) == OK
    assert vd(H.RULE_MEMORY, H.memory_mxfp8_params(drop=H.DYNAMIC_SCALES), H.comm()) == BAD
    assert vd(H.RULE_MEMORY, H.memory_mxfp8_params(expandXOutDtype=ep.DT_INT8), H.comm()) == BAD
    shared = H.dispatch_v2_params(epWorldSize=4, globalBs=16, sharedExpertNum=1, sharedExpertRankNum=1, moeExpertNum=6)
    assert vd(H.RULE_MEMORY, shared, H.comm(rank_size=4)) == OK
    assert vd(H.RULE_MEMORY, H.dispatch_v2_params(drop=H.ACTIVE_MASK), H.comm()) == BAD
    assert vd(H.RULE_MEMORY, H.dispatch_v2_params(activeMaskType=ep.MASK_NONE), H.comm()) == BAD
    assert vd(H.RULE_MEMORY, H.dispatch_v2_params(activeMaskType=ep.MASK_EXPERT), H.comm()) == OK
    assert vd(H.RULE_MEMORY, H.dispatch_v2_params(activeMaskType=3), H.comm()) == BAD
    groups = H.dispatch_v2_params(epWorldSize=8, globalBs=32, sharedExpertNum=2, sharedExpertRankNum=4, moeExpertNum=8)
    assert vd(H.RULE_MEMORY, groups, H.comm(rank_size=8)) == OK
    groups.sharedExpertRankNum = 3
    assert vd(H.RULE_MEMORY, groups, H.comm(rank_size=8)) == BAD
    assert vd(H.RULE_MVP, H.dispatch_params(add=H.WORKSPACE), H.cross_node_comm(udma=True)) == OK
    assert vd(H.RULE_MVP, H.dispatch_params(moeExpertNum=7), H.comm()) == BAD
    # quant modes of the other route
    assert vd(H.RULE_MEMORY, H.dispatch_v2_params(quantMode=2), H.comm()) == UNSUP
    assert vd(H.RULE_MEMORY, H.dispatch_v2_params(globalBs=9), H.comm()) == BAD


def test_window_capacity_is_only_applied_when_asked():
    big = H.dispatch_params(bs=4096, h=7168, topK=8, moeExpertNum=256, dtype=ep.DT_BF16)
    one = H.comm(rank_size=1)
    assert vd(H.RULE_MEMORY, big, one) == BAD               # the reference's staged window cannot hold it
    assert vd(H.RULE_MEMORY_UNCAPPED, big, one) == OK       # rows never pass through such a window here
    bigc = H.combine_params(bs=4096, h=7168, topK=8, moeExpertNum=256, dtype=ep.DT_BF16)
    assert vc(H.RULE_MEMORY, bigc, one) == BAD
    assert vc(H.RULE_MEMORY_UNCAPPED, bigc, one) == OK
    # argument rules still hold without the capacity
    assert vd(H.RULE_MEMORY_UNCAPPED, H.dispatch_params(bs=4096, h=7168, topK=8, moeExpertNum=255), H.comm()) == BAD


def test_combine_rules():
    assert vc(H.RULE_BASIC, H.combine_params()) == OK
    for missing in (H.X, H.ASSIST, H.COUNTS, H.EXPAND_X, H.COMM, H.STREAM):
        assert vc(H.RULE_BASIC, H.combine_params(drop=missing)) == BAD
    assert vc(H.RULE_MVP, H.combine_params(), H.comm()) == OK
    assert vc(H.RULE_MVP, H.combine_params(), H.comm(null_peer=1)) == NOINIT
    assert vc(H.RULE_MVP, H.combine_params(), H.cross_node_comm()) == NOINIT
    assert vc(H.RULE_MVP, H.combine_params(), H.cross_node_comm(udma=True)) == NOINIT      # no workspace
    assert vc(H.RULE_MVP, H.combine_params(add=H.WORKSPACE), H.cross_node_comm(udma=True)) == OK
    assert vc(H.RULE_MEMORY, H.memory_combine_mxfp8_params(3), H.comm()) == OK
    assert vc(H.RULE_MEMORY, H.memory_combine_mxfp8_params(4), H.comm()) == OK
    assert vc(H.RULE_MEMORY, H.memory_combine_mxfp8_params(4, drop=H.EXPERT_SCALES), H.comm()) == BAD
    assert vc(H.RULE_MEMORY, H.memory_combine_mxfp8_params(2), H.comm()) == UNSUP
    # masks (reference: src/ep/host/ep_combine_memory_host.cpp:27-39)
    assert vc(H.RULE_MEMORY, H.combine_params(activeMaskType=ep.MASK_TOKEN, add=H.ACTIVE_MASK), H.comm()) == OK
    assert vc(H.RULE_MEMORY, H.combine_params(activeMaskType=ep.MASK_TOKEN), H.comm()) == BAD
    assert vc(H.RULE_MEMORY, H.combine_params(add=H.ACTIVE_MASK), H.comm()) == BAD
    assert vc(H.RULE_MEMORY, H.combine_params(activeMaskType=ep.MASK_EXPERT, add=H.ACTIVE_MASK), H.comm()) == UNSUP
    assert vc(H.RULE_MEMORY, H.combine_params(tpWorldSize=2), H.comm()) == UNSUP


def test_dispatch_v2_capability_rules():
    two = H.comm()
    four = H.comm(rank_size=4)
    eight = H.comm(rank_size=8)
    V = H.dispatch_v2_params
    table = [
        (V(), two, OK),
        (V(tpWorldSize=0), two, OK),
        (V(add=H.TP_COUNTS), two, OK),
        (V(expertTokenNumsType=0), two, OK),
        (V(expertTokenNumsType=2), two, UNSUP),
        (V(quantMode=1), two, BAD),                                   # static quant needs int8 output
        (H.static_quant_params(), two, OK),
        (H.static_quant_params(drop=H.SCALES), two, BAD),
        (H.token_quant_params(), two, OK),
        (H.token_quant_params(drop=H.DYNAMIC_SCALES), two, BAD),
        (H.token_quant_params(add=H.SCALES), two, BAD),
        (V(quantMode=3), two, UNSUP),
        (V(tpWorldSize=2, epWorldSize=1, add=H.TP_COUNTS), two, OK),
        (V(tpWorldSize=2, epWorldSize=1, tpRankId=2, add=H.TP_COUNTS), two, BAD),
        (V(tpWorldSize=2, epWorldSize=1), two, BAD),                  # tp needs tpRecvCounts
        (V(tpWorldSize=4, epWorldSize=1, globalBs=16, add=H.TP_COUNTS), four, OK),
        (V(sharedExpertNum=1), four, UNSUP),
        (V(epWorldSize=4, globalBs=16, sharedExpertNum=1, sharedExpertRankNum=1, moeExpertNum=6), four, OK),
        (V(epWorldSize=4, globalBs=32, tpWorldSize=2, sharedExpertNum=1, sharedExpertRankNum=1, moeExpertNum=6,
           add=H.TP_COUNTS), eight, OK),
        (V(expertShardType=1), eight, UNSUP),
        (V(epWorldSize=4), eight, BAD),
        (V(epRankId=1), two, BAD),
        (V(sharedExpertNum=-1), two, BAD),
        (V(sharedExpertNum=1, sharedExpertRankNum=2), four, UNSUP),
    ]
    for i, (params, comm, want) in enumerate(table):
        assert vd(H.RULE_V2, params, comm) == want, i


# ---------------------------------------------------------------------------------------------
# entry points without a GPU: validation order and status codes
# ---------------------------------------------------------------------------------------------
@pytest.mark.skipif(torch.cuda.is_available(), reason="fabricated pointers must never reach a real device")
def test_entry_points_reject_before_touching_a_device():
    fake = 0x1000
    with ep.Comm(1, 0) as comm:
        assert comm.next_magic() == 1 and comm.next_magic() == 2     # starts at 1 (src/comm/tilexr_comm.h:101)
        args = dict(x=fake, expert_ids=fake, comm=comm, bs=4, h=8, top_k=2, experts=8, expand_x=fake,
                    token_nums=fake, assist=fake, dtype=ep.DT_FP16, stream=fake)
        # a box without a GPU gives a communicator without peer memory: NOT_INITIALIZED after the argument checks
        assert ep.dispatch(recv_counts=fake, **args) == ep.ERR_NOT_INITIALIZED
        assert ep.dispatch_memory(send_counts=fake, **args) == ep.ERR_NOT_INITIALIZED
        bad = dict(args, x=None)
        assert ep.dispatch(recv_counts=fake, **bad) == ep.ERR_PARA_CHECK_FAIL
        assert ep.dispatch_memory(send_counts=fake, **bad) == ep.ERR_PARA_CHECK_FAIL
        assert ep.dispatch(recv_counts=fake, **dict(args, stream=None)) == ep.ERR_PARA_CHECK_FAIL
        assert ep.dispatch(recv_counts=fake, **dict(args, dtype=ep.DT_FP32)) == ep.ERR_PARA_CHECK_FAIL
        cargs = dict(expert_out=fake, assist=fake, comm=comm, bs=4, h=8, top_k=2, experts=8, y=fake,
                     dtype=ep.DT_FP16, stream=fake)
        assert ep.combine(recv_counts=fake, **cargs) == ep.ERR_NOT_INITIALIZED
        assert ep.combine_memory(send_counts=fake, **cargs) == ep.ERR_NOT_INITIALIZED
        assert ep.combine_memory(send_counts=None, **cargs) == ep.ERR_PARA_CHECK_FAIL
        # readiness flags: tile sizes are checked before anything else of the extended calls, and a combine that
        # waits on flags must be given the status word an expired wait is reported through
        ex = (fake, fake, comm, 4, 8, 2, 8, fake, fake, fake, fake, ep.DT_BF16, fake)
        for tile_rows in (0, -1, 1 << 31, 1 << 40):
            st, _ = ep.dispatch_memory_ex(*ex, tile_flags=fake, tile_rows=tile_rows)
            assert st == ep.ERR_PARA_CHECK_FAIL, tile_rows
        st, _ = ep.dispatch_memory_ex(*ex, tile_flags=fake, tile_rows=(1 << 31) - 1)
        assert st == ep.ERR_NOT_INITIALIZED
        cex = (fake, fake, fake, comm, 4, 8, 2, 8, fake, ep.DT_BF16, fake)
        for tile_rows in (0, -1, 1 << 31):
            assert ep.combine_memory_ex(*cex, tile_flags=fake, tile_rows=tile_rows, flag_epoch=1,
                                        device_status=fake) == ep.ERR_PARA_CHECK_FAIL
        assert ep.combine_memory_ex(*cex, tile_flags=fake, tile_rows=8, flag_epoch=1) == ep.ERR_PARA_CHECK_FAIL
        assert ep.combine_memory_ex(*cex, tile_flags=fake, tile_rows=8, flag_epoch=1,
                                    device_status=fake) == ep.ERR_NOT_INITIALIZED
        assert ep.combine_memory_ex(*cex, tile_flags=fake, tile_rows=8, flag_epoch=1, device_status=fake,
                                    wait_timeout_us=-5) == ep.ERR_PARA_CHECK_FAIL
        assert comm.next_magic() == 3                                 # no magic was consumed by rejected calls
    # an unknown communicator handle
    args = dict(x=fake, expert_ids=fake, comm=0xdead0, bs=4, h=8, top_k=2, experts=8, expand_x=fake,
                token_nums=fake, assist=fake, dtype=ep.DT_FP16, stream=fake)
    assert ep.dispatch(recv_counts=fake, **args) == ep.ERR_NOT_INITIALIZED
    st, _ = ep.dispatch_memory_ex(fake, fake, 0xdead0, 4, 8, 2, 8, fake, fake, fake, fake, ep.DT_BF16, fake)
    assert st == ep.ERR_NOT_INITIALIZED


def test_comm_shim_rules():
    lib = ep.lib()
    h = C.c_void_p()
    assert lib.TileXRCommInitRankLocal(0, 0, C.byref(h)) == ep.ERR_PARA_CHECK_FAIL
    assert lib.TileXRCommInitRankLocal(2, 2, C.byref(h)) == ep.ERR_PARA_CHECK_FAIL
    assert lib.TileXRCommInitRankLocal(129, 0, C.byref(h)) == ep.ERR_PARA_CHECK_FAIL
    assert lib.TileXRCommInitRankLocal(1, 0, None) == ep.ERR_PARA_CHECK_FAIL
    assert lib.TileXRCommDestroy(C.c_void_p(0x1234)) == ep.ERR_PARA_CHECK_FAIL
    a, b = ep.Comm(2, 0), ep.Comm(2, 1)          # one world
    c = ep.Comm(2, 0)                            # a second world with the same size
    host = C.c_void_p()
    assert lib.TileXRGetCommArgsHost(a.handle, C.byref(host)) == 0 and host.value
    ints = C.cast(host, C.POINTER(C.c_int))
    assert [ints[i] for i in range(4)] == [0, 0, 2, 2]          # rank, localRank, rankSize, localRankSize
    assert lib.TileXRGetCommArgsHost(b.handle, C.byref(host)) == 0
    assert C.cast(host, C.POINTER(C.c_int))[0] == 1
    assert lib.TileXRGetCommArgsHost(C.c_void_p(0x1234), C.byref(host)) == ep.ERR_NOT_INITIALIZED
    for comm in (a, b, c):
        comm.destroy()


# ---------------------------------------------------------------------------------------------
# a C++ caller built against include/ only, as the reference's demo is built against its installed headers
# ---------------------------------------------------------------------------------------------
@pytest.mark.skipif(torch.cuda.is_available(), reason="fabricated pointers must never reach a real device")
def test_cxx_caller_links_against_the_headers_and_the_library(tmp_path):
    import os
    import shutil
    import subprocess

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    gxx = shutil.which("g++")
    if gxx is None:
        pytest.skip("no host C++ compiler")
    exe = str(tmp_path / "caller")
    lib_dir = os.path.join(root, "tilexr_amd", "lib")
    # C++14 like the reference's host code; no HIP or torch header is on the include path
    subprocess.run([gxx, "-std=c++14", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(root, "include"),
                    os.path.join(root, "tests", "cxx", "caller.cpp"), "-o", exe, "-L", lib_dir, "-ltilexr-ep",
                    f"-Wl,-rpath,{lib_dir}", f"-Wl,-rpath-link,{os.environ.get('ROCM_PATH', '/opt/rocm')}/lib"], check=True)
    run = subprocess.run([exe], capture_output=True, text=True)
    assert run.returncode == 0, run.stdout + run.stderr
    assert "caller ok" in run.stdout


# ---------------------------------------------------------------------------------------------
# readiness-tile bookkeeping: the scatter kernels' counting code, run on CPU threads with random landing orders
# ---------------------------------------------------------------------------------------------
def _publish_stress(*args):
    fn = H.lib().TileXREpHookTilePublishStress
    fn.argtypes = [C.c_int] * 6 + [C.c_uint32, C.c_int]
    return fn(*args)


@pytest.mark.parametrize("rows,max_rows,tile_rows,parts", [
    (1000, 1024, 1, 1), (1000, 1024, 1, 2), (1000, 1024, 7, 1), (1000, 1024, 16, 2), (1000, 1024, 17, 2),
    (1000, 1024, 100, 2), (4096, 4096, 256, 2), (4095, 5000, 1024, 3), (0, 64, 8, 1), (5, 64, 64, 2), (33, 33, 32, 1)])
def test_tile_publication_holds_under_random_landing_orders(rows, max_rows, tile_rows, parts):
    # invariants checked inside the hook: a readiness word is stored once per dispatch and only after every part of
    # every row of its tile has landed; afterwards every word is (epoch << 32) | rows in the tile and every counter is
    # zero again, over several dispatches on the same scratch
    for seed in (1, 2, 3):
        assert _publish_stress(rows, max_rows, tile_rows, parts, 8, 6, seed, 0) == 0


def test_tile_publication_checks_catch_planted_mistakes():
    # a part reported before it has landed: some tile is published too early (one-row tiles make every report a store)
    assert _publish_stress(4096, 4096, 1, 1, 8, 4, 7, 1) == -1
    # a part reported twice: the tile's counter overshoots, so the tile is published early, twice or never
    assert _publish_stress(4096, 4096, 64, 2, 8, 4, 7, 2) in (-1, -2, -3, -4)
