"""CPU tests of the host side of the plan-driven (MoonEP) stages: exported symbols, structure layouts and the
argument rules that are decided before anything touches a device.  No call here can reach a kernel launch."""
import ctypes as C
import os
import subprocess

import pytest

from tilexr_amd import ep, moonep as mp

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_exports_and_versions():
    lib = mp.lib()
    for name in mp.EXPORTS:
        assert hasattr(lib, name), name
    # every function the header declares is in that list
    import re
    header = open(os.path.join(ROOT, "include", "tilexr_moonep.h")).read()
    declared = set(re.findall(r"^(?:int|uint32_t|int64_t)\s+(TileXRMoonEp\w+)\(", header, flags=re.M))
    assert declared == set(mp.EXPORTS), sorted(declared ^ set(mp.EXPORTS))
    assert mp.abi_version() == 2
    for version in (1, 2):
        ret, native, stub = mp.capabilities(version)
        assert ret == 0 and native == (mp.STAGE_DISPATCH | mp.STAGE_COMBINE) and stub == 0
    assert lib.TileXRMoonEpGetCapabilitiesV1(None, None) == mp.ERR_INVALID_ARGUMENT


# sizes and offsets the reference pins for the structures the two stages use
# (tests/moonep/unit/test_tilexr_moonep_abi_layout.cpp:24-81)
LAYOUT = {
    "TileXRMoonEpTensorV1": (64, {"data": 8, "elementCount": 16, "shape": 32}),
    "TileXRMoonEpPlanV1": (120, {"n": 8, "nvS": 40, "dst": 56, "dupGroups": 88, "status": 112}),
    "TileXRMoonEpDispatchTraceV1": (40, {"buffer": 8, "iteration": 24}),
    "TileXRMoonEpDispatchArgsV1": (88, {"hiddenSh": 24, "routeWeightsNvs": 48, "registeredWorkspace": 64,
                                        "registeredWorkspaceBytes": 72, "trace": 80}),
    "TileXRMoonEpCombineArgsV1": (72, {"dstLocal": 24, "hiddenNvsh": 32}),
}


def test_header_layout_matches_the_reference_abi(tmp_path):
    """The C header itself, compiled as C and as C++."""
    lines = ['#include <stddef.h>', '#include "tilexr_moonep.h"']
    for name, (size, offsets) in LAYOUT.items():
        lines.append(f'_Static_assert(sizeof({name}) == {size}, "{name} size");')
        for field, off in offsets.items():
            lines.append(f'_Static_assert(offsetof({name}, {field}) == {off}, "{name}.{field}");')
    lines.append("int main(void) { return TILEXR_MOONEP_FLAG_BUILD_DEDUP == 1 && TILEXR_MOONEP_ERROR_NOT_SUPPORTED == -6 ? 0 : 1; }")
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines) + "\n")
    inc = os.path.join(ROOT, "include")
    subprocess.run(["gcc", "-std=c11", "-Wall", "-Werror", "-I", inc, "-c", str(src), "-o", str(tmp_path / "layout.o")], check=True)
    cxx = tmp_path / "layout.cpp"
    cxx.write_text("\n".join(l.replace("_Static_assert", "static_assert") for l in lines) + "\n")
    subprocess.run(["g++", "-std=c++17", "-Wall", "-Werror", "-I", inc, "-c", str(cxx), "-o", str(tmp_path / "layoutxx.o")], check=True)


def test_ctypes_structures_match_the_header():
    structs = {"TileXRMoonEpTensorV1": mp.TensorV1, "TileXRMoonEpPlanV1": mp.PlanV1,
               "TileXRMoonEpDispatchTraceV1": mp.DispatchTraceV1, "TileXRMoonEpDispatchArgsV1": mp.DispatchArgsV1,
               "TileXRMoonEpCombineArgsV1": mp.CombineArgsV1}
    for name, (size, offsets) in LAYOUT.items():
        assert C.sizeof(structs[name]) == size
        for field, off in offsets.items():
            assert getattr(structs[name], field).offset == off


FAKE = 0x1000   # a non-null address that is never dereferenced: every call below is rejected on the host


def _plan(n=6, r=2, e=4, b=2, nvs=8, k=2):
    return mp.plan(n, r, e, b, nvs, k, FAKE, FAKE, FAKE, FAKE, FAKE)


@pytest.fixture()
def comms():
    made = [ep.Comm(2, r) for r in range(2)]
    yield made
    for c in made:
        c.destroy()


def test_dispatch_argument_rules(comms):
    """reference: src/moonep/host/tilexr_moonep.cpp:300-320, dispatch_host.cpp:17-28, dispatch_layout.cpp:12-62 and the
    cases of tests/moonep/unit/test_tilexr_moonep_stage_layout.cpp:80-111"""
    c = comms[1]
    hid = mp.tensor(FAKE, mp.DT_BF16, (3, 17))
    out = mp.tensor(FAKE, mp.DT_BF16, (8, 17))
    wsk = mp.tensor(FAKE, mp.DT_FP32, (3, 2))
    wnv = mp.tensor(FAKE, mp.DT_FP32, (8,))
    INV, NS = mp.ERR_INVALID_ARGUMENT, mp.ERR_NOT_SUPPORTED
    assert mp.lib().TileXRMoonEpDispatchV1(None, FAKE) == INV
    assert mp.dispatch_v1(c, _plan(), hid, out, None) == INV                                   # null stream
    assert mp.dispatch_v1(None, _plan(), hid, out, FAKE) == INV
    assert mp.dispatch_v1(c, None, hid, out, FAKE) == INV
    assert mp.dispatch_v1(c, _plan(), None, out, FAKE) == INV
    assert mp.dispatch_v1(c, _plan(), hid, None, FAKE) == INV
    assert mp.dispatch_v1(c, _plan(), hid, out, FAKE, struct_size=56) == INV                   # shorter than the oldest layout
    assert mp.dispatch_v1(c, _plan(), hid, out, FAKE, registered_workspace=FAKE) == NS
    assert mp.dispatch_v1(c, _plan(), hid, out, FAKE, registered_workspace_bytes=64) == NS
    # a caller built before `trace` was added still selects the registered-workspace variant
    # (reference: tests/moonep/unit/test_tilexr_moonep_host.cpp:302-306)
    assert mp.dispatch_v1(c, _plan(), hid, out, FAKE, struct_size=80, registered_workspace=FAKE) == NS
    assert mp.dispatch_v1(c, _plan(), hid, out, FAKE, trace=mp.DispatchTraceV1()) == INV
    assert mp.dispatch_v1(c, _plan(), hid, out, FAKE, flags=mp.FLAG_ZERO_COPY) == NS
    assert mp.dispatch_v1(0xdead0, _plan(), hid, out, FAKE) == ep.ERR_NOT_INITIALIZED          # not a communicator
    assert mp.dispatch_v1(c, _plan(), hid, out, FAKE, weights_sk=wsk) == INV                   # unpaired weights
    assert mp.dispatch_v1(c, _plan(), hid, out, FAKE, weights_nvs=wnv) == INV
    assert mp.dispatch_v1(c, _plan(), hid, out, FAKE, flags=1 << 20) == INV                    # unknown flag
    assert mp.dispatch_v1(c, _plan(), hid, out, FAKE, flags=mp.FLAG_COMBINE_PUBLISH_ONLY) == INV
    # plan rules (src/moonep/common/moonep_stage_layout.h:74-99)
    for bad in (dict(r=4), dict(n=7), dict(nvs=5), dict(k=33, n=66, nvs=66), dict(e=5), dict(b=3), dict(b=0),
                dict(nvs=2 ** 30 + 1)):
        assert mp.dispatch_v1(c, _plan(**bad), hid, out, FAKE) == INV, bad
    p = _plan()
    p.dupLoffs = None
    assert mp.dispatch_v1(c, p, hid, out, FAKE) == INV
    p = _plan()
    p.abiVersion = 2
    assert mp.dispatch_v1(c, p, hid, out, FAKE) == INV
    # tensor rules
    assert mp.dispatch_v1(c, _plan(), mp.tensor(FAKE, mp.DT_FP16, (3, 17)), out, FAKE) == INV  # bf16 only
    assert mp.dispatch_v1(c, _plan(), mp.tensor(FAKE, mp.DT_BF16, (4, 17)), out, FAKE) == INV  # S from the plan
    assert mp.dispatch_v1(c, _plan(), hid, mp.tensor(FAKE, mp.DT_BF16, (8, 16)), FAKE) == INV  # same H
    assert mp.dispatch_v1(c, _plan(), hid, mp.tensor(FAKE, mp.DT_BF16, (6, 17)), FAKE) == INV  # NvS rows
    t = mp.tensor(FAKE, mp.DT_BF16, (3, 17))
    t.elementCount = 50
    assert mp.dispatch_v1(c, _plan(), t, out, FAKE) == INV
    t = mp.tensor(FAKE, mp.DT_BF16, (3, 17))
    t.shape[2] = 1                                                                             # beyond the rank: must be 0
    assert mp.dispatch_v1(c, _plan(), t, out, FAKE) == INV
    assert mp.dispatch_v1(c, _plan(), hid, out, FAKE, weights_sk=mp.tensor(FAKE, mp.DT_FP32, (3, 3)), weights_nvs=wnv) == INV
    # no magic was drawn by any rejected call
    assert c.next_magic() == 1


def test_combine_argument_rules(comms):
    """reference: combine_host.cpp:15-25, combine_layout.cpp:13-37, 101-120 and the cases of
    tests/moonep/unit/test_tilexr_moonep_stage_layout.cpp:161-199"""
    c = comms[0]
    plan = _plan(n=8, r=2, e=4, b=2, nvs=12, k=2)
    rows = mp.tensor(FAKE, mp.DT_BF16, (12, 16))
    y = mp.tensor(FAKE, mp.DT_BF16, (4, 16))
    wnv = mp.tensor(FAKE, mp.DT_FP32, (12,))
    wsk = mp.tensor(FAKE, mp.DT_FP32, (4, 2))
    INV, NS = mp.ERR_INVALID_ARGUMENT, mp.ERR_NOT_SUPPORTED
    assert mp.lib().TileXRMoonEpCombineV1(None, FAKE) == INV
    assert mp.combine_v1(c, plan, FAKE, rows, y, None) == INV
    assert mp.combine_v1(c, plan, None, rows, y, FAKE) == INV                                  # dstLocal is required
    assert mp.combine_v1(c, plan, FAKE, None, y, FAKE) == INV
    assert mp.combine_v1(c, plan, FAKE, rows, None, FAKE) == INV
    assert mp.combine_v1(c, plan, FAKE, rows, y, FAKE, struct_size=64) == INV
    assert mp.combine_v1(c, plan, FAKE, rows, y, FAKE, flags=mp.FLAG_ZERO_COPY) == NS
    for flags in (mp.FLAG_COMBINE_PUBLISH_ONLY, mp.FLAG_COMBINE_CONSUME_ONLY,
                  mp.FLAG_COMBINE_PUBLISH_ONLY | mp.FLAG_COMBINE_CONSUME_ONLY, mp.FLAG_BUILD_DEDUP):
        assert mp.combine_v1(c, plan, FAKE, rows, y, FAKE, weights_nvs=wnv, weights_sk=wsk, flags=flags) == INV
    assert mp.combine_v1(c, plan, FAKE, rows, y, FAKE, weights_nvs=wnv) == INV
    assert mp.combine_v1(c, plan, FAKE, rows, y, FAKE, weights_nvs=wnv, weights_sk=mp.tensor(FAKE, mp.DT_FP32, (4, 3))) == INV
    assert mp.combine_v1(c, _plan(n=8, r=4, e=4, b=1, nvs=12, k=2), FAKE, rows, y, FAKE) == INV   # world mismatch
    assert mp.combine_v1(c, plan, FAKE, mp.tensor(FAKE, mp.DT_BF16, (8, 16)), y, FAKE) == INV
    assert mp.combine_v1(c, plan, FAKE, rows, mp.tensor(FAKE, mp.DT_BF16, (4, 8)), FAKE) == INV
    big = _plan(n=8, r=2, e=2 ** 63 - 2, b=2, nvs=12, k=2)                                     # e + b overflows
    assert mp.combine_v1(c, big, FAKE, rows, y, FAKE) == INV
    assert c.next_magic() == 1
