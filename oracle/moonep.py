"""numpy-facing bindings of the MoonEP stage oracle (libtilexr_moonep_oracle.so) and, where it was built, of the
reference's own CPU model of the stages (oracle/_ref/libtilexr_moonep_ref.so).  Test infrastructure only."""
import ctypes as C
import os
from dataclasses import dataclass

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libtilexr_moonep_oracle.so")
_REF_SO = os.path.join(_HERE, "_ref", "libtilexr_moonep_ref.so")

FLAG_BUILD_DEDUP = 1
DISPATCH_OK, DISPATCH_INVALID_ROUTE, DISPATCH_REMOTE_FAILURE_BASE = 2000, 2001, 2100
COMBINE_OK, COMBINE_INVALID_ROUTE, COMBINE_REMOTE_FAILURE_BASE = 0, 3001, 3100


class _Shape(C.Structure):
    _fields_ = [("world", C.c_int64), ("s", C.c_int64), ("k", C.c_int64), ("h", C.c_int64), ("nvs", C.c_int64)]


@dataclass
class Shape:
    world: int
    s: int
    k: int
    h: int
    nvs: int

    @property
    def n(self):
        return self.s * self.k

    def c(self):
        return _Shape(self.world, self.s, self.k, self.h, self.nvs)


_lib = None
_ref = None


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            raise RuntimeError("oracle library missing: run `make -C oracle`")
        _lib = C.CDLL(_SO)
        i64, vp = C.c_int64, C.c_void_p
        sp = C.POINTER(_Shape)
        _lib.orc_moon_compute_nvs.argtypes = [i64] * 5 + [C.POINTER(i64)]
        _lib.orc_moon_padded_layout.argtypes = [vp, i64, i64, i64, vp, vp]
        _lib.orc_moon_decode_route.argtypes = [C.c_int32, i64, i64, C.POINTER(i64), C.POINTER(i64), C.POINTER(C.c_int32)]
        _lib.orc_moon_build_dst_local.argtypes = [sp, vp, vp]
        _lib.orc_moon_dispatch_world.argtypes = [sp, vp, vp, vp, C.c_uint64, vp, vp, vp, vp, vp, vp]
        _lib.orc_moon_combine_world.argtypes = [sp, vp, vp, vp, vp, vp, vp, vp, vp, vp]
        for f in ("orc_moon_compute_nvs", "orc_moon_padded_layout", "orc_moon_decode_route", "orc_moon_build_dst_local",
                  "orc_moon_dispatch_world", "orc_moon_combine_world"):
            getattr(_lib, f).restype = C.c_int
    return _lib


def compute_nvs(s, k, e, world, token_padding):
    out = C.c_int64(0)
    ret = lib().orc_moon_compute_nvs(s, k, e, world, token_padding, C.byref(out))
    return ret, out.value


def padded_layout(counts, token_padding, nvs):
    counts = np.ascontiguousarray(counts, np.int32)
    cu = np.zeros(len(counts), np.int32)
    ranges = np.zeros((len(counts), 2), np.int32)
    ret = lib().orc_moon_padded_layout(_p(counts), len(counts), token_padding, nvs, _p(cu), _p(ranges))
    return ret, cu, ranges


def decode_route(encoded, nvs, world):
    rank, off, dup = C.c_int64(0), C.c_int64(0), C.c_int32(0)
    ret = lib().orc_moon_decode_route(int(encoded), nvs, world, C.byref(rank), C.byref(off), C.byref(dup))
    return ret, rank.value, off.value, bool(dup.value)


def build_dst_local(sh: Shape, dst):
    dst = np.ascontiguousarray(dst, np.int32).reshape(sh.world, sh.n)
    out = np.zeros((sh.world, sh.nvs), np.int32)
    shape = sh.c()
    ret = lib().orc_moon_build_dst_local(C.byref(shape), _p(dst), _p(out))
    if ret != 0:
        raise ValueError("invalid route in dst")
    return out


@dataclass
class DupPlan:
    groups: np.ndarray   # [world, nvs, 3] int32 {primary row, first index into loffs, count}
    loffs: np.ndarray    # [world, nvs] int32
    counts: np.ndarray   # [world, 2] int32 {groups, duplicates}

    @staticmethod
    def empty(sh: Shape):
        return DupPlan(np.zeros((sh.world, sh.nvs, 3), np.int32), np.zeros((sh.world, sh.nvs), np.int32),
                       np.zeros((sh.world, 2), np.int32))

    def copy(self):
        return DupPlan(self.groups.copy(), self.loffs.copy(), self.counts.copy())


def dispatch_world(sh: Shape, dst, hidden, weights=None, flags=0, dup: DupPlan = None):
    """Returns (hidden_nvsh [world, nvs, h] uint16, weights_nvs [world, nvs] or None, status [world], dup plan)."""
    dst = np.ascontiguousarray(dst, np.int32).reshape(sh.world, sh.n)
    hidden = np.ascontiguousarray(hidden, np.uint16).reshape(sh.world, sh.s, sh.h)
    w = None if weights is None else np.ascontiguousarray(weights, np.float32).reshape(sh.world, sh.n)
    dup = DupPlan.empty(sh) if dup is None else dup.copy()
    out = np.zeros((sh.world, sh.nvs, sh.h), np.uint16)
    wout = None if w is None else np.zeros((sh.world, sh.nvs), np.float32)
    status = np.zeros(sh.world, np.int32)
    shape = sh.c()
    ret = lib().orc_moon_dispatch_world(C.byref(shape), _p(dst), _p(hidden), _p(w), flags, _p(dup.groups), _p(dup.loffs),
                                        _p(dup.counts), _p(out), _p(wout), _p(status))
    if ret != 0:
        raise RuntimeError("oracle dispatch failed")
    return out, wout, status, dup


def combine_world(sh: Shape, dst_local, dup: DupPlan, hidden_nvsh, weights_nvs=None):
    """Returns (hidden_sh [world, s, h] uint16, weights_sk [world, s, k] or None, status [world])."""
    dst_local = np.ascontiguousarray(dst_local, np.int32).reshape(sh.world, sh.nvs)
    hidden_nvsh = np.ascontiguousarray(hidden_nvsh, np.uint16).reshape(sh.world, sh.nvs, sh.h)
    w = None if weights_nvs is None else np.ascontiguousarray(weights_nvs, np.float32).reshape(sh.world, sh.nvs)
    out = np.zeros((sh.world, sh.s, sh.h), np.uint16)
    wout = None if w is None else np.zeros((sh.world, sh.s, sh.k), np.float32)
    status = np.zeros(sh.world, np.int32)
    shape = sh.c()
    ret = lib().orc_moon_combine_world(C.byref(shape), _p(dst_local), _p(dup.groups), _p(dup.loffs), _p(dup.counts),
                                       _p(hidden_nvsh), _p(w), _p(out), _p(wout), _p(status))
    if ret != 0:
        raise RuntimeError("oracle combine failed")
    return out, wout, status


# ---- the reference's own CPU model, compiled where it lies ------------------------------------------------------

def ref_available():
    return os.path.exists(_REF_SO)


def ref():
    global _ref
    if _ref is None:
        _ref = C.CDLL(_REF_SO)
        i64, vp = C.c_int64, C.c_void_p
        _ref.ref_moon_compute_nvs.argtypes = [i64] * 5 + [C.POINTER(i64)]
        _ref.ref_moon_padded_layout.argtypes = [vp, i64, i64, i64, vp, vp]
        _ref.ref_moon_decode_route.argtypes = [C.c_int32, i64, i64, C.POINTER(i64), C.POINTER(i64), C.POINTER(C.c_int32)]
        _ref.ref_moon_float_to_bf16.argtypes = [C.c_float]
        _ref.ref_moon_float_to_bf16.restype = C.c_uint16
        _ref.ref_moon_dispatch_bf16.argtypes = [i64] * 5 + [vp, vp, vp]
        _ref.ref_moon_dispatch_f32.argtypes = [i64] * 4 + [vp, vp, vp]
        _ref.ref_moon_combine_bf16.argtypes = [i64] * 5 + [vp, vp, vp]
        _ref.ref_moon_combine_f32.argtypes = [i64] * 4 + [vp, vp, vp]
        _ref.ref_moon_duplicate_plans.argtypes = [i64] * 4 + [vp, vp, vp, vp]
    return _ref


def ref_compute_nvs(s, k, e, world, token_padding):
    out = C.c_int64(0)
    ret = ref().ref_moon_compute_nvs(s, k, e, world, token_padding, C.byref(out))
    return ret, out.value


def ref_padded_layout(counts, token_padding, nvs):
    counts = np.ascontiguousarray(counts, np.int32)
    cu = np.zeros(len(counts), np.int32)
    ranges = np.zeros((len(counts), 2), np.int32)
    ret = ref().ref_moon_padded_layout(_p(counts), len(counts), token_padding, nvs, _p(cu), _p(ranges))
    return ret, cu, ranges


def ref_decode_route(encoded, capacity, world):
    rank, off, dup = C.c_int64(0), C.c_int64(0), C.c_int32(0)
    ret = ref().ref_moon_decode_route(int(encoded), capacity, world, C.byref(rank), C.byref(off), C.byref(dup))
    return ret, rank.value, off.value, bool(dup.value)


def ref_dispatch(sh: Shape, dst, hidden=None, weights=None):
    dst = np.ascontiguousarray(dst, np.int32).reshape(sh.world, sh.n)
    out = wout = None
    if hidden is not None:
        hidden = np.ascontiguousarray(hidden, np.uint16)
        out = np.zeros((sh.world, sh.nvs, sh.h), np.uint16)
        if ref().ref_moon_dispatch_bf16(sh.world, sh.s, sh.k, sh.h, sh.nvs, _p(dst), _p(hidden), _p(out)) != 0:
            raise ValueError("reference model rejected the case")
    if weights is not None:
        weights = np.ascontiguousarray(weights, np.float32)
        wout = np.zeros((sh.world, sh.nvs), np.float32)
        if ref().ref_moon_dispatch_f32(sh.world, sh.s, sh.k, sh.nvs, _p(dst), _p(weights), _p(wout)) != 0:
            raise ValueError("reference model rejected the case")
    return out, wout


def ref_combine(sh: Shape, dst, hidden_nvsh=None, weights_nvs=None):
    dst = np.ascontiguousarray(dst, np.int32).reshape(sh.world, sh.n)
    out = wout = None
    if hidden_nvsh is not None:
        hidden_nvsh = np.ascontiguousarray(hidden_nvsh, np.uint16)
        out = np.zeros((sh.world, sh.s, sh.h), np.uint16)
        if ref().ref_moon_combine_bf16(sh.world, sh.s, sh.k, sh.h, sh.nvs, _p(dst), _p(hidden_nvsh), _p(out)) != 0:
            raise ValueError("reference model rejected the case")
    if weights_nvs is not None:
        weights_nvs = np.ascontiguousarray(weights_nvs, np.float32)
        wout = np.zeros((sh.world, sh.s, sh.k), np.float32)
        if ref().ref_moon_combine_f32(sh.world, sh.s, sh.k, sh.nvs, _p(dst), _p(weights_nvs), _p(wout)) != 0:
            raise ValueError("reference model rejected the case")
    return out, wout


def ref_duplicate_plans(sh: Shape, dst):
    dst = np.ascontiguousarray(dst, np.int32).reshape(sh.world, sh.n)
    plan = DupPlan.empty(sh)
    if ref().ref_moon_duplicate_plans(sh.world, sh.s, sh.k, sh.nvs, _p(dst), _p(plan.groups), _p(plan.loffs),
                                      _p(plan.counts)) != 0:
        raise ValueError("reference model rejected the case")
    return plan
