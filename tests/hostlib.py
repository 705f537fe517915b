"""ctypes view of the test-only companion library libtilexr-ep-hooks.so for the CPU tests: the plain-C hooks into the
host-side rules (tilexr_amd/csrc/hooks.h) and the CPU model of the readiness-flag protocol (tilexr_amd/csrc/flag_trace.h).
It is linked from the same objects as libtilexr-ep.so, which itself exports the declared entry points only."""
import ctypes as C
import os

from tilexr_amd import ep

HOOKS_PATH = os.path.join(os.path.dirname(ep.LIB_PATH), "libtilexr-ep-hooks.so")
_hooks = None

X, EXPERT_IDS, SCALES, ACTIVE_MASK, EXPERT_SCALES, COMM, EXPAND_X, DYNAMIC_SCALES, ASSIST, TOKEN_NUMS, COUNTS, \
    TP_COUNTS, EXPAND_SCALES, WORKSPACE, STREAM = (1 << i for i in range(15))
RULE_BASIC, RULE_V2, RULE_MVP, RULE_MEMORY, RULE_MEMORY_UNCAPPED = range(5)
UDMA_FLAG = 1 << 10


class HookComm(C.Structure):
    _fields_ = [("rank", C.c_int32), ("rankSize", C.c_int32), ("localRankSize", C.c_int32),
                ("extraFlag", C.c_uint32), ("nullPeer", C.c_int32), ("hasUdma", C.c_int32),
                ("blockDim", C.c_uint32)]


_D_FIELDS = ["activeMaskType", "bs", "h", "topK", "moeExpertNum", "epWorldSize", "epRankId", "tpWorldSize",
             "tpRankId", "expertShardType", "sharedExpertNum", "sharedExpertRankNum", "quantMode", "globalBs",
             "expertTokenNumsType"]


class HookDispatch(C.Structure):
    _fields_ = [("has", C.c_uint32)] + [(f, C.c_int64) for f in _D_FIELDS] + \
               [("dtype", C.c_int32), ("expandXOutDtype", C.c_int32)]


class HookCombine(C.Structure):
    _fields_ = [("has", C.c_uint32)] + [(f, C.c_int64) for f in _D_FIELDS[:-1]] + [("dtype", C.c_int32)]


def lib():
    global _hooks
    if _hooks is None:
        if not os.path.exists(HOOKS_PATH):
            raise ImportError(f"{HOOKS_PATH} is missing: build it with `make -C tilexr_amd/csrc`")
        _hooks = C.CDLL(HOOKS_PATH)
    l = _hooks
    if not getattr(l, "_hooks_ready", False):
        i64, i32, u32, vp = C.c_int64, C.c_int, C.c_uint32, C.c_void_p
        l.TileXREpHookValidateDispatch.argtypes = [i32, C.POINTER(HookDispatch), C.POINTER(HookComm)]
        l.TileXREpHookValidateCombine.argtypes = [i32, C.POINTER(HookCombine), C.POINTER(HookComm)]
        l.TileXREpHookWindowConfig.argtypes = [i64] * 8 + [i32, i64, vp]
        l.TileXREpHookMemoryDispatchConfig.argtypes = [i64] * 9 + [i32, i32, i64, u32, vp]
        l.TileXREpHookMemoryCombineConfig.argtypes = [i64] * 9 + [i32, i64, u32, vp]
        l.TileXREpHookMemoryCountCoreNum.argtypes = [i64, i64, u32]
        l.TileXREpHookMemoryCountCoreNum.restype = u32
        l.TileXREpHookDstRank.argtypes = [C.c_int32, i64]
        l.TileXREpHookLocalExpert.argtypes = [C.c_int32, i64]
        for name in ("TileXREpHookDataTypeSize", "TileXREpHookAlignUp", "TileXREpHookUdmaOperationBytes",
                     "TileXREpHookUdmaWorkspaceBytes"):
            getattr(l, name).restype = i64
        l.TileXREpHookDataTypeSize.argtypes = [i32]
        l.TileXREpHookAlignUp.argtypes = [i64, i64]
        l.TileXREpHookUdmaOperationBytes.argtypes = [i64] * 3
        l.TileXREpHookUdmaWorkspaceBytes.argtypes = [i64] * 3
        l._hooks_ready = True
    return l


# ---- fabricated arguments in the shape of the reference's host tests --------------------------------------
# tests/ep/unit/test_tilexr_ep_host_validation.cpp:32-177
def comm(rank=0, rank_size=2, local_rank_size=None, extra=0, null_peer=-1, udma=False, block_dim=48):
    return HookComm(rank, rank_size, rank_size if local_rank_size is None else local_rank_size, extra, null_peer,
                    1 if udma else 0, block_dim)


def cross_node_comm(udma=False):
    return comm(0, 8, 4, UDMA_FLAG if udma else 0, -1, udma)


def dispatch_params(**kw):
    d = HookDispatch()
    d.has = X | EXPERT_IDS | COMM | EXPAND_X | TOKEN_NUMS | COUNTS | ASSIST | STREAM
    d.bs, d.h, d.topK, d.moeExpertNum = 4, 8, 2, 8
    d.dtype = ep.DT_FP16
    d.expandXOutDtype = ep.DT_RESERVED
    return _apply(d, kw)


def dispatch_v2_params(**kw):
    d = dispatch_params()
    d.has |= ACTIVE_MASK
    d.activeMaskType = ep.MASK_TOKEN
    d.epWorldSize, d.tpWorldSize, d.globalBs, d.expertTokenNumsType = 2, 1, 8, 1
    return _apply(d, kw)


def static_quant_params(**kw):
    d = dispatch_v2_params()
    d.has |= SCALES
    d.quantMode, d.dtype = 1, ep.DT_INT8
    return _apply(d, kw)


def token_quant_params(**kw):
    d = dispatch_v2_params()
    d.has |= DYNAMIC_SCALES
    d.quantMode, d.dtype = 2, ep.DT_INT8
    return _apply(d, kw)


def memory_mxfp8_params(**kw):
    d = dispatch_v2_params()
    d.has |= DYNAMIC_SCALES
    d.quantMode, d.expandXOutDtype = 4, ep.DT_FP8E4M3
    return _apply(d, kw)


def combine_params(**kw):
    c = HookCombine()
    c.has = X | ASSIST | COUNTS | COMM | EXPAND_X | STREAM
    c.bs, c.h, c.topK, c.moeExpertNum = 4, 8, 2, 8
    c.dtype = ep.DT_FP16
    return _apply(c, kw)


def memory_combine_mxfp8_params(quant_mode, **kw):
    c = combine_params()
    c.has |= EXPERT_SCALES
    c.quantMode, c.globalBs = quant_mode, 8
    return _apply(c, kw)


def _apply(s, kw):
    for k, v in kw.items():
        if k == "drop":
            s.has &= ~v
        elif k == "add":
            s.has |= v
        else:
            setattr(s, k, v)
    return s
