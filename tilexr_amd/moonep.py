"""ctypes binding of the plan-driven (MoonEP) Dispatch / Combine entry points of libtilexr-ep.so
(include/tilexr_moonep.h) for Python callers.

The structures mirror the C header field for field.  Device memory is passed as torch tensors; `stream` is a
torch.cuda.Stream.  Functions return the library's status code.
"""
import ctypes as C

from . import ep

ABI_V1, ABI_V2 = 1, 2
FLAG_NONE, FLAG_BUILD_DEDUP, FLAG_SKIP_INTER_RANK_SYNC, FLAG_ZERO_COPY = 0, 1, 2, 4
FLAG_COMBINE_PUBLISH_ONLY, FLAG_COMBINE_CONSUME_ONLY, FLAG_RESET_STATUS = 8, 16, 32
SUCCESS, ERR_INVALID_ARGUMENT, ERR_INTERNAL, ERR_NOT_SUPPORTED = 0, -3, -4, -6
DT_INT32, DT_FP16, DT_FP32, DT_BF16 = 2, 3, 4, 11
STAGE_PLANNING, STAGE_DISPATCH, STAGE_PREFETCH_WEIGHT, STAGE_COMBINE, STAGE_REDUCE_GRAD = 1, 2, 4, 8, 16
DISPATCH_STATUS_SUCCESS, DISPATCH_STATUS_INVALID_ROUTE, DISPATCH_STATUS_REMOTE_FAILURE_BASE = 2000, 2001, 2100
COMBINE_STATUS_SUCCESS, COMBINE_STATUS_INVALID_ROUTE, COMBINE_STATUS_REMOTE_FAILURE_BASE = 0, 3001, 3100

EXPORTS = ("TileXRMoonEpGetAbiVersion", "TileXRMoonEpGetCapabilitiesV1", "TileXRMoonEpGetCapabilitiesV2",
           "TileXRMoonEpDispatchV1", "TileXRMoonEpCombineV1", "TileXRMoonEpSetCachedRowBytes")


class TensorV1(C.Structure):
    _fields_ = [("structSize", C.c_uint32), ("abiVersion", C.c_uint32), ("data", C.c_void_p),
                ("elementCount", C.c_uint64), ("dtype", C.c_uint32), ("rank", C.c_uint32), ("shape", C.c_int64 * 4)]


class PlanV1(C.Structure):
    _fields_ = [("structSize", C.c_uint32), ("abiVersion", C.c_uint32), ("n", C.c_int64), ("r", C.c_int64),
                ("e", C.c_int64), ("b", C.c_int64), ("nvS", C.c_int64), ("k", C.c_int64), ("dst", C.c_void_p),
                ("expertsToCopy", C.c_void_p), ("zeroFillRanges", C.c_void_p), ("remoteStats", C.c_void_p),
                ("dupGroups", C.c_void_p), ("dupLoffs", C.c_void_p), ("dupCounts", C.c_void_p),
                ("status", C.c_void_p)]


class DispatchTraceV1(C.Structure):
    _fields_ = [("structSize", C.c_uint32), ("abiVersion", C.c_uint32), ("buffer", C.c_void_p),
                ("bufferBytes", C.c_uint64), ("iteration", C.c_uint32), ("iterationCount", C.c_uint32),
                ("eventCapacity", C.c_uint32), ("reserved", C.c_uint32)]


class DispatchArgsV1(C.Structure):
    _fields_ = [("structSize", C.c_uint32), ("abiVersion", C.c_uint32), ("comm", C.c_void_p),
                ("plan", C.POINTER(PlanV1)), ("hiddenSh", C.POINTER(TensorV1)), ("routeWeightsSk", C.POINTER(TensorV1)),
                ("hiddenNvsh", C.POINTER(TensorV1)), ("routeWeightsNvs", C.POINTER(TensorV1)), ("flags", C.c_uint64),
                ("registeredWorkspace", C.c_void_p), ("registeredWorkspaceBytes", C.c_uint64),
                ("trace", C.POINTER(DispatchTraceV1))]


class CombineArgsV1(C.Structure):
    _fields_ = [("structSize", C.c_uint32), ("abiVersion", C.c_uint32), ("comm", C.c_void_p),
                ("plan", C.POINTER(PlanV1)), ("dstLocal", C.c_void_p), ("hiddenNvsh", C.POINTER(TensorV1)),
                ("routeWeightsNvs", C.POINTER(TensorV1)), ("hiddenSh", C.POINTER(TensorV1)),
                ("routeWeightsSk", C.POINTER(TensorV1)), ("flags", C.c_uint64)]


_bound = False


def lib():
    global _bound
    l = ep.lib()
    if not _bound:
        l.TileXRMoonEpGetAbiVersion.restype = C.c_uint32
        l.TileXRMoonEpGetAbiVersion.argtypes = []
        for name in ("TileXRMoonEpGetCapabilitiesV1", "TileXRMoonEpGetCapabilitiesV2"):
            getattr(l, name).restype = C.c_int
            getattr(l, name).argtypes = [C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]
        l.TileXRMoonEpDispatchV1.restype = C.c_int
        l.TileXRMoonEpDispatchV1.argtypes = [C.POINTER(DispatchArgsV1), C.c_void_p]
        l.TileXRMoonEpCombineV1.restype = C.c_int
        l.TileXRMoonEpCombineV1.argtypes = [C.POINTER(CombineArgsV1), C.c_void_p]
        _bound = True
    return l


def abi_version():
    return lib().TileXRMoonEpGetAbiVersion()


def set_cached_row_bytes(nbytes):
    """Bytes of token rows up to which dispatch assumes they are still in the device's memory-side cache (picks the
    scatter kernel); returns the previous value."""
    fn = lib().TileXRMoonEpSetCachedRowBytes
    fn.argtypes = [C.c_int64]
    fn.restype = C.c_int64
    return fn(int(nbytes))


def capabilities(version=1):
    native, stub = C.c_uint64(0), C.c_uint64(0)
    fn = lib().TileXRMoonEpGetCapabilitiesV1 if version == 1 else lib().TileXRMoonEpGetCapabilitiesV2
    ret = fn(C.byref(native), C.byref(stub))
    return ret, native.value, stub.value


def _addr(t):
    if t is None:
        return None
    return t if isinstance(t, int) else t.data_ptr()


def tensor(data, dtype, shape):
    """Descriptor of a device tensor; `data` is a torch tensor or a raw address."""
    t = TensorV1()
    t.structSize = C.sizeof(TensorV1)
    t.abiVersion = ABI_V1
    t.data = _addr(data)
    count = 1
    for i, d in enumerate(shape):
        t.shape[i] = d
        count *= d
    t.elementCount = count
    t.dtype = dtype
    t.rank = len(shape)
    return t


def plan(n, r, e, b, nvs, k, dst, dup_groups, dup_loffs, dup_counts, status, experts_to_copy=None, zero_fill_ranges=None,
         remote_stats=None):
    """Plan descriptor.  The three tables the two stages never read may be given as any non-null address; by default
    they point at `status`."""
    p = PlanV1()
    p.structSize = C.sizeof(PlanV1)
    p.abiVersion = ABI_V1
    p.n, p.r, p.e, p.b, p.nvS, p.k = n, r, e, b, nvs, k
    p.dst = _addr(dst)
    p.dupGroups = _addr(dup_groups)
    p.dupLoffs = _addr(dup_loffs)
    p.dupCounts = _addr(dup_counts)
    p.status = _addr(status)
    p.expertsToCopy = _addr(experts_to_copy if experts_to_copy is not None else status)
    p.zeroFillRanges = _addr(zero_fill_ranges if zero_fill_ranges is not None else status)
    p.remoteStats = _addr(remote_stats if remote_stats is not None else status)
    return p


def _tp(t):
    return None if t is None else C.pointer(t)


def dispatch_v1(comm, plan_desc, hidden_sh, hidden_nvsh, stream, weights_sk=None, weights_nvs=None, flags=0,
                struct_size=None, registered_workspace=None, registered_workspace_bytes=0, trace=None):
    """hidden_sh / hidden_nvsh / weights_* are TensorV1 descriptors (see tensor())."""
    a = DispatchArgsV1()
    a.structSize = C.sizeof(DispatchArgsV1) if struct_size is None else struct_size
    a.abiVersion = ABI_V1
    a.comm = None if comm is None else (comm.handle if isinstance(comm, ep.Comm) else comm)
    a.plan = _tp(plan_desc)
    a.hiddenSh = _tp(hidden_sh)
    a.routeWeightsSk = _tp(weights_sk)
    a.hiddenNvsh = _tp(hidden_nvsh)
    a.routeWeightsNvs = _tp(weights_nvs)
    a.flags = flags
    a.registeredWorkspace = registered_workspace
    a.registeredWorkspaceBytes = registered_workspace_bytes
    a.trace = _tp(trace)
    return lib().TileXRMoonEpDispatchV1(C.byref(a), ep._stream(stream))


def combine_v1(comm, plan_desc, dst_local, hidden_nvsh, hidden_sh, stream, weights_nvs=None, weights_sk=None, flags=0,
               struct_size=None):
    a = CombineArgsV1()
    a.structSize = C.sizeof(CombineArgsV1) if struct_size is None else struct_size
    a.abiVersion = ABI_V1
    a.comm = None if comm is None else (comm.handle if isinstance(comm, ep.Comm) else comm)
    a.plan = _tp(plan_desc)
    a.dstLocal = _addr(dst_local)
    a.hiddenNvsh = _tp(hidden_nvsh)
    a.routeWeightsNvs = _tp(weights_nvs)
    a.hiddenSh = _tp(hidden_sh)
    a.routeWeightsSk = _tp(weights_sk)
    a.flags = flags
    return lib().TileXRMoonEpCombineV1(C.byref(a), ep._stream(stream))
