"""ctypes binding of libtilexr-ep.so: the calls of include/tilexr_ep.h and include/tilexr_api.h for Python callers.

Device memory is passed as torch tensors (or None for optional arguments); `stream` is a torch.cuda.Stream (the
C ABI rejects a null stream, as the reference does, so the legacy default stream cannot be used).  Every function
returns the library's status code; `check()` turns a non-zero code into an exception.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libtilexr-ep.so")
# test- and bench-only companion (memory-system yardsticks, a stand-in expert stage): not part of the product library
PROBES_PATH = os.path.join(_HERE, "lib", "libtilexr-ep-probes.so")

# status codes (include/tilexr_types.h)
SUCCESS, ERR_NOT_INITIALIZED, ERR_MKIRT, ERR_PARA_CHECK_FAIL, ERR_INTERNAL, ERR_TIMEOUT, ERR_NOT_SUPPORT, \
    ERR_NOT_FOUND = 0, -1, -2, -3, -4, -5, -6, -7
# element types
DT_INT8, DT_FP16, DT_FP32, DT_BF16, DT_FP8E4M3, DT_FP8E5M2, DT_RESERVED = 0, 3, 4, 11, 15, 16, 255
# masks / quant modes
MASK_NONE, MASK_TOKEN, MASK_EXPERT = 0, 1, 2
Q_NONE, Q_STATIC_INT8, Q_TOKEN_INT8, Q_COMM_E5M2, Q_MXFP8, Q_FP8_BLOCK128 = 0, 1, 2, 3, 4, 5

EXPORTS = (
    "TileXRMoeEpDispatch", "TileXRMoeEpDispatchV2", "TileXRMoeEpDispatchMemory", "TileXRMoeEpDispatchMemoryV2",
    "TileXRMoeEpCombine", "TileXRMoeEpCombineV2", "TileXRMoeEpCombineMemory", "TileXRMoeEpCombineMemoryV2",
    "TileXRMoeEpDispatchMemoryEx", "TileXRMoeEpCombineMemoryEx", "TileXRMoeEpDispatchMemoryNoAlloc", "TileXREpVersion", "TileXREpSetKernelTimingEvents",
    "TileXREpLastKernelName", "TileXREpSetDebugOptions",
    "TileXRCommInitRankLocal", "TileXRCommDestroy", "TileXRGetCommArgsHost", "TileXRGetCommArgsDev",
    "TileXRCommNextMagic",
)


class EpError(RuntimeError):
    def __init__(self, code, what):
        super().__init__(f"{what} returned {code}")
        self.code = code


def check(code, what="tilexr-ep call"):
    if code != SUCCESS:
        raise EpError(code, what)
    return code


class DispatchExOptions(C.Structure):
    _fields_ = [
        ("quantMode", C.c_int64), ("expertCapacity", C.c_int64), ("expertTokenNumsType", C.c_int64),
        ("activeMaskType", C.c_int64), ("xActiveMask", C.c_void_p), ("rowIndexMapOut", C.c_void_p),
        ("tileFlagsOut", C.c_void_p), ("tileRows", C.c_int64), ("epochOut", C.POINTER(C.c_int64)),
        ("metaReadyEvent", C.c_void_p),
    ]


class CombineExOptions(C.Structure):
    _fields_ = [
        ("commQuantMode", C.c_int64), ("expertOutQuantMode", C.c_int64), ("expertOutScales", C.c_void_p),
        ("expertScales", C.c_void_p), ("activeMaskType", C.c_int64), ("xActiveMask", C.c_void_p),
        ("sharedExpertX", C.c_void_p), ("rowIndexMap", C.c_void_p), ("tileFlags", C.c_void_p),
        ("tileRows", C.c_int64), ("flagEpoch", C.c_int64), ("waitTimeoutUs", C.c_int64),
        ("deviceStatusOut", C.c_void_p),
    ]


_lib = None


def lib():
    """Loads the library once.  Raises if it has not been built: there is no other implementation to fall back to."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(f"{LIB_PATH} is missing: build it with `make -C tilexr_amd/csrc` "
                              "(or __graft_entry__.build())")
        _lib = C.CDLL(LIB_PATH)
        i64, vp, i32 = C.c_int64, C.c_void_p, C.c_int
        _lib.TileXREpVersion.restype = C.c_char_p
        _lib.TileXREpLastKernelName.restype = C.c_char_p
        _lib.TileXREpLastKernelName.argtypes = [C.c_void_p, C.c_int]
        _lib.TileXRCommInitRankLocal.argtypes = [i32, i32, C.POINTER(vp)]
        _lib.TileXRCommDestroy.argtypes = [vp]
        _lib.TileXRCommNextMagic.argtypes = [vp, C.POINTER(i64)]
        _lib.TileXRGetCommArgsHost.argtypes = [vp, C.POINTER(vp)]
        _lib.TileXRGetCommArgsDev.argtypes = [vp, C.POINTER(vp)]
        simple_dispatch = [vp, vp, vp, i64, i64, i64, i64, vp, vp, vp, vp, i32, vp]
        _lib.TileXRMoeEpDispatch.argtypes = simple_dispatch
        _lib.TileXRMoeEpDispatchMemory.argtypes = simple_dispatch
        _lib.TileXRMoeEpDispatchMemoryNoAlloc.argtypes = simple_dispatch
        simple_combine = [vp, vp, vp, vp, i64, i64, i64, i64, vp, i32, vp]
        _lib.TileXRMoeEpCombine.argtypes = simple_combine
        _lib.TileXRMoeEpCombineMemory.argtypes = simple_combine
        _lib.TileXRMoeEpCombineV2.argtypes = [vp, vp, vp, vp, i64, i64, i64, i64, vp, vp, i32, vp]
        _lib.TileXRMoeEpCombineMemoryV2.argtypes = ([vp] * 5 + [i64, vp, vp] + [i64] * 13 + [vp, i32, vp])
        _lib.TileXRMoeEpDispatchV2.argtypes = ([vp] * 6 + [i64] * 14 + [vp] * 8 + [i32, vp])
        _lib.TileXRMoeEpDispatchMemoryV2.argtypes = ([vp] * 4 + [i64, vp, vp] + [i64] * 14 + [vp] * 7 + [i32, i32, vp])
        _lib.TileXRMoeEpDispatchMemoryEx.argtypes = [vp, vp, vp, i64, i64, i64, i64, C.POINTER(DispatchExOptions),
                                                      vp, vp, vp, vp, vp, i32, i32, vp]
        _lib.TileXRMoeEpCombineMemoryEx.argtypes = [vp, vp, vp, vp, i64, i64, i64, i64, C.POINTER(CombineExOptions),
                                                     vp, i32, vp]
        _lib.TileXREpSetKernelTimingEvents.argtypes = [vp, i32, vp, vp]
        for name in EXPORTS:
            fn = getattr(_lib, name)
            if name not in ("TileXREpVersion", "TileXREpLastKernelName"):
                fn.restype = C.c_int
    return _lib


def version():
    return lib().TileXREpVersion().decode()


def _ptr(t):
    if t is None:
        return None
    if isinstance(t, int):
        return C.c_void_p(t)
    return C.c_void_p(t.data_ptr())


def _stream(s):
    if s is None:
        return None
    if isinstance(s, int):
        return C.c_void_p(s)
    return C.c_void_p(s.cuda_stream)


class Comm:
    """One logical rank's communicator (include/tilexr_api.h)."""

    def __init__(self, rank_size, rank):
        handle = C.c_void_p()
        check(lib().TileXRCommInitRankLocal(rank_size, rank, C.byref(handle)), "TileXRCommInitRankLocal")
        self.handle = handle
        self.rank_size = rank_size
        self.rank = rank

    def next_magic(self):
        m = C.c_int64()
        check(lib().TileXRCommNextMagic(self.handle, C.byref(m)), "TileXRCommNextMagic")
        return m.value

    def destroy(self):
        if self.handle is not None:
            check(lib().TileXRCommDestroy(self.handle), "TileXRCommDestroy")
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.destroy()


def _h(comm):
    if comm is None:
        return None
    return comm.handle if isinstance(comm, Comm) else C.c_void_p(comm)


# ---- the reference's eight entry points ------------------------------------------------------------------
def dispatch(x, expert_ids, comm, bs, h, top_k, experts, expand_x, token_nums, recv_counts, assist, dtype, stream):
    return lib().TileXRMoeEpDispatch(_ptr(x), _ptr(expert_ids), _h(comm), bs, h, top_k, experts, _ptr(expand_x),
                                     _ptr(token_nums), _ptr(recv_counts), _ptr(assist), dtype, _stream(stream))


def dispatch_memory(x, expert_ids, comm, bs, h, top_k, experts, expand_x, token_nums, send_counts, assist, dtype,
                    stream):
    return lib().TileXRMoeEpDispatchMemory(_ptr(x), _ptr(expert_ids), _h(comm), bs, h, top_k, experts,
                                           _ptr(expand_x), _ptr(token_nums), _ptr(send_counts), _ptr(assist), dtype,
                                           _stream(stream))


def dispatch_memory_no_alloc(x, expert_ids, comm, bs, h, top_k, experts, expand_x, token_nums, send_counts, assist,
                             dtype, stream):
    """TileXRMoeEpDispatchMemory with the kernels' scratch in the library's static per-GPU array: allocates nothing."""
    return lib().TileXRMoeEpDispatchMemoryNoAlloc(_ptr(x), _ptr(expert_ids), _h(comm), bs, h, top_k, experts,
                                                  _ptr(expand_x), _ptr(token_nums), _ptr(send_counts), _ptr(assist),
                                                  dtype, _stream(stream))


def dispatch_v2(x, expert_ids, comm, bs, h, top_k, experts, expand_x, assist, token_nums, recv_counts, dtype, stream,
                scales=None, active_mask=None, expert_scales=None, ep_world_size=0, ep_rank_id=0, tp_world_size=0,
                tp_rank_id=0, expert_shard_type=0, shared_expert_num=0, shared_expert_rank_num=0, quant_mode=0,
                global_bs=0, token_nums_type=1, dynamic_scales=None, tp_recv_counts=None, expand_scales=None,
                workspace=None):
    return lib().TileXRMoeEpDispatchV2(
        _ptr(x), _ptr(expert_ids), _ptr(scales), _ptr(active_mask), _ptr(expert_scales), _h(comm), bs, h, top_k,
        experts, ep_world_size, ep_rank_id, tp_world_size, tp_rank_id, expert_shard_type, shared_expert_num,
        shared_expert_rank_num, quant_mode, global_bs, token_nums_type, _ptr(expand_x), _ptr(dynamic_scales),
        _ptr(assist), _ptr(token_nums), _ptr(recv_counts), _ptr(tp_recv_counts), _ptr(expand_scales),
        _ptr(workspace), dtype, _stream(stream))


def dispatch_memory_v2(x, expert_ids, comm, bs, h, top_k, experts, expand_x, assist, token_nums, send_counts, dtype,
                       stream, scales=None, active_mask=None, active_mask_type=MASK_NONE, expert_scales=None,
                       ep_world_size=0, ep_rank_id=0, tp_world_size=1, tp_rank_id=0, expert_shard_type=0,
                       shared_expert_num=0, shared_expert_rank_num=0, quant_mode=0, global_bs=0, token_nums_type=1,
                       dynamic_scales=None, tp_recv_counts=None, expand_scales=None, expand_x_dtype=DT_RESERVED):
    return lib().TileXRMoeEpDispatchMemoryV2(
        _ptr(x), _ptr(expert_ids), _ptr(scales), _ptr(active_mask), active_mask_type, _ptr(expert_scales), _h(comm),
        bs, h, top_k, experts, ep_world_size, ep_rank_id, tp_world_size, tp_rank_id, expert_shard_type,
        shared_expert_num, shared_expert_rank_num, quant_mode, global_bs, token_nums_type, _ptr(expand_x),
        _ptr(dynamic_scales), _ptr(assist), _ptr(token_nums), _ptr(send_counts), _ptr(tp_recv_counts),
        _ptr(expand_scales), dtype, expand_x_dtype, _stream(stream))


def combine(expert_out, assist, recv_counts, comm, bs, h, top_k, experts, y, dtype, stream):
    return lib().TileXRMoeEpCombine(_ptr(expert_out), _ptr(assist), _ptr(recv_counts), _h(comm), bs, h, top_k,
                                    experts, _ptr(y), dtype, _stream(stream))


def combine_v2(expert_out, assist, recv_counts, comm, bs, h, top_k, experts, y, dtype, stream, workspace=None):
    return lib().TileXRMoeEpCombineV2(_ptr(expert_out), _ptr(assist), _ptr(recv_counts), _h(comm), bs, h, top_k,
                                      experts, _ptr(y), _ptr(workspace), dtype, _stream(stream))


def combine_memory(expert_out, assist, send_counts, comm, bs, h, top_k, experts, y, dtype, stream):
    return lib().TileXRMoeEpCombineMemory(_ptr(expert_out), _ptr(assist), _ptr(send_counts), _h(comm), bs, h, top_k,
                                          experts, _ptr(y), dtype, _stream(stream))


def combine_memory_v2(expert_out, assist, send_counts, comm, bs, h, top_k, experts, y, dtype, stream,
                      expert_scales=None, active_mask=None, active_mask_type=MASK_NONE, shared_expert_x=None,
                      ep_world_size=0, ep_rank_id=0, tp_world_size=1, tp_rank_id=0, expert_shard_type=0,
                      shared_expert_num=0, shared_expert_rank_num=0, quant_mode=0, global_bs=0):
    return lib().TileXRMoeEpCombineMemoryV2(
        _ptr(expert_out), _ptr(assist), _ptr(send_counts), _ptr(expert_scales), _ptr(active_mask), active_mask_type,
        _ptr(shared_expert_x), _h(comm), bs, h, top_k, experts, ep_world_size, ep_rank_id, tp_world_size, tp_rank_id,
        expert_shard_type, shared_expert_num, shared_expert_rank_num, quant_mode, global_bs, _ptr(y), dtype,
        _stream(stream))


# ---- additions -------------------------------------------------------------------------------------------
def dispatch_memory_ex(x, expert_ids, comm, bs, h, top_k, experts, expand_x, assist, token_nums, send_counts, dtype,
                       stream, quant_mode=0, expert_capacity=0, token_nums_type=1, active_mask=None,
                       active_mask_type=MASK_NONE, dynamic_scales=None, expand_x_dtype=None, row_index_map=None,
                       tile_flags=None, tile_rows=0, meta_ready_event=None):
    """Returns (status, epoch)."""
    epoch = C.c_int64(0)
    opt = DispatchExOptions()
    opt.quantMode = quant_mode
    opt.expertCapacity = expert_capacity
    opt.expertTokenNumsType = token_nums_type
    opt.activeMaskType = active_mask_type
    opt.xActiveMask = _ptr(active_mask)
    opt.rowIndexMapOut = _ptr(row_index_map)
    opt.tileFlagsOut = _ptr(tile_flags)
    opt.tileRows = tile_rows
    opt.epochOut = C.pointer(epoch)
    opt.metaReadyEvent = C.c_void_p(meta_ready_event) if meta_ready_event else None
    if expand_x_dtype is None:
        expand_x_dtype = {Q_NONE: dtype, Q_TOKEN_INT8: DT_INT8, Q_MXFP8: DT_FP8E4M3, Q_FP8_BLOCK128: DT_FP8E4M3}.get(
            quant_mode, dtype)
    ret = lib().TileXRMoeEpDispatchMemoryEx(_ptr(x), _ptr(expert_ids), _h(comm), bs, h, top_k, experts, C.byref(opt),
                                            _ptr(expand_x), _ptr(dynamic_scales), _ptr(assist), _ptr(token_nums),
                                            _ptr(send_counts), dtype, expand_x_dtype, _stream(stream))
    return ret, epoch.value


def combine_memory_ex(expert_out, assist, send_counts, comm, bs, h, top_k, experts, y, dtype, stream,
                      comm_quant_mode=0, expert_out_quant_mode=0, expert_out_scales=None, expert_scales=None,
                      active_mask=None, active_mask_type=MASK_NONE, shared_expert_x=None, row_index_map=None,
                      tile_flags=None, tile_rows=0, flag_epoch=0, wait_timeout_us=0, device_status=None):
    opt = CombineExOptions()
    opt.commQuantMode = comm_quant_mode
    opt.expertOutQuantMode = expert_out_quant_mode
    opt.expertOutScales = _ptr(expert_out_scales)
    opt.expertScales = _ptr(expert_scales)
    opt.activeMaskType = active_mask_type
    opt.xActiveMask = _ptr(active_mask)
    opt.sharedExpertX = _ptr(shared_expert_x)
    opt.rowIndexMap = _ptr(row_index_map)
    opt.tileFlags = _ptr(tile_flags)
    opt.tileRows = tile_rows
    opt.flagEpoch = flag_epoch
    opt.waitTimeoutUs = wait_timeout_us
    opt.deviceStatusOut = _ptr(device_status)
    return lib().TileXRMoeEpCombineMemoryEx(_ptr(expert_out), _ptr(assist), _ptr(send_counts), _h(comm), bs, h, top_k,
                                            experts, C.byref(opt), _ptr(y), dtype, _stream(stream))


K_COUNT, K_PLACE, K_SCATTER, K_INVERT, K_REDUCE = range(5)


def set_kernel_timing_events(comm, kernel, start=None, stop=None):
    return lib().TileXREpSetKernelTimingEvents(_h(comm), kernel, start.handle if start else None,
                                               stop.handle if stop else None)


PROBE_READ, PROBE_WRITE, PROBE_COPY, PROBE_FAN_OUT, PROBE_FAN_IN, PROBE_GATHER_ROWS, PROBE_GATHER_ROWS_2K_X8, \
    PROBE_GATHER_ROWS_4K_X6 = range(8)


_probes = None


def probes():
    """The probe library (csrc/ep_probe.h), loaded once; raises if it has not been built."""
    global _probes
    if _probes is None:
        if not os.path.exists(PROBES_PATH):
            raise ImportError(f"{PROBES_PATH} is missing: build it with `make -C tilexr_amd/csrc`")
        _probes = C.CDLL(PROBES_PATH)
    return _probes


def memory_probe(pattern, src, dst, nbytes, stream):
    """One launch of a kernel that does nothing but the memory traffic of `pattern` (see csrc/ep_probe.h)."""
    fn = probes().TileXREpMemoryProbe
    fn.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p]
    return fn(pattern, _ptr(src), _ptr(dst), int(nbytes), _stream(stream))


def tile_producer_probe(src, dst, rows, row_bytes, tile_flags, tile_rows, epoch, workgroups, min_tile_ns, stream,
                        stagger_ns=0):
    """A stand-in for an expert stage: copies rows src -> dst tile by tile at a set pace and publishes each tile's
    readiness word (see csrc/ep_probe.h)."""
    fn = probes().TileXREpTileProducerProbe
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int64,
                   C.c_int64, C.c_void_p]
    return fn(_ptr(src), _ptr(dst), int(rows), int(row_bytes), _ptr(tile_flags), int(tile_rows), int(epoch),
              int(workgroups), int(min_tile_ns), int(stagger_ns), _stream(stream))


class DebugOptions(C.Structure):
    _fields_ = [("phaseStamps", C.c_void_p), ("phaseStampCapacity", C.c_int64), ("poisonUnwrittenRows", C.c_int64)]


def set_debug_options(comm, phase_stamps=None, poison=False):
    """phase_stamps: int64 / uint64 device tensor [capacity, 4] or None; poison: fill the rows a dispatch may write with
    0x7f bytes first.  Both off: clears the options."""
    fn = lib().TileXREpSetDebugOptions
    fn.argtypes = [C.c_void_p, C.POINTER(DebugOptions)]
    if phase_stamps is None and not poison:
        return fn(_h(comm), None)
    opt = DebugOptions(None if phase_stamps is None else phase_stamps.data_ptr(),
                       0 if phase_stamps is None else phase_stamps.shape[0], 1 if poison else 0)
    return fn(_h(comm), C.byref(opt))


def last_kernel_name(comm, kernel):
    name = lib().TileXREpLastKernelName(_h(comm), kernel)
    return name.decode() if name else None


# ---- HIP events for the dispatch/combine overlap (hipEvent_t handles usable with the C ABI) ---------------
_hip = None


def _hiprt():
    global _hip
    if _hip is None:
        _hip = C.CDLL("libamdhip64.so")
        _hip.hipEventCreateWithFlags.argtypes = [C.POINTER(C.c_void_p), C.c_uint]
        _hip.hipEventDestroy.argtypes = [C.c_void_p]
        _hip.hipStreamWaitEvent.argtypes = [C.c_void_p, C.c_void_p, C.c_uint]
        _hip.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        _hip.hipEventSynchronize.argtypes = [C.c_void_p]
        _hip.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
    return _hip


class HipEvent:
    def __init__(self, timing=False):
        self.handle = C.c_void_p()
        flags = 0 if timing else 0x2   # hipEventDisableTiming
        if _hiprt().hipEventCreateWithFlags(C.byref(self.handle), flags) != 0:
            raise RuntimeError("hipEventCreateWithFlags failed")

    @property
    def value(self):
        return self.handle.value

    def record(self, stream):
        if _hiprt().hipEventRecord(self.handle, _stream(stream)) != 0:
            raise RuntimeError("hipEventRecord failed")

    def synchronize(self):
        if _hiprt().hipEventSynchronize(self.handle) != 0:
            raise RuntimeError("hipEventSynchronize failed")

    def elapsed_ms(self, end):
        ms = C.c_float()
        if _hiprt().hipEventElapsedTime(C.byref(ms), self.handle, end.handle) != 0:
            raise RuntimeError("hipEventElapsedTime failed")
        return ms.value

    def wait_on(self, stream):
        """Makes `stream` wait for this event."""
        if _hiprt().hipStreamWaitEvent(_stream(stream), self.handle, 0) != 0:
            raise RuntimeError("hipStreamWaitEvent failed")

    def destroy(self):
        if self.handle:
            _hiprt().hipEventDestroy(self.handle)
            self.handle = C.c_void_p()
