"""Bindings of oracle/_ref/libtilexr_ep_ref.so: the reference's own host sources (layout arithmetic, MXFP8
golden model, no-NPU checker) compiled where they lie.  Test infrastructure only; `available()` is False
where the library was never built (the reference checkout does not travel)."""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_ref", "libtilexr_ep_ref.so")

_lib = None

WINDOW_FIELDS = ("localExpertNum", "dtypeBytes", "maxRoutesPerSrc", "rowBytes", "payloadRowBytes",
                 "payloadBytesPerSlot", "assistBytesPerSlot", "slotBytes", "totalBytes")
MEM_DISPATCH_FIELDS = ("localExpertNum", "rscvStatusNum", "blockDim", "aivUsedCumSum", "aivUsedAllToAll",
                       "sharedUsedAivNum", "moeUsedAivNum", "hCommuSize", "hOutSize", "scaleOutBytes",
                       "tokenQuantAlignBytes", "expertPerSizeOnWin", "combineReserveBytes", "workspaceBytes",
                       "totalWinSize", "dispatchHalfBytes", "maxSizeForUbBuffer", "totalUbSize",
                       "allToAllUbBytes")
MEM_COMBINE_FIELDS = ("moeExpertNumPerRank", "blockDim", "blockCntPerToken", "packedRowBytes",
                      "combineReserveBytes", "workspaceBytes", "totalWinSize", "combineHalfBytes",
                      "receiveUbBytes", "sendUbBytes")


def available():
    return os.path.exists(_SO)


def lib():
    global _lib
    if _lib is None:
        _lib = C.CDLL(_SO)
        i64, i32, u32, vp = C.c_int64, C.c_int, C.c_uint32, C.c_void_p
        _lib.ref_window_config.restype = i32
        _lib.ref_window_config.argtypes = [i64] * 8 + [i32, i64, vp]
        _lib.ref_udma_operation_bytes.restype = i64
        _lib.ref_udma_operation_bytes.argtypes = [i64] * 3
        _lib.ref_udma_workspace_bytes.restype = i64
        _lib.ref_udma_workspace_bytes.argtypes = [i64] * 3
        _lib.ref_memory_count_core_num.restype = u32
        _lib.ref_memory_count_core_num.argtypes = [i64, i64, u32]
        _lib.ref_memory_dispatch_config.restype = i32
        _lib.ref_memory_dispatch_config.argtypes = [i64] * 9 + [i32, i32, i64, u32, vp]
        _lib.ref_memory_combine_config.restype = i32
        _lib.ref_memory_combine_config.argtypes = [i64] * 9 + [i32, i64, u32, vp]
        _lib.ref_dst_rank.restype = i32
        _lib.ref_dst_rank.argtypes = [C.c_int32, i64]
        _lib.ref_local_expert.restype = i32
        _lib.ref_local_expert.argtypes = [C.c_int32, i64]
        _lib.ref_mxfp8_scale_count.restype = i64
        _lib.ref_mxfp8_scale_count.argtypes = [i64]
        _lib.ref_mxfp8_quant_row.restype = None
        _lib.ref_mxfp8_quant_row.argtypes = [vp, i64, i32, vp, vp]
        _lib.ref_fp8_encode.restype = C.c_uint8
        _lib.ref_fp8_encode.argtypes = [C.c_float, i32]
        _lib.ref_fp8_decode.restype = C.c_float
        _lib.ref_fp8_decode.argtypes = [C.c_uint8, i32]
        _lib.ref_checker_default_ids.restype = i64
        _lib.ref_checker_default_ids.argtypes = [i32, i64, i64, i64, vp]
        _lib.ref_checker_routes.restype = i64
        _lib.ref_checker_routes.argtypes = [i32, i64, i64, i64, vp, i32, vp]
        _lib.ref_checker_input_value.restype = C.c_uint16
        _lib.ref_checker_input_value.argtypes = [i32, i64, i64]
        _lib.ref_checker_output_bytes.restype = i64
        _lib.ref_checker_output_bytes.argtypes = [i32, i32, i64, i64, i64, i64, i32]
        _lib.ref_checker_run.restype = i32
        _lib.ref_checker_run.argtypes = [i32, i32, i64, i64, i64, i64, i32, vp, vp]
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def window_config(rank_size, expert_rank_size, bs, h, top_k, experts, shared_num, shared_rank_num, dtype,
                  payload_extra=0):
    out = np.zeros(len(WINDOW_FIELDS), np.int64)
    ret = lib().ref_window_config(rank_size, expert_rank_size, bs, h, top_k, experts, shared_num, shared_rank_num,
                                  dtype, payload_extra, _p(out))
    return ret, dict(zip(WINDOW_FIELDS, (int(v) for v in out)))


def memory_dispatch_config(rank_size, rank, bs, h, top_k, experts, shared_num, shared_rank_num, global_bs, dtype,
                           out_dtype, quant_mode, block_dim):
    out = np.zeros(len(MEM_DISPATCH_FIELDS), np.int64)
    ret = lib().ref_memory_dispatch_config(rank_size, rank, bs, h, top_k, experts, shared_num, shared_rank_num,
                                           global_bs, dtype, out_dtype, quant_mode, block_dim, _p(out))
    return ret, dict(zip(MEM_DISPATCH_FIELDS, (int(v) for v in out)))


def memory_combine_config(rank_size, rank, bs, h, top_k, experts, shared_num, shared_rank_num, global_bs, dtype,
                          quant_mode, block_dim):
    out = np.zeros(len(MEM_COMBINE_FIELDS), np.int64)
    ret = lib().ref_memory_combine_config(rank_size, rank, bs, h, top_k, experts, shared_num, shared_rank_num,
                                          global_bs, dtype, quant_mode, block_dim, _p(out))
    return ret, dict(zip(MEM_COMBINE_FIELDS, (int(v) for v in out)))


def mxfp8_quant_row(row_f32, e5m2):
    row = np.ascontiguousarray(row_f32, np.float32)
    h = row.shape[0]
    elements = np.zeros(h, np.uint8)
    scales = np.zeros(int(lib().ref_mxfp8_scale_count(h)), np.uint8)
    lib().ref_mxfp8_quant_row(_p(row), h, int(e5m2), _p(elements), _p(scales))
    return elements, scales


def checker_default_ids(rank_size, bs, top_k, experts):
    out = np.zeros(bs * top_k, np.int32)
    n = lib().ref_checker_default_ids(rank_size, bs, top_k, experts, _p(out))
    return out[:n].reshape(bs, top_k)


def checker_routes(rank_size, bs, top_k, experts, ids, dst_rank):
    ids = np.ascontiguousarray(ids, np.int32)
    n = lib().ref_checker_routes(rank_size, bs, top_k, experts, _p(ids), dst_rank, None)
    out = np.zeros((max(n, 1), 4), np.int32)
    lib().ref_checker_routes(rank_size, bs, top_k, experts, _p(ids), dst_rank, _p(out))
    return out[:n]


def checker_run(op, rank_size, bs, h, top_k, experts, dtype):
    """op 0 = ep_dispatch, 1 = ep_combine.  Returns (status, blobs[rank, bytes], event_count)."""
    nbytes = int(lib().ref_checker_output_bytes(op, rank_size, bs, h, top_k, experts, dtype))
    out = np.zeros((rank_size, nbytes), np.uint8)
    events = C.c_int64(0)
    st = lib().ref_checker_run(op, rank_size, bs, h, top_k, experts, dtype, _p(out), C.byref(events))
    return st, out, events.value
