"""numpy-facing bindings of the C oracle (libtilexr_ep_oracle.so).  Test infrastructure only."""
import ctypes as C
import os
import subprocess
from dataclasses import dataclass

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libtilexr_ep_oracle.so")

DT_INT8, DT_FP16, DT_BF16, DT_FP8E4M3, DT_FP8E5M2 = 0, 3, 11, 15, 16
Q_NONE, Q_STATIC_INT8, Q_TOKEN_INT8, Q_COMM_E5M2, Q_MXFP8, Q_FP8_BLOCK128 = 0, 1, 2, 3, 4, 5
MASK_NONE, MASK_TOKEN, MASK_EXPERT = 0, 1, 2


class _Case(C.Structure):
    _fields_ = [
        ("rank_size", C.c_int32),
        ("bs", C.c_int64),
        ("h", C.c_int64),
        ("top_k", C.c_int64),
        ("moe_expert_num", C.c_int64),
        ("dtype", C.c_int32),
        ("quant_mode", C.c_int32),
        ("out_dtype", C.c_int32),
        ("token_nums_type", C.c_int32),
        ("mask_type", C.c_int32),
        ("capacity", C.c_int64),
        ("shared_expert_num", C.c_int64),
        ("shared_expert_rank_num", C.c_int64),
        ("tp_world_size", C.c_int64),
    ]


@dataclass
class Case:
    rank_size: int
    bs: int
    h: int
    top_k: int
    moe_expert_num: int
    dtype: int = DT_BF16
    quant_mode: int = Q_NONE
    out_dtype: int = DT_FP8E4M3
    token_nums_type: int = 1
    mask_type: int = MASK_NONE
    capacity: int = 0
    shared_expert_num: int = 0
    shared_expert_rank_num: int = 0
    tp_world_size: int = 0

    def c(self):
        return _Case(self.rank_size, self.bs, self.h, self.top_k, self.moe_expert_num, self.dtype,
                     self.quant_mode, self.out_dtype, self.token_nums_type, self.mask_type, self.capacity,
                     self.shared_expert_num, self.shared_expert_rank_num, self.tp_world_size)

    @property
    def local_experts(self):
        return self.moe_expert_num // (self.rank_size // max(self.tp_world_size, 1) - self.shared_expert_rank_num)

    def out_local_experts(self, rank):
        return 1 if rank < self.shared_expert_rank_num else self.local_experts

    @property
    def max_rows(self):
        return self.rank_size * self.bs * (self.top_k + self.shared_expert_num)     # tp lanes included

    @property
    def out_row_bytes(self):
        return self.h * 2 if self.quant_mode == Q_NONE else self.h

    def scales_per_row(self):
        if self.quant_mode == Q_MXFP8:
            return mxfp8_scale_count(self.h)  # bytes
        if self.quant_mode == Q_FP8_BLOCK128:
            return (self.h + 127) // 128      # floats
        if self.quant_mode in (Q_TOKEN_INT8,):
            return 1                          # floats
        return 0


def build():
    subprocess.run(["make", "-s", "-C", _HERE, "oracle"], check=True)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = C.CDLL(_SO)
        _lib.orc_half_to_float.restype = C.c_float
        _lib.orc_half_to_float.argtypes = [C.c_uint16]
        _lib.orc_bf16_to_float.restype = C.c_float
        _lib.orc_bf16_to_float.argtypes = [C.c_uint16]
        for name in ("orc_float_to_half_rne_sat", "orc_float_to_half_rne", "orc_float_to_bf16_rne"):
            getattr(_lib, name).restype = C.c_uint16
            getattr(_lib, name).argtypes = [C.c_float]
        _lib.orc_clamp_int8.restype = C.c_int8
        _lib.orc_clamp_int8.argtypes = [C.c_float]
        _lib.orc_fp8_encode.restype = C.c_uint8
        _lib.orc_fp8_encode.argtypes = [C.c_float, C.c_int32]
        _lib.orc_fp8_decode.restype = C.c_float
        _lib.orc_fp8_decode.argtypes = [C.c_uint8, C.c_int32]
        _lib.orc_mxfp8_scale_count.restype = C.c_int64
        _lib.orc_mxfp8_scale_count.argtypes = [C.c_int64]
        _lib.orc_quant_row_token_int8.restype = C.c_float
        _lib.orc_quant_row_token_int8.argtypes = [C.c_void_p, C.c_int64, C.c_int32, C.c_void_p]
        _lib.orc_quant_row_static_int8.restype = None
        _lib.orc_quant_row_static_int8.argtypes = [C.c_void_p, C.c_int64, C.c_float, C.c_void_p]
        _lib.orc_quant_row_mxfp8.restype = None
        _lib.orc_quant_row_mxfp8.argtypes = [C.c_void_p, C.c_int64, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p]
        _lib.orc_quant_row_fp8_block128.restype = None
        _lib.orc_quant_row_fp8_block128.argtypes = [C.c_void_p, C.c_int64, C.c_int32, C.c_void_p, C.c_void_p]
        _lib.orc_mvp_dispatch_rank.restype = C.c_int64
        _lib.orc_mvp_dispatch_rank.argtypes = [C.POINTER(_Case), C.c_int32] + [C.c_void_p] * 10
        _lib.orc_mem_dispatch_rank.restype = C.c_int64
        _lib.orc_mem_dispatch_rank.argtypes = [C.POINTER(_Case), C.c_int32] + [C.c_void_p] * 8
        _lib.orc_mvp_combine_rank.restype = None
        _lib.orc_mvp_combine_rank.argtypes = [C.POINTER(_Case), C.c_int32, C.c_int64] + [C.c_void_p] * 4
        _lib.orc_mem_combine_rank.restype = None
        _lib.orc_mem_combine_rank.argtypes = ([C.POINTER(_Case), C.c_int32, C.c_int64] + [C.c_void_p] * 6 +
                                              [C.c_int32, C.c_int32, C.c_void_p, C.c_void_p])
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dtype):
    return None if a is None else np.ascontiguousarray(a, dtype=dtype)


# ---- scalar helpers (vectorised through python loops only for small inputs) ----
def half_to_float(bits):
    return lib().orc_half_to_float(int(bits))


def bf16_to_float(bits):
    return lib().orc_bf16_to_float(int(bits))


def float_to_bf16(v):
    return lib().orc_float_to_bf16_rne(float(v))


def float_to_half(v, saturate=False):
    fn = lib().orc_float_to_half_rne_sat if saturate else lib().orc_float_to_half_rne
    return fn(float(v))


def clamp_int8(v):
    return lib().orc_clamp_int8(float(v))


def fp8_encode(v, fp8_dtype=DT_FP8E4M3):
    return lib().orc_fp8_encode(float(v), fp8_dtype)


def fp8_decode(b, fp8_dtype=DT_FP8E4M3):
    return lib().orc_fp8_decode(int(b), fp8_dtype)


def mxfp8_scale_count(h):
    return int(lib().orc_mxfp8_scale_count(h))


# ---- row quantisers ----
def quant_row_token_int8(row_u16, decode_dtype):
    row = _c(row_u16, np.uint16)
    out = np.empty(row.shape[0], np.int8)
    scale = lib().orc_quant_row_token_int8(_p(row), row.shape[0], decode_dtype, _p(out))
    return out, np.float32(scale)


def quant_row_static_int8(row_u16, scale):
    row = _c(row_u16, np.uint16)
    out = np.empty(row.shape[0], np.int8)
    lib().orc_quant_row_static_int8(_p(row), row.shape[0], float(scale), _p(out))
    return out


def quant_row_mxfp8(row_u16, dtype, fp8_dtype):
    row = _c(row_u16, np.uint16)
    out = np.empty(row.shape[0], np.uint8)
    scales = np.empty(mxfp8_scale_count(row.shape[0]), np.uint8)
    lib().orc_quant_row_mxfp8(_p(row), row.shape[0], dtype, fp8_dtype, _p(out), _p(scales))
    return out, scales


def quant_row_fp8_block128(row_u16, dtype):
    row = _c(row_u16, np.uint16)
    out = np.empty(row.shape[0], np.uint8)
    scales = np.empty((row.shape[0] + 127) // 128, np.float32)
    lib().orc_quant_row_fp8_block128(_p(row), row.shape[0], dtype, _p(out), _p(scales))
    return out, scales


# ---- dispatch ----
def mvp_dispatch(case, dst_rank, x, ids, mask=None, static_scale=None, count_fill=0):
    """x [R, bs, h] u16, ids [R, bs, K] i32, mask [R, bs] u8 -> dict of this destination rank's outputs.
    `count_fill` is what the count arrays hold before the call (entries the path does not write keep it)."""
    x = _c(x, np.uint16)
    ids = _c(ids, np.int32)
    mask = _c(mask, np.uint8)
    static_scale = _c(static_scale, np.float32)
    rows = case.max_rows
    expand = np.zeros((rows, case.out_row_bytes), np.uint8)
    scales = np.zeros(rows, np.float32)
    assist = np.zeros((rows, 4), np.int32)
    recv = np.full(case.rank_size, count_fill, np.int32)
    tp_recv = np.full(case.rank_size, count_fill, np.int32)
    nums = np.zeros(case.local_experts, np.int64)
    cc = case.c()
    n = lib().orc_mvp_dispatch_rank(C.byref(cc), dst_rank, _p(x), _p(ids), _p(mask), _p(static_scale),
                                    _p(expand), _p(scales), _p(assist), _p(recv), _p(tp_recv), _p(nums))
    return dict(rows=int(n), expand_x=expand, dyn_scales=scales, assist=assist, recv_counts=recv,
                tp_recv_counts=tp_recv, expert_token_nums=nums)


def mem_dispatch(case, dst_rank, x, ids, mask=None):
    x = _c(x, np.uint16)
    ids = _c(ids, np.int32)
    mask = _c(mask, np.uint8)
    rows = case.max_rows
    expand = np.zeros((rows, case.out_row_bytes), np.uint8)
    spr = case.scales_per_row()
    if case.quant_mode == Q_MXFP8:
        scales = np.zeros((rows, spr), np.uint8)
    else:
        scales = np.zeros((rows, max(spr, 1)), np.float32)
    assist = np.zeros((rows, 4), np.int32)
    send = np.zeros(case.out_local_experts(dst_rank) * case.rank_size, np.int32)
    nums = np.zeros(case.out_local_experts(dst_rank), np.int64)
    cc = case.c()
    n = lib().orc_mem_dispatch_rank(C.byref(cc), dst_rank, _p(x), _p(ids), _p(mask), _p(expand), _p(scales),
                                    _p(assist), _p(send), _p(nums))
    return dict(rows=int(n), expand_x=expand, dyn_scales=scales, assist=assist, send_counts=send,
                expert_token_nums=nums)


# ---- combine ----
def mvp_combine(case, rank, expert_out, assist, recv_counts):
    """expert_out [R, max_rows, h] u16, assist [R, max_rows, 4], recv_counts [R, R] -> y [bs, h] u16."""
    expert_out = _c(expert_out, np.uint16)
    assist = _c(assist, np.int32)
    recv_counts = _c(recv_counts, np.int32)
    max_rows = expert_out.shape[1]
    y = np.zeros((case.bs, case.h), np.uint16)
    cc = case.c()
    lib().orc_mvp_combine_rank(C.byref(cc), rank, max_rows, _p(expert_out), _p(assist), _p(recv_counts), _p(y))
    return y


def mem_combine(case, rank, expert_out, assist, send_counts, expert_scales=None, token_mask=None,
                shared_expert_x=None, comm_quant=0, in_quant=0, in_scales=None):
    """expert_out [R, max_rows, row_bytes-as-u16-or-u8], assist [R, max_rows, 4], send_counts [R, localE*R]."""
    expert_out = np.ascontiguousarray(expert_out)
    assist = _c(assist, np.int32)
    send_counts = _c(send_counts, np.int32)
    expert_scales = _c(expert_scales, np.float32)
    token_mask = _c(token_mask, np.uint8)
    shared_expert_x = _c(shared_expert_x, np.uint16)
    in_scales = _c(in_scales, np.float32)
    max_rows = expert_out.shape[1]
    y = np.zeros((case.bs, case.h), np.uint16)
    cc = case.c()
    lib().orc_mem_combine_rank(C.byref(cc), rank, max_rows, _p(expert_out), _p(assist), _p(send_counts),
                               _p(expert_scales), _p(token_mask), _p(shared_expert_x), comm_quant, in_quant,
                               _p(in_scales), _p(y))
    return y
