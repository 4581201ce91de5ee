"""ctypes view of the C ABI in include/moe_gfx950.h (libmoe_gfx950.so).

This is the torch-free way into the kernels: raw device pointers, sizes and a HIP
stream handle.  `cinfer_ascendc` (the drop-in module with the reference's Python
API) sits on the same ABI.  There is no CPU fallback: if the library has not been
built, importing this module raises.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmoe_gfx950.so")

MOE_OK = 0
EPILOGUE_NONE, EPILOGUE_SWIGLU = 0, 1
FMT_FP4_REF, FMT_FP8_REF, FMT_INT8, FMT_INT4, FMT_FP4_B32, FMT_BF16, FMT_FP4_B16 = range(7)
ERR_NULL_POINTER, ERR_BAD_FORMAT, ERR_BAD_SHAPE, ERR_BAD_ALIGNMENT, ERR_TOO_LARGE, ERR_LAUNCH, ERR_NO_DEVICE = (
    -1, -2, -3, -4, -5, -6, -7)

# every symbol include/moe_gfx950.h declares
SYMBOLS = (
    "moe_abi_version", "moe_strerror", "moe_format_from_compute_type",
    "moe_dequant_fp4_bf16_validate", "moe_grouped_gemm_validate", "moe_grouped_gemv_validate",
    "moe_dequant_fp4_bf16_workspace_bytes", "moe_grouped_gemm_workspace_bytes", "moe_grouped_gemv_workspace_bytes",
    "moe_dequant_fp4_bf16", "moe_grouped_gemm", "moe_grouped_gemv",
    "moe_prepack_fp4_ref_validate", "moe_prepack_fp4_ref_workspace_bytes", "moe_prepack_fp4_ref",
    "moe_route_validate", "moe_route_workspace_bytes", "moe_route", "moe_route_static", "moe_test_shift_launch_number",
)


class GroupedArgs(ctypes.Structure):
    _fields_ = [("x", ctypes.c_void_p), ("weight", ctypes.c_void_p), ("scale", ctypes.c_void_p),
                ("offset", ctypes.c_void_p), ("group_list", ctypes.c_void_p), ("y", ctypes.c_void_p),
                ("M", ctypes.c_int64), ("K", ctypes.c_int64), ("N", ctypes.c_int64), ("G", ctypes.c_int64),
                ("scale_rows", ctypes.c_int64), ("format", ctypes.c_int32), ("epilogue", ctypes.c_int32)]


class DequantArgs(ctypes.Structure):
    _fields_ = [("codes", ctypes.c_void_p), ("scale", ctypes.c_void_p), ("out", ctypes.c_void_p),
                ("rows", ctypes.c_int64), ("cols", ctypes.c_int64), ("block", ctypes.c_int32),
                ("reserved", ctypes.c_int32)]


class PrepackFp4Args(ctypes.Structure):
    _fields_ = [("codes", ctypes.c_void_p), ("scale", ctypes.c_void_p), ("scale2", ctypes.c_void_p),
                ("weight_out", ctypes.c_void_p), ("scale_out", ctypes.c_void_p),
                ("G", ctypes.c_int64), ("N", ctypes.c_int64), ("K", ctypes.c_int64),
                ("scale2_cols", ctypes.c_int32), ("reserved", ctypes.c_int32)]


class RouteArgs(ctypes.Structure):
    _fields_ = [("logits", ctypes.c_void_p), ("x", ctypes.c_void_p), ("topk_ids", ctypes.c_void_p),
                ("topk_weight", ctypes.c_void_p), ("group_list", ctypes.c_void_p), ("row_token", ctypes.c_void_p),
                ("row_of_choice", ctypes.c_void_p), ("x_sorted", ctypes.c_void_p), ("workspace", ctypes.c_void_p),
                ("T", ctypes.c_int64), ("E", ctypes.c_int64), ("K", ctypes.c_int64),
                ("topk", ctypes.c_int32), ("reserved", ctypes.c_int32)]


if not os.path.exists(LIB_PATH):
    raise ImportError(f"{LIB_PATH} is missing: build it with `python ascend-kernel_amd/build.py` "
                      "(there is no CPU fallback)")

lib = ctypes.CDLL(LIB_PATH)
lib.moe_abi_version.restype = ctypes.c_int
lib.moe_strerror.restype = ctypes.c_char_p
lib.moe_strerror.argtypes = [ctypes.c_int]
lib.moe_format_from_compute_type.restype = ctypes.c_int
lib.moe_format_from_compute_type.argtypes = [ctypes.c_char_p]
for _n, _t in (("dequant_fp4_bf16", DequantArgs), ("grouped_gemm", GroupedArgs), ("grouped_gemv", GroupedArgs),
               ("prepack_fp4_ref", PrepackFp4Args), ("route", RouteArgs)):
    getattr(lib, f"moe_{_n}_validate").restype = ctypes.c_int
    getattr(lib, f"moe_{_n}_validate").argtypes = [ctypes.POINTER(_t)]
    getattr(lib, f"moe_{_n}_workspace_bytes").restype = ctypes.c_size_t
    getattr(lib, f"moe_{_n}_workspace_bytes").argtypes = [ctypes.POINTER(_t)]
    getattr(lib, f"moe_{_n}").restype = ctypes.c_int
    getattr(lib, f"moe_{_n}").argtypes = [ctypes.POINTER(_t), ctypes.c_void_p]


lib.moe_route_static.restype = ctypes.c_int
lib.moe_test_shift_launch_number.restype = ctypes.c_int64
lib.moe_test_shift_launch_number.argtypes = [ctypes.c_int64]
lib.moe_route_static.argtypes = [ctypes.POINTER(RouteArgs), ctypes.c_void_p]
ROUTE_STATIC_SCRATCH_BYTES = 2 << 20


class MoeError(RuntimeError):
    def __init__(self, status: int, op: str):
        self.status = status
        super().__init__(f"{op}: {strerror(status)} (moe_status {status})")


def strerror(status: int) -> str:
    return lib.moe_strerror(status).decode()


def format_from_compute_type(name: str) -> int:
    return lib.moe_format_from_compute_type(name.encode())


def _check(rc: int, op: str) -> None:
    if rc != MOE_OK:
        raise MoeError(rc, op)


def dequant_fp4_bf16(codes_ptr: int, scale_ptr: int, out_ptr: int, rows: int, cols: int, block: int = 32,
                     stream: int = 0) -> None:
    a = DequantArgs(codes_ptr, scale_ptr, out_ptr, rows, cols, block, 0)
    _check(lib.moe_dequant_fp4_bf16(ctypes.byref(a), ctypes.c_void_p(stream)), "moe_dequant_fp4_bf16")


def grouped_args(fmt: int, x_ptr: int, w_ptr: int, scale_ptr, offset_ptr, gl_ptr: int, y_ptr: int, M: int, K: int,
                 N: int, G: int, scale_rows: int = 1, epilogue: int = EPILOGUE_NONE) -> GroupedArgs:
    return GroupedArgs(x_ptr, w_ptr, scale_ptr or None, offset_ptr or None, gl_ptr, y_ptr, M, K, N, G, scale_rows,
                       fmt, epilogue)


def grouped_gemm(args: GroupedArgs, stream: int = 0) -> None:
    _check(lib.moe_grouped_gemm(ctypes.byref(args), ctypes.c_void_p(stream)), "moe_grouped_gemm")


def grouped_gemv(args: GroupedArgs, stream: int = 0) -> None:
    _check(lib.moe_grouped_gemv(ctypes.byref(args), ctypes.c_void_p(stream)), "moe_grouped_gemv")


def prepack_fp4_ref(codes_ptr, scale_ptr, scale2_ptr, weight_out_ptr, scale_out_ptr, G: int, N: int, K: int,
                    scale2_cols: int = 0, stream: int = 0) -> None:
    """Checkpoint codes [G,N,K/2] / scales [G,N,K/16] -> the "fp4" container [G,K,N/2] / [G,K/16,N]."""
    a = PrepackFp4Args(codes_ptr or None, scale_ptr or None, scale2_ptr or None, weight_out_ptr or None,
                       scale_out_ptr or None, G, N, K, scale2_cols, 0)
    _check(lib.moe_prepack_fp4_ref(ctypes.byref(a), ctypes.c_void_p(stream)), "moe_prepack_fp4_ref")


def route_args(logits_ptr, x_ptr, topk_ids_ptr, topk_weight_ptr, group_list_ptr, row_token_ptr, row_of_choice_ptr,
               x_sorted_ptr, workspace_ptr, T: int, E: int, K: int, topk: int) -> RouteArgs:
    n = lambda p: p or None
    return RouteArgs(n(logits_ptr), n(x_ptr), n(topk_ids_ptr), n(topk_weight_ptr), n(group_list_ptr), n(row_token_ptr),
                     n(row_of_choice_ptr), n(x_sorted_ptr), n(workspace_ptr), T, E, K, topk, 0)


def route_workspace_bytes(args: RouteArgs) -> int:
    return int(lib.moe_route_workspace_bytes(ctypes.byref(args)))


def route(args: RouteArgs, stream: int = 0) -> None:
    _check(lib.moe_route(ctypes.byref(args), ctypes.c_void_p(stream)), "moe_route")


def route_static(args: RouteArgs, stream: int = 0) -> None:
    """moe_route with the library's own static scratch: args.workspace is ignored, nothing is allocated."""
    _check(lib.moe_route_static(ctypes.byref(args), ctypes.c_void_p(stream)), "moe_route_static")
