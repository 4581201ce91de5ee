"""CPU oracle for the MoE antiquant ops -- TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may
import this package.  The product (ascend-kernel_amd/) never does; it has no
CPU fallback and fails loudly when its HIP library is missing.

moe_oracle.c holds the arithmetic (plain C, loaded through ctypes);
layouts.py holds the byte-layout restatements (numpy reshape/permute).
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmoe_oracle.so")

FMT_FP4_REF, FMT_FP8_REF, FMT_INT8, FMT_INT4, FMT_FP4_B32, FMT_BF16, FMT_FP4_B16 = range(7)
FMT_BY_NAME = {
    "fp4": FMT_FP4_REF,
    "fp8": FMT_FP8_REF,
    "int8": FMT_INT8,
    "int4": FMT_INT4,
    "fp4_b32": FMT_FP4_B32,
    "bf16": FMT_BF16,
    "fp4_b16": FMT_FP4_B16,
}


def build(force: bool = False) -> str:
    """Compile libmoe_oracle.so with the Makefile beside this file."""
    src = os.path.join(_HERE, "moe_oracle.c")
    stale = (not os.path.exists(_LIB_PATH)) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src)
    if force or stale:
        subprocess.check_call(["make", "-C", _HERE, "-B", "libmoe_oracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
        L.orc_num_threads.restype = ctypes.c_int
        L.orc_e2m1_decode.restype = ctypes.c_float
        L.orc_e2m1_decode.argtypes = [ctypes.c_uint8]
        L.orc_e4m3_decode.restype = ctypes.c_float
        L.orc_e4m3_decode.argtypes = [ctypes.c_uint8]
        L.orc_f32_to_bf16.restype = ctypes.c_uint16
        L.orc_f32_to_bf16.argtypes = [ctypes.c_float]
        L.orc_bf16_to_f32.restype = ctypes.c_float
        L.orc_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.orc_fp4ref_locate.restype = i64
        L.orc_fp4ref_locate.argtypes = [i64, i64, i64, ctypes.POINTER(i32)]
        L.orc_dequant_fp4_bf16.restype = None
        L.orc_dequant_fp4_bf16.argtypes = [vp, vp, vp, i64, i64, i64]
        L.orc_expand_weight.restype = i32
        L.orc_expand_weight.argtypes = [i32, vp, vp, vp, i64, i64, i64, i64, i32, vp]
        L.orc_grouped_gemm.restype = i32
        L.orc_grouped_gemm.argtypes = [i32, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i32, vp, vp, vp]
        _lib = L
    return _lib


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype=None):
    if a is None:
        return None
    a = np.ascontiguousarray(a)
    if dtype is not None and a.dtype != dtype:
        raise TypeError(f"expected {dtype}, got {a.dtype}")
    return a


def num_threads() -> int:
    return int(lib().orc_num_threads())


def e2m1_decode(code: int) -> float:
    return float(lib().orc_e2m1_decode(int(code) & 0xFF))


def e4m3_decode(code: int) -> float:
    return float(lib().orc_e4m3_decode(int(code) & 0xFF))


def f32_to_bf16_bits(a: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 bit patterns (uint16), round to nearest even."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    return r.astype(np.uint16)


def bf16_bits_to_f32(a: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(a, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def fp4ref_locate(k: int, n: int, N: int):
    nib = ctypes.c_int(0)
    idx = lib().orc_fp4ref_locate(k, n, N, ctypes.byref(nib))
    return int(idx), int(nib.value)


def dequant_fp4_bf16(codes: np.ndarray, scale_bits: np.ndarray, block: int = 32) -> np.ndarray:
    """codes uint8 [R, C/2], scale bf16 bits uint16 [R, C/block] -> bf16 bits uint16 [R, C]."""
    codes = _c(codes, np.uint8)
    scale_bits = _c(scale_bits, np.uint16)
    R, C = codes.shape[0], codes.shape[1] * 2
    assert scale_bits.shape == (R, C // block), (scale_bits.shape, R, C, block)
    out = np.empty((R, C), dtype=np.uint16)
    lib().orc_dequant_fp4_bf16(_ptr(codes), _ptr(scale_bits), _ptr(out), R, C, block)
    return out


def _logical_knG(fmt: int, w: np.ndarray):
    """(G, K, N) of the logical weight held by container w."""
    G = w.shape[0]
    if fmt in (FMT_FP4_REF, FMT_INT4):
        return G, w.shape[1], w.shape[2] * 2
    if fmt in (FMT_FP8_REF, FMT_INT8):
        return G, w.shape[1], w.shape[2]
    if fmt in (FMT_FP4_B32, FMT_FP4_B16):
        return G, w.shape[2] * 2, w.shape[1]
    if fmt == FMT_BF16:
        return G, w.shape[2], w.shape[1]
    raise ValueError(fmt)


def _scale_rows(fmt: int, scale, K: int) -> int:
    if fmt in (FMT_FP4_REF, FMT_INT4):
        return int(scale.shape[-2])
    return 1


def expand_weight(fmt: int, w, scale, offset, g: int, round_bf16: bool) -> np.ndarray:
    """Dense fp32 W[K, N] of expert g (bf16-rounded values if round_bf16)."""
    w = _c(w)
    scale = _c(scale)
    offset = _c(offset)
    G, K, N = _logical_knG(fmt, w)
    out = np.empty((K, N), dtype=np.float32)
    rc = lib().orc_expand_weight(fmt, _ptr(w), _ptr(scale), _ptr(offset), g, K, N,
                                 _scale_rows(fmt, scale, K), int(round_bf16), _ptr(out))
    if rc:
        raise RuntimeError(f"orc_expand_weight rc={rc}")
    return out


def grouped_gemm(fmt: int, x_bits, w, scale, offset, group_list, *, round_bf16: bool = True,
                 row_mask=None, want_f32: bool = False):
    """x bf16 bits uint16 [M,K]; returns y bf16 bits uint16 [M,N] (zeros where untouched)
    and, if want_f32, the un-rounded fp32 accumulators as well."""
    x_bits = _c(x_bits, np.uint16)
    w = _c(w)
    scale = _c(scale)
    offset = _c(offset)
    gl = _c(np.asarray(group_list, dtype=np.int64))
    G, K, N = _logical_knG(fmt, w)
    M = x_bits.shape[0]
    assert x_bits.shape[1] == K and gl.shape[0] == G
    y16 = np.zeros((M, N), dtype=np.uint16)
    y32 = np.zeros((M, N), dtype=np.float32) if want_f32 else None
    mask = _c(np.asarray(row_mask, dtype=np.uint8)) if row_mask is not None else None
    rc = lib().orc_grouped_gemm(fmt, _ptr(x_bits), _ptr(w), _ptr(scale), _ptr(offset), _ptr(gl),
                                M, K, N, G, _scale_rows(fmt, scale, K), int(round_bf16),
                                _ptr(mask), _ptr(y16), _ptr(y32))
    if rc:
        raise RuntimeError(f"orc_grouped_gemm rc={rc}")
    return (y16, y32) if want_f32 else y16


def swiglu_interleaved(z: np.ndarray) -> np.ndarray:
    """fp32 accumulators [M, N] whose columns come in groups of 4 = (gate 2j, gate 2j+1, up 2j, up 2j+1)
    -> bf16 bits [M, N/2], out[:, 2j+e] = silu(z[:, 4j+e]) * z[:, 4j+2+e] with silu(v) = v / (1 + exp(-v)),
    evaluated in float64 and rounded once.  The fused activation has no counterpart in the reference
    (its caller applies the activation to grouped_gemm's output as a separate op); this is the
    definition the GPU epilogue is checked against, pinned to torch.nn.functional.silu in
    tests/test_oracle.py."""
    z = np.asarray(z, dtype=np.float64)
    M, N = z.shape
    assert N % 4 == 0
    q = z.reshape(M, N // 4, 4)
    gate, up = q[:, :, 0:2], q[:, :, 2:4]
    out = (gate / (1.0 + np.exp(-gate)) * up).reshape(M, N // 2)
    return f32_to_bf16_bits(out.astype(np.float32))


def swiglu_blocked16(z: np.ndarray) -> np.ndarray:
    """The fused activation on the K-contiguous containers: the weight rows (columns of z) come in blocks of
    32 = (gate 16j..16j+15, up 16j..16j+15); out[:, 16j+i] = silu(z[:, 32j+i]) * z[:, 32j+16+i], float64, one
    rounding to bf16.  Same definition of silu as swiglu_interleaved; pinned to torch in tests/test_oracle.py."""
    z = np.asarray(z, dtype=np.float64)
    M, N = z.shape
    assert N % 32 == 0
    b = z.reshape(M, N // 32, 2, 16)
    gate, up = b[:, :, 0, :], b[:, :, 1, :]
    out = (gate / (1.0 + np.exp(-gate)) * up).reshape(M, N // 2)
    return f32_to_bf16_bits(out.astype(np.float32))
