"""Byte layouts of the reference's weight containers, restated in numpy.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).  Each function restates one
helper of the reference's test scripts; paths are relative to the reference tree.
"""
from __future__ import annotations

import numpy as np

E2M1_LEVELS = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], dtype=np.float32)


def pack_nibbles_last(codes: np.ndarray) -> np.ndarray:
    """[..., C] 4-bit codes -> uint8 [..., C/2]; the even element goes to the LOW nibble.
    grouped_gemm/test/python/test_group_gemm_fp4.py:29-35."""
    codes = np.asarray(codes, dtype=np.uint8)
    assert codes.shape[-1] % 2 == 0 and int(codes.max(initial=0)) < 16
    return (codes[..., 0::2] | (codes[..., 1::2] << 4)).astype(np.uint8)


def unpack_nibbles_last(packed: np.ndarray) -> np.ndarray:
    """Inverse of pack_nibbles_last.  test_group_gemm_fp4.py:38-43."""
    packed = np.asarray(packed, dtype=np.uint8)
    out = np.empty(packed.shape[:-1] + (packed.shape[-1] * 2,), dtype=np.uint8)
    out[..., 0::2] = packed & 0x0F
    out[..., 1::2] = packed >> 4
    return out


def fp4ref_stage1(ckpt: np.ndarray) -> np.ndarray:
    """Checkpoint form uint8 [G, N, K/2] (packed along K) -> int8 [G, K, N/2]
    packed along N: byte (k, c) = code(k, 2c) | code(k, 2c+1) << 4.
    `repack_weight`, test_group_gemm_fp4.py:105-117."""
    codes_nk = unpack_nibbles_last(ckpt)                 # [G, N, K]
    codes_kn = np.ascontiguousarray(np.swapaxes(codes_nk, -1, -2))  # [G, K, N]
    return pack_nibbles_last(codes_kn).view(np.int8)


def fp4ref_stage2(w: np.ndarray) -> np.ndarray:
    """Byte permutation inside every 64(k) x 128(byte) tile of [G, K, N/2].
    `repack_weight_step2`, test_group_gemm_fp4.py:129-142."""
    G, K, NB = w.shape
    assert K % 64 == 0 and NB % 128 == 0
    t = w.reshape(G * K // 64, 4, 2, 8, NB // 128, 8, 4, 4)
    t = np.ascontiguousarray(t.transpose(0, 2, 1, 5, 4, 6, 3, 7))
    return t.reshape(G, K, NB)


def fp4ref_stage2_inverse(w: np.ndarray) -> np.ndarray:
    G, K, NB = w.shape
    t = w.reshape(G * K // 64, 2, 4, 8, NB // 128, 4, 8, 4)
    t = np.ascontiguousarray(t.transpose(0, 2, 1, 6, 4, 3, 5, 7))
    return t.reshape(G, K, NB)


def fp4ref_from_checkpoint(ckpt: np.ndarray) -> np.ndarray:
    """What the reference test feeds the op: stage 1 then stage 2
    (test_group_gemm_fp4.py:180-181)."""
    return fp4ref_stage2(fp4ref_stage1(ckpt))


def fp4ref_codes_kn(w: np.ndarray) -> np.ndarray:
    """Logical codes [G, K, N] held by an op-input container int8 [G, K, N/2]."""
    return unpack_nibbles_last(fp4ref_stage2_inverse(np.asarray(w).view(np.uint8)))


def e2m1_quantize_to_codes(x: np.ndarray) -> np.ndarray:
    """Exact-match quantizer of the reference test (values already on the e2m1 grid
    map to their code; anything else maps to magnitude index 0).
    `to_fp4_e2m1_in_uint8`, test_group_gemm_fp4.py:11-18."""
    x = np.asarray(x, dtype=np.float32)
    idx = (np.abs(x)[..., None] == E2M1_LEVELS).astype(np.uint8).argmax(-1).astype(np.uint8)
    return ((x < 0).astype(np.uint8) << 3) | idx


def fp8ref_dequant_numpy(w: np.ndarray, scale: np.ndarray, round_bf16: bool) -> np.ndarray:
    """The reference test's fp8 dequant, reshape/permute form, in numpy fp32.
    `anti_quant_fp8`, test_group_gemm_fp8.py:7-32 (bf16-rounded) and
    test_group_soft_gemv_fp8.py:7-34 (un-rounded).  Needs K, N multiples of 128."""
    from . import bf16_bits_to_f32, f32_to_bf16_bits

    G, K, N = w.shape
    wi = w.astype(np.int16)
    bits = (((wi & 0x80) << 8) | ((wi & 0x7F) << 4)).astype(np.uint16)
    # bf16 * bf16 -> bf16 (exact here: one operand is the power of two 0x7B80 = 2^120)
    val = bf16_bits_to_f32(f32_to_bf16_bits(bf16_bits_to_f32(bits) * bf16_bits_to_f32(np.uint16(0x7B80))))
    val = val.reshape(G, K // 128, 128, N // 128, 128).transpose(0, 1, 3, 2, 4)
    val = val.reshape(G, -1, 128 * 128) * scale.reshape(G, -1)[..., None].astype(np.float32)
    if round_bf16:
        val = bf16_bits_to_f32(f32_to_bf16_bits(val))
    val = val.reshape(G, K // 128, N // 128, 128, 128).transpose(0, 1, 3, 2, 4)
    return np.ascontiguousarray(val).reshape(G, K, N)


def fp4ref_scale_from_checkpoint(scale_bits: np.ndarray, scale2: np.ndarray | None = None) -> np.ndarray:
    """Checkpoint block scales bf16 bits [G, N, K/16] (+ optional fp32 second-level scale
    [G, 1] or [G, 2]) -> the op's scale tensor, bf16 bits [G, K/16, N].

    anti_quant_fp8_scale (test_group_gemm_fp4.py:86-94): the bf16 tensor is multiplied in place by
    the fp32 factor -- an fp32 product rounded to nearest even -- one factor per expert, or one
    for each half of the N rows; then transposed (:185-186)."""
    from . import bf16_bits_to_f32, f32_to_bf16_bits

    s = np.asarray(scale_bits, dtype=np.uint16)
    G, N, KB = s.shape
    if scale2 is not None:
        s2 = np.asarray(scale2, dtype=np.float32).reshape(G, -1)
        f = bf16_bits_to_f32(s)
        if s2.shape[1] == 1:
            f = f * s2[:, :, None]
        else:
            assert s2.shape[1] == 2 and N % 2 == 0
            f = f.copy()
            f[:, : N // 2, :] *= s2[:, 0, None, None]
            f[:, N // 2 :, :] *= s2[:, 1, None, None]
        s = f32_to_bf16_bits(f.astype(np.float32))
    return np.ascontiguousarray(s.transpose(0, 2, 1))
