"""Writes the known-answer fixtures of this directory (`python tests/golden/make_fixtures.py`).

Every expected value here is computed with numpy / torch library routines only, straight from the
definitions in the reference's test scripts (cited where used): loops over the index formulas,
torch's float8_e4m3fn and bfloat16 casts, float64 matmul.  Nothing is imported from oracle/ or from
the GPU package, so the files check both of them against a third, independent computation.

Fixtures (numpy .npz, a few tens of KB each; bf16 tensors are stored as uint16 bit patterns):
  grouped_<format>.npz   inputs of one small grouped call + y_gemm (weights rounded to bf16, the
                         GEMM op) and y_gemv (fp32 weights, the GEMV op), fp64-accumulated
  dequant_fp4.npz        every byte value x edge-case scales -> bf16 bits, blocks of 32 and of 16
  prepack_fp4.npz        checkpoint codes / scales / second-level scale -> the "fp4" container
  route.npz              logits -> top-k ids and weights, group_list, sorted row order
"""
from __future__ import annotations

import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))

# e2m1 magnitudes, sign in bit 3: grouped_gemm/test/python/test_group_gemm_fp4.py:6-8, :15, :22
E2M1 = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], dtype=np.float32)


def e2m1(codes: np.ndarray) -> np.ndarray:
    mag = E2M1[codes & 7]
    return np.where(codes & 8, -mag, mag).astype(np.float32)   # code 8 is -0.0


def e4m3(codes: np.ndarray) -> np.ndarray:
    """OCP e4m3 by torch's cast; the two NaN codes decode to +-480 as the reference's bit trick does
    (grouped_gemm/op_kernel/antiquant_impl.h:87-129: no NaN handling)."""
    v = torch.from_numpy(codes.astype(np.uint8)).view(torch.float8_e4m3fn).float().numpy()
    v = np.where(codes == 0x7F, np.float32(480.0), v)
    return np.where(codes == 0xFF, np.float32(-480.0), v).astype(np.float32)


def to_bf16_bits(a: np.ndarray) -> np.ndarray:
    t = torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.bfloat16)
    return t.view(torch.int16).numpy().view(np.uint16)


def from_bf16_bits(b: np.ndarray) -> np.ndarray:
    return torch.from_numpy(np.ascontiguousarray(b).view(np.int16)).view(torch.bfloat16).float().numpy()


def round_bf16(a: np.ndarray) -> np.ndarray:
    return from_bf16_bits(to_bf16_bits(a))


def pack_low_first(codes: np.ndarray) -> np.ndarray:
    """Two 4-bit codes per byte along the last axis, even index in the low nibble
    (test_group_gemm_fp4.py:29-35)."""
    return (codes[..., 0::2] | (codes[..., 1::2] << 4)).astype(np.uint8)


def fp4_container(codes_gnk: np.ndarray) -> np.ndarray:
    """codes [G, N, K] -> the op's int8 [G, K, N/2]: K-major, two codes per byte along N
    (repack_weight, test_group_gemm_fp4.py:105-117), then the byte permutation inside every
    64(k) x 128(byte) tile (repack_weight_step2, :129-142), written as plain loops over the
    destination index: row R = 32 j + 8 i + p, byte b = 32 q + 4 r + s of a tile hold source row
    16 i + 8 j + r and source byte 16 p + 4 q + s."""
    G, N, K = codes_gnk.shape
    stage1 = pack_low_first(np.transpose(codes_gnk, (0, 2, 1)))   # [G, K, N/2]
    out = np.empty_like(stage1)
    for R in range(64):
        j, i, p = R >> 5, (R >> 3) & 3, R & 7
        for b in range(128):
            q, r, s = b >> 5, (b >> 2) & 7, b & 3
            out[:, R::64, b::128] = stage1[:, (16 * i + 8 * j + r)::64, (16 * p + 4 * q + s)::128]
    return out.view(np.int8)


def grouped_expected(x_bits, W, group_list):
    """y = x . W per expert, float64 accumulation, for weights W [G, K, N] (float32 values):
    returns (y with W rounded to bf16, y with W as is), both rounded to bf16 once."""
    x = from_bf16_bits(x_bits).astype(np.float64)
    M, N = x.shape[0], W.shape[2]
    yg, yv = np.zeros((M, N), np.float32), np.zeros((M, N), np.float32)
    lo = 0
    for g, hi in enumerate(group_list):
        hi = int(hi)
        yg[lo:hi] = x[lo:hi] @ round_bf16(W[g]).astype(np.float64)
        yv[lo:hi] = x[lo:hi] @ W[g].astype(np.float64)
        lo = hi
    return to_bf16_bits(yg), to_bf16_bits(yv)


def grouped_fixture(fmt: str, seed: int):
    rng = np.random.default_rng(seed)
    G, K, N = 3, 128, 256
    gl = np.array([2, 2, 7], dtype=np.int64)                  # the second expert has no rows
    M = int(gl[-1])
    x = to_bf16_bits(rng.standard_normal((M, K)).astype(np.float32))
    d = dict(fmt=fmt, x=x, group_list=gl, K=K, N=N, G=G, scale_rows=1)
    if fmt in ("fp4", "fp4_b32", "fp4_b16"):
        codes = rng.integers(0, 16, (G, N, K), dtype=np.uint8)            # checkpoint orientation
        blk = 32 if fmt == "fp4_b32" else 16
        s_bits = to_bf16_bits(rng.uniform(2.0 ** -8, 2.0 ** -2, (G, N, K // blk)).astype(np.float32))
        s = from_bf16_bits(s_bits)
        W = np.transpose(e2m1(codes) * np.repeat(s, blk, axis=2), (0, 2, 1))   # fp32 product, [G, K, N]
        if fmt == "fp4":
            d.update(weight=fp4_container(codes), scale=np.ascontiguousarray(np.transpose(s_bits, (0, 2, 1))),
                     scale_rows=K // 16)                                    # scale [G, K/16, N] (:185-186)
        else:
            d.update(weight=pack_low_first(codes), scale=s_bits)
    elif fmt == "fp8":
        w = rng.integers(0, 256, (G, K, N), dtype=np.uint8)
        s = (rng.standard_normal((G, K // 128, N // 128)) * 0.01).astype(np.float32)
        # 128 x 128 block scales (grouped_gemm/test/python/test_group_gemm_fp8.py:41-44)
        W = e4m3(w) * np.repeat(np.repeat(s, 128, axis=1), 128, axis=2)
        d.update(weight=w, scale=s)
    elif fmt == "int8":
        w = rng.integers(-127, 128, (G, K, N), dtype=np.int8)
        s_bits = to_bf16_bits(rng.uniform(1e-3, 1e-2, (G, N)).astype(np.float32))
        o_bits = to_bf16_bits(rng.uniform(-2.0, 2.0, (G, N)).astype(np.float32))
        # (w + offset) * scale, each operation rounded to fp32
        W = (w.astype(np.float32) + from_bf16_bits(o_bits)[:, None, :]) * from_bf16_bits(s_bits)[:, None, :]
        d.update(weight=w, scale=s_bits, offset=o_bits)
    elif fmt == "int4":
        group = 64
        q = rng.integers(0, 16, (G, K, N), dtype=np.uint8)
        s_bits = to_bf16_bits(rng.uniform(1e-3, 1e-2, (G, K // group, N)).astype(np.float32))
        W = (q.astype(np.float32) - 8.0) * np.repeat(from_bf16_bits(s_bits), group, axis=1)
        d.update(weight=pack_low_first(q), scale=s_bits, scale_rows=K // group)
    elif fmt == "bf16":
        w_bits = to_bf16_bits((rng.standard_normal((G, N, K)) * 0.02).astype(np.float32))
        W = np.transpose(from_bf16_bits(w_bits), (0, 2, 1))
        d.update(weight=w_bits)
    else:
        raise ValueError(fmt)
    d["y_gemm"], d["y_gemv"] = grouped_expected(x, W.astype(np.float32), gl)
    return d


def dequant_fixture():
    # 16 x 64 codes = 512 bytes: every byte value twice; scales from a list of edge cases
    # (smallest and largest normal bf16, 1, negative, a value whose product needs rounding, zero)
    codes = (np.arange(16 * 32) % 256).astype(np.uint8).reshape(16, 32)
    edge = np.array([0x0080, 0x7F7F, 0x3F80, 0xBF80, 0x3FB5, 0x0000, 0x3DCD, 0xC2F7], dtype=np.uint16)
    d = dict(codes=codes)
    nib = np.stack([codes & 15, codes >> 4], axis=-1).reshape(16, 64)      # even element in the low nibble
    for blk in (32, 16):
        s_bits = edge[(np.arange(16 * (64 // blk)) * 5 + 1) % edge.size].reshape(16, 64 // blk)
        with np.errstate(over="ignore"):
            prod = e2m1(nib) * np.repeat(from_bf16_bits(s_bits), blk, axis=1)   # fp32 product, one rounding to bf16
        d[f"scale_b{blk}"] = s_bits
        d[f"out_b{blk}"] = to_bf16_bits(prod)
    return d


def prepack_fixture():
    rng = np.random.default_rng(21)
    G, N, K = 2, 256, 128
    codes = rng.integers(0, 16, (G, N, K), dtype=np.uint8)
    s_bits = to_bf16_bits(rng.uniform(1.0, 448.0, (G, N, K // 16)).astype(np.float32))
    s2 = rng.uniform(1e-4, 1e-2, (G, 1)).astype(np.float32)
    # scale *= scale_2 on a bf16 tensor (anti_quant_fp8_scale, test_group_gemm_fp4.py:86-94), then the
    # transpose to [G, K/16, N] (:185-186)
    merged = to_bf16_bits(from_bf16_bits(s_bits) * s2[:, :, None])
    return dict(ckpt=pack_low_first(codes), scale=s_bits, scale2=s2, weight_out=fp4_container(codes),
                scale_out=np.ascontiguousarray(np.transpose(merged, (0, 2, 1))))


def route_fixture():
    rng = np.random.default_rng(22)
    T, E, topk = 37, 16, 4
    logits = rng.standard_normal((T, E)).astype(np.float32)
    ids = np.argsort(-logits, axis=1, kind="stable")[:, :topk].astype(np.int32)   # ties: the lower expert id
    p = np.exp(logits.astype(np.float64) - logits.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    weight = np.take_along_axis(p, ids.astype(np.int64), axis=1).astype(np.float32)
    flat = ids.reshape(-1)
    order = np.argsort(flat, kind="stable")                  # by expert, then by flat choice index
    group_list = np.cumsum(np.bincount(flat, minlength=E)).astype(np.int64)
    row_of_choice = np.empty(flat.size, np.int32)
    row_of_choice[order] = np.arange(flat.size, dtype=np.int32)
    return dict(logits=logits, topk=np.int32(topk), ids=ids, weight=weight, group_list=group_list,
                row_token=(order // topk).astype(np.int32), row_of_choice=row_of_choice)


GROUPED_FORMATS = ["fp4", "fp8", "int8", "int4", "fp4_b32", "fp4_b16", "bf16"]


def all_fixtures():
    out = {f"grouped_{fmt}": grouped_fixture(fmt, 100 + i) for i, fmt in enumerate(GROUPED_FORMATS)}
    out["dequant_fp4"] = dequant_fixture()
    out["prepack_fp4"] = prepack_fixture()
    out["route"] = route_fixture()
    return out


def main():
    for name, d in all_fixtures().items():
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, **{k: v for k, v in d.items() if v is not None})
        print(f"{name}.npz: {os.path.getsize(path)} bytes")


if __name__ == "__main__":
    main()
