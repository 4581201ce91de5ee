"""Seeded inputs for the MoE ops, the oracle's answer for them, and thin wrappers that
call the GPU library through its C ABI.  Shared by the parity tests, smoke() and bench.py."""
from __future__ import annotations

import numpy as np
import torch

import oracle
from oracle import layouts as L

FORMATS = ["fp4", "fp8", "int8", "int4", "fp4_b32", "bf16", "fp4_b16"]
GEMV_FORMATS = ["fp4", "fp8", "int4", "fp4_b32", "bf16", "fp4_b16"]


def bits(t: torch.Tensor) -> np.ndarray:
    """bf16 tensor (CPU) -> uint16 bit patterns."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def from_bits(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).view(torch.bfloat16)


def bf16_uniform(rng, lo, hi, shape) -> torch.Tensor:
    return torch.from_numpy(rng.uniform(lo, hi, shape).astype(np.float32)).to(torch.bfloat16)


def routed_group_list(rng, tokens: int, experts: int, topk: int, max_rows: int | None = None) -> np.ndarray:
    """Cumulative group_list of top-k routing from softmax(N(0,1)) logits; softmax is
    monotone, so top-k of the logits picks the same experts."""
    while True:
        logits = rng.standard_normal((tokens, experts)).astype(np.float32)
        ids = np.argpartition(-logits, topk - 1, axis=1)[:, :topk].reshape(-1)
        counts = np.bincount(ids, minlength=experts)
        if max_rows is None or counts.max() <= max_rows:
            return np.cumsum(counts).astype(np.int64)


def multinomial_group_list(rng, total: int, experts: int) -> np.ndarray:
    return np.cumsum(rng.multinomial(total, np.full(experts, 1.0 / experts))).astype(np.int64)


def make_weights(fmt: str, rng, G: int, K: int, N: int, group: int = 128):
    """Returns dict(weight=np array in the op's container, scale=np array or None, offset=...)
    with the distributions the benchmark configurations name."""
    if fmt == "fp4":
        codes = rng.integers(0, 16, (G, N, K), dtype=np.uint8)          # checkpoint orientation [G, N, K]
        w = L.fp4ref_from_checkpoint(L.pack_nibbles_last(codes))        # int8 [G, K, N/2], pre-shuffled
        scale = bits(bf16_uniform(rng, 2.0 ** -8, 2.0 ** -2, (G, K // 16, N)))
        return dict(weight=w, scale=scale, offset=None, scale_rows=K // 16)
    if fmt == "fp8":
        w = rng.integers(0, 256, (G, K, N), dtype=np.uint8)
        scale = (rng.standard_normal((G, K // 128, N // 128)) * 0.01).astype(np.float32)
        return dict(weight=w, scale=scale, offset=None, scale_rows=1)
    if fmt == "int8":
        w = rng.integers(-127, 128, (G, K, N), dtype=np.int8)
        scale = bits(bf16_uniform(rng, 1e-3, 1e-2, (G, N)))
        offset = bits(bf16_uniform(rng, -2.0, 2.0, (G, N)))
        return dict(weight=w, scale=scale, offset=offset, scale_rows=1)
    if fmt == "int4":
        codes = rng.integers(0, 16, (G, K, N), dtype=np.uint8)
        w = L.pack_nibbles_last(codes)
        scale = bits(bf16_uniform(rng, 1e-3, 1e-2, (G, K // group, N)))
        return dict(weight=w, scale=scale, offset=None, scale_rows=K // group)
    if fmt == "fp4_b32":
        codes = rng.integers(0, 16, (G, N, K), dtype=np.uint8)
        w = L.pack_nibbles_last(codes)
        scale = bits(bf16_uniform(rng, 2.0 ** -8, 2.0 ** -2, (G, N, K // 32)))
        return dict(weight=w, scale=scale, offset=None, scale_rows=1)
    if fmt == "fp4_b16":
        codes = rng.integers(0, 16, (G, N, K), dtype=np.uint8)
        w = L.pack_nibbles_last(codes)
        scale = bits(bf16_uniform(rng, 2.0 ** -8, 2.0 ** -2, (G, N, K // 16)))
        return dict(weight=w, scale=scale, offset=None, scale_rows=1)
    if fmt == "bf16":
        w = bits((torch.from_numpy(rng.standard_normal((G, N, K)).astype(np.float32)) * 0.02).to(torch.bfloat16))
        return dict(weight=w, scale=None, offset=None, scale_rows=1)
    raise ValueError(fmt)


def make_case(fmt: str, G: int, K: int, N: int, group_list, seed: int, extra_rows: int = 0, group: int = 128):
    rng = np.random.default_rng(seed)
    gl = np.asarray(group_list, dtype=np.int64)
    M = int(gl[-1]) + extra_rows
    case = make_weights(fmt, rng, G, K, N, group)
    x = torch.from_numpy(rng.standard_normal((max(M, 1), K)).astype(np.float32)).to(torch.bfloat16)[:M]
    case.update(fmt=fmt, G=G, K=K, N=N, M=M, group_list=gl, x=bits(x))
    return case


def oracle_out(case, gemv: bool = False, row_mask=None) -> np.ndarray:
    """bf16 bits [M, N] from the CPU oracle (GEMM: bf16-rounded weights; GEMV: fp32 weights)."""
    return oracle.grouped_gemm(oracle.FMT_BY_NAME[case["fmt"]], case["x"], case["weight"], case["scale"],
                               case["offset"], case["group_list"], round_bf16=not gemv, row_mask=row_mask)


# ----------------------------------------------------------------------------- GPU side
def to_dev(a, device="cuda"):
    if a is None:
        return None
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).to(device)
    return torch.from_numpy(a).to(device)


def upload(case, device="cuda"):
    """Device copies of a case's tensors (bf16 tensors travel as int16 bit patterns)."""
    d = {k: to_dev(case[k], device) for k in ("x", "weight", "scale", "offset")}
    d["group_list"] = torch.from_numpy(case["group_list"]).to(device)
    return d


def run_cabi(case, dev, op: str, y: torch.Tensor | None = None, fill: int = 0x7FC0) -> np.ndarray:
    """Calls moe_grouped_gemm / moe_grouped_gemv through the C ABI; returns bf16 bits [M, N].
    y is pre-filled with a NaN pattern so that rows the op must not write are visible."""
    import moe_gfx950 as mg

    M, K, N, G = case["M"], case["K"], case["N"], case["G"]
    if y is None:
        y = torch.full((M, N), fill, dtype=torch.int16, device=dev["x"].device)
    p = lambda t: 0 if t is None else t.data_ptr()
    args = mg.grouped_args(mg.format_from_compute_type(case["fmt"]), p(dev["x"]), p(dev["weight"]), p(dev["scale"]),
                           p(dev["offset"]), p(dev["group_list"]), p(y), M, K, N, G, case["scale_rows"])
    stream = torch.cuda.current_stream().cuda_stream
    (mg.grouped_gemm if op == "gemm" else mg.grouped_gemv)(args, stream)
    torch.cuda.synchronize()
    return y.cpu().numpy().view(np.uint16)


# ------------------------------------------------------------------------------ checking
REL_TOL = 1e-2   # max|d| / max|ref|
ABS_TOL = 2e-2   # |d| <= ABS_TOL * max(1, |ref|), both sides rounded to bf16


def compare(got_bits: np.ndarray, ref_bits: np.ndarray, rows=None):
    """Returns (rel_err, worst scaled abs err) over the selected rows."""
    g = oracle.bf16_bits_to_f32(got_bits).astype(np.float64)
    r = oracle.bf16_bits_to_f32(ref_bits).astype(np.float64)
    if rows is not None:
        g, r = g[rows], r[rows]
    if g.size == 0:
        return 0.0, 0.0
    assert np.isfinite(g).all(), "non-finite values in the GPU result"
    d = np.abs(g - r)
    rel = float(d.max() / max(np.abs(r).max(), 1e-30))
    scaled = float((d / np.maximum(1.0, np.abs(r))).max())
    return rel, scaled


def assert_close(got_bits, ref_bits, rows=None, what=""):
    rel, scaled = compare(got_bits, ref_bits, rows)
    assert rel <= REL_TOL and scaled <= ABS_TOL, f"{what}: rel {rel:.3e} (tol {REL_TOL}), abs {scaled:.3e} (tol {ABS_TOL})"
    return rel, scaled
