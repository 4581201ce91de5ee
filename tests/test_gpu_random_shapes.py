"""Seeded random sweep of shapes, group lists and batch sizes through both grouped ops and every
weight format, against the oracle.  The cases are drawn so that every dispatch branch is hit: decode
batches (at most 4 rows per expert on average), the matrix-core GEMV range, the small-tile GEMM range
and prefill tiles, with empty experts, single rows and row counts around the 16-row block size."""
import sys
import zlib

import numpy as np
import pytest

import helpers as H

pytestmark = pytest.mark.gpu

K_STEP = {"fp4": 64, "fp8": 128, "int8": 64, "int4": 128, "fp4_b32": 128, "bf16": 64, "fp4_b16": 128}


def _say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def _random_counts(rng, G, regime):
    if regime == "decode":        # M <= 4 G
        c = rng.integers(0, 5, G)
    elif regime == "mid":         # around the 16-row block size: both sides of the GEMV / GEMM kernel dispatch bound (12 G)
        c = rng.choice([0, 1, 5, 8, 15, 16, 17, 19], G)
    elif regime == "small_tile":  # 20 G < M <= 24 G (bf16: the small-tile kernel)
        c = np.full(G, 22) + rng.integers(-1, 2, G)
    else:                         # prefill: ragged, up to a few row blocks, some empty experts
        c = rng.choice([0, 3, 31, 33, 64, 100, 161, 200], G)
    if c.sum() == 0:
        c[rng.integers(0, G)] = 1
    return c


@pytest.mark.parametrize("regime", ["decode", "mid", "small_tile", "prefill"])
@pytest.mark.parametrize("fmt", H.FORMATS)
def test_random_gemm(fmt, regime):
    seed = zlib.crc32(f"rand-gemm/{fmt}/{regime}".encode())
    rng = np.random.default_rng(seed)
    for rep in range(2):
        G = int(rng.integers(1, 8))
        K = int(rng.integers(1, 9)) * K_STEP[fmt] * (4 if rep else 1)      # the second draw is a multiple of 512 for the 128-step formats
        N = int(rng.integers(1, 4)) * 256
        counts = _random_counts(rng, G, regime)
        gl = list(np.cumsum(counts))
        _say(f"random gemm fmt={fmt} regime={regime} G={G} K={K} N={N} counts={list(counts)}")
        group = 128 if K % 128 == 0 else 64
        case = H.make_case(fmt, G, K, N, gl, seed=seed % 1000 + rep, extra_rows=int(rng.integers(0, 3)), group=group)
        got = H.run_cabi(case, H.upload(case), "gemm")
        H.assert_close(got, H.oracle_out(case), rows=slice(0, gl[-1]), what=f"{fmt}/{regime}/{rep}")
        assert (got[gl[-1]:] == 0x7FC0).all(), "rows beyond group_list[-1] were written"


@pytest.mark.parametrize("regime", ["decode", "mid"])
@pytest.mark.parametrize("fmt", H.GEMV_FORMATS)
def test_random_gemv(fmt, regime):
    seed = zlib.crc32(f"rand-gemv/{fmt}/{regime}".encode())
    rng = np.random.default_rng(seed)
    k_major = fmt in ("fp4_b32", "bf16", "fp4_b16")
    for rep in range(2):
        G = int(rng.integers(1, 8))
        K = int(rng.integers(1, 9)) * (32 if k_major and rep == 0 else K_STEP[fmt] * (4 if rep else 1))
        N = int(rng.integers(1, 700)) if k_major else int(rng.integers(1, 4)) * 256
        counts = _random_counts(rng, G, regime)
        gl = list(np.cumsum(counts))
        _say(f"random gemv fmt={fmt} regime={regime} G={G} K={K} N={N} counts={list(counts)}")
        group = 128 if K % 128 == 0 else 64
        case = H.make_case(fmt, G, K, N, gl, seed=seed % 1000 + rep, extra_rows=int(rng.integers(0, 3)), group=group)
        got = H.run_cabi(case, H.upload(case), "gemv")
        H.assert_close(got, H.oracle_out(case, gemv=True), rows=slice(0, gl[-1]), what=f"gemv {fmt}/{regime}/{rep}")
        assert (got[gl[-1]:] == 0x7FC0).all(), "rows beyond group_list[-1] were written"
