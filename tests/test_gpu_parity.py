"""GPU parity tests: the HIP kernels, called through the C ABI (and through the
cinfer_ascendc module), against the CPU oracle on identical seeded inputs.

Bars: FP4 dequant bit-exact; grouped GEMM / GEMV max|d|/max|ref| <= 1e-2 and
|d| <= 2e-2 * max(1, |ref|), both sides rounded to bf16 (helpers.REL_TOL / ABS_TOL)."""
import zlib

import numpy as np
import pytest
import torch

import helpers as H
import oracle
from oracle import layouts as L

pytestmark = pytest.mark.gpu


def _say(msg):
    print(msg, flush=True)


# ------------------------------------------------------------------------ FP4 dequant
def _dequant_gpu(codes: np.ndarray, scale_bits: np.ndarray, block: int) -> np.ndarray:
    import moe_gfx950 as mg

    R, C = codes.shape[0], codes.shape[1] * 2
    d_codes, d_scale = torch.from_numpy(codes).cuda(), H.to_dev(scale_bits)
    out = torch.full((R, C), 0x7FC0, dtype=torch.int16, device="cuda")
    mg.dequant_fp4_bf16(d_codes.data_ptr(), d_scale.data_ptr(), out.data_ptr(), R, C, block,
                        torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return out.cpu().numpy().view(np.uint16)


@pytest.mark.parametrize("R,C,block", [(64, 256, 32), (7, 96, 32), (3, 48, 16), (1, 32, 32), (257, 2048, 32)])
def test_dequant_bit_exact_small(R, C, block):
    _say(f"dequant R={R} C={C} block={block}")
    rng = np.random.default_rng(100 + R)
    codes = rng.integers(0, 256, (R, C // 2), dtype=np.uint8)
    scale = H.bits(H.bf16_uniform(rng, 2.0 ** -8, 2.0 ** -2, (R, C // block)))
    assert np.array_equal(_dequant_gpu(codes, scale, block), oracle.dequant_fp4_bf16(codes, scale, block))


def test_dequant_bit_exact_all_codes_and_edge_scales():
    # every byte value against scales that hit rounding ties, tiny and huge magnitudes, negative scales
    _say("dequant all codes x edge scales")
    sc = np.array([0x3F80, 0x3F81, 0x3FFF, 0x0080, 0x0001, 0x7F00, 0xBF80, 0x3C58, 0x4049, 0x0000, 0x8000, 0x3EAB,
                   0x1234, 0x7E80, 0x00FF, 0x807F], dtype=np.uint16)
    codes = np.tile(np.arange(256, dtype=np.uint8).reshape(16, 16), (len(sc), 1))  # [16*len, 16] -> 32 cols
    scale = np.repeat(sc, 16).reshape(-1, 1)
    got = _dequant_gpu(codes, scale, 32)
    ref = oracle.dequant_fp4_bf16(codes, scale, 32)
    assert np.array_equal(got, ref)
    # code 8 is -0.0 whatever the (positive) scale
    z = _dequant_gpu(np.full((1, 16), 0x88, np.uint8), np.array([[0x3F80]], np.uint16), 32)
    assert (z == 0x8000).all()


def test_dequant_full_size_config():
    # 7168 x 2048 weight of the benchmark configuration, bit-exact against the oracle
    _say("dequant 7168x2048")
    rng = np.random.default_rng(1)
    codes = rng.integers(0, 256, (7168, 1024), dtype=np.uint8)
    scale = H.bits(H.bf16_uniform(rng, 2.0 ** -8, 2.0 ** -2, (7168, 64)))
    assert np.array_equal(_dequant_gpu(codes, scale, 32), oracle.dequant_fp4_bf16(codes, scale, 32))


@pytest.mark.parametrize("block", [32, 16])
def test_dequant_large_tensor_path(block):
    """Tensors of 128 Mi elements and more run on 1024-thread workgroups: bit-identical to the same rows taken
    through the small-tensor path slice by slice, and to the oracle on a sample of rows."""
    import moe_gfx950 as mg

    _say(f"dequant large block={block}")
    R, C = 16384 + 3, 8192                     # 134 Mi elements, not a multiple of the workgroup's span
    gen = torch.Generator(device="cuda").manual_seed(block)
    codes = torch.randint(0, 256, (R, C // 2), dtype=torch.uint8, device="cuda", generator=gen)
    scale = (torch.rand(R, C // block, device="cuda", generator=gen) * 0.24 + 2.0 ** -8).to(torch.bfloat16)
    whole = torch.full((R, C), 0x7FC0, dtype=torch.int16, device="cuda")
    parts = torch.full((R, C), 0x7FC0, dtype=torch.int16, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    mg.dequant_fp4_bf16(codes.data_ptr(), scale.data_ptr(), whole.data_ptr(), R, C, block, st)
    step = 2048
    for r0 in range(0, R, step):
        n = min(step, R - r0)
        mg.dequant_fp4_bf16(codes[r0:].data_ptr(), scale[r0:].data_ptr(), parts[r0:].data_ptr(), n, C, block, st)
    torch.cuda.synchronize()
    assert torch.equal(whole, parts)
    rows = [0, 1, 4095, 8192, R - 1]
    got = whole[rows].cpu().numpy().view(np.uint16)
    want = oracle.dequant_fp4_bf16(codes[rows].cpu().numpy(), H.bits(scale[rows].cpu()), block)
    assert np.array_equal(got, want)


def test_dequant_module_entry_point_and_empty():
    import cinfer_ascendc

    _say("dequant via module")
    rng = np.random.default_rng(2)
    codes = rng.integers(0, 256, (33, 64), dtype=np.uint8)
    scale = H.bits(H.bf16_uniform(rng, 2.0 ** -8, 2.0 ** -2, (33, 4)))
    out = torch.empty(33, 128, dtype=torch.bfloat16, device="cuda")
    cinfer_ascendc.dequant_fp4(weight=torch.from_numpy(codes).cuda(), scale=H.to_dev(scale).view(torch.bfloat16),
                               output=out)
    torch.cuda.synchronize()
    assert np.array_equal(H.bits(out), oracle.dequant_fp4_bf16(codes, scale, 32))
    cinfer_ascendc.dequant_fp4(torch.empty(0, 64, dtype=torch.uint8, device="cuda"),
                               torch.empty(0, 4, dtype=torch.bfloat16, device="cuda"),
                               torch.empty(0, 128, dtype=torch.bfloat16, device="cuda"))


# ------------------------------------------------------------------------ grouped GEMM
GEMM_GROUP_LISTS = {
    "ref_fp4": [2, 3, 4, 256],        # test_group_gemm_fp4.py:172
    "ref_fp8": [12, 25, 44, 48],      # test_group_gemm_fp8.py:50
    "empties": [0, 0, 37, 37, 37, 150, 150, 151],
    "one_big": [0, 500, 500, 500],    # > 192 rows: several row chunks
    "all_empty": [0, 0, 0],
}


@pytest.mark.parametrize("fmt", H.FORMATS)
@pytest.mark.parametrize("gl_name", list(GEMM_GROUP_LISTS))
def test_gemm_parity_small(fmt, gl_name):
    gl = GEMM_GROUP_LISTS[gl_name]
    G, K, N = len(gl), 512, 512
    _say(f"gemm fmt={fmt} gl={gl_name} G={G} K={K} N={N}")
    case = H.make_case(fmt, G, K, N, gl, seed=zlib.crc32(f"{fmt}/{gl_name}".encode()) % 1000, extra_rows=5)
    got = H.run_cabi(case, H.upload(case), "gemm")
    ref = H.oracle_out(case)
    M_used = gl[-1]
    H.assert_close(got, ref, rows=slice(0, M_used), what=f"{fmt}/{gl_name}")
    assert (got[M_used:] == 0x7FC0).all(), "rows beyond group_list[-1] were written"


@pytest.mark.parametrize("fmt,K,N", [("int4", 7168, 256), ("int8", 4096, 512), ("fp4", 1024, 1024),
                                     ("fp8", 1536, 768), ("fp4_b32", 7168, 256), ("bf16", 2048, 256),
                                     ("int4", 2048, 1792)])
def test_gemm_parity_deep_k_and_wide_n(fmt, K, N):
    _say(f"gemm deep fmt={fmt} K={K} N={N}")
    gl = [130, 130, 143, 300, 301]
    case = H.make_case(fmt, len(gl), K, N, gl, seed=K + N)
    got = H.run_cabi(case, H.upload(case), "gemm")
    H.assert_close(got, H.oracle_out(case), what=f"{fmt} K={K} N={N}")


@pytest.mark.parametrize("op", ["gemm", "gemv"])
@pytest.mark.parametrize("N", [128, 384, 1408])
def test_fp8_n_multiple_of_128(N, op):
    """The reference tiles uint8 weights 128 columns wide (grouped_gemm/op_host/grouped_matmul_antiquant_tiling.cpp:616-621,
    grouped_soft_gemv/op_host/grouped_soft_gemv_tiling.cpp:105-128): N need not be a multiple of the 256-column
    tile here.  The half-empty last tile must write nothing past column N (the row's successor starts there)."""
    _say(f"fp8 N={N} op={op}")
    gl = [3, 3, 40, 41] if op == "gemv" else [5, 140, 140, 301]
    case = H.make_case("fp8", len(gl), 512, N, gl, seed=N, extra_rows=2)
    got = H.run_cabi(case, H.upload(case), op)
    H.assert_close(got, H.oracle_out(case, gemv=op == "gemv"), rows=slice(0, gl[-1]), what=f"fp8 N={N} {op}")
    assert (got[gl[-1]:] == 0x7FC0).all()


@pytest.mark.parametrize("op", ["gemm", "gemv"])
@pytest.mark.parametrize("fmt", ["fp4", "fp8", "int8", "int4", "fp4_b32", "fp4_b16"])
def test_several_tiles_per_workgroup(fmt, op):
    """More tiles than the persistent grid has workgroups (256): every workgroup runs several tiles in a
    row, of different experts, row counts and column blocks, re-using its LDS ring."""
    if op == "gemv" and fmt not in H.GEMV_FORMATS:
        pytest.skip("the GEMV op has no such container")
    _say(f"several tiles per workgroup fmt={fmt} op={op}")
    rng = np.random.default_rng(zlib.crc32(f"tiles/{fmt}/{op}".encode()))
    G, K, N = 96, 256, 2048
    counts = rng.choice([0, 1, 3, 16, 17, 33, 40], G)
    gl = list(np.cumsum(counts))
    case = H.make_case(fmt, G, K, N, gl, seed=3, extra_rows=1, group=64)
    got = H.run_cabi(case, H.upload(case), op)
    H.assert_close(got, H.oracle_out(case, gemv=op == "gemv"), rows=slice(0, gl[-1]), what=f"tiles {fmt}/{op}")
    assert (got[gl[-1]:] == 0x7FC0).all()


@pytest.mark.parametrize("op", ["gemm", "gemv"])
@pytest.mark.parametrize("fmt", ["int4", "fp4"])
@pytest.mark.parametrize("shape", ["row_counts", "many_tiles"])
def test_decode_batches_on_the_small_tile_kinds(fmt, shape, op):
    """Batches of at most 12 rows per expert on average run the 4-bit N-contiguous containers in tiles of at most
    32 rows (the GEMV op on fp4: 16 rows, with the two scale groups of an MFMA stacked for tiles of at most 8),
    two workgroups per CU: experts of 0 to 70 rows (several row chunks per expert), and more tiles than the grid
    has workgroups."""
    _say(f"{op} small tiles fmt={fmt} {shape}")
    if shape == "row_counts":
        counts, K, N = [1, 0, 4, 5, 16, 17, 32, 33, 70, 0, 3, 8, 9, 7] + [0] * 8, 1024, 512
    else:
        rng = np.random.default_rng(zlib.crc32(f"small/{fmt}".encode()))
        counts, K, N = list(rng.choice([0] * 6 + [1, 3, 16, 17, 33, 40], 160)), 256, 2048
    gl = list(np.cumsum(counts))
    assert gl[-1] <= 12 * len(gl)
    case = H.make_case(fmt, len(gl), K, N, gl, seed=len(gl), extra_rows=2, group=64)
    got = H.run_cabi(case, H.upload(case), op)
    H.assert_close(got, H.oracle_out(case, gemv=op == "gemv"), rows=slice(0, gl[-1]), what=f"small tiles {op} {fmt}/{shape}")
    assert (got[gl[-1]:] == 0x7FC0).all()


def test_gemm_tile_counters_are_reused_and_taken_over_safely():
    """The persistent grid takes its last tiles from a counter in device memory; every launch uses one of 4096
    slots and raises the counter to a stamp that grows with every use of the slot, so whatever an earlier launch
    left there counts as nothing.  A launch misled by a slot's content would skip tiles (rows left unwritten).
    The library's launch number is moved (test hook) so that (1) slots are used again with the next stamp,
    (2) launches find their slot already stamped by a later launch and fall back to the fixed order, and (3) a
    launch has its slot taken over while it runs: its own result must still be right."""
    import moe_gfx950 as mg
    slots = 4096
    _say("gemm tile counters: reuse, late start, take-over")
    rng = np.random.default_rng(5)
    counts = rng.choice([0, 1, 3, 16, 17, 33], 40)
    gl = list(np.cumsum(counts))
    cases = [H.make_case(fmt, len(gl), 128, 2048, gl, seed=7 + i, group=64) for i, fmt in enumerate(("int4", "bf16"))]
    devs = [H.upload(c) for c in cases]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    p = lambda t: 0 if t is None else t.data_ptr()
    ys, argss = [], []
    for c, d in zip(cases, devs):
        y = torch.full((c["M"], c["N"]), 0x7FC0, dtype=torch.int16, device="cuda")
        ys.append(y)
        argss.append(mg.grouped_args(mg.format_from_compute_type(c["fmt"]), p(d["x"]), p(d["weight"]), p(d["scale"]),
                                     p(d["offset"]), p(d["group_list"]), p(y), c["M"], c["K"], c["N"], c["G"], c["scale_rows"]))

    def check(what):
        torch.cuda.synchronize()
        for c, y in zip(cases, ys):
            got = y.cpu().numpy().view(np.uint16)
            H.assert_close(got, H.oracle_out(c), rows=slice(0, gl[-1]), what=f"{what} {c['fmt']}")
            y.fill_(0x7FC0)
        torch.cuda.synchronize()

    def run(iters, what):
        for it in range(iters):
            for st, args in zip(streams, argss):
                mg.grouped_gemm(args, st.cuda_stream)
            if it in (0, iters - 1):
                check(f"{what}, launch {it}")

    torch.cuda.synchronize()
    try:
        run(300, "fresh slots")
        mg.lib.moe_test_shift_launch_number(slots - 600)
        run(300, "the same slots, next stamp")
        mg.lib.moe_test_shift_launch_number(-slots)
        run(20, "slots that a later launch has stamped")
        mg.lib.moe_test_shift_launch_number(2 * slots)
        run(2, "back to normal")
        # (3): A runs on one stream; the launch number is moved so that B, on another stream, gets A's slot with
        # the next stamp and starts as soon as A's first workgroups leave.  A's last draws then fail and its
        # workgroups finish their share in the fixed order.  Only A's result is defined.
        big = H.make_case("int4", 48, 1024, 2048, [128 * (g + 1) for g in range(48)], seed=3, group=128)
        dev = H.upload(big)
        ya = torch.full((big["M"], big["N"]), 0x7FC0, dtype=torch.int16, device="cuda")
        yb = torch.empty_like(ya)
        mk = lambda y: mg.grouped_args(mg.format_from_compute_type("int4"), p(dev["x"]), p(dev["weight"]), p(dev["scale"]), p(dev["offset"]),
                                       p(dev["group_list"]), p(y), big["M"], big["K"], big["N"], big["G"], big["scale_rows"])
        a_args, b_args = mk(ya), mk(yb)
        torch.cuda.synchronize()
        for rep in range(3):
            mg.grouped_gemm(a_args, streams[0].cuda_stream)
            mg.lib.moe_test_shift_launch_number(slots - 1)
            mg.grouped_gemm(b_args, streams[1].cuda_stream)
            torch.cuda.synchronize()
            H.assert_close(ya.cpu().numpy().view(np.uint16), H.oracle_out(big), what=f"launch whose slot is taken over, rep {rep}")
            ya.fill_(0x7FC0)
            torch.cuda.synchronize()
    finally:
        mg.lib.moe_test_shift_launch_number(2 * slots)   # past every stamp written above


def test_gemm_int4_group_size_32_and_64():
    for group in (32, 64, 256):
        _say(f"gemm int4 group={group}")
        case = H.make_case("int4", 3, 512, 256, [20, 20, 77], seed=group, group=group)
        got = H.run_cabi(case, H.upload(case), "gemm")
        H.assert_close(got, H.oracle_out(case), what=f"int4 group {group}")


def test_gemm_reference_fp4_test_shape_via_module():
    """The reference's own fp4 GEMM test (test_group_gemm_fp4.py:164-230): G=4, dim 256,
    block 16, the same weight for every expert, group_list [2,3,4,256], called with its
    keyword order; checked at the reference's atol 0.15 and at this project's bar."""
    import cinfer_ascendc

    _say("gemm reference fp4 test shape")
    dim, block, G = 256, 16, 4
    g = torch.Generator().manual_seed(0)
    b = torch.randn(dim, dim // block, block, generator=g)
    b_s_2 = b.abs().max() / (448 * 6)
    b_s = torch.clamp(b.amax(dim=2, keepdim=True) / (6 * b_s_2), -448, 448)
    levels = torch.tensor(L.E2M1_LEVELS)
    bq = b / (b_s * b_s_2)
    idx = (bq.abs().unsqueeze(-1) - levels).abs().argmin(-1)          # snap to the e2m1 grid
    codes = (idx.to(torch.uint8) | ((bq < 0).to(torch.uint8) << 3)).view(dim, dim).numpy()
    ckpt = np.repeat(L.pack_nibbles_last(codes)[None], G, 0)          # [G, N, K/2]
    scale_nk = (b_s.view(dim, dim // block) * b_s_2).to(torch.bfloat16)   # merged two-level scale, :86-94
    w1w3 = L.fp4ref_from_checkpoint(ckpt)
    new_scale = scale_nk.t().contiguous().unsqueeze(0).repeat(G, 1, 1)    # [G, K/16, N], :185-186
    x = torch.randn(dim, dim, generator=g).to(torch.bfloat16)
    expert_tokens = torch.tensor([2, 3, 4, 256], dtype=torch.int64)
    output = torch.zeros(dim, dim, dtype=torch.bfloat16, device="cuda")
    cinfer_ascendc.grouped_gemm(
        x.cuda(), torch.from_numpy(w1w3).cuda(), output=output,
        antiquantOffsetOptional=torch.zeros_like(new_scale).cuda(), antiquantScaleOptional=new_scale.cuda(),
        groupListOptional=expert_tokens.cuda(), computeType="fp4")
    torch.cuda.synchronize()
    # expected value exactly as the reference test builds it (:199-217), torch on the CPU
    lut = torch.tensor([0, .5, 1, 1.5, 2, 3, 4, 6, -0., -.5, -1, -1.5, -2, -3, -4, -6], dtype=torch.bfloat16)
    w = lut[torch.from_numpy(codes.astype(np.int64))]                                     # [N, K]
    for i in range(dim // block):
        w[:, i * block:(i + 1) * block] *= scale_nk[:, i].unsqueeze(-1)
    exp = (x.float() @ w.t().float()).to(torch.bfloat16)
    assert torch.allclose(exp, output.cpu(), atol=0.15)
    H.assert_close(H.bits(output), H.bits(exp), what="reference fp4 test")


def test_gemm_reference_fp8_test_shape_all_ones_x():
    """The reference's fp8 GEMM test (test_group_gemm_fp8.py:35-71): G=4, M=48, K=512,
    N=1536, x = ones, randn fp32 block scales, group_list [12,25,44,48]; with x = 1 the
    output is the column sums of the dequantized weight."""
    import cinfer_ascendc

    _say("gemm reference fp8 test shape")
    rng = np.random.default_rng(3)
    G, M, K, N = 4, 48, 512, 1536
    w = rng.integers(0, 255, (G, K, N), dtype=np.uint8)
    scale = rng.standard_normal((G, 4, 12)).astype(np.float32)
    gl = [12, 25, 44, 48]
    out = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
    scale_d = torch.from_numpy(scale).cuda()
    cinfer_ascendc.grouped_gemm(
        torch.ones(M, K, dtype=torch.bfloat16, device="cuda"), torch.from_numpy(w).cuda(), output=out,
        antiquantOffsetOptional=torch.zeros_like(scale_d), antiquantScaleOptional=scale_d,
        groupListOptional=torch.tensor(gl).cuda(), computeType="fp8")
    torch.cuda.synchronize()
    Wd = L.fp8ref_dequant_numpy(w, scale, True).astype(np.float64)
    exp = np.zeros((M, N))
    prev = 0
    for g, end in enumerate(gl):
        exp[prev:end] = Wd[g].sum(0)
        prev = end
    got = out.float().cpu().numpy()
    assert np.allclose(got, exp, atol=0.02 + 2 ** -8 * np.abs(exp).max())   # reference atol + one bf16 ulp
    H.assert_close(H.bits(out), oracle.f32_to_bf16_bits(exp.astype(np.float32)), what="reference fp8 test")


def test_gemm_linearity_and_determinism():
    # y(x1 + x2) == y(x1) + y(x2) up to rounding; two launches give identical bits
    _say("gemm linearity")
    gl = [100, 260, 300]
    case = H.make_case("int4", 3, 1024, 512, gl, seed=5)
    dev = H.upload(case)
    y1 = H.run_cabi(case, dev, "gemm")
    assert np.array_equal(y1, H.run_cabi(case, dev, "gemm"))
    case2 = dict(case)
    x2 = oracle.f32_to_bf16_bits(oracle.bf16_bits_to_f32(case["x"]) * 2.0)   # exact scaling by 2
    case2["x"] = x2
    y2 = H.run_cabi(case2, H.upload(case2), "gemm")
    assert np.array_equal(oracle.bf16_bits_to_f32(y2), 2.0 * oracle.bf16_bits_to_f32(y1))


# ------------------------------------------------------------------------ grouped GEMV
GEMV_GROUP_LISTS = {
    "ref": [1, 2, 3, 4],                       # test_group_soft_gemv_fp4.py:172
    "ragged": [0, 4, 4, 6, 7, 7, 11],
    "more_than_4": [9, 9, 10],                 # beyond the reference's MAX_BSZ: rows taken 4 at a time
    "all_empty": [0, 0],
}


@pytest.mark.parametrize("fmt", H.GEMV_FORMATS)
@pytest.mark.parametrize("gl_name", list(GEMV_GROUP_LISTS))
def test_gemv_parity_small(fmt, gl_name):
    gl = GEMV_GROUP_LISTS[gl_name]
    G, K, N = len(gl), 1024, 512
    _say(f"gemv fmt={fmt} gl={gl_name}")
    case = H.make_case(fmt, G, K, N, gl, seed=zlib.crc32(f"gemv/{fmt}/{gl_name}".encode()) % 1000, extra_rows=3)
    got = H.run_cabi(case, H.upload(case), "gemv")
    ref = H.oracle_out(case, gemv=True)
    H.assert_close(got, ref, rows=slice(0, gl[-1]), what=f"gemv {fmt}/{gl_name}")
    assert (got[gl[-1]:] == 0x7FC0).all()


@pytest.mark.parametrize("fmt,K,N", [("bf16", 7168, 2048), ("fp4_b32", 7168, 2048), ("fp4", 7168, 512),
                                     ("fp8", 7168, 256), ("bf16", 9216, 200), ("fp4_b32", 16384, 64)])
def test_gemv_parity_decode_shapes(fmt, K, N):
    _say(f"gemv decode fmt={fmt} K={K} N={N}")
    gl = [3, 3, 7, 8]
    case = H.make_case(fmt, 4, K, N, gl, seed=K % 97)
    got = H.run_cabi(case, H.upload(case), "gemv")
    H.assert_close(got, H.oracle_out(case, gemv=True), what=f"gemv {fmt} K={K} N={N}")


@pytest.mark.parametrize("fmt", ["fp4_b32", "fp4_b16"])
@pytest.mark.parametrize("K,N", [(1024, 256), (7168, 256), (8192 + 512, 256), (192, 256)])
def test_gemv_fp4_b32_row_counts_up_to_and_beyond_16(K, N, fmt):
    """The K-contiguous fp4 GEMV (scales per 32 or per 16 k) multiplies up to 16 rows of an expert per pass on the matrix cores (staging
    4, 8 or 16 rows) and takes more rows 16 at a time; K = 192 is not a multiple of 512 and goes
    through the vector path."""
    _say(f"gemv {fmt} rows K={K} N={N}")
    counts = [1, 0, 4, 5, 8, 9, 16, 17, 40, 0, 3]
    gl = list(np.cumsum(counts))
    case = H.make_case(fmt, len(gl), K, N, gl, seed=K + N, extra_rows=2)
    dev = H.upload(case)
    got = H.run_cabi(case, dev, "gemv")
    H.assert_close(got, H.oracle_out(case, gemv=True), rows=slice(0, gl[-1]), what=f"gemv {fmt} rows K={K} N={N}")
    assert (got[gl[-1]:] == 0x7FC0).all()
    if K % 128:
        return  # the GEMM op takes these containers with K % 128 == 0 only
    # the grouped GEMM op at these sizes runs the same kernel with the GEMM's weight rounding
    got = H.run_cabi(case, dev, "gemm")
    H.assert_close(got, H.oracle_out(case), rows=slice(0, gl[-1]), what=f"gemm {fmt} rows K={K} N={N}")
    assert (got[gl[-1]:] == 0x7FC0).all()


@pytest.mark.parametrize("fmt,K,N,group", [("fp4", 1024, 256, 16), ("fp4", 7168, 512, 16), ("fp4", 64, 256, 16),
                                           ("int4", 1024, 256, 128), ("int4", 7168, 512, 128), ("int4", 192, 256, 32),
                                           ("int4", 256, 256, 64), ("fp8", 1024, 256, 128), ("fp8", 7168, 512, 128),
                                           ("fp8", 128, 256, 128)])
def test_gemv_n_contiguous_row_counts_up_to_and_beyond_32(fmt, K, N, group):
    """The GEMV op on the reference fp4 / fp8 containers and on int4 runs on the matrix cores with weights
    that are not rounded to bf16 (the codes go through the MFMA, the fp32 scales are applied to its
    results), in tiles of up to 32 rows of an expert; K = 64 (fp8: 128) is a single scale block."""
    _say(f"gemv {fmt} rows K={K} N={N} group={group}")
    counts = [1, 0, 4, 5, 16, 17, 32, 33, 70, 0, 3]
    gl = list(np.cumsum(counts))
    case = H.make_case(fmt, len(gl), K, N, gl, seed=K + N + group, extra_rows=2, group=group)
    got = H.run_cabi(case, H.upload(case), "gemv")
    H.assert_close(got, H.oracle_out(case, gemv=True), rows=slice(0, gl[-1]), what=f"gemv {fmt} rows K={K} N={N}")
    assert (got[gl[-1]:] == 0x7FC0).all()


@pytest.mark.parametrize("fmt,op,G,style", [
    ("int4", "gemv", 2100, "decode"), ("fp4", "gemv", 2100, "decode"), ("fp8", "gemv", 2100, "decode"),
    ("int4", "gemm", 2100, "decode"), ("int4", "gemm", 2100, "prefill"),
    # beyond what LDS holds a table for (about 3000 experts next to the small stages, 2700 / 5000 next to the large)
    ("int4", "gemv", 6000, "decode"), ("int4", "gemm", 6000, "decode"), ("fp8", "gemv", 6000, "decode"),
    ("int4", "gemm", 6000, "prefill"), ("fp4", "gemm", 6000, "prefill"), ("int8", "gemm", 6000, "prefill"),
    ("fp4_b32", "gemm", 6000, "prefill"), ("bf16", "gemm", 12000, "decode")])
def test_any_number_of_experts(fmt, op, G, style):
    """The grouped GEMM kernels keep the first tile of every expert in LDS while that fits; with more experts (the
    reference loops over any number, grouped_gemm/op_kernel/grouped_matmul_antiquant.h:241-242) they keep one entry
    per thread and walk group_list from there.  Empty experts, experts of several row chunks and rows past
    group_list[-1] included."""
    _say(f"{op} {fmt} G={G} {style}")
    rng = np.random.default_rng(G)
    if style == "decode":
        counts = rng.integers(0, 3, G)
        counts[[3, G // 2, G - 2]] = [5, 9, 4]
    else:
        counts = rng.integers(0, 30, G)                      # on average more than 12 rows per expert
        counts[[3, G // 2, G - 2]] = [170, 400, 33]
    gl = list(np.cumsum(counts))
    K, N = (64, 256) if fmt == "bf16" else (128, 256)
    case = H.make_case(fmt, G, K, N, gl, seed=12, group=32 if fmt == "int4" else 128 if fmt == "fp8" else 16, extra_rows=3)
    got = H.run_cabi(case, H.upload(case), op)
    H.assert_close(got, H.oracle_out(case, gemv=op == "gemv"), rows=slice(0, gl[-1]), what=f"{op} {fmt} G={G}")
    assert (got[gl[-1]:] == 0x7FC0).all()


@pytest.mark.parametrize("fmt,tiles", [("int4", 511), ("int4", 512), ("int4", 513), ("int4", 1023), ("int4", 1025), ("int4", 1537),
                                       ("int8", 255), ("int8", 257), ("int8", 513), ("int8", 769)])
def test_tile_counts_around_the_grid_size(fmt, tiles):
    """The persistent grid is 512 workgroups for the 4-wavefront kind (int4 prefill) and 256 for the 8-wavefront kind
    (int8) on a 256-CU part.  Launches of at most one tile per workgroup use no tile counter, larger ones run at least
    one sweep in the fixed order before the first draw, and a launch without a counter deals its last, partial sweep out
    in launch order: tile counts on either side of one, two and three sweeps, eagerly and replayed from a graph."""
    _say(f"tile counts around the grid size: {fmt} {tiles} tiles")
    G = tiles                                            # one 16-row chunk x one 256-column tile per expert
    gl = list(16 * np.arange(1, G + 1))                  # 16 rows per expert: more than 12 on average, so the prefill kinds run
    case = H.make_case(fmt, G, 128, 256, gl, seed=tiles, group=32, extra_rows=2)
    dev = H.upload(case)
    ref = H.oracle_out(case)
    got = H.run_cabi(case, dev, "gemm")
    H.assert_close(got, ref, rows=slice(0, gl[-1]), what=f"{fmt} {tiles} tiles, eager")
    assert (got[gl[-1]:] == 0x7FC0).all()
    # the same launch captured (no counter: every tile in the fixed order) and replayed twice
    import moe_gfx950 as mg
    p = lambda t: 0 if t is None else t.data_ptr()
    y = torch.full((case["M"], case["N"]), 0x7FC0, dtype=torch.int16, device="cuda")
    args = mg.grouped_args(mg.format_from_compute_type(fmt), p(dev["x"]), p(dev["weight"]), p(dev["scale"]), p(dev["offset"]),
                           p(dev["group_list"]), p(y), case["M"], case["K"], case["N"], case["G"], case["scale_rows"])
    st = torch.cuda.Stream()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(st):
        with torch.cuda.graph(g, stream=st):
            mg.grouped_gemm(args, st.cuda_stream)
    for rep in range(2):
        y.fill_(0x7FC0)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        got = y.cpu().numpy().view(np.uint16)
        H.assert_close(got, ref, rows=slice(0, gl[-1]), what=f"{fmt} {tiles} tiles, replay {rep}")
        assert (got[gl[-1]:] == 0x7FC0).all()


@pytest.mark.parametrize("fmt,N", [("int8", 512), ("fp8", 512), ("fp8", 384)])
def test_one_byte_containers_with_many_rows_per_expert(fmt, N):
    """int8 and the reference's fp8 run on the 4-wavefront kind (two workgroups per CU, no k split) once an expert has
    more rows than one tile takes on average: every row-block count of its tiles, several row chunks per expert, empty
    experts, ragged last blocks, and for fp8 a half-empty last column tile."""
    _say(f"{fmt} N={N} on the 4-wavefront kind")
    counts = [400, 0, 333, 161, 170, 529, 16, 1, 320, 200, 0, 145, 159, 160, 97]
    gl = list(np.cumsum(counts))
    assert gl[-1] > 160 * len(gl)
    case = H.make_case(fmt, len(gl), 512, N, gl, seed=31 + N, extra_rows=3)
    got = H.run_cabi(case, H.upload(case), "gemm")
    H.assert_close(got, H.oracle_out(case), rows=slice(0, gl[-1]), what=f"{fmt} N={N}, many rows per expert")
    assert (got[gl[-1]:] == 0x7FC0).all()


def test_gemv_reference_fp8_test_shape_via_module():
    """test_group_soft_gemv_fp8.py:37-88: G=4, M=4, K=512, N=1536, x = ones, expected value
    from fp32 (un-rounded) weights, rtol 0.02."""
    import cinfer_ascendc

    _say("gemv reference fp8 test shape")
    rng = np.random.default_rng(4)
    G, M, K, N = 4, 4, 512, 1536
    w = rng.integers(0, 255, (G, K, N), dtype=np.uint8)
    scale = rng.standard_normal((G, 4, 12)).astype(np.float32)
    out = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
    cinfer_ascendc.grouped_soft_gemv(torch.ones(M, K, dtype=torch.bfloat16, device="cuda"), torch.from_numpy(w).cuda(),
                                     output=out, scale=torch.from_numpy(scale).cuda(),
                                     groupList=torch.tensor([1, 2, 3, 4]).cuda(), computeType="fp8")
    torch.cuda.synchronize()
    Wd = L.fp8ref_dequant_numpy(w, scale, False).astype(np.float64)
    exp = np.stack([Wd[g].sum(0) for g in range(G)])
    exp_bf16 = torch.from_numpy(exp.astype(np.float32)).to(torch.bfloat16)
    assert torch.allclose(out.cpu(), exp_bf16, rtol=0.02, atol=2 ** -8 * float(np.abs(exp).max()))
    H.assert_close(H.bits(out), H.bits(exp_bf16), what="reference gemv fp8 test")


def test_gemv_matches_gemm_on_the_same_inputs():
    # the two ops differ only in weight rounding; on bf16 weights they must agree to rounding
    _say("gemv vs gemm bf16")
    case = H.make_case("bf16", 4, 2048, 256, [2, 2, 5, 9], seed=6)
    dev = H.upload(case)
    a, b = H.run_cabi(case, dev, "gemv"), H.run_cabi(case, dev, "gemm")
    H.assert_close(a, b, what="gemv vs gemm")


# -------------------------------------------------- error behaviour through the module
@pytest.mark.parametrize("gl_name,gl", [("decode", [3, 3, 7, 9]), ("prefill", [40, 90, 130, 200])])
@pytest.mark.parametrize("fmt", ["int4", "fp4", "fp8", "fp4_b32", "fp4_b16"])
def test_each_op_uses_its_own_weight_rounding(fmt, gl_name, gl):
    """The GEMM op multiplies weights rounded to bf16 (the reference's phase 1), the GEMV op un-rounded fp32
    weights (gemv_impl.h:147-199).  The two differ by about a quarter of an output ulp, far inside the parity
    tolerance, so they are told apart by counting outputs whose bf16 bits differ: against the oracle of its own
    arithmetic an op differs only where the summation order moves a sum across a rounding boundary, against the
    other arithmetic in a sizeable share of the outputs.  Covers every dispatch: k-split tiles, the matrix-core
    GEMV kernels run with either rounding, decode and prefill sized batches."""
    _say(f"rounding fmt={fmt} gl={gl_name}")
    case = H.make_case(fmt, len(gl), 2048, 512, gl, seed=len(fmt) + gl[0])
    dev = H.upload(case)
    ref = {False: H.oracle_out(case, gemv=False), True: H.oracle_out(case, gemv=True)}
    apart = float(np.mean(ref[False] != ref[True]))
    assert apart > 0.03, "the case does not separate the two arithmetics"
    for op in ("gemm", "gemv"):
        got = H.run_cabi(case, dev, op)
        own = float(np.mean(got != ref[op == "gemv"]))
        other = float(np.mean(got != ref[op != "gemv"]))
        assert own < 0.25 * other, f"{fmt}/{op}: {own:.4f} of the outputs differ from its own arithmetic, {other:.4f} from the other"


def test_module_errors_on_gpu_tensors():
    import cinfer_ascendc

    x = torch.zeros(4, 256, dtype=torch.bfloat16, device="cuda")
    w = torch.zeros(2, 256, 128, dtype=torch.int8, device="cuda")
    s = torch.zeros(2, 16, 256, dtype=torch.bfloat16, device="cuda")
    gl = torch.tensor([2, 4], device="cuda")
    y = torch.zeros(4, 256, dtype=torch.bfloat16, device="cuda")
    cinfer_ascendc.grouped_gemm(x, w, s, s, gl, "fp4", y)          # valid call
    with pytest.raises(RuntimeError, match="Invalid compute type"):
        cinfer_ascendc.grouped_gemm(x, w, s, s, gl, "fp5", y)
    with pytest.raises(RuntimeError, match="shape"):
        cinfer_ascendc.grouped_gemm(x, w, s[:, :8].contiguous(), s, gl, "fp4", y)
    with pytest.raises(RuntimeError, match="dtype"):
        cinfer_ascendc.grouped_gemm(x.float(), w, s, s, gl, "fp4", y)
    with pytest.raises(RuntimeError, match="contiguous"):
        cinfer_ascendc.grouped_gemm(x, w, s, s, gl, "fp4", torch.zeros(256, 4, dtype=torch.bfloat16, device="cuda").t())
    with pytest.raises(RuntimeError, match="alignment"):
        cinfer_ascendc.grouped_gemm(torch.zeros(4, 96, dtype=torch.bfloat16, device="cuda"),
                                    torch.zeros(2, 96, 128, dtype=torch.int8, device="cuda"),
                                    torch.zeros(2, 6, 256, dtype=torch.bfloat16, device="cuda"), s, gl, "fp4", y)
    torch.cuda.synchronize()
