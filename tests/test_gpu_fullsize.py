"""The benchmark configurations at their full sizes on the GPU.  The oracle checks a sample
(whole experts, so that every tile shape of those experts is covered, and a few rows of many
more experts spread over the list, so that every part of the tile order is); size-independent
properties cover the rest: exact linearity in x, determinism, untouched trailing rows, and
agreement between the fused and the separate FP4 paths."""
import numpy as np
import pytest
import torch

import helpers as H
import oracle

pytestmark = pytest.mark.gpu


def _say(msg):
    print(msg, flush=True)


def _bf16_normal(shape, std=1.0):
    return (torch.randn(shape, device="cuda") * std).to(torch.bfloat16)


def _bf16_uniform(shape, lo, hi):
    return (torch.rand(shape, device="cuda") * (hi - lo) + lo).to(torch.bfloat16)


def _routed(tokens, experts, topk, gen):
    logits = torch.randn(tokens, experts, generator=gen)
    ids = logits.topk(topk, dim=1).indices.reshape(-1)
    return torch.bincount(ids, minlength=experts)


def _launch(op, fmt, x, w, s, o, gl, y, scale_rows=1):
    import moe_gfx950 as mg

    p = lambda t: 0 if t is None else t.data_ptr()
    if fmt in ("fp4_b32", "bf16"):
        N, K = w.shape[1], x.shape[1]
    else:
        K, N = x.shape[1], y.shape[1]
    args = mg.grouped_args(mg.format_from_compute_type(fmt), p(x), p(w), p(s), p(o), p(gl), p(y), x.shape[0], K, N,
                           gl.shape[0], scale_rows)
    (mg.grouped_gemm if op == "gemm" else mg.grouped_gemv)(args, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()


def _replayed(op, fmt, x, w, s, o, gl, y, scale_rows=1):
    """The same call captured into a HIP graph (no tile counter: every tile in the fixed order) and replayed into y."""
    import moe_gfx950 as mg

    p = lambda t: 0 if t is None else t.data_ptr()
    K, N = x.shape[1], y.shape[1]
    args = mg.grouped_args(mg.format_from_compute_type(fmt), p(x), p(w), p(s), p(o), p(gl), p(y), x.shape[0], K, N,
                           gl.shape[0], scale_rows)
    st = torch.cuda.Stream()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(st):
        with torch.cuda.graph(g, stream=st):
            (mg.grouped_gemm if op == "gemm" else mg.grouped_gemv)(args, st.cuda_stream)
    g.replay()
    torch.cuda.synchronize()


def _oracle_subset(fmt, x, w, s, o, counts, experts, gemv=False):
    """Oracle output for the rows of the chosen experts only (a reduced problem built from the
    device tensors): returns (row indices into the full problem, bf16 bits [rows, N])."""
    starts = torch.cumsum(counts, 0) - counts
    rows = torch.cat([torch.arange(int(starts[g]), int(starts[g] + counts[g])) for g in experts])
    gl_sub = np.cumsum([int(counts[g]) for g in experts]).astype(np.int64)
    xb = H.bits(x[rows.cuda()])
    cpu = lambda t: None if t is None else t[torch.tensor(experts).cuda()].cpu()
    wc, sc, oc = cpu(w), cpu(s), cpu(o)
    as_np = lambda t: None if t is None else (H.bits(t) if t.dtype == torch.bfloat16 else t.numpy())
    ref = oracle.grouped_gemm(oracle.FMT_BY_NAME[fmt], xb, as_np(wc), as_np(sc), as_np(oc), gl_sub, round_bf16=not gemv)
    return rows, ref


def _oracle_rows(fmt, x, w, s, o, counts, picks, gemv=False):
    """Oracle output for a few rows of many experts: picks maps an expert to row offsets within it.  A reduced
    problem (those experts, those rows) built from the device tensors; returns (row indices into the full
    problem, bf16 bits [rows, N])."""
    starts = torch.cumsum(counts, 0) - counts
    experts = sorted(picks)
    rows = torch.tensor([int(starts[g]) + r for g in experts for r in picks[g]])
    gl_sub = np.cumsum([len(picks[g]) for g in experts]).astype(np.int64)
    xb = H.bits(x[rows.cuda()])
    cpu = lambda t: None if t is None else t[torch.tensor(experts).cuda()].cpu()
    as_np = lambda t: None if t is None else (H.bits(t) if t.dtype == torch.bfloat16 else t.numpy())
    ref = oracle.grouped_gemm(oracle.FMT_BY_NAME[fmt], xb, as_np(cpu(w)), as_np(cpu(s)), as_np(cpu(o)), gl_sub,
                              round_bf16=not gemv)
    return rows, ref


def _spread_picks(counts, n_experts, rng):
    """First row, last row and one row in between of n_experts experts spread evenly over the list (so that tiles
    of every part of the tile order, fixed sweeps and work-counter tail alike, are sampled)."""
    G = counts.shape[0]
    picks = {}
    for g in np.linspace(0, G - 1, n_experts).round().astype(int):
        m = int(counts[g])
        if m > 0:
            picks[int(g)] = sorted({0, m - 1, int(rng.integers(0, m))})
    return picks


def test_dsv3_int4_prefill_gate_up_and_down():
    _say("full size: DSV3 int4 prefill")
    gen = torch.Generator().manual_seed(0)
    torch.manual_seed(0)
    G, tokens, topk = 256, 4096, 8
    counts = _routed(tokens, G, topk, gen)
    gl = counts.cumsum(0).to(torch.int64).cuda()
    M = tokens * topk
    # experts to check against the oracle: the smallest, the largest and two more
    order = torch.argsort(counts)
    experts = sorted({int(order[0]), int(order[-1]), 7, 200})
    for name, K, N in (("gate_up", 7168, 4096), ("down", 2048, 7168)):
        _say(f"  {name} K={K} N={N}, oracle on experts {experts} with {[int(counts[g]) for g in experts]} rows")
        x = _bf16_normal((M + 3, K))                      # 3 trailing rows beyond group_list[-1]
        w = torch.randint(0, 256, (G, K, N // 2), dtype=torch.uint8, device="cuda")
        s = _bf16_uniform((G, K // 128, N), 1e-3, 1e-2)
        y = torch.full((M + 3, N), float("nan"), dtype=torch.bfloat16, device="cuda")
        _launch("gemm", "int4", x, w, s, None, gl, y, K // 128)
        assert torch.isnan(y[M:]).all() and not torch.isnan(y[:M]).any()
        rows, ref = _oracle_subset("int4", x, w, s, None, counts, experts)
        H.assert_close(H.bits(y[rows.cuda()]), ref, what=f"int4 {name}")
        # and a few rows of 40 more experts spread over the whole list
        picks = _spread_picks(counts, 40, np.random.default_rng(K))
        rows, ref = _oracle_rows("int4", x, w, s, None, counts, picks)
        H.assert_close(H.bits(y[rows.cuda()]), ref, what=f"int4 {name}, rows of {len(picks)} experts")
        # determinism and exact linearity: y(2x) == 2 y(x) bit for bit (scaling by 2 is exact)
        y2 = torch.empty_like(y)
        _launch("gemm", "int4", x, w, s, None, gl, y2, K // 128)
        assert torch.equal(y[:M].view(torch.int16), y2[:M].view(torch.int16))
        # the order of the tiles does not enter the results: replayed from a graph (fixed order, no work counter)
        y2.fill_(float("nan"))
        _replayed("gemm", "int4", x, w, s, None, gl, y2, K // 128)
        assert torch.equal(y[:M].view(torch.int16), y2[:M].view(torch.int16)) and torch.isnan(y2[M:]).all()
        _launch("gemm", "int4", (x.float() * 2).to(torch.bfloat16), w, s, None, gl, y2, K // 128)
        assert torch.equal((y[:M].float() * 2), y2[:M].float())
        del x, w, s, y, y2
        torch.cuda.empty_cache()


def test_int8_grouped_gemm_8_experts():
    _say("full size: int8 grouped GEMM, 8 experts")
    torch.manual_seed(1)
    G, M, K, N = 8, 4096, 4096, 14336
    counts = torch.distributions.Multinomial(M, torch.full((G,), 1.0 / G)).sample().to(torch.int64)
    gl = counts.cumsum(0).cuda()
    x = _bf16_normal((M, K))
    w = torch.randint(-127, 128, (G, K, N), dtype=torch.int8, device="cuda")
    s, o = _bf16_uniform((G, N), 1e-3, 1e-2), _bf16_uniform((G, N), -2.0, 2.0)
    y = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    _launch("gemm", "int8", x, w, s, o, gl, y)
    rows, ref = _oracle_subset("int8", x, w, s, o, counts, [int(torch.argmin(counts))])
    H.assert_close(H.bits(y[rows.cuda()]), ref, what="int8")
    # rows of every expert: first, last, and some of every 128-row chunk in between
    picks = {g: sorted({0, int(counts[g]) - 1, *range(5, int(counts[g]), 61)}) for g in range(G)}
    rows, ref = _oracle_rows("int8", x, w, s, o, counts, picks)
    H.assert_close(H.bits(y[rows.cuda()]), ref, what="int8, rows of all experts")


def test_grouped_gemv_64_experts_bf16():
    _say("full size: grouped GEMV, 64 experts, bf16 weights")
    gen = torch.Generator().manual_seed(2)
    torch.manual_seed(2)
    G, K, N = 64, 7168, 2048
    while True:
        counts = _routed(4, G, 8, gen)
        if int(counts.max()) <= 4:
            break
    gl = counts.cumsum(0).to(torch.int64).cuda()
    M = int(counts.sum())
    x = _bf16_normal((M, K))
    w = _bf16_normal((G, N, K), 0.02)
    y = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    _launch("gemv", "bf16", x, w, None, None, gl, y)
    active = [g for g in range(G) if int(counts[g]) > 0]
    rows, ref = _oracle_subset("bf16", x, w, None, None, counts, active, gemv=True)
    assert len(rows) == M
    H.assert_close(H.bits(y[rows.cuda()]), ref, what="gemv bf16")


def test_fused_fp4_decode_against_separate_path_and_oracle():
    _say("full size: fused FP4 grouped GEMM at decode shape vs dequant + bf16 GEMM")
    import moe_gfx950 as mg

    gen = torch.Generator().manual_seed(3)
    torch.manual_seed(3)
    G, K, N = 256, 7168, 2048
    counts = _routed(64, G, 8, gen)
    gl = counts.cumsum(0).to(torch.int64).cuda()
    M = int(counts.sum())
    x = _bf16_normal((M, K))
    w = torch.randint(0, 256, (G, N, K // 2), dtype=torch.uint8, device="cuda")
    # both paths multiply the same bf16-rounded weights (the grouped GEMM op rounds code*scale to
    # bf16 like the reference's antiquant phase), so they differ only in summation order; the
    # GEMV op on the same inputs keeps fp32 weights and is checked against that arithmetic
    s = _bf16_uniform((G, N, K // 32), 2.0 ** -8, 2.0 ** -2)
    y_fused = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    _launch("gemm", "fp4_b32", x, w, s, None, gl, y_fused)
    wd = torch.empty(G, N, K, dtype=torch.bfloat16, device="cuda")
    mg.dequant_fp4_bf16(w.data_ptr(), s.data_ptr(), wd.data_ptr(), G * N, K, 32, torch.cuda.current_stream().cuda_stream)
    y_sep = torch.empty_like(y_fused)
    _launch("gemm", "bf16", x, wd, None, None, gl, y_sep)
    H.assert_close(H.bits(y_fused), H.bits(y_sep), what="fused vs separate")
    experts = [int(torch.argmax(counts)), int(torch.nonzero(counts > 0)[0])]
    rows, ref = _oracle_subset("fp4_b32", x, w, s, None, counts, sorted(set(experts)))
    H.assert_close(H.bits(y_fused[rows.cuda()]), ref, what="fused fp4 GEMM vs oracle")
    y_gemv = torch.empty_like(y_fused)
    _launch("gemv", "fp4_b32", x, w, s, None, gl, y_gemv)
    rows, ref = _oracle_subset("fp4_b32", x, w, s, None, counts, sorted(set(experts)), gemv=True)
    H.assert_close(H.bits(y_gemv[rows.cuda()]), ref, what="fp4 GEMV vs oracle")
    # the dequantized copy itself is bit-exact for one expert
    g = experts[0]
    ref_w = oracle.dequant_fp4_bf16(w[g].cpu().numpy(), H.bits(s[g].cpu()), 32)
    assert np.array_equal(H.bits(wd[g].cpu()), ref_w)


@pytest.mark.parametrize("fmt", ["fp4", "int4", "fp8"])
def test_decode_batch_on_the_n_contiguous_containers(fmt):
    """256 experts of 7168 x 2048, 512 routed rows, through both ops on the reference's own containers and on
    int4: the small-tile kinds with two workgroups per CU and tiles taken from the work counter.  The oracle
    checks whole experts (the largest, the first and the last with rows); every other row must agree between
    the two ops up to the rounding of the weights, be finite, and rows past group_list[-1] stay untouched."""
    _say(f"full size: decode batch on {fmt}")
    gen = torch.Generator().manual_seed(11)
    torch.manual_seed(11)
    G, K, N = 256, 7168, 2048
    counts = _routed(64, G, 8, gen)
    gl = counts.cumsum(0).to(torch.int64).cuda()
    M = int(counts.sum())
    x = _bf16_normal((M + 3, K))
    if fmt == "fp8":
        w = torch.randint(0, 255, (G, K, N), dtype=torch.uint8, device="cuda")
        s = torch.rand((G, K // 128, N // 128), device="cuda") * 1e-2 + 1e-3
        srows = K // 128
    else:
        group = 16 if fmt == "fp4" else 128
        w = torch.randint(0, 256, (G, K, N // 2), dtype=torch.uint8, device="cuda")
        w = w.view(torch.int8) if fmt == "fp4" else w
        s = _bf16_uniform((G, K // group, N), 2.0 ** -8, 2.0 ** -2)
        srows = K // group
    active = torch.nonzero(counts > 0).flatten().tolist()
    experts = sorted({int(torch.argmax(counts)), active[0], active[-1]})
    ys = {}
    for op in ("gemm", "gemv"):
        y = torch.full((M + 3, N), float("nan"), dtype=torch.bfloat16, device="cuda")
        _launch(op, fmt, x, w, s, None, gl, y, scale_rows=srows)
        assert torch.isnan(y[M:]).all(), "rows beyond group_list[-1] were written"
        assert torch.isfinite(y[:M].float()).all()
        rows, ref = _oracle_subset(fmt, x, w, s, None, counts, experts, gemv=op == "gemv")
        H.assert_close(H.bits(y[rows.cuda()]), ref, what=f"{fmt} {op} vs oracle")
        y2 = torch.full_like(y, float("nan"))
        _replayed(op, fmt, x, w, s, None, gl, y2, scale_rows=srows)
        assert torch.equal(y[:M].view(torch.int16), y2[:M].view(torch.int16)) and torch.isnan(y2[M:]).all(), "graph replay differs"
        del y2
        ys[op] = y[:M]
    # the ops differ by the rounding of the weights to bf16 (2^-9 per weight, summed over K = 7168): small against
    # the largest outputs, not against every single one
    rel, _ = H.compare(H.bits(ys["gemm"]), H.bits(ys["gemv"]))
    assert rel <= H.REL_TOL, f"{fmt}: GEMM op vs GEMV op rel {rel:.3e}"
