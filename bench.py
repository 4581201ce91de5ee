#!/usr/bin/env python3
"""Benchmark of the MoE antiquant ops on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload dsv3_int4_prefill] [--no-extra] [--no-cpu]
                    [--only headline|dequant|route|gemv_bf16|gemm_int8|fused_fp4|reference_containers|prepack]

A step is one pass of the hot path over one batch of synthetic input that is already
resident in HBM.  The headline workload is the DeepSeek-V3-shaped int4-antiquant MoE
prefill: 256 experts, 4096 tokens x top-8 = 32768 sorted rows, gate_up (K=7168, N=4096)
followed by down (K=2048, N=7168), int4 weights with zero point 8 and bf16 per-group-128
scales.  One JSON line is printed: whole-step TFLOP/s, the roofline of the dominant kernel
(measured with events on the launch stream), the CPU baselines (a torch restatement of the
reference's host-side check and the C oracle, timed on bounded samples), and -- unless --no-extra -- the other benchmark configurations
(FP4 dequant, grouped GEMV, int8 GEMM, fused FP4 GEMM at decode shape vs dequant + bf16
GEMM) as GB/s or TFLOP/s with their own roofline fractions.

Everything on the GPU goes through the C ABI of libmoe_gfx950.so; the oracle is used only
for the cpu_baseline figure.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "ascend-kernel_amd"))
sys.path.insert(0, ROOT)

PEAK_HBM_GBS = 8000.0        # MI355X HBM3E, 8 TB/s
PEAK_BF16_TFLOPS = 2500.0    # MI355X dense bf16 MFMA, 2.5 PFLOP/s
# HBM bytes per launch of the int4 grouped GEMM on this workload (mean of the gate_up and down launches) are
# not something a timing run can see: they come from two rocprofv3 --pmc runs of this script (FETCH_SIZE,
# WRITE_SIZE), scaled by the --copy-calibration copy.  The figure, the kernel it was taken on and the summary
# it comes from are kept in this file next to the profile summaries.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "grouped_gemm_int4_dsv3_prefill_hbm_traffic.json")


def measured_traffic():
    """(bytes per launch, provenance) from the committed counter summary, or (None, None)."""
    try:
        with open(TRAFFIC_FILE) as f:
            t = json.load(f)
        return float(t["hbm_bytes_per_launch"]), {k: t[k] for k in ("source", "measured_on", "kernel") if k in t}
    except (OSError, ValueError, KeyError):
        return None, None


def board_state():
    """Socket power (W) and mean shader clock over the XCDs (MHz) as amd-smi reports them right now, or Nones."""
    import re
    import subprocess
    try:
        out = subprocess.run(["/opt/rocm/bin/amd-smi", "metric", "-p", "-c"], capture_output=True, text=True, timeout=30).stdout
        p = re.search(r"SOCKET_POWER: *(\d+) *W", out)
        clk = [int(v) for v in re.findall(r"GFX_\d+:\s*\n\s*CLK: *(\d+) *MHz", out)]
        return (int(p.group(1)) if p else None), (sum(clk) / len(clk) if clk else None)
    except Exception:  # noqa: BLE001
        return None, None


def routed_counts(torch, tokens, experts, topk, gen, max_rows=None):
    """Rows per expert for top-k routing of softmax(N(0,1)) logits (softmax is monotone)."""
    while True:
        logits = torch.randn(tokens, experts, generator=gen)
        ids = logits.topk(topk, dim=1).indices.reshape(-1)
        counts = torch.bincount(ids, minlength=experts)
        if max_rows is None or int(counts.max()) <= max_rows:
            return counts


class Op:
    """One launch of a grouped op through the C ABI with fixed device tensors."""

    def __init__(self, mg, torch, op, fmt, x, w, scale, offset, gl, y, scale_rows=1):
        self.mg, self.torch, self.op = mg, torch, op
        self.keep = (x, w, scale, offset, gl, y)
        p = lambda t: 0 if t is None else t.data_ptr()
        if fmt in ("fp4_b32", "bf16"):
            N, K = w.shape[1], x.shape[1]
        else:
            K, N = x.shape[1], y.shape[1]
        self.args = mg.grouped_args(mg.format_from_compute_type(fmt), p(x), p(w), p(scale), p(offset), p(gl), p(y),
                                    x.shape[0], K, N, gl.shape[0], scale_rows)
        self.fn = mg.grouped_gemm if op == "gemm" else mg.grouped_gemv

    def __call__(self):
        self.fn(self.args, self.torch.cuda.current_stream().cuda_stream)


def time_launches(torch, fns, iters, warmup):
    """Average duration (s) of each callable in fns, measured with events recorded on the
    launch stream around every single launch."""
    for _ in range(warmup):
        for f in fns:
            f()
    torch.cuda.synchronize()
    ev = [[(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in fns]
          for _ in range(iters)]
    for i in range(iters):
        for j, f in enumerate(fns):
            ev[i][j][0].record()
            f()
            ev[i][j][1].record()
    torch.cuda.synchronize()
    return [sum(ev[i][j][0].elapsed_time(ev[i][j][1]) for i in range(iters)) / iters * 1e-3 for j in range(len(fns))]


def time_batch(torch, fn, iters, warmup):
    """Average time (s) per launch of `iters` back-to-back launches between two events on the
    launch stream: for kernels of a few microseconds, where an event pair around every launch
    costs about as much as the kernel.  Includes the gaps between consecutive launches."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters * 1e-3


def time_graph(torch, fn, iters, warmup):
    """Like time_batch, but the `iters` launches are captured into one HIP graph and replayed, so
    that the host's launch rate (a few microseconds per call from Python) does not enter.
    Returns None if the capture fails."""
    try:
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            for _ in range(iters):
                fn()
        g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        g.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / iters * 1e-3
    except Exception as ex:  # noqa: BLE001
        print(f"graph timing unavailable: {ex}", file=sys.stderr)
        return None


def bf16_normal(torch, shape, std=1.0):
    return (torch.randn(shape, device="cuda", dtype=torch.float32) * std).to(torch.bfloat16)


def bf16_uniform(torch, shape, lo, hi):
    return (torch.rand(shape, device="cuda", dtype=torch.float32) * (hi - lo) + lo).to(torch.bfloat16)


# --------------------------------------------------------------------------- workloads
def build_dsv3_int4_prefill(torch, mg, gen):
    G, tokens, topk, H, I = 256, 4096, 8, 7168, 2048
    counts = routed_counts(torch, tokens, G, topk, gen)
    gl = counts.cumsum(0).to(torch.int64).cuda()
    M = tokens * topk
    ops, flops, nbytes = [], [], []
    for name, K, N in (("gate_up", H, 2 * I), ("down", I, H)):
        x = bf16_normal(torch, (M, K))
        w = torch.randint(0, 256, (G, K, N // 2), dtype=torch.uint8, device="cuda")   # two uniform nibbles per byte
        s = bf16_uniform(torch, (G, K // 128, N), 1e-3, 1e-2)
        y = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
        ops.append(Op(mg, torch, "gemm", "int4", x, w, s, None, gl, y, scale_rows=K // 128))
        flops.append(2.0 * M * K * N)
        nbytes.append(x.numel() * 2 + w.numel() + s.numel() * 2 + y.numel() * 2)
    return dict(ops=ops, flops=flops, names=["gate_up", "down"], M=M, G=G, bytes_per_launch=sum(nbytes) / len(nbytes),
                desc="DeepSeek-V3 MoE prefill, int4 antiquant: 256 experts, 4096 tokens x top-8 = 32768 rows, "
                     "gate_up K=7168 N=4096 + down K=2048 N=7168, zero point 8, bf16 scales per 128 k")


EXTRA = ("dequant", "prepack", "route", "gemv_bf16", "gemm_int8", "fused_fp4", "reference_containers")


def settle(torch, fn, ms):
    """Runs fn untimed for about ms milliseconds of queued launches: a matrix-bound kernel that follows a light
    phase is measured at the clocks the board settles to under it, not while they are still moving (measured on
    the int8 workload: 565 us per launch in the first 20 launches after a pause, 475 us from the 40th on)."""
    if ms <= 0:
        return
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < ms:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()


def run_extra(torch, mg, gen, iters, warmup, only=None, settle_ms=0.0):
    """The other benchmark configurations; `only` names one of EXTRA to run just that one (for profiles that
    must hold a single workload's kernels)."""
    out = {}
    want = lambda name: only is None or only == name
    if want("dequant"):
        out.update(extra_dequant(torch, mg, warmup))
    if want("prepack"):
        out.update(extra_prepack(torch, mg, warmup))
    if want("route"):
        out.update(extra_route(torch, mg, warmup))
    if want("gemv_bf16"):
        out.update(extra_gemv_bf16(torch, mg, gen, iters, warmup))
    if want("gemm_int8"):
        out.update(extra_gemm_int8(torch, mg, iters, warmup, settle_ms))
    if want("fused_fp4") or want("reference_containers"):
        out.update(extra_decode_256e(torch, mg, gen, iters, warmup, fused=want("fused_fp4"), ref=want("reference_containers"), settle_ms=settle_ms))
    return out


def extra_dequant(torch, mg, warmup):
    out = {}
    # c1: FP4 e2m1 -> BF16 dequant of a 7168 x 2048 weight, per-32 bf16 scales
    R, C = 7168, 2048
    nbuf = 16   # 16 x 37.6 MB > 2 x the 256 MB Infinity Cache: the rotating variant reads and writes cold lines
    codes = [torch.randint(0, 256, (R, C // 2), dtype=torch.uint8, device="cuda") for _ in range(nbuf)]
    scales = [bf16_uniform(torch, (R, C // 32), 2.0 ** -8, 2.0 ** -2) for _ in range(nbuf)]
    outs = [torch.empty(R, C, dtype=torch.bfloat16, device="cuda") for _ in range(nbuf)]
    stream = lambda: torch.cuda.current_stream().cuda_stream
    state = {"i": 0}

    def dq_rot():
        i = state["i"] = (state["i"] + 1) % nbuf
        mg.dequant_fp4_bf16(codes[i].data_ptr(), scales[i].data_ptr(), outs[i].data_ptr(), R, C, 32, stream())

    def dq_same():
        mg.dequant_fp4_bf16(codes[0].data_ptr(), scales[0].data_ptr(), outs[0].data_ptr(), R, C, 32, stream())

    nbytes = R * C // 2 + R * (C // 32) * 2 + R * C * 2
    t_rot = time_batch(torch, dq_rot, 320, warmup + nbuf)
    t_same = time_batch(torch, dq_same, 320, warmup)
    t_graph = time_graph(torch, dq_rot, 320, warmup)

    def fill_rot():   # a plain device fill of the same output tensors: what writing 29.4 MB alone costs here
        i = state["i"] = (state["i"] + 1) % nbuf
        outs[i].zero_()

    t_fill = time_batch(torch, fill_rot, 320, warmup)
    out["fp4_dequant_7168x2048"] = dict(bytes=nbytes, us=t_rot * 1e6, GBps=nbytes / t_rot / 1e9,
                                        frac_hbm=nbytes / t_rot / 1e9 / PEAK_HBM_GBS, us_same_buffer=t_same * 1e6,
                                        GBps_same_buffer=nbytes / t_same / 1e9,
                                        us_graph_replay=None if t_graph is None else t_graph * 1e6,
                                        frac_hbm_graph_replay=None if t_graph is None else nbytes / t_graph / 1e9 / PEAK_HBM_GBS,
                                        us_fill_of_the_output_alone=t_fill * 1e6,
                                        note="320 back-to-back launches between two events, rotating over 16 buffer "
                                             "sets (cold) / on the same buffers (Infinity Cache warm); graph_replay: the same 320 "
                                             "rotating launches captured in one HIP graph (no host launch cost)")
    del codes, scales, outs
    return out


def extra_prepack(torch, mg, warmup):
    out = {}
    stream = lambda: torch.cuda.current_stream().cuda_stream
    # weight preparation for the reference's "fp4" container: checkpoint codes [G, N, K/2] + scales [G, N, K/16]
    # -> [G, K, N/2] + [G, K/16, N] (nibble transpose + tile permutation, scale merge + transpose)
    G, K, N = 32, 7168, 2048
    ck = torch.randint(0, 256, (G, N, K // 2), dtype=torch.uint8, device="cuda")
    sck = bf16_uniform(torch, (G, N, K // 16), 1.0, 448.0)
    s2 = torch.rand(G, 1, device="cuda") * 1e-2
    wo = torch.empty(G, K, N // 2, dtype=torch.int8, device="cuda")
    so = torch.empty(G, K // 16, N, dtype=torch.bfloat16, device="cuda")

    def pp():
        mg.prepack_fp4_ref(ck.data_ptr(), sck.data_ptr(), s2.data_ptr(), wo.data_ptr(), so.data_ptr(), G, N, K, 1, stream())

    t = time_batch(torch, pp, 20, warmup)
    nbytes = 2 * (ck.numel() + sck.numel() * 2)
    out["prepack_fp4_ref_32e"] = dict(bytes=nbytes, us=t * 1e6, GBps=nbytes / t / 1e9, frac_hbm=nbytes / t / 1e9 / PEAK_HBM_GBS)
    del ck, sck, wo, so
    return out


def extra_route(torch, mg, warmup):
    out = {}
    stream = lambda: torch.cuda.current_stream().cuda_stream
    # routing for configuration 4: 4096 tokens, 256 experts, top-8, K = 7168: logits -> top-k -> group_list
    # and the token rows gathered into expert order
    T, E, K, topk = 4096, 256, 7168, 8
    lg = torch.randn(T, E, device="cuda")
    xr = bf16_normal(torch, (T, K))
    n = T * topk
    ids = torch.empty(n, dtype=torch.int32, device="cuda"); wt = torch.empty(n, device="cuda")
    glr = torch.empty(E, dtype=torch.int64, device="cuda")
    rt = torch.empty(n, dtype=torch.int32, device="cuda"); roc = torch.empty(n, dtype=torch.int32, device="cuda")
    xs = torch.empty(n, K, dtype=torch.bfloat16, device="cuda")
    ra = mg.route_args(lg.data_ptr(), xr.data_ptr(), ids.data_ptr(), wt.data_ptr(), glr.data_ptr(), rt.data_ptr(),
                       roc.data_ptr(), xs.data_ptr(), 0, T, E, K, topk)
    ws = torch.empty(mg.route_workspace_bytes(ra) + 4, dtype=torch.uint8, device="cuda")
    ra.workspace = ws.data_ptr()
    t = time_batch(torch, lambda: mg.route(ra, stream()), 20, warmup)
    nbytes = T * E * 4 + T * K * 2 + n * K * 2      # logits + x read (x rows are re-read from cache) + sorted rows written
    out["routing_4096x256_top8"] = dict(bytes=nbytes, us=t * 1e6, GBps=nbytes / t / 1e9, frac_hbm=nbytes / t / 1e9 / PEAK_HBM_GBS,
                                        note="4 kernels: top-k, histogram, scan + rank, row scatter")
    del lg, xr, xs
    return out


def extra_gemv_bf16(torch, mg, gen, iters, warmup):
    out = {}
    # c2: grouped GEMV decode, 64 experts, 32 rows (4 tokens x top-8), K=7168, N=2048, bf16 weights [G,N,K]
    G, K, N = 64, 7168, 2048
    counts = routed_counts(torch, 4, G, 8, gen, max_rows=4)
    gl = counts.cumsum(0).to(torch.int64).cuda()
    M = int(counts.sum())
    A = int((counts > 0).sum())
    x = bf16_normal(torch, (M, K))
    w = bf16_normal(torch, (G, N, K), 0.02)
    y = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    op = Op(mg, torch, "gemv", "bf16", x, w, None, None, gl, y)
    t = time_batch(torch, op, iters, warmup)
    nbytes = A * N * K * 2 + M * K * 2 + M * N * 2
    out["grouped_gemv_bf16_64e"] = dict(active_experts=A, rows=M, bytes=nbytes, us=t * 1e6, GBps=nbytes / t / 1e9,
                                        frac_hbm=nbytes / t / 1e9 / PEAK_HBM_GBS)
    del x, w, y, op
    return out


def extra_gemm_int8(torch, mg, iters, warmup, settle_ms=0.0):
    out = {}
    # c3: int8 antiquant grouped GEMM, 8 experts, multinomial 4096 rows, K=4096, N=14336
    G, M, K, N = 8, 4096, 4096, 14336
    counts = torch.distributions.Multinomial(M, torch.full((G,), 1.0 / G)).sample().to(torch.int64)
    gl = counts.cumsum(0).cuda()
    x = bf16_normal(torch, (M, K))
    w = torch.randint(-127, 128, (G, K, N), dtype=torch.int8, device="cuda")
    s = bf16_uniform(torch, (G, N), 1e-3, 1e-2)
    o = bf16_uniform(torch, (G, N), -2.0, 2.0)
    y = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    op = Op(mg, torch, "gemm", "int8", x, w, s, o, gl, y)
    settle(torch, op, settle_ms / 2)
    t, = time_launches(torch, [op], iters, warmup)
    fl = 2.0 * M * K * N
    out["grouped_gemm_int8_8e"] = dict(flops=fl, us=t * 1e6, TFLOPs=fl / t / 1e12,
                                       frac_mfma=fl / t / 1e12 / PEAK_BF16_TFLOPS)
    del x, w, s, o, y, op
    return out


def extra_decode_256e(torch, mg, gen, iters, warmup, fused=True, ref=True, settle_ms=0.0):
    out = {}
    stream = lambda: torch.cuda.current_stream().cuda_stream
    run_fused, run_ref = fused, ref
    # c5: fused FP4 (e2m1, per-32 bf16 scales) grouped GEMM at decode shape vs dequant + bf16 grouped GEMM
    G, K, N = 256, 7168, 2048
    counts = routed_counts(torch, 64, G, 8, gen)
    gl = counts.cumsum(0).to(torch.int64).cuda()
    M = int(counts.sum())
    A = int((counts > 0).sum())
    x = bf16_normal(torch, (M, K))
    y = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    if run_fused:
        out.update(decode_fused_fp4(torch, mg, iters, warmup, G, K, N, M, A, x, gl, y, settle_ms))
    if run_ref:
        out.update(decode_reference_containers(torch, mg, iters, warmup, G, K, N, M, A, x, gl, y, settle_ms))
    return out


def decode_fused_fp4(torch, mg, iters, warmup, G, K, N, M, A, x, gl, y, settle_ms=0.0):
    out = {}
    stream = lambda: torch.cuda.current_stream().cuda_stream
    w = torch.randint(0, 256, (G, N, K // 2), dtype=torch.uint8, device="cuda")
    s = bf16_uniform(torch, (G, N, K // 32), 2.0 ** -8, 2.0 ** -2)
    fused = Op(mg, torch, "gemm", "fp4_b32", x, w, s, None, gl, y)
    wd = torch.empty(G, N, K, dtype=torch.bfloat16, device="cuda")
    y2 = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")

    def dq_all():
        mg.dequant_fp4_bf16(w.data_ptr(), s.data_ptr(), wd.data_ptr(), G * N, K, 32, stream())

    sep = Op(mg, torch, "gemm", "bf16", x, wd, None, None, gl, y2)
    y3 = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    gemv = Op(mg, torch, "gemv", "fp4_b32", x, w, s, None, gl, y3)   # same kernel with the GEMV op's fp32 weights
    settle(torch, lambda: (fused(), gemv()), settle_ms / 4)
    t_f, t_d, t_s, t_v = time_launches(torch, [fused, dq_all, sep, gemv], max(iters // 2, 5), warmup)
    nbytes = A * (N * K // 2 + N * (K // 32) * 2) + M * K * 2 + M * N * 2
    diff = float((y.float() - y2.float()).abs().max())
    out["fused_fp4_gemm_decode_256e"] = dict(active_experts=A, rows=M, bytes=nbytes, us=t_f * 1e6,
                                             GBps=nbytes / t_f / 1e9, frac_hbm=nbytes / t_f / 1e9 / PEAK_HBM_GBS,
                                             separate_us=(t_d + t_s) * 1e6, separate_dequant_us=t_d * 1e6,
                                             separate_gemm_us=t_s * 1e6, speedup_vs_separate=(t_d + t_s) / t_f,
                                             gemv_op_us=t_v * 1e6, gemv_op_frac_hbm=nbytes / t_v / 1e9 / PEAK_HBM_GBS,
                                             max_abs_diff_fused_vs_separate=diff)
    del w, s, wd, y2, y3, fused, sep, gemv
    return out


def decode_reference_containers(torch, mg, iters, warmup, G, K, N, M, A, x, gl, y, settle_ms=0.0):
    out = {}
    # the same decode batch on the reference's own containers (N-contiguous: pre-shuffled fp4 with per-16
    # scales, fp8 with 128 x 128 block scales) and on int4 group-128, through both ops
    ref = {}
    for fmt, wshape, sshape, srows, wbytes in (
            ("fp4", (G, K, N // 2), (G, K // 16, N), K // 16, N * K // 2 + (K // 16) * N * 2),
            ("int4", (G, K, N // 2), (G, K // 128, N), K // 128, N * K // 2 + (K // 128) * N * 2),
            ("fp8", (G, K, N), (G, K // 128, N // 128), K // 128, N * K + (K // 128) * (N // 128) * 4)):
        w = torch.randint(0, 255, wshape, dtype=torch.uint8, device="cuda")
        if fmt == "fp8":
            s = torch.rand(sshape, device="cuda") * 1e-2 + 1e-3
        else:
            s = bf16_uniform(torch, sshape, 2.0 ** -8, 2.0 ** -2)
        w = w.view(torch.int8) if fmt == "fp4" else w
        ops = [Op(mg, torch, kind, fmt, x, w, s, None, gl, y, scale_rows=srows) for kind in ("gemv", "gemm")]
        settle(torch, lambda: (ops[0](), ops[1]()), settle_ms / 4)
        t_v, t_m = time_launches(torch, ops, max(iters // 2, 5), warmup)
        nbytes = A * wbytes + M * K * 2 + M * N * 2
        ref[fmt] = dict(bytes=nbytes, gemv_op_us=t_v * 1e6, gemv_op_frac_hbm=nbytes / t_v / 1e9 / PEAK_HBM_GBS,
                        gemm_op_us=t_m * 1e6, gemm_op_frac_hbm=nbytes / t_m / 1e9 / PEAK_HBM_GBS)
        del w, s, ops
    out["decode_256e_reference_containers"] = dict(active_experts=A, rows=M, **ref)
    return out


# --------------------------------------------------------------------------- CPU baselines
# The reference checks its NPU ops against torch code on the host: unpack the codes with int16 shifts, decode them
# with a bit trick into bf16, apply the scales block by block in a Python loop, then one matmul per expert
# (grouped_gemm/test/python/test_group_gemm_fp4.py:86-102 and :196-217, test_group_gemm_fp8.py:16-47).  The
# functions below restate those loops in torch for each benchmark configuration and are timed on the host's
# cores on a bounded sample; the C/OpenMP oracle is timed beside them on the headline workload.
def _timed(fn, budget_s):
    reps, t0 = 0, time.perf_counter()
    while reps == 0 or time.perf_counter() - t0 < budget_s:
        fn()
        reps += 1
    return reps, time.perf_counter() - t0


def _unpack_nibbles(torch, packed):
    """uint8 [..., n/2] (even element in the low nibble) -> uint8 [..., n], one code per byte (unpack_weight)."""
    t = packed.to(torch.int16)
    t = ((t & 0x00F0) << 4) | (t & 0x000F)
    return t.view(torch.uint8)


def _e2m1_to_bf16(torch, codes):
    """e2m1 codes (one per byte) -> bf16 by the reference's bit trick (fp4_dequant): sign to bit 15, the three
    magnitude bits to the top of a bf16 subnormal-range pattern, times 2^126."""
    w = codes.to(torch.int16)
    w = ((w & 0x0008) << 12) | ((w & 0x0007) << 6)
    return w.view(torch.bfloat16) * torch.tensor(0x7E80, dtype=torch.int16).view(torch.bfloat16)


def torch_cpu_fp4_dequant(torch, codes, scale, block):
    w = _e2m1_to_bf16(torch, _unpack_nibbles(torch, codes))
    for i in range(scale.shape[-1]):
        w[..., i * block:(i + 1) * block] *= scale[..., i].unsqueeze(-1)
    return w


def torch_cpu_int4_weights(torch, packed, scale, group):
    """int4 [G, K, N/2], zero point 8, scale bf16 [G, K/group, N] -> bf16 [G, K, N]."""
    w = _unpack_nibbles(torch, packed).to(torch.bfloat16) - 8
    for i in range(scale.shape[-2]):
        w[:, i * group:(i + 1) * group, :] *= scale[:, i, :].unsqueeze(-2)
    return w


def torch_cpu_grouped_matmul(torch, x, w_kn, counts):
    """One fp32 matmul per expert over its rows (what npu_grouped_matmul is checked against); w_kn[g] is [K, N]."""
    y = torch.empty(x.shape[0], w_kn.shape[-1], dtype=torch.bfloat16)
    r0 = 0
    for g, m in enumerate(counts):
        if m:
            y[r0:r0 + m] = (x[r0:r0 + m].float() @ w_kn[g].float()).to(torch.bfloat16)
        r0 += m
    return y


def cpu_baseline(torch, seed, extra=True):
    import numpy as np

    import oracle

    torch.manual_seed(seed)
    cores = torch.get_num_threads()
    bf = torch.bfloat16
    uni = lambda shape, lo, hi: (torch.rand(shape) * (hi - lo) + lo).to(bf)

    # headline: the gate_up GEMM (K=7168, N=4096, int4 group 128) of 4 of the 256 experts, 128 rows each
    G, K, N = 4, 7168, 4096
    counts = [128] * G
    M = sum(counts)
    x = torch.randn(M, K).to(bf)
    w = torch.randint(0, 256, (G, K, N // 2), dtype=torch.uint8)
    sc = uni((G, K // 128, N), 1e-3, 1e-2)
    reps, dt = _timed(lambda: torch_cpu_grouped_matmul(torch, x, torch_cpu_int4_weights(torch, w, sc, 128), counts), 5.0)
    fl = 2.0 * M * K * N
    res = dict(value=fl * reps / dt / 1e12, unit="TFLOP/s", cores=cores, kind="port",
               sample=f"torch restatement of the reference's host check (int16 unpack, bf16 decode, per-group scale loop, "
                      f"one fp32 matmul per expert): {reps} x gate_up GEMM of {G} experts ({M} rows, K={K}, N={N}, int4 "
                      f"group 128) in {dt:.2f} s on {cores} torch threads, dequant included")
    # the C / OpenMP oracle on the same shape, 16 experts
    rng = np.random.default_rng(seed)
    Gc = 16
    cnt = rng.multinomial(128 * Gc, np.full(Gc, 1.0 / Gc))
    glc = np.cumsum(cnt).astype(np.int64)
    Mc = int(glc[-1])
    xb = torch.randn(Mc, K).to(bf).view(torch.int16).numpy().view(np.uint16)
    wc = rng.integers(0, 256, (Gc, K, N // 2), dtype=np.uint8)
    sb = uni((Gc, K // 128, N), 1e-3, 1e-2).view(torch.int16).numpy().view(np.uint16)
    oracle.lib()
    reps, dt = _timed(lambda: oracle.grouped_gemm(oracle.FMT_INT4, xb, wc, sb, None, glc), 5.0)
    res["c_port"] = dict(value=2.0 * Mc * K * N * reps / dt / 1e12, unit="TFLOP/s", cores=oracle.num_threads(),
                         sample=f"{reps} x gate_up GEMM of {Gc} experts ({Mc} rows) in {dt:.2f} s on the oracle's OpenMP loops")
    del x, w, sc, xb, wc, sb
    if not extra:
        return res
    wl = {}
    # c1: FP4 dequant of 7168 x 2048, per-32 scales
    R, C = 7168, 2048
    codes = torch.randint(0, 256, (R, C // 2), dtype=torch.uint8)
    s1 = uni((R, C // 32), 2.0 ** -8, 2.0 ** -2)
    reps, dt = _timed(lambda: torch_cpu_fp4_dequant(torch, codes, s1, 32), 2.5)
    nb = R * C // 2 + R * (C // 32) * 2 + R * C * 2
    wl["fp4_dequant_7168x2048"] = dict(value=nb * reps / dt / 1e9, unit="GB/s", sample=f"{reps} x the full weight in {dt:.2f} s")
    # c2: bf16 grouped GEMV, 64 experts, 32 rows
    G, K, N = 64, 7168, 2048
    counts = [1] * 16 + [2] * 8          # the active experts; the other 40 have no rows and are never touched
    x = torch.randn(sum(counts), K).to(bf)
    w = (torch.randn(len(counts), N, K) * 0.02).to(bf)
    A = len(counts)

    def gemv():
        r0 = 0
        for g, m in enumerate(counts):
            if m:
                (x[r0:r0 + m].float() @ w[g].float().t()).to(bf)
            r0 += m

    reps, dt = _timed(gemv, 2.5)
    nb = A * N * K * 2 + sum(counts) * (K + N) * 2
    wl["grouped_gemv_bf16_64e"] = dict(value=nb * reps / dt / 1e9, unit="GB/s",
                                       sample=f"{reps} x {A} active experts, {sum(counts)} rows in {dt:.2f} s")
    del x, w
    # c3: int8 antiquant GEMM, 1 of the 8 experts (512 rows)
    K, N, m = 4096, 14336, 512
    x = torch.randn(m, K).to(bf)
    q = torch.randint(-127, 128, (K, N), dtype=torch.int8)
    s3, o3 = uni((N,), 1e-3, 1e-2), uni((N,), -2.0, 2.0)
    reps, dt = _timed(lambda: (x.float() @ ((q.float() + o3.float()) * s3.float()).to(bf).float()).to(bf), 2.5)
    wl["grouped_gemm_int8_8e"] = dict(value=2.0 * m * K * N * reps / dt / 1e12, unit="TFLOP/s",
                                      sample=f"{reps} x one expert of 512 rows (K={K}, N={N}) in {dt:.2f} s, dequant included")
    del x, q
    # c5: FP4 weights at decode shape: dequant + matmul of 8 active experts, 2 rows each
    G, K, N = 8, 7168, 2048
    codes = torch.randint(0, 256, (G, N, K // 2), dtype=torch.uint8)
    s5 = uni((G, N, K // 32), 2.0 ** -8, 2.0 ** -2)
    x = torch.randn(2 * G, K).to(bf)

    def fused():
        wd = torch_cpu_fp4_dequant(torch, codes, s5, 32)
        for g in range(G):
            (x[2 * g:2 * g + 2].float() @ wd[g].float().t()).to(bf)

    reps, dt = _timed(fused, 2.5)
    nb = G * (N * K // 2 + N * (K // 32) * 2) + 2 * G * (K + N) * 2
    wl["fused_fp4_gemm_decode_256e"] = dict(value=nb * reps / dt / 1e9, unit="GB/s",
                                            sample=f"{reps} x 8 active experts, 16 rows in {dt:.2f} s (packed bytes / time)")
    res["workloads"] = wl
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="dsv3_int4_prefill")
    ap.add_argument("--settle-ms", type=float, default=300.0,
                    help="untimed run of the workload before the warmup steps, until the clocks have settled")
    ap.add_argument("--no-extra", action="store_true", help="skip the other benchmark configurations")
    ap.add_argument("--only", choices=("headline",) + EXTRA, default=None,
                    help="run just this workload's GPU launches and print its figures (for profiles of one kernel)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU oracle baseline")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain 1 GiB device copy (known traffic) to scale FETCH_SIZE / WRITE_SIZE")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this build runs on one GPU only (--gpus 1); the ops shard by expert across GPUs, "
                 "with the token exchange left to the caller")
    if args.workload != "dsv3_int4_prefill":
        sys.exit("bench.py: the only headline workload is dsv3_int4_prefill")

    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    import moe_gfx950 as mg   # raises if the HIP library has not been built

    torch.cuda.set_device(0)
    gen = torch.Generator().manual_seed(0)
    torch.manual_seed(0)

    if args.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)   # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst

    if args.only in EXTRA:
        print(json.dumps({"only": args.only, "workloads": run_extra(torch, mg, gen, max(args.steps, 20), args.warmup, only=args.only, settle_ms=args.settle_ms)}),
              flush=True)
        return
    if args.only == "headline":
        args.no_extra = args.no_cpu = True

    wl = build_dsv3_int4_prefill(torch, mg, gen)
    ops = wl["ops"]
    # The board settles its clocks over the first tenths of a second under this load (measured: the first 20
    # launches after an idle phase run about 5 % slower than the following ones), so the workload runs untimed for
    # --settle-ms before the W warmup steps.
    torch.cuda.synchronize()
    board = {"socket_power_w_idle": None, "sclk_mhz_idle": None, "socket_power_w_under_load": None, "sclk_mhz_under_load": None,
             "board_power_limit_w": 1400}
    if args.settle_ms > 0:
        board["socket_power_w_idle"], board["sclk_mhz_idle"] = board_state()
    t_settle = time.perf_counter()
    while (time.perf_counter() - t_settle) * 1e3 < args.settle_ms:
        first = board["socket_power_w_under_load"] is None
        for _ in range(900 if first else 40):         # about 3 s (the first time) / 130 ms of queued launches
            for op in ops:
                op()
        if first:
            # read the board while the queue is still running: the metrics table is refreshed about once a second,
            # so the highest of three readings is taken
            board["socket_power_w_under_load"] = 0
            for _ in range(3):
                time.sleep(0.4)
                pw, ck = board_state()
                if pw and pw > board["socket_power_w_under_load"]:
                    board["socket_power_w_under_load"], board["sclk_mhz_under_load"] = pw, ck
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        for op in ops:
            op()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        for op in ops:
            op()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    step_flops = sum(wl["flops"])
    value = step_flops * args.steps / dt / 1e12

    # per-launch durations of the dominant kernel (the int4 grouped GEMM), events on the launch stream
    t_each = time_launches(torch, ops, args.steps, 1)
    avg_launch = sum(t_each) / len(t_each)
    achieved = (step_flops / len(ops)) / avg_launch / 1e12
    traffic, traffic_from = measured_traffic()
    roofline = dict(bound="mfma", achieved=achieved, peak=PEAK_BF16_TFLOPS, unit="TFLOP/s",
                    frac=achieved / PEAK_BF16_TFLOPS, traffic=traffic, traffic_from=traffic_from,
                    algorithmic_bytes_per_launch=wl["bytes_per_launch"],
                    kernel="moe::grouped_gemm_kernel<int4>",
                    per_launch={n: dict(us=t * 1e6, TFLOPs=f / t / 1e12, frac=f / t / 1e12 / PEAK_BF16_TFLOPS)
                                for n, t, f in zip(wl["names"], t_each, wl["flops"])})
    # gate_up with the SwiGLU activation fused into its epilogue (same tensors; the weight columns are then read as
    # groups of (gate, gate, up, up)): writes [M, N/2] instead of [M, N] and spares a separate activation pass
    fused = None
    if not args.no_extra:
        gu = ops[0]
        xg, wg, sg, _, glg, yg = gu.keep
        y_half = torch.empty(yg.shape[0], yg.shape[1] // 2, dtype=torch.bfloat16, device="cuda")
        a = mg.grouped_args(mg.format_from_compute_type("int4"), xg.data_ptr(), wg.data_ptr(), sg.data_ptr(), 0,
                            glg.data_ptr(), y_half.data_ptr(), xg.shape[0], xg.shape[1], yg.shape[1], glg.shape[0],
                            xg.shape[1] // 128, epilogue=mg.EPILOGUE_SWIGLU)
        t_plain, t_fused = time_launches(
            torch, [gu, lambda: mg.grouped_gemm(a, torch.cuda.current_stream().cuda_stream)], args.steps, 1)
        fused = dict(us=t_fused * 1e6, plain_us=t_plain * 1e6, TFLOPs=wl["flops"][0] / t_fused / 1e12,
                     y_bytes_saved=int(yg.numel()))   # bf16 [M, N] -> [M, N/2]
        del y_half
    del wl, ops
    torch.cuda.empty_cache()

    result = {
        "metric": "grouped-GEMM TFLOPS + GEMV/dequant HBM GB/s (% of MI355X peak), DSV3 MoE",
        "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "settle_ms": args.settle_ms, "ms_per_step": dt / args.steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "dsv3_int4_prefill: 256 experts, 4096 tokens x top-8 (32768 rows), gate_up "
                               "7168->4096 + down 2048->7168, int4 zp8 group-128 bf16 scales, bf16 activations",
                   "flops_per_step": step_flops},
        "roofline": roofline,
        # socket power and shader clock before and during the settle phase: this workload runs at the board's power limit
        "board": board,
    }
    if not args.no_extra:
        result["workloads"] = run_extra(torch, mg, gen, max(args.steps, 20), args.warmup, settle_ms=args.settle_ms)
        result["workloads"]["gate_up_swiglu_fused"] = fused
        torch.cuda.empty_cache()
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(torch, 0, extra=not args.no_extra)
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
