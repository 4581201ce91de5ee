"""The C ABI's launch contract: asynchronous on the caller's stream, no allocation, no state that outlives a launch.
Checked by capturing the ops into a HIP graph and replaying it, and by calling them from several
host threads on their own streams; results must equal the eager, single-stream ones bit for bit
(every kernel here is deterministic)."""
import sys
import threading

import numpy as np
import pytest
import torch

import helpers as H

pytestmark = pytest.mark.gpu


def _say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def _launcher(case, dev, op):
    import moe_gfx950 as mg

    y = torch.full((case["M"], case["N"]), 0x7FC0, dtype=torch.int16, device="cuda")
    p = lambda t: 0 if t is None else t.data_ptr()
    args = mg.grouped_args(mg.format_from_compute_type(case["fmt"]), p(dev["x"]), p(dev["weight"]), p(dev["scale"]),
                           p(dev["offset"]), p(dev["group_list"]), p(y), case["M"], case["K"], case["N"], case["G"],
                           case["scale_rows"])
    fn = mg.grouped_gemm if op == "gemm" else mg.grouped_gemv
    return y, (lambda: fn(args, torch.cuda.current_stream().cuda_stream))


CASES = [("int4", "gemm", [130, 130, 143, 300, 301], 1024, 512), ("fp4_b32", "gemm", [3, 3, 7, 8, 20], 1024, 256),
         ("bf16", "gemv", [1, 1, 4, 6], 2048, 256), ("fp4", "gemm", [12, 25, 44, 48], 512, 512),
         ("int8", "gemm", [100, 230, 231], 512, 256)]


def test_ops_replay_from_a_hip_graph():
    _say("graph capture / replay")
    built = []
    for n, (fmt, op, gl, K, N) in enumerate(CASES):
        case = H.make_case(fmt, len(gl), K, N, gl, seed=40 + n)
        dev = H.upload(case)
        y, launch = _launcher(case, dev, op)
        launch()
        torch.cuda.synchronize()
        built.append((y, launch, y.clone(), dev))
    side = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    for y, _, _, _ in built:
        y.fill_(0x7FC0)
    torch.cuda.synchronize()
    with torch.cuda.graph(g, stream=side):
        for _, launch, _, _ in built:
            launch()
    for rep in range(3):
        for y, _, _, _ in built:
            y.fill_(0x7FC0)                       # eager work between the replays
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for n, (y, _, want, _) in enumerate(built):
            assert torch.equal(y, want), f"replay {rep}: case {CASES[n][0]} differs from the eager result"


def test_graph_replays_run_beside_eager_launches_on_other_streams():
    """Kernel nodes of a graph keep their arguments for every replay, so a captured grouped GEMM must not own
    state that eager launches hand out again: here two graphs are captured 1024 eager launches apart (the
    distance at which eager launches reuse a tile-counter slot) and then replayed at the same time on two
    streams while eager GEMMs of another grid size run on a third; every result must equal the oracle's."""
    import moe_gfx950 as mg
    _say("graphs beside eager launches")
    rng = np.random.default_rng(11)
    gls = [list(np.cumsum(rng.choice([0, 1, 3, 16, 17, 33, 70], 40))) for _ in range(3)]
    shapes = [("int4", 128, 2048), ("fp4", 128, 1024), ("int4", 256, 512)]
    cases = [H.make_case(fmt, len(gl), K, N, gl, seed=60 + i, group=64) for i, ((fmt, K, N), gl) in enumerate(zip(shapes, gls))]
    devs = [H.upload(c) for c in cases]
    p = lambda t: 0 if t is None else t.data_ptr()
    ys, argss = [], []
    for c, d in zip(cases, devs):
        y = torch.full((c["M"], c["N"]), 0x7FC0, dtype=torch.int16, device="cuda")
        ys.append(y)
        argss.append(mg.grouped_args(mg.format_from_compute_type(c["fmt"]), p(d["x"]), p(d["weight"]), p(d["scale"]),
                                     p(d["offset"]), p(d["group_list"]), p(y), c["M"], c["K"], c["N"], c["G"], c["scale_rows"]))
    refs = [H.oracle_out(c) for c in cases]
    streams = [torch.cuda.Stream() for _ in range(3)]
    torch.cuda.synchronize()

    def capture(i):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=streams[i]):
            for _ in range(4):
                mg.grouped_gemm(argss[i], torch.cuda.current_stream().cuda_stream)
        return g

    g0 = capture(0)
    for _ in range(1024):                       # the eager launches between the two captures
        mg.grouped_gemm(argss[2], streams[2].cuda_stream)
    torch.cuda.synchronize()
    g1 = capture(1)
    for rep in range(3):
        for y in ys:
            y.fill_(0x7FC0)
        torch.cuda.synchronize()
        for _ in range(6):
            with torch.cuda.stream(streams[0]):
                g0.replay()
            with torch.cuda.stream(streams[1]):
                g1.replay()
            for _ in range(8):
                mg.grouped_gemm(argss[2], streams[2].cuda_stream)
        torch.cuda.synchronize()
        for c, y, ref in zip(cases, ys, refs):
            got = y.cpu().numpy().view(np.uint16)
            H.assert_close(got, ref, rows=slice(0, c["group_list"][-1]), what=f"replay {rep} {c['fmt']} N={c['N']}")
            assert (got[c["group_list"][-1]:] == 0x7FC0).all()


def test_ops_from_several_threads_on_their_own_streams():
    _say("threads / streams")
    results, errors = {}, []

    def worker(n, fmt, op, gl, K, N):
        try:
            torch.cuda.set_device(0)
            stream = torch.cuda.Stream()
            case = H.make_case(fmt, len(gl), K, N, gl, seed=40 + n)
            with torch.cuda.stream(stream):
                dev = H.upload(case)
                y, launch = _launcher(case, dev, op)
                for _ in range(5):
                    launch()
            stream.synchronize()
            results[n] = (case, y.cpu().numpy().view(np.uint16))
        except Exception as ex:  # noqa: BLE001
            errors.append((n, repr(ex)))

    threads = [threading.Thread(target=worker, args=(n, *c)) for n, c in enumerate(CASES)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for n, (fmt, op, gl, K, N) in enumerate(CASES):
        case, got = results[n]
        ref = H.oracle_out(case, gemv=(op == "gemv"))
        H.assert_close(got, ref, rows=slice(0, gl[-1]), what=f"thread {n} {fmt}")
