"""moe_route_static (the routing entry point that allocates nothing: its scratch is a static device array
inside the library) against moe_route on the same inputs, through the C ABI.  Two calls in a row, the second
with a smaller input, so that what the first call left in the shared array is there when the second runs.
Indices and group_list bit-exact, softmax weights bit-exact too (same kernels)."""
import sys

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _run(entry, logits, x, T, E, K, topk):
    import moe_gfx950 as mg

    dev = torch.device("cuda")
    n = T * topk
    d_logits = torch.from_numpy(logits).to(dev)
    d_ids = torch.full((n,), -7, dtype=torch.int32, device=dev)
    d_w = torch.full((n,), float("nan"), dtype=torch.float32, device=dev)
    d_gl = torch.full((E,), -1, dtype=torch.int64, device=dev)
    d_rt = torch.full((n,), -5, dtype=torch.int32, device=dev)
    d_roc = torch.full((n,), -5, dtype=torch.int32, device=dev)
    d_x = torch.from_numpy(x.view(np.int16)).to(dev)
    d_xs = torch.full((n, K), 0x7FC0, dtype=torch.int16, device=dev)
    args = mg.route_args(d_logits.data_ptr(), d_x.data_ptr(), d_ids.data_ptr(), d_w.data_ptr(), d_gl.data_ptr(),
                         d_rt.data_ptr(), d_roc.data_ptr(), d_xs.data_ptr(), 0, T, E, K, topk)
    stream = torch.cuda.current_stream().cuda_stream
    if entry == "static":
        mg.route_static(args, stream)          # workspace stays NULL
    else:
        ws = torch.empty(max(mg.route_workspace_bytes(args), 4), dtype=torch.uint8, device=dev)
        args.workspace = ws.data_ptr()
        mg.route(args, stream)
    torch.cuda.synchronize()
    return [t.cpu().numpy() for t in (d_ids, d_w, d_gl, d_rt, d_roc, d_xs)]


def test_route_static_matches_route_twice_second_smaller():
    import moe_gfx950 as mg
    import oracle

    for T, E, K, topk in ((4096, 256, 512, 8), (517, 64, 128, 6)):
        print(f"route_static T={T} E={E} K={K} topk={topk}", flush=True)
        sys.stdout.flush()
        rng = np.random.default_rng(T)
        logits = rng.standard_normal((T, E)).astype(np.float32)
        x = oracle.f32_to_bf16_bits(rng.standard_normal((T, K)).astype(np.float32))
        got = _run("static", logits, x, T, E, K, topk)
        want = _run("plain", logits, x, T, E, K, topk)
        for g, w, name in zip(got, want, ("topk_ids", "topk_weight", "group_list", "row_token", "row_of_choice", "x_sorted")):
            assert np.array_equal(g, w), name
        assert got[2][-1] == T * topk


def test_route_static_allocates_nothing_and_replays_from_a_graph():
    """The contract of the entry point: after its first call on a GPU (the one that looks the scratch array's
    address up) it allocates no device memory -- the free memory the driver reports does not change over
    further calls -- and it can be captured into a HIP graph; every replay must give moe_route's result."""
    import moe_gfx950 as mg
    import oracle

    T, E, K, topk = 1500, 96, 256, 4
    print(f"route_static no-alloc / graph T={T} E={E}", flush=True)
    sys.stdout.flush()
    rng = np.random.default_rng(3)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    x = oracle.f32_to_bf16_bits(rng.standard_normal((T, K)).astype(np.float32))
    want = _run("plain", logits, x, T, E, K, topk)
    _run("static", logits, x, T, E, K, topk)                 # first call on this GPU, outside any capture
    dev = torch.device("cuda")
    n = T * topk
    d_logits = torch.from_numpy(logits).to(dev)
    d_x = torch.from_numpy(x.view(np.int16)).to(dev)
    outs = [torch.empty((n,), dtype=torch.int32, device=dev), torch.empty((n,), dtype=torch.float32, device=dev),
            torch.empty((E,), dtype=torch.int64, device=dev), torch.empty((n,), dtype=torch.int32, device=dev),
            torch.empty((n,), dtype=torch.int32, device=dev), torch.empty((n, K), dtype=torch.int16, device=dev)]
    args = mg.route_args(d_logits.data_ptr(), d_x.data_ptr(), outs[0].data_ptr(), outs[1].data_ptr(), outs[2].data_ptr(),
                         outs[3].data_ptr(), outs[4].data_ptr(), outs[5].data_ptr(), 0, T, E, K, topk)
    side = torch.cuda.Stream()
    mg.route_static(args, side.cuda_stream)                   # the runtime's own set-up of a new stream happens here
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    reserved_before = torch.cuda.memory_reserved()
    for _ in range(3):
        mg.route_static(args, side.cuda_stream)
    side.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before and torch.cuda.memory_reserved() == reserved_before
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        mg.route_static(args, torch.cuda.current_stream().cuda_stream)
    for rep in range(3):
        for t in outs:
            t.fill_(-3)                                       # eager work between the replays
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for t, w, name in zip(outs, want, ("topk_ids", "topk_weight", "group_list", "row_token", "row_of_choice", "x_sorted")):
            assert np.array_equal(t.cpu().numpy(), w), f"replay {rep}: {name}"


def test_route_static_rejects_sizes_beyond_its_scratch():
    import moe_gfx950 as mg

    # (ceil(T * topk / 1024) + 1) * E * 4 bytes of scratch: 1024 experts, 2^20 choices -> 4 MiB > 2 MiB
    args = mg.route_args(16, 0, 16, 16, 16, 16, 16, 0, 0, 1 << 17, 1024, 0, 8)
    assert mg.route_workspace_bytes(args) > mg.ROUTE_STATIC_SCRATCH_BYTES
    with pytest.raises(mg.MoeError) as e:
        mg.route_static(args, 0)
    assert e.value.status == mg.ERR_TOO_LARGE
