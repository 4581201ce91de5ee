"""GPU parity of the routing op (logits -> top-k -> rows sorted by expert + group_list) against the
numpy restatement.  Indices and group_list are bit-exact; the softmax weights to 1e-5."""
import sys

import numpy as np
import pytest
import torch

import helpers as H
import oracle
from oracle import routing as R

pytestmark = pytest.mark.gpu


def _say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def _route(logits, ids, x, T, E, K, topk):
    import moe_gfx950 as mg

    dev = torch.device("cuda")
    n = T * topk
    d_logits = torch.from_numpy(logits).to(dev) if logits is not None else None
    d_ids = torch.from_numpy(ids).to(dev) if ids is not None else torch.full((max(n, 1),), -7, dtype=torch.int32, device=dev)
    d_w = torch.full((max(n, 1),), float("nan"), dtype=torch.float32, device=dev)
    d_gl = torch.full((E,), -1, dtype=torch.int64, device=dev)
    d_rt = torch.full((max(n, 1),), -5, dtype=torch.int32, device=dev)
    d_roc = torch.full((max(n, 1),), -5, dtype=torch.int32, device=dev)
    d_x = torch.from_numpy(x.view(np.int16)).to(dev) if x is not None else None
    d_xs = torch.full((max(n, 1), K), 0x7FC0, dtype=torch.int16, device=dev) if x is not None else None
    p = lambda t: 0 if t is None else t.data_ptr()
    args = mg.route_args(p(d_logits), p(d_x), p(d_ids), p(d_w), p(d_gl), p(d_rt), p(d_roc), p(d_xs), 0, T, E, K, topk)
    ws = torch.empty(max(mg.route_workspace_bytes(args), 4), dtype=torch.uint8, device=dev)
    args.workspace = ws.data_ptr()
    mg.route(args, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return (d_ids.cpu().numpy()[:n].reshape(T, topk), d_w.cpu().numpy()[:n].reshape(T, topk), d_gl.cpu().numpy(),
            d_rt.cpu().numpy()[:n], d_roc.cpu().numpy()[:n],
            None if d_xs is None else d_xs.cpu().numpy().view(np.uint16)[:n])


@pytest.mark.parametrize("T,E,K,topk", [(1, 8, 64, 2), (37, 7, 128, 3), (64, 256, 256, 8), (4096, 256, 512, 8),
                                        (300, 1024, 64, 6), (1030, 64, 64, 1)])
def test_route_from_logits(T, E, K, topk):
    _say(f"route T={T} E={E} K={K} topk={topk}")
    rng = np.random.default_rng(T + E + topk)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    x = oracle.f32_to_bf16_bits(rng.standard_normal((T, K)).astype(np.float32))
    ids, w, gl, rt, roc, xs = _route(logits, None, x, T, E, K, topk)
    ref_ids, ref_w = R.route_topk(logits, topk)
    assert np.array_equal(ids, ref_ids)
    assert np.allclose(w, ref_w, rtol=1e-5, atol=1e-9)
    ref_gl, ref_rt, ref_roc = R.route_sort(ref_ids, E)
    assert np.array_equal(gl, ref_gl) and np.array_equal(rt, ref_rt) and np.array_equal(roc, ref_roc)
    assert np.array_equal(xs, x[ref_rt])


@pytest.mark.parametrize("E", [48, 200, 300, 1000])
def test_route_topk_with_many_equal_logits(E):
    """Few distinct logit values: every arg-max has several holders, in different lanes and in different
    64-expert slices of a lane; ties go to the lower expert id."""
    _say(f"route ties E={E}")
    T, topk = 130, 6
    rng = np.random.default_rng(E)
    logits = rng.integers(0, 4, (T, E)).astype(np.float32)
    ids, w, gl, rt, roc, _ = _route(logits, None, None, T, E, 0, topk)
    ref_ids, ref_w = R.route_topk(logits, topk)
    assert np.array_equal(ids, ref_ids)
    assert np.allclose(w, ref_w, rtol=1e-5, atol=1e-9)


def test_route_ties_and_given_ids_with_dropped_choices():
    _say("route ties / given ids")
    # all-equal logits: the k lowest expert ids, in order
    T, E, topk = 5, 16, 4
    ids, w, gl, rt, roc, _ = _route(np.zeros((T, E), dtype=np.float32), None, None, T, E, 0, topk)
    assert np.array_equal(ids, np.tile(np.arange(topk, dtype=np.int32), (T, 1)))
    assert np.allclose(w, 1.0 / E)
    assert list(gl[:topk]) == [T, 2 * T, 3 * T, 4 * T] and (gl[topk:] == T * topk).all()
    # ids supplied by the caller, some outside [0, E): dropped
    rng = np.random.default_rng(3)
    T, E, topk = 700, 9, 5
    given = rng.integers(-1, E + 1, (T, topk)).astype(np.int32)
    ids, _, gl, rt, roc, _ = _route(None, given, None, T, E, 0, topk)
    ref_gl, ref_rt, ref_roc = R.route_sort(given, E)
    assert np.array_equal(ids, given)
    assert np.array_equal(gl, ref_gl) and np.array_equal(roc, ref_roc)
    assert np.array_equal(rt[: ref_rt.size], ref_rt)


def test_route_dropped_choices_with_rows_gathered():
    """Dropped choices (ids outside [0, E)) together with the row gather: only rows below
    group_list[E - 1] have a token; the gather must leave the rest of x_sorted untouched and must not
    read the unwritten tail of row_token."""
    _say("route dropped ids + gather")
    rng = np.random.default_rng(11)
    T, E, K, topk = 700, 9, 128, 5
    given = rng.integers(-2, E + 2, (T, topk)).astype(np.int32)
    x = oracle.f32_to_bf16_bits(rng.standard_normal((T, K)).astype(np.float32))
    ids, _, gl, rt, roc, xs = _route(None, given, x, T, E, K, topk)
    ref_gl, ref_rt, ref_roc = R.route_sort(given, E)
    total = int(ref_gl[-1])
    assert 0 < total < T * topk
    assert np.array_equal(gl, ref_gl) and np.array_equal(roc, ref_roc)
    assert np.array_equal(rt[:total], ref_rt) and (rt[total:] == -5).all()
    assert np.array_equal(xs[:total], x[ref_rt])
    assert (xs[total:] == 0x7FC0).all()          # sentinel rows untouched
    # a row of NaN logits selects no expert (every comparison fails): its choices are dropped too
    T, E, K, topk = 6, 8, 64, 2
    logits = rng.standard_normal((T, E)).astype(np.float32)
    logits[2, :] = np.nan
    x = oracle.f32_to_bf16_bits(rng.standard_normal((T, K)).astype(np.float32))
    ids, _, gl, rt, roc, xs = _route(logits, None, x, T, E, K, topk)
    assert int(gl[-1]) == (T - 1) * topk and (roc.reshape(T, topk)[2] == -1).all()
    valid = [t for t in range(T) if t != 2]
    ref_ids, _ = R.route_topk(logits[valid], topk)
    full = np.full((T, topk), -1, dtype=np.int32)
    full[valid] = ref_ids
    ref_gl, ref_rt, _ = R.route_sort(full, E)
    assert np.array_equal(gl, ref_gl) and np.array_equal(rt[: ref_rt.size], ref_rt)
    assert np.array_equal(xs[: ref_rt.size], x[ref_rt]) and (xs[ref_rt.size:] == 0x7FC0).all()


def test_route_rows_with_fewer_finite_logits_than_topk():
    """Masked experts carry -inf logits.  A row with fewer than topk finite logits fills up with masked experts in
    ascending id order (a stable sort by descending logit) and never names an expert twice."""
    _say("route masked logits")
    rng = np.random.default_rng(21)
    T, E, K, topk = 40, 200, 64, 6
    logits = rng.standard_normal((T, E)).astype(np.float32)
    for t in range(T):
        keep = rng.choice(E, size=t % (topk + 2), replace=False)     # 0 .. topk + 1 finite logits
        row = np.full(E, -np.inf, dtype=np.float32)
        row[keep] = logits[t, keep]
        logits[t] = row
    x = oracle.f32_to_bf16_bits(rng.standard_normal((T, K)).astype(np.float32))
    ids, w, gl, rt, roc, xs = _route(logits, None, x, T, E, K, topk)
    for t in range(T):
        assert len(set(ids[t])) == topk, f"row {t} names an expert twice: {ids[t]}"
    finite = [t for t in range(T) if t % (topk + 2) > 0]          # a row of -inf only has no softmax (NaN weights)
    ref_ids, ref_w = R.route_topk(logits[finite], topk)
    assert np.array_equal(ids[finite], ref_ids)
    assert np.allclose(w[finite], ref_w, rtol=1e-5, atol=1e-9)
    all_ref = np.argsort(-logits, axis=1, kind="stable")[:, :topk].astype(np.int32)
    assert np.array_equal(ids, all_ref)
    ref_gl, ref_rt, ref_roc = R.route_sort(all_ref, E)
    assert np.array_equal(gl, ref_gl) and np.array_equal(rt, ref_rt) and np.array_equal(roc, ref_roc)


def test_route_many_blocks_uses_the_scan_kernel():
    """More than 64 blocks of 1024 choices: the per-block counts go through a scan kernel of their own."""
    _say("route many blocks")
    rng = np.random.default_rng(22)
    T, E, K, topk = 20000, 160, 64, 8                  # 157 blocks
    logits = rng.standard_normal((T, E)).astype(np.float32)
    x = oracle.f32_to_bf16_bits(rng.standard_normal((T, K)).astype(np.float32))
    ids, w, gl, rt, roc, xs = _route(logits, None, x, T, E, K, topk)
    ref_ids, _ = R.route_topk(logits, topk)
    assert np.array_equal(ids, ref_ids)
    ref_gl, ref_rt, ref_roc = R.route_sort(ref_ids, E)
    assert np.array_equal(gl, ref_gl) and np.array_equal(rt, ref_rt) and np.array_equal(roc, ref_roc)
    assert np.array_equal(xs, x[ref_rt])


def test_routed_rows_feed_the_grouped_gemm():
    """End to end on the device: logits -> routing -> grouped GEMM on the sorted rows with the
    group_list the routing wrote; expected value from the oracle on the oracle's own sort."""
    import moe_gfx950 as mg

    _say("route -> gemm")
    rng = np.random.default_rng(8)
    T, E, K, N, topk = 96, 8, 256, 256, 2
    logits = rng.standard_normal((T, E)).astype(np.float32)
    x = oracle.f32_to_bf16_bits(rng.standard_normal((T, K)).astype(np.float32))
    ids, w, gl, rt, roc, xs = _route(logits, None, x, T, E, K, topk)
    case = H.make_case("int4", E, K, N, list(gl), seed=2)
    case["x"] = xs
    got = H.run_cabi(case, H.upload(case), "gemm")
    ref_ids, _ = R.route_topk(logits, topk)
    ref_gl, ref_rt, _ = R.route_sort(ref_ids, E)
    ref_case = dict(case)
    ref_case["x"] = x[ref_rt]
    ref_case["group_list"] = ref_gl
    H.assert_close(got, H.oracle_out(ref_case), what="route -> gemm")


def test_module_moe_route_returns_sorted_rows_and_group_list():
    import cinfer_ascendc

    _say("route via cinfer_ascendc")
    g = torch.Generator().manual_seed(12)
    T, E, K, topk = 200, 32, 128, 4
    logits = torch.randn(T, E, generator=g)
    x = torch.randn(T, K, generator=g).to(torch.bfloat16)
    xs, gl, w, ids, roc = cinfer_ascendc.moe_route(logits.cuda(), x.cuda(), topk)
    torch.cuda.synchronize()
    ref_ids, ref_w = R.route_topk(logits.numpy(), topk)
    ref_gl, ref_rt, ref_roc = R.route_sort(ref_ids, E)
    assert np.array_equal(ids.cpu().numpy(), ref_ids) and np.array_equal(gl.cpu().numpy(), ref_gl)
    assert np.array_equal(roc.cpu().numpy(), ref_roc)
    assert np.allclose(w.cpu().numpy(), ref_w, rtol=1e-5, atol=1e-9)
    assert torch.equal(xs.cpu(), x[torch.from_numpy(ref_rt.astype(np.int64))])


def test_route_rejects_bad_arguments():
    import moe_gfx950 as mg

    t = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    a = mg.route_args(t.data_ptr(), 0, t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), 0,
                      t.data_ptr(), 4, 2048, 0, 2)
    with pytest.raises(mg.MoeError) as e:
        mg.route(a)
    assert e.value.status == mg.ERR_BAD_SHAPE          # more than 1024 experts
    a = mg.route_args(t.data_ptr(), 0, t.data_ptr(), t.data_ptr(), 0, t.data_ptr(), t.data_ptr(), 0, t.data_ptr(), 4, 8,
                      0, 2)
    with pytest.raises(mg.MoeError) as e:
        mg.route(a)
    assert e.value.status == mg.ERR_NULL_POINTER       # no group_list
