"""The GPU library, through its C ABI, against the committed known-answer fixtures of tests/golden/
(computed with numpy / torch only, independently of the oracle and of the kernels)."""
import sys

import numpy as np
import pytest
import torch

import helpers as H
from test_golden import load

pytestmark = pytest.mark.gpu


def _say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


@pytest.mark.parametrize("fmt", H.FORMATS)
def test_grouped_ops_match_the_fixtures(fmt):
    d = load("grouped_" + fmt)
    case = dict(fmt=fmt, G=int(d["G"]), K=int(d["K"]), N=int(d["N"]), M=d["x"].shape[0], x=d["x"], weight=d["weight"],
                scale=d.get("scale"), offset=d.get("offset"), group_list=d["group_list"], scale_rows=int(d["scale_rows"]))
    dev = H.upload(case)
    _say(f"golden gemm {fmt}")
    H.assert_close(H.run_cabi(case, dev, "gemm"), d["y_gemm"], what=f"golden gemm {fmt}")
    if fmt in H.GEMV_FORMATS:
        _say(f"golden gemv {fmt}")
        H.assert_close(H.run_cabi(case, dev, "gemv"), d["y_gemv"], what=f"golden gemv {fmt}")


@pytest.mark.parametrize("block", [32, 16])
def test_dequant_matches_the_fixture_bit_for_bit(block):
    import moe_gfx950 as mg

    _say(f"golden dequant block {block}")
    d = load("dequant_fp4")
    codes = torch.from_numpy(d["codes"]).cuda()
    scale = torch.from_numpy(d[f"scale_b{block}"].view(np.int16)).cuda()
    R, C = codes.shape[0], codes.shape[1] * 2
    out = torch.full((R, C), 0x7FC0, dtype=torch.int16, device="cuda")
    mg.dequant_fp4_bf16(codes.data_ptr(), scale.data_ptr(), out.data_ptr(), R, C, block, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy().view(np.uint16), d[f"out_b{block}"])


def test_prepack_matches_the_fixture_bit_for_bit():
    import moe_gfx950 as mg

    _say("golden prepack")
    d = load("prepack_fp4")
    G, N, K = d["ckpt"].shape[0], d["ckpt"].shape[1], d["ckpt"].shape[2] * 2
    ck = torch.from_numpy(d["ckpt"]).cuda()
    sc = torch.from_numpy(d["scale"].view(np.int16)).cuda()
    s2 = torch.from_numpy(d["scale2"]).cuda()
    w_out = torch.full((G, K, N // 2), 0x55, dtype=torch.uint8, device="cuda")
    s_out = torch.full((G, K // 16, N), 0x7FC0, dtype=torch.int16, device="cuda")
    mg.prepack_fp4_ref(ck.data_ptr(), sc.data_ptr(), s2.data_ptr(), w_out.data_ptr(), s_out.data_ptr(), G, N, K,
                       d["scale2"].shape[1], torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert np.array_equal(w_out.cpu().numpy().view(np.int8), d["weight_out"])
    assert np.array_equal(s_out.cpu().numpy().view(np.uint16), d["scale_out"])


def test_routing_matches_the_fixture():
    import moe_gfx950 as mg

    _say("golden route")
    d = load("route")
    T, E = d["logits"].shape
    topk = int(d["topk"])
    n = T * topk
    dev = torch.device("cuda")
    lg = torch.from_numpy(d["logits"]).to(dev)
    ids = torch.full((n,), -7, dtype=torch.int32, device=dev)
    w = torch.full((n,), float("nan"), dtype=torch.float32, device=dev)
    gl = torch.full((E,), -1, dtype=torch.int64, device=dev)
    rt = torch.full((n,), -5, dtype=torch.int32, device=dev)
    roc = torch.full((n,), -5, dtype=torch.int32, device=dev)
    args = mg.route_args(lg.data_ptr(), 0, ids.data_ptr(), w.data_ptr(), gl.data_ptr(), rt.data_ptr(), roc.data_ptr(), 0, 0,
                         T, E, 0, topk)
    ws = torch.empty(max(mg.route_workspace_bytes(args), 4), dtype=torch.uint8, device=dev)
    args.workspace = ws.data_ptr()
    mg.route(args, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert np.array_equal(ids.cpu().numpy().reshape(T, topk), d["ids"])
    assert np.allclose(w.cpu().numpy().reshape(T, topk), d["weight"], rtol=1e-5, atol=1e-9)
    assert np.array_equal(gl.cpu().numpy(), d["group_list"])
    assert np.array_equal(rt.cpu().numpy(), d["row_token"]) and np.array_equal(roc.cpu().numpy(), d["row_of_choice"])
