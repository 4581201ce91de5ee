"""GPU parity of the fp4 weight preparation (checkpoint tensors -> the reference's "fp4" container)
against the numpy restatements of the reference's test helpers.  Bit-exact."""
import sys

import numpy as np
import pytest
import torch

import helpers as H
import oracle
from oracle import layouts as L

pytestmark = pytest.mark.gpu


def _say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def _prepack(ckpt, scale_bits, scale2, G, N, K):
    import moe_gfx950 as mg

    dev = torch.device("cuda")
    c = torch.from_numpy(ckpt).to(dev) if ckpt is not None else None
    s = torch.from_numpy(scale_bits.view(np.int16)).to(dev) if scale_bits is not None else None
    s2 = torch.from_numpy(scale2).to(dev) if scale2 is not None else None
    w_out = torch.full((G, K, N // 2), 0x55, dtype=torch.uint8, device=dev) if c is not None else None
    s_out = torch.full((G, K // 16, N), 0x7FC0, dtype=torch.int16, device=dev) if s is not None else None
    p = lambda t: 0 if t is None else t.data_ptr()
    mg.prepack_fp4_ref(p(c), p(s), p(s2), p(w_out), p(s_out), G, N, K, 0 if scale2 is None else scale2.shape[1],
                       torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return (None if w_out is None else w_out.cpu().numpy(),
            None if s_out is None else s_out.cpu().numpy().view(np.uint16))


@pytest.mark.parametrize("G,N,K", [(1, 256, 64), (2, 256, 256), (3, 512, 320), (2, 768, 1024), (1, 256, 7168)])
def test_codes_match_reference_repack(G, N, K):
    _say(f"prepack codes G={G} N={N} K={K}")
    rng = np.random.default_rng(G * 1000 + N + K)
    ckpt = rng.integers(0, 256, (G, N, K // 2), dtype=np.uint8)
    got, _ = _prepack(ckpt, None, None, G, N, K)
    ref = L.fp4ref_from_checkpoint(ckpt).view(np.uint8)
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("cols", [0, 1, 2])
@pytest.mark.parametrize("G,N,K", [(2, 256, 64), (3, 512, 1088), (1, 256, 7168)])
def test_scales_match_reference_merge_and_transpose(G, N, K, cols):
    _say(f"prepack scales G={G} N={N} K={K} scale2 cols={cols}")
    rng = np.random.default_rng(N + K + cols)
    sc = oracle.f32_to_bf16_bits(rng.uniform(1.0, 448.0, (G, N, K // 16)).astype(np.float32))
    s2 = rng.uniform(1e-4, 1e-2, (G, cols)).astype(np.float32) if cols else None
    _, got = _prepack(None, sc, s2, G, N, K)
    assert np.array_equal(got, L.fp4ref_scale_from_checkpoint(sc, s2))


def test_prepacked_weights_feed_the_fp4_gemm():
    """End to end: checkpoint tensors -> GPU prepack -> grouped_gemm "fp4"; the expected value comes
    from the logical weights (codes and merged scales) through the oracle's GEMM."""
    _say("prepack -> fp4 gemm")
    rng = np.random.default_rng(5)
    G, K, N = 4, 512, 512
    gl = [12, 25, 44, 48]
    codes = rng.integers(0, 16, (G, N, K), dtype=np.uint8)            # checkpoint orientation [G, N, K]
    ckpt = L.pack_nibbles_last(codes)
    sc = oracle.f32_to_bf16_bits(rng.uniform(0.5, 2.0, (G, N, K // 16)).astype(np.float32))
    s2 = rng.uniform(1e-2, 3e-2, (G, 1)).astype(np.float32)
    w_dev, s_dev = _prepack(ckpt, sc, s2, G, N, K)
    case = H.make_case("fp4", G, K, N, gl, seed=9)
    case["weight"] = w_dev.view(np.int8)
    case["scale"] = s_dev
    got = H.run_cabi(case, H.upload(case), "gemm")
    ref_case = dict(case)
    ref_case["weight"] = L.fp4ref_from_checkpoint(ckpt)
    ref_case["scale"] = L.fp4ref_scale_from_checkpoint(sc, s2)
    H.assert_close(got, H.oracle_out(ref_case), rows=slice(0, gl[-1]), what="prepack -> gemm")


def test_prepack_rejects_bad_arguments():
    import moe_gfx950 as mg

    t = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    with pytest.raises(mg.MoeError) as e:
        mg.prepack_fp4_ref(t.data_ptr(), 0, 0, t.data_ptr(), 0, 1, 200, 64)      # N % 256
    assert e.value.status == mg.ERR_BAD_ALIGNMENT
    with pytest.raises(mg.MoeError) as e:
        mg.prepack_fp4_ref(t.data_ptr(), 0, 0, 0, 0, 1, 256, 64)                 # codes without an output
    assert e.value.status == mg.ERR_NULL_POINTER


def test_module_functions_follow_the_reference_test_flow():
    """test_group_gemm_fp4.py:175-196 with the host-side torch reshapes replaced by the module's GPU
    ops: init weights in checkpoint form, repack, merge + transpose the scales, call grouped_gemm."""
    import cinfer_ascendc

    _say("prepack via cinfer_ascendc")
    rng = np.random.default_rng(17)
    G, K, N = 4, 256, 256
    gl = [2, 3, 4, 256]
    ckpt = L.pack_nibbles_last(rng.integers(0, 16, (G, N, K), dtype=np.uint8))
    sc = oracle.f32_to_bf16_bits(rng.uniform(0.5, 2.0, (G, N, K // 16)).astype(np.float32))
    s2 = rng.uniform(1e-2, 3e-2, (G, 2, 1)).astype(np.float32)
    w_dev = cinfer_ascendc.repack_weight_fp4(torch.from_numpy(ckpt).cuda())
    s_dev = cinfer_ascendc.merge_scale_fp4(torch.from_numpy(sc.view(np.int16)).cuda().view(torch.bfloat16),
                                           torch.from_numpy(s2).cuda())
    assert w_dev.dtype == torch.int8 and tuple(w_dev.shape) == (G, K, N // 2)
    assert s_dev.dtype == torch.bfloat16 and tuple(s_dev.shape) == (G, K // 16, N)
    assert np.array_equal(w_dev.cpu().numpy(), L.fp4ref_from_checkpoint(ckpt))
    assert np.array_equal(H.bits(s_dev.cpu()), L.fp4ref_scale_from_checkpoint(sc, s2.reshape(G, 2)))
    x = (torch.randn(gl[-1], K, generator=torch.Generator().manual_seed(1)) * 0.5).to(torch.bfloat16)
    out = torch.zeros(gl[-1], N, dtype=torch.bfloat16, device="cuda")
    cinfer_ascendc.grouped_gemm(x.cuda(), w_dev, output=out, antiquantOffsetOptional=torch.zeros_like(s_dev),
                                antiquantScaleOptional=s_dev, groupListOptional=torch.tensor(gl).cuda(),
                                computeType="fp4")
    torch.cuda.synchronize()
    ref = oracle.grouped_gemm(oracle.FMT_FP4_REF, H.bits(x), L.fp4ref_from_checkpoint(ckpt),
                              L.fp4ref_scale_from_checkpoint(sc, s2.reshape(G, 2)), None, np.asarray(gl, dtype=np.int64))
    H.assert_close(H.bits(out.cpu()), ref, what="module prepack -> gemm")
