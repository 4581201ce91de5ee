"""GPU parity of grouped GEMM with the fused SwiGLU epilogue: y[m, 2j+e] = silu(z[m, 4j+e]) * z[m, 4j+2+e]
on the fp32 accumulators z, for the N-contiguous containers, against the oracle's GEMM accumulators put
through oracle.swiglu_interleaved."""
import sys

import numpy as np
import pytest
import torch

import helpers as H
import oracle

pytestmark = pytest.mark.gpu
N_CONTIG = ["fp4", "fp8", "int8", "int4"]
K_CONTIG = ["fp4_b32", "fp4_b16", "bf16"]


def _say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def _run(case):
    import moe_gfx950 as mg

    dev = H.upload(case)
    M, K, N, G = case["M"], case["K"], case["N"], case["G"]
    y = torch.full((M, N // 2), 0x7FC0, dtype=torch.int16, device="cuda")
    p = lambda t: 0 if t is None else t.data_ptr()
    args = mg.grouped_args(mg.format_from_compute_type(case["fmt"]), p(dev["x"]), p(dev["weight"]), p(dev["scale"]),
                           p(dev["offset"]), p(dev["group_list"]), p(y), M, K, N, G, case["scale_rows"],
                           epilogue=mg.EPILOGUE_SWIGLU)
    mg.grouped_gemm(args, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return y.cpu().numpy().view(np.uint16)


def _expected(case):
    _, z = oracle.grouped_gemm(oracle.FMT_BY_NAME[case["fmt"]], case["x"], case["weight"], case["scale"], case["offset"],
                               case["group_list"], want_f32=True)
    return oracle.swiglu_blocked16(z) if case["fmt"] in K_CONTIG else oracle.swiglu_interleaved(z)


@pytest.mark.parametrize("fmt", N_CONTIG)
@pytest.mark.parametrize("gl", [[2, 3, 4, 40], [130, 130, 143, 300, 301], [0, 7, 7, 8]], ids=["small", "prefill", "decode"])
def test_swiglu_epilogue(fmt, gl):
    _say(f"swiglu fmt={fmt} gl={gl}")
    K = 512 if fmt != "fp8" else 256
    case = H.make_case(fmt, len(gl), K, 512, gl, seed=len(gl) * 7 + K, extra_rows=2)
    if fmt in ("int4", "int8"):
        # larger outputs so that silu is exercised away from 0 as well
        case["x"] = oracle.f32_to_bf16_bits(oracle.bf16_bits_to_f32(case["x"]) * 4.0)
    got = _run(case)
    H.assert_close(got, _expected(case), rows=slice(0, gl[-1]), what=f"swiglu {fmt}")
    assert (got[gl[-1]:] == 0x7FC0).all(), "rows beyond group_list[-1] were written"


@pytest.mark.parametrize("fmt", K_CONTIG)
@pytest.mark.parametrize("gl", [[2, 3, 4, 40], [130, 130, 143, 300, 301], [0, 7, 7, 8], [0, 200, 200, 200]],
                         ids=["small", "prefill", "decode", "one_big"])
def test_swiglu_epilogue_k_contiguous(fmt, gl):
    """K-contiguous containers: gate and up rows interleaved in blocks of 16 (the decode-sized batches stay on
    the GEMM kernels: the weight-streaming GEMV kernels have no fused activation)."""
    _say(f"swiglu fmt={fmt} gl={gl}")
    case = H.make_case(fmt, len(gl), 512, 512, gl, seed=len(gl) * 11 + len(fmt), extra_rows=2)
    if fmt == "bf16":
        case["x"] = oracle.f32_to_bf16_bits(oracle.bf16_bits_to_f32(case["x"]) * 4.0)
    got = _run(case)
    H.assert_close(got, _expected(case), rows=slice(0, gl[-1]), what=f"swiglu {fmt}")
    assert (got[gl[-1]:] == 0x7FC0).all(), "rows beyond group_list[-1] were written"


def test_swiglu_fp8_half_empty_last_tile():
    _say("swiglu fp8 N=384")
    gl = [5, 140, 140, 301]
    case = H.make_case("fp8", len(gl), 256, 384, gl, seed=5, extra_rows=2)
    got = _run(case)
    H.assert_close(got, _expected(case), rows=slice(0, gl[-1]), what="swiglu fp8 N=384")
    assert (got[gl[-1]:] == 0x7FC0).all(), "rows beyond group_list[-1] were written"


@pytest.mark.parametrize("fmt,N", [("int8", 512), ("fp8", 512), ("fp8", 384)])
def test_swiglu_one_byte_containers_with_many_rows_per_expert(fmt, N):
    """The fused activation on the 4-wavefront kind as the one-byte containers use it (more than 160 rows per expert on
    average)."""
    _say(f"swiglu {fmt} N={N}, many rows per expert")
    counts = [400, 0, 333, 161, 170, 529, 16, 1, 320, 200]
    gl = list(np.cumsum(counts))
    case = H.make_case(fmt, len(gl), 256, N, gl, seed=9 + N, extra_rows=2)
    if fmt == "int8":
        case["x"] = oracle.f32_to_bf16_bits(oracle.bf16_bits_to_f32(case["x"]) * 4.0)
    got = _run(case)
    H.assert_close(got, _expected(case), rows=slice(0, gl[-1]), what=f"swiglu {fmt} N={N}")
    assert (got[gl[-1]:] == 0x7FC0).all(), "rows beyond group_list[-1] were written"


def test_swiglu_int4_prefill_tile_sizes():
    """Every row-block count of the int4 prefill kernel (1..10 blocks of 16 rows) and ragged last blocks."""
    _say("swiglu int4 tile sizes")
    counts = [160, 1, 17, 33, 49, 65, 81, 97, 113, 129, 145, 159]
    gl = list(np.cumsum(counts))
    case = H.make_case("int4", len(gl), 256, 256, gl, seed=77)
    case["x"] = oracle.f32_to_bf16_bits(oracle.bf16_bits_to_f32(case["x"]) * 8.0)
    got = _run(case)
    H.assert_close(got, _expected(case), what="swiglu int4 tiles")


def test_swiglu_via_module_and_rejections():
    import cinfer_ascendc
    import moe_gfx950 as mg

    _say("swiglu via cinfer_ascendc")
    gl = [12, 25, 44, 48]
    case = H.make_case("int4", 4, 512, 512, gl, seed=5)
    dev = H.upload(case)
    out = torch.zeros(case["M"], 256, dtype=torch.bfloat16, device="cuda")
    cinfer_ascendc.grouped_gemm_swiglu(dev["x"].view(torch.bfloat16), dev["weight"], dev["scale"].view(torch.bfloat16),
                                       torch.zeros(1, dtype=torch.bfloat16, device="cuda"), dev["group_list"], "int4", out)
    torch.cuda.synchronize()
    H.assert_close(H.bits(out.cpu()), _expected(case), what="module swiglu")
    # the GEMV op has no fused epilogue
    t = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    a = mg.grouped_args(mg.FMT_INT4, t.data_ptr(), t.data_ptr(), t.data_ptr(), 0, t.data_ptr(), t.data_ptr(), 4, 256, 256, 2,
                        2, epilogue=mg.EPILOGUE_SWIGLU)
    with pytest.raises(mg.MoeError) as e:
        mg.grouped_gemv(a)
    assert e.value.status == mg.ERR_BAD_FORMAT
