"""Host-side checks that need no GPU: the C ABI library loads and exports every
declared symbol, argument validation returns the documented codes, the Python
module keeps the reference's names, and the header and the library agree."""
import ctypes
import os
import re

import pytest

import moe_gfx950 as mg

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
P = 0x1000  # a fake, 16-byte-aligned, non-NULL device address (never dereferenced by validate)


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "moe_gfx950.h")).read()
    declared = set(re.findall(r"\b(moe_[a-z0-9_]+)\s*\(", header))
    assert declared == set(mg.SYMBOLS)
    for name in declared:
        assert hasattr(mg.lib, name), name
    assert mg.lib.moe_abi_version() == int(re.search(r"MOE_GFX950_ABI_VERSION (\d+)", header).group(1))


def test_struct_sizes_match_header_layout():
    assert ctypes.sizeof(mg.GroupedArgs) == 6 * 8 + 5 * 8 + 2 * 4
    assert ctypes.sizeof(mg.DequantArgs) == 3 * 8 + 2 * 8 + 2 * 4


def test_compute_type_strings():
    # "fp4" / "fp8" are the reference's values (grouped_gemm/src/grouped_gemm.cpp:129-135)
    assert mg.format_from_compute_type("fp4") == mg.FMT_FP4_REF
    assert mg.format_from_compute_type("fp8") == mg.FMT_FP8_REF
    assert [mg.format_from_compute_type(s) for s in ("int8", "int4", "fp4_b32", "bf16", "fp4_b16")] == [2, 3, 4, 5, 6]
    for bad in ("", "FP4", "fp16", "int2"):
        assert mg.format_from_compute_type(bad) == mg.ERR_BAD_FORMAT
    assert mg.lib.moe_format_from_compute_type(None) == mg.ERR_BAD_FORMAT


def test_strerror_covers_all_codes():
    seen = {mg.strerror(c) for c in range(0, -8, -1)}
    assert len(seen) == 8 and "unknown moe_status" not in seen
    assert "unknown" in mg.strerror(-99)


def gargs(fmt, M=8, K=256, N=512, G=2, scale_rows=None, **kw):
    if scale_rows is None:
        scale_rows = {mg.FMT_FP4_REF: K // 16, mg.FMT_INT4: K // 128}.get(fmt, 1)
    a = mg.grouped_args(fmt, P, P, P, P, P, P, M, K, N, G, scale_rows)
    for k, v in kw.items():
        setattr(a, k, v)
    return a


@pytest.mark.parametrize("op", ["gemm", "gemv"])
def test_grouped_validate_accepts_good_and_rejects_bad(op):
    val = getattr(mg.lib, f"moe_grouped_{op}_validate")
    fmts = [0, 1, 2, 3, 4, 5, 6] if op == "gemm" else [0, 1, 3, 4, 5, 6]
    for fmt in fmts:
        assert val(ctypes.byref(gargs(fmt))) == mg.MOE_OK, fmt
    assert val(None) == mg.ERR_NULL_POINTER
    assert val(ctypes.byref(gargs(0, format=7))) == mg.ERR_BAD_FORMAT
    assert val(ctypes.byref(gargs(0, format=-1))) == mg.ERR_BAD_FORMAT
    assert val(ctypes.byref(gargs(0, epilogue=2))) == mg.ERR_BAD_FORMAT       # unknown epilogue
    assert val(ctypes.byref(gargs(0, epilogue=1))) == (mg.MOE_OK if op == "gemm" else mg.ERR_BAD_FORMAT)
    assert val(ctypes.byref(gargs(4, epilogue=1))) == (mg.MOE_OK if op == "gemm" else mg.ERR_BAD_FORMAT)
    assert val(ctypes.byref(gargs(0, M=-1))) == mg.ERR_BAD_SHAPE
    assert val(ctypes.byref(gargs(0, G=0))) == mg.ERR_BAD_SHAPE
    assert val(ctypes.byref(gargs(0, K=1 << 31, scale_rows=(1 << 31) // 16))) == mg.ERR_TOO_LARGE  # reference limit
    # any expert count up to 65535 (beyond what LDS holds a tile table for, the kernels walk group_list instead)
    assert val(ctypes.byref(gargs(0, G=1025))) == mg.MOE_OK
    assert val(ctypes.byref(gargs(0, G=65535))) == mg.MOE_OK
    assert val(ctypes.byref(gargs(0, G=65536))) == mg.ERR_TOO_LARGE
    assert val(ctypes.byref(gargs(0, weight=None))) == mg.ERR_NULL_POINTER
    assert val(ctypes.byref(gargs(0, group_list=None))) == mg.ERR_NULL_POINTER
    assert val(ctypes.byref(gargs(0, scale=None))) == mg.ERR_NULL_POINTER
    assert val(ctypes.byref(gargs(5, scale=None))) == mg.MOE_OK            # bf16 has no scale
    assert val(ctypes.byref(gargs(0, M=0, x=None, y=None))) == mg.MOE_OK   # empty batch
    assert val(ctypes.byref(gargs(0, x=None))) == mg.ERR_NULL_POINTER
    assert val(ctypes.byref(gargs(0, N=384))) == mg.ERR_BAD_ALIGNMENT      # fp4 tiles are 256 columns wide
    assert val(ctypes.byref(gargs(0, K=96, scale_rows=6))) == mg.ERR_BAD_ALIGNMENT
    assert val(ctypes.byref(gargs(0, scale_rows=3))) == mg.ERR_BAD_SHAPE   # fp4 scale groups are 16 k
    assert val(ctypes.byref(gargs(3, scale_rows=16))) == mg.ERR_BAD_ALIGNMENT  # int4 group of 16 < 32
    assert val(ctypes.byref(gargs(3, scale_rows=3))) == mg.ERR_BAD_SHAPE
    assert val(ctypes.byref(gargs(0, x=P + 2))) == mg.ERR_BAD_ALIGNMENT
    assert val(ctypes.byref(gargs(0, group_list=P + 4))) == mg.ERR_BAD_ALIGNMENT


@pytest.mark.parametrize("op", ["gemm", "gemv"])
def test_slab_and_grid_limits(op):
    """One expert's weight / scale slab is addressed with 32-bit byte offsets, and the GEMV grids carry the
    expert index in their y dimension: sizes beyond either are refused, not wrapped."""
    val = getattr(mg.lib, f"moe_grouped_{op}_validate")
    # bf16 [N, K]: 32768 x 32768 x 2 bytes = 2 GiB per expert; one row of tiles less fits
    assert val(ctypes.byref(gargs(5, K=32768, N=32768))) == mg.ERR_TOO_LARGE
    assert val(ctypes.byref(gargs(5, K=32768, N=32768 - 256))) == mg.MOE_OK
    # fp8: one byte per weight, 46336 x 46336 < 2 GiB <= 46464 x 46464
    assert val(ctypes.byref(gargs(1, K=46336, N=46336))) == mg.MOE_OK
    assert val(ctypes.byref(gargs(1, K=46464, N=46464))) == mg.ERR_TOO_LARGE
    # 4-bit codes: the fp4_b16 scales (K N / 8 bytes) stay below the codes (K N / 2 bytes)
    assert val(ctypes.byref(gargs(6, K=65536, N=65536))) == mg.ERR_TOO_LARGE
    assert val(ctypes.byref(gargs(6, K=65536, N=32768))) == mg.MOE_OK
    # a 256-row tile of x or y must stay below 2 GiB as well
    assert val(ctypes.byref(gargs(5, K=1 << 22, N=256))) == mg.ERR_TOO_LARGE
    if op == "gemv":
        assert val(ctypes.byref(gargs(5, G=65535))) == mg.MOE_OK
        assert val(ctypes.byref(gargs(5, G=65536))) == mg.ERR_TOO_LARGE


@pytest.mark.parametrize("op", ["gemm", "gemv"])
def test_fp8_accepts_n_multiple_of_128(op):
    # the reference tiles uint8 weights 128 columns wide (grouped_gemm/op_host/grouped_matmul_antiquant_tiling.cpp:616-621)
    val = getattr(mg.lib, f"moe_grouped_{op}_validate")
    assert val(ctypes.byref(gargs(1, N=384))) == mg.MOE_OK
    assert val(ctypes.byref(gargs(1, N=1408))) == mg.MOE_OK
    assert val(ctypes.byref(gargs(1, N=320))) == mg.ERR_BAD_ALIGNMENT
    assert val(ctypes.byref(gargs(3, N=384))) == mg.ERR_BAD_ALIGNMENT      # the other N-contiguous containers: 256
    assert val(ctypes.byref(gargs(1, N=384, G=1025))) == mg.MOE_OK


def test_route_static_limit_is_checked_on_the_host():
    # (ceil(T * topk / 1024) + 1) * E * 4 bytes of scratch: 1024 experts, 2^20 choices -> 4 MiB > 2 MiB
    a = mg.route_args(P, 0, P, P, P, P, P, 0, 0, 1 << 17, 1024, 0, 8)
    assert mg.route_workspace_bytes(a) > mg.ROUTE_STATIC_SCRATCH_BYTES
    assert mg.lib.moe_route_static(ctypes.byref(a), None) == mg.ERR_TOO_LARGE
    assert mg.lib.moe_route_static(None, None) == mg.ERR_NULL_POINTER


def test_gemm_needs_offset_only_for_int8_and_gemv_rejects_int8():
    assert mg.lib.moe_grouped_gemm_validate(ctypes.byref(gargs(2, offset=None))) == mg.ERR_NULL_POINTER
    assert mg.lib.moe_grouped_gemm_validate(ctypes.byref(gargs(3, offset=None))) == mg.MOE_OK
    assert mg.lib.moe_grouped_gemv_validate(ctypes.byref(gargs(2))) == mg.ERR_BAD_FORMAT


def test_fp4_b32_k_alignment_differs_between_gemm_and_gemv():
    # the GEMM tile routine of fp4_b32 steps through K 128 at a time; the GEMV reads whole 32-k blocks
    assert mg.lib.moe_grouped_gemm_validate(ctypes.byref(gargs(4, K=192, scale_rows=6))) == mg.ERR_BAD_ALIGNMENT
    assert mg.lib.moe_grouped_gemm_validate(ctypes.byref(gargs(4, K=256, scale_rows=8))) == mg.MOE_OK
    assert mg.lib.moe_grouped_gemv_validate(ctypes.byref(gargs(4, K=192, scale_rows=6))) == mg.MOE_OK
    assert mg.lib.moe_grouped_gemv_validate(ctypes.byref(gargs(4, K=48, scale_rows=1))) == mg.ERR_BAD_ALIGNMENT


def test_dequant_validate():
    val = mg.lib.moe_dequant_fp4_bf16_validate
    ok = mg.DequantArgs(P, P, P, 16, 256, 32, 0)
    assert val(ctypes.byref(ok)) == mg.MOE_OK
    assert val(None) == mg.ERR_NULL_POINTER
    assert val(ctypes.byref(mg.DequantArgs(P, P, P, 16, 256, 64, 0))) == mg.ERR_BAD_FORMAT
    assert val(ctypes.byref(mg.DequantArgs(P, P, P, 16, 256, 32, 1))) == mg.ERR_BAD_FORMAT
    assert val(ctypes.byref(mg.DequantArgs(P, P, P, -1, 256, 32, 0))) == mg.ERR_BAD_SHAPE
    assert val(ctypes.byref(mg.DequantArgs(P, P, P, 16, 250, 32, 0))) == mg.ERR_BAD_ALIGNMENT
    assert val(ctypes.byref(mg.DequantArgs(P, P, P, 16, 48, 16, 0))) == mg.MOE_OK
    assert val(ctypes.byref(mg.DequantArgs(None, P, P, 16, 256, 32, 0))) == mg.ERR_NULL_POINTER
    assert val(ctypes.byref(mg.DequantArgs(None, None, None, 0, 256, 32, 0))) == mg.MOE_OK
    assert val(ctypes.byref(mg.DequantArgs(P + 4, P, P, 16, 256, 32, 0))) == mg.ERR_BAD_ALIGNMENT


def test_workspace_is_zero_for_every_op():
    assert mg.lib.moe_grouped_gemm_workspace_bytes(ctypes.byref(gargs(3))) == 0
    assert mg.lib.moe_grouped_gemv_workspace_bytes(ctypes.byref(gargs(5))) == 0
    assert mg.lib.moe_dequant_fp4_bf16_workspace_bytes(ctypes.byref(mg.DequantArgs(P, P, P, 1, 32, 32, 0))) == 0


def test_launch_entry_points_validate_before_touching_the_gpu():
    # invalid arguments must come back as codes even on a machine without a GPU
    assert mg.lib.moe_grouped_gemm(ctypes.byref(gargs(0, N=384)), None) == mg.ERR_BAD_ALIGNMENT
    assert mg.lib.moe_grouped_gemv(ctypes.byref(gargs(2)), None) == mg.ERR_BAD_FORMAT
    assert mg.lib.moe_dequant_fp4_bf16(ctypes.byref(mg.DequantArgs(P, P, P, 1, 30, 32, 0)), None) == mg.ERR_BAD_ALIGNMENT
    with pytest.raises(mg.MoeError) as e:
        mg.grouped_gemm(gargs(0, N=384))
    assert e.value.status == mg.ERR_BAD_ALIGNMENT
    # an empty batch is a no-op
    assert mg.lib.moe_grouped_gemm(ctypes.byref(gargs(0, M=0, x=None, y=None)), None) == mg.MOE_OK


def test_python_module_keeps_the_reference_api():
    # pybind.cpp:14-19: function names and keyword names, in order
    import cinfer_ascendc

    doc = cinfer_ascendc.grouped_gemm.__doc__
    assert re.search(r"grouped_gemm\(x: .*, weight: .*, antiquantScaleOptional: .*, antiquantOffsetOptional: .*, "
                     r"groupListOptional: .*, computeType: str, output: .*\) -> None", doc)
    doc = cinfer_ascendc.grouped_soft_gemv.__doc__
    assert re.search(r"grouped_soft_gemv\(x: .*, weight: .*, scale: .*, groupList: .*, computeType: str, "
                     r"output: .*\) -> None", doc)
    for op in ("grouped_gemm", "grouped_soft_gemv"):   # check_installed_ops.py:14-19
        assert hasattr(cinfer_ascendc, op)


def test_python_module_rejects_bad_arguments_on_cpu():
    import torch

    import cinfer_ascendc

    x = torch.zeros(4, 256, dtype=torch.bfloat16)
    w = torch.zeros(2, 256, 256, dtype=torch.int8)
    s = torch.zeros(2, 16, 512, dtype=torch.bfloat16)
    gl = torch.tensor([2, 4])
    y = torch.zeros(4, 512, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="Invalid compute type"):   # grouped_gemm.cpp:129-133
        cinfer_ascendc.grouped_gemm(x, w, s, s, gl, "fp16", y)
    with pytest.raises(RuntimeError, match="GPU"):
        cinfer_ascendc.grouped_gemm(x=x, weight=w, output=y, antiquantOffsetOptional=s, antiquantScaleOptional=s,
                                    groupListOptional=gl, computeType="fp4")
    with pytest.raises(RuntimeError):
        cinfer_ascendc.grouped_soft_gemv(x, w, s, gl, "nope", y)
