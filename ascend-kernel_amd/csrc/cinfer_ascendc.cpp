// Python module `cinfer_ascendc`: same functions, keyword names and argument order as
// the reference's pybind module (pybind.cpp:13-19), on top of the C ABI of
// libmoe_gfx950.so.  This file is host glue only: argument checks, the current HIP
// stream, and the translation of at::Tensor into raw pointers and sizes.
//
// Differences from the reference adapters (grouped_gemm/src/grouped_gemm.cpp:122-161,
// grouped_soft_gemv/src/grouped_soft_gemv.cpp:123-155): shapes, dtypes, devices and
// contiguity are validated before the launch; no workspace is allocated or cached;
// computeType accepts "int8", "int4", "fp4_b32", "fp4_b16" and "bf16" besides "fp4" and "fp8";
// dequant_fp4, the fp4 weight preparation, routing and the fused-SwiGLU GEMM are extra entry points.  Every failure raises RuntimeError, as the
// reference does.
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>

#include <tuple>
#include <torch/extension.h>

#include <stdexcept>
#include <string>

#include "moe_gfx950.h"

namespace {

[[noreturn]] void fail(const std::string& what) { throw std::runtime_error("cinfer_ascendc: " + what); }

void check_status(int rc, const char* op) {
    if (rc != MOE_OK) fail(std::string(op) + ": " + moe_strerror(rc));
}

void check_tensor(const at::Tensor& t, const char* name, at::ScalarType dtype, int64_t dim, const at::Tensor& like) {
    if (!t.defined()) fail(std::string(name) + " is undefined");
    if (!t.is_cuda()) fail(std::string(name) + " must be on the GPU");
    if (t.device() != like.device()) fail(std::string(name) + " is on a different device than x");
    if (t.scalar_type() != dtype) fail(std::string(name) + " has dtype " + c10::toString(t.scalar_type()) +
                                       ", expected " + c10::toString(dtype));
    if (t.dim() != dim) fail(std::string(name) + " must have " + std::to_string(dim) + " dimensions");
    if (!t.is_contiguous()) fail(std::string(name) + " must be contiguous");
}

int parse_format(const char* computeType) {
    const int fmt = moe_format_from_compute_type(computeType);
    if (fmt < 0)
        fail(std::string("Invalid compute type: ") + (computeType ? computeType : "(null)") +
             ". Supported: \"fp4\", \"fp8\", \"int8\", \"int4\", \"fp4_b32\", \"fp4_b16\", \"bf16\"");
    return fmt;
}

// Fills args from the tensors; returns the logical (K, N) through args.
void fill_grouped(moe_grouped_args& a, const at::Tensor& x, const at::Tensor& weight, const at::Tensor& scale,
                  const at::Tensor* offset, const at::Tensor& groupList, int fmt, const at::Tensor& output,
                  int epilogue = MOE_EPILOGUE_NONE) {
    if (!x.defined() || !x.is_cuda()) fail("x must be a GPU tensor");
    check_tensor(x, "x", at::kBFloat16, 2, x);
    check_tensor(output, "output", at::kBFloat16, 2, x);
    check_tensor(groupList, "groupList", at::kLong, 1, x);
    const int64_t M = x.size(0), K = x.size(1), G = groupList.size(0);
    int64_t N = 0, scale_rows = 1;
    auto want = [&](const at::Tensor& t, const char* name, std::initializer_list<int64_t> shape) {
        if (t.sizes() != at::IntArrayRef(shape)) {
            std::string s = std::string(name) + " has shape [";
            for (auto d : t.sizes()) s += std::to_string(d) + ",";
            s += "], expected [";
            for (auto d : shape) s += std::to_string(d) + ",";
            fail(s + "]");
        }
    };
    switch (fmt) {
        case MOE_FMT_FP4_REF:
            // int8 [G, K, N/2] (grouped_gemm/src/grouped_gemm.cpp:134-135 re-describes it as INT4 [G, K, N])
            check_tensor(weight, "weight", at::kChar, 3, x);
            N = weight.size(2) * 2;
            want(weight, "weight", {G, K, N / 2});
            check_tensor(scale, "scale", at::kBFloat16, 3, x);
            want(scale, "scale", {G, K / 16, N});
            scale_rows = K / 16;
            break;
        case MOE_FMT_FP8_REF:
            check_tensor(weight, "weight", at::kByte, 3, x);
            N = weight.size(2);
            want(weight, "weight", {G, K, N});
            check_tensor(scale, "scale", at::kFloat, 3, x);
            want(scale, "scale", {G, (K + 127) / 128, (N + 127) / 128});
            break;
        case MOE_FMT_INT8:
            check_tensor(weight, "weight", at::kChar, 3, x);
            N = weight.size(2);
            want(weight, "weight", {G, K, N});
            check_tensor(scale, "scale", at::kBFloat16, 2, x);
            want(scale, "scale", {G, N});
            if (!offset) fail("computeType \"int8\" needs an offset tensor");
            check_tensor(*offset, "offset", at::kBFloat16, 2, x);
            want(*offset, "offset", {G, N});
            break;
        case MOE_FMT_INT4:
            if (weight.defined() && weight.scalar_type() == at::kChar)
                check_tensor(weight, "weight", at::kChar, 3, x);
            else
                check_tensor(weight, "weight", at::kByte, 3, x);
            N = weight.size(2) * 2;
            want(weight, "weight", {G, K, N / 2});
            check_tensor(scale, "scale", at::kBFloat16, 3, x);
            scale_rows = scale.size(1);
            want(scale, "scale", {G, scale_rows, N});
            break;
        case MOE_FMT_FP4_B32:
        case MOE_FMT_FP4_B16:
            check_tensor(weight, "weight", at::kByte, 3, x);
            N = weight.size(1);
            want(weight, "weight", {G, N, K / 2});
            check_tensor(scale, "scale", at::kBFloat16, 3, x);
            want(scale, "scale", {G, N, K / (fmt == MOE_FMT_FP4_B32 ? 32 : 16)});
            break;
        default:  // MOE_FMT_BF16
            check_tensor(weight, "weight", at::kBFloat16, 3, x);
            N = weight.size(1);
            want(weight, "weight", {G, N, K});
            break;
    }
    want(output, "output", {M, epilogue == MOE_EPILOGUE_SWIGLU ? N / 2 : N});
    a.x = x.data_ptr();
    a.weight = weight.data_ptr();
    a.scale = fmt == MOE_FMT_BF16 ? nullptr : scale.data_ptr();
    a.offset = (fmt == MOE_FMT_INT8 && offset) ? offset->data_ptr() : nullptr;
    a.group_list = groupList.data_ptr<int64_t>();
    a.y = output.data_ptr();
    a.M = M; a.K = K; a.N = N; a.G = G;
    a.scale_rows = scale_rows;
    a.format = fmt;
    a.epilogue = epilogue;
}

moe_stream_t current_stream(const at::Tensor& x) {
    return static_cast<moe_stream_t>(c10::hip::getCurrentHIPStream(x.device().index()).stream());
}

// pybind.cpp:17-19
void GroupedGemm(at::Tensor x, at::Tensor weight, at::Tensor antiquantScaleOptional,
                 at::Tensor antiquantOffsetOptional, at::Tensor groupListOptional, const char* computeType,
                 at::Tensor output) {
    const int fmt = parse_format(computeType);
    moe_grouped_args a;
    fill_grouped(a, x, weight, antiquantScaleOptional, &antiquantOffsetOptional, groupListOptional, fmt, output);
    c10::DeviceGuard guard(x.device());
    check_status(moe_grouped_gemm(&a, current_stream(x)), "grouped_gemm");
}

// Extra entry point: grouped_gemm with the SwiGLU activation fused into its epilogue (see moe_epilogue in
// moe_gfx950.h): weight columns in groups of (gate 2j, gate 2j+1, up 2j, up 2j+1) on the N-contiguous containers, weight rows
// in blocks of (16 gate, 16 up) on the K-contiguous ones; output [M, N/2].
void GroupedGemmSwiglu(at::Tensor x, at::Tensor weight, at::Tensor antiquantScaleOptional,
                       at::Tensor antiquantOffsetOptional, at::Tensor groupListOptional, const char* computeType,
                       at::Tensor output) {
    const int fmt = parse_format(computeType);
    moe_grouped_args a;
    fill_grouped(a, x, weight, antiquantScaleOptional, &antiquantOffsetOptional, groupListOptional, fmt, output,
                 MOE_EPILOGUE_SWIGLU);
    c10::DeviceGuard guard(x.device());
    check_status(moe_grouped_gemm(&a, current_stream(x)), "grouped_gemm_swiglu");
}

// pybind.cpp:14-16
void GroupedSoftGemv(at::Tensor x, at::Tensor weight, at::Tensor scale, at::Tensor groupList,
                     const char* computeType, at::Tensor output) {
    const int fmt = parse_format(computeType);
    moe_grouped_args a;
    fill_grouped(a, x, weight, scale, nullptr, groupList, fmt, output);
    c10::DeviceGuard guard(x.device());
    check_status(moe_grouped_gemv(&a, current_stream(x)), "grouped_soft_gemv");
}

// Extra entry point: codes uint8 [R, C/2], scale bf16 [R, C/block] -> output bf16 [R, C].
void DequantFp4(at::Tensor weight, at::Tensor scale, at::Tensor output) {
    if (!weight.defined() || !weight.is_cuda()) fail("weight must be a GPU tensor");
    check_tensor(weight, "weight", at::kByte, 2, weight);
    check_tensor(scale, "scale", at::kBFloat16, 2, weight);
    check_tensor(output, "output", at::kBFloat16, 2, weight);
    const int64_t R = weight.size(0), C = weight.size(1) * 2;
    if (output.size(0) != R || output.size(1) != C) fail("output must be [rows, 2 * weight.shape[1]]");
    if (scale.size(0) != R || scale.size(1) == 0 || C % scale.size(1)) fail("scale must be [rows, cols / block]");
    moe_dequant_args a;
    a.codes = weight.data_ptr();
    a.scale = scale.data_ptr();
    a.out = output.data_ptr();
    a.rows = R; a.cols = C;
    a.block = static_cast<int32_t>(C / scale.size(1));
    a.reserved = 0;
    c10::DeviceGuard guard(weight.device());
    check_status(moe_dequant_fp4_bf16(&a, current_stream(weight)), "dequant_fp4");
}

// Extra entry points: the weight preparation the reference's tests do on the host with torch
// reshapes (repack_weight + repack_weight_step2, anti_quant_fp8_scale + transpose;
// grouped_gemm/test/python/test_group_gemm_fp4.py:86-142, :180-186), as GPU ops that return new tensors.

// checkpoint codes uint8 [G, N, K/2] -> "fp4" op weight int8 [G, K, N/2]
at::Tensor RepackWeightFp4(at::Tensor weight) {
    if (!weight.defined() || !weight.is_cuda()) fail("weight must be a GPU tensor");
    check_tensor(weight, "weight", at::kByte, 3, weight);
    const int64_t G = weight.size(0), N = weight.size(1), K = weight.size(2) * 2;
    at::Tensor out = at::empty({G, K, N / 2}, weight.options().dtype(at::kChar));
    moe_prepack_fp4_args a = {};
    a.codes = weight.data_ptr();
    a.weight_out = out.data_ptr();
    a.G = G; a.N = N; a.K = K;
    c10::DeviceGuard guard(weight.device());
    check_status(moe_prepack_fp4_ref(&a, current_stream(weight)), "repack_weight_fp4");
    return out;
}

// checkpoint scales bf16 [G, N, K/16] (x optional fp32 scale_2 [G, 1 or 2, 1]) -> bf16 [G, K/16, N]
at::Tensor MergeScaleFp4(at::Tensor scale, c10::optional<at::Tensor> scale_2) {
    if (!scale.defined() || !scale.is_cuda()) fail("scale must be a GPU tensor");
    check_tensor(scale, "scale", at::kBFloat16, 3, scale);
    const int64_t G = scale.size(0), N = scale.size(1), KB = scale.size(2);
    at::Tensor out = at::empty({G, KB, N}, scale.options());
    moe_prepack_fp4_args a = {};
    a.scale = scale.data_ptr();
    a.scale_out = out.data_ptr();
    a.G = G; a.N = N; a.K = KB * 16;
    at::Tensor s2;
    if (scale_2 && scale_2->defined()) {
        s2 = *scale_2;
        if (!s2.is_cuda() || s2.device() != scale.device()) fail("scale_2 must be on the same device as scale");
        if (s2.scalar_type() != at::kFloat || !s2.is_contiguous()) fail("scale_2 must be a contiguous float32 tensor");
        if (s2.numel() != G && s2.numel() != 2 * G) fail("scale_2 must hold one or two factors per expert");
        a.scale2 = s2.data_ptr();
        a.scale2_cols = static_cast<int32_t>(s2.numel() / G);
    }
    c10::DeviceGuard guard(scale.device());
    check_status(moe_prepack_fp4_ref(&a, current_stream(scale)), "merge_scale_fp4");
    return out;
}

// Extra entry point: routing.  logits fp32 [T, E], x bf16 [T, K] -> (x_sorted bf16 [T*topk, K],
// group_list int64 [E], topk_weight fp32 [T, topk], topk_ids int32 [T, topk], row_of_choice int32
// [T*topk]): what a caller needs before grouped_gemm (rows sorted by expert + the cumulative
// group_list of grouped_matmul_utils.h:304-320) and after it (where each token's k results are).
std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor> MoeRoute(at::Tensor logits, at::Tensor x, int64_t topk) {
    if (!logits.defined() || !logits.is_cuda()) fail("logits must be a GPU tensor");
    check_tensor(logits, "logits", at::kFloat, 2, logits);
    check_tensor(x, "x", at::kBFloat16, 2, logits);
    const int64_t T = logits.size(0), E = logits.size(1), K = x.size(1);
    if (x.size(0) != T) fail("x must have one row per row of logits");
    if (topk <= 0 || topk > E) fail("topk must be in [1, number of experts]");
    const auto opt = logits.options();
    at::Tensor x_sorted = at::empty({T * topk, K}, x.options());
    at::Tensor group_list = at::empty({E}, opt.dtype(at::kLong));
    at::Tensor weight = at::empty({T, topk}, opt);
    at::Tensor ids = at::empty({T, topk}, opt.dtype(at::kInt));
    at::Tensor row_token = at::empty({T * topk}, opt.dtype(at::kInt));
    at::Tensor row_of_choice = at::empty({T * topk}, opt.dtype(at::kInt));
    moe_route_args a = {};
    a.logits = logits.data_ptr();
    a.x = x.data_ptr();
    a.topk_ids = ids.data_ptr();
    a.topk_weight = weight.data_ptr();
    a.group_list = group_list.data_ptr<int64_t>();
    a.row_token = row_token.data_ptr();
    a.row_of_choice = row_of_choice.data_ptr();
    a.x_sorted = x_sorted.data_ptr();
    a.T = T; a.E = E; a.K = K;
    a.topk = static_cast<int32_t>(topk);
    at::Tensor ws = at::empty({static_cast<int64_t>(moe_route_workspace_bytes(&a)) + 4}, opt.dtype(at::kByte));
    a.workspace = ws.data_ptr();
    c10::DeviceGuard guard(logits.device());
    check_status(moe_route(&a, current_stream(logits)), "moe_route");
    return {x_sorted, group_list, weight, ids, row_of_choice};
}

}  // namespace

PYBIND11_MODULE(cinfer_ascendc, m) {
    using namespace pybind11::literals;
    m.def("grouped_soft_gemv", &GroupedSoftGemv, "x"_a, "weight"_a, "scale"_a, "groupList"_a, "computeType"_a,
          "output"_a, "GROUP GEMV.");
    m.def("grouped_gemm", &GroupedGemm, "x"_a, "weight"_a, "antiquantScaleOptional"_a, "antiquantOffsetOptional"_a,
          "groupListOptional"_a, "computeType"_a, "output"_a, "GROUP GEMM.");
    m.def("grouped_gemm_swiglu", &GroupedGemmSwiglu, "x"_a, "weight"_a, "antiquantScaleOptional"_a,
          "antiquantOffsetOptional"_a, "groupListOptional"_a, "computeType"_a, "output"_a,
          "GROUP GEMM with silu(gate) * up fused into the epilogue; output [M, N/2].");
    m.def("dequant_fp4", &DequantFp4, "weight"_a, "scale"_a, "output"_a, "FP4 (e2m1) -> BF16 block dequant.");
    m.def("moe_route", &MoeRoute, "logits"_a, "x"_a, "topk"_a,
          "Router logits -> (x_sorted, group_list, topk_weight, topk_ids, row_of_choice).");
    m.def("repack_weight_fp4", &RepackWeightFp4, "weight"_a,
          "Checkpoint fp4 codes [G, N, K/2] -> the \"fp4\" op weight [G, K, N/2].");
    m.def("merge_scale_fp4", &MergeScaleFp4, "scale"_a, "scale_2"_a = pybind11::none(),
          "Checkpoint block scales [G, N, K/16] (x scale_2) -> the \"fp4\" op scale [G, K/16, N].");
}
