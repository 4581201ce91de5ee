// C ABI of libmoe_gfx950.so: argument validation (host only, usable without a GPU),
// error strings, and the extern "C" entry points that hand over to the launchers.
#include <cstdint>
#include <cstring>
#include <initializer_list>

#include "moe_internal.h"

namespace {

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline bool fits_i32(int64_t v) { return v >= 0 && v <= 0x7fffffffLL; }

// Checks shared by GEMM and GEMV.  k_mult / n_mult are what the op's kernels
// need on top of what the container itself implies.
int validate_grouped(const moe_grouped_args* a, int64_t k_mult, int64_t n_mult, bool allow_epilogue) {
    if (!a) return MOE_ERR_NULL_POINTER;
    if (a->format < 0 || a->format >= MOE_FMT_COUNT) return MOE_ERR_BAD_FORMAT;
    if (a->epilogue != MOE_EPILOGUE_NONE && (a->epilogue != MOE_EPILOGUE_SWIGLU || !allow_epilogue)) return MOE_ERR_BAD_FORMAT;
    if (a->M < 0 || a->K <= 0 || a->N <= 0 || a->G <= 0) return MOE_ERR_BAD_SHAPE;
    // same limit as the reference: grouped_matmul_antiquant_tiling.cpp:260-264
    if (!fits_i32(a->M) || !fits_i32(a->K) || !fits_i32(a->N) || !fits_i32(a->G)) return MOE_ERR_TOO_LARGE;
    if (!a->weight || !a->group_list) return MOE_ERR_NULL_POINTER;
    if (a->M > 0 && (!a->x || !a->y)) return MOE_ERR_NULL_POINTER;
    if (a->format != MOE_FMT_BF16 && !a->scale) return MOE_ERR_NULL_POINTER;
    if (a->format == MOE_FMT_INT8 && !a->offset) return MOE_ERR_NULL_POINTER;
    if (a->K % k_mult || a->N % n_mult) return MOE_ERR_BAD_ALIGNMENT;
    switch (a->format) {
        case MOE_FMT_FP4_REF:
            // the byte permutation works on 64(k) x 256(n) tiles; groups of 16 along K
            if (a->K % 64 || a->N % 256) return MOE_ERR_BAD_ALIGNMENT;
            if (a->scale_rows * 16 != a->K) return MOE_ERR_BAD_SHAPE;
            break;
        case MOE_FMT_FP8_REF:
            if (a->K % 128 || a->N % 128) return MOE_ERR_BAD_ALIGNMENT;
            break;
        case MOE_FMT_INT4:
            if (a->scale_rows <= 0 || a->K % a->scale_rows) return MOE_ERR_BAD_SHAPE;
            if ((a->K / a->scale_rows) % 32) return MOE_ERR_BAD_ALIGNMENT;
            break;
        case MOE_FMT_FP4_B32:
        case MOE_FMT_FP4_B16:
            if (a->K % 32) return MOE_ERR_BAD_ALIGNMENT;
            break;
        default:
            break;
    }
    if (!aligned16(a->x) || !aligned16(a->weight) || !aligned16(a->y) || !aligned16(a->scale) ||
        !aligned16(a->offset) || (reinterpret_cast<uintptr_t>(a->group_list) & 7u))
        return MOE_ERR_BAD_ALIGNMENT;
    // The kernels address one expert's weight and scale slab, and one tile's rows of x and y, with 32-bit
    // byte offsets through buffer resources: each must stay below 2 GiB.
    const int64_t lim = int64_t{1} << 31;
    const int64_t kn = a->K * a->N;   // both fit int32
    int64_t wbytes = kn, sbytes = 0;
    switch (a->format) {
        case MOE_FMT_FP4_REF: wbytes = kn / 2; sbytes = a->scale_rows * a->N * 2; break;
        case MOE_FMT_FP8_REF: sbytes = (a->K / 128) * (a->N / 128) * 4; break;
        case MOE_FMT_INT8: sbytes = a->N * 2; break;
        case MOE_FMT_INT4: wbytes = kn / 2; sbytes = a->scale_rows * a->N * 2; break;
        case MOE_FMT_FP4_B32: wbytes = kn / 2; sbytes = kn / 32 * 2; break;
        case MOE_FMT_FP4_B16: wbytes = kn / 2; sbytes = kn / 16 * 2; break;
        case MOE_FMT_BF16: wbytes = kn * 2; break;
        default: break;
    }
    const int64_t tile_rows = 256;   // upper bound on the rows of one tile
    if (wbytes >= lim || sbytes >= lim || tile_rows * a->K * 2 >= lim || tile_rows * a->N * 2 >= lim) return MOE_ERR_TOO_LARGE;
    return MOE_OK;
}

}  // namespace

extern "C" {

int moe_abi_version(void) { return MOE_GFX950_ABI_VERSION; }

const char* moe_strerror(int status) {
    switch (status) {
        case MOE_OK: return "ok";
        case MOE_ERR_NULL_POINTER: return "a required pointer is NULL";
        case MOE_ERR_BAD_FORMAT: return "unknown weight format / computeType";
        case MOE_ERR_BAD_SHAPE: return "shape not valid for this weight format";
        case MOE_ERR_BAD_ALIGNMENT: return "size or pointer alignment not supported by the kernels";
        case MOE_ERR_TOO_LARGE: return "M, K, N or G out of int32 range, an expert's weight or scale slab of 2 GiB or more, or more experts than the op supports";
        case MOE_ERR_LAUNCH: return "kernel launch failed";
        case MOE_ERR_NO_DEVICE: return "no gfx950 device";
        default: return "unknown moe_status";
    }
}

int moe_format_from_compute_type(const char* s) {
    if (!s) return MOE_ERR_BAD_FORMAT;
    if (!std::strcmp(s, "fp4")) return MOE_FMT_FP4_REF;
    if (!std::strcmp(s, "fp8")) return MOE_FMT_FP8_REF;
    if (!std::strcmp(s, "int8")) return MOE_FMT_INT8;
    if (!std::strcmp(s, "int4")) return MOE_FMT_INT4;
    if (!std::strcmp(s, "fp4_b32")) return MOE_FMT_FP4_B32;
    if (!std::strcmp(s, "fp4_b16")) return MOE_FMT_FP4_B16;
    if (!std::strcmp(s, "bf16")) return MOE_FMT_BF16;
    return MOE_ERR_BAD_FORMAT;
}

int moe_dequant_fp4_bf16_validate(const moe_dequant_args* a) {
    if (!a) return MOE_ERR_NULL_POINTER;
    if (a->reserved != 0 || (a->block != 16 && a->block != 32)) return MOE_ERR_BAD_FORMAT;
    if (a->rows < 0 || a->cols < 0) return MOE_ERR_BAD_SHAPE;
    if (a->cols % a->block) return MOE_ERR_BAD_ALIGNMENT;
    if (a->rows > 0 && a->cols > 0 && a->rows > (INT64_MAX / 4) / a->cols) return MOE_ERR_TOO_LARGE;
    if (a->rows * a->cols > 0 && (!a->codes || !a->scale || !a->out)) return MOE_ERR_NULL_POINTER;
    if (!aligned16(a->codes) || !aligned16(a->out) || (reinterpret_cast<uintptr_t>(a->scale) & 1u))
        return MOE_ERR_BAD_ALIGNMENT;
    return MOE_OK;
}

// GEMM: the workgroup tile spans 64 k and 256 n.
int moe_grouped_gemm_validate(const moe_grouped_args* a) {
    // the fp4_b32 tile routine steps through K 128 at a time
    const bool fp4_k = a && (a->format == MOE_FMT_FP4_B32 || a->format == MOE_FMT_FP4_B16);
    // columns: tiles of 256; the reference's fp8 container comes in multiples of 128
    // (grouped_gemm/op_host/grouped_matmul_antiquant_tiling.cpp:616-621), its last tile may be half empty
    const int rc = validate_grouped(a, fp4_k ? 128 : 64, a && a->format == MOE_FMT_FP8_REF ? 128 : 256, true);
    if (rc != MOE_OK) return rc;
    return a->G > MOE_GEMM_MAX_EXPERTS ? MOE_ERR_TOO_LARGE : MOE_OK;
}

// GEMV: N-contiguous containers are read 256 columns per wavefront step,
// K-contiguous ones 8 k per lane.
int moe_grouped_gemv_validate(const moe_grouped_args* a) {
    if (a && a->format == MOE_FMT_INT8) return MOE_ERR_BAD_FORMAT;  // the GEMV op has no offset operand
    const bool k_major = a && (a->format == MOE_FMT_BF16 || a->format == MOE_FMT_FP4_B32 || a->format == MOE_FMT_FP4_B16);
    const int rc = validate_grouped(a, k_major ? 32 : 64, k_major ? 1 : a && a->format == MOE_FMT_FP8_REF ? 128 : 256, false);
    if (rc != MOE_OK) return rc;
    // experts are the y dimension of the GEMV grids
    if (a->G > MOE_GEMM_MAX_EXPERTS) return MOE_ERR_TOO_LARGE;
    return MOE_OK;
}

int moe_prepack_fp4_ref_validate(const moe_prepack_fp4_args* a) {
    if (!a) return MOE_ERR_NULL_POINTER;
    if (a->reserved != 0 || a->scale2_cols < 0 || a->scale2_cols > 2) return MOE_ERR_BAD_FORMAT;
    if (a->G <= 0 || a->N <= 0 || a->K <= 0) return MOE_ERR_BAD_SHAPE;
    if (!fits_i32(a->G) || !fits_i32(a->N) || !fits_i32(a->K)) return MOE_ERR_TOO_LARGE;
    if (a->K % 64 || a->N % 256) return MOE_ERR_BAD_ALIGNMENT;
    // grid dimensions: experts in z, 64-row tiles of N in y
    if (a->G > 65535 || a->N / 64 > 65535) return MOE_ERR_TOO_LARGE;
    if (!a->codes != !a->weight_out || !a->scale != !a->scale_out) return MOE_ERR_NULL_POINTER;
    if (!a->codes && !a->scale) return MOE_ERR_NULL_POINTER;
    if (a->scale2_cols > 0 && a->scale && !a->scale2) return MOE_ERR_NULL_POINTER;
    if (!aligned16(a->codes) || !aligned16(a->weight_out) || !aligned16(a->scale) || !aligned16(a->scale_out) ||
        (reinterpret_cast<uintptr_t>(a->scale2) & 3u))
        return MOE_ERR_BAD_ALIGNMENT;
    return MOE_OK;
}

int moe_route_validate(const moe_route_args* a) {
    if (!a) return MOE_ERR_NULL_POINTER;
    if (a->reserved != 0) return MOE_ERR_BAD_FORMAT;
    if (a->T < 0 || a->E <= 0 || a->topk <= 0 || a->K < 0) return MOE_ERR_BAD_SHAPE;
    if (a->E > 1024 || a->topk > a->E) return MOE_ERR_BAD_SHAPE;
    if (!fits_i32(a->T) || !fits_i32(a->K) || !fits_i32(a->T * a->topk)) return MOE_ERR_TOO_LARGE;
    if (!a->group_list) return MOE_ERR_NULL_POINTER;
    if (a->T > 0 && (!a->topk_ids || !a->row_token || !a->row_of_choice || !a->workspace)) return MOE_ERR_NULL_POINTER;
    if (a->T > 0 && a->logits && !a->topk_weight) return MOE_ERR_NULL_POINTER;
    if (!a->x != !a->x_sorted) return MOE_ERR_NULL_POINTER;
    if (a->x && (a->K <= 0 || a->K % 8)) return MOE_ERR_BAD_ALIGNMENT;
    if (!aligned16(a->x) || !aligned16(a->x_sorted) || (reinterpret_cast<uintptr_t>(a->group_list) & 7u)) return MOE_ERR_BAD_ALIGNMENT;
    for (const void* p : {a->logits, static_cast<const void*>(a->topk_ids), static_cast<const void*>(a->topk_weight),
                          static_cast<const void*>(a->row_token), static_cast<const void*>(a->row_of_choice),
                          static_cast<const void*>(a->workspace)})
        if (reinterpret_cast<uintptr_t>(p) & 3u) return MOE_ERR_BAD_ALIGNMENT;
    return MOE_OK;
}

size_t moe_route_workspace_bytes(const moe_route_args* a) {
    if (!a || a->T <= 0 || a->E <= 0 || a->topk <= 0) return 0;
    return moe::route_workspace_bytes(a);
}

size_t moe_dequant_fp4_bf16_workspace_bytes(const moe_dequant_args*) { return 0; }
size_t moe_prepack_fp4_ref_workspace_bytes(const moe_prepack_fp4_args*) { return 0; }
size_t moe_grouped_gemm_workspace_bytes(const moe_grouped_args*) { return 0; }
size_t moe_grouped_gemv_workspace_bytes(const moe_grouped_args*) { return 0; }

int moe_dequant_fp4_bf16(const moe_dequant_args* a, moe_stream_t stream) {
    int rc = moe_dequant_fp4_bf16_validate(a);
    if (rc != MOE_OK) return rc;
    return moe::launch_dequant_fp4_bf16(a, static_cast<hipStream_t>(stream));
}

int moe_prepack_fp4_ref(const moe_prepack_fp4_args* a, moe_stream_t stream) {
    int rc = moe_prepack_fp4_ref_validate(a);
    if (rc != MOE_OK) return rc;
    return moe::launch_prepack_fp4_ref(a, static_cast<hipStream_t>(stream));
}

int moe_route(const moe_route_args* a, moe_stream_t stream) {
    int rc = moe_route_validate(a);
    if (rc != MOE_OK) return rc;
    return moe::launch_route(a, static_cast<hipStream_t>(stream));
}

int moe_route_static(const moe_route_args* a, moe_stream_t stream) {
    if (!a) return MOE_ERR_NULL_POINTER;
    // args->workspace is not used: validate with a stand-in so that NULL is accepted there
    moe_route_args b = *a;
    b.workspace = reinterpret_cast<void*>(uintptr_t{256});
    int rc = moe_route_validate(&b);
    if (rc != MOE_OK) return rc;
    if (b.T == 0) return moe::launch_route(&b, static_cast<hipStream_t>(stream));   // one kernel that zeroes group_list
    return moe::launch_route_static(a, static_cast<hipStream_t>(stream));
}

int moe_grouped_gemm(const moe_grouped_args* a, moe_stream_t stream) {
    int rc = moe_grouped_gemm_validate(a);
    if (rc != MOE_OK) return rc;
    if (a->M == 0) return MOE_OK;
    return moe::launch_grouped_gemm(a, static_cast<hipStream_t>(stream));
}

int moe_grouped_gemv(const moe_grouped_args* a, moe_stream_t stream) {
    int rc = moe_grouped_gemv_validate(a);
    if (rc != MOE_OK) return rc;
    if (a->M == 0) return MOE_OK;
    return moe::launch_grouped_gemv(a, static_cast<hipStream_t>(stream));
}

int64_t moe_test_shift_launch_number(int64_t delta) { return moe::gemm_shift_launch_number(delta); }

}  // extern "C"
