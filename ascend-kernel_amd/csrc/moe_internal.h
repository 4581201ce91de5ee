// Host-side declarations shared by the launchers and the C ABI.
#pragma once
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdint>

#include "moe_gfx950.h"

namespace moe {
// Raises a kernel's dynamic LDS limit once per GPU (the attribute belongs to the kernel's image on the
// current device).  `done` is that kernel's bit mask of devices already set up: the only state the
// launchers keep.  A race repeats the same call.
inline int ensure_dynamic_lds(const void* kernel, int bytes, std::atomic<uint64_t>& done) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return MOE_ERR_NO_DEVICE;
    if (!((done.load(std::memory_order_acquire) >> dev) & 1u)) {
        if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) return MOE_ERR_LAUNCH;
        done.fetch_or(uint64_t{1} << dev, std::memory_order_release);
    }
    return MOE_OK;
}

int launch_dequant_fp4_bf16(const moe_dequant_args* a, hipStream_t stream);
// gemm_rounding: use the grouped GEMM's arithmetic (weights rounded to bf16) where the two ops differ.
int launch_grouped_gemv(const moe_grouped_args* a, hipStream_t stream, bool gemm_rounding = false);
// True when the GEMV launcher is the faster path for a grouped GEMM call of this shape.
bool gemv_preferred(const moe_grouped_args* a);
// grouped GEMV on the fp4 / int4 N-contiguous containers by the k-split GEMM kernel run with the GEMV
// op's arithmetic; MOE_ERR_TOO_LARGE when the expert count does not fit its LDS
int launch_gemm_exact(const moe_grouped_args* a, hipStream_t stream);
int launch_grouped_gemm(const moe_grouped_args* a, hipStream_t stream);
// moves the grouped GEMM's launch number (which picks a launch's tile counter and stamp) by delta; returns the new number
int64_t gemm_shift_launch_number(int64_t delta);
int launch_prepack_fp4_ref(const moe_prepack_fp4_args* a, hipStream_t stream);
int launch_route(const moe_route_args* a, hipStream_t stream);
// the same with the workspace in the library's own static device array (a->workspace is ignored)
int launch_route_static(const moe_route_args* a, hipStream_t stream);
size_t route_workspace_bytes(const moe_route_args* a);
}  // namespace moe
