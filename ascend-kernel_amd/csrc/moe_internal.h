// Host-side declarations shared by the launchers and the C ABI.
#pragma once
#include <hip/hip_runtime.h>

#include "moe_gfx950.h"

namespace moe {
int launch_dequant_fp4_bf16(const moe_dequant_args* a, hipStream_t stream);
int launch_grouped_gemv(const moe_grouped_args* a, hipStream_t stream);
int launch_grouped_gemm(const moe_grouped_args* a, hipStream_t stream);
}  // namespace moe
