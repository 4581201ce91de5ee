// FP4 (e2m1) -> BF16 block-scaled dequantization for gfx950: a pure streaming
// kernel.  HBM bound: 0.5 B (code) + 2/block B (scale) read and 2 B written per
// element.  Replaces phase 1 of the reference GEMM kernel (CastWeightProcess,
// grouped_gemm/op_kernel/grouped_matmul_antiquant.h:537-662) as a stand-alone op.
#include "moe_device.h"
#include "moe_internal.h"

namespace moe {

// One thread decodes UNROLL independent dwords (8 codes each) and writes UNROLL
// 16-byte vectors.  Consecutive lanes take consecutive dwords, so every load
// instruction of a wavefront covers 256 contiguous bytes and every store 1 KiB.
// The tensors are addressed flat: rows are contiguous and cols % BLOCK == 0, so
// element e uses scale e / BLOCK.  Measured on MI355X (7168 x 2048 and 64 times that):
// one dword per thread, ordinary loads and nontemporal stores is the fastest combination
// at both sizes (nontemporal loads cost 25 % at the small size, 4 dwords per thread 12 % at
// the large one); at 7168 x 2048 it takes 6.6 us where writing the output alone takes 6.4.
// Workgroups of 256 threads are best at that size (6.4 - 6.5 us against 6.6 with 1024), workgroups
// of 1024 on large tensors (9.6 GB: 6.1 TB/s against 5.6).
template <int BLOCK, int UNROLL, int TPB>
__global__ __launch_bounds__(TPB) void dequant_fp4_bf16_kernel(const uint32_t* __restrict__ codes,
                                                               const uint16_t* __restrict__ scale,
                                                               u32x4_t* __restrict__ out,
                                                               int64_t nwords) {
    const int64_t base = (int64_t)blockIdx.x * (TPB * UNROLL) + threadIdx.x;
    uint32_t w[UNROLL];
    float s[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const int64_t i = base + u * TPB;
        if (i < nwords) {
            w[u] = codes[i];
            s[u] = bf16_bits_to_f32(scale[(i * 8) / BLOCK]);
        }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const int64_t i = base + u * TPB;
        if (i < nwords) {
            u32x4_t o;
            o[0] = e2m1_pair_scaled_bf16<0>(w[u], s[u]);
            o[1] = e2m1_pair_scaled_bf16<1>(w[u], s[u]);
            o[2] = e2m1_pair_scaled_bf16<2>(w[u], s[u]);
            o[3] = e2m1_pair_scaled_bf16<3>(w[u], s[u]);
            __builtin_nontemporal_store(o, out + i);
        }
    }
}

template <int BLOCK, int TPB>
static int launch_dequant(const moe_dequant_args* a, int64_t nwords, hipStream_t stream) {
    constexpr int UNROLL = 1;
    const int64_t blocks = (nwords + TPB * UNROLL - 1) / (TPB * UNROLL);
    if (blocks > 0x7fffffffLL) return MOE_ERR_TOO_LARGE;
    hipLaunchKernelGGL((dequant_fp4_bf16_kernel<BLOCK, UNROLL, TPB>), dim3((unsigned)blocks), dim3(TPB), 0, stream,
                       static_cast<const uint32_t*>(a->codes), static_cast<const uint16_t*>(a->scale),
                       static_cast<u32x4_t*>(a->out), nwords);
    return hipGetLastError() == hipSuccess ? MOE_OK : MOE_ERR_LAUNCH;
}

int launch_dequant_fp4_bf16(const moe_dequant_args* a, hipStream_t stream) {
    const int64_t nwords = a->rows * a->cols / 8;
    if (nwords == 0) return MOE_OK;
    const bool large = nwords >= (int64_t{1} << 24);   // 128 Mi elements: 64 MiB of codes
    if (a->block == 32) return large ? launch_dequant<32, 1024>(a, nwords, stream) : launch_dequant<32, 256>(a, nwords, stream);
    return large ? launch_dequant<16, 1024>(a, nwords, stream) : launch_dequant<16, 256>(a, nwords, stream);
}

}  // namespace moe
