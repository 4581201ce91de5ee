// Weight preparation for the reference's "fp4" container on gfx950: checkpoint tensors ->
// what grouped_gemm / grouped_soft_gemv with computeType "fp4" consume.  Pure byte and
// nibble movement, HBM bound, bit-exact.
//
//   codes   uint8 [G, N, K/2]  (even k in the low nibble)
//        -> int8  [G, K, N/2]  nibble transpose (repack_weight,
//                              grouped_gemm/test/python/test_group_gemm_fp4.py:105-117) followed
//                              by the byte permutation inside every 64(k) x 128(byte) tile
//                              (repack_weight_step2, :129-142)
//   scale   bf16  [G, N, K/16] (x optional fp32 second-level scale, anti_quant_fp8_scale, :86-94)
//        -> bf16  [G, K/16, N] (the transpose of :185-186)
//
// The reference does this on the host side of its tests with torch reshapes; here each is one
// kernel that reads and writes every byte once, in full cache lines on both sides.
#include "moe_device.h"
#include "moe_internal.h"

namespace moe {

// ---------------------------------------------------------------------------------
// Codes.  A workgroup takes 256 weight rows (n) x up to 256 k of one expert: 128 contiguous
// bytes of each checkpoint row go to LDS (rows padded by one dword), then for each of the up to
// four 64-k tiles every thread produces 32 contiguous output bytes.
//
// Destination row R (0..63) of a tile and byte b (0..127), with j = R >> 5, i = (R >> 3) & 3,
// p = R & 7, q = b >> 5, r = (b >> 2) & 7, s = b & 3, hold k = 16 i + 8 j + r of the tile and the
// columns n = 32 p + 8 q + 2 s + {0, 1}: a 4-byte word is 8 consecutive n at one k, a 32-byte
// run (fixed R, q) is the 8 x 8 nibble transpose of one dword (8 consecutive k) of each of
// the 8 checkpoint rows 32 p + 8 q .. + 7.
// ---------------------------------------------------------------------------------
constexpr int PP_ROWS = 256;     // weight rows per workgroup
constexpr int PP_STRIDE = 33;    // LDS row stride in dwords (32 + 1 pad)

__global__ __launch_bounds__(256) void prepack_fp4_codes_kernel(const uint8_t* __restrict__ ckpt,
                                                                uint8_t* __restrict__ out, int N, int K) {
    __shared__ uint32_t tile[PP_ROWS * PP_STRIDE];
    const int tid = threadIdx.x;
    const int kg = blockIdx.x, t = blockIdx.y, g = blockIdx.z;
    const int ntile = min(4, K / 64 - 4 * kg);   // 64-k tiles in this group
    const int chunks = 2 * ntile;                // 16-byte chunks per row
    const uint8_t* src = ckpt + ((int64_t)g * N + (int64_t)t * PP_ROWS) * (K / 2) + kg * 128;
    for (int idx = tid; idx < PP_ROWS * chunks; idx += 256) {
        const int row = idx / chunks, c = idx % chunks;
        const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(src + (int64_t)row * (K / 2) + c * 16));
#pragma unroll
        for (int d = 0; d < 4; ++d) tile[row * PP_STRIDE + 4 * c + d] = v[d];
    }
    __syncthreads();

    const int R = tid >> 2, q = tid & 3;
    const int j = R >> 5, i = (R >> 3) & 3, p = R & 7;
    const int n0 = 32 * p + 8 * q;
    uint8_t* dst = out + ((int64_t)g * K + 256 * kg + R) * (N / 2) + 128 * t + 32 * q;
    for (int a = 0; a < ntile; ++a) {
        uint32_t d[8];
#pragma unroll
        for (int m = 0; m < 8; ++m) d[m] = tile[(n0 + m) * PP_STRIDE + 8 * a + 2 * i + j];
        // 8 x 8 nibble transpose: afterwards nibble m of d[r] is what nibble r of d[m] was
#pragma unroll
        for (int m = 0; m < 8; m += 2) {
            const uint32_t x = ((d[m] >> 4) ^ d[m + 1]) & 0x0f0f0f0fu;
            d[m + 1] ^= x;
            d[m] ^= x << 4;
        }
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            if (m & 2) continue;
            const uint32_t x = ((d[m] >> 8) ^ d[m + 2]) & 0x00ff00ffu;
            d[m + 2] ^= x;
            d[m] ^= x << 8;
        }
#pragma unroll
        for (int m = 0; m < 4; ++m) {
            const uint32_t x = ((d[m] >> 16) ^ d[m + 4]) & 0x0000ffffu;
            d[m + 4] ^= x;
            d[m] ^= x << 16;
        }
        u32x4_t* o = reinterpret_cast<u32x4_t*>(dst + (int64_t)a * 64 * (N / 2));
        __builtin_nontemporal_store(u32x4_t{d[0], d[1], d[2], d[3]}, o);
        __builtin_nontemporal_store(u32x4_t{d[4], d[5], d[6], d[7]}, o + 1);
    }
}

// ---------------------------------------------------------------------------------
// Scales: [G, N, KB] -> [G, KB, N] in tiles of 64 x 64 through LDS, each value multiplied in
// fp32 by the expert's second-level scale (one, or one for each half of the N rows) and
// rounded to bf16 -- the in-place `scale *= scale_2` of the reference on a bf16 tensor.
// ---------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void prepack_fp4_scale_kernel(const uint16_t* __restrict__ in,
                                                                const float* __restrict__ scale2,
                                                                uint16_t* __restrict__ out, int N, int KB, int s2cols) {
    __shared__ uint16_t tile[64 * 66];
    const int tid = threadIdx.x;
    const int kb0 = blockIdx.x * 64, n0 = blockIdx.y * 64, g = blockIdx.z;
    const uint16_t* src = in + ((int64_t)g * N + n0) * KB + kb0;
    // KB is a multiple of 4: 8-byte chunks along kb
    for (int idx = tid; idx < 64 * 16; idx += 256) {
        const int row = idx >> 4, c = idx & 15;
        u32x2_t v = {0u, 0u};
        if (kb0 + 4 * c < KB) v = *reinterpret_cast<const u32x2_t*>(src + (int64_t)row * KB + 4 * c);
        uint32_t* tp = reinterpret_cast<uint32_t*>(tile + row * 66 + 4 * c);   // 66 and 4 c are even: 4-byte aligned
        tp[0] = v[0];
        tp[1] = v[1];
    }
    __syncthreads();
    float m[2] = {1.f, 1.f};
    if (s2cols == 1) m[0] = m[1] = scale2[g];
    if (s2cols == 2) { m[0] = scale2[2 * g]; m[1] = scale2[2 * g + 1]; }
    // output rows kb, 16-byte chunks of 8 n
    for (int idx = tid; idx < 64 * 8; idx += 256) {
        const int kb = idx >> 3, c = idx & 7;
        if (kb0 + kb >= KB) continue;
        const float mul = (n0 + 8 * c) * 2 < N ? m[0] : m[1];   // N % 256 == 0: a chunk never straddles the halves
        uint32_t w[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint32_t lo = tile[(8 * c + 2 * e) * 66 + kb], hi = tile[(8 * c + 2 * e + 1) * 66 + kb];
            w[e] = s2cols ? pack_bf16_rne(bf16_bits_to_f32(lo) * mul, bf16_bits_to_f32(hi) * mul) : (lo | (hi << 16));
        }
        *reinterpret_cast<u32x4_t*>(out + ((int64_t)g * KB + kb0 + kb) * N + n0 + 8 * c) = u32x4_t{w[0], w[1], w[2], w[3]};
    }
}

int launch_prepack_fp4_ref(const moe_prepack_fp4_args* a, hipStream_t stream) {
    if (a->codes) {
        dim3 grid((unsigned)((a->K / 64 + 3) / 4), (unsigned)(a->N / PP_ROWS), (unsigned)a->G);
        hipLaunchKernelGGL(prepack_fp4_codes_kernel, grid, dim3(256), 0, stream,
                           static_cast<const uint8_t*>(a->codes), static_cast<uint8_t*>(a->weight_out), (int)a->N,
                           (int)a->K);
        if (hipGetLastError() != hipSuccess) return MOE_ERR_LAUNCH;
    }
    if (a->scale) {
        const int KB = (int)(a->K / 16);
        dim3 grid((unsigned)((KB + 63) / 64), (unsigned)(a->N / 64), (unsigned)a->G);
        hipLaunchKernelGGL(prepack_fp4_scale_kernel, grid, dim3(256), 0, stream,
                           static_cast<const uint16_t*>(a->scale), static_cast<const float*>(a->scale2),
                           static_cast<uint16_t*>(a->scale_out), (int)a->N, KB, a->scale2 ? (int)a->scale2_cols : 0);
        if (hipGetLastError() != hipSuccess) return MOE_ERR_LAUNCH;
    }
    return MOE_OK;
}

}  // namespace moe
