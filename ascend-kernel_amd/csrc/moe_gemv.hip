// Grouped GEMV for MoE decode on gfx950 (few rows per expert).  HBM bound: every weight byte of an expert
// that owns at least one row is read exactly once per pass over its rows; experts without rows cost one
// group_list read.  Replaces grouped_soft_gemv (grouped_soft_gemv/op_kernel/grouped_soft_gemv.h:235-293,
// gemv_impl.h:201-398).  Unlike the reference, more than 4 rows per expert are accepted.
//
// Two kernels live here, both for the K-contiguous containers:
//   gemv_kmajor_kernel    bf16 weights (and fp4 with K % 512 != 0): no matrix cores -- wide vector loads, packed-bf16
//                         dot products (v_dot2c_f32_bf16), wavefront shuffles for the reductions, 4 rows per pass
//   gemv_fp4_mfma_kernel  fp4 codes: one v_mfma_f32_16x16x32_bf16 per 32-k block and 16 weight rows (a vector kernel
//                         needs (1 + rows) / 2 instructions per 4-bit weight, more than the chip can issue while HBM
//                         delivers the codes at full rate), wave-private streaming, no workgroup barrier in the k loop
// The N-contiguous containers (reference fp4 / fp8, int4) run on the k-split matrix-core kernel of moe_gemm.hip with
// this op's arithmetic (launch_gemm_exact): measured 3 times faster than a vector kernel on that layout.
//
// Numerics (gemv_impl.h:147-199): weights are decode * scale in fp32, NOT rounded
// to bf16; fp32 accumulation; one RNE to bf16 at the end (grouped_soft_gemv.h:218-233).
#include "moe_device.h"
#include "moe_internal.h"

namespace moe {

constexpr int GV_ROWS = 4;        // activation rows per pass (MAX_BSZ of the reference)
constexpr int GV_KC = 8192;       // k elements of x staged in LDS per pass (4 rows -> 64 KiB)

__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), c,
                                           false);
}

__device__ __forceinline__ void group_rows(const int64_t* gl, int g, int64_t M, int64_t& start, int64_t& end) {
    start = g ? gl[g - 1] : 0;
    end = gl[g];
    if (start < 0) start = 0;
    if (end > M) end = M;
}

// ---------------------------------------------------------------------------------
// K-contiguous containers: MOE_FMT_BF16 [G,N,K] and MOE_FMT_FP4_B32 [G,N,K/2].
// A workgroup owns NR_WG weight rows (n) of one expert; each wavefront takes 8 rows at
// a time and all of K: a lane reads CH consecutive k (16 bytes) of each of the 8
// rows per step, so a step has 8 independent 1 KiB loads in flight per wavefront.
// x (<= 4 rows) is staged once in LDS.
// ---------------------------------------------------------------------------------
constexpr int GVK_NRW = 8;  // weight rows per wavefront step

template <int FMT>
struct KMajor;
template <>
struct KMajor<MOE_FMT_BF16> {
    static constexpr int CH = 8;      // k per lane per step (16 B of weights)
    static constexpr int NR_WG = 32;  // weight rows per workgroup: small enough that the last
                                      // round of workgroups does not leave CUs idle for long
    static constexpr int BLK = 1;     // no scales (kept non-zero: it appears as a divisor in code shared with fp4)
};
template <>
struct KMajor<MOE_FMT_FP4_B32> {
    static constexpr int CH = 32;     // one scale block (16 B of codes)
    static constexpr int NR_WG = 64;  // decode-bound: fewer x refills per weight byte pay more
    static constexpr int BLK = 32;
};
template <>
struct KMajor<MOE_FMT_FP4_B16> {
    static constexpr int CH = 32;     // two scale blocks per 16 B of codes
    static constexpr int NR_WG = 64;
    static constexpr int BLK = 16;
};

// LDS position (in 16-byte units) of the 8 k starting at k8*8, laid out so that the
// lanes of a wavefront read consecutive units whatever CH is.
template <int CH>
__device__ __forceinline__ int xs_unit(int k8) {
    constexpr int U = CH / 8;  // units per lane per step
    if (U == 1) return k8;
    const int lane_k = k8 / U, c = k8 % U;
    return ((lane_k >> 6) * U + c) * 64 + (lane_k & 63);
}

template <int FMT, int MG>
__device__ __forceinline__ void gemv_kmajor_rows(const uint8_t* __restrict__ wg, const uint16_t* __restrict__ sg,
                                                 const uint16_t* __restrict__ x, uint16_t* __restrict__ y,
                                                 u32x4_t* xs, int64_t row0, int n0, int N, int K) {
    constexpr int CH = KMajor<FMT>::CH;
    constexpr int U = CH / 8;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nchunks = (K + GV_KC - 1) / GV_KC;
    const int64_t wrow_bytes = FMT == MOE_FMT_BF16 ? (int64_t)K * 2 : (int64_t)K / 2;

    for (int it = 0; it < KMajor<FMT>::NR_WG / (4 * GVK_NRW); ++it) {
        const int n = n0 + (it * 4 + wave) * GVK_NRW;
        float acc[GVK_NRW][MG];
#pragma unroll
        for (int j = 0; j < GVK_NRW; ++j)
#pragma unroll
            for (int r = 0; r < MG; ++r) acc[j][r] = 0.f;

        for (int c = 0; c < nchunks; ++c) {
            const int kc0 = c * GV_KC;
            const int klen = min(GV_KC, K - kc0);
            if (nchunks > 1 || it == 0) {
                __syncthreads();
                for (int i = threadIdx.x; i < MG * (klen / 8); i += 256) {
                    const int r = i / (klen / 8), k8 = i % (klen / 8);
                    xs[r * (GV_KC / 8) + xs_unit<CH>(k8)] =
                        *reinterpret_cast<const u32x4_t*>(x + (row0 + r) * (int64_t)K + kc0 + k8 * 8);
                }
                __syncthreads();
            }
            for (int k = lane * CH; k < klen; k += 64 * CH) {
                u32x4_t w[GVK_NRW];
#pragma unroll
                for (int j = 0; j < GVK_NRW; ++j) {
                    const int nn = min(n + j, N - 1);
                    const uint8_t* p = wg + nn * wrow_bytes + (FMT == MOE_FMT_BF16 ? (int64_t)(kc0 + k) * 2
                                                                                    : (int64_t)(kc0 + k) / 2);
                    w[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
                }
                u32x4_t xv[MG][U];
#pragma unroll
                for (int r = 0; r < MG; ++r)
#pragma unroll
                    for (int u = 0; u < U; ++u) xv[r][u] = xs[r * (GV_KC / 8) + xs_unit<CH>(k / 8 + u)];

                if (FMT == MOE_FMT_BF16) {
#pragma unroll
                    for (int j = 0; j < GVK_NRW; ++j)
#pragma unroll
                        for (int r = 0; r < MG; ++r)
#pragma unroll
                            for (int d = 0; d < 4; ++d) acc[j][r] = dot2_bf16(w[j][d], xv[r][0][d], acc[j][r]);
                } else {
#pragma unroll
                    for (int j = 0; j < GVK_NRW; ++j) {
                        const int nn = min(n + j, N - 1);
                        constexpr int BLK = KMajor<FMT>::BLK;
                        const uint16_t* sp = sg + (int64_t)nn * (K / BLK) + (kc0 + k) / BLK;
                        const float s = bf16_bits_to_f32(sp[0]);
                        float part[MG];
#pragma unroll
                        for (int r = 0; r < MG; ++r) part[r] = 0.f;
#pragma unroll
                        for (int d = 0; d < 4; ++d) {
                            if (BLK == 16 && d == 2) {
                                // second block of 16: close the first one
#pragma unroll
                                for (int r = 0; r < MG; ++r) { acc[j][r] = fmaf(part[r], s, acc[j][r]); part[r] = 0.f; }
                            }
                            // exact e2m1 -> bf16 pairs (scale 1.0); the block scale is applied to the
                            // 32-element partial sum
                            uint32_t p0 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[j][d], 1.0f, 0));
                            uint32_t p1 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[j][d], 1.0f, 1));
                            uint32_t p2 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[j][d], 1.0f, 2));
                            uint32_t p3 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[j][d], 1.0f, 3));
#pragma unroll
                            for (int r = 0; r < MG; ++r) {
                                part[r] = dot2_bf16(p0, xv[r][d][0], part[r]);
                                part[r] = dot2_bf16(p1, xv[r][d][1], part[r]);
                                part[r] = dot2_bf16(p2, xv[r][d][2], part[r]);
                                part[r] = dot2_bf16(p3, xv[r][d][3], part[r]);
                            }
                        }
                        const float s_last = BLK == 16 ? bf16_bits_to_f32(sp[1]) : s;
#pragma unroll
                        for (int r = 0; r < MG; ++r) acc[j][r] = fmaf(part[r], s_last, acc[j][r]);
                    }
                }
            }
        }
#pragma unroll
        for (int j = 0; j < GVK_NRW; ++j)
#pragma unroll
            for (int r = 0; r < MG; ++r) {
                const float v = wave_reduce_sum(acc[j][r]);
                if (lane == 0 && n + j < N) y[(row0 + r) * (int64_t)N + n + j] = (uint16_t)(pack_bf16_rne(v, 0.f) & 0xffffu);
            }
    }
}

template <int FMT>
__global__ __launch_bounds__(256) void gemv_kmajor_kernel(const uint16_t* __restrict__ x,
                                                          const uint8_t* __restrict__ w,
                                                          const uint16_t* __restrict__ scale,
                                                          const int64_t* __restrict__ gl, uint16_t* __restrict__ y,
                                                          int64_t M, int K, int N) {
    extern __shared__ u32x4_t xs[];
    const int g = blockIdx.y, n0 = blockIdx.x * KMajor<FMT>::NR_WG;
    int64_t start, end;
    group_rows(gl, g, M, start, end);
    if (end <= start) return;
    const uint8_t* wg = w + (int64_t)g * N * (FMT == MOE_FMT_BF16 ? (int64_t)K * 2 : (int64_t)K / 2);
    const uint16_t* sg = FMT == MOE_FMT_BF16 ? nullptr : scale + (int64_t)g * N * (K / KMajor<FMT>::BLK);
    for (int64_t row0 = start; row0 < end; row0 += GV_ROWS) {
        const int mg = (int)min((int64_t)GV_ROWS, end - row0);
        switch (mg) {
            case 1: gemv_kmajor_rows<FMT, 1>(wg, sg, x, y, xs, row0, n0, N, K); break;
            case 2: gemv_kmajor_rows<FMT, 2>(wg, sg, x, y, xs, row0, n0, N, K); break;
            case 3: gemv_kmajor_rows<FMT, 3>(wg, sg, x, y, xs, row0, n0, N, K); break;
            default: gemv_kmajor_rows<FMT, 4>(wg, sg, x, y, xs, row0, n0, N, K); break;
        }
    }
}

// ---------------------------------------------------------------------------------
// MOE_FMT_FP4_B32 on the matrix cores.  The VALU path above spends (1 + rows) / 2
// instructions per weight element, more than the ~2.4 per element the chip can issue while
// HBM delivers 4-bit codes at full rate.  Here a wavefront owns 16 weight rows (the MFMA
// columns) and up to 16 activation rows (the MFMA rows): per 32-k scale block one
// v_mfma_f32_16x16x32_bf16 on exactly decoded e2m1 values (v_cvt_scalef32_pk_bf16_fp4 with
// scale 1.0, two codes per instruction) and one fma per accumulator register that applies
// the block's scale to the partial sum -- the same arithmetic as the VALU path (weights are
// not rounded to bf16).
//
// Weight loads stay 16 bytes per lane: lane (i, q) = (lane & 15, lane >> 4) reads scale block
// 4 c + q of weight row i, so a load instruction covers 64 contiguous bytes of 16 rows.
// The MFMA wants the 4 q lanes of a column to hold the 4 dwords of ONE block (a block has
// one scale, and the MFMA sums over q): a 4x4 transpose of the dwords across the q lanes,
// two v_permlane32_swap and two v_permlane16_swap per 16 bytes.
//
// Scales: every lane of a column needs the same 4 scales per load, 8 bytes of a row -- read
// that way, each 64-byte piece of a scale row is fetched from HBM several times.  Instead the
// 4 q lanes of a row read 128 contiguous bytes of it once per 4 loop iterations (lane q: the
// 16 scales of iteration 4 T + q) and the iteration's scales are picked up from the lane that
// holds them through a wavefront's own 2 KB of LDS (written once per 4 iterations, read with 16-byte loads that
// the 4 q lanes share: ds_bpermute, which this replaced, serves 4 lanes that ask for one lane's register one after
// the other -- the counters showed it as bank conflicts in 39 % of the LDS cycles).
//
// x (<= 16 rows of a chunk of K) is staged in LDS; the 16-byte units of row r are XOR-swizzled
// with r so that the fragment reads of the 16 lanes of a q group fall into different banks.
// ---------------------------------------------------------------------------------
constexpr int GF_WAVES = 8;               // wavefronts per workgroup
constexpr int GF_NR_WG = 16 * GF_WAVES;   // weight rows per workgroup
constexpr int GF_ROWS = 16;               // activation rows per pass
constexpr int GF_LDS_UNITS = 3584;        // 56 KiB of x per staged chunk
constexpr int GF_SCALE_UNITS = 128;       // per wavefront: the 4 q lanes' 2 x 16 bytes of scales for 16 rows
constexpr int GF_U = 4;                   // 128-k groups (one 16-byte load per lane each) per loop iteration
constexpr int GF_KSTEP = 128 * GF_U;      // k per loop iteration; K must be a multiple
constexpr int GF_GEMM_ROWS_PER_EXPERT = 12;// grouped GEMM calls with at most this many rows per expert on average come here

__device__ __forceinline__ uint32_t e2m1_pair_bf16(uint32_t word, int sel) {
    switch (sel) {
        case 0: return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(word, 1.0f, 0));
        case 1: return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(word, 1.0f, 1));
        case 2: return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(word, 1.0f, 2));
        default: return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(word, 1.0f, 3));
    }
}

// MB = activation rows staged and multiplied (4, 8 or 16).  ROUNDW selects the arithmetic of the
// grouped GEMM op (grouped_matmul_antiquant.h:537-662: weights are RNE_bf16(e2m1 * scale), so the
// scale has to be applied per element before the MFMA: ~2 VALU instructions per element) instead of
// that of the GEMV op (fp32 weights: the scale is applied to the block's partial sum).
// BLK = k per scale (32 or 16).  With 16, a 32-k block of a lane's row has two scales: the lanes
// q < 2 of a column hold its first half, q >= 2 the second, so with the GEMM's rounding each lane
// simply uses its half's scale, and with the GEMV's arithmetic the block takes two MFMAs, each on
// one half of the lanes' codes (the other half zeroed), each partial sum scaled by its own scale.
// With at most 8 activation rows (STACK below) one MFMA does: fragment row r < 8 of x keeps only the first
// 16 k of x row r, row 8 + r only the last 16 k, so the product's rows < 8 (lanes q < 2) are the first
// scale's partial sums and rows >= 8 (q >= 2) the second's; each lane applies its own half's scale and the
// halves are added once at the end.
template <int MB, bool ROUNDW, int BLK>
__device__ __forceinline__ void gemv_fp4_mfma_rows(const uint8_t* __restrict__ wg, const uint16_t* __restrict__ sg,
                                                   const uint16_t* __restrict__ x, uint16_t* __restrict__ y,
                                                   u32x4_t* xs, int64_t row0, int mg, int n0, int N, int K) {
    constexpr int KC = GF_LDS_UNITS / MB * 8 / GF_KSTEP * GF_KSTEP;   // k per staged chunk: 7168, 3584 or 1536
    constexpr int RS = KC / 8;                  // row stride in 16-byte units
    constexpr int U = GF_U;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int i = lane & 15, q = lane >> 4;
    // this wavefront's scale exchange: unit (2 q' + e) * 16 + i holds register e of lane (i, q')
    u32x4_t* ss = xs + GF_LDS_UNITS + wave * GF_SCALE_UNITS;
    const int n = n0 + wave * 16 + i;
    const int nn = min(n, N - 1);
    // 32-bit byte offsets from the expert's (wavefront-uniform) base pointers: an expert's weight
    // slab is smaller than 4 GiB
    const uint32_t woff = (uint32_t)nn * (uint32_t)(K / 2) + q * 16;
    const uint32_t soff = (uint32_t)nn * (uint32_t)(K / BLK) * 2;
    constexpr int PER = BLK / 8;                // loop iterations per 128 bytes (64 scales) of a scale row
    const bool hi_half = (q & 2) != 0;          // block 16: this lane's codes belong to the second scale of a block
    constexpr bool STACK = BLK == 16 && !ROUNDW && MB <= 8;
    // STACK: fragment row i of x is live only in the k half that matches i >> 3
    const uint32_t x_keep = ((i >> 3) == (q >> 1)) ? 0xffffffffu : 0u;
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f}, acc2 = {0.f, 0.f, 0.f, 0.f};

    for (int kc0 = 0; kc0 < K; kc0 += KC) {
        const int klen = min(KC, K - kc0);
        const int niter = klen / GF_KSTEP;             // iterations of U groups
        const int nblk = klen / BLK;                   // scales of the chunk (>= 16)
        const uint8_t* wp = wg + (kc0 >> 1);                                   // group c of the chunk: + 64 c bytes
        const uint8_t* sp = reinterpret_cast<const uint8_t*>(sg) + (kc0 / BLK) * 2;  // scale b of the chunk: + 2 b bytes
        // x fragment of block 4 c + j: unit (16 c + 4 j + q) ^ r of row r = xj[j][16 c].  MFMA rows
        // >= MB read row i % MB again: their products land in accumulator rows that are not stored
        // (lanes that read the same unit are served together: timed alone, this pattern reads as fast as
        // 64 consecutive units, and sending the repeated rows to other units was slower).
        const int r = i % MB;
        const u32x4_t* xj[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) xj[j] = xs + r * RS + ((4 * j + q) ^ r);

        // one 128-k group: w = this lane's 16 bytes (block 4 c + q of its row), s0/s1 = the 4 scales of
        // blocks 4 c .. 4 c + 3 as two bf16 pairs
        auto group = [&](const u32x4_t& w, const uint32_t (&sd)[BLK == 32 ? 2 : 4], int c) {
            // 4x4 transpose of the dwords over the q lanes: b[j] = this lane's 8 codes of block 4 c + j
            const u32x2_t t02 = __builtin_amdgcn_permlane32_swap(w[0], w[2], false, false);
            const u32x2_t t13 = __builtin_amdgcn_permlane32_swap(w[1], w[3], false, false);
            const u32x2_t b01 = __builtin_amdgcn_permlane16_swap(t02[0], t13[0], false, false);
            const u32x2_t b23 = __builtin_amdgcn_permlane16_swap(t02[1], t13[1], false, false);
            const uint32_t b[4] = {b01[0], b01[1], b23[0], b23[1]};
            // s[j]: block 32: the scale of block j; block 16: the scale of this lane's half of block j
            // (ROUNDW) / of the first half (else), s2[j] that of the second half
            float s[4], s2[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if constexpr (BLK == 32) {
                    s[j] = (j & 1) ? bf16_hi(sd[j >> 1]) : bf16_lo(sd[j >> 1]);
                    s2[j] = 0.f;
                } else if constexpr (ROUNDW || STACK) {
                    s[j] = hi_half ? bf16_hi(sd[j]) : bf16_lo(sd[j]);
                    s2[j] = 0.f;
                } else {
                    s[j] = bf16_lo(sd[j]);
                    s2[j] = bf16_hi(sd[j]);
                }
            }
            // two blocks at a time: enough independent MFMAs to cover their latency, few enough
            // live registers for 4 wavefronts per SIMD
#pragma unroll
            for (int j0 = 0; j0 < 4; j0 += 2) {
                u32x4_t aw[2], bw[2];
#pragma unroll
                for (int j = 0; j < 2; ++j) aw[j] = xj[j0 + j][16 * c];
                if constexpr (ROUNDW) {
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        bw[j][0] = e2m1_pair_scaled_bf16<0>(b[j0 + j], s[j0 + j]);
                        bw[j][1] = e2m1_pair_scaled_bf16<1>(b[j0 + j], s[j0 + j]);
                        bw[j][2] = e2m1_pair_scaled_bf16<2>(b[j0 + j], s[j0 + j]);
                        bw[j][3] = e2m1_pair_scaled_bf16<3>(b[j0 + j], s[j0 + j]);
                    }
                    // two accumulators, so that consecutive MFMAs do not depend on each other
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, aw[0]),
                                                                  __builtin_bit_cast(bf16x8_t, bw[0]), acc, 0, 0, 0);
                    acc2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, aw[1]),
                                                                   __builtin_bit_cast(bf16x8_t, bw[1]), acc2, 0, 0, 0);
                } else if constexpr (STACK) {
                    f32x4_t part[2];
#pragma unroll
                    for (int j = 0; j < 2; ++j)
#pragma unroll
                        for (int d = 0; d < 4; ++d) {
                            bw[j][d] = e2m1_pair_bf16(b[j0 + j], d);
                            aw[j][d] &= x_keep;
                        }
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        part[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, aw[j]),
                                                                          __builtin_bit_cast(bf16x8_t, bw[j]),
                                                                          f32x4_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
#pragma unroll
                    for (int j = 0; j < 2; ++j)
#pragma unroll
                        for (int rr = 0; rr < 4; ++rr) acc[rr] = fmaf(part[j][rr], s[j0 + j], acc[rr]);
                } else if constexpr (BLK == 16) {
                    // per block: first-half lanes' codes, then second-half lanes' codes
                    const uint32_t keep_lo = hi_half ? 0u : 0xffffffffu;
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        u32x4_t b_lo, b_hi;
#pragma unroll
                        for (int d = 0; d < 4; ++d) {
                            b_lo[d] = e2m1_pair_bf16(b[j0 + j] & keep_lo, d);
                            b_hi[d] = e2m1_pair_bf16(b[j0 + j] & ~keep_lo, d);
                        }
                        const f32x4_t p_lo = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            __builtin_bit_cast(bf16x8_t, aw[j]), __builtin_bit_cast(bf16x8_t, b_lo), f32x4_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                        const f32x4_t p_hi = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            __builtin_bit_cast(bf16x8_t, aw[j]), __builtin_bit_cast(bf16x8_t, b_hi), f32x4_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
#pragma unroll
                        for (int rr = 0; rr < 4; ++rr) {
                            acc[rr] = fmaf(p_lo[rr], s[j0 + j], acc[rr]);
                            acc2[rr] = fmaf(p_hi[rr], s2[j0 + j], acc2[rr]);
                        }
                    }
                } else {
                    f32x4_t part[2];
#pragma unroll
                    for (int j = 0; j < 2; ++j)
#pragma unroll
                        for (int d = 0; d < 4; ++d) bw[j][d] = e2m1_pair_bf16(b[j0 + j], d);
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        part[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, aw[j]),
                                                                          __builtin_bit_cast(bf16x8_t, bw[j]),
                                                                          f32x4_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
#pragma unroll
                    for (int j = 0; j < 2; ++j)
#pragma unroll
                        for (int rr = 0; rr < 4; ++rr) acc[rr] = fmaf(part[j][rr], s[j0 + j], acc[rr]);
                }
            }
        };
        auto fetch_w = [&](u32x4_t (&w)[U], int it) {
#pragma unroll
            for (int u = 0; u < U; ++u)
                // ordinary loads: an instruction covers 64 bytes of each of 16 rows, half a cache line; the other half
                // comes with the next instruction and must still find the line (measured on this pattern alone:
                // 6.3 TB/s with ordinary loads, 5.7 with nontemporal ones)
                w[u] = *reinterpret_cast<const u32x4_t*>(wp + (woff + (uint32_t)((it * U + u) * 64)));
        };
        // scales 64 T + 16 q .. + 15 of this lane's row in the chunk: those of iteration 4 T + q (block 32)
        // or of half of iteration 2 T + (q >> 1) (block 16); clamped into the chunk (iterations past its
        // end do not exist)
        auto fetch_s = [&](u32x4_t (&sv)[2], int T) {
            const int b0 = min(64 * T + 16 * q, nblk - 16);
            sv[0] = *reinterpret_cast<const u32x4_t*>(sp + (soff + (uint32_t)(b0 * 2)));
            sv[1] = *reinterpret_cast<const u32x4_t*>(sp + (soff + (uint32_t)(b0 * 2 + 16)));
        };
        u32x4_t sc[2], sn[2];
        // iteration `it` on the weights in w; rotates the scale registers every PER iterations
        auto iteration = [&](const u32x4_t (&w)[U], int it) {
            const int t = it & (PER - 1);
            if (t == 0) {
                // (a wavefront's LDS accesses complete in order: the reads of the previous scales are done)
                ss[(2 * q) * 16 + i] = sn[0];
                ss[(2 * q + 1) * 16 + i] = sn[1];
                if (it + PER < niter) fetch_s(sn, it / PER + 1);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if constexpr (BLK == 32) {
                    // this iteration's scales are those of lane (i, t): 2 dwords per group
                    if (u == 0) {
                        sc[0] = ss[(2 * t) * 16 + i];
                        sc[1] = ss[(2 * t + 1) * 16 + i];
                    }
                    const uint32_t sd[2] = {sc[u >> 1][2 * (u & 1)], sc[u >> 1][2 * (u & 1) + 1]};
                    group(w[u], sd, it * U + u);
                } else {
                    // groups 0, 1 of the iteration are with lane (i, 2 t), groups 2, 3 with lane (i, 2 t + 1): 4 dwords each
                    const u32x4_t sv = ss[(2 * (2 * t + (u >> 1)) + (u & 1)) * 16 + i];
                    const uint32_t sd[4] = {sv[0], sv[1], sv[2], sv[3]};
                    group(w[u], sd, it * U + u);
                }
            }
        };
        // two register sets of weights: the loads of iteration it + 1 are in flight behind iteration it
        u32x4_t wa[U], wb[U];
        fetch_s(sn, 0);
        fetch_w(wa, 0);
        // stage this chunk of x while the first weights are on their way
        __syncthreads();
        for (int t = threadIdx.x; t < MB * (klen / 8); t += 64 * GF_WAVES) {
            const int r = t / (klen / 8), k8 = t % (klen / 8);
            u32x4_t v = {0u, 0u, 0u, 0u};
            if (r < mg) v = *reinterpret_cast<const u32x4_t*>(x + (row0 + r) * (int64_t)K + kc0 + k8 * 8);
            xs[r * RS + (k8 ^ r)] = v;
        }
        __syncthreads();
        for (int it = 0; it < niter; it += 2) {
            if (it + 1 < niter) fetch_w(wb, it + 1);
            iteration(wa, it);
            if (it + 1 < niter) {
                if (it + 2 < niter) fetch_w(wa, it + 2);
                iteration(wb, it + 1);
            }
        }
    }
    if constexpr (STACK) {
        // lanes q and q + 2 hold the two scales' sums of the same rows
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[r] += __shfl_xor(acc[r], 32);
    }
    // lane (i, q) holds column n, rows 4 q .. 4 q + 3
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int m = 4 * q + r;
        if (m < mg && n < N) y[(row0 + m) * (int64_t)N + n] = (uint16_t)(pack_bf16_rne(acc[r] + acc2[r], 0.f) & 0xffffu);
    }
}

template <bool ROUNDW, int BLK>
__global__ __launch_bounds__(64 * GF_WAVES, 4) void gemv_fp4_mfma_kernel(const uint16_t* __restrict__ x,
                                                                         const uint8_t* __restrict__ w,
                                                                         const uint16_t* __restrict__ scale,
                                                                         const int64_t* __restrict__ gl,
                                                                         uint16_t* __restrict__ y, int64_t M, int K,
                                                                         int N) {
    extern __shared__ u32x4_t xs[];
    const int g = blockIdx.y, n0 = blockIdx.x * GF_NR_WG;
    int64_t start, end;
    group_rows(gl, g, M, start, end);
    if (end <= start) return;
    const uint8_t* wg = w + (int64_t)g * N * ((int64_t)K / 2);
    const uint16_t* sg = scale + (int64_t)g * N * (K / BLK);
    for (int64_t row0 = start; row0 < end; row0 += GF_ROWS) {
        const int mg = (int)min((int64_t)GF_ROWS, end - row0);
        if (mg <= 4) gemv_fp4_mfma_rows<4, ROUNDW, BLK>(wg, sg, x, y, xs, row0, mg, n0, N, K);
        else if (mg <= 8) gemv_fp4_mfma_rows<8, ROUNDW, BLK>(wg, sg, x, y, xs, row0, mg, n0, N, K);
        else gemv_fp4_mfma_rows<16, ROUNDW, BLK>(wg, sg, x, y, xs, row0, mg, n0, N, K);
    }
}

template <bool ROUNDW, int BLK>
static int launch_fp4_mfma(const moe_grouped_args* a, hipStream_t stream) {
    dim3 grid((unsigned)((a->N + GF_NR_WG - 1) / GF_NR_WG), (unsigned)a->G);
    constexpr size_t lds = (size_t)(GF_LDS_UNITS + GF_WAVES * GF_SCALE_UNITS) * 16;   // 72 KB: two workgroups per CU
    static std::atomic<uint64_t> lds_set{0};
    if (const int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(&gemv_fp4_mfma_kernel<ROUNDW, BLK>), (int)lds, lds_set)) return rc;
    hipLaunchKernelGGL((gemv_fp4_mfma_kernel<ROUNDW, BLK>), grid, dim3(64 * GF_WAVES), lds, stream,
                       static_cast<const uint16_t*>(a->x), static_cast<const uint8_t*>(a->weight),
                       static_cast<const uint16_t*>(a->scale), a->group_list, static_cast<uint16_t*>(a->y), a->M,
                       (int)a->K, (int)a->N);
    return hipGetLastError() == hipSuccess ? MOE_OK : MOE_ERR_LAUNCH;
}

template <int FMT>
static int launch_kmajor(const moe_grouped_args* a, hipStream_t stream) {
    const int kc = (int)(a->K < GV_KC ? a->K : GV_KC);
    const size_t lds = (size_t)GV_ROWS * GV_KC / 8 * 16;
    (void)kc;
    dim3 grid((unsigned)((a->N + KMajor<FMT>::NR_WG - 1) / KMajor<FMT>::NR_WG), (unsigned)a->G);
    hipLaunchKernelGGL((gemv_kmajor_kernel<FMT>), grid, dim3(256), lds, stream,
                       static_cast<const uint16_t*>(a->x), static_cast<const uint8_t*>(a->weight),
                       static_cast<const uint16_t*>(a->scale), a->group_list, static_cast<uint16_t*>(a->y), a->M,
                       (int)a->K, (int)a->N);
    return hipGetLastError() == hipSuccess ? MOE_OK : MOE_ERR_LAUNCH;
}

bool gemv_preferred(const moe_grouped_args* a) {
    // Decode-sized batches on the K-contiguous containers are pure weight streaming: these kernels
    // read every weight row as contiguous runs.  The bf16 vector kernel takes 4 rows of an expert per
    // pass over its weights (same arithmetic as the GEMM: the weights are bf16 already).  The
    // matrix-core fp4_b32 kernel takes 16 and has a variant with the GEMM's weight rounding; the
    // bound is where the k-split GEMM kernel overtakes it (measured at DeepSeek-V3 shapes, 256 experts of
    // 7168 x 2048: 8 rows per expert 496 vs 631 us, 16 rows 754 vs 651 us).
    if (a->format == MOE_FMT_FP4_B32 || a->format == MOE_FMT_FP4_B16)
        return a->K % GF_KSTEP == 0 && a->M <= GF_GEMM_ROWS_PER_EXPERT * a->G;
    if (a->format == MOE_FMT_BF16) return a->M <= 4 * a->G;
    return false;
}

int launch_grouped_gemv(const moe_grouped_args* a, hipStream_t stream, bool gemm_rounding) {
    switch (a->format) {
        case MOE_FMT_BF16: return launch_kmajor<MOE_FMT_BF16>(a, stream);
        case MOE_FMT_FP4_B32:
            // the matrix-core kernel takes K in whole loop iterations
            if (a->K % GF_KSTEP != 0) return gemm_rounding ? MOE_ERR_BAD_SHAPE : launch_kmajor<MOE_FMT_FP4_B32>(a, stream);
            return gemm_rounding ? launch_fp4_mfma<true, 32>(a, stream) : launch_fp4_mfma<false, 32>(a, stream);
        case MOE_FMT_FP4_B16:
            if (a->K % GF_KSTEP != 0) return gemm_rounding ? MOE_ERR_BAD_SHAPE : launch_kmajor<MOE_FMT_FP4_B16>(a, stream);
            return gemm_rounding ? launch_fp4_mfma<true, 16>(a, stream) : launch_fp4_mfma<false, 16>(a, stream);
        case MOE_FMT_FP4_REF:
        case MOE_FMT_INT4:
        case MOE_FMT_FP8_REF: {
            // the matrix-core GEMM kernels run with this op's arithmetic (fp32 weights)
            return launch_gemm_exact(a, stream);
        }
        default: return MOE_ERR_BAD_FORMAT;
    }
}

}  // namespace moe
