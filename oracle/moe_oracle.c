/*
 * moe_oracle.c -- CPU restatement of the reference's MoE weight-antiquant maths.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker for the HIP kernels: it is
 * compiled into oracle/libmoe_oracle.so and may be loaded only by tests/, by
 * __graft_entry__.smoke() and by the cpu_baseline leg of bench.py.  Nothing in
 * the shipped package links, imports or calls it, and there is no CPU fallback
 * in the product.
 *
 * Every function names the reference file:line whose behaviour it restates
 * (paths are relative to the QingCheng-AI/ascend-kernel tree).  Only the
 * Apache-2.0 test scripts and adapters were used as the specification.
 *
 * How each function is pinned (tests/test_oracle.py holds the checks):
 *   orc_e2m1_decode        LUT literal of the reference test + both of the
 *                          reference's bit-trick forms evaluated independently
 *   orc_e4m3_decode        torch.float8_e4m3fn on the 254 non-NaN codes, +-480
 *                          on the two NaN codes (what the bit trick yields)
 *   orc_fp4ref_locate      numpy restatement of the two reshape/permute stages
 *                          + a brute-force scan on a tiny tensor + round trip
 *   orc_dequant_fp4_bf16   torch CPU bf16*bf16 multiply (fp32 product, one RNE)
 *   orc_expand_weight      per-format closed forms; fp8 against the reference
 *                          test's own reshape/permute dequant written in numpy
 *   orc_grouped_gemm       torch.matmul per expert in fp64; the reference fp8
 *                          tests' all-ones x (output = column sums)
 *   "int8" (scale+offset) follows the CANN formula (w + offset) * scale; the
 *   reference never reads antiquant_offset, so no reference test covers it:
 *   parity unpinned beyond that formula.
 */
#include <math.h>
#ifdef _OPENMP
#include <omp.h>
#endif
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

enum {
    ORC_FMT_FP4_REF = 0, /* int8 [G,K,N/2] two-stage pre-shuffled e2m1; scale bf16 [G,K/16,N] */
    ORC_FMT_FP8_REF = 1, /* uint8 [G,K,N] e4m3 bits; scale fp32 [G,ceil(K/128),ceil(N/128)]   */
    ORC_FMT_INT8 = 2,    /* int8 [G,K,N]; scale bf16 [G,N]; offset bf16 [G,N]                 */
    ORC_FMT_INT4 = 3,    /* uint8 [G,K,N/2] low nibble = even n; zero point 8; scale bf16 [G,K/gs,N] */
    ORC_FMT_FP4_B32 = 4, /* uint8 [G,N,K/2] low nibble = even k; scale bf16 [G,N,K/32]        */
    ORC_FMT_BF16 = 5,    /* bf16 [G,N,K]                                                       */
    ORC_FMT_FP4_B16 = 6  /* as ORC_FMT_FP4_B32 with scale bf16 [G,N,K/16]: the checkpoint orientation of
                            grouped_gemm/test/python/test_group_gemm_fp4.py:46-64                     */
};

static inline float bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* fp32 -> bf16, round to nearest even (CAST_RINT in
 * grouped_gemm/op_kernel/antiquant_impl.h:162-165; torch's .to(bfloat16)). */
static inline uint16_t f32_to_bf16_rne(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u); /* quiet NaN */
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

/* Threads the parallel loops of this file use. */
int orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

uint16_t orc_f32_to_bf16(float f) { return f32_to_bf16_rne(f); }
float orc_bf16_to_f32(uint16_t h) { return bf16_to_f32(h); }

/* e2m1 decode: magnitude LUT {0,.5,1,1.5,2,3,4,6}, sign in bit 3; code 8 is -0.0.
 * grouped_gemm/test/python/test_group_gemm_fp4.py:6-8, :20-26. */
float orc_e2m1_decode(uint8_t code) {
    static const float lut[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};
    float v = lut[code & 7];
    return (code & 8) ? -v : v;
}

/* e4m3 decode as the reference does it: sign -> bit 15, low 7 bits -> bits 10:4
 * of a bf16 pattern, times 2^120.  No NaN handling: 0x7F/0xFF give +-480.
 * grouped_gemm/test/python/test_group_gemm_fp8.py:11-14;
 * grouped_gemm/op_kernel/antiquant_impl.h:87-129. */
float orc_e4m3_decode(uint8_t code) {
    int e = (code >> 3) & 15, m = code & 7;
    float v = e ? ldexpf(1.0f + (float)m / 8.0f, e - 7) : ldexpf((float)m / 8.0f, -6);
    return (code & 0x80) ? -v : v;
}

/* Where the reference's pre-shuffled fp4 container keeps logical element (k, n)
 * of one expert: returns the byte index inside the expert's [K, N/2] slab and
 * the nibble (0 = low).  Stage 1 packs along N (byte (k,c) = code(k,2c) |
 * code(k,2c+1) << 4); stage 2 permutes bytes inside every 64(k) x 128(byte)
 * tile.  grouped_gemm/test/python/test_group_gemm_fp4.py:105-117, :129-142. */
int64_t orc_fp4ref_locate(int64_t k, int64_t n, int64_t N, int *nibble) {
    int64_t nb = N / 2, c = n >> 1;
    int64_t a = k >> 6, kk = k & 63, t = c >> 7, cc = c & 127;
    int64_t i = kk >> 4, j = (kk >> 3) & 1, r = kk & 7;
    int64_t p = cc >> 4, q = (cc >> 2) & 3, s = cc & 3;
    int64_t R = (j << 5) | (i << 3) | p, b = (q << 5) | (r << 2) | s;
    *nibble = (int)(n & 1);
    return (a * 64 + R) * nb + t * 128 + b;
}

/* Stand-alone FP4(e2m1) -> BF16 dequant: codes uint8 [R, C/2] (even element in
 * the low nibble, test_group_gemm_fp4.py:29-35), scale bf16 [R, C/block], out
 * bf16 [R, C] = RNE_bf16(float(decode) * float(scale)).  Twin of fp4_dequant +
 * the per-block scale loop, test_group_gemm_fp4.py:97-102, :205-207, and of
 * antiquantProcess, grouped_gemm/op_kernel/antiquant_impl.h:146-208. */
void orc_dequant_fp4_bf16(const uint8_t *codes, const uint16_t *scale, uint16_t *out,
                          int64_t R, int64_t C, int64_t block) {
    int64_t nblk = C / block;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < R; ++r) {
        const uint8_t *cr = codes + r * (C / 2);
        const uint16_t *sr = scale + r * nblk;
        uint16_t *orow = out + r * C;
        for (int64_t c = 0; c < C; ++c) {
            uint8_t byte = cr[c >> 1];
            uint8_t code = (c & 1) ? (byte >> 4) : (byte & 15);
            orow[c] = f32_to_bf16_rne(orc_e2m1_decode(code) * bf16_to_f32(sr[c / block]));
        }
    }
}

/* Dequantize expert g of a weight container into a dense float W[K][N].
 * round_bf16 = 1: GEMM numerics, W = RNE_bf16(decode * scale) held as float
 *   (grouped_gemm/op_kernel/antiquant_impl.h:146-208; test_group_gemm_fp4.py:205-207;
 *   test_group_gemm_fp8.py:23-27).
 * round_bf16 = 0: GEMV numerics, the fp32 product is used un-rounded
 *   (grouped_soft_gemv/op_kernel/gemv_impl.h:147-199;
 *   test_group_soft_gemv_fp8.py:24-33).
 * scale_rows = scale.shape[-2] for the grouped formats (K/16 for fp4,
 * K/group for int4); offset is used by ORC_FMT_INT8 only. */
int orc_expand_weight(int fmt, const void *w, const void *scale, const void *offset, int64_t g,
                      int64_t K, int64_t N, int64_t scale_rows, int round_bf16, float *out) {
    if (fmt == ORC_FMT_FP4_REF) {
        const uint8_t *wb = (const uint8_t *)w + g * K * (N / 2);
        const uint16_t *sc = (const uint16_t *)scale + g * scale_rows * N;
        int64_t gs = K / scale_rows;
#pragma omp parallel for schedule(static)
        for (int64_t k = 0; k < K; ++k)
            for (int64_t n = 0; n < N; ++n) {
                int nib;
                int64_t idx = orc_fp4ref_locate(k, n, N, &nib);
                uint8_t code = nib ? (wb[idx] >> 4) : (wb[idx] & 15);
                float v = orc_e2m1_decode(code) * bf16_to_f32(sc[(k / gs) * N + n]);
                out[k * N + n] = round_bf16 ? bf16_to_f32(f32_to_bf16_rne(v)) : v;
            }
    } else if (fmt == ORC_FMT_FP8_REF) {
        const uint8_t *wb = (const uint8_t *)w + g * K * N;
        int64_t sk = (K + 127) / 128, sn = (N + 127) / 128;
        const float *sc = (const float *)scale + g * sk * sn;
#pragma omp parallel for schedule(static)
        for (int64_t k = 0; k < K; ++k)
            for (int64_t n = 0; n < N; ++n) {
                float v = orc_e4m3_decode(wb[k * N + n]) * sc[(k / 128) * sn + n / 128];
                out[k * N + n] = round_bf16 ? bf16_to_f32(f32_to_bf16_rne(v)) : v;
            }
    } else if (fmt == ORC_FMT_INT8) {
        /* CANN antiquant convention (weight + offset) * scale, per output channel. */
        const int8_t *wb = (const int8_t *)w + g * K * N;
        const uint16_t *sc = (const uint16_t *)scale + g * N;
        const uint16_t *of = (const uint16_t *)offset + g * N;
#pragma omp parallel for schedule(static)
        for (int64_t k = 0; k < K; ++k)
            for (int64_t n = 0; n < N; ++n) {
                float sum = (float)wb[k * N + n] + bf16_to_f32(of[n]); /* built with -ffp-contract=off */
                float v = sum * bf16_to_f32(sc[n]);
                out[k * N + n] = round_bf16 ? bf16_to_f32(f32_to_bf16_rne(v)) : v;
            }
    } else if (fmt == ORC_FMT_INT4) {
        const uint8_t *wb = (const uint8_t *)w + g * K * (N / 2);
        const uint16_t *sc = (const uint16_t *)scale + g * scale_rows * N;
        int64_t gs = K / scale_rows;
#pragma omp parallel for schedule(static)
        for (int64_t k = 0; k < K; ++k)
            for (int64_t n = 0; n < N; ++n) {
                uint8_t byte = wb[k * (N / 2) + (n >> 1)];
                int q = (n & 1) ? (byte >> 4) : (byte & 15);
                float v = (float)(q - 8) * bf16_to_f32(sc[(k / gs) * N + n]);
                out[k * N + n] = round_bf16 ? bf16_to_f32(f32_to_bf16_rne(v)) : v;
            }
    } else if (fmt == ORC_FMT_FP4_B32 || fmt == ORC_FMT_FP4_B16) {
        const int64_t blk = fmt == ORC_FMT_FP4_B32 ? 32 : 16;
        const uint8_t *wb = (const uint8_t *)w + g * N * (K / 2);
        const uint16_t *sc = (const uint16_t *)scale + g * N * (K / blk);
#pragma omp parallel for schedule(static)
        for (int64_t k = 0; k < K; ++k)
            for (int64_t n = 0; n < N; ++n) {
                uint8_t byte = wb[n * (K / 2) + (k >> 1)];
                uint8_t code = (k & 1) ? (byte >> 4) : (byte & 15);
                float v = orc_e2m1_decode(code) * bf16_to_f32(sc[n * (K / blk) + k / blk]);
                out[k * N + n] = round_bf16 ? bf16_to_f32(f32_to_bf16_rne(v)) : v;
            }
    } else if (fmt == ORC_FMT_BF16) {
        const uint16_t *wb = (const uint16_t *)w + g * N * K;
#pragma omp parallel for schedule(static)
        for (int64_t k = 0; k < K; ++k)
            for (int64_t n = 0; n < N; ++n) out[k * N + n] = bf16_to_f32(wb[n * K + k]);
    } else {
        return -1;
    }
    return 0;
}

/* y[rows] = x[rows] . W for the listed rows of one expert; fp32 accumulation in
 * ascending k.  Blocked (MB rows x NB columns of accumulators) so the dense W
 * is streamed once per row block. */
#define ORC_MB 8
#define ORC_NB 512
static void matmul_rows(const uint16_t *x, const float *W, const int64_t *rows, int64_t nrows,
                        int64_t K, int64_t N, float *y32, uint16_t *y16) {
    int64_t nmb = (nrows + ORC_MB - 1) / ORC_MB, nnb = (N + ORC_NB - 1) / ORC_NB;
#pragma omp parallel for schedule(dynamic) collapse(2)
    for (int64_t mb = 0; mb < nmb; ++mb)
        for (int64_t nb = 0; nb < nnb; ++nb) {
            float acc[ORC_MB][ORC_NB];
            int64_t m0 = mb * ORC_MB, m1 = m0 + ORC_MB < nrows ? m0 + ORC_MB : nrows;
            int64_t n0 = nb * ORC_NB, n1 = n0 + ORC_NB < N ? n0 + ORC_NB : N;
            memset(acc, 0, sizeof(acc));
            for (int64_t k = 0; k < K; ++k) {
                const float *wr = W + k * N + n0;
                for (int64_t mi = m0; mi < m1; ++mi) {
                    float xv = bf16_to_f32(x[rows[mi] * K + k]);
                    float *a = acc[mi - m0];
                    for (int64_t n = 0; n < n1 - n0; ++n) a[n] += xv * wr[n];
                }
            }
            for (int64_t mi = m0; mi < m1; ++mi)
                for (int64_t n = n0; n < n1; ++n) {
                    float v = acc[mi - m0][n - n0];
                    if (y32) y32[rows[mi] * N + n] = v;
                    if (y16) y16[rows[mi] * N + n] = f32_to_bf16_rne(v);
                }
        }
}

/* Grouped matmul with weight antiquant.
 * group_list is cumulative: rows [gl[g-1], gl[g]) of x and y belong to expert g,
 * gl[-1] = 0; rows at or beyond gl[G-1] are left untouched
 * (grouped_gemm/op_kernel/grouped_matmul_utils.h:304-320;
 * grouped_soft_gemv/op_kernel/grouped_soft_gemv.h:10-16, :235-266;
 * expected value of the tests: per-expert y = x . dequant(W), fp32 accumulate,
 * bf16 output, test_group_gemm_fp4.py:199-217, test_group_gemm_fp8.py:52-59).
 * row_mask (optional, uint8 [M]) limits the work to rows whose mask is set.
 * y16 (bf16 [M,N]) and y32 (fp32 [M,N]) are both optional outputs. */
int orc_grouped_gemm(int fmt, const uint16_t *x, const void *w, const void *scale,
                     const void *offset, const int64_t *group_list, int64_t M, int64_t K,
                     int64_t N, int64_t G, int64_t scale_rows, int round_bf16,
                     const uint8_t *row_mask, uint16_t *y16, float *y32) {
    float *W = (float *)malloc((size_t)K * N * sizeof(float));
    int64_t *rows = (int64_t *)malloc((size_t)(M > 0 ? M : 1) * sizeof(int64_t));
    if (!W || !rows) {
        free(W);
        free(rows);
        return -2;
    }
    int64_t prev = 0;
    int rc = 0;
    for (int64_t g = 0; g < G && rc == 0; ++g) {
        int64_t end = group_list[g];
        if (end < prev || end > M) {
            rc = -3;
            break;
        }
        int64_t nrows = 0;
        for (int64_t m = prev; m < end; ++m)
            if (!row_mask || row_mask[m]) rows[nrows++] = m;
        prev = end;
        if (nrows == 0) continue;
        rc = orc_expand_weight(fmt, w, scale, offset, g, K, N, scale_rows, round_bf16, W);
        if (rc == 0) matmul_rows(x, W, rows, nrows, K, N, y32, y16);
    }
    free(W);
    free(rows);
    return rc;
}
