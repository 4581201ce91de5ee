/* Host-side sanitizer run of the CPU oracle (test infrastructure): every entry point of moe_oracle.c on exactly
 * sized heap buffers, so that AddressSanitizer / UBSan see any read or write past an operand.  Built and run by
 * `make -C oracle asan`; prints "sanitize_check ok" and returns 0 when nothing was flagged. */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

float orc_e2m1_decode(uint8_t code);
float orc_e4m3_decode(uint8_t code);
uint16_t orc_f32_to_bf16(float f);
int64_t orc_fp4ref_locate(int64_t k, int64_t n, int64_t N, int *nibble);
void orc_dequant_fp4_bf16(const uint8_t *codes, const uint16_t *scale, uint16_t *out, int64_t R, int64_t C, int64_t block);
int orc_grouped_gemm(int fmt, const uint16_t *x, const void *w, const void *scale, const void *offset,
                     const int64_t *group_list, int64_t M, int64_t K, int64_t N, int64_t G, int64_t scale_rows,
                     int round_bf16, const uint8_t *row_mask, uint16_t *y16, float *y32);

static uint32_t rng_state = 12345u;
static uint32_t rnd(void) { return rng_state = rng_state * 1664525u + 1013904223u; }
static void *filled(size_t bytes, int bf16_small) {
    uint8_t *p = (uint8_t *)malloc(bytes ? bytes : 1);
    if (!p) exit(2);
    for (size_t i = 0; i < bytes; ++i) p[i] = (uint8_t)(rnd() >> 24);
    if (bf16_small)   /* bf16 values of moderate size: exponent byte 0x3c..0x3f */
        for (size_t i = 1; i < bytes; i += 2) p[i] = (uint8_t)(0x3c + (p[i] & 3)) | (p[i] & 0x80);
    return p;
}

int main(void) {
    for (int c = 0; c < 256; ++c) { (void)orc_e2m1_decode((uint8_t)(c & 15)); (void)orc_e4m3_decode((uint8_t)c); }
    (void)orc_f32_to_bf16(1.0f);
    /* dequant: blocks of 32 and 16, a row count that is not a multiple of anything */
    for (int block = 16; block <= 32; block += 16) {
        const int64_t R = 7, C = 96;
        uint8_t *codes = filled((size_t)(R * C / 2), 0);
        uint16_t *scale = filled((size_t)(R * (C / block) * 2), 1);
        uint16_t *out = malloc((size_t)(R * C * 2));
        orc_dequant_fp4_bf16(codes, scale, out, R, C, block);
        free(codes); free(scale); free(out);
    }
    /* grouped GEMM on every container (formats 0..6 of moe_weight_format), both roundings, with an empty
     * expert, rows beyond group_list[-1] and a row mask */
    const int64_t G = 3, K = 128, N = 256, M = 9;
    const int64_t gl[3] = {4, 4, 7};
    uint8_t mask[9] = {1, 0, 1, 1, 1, 1, 0, 1, 1};
    for (int fmt = 0; fmt < 7; ++fmt) {
        int nib;
        if (fmt == 0) (void)orc_fp4ref_locate(K - 1, N - 1, N, &nib);
        size_t wbytes, sbytes;
        int64_t scale_rows = 1;
        switch (fmt) {
            case 0: wbytes = G * K * N / 2; scale_rows = K / 16; sbytes = G * scale_rows * N * 2; break;
            case 1: wbytes = G * K * N; sbytes = G * (K / 128) * (N / 128) * 4; break;
            case 2: wbytes = G * K * N; sbytes = G * N * 2; break;
            case 3: wbytes = G * K * N / 2; scale_rows = K / 64; sbytes = G * scale_rows * N * 2; break;
            case 4: wbytes = G * K * N / 2; sbytes = G * N * (K / 32) * 2; break;
            case 5: wbytes = G * K * N * 2; sbytes = 0; break;
            default: wbytes = G * K * N / 2; sbytes = G * N * (K / 16) * 2; break;
        }
        uint16_t *x = filled((size_t)(M * K * 2), 1);
        void *w = filled(wbytes, fmt == 5);
        void *scale;
        if (fmt == 1) {
            float *s = malloc(sbytes);
            for (size_t i = 0; i < sbytes / 4; ++i) s[i] = 1e-3f * (float)(1 + (rnd() >> 28));
            scale = s;
        } else {
            scale = filled(sbytes, 1);
        }
        void *offset = filled((size_t)(G * N * 2), 1);
        for (int round_bf16 = 0; round_bf16 < 2; ++round_bf16) {
            uint16_t *y16 = malloc((size_t)(M * N * 2));
            float *y32 = malloc((size_t)(M * N * 4));
            memset(y16, 0, (size_t)(M * N * 2));
            int rc = orc_grouped_gemm(fmt, x, w, fmt == 5 ? NULL : scale, fmt == 2 ? offset : NULL, gl, M, K, N, G, scale_rows,
                                      round_bf16, round_bf16 ? mask : NULL, y16, round_bf16 ? NULL : y32);
            if (rc != 0) { printf("orc_grouped_gemm(fmt %d) returned %d\n", fmt, rc); return 1; }
            free(y16); free(y32);
        }
        free(x); free(w); free(scale); free(offset);
    }
    printf("sanitize_check ok\n");
    return 0;
}
