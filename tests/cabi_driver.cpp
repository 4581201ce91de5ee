// Torch-free driver of the C ABI in include/moe_gfx950.h: plain HIP allocations, the library's entry points, and
// the CPU oracle (oracle/libmoe_oracle.so, loaded with dlopen) as the checker.  What a C++ caller of the reference's
// adapters (grouped_gemm/src/grouped_gemm.cpp:122-161) would do with this library instead of the aclnn calls.
// Built by ascend-kernel_amd/build.py into ascend-kernel_amd/cabi_driver; run by tests/test_gpu_cabi_driver.py.
//   cabi_driver <path to libmoe_oracle.so>      exit code 0 = all checks passed
#include <dlfcn.h>
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "moe_gfx950.h"

#define HIP_OK(x)                                                                     \
    do {                                                                              \
        hipError_t e_ = (x);                                                          \
        if (e_ != hipSuccess) {                                                       \
            std::printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); \
            return 2;                                                                 \
        }                                                                             \
    } while (0)

typedef void (*orc_dequant_t)(const uint8_t*, const uint16_t*, uint16_t*, int64_t, int64_t, int64_t);
typedef int (*orc_gemm_t)(int, const uint16_t*, const void*, const void*, const void*, const int64_t*, int64_t, int64_t, int64_t,
                          int64_t, int64_t, int, const uint8_t*, uint16_t*, float*);

static uint32_t rng_state = 2024u;
static uint32_t rnd() { return rng_state = rng_state * 1664525u + 1013904223u; }
static float bf16_to_f32(uint16_t h) { uint32_t u = (uint32_t)h << 16; float f; std::memcpy(&f, &u, 4); return f; }
static uint16_t f32_to_bf16(float f) { uint32_t u; std::memcpy(&u, &f, 4); u += 0x7fffu + ((u >> 16) & 1u); return (uint16_t)(u >> 16); }

template <typename T>
static T* to_device(const std::vector<T>& h) {
    T* d = nullptr;
    if (hipMalloc(reinterpret_cast<void**>(&d), h.size() * sizeof(T) + 16) != hipSuccess) return nullptr;
    if (hipMemcpy(d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice) != hipSuccess) return nullptr;
    return d;
}

int main(int argc, char** argv) {
    if (argc < 2) { std::printf("usage: cabi_driver <libmoe_oracle.so>\n"); return 2; }
    void* orc = dlopen(argv[1], RTLD_NOW);
    if (!orc) { std::printf("cannot load the oracle: %s\n", dlerror()); return 2; }
    auto orc_dequant = reinterpret_cast<orc_dequant_t>(dlsym(orc, "orc_dequant_fp4_bf16"));
    auto orc_gemm = reinterpret_cast<orc_gemm_t>(dlsym(orc, "orc_grouped_gemm"));
    if (!orc_dequant || !orc_gemm) { std::printf("oracle symbols missing\n"); return 2; }
    if (moe_abi_version() != MOE_GFX950_ABI_VERSION) { std::printf("ABI version mismatch\n"); return 1; }
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));

    // ---- FP4 -> BF16 dequant, bit-exact
    {
        const int64_t R = 300, C = 1024, block = 32;
        std::vector<uint8_t> codes(R * C / 2);
        std::vector<uint16_t> scale(R * C / block), want(R * C), got(R * C);
        for (auto& c : codes) c = (uint8_t)(rnd() >> 24);
        for (auto& s : scale) s = f32_to_bf16(0.004f + 0.24f * (float)(rnd() >> 8) / 16777216.f);
        orc_dequant(codes.data(), scale.data(), want.data(), R, C, block);
        uint8_t* d_codes = to_device(codes);
        uint16_t* d_scale = to_device(scale);
        uint16_t* d_out = to_device(got);
        if (!d_codes || !d_scale || !d_out) return 2;
        moe_dequant_args a = {d_codes, d_scale, d_out, R, C, (int32_t)block, 0};
        if (moe_dequant_fp4_bf16_workspace_bytes(&a) != 0) { std::printf("dequant wants a workspace\n"); return 1; }
        int rc = moe_dequant_fp4_bf16(&a, stream);
        if (rc != MOE_OK) { std::printf("moe_dequant_fp4_bf16: %s\n", moe_strerror(rc)); return 1; }
        HIP_OK(hipStreamSynchronize(stream));
        HIP_OK(hipMemcpy(got.data(), d_out, got.size() * 2, hipMemcpyDeviceToHost));
        if (std::memcmp(got.data(), want.data(), got.size() * 2) != 0) { std::printf("dequant differs from the oracle\n"); return 1; }
        std::printf("dequant %lld x %lld: bit-exact\n", (long long)R, (long long)C);
        (void)hipFree(d_codes); (void)hipFree(d_scale); (void)hipFree(d_out);
    }
    // ---- grouped GEMM and grouped GEMV on int4 (zero point 8, groups of 128), within the parity tolerances
    for (int op = 0; op < 2; ++op) {
        const int64_t G = 4, K = 512, N = 512, group = 128;
        const int64_t gl_h[4] = {op ? 3 : 5, op ? 3 : 140, op ? 6 : 141, op ? 10 : 300};
        const int64_t M = gl_h[3] + 2;   // two rows beyond group_list[-1]: must stay untouched
        std::vector<uint16_t> x(M * K), scale(G * (K / group) * N), y(M * N, 0x7fc0), want(M * N, 0);
        std::vector<uint8_t> w(G * K * N / 2);
        std::vector<int64_t> gl(gl_h, gl_h + 4);
        for (auto& v : x) v = f32_to_bf16(((float)(rnd() >> 8) / 8388608.f - 1.f) * 1.7f);
        for (auto& v : w) v = (uint8_t)(rnd() >> 24);
        for (auto& v : scale) v = f32_to_bf16(1e-3f + 9e-3f * (float)(rnd() >> 8) / 16777216.f);
        int rc = orc_gemm(MOE_FMT_INT4, x.data(), w.data(), scale.data(), nullptr, gl.data(), M, K, N, G, K / group, op == 0,
                          nullptr, want.data(), nullptr);
        if (rc != 0) { std::printf("oracle failed: %d\n", rc); return 2; }
        uint16_t* d_x = to_device(x);
        uint8_t* d_w = to_device(w);
        uint16_t* d_s = to_device(scale);
        int64_t* d_gl = to_device(gl);
        uint16_t* d_y = to_device(y);
        if (!d_x || !d_w || !d_s || !d_gl || !d_y) return 2;
        moe_grouped_args a;
        std::memset(&a, 0, sizeof a);
        a.x = d_x; a.weight = d_w; a.scale = d_s; a.offset = nullptr; a.group_list = d_gl; a.y = d_y;
        a.M = M; a.K = K; a.N = N; a.G = G; a.scale_rows = K / group; a.format = MOE_FMT_INT4; a.epilogue = MOE_EPILOGUE_NONE;
        rc = op == 0 ? moe_grouped_gemm(&a, stream) : moe_grouped_gemv(&a, stream);
        if (rc != MOE_OK) { std::printf("%s: %s\n", op ? "moe_grouped_gemv" : "moe_grouped_gemm", moe_strerror(rc)); return 1; }
        HIP_OK(hipStreamSynchronize(stream));
        HIP_OK(hipMemcpy(y.data(), d_y, y.size() * 2, hipMemcpyDeviceToHost));
        double max_ref = 0, max_d = 0;
        for (int64_t i = 0; i < gl_h[3] * N; ++i) {
            const double r = bf16_to_f32(want[i]), g = bf16_to_f32(y[i]);
            max_ref = std::fmax(max_ref, std::fabs(r));
            max_d = std::fmax(max_d, std::fabs(g - r));
        }
        for (int64_t i = gl_h[3] * N; i < M * N; ++i)
            if (y[i] != 0x7fc0) { std::printf("a row beyond group_list[-1] was written\n"); return 1; }
        std::printf("%s int4: max|d| / max|ref| = %.3e\n", op ? "grouped_gemv" : "grouped_gemm", max_d / max_ref);
        if (!(max_d <= 1e-2 * max_ref)) return 1;
        (void)hipFree(d_x); (void)hipFree(d_w); (void)hipFree(d_s); (void)hipFree(d_gl); (void)hipFree(d_y);
    }
    // ---- error path: no launch, a negative status
    {
        moe_grouped_args a;
        std::memset(&a, 0, sizeof a);
        if (moe_grouped_gemm(&a, stream) >= 0) { std::printf("an empty argument block was accepted\n"); return 1; }
    }
    HIP_OK(hipStreamDestroy(stream));
    std::printf("cabi_driver ok\n");
    return 0;
}
