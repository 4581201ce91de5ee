/*
 * moe_gfx950.h -- C ABI of libmoe_gfx950.so: MI355X (gfx950) kernels for the three
 * MoE inference ops that QingCheng-AI/ascend-kernel exposes as `cinfer_ascendc`.
 *
 * Plain C: raw device pointers, sizes, an opaque stream handle.  No torch types.
 * Every launch is asynchronous on the given stream, never synchronizes the
 * device, never copies group_list to the host and allocates nothing.  The only
 * state between calls is set-up done once per process or GPU (a kernel attribute,
 * the CU count, the address of moe_route_static's scratch array) and the tile counters
 * of the grouped GEMM kernels: 256 KB of the library's own device memory, 4096 slots of
 * one counter.  An eager launch takes the next slot and raises its counter to a stamp
 * that grows with every use of the slot, so nothing a kernel leaves in a slot can mislead
 * a later one; launches may overlap on different streams.  The one arrangement to avoid:
 * a launch that is still running when the 4096th grouped launch after it starts (that
 * later launch may then miss tiles; a launch that merely starts that late notices and
 * disturbs nobody).  A launch made while its stream is being captured into a HIP graph
 * takes no slot and walks its tiles in a fixed order, so graphs may be replayed any
 * number of times, beside each other and beside eager launches.
 * Calls are re-entrant except where moe_route_static says otherwise.  All functions
 * return MOE_OK (0) or a negative moe_status; nothing throws across this boundary.
 *
 * What each entry point replaces in the reference (paths relative to its tree):
 *   moe_grouped_gemm            aclnnGroupedMatmulAntiquant{GetWorkspaceSize,}
 *                               as called at grouped_gemm/src/grouped_gemm.cpp:145-157,
 *                               i.e. kernel grouped_matmul_antiquant,
 *                               grouped_gemm/op_kernel/grouped_matmul_antiquant.cpp:146-162
 *   moe_grouped_gemv            aclnnGroupedSoftGemv{GetWorkspaceSize,} as called at
 *                               grouped_soft_gemv/src/grouped_soft_gemv.cpp:141-150,
 *                               i.e. kernel grouped_soft_gemv,
 *                               grouped_soft_gemv/op_kernel/grouped_soft_gemv.cpp:24-37
 *   moe_dequant_fp4_bf16        phase 1 of the GEMM kernel made a stand-alone op:
 *                               CastWeightProcess, grouped_gemm/op_kernel/grouped_matmul_antiquant.h:537-662
 *                               + antiquantProcess, grouped_gemm/op_kernel/antiquant_impl.h:146-208
 *   moe_*_validate              the shape/dtype checks of op_host tiling,
 *                               grouped_gemm/op_host/grouped_matmul_antiquant_tiling.cpp:246-313
 *   moe_*_workspace_bytes       the GetWorkspaceSize half of the aclnn pair
 *                               (grouped_gemm/src/grouped_gemm.cpp:145-154); always 0 here
 *   moe_format_from_compute_type  the computeType string switch,
 *                               grouped_gemm/src/grouped_gemm.cpp:129-135
 */
#ifndef MOE_GFX950_H
#define MOE_GFX950_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MOE_GFX950_ABI_VERSION 1

/* hipStream_t, passed opaquely so that this header needs no HIP include. */
typedef void *moe_stream_t;

/* Experts per call of either grouped op.  (moe_grouped_gemm keeps a table of G + 1 tile counts in LDS next to its
 * tile buffers while that fits -- about 2500 to 5300 experts, depending on the kernel -- and beyond that one
 * entry per thread, walking group_list for the rest: any count works, small ones are faster.) */
#define MOE_GEMM_MAX_EXPERTS 65535

typedef enum moe_status {
    MOE_OK = 0,
    MOE_ERR_NULL_POINTER = -1,   /* a required pointer is NULL                        */
    MOE_ERR_BAD_FORMAT = -2,     /* unknown weight format / computeType               */
    MOE_ERR_BAD_SHAPE = -3,      /* negative size, or a size the format cannot hold   */
    MOE_ERR_BAD_ALIGNMENT = -4,  /* K/N/cols not a multiple the kernels need, or a
                                    pointer not aligned to 16 bytes                   */
    MOE_ERR_TOO_LARGE = -5,      /* M, K, N or G beyond int32 (reference limit,
                                    grouped_matmul_antiquant_tiling.cpp:260-264); one
                                    expert's weight or scale slab of 2 GiB or more, or
                                    K or N of 4194304 or more (32-bit byte offsets);
                                    more than MOE_GEMM_MAX_EXPERTS (65535) experts    */
    MOE_ERR_LAUNCH = -6,         /* hipLaunchKernel reported an error                 */
    MOE_ERR_NO_DEVICE = -7       /* no gfx950 device / wrong architecture             */
} moe_status;

/*
 * Weight containers.  G experts; logical weight of expert g is B[g][k][n] with
 * y = x . dequant(B).  "scale_rows" below is scale.shape[-2].
 *
 * MOE_FMT_FP4_REF  reference computeType "fp4": int8 [G, K, N/2], e2m1 codes packed
 *                  along N (low nibble = even n) then byte-permuted inside every
 *                  64(k) x 128(byte) tile exactly as the reference test prepares it
 *                  (grouped_gemm/test/python/test_group_gemm_fp4.py:105-117, :129-142);
 *                  scale bf16 [G, K/16, N]; offset ignored (the reference never reads it).
 *                  K % 64 == 0, N % 256 == 0.
 * MOE_FMT_FP8_REF  reference computeType "fp8": uint8 [G, K, N] e4m3 bits decoded with
 *                  the reference's bit trick (0x7F/0xFF give +-480, no NaN);
 *                  scale fp32 [G, K/128, N/128]; offset ignored.  K % 128 == 0, N % 128 == 0
 *                  (every other N-contiguous container: N % 256 == 0).
 * MOE_FMT_INT8     int8 [G, K, N]; scale bf16 [G, N]; offset bf16 [G, N];
 *                  W = bf16((float(q) + float(offset)) * float(scale)).
 * MOE_FMT_INT4     uint8 [G, K, N/2], low nibble = even n, codes 0..15, zero point 8;
 *                  scale bf16 [G, K/group, N] (group = K / scale_rows, a multiple of 32);
 *                  W = bf16(float(q - 8) * float(scale)).
 * MOE_FMT_FP4_B32  uint8 [G, N, K/2] e2m1, K-contiguous, low nibble = even k;
 *                  scale bf16 [G, N, K/32]; W = bf16(e2m1(code) * float(scale)).
 *                  One expert is exactly a moe_dequant_fp4_bf16 input of N rows, K cols.
 *                  K % 32 == 0 (grouped GEMM: K % 128 == 0).
 * MOE_FMT_BF16     bf16 [G, N, K], K-contiguous; no scale.
 * MOE_FMT_FP4_B16  as MOE_FMT_FP4_B32 with one scale per 16 k: scale bf16 [G, N, K/16].  This is the
 *                  reference checkpoint's own orientation (codes [G, N, K/2], block scales
 *                  [G, N, K/16], grouped_gemm/test/python/test_group_gemm_fp4.py:46-64) with the
 *                  second-level scale multiplied in: no repacking between checkpoint and op.
 *                  K % 32 == 0 (grouped GEMM: K % 128 == 0).
 *
 * GEMM rounds W to bf16 before the product (reference phase 1); GEMV keeps the
 * fp32 product un-rounded (grouped_soft_gemv/op_kernel/gemv_impl.h:147-199).
 */
typedef enum moe_weight_format {
    MOE_FMT_FP4_REF = 0,
    MOE_FMT_FP8_REF = 1,
    MOE_FMT_INT8 = 2,
    MOE_FMT_INT4 = 3,
    MOE_FMT_FP4_B32 = 4,
    MOE_FMT_BF16 = 5,
    MOE_FMT_FP4_B16 = 6,
    MOE_FMT_COUNT = 7
} moe_weight_format;

/* What the grouped GEMM writes.  MOE_EPILOGUE_SWIGLU fuses the activation that sits between the
 * gate_up and the down projection of an MoE layer into the GEMM (no counterpart in the reference,
 * whose caller runs it as a separate op on the [M, N] result): y is bf16 [M, N/2] with
 *     y[m, c] = silu(z[m, gate(c)]) * z[m, up(c)],   silu(v) = v / (1 + exp(-v)),
 * z the fp32 accumulators of x . dequant(W).  The gate and up columns are interleaved the way each
 * container's lanes hold them:
 *   N-contiguous containers (MOE_FMT_FP4_REF, MOE_FMT_FP8_REF, MOE_FMT_INT8, MOE_FMT_INT4): groups of 4
 *   columns = (gate 2j, gate 2j+1, up 2j, up 2j+1): gate(2j+e) = 4j+e, up(2j+e) = 4j+2+e;
 *   K-contiguous containers (MOE_FMT_FP4_B32, MOE_FMT_FP4_B16, MOE_FMT_BF16): blocks of 32 weight rows =
 *   (gate 16j .. 16j+15, up 16j .. 16j+15): gate(16j+i) = 32j+i, up(16j+i) = 32j+16+i.
 * Grouped GEMM only. */
typedef enum moe_epilogue {
    MOE_EPILOGUE_NONE = 0,
    MOE_EPILOGUE_SWIGLU = 1
} moe_epilogue;

/* Arguments of both grouped ops.  x, y are row-major bf16; group_list is the
 * cumulative int64 [G] device tensor of the reference (rows [gl[g-1], gl[g]) belong
 * to expert g, gl[-1] = 0; rows at or beyond gl[G-1] are not written;
 * grouped_gemm/op_kernel/grouped_matmul_utils.h:304-320). */
typedef struct moe_grouped_args {
    const void *x;             /* bf16 [M, K]                                       */
    const void *weight;        /* container, see moe_weight_format                  */
    const void *scale;         /* NULL only for MOE_FMT_BF16                        */
    const void *offset;        /* read by MOE_FMT_INT8 only; may be NULL otherwise  */
    const int64_t *group_list; /* device int64 [G], cumulative                      */
    void *y;                   /* bf16 [M, N]  ([M, N/2] with MOE_EPILOGUE_SWIGLU)  */
    int64_t M, K, N, G;
    int64_t scale_rows;        /* scale.shape[-2]; used by FP4_REF (K/16) and INT4  */
    int32_t format;            /* moe_weight_format                                 */
    int32_t epilogue;          /* moe_epilogue; MOE_EPILOGUE_NONE (0) for the reference's ops */
} moe_grouped_args;

/* codes uint8 [rows, cols/2] (even element in the low nibble), scale bf16
 * [rows, cols/block], out bf16 [rows, cols]; block is 16 or 32.  Bit-exact:
 * out = RNE_bf16(float(e2m1(code)) * float(scale)), code 8 gives -0.0. */
typedef struct moe_dequant_args {
    const void *codes;
    const void *scale;
    void *out;
    int64_t rows, cols;
    int32_t block;
    int32_t reserved; /* must be 0 */
} moe_dequant_args;

/* Checkpoint tensors of the reference's NVFP4-style weights -> the MOE_FMT_FP4_REF container
 * (what the reference test builds on the host with repack_weight + repack_weight_step2 and the
 * scale merge / transpose, grouped_gemm/test/python/test_group_gemm_fp4.py:86-94, :105-142,
 * :180-186).  Bit-exact.  Either half may be skipped by passing NULL for both of its pointers.
 *   codes       uint8 [G, N, K/2], even k in the low nibble   -> weight_out int8 [G, K, N/2]
 *   scale       bf16  [G, N, K/16]                            -> scale_out  bf16 [G, K/16, N]
 *   scale2      optional fp32 [G, scale2_cols] second-level scale, multiplied in (fp32 product,
 *               RNE to bf16): scale2_cols = 1, or 2 for one factor per half of the N rows
 * K % 64 == 0, N % 256 == 0. */
typedef struct moe_prepack_fp4_args {
    const void *codes;
    const void *scale;
    const void *scale2;
    void *weight_out;
    void *scale_out;
    int64_t G, N, K;
    int32_t scale2_cols; /* 0 (scale2 ignored), 1 or 2 */
    int32_t reserved;    /* must be 0 */
} moe_prepack_fp4_args;

/* Routing: router logits -> top-k experts per token -> rows sorted by expert and the cumulative
 * group_list the grouped ops read (the reference leaves this step to its caller, which uses
 * torch_npu.npu_moe_init_routing for it; group_list as in
 * grouped_gemm/op_kernel/grouped_matmul_utils.h:304-320).  All device pointers.
 *   logits       fp32 [T, E], or NULL when topk_ids is already filled by the caller
 *   topk_ids     int32 [T, topk]   out (in, if logits is NULL); ids outside [0, E) are dropped
 *   topk_weight  fp32 [T, topk]    out: softmax probability of each chosen expert (not
 *                                  renormalised over the k); ignored if logits is NULL
 *   group_list   int64 [E]         out: rows of experts 0..e, cumulative
 *   row_token    int32 [T * topk]  out: token whose activations sorted row r holds
 *   row_of_choice int32 [T * topk] out: sorted row of choice (t, j) at [t * topk + j], -1 if dropped
 *   x            bf16 [T, K] or NULL;  x_sorted  bf16 [T * topk, K] out: x[row_token[r]]
 *   workspace    moe_route_workspace_bytes(args) bytes of device scratch, 4-byte aligned
 * Sorted order: by expert id, then by t * topk + j (stable).  Ties between logits go to the
 * lower expert id.  E <= 1024, topk <= E, K % 8 == 0. */
typedef struct moe_route_args {
    const void *logits;
    const void *x;
    void *topk_ids;
    void *topk_weight;
    int64_t *group_list;
    void *row_token;
    void *row_of_choice;
    void *x_sorted;
    void *workspace;
    int64_t T, E, K;
    int32_t topk;
    int32_t reserved; /* must be 0 */
} moe_route_args;

int moe_abi_version(void);
const char *moe_strerror(int status);

/* "fp4" | "fp8" (reference values) | "int8" | "int4" | "fp4_b32" | "bf16" | "fp4_b16";
 * returns the moe_weight_format or MOE_ERR_BAD_FORMAT. */
int moe_format_from_compute_type(const char *compute_type);

/* Host-only argument checks (usable without a GPU). */
int moe_dequant_fp4_bf16_validate(const moe_dequant_args *args);
int moe_grouped_gemm_validate(const moe_grouped_args *args);
int moe_grouped_gemv_validate(const moe_grouped_args *args);
int moe_prepack_fp4_ref_validate(const moe_prepack_fp4_args *args);
int moe_route_validate(const moe_route_args *args);

/* Device scratch the launch needs (the reference's two-phase GetWorkspaceSize protocol): 0 for
 * every op except moe_route, whose caller passes that many bytes in args->workspace. */
size_t moe_dequant_fp4_bf16_workspace_bytes(const moe_dequant_args *args);
size_t moe_grouped_gemm_workspace_bytes(const moe_grouped_args *args);
size_t moe_grouped_gemv_workspace_bytes(const moe_grouped_args *args);
size_t moe_prepack_fp4_ref_workspace_bytes(const moe_prepack_fp4_args *args);
size_t moe_route_workspace_bytes(const moe_route_args *args);

/* Launches (validate first, then enqueue on `stream`). */
int moe_dequant_fp4_bf16(const moe_dequant_args *args, moe_stream_t stream);
int moe_grouped_gemm(const moe_grouped_args *args, moe_stream_t stream);
int moe_grouped_gemv(const moe_grouped_args *args, moe_stream_t stream);
int moe_prepack_fp4_ref(const moe_prepack_fp4_args *args, moe_stream_t stream);
int moe_route(const moe_route_args *args, moe_stream_t stream);

/* moe_route for callers that cannot allocate device memory or carry a workspace around (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the
 * reference.  Same arguments and results as moe_route; args->workspace is ignored (may be NULL): the
 * scratch is a static device array inside the library, MOE_ROUTE_STATIC_SCRATCH_BYTES per GPU, held
 * until the process ends.  Calls whose moe_route_workspace_bytes() exceeds it return MOE_ERR_TOO_LARGE
 * (with 256 experts that is more than 2096128 routed choices T * topk).  Allocates nothing; the first
 * call on a GPU looks the array's address up (hipGetSymbolAddress), so make that call with the GPU
 * current and outside a stream capture.  All calls on one GPU share the array: calls that overlap in
 * time on the same GPU race on it -- keep them on one stream or otherwise ordered. */
#define MOE_ROUTE_STATIC_SCRATCH_BYTES (2u << 20)
int moe_route_static(const moe_route_args *args, moe_stream_t stream);

/* Test support, no counterpart in the reference and no use in production: moves the library's count of
 * grouped launches (which picks a launch's tile counter and stamp) by delta and returns the new count, so
 * that a test can make a launch find its counter taken over by a later one. */
int64_t moe_test_shift_launch_number(int64_t delta);

#ifdef __cplusplus
}
#endif
#endif /* MOE_GFX950_H */
