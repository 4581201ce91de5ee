// Routing for the grouped ops on gfx950: router logits -> top-k experts per token -> rows sorted
// by expert + the cumulative group_list that grouped_gemm / grouped_soft_gemv read
// (grouped_gemm/op_kernel/grouped_matmul_utils.h:304-320 defines that tensor; the reference leaves
// building it to its caller).  Everything stays on the device: no host round trip between the
// router and the expert GEMMs.
//
// Order of the sorted rows: by expert id, then by flat choice index t * topk + j (a stable sort), so
// the result is deterministic and independent of the launch geometry.
//
//   route_topk_kernel    one wavefront per token: softmax statistics and top-k by repeated arg-max
//   route_count_kernel   per 1024-choice block, a histogram over experts (LDS atomics)
//   route_scan_kernel    one workgroup: per expert, prefix over the blocks; then over experts
//   route_rank_kernel    per block, every choice's rank among the earlier choices of its expert
//   route_gather_kernel  x rows copied into sorted order, 16 bytes per lane
#include <atomic>

#include "moe_device.h"
#include "moe_internal.h"

namespace moe {

constexpr int RT_BLOCK = 1024;     // choices per block of the count / rank kernels
constexpr int RT_MAX_E = 1024;     // experts (one thread each in the scan kernel)
constexpr int RT_MAX_PER_LANE = RT_MAX_E / 64;

__global__ __launch_bounds__(256) void route_topk_kernel(const float* __restrict__ logits, float* __restrict__ weight,
                                                         int32_t* __restrict__ ids, int T, int E, int topk) {
    const int lane = threadIdx.x & 63;
    const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= T) return;
    const float* row = logits + (int64_t)t * E;
    float v[RT_MAX_PER_LANE];
    float mx = -INFINITY;
#pragma unroll
    for (int c = 0; c < RT_MAX_PER_LANE; ++c) {
        const int e = c * 64 + lane;
        v[c] = e < E ? row[e] : -INFINITY;
        mx = fmaxf(mx, v[c]);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
    float sum = 0.f;
#pragma unroll
    for (int c = 0; c < RT_MAX_PER_LANE; ++c)
        if (c * 64 + lane < E) sum += __expf(v[c] - mx);
    sum = wave_reduce_sum(sum);
    const float inv = 1.f / sum;
    for (int j = 0; j < topk; ++j) {
        // arg-max over what is left; ties go to the lower expert id
        float bv = -INFINITY;
        int be = 0x7fffffff;
#pragma unroll
        for (int c = 0; c < RT_MAX_PER_LANE; ++c) {
            const int e = c * 64 + lane;
            if (e < E && (v[c] > bv || (v[c] == bv && e < be))) { bv = v[c]; be = e; }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float ov = __shfl_xor(bv, off, 64);
            const int oe = __shfl_xor(be, off, 64);
            if (ov > bv || (ov == bv && oe < be)) { bv = ov; be = oe; }
        }
        if (lane == 0) {
            ids[(int64_t)t * topk + j] = be;
            weight[(int64_t)t * topk + j] = __expf(bv - mx) * inv;
        }
#pragma unroll
        for (int c = 0; c < RT_MAX_PER_LANE; ++c)
            if (c * 64 + lane == be) v[c] = -INFINITY;
    }
}

__global__ __launch_bounds__(RT_BLOCK) void route_count_kernel(const int32_t* __restrict__ ids, int32_t* __restrict__ block_counts,
                                                               int64_t n, int E) {
    __shared__ int hist[RT_MAX_E];
    for (int e = threadIdx.x; e < E; e += RT_BLOCK) hist[e] = 0;
    __syncthreads();
    const int64_t i = (int64_t)blockIdx.x * RT_BLOCK + threadIdx.x;
    if (i < n) {
        const int e = ids[i];
        if ((unsigned)e < (unsigned)E) atomicAdd(&hist[e], 1);   // ids outside [0, E) are dropped
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += RT_BLOCK) block_counts[(int64_t)blockIdx.x * E + e] = hist[e];
}

// block_counts[b][e] -> block_base[b][e] = first sorted row of block b's choices of expert e;
// group_list[e] = rows of experts <= e.  Input and output are separate arrays so that the loads of
// a thread's column do not have to wait for its stores.
__global__ __launch_bounds__(RT_MAX_E) void route_scan_kernel(const int32_t* __restrict__ block_counts,
                                                              int32_t* __restrict__ block_base,
                                                              int64_t* __restrict__ group_list, int nblocks, int E) {
    __shared__ int scan[RT_MAX_E];
    const int e = threadIdx.x;
    int total = 0;
    if (e < E)
        for (int b = 0; b < nblocks; ++b) total += block_counts[(int64_t)b * E + e];
    scan[e] = e < E ? total : 0;
    __syncthreads();
    // inclusive scan over experts (Hillis-Steele, 10 steps for 1024)
    for (int off = 1; off < RT_MAX_E; off <<= 1) {
        const int add = e >= off ? scan[e - off] : 0;
        __syncthreads();
        scan[e] += add;
        __syncthreads();
    }
    if (e < E) {
        group_list[e] = scan[e];
        int run = scan[e] - total;
        for (int b = 0; b < nblocks; ++b) {
            block_base[(int64_t)b * E + e] = run;
            run += block_counts[(int64_t)b * E + e];
        }
    }
}

__global__ __launch_bounds__(RT_BLOCK) void route_rank_kernel(const int32_t* __restrict__ ids, const int32_t* __restrict__ block_base,
                                                              int32_t* __restrict__ row_token, int32_t* __restrict__ row_of_choice,
                                                              int64_t n, int E, int topk) {
    __shared__ int sid[RT_BLOCK];
    const int64_t i = (int64_t)blockIdx.x * RT_BLOCK + threadIdx.x;
    const int my = i < n ? ids[i] : -1;
    sid[threadIdx.x] = my;
    __syncthreads();
    if (i >= n) return;
    if ((unsigned)my >= (unsigned)E) {
        row_of_choice[i] = -1;
        return;
    }
    int rank = 0;
    for (int j = 0; j < (int)threadIdx.x; ++j) rank += sid[j] == my;
    const int dst = block_base[(int64_t)blockIdx.x * E + my] + rank;
    row_token[dst] = (int32_t)(i / topk);
    row_of_choice[i] = dst;
}

__global__ __launch_bounds__(256) void route_gather_kernel(const u32x4_t* __restrict__ x, const int32_t* __restrict__ row_token,
                                                           const int64_t* __restrict__ group_list, int E,
                                                           u32x4_t* __restrict__ x_sorted, int64_t n, int units) {
    // 4 rows per workgroup, one wavefront each
    const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    // Only rows below group_list[E - 1] (written by the scan kernel earlier on this stream) have a token:
    // dropped choices leave the tail of row_token unwritten, and the tail of x_sorted stays untouched.
    if (r >= n || r >= group_list[E - 1]) return;
    const u32x4_t* src = x + (int64_t)row_token[r] * units;
    u32x4_t* dst = x_sorted + r * units;
    // 8 independent 16-byte loads in flight per lane
    for (int u0 = threadIdx.x & 63; u0 < units; u0 += 8 * 64) {
        u32x4_t v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j)
            if (u0 + 64 * j < units) v[j] = src[u0 + 64 * j];
#pragma unroll
        for (int j = 0; j < 8; ++j)
            if (u0 + 64 * j < units) __builtin_nontemporal_store(v[j], dst + u0 + 64 * j);
    }
}

size_t route_workspace_bytes(const moe_route_args* a) {
    const int64_t n = a->T * a->topk;
    const int64_t nblocks = (n + RT_BLOCK - 1) / RT_BLOCK;
    return (size_t)(2 * nblocks * a->E) * sizeof(int32_t);   // per-block counts and per-block first rows
}

// Scratch of moe_route_static: the per-block counts and first rows live in this array instead of a
// caller-provided workspace.  One copy per GPU, held until the process ends; every call on a GPU uses
// that GPU's copy (the count kernel rewrites all of the part a call reads, so nothing needs clearing,
// but two calls that overlap in time on one GPU race on it).
static __device__ __align__(256) unsigned char scratch[MOE_ROUTE_STATIC_SCRATCH_BYTES];

// Device address of `scratch` on each GPU (the array's name is only a host-side handle).  Filled on the
// first call on a device, with that device current.
constexpr int RT_MAX_DEVICES = 64;
static std::atomic<void*> scratch_addr[RT_MAX_DEVICES];

int launch_route_static(const moe_route_args* a, hipStream_t stream) {
    if (route_workspace_bytes(a) > (size_t)MOE_ROUTE_STATIC_SCRATCH_BYTES) return MOE_ERR_TOO_LARGE;
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= RT_MAX_DEVICES) return MOE_ERR_NO_DEVICE;
    void* ptr = scratch_addr[dev].load(std::memory_order_acquire);
    if (!ptr) {
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return MOE_ERR_NO_DEVICE;
        scratch_addr[dev].store(ptr, std::memory_order_release);   // a race stores the same address twice
    }
    moe_route_args b = *a;
    b.workspace = ptr;
    return launch_route(&b, stream);
}

int launch_route(const moe_route_args* a, hipStream_t stream) {
    const int64_t n = a->T * a->topk;
    const int nblocks = (int)((n + RT_BLOCK - 1) / RT_BLOCK);
    int32_t* ids = static_cast<int32_t*>(a->topk_ids);
    int32_t* counts = static_cast<int32_t*>(a->workspace);
    int32_t* base = counts + (int64_t)nblocks * a->E;
    if (a->logits && a->T > 0) {
        hipLaunchKernelGGL(route_topk_kernel, dim3((unsigned)((a->T + 3) / 4)), dim3(256), 0, stream,
                           static_cast<const float*>(a->logits), static_cast<float*>(a->topk_weight), ids, (int)a->T,
                           (int)a->E, (int)a->topk);
        if (hipGetLastError() != hipSuccess) return MOE_ERR_LAUNCH;
    }
    if (nblocks > 0)
        hipLaunchKernelGGL(route_count_kernel, dim3((unsigned)nblocks), dim3(RT_BLOCK), 0, stream, ids, counts, n, (int)a->E);
    hipLaunchKernelGGL(route_scan_kernel, dim3(1), dim3(RT_MAX_E), 0, stream, counts, base,
                       static_cast<int64_t*>(a->group_list), nblocks, (int)a->E);
    if (nblocks > 0)
        hipLaunchKernelGGL(route_rank_kernel, dim3((unsigned)nblocks), dim3(RT_BLOCK), 0, stream, ids, base,
                           static_cast<int32_t*>(a->row_token), static_cast<int32_t*>(a->row_of_choice), n, (int)a->E,
                           (int)a->topk);
    if (hipGetLastError() != hipSuccess) return MOE_ERR_LAUNCH;
    if (a->x && n > 0) {
        hipLaunchKernelGGL(route_gather_kernel, dim3((unsigned)((n + 3) / 4)), dim3(256), 0, stream,
                           static_cast<const u32x4_t*>(a->x), static_cast<const int32_t*>(a->row_token),
                           static_cast<const int64_t*>(a->group_list), (int)a->E, static_cast<u32x4_t*>(a->x_sorted), n,
                           (int)(a->K / 8));
        if (hipGetLastError() != hipSuccess) return MOE_ERR_LAUNCH;
    }
    return MOE_OK;
}

}  // namespace moe
