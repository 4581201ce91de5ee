// Routing for the grouped ops on gfx950: router logits -> top-k experts per token -> rows sorted
// by expert + the cumulative group_list that grouped_gemm / grouped_soft_gemv read
// (grouped_gemm/op_kernel/grouped_matmul_utils.h:304-320 defines that tensor; the reference leaves
// building it to its caller).  Everything stays on the device: no host round trip between the
// router and the expert GEMMs.
//
// Order of the sorted rows: by expert id, then by flat choice index t * topk + j (a stable sort), so
// the result is deterministic and independent of the launch geometry.
//
//   route_topk_kernel     one wavefront per token: softmax statistics and top-k by repeated arg-max
//   route_count_kernel    per 1024-choice block, a histogram over experts (LDS atomics)
//   route_scan_kernel     (many blocks only) the counts' prefix over the blocks, per expert
//   route_rank_kernel     per block: prefix of the counts over experts and earlier blocks (group_list), then every
//                         choice's rank among the earlier choices of its expert -> its sorted row
//   route_scatter_kernel  a token's x row read once and written to the sorted row of each of its choices
#include <atomic>

#include "moe_device.h"
#include "moe_internal.h"

namespace moe {

constexpr int RT_BLOCK = 1024;     // choices per block of the count / rank kernels
constexpr int RT_MAX_E = 1024;     // experts (one thread each in the scan kernel)
constexpr int RT_MAX_PER_LANE = RT_MAX_E / 64;

// PL = logits per lane (E <= 64 PL).  The arg-max over the wavefront is lexicographic in (value descending, expert
// ascending): a max-reduction of the lanes' best values, then the expert of the one lane that holds it (read with
// v_readlane); only when several lanes hold the maximum a second reduction picks the lowest expert among them.
template <int PL>
__global__ __launch_bounds__(256) void route_topk_kernel(const float* __restrict__ logits, float* __restrict__ weight,
                                                         int32_t* __restrict__ ids, int T, int E, int topk) {
    const int lane = threadIdx.x & 63;
    const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= T) return;
    const float* row = logits + (int64_t)t * E;
    float v[PL];
    float mx = -INFINITY;
#pragma unroll
    for (int c = 0; c < PL; ++c) {
        const int e = c * 64 + lane;
        v[c] = e < E ? row[e] : -INFINITY;
        mx = fmaxf(mx, v[c]);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
    float sum = 0.f;
#pragma unroll
    for (int c = 0; c < PL; ++c)
        if (c * 64 + lane < E) sum += __expf(v[c] - mx);
    sum = wave_reduce_sum(sum);
    const float inv = 1.f / sum;
    // experts already chosen, one bit per logit of this lane (a chosen expert cannot be marked with -inf: a
    // masked logit is -inf too, and a row with fewer than topk finite logits would pick it twice)
    unsigned taken = 0;
    for (int j = 0; j < topk; ++j) {
        // arg-max over what is left; ties go to the lower expert id
        float bv = -INFINITY;
        int be = 0x7fffffff;
#pragma unroll
        for (int c = 0; c < PL; ++c) {
            const int e = c * 64 + lane;
            if (e < E && !((taken >> c) & 1u) && (v[c] > bv || (v[c] == bv && e < be))) { bv = v[c]; be = e; }
        }
        float gv = bv;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) gv = fmaxf(gv, __shfl_xor(gv, off, 64));
        const unsigned long long holders = __ballot(bv == gv);
        int ge;
        if (__popcll(holders) == 1) {
            ge = __shfl(be, __ffsll(holders) - 1, 64);
        } else {
            ge = bv == gv ? be : 0x7fffffff;
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) ge = min(ge, __shfl_xor(ge, off, 64));
        }
        if (lane == 0) {
            ids[(int64_t)t * topk + j] = ge;
            weight[(int64_t)t * topk + j] = __expf(gv - mx) * inv;
        }
#pragma unroll
        for (int c = 0; c < PL; ++c)
            if (c * 64 + lane == ge) taken |= 1u << c;
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

// Many blocks: the per-block counts [nblocks][E] become, in place, each expert's exclusive prefix over the
// blocks, and row nblocks receives the experts' totals.  One wavefront per expert, 64 blocks per round
// (wavefront scan by shuffles, the running total carried from round to round).
constexpr int RT_FUSED_SCAN_MAX_BLOCKS = 64;   // up to here every rank block sums the counts itself
__global__ __launch_bounds__(256) void route_scan_kernel(int32_t* __restrict__ block_counts, int E, int nblocks) {
    const int lane = threadIdx.x & 63;
    const int e = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (e >= E) return;
    int carry = 0;
    for (int b0 = 0; b0 < nblocks; b0 += 64) {
        const int b = b0 + lane;
        const int c = b < nblocks ? block_counts[(int64_t)b * E + e] : 0;
        int incl = c;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int up = __shfl_up(incl, off, 64);
            if (lane >= off) incl += up;
        }
        if (b < nblocks) block_counts[(int64_t)b * E + e] = carry + incl - c;
        carry += __shfl(incl, 63, 64);
    }
    if (lane == 0) block_counts[(int64_t)nblocks * E + e] = carry;
}

// Rank of every choice of block b among the choices of its expert, and with it the sorted row:
//   row = (choices of lower experts) + (choices of this expert in earlier blocks) + (in earlier wavefronts of
//         this block) + (in lower lanes of this wavefront)
// With few blocks every block derives the first two terms from the per-block counts itself (nblocks x E integers
// per block: cheaper than a kernel of its own for the scan, but quadratic in the number of blocks); with more than
// RT_FUSED_SCAN_MAX_BLOCKS of them route_scan_kernel has turned the counts into prefixes and totals (prefixed != 0).
// Block 0 also writes group_list.  The third term comes from per-wavefront histograms in LDS, the fourth from
// comparing with the lanes below.  Dynamic LDS: (16 + 2) * E integers.
__global__ __launch_bounds__(RT_BLOCK) void route_rank_kernel(const int32_t* __restrict__ ids, const int32_t* __restrict__ block_counts,
                                                              int64_t* __restrict__ group_list,
                                                              int32_t* __restrict__ row_token, int32_t* __restrict__ row_of_choice,
                                                              int64_t n, int E, int topk, int nblocks, int prefixed) {
    extern __shared__ int rank_lds[];
    int* scan = rank_lds;            // [E] inclusive scan of the experts' totals
    int* base = scan + E;            // [E] first sorted row of this block's choices of expert e
    int* wh = base + E;              // [16][E] choices of expert e in wavefront w -> in the wavefronts before w
    const int e = threadIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int blk = blockIdx.x;
    int total = 0, before = 0;
    if (e < E && prefixed) {
        before = block_counts[(int64_t)blk * E + e];
        total = block_counts[(int64_t)nblocks * E + e];
        scan[e] = total;
    } else if (e < E) {
        // independent loads, 4 blocks at a time
        int b = 0;
        for (; b + 4 <= nblocks; b += 4) {
            const int c0 = block_counts[(int64_t)b * E + e], c1 = block_counts[(int64_t)(b + 1) * E + e];
            const int c2 = block_counts[(int64_t)(b + 2) * E + e], c3 = block_counts[(int64_t)(b + 3) * E + e];
            total += c0 + c1 + c2 + c3;
            before += (b < blk ? c0 : 0) + (b + 1 < blk ? c1 : 0) + (b + 2 < blk ? c2 : 0) + (b + 3 < blk ? c3 : 0);
        }
        for (; b < nblocks; ++b) {
            const int c = block_counts[(int64_t)b * E + e];
            total += c;
            before += b < blk ? c : 0;
        }
        scan[e] = total;
    }
    for (int j = threadIdx.x; j < 16 * E; j += RT_BLOCK) wh[j] = 0;
    __syncthreads();
    // inclusive scan over experts (Hillis-Steele)
    for (int off = 1; off < E; off <<= 1) {
        const int add = (e < E && e >= off) ? scan[e - off] : 0;
        __syncthreads();
        if (e < E) scan[e] += add;
        __syncthreads();
    }
    if (e < E) {
        base[e] = scan[e] - total + before;
        if (blk == 0) group_list[e] = scan[e];
    }
    const int64_t i = (int64_t)blk * RT_BLOCK + threadIdx.x;
    const int my = i < n ? ids[i] : -1;
    const bool valid = (unsigned)my < (unsigned)E;   // ids outside [0, E) are dropped
    if (valid) atomicAdd(&wh[wave * E + my], 1);
    __syncthreads();
    if (e < E) {
        int run = 0;
#pragma unroll
        for (int w = 0; w < 16; ++w) {
            const int t = wh[w * E + e];
            wh[w * E + e] = run;
            run += t;
        }
    }
    // equal ids in the lanes below this one
    int lower = 0;
    for (int k = 0; k < 63; ++k) {
        const int ek = __builtin_amdgcn_readlane(my, k);
        lower += (ek == my && k < lane) ? 1 : 0;
    }
    __syncthreads();
    if (i >= n) return;
    if (!valid) {
        row_of_choice[i] = -1;
        return;
    }
    const int dst = base[my] + wh[wave * E + my] + lower;
    row_token[dst] = (int32_t)(i / topk);
    row_of_choice[i] = dst;
}

// x rows copied into sorted order, token by token: a workgroup reads one token's row once (16 bytes per
// thread and load, 4 loads in flight) and writes it to the sorted row of each of its choices.  Dropped
// choices (row_of_choice < 0) write nothing, so the rows past group_list[E - 1] stay untouched.
__global__ __launch_bounds__(256) void route_scatter_kernel(const u32x4_t* __restrict__ x, const int32_t* __restrict__ row_of_choice,
                                                            u32x4_t* __restrict__ x_sorted, int topk, int units) {
    const int t = blockIdx.x;
    const u32x4_t* src = x + (int64_t)t * units;
    const int32_t* roc = row_of_choice + (int64_t)t * topk;
    for (int u0 = threadIdx.x; u0 < units; u0 += 4 * 256) {
        u32x4_t v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (u0 + 256 * j < units) v[j] = src[u0 + 256 * j];
        for (int c = 0; c < topk; ++c) {
            const int r = __builtin_amdgcn_readfirstlane(roc[c]);
            if (r < 0) continue;
            u32x4_t* dst = x_sorted + (int64_t)r * units;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (u0 + 256 * j < units) __builtin_nontemporal_store(v[j], dst + u0 + 256 * j);
        }
    }
}

size_t route_workspace_bytes(const moe_route_args* a) {
    const int64_t n = a->T * a->topk;
    const int64_t nblocks = (n + RT_BLOCK - 1) / RT_BLOCK;
    return (size_t)((nblocks + 1) * a->E) * sizeof(int32_t);   // per-block counts, and a row of totals
}

// Scratch of moe_route_static: the per-block counts (and the row of totals) live in this array instead of a
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
    if (a->logits && a->T > 0) {
        const dim3 grid((unsigned)((a->T + 3) / 4));
        const float* lg = static_cast<const float*>(a->logits);
        float* tw = static_cast<float*>(a->topk_weight);
        const int T = (int)a->T, E = (int)a->E, topk = (int)a->topk;
        if (E <= 64) hipLaunchKernelGGL(route_topk_kernel<1>, grid, dim3(256), 0, stream, lg, tw, ids, T, E, topk);
        else if (E <= 128) hipLaunchKernelGGL(route_topk_kernel<2>, grid, dim3(256), 0, stream, lg, tw, ids, T, E, topk);
        else if (E <= 256) hipLaunchKernelGGL(route_topk_kernel<4>, grid, dim3(256), 0, stream, lg, tw, ids, T, E, topk);
        else if (E <= 512) hipLaunchKernelGGL(route_topk_kernel<8>, grid, dim3(256), 0, stream, lg, tw, ids, T, E, topk);
        else hipLaunchKernelGGL(route_topk_kernel<RT_MAX_PER_LANE>, grid, dim3(256), 0, stream, lg, tw, ids, T, E, topk);
        if (hipGetLastError() != hipSuccess) return MOE_ERR_LAUNCH;
    }
    if (nblocks > 0)
        hipLaunchKernelGGL(route_count_kernel, dim3((unsigned)nblocks), dim3(RT_BLOCK), 0, stream, ids, counts, n, (int)a->E);
    const int prefixed = nblocks > RT_FUSED_SCAN_MAX_BLOCKS ? 1 : 0;
    if (prefixed)
        hipLaunchKernelGGL(route_scan_kernel, dim3((unsigned)((a->E + 3) / 4)), dim3(256), 0, stream, counts, (int)a->E, nblocks);
    // one block even without choices: it writes group_list (all zeros then)
    const size_t lds = (size_t)18 * a->E * sizeof(int);
    static std::atomic<uint64_t> lds_set{0};
    if (const int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(&route_rank_kernel), 18 * RT_MAX_E * (int)sizeof(int), lds_set))
        return rc;
    hipLaunchKernelGGL(route_rank_kernel, dim3((unsigned)(nblocks > 0 ? nblocks : 1)), dim3(RT_BLOCK), lds, stream, ids, counts,
                       static_cast<int64_t*>(a->group_list), static_cast<int32_t*>(a->row_token),
                       static_cast<int32_t*>(a->row_of_choice), n, (int)a->E, (int)a->topk, nblocks, prefixed);
    if (hipGetLastError() != hipSuccess) return MOE_ERR_LAUNCH;
    if (a->x && n > 0) {
        hipLaunchKernelGGL(route_scatter_kernel, dim3((unsigned)a->T), dim3(256), 0, stream,
                           static_cast<const u32x4_t*>(a->x), static_cast<const int32_t*>(a->row_of_choice),
                           static_cast<u32x4_t*>(a->x_sorted), (int)a->topk, (int)(a->K / 8));
        if (hipGetLastError() != hipSuccess) return MOE_ERR_LAUNCH;
    }
    return MOE_OK;
}

}  // namespace moe
