// Grouped GEMM with weight antiquant for MoE prefill on gfx950.
//
//   y[rows of expert g, :] = x[rows of expert g, :] . dequant(W[g])     bf16 x bf16 -> fp32 -> bf16
//
// Replaces grouped_matmul_antiquant (grouped_gemm/op_kernel/grouped_matmul_antiquant.h:225-364,
// grouped_matmul.h:147-463).  The reference decodes each weight slab to a bf16 copy in
// global memory and then runs a bf16 matmul on it; here the packed weights are decoded
// in registers straight into bf16 MFMA fragments and never go back to HBM.
//
// Work decomposition.  A tile is (expert, chunk of rows, 256 columns).  The tile list is derived
// inside the kernel from the device-resident cumulative group_list (no host sync); a persistent
// grid walks it with an XCD-aware order so that the workgroups of one XCD share the x rows and
// weight slices of the same experts in that XCD's L2, and takes the last two or three tiles of every
// workgroup from a work counter (see tile_queue).  Every wavefront owns its columns for ALL
// rows of the tile, so each weight element is dequantized exactly once per tile.  Two tile routines:
//   gemm_tile_pair  every quantized container (int4, int8, the K-contiguous fp4 containers, the
//                   reference's fp4 and fp8); x, packed weights and scales arrive by LDS-direct loads into a
//                   ring of stages walked by an unrolled k loop.  Either 8 wavefronts, the two of a SIMD
//                   splitting the k range (int8, fp8, K-contiguous fp4), or 4 wavefronts that each take their
//                   64 columns through all of k, two such workgroups per CU (int4 and fp4 prefill);
//                   tiles of up to 160 rows, or of up to 32 / 16 rows with small stages (decode batches,
//                   and the GEMV op's arithmetic on the N-contiguous containers)
//   gemm_tile       the bf16 container: 4 wavefronts of 64 columns, x through a double-buffered,
//                   XOR-swizzled LDS tile, weights from registers; tiles of up to 176 rows, or 32 rows
//                   and several workgroups per CU for decode-sized batches
//
// MFMA: v_mfma_f32_16x16x32_bf16.  Lane l = 16*q + i holds, for A, row i and
// k = 8q..8q+7 of the 16x32 block; for B, column i and the same k; for the result,
// column i and rows 4q..4q+3.  The contraction index may be permuted freely as long
// as A and B agree, and so may the column <-> (MFMA, lane) assignment; each weight
// container picks the assignment that makes its global loads wide and contiguous.
#include <type_traits>

#include "moe_device.h"
#include "moe_internal.h"

namespace moe {

constexpr int GM_BN = 256;     // columns per workgroup
constexpr int GM_MT_MAX = 12;  // 16-row blocks per tile the LDS buffers are sized for (192 rows)
constexpr int GM_THREADS = 256;
constexpr int GM_SKINNY_BLOCKS = 2;  // decode kernel: tiles of at most 32 rows ...
constexpr int GM_SKINNY_WAVES = 3;   // ... and at least this many wavefronts per SIMD

struct GemmParams {
    const uint16_t* x;
    const uint8_t* w;
    const void* scale;
    const uint16_t* offset;
    const int64_t* gl;
    uint16_t* y;
    int64_t M;
    int K, N, G, scale_rows;
    int epilogue;   // moe_epilogue
    int slot;       // this launch's counter in tile_queue; -1: none, every tile in the fixed order
    unsigned long long stamp;   // what this launch raises its counter to before it draws from it
    // what the scheduler keeps in LDS: 2 the first tile of every expert and the experts' clamped row bounds; 1 the
    // first tiles only (the row bounds are read from group_list per tile); 0 neither fits: the first tile of every
    // thread's run of experts only, and a tile is found by walking its run (any number of experts)
    int table_mode;
    // N-contiguous 4-bit containers: the multiplier that turns a 32-k sub-step index into its scale row, i.e.
    // divides by the sub-steps per scale group (0: identity)
    uint32_t sub_to_group;
};

// Work queue of the persistent grid.  Workgroups do not run at one speed (of two that share a CU the one
// placed first runs about 1.5 times as fast as the other while both are resident, and the XCDs differ by a few
// per cent), so an even split of the tiles leaves most of the chip waiting for the slowest workgroup.  All but
// the last two or three tiles of a workgroup's share are handed out in a fixed, XCD-aware order; the rest
// (the tail) are taken one at a time, front to back, from a counter in the library's device memory.  (One
// counter per XCD, each for a run of its own or for every eighth chunk of the tail, and stealing between them
// at the end, kept more of the tail's reads in the XCDs' L2s but was 1.5 - 2 % slower on the prefill shapes and
// 5 % on the weight-streaming decode shapes.)
//
// A launch owns one slot = one 64-bit counter.  The host numbers the launches (64 bits, never reused); launch L
// uses slot L % GM_QUEUE_SLOTS and the stamp (L / GM_QUEUE_SLOTS + 1) << GM_QUEUE_COUNT_BITS, which grows with
// every use of the slot.  The first workgroups raise the counter to the stamp when they start (atomic max, fire and
// forget, one tile's time before anybody's first draw); a draw is a fetch-and-add, and the value it returns minus
// the stamp is the ticket.  Whatever an earlier launch left in the slot is smaller than the stamp and simply disappears, so
// nothing has to be cleared at the end of a kernel and no state a kernel leaves behind can mislead a later one.
// A launch that only starts after a later launch has taken its slot (its stream was held back for
// GM_QUEUE_SLOTS launches) sees that from the counter, which every workgroup reads once when it starts, and never draws:
// it walks all of its tiles in the fixed order and disturbs nobody.  A draw that returns a value outside
// [stamp, stamp + 2^GM_QUEUE_COUNT_BITS) means that the slot was taken over while this launch was running: the
// workgroup then walks its share of the tail in the fixed order -- tiles that were already handed out get
// computed twice, which only rewrites the same values -- but its stray draws have cost the later launch
// tickets, i.e. tiles: a launch that is still running when the GM_QUEUE_SLOTS-th launch after it starts is
// the one thing callers must not arrange.  A launch that is being captured into a HIP graph gets no slot at
// all (slot -1): its kernel node would keep slot and stamp for every replay while the ring moves on, so it
// walks all of its tiles in the fixed order.
constexpr int GM_QUEUE_SLOTS = 4096;
constexpr int GM_QUEUE_STRIDE = 8;        // 64-bit words per slot: a cache line of its own
constexpr int GM_QUEUE_TAIL_SWEEPS = 2;   // tiles per workgroup that are left to the counter (plus the remainder)
constexpr unsigned GM_QUEUE_COUNT_BITS = 24;
typedef unsigned long long queue_word_t;
__device__ queue_word_t tile_queue[GM_QUEUE_SLOTS * GM_QUEUE_STRIDE];
static std::atomic<uint64_t> queue_launches{0};   // launches of every kind of kernel in this file, for slot and stamp

// What a workgroup does with the launch's counter when it starts: it reads it (an ordinary load, issued ahead of the
// group_list loads and back with them) to see whether the slot is still this launch's, and the first 8 workgroups,
// one per XCD, raise it to the launch's stamp.  Not every workgroup: 512 atomics on one address at the start of a
// kernel held everybody's first loads up (tile table ready after 8 us instead of 2), and an atomic's own return
// value came back 2.5 us behind the loads.  A workgroup that draws before any of those stamps has arrived (it
// cannot be the usual case: draws start one tile into the kernel) gets a value below the stamp, takes it for a lost
// slot and does its share in the fixed order.
__device__ __forceinline__ bool queue_open(queue_word_t* q, queue_word_t stamp, bool stamps) {
    const queue_word_t now = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (stamps) (void)__hip_atomic_fetch_max(q, stamp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return now < stamp + (1ull << GM_QUEUE_COUNT_BITS);   // else: a later launch holds the slot
}
// A draw adds 1 to the counter's low word only (the count never carries out of it) and gets that word back: one
// register in flight instead of two in the tile routines, which have none to spare.  The word still shows the
// low 32 - GM_QUEUE_COUNT_BITS bits of the launch's use of the slot, enough to tell a slot that was taken over.
__device__ __forceinline__ unsigned queue_draw_raw(queue_word_t* q) {
    return __hip_atomic_fetch_add(reinterpret_cast<unsigned*>(q), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// The ticket in a counter's low word raw, for a launch with the given stamp; -1: the slot is not this launch's
__device__ __forceinline__ int queue_ticket_of_draw(unsigned raw, queue_word_t stamp) {
    const unsigned d = raw - (unsigned)stamp;
    return d < (1u << GM_QUEUE_COUNT_BITS) ? (int)d : -1;
}
__device__ __forceinline__ int queue_draw(queue_word_t* q, queue_word_t stamp) { return queue_ticket_of_draw(queue_draw_raw(q), stamp); }
// A tile routine that is handed a counter draws the workgroup's next ticket from it while it finishes its own
// tile (the counter's round trip, about 3 us under load, overlaps the tile's reduction and stores) and leaves
// the ticket in *out behind its last barrier.
struct Ticket {
    queue_word_t* counter;   // null: the caller draws the ticket itself
    int* out;
    int* arrivals;           // a word of LDS for the tile routine's arrival counter (see gemm_tile_pair)
};

// Buffer resources keep the addressing compact: one 128-bit descriptor in SGPRs per
// tensor slab, one 32-bit per-lane offset that is constant for the whole tile, and a
// wave-uniform (scalar) offset per load.  Reads beyond the slab return 0.
typedef __amdgpu_buffer_rsrc_t rsrc_t;
__device__ __forceinline__ rsrc_t make_rsrc(const void* p, int64_t bytes) {
    const uint32_t n = bytes > 0xffffffffLL ? 0xffffffffu : (uint32_t)bytes;
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, n, 0x00020000);
}
__device__ __forceinline__ uint32_t ldg_b32(rsrc_t r, int voff, int soff) {
    return __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0);
}
__device__ __forceinline__ u32x2_t ldg_b64(rsrc_t r, int voff, int soff) {
    return __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, 0);
}
__device__ __forceinline__ u32x4_t ldg_b128(rsrc_t r, int voff, int soff) {
    return __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0);
}

// D = A * B + D with the accumulator tied to AGPRs.  Written as inline asm because the
// compiler, given many live accumulators, stops accumulating in place and shuttles them
// through copies, which halves the MFMA rate.  Hazards: A/B come from VALU or waited
// loads (interlocked); accumulators are only read by other MFMAs until the epilogue,
// which waits out the MFMA latency first.
__device__ __forceinline__ void mfma_16x16x32(f32x4_t& acc, const u32x4_t& a, const u32x4_t& b) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}

// Same with the accumulator in ordinary VGPRs.  A kernel that uses no AGPRs at all may use
// the whole unified register file as VGPRs (otherwise the compiler splits it in two halves).
__device__ __forceinline__ void mfma_16x16x32_v(f32x4_t& acc, const u32x4_t& a, const u32x4_t& b) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b));
}

// silu(g) * u on fp32 accumulators: g / (1 + exp(-g)) with the hardware exp and reciprocal.
__device__ __forceinline__ float swiglu(float g, float u) {
    return g * __builtin_amdgcn_rcpf(1.f + __expf(-g)) * u;
}

// Ties a value to the chain of volatile asm statements (the MFMAs): whatever is computed
// from the returned value is emitted after every earlier volatile asm, whatever produced the
// argument before every later one.  Emits no instruction.  Used to pin each decode unit
// between two MFMAs; sched_barrier alone only constrains the machine scheduler, not the
// instruction order chosen at selection time.
template <typename V>
__device__ __forceinline__ V pinned(V v) {
    asm volatile("" : "+v"(v));
    return v;
}

// Per-lane view of one tile for the weight loaders.
struct BCtx {
    rsrc_t rw, rs;       // weight / scale slab of the expert
    int vw, vs;          // per-lane byte offsets into them (constant over the tile)
    int K, N, n0;
    int i, q, w;         // lane & 15, lane >> 4, wavefront (scalar)
};

// Each weight container provides
//   Raw        packed registers of one k step
//   load_sub   global loads of 32-k sub-step s of the step starting at k0
//   Dq         the decode, cut into units so that it can be interleaved with MFMAs:
//              prep(raw, c, s) once per sub-step, then unit(raw, c, s, p, t, out) for
//              p, t in [0,4) writes dword p (k pair) of the fragment of MFMA t
//   a_chunk    which 16-byte chunk of the x tile row matches the k values of (s, q)
//   col        output column (relative to n0) of MFMA t in this lane
template <int FMT>
struct BTraits;

// ------------------------------------------------------------------ bf16, [N, K]
// K-contiguous: lane (i, q) loads 32 contiguous bytes, k = k0 + 16q + [0,16); sub-step
// s uses the half k0 + 16q + 8s + [0,8), so the matching x chunk is 2q + s.
template <>
struct BTraits<MOE_FMT_BF16> {
    static constexpr int BK = 64, NS = 2;
    static constexpr int MT_MAX = 11;
    struct Raw {
        u32x4_t r[4][2];
    };
    __device__ static __forceinline__ int a_chunk(int s, int q) { return 2 * q + s; }
    __device__ static __forceinline__ int col(const BCtx& c, int t) { return 64 * c.w + 16 * t + c.i; }
    __device__ static __forceinline__ void init(BCtx& c) {
        c.vw = (64 * c.w + c.i) * c.K * 2 + 32 * c.q;
        c.vs = 0;
    }
    __device__ static __forceinline__ void load_sub(Raw& raw, const BCtx& c, int k0, int s) {
#pragma unroll
        for (int t = 0; t < 4; ++t) raw.r[t][s] = ldg_b128(c.rw, c.vw, ((c.n0 + 16 * t) * c.K + k0) * 2 + 16 * s);
    }
    struct Dq {
        __device__ __forceinline__ void init_tile(const BCtx&) {}
        __device__ __forceinline__ void prep(const Raw&, const BCtx&, int) {}
        __device__ __forceinline__ void unit(const Raw& raw, const BCtx&, int s, int p, int t, u32x4_t out[4]) {
            out[t][p] = pinned(raw.r[t][s][p]);
        }
    };
};

// ---------------------------------------------------------------------------------
// x tile: rows x BK bf16 in LDS, 16-byte chunks, chunk c of row r stored at
// position c ^ (r & 7) so that the 8 lanes a ds_read_b128 serves together hit
// distinct banks both when writing (consecutive chunks of one row) and when
// reading fragments (same chunk of 8 consecutive rows).
// ---------------------------------------------------------------------------------
template <int BK>
__device__ __forceinline__ int a_lds_unit(int row, int c) {
    return row * (BK / 8) + (c ^ (row & 7));
}

// The same for tile rows of 32 k (four 16-byte chunks, 64 bytes): chunk c of row r at position c ^ ((r >> 1) & 3).
// A 16-byte LDS read is served 8 lanes (128 bytes of banks) at a time: the 8 consecutive rows such a group reads the
// same chunk of then lie in 8 different 16-byte slots modulo 128 bytes (two rows share a 128-byte line; the pairs
// take the four positions in turn).  (With (r >> 2) & 3 in its place the counters showed two lanes per slot:
// SQ_LDS_BANK_CONFLICT at 39 % of the cycles the LDS was active.)
__device__ __forceinline__ int a_lds_unit32(int row, int c) {
    return row * 4 + (c ^ ((row >> 1) & 3));
}

// Per-tile context: lane coordinates and the buffer resources of expert g.
template <int FMT>
__device__ __forceinline__ void make_ctx(BCtx& c, const GemmParams& P, int g, int n0) {
    const int tid = threadIdx.x, lane = tid & 63;
    c.K = P.K; c.N = P.N; c.n0 = n0;
    c.i = lane & 15; c.q = lane >> 4; c.w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int64_t KN = (int64_t)P.K * P.N;
    static_assert(FMT == MOE_FMT_BF16, "the 4-wavefront tile routine serves the bf16 container");
    c.rw = make_rsrc(P.w + g * KN * 2, KN * 2);
    c.rs = c.rw;
}

// Epilogue: fp32 -> bf16 (RNE), rows beyond the chunk are dropped.
template <int FMT, int MT>
__device__ __forceinline__ void store_tile(const GemmParams& P, const BCtx& c, f32x4_t (&acc)[MT][4], int64_t row0, int rows,
                                           int n0) {
    using T = BTraits<FMT>;
    // through a buffer resource that ends after the tile's last valid row: stores to padded
    // rows fall outside it and are dropped (the containers of this routine are K-contiguous: a lane's
    // 4 accumulators of a row are 16 columns apart)
    if (P.epilogue == MOE_EPILOGUE_SWIGLU) {
        // weight rows in blocks of 32 = (16 gate rows, 16 up rows): MFMAs (0, 1) and (2, 3); y has N / 2 columns
        const int NO = P.N >> 1;
        const rsrc_t ro = make_rsrc(P.y + row0 * (int64_t)NO, (int64_t)rows * NO * 2);
        const int vo = (4 * c.q * NO + ((n0 + 64 * c.w) >> 1) + c.i) * 2;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int u = 0; u < 2; ++u)
                    __builtin_amdgcn_raw_buffer_store_b16(
                        (uint16_t)(pack_bf16_rne(swiglu(acc[mt][2 * u][r], acc[mt][2 * u + 1][r]), 0.f) & 0xffffu), ro,
                        vo + 32 * u, (16 * mt + r) * NO * 2, 0);
        return;
    }
    const rsrc_t ry = make_rsrc(P.y + row0 * (int64_t)P.N, (int64_t)rows * P.N * 2);
    const int vy = (4 * c.q * P.N + n0) * 2;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int so = (16 * mt + r) * P.N * 2;
#pragma unroll
            for (int t = 0; t < 4; ++t)
                __builtin_amdgcn_raw_buffer_store_b16((uint16_t)(pack_bf16_rne(acc[mt][t][r], 0.f) & 0xffffu), ry,
                                                      vy + T::col(c, t) * 2, so, 0);
        }
}

template <int FMT, int MT, int CAPB>
__device__ __forceinline__ void gemm_tile(const GemmParams& P, u32x4_t* lds_a, int g, int64_t row0, int rows, int n0) {
    using T = BTraits<FMT>;
    constexpr int BK = T::BK, NS = T::NS;
    constexpr int CPR = BK / 8;               // 16-byte chunks per tile row
    constexpr int RPP = GM_THREADS / CPR;     // rows loaded per pass
    constexpr int PASSES = (16 * MT + RPP - 1) / RPP;
    constexpr int ABUF = 16 * CAPB * CPR;  // units per buffer (CAPB row blocks)

    const int tid = threadIdx.x;
    BCtx c;
    make_ctx<FMT>(c, P, g, n0);
    T::init(c);
    typename T::Dq dq;
    dq.init_tile(c);

    // x rows of this tile through a buffer resource that ends after the last valid row:
    // padded rows read as zeros.  This thread loads chunk ac of rows ar + RPP*p.
    const int ar = tid / CPR, ac = tid % CPR;
    const rsrc_t rx = make_rsrc(P.x + row0 * (int64_t)P.K, (int64_t)rows * P.K * 2);
    const int vx = (ar * P.K + ac * 8) * 2;

    f32x4_t acc[MT][4];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[mt][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    u32x4_t areg[PASSES];
    typename T::Raw raw;
    const int nk = P.K / BK;

    // Every pass is done by all threads: rows past the tile read as zeros (they lie beyond the
    // buffer resource) and land in LDS rows that exist (the buffers hold 16 * CAPB rows)
    // but are never read.  No divergent branch, so the loop body stays one scheduling region.
    static_assert(PASSES * RPP <= 16 * CAPB, "x tile passes overrun the LDS buffer");
    auto load_a = [&](int kt) {
#pragma unroll
        for (int p = 0; p < PASSES; ++p) areg[p] = ldg_b128(rx, vx, (p * RPP * P.K + kt * BK) * 2);
    };
    auto store_a = [&](int buf) {
#pragma unroll
        for (int p = 0; p < PASSES; ++p) lds_a[buf * ABUF + a_lds_unit<BK>(ar + RPP * p, ac)] = areg[p];
    };

    // Software pipeline, one barrier per k step (BK = NS sub-steps of 32 k), every
    // instruction placed by hand (sched_barrier after each MFMA slot):
    //  * weights: while the MFMAs of sub-step f run, the fragments of sub-step f+1 are
    //    decoded, one unit (two elements of one column) at a time between MFMAs; as soon as
    //    a sub-step's packed registers have been decoded they are refilled with the same
    //    sub-step of the next k step, straight from global memory a full step ahead;
    //  * x: fragments come from LDS through a ring of 4 register sets, read RING
    //    fragments ahead of their MFMAs; the x tile of step kt+1 travels through registers
    //    into the other LDS buffer.
    // The last steps prefetch past K: buffer loads beyond a slab return 0 and the x rows
    // read are inside the tensor; neither is used.
    constexpr int RING = 3, F = NS * MT;
    constexpr int SLOTS = 4 * MT;   // MFMAs per sub-step
    constexpr int UNITS = 17;       // prep + 16 decode units per sub-step

    __syncthreads();  // previous tile's readers are done with both buffers
    load_a(0);
    store_a(0);
#pragma unroll
    for (int s = 0; s < NS; ++s) T::load_sub(raw, c, 0, s);
    u32x4_t bf[2][4];
    dq.prep(raw, c, 0);
#pragma unroll
    for (int p = 0; p < 4; ++p)
#pragma unroll
        for (int t = 0; t < 4; ++t) dq.unit(raw, c, 0, p, t, bf[0]);
    __syncthreads();
    // raw[0] <- sub-step 0 of step 1, a full step ahead
    T::load_sub(raw, c, BK, 0);

    // One k step.  The global loads of the next x tile are issued one per MFMA slot at the start
    // of the first sub-step, the LDS writes one per slot at the end of the last one, so that
    // neither sits between the barrier and the first MFMA or between the last MFMA and the barrier.
    constexpr int NW = PASSES;   // write slots: one per x pass
    static_assert(NW + 1 <= SLOTS, "not enough MFMA slots to spread the tile transfers over");
    auto step = [&](int kt) {
        const u32x4_t* la = lds_a + (kt & 1) * ABUF;
        u32x4_t afr[4];
        auto read_a = [&](int f) {
            afr[f & 3] = la[a_lds_unit<BK>(16 * (f % MT) + c.i, T::a_chunk(f / MT, c.q))];
        };
#pragma unroll
        for (int f = 0; f < (RING < F ? RING : F); ++f) read_a(f);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            const int sn = (s + 1) % NS;                 // sub-step being decoded
            u32x4_t* bcur = bf[s & 1];
            u32x4_t* bnxt = bf[(s + 1) & 1];
#pragma unroll
            for (int slot = 0; slot < SLOTS; ++slot) {
                const int mt = slot >> 2, t = slot & 3, f = s * MT + mt;
                if (t == 0 && f + RING < F) read_a(f + RING);
                mfma_16x16x32(acc[mt][t], afr[f & 3], bcur[t]);
                // fetch the x tile of step kt+1
                if (s == 0 && slot < PASSES) areg[slot] = ldg_b128(rx, vx, (slot * RPP * P.K + (kt + 1) * BK) * 2);
                // decode units u with floor(u * SLOTS / UNITS) == slot
#pragma unroll
                for (int u = (slot * UNITS + SLOTS - 1) / SLOTS; u < ((slot + 1) * UNITS + SLOTS - 1) / SLOTS; ++u) {
                    if (u == 0)
                        dq.prep(raw, c, sn);
                    else
                        dq.unit(raw, c, sn, (u - 1) >> 2, (u - 1) & 3, bnxt);
                }
                if (slot == ((UNITS - 1) * SLOTS) / UNITS) {
                    // everything of sub-step sn has been decoded: refill its registers
                    T::load_sub(raw, c, (kt + (sn == 0 ? 2 : 1)) * BK, sn);
                }
                if (s == NS - 1 && slot >= SLOTS - NW) {
                    const int wi = slot - (SLOTS - NW);
                    lds_a[((kt + 1) & 1) * ABUF + a_lds_unit<BK>(ar + RPP * wi, ac)] = areg[wi];
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        __syncthreads();
    };
    for (int kt = 0; kt < nk; ++kt) step(kt);
    // the accumulators were last written by MFMAs the compiler cannot see: wait out their latency
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");

    store_tile<FMT, MT>(P, c, acc, row0, rows, n0);
}

// ---------------------------------------------------------------------------------
// LDS-direct loads (buffer_load_dwordx4 ... lds): lane l of the wavefront writes bytes
// [16 l, 16 l + 16) after the instruction's LDS base.  No staging registers and no LDS store
// instructions, so a tile routine can keep a ring of stages filled several k steps (a few
// microseconds of HBM latency) ahead of their use.
// ---------------------------------------------------------------------------------
#define MOE_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
__device__ __forceinline__ void lds_load16(rsrc_t r, const u32x4_t* dst, int voff, int soff) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, MOE_LDS_PTR(const_cast<u32x4_t*>(dst)), 16, voff, soff, 0, 0);
}
// The same with the destination as a byte address in LDS (wave-uniform).
__device__ __forceinline__ uint32_t lds_address(const void* p) {
    return (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uintptr_t)MOE_LDS_PTR(p));
}
__device__ __forceinline__ void lds_load16_at(rsrc_t r, uint32_t dst, int voff, int soff) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (__attribute__((address_space(3))) void*)(uintptr_t)dst, 16, voff, soff, 0, 0);
}
// A wave-uniform value the compiler must take as it finds it: whatever is derived from the result is computed
// where it is used instead of once per variant ahead of an unrolled loop (where it would occupy an SGPR each).
__device__ __forceinline__ uint32_t here(uint32_t v) {
    asm volatile("" : "+s"(v));
    return v;
}

// ---------------------------------------------------------------------------------
// Tile routine for the quantized containers (int4, int8, reference fp4 / fp8, K-contiguous fp4) with two
// wavefronts per SIMD that split the k range.  Described for int4; what differs for the others follows.
//
// A single wavefront issues at most one instruction every ~5 cycles whatever its kind, and an
// MFMA holds the SIMD's vector issue port for about 8 of its 16 cycles: with one wavefront
// per SIMD the decode instructions and the MFMAs of a k step add up instead of overlapping.
// Here the workgroup has 8 wavefronts.  Wavefront wv owns the 64 columns of group wv & 3 for
// all rows of the tile (4 MFMAs per x fragment), but only one of the two 32-k sub-steps of
// every 64-k step: the pair (wv, wv + 4) shares a SIMD and accumulates two partial sums that
// are added once per tile through LDS.  Every weight element is still decoded exactly once
// per tile, a lane decodes 4 nibbles of a dword at a time (2.5 VALU instructions per
// element), and each wavefront reads half of the x fragments.
//
// Each wavefront alternates a decode phase (its sub-step of the packed stage -> 4 bf16 B
// fragments in registers) and an MFMA phase; one wavefront of a SIMD multiplies while the other
// decodes.  The steps of the 8 wavefronts are tied together by a split barrier, an arrival counter
// in LDS (see ring_arrive / ring_wait in gemm_tile_pair): a wavefront that is done with a step says
// so and goes on decoding the next one; it waits for the others only in front of its next MFMA phase.
//
// Everything the k loop consumes -- x tile, packed weight tile, scales -- is brought in by
// LDS-direct loads into a ring of S = 5 stages.  The loads of stage kt+4 (it replaces stage kt-1,
// which every wavefront has left when all have arrived kt times) and the LDS reads of the packed
// dwords of stage kt+1 are spread between the MFMAs of step kt; before it arrives at the end of step
// kt each wavefront waits until its own loads of stage kt+2 have landed.  vmcnt counts a wavefront's loads in order and every
// wavefront issues the same number NI of them per step (waves without a row block of their
// own repeat one: measured, the repeated loads cost nothing, a branch around them does), so "at most
// (S - 3) NI outstanding" means exactly that.
//
// Decode of a k-row pair (a, b) of one dword column: v_perm gathers the two bytes of each row
// this lane owns, the low nibbles (& 0x0f0f0f0f) and high nibbles (>> 4 & 0x0f0f0f0f) are bytes
// 0x00..0x0f, which read as OCP e4m3 are exactly q / 512 -- v_cvt_pk_f32_fp8 converts two at
// once -- and one fma per element applies 512 * scale and the zero point:
// q s - 8 s = (q - 8) s exactly.
//
// The same routine serves the reference's pre-shuffled fp4 container: its 64 x 128-byte tile is
// brought in by the same loads, a lane's 8 k rows of its 2 bytes are two 16-byte LDS reads, each
// byte pair decodes to 4 floats with v_cvt_scalef32_pk_f32_fp4 and takes one multiply by the
// column's scale of that 16-k block (4 scale rows per step instead of 2).
//
// int8 and the reference fp8 container: a step's tile is 64 rows of 256 bytes (two load instructions
// per wavefront), which leaves room for S = 4 stages; a lane's 4 columns are one dword of each of its 8 k
// rows.  int8 keeps its per-channel scale and offset in registers (and folds them into one fma where that gives
// the bits of the two rounded operations, see i8_one_rounding); fp8 decodes two codes at a time through
// fp16 (see e4m3_ref_pair_over_256_fp16) and gets the fp32 scale of its 128 x 128 block through the ring,
// 4 bytes per wavefront and step.
//
// K-contiguous fp4 (weight [N, K/2]): a step's tile is 256 weight rows x 32 bytes; MFMA t of a lane takes
// weight row 64 cw + 16 t + i, whose 8 codes of the sub-step are one dword; the scales [N, K/block] are
// fetched 16 bytes per row at a time into buffers of their own (see kc_issue_scale).
// ---------------------------------------------------------------------------------
// Kernel variants.
//   GK_GENERAL  4 wavefronts of 64 columns, one workgroup per CU, tiles of up to 176 rows (bf16 only)
//   GK_SKINNY   the same tile routine with tiles of at most 32 rows and several workgroups per CU
//               (decode-sized batches are HBM bound: more weight bytes in flight)
//   GK_PAIR     quantized containers: 8 wavefronts, k range split between the two wavefronts of a SIMD, tiles of
//               up to 160 rows
//   GK_PAIR_SMALL  GK_PAIR with tiles of at most 32 rows: x stages of 4 KB leave LDS for a second workgroup per
//               CU (decode-sized batches on the 4-bit containers)
//   GK_PAIR_EXACT  GK_PAIR_SMALL with the GEMV op's arithmetic (weights not rounded to bf16)
//   GK_PAIR_EXACT16  GK_PAIR_EXACT with tiles of at most 16 rows (the fp4 container: its 32-row tile routine
//               needs 153 registers, the 16-row one 97, which lets two workgroups share a CU)
//   GK_QUAD     the large tiles of GK_PAIR without the k split: workgroups of 4 wavefronts, each wavefront takes its
//               64 columns through the whole k range in steps of 32 k, two workgroups per CU.  The two wavefronts
//               of a SIMD belong to different workgroups and work on different tiles: no partial sums to
//               exchange, a barrier spans 4 wavefronts instead of 8, and while one workgroup is between two tiles
//               (stores, tile search, first loads) the other has the SIMDs to itself.  (The N-contiguous containers.)
enum { GK_GENERAL = 0, GK_SKINNY = 1, GK_PAIR = 2, GK_PAIR_EXACT = 3, GK_PAIR_SMALL = 4, GK_PAIR_EXACT16 = 5, GK_QUAD = 6 };
constexpr bool pair_exact(int kind) { return kind == GK_PAIR_EXACT || kind == GK_PAIR_EXACT16; }
constexpr int pair_waves(int kind) { return kind == GK_QUAD ? 4 : 8; }
constexpr int pair_bk(int kind) { return kind == GK_QUAD ? 32 : 64; }   // k per step

constexpr int PAIR_CAPB = 10;                         // x stages hold 160 rows
constexpr int PAIR_MT_MAX = 10;
constexpr int PAIR_SMALL_MT_MAX = 2;                  // row blocks per tile of the small-stage kinds
constexpr bool pair_small(int kind) { return kind != GK_PAIR && kind != GK_QUAD; }
// 16-byte units of one x stage: 160 rows, or the 32 rows of the small-stage kinds
constexpr int pair_mt_max(int kind) { return !pair_small(kind) ? PAIR_MT_MAX : kind == GK_PAIR_EXACT16 ? 1 : PAIR_SMALL_MT_MAX; }
constexpr int pair_a_units(int kind) { return 16 * (pair_small(kind) ? pair_mt_max(kind) : PAIR_CAPB) * (pair_bk(kind) / 8); }
// packed tile of one k step: rows of 128 bytes (4-bit codes) or of 256 bytes (int8, fp8)
template <int FMT>
constexpr int pair_b_units(int kind) { return pair_bk(kind) * ((FMT == MOE_FMT_INT8 || FMT == MOE_FMT_FP8_REF) ? 16 : 8); }
// Small-stage kinds on the 4-bit N-contiguous containers: two workgroups per CU, one computes while the other
// waits at its barrier or between two tiles (512 rows over 256 experts of 7168 x 2048: int4 425 -> 387 us, fp4
// 440 -> 425 us; the fp4 tile routine with the GEMV op's arithmetic fits four wavefronts per SIMD only in its
// 16-row form).  A deeper ring in the LDS the small x stages free does not pay instead (fp4 10 stages
// 515 us against 510 us with 5; fp8 7 stages 572 us against 552 us with 4: a tile's first stages take longer
// to fill), and the one-byte containers at two workgroups per CU are left with 3 stages (fp8 641 us).
template <int FMT>
constexpr int pair_wg_per_cu(int kind) {
    if (kind == GK_QUAD) return 2;
    if (!pair_small(kind)) return 1;
    return (FMT == MOE_FMT_INT4 || (FMT == MOE_FMT_FP4_REF && kind != GK_PAIR_EXACT)) ? 2 : 1;
}
// ring depth: what fits into LDS next to the 160-row x stages; the 4-wavefront kind runs best with 4 stages (a tile's
// first stages are filled sooner: int4 1790 against 1818 us at K = 7168, 949 against 952 us at K = 2048)
template <int FMT>
constexpr int pair_stages(int kind) { return (FMT == MOE_FMT_INT8 || FMT == MOE_FMT_FP8_REF || kind == GK_QUAD) ? 4 : 5; }
// 16-byte units of scales per k step: rows of 256 bf16, int4 one per 32-k sub-step (groups are multiples
// of 32), the reference fp4 container one per 16 k; fp8 one unit per wavefront holding the fp32 scale of
// its 128 x 128 block; int8 none (per-channel scales stay in registers)
template <int FMT>
constexpr int pair_sc_units(int kind) {
    return (FMT == MOE_FMT_FP4_REF ? 128 : FMT == MOE_FMT_INT4 ? 64 : FMT == MOE_FMT_FP8_REF ? 8 : 0) * pair_bk(kind) / 64;
}
// The K-contiguous fp4 containers keep their scales [N, K/block] outside the stages: 16 bytes (2 or 4 steps'
// worth) per weight row at a time, three buffers of 256 rows
template <int FMT>
constexpr int pair_kc_scale_units() { return (FMT == MOE_FMT_FP4_B32 || FMT == MOE_FMT_FP4_B16) ? 3 * 256 : 0; }
template <int FMT>
constexpr int pair_lds_units(int kind) {
    return pair_stages<FMT>(kind) * (pair_a_units(kind) + pair_b_units<FMT>(kind) + pair_sc_units<FMT>(kind)) + pair_kc_scale_units<FMT>();
}

// End of a k-split tile.  The two wavefronts of a pair (same columns, the two k halves) hold partial sums of the
// whole tile; each hands the row blocks the other will finish to it through LDS, adds what it receives to the
// row blocks it keeps and stores those: the first half of the tile's 16-row blocks is finished by the h == 0
// wavefront, the second by h == 1, so both reduce and store at the same time.  Rounds of at most 4 row
// blocks (8 wavefronts x 4 blocks x 4 KB fit the x stage area, free now).
// WHOLE: the wavefront holds the whole sums (no k split): it stores all of its row blocks, nothing is exchanged.
template <int MT, bool KC, bool WHOLE = false>
__device__ __forceinline__ void pair_finish(const GemmParams& P, u32x4_t* smem, f32x4_t (&acc)[MT][4], int h, int cw, int lane,
                                            int col0, int64_t row0, int rows, int n0, const Ticket& tk) {
    const int i = lane & 15, q = lane >> 4;
    const bool takes = tk.counter != nullptr && threadIdx.x == 0;
    unsigned next_tile = 0;
    if (takes) next_tile = queue_draw_raw(tk.counter);
    constexpr int MH = (MT + 1) / 2, RR = MH < 4 ? MH : 4, ROUNDS = (MH + RR - 1) / RR;
    // the last tile of an N that is not a multiple of 256 (the reference's fp8 container: multiples of 128)
    // computes columns past N from whatever follows in the slab: they are not stored
    const bool live = KC || n0 + col0 < P.N;
    const bool swi = P.epilogue == MOE_EPILOGUE_SWIGLU;
    // stores go through a buffer resource that ends after the tile's last valid row: those to padded rows
    // fall outside it and are dropped
    const int NO = swi ? P.N >> 1 : P.N;
    const rsrc_t ry = make_rsrc(P.y + row0 * (int64_t)NO, (int64_t)rows * NO * 2);
    auto store_block = [&](int mt) {
        if (!live) return;
        if (swi && KC) {
            // K-contiguous containers: the weight rows come in blocks of 32 = (16 gate rows, 16 up rows), which are
            // the MFMAs t = (0, 1) and (2, 3) of this lane; y has N / 2 columns
            const int vo = (4 * q * NO + ((n0 + 64 * cw) >> 1) + i) * 2;
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int u = 0; u < 2; ++u)
                    __builtin_amdgcn_raw_buffer_store_b16(
                        (uint16_t)(pack_bf16_rne(swiglu(acc[mt][2 * u][r], acc[mt][2 * u + 1][r]), 0.f) & 0xffffu), ry,
                        vo + 32 * u, (16 * mt + r) * NO * 2, 0);
        } else if (swi) {
            // this lane's 4 columns are (gate, gate, up, up) of 2 output columns; y has N / 2 columns
            const int vo = (4 * q * NO + ((n0 + col0) >> 1)) * 2;
#pragma unroll
            for (int r = 0; r < 4; ++r)
                __builtin_amdgcn_raw_buffer_store_b32(
                    pack_bf16_rne(swiglu(acc[mt][0][r], acc[mt][2][r]), swiglu(acc[mt][1][r], acc[mt][3][r])), ry, vo,
                    (16 * mt + r) * NO * 2, 0);
        } else if (KC) {
            // K-contiguous containers: MFMA t holds column 64 cw + 16 t + i, one 2-byte store each
            const int vy = (4 * q * P.N + n0 + 64 * cw + i) * 2;
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    __builtin_amdgcn_raw_buffer_store_b16((uint16_t)(pack_bf16_rne(acc[mt][t][r], 0.f) & 0xffffu), ry,
                                                          vy + 32 * t, (16 * mt + r) * P.N * 2, 0);
        } else {
            const int vy = (4 * q * P.N + n0 + col0) * 2;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                u32x2_t v;
                v[0] = pack_bf16_rne(acc[mt][0][r], acc[mt][1][r]);
                v[1] = pack_bf16_rne(acc[mt][2][r], acc[mt][3][r]);
                __builtin_amdgcn_raw_buffer_store_b64(v, ry, vy, (16 * mt + r) * P.N * 2, 0);
            }
        }
    };
    // Barrier between the LDS writes and reads of the exchange: it orders LDS traffic only.  (__syncthreads
    // would also wait for this wavefront's global stores of the previous round to complete, 2-3 us each time.)
    auto lds_barrier = []() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
    // H: which half this wavefront finishes (a compile-time constant in each branch, so that every register
    // index is one); both kinds of wavefront take the same barriers
    auto finish = [&](auto HC) __attribute__((always_inline)) {
        constexpr int H = decltype(HC)::value;
        constexpr int KEEP0 = H == 0 ? 0 : MH, KEEPN = H == 0 ? MH : MT - MH;
        constexpr int SEND0 = H == 0 ? MH : 0, SENDN = MT - KEEPN;
        u32x4_t* out_slot = smem + (cw * 2 + (1 - H)) * (RR * 4 * 64) + lane;
        const u32x4_t* in_slot = smem + (cw * 2 + H) * (RR * 4 * 64) + lane;
#pragma unroll
        for (int rd = 0; rd < ROUNDS; ++rd) {
            if (rd > 0) lds_barrier();   // the previous round's slots are read
#pragma unroll
            for (int b = rd * RR; b < (rd + 1) * RR && b < SENDN; ++b)
#pragma unroll
                for (int t = 0; t < 4; ++t) out_slot[((b - rd * RR) * 4 + t) * 64] = __builtin_bit_cast(u32x4_t, acc[SEND0 + b][t]);
            lds_barrier();
#pragma unroll
            for (int b = rd * RR; b < (rd + 1) * RR && b < KEEPN; ++b) {
#pragma unroll
                for (int t = 0; t < 4; ++t) acc[KEEP0 + b][t] += __builtin_bit_cast(f32x4_t, in_slot[((b - rd * RR) * 4 + t) * 64]);
                store_block(KEEP0 + b);
            }
        }
    };
    if constexpr (WHOLE) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) store_block(mt);
    } else if (h == 0) {
        finish(std::integral_constant<int, 0>{});
    } else {
        finish(std::integral_constant<int, 1>{});
    }
    if (takes) *tk.out = queue_ticket_of_draw(next_tile, P.stamp);
    lds_barrier();   // the slots are read: the next tile may load into the ring (the stores are still in flight)
}

// EXACT selects the arithmetic of the GEMV op (grouped_soft_gemv/op_kernel/gemv_impl.h:147-199: the
// dequantized weights stay fp32): the B fragments then hold the codes themselves, which are exact in
// bf16, every MFMA covers k of one scale group only and its result is multiplied by that group's fp32
// scale on the way into the accumulators.  The fp4 container has a scale per 16 k, half an MFMA: the x
// fragment is split into its lanes q < 2 and q >= 2 (the other half zeroed) and each half takes its
// own MFMA.  These MFMAs are compiler-visible builtins (their results feed ordinary VALU code).
//
// STACK2 (that arithmetic on the fp4 container, tiles of at most 8 rows): the two scale groups of an MFMA's 32 k
// are told apart by the row of the 16 x 16 product instead of by two MFMAs.  Row r < 8 of the x fragment holds
// x row r in its first 16 k and zeros in the others, row 8 + r holds x row r in the last 16 k only (the zeros are
// read from the rows 8..15 of the x stage, which are padding for such a tile).  One MFMA per 16 columns then
// leaves the first group's sums in the lanes q < 2 and the second group's in q >= 2, each lane applies the
// scale of its own group, and the two halves are added once at the end of the tile: half the MFMAs and half
// the multiplies of the general case, and no masking.
template <int FMT, int MT, int KIND, bool STACK2 = false>
__device__ __forceinline__ void gemm_tile_pair(const GemmParams& P, u32x4_t* smem, int g, int64_t row0, int rows, int n0, const Ticket& tk) {
    static_assert(FMT != MOE_FMT_BF16, "the k-split tile routine decodes quantized containers");
    constexpr bool EXACT = pair_exact(KIND);
    static_assert(!STACK2 || (EXACT && FMT == MOE_FMT_FP4_REF && MT == 1), "two scale groups stacked in one MFMA: fp4, at most 8 rows");
    static_assert(!EXACT || FMT == MOE_FMT_INT4 || FMT == MOE_FMT_FP4_REF || FMT == MOE_FMT_FP8_REF,
                  "un-rounded weights: the N-contiguous containers of the GEMV op");
    constexpr bool FP4 = FMT == MOE_FMT_FP4_REF, I8 = FMT == MOE_FMT_INT8, F8 = FMT == MOE_FMT_FP8_REF;
    // K-contiguous fp4 (weight [N, K/2], scales [N, K/KBLK]): the step's tile is 256 weight rows x 32 bytes
    constexpr bool KC = FMT == MOE_FMT_FP4_B32 || FMT == MOE_FMT_FP4_B16;
    constexpr int KBLK = FMT == MOE_FMT_FP4_B32 ? 32 : 16;
    constexpr bool B8 = I8 || F8;   // one byte per weight: tiles of 64 rows x 256 bytes
    // Q4: the kind without the k split (GK_QUAD): 4 wavefronts, steps of 32 k, every wavefront in every step
    constexpr bool Q4 = KIND == GK_QUAD;
    static_assert(!Q4 || FMT == MOE_FMT_INT4 || FMT == MOE_FMT_INT8 || FMT == MOE_FMT_FP4_REF || FMT == MOE_FMT_FP8_REF,
                  "the 4-wavefront kind serves the N-contiguous containers");
    constexpr int NW = pair_waves(KIND);
    constexpr int BK = pair_bk(KIND), S = pair_stages<FMT>(KIND), PAIR_SC_UNITS = pair_sc_units<FMT>(KIND);
    constexpr int PAIR_B_UNITS = pair_b_units<FMT>(KIND);
    constexpr int AHEAD = S - 1;   // a step's loads fill the stage of step kt + AHEAD
    // Kinds of which two workgroups share a CU (decode batches, HBM bound) keep one s_barrier per step, placed so
    // that the two wavefronts of a SIMD alternate (those of sub-step 0 take it after their MFMA phase, those of
    // sub-step 1 half way through their decode); with one workgroup per CU the split barrier described below is
    // faster (measured on 512 rows over 256 experts of 7168 x 2048: two per CU 335 against 340 us (int4), 390 against
    // 395 us (fp4) with the plain barrier; one per CU, fp8, 555 against 580 us with the split one).
    constexpr bool SPLIT_BARRIER = pair_wg_per_cu<FMT>(KIND) == 1;
    constexpr int PAIR_A_UNITS = pair_a_units(KIND);
    static_assert(16 * MT * (BK / 8) <= PAIR_A_UNITS, "tile rows beyond the x stage");
    u32x4_t* lds_a = smem;
    u32x4_t* lds_b = lds_a + S * PAIR_A_UNITS;
    u32x4_t* lds_s = lds_b + S * PAIR_B_UNITS;

    // (the thread id is taken as found: what is derived from it is worked out per tile and does not hold
    // registers from tile to tile, where the routine has none to spare)
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    const int lane = tid & 63;
    const int i = lane & 15, q = lane >> 4;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int cw = wv & 3;                                    // column group: 64 columns
    // the sub-step of every step this wavefront owns (Q4: a step is one sub-step)
    const int h = Q4 ? 0 : 1 - (wv >> 2);
    // this lane's 4 columns (MFMA t = column col0 + t): half of a dword of 8 4-bit codes, or a dword of 4 bytes
    const int col0 = B8 ? 64 * cw + 4 * i : 128 * (cw >> 1) + 8 * i + 4 * (cw & 1);
    const int nk = P.K / BK;

    const int64_t KN = (int64_t)P.K * P.N;
    const rsrc_t rw = B8 ? make_rsrc(P.w + g * KN, KN) : make_rsrc(P.w + g * (KN >> 1), KN >> 1);
    const rsrc_t rs = KC ? make_rsrc(static_cast<const uint16_t*>(P.scale) + g * (KN / KBLK), (KN / KBLK) * 2)
                         : make_rsrc(static_cast<const uint16_t*>(P.scale) + (int64_t)g * P.scale_rows * P.N,
                                     (int64_t)P.scale_rows * P.N * 2);
    // fp8: the expert's fp32 block scales [K/128, N/128]; this wavefront's 128-column block
    const rsrc_t rs8 = make_rsrc(static_cast<const float*>(P.scale) + (int64_t)g * (P.K >> 7) * (P.N >> 7),
                                 (int64_t)(P.K >> 7) * (P.N >> 7) * 4);
    const int cs8 = ((n0 + 64 * cw) >> 7) * 4;
    // sub-step -> scale row as a multiply (worked out on the host from the 32-k sub-steps per scale group)
    const uint32_t gmul = (B8 || KC) ? 0u : P.sub_to_group;
    auto scale_row = [&](uint32_t sub) { return gmul ? (int)__umulhi(sub, gmul) : (int)sub; };
    // x rows through a buffer resource that ends after the last valid row (padded rows read as
    // zeros).  Load instruction j covers rows 8j + (lane >> 3); position lane & 7 of a row
    // holds chunk (lane & 7) ^ (row & 7), the swizzle a_lds_unit expects.
    // (Q4, rows of 64 bytes: instruction j covers rows 16j + (lane >> 2); position lane & 3 of a row holds
    // chunk (lane & 3) ^ ((row >> 1) & 3), see a_lds_unit32)
    const rsrc_t rx = make_rsrc(P.x + row0 * (int64_t)P.K, (int64_t)rows * P.K * 2);
    const int va = Q4 ? ((lane >> 2) * P.K + (((lane & 3) ^ ((lane >> 3) & 3)) * 8)) * 2
                      : ((lane >> 3) * P.K + (((lane & 7) ^ (lane >> 3)) * 8)) * 2;
    // packed tile: instruction wv brings rows 8 wv + (lane >> 3) into the 1 KB block wv of the stage;
    // the two 64-byte halves of the rows with odd (row >> 3) are swapped, so that the four q groups
    // of a wavefront read from both halves of the banks
    // int8 / fp8 (rows of 256 bytes): instruction e of wavefront wv brings rows 8 wv + 4 e + (lane >> 4); the
    // 64-byte quarters of a row are permuted by (row >> 3) & 3 = wv & 3, so that the four q groups read
    // from different quarters of the banks
    // K-contiguous fp4: LDS unit 64 wv + lane of the stage holds one 16-byte half of weight row
    // n = 32 wv + (lane >> 1); the halves of the rows with odd (n >> 3) are swapped (bank spread)
    const int kc_n = 32 * wv + (lane >> 1);
    const int vb = KC   ? kc_n * (P.K >> 1) + 16 * ((lane & 1) ^ ((kc_n >> 3) & 1))
                   : B8 ? (lane >> 4) * P.N + (((lane & 15) ^ (4 * (wv & 3))) * 16)
                        : (lane >> 3) * (P.N >> 1) + (((lane & 7) ^ (4 * (wv & 1))) * 16);
    constexpr int XI = Q4 ? MT : 2 * MT;          // x load instructions per step (1 KB each: 16 or 8 rows)
    constexpr int XROWS = Q4 ? 16 : 8;
    constexpr int NA = (XI + NW - 1) / NW;        // ... per wavefront
    constexpr int NB = B8 ? 2 : 1;                // packed-tile instructions
    constexpr int NI = NA + NB + ((PAIR_SC_UNITS || KC) ? 1 : 0);   // + this wavefront's share of the step's scales
    int ja[NA], ca[NA];
#pragma unroll
    for (int m = 0; m < NA; ++m) {
        int j = wv + NW * m;
        if (NW * NA > XI) j = j % XI;   // repeat a block rather than issue fewer loads
        ja[m] = j * 64;
        ca[m] = XROWS * j * P.K * 2;
    }
    // (Q4 on the reference's fp4 container: the 32 k of a step are the rows [16 hp, +16) and [32 + 16 hp, +16) of the
    // container's 64-row tile, hp = step & 1: wavefront wv brings the 8 rows from 32 (wv >> 1) + 16 hp + 8 (wv & 1) on)
    const int cb = KC            ? n0 * (P.K >> 1)
                   : B8          ? 8 * wv * P.N + n0
                   : (Q4 && FP4) ? (32 * (wv >> 1) + 8 * (wv & 1)) * (P.N >> 1) + (n0 >> 1)
                                 : 8 * wv * (P.N >> 1) + (n0 >> 1);
    const int kb_step = KC ? BK / 2 : B8 ? BK * P.N : BK * (P.N >> 1);
    // byte offset of step kp's packed rows in the expert's slab
    auto b_step_offset = [&](int kp) {
        if constexpr (Q4 && FP4)
            return ((kp >> 1) * 64 + (kp & 1) * 16) * (P.N >> 1);
        else
            return kp * kb_step;
    };
    // K-contiguous fp4 scales.  Fetching the 4 or 8 bytes a weight row needs per step costs a request per
    // row and step (measured: 20 % of the kernel); instead 16 bytes of a row -- the scales of SUP steps --
    // are fetched at a time: the load slot of step kt brings, for step index kp = kt + KC_D, the rows
    // [RPS (kp % SUP), + RPS) of super-block kp / SUP (one lane per row, RPW rows per wavefront) into buffer
    // (kp / SUP) % 3 of 256 rows x 16 bytes behind the stages.  KC_D = SUP + 3: a load issued in step t is
    // visible after barrier t + 2, and the scales of step s are read during step s - 1.  Three buffers: the
    // first load into a buffer comes after the last read of its previous occupant.
    constexpr int SUP = KBLK == 32 ? 4 : 2, KC_D = SUP + 3, RPS = 256 / SUP, RPW = RPS / 8;
    const int kc_vs = lane * (P.K / KBLK) * 2;
    auto kc_issue_scale = [&](int kp) {
        const int sb = kp / SUP, j = kp % SUP, row = RPS * j + RPW * wv;
        if (lane < RPW)
            lds_load16(rs, lds_s + (sb % 3) * 256 + row, kc_vs, (n0 + row) * (P.K / KBLK) * 2 + sb * 16);
    };
    // scales of a step: int4 2 rows of 512 bytes, 128 bytes (8 lanes) per wavefront: bytes [128 (wv & 3), +128) of
    // row wv >> 2; fp4 4 rows (one per 16 k), 256 bytes (16 lanes) per wavefront: bytes [256 (wv & 1), +256) of row wv >> 1
    const int cs = FP4 ? n0 * 2 + (wv & 1) * 256 : n0 * 2 + (wv & 3) * 128;
    const int lane16 = lane * 16;
    const bool s_lane = lane < (FP4 ? 16 : 8);
    // where this wavefront's loads land in stage 0 (byte addresses in LDS)
    uint32_t a_at[NA];
#pragma unroll
    for (int m = 0; m < NA; ++m) a_at[m] = lds_address(lds_a + ja[m]);
    const uint32_t b_at = lds_address(lds_b + wv * (PAIR_B_UNITS / NW));
    const uint32_t s_at = lds_address(lds_s + wv * (F8 ? 1 : PAIR_SC_UNITS / NW));
    // m-th load of group kt (stage kt+AHEAD of x, packed tile and scales), into LDS stage ST
    auto issue = [&](int m, int kt, int ST) {
        if (m < NA) {
            lds_load16_at(rx, here(a_at[m]) + ST * (PAIR_A_UNITS * 16), va, ca[m] + (kt + AHEAD) * (BK * 2));
        } else if (m < NA + NB) {
            const int e = m - NA;
            lds_load16_at(rw, here(b_at) + ST * (PAIR_B_UNITS * 16) + e * 1024, vb,
                          cb + (B8 ? 4 * e * P.N : 0) + b_step_offset(kt + AHEAD));
        } else if constexpr (KC) {
            kc_issue_scale(kt + KC_D);
        } else if constexpr (F8) {
            // the block scale of the stage's 128-k block, 4 bytes by lane 0 (past K: reads as 0, unused)
            if (lane == 0)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(
                    rs8, (__attribute__((address_space(3))) void*)(uintptr_t)(here(s_at) + ST * (PAIR_SC_UNITS * 16)), 4, 0,
                    ((kt + AHEAD) >> (Q4 ? 2 : 1)) * (P.N >> 7) * 4 + cs8, 0, 0);
        } else {
            const int grow = FP4  ? (kt + AHEAD) * (Q4 ? 2 : 4) + (wv >> 1)
                             : Q4 ? scale_row((uint32_t)(kt + AHEAD))
                                  : scale_row((uint32_t)((kt + AHEAD) * 2 + (wv >> 2)));
            if (s_lane) lds_load16_at(rs, here(s_at) + ST * (PAIR_SC_UNITS * 16), lane16, grow * (P.N * 2) + cs);
        }
    };
    auto issue_group = [&](int kt, int ST) {
#pragma unroll
        for (int m = 0; m < NI; ++m) issue(m, kt, ST);
    };

    // perm selector: bytes 2hh, 2hh+1 of row a, then of row b (hh = half of the dword this lane owns)
    const uint32_t h2 = 2u * (uint32_t)(cw & 1);
    // (int4 with the GEMV op's arithmetic: row a and row b interleaved, so that a 16-bit word holds a k pair)
    constexpr bool I4X = EXACT && FMT == MOE_FMT_INT4;
    uint32_t sel = I4X ? h2 | ((4u + h2) << 8) | ((h2 + 1u) << 16) | ((5u + h2) << 24)
                       : h2 | ((h2 + 1u) << 8) | ((4u + h2) << 16) | ((5u + h2) << 24);
    uint32_t mask = 0x0f0f0f0fu;
    asm volatile("" : "+s"(mask), "+s"(sel));   // kept opaque so that each stays one SGPR operand
    const int d = 16 * (cw >> 1) + i;            // dword column of this lane
    const int unit = (d >> 2) ^ (4 * (q & 1));
    // row of the x stage this lane's fragment row i comes from (STACK2: see above)
    const int xrow = STACK2 ? (((i >> 3) == (q >> 1)) ? (i & 7) : 8 + (i & 7)) : i;
    // LDS unit (within a stage) of this lane's 8 k of tile row `row`
    auto x_unit = [&](int row) {
        if constexpr (Q4)
            return a_lds_unit32(row, q);
        else
            return a_lds_unit<64>(row, 4 * h + q);
    };

    // The accumulators are zeroed by asm so that the compiler cannot re-materialize the zeros
    // right in front of the first MFMA that accumulates into them: a VALU write of an MFMA's
    // accumulator input needs wait states the compiler only inserts for MFMAs it can see.
    // (Done behind the prologue's loads, below: up to 160 moves that would otherwise delay the first request.)
    f32x4_t acc[MT][4];
    u32x4_t bf[4], afr[4];
    constexpr int RING = 3;
    constexpr int R = RING < MT ? RING : MT;   // x fragments read ahead of their MFMAs

    // int8: per-channel scale and offset of this lane's 4 columns, fixed for the tile (ordinary loads,
    // older than every ring load: the counted waits below cover them)
    float ch_s[4] = {0.f, 0.f, 0.f, 0.f}, ch_o[4] = {0.f, 0.f, 0.f, 0.f};
    u32x2_t ch_sb = {0u, 0u}, ch_ob = {0u, 0u};
    if constexpr (I8) {
        ch_sb = *reinterpret_cast<const u32x2_t*>(static_cast<const uint16_t*>(P.scale) + (int64_t)g * P.N + n0 + col0);
        ch_ob = *reinterpret_cast<const u32x2_t*>(P.offset + (int64_t)g * P.N + n0 + col0);
    }
    // groups -AHEAD .. -1: stages 0 .. AHEAD-1; stages 0 and 1 must have landed before the first barrier
    // (WAITN: the loads of the S - 3 youngest groups may still be in flight at a barrier)
    constexpr int WAITN = (S - 3) * NI;
    // wait until this wavefront's loads of all but the S - 3 youngest groups have landed, then a barrier (prologue)
    auto ring_barrier = [&]() { asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(WAITN) : "memory"); };
    // Inside the k loop the step's barrier is split in two.  A wavefront "arrives" at the end of step kt: it is
    // done with stage kt, and its loads of stage kt + 2 have landed; it adds 1 to a counter in LDS.  It only
    // "waits" -- polls the counter until all 8 wavefronts have arrived kt times -- at the start of the MFMA phase
    // of step kt + 1, in front of the first things that need the others: the loads that overwrite stage kt and
    // the packed dwords of stage kt + 2.  A whole decode phase lies between the two, so a wavefront that is late
    // by less than that stalls nobody (measured against one s_barrier per step: 7 % at K = 7168, 4 % at K = 2048).
    // Everything is inline asm so that the compiler can move nothing across it; every wavefront arrives once in
    // every step of a tile, so every wait ends.  The counter is zeroed per tile, ahead of the prologue's barrier.
    // (the counter's address stays in an SGPR; the asm makes its vector operands on the spot, so that no vector
    // register is held for them through the decode)
    const uint32_t arrivals_at = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uintptr_t)MOE_LDS_PTR(tk.arrivals));
    const __attribute__((address_space(3))) uint32_t* arrivals_lds =
        reinterpret_cast<const __attribute__((address_space(3))) uint32_t*>(MOE_LDS_PTR(tk.arrivals));
    uint32_t arrivals_seen = 0u;
    if (tid == 0) {
        uint32_t va, vz;
        asm volatile("v_mov_b32 %0, %2\n\tv_mov_b32 %1, 0\n\ts_nop 0\n\tds_write_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)"
                     : "=&v"(va), "=&v"(vz) : "s"(arrivals_at) : "memory");
    }
    auto ring_arrive = [&]() {
        uint32_t va, v1;
        asm volatile("s_waitcnt vmcnt(%2)\n\tv_mov_b32 %0, %3\n\tv_mov_b32 %1, 1\n\ts_mov_b64 exec, 1\n\tds_add_u32 %0, %1\n\ts_mov_b64 exec, -1"
                     : "=&v"(va), "=&v"(v1) : "n"(WAITN), "s"(arrivals_at) : "memory");
    };
    // early: the counter as read half a decode phase ago (usually enough, and its latency is hidden)
    auto ring_wait = [&](uint32_t steps, uint32_t early) {
        uint32_t seen_v, seen_s;
        asm volatile("v_readfirstlane_b32 %1, %4\n\ts_cmp_ge_u32 %1, %3\n\ts_cbranch_scc1 2f\n"
                     "1:\n\tv_mov_b32 %0, %2\n\ts_nop 0\n\tds_read_b32 %0, %0\n\ts_waitcnt lgkmcnt(0)\n\tv_readfirstlane_b32 %1, %0\n\ts_cmp_ge_u32 %1, %3\n\t"
                     "s_cbranch_scc1 2f\n\ts_sleep 1\n\ts_branch 1b\n2:"
                     : "=&v"(seen_v), "=&s"(seen_s) : "s"(arrivals_at), "s"((uint32_t)NW * steps), "v"(early) : "memory", "scc");
    };
    if constexpr (KC) {
        // the scale loads the groups below do not cover (older than all of them: landed by the first barrier)
#pragma unroll
        for (int kp = 0; kp < KC_D - AHEAD; ++kp) kc_issue_scale(kp);
    }
#pragma unroll
    for (int st0 = 0; st0 < AHEAD; ++st0) issue_group(st0 - AHEAD, st0);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            if constexpr (EXACT)
                acc[mt][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            else
                asm volatile("v_mov_b32 %0, 0\n\tv_mov_b32 %1, 0\n\tv_mov_b32 %2, 0\n\tv_mov_b32 %3, 0"
                             : "=v"(acc[mt][t][0]), "=v"(acc[mt][t][1]), "=v"(acc[mt][t][2]), "=v"(acc[mt][t][3]));
        }
    ring_barrier();
    // int8: (q + offset) * scale is defined as two rounded fp32 operations.  Where q + offset cannot round (an
    // offset of 0, or of a magnitude in [2^-8, 2^22]: the sum of an 8-bit integer and an 8-bit significand then fits
    // 24 bits) and offset * scale is exact and normal (scale positive and far from the ends of the range), one fma
    // q * scale + offset * scale rounds the same real number once and gives the same bits: 2.5 instead of 3.5
    // instructions per weight.  Decided per wavefront and tile from its lanes' channels.
    float ch_os[4] = {0.f, 0.f, 0.f, 0.f};
    bool i8_one_rounding = false;
    if constexpr (I8) {
        ch_s[0] = bf16_lo(ch_sb[0]); ch_s[1] = bf16_hi(ch_sb[0]); ch_s[2] = bf16_lo(ch_sb[1]); ch_s[3] = bf16_hi(ch_sb[1]);
        ch_o[0] = bf16_lo(ch_ob[0]); ch_o[1] = bf16_hi(ch_ob[0]); ch_o[2] = bf16_lo(ch_ob[1]); ch_o[3] = bf16_hi(ch_ob[1]);
        bool ok = true;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const float ao = fabsf(ch_o[t]);
            ok = ok && ch_s[t] >= 0x1p-60f && ch_s[t] <= 0x1p60f && (ao == 0.f || (ao >= 0x1p-8f && ao <= 0x1p22f));
            ch_os[t] = ch_o[t] * ch_s[t];
        }
        i8_one_rounding = __all(ok);
    }

    // this lane's packed dwords and scales of its sub-step of LDS stage st
    uint32_t r[8];
    u32x2_t sc = {0u, 0u}, sc2 = {0u, 0u};   // sc2: with EXACT, the fp4 scales of the second 16 k of the sub-step
    // (s: the step the stage belongs to)
    auto read_raw = [&](int st, int s) {
        const uint16_t* sc16 = reinterpret_cast<const uint16_t*>(lds_s + st * PAIR_SC_UNITS);
        if constexpr (FP4) {
            // Reference pre-shuffle (grouped_gemm/test/python/test_group_gemm_fp4.py:129-142): the tile row
            // 32 j + 8 i' + p holds, in its 32-byte run q', the 8 k rows 16 i' + 8 j + [0, 8) (one dword each)
            // of byte columns 16 p + 4 q' + [0, 4).  This lane's 8 k are 32 h + 8 q + [0, 8) and its two
            // bytes start at byte column 64 (cw >> 1) + 4 i + 2 (cw & 1): p = 4 (cw >> 1) + (i >> 2), q' = i & 3.
            // (Q4: the stage holds the step's 32 rows of that tile packed together, see cb)
            const int trow = Q4 ? 16 * (q & 1) + 8 * (q >> 1) + 4 * (cw >> 1) + (i >> 2)
                                : 32 * (q & 1) + 8 * (2 * h + (q >> 1)) + 4 * (cw >> 1) + (i >> 2);
            const int swz = 4 * ((trow >> 3) & 1);   // the halves of the rows with odd (row >> 3) are swapped (see vb)
            const u32x4_t* tb = lds_b + st * PAIR_B_UNITS + trow * 8;
            const u32x4_t lo4 = tb[(2 * (i & 3)) ^ swz], hi4 = tb[(2 * (i & 3) + 1) ^ swz];
#pragma unroll
            for (int j = 0; j < 4; ++j) { r[j] = lo4[j]; r[4 + j] = hi4[j]; }
            if constexpr (EXACT && !STACK2) {
                sc = *reinterpret_cast<const u32x2_t*>(sc16 + 256 * (2 * h) + col0);
                sc2 = *reinterpret_cast<const u32x2_t*>(sc16 + 256 * (2 * h + 1) + col0);
            } else {
                sc = *reinterpret_cast<const u32x2_t*>(sc16 + 256 * (2 * h + (q >> 1)) + col0);
            }
        } else if constexpr (KC) {
            // MFMA t takes weight row n = 64 cw + 16 t + i: its 8 codes k = 32 h + 8 q + [0, 8) are dword q of
            // the row's half h; the scale of that block
            const uint32_t* t32 = reinterpret_cast<const uint32_t*>(lds_b + st * PAIR_B_UNITS);
            // the row's 8 scales of super-block s / SUP; this lane's block among them
            const uint16_t* sup = reinterpret_cast<const uint16_t*>(lds_s + ((s / SUP) % 3) * 256) +
                                  (KBLK == 16 ? 4 * (s % SUP) + 2 * h + (q >> 1) : 2 * (s % SUP) + h);
            uint32_t s4[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const int n = 64 * cw + 16 * t + i;
                r[t] = t32[(2 * n + (h ^ ((i >> 3) & 1))) * 4 + q];
                s4[t] = sup[8 * n];
            }
            sc[0] = s4[0] | (s4[1] << 16);
            sc[1] = s4[2] | (s4[3] << 16);
        } else if constexpr (B8) {
            // dword 16 cw + i of each of this lane's 8 k rows; the quarter of the row it lies in is
            // permuted by (row >> 3) & 3 = q (see vb)
            const uint32_t* t32 = reinterpret_cast<const uint32_t*>(lds_b + st * PAIR_B_UNITS);
#pragma unroll
            for (int j = 0; j < 8; ++j) r[j] = t32[(32 * h + 8 * q + j) * 64 + 16 * (cw ^ q) + i];
            if constexpr (F8) sc[0] = *reinterpret_cast<const uint32_t*>(lds_s + st * PAIR_SC_UNITS + wv);
        } else {
            const uint32_t* t32 = reinterpret_cast<const uint32_t*>(lds_b + st * PAIR_B_UNITS);
#pragma unroll
            for (int j = 0; j < 8; ++j) r[j] = t32[((32 * h + 8 * q + j) * 8 + unit) * 4 + (d & 3)];
            sc = *reinterpret_cast<const u32x2_t*>(sc16 + 256 * h + col0);
        }
    };
    read_raw(0, 0);

    // One data step; st = step mod S is its LDS stage, sn the next one, sl the stage this step's loads
    // go to (wave-uniform).
    auto step = [&](int kt, int st, int sn, int sl) __attribute__((always_inline)) {
        const u32x4_t* la = lds_a + st * PAIR_A_UNITS;
        // ---- decode phase: this wavefront's sub-step of the packed stage -> bf[0..3]
        float m[4], z[4];
        const float s0 = bf16_lo(sc[0]), s1 = bf16_hi(sc[0]), s2 = bf16_lo(sc[1]), s3 = bf16_hi(sc[1]);
        // with EXACT: the scales of the step being multiplied (sc is refilled during the MFMA phase)
        const float f8s = __uint_as_float(sc[0]) * 256.f;   // fp8: the step's block scale (times the 2^8 the decode leaves out)
        const float sa[4] = {F8 ? f8s : s0, F8 ? f8s : s1, F8 ? f8s : s2, F8 ? f8s : s3};
        const float sb[4] = {bf16_lo(sc2[0]), bf16_hi(sc2[0]), bf16_lo(sc2[1]), bf16_hi(sc2[1])};
        if constexpr (EXACT) {
            m[0] = m[1] = m[2] = m[3] = FP4 ? 1.f : 512.f;
            z[0] = z[1] = z[2] = z[3] = FP4 ? 0.f : -8.f;
        } else if constexpr (FP4 || KC) {
            m[0] = s0; m[1] = s1; m[2] = s2; m[3] = s3;
            z[0] = z[1] = z[2] = z[3] = 0.f;
        } else {
            m[0] = s0 * 512.f; m[1] = s1 * 512.f; m[2] = s2 * 512.f; m[3] = s3 * 512.f;
            z[0] = -8.f * s0; z[1] = -8.f * s1; z[2] = -8.f * s2; z[3] = -8.f * s3;
        }
        // Written stage by stage over two row pairs at a time so that consecutive instructions are
        // independent (a VALU result is not available to the very next instruction); the fences
        // keep the scheduler from folding the stages back into per-element chains.
#pragma unroll
        for (int p0 = 0; p0 < 4; p0 += 2) {
            if (p0 == 2) {
                if constexpr (SPLIT_BARRIER) {
                    arrivals_seen = *arrivals_lds;   // a first look at the counter, checked after the decode
                } else if (h == 1) {
                    // barrier kt-1 for the wavefronts that own sub-step 1, half way through their decode
                    // (not in the tile's first step: the barrier of the prologue stands for it)
                    if (kt > 0) ring_barrier();
                }
                // first x fragments of the MFMA phase, read under the rest of the decode
#pragma unroll
                for (int f = 0; f < R; ++f) afr[f & 3] = la[x_unit(16 * f + xrow)];
            }
            if constexpr (KC) {
                // dword r[t] = 8 consecutive k of MFMA t's weight row: byte p = the k pair p
#pragma unroll
                for (int t = p0; t < p0 + 2; ++t) {
                    const f32x2_t f0 = e2m1_pair_to_f32<0>(r[t]), f1 = e2m1_pair_to_f32<1>(r[t]);
                    const f32x2_t f2 = e2m1_pair_to_f32<2>(r[t]), f3 = e2m1_pair_to_f32<3>(r[t]);
                    bf[t][0] = pack_bf16_rne(f0[0] * m[t], f0[1] * m[t]);
                    bf[t][1] = pack_bf16_rne(f1[0] * m[t], f1[1] * m[t]);
                    bf[t][2] = pack_bf16_rne(f2[0] * m[t], f2[1] * m[t]);
                    bf[t][3] = pack_bf16_rne(f3[0] * m[t], f3[1] * m[t]);
                }
                __builtin_amdgcn_sched_barrier(0);
                continue;
            }
            if constexpr (F8) {
                // byte t of the dwords of k rows 2p, 2p+1, decoded as a pair through fp16 (see
                // e4m3_ref_pair_over_256); the 2^8 goes into the block scale
                const float scl = __uint_as_float(sc[0]) * 256.f;
                float nz = -0.0f;
                asm volatile("" : "+v"(nz));   // kept in a register: not an inline constant
#pragma unroll
                for (int p = 0; p < 2; ++p) {
                    const uint32_t a = r[2 * (p0 + p)], b = r[2 * (p0 + p) + 1];
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const uint32_t sel8 = (uint32_t)t | 0x0c00u | ((uint32_t)(4 + t) << 16) | 0x0c000000u;   // [a.byte t, 0, b.byte t, 0]
                        const uint32_t h2 = e4m3_ref_pair_over_256_fp16(__builtin_amdgcn_perm(b, a, sel8));
                        if constexpr (EXACT) {
                            // the e4m3 values themselves (worth 2^-8): exact in bf16
                            typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
                            const half2_t hv = __builtin_bit_cast(half2_t, h2);
                            bf[t][p0 + p] = pack_bf16_rne((float)hv[0], (float)hv[1]);
                        } else {
                            bf[t][p0 + p] = pack_bf16_rne(fp16_lo_times(h2, scl, nz), fp16_hi_times(h2, scl, nz));
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                continue;
            }
            if constexpr (I8) {
                // byte t of the dwords of k rows 2p, 2p+1 -> (q + offset) * scale as two rounded fp32
                // operations (or the one fma that equals them, see i8_one_rounding) -> bf16 pair along k
                if (i8_one_rounding) {
#pragma unroll
                    for (int p = 0; p < 2; ++p) {
                        const uint32_t a = r[2 * (p0 + p)], b = r[2 * (p0 + p) + 1];
#pragma unroll
                        for (int t = 0; t < 4; ++t) {
                            const float qa = (float)(int)(int8_t)(a >> (8 * t)), qb = (float)(int)(int8_t)(b >> (8 * t));
                            bf[t][p0 + p] = pack_bf16_rne(__fmaf_rn(qa, ch_s[t], ch_os[t]), __fmaf_rn(qb, ch_s[t], ch_os[t]));
                        }
                    }
                } else {
#pragma unroll
                    for (int p = 0; p < 2; ++p) {
                        const uint32_t a = r[2 * (p0 + p)], b = r[2 * (p0 + p) + 1];
#pragma unroll
                        for (int t = 0; t < 4; ++t) {
                            const float qa = (float)(int)(int8_t)(a >> (8 * t)), qb = (float)(int)(int8_t)(b >> (8 * t));
                            bf[t][p0 + p] = pack_bf16_rne(__fmul_rn(__fadd_rn(qa, ch_o[t]), ch_s[t]),
                                                          __fmul_rn(__fadd_rn(qb, ch_o[t]), ch_s[t]));
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                continue;
            }
            uint32_t pr[2], lo[2], hi[2];
            f32x2_t a02[2], b02[2], a13[2], b13[2];
            float wa[2][4], wb[2][4];
#pragma unroll
            for (int p = 0; p < 2; ++p) pr[p] = __builtin_amdgcn_perm(r[2 * (p0 + p) + 1], r[2 * (p0 + p)], sel);   // a.b0 a.b1 b.b0 b.b1
            if constexpr (FP4) {
                // e2m1: each byte of pr is two columns of one k row; exact decode, one multiply by the
                // column's scale, RNE to bf16 (W = bf16(e2m1 * scale) as the reference's antiquant phase)
#pragma unroll
                for (int p = 0; p < 2; ++p) {
                    const f32x2_t a01 = e2m1_pair_to_f32<0>(pr[p]), a23 = e2m1_pair_to_f32<1>(pr[p]);
                    const f32x2_t b01 = e2m1_pair_to_f32<2>(pr[p]), b23 = e2m1_pair_to_f32<3>(pr[p]);
                    if constexpr (EXACT) {
                        bf[0][p0 + p] = pack_bf16_rne(a01[0], b01[0]);
                        bf[1][p0 + p] = pack_bf16_rne(a01[1], b01[1]);
                        bf[2][p0 + p] = pack_bf16_rne(a23[0], b23[0]);
                        bf[3][p0 + p] = pack_bf16_rne(a23[1], b23[1]);
                    } else {
                        bf[0][p0 + p] = pack_bf16_rne(a01[0] * m[0], b01[0] * m[0]);
                        bf[1][p0 + p] = pack_bf16_rne(a01[1] * m[1], b01[1] * m[1]);
                        bf[2][p0 + p] = pack_bf16_rne(a23[0] * m[2], b23[0] * m[2]);
                        bf[3][p0 + p] = pack_bf16_rne(a23[1] * m[3], b23[1] * m[3]);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                continue;
            }
#pragma unroll
            for (int p = 0; p < 2; ++p) { lo[p] = pr[p] & mask; hi[p] = pr[p] >> 4; }
            if constexpr (I4X) {
                // The codes themselves as bf16, two at a time: a nibble read as e4m3 is q / 512, and the scaled
                // convert (scale 2^9: only the exponent of that operand counts) yields the bf16 pair (q_a, q_b) of
                // one column.  The zero point is taken off in the MFMA phase.
#pragma unroll
                for (int p = 0; p < 2; ++p) {
                    hi[p] &= mask;
                    bf[0][p0 + p] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo[p], 512.f, false));
                    bf[2][p0 + p] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo[p], 512.f, true));
                    bf[1][p0 + p] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi[p], 512.f, false));
                    bf[3][p0 + p] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi[p], 512.f, true));
                }
                __builtin_amdgcn_sched_barrier(0);
                continue;
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                hi[p] &= mask;
                a02[p] = __builtin_amdgcn_cvt_pk_f32_fp8(lo[p], false);
                b02[p] = __builtin_amdgcn_cvt_pk_f32_fp8(lo[p], true);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                a13[p] = __builtin_amdgcn_cvt_pk_f32_fp8(hi[p], false);
                b13[p] = __builtin_amdgcn_cvt_pk_f32_fp8(hi[p], true);
            }
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                wa[p][0] = fmaf(a02[p][0], m[0], z[0]); wb[p][0] = fmaf(b02[p][0], m[0], z[0]);
                wa[p][2] = fmaf(a02[p][1], m[2], z[2]); wb[p][2] = fmaf(b02[p][1], m[2], z[2]);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                wa[p][1] = fmaf(a13[p][0], m[1], z[1]); wb[p][1] = fmaf(b13[p][0], m[1], z[1]);
                wa[p][3] = fmaf(a13[p][1], m[3], z[3]); wb[p][3] = fmaf(b13[p][1], m[3], z[3]);
            }
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                bf[0][p0 + p] = pack_bf16_rne(wa[p][0], wb[p][0]);
                bf[2][p0 + p] = pack_bf16_rne(wa[p][2], wb[p][2]);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                bf[1][p0 + p] = pack_bf16_rne(wa[p][1], wb[p][1]);
                bf[3][p0 + p] = pack_bf16_rne(wa[p][3], wb[p][3]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // ---- MFMA phase, at raised issue priority: the other wavefront of the SIMD is decoding
        // meanwhile and would otherwise win the arbitration whenever both are ready, starving
        // the matrix pipe; its VALU instructions fit into the gaps the MFMAs leave
        // every wavefront has arrived kt times (none in the tile's first step: the prologue's barrier stands for it)
        if constexpr (SPLIT_BARRIER) ring_wait((uint32_t)kt, arrivals_seen);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_setprio(3);
        // Everybody is done with stage kt-1 and has its part of stage kt+1 in LDS: this step's loads (stage kt+4
        // replaces stage kt-1) and the packed dwords of the next step (stage kt+1) are fetched between the MFMAs.
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            if (mt + R < MT) afr[(mt + R) & 3] = la[x_unit(16 * (mt + R) + xrow)];
            if constexpr (EXACT) {
                const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
                if constexpr (STACK2) {
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const f32x4_t dd = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            __builtin_bit_cast(bf16x8_t, afr[mt & 3]), __builtin_bit_cast(bf16x8_t, bf[t]), zero, 0, 0, 0);
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[mt][t][e] = fmaf(dd[e], sa[t], acc[mt][t][e]);
                    }
                } else if constexpr (FP4) {
                    const uint32_t mlo = q < 2 ? 0xffffffffu : 0u;
                    u32x4_t xlo, xhi;
#pragma unroll
                    for (int j = 0; j < 4; ++j) { xlo[j] = afr[mt & 3][j] & mlo; xhi[j] = afr[mt & 3][j] & ~mlo; }
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const f32x4_t dlo = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            __builtin_bit_cast(bf16x8_t, xlo), __builtin_bit_cast(bf16x8_t, bf[t]), zero, 0, 0, 0);
                        const f32x4_t dhi = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            __builtin_bit_cast(bf16x8_t, xhi), __builtin_bit_cast(bf16x8_t, bf[t]), zero, 0, 0, 0);
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[mt][t][e] = fmaf(dhi[e], sb[t], fmaf(dlo[e], sa[t], acc[mt][t][e]));
                    }
                } else {
                    // int4: the fragments hold q, not q - 8: each product starts from -8 sum_k x[m][k] (one more
                    // MFMA per x fragment, against a constant fragment of -8.0), so dd = sum_k x (q - 8)
                    f32x4_t start = zero;
                    if constexpr (I4X) {
                        const u32x4_t m8 = {0xc100c100u, 0xc100c100u, 0xc100c100u, 0xc100c100u};
                        start = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            __builtin_bit_cast(bf16x8_t, afr[mt & 3]), __builtin_bit_cast(bf16x8_t, m8), zero, 0, 0, 0);
                    }
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const f32x4_t dd = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            __builtin_bit_cast(bf16x8_t, afr[mt & 3]), __builtin_bit_cast(bf16x8_t, bf[t]), start, 0, 0, 0);
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[mt][t][e] = fmaf(dd[e], sa[t], acc[mt][t][e]);
                    }
                }
            } else {
#pragma unroll
                for (int t = 0; t < 4; ++t) mfma_16x16x32_v(acc[mt][t], afr[mt & 3], bf[t]);
            }
#pragma unroll
            for (int m = (mt * NI + MT - 1) / MT; m < ((mt + 1) * NI + MT - 1) / MT; ++m) issue(m, kt, sl);
            if (mt == 0) read_raw(sn, kt + 1);
            __builtin_amdgcn_sched_barrier(0);
        }
        __builtin_amdgcn_s_setprio(0);
        if constexpr (SPLIT_BARRIER) {
            ring_arrive();
        } else if (h == 0) {
            ring_barrier();   // barrier kt
        }
    };
    // unrolled over the ring, so that every stage number is a constant and the LDS addresses of a step are
    // immediate offsets (with run-time stage numbers a step spent 9 vector and about 25 scalar instructions on
    // them: measured 10 % of the kernel's time at K = 7168); a tile starts at stage 0
    // (the K-contiguous containers keep run-time stage numbers: their routine has no registers left for the
    // unrolled form)
    if constexpr (!KC) {
        for (int kt0 = 0; kt0 < nk; kt0 += S) {
#pragma unroll
            for (int u = 0; u < S; ++u)
                if (kt0 + u < nk) step(kt0 + u, u, (u + 1) % S, (u + S - 1) % S);
        }
    } else {
        for (int kt = 0, st = 0, sl = S - 1; kt < nk; ++kt) {
            const int sn = st == S - 1 ? 0 : st + 1;
            step(kt, st, sn, sl);
            st = sn;
            sl = sl == S - 1 ? 0 : sl + 1;
        }
    }
    if constexpr (!SPLIT_BARRIER)
        if (h == 1) ring_barrier();   // barrier nk-1
    // drain this wavefront's loads (they target stages past K and are never read); the
    // accumulators were last written by MFMAs the compiler cannot see: wait out their latency
    // (and the last arrivals are counted before anybody zeroes the counter for the next tile)
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_nop 15\n\ts_nop 15\n\ts_barrier" ::: "memory");

    if constexpr (STACK2) {
        // the lanes q and q + 2 hold the two scale groups' sums of the same rows
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[0][t][e] += __shfl_xor(acc[0][t][e], 32);
    }
    pair_finish<MT, KC, Q4>(P, smem, acc, h, cw, lane, col0, row0, rows, n0, tk);
}

// ---------------------------------------------------------------------------------
// Tile scheduler (role of GMMAntiquantProcess::Process,
// grouped_gemm/op_kernel/grouped_matmul_antiquant.h:241-288).  Expert g with m_g rows
// has ceil(m_g/16) row blocks, cut into the fewest chunks of <= MT_MAX blocks, as
// even as possible; each chunk has N/256 tiles.  prefix[] (in LDS) is the exclusive
// scan of the tile counts.
// ---------------------------------------------------------------------------------
template <int MT_MAX>
__device__ __forceinline__ void expert_chunks(int m, int& chunks, int& bpc) {
    const int nblk = (m + 15) >> 4;
    if (nblk <= MT_MAX) {   // the usual case, without the division
        chunks = nblk ? 1 : 0;
        bpc = nblk;
        return;
    }
    chunks = (nblk + MT_MAX - 1) / MT_MAX;
    bpc = (nblk + chunks - 1) / chunks;
}

template <int FMT, int KIND>
struct KernelCfg {
    static constexpr bool PAIR = KIND == GK_PAIR || KIND == GK_PAIR_SMALL || KIND == GK_QUAD || pair_exact(KIND);
    static constexpr bool SKINNY = KIND == GK_SKINNY;
    static_assert(!PAIR || FMT != MOE_FMT_BF16, "the k-split tile routine decodes quantized containers");
    static constexpr int WAVES = PAIR ? pair_waves(KIND) : 4;
    static constexpr int BN = GM_BN;                                             // columns per tile
    static constexpr int pair_wgs() {
        if constexpr (PAIR) return pair_wg_per_cu<FMT>(KIND); else return 1;
    }
    static constexpr int WG_PER_CU = SKINNY ? GM_SKINNY_WAVES : pair_wgs();
    static constexpr int WAVES_PER_SIMD = WG_PER_CU * WAVES / 4;
    static constexpr int CAPB = SKINNY ? GM_SKINNY_BLOCKS : PAIR ? PAIR_CAPB : GM_MT_MAX;
    static constexpr int fmt_mt_max() {
        if constexpr (PAIR)
            return pair_mt_max(KIND);
        else
            return BTraits<FMT>::MT_MAX;
    }
    static constexpr int MTM = CAPB < fmt_mt_max() ? CAPB : fmt_mt_max();        // row blocks per tile
    // 16-byte LDS units of the tile routine (the tile prefix array follows them)
    static constexpr int lds_units() {
        if constexpr (PAIR)
            return pair_lds_units<FMT>(KIND);
        else
            return 2 * 16 * CAPB * (BTraits<FMT>::BK / 8);
    }
};

template <int FMT, int MT, int KIND>
__device__ __forceinline__ void run_tile(const GemmParams& P, u32x4_t* smem, int g, int64_t row0, int rows, int n0, const Ticket& tk) {
    using C = KernelCfg<FMT, KIND>;
    if constexpr (C::PAIR) {
        if constexpr (FMT == MOE_FMT_FP4_REF && pair_exact(KIND) && MT == 1) {
            if (rows <= 8) return gemm_tile_pair<FMT, MT, KIND, true>(P, smem, g, row0, rows, n0, tk);
        }
        gemm_tile_pair<FMT, MT, KIND>(P, smem, g, row0, rows, n0, tk);
    }
    else
        gemm_tile<FMT, MT, C::CAPB>(P, smem, g, row0, rows, n0);
}

template <int FMT, int KIND>
__global__ __launch_bounds__((64 * KernelCfg<FMT, KIND>::WAVES), (KernelCfg<FMT, KIND>::WAVES_PER_SIMD)) void grouped_gemm_kernel(GemmParams P) {
    using C = KernelCfg<FMT, KIND>;
    constexpr int WAVES = C::WAVES;
    extern __shared__ u32x4_t smem[];
    constexpr int THREADS = 64 * WAVES;
    constexpr int MTM = C::MTM;
    // [G + 1] first tile of every expert; table_mode 0: [THREADS + 1] first tile of every thread's run of experts
    int* prefix = reinterpret_cast<int*>(smem + C::lds_units());
    // [G + 1] row bounds: rowc[g] = group_list[g - 1] clamped to [0, M] (rowc[0] = 0); expert g owns the rows
    // [rowc[g], rowc[g + 1]) if that is not empty (same result as clamping start and end separately).  Kept in
    // LDS so that the scheduler does not wait for a global load per tile (2 to 4 us under a streaming kernel).
    int* rowc = prefix + (P.G + 1);
    const int tid = threadIdx.x;
    const int ntile_n = (P.N + C::BN - 1) / C::BN;
    // scan partials (one per wavefront); later part[0] carries the ticket drawn from the queue, part[1] the tile
    // resolved from it, part[2] the tile routine's arrival counter
    __shared__ int part[THREADS];
    constexpr int PART_FIXED = 16;   // first whether this workgroup uses the launch's counter, then its number of fixed sweeps
    auto clamp_row = [&](int64_t v) { return (int)min(max(v, (int64_t)0), P.M); };
    auto expert_rows = [&](int g, int& first) {
        int hi;
        if (P.table_mode == 2) {
            first = rowc[g];
            hi = rowc[g + 1];
        } else {
            first = g ? clamp_row(P.gl[g - 1]) : 0;
            hi = clamp_row(P.gl[g]);
        }
        return max(hi - first, 0);
    };

    // the launch's counter is looked at, and raised to the launch's stamp, now: long before the first draw from it
    if (tid == 0) part[PART_FIXED] = P.slot >= 0 && queue_open(tile_queue + GM_QUEUE_STRIDE * max(P.slot, 0), P.stamp, blockIdx.x < 8);

    // exclusive scan of tiles per expert: each thread takes a contiguous run of experts
    const int per = (P.G + THREADS - 1) / THREADS;
    const int entries = P.table_mode ? P.G : THREADS;   // the table has entries + 1 elements
    {
        const int g0 = min(P.G, tid * per), g1 = min(P.G, g0 + per);
        if (P.table_mode == 2) {
            for (int g = g0; g < g1; ++g) rowc[g + 1] = clamp_row(P.gl[g]);
            if (tid == 0) rowc[0] = 0;
            __syncthreads();
        }
        int sum = 0;
        for (int g = g0; g < g1; ++g) {
            int first, chunks, bpc;
            expert_chunks<MTM>(expert_rows(g, first), chunks, bpc);
            sum += chunks * ntile_n;
        }
        // scan over the threads: within a wavefront by shuffles, across wavefronts through their totals in
        // LDS (a loop of one thread over all partial sums took 8 us at the start of every workgroup)
        const int lane = tid & 63, wave = tid >> 6;
        int incl = sum;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int up = __shfl_up(incl, off, 64);
            if (lane >= off) incl += up;
        }
        if (lane == 63) part[wave] = incl;
        __syncthreads();
        int before = 0, all = 0;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            const int v = part[w];
            before += w < wave ? v : 0;
            all += v;
        }
        if (tid == 0) prefix[entries] = all;
        int run = before + incl - sum;
        if (P.table_mode) {
            for (int g = g0; g < g1; ++g) {
                int first, chunks, bpc;
                expert_chunks<MTM>(expert_rows(g, first), chunks, bpc);
                prefix[g] = run;
                run += chunks * ntile_n;
            }
        } else {
            prefix[tid] = run;
        }
        __syncthreads();
    }
    const int total = __builtin_amdgcn_readfirstlane(prefix[entries]);

    // XCD-aware order: workgroup b runs on XCD b % 8; give each XCD a contiguous run of
    // tiles in every sweep so that its workgroups share x rows in its own L2.
    const int nwg = gridDim.x;
    const int per_xcd = (nwg + 7) / 8;
    const int vid = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    const int sweep = per_xcd * 8;   // == nwg: the grid is a multiple of 8
    // The number of sweeps in the fixed order lives in LDS, not in a register that would stay live across the tile
    // routines; GM_NO_QUEUE: a launch without counters (captured into a HIP graph, or one whose slot a later launch
    // holds by now) walks every tile in the fixed order, sweep after sweep until the tile number passes the last.
    constexpr int GM_NO_QUEUE = 0x7fffffff;
    // (at least one sweep in the fixed order before the first draw, so that the stamp is there by then; launches of
    // at most one tile per workgroup have nothing to balance)
    if (tid == 0) part[PART_FIXED] = part[PART_FIXED] && total > sweep ? max(1, total / sweep - GM_QUEUE_TAIL_SWEEPS) : GM_NO_QUEUE;
    __syncthreads();

    bool have_ticket = false;   // the previous tile routine left its ticket in part[0]
    queue_word_t* const q_own = tile_queue + GM_QUEUE_STRIDE * max(P.slot, 0);
    for (int sw = 0;; ++sw) {
        int T;
        int fixed = __builtin_amdgcn_readfirstlane(part[PART_FIXED]);
        if (sw >= fixed) {
            if (fixed == GM_NO_QUEUE) break;
            if (!have_ticket) {
                __syncthreads();   // part[] of the previous round is read
                if (tid == 0) part[0] = queue_draw(q_own, P.stamp);
                __syncthreads();
            }
            const int own = __builtin_amdgcn_readfirstlane(part[0]);
            if (own >= 0) {
                T = fixed * sweep + own;
                if (T >= total) break;
            } else {
                // the slot belongs to a later launch: this workgroup's share of the tail in the fixed order
                __syncthreads();   // everyone has read this round's part[PART_FIXED]
                if (tid == 0) part[PART_FIXED] = GM_NO_QUEUE;
                sw = fixed;
                fixed = GM_NO_QUEUE;
            }
        }
        if (sw < fixed) {
            // (the last, partial sweep of a launch without a counter goes to the workgroups in launch order, i.e.
            // round-robin over the XCDs and to different CUs first, not to the first XCDs' workgroups only: where two
            // workgroups share a CU the tiles per CU, which is what its time follows, then differ by at most one)
            T = sw * sweep + ((sw + 1) * sweep > total ? (int)blockIdx.x : vid);
            if (T >= total) break;
        }
        // from the last tile of the fixed order on, the k-split tile routines draw the next ticket themselves
        const bool take = C::PAIR && fixed != GM_NO_QUEUE && sw + 1 >= fixed;
        const Ticket tk = {take ? q_own : nullptr, part, part + 2};
        have_ticket = take;
        // largest e with prefix[e] <= T (empty experts have prefix[e] == prefix[e+1]): every wavefront looks at 64
        // evenly spaced entries at once, then at the entries between two of them -- two LDS round trips
        // instead of the ten of a binary search
        const int lane64 = tid & 63;
        const int stride = (entries + 63) >> 6;                  // entries per lane of the first step
        const int probe = min(lane64 * stride, entries);
        const unsigned long long le1 = __ballot(prefix[probe] <= T && lane64 * stride <= entries);
        const int seg = 63 - __builtin_clzll(le1 | 1ull);        // last lane whose entry is <= T (lane 0: prefix[0] = 0)
        // (the entries <= T of a segment are its first ones: count them, 64 at a time; one pass up to 4096 entries)
        int upto = 0;
        for (int o = 0; o < stride; o += 64) {
            const int idx2 = seg * stride + o + lane64;
            const int n_le = __popcll(__ballot(o + lane64 < stride && idx2 < entries && prefix[idx2] <= T));
            upto += n_le;
            if (n_le < 64) break;
        }
        // everything below is wave-uniform; readfirstlane lets the compiler keep it in SGPRs
        const int found = __builtin_amdgcn_readfirstlane(seg * stride + max(upto, 1) - 1);
        int g = found, local = __builtin_amdgcn_readfirstlane(T - prefix[found]);
        if (P.table_mode == 0) {
            // found is a thread's run of experts: walk it 64 experts at a time (group_list from memory, the tile
            // counts summed across the wavefront) up to the expert that holds tile number `local` of the run
            const int e_end = min(P.G, (found + 1) * per);
            g = -1;
            for (int e0 = found * per, base = 0; e0 < e_end && g < 0; e0 += 64) {
                const int ge = e0 + lane64;
                int tiles = 0;
                if (ge < e_end) {
                    int first, ch, bp;
                    expert_chunks<MTM>(expert_rows(ge, first), ch, bp);
                    tiles = ch * ntile_n;
                }
                int incl = tiles;
#pragma unroll
                for (int off = 1; off < 64; off <<= 1) {
                    const int up = __shfl_up(incl, off, 64);
                    if (lane64 >= off) incl += up;
                }
                const unsigned long long hit = __ballot(base + incl > local);
                if (hit) {
                    const int l = __ffsll(hit) - 1;
                    g = e0 + l;
                    local -= base + __shfl(incl - tiles, l, 64);
                } else {
                    base += __shfl(incl, 63, 64);
                }
            }
            g = __builtin_amdgcn_readfirstlane(g);
            local = __builtin_amdgcn_readfirstlane(local);
            if (g < 0) break;   // cannot happen: the run holds the tile
        }
        int gfirst;
        const int m = __builtin_amdgcn_readfirstlane(expert_rows(g, gfirst));
        const int64_t gbeg = gfirst;
        int chunks, bpc;
        expert_chunks<MTM>(m, chunks, bpc);
        // row chunks innermost: the tiles that share a weight column tile are neighbours in the order, run at
        // the same time on one XCD and pull that slice of the expert's weights into its L2 once
        const int nt = chunks == 1 ? local : local / chunks, chunk = chunks == 1 ? 0 : local % chunks;
        const int rbeg = chunk * bpc * 16;
        const int rows = min(m - rbeg, bpc * 16);
        const int mt = (rows + 15) >> 4;
        const int rlo = __builtin_amdgcn_readfirstlane((int)(uint32_t)(gbeg & 0xffffffffLL));
        const int rhi = __builtin_amdgcn_readfirstlane((int)(gbeg >> 32));
        const int64_t row0 = (((int64_t)rhi << 32) | (uint32_t)rlo) + rbeg;
        const int n0 = nt * C::BN;
        switch (mt) {
            case 1:
                if constexpr (MTM >= 1) run_tile<FMT, 1, KIND>(P, smem, g, row0, rows, n0, tk);
                break;
            case 2:
                if constexpr (MTM >= 2) run_tile<FMT, 2, KIND>(P, smem, g, row0, rows, n0, tk);
                break;
            case 3:
                if constexpr (MTM >= 3) run_tile<FMT, 3, KIND>(P, smem, g, row0, rows, n0, tk);
                break;
            case 4:
                if constexpr (MTM >= 4) run_tile<FMT, 4, KIND>(P, smem, g, row0, rows, n0, tk);
                break;
            case 5:
                if constexpr (MTM >= 5) run_tile<FMT, 5, KIND>(P, smem, g, row0, rows, n0, tk);
                break;
            case 6:
                if constexpr (MTM >= 6) run_tile<FMT, 6, KIND>(P, smem, g, row0, rows, n0, tk);
                break;
            case 7:
                if constexpr (MTM >= 7) run_tile<FMT, 7, KIND>(P, smem, g, row0, rows, n0, tk);
                break;
            case 8:
                if constexpr (MTM >= 8) run_tile<FMT, 8, KIND>(P, smem, g, row0, rows, n0, tk);
                break;
            case 9:
                if constexpr (MTM >= 9) run_tile<FMT, 9, KIND>(P, smem, g, row0, rows, n0, tk);
                break;
            case 10:
                if constexpr (MTM >= 10) run_tile<FMT, 10, KIND>(P, smem, g, row0, rows, n0, tk);
                break;
            case 11:
                if constexpr (MTM >= 11) run_tile<FMT, 11, KIND>(P, smem, g, row0, rows, n0, tk);
                break;
            case 12:
                if constexpr (MTM >= 12) run_tile<FMT, 12, KIND>(P, smem, g, row0, rows, n0, tk);
                break;
            default: have_ticket = false; break;
        }
    }
}

int64_t gemm_shift_launch_number(int64_t delta) {
    return (int64_t)(queue_launches.fetch_add((uint64_t)delta, std::memory_order_relaxed) + (uint64_t)delta);
}

// Compute units of the current device, looked up once per device.
static int device_cu_count() {
    static std::atomic<int> cached[64];
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return -1;
    int cus = cached[dev].load(std::memory_order_relaxed);
    if (cus == 0) {
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) return -1;
        cached[dev].store(cus, std::memory_order_relaxed);
    }
    return cus;
}

template <int FMT, int KIND>
static int launch_gemm_kind(const GemmParams& P, const moe_grouped_args* a, hipStream_t stream) {
    using C = KernelCfg<FMT, KIND>;
    const size_t lds_max = (160 * 1024 - 2048) / C::WG_PER_CU;
    const size_t table = ((size_t)a->G + 1) * sizeof(int);
    // tile table, and the row bounds next to it where they fit; else the scheduler reads group_list per tile; else,
    // with more experts than LDS holds a table for, it keeps one entry per thread and walks group_list (see
    // GemmParams::table_mode)
    const size_t units = (size_t)C::lds_units() * 16;
    const int table_mode = units + 2 * table <= lds_max ? 2 : units + table <= lds_max ? 1 : 0;
    const size_t lds = units + (table_mode ? table_mode * table : (size_t)(64 * C::WAVES + 1) * sizeof(int));
    if (lds > lds_max) return MOE_ERR_TOO_LARGE;
    static std::atomic<uint64_t> lds_set{0};
    if (const int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(&grouped_gemm_kernel<FMT, KIND>), (int)lds_max, lds_set))
        return rc;
    const int cus = device_cu_count();
    if (cus <= 0) return MOE_ERR_NO_DEVICE;
    // persistent grid: as many workgroups as the CUs hold, but no more than an upper bound on the
    // tile count that needs no look at group_list (every expert adds at most one partly filled chunk)
    const int64_t max_chunks = a->M / (16 * C::MTM) + a->G;
    const int64_t max_tiles = max_chunks * ((a->N + C::BN - 1) / C::BN);
    const int64_t want = max_tiles < (int64_t)cus * C::WG_PER_CU ? max_tiles : (int64_t)cus * C::WG_PER_CU;
    // a multiple of 8 so that the XCD-aware order covers every tile index
    const int64_t grid = want > 0 ? (want + 7) / 8 * 8 : 8;
    GemmParams Q = P;
    // A launch that is being captured into a graph gets no counters (see tile_queue); so does one whose
    // stream cannot be queried.  (The null stream cannot be captured and is not asked.)
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (stream != nullptr && hipStreamIsCapturing(stream, &capture) != hipSuccess) {
        (void)hipGetLastError();
        capture = hipStreamCaptureStatusActive;
    }
    if (capture == hipStreamCaptureStatusNone) {
        const uint64_t launch = queue_launches.fetch_add(1, std::memory_order_relaxed);
        Q.slot = (int)(launch % GM_QUEUE_SLOTS);
        Q.stamp = (launch / GM_QUEUE_SLOTS + 1) << GM_QUEUE_COUNT_BITS;
    } else {
        Q.slot = -1;
        Q.stamp = 0;
    }
    Q.table_mode = table_mode;
    hipLaunchKernelGGL((grouped_gemm_kernel<FMT, KIND>), dim3((unsigned)grid), dim3(64 * C::WAVES), lds, stream, Q);
    return hipGetLastError() == hipSuccess ? MOE_OK : MOE_ERR_LAUNCH;
}

static GemmParams gemm_params(const moe_grouped_args* a) {
    GemmParams P;
    P.x = static_cast<const uint16_t*>(a->x);
    P.w = static_cast<const uint8_t*>(a->weight);
    P.scale = a->scale;
    P.offset = static_cast<const uint16_t*>(a->offset);
    P.gl = a->group_list;
    P.y = static_cast<uint16_t*>(a->y);
    P.M = a->M; P.K = (int)a->K; P.N = (int)a->N; P.G = (int)a->G; P.scale_rows = (int)a->scale_rows;
    P.epilogue = a->epilogue;
    P.slot = -1;
    P.stamp = 0;
    P.table_mode = 0;
    const uint32_t per = a->scale_rows > 0 ? (uint32_t)((a->K / a->scale_rows) >> 5) : 1u;
    P.sub_to_group = per <= 1 ? 0u : 0xffffffffu / per + 1u;
    return P;
}

template <int FMT>
static int launch_gemm_fmt(const moe_grouped_args* a, hipStream_t stream) {
    const GemmParams P = gemm_params(a);
    // The N-contiguous containers run on the k-split kernel at every batch size: measured faster than the
    // small-tile kernel down to decode batches of 1-2 rows per expert (256 experts of 7168 x 2048: int4
    // 243 vs 344 us at 128 rows, fp4 476 vs 519 us and fp8 610 vs 784 us at 512 rows).
    if constexpr (FMT != MOE_FMT_BF16) {
        // decode-like batches (on average at most 12 rows per expert) on the 4-bit N-contiguous containers: the
        // small-stage kind (at 8 rows per expert int4 409 vs 506 us, fp4 448 vs 474 us; at 24 the large tiles win,
        // 531 vs 549 us and 512 vs 609 us).  The one-byte containers gain nothing from it.
        if constexpr (FMT == MOE_FMT_INT4 || FMT == MOE_FMT_FP4_REF)
            if (a->M <= 12 * a->G) return launch_gemm_kind<FMT, GK_PAIR_SMALL>(P, a, stream);
        // prefill on the N-contiguous containers: workgroups of 4 wavefronts without the k split, two per CU.  The 4-bit
        // ones always (256 experts of 128 rows, K = 7168, N = 4096: int4 1792 against 1905 us, fp4 1724 against 1867 us
        // with the k-split kind).  The one-byte ones, whose tiles move twice the bytes, when an expert has more rows than
        // one tile takes on average, so that its row chunks share a weight slice in L2: 8 experts of 512 rows, K = 4096,
        // N = 14336: int8 454 against 476 us, fp8 480 against 495 us; 64 experts of 512 rows at K = 7168, N = 4096: 1755
        // against 1870 us and 1872 against 1929 us; but with 128 rows per expert, every weight tile read once from HBM,
        // 1090 - 1110 against 1063 - 1098 us (int8) and 1125 - 1152 against 1088 - 1136 us (fp8) on 128 experts
        constexpr bool four_bit = FMT == MOE_FMT_INT4 || FMT == MOE_FMT_FP4_REF;
        constexpr bool one_byte = FMT == MOE_FMT_INT8 || FMT == MOE_FMT_FP8_REF;
        if constexpr (four_bit || one_byte) {
            if (four_bit || a->M > (int64_t)(16 * PAIR_CAPB) * a->G) {
                const int rc = launch_gemm_kind<FMT, GK_QUAD>(P, a, stream);
                if (rc != MOE_ERR_TOO_LARGE) return rc;
            }
        }
        return launch_gemm_kind<FMT, GK_PAIR>(P, a, stream);
    } else {
        // Decode-like batches (on average at most 24 rows per expert; group_list itself stays on the
        // device) are HBM bound: use the small-tile kernel.  An expert with more than 32 rows then
        // costs one pass over its weights per 32 rows.
        if (a->M <= 24 * a->G) return launch_gemm_kind<FMT, GK_SKINNY>(P, a, stream);
        return launch_gemm_kind<FMT, GK_GENERAL>(P, a, stream);
    }
}

int launch_gemm_exact(const moe_grouped_args* a, hipStream_t stream) {
    const GemmParams P = gemm_params(a);
    switch (a->format) {
        case MOE_FMT_FP4_REF:
            // decode-like batches (on average at most 12 rows per expert): 16-row tiles, two workgroups per CU; an
            // expert with more rows than that costs a pass over its weights per 16 rows
            if (a->M <= 12 * a->G) return launch_gemm_kind<MOE_FMT_FP4_REF, GK_PAIR_EXACT16>(P, a, stream);
            return launch_gemm_kind<MOE_FMT_FP4_REF, GK_PAIR_EXACT>(P, a, stream);
        case MOE_FMT_INT4: return launch_gemm_kind<MOE_FMT_INT4, GK_PAIR_EXACT>(P, a, stream);
        case MOE_FMT_FP8_REF: return launch_gemm_kind<MOE_FMT_FP8_REF, GK_PAIR_EXACT>(P, a, stream);
        default: return MOE_ERR_BAD_FORMAT;
    }
}

int launch_grouped_gemm(const moe_grouped_args* a, hipStream_t stream) {
    // Decode-sized batches on the K-contiguous containers go to the weight-streaming GEMV kernels,
    // run with this op's arithmetic.
    // (the GEMV kernels have no fused activation: such calls stay on the GEMM kernels)
    if (a->epilogue == MOE_EPILOGUE_NONE && gemv_preferred(a)) return launch_grouped_gemv(a, stream, true);
    switch (a->format) {
        case MOE_FMT_FP4_REF: return launch_gemm_fmt<MOE_FMT_FP4_REF>(a, stream);
        case MOE_FMT_FP8_REF: return launch_gemm_fmt<MOE_FMT_FP8_REF>(a, stream);
        case MOE_FMT_INT8: return launch_gemm_fmt<MOE_FMT_INT8>(a, stream);
        case MOE_FMT_INT4: return launch_gemm_fmt<MOE_FMT_INT4>(a, stream);
        case MOE_FMT_FP4_B32: return launch_gemm_fmt<MOE_FMT_FP4_B32>(a, stream);
        case MOE_FMT_FP4_B16: return launch_gemm_fmt<MOE_FMT_FP4_B16>(a, stream);
        case MOE_FMT_BF16: return launch_gemm_fmt<MOE_FMT_BF16>(a, stream);
        default: return MOE_ERR_BAD_FORMAT;
    }
}

}  // namespace moe
