// Expert histogram (continuous_count) and stable counting-sort index construction for the MoE layer.
//
// continuous_count: one launch. Every workgroup streams a contiguous chunk of ids with 16-byte loads and
// counts into an LDS histogram that holds NREP lane-private copies of every bin (address = id*NREP + lane%NREP),
// so lanes that carry the same id still hit different LDS banks and a skewed distribution costs the same as a
// uniform one. The copies are folded and the per-workgroup histogram is written to a workspace row; a second, tiny
// launch sums the rows into the output. No zeroing pass, no atomics on global memory and no fences: a last-arriver
// ticket inside one launch needs agent-scope release/acquire fences, which on this multi-XCD part write back and
// invalidate the L2 once per workgroup and cost twenty times the streaming itself.
//
// index construction: three small launches (per-chunk histogram, scan, placement). Chunks are contiguous
// ranges of slots, so "expert-major, chunk-minor, slot order inside the chunk" is exactly the stable order.
#include <mutex>

#include "common.h"

// Device-resident scratch of fma_moe_build_index_static (the per-chunk histograms of the counting sort), for callers
// that cannot hand over a workspace. One copy per GPU, held until the process ends; host code never uses this name as
// an address: static_scratch() below asks the runtime for the array's address on the current device.
#define FMA_STATIC_INDEX_WORDS (1 << 20)
static __device__ __align__(256) uint32_t scratch[FMA_STATIC_INDEX_WORDS];

namespace fmahip {
namespace {

constexpr int kCountThreads = 1024;
constexpr int kCountUnroll = 4;
constexpr int kCountBlocksPerCu = 2;
constexpr int kCountLdsWords = 16384;  // 64 KB of bins (all copies)

__host__ __device__ inline uint32_t floor_pow2(uint32_t x) {
    uint32_t p = 1;
    while ((p << 1) != 0 && (p << 1) <= x) p <<= 1;
    return p;
}

// number of lane-private copies of each bin
__host__ __device__ inline uint32_t count_nrep(uint32_t E) {
    uint32_t r = floor_pow2(kCountLdsWords / (E ? E : 1));
    return r > 64 ? 64 : (r ? r : 1);
}

struct CountPlan {
    uint32_t grid;
    uint64_t chunk;  // ids per workgroup (multiple of the 16-byte vector width)
};

inline CountPlan plan_count(uint64_t n, int id_bytes, int cus) {
    const uint64_t vec = 16 / id_bytes;
    const uint64_t min_ids = (uint64_t)kCountThreads * vec * 2;  // at least two vectors per thread
    uint64_t grid = (n + min_ids - 1) / min_ids;
    const uint64_t max_grid = (uint64_t)(cus > 0 ? cus : 256) * kCountBlocksPerCu;
    if (grid > max_grid) grid = max_grid;
    if (grid < 1) grid = 1;
    uint64_t chunk = (n + grid - 1) / grid;
    chunk = (chunk + vec - 1) / vec * vec;
    if (chunk == 0) chunk = vec;
    grid = (n + chunk - 1) / chunk;
    if (grid < 1) grid = 1;
    return CountPlan{(uint32_t)grid, chunk};
}

template <typename id_t>
__device__ __forceinline__ void count_one(id_t id, uint32_t E, uint32_t nrep_log2, uint32_t rep, uint32_t* bins) {
    // unsigned compare drops negative ids as well as ids >= E
    if ((uint64_t)id < (uint64_t)E) {
        __hip_atomic_fetch_add(&bins[((uint32_t)id << nrep_log2) + rep], 1u, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_WORKGROUP);
    }
}

template <typename id_t>
__global__ __launch_bounds__(kCountThreads) void continuous_count_kernel(const id_t* __restrict__ ids, uint64_t n,
                                                                         uint32_t E, uint32_t nrep_log2,
                                                                         uint64_t chunk,
                                                                         uint32_t* __restrict__ partials) {
    extern __shared__ uint32_t bins[];

    constexpr int VEC = 16 / sizeof(id_t);
    struct alignas(16) IdVec {
        id_t v[VEC];
    };

    const uint32_t tid = threadIdx.x;
    const uint32_t nrep = 1u << nrep_log2;
    const uint32_t rep = tid & (nrep - 1);
    const uint32_t words = E << nrep_log2;

    for (uint32_t i = tid; i < words; i += kCountThreads) bins[i] = 0;
    __syncthreads();

    const uint64_t lo = (uint64_t)blockIdx.x * chunk;
    uint64_t hi = lo + chunk;
    if (hi > n) hi = n;
    if (lo < hi) {
        const uint64_t len = hi - lo;
        const uint64_t nvec = len / VEC;
        const IdVec* vp = reinterpret_cast<const IdVec*>(ids + lo);
        uint64_t v = tid;
        // main loop: kCountUnroll independent 16-byte loads in flight per lane
        for (; v + (uint64_t)(kCountUnroll - 1) * kCountThreads < nvec; v += (uint64_t)kCountUnroll * kCountThreads) {
            IdVec r[kCountUnroll];
#pragma unroll
            for (int u = 0; u < kCountUnroll; ++u) {
                // streamed once: non-temporal loads keep the ids from displacing useful lines in L2 (measured
                // 14.3 us instead of 15.5 us per 64 MiB)
                typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
                const u32x4 raw =
                    __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(&vp[v + (uint64_t)u * kCountThreads]));
                r[u] = __builtin_bit_cast(IdVec, raw);
            }
#pragma unroll
            for (int u = 0; u < kCountUnroll; ++u) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) count_one<id_t>(r[u].v[j], E, nrep_log2, rep, bins);
            }
        }
        for (; v < nvec; v += kCountThreads) {
            IdVec r = vp[v];
#pragma unroll
            for (int j = 0; j < VEC; ++j) count_one<id_t>(r.v[j], E, nrep_log2, rep, bins);
        }
        const uint64_t tail = lo + nvec * VEC + tid;
        if (tail < hi) count_one<id_t>(ids[tail], E, nrep_log2, rep, bins);
    }
    __syncthreads();

    // fold the copies: tpb lanes share one bin, each sums nrep/tpb copies, then a butterfly inside the group
    uint32_t tpb = floor_pow2(kCountThreads / E ? kCountThreads / E : 1);
    if (tpb > nrep) tpb = nrep;
    if (tpb > (uint32_t)kWave) tpb = kWave;
    const uint32_t bins_per_pass = kCountThreads / tpb;
    const uint32_t sub = tid & (tpb - 1);
    uint32_t* my_row = partials + (uint64_t)blockIdx.x * E;
    for (uint32_t e0 = 0; e0 < E; e0 += bins_per_pass) {
        const uint32_t e = e0 + tid / tpb;
        uint32_t s = 0;
        if (e < E) {
            for (uint32_t r = sub; r < nrep; r += tpb) s += bins[(e << nrep_log2) + ((r + e) & (nrep - 1))];
        }
        for (uint32_t d = tpb >> 1; d > 0; d >>= 1) s += __shfl_xor(s, d, kWave);
        if (e < E && sub == 0) my_row[e] = s;
    }

}

// out[e] = sum over the `rows` workgroup histograms; one workgroup per 64 bins, 16 lanes-groups share the rows
constexpr int kReduceThreads = 1024;
constexpr int kReduceBins = 64;

__global__ __launch_bounds__(kReduceThreads) void count_reduce_kernel(const uint32_t* __restrict__ partials,
                                                                      uint32_t rows, uint32_t E,
                                                                      uint32_t* __restrict__ out) {
    __shared__ uint32_t s_sum[kReduceThreads];
    const uint32_t tid = threadIdx.x;
    const uint32_t e = blockIdx.x * kReduceBins + (tid % kReduceBins);
    const uint32_t part = tid / kReduceBins;
    constexpr uint32_t parts = kReduceThreads / kReduceBins;
    uint32_t s = 0;
    if (e < E) {
        // the rows are few and the latency of a load is what costs: all of a thread's rows (32 of them when two
        // workgroups per compute unit counted on 256 units) are requested before the first is added
        constexpr int kInFlight = 32;
        for (uint32_t b0 = part; b0 < rows; b0 += kInFlight * parts) {
            uint32_t r[kInFlight];
#pragma unroll
            for (int u = 0; u < kInFlight; ++u) {
                const uint32_t b = b0 + u * parts;
                r[u] = b < rows ? partials[(uint64_t)b * E + e] : 0u;
            }
#pragma unroll
            for (int u = 0; u < kInFlight; ++u) s += r[u];
        }
    }
    s_sum[tid] = s;
    __syncthreads();
    if (tid < kReduceBins && e < E) {
        uint32_t total = 0;
#pragma unroll
        for (uint32_t p = 0; p < parts; ++p) total += s_sum[p * kReduceBins + tid];
        out[e] = total;
    }
}

// ---- index construction ---------------------------------------------------------------------

constexpr int kIdxSteps = 8;                  // 64-slot steps per chunk
constexpr int kIdxChunk = kIdxSteps * kWave;  // 512 slots per wavefront
constexpr int kIdxWaves = 4;                  // wavefronts (= chunks) per workgroup
constexpr int kIdxThreads = kIdxWaves * kWave;
constexpr int kScanThreads = 1024;

template <typename id_t>
__device__ __forceinline__ int32_t load_id(const id_t* ids, int64_t s, int64_t R, uint32_t E) {
    if (s >= R) return -1;
    const id_t v = ids[s];
    return ((uint64_t)v < (uint64_t)E) ? (int32_t)v : -1;
}

// hist[c][e] = number of slots of chunk c routed to expert e
template <typename id_t>
__global__ __launch_bounds__(kIdxThreads) void index_hist_kernel(const id_t* __restrict__ ids, int64_t R, uint32_t E,
                                                                 uint32_t nchunks, uint32_t* __restrict__ hist) {
    extern __shared__ uint32_t lds[];
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = threadIdx.x / kWave;
    uint32_t* h = lds + wave * E;
    const uint32_t c = blockIdx.x * kIdxWaves + wave;
    for (uint32_t e = lane; e < E; e += kWave) h[e] = 0;
    __syncthreads();
    if (c < nchunks) {
        const int64_t base = (int64_t)c * kIdxChunk;
#pragma unroll
        for (int s = 0; s < kIdxSteps; ++s) {
            const int32_t id = load_id<id_t>(ids, base + s * kWave + lane, R, E);
            if (id >= 0) __hip_atomic_fetch_add(&h[id], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
    }
    __syncthreads();
    if (c < nchunks) {
        for (uint32_t e = lane; e < E; e += kWave) hist[(uint64_t)c * E + e] = h[e];
    }
}

// counts, inclusive offsets, and hist[c * rows][e] <- first output position of chunk c's slots of expert e.
// A chunk's histogram is the sum of `rows` consecutive rows of hist (the last chunk may have fewer: nrows in all).
__global__ __launch_bounds__(kScanThreads) void index_scan_kernel(uint32_t E, uint32_t nchunks, uint32_t rows,
                                                                  uint32_t nrows, uint32_t* hist,
                                                                  uint32_t* __restrict__ counts,
                                                                  uint32_t* __restrict__ offsets) {
    __shared__ uint32_t s_seg[kScanThreads];  // [part][e]
    __shared__ uint32_t s_start[FMA_MAX_GROUPS];
    __shared__ uint32_t s_wave_tot[kScanThreads / kWave];

    const uint32_t tid = threadIdx.x;
    const uint32_t parts = kScanThreads / E;  // E <= 1024 so parts >= 1
    const uint32_t e = tid % E;
    const uint32_t part = tid / E;
    const bool active = part < parts;
    const uint32_t seg = (nchunks + parts - 1) / parts;
    const uint32_t c_lo = part * seg;
    uint32_t c_hi = c_lo + seg;
    if (c_hi > nchunks) c_hi = nchunks;

    uint32_t s = 0;
    if (active) {
        const uint32_t r_lo = c_lo * rows;
        uint32_t r_hi = c_hi * rows;
        if (r_hi > nrows) r_hi = nrows;
        for (uint32_t r = r_lo; r < r_hi; ++r) s += hist[(uint64_t)r * E + e];
        s_seg[part * E + e] = s;
    }
    __syncthreads();

    // per-expert totals and exclusive prefix over the segments (thread e < E walks its column)
    uint32_t total = 0;
    if (tid < E) {
        for (uint32_t p = 0; p < parts; ++p) {
            const uint32_t v = s_seg[p * E + tid];
            s_seg[p * E + tid] = total;
            total += v;
        }
    }
    // block-wide inclusive scan of the totals over experts
    uint32_t incl = wave_inclusive_scan<uint32_t>(tid < E ? total : 0u);
    if ((tid & (kWave - 1)) == kWave - 1) s_wave_tot[tid / kWave] = incl;
    __syncthreads();
    if (tid < kWave) {
        const uint32_t nw = kScanThreads / kWave;
        uint32_t w = tid < nw ? s_wave_tot[tid] : 0u;
        w = wave_inclusive_scan<uint32_t>(w);
        if (tid < nw) s_wave_tot[tid] = w;
    }
    __syncthreads();
    if (tid >= kWave) incl += s_wave_tot[tid / kWave - 1];
    if (tid < E) {
        counts[tid] = total;
        offsets[tid] = incl;
        s_start[tid] = incl - total;
    }
    __syncthreads();

    if (active) {
        uint32_t running = s_start[e] + s_seg[part * E + e];
        for (uint32_t c = c_lo; c < c_hi; ++c) {
            const uint32_t r0 = c * rows;
            uint32_t r1 = r0 + rows;
            if (r1 > nrows) r1 = nrows;
            uint32_t v = 0;
            for (uint32_t r = r0; r < r1; ++r) v += hist[(uint64_t)r * E + e];
            hist[(uint64_t)r0 * E + e] = running;
            running += v;
        }
    }
}

// One wavefront per chunk walks its slots in order; lanes with the same expert id find each other with
// ballots, the lowest of them advances the expert's cursor, each takes cursor + its rank in the group.
// A chunk is chunk_slots <= STEPS * 64 consecutive slots; its cursors start at base[c * base_stride + e].
template <typename id_t, int STEPS>
__global__ __launch_bounds__(kIdxThreads) void index_place_kernel(const id_t* __restrict__ ids, int64_t R, uint32_t E,
                                                                  uint32_t nbits, uint32_t nchunks, uint32_t chunk_slots,
                                                                  uint64_t base_stride,
                                                                  const uint32_t* __restrict__ base,
                                                                  int32_t* __restrict__ perm, int32_t* __restrict__ eid,
                                                                  int32_t* __restrict__ inv) {
    extern __shared__ uint32_t lds[];
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = threadIdx.x / kWave;
    uint32_t* cur = lds + wave * E;
    const uint32_t c = blockIdx.x * kIdxWaves + wave;
    const bool live = c < nchunks;
    if (live) {
        for (uint32_t e = lane; e < E; e += kWave) cur[e] = base[(uint64_t)c * base_stride + e];
    }
    __syncthreads();
    if (!live) return;

    const int64_t first = (int64_t)c * chunk_slots;
    const int64_t end = first + chunk_slots < R ? first + chunk_slots : R;  // slots past the chunk read as "no id"
    int32_t id[STEPS];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) id[s] = load_id<id_t>(ids, first + s * kWave + lane, end, E);

    const uint64_t below = (1ull << lane) - 1ull;
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
        if (s * kWave >= (int)chunk_slots) break;
        const bool valid = id[s] >= 0;
        uint64_t mask = __ballot(valid);
        for (uint32_t b = 0; b < nbits; ++b) {
            const bool bit = (id[s] >> b) & 1;
            const uint64_t bal = __ballot(bit);
            mask &= bit ? bal : ~bal;
        }
        if (valid) {
            const uint32_t rank = __popcll(mask & below);
            const uint32_t old = cur[id[s]];
            if (rank == 0) cur[id[s]] = old + (uint32_t)__popcll(mask);
            const int32_t pos = (int32_t)(old + rank);
            const int64_t slot = first + s * kWave + lane;
            perm[pos] = (int32_t)slot;
            eid[pos] = id[s];
            inv[slot] = pos;
        }
    }
}

inline uint32_t index_nchunks(int64_t R) { return (uint32_t)((R + kIdxChunk - 1) / kIdxChunk); }

int check_build_index(const void* ids, int id_bytes, int64_t R, int64_t E, uint32_t* counts, uint32_t* offsets,
                      int32_t* perm, int32_t* eid, int32_t* inv) {
    FMA_REQUIRE(id_bytes == 4 || id_bytes == 8, FMA_ERR_BAD_DTYPE,
                "moe_build_index: ids must be int32 or int64 (id_bytes=%d)", id_bytes);
    FMA_REQUIRE(E >= 1, FMA_ERR_BAD_SIZE, "moe_build_index: E must be >= 1 (got %lld)", (long long)E);
    FMA_REQUIRE(E <= FMA_MAX_GROUPS, FMA_ERR_TOO_MANY_EXPERTS, "moe_build_index: E=%lld exceeds the limit %d",
                (long long)E, FMA_MAX_GROUPS);
    FMA_REQUIRE(R >= 0, FMA_ERR_BAD_SIZE, "moe_build_index: negative slot count %lld", (long long)R);
    FMA_REQUIRE(R <= 0x7fffffffll, FMA_ERR_TOO_MANY_ELEMENTS, "moe_build_index: R=%lld exceeds 2^31-1", (long long)R);
    FMA_REQUIRE(counts && offsets, FMA_ERR_NULL_POINTER, "moe_build_index: counts/offsets is NULL");
    FMA_REQUIRE(R == 0 || (ids && perm && eid && inv), FMA_ERR_NULL_POINTER,
                "moe_build_index: ids/perm/eid/inv is NULL");
    return FMA_OK;
}

// the three launches of the counting sort; hist: nchunks * E words of scratch (every word is written before it is read)
int launch_build_index(const void* ids, int id_bytes, int64_t R, int64_t E, uint32_t* counts, uint32_t* offsets,
                       int32_t* perm, int32_t* eid, int32_t* inv, uint32_t* hist, hipStream_t st) {
    const uint32_t nchunks = index_nchunks(R);
    const uint32_t blocks = (nchunks + kIdxWaves - 1) / kIdxWaves;
    const size_t lds_bytes = (size_t)kIdxWaves * E * 4;
    uint32_t nbits = 0;
    while ((1ll << nbits) < E) ++nbits;

    if (nchunks > 0) {
        if (id_bytes == 4)
            hipLaunchKernelGGL(index_hist_kernel<int32_t>, dim3(blocks), dim3(kIdxThreads), lds_bytes, st,
                               (const int32_t*)ids, R, (uint32_t)E, nchunks, hist);
        else
            hipLaunchKernelGGL(index_hist_kernel<int64_t>, dim3(blocks), dim3(kIdxThreads), lds_bytes, st,
                               (const int64_t*)ids, R, (uint32_t)E, nchunks, hist);
        int rc = launch_status("moe_build_index(hist)");
        if (rc) return rc;
    }
    hipLaunchKernelGGL(index_scan_kernel, dim3(1), dim3(kScanThreads), 0, st, (uint32_t)E, nchunks, 1u, nchunks, hist,
                       counts, offsets);
    int rc = launch_status("moe_build_index(scan)");
    if (rc) return rc;
    if (nchunks > 0) {
        if (id_bytes == 4)
            hipLaunchKernelGGL((index_place_kernel<int32_t, kIdxSteps>), dim3(blocks), dim3(kIdxThreads), lds_bytes, st,
                               (const int32_t*)ids, R, (uint32_t)E, nbits, nchunks, (uint32_t)kIdxChunk, (uint64_t)E,
                               hist, perm, eid, inv);
        else
            hipLaunchKernelGGL((index_place_kernel<int64_t, kIdxSteps>), dim3(blocks), dim3(kIdxThreads), lds_bytes, st,
                               (const int64_t*)ids, R, (uint32_t)E, nbits, nchunks, (uint32_t)kIdxChunk, (uint64_t)E,
                               hist, perm, eid, inv);
        rc = launch_status("moe_build_index(place)");
    }
    return rc;
}

// The same sort from histograms the caller already has: hist[r][e] = number of slots of the r-th block of
// 16 * top_k consecutive slots (16 tokens) that go to expert e. Two launches: scan and placement. A chunk of the
// placement is `rows` consecutive blocks, about 512 slots.
int launch_build_index_from_hist(const int32_t* ids, int64_t R, int64_t E, int64_t top_k, uint32_t* counts,
                                 uint32_t* offsets, int32_t* perm, int32_t* eid, int32_t* inv, uint32_t* hist,
                                 hipStream_t st) {
    const int64_t block_slots = 16 * top_k;
    const uint32_t nrows = (uint32_t)((R + block_slots - 1) / block_slots);
    const uint32_t rows = (uint32_t)(block_slots >= kIdxChunk ? 1 : kIdxChunk / block_slots);
    const uint32_t chunk_slots = (uint32_t)(rows * block_slots);  // <= 1024 (top_k <= 64)
    const uint32_t nchunks = (nrows + rows - 1) / rows;
    const uint32_t blocks = (nchunks + kIdxWaves - 1) / kIdxWaves;
    const size_t lds_bytes = (size_t)kIdxWaves * E * 4;
    uint32_t nbits = 0;
    while ((1ll << nbits) < E) ++nbits;
    hipLaunchKernelGGL(index_scan_kernel, dim3(1), dim3(kScanThreads), 0, st, (uint32_t)E, nchunks, rows, nrows, hist,
                       counts, offsets);
    int rc = launch_status("moe_build_index_from_hist(scan)");
    if (rc || nchunks == 0) return rc;
    if (chunk_slots <= kIdxSteps * kWave)
        hipLaunchKernelGGL((index_place_kernel<int32_t, kIdxSteps>), dim3(blocks), dim3(kIdxThreads), lds_bytes, st, ids, R,
                           (uint32_t)E, nbits, nchunks, chunk_slots, (uint64_t)rows * (uint64_t)E, hist, perm, eid, inv);
    else
        hipLaunchKernelGGL((index_place_kernel<int32_t, 2 * kIdxSteps>), dim3(blocks), dim3(kIdxThreads), lds_bytes, st, ids,
                           R, (uint32_t)E, nbits, nchunks, chunk_slots, (uint64_t)rows * (uint64_t)E, hist, perm, eid, inv);
    return launch_status("moe_build_index_from_hist(place)");
}

// Address of `scratch` on the current device, looked up once per device (each GPU holds its own copy of the array at
// its own address). Only this pointer is ever handed to kernels.
constexpr int kMaxDevices = 64;
int static_scratch(uint32_t** out) {
    static std::mutex mu;
    static uint32_t* ptrs[kMaxDevices] = {};
    int dev = -1;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) return fail((int)err, "moe_build_index_static: hipGetDevice: %s", hipGetErrorString(err));
    FMA_REQUIRE(dev >= 0 && dev < kMaxDevices, FMA_ERR_UNSUPPORTED, "moe_build_index_static: device index %d", dev);
    std::lock_guard<std::mutex> lock(mu);
    if (!ptrs[dev]) {
        void* p = nullptr;
        err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (err != hipSuccess || !p)
            return fail(err != hipSuccess ? (int)err : FMA_ERR_NULL_POINTER,
                        "moe_build_index_static: hipGetSymbolAddress(scratch): %s", hipGetErrorString(err));
        ptrs[dev] = (uint32_t*)p;
    }
    *out = ptrs[dev];
    return FMA_OK;
}

}  // namespace
}  // namespace fmahip

extern "C" {

int64_t fma_continuous_count_workspace_bytes(int64_t n, int64_t E) {
    if (n < 0 || E < 1) return 0;
    // independent of id width and device: sized for the largest grid any call may use
    const int cus = fmahip::num_compute_units();
    const int64_t max_grid = (int64_t)(cus > 0 ? cus : 256) * fmahip::kCountBlocksPerCu;
    return max_grid * E * 4;
}

int fma_continuous_count(const void* ids, int id_bytes, int64_t n, uint32_t* counts, int64_t E, void* workspace,
                         int64_t workspace_bytes, void* stream) {
    using namespace fmahip;
    FMA_REQUIRE(id_bytes == 4 || id_bytes == 8, FMA_ERR_BAD_DTYPE,
                "continuous_count: ids must be int32 or int64 (id_bytes=%d)", id_bytes);
    FMA_REQUIRE(E >= 1, FMA_ERR_BAD_SIZE, "continuous_count: E must be >= 1 (got %lld)", (long long)E);
    FMA_REQUIRE(E <= FMA_MAX_COUNT_BINS, FMA_ERR_TOO_MANY_EXPERTS, "continuous_count: E=%lld exceeds the limit %d",
                (long long)E, FMA_MAX_COUNT_BINS);
    FMA_REQUIRE(n >= 0, FMA_ERR_BAD_SIZE, "continuous_count: negative element count %lld", (long long)n);
    FMA_REQUIRE((uint64_t)n <= 0xffffffffull, FMA_ERR_TOO_MANY_ELEMENTS,
                "continuous_count: n=%lld exceeds 2^32-1", (long long)n);
    FMA_REQUIRE(counts != nullptr, FMA_ERR_NULL_POINTER, "continuous_count: counts is NULL");
    FMA_REQUIRE(ids != nullptr || n == 0, FMA_ERR_NULL_POINTER, "continuous_count: ids is NULL");
    FMA_REQUIRE(workspace != nullptr, FMA_ERR_NULL_POINTER, "continuous_count: workspace is NULL");
    FMA_REQUIRE(aligned16(ids), FMA_ERR_MISALIGNED, "continuous_count: ids must be 16-byte aligned");
    FMA_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 3u) == 0, FMA_ERR_MISALIGNED,
                "continuous_count: workspace must be 4-byte aligned");

    const int cus = num_compute_units();
    const CountPlan plan = plan_count((uint64_t)n, id_bytes, cus);
    const int64_t need = (int64_t)plan.grid * E * 4;
    FMA_REQUIRE(workspace_bytes >= need, FMA_ERR_WORKSPACE_TOO_SMALL,
                "continuous_count: workspace of %lld bytes is smaller than the %lld needed", (long long)workspace_bytes,
                (long long)need);

    const uint32_t nrep = count_nrep((uint32_t)E);
    uint32_t nrep_log2 = 0;
    while ((1u << nrep_log2) < nrep) ++nrep_log2;
    const size_t lds_bytes = (size_t)E * nrep * 4;
    hipStream_t st = (hipStream_t)stream;
    if (id_bytes == 4) {
        hipLaunchKernelGGL(continuous_count_kernel<int32_t>, dim3(plan.grid), dim3(kCountThreads), lds_bytes, st,
                           (const int32_t*)ids, (uint64_t)n, (uint32_t)E, nrep_log2, plan.chunk, (uint32_t*)workspace);
    } else {
        hipLaunchKernelGGL(continuous_count_kernel<int64_t>, dim3(plan.grid), dim3(kCountThreads), lds_bytes, st,
                           (const int64_t*)ids, (uint64_t)n, (uint32_t)E, nrep_log2, plan.chunk, (uint32_t*)workspace);
    }
    int rc = launch_status("continuous_count");
    if (rc) return rc;
    hipLaunchKernelGGL(count_reduce_kernel, dim3((uint32_t)((E + kReduceBins - 1) / kReduceBins)), dim3(kReduceThreads),
                       0, st, (const uint32_t*)workspace, plan.grid, (uint32_t)E, counts);
    return launch_status("continuous_count(reduce)");
}

int64_t fma_moe_build_index_workspace_bytes(int64_t R, int64_t E) {
    if (R < 0 || E < 1) return 0;
    const int64_t nchunks = fmahip::index_nchunks(R);
    return (nchunks > 0 ? nchunks : 1) * E * 4;
}

int fma_moe_build_index(const void* ids, int id_bytes, int64_t R, int64_t E, uint32_t* counts, uint32_t* offsets,
                        int32_t* perm, int32_t* eid, int32_t* inv, void* workspace, int64_t workspace_bytes,
                        void* stream) {
    using namespace fmahip;
    int rc = check_build_index(ids, id_bytes, R, E, counts, offsets, perm, eid, inv);
    if (rc) return rc;
    FMA_REQUIRE(workspace != nullptr, FMA_ERR_NULL_POINTER, "moe_build_index: workspace is NULL");
    const int64_t need = fma_moe_build_index_workspace_bytes(R, E);
    FMA_REQUIRE(workspace_bytes >= need, FMA_ERR_WORKSPACE_TOO_SMALL,
                "moe_build_index: workspace of %lld bytes is smaller than the %lld needed", (long long)workspace_bytes,
                (long long)need);
    return launch_build_index(ids, id_bytes, R, E, counts, offsets, perm, eid, inv, (uint32_t*)workspace,
                              (hipStream_t)stream);
}

int fma_moe_build_index_from_hist(const int32_t* ids, int64_t R, int64_t E, int64_t top_k, uint32_t* token_block_hist,
                                  uint32_t* counts, uint32_t* offsets, int32_t* perm, int32_t* eid, int32_t* inv,
                                  void* stream) {
    using namespace fmahip;
    int rc = check_build_index(ids, 4, R, E, counts, offsets, perm, eid, inv);
    if (rc) return rc;
    FMA_REQUIRE(top_k >= 1 && top_k <= 64 && R % top_k == 0, FMA_ERR_BAD_SIZE,
                "moe_build_index_from_hist: top_k must lie in [1, 64] and divide R (top_k=%lld, R=%lld)",
                (long long)top_k, (long long)R);
    FMA_REQUIRE(R == 0 || token_block_hist, FMA_ERR_NULL_POINTER, "moe_build_index_from_hist: the histogram is NULL");
    return launch_build_index_from_hist(ids, R, E, top_k, counts, offsets, perm, eid, inv, token_block_hist,
                                        (hipStream_t)stream);
}

int64_t fma_moe_build_index_static_max_words(void) {
    // The first call on a device looks the array's address up (hipGetSymbolAddress, under a mutex). Doing it here, where a
    // caller asks for the limit before its first build, keeps that lookup out of a stream capture; the result is ignored
    // (a failure is reported by the build itself).
    uint32_t* unused = nullptr;
    (void)fmahip::static_scratch(&unused);
    return FMA_STATIC_INDEX_WORDS;
}

int fma_moe_build_index_static(const void* ids, int id_bytes, int64_t R, int64_t E, uint32_t* counts, uint32_t* offsets,
                               int32_t* perm, int32_t* eid, int32_t* inv, void* stream) {
    using namespace fmahip;
    int rc = check_build_index(ids, id_bytes, R, E, counts, offsets, perm, eid, inv);
    if (rc) return rc;
    const int64_t need = fma_moe_build_index_workspace_bytes(R, E);
    FMA_REQUIRE(need <= (int64_t)FMA_STATIC_INDEX_WORDS * 4, FMA_ERR_WORKSPACE_TOO_SMALL,
                "moe_build_index_static: R=%lld slots with E=%lld experts need %lld bytes of scratch, the built-in "
                "array holds %lld (use fma_moe_build_index with a workspace)",
                (long long)R, (long long)E, (long long)need, (long long)FMA_STATIC_INDEX_WORDS * 4);
    uint32_t* hist = nullptr;
    rc = static_scratch(&hist);
    if (rc) return rc;
    return launch_build_index(ids, id_bytes, R, E, counts, offsets, perm, eid, inv, hist, (hipStream_t)stream);
}

}  // extern "C"
