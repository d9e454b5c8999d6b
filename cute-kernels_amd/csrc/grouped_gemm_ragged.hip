// Grouped GEMM for launches whose groups differ in ONE dimension (every grouped GEMM of an MoE layer: rows per expert
// in forward and input gradient, reduction length per expert in the weight gradient) for gfx950: bf16 or fp16 operands,
// fp32 accumulation on the matrix cores, optional SwiGLU epilogue. The tile kernel of grouped_gemm.hip (256x256x64
// tiles, eight wavefronts, two LDS stages filled by direct global -> LDS loads, the same LDS layouts) with another
// matrix instruction and a different tile boundary:
//
//  * The products are 16x16x32 instructions (v_mfma_f32_16x16x32), not 32x32x16: the same arithmetic rate per
//    instruction cycle, but the part holds a higher clock on them. Measured on N(0,1) operands: a loop of nothing but
//    matrix instructions sustains 0.79 of the peak rate against 0.70, and this kernel ran 3.5 to 6 % faster on the
//    Mixtral-shape layer's GEMMs than the same kernel on 32x32x16. A wavefront's 128 x 64 sub-tile is 8 x 4 blocks; a K
//    step is two 32-wide slices, each worked through in four phases of two row blocks (see the K loop).
//  * With two dimensions known on the host, a group's operand offsets follow from one 32-bit prefix of the varying
//    dimension, so the group table takes 10 bytes per group instead of 30. The LDS that frees (16 KB) is a staging
//    buffer of its own for the epilogue, which therefore no longer needs a piece of an operand stage.
//  * The operand loads run as ONE stream over the tile sequence: the load slots of a tile's last two K steps carry the
//    first two K steps of the NEXT tile (the loaders of both tiles are kept, a scalar select picks one per step), so that
//    when a tile's K loop ends the next tile's first step is already in LDS and its second on the way. The tile boundary
//    is then the epilogue alone: no loader set-up, no burst of 16 loads per wavefront competing with the 16 stores for the
//    compute unit's one address path, no wait for first operands, no barrier.
//  * The epilogue's stores stay outstanding across the start of the next tile: they are issued after that tile's first
//    loads, and loads and stores of a wavefront complete in issue order, so the first K step waits for "all but the
//    stores and the newest prefetch" (an exact count) and the second for everything, two K steps after the stores went out.
//  * A K loop always runs an even number of steps (a step of zeros is appended to an odd reduction length), so every tile
//    starts in LDS stage 0 and the loop body stays two straight-line steps.
//  * Tiles that break the pattern (groups of at most 64 rows on their three-stage loop, groups without reduction, groups
//    that need the element-wise path) start cold: the tile before them lets its last two load slots fetch nothing and
//    drains, and they issue their first loads themselves, followed by as many stores outside every buffer as an epilogue
//    issues, so that the waits of the K loop are the same constants in both cases.
//  * Two kinds of kernels read one operand through an index instead of a packed copy (GATHER): the forward product takes
//    the rows of A as rows row_index[i] / divisor of the token matrix (a table of the tile's 256 entries in LDS, four
//    per-lane offsets per K step), the weight gradient takes the reduction rows of B the same way (eight entries per
//    wavefront and K step, requested two steps ahead). Both give the bits of the packed kernel on a gathered copy.
#include "gemm_parts.h"

namespace fmahip {
namespace gemm {
namespace ragged {

constexpr uint32_t kPfDist = 4;     // K steps between a line's prefetch and the step that loads it
constexpr int kBwdAhead = 2;        // passes of the SwiGLU-gradient epilogue whose h values are requested ahead
constexpr uint32_t kStreamOutSteps = 16;  // weight-gradient tiles of at most this many K steps store with the non-temporal hint

constexpr int NWM = 2, NWN = 4, NW = NWM * NWN, NT = NW * 64;
constexpr int WM = BM / NWM, WN = BN / NWN;  // 128 x 64 per wavefront
constexpr int RB = WM / 16, CB = WN / 16;    // 8 x 4 accumulator blocks of 16 x 16 (the 16x16x32 matrix instruction)
constexpr int kStageBytes = 2048;            // epilogue staging per wavefront: 16 rows of 128 bytes or 32 rows of 64

struct Args {
    const uint16_t* A;
    const uint16_t* B;
    uint16_t* D;            // plain: output; swiglu: pre-activation h (may be NULL)
    uint16_t* ACT;          // swiglu only: activation output
    const uint32_t* sizes;  // E values of the varying dimension
    const uint16_t* bias;   // BIAS kernels: [E, n] added to the rounded product before anything else
    const uint16_t* h_in;   // EPI_SWIGLU_BWD: the packed pre-activation [rows, 2 n] whose gradient goes to D
    // GATHER kernels, rows vary: row i of the packed A operand is row row_index[i] / divisor of A, which has a_rows rows.
    // GATHER kernels, reduction varies (weight gradient): reduction row i of the packed B operand is row
    // row_index[i] / divisor of B, which has a_rows rows of n elements.
    const int32_t* row_index;
    uint32_t divisor, a_rows;
    uint32_t E;
    uint32_t m, n, k;  // the dimensions all groups share (the varying one is ignored)
    float alpha;
    // fma_grouped_gemm (per-group M, N and K arrays in device memory): when n_dev is set, the shared dimensions are the
    // first entries of the arrays, and the kernel runs only if the launch has its form (see the top of the kernel)
    const uint32_t* m_dev;
    const uint32_t* n_dev;
    const uint32_t* k_dev;
};

// s_waitcnt immediate: vmcnt(vm), and lgkmcnt(0) too if lgkm0 (expcnt untouched)
constexpr int waitcnt_imm(int vm, bool lgkm0) {
    return (vm & 15) | ((vm >> 4) << 14) | (7 << 4) | ((lgkm0 ? 0 : 15) << 8);
}

// The per-tile part of a loader's state (everything else depends on lane, wavefront and the shared dimensions only)
template <bool KC>
struct Feed {
    const uint16_t* base0;
    const uint16_t* base1;  // second row range of a split [row][k] tile
    uint32_t extent;        // [row][k] tile: valid bytes from a base; [k][out] tile: reduction length
    uint32_t ldb;           // row pitch of the operand in bytes
    uint32_t col_bytes;     // [k][out] tile: byte offset of the tile's first column inside a row
};


// Names an accumulator value as one 16-register value (no instruction, no ordering).
__device__ __forceinline__ void anchor_value(f32x16& c) { asm("" : "+v"(c)); }

template <typename EL, bool A_KC, bool B_KC, int EPI, bool VARY_K, bool BIAS, bool GATHER_ANY>
__global__ __launch_bounds__(NT) void ragged_gemm_kernel(const Args args) {
    // GATHER: the rows of A are picked through row_index (forward); kGatherK: the reduction rows of B are (weight gradient)
    constexpr bool GATHER = GATHER_ANY && !VARY_K;
    constexpr bool kGatherK = GATHER_ANY && VARY_K;
    // kGlu: a forward SwiGLU epilogue (the tile holds 128 "up" and 128 "gate" columns of the product)
    constexpr bool kGlu = EPI == EPI_SWIGLU || EPI == EPI_SWIGLU_ACT;
    static_assert(!kGlu || (A_KC && B_KC && !VARY_K), "the SwiGLU epilogue exists for the NT layout only");
    static_assert(EPI != EPI_SWIGLU_BWD || (A_KC && !B_KC && !VARY_K && !BIAS && !GATHER_ANY),
                  "the SwiGLU-gradient epilogue exists for the input-gradient (NN) layout only");
    static_assert(!BIAS || (A_KC && B_KC && !VARY_K), "the bias term exists for the forward (NT) layout only");
    static_assert(!GATHER || (A_KC && B_KC), "rows are gathered in the forward (NT) layout only");
    static_assert(!kGatherK || (!A_KC && !B_KC && EPI == EPI_PLAIN), "reduction rows are gathered in the weight-gradient (TN) layout only");

    // one array per stage and operand: distinct LDS objects let the compiler see that a direct-to-LDS load
    // into one stage cannot alias the fragment reads of the other, so it does not wait for the load first
    __shared__ __attribute__((aligned(1024))) uint8_t s_a0[kTileBytes];
    __shared__ __attribute__((aligned(1024))) uint8_t s_b0[kTileBytes];
    __shared__ __attribute__((aligned(1024))) uint8_t s_a1[kTileBytes];
    __shared__ __attribute__((aligned(1024))) uint8_t s_b1[kTileBytes];
    __shared__ __attribute__((aligned(1024))) uint8_t s_stage[NW * kStageBytes];
    __shared__ uint32_t s_pf[64];  // where the dwords fetched by the L2 prefetch end up (never read)
    // BIAS: per wavefront, the bias values of its own 64 columns (plain) or 32 "up" | 32 "gate" columns
    constexpr int kBiasBytes = 128;
    __shared__ __attribute__((aligned(256))) uint8_t s_bias[BIAS ? NW * kBiasBytes : 16];
    // GATHER: the row_index entries of the 256 rows of a tile, for the tile of round r in half r % 2. Filled by
    // direct-to-LDS loads and read in assembly: the compiler never sees an access to it.
    __shared__ __attribute__((aligned(256))) uint32_t s_rows[GATHER ? 512 : 4];
    // kGatherK: row_index entries on their way from one tile's last two steps (or a cold start) to the next tile's first two:
    // per LDS stage and wavefront the 64 dwords of one direct-to-LDS load. Read in assembly only.
    __shared__ __attribute__((aligned(256))) uint32_t s_gk[kGatherK ? 2 * NW * 64 : 4];
    // The group table, one LDS object: first tile of the group at position p of the tile sequence, exclusive prefix of the
    // varying dimension over the groups, and which group is at position p.
    __shared__ uint32_t s_table[2 * (FMA_MAX_GROUPS + 1) + FMA_MAX_GROUPS / 2];
    uint32_t* const s_tile_start = s_table;
    uint32_t* const s_prefix = s_table + (FMA_MAX_GROUPS + 1);
    uint16_t* const s_order = reinterpret_cast<uint16_t*>(s_table + 2 * (FMA_MAX_GROUPS + 1));

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t wm = wave / NWN;
    const uint32_t wn = wave % NWN;
    const uint32_t E = args.E;

    // The dimensions all groups share. Called with per-group arrays of all three dimensions (fma_grouped_gemm), the kernel
    // first looks whether the launch has its form: rows vary -> N and K the same for every group; reduction varies -> M and
    // N the same and K not (when all three are the same the rows-vary kernel runs). If not, it leaves the launch to the
    // kernel launched beside it: the three kernels of fma_grouped_gemm agree on one of them without a word to the host.
    uint32_t dim_m = args.m, dim_n = args.n, dim_k = args.k;
    if (args.n_dev) {
        typedef const __attribute__((address_space(4))) uint32_t* const_dim_ptr;
        const const_dim_ptr ma = (const_dim_ptr)args.m_dev, na = (const_dim_ptr)args.n_dev, ka = (const_dim_ptr)args.k_dev;
        dim_m = ma[0];
        dim_n = na[0];
        dim_k = ka[0];
        bool m_differs = false, n_differs = false, k_differs = false;
        for (uint32_t e = tid; e < E; e += NT) {
            m_differs = m_differs || args.m_dev[e] != dim_m;
            n_differs = n_differs || args.n_dev[e] != dim_n;
            k_differs = k_differs || args.k_dev[e] != dim_k;
        }
        const bool m_same = !__syncthreads_or(m_differs), n_same = !__syncthreads_or(n_differs), k_same = !__syncthreads_or(k_differs);
        const bool mine = VARY_K ? (m_same && n_same && !k_same) : (n_same && k_same);
        if (!mine) return;
    }

    // The compiler orders LDS accesses behind direct-to-LDS loads in flight per LDS object: an access to an object that
    // some load has written waits for the loads into THAT object only, an access to an object no load has ever written
    // waits for all of them. The group table is read while the next tile's operand loads are in flight, so it gets
    // one load that fetches nothing, here, to be known as an object of its own.
    {
        const __amdgpu_buffer_rsrc_t nowhere = make_rsrc(args.A, 0u);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(nowhere, (lds_void*)s_table, 4, kOutOfRange, 0, 0, 0);
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, false));
        __syncthreads();
    }

    // The size array is read through the constant address space: with a wavefront-uniform index that is a scalar load
    // (nothing writes the array while the kernel runs), not a vector load that every tile would wait for.
    typedef const __attribute__((address_space(4))) uint32_t* const_u32_ptr;
    const const_u32_ptr sizes = (const_u32_ptr)args.sizes;
    auto group_m = [&](uint32_t e) { return VARY_K ? dim_m : sizes[e]; };
    auto group_k = [&](uint32_t e) { return VARY_K ? sizes[e] : dim_k; };
    const uint32_t Ne = dim_n;
    constexpr bool kCanNarrow = A_KC && B_KC;
    constexpr uint32_t kTileN = kGlu ? BN / 2 : BN;  // columns of the tile grid one tile covers
    const uint32_t n_span = kGlu ? Ne / 2 : Ne;      // columns the tile grid runs over
    bool narrow = false;
    auto tiles_of = [&](uint32_t m) -> uint32_t {
        if (m == 0 || Ne == 0) return 0;
        const uint32_t width = (kCanNarrow && narrow && m <= 64u) ? kTileN / 2 : kTileN;
        return ((m + BM - 1) / BM) * ((n_span + width - 1) / width);
    };

    // ---- order of the groups in the tile sequence: by K steps per tile, longest first (see grouped_gemm.hip) ----
    {
        uint32_t* const key = reinterpret_cast<uint32_t*>(s_a0);  // K steps per tile of group e; 0 if it has no tiles
        const uint32_t key0 = tiles_of(group_m(0)) ? (group_k(0) + BK - 1) / BK : 0u;
        bool differs = false;
        for (uint32_t e = tid; e < E; e += NT) {
            const uint32_t k = tiles_of(group_m(e)) ? (group_k(e) + BK - 1) / BK : 0u;
            key[e] = k;
            differs = differs || k != key0;
        }
        if (__syncthreads_or(differs)) {
            for (uint32_t e = tid; e < E; e += NT) {
                const uint32_t mine = key[e];
                uint32_t rank = 0;
                for (uint32_t j = 0; j < E; ++j) {
                    const uint32_t other = key[j];
                    rank += (other > mine || (other == mine && j < e)) ? 1u : 0u;
                }
                s_order[rank] = (uint16_t)e;
            }
        } else {
            for (uint32_t e = tid; e < E; e += NT) s_order[e] = (uint16_t)e;
        }
        __syncthreads();
    }

    if constexpr (kCanNarrow) {
        // half-width column tiles for groups of at most 64 rows when that fills the workgroups better (grouped_gemm.hip)
        uint32_t mine_small = 0, mine_other = 0;
        for (uint32_t e = tid; e < E; e += NT) {
            const uint32_t m = group_m(e), t = tiles_of(m);
            if (m <= 64u) mine_small += t;
            else mine_other += t;
        }
        uint32_t* const total = reinterpret_cast<uint32_t*>(s_a0);
        if (tid < 2) total[tid] = 0;
        __syncthreads();
        if (mine_small) atomicAdd(total, mine_small);
        if (mine_other) atomicAdd(total + 1, mine_other);
        __syncthreads();
        const uint32_t t_small = uniform(total[0]), t_other = uniform(total[1]), g = gridDim.x;
        const uint32_t rounds = (t_small + t_other + g - 1) / g;
        const uint32_t half_rounds = (2 * t_small + g - 1) / g;
        narrow = t_other == 0 ? half_rounds * 10u <= 2u * rounds * 9u : (t_small + t_other) * 2u <= g;
        __syncthreads();
    }

    // ---- group table, built by wavefront 0: exclusive prefix of tiles over the order above, exclusive prefix of the
    // varying dimension over the groups as they lie in memory ----
    if (wave == 0) {
        uint32_t carry_t = 0, carry_s = 0;
        for (uint32_t base = 0; base < E; base += 64) {
            const uint32_t e = base + lane;
            uint32_t sz = 0, t = 0;
            if (e < E) {
                sz = sizes[e];
                t = tiles_of(group_m(s_order[e]));  // the group at position e of the tile sequence
            }
            const uint32_t it = wave_inclusive_scan<uint32_t>(t);
            const uint32_t is = wave_inclusive_scan<uint32_t>(sz);
            if (e < E) {
                s_tile_start[e] = carry_t + it - t;
                s_prefix[e] = carry_s + is - sz;
            }
            carry_t += __shfl(it, 63, 64);
            carry_s += __shfl(is, 63, 64);
        }
        if (lane == 0) {
            s_tile_start[E] = carry_t;
            s_prefix[E] = carry_s;
        }
    }
    __syncthreads();
    const uint32_t total_tiles = s_tile_start[E];

    // first tile row of B fragment j (16 rows) of this wavefront
    auto b_frag_row = [&](int j) -> uint32_t {
        if constexpr (kGlu) {
            return j < CB / 2 ? wn * (WN / 2) + j * 16 : BN / 2 + wn * (WN / 2) + (j - CB / 2) * 16;
        } else {
            return wn * WN + j * 16;
        }
    };
    // per-lane LDS byte offsets of this wavefront's fragments for k slice 0 of the two 32-wide slices of a K step
    // (slice 1 adds a constant). A fragment is 16 rows: lane l holds row l % 16, k 8 (l / 16) .. + 7 of the slice.
    uint32_t a_off[RB], b_off[CB];
#pragma unroll
    for (int i = 0; i < RB; ++i) {
        const uint32_t r0 = wm * WM + i * 16;
        a_off[i] = A_KC ? r0 * kRowBytes : mc_frag_off16(r0, lane);
    }
#pragma unroll
    for (int j = 0; j < CB; ++j) {
        const uint32_t r0 = b_frag_row(j);
        b_off[j] = B_KC ? r0 * kRowBytes : mc_frag_off16(r0, lane);
    }
    uint32_t kc_slice[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) kc_slice[ks] = kc_off(lane & 15u, (uint32_t)ks * 4u + (lane >> 4));
    constexpr uint32_t kSliceT = 32 * kTRowBytes;  // from slice 0 to slice 1 in a [k][out] tile

    // workgroup id -> position in the round of gridDim.x tiles: workgroups of one XCD take 32 neighbours
    const uint32_t grid = gridDim.x;
    const uint32_t per_xcd = grid / kXcds;
    const uint32_t slot = (grid % kXcds == 0) ? (blockIdx.x % kXcds) * per_xcd + blockIdx.x / kXcds : blockIdx.x;

    // Everything that identifies one output tile; the same in every lane.
    struct Tile {
        bool valid, fast;
        uint32_t Me, Ke, m0, n0, n_lim;  // n_lim: first column past the tile (kTileN columns wide, or half of that)
        uint32_t e;                      // the group
        uint32_t row0;                   // first packed row (reduction row, if the reduction varies) of the group
        uint64_t off_a, off_b, off_d;
        uint32_t pf_r, pf_c;  // position of the tile in its XCD's 8 x 4 block of tiles (row, column)
    };
    auto lookup = [&](uint32_t round) -> Tile {
        Tile t{};
        const uint32_t v = round * grid + ((round & 1u) ? grid - 1u - slot : slot);
        if ((uint64_t)round * grid >= total_tiles || v >= total_tiles) return t;
        // position of the group that holds tile v: the number of groups whose tiles end at or before v. Every lane
        // compares one table entry per 64 groups and a ballot counts them (a binary search would be ten dependent LDS
        // round trips for 1024 groups; this is one per 64 groups, issued back to back).
        uint32_t groups_before = 0;
        for (uint32_t base = 0; base < E; base += 64u) {
            const uint32_t p = base + lane;
            const bool ends_before = p < E && s_tile_start[p + 1] <= v;
            groups_before += (uint32_t)__builtin_popcountll(__ballot(ends_before));
        }
        const uint32_t pos = uniform(groups_before);
        const uint32_t e = uniform((uint32_t)s_order[pos]);
        t.valid = true;
        t.e = e;
        t.Me = group_m(e);
        t.Ke = group_k(e);
        const uint32_t tiles_m = (t.Me + BM - 1) / BM;
        const uint32_t tile_n = (kCanNarrow && narrow && t.Me <= 64u) ? kTileN / 2 : kTileN;
        const uint32_t tiles_n = (n_span + tile_n - 1) / tile_n;
        const uint32_t local = v - uniform(s_tile_start[pos]);
        const uint32_t band = kGroupM * tiles_n;
        const uint32_t first_m = (local / band) * kGroupM;
        const uint32_t band_m = tiles_m - first_m < (uint32_t)kGroupM ? tiles_m - first_m : (uint32_t)kGroupM;
        const uint32_t mt = first_m + (local % band) % band_m;
        const uint32_t nt = (local % band) / band_m;
        t.pf_r = (local % band) % band_m;
        t.pf_c = nt & 3u;
        t.m0 = mt * BM;
        t.n0 = nt * tile_n;
        t.n_lim = n_span - t.n0 < tile_n ? n_span : t.n0 + tile_n;
        // packed element offsets of the group: the varying dimension's prefix times the other dimension of the operand
        const uint64_t before = uniform(s_prefix[e]);
        t.row0 = (uint32_t)before;
        if constexpr (VARY_K) {
            t.off_a = before * dim_m;
            t.off_b = kGatherK ? 0u : before * Ne;  // gathered: the loads address all of B
            t.off_d = (uint64_t)e * dim_m * Ne;
        } else {
            t.off_a = before * dim_k;
            t.off_b = (uint64_t)e * Ne * dim_k;
            t.off_d = before * Ne;
        }
        // 16-byte accesses need every contiguous dimension a multiple of 8 elements and packed group bases that stayed
        // multiples of 8; loads and stores address a tile with 32-bit byte offsets below 2^31 (grouped_gemm.hip)
        bool fast = (Ne % 8u == 0) && (Ne < (1u << 23)) && (t.off_a % 8u == 0) && (t.off_b % 8u == 0) && (t.off_d % 8u == 0);
        if (A_KC || B_KC) fast = fast && (t.Ke % 8u == 0) && (t.Ke < (1u << 21));
        if (!A_KC) fast = fast && (t.Me % 8u == 0) && (t.Me < (1u << 23));
        if (kGlu) fast = fast && (n_span % 8u == 0);
        t.fast = fast;
        return t;
    };
    auto k_steps = [&](const Tile& t) { return (t.Ke + BK - 1) / BK; };
    // groups of at most 64 rows run a K loop of their own with a third LDS stage (grouped_gemm.hip); they start cold
    auto is_thin = [&](const Tile& t) { return A_KC && t.Me <= 64u && k_steps(t) >= 3u; };
    // a tile whose first two K steps can be fetched by the tile before it, and which can fetch the next tile's
    // (gathered reduction rows: their indices are fetched two K steps ahead of the loads, four ahead of the step itself,
    // which looks at most one tile ahead if every tile in the stream has four steps)
    auto streams = [&](const Tile& t) { return t.valid && t.fast && t.Ke > 0 && !is_thin(t) && (!kGatherK || k_steps(t) >= 3u); };

    uint32_t round = 0;  // tiles this workgroup has finished

    // ---- loaders: `cur` feeds the tile being computed, `nxt` the tile after it ----
    LoaderK<NW, false> lk_a;
    LoaderK<NW, kGlu> lk_b;
    LoaderT<NW, true> lt_a, lt_b;
    Feed<A_KC> fa_cur{}, fa_nxt{};
    Feed<B_KC> fb_cur{}, fb_nxt{};
    uint32_t va_cur = 0, va_nxt = 0, vb_cur = 0, vb_nxt = 0;  // the loaders' per-lane offsets (they depend on the pitch)
    // sets a loader object up for tile t and keeps what is specific to the tile
    auto setup_a = [&](const Tile& t, Feed<A_KC>& f, uint32_t& v) {
        if constexpr (GATHER) return;  // nothing per tile: the rows come from the table in s_rows
        const uint16_t* Ae = args.A + t.off_a;
        if constexpr (A_KC) {
            lk_a.setup(Ae + (uint64_t)t.m0 * t.Ke, nullptr, t.Me - t.m0 < (uint32_t)BM ? t.Me - t.m0 : (uint32_t)BM, t.Ke, wave, lane);
            f = Feed<A_KC>{lk_a.base0, nullptr, lk_a.bytes, lk_a.ldb, 0u};
            v = lk_a.voff;
        } else {
            lt_a.setup(Ae, t.Me, t.Ke, t.m0, wave, lane);
            f = Feed<A_KC>{lt_a.base, nullptr, t.Ke, lt_a.ldb, lt_a.col_bytes};
            v = lt_a.voff;
        }
    };
    auto setup_b = [&](const Tile& t, Feed<B_KC>& f, uint32_t& v) {
        const uint16_t* Be = args.B + t.off_b;
        if constexpr (B_KC) {
            if constexpr (kGlu) {
                // tile rows 0..127: "up" rows n0.. of the weight; rows 128..255: "gate" rows I + n0..
                lk_b.setup(Be + (uint64_t)t.n0 * t.Ke, Be + (uint64_t)(n_span + t.n0) * t.Ke, t.n_lim - t.n0, t.Ke, wave, lane);
            } else {
                lk_b.setup(Be + (uint64_t)t.n0 * t.Ke, nullptr, t.n_lim - t.n0, t.Ke, wave, lane);
            }
            f = Feed<B_KC>{lk_b.base0, lk_b.base1, lk_b.bytes, lk_b.ldb, 0u};
            v = lk_b.voff;
        } else {
            lt_b.setup(Be, Ne, t.Ke, t.n0, wave, lane);
            f = Feed<B_KC>{lt_b.base, nullptr, t.Ke, lt_b.ldb, lt_b.col_bytes};
            v = kGatherK ? t.row0 : lt_b.voff;  // gathered: where the group's entries of row_index begin (same in every lane)
        }
    };
    // points a loader object at a feed (what depends on lane and wavefront only stays as the last setup left it)
    auto aim_a = [&](const Feed<A_KC>& f, uint32_t v) {
        if constexpr (GATHER) return;
        if constexpr (A_KC) { lk_a.base0 = f.base0; lk_a.bytes = f.extent; lk_a.ldb = f.ldb; lk_a.kdim = f.ldb / 2u; lk_a.voff = v; }
        else { lt_a.base = f.base0; lt_a.kdim = f.extent; lt_a.ldb = f.ldb; lt_a.col_bytes = f.col_bytes; lt_a.voff = v; }
    };
    auto aim_b = [&](const Feed<B_KC>& f, uint32_t v) {
        if constexpr (B_KC) { lk_b.base0 = f.base0; lk_b.base1 = f.base1; lk_b.bytes = f.extent; lk_b.ldb = f.ldb; lk_b.kdim = f.ldb / 2u; lk_b.voff = v; }
        else { lt_b.base = f.base0; lt_b.kdim = f.extent; lt_b.ldb = f.ldb; lt_b.col_bytes = f.col_bytes; lt_b.voff = v; }
    };

    // ---- GATHER: the A operand's rows are rows of args.A picked through args.row_index ----
    // The tile of round r keeps the row_index entries of its 256 rows in half r % 2 of s_rows. A wavefront's four load
    // instructions of a K step fetch tile rows g_row, g_row + 64, + 128, + 192 of this lane: four table entries, divided by
    // the divisor, times the row pitch. Entries past the group's rows read as zero (row 0 of A: rows never stored).
    const uint32_t g_full = GATHER ? args.a_rows * dim_k * 2u : 0u;  // bytes of A (below 2^31)
    const uint32_t g_ldb = dim_k * 2u;
    const uint32_t g_row = logical_row(wave * 8u + (lane >> 3));
    const uint32_t g_chunk = (lane & 7u) ^ (g_row & 7u);
    // The row an entry n of row_index names, n / divisor, or a number no row has if the entry is negative: for n < 2^31 the
    // high word of n * floor((2^32 - 1) / divisor) is the quotient or one less (any divisor from 1 on, no branch).
    const uint32_t g_magic = GATHER_ANY ? 0xffffffffu / args.divisor : 0u;
    auto g_source_row = [&](uint32_t n) -> uint32_t {
        uint32_t q = __umulhi(n, g_magic);
        q += (n - q * args.divisor >= args.divisor) ? 1u : 0u;
        return q | (n & 0x80000000u);
    };
    uint32_t g_bytes_nxt = 0;  // bytes of A the loads for the next tile may read: all of it, or nothing when nothing follows
    // per-lane offsets of the four loads of a K step of the tile in table half `half` (the step's k0 goes into the
    // instruction's scalar offset)
    auto g_tile_offsets = [&](uint32_t half, uint32_t (&v)[4]) {
        uint32_t n[4];
        lds_read4_stride64_quiet(lds_address(reinterpret_cast<const uint8_t*>(s_rows)) + half * 1024u + g_row * 4u, n);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            // an entry that names no row of A (negative, or past the last row) reads as a row of zeros
            const uint32_t src = g_source_row(n[i]);
            v[i] = src < args.a_rows ? src * g_ldb + g_chunk * 16u : kOutOfRange;
        }
    };
    // last, partial K step: chunks past the end of K are pushed out of range, which zero-fills them
    auto g_clip = [&](uint32_t k0, uint32_t (&v)[4]) {
        const bool past = k0 + (uint32_t)BK > dim_k && k0 + g_chunk * 8u >= dim_k;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = past ? kOutOfRange : v[i];
    };
    auto g_offsets = [&](uint32_t half, uint32_t k0, uint32_t (&v)[4]) {
        g_tile_offsets(half, v);
        g_clip(k0, v);
    };
    uint32_t g_kept[4] = {0u, 0u, 0u, 0u};  // g_tile_offsets of the tile the full-tile K loop is loading from
    // the table of tile t into half `half`: 32 entries per wavefront, in assembly (one load per wavefront)
    auto g_issue_table = [&](const Tile& t, uint32_t half) {
        if constexpr (GATHER) {
            const bool real = t.valid && t.Me > t.m0;
            const uint32_t rows = real ? (t.Me - t.m0 < (uint32_t)BM ? t.Me - t.m0 : (uint32_t)BM) : 0u;
            const u32x4 rs = make_rsrc_words(reinterpret_cast<const uint16_t*>(args.row_index + (real ? (uint64_t)t.row0 + t.m0 : 0u)),
                                             rows * 4u);
            const uint32_t to = lds_address(reinterpret_cast<const uint8_t*>(s_rows)) + half * 1024u + wave * 128u;
            if (lane < 32u) buffer_load_lds_quiet_b32(rs, (wave * 32u + lane) * 4u, 0u, to);
        }
    };
    static_assert(!GATHER_ANY || 32 / NW == 4, "four load instructions per wavefront and K step");

    // ---- kGatherK: the reduction rows of the B operand are rows of args.B picked through args.row_index ----
    // A wavefront's four load instructions of a K step fetch the step's reduction rows 8 wave + 2 i + (lane >> 5), i = 0..3
    // (the packed loader's are 16 i + 2 wave + (lane >> 5)): eight consecutive entries of row_index per wavefront and step.
    // They land where the packed loader puts the same rows: rows 2 s and 2 s + 1 of the step lie in kilobyte s of the stage
    // either way, so the LDS image, the fragment reads and the order of the sums are those of the packed kernel.
    // The eight entries are one vector load per wavefront and step (lane l: entry l % 8; a position past the end of
    // row_index reads as 0), issued two steps ahead of the loads that use them, behind the step's own loads: a step's loads
    // for K step kt + 2 go out with the entries requested in step kt - 2, which the wait of step kt - 1 has seen arrive
    // (loads complete in issue order). Inside a tile the entries travel in a register (gk_ring[s]: requested in the latest
    // step that ran in LDS stage s). Across a tile boundary they travel through LDS (s_gk, a direct-to-LDS load read back
    // in assembly): a register loaded in one tile and used in the next makes the compiler, which cannot count the
    // epilogue's stores, wait for everything in flight at the top of the tile.
    const __amdgpu_buffer_rsrc_t gk_index = make_rsrc(reinterpret_cast<const uint16_t*>(args.row_index),
                                                      kGatherK ? uniform(s_prefix[E]) * 4u : 0u);
    const uint32_t gk_bytes = kGatherK ? args.a_rows * Ne * 2u : 0u;  // bytes of B (below 2^31)
    const uint32_t gk_half = lane >> 5;
    // the 16-byte chunk of a row this lane loads, swizzled as the packed loader does it for the row's place in the step;
    // instruction i: ^ 128 (i & 1)
    const uint32_t gk_chunk = ((lane & 31u) ^ (4u * gk_half) ^ (2u * (wave & 1u))) << 4;
    uint32_t gk_v[4] = {0u, 0u, 0u, 0u};
    // this lane's entry of the eight that begin at position `first` of row_index. pinned: the request may not be issued
    // ahead of anything that precedes it in the program (the empty statement the lane's offset passes through is ordered
    // behind every load before it): the step waits count on the request being the newest load of its step
    auto gk_request = [&](uint32_t first, bool pinned) __attribute__((always_inline)) -> uint32_t {
        uint32_t mine = (lane & 7u) * 4u;
        if (pinned) asm volatile("" : "+v"(mine));
        return __builtin_amdgcn_raw_buffer_load_b32(gk_index, mine, first * 4u, 0);
    };
    // the same request into this wavefront's dwords of LDS stage `slot` of s_gk, and the entry read back from there
    auto gk_request_lds = [&](uint32_t first, int slot, bool pinned) __attribute__((always_inline)) {
        uint32_t mine = (lane & 7u) * 4u;
        if (pinned) asm volatile("" : "+v"(mine));
        __builtin_amdgcn_raw_ptr_buffer_load_lds(gk_index, (lds_void*)(s_gk + (slot * NW + wave) * 64), 4, mine, first * 4u, 0, 0);
    };
    auto gk_from_lds = [&](int slot) __attribute__((always_inline)) -> uint32_t {
        return lds_read1_quiet(lds_address(reinterpret_cast<const uint8_t*>(s_gk)) + (((uint32_t)slot * NW + wave) * 64u + lane) * 4u);
    };
    // per-lane offsets of the four loads of the K step at k0 of a group with `limit` reduction rows, from the entries n
    // (lane l holds entry l % 8): every lane forms the byte offset of its entry's row, then picks, per instruction, the
    // offset of one of the instruction's two rows from the lane that holds it, and adds its chunk.
    auto gk_offsets = [&](uint32_t k0, uint32_t limit, uint32_t n, uint32_t (&v)[4]) {
        // an entry that names no row of B (negative, or past the last row) reads as a row of zeros, and so does a
        // reduction row past the group's end
        uint32_t q = g_source_row(n);
        q = k0 + wave * 8u + (lane & 7u) < limit ? q : 0xffffffffu;
        const uint32_t off = q < args.a_rows ? q * (Ne * 2u) : kOutOfRange;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t even = (uint32_t)__builtin_amdgcn_readlane((int)off, 2 * i);
            const uint32_t odd = (uint32_t)__builtin_amdgcn_readlane((int)off, 2 * i + 1);
            v[i] = (gk_half ? odd : even) + (gk_chunk ^ (128u * ((uint32_t)i & 1u)));
        }
    };

    // ---- L2 prefetch by designated workgroups (grouped_gemm.hip): one 4-byte load per shared line, kPfDist steps ahead ----
    constexpr bool kPrefetch = A_KC == B_KC;
    uint32_t pf_voff = kOutOfRange;
    const uint16_t* pf_base = nullptr;
    uint32_t pf_bytes = 0, pf_ldb = 0, pf_col_bytes = 0, pf_kdim = 0, pf_steps = 0;
    const bool pf_is_b = (wave & 1u) != 0;
    const bool pf_t = pf_is_b ? !B_KC : !A_KC;
    auto setup_prefetch = [&](const Tile& t) {
        if constexpr (!kPrefetch) return;
        const uint32_t p = wave >> 1;
        pf_steps = k_steps(t);
        if (!pf_is_b) {
            const uint32_t i = p * 16u + lane;
            if constexpr (GATHER) {
                const uint32_t n = lds_read1_quiet(lds_address(reinterpret_cast<const uint8_t*>(s_rows)) + (round & 1u) * 1024u +
                                                   (lane < 16u ? 4u * i + t.pf_c : 0u) * 4u);
                pf_base = args.A; pf_bytes = g_full;
                const uint32_t src = lane < 16u ? g_source_row(n) : 0xffffffffu;
                pf_voff = src < args.a_rows ? src * g_ldb : kOutOfRange;
            } else if constexpr (A_KC) {
                pf_base = fa_cur.base0; pf_bytes = fa_cur.extent;
                pf_voff = lane < 16u ? (4u * i + t.pf_c) * (t.Ke * 2u) : kOutOfRange;
            } else {
                pf_base = fa_cur.base0; pf_ldb = fa_cur.ldb; pf_col_bytes = fa_cur.col_bytes; pf_kdim = t.Ke;
                pf_voff = lane < 16u ? i * fa_cur.ldb + t.pf_c * 128u : kOutOfRange;
            }
        } else {
            if constexpr (B_KC) {
                pf_bytes = fb_cur.extent;
                if constexpr (kGlu) {
                    pf_base = (p >> 1) ? fb_cur.base1 : fb_cur.base0;
                    pf_voff = lane < 8u ? (8u * ((p & 1u) * 8u + lane) + t.pf_r) * (t.Ke * 2u) : kOutOfRange;
                } else {
                    pf_base = fb_cur.base0;
                    pf_voff = lane < 8u ? (8u * (p * 8u + lane) + t.pf_r) * (t.Ke * 2u) : kOutOfRange;
                }
            } else {
                pf_base = fb_cur.base0; pf_ldb = fb_cur.ldb; pf_col_bytes = fb_cur.col_bytes; pf_kdim = t.Ke;
                // (gathered reduction rows: no prefetch of B, the instruction fetches nothing)
                pf_voff = (!kGatherK && lane < 8u) ? (2u * (p * 8u + lane) + (t.pf_r >> 2)) * fb_cur.ldb + (t.pf_r & 3u) * 128u : kOutOfRange;
            }
        }
    };
    // requests this wavefront's lines of K step `kstep` of the current tile (nothing past its last step)
    auto issue_prefetch = [&](uint32_t kstep) {
        if constexpr (!kPrefetch) return;
        const uint32_t k0 = kstep * (uint32_t)BK;
        const bool inside = kstep < pf_steps;
        const uint32_t rows = k0 >= pf_kdim ? 0u : (pf_kdim - k0 < (uint32_t)BK ? pf_kdim - k0 : (uint32_t)BK);
        const uint16_t* base = pf_t ? pf_base + (uint64_t)k0 * (pf_ldb / 2u) : pf_base;
        uint32_t bytes = !inside ? 0u : (pf_t ? (rows ? rows * pf_ldb - pf_col_bytes : 0u) : pf_bytes);
        if constexpr (GATHER) {
            // (the same in every lane, which the compiler does not see in these kernels: without this it wraps the load
            // in a loop over the distinct descriptors it fears)
            base = reinterpret_cast<const uint16_t*>(uniform((uint64_t)(uintptr_t)base));
            bytes = uniform(bytes);
        }
        __builtin_amdgcn_raw_ptr_buffer_load_lds(make_rsrc(base, bytes), (lds_void*)s_pf, 4, pf_voff, pf_t ? 0u : k0 * 2u, 0, 0);
    };

    constexpr int kLoads = 32 / NW;                // load instructions per wavefront, operand and K step
    constexpr uint32_t kStepLoads = 2 * kLoads;    // per wavefront and K step
    // store instructions per wavefront and tile (the epilogue issues a fixed number)
    constexpr uint32_t kTileStores = EPI == EPI_PLAIN        ? WM * WN * 2 / 1024
                                     : EPI == EPI_SWIGLU_BWD ? 2 * (WM * WN * 2 / 1024)  // two columns written per column
                                                             : (EPI == EPI_SWIGLU ? WM * WN * 2 / 1024 : 0) + WM * WN / 1024;

    // loads of one K step of the CURRENT loaders' aim into `stage` (compiler-visible: placed by the scheduling hints)
    // (i0_c, i1_c: which of the kLoads instructions)
    auto issue_a = [&](int stage, uint32_t k0, auto i0_c, auto i1_c) __attribute__((always_inline)) {
        constexpr int I0 = decltype(i0_c)::value, I1 = decltype(i1_c)::value;
        if constexpr (A_KC) lk_a.template issue_range<I0, I1>(stage ? s_a1 : s_a0, k0);
        else lt_a.template issue_range<I0, I1>(stage ? s_a1 : s_a0, k0);
    };
    // GATHER: the same four loads through the row table in half `half`; `bytes`: how much of A they may read
    // kept: take the offsets from g_kept (the caller has set it for that tile) instead of reading the table
    auto issue_a_gathered = [&](int stage, uint32_t k0, uint32_t half, uint32_t bytes, bool kept, auto i0_c, auto i1_c)
                                __attribute__((always_inline)) {
        constexpr int I0 = decltype(i0_c)::value, I1 = decltype(i1_c)::value;
        uint32_t v[4];
        if (kept) {
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] = g_kept[i];
            g_clip(k0, v);
        } else {
            g_offsets(half, k0, v);
        }
        const __amdgpu_buffer_rsrc_t r = make_rsrc(args.A, uniform(bytes));
        uint8_t* tile = stage ? s_a1 : s_a0;
#pragma unroll
        for (int i = I0; i < I1; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_void*)(tile + (i * NW + wave) * 1024), 16, v[i], k0 * 2u, 0, 0);
    };
    auto issue_b = [&](int stage, uint32_t k0, auto i0_c, auto i1_c) __attribute__((always_inline)) {
        constexpr int I0 = decltype(i0_c)::value, I1 = decltype(i1_c)::value;
        if constexpr (kGatherK) {
            // (gk_v: the offsets of the step's four loads, formed by the caller from the entries requested two steps ago)
            const __amdgpu_buffer_rsrc_t r = make_rsrc(lt_b.base, gk_bytes - lt_b.col_bytes);
            uint8_t* tile = stage ? s_b1 : s_b0;
#pragma unroll
            for (int i = I0; i < I1; ++i)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_void*)(tile + (wave * 4 + i) * 1024), 16, gk_v[i], 0u, 0, 0);
        } else if constexpr (B_KC) lk_b.template issue_range<I0, I1>(stage ? s_b1 : s_b0, k0);
        else lt_b.template issue_range<I0, I1>(stage ? s_b1 : s_b0, k0);
    };
    // ... and written in assembly, for a cold start
    auto issue_quiet = [&](int stage, uint32_t k0) {
        if constexpr (GATHER) {
            uint32_t v[4];
            g_offsets(round & 1u, k0, v);
            const u32x4 r = make_rsrc_words(args.A, g_full);
            const uint32_t lds0 = lds_address(stage ? s_a1 : s_a0) + wave * 1024u;
#pragma unroll
            for (int i = 0; i < 4; ++i) buffer_load_lds_quiet(r, v[i], k0 * 2u, lds0 + (uint32_t)(i * NW) * 1024u);
        } else if constexpr (A_KC) lk_a.issue_quiet(stage ? s_a1 : s_a0, k0);
        else lt_a.issue_quiet(stage ? s_a1 : s_a0, k0);
        if constexpr (kGatherK) {
            uint32_t v[4];
            gk_offsets(k0, lt_b.kdim, gk_request(vb_cur + k0 + wave * 8u, false), v);
            const u32x4 r = make_rsrc_words(lt_b.base, gk_bytes - lt_b.col_bytes);
            const uint32_t lds0 = lds_address(stage ? s_b1 : s_b0) + wave * 4096u;
#pragma unroll
            for (int i = 0; i < 4; ++i) buffer_load_lds_quiet(r, v[i], 0u, lds0 + (uint32_t)i * 1024u);
        } else if constexpr (B_KC) lk_b.issue_quiet(stage ? s_b1 : s_b0, k0);
        else lt_b.issue_quiet(stage ? s_b1 : s_b0, k0);
    };

    Tile cur = lookup(0), nxt = lookup(1);
    // GATHER: the second tile's rows (the first tile fetches its own in its cold start; from then on every tile
    // fetches those of the tile after next, before its epilogue)
    g_issue_table(nxt, 1u);
    bool streamed = false;  // the first two K steps of `cur` were fetched by the tile before it
    while (cur.valid) {
        const uint32_t Me = cur.Me, Ke = cur.Ke, m0 = cur.m0, n0 = cur.n0, n_lim = cur.n_lim;
        const uint64_t off_d = cur.off_d;

        if (!streamed) {
            if (!cur.fast) {
                if constexpr (EPI == EPI_PLAIN && !kGatherK) {  // (the gathered entry point admits only sizes without such tiles)
                    scalar_tile<EL, A_KC, B_KC, BM, BN>(args.A + cur.off_a, args.B + cur.off_b, args.D + off_d, Me, Ne, Ke, m0, n0,
                                                        args.alpha, NT);
                }
                cur = nxt;
                nxt = lookup(round + 2);
                ++round;
                continue;
            }
            setup_a(cur, fa_cur, va_cur);
            setup_b(cur, fb_cur, vb_cur);
        }
        if (GATHER && !streamed) {
            // a tile that starts cold fetches its own rows and waits for them (and for everything else in flight)
            g_issue_table(cur, round & 1u);
            __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, false));
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        }
        setup_prefetch(cur);
        const uint32_t KT = (Ke + BK - 1) / BK;
        const uint32_t KT2 = (KT + 1u) & ~1u;  // steps of the K loop: an odd count gets a step of zeros
        const bool thin = is_thin(cur);
        // kGatherK: where in row_index the entries of this wavefront for K step `abs_step` of the load stream begin: a step
        // of this tile, or, past its end, of the next (vb_cur, vb_nxt: where the two groups' entries begin)
        auto gk_first = [&](uint32_t abs_step) __attribute__((always_inline)) -> uint32_t {
            const bool of_next = abs_step >= KT2;
            return (of_next ? vb_nxt + (abs_step - KT2) * (uint32_t)BK : vb_cur + abs_step * (uint32_t)BK) + wave * 8u;
        };
        uint32_t gk_ring[2] = {0u, 0u};
        // the next tile's first two K steps ride on this tile's last two load slots
        const bool stream_next = streams(cur) && streams(nxt);
        if (stream_next) {
            setup_a(nxt, fa_nxt, va_nxt);
            setup_b(nxt, fb_nxt, vb_nxt);
        } else {
            // a feed that fetches nothing: every load of it zero-fills
            if constexpr (!GATHER) {
                fa_nxt = fa_cur;
                fa_nxt.extent = 0u;
                va_nxt = va_cur;
            }
            fb_nxt = fb_cur;
            fb_nxt.extent = 0u;
            vb_nxt = vb_cur;
        }
        g_bytes_nxt = stream_next ? g_full : 0u;
        // (the set-ups above left the loader objects aimed at the last tile set up)
        aim_a(fa_cur, va_cur);
        aim_b(fb_cur, vb_cur);

        // The CB column blocks of a row block are one 16-register value (block j in elements 4 j ..), and every matrix
        // instruction's result is named as part of that value again (anchor_value): the result then stays in the register
        // quadruple its addend came from. The compiler has no tied-operand form of the 4-register instruction; as 32 separate
        // quadruples the results wandered through the register file and the allocator spilled 3 to 40 registers.
        f32x16 acc[RB];
#pragma unroll
        for (int i = 0; i < RB; ++i)
#pragma unroll
            for (int x = 0; x < 16; ++x) acc[i][x] = 0.0f;
        auto mfma_block = [&](f32x16& c, int j, typename EL::frag b, typename EL::frag a) __attribute__((always_inline)) {
            f32x4 q = {c[4 * j], c[4 * j + 1], c[4 * j + 2], c[4 * j + 3]};
            q = EL::mfma16(b, a, q);
            c[4 * j] = q[0];
            c[4 * j + 1] = q[1];
            c[4 * j + 2] = q[2];
            c[4 * j + 3] = q[3];
            anchor_value(c);
        };

        // MFMA operand fragments of one 32-wide k slice: the A fragments of two row blocks (a "pair"), in four buffers (full
        // tiles read them two phases ahead and hold three pairs across the step's barrier; the other versions use two), and
        // the B fragments of the four column blocks. A phase is one pair times the four column blocks, column block by
        // column block. In the last phase of a slice every B fragment is replaced by the next slice's as soon as its two
        // matrix instructions have been issued (one set of B registers).
        // The K loop exists in five versions, for wavefronts whose first FA = 8, 4, 2, 1 or 0 row blocks (of 16 rows)
        // hold rows of the group.
        typename EL::frag fa[4][2], fb[CB];
        // A fragments of pair `pair` of slice ks into buffer buf
        auto load_a = [&](auto fa_c, int stage, int ks, int pair, int buf) __attribute__((always_inline)) {
            constexpr int FA = decltype(fa_c)::value;
            constexpr int AB = FA < 2 ? FA : 2;
            const uint8_t* ta = stage ? s_a1 : s_a0;
#pragma unroll
            for (int i = 0; i < AB; ++i) {
                const int b = pair * 2 + i;
                if constexpr (A_KC) fa[buf][i] = __builtin_bit_cast(typename EL::frag, read_kc_frag(ta + a_off[b] + kc_slice[ks]));
                else fa[buf][i] = __builtin_bit_cast(typename EL::frag, read_tr_frag(ta + a_off[b] + ks * kSliceT));
            }
        };
        auto load_b = [&](int stage, int ks, int j) __attribute__((always_inline)) {
            const uint8_t* tb = stage ? s_b1 : s_b0;
            if constexpr (B_KC) fb[j] = __builtin_bit_cast(typename EL::frag, read_kc_frag(tb + b_off[j] + kc_slice[ks]));
            else fb[j] = __builtin_bit_cast(typename EL::frag, read_tr_frag(tb + b_off[j] + ks * kSliceT));
        };
        // pair `pair` from A buffer abuf times the B fragments; reload: each B fragment is then read anew from slice
        // next_ks of stage next_stage
        auto mma = [&](auto fa_c, int pair, int abuf, bool reload, int next_stage, int next_ks) __attribute__((always_inline)) {
            constexpr int FA = decltype(fa_c)::value;
            constexpr int AB = FA < 2 ? FA : 2;
            if constexpr (FA > 0) {
#pragma unroll
                for (int j = 0; j < CB; ++j) {
#pragma unroll
                    for (int i = 0; i < AB; ++i)
                        mfma_block(acc[pair * 2 + i], j, fb[j], fa[abuf][i]);
                    if (reload) load_b(next_stage, next_ks, j);
                }
            }
        };

        // ---- one K step (see grouped_gemm.hip for the placement of barrier, waits and loads) ----
        // WAIT: the s_waitcnt immediate in front of the barrier. The loads issued after the barrier are those of step
        // kt + 2: of this tile, or, in the last two steps, steps 0 and 1 of the next tile (or nothing).
        // SRC: which tile the loads issued in the step belong to: 0 the current one, 1 the next one (the loaders are aimed
        // by the caller in both cases), 2 decided here (first steps of a tile, and the versions for tiles with few rows).
        auto step = [&](auto fa_c, auto wait_c, auto src_c, int stage, uint32_t kt) __attribute__((always_inline)) {
            constexpr int FA = decltype(fa_c)::value;
            constexpr int SRC = decltype(src_c)::value;
            constexpr int AB = FA < 2 ? FA : 2;       // row blocks per phase
            constexpr int PP = FA >= 2 ? FA / 2 : 1;  // phases per k slice
            constexpr int NPH = 2 * PP;               // phases of the step
            constexpr int kReadsA = (A_KC ? 1 : 2) * AB, kReadsB = (B_KC ? 1 : 2);  // LDS reads per pair, per B fragment
            // On entry A buffer 0 and the B registers hold the fragments of the first phase.
            typedef std::integral_constant<int, 0> I0_;
            typedef std::integral_constant<int, 2> I2_;
            typedef std::integral_constant<int, 3> I3_;
            typedef std::integral_constant<int, kLoads> IN_;
            static_assert(kLoads == 4, "the split of a step's loads over three phases is written for four per operand");
            // the A loads [i0, i1) of the step's load slot
            auto issue_a_part = [&](uint32_t k0, auto i0_c, auto i1_c) __attribute__((always_inline)) {
                if constexpr (GATHER) {
                    const bool of_next = SRC == 1 || (SRC == 2 && kt + 2u >= KT2);
                    issue_a_gathered(stage, k0, (of_next ? round + 1u : round) & 1u, of_next ? g_bytes_nxt : g_full, SRC != 2, i0_c, i1_c);
                } else {
                    issue_a(stage, k0, i0_c, i1_c);
                }
            };
            // kGatherK: the entries for this step's loads were requested two steps ago: by a step of this tile into a register,
            // or, for a tile's first two steps (SRC == 2 in a full tile), by the tile before or the cold start into LDS; the
            // versions for tiles with few rows do not know at compile time which of their steps are the last two and use LDS
            // throughout
            auto gk_step_offsets = [&](uint32_t k0) __attribute__((always_inline)) {
                if constexpr (kGatherK) {
                    constexpr bool kFromLds = FA != RB || SRC == 2;
                    gk_offsets(k0, lt_b.kdim, kFromLds ? gk_from_lds(stage) : gk_ring[stage], gk_v);
                }
            };
            // ... and the entries for the loads of step kt + 2 (K step kt + 4 of the stream) are requested as the step's last
            // load: into LDS by a full tile's last two steps (SRC == 1)
            auto gk_step_request = [&]() __attribute__((always_inline)) {
                if constexpr (kGatherK) {
                    constexpr bool kToLds = FA != RB || SRC == 1;
                    if constexpr (kToLds) gk_request_lds(gk_first(kt + 4u), stage, true);
                    else gk_ring[stage] = gk_request(gk_first(kt + 4u), true);
                }
            };
            // what the loads issued in this step fetch: the K offset (returned) and, decided here (SRC == 2), whether the
            // loaders aim at the current tile's operands or the next one's
            auto aim_loads = [&]() __attribute__((always_inline)) -> uint32_t {
                uint32_t k0;
                if constexpr (SRC == 0) {
                    k0 = (kt + 2u) * (uint32_t)BK;
                } else if constexpr (SRC == 1) {
                    k0 = (kt + 2u - KT2) * (uint32_t)BK;
                } else {
                    const bool of_next = kt + 2u >= KT2;
                    k0 = (of_next ? kt + 2u - KT2 : kt + 2u) * (uint32_t)BK;
                    if constexpr (!GATHER)
                        aim_a(Feed<A_KC>{of_next ? fa_nxt.base0 : fa_cur.base0, nullptr, of_next ? fa_nxt.extent : fa_cur.extent,
                                         of_next ? fa_nxt.ldb : fa_cur.ldb, of_next ? fa_nxt.col_bytes : fa_cur.col_bytes},
                              of_next ? va_nxt : va_cur);
                    aim_b(Feed<B_KC>{of_next ? fb_nxt.base0 : fb_cur.base0, of_next ? fb_nxt.base1 : fb_cur.base1,
                                     of_next ? fb_nxt.extent : fb_cur.extent, of_next ? fb_nxt.ldb : fb_cur.ldb,
                                     of_next ? fb_nxt.col_bytes : fb_cur.col_bytes},
                          of_next ? vb_nxt : vb_cur);
                }
                return k0;
            };
            if constexpr (FA == RB) {
                // Full tiles: the barrier comes after five of the eight phases, with the A fragments of the last three phases
                // already in registers (four A buffers), so that the step's loads go out over three phases instead of one:
                // eight wavefronts that leave the barrier together otherwise queue 72 loads on the one address path at once.
                // A fragments are read two phases ahead (phase p's pair sits in buffer p % 4): phase 0 reads those of phases 1
                // (the step before could not: they are behind its barrier) and 2, phase 4 those of 6 and 7 first thing
                load_a(fa_c, stage, 0, 1, 1);
#pragma unroll
                for (int ph = 0; ph < 4; ++ph) {
                    load_a(fa_c, stage, (ph + 2) / PP, (ph + 2) % PP, (ph + 2) & 3);
                    mma(fa_c, ph, ph, ph == 3, stage, 1);
                    if (ph == 3) {
                        __builtin_amdgcn_sched_group_barrier(0x100, kReadsA, 0);
#pragma unroll
                        for (int j = 0; j < CB; ++j) {
                            __builtin_amdgcn_sched_group_barrier(0x008, AB, 0);
                            __builtin_amdgcn_sched_group_barrier(0x100, kReadsB, 0);
                        }
                    } else {
                        if (ph == 0) interleave3<0, AB * CB, 2 * kReadsA, 0>();
                        else interleave3<0, AB * CB, kReadsA, 0>();
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
                load_a(fa_c, stage, 1, 2, 2);
                load_a(fa_c, stage, 1, 3, 3);
                mma(fa_c, 0, 0, false, stage, 1);
                __builtin_amdgcn_sched_group_barrier(0x100, 2 * kReadsA, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, AB * CB, 0);
                // every load of step kt+1 has landed and every LDS read of this stage has returned
                __builtin_amdgcn_s_waitcnt(decltype(wait_c)::value);
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                const uint32_t k0 = aim_loads();
                issue_a_part(k0, I0_{}, I3_{});
                mma(fa_c, 1, 1, false, stage, 1);
                spread_mfma_vmem<0, AB * CB, 3>();
                __builtin_amdgcn_sched_barrier(0);
                issue_a_part(k0, I3_{}, IN_{});
                gk_step_offsets(k0);
                issue_b(stage, k0, I0_{}, I2_{});
                mma(fa_c, 2, 2, false, stage, 1);
                spread_mfma_vmem<0, AB * CB, 3>();
                __builtin_amdgcn_sched_barrier(0);
                load_a(fa_c, stage ^ 1, 0, 0, 0);
                issue_b(stage, k0, I2_{}, IN_{});
                if constexpr (kPrefetch) asm volatile("" : "+v"(pf_voff));
                issue_prefetch(kt + kPfDist);
                gk_step_request();
                mma(fa_c, 3, 3, true, stage ^ 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, kReadsA, 0);
#pragma unroll
                for (int j = 0; j < CB; ++j) {
#pragma unroll
                    for (int i = 0; i < AB; ++i) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                        if (j * AB + i < 2 + (kPrefetch ? 1 : 0) + (kGatherK ? 1 : 0)) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                    }
                    __builtin_amdgcn_sched_group_barrier(0x100, kReadsB, 0);
                }
            } else {
#pragma unroll
                for (int ph = 0; ph < NPH - 1; ++ph) {
                    const bool last_of_slice = ph == PP - 1;
                    load_a(fa_c, stage, (ph + 1) / PP, (ph + 1) % PP, (ph + 1) & 1);
                    mma(fa_c, ph % PP, ph & 1, last_of_slice, stage, 1);
                    if constexpr (FA > 0) {
                        if (last_of_slice) {
                            // the A reads, then per column block its matrix instructions and the read of its next fragment
                            __builtin_amdgcn_sched_group_barrier(0x100, kReadsA, 0);
#pragma unroll
                            for (int j = 0; j < CB; ++j) {
                                __builtin_amdgcn_sched_group_barrier(0x008, AB, 0);
                                __builtin_amdgcn_sched_group_barrier(0x100, kReadsB, 0);
                            }
                        } else {
                            interleave3<0, AB * CB, kReadsA, 0>();
                        }
                        // nothing moves from one phase into another: reads issued earlier would hold their registers longer
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
                // every load of step kt+1 has landed and every LDS read of this stage has returned
                __builtin_amdgcn_s_waitcnt(decltype(wait_c)::value);
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                load_a(fa_c, stage ^ 1, 0, 0, 0);
                const uint32_t k0 = aim_loads();
                issue_a_part(k0, I0_{}, IN_{});
                gk_step_offsets(k0);
                issue_b(stage, k0, I0_{}, IN_{});
                // the prefetch goes out behind this step's loads (the empty statement orders it: the wait of the next step
                // counts on it being the newest load)
                if constexpr (kPrefetch) asm volatile("" : "+v"(pf_voff));
                issue_prefetch(kt + kPfDist);
                gk_step_request();
                mma(fa_c, PP - 1, 1, true, stage ^ 1, 0);
                if constexpr (FA > 0) {
                    // the A reads; per column block its matrix instructions, each followed by its share of the step's loads,
                    // and the read of the block's next fragment; the prefetch last
                    constexpr int kLoadsPer = (int)kStepLoads / (AB * CB);
                    static_assert(kLoadsPer * AB * CB == (int)kStepLoads, "the loads divide evenly over the matrix instructions");
                    __builtin_amdgcn_sched_group_barrier(0x100, kReadsA, 0);
#pragma unroll
                    for (int j = 0; j < CB; ++j) {
#pragma unroll
                        for (int i = 0; i < AB; ++i) {
                            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(0x020, kLoadsPer, 0);
                        }
                        __builtin_amdgcn_sched_group_barrier(0x100, kReadsB, 0);
                    }
                    if constexpr (kPrefetch) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                    if constexpr (kGatherK) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                }
            }
        };
        // waits of a step: all but the newest load when that is the previous step's prefetch; in a tile's first step the
        // stores of the previous epilogue (or the cold start's stand-ins) and the one load of the bias values are newer
        // than the loads waited for as well
        // (kGatherK: and the request for row_index entries that follows every step's loads. In a tile's first step that
        // request, like the prefetch of the same step, is older than the stores, and a cold start issues none behind the
        // loads waited for: the count stays the one of the cold start, which only waits for more in a streamed tile)
        using WaitStep = std::integral_constant<int, waitcnt_imm((kPrefetch ? 1 : 0) + (kGatherK ? 1 : 0), true)>;
        using WaitFirst = std::integral_constant<int, waitcnt_imm((int)kTileStores + (kPrefetch ? 1 : 0) + (BIAS ? 1 : 0), true)>;

        // BIAS: the bias values of this wavefront's columns of the tile into its 128 bytes of LDS: one load by 32 lanes
        // (every wavefront issues it, so that all count the same loads), complete (loads and stores complete in issue
        // order) long before the epilogue reads them. Columns past the end zero-fill.
        auto issue_bias = [&]() {
            if constexpr (BIAS) {
                const uint16_t* row = args.bias + (uint64_t)cur.e * Ne;
                const u32x4 rs = make_rsrc_words(row, Ne * 2u);
                const uint32_t to = lds_address(s_bias) + wave * (uint32_t)kBiasBytes;
                // plain: columns n0 + wn*64 + 2*lane; swiglu: lanes 0..15 the 32 "up" columns, lanes 16..31 the "gate" ones
                const uint32_t col = EPI == EPI_PLAIN ? n0 + wn * WN + 2u * lane
                                                      : n0 + wn * (WN / 2) + 2u * (lane & 15u) + (lane >= 16u ? n_span : 0u);
                if (lane < 32u) buffer_load_lds_quiet_b32(rs, col * 2u, 0u, to);
            }
        };
        Tile nn{};  // the tile after next
        const uint32_t tile_rows = Me - m0 < (uint32_t)BM ? Me - m0 : (uint32_t)BM;
        const uint32_t wave_rows = tile_rows > wm * WM ? tile_rows - wm * WM : 0u;
        const bool has_columns = n0 + wn * (kGlu ? WN / 2 : WN) < n_lim;
        const uint32_t row_blocks = has_columns ? uniform((wave_rows + 15u) / 16u) : 0u;  // of 16 rows
        if (thin) {
            // three LDS stages in the space a tile of at most 64 rows leaves unused (grouped_gemm.hip); cold start
            constexpr uint32_t kThinLoads = 1 + kLoads;
            static_assert(kThinLoads == 5, "the waits below are written for five loads per step");
            const uint8_t* const a_at[3] = {s_a0, s_a1, s_a0 + 8192};
            const uint8_t* const b_lo[3] = {s_b0, s_b1, s_a0 + 16384};
            const uint8_t* const b_hi[3] = {s_b0 + 16384, s_b1 + 16384, s_a1 + 16384};
            auto issue_thin = [&](int st, uint32_t k0) {
                if constexpr (GATHER) {
                    uint32_t v[4];
                    g_offsets(round & 1u, k0, v);
                    buffer_load_lds_quiet(make_rsrc_words(args.A, g_full), v[0], k0 * 2u, lds_address(a_at[st]) + wave * 1024u);
                } else if constexpr (A_KC) lk_a.issue_quiet_first_rows(lds_address(a_at[st]), k0);
                if constexpr (B_KC) lk_b.issue_quiet_halves(lds_address(b_lo[st]), lds_address(b_hi[st]), k0);
                else lt_b.issue_quiet_halves(lds_address(b_lo[st]), lds_address(b_hi[st]), k0);
            };
            issue_bias();
            issue_thin(0, 0);
            issue_thin(1, BK);
            __builtin_amdgcn_s_waitcnt(waitcnt_imm((int)kThinLoads, false));
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            issue_thin(2, 2 * BK);
            auto thin_loop = [&](auto fa_c) {
                constexpr int FA = decltype(fa_c)::value;
                auto thin_step = [&](int st, uint32_t kt) {
                    if constexpr (FA > 0) {
#pragma unroll
                        for (int ks = 0; ks < 2; ++ks) {
                            typename EL::frag ta[FA], tb[CB];
#pragma unroll
                            for (int i = 0; i < FA; ++i)
                                ta[i] = __builtin_bit_cast(typename EL::frag, read_kc_frag(a_at[st] + a_off[i] + kc_slice[ks]));
#pragma unroll
                            for (int j = 0; j < CB; ++j) {
                                if constexpr (B_KC) {
                                    const uint8_t* half = b_frag_row(j) < 128u ? b_lo[st] + b_off[j] : b_hi[st] + (b_off[j] - 128u * kRowBytes);
                                    tb[j] = __builtin_bit_cast(typename EL::frag, read_kc_frag(half + kc_slice[ks]));
                                } else {
                                    const uint8_t* half = ks == 0 ? b_lo[st] : b_hi[st];  // k rows 0..31 and 32..63 of the step
                                    tb[j] = __builtin_bit_cast(typename EL::frag, read_tr_frag(half + b_off[j]));
                                }
                            }
#pragma unroll
                            for (int i = 0; i < FA; ++i)
#pragma unroll
                                for (int j = 0; j < CB; ++j) mfma_block(acc[i], j, tb[j], ta[i]);
                        }
                    }
                    __builtin_amdgcn_s_waitcnt(waitcnt_imm((int)kThinLoads, false));
                    __builtin_amdgcn_s_barrier();
                    asm volatile("" ::: "memory");
                    issue_thin(st, (kt + 3) * BK);
                };
                uint32_t kt = 0;
                for (; kt + 2 < KT; kt += 3) {
                    thin_step(0, kt);
                    thin_step(1, kt + 1);
                    thin_step(2, kt + 2);
                }
                if (kt < KT) thin_step(0, kt);
                if (kt + 1 < KT) thin_step(1, kt + 1);
            };
            if (row_blocks > 2) thin_loop(std::integral_constant<int, 4>{});
            else if (row_blocks == 2) thin_loop(std::integral_constant<int, 2>{});
            else if (row_blocks == 1) thin_loop(std::integral_constant<int, 1>{});
            else thin_loop(std::integral_constant<int, 0>{});
            __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, false));
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        } else if (KT > 0) {
            if (!streamed) {
                // cold start: the first two K steps, then as many stores outside every buffer as an epilogue issues
                // (kGatherK: the entries for the loads of steps 0 and 1 first, so that everything the waits below leave
                // outstanding is what they count; a streamed tile has them from the last two steps of the tile before it)
                if constexpr (kGatherK) {
                    gk_request_lds(gk_first(2u), 0, false);
                    gk_request_lds(gk_first(3u), 1, false);
                }
                issue_quiet(0, 0);
                issue_quiet(1, BK);
                const __amdgpu_buffer_rsrc_t nowhere = make_rsrc(args.D, 0u);
#pragma unroll
                for (uint32_t i = 0; i < kTileStores; ++i)  // (distinct offsets: identical stores would be merged into one)
                    store_tile16<false>(nowhere, kOutOfRange + i * 16u, uint4{0u, 0u, 0u, 0u});
                // the first step's loads have landed; the second step's, and the stand-in stores, may be out
                __builtin_amdgcn_s_waitcnt(waitcnt_imm((int)(kStepLoads + kTileStores), false));
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
            }
            issue_bias();
            issue_prefetch(kPfDist - 1);
            using SrcCur = std::integral_constant<int, 0>;
            using SrcNext = std::integral_constant<int, 1>;
            using SrcEither = std::integral_constant<int, 2>;
            auto k_loop = [&](auto fa_c) {
                constexpr int FA = decltype(fa_c)::value;
                load_a(fa_c, 0, 0, 0, 0);
                if constexpr (FA > 0) {
#pragma unroll
                    for (int j = 0; j < CB; ++j) load_b(0, 0, j);
                }
                step(fa_c, WaitFirst{}, SrcEither{}, 0, 0);
                step(fa_c, WaitStep{}, SrcEither{}, 1, 1);
                if constexpr (FA == RB) {
                    // full tiles: the steps in the middle load from the current tile and the last two from the next, each
                    // with the loaders aimed once, so that the loop body carries no selects
                    if (KT2 > 2u) {
                        aim_a(fa_cur, va_cur);
                        aim_b(fb_cur, vb_cur);
                        if constexpr (GATHER) g_tile_offsets(round & 1u, g_kept);
                        uint32_t kt = 2;
                        for (; kt + 2u < KT2; kt += 2) {  // two steps per iteration without a branch between them
                            step(fa_c, WaitStep{}, SrcCur{}, 0, kt);
                            step(fa_c, WaitStep{}, SrcCur{}, 1, kt + 1);
                        }
                        aim_a(fa_nxt, va_nxt);
                        aim_b(fb_nxt, vb_nxt);
                        if constexpr (GATHER) g_tile_offsets((round + 1u) & 1u, g_kept);
                        step(fa_c, WaitStep{}, SrcNext{}, 0, kt);
                        step(fa_c, WaitStep{}, SrcNext{}, 1, kt + 1);
                    }
                } else {
                    for (uint32_t kt = 2; kt < KT2; kt += 2) {
                        step(fa_c, WaitStep{}, SrcEither{}, 0, kt);
                        step(fa_c, WaitStep{}, SrcEither{}, 1, kt + 1);
                    }
                }
            };
            static_assert(RB == 8, "the versions below are for eight row blocks per wavefront");
            if (row_blocks > 4) k_loop(std::integral_constant<int, 8>{});
            else if (row_blocks > 2) k_loop(std::integral_constant<int, 4>{});
            else if (row_blocks == 2) k_loop(std::integral_constant<int, 2>{});
            else if (row_blocks == 1) k_loop(std::integral_constant<int, 1>{});
            else k_loop(std::integral_constant<int, 0>{});
            if (!stream_next) {
                // nothing rides behind this tile: its last two load slots zero-filled the stages; they must have landed,
                // and every wavefront must be past its last read, before anyone starts cold
                __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, false));
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
            }
        }

        if (BIAS && KT == 0) {  // a group without reduction: the result is the bias
            issue_bias();
            __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, false));
        }
        // the tile after next is looked up here: scalar work beside an epilogue that is bound by the store path
        nn = lookup(round + 2);
        // GATHER: its rows go where this tile's were (no load of this tile is left to be issued). The load is older than
        // this tile's stores, so the first wait of the next tile covers it.
        g_issue_table(nn, round & 1u);

        // ---- epilogue: through this wavefront's 2 KB of the staging buffer, 16 rows of 128 bytes at a time ----
        // A lane holds row (lane & 15), columns (lane >> 4)*4 + 0..3 of each 16x16 accumulator block.
        // (the lane id is made opaque so that the per-lane address arithmetic is redone per tile, not hoisted out of the
        // tile loop where it would occupy registers throughout the K loop)
        uint32_t el = lane;
        asm volatile("" : "+v"(el));
        const uint32_t img = lds_address(s_stage) + wave * (uint32_t)kStageBytes;
        if (EPI == EPI_PLAIN && args.alpha != 1.0f) {
            const float alpha = args.alpha;
#pragma unroll
            for (int i = 0; i < RB; ++i) acc[i] *= alpha;
        }
        // Tiles with a short reduction write much per flop (a weight gradient over ~500 rows: 8 K steps per 128 KB tile):
        // their stores carry the non-temporal hint (+4 to 5 % there); for long reductions plain stores are faster by 0 to 1 %
        const bool stream_out = VARY_K && KT <= kStreamOutSteps;
        // BIAS: the four groups of four columns this lane holds of every row block, as fp32
        float bias_f[CB][4];
        if constexpr (BIAS) {
            uint32_t at[4];
            uint2 raw[4];
            const uint32_t mine = lds_address(s_bias) + wave * (uint32_t)kBiasBytes;
            // plain: 64 columns; swiglu: 32 "up" columns (j = 0, 1), then 32 "gate" columns
#pragma unroll
            for (int j = 0; j < CB; ++j) at[j] = mine + ((uint32_t)j * 16u + (el >> 4) * 4u) * 2u;
            lds_read4x8_quiet(at, raw);
#pragma unroll
            for (int j = 0; j < CB; ++j) {
                const uint2 r = raw[j];
                bias_f[j][0] = EL::from_bits((uint16_t)(r.x & 0xffffu));
                bias_f[j][1] = EL::from_bits((uint16_t)(r.x >> 16));
                bias_f[j][2] = EL::from_bits((uint16_t)(r.y & 0xffffu));
                bias_f[j][3] = EL::from_bits((uint16_t)(r.y >> 16));
            }
        }
        // the value that is stored (plain) or activated (swiglu): the rounded product, plus the bias rounded again, which is
        // what the product followed by a separate bias pass gives
        auto with_bias = [&](float product, int j, int x) -> float {
            if constexpr (BIAS) return EL::round(product) + bias_f[j][x];
            else return product;
        };
        // EPI_SWIGLU_BWD: the h values of the eight passes (16 rows each) of this wavefront's sub-tile: [pass][row 0/1][up, gate]
        u32x4 bwd_h[EPI == EPI_SWIGLU_BWD ? RB : 1][2][2];
        // byte offset of this lane's piece of row `r` (0 or 1: rows lane / 8 and 8 + lane / 8 of the pass) from the pass's
        // first row and the wavefront's first column, or out of range
        auto bwd_offset = [&](int r, uint32_t cols_valid) -> uint32_t {
            const uint32_t c16 = el & 7u;
            const uint32_t row = (uint32_t)r * 8u + (el >> 3);
            return c16 * 8u < cols_valid ? row * (Ne * 4u) + c16 * 16u : kOutOfRange;
        };
        auto bwd_rows = [&](int pass) -> uint32_t {  // rows of the pass inside the group
            const uint32_t r0 = m0 + wm * WM + (uint32_t)pass * 16u;
            return r0 < Me ? (Me - r0 < 16u ? Me - r0 : 16u) : 0u;
        };
        auto bwd_origin = [&](int pass, uint32_t col0) -> uint64_t {  // element offset of the pass's first row and column
            return ((uint64_t)cur.row0 + m0 + wm * WM + (uint32_t)pass * 16u) * (2ull * Ne) + col0;
        };
        // h is read once and its gradient written once, in whole 128-byte lines: both carry the non-temporal hint, which
        // keeps them from displacing the operand panels in the L2 (+3 % on the Mixtral shape, +2 % large-E, +0.5 % fine-grained)
        constexpr int kStreamAux = 2;
        auto bwd_request = [&](int pass, uint32_t col0, uint32_t cols_valid) {
            if constexpr (EPI == EPI_SWIGLU_BWD) {
                const __amdgpu_buffer_rsrc_t rs = make_rsrc(args.h_in + bwd_origin(pass, col0), bwd_rows(pass) * (Ne * 4u));
#pragma unroll
                for (int r = 0; r < 2; ++r) {
                    const uint32_t off = bwd_offset(r, cols_valid);
                    bwd_h[pass][r][0] = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)off, 0, kStreamAux);
                    bwd_h[pass][r][1] = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)off, (int)(Ne * 2u), kStreamAux);
                }
            }
        };
        auto bwd_finish = [&](int pass, uint32_t col0, uint32_t cols_valid) {
            if constexpr (EPI == EPI_SWIGLU_BWD) {
                const uint32_t c16 = el & 7u;
                u32x4 dy[2];
                stage_get2_quiet(img, stage_off<WN * 2>(el >> 3, c16), stage_off<WN * 2>(8u + (el >> 3), c16), dy[0], dy[1]);
                const u32x4 rs = make_rsrc_words(args.D + bwd_origin(pass, col0), bwd_rows(pass) * (Ne * 4u));
#pragma unroll
                for (int r = 0; r < 2; ++r) {
                    u32x4 du, dg;
#pragma unroll
                    for (int x = 0; x < 4; ++x) {
                        float gu[2], gg[2];
#pragma unroll
                        for (int hlf = 0; hlf < 2; ++hlf) {
                            const int sh = hlf * 16;
                            const float d = EL::from_bits((uint16_t)(dy[r][x] >> sh));
                            const float u = EL::from_bits((uint16_t)(bwd_h[pass][r][0][x] >> sh));
                            const float g = EL::from_bits((uint16_t)(bwd_h[pass][r][1][x] >> sh));
                            swiglu_b<typename EL::act_t>(g, u, d, gg[hlf], gu[hlf]);
                        }
                        du[x] = EL::pack2(gu[0], gu[1]);
                        dg[x] = EL::pack2(gg[0], gg[1]);
                    }
                    // The "gate" half's column offset goes into the per-lane offset, not into the instruction's scalar
                    // offset: a 16-byte store with a scalar-register offset whose first data register the next VALU
                    // instruction overwrites lost that dword in some lanes on this part, and the compiler leaves no wait state
                    // there (it does for stores with a constant scalar offset, as every other store of this library has).
                    const uint32_t off = bwd_offset(r, cols_valid);
                    const uint32_t off_gate = off == kOutOfRange ? kOutOfRange : off + Ne * 2u;
                    // (in assembly: the next tile's first wait counts these stores, so their number must be exactly this)
                    store_tile16_quiet_nt(rs, off, du);
                    store_tile16_quiet_nt(rs, off_gate, dg);
                }
            }
        };
        const uint32_t put_row = el & 15u, put_col = (el >> 4) * 4u;  // this lane's place in a 16 x 16 block
        uint32_t ypack[2][2][2];  // swiglu: the activation of two row blocks, which share one image: [block][column block][2]
#pragma unroll
        for (int i = 0; i < RB; ++i) {
            const uint32_t r0 = m0 + wm * WM + i * 16;  // first output row of this block
            const uint32_t rows_valid = r0 < Me ? (Me - r0 < 16u ? Me - r0 : 16u) : 0u;
            if constexpr (EPI == EPI_PLAIN || EPI == EPI_SWIGLU_BWD) {
                const uint32_t col0 = n0 + wn * WN;
                const uint32_t cols_valid = col0 < n_lim ? n_lim - col0 : 0u;
                uint2 w[CB];
#pragma unroll
                for (int j = 0; j < CB; ++j) {
                    const f32x16& c = acc[i];
                    w[j].x = EL::pack2(with_bias(c[4 * j + 0], j, 0), with_bias(c[4 * j + 1], j, 1));
                    w[j].y = EL::pack2(with_bias(c[4 * j + 2], j, 2), with_bias(c[4 * j + 3], j, 3));
                }
                if constexpr (EPI == EPI_PLAIN) {
#pragma unroll
                    for (int j = 0; j < CB; ++j) stage_put_quiet<WN * 2>(img, put_row, j * 16 + put_col, w[j]);
                    stage_flush_quiet<WN * 2, 16>(img, args.D + off_d + (uint64_t)r0 * Ne + col0, Ne, rows_valid, cols_valid, el,
                                                  stream_out);
                } else {
                    // The product (rounded) is the gradient of the activation; h and its gradient are [rows, 2 Ne] with "up" in
                    // columns 0.., "gate" in columns Ne... A pass is 16 rows x 64 columns: a lane takes 8 columns of two rows,
                    // fetches the 8 up and 8 gate values of each (requested two passes ahead), and stores both gradients.
                    constexpr int kAhead = kBwdAhead;
                    if (i == 0) {
#pragma unroll
                        for (int a = 0; a < kAhead; ++a) bwd_request(a, col0, cols_valid);
                    }
#pragma unroll
                    for (int j = 0; j < CB; ++j) stage_put_quiet<WN * 2>(img, put_row, j * 16 + put_col, w[j]);
                    bwd_finish(i, col0, cols_valid);
                    if (i + kAhead < RB) bwd_request(i + kAhead, col0, cols_valid);
                }
            } else {
                // first the rounded pre-activation (32 "up" columns | 32 "gate" columns per row) of this row block, then,
                // after every second block, the activation of both
                constexpr int HB = WN * 2;
                constexpr int YB = WN;
                static_assert(CB == 4, "two up blocks and two gate blocks per wavefront and row block");
                const uint32_t col0 = n0 + wn * (WN / 2);
                const uint32_t cols_valid = col0 < n_lim ? n_lim - col0 : 0u;
                uint2 wu[2], wg[2];
#pragma unroll
                for (int jj = 0; jj < 2; ++jj) {
                    float u[4], g[4], y[4];
#pragma unroll
                    for (int x = 0; x < 4; ++x) {
                        u[x] = EL::round(with_bias(acc[i][4 * jj + x], jj, x));
                        g[x] = EL::round(with_bias(acc[i][4 * (2 + jj) + x], 2 + jj, x));
                        y[x] = u[x] * g[x] * sigmoid_for<typename EL::act_t>(g[x]);
                    }
                    ypack[i & 1][jj][0] = EL::pack2(y[0], y[1]);
                    ypack[i & 1][jj][1] = EL::pack2(y[2], y[3]);
                    if constexpr (EPI == EPI_SWIGLU) {
                        wu[jj].x = EL::pack2(u[0], u[1]);
                        wu[jj].y = EL::pack2(u[2], u[3]);
                        wg[jj].x = EL::pack2(g[0], g[1]);
                        wg[jj].y = EL::pack2(g[2], g[3]);
                    }
                }
                if constexpr (EPI == EPI_SWIGLU) {
#pragma unroll
                    for (int jj = 0; jj < 2; ++jj) {
                        stage_put_quiet<HB>(img, put_row, jj * 16 + put_col, wu[jj]);
                        stage_put_quiet<HB>(img, put_row, WN / 2 + jj * 16 + put_col, wg[jj]);
                    }
                    stage_flush_split_quiet<HB, 16, WN / 2>(img, args.D + off_d + (uint64_t)r0 * Ne + col0, Ne, rows_valid, cols_valid,
                                                            n_span, el);
                }
                if (i & 1) {
                    const uint32_t row0 = r0 - 16u;  // first row of the pair of blocks
                    const uint32_t rows_pair = row0 < Me ? (Me - row0 < 32u ? Me - row0 : 32u) : 0u;
#pragma unroll
                    for (int b = 0; b < 2; ++b)
#pragma unroll
                        for (int jj = 0; jj < 2; ++jj) {
                            uint2 wy;
                            wy.x = ypack[b][jj][0];
                            wy.y = ypack[b][jj][1];
                            stage_put_quiet<YB>(img, b * 16 + put_row, jj * 16 + put_col, wy);
                        }
                    stage_flush_quiet<YB, 32>(img, args.ACT + off_d / 2 + (uint64_t)row0 * n_span + col0, n_span, rows_pair, cols_valid, el);
                }
            }
        }

        // ---- on to the next tile ----
        streamed = stream_next;
        if (stream_next) {
            if constexpr (!GATHER) {
                fa_cur = fa_nxt;
                va_cur = va_nxt;
            }
            fb_cur = fb_nxt;
            vb_cur = vb_nxt;
        }
        cur = nxt;
        nxt = nn;
        ++round;
    }
}

// every instantiation the entry points launch (explicit, so that host stub and device code are both emitted)
#define FMA_RAGGED_INSTANTIATE(EL)                                                                          \
    template __global__ void ragged_gemm_kernel<EL, true, true, EPI_PLAIN, false, false, false>(const Args);    \
    template __global__ void ragged_gemm_kernel<EL, true, false, EPI_PLAIN, false, false, false>(const Args);   \
    template __global__ void ragged_gemm_kernel<EL, false, true, EPI_PLAIN, false, false, false>(const Args);   \
    template __global__ void ragged_gemm_kernel<EL, false, false, EPI_PLAIN, false, false, false>(const Args);  \
    template __global__ void ragged_gemm_kernel<EL, true, true, EPI_PLAIN, true, false, false>(const Args);     \
    template __global__ void ragged_gemm_kernel<EL, true, false, EPI_PLAIN, true, false, false>(const Args);    \
    template __global__ void ragged_gemm_kernel<EL, false, true, EPI_PLAIN, true, false, false>(const Args);    \
    template __global__ void ragged_gemm_kernel<EL, false, false, EPI_PLAIN, true, false, false>(const Args);   \
    template __global__ void ragged_gemm_kernel<EL, true, true, EPI_SWIGLU, false, false, false>(const Args);   \
    template __global__ void ragged_gemm_kernel<EL, true, true, EPI_SWIGLU_ACT, false, false, false>(const Args); \
    template __global__ void ragged_gemm_kernel<EL, true, true, EPI_PLAIN, false, true, false>(const Args);     \
    template __global__ void ragged_gemm_kernel<EL, true, true, EPI_SWIGLU, false, true, false>(const Args);    \
    template __global__ void ragged_gemm_kernel<EL, true, true, EPI_SWIGLU_ACT, false, true, false>(const Args); \
    template __global__ void ragged_gemm_kernel<EL, true, false, EPI_SWIGLU_BWD, false, false, false>(const Args); \
    template __global__ void ragged_gemm_kernel<EL, true, true, EPI_PLAIN, false, false, true>(const Args);     \
    template __global__ void ragged_gemm_kernel<EL, true, true, EPI_SWIGLU, false, false, true>(const Args);    \
    template __global__ void ragged_gemm_kernel<EL, true, true, EPI_SWIGLU_ACT, false, false, true>(const Args); \
    template __global__ void ragged_gemm_kernel<EL, true, true, EPI_PLAIN, false, true, true>(const Args);      \
    template __global__ void ragged_gemm_kernel<EL, true, true, EPI_SWIGLU, false, true, true>(const Args);     \
    template __global__ void ragged_gemm_kernel<EL, true, true, EPI_SWIGLU_ACT, false, true, true>(const Args); \
    template __global__ void ragged_gemm_kernel<EL, false, false, EPI_PLAIN, true, false, true>(const Args);
FMA_RAGGED_INSTANTIATE(ElemBf16)
FMA_RAGGED_INSTANTIATE(ElemF16)
#undef FMA_RAGGED_INSTANTIATE

template <typename EL, bool A_KC, bool B_KC, int EPI, bool VARY_K, bool BIAS = false, bool GATHER = false>
int launch(const Args& args, hipStream_t st) {
    int cus = num_compute_units();
    if (cus <= 0) cus = 256;
    hipLaunchKernelGGL((ragged_gemm_kernel<EL, A_KC, B_KC, EPI, VARY_K, BIAS, GATHER>), dim3((uint32_t)cus), dim3(NT), 0, st,
                       args);
    return launch_status("grouped_gemm_ragged");
}

// the forward (NT) kernels by epilogue, bias and gather
template <typename EL, int EPI>
int launch_forward(const Args& args, hipStream_t st) {
    const bool bias = args.bias != nullptr, gather = args.row_index != nullptr;
    if (bias && gather) return launch<EL, true, true, EPI, false, true, true>(args, st);
    if (bias) return launch<EL, true, true, EPI, false, true, false>(args, st);
    if (gather) return launch<EL, true, true, EPI, false, false, true>(args, st);
    return launch<EL, true, true, EPI, false, false, false>(args, st);
}

template <typename EL, bool VARY_K>
int launch_plain(const Args& args, bool a_kc, bool b_kc, hipStream_t st) {
    if (a_kc && b_kc) return launch<EL, true, true, EPI_PLAIN, VARY_K>(args, st);
    if (a_kc && !b_kc) return launch<EL, true, false, EPI_PLAIN, VARY_K>(args, st);
    if (!a_kc && b_kc) return launch<EL, false, true, EPI_PLAIN, VARY_K>(args, st);
    return launch<EL, false, false, EPI_PLAIN, VARY_K>(args, st);
}

// The forward product of an expert projection, out_e = x_e W_e^T (+ bias_e), with the rows of x_e packed (row_index
// NULL) or picked through row_index; swiglu: N = 2 I, out is the pre-activation (may be NULL) and act its activation.
int up_projection(const char* who, const void* x, int64_t x_rows, const int32_t* row_index, int32_t divisor, const void* W,
                  const void* bias, void* out, void* act, const uint32_t* M_arr, int64_t E, int64_t N, int64_t K, int swiglu,
                  int dtype, hipStream_t st) {
    FMA_REQUIRE(dtype == FMA_BF16 || dtype == FMA_F16, dtype_bytes(dtype) ? FMA_ERR_UNSUPPORTED : FMA_ERR_BAD_DTYPE,
                "%s: bf16 and fp16 operands are implemented (dtype code %d)", who, dtype);
    FMA_REQUIRE(E >= 0, FMA_ERR_BAD_SIZE, "%s: negative group count %lld", who, (long long)E);
    FMA_REQUIRE(E <= FMA_MAX_GROUPS, FMA_ERR_TOO_MANY_EXPERTS, "%s: E=%lld exceeds the limit %d", who, (long long)E,
                FMA_MAX_GROUPS);
    // the upper bounds are those of the kernel's 32-bit tile offsets; these entry points have no scalar path beyond them
    if (swiglu) {
        FMA_REQUIRE(N >= 16 && N % 16 == 0 && N < (1ll << 23), FMA_ERR_BAD_SIZE,
                    "%s: intermediate size %lld must be a positive multiple of 8 below 2^22", who, (long long)(N / 2));
    } else {
        FMA_REQUIRE(N >= 8 && N % 8 == 0 && N < (1ll << 23), FMA_ERR_BAD_SIZE,
                    "%s: N=%lld must be a positive multiple of 8 below 2^23", who, (long long)N);
    }
    FMA_REQUIRE(K >= 8 && K % 8 == 0 && K < (1ll << 21), FMA_ERR_BAD_SIZE,
                "%s: K=%lld must be a positive multiple of 8 below 2^21", who, (long long)K);
    if (E == 0) return FMA_OK;
    FMA_REQUIRE(x && W && M_arr && (swiglu ? act != nullptr : out != nullptr), FMA_ERR_NULL_POINTER, "%s: NULL pointer", who);
    FMA_REQUIRE(aligned16(x) && aligned16(W) && aligned16(act) && aligned16(out), FMA_ERR_MISALIGNED,
                "%s: x, W and the outputs must be 16-byte aligned", who);
    FMA_REQUIRE((reinterpret_cast<uintptr_t>(bias) & 3u) == 0 && (reinterpret_cast<uintptr_t>(row_index) & 3u) == 0,
                FMA_ERR_MISALIGNED, "%s: bias and row_index must be 4-byte aligned", who);
    Args args{};
    args.A = (const uint16_t*)x;
    args.B = (const uint16_t*)W;
    args.D = (uint16_t*)out;
    args.ACT = swiglu ? (uint16_t*)act : nullptr;
    args.sizes = M_arr;
    args.bias = (const uint16_t*)bias;
    args.row_index = row_index;
    args.divisor = (uint32_t)divisor;
    args.a_rows = (uint32_t)x_rows;
    args.E = (uint32_t)E;
    args.m = 0;
    args.n = (uint32_t)N;
    args.k = (uint32_t)K;
    args.alpha = 1.0f;
    // whether the pre-activation is stored is a compile-time property of the kernel: the epilogue is then one
    // straight-line block
    if (!swiglu) return dtype == FMA_BF16 ? launch_forward<ElemBf16, EPI_PLAIN>(args, st) : launch_forward<ElemF16, EPI_PLAIN>(args, st);
    if (out) return dtype == FMA_BF16 ? launch_forward<ElemBf16, EPI_SWIGLU>(args, st) : launch_forward<ElemF16, EPI_SWIGLU>(args, st);
    return dtype == FMA_BF16 ? launch_forward<ElemBf16, EPI_SWIGLU_ACT>(args, st) : launch_forward<ElemF16, EPI_SWIGLU_ACT>(args, st);
}

}  // namespace ragged

// fma_grouped_gemm's launch (per-group M, N and K arrays in device memory) offered to the two kernels of this file: each
// reads the arrays and runs only if the launch has its form (one varying dimension), otherwise it ends at once.
int launch_ragged_from_arrays(const void* A, const void* B, void* D, const uint32_t* M_arr, const uint32_t* N_arr,
                              const uint32_t* K_arr, int64_t E, bool a_kc, bool b_kc, float alpha, int dtype, hipStream_t st) {
    ragged::Args args{};
    args.A = (const uint16_t*)A;
    args.B = (const uint16_t*)B;
    args.D = (uint16_t*)D;
    args.E = (uint32_t)E;
    args.alpha = alpha;
    args.m_dev = M_arr;
    args.n_dev = N_arr;
    args.k_dev = K_arr;
    args.sizes = M_arr;
    int rc = dtype == FMA_BF16 ? ragged::launch_plain<ElemBf16, false>(args, a_kc, b_kc, st)
                               : ragged::launch_plain<ElemF16, false>(args, a_kc, b_kc, st);
    if (rc != FMA_OK) return rc;
    args.sizes = K_arr;
    return dtype == FMA_BF16 ? ragged::launch_plain<ElemBf16, true>(args, a_kc, b_kc, st)
                             : ragged::launch_plain<ElemF16, true>(args, a_kc, b_kc, st);
}

}  // namespace gemm
}  // namespace fmahip

extern "C" {


int fma_grouped_gemm_ragged(const void* A, const void* B, void* D, const uint32_t* sizes, const void* bias, int64_t E,
                            int vary, int64_t M, int64_t N, int64_t K, int trans_a, int trans_b, float alpha, int dtype,
                            void* stream) {
    using namespace fmahip;
    using namespace fmahip::gemm;
    FMA_REQUIRE(dtype == FMA_BF16 || dtype == FMA_F16, dtype_bytes(dtype) ? FMA_ERR_UNSUPPORTED : FMA_ERR_BAD_DTYPE,
                "grouped_gemm_ragged: bf16 and fp16 operands are implemented (dtype code %d)", dtype);
    FMA_REQUIRE(vary == FMA_VARY_M || vary == FMA_VARY_K, FMA_ERR_BAD_SIZE,
                "grouped_gemm_ragged: vary must be FMA_VARY_M or FMA_VARY_K (got %d)", vary);
    FMA_REQUIRE(E >= 0, FMA_ERR_BAD_SIZE, "grouped_gemm_ragged: negative group count %lld", (long long)E);
    FMA_REQUIRE(E <= FMA_MAX_GROUPS, FMA_ERR_TOO_MANY_EXPERTS, "grouped_gemm_ragged: E=%lld exceeds the limit %d",
                (long long)E, FMA_MAX_GROUPS);
    if (vary == FMA_VARY_M) M = 0;
    else K = 0;
    FMA_REQUIRE(M >= 0 && N >= 0 && K >= 0 && M <= 0xffffffffll && N <= 0xffffffffll && K <= 0xffffffffll, FMA_ERR_BAD_SIZE,
                "grouped_gemm_ragged: dimensions must lie in [0, 2^32) (M=%lld N=%lld K=%lld)", (long long)M, (long long)N,
                (long long)K);
    if (E == 0) return FMA_OK;
    FMA_REQUIRE(A && B && D && sizes, FMA_ERR_NULL_POINTER, "grouped_gemm_ragged: NULL pointer");
    FMA_REQUIRE(aligned16(A) && aligned16(B) && aligned16(D), FMA_ERR_MISALIGNED,
                "grouped_gemm_ragged: A, B and D must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    const bool a_kc = trans_a == 0;  // A stored [M, K]: reduction dim contiguous
    const bool b_kc = trans_b != 0;  // B stored [N, K]: reduction dim contiguous
    FMA_REQUIRE(!bias || (vary == FMA_VARY_M && a_kc && b_kc && alpha == 1.0f), FMA_ERR_UNSUPPORTED,
                "grouped_gemm_ragged: a bias is added in the forward form only (rows vary, A not transposed, B transposed, "
                "alpha 1)");
    // (with these sizes every tile takes the matrix-instruction path, the only one that adds the bias)
    FMA_REQUIRE(!bias || (N % 8 == 0 && K % 8 == 0 && N < (1 << 23) && K < (1 << 21)), FMA_ERR_UNSUPPORTED,
                "grouped_gemm_ragged: with a bias, N and K must be multiples of 8, N < 2^23 and K < 2^21");
    FMA_REQUIRE(!bias || (reinterpret_cast<uintptr_t>(bias) & 3u) == 0, FMA_ERR_MISALIGNED,
                "grouped_gemm_ragged: the bias must be 4-byte aligned");
    ragged::Args args{};
    args.A = (const uint16_t*)A;
    args.B = (const uint16_t*)B;
    args.D = (uint16_t*)D;
    args.ACT = nullptr;
    args.sizes = sizes;
    args.bias = (const uint16_t*)bias;
    args.E = (uint32_t)E;
    args.m = (uint32_t)M;
    args.n = (uint32_t)N;
    args.k = (uint32_t)K;
    args.alpha = alpha;
    if (bias)
        return dtype == FMA_BF16 ? ragged::launch_forward<ElemBf16, EPI_PLAIN>(args, st)
                                 : ragged::launch_forward<ElemF16, EPI_PLAIN>(args, st);
    if (vary == FMA_VARY_K)
        return dtype == FMA_BF16 ? ragged::launch_plain<ElemBf16, true>(args, a_kc, b_kc, st)
                                 : ragged::launch_plain<ElemF16, true>(args, a_kc, b_kc, st);
    return dtype == FMA_BF16 ? ragged::launch_plain<ElemBf16, false>(args, a_kc, b_kc, st)
                             : ragged::launch_plain<ElemF16, false>(args, a_kc, b_kc, st);
}

int fma_grouped_gemm_swiglu(const void* x, const void* W, const void* bias, void* h, void* act, const uint32_t* M_arr,
                            int64_t E, int64_t I, int64_t K, int dtype, void* stream) {
    return fmahip::gemm::ragged::up_projection("grouped_gemm_swiglu", x, 0, nullptr, 1, W, bias, h, act, M_arr, E, 2 * I, K,
                                               1, dtype, (hipStream_t)stream);
}

int fma_grouped_gemm_swiglu_bwd(const void* dy, const void* W, const void* h, void* dh, const uint32_t* M_arr, int64_t E,
                                int64_t I, int64_t K, int dtype, void* stream) {
    using namespace fmahip;
    using namespace fmahip::gemm;
    FMA_REQUIRE(dtype == FMA_BF16 || dtype == FMA_F16, dtype_bytes(dtype) ? FMA_ERR_UNSUPPORTED : FMA_ERR_BAD_DTYPE,
                "grouped_gemm_swiglu_bwd: bf16 and fp16 operands are implemented (dtype code %d)", dtype);
    FMA_REQUIRE(E >= 0, FMA_ERR_BAD_SIZE, "grouped_gemm_swiglu_bwd: negative group count %lld", (long long)E);
    FMA_REQUIRE(E <= FMA_MAX_GROUPS, FMA_ERR_TOO_MANY_EXPERTS, "grouped_gemm_swiglu_bwd: E=%lld exceeds the limit %d",
                (long long)E, FMA_MAX_GROUPS);
    // (with these sizes every tile takes the matrix-instruction path, the only one with this epilogue)
    FMA_REQUIRE(I >= 8 && I % 8 == 0 && I < (1ll << 22), FMA_ERR_BAD_SIZE,
                "grouped_gemm_swiglu_bwd: intermediate size %lld must be a positive multiple of 8 below 2^22", (long long)I);
    FMA_REQUIRE(K >= 8 && K % 8 == 0 && K < (1ll << 21), FMA_ERR_BAD_SIZE,
                "grouped_gemm_swiglu_bwd: K=%lld must be a positive multiple of 8 below 2^21", (long long)K);
    if (E == 0) return FMA_OK;
    FMA_REQUIRE(dy && W && h && dh && M_arr, FMA_ERR_NULL_POINTER, "grouped_gemm_swiglu_bwd: NULL pointer");
    FMA_REQUIRE(aligned16(dy) && aligned16(W) && aligned16(h) && aligned16(dh), FMA_ERR_MISALIGNED,
                "grouped_gemm_swiglu_bwd: dy, W, h and dh must be 16-byte aligned");
    ragged::Args args{};
    args.A = (const uint16_t*)dy;
    args.B = (const uint16_t*)W;
    args.D = (uint16_t*)dh;
    args.h_in = (const uint16_t*)h;
    args.sizes = M_arr;
    args.E = (uint32_t)E;
    args.m = 0;
    args.n = (uint32_t)I;
    args.k = (uint32_t)K;
    args.alpha = 1.0f;
    hipStream_t st = (hipStream_t)stream;
    return dtype == FMA_BF16 ? ragged::launch<ElemBf16, true, false, EPI_SWIGLU_BWD, false>(args, st)
                             : ragged::launch<ElemF16, true, false, EPI_SWIGLU_BWD, false>(args, st);
}

int fma_grouped_gemm_gathered_wgrad(const void* dy, const void* x, int64_t x_rows, const int32_t* row_index, int32_t divisor,
                                    void* dW, const uint32_t* K_arr, int64_t E, int64_t M, int64_t N, float alpha, int dtype,
                                    void* stream) {
    using namespace fmahip;
    using namespace fmahip::gemm;
    const char* who = "grouped_gemm_gathered_wgrad";
    FMA_REQUIRE(dtype == FMA_BF16 || dtype == FMA_F16, dtype_bytes(dtype) ? FMA_ERR_UNSUPPORTED : FMA_ERR_BAD_DTYPE,
                "%s: bf16 and fp16 operands are implemented (dtype code %d)", who, dtype);
    FMA_REQUIRE(E >= 0, FMA_ERR_BAD_SIZE, "%s: negative group count %lld", who, (long long)E);
    FMA_REQUIRE(E <= FMA_MAX_GROUPS, FMA_ERR_TOO_MANY_EXPERTS, "%s: E=%lld exceeds the limit %d", who, (long long)E,
                FMA_MAX_GROUPS);
    // (with these sizes every tile takes the matrix-instruction path, the only one that gathers)
    FMA_REQUIRE(M >= 8 && M % 8 == 0 && M < (1ll << 23) && N >= 8 && N % 8 == 0 && N < (1ll << 23), FMA_ERR_BAD_SIZE,
                "%s: M=%lld and N=%lld must be positive multiples of 8 below 2^23", who, (long long)M, (long long)N);
    FMA_REQUIRE(divisor >= 1 && divisor <= 65536, FMA_ERR_BAD_SIZE, "%s: divisor must lie in [1, 65536] (got %d)", who, divisor);
    if (E == 0) return FMA_OK;
    FMA_REQUIRE(dy && x && row_index && dW && K_arr, FMA_ERR_NULL_POINTER, "%s: NULL pointer", who);
    FMA_REQUIRE(x_rows >= 1, FMA_ERR_BAD_SIZE, "%s: x has no rows (%lld)", who, (long long)x_rows);
    // the loads address x with 32-bit byte offsets below 2^31
    FMA_REQUIRE(x_rows <= ((1ll << 31) - 1) / (2 * N), FMA_ERR_UNSUPPORTED,
                "%s: x must be smaller than 2 GiB (%lld rows of %lld elements)", who, (long long)x_rows, (long long)N);
    FMA_REQUIRE(aligned16(dy) && aligned16(x) && aligned16(dW), FMA_ERR_MISALIGNED, "%s: dy, x and dW must be 16-byte aligned", who);
    FMA_REQUIRE((reinterpret_cast<uintptr_t>(row_index) & 3u) == 0, FMA_ERR_MISALIGNED, "%s: row_index must be 4-byte aligned", who);
    ragged::Args args{};
    args.A = (const uint16_t*)dy;
    args.B = (const uint16_t*)x;
    args.D = (uint16_t*)dW;
    args.sizes = K_arr;
    args.row_index = row_index;
    args.divisor = (uint32_t)divisor;
    args.a_rows = (uint32_t)x_rows;
    args.E = (uint32_t)E;
    args.m = (uint32_t)M;
    args.n = (uint32_t)N;
    args.k = 0;
    args.alpha = alpha;
    hipStream_t st = (hipStream_t)stream;
    return dtype == FMA_BF16 ? ragged::launch<ElemBf16, false, false, EPI_PLAIN, true, false, true>(args, st)
                             : ragged::launch<ElemF16, false, false, EPI_PLAIN, true, false, true>(args, st);
}

int fma_grouped_gemm_gathered(const void* x, int64_t x_rows, const int32_t* row_index, int32_t divisor, const void* W,
                              const void* bias, void* out, void* act, const uint32_t* M_arr, int64_t E, int64_t N,
                              int64_t K, int swiglu, int dtype, void* stream) {
    using namespace fmahip;
    FMA_REQUIRE(row_index != nullptr || E == 0, FMA_ERR_NULL_POINTER, "grouped_gemm_gathered: row_index is NULL");
    FMA_REQUIRE(divisor >= 1 && divisor <= 65536, FMA_ERR_BAD_SIZE,
                "grouped_gemm_gathered: divisor must lie in [1, 65536] (got %d)", divisor);
    FMA_REQUIRE(x_rows >= 1 || E == 0, FMA_ERR_BAD_SIZE, "grouped_gemm_gathered: x has no rows (%lld)", (long long)x_rows);
    // the loads address x with 32-bit byte offsets below 2^31
    FMA_REQUIRE(K <= 0 || x_rows <= ((1ll << 31) - 1) / (2 * K), FMA_ERR_UNSUPPORTED,
                "grouped_gemm_gathered: x must be smaller than 2 GiB (%lld rows of %lld elements)", (long long)x_rows,
                (long long)K);
    return gemm::ragged::up_projection("grouped_gemm_gathered", x, x_rows, row_index, divisor, W, bias, out, act, M_arr, E,
                                       N, K, swiglu, dtype, (hipStream_t)stream);
}

}  // extern "C"
