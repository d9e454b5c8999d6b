// Grouped GEMM over ragged expert groups for gfx950: bf16 or fp16 operands, fp32 accumulation on the matrix cores
// (v_mfma_f32_32x32x16_bf16 / _f16), optional SwiGLU epilogue.
//
// Shape of the kernel
//  * Persistent: the grid is one workgroup per compute unit. Each workgroup builds the group table (tile
//    prefix and packed element offsets of every group) in LDS from the device-side M/N/K arrays, then walks
//    256x256 output tiles. Groups enter the tile sequence longest reduction first and rounds of tiles are dealt in
//    alternating directions (balance under ragged reduction lengths); within a round the 32 workgroups of one XCD
//    (workgroup id mod 8) hold a compact 8x4 block of tiles of the same group: they share A and B panels in that
//    XCD's L2.
//  * K is consumed in steps of 64 through two LDS stages of 2 x 32 KB. Every operand tile goes global -> LDS directly
//    (buffer_load_dwordx4 ... lds, 1 KB per wavefront instruction, no staging registers; the buffer descriptor's range
//    check zero-fills rows and reduction steps past the edge of a group), in one of two layouts:
//      - an operand whose reduction dimension is contiguous in memory is kept as [row][64 k] (128-byte rows); row r,
//        16-byte chunk c sits at phys_row(r)*128 + ((c ^ (r & 7)) << 4), phys_row rotating the low four row bits
//        left by one, and an MFMA fragment (32 rows x 16 k) is one ds_read_b128 per lane;
//      - an operand stored with the reduction dimension as the row index is kept as it is in memory, [64 k][256 out]
//        (512-byte rows), chunk c of row k at k*512 + ((c ^ (4*(k & 3))) << 4), and a fragment is two
//        ds_read_b64_tr_b16 per lane: the transposing LDS read hands lane i of a 16-lane group the four k values of
//        out column i when lane j of the group addresses row j/4, columns 4*(j%4)..+3.
//    Both swizzles are applied on the source side of the direct load (which lane fetches which chunk) and make the
//    fragment reads touch every LDS bank once per pass.
//  * Fragments are double buffered in registers and the workgroup barrier of a K step sits before the MFMAs of its
//    last k slice, so the LDS and barrier latencies are covered by matrix work.
//  * The MFMA is issued with B as the first operand, so a lane ends up holding four consecutive output
//    columns of one output row. The epilogue transposes the wavefront's sub-tile through LDS (stage 1) and stores
//    whole 128-byte row segments; the next tile's first loads are already on their way into stage 0 by then.
#include "gemm_parts.h"
#include "grouped_gemm_f32.h"

namespace fmahip {
namespace gemm {

// how the load instructions of a K step are spread over the slices after the barrier that frees their stage
constexpr uint32_t kPfDist = 4;  // K steps between a line's prefetch and the step that loads it
// how many of a K step's eight loads per wavefront go out in the last k slice of the step (kLoadsS3) and in the first
// three slices of the next one
constexpr int kLoadsS3 = 8, kLoadsS0 = 0, kLoadsS1 = 0, kLoadsS2 = 0;



struct GemmArgs {
    const uint16_t* A;
    const uint16_t* B;
    uint16_t* D;    // plain: output; swiglu: pre-activation h (may be NULL)
    uint16_t* ACT;  // swiglu only: activation output
    const uint32_t* M_arr;  // NULL: every group uses const_m
    const uint32_t* N_arr;  // NULL: every group uses const_n
    const uint32_t* K_arr;  // NULL: every group uses const_k
    uint32_t E;
    uint32_t const_m;
    uint32_t const_n;
    uint32_t const_k;
    float alpha;
    // fma_grouped_gemm also offers its launch to the kernels of grouped_gemm_ragged.hip, which take it when the groups differ
    // in one dimension only; with this flag set the kernel here applies the same test and ends at once in that case
    uint32_t only_if_irregular;
};

template <typename EL, int NWM, int NWN, bool A_KC, bool B_KC, int EPI>
__global__ __launch_bounds__(NWM* NWN * 64) void grouped_gemm_kernel(const GemmArgs args) {
    constexpr int NW = NWM * NWN;
    constexpr int NT = NW * 64;
    constexpr int WM = BM / NWM;
    constexpr int WN = BN / NWN;
    constexpr int FM = WM / 32;
    constexpr int FN = WN / 32;
    static_assert(EPI == EPI_PLAIN || (A_KC && B_KC), "the SwiGLU epilogue exists for the NT layout only");

    // one array per stage and operand: distinct LDS objects let the compiler see that a direct-to-LDS load
    // into one stage cannot alias the fragment reads of the other, so it does not wait for the load first
    __shared__ __attribute__((aligned(1024))) uint8_t s_a0[kTileBytes];
    __shared__ __attribute__((aligned(1024))) uint8_t s_b0[kTileBytes];
    __shared__ __attribute__((aligned(1024))) uint8_t s_a1[kTileBytes];
    __shared__ __attribute__((aligned(1024))) uint8_t s_b1[kTileBytes];
    __shared__ uint32_t s_pf[64];  // where the dwords fetched by the L2 prefetch end up (never read)
    __shared__ uint32_t s_tile_start[FMA_MAX_GROUPS + 1];  // first tile of the group at position p of the tile sequence
    __shared__ uint16_t s_order[FMA_MAX_GROUPS];           // which group that is
    __shared__ uint64_t s_off_a[FMA_MAX_GROUPS + 1];
    __shared__ uint64_t s_off_b[FMA_MAX_GROUPS + 1];
    __shared__ uint64_t s_off_d[FMA_MAX_GROUPS + 1];

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t wm = wave / NWN;
    const uint32_t wn = wave % NWN;
    const uint32_t E = args.E;

    // The size arrays are read through the constant address space: with a wavefront-uniform index that is a scalar
    // load (nothing writes the arrays while the kernel runs), not a vector load that every tile would wait for.
    typedef const __attribute__((address_space(4))) uint32_t* const_u32_ptr;
    const const_u32_ptr m_arr = (const_u32_ptr)args.M_arr, n_arr = (const_u32_ptr)args.N_arr, k_arr = (const_u32_ptr)args.K_arr;
    auto group_m = [&](uint32_t e) { return m_arr ? m_arr[e] : args.const_m; };
    auto group_n = [&](uint32_t e) { return n_arr ? n_arr[e] : args.const_n; };
    auto group_k = [&](uint32_t e) { return k_arr ? k_arr[e] : args.const_k; };
    if (args.only_if_irregular) {
        // (the test of ragged_gemm_kernel: rows vary with N and K shared, or the reduction varies with M and N shared)
        const uint32_t m0 = group_m(0), n0 = group_n(0), k0 = group_k(0);
        bool m_differs = false, n_differs = false, k_differs = false;
        for (uint32_t e = tid; e < E; e += NT) {
            m_differs = m_differs || args.M_arr[e] != m0;
            n_differs = n_differs || args.N_arr[e] != n0;
            k_differs = k_differs || args.K_arr[e] != k0;
        }
        const bool m_same = !__syncthreads_or(m_differs), n_same = !__syncthreads_or(n_differs), k_same = !__syncthreads_or(k_differs);
        if ((n_same && k_same) || (m_same && n_same)) return;
    }
    // Column tiles of half the width for groups of at most 64 rows (a few rows per group: the kernel is then a stream of
    // the B operand), when that fills the workgroups better: a launch with tiles for at most half of them, or one made of
    // such groups only whose last round of tiles would be at most half full. Decided once per launch, below, from the
    // group sizes; NT only (a reduction-major B operand is loaded in rows of 256 columns whatever the tile's width).
    constexpr bool kCanNarrow = A_KC && B_KC;
    constexpr uint32_t kTileN = EPI != EPI_PLAIN ? BN / 2 : BN;  // columns of the tile grid one tile covers
    bool narrow = false;
    // n-extent covered by the tile grid: for the SwiGLU epilogue a tile spans 128 up + 128 gate columns
    auto tiles_of = [&](uint32_t m, uint32_t n) -> uint32_t {
        if (m == 0 || n == 0) return 0;
        const uint32_t span = EPI != EPI_PLAIN ? n / 2 : n;
        const uint32_t width = (kCanNarrow && narrow && m <= 64u) ? kTileN / 2 : kTileN;
        return ((m + BM - 1) / BM) * ((span + width - 1) / width);
    };

    // ---- order of the groups in the tile sequence: by K steps per tile, longest first ----
    // With the reduction length varying between groups (weight gradients: it is the number of rows routed to the expert)
    // tiles differ in cost; handing them out expensive-first, in alternating directions (below), keeps the workgroups'
    // totals close. Ranks come from an all-pairs comparison over keys parked in the (still unused) LDS stages; groups of
    // equal cost keep their order, and when every group costs the same the order is the identity.
    {
        uint32_t* const key = reinterpret_cast<uint32_t*>(s_a0);  // K steps per tile of group e; 0 if it has no tiles
        const uint32_t key0 = tiles_of(group_m(0), group_n(0)) ? (group_k(0) + BK - 1) / BK : 0u;
        bool differs = false;
        for (uint32_t e = tid; e < E; e += NT) {
            const uint32_t k = tiles_of(group_m(e), group_n(e)) ? (group_k(e) + BK - 1) / BK : 0u;
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
        // tiles of the launch at full width, those of small groups apart; every thread adds up its groups
        uint32_t mine_small = 0, mine_other = 0;
        for (uint32_t e = tid; e < E; e += NT) {
            const uint32_t m = group_m(e), t = tiles_of(m, group_n(e));
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
        const uint32_t rounds = (t_small + t_other + g - 1) / g;  // as it is; at half width: half-cost rounds
        const uint32_t half_rounds = (2 * t_small + g - 1) / g;
        narrow = t_other == 0 ? half_rounds * 10u <= 2u * rounds * 9u : (t_small + t_other) * 2u <= g;
        __syncthreads();
    }

    // ---- group table, built by wavefront 0: exclusive prefix of tiles over the order above, exclusive prefixes of the
    // packed element counts over the groups as they lie in memory ----
    if (wave == 0) {
        uint32_t carry_t = 0;
        uint64_t carry_a = 0, carry_b = 0, carry_d = 0;
        for (uint32_t base = 0; base < E; base += 64) {
            const uint32_t e = base + lane;
            uint32_t m = 0, n = 0, k = 0, t = 0;
            if (e < E) {
                m = group_m(e);
                n = group_n(e);
                k = group_k(e);
                const uint32_t at = s_order[e];  // the group at position e of the tile sequence
                t = tiles_of(group_m(at), group_n(at));
            }
            const uint64_t sa = (uint64_t)m * k, sb = (uint64_t)k * n, sd = (uint64_t)m * n;
            const uint32_t it = wave_inclusive_scan<uint32_t>(t);
            const uint64_t ia = wave_inclusive_scan<uint64_t>(sa);
            const uint64_t ib = wave_inclusive_scan<uint64_t>(sb);
            const uint64_t id = wave_inclusive_scan<uint64_t>(sd);
            if (e < E) {
                s_tile_start[e] = carry_t + it - t;
                s_off_a[e] = carry_a + ia - sa;
                s_off_b[e] = carry_b + ib - sb;
                s_off_d[e] = carry_d + id - sd;
            }
            carry_t += __shfl(it, 63, 64);
            carry_a += __shfl(ia, 63, 64);
            carry_b += __shfl(ib, 63, 64);
            carry_d += __shfl(id, 63, 64);
        }
        if (lane == 0) {
            s_tile_start[E] = carry_t;
            s_off_a[E] = carry_a;
            s_off_b[E] = carry_b;
            s_off_d[E] = carry_d;
        }
    }
    __syncthreads();
    const uint32_t total_tiles = s_tile_start[E];

    // first tile row of B fragment j of this wavefront
    auto b_frag_row = [&](int j) -> uint32_t {
        if constexpr (EPI != EPI_PLAIN) {
            return j < FN / 2 ? wn * (WN / 2) + j * 32 : BN / 2 + wn * (WN / 2) + (j - FN / 2) * 32;
        } else {
            return wn * WN + j * 32;
        }
    };
    // per-lane LDS byte offsets of this wavefront's fragments for k slice 0 (slice ks adds a constant)
    uint32_t a_off[FM], b_off[FN];
#pragma unroll
    for (int i = 0; i < FM; ++i) {
        const uint32_t r0 = wm * WM + i * 32;
        a_off[i] = A_KC ? r0 * kRowBytes : mc_frag_off(r0, lane);
    }
#pragma unroll
    for (int j = 0; j < FN; ++j) {
        const uint32_t r0 = b_frag_row(j);
        b_off[j] = B_KC ? r0 * kRowBytes : mc_frag_off(r0, lane);
    }
    // [row][64 k] tiles: offset of this lane's row and chunk inside a 32-row fragment, per k slice
    uint32_t kc_slice[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) kc_slice[ks] = kc_off(lane & 31u, (uint32_t)ks * 2u + (lane >> 5));

    // workgroup id -> position in the round of gridDim.x tiles: workgroups of one XCD take 32 neighbours
    const uint32_t grid = gridDim.x;
    const uint32_t per_xcd = grid / kXcds;
    const uint32_t slot = (grid % kXcds == 0) ? (blockIdx.x % kXcds) * per_xcd + blockIdx.x / kXcds : blockIdx.x;

    // Everything that identifies one output tile; the same in every lane.
    struct Tile {
        bool valid, fast;
        uint32_t Me, Ne, Ke, n_span, m0, n0, n_lim;  // n_lim: first column past the tile (kTileN columns wide, or half of that)
        uint64_t off_a, off_b, off_d;
        uint32_t pf_r, pf_c;  // position of the tile in its XCD's 8 x 4 block of tiles (row, column)
    };
    // Rounds of `grid` tiles are dealt in alternating directions (slot s takes tile s of even rounds and tile
    // grid-1-s of odd ones): when the tiles get cheaper along the tile order (groups with shrinking reduction length, as in
    // weight gradients under skewed routing) a workgroup that drew an expensive tile in one round draws a cheap one in the
    // next. Blocks of 32 neighbouring tiles still go to one XCD. Only the last round can leave a slot without a tile.
    auto lookup = [&](uint32_t round) -> Tile {
        Tile t{};
        const uint32_t v = round * grid + ((round & 1u) ? grid - 1u - slot : slot);
        if ((uint64_t)round * grid >= total_tiles || v >= total_tiles) return t;
        uint32_t lo = 0, hi = E;
        while (lo < hi) {
            const uint32_t mid = (lo + hi) >> 1;
            if (s_tile_start[mid + 1] <= v) lo = mid + 1;
            else hi = mid;
        }
        const uint32_t pos = uniform(lo);
        const uint32_t e = uniform((uint32_t)s_order[pos]);
        t.valid = true;
        t.Me = group_m(e);
        t.Ne = group_n(e);
        t.Ke = group_k(e);
        t.n_span = EPI != EPI_PLAIN ? t.Ne / 2 : t.Ne;  // columns the tile grid runs over
        const uint32_t tiles_m = (t.Me + BM - 1) / BM;
        const uint32_t tile_n = (kCanNarrow && narrow && t.Me <= 64u) ? kTileN / 2 : kTileN;
        const uint32_t tiles_n = (t.n_span + tile_n - 1) / tile_n;
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
        t.n_lim = t.n_span - t.n0 < tile_n ? t.n_span : t.n0 + tile_n;
        t.off_a = uniform(s_off_a[e]);
        t.off_b = uniform(s_off_b[e]);
        t.off_d = uniform(s_off_d[e]);
        // 16-byte accesses need: every contiguous dimension a multiple of 8 elements (K for an operand whose
        // reduction dim is contiguous, M / N for one stored reduction-major, N for the output rows) and packed
        // group bases that stayed multiples of 8. A ragged reduction length is fine for reduction-major operands.
        // Loads and stores address a tile with 32-bit byte offsets below 2^31: 256 rows of K elements, 64 rows of M / N.
        bool fast = (t.Ne % 8u == 0) && (t.Ne < (1u << 23)) && (t.off_a % 8u == 0) && (t.off_b % 8u == 0) &&
                    (t.off_d % 8u == 0);
        if (A_KC || B_KC) fast = fast && (t.Ke % 8u == 0) && (t.Ke < (1u << 21));
        if (!A_KC) fast = fast && (t.Me % 8u == 0) && (t.Me < (1u << 23));
        if (EPI != EPI_PLAIN) fast = fast && (t.n_span % 8u == 0);
        t.fast = fast;
        return t;
    };

    // ---- loaders (state of the tile whose operands are being loaded) ----
    LoaderK<NW, false> lk_a;
    LoaderK<NW, EPI != EPI_PLAIN> lk_b;
    LoaderT<NW> lt_a, lt_b;
    auto setup_loaders = [&](const Tile& t) {
        const uint16_t* Ae = args.A + t.off_a;
        const uint16_t* Be = args.B + t.off_b;
        if constexpr (A_KC) {
            lk_a.setup(Ae + (uint64_t)t.m0 * t.Ke, nullptr, t.Me - t.m0 < (uint32_t)BM ? t.Me - t.m0 : (uint32_t)BM, t.Ke,
                       wave, lane);
        } else {
            lt_a.setup(Ae, t.Me, t.Ke, t.m0, wave, lane);
        }
        if constexpr (B_KC) {
            if constexpr (EPI != EPI_PLAIN) {
                // tile rows 0..127: "up" rows n0.. of the weight; rows 128..255: "gate" rows I + n0..
                const uint32_t rows = t.n_lim - t.n0;
                lk_b.setup(Be + (uint64_t)t.n0 * t.Ke, Be + (uint64_t)(t.n_span + t.n0) * t.Ke, rows, t.Ke, wave, lane);
            } else {
                lk_b.setup(Be + (uint64_t)t.n0 * t.Ke, nullptr, t.n_lim - t.n0, t.Ke, wave, lane);
            }
        } else {
            lt_b.setup(Be, t.Ne, t.Ke, t.n0, wave, lane);
        }
    };
    // ---- L2 prefetch by designated workgroups ----
    // The 32 workgroups of an XCD work on an 8 x 4 block of tiles: an A panel is shared by the 4 tiles of a block row, a
    // B panel by the 8 tiles of a block column, and whichever workgroup asks for a 128-byte line first waits for it to
    // come from beyond the L2 while the K step's window is one step long. Every workgroup therefore requests, kPfDist K
    // steps ahead, its share of the lines its block neighbours will load (a quarter of its A tile's lines, an eighth of
    // its B tile's): one 4-byte load per line and one instruction per wavefront and K step (even wavefronts: A, 16
    // lanes each; odd ones: B, 8 lanes each; the other lanes are out of the descriptor's range and fetch nothing).
    uint32_t pf_voff = kOutOfRange;
    const uint16_t* pf_base = nullptr;
    uint32_t pf_bytes = 0, pf_ldb = 0, pf_col_bytes = 0, pf_kdim = 0;
    const bool pf_is_b = (wave & 1u) != 0;
    const bool pf_t = pf_is_b ? !B_KC : !A_KC;  // reduction-major operand: the descriptor moves with the K step
    auto setup_prefetch = [&](const Tile& t) {
        const uint32_t p = wave >> 1;  // 0..3 among the wavefronts that serve the same operand
        if (!pf_is_b) {
            const uint32_t i = p * 16u + lane;  // 64 lines of the A tile's 256
            if constexpr (A_KC) {
                pf_base = lk_a.base0; pf_bytes = lk_a.bytes;
                pf_voff = lane < 16u ? (4u * i + t.pf_c) * lk_a.ldb : kOutOfRange;
            } else {
                pf_base = lt_a.base; pf_ldb = lt_a.ldb; pf_col_bytes = lt_a.col_bytes; pf_kdim = lt_a.kdim;
                pf_voff = lane < 16u ? i * lt_a.ldb + t.pf_c * 128u : kOutOfRange;
            }
        } else {
            if constexpr (B_KC) {
                pf_bytes = lk_b.bytes;
                if constexpr (EPI != EPI_PLAIN) {
                    pf_base = (p >> 1) ? lk_b.base1 : lk_b.base0;  // "up" rows, "gate" rows
                    pf_voff = lane < 8u ? (8u * ((p & 1u) * 8u + lane) + t.pf_r) * lk_b.ldb : kOutOfRange;
                } else {
                    pf_base = lk_b.base0;
                    pf_voff = lane < 8u ? (8u * (p * 8u + lane) + t.pf_r) * lk_b.ldb : kOutOfRange;
                }
            } else {
                pf_base = lt_b.base; pf_ldb = lt_b.ldb; pf_col_bytes = lt_b.col_bytes; pf_kdim = lt_b.kdim;
                pf_voff = lane < 8u ? (2u * (p * 8u + lane) + (t.pf_r >> 2)) * lt_b.ldb + (t.pf_r & 3u) * 128u : kOutOfRange;
            }
        }
    };
    // requests this wavefront's lines of K step `kstep` (any value: past the end of K it fetches nothing or a line of a
    // later row, which is valid memory inside the descriptor's range)
    // (measured on the Mixtral shapes: +1 point of peak where both operands have the same storage order; with one of
    // each, where the two halves of the workgroup build different descriptors per step, -1.5: switched off there)
    constexpr bool kPrefetch = A_KC == B_KC;
    auto issue_prefetch = [&](uint32_t kstep) {
        if constexpr (!kPrefetch) return;
        const uint32_t k0 = kstep * (uint32_t)BK;
        const uint32_t rows = k0 >= pf_kdim ? 0u : (pf_kdim - k0 < (uint32_t)BK ? pf_kdim - k0 : (uint32_t)BK);
        const uint16_t* base = pf_t ? pf_base + (uint64_t)k0 * (pf_ldb / 2u) : pf_base;
        const uint32_t bytes = pf_t ? (rows ? rows * pf_ldb - pf_col_bytes : 0u) : pf_bytes;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(make_rsrc(base, bytes), (lds_void*)s_pf, 4, pf_voff, pf_t ? 0u : k0 * 2u, 0, 0);
    };
    // loads of the K step at k0 into `stage`: inside the K loop (compiler-visible, placed by the scheduling hints) ...
    auto issue = [&](int stage, uint32_t k0) {
        if constexpr (A_KC) lk_a.issue(stage ? s_a1 : s_a0, k0);
        else lt_a.issue(stage ? s_a1 : s_a0, k0);
        if constexpr (B_KC) lk_b.issue(stage ? s_b1 : s_b0, k0);
        else lt_b.issue(stage ? s_b1 : s_b0, k0);
    };
    // load instructions FIRST .. FIRST+COUNT-1 of a K step (the A operand's come first)
    auto issue_some = [&](auto first_c, auto count_c, int stage, uint32_t k0) {
        constexpr int FIRST = decltype(first_c)::value, COUNT = decltype(count_c)::value;
        constexpr int NI = 32 / NW;
        constexpr int A0 = FIRST < NI ? FIRST : NI, A1 = FIRST + COUNT < NI ? FIRST + COUNT : NI;
        constexpr int B0 = FIRST > NI ? FIRST - NI : 0, B1 = FIRST + COUNT > NI ? FIRST + COUNT - NI : 0;
        if constexpr (A1 > A0) {
            if constexpr (A_KC) lk_a.template issue_range<A0, A1>(stage ? s_a1 : s_a0, k0);
            else lt_a.template issue_range<A0, A1>(stage ? s_a1 : s_a0, k0);
        }
        if constexpr (B1 > B0) {
            if constexpr (B_KC) lk_b.template issue_range<B0, B1>(stage ? s_b1 : s_b0, k0);
            else lt_b.template issue_range<B0, B1>(stage ? s_b1 : s_b0, k0);
        }
    };
    // ... and at the head of a tile
    auto issue_quiet_a = [&](int stage, uint32_t k0) {
        if constexpr (A_KC) lk_a.issue_quiet(stage ? s_a1 : s_a0, k0);
        else lt_a.issue_quiet(stage ? s_a1 : s_a0, k0);
    };
    auto issue_quiet_b = [&](int stage, uint32_t k0) {
        if constexpr (B_KC) lk_b.issue_quiet(stage ? s_b1 : s_b0, k0);
        else lt_b.issue_quiet(stage ? s_b1 : s_b0, k0);
    };
    auto issue_quiet = [&](int stage, uint32_t k0) {
        issue_quiet_a(stage, k0);
        issue_quiet_b(stage, k0);
    };
    constexpr uint32_t kStepLoads = 2 * (32 / NW);  // load instructions per wavefront and K step
    // store instructions per wavefront and tile (stage_flush issues a fixed number)
    const uint32_t tile_stores = EPI == EPI_PLAIN ? WM * WN * 2 / 1024 : (EPI == EPI_SWIGLU ? WM * WN * 2 / 1024 : 0) + WM * WN / 1024;
    // waits until at most n of this wavefront's loads and stores are outstanding (they complete in issue order).
    // The counts passed here are the instructions this source issues: they are valid only while the compiler adds no
    // memory instructions of its own, i.e. while the kernel has no register spills (the build fails if it has any).
    auto wait_outstanding = [&](uint32_t n) {
        if (n >= 40) __builtin_amdgcn_s_waitcnt(0x8f78);       // vmcnt(40)
        else if (n >= 32) __builtin_amdgcn_s_waitcnt(0x8f70);  // vmcnt(32)
        else if (n >= 24) __builtin_amdgcn_s_waitcnt(0x4f78);  // vmcnt(24)
        else if (n >= 16) __builtin_amdgcn_s_waitcnt(0x4f70);  // vmcnt(16)
        else if (n >= 8) __builtin_amdgcn_s_waitcnt(0x0f78);   // vmcnt(8)
        else if (n >= 5) __builtin_amdgcn_s_waitcnt(0x0f75);   // vmcnt(5)
        else __builtin_amdgcn_s_waitcnt(0x0f70);               // vmcnt(0)
    };

    uint32_t round = 0;
    Tile cur = lookup(0);
    // prefetched: the loaders are set up for `cur` and the loads of its first K step went out (into stage 0) before the
    // epilogue of the previous tile, followed by exactly tile_stores stores
    bool prefetched = false;
    // prefetched_b1: the B operand of its second K step is on its way into stage 1 as well (the A half of stage 1 is the
    // epilogue's staging space, so A's second step follows the epilogue)
    bool prefetched_b1 = false;
    while (cur.valid) {
        const uint32_t Me = cur.Me, Ne = cur.Ne, Ke = cur.Ke, n_span = cur.n_span, m0 = cur.m0, n0 = cur.n0, n_lim = cur.n_lim;
        const uint64_t off_d = cur.off_d;

        if (!prefetched) {
            if (!cur.fast) {
                if constexpr (EPI == EPI_PLAIN) {
                    scalar_tile<EL, A_KC, B_KC, BM, BN>(args.A + cur.off_a, args.B + cur.off_b, args.D + off_d, Me, Ne, Ke, m0, n0,
                                                args.alpha, NT);
                }
                cur = lookup(++round);
                continue;
            }
            setup_loaders(cur);
            setup_prefetch(cur);
        }
        f32x16 acc[FM][FN];
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int x = 0; x < 16; ++x) acc[i][j][x] = 0.0f;

        // MFMA operand fragments of one 16-wide k slice, double buffered in registers
        // The K loop exists in four versions, for wavefronts whose first FA = 4, 2, 1 or 0 row blocks (of 32 rows) hold
        // rows of the group: the other blocks would multiply rows that the loads zero-filled, so their LDS reads and
        // MFMAs are left out (their accumulators stay zero and the stores mask them). The last row tile of a group, and
        // every tile of a group with few rows, then costs what its loads cost instead of a full tile's matrix work.
        // FA is passed as an integral_constant so that each version is straight-line code.
        typename EL::frag fa[2][FM], fb[2][FN];
        auto load_frags = [&](auto fa_c, int stage, int ks, int buf) {
            constexpr int FA = decltype(fa_c)::value;
            if constexpr (FA > 0) {
                const uint8_t* ta = stage ? s_a1 : s_a0;
                const uint8_t* tb = stage ? s_b1 : s_b0;
#pragma unroll
                for (int i = 0; i < FA; ++i) {
                    if constexpr (A_KC) fa[buf][i] = __builtin_bit_cast(typename EL::frag, read_kc_frag(ta + a_off[i] + kc_slice[ks]));
                    else fa[buf][i] = __builtin_bit_cast(typename EL::frag, read_tr_frag(ta + a_off[i] + ks * 16 * kTRowBytes));
                }
#pragma unroll
                for (int j = 0; j < FN; ++j) {
                    if constexpr (B_KC) fb[buf][j] = __builtin_bit_cast(typename EL::frag, read_kc_frag(tb + b_off[j] + kc_slice[ks]));
                    else fb[buf][j] = __builtin_bit_cast(typename EL::frag, read_tr_frag(tb + b_off[j] + ks * 16 * kTRowBytes));
                }
            }
        };
        auto mma = [&](auto fa_c, int buf) {
            constexpr int FA = decltype(fa_c)::value;
#pragma unroll
            for (int i = 0; i < FA; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    acc[i][j] = EL::mfma(fb[buf][j], fa[buf][i], acc[i][j]);
        };
        // ask the scheduler to alternate the MFMAs of one slice with the LDS reads of the next
        auto interleave_reads = [&](auto fa_c) {
            constexpr int FA = decltype(fa_c)::value;
            constexpr int kReads = (A_KC ? FA : 2 * FA) + (B_KC ? FN : 2 * FN);
            if constexpr (FA > 0) interleave_mfma_lds<0, FA * FN, kReads>();
        };

        // ---- main loop over K ----
        // Step kt computes from stage kt&1. The workgroup barrier of a step sits between the LDS reads of its last
        // k slice and the MFMAs of that slice: once it is passed, the stage just read is free (the loads of step kt+2
        // are issued into it) and the other stage is complete (its first fragments are fetched), and both overlap
        // with the MFMAs still to be issued, so the matrix pipe has work while the barrier's latencies play out.
        // The 2*(32/NW) loads of a K step are spread over the four slices that follow the barrier which frees their stage:
        // kLd3 of them in the last slice of the step that frees it, kLd0 / kLd1 / kLd2 in slices 0 / 1 / 2 of the next step.
        // A burst right after the barrier fills the address unit's queue; the wavefronts then block at a load with their
        // matrix instructions behind it.
        auto step = [&](auto fa_c, int stage, uint32_t kt) {
            constexpr int FA = decltype(fa_c)::value;
            constexpr int kReads = (A_KC ? FA : 2 * FA) + (B_KC ? FN : 2 * FN);
            using L3 = std::integral_constant<int, kLoadsS3>;
            using L0 = std::integral_constant<int, kLoadsS0>;
            using L1 = std::integral_constant<int, kLoadsS1>;
            using L2 = std::integral_constant<int, kLoadsS2>;
            static_assert(kLoadsS3 + kLoadsS0 + kLoadsS1 + kLoadsS2 == 2 * (32 / NW), "every load of a step is issued once");
            load_frags(fa_c, stage, 1, 1);
            issue_some(L3{}, L0{}, stage ^ 1, (kt + 1) * BK);
            mma(fa_c, 0);
            if constexpr (FA > 0) interleave3<0, FA * FN, kReads, kLoadsS0>();
            load_frags(fa_c, stage, 2, 0);
            issue_some(std::integral_constant<int, kLoadsS3 + kLoadsS0>{}, L1{}, stage ^ 1, (kt + 1) * BK);
            mma(fa_c, 1);
            if constexpr (FA > 0) interleave3<0, FA * FN, kReads, kLoadsS1>();
            load_frags(fa_c, stage, 3, 1);
            issue_some(std::integral_constant<int, kLoadsS3 + kLoadsS0 + kLoadsS1>{}, L2{}, stage ^ 1, (kt + 1) * BK);
            mma(fa_c, 0);
            if constexpr (FA > 0) interleave3<0, FA * FN, kReads, kLoadsS2>();
            // every load of step kt+1 has landed and every LDS read of this stage has returned
            // all but the newest load when that is the previous step's prefetch, else all
            if constexpr (kPrefetch) __builtin_amdgcn_s_waitcnt(0x0071);
            else __builtin_amdgcn_s_waitcnt(0x0070);
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            // unconditional (after the last step the fragments are simply not used): straight-line code lets the
            // compiler count outstanding LDS reads exactly, so the MFMAs below do not wait for these reads
            load_frags(fa_c, stage ^ 1, 0, 0);
            // past the end of K the loads are all out of range (zero-fill), which keeps the loop body free of branches
            issue_some(std::integral_constant<int, 0>{}, L3{}, stage, (kt + 2) * BK);
            // the prefetch goes out behind this step's loads (the empty statement orders it: the wait of the next step
            // counts on it being the newest load) and has until the wait of the step after next to complete
            if constexpr (kPrefetch) asm volatile("" : "+v"(pf_voff));
            issue_prefetch(kt + kPfDist);
            mma(fa_c, 1);
            if constexpr (FA > 0) {
                __builtin_amdgcn_sched_group_barrier(0x100, kReads, 0);
                spread_mfma_vmem<0, FA * FN, kLoadsS3>();
                if constexpr (kPrefetch) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
            }
        };
        const uint32_t KT = (Ke + BK - 1) / BK;
        Tile nxt{};
        if (KT == 0) nxt = lookup(++round);
        // rows of the group inside the tile, and inside this wavefront's WM rows of it in blocks of 32
        const uint32_t tile_rows = Me - m0 < (uint32_t)BM ? Me - m0 : (uint32_t)BM;
        const uint32_t wave_rows = tile_rows > wm * WM ? tile_rows - wm * WM : 0u;
        // (a wavefront whose columns all lie past the end of the tile has nothing to compute either)
        const bool has_columns = n0 + wn * (EPI != EPI_PLAIN ? WN / 2 : WN) < n_lim;
        const uint32_t row_blocks = has_columns ? uniform((wave_rows + 31u) / 32u) : 0u;
        // A tile with at most 64 rows leaves three quarters of the A stages unused, and its K steps cost what the latency
        // of their loads costs. It runs a K loop of its own with a third LDS stage in that unused space (A rows 0..63 are
        // 8 KB; the B tile of stage 2 lies in two halves behind the A tiles of stages 0 and 1), so that two steps of
        // loads are in flight instead of one. All of its loads are the assembly-written ones, counted by hand.
        // Only groups that consist of such a tile alone take it (batches of a few rows per group, where the kernel is a
        // stream of the B operand): the short last tile of a larger group gains nothing from running ahead of the full
        // tiles beside it, whose loads of the same B panel it otherwise shares in the L2 (measured: 3 % slower).
        const bool thin = A_KC && Me <= 64u && KT >= 3u;
        if (thin) {
            constexpr uint32_t kThinLoads = 1 + 32 / NW;  // per wavefront and K step: one for A, the usual ones for B
            static_assert(kThinLoads == 5, "the waits below are written for five loads per step");
            const uint8_t* const a_at[3] = {s_a0, s_a1, s_a0 + 8192};
            const uint8_t* const b_lo[3] = {s_b0, s_b1, s_a0 + 16384};
            const uint8_t* const b_hi[3] = {s_b0 + 16384, s_b1 + 16384, s_a1 + 16384};
            auto issue_thin = [&](int st, uint32_t k0) {
                if constexpr (A_KC) lk_a.issue_quiet_first_rows(lds_address(a_at[st]), k0);
                if constexpr (B_KC) lk_b.issue_quiet_halves(lds_address(b_lo[st]), lds_address(b_hi[st]), k0);
                else lt_b.issue_quiet_halves(lds_address(b_lo[st]), lds_address(b_hi[st]), k0);
            };
            // stage 0 in the usual places (an earlier prefetch put it there; the zero rows it wrote behind A's first
            // 8 KB are complete, for every wavefront, once the barrier below is passed), stage 1 likewise
            if (!prefetched) issue_thin(0, 0);
            issue_thin(1, BK);
            nxt = lookup(++round);
            wait_outstanding((prefetched ? tile_stores : 0u) + kThinLoads);
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            issue_thin(2, 2 * BK);
            auto thin_loop = [&](auto fa_c) {
                constexpr int FA = decltype(fa_c)::value;
                auto thin_step = [&](int st, uint32_t kt) {
                    if constexpr (FA > 0) {
#pragma unroll
                        for (int ks = 0; ks < 4; ++ks) {
                            typename EL::frag ta[FA], tb[FN];
#pragma unroll
                            for (int i = 0; i < FA; ++i)
                                ta[i] = __builtin_bit_cast(typename EL::frag, read_kc_frag(a_at[st] + a_off[i] + kc_slice[ks]));
#pragma unroll
                            for (int j = 0; j < FN; ++j) {
                                if constexpr (B_KC) {
                                    // tile rows 0..127 are the first half of the B tile, rows 128..255 the second
                                    const uint8_t* half = b_frag_row(j) < 128u ? b_lo[st] + b_off[j] : b_hi[st] + (b_off[j] - 128u * kRowBytes);
                                    tb[j] = __builtin_bit_cast(typename EL::frag, read_kc_frag(half + kc_slice[ks]));
                                } else {
                                    // k rows 0..31 of the step are the first half, 32..63 the second
                                    const uint8_t* half = ks < 2 ? b_lo[st] + ks * 16 * kTRowBytes : b_hi[st] + (ks - 2) * 16 * kTRowBytes;
                                    tb[j] = __builtin_bit_cast(typename EL::frag, read_tr_frag(half + b_off[j]));
                                }
                            }
#pragma unroll
                            for (int i = 0; i < FA; ++i)
#pragma unroll
                                for (int j = 0; j < FN; ++j) acc[i][j] = EL::mfma(tb[j], ta[i], acc[i][j]);
                        }
                    }
                    // all but the newest five loads: step kt+1 has landed (step kt+2 may still be on its way); past the
                    // barrier every wavefront has finished reading this stage, which then takes the loads of step kt+3
                    // (zero-filling ones past the end of K, so that the count stays the same)
                    __builtin_amdgcn_s_waitcnt(0x0f75);
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
            if (row_blocks == 2) thin_loop(std::integral_constant<int, 2>{});
            else if (row_blocks == 1) thin_loop(std::integral_constant<int, 1>{});
            else thin_loop(std::integral_constant<int, 0>{});
            __builtin_amdgcn_s_waitcnt(0x0f70);
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        } else if (KT > 0) {
            if (!prefetched) issue_quiet(0, 0);
            if (KT > 1) {
                issue_quiet_a(1, BK);
                if (!prefetched_b1) issue_quiet_b(1, BK);
            }
            nxt = lookup(++round);  // in the shadow of the loads
            // the first K step's loads have landed; the second step's, and the previous tile's stores, may still be out
            wait_outstanding((prefetched ? tile_stores : 0u) + (KT > 1 ? kStepLoads : 0u));
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            issue_prefetch(kPfDist - 1);
            auto k_loop = [&](auto fa_c) {
                load_frags(fa_c, 0, 0, 0);
                // two steps per iteration without a branch between them (a branch there makes the compiler wait for
                // the loads in flight before every LDS read at the top of the loop); an odd last step is peeled
                uint32_t kt = 0;
                for (; kt + 1 < KT; kt += 2) {
                    step(fa_c, 0, kt);
                    step(fa_c, 1, kt + 1);
                }
                if (kt < KT) step(fa_c, 0, kt);
            };
            static_assert(FM == 4, "the versions below are for four row blocks per wavefront");
            if (row_blocks > 2) k_loop(std::integral_constant<int, 4>{});
            else if (row_blocks == 2) k_loop(std::integral_constant<int, 2>{});
            else if (row_blocks == 1) k_loop(std::integral_constant<int, 1>{});
            else k_loop(std::integral_constant<int, 0>{});
            // the zero-fill loads issued past the end of K must have landed before the stages are reused below
            __builtin_amdgcn_s_waitcnt(0x0f70);
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        }

        // ---- next tile: its first loads go out now, into stage 0, and fly while this tile's results are stored ----
        prefetched = nxt.valid && nxt.fast && nxt.Ke > 0;
        prefetched_b1 = false;
        if (prefetched) {
            setup_loaders(nxt);
            setup_prefetch(nxt);
            issue_quiet(0, 0);
            const uint32_t next_kt = (nxt.Ke + BK - 1) / BK;
            const bool next_thin = A_KC && nxt.Me <= 64u && next_kt >= 3u;  // (has its own LDS layout and loads)
            if (next_kt > 1 && !next_thin) {
                issue_quiet_b(1, BK);
                prefetched_b1 = true;
            }
        }

        // ---- epilogue ----
        // Past the last barrier of the K loop nobody reads the LDS stages any more. The A half of stage 1 is the staging
        // space: each wavefront takes the four 1 KB pieces of it that it itself loads, for one 32-row block of its
        // sub-tile at a time (stage 0 and the B half of stage 1 already receive the next tile's operands).
        // A lane holds row (lane & 31), columns q*8 + (lane >> 5)*4 + 0..3 of each 32x32 accumulator block.
        static_assert(32 * WN * 2 == (32 / NW) * 1024, "one 32-row block of a wavefront's sub-tile fills its pieces of one operand array");
        // the lane id is made opaque here so that the epilogue's per-lane address arithmetic is redone per tile instead
        // of being hoisted out of the tile loop, where it would occupy registers throughout the K loop
        uint32_t el = lane;
        asm volatile("" : "+v"(el));
        const StagingSlice<NW> img{s_a1 + wave * 1024u, s_a1 + wave * 1024u};
        // alpha is applied up front, and only when it is not 1 (the usual case, and always so for the SwiGLU epilogue)
        if (EPI == EPI_PLAIN && args.alpha != 1.0f) {
            const float alpha = args.alpha;
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j) acc[i][j] *= alpha;
        }
#pragma unroll
        for (int i = 0; i < FM; ++i) {
            const uint32_t row0 = m0 + wm * WM + i * 32;  // first output row of this pass
            const uint32_t rows_valid = row0 < Me ? (Me - row0 < 32u ? Me - row0 : 32u) : 0u;
            if constexpr (EPI == EPI_PLAIN) {
                const uint32_t col0 = n0 + wn * WN;
                const uint32_t cols_valid = col0 < n_lim ? n_lim - col0 : 0u;
#pragma unroll
                for (int j = 0; j < FN; ++j)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const f32x16& c = acc[i][j];
                        uint2 w;
                        w.x = EL::pack2(c[q * 4 + 0], c[q * 4 + 1]);
                        w.y = EL::pack2(c[q * 4 + 2], c[q * 4 + 3]);
                        stage_put<WN * 2>(img, el & 31u, j * 32 + q * 8 + (el >> 5) * 4, w);
                    }
                stage_flush<WN * 2, 32>(img, args.D + off_d + (uint64_t)row0 * Ne + col0, Ne, rows_valid, cols_valid, el);
            } else {
                // first the rounded pre-activation (32 "up" columns | 32 "gate" columns per row), then the activation
                constexpr int HB = WN * 2;  // bytes per staged row of h: 32 "up" columns | 32 "gate" columns
                constexpr int YB = WN;      // bytes per staged row of the activation
                static_assert(FN == 2, "one up block and one gate block per wavefront and row block");
                const uint32_t col0 = n0 + wn * (WN / 2);
                const uint32_t cols_valid = col0 < n_lim ? n_lim - col0 : 0u;
                uint32_t ypack[4][2];  // the packed activation waits here until h has left the staging slice
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    float u[4], g[4], y[4];
#pragma unroll
                    for (int x = 0; x < 4; ++x) {
                        u[x] = EL::round(acc[i][0][q * 4 + x]);
                        g[x] = EL::round(acc[i][1][q * 4 + x]);
                        y[x] = u[x] * g[x] * sigmoid_for<typename EL::act_t>(g[x]);
                    }
                    ypack[q][0] = EL::pack2(y[0], y[1]);
                    ypack[q][1] = EL::pack2(y[2], y[3]);
                    if constexpr (EPI == EPI_SWIGLU) {
                        const uint32_t c = q * 8 + (el >> 5) * 4;
                        uint2 wu, wg;
                        wu.x = EL::pack2(u[0], u[1]);
                        wu.y = EL::pack2(u[2], u[3]);
                        wg.x = EL::pack2(g[0], g[1]);
                        wg.y = EL::pack2(g[2], g[3]);
                        stage_put<HB>(img, el & 31u, c, wu);
                        stage_put<HB>(img, el & 31u, WN / 2 + c, wg);
                    }
                }
                if constexpr (EPI == EPI_SWIGLU)
                    stage_flush_split<HB, 32, WN / 2>(img, args.D + off_d + (uint64_t)row0 * Ne + col0, Ne, rows_valid,
                                                      cols_valid, n_span, el);
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    uint2 wy;
                    wy.x = ypack[q][0];
                    wy.y = ypack[q][1];
                    stage_put<YB>(img, el & 31u, q * 8 + (el >> 5) * 4, wy);
                }
                stage_flush<YB, 32>(img, args.ACT + off_d / 2 + (uint64_t)row0 * n_span + col0, n_span, rows_valid, cols_valid, el);
            }
        }
        cur = nxt;
    }
}

// wavefronts per workgroup: kWavesM x kWavesN = eight 128x64 wave tiles (the hand-counted waits are written for eight)
constexpr int kWavesM = 2;
constexpr int kWavesN = 4;

// every instantiation the entry points launch (explicit, so that host stub and device code are both emitted)
#define FMA_GEMM_INSTANTIATE(EL)                                                                             \
    template __global__ void grouped_gemm_kernel<EL, kWavesM, kWavesN, true, true, EPI_PLAIN>(const GemmArgs);  \
    template __global__ void grouped_gemm_kernel<EL, kWavesM, kWavesN, true, false, EPI_PLAIN>(const GemmArgs); \
    template __global__ void grouped_gemm_kernel<EL, kWavesM, kWavesN, false, true, EPI_PLAIN>(const GemmArgs); \
    template __global__ void grouped_gemm_kernel<EL, kWavesM, kWavesN, false, false, EPI_PLAIN>(const GemmArgs);
FMA_GEMM_INSTANTIATE(ElemBf16)
FMA_GEMM_INSTANTIATE(ElemF16)
#undef FMA_GEMM_INSTANTIATE

template <typename EL, bool A_KC, bool B_KC, int EPI>
int launch(const GemmArgs& args, hipStream_t st) {
    int cus = num_compute_units();
    if (cus <= 0) cus = 256;
    hipLaunchKernelGGL((grouped_gemm_kernel<EL, kWavesM, kWavesN, A_KC, B_KC, EPI>), dim3((uint32_t)cus),
                       dim3(kWavesM * kWavesN * 64), 0, st, args);
    return launch_status("grouped_gemm");
}

template <typename EL>
int launch_plain(const GemmArgs& args, bool a_kc, bool b_kc, hipStream_t st) {
    if (a_kc && b_kc) return launch<EL, true, true, EPI_PLAIN>(args, st);
    if (a_kc && !b_kc) return launch<EL, true, false, EPI_PLAIN>(args, st);
    if (!a_kc && b_kc) return launch<EL, false, true, EPI_PLAIN>(args, st);
    return launch<EL, false, false, EPI_PLAIN>(args, st);
}

}  // namespace gemm
}  // namespace fmahip

namespace fmahip {
namespace gemm {
// grouped_gemm_ragged.hip
int launch_ragged_from_arrays(const void* A, const void* B, void* D, const uint32_t* M_arr, const uint32_t* N_arr,
                              const uint32_t* K_arr, int64_t E, bool a_kc, bool b_kc, float alpha, int dtype, hipStream_t st);
}  // namespace gemm
}  // namespace fmahip

extern "C" {

int fma_grouped_gemm(const void* A, const void* B, void* D, const uint32_t* M_arr, const uint32_t* N_arr,
                     const uint32_t* K_arr, int64_t E, int trans_a, int trans_b, float alpha, int dtype,
                     void* stream) {
    using namespace fmahip;
    using namespace fmahip::gemm;
    FMA_REQUIRE(dtype_bytes(dtype) != 0, FMA_ERR_BAD_DTYPE, "grouped_gemm: unknown dtype code %d", dtype);
    FMA_REQUIRE(E >= 0, FMA_ERR_BAD_SIZE, "grouped_gemm: negative group count %lld", (long long)E);
    FMA_REQUIRE(E <= FMA_MAX_GROUPS, FMA_ERR_TOO_MANY_EXPERTS, "grouped_gemm: E=%lld exceeds the limit %d",
                (long long)E, FMA_MAX_GROUPS);
    if (E == 0) return FMA_OK;
    FMA_REQUIRE(A && B && D && M_arr && N_arr && K_arr, FMA_ERR_NULL_POINTER, "grouped_gemm: NULL pointer");
    FMA_REQUIRE(aligned16(A) && aligned16(B) && aligned16(D), FMA_ERR_MISALIGNED,
                "grouped_gemm: A, B and D must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    const bool a_kc = trans_a == 0;  // A stored [M, K]: reduction dim contiguous
    const bool b_kc = trans_b != 0;  // B stored [N, K]: reduction dim contiguous
    if (dtype == FMA_F32) return gemm_f32::launch(A, B, D, M_arr, N_arr, K_arr, E, a_kc, b_kc, alpha, st);
    // Three launches, of which one does the work: the group sizes live in device memory, so each kernel decides for itself
    // (reading the arrays costs a kernel that then ends about 2 us). Launches whose groups differ in one dimension only
    // (every grouped GEMM of an MoE layer, the reference's own test shapes) go to the streaming kernels of
    // grouped_gemm_ragged.hip, anything else to the kernel of this file.
    const int rc = launch_ragged_from_arrays(A, B, D, M_arr, N_arr, K_arr, E, a_kc, b_kc, alpha, dtype, st);
    if (rc != FMA_OK) return rc;
    GemmArgs args{};
    args.A = (const uint16_t*)A;
    args.B = (const uint16_t*)B;
    args.D = (uint16_t*)D;
    args.ACT = nullptr;
    args.M_arr = M_arr;
    args.N_arr = N_arr;
    args.K_arr = K_arr;
    args.E = (uint32_t)E;
    args.alpha = alpha;
    args.only_if_irregular = 1u;
    return dtype == FMA_BF16 ? launch_plain<ElemBf16>(args, a_kc, b_kc, st) : launch_plain<ElemF16>(args, a_kc, b_kc, st);
}

}  // extern "C"
