// Grouped GEMM over ragged expert groups for gfx950: bf16 operands, fp32 accumulation on the matrix cores
// (v_mfma_f32_32x32x16_bf16), optional SwiGLU epilogue.
//
// Shape of the kernel
//  * Persistent: the grid is one workgroup per compute unit. Each workgroup builds the group table (tile
//    prefix and packed element offsets of every group) in LDS from the device-side M/N/K arrays, then walks
//    256x256 output tiles. Tile ids are handed out so that the 32 workgroups of one XCD (workgroup id mod 8)
//    always hold a compact 8x4 block of tiles of the same group: they share A and B panels in that XCD's L2.
//  * K is consumed in steps of 64 through two LDS stages of 2 x 32 KB. Both operand tiles live in LDS as
//    [row][64 k] (k contiguous, 128-byte rows) whatever their layout in memory:
//      - an operand whose reduction dimension is contiguous in memory goes global -> LDS directly
//        (global_load_lds_dwordx4, 1 KB per wavefront instruction, no staging registers);
//      - an operand stored with the reduction dimension as the row index is loaded as 8x8 blocks (eight
//        16-byte loads per lane), transposed in registers with byte permutes and written as 16-byte rows.
//    Row r / 16-byte chunk c of a tile sits at  phys_row(r)*128 + ((c ^ (r & 7)) << 4)  where phys_row rotates
//    the low four row bits left by one. With it the MFMA operand reads (32 consecutive rows, one chunk), the
//    direct loads (whole 128-byte rows) and the transposed stores (rows 8 apart, 8 chunks) each touch every
//    LDS bank group once.
//  * The MFMA is issued with B as the first operand, so a lane ends up holding four consecutive output
//    columns of one output row and stores them as one 8-byte word.
#include "common.h"

namespace fmahip {
namespace gemm {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((address_space(3))) void lds_void;

constexpr int BM = 256;
constexpr int BN = 256;
constexpr int BK = 64;
constexpr int kRowBytes = BK * 2;           // 128
constexpr int kTileBytes = BM * kRowBytes;  // 32 KB per operand per stage
constexpr int kGroupM = 8;                  // m-tiles that share one column sweep of the tile order
constexpr int kXcds = 8;

constexpr int EPI_PLAIN = 0;
constexpr int EPI_SWIGLU = 1;

struct GemmArgs {
    const uint16_t* A;
    const uint16_t* B;
    uint16_t* D;    // plain: output; swiglu: pre-activation h (may be NULL)
    uint16_t* ACT;  // swiglu only: activation output
    const uint32_t* M_arr;
    const uint32_t* N_arr;  // NULL: every group uses const_n
    const uint32_t* K_arr;  // NULL: every group uses const_k
    uint32_t E;
    uint32_t const_n;
    uint32_t const_k;
    uint32_t inter;  // swiglu only: I (N = 2*I)
    float alpha;
};

__device__ __forceinline__ uint32_t phys_row(uint32_t r) { return (r & ~15u) | ((r & 7u) << 1) | ((r >> 3) & 1u); }
__device__ __forceinline__ uint32_t logical_row(uint32_t pr) {
    return (pr & ~15u) | ((pr & 15u) >> 1) | ((pr & 1u) << 3);
}
__device__ __forceinline__ uint32_t lds_off(uint32_t r, uint32_t chunk) {
    return phys_row(r) * kRowBytes + ((chunk ^ (r & 7u)) << 4);
}

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    f32x2 f = {lo, hi};
    bf16x2 b = __builtin_convertvector(f, bf16x2);
    return __builtin_bit_cast(uint32_t, b);
}

__device__ __forceinline__ float round_bf16(float x) {
    const __bf16 b = (__bf16)x;
    return (float)b;
}

// ---- loader for an operand whose reduction dimension is contiguous in memory ---------------------
// The tile has 256 rows; a wavefront instruction moves 8 physical rows (1 KB). NI instructions per wavefront.
template <int NW>
struct DirectLoader {
    static constexpr int NI = 32 / NW;
    const uint16_t* gp[NI];  // this lane's source of each instruction at k0 = 0
    uint32_t chunk;          // this lane's logical 16-byte chunk (same for every instruction)
    uint32_t kdim;
    uint32_t wave;

    // row_of(r): global row index of tile row r (already clamped into the valid range)
    template <typename RowFn>
    __device__ __forceinline__ void setup(const uint16_t* base, uint64_t ld, uint32_t kdim_, uint32_t wave_,
                                          uint32_t lane, RowFn row_of) {
        kdim = kdim_;
        wave = wave_;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const uint32_t pr = (uint32_t)(i * NW + wave_) * 8u + (lane >> 3);
            const uint32_t r = logical_row(pr);
            chunk = (lane & 7u) ^ (r & 7u);
            gp[i] = base + (uint64_t)row_of(r) * ld + chunk * 8u;
        }
    }

    __device__ __forceinline__ void issue(uint8_t* tile, uint32_t k0, uint32_t lane) const {
        if (k0 + BK <= kdim) {
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                __builtin_amdgcn_global_load_lds(gp[i] + k0, (lds_void*)(tile + (i * NW + wave) * 1024), 16, 0, 0);
            }
        } else {
            // last, partial K step: chunks past the end of K are zero-filled instead of loaded
            const bool valid = k0 + chunk * 8u < kdim;
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                uint8_t* dst = tile + (i * NW + wave) * 1024;
                if (valid) {
                    __builtin_amdgcn_global_load_lds(gp[i] + k0, (lds_void*)dst, 16, 0, 0);
                } else {
                    *reinterpret_cast<uint4*>(dst + lane * 16u) = make_uint4(0, 0, 0, 0);
                }
            }
        }
    }
};

// ---- loader for an operand stored [reduction][out] (out contiguous): 8x8 blocks, register transpose ----
struct TransposeLoader {
    const uint16_t* gp;  // base + (kb*8)*ld + out chunk of this lane
    uint64_t ld;
    uint32_t kb, ob;  // 8-row block of the reduction dim (0..7), 8-column block of the out dim (0..31)
    uint32_t kdim;
    uint4 st[8];

    __device__ __forceinline__ void setup(const uint16_t* base, uint64_t ld_, uint32_t kdim_, uint32_t out0,
                                          uint32_t out_total, uint32_t tl) {
        const uint32_t lane = tl & 63u;
        kb = lane & 7u;
        ob = (tl >> 6) * 8u + (lane >> 3);
        ld = ld_;
        kdim = kdim_;
        uint32_t oc = out0 + ob * 8u;
        if (oc + 8u > out_total) oc = out_total - 8u;  // columns past the edge: results are never stored
        gp = base + (uint64_t)(kb * 8u) * ld_ + oc;
    }

    __device__ __forceinline__ void load(uint32_t k0) {
        const uint16_t* p = gp + (uint64_t)k0 * ld;
        if (k0 + BK <= kdim) {
#pragma unroll
            for (int j = 0; j < 8; ++j) st[j] = *reinterpret_cast<const uint4*>(p + (uint64_t)j * ld);
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                if (k0 + kb * 8u + j < kdim)
                    st[j] = *reinterpret_cast<const uint4*>(p + (uint64_t)j * ld);
                else
                    st[j] = make_uint4(0, 0, 0, 0);
            }
        }
    }

    __device__ __forceinline__ void store(uint8_t* tile) const {
        // st[j] holds out columns 0..7 of reduction row j; column c must become 8 reduction values
        const uint32_t* w = reinterpret_cast<const uint32_t*>(st);  // w[j*4 + d]: columns 2d, 2d+1 of row j
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            uint32_t lo[4], hi[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t even = w[(2 * q) * 4 + d];
                const uint32_t odd = w[(2 * q + 1) * 4 + d];
                lo[q] = __builtin_amdgcn_perm(odd, even, 0x05040100u);  // column 2d  : rows 2q, 2q+1
                hi[q] = __builtin_amdgcn_perm(odd, even, 0x07060302u);  // column 2d+1: rows 2q, 2q+1
            }
            *reinterpret_cast<uint4*>(tile + lds_off(ob * 8u + 2 * d, kb)) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
            *reinterpret_cast<uint4*>(tile + lds_off(ob * 8u + 2 * d + 1, kb)) = make_uint4(hi[0], hi[1], hi[2], hi[3]);
        }
    }
};

// Slow, layout-agnostic path for a group whose contiguous dimensions are not multiples of 8 elements.
template <bool A_KC, bool B_KC>
__device__ void scalar_tile(const uint16_t* Ae, const uint16_t* Be, uint16_t* De, uint32_t Me, uint32_t Ne,
                            uint32_t Ke, uint32_t m0, uint32_t n0, float alpha, uint32_t nthreads) {
    for (uint32_t idx = threadIdx.x; idx < (uint32_t)(BM * BN); idx += nthreads) {
        const uint32_t m = m0 + idx / BN;
        const uint32_t n = n0 + idx % BN;
        if (m >= Me || n >= Ne) continue;
        float acc = 0.0f;
        for (uint32_t k = 0; k < Ke; ++k) {
            const uint16_t a = A_KC ? Ae[(uint64_t)m * Ke + k] : Ae[(uint64_t)k * Me + m];
            const uint16_t b = B_KC ? Be[(uint64_t)n * Ke + k] : Be[(uint64_t)k * Ne + n];
            acc = fmaf(bf16_bits_to_float(a), bf16_bits_to_float(b), acc);
        }
        De[(uint64_t)m * Ne + n] = (uint16_t)(pack_bf16x2(alpha * acc, 0.0f) & 0xffffu);
    }
}

template <int NWM, int NWN, bool A_KC, bool B_KC, int EPI>
__global__ __launch_bounds__(NWM* NWN * 64) void grouped_gemm_kernel(const GemmArgs args) {
    constexpr int NW = NWM * NWN;
    constexpr int NT = NW * 64;
    constexpr int WM = BM / NWM;
    constexpr int WN = BN / NWN;
    constexpr int FM = WM / 32;
    constexpr int FN = WN / 32;
    static_assert(EPI == EPI_PLAIN || (A_KC && B_KC), "the SwiGLU epilogue exists for the NT layout only");
    static_assert(NT == 256 || NT == 512, "the transpose loader is written for 256-thread groups");

    // one array per stage and operand: distinct LDS objects let the compiler see that a direct-to-LDS load
    // into one stage cannot alias the fragment reads of the other, so it does not wait for the load first
    __shared__ __attribute__((aligned(1024))) uint8_t s_a0[kTileBytes];
    __shared__ __attribute__((aligned(1024))) uint8_t s_b0[kTileBytes];
    __shared__ __attribute__((aligned(1024))) uint8_t s_a1[kTileBytes];
    __shared__ __attribute__((aligned(1024))) uint8_t s_b1[kTileBytes];
    __shared__ uint32_t s_tile_start[FMA_MAX_GROUPS + 1];
    __shared__ uint64_t s_off_a[FMA_MAX_GROUPS + 1];
    __shared__ uint64_t s_off_b[FMA_MAX_GROUPS + 1];
    __shared__ uint64_t s_off_d[FMA_MAX_GROUPS + 1];

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t wm = wave / NWN;
    const uint32_t wn = wave % NWN;
    const uint32_t E = args.E;

    auto group_m = [&](uint32_t e) { return args.M_arr[e]; };
    auto group_n = [&](uint32_t e) { return args.N_arr ? args.N_arr[e] : args.const_n; };
    auto group_k = [&](uint32_t e) { return args.K_arr ? args.K_arr[e] : args.const_k; };
    // n-extent covered by the tile grid: for the SwiGLU epilogue a tile spans 128 up + 128 gate columns
    auto tiles_of = [&](uint32_t m, uint32_t n) -> uint32_t {
        if (m == 0 || n == 0) return 0;
        const uint32_t tn = EPI == EPI_SWIGLU ? (n / 2 + BN / 2 - 1) / (BN / 2) : (n + BN - 1) / BN;
        return ((m + BM - 1) / BM) * tn;
    };

    // ---- group table: exclusive prefixes of tiles and of packed element counts, built by wavefront 0 ----
    if (wave == 0) {
        uint32_t carry_t = 0;
        uint64_t carry_a = 0, carry_b = 0, carry_d = 0;
        for (uint32_t base = 0; base < E; base += 64) {
            const uint32_t e = base + lane;
            uint32_t m = 0, n = 0, k = 0;
            if (e < E) {
                m = group_m(e);
                n = group_n(e);
                k = group_k(e);
            }
            const uint32_t t = tiles_of(m, n);
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

    // per-lane LDS read offsets of an MFMA operand fragment whose first row is a multiple of 32
    uint32_t frag_off[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) frag_off[ks] = lds_off(lane & 31u, (uint32_t)ks * 2u + (lane >> 5));
    const uint32_t a_wave_off = wm * WM * kRowBytes;
    // first LDS row of B fragment j of this wavefront
    auto b_frag_row = [&](int j) -> uint32_t {
        if constexpr (EPI == EPI_SWIGLU) {
            return j < FN / 2 ? wn * (WN / 2) + j * 32 : BN / 2 + wn * (WN / 2) + (j - FN / 2) * 32;
        } else {
            return wn * WN + j * 32;
        }
    };

    // workgroup id -> position in the round of gridDim.x tiles: workgroups of one XCD take 32 neighbours
    const uint32_t grid = gridDim.x;
    const uint32_t per_xcd = grid / kXcds;
    const uint32_t slot = (grid % kXcds == 0) ? (blockIdx.x % kXcds) * per_xcd + blockIdx.x / kXcds : blockIdx.x;

    for (uint32_t v = slot; v < total_tiles; v += grid) {
        // ---- which group, which tile ----
        uint32_t lo = 0, hi = E;
        while (lo < hi) {
            const uint32_t mid = (lo + hi) >> 1;
            if (s_tile_start[mid + 1] <= v) lo = mid + 1;
            else hi = mid;
        }
        const uint32_t e = lo;
        const uint32_t Me = group_m(e), Ne = group_n(e), Ke = group_k(e);
        const uint32_t n_span = EPI == EPI_SWIGLU ? Ne / 2 : Ne;  // columns the tile grid runs over
        constexpr uint32_t TN = EPI == EPI_SWIGLU ? BN / 2 : BN;  // of which one tile covers this many
        const uint32_t tiles_m = (Me + BM - 1) / BM;
        const uint32_t tiles_n = (n_span + TN - 1) / TN;
        const uint32_t local = v - s_tile_start[e];
        const uint32_t band = kGroupM * tiles_n;
        const uint32_t first_m = (local / band) * kGroupM;
        const uint32_t band_m = tiles_m - first_m < (uint32_t)kGroupM ? tiles_m - first_m : (uint32_t)kGroupM;
        const uint32_t mt = first_m + (local % band) % band_m;
        const uint32_t nt = (local % band) / band_m;
        const uint32_t m0 = mt * BM;
        const uint32_t n0 = nt * TN;

        const uint16_t* Ae = args.A + s_off_a[e];
        const uint16_t* Be = args.B + s_off_b[e];
        const uint64_t off_d = s_off_d[e];

        bool fast = (Ke % 8u == 0) && (Ne % 8u == 0) && (s_off_a[e] % 8u == 0) && (s_off_b[e] % 8u == 0) &&
                    (off_d % 8u == 0);
        if (!A_KC) fast = fast && (Me % 8u == 0);
        if (EPI == EPI_SWIGLU) fast = fast && (n_span % 8u == 0);

        __syncthreads();  // every wavefront is done with the previous tile's LDS stages

        if (!fast) {
            if constexpr (EPI == EPI_PLAIN) {
                scalar_tile<A_KC, B_KC>(Ae, Be, args.D + off_d, Me, Ne, Ke, m0, n0, args.alpha, NT);
            }
            continue;
        }

        // ---- loaders ----
        DirectLoader<NW> dl_a, dl_b;
        TransposeLoader tl_a, tl_b;
        const bool mc_a_on = !A_KC && (NT == 256 || wave < 4);
        const bool mc_b_on = !B_KC && (NT == 256 || (A_KC ? wave < 4 : wave >= 4));
        if constexpr (A_KC) {
            dl_a.setup(Ae, Ke, Ke, wave, lane, [&](uint32_t r) {
                const uint32_t m = m0 + r;
                return m < Me ? m : Me - 1;
            });
        } else {
            if (mc_a_on) tl_a.setup(Ae, Me, Ke, m0, Me, tid & 255u);
        }
        if constexpr (B_KC) {
            dl_b.setup(Be, Ke, Ke, wave, lane, [&](uint32_t r) {
                uint32_t n;
                if constexpr (EPI == EPI_SWIGLU) {
                    // rows 0..127: "up" rows n0 + r; rows 128..255: "gate" rows I + n0 + (r - 128)
                    const uint32_t c = n0 + (r & (BN / 2 - 1));
                    n = (c < n_span ? c : n_span - 1) + (r >= BN / 2 ? n_span : 0u);
                } else {
                    n = n0 + r;
                    n = n < Ne ? n : Ne - 1;
                }
                return n;
            });
        } else {
            if (mc_b_on) tl_b.setup(Be, Ne, Ke, n0, Ne, tid & 255u);
        }

        auto issue = [&](int stage, uint32_t k0) {
            if constexpr (A_KC) dl_a.issue(stage ? s_a1 : s_a0, k0, lane);
            else if (mc_a_on) tl_a.load(k0);
            if constexpr (B_KC) dl_b.issue(stage ? s_b1 : s_b0, k0, lane);
            else if (mc_b_on) tl_b.load(k0);
        };
        auto finish = [&](int stage) {
            if constexpr (!A_KC) {
                if (mc_a_on) tl_a.store(stage ? s_a1 : s_a0);
            }
            if constexpr (!B_KC) {
                if (mc_b_on) tl_b.store(stage ? s_b1 : s_b0);
            }
        };

        f32x16 acc[FM][FN];
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int x = 0; x < 16; ++x) acc[i][j][x] = 0.0f;

        auto compute = [&](int stage) {
            const uint8_t* ta = (stage ? s_a1 : s_a0) + a_wave_off;
            const uint8_t* tb = stage ? s_b1 : s_b0;
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                bf16x8 a[FM], b[FN];
#pragma unroll
                for (int i = 0; i < FM; ++i)
                    a[i] = *reinterpret_cast<const bf16x8*>(ta + i * 32 * kRowBytes + frag_off[ks]);
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    b[j] = *reinterpret_cast<const bf16x8*>(tb + b_frag_row(j) * kRowBytes + frag_off[ks]);
#pragma unroll
                for (int i = 0; i < FM; ++i)
#pragma unroll
                    for (int j = 0; j < FN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b[j], a[i], acc[i][j], 0, 0, 0);
            }
        };

        // ---- main loop over K: stage s is computed while stage s^1 is being filled ----
        const uint32_t KT = (Ke + BK - 1) / BK;
        if (KT > 0) {
            issue(0, 0);
            finish(0);
        }
        for (uint32_t kt = 0; kt < KT; kt += 2) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if (kt + 1 < KT) issue(1, (kt + 1) * BK);
            compute(0);
            if (kt + 1 < KT) {
                finish(1);
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __syncthreads();
                if (kt + 2 < KT) issue(0, (kt + 2) * BK);
                compute(1);
                if (kt + 2 < KT) finish(0);
            }
        }

        // ---- epilogue: lane holds row m = (lane & 31), columns q*8 + (lane >> 5)*4 + 0..3 of each 32x32 block ----
        const float alpha = args.alpha;
        if constexpr (EPI == EPI_PLAIN) {
            uint16_t* De = args.D + off_d;
#pragma unroll
            for (int i = 0; i < FM; ++i) {
                const uint32_t m = m0 + wm * WM + i * 32 + (lane & 31u);
                if (m >= Me) continue;
                uint16_t* drow = De + (uint64_t)m * Ne;
#pragma unroll
                for (int j = 0; j < FN; ++j) {
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const uint32_t n = n0 + wn * WN + j * 32 + q * 8 + (lane >> 5) * 4;
                        if (n < Ne) {
                            uint2 w;
                            w.x = pack_bf16x2(alpha * acc[i][j][q * 4 + 0], alpha * acc[i][j][q * 4 + 1]);
                            w.y = pack_bf16x2(alpha * acc[i][j][q * 4 + 2], alpha * acc[i][j][q * 4 + 3]);
                            *reinterpret_cast<uint2*>(drow + n) = w;
                        }
                    }
                }
            }
        } else {
            uint16_t* He = args.D ? args.D + off_d : nullptr;
            uint16_t* Ce = args.ACT + off_d / 2;
#pragma unroll
            for (int i = 0; i < FM; ++i) {
                const uint32_t m = m0 + wm * WM + i * 32 + (lane & 31u);
                if (m >= Me) continue;
#pragma unroll
                for (int j = 0; j < FN / 2; ++j) {
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const uint32_t n = n0 + wn * (WN / 2) + j * 32 + q * 8 + (lane >> 5) * 4;
                        if (n < n_span) {
                            float u[4], g[4], y[4];
#pragma unroll
                            for (int x = 0; x < 4; ++x) {
                                u[x] = round_bf16(alpha * acc[i][j][q * 4 + x]);
                                g[x] = round_bf16(alpha * acc[i][j + FN / 2][q * 4 + x]);
                                y[x] = u[x] * g[x] * sigmoid_clamped(g[x]);
                            }
                            if (He) {
                                uint2 wu, wg;
                                wu.x = pack_bf16x2(u[0], u[1]);
                                wu.y = pack_bf16x2(u[2], u[3]);
                                wg.x = pack_bf16x2(g[0], g[1]);
                                wg.y = pack_bf16x2(g[2], g[3]);
                                *reinterpret_cast<uint2*>(He + (uint64_t)m * Ne + n) = wu;
                                *reinterpret_cast<uint2*>(He + (uint64_t)m * Ne + n_span + n) = wg;
                            }
                            uint2 wy;
                            wy.x = pack_bf16x2(y[0], y[1]);
                            wy.y = pack_bf16x2(y[2], y[3]);
                            *reinterpret_cast<uint2*>(Ce + (uint64_t)m * n_span + n) = wy;
                        }
                    }
                }
            }
        }
    }
}

// every instantiation the entry points launch (explicit, so that host stub and device code are both emitted)
template __global__ void grouped_gemm_kernel<2, 4, true, true, EPI_PLAIN>(const GemmArgs);
template __global__ void grouped_gemm_kernel<2, 4, true, false, EPI_PLAIN>(const GemmArgs);
template __global__ void grouped_gemm_kernel<2, 4, false, true, EPI_PLAIN>(const GemmArgs);
template __global__ void grouped_gemm_kernel<2, 4, false, false, EPI_PLAIN>(const GemmArgs);
template __global__ void grouped_gemm_kernel<2, 4, true, true, EPI_SWIGLU>(const GemmArgs);

template <int NWM, int NWN, bool A_KC, bool B_KC, int EPI>
int launch(const GemmArgs& args, hipStream_t st) {
    int cus = num_compute_units();
    if (cus <= 0) cus = 256;
    hipLaunchKernelGGL((grouped_gemm_kernel<NWM, NWN, A_KC, B_KC, EPI>), dim3((uint32_t)cus), dim3(NWM * NWN * 64), 0,
                       st, args);
    return launch_status("grouped_gemm");
}

}  // namespace gemm
}  // namespace fmahip

extern "C" {

int fma_grouped_gemm(const void* A, const void* B, void* D, const uint32_t* M_arr, const uint32_t* N_arr,
                     const uint32_t* K_arr, int64_t E, int trans_a, int trans_b, float alpha, int dtype,
                     void* stream) {
    using namespace fmahip;
    using namespace fmahip::gemm;
    FMA_REQUIRE(dtype == FMA_BF16, dtype_bytes(dtype) ? FMA_ERR_UNSUPPORTED : FMA_ERR_BAD_DTYPE,
                "grouped_gemm: only bf16 operands are implemented (dtype code %d)", dtype);
    FMA_REQUIRE(E >= 0, FMA_ERR_BAD_SIZE, "grouped_gemm: negative group count %lld", (long long)E);
    FMA_REQUIRE(E <= FMA_MAX_GROUPS, FMA_ERR_TOO_MANY_EXPERTS, "grouped_gemm: E=%lld exceeds the limit %d",
                (long long)E, FMA_MAX_GROUPS);
    if (E == 0) return FMA_OK;
    FMA_REQUIRE(A && B && D && M_arr && N_arr && K_arr, FMA_ERR_NULL_POINTER, "grouped_gemm: NULL pointer");
    FMA_REQUIRE(aligned16(A) && aligned16(B) && aligned16(D), FMA_ERR_MISALIGNED,
                "grouped_gemm: A, B and D must be 16-byte aligned");
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
    hipStream_t st = (hipStream_t)stream;
    const bool a_kc = trans_a == 0;  // A stored [M, K]: reduction dim contiguous
    const bool b_kc = trans_b != 0;  // B stored [N, K]: reduction dim contiguous
    if (a_kc && b_kc) return launch<2, 4, true, true, EPI_PLAIN>(args, st);
    if (a_kc && !b_kc) return launch<2, 4, true, false, EPI_PLAIN>(args, st);
    if (!a_kc && b_kc) return launch<2, 4, false, true, EPI_PLAIN>(args, st);
    return launch<2, 4, false, false, EPI_PLAIN>(args, st);
}

int fma_grouped_gemm_swiglu(const void* x, const void* W, void* h, void* act, const uint32_t* M_arr, int64_t E,
                            int64_t I, int64_t K, int dtype, void* stream) {
    using namespace fmahip;
    using namespace fmahip::gemm;
    FMA_REQUIRE(dtype == FMA_BF16, dtype_bytes(dtype) ? FMA_ERR_UNSUPPORTED : FMA_ERR_BAD_DTYPE,
                "grouped_gemm_swiglu: only bf16 operands are implemented (dtype code %d)", dtype);
    FMA_REQUIRE(E >= 0, FMA_ERR_BAD_SIZE, "grouped_gemm_swiglu: negative group count %lld", (long long)E);
    FMA_REQUIRE(E <= FMA_MAX_GROUPS, FMA_ERR_TOO_MANY_EXPERTS, "grouped_gemm_swiglu: E=%lld exceeds the limit %d",
                (long long)E, FMA_MAX_GROUPS);
    FMA_REQUIRE(I >= 8 && I % 8 == 0 && I <= 0x3fffffffll, FMA_ERR_BAD_SIZE,
                "grouped_gemm_swiglu: intermediate size %lld must be a positive multiple of 8", (long long)I);
    FMA_REQUIRE(K >= 8 && K % 8 == 0 && K <= 0x7fffffffll, FMA_ERR_BAD_SIZE,
                "grouped_gemm_swiglu: K=%lld must be a positive multiple of 8", (long long)K);
    if (E == 0) return FMA_OK;
    FMA_REQUIRE(x && W && act && M_arr, FMA_ERR_NULL_POINTER, "grouped_gemm_swiglu: NULL pointer");
    FMA_REQUIRE(aligned16(x) && aligned16(W) && aligned16(act) && aligned16(h), FMA_ERR_MISALIGNED,
                "grouped_gemm_swiglu: x, W, h and act must be 16-byte aligned");
    GemmArgs args{};
    args.A = (const uint16_t*)x;
    args.B = (const uint16_t*)W;
    args.D = (uint16_t*)h;
    args.ACT = (uint16_t*)act;
    args.M_arr = M_arr;
    args.N_arr = nullptr;
    args.K_arr = nullptr;
    args.E = (uint32_t)E;
    args.const_n = (uint32_t)(2 * I);
    args.const_k = (uint32_t)K;
    args.inter = (uint32_t)I;
    args.alpha = 1.0f;
    return launch<2, 4, true, true, EPI_SWIGLU>(args, (hipStream_t)stream);
}

}  // extern "C"
