// The MoE router in one pass over the activations: logits = x @ Wg^T, top-k, softmax over the k kept logits and
// the histogram of the chosen experts; and the backward of the top-k + softmax part.
//
// The forward is bound by reading x once from HBM (T*H elements against T*E outputs, E << H). A workgroup owns 16, 32
// or 64 tokens; its four wavefronts split the reduction dimension, each accumulating partial logits for all of the
// workgroup's tokens on the matrix cores, and the partials are summed through LDS in a fixed order. Operand fragments come straight from global
// memory: the 16x16x32 MFMA wants, per lane, 8 consecutive K elements of one row, and since a dot product does not care
// about the order of its terms as long as both operands use the same one, each lane takes 32 consecutive elements
// (four 16-byte loads) per step and feeds the four MFMAs of the step from them. A row is then read in 256-byte pieces
// per wavefront, 1 KB per workgroup. The router weight matrix (E*H elements, at most a few MB) is re-read by every
// workgroup from the L2.
#include "common.h"


namespace fmahip {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

constexpr int kRouterThreads = 256;
constexpr int kRouterWaves = kRouterThreads / kWave;
constexpr int kTok = 16;         // tokens per workgroup = rows of one MFMA tile
constexpr int kStepK = 128;      // reduction elements per step of one wavefront: 4 lane groups x 32 elements
constexpr int kMaxTopK = 64;     // top_k limit (FMA_MAX_ROUTER_TOP_K)
constexpr int kRowPad = 16;      // keeps the four token rows one wavefront scans in different LDS banks

struct RouterBf16 {
    using frag = bf16x8;
    static constexpr uint32_t kInfBits = 0x7f80u, kNanBits = 0x7fc0u;
    static __device__ __forceinline__ float round(float x) { return (float)(__bf16)x; }
    static __device__ __forceinline__ uint16_t bits(float x) { return __builtin_bit_cast(uint16_t, (__bf16)x); }
    static __device__ __forceinline__ float from_bits(uint16_t b) { return bf16_bits_to_float(b); }
    static __device__ __forceinline__ f32x4 mfma(frag a, frag b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
};
struct RouterF16 {
    using frag = f16x8;
    static constexpr uint32_t kInfBits = 0x7c00u, kNanBits = 0x7e00u;
    static __device__ __forceinline__ float round(float x) { return (float)(_Float16)x; }
    static __device__ __forceinline__ uint16_t bits(float x) { return __builtin_bit_cast(uint16_t, (_Float16)x); }
    static __device__ __forceinline__ float from_bits(uint16_t b) { return (float)__builtin_bit_cast(_Float16, b); }
    static __device__ __forceinline__ f32x4 mfma(frag a, frag b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
};

struct RouterArgs {
    const uint16_t* x;       // [T, H]
    const uint16_t* w;       // [E, H]
    uint16_t* logits;        // [T, E]
    uint16_t* weights;       // [T, k]
    int32_t* selected;       // [T, k]
    uint32_t* counts;        // [E] or null
    uint32_t* hist;          // [ceil(T / 16), E] or null: choices per expert among each 16 consecutive tokens
    int64_t T;
    int32_t H, E, k;
};

template <typename F>
__device__ __forceinline__ F load_frag(const uint16_t* p) {
    return __builtin_bit_cast(F, *reinterpret_cast<const u32x4*>(p));
}

// ---- sort keys ------------------------------------------------------------------------------------------------------
// The top-k works on one 32-bit key per logit: the 16 bits of the (already rounded) logit mapped so that unsigned order
// equals numeric order, with NaN above everything (where torch.topk puts it) and -0 equal to +0, then 0xffff - column
// in the low half. The unsigned maximum of such keys is the largest logit and, among equal logits, the lowest column.
// Key 0 marks a column that is already taken (no real key is 0: the low half of a real key is at least 0xffff - 1023).
template <typename EL>
__device__ __forceinline__ uint32_t make_key(uint32_t bits, int column) {
    uint32_t ord;
    if ((bits & 0x7fffu) > EL::kInfBits) ord = 0xffffu;
    else {
        if (bits == 0x8000u) bits = 0;
        ord = (bits & 0x8000u) ? (~bits & 0xffffu) : (bits | 0x8000u);
    }
    return (ord << 16) | (0xffffu - (uint32_t)column);
}
template <typename EL>
__device__ __forceinline__ float key_value(uint32_t key) {
    const uint32_t ord = key >> 16;
    const uint32_t bits = ord == 0xffffu ? EL::kNanBits : ((ord & 0x8000u) ? (ord & 0x7fffu) : (~ord & 0xffffu));
    return EL::from_bits((uint16_t)bits);
}
__device__ __forceinline__ int key_column(uint32_t key) { return (int)(0xffffu - (key & 0xffffu)); }

// All-reduce over the 16 lanes of a DPP row (lanes 16g .. 16g+15 of the wavefront) with data-parallel-primitive
// moves: neighbours inside a quad, the other pair of the quad, the mirrored quad of the half row, the mirrored half.
// Every lane ends up with the same value; for the float sum the order of additions is the same fixed tree in all lanes.
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, false);
}
constexpr int kDppXor1 = 0xb1, kDppXor2 = 0x4e, kDppHalfMirror = 0x141, kDppMirror = 0x140;
__device__ __forceinline__ uint32_t row16_max(uint32_t v) {
    v = max(v, dpp_u32<kDppXor1>(v));
    v = max(v, dpp_u32<kDppXor2>(v));
    v = max(v, dpp_u32<kDppHalfMirror>(v));
    v = max(v, dpp_u32<kDppMirror>(v));
    return v;
}
__device__ __forceinline__ float row16_sum(float v) {
    v += __uint_as_float(dpp_u32<kDppXor1>(__float_as_uint(v)));
    v += __uint_as_float(dpp_u32<kDppXor2>(__float_as_uint(v)));
    v += __uint_as_float(dpp_u32<kDppHalfMirror>(__float_as_uint(v)));
    v += __uint_as_float(dpp_u32<kDppMirror>(__float_as_uint(v)));
    return v;
}

__global__ __launch_bounds__(kRouterThreads) void fill_u32_kernel(uint32_t* p, int64_t n, uint32_t v) {
    const int64_t i = (int64_t)blockIdx.x * kRouterThreads + threadIdx.x;
    if (i < n) p[i] = v;
}

// Top-k and softmax of NR tokens at once by the 16 lanes of a DPP row (the NR chains of dependent reductions are
// independent of each other, which is what hides their latency); keys[t] is token t's row of sort keys in LDS, of which
// lane c owns (reads, and clears when chosen) the columns congruent to c mod 16. Choice j is remembered by lane
// j % 16, so that after the k rounds every lane turns its own choices into weights and writes them.
template <typename EL, int NR>
__device__ __forceinline__ void topk_softmax_tokens(uint32_t* const (&keys)[NR], int c, const int64_t (&token)[NR],
                                                    const int64_t tok0, const RouterArgs& a, uint32_t* s_hist) {
    const int E = a.E, k = a.k;
    uint32_t mine[NR][kMaxTopK / 16];
    uint32_t first[NR];
#pragma unroll
    for (int t = 0; t < NR; ++t) {
        first[t] = 0;
#pragma unroll
        for (int i = 0; i < kMaxTopK / 16; ++i) mine[t][i] = 0;
    }
    for (int j = 0; j < k; ++j) {
        uint32_t best[NR];
#pragma unroll
        for (int t = 0; t < NR; ++t) best[t] = 0;
        for (int n = c; n < E; n += 16)
#pragma unroll
            for (int t = 0; t < NR; ++t) best[t] = max(best[t], keys[t][n]);
#pragma unroll
        for (int t = 0; t < NR; ++t) best[t] = row16_max(best[t]);  // top_k <= E: a real key
#pragma unroll
        for (int t = 0; t < NR; ++t) {
            const int col = key_column(best[t]);
            if ((col & 15) == c) keys[t][col] = 0;
            if (j == 0) first[t] = best[t];
#pragma unroll
            for (int i = 0; i < kMaxTopK / 16; ++i)
                if (c == (j & 15) && (j >> 4) == i) mine[t][i] = best[t];
        }
    }
#pragma unroll
    for (int t = 0; t < NR; ++t) {
        const float vmax = key_value<EL>(first[t]);
        float e[kMaxTopK / 16];
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < kMaxTopK / 16; ++i) {
            e[i] = c + 16 * i < k ? expf(key_value<EL>(mine[t][i]) - vmax) : 0.f;
            sum += e[i];
        }
        sum = row16_sum(sum);
        if (token[t] < a.T) {
#pragma unroll
            for (int i = 0; i < kMaxTopK / 16; ++i) {
                const int j = c + 16 * i;
                if (j < k) {
                    const int col = key_column(mine[t][i]);
                    a.selected[token[t] * k + j] = col;
                    a.weights[token[t] * k + j] = EL::bits(e[i] / sum);
                    if (a.counts || a.hist) atomicAdd(&s_hist[(int)((token[t] - tok0) >> 4) * E + col], 1u);
                }
            }
        }
    }
}

// s_hist: [groups][E], one row per 16 consecutive tokens of the workgroup (its first token tok0 is a multiple of 16)
__device__ __forceinline__ void clear_histogram(const RouterArgs& a, uint32_t* s_hist, int groups, int tid, int nthreads) {
    if (a.counts || a.hist)
        for (int n = tid; n < groups * a.E; n += nthreads) s_hist[n] = 0;
}
__device__ __forceinline__ void flush_histogram(const RouterArgs& a, const uint32_t* s_hist, int groups, int64_t tok0,
                                                int tid, int nthreads) {
    if (!a.counts && !a.hist) return;
    __syncthreads();
    if (a.hist) {
        // every row of 16 tokens belongs to one workgroup: plain stores, nothing to clear beforehand
        const int64_t row0 = tok0 >> 4, nrows = (a.T + 15) >> 4;
        for (int g = 0; g < groups; ++g)
            if (row0 + g < nrows)
                for (int n = tid; n < a.E; n += nthreads) a.hist[(row0 + g) * a.E + n] = s_hist[g * a.E + n];
    }
    if (a.counts) {
        for (int n = tid; n < a.E; n += nthreads) {
            uint32_t h = 0;
            for (int g = 0; g < groups; ++g) h += s_hist[g * a.E + n];
            if (h) atomicAdd(a.counts + n, h);
        }
    }
}

// NBLK: 16-expert column blocks accumulated per pass over x; RB: 16-token row blocks per workgroup (each weight
// fragment fetched from the L2 is used RB times); EMAX: capacity of the LDS key rows (E <= EMAX)
template <typename EL, int NBLK, int RB, int EMAX>
__global__ __launch_bounds__(kRouterThreads) void router_topk_kernel(const RouterArgs a) {
    using frag = typename EL::frag;
    constexpr int kCols = NBLK * 16, kToks = RB * kTok;
    __shared__ float s_part[kRouterWaves][kToks][kCols];
    __shared__ uint32_t s_key[kToks][EMAX + kRowPad];
    __shared__ uint32_t s_hist[RB * EMAX];

    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const int r = lane & 15, q = lane >> 4;
    const int H = a.H, E = a.E;
    const int64_t tok0 = (int64_t)blockIdx.x * kToks;

    clear_histogram(a, s_hist, RB, tid, kRouterThreads);

    // ---- logits: 16 RB tokens x E, this wavefront's share of the reduction dimension -------------------------------
    const uint16_t* xa[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        const int64_t t = tok0 + rb * kTok + r;
        xa[rb] = a.x + (t < a.T ? t : a.T - 1) * H + q * 32;  // rows past the end repeat the last token, never stored
    }
    const int nfull = H / kStepK;           // whole steps; step ms belongs to wavefront ms % 4
    const bool has_tail = (H % kStepK) != 0;  // the partial last step belongs to wavefront nfull % 4

    for (int col0 = 0; col0 < E; col0 += kCols) {
        f32x4 acc[RB][NBLK];
        const uint16_t* wb[NBLK];
#pragma unroll
        for (int b = 0; b < NBLK; ++b) {
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) acc[rb][b] = f32x4{0.f, 0.f, 0.f, 0.f};
            const int n = col0 + b * 16 + r;
            wb[b] = a.w + (int64_t)(n < E ? n : E - 1) * H + q * 32;  // columns past E repeat the last expert
        }
        // The activations of the next step are requested after the weights of this one and before this step's MFMAs:
        // loads return in order, so waiting for the weights then leaves only the next step's activations in flight,
        // and their (HBM) latency runs under this step's arithmetic and the next step's weight fetch.
        int ms = wave;
        frag cur[RB][4];
        if (ms < nfull) {
#pragma unroll
            for (int rb = 0; rb < RB; ++rb)
#pragma unroll
                for (int j = 0; j < 4; ++j) cur[rb][j] = load_frag<frag>(xa[rb] + ms * kStepK + j * 8);
        }
        while (ms < nfull) {
            const int k0 = ms * kStepK;
            const int nx = ms + kRouterWaves;
            const int kp = (nx < nfull ? nx : ms) * kStepK;  // nothing follows: fetch this step again, unused
            frag bf[NBLK][4];
#pragma unroll
            for (int b = 0; b < NBLK; ++b)
#pragma unroll
                for (int j = 0; j < 4; ++j) bf[b][j] = load_frag<frag>(wb[b] + k0 + j * 8);
            __builtin_amdgcn_sched_barrier(0);
            frag nxt[RB][4];
#pragma unroll
            for (int rb = 0; rb < RB; ++rb)
#pragma unroll
                for (int j = 0; j < 4; ++j) nxt[rb][j] = load_frag<frag>(xa[rb] + kp + j * 8);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int b = 0; b < NBLK; ++b)
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int rb = 0; rb < RB; ++rb) acc[rb][b] = EL::mfma(cur[rb][j], bf[b][j], acc[rb][b]);
#pragma unroll
            for (int rb = 0; rb < RB; ++rb)
#pragma unroll
                for (int j = 0; j < 4; ++j) cur[rb][j] = nxt[rb][j];
            ms = nx;
        }
        if (has_tail && wave == (nfull & (kRouterWaves - 1))) {
            // partial last step: 16-byte units past the end of the row contribute zeros (H is a multiple of 8)
            const int k0 = nfull * kStepK;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const bool in = k0 + q * 32 + j * 8 < H;
                const int off = in ? k0 + j * 8 : -(q * 32);  // an address inside the row either way
                const frag zero = __builtin_bit_cast(frag, u32x4{0u, 0u, 0u, 0u});
                frag af[RB];
#pragma unroll
                for (int rb = 0; rb < RB; ++rb) {
                    af[rb] = load_frag<frag>(xa[rb] + off);
                    if (!in) af[rb] = zero;
                }
#pragma unroll
                for (int b = 0; b < NBLK; ++b) {
                    frag bw = load_frag<frag>(wb[b] + off);
                    if (!in) bw = zero;
#pragma unroll
                    for (int rb = 0; rb < RB; ++rb) acc[rb][b] = EL::mfma(af[rb], bw, acc[rb][b]);
                }
            }
        }
        // accumulator element i of a lane is row (lane / 16) * 4 + i, column lane % 16 of the 16 x 16 tile
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int b = 0; b < NBLK; ++b)
#pragma unroll
                for (int i = 0; i < 4; ++i) s_part[wave][rb * kTok + q * 4 + i][b * 16 + r] = acc[rb][b][i];
        __syncthreads();
        // sum of the four partial results in a fixed order, one rounding; thread (token, c) handles the columns
        // congruent to c mod 16, which are also the columns it scans in the top-k below
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            const int tok = rb * kTok + (tid >> 4), c = tid & 15;
#pragma unroll
            for (int b = 0; b < NBLK; ++b) {
                const int col = b * 16 + c, n = col0 + col;
                const float v = (s_part[0][tok][col] + s_part[1][tok][col]) + (s_part[2][tok][col] + s_part[3][tok][col]);
                if (n < E) {
                    const uint16_t bits = EL::bits(v);
                    s_key[tok][n] = make_key<EL>(bits, n);
                    if (tok0 + tok < a.T) a.logits[(tok0 + tok) * E + n] = bits;
                }
            }
        }
        __syncthreads();  // s_part is rewritten by the next pass
    }

    // ---- top-k and softmax over the kept logits ----------------------------------------------------------------------
    {
        uint32_t* rows[RB];
        int64_t tokens[RB];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            rows[rb] = s_key[rb * kTok + (tid >> 4)];
            tokens[rb] = tok0 + rb * kTok + (tid >> 4);
        }
        topk_softmax_tokens<EL, RB>(rows, tid & 15, tokens, tok0, a, s_hist);
    }
    flush_histogram(a, s_hist, RB, tok0, tid, kRouterThreads);
}

// ---- the same for more than 16 experts -------------------------------------------------------------------------------
// With many experts the router weights are the larger operand per token block, and fetching them once per wavefront
// (as above) makes the L2 the bottleneck. Here the four wavefronts of a workgroup own 16 tokens each, over the whole
// reduction dimension, and share the weights through LDS: per 128-element step the workgroup stages one
// [16 NBLK experts] x [128] tile (double-buffered, one barrier per step), every wavefront reads its B fragments from
// it, and the activations stream from global memory into registers kRing - 1 steps ahead. No cross-wavefront reduction:
// each accumulator tile is a finished 16 x 16 block of logits.
constexpr int kRing = 4;                        // operands are requested kRing - 1 steps before their use (even: the
                                                // LDS tile index step % 2 is taken from the ring index)
constexpr int kTileRowBytes = kStepK * 2 + 16;  // 16 bytes of padding: consecutive expert rows start 4 banks apart

// W: wavefronts (of 16 tokens each) per workgroup: 4, or 2 when the token count would otherwise leave compute units idle
template <typename EL, int NBLK, int EMAX, int W>
__global__ __launch_bounds__(W * kWave) void router_topk_wide_kernel(const RouterArgs a) {
    using frag = typename EL::frag;
    constexpr int kThreadsW = W * kWave;
    constexpr int kUnits = NBLK * 256 / kThreadsW;  // 16-byte units of a weight tile per thread
    constexpr int kCols = NBLK * 16, kToks = W * kTok;
    __shared__ __attribute__((aligned(16))) uint8_t s_tile[2][kCols * kTileRowBytes];
    __shared__ uint32_t s_key[kToks][EMAX + kRowPad];
    __shared__ uint32_t s_hist[W * EMAX];

    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const int r = lane & 15, q = lane >> 4;
    const int H = a.H, E = a.E;
    const int64_t tok0 = (int64_t)blockIdx.x * kToks;

    clear_histogram(a, s_hist, W, tid, kThreadsW);

    const int64_t t_mine = tok0 + wave * kTok + r;
    const uint16_t* xa = a.x + (t_mine < a.T ? t_mine : a.T - 1) * H + q * 32;  // past the end: the last token again
    const int nsteps = (H + kStepK - 1) / kStepK;
    const frag zero = __builtin_bit_cast(frag, u32x4{0u, 0u, 0u, 0u});

    // 16-byte unit u of a weight tile: expert row u / 16, reduction offset (u % 16) * 8; thread t moves the units
    // t, t + 256, ...: 16 consecutive threads fetch 256 consecutive bytes of one expert's row.
    // The unchecked forms are for whole steps of the pipelined loop (nothing may consume a loaded register right after
    // the load there, or the wavefront waits for it on the spot); the checked forms zero what lies past the end of the
    // row (H is a multiple of 8: a 16-byte unit is inside the row or outside).
    auto fetch_tile = [&](u32x4 (&regs)[kUnits], int col0, int step) {
#pragma unroll
        for (int i = 0; i < kUnits; ++i) {
            const int u = tid + i * kThreadsW;
            const int n = col0 + (u >> 4);
            regs[i] = *reinterpret_cast<const u32x4*>(a.w + (int64_t)(n < E ? n : E - 1) * H + step * kStepK + (u & 15) * 8);
        }
    };
    auto fetch_tile_checked = [&](u32x4 (&regs)[kUnits], int col0, int step) {
#pragma unroll
        for (int i = 0; i < kUnits; ++i) {
            const int u = tid + i * kThreadsW;
            const int n = col0 + (u >> 4), kk = step * kStepK + (u & 15) * 8;
            const bool in = kk < H;
            regs[i] = *reinterpret_cast<const u32x4*>(a.w + (int64_t)(n < E ? n : E - 1) * H + (in ? kk : 0));
            if (!in) regs[i] = u32x4{0u, 0u, 0u, 0u};
        }
    };
    auto store_tile = [&](const u32x4 (&regs)[kUnits], int buf) {
#pragma unroll
        for (int i = 0; i < kUnits; ++i) {
            const int u = tid + i * kThreadsW;
            *reinterpret_cast<u32x4*>(&s_tile[buf][(u >> 4) * kTileRowBytes + (u & 15) * 16]) = regs[i];
        }
    };
    auto fetch_x = [&](frag (&dst)[4], int step) {
#pragma unroll
        for (int j = 0; j < 4; ++j) dst[j] = load_frag<frag>(xa + step * kStepK + j * 8);
    };
    auto fetch_x_checked = [&](frag (&dst)[4], int step) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const bool in = step * kStepK + q * 32 + j * 8 < H;
            dst[j] = load_frag<frag>(xa + (in ? step * kStepK + j * 8 : -(q * 32)));
            if (!in) dst[j] = zero;
        }
    };
    auto multiply = [&](f32x4 (&acc)[NBLK], const frag (&xf)[4], int buf) {
#pragma unroll
        for (int b = 0; b < NBLK; ++b) {
            frag bw[4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
                bw[j] = __builtin_bit_cast(
                    frag, *reinterpret_cast<const u32x4*>(&s_tile[buf][(b * 16 + r) * kTileRowBytes + q * 64 + j * 16]));
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[b] = EL::mfma(xf[j], bw[j], acc[b]);
        }
    };

    // whole steps in groups of kRing run in the pipelined loop, the rest (fewer than kRing whole steps and the partial
    // last one) one at a time after it
    const int npipe = (H / kStepK) / kRing * kRing;

    for (int col0 = 0; col0 < E; col0 += kCols) {
        f32x4 acc[NBLK];
#pragma unroll
        for (int b = 0; b < NBLK; ++b) acc[b] = f32x4{0.f, 0.f, 0.f, 0.f};
        __syncthreads();  // the previous pass (or the histogram clearing) is done with LDS

        if (npipe > 0) {
            // Rings of kRing steps, indexed by step % kRing: step s uses xq[s % kRing] and the LDS tile s % 2,
            // requests the operands of step s + kRing - 1 (past the end of the loop: of its last step again, unused),
            // and moves the weight tile of step s + 1, requested two steps earlier, from registers to LDS. One
            // wavefront per SIMD is the usual occupancy here (a wavefront per 16 tokens), so the latency of the L2 and
            // of HBM is covered by this distance, not by other wavefronts.
            frag xq[kRing][4];
            u32x4 staged[kRing][kUnits];
#pragma unroll
            for (int d = 0; d < kRing - 1; ++d) {
                fetch_tile(staged[d], col0, d);
                fetch_x(xq[d], d);
            }
            store_tile(staged[0], 0);
            __syncthreads();
            for (int base = 0; base < npipe; base += kRing) {
#pragma unroll
                for (int ph = 0; ph < kRing; ++ph) {
                    const int ahead = base + ph + kRing - 1 < npipe ? base + ph + kRing - 1 : npipe - 1;
                    fetch_tile(staged[(ph + kRing - 1) % kRing], col0, ahead);
                    fetch_x(xq[(ph + kRing - 1) % kRing], ahead);
                    multiply(acc, xq[ph], ph & 1);
                    store_tile(staged[(ph + 1) % kRing], (ph + 1) & 1);
                    __syncthreads();  // tile step + 1 is complete; tile step may be overwritten in the next step
                }
            }
        }
        for (int step = npipe; step < nsteps; ++step) {
            u32x4 staged[kUnits];
            frag xf[4];
            fetch_tile_checked(staged, col0, step);
            fetch_x_checked(xf, step);
            store_tile(staged, 0);
            __syncthreads();
            multiply(acc, xf, 0);
            __syncthreads();
        }

        // accumulator element i of a lane: token (lane / 16) * 4 + i of this wavefront, column lane % 16 of block b
#pragma unroll
        for (int b = 0; b < NBLK; ++b) {
            const int n = col0 + b * 16 + r;
            if (n < E) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int tok = wave * kTok + q * 4 + i;
                    const uint16_t bits = EL::bits(acc[b][i]);
                    s_key[tok][n] = make_key<EL>(bits, n);
                    if (tok0 + tok < a.T) a.logits[(tok0 + tok) * E + n] = bits;
                }
            }
        }
    }
    __syncthreads();

    // ---- top-k and softmax over the kept logits ----------------------------------------------------------------------
    {
        // 16 lanes per token: W * 4 tokens at a time, four rounds
        uint32_t* rows[4];
        int64_t tokens[4];
#pragma unroll
        for (int round = 0; round < 4; ++round) {
            rows[round] = s_key[round * (W * 4) + (tid >> 4)];
            tokens[round] = tok0 + round * (W * 4) + (tid >> 4);
        }
        topk_softmax_tokens<EL, 4>(rows, tid & 15, tokens, tok0, a, s_hist);
    }
    flush_histogram(a, s_hist, W, tok0, tid, kThreadsW);
}

template <typename EL, int NBLK, int EMAX>
int launch_router_wide(const RouterArgs& a, hipStream_t st) {
    // 64 tokens per workgroup share each weight tile four ways; with too few tokens to give every compute unit such a
    // workgroup, 32 tokens per workgroup keep twice as many units busy
    const int64_t cus = num_compute_units() > 0 ? num_compute_units() : 256;
    if ((a.T + 63) / 64 >= cus) {
        const uint32_t blocks = (uint32_t)((a.T + 63) / 64);
        hipLaunchKernelGGL((router_topk_wide_kernel<EL, NBLK, EMAX, 4>), dim3(blocks), dim3(256), 0, st, a);
    } else {
        const uint32_t blocks = (uint32_t)((a.T + 31) / 32);
        hipLaunchKernelGGL((router_topk_wide_kernel<EL, NBLK, EMAX, 2>), dim3(blocks), dim3(128), 0, st, a);
    }
    return launch_status("router_topk");
}

template <typename EL, int NBLK, int RB, int EMAX>
int launch_router_as(const RouterArgs& a, hipStream_t st) {
    const int64_t toks = (int64_t)RB * kTok;
    const uint32_t blocks = (uint32_t)((a.T + toks - 1) / toks);
    hipLaunchKernelGGL((router_topk_kernel<EL, NBLK, RB, EMAX>), dim3(blocks), dim3(kRouterThreads), 0, st, a);
    return launch_status("router_topk");
}

// More tokens per workgroup mean fewer fetches of the router weights, fewer tokens mean more workgroups: take the most
// tokens that still leave two workgroups per compute unit.
template <typename EL, int NBLK, int EMAX, int RBMAX>
int launch_router_rows(const RouterArgs& a, hipStream_t st) {
    const int64_t want = 2 * (int64_t)(num_compute_units() > 0 ? num_compute_units() : 256);
    int rb = 1;
    if (RBMAX >= 4 && a.T >= want * 4 * kTok) rb = 4;
    else if (RBMAX >= 2 && a.T >= want * 2 * kTok) rb = 2;
    if constexpr (RBMAX >= 4)
        if (rb == 4) return launch_router_as<EL, NBLK, 4, EMAX>(a, st);
    if constexpr (RBMAX >= 2)
        if (rb == 2) return launch_router_as<EL, NBLK, 2, EMAX>(a, st);
    return launch_router_as<EL, NBLK, 1, EMAX>(a, st);
}

template <typename EL>
int launch_router(const RouterArgs& a, hipStream_t st) {
    if (a.counts) {
        hipLaunchKernelGGL(fill_u32_kernel, dim3((a.E + kRouterThreads - 1) / kRouterThreads), dim3(kRouterThreads), 0,
                           st, a.counts, (int64_t)a.E, 0u);
        int rc = launch_status("router_topk (clearing counts)");
        if (rc) return rc;
    }
    if (a.E <= 16) return launch_router_rows<EL, 1, 16, 4>(a, st);
    if (a.E <= 32) return launch_router_wide<EL, 2, 32>(a, st);
    if (a.E <= 64) return launch_router_wide<EL, 4, 64>(a, st);
    if (a.E <= 128) return launch_router_wide<EL, 8, 128>(a, st);
    if (a.E <= 256) return launch_router_wide<EL, 8, 256>(a, st);  // two passes over the activations
    // beyond that the key rows of 64 tokens no longer fit in LDS: 16 tokens per workgroup, weights straight from the L2
    return launch_router_rows<EL, 4, FMA_MAX_GROUPS, 1>(a, st);
}

// ---- backward of top-k + softmax ------------------------------------------------------------------------------------
// d_out[t, :] = d_logits[t, :] (zeros if absent), and at the k chosen columns additionally the softmax backward
// ds_j = s_j (dw_j - sum_i s_i dw_i), rounded to the activation dtype before the addition (autograd hands the gradient
// of `values.float()` back in the activation dtype, and adds the two contributions to the logits in that dtype).
// 16 lanes per token.
template <typename EL>
__global__ __launch_bounds__(kRouterThreads) void router_topk_bwd_kernel(const uint16_t* __restrict__ logits,
                                                                         const int32_t* __restrict__ selected,
                                                                         const uint16_t* __restrict__ d_weights,
                                                                         const uint16_t* __restrict__ d_logits,
                                                                         int64_t T, int E, int k,
                                                                         uint16_t* __restrict__ d_out) {
    __shared__ int32_t s_sel[kTok][kMaxTopK];
    __shared__ float s_ds[kTok][kMaxTopK];
    const int tid = threadIdx.x, tok = tid >> 4, c = tid & 15;
    const int64_t t = (int64_t)blockIdx.x * kTok + tok;
    const bool live = t < T;
    const int64_t tt = live ? t : T - 1;

    // kMaxTopK / 16 = 4 choices per lane at most
    float val[kMaxTopK / 16], dw[kMaxTopK / 16];
    int sel[kMaxTopK / 16];
    float vmax = 0.f;
    {
        const int s0 = selected[tt * k];
        vmax = EL::from_bits(logits[tt * E + (s0 < 0 ? 0 : (s0 < E ? s0 : E - 1))]);  // the first choice is the largest kept logit
    }
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < kMaxTopK / 16; ++i) {
        const int j = c + 16 * i;
        sel[i] = -1;
        val[i] = 0.f;
        dw[i] = 0.f;
        if (j < k) {
            sel[i] = selected[tt * k + j];
            const int col = sel[i] < 0 ? 0 : (sel[i] < E ? sel[i] : E - 1);  // a corrupt index must not become a wild read
            val[i] = expf(EL::from_bits(logits[tt * E + col]) - vmax);
            dw[i] = d_weights ? EL::from_bits(d_weights[tt * k + j]) : 0.f;
            sum += val[i];
        }
    }
#pragma unroll
    for (int d = 1; d < 16; d <<= 1) sum += __shfl_xor(sum, d, kWave);
    float dot = 0.f;
#pragma unroll
    for (int i = 0; i < kMaxTopK / 16; ++i) {
        val[i] = val[i] / sum;  // s_j
        dot += val[i] * dw[i];
    }
#pragma unroll
    for (int d = 1; d < 16; d <<= 1) dot += __shfl_xor(dot, d, kWave);
#pragma unroll
    for (int i = 0; i < kMaxTopK / 16; ++i) {
        const int j = c + 16 * i;
        if (j < k) {
            s_sel[tok][j] = sel[i];
            s_ds[tok][j] = EL::round(val[i] * (dw[i] - dot));
        }
    }
    __syncthreads();
    if (!live) return;
    for (int n = c; n < E; n += 16) {
        float v = d_logits ? EL::from_bits(d_logits[t * E + n]) : 0.f;
        for (int j = 0; j < k; ++j)
            if (s_sel[tok][j] == n) v = s_ds[tok][j] + v;
        d_out[t * E + n] = EL::bits(v);
    }
}

int check_router(const char* what, int dtype, int64_t T, int64_t E, int64_t k) {
    FMA_REQUIRE(dtype == FMA_BF16 || dtype == FMA_F16, FMA_ERR_BAD_DTYPE, "%s: dtype must be FMA_BF16 or FMA_F16 (got %d)",
                what, dtype);
    FMA_REQUIRE(T >= 0 && T <= 0x7fffffffll, FMA_ERR_BAD_SIZE, "%s: bad token count %lld", what, (long long)T);
    FMA_REQUIRE(E >= 1 && E <= FMA_MAX_GROUPS, FMA_ERR_TOO_MANY_EXPERTS, "%s: E must be in [1, %d] (got %lld)", what,
                FMA_MAX_GROUPS, (long long)E);
    FMA_REQUIRE(k >= 1 && k <= E && k <= FMA_MAX_ROUTER_TOP_K, FMA_ERR_BAD_SIZE,
                "%s: top_k must be in [1, min(E, %d)] (got %lld, E = %lld)", what, FMA_MAX_ROUTER_TOP_K, (long long)k,
                (long long)E);
    FMA_REQUIRE(T * E <= 0x7fffffffll && T * k <= 0x7fffffffll, FMA_ERR_TOO_MANY_ELEMENTS,
                "%s: T*E and T*top_k must stay below 2^31", what);
    return FMA_OK;
}

}  // namespace
}  // namespace fmahip

extern "C" {

int fma_router_topk(const void* x, const void* gate_weight, int64_t T, int64_t H, int64_t E, int64_t top_k,
                    void* logits, void* weights, int32_t* selected, uint32_t* counts, uint32_t* token_block_hist,
                    int dtype, void* stream) {
    using namespace fmahip;
    static_assert(kMaxTopK == FMA_MAX_ROUTER_TOP_K, "header and kernel disagree on the top_k limit");
    int rc = check_router("router_topk", dtype, T, E, top_k);
    if (rc) return rc;
    FMA_REQUIRE(H >= 8 && H % 8 == 0 && H <= (1 << 24), FMA_ERR_BAD_SIZE,
                "router_topk: H must be a multiple of 8 in [8, 2^24] (got %lld)", (long long)H);
    if (T == 0) {
        if (counts) {
            hipLaunchKernelGGL(fill_u32_kernel, dim3((uint32_t)((E + kRouterThreads - 1) / kRouterThreads)),
                               dim3(kRouterThreads), 0, (hipStream_t)stream, counts, E, 0u);
            return launch_status("router_topk (clearing counts)");
        }
        return FMA_OK;
    }
    FMA_REQUIRE(x && gate_weight && logits && weights && selected, FMA_ERR_NULL_POINTER, "router_topk: NULL pointer");
    FMA_REQUIRE(aligned16(x) && aligned16(gate_weight), FMA_ERR_MISALIGNED,
                "router_topk: x and gate_weight must be 16-byte aligned");
    RouterArgs a;
    a.x = (const uint16_t*)x;
    a.w = (const uint16_t*)gate_weight;
    a.logits = (uint16_t*)logits;
    a.weights = (uint16_t*)weights;
    a.selected = selected;
    a.counts = counts;
    a.hist = token_block_hist;
    a.T = T;
    a.H = (int32_t)H;
    a.E = (int32_t)E;
    a.k = (int32_t)top_k;
    return dtype == FMA_BF16 ? launch_router<RouterBf16>(a, (hipStream_t)stream)
                             : launch_router<RouterF16>(a, (hipStream_t)stream);
}

int fma_router_topk_bwd(const void* logits, const int32_t* selected, const void* d_weights, const void* d_logits,
                        int64_t T, int64_t E, int64_t top_k, void* d_out, int dtype, void* stream) {
    using namespace fmahip;
    int rc = check_router("router_topk_bwd", dtype, T, E, top_k);
    if (rc) return rc;
    if (T == 0) return FMA_OK;
    FMA_REQUIRE(logits && selected && d_out, FMA_ERR_NULL_POINTER, "router_topk_bwd: NULL pointer");
    const uint32_t blocks = (uint32_t)((T + kTok - 1) / kTok);
    if (dtype == FMA_BF16)
        hipLaunchKernelGGL(router_topk_bwd_kernel<RouterBf16>, dim3(blocks), dim3(kRouterThreads), 0,
                           (hipStream_t)stream, (const uint16_t*)logits, selected, (const uint16_t*)d_weights,
                           (const uint16_t*)d_logits, T, (int)E, (int)top_k, (uint16_t*)d_out);
    else
        hipLaunchKernelGGL(router_topk_bwd_kernel<RouterF16>, dim3(blocks), dim3(kRouterThreads), 0,
                           (hipStream_t)stream, (const uint16_t*)logits, selected, (const uint16_t*)d_weights,
                           (const uint16_t*)d_logits, T, (int)E, (int)top_k, (uint16_t*)d_out);
    return launch_status("router_topk_bwd");
}

}  // extern "C"
