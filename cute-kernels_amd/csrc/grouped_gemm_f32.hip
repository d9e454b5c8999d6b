// Grouped GEMM for fp32 operands: D_e = alpha * op(A_e) op(B_e) on the fp32 matrix instruction (v_mfma_f32_32x32x2_f32,
// 157 TFLOP/s peak: one sixteenth of the bf16 rate, so this kernel is bound by the matrix pipe long before memory and is
// kept simple). 128 x 128 output tiles, 16-wide K steps, four wavefronts of 64 x 64 each. Operands are fetched element
// by element with bounds checks (any M, N, K and either storage order; rows past a group's edge and K past its end read as
// zero) two K steps ahead into registers, staged in LDS as [row][16 k] with rows padded to 20 floats, double-buffered
// with one barrier per K step. The instruction multiplies two k values at a time (lane half h supplies one of them);
// since the order of a sum's terms is free, half h takes k = 8 h .. 8 h + 7 of the step, so a lane's eight values of a
// fragment are contiguous in LDS and come with two 16-byte reads (the padded rows make those conflict-free).
// Workgroups are persistent and find their tiles in a per-workgroup prefix table of the groups' tile counts, like the
// 16-bit kernel.
#include "common.h"
#include "grouped_gemm_f32.h"

namespace fmahip {
namespace gemm_f32 {
namespace {

typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int BM = 128, BN = 128, BK = 16;
constexpr int kThreads = 256;
constexpr int kPitch = 20;                           // floats per LDS row: 16 k + 4 of padding
constexpr int kPerThread = BM * BK / kThreads;       // operand elements per thread and K step (8)
static_assert(BM == BN, "one staging routine serves both operands");

struct Args {
    const float* A;
    const float* B;
    float* D;
    const uint32_t* M_arr;
    const uint32_t* N_arr;
    const uint32_t* K_arr;
    uint32_t E;
    float alpha;
};

// Element (row, k) of an operand tile for thread-local index i: consecutive threads walk the operand's contiguous
// dimension. K_CONTIG: stored [rows, K]; otherwise stored [K, rows].
template <bool K_CONTIG>
__device__ __forceinline__ void element_of(int i, int tid, int& row, int& k) {
    const int e = tid + i * kThreads;
    if constexpr (K_CONTIG) {
        row = e / BK;
        k = e % BK;
    } else {
        k = e / BM;
        row = e % BM;
    }
}

// Requests the thread's elements of the operand tile at (row0, k0). Elements outside the operand are requested from
// its first element instead (a valid address: a tile exists only if M, N >= 1, a K step only if K >= 1) and replaced by
// zeros in stage(): nothing here consumes a loaded value, so the loads stay in flight until the data is needed.
template <bool K_CONTIG>
__device__ __forceinline__ void fetch(float (&regs)[kPerThread], const float* __restrict__ base, uint32_t rows,
                                      uint32_t K, uint32_t row0, uint32_t k0, int tid) {
#pragma unroll
    for (int i = 0; i < kPerThread; ++i) {
        int r, k;
        element_of<K_CONTIG>(i, tid, r, k);
        const uint32_t row = row0 + r, kk = k0 + k;
        const bool in = row < rows && kk < K;
        const uint64_t idx = K_CONTIG ? (uint64_t)row * K + kk : (uint64_t)kk * rows + row;
        regs[i] = base[in ? idx : 0];
    }
}

template <bool K_CONTIG>
__device__ __forceinline__ void stage(const float (&regs)[kPerThread], float* __restrict__ tile, uint32_t rows,
                                      uint32_t K, uint32_t row0, uint32_t k0, int tid) {
#pragma unroll
    for (int i = 0; i < kPerThread; ++i) {
        int r, k;
        element_of<K_CONTIG>(i, tid, r, k);
        const bool in = row0 + r < rows && k0 + k < K;
        tile[r * kPitch + k] = in ? regs[i] : 0.0f;
    }
}

template <bool A_KC, bool B_KC>
__global__ __launch_bounds__(kThreads) void grouped_gemm_f32_kernel(const Args args) {
    __shared__ __attribute__((aligned(16))) float s_a[2][BM * kPitch];
    __shared__ __attribute__((aligned(16))) float s_b[2][BN * kPitch];
    __shared__ uint32_t s_tile_start[FMA_MAX_GROUPS + 1];
    __shared__ uint64_t s_off_a[FMA_MAX_GROUPS], s_off_b[FMA_MAX_GROUPS], s_off_d[FMA_MAX_GROUPS];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;  // 2 x 2 wavefronts of 64 x 64

    if (tid == 0) {
        uint32_t tiles = 0;
        uint64_t oa = 0, ob = 0, od = 0;
        for (uint32_t e = 0; e < args.E; ++e) {
            const uint64_t M = args.M_arr[e], N = args.N_arr[e], K = args.K_arr[e];
            s_tile_start[e] = tiles;
            s_off_a[e] = oa;
            s_off_b[e] = ob;
            s_off_d[e] = od;
            tiles += (uint32_t)(((M + BM - 1) / BM) * ((N + BN - 1) / BN));
            oa += M * K;
            ob += K * N;
            od += M * N;
        }
        s_tile_start[args.E] = tiles;
    }
    __syncthreads();
    const uint32_t total = s_tile_start[args.E];

    for (uint32_t tile = blockIdx.x; tile < total; tile += gridDim.x) {
        // the group of this tile: last e with s_tile_start[e] <= tile (empty groups share their start with the next)
        uint32_t lo = 0, hi = args.E;
        while (hi - lo > 1) {
            const uint32_t mid = (lo + hi) >> 1;
            if (s_tile_start[mid] <= tile) lo = mid;
            else hi = mid;
        }
        while (s_tile_start[lo + 1] <= tile) ++lo;  // skip groups without tiles
        const uint32_t e = lo;
        const uint32_t Me = args.M_arr[e], Ne = args.N_arr[e], Ke = args.K_arr[e];
        const uint32_t tiles_n = (Ne + BN - 1) / BN;
        const uint32_t local = tile - s_tile_start[e];
        const uint32_t m0 = (local / tiles_n) * BM, n0 = (local % tiles_n) * BN;
        const float* Ae = args.A + s_off_a[e];
        const float* Be = args.B + s_off_b[e];
        float* De = args.D + s_off_d[e];

        f32x16 acc[2][2];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int x = 0; x < 16; ++x) acc[i][j][x] = 0.0f;

        const uint32_t KT = (Ke + BK - 1) / BK;
        // two register sets: set s holds the operands of the steps with kt % 2 == s, fetched two steps before their use
        float ra[2][kPerThread], rb[2][kPerThread];
        auto compute = [&](int buf) {
            // lane l: row (l % 32) of a 32-row block, k values 8 (l / 32) .. + 7 of the step
            const float* ta = s_a[buf] + (wm * 64 + (lane & 31)) * kPitch + (lane >> 5) * 8;
            const float* tb = s_b[buf] + (wn * 64 + (lane & 31)) * kPitch + (lane >> 5) * 8;
            float4 fa[2][2], fb[2][2];
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int hh = 0; hh < 2; ++hh) {
                    fa[i][hh] = *reinterpret_cast<const float4*>(ta + i * 32 * kPitch + hh * 4);
                    fb[i][hh] = *reinterpret_cast<const float4*>(tb + i * 32 * kPitch + hh * 4);
                }
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) {
                // B first: a lane then owns one output row and four consecutive output columns per register quad
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        const float av = reinterpret_cast<const float*>(&fa[i][kk >> 2])[kk & 3];
                        const float bv = reinterpret_cast<const float*>(&fb[j][kk >> 2])[kk & 3];
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv, av, acc[i][j], 0, 0, 0);
                    }
            }
        };
        if (KT > 0) {
            fetch<A_KC>(ra[0], Ae, Me, Ke, m0, 0, tid);
            fetch<B_KC>(rb[0], Be, Ne, Ke, n0, 0, tid);
            fetch<A_KC>(ra[1], Ae, Me, Ke, m0, BK, tid);  // past the end of K: zeros
            fetch<B_KC>(rb[1], Be, Ne, Ke, n0, BK, tid);
            __syncthreads();  // the previous tile is done with the LDS stages
            stage<A_KC>(ra[0], s_a[0], Me, Ke, m0, 0, tid);
            stage<B_KC>(rb[0], s_b[0], Ne, Ke, n0, 0, tid);
            __syncthreads();
        }
        for (uint32_t kt = 0; kt < KT; kt += 2) {
#pragma unroll
            for (int ph = 0; ph < 2; ++ph) {
                // step kt + ph (a step past the last one multiplies zeros): request step + 2 into the set this step's
                // operands came from, multiply from stage ph, move step + 1 from its registers to the other stage
                fetch<A_KC>(ra[ph], Ae, Me, Ke, m0, (kt + ph + 2) * BK, tid);
                fetch<B_KC>(rb[ph], Be, Ne, Ke, n0, (kt + ph + 2) * BK, tid);
                compute(ph);
                stage<A_KC>(ra[ph ^ 1], s_a[ph ^ 1], Me, Ke, m0, (kt + ph + 1) * BK, tid);
                stage<B_KC>(rb[ph ^ 1], s_b[ph ^ 1], Ne, Ke, n0, (kt + ph + 1) * BK, tid);
                __syncthreads();  // stage ph^1 is complete; stage ph may be overwritten in the next step
            }
        }

        // accumulator register 4 q + j of block (i, j'): row m = ... + (lane % 32), column n = ... + 8 q + 4 (lane / 32) + j
        const float alpha = args.alpha;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const uint32_t m = m0 + wm * 64 + i * 32 + (lane & 31);
            if (m >= Me) continue;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const uint32_t n = n0 + wn * 64 + j * 32 + q * 8 + (lane >> 5) * 4;
                    float* dst = De + (uint64_t)m * Ne + n;
                    if (n + 3 < Ne && (reinterpret_cast<uintptr_t>(dst) & 15u) == 0) {
                        float4 v = {alpha * acc[i][j][q * 4 + 0], alpha * acc[i][j][q * 4 + 1], alpha * acc[i][j][q * 4 + 2],
                                    alpha * acc[i][j][q * 4 + 3]};
                        *reinterpret_cast<float4*>(dst) = v;
                    } else {
#pragma unroll
                        for (int x = 0; x < 4; ++x)
                            if (n + x < Ne) dst[x] = alpha * acc[i][j][q * 4 + x];
                    }
                }
            }
        }
    }
}

}  // namespace

int launch(const void* A, const void* B, void* D, const uint32_t* M_arr, const uint32_t* N_arr, const uint32_t* K_arr,
           int64_t E, bool a_kc, bool b_kc, float alpha, hipStream_t st) {
    Args args;
    args.A = (const float*)A;
    args.B = (const float*)B;
    args.D = (float*)D;
    args.M_arr = M_arr;
    args.N_arr = N_arr;
    args.K_arr = K_arr;
    args.E = (uint32_t)E;
    args.alpha = alpha;
    const int cus = num_compute_units() > 0 ? num_compute_units() : 256;
    const dim3 grid((uint32_t)(2 * cus)), block(kThreads);
    if (a_kc && b_kc) hipLaunchKernelGGL((grouped_gemm_f32_kernel<true, true>), grid, block, 0, st, args);
    else if (a_kc) hipLaunchKernelGGL((grouped_gemm_f32_kernel<true, false>), grid, block, 0, st, args);
    else if (b_kc) hipLaunchKernelGGL((grouped_gemm_f32_kernel<false, true>), grid, block, 0, st, args);
    else hipLaunchKernelGGL((grouped_gemm_f32_kernel<false, false>), grid, block, 0, st, args);
    return launch_status("grouped_gemm (fp32)");
}

}  // namespace gemm_f32
}  // namespace fmahip
