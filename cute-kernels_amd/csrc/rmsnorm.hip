// Residual add fused with RMSNorm, forward and backward: HBM-bound row kernels (every element is read once and written
// once; the per-row statistics stay in registers).
//
//   r = x * multiplier + residual            (fp32, stored rounded)
//   inv = 1 / sqrt(mean(r^2) + eps)          (from the unrounded r)
//   out = r * inv * weight                   (one rounding)
//
// One workgroup of 256 threads per row at a time, each thread holding up to VPT 16-byte vectors of the row in
// registers; rows that are longer than that, or whose length in bytes is not a multiple of 16, take a two-pass
// element-wise kernel that reads its inputs twice (the second time from the L2). The backward gives every workgroup a
// contiguous chunk of rows so that it can keep the weight gradient of its chunk in registers across rows; the chunks'
// partial gradients go to a workspace and a second launch adds them up in a fixed order (the reference adds them with
// atomics, in arrival order).
#include "common.h"

namespace fmahip {
namespace {

constexpr int kNormThreads = 256;
constexpr int kNormWaves = kNormThreads / kWave;
// chunks of rows (= rows of the weight-gradient workspace) per compute unit; measured on [16384, 4096] bf16: 1 -> 214 us,
// 2 -> 143 us, 3 -> 151 us, 4 -> 173 us, 8 -> 162 us for both launches
constexpr int kBwdWorkgroupsPerCU = 2;

struct Sum2 {
    float a, b;
};

// Sum over the workgroup of two floats per thread; every thread gets both totals. `slot` is one of two alternating
// LDS areas, so a single barrier per use is enough (the next use writes the other area).
__device__ __forceinline__ Sum2 block_sum2(float a, float b, float (*slot)[2]) {
    a = wave_sum(a);
    b = wave_sum(b);
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    if (lane == 0) {
        slot[wave][0] = a;
        slot[wave][1] = b;
    }
    __syncthreads();
    Sum2 t;
    t.a = (slot[0][0] + slot[1][0]) + (slot[2][0] + slot[3][0]);
    t.b = (slot[0][1] + slot[1][1]) + (slot[2][1] + slot[3][1]);
    return t;
}

// x * multiplier + residual with the product rounded before the addition (no fused multiply-add), so that the residual
// stream has the bits of `x * multiplier + residual` evaluated op by op, as the reference's torch formulation does.
// For short rows the gradient is very sensitive to the last bit of r (H = 1: d_added = g * inv * eps / (r^2 + eps)).
__device__ __forceinline__ float scaled_add(float x, float multiplier, float residual) {
#pragma clang fp contract(off)
    const float scaled = x * multiplier;
    return scaled + residual;
}

__device__ __forceinline__ float inverse_rms(float sum_of_squares, float inv_H, float eps) {
    return 1.0f / sqrtf(sum_of_squares * inv_H + eps);
}

// ---- forward ----------------------------------------------------------------------------------------------------------

template <typename T, int VPT, bool HAS_W>
__global__ __launch_bounds__(kNormThreads) void rmsnorm_fwd_kernel(const Vec16<T>* __restrict__ x,
                                                                   const Vec16<T>* __restrict__ residual,
                                                                   const Vec16<T>* __restrict__ weight,
                                                                   Vec16<T>* __restrict__ out,
                                                                   Vec16<T>* __restrict__ added, float* __restrict__ denom,
                                                                   int64_t B, int nvec, float inv_H, float eps,
                                                                   float multiplier) {
    constexpr int N = Vec16<T>::N;
    __shared__ float s_red[2][kNormWaves][2];
    const int tid = threadIdx.x;
    Vec16<T> wv[VPT];
    if constexpr (HAS_W) {
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int v = tid + i * kNormThreads;
            if (v < nvec) wv[i] = weight[v];
        }
    }
    int parity = 0;
    for (int64_t row = blockIdx.x; row < B; row += gridDim.x, parity ^= 1) {
        const int64_t base = row * nvec;
        Vec16<T> xv[VPT], rv[VPT];
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int v = tid + i * kNormThreads;
            if (v < nvec) {
                xv[i] = load_streaming16(x + base + v);
                rv[i] = load_streaming16(residual + base + v);
            }
        }
        float f[VPT][N];
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int v = tid + i * kNormThreads;
            if (v < nvec) {
                Vec16<T> o;
#pragma unroll
                for (int e = 0; e < N; ++e) {
                    f[i][e] = scaled_add(Num<T>::up(xv[i].v[e]), multiplier, Num<T>::up(rv[i].v[e]));
                    ss += f[i][e] * f[i][e];
                    o.v[e] = Num<T>::down(f[i][e]);
                }
                added[base + v] = o;
            }
        }
        const float inv = inverse_rms(block_sum2(ss, 0.f, s_red[parity]).a, inv_H, eps);
        if (denom && tid == 0) denom[row] = inv;
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int v = tid + i * kNormThreads;
            if (v < nvec) {
                Vec16<T> o;
#pragma unroll
                for (int e = 0; e < N; ++e) {
                    float y = f[i][e] * inv;
                    if constexpr (HAS_W) y *= Num<T>::up(wv[i].v[e]);
                    o.v[e] = Num<T>::down(y);
                }
                out[base + v] = o;
            }
        }
    }
}

// any H, any alignment: element-wise, inputs read twice
template <typename T>
__global__ __launch_bounds__(kNormThreads) void rmsnorm_fwd_generic_kernel(const T* __restrict__ x,
                                                                           const T* __restrict__ residual,
                                                                           const T* __restrict__ weight,
                                                                           T* __restrict__ out, T* __restrict__ added,
                                                                           float* __restrict__ denom, int64_t B, int64_t H,
                                                                           float inv_H, float eps, float multiplier) {
    __shared__ float s_red[2][kNormWaves][2];
    const int tid = threadIdx.x;
    int parity = 0;
    for (int64_t row = blockIdx.x; row < B; row += gridDim.x, parity ^= 1) {
        const int64_t base = row * H;
        float ss = 0.f;
        for (int64_t h = tid; h < H; h += kNormThreads) {
            const float f = scaled_add(Num<T>::up(x[base + h]), multiplier, Num<T>::up(residual[base + h]));
            ss += f * f;
            added[base + h] = Num<T>::down(f);
        }
        const float inv = inverse_rms(block_sum2(ss, 0.f, s_red[parity]).a, inv_H, eps);
        if (denom && tid == 0) denom[row] = inv;
        for (int64_t h = tid; h < H; h += kNormThreads) {
            float y = scaled_add(Num<T>::up(x[base + h]), multiplier, Num<T>::up(residual[base + h])) * inv;
            if (weight) y *= Num<T>::up(weight[h]);
            out[base + h] = Num<T>::down(y);
        }
    }
}

// ---- backward ---------------------------------------------------------------------------------------------------------
// With g = dy * weight:  d_added = inv * g - inv^3 / H * r * <g, r> + d_added_in;  dx = multiplier * d_added;
// d_residual = d_added;  d_weight[h] = sum over rows of dy * round(r * inv).

template <typename T, int VPT, bool HAS_W>
__global__ __launch_bounds__(kNormThreads) void rmsnorm_bwd_kernel(
    const Vec16<T>* __restrict__ added, const Vec16<T>* __restrict__ weight, const Vec16<T>* __restrict__ dy,
    const Vec16<T>* __restrict__ d_added_in, const float* __restrict__ denom, Vec16<T>* __restrict__ dx,
    Vec16<T>* __restrict__ d_residual, float* __restrict__ dw_partial, int64_t B, int64_t rows_per_workgroup, int nvec,
    float inv_H, float eps, float multiplier) {
    constexpr int N = Vec16<T>::N;
    __shared__ float s_red[2][kNormWaves][2];
    const int tid = threadIdx.x;
    Vec16<T> wv[VPT];
    float dw[VPT][N];
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int v = tid + i * kNormThreads;
        if constexpr (HAS_W)
            if (v < nvec) wv[i] = weight[v];
#pragma unroll
        for (int e = 0; e < N; ++e) dw[i][e] = 0.f;
    }
    const int64_t row0 = (int64_t)blockIdx.x * rows_per_workgroup;
    const int64_t row1 = row0 + rows_per_workgroup < B ? row0 + rows_per_workgroup : B;
    // the vectors of the next row are requested before this row is worked on, so that their latency runs under this row's
    // arithmetic, barrier and stores (a workgroup handles its rows one after the other)
    Vec16<T> rv[VPT], gv[VPT], av[VPT];
    auto fetch = [&](Vec16<T> (&r_)[VPT], Vec16<T> (&g_)[VPT], Vec16<T> (&a_)[VPT], int64_t row) {
        const int64_t base = row * nvec;
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int v = tid + i * kNormThreads;
            if (v < nvec) {
                r_[i] = load_streaming16(added + base + v);
                g_[i] = load_streaming16(dy + base + v);
                if (d_added_in) a_[i] = load_streaming16(d_added_in + base + v);
            }
        }
    };
    if (row0 < row1) fetch(rv, gv, av, row0);
    int parity = 0;
    for (int64_t row = row0; row < row1; ++row, parity ^= 1) {
        const int64_t base = row * nvec;
        Vec16<T> rn[VPT], gn[VPT], an[VPT];
        fetch(rn, gn, an, row + 1 < row1 ? row + 1 : row);  // after the last row: this row again, unused
        float dot = 0.f, ss = 0.f;
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int v = tid + i * kNormThreads;
            if (v < nvec) {
#pragma unroll
                for (int e = 0; e < N; ++e) {
                    const float r = Num<T>::up(rv[i].v[e]);
                    float g = Num<T>::up(gv[i].v[e]);
                    if constexpr (HAS_W) g *= Num<T>::up(wv[i].v[e]);
                    dot += g * r;
                    ss += r * r;
                }
            }
        }
        const Sum2 total = block_sum2(dot, ss, s_red[parity]);
        const float inv = denom ? denom[row] : inverse_rms(total.b, inv_H, eps);
        const float c = inv * inv * inv * inv_H * total.a;
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int v = tid + i * kNormThreads;
            if (v < nvec) {
                Vec16<T> o_res, o_x;
#pragma unroll
                for (int e = 0; e < N; ++e) {
                    const float r = Num<T>::up(rv[i].v[e]);
                    const float d = Num<T>::up(gv[i].v[e]);
                    float g = d;
                    if constexpr (HAS_W) g *= Num<T>::up(wv[i].v[e]);
                    float t = inv * g - c * r;
                    if (d_added_in) t += Num<T>::up(av[i].v[e]);
                    o_res.v[e] = Num<T>::down(t);
                    o_x.v[e] = Num<T>::down(t * multiplier);
                    if constexpr (HAS_W) dw[i][e] += d * Num<T>::up(Num<T>::down(r * inv));
                }
                store_streaming16(d_residual + base + v, o_res);
                store_streaming16(dx + base + v, o_x);
            }
        }
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            rv[i] = rn[i];
            gv[i] = gn[i];
            av[i] = an[i];
        }
    }
    if constexpr (HAS_W) {
        float* mine = dw_partial + (int64_t)blockIdx.x * nvec * N;
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int v = tid + i * kNormThreads;
            if (v < nvec) {
#pragma unroll
                for (int e = 0; e < N; ++e) mine[v * N + e] = dw[i][e];
            }
        }
    }
}

template <typename T>
__global__ __launch_bounds__(kNormThreads) void rmsnorm_bwd_generic_kernel(
    const T* __restrict__ added, const T* __restrict__ weight, const T* __restrict__ dy, const T* __restrict__ d_added_in,
    const float* __restrict__ denom, T* __restrict__ dx, T* __restrict__ d_residual, float* __restrict__ dw_partial,
    int64_t B, int64_t rows_per_workgroup, int64_t H, float inv_H, float eps, float multiplier) {
    __shared__ float s_red[2][kNormWaves][2];
    const int tid = threadIdx.x;
    const int64_t row0 = (int64_t)blockIdx.x * rows_per_workgroup;
    const int64_t row1 = row0 + rows_per_workgroup < B ? row0 + rows_per_workgroup : B;
    // this workgroup's row of the workspace; column h is only ever touched by thread h % 256
    float* mine = weight ? dw_partial + (int64_t)blockIdx.x * H : nullptr;
    if (mine)
        for (int64_t h = tid; h < H; h += kNormThreads) mine[h] = 0.f;
    int parity = 0;
    for (int64_t row = row0; row < row1; ++row, parity ^= 1) {
        const int64_t base = row * H;
        float dot = 0.f, ss = 0.f;
        for (int64_t h = tid; h < H; h += kNormThreads) {
            const float r = Num<T>::up(added[base + h]);
            float g = Num<T>::up(dy[base + h]);
            if (weight) g *= Num<T>::up(weight[h]);
            dot += g * r;
            ss += r * r;
        }
        const Sum2 total = block_sum2(dot, ss, s_red[parity]);
        const float inv = denom ? denom[row] : inverse_rms(total.b, inv_H, eps);
        const float c = inv * inv * inv * inv_H * total.a;
        for (int64_t h = tid; h < H; h += kNormThreads) {
            const float r = Num<T>::up(added[base + h]);
            const float d = Num<T>::up(dy[base + h]);
            float g = d;
            if (weight) g *= Num<T>::up(weight[h]);
            float t = inv * g - c * r;
            if (d_added_in) t += Num<T>::up(d_added_in[base + h]);
            d_residual[base + h] = Num<T>::down(t);
            dx[base + h] = Num<T>::down(t * multiplier);
            if (mine) mine[h] += d * Num<T>::up(Num<T>::down(r * inv));
        }
    }
}

// d_weight[h] = sum over the G rows of the workspace. A workgroup owns 32 columns; its 8 groups of 32 threads each add
// every 8th row, in fp64 (so that the long sums add no rounding error of their own), and the 8 results are added in a
// fixed order: the same bits on every run.
constexpr int kReduceCols = 32, kReduceGroups = kNormThreads / kReduceCols;
__global__ __launch_bounds__(kNormThreads) void rmsnorm_dw_reduce_kernel(const float* __restrict__ partial, int64_t G,
                                                                         int64_t H, float* __restrict__ d_weight) {
    __shared__ double s_acc[kReduceGroups][kReduceCols];
    const int col = threadIdx.x % kReduceCols, group = threadIdx.x / kReduceCols;
    const int64_t h = (int64_t)blockIdx.x * kReduceCols + col;
    double acc = 0.0;
    if (h < H) {
        int64_t g = group;
        for (; g + 3 * kReduceGroups < G; g += 4 * kReduceGroups) {
            const float a0 = partial[g * H + h], a1 = partial[(g + kReduceGroups) * H + h];
            const float a2 = partial[(g + 2 * kReduceGroups) * H + h], a3 = partial[(g + 3 * kReduceGroups) * H + h];
            acc += (double)a0;
            acc += (double)a1;
            acc += (double)a2;
            acc += (double)a3;
        }
        for (; g < G; g += kReduceGroups) acc += (double)partial[g * H + h];
    }
    s_acc[group][col] = acc;
    __syncthreads();
    if (group == 0 && h < H) {
        double total = 0.0;
#pragma unroll
        for (int i = 0; i < kReduceGroups; ++i) total += s_acc[i][col];
        d_weight[h] = (float)total;
    }
}

// ---- launch -----------------------------------------------------------------------------------------------------------

// vectors per thread the register kernels need for a row of `row_bytes`, or 0 if the row takes the generic kernel
int vectors_per_thread(int64_t row_bytes, bool all_aligned) {
    if (!all_aligned || row_bytes % 16 != 0) return 0;
    const int64_t nvec = row_bytes / 16;
    for (int vpt = 1; vpt <= 8; vpt *= 2)
        if (nvec <= (int64_t)vpt * kNormThreads) return vpt;
    return 0;
}

int64_t backward_workgroups(int64_t B) {
    const int64_t cus = num_compute_units() > 0 ? num_compute_units() : 256;
    const int64_t want = cus * kBwdWorkgroupsPerCU;
    return B < want ? (B > 0 ? B : 1) : want;
}

template <typename T, int VPT>
void launch_fwd_vec(bool has_w, dim3 grid, hipStream_t st, const void* x, const void* residual, const void* weight,
                    void* out, void* added, float* denom, int64_t B, int nvec, float inv_H, float eps, float mult) {
    using V = Vec16<T>;
    if (has_w)
        hipLaunchKernelGGL((rmsnorm_fwd_kernel<T, VPT, true>), grid, dim3(kNormThreads), 0, st, (const V*)x,
                           (const V*)residual, (const V*)weight, (V*)out, (V*)added, denom, B, nvec, inv_H, eps, mult);
    else
        hipLaunchKernelGGL((rmsnorm_fwd_kernel<T, VPT, false>), grid, dim3(kNormThreads), 0, st, (const V*)x,
                           (const V*)residual, (const V*)weight, (V*)out, (V*)added, denom, B, nvec, inv_H, eps, mult);
}

template <typename T>
int launch_fwd(const void* x, const void* residual, const void* weight, void* out, void* added, float* denom, int64_t B,
               int64_t H, float eps, float mult, hipStream_t st) {
    const bool aligned = aligned16(x) && aligned16(residual) && aligned16(out) && aligned16(added) &&
                         (!weight || aligned16(weight));
    const int vpt = vectors_per_thread(H * (int64_t)sizeof(T), aligned);
    const int64_t cus = num_compute_units() > 0 ? num_compute_units() : 256;
    const dim3 grid((uint32_t)(B < cus * 16 ? B : cus * 16));
    const float inv_H = 1.0f / (float)H;
    const int nvec = (int)(H * (int64_t)sizeof(T) / 16);
    switch (vpt) {
        case 1: launch_fwd_vec<T, 1>(weight, grid, st, x, residual, weight, out, added, denom, B, nvec, inv_H, eps, mult); break;
        case 2: launch_fwd_vec<T, 2>(weight, grid, st, x, residual, weight, out, added, denom, B, nvec, inv_H, eps, mult); break;
        case 4: launch_fwd_vec<T, 4>(weight, grid, st, x, residual, weight, out, added, denom, B, nvec, inv_H, eps, mult); break;
        case 8: launch_fwd_vec<T, 8>(weight, grid, st, x, residual, weight, out, added, denom, B, nvec, inv_H, eps, mult); break;
        default:
            hipLaunchKernelGGL(rmsnorm_fwd_generic_kernel<T>, grid, dim3(kNormThreads), 0, st, (const T*)x,
                               (const T*)residual, (const T*)weight, (T*)out, (T*)added, denom, B, H, inv_H, eps, mult);
    }
    return launch_status("fused_residual_add_rmsnorm_fwd");
}

template <typename T, int VPT>
void launch_bwd_vec(bool has_w, dim3 grid, hipStream_t st, const void* added, const void* weight, const void* dy,
                    const void* d_added_in, const float* denom, void* dx, void* d_residual, float* partial, int64_t B,
                    int64_t rows_per, int nvec, float inv_H, float eps, float mult) {
    using V = Vec16<T>;
    if (has_w)
        hipLaunchKernelGGL((rmsnorm_bwd_kernel<T, VPT, true>), grid, dim3(kNormThreads), 0, st, (const V*)added,
                           (const V*)weight, (const V*)dy, (const V*)d_added_in, denom, (V*)dx, (V*)d_residual, partial, B,
                           rows_per, nvec, inv_H, eps, mult);
    else
        hipLaunchKernelGGL((rmsnorm_bwd_kernel<T, VPT, false>), grid, dim3(kNormThreads), 0, st, (const V*)added,
                           (const V*)weight, (const V*)dy, (const V*)d_added_in, denom, (V*)dx, (V*)d_residual, partial, B,
                           rows_per, nvec, inv_H, eps, mult);
}

template <typename T>
int launch_bwd(const void* added, const void* weight, const void* dy, const void* d_added_in, const float* denom, void* dx,
               void* d_residual, float* d_weight, float* partial, int64_t G, int64_t B, int64_t H, float eps, float mult,
               hipStream_t st) {
    const bool aligned = aligned16(added) && aligned16(dy) && aligned16(dx) && aligned16(d_residual) &&
                         (!weight || aligned16(weight)) && (!d_added_in || aligned16(d_added_in));
    const int vpt = vectors_per_thread(H * (int64_t)sizeof(T), aligned);
    const int64_t rows_per = (B + G - 1) / G;
    const dim3 grid((uint32_t)G);
    const float inv_H = 1.0f / (float)H;
    const int nvec = (int)(H * (int64_t)sizeof(T) / 16);
    switch (vpt) {
        case 1: launch_bwd_vec<T, 1>(weight, grid, st, added, weight, dy, d_added_in, denom, dx, d_residual, partial, B, rows_per, nvec, inv_H, eps, mult); break;
        case 2: launch_bwd_vec<T, 2>(weight, grid, st, added, weight, dy, d_added_in, denom, dx, d_residual, partial, B, rows_per, nvec, inv_H, eps, mult); break;
        case 4: launch_bwd_vec<T, 4>(weight, grid, st, added, weight, dy, d_added_in, denom, dx, d_residual, partial, B, rows_per, nvec, inv_H, eps, mult); break;
        case 8: launch_bwd_vec<T, 8>(weight, grid, st, added, weight, dy, d_added_in, denom, dx, d_residual, partial, B, rows_per, nvec, inv_H, eps, mult); break;
        default:
            hipLaunchKernelGGL(rmsnorm_bwd_generic_kernel<T>, grid, dim3(kNormThreads), 0, st, (const T*)added,
                               (const T*)weight, (const T*)dy, (const T*)d_added_in, denom, (T*)dx, (T*)d_residual, partial,
                               B, rows_per, H, inv_H, eps, mult);
    }
    int rc = launch_status("fused_residual_add_rmsnorm_bwd");
    if (rc || !weight) return rc;
    hipLaunchKernelGGL(rmsnorm_dw_reduce_kernel, dim3((uint32_t)((H + kReduceCols - 1) / kReduceCols)),
                       dim3(kNormThreads), 0, st, (const float*)partial, G, H, d_weight);
    return launch_status("fused_residual_add_rmsnorm_bwd (weight gradient)");
}

int check_norm(const char* what, int dtype, int64_t B, int64_t H) {
    FMA_REQUIRE(dtype_bytes(dtype) != 0, FMA_ERR_BAD_DTYPE, "%s: unknown dtype code %d", what, dtype);
    FMA_REQUIRE(B >= 0 && B <= 0x7fffffffll, FMA_ERR_BAD_SIZE, "%s: bad row count %lld", what, (long long)B);
    FMA_REQUIRE(H >= 1 && H <= FMA_MAX_NORM_HIDDEN, FMA_ERR_BAD_SIZE, "%s: H must be in [1, %d] (got %lld)", what,
                FMA_MAX_NORM_HIDDEN, (long long)H);
    return FMA_OK;
}

}  // namespace
}  // namespace fmahip

extern "C" {

int fma_fused_residual_add_rmsnorm_fwd(const void* x, const void* residual, const void* weight, void* output,
                                       void* added_x_residual, float* rmsnorm_denominator, int64_t B, int64_t H,
                                       float eps, float multiplier, int dtype, void* stream) {
    using namespace fmahip;
    int rc = check_norm("fused_residual_add_rmsnorm_fwd", dtype, B, H);
    if (rc) return rc;
    if (B == 0) return FMA_OK;
    FMA_REQUIRE(x && residual && output && added_x_residual, FMA_ERR_NULL_POINTER,
                "fused_residual_add_rmsnorm_fwd: NULL pointer");
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case FMA_F32:
            return launch_fwd<float>(x, residual, weight, output, added_x_residual, rmsnorm_denominator, B, H, eps,
                                     multiplier, st);
        case FMA_F16:
            return launch_fwd<f16_t>(x, residual, weight, output, added_x_residual, rmsnorm_denominator, B, H, eps,
                                     multiplier, st);
        default:
            return launch_fwd<bf16_t>(x, residual, weight, output, added_x_residual, rmsnorm_denominator, B, H, eps,
                                      multiplier, st);
    }
}

int64_t fma_fused_residual_add_rmsnorm_bwd_workspace_bytes(int64_t B, int64_t H) {
    if (B <= 0 || H <= 0) return 0;
    return fmahip::backward_workgroups(B) * H * 4;
}

int fma_fused_residual_add_rmsnorm_bwd(const void* added_x_residual, const void* weight, const void* output_grad,
                                       const void* added_x_residual_grad, const float* rmsnorm_denominator, void* x_grad,
                                       void* residual_grad, float* weight_grad, int64_t B, int64_t H, float eps,
                                       float multiplier, void* workspace, int64_t workspace_bytes, int dtype,
                                       void* stream) {
    using namespace fmahip;
    int rc = check_norm("fused_residual_add_rmsnorm_bwd", dtype, B, H);
    if (rc) return rc;
    FMA_REQUIRE((weight == nullptr) == (weight_grad == nullptr), FMA_ERR_NULL_POINTER,
                "fused_residual_add_rmsnorm_bwd: weight and weight_grad must be given together");
    hipStream_t st = (hipStream_t)stream;
    if (B == 0) {
        if (weight_grad) {  // no rows: the gradient is zero
            hipLaunchKernelGGL(rmsnorm_dw_reduce_kernel, dim3((uint32_t)((H + kReduceCols - 1) / kReduceCols)),
                               dim3(kNormThreads), 0, st, (const float*)nullptr, (int64_t)0, H, weight_grad);
            return launch_status("fused_residual_add_rmsnorm_bwd (weight gradient)");
        }
        return FMA_OK;
    }
    FMA_REQUIRE(added_x_residual && output_grad && x_grad && residual_grad, FMA_ERR_NULL_POINTER,
                "fused_residual_add_rmsnorm_bwd: NULL pointer");
    int64_t G = backward_workgroups(B);
    if (weight) {
        FMA_REQUIRE(workspace != nullptr, FMA_ERR_NULL_POINTER, "fused_residual_add_rmsnorm_bwd: NULL workspace");
        FMA_REQUIRE(workspace_bytes >= G * H * 4, FMA_ERR_WORKSPACE_TOO_SMALL,
                    "fused_residual_add_rmsnorm_bwd: workspace of %lld bytes, %lld needed", (long long)workspace_bytes,
                    (long long)(G * H * 4));
        FMA_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 3u) == 0, FMA_ERR_MISALIGNED,
                    "fused_residual_add_rmsnorm_bwd: workspace must be 4-byte aligned");
    }
    float* partial = (float*)workspace;
    switch (dtype) {
        case FMA_F32:
            return launch_bwd<float>(added_x_residual, weight, output_grad, added_x_residual_grad, rmsnorm_denominator,
                                     x_grad, residual_grad, weight_grad, partial, G, B, H, eps, multiplier, st);
        case FMA_F16:
            return launch_bwd<f16_t>(added_x_residual, weight, output_grad, added_x_residual_grad, rmsnorm_denominator,
                                     x_grad, residual_grad, weight_grad, partial, G, B, H, eps, multiplier, st);
        default:
            return launch_bwd<bf16_t>(added_x_residual, weight, output_grad, added_x_residual_grad,
                                      rmsnorm_denominator, x_grad, residual_grad, weight_grad, partial, G, B, H, eps,
                                      multiplier, st);
    }
}

}  // extern "C"
