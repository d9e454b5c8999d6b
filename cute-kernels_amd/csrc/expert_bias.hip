// Per-expert bias of the grouped linear layers: y[i, :] += bias[e(i), :] over rows packed expert by expert, and its
// gradient d_bias[e, :] = sum of the rows of expert e. Both are HBM-bound passes over a [R, N] tensor.
//
// Work is cut as (column block, slice): a slice is up to kSliceRows consecutive rows of ONE expert (expert e has
// ceil(M_e / kSliceRows) of them, so a skewed routing still gives evenly sized pieces), and a workgroup owns 256 16-byte
// column vectors of one slice: the bias vector (or the running sum) of its columns stays in registers while the rows
// stream by. Group sizes live on the device, so the launch covers the upper bound ceil(R / kSliceRows) + E slices and
// every workgroup walks the group sizes to find its expert (or that it has none). The gradient's per-slice sums go to a
// workspace and a second launch adds each expert's slices in order (fixed order: the same bits on every run).
#include "common.h"

namespace fmahip {
namespace {

constexpr int kBiasThreads = 256;
constexpr int kSliceRows = 256;

// the expert that slice z belongs to and its rows [begin, end); false if z is past the last slice
__device__ __forceinline__ bool find_slice(const uint32_t* __restrict__ M_arr, uint32_t E, uint32_t z, uint32_t& expert,
                                           int64_t& begin, int64_t& end) {
    uint32_t slices = 0;
    int64_t first = 0;
    for (uint32_t e = 0; e < E; ++e) {
        const uint32_t rows = M_arr[e];
        const uint32_t n = (rows + kSliceRows - 1) / kSliceRows;
        if (z < slices + n) {
            expert = e;
            begin = first + (int64_t)(z - slices) * kSliceRows;
            end = begin + kSliceRows < first + rows ? begin + kSliceRows : first + rows;
            return true;
        }
        slices += n;
        first += rows;
    }
    return false;
}

template <typename T>
__global__ __launch_bounds__(kBiasThreads) void expert_bias_add_kernel(Vec16<T>* __restrict__ y,
                                                                       const Vec16<T>* __restrict__ bias,
                                                                       const uint32_t* __restrict__ M_arr, uint32_t E,
                                                                       int64_t R, int nvec) {
    constexpr int N = Vec16<T>::N;
    const int v = blockIdx.y * kBiasThreads + threadIdx.x;
    uint32_t expert;
    int64_t begin, end;
    if (!find_slice(M_arr, E, blockIdx.x, expert, begin, end)) return;
    if (end > R) end = R;  // group sizes that overrun the buffer must not become wild accesses
    if (v >= nvec) return;
    const Vec16<T> b = bias[(int64_t)expert * nvec + v];
    float bf[N];
#pragma unroll
    for (int e = 0; e < N; ++e) bf[e] = Num<T>::up(b.v[e]);
    int64_t row = begin;
    for (; row + 3 < end; row += 4) {  // four rows in flight
        Vec16<T> a[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) a[u] = y[(row + u) * nvec + v];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
#pragma unroll
            for (int e = 0; e < N; ++e) a[u].v[e] = Num<T>::down(Num<T>::up(a[u].v[e]) + bf[e]);
            y[(row + u) * nvec + v] = a[u];
        }
    }
    for (; row < end; ++row) {
        Vec16<T> a0 = y[row * nvec + v];
#pragma unroll
        for (int e = 0; e < N; ++e) a0.v[e] = Num<T>::down(Num<T>::up(a0.v[e]) + bf[e]);
        y[row * nvec + v] = a0;
    }
}

// partial[z * N_elems + column] = sum over the rows of slice z, in row order
template <typename T>
__global__ __launch_bounds__(kBiasThreads) void expert_bias_grad_kernel(const Vec16<T>* __restrict__ dy,
                                                                        const uint32_t* __restrict__ M_arr, uint32_t E,
                                                                        int64_t R, int nvec, float* __restrict__ partial) {
    constexpr int N = Vec16<T>::N;
    const int v = blockIdx.y * kBiasThreads + threadIdx.x;
    uint32_t expert;
    int64_t begin, end;
    if (!find_slice(M_arr, E, blockIdx.x, expert, begin, end)) return;
    if (end > R) end = R;
    if (v >= nvec) return;
    float acc[N];
#pragma unroll
    for (int e = 0; e < N; ++e) acc[e] = 0.f;
    int64_t row = begin;
    for (; row + 3 < end; row += 4) {  // four rows in flight, added in row order
        Vec16<T> a[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) a[u] = load_streaming16(dy + (row + u) * nvec + v);
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int e = 0; e < N; ++e) acc[e] += Num<T>::up(a[u].v[e]);
    }
    for (; row < end; ++row) {
        const Vec16<T> a = load_streaming16(dy + row * nvec + v);
#pragma unroll
        for (int e = 0; e < N; ++e) acc[e] += Num<T>::up(a.v[e]);
    }
    float* mine = partial + ((int64_t)blockIdx.x * nvec + v) * N;
#pragma unroll
    for (int e = 0; e < N; ++e) mine[e] = acc[e];
}

// d_bias[e, n] = sum of expert e's slices in order, in fp64, rounded once to the output type (zero without rows)
template <typename T>
__global__ __launch_bounds__(kBiasThreads) void expert_bias_grad_reduce_kernel(const float* __restrict__ partial,
                                                                               const uint32_t* __restrict__ M_arr,
                                                                               int64_t N_elems, T* __restrict__ d_bias) {
    const int64_t n = (int64_t)blockIdx.x * kBiasThreads + threadIdx.x;
    const uint32_t expert = blockIdx.y;
    if (n >= N_elems) return;
    int64_t z0 = 0;
    for (uint32_t e = 0; e < expert; ++e) z0 += (M_arr[e] + kSliceRows - 1) / kSliceRows;
    const int64_t count = (M_arr[expert] + kSliceRows - 1) / kSliceRows;
    double acc = 0.0;
    for (int64_t z = z0; z < z0 + count; ++z) acc += (double)partial[z * N_elems + n];
    d_bias[(int64_t)expert * N_elems + n] = Num<T>::down((float)acc);
}

// upper bound on the number of slices that needs no look at the device-side group sizes
int64_t max_slices(int64_t E, int64_t R) { return (R + kSliceRows - 1) / kSliceRows + E; }

int check_bias(const char* what, int dtype, int64_t E, int64_t R, int64_t N) {
    FMA_REQUIRE(dtype_bytes(dtype) != 0, FMA_ERR_BAD_DTYPE, "%s: unknown dtype code %d", what, dtype);
    FMA_REQUIRE(E >= 1 && E <= FMA_MAX_GROUPS, FMA_ERR_TOO_MANY_EXPERTS, "%s: E must be in [1, %d] (got %lld)", what,
                FMA_MAX_GROUPS, (long long)E);
    FMA_REQUIRE(R >= 0 && R <= 0x7fffffffll, FMA_ERR_BAD_SIZE, "%s: bad row count %lld", what, (long long)R);
    FMA_REQUIRE(N >= 1 && N * dtype_bytes(dtype) % 16 == 0 && N <= (1ll << 24), FMA_ERR_BAD_SIZE,
                "%s: a row of N = %lld elements must be a multiple of 16 bytes", what, (long long)N);
    return FMA_OK;
}

}  // namespace
}  // namespace fmahip

extern "C" {

int fma_expert_bias_add(void* y, const void* bias, const uint32_t* M_arr, int64_t E, int64_t R, int64_t N, int dtype,
                        void* stream) {
    using namespace fmahip;
    int rc = check_bias("expert_bias_add", dtype, E, R, N);
    if (rc) return rc;
    if (R == 0) return FMA_OK;
    FMA_REQUIRE(y && bias && M_arr, FMA_ERR_NULL_POINTER, "expert_bias_add: NULL pointer");
    FMA_REQUIRE(aligned16(y) && aligned16(bias), FMA_ERR_MISALIGNED, "expert_bias_add: y and bias must be 16-byte aligned");
    const int nvec = (int)(N * dtype_bytes(dtype) / 16);
    const dim3 grid((uint32_t)max_slices(E, R), (uint32_t)((nvec + kBiasThreads - 1) / kBiasThreads));
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case FMA_F32:
            hipLaunchKernelGGL(expert_bias_add_kernel<float>, grid, dim3(kBiasThreads), 0, st, (Vec16<float>*)y,
                               (const Vec16<float>*)bias, M_arr, (uint32_t)E, R, nvec);
            break;
        case FMA_F16:
            hipLaunchKernelGGL(expert_bias_add_kernel<f16_t>, grid, dim3(kBiasThreads), 0, st, (Vec16<f16_t>*)y,
                               (const Vec16<f16_t>*)bias, M_arr, (uint32_t)E, R, nvec);
            break;
        default:
            hipLaunchKernelGGL(expert_bias_add_kernel<bf16_t>, grid, dim3(kBiasThreads), 0, st, (Vec16<bf16_t>*)y,
                               (const Vec16<bf16_t>*)bias, M_arr, (uint32_t)E, R, nvec);
    }
    return launch_status("expert_bias_add");
}

int64_t fma_expert_bias_grad_workspace_bytes(int64_t E, int64_t R, int64_t N) {
    if (E <= 0 || N <= 0 || R < 0) return 0;
    return fmahip::max_slices(E, R) * N * 4;
}

int fma_expert_bias_grad(const void* dy, const uint32_t* M_arr, int64_t E, int64_t R, int64_t N, void* d_bias,
                         void* workspace, int64_t workspace_bytes, int dtype, void* stream) {
    using namespace fmahip;
    int rc = check_bias("expert_bias_grad", dtype, E, R, N);
    if (rc) return rc;
    FMA_REQUIRE(d_bias && M_arr && workspace && (dy || R == 0), FMA_ERR_NULL_POINTER, "expert_bias_grad: NULL pointer");
    FMA_REQUIRE(aligned16(dy) && (reinterpret_cast<uintptr_t>(workspace) & 3u) == 0, FMA_ERR_MISALIGNED,
                "expert_bias_grad: dy must be 16-byte aligned, the workspace 4-byte aligned");
    const int nvec = (int)(N * dtype_bytes(dtype) / 16);
    const int64_t slices = max_slices(E, R);
    FMA_REQUIRE(workspace_bytes >= slices * N * 4, FMA_ERR_WORKSPACE_TOO_SMALL,
                "expert_bias_grad: workspace of %lld bytes, %lld needed", (long long)workspace_bytes,
                (long long)(slices * N * 4));
    const dim3 grid((uint32_t)slices, (uint32_t)((nvec + kBiasThreads - 1) / kBiasThreads));
    const dim3 rgrid((uint32_t)((N + kBiasThreads - 1) / kBiasThreads), (uint32_t)E);
    hipStream_t st = (hipStream_t)stream;
    float* partial = (float*)workspace;
    switch (dtype) {
        case FMA_F32:
            hipLaunchKernelGGL(expert_bias_grad_kernel<float>, grid, dim3(kBiasThreads), 0, st, (const Vec16<float>*)dy,
                               M_arr, (uint32_t)E, R, nvec, partial);
            hipLaunchKernelGGL(expert_bias_grad_reduce_kernel<float>, rgrid, dim3(kBiasThreads), 0, st,
                               (const float*)partial, M_arr, N, (float*)d_bias);
            break;
        case FMA_F16:
            hipLaunchKernelGGL(expert_bias_grad_kernel<f16_t>, grid, dim3(kBiasThreads), 0, st, (const Vec16<f16_t>*)dy,
                               M_arr, (uint32_t)E, R, nvec, partial);
            hipLaunchKernelGGL(expert_bias_grad_reduce_kernel<f16_t>, rgrid, dim3(kBiasThreads), 0, st,
                               (const float*)partial, M_arr, N, (f16_t*)d_bias);
            break;
        default:
            hipLaunchKernelGGL(expert_bias_grad_kernel<bf16_t>, grid, dim3(kBiasThreads), 0, st,
                               (const Vec16<bf16_t>*)dy, M_arr, (uint32_t)E, R, nvec, partial);
            hipLaunchKernelGGL(expert_bias_grad_reduce_kernel<bf16_t>, rgrid, dim3(kBiasThreads), 0, st,
                               (const float*)partial, M_arr, N, (bf16_t*)d_bias);
    }
    return launch_status("expert_bias_grad");
}

}  // extern "C"
