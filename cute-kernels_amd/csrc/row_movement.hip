// Row gather, router-weighted combine and the combine's backward: HBM-bound kernels that move whole rows of H
// elements with 16-byte lanes. One wavefront reads/writes 1 KB of a row per instruction, so every access is a
// full-line burst no matter how the row indices are scattered.
// Rows that are not a whole number of 16-byte pieces (or buffers that are not 16-byte aligned) run the same kernels with
// one element as the unit: correct for any H, at a fraction of the bandwidth.
#include <initializer_list>

#include "common.h"

namespace fmahip {
namespace {

constexpr int kRowThreads = 256;
// rows per workgroup in the gather, tokens per workgroup in the dispatch: one each. Small one-shot workgroups stream
// best on this part (dispatch at 4 / 2 / 1 tokens per workgroup: 92 / 87 / 74 us; gather at 4 / 2 / 1 rows: 81 / 80 / 79 us)
constexpr int kGatherRows = 1;

// One element standing in for a 16-byte vector.
template <typename T>
struct Vec1 {
    static constexpr int N = 1;
    T v[1];
};
// streaming (non-temporal) access for 16-byte units, plain access for single elements
template <typename U>
__device__ __forceinline__ U load_unit(const U* p) {
    if constexpr (sizeof(U) == 16) return load_streaming16(p);
    else return *p;
}
template <typename U>
__device__ __forceinline__ void store_unit(U* p, const U& v) {
    if constexpr (sizeof(U) == 16) store_streaming16(p, v);
    else *p = v;
}

// out[i] = x[idx[i] / divisor], rows of `vecs` units (16-byte vectors, or single elements of 2 or 4 bytes)
template <typename U>
__global__ __launch_bounds__(kRowThreads) void gather_rows_kernel(const U* __restrict__ x,
                                                                  const int32_t* __restrict__ idx, int64_t R,
                                                                  int64_t vecs, int32_t divisor,
                                                                  U* __restrict__ out) {
    const int64_t i0 = (int64_t)blockIdx.x * kGatherRows;
    const U* src[kGatherRows];
#pragma unroll
    for (int r = 0; r < kGatherRows; ++r) {
        const int64_t i = i0 + r < R ? i0 + r : R - 1;
        src[r] = x + (int64_t)(idx[i] / divisor) * vecs;
    }
    for (int64_t v = threadIdx.x; v < vecs; v += kRowThreads) {
        U t[kGatherRows];
#pragma unroll
        for (int r = 0; r < kGatherRows; ++r) t[r] = src[r][v];  // plain loads: a row is fetched once per expert choice
#pragma unroll
        for (int r = 0; r < kGatherRows; ++r) {
            if (i0 + r < R) store_unit(out + (i0 + r) * vecs + v, t[r]);
        }
    }
}

// out[inv[t*k + j]] = x[t] for j < k: the same gather written from the token's side, so that every input row is
// fetched once however many experts it is routed to
constexpr int kDispatchTokens = 1;
template <typename U>
__global__ __launch_bounds__(kRowThreads) void dispatch_rows_kernel(const U* __restrict__ x,
                                                                    const int32_t* __restrict__ inv, int64_t T,
                                                                    int64_t k, int64_t vecs, U* __restrict__ out) {
    const int64_t t0 = (int64_t)blockIdx.x * kDispatchTokens;
    for (int64_t v = threadIdx.x; v < vecs; v += kRowThreads) {
        U row[kDispatchTokens];
#pragma unroll
        for (int u = 0; u < kDispatchTokens; ++u) row[u] = load_unit(x + (t0 + u < T ? t0 + u : T - 1) * vecs + v);
#pragma unroll
        for (int u = 0; u < kDispatchTokens; ++u) {
            if (t0 + u < T) {
                const int32_t* dst = inv + (t0 + u) * k;
                for (int64_t j = 0; j < k; ++j) store_unit(out + (int64_t)dst[j] * vecs + v, row[u]);
            }
        }
    }
}

// y[t] = sum_j gates[t,j] * o[inv[t,j]]; one workgroup per token, fp32 accumulation in ascending j.
// KC > 0: top_k known at compile time. All KC row loads of a vector position (of two positions per thread for KC <= 4)
// are issued before the first multiply, as streaming loads: the expert rows are read exactly once.
template <typename T, typename V, int KC>
__global__ __launch_bounds__(kRowThreads) void combine_kernel(const V* __restrict__ o,
                                                              const int32_t* __restrict__ inv,
                                                              const T* __restrict__ gates, int64_t k, int64_t vecs,
                                                              V* __restrict__ y) {
    constexpr int N = V::N;
    const int64_t t = blockIdx.x;
    const int32_t* my_inv = inv + t * k;
    const T* my_gates = gates ? gates + t * k : nullptr;
    if constexpr (KC > 0) {
        constexpr int VU = KC <= 4 ? 2 : 1;  // vector positions in flight per thread
        const V* rows[KC];
        float g[KC];
#pragma unroll
        for (int j = 0; j < KC; ++j) {
            rows[j] = o + (int64_t)my_inv[j] * vecs;
            g[j] = my_gates ? Num<T>::up(my_gates[j]) : 1.0f;
        }
        for (int64_t v0 = threadIdx.x; v0 < vecs; v0 += (int64_t)VU * kRowThreads) {
            V r[VU][KC];
#pragma unroll
            for (int u = 0; u < VU; ++u) {
                const int64_t v = v0 + (int64_t)u * kRowThreads;
                const int64_t vc = v < vecs ? v : v0;
#pragma unroll
                for (int j = 0; j < KC; ++j) r[u][j] = load_unit(rows[j] + vc);
            }
#pragma unroll
            for (int u = 0; u < VU; ++u) {
                const int64_t v = v0 + (int64_t)u * kRowThreads;
                if (v < vecs) {
                    float acc[N];
#pragma unroll
                    for (int c = 0; c < N; ++c) acc[c] = 0.0f;
#pragma unroll
                    for (int j = 0; j < KC; ++j)
#pragma unroll
                        for (int c = 0; c < N; ++c) acc[c] = fmaf(g[j], Num<T>::up(r[u][j].v[c]), acc[c]);
                    V w;
#pragma unroll
                    for (int c = 0; c < N; ++c) w.v[c] = Num<T>::down(acc[c]);
                    store_unit(y + t * vecs + v, w);
                }
            }
        }
    } else {
        for (int64_t v = threadIdx.x; v < vecs; v += kRowThreads) {
            float acc[N];
#pragma unroll
            for (int c = 0; c < N; ++c) acc[c] = 0.0f;
            int64_t j = 0;
            for (; j + 4 <= k; j += 4) {
                V r[4];
                float g[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    r[u] = load_unit(o + (int64_t)my_inv[j + u] * vecs + v);
                    g[u] = my_gates ? Num<T>::up(my_gates[j + u]) : 1.0f;
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
#pragma unroll
                    for (int c = 0; c < N; ++c) acc[c] = fmaf(g[u], Num<T>::up(r[u].v[c]), acc[c]);
                }
            }
            for (; j < k; ++j) {
                const V r = load_unit(o + (int64_t)my_inv[j] * vecs + v);
                const float g = my_gates ? Num<T>::up(my_gates[j]) : 1.0f;
#pragma unroll
                for (int c = 0; c < N; ++c) acc[c] = fmaf(g, Num<T>::up(r.v[c]), acc[c]);
            }
            V w;
#pragma unroll
            for (int c = 0; c < N; ++c) w.v[c] = Num<T>::down(acc[c]);
            store_unit(y + t * vecs + v, w);
        }
    }
}

// d_o[inv[t,j]] = gates[t,j] * dy[t];  d_gates[t,j] = <dy[t], o[inv[t,j]]>
// One workgroup per token. dy[t] is read once and kept in registers (up to kBwdVecs units per thread, i.e. rows of
// up to 4096 bf16 in 16-byte vectors); longer rows fall back to re-reading it per expert choice.
constexpr int kBwdVecs = 2;
template <typename T, typename V, bool CACHED>
__global__ __launch_bounds__(kRowThreads) void combine_bwd_kernel(const V* __restrict__ dy,
                                                                  const V* __restrict__ o,
                                                                  const int32_t* __restrict__ inv,
                                                                  const T* __restrict__ gates, int64_t k, int64_t vecs,
                                                                  V* __restrict__ d_o, T* __restrict__ d_gates) {
    constexpr int N = V::N;
    constexpr int NW = kRowThreads / kWave;
    __shared__ float s_part[NW];
    const int64_t t = blockIdx.x;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    V d_reg[kBwdVecs];
    if constexpr (CACHED) {
#pragma unroll
        for (int u = 0; u < kBwdVecs; ++u) {
            const int64_t v = threadIdx.x + (int64_t)u * kRowThreads;
            if (v < vecs) d_reg[u] = dy[t * vecs + v];
        }
    }
    for (int64_t j = 0; j < k; ++j) {
        const int64_t row = inv[t * k + j];
        const float g = gates ? Num<T>::up(gates[t * k + j]) : 1.0f;
        float dot = 0.0f;
        auto one = [&](int64_t v, const V& d) {
            V w;
            if (d_gates) {
                const V ov = load_unit(o + row * vecs + v);
#pragma unroll
                for (int c = 0; c < N; ++c) dot = fmaf(Num<T>::up(d.v[c]), Num<T>::up(ov.v[c]), dot);
            }
#pragma unroll
            for (int c = 0; c < N; ++c) w.v[c] = Num<T>::down(g * Num<T>::up(d.v[c]));
            store_unit(d_o + row * vecs + v, w);
        };
        if constexpr (CACHED) {
#pragma unroll
            for (int u = 0; u < kBwdVecs; ++u) {
                const int64_t v = threadIdx.x + (int64_t)u * kRowThreads;
                if (v < vecs) one(v, d_reg[u]);
            }
        } else {
            for (int64_t v = threadIdx.x; v < vecs; v += kRowThreads) one(v, dy[t * vecs + v]);
        }
        if (d_gates) {
            dot = wave_sum(dot);
            if (lane == 0) s_part[wave] = dot;
            __syncthreads();
            if (threadIdx.x == 0) {
                float sum = 0.0f;
#pragma unroll
                for (int w = 0; w < NW; ++w) sum += s_part[w];
                d_gates[t * k + j] = Num<T>::down(sum);
            }
            __syncthreads();
        }
    }
}

template <typename T, typename V>
int launch_combine(const void* o, const int32_t* inv, const void* gates, int64_t T_, int64_t k, int64_t H, void* y,
                   hipStream_t st) {
    const int64_t vecs = H / V::N;
#define FMA_COMBINE_CASE(KC)                                                                                     \
    case KC:                                                                                                     \
        hipLaunchKernelGGL((combine_kernel<T, V, KC>), dim3((uint32_t)T_), dim3(kRowThreads), 0, st, (const V*)o, inv, \
                           (const T*)gates, k, vecs, (V*)y);                                                     \
        break;
    switch (sizeof(V) == 16 ? k : 0) {  // the element-wise form keeps the generic loop
        FMA_COMBINE_CASE(1)
        FMA_COMBINE_CASE(2)
        FMA_COMBINE_CASE(3)
        FMA_COMBINE_CASE(4)
        FMA_COMBINE_CASE(6)
        FMA_COMBINE_CASE(8)
        default:
            hipLaunchKernelGGL((combine_kernel<T, V, 0>), dim3((uint32_t)T_), dim3(kRowThreads), 0, st, (const V*)o, inv,
                               (const T*)gates, k, vecs, (V*)y);
    }
#undef FMA_COMBINE_CASE
    return launch_status("combine");
}

template <typename T, typename V>
int launch_combine_bwd(const void* dy, const void* o, const int32_t* inv, const void* gates, int64_t T_, int64_t k,
                       int64_t H, void* d_o, void* d_gates, hipStream_t st) {
    const int64_t vecs = H / V::N;
    if (vecs <= (int64_t)kBwdVecs * kRowThreads)
        hipLaunchKernelGGL((combine_bwd_kernel<T, V, true>), dim3((uint32_t)T_), dim3(kRowThreads), 0, st, (const V*)dy,
                           (const V*)o, inv, (const T*)gates, k, vecs, (V*)d_o, (T*)d_gates);
    else
        hipLaunchKernelGGL((combine_bwd_kernel<T, V, false>), dim3((uint32_t)T_), dim3(kRowThreads), 0, st, (const V*)dy,
                           (const V*)o, inv, (const T*)gates, k, vecs, (V*)d_o, (T*)d_gates);
    return launch_status("combine_bwd");
}

int check_rows(const char* who, int dtype, int64_t H) {
    const int eb = dtype_bytes(dtype);
    FMA_REQUIRE(eb != 0, FMA_ERR_BAD_DTYPE, "%s: unknown dtype code %d", who, dtype);
    FMA_REQUIRE(H > 0, FMA_ERR_BAD_SIZE, "%s: bad row length %lld", who, (long long)H);
    return FMA_OK;
}

// 16-byte units when every row starts and ends on a 16-byte boundary, single elements otherwise
bool rows_vectorise(int dtype, int64_t H, std::initializer_list<const void*> buffers) {
    if ((H * dtype_bytes(dtype)) % 16 != 0) return false;
    for (const void* p : buffers)
        if (p && !aligned16(p)) return false;
    return true;
}
bool element_aligned(int dtype, std::initializer_list<const void*> buffers) {
    for (const void* p : buffers)
        if (p && reinterpret_cast<uintptr_t>(p) % (uintptr_t)dtype_bytes(dtype) != 0) return false;
    return true;
}

template <typename U>
int launch_gather(const void* x, const int32_t* idx, int64_t R, int64_t units, int32_t divisor, void* out, hipStream_t st) {
    const uint32_t blocks = (uint32_t)((R + kGatherRows - 1) / kGatherRows);
    hipLaunchKernelGGL(gather_rows_kernel<U>, dim3(blocks), dim3(kRowThreads), 0, st, (const U*)x, idx, R, units, divisor,
                       (U*)out);
    return launch_status("gather_rows");
}
template <typename U>
int launch_dispatch(const void* x, const int32_t* inv, int64_t T, int64_t k, int64_t units, void* out, hipStream_t st) {
    const uint32_t blocks = (uint32_t)((T + kDispatchTokens - 1) / kDispatchTokens);
    hipLaunchKernelGGL(dispatch_rows_kernel<U>, dim3(blocks), dim3(kRowThreads), 0, st, (const U*)x, inv, T, k, units,
                       (U*)out);
    return launch_status("dispatch_rows");
}

}  // namespace
}  // namespace fmahip

extern "C" {

int fma_gather_rows(const void* x, const int32_t* idx, int64_t R, int64_t H, int32_t divisor, void* out, int dtype,
                    void* stream) {
    using namespace fmahip;
    int rc = check_rows("gather_rows", dtype, H);
    if (rc) return rc;
    FMA_REQUIRE(R >= 0 && R <= 0x7fffffffll, FMA_ERR_BAD_SIZE, "gather_rows: bad row count %lld", (long long)R);
    FMA_REQUIRE(divisor >= 1, FMA_ERR_BAD_SIZE, "gather_rows: divisor must be >= 1 (got %d)", divisor);
    if (R == 0) return FMA_OK;
    FMA_REQUIRE(x && idx && out, FMA_ERR_NULL_POINTER, "gather_rows: NULL pointer");
    FMA_REQUIRE(element_aligned(dtype, {x, out}), FMA_ERR_MISALIGNED, "gather_rows: x/out not aligned to the element size");
    hipStream_t st = (hipStream_t)stream;
    if (rows_vectorise(dtype, H, {x, out})) return launch_gather<uint4>(x, idx, R, H * dtype_bytes(dtype) / 16, divisor, out, st);
    if (dtype_bytes(dtype) == 4) return launch_gather<uint32_t>(x, idx, R, H, divisor, out, st);
    return launch_gather<uint16_t>(x, idx, R, H, divisor, out, st);
}

int fma_dispatch_rows(const void* x, const int32_t* inv, int64_t T, int64_t k, int64_t H, void* out, int dtype,
                      void* stream) {
    using namespace fmahip;
    int rc = check_rows("dispatch_rows", dtype, H);
    if (rc) return rc;
    FMA_REQUIRE(T >= 0 && T <= 0x7fffffffll, FMA_ERR_BAD_SIZE, "dispatch_rows: bad token count %lld", (long long)T);
    FMA_REQUIRE(k >= 1 && T * k <= 0x7fffffffll, FMA_ERR_BAD_SIZE, "dispatch_rows: bad top_k %lld", (long long)k);
    if (T == 0) return FMA_OK;
    FMA_REQUIRE(x && inv && out, FMA_ERR_NULL_POINTER, "dispatch_rows: NULL pointer");
    FMA_REQUIRE(element_aligned(dtype, {x, out}), FMA_ERR_MISALIGNED, "dispatch_rows: x/out not aligned to the element size");
    hipStream_t st = (hipStream_t)stream;
    if (rows_vectorise(dtype, H, {x, out})) return launch_dispatch<uint4>(x, inv, T, k, H * dtype_bytes(dtype) / 16, out, st);
    if (dtype_bytes(dtype) == 4) return launch_dispatch<uint32_t>(x, inv, T, k, H, out, st);
    return launch_dispatch<uint16_t>(x, inv, T, k, H, out, st);
}

int fma_combine(const void* o, const int32_t* inv, const void* gates, int64_t T, int64_t k, int64_t H, void* y,
                int dtype, void* stream) {
    using namespace fmahip;
    int rc = check_rows("combine", dtype, H);
    if (rc) return rc;
    FMA_REQUIRE(T >= 0 && T <= 0x7fffffffll, FMA_ERR_BAD_SIZE, "combine: bad token count %lld", (long long)T);
    FMA_REQUIRE(k >= 1 && T * k <= 0x7fffffffll, FMA_ERR_BAD_SIZE, "combine: bad top_k %lld", (long long)k);
    if (T == 0) return FMA_OK;
    FMA_REQUIRE(o && inv && y, FMA_ERR_NULL_POINTER, "combine: NULL pointer");
    FMA_REQUIRE(element_aligned(dtype, {o, y, gates}), FMA_ERR_MISALIGNED, "combine: o/y/gates not aligned to the element size");
    hipStream_t st = (hipStream_t)stream;
    if (rows_vectorise(dtype, H, {o, y})) {
        switch (dtype) {
            case FMA_F32: return launch_combine<float, Vec16<float>>(o, inv, gates, T, k, H, y, st);
            case FMA_F16: return launch_combine<f16_t, Vec16<f16_t>>(o, inv, gates, T, k, H, y, st);
            default: return launch_combine<bf16_t, Vec16<bf16_t>>(o, inv, gates, T, k, H, y, st);
        }
    }
    switch (dtype) {
        case FMA_F32: return launch_combine<float, Vec1<float>>(o, inv, gates, T, k, H, y, st);
        case FMA_F16: return launch_combine<f16_t, Vec1<f16_t>>(o, inv, gates, T, k, H, y, st);
        default: return launch_combine<bf16_t, Vec1<bf16_t>>(o, inv, gates, T, k, H, y, st);
    }
}

int fma_combine_bwd(const void* dy, const void* o, const int32_t* inv, const void* gates, int64_t T, int64_t k,
                    int64_t H, void* d_o, void* d_gates, int dtype, void* stream) {
    using namespace fmahip;
    int rc = check_rows("combine_bwd", dtype, H);
    if (rc) return rc;
    FMA_REQUIRE(T >= 0 && T <= 0x7fffffffll, FMA_ERR_BAD_SIZE, "combine_bwd: bad token count %lld", (long long)T);
    FMA_REQUIRE(k >= 1 && T * k <= 0x7fffffffll, FMA_ERR_BAD_SIZE, "combine_bwd: bad top_k %lld", (long long)k);
    if (T == 0) return FMA_OK;
    FMA_REQUIRE(dy && inv && d_o, FMA_ERR_NULL_POINTER, "combine_bwd: NULL pointer");
    FMA_REQUIRE(o || !d_gates, FMA_ERR_NULL_POINTER, "combine_bwd: d_gates requested but o is NULL");
    FMA_REQUIRE(element_aligned(dtype, {dy, d_o, o, gates, d_gates}), FMA_ERR_MISALIGNED,
                "combine_bwd: dy/o/d_o/gates/d_gates not aligned to the element size");
    hipStream_t st = (hipStream_t)stream;
    if (rows_vectorise(dtype, H, {dy, d_o, o})) {
        switch (dtype) {
            case FMA_F32: return launch_combine_bwd<float, Vec16<float>>(dy, o, inv, gates, T, k, H, d_o, d_gates, st);
            case FMA_F16: return launch_combine_bwd<f16_t, Vec16<f16_t>>(dy, o, inv, gates, T, k, H, d_o, d_gates, st);
            default: return launch_combine_bwd<bf16_t, Vec16<bf16_t>>(dy, o, inv, gates, T, k, H, d_o, d_gates, st);
        }
    }
    switch (dtype) {
        case FMA_F32: return launch_combine_bwd<float, Vec1<float>>(dy, o, inv, gates, T, k, H, d_o, d_gates, st);
        case FMA_F16: return launch_combine_bwd<f16_t, Vec1<f16_t>>(dy, o, inv, gates, T, k, H, d_o, d_gates, st);
        default: return launch_combine_bwd<bf16_t, Vec1<bf16_t>>(dy, o, inv, gates, T, k, H, d_o, d_gates, st);
    }
}

}  // extern "C"
