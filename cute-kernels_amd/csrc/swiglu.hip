// Standalone SwiGLU forward / backward: y = up * gate * sigmoid(gate), all arithmetic in fp32.
// Operands are 2-D with independent row strides, so the two halves of a packed [rows, 2*cols] activation
// (first half = up, second half = gate) are passed as views without a copy. 16-byte lanes when every stride,
// the column count and every base pointer allow it; otherwise a scalar kernel with the same arithmetic.
#include "common.h"

namespace fmahip {
namespace {

constexpr int kSwThreads = 256;

// (the arithmetic itself, swiglu_f / swiglu_b, is shared with the GEMM epilogues: common.h)

struct Strides2 {
    int64_t gate, up, out;
};
struct Strides5 {
    int64_t gate, up, dy, dgate, dup;
};

// The 16-byte kernels are one-shot: a workgroup takes kSwUnroll * 256 consecutive vectors of the flattened rows x cvec grid
// of vectors, issues all of its loads (streaming: every byte is touched once), computes, stores (streaming) and exits.
// Measured against persistent grid-stride loops on 1 GiB streams: two reads + one write 6.4 against 6.0 TB/s, three reads
// + two writes 5.7 against 4.4-5.1 TB/s; the non-temporal hints are worth 0.5 TB/s in either form.
constexpr int kSwUnroll = 4;

// row and vector column of flat vector index i (32-bit division whenever the grid of vectors allows it)
__device__ __forceinline__ void split_index(int64_t i, int64_t cvec, bool small, int64_t& r, int64_t& c) {
    if (small) {
        const uint32_t q = (uint32_t)i / (uint32_t)cvec;
        r = q;
        c = (uint32_t)i - q * (uint32_t)cvec;
    } else {
        r = i / cvec;
        c = i - r * cvec;
    }
}

template <typename T, bool VEC>
__global__ __launch_bounds__(kSwThreads) void swiglu_fwd_kernel(const T* __restrict__ gate, const T* __restrict__ up,
                                                                T* __restrict__ out, int64_t rows, int64_t cols,
                                                                Strides2 s) {
    constexpr int N = VEC ? Vec16<T>::N : 1;
    const int64_t cvec = cols / N;
    const int64_t total = rows * cvec;
    if constexpr (VEC) {
        typedef Vec16<T> V;
        auto compute = [](const V& g, const V& u) {
            V y;
#pragma unroll
            for (int e = 0; e < N; ++e) y.v[e] = Num<T>::down(swiglu_f<T>(Num<T>::up(g.v[e]), Num<T>::up(u.v[e])));
            return y;
        };
        const bool small = total <= 0xffffffffll;
        const int64_t first = (int64_t)blockIdx.x * (kSwThreads * kSwUnroll) + threadIdx.x;
        int64_t og[kSwUnroll], ou[kSwUnroll], oo[kSwUnroll];
        V g[kSwUnroll], u[kSwUnroll];
#pragma unroll
        for (int k = 0; k < kSwUnroll; ++k) {
            const int64_t i = first + k * kSwThreads;
            int64_t r, c;
            split_index(i < total ? i : total - 1, cvec, small, r, c);
            og[k] = r * s.gate + c * N;
            ou[k] = r * s.up + c * N;
            oo[k] = i < total ? r * s.out + c * N : -1;
        }
#pragma unroll
        for (int k = 0; k < kSwUnroll; ++k) {
            g[k] = load_streaming16(reinterpret_cast<const V*>(gate + og[k]));
            u[k] = load_streaming16(reinterpret_cast<const V*>(up + ou[k]));
        }
#pragma unroll
        for (int k = 0; k < kSwUnroll; ++k)
            if (oo[k] >= 0) store_streaming16(reinterpret_cast<V*>(out + oo[k]), compute(g[k], u[k]));
    } else {
        for (int64_t i = (int64_t)blockIdx.x * kSwThreads + threadIdx.x; i < total; i += (int64_t)gridDim.x * kSwThreads) {
            const int64_t r = i / cvec;
            const int64_t c = i - r * cvec;
            out[r * s.out + c] = Num<T>::down(swiglu_f<T>(Num<T>::up(gate[r * s.gate + c]), Num<T>::up(up[r * s.up + c])));
        }
    }
}

template <typename T, bool VEC>
__global__ __launch_bounds__(kSwThreads) void swiglu_bwd_kernel(const T* __restrict__ gate, const T* __restrict__ up,
                                                                const T* __restrict__ dy, T* __restrict__ dgate,
                                                                T* __restrict__ dup, int64_t rows, int64_t cols,
                                                                Strides5 s) {
    constexpr int N = VEC ? Vec16<T>::N : 1;
    const int64_t cvec = cols / N;
    const int64_t total = rows * cvec;
    if constexpr (VEC) {
        typedef Vec16<T> V;
        auto compute = [](const V& g, const V& u, const V& d, V& og, V& ou) {
#pragma unroll
            for (int e = 0; e < N; ++e) {
                float a, b;
                swiglu_b<T>(Num<T>::up(g.v[e]), Num<T>::up(u.v[e]), Num<T>::up(d.v[e]), a, b);
                og.v[e] = Num<T>::down(a);
                ou.v[e] = Num<T>::down(b);
            }
        };
        const bool small = total <= 0xffffffffll;
        const int64_t first = (int64_t)blockIdx.x * (kSwThreads * kSwUnroll) + threadIdx.x;
        int64_t o_g[kSwUnroll], o_u[kSwUnroll], o_d[kSwUnroll], o_dg[kSwUnroll], o_du[kSwUnroll];
        V g[kSwUnroll], u[kSwUnroll], d[kSwUnroll];
#pragma unroll
        for (int k = 0; k < kSwUnroll; ++k) {
            const int64_t i = first + k * kSwThreads;
            int64_t r, c;
            split_index(i < total ? i : total - 1, cvec, small, r, c);
            o_g[k] = r * s.gate + c * N;
            o_u[k] = r * s.up + c * N;
            o_d[k] = r * s.dy + c * N;
            o_dg[k] = i < total ? r * s.dgate + c * N : -1;
            o_du[k] = r * s.dup + c * N;
        }
#pragma unroll
        for (int k = 0; k < kSwUnroll; ++k) {
            g[k] = load_streaming16(reinterpret_cast<const V*>(gate + o_g[k]));
            u[k] = load_streaming16(reinterpret_cast<const V*>(up + o_u[k]));
            d[k] = load_streaming16(reinterpret_cast<const V*>(dy + o_d[k]));
        }
#pragma unroll
        for (int k = 0; k < kSwUnroll; ++k) {
            if (o_dg[k] >= 0) {
                V og, ou;
                compute(g[k], u[k], d[k], og, ou);
                store_streaming16(reinterpret_cast<V*>(dgate + o_dg[k]), og);
                store_streaming16(reinterpret_cast<V*>(dup + o_du[k]), ou);
            }
        }
    } else {
        for (int64_t i = (int64_t)blockIdx.x * kSwThreads + threadIdx.x; i < total; i += (int64_t)gridDim.x * kSwThreads) {
            const int64_t r = i / cvec;
            const int64_t c = i - r * cvec;
            float a, b;
            swiglu_b<T>(Num<T>::up(gate[r * s.gate + c]), Num<T>::up(up[r * s.up + c]), Num<T>::up(dy[r * s.dy + c]), a, b);
            dgate[r * s.dgate + c] = Num<T>::down(a);
            dup[r * s.dup + c] = Num<T>::down(b);
        }
    }
}

inline uint32_t grid_for(int64_t work_items) {
    int64_t blocks = (work_items + kSwThreads - 1) / kSwThreads;
    const int64_t cap = (int64_t)(num_compute_units() > 0 ? num_compute_units() : 256) * 32;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    return (uint32_t)blocks;
}

inline uint32_t one_shot_grid(int64_t vectors) {
    return (uint32_t)((vectors + kSwThreads * kSwUnroll - 1) / (kSwThreads * kSwUnroll));
}

template <typename T>
int run_fwd(const void* gate, const void* up, void* out, int64_t rows, int64_t cols, Strides2 s, hipStream_t st) {
    constexpr int N = Vec16<T>::N;
    const bool vec = cols % N == 0 && s.gate % N == 0 && s.up % N == 0 && s.out % N == 0 && aligned16(gate) &&
                     aligned16(up) && aligned16(out);
    if (vec)
        hipLaunchKernelGGL((swiglu_fwd_kernel<T, true>), dim3(one_shot_grid(rows * (cols / N))), dim3(kSwThreads), 0, st,
                           (const T*)gate, (const T*)up, (T*)out, rows, cols, s);
    else
        hipLaunchKernelGGL((swiglu_fwd_kernel<T, false>), dim3(grid_for(rows * cols)), dim3(kSwThreads), 0, st,
                           (const T*)gate, (const T*)up, (T*)out, rows, cols, s);
    return launch_status("swiglu_forward");
}

template <typename T>
int run_bwd(const void* gate, const void* up, const void* dy, void* dgate, void* dup, int64_t rows, int64_t cols,
            Strides5 s, hipStream_t st) {
    constexpr int N = Vec16<T>::N;
    const bool vec = cols % N == 0 && s.gate % N == 0 && s.up % N == 0 && s.dy % N == 0 && s.dgate % N == 0 &&
                     s.dup % N == 0 && aligned16(gate) && aligned16(up) && aligned16(dy) && aligned16(dgate) &&
                     aligned16(dup);
    if (vec)
        hipLaunchKernelGGL((swiglu_bwd_kernel<T, true>), dim3(one_shot_grid(rows * (cols / N))), dim3(kSwThreads), 0, st,
                           (const T*)gate, (const T*)up, (const T*)dy, (T*)dgate, (T*)dup, rows, cols, s);
    else
        hipLaunchKernelGGL((swiglu_bwd_kernel<T, false>), dim3(grid_for(rows * cols)), dim3(kSwThreads), 0, st,
                           (const T*)gate, (const T*)up, (const T*)dy, (T*)dgate, (T*)dup, rows, cols, s);
    return launch_status("swiglu_backward");
}

}  // namespace
}  // namespace fmahip

extern "C" {

int fma_swiglu_forward(const void* gate, const void* up, void* out, int64_t rows, int64_t cols, int64_t gate_stride,
                       int64_t up_stride, int64_t out_stride, int dtype, void* stream) {
    using namespace fmahip;
    FMA_REQUIRE(dtype_bytes(dtype) != 0, FMA_ERR_BAD_DTYPE, "swiglu_forward: unknown dtype code %d", dtype);
    FMA_REQUIRE(rows >= 0 && cols >= 0, FMA_ERR_BAD_SIZE, "swiglu_forward: negative shape %lld x %lld", (long long)rows,
                (long long)cols);
    FMA_REQUIRE(gate_stride >= cols && up_stride >= cols && out_stride >= cols, FMA_ERR_BAD_SIZE,
                "swiglu_forward: a row stride is smaller than the %lld columns", (long long)cols);
    if (rows == 0 || cols == 0) return FMA_OK;
    FMA_REQUIRE(gate && up && out, FMA_ERR_NULL_POINTER, "swiglu_forward: NULL pointer");
    const Strides2 s{gate_stride, up_stride, out_stride};
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case FMA_F32: return run_fwd<float>(gate, up, out, rows, cols, s, st);
        case FMA_F16: return run_fwd<f16_t>(gate, up, out, rows, cols, s, st);
        default: return run_fwd<bf16_t>(gate, up, out, rows, cols, s, st);
    }
}

int fma_swiglu_backward(const void* gate, const void* up, const void* dy, void* gate_grad, void* up_grad, int64_t rows,
                        int64_t cols, int64_t gate_stride, int64_t up_stride, int64_t dy_stride,
                        int64_t gate_grad_stride, int64_t up_grad_stride, int dtype, void* stream) {
    using namespace fmahip;
    FMA_REQUIRE(dtype_bytes(dtype) != 0, FMA_ERR_BAD_DTYPE, "swiglu_backward: unknown dtype code %d", dtype);
    FMA_REQUIRE(rows >= 0 && cols >= 0, FMA_ERR_BAD_SIZE, "swiglu_backward: negative shape %lld x %lld",
                (long long)rows, (long long)cols);
    FMA_REQUIRE(gate_stride >= cols && up_stride >= cols && dy_stride >= cols && gate_grad_stride >= cols &&
                    up_grad_stride >= cols,
                FMA_ERR_BAD_SIZE, "swiglu_backward: a row stride is smaller than the %lld columns", (long long)cols);
    if (rows == 0 || cols == 0) return FMA_OK;
    FMA_REQUIRE(gate && up && dy && gate_grad && up_grad, FMA_ERR_NULL_POINTER, "swiglu_backward: NULL pointer");
    const Strides5 s{gate_stride, up_stride, dy_stride, gate_grad_stride, up_grad_stride};
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case FMA_F32: return run_bwd<float>(gate, up, dy, gate_grad, up_grad, rows, cols, s, st);
        case FMA_F16: return run_bwd<f16_t>(gate, up, dy, gate_grad, up_grad, rows, cols, s, st);
        default: return run_bwd<bf16_t>(gate, up, dy, gate_grad, up_grad, rows, cols, s, st);
    }
}

}  // extern "C"
