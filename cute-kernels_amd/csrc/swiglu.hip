// Standalone SwiGLU forward / backward: y = up * gate * sigmoid(gate), all arithmetic in fp32.
// Operands are 2-D with independent row strides, so the two halves of a packed [rows, 2*cols] activation
// (first half = up, second half = gate) are passed as views without a copy. 16-byte lanes when every stride,
// the column count and every base pointer allow it; otherwise a scalar kernel with the same arithmetic.
#include "common.h"

namespace fmahip {
namespace {

constexpr int kSwThreads = 256;

template <typename T>
__device__ __forceinline__ float swiglu_f(float g, float u) {
    return u * g * sigmoid_for<T>(g);
}

template <typename T>
__device__ __forceinline__ void swiglu_b(float g, float u, float dy, float& dg, float& du) {
    const float s = sigmoid_for<T>(g);
    dg = dy * u * (s + g * s * (1.0f - s));
    du = dy * g * s;
}

struct Strides2 {
    int64_t gate, up, out;
};
struct Strides5 {
    int64_t gate, up, dy, dgate, dup;
};

// Position of a thread's current 16-byte vector in a rows x cvec grid of vectors, advanced by a fixed number of vectors
// per iteration without a division inside the loop.
struct VecCursor {
    int64_t i, r, c;   // flat index, row, vector column
    int64_t di, dr, dc;
    __device__ __forceinline__ VecCursor(int64_t first, int64_t stride, int64_t cvec)
        : i(first), r(first / cvec), c(first - (first / cvec) * cvec), di(stride), dr(stride / cvec),
          dc(stride - (stride / cvec) * cvec) {}
    __device__ __forceinline__ void advance(int64_t cvec) {
        i += di;
        r += dr;
        c += dc;
        if (c >= cvec) {
            c -= cvec;
            ++r;
        }
    }
};

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
        VecCursor p((int64_t)blockIdx.x * kSwThreads + threadIdx.x, (int64_t)gridDim.x * kSwThreads, cvec);
        // two vectors per iteration: four loads in flight per thread
        while (p.i + p.di < total) {
            const int64_t r0 = p.r, c0 = p.c * N;
            p.advance(cvec);
            const int64_t r1 = p.r, c1 = p.c * N;
            p.advance(cvec);
            const V g0 = *reinterpret_cast<const V*>(gate + r0 * s.gate + c0);
            const V u0 = *reinterpret_cast<const V*>(up + r0 * s.up + c0);
            const V g1 = *reinterpret_cast<const V*>(gate + r1 * s.gate + c1);
            const V u1 = *reinterpret_cast<const V*>(up + r1 * s.up + c1);
            *reinterpret_cast<V*>(out + r0 * s.out + c0) = compute(g0, u0);
            *reinterpret_cast<V*>(out + r1 * s.out + c1) = compute(g1, u1);
        }
        if (p.i < total) {
            const int64_t r0 = p.r, c0 = p.c * N;
            const V g0 = *reinterpret_cast<const V*>(gate + r0 * s.gate + c0);
            const V u0 = *reinterpret_cast<const V*>(up + r0 * s.up + c0);
            *reinterpret_cast<V*>(out + r0 * s.out + c0) = compute(g0, u0);
        }
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
        VecCursor p((int64_t)blockIdx.x * kSwThreads + threadIdx.x, (int64_t)gridDim.x * kSwThreads, cvec);
        // two vectors per iteration: six loads in flight per thread
        while (p.i + p.di < total) {
            const int64_t r0 = p.r, c0 = p.c * N;
            p.advance(cvec);
            const int64_t r1 = p.r, c1 = p.c * N;
            p.advance(cvec);
            const V g0 = *reinterpret_cast<const V*>(gate + r0 * s.gate + c0);
            const V u0 = *reinterpret_cast<const V*>(up + r0 * s.up + c0);
            const V d0 = *reinterpret_cast<const V*>(dy + r0 * s.dy + c0);
            const V g1 = *reinterpret_cast<const V*>(gate + r1 * s.gate + c1);
            const V u1 = *reinterpret_cast<const V*>(up + r1 * s.up + c1);
            const V d1 = *reinterpret_cast<const V*>(dy + r1 * s.dy + c1);
            V og, ou;
            compute(g0, u0, d0, og, ou);
            *reinterpret_cast<V*>(dgate + r0 * s.dgate + c0) = og;
            *reinterpret_cast<V*>(dup + r0 * s.dup + c0) = ou;
            compute(g1, u1, d1, og, ou);
            *reinterpret_cast<V*>(dgate + r1 * s.dgate + c1) = og;
            *reinterpret_cast<V*>(dup + r1 * s.dup + c1) = ou;
        }
        if (p.i < total) {
            const int64_t r0 = p.r, c0 = p.c * N;
            const V g0 = *reinterpret_cast<const V*>(gate + r0 * s.gate + c0);
            const V u0 = *reinterpret_cast<const V*>(up + r0 * s.up + c0);
            const V d0 = *reinterpret_cast<const V*>(dy + r0 * s.dy + c0);
            V og, ou;
            compute(g0, u0, d0, og, ou);
            *reinterpret_cast<V*>(dgate + r0 * s.dgate + c0) = og;
            *reinterpret_cast<V*>(dup + r0 * s.dup + c0) = ou;
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

template <typename T>
int run_fwd(const void* gate, const void* up, void* out, int64_t rows, int64_t cols, Strides2 s, hipStream_t st) {
    constexpr int N = Vec16<T>::N;
    const bool vec = cols % N == 0 && s.gate % N == 0 && s.up % N == 0 && s.out % N == 0 && aligned16(gate) &&
                     aligned16(up) && aligned16(out);
    if (vec)
        hipLaunchKernelGGL((swiglu_fwd_kernel<T, true>), dim3(grid_for(rows * (cols / N))), dim3(kSwThreads), 0, st,
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
        hipLaunchKernelGGL((swiglu_bwd_kernel<T, true>), dim3(grid_for(rows * (cols / N))), dim3(kSwThreads), 0, st,
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
