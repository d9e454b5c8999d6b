// Shared host/device helpers for libfma_hip.so (gfx950 only: 64-wide wavefronts, 16-byte vector memory ops).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fma_hip.h"

namespace fmahip {

constexpr int kWave = 64;

// ---- error reporting (host) ---------------------------------------------------------------
// Stores a printf-formatted message in the calling thread's error slot and returns `code`.
int fail(int code, const char* fmt, ...);
// Maps the result of the launch that just happened (hipGetLastError) to a return code.
int launch_status(const char* what);

#define FMA_REQUIRE(cond, code, ...)                  \
    do {                                              \
        if (!(cond)) return ::fmahip::fail(code, __VA_ARGS__); \
    } while (0)

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

static inline int dtype_bytes(int dtype) {
    switch (dtype) {
        case FMA_F32: return 4;
        case FMA_F16: return 2;
        case FMA_BF16: return 2;
        default: return 0;
    }
}

int num_compute_units();

// ---- device-side numeric types -------------------------------------------------------------
struct bf16_t {
    uint16_t bits;
};
struct f16_t {
    _Float16 v;
};

__device__ __forceinline__ float bf16_bits_to_float(uint32_t bits16) { return __uint_as_float(bits16 << 16); }

// round-to-nearest-even fp32 -> bf16 (NaN stays NaN), same rounding as torch's .to(torch.bfloat16)
__device__ __forceinline__ uint32_t float_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}

template <typename T>
struct Num;

template <>
struct Num<float> {
    static __device__ __forceinline__ float up(float x) { return x; }
    static __device__ __forceinline__ float down(float x) { return x; }
};
template <>
struct Num<bf16_t> {
    static __device__ __forceinline__ float up(bf16_t x) { return bf16_bits_to_float(x.bits); }
    static __device__ __forceinline__ bf16_t down(float x) { return bf16_t{(uint16_t)float_to_bf16_bits(x)}; }
};
template <>
struct Num<f16_t> {
    static __device__ __forceinline__ float up(f16_t x) { return (float)x.v; }
    static __device__ __forceinline__ f16_t down(float x) { return f16_t{(_Float16)x}; }
};

// A 16-byte vector of T (4 floats or 8 halves), the unit of every global load/store in the row kernels.
template <typename T>
struct alignas(16) Vec16 {
    static constexpr int N = 16 / sizeof(T);
    T v[N];
};

// 16-byte store with the non-temporal hint, for outputs much larger than the caches that the kernel does not read back
template <typename V>
__device__ __forceinline__ void store_streaming16(V* p, const V& v) {
    static_assert(sizeof(V) == 16, "16-byte vectors only");
    typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
    __builtin_nontemporal_store(__builtin_bit_cast(u32x4, v), reinterpret_cast<u32x4*>(p));
}

// 16-byte load with the non-temporal hint, for inputs that are read exactly once
template <typename V>
__device__ __forceinline__ V load_streaming16(const V* p) {
    static_assert(sizeof(V) == 16, "16-byte vectors only");
    typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
    return __builtin_bit_cast(V, __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p)));
}

// sigmoid with the argument clamped to +-88.3762626647949 (the reference's fma/include/activations.h:9-22),
// which keeps expf finite and changes no finite result.
__device__ __forceinline__ float sigmoid_clamped(float x) {
    x = fmaxf(-88.3762626647949f, x);
    x = fminf(88.3762626647949f, x);
    return 1.0f / (1.0f + expf(-x));
}

// The same sigmoid from the hardware's exp2 and reciprocal instructions (about 2 ulp in fp32): used wherever the result
// is rounded to a 16-bit type, where the difference is far below half an ulp of the output.
__device__ __forceinline__ float sigmoid_clamped_fast(float x) {
    x = __builtin_amdgcn_fmed3f(x, -88.3762626647949f, 88.3762626647949f);  // the clamp as one instruction
    // v_rcp_f32 (1 ulp); a correctly rounded reciprocal would expand to the ten-instruction division sequence
    return __builtin_amdgcn_rcpf(1.0f + __expf(-x));
}

// sigmoid for an op whose output type is T
template <typename T>
__device__ __forceinline__ float sigmoid_for(float x) {
    if constexpr (sizeof(T) == 4) return sigmoid_clamped(x);
    else return sigmoid_clamped_fast(x);
}

// SwiGLU y = up * gate * sigmoid(gate) and its gradients, in fp32, for an op whose tensors have type T
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

// inclusive prefix sum across the 64 lanes of a wavefront
template <typename T>
__device__ __forceinline__ T wave_inclusive_scan(T v) {
    const int lane = threadIdx.x & (kWave - 1);
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        T o = __shfl_up(v, d, kWave);
        if (lane >= d) v += o;
    }
    return v;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int d = kWave / 2; d > 0; d >>= 1) v += __shfl_xor(v, d, kWave);
    return v;
}

}  // namespace fmahip
