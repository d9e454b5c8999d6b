// Launch of the fp32 grouped GEMM (grouped_gemm_f32.hip) for fma_grouped_gemm.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fmahip {
namespace gemm_f32 {

// a_kc: A_e stored [M, K] (reduction dimension contiguous), else [K, M]; b_kc: B_e stored [N, K], else [K, N].
// Returns 0 or the launch error, with the message stored for fma_last_error_string().
int launch(const void* A, const void* B, void* D, const uint32_t* M_arr, const uint32_t* N_arr, const uint32_t* K_arr,
           int64_t E, bool a_kc, bool b_kc, float alpha, hipStream_t st);

}  // namespace gemm_f32
}  // namespace fmahip
