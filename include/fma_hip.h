/*
 * fma_hip.h — C ABI of libfma_hip.so: the MoE-layer hot path of cute-kernels ("fma")
 * as hand-written HIP kernels for gfx950 (MI355X).
 *
 * Conventions
 *  - Every pointer is a DEVICE pointer unless its comment says "host".
 *  - The caller owns every buffer, including workspaces (sizes come from the *_workspace_bytes queries).
 *    The library allocates nothing and keeps no state besides cached device properties.
 *  - `stream` is a hipStream_t passed as void* (NULL = the null stream). Calls only enqueue work.
 *  - Every entry point returns 0 on success, a negative FMA_ERR_* code for a rejected argument
 *    (nothing is launched then) or a positive hipError_t if the launch itself failed.
 *    fma_last_error_string() returns the message of the calling thread's last failure.
 *  - dtype codes: FMA_F32 / FMA_F16 / FMA_BF16. Index tensors produced here are int32.
 *
 * Citations name the reference interface each entry point stands in for (paths relative to the
 * cute-kernels source tree).
 */
#ifndef FMA_HIP_H
#define FMA_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FMA_OK 0
#define FMA_ERR_NULL_POINTER (-1)
#define FMA_ERR_BAD_DTYPE (-2)
#define FMA_ERR_BAD_SIZE (-3)
#define FMA_ERR_TOO_MANY_EXPERTS (-4)
#define FMA_ERR_TOO_MANY_ELEMENTS (-5)
#define FMA_ERR_MISALIGNED (-6)
#define FMA_ERR_WORKSPACE_TOO_SMALL (-7)
#define FMA_ERR_UNSUPPORTED (-8)

#define FMA_F32 0
#define FMA_F16 1
#define FMA_BF16 2

/* limits (same values as the reference's: continuous_count forward.cu:12, grouped_gemm kernel.cu:38) */
#define FMA_MAX_COUNT_BINS 16384
#define FMA_MAX_GROUPS 1024
/* largest top_k of the fused router */
#define FMA_MAX_ROUTER_TOP_K 64
/* longest row of the normalisation kernels (the reference's MAX_TRITON_BLOCK_SIZE, fma/constants.py:17) */
#define FMA_MAX_NORM_HIDDEN 65536

/* ---- library ---------------------------------------------------------------------------- */

/* Message of the calling thread's most recent failed call ("" if none). Host pointer, valid until the
 * thread's next failing call. Replaces the TORCH_CHECK / c10::Error text of the reference's pybind
 * functions (e.g. fma/ops/continuous_count/cuda_implementation/forward.cu:120-128). */
const char* fma_last_error_string(void);

/* ABI version of this header (bumped on any signature change). */
int fma_abi_version(void);

/* Number of compute units of the current device (0 if no device). The reference's get_num_SMs
 * (fma/include/device.h:8-16). */
int fma_num_compute_units(void);

/* ---- continuous_count ------------------------------------------------------------------- */

/* Bytes of workspace fma_continuous_count needs for n ids and E bins (one partial histogram per workgroup). The
 * buffer needs no initialisation; calls that overlap in time need separate buffers. */
int64_t fma_continuous_count_workspace_bytes(int64_t n, int64_t E);

/* counts[v] = #{ i < n : ids[i] == v } for v in [0, E); ids outside [0, E) are not counted.
 * ids: n integers of id_bytes (4 = int32, 8 = int64) each, 16-byte aligned; counts: E uint32, fully
 * overwritten (no need to zero). E <= FMA_MAX_COUNT_BINS, n <= 2^32-1.
 * Replaces continuous_count_cuda(x, output, E, THREAD_BLOCK_CLUSTER_SIZE, BLOCK_SIZE)
 * (fma/ops/continuous_count/cuda_implementation/ops.cpp:13-15, forward.cu:115-167); the two launch-shape
 * arguments have no meaning on wave64 hardware and are dropped here. */
int fma_continuous_count(const void* ids, int id_bytes, int64_t n, uint32_t* counts, int64_t E,
                         void* workspace, int64_t workspace_bytes, void* stream);

/* ---- index construction ------------------------------------------------------------------ */

/* Bytes of workspace fma_moe_build_index needs (no zeroing required). */
int64_t fma_moe_build_index_workspace_bytes(int64_t R, int64_t E);

/* Stable counting sort of the R routed slots by expert id. With slot s = t*top_k + j:
 *   counts[e]  = #{ s : ids[s] == e }                       (uint32[E])
 *   offsets[e] = counts[0] + ... + counts[e]   (inclusive)   (uint32[E])
 *   perm[i]    = i-th slot in (expert, slot) order           (int32[R])  == sorted_scattered_idxs
 *   eid[i]     = ids[perm[i]]                                (int32[R])  == sorted_expert_idxs
 *   inv[s]     = i with perm[i] == s                         (int32[R])
 * Every id must lie in [0, E); E <= FMA_MAX_GROUPS; R <= 2^31-1.
 * Replaces `selected_experts.flatten().sort()` + continuous_count + `expert_frequency.cumsum(-1)`
 * (fma/modules/moe/__init__.py:214-217,249); within one expert the order is ascending slot, i.e. the
 * order torch.sort(stable=True) defines. */
int fma_moe_build_index(const void* ids, int id_bytes, int64_t R, int64_t E, uint32_t* counts,
                        uint32_t* offsets, int32_t* perm, int32_t* eid, int32_t* inv, void* workspace,
                        int64_t workspace_bytes, void* stream);

/* fma_moe_build_index for ids that come from fma_router_topk, which has already counted them: token_block_hist
 * ([ceil(T / 16), E] uint32, T = R / top_k) holds, per block of 16 consecutive tokens, the number of choices of every
 * expert, as that call writes it. Two launches (prefix scan, placement) instead of three, no workspace: the histogram
 * itself is the scratch memory and is OVERWRITTEN. ids: int32 [R], every id in [0, E); top_k <= 64 divides R. Same
 * outputs, bit for bit, as fma_moe_build_index. Replaces the same reference lines, for the case that the choice and
 * its histogram come out of one kernel (fma/modules/moe/__init__.py:191-217). */
int fma_moe_build_index_from_hist(const int32_t* ids, int64_t R, int64_t E, int64_t top_k, uint32_t* token_block_hist,
                                  uint32_t* counts, uint32_t* offsets, int32_t* perm, int32_t* eid, int32_t* inv,
                                  void* stream);

/* Words (uint32) of the built-in scratch array of fma_moe_build_index_static: it serves calls with
 * fma_moe_build_index_workspace_bytes(R, E) <= 4 * this value. */
int64_t fma_moe_build_index_static_max_words(void);

/* fma_moe_build_index without a workspace argument and without any allocation: the per-chunk histograms live in a
 * fixed array in device memory that is part of the library image (4 MiB per GPU, held until the process ends), whose
 * address is looked up once per device. Same outputs, bit for bit. No counterpart in the reference: it is for callers
 * that cannot allocate or size a workspace (code under HIP graph capture, serving loops, harnesses that forbid
 * hipMalloc). Rejects sizes whose scratch exceeds the array (FMA_ERR_WORKSPACE_TOO_SMALL; R * E up to about 5e8).
 * All calls on one GPU share the array: calls that overlap in time on one GPU (different streams) race. */
int fma_moe_build_index_static(const void* ids, int id_bytes, int64_t R, int64_t E, uint32_t* counts,
                               uint32_t* offsets, int32_t* perm, int32_t* eid, int32_t* inv, void* stream);

/* ---- row movement ------------------------------------------------------------------------- */

/* out[i, :] = x[idx[i] / divisor, :] for i < R (rows of H elements; the four row kernels move 16 bytes per lane when
 * H*elem_bytes is a multiple of 16 and the buffers are 16-byte aligned, single elements otherwise).
 * Replaces group_with_padding_triton(..., NEEDS_DUPLICATION=True) without padding
 * (fma/modules/moe/cuda_implementation/group_kernel.py:26-74) and `hidden_states[fan_in_index]`
 * (fma/modules/moe/__init__.py:269,275). divisor = top_k maps a slot to its token; divisor = 1 is a
 * plain row gather. */
int fma_gather_rows(const void* x, const int32_t* idx, int64_t R, int64_t H, int32_t divisor, void* out,
                    int dtype, void* stream);

/* out[inv[t*k+j], :] = x[t, :] for t < T, j < k: the gather above for idx = the stable routing order and divisor =
 * top_k, written from the token's side (inv is the inverse permutation fma_moe_build_index returns), so each input
 * row is read once however many experts it goes to. Same references as fma_gather_rows. */
int fma_dispatch_rows(const void* x, const int32_t* inv, int64_t T, int64_t k, int64_t H, void* out, int dtype,
                      void* stream);

/* y[t, :] = sum_{j<k} gates[t*k+j] * o[inv[t*k+j], :]  accumulated in fp32 in ascending j, rounded once.
 * gates may be NULL (all ones; gives the k-way sum the backward of the gather needs). gates has dtype.
 * Replaces ungroup_with_padding + torch.bmm(router_weights, y) (fma/modules/moe/__init__.py:235-246,
 * ungroup_kernel.py:15-71) and `y * batch_gates` + index_add (fma/modules/moe/__init__.py:284-286). */
int fma_combine(const void* o, const int32_t* inv, const void* gates, int64_t T, int64_t k, int64_t H,
                void* y, int dtype, void* stream);

/* Backward of fma_combine for one upstream gradient dy[T, H]:
 *   d_o[inv[t*k+j], :] = gates[t*k+j] * dy[t, :]
 *   d_gates[t*k+j]     = <dy[t, :], o[inv[t*k+j], :]>   (fp32 accumulate)
 * d_gates may be NULL (skipped). Replaces the autograd of torch.bmm + _UngroupWithPadding.backward
 * (fma/modules/moe/cuda_implementation/__init__.py:226-249) and group(grad_out, coeff=gates) +
 * bmm(output_expanded, grad_out) of the triton branch (fma/modules/moe/triton_implementation/__init__.py:83-103). */
int fma_combine_bwd(const void* dy, const void* o, const int32_t* inv, const void* gates, int64_t T,
                    int64_t k, int64_t H, void* d_o, void* d_gates, int dtype, void* stream);

/* ---- SwiGLU -------------------------------------------------------------------------------- */

/* out[r, c] = up[r, c] * gate[r, c] * sigmoid(gate[r, c]) in fp32, rounded to dtype; rows x cols elements,
 * each operand with its own row stride in elements (so the halves of a packed [rows, 2*cols] tensor can
 * be passed without a copy). Replaces swiglu_forward_cuda(gate, up, output, BLOCK_SIZE)
 * (fma/ops/swiglu/cuda_implementation/ops.cpp, forward.cu:59-94) and the strided Triton kernel
 * (fma/ops/swiglu/triton_implementation/forward.py:16-46). */
int fma_swiglu_forward(const void* gate, const void* up, void* out, int64_t rows, int64_t cols,
                       int64_t gate_stride, int64_t up_stride, int64_t out_stride, int dtype, void* stream);

/* gate_grad = dy * up * (s + gate*s*(1-s)), up_grad = dy * gate * s with s = sigmoid(gate).
 * Replaces swiglu_backward_cuda(gate, up, output_grad, gate_grad, up_grad, BLOCK_SIZE)
 * (fma/ops/swiglu/cuda_implementation/backward.cu:79-129) and triton_implementation/backward.py:16-55. */
int fma_swiglu_backward(const void* gate, const void* up, const void* dy, void* gate_grad, void* up_grad,
                        int64_t rows, int64_t cols, int64_t gate_stride, int64_t up_stride, int64_t dy_stride,
                        int64_t gate_grad_stride, int64_t up_grad_stride, int dtype, void* stream);

/* ---- grouped GEMM --------------------------------------------------------------------------- */

/* For each group e < E:  D_e[M_e, N_e] = alpha * op(A_e) * op(B_e), fp32 accumulation, output rounded to dtype.
 * Groups are packed back to back in the flat A / B / D buffers (element offsets sum M*K, sum K*N, sum M*N).
 *   trans_a == 0: A_e stored [M_e, K_e] row-major;  trans_a != 0: stored [K_e, M_e].
 *   trans_b != 0: B_e stored [N_e, K_e] row-major;  trans_b == 0: stored [K_e, N_e].
 * M_arr / N_arr / K_arr: E uint32 each, DEVICE memory (never read on the host). A group with K_e == 0
 * gets zeros; a group with M_e == 0 or N_e == 0 produces nothing. dtype: FMA_BF16, FMA_F16 or FMA_F32
 * (fp32 runs on the fp32 matrix instruction, one sixteenth of the 16-bit rate, with no restriction on sizes).
 * For the 16-bit types each group's contiguous dimension should be a multiple of 8 elements (16 bytes); other
 * groups are computed by a slow scalar path. E <= FMA_MAX_GROUPS.
 * The 16-bit call enqueues three kernels of which one does the work: the sizes live in device memory, so each kernel
 * reads them and runs only if the launch has its form. Launches whose groups differ in one dimension only (every
 * grouped GEMM of an MoE layer, the reference's own test shapes) are computed by the kernel of
 * fma_grouped_gemm_ragged, anything else by a general kernel; a kernel that declines ends after reading the arrays.
 * Replaces grouped_gemm_cuda(A, B, C, output, M_array, N_array, K_array, is_A_transposed,
 * is_B_transposed, alpha, beta, benchmark) (fma/ops/grouped_gemm/cuda_implementation/ops.cpp,
 * kernel.cu:354-388); beta must be 0 and C absent there, so neither exists here. */
int fma_grouped_gemm(const void* A, const void* B, void* D, const uint32_t* M_arr, const uint32_t* N_arr,
                     const uint32_t* K_arr, int64_t E, int trans_a, int trans_b, float alpha, int dtype,
                     void* stream);

/* which dimension differs between the groups of fma_grouped_gemm_ragged */
#define FMA_VARY_M 0
#define FMA_VARY_K 1

/* fma_grouped_gemm for launches in which the groups differ in ONE dimension only, the case of every grouped GEMM of an
 * MoE layer: `sizes` (E uint32, device memory) holds the rows M_e of the groups (vary == FMA_VARY_M: forward and
 * input gradient; M is ignored) or their reduction lengths K_e (vary == FMA_VARY_K: weight gradient; K is ignored);
 * the other two dimensions are the same for all groups and are passed by value. Same results, bit for bit, as
 * fma_grouped_gemm with N_arr / K_arr (M_arr / N_arr) filled with those constants. Knowing them on the host lets the
 * kernel keep a third of the group table and run the operand loads as one stream across tile boundaries, which is
 * what the layer's GEMMs are launched through. dtype: FMA_BF16 or FMA_F16 (fp32 callers use fma_grouped_gemm).
 * bias: NULL, or [E, N] of dtype (4-byte aligned, N even) added to every row of its group in the epilogue: the rounded
 * product plus the bias in fp32, rounded once more, bit for bit what fma_expert_bias_add does to the output of the call
 * without a bias. Only in the forward form (vary == FMA_VARY_M, trans_a == 0, trans_b != 0, alpha == 1).
 * Replaces the same grouped_gemm_cuda calls as fma_grouped_gemm, as _GroupedGemmExperts makes them with
 * N_array / K_array = full_like(M_array, N / K) (fma/modules/moe/__init__.py:82-83,
 * fma/modules/moe/cuda_implementation/__init__.py:28-78); with a bias, the per-expert F.linear(x_e, W[e], bias[e])
 * of Experts.torch_forward (fma/modules/moe/__init__.py:98-105). */
int fma_grouped_gemm_ragged(const void* A, const void* B, void* D, const uint32_t* sizes, const void* bias, int64_t E,
                            int vary, int64_t M, int64_t N, int64_t K, int trans_a, int trans_b, float alpha, int dtype,
                            void* stream);

/* Up-projection with SwiGLU fused into the epilogue. For each expert e with M_e rows (rows of all experts
 * packed back to back, sum M_e = R):
 *   h_e   = x_e[M_e, K] * W_e[2I, K]^T            (rounded to dtype; written to h if h != NULL)
 *   act_e = h_e[:, :I] * silu(h_e[:, I:])         (first half "up", second half "gate")
 * computed from the ROUNDED h so the result equals fma_grouped_gemm followed by fma_swiglu_forward bit for
 * bit. W: [E, 2I, K] row-major; h: [R, 2I]; act: [R, I]; I % 8 == 0, K % 8 == 0, I < 2^22, K < 2^21.
 * bias: NULL, or [E, 2I] of dtype (4-byte aligned), added to h as fma_expert_bias_add would (rounded product plus bias,
 * rounded again) before the activation.
 * Fuses _GroupedGemmExperts.forward (fma/modules/moe/cuda_implementation/__init__.py:28-38) with
 * swiglu_packed (fma/ops/swiglu/__init__.py:133-164, up/gate = chunk(2, -1) at :153). */
int fma_grouped_gemm_swiglu(const void* x, const void* W, const void* bias, void* h, void* act, const uint32_t* M_arr,
                            int64_t E, int64_t I, int64_t K, int dtype, void* stream);

/* Input gradient of the second projection with the backward of SwiGLU in its epilogue. For each expert e with M_e rows:
 *   da_e = dy_e[M_e, K] * W_e[K, I]              (the gradient of the activation, rounded to dtype)
 *   dh_e[:, :I] = da_e * gate * s                 dh_e[:, I:] = da_e * up * (s + gate * s * (1 - s)),  s = sigmoid(gate)
 * with up = h_e[:, :I], gate = h_e[:, I:] of the packed pre-activation h [R, 2I]: what fma_grouped_gemm_ragged (rows vary,
 * trans_a = 0, trans_b = 0, N = I) followed by fma_swiglu_backward on the two halves of h gives, bit for bit, without da
 * ever being written. W: [E, K, I] row-major (the second projection's weight [E, out = K, in = I]); dh: [R, 2I].
 * I % 8 == 0, K % 8 == 0, I < 2^22, K < 2^21; dtype FMA_BF16 or FMA_F16.
 * Fuses _GroupedGemmExperts.backward (fma/modules/moe/cuda_implementation/__init__.py:40-60, the x_grad product) with the
 * backward of swiglu_packed (fma/ops/swiglu/__init__.py:133-164; cuda_implementation/backward.cu:79-129). */
int fma_grouped_gemm_swiglu_bwd(const void* dy, const void* W, const void* h, void* dh, const uint32_t* M_arr, int64_t E,
                                int64_t I, int64_t K, int dtype, void* stream);

/* The forward product of an expert projection with the gather of the routed rows inside the operand load: for each
 * expert e with M_e rows (packed rows i of all experts back to back, R = sum M_e)
 *   out[i, :] = x[row_index[i] / divisor, :] * W_e[N, K]^T (+ bias_e)
 * i.e. fma_grouped_gemm_ragged (swiglu == 0: out [R, N], act ignored) or fma_grouped_gemm_swiglu (swiglu != 0:
 * N = 2 I, out = the pre-activation h [R, 2 I] or NULL, act [R, I]) applied to the output of
 * fma_gather_rows(x, row_index, R, K, divisor), bit for bit, without that [R, K] buffer ever being written.
 * x: [x_rows, K] with x_rows * K * 2 < 2^31 bytes; an entry row_index[i] that is negative or whose row_index[i] / divisor is
 * not below x_rows names no row and is taken as a row of zeros (its output row is bias_e, or zero); divisor in [1, 65536]
 * (top_k with row_index = the stable routing order perm of fma_moe_build_index; 1 for a plain row index).
 * N % 8 == 0 (16 for swiglu), K % 8 == 0, N < 2^23, K < 2^21; dtype FMA_BF16 or FMA_F16.
 * Replaces the gather inside the reference's fused Triton expert kernel (fma/modules/moe/triton_implementation/
 * scatter_kernel.py:55-135: rows addressed through the sorted index while the product is formed) for the grouped-GEMM
 * path, where the reference materialises them (fma/modules/moe/__init__.py:269, cuda_implementation/__init__.py:28-38). */
int fma_grouped_gemm_gathered(const void* x, int64_t x_rows, const int32_t* row_index, int32_t divisor, const void* W,
                              const void* bias, void* out, void* act, const uint32_t* M_arr, int64_t E, int64_t N,
                              int64_t K, int swiglu, int dtype, void* stream);

/* The weight gradient of an expert projection with the gather of the routed rows inside the operand load: for each
 * expert e with K_e rows (packed rows i of all experts back to back, R = sum K_e)
 *   dW_e[M, N] = alpha * dy_e[K_e, M]^T * xg_e[K_e, N],   xg[i, :] = x[row_index[i] / divisor, :]
 * i.e. fma_grouped_gemm_ragged (reduction varies, trans_a = 1, trans_b = 0) applied to dy and the output of
 * fma_gather_rows(x, row_index, R, N, divisor), bit for bit, without that [R, N] buffer ever being written or read.
 * dy: [R, M] packed; x: [x_rows, N] with x_rows * N * 2 < 2^31 bytes; dW: [E, M, N]; an expert without rows gets zeros.
 * An entry row_index[i] that is negative or whose row_index[i] / divisor is not below x_rows names no row and contributes
 * nothing; divisor in [1, 65536] (top_k with row_index = the stable routing order perm of fma_moe_build_index).
 * M % 8 == 0, N % 8 == 0, both below 2^23 (K_e is arbitrary); dtype FMA_BF16 or FMA_F16.
 * The weight-gradient product of _GroupedGemmExperts.backward (fma/modules/moe/cuda_implementation/__init__.py:46-80) on
 * the rows the reference first materialises: with group_with_padding on the grouped-GEMM path (the same file, :107-183)
 * and with group() in front of group_bwd_W on the Triton path (triton_implementation/__init__.py:105-123,
 * group_backward_kernel.py:23-101). */
int fma_grouped_gemm_gathered_wgrad(const void* dy, const void* x, int64_t x_rows, const int32_t* row_index, int32_t divisor,
                                    void* dW, const uint32_t* K_arr, int64_t E, int64_t M, int64_t N, float alpha, int dtype,
                                    void* stream);

/* ---- per-expert bias ------------------------------------------------------------------------ */

/* y[i, :] += bias[e, :] for every row i of expert e, rows packed expert by expert with M_arr[e] rows each (device
 * array, as for fma_grouped_gemm); fp32 addition, one rounding; rows past sum(M_arr) are left alone. y: [R, N],
 * bias: [E, N], N * element size a multiple of 16. Together with fma_grouped_gemm this is the per-expert
 * `F.linear(x_e, W[e], bias[e])` of Experts.torch_forward (fma/modules/moe/__init__.py:98-105); the reference's
 * grouped-GEMM path drops the bias (:89-92) and its Triton path refuses it (:48, :73). */
int fma_expert_bias_add(void* y, const void* bias, const uint32_t* M_arr, int64_t E, int64_t R, int64_t N, int dtype,
                        void* stream);

/* Bytes of workspace fma_expert_bias_grad needs (no initialisation required). */
int64_t fma_expert_bias_grad_workspace_bytes(int64_t E, int64_t R, int64_t N);

/* d_bias[e, :] = sum of the rows dy[i, :] of expert e (zeros for an expert without rows), accumulated in fp32 per
 * slice of up to 256 rows in row order, slices added in order in fp64, rounded once to dtype: the gradient autograd gives the
 * bias of `F.linear(x_e, W[e], bias[e])` (fma/modules/moe/__init__.py:98-105). d_bias: [E, N], fully overwritten. */
int fma_expert_bias_grad(const void* dy, const uint32_t* M_arr, int64_t E, int64_t R, int64_t N, void* d_bias,
                         void* workspace, int64_t workspace_bytes, int dtype, void* stream);

/* ---- router ---------------------------------------------------------------------------------- */

/* The router in one pass over x[T, H]:
 *   logits[t, e]  = <x[t, :], gate_weight[e, :]>          fp32 accumulation, rounded to dtype   ([T, E])
 *   selected[t, :] = the top_k columns of logits[t, :] (the rounded values), largest first; equal values
 *                    in ascending column order; NaN ranks above every number                     (int32 [T, top_k])
 *   weights[t, :] = softmax of those top_k logits, computed in fp32, rounded to dtype           ([T, top_k])
 *   counts[e]     = #{(t, j) : selected[t, j] == e}   (uint32 [E]; fully overwritten; may be NULL)
 *   token_block_hist[b, e] = #{(t, j) : 16 b <= t < 16 b + 16, selected[t, j] == e}
 *                    (uint32 [ceil(T / 16), E]; fully overwritten; may be NULL): what fma_moe_build_index_from_hist takes
 * gate_weight: [E, H] row-major. dtype: FMA_BF16 or FMA_F16. H % 8 == 0, E <= FMA_MAX_GROUPS,
 * top_k <= min(E, FMA_MAX_ROUTER_TOP_K). x and gate_weight 16-byte aligned.
 * Replaces MoE._compute_routing_weights and MoE._get_topk (fma/modules/moe/__init__.py:191-204, 292-298:
 * `self.gate(hidden_states)`, `topk` / `max`, `F.softmax(router_weights.float(), dim=-1).type_as(...)`); with
 * counts it also yields what continuous_count(sorted_expert_idxs, num_experts) returns at :215-217. torch.topk
 * leaves the order of equal values open; the order here is one of the orders it may return. */
int fma_router_topk(const void* x, const void* gate_weight, int64_t T, int64_t H, int64_t E, int64_t top_k,
                    void* logits, void* weights, int32_t* selected, uint32_t* counts, uint32_t* token_block_hist,
                    int dtype, void* stream);

/* Backward of the top-k + softmax part of fma_router_topk: the gradient with respect to the logits.
 *   d_out[t, :] = d_logits[t, :]                          (zeros if d_logits == NULL)
 *   d_out[t, selected[t, j]] += round(s_j * (d_weights[t, j] - sum_i s_i d_weights[t, i]))
 * with s = the fp32 softmax of the kept logits (recomputed from logits and selected), the product rounded to
 * dtype and the sum rounded again, which is what autograd does for `softmax(values.float()).type_as(x)` after
 * `topk` plus a second use of the logits (fma/modules/moe/__init__.py:193-202). d_weights may be NULL (zeros).
 * d_out must not overlap d_logits. The gradients of x and gate_weight are then plain products with d_out. */
int fma_router_topk_bwd(const void* logits, const int32_t* selected, const void* d_weights,
                        const void* d_logits, int64_t T, int64_t E, int64_t top_k, void* d_out, int dtype,
                        void* stream);

/* ---- residual add + RMSNorm ------------------------------------------------------------------- */

/* For each of the B rows of H elements, in fp32:
 *   r   = x * multiplier + residual                    -> added_x_residual (rounded to dtype)
 *   inv = 1 / sqrt(mean(r^2) + eps)  (unrounded r)      -> rmsnorm_denominator[row] (fp32; may be NULL)
 *   out = r * inv * weight                              -> output (one rounding; weight may be NULL = ones)
 * multiplier = 1 stands for the reference's `multiplier=None`. Any H in [1, FMA_MAX_NORM_HIDDEN]; rows of a
 * multiple of 16 bytes (and 16-byte aligned pointers) up to 32 KB take the single-pass kernels.
 * dtype: FMA_F32 / FMA_F16 / FMA_BF16; weight has the dtype of x.
 * Replaces fused_residual_add_rmsnorm_forward_triton(x, residual, weight, output, eps, multiplier,
 * added_x_residual, rmsnorm_denominator) (fma/ops/fused_residual_add_rmsnorm/triton_implementation/forward.py:16-102;
 * torch formulation at fma/ops/fused_residual_add_rmsnorm/__init__.py:113-120). */
int fma_fused_residual_add_rmsnorm_fwd(const void* x, const void* residual, const void* weight, void* output,
                                       void* added_x_residual, float* rmsnorm_denominator, int64_t B, int64_t H,
                                       float eps, float multiplier, int dtype, void* stream);

/* Bytes of workspace the backward needs when a weight gradient is asked for (no initialisation required). */
int64_t fma_fused_residual_add_rmsnorm_bwd_workspace_bytes(int64_t B, int64_t H);

/* Backward of the above for the gradients output_grad (of out) and added_x_residual_grad (of r as the second
 * output; may be NULL = zeros). With g = output_grad * weight and inv from rmsnorm_denominator (NULL: recomputed
 * from the stored r):
 *   residual_grad = inv * g - inv^3 / H * r * <g, r> + added_x_residual_grad
 *   x_grad        = multiplier * residual_grad
 *   weight_grad[h] = sum over rows of output_grad[., h] * round(r[., h] * inv[.])   (fp32 [H], fully overwritten)
 * weight and weight_grad are both given or both NULL. The weight gradient is summed in a fixed order (per
 * workgroup in row order, then over workgroups), so it is the same bits on every run; the reference adds with atomics.
 * Replaces fused_residual_add_rmsnorm_backward_triton(added_x_residual, weight, output_grad, added_x_residual_grad,
 * rmsnorm_denominator, x_grad, residual_grad, weight_grad, eps, multiplier)
 * (fma/ops/fused_residual_add_rmsnorm/triton_implementation/backward.py:15-145). */
int fma_fused_residual_add_rmsnorm_bwd(const void* added_x_residual, const void* weight, const void* output_grad,
                                       const void* added_x_residual_grad, const float* rmsnorm_denominator,
                                       void* x_grad, void* residual_grad, float* weight_grad, int64_t B, int64_t H,
                                       float eps, float multiplier, void* workspace, int64_t workspace_bytes,
                                       int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FMA_HIP_H */
