"""Mixture-of-Experts layer: the reference's `Experts` and `MoE` modules (fma/modules/moe/__init__.py:17-298) with the
expert computation done by the HIP kernels of libfma_hip.so.

Parameter and buffer names and shapes are the reference's (`gate.weight [E, H]`, `c_fc.weight [E, 2I or I, H]`,
`c_proj.weight [E, H, I]`, uint32 buffers `N_array` / `K_array`), so its state_dicts load unchanged.
"""

from typing import Callable

import torch
import torch.nn as nn
import torch.nn.functional as F

from ...kernel_backend import KernelBackend, is_hip_kernel_backend
from ...ops.swiglu import swiglu_packed
from .cuda_implementation import (
    add_expert_bias,
    build_routing_index,
    combine,
    fused_router,
    fused_router_with_histogram,
    gathered_swiglu_experts,
    gathered_up_projection_experts,
    swiglu_experts,
    can_gather_inside_gemm,
    gather_rows,
    grouped_gemm_experts,
    up_projection_swiglu_experts,
)


class Experts(nn.Module):
    """The weights (and optional biases) of all experts of one projection: `weight[e]` is expert e's [out, in] matrix."""

    def __init__(
        self, num_experts: int, in_features: int, out_features: int, add_bias: bool = True, std: float | None = None
    ) -> None:
        super().__init__()
        self.num_experts, self.in_features, self.out_features, self.std = num_experts, in_features, out_features, std

        self.weight = nn.Parameter(torch.empty(num_experts, out_features, in_features))
        self.bias = nn.Parameter(torch.empty(num_experts, out_features)) if add_bias else None
        # per-group N and K of the grouped GEMM, kept on the device next to the weights (buffers of the state_dict)
        for name in ("N_array", "K_array"):
            self.register_buffer(name, torch.empty((num_experts,), dtype=torch.uint32))

        self.reset_parameters()

    def cuda_forward(self, input: torch.Tensor, expert_frequency: torch.Tensor) -> torch.Tensor:
        # the reference's cuda_forward (fma/modules/moe/__init__.py:89-92) silently drops the bias; here it is added
        # to the rows of every expert (in the GEMM's epilogue for 16-bit types), which is what its torch_forward
        # computes (:98-105)
        return grouped_gemm_experts(
            x=input, weight=self.weight, M_array=expert_frequency, N_array=self.N_array, K_array=self.K_array,
            bias=self.bias,
        )

    def cuda_forward_swiglu(self, input: torch.Tensor, expert_frequency: torch.Tensor) -> torch.Tensor:
        """up-projection with swiglu_packed fused into the GEMM epilogue: returns [sum(M), out_features / 2]"""
        return up_projection_swiglu_experts(
            x=input, weight=self.weight, M_array=expert_frequency, N_array=self.N_array, K_array=self.K_array,
            bias=self.bias,
        )

    @staticmethod
    def _routing_tensors(
        sorted_scattered_idxs: torch.Tensor, expert_offsets: torch.Tensor
    ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        """rows per expert (uint32), the routing order and its inverse (int32) from what the reference's callers hold:
        the order of the (token, choice) slots sorted by expert and the inclusive offsets of the experts in it"""
        perm = sorted_scattered_idxs.to(torch.int32).contiguous()
        inverse = torch.empty_like(perm)
        inverse[perm.long()] = torch.arange(perm.numel(), dtype=torch.int32, device=perm.device)
        offsets = expert_offsets.to(torch.int32)
        counts = torch.diff(offsets, prepend=offsets.new_zeros(1))
        return counts.contiguous().view(torch.uint32), perm, inverse

    def up_projection_triton_forward(
        self,
        input: torch.Tensor,
        num_experts_per_token: int | None = None,
        sorted_expert_idxs: torch.Tensor | None = None,
        sorted_scattered_idxs: torch.Tensor | None = None,
        expert_offsets: torch.Tensor | None = None,
    ) -> torch.Tensor:
        """The reference's entry point of this name (fma/modules/moe/__init__.py:40-62: scattered_experts with the tokens
        as input and grouped rows as output), on the HIP kernels: row i of the result is input[sorted_scattered_idxs[i] //
        num_experts_per_token] @ weight[expert of row i]^T, the rows gathered inside the GEMM where its limits allow."""
        assert self.bias is None
        expert_frequency, perm, inverse = self._routing_tensors(sorted_scattered_idxs, expert_offsets)
        if can_gather_inside_gemm(input, self.weight, None):
            return gathered_up_projection_experts(
                input, self.weight, None, perm, inverse, expert_frequency, self.N_array, self.K_array,
                num_experts_per_token, False,
            )  # fmt: skip
        return self.cuda_forward(gather_rows(input, perm, inverse, num_experts_per_token), expert_frequency)

    def down_projection_triton_forward(
        self,
        input: torch.Tensor,
        num_experts_per_token: int | None = None,
        sorted_expert_idxs: torch.Tensor | None = None,
        sorted_scattered_idxs: torch.Tensor | None = None,
        expert_offsets: torch.Tensor | None = None,
        gates: torch.Tensor | None = None,
    ) -> torch.Tensor:
        """The reference's entry point of this name (fma/modules/moe/__init__.py:64-87: scattered_experts with grouped rows
        as input), on the HIP kernels: the projection of the grouped rows, returned per (token, choice) slot, or, with
        `gates` [T, k], as the gate-weighted sum over every token's k rows."""
        assert self.bias is None
        expert_frequency, perm, inverse = self._routing_tensors(sorted_scattered_idxs, expert_offsets)
        output = self.cuda_forward(input, expert_frequency)
        if gates is None:
            # out[slot] = output[row of slot]: the row movement of gather_rows with the two index arrays exchanged
            return gather_rows(output, inverse, perm, 1)
        return combine(output, gates, inverse)

    def extra_repr(self) -> str:
        return f"num_experts={self.num_experts}, in_features={self.in_features}, out_features={self.out_features}"

    @torch.no_grad()
    def reset_parameters(self) -> None:
        # N(0, std) weights, zero biases (fma/modules/moe/__init__.py:112-121), and the two size buffers
        nn.init.normal_(self.weight, mean=0, std=self.std)
        if getattr(self, "bias", None) is not None:
            self.bias.zero_()
        self.N_array.fill_(self.out_features)
        self.K_array.fill_(self.in_features)


def _is_swiglu_packed(activation_function: Callable) -> bool:
    fn = getattr(activation_function, "func", activation_function)  # functools.partial(swiglu_packed, ...)
    return fn is swiglu_packed


class MoE(nn.Module):
    def __init__(
        self,
        num_experts: int,
        num_experts_per_tok: int,
        hidden_size: int,
        intermediate_size: int,
        activation_function: Callable,
        is_glu: bool,
        add_bias: bool,
        std: float,
    ) -> None:
        super().__init__()

        self.num_experts = num_experts
        self.top_k = num_experts_per_tok

        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size

        self.gate = nn.Linear(in_features=self.hidden_size, out_features=num_experts, bias=False)
        # gate GEMM, top-k and softmax in one kernel wherever that kernel applies (16-bit activations on the GPU)
        self.fuse_router = True

        self.c_fc = Experts(
            num_experts=num_experts,
            in_features=self.hidden_size,
            out_features=2 * self.intermediate_size if is_glu else self.intermediate_size,
            add_bias=add_bias,
            std=std,
        )

        # None: decided per call (see _gathers_inside_gemm); True / False: always / never
        self.gather_in_gemm: bool | None = None
        # the activation's backward inside the second projection's input-gradient GEMM (see _runs_swiglu_experts_as_one_node)
        self.fuse_swiglu_backward = True

        self.act = activation_function
        # swiglu_packed as the activation of a GLU layer is computed inside the up-projection's epilogue (a kernel for
        # rows of whole 16-byte pieces; other sizes run the GEMM's element-wise path and the activation after it)
        self.fuse_swiglu = (
            is_glu
            and _is_swiglu_packed(activation_function)
            and self.hidden_size % 8 == 0
            and self.intermediate_size % 8 == 0
        )

        self.c_proj = Experts(
            num_experts=num_experts,
            in_features=self.intermediate_size,
            out_features=self.hidden_size,
            add_bias=add_bias,
            std=std,
        )

    def forward(
        self, hidden_states: torch.Tensor, kernel_backend: KernelBackend = KernelBackend.triton
    ) -> tuple[torch.Tensor, torch.Tensor]:
        original_shape = hidden_states.shape

        # hidden_states -> (total_q, hidden_size)
        hidden_states = hidden_states.view(-1, self.hidden_size)
        token_block_histogram = None
        if self._router_is_fusable(hidden_states):
            # the router kernel counts its choices as it makes them; the index build starts from those counts
            router_logits, router_weights, selected_experts, token_block_histogram = fused_router_with_histogram(
                hidden_states, self.gate.weight, self.top_k
            )
        else:
            router_logits, router_weights, selected_experts = self._compute_routing_weights(hidden_states)

        # router_logits -> (total_q, num_experts); router_weights, selected_experts -> (total_q, top_k)
        hidden_states = self._compute_experts(
            hidden_states,
            router_weights,
            selected_experts,
            kernel_backend=kernel_backend,
            token_block_histogram=token_block_histogram,
        )

        hidden_states = hidden_states.view(original_shape)

        return hidden_states, router_logits

    def _router_is_fusable(self, hidden_states: torch.Tensor) -> bool:
        # the last three lines are the size limits of fma_router_topk (32-bit offsets into logits and choices): larger
        # inputs take the library calls below instead of raising
        T = hidden_states.size(0)
        return (
            self.fuse_router
            and hidden_states.is_cuda
            and hidden_states.dtype in (torch.bfloat16, torch.float16)
            and self.gate.weight.dtype == hidden_states.dtype
            and self.hidden_size % 8 == 0
            and self.num_experts <= 1024
            and self.top_k <= 64
            and self.hidden_size <= (1 << 24)
            and T * self.num_experts <= 2**31 - 1
            and T * self.top_k <= 2**31 - 1
        )

    def _compute_routing_weights(self, hidden_states: torch.Tensor) -> tuple[torch.Tensor]:
        if self._router_is_fusable(hidden_states):
            # same three results; selected_experts comes back as int32, sorted by descending logit
            return fused_router(hidden_states, self.gate.weight, self.top_k)

        router_logits = self.gate(hidden_states)
        router_weights, selected_experts = self._get_topk(router_logits)

        # softmax over the k kept logits, in fp32
        router_weights = F.softmax(router_weights.float(), dim=-1)
        router_weights = router_weights.type_as(hidden_states)

        return router_logits, router_weights, selected_experts

    def _compute_experts(
        self,
        hidden_states: torch.Tensor,
        router_weights: torch.Tensor,
        selected_experts: torch.Tensor,
        kernel_backend: KernelBackend,
        token_block_histogram: torch.Tensor | None = None,
    ) -> torch.Tensor:
        if not is_hip_kernel_backend(kernel_backend):
            raise ValueError(f"unexpected kernel_backend ({kernel_backend})")

        # counts, offsets and the stable expert-major order of the (token, choice) slots, with its inverse
        expert_frequency, _, sorted_scattered_idxs, _, inverse = build_routing_index(
            selected_experts, self.num_experts, token_block_histogram
        )

        if self._gathers_inside_gemm(hidden_states):
            # the first projection (and its weight gradient) reads its rows x[slot // top_k] through the routing order: no
            # grouped copy of x
            if self._runs_swiglu_experts_as_one_node(hidden_states):
                hidden_states = gathered_swiglu_experts(
                    hidden_states, self.c_fc.weight, self.c_fc.bias, self.c_proj.weight, self.c_proj.bias,
                    sorted_scattered_idxs, inverse, expert_frequency, self.c_fc.N_array, self.c_fc.K_array,
                    self.c_proj.N_array, self.c_proj.K_array, self.top_k,
                )  # fmt: skip
                return combine(hidden_states, router_weights, inverse)
            fused = self.fuse_swiglu
            hidden_states = gathered_up_projection_experts(
                hidden_states, self.c_fc.weight, self.c_fc.bias, sorted_scattered_idxs, inverse, expert_frequency,
                self.c_fc.N_array, self.c_fc.K_array, self.top_k, fused,
            )  # fmt: skip
            if not fused:
                hidden_states = self.act(hidden_states)
            hidden_states = self.c_proj.cuda_forward(input=hidden_states, expert_frequency=expert_frequency)
            return combine(hidden_states, router_weights, inverse)

        # rows of every expert back to back: x[slot // top_k]
        hidden_states = gather_rows(hidden_states, sorted_scattered_idxs, inverse, self.top_k)

        if self._runs_swiglu_experts_as_one_node(hidden_states):
            # both projections in one autograd node: its backward forms the pre-activation's gradient in one kernel
            hidden_states = swiglu_experts(
                hidden_states, self.c_fc.weight, self.c_fc.bias, self.c_proj.weight, self.c_proj.bias, expert_frequency,
                self.c_fc.N_array, self.c_fc.K_array, self.c_proj.N_array, self.c_proj.K_array,
            )  # fmt: skip
            return combine(hidden_states, router_weights, inverse)

        if self.fuse_swiglu and hidden_states.dtype in (torch.bfloat16, torch.float16):
            hidden_states = self.c_fc.cuda_forward_swiglu(input=hidden_states, expert_frequency=expert_frequency)
        else:
            hidden_states = self.c_fc.cuda_forward(input=hidden_states, expert_frequency=expert_frequency)
            hidden_states = self.act(hidden_states)

        hidden_states = self.c_proj.cuda_forward(input=hidden_states, expert_frequency=expert_frequency)

        # y[t] = sum_j router_weights[t, j] * expert_output[row of slot (t, j)]
        hidden_states = combine(hidden_states, router_weights, inverse)

        return hidden_states

    def _runs_swiglu_experts_as_one_node(self, hidden_states: torch.Tensor) -> bool:
        """fuse_swiglu_backward: with the fused SwiGLU up-projection, run the second projection in the same autograd node
        so that its input gradient and the activation's backward are one kernel (16-bit types; the sizes that kernel takes)"""
        return (
            self.fuse_swiglu
            and self.fuse_swiglu_backward
            and hidden_states.dtype in (torch.bfloat16, torch.float16)
            and self.c_proj.weight.dtype == hidden_states.dtype
            and self.c_fc.weight.dtype == hidden_states.dtype
            and (self.c_fc.bias is None or self.c_fc.bias.dtype == hidden_states.dtype)
            and (self.c_proj.bias is None or self.c_proj.bias.dtype == hidden_states.dtype)
            and self.intermediate_size < (1 << 22)
            and self.hidden_size < (1 << 21)
        )

    def _gathers_inside_gemm(self, hidden_states: torch.Tensor) -> bool:
        """Whether the first projection (forward and weight gradient) gathers its rows itself instead of reading a grouped
        copy of the tokens. gather_in_gemm None: when the projection is narrow enough for the saved row-movement pass to
        outweigh the slower operand fetch of scattered rows (measured: 1 to 5 % of the forward product and -2 to +4 % of the
        weight-gradient product, against one pass that reads T and writes T * top_k rows); True / False force it."""
        if self.gather_in_gemm is False or not can_gather_inside_gemm(hidden_states, self.c_fc.weight, self.c_fc.bias):
            return False
        if self.gather_in_gemm:
            return True
        return self.c_fc.out_features <= 6144

    def _get_topk(self, x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        if self.top_k == 1:
            x, indices = x.max(dim=-1, keepdim=True)
        else:
            x, indices = x.topk(self.top_k, dim=-1)

        return x, indices
