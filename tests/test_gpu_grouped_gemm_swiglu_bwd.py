"""GPU parity of fma_grouped_gemm_swiglu_bwd (input gradient of the second expert projection with the backward of SwiGLU in
its epilogue) against the two launches it replaces: the NN grouped GEMM, then swiglu_backward on the halves of h. Same bits."""

import pytest
import torch

from fma import _lib
from fma.modules.moe.cuda_implementation import grouped_gemm_ragged_cuda, grouped_gemm_swiglu_bwd_cuda
from fma.ops.swiglu.cuda_implementation import swiglu_backward_cuda

from gpu_util import DEV

pytestmark = pytest.mark.gpu


def _u32(values):
    return torch.tensor(values, dtype=torch.int64).to(torch.uint32).to(DEV)


def _two_launches(dy, w, h, M, inter):
    R, K = dy.shape
    da = torch.empty(R, inter, dtype=dy.dtype, device=DEV)
    grouped_gemm_ragged_cuda(dy, w, da, M, False, 0, inter, K, False, False)
    dh = torch.full_like(h, 7.0)
    up, gate = h.chunk(2, dim=-1)
    up_grad, gate_grad = dh.chunk(2, dim=-1)
    swiglu_backward_cuda(gate=gate, up=up, output_grad=da, gate_grad=gate_grad, up_grad=up_grad, BLOCK_SIZE=1024)
    return dh


CASES = [
    # rows per expert, I, K (= the layer's hidden size)
    ([2048 + 8 * (e % 7) for e in range(24)], 512, 512),  # every workgroup streams through several tiles
    ([1500, 0, 264, 8, 3000, 40, 777 * 8], 384, 192),  # 3 K steps, small and empty groups between
    ([520] * 40, 256, 64),  # one K step per tile
    ([300, 5000, 16, 16, 16, 2000], 136, 1088),  # 17 K steps; a last column tile of 8 columns
    ([1000, 1003, 2000], 72, 136),  # columns end inside a wavefront's 64; a partial last K step
    ([1], 8, 8),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("counts,inter,K", CASES)
def test_equals_gemm_then_swiglu_backward(counts, inter, K, dtype):
    g = torch.Generator(device=DEV).manual_seed(inter + K)
    R, E = sum(counts), len(counts)
    dy = torch.randn(R, K, device=DEV, generator=g).to(dtype)
    w = (torch.randn(E, K, inter, device=DEV, generator=g) * 0.1).to(dtype)
    h = (torch.randn(R, 2 * inter, device=DEV, generator=g) * 2).to(dtype)
    M = _u32(counts)
    expect = _two_launches(dy, w, h, M, inter)
    for _ in range(2):
        got = torch.full_like(h, 7.0)
        grouped_gemm_swiglu_bwd_cuda(dy, w, h, M, got)
        assert torch.equal(got, expect)


def test_extreme_gates():
    # saturated sigmoids, zeros and negative zeros in h: the same bits as the standalone kernel
    counts, inter, K = [300, 77], 64, 128
    g = torch.Generator(device=DEV).manual_seed(1)
    R = sum(counts)
    dy = torch.randn(R, K, device=DEV, generator=g).bfloat16()
    w = (torch.randn(2, K, inter, device=DEV, generator=g) * 0.1).bfloat16()
    h = (torch.randn(R, 2 * inter, device=DEV, generator=g) * 60).bfloat16()
    h[::7] = 0.0
    h[1::7] = -0.0
    h[2::7, inter:] = 200.0
    h[3::7, inter:] = -200.0
    M = _u32(counts)
    got = torch.empty_like(h)
    grouped_gemm_swiglu_bwd_cuda(dy, w, h, M, got)
    assert torch.equal(got, _two_launches(dy, w, h, M, inter))


def test_argument_validation():
    lib = _lib.load()
    p = torch.zeros(4096, dtype=torch.bfloat16, device=DEV).data_ptr()
    m = _u32([8]).data_ptr()
    call = lib.fma_grouped_gemm_swiglu_bwd
    assert call(p, p, p, p, m, 1, 12, 16, _lib.FMA_BF16, None) == -3  # I % 8
    assert call(p, p, p, p, m, 1, 16, 12, _lib.FMA_BF16, None) == -3  # K % 8
    assert call(p, p, None, p, m, 1, 16, 16, _lib.FMA_BF16, None) == -1
    assert call(p, p, p, p + 2, m, 1, 16, 16, _lib.FMA_BF16, None) == -6
    assert call(p, p, p, p, m, 1, 16, 16, _lib.FMA_F32, None) != 0
    assert call(p, p, p, p, m, 0, 16, 16, _lib.FMA_BF16, None) == 0


@pytest.mark.parametrize("add_bias", [False, True])
@pytest.mark.parametrize("E,k,H,I,T", [(8, 2, 256, 512, 300), (64, 8, 128, 72, 1000)])
def test_layer_with_the_activation_backward_inside_the_gemm(E, k, H, I, T, add_bias):
    # the layer with its two projections as one autograd node (d_h from one kernel) and as two nodes with swiglu_backward
    # between them: the same bits in the output and in every gradient
    from fma import KernelBackend, MoE, swiglu_packed

    torch.manual_seed(E + I)
    moe = MoE(E, k, H, I, swiglu_packed, True, add_bias, 0.02).to(torch.bfloat16).to(DEV)
    if add_bias:
        with torch.no_grad():
            moe.c_fc.bias.normal_(0, 0.5)
            moe.c_proj.bias.normal_(0, 0.5)
    x = torch.randn(T, H, device=DEV).bfloat16()
    dy = torch.randn(T, H, device=DEV).bfloat16()
    results = []
    for fused in (False, True):
        moe.fuse_swiglu_backward = fused
        assert moe._runs_swiglu_experts_as_one_node(x) == fused
        moe.zero_grad()
        xi = x.clone().requires_grad_()
        y, _ = moe(xi, kernel_backend=KernelBackend.cuda)
        y.backward(dy)
        results.append([y.detach(), xi.grad] + [p.grad.clone() for p in moe.parameters()])
    for a, b in zip(*results):
        assert torch.equal(a, b)
