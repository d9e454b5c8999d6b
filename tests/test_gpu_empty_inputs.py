"""Calls without elements: every op of the path on tensors with zero rows, and the whole layer with zero tokens, forward
and backward (torch's own ops accept these and return empty results and zero parameter gradients; an empty tensor has no
device address, so each wrapper has to return before it would hand one to the library)."""

import pytest
import torch

from fma import KernelBackend, MoE, continuous_count, fused_residual_add_rmsnorm, swiglu, swiglu_packed

from gpu_util import DEV

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.int32, torch.int64])
def test_continuous_count_of_nothing(dtype):
    # torch.bincount(empty, minlength=8) is eight zeros (the reference's torch branch, fma/ops/continuous_count/__init__.py:38-39)
    out = continuous_count(x=torch.empty(0, dtype=dtype, device=DEV), size=8)
    assert out.dtype == torch.uint32 and out.tolist() == [0] * 8


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_swiglu_without_rows(dtype):
    gate = torch.empty(0, 64, device=DEV, dtype=dtype, requires_grad=True)
    up = torch.empty(0, 64, device=DEV, dtype=dtype, requires_grad=True)
    z = swiglu(gate, up)
    z.sum().backward()
    assert z.shape == (0, 64) and gate.grad.shape == (0, 64) and up.grad.shape == (0, 64)
    x = torch.empty(0, 128, device=DEV, dtype=dtype, requires_grad=True)
    z = swiglu_packed(x)
    z.sum().backward()
    assert z.shape == (0, 64) and x.grad.shape == (0, 128)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_residual_add_rmsnorm_without_rows(dtype):
    x = torch.empty(0, 64, device=DEV, dtype=dtype, requires_grad=True)
    residual = torch.empty(0, 64, device=DEV, dtype=dtype, requires_grad=True)
    weight = torch.ones(64, device=DEV, dtype=dtype, requires_grad=True)
    y, r = fused_residual_add_rmsnorm(x, residual, weight, 1e-5)
    (y.sum() + r.sum()).backward()
    assert y.shape == (0, 64) and r.shape == (0, 64) and x.grad.shape == (0, 64) and residual.grad.shape == (0, 64)
    assert weight.grad.shape == (64,) and float(weight.grad.abs().sum()) == 0.0


@pytest.mark.parametrize("add_bias", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_layer_without_tokens(dtype, add_bias):
    # 16-bit without bias takes the fused router and the fused SwiGLU epilogue, with bias the unfused chain, fp32 the
    # ATen router and the fp32 GEMM
    moe = MoE(8, 2, 64, 128, swiglu_packed, True, add_bias, 0.02).to(DEV).to(dtype)
    x = torch.empty(0, 64, device=DEV, dtype=dtype, requires_grad=True)
    y, logits = moe(x, kernel_backend=KernelBackend.cuda)
    assert y.shape == (0, 64) and logits.shape == (0, 8) and y.dtype == dtype
    (y.sum() + logits.sum()).backward()
    assert x.grad.shape == (0, 64)
    for name, p in moe.named_parameters():
        assert p.grad is not None and p.grad.shape == p.shape and float(p.grad.abs().sum()) == 0.0, name
