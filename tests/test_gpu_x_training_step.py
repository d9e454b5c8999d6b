"""End-to-end use of the path as a transformer block would use it: residual add + RMSNorm, the MoE layer (router included)
and the residual connection, trained for a few optimiser steps on a fixed regression target. Every gradient of the block
flows through the HIP kernels (norm weight, gate, both expert projections), so a wrong sign or a missing term anywhere
shows up as a loss that does not fall."""

import pytest
import torch

from fma import KernelBackend, MoE, fused_residual_add_rmsnorm, swiglu_packed

from gpu_util import DEV

pytestmark = pytest.mark.gpu


class _Block(torch.nn.Module):
    def __init__(self, E, k, H, I, add_bias):
        super().__init__()
        self.norm_weight = torch.nn.Parameter(torch.ones(H))
        self.moe = MoE(E, k, H, I, swiglu_packed, True, add_bias, 0.05)

    def forward(self, x, residual):
        normed, residual = fused_residual_add_rmsnorm(x, residual, self.norm_weight, 1e-5)
        y, router_logits = self.moe(normed, kernel_backend=KernelBackend.cuda)
        return y + residual, router_logits


@pytest.mark.parametrize("dtype,add_bias,factor", [(torch.float32, False, 0.1), (torch.float32, True, 0.1), (torch.bfloat16, False, 0.1)])
def test_block_trains(dtype, add_bias, factor):
    torch.manual_seed(3)
    T, H, I, E, k = 512, 128, 256, 8, 2
    block = _Block(E, k, H, I, add_bias).to(DEV)
    x = torch.randn(T, H, device=DEV)
    residual = torch.randn(T, H, device=DEV)
    target = torch.tanh(x @ torch.randn(H, H, device=DEV) / H**0.5) + residual
    # fp32 master parameters; the block runs in `dtype`
    optimiser = torch.optim.Adam(block.parameters(), lr=3e-3)
    losses = []
    for _ in range(40):
        optimiser.zero_grad(set_to_none=True)
        if dtype == torch.float32:
            out, logits = block(x, residual)
        else:
            with torch.no_grad():
                shadow = _Block(E, k, H, I, add_bias).to(DEV).to(dtype)
                shadow.load_state_dict({n: (p.to(dtype) if p.is_floating_point() else p) for n, p in block.state_dict().items()})
            for p in shadow.parameters():
                p.requires_grad_()
            out, logits = shadow(x.to(dtype), residual.to(dtype))
        # a small auxiliary term on the router logits, as load-balancing losses add: exercises the logits' own gradient
        loss = (out.float() - target).pow(2).mean() + 1e-3 * logits.float().pow(2).mean()
        loss.backward()
        if dtype != torch.float32:
            for (_, p), (_, q) in zip(block.named_parameters(), shadow.named_parameters()):
                p.grad = q.grad.float()
        assert all(p.grad is not None and bool(torch.isfinite(p.grad).all()) for p in block.parameters())
        optimiser.step()
        losses.append(float(loss.detach()))
    assert losses[-1] < factor * losses[0], f"loss went from {losses[0]:.4f} to {losses[-1]:.4f}"
    assert losses[-1] == min(losses[-5:]) or losses[-1] < 1.05 * min(losses), losses[-5:]
