"""The reference runs every op of this path under torch.compile(fullgraph=True) as well (e.g.
tests/ops/continuous_count_test.py:25, grouped_gemm_test.py:25, swiglu_test.py:22, modules/moe_test.py:97-98): the
custom ops must trace without graph breaks and give the eager results."""

import pytest
import torch

from fma import KernelBackend, MoE, continuous_count, fused_residual_add_rmsnorm, grouped_gemm, swiglu, swiglu_packed
from oracle import moe_oracle as O

from gpu_util import DEV, to_np

pytestmark = pytest.mark.gpu


def test_continuous_count_compiled():
    f = torch.compile(continuous_count, fullgraph=True)
    for n in (1, 1000, 100_003):
        torch.manual_seed(42)
        x = torch.randint(0, 72, (n,))
        assert (to_np(f(x=x.to(DEV), size=72)) == O.continuous_count(x.numpy(), 72)).all()


def test_swiglu_compiled():
    torch.manual_seed(0)
    g_ref = torch.randn(65, 130).requires_grad_()
    u_ref = torch.randn(65, 130).requires_grad_()
    O.swiglu(g_ref, u_ref).mean().backward()
    g, u = g_ref.detach().to(DEV).requires_grad_(), u_ref.detach().to(DEV).requires_grad_()
    z = torch.compile(swiglu, fullgraph=True)(g, u)
    z.mean().backward()
    torch.testing.assert_close(z.cpu(), O.swiglu(g_ref, u_ref), atol=5.5e-6, rtol=0)
    torch.testing.assert_close(g.grad.cpu(), g_ref.grad, atol=5e-6, rtol=0)
    torch.testing.assert_close(u.grad.cpu(), u_ref.grad, atol=5e-6, rtol=0)

    x_ref = torch.randn(33, 258).requires_grad_()
    O.swiglu_packed(x_ref).mean().backward()
    x = x_ref.detach().to(DEV).requires_grad_()
    zp = torch.compile(swiglu_packed, fullgraph=True)(x)
    zp.mean().backward()
    torch.testing.assert_close(zp.cpu(), O.swiglu_packed(x_ref), atol=5.5e-6, rtol=0)
    torch.testing.assert_close(x.grad.cpu(), x_ref.grad, atol=5e-6, rtol=0)


def test_grouped_gemm_compiled():
    g = torch.Generator().manual_seed(42)
    M_list, N, K = [40, 0, 264], 72, 136
    A = torch.cat([torch.randint(-8, 9, (m * K,), generator=g) for m in M_list]).bfloat16()
    B = torch.cat([torch.randint(-8, 9, (N * K,), generator=g) for _ in M_list]).bfloat16()
    u32 = lambda v: torch.tensor(v, dtype=torch.int64).to(torch.uint32).to(DEV)
    out = torch.compile(grouped_gemm, fullgraph=True)(
        A=A.to(DEV), B=B.to(DEV), C=None, M_array=u32(M_list), N_array=u32([N] * 3), K_array=u32([K] * 3),
        output_shape=(sum(M_list) * N,), is_A_transposed=False, is_B_transposed=True,
    )
    assert torch.equal(out.cpu(), O.grouped_gemm(A, B, M_list, [N] * 3, [K] * 3, False, True))


def test_moe_compiled_matches_eager():
    torch.manual_seed(42)
    moe = MoE(8, 2, 256, 512, swiglu_packed, True, False, 0.02).to(torch.bfloat16).to(DEV)
    x = torch.randn(7, 256).bfloat16().to(DEV)
    xe, xc = x.clone().requires_grad_(), x.clone().requires_grad_()
    ye = moe(xe, kernel_backend=KernelBackend.cuda)[0]
    ye.sum().backward()
    grads_e = {k: p.grad.clone() for k, p in moe.named_parameters()}
    moe.zero_grad()
    yc = torch.compile(moe, fullgraph=True)(xc, kernel_backend=KernelBackend.cuda)[0]
    yc.sum().backward()
    assert torch.equal(yc, ye)
    # Inductor fuses the ATen glue around the custom ops (the loss, dtype casts, the matrix products of the router's
    # backward) and rounds it differently in bf16; the custom ops themselves see identical inputs
    torch.testing.assert_close(xc.grad, xe.grad, rtol=1.6e-2, atol=2e-3)
    for k, p in moe.named_parameters():
        torch.testing.assert_close(p.grad, grads_e[k], rtol=1.6e-2, atol=2e-3, msg=k)


class _Block(torch.nn.Module):
    def __init__(self, E, k, H, I, add_bias, activation, is_glu):
        super().__init__()
        self.norm_weight = torch.nn.Parameter(torch.ones(H))
        self.moe = MoE(E, k, H, I, activation, is_glu, add_bias, 0.05)

    def forward(self, x, residual):
        normed, residual = fused_residual_add_rmsnorm(x, residual, self.norm_weight, 1e-5)
        y, router_logits = self.moe(normed, kernel_backend=KernelBackend.cuda)
        return y + residual, router_logits


@pytest.mark.parametrize(
    "dtype,add_bias,activation,is_glu",
    [
        (torch.bfloat16, False, swiglu_packed, True),  # fused router, fused SwiGLU epilogue
        (torch.bfloat16, True, swiglu_packed, True),  # fused router, GEMM + in-place bias + activation
        (torch.bfloat16, False, torch.nn.GELU(approximate="tanh"), False),
        (torch.float32, True, swiglu_packed, True),  # ATen router, fp32 GEMM
    ],
)
def test_block_compiled_matches_eager(dtype, add_bias, activation, is_glu):
    # residual add + RMSNorm, the layer with its router, the residual connection: one graph without breaks, forward and
    # backward, against the eager run of the same modules
    torch.manual_seed(0)
    block = _Block(8, 2, 64, 128, add_bias, activation, is_glu).to(DEV).to(dtype)
    x = torch.randn(50, 64, device=DEV).to(dtype)
    residual = torch.randn(50, 64, device=DEV).to(dtype)

    def step(f):
        block.zero_grad(set_to_none=True)
        xa, ra = x.clone().requires_grad_(), residual.clone().requires_grad_()
        out, logits = f(xa, ra)
        (out.float().pow(2).mean() + logits.float().pow(2).mean()).backward()
        return [out.detach(), logits.detach(), xa.grad, ra.grad] + [p.grad.clone() for p in block.parameters()]

    eager = step(block)
    compiled = step(torch.compile(block, fullgraph=True))
    bar = 1.6e-2 if dtype == torch.bfloat16 else 1e-5  # two bf16 ulps of the largest value for the re-fused glue
    for a, b in zip(eager, compiled):
        assert float((a.float() - b.float()).abs().max()) <= bar * float(a.float().abs().max())
