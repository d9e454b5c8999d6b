"""GPU parity of the row-movement kernels (gather, combine, combine backward) and of SwiGLU forward / backward."""

import numpy as np
import pytest
import torch

from fma import KernelBackend, swiglu, swiglu_packed
from fma.modules.moe.cuda_implementation import build_routing_index, combine, gather_rows, gather_rows_cuda
from oracle import moe_oracle as O
from synthetic_inputs import make_routing

from gpu_util import DEV, rel_err

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize(
    "T,H,E,k",
    [(7, 64, 4, 2), (300, 4096, 8, 2), (257, 2048, 64, 8), (100, 576, 128, 8), (33, 8, 3, 1),
     (33, 4, 3, 1), (64, 13, 17, 1), (50, 1, 4, 2), (40, 1001, 8, 3)],  # rows that are not whole 16-byte pieces: element-wise kernels
)
def test_gather_is_bit_exact(dtype, T, H, E, k):
    torch.manual_seed(T)
    x = torch.randn(T, H).to(dtype)
    selected, _ = make_routing(T, E, k, "uniform", seed=1)
    idx = O.routing_index(selected.numpy(), E)
    _, _, perm, _, inv = build_routing_index(selected.to(DEV), E)
    got = gather_rows(x.to(DEV), perm, inv, k).cpu()  # token-side form (fma_dispatch_rows)
    expect = x[torch.from_numpy(idx["perm"].astype(np.int64)) // k]  # fma/modules/moe/__init__.py:269,275
    assert torch.equal(got, expect)
    out = torch.empty(T * k, H, dtype=dtype, device=DEV)  # row-side form (fma_gather_rows)
    gather_rows_cuda(x.to(DEV), perm, k, out)
    assert torch.equal(out.cpu(), expect)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize(
    "T,H,E,k",
    [(7, 64, 4, 2), (300, 4096, 8, 2), (257, 2048, 64, 8), (64, 576, 128, 8), (50, 128, 16, 5),
     (64, 13, 17, 1), (50, 1, 4, 2), (40, 1001, 8, 3), (9, 700, 16, 6)],  # element-wise kernels, cached and re-read dy rows
)
def test_combine_forward_and_backward(dtype, T, H, E, k):
    torch.manual_seed(T + k)
    selected, gates = make_routing(T, E, k, "uniform", seed=2)
    idx = O.routing_index(selected.numpy(), E)
    perm = torch.from_numpy(idx["perm"].astype(np.int64))
    o = torch.randn(T * k, H).to(dtype)
    gates = gates.to(dtype)
    dy = torch.randn(T, H).to(dtype)

    # oracle: scale by the gathered gates, index_add by token (fma/modules/moe/__init__.py:284-286), in fp64
    o64 = o.double().requires_grad_()
    g64 = gates.double().requires_grad_()
    y64 = torch.zeros(T, H, dtype=torch.float64).index_add(0, perm // k, o64 * g64.flatten()[perm].unsqueeze(-1))
    y64.backward(dy.double())

    _, _, _, _, inv = build_routing_index(selected.to(DEV), E)
    o_d = o.to(DEV).requires_grad_()
    g_d = gates.to(DEV).requires_grad_()
    y = combine(o_d, g_d, inv)
    y.backward(dy.to(DEV))

    # one rounding of an fp32-accumulated sum: half an ulp of the output dtype, relative to the largest value
    eps = {torch.float32: 1e-6, torch.float16: 1e-3, torch.bfloat16: 8e-3}[dtype]
    assert rel_err(y, y64.detach())[0] <= eps
    assert rel_err(o_d.grad, o64.grad)[0] <= eps
    assert rel_err(g_d.grad, g64.grad)[0] <= eps


def test_combine_k1_unit_gate_is_the_inverse_permutation():
    T, H, E = 129, 256, 8
    torch.manual_seed(0)
    x = torch.randn(T, H).bfloat16().to(DEV)
    selected, _ = make_routing(T, E, 1, "uniform", seed=3)
    _, _, perm, _, inv = build_routing_index(selected.to(DEV), E)
    xg = gather_rows(x, perm, inv, 1)
    back = combine(xg, torch.ones(T, 1, dtype=torch.bfloat16, device=DEV), inv)
    assert torch.equal(back, x)


def _sizes_2d():
    sizes = [(2**i + j, 2**i + j) for i in range(0, 12, 2) for j in range(2)]
    return sizes + [(3001, 2999), (2048, 4096), (7, 28672)]


@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu_forward_backward(dtype):
    # the reference's test (tests/ops/swiglu_test.py:16-46): mean() loss, fp32 atol 5.5e-6 / 5e-6, rtol 0;
    # fp16 / bf16: torch.testing.assert_close defaults
    for size in _sizes_2d():
        torch.manual_seed(size[0])
        g_ref = torch.randn(size).to(dtype).requires_grad_()
        u_ref = torch.randn(size).to(dtype).requires_grad_()
        z_ref = O.swiglu(g_ref, u_ref)
        z_ref.mean().backward()
        g = g_ref.detach().to(DEV).requires_grad_()
        u = u_ref.detach().to(DEV).requires_grad_()
        z = swiglu(g, u, kernel_backend_forward=KernelBackend.cuda, kernel_backend_backward=KernelBackend.cuda)
        z.mean().backward()
        if dtype == torch.float32:
            torch.testing.assert_close(z.cpu(), z_ref, atol=5.5e-6, rtol=0)
            torch.testing.assert_close(g.grad.cpu(), g_ref.grad, atol=5e-6, rtol=0)
            torch.testing.assert_close(u.grad.cpu(), u_ref.grad, atol=5e-6, rtol=0)
        else:
            torch.testing.assert_close(z.cpu(), z_ref)
            torch.testing.assert_close(g.grad.cpu(), g_ref.grad)
            torch.testing.assert_close(u.grad.cpu(), u_ref.grad)


@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu_packed(dtype):
    for size in [(1, 2), (5, 6), (129, 258), (1000, 2816), (64, 28672), (3, 4, 16)]:
        torch.manual_seed(size[-1])
        x_ref = torch.randn(size).to(dtype).requires_grad_()
        z_ref = O.swiglu_packed(x_ref)
        z_ref.mean().backward()
        x = x_ref.detach().to(DEV).requires_grad_()
        z = swiglu_packed(x)
        z.mean().backward()
        if dtype == torch.float32:
            torch.testing.assert_close(z.cpu(), z_ref, atol=5.5e-6, rtol=0)
            torch.testing.assert_close(x.grad.cpu(), x_ref.grad, atol=5e-6, rtol=0)
        else:
            torch.testing.assert_close(z.cpu(), z_ref)
            torch.testing.assert_close(x.grad.cpu(), x_ref.grad)


def test_swiglu_saturation_and_closed_forms():
    g = torch.tensor([0.0, 100.0, -100.0, 1e4, -1e4, 88.0, -88.0], device=DEV)
    u = torch.full_like(g, 2.0)
    y = swiglu(g, u).cpu()
    assert y[0] == 0 and y[1] == 200.0 and abs(float(y[2])) < 1e-30 and y[3] == 2e4 and abs(float(y[4])) < 1e-30  # the clamp keeps sigmoid(-1e4) at sigmoid(-88.376) > 0
    assert torch.isfinite(y).all()
