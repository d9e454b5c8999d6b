"""GPU parity of fused_residual_add_rmsnorm (forward and backward through the C ABI) against the oracle.

The fp32 cases restate the reference's test (tests/ops/fused_residual_add_rmsnorm_test.py:20-96): sizes (H,) and
(400, H) over powers of two, their neighbours and odd lengths, with and without weight / multiplier / cached
denominator, loss = sum(2 * out + 3 * residual_out), absolute tolerances 1.4e-4 (combined output), 1.5e-4 (x grad),
1.6e-4 (residual grad), 1.1e-4 (weight grad), rtol 0.
"""

import pytest
import torch

from fma import KernelBackend, fused_residual_add_rmsnorm
from oracle import moe_oracle as O

from gpu_util import DEV, rel_err

pytestmark = pytest.mark.gpu

_EPSILON = 1e-5

# the reference draws its lengths from 2^i + j (i < 15, j < 10) and 50 random values around 3000; a spread of those,
# chosen to reach every kernel variant: rows below one vector, unaligned rows, 1 / 2 / 4 / 8 vectors per thread, and
# rows too long for the register kernels
HIDDEN = [1, 2, 3, 5, 8, 9, 16, 23, 64, 73, 128, 137, 512, 1024, 1031, 2048, 2052, 2391, 3000, 3608, 4096, 4100, 8192, 8200, 16384, 16393]


def _run_case(size, dtype, memory_efficient, has_weight, multiplier, function=fused_residual_add_rmsnorm):
    torch.manual_seed(42)
    x = torch.randn(size, dtype=dtype)
    residual = torch.randn(size, dtype=dtype)
    weight = torch.randn(size[-1], dtype=dtype) if has_weight else None

    leaves = [t.clone().to(DEV).requires_grad_() if t is not None else None for t in (x, residual, weight)]
    z, r = function(
        x=leaves[0], residual=leaves[1], weight=leaves[2], eps=_EPSILON, multiplier=multiplier, memory_efficient=memory_efficient
    )
    combined = z * 2 + r * 3
    combined.sum().backward()
    return (x, residual, weight), leaves, combined, (z, r)


@pytest.mark.parametrize("H", HIDDEN)
@pytest.mark.parametrize("rows", [None, 400])
@pytest.mark.parametrize("memory_efficient", [True, False])
@pytest.mark.parametrize("has_weight", [True, False])
@pytest.mark.parametrize("multiplier", [None, 0.9])
def test_reference_cases_fp32(H, rows, memory_efficient, has_weight, multiplier):
    size = (H,) if rows is None else (rows, H)
    inputs, leaves, combined, _ = _run_case(size, torch.float32, memory_efficient, has_weight, multiplier)

    ref = [t.clone().requires_grad_() if t is not None else None for t in inputs]
    z, r = O.fused_residual_add_rmsnorm(ref[0], ref[1], ref[2], _EPSILON, multiplier)
    expected = z * 2 + r * 3
    expected.sum().backward()

    def close(a, b, atol, what):
        err = float((a.detach().cpu() - b.detach()).abs().max())
        assert err <= atol, f"{what}: {err}"

    close(combined, expected, 1.4e-4, "output")
    close(leaves[0].grad, ref[0].grad, 1.5e-4, "x grad")
    close(leaves[1].grad, ref[1].grad, 1.6e-4, "residual grad")
    if has_weight:
        close(leaves[2].grad, ref[2].grad, 1.1e-4, "weight grad")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("size", [(7, 64), (400, 1031), (400, 2048), (300, 4096), (64, 8192), (33, 16384), (9, 20000), (5, 3)])
@pytest.mark.parametrize("memory_efficient", [True, False])
@pytest.mark.parametrize("multiplier", [None, 0.9])
def test_sixteen_bit_against_fp64(dtype, size, memory_efficient, multiplier):
    eps_dtype = {torch.float16: 2.0**-10, torch.bfloat16: 2.0**-7}[dtype]
    inputs, leaves, _, (z, r) = _run_case(size, dtype, memory_efficient, True, multiplier)
    ref = [t.double().requires_grad_() for t in inputs]
    z64, r64 = O.fused_residual_add_rmsnorm(ref[0], ref[1], ref[2], _EPSILON, multiplier)
    (z64 * 2 + r64 * 3).sum().backward()

    # forward: one rounding of a value computed in fp32
    assert bool(((r.detach().cpu().double() - r64).abs() <= 0.5 * eps_dtype * r64.abs() * 1.001 + 1e-6).all())
    assert bool(((z.detach().cpu().double() - z64).abs() <= 0.5 * eps_dtype * z64.abs() * 1.001 + 1e-5).all())
    # backward: the kernel starts from the ROUNDED residual stream (as the reference's does); against the exact
    # gradient that is a relative perturbation of the order of the dtype's spacing
    for name, a, b in [("x grad", leaves[0].grad, ref[0].grad), ("residual grad", leaves[1].grad, ref[1].grad)]:
        max_rel, frob_rel = rel_err(a, b)
        assert max_rel <= 2 * eps_dtype and frob_rel <= eps_dtype, f"{name}: {max_rel:.3g} {frob_rel:.3g}"
    max_rel, frob_rel = rel_err(leaves[2].grad, ref[2].grad)
    assert max_rel <= 2 * eps_dtype and frob_rel <= 2 * eps_dtype, f"weight grad: {max_rel:.3g} {frob_rel:.3g}"


def test_transformer_block_shape_and_determinism():
    # the residual stream of the Mixtral-like benchmark layer: T = 16384 tokens of 4096, bf16
    torch.manual_seed(0)
    T, H = 16384, 4096
    x = torch.randn(T, H, device=DEV).bfloat16().requires_grad_()
    res = torch.randn(T, H, device=DEV).bfloat16().requires_grad_()
    w = (1 + 0.1 * torch.randn(H, device=DEV)).bfloat16().requires_grad_()
    dz = torch.randn(T, H, device=DEV).bfloat16()
    dr = torch.randn(T, H, device=DEV).bfloat16()

    grads = []
    for _ in range(2):
        x.grad = res.grad = w.grad = None
        z, r = fused_residual_add_rmsnorm(x, res, w, _EPSILON)
        torch.autograd.backward([z, r], [dz, dr])
        grads.append((x.grad.clone(), res.grad.clone(), w.grad.clone()))
    # fixed summation order: the weight gradient is the same bits on every run (the reference's atomics are not)
    assert all(torch.equal(a, b) for a, b in zip(*grads))

    # the same computation by library calls on the GPU, in fp32 from the same bf16 inputs
    xf, rf, wf = (t.detach().float().requires_grad_() for t in (x, res, w))
    zf, rr = O.fused_residual_add_rmsnorm(xf, rf, wf, _EPSILON)
    torch.autograd.backward([zf, rr], [dz.float(), dr.float()])
    assert rel_err(z, zf)[0] <= 2.0**-8 and rel_err(r, rr)[0] <= 2.0**-8
    for a, b in zip(grads[0], (xf.grad, rf.grad, wf.grad)):
        max_rel, frob_rel = rel_err(a, b)
        assert max_rel <= 2.0**-6 and frob_rel <= 2.0**-7, f"{max_rel:.3g} {frob_rel:.3g}"
    # unit root-mean-square before the weight
    rms = (z.detach().float() / w.detach().float()).pow(2).mean(-1).sqrt()
    assert float((rms - 1).abs().max()) < 2e-2


def test_only_one_output_used_and_no_weight():
    torch.manual_seed(1)
    x = torch.randn(50, 256, device=DEV).requires_grad_()
    res = torch.randn(50, 256, device=DEV).requires_grad_()
    for use in (0, 1):
        x.grad = res.grad = None
        outs = fused_residual_add_rmsnorm(x, res, None, _EPSILON, multiplier=0.5)
        outs[use].sum().backward()
        xr, rr = x.detach().cpu().clone().requires_grad_(), res.detach().cpu().clone().requires_grad_()
        O.fused_residual_add_rmsnorm(xr, rr, None, _EPSILON, 0.5)[use].sum().backward()
        assert float((x.grad.cpu() - xr.grad).abs().max()) <= 1.5e-4
        assert float((res.grad.cpu() - rr.grad).abs().max()) <= 1.6e-4


def test_compiled_matches_eager():
    torch.manual_seed(2)
    x = torch.randn(400, 1024, device=DEV).requires_grad_()
    res = torch.randn(400, 1024, device=DEV).requires_grad_()
    w = torch.randn(1024, device=DEV).requires_grad_()
    ze, re_ = fused_residual_add_rmsnorm(x, res, w, _EPSILON, multiplier=0.9)
    (ze * 2 + re_ * 3).sum().backward()
    eager = (ze.detach().clone(), x.grad.clone(), w.grad.clone())
    x.grad = res.grad = w.grad = None
    zc, rc = torch.compile(fused_residual_add_rmsnorm, fullgraph=True)(x, res, w, _EPSILON, multiplier=0.9)
    (zc * 2 + rc * 3).sum().backward()
    assert torch.equal(zc, eager[0]) and torch.equal(x.grad, eager[1]) and torch.equal(w.grad, eager[2])


def test_rejects_what_it_does_not_implement():
    x = torch.randn(4, 8, device=DEV)
    with pytest.raises(ValueError):
        fused_residual_add_rmsnorm(x, x, None, _EPSILON, kernel_backend=KernelBackend.torch)
    with pytest.raises(RuntimeError):
        fused_residual_add_rmsnorm(x.cpu(), x.cpu(), None, _EPSILON)
    with pytest.raises(AssertionError):
        fused_residual_add_rmsnorm(x, x, torch.randn(8, device=DEV).double(), _EPSILON)
    # eps=None is the dtype's machine epsilon (fma/ops/fused_residual_add_rmsnorm/__init__.py:35-36)
    a = fused_residual_add_rmsnorm(x, x, None, None)[0]
    b = fused_residual_add_rmsnorm(x, x, None, torch.finfo(torch.float32).eps)[0]
    assert torch.equal(a, b)
