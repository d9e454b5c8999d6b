"""The layer as callers hand it things: views that are not contiguous, inputs with a batch dimension, every expert
selected (top_k == E) or a single expert, parameters that are frozen, and calls under no_grad / inference_mode. The
reference makes operands contiguous at the autograd boundary (fma/utils/contiguous.py), flattens the leading dimensions
(fma/modules/moe/__init__.py:167-189) and lets autograd skip what needs no gradient."""

import pytest
import torch

from fma import KernelBackend, MoE, swiglu_packed

from gpu_util import DEV

pytestmark = pytest.mark.gpu


def _step(moe, x):
    x = x.detach().requires_grad_()
    moe.zero_grad(set_to_none=True)
    y, logits = moe(x, kernel_backend=KernelBackend.cuda)
    (y.float().pow(2).sum() + logits.float().sum()).backward()
    return y.detach(), logits.detach(), x.grad, {n: p.grad.clone() for n, p in moe.named_parameters() if p.grad is not None}


def _assert_same(a, b, what):
    assert a.shape == b.shape and torch.equal(a, b), f"{what}: max diff {float((a.float() - b.float()).abs().max())}"


def test_views_that_are_not_contiguous():
    # bf16: the router is this library's kernel too, so the whole step has to be bit-identical to the contiguous call
    torch.manual_seed(1)
    moe = MoE(8, 2, 64, 128, swiglu_packed, True, False, 0.02).to(DEV).to(torch.bfloat16)
    for view in (torch.randn(33, 128, device=DEV).bfloat16()[:, ::2], torch.randn(64, 33, device=DEV).bfloat16().t()):
        assert not view.is_contiguous()
        ref, got = _step(moe, view.contiguous()), _step(moe, view)
        for a, b, what in zip(ref[:3], got[:3], ("output", "router logits", "input gradient")):
            _assert_same(a, b, what)
        for name in ref[3]:
            _assert_same(ref[3][name], got[3][name], name)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_input_with_batch_dimensions(dtype):
    torch.manual_seed(2)
    moe = MoE(8, 2, 64, 128, swiglu_packed, True, True, 0.02).to(DEV).to(dtype)
    x = torch.randn(3, 5, 64, device=DEV).to(dtype)
    ref, got = _step(moe, x.reshape(15, 64)), _step(moe, x)
    assert got[0].shape == (3, 5, 64) and got[2].shape == (3, 5, 64) and got[1].shape == (15, 8)
    _assert_same(ref[0], got[0].reshape(15, 64), "output")
    _assert_same(ref[2], got[2].reshape(15, 64), "input gradient")
    for name in ref[3]:
        _assert_same(ref[3][name], got[3][name], name)


@pytest.mark.parametrize("dtype,rtol", [(torch.bfloat16, 2e-2), (torch.float32, 1e-5)])
@pytest.mark.parametrize("E,k", [(4, 4), (8, 1), (1, 1), (16, 16), (17, 17), (64, 64)])
def test_every_expert_selected_or_only_one(E, k, dtype, rtol):
    # against the layer's definition (fma/modules/moe/__init__.py:267-286) evaluated token by token in fp64 from the
    # routing the layer itself chose
    torch.manual_seed(3)
    T, H, I = 19, 64, 64
    moe = MoE(E, k, H, I, swiglu_packed, True, False, 0.02).to(DEV).to(dtype)
    x = torch.randn(T, H, device=DEV).to(dtype)
    with torch.no_grad():
        y, _ = moe(x, kernel_backend=KernelBackend.cuda)
        _, weights, selected = moe._compute_routing_weights(x)
    assert sorted(selected[0].tolist()) == list(range(E)) if k == E else selected.shape == (T, k)
    weights, selected = weights.double().cpu(), selected.long().cpu()
    xd, W1, W2 = x.double().cpu(), moe.c_fc.weight.detach().double().cpu(), moe.c_proj.weight.detach().double().cpu()
    expect = torch.zeros(T, H, dtype=torch.float64)
    for t in range(T):
        for j in range(k):
            e = int(selected[t, j])
            h = W1[e] @ xd[t]
            up, gate = h[:I], h[I:]
            expect[t] += weights[t, j] * (W2[e] @ (up * gate * torch.sigmoid(gate)))
    err = float((y.double().cpu() - expect).abs().max())
    assert err <= rtol * float(expect.abs().max()), f"max error {err} against scale {float(expect.abs().max())}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_frozen_parameters_and_inference(dtype):
    torch.manual_seed(4)
    moe = MoE(8, 2, 64, 128, swiglu_packed, True, True, 0.02).to(DEV).to(dtype)
    x = torch.randn(21, 64, device=DEV).to(dtype)
    y_full, _, dx_full, grads_full = _step(moe, x)

    def backward_of(inp):
        moe.zero_grad(set_to_none=True)
        y, logits = moe(inp, kernel_backend=KernelBackend.cuda)
        (y.float().pow(2).sum() + logits.float().sum()).backward()

    # an input that needs no gradient: the parameters get the same gradients
    backward_of(x)
    for name, p in moe.named_parameters():
        _assert_same(grads_full[name], p.grad, f"{name} (input without gradient)")
    # experts frozen: the input and the gate still get theirs, the experts get none
    for name, p in moe.named_parameters():
        p.requires_grad_(name.startswith("gate"))
    xg = x.clone().requires_grad_()
    backward_of(xg)
    _assert_same(dx_full, xg.grad, "input gradient (experts frozen)")
    _assert_same(grads_full["gate.weight"], moe.gate.weight.grad, "gate gradient (experts frozen)")
    assert all(p.grad is None for name, p in moe.named_parameters() if not name.startswith("gate"))
    # gate frozen, input without gradient: only the experts
    for name, p in moe.named_parameters():
        p.requires_grad_(not name.startswith("gate"))
    backward_of(x)
    assert moe.gate.weight.grad is None
    for name, p in moe.named_parameters():
        if not name.startswith("gate"):
            _assert_same(grads_full[name], p.grad, f"{name} (gate frozen)")
    # no graph at all
    with torch.no_grad():
        _assert_same(y_full, moe(x, kernel_backend=KernelBackend.cuda)[0], "output under no_grad")
    with torch.inference_mode():
        _assert_same(y_full, moe(x, kernel_backend=KernelBackend.cuda)[0], "output under inference_mode")


@pytest.mark.parametrize("mode", ["no_grad", "inference_mode"])
def test_evaluation_with_trainable_weights_does_not_store_the_preactivation(mode, monkeypatch):
    # a model whose parameters require grad, evaluated with autograd off (the usual eval / decode call): the fused
    # up-projection must run without the [R, 2I] pre-activation buffer, and give the bits of the training forward
    from fma.modules.moe import cuda_implementation as ci

    torch.manual_seed(6)
    moe = MoE(8, 2, 256, 512, swiglu_packed, True, False, 0.02).to(DEV).to(torch.bfloat16)
    assert moe.fuse_swiglu and all(p.requires_grad for p in moe.parameters())
    x = torch.randn(300, 256, device=DEV).bfloat16()
    seen = []
    real, real_gathered = ci.grouped_gemm_swiglu_cuda, ci.grouped_gemm_gathered_cuda

    def spy(x_, weight, M_array, h, act, bias=None):
        seen.append(h is not None)
        return real(x_, weight, M_array, h, act, bias)

    def spy_gathered(x_, row_index, divisor, weight, bias, M_array, out, act):  # the evaluation call gathers by itself
        seen.append(out is not None)
        return real_gathered(x_, row_index, divisor, weight, bias, M_array, out, act)

    monkeypatch.setattr(ci, "grouped_gemm_swiglu_cuda", spy)
    monkeypatch.setattr(ci, "grouped_gemm_gathered_cuda", spy_gathered)
    y_train, _ = moe(x.clone().requires_grad_(), kernel_backend=KernelBackend.cuda)
    assert seen == [True]
    with torch.no_grad() if mode == "no_grad" else torch.inference_mode():
        y_eval, _ = moe(x, kernel_backend=KernelBackend.cuda)
    assert seen == [True, False], "the pre-activation was stored although no backward can follow"
    _assert_same(y_train.detach(), y_eval, f"output under {mode}")


@pytest.mark.parametrize("add_bias", [False, True])
def test_training_step_is_bit_reproducible(add_bias):
    # nothing on the path accumulates with floating-point atomics (the reference's grouped rows, weight gradients and
    # norm weight gradient do): two runs of one step on skewed routing over many experts give the same bits everywhere
    from fma import fused_residual_add_rmsnorm

    torch.manual_seed(5)
    T, H, I, E, k = 4096, 256, 192, 64, 8
    moe = MoE(E, k, H, I, swiglu_packed, True, add_bias, 0.02).to(DEV).to(torch.bfloat16)
    with torch.no_grad():  # skew the routing: logits of the first experts spread wider, so they win the top-k more often
        moe.gate.weight.mul_(torch.linspace(3.0, 0.2, E, device=DEV).bfloat16()[:, None])
    norm_weight = torch.ones(H, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    x0 = torch.randn(T, H, device=DEV).bfloat16()
    r0 = torch.randn(T, H, device=DEV).bfloat16()

    def step():
        moe.zero_grad(set_to_none=True)
        norm_weight.grad = None
        x, r = x0.clone().requires_grad_(), r0.clone().requires_grad_()
        normed, residual = fused_residual_add_rmsnorm(x, r, norm_weight, 1e-5)
        y, logits = moe(normed, kernel_backend=KernelBackend.cuda)
        out = y + residual
        (out.float().pow(2).mean() + 1e-2 * logits.float().pow(2).mean()).backward()
        grads = {n: p.grad.clone() for n, p in moe.named_parameters()}
        grads.update(x=x.grad, r=r.grad, norm_weight=norm_weight.grad.clone(), out=out.detach(), logits=logits.detach())
        return grads

    first, second = step(), step()
    for name in first:
        assert torch.equal(first[name], second[name]), name
    counts = torch.bincount(moe._compute_routing_weights(x0)[2].flatten().long(), minlength=E)
    assert int(counts.max()) > 4 * max(int(counts.min()), 1), "the routing of this test is meant to be skewed"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_the_reference_s_two_projection_entry_points(dtype):
    # Experts.up_projection_triton_forward / down_projection_triton_forward (fma/modules/moe/__init__.py:40-87), called as
    # the reference's triton branch calls them (:247-265) with torch's own sort as routing order: the layer's result and
    # gradients (bit for bit in bf16, where both run the same kernels; fp32 goes through the grouped copy)
    torch.manual_seed(11)
    E, k, H, I, T = 8, 2, 256, 384, 500
    moe = MoE(E, k, H, I, swiglu_packed, True, False, 0.05).to(dtype).to(DEV)
    x = torch.randn(T, H, device=DEV).to(dtype)
    dy = torch.randn(T, H, device=DEV).to(dtype)
    selected = torch.randint(0, E - 1, (T, k), device=DEV)  # the last expert gets no rows
    weights = torch.softmax(torch.randn(T, k, device=DEV), dim=-1).to(dtype)

    def run(through_entry_points):
        moe.zero_grad(set_to_none=True)
        xi, wi = x.clone().requires_grad_(), weights.clone().requires_grad_()
        if through_entry_points:
            sorted_expert_idxs, sorted_scattered_idxs = selected.flatten().sort(stable=True)
            expert_offsets = torch.bincount(sorted_expert_idxs, minlength=E).cumsum(-1)
            routing = dict(sorted_expert_idxs=sorted_expert_idxs, sorted_scattered_idxs=sorted_scattered_idxs,
                           expert_offsets=expert_offsets)
            h = moe.c_fc.up_projection_triton_forward(input=xi, num_experts_per_token=k, **routing)
            y = moe.c_proj.down_projection_triton_forward(input=moe.act(h), num_experts_per_token=1, gates=wi, **routing)
        else:
            y = moe._compute_experts(xi, wi, selected, KernelBackend.cuda)
        y.backward(dy)
        return [y.detach(), xi.grad, wi.grad, moe.c_fc.weight.grad.clone(), moe.c_proj.weight.grad.clone()]

    for name, a, b in zip(("y", "dx", "dgates", "dW1", "dW2"), run(True), run(False)):
        if dtype == torch.bfloat16:
            _assert_same(a, b, name)
        else:
            assert float((a - b).abs().max()) <= 1e-5 * max(1.0, float(b.abs().max())), name
    # without gates the second entry point returns the rows per (token, choice) slot
    sorted_expert_idxs, sorted_scattered_idxs = selected.flatten().sort(stable=True)
    expert_offsets = torch.bincount(sorted_expert_idxs, minlength=E).cumsum(-1)
    grouped = torch.randn(T * k, I, device=DEV).to(dtype)
    per_slot = moe.c_proj.down_projection_triton_forward(
        input=grouped, num_experts_per_token=1, sorted_expert_idxs=sorted_expert_idxs,
        sorted_scattered_idxs=sorted_scattered_idxs, expert_offsets=expert_offsets,
    )
    counts = torch.bincount(sorted_expert_idxs, minlength=E).to(torch.int32).view(torch.uint32)
    rows = moe.c_proj.cuda_forward(grouped, counts)
    expect = torch.empty_like(rows)
    expect[sorted_scattered_idxs] = rows
    _assert_same(per_slot.detach(), expect.detach(), "rows per slot")
