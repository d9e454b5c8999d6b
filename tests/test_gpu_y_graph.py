"""HIP graph capture of the expert path: the entry points only enqueue kernels on the stream they are given (no
allocation, no memset, no synchronisation inside the library), so a forward pass, or a whole forward + backward step,
can be captured once and replayed. Every replay is checked against the eager result, with eager work and
synchronisations between the replays."""

import pytest
import torch

from fma import KernelBackend, MoE, swiglu_packed

from gpu_util import DEV

pytestmark = pytest.mark.gpu


def test_expert_path_replays_from_a_captured_graph():
    torch.manual_seed(7)
    T, H, I, E, k = 300, 256, 512, 8, 2
    moe = MoE(E, k, H, I, swiglu_packed, True, False, 0.02).to(torch.bfloat16).to(DEV)
    x_static = torch.zeros(T, H, dtype=torch.bfloat16, device=DEV)
    w_static = torch.zeros(T, k, dtype=torch.bfloat16, device=DEV)
    sel_static = torch.zeros(T, k, dtype=torch.int64, device=DEV)

    def draw(seed):
        g = torch.Generator().manual_seed(seed)
        x = torch.randn(T, H, generator=g).bfloat16().to(DEV)
        with torch.no_grad():
            _, w, sel = moe._compute_routing_weights(x)
        return x, w, sel

    def load(batch):
        for dst, src in zip((x_static, w_static, sel_static), batch):
            dst.copy_(src)

    with torch.no_grad():
        load(draw(0))
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):  # warm-up on the capture stream, as torch's graph recipe asks
            for _ in range(2):
                moe._compute_experts(x_static, w_static, sel_static, KernelBackend.cuda)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            y_static = moe._compute_experts(x_static, w_static, sel_static, KernelBackend.cuda)

        for seed in (1, 2, 3, 4):
            batch = draw(seed)
            expect = moe._compute_experts(*batch, KernelBackend.cuda)  # eager, between the replays
            torch.cuda.synchronize()
            load(batch)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(y_static, expect), f"replay with batch {seed} differs from the eager result"


def test_whole_layer_with_the_fused_router_replays_from_a_captured_graph():
    # the same with the router inside the captured region: gate product, top-k and softmax are one kernel that clears
    # nothing (the optional histogram, which a fill kernel would clear, is not requested by the module)
    torch.manual_seed(8)
    T, H, I, E, k = 200, 512, 256, 64, 8
    moe = MoE(E, k, H, I, swiglu_packed, True, False, 0.02).to(torch.bfloat16).to(DEV)
    assert moe._router_is_fusable(torch.zeros(1, H, dtype=torch.bfloat16, device=DEV))
    x_static = torch.zeros(T, H, dtype=torch.bfloat16, device=DEV)

    def draw(seed):
        return torch.randn(T, H, generator=torch.Generator().manual_seed(seed)).bfloat16().to(DEV)

    with torch.no_grad():
        x_static.copy_(draw(0))
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                moe(x_static, kernel_backend=KernelBackend.cuda)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            y_static, logits_static = moe(x_static, kernel_backend=KernelBackend.cuda)

        for seed in (1, 2, 3, 4):
            x = draw(seed)
            expect, expect_logits = moe(x, kernel_backend=KernelBackend.cuda)  # eager, between the replays
            torch.cuda.synchronize()
            x_static.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(logits_static, expect_logits), f"router logits of replay {seed} differ"
            assert torch.equal(y_static, expect), f"replay with batch {seed} differs from the eager result"


@pytest.mark.parametrize("add_bias", [False, True])
def test_training_step_replays_from_a_captured_graph(add_bias):
    # forward and backward of residual add + RMSNorm and the layer (fused router; with biases also the in-place bias add
    # and its two-launch gradient) captured as one graph with an explicit upstream gradient; every replay against the
    # eager step on the same data
    from fma import fused_residual_add_rmsnorm

    torch.manual_seed(9)
    T, H, I, E, k = 320, 256, 384, 16, 4
    moe = MoE(E, k, H, I, swiglu_packed, True, add_bias, 0.05).to(torch.bfloat16).to(DEV)
    norm_weight = torch.ones(H, dtype=torch.bfloat16, device=DEV, requires_grad=True)
    params = [norm_weight] + list(moe.parameters())
    static = [torch.zeros(T, H, dtype=torch.bfloat16, device=DEV) for _ in range(3)]  # x, residual, upstream gradient

    def draw(seed):
        g = torch.Generator().manual_seed(seed)
        return [torch.randn(T, H, generator=g).bfloat16().to(DEV) for _ in range(3)]

    def step(x, residual, dy):
        x, residual = x.detach().requires_grad_(), residual.detach().requires_grad_()
        normed, res = fused_residual_add_rmsnorm(x, residual, norm_weight, 1e-5)
        y, logits = moe(normed, kernel_backend=KernelBackend.cuda)
        out = y + res
        torch.autograd.backward([out, logits], [dy, logits.detach() * 0.01])
        return out.detach(), x.grad, residual.grad

    def clear():
        for p in params:
            p.grad = None

    for dst, src in zip(static, draw(0)):
        dst.copy_(src)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            clear()
            step(*static)
    torch.cuda.current_stream().wait_stream(side)
    clear()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_static, dx_static, dr_static = step(*static)
    grads_static = [p.grad for p in params]  # allocated inside the capture: rewritten by every replay

    for seed in (1, 2, 3, 4):
        batch = draw(seed)
        for dst, src in zip(static, batch):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        replayed = [t.clone() for t in [out_static, dx_static, dr_static] + grads_static]
        clear()
        expect = list(step(*batch))  # eager, between the replays
        expect += [p.grad.clone() for p in params]
        torch.cuda.synchronize()
        for p, g in zip(params, grads_static):
            p.grad = g  # the graph writes into these tensors
        for i, (a, b) in enumerate(zip(replayed, expect)):
            assert torch.equal(a, b), f"replay {seed}: tensor {i} differs from the eager step"
