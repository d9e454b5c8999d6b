"""Seeded random configurations of the whole layer (three dtypes, 1 to 257 experts, top_k up to 9, token counts and sizes
that are multiples of 8 but of nothing larger, the three activations, with and without expert biases), forward and
backward with the router differentiated too, against the oracle evaluated one precision up (fp32 for 16-bit layers, fp64
for fp32 ones) on the GPU from the routing the layer chose. The fixed cases of tests/test_gpu_moe.py follow the
reference's test file; this sweep covers the combinations between them."""

import random

import pytest
import torch
import torch.nn as nn

from fma import KernelBackend, MoE, swiglu_packed
from oracle import moe_oracle as O

from gpu_util import DEV, rel_err

pytestmark = pytest.mark.gpu


def _glu(x):
    a, b = x.chunk(2, dim=-1)
    return a * torch.sigmoid(b)


ACTIVATIONS = {
    "swiglu": (swiglu_packed, O.swiglu_packed, True),
    "glu": (nn.GLU(), _glu, True),
    "gelu": (nn.GELU(approximate="tanh"), nn.GELU(approximate="tanh"), False),
}
# (max relative to the largest value, relative Frobenius) per dtype: a few roundings of the dtype
BARS = {torch.bfloat16: (4e-2, 1.5e-2), torch.float16: (8e-3, 3e-3), torch.float32: (2e-4, 5e-5)}


@pytest.mark.parametrize("seed", range(40))
def test_random_layer_configuration(seed):
    rng = random.Random(seed)
    dtype = rng.choice([torch.bfloat16, torch.bfloat16, torch.float16, torch.float32])
    E = rng.choice([1, 2, 3, 5, 8, 16, 17, 33, 64, 100, 128, 257])
    k = rng.randint(1, min(E, 9))
    T = rng.choice([1, 2, 5, 31, 64, 100, 257, 700, 1500])
    # the reference's grouped-GEMM experts assert N % 8 == 0 and K % 8 == 0 (moe/cuda_implementation/__init__.py:25-26)
    H = rng.choice([8, 16, 24, 40, 64, 72, 136, 256, 520, 1000, 1024])
    I = rng.choice([8, 16, 24, 48, 64, 136, 256, 384, 1000])
    act_name = rng.choice(["swiglu", "swiglu", "glu", "gelu"])
    add_bias = rng.random() < 0.3
    act, oracle_act, is_glu = ACTIVATIONS[act_name]
    case = f"{dtype} E={E} k={k} T={T} H={H} I={I} {act_name} bias={add_bias}"

    torch.manual_seed(seed)
    moe = MoE(E, k, H, I, act, is_glu, add_bias, 0.05).to(DEV).to(dtype)
    if add_bias:
        with torch.no_grad():
            moe.c_fc.bias.normal_(0, 0.3)
            moe.c_proj.bias.normal_(0, 0.3)
    x = torch.randn(T, H, device=DEV).to(dtype).requires_grad_()
    dy = torch.randn(T, H, device=DEV).to(dtype)
    y, _ = moe(x, kernel_backend=KernelBackend.cuda)
    y.backward(dy)
    with torch.no_grad():
        _, _, selected = moe._compute_routing_weights(x.detach())
    selected = selected.long()

    hp = torch.float64 if dtype == torch.float32 else torch.float32
    xo = x.detach().to(hp).requires_grad_()
    P = {n: p.detach().to(hp).requires_grad_() for n, p in moe.named_parameters()}
    # fma/modules/moe/__init__.py:191-204: logits, the chosen ones, softmax over them
    chosen = torch.nn.functional.linear(xo, P["gate.weight"]).gather(1, selected)
    weights = torch.softmax(chosen, dim=-1)
    yo = O.moe_experts(xo, weights, selected, P["c_fc.weight"], P["c_proj.weight"], oracle_act, P.get("c_fc.bias"), P.get("c_proj.bias"))
    yo.backward(dy.to(hp))

    pairs = [("output", y, yo), ("input gradient", x.grad, xo.grad)]
    pairs += [(name, p.grad, P[name].grad) for name, p in moe.named_parameters()]
    for name, got, expect in pairs:
        assert got is not None and bool(torch.isfinite(got.float()).all()), f"{case}: {name}"
        if float(expect.detach().abs().max()) == 0:
            assert float(got.float().abs().max()) == 0, f"{case}: {name} should be all zeros"
            continue
        max_rel, frob_rel = rel_err(got.detach(), expect.detach())
        assert max_rel <= BARS[dtype][0] and frob_rel <= BARS[dtype][1], f"{case}: {name} max_rel={max_rel:.3g} frob_rel={frob_rel:.3g}"
