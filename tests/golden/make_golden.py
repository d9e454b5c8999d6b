"""Writes tests/golden/c1_moe_fp32.npz: the small CPU-runnable configuration (T=512 tokens, hidden 256, SwiGLU intermediate 512,
E=8, top-k 2, fp32; activations ~N(0,1), expert weights ~N(0,0.02), softmax top-k routing, seed 42) evaluated by the
CPU oracle (oracle/moe_oracle.py). The reference's own tests hold no stored vectors for this path, and its Python
is never imported: the oracle is pinned by tests/test_oracle.py instead.

Run from the repository root:  python -m tests.golden.make_golden
Inputs are regenerated from the seed by c1_inputs() wherever the fixture is used; the file stores a checksum of them,
the routing, the output, the input gradient and strided samples of the weight gradients (loss = sum of outputs).
"""

import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def c1_inputs() -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    g = torch.Generator().manual_seed(42)
    x = torch.randn(512, 256, generator=g)
    bound = 1.0 / 16.0  # nn.Linear's default init for in_features = 256: U(-1/sqrt(256), 1/sqrt(256))
    wg = (torch.rand(8, 256, generator=g) * 2 - 1) * bound
    w1 = torch.randn(8, 1024, 256, generator=g) * 0.02
    w2 = torch.randn(8, 256, 512, generator=g) * 0.02
    return x, wg, w1, w2


def main() -> None:
    sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
    from oracle import moe_oracle as O

    x, wg, w1, w2 = c1_inputs()
    xr, w1r, w2r = x.clone().requires_grad_(), w1.clone().requires_grad_(), w2.clone().requires_grad_()
    _, weights, selected = O.routing_weights(xr.detach(), wg, 2)
    y = O.moe_experts(xr, weights, selected, w1r, w2r)
    y.sum().backward()
    index = O.routing_index(selected.numpy(), 8)
    np.savez_compressed(
        os.path.join(HERE, "c1_moe_fp32.npz"),
        x_sum=np.float64(x.double().sum().item()),
        selected=selected.numpy(),
        router_weights=weights.numpy(),
        counts=index["counts"],
        offsets=index["offsets"],
        perm=index["perm"],
        y=y.detach().numpy(),
        dx=xr.grad.numpy(),
        dw1_sample=w1r.grad[:, ::16, ::8].numpy(),
        dw2_sample=w2r.grad[:, ::8, ::16].numpy(),
    )


if __name__ == "__main__":
    main()
