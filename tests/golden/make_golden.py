"""Writes tests/golden/c1_moe_fp32.npz: the small CPU-runnable configuration (T=512 tokens, hidden 256, SwiGLU intermediate 512,
E=8, top-k 2, fp32; activations ~N(0,1), expert weights ~N(0,0.02), softmax top-k routing, seed 42) evaluated by the
CPU oracle (oracle/moe_oracle.py). The reference's own tests hold no stored vectors for this path, and its Python
is never imported: the oracle is pinned by tests/test_oracle.py instead.

Run from the repository root:  python -m tests.golden.make_golden
Inputs are regenerated from the seed by c1_inputs() wherever the fixture is used; the file stores a checksum of them,
the routing, the output, the input gradient and strided samples of the weight gradients (loss = sum of outputs).

Two small fixtures are written with plain numpy, without the oracle's functions, so that they pin the oracle as well as
the kernels: routing_index_4096.npz (4096 skewed expert ids in [0, 64) with their histogram, inclusive offsets, stable
expert-major permutation and its inverse, from numpy.bincount / cumsum / argsort(kind="stable")) and grouped_gemm_kat.npz
(the reference's integer known-answer construction, tests/ops/grouped_gemm_test.py:38-92, at a small size: three groups with
ragged sizes, operands in [-8, 8], all four storage layouts, the products from int64 matrix multiplication).
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


def kat_problem(layout: str):
    """Operands of the known-answer grouped GEMM for one layout ("NT", "NN", "TN", "TT": A then B, T = stored transposed,
    i.e. is_A_transposed / is_B_transposed of fma/ops/grouped_gemm/__init__.py:11-46), regenerated from a seed."""
    M, N, K = [40, 0, 72, 9], [24, 24, 56, 8], [16, 16, 48, 72]
    tA, tB = layout[0] == "T", layout[1] == "T"  # "NT" is the forward form: A stored [M, K], B stored [N, K]
    rng = np.random.default_rng(1234 + ["NT", "NN", "TN", "TT"].index(layout))
    As = [rng.integers(-8, 9, size=((k, m) if tA else (m, k))) for m, k in zip(M, K)]
    Bs = [rng.integers(-8, 9, size=((n, k) if tB else (k, n))) for n, k in zip(N, K)]
    return M, N, K, tA, tB, As, Bs


def write_small_fixtures() -> None:
    rng = np.random.default_rng(7)
    p = 1.0 / np.arange(1, 65) ** 1.2
    p[-3:] = 0.0  # three experts receive nothing
    ids = rng.choice(64, size=4096, p=p / p.sum()).astype(np.int32)
    counts = np.bincount(ids, minlength=64).astype(np.uint32)
    perm = np.argsort(ids, kind="stable").astype(np.int32)
    inv = np.empty(4096, dtype=np.int32)
    inv[perm] = np.arange(4096, dtype=np.int32)
    np.savez_compressed(
        os.path.join(HERE, "routing_index_4096.npz"),
        ids=ids, counts=counts, offsets=np.cumsum(counts).astype(np.uint32), perm=perm, eid=ids[perm], inv=inv,
    )
    out = {}
    for layout in ("NT", "NN", "TN", "TT"):
        M, N, K, tA, tB, As, Bs = kat_problem(layout)
        Ds = [(a.T if tA else a).astype(np.int64) @ (b.T if tB else b).astype(np.int64) for a, b in zip(As, Bs)]
        out[layout] = np.concatenate([d.reshape(-1) for d in Ds]).astype(np.int64)
    np.savez_compressed(os.path.join(HERE, "grouped_gemm_kat.npz"), **out)


if __name__ == "__main__":
    main()
    write_small_fixtures()
