"""Seeded synthetic inputs of the benchmark workloads, shared by bench.py and the tests: expert choices with router
weights for a layer, and flat arrays of expert ids for the histogram. Plain torch / numpy on the CPU, deterministic in
the seed; nothing here computes an expected result."""

import numpy as np
import torch
import torch.nn.functional as F


def make_routing(T: int, E: int, top_k: int, kind: str, seed: int, empty_tail: int = 0) -> tuple[torch.Tensor, torch.Tensor]:
    """(selected_experts int64 [T,k], router_weights fp32 [T,k]) on the CPU, deterministic in `seed`.

    kind "uniform": top-k of N(0,1) logits, softmax over the kept logits. kind "zipf": k distinct experts per token
    drawn without replacement with p_e ~ 1/(e+1), the last `empty_tail` experts given probability 0 (so that they
    receive no token), weights = softmax of N(0,1) logits.
    """
    g = torch.Generator().manual_seed(seed)
    if kind == "uniform":
        logits = torch.randn(T, E, generator=g)
        values, selected = logits.topk(top_k, dim=-1)
        return selected, F.softmax(values, dim=-1)
    if kind == "zipf":
        p = 1.0 / torch.arange(1, E + 1, dtype=torch.float64)
        if empty_tail:
            p[E - empty_tail :] = 0
        selected = torch.multinomial((p / p.sum()).expand(T, E), top_k, replacement=False, generator=g)
        values = torch.randn(T, top_k, generator=g)
        return selected, F.softmax(values, dim=-1)
    raise ValueError(kind)


def make_ids(n: int, E: int, kind: str, seed: int, dtype=np.int32, s: float = 1.2) -> np.ndarray:
    """n expert ids in [0, E): "uniform", or "zipf" with p_e ~ (e+1)^-s (inverse-CDF sampling)."""
    rng = np.random.default_rng(seed)
    if kind == "uniform":
        return rng.integers(0, E, size=n, dtype=np.int64).astype(dtype)
    if kind == "zipf":
        p = (np.arange(1, E + 1, dtype=np.float64)) ** (-s)
        cdf = np.cumsum(p / p.sum())
        cdf[-1] = 1.0
        return np.searchsorted(cdf, rng.random(n), side="right").clip(0, E - 1).astype(dtype)
    raise ValueError(kind)
