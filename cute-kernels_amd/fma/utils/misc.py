"""Small helpers that keep the names the reference's callers use: `set_seed` (fma/utils/random.py:11-16) and
`get_num_elements_and_hidden_size` (fma/utils/tensor.py:8-11)."""

import random

import numpy
import torch


def set_seed(seed: int) -> None:
    """Seeds every generator a test draws from: python's, numpy's, torch's on the CPU and on all GPUs."""
    for seeder in (random.seed, numpy.random.seed, torch.manual_seed, torch.cuda.manual_seed_all):
        seeder(seed)


def get_num_elements_and_hidden_size(x: torch.Tensor) -> tuple[int, int]:
    """(rows, row length) of x read as a matrix whose rows are its last dimension."""
    row_length = x.shape[-1]
    return (x.numel() // row_length if row_length else 0), row_length
