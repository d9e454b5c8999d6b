"""`set_seed` (the reference's fma/utils/random.py:11-16): seeds python, numpy and torch (CPU and every GPU)."""

import random

import numpy as np
import torch


def set_seed(seed: int) -> None:
    random.seed(seed)
    np.random.seed(seed)
    torch.manual_seed(seed)
    torch.cuda.manual_seed_all(seed)
