"""`ensure_contiguous` decorator (the reference's fma/utils/contiguous.py:15-21): every tensor argument, also inside
containers, is made contiguous before the wrapped function sees it."""

from functools import wraps
from typing import Any, Callable

import torch
from torch.utils._pytree import tree_map


def _contiguous(x: Any) -> Any:
    return x.contiguous() if isinstance(x, torch.Tensor) else x


def ensure_contiguous(func: Callable) -> Callable:
    @wraps(func)
    def inner(*args, **kwargs):
        return func(*tree_map(_contiguous, args), **tree_map(_contiguous, kwargs))

    return inner
