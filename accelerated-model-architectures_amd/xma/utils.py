"""Small helpers the path needs (reference: xma/utils/random.py:12-20, xma/math.py)."""

from __future__ import annotations

import random

import numpy as np
import torch


def set_seed(seed: int) -> None:
    """Seed python, numpy and torch (CPU and every GPU), as xma/utils/random.py:12-20."""
    random.seed(seed)
    np.random.seed(seed)
    torch.manual_seed(seed)
    if torch.cuda.is_available():
        torch.cuda.manual_seed_all(seed)


def ceil_divide(x: int, y: int) -> int:
    return (x + y - 1) // y
