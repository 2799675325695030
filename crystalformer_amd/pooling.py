"""Crystal-level pooling (models/pooling.py:14-25 of the reference)."""
from __future__ import annotations

import torch

from . import global_config as config
from . import hip_funcs


def max_pool(x, batch, sizes):
    parts = torch.split_with_sizes(x, sizes.tolist(), 0)
    return torch.stack([torch.max(p, dim=0)[0] for p in parts])


def avr_pool(x, batch, sizes):
    """Mean over the atoms of each crystal; the irregular-mean kernel when the
    numerics switch is >= 1, otherwise the per-crystal torch loop."""
    if config.REPRODUCIBLITY_STATE >= 1 and x.is_cuda:
        return hip_funcs.call(hip_funcs.IrregularMeanCUDA, x, batch, sizes)
    parts = torch.split_with_sizes(x, sizes.tolist(), 0)
    return torch.stack([torch.mean(p, dim=0) for p in parts])
