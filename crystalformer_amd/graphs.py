"""HIP-graph replay of a fixed-shape forward.

The model's forward issues ~170 small launches per step; for a batch layout
that repeats (same crystal sizes, hence same N and E) the whole step is
captured once into a HIP graph and replayed with a single submission.  Inputs
live in static buffers that :meth:`GraphedForward.__call__` refreshes in place.

Nothing in the captured region synchronises with the host or records a
memset node: index caches are primed by the eager warm-up forwards, and the
kernels clear what they need themselves.
"""
from __future__ import annotations

from typing import Optional

import torch

from .synthetic import CrystalBatch


class GraphedForward:
    """Capture ``model(batch)`` (inference, no autograd) and replay it.

    ``batch`` fixes the layout: later calls may pass a batch with different
    positions, lattices or species but identical ``sizes``.
    """

    def __init__(self, model: torch.nn.Module, batch: CrystalBatch, warmup: int = 3):
        if not batch.pos.is_cuda:
            raise ValueError("GraphedForward needs a batch on the GPU")
        self.model = model
        self.static = CrystalBatch(batch.x.clone(), batch.pos.clone(), batch.batch.clone(),
                                   batch.trans_vec.clone(), batch.sizes.clone(),
                                   None if batch.y is None else batch.y.clone())
        self._sizes_host = batch.sizes.tolist()
        self.graph = torch.cuda.CUDAGraph()
        stream = torch.cuda.Stream()            # default priority
        stream.wait_stream(torch.cuda.current_stream())
        with torch.no_grad(), torch.cuda.stream(stream):
            for _ in range(max(warmup, 1)):     # primes index caches and library workspaces
                model(self.static)
        torch.cuda.current_stream().wait_stream(stream)
        torch.cuda.synchronize()
        with torch.no_grad(), torch.cuda.graph(self.graph):
            self.output = model(self.static)
        torch.cuda.synchronize()

    def __call__(self, batch: Optional[CrystalBatch] = None) -> torch.Tensor:
        if batch is not None and batch is not self.static:
            if batch.pos.shape != self.static.pos.shape or batch.sizes.shape != self.static.sizes.shape:
                raise ValueError("batch layout differs from the captured one")
            self.static.x.copy_(batch.x)
            self.static.pos.copy_(batch.pos)
            self.static.trans_vec.copy_(batch.trans_vec)
        self.graph.replay()
        return self.output
