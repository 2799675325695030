"""HIP-graph replay of a fixed-shape forward.

The model's forward issues about 40 launches per step; for a batch layout
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

from . import ops
from .synthetic import CrystalBatch


def _same_layout(owner, batch: CrystalBatch) -> None:
    """Raise unless ``batch`` has exactly the crystal sizes the graph of ``owner`` was captured
    with: edges, pair list and row offsets are baked into it.  The comparison reads ``sizes``
    back once per tensor (identity and version are remembered)."""
    if batch.pos.shape != owner.static.pos.shape or batch.sizes.shape != owner.static.sizes.shape:
        raise ValueError("batch layout differs from the captured one")
    key = (id(batch.sizes), batch.sizes.data_ptr(), batch.sizes._version)
    if key in owner._checked:
        return
    if batch.sizes.tolist() != owner._sizes_host:
        raise ValueError("crystal sizes differ from the captured batch (same totals, other layout)")
    if len(owner._checked) > 64:
        owner._checked.clear()
    owner._checked[key] = batch.sizes          # keeps the tensor alive: its identity stays unique


class GraphedForward:
    """Capture ``model(batch)`` (inference, no autograd) and replay it.

    ``batch`` fixes the layout: later calls may pass a batch with different
    positions, lattices or species but identical ``sizes``.

    ``launch_share`` (0 < share <= 1) is for several graphs replayed concurrently on
    different streams: the periodic-encoding launches of this graph then take that share
    of the GPU each (:class:`crystalformer_amd.ops.launch_share`), which lengthens one
    replay on its own and shortens the steps when several are in flight.
    """

    def __init__(self, model: torch.nn.Module, batch: CrystalBatch, warmup: int = 3,
                 launch_share: float = 1.0):
        if not batch.pos.is_cuda:
            raise ValueError("GraphedForward needs a batch on the GPU")
        self.model = model
        self.static = CrystalBatch(batch.x.clone(), batch.pos.clone(), batch.batch.clone(),
                                   batch.trans_vec.clone(), batch.sizes.clone(),
                                   None if batch.y is None else batch.y.clone())
        self._sizes_host = batch.sizes.tolist()
        self._checked: dict = {}
        self.graph = torch.cuda.CUDAGraph()
        stream = torch.cuda.Stream()            # default priority
        stream.wait_stream(torch.cuda.current_stream())
        with torch.no_grad(), torch.cuda.stream(stream):
            for _ in range(max(warmup, 1)):     # primes index caches and library workspaces
                model(self.static)
        torch.cuda.current_stream().wait_stream(stream)
        torch.cuda.synchronize()
        with torch.no_grad(), ops.launch_share(launch_share), torch.cuda.graph(self.graph):
            self.output = model(self.static)
        # the graph holds raw addresses of the cached index tensors of this layout
        self._keepalive = ops.index_cache_snapshot()
        torch.cuda.synchronize()

    def __call__(self, batch: Optional[CrystalBatch] = None) -> torch.Tensor:
        if batch is not None and batch is not self.static:
            _same_layout(self, batch)
            self.static.x.copy_(batch.x)
            self.static.pos.copy_(batch.pos)
            self.static.trans_vec.copy_(batch.trans_vec)
        self.graph.replay()
        return self.output


class GraphedTrainStep:
    """One whole training step -- forward, L1 loss, backward, gradient-norm clip,
    AdamW update and learning-rate schedule -- captured into a HIP graph and
    replayed with a single submission.

    Optimiser settings are those of :func:`crystalformer_amd.training.make_optimizer`;
    the schedule lr0 * sqrt(decay / (decay + t)) is evaluated on the device from a
    step counter that lives in the graph, so no host value is baked into it.
    ``batch`` fixes the layout; later calls may pass other positions, lattices,
    species and targets with identical ``sizes``.

    Tensors that still hold the autograd graph of an earlier eager step of ``model`` (a
    loss, an output, a non-detached view of a parameter) must be dropped first: their
    gradient-accumulation nodes are bound to the stream of that step, and a backward pass
    under capture that has to synchronise with it aborts the capture.
    """

    def __init__(self, model: torch.nn.Module, batch: CrystalBatch, lr: float = 5e-4, sch_decay: float = 4000.0,
                 clip_norm: float = 1.0, warmup: int = 3, capture: bool = True):
        from .training import FusedAdamW
        if not batch.pos.is_cuda or batch.y is None:
            raise ValueError("GraphedTrainStep needs a batch with targets on the GPU")
        dev = batch.pos.device
        self.model = model
        self.static = CrystalBatch(batch.x.clone(), batch.pos.clone(), batch.batch.clone(),
                                   batch.trans_vec.clone(), batch.sizes.clone(), batch.y.clone())
        self._sizes_host = batch.sizes.tolist()
        self._checked: dict = {}
        self.clip_norm = clip_norm
        self.lr0, self.decay = lr, sch_decay
        # clip + AdamW + schedule as one device-side update; its step counter lives on the device
        self.opt = FusedAdamW(model, lr=lr, sch_decay=sch_decay, clip_norm=clip_norm)
        model.train()
        stream = torch.cuda.Stream()                      # default priority
        stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(stream):
            for _ in range(max(warmup, 1)):               # primes caches, optimiser state and workspaces
                self.opt.zero_grad(set_to_none=True)
                self._step()
        torch.cuda.current_stream().wait_stream(stream)
        torch.cuda.synchronize()
        self.graph = None
        self.opt.zero_grad(set_to_none=True)
        if capture:                                       # capture=False: same step, launched eagerly
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph):
                self.loss = self._step()
            self._keepalive = ops.index_cache_snapshot()
            torch.cuda.synchronize()

    def _step(self) -> torch.Tensor:
        from .training import fused_training_step
        return fused_training_step(self.model, self.static, self.opt, zero_grad=False)

    def __call__(self, batch: Optional[CrystalBatch] = None) -> torch.Tensor:
        if batch is not None and batch is not self.static:
            _same_layout(self, batch)
            self.static.x.copy_(batch.x)
            self.static.pos.copy_(batch.pos)
            self.static.trans_vec.copy_(batch.trans_vec)
            self.static.y.copy_(batch.y)
        if self.graph is None:
            self.opt.zero_grad(set_to_none=True)
            self.loss = self._step()
        else:
            self.graph.replay()
        return self.loss
