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

import contextlib
from typing import Optional, Tuple

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

    Without ``capacity``, ``batch`` fixes the layout: later calls may pass a batch with
    different positions, lattices or species but identical ``sizes``.

    With ``capacity = (crystals, atoms, edges)`` one graph serves ANY batch within those
    bounds (edges = sum of squared crystal sizes): the buffers and launch grids have the
    capacity's size, a call copies the batch into their front, and the graph itself works
    out the index structure and the counts from the crystal sizes on the device
    (:class:`crystalformer_amd.ops.live_sizes`); nothing is read back to the host, so a new
    batch costs five small device copies and one submission.  Results are those of an eager
    forward over the same batch, bit for bit.  A batch with more edges than the capacity
    cannot be detected without a read-back: the layout kernels turn it into a batch of empty
    crystals, whose pooled features -- means over no atoms -- and outputs are NaN, and
    :meth:`overflowed` reports it.

    ``launch_share`` (0 < share <= 1) is for several graphs replayed concurrently on
    different streams: the periodic-encoding launches of this graph then take that share
    of the GPU each (:class:`crystalformer_amd.ops.launch_share`), which lengthens one
    replay on its own and shortens the steps when several are in flight.
    """

    def __init__(self, model: torch.nn.Module, batch: CrystalBatch, warmup: int = 3,
                 launch_share: float = 1.0, capacity: Optional[Tuple[int, int, int]] = None):
        if not batch.pos.is_cuda:
            raise ValueError("GraphedForward needs a batch on the GPU")
        self.model = model
        self.capacity = None
        self._checked: dict = {}
        if capacity is None:
            self.static = CrystalBatch(batch.x.clone(), batch.pos.clone(), batch.batch.clone(),
                                       batch.trans_vec.clone(), batch.sizes.clone(),
                                       None if batch.y is None else batch.y.clone())
            self._sizes_host = batch.sizes.tolist()
            self._live = contextlib.nullcontext()
        else:
            B, N, E = (int(c) for c in capacity)
            if B < 1 or N < B or E < N:
                raise ValueError("capacity is (crystals, atoms, edges) with crystals <= atoms <= edges")
            # Inside the graph the tail of every per-atom / per-edge tensor is unwritten memory: only
            # operators that read the live counts may see them.  The real-space blocks with one
            # projection do; reciprocal-space blocks, species-conditioned projections and the
            # per-crystal torch loop index with whole edge lists, and exponents worked out by torch
            # expressions take their statistics over whole tensors: refused here.
            for m in model.modules():
                P = getattr(m, "params", None)
                if P is None or not hasattr(m, "pe_dist_proj"):
                    continue
                from .attention import fused_exponents_spec
                if (P.domain != "real" or P.value_pe_condproj != "no" or P.norm_func_mode != 0
                        or fused_exponents_spec(P) is None):
                    raise ValueError("GraphedForward(capacity=...) serves real-space attention blocks with one "
                                     "projection, the plain softmax and exponents from the query through the "
                                     "exponent kernel (domain 'real', value_pe_condproj 'no', norm_func_mode 0, "
                                     f"gauss_state 'q*', positive_func elu/abs/exp); got domain {P.domain!r}, "
                                     f"value_pe_condproj {P.value_pe_condproj!r}, norm_func_mode "
                                     f"{P.norm_func_mode}, gauss_state {P.gauss_state!r}, positive_func "
                                     f"{P.positive_func!r}")
            E += (N + E) % 2                    # (atoms + edges is even for any batch)
            self.capacity = (B, N, E)
            dev = batch.pos.device
            eye = torch.eye(3, dtype=batch.trans_vec.dtype, device=dev)
            self.static = CrystalBatch(
                torch.zeros((N,) + tuple(batch.x.shape[1:]), dtype=batch.x.dtype, device=dev),
                torch.zeros((N, 3), dtype=batch.pos.dtype, device=dev),
                torch.zeros(N, dtype=torch.int64, device=dev),
                eye.repeat(B, 1, 1),            # unused slots hold a valid lattice
                torch.zeros(B, dtype=torch.int64, device=dev), None)
            self.header = torch.zeros(4, dtype=torch.int64, device=dev)
            self._live = ops.live_sizes(self.header, N, E)
            self.crystals = 0
            self._load(batch)
        self.graph = torch.cuda.CUDAGraph()
        stream = torch.cuda.Stream()            # default priority
        stream.wait_stream(torch.cuda.current_stream())
        with torch.no_grad(), torch.cuda.stream(stream), self._live:
            for _ in range(max(warmup, 1)):     # primes index caches and library workspaces
                model(self.static)
        torch.cuda.current_stream().wait_stream(stream)
        torch.cuda.synchronize()
        with torch.no_grad(), ops.launch_share(launch_share), self._live, torch.cuda.graph(self.graph):
            self.output = model(self.static)
        # the graph holds raw addresses of the cached index tensors of this layout
        self._keepalive = ops.index_cache_snapshot()
        torch.cuda.synchronize()

    def _load(self, batch: CrystalBatch) -> None:
        """Copy a batch into the front of the capacity buffers (device copies, no read-back)."""
        Bc, Nc, _ = self.capacity
        B, N = batch.sizes.numel(), batch.pos.shape[0]
        if B > Bc or N > Nc or B < 1:
            raise ValueError(f"batch of {B} crystals / {N} atoms exceeds the capacity {Bc} / {Nc}")
        if batch.x.shape[0] != N or batch.batch.numel() != N or batch.trans_vec.shape[0] != B:
            raise ValueError("inconsistent batch")
        st = self.static
        # (the crystal index per atom is not copied: inside the graph the layout kernels write it)
        moves = [(st.x[:N], batch.x), (st.pos[:N], batch.pos), (st.trans_vec[:B], batch.trans_vec),
                 (st.sizes[:B], batch.sizes)]
        if B < self.crystals:                   # slots the previous batch used and this one does not
            moves.append((st.sizes[B:self.crystals], None))
        if all(s is None or (s.is_cuda and s.is_contiguous() and s.dtype == d.dtype) for d, s in moves):
            ops.copy_segments(moves)            # one launch
        else:
            for d, s in moves:
                d.zero_() if s is None else d.copy_(s, non_blocking=True)
        self.crystals = B

    def overflowed(self) -> bool:
        """Whether the batch of the last call exceeded the edge capacity (reads the status word
        back: a host synchronisation, for when the caller has one anyway)."""
        return self.capacity is not None and bool(self.header[3].item())

    def __call__(self, batch: Optional[CrystalBatch] = None) -> torch.Tensor:
        if self.capacity is not None:
            if batch is not None and batch is not self.static:
                self._load(batch)
            self.graph.replay()
            return self.output[:self.crystals]
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
