"""Deterministic synthetic crystals for tests and benchmarks.

A batch carries the same fields the reference's data objects do
(dataloaders/dataset_latticeformer.py:32-38): ``x`` one-hot(98) atom types,
``pos`` Cartesian positions, ``batch`` crystal index per atom, ``trans_vec``
lattice rows, ``sizes`` atoms per crystal.  No dataset or network is involved.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional, Tuple

import torch
from torch import Tensor

ATOM_FEAT_DIM = 98


@dataclass
class CrystalBatch:
    x: Tensor            # (N,98) float32 one-hot
    pos: Tensor          # (N,3)  float32
    batch: Tensor        # (N,)   int64
    trans_vec: Tensor    # (B,3,3) float32, rows are lattice vectors
    sizes: Tensor        # (B,)   int64
    y: Optional[Tensor] = None   # (B,) regression targets

    def to(self, device) -> "CrystalBatch":
        mv = lambda t: None if t is None else t.to(device)
        return CrystalBatch(mv(self.x), mv(self.pos), mv(self.batch), mv(self.trans_vec),
                            mv(self.sizes), mv(self.y))

    @property
    def num_edges(self) -> int:
        return int((self.sizes * self.sizes).sum().item())


def lattice_from_parameters(lengths: Tensor, angles_deg: Tensor) -> Tensor:
    """(B,3),(B,3) -> (B,3,3) with rows a=(a,0,0), b=(b cos g, b sin g, 0),
    c=(c cos b, c (cos a - cos b cos g)/sin g, c*sqrt(...))."""
    a, b, c = lengths.double().unbind(-1)
    al, be, ga = (angles_deg.double() * (math.pi / 180.0)).unbind(-1)
    ca, cb, cg, sg = torch.cos(al), torch.cos(be), torch.cos(ga), torch.sin(ga)
    cy = (ca - cb * cg) / sg
    cz = torch.sqrt(torch.clamp(1.0 - cb * cb - cy * cy, min=1e-12))
    zero = torch.zeros_like(a)
    rows = torch.stack([
        torch.stack([a, zero, zero], -1),
        torch.stack([b * cg, b * sg, zero], -1),
        torch.stack([c * cb, c * cy, c * cz], -1)], dim=1)
    return rows.float()


def _valid_angles(angles_deg: Tensor) -> Tensor:
    ca, cb, cg = torch.cos(angles_deg.double() * (math.pi / 180.0)).unbind(-1)
    return (1 - ca * ca - cb * cb - cg * cg + 2 * ca * cb * cg) > 1e-3


def make_batch(num_crystals: int, size_range: Tuple[int, int], log_uniform: bool,
               length_range: Tuple[float, float], angle_range: Tuple[float, float],
               seed: int = 0, long_axis: Optional[Tuple[float, float]] = None,
               with_targets: bool = False) -> CrystalBatch:
    """Draw a batch.  ``size_range`` is inclusive.  ``long_axis`` replaces the
    first lattice length by a draw from that interval (elongated cells)."""
    g = torch.Generator().manual_seed(seed)
    lo, hi = size_range
    if log_uniform:
        u = torch.rand(num_crystals, generator=g)
        sizes = torch.floor(torch.exp(u * math.log(hi + 1.0) + (1 - u) * math.log(lo))).long()
        sizes = sizes.clamp(lo, hi)
    else:
        sizes = torch.randint(lo, hi + 1, (num_crystals,), generator=g)
    lengths = torch.empty(num_crystals, 3).uniform_(*length_range, generator=g)
    if long_axis is not None:
        lengths[:, 0] = torch.empty(num_crystals).uniform_(*long_axis, generator=g)
    angles = torch.empty(num_crystals, 3).uniform_(*angle_range, generator=g)
    for _ in range(1000):
        bad = ~_valid_angles(angles)
        if not bool(bad.any()):
            break
        angles[bad] = torch.empty(int(bad.sum()), 3).uniform_(*angle_range, generator=g)
    trans = lattice_from_parameters(lengths, angles)
    N = int(sizes.sum())
    batch = torch.repeat_interleave(torch.arange(num_crystals), sizes)
    frac = torch.rand(N, 3, generator=g)
    pos = (frac[:, None, :] @ trans[batch]).squeeze(1)
    Z = torch.randint(1, 95, (N,), generator=g)
    x = torch.eye(ATOM_FEAT_DIM)[Z - 1]
    y = torch.randn(num_crystals, generator=g) if with_targets else None
    return CrystalBatch(x, pos.contiguous(), batch, trans.contiguous(), sizes, y)


# The five benchmark workloads (sizes, cells and model settings).
CONFIGS = {
    "cfg1_simplified_b32": dict(
        batch=dict(num_crystals=32, size_range=(1, 16), log_uniform=False,
                   length_range=(3.0, 12.0), angle_range=(70.0, 110.0)),
        model=dict(num_layers=4, value_pe_dist_real=0, scale_real=[1.4])),
    "cfg2_default_b128": dict(
        batch=dict(num_crystals=128, size_range=(1, 64), log_uniform=True,
                   length_range=(3.0, 15.0), angle_range=(60.0, 120.0)),
        model=dict(num_layers=4, value_pe_dist_real=64, scale_real=[1.4])),
    "cfg3_7block_b256": dict(
        batch=dict(num_crystals=256, size_range=(1, 96), log_uniform=True,
                   length_range=(3.0, 15.0), angle_range=(60.0, 120.0)),
        model=dict(num_layers=7, value_pe_dist_real=64,
                   scale_real=[1.4, 1.4, 2.0, 2.0, 3.0, 3.0, 3.0])),
    "cfg4_train_b128": dict(
        batch=dict(num_crystals=128, size_range=(1, 64), log_uniform=True,
                   length_range=(3.0, 15.0), angle_range=(60.0, 120.0), with_targets=True),
        model=dict(num_layers=4, value_pe_dist_real=64, scale_real=[1.4])),
    "cfg5_stress_b16": dict(
        batch=dict(num_crystals=16, size_range=(200, 444), log_uniform=False,
                   length_range=(4.0, 8.0), angle_range=(50.0, 130.0), long_axis=(20.0, 40.0)),
        model=dict(num_layers=4, value_pe_dist_real=64, scale_real=[3.0])),
}


def make_config_batch(name: str, seed: int = 0) -> CrystalBatch:
    return make_batch(seed=seed, **CONFIGS[name]["batch"])


def select_crystals(b: CrystalBatch, crystals) -> CrystalBatch:
    """The batch made of the listed crystals of ``b`` (in the order given), renumbered from 0."""
    idx = torch.as_tensor(list(crystals), dtype=torch.long)
    start = torch.cat([torch.zeros(1, dtype=torch.long), b.sizes.cumsum(0)])
    atoms = torch.cat([torch.arange(int(start[c]), int(start[c + 1])) for c in idx.tolist()])
    sizes = b.sizes[idx]
    batch = torch.repeat_interleave(torch.arange(idx.numel()), sizes)
    return CrystalBatch(b.x[atoms], b.pos[atoms].contiguous(), batch, b.trans_vec[idx].contiguous(), sizes,
                        None if b.y is None else b.y[idx])
