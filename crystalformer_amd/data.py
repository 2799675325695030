"""Data contract and checkpoint compatibility, free of dataset libraries.

* :func:`crystal_data` / :func:`collate`: what the reference's ``make_data`` and the
  torch_geometric collation produce for this model (dataloaders/dataset_latticeformer.py:32-38:
  ``x`` one-hot(98) site species, ``pos`` Cartesian coordinates, ``trans_vec`` (1,3,3)
  lattice rows, ``sizes`` (1,); batching concatenates atoms and numbers the crystals),
  from plain arrays: atomic numbers, coordinates, lattice matrix.
* :func:`load_reference_checkpoint`: loads a Lightning checkpoint of the reference's
  regression module into :class:`crystalformer_amd.latticeformer.Latticeformer` the way the
  reference's demo does (demo.py:67-89): keys under ``swa_model.module.`` are the model's
  own state dict, and ``target_std`` / ``target_mean`` are folded into the last linear layer
  so that the model outputs de-normalised targets.

Files are opened with ``torch.load(..., weights_only=True)`` only: nothing stored in a
checkpoint is executed.  A checkpoint that the safe loader refuses (Lightning stores the
hyper-parameter namespace as a pickled object) has to be re-saved by its owner as a plain
dictionary of tensors, e.g. ``torch.save({"state_dict": ckpt["state_dict"]}, path)``.
"""
from __future__ import annotations

from typing import Iterable, Mapping, Optional, Sequence, Union

import torch
from torch import Tensor

from .synthetic import ATOM_FEAT_DIM, CrystalBatch

MODEL_PREFIX = "swa_model.module."


def crystal_data(atomic_numbers: Sequence[int], cart_coords, lattice_matrix, y: Optional[float] = None,
                 frac_coords: bool = False) -> CrystalBatch:
    """One crystal as a batch of one.  ``atomic_numbers`` 1..98, ``cart_coords`` (n,3) in the
    lattice's length unit (``frac_coords=True``: fractional, converted with the lattice rows),
    ``lattice_matrix`` (3,3) with the lattice vectors as rows."""
    z = torch.as_tensor(atomic_numbers, dtype=torch.long).reshape(-1)
    n = z.numel()
    if n == 0:
        raise ValueError("a crystal needs at least one atom")
    if int(z.min()) < 1 or int(z.max()) > ATOM_FEAT_DIM:
        raise ValueError(f"atomic numbers must lie in 1..{ATOM_FEAT_DIM}")
    lattice = torch.as_tensor(lattice_matrix, dtype=torch.float32).reshape(3, 3)
    pos = torch.as_tensor(cart_coords, dtype=torch.float32).reshape(n, 3)
    if frac_coords:
        pos = pos @ lattice
    x = torch.eye(ATOM_FEAT_DIM)[z - 1]                     # dataloaders/common.py:44-46
    target = None if y is None else torch.tensor([float(y)])
    return CrystalBatch(x, pos, torch.zeros(n, dtype=torch.long), lattice[None].clone(),
                        torch.tensor([n], dtype=torch.long), target)


def collate(crystals: Iterable[CrystalBatch]) -> CrystalBatch:
    """Concatenate crystals (or batches) into one batch: atoms in order, crystal indices
    renumbered consecutively, targets kept only if every part has them."""
    parts = list(crystals)
    if not parts:
        raise ValueError("nothing to collate")
    offsets, total = [], 0
    for p in parts:
        offsets.append(total)
        total += p.sizes.numel()
    ys = [p.y for p in parts]
    return CrystalBatch(
        torch.cat([p.x for p in parts]), torch.cat([p.pos for p in parts]),
        torch.cat([p.batch + off for p, off in zip(parts, offsets)]),
        torch.cat([p.trans_vec for p in parts]), torch.cat([p.sizes for p in parts]),
        torch.cat(ys) if all(y is not None for y in ys) else None)


def reference_state_dict(checkpoint: Mapping, prefix: str = MODEL_PREFIX) -> dict:
    """The model's state dict inside a reference checkpoint: entries of
    ``checkpoint['state_dict']`` whose key starts with ``prefix``, prefix removed
    (demo.py:74-83)."""
    state = checkpoint["state_dict"] if "state_dict" in checkpoint else checkpoint
    out = {k[len(prefix):]: v for k, v in state.items() if k.startswith(prefix)}
    if not out:
        raise KeyError(f"no entries under {prefix!r} in the checkpoint "
                       f"(first keys: {list(state)[:5]})")
    return out


def load_reference_checkpoint(model: torch.nn.Module, checkpoint: Union[str, Mapping],
                              prefix: str = MODEL_PREFIX, fold_target_normalisation: bool = True,
                              strict: bool = True) -> torch.nn.Module:
    """Load a checkpoint of the reference's training module into ``model`` (demo.py:67-89).
    ``checkpoint`` is a path (opened with the safe loader) or an already loaded mapping.
    With ``fold_target_normalisation`` the stored ``target_std`` / ``target_mean`` rescale the
    last linear layer: ``W <- W * std[:, None]``, ``b <- b * std + mean``."""
    if isinstance(checkpoint, (str, bytes)) or hasattr(checkpoint, "__fspath__"):
        checkpoint = torch.load(checkpoint, map_location="cpu", weights_only=True)
    state = checkpoint["state_dict"] if "state_dict" in checkpoint else checkpoint
    model.load_state_dict(reference_state_dict(checkpoint, prefix), strict=strict)
    if fold_target_normalisation:
        if "target_std" not in state or "target_mean" not in state:
            raise KeyError("the checkpoint holds no target_std / target_mean to fold in")
        last = model.mlp[-1]
        std = torch.as_tensor(state["target_std"], dtype=last.weight.dtype, device=last.weight.device).reshape(-1)
        mean = torch.as_tensor(state["target_mean"], dtype=last.weight.dtype, device=last.weight.device).reshape(-1)
        if std.numel() != last.weight.shape[0] or mean.numel() != last.weight.shape[0]:
            raise ValueError(f"target statistics have {std.numel()} entries, the head has {last.weight.shape[0]} outputs")
        with torch.no_grad():
            last.weight.mul_(std[:, None])
            last.bias.mul_(std).add_(mean)
    return model
