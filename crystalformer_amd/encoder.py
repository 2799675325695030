"""Encoder stack on the HIP operator path.

Drop-in for ``CrystalformerEncoderCUDA`` / ``CrystalformerEncoderLayerCUDA``
(models/indexed_latticeformer_encoder.py:620-890): same constructor arguments,
sub-module names (``layers.N.self_attn``, ``linear1``, ``linear2``), t-fixup
scaling and ``forward(src, pos, batch, trans, sizes, onehot=None)``.
The geometry prologue (edge list, p_j - p_i, reciprocal vectors) runs on the
device.
"""
from __future__ import annotations

import math
from typing import Callable, Optional, Union

import torch
import torch.nn.functional as F
from torch import Tensor
from torch.nn import Dropout, Identity, LayerNorm, Linear, Module, ModuleList
from torch.nn.init import constant_, xavier_uniform_

from . import ops
from .attention import CrystalformerMultiheadAttentionCUDA
from .hip_funcs import compile_kernels
from . import hip_funcs
from .hip_funcs import linear as linear_hip
from .params import LatticeformerParams


def get_edge_index(sizes, device) -> Tensor:
    """(2,E) int64 edge list of all atom pairs inside each crystal, rows (i, j) of a crystal's
    dense block in i-major order (models/indexed_latticeformer_encoder.py:15-32), built by the
    device kernel instead of a host loop over crystals."""
    if not torch.is_tensor(sizes):
        sizes = torch.tensor(list(sizes), dtype=torch.int64)
    sizes = sizes.to(device=device, dtype=torch.int64)
    if sizes.numel() == 0 or int(sizes.sum()) == 0:
        return torch.zeros((2, 0), dtype=torch.int64, device=device)
    return ops.edge_index(sizes)[0]


def det_3x3(m: Tensor) -> Tensor:
    """Cofactor expansion, term order of models/indexed_latticeformer_encoder.py:34-44."""
    return (m[:, 0, 0] * m[:, 1, 1] * m[:, 2, 2] + m[:, 0, 1] * m[:, 1, 2] * m[:, 2, 0]
            + m[:, 0, 2] * m[:, 1, 0] * m[:, 2, 1] - m[:, 0, 2] * m[:, 1, 1] * m[:, 2, 0]
            - m[:, 0, 0] * m[:, 1, 2] * m[:, 2, 1] - m[:, 0, 1] * m[:, 1, 0] * m[:, 2, 2])


def _sizes_on_device(sizes, batch: Tensor, num_crystals: int, device) -> Tensor:
    if sizes is None:
        sizes = torch.zeros(num_crystals, dtype=torch.long, device=device)
        sizes.scatter_add_(0, batch, torch.ones_like(batch))
    if not torch.is_tensor(sizes):
        sizes = torch.tensor(sizes, dtype=torch.long, device=device)
    return sizes.to(device=device, dtype=torch.long)


def compute_lattice_distances_for_cuda(pos: Tensor, batch: Tensor, trans_vec: Tensor, sizes, lattice_range,
                                       cutoff_radius=0, output_real=False, output_reci=False):
    """Geometry prologue of the kernel path
    (models/indexed_latticeformer_encoder.py:183-253): relative positions per
    edge, reciprocal vectors, cell volume and the dense edge list.  Returns
    ``(pos_ij, dist2_min, kr_base, recip_vec, vcell, edges)``; ``dist2_min`` is None (the
    kernels find the minimum themselves), ``kr_base`` (E,3) the reciprocal-space phases when
    ``output_reci``."""
    sizes = _sizes_on_device(sizes, batch, trans_vec.shape[0], pos.device)
    vcell, recip_vec, _ = ops.lattice_geometry(trans_vec)
    edges, pos_ij = ops.edge_index(sizes, pos.contiguous())
    kr_base = ops.kr_base(pos_ij, recip_vec, batch - batch[0], edges) if output_reci else None
    return pos_ij, None, kr_base, recip_vec, vcell, edges


def _activation(name):
    if callable(name):
        return name
    if name == "relu":
        return F.relu
    if name == "gelu":
        return F.gelu
    raise RuntimeError(f"activation should be relu/gelu, not {name}")


class CrystalformerEncoderLayerCUDA(Module):
    def __init__(self, d_model: int, nhead: int, dim_feedforward: int = 2048, dropout: float = 0.1,
                 activation: Union[str, Callable[[Tensor], Tensor]] = F.relu, layer_norm_eps: float = 1e-5,
                 norm_first: bool = False, no_layer_norm=False, params=LatticeformerParams(),
                 k_dim=0, v_dim=0, device=None, dtype=None) -> None:
        super().__init__()
        assert params.domain in ("real", "reci", "RECI", "multihead")
        self.domain = params.domain
        self.self_attn = CrystalformerMultiheadAttentionCUDA(d_model, nhead, dropout=dropout, kdim=k_dim,
                                                             vdim=v_dim, params=params)
        self.linear1 = Linear(d_model, dim_feedforward)
        self.dropout = Dropout(dropout) if dropout > 0 else Identity()
        self.linear2 = Linear(dim_feedforward, d_model)
        self.norm_first = norm_first
        self.norm1 = LayerNorm(d_model, eps=layer_norm_eps) if not no_layer_norm else Identity()
        self.norm2 = LayerNorm(d_model, eps=layer_norm_eps) if not no_layer_norm else Identity()
        self.dropout1 = Dropout(dropout) if dropout > 0 else Identity()
        self.dropout2 = Dropout(dropout) if dropout > 0 else Identity()
        self.activation = _activation(activation)
        self._reset_parameters()

    def _reset_parameters(self):
        xavier_uniform_(self.linear1.weight)
        xavier_uniform_(self.linear2.weight)
        constant_(self.linear1.bias, 0)
        constant_(self.linear2.bias, 0)

    def fixup_initialization(self, num_layers: int) -> None:
        """t-fixup: scale the value path by 0.67 L^-1/4
        (models/indexed_latticeformer_encoder.py:832-850)."""
        factor = 0.67 * num_layers ** (-1.0 / 4.0)
        scaled = ("linear1.weight", "linear2.weight", "self_attn.out_proj.weight", "self_attn.v_proj_weight")
        with torch.no_grad():
            for name, param in self.named_parameters():
                if name in scaled:
                    param.copy_(factor * param)

    def forward(self, src: Tensor, batch: Tensor, edges: Tensor, pos_ij: Tensor = None,
                dist2_min: Tensor = None, trans: Tensor = None, kr_base: Tensor = None,
                rvecs: Tensor = None, vcell: Tensor = None, onehot: Tensor = None) -> Tensor:
        if self.domain in ("real", "multihead"):
            assert pos_ij is not None and trans is not None
        if self.domain in ("reci", "multihead", "RECI"):
            assert kr_base is not None and rvecs is not None and rvecs.dim() == 3 and vcell is not None
        x = src
        if self._fused_tail(x):
            # inference without norm layers: residuals, bias and ReLU ride in the epilogues of
            # three row-block linear launches (out_proj, linear1, linear2)
            x = self.self_attn(x, x, x, batch, batch, edges, pos_ij, dist2_min, trans, kr_base, rvecs, vcell,
                               onehot, need_weights=False, residual=x)[0]
            h, = ops.linear_rows(x, (self.linear1.weight,), self.linear1.bias, relu=True)
            x, = ops.linear_rows(h, (self.linear2.weight,), self.linear2.bias, residual=x)
            return x
        if self._fused_train(x):
            # the same epilogues with autograd (graphed training step, no norm layers, no dropout)
            x = self.self_attn(x, x, x, batch, batch, edges, pos_ij, dist2_min, trans, kr_base, rvecs, vcell,
                               onehot, need_weights=False, residual=x)[0]
            return hip_funcs.FusedFeedForwardHIP.apply(x, self.linear1.weight, self.linear1.bias,
                                                       self.linear2.weight, self.linear2.bias)
        if self.norm_first:
            x = x + self._sa_block(self.norm1(x), batch, edges, pos_ij, dist2_min, trans, kr_base, rvecs, vcell, onehot)
            x = x + self._ff_block(self.norm2(x))
        else:
            x = self.norm1(x + self._sa_block(x, batch, edges, pos_ij, dist2_min, trans, kr_base, rvecs, vcell, onehot))
            x = self.norm2(x + self._ff_block(x))
        return x

    def _fused_tail(self, x: Tensor) -> bool:
        from .attention import inference_only
        plain = isinstance(self.norm1, Identity) and isinstance(self.norm2, Identity)
        no_drop = not self.training or all(isinstance(d, Identity) for d in (self.dropout, self.dropout1,
                                                                            self.dropout2))
        return (plain and no_drop and self.activation is F.relu
                and inference_only(x, self.parameters)
                and ops.linear_rows_supported(x, self.linear1.weight)
                and ops.linear_rows_supported(x, self.self_attn.out_proj.weight)
                and self.linear2.weight.is_cuda and self.linear2.weight.shape[1] % 16 == 0)

    def _fused_train(self, x: Tensor) -> bool:
        plain = isinstance(self.norm1, Identity) and isinstance(self.norm2, Identity)
        no_drop = all(isinstance(d, Identity) for d in (self.dropout, self.dropout1, self.dropout2))
        return (hip_funcs.USE_LINEAR_FUNCTION and torch.is_grad_enabled() and plain and no_drop
                and self.activation is F.relu and ops.linear_rows_supported(x, self.linear1.weight)
                and self.linear2.weight.shape[1] % 16 == 0)

    def _sa_block(self, x, batch, edges, pos_ij, dist2_min, trans, kr_base, rvecs, vcell, onehot):
        x = self.self_attn(x, x, x, batch, batch, edges, pos_ij, dist2_min, trans, kr_base, rvecs, vcell,
                           onehot, need_weights=False)[0]
        return self.dropout1(x)

    def _ff_block(self, x: Tensor) -> Tensor:
        h = self.activation(linear_hip(x, self.linear1.weight, self.linear1.bias))
        return self.dropout2(linear_hip(self.dropout(h), self.linear2.weight, self.linear2.bias))


class CrystalformerEncoderCUDA(Module):
    def __init__(self, d_model: int = 512, nhead: int = 8, num_encoder_layers: int = 6,
                 dim_feedforward: int = 2048, dropout: float = 0.1,
                 activation: Union[str, Callable[[Tensor], Tensor]] = F.relu, layer_norm_eps: float = 1e-5,
                 norm_first: bool = False, t_fixup_init=False, no_layer_norm=False,
                 lattice_params: LatticeformerParams = LatticeformerParams(), k_dim=0, v_dim=0,
                 device=None, dtype=None) -> None:
        super().__init__()
        self.lattice_params = lattice_params
        self.layers = ModuleList([
            CrystalformerEncoderLayerCUDA(d_model, nhead, dim_feedforward, dropout, activation, layer_norm_eps,
                                          norm_first, no_layer_norm,
                                          params=lattice_params.getLayerParameters(i), k_dim=k_dim, v_dim=v_dim)
            for i in range(num_encoder_layers)])
        if t_fixup_init:
            for layer in self.layers:
                layer.fixup_initialization(num_encoder_layers)
        self.num_layers = num_encoder_layers
        self.norm = LayerNorm(d_model, eps=layer_norm_eps) if not no_layer_norm else None
        self.d_model = d_model
        self.nhead = nhead
        compile_kernels(lattice_params.lattice_range, nhead, k_dim if k_dim > 0 else d_model // nhead,
                        lattice_params.value_pe_dist_real, v_dim if v_dim > 0 else d_model // nhead,
                        lattice_params.minimum_range)

    def forward(self, src: Tensor, pos: Tensor, batch: Tensor, trans: Tensor, sizes: Tensor,
                onehot: Optional[Tensor] = None) -> Tensor:
        if src.size(-1) != self.d_model:
            raise RuntimeError("the feature number of src and tgt must be equal to d_model")
        P = self.lattice_params
        # geometry prologue of compute_lattice_distances_for_cuda, plus the lengths of the
        # reciprocal vectors (all a block needs of them), in two launches
        if not torch.is_tensor(sizes) or sizes.device != pos.device or sizes.dtype != torch.long:
            sizes = _sizes_on_device(sizes, batch, trans.shape[0], pos.device)
        layout = ops.batch_layout(sizes, batch)       # index structure: built once per batch
        batch, edges = layout.batch, layout.edges
        vcell, recip, rvlen = ops.lattice_geometry(trans)
        pos_ij = ops.relative_positions(layout, pos)
        dist2_min = kr_base = None
        rvecs = rvlen                                  # real-space blocks only need the lengths
        if any(layer.domain != "real" for layer in self.layers):
            # reciprocal-space blocks: the vectors themselves and the phases <b_d, p_j - p_i>
            rvecs = recip
            kr_base = ops.kr_base(pos_ij, recip, batch, edges)
        output = src
        for layer in self.layers:
            output = layer(output, batch, edges, pos_ij, dist2_min, trans, kr_base, rvecs, vcell, onehot)
        if self.norm is not None:
            output = self.norm(output)
        return output


CrystalformerEncoderHIP = CrystalformerEncoderCUDA
CrystalformerEncoderLayerHIP = CrystalformerEncoderLayerCUDA
