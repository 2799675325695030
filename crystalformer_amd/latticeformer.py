"""Whole-model host for the hot path: atom embedding -> encoder -> pooling ->
MLP head, single GPU (models/latticeformer.py:31-224, 291-302 of the
reference; its single-process multi-GPU branch is not reproduced).

``params`` is any attribute bag with the reference's JSON keys
(params/latticeformer/default.json); missing keys take the same defaults as
the reference constructor.
"""
from __future__ import annotations

import copy
from types import SimpleNamespace

import torch
import torch.nn as nn

from . import pooling
from .encoder import CrystalformerEncoderCUDA
from .params import LatticeformerParams

ATOM_FEAT_DIM = 98

# values of params/latticeformer/default.json that shape the model
DEFAULT_MODEL_PARAMS = dict(
    num_layers=4, lattice_range=2, adaptive_cutoff_sigma=-3.5, minimum_range=True, model_dim=128,
    k_dim=0, v_dim=0, head_num=8, ff_dim=512, t_fixup_init=True, embedding_dim=[128], t_activation="relu",
    domain="real", gauss_lb_real=0.5, gauss_lb_reci=0.5, gauss_state="q", normalize_gauss=True,
    positive_func="elu=0.1", use_cgcnn_feat=False, scale_real=[1.4], scale_reci=[2.2],
    value_pe_dist_real=64, value_pe_dist_reci=0, value_pe_wave_real=0, value_pe_wave_reci=0,
    value_pe_dist_max=-10.0, value_pe_width_scale=1.0, value_pe_headed=True, value_pe_condproj="no",
    exclude_self=False, norm_func_mode=0, pooling="avr", pre_pooling_op="no", norm_type="no",
    dropout=0.0, scale_grad=0.0, use_cuda_code=True, use_low_memory=True, targets="bandgap")


def default_params(**overrides) -> SimpleNamespace:
    cfg = copy.deepcopy(DEFAULT_MODEL_PARAMS)
    cfg.update(overrides)
    return SimpleNamespace(**cfg)


class Latticeformer(nn.Module):
    def __init__(self, params):
        super().__init__()
        self.params = params
        embedding_dim = copy.deepcopy(params.embedding_dim)
        num_layers = getattr(params, "num_layers", 4)
        model_dim = getattr(params, "model_dim", 128)
        ff_dim = getattr(params, "ff_dim", 512)
        t_fixup_init = getattr(params, "t_fixup_init", True)
        self.pooling = getattr(params, "pooling", "max")
        pre_pooling_op = getattr(params, "pre_pooling_op", "w+bn+relu")
        dropout = getattr(params, "dropout", 0.1)
        head_num = getattr(params, "head_num", 8)
        norm_type = getattr(params, "norm_type", "bn")
        # Two options that cannot run in the reference either: its forward multiplies by an `atom_feat`
        # table that no code creates (models/latticeformer.py:219-223), and its gradient scaler calls
        # avr_pool with two arguments where the function takes three (models/latticeformer.py:23,
        # models/pooling.py:19).  There is no behaviour to reproduce, so they are refused by name.
        if getattr(params, "use_cgcnn_feat", False):
            raise NotImplementedError("use_cgcnn_feat: the reference defines no atom_feat table for it")
        if getattr(params, "scale_grad", 0.0) > 0:
            raise NotImplementedError("scale_grad: the reference's GradientScaler cannot run (avr_pool arity)")

        lattice_params = LatticeformerParams()
        lattice_params.parseFromArgs(params)

        self.input_embeddings = nn.Linear(ATOM_FEAT_DIM, model_dim, bias=False)
        emb_scale = model_dim ** (-0.5)
        if t_fixup_init:
            emb_scale *= (9 * num_layers) ** (-1 / 4)
        nn.init.normal_(self.input_embeddings.weight, mean=0, std=emb_scale)

        self.encoder = CrystalformerEncoderCUDA(
            model_dim, head_num, activation=getattr(params, "t_activation", "relu"),
            num_encoder_layers=num_layers, dim_feedforward=ff_dim, dropout=dropout,
            t_fixup_init=t_fixup_init, no_layer_norm=t_fixup_init, lattice_params=lattice_params,
            k_dim=getattr(params, "k_dim", 0), v_dim=getattr(params, "v_dim", 0))

        norms = {"bn": nn.BatchNorm1d, "ln": nn.LayerNorm, "in": nn.InstanceNorm1d,
                 "id": nn.Identity, "no": nn.Identity}
        if norm_type not in norms:
            raise NotImplementedError(f"norm_type: {norm_type}")
        norm = norms[norm_type]

        dim_pooled = model_dim
        self.proj_before_pooling = nn.Identity()
        if pre_pooling_op == "w+bn+relu":
            dim_pooled = embedding_dim.pop(0)
            self.proj_before_pooling = nn.Sequential(nn.Linear(model_dim, dim_pooled), norm(dim_pooled),
                                                     nn.ReLU(True))
        elif pre_pooling_op == "w+relu":
            dim_pooled = embedding_dim.pop(0)
            self.proj_before_pooling = nn.Sequential(nn.Linear(model_dim, dim_pooled), nn.ReLU(True))
        elif pre_pooling_op == "relu":
            self.proj_before_pooling = nn.ReLU(True)
        elif pre_pooling_op != "no":
            raise NotImplementedError(f"pre_pooling_op: {pre_pooling_op}")

        if self.pooling == "max":
            self.pooling_layer = pooling.max_pool
        elif self.pooling == "avr":
            self.pooling_layer = pooling.avr_pool
        else:
            raise NotImplementedError(f"pooling: {self.pooling}")

        final_dim = 1 if isinstance(params.targets, str) else len(params.targets)
        in_dim = [dim_pooled] + embedding_dim[:-1]
        layers = []
        for di, do in zip(in_dim, embedding_dim):
            layers += [nn.Linear(di, do), norm(do), nn.ReLU(True)]
        layers.append(nn.Linear(embedding_dim[-1], final_dim))
        self.mlp = nn.Sequential(*layers)

    def forward(self, data):
        # (inside a fused training step the embedding's and the head's weight gradients join the
        # grouped weight-gradient launch; otherwise these are the stock linear ops)
        from . import hip_funcs
        x = hip_funcs.linear(data.x, self.input_embeddings.weight, self.input_embeddings.bias)
        x = self.encoder(x, data.pos, data.batch, data.trans_vec, data.sizes, data.x)
        x = self.proj_before_pooling(x)
        x = self.pooling_layer(x, data.batch, data.sizes)
        return self._head(x)

    def _head(self, x):
        """The regression head; on the inference path each Linear (+ ReLU) of a head without
        norm layers is one row-block launch instead of a library GEMM plus elementwise launches."""
        from . import ops
        from .attention import inference_only
        mods = list(self.mlp)
        plain = all(isinstance(m, (nn.Linear, nn.ReLU, nn.Identity)) for m in mods)
        if not (plain and x.is_cuda and inference_only(x, self.mlp.parameters)):
            from . import hip_funcs
            for m in mods:
                x = hip_funcs.linear(x, m.weight, m.bias) if isinstance(m, nn.Linear) else m(x)
            return x
        i = 0
        while i < len(mods):
            m = mods[i]
            if isinstance(m, nn.Linear) and ops.linear_rows_supported(x, m.weight):
                j = i + 1
                while j < len(mods) and isinstance(mods[j], nn.Identity):
                    j += 1
                relu = j < len(mods) and isinstance(mods[j], nn.ReLU)
                x, = ops.linear_rows(x, (m.weight,), m.bias, relu=relu)
                i = j + 1 if relu else j
            else:
                x = m(x)
                i += 1
        return x
