"""CPU oracle for the whole forward: embedding -> encoder blocks -> mean pooling
-> MLP head, written functionally over a name->tensor dictionary (the
``state_dict`` / ``named_parameters`` layout shared with the reference).

TEST INFRASTRUCTURE ONLY (see oracle/torch_path.py).  Restates the reference's
PyTorch path with the fixed translation cube:

* block structure, no norms under t-fixup   models/indexed_latticeformer_encoder.py:575-616
* attention forward                          models/indexed_lattice_multi_head_attention.py:1148-1499
  (real, reciprocal and half-and-half "multihead" blocks, :1355-1376)
* model head                                 models/latticeformer.py:211-224, 291-302

Pinned by the golden vectors under tests/golden/ (written by importing the
reference model itself) and, piecewise, by the pins of torch_path.py.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch
import torch.nn.functional as F
from torch import Tensor

from . import torch_path as tp


def _layer_scale(cfg, name: str, layer: int):
    v = getattr(cfg, name)
    if isinstance(v, (list, tuple)):
        v = v[layer % len(v)]
    return v


def layer_domain(cfg, layer: int) -> str:
    """Domain of one block: 'real', 'reci', 'RECI', 'multihead', or the parts of a
    dash-separated list taken in turn (models/latticeformer_params.py, getLayerParameters)."""
    domain = getattr(cfg, "domain", "real")
    if domain in ("real", "reci", "RECI", "multihead"):
        return domain
    parts = domain.split("-")
    return parts[layer % len(parts)]


def attention_block(P: Dict[str, Tensor], prefix: str, cfg, layer: int, x: Tensor, pos: Tensor,
                    batch: Tensor, trans: Tensor, sizes, edges: Tensor, training: bool,
                    capture: Optional[dict] = None, multihead_values: bool = False) -> Tensor:
    H = cfg.head_num
    n = x.shape[0]
    wq, wk, wv = P[prefix + "q_proj_weight"], P[prefix + "k_proj_weight"], P[prefix + "v_proj_weight"]
    bq, bk, bv = P[prefix + "in_proj_bias"].split([wq.shape[0], wk.shape[0], wv.shape[0]])
    q = F.linear(x, wq, bq).view(n, H, -1)
    k = F.linear(x, wk, bk).view(n, H, -1)
    v = F.linear(x, wv, bv).view(n, H, -1)
    beta = float(cfg.positive_func.split("=")[1]) if "=" in cfg.positive_func else 1.0
    assert cfg.positive_func.startswith("elu") and cfg.gauss_state == "q"
    r0 = _layer_scale(cfg, "scale_real", layer)
    domain = layer_domain(cfg, layer)
    K = cfg.value_pe_dist_real
    dist_max = cfg.value_pe_dist_max
    if dist_max < 0:
        dist_max = -dist_max * r0
    W = P.get(prefix + "pe_dist_proj") if K > 0 else None
    if domain == "real":
        alpha = tp.gaussian_exponents(q, P[prefix + "lattice_pos_weights"], P[prefix + "gauss_scale"],
                                      training, cfg.normalize_gauss, cfg.gauss_lb_real, beta, r0)
        z, vpe = tp.periodic_encoding(alpha, pos, batch, trans, edges, cfg.lattice_range, K, dist_max,
                                      cfg.value_pe_width_scale, W)
    else:
        # models/indexed_lattice_multi_head_attention.py:1359-1376
        an = tp.normalised_alpha(q, P[prefix + "lattice_pos_weights"], P[prefix + "gauss_scale"], training,
                                 cfg.normalize_gauss)
        s_reci = _layer_scale(cfg, "scale_reci", layer)
        cos_kr, k2, vcell = tp.reciprocal_half_terms(pos, batch, trans, edges, cfg.lattice_range)
        rho_reci = lambda x: tp.positive_elu(x, cfg.gauss_lb_reci, beta)
        vpe = None
        if domain == "reci":
            alpha = rho_reci(an) * (-0.5 * s_reci ** 2)
            z = tp.reciprocal_bias(alpha, cos_kr, k2, vcell, edges[0], batch)
        elif domain == "RECI":
            alpha = 1 / rho_reci(an) * (-0.5 * s_reci ** 2)
            z = tp.reciprocal_bias(alpha, cos_kr, k2, vcell, edges[0], batch)
        elif domain == "multihead":
            a1, a2 = an.chunk(2, 1)
            a1 = tp.positive_elu(a1, cfg.gauss_lb_real, beta) * (-0.5 * r0 ** -2)
            a2 = rho_reci(a2) * (-0.5 * s_reci ** 2)
            # real half: bias (and, with multihead_values, the value encoding of its heads as the
            # reference's kernel path computes it, zero for the reciprocal half,
            # models/indexed_lattice_multi_head_attention_cuda.py:731-746; the PyTorch path yields
            # no value encoding for this domain, :1433 tests `domain in "real"`)
            Wh = W[:, :H // 2] if (W is not None and W.shape[1] > 1) else W
            z1, v1 = tp.periodic_encoding(a1, pos, batch, trans, edges, cfg.lattice_range,
                                          K if multihead_values else 0, dist_max, cfg.value_pe_width_scale,
                                          Wh if multihead_values else None)
            z2 = tp.reciprocal_bias(a2, cos_kr, k2, vcell, edges[0], batch)
            z = torch.cat([z1, z2], dim=-1)
            alpha = torch.cat([a1, a2], dim=1)
            if v1 is not None:
                vpe = torch.cat([v1, torch.zeros_like(v1)], dim=1)
        else:
            raise NotImplementedError(domain)
    out, prob = tp.indexed_attention(q, k, v, sizes, edges, z, vpe)
    if capture is not None:
        capture[f"layer{layer}.alpha"] = alpha.detach()
        capture[f"layer{layer}.attn_weights"] = z.detach()
        if vpe is not None:
            capture[f"layer{layer}.values"] = vpe.detach()
    out = out.reshape(n, -1)
    return F.linear(out, P[prefix + "out_proj.weight"], P[prefix + "out_proj.bias"])


def encoder_forward(P: Dict[str, Tensor], cfg, x: Tensor, pos: Tensor, batch: Tensor, trans: Tensor,
                    sizes, training: bool = False, prefix: str = "encoder.",
                    capture: Optional[dict] = None, multihead_values: bool = False) -> Tensor:
    batch = batch - batch[0]
    sizes_l = sizes.tolist() if torch.is_tensor(sizes) else list(sizes)
    edges = tp.get_edge_index(sizes_l)
    for layer in range(cfg.num_layers):
        lp = f"{prefix}layers.{layer}."
        x = x + attention_block(P, lp + "self_attn.", cfg, layer, x, pos, batch, trans, sizes_l, edges,
                                training, capture, multihead_values)
        h = F.relu(F.linear(x, P[lp + "linear1.weight"], P[lp + "linear1.bias"]))
        x = x + F.linear(h, P[lp + "linear2.weight"], P[lp + "linear2.bias"])
        if capture is not None:
            capture[f"layer{layer}.out"] = x.detach()
    return x


def latticeformer_forward(P: Dict[str, Tensor], cfg, data, training: bool = False,
                          capture: Optional[dict] = None, multihead_values: bool = False) -> Tensor:
    """Default head: no pre-pooling op, mean pooling, Linear-ReLU-Linear MLP
    with identity norms (norm_type 'no')."""
    assert cfg.pooling == "avr" and cfg.pre_pooling_op == "no" and cfg.norm_type in ("no", "id")
    assert cfg.t_fixup_init, "the oracle covers the norm-free t-fixup blocks"
    x = F.linear(data.x, P["input_embeddings.weight"])
    x = encoder_forward(P, cfg, x, data.pos, data.batch, data.trans_vec, data.sizes, training, capture=capture,
                        multihead_values=multihead_values)
    x = tp.avr_pool(x, data.sizes)
    if capture is not None:
        capture["pooled"] = x.detach()
    idx = 0
    while f"mlp.{idx + 3}.weight" in P:
        x = F.relu(F.linear(x, P[f"mlp.{idx}.weight"], P[f"mlp.{idx}.bias"]))
        idx += 3
    return F.linear(x, P[f"mlp.{idx}.weight"], P[f"mlp.{idx}.bias"])
