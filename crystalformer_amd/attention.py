"""Lattice multi-head attention module on the HIP operator path.

Drop-in for ``CrystalformerMultiheadAttentionCUDA``
(models/indexed_lattice_multi_head_attention_cuda.py:790-1016): same
constructor, parameter names/shapes (``gauss_scale``, ``atten_scale``,
``q/k/v_proj_weight``, ``in_proj_bias``, ``out_proj``, ``lattice_pos_weights``,
``pe_dist_proj``), initialisation order and ``forward`` signature.  Only the
real-space domain (and ``"no"``) is served; the dense projections stay on
torch / rocBLAS.
"""
from __future__ import annotations

import math
import warnings
from typing import Optional, Tuple

import torch
import torch.nn.functional as F
from torch import Tensor
from torch.nn import Module, Parameter
from torch.nn.init import constant_, normal_, xavier_uniform_

from . import global_config as config
from . import ops
from . import hip_funcs
from .hip_funcs import linear as linear_hip
from .hip_funcs import (FusedDotProductAttentionCUDA, GaussianExponentsHIP, RealPeriodicEncodingFuncCUDA,
                        RealPeriodicEncodingWithProjFuncCUDA, ReciPeriodicEncodingFuncCUDA)
from .params import LatticeformerParams

ATOM_NUM = 98


def make_positive_func(spec: str):
    """rho(x, lower_bound) for the Gaussian widths
    (models/indexed_lattice_multi_head_attention_cuda.py:675-692)."""
    beta = float(spec.split("=")[1]) if "=" in spec else 1.0
    if spec == "abs":
        return lambda x, lb: (1 - lb) * x.abs() + lb
    if spec.startswith("softplus"):
        return lambda x, lb: F.softplus(x + 1 / beta * math.log(math.exp(beta * (1 - lb)) - 1), beta=beta) + lb
    if spec.startswith("exp"):
        return lambda x, lb: (1.0 - lb) * torch.exp(x * (beta / (1.0 - lb))) + lb
    if spec.startswith("elu"):
        return lambda x, lb: (1.0 - lb) * F.elu(x * (beta / (1.0 - lb))) + 1.0
    if spec.startswith("sigmoid"):
        return lambda x, lb: (1 / lb - lb) * torch.sigmoid(x * (beta * (1 + lb) / (1.0 - lb)) + math.log(lb)) + lb
    raise NotImplementedError(f"Unknown positive_func: {spec}")


def normalised_alpha(q: Tensor, query: Tensor, lattice_pos_weights: Tensor, gauss_scale: Tensor,
                     params: LatticeformerParams, training: bool) -> Tensor:
    """alpha[i,h] from the un-scaled per-head query, normalised by the stored or the batch
    statistics (models/indexed_lattice_multi_head_attention_cuda.py:636-673)."""
    n, h, d = q.shape
    # (per-head dot products; written as a product + sum rather than the reference's
    # batch of N*H 1xd @ dx1 matmuls, which is two orders of magnitude slower on hipBLASLt)
    if params.gauss_state.startswith("q"):
        alpha = (q * lattice_pos_weights.reshape(1, h, d)).sum(-1)
    elif params.gauss_state == "1":
        alpha = lattice_pos_weights.reshape(1, h, d).sum(-1).expand(n, h)
    else:
        alpha = F.linear(query, lattice_pos_weights)
    alpha = alpha.view(n, h)
    if params.normalize_gauss:
        # Stored statistics (gauss_scale[0] > 0) win over the statistics of this batch.
        # Selected on the device: no host synchronisation in the attention block.
        stored = gauss_scale[0] > 0
        scale = torch.where(stored, gauss_scale[0], torch.reciprocal(alpha.detach().std()))
        shift = torch.where(stored, gauss_scale[1], -alpha.detach().mean())
        alpha = (alpha + shift) * scale
        if training:   # written once, by the first training step
            with torch.no_grad():
                gauss_scale.copy_(torch.stack([scale, shift]))
    return alpha


def gaussian_exponents(q: Tensor, query: Tensor, lattice_pos_weights: Tensor, gauss_scale: Tensor,
                       params: LatticeformerParams, training: bool) -> Tensor:
    """a[i,h] = -rho(normalised alpha) / (2 r0^2)
    (models/indexed_lattice_multi_head_attention_cuda.py:636-722, real domain)."""
    alpha = normalised_alpha(q, query, lattice_pos_weights, gauss_scale, params, training)
    rho = make_positive_func(params.positive_func)(alpha, params.gauss_lb_real)
    return rho * (-0.5 * params.scale_real ** -2)


def inference_only(*tensors: Optional[Tensor]) -> bool:
    """True when no gradient can be asked of an op on these tensors: the fused
    row-block linear kernels (no autograd) may then replace F.linear."""
    if not torch.is_grad_enabled():
        return True
    for t in tensors:
        if callable(t):                               # lazily listed tensors (e.g. module.parameters)
            if any(u.requires_grad for u in t()):
                return False
        elif t is not None and t.requires_grad:
            return False
    return True


def fused_exponents_spec(params: LatticeformerParams):
    """(name, beta) when the Gaussian-exponent kernel serves this configuration, else None."""
    if not params.gauss_state.startswith("q"):
        return None
    name, _, beta = params.positive_func.partition("=")
    if name not in ("elu", "abs", "exp"):
        return None
    return name, (float(beta) if beta else 1.0)


def conditional_projection(proj: Tensor, onehot: Tensor, edges: Tensor, mode: str) -> Tensor:
    """Species-conditioned projection, one matrix per edge
    (models/indexed_lattice_multi_head_attention_cuda.py:612-626)."""
    W = onehot @ proj.reshape(proj.shape[0], -1)
    if mode in ("i", "I"):
        W = W[edges[0]]
    elif mode in ("j", "J"):
        W = W[edges[1]]
    elif mode in ("ij", "IJ"):
        W = (W[edges[0]] + W[edges[1]]) * 0.5
    else:
        raise NotImplementedError(mode)
    return W.reshape(-1, proj.shape[1], proj.shape[2], proj.shape[3])


NORM_FUNC_MODES = {"default": 0, "softmax": 1, "exp": 2, "linear": 3, "sigmoid": 4, "softplus": 5, "elu": 6,
                   "elu+1": 7, "abs": 8}


def loop_attention(q: Tensor, k: Tensor, v: Tensor, batch: Tensor, edges: Tensor,
                   bias: Optional[Tensor], values: Optional[Tensor], norm_func_mode=0,
                   dropout_p: float = 0.0) -> Tuple[Tensor, Tensor]:
    """Per-crystal normalise/aggregate with stock torch ops: what the reference itself runs, on its
    kernel path too, whenever its fused operator does not apply -- numerics switch below 2, a
    normalisation other than the softmax over all keys, or dropout on the weights
    (models/indexed_lattice_multi_head_attention_cuda.py:231-306).  Returns (output, weights (E,H))."""
    logits = (q[edges[0]] * k[edges[1]]).sum(dim=-1)
    sizes = torch.zeros(int(batch.max().item()) + 1, dtype=torch.long, device=q.device)
    sizes.scatter_add_(0, batch, torch.ones_like(batch))
    sizes = sizes.tolist()
    esz = [s * s for s in sizes]

    def row_softmax(x):
        return torch.cat([F.softmax(a.view(s, s, -1), dim=1).view(s * s, -1)
                          for a, s in zip(torch.split_with_sizes(x, esz), sizes)])
    mode = NORM_FUNC_MODES.get(norm_func_mode, norm_func_mode)
    mode = abs(mode) if isinstance(mode, int) else mode
    w = 0 if bias is None else bias
    if mode == 0:
        prob = row_softmax(logits + w)                       # softmax over all keys of the crystal
    elif mode == 1:
        prob = row_softmax(logits) * torch.exp(w) if bias is not None else row_softmax(logits)
    elif mode == 2:
        prob = torch.exp(logits + w)
    elif mode in (3, 4, 5, 6, 7, 8):
        f = {3: lambda x: x, 4: torch.sigmoid, 5: F.softplus, 6: F.elu, 7: lambda x: F.elu(x) + 1, 8: torch.abs}[mode]
        prob = f(logits) * (torch.exp(w) if bias is not None else 1.0)
    else:
        raise ValueError(f"norm_func_mode must be 0 to 8 but {norm_func_mode} is given.")
    if dropout_p > 0.0:
        prob = F.dropout(prob, p=dropout_p)
    msg = v[edges[1]] if values is None else v[edges[1]] + values
    msg = prob[..., None] * msg
    out = torch.cat([m.view((s, s) + m.shape[1:]).sum(dim=1)
                     for m, s in zip(torch.split_with_sizes(msg, esz), sizes)])
    return out, prob


class CrystalformerMultiheadAttentionCUDA(Module):
    def __init__(self, embed_dim, num_heads, dropout=0., bias=True, kdim=None, vdim=None,
                 params: LatticeformerParams = LatticeformerParams(), device=None, dtype=None) -> None:
        kw = {"device": device, "dtype": dtype}
        super().__init__()
        assert params.domain in ("real", "reci", "RECI", "multihead", "no")
        if params.domain == "multihead":
            assert num_heads % 2 == 0, "multihead: each domain takes half of the heads"
        self.embed_dim = embed_dim
        self.kdim = kdim * num_heads if kdim is not None and kdim > 0 else embed_dim
        self.vdim = vdim * num_heads if vdim is not None and vdim > 0 else embed_dim
        self.params = params
        self.gauss_scale = Parameter(torch.zeros(2, **kw), requires_grad=False)
        self.atten_scale = Parameter(torch.zeros(1, **kw), requires_grad=False)
        self.num_heads = num_heads
        self.dropout = dropout
        self.head_dim = embed_dim // num_heads
        assert self.head_dim * num_heads == embed_dim, "embed_dim must be divisible by num_heads"

        self.q_proj_weight = Parameter(torch.empty((self.kdim, embed_dim), **kw))
        self.k_proj_weight = Parameter(torch.empty((self.kdim, embed_dim), **kw))
        self.v_proj_weight = Parameter(torch.empty((self.vdim, embed_dim), **kw))
        if bias:
            self.in_proj_bias = Parameter(torch.empty(self.kdim * 2 + self.vdim, **kw))
        else:
            self.register_parameter("in_proj_bias", None)
        self.out_proj = torch.nn.Linear(self.vdim, embed_dim, bias=bias, **kw)

        if params.domain == "no":
            self.lattice_pos_weights = None
        elif params.gauss_state.startswith("q") or params.gauss_state == "1":
            self.lattice_pos_weights = Parameter(torch.empty((self.kdim), **kw))
        elif params.gauss_state == "x-xn":
            # two factors, multiplied in forward (models/indexed_lattice_multi_head_attention_cuda.py:859-861, 993-997)
            self.lattice_pos_weights = Parameter(torch.empty((self.kdim, embed_dim), **kw))
            self.lattice_pos_weights2 = Parameter(torch.empty((self.kdim), **kw))
        elif params.gauss_state.startswith("x"):
            self.lattice_pos_weights = Parameter(torch.empty((num_heads, embed_dim), **kw))
        else:
            raise NotImplementedError(f"gauss_state={params.gauss_state!r}")

        heads = num_heads if params.value_pe_headed else 1
        cond = 1 if params.value_pe_condproj == "no" else ATOM_NUM
        self.pe_dist_proj = None
        self.pe_wave_proj = None
        # (models/indexed_lattice_multi_head_attention_cuda.py:869-878: the reciprocal-space blocks own a
        # projection too when value_pe_dist_reci > 0, although their kernel path yields no value encoding)
        bins = params.value_pe_dist_real if params.domain in ("real", "multihead") else \
            (params.value_pe_dist_reci if params.domain in ("reci", "RECI") else 0)
        if bins > 0:
            self.pe_dist_proj = Parameter(torch.empty(cond, heads, self.head_dim, bins, **kw))
        waves = params.value_pe_wave_real if params.domain in ("real", "multihead") else \
            (params.value_pe_wave_reci if params.domain in ("reci", "RECI") else 0)
        if waves > 0:
            # As on the reference's kernel path (models/indexed_lattice_multi_head_attention_cuda.py:872-878,
            # 600-614, 938-947): the parameter exists, is initialised in the same order and travels in the
            # state_dict, and nothing computes a value encoding from it (only the reference's PyTorch path
            # evaluates the plane-wave encodings).
            self.pe_wave_proj = Parameter(torch.empty(cond, heads, self.head_dim, waves ** 3, **kw))
            warnings.warn("value_pe_wave_* > 0: pe_wave_proj is kept for state_dict compatibility and has no effect "
                          "on the output, as on the reference's kernel path", stacklevel=2)
        self._reset_parameters()

    def position_weights(self) -> Optional[Tensor]:
        """The weights that turn a query (or the block input) into the Gaussian exponents' raw value:
        the parameter itself, or for ``gauss_state="x-xn"`` the product of its two factors, (H, embed_dim)
        (models/indexed_lattice_multi_head_attention_cuda.py:992-997)."""
        W = self.lattice_pos_weights
        if W is not None and self.params.gauss_state == "x-xn":
            H, K, D = self.num_heads, self.kdim, self.embed_dim
            W = (self.lattice_pos_weights2.view(H, 1, K // H) @ W.reshape(H, K // H, D)).reshape(H, D)
        return W

    def _reset_parameters(self):
        xavier_uniform_(self.q_proj_weight)
        xavier_uniform_(self.k_proj_weight)
        xavier_uniform_(self.v_proj_weight)
        xavier_uniform_(self.out_proj.weight)
        if self.in_proj_bias is not None:
            constant_(self.in_proj_bias, 0.)
            constant_(self.out_proj.bias, 0.)
        if self.lattice_pos_weights is not None:
            gs = self.params.gauss_state
            if gs in ("q", "q-headdim", "1"):
                normal_(self.lattice_pos_weights, 0., (self.kdim // self.num_heads) ** -0.5)
            elif gs == "q-kdim":
                normal_(self.lattice_pos_weights, 0., self.kdim ** -0.5)
            elif gs in ("x", "x-norm"):
                normal_(self.lattice_pos_weights, 0., self.embed_dim ** -0.5)
            elif gs == "x-xavier":
                xavier_uniform_(self.lattice_pos_weights)
            elif gs == "x-xn":
                xavier_uniform_(self.lattice_pos_weights)
                normal_(self.lattice_pos_weights2, 0., (self.kdim // self.num_heads) ** -0.5)
            elif gs == "x-xn2":
                # the product of the two factors of "x-xn", drawn once
                # (models/indexed_lattice_multi_head_attention_cuda.py:905-915)
                H, K, D = self.num_heads, self.kdim, self.embed_dim
                W = self.lattice_pos_weights
                W1 = torch.empty((K, D), device=W.device, dtype=W.dtype)
                W2 = torch.empty((H, 1, K // H), device=W.device, dtype=W.dtype)
                xavier_uniform_(W1)
                normal_(W2, 0., (K // H) ** -0.5)
                with torch.no_grad():
                    W.copy_((W2 @ W1.reshape(H, K // H, D)).reshape_as(W))
            else:
                raise NotImplementedError(gs)
        if self.pe_dist_proj is not None:
            with torch.no_grad():
                for idx, W in enumerate(self.pe_dist_proj):
                    if idx != 0 and self.params.value_pe_condproj in ("I", "J", "IJ"):
                        W.set_(self.pe_dist_proj[0])
                    else:
                        flat = W.view(-1, W.shape[-1])
                        xavier_uniform_(flat, flat.shape[1] ** -0.5)
        if self.pe_wave_proj is not None:
            with torch.no_grad():
                for idx, W in enumerate(self.pe_wave_proj):
                    if idx != 0 and self.params.value_pe_condproj in ("I", "J", "IJ"):
                        W.set_(self.pe_wave_proj[0])
                    else:
                        flat = W.view(-1, W.shape[-1])
                        xavier_uniform_(flat, flat.shape[1] ** -0.5)

    def forward(self, query: Tensor, key: Tensor, value: Tensor, batch_q: Tensor, batch_kv: Tensor,
                edges: Tensor, points: Tensor, dist2_min: Optional[Tensor], tvecs: Tensor,
                kr_base: Optional[Tensor] = None, rvecs: Optional[Tensor] = None,
                vcell: Optional[Tensor] = None, onehot: Optional[Tensor] = None,
                need_weights: bool = True, residual: Optional[Tensor] = None) -> Tuple[Tensor, Optional[Tensor]]:
        """Same arguments as the reference module; ``residual`` (an extension, default None)
        is added to the output projection, in its epilogue on the inference path."""
        P = self.params
        H = self.num_heads
        n = query.shape[0]
        kd, vd = self.kdim, self.vdim
        b_q = b_k = b_v = None
        if self.in_proj_bias is not None:
            b_q, b_k, b_v = self.in_proj_bias.split([kd, kd, vd])
        fused_linear = (query is key and key is value and kd == vd
                        and inference_only(query, self.q_proj_weight, self.k_proj_weight, self.v_proj_weight,
                                           self.in_proj_bias, self.out_proj.weight, self.out_proj.bias, residual)
                        and ops.linear_rows_supported(query, self.q_proj_weight, self.k_proj_weight,
                                                      self.v_proj_weight)
                        and vd % 16 == 0)
        # the same launches with autograd, inside a graphed training step
        fused_train = (not fused_linear and hip_funcs.USE_LINEAR_FUNCTION and torch.is_grad_enabled()
                       and query is key and key is value and kd == vd and vd % 16 == 0
                       and ops.linear_rows_supported(query, self.q_proj_weight, self.k_proj_weight,
                                                     self.v_proj_weight))
        if fused_linear:
            # the three projections in one launch
            q, k, v = ops.linear_rows(query, (self.q_proj_weight, self.k_proj_weight, self.v_proj_weight),
                                      self.in_proj_bias)
            q, k, v = q.view(n, H, kd // H), k.view(n, H, kd // H), v.view(n, H, vd // H)
        elif fused_train:
            # a residual that is the input itself rides through the projection node (see its docstring)
            carry = residual is query and query.is_contiguous()
            out = hip_funcs.FusedLinearHIP.apply(query, self.in_proj_bias, None, False, carry, self.q_proj_weight,
                                                 self.k_proj_weight, self.v_proj_weight)
            q, k, v = out[:3]
            if carry:
                residual = out[3]
            q, k, v = q.view(n, H, kd // H), k.view(n, H, kd // H), v.view(n, H, vd // H)
        else:
            q = linear_hip(query, self.q_proj_weight, b_q).contiguous().view(n, H, kd // H)
            k = linear_hip(key, self.k_proj_weight, b_k).contiguous().view(key.shape[0], H, kd // H)
            v = linear_hip(value, self.v_proj_weight, b_v).contiguous().view(value.shape[0], H, vd // H)

        bias = values = qs = None
        if P.domain in ("reci", "RECI", "multihead"):
            bias, values, qs = self._reciprocal_domains(q, query, batch_q, edges, points, dist2_min, tvecs,
                                                        kr_base, rvecs, vcell, onehot)
        if P.domain == "real":
            proj = self.pe_dist_proj
            if proj is not None and P.value_pe_condproj != "no":
                proj = conditional_projection(proj, onehot, edges, P.value_pe_condproj)
            spec = fused_exponents_spec(P) if q.is_cuda else None
            if spec is not None:
                # alpha, its normalisation, the positive map and the query scaling in two launches
                a, qs = hip_funcs.call(
                    GaussianExponentsHIP, q, self.lattice_pos_weights, self.gauss_scale, P.normalize_gauss,
                    self.training, spec[0], spec[1], P.gauss_lb_real, -0.5 * P.scale_real ** -2,
                    1.0 / math.sqrt(q.shape[-1]))
            else:
                a = gaussian_exponents(q, query, self.position_weights(), self.gauss_scale, P, self.training)
            dist_max = P.value_pe_dist_max
            if dist_max < 0:
                dist_max = (-dist_max) * P.scale_real
            adaptive = ()
            if P.adaptive_cutoff_sigma != 0:
                # lengths of the reciprocal vectors; the encoder passes them precomputed as (B,3)
                rvlen = rvecs if rvecs.dim() == 2 else torch.norm(rvecs, 2, dim=-1)
                cutoff = P.adaptive_cutoff_sigma if P.adaptive_cutoff_sigma < 0 else \
                    P.scale_real * P.gauss_lb_real ** (-0.5) * P.adaptive_cutoff_sigma
                adaptive = (rvlen, cutoff)
            if proj is not None and not P.value_pe_headed:
                proj = proj.expand(proj.shape[0], H, proj.shape[2], proj.shape[3])
            attn = None
            if (P.value_pe_dist_real <= 0 and qs is not None and not need_weights and P.norm_func_mode == 0
                    and config.REPRODUCIBLITY_STATE >= 2 and batch_q is batch_kv and not torch.is_grad_enabled()
                    and not (self.training and self.dropout > 0.0)):     # (dropout on the weights: the loop below)
                # no value bins and nobody asks for the bias: lattice sums and attention in one launch
                attn = hip_funcs.fused_encoding_attention(a, points, tvecs, batch_q, edges, qs, k, v, *adaptive)
            if attn is None:
                enc = RealPeriodicEncodingWithProjFuncCUDA if P.use_low_memory else RealPeriodicEncodingFuncCUDA
                # every positive map keeps rho >= gauss_lb, so no exponent of this block lies above this bound
                # (it lets the encoding share its staged translations between the blocks of a model)
                # (a few ulps of slack for the positive map's own rounding)
                weakest = -0.5 * P.gauss_lb_real * P.scale_real ** -2 * (1 - 1e-5)
                out = hip_funcs.call(enc, a, points, dist2_min, tvecs, batch_q, edges, P.value_pe_dist_real,
                                     dist_max, P.value_pe_width_scale, proj, *(adaptive or (None, None)), weakest)
                bias = out[0]
                values = out[1] if len(out) >= 2 else None
            else:
                return self._project_output(attn, n, vd, fused_linear, fused_train, residual, need_weights, None)

        if qs is None:
            qs = q / math.sqrt(q.shape[-1])
        weights = None
        dropout_p = self.dropout if self.training else 0.0
        plain = P.norm_func_mode in (0, "default") and dropout_p == 0.0
        if not plain or config.REPRODUCIBLITY_STATE < 2 or batch_q is not batch_kv:
            # other normalisations, dropout on the weights, or the numerics switch: the per-crystal
            # torch loop, as in the reference
            attn, prob = loop_attention(qs, k, v, batch_q, edges, bias, values, P.norm_func_mode, dropout_p)
            if isinstance(P.norm_func_mode, int) and P.norm_func_mode < 0:
                attn = attn * self._attention_scale(prob, batch_q)
            if need_weights:
                weights = prob.detach().mean(dim=1)
        elif need_weights:
            # softmax weights averaged over the heads, (E,), as the reference's loop path returns them
            # (models/indexed_lattice_multi_head_attention_cuda.py:782-786)
            attn, prob = hip_funcs.call(hip_funcs.FusedDotProductAttentionWithWeights, qs, k, v, bias, values,
                                        batch_q, edges)
            weights = prob.mean(dim=1)
        else:
            attn = hip_funcs.call(FusedDotProductAttentionCUDA, qs, k, v, bias, values, batch_q, edges)
        return self._project_output(attn, n, vd, fused_linear, fused_train, residual, need_weights,
                                    weights if need_weights else values)

    def _attention_scale(self, prob: Tensor, batch_q: Tensor) -> Tensor:
        """Negative norm_func_mode: outputs times the stored scale, or the reciprocal of the mean (over
        crystals, of the mean over queries and heads) total |weight| per query, stored once in training
        (models/indexed_lattice_multi_head_attention_cuda.py:760-777)."""
        if bool(self.atten_scale[0] > 0):
            return self.atten_scale[0]
        sizes = torch.zeros(int(batch_q.max().item()) + 1, dtype=torch.long, device=prob.device)
        sizes.scatter_add_(0, batch_q, torch.ones_like(batch_q))
        sizes = sizes.tolist()
        parts = torch.split_with_sizes(prob.detach().abs(), [s * s for s in sizes])
        scale = torch.stack([x.view(s, s, -1).sum(dim=1).mean() for x, s in zip(parts, sizes)]).mean().reciprocal()
        if self.training:
            with torch.no_grad():
                self.atten_scale[0] = scale
        return scale

    def _project_output(self, attn, n, vd, fused_linear, fused_train, residual, need_weights, values):
        attn = attn.contiguous().view(n, vd)
        if fused_linear:
            attn, = ops.linear_rows(attn, (self.out_proj.weight,), self.out_proj.bias, residual=residual)
        elif fused_train and ops.linear_rows_supported(attn, self.out_proj.weight):
            attn, = hip_funcs.FusedLinearHIP.apply(attn, self.out_proj.bias, residual, False, False,
                                                   self.out_proj.weight)
        else:
            attn = linear_hip(attn, self.out_proj.weight, self.out_proj.bias)
            if residual is not None:
                attn = residual + attn
        return attn, values


    def _real_encoding(self, a: Tensor, proj: Optional[Tensor], heads: int, batch_q, edges, points, dist2_min,
                       tvecs, rvecs, onehot):
        """Real-space bias and value encoding for ``heads`` heads with exponents ``a``
        (models/indexed_lattice_multi_head_attention_cuda.py:393-421, 694-723)."""
        P = self.params
        if proj is not None and P.value_pe_condproj != "no":
            proj = conditional_projection(proj, onehot, edges, P.value_pe_condproj)
        dist_max = P.value_pe_dist_max
        if dist_max < 0:
            dist_max = (-dist_max) * P.scale_real
        adaptive = ()
        if P.adaptive_cutoff_sigma != 0:
            rvlen = rvecs if rvecs.dim() == 2 else torch.norm(rvecs, 2, dim=-1)
            cutoff = P.adaptive_cutoff_sigma if P.adaptive_cutoff_sigma < 0 else \
                P.scale_real * P.gauss_lb_real ** (-0.5) * P.adaptive_cutoff_sigma
            adaptive = (rvlen, cutoff)
        if proj is not None and proj.shape[1] == 1 and heads > 1:
            proj = proj.expand(proj.shape[0], heads, proj.shape[2], proj.shape[3])
        enc = RealPeriodicEncodingWithProjFuncCUDA if P.use_low_memory else RealPeriodicEncodingFuncCUDA
        out = enc.apply(a.contiguous(), points, dist2_min, tvecs, batch_q, edges, P.value_pe_dist_real, dist_max,
                        P.value_pe_width_scale, proj, *adaptive)
        return out[0], (out[1] if len(out) >= 2 else None)

    def _reciprocal_domains(self, q, query, batch_q, edges, points, dist2_min, tvecs, kr_base, rvecs, vcell,
                            onehot):
        """Bias (and value encoding) of the blocks that involve the reciprocal-space lattice sum
        (models/indexed_lattice_multi_head_attention_cuda.py:724-746)."""
        P = self.params
        H = self.num_heads
        if kr_base is None or rvecs is None or rvecs.dim() != 3 or vcell is None:
            raise ValueError("reciprocal-space blocks need kr_base (E,3), rvecs (B,3,3) and vcell (B)")
        coef_real, coef_reci = -0.5 * P.scale_real ** -2, -0.5 * P.scale_reci ** 2
        qs = None
        spec = fused_exponents_spec(P) if q.is_cuda else None
        if spec is not None and (P.domain == "reci" or
                                 (P.domain == "multihead" and P.gauss_lb_real == P.gauss_lb_reci)):
            # rho(normalised alpha) and the scaled query from the fused kernel (two launches);
            # the domains differ in the factor applied to rho only
            rho, qs = GaussianExponentsHIP.apply(
                q, self.lattice_pos_weights, self.gauss_scale, P.normalize_gauss, self.training, spec[0], spec[1],
                P.gauss_lb_reci, 1.0, 1.0 / math.sqrt(q.shape[-1]))
            if P.domain == "reci":
                return ReciPeriodicEncodingFuncCUDA.apply(rho * coef_reci, kr_base, rvecs, vcell, batch_q,
                                                          edges), None, qs
            a1, a2 = rho[:, :H // 2] * coef_real, rho[:, H // 2:] * coef_reci
        else:
            func = make_positive_func(P.positive_func)
            alpha = normalised_alpha(q, query, self.position_weights(), self.gauss_scale, P, self.training)
            if P.domain == "reci":
                a = func(alpha, P.gauss_lb_reci) * coef_reci
                return ReciPeriodicEncodingFuncCUDA.apply(a, kr_base, rvecs, vcell, batch_q, edges), None, qs
            if P.domain == "RECI":
                a = 1 / func(alpha, P.gauss_lb_reci) * coef_reci
                return ReciPeriodicEncodingFuncCUDA.apply(a, kr_base, rvecs, vcell, batch_q, edges), None, qs
            a1, a2 = alpha.chunk(2, 1)
            a1 = func(a1, P.gauss_lb_real) * coef_real
            a2 = func(a2, P.gauss_lb_reci) * coef_reci
        # multihead: first half of the heads in real space, second half in reciprocal space
        proj = self.pe_dist_proj[:, :H // 2] if self.pe_dist_proj is not None else None
        w1, v1 = self._real_encoding(a1, proj, H // 2, batch_q, edges, points, dist2_min, tvecs, rvecs, onehot)
        w2 = ReciPeriodicEncodingFuncCUDA.apply(a2.contiguous(), kr_base, rvecs, vcell, batch_q, edges)
        bias = torch.cat([w1, w2], dim=1)
        values = None if v1 is None else torch.cat([v1, torch.zeros_like(v1)], dim=1)
        return bias, values, qs


CrystalformerMultiheadAttentionHIP = CrystalformerMultiheadAttentionCUDA
