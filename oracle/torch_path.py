"""CPU oracle: a from-scratch restatement of Crystalformer's *PyTorch path*.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package may import this
module; it is the checker for the HIP kernels (tests/, the smoke check and the
``cpu_baseline`` leg of the benchmark).  It runs on CPU tensors with stock
torch ops and is written for clarity, not speed.

What it restates (all paths relative to the reference checkout):

* edge indexing                 models/indexed_latticeformer_encoder.py:15-32
* rule-A lattice geometry       models/indexed_latticeformer_encoder.py:46-180, 450-452
* alpha pipeline                models/indexed_lattice_multi_head_attention.py:1291-1357
* lattice-sum bias (logsumexp)  models/indexed_lattice_multi_head_attention.py:309-355, 913-923
* Gaussian basis                models/indexed_lattice_multi_head_attention.py:613-621
* Gaussian value PE + proj      models/indexed_lattice_multi_head_attention.py:741-815, 1433-1445
* per-crystal softmax/aggregate models/indexed_lattice_multi_head_attention.py:140-272
* mean pooling                  models/pooling.py:19-25
* reciprocal-space geometry     models/indexed_latticeformer_encoder.py:138-161
* reciprocal-space lattice sum  models/indexed_lattice_multi_head_attention.py:925-950

The translation set here is the fixed cube n in [-r, r]^3 ("rule A").  The
adaptive per-head boxes of the device kernels ("rule B") live in
``oracle/kernel_semantics.py`` and ``oracle/kernels_ref.c``.

Parity pins (tests/test_oracle_*.py): brute-force Python loops in float64,
the factorised closed form for orthorhombic cells, r=0 special cases,
``torch.logsumexp`` / ``F.scaled_dot_product_attention`` library routines,
finite-difference gradient checks, and golden vectors written by importing the
reference itself (tests/golden/).  Every function below is covered by at least
one of those.

All differentiable functions are plain torch ops, so autograd supplies the
backward oracle (the reference's hand-written backward passes exist to save
memory, not to change the mathematics).
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

import torch
import torch.nn.functional as F
from torch import Tensor


# --------------------------------------------------------------------------
# integer indexing (bit-exact)
# --------------------------------------------------------------------------
def get_edge_index(sizes: Sequence[int] | Tensor) -> Tensor:
    """Dense intra-crystal edge list, query-major.

    Crystal with atom offset c and n atoms contributes (c+i, c+j) for
    i = 0..n-1 (outer), j = 0..n-1 (inner).
    Follows models/indexed_latticeformer_encoder.py:15-32.
    """
    if torch.is_tensor(sizes):
        sizes = sizes.tolist()
    src: List[Tensor] = []
    dst: List[Tensor] = []
    offset = 0
    for n in sizes:
        idx = torch.arange(offset, offset + n, dtype=torch.long)
        src.append(idx.repeat_interleave(n))
        dst.append(idx.repeat(n))
        offset += n
    if not src:
        return torch.zeros((2, 0), dtype=torch.long)
    return torch.stack((torch.cat(src), torch.cat(dst))).contiguous()


def edge_row_offsets(edges: Tensor, num_atoms: int) -> Tensor:
    """CSR offsets over the query index: cumsum(bincount(edges[0])) with a
    leading zero.  Follows models/cuda_funcs/fused_dpa.py:24-26."""
    start = torch.zeros(num_atoms + 1, dtype=torch.long)
    start.scatter_add_(0, edges[0] + 1, torch.ones_like(edges[0]))
    return start.cumsum(0)


def crystal_sizes(batch: Tensor, num_crystals: Optional[int] = None) -> Tensor:
    """Atoms per crystal from the flat batch index.
    Follows models/cuda_funcs/irregular_mean.py:29-32."""
    if num_crystals is None:
        num_crystals = int(batch.max().item()) + 1 if batch.numel() else 0
    sizes = torch.zeros(num_crystals, dtype=torch.long)
    sizes.scatter_add_(0, batch, torch.ones_like(batch))
    return sizes


def crystal_starts(sizes: Tensor) -> Tensor:
    """Leading-zero cumulative sum of ``sizes``.
    Follows models/cuda_funcs/irregular_mean.py:36."""
    return F.pad(torch.cumsum(sizes, 0), (1, 0))


# --------------------------------------------------------------------------
# geometry, rule A
# --------------------------------------------------------------------------
def translation_grid(lattice_range: int, dtype=torch.float32) -> Tensor:
    """(R,3) integer translations of the cube [-r,r]^3, first index slowest.
    Follows models/indexed_latticeformer_encoder.py:70-74 (meshgrid 'ij')."""
    g = torch.arange(-lattice_range, lattice_range + 1, dtype=dtype)
    return torch.stack(torch.meshgrid(g, g, g, indexing="ij"), dim=-1).reshape(-1, 3)


def det_3x3(m: Tensor) -> Tensor:
    """Determinant by cofactor expansion in the reference's term order
    (models/indexed_latticeformer_encoder.py:34-44)."""
    return (m[:, 0, 0] * m[:, 1, 1] * m[:, 2, 2]
            + m[:, 0, 1] * m[:, 1, 2] * m[:, 2, 0]
            + m[:, 0, 2] * m[:, 1, 0] * m[:, 2, 1]
            - m[:, 0, 2] * m[:, 1, 1] * m[:, 2, 0]
            - m[:, 0, 0] * m[:, 1, 2] * m[:, 2, 1]
            - m[:, 0, 1] * m[:, 1, 0] * m[:, 2, 2])


def reciprocal_vectors(trans: Tensor) -> Tuple[Tensor, Tensor]:
    """(B,3,3) reciprocal lattice rows 2*pi*(t2xt3, t3xt1, t1xt2)/V and the
    cell volume V.  Follows models/indexed_latticeformer_encoder.py:204-212."""
    vcell = det_3x3(trans)
    rec = torch.stack([
        torch.cross(trans[:, 1], trans[:, 2], dim=1),
        torch.cross(trans[:, 2], trans[:, 0], dim=1),
        torch.cross(trans[:, 0], trans[:, 1], dim=1),
    ], dim=1) * (2.0 * math.pi / vcell[:, None, None])
    return rec, vcell


def relative_positions(pos: Tensor, edges: Tensor) -> Tensor:
    """p_j - p_i per edge (models/indexed_latticeformer_encoder.py:98, 214)."""
    return pos[edges[1]] - pos[edges[0]]


def lattice_dist2(pos: Tensor, batch: Tensor, trans: Tensor, edges: Tensor,
                  lattice_range: int, e0: int = 0, e1: Optional[int] = None) -> Tensor:
    """dist2[e,r] = ||p_j - p_i + n_r . L_b||^2 for edges e0..e1, computed the
    way the reference's PyTorch path does: ``torch.norm`` first, then squared
    (models/indexed_latticeformer_encoder.py:97-100, 136, 450-452)."""
    e1 = edges.shape[1] if e1 is None else e1
    grid = translation_grid(lattice_range, pos.dtype)
    ei, ej = edges[0, e0:e1], edges[1, e0:e1]
    rel = pos[ej] - pos[ei]                              # (e,3)
    shifts = grid @ trans                                # (B,R,3)
    disp = rel[:, None] + shifts[batch[ei]]              # (e,R,3)
    dist = torch.norm(disp, dim=-1)
    return dist * dist


# --------------------------------------------------------------------------
# reciprocal space
# --------------------------------------------------------------------------
def reciprocal_half_terms(pos: Tensor, batch: Tensor, trans: Tensor, edges: Tensor,
                          lattice_range: int) -> Tuple[Tensor, Tensor, Tensor]:
    """(cos_kr (E,Rh), k2 (B,Rh), vcell (B)) over the half grid: the second half of the
    'ij'-ordered cube starting at its centre n = 0 (Rh = ((2r+1)^3 + 1) / 2 points), every
    cosine but the first doubled to stand for the mirrored point.  k2 through the Gram
    matrix of the reciprocal rows, as the reference prefers for accuracy.
    Follows models/indexed_latticeformer_encoder.py:138-161."""
    rec, vcell = reciprocal_vectors(trans)
    grid = translation_grid(lattice_range, pos.dtype)
    half = grid[grid.shape[0] // 2:]
    rel = relative_positions(pos, edges)
    b2e = batch[edges[0]]
    kr = (rel[:, None] @ rec.transpose(1, 2)[b2e]).squeeze(1)           # (E,3): <r, b_d>
    cos_kr = torch.cos((half @ kr[..., None]).squeeze(2))               # (E,Rh)
    cos_kr[:, 1:] += cos_kr[:, 1:]
    gram = rec @ rec.transpose(1, 2)                                    # (B,3,3)
    outer = half[:, :, None] @ half[:, None, :]                         # (Rh,3,3)
    k2 = (gram[:, None] * outer[None]).sum(dim=(2, 3))                  # (B,Rh)
    return cos_kr, k2, vcell


def reciprocal_bias(alpha: Tensor, cos_kr: Tensor, k2: Tensor, vcell: Tensor, edges0: Tensor,
                    batch: Tensor) -> Tensor:
    """z[e,h] = log(max(sum_k exp(a[i,h] k^2) cos(k.r), 1e-6)) + 1.5 log(-4 pi a[i,h]) - log V.
    Follows models/indexed_lattice_multi_head_attention.py:925-950."""
    alpha_k2 = alpha.unsqueeze(2) * k2.unsqueeze(1)[batch]              # (N,H,Rh)
    s = (torch.exp(alpha_k2)[edges0] * cos_kr.unsqueeze(1)).sum(dim=-1)
    z = torch.log(s.clamp(min=1e-6))
    log_ci = 1.5 * torch.log((-4 * math.pi) * alpha) - torch.log(vcell)[batch, None]
    return z + log_ci[edges0]


def kr_base(pos: Tensor, batch: Tensor, trans: Tensor, edges: Tensor) -> Tensor:
    """(E,3) phases <b_d, p_j - p_i> handed to the reciprocal-space kernels
    (models/indexed_latticeformer_encoder.py:245-251)."""
    rec, _ = reciprocal_vectors(trans)
    rel = relative_positions(pos, edges)
    return (rec[batch[edges[0]]] @ rel[..., None]).squeeze(2)


# --------------------------------------------------------------------------
# alpha pipeline
# --------------------------------------------------------------------------
def positive_elu(x: Tensor, lower_bound: float, beta: float) -> Tensor:
    """rho = (1-lb)*elu(x*beta/(1-lb)) + 1  ('elu=beta').
    Follows models/indexed_lattice_multi_head_attention.py:1337-1339."""
    return (1.0 - lower_bound) * F.elu(x * (beta / (1.0 - lower_bound))) + 1.0


def normalised_alpha(q: Tensor, lattice_pos_weights: Tensor, gauss_scale: Tensor,
                     training: bool, normalize: bool) -> Tensor:
    """alpha[i,h] = q_h . w_h, shifted and scaled by the stored or the batch statistics.

    q is the *unscaled* query (N,H,D).  When ``gauss_scale[0]`` is not
    positive the normalisation uses the statistics of this very batch
    (unbiased std over all N*H entries), and in training mode stores them
    once.  Follows models/indexed_lattice_multi_head_attention.py:1300-1330.
    """
    n, h, d = q.shape
    alpha = (q.reshape(n, h, 1, d) @ lattice_pos_weights.reshape(h, d, 1)).view(n, h)
    if normalize:
        if bool(gauss_scale[0] > 0):
            scale, shift = gauss_scale[0], gauss_scale[1]
        else:
            scale = torch.reciprocal(alpha.detach().std())
            shift = -alpha.detach().mean()
            if training:
                with torch.no_grad():
                    gauss_scale[0] = scale
                    gauss_scale[1] = shift
        alpha = (alpha + shift) * scale
    return alpha


def gaussian_exponents(q: Tensor, lattice_pos_weights: Tensor, gauss_scale: Tensor,
                       training: bool, normalize: bool, lower_bound: float,
                       beta: float, scale_real: float) -> Tensor:
    """a[i,h] = -rho(normalised q_h . w_h) / (2 r0^2)   (negative).
    Follows models/indexed_lattice_multi_head_attention.py:1300-1357.
    """
    n, h, d = q.shape
    alpha = (q.reshape(n, h, 1, d) @ lattice_pos_weights.reshape(h, d, 1)).view(n, h)
    if normalize:
        if bool(gauss_scale[0] > 0):
            scale, shift = gauss_scale[0], gauss_scale[1]
        else:
            scale = torch.reciprocal(alpha.detach().std())
            shift = -alpha.detach().mean()
            if training:
                with torch.no_grad():
                    gauss_scale[0] = scale
                    gauss_scale[1] = shift
        alpha = (alpha + shift) * scale
    return positive_elu(alpha, lower_bound, beta) * (-0.5 * scale_real ** -2)


# --------------------------------------------------------------------------
# periodic encoding on a materialised dist2 (rule A)
# --------------------------------------------------------------------------
def lattice_logsumexp(alpha_e: Tensor, dist2: Tensor) -> Tensor:
    """z[e,h] = log sum_r exp(a[e,h] * dist2[e,r]).
    Follows models/indexed_lattice_multi_head_attention.py:913-923, 309-325."""
    return torch.logsumexp(dist2[:, None, :] * alpha_e[:, :, None], dim=-1)


def gaussian_basis(dist2: Tensor, dist_max: float, K: int, width_scale: float) -> Tensor:
    """g[e,r,k] = exp(-((k*m/K - sqrt(dist2)) / (sqrt2*ws*m/K))^2), k = 1..K.
    Follows models/indexed_lattice_multi_head_attention.py:613-621."""
    centers = torch.arange(1, K + 1, dtype=dist2.dtype) * (dist_max / K)
    t = (centers - dist2[..., None] ** 0.5) / ((2 ** 0.5) * (width_scale * dist_max / K))
    return torch.exp(-(t * t))


def gaussian_value_average(alpha_e: Tensor, dist2: Tensor, dist_max: float, K: int,
                           width_scale: float) -> Tensor:
    """s[e,h,k] = sum_r softmax_r(a*dist2)[r] * g[e,r,k]   -> (e,H,K).
    Follows models/indexed_lattice_multi_head_attention.py:754-773."""
    p = torch.softmax(dist2[:, None, :] * alpha_e[:, :, None], dim=-1)   # (e,H,R)
    g = gaussian_basis(dist2, dist_max, K, width_scale)                   # (e,R,K)
    return p @ g


def project_value_pe(s: Tensor, W: Tensor) -> Tensor:
    """v[e,h,:] = W_h s[e,h,:];  W is (H,D,K), (1,H,D,K) or (E,H,D,K).
    Follows models/indexed_lattice_multi_head_attention.py:776-798."""
    if W.dim() == 3:
        W = W[None]
    return (W @ s[..., None]).squeeze(-1)


def periodic_encoding(alpha: Tensor, pos: Tensor, batch: Tensor, trans: Tensor,
                      edges: Tensor, lattice_range: int, K: int = 0,
                      dist_max: float = 0.0, width_scale: float = 1.0,
                      W: Optional[Tensor] = None,
                      chunk_elems: int = 1 << 26) -> Tuple[Tensor, Optional[Tensor]]:
    """Bias z (E,H) and value PE (E,H,K) / (E,H,D) for all edges, evaluated in
    chunks of edges so that the (e,R,K) temporary stays bounded.  Chunking does
    not change any per-edge arithmetic."""
    E = edges.shape[1]
    R = (2 * lattice_range + 1) ** 3
    step = max(1, chunk_elems // (R * max(K, alpha.shape[1], 1)))
    zs, vs = [], []
    for e0 in range(0, E, step):
        e1 = min(E, e0 + step)
        d2 = lattice_dist2(pos, batch, trans, edges, lattice_range, e0, e1)
        a_e = alpha[edges[0, e0:e1]]
        zs.append(lattice_logsumexp(a_e, d2))
        if K > 0:
            s = gaussian_value_average(a_e, d2, dist_max, K, width_scale)
            if W is not None:
                Wc = W
                if W.dim() == 4 and W.shape[0] == E:
                    Wc = W[e0:e1]
                s = project_value_pe(s, Wc)
            vs.append(s)
    H = alpha.shape[1]
    z = torch.cat(zs) if zs else alpha.new_zeros((0, H))
    if K <= 0:
        return z, None
    if vs:
        return z, torch.cat(vs)
    last = K if W is None else W.shape[-2]
    return z, alpha.new_zeros((0, H, last))


# --------------------------------------------------------------------------
# edge-indexed attention and pooling
# --------------------------------------------------------------------------
def indexed_attention(q: Tensor, k: Tensor, v: Tensor, sizes: Sequence[int],
                      edges: Tensor, bias: Optional[Tensor],
                      values: Optional[Tensor]) -> Tuple[Tensor, Tensor]:
    """Per-crystal softmax over keys and aggregation of (v_j + values_ij).

    q (N,H,D) is the *unscaled* query; the 1/sqrt(D) factor is applied here.
    Returns (out (N,H,D), prob (E,H)).
    Follows models/indexed_lattice_multi_head_attention.py:176-178, 209-213,
    249-254."""
    if torch.is_tensor(sizes):
        sizes = sizes.tolist()
    qs = q / math.sqrt(q.shape[-1])
    logits = (qs[edges[0]] * k[edges[1]]).sum(-1)
    if bias is not None:
        logits = logits + bias
    esz = [n * n for n in sizes]
    prob = torch.cat([F.softmax(a.view(n, n, -1), dim=1).view(n * n, -1)
                      for a, n in zip(torch.split_with_sizes(logits, esz), sizes)]) \
        if len(sizes) else logits
    msg = v[edges[1]] if values is None else v[edges[1]] + values
    msg = prob[..., None] * msg
    out = torch.cat([m.view((n, n) + m.shape[1:]).sum(dim=1)
                     for m, n in zip(torch.split_with_sizes(msg, esz), sizes)]) \
        if len(sizes) else msg
    return out, prob


def avr_pool(x: Tensor, sizes: Sequence[int]) -> Tensor:
    """Per-crystal mean over atoms (models/pooling.py:19-25)."""
    if torch.is_tensor(sizes):
        sizes = sizes.tolist()
    return torch.stack([torch.mean(c, dim=0) for c in torch.split_with_sizes(x, sizes, 0)])


def l1_training_loss(pred: Tensor, target: Tensor) -> Tensor:
    """Scalar training loss: per-sample L1 losses summed over the target columns
    (losses/regression_loss.py:17-20, loss_fn "l1"), then the mean over the batch
    (models/regression.py:117-118).  ``pred`` and ``target`` are (B, T)."""
    loss = 0
    for i in range(pred.shape[1]):
        loss = loss + F.l1_loss(pred[:, i], target[:, i], reduction="none")
    return loss.mean()
