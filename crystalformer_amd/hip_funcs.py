"""Operator boundary: the ``torch.autograd.Function`` classes and the compile hook
that Crystalformer's attention module imports from its ``cuda_funcs`` package
(models/cuda_funcs/__init__.py:12-27), served by the gfx950 kernels.

Same class names, positional arguments, outputs and gradients as the
reference, so ``from crystalformer_amd.hip_funcs import *`` can stand in for
``from .cuda_funcs import *``:

* ``RealPeriodicEncodingFuncCUDA``          models/cuda_funcs/real_space_enc.py:17-247
* ``RealPeriodicEncodingWithProjFuncCUDA``  models/cuda_funcs/real_space_enc_proj.py:18-178
* ``FusedDotProductAttentionCUDA``          models/cuda_funcs/fused_dpa.py:17-208
* ``IrregularMeanCUDA``                     models/cuda_funcs/irregular_mean.py:19-69
* ``compile_kernels`` / ``KernelManager``   models/cuda_funcs/kernel_manager.py:24-134

Differences by design: kernels are built ahead of time, so ``compile_kernels``
only records the constants the reference substitutes into its sources
(lattice range, minimum range) and checks that the library supports the shapes;
there is no limit on atoms per crystal; ``gW`` comes back already reduced to the
shape of ``W``.
"""
from __future__ import annotations

from typing import Optional

import torch
from torch import Tensor

from . import lib as _lib
from . import ops

__all__ = [
    "KernelManager", "Kernel", "compile_kernels", "CUPY_AVAILABLE", "HIP_AVAILABLE",
    "RealPeriodicEncodingFuncCUDA", "RealPeriodicEncodingWithProjFuncCUDA",
    "FusedDotProductAttentionCUDA", "IrregularMeanCUDA", "compute_minimum_distance",
    "ReciPeriodicEncodingFuncCUDA", "fused_encoding_attention",
]


def _hip_available() -> bool:
    return _lib.is_built() and torch.cuda.is_available()


HIP_AVAILABLE = _hip_available()
# The reference gates its kernel path on this flag (models/latticeformer.py:139-143).
CUPY_AVAILABLE = HIP_AVAILABLE


class Kernel:
    """A named entry point of the HIP library: the counterpart of the reference's holder of one
    compiled CuPy kernel (models/cuda_funcs/kernel_manager.py:15-22).  ``Kernel(name)(grid, block,
    args)`` keeps the reference's call shape; the launch geometry is the library's own business, so
    ``grid`` and ``block`` are ignored and ``args`` (raw pointers, sizes, stream handle) go to the C
    function, whose status code is returned.  ``Kernel(name)(*args)`` does the same."""

    def __init__(self, name: str):
        self.name = name
        self.code = None            # (no source text: the library is built ahead of time)
        self.raw_kernel = None

    def __call__(self, *call_args, **_ignored):
        if self.raw_kernel is None:
            self.raw_kernel = getattr(_lib.load(), self.name)
        if len(call_args) == 3 and isinstance(call_args[2], (tuple, list)):
            call_args = tuple(call_args[2])
        return self.raw_kernel(*call_args)


class KernelManager:
    """Constants shared by all launches, set by ``compile_kernels``."""
    LATTICE_RANGE: int = 2
    MINIMUM_RANGE: int = 0
    HEAD_NUM: int = 8
    K_HEAD_DIM: int = 16
    V_HEAD_DIM: int = 16
    VPE_DIM: int = 64
    # kept for code that reads them; the kernels have no per-crystal size limit
    MAX_SYSTEM_SIZE: int = 1 << 30
    MAX_SYSTEM_SIZE_POW2: int = 1 << 30
    RUNNING_SUM_LEN: int = 8
    # The edge list is the dense per-crystal block layout of get_edge_index
    # (edge (i,j) of a crystal with n atoms at e0 + i*n + j).  The reference's
    # transposes assume it too (models/cuda_funcs/fused_dpa.py:141-159).  With it
    # the encoding evaluates both directions of an atom pair together.  An edge
    # list is checked against that layout the first time it is seen: any other list
    # takes the per-edge kernels, and the attention backward raises for it.  False
    # forces the per-edge kernels.
    DENSE_EDGE_BLOCKS: bool = True
    # The reference's reciprocal-space backward kernel differentiates log(sum) only and drops
    # d/da of the normalisation term 1.5 log(-4 pi a) (models/kernels/reci_enc_bwd.cu:41-69),
    # unlike autograd on its PyTorch path.  False reproduces the kernel, True the full derivative.
    RECI_NORMALISATION_GRAD: bool = False
    # Blocks without Gaussian value bins (value_pe_dim 0), inference: lattice-sum bias and
    # attention in one launch, the bias never written to memory (fused_encoding_attention).
    FUSE_ENCODING_ATTENTION: bool = True
    # Inside a captured graph the two operators are the faster choice (measured on the 32-crystal
    # simplified model: 0.173 ms per replayed forward against 0.183 ms with the one-launch blocks,
    # whose work-group per atom is bound by its chain of dependent loads), eager launches gain
    # from the launch saved (0.55 against 0.78 ms), so capture keeps the two operators.
    FUSE_ENCODING_ATTENTION_IN_GRAPHS: bool = False
    # Fixed cube: the geometry-only part of the encoding (which translations reach a bin, in which
    # order, their distances) is staged once per forward pass and shared by all blocks
    # (ops.staged_rings).  Needs an upper bound of the exponents the rings will meet, which the
    # attention module passes with its call (-gauss_lb / (2 r0^2), the encoding Function's last
    # argument); without one every launch stages for itself.
    STAGED_RINGS: bool = True
    # Adaptive boxes from the staged rings (forward, up to 8 heads): the atom pairs whose half-widths all
    # come out as LATTICE_RANGE have exactly the cube and start from their rings, the others are staged by
    # the pair kernel; two stably ordered lists of units and their counts are worked out on the device,
    # and each kernel walks dense rounds of its own list, whatever the split is.
    ADAPTIVE_RINGS = True
    compiled: bool = False

    # The reference's kernel slots (models/cuda_funcs/kernel_manager.py:27-53), each naming the entry
    # point of the library that does that kernel's work (the *_v2 dynamic-parallelism variants and the
    # transposes, which nothing here needs, have none).
    real_enc_fwd: Kernel = Kernel("cf_real_enc_fwd")
    real_enc_bwd: Kernel = Kernel("cf_real_enc_bwd")
    real_enc_proj_fwd: Kernel = Kernel("cf_real_enc_fwd")
    real_enc_proj_bwd: Kernel = Kernel("cf_real_enc_bwd")
    reci_enc_fwd: Kernel = Kernel("cf_reci_enc_fwd")
    reci_enc_bwd: Kernel = Kernel("cf_reci_enc_bwd")
    fused_dpa_fwd: Kernel = Kernel("cf_fused_dpa_fwd")
    fused_dpa_fwd_v3: Kernel = Kernel("cf_fused_dpa_fwd")
    fused_dpa_bwd: Kernel = Kernel("cf_fused_dpa_bwd")
    fused_dpa_bwd_v3: Kernel = Kernel("cf_fused_dpa_bwd")
    fused_dpa_bwd_q: Kernel = Kernel("cf_fused_dpa_bwd")
    fused_dpa_bwd_q_v3: Kernel = Kernel("cf_fused_dpa_bwd")
    irregular_mean_fwd: Kernel = Kernel("cf_irregular_mean_fwd")
    minimum_distance: Kernel = Kernel("cf_minimum_distance")

    @staticmethod
    def get_kernel_names():
        """Names of the kernel slots (models/cuda_funcs/kernel_manager.py:60-66)."""
        return sorted(name for name, value in KernelManager.__dict__.items() if isinstance(value, Kernel))

    @staticmethod
    def get_kernel(name: str) -> "Kernel":
        return KernelManager.__dict__[name]

    @staticmethod
    def set_kernel(name: str, kernel: "Kernel") -> None:
        setattr(KernelManager, name, kernel)


def compile_kernels(lattice_range: int, head_num: int, key_head_dim: int, value_pe_dim: int,
                    value_head_dim: int, set_minimum_range: bool) -> None:
    """Record the launch constants (models/cuda_funcs/kernel_manager.py:109-134)
    and verify that the prebuilt library covers the requested shapes."""
    if head_num not in (1, 2, 4, 8, 16):
        raise _lib.CrystalformerHipError(f"head_num={head_num} not supported (1,2,4,8,16)")
    if not 0 <= value_pe_dim <= 128:
        raise _lib.CrystalformerHipError(f"value_pe_dim={value_pe_dim} outside 0..128")
    if value_pe_dim > 0 and not 1 <= value_head_dim <= 64:
        raise _lib.CrystalformerHipError(f"value_head_dim={value_head_dim} outside 1..64")
    KernelManager.LATTICE_RANGE = int(lattice_range)
    KernelManager.MINIMUM_RANGE = int(lattice_range) if set_minimum_range else 0
    KernelManager.HEAD_NUM = int(head_num)
    KernelManager.K_HEAD_DIM = int(key_head_dim)
    KernelManager.V_HEAD_DIM = int(value_head_dim)
    KernelManager.VPE_DIM = int(value_pe_dim)
    _lib.load()
    KernelManager.compiled = True


def _pairs(batch_i: Tensor, edge_ij_e: Tensor, tvecs_n: Tensor, K: int) -> Optional[Tensor]:
    if not KernelManager.DENSE_EDGE_BLOCKS or edge_ij_e.shape[1] == 0:
        return None
    return ops.cached_edge_pairs(batch_i, edge_ij_e, tvecs_n.shape[0])


def _w_leading(W_k: Optional[Tensor]) -> int:
    if W_k is None:
        return 0
    assert W_k.dim() in (3, 4)
    return 1 if W_k.dim() == 3 else W_k.shape[0]


class _NoGradCtx:
    """Stand-in for the autograd context when a Function's forward is called directly."""
    needs_input_grad = (False,) * 16

    def save_for_backward(self, *tensors):
        pass


def call(function, *args):
    """``function.apply(*args)``; with autograd switched off the forward is called directly,
    which spares the dispatch through the autograd machinery (several microseconds a call,
    thirteen calls in a forward of the four-block model)."""
    if torch.is_grad_enabled():
        return function.apply(*args)
    return function.forward(_NoGradCtx(), *args)


class _Absent:
    """Default of the optional trailing arguments of the encoding Functions: tells an argument that
    was not passed from one passed as None (backward returns one gradient per argument passed)."""

    def __repr__(self):
        return "<not passed>"


_ABSENT = _Absent()


def _optional_args(*values):
    """(values with the absent ones as None, number of them that were passed)."""
    return tuple(None if v is _ABSENT else v for v in values), sum(v is not _ABSENT for v in values)


def _enc_backward_tail(ga_ik, gW_k, optional_passed: int):
    return (ga_ik, None, None, None, None, None, None, None, None, gW_k) + (None,) * optional_passed


class RealPeriodicEncodingWithProjFuncCUDA(torch.autograd.Function):
    """z[e,h] = log sum_n exp(a[i,h] |r_ij + n.L|^2) and the Gaussian value
    encoding with the per-head projection fused into the kernel.

    Returns ``(z_ek,)`` when ``K <= 0`` else ``(z_ek, v_ekd)`` with v of shape
    (E,H,D) when ``W_k`` is given and (E,H,K) otherwise.
    """

    @staticmethod
    def forward(ctx, a_ik, rpos_ij_e, dist2_min_e, tvecs_n, batch_i, edge_ij_e, K, dist_max, wscale,
                W_k, rvlen_n=_ABSENT, cutoff_radius=_ABSENT, weakest_exponent=_ABSENT):
        """``weakest_exponent`` (an extension, after the reference's arguments): an upper bound
        (<= 0) of every entry of ``a_ik``, e.g. -gauss_lb / (2 r0^2).  With it the geometry-only part
        of the encoding is staged once per geometry and shared by the blocks of a model
        (:func:`crystalformer_amd.ops.staged_rings`); without, every call stages for itself."""
        (rvlen_n, cutoff_radius, weakest_exponent), ctx.optional_passed = _optional_args(
            rvlen_n, cutoff_radius, weakest_exponent)
        a_ik = a_ik.contiguous().detach()
        rpos_ij_e = rpos_ij_e.contiguous()
        tvecs_n = tvecs_n.contiguous()
        batch_i = batch_i.contiguous()
        edge_ij_e = edge_ij_e.contiguous()
        W_k = W_k.detach().contiguous() if W_k is not None else None
        pairs_u = _pairs(batch_i, edge_ij_e, tvecs_n, K)
        rings = None
        fixed_cube = rvlen_n is None or cutoff_radius is None or float(cutoff_radius) == 0.0
        # (adaptive boxes too: atom pairs whose half-widths all come out as LATTICE_RANGE have exactly
        # the cube and start from the rings, the others are staged by the pair kernel)
        worth_it = fixed_cube or (KernelManager.ADAPTIVE_RINGS and a_ik.shape[1] <= 8)
        if (KernelManager.STAGED_RINGS and weakest_exponent is not None and pairs_u is not None
                and worth_it and K > 0 and W_k is not None and _w_leading(W_k) == 1 and W_k.shape[-2] <= 32):
            rings = ops.staged_rings(rpos_ij_e, tvecs_n, pairs_u, K, dist_max, wscale, KernelManager.LATTICE_RANGE,
                                     float(weakest_exponent))
        if rings is not None:
            z_ek, v_ekd = ops.real_enc_fwd_rings(
                a_ik, edge_ij_e, pairs_u, rings, K, dist_max, wscale, W_k, KernelManager.LATTICE_RANGE,
                rpos_ij_e, tvecs_n, batch_i, None if fixed_cube else rvlen_n, None if fixed_cube else cutoff_radius,
                KernelManager.MINIMUM_RANGE)
        else:
            z_ek, v_ekd = ops.real_enc_fwd(
                a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, K, dist_max, wscale, W_k, rvlen_n,
                cutoff_radius, KernelManager.LATTICE_RANGE, KernelManager.MINIMUM_RANGE, pairs_u=pairs_u)
        ctx.save_for_backward(a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, rvlen_n, W_k, z_ek)
        ctx.K, ctx.dist_max, ctx.wscale, ctx.cutoff_radius = K, dist_max, wscale, cutoff_radius
        ctx.ranges = (KernelManager.LATTICE_RANGE, KernelManager.MINIMUM_RANGE)
        # the backward's pair kernel (K <= 64, D <= 16) starts from the same staged translations
        ctx.rings = rings if (rings is not None and fixed_cube and K <= 64 and W_k.shape[-2] <= 16) else None
        if K <= 0:
            return (z_ek,)
        return z_ek, v_ekd

    @staticmethod
    def backward(ctx, gz_ek, gv_ekd=None):
        a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, rvlen_n, W_k, z_ek = ctx.saved_tensors
        e_start_i = ops.cached_edge_row_offsets(edge_ij_e, a_ik.shape[0])
        gz = gz_ek.detach().contiguous() if gz_ek is not None else None
        gv = gv_ekd.detach().contiguous() if gv_ekd is not None else None
        ga_ik, gW_k = ops.real_enc_bwd(
            a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, e_start_i, z_ek, gz, gv, ctx.K, ctx.dist_max,
            ctx.wscale, W_k, rvlen_n, ctx.cutoff_radius, ctx.ranges[0], ctx.ranges[1],
            want_gW=W_k is not None and ctx.needs_input_grad[9],
            pairs_u=_pairs(batch_i, edge_ij_e, tvecs_n, ctx.K), rings=ctx.rings)
        return _enc_backward_tail(ga_ik, gW_k, ctx.optional_passed)


class RealPeriodicEncodingFuncCUDA(torch.autograd.Function):
    """Same encoding with the projection left to a batched matmul: the kernel
    produces the (E,H,K) Gaussian averages and ``W_k`` is applied outside, as in
    the reference's unfused path (``W_k`` leading size 1 or E)."""

    @staticmethod
    def forward(ctx, a_ik, rpos_ij_e, dist2_min_e, tvecs_n, batch_i, edge_ij_e, K, dist_max, wscale,
                W_k, rvlen_n=_ABSENT, cutoff_radius=_ABSENT, weakest_exponent=_ABSENT):
        # (weakest_exponent: accepted for a common call signature; this path stages per call)
        (rvlen_n, cutoff_radius, _), ctx.optional_passed = _optional_args(rvlen_n, cutoff_radius, weakest_exponent)
        a_ik = a_ik.contiguous().detach()
        rpos_ij_e = rpos_ij_e.contiguous()
        tvecs_n = tvecs_n.contiguous()
        batch_i = batch_i.contiguous()
        edge_ij_e = edge_ij_e.contiguous()
        E = edge_ij_e.shape[1]
        z_ek, s_ekk = ops.real_enc_fwd(
            a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, K, dist_max, wscale, None, rvlen_n,
            cutoff_radius, KernelManager.LATTICE_RANGE, KernelManager.MINIMUM_RANGE,
            pairs_u=_pairs(batch_i, edge_ij_e, tvecs_n, K))
        v_out = s_ekk
        if W_k is not None and K > 0:
            W_k = W_k.detach().contiguous()
            assert _w_leading(W_k) in (E, 1)
            v_out = (W_k @ s_ekk[..., None]).reshape(E, a_ik.shape[1], -1)
        else:
            W_k = None
        ctx.save_for_backward(a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, rvlen_n, W_k, z_ek,
                              s_ekk if W_k is not None else None)
        ctx.K, ctx.dist_max, ctx.wscale, ctx.cutoff_radius = K, dist_max, wscale, cutoff_radius
        ctx.ranges = (KernelManager.LATTICE_RANGE, KernelManager.MINIMUM_RANGE)
        if K <= 0:
            return (z_ek,)
        return z_ek, v_out

    @staticmethod
    def backward(ctx, gz_ek, gv_ekd=None):
        a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, rvlen_n, W_k, z_ek, s_ekk = ctx.saved_tensors
        e_start_i = ops.cached_edge_row_offsets(edge_ij_e, a_ik.shape[0])
        gW_k = None
        gv = gv_ekd.detach().contiguous() if gv_ekd is not None else None
        if W_k is not None and gv is not None:
            # dv/dW: outer product per edge; autograd sums it down to W's shape
            gW_k = gv[..., :, None] * s_ekk[..., None, :]
            gv = (W_k.transpose(-1, -2) @ gv[..., None]).squeeze(-1).contiguous()
        gz = gz_ek.detach().contiguous() if gz_ek is not None else None
        ga_ik, _ = ops.real_enc_bwd(
            a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, e_start_i, z_ek, gz, gv, ctx.K, ctx.dist_max,
            ctx.wscale, None, rvlen_n, ctx.cutoff_radius, ctx.ranges[0], ctx.ranges[1], want_gW=False)
        return _enc_backward_tail(ga_ik, gW_k, ctx.optional_passed)


def _dpa_forward(ctx, que_ihk, key_ihk, val_ihk, aij_eh, bij_ehk, batch_i, edge_ij_e):
    que_ihk = que_ihk.contiguous().detach()
    key_ihk = key_ihk.contiguous().detach()
    val_ihk = val_ihk.contiguous().detach()
    aij_eh = aij_eh.contiguous().detach() if aij_eh is not None else None
    bij_ehk = bij_ehk.contiguous().detach() if bij_ehk is not None else None
    batch_i = batch_i.contiguous()
    edge_ij_e = edge_ij_e.contiguous()
    e_start_i = ops.cached_edge_row_offsets(edge_ij_e, que_ihk.shape[0])
    output, prob_eh = ops.fused_dpa_fwd(que_ihk, key_ihk, val_ihk, aij_eh, bij_ehk, edge_ij_e, e_start_i)
    ctx.save_for_backward(que_ihk, key_ihk, val_ihk, bij_ehk, batch_i, edge_ij_e, e_start_i, prob_eh, output)
    ctx.has_aij = aij_eh is not None
    return output, prob_eh


class FusedDotProductAttentionCUDA(torch.autograd.Function):
    """out[i,h,:] = sum_j softmax_j(q_i.k_j + a_ij) (v_j + b_ij) over each atom's
    edge row.  ``que_ihk`` is expected pre-divided by sqrt(head dim)."""

    @staticmethod
    def forward(ctx, que_ihk, key_ihk, val_ihk, aij_eh, bij_ehk, batch_i, edge_ij_e):
        return _dpa_forward(ctx, que_ihk, key_ihk, val_ihk, aij_eh, bij_ehk, batch_i, edge_ij_e)[0]

    @staticmethod
    def backward(ctx, go_ihk):
        que_ihk, key_ihk, val_ihk, bij_ehk, batch_i, edge_ij_e, e_start_i, prob_eh, output = ctx.saved_tensors
        gque, gkey, gval, gaij, gbij = ops.fused_dpa_bwd(
            que_ihk, key_ihk, val_ihk, bij_ehk, batch_i, edge_ij_e, e_start_i, prob_eh, output,
            go_ihk.contiguous().detach())
        return gque, gkey, gval, (gaij if ctx.has_aij else None), gbij, None, None


def fused_encoding_attention(a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, que_ihk, key_ihk, val_ihk,
                             rvlen_n=None, cutoff_radius=None) -> Optional[Tensor]:
    """``FusedDotProductAttentionCUDA(que, key, val, RealPeriodicEncoding...(a, ..., K=0)[0], None, ...)``
    as one launch, for inference (no autograd graph is recorded and nothing is saved for a
    backward pass).  Returns ``None`` when the fused kernel does not serve the call (switched off,
    rows too long for it, row lengths unknown under stream capture): the caller then runs the two
    operators."""
    if not KernelManager.FUSE_ENCODING_ATTENTION or not a_ik.is_cuda:
        return None
    if ops.current_live_sizes() is not None:          # (its row bound would have to be read back)
        return None
    if torch.cuda.is_current_stream_capturing() and not KernelManager.FUSE_ENCODING_ATTENTION_IN_GRAPHS:
        return None
    edge_ij_e = edge_ij_e.contiguous()
    N, H = a_ik.shape
    e_start_i = ops.cached_edge_row_offsets(edge_ij_e, N)
    max_row = ops.cached_max_row(edge_ij_e, e_start_i)
    if max_row is None or max_row * (H + 1) * 4 > 64 * 1024 or H not in (1, 2, 4, 8, 16):
        return None
    return ops.fused_enc_dpa_fwd(a_ik.detach(), rpos_ij_e, tvecs_n, batch_i, edge_ij_e, e_start_i,
                                 que_ihk.detach(), key_ihk.detach(), val_ihk.detach(), max_row, rvlen_n,
                                 cutoff_radius, KernelManager.LATTICE_RANGE, KernelManager.MINIMUM_RANGE)


class FusedDotProductAttentionWithWeights(torch.autograd.Function):
    """:class:`FusedDotProductAttentionCUDA` that also hands out the softmax weights (E,H), which
    the kernel writes anyway; they carry no gradient.  For ``need_weights=True`` of the module
    (the reference's fused operator returns no weights, so its module can only serve that option
    through the per-crystal loop, models/indexed_lattice_multi_head_attention_cuda.py:181-186, 782-786)."""

    @staticmethod
    def forward(ctx, que_ihk, key_ihk, val_ihk, aij_eh, bij_ehk, batch_i, edge_ij_e):
        out, prob = _dpa_forward(ctx, que_ihk, key_ihk, val_ihk, aij_eh, bij_ehk, batch_i, edge_ij_e)
        weights = prob.clone()          # (the saved tensor itself must not be an output)
        if hasattr(ctx, "mark_non_differentiable"):
            ctx.mark_non_differentiable(weights)
        return out, weights

    @staticmethod
    def backward(ctx, go_ihk, _gprob):
        return FusedDotProductAttentionCUDA.backward(ctx, go_ihk)


class ReciPeriodicEncodingFuncCUDA(torch.autograd.Function):
    """z[e,h] = log(max(sum_k exp(a[i,h] k^2) cos(k.r_e), 1e-6)) + 1.5 log(-4 pi a[i,h]) - log V, the
    reciprocal-space lattice sum over the cube of ``KernelManager.LATTICE_RANGE``; gradient for
    ``a_ik`` only, as the reference defines it (models/cuda_funcs/reci_space_enc.py:17-99: the
    backward kernel differentiates the logarithm of the sum, not the normalisation term)."""

    @staticmethod
    def forward(ctx, a_ik, kr_base_e, rvecs_n, vcell_n, batch_i, edge_ij_e):
        a_ik = a_ik.contiguous().detach()
        kr_base_e, rvecs_n, vcell_n = kr_base_e.contiguous(), rvecs_n.contiguous(), vcell_n.contiguous()
        batch_i, edge_ij_e = batch_i.contiguous(), edge_ij_e.contiguous()
        e_start_i = ops.cached_edge_row_offsets(edge_ij_e, a_ik.shape[0])
        z_ek, sumexp_ek = ops.reci_enc_fwd(a_ik, kr_base_e, rvecs_n, vcell_n, batch_i, e_start_i,
                                           KernelManager.LATTICE_RANGE)
        ctx.save_for_backward(a_ik, kr_base_e, rvecs_n, batch_i, e_start_i, sumexp_ek)
        ctx.lattice_range = KernelManager.LATTICE_RANGE
        return z_ek

    @staticmethod
    def backward(ctx, gz_ek):
        a_ik, kr_base_e, rvecs_n, batch_i, e_start_i, sumexp_ek = ctx.saved_tensors
        ga_ik = ops.reci_enc_bwd(a_ik, kr_base_e, rvecs_n, batch_i, e_start_i, gz_ek.detach().contiguous(),
                                 sumexp_ek, ctx.lattice_range, KernelManager.RECI_NORMALISATION_GRAD)
        return ga_ik, None, None, None, None, None


class GaussianExponentsHIP(torch.autograd.Function):
    """(a, q_scaled) from the per-head query: a = coef * rho(normalised <q, w>),
    q_scaled = q * q_scale.  The normalisation statistics are constants of the
    backward pass, as in the reference, which detaches them
    (models/indexed_lattice_multi_head_attention_cuda.py:700-712)."""

    @staticmethod
    def forward(ctx, q_ihd, w_hd, gauss_scale, normalize, update_stats, positive_func, beta, lower_bound,
                coef, q_scale):
        q_ihd = q_ihd.contiguous().detach()
        w_hd = w_hd.contiguous().detach()
        need_grad = any(ctx.needs_input_grad[:2])
        a, qs, alpha_n, used = ops.gauss_exponents(q_ihd, w_hd, gauss_scale, normalize, update_stats,
                                                   positive_func, beta, lower_bound, coef, q_scale,
                                                   want_alpha=need_grad)
        if need_grad:
            ctx.save_for_backward(q_ihd, w_hd, alpha_n, used)
        ctx.conf = (positive_func, beta, lower_bound, coef, q_scale)
        ctx.w_shape = w_hd.shape
        return a, qs

    @staticmethod
    def backward(ctx, ga, gqs):
        q_ihd, w_hd, alpha_n, used = ctx.saved_tensors
        func, beta, lb, coef, q_scale = ctx.conf
        gq, gw = ops.gauss_exponents_bwd(ga, gqs, q_ihd, w_hd, alpha_n, used, func, beta, lb, coef,
                                         q_scale if q_scale is not None else 1.0,
                                         want_gq=ctx.needs_input_grad[0], want_gw=ctx.needs_input_grad[1])
        if gw is not None:
            gw = gw.reshape(ctx.w_shape)
        return gq, gw, None, None, None, None, None, None, None, None


class LinearRowsHIP(torch.autograd.Function):
    """y = x W^T + b for 2-D x on the training path: library GEMMs for the forward and the
    input gradient; weight and bias gradient from one fixed-order pass over the output
    gradient (autograd's own bias reduction records a memset node per call under stream
    capture and takes three times as long)."""

    @staticmethod
    def forward(ctx, x, weight, bias):
        ctx.save_for_backward(x, weight)
        ctx.has_bias = bias is not None
        # the parameters themselves (leaves only: no cycle through the graph), for deferred gradients
        ctx.leaves = (weight if weight.is_leaf else None, bias if (bias is not None and bias.is_leaf) else None)
        return torch.nn.functional.linear(x, weight, bias)

    @staticmethod
    def backward(ctx, g):
        x, weight = ctx.saved_tensors
        g = g.contiguous()
        gx = g @ weight if ctx.needs_input_grad[0] else None
        want_b = ctx.has_bias and ctx.needs_input_grad[2]
        gw = gb = None
        weight_p, bias_p = ctx.leaves
        if _deferred is not None and ctx.needs_input_grad[1] and weight_p is not None and weight_p.grad is None \
                and (not want_b or (bias_p is not None and bias_p.grad is None)):
            # all layers' weight gradients are computed together after the backward pass
            _deferred.append((g, x.contiguous(), weight_p, bias_p if want_b else None, 0))
        elif ctx.needs_input_grad[1]:
            gw = ops.linear_weight_grad(g, x.contiguous(), with_bias=want_b)
            if want_b:
                gw, gb = gw
        elif want_b:
            gb = ops.column_sum(g)
        return gx, gw, gb


def input_gradient(gs, weights, add: Optional[Tensor], mask: Optional[Tensor], like: Tensor) -> Tensor:
    """``mask(sum_i gs[i] @ weights[i]) + add``: one row-block launch for all terms, the mask and
    the addend where the shapes allow it (at 1774 rows as fast as the library GEMM for a single
    plain product -- 3.3 against 4.0 us for 128 -> 128, 6.8 against 6.5 us for 512 -> 128 -- and
    ahead of it with an addend or several terms), else library GEMMs and element-wise launches."""
    if not gs:
        return add if add is not None else torch.zeros_like(like)
    if ops.linear_rows_nn_supported(gs[0], weights[0]):
        return ops.linear_rows_nn(gs, weights, add=add.contiguous() if add is not None else None, mask=mask)
    gx = torch.mm(gs[0], weights[0])
    for g, w in zip(gs[1:], weights[1:]):
        gx.addmm_(g, w)
    if mask is not None:
        gx = torch.ops.aten.threshold_backward(gx, mask, 0)
    return gx + add if add is not None else gx


class FusedFeedForwardHIP(torch.autograd.Function):
    """``y = x + W2 relu(W1 x + b1) + b2`` (the feed-forward half of a block without norm layers
    and dropout): two row-block launches forward, two backward -- the ReLU mask rides in the
    epilogue of the first input-gradient kernel, the residual gradient in that of the second --
    and both layers' weight and bias gradients from the grouped fixed-order kernel (deferred
    inside :class:`deferred_weight_grads`)."""

    @staticmethod
    def forward(ctx, x, w1, b1, w2, b2):
        x = x.contiguous()
        h, = ops.linear_rows(x, (w1,), b1, relu=True)
        y, = ops.linear_rows(h, (w2,), b2, residual=x)
        ctx.save_for_backward(x, h, w1, w2)
        ctx.leaves = tuple(t if (t is not None and t.is_leaf) else None for t in (w1, b1, w2, b2))
        ctx.has_bias = (b1 is not None, b2 is not None)
        return y

    @staticmethod
    def backward(ctx, g):
        x, h, w1, w2 = ctx.saved_tensors
        g = g.contiguous()
        gh = input_gradient([g], [w2], None, h, h)                 # (g W2) where the ReLU was open
        gx = input_gradient([gh], [w1], g, None, x) if ctx.needs_input_grad[0] else None
        w1_p, b1_p, w2_p, b2_p = ctx.leaves
        need = ctx.needs_input_grad
        layers = [(gh, x, w1, w1_p, b1_p, need[1], ctx.has_bias[0] and need[2]),
                  (g, h, w2, w2_p, b2_p, need[3], ctx.has_bias[1] and need[4])]
        out = [None, None, None, None]                             # gw1, gb1, gw2, gb2
        immediate = []
        for k, (gg, xx, w, w_p, b_p, want_w, want_b) in enumerate(layers):
            if not want_w and not want_b:
                continue
            if _deferred is not None and want_w and w_p is not None and w_p.grad is None and \
                    (not ctx.has_bias[k] or (want_b and b_p is not None and b_p.grad is None)):
                _deferred.append((gg, xx, w_p, b_p if want_b else None, 0))
            else:
                gw = torch.empty_like(w, memory_format=torch.contiguous_format)
                gb = torch.empty(w.shape[0], dtype=w.dtype, device=w.device) if want_b else None
                immediate.append((gg, xx, gw, gb))
                out[2 * k], out[2 * k + 1] = (gw if want_w else None), gb
        if immediate:
            ops.linear_weight_grad_grouped(immediate)
        return (gx, *out)


class FusedLinearHIP(torch.autograd.Function):
    """``(y_0, ..)`` with ``y_i = act(x W_i^T + b_i) (+ residual)`` for up to three equally
    shaped weights sharing the input (query / key / value projections) in one row-block
    launch, bias, ReLU and residual in its epilogue.  ``bias`` is one vector over all
    outputs (n_weights * C).  With ``carry`` the input itself is returned as one more output
    (an identity whose gradient this node adds to the input gradient in the epilogue of its
    own kernel, where autograd would launch an addition for a residual branch that leaves the
    input here).  Backward: the input gradient from the row-block kernel for all terms at
    once, weight and bias gradients from the grouped fixed-order kernel (deferred to the end
    of the backward pass inside :class:`deferred_weight_grads`)."""

    @staticmethod
    def forward(ctx, x, bias, residual, relu, carry, *weights):
        if relu and (residual is not None or len(weights) != 1):
            raise ValueError("FusedLinearHIP: ReLU goes with a single weight and no residual")
        if carry and not x.is_contiguous():
            raise ValueError("FusedLinearHIP: a carried input must be contiguous")
        xc = x.contiguous()
        ys = ops.linear_rows(xc, weights, bias, residual=residual, relu=relu)
        ctx.save_for_backward(xc, *weights, *((ys[0],) if relu else ()))
        ctx.relu, ctx.nw, ctx.carry = relu, len(weights), carry
        # the parameters themselves (leaves only: no cycle through the graph), for deferred gradients
        ctx.leaves = ([w if w.is_leaf else None for w in weights],
                      bias if (bias is not None and bias.is_leaf) else None, bias is not None)
        return (*ys, x) if carry else tuple(ys)

    @staticmethod
    def backward(ctx, *gs):
        saved = ctx.saved_tensors
        x, weights = saved[0], saved[1:1 + ctx.nw]
        C = weights[0].shape[0]
        g_carry = gs[ctx.nw] if ctx.carry else None
        gs = [g.contiguous() if g is not None else None for g in gs[:ctx.nw]]
        if ctx.relu and gs[0] is not None:
            gs[0] = torch.ops.aten.threshold_backward(gs[0], saved[-1], 0)
        g_res = gs[0] if ctx.needs_input_grad[2] else None
        gx = None
        if ctx.needs_input_grad[0]:
            gx = input_gradient([g for g in gs if g is not None],
                                [w for g, w in zip(gs, weights) if g is not None], g_carry, None, x)
        need_w = [ctx.needs_input_grad[5 + i] for i in range(ctx.nw)]
        leaves_w, bias_p, has_bias = ctx.leaves
        want_b = has_bias and ctx.needs_input_grad[1]
        gws = [None] * ctx.nw
        gb = None
        if any(need_w) or want_b:
            gs = [g if g is not None else torch.zeros((x.shape[0], C), dtype=x.dtype, device=x.device) for g in gs]
            if _deferred is not None and all(need_w) and all(w is not None and w.grad is None for w in leaves_w) \
                    and (not has_bias or (want_b and bias_p is not None and bias_p.grad is None)):
                for i in range(ctx.nw):
                    _deferred.append((gs[i], x, leaves_w[i], bias_p, i * C))
            else:
                gb = torch.empty(ctx.nw * C, dtype=x.dtype, device=x.device) if want_b else None
                gws = [torch.empty_like(w, memory_format=torch.contiguous_format) for w in weights]
                ops.linear_weight_grad_grouped([(gs[i], x, gws[i], gb[i * C:(i + 1) * C] if want_b else None)
                                                for i in range(ctx.nw)])
                gws = [gw if need else None for gw, need in zip(gws, need_w)]
        return (gx, gb, g_res, None, None, *gws)


# A list while a training step defers its linear layers' weight gradients (see
# :func:`deferred_weight_grads`), else None.
_deferred = None


class deferred_weight_grads:
    """Context for ``loss.backward()``: linear layers routed through :class:`LinearRowsHIP`
    leave their parameters' gradients unset during the backward pass and the context's exit
    computes them all in one grouped launch pair, writing ``.grad`` directly.  Only
    parameters without an existing gradient take part (no accumulation)."""

    def __enter__(self):
        global _deferred
        self.previous = _deferred
        _deferred = []
        return self

    def __exit__(self, exc_type, exc, tb):
        global _deferred
        pending, _deferred = _deferred, self.previous
        if exc_type is not None or not pending:
            return False
        layers, seen, bias_grads = [], set(), {}
        for g, x, weight_p, bias_p, bias_off in pending:
            if id(weight_p) in seen or weight_p.grad is not None or (bias_p is not None and bias_p.grad is not None):
                raise RuntimeError("deferred weight gradients: a parameter is used by more than one layer")
            seen.add(id(weight_p))
            gw = torch.empty_like(weight_p, memory_format=torch.contiguous_format)
            gb = None
            if bias_p is not None:                  # several layers may own slices of one bias vector
                entry = bias_grads.setdefault(id(bias_p), [bias_p, torch.empty(bias_p.numel(), dtype=bias_p.dtype,
                                                                               device=bias_p.device), 0])
                gb = entry[1][bias_off:bias_off + g.shape[1]]
                entry[2] += g.shape[1]
            layers.append((g, x, gw, gb))
        for bias_p, full, covered in bias_grads.values():
            if covered != bias_p.numel():
                raise RuntimeError("deferred weight gradients: a bias vector is only partly used")
        ops.linear_weight_grad_grouped(layers)
        for (g, x, gw, gb), (_, _, weight_p, _, _) in zip(layers, pending):
            weight_p.grad = gw
        for bias_p, full, covered in bias_grads.values():
            bias_p.grad = full.view(bias_p.shape)
        return False


# Set by the graphed training step (around capture and around its eager twin); plain eager
# training keeps the stock op, whose autograd runs without Python in the loop.
USE_LINEAR_FUNCTION = False


def linear(x: Tensor, weight: Tensor, bias: Optional[Tensor]) -> Tensor:
    """F.linear; inside a graphed training step through :class:`LinearRowsHIP` (fewer and
    memset-free nodes)."""
    if USE_LINEAR_FUNCTION and x.is_cuda and x.dim() == 2 and x.dtype == torch.float32 and \
            torch.is_grad_enabled() and (x.requires_grad or weight.requires_grad):
        return LinearRowsHIP.apply(x, weight, bias)
    return torch.nn.functional.linear(x, weight, bias)


class L1MeanLossHIP(torch.autograd.Function):
    """Scalar training loss ``mean_b sum_i |pred[b,i] - target[b,i]|`` (the reference's
    ``regression_loss(..., "l1").mean()``, losses/regression_loss.py:10-20 and
    models/regression.py:117-118) with its gradient computed by the same launch, where the
    stock ops take about ten launches forward and backward."""

    @staticmethod
    def forward(ctx, pred: Tensor, target: Tensor):
        loss, grad = ops.l1_mean_loss(pred.detach(), target.detach(), with_grad=ctx.needs_input_grad[0])
        ctx.save_for_backward(grad)
        return loss.reshape(())

    @staticmethod
    def backward(ctx, gloss):
        grad, = ctx.saved_tensors
        return (grad * gloss if grad is not None else None), None


class IrregularMeanCUDA(torch.autograd.Function):
    """Per-crystal mean over atoms with a fixed summation order."""

    @staticmethod
    def forward(ctx, x_ik: Tensor, batch_i: Tensor, sizes: Optional[Tensor]):
        if sizes is None:
            B = int(batch_i.max().item()) + 1
            sizes = torch.zeros(B, dtype=torch.long, device=x_ik.device)
            sizes.scatter_add_(0, batch_i, torch.ones_like(batch_i))
        sig, start_n = ops._cache_lookup("mean_start", sizes)
        if start_n is None:
            start_n = ops._cache_store(
                sig, (sizes,), torch.constant_pad_nd(torch.cumsum(sizes, 0), (1, 0)).contiguous())
        o_nk = ops.irregular_mean_fwd(x_ik.contiguous().detach(), start_n)
        ctx.save_for_backward(batch_i.contiguous(), start_n)
        return o_nk

    @staticmethod
    def backward(ctx, go_nk):
        batch_i, start_n = ctx.saved_tensors
        return ops.irregular_mean_bwd(go_nk.contiguous(), batch_i, start_n), None, None


def compute_minimum_distance(rpos_ij_e, tvecs_n, batch_i, edge_ij_e, rvlen_n, cutoff_radius):
    """Per-edge minimum squared distance (models/cuda_funcs/minimum_distance.py:18-41)."""
    assert cutoff_radius >= 0
    return ops.minimum_distance(rpos_ij_e, tvecs_n, batch_i, edge_ij_e, rvlen_n, cutoff_radius,
                                KernelManager.LATTICE_RANGE, KernelManager.MINIMUM_RANGE)
