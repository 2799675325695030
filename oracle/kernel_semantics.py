"""ctypes front-end to ``oracle/kernels_ref.c`` (kernel-level CPU oracle).

TEST INFRASTRUCTURE ONLY — used by tests/, the smoke check and the benchmark's
cpu_baseline leg; never imported by the product package.

Every function takes and returns CPU torch tensors (float32 / int64) and mirrors
one device kernel of the reference, including the adaptive translation boxes
(see the header of kernels_ref.c for the file:line map).
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Optional, Tuple

import torch
from torch import Tensor

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libcf_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile kernels_ref.c with gcc (seconds)."""
    if force or not os.path.exists(_LIB_PATH) or \
            os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "kernels_ref.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libcf_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def _p(t: Optional[Tensor]):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _f(t: Optional[Tensor]) -> Optional[Tensor]:
    return None if t is None else t.detach().to(torch.float32).contiguous()


def _l(t: Tensor) -> Tensor:
    return t.detach().to(torch.int64).contiguous()


_i64 = ctypes.c_longlong
_dbl = ctypes.c_double
_int = ctypes.c_int


def translation_ranges(a_ik: Tensor, rvlen_n: Optional[Tensor], batch_i: Tensor,
                       cutoff_radius: float, lattice_range: int, minimum_range: int) -> Tensor:
    a_ik, rvlen_n, batch_i = _f(a_ik), _f(rvlen_n), _l(batch_i)
    N, H = a_ik.shape
    out = torch.empty((N, H, 3), dtype=torch.int32)
    lib().ref_translation_ranges(_p(a_ik), _p(rvlen_n), _p(batch_i), _i64(N), _i64(H),
                                 _dbl(cutoff_radius), _int(lattice_range), _int(minimum_range),
                                 _p(out))
    return out


def real_enc_fwd(a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, K, dist_max, wscale,
                 W_k=None, rvlen_n=None, cutoff_radius=0.0, lattice_range=2,
                 minimum_range=0) -> Tuple[Tensor, Optional[Tensor]]:
    a_ik, rpos_ij_e, tvecs_n = _f(a_ik), _f(rpos_ij_e), _f(tvecs_n)
    batch_i, edge_ij_e, W_k, rvlen_n = _l(batch_i), _l(edge_ij_e), _f(W_k), _f(rvlen_n)
    N, H = a_ik.shape
    E = edge_ij_e.shape[1]
    D, W_num = 0, 0
    if W_k is not None:
        W_num = 1 if W_k.dim() == 3 else W_k.shape[0]
        D = W_k.shape[-2]
    z = torch.empty((E, H), dtype=torch.float32)
    v = torch.empty((E, H, D if W_k is not None else K), dtype=torch.float32) if K > 0 else None
    lib().ref_real_enc_fwd(_p(a_ik), _p(rpos_ij_e), _p(tvecs_n), _p(batch_i), _p(edge_ij_e),
                           _i64(N), _i64(H), _i64(E), _i64(K), _i64(D), _dbl(dist_max),
                           _dbl(wscale), _p(W_k), _i64(W_num), _p(rvlen_n),
                           _dbl(cutoff_radius if cutoff_radius is not None else 0.0),
                           _int(lattice_range), _int(minimum_range), _p(z), _p(v))
    return z, v


def real_enc_fwd_cond(a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, K, dist_max, wscale, rvlen_n=None,
                      cutoff_radius=0.0, lattice_range=2, minimum_range=0) -> Tensor:
    """(E,H,K) first-order float32 conditioning of the Gaussian averages (see kernels_ref.c):
    a tolerance, not a restatement of reference code."""
    a_ik, rpos_ij_e, tvecs_n, rvlen_n = _f(a_ik), _f(rpos_ij_e), _f(tvecs_n), _f(rvlen_n)
    batch_i, edge_ij_e = _l(batch_i), _l(edge_ij_e)
    N, H = a_ik.shape
    E = edge_ij_e.shape[1]
    cond = torch.empty((E, H, K), dtype=torch.float32)
    lib().ref_real_enc_fwd_cond(_p(a_ik), _p(rpos_ij_e), _p(tvecs_n), _p(batch_i), _p(edge_ij_e), _i64(N),
                                _i64(H), _i64(E), _i64(K), _dbl(dist_max), _dbl(wscale), _p(rvlen_n),
                                _dbl(cutoff_radius if cutoff_radius is not None else 0.0),
                                _int(lattice_range), _int(minimum_range), _p(cond))
    return cond


def real_enc_bwd(a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, e_start_i, z_ek, gz_ek, gv_ekd,
                 K, dist_max, wscale, W_k=None, rvlen_n=None, cutoff_radius=0.0,
                 lattice_range=2, minimum_range=0, magnitude=False) -> Tuple[Tensor, Optional[Tensor]]:
    """``magnitude``: the same sums over the magnitudes of their terms (a tolerance for the
    tests, see kernels_ref.c), not the gradients."""
    a_ik, rpos_ij_e, tvecs_n = _f(a_ik), _f(rpos_ij_e), _f(tvecs_n)
    batch_i, edge_ij_e, e_start_i = _l(batch_i), _l(edge_ij_e), _l(e_start_i)
    W_k, rvlen_n, z_ek, gz_ek, gv_ekd = _f(W_k), _f(rvlen_n), _f(z_ek), _f(gz_ek), _f(gv_ekd)
    N, H = a_ik.shape
    E = edge_ij_e.shape[1]
    D, W_num = 0, 0
    gW = None
    if W_k is not None:
        W_num = 1 if W_k.dim() == 3 else W_k.shape[0]
        D = W_k.shape[-2]
        gW = torch.zeros_like(W_k)
    ga = torch.empty_like(a_ik)
    fn = lib().ref_real_enc_bwd_magnitude if magnitude else lib().ref_real_enc_bwd
    fn(_p(a_ik), _p(rpos_ij_e), _p(tvecs_n), _p(batch_i), _p(edge_ij_e), _p(e_start_i), _p(z_ek), _p(gz_ek),
       _p(gv_ekd), _i64(N), _i64(H), _i64(E), _i64(K), _i64(D), _dbl(dist_max), _dbl(wscale), _p(W_k),
       _i64(W_num), _p(rvlen_n), _dbl(cutoff_radius if cutoff_radius is not None else 0.0),
       _int(lattice_range), _int(minimum_range), _p(ga), _p(gW))
    return ga, gW


def fused_dpa_fwd(que, key, val, aij_eh, bij_ehd, edge_ij_e, e_start_i) -> Tuple[Tensor, Tensor]:
    que, key, val, aij_eh, bij_ehd = _f(que), _f(key), _f(val), _f(aij_eh), _f(bij_ehd)
    edge_ij_e, e_start_i = _l(edge_ij_e), _l(e_start_i)
    N, H, Dk = que.shape
    Dv = val.shape[-1]
    E = edge_ij_e.shape[1]
    prob = torch.empty((E, H), dtype=torch.float32)
    out = torch.empty((N, H, Dv), dtype=torch.float32)
    lib().ref_fused_dpa_fwd(_p(que), _p(key), _p(val), _p(aij_eh), _p(bij_ehd), _p(edge_ij_e),
                            _p(e_start_i), _i64(N), _i64(H), _i64(E), _i64(Dk), _i64(Dv),
                            _p(prob), _p(out))
    return out, prob


def fused_dpa_bwd(que, key, val, bij_ehd, edge_ij_e, e_start_i, prob_eh, out, gout):
    que, key, val, bij_ehd = _f(que), _f(key), _f(val), _f(bij_ehd)
    prob_eh, out, gout = _f(prob_eh), _f(out), _f(gout)
    edge_ij_e, e_start_i = _l(edge_ij_e), _l(e_start_i)
    N, H, Dk = que.shape
    Dv = val.shape[-1]
    E = edge_ij_e.shape[1]
    gq, gk, gv = torch.empty_like(que), torch.empty_like(key), torch.empty_like(val)
    ga = torch.empty((E, H), dtype=torch.float32)
    gb = torch.empty((E, H, Dv), dtype=torch.float32) if bij_ehd is not None else None
    lib().ref_fused_dpa_bwd(_p(que), _p(key), _p(val), _p(bij_ehd), _p(edge_ij_e), _p(e_start_i),
                            _i64(N), _i64(H), _i64(E), _i64(Dk), _i64(Dv), _p(prob_eh), _p(out),
                            _p(gout), _p(gq), _p(gk), _p(gv), _p(ga), _p(gb))
    return gq, gk, gv, ga, gb


def irregular_mean(src: Tensor, start_n: Tensor) -> Tensor:
    src, start_n = _f(src), _l(start_n)
    B = start_n.numel() - 1
    D = src.numel() // max(src.shape[0], 1)
    dst = torch.empty((B,) + tuple(src.shape[1:]), dtype=torch.float32)
    lib().ref_irregular_mean(_p(src), _p(start_n), _i64(B), _i64(D), _p(dst))
    return dst


def minimum_distance(rpos_ij_e, tvecs_n, batch_i, edge_ij_e, rvlen_n, cutoff_radius,
                     lattice_range=2, minimum_range=0) -> Tensor:
    rpos_ij_e, tvecs_n, rvlen_n = _f(rpos_ij_e), _f(tvecs_n), _f(rvlen_n)
    batch_i, edge_ij_e = _l(batch_i), _l(edge_ij_e)
    E = edge_ij_e.shape[1]
    out = torch.empty((E,), dtype=torch.float32)
    lib().ref_minimum_distance(_p(rpos_ij_e), _p(tvecs_n), _p(batch_i), _p(edge_ij_e), _i64(E),
                               _p(rvlen_n), _dbl(cutoff_radius), _int(lattice_range),
                               _int(minimum_range), _p(out))
    return out


def reci_enc_fwd(a_ik, kr_base_e, rvecs_n, vcell_n, batch_i, edge_ij_e, lattice_range=2) -> Tuple[Tensor, Tensor]:
    """(z_ek, sumexp_ek) of the reciprocal-space lattice sum (models/kernels/reci_enc_fwd.cu)."""
    a_ik, kr_base_e, rvecs_n, vcell_n = _f(a_ik), _f(kr_base_e), _f(rvecs_n), _f(vcell_n)
    batch_i, edge_ij_e = _l(batch_i), _l(edge_ij_e)
    N, H = a_ik.shape
    E = edge_ij_e.shape[1]
    z = torch.empty((E, H), dtype=torch.float32)
    se = torch.empty((E, H), dtype=torch.float32)
    lib().ref_reci_enc_fwd(_p(a_ik), _p(kr_base_e), _p(rvecs_n), _p(vcell_n), _p(batch_i), _p(edge_ij_e),
                           _i64(N), _i64(H), _i64(E), _int(lattice_range), _p(z), _p(se))
    return z, se


def reci_enc_bwd(a_ik, kr_base_e, rvecs_n, batch_i, e_start_i, gz_ek, sumexp_ek, lattice_range=2,
                 normalisation_grad=False) -> Tensor:
    """ga_ik (models/kernels/reci_enc_bwd.cu: without the normalisation term's derivative unless
    ``normalisation_grad``)."""
    a_ik, kr_base_e, rvecs_n, gz_ek, sumexp_ek = _f(a_ik), _f(kr_base_e), _f(rvecs_n), _f(gz_ek), _f(sumexp_ek)
    batch_i, e_start_i = _l(batch_i), _l(e_start_i)
    N, H = a_ik.shape
    ga = torch.empty((N, H), dtype=torch.float32)
    lib().ref_reci_enc_bwd(_p(a_ik), _p(kr_base_e), _p(rvecs_n), _p(batch_i), _p(e_start_i), _p(gz_ek),
                           _p(sumexp_ek), _i64(N), _i64(H), _int(lattice_range), _int(int(normalisation_grad)),
                           _p(ga))
    return ga
