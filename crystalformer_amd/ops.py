"""Thin functional wrappers over the C ABI: validate, allocate outputs with
torch, pass raw device pointers and torch's current stream.  No autograd here
(see ``hip_funcs.py``) and no CPU fallback.
"""
from __future__ import annotations

import threading
from typing import Optional, Tuple

import torch
import torch.nn.functional as F
from torch import Tensor

from . import lib as _lib
from .lib import check, device_guard, ptr, require_device, stream_handle


# Optional kernel timing: when a list is installed, every encoding / attention
# launch is bracketed by a pair of HIP events recorded on the launch stream and
# (name, start, stop, info) is appended to it.
_event_log: Optional[list] = None


def set_event_log(log: Optional[list]) -> None:
    global _event_log
    _event_log = log


# Optional work counter: when a list is installed, every encoding launch appends
# the number of (edge, translation) pairs its kernel walks (the box of an edge is
# the union over heads of the per-head boxes).  Costs a host sync; not for timed runs.
_eval_counter: Optional[list] = None


def set_eval_counter(counter: Optional[list]) -> None:
    global _eval_counter
    _eval_counter = counter


def count_translation_evals(a_ik: Tensor, rvlen_n: Optional[Tensor], batch_i: Tensor, edge_ij_e: Tensor,
                            cutoff: float, lattice_range: int, minimum_range: int) -> float:
    E = edge_ij_e.shape[1]
    if cutoff == 0.0 or rvlen_n is None:
        return float(E) * (2 * lattice_range + 1) ** 3
    R = translation_ranges(a_ik, rvlen_n, batch_i, cutoff, lattice_range, minimum_range)
    T = (2 * R.max(dim=1).values.long() + 1).prod(dim=1).double()          # per source atom
    return float(T[edge_ij_e[0]].sum().item())


class launch_share:
    """Context manager: within it, forward launches of the periodic encoding made by this
    thread occupy at most ``share`` of the GPU (``cf_set_launch_share``), so that kernels of
    other streams run beside them.  For callers that keep several forwards in flight; a
    graph captured inside keeps the share.  Results do not depend on it."""

    def __init__(self, share: float):
        self.share = float(share)
        self.previous = 1.0

    def __enter__(self):
        lib = _lib.load()
        self.previous = float(lib.cf_get_launch_share())
        check(lib.cf_set_launch_share(self.share), "cf_set_launch_share")
        return self

    def __exit__(self, *exc):
        check(_lib.load().cf_set_launch_share(self.previous), "cf_set_launch_share")
        return False


class live_sizes:
    """Context manager: within it the operators of this thread take the atom, edge and pair counts
    of a batch from ``header`` (4 int64 words on the device: atoms, edges, atom pairs, status) instead
    of from their arguments, whose sizes are then capacities (``cf_set_size_header``).  For one set
    of buffers -- one captured graph -- served to batches whose crystal sizes differ:
    :func:`batch_layout` called inside fills the header from ``sizes`` as it finds it when its
    kernels run, without reading anything back to the host, and every tensor downstream has the
    capacity's shape with the live items in front.  A captured graph keeps the header's address."""

    def __init__(self, header: Tensor, atom_capacity: int, edge_capacity: int):
        if header.dtype != torch.int64 or header.numel() != 4 or not header.is_cuda or not header.is_contiguous():
            raise _lib.CrystalformerHipError("live_sizes: the header is 4 contiguous int64 words on the GPU")
        self.header, self.atoms, self.edges = header, int(atom_capacity), int(edge_capacity)
        self.units = (self.atoms + self.edges) // 2
        self.previous = None

    def __enter__(self):
        self.previous = getattr(_live, "current", None)
        check(_lib.load().cf_set_size_header(ptr(self.header), self.atoms, self.edges), "cf_set_size_header")
        _live.current = self
        return self

    def __exit__(self, *exc):
        prev = self.previous
        _live.current = prev
        if prev is None:
            check(_lib.load().cf_set_size_header(None, 0, 0), "cf_set_size_header")
        else:
            check(_lib.load().cf_set_size_header(ptr(prev.header), prev.atoms, prev.edges), "cf_set_size_header")
        return False


_live = threading.local()


def current_live_sizes() -> Optional[live_sizes]:
    return getattr(_live, "current", None)


def _refuse_live_sizes(what: str) -> None:
    """Operators whose kernels take their counts from the arguments walk whole tensors: under a size
    header the tails of those tensors are unwritten memory, so they refuse to run there."""
    if current_live_sizes() is not None:
        raise _lib.CrystalformerHipError(f"{what} does not run under a size header (it walks whole tensors); "
                                         f"leave the live_sizes context first")


class _timed:
    def __init__(self, name: str, **info):
        self.name, self.info = name, info

    def __enter__(self):
        if _event_log is not None:
            self.start = torch.cuda.Event(enable_timing=True)
            self.stop = torch.cuda.Event(enable_timing=True)
            self.start.record()
        return self

    def __exit__(self, *exc):
        if _event_log is not None:
            self.stop.record()
            _event_log.append((self.name, self.start, self.stop, self.info))
        return False


# Small caches of per-batch index structures derived from (batch_i, edge_ij_e):
# the attention blocks of one forward all see the same tensors, so the pair list
# and the CSR offsets are built once.  Entries keep their key tensors alive, so a
# recycled address can never alias a stale entry.
_index_cache: list = []
_INDEX_CACHE_SIZE = 64


def _cache_lookup(kind: str, *keys: Tensor):
    sig = (kind,) + tuple((k.data_ptr(), tuple(k.shape), k._version) for k in keys)
    for entry in _index_cache:
        if entry[0] == sig:
            return sig, entry[2]
    return sig, None


def index_cache_snapshot() -> list:
    """The current cache entries (key tensors and derived tensors).  A captured graph bakes in
    the addresses of the derived tensors it found here; whoever owns the graph keeps this list,
    so that eviction from the cache can never free them."""
    return list(_index_cache)


def _cache_store(sig, keys, value):
    _index_cache.insert(0, (sig, keys, value))
    del _index_cache[_INDEX_CACHE_SIZE:]
    return value


def _f32(t: Optional[Tensor], name: str) -> Optional[Tensor]:
    if t is None:
        return None
    if t.dtype != torch.float32:
        raise _lib.CrystalformerHipError(f"{name} must be float32, got {t.dtype}")
    return t.contiguous()


def _i64(t: Optional[Tensor], name: str) -> Optional[Tensor]:
    if t is None:
        return None
    if t.dtype != torch.int64:
        raise _lib.CrystalformerHipError(f"{name} must be int64, got {t.dtype}")
    return t.contiguous()


def _w_shape(W_k: Optional[Tensor], H: int, K: int) -> Tuple[int, int]:
    if W_k is None:
        return 0, 0
    if W_k.dim() not in (3, 4):
        raise _lib.CrystalformerHipError("W_k must be (H,D,K) or (W_num,H,D,K)")
    if W_k.shape[-3] != H or W_k.shape[-1] != K:
        raise _lib.CrystalformerHipError(
            f"W_k shape {tuple(W_k.shape)} does not match H={H}, K={K}")
    return (1 if W_k.dim() == 3 else W_k.shape[0]), W_k.shape[-2]


def edge_row_offsets(edge_ij_e: Tensor, num_atoms: int) -> Tensor:
    """CSR offsets of each source atom's edges, (N+1) int64, computed on the
    device without a host sync (models/cuda_funcs/fused_dpa.py:24-26)."""
    start = torch.zeros(num_atoms + 1, dtype=torch.int64, device=edge_ij_e.device)
    start.scatter_add_(0, edge_ij_e[0] + 1, torch.ones_like(edge_ij_e[0]))
    return start.cumsum(0)


def crystal_offsets(batch_i: Tensor, num_slots: Optional[int] = None) -> Tuple[Tensor, Tensor]:
    """(atom_start, edge_start): leading-zero cumulative sums of the crystal
    sizes and of their squares.  ``num_slots`` defaults to the atom count, an
    upper bound on the number of crystals that needs no host sync."""
    slots = batch_i.numel() if num_slots is None else num_slots
    sizes = torch.zeros(slots, dtype=torch.int64, device=batch_i.device)
    sizes.scatter_add_(0, batch_i, torch.ones_like(batch_i))
    atom_start = F.pad(sizes.cumsum(0), (1, 0))
    edge_start = F.pad((sizes * sizes).cumsum(0), (1, 0))
    return atom_start, edge_start


# Scheduling words of the pair-evaluated forward (two zeroed int32 the work-groups draw their
# rounds from; the kernel leaves them zeroed).  Launches that may overlap need words of their
# own: eager launches on one stream run in order and share one pair per (device, stream).
# Graphs captured on one stream can later be replayed side by side, so under stream capture
# every launch gets a pair no other launch ever uses, cut from a zeroed per-device buffer
# that lives as long as the process (no fill node in the graph); once that is used up, or if
# nothing ran eagerly on the device before the capture, a fresh zero-filled pair.
DYNAMIC_ROUNDS = True
_sched_words: dict = {}
_capture_words: dict = {}            # device index -> [buffer, pairs handed out]
_CAPTURE_PAIRS = 8192


def _scheduling_words(dev: torch.device) -> Tensor:
    if torch.cuda.is_current_stream_capturing():
        pool = _capture_words.get(dev.index)
        if pool is None or pool[1] >= _CAPTURE_PAIRS:
            return torch.zeros(2, dtype=torch.int32, device=dev)
        k = pool[1]
        pool[1] = k + 1
        return pool[0][2 * k:2 * k + 2]
    if dev.index not in _capture_words:
        _capture_words[dev.index] = [torch.zeros(2 * _CAPTURE_PAIRS, dtype=torch.int32, device=dev), 0]
    key = (dev.index, stream_handle(dev))
    words = _sched_words.get(key)
    if words is None:
        words = _sched_words[key] = torch.zeros(2, dtype=torch.int32, device=dev)
    return words


def real_enc_fwd(a_ik: Tensor, rpos_ij_e: Tensor, tvecs_n: Tensor, batch_i: Tensor, edge_ij_e: Tensor,
                 K: int, dist_max: float, wscale: float, W_k: Optional[Tensor] = None,
                 rvlen_n: Optional[Tensor] = None, cutoff_radius: Optional[float] = None,
                 lattice_range: int = 2, minimum_range: int = 0,
                 pairs_u: Optional[Tensor] = None) -> Tuple[Tensor, Optional[Tensor]]:
    """``pairs_u`` (U,5) from :func:`edge_pairs` selects the matrix-core kernel
    that evaluates both directions of an atom pair together."""
    dev = require_device(a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, W_k, rvlen_n, pairs_u)
    pairs_u = _i64(pairs_u, "pairs_u")
    a_ik, rpos_ij_e, tvecs_n = _f32(a_ik, "a_ik"), _f32(rpos_ij_e, "rpos_ij_e"), _f32(tvecs_n, "tvecs_n")
    batch_i, edge_ij_e = _i64(batch_i, "batch_i"), _i64(edge_ij_e, "edge_ij_e")
    W_k, rvlen_n = _f32(W_k, "W_k"), _f32(rvlen_n, "rvlen_n")
    N, H = a_ik.shape
    E = edge_ij_e.shape[1]
    B = tvecs_n.shape[0]
    if rpos_ij_e.shape != (E, 3) or batch_i.shape != (N,) or tvecs_n.shape[1:] != (3, 3):
        raise _lib.CrystalformerHipError("real_enc_fwd: inconsistent input shapes")
    if rvlen_n is not None and rvlen_n.shape != (B, 3):
        raise _lib.CrystalformerHipError("real_enc_fwd: rvlen_n must be (B,3)")
    K = int(K)
    W_num, D = _w_shape(W_k, H, K) if K > 0 else (0, 0)
    cutoff = 0.0 if (cutoff_radius is None or rvlen_n is None) else float(cutoff_radius)
    z = torch.empty((E, H), dtype=torch.float32, device=dev)
    v = None
    if K > 0:
        v = torch.empty((E, H, D if W_k is not None else K), dtype=torch.float32, device=dev)
    if _eval_counter is not None:
        _eval_counter.append(count_translation_evals(a_ik, rvlen_n, batch_i, edge_ij_e, cutoff,
                                                     int(lattice_range), int(minimum_range)))
    with device_guard(dev), _timed("real_enc_fwd", E=E, H=H, K=K, D=D, proj=W_k is not None):
        rc = _lib.load().cf_real_enc_fwd(
            ptr(a_ik), ptr(rpos_ij_e), ptr(tvecs_n), ptr(batch_i), ptr(edge_ij_e), N, H, E, B, K, D,
            float(dist_max), float(wscale), ptr(W_k if K > 0 else None), W_num,
            ptr(rvlen_n), cutoff, int(lattice_range), int(minimum_range), ptr(pairs_u),
            0 if pairs_u is None else pairs_u.shape[0],
            ptr(_scheduling_words(dev) if (pairs_u is not None and DYNAMIC_ROUNDS) else None),
            ptr(z), ptr(v), stream_handle(dev))
    check(rc, "cf_real_enc_fwd")
    return z, v


# Staged translation rings of the latest geometries (see staged_rings): large buffers, so only a
# couple are kept, and only while the tensors they were built from are alive and unmodified.
_ring_cache: list = []
_RING_CACHE_SIZE = 2
STAGED_RINGS_MAX_BYTES = 1 << 30     # 1744 bytes per atom pair: beyond this the blocks stage for themselves


def staged_rings(rpos_ij_e: Tensor, tvecs_n: Tensor, pairs_u: Tensor, K: int, dist_max: float, wscale: float,
                 lattice_range: int, weakest_exponent: float) -> Optional[Tensor]:
    """Per-unit staged translations for :func:`real_enc_fwd_rings` (fixed cube of at most 128
    translations), built once per geometry and bin grid: the blocks of a forward pass hand in the
    same ``rpos_ij_e`` / ``tvecs_n`` / ``pairs_u`` tensors and share one buffer.  ``None`` when the
    cube is too large for the staged kernels."""
    if (2 * int(lattice_range) + 1) ** 3 > 128 or K < 1 or K > 128:
        return None
    # (a launch recorded into a graph and an eager one never share a buffer: a replay stages again)
    dev = require_device(rpos_ij_e, tvecs_n, pairs_u)
    # (the stream is part of the key: rings staged on one stream are not handed to work on another,
    # which nothing orders behind the staging)
    sig = tuple((t.data_ptr(), tuple(t.shape), t._version) for t in (rpos_ij_e, tvecs_n, pairs_u)) + \
        (bool(torch.cuda.is_current_stream_capturing()), stream_handle(dev), int(K), float(dist_max),
         float(wscale), int(lattice_range), float(weakest_exponent))
    for entry in _ring_cache:
        if entry[0] == sig:
            return entry[2]
    L = _lib.load()
    U = pairs_u.shape[0]
    if int(L.cf_real_enc_ring_bytes(U)) > STAGED_RINGS_MAX_BYTES:
        return None
    rings = torch.empty(max(int(L.cf_real_enc_ring_bytes(U)) // 4, 1), dtype=torch.float32, device=dev)
    with device_guard(dev), _timed("real_enc_ring_stage", U=U, K=K):
        rc = L.cf_real_enc_ring_stage(ptr(rpos_ij_e), ptr(tvecs_n), ptr(pairs_u), U, int(K), float(dist_max),
                                      float(wscale), int(lattice_range), float(weakest_exponent), ptr(rings),
                                      stream_handle(dev))
    check(rc, "cf_real_enc_ring_stage")
    _ring_cache.insert(0, (sig, (rpos_ij_e, tvecs_n, pairs_u), rings))
    del _ring_cache[_RING_CACHE_SIZE:]
    return rings


def real_enc_fwd_rings(a_ik: Tensor, edge_ij_e: Tensor, pairs_u: Tensor, rings: Tensor, K: int, dist_max: float,
                       wscale: float, W_k: Tensor, lattice_range: int = 2, rpos_ij_e: Optional[Tensor] = None,
                       tvecs_n: Optional[Tensor] = None, batch_i: Optional[Tensor] = None,
                       rvlen_n: Optional[Tensor] = None, cutoff_radius: Optional[float] = None,
                       minimum_range: int = 0) -> Tuple[Tensor, Tensor]:
    """:func:`real_enc_fwd` for a shared projection from the staged rings (``lattice_range`` the one
    they were staged for).  Fixed cube: every atom pair starts from its ring.  Adaptive boxes
    (``rvlen_n`` and a non-zero ``cutoff_radius``; needs ``rpos_ij_e``, ``tvecs_n`` and ``batch_i`` too):
    the pairs whose half-widths all come out as ``lattice_range`` start from their rings, the others are
    staged by the pair kernel's body; a selection launch, then one launch with both roles."""
    dev = require_device(a_ik, edge_ij_e, pairs_u, rings, W_k, rpos_ij_e, tvecs_n, batch_i, rvlen_n)
    a_ik, W_k = _f32(a_ik, "a_ik"), _f32(W_k, "W_k")
    pairs_u, edge_ij_e = _i64(pairs_u, "pairs_u"), _i64(edge_ij_e, "edge_ij_e")
    N, H = a_ik.shape
    E = edge_ij_e.shape[1]
    U = pairs_u.shape[0]
    W_num, D = _w_shape(W_k, H, int(K))
    L = _lib.load()
    if W_num != 1:
        raise _lib.CrystalformerHipError("real_enc_fwd_rings: one projection per head only")
    if rings.dtype != torch.float32 or rings.numel() * 4 < int(L.cf_real_enc_ring_bytes(U)):
        raise _lib.CrystalformerHipError("real_enc_fwd_rings: rings buffer too small for this pair list")
    cutoff = 0.0 if (cutoff_radius is None or rvlen_n is None) else float(cutoff_radius)
    flags, flag_bytes = None, 0
    if cutoff != 0.0:
        if rpos_ij_e is None or tvecs_n is None or batch_i is None:
            raise _lib.CrystalformerHipError("real_enc_fwd_rings: adaptive boxes need rpos_ij_e, tvecs_n and batch_i")
        rpos_ij_e, tvecs_n, rvlen_n = _f32(rpos_ij_e, "rpos_ij_e"), _f32(tvecs_n, "tvecs_n"), _f32(rvlen_n, "rvlen_n")
        batch_i = _i64(batch_i, "batch_i")
        if rpos_ij_e.shape != (E, 3) or batch_i.shape != (N,) or rvlen_n.shape != (tvecs_n.shape[0], 3):
            raise _lib.CrystalformerHipError("real_enc_fwd_rings: inconsistent input shapes")
        flag_bytes = int(L.cf_real_enc_flag_bytes(U, H))
        flags = torch.empty(max(flag_bytes, 1), dtype=torch.uint8, device=dev)
    z = torch.empty((E, H), dtype=torch.float32, device=dev)
    v = torch.empty((E, H, D), dtype=torch.float32, device=dev)
    if _eval_counter is not None:
        if cutoff == 0.0:
            _eval_counter.append(float(E) * (2 * int(lattice_range) + 1) ** 3)
        else:
            _eval_counter.append(count_translation_evals(a_ik, rvlen_n, batch_i, edge_ij_e, cutoff, int(lattice_range),
                                                         int(minimum_range)))
    with device_guard(dev), _timed("real_enc_fwd", E=E, H=H, K=K, D=D, proj=True):
        rc = L.cf_real_enc_fwd_rings(
            ptr(a_ik), ptr(rpos_ij_e if cutoff != 0.0 else None), ptr(tvecs_n if cutoff != 0.0 else None),
            ptr(batch_i if cutoff != 0.0 else None), ptr(edge_ij_e), ptr(pairs_u), U, N, H, E, int(K), D,
            float(dist_max), float(wscale), ptr(W_k), ptr(rvlen_n if cutoff != 0.0 else None), cutoff,
            int(lattice_range), int(minimum_range), ptr(rings), ptr(flags), flag_bytes, ptr(z), ptr(v),
            stream_handle(dev))
    check(rc, "cf_real_enc_fwd_rings")
    return z, v


def real_enc_bwd(a_ik: Tensor, rpos_ij_e: Tensor, tvecs_n: Tensor, batch_i: Tensor, edge_ij_e: Tensor,
                 e_start_i: Tensor, z_ek: Tensor, gz_ek: Optional[Tensor], gv_ekd: Optional[Tensor],
                 K: int, dist_max: float, wscale: float, W_k: Optional[Tensor] = None,
                 rvlen_n: Optional[Tensor] = None, cutoff_radius: Optional[float] = None,
                 lattice_range: int = 2, minimum_range: int = 0,
                 want_gW: bool = True, pairs_u: Optional[Tensor] = None,
                 rings: Optional[Tensor] = None) -> Tuple[Tensor, Optional[Tensor]]:
    """``rings`` from :func:`staged_rings` (same geometry, pair list, bin grid and cube): the pair
    kernel starts from the staged translations instead of working them out again."""
    _refuse_live_sizes("real_enc_bwd")
    dev = require_device(a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, e_start_i, z_ek, gz_ek, gv_ekd,
                         W_k, rvlen_n, pairs_u, rings)
    pairs_u = _i64(pairs_u, "pairs_u")
    a_ik, rpos_ij_e, tvecs_n = _f32(a_ik, "a_ik"), _f32(rpos_ij_e, "rpos_ij_e"), _f32(tvecs_n, "tvecs_n")
    batch_i, edge_ij_e, e_start_i = _i64(batch_i, "batch_i"), _i64(edge_ij_e, "edge_ij_e"), \
        _i64(e_start_i, "e_start_i")
    z_ek, gz_ek, gv_ekd = _f32(z_ek, "z_ek"), _f32(gz_ek, "gz_ek"), _f32(gv_ekd, "gv_ekd")
    W_k, rvlen_n = _f32(W_k, "W_k"), _f32(rvlen_n, "rvlen_n")
    N, H = a_ik.shape
    E = edge_ij_e.shape[1]
    B = tvecs_n.shape[0]
    K = int(K)
    W_num, D = _w_shape(W_k, H, K) if K > 0 else (0, 0)
    if e_start_i.shape != (N + 1,) or z_ek.shape != (E, H):
        raise _lib.CrystalformerHipError("real_enc_bwd: inconsistent input shapes")
    if gz_ek is not None and gz_ek.shape != (E, H):
        raise _lib.CrystalformerHipError("real_enc_bwd: gz_ek must be (E,H)")
    if gv_ekd is not None and K > 0:
        last = D if W_k is not None else K
        if gv_ekd.shape != (E, H, last):
            raise _lib.CrystalformerHipError(f"real_enc_bwd: gv_ekd must be (E,H,{last})")
    cutoff = 0.0 if (cutoff_radius is None or rvlen_n is None) else float(cutoff_radius)
    want_gW = bool(want_gW and W_k is not None and K > 0)
    ga = torch.empty_like(a_ik)
    gW = torch.empty_like(W_k) if want_gW else None
    L = _lib.load()
    ws_bytes = int(L.cf_real_enc_bwd_workspace(N, H, E, K, D, W_num, 1 if want_gW else 0))
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
    if rings is not None:
        if pairs_u is None or W_k is None or W_num != 1 or cutoff != 0.0:
            raise _lib.CrystalformerHipError("real_enc_bwd: staged rings need the pair list, one projection per "
                                             "head and the fixed cube")
        if rings.dtype != torch.float32 or rings.numel() * 4 < int(L.cf_real_enc_ring_bytes(pairs_u.shape[0])):
            raise _lib.CrystalformerHipError("real_enc_bwd: rings buffer too small for this pair list")
        with device_guard(dev), _timed("real_enc_bwd", E=E, H=H, K=K, D=D, proj=True):
            rc = L.cf_real_enc_bwd_rings(
                ptr(a_ik), ptr(rpos_ij_e), ptr(tvecs_n), ptr(batch_i), ptr(edge_ij_e), ptr(e_start_i),
                ptr(z_ek), ptr(gz_ek), ptr(gv_ekd), N, H, E, B, K, D, float(dist_max), float(wscale), ptr(W_k),
                int(lattice_range), ptr(pairs_u), pairs_u.shape[0], ptr(rings), ptr(ws), ws_bytes,
                ptr(ga), ptr(gW), stream_handle(dev))
        check(rc, "cf_real_enc_bwd_rings")
        return ga, gW
    with device_guard(dev), _timed("real_enc_bwd", E=E, H=H, K=K, D=D, proj=W_k is not None):
        rc = L.cf_real_enc_bwd(
            ptr(a_ik), ptr(rpos_ij_e), ptr(tvecs_n), ptr(batch_i), ptr(edge_ij_e), ptr(e_start_i),
            ptr(z_ek), ptr(gz_ek), ptr(gv_ekd if K > 0 else None), N, H, E, B, K, D, float(dist_max),
            float(wscale), ptr(W_k if K > 0 else None), W_num, ptr(rvlen_n), cutoff, int(lattice_range),
            int(minimum_range), ptr(pairs_u), 0 if pairs_u is None else pairs_u.shape[0], ptr(ws), ws_bytes,
            ptr(ga), ptr(gW), stream_handle(dev))
    check(rc, "cf_real_enc_bwd")
    return ga, gW


def cached_max_row(edge_ij_e: Tensor, e_start_i: Tensor) -> Optional[int]:
    """Largest number of edges of one source atom, read back once per edge list (batch layouts
    know it from their sizes).  ``None`` when it is not known and cannot be read (stream capture)."""
    sig, hit = _cache_lookup("max_row", edge_ij_e)
    if hit is not None:
        return hit
    if edge_ij_e.is_cuda and torch.cuda.is_current_stream_capturing():
        return None
    rows = e_start_i[1:] - e_start_i[:-1]
    return _cache_store(sig, (edge_ij_e,), int(rows.max().item()) if rows.numel() else 0)


def fused_enc_dpa_fwd(a_ik: Tensor, rpos_ij_e: Tensor, tvecs_n: Tensor, batch_i: Tensor, edge_ij_e: Tensor,
                      e_start_i: Tensor, que: Tensor, key: Tensor, val: Tensor, max_row: int,
                      rvlen_n: Optional[Tensor] = None, cutoff_radius: Optional[float] = None,
                      lattice_range: int = 2, minimum_range: int = 0) -> Tensor:
    """Lattice-sum bias (no Gaussian value bins) and attention in one launch, inference only:
    what ``real_enc_fwd(K=0)`` followed by ``fused_dpa_fwd`` yield, without ``z`` in memory."""
    dev = require_device(a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, e_start_i, que, key, val, rvlen_n)
    a_ik, rpos_ij_e, tvecs_n = _f32(a_ik, "a_ik"), _f32(rpos_ij_e, "rpos_ij_e"), _f32(tvecs_n, "tvecs_n")
    que, key, val, rvlen_n = _f32(que, "que"), _f32(key, "key"), _f32(val, "val"), _f32(rvlen_n, "rvlen_n")
    batch_i, edge_ij_e, e_start_i = _i64(batch_i, "batch_i"), _i64(edge_ij_e, "edge_ij_e"), \
        _i64(e_start_i, "e_start_i")
    N, H = a_ik.shape
    E = edge_ij_e.shape[1]
    B = tvecs_n.shape[0]
    Dk, Dv = que.shape[-1], val.shape[-1]
    if que.shape != (N, H, Dk) or key.shape != (N, H, Dk) or val.shape != (N, H, Dv):
        raise _lib.CrystalformerHipError("fused_enc_dpa_fwd: q/k/v must be (N,H,Dk), (N,H,Dk), (N,H,Dv)")
    if rpos_ij_e.shape != (E, 3) or batch_i.shape != (N,) or e_start_i.shape != (N + 1,):
        raise _lib.CrystalformerHipError("fused_enc_dpa_fwd: inconsistent input shapes")
    cutoff = 0.0 if (cutoff_radius is None or rvlen_n is None) else float(cutoff_radius)
    out = torch.empty((N, H, Dv), dtype=torch.float32, device=dev)
    if _eval_counter is not None:
        _eval_counter.append(count_translation_evals(a_ik, rvlen_n, batch_i, edge_ij_e, cutoff,
                                                     int(lattice_range), int(minimum_range)))
    with device_guard(dev), _timed("fused_enc_dpa_fwd", E=E, H=H, Dk=Dk, Dv=Dv):
        rc = _lib.load().cf_fused_enc_dpa_fwd(
            ptr(a_ik), ptr(rpos_ij_e), ptr(tvecs_n), ptr(batch_i), ptr(edge_ij_e), ptr(e_start_i), ptr(que),
            ptr(key), ptr(val), N, H, E, B, Dk, Dv, ptr(rvlen_n), cutoff, int(lattice_range), int(minimum_range),
            int(max_row), ptr(out), stream_handle(dev))
    check(rc, "cf_fused_enc_dpa_fwd")
    return out


def translation_ranges(a_ik: Tensor, rvlen_n: Optional[Tensor], batch_i: Tensor,
                       cutoff_radius: float, lattice_range: int, minimum_range: int) -> Tensor:
    _refuse_live_sizes("translation_ranges")
    dev = require_device(a_ik, rvlen_n, batch_i)
    a_ik, rvlen_n, batch_i = _f32(a_ik, "a_ik"), _f32(rvlen_n, "rvlen_n"), _i64(batch_i, "batch_i")
    N, H = a_ik.shape
    out = torch.empty((N, H, 3), dtype=torch.int32, device=dev)
    with device_guard(dev):
        rc = _lib.load().cf_translation_ranges(ptr(a_ik), ptr(rvlen_n), ptr(batch_i), N, H,
                                               float(cutoff_radius), int(lattice_range),
                                               int(minimum_range), ptr(out), stream_handle(dev))
    check(rc, "cf_translation_ranges")
    return out


def fused_dpa_fwd(que: Tensor, key: Tensor, val: Tensor, aij_eh: Optional[Tensor],
                  bij_ehd: Optional[Tensor], edge_ij_e: Tensor,
                  e_start_i: Tensor) -> Tuple[Tensor, Tensor]:
    dev = require_device(que, key, val, aij_eh, bij_ehd, edge_ij_e, e_start_i)
    que, key, val = _f32(que, "que"), _f32(key, "key"), _f32(val, "val")
    aij_eh, bij_ehd = _f32(aij_eh, "aij_eh"), _f32(bij_ehd, "bij_ehd")
    edge_ij_e, e_start_i = _i64(edge_ij_e, "edge_ij_e"), _i64(e_start_i, "e_start_i")
    N, H, Dk = que.shape
    Dv = val.shape[-1]
    E = edge_ij_e.shape[1]
    if key.shape != (key.shape[0], H, Dk) or val.shape[:2] != (key.shape[0], H):
        raise _lib.CrystalformerHipError("fused_dpa_fwd: inconsistent q/k/v shapes")
    if key.shape[0] != N:
        raise _lib.CrystalformerHipError("fused_dpa_fwd: self-attention only (same atoms for q and k/v)")
    if aij_eh is not None and aij_eh.shape != (E, H):
        raise _lib.CrystalformerHipError("fused_dpa_fwd: aij_eh must be (E,H)")
    if bij_ehd is not None and bij_ehd.shape != (E, H, Dv):
        raise _lib.CrystalformerHipError("fused_dpa_fwd: bij_ehd must be (E,H,Dv)")
    if e_start_i.shape != (N + 1,):
        raise _lib.CrystalformerHipError("fused_dpa_fwd: e_start_i must be (N+1,)")
    prob = torch.empty((E, H), dtype=torch.float32, device=dev)
    out = torch.empty((N, H, Dv), dtype=torch.float32, device=dev)
    with device_guard(dev), _timed("fused_dpa_fwd", E=E, H=H, Dk=Dk, Dv=Dv, bij=bij_ehd is not None):
        rc = _lib.load().cf_fused_dpa_fwd(ptr(que), ptr(key), ptr(val), ptr(aij_eh), ptr(bij_ehd),
                                          ptr(edge_ij_e), ptr(e_start_i), N, H, E, Dk, Dv, ptr(prob),
                                          ptr(out), stream_handle(dev))
    check(rc, "cf_fused_dpa_fwd")
    return out, prob


def fused_dpa_bwd(que: Tensor, key: Tensor, val: Tensor, bij_ehd: Optional[Tensor], batch_i: Tensor,
                  edge_ij_e: Tensor, e_start_i: Tensor, prob_eh: Tensor, out: Tensor, gout: Tensor,
                  atom_start_n: Optional[Tensor] = None, edge_start_n: Optional[Tensor] = None):
    _refuse_live_sizes("fused_dpa_bwd")
    dev = require_device(que, key, val, bij_ehd, batch_i, edge_ij_e, e_start_i, prob_eh, out, gout)
    que, key, val, bij_ehd = _f32(que, "que"), _f32(key, "key"), _f32(val, "val"), _f32(bij_ehd, "bij_ehd")
    prob_eh, out, gout = _f32(prob_eh, "prob_eh"), _f32(out, "out"), _f32(gout, "gout")
    batch_i, edge_ij_e, e_start_i = _i64(batch_i, "batch_i"), _i64(edge_ij_e, "edge_ij_e"), \
        _i64(e_start_i, "e_start_i")
    N, H, Dk = que.shape
    Dv = val.shape[-1]
    E = edge_ij_e.shape[1]
    # the key-side kernel walks the column (i,j) of a crystal's block at e0 + i*n + j
    if cached_dense_sizes(batch_i, edge_ij_e) is None:
        raise _lib.CrystalformerHipError(
            "fused_dpa_bwd needs the dense per-crystal edge blocks of get_edge_index "
            "(sorted batch_i, edge (i,j) at e0 + i*n + j); this edge list is not of that form")
    if atom_start_n is None or edge_start_n is None:
        atom_start_n, edge_start_n = cached_crystal_offsets(batch_i)
    atom_start_n, edge_start_n = _i64(atom_start_n, "atom_start_n"), _i64(edge_start_n, "edge_start_n")
    B = atom_start_n.numel() - 1
    gq, gk, gv = torch.empty_like(que), torch.empty_like(key), torch.empty_like(val)
    ga = torch.empty((E, H), dtype=torch.float32, device=dev)
    gb = torch.empty((E, H, Dv), dtype=torch.float32, device=dev) if bij_ehd is not None else None
    with device_guard(dev), _timed("fused_dpa_bwd", E=E, H=H, Dk=Dk, Dv=Dv, bij=bij_ehd is not None):
        rc = _lib.load().cf_fused_dpa_bwd(
            ptr(que), ptr(key), ptr(val), ptr(bij_ehd), ptr(batch_i), ptr(edge_ij_e), ptr(e_start_i),
            ptr(atom_start_n), ptr(edge_start_n), N, H, E, B, Dk, Dv, ptr(prob_eh), ptr(out), ptr(gout),
            ptr(gq), ptr(gk), ptr(gv), ptr(ga), ptr(gb), stream_handle(dev))
    check(rc, "cf_fused_dpa_bwd")
    return gq, gk, gv, ga, gb


def irregular_mean_fwd(x_ik: Tensor, start_n: Tensor) -> Tensor:
    dev = require_device(x_ik, start_n)
    x_ik, start_n = _f32(x_ik, "x_ik"), _i64(start_n, "start_n")
    N = x_ik.shape[0]
    B = start_n.numel() - 1
    D = x_ik.numel() // N if N > 0 else 0
    out = torch.empty((B,) + tuple(x_ik.shape[1:]), dtype=torch.float32, device=dev)
    with device_guard(dev):
        rc = _lib.load().cf_irregular_mean_fwd(ptr(x_ik), ptr(start_n), B, D, ptr(out), stream_handle(dev))
    check(rc, "cf_irregular_mean_fwd")
    return out


def irregular_mean_bwd(go_nk: Tensor, batch_i: Tensor, start_n: Tensor) -> Tensor:
    _refuse_live_sizes("irregular_mean_bwd")
    dev = require_device(go_nk, batch_i, start_n)
    go_nk, batch_i, start_n = _f32(go_nk, "go_nk"), _i64(batch_i, "batch_i"), _i64(start_n, "start_n")
    N = batch_i.numel()
    D = go_nk.numel() // go_nk.shape[0] if go_nk.shape[0] > 0 else 0
    gx = torch.empty((N,) + tuple(go_nk.shape[1:]), dtype=torch.float32, device=dev)
    with device_guard(dev):
        rc = _lib.load().cf_irregular_mean_bwd(ptr(go_nk), ptr(batch_i), ptr(start_n), N, D, ptr(gx),
                                               stream_handle(dev))
    check(rc, "cf_irregular_mean_bwd")
    return gx


def minimum_distance(rpos_ij_e: Tensor, tvecs_n: Tensor, batch_i: Tensor, edge_ij_e: Tensor,
                     rvlen_n: Optional[Tensor], cutoff_radius: float, lattice_range: int = 2,
                     minimum_range: int = 0) -> Tensor:
    _refuse_live_sizes("minimum_distance")
    dev = require_device(rpos_ij_e, tvecs_n, batch_i, edge_ij_e, rvlen_n)
    rpos_ij_e, tvecs_n, rvlen_n = _f32(rpos_ij_e, "rpos_ij_e"), _f32(tvecs_n, "tvecs_n"), \
        _f32(rvlen_n, "rvlen_n")
    batch_i, edge_ij_e = _i64(batch_i, "batch_i"), _i64(edge_ij_e, "edge_ij_e")
    E = edge_ij_e.shape[1]
    out = torch.empty((E,), dtype=torch.float32, device=dev)
    with device_guard(dev):
        rc = _lib.load().cf_minimum_distance(ptr(rpos_ij_e), ptr(tvecs_n), ptr(batch_i), ptr(edge_ij_e), E,
                                             ptr(rvlen_n), float(cutoff_radius), int(lattice_range),
                                             int(minimum_range), ptr(out), stream_handle(dev))
    check(rc, "cf_minimum_distance")
    return out


def edge_index(sizes: Tensor, pos: Optional[Tensor] = None,
               num_edges: Optional[int] = None) -> Tuple[Tensor, Optional[Tensor]]:
    """Dense intra-crystal edge list (2,E) and, with ``pos``, p_j - p_i (E,3),
    built on the device.  ``num_edges`` (sum of sizes^2) avoids a host sync when
    the caller already knows it."""
    dev = require_device(sizes, pos)
    sizes = _i64(sizes, "sizes")
    pos = _f32(pos, "pos")
    B = sizes.numel()
    atom_start = F.pad(sizes.cumsum(0), (1, 0))
    edge_start = F.pad((sizes * sizes).cumsum(0), (1, 0))
    if num_edges is None:
        # one host read per distinct ``sizes`` tensor; repeated forwards over the same batch
        # (and stream capture after a warm-up) find the count in the cache
        sig, hit = _cache_lookup("num_edges", sizes)
        if hit is None:
            hit = _cache_store(sig, (sizes,), int(edge_start[-1].item()))
        num_edges = hit
    E = int(num_edges)
    edges = torch.empty((2, E), dtype=torch.int64, device=dev)
    rpos = torch.empty((E, 3), dtype=torch.float32, device=dev) if pos is not None else None
    with device_guard(dev):
        rc = _lib.load().cf_edge_index(ptr(atom_start), ptr(edge_start), B, E, ptr(pos), ptr(edges),
                                       ptr(rpos), stream_handle(dev))
    check(rc, "cf_edge_index")
    return edges, rpos


PAIR_FIELDS = 5   # words per unit descriptor: e_ij, e_ji, i, j, crystal


def edge_pairs(sizes: Tensor, num_atoms: Optional[int] = None, num_edges: Optional[int] = None) -> Tensor:
    """(U,5) int64 unit descriptors: for every unordered atom pair of each crystal's
    dense edge block the edge (i->j), i <= j, its reverse (j->i), the atoms i and j
    and the crystal.  U = (E + N)/2; pass
    ``num_atoms`` and ``num_edges`` when known to avoid a host sync."""
    dev = require_device(sizes)
    sizes = _i64(sizes, "sizes")
    B = sizes.numel()
    atom_start = F.pad(sizes.cumsum(0), (1, 0))
    edge_start = F.pad((sizes * sizes).cumsum(0), (1, 0))
    unit_start = F.pad((sizes * (sizes + 1) // 2).cumsum(0), (1, 0))
    if num_atoms is None or num_edges is None:
        tail = torch.stack([atom_start[-1], edge_start[-1]]).tolist() if B > 0 else [0, 0]
        num_atoms, num_edges = int(tail[0]), int(tail[1])
    U = (num_edges + num_atoms) // 2
    pairs = torch.empty((U, PAIR_FIELDS), dtype=torch.int64, device=dev)
    with device_guard(dev):
        rc = _lib.load().cf_edge_pairs(ptr(atom_start), ptr(edge_start), ptr(unit_start), B, num_edges,
                                       ptr(pairs), stream_handle(dev))
    check(rc, "cf_edge_pairs")
    return pairs


def cached_edge_row_offsets(edge_ij_e: Tensor, num_atoms: int) -> Tensor:
    sig, hit = _cache_lookup("e_start", edge_ij_e)
    if hit is not None and hit.numel() == num_atoms + 1:
        return hit
    return _cache_store(sig, (edge_ij_e,), edge_row_offsets(edge_ij_e, num_atoms))


def dense_block_layout(batch_i: Tensor, edge_ij_e: Tensor) -> Optional[Tensor]:
    """Crystal sizes (B,) if ``edge_ij_e`` is exactly the dense per-crystal block list of
    ``get_edge_index`` for the crystals of ``batch_i`` (atoms of a crystal contiguous, edge
    (i,j) of a crystal with n atoms at e0 + i*n + j), else ``None``.  Plain torch ops on the
    tensors' own device; reads three small results back to the host, so it is meant for the
    first sight of a batch, not for every launch."""
    N, E = batch_i.numel(), edge_ij_e.shape[1]
    dev = batch_i.device
    if edge_ij_e.dim() != 2 or edge_ij_e.shape[0] != 2:
        return None
    if N == 0:
        return torch.zeros(0, dtype=torch.int64, device=dev) if E == 0 else None
    head = torch.stack([(batch_i[1:] >= batch_i[:-1]).all().long(), batch_i[0], batch_i[-1]]).tolist()
    if not head[0] or head[1] < 0 or head[2] >= (1 << 24):
        return None
    B = head[2] + 1                       # crystal ids index the lattices as they are
    sizes = torch.zeros(B, dtype=torch.int64, device=dev)
    sizes.scatter_add_(0, batch_i, torch.ones_like(batch_i))
    if int((sizes * sizes).sum().item()) != E:
        return None
    atom_start = F.pad(sizes.cumsum(0), (1, 0))
    edge_start = F.pad((sizes * sizes).cumsum(0), (1, 0))
    crystal = torch.repeat_interleave(torch.arange(B, device=dev), sizes * sizes, output_size=E)
    local = torch.arange(E, device=dev) - edge_start[crystal]
    n_e = sizes[crystal]
    dense = torch.stack([local // n_e, local % n_e]) + atom_start[crystal]
    return sizes if torch.equal(dense, edge_ij_e) else None


def cached_dense_sizes(batch_i: Tensor, edge_ij_e: Tensor) -> Optional[Tensor]:
    """:func:`dense_block_layout`, verified once per (batch_i, edge_ij_e) pair."""
    sig, hit = _cache_lookup("dense", batch_i, edge_ij_e)
    if hit is not None:
        return hit[0]
    if batch_i.is_cuda and torch.cuda.is_current_stream_capturing():
        raise _lib.CrystalformerHipError(
            "an edge list first seen under stream capture cannot be checked for the dense block "
            "layout (the check reads back to the host): run one eager call on it first")
    return _cache_store(sig, (batch_i, edge_ij_e), (dense_block_layout(batch_i, edge_ij_e),))[0]


def cached_edge_pairs(batch_i: Tensor, edge_ij_e: Tensor, num_crystals: int) -> Optional[Tensor]:
    """Pair list (see :func:`edge_pairs`) if the edge list is the dense per-crystal block
    layout, verified on first sight; ``None`` for any other edge list (the callers then take
    the per-edge kernels, which read the list as it is)."""
    sig, hit = _cache_lookup("pairs", batch_i, edge_ij_e)
    if hit is not None:
        return hit
    sizes = cached_dense_sizes(batch_i, edge_ij_e)
    if sizes is None:
        return None
    if sizes.numel() > num_crystals:
        raise _lib.CrystalformerHipError(
            f"batch_i names {sizes.numel()} crystals but only {num_crystals} lattices were given")
    pairs = edge_pairs(sizes, batch_i.numel(), edge_ij_e.shape[1])
    return _cache_store(sig, (batch_i, edge_ij_e), pairs)


def cached_crystal_offsets(batch_i: Tensor) -> Tuple[Tensor, Tensor]:
    sig, hit = _cache_lookup("offsets", batch_i)
    if hit is not None:
        return hit
    return _cache_store(sig, (batch_i,), crystal_offsets(batch_i))


class BatchLayout:
    """Index structure of a batch of crystals with dense intra-crystal edges.
    Depends on the crystal sizes only, so it is built once per ``sizes`` tensor and
    reused by every forward over that batch (and baked into a captured graph)."""

    __slots__ = ("sizes", "batch", "atom_start", "edge_start", "num_atoms", "num_edges", "edges",
                 "e_start", "pairs")


def batch_layout(sizes: Tensor, batch_i: Tensor) -> BatchLayout:
    """Layout for ``sizes`` (B,) / ``batch_i`` (N,), cached on the identity and version
    of both tensors.  ``layout.batch`` is ``batch_i`` renumbered from 0.  The derived
    tensors are also entered in the index caches under the keys the operators use."""
    live = current_live_sizes()
    if live is not None:
        return _live_batch_layout(sizes, batch_i, live)
    sig, hit = _cache_lookup("layout", sizes, batch_i)
    if hit is not None:
        return hit
    dev = require_device(sizes, batch_i)
    sizes = _i64(sizes, "sizes")
    lay = BatchLayout()
    lay.sizes = sizes
    lay.batch = (batch_i - batch_i[0]) if batch_i.numel() else batch_i
    # the one host read per distinct batch: the atom and edge counts size everything below
    sizes_host = sizes.tolist()
    B = len(sizes_host)
    lay.num_atoms = sum(sizes_host)
    lay.num_edges = sum(n * n for n in sizes_host)
    if lay.num_atoms != batch_i.numel():
        raise _lib.CrystalformerHipError(
            f"sizes sum to {lay.num_atoms} atoms but batch has {batch_i.numel()} entries")
    if B == 0 or lay.num_edges == 0 or min(sizes_host) < 0:
        lay.atom_start = F.pad(sizes.cumsum(0), (1, 0))
        lay.edge_start = F.pad((sizes * sizes).cumsum(0), (1, 0))
        lay.edges, _ = edge_index(sizes, None, lay.num_edges)
        lay.e_start = edge_row_offsets(lay.edges, lay.num_atoms)
        lay.pairs = edge_pairs(sizes, lay.num_atoms, lay.num_edges) if lay.num_edges else None
    else:
        # prefix sums, row offsets, edge list and pair list in four launches
        N, E = lay.num_atoms, lay.num_edges
        starts = torch.empty((3, B + 1), dtype=torch.int64, device=dev)
        lay.atom_start, lay.edge_start = starts[0], starts[1]
        lay.e_start = torch.empty(N + 1, dtype=torch.int64, device=dev)
        lay.edges = torch.empty((2, E), dtype=torch.int64, device=dev)
        lay.pairs = torch.empty(((E + N) // 2, PAIR_FIELDS), dtype=torch.int64, device=dev)
        with device_guard(dev):
            rc = _lib.load().cf_batch_layout(ptr(sizes), B, N, E, ptr(starts[0]), ptr(starts[1]), ptr(starts[2]),
                                             ptr(lay.e_start), ptr(lay.edges), ptr(lay.pairs), None,
                                             stream_handle(dev))
        check(rc, "cf_batch_layout")
    _enter_layout(lay, max(sizes_host) if sizes_host else 0)
    return _cache_store(sig, (sizes, batch_i), lay)


def _enter_layout(lay: BatchLayout, max_row: Optional[int]) -> None:
    """The derived tensors of a layout under the keys the operators look them up with."""
    s_, _ = _cache_lookup("e_start", lay.edges)
    _cache_store(s_, (lay.edges,), lay.e_start)
    if lay.pairs is not None:
        s_, _ = _cache_lookup("pairs", lay.batch, lay.edges)
        _cache_store(s_, (lay.batch, lay.edges), lay.pairs)
    if max_row is not None:
        s_, _ = _cache_lookup("max_row", lay.edges)            # a row has as many edges as its crystal atoms
        _cache_store(s_, (lay.edges,), max_row)
    s_, _ = _cache_lookup("dense", lay.batch, lay.edges)       # dense by construction
    _cache_store(s_, (lay.batch, lay.edges), (lay.sizes,))
    s_, _ = _cache_lookup("offsets", lay.batch)
    _cache_store(s_, (lay.batch,), (lay.atom_start, lay.edge_start))
    s_, _ = _cache_lookup("mean_start", lay.sizes)
    _cache_store(s_, (lay.sizes,), lay.atom_start)


def _live_batch_layout(sizes: Tensor, batch_i: Tensor, live: "live_sizes") -> BatchLayout:
    """:func:`batch_layout` inside :class:`live_sizes`: every tensor has the capacity's shape, the
    kernels work out the counts from ``sizes`` (crystals past the live ones hold 0) and leave them
    in the header.  Nothing is read back and nothing is cached on ``sizes``, whose contents change
    from one use of the buffers to the next."""
    dev = require_device(sizes, batch_i, live.header)
    sizes = _i64(sizes, "sizes")
    N, E = live.atoms, live.edges
    B = sizes.numel()
    if batch_i.numel() != N:
        raise _lib.CrystalformerHipError(
            f"live sizes: batch has {batch_i.numel()} entries, the atom capacity is {N}")
    if B < 1:
        raise _lib.CrystalformerHipError("live sizes: no crystal slots")
    lay = BatchLayout()
    lay.sizes = sizes
    lay.batch = torch.empty(N, dtype=torch.int64, device=dev)      # written by the layout kernels
    lay.num_atoms, lay.num_edges = N, E
    starts = torch.empty((3, B + 1), dtype=torch.int64, device=dev)
    lay.atom_start, lay.edge_start = starts[0], starts[1]
    lay.e_start = torch.empty(N + 1, dtype=torch.int64, device=dev)
    lay.edges = torch.empty((2, E), dtype=torch.int64, device=dev)
    lay.pairs = torch.empty((live.units, PAIR_FIELDS), dtype=torch.int64, device=dev)
    with device_guard(dev):
        rc = _lib.load().cf_batch_layout(ptr(sizes), B, N, E, ptr(starts[0]), ptr(starts[1]), ptr(starts[2]),
                                         ptr(lay.e_start), ptr(lay.edges), ptr(lay.pairs), ptr(lay.batch),
                                         stream_handle(dev))
    check(rc, "cf_batch_layout")
    _enter_layout(lay, None)
    return lay


def copy_segments(pairs) -> None:
    """``dst.copy_(src)`` for up to eight ``(dst, src)`` pairs of contiguous tensors on one GPU in a
    single launch; ``src`` None fills ``dst`` with zeros.  Element counts and types must agree."""
    import ctypes
    pairs = [(d, s) for d, s in pairs if d.numel() > 0]
    if not pairs:
        return
    dev = require_device(*[t for pr in pairs for t in pr if t is not None])
    for d, s in pairs:
        if not d.is_contiguous() or (s is not None and (not s.is_contiguous() or s.dtype != d.dtype
                                                         or s.numel() != d.numel())):
            raise _lib.CrystalformerHipError("copy_segments: contiguous tensors of equal type and size expected")
    n = len(pairs)
    src = (ctypes.c_void_p * n)(*[None if s is None else s.data_ptr() for _, s in pairs])
    dst = (ctypes.c_void_p * n)(*[d.data_ptr() for d, _ in pairs])
    nbytes = (ctypes.c_int64 * n)(*[d.numel() * d.element_size() for d, _ in pairs])
    with device_guard(dev):
        rc = _lib.load().cf_copy_segments(n, src, dst, nbytes, stream_handle(dev))
    check(rc, "cf_copy_segments")


def relative_positions(layout: BatchLayout, pos: Tensor) -> Tensor:
    """p_j - p_i for every edge of the layout, (E,3)
    (models/indexed_latticeformer_encoder.py:214)."""
    dev = require_device(pos)
    pos = _f32(pos, "pos")
    if pos.shape != (layout.num_atoms, 3):
        raise _lib.CrystalformerHipError(f"pos must be ({layout.num_atoms},3), got {tuple(pos.shape)}")
    rpos = torch.empty((layout.num_edges, 3), dtype=torch.float32, device=dev)
    with device_guard(dev):
        rc = _lib.load().cf_edge_index(ptr(layout.atom_start), ptr(layout.edge_start), layout.sizes.numel(),
                                       layout.num_edges, ptr(pos), None, ptr(rpos), stream_handle(dev))
    check(rc, "cf_edge_index")
    return rpos


def lattice_geometry(trans_n: Tensor) -> Tuple[Tensor, Tensor, Tensor]:
    """(vcell (B), recip (B,3,3), rvlen (B,3)) of the lattices ``trans_n`` (B,3,3)
    in one launch (models/indexed_latticeformer_encoder.py:34-44, 206-212)."""
    dev = require_device(trans_n)
    trans_n = _f32(trans_n, "trans_n")
    if trans_n.dim() != 3 or trans_n.shape[1:] != (3, 3):
        raise _lib.CrystalformerHipError(f"trans_n must be (B,3,3), got {tuple(trans_n.shape)}")
    B = trans_n.shape[0]
    vcell = torch.empty(B, dtype=torch.float32, device=dev)
    recip = torch.empty((B, 3, 3), dtype=torch.float32, device=dev)
    rvlen = torch.empty((B, 3), dtype=torch.float32, device=dev)
    with device_guard(dev):
        rc = _lib.load().cf_lattice_geometry(ptr(trans_n), B, ptr(vcell), ptr(recip), ptr(rvlen),
                                             stream_handle(dev))
    check(rc, "cf_lattice_geometry")
    return vcell, recip, rvlen


POSITIVE_FUNCS = {"elu": 0, "abs": 1, "exp": 2}


def gauss_exponents(q_ihd: Tensor, w_hd: Tensor, gauss_scale: Optional[Tensor], normalize: bool,
                    update_stats: bool, positive_func: str, beta: float, lower_bound: float, coef: float,
                    q_scale: Optional[float] = None,
                    want_alpha: bool = False) -> Tuple[Tensor, Optional[Tensor], Optional[Tensor], Optional[Tensor]]:
    """a[i,h] = coef * rho(normalised <q[i,h], w[h]>), the scaled query and
    (optionally) the normalised alpha, in two launches
    (models/indexed_lattice_multi_head_attention_cuda.py:636-722).
    ``gauss_scale`` (2,) is read, and written in place when ``update_stats``.
    Returns ``(a, q_scaled, alpha_n, used)``; ``used`` is the (scale, shift) pair
    applied (None without normalisation)."""
    dev = require_device(q_ihd, w_hd, gauss_scale)
    q_ihd = _f32(q_ihd, "q_ihd")
    w_hd = _f32(w_hd, "w_hd")
    if q_ihd.dim() != 3:
        raise _lib.CrystalformerHipError("q_ihd must be (N,H,D)")
    N, H, D = q_ihd.shape
    if w_hd.numel() != H * D:
        raise _lib.CrystalformerHipError(f"w_hd has {w_hd.numel()} elements, expected H*D = {H * D}")
    if positive_func not in POSITIVE_FUNCS:
        raise _lib.CrystalformerHipError(f"positive map {positive_func!r} has no kernel")
    if normalize:
        if gauss_scale is None or gauss_scale.numel() != 2 or gauss_scale.dtype != torch.float32 \
                or not gauss_scale.is_contiguous():
            raise _lib.CrystalformerHipError("gauss_scale must be a contiguous float32 tensor of 2 elements")
    lib = _lib.load()
    a = torch.empty((N, H), dtype=torch.float32, device=dev)
    qs = torch.empty_like(q_ihd) if q_scale is not None else None
    alpha_n = torch.empty((N, H), dtype=torch.float32, device=dev) if want_alpha else None
    ws_bytes = int(lib.cf_gauss_exponents_workspace(N, H)) if normalize else 0
    ws = torch.empty(max(ws_bytes // 4, 1), dtype=torch.float32, device=dev) if normalize else None
    with device_guard(dev):
        rc = lib.cf_gauss_exponents(ptr(q_ihd), ptr(w_hd), ptr(gauss_scale) if normalize else None, N, H, D,
                                    int(bool(normalize)), int(bool(update_stats)),
                                    POSITIVE_FUNCS[positive_func], float(beta), float(lower_bound), float(coef),
                                    float(q_scale if q_scale is not None else 1.0), ptr(ws), ws_bytes,
                                    ptr(alpha_n), ptr(a), ptr(qs), stream_handle(dev))
    check(rc, "cf_gauss_exponents")
    return a, qs, alpha_n, (ws[-4:-2] if normalize else None)


def kr_base(rpos_ij_e: Tensor, rvecs_n: Tensor, batch_i: Tensor, edge_ij_e: Tensor) -> Tensor:
    """(E,3) phases <b_d, p_j - p_i> of the reciprocal-space encoding
    (models/indexed_latticeformer_encoder.py:245-251)."""
    _refuse_live_sizes("the reciprocal-space encoding")
    dev = require_device(rpos_ij_e, rvecs_n, batch_i, edge_ij_e)
    rpos_ij_e, rvecs_n = _f32(rpos_ij_e, "rpos_ij_e"), _f32(rvecs_n, "rvecs_n")
    batch_i, edge_ij_e = _i64(batch_i, "batch_i"), _i64(edge_ij_e, "edge_ij_e")
    E = edge_ij_e.shape[1]
    if rpos_ij_e.shape != (E, 3) or rvecs_n.shape[1:] != (3, 3):
        raise _lib.CrystalformerHipError("kr_base: rpos (E,3) and rvecs (B,3,3) expected")
    out = torch.empty((E, 3), dtype=torch.float32, device=dev)
    with device_guard(dev):
        rc = _lib.load().cf_kr_base(ptr(rpos_ij_e), ptr(rvecs_n), ptr(batch_i), ptr(edge_ij_e), E, ptr(out),
                                    stream_handle(dev))
    check(rc, "cf_kr_base")
    return out


def _reci_operands(a_ik, kr_base_e, rvecs_n, batch_i, e_start_i):
    a_ik, kr_base_e, rvecs_n = _f32(a_ik, "a_ik"), _f32(kr_base_e, "kr_base_e"), _f32(rvecs_n, "rvecs_n")
    batch_i, e_start_i = _i64(batch_i, "batch_i"), _i64(e_start_i, "e_start_i")
    if a_ik.dim() != 2 or kr_base_e.dim() != 2 or kr_base_e.shape[1] != 3 or rvecs_n.shape[1:] != (3, 3) \
            or batch_i.shape != (a_ik.shape[0],) or e_start_i.shape != (a_ik.shape[0] + 1,):
        raise _lib.CrystalformerHipError("reciprocal encoding: a (N,H), kr_base (E,3), rvecs (B,3,3), batch (N), "
                                         "e_start (N+1) expected")
    return a_ik, kr_base_e, rvecs_n, batch_i, e_start_i


def reci_enc_fwd(a_ik: Tensor, kr_base_e: Tensor, rvecs_n: Tensor, vcell_n: Tensor, batch_i: Tensor,
                 e_start_i: Tensor, lattice_range: int) -> Tuple[Tensor, Tensor]:
    """``(z_ek, sumexp_ek)`` of the reciprocal-space lattice sum."""
    _refuse_live_sizes("the reciprocal-space encoding")
    dev = require_device(a_ik, kr_base_e, rvecs_n, vcell_n, batch_i, e_start_i)
    a_ik, kr_base_e, rvecs_n, batch_i, e_start_i = _reci_operands(a_ik, kr_base_e, rvecs_n, batch_i, e_start_i)
    vcell_n = _f32(vcell_n, "vcell_n")
    N, H = a_ik.shape
    E = kr_base_e.shape[0]
    if vcell_n.numel() != rvecs_n.shape[0]:
        raise _lib.CrystalformerHipError("reciprocal encoding: one cell volume per crystal expected")
    z = torch.empty((E, H), dtype=torch.float32, device=dev)
    se = torch.empty((E, H), dtype=torch.float32, device=dev)
    with device_guard(dev):
        rc = _lib.load().cf_reci_enc_fwd(ptr(a_ik), ptr(kr_base_e), ptr(rvecs_n), ptr(vcell_n), ptr(batch_i),
                                         ptr(e_start_i), N, H, E, int(lattice_range), ptr(z), ptr(se),
                                         stream_handle(dev))
    check(rc, "cf_reci_enc_fwd")
    return z, se


def reci_enc_bwd(a_ik: Tensor, kr_base_e: Tensor, rvecs_n: Tensor, batch_i: Tensor, e_start_i: Tensor,
                 gz_ek: Tensor, sumexp_ek: Tensor, lattice_range: int, normalisation_grad: bool = False) -> Tensor:
    """``ga_ik`` of the reciprocal-space lattice sum: by default the reference kernel's
    definition, which leaves the normalisation term's derivative out; with
    ``normalisation_grad`` the full derivative of z."""
    _refuse_live_sizes("reci_enc_bwd")
    dev = require_device(a_ik, kr_base_e, rvecs_n, batch_i, e_start_i, gz_ek, sumexp_ek)
    a_ik, kr_base_e, rvecs_n, batch_i, e_start_i = _reci_operands(a_ik, kr_base_e, rvecs_n, batch_i, e_start_i)
    gz_ek, sumexp_ek = _f32(gz_ek, "gz_ek"), _f32(sumexp_ek, "sumexp_ek")
    N, H = a_ik.shape
    E = kr_base_e.shape[0]
    if gz_ek.shape != (E, H) or sumexp_ek.shape != (E, H):
        raise _lib.CrystalformerHipError("reciprocal encoding: gz and sumexp must be (E,H)")
    ga = torch.empty((N, H), dtype=torch.float32, device=dev)
    with device_guard(dev):
        rc = _lib.load().cf_reci_enc_bwd(ptr(a_ik), ptr(kr_base_e), ptr(rvecs_n), ptr(batch_i), ptr(e_start_i),
                                         ptr(gz_ek), ptr(sumexp_ek), N, H, E, int(lattice_range),
                                         int(bool(normalisation_grad)), ptr(ga),
                                         stream_handle(dev))
    check(rc, "cf_reci_enc_bwd")
    return ga


def gauss_exponents_bwd(ga: Optional[Tensor], gqs: Optional[Tensor], q_ihd: Tensor, w_hd: Tensor,
                        alpha_n: Tensor, used: Optional[Tensor], positive_func: str, beta: float,
                        lower_bound: float, coef: float, q_scale: float, want_gq: bool = True,
                        want_gw: bool = True) -> Tuple[Optional[Tensor], Optional[Tensor]]:
    """Gradients of :func:`gauss_exponents` with respect to the query and the head weights
    (statistics held constant), one launch plus a fixed-order reduction."""
    dev = require_device(ga, gqs, q_ihd, w_hd, alpha_n, used)
    ga, gqs, q_ihd, w_hd, alpha_n = (_f32(t, n) for t, n in ((ga, "ga"), (gqs, "gqs"), (q_ihd, "q_ihd"),
                                                              (w_hd, "w_hd"), (alpha_n, "alpha_n")))
    N, H, D = q_ihd.shape
    if w_hd.numel() != H * D or alpha_n.numel() != N * H or (ga is not None and ga.numel() != N * H) \
            or (gqs is not None and gqs.shape != q_ihd.shape):
        raise _lib.CrystalformerHipError("gauss_exponents_bwd: operand shapes disagree")
    if positive_func not in POSITIVE_FUNCS:
        raise _lib.CrystalformerHipError(f"positive map {positive_func!r} has no kernel")
    if used is not None:
        used = _f32(used, "used")
    lib = _lib.load()
    gq = torch.empty_like(q_ihd) if want_gq else None
    gw = torch.empty((H, D), dtype=torch.float32, device=dev) if want_gw else None
    if gq is None and gw is None:
        return None, None
    ws_bytes = int(lib.cf_gauss_exponents_bwd_workspace(N, H, D)) if want_gw else 0
    ws = torch.empty(max(ws_bytes // 4, 1), dtype=torch.float32, device=dev) if want_gw else None
    with device_guard(dev):
        rc = lib.cf_gauss_exponents_bwd(ptr(ga), ptr(gqs), ptr(q_ihd), ptr(w_hd), ptr(alpha_n), ptr(used), N, H, D,
                                        POSITIVE_FUNCS[positive_func], float(beta), float(lower_bound), float(coef),
                                        float(q_scale), ptr(ws), ws_bytes, ptr(gq), ptr(gw), stream_handle(dev))
    check(rc, "cf_gauss_exponents_bwd")
    return gq, gw


def linear_rows_supported(x: Tensor, *weights: Tensor) -> bool:
    """True when :func:`linear_rows` serves these operands (float32 on the GPU, input
    width a multiple of 16, equal weight shapes)."""
    if not x.is_cuda or x.dtype != torch.float32 or x.dim() != 2 or x.shape[1] % 16 != 0:
        return False
    return all(w.is_cuda and w.dtype == torch.float32 and w.dim() == 2 and w.shape == weights[0].shape
               and w.shape[1] == x.shape[1] for w in weights) and 1 <= len(weights) <= 3


def _plain_f32(t: Tensor, dev: torch.device) -> bool:
    return t.dtype is torch.float32 and t.device == dev and t.is_contiguous()


def linear_rows(x: Tensor, weights, bias: Optional[Tensor] = None, residual: Optional[Tensor] = None,
                relu: bool = False):
    """``act(x @ w.T + b) (+ residual)`` for up to three equally shaped weights in one
    launch; returns a tuple of outputs, one per weight.  No autograd."""
    dev = x.device
    nw = len(weights)
    # operands that need no conversion and no message (the hot case: this wrapper runs 18 times
    # in a forward of the four-block model) skip the general checks below
    lean = (dev.type == "cuda" and x.dim() == 2 and 1 <= nw <= 3 and _plain_f32(x, dev)
            and (bias is None or _plain_f32(bias, dev)) and (residual is None or _plain_f32(residual, dev)))
    if lean:
        for w in weights:
            if not (_plain_f32(w, dev) and w.dim() == 2):
                lean = False
                break
    if not lean:
        weights = [_f32(w, "weight") for w in weights]
        dev = require_device(x, *weights, bias, residual)
        x = _f32(x, "x")
        bias = _f32(bias, "bias")
        residual = _f32(residual, "residual")
        if x.dim() != 2 or not 1 <= nw <= 3 or any(w.dim() != 2 for w in weights):
            raise _lib.CrystalformerHipError("linear_rows: x (N, K) and one to three weights (C, K) expected")
    N, K = x.shape
    C = weights[0].shape[0]
    for w in weights:
        if w.shape[0] != C or w.shape[1] != K:
            raise _lib.CrystalformerHipError("linear_rows: weights must all be (C, K) with K = x.shape[1]")
    if bias is not None and bias.numel() != nw * C:
        raise _lib.CrystalformerHipError("linear_rows: bias must have one entry per output column")
    if residual is not None and (nw != 1 or residual.shape != (N, C)):
        raise _lib.CrystalformerHipError("linear_rows: residual must be (N, C) with a single weight")
    y0 = torch.empty((N, C), dtype=torch.float32, device=dev)
    y1 = torch.empty((N, C), dtype=torch.float32, device=dev) if nw > 1 else None
    y2 = torch.empty((N, C), dtype=torch.float32, device=dev) if nw > 2 else None
    with device_guard(dev):
        rc = _lib.load().cf_linear_rows(
            x.data_ptr(), N, K, weights[0].data_ptr(), weights[1].data_ptr() if nw > 1 else None,
            weights[2].data_ptr() if nw > 2 else None, nw, C, ptr(bias), ptr(residual), 1 if relu else 0,
            y0.data_ptr(), ptr(y1), ptr(y2), stream_handle(dev))
    if rc:
        check(rc, "cf_linear_rows")
    return (y0,) if nw == 1 else ((y0, y1) if nw == 2 else (y0, y1, y2))


def linear_rows_nn_supported(g: Tensor, w: Tensor) -> bool:
    """True when :func:`linear_rows_nn` serves g (N,C) @ w (C,K): float32 on the GPU, C a
    multiple of 64, K a multiple of 4."""
    return (g.is_cuda and w.is_cuda and g.dtype == torch.float32 and w.dtype == torch.float32 and g.dim() == 2
            and w.dim() == 2 and g.shape[1] == w.shape[0] and g.shape[1] % 64 == 0 and w.shape[1] % 4 == 0)


def linear_rows_nn(gs, weights, add: Optional[Tensor] = None, mask: Optional[Tensor] = None) -> Tensor:
    """``mask(sum_i gs[i] @ weights[i]) + add`` for up to three terms of equal shapes in one
    launch: the input gradient of linear layers ``y = x W^T`` (``weights[i]`` is W as stored,
    (C,K) = (out, in)).  ``mask`` zeroes the product where it is not positive."""
    gs = [_f32(g, "g") for g in gs]
    weights = [_f32(w, "weight") for w in weights]
    dev = require_device(*gs, *weights, add, mask)
    add, mask = _f32(add, "add"), _f32(mask, "mask")
    if not 1 <= len(gs) <= 3 or len(gs) != len(weights):
        raise _lib.CrystalformerHipError("linear_rows_nn: one to three (g, weight) pairs expected")
    N, C = gs[0].shape
    K = weights[0].shape[1]
    if any(g.shape != (N, C) for g in gs) or any(w.shape != (C, K) for w in weights):
        raise _lib.CrystalformerHipError("linear_rows_nn: g (N,C) and weight (C,K) of equal shapes expected")
    for t, name in ((add, "add"), (mask, "mask")):
        if t is not None and t.shape != (N, K):
            raise _lib.CrystalformerHipError(f"linear_rows_nn: {name} must be (N,K)")
    y = torch.empty((N, K), dtype=torch.float32, device=dev)
    g3 = gs + [None] * (3 - len(gs))
    w3 = weights + [None] * (3 - len(weights))
    with device_guard(dev):
        rc = _lib.load().cf_linear_rows_nn(ptr(g3[0]), ptr(g3[1]), ptr(g3[2]), len(gs), ptr(w3[0]), ptr(w3[1]),
                                           ptr(w3[2]), N, C, K, ptr(add), ptr(mask), ptr(y), stream_handle(dev))
    check(rc, "cf_linear_rows_nn")
    return y


def column_sum(g: Tensor) -> Tensor:
    """Sum over the rows of a (N,C) float32 matrix, fixed order, one launch."""
    dev = require_device(g)
    g = _f32(g, "g")
    if g.dim() != 2:
        raise _lib.CrystalformerHipError("column_sum: g must be (N,C)")
    N, C = g.shape
    out = torch.empty(C, dtype=torch.float32, device=dev)
    with device_guard(dev):
        rc = _lib.load().cf_column_sum(ptr(g), N, C, ptr(out), stream_handle(dev))
    check(rc, "cf_column_sum")
    return out


def linear_weight_grad(g: Tensor, x: Tensor, with_bias: bool = False):
    """``g.T @ x`` for g (N,C), x (N,K): the weight gradient of a linear layer, fixed order.
    ``with_bias``: returns ``(gW, gb)``, gb the column sums of g from the same pass."""
    dev = require_device(g, x)
    g, x = _f32(g, "g"), _f32(x, "x")
    if g.dim() != 2 or x.dim() != 2 or g.shape[0] != x.shape[0]:
        raise _lib.CrystalformerHipError("linear_weight_grad: g (N,C) and x (N,K) expected")
    N, C = g.shape
    K = x.shape[1]
    lib = _lib.load()
    ws_bytes = int(lib.cf_linear_weight_grad_workspace(N, C, K))
    ws = torch.empty(max(ws_bytes // 4, 1), dtype=torch.float32, device=dev)
    out = torch.empty((C, K), dtype=torch.float32, device=dev)
    gb = torch.empty((C,), dtype=torch.float32, device=dev) if with_bias else None
    with device_guard(dev):
        rc = lib.cf_linear_weight_grad(ptr(g), ptr(x), N, C, K, ptr(ws), ws_bytes, ptr(out), ptr(gb),
                                       stream_handle(dev))
    check(rc, "cf_linear_weight_grad")
    return (out, gb) if with_bias else out


def linear_weight_grad_grouped(layers) -> None:
    """Weight and bias gradients of several linear layers in two launches.  ``layers`` is a
    list of ``(g (N,C), x (N,K), gW out (C,K), gb out (C) or None)``; the outputs are
    written in place and equal :func:`linear_weight_grad` bit for bit."""
    import ctypes
    if not layers:
        return
    flat = [t for layer in layers for t in layer]
    dev = require_device(*flat)
    n = len(layers)
    for g, x, gw, gb in layers:
        for t in (g, x, gw, gb):
            if t is not None and (t.dtype != torch.float32 or not t.is_contiguous()):
                raise _lib.CrystalformerHipError("linear_weight_grad_grouped: contiguous float32 tensors expected")
        if g.dim() != 2 or x.dim() != 2 or g.shape[0] != x.shape[0] or gw.shape != (g.shape[1], x.shape[1]) \
                or (gb is not None and gb.numel() != g.shape[1]):
            raise _lib.CrystalformerHipError("linear_weight_grad_grouped: g (N,C), x (N,K), gW (C,K), gb (C) expected")
    PtrArr, I64Arr = ctypes.c_void_p * n, ctypes.c_int64 * n
    Ns = I64Arr(*[l[0].shape[0] for l in layers])
    Cs = I64Arr(*[l[0].shape[1] for l in layers])
    Ks = I64Arr(*[l[1].shape[1] for l in layers])
    lib = _lib.load()
    ws_bytes = int(lib.cf_linear_weight_grad_grouped_workspace(n, Ns, Cs, Ks))
    ws = torch.empty(max(ws_bytes // 4, 1), dtype=torch.float32, device=dev)
    with device_guard(dev):
        rc = lib.cf_linear_weight_grad_grouped(
            n, PtrArr(*[l[0].data_ptr() for l in layers]), PtrArr(*[l[1].data_ptr() for l in layers]), Ns, Cs, Ks,
            PtrArr(*[l[2].data_ptr() for l in layers]),
            PtrArr(*[(l[3].data_ptr() if l[3] is not None else None) for l in layers]),
            ptr(ws), ws_bytes, stream_handle(dev))
    check(rc, "cf_linear_weight_grad_grouped")


class AdamWPlan:
    """Host-side tables for :func:`adamw_step`: the pointer arrays of the parameters and
    moments (fixed for the life of the optimiser), element counts, decay factors and the
    chunk-sum workspace."""

    def __init__(self, params, exp_avg, exp_avg_sq, weight_decay):
        import ctypes
        dev = require_device(*params)
        n = len(params)
        for t in list(params) + list(exp_avg) + list(exp_avg_sq):
            if t.dtype != torch.float32 or not t.is_contiguous() or t.device != dev:
                raise _lib.CrystalformerHipError("adamw_step: contiguous float32 tensors on one GPU expected")
        self.device, self.n = dev, n
        self.keep = (list(params), list(exp_avg), list(exp_avg_sq))
        self.p = (ctypes.c_void_p * n)(*[t.data_ptr() for t in params])
        self.m = (ctypes.c_void_p * n)(*[t.data_ptr() for t in exp_avg])
        self.v = (ctypes.c_void_p * n)(*[t.data_ptr() for t in exp_avg_sq])
        self.numel = (ctypes.c_int64 * n)(*[t.numel() for t in params])
        self.wd = (ctypes.c_float * n)(*[float(w) for w in weight_decay])
        self.GradArray = ctypes.c_void_p * n
        self.ws_bytes = int(_lib.load().cf_adamw_step_workspace(n, self.numel))
        if self.ws_bytes < 0:
            raise _lib.CrystalformerHipError("adamw_step: bad tensor sizes")
        self.ws = torch.empty(max(self.ws_bytes // 4, 1), dtype=torch.float32, device=dev)


def adamw_step(plan: AdamWPlan, grads, lr0: float, sch_decay: float, beta1: float, beta2: float, eps: float,
               clip_norm: float, state: Tensor) -> None:
    """In place: clip the gradients' global norm, AdamW-update the plan's parameters and
    moments, advance ``state`` (3 floats on the device: updates taken, gradient norm, lr)."""
    dev = plan.device
    if len(grads) != plan.n:
        raise _lib.CrystalformerHipError("adamw_step: one gradient per parameter expected")
    for g, p in zip(grads, plan.keep[0]):
        if g is None:
            raise _lib.CrystalformerHipError("adamw_step: a parameter has no gradient")
        if g.dtype != torch.float32 or not g.is_contiguous() or g.device != dev or g.numel() != p.numel():
            raise _lib.CrystalformerHipError("adamw_step: gradients must be contiguous float32 of the parameter's size")
    if state.dtype != torch.float32 or state.numel() != 3 or state.device != dev:
        raise _lib.CrystalformerHipError("adamw_step: state is 3 floats on the device")
    g_arr = plan.GradArray(*[g.data_ptr() for g in grads])
    with device_guard(dev):
        rc = _lib.load().cf_adamw_step(plan.n, plan.p, g_arr, plan.m, plan.v, plan.numel, plan.wd, lr0, sch_decay,
                                       beta1, beta2, eps, clip_norm, ptr(state), ptr(plan.ws), plan.ws_bytes,
                                       stream_handle(dev))
    check(rc, "cf_adamw_step")


def l1_mean_loss(pred: Tensor, target: Tensor, with_grad: bool = True):
    """``(loss, grad)``: the L1 losses of a batch summed over the targets and averaged over the
    batch (one float on the device), and ``sign(pred - target) / B`` (None without
    ``with_grad``), in one launch.  ``pred`` and ``target`` are (B, T)."""
    dev = require_device(pred, target)
    pred, target = _f32(pred, "pred"), _f32(target, "target")
    if pred.dim() != 2 or target.shape != pred.shape or pred.shape[0] < 1 or pred.shape[1] < 1:
        raise _lib.CrystalformerHipError("l1_mean_loss: pred and target must both be (B, T), B and T at least 1")
    B, T = pred.shape
    loss = torch.empty(1, dtype=torch.float32, device=dev)
    grad = torch.empty_like(pred) if with_grad else None
    with device_guard(dev):
        rc = _lib.load().cf_l1_mean_loss(ptr(pred), ptr(target), B, T, ptr(loss), ptr(grad), stream_handle(dev))
    check(rc, "cf_l1_mean_loss")
    return loss, grad
