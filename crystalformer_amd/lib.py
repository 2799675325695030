"""ctypes binding of ``libcrystalformer_hip.so`` (the C ABI declared in
``include/crystalformer_hip.h``).

The library is built ahead of time for gfx950 with ``hipcc`` (see
``csrc/Makefile``); there is no CPU fallback: every call raises if the shared
object is missing or a kernel launch is rejected.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Optional

import torch

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libcrystalformer_hip.so")
CSRC_DIR = os.path.join(_PKG_DIR, "csrc")

_i64 = ctypes.c_int64
_int = ctypes.c_int
_dbl = ctypes.c_double
_f32 = ctypes.c_float
_ptr = ctypes.c_void_p

# name -> (restype, argtypes); mirrors include/crystalformer_hip.h
SIGNATURES = {
    "cf_version": (_int, []),
    "cf_last_error": (ctypes.c_char_p, []),
    "cf_max_translation_range": (_int, []),
    "cf_set_launch_share": (_int, [_dbl]),
    "cf_get_launch_share": (_dbl, []),
    "cf_set_size_header": (_int, [_ptr, _i64, _i64]),
    "cf_get_size_header": (_ptr, []),
    "cf_real_enc_fwd": (_int, [_ptr] * 5 + [_i64] * 6 + [_dbl, _dbl, _ptr, _i64, _ptr, _dbl, _int, _int,
                                                         _ptr, _i64, _ptr, _ptr, _ptr, _ptr]),
    "cf_real_enc_ring_bytes": (_i64, [_i64]),
    "cf_real_enc_ring_stage": (_int, [_ptr, _ptr, _ptr, _i64, _i64, _dbl, _dbl, _int, _dbl, _ptr, _ptr]),
    "cf_real_enc_flag_bytes": (_i64, [_i64, _i64]),
    "cf_real_enc_fwd_rings": (_int, [_ptr] * 6 + [_i64] * 6 + [_dbl, _dbl, _ptr, _ptr, _dbl, _int, _int, _ptr, _ptr,
                                                               _i64, _ptr, _ptr, _ptr]),
    "cf_real_enc_bwd_workspace": (_i64, [_i64] * 6 + [_int]),
    "cf_real_enc_bwd": (_int, [_ptr] * 9 + [_i64] * 6 + [_dbl, _dbl, _ptr, _i64, _ptr, _dbl, _int, _int,
                                                         _ptr, _i64, _ptr, _i64, _ptr, _ptr, _ptr]),
    "cf_real_enc_bwd_rings": (_int, [_ptr] * 9 + [_i64] * 6 + [_dbl, _dbl, _ptr, _int, _ptr, _i64, _ptr, _ptr, _i64,
                                                               _ptr, _ptr, _ptr]),
    "cf_static_scratch_bytes": (_i64, []),
    "cf_real_enc_bwd_static": (_int, [_ptr] * 9 + [_i64] * 6 + [_dbl, _dbl, _ptr, _i64, _ptr, _dbl, _int, _int,
                                                                _ptr, _i64, _ptr, _ptr, _ptr]),
    "cf_fused_enc_dpa_fwd": (_int, [_ptr] * 9 + [_i64] * 6 + [_ptr, _dbl, _int, _int, _i64, _ptr, _ptr]),
    "cf_translation_ranges": (_int, [_ptr, _ptr, _ptr, _i64, _i64, _dbl, _int, _int, _ptr, _ptr]),
    "cf_fused_dpa_fwd": (_int, [_ptr] * 7 + [_i64] * 5 + [_ptr, _ptr, _ptr]),
    "cf_fused_dpa_bwd": (_int, [_ptr] * 9 + [_i64] * 6 + [_ptr] * 9),
    "cf_irregular_mean_fwd": (_int, [_ptr, _ptr, _i64, _i64, _ptr, _ptr]),
    "cf_irregular_mean_bwd": (_int, [_ptr, _ptr, _ptr, _i64, _i64, _ptr, _ptr]),
    "cf_minimum_distance": (_int, [_ptr] * 4 + [_i64, _ptr, _dbl, _int, _int, _ptr, _ptr]),
    "cf_edge_index": (_int, [_ptr, _ptr, _i64, _i64, _ptr, _ptr, _ptr, _ptr]),
    "cf_edge_pairs": (_int, [_ptr, _ptr, _ptr, _i64, _i64, _ptr, _ptr]),
    "cf_linear_rows": (_int, [_ptr, _i64, _i64, _ptr, _ptr, _ptr, _int, _i64, _ptr, _ptr, _int, _ptr, _ptr, _ptr, _ptr]),
    "cf_linear_rows_nn": (_int, [_ptr, _ptr, _ptr, _int, _ptr, _ptr, _ptr, _i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr]),
    "cf_linear_weight_grad_workspace": (_i64, [_i64, _i64, _i64]),
    "cf_linear_weight_grad": (_int, [_ptr, _ptr, _i64, _i64, _i64, _ptr, _i64, _ptr, _ptr, _ptr]),
    "cf_linear_weight_grad_grouped_workspace": (_i64, [_int, _ptr, _ptr, _ptr]),
    "cf_linear_weight_grad_grouped": (_int, [_int, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _ptr]),
    "cf_column_sum": (_int, [_ptr, _i64, _i64, _ptr, _ptr]),
    "cf_gauss_exponents_bwd_workspace": (_i64, [_i64, _i64, _i64]),
    "cf_gauss_exponents_bwd": (_int, [_ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _i64, _int, _f32, _f32, _f32,
                                      _f32, _ptr, _i64, _ptr, _ptr, _ptr]),
    "cf_kr_base": (_int, [_ptr, _ptr, _ptr, _ptr, _i64, _ptr, _ptr]),
    "cf_reci_enc_fwd": (_int, [_ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _i64, _int, _ptr, _ptr, _ptr]),
    "cf_reci_enc_bwd": (_int, [_ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _i64, _int, _int, _ptr, _ptr]),
    "cf_adamw_step_workspace": (_i64, [_int, _ptr]),
    "cf_adamw_step": (_int, [_int, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _f32, _f32, _f32, _f32, _f32, _f32, _ptr,
                             _ptr, _i64, _ptr]),
    "cf_l1_mean_loss": (_int, [_ptr, _ptr, _i64, _i64, _ptr, _ptr, _ptr]),
    "cf_batch_layout": (_int, [_ptr, _i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr]),
    "cf_copy_segments": (_int, [_int, _ptr, _ptr, _ptr, _ptr]),
    "cf_lattice_geometry": (_int, [_ptr, _i64, _ptr, _ptr, _ptr, _ptr]),
    "cf_gauss_exponents_workspace": (_i64, [_i64, _i64]),
    "cf_gauss_exponents": (_int, [_ptr, _ptr, _ptr, _i64, _i64, _i64, _int, _int, _int, _f32, _f32, _f32, _f32,
                                  _ptr, _i64, _ptr, _ptr, _ptr, _ptr]),
}

_lib: Optional[ctypes.CDLL] = None


class CrystalformerHipError(RuntimeError):
    pass


def build(verbose: bool = False) -> str:
    """(Re)compile the HIP sources for gfx950.  Works without a GPU."""
    cmd = ["make", "-C", CSRC_DIR, "-B", "-j8"]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose or res.returncode != 0:
        print(res.stdout)
    if res.returncode != 0:
        raise CrystalformerHipError("building libcrystalformer_hip.so failed")
    global _lib
    _lib = None
    return LIB_PATH


def is_built() -> bool:
    return os.path.exists(LIB_PATH)


def load() -> ctypes.CDLL:
    """Load the shared object and attach the declared signatures."""
    global _lib
    if _lib is not None:
        return _lib
    if not is_built():
        raise CrystalformerHipError(
            f"{LIB_PATH} is missing: build it with `make -C {CSRC_DIR}` "
            "(hipcc --offload-arch=gfx950); there is no CPU fallback")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().cf_last_error().decode("utf-8", "replace")
        raise CrystalformerHipError(f"{what} failed ({rc}): {msg}")


def ptr(t: Optional[torch.Tensor]) -> int:
    """Device address of a tensor (0 for None)."""
    return 0 if t is None else t.data_ptr()


class _NoGuard:
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def device_guard(device: torch.device):
    """Context that makes ``device`` current for a launch; free when it already is (the
    common case: switching the device context costs microseconds per call)."""
    if torch.cuda.current_device() == device.index:
        return _NO_GUARD
    return torch.cuda.device(device)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_handle(device: torch.device) -> int:
    """hipStream_t of torch's current stream on ``device``."""
    if _raw_stream is not None:                       # same value, a tenth of the cost
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


def require_device(*tensors: Optional[torch.Tensor]) -> torch.device:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise CrystalformerHipError(
                "HIP operators need tensors on a GPU device; got a CPU tensor (there is no CPU fallback)")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise CrystalformerHipError("all tensors must live on the same device")
    if dev is None:
        raise CrystalformerHipError("no tensor given")
    return dev
