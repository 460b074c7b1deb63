"""ctypes binding of liblookupffn_hip.so (the C ABI declared in include/lookupffn_hip.h).

There is no CPU implementation behind this module and no fallback: if the
library is missing or does not load, every entry point raises.
"""
from __future__ import annotations

import ctypes
import os
import threading

import torch

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
# LOOKUPFFN_HIP_LIB points at another build of the same ABI (e.g. a tuning build)
LIB_PATH = os.environ.get("LOOKUPFFN_HIP_LIB") or os.path.join(_PKG_DIR, "liblookupffn_hip.so")

ABI_VERSION = 7

LFFN_OK = 0
LFFN_ERR_BAD_ARG = -1
LFFN_ERR_UNSUPPORTED = -2
LFFN_ERR_LAUNCH = -3
LFFN_ERR_SCRATCH = -4

_vp = ctypes.c_void_p
_i64 = ctypes.c_int64
_f32 = ctypes.c_float
_i32 = ctypes.c_int32

# name -> argument types (every entry point returns int except the two below)
SIGNATURES = {
    "lffn_fht_f32": [_vp, _vp, _i64, _i64, _vp],
    "lffn_fht_f16": [_vp, _vp, _i64, _i64, _vp],
    "lffn_fht_bf16": [_vp, _vp, _i64, _i64, _vp],
    "lffn_bh4_diag_f32": [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp],
    "lffn_mix_code_score_f32": [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64,
                                ctypes.c_float, ctypes.c_float, _vp],
    "lffn_ln_bh4_block_hash_f32": [_vp, _vp, _vp, ctypes.c_float, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64,
                                   _i64, _i64, ctypes.c_float, ctypes.c_float, _vp],
    "lffn_project_hash_bwd_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64,
                                  ctypes.c_float, ctypes.c_float, _vp],
    "lffn_bh4_block_hash_train_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64,
                                      ctypes.c_float, ctypes.c_float, _vp],
    "lffn_ln_bh4_block_hash_train_f32": [_vp, _vp, _vp, _f32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64,
                                         _i64, _i64, _f32, _f32, _vp],
    "lffn_ln_bh4_block_wgrad_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _vp],
    "lffn_bh4_fold_mode_f32": [_vp, _vp, _i64, _i64, ctypes.c_int32, _vp],
    "lffn_bh4_block_bwd_f32": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64,
                               ctypes.c_float, ctypes.c_float, _vp],
    "lffn_lookup_ffn_fused_f32": [_vp, _vp, _vp, ctypes.c_float, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64,
                                  _i64, _i64, _i64, ctypes.c_float, ctypes.c_float, _vp],
    "lffn_layer_norm_bwd_f32": [_vp, _vp, ctypes.c_float, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp],
    "lffn_layer_norm_bwd_noalloc_f32": [_vp, _vp, ctypes.c_float, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp],
    "lffn_bh4_block_wgrad_f32": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _vp],
    "lffn_bh4_fold_f32": [_vp, _vp, _i64, _i64, _i64, _i64, _vp],
    "lffn_bh4_block_f32": [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _vp],
    "lffn_project_hash_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _f32, _vp],
    "lffn_ln_project_hash_f32": [_vp, _vp, _vp, _f32, _vp, _vp, _vp, _vp, _vp,
                                 _i64, _i64, _i64, _i64, _i64, _i64, _f32, _f32, _vp],
    "lffn_ln_project_hash_bwd_f32": [_vp, _vp, _vp, _f32, _vp, _vp, _vp, _vp, _vp, _vp,
                                     _i64, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _f32, _vp],
    "lffn_sum_partials_f32": [_vp, _vp, _i64, _vp, _vp, _i64, _i64, _i64, _vp],
    "lffn_code_score_f32": [_vp, _vp, _vp, _i64, _i64, _vp],
    "lffn_code_score_bwd_f32": [_vp, _vp, _vp, _i64, _i64, _vp],
    "lffn_gather_add_f32": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp],
    "lffn_gather_add_bf16": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp],
    "lffn_gather_add_f16": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp],
    "lffn_lookup_gather_f32": [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp],
    "lffn_lookup_gather_bf16": [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp],
    "lffn_lookup_gather_residual_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp],
    "lffn_lookup_gather_residual_bf16": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp],
    "lffn_lookup_gather_planned_f32": [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64,
                                       ctypes.c_int32, ctypes.c_int32, _vp],
    "lffn_lookup_gather_planned_bf16": [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64,
                                        ctypes.c_int32, ctypes.c_int32, _vp],
    "lffn_lookup_gather_workspace_bytes": [_i64, _i64, _i64, _i64, ctypes.c_int32, ctypes.POINTER(ctypes.c_int64)],
    "lffn_lookup_gather_ws_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp],
    "lffn_lookup_gather_ws_bf16": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp],
    "lffn_lookup_gather_ws_f16": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp],
    "lffn_lookup_gather_ws_plan": [_i64, _i64, _i64, _i64, ctypes.c_int32, _i64, ctypes.POINTER(ctypes.c_int32)],
    "lffn_lookup_gather_ws_planned_rows": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, ctypes.c_int32,
                                           ctypes.c_int32, ctypes.c_int32, _vp],
    "lffn_lookup_gather_ws_planned_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, ctypes.c_int32, ctypes.c_int32, _vp],
    "lffn_ln_project_hash_records_f32": [_vp, _vp, _vp, _f32, _vp, _vp, _vp, _i64, _i32, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _f32, _vp],
    "lffn_ln_bh4_block_hash_records_f32": [_vp, _vp, _vp, _f32, _vp, _vp, _vp, _i64, _i32, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _f32, _vp],
    "lffn_lookup_gather_records_plan": [_i64, _i64, _i64, _i64, ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int64)],
    "lffn_lookup_gather_records_f32": [_vp, _i64, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, ctypes.c_int32, _vp],
    "lffn_lookup_gather_records_plan_rows": [_i64, _i64, _i64, _i64, ctypes.c_int32, ctypes.POINTER(ctypes.c_int32),
                                             ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int64)],
    "lffn_lookup_gather_records_rows": [_vp, _i64, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, ctypes.c_int32, ctypes.c_int32, _vp],
    "lffn_lookup_gather_plan": [_i64, _i64, _i64, _i64, ctypes.c_int32, ctypes.POINTER(ctypes.c_int32)],
    "lffn_indexed_inner_product_f32": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp],
    "lffn_scatter_add_f32": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp],
    "lffn_indexed_inner_product_f16": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp],
    "lffn_scatter_add_f16": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp],
    "lffn_lookup_scatter_f32": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, ctypes.c_int32, _vp],
    "lffn_lookup_scatter_workspace_bytes": [_i64, _i64, _i64, _i64, ctypes.POINTER(ctypes.c_int64)],
    "lffn_lookup_scatter_sorted_f32": [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, ctypes.c_int32, _vp],
    "lffn_lookup_backward_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, ctypes.c_int32, _vp],
    "lffn_lookup_inner_f32": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp],
}

class FusedLayer(ctypes.Structure):
    """struct lffn_fused_layer of include/lookupffn_hip.h."""
    _fields_ = [("ln_weight", _vp), ("ln_bias", _vp), ("diag", _vp), ("proj_bias", _vp), ("tables", _vp), ("out_bias", _vp),
                ("H", _i64), ("D", _i64), ("R", _i64), ("J", _i64), ("T", _i64), ("S", _i64), ("Do", _i64),
                ("ln_eps", _f32), ("decay", _f32), ("residual", _f32)]


SIGNATURES["lffn_lookup_ffn_fused_layer_f32"] = [ctypes.POINTER(FusedLayer), _vp, _vp, _vp, _i64, _vp]

_lib = None
_lock = threading.Lock()


class LookupFFNLibraryError(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    """Load the kernel library once; raise if it is absent or of another ABI version."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise LookupFFNLibraryError(
                f"{LIB_PATH} is missing: build it with `python -m lookupffn_amd._build` "
                "(hipcc, gfx950). lookupffn_amd has no CPU or PyTorch fallback.")
        try:
            lib = ctypes.CDLL(LIB_PATH)
        except OSError as e:
            raise LookupFFNLibraryError(f"cannot load {LIB_PATH}: {e}") from e
        lib.lffn_version.restype = ctypes.c_int
        lib.lffn_version.argtypes = []
        lib.lffn_error_string.restype = ctypes.c_char_p
        lib.lffn_error_string.argtypes = [ctypes.c_int]
        if lib.lffn_version() != ABI_VERSION:          # first: an older library lacks some of the entry points below
            raise LookupFFNLibraryError(
                f"{LIB_PATH} has ABI version {lib.lffn_version()}, this package needs {ABI_VERSION}: rebuild it")
        for name, argtypes in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = ctypes.c_int
            fn.argtypes = argtypes
        _lib = lib
        return _lib


def exported_symbols():
    return ["lffn_version", "lffn_error_string", *SIGNATURES.keys()]


def check(rc: int, what: str) -> None:
    if rc != LFFN_OK:
        msg = load().lffn_error_string(rc).decode()
        raise RuntimeError(f"{what}: {msg} (code {rc})")


def ptr(t):
    return None if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_of(t: torch.Tensor) -> int:
    """The HIP stream torch currently launches on for t's device, as an integer handle."""
    if _raw_stream is not None:          # a tenth of the cost of building a torch.cuda.Stream object
        idx = t.device.index
        return _raw_stream(torch.cuda.current_device() if idx is None else idx)
    return torch.cuda.current_stream(t.device).cuda_stream


def require_gpu(*tensors) -> torch.device:
    """All tensors must live on one GPU; return it.  CPU tensors are an error:
    this package only runs on the GPU."""
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError(
                "lookupffn_amd: got a CPU tensor; the kernels run on an MI355X only "
                "(there is no CPU path in this package)")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f"lookupffn_amd: tensors on different devices ({dev} and {t.device})")
    return dev
