"""TEST INFRASTRUCTURE ONLY: numpy front-end of the C restatement in this directory.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package.  The product package never does.

Every function takes and returns numpy arrays; ``dtype`` float32 runs the
reference's arithmetic in the reference's order, float64 is the truth used for
tolerances.  The C library is built by ``oracle/Makefile``.
"""
from __future__ import annotations

import ctypes
import importlib.util
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liblffn_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile the C restatement (and oracle/_ref where the reference is present)."""
    if force:
        subprocess.run(["make", "-C", _HERE, "-B", "liblffn_oracle.so"], check=True)
        subprocess.run(["make", "-C", _HERE, "ref"], check=True)
    elif not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE, "liblffn_oracle.so"], check=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def num_threads() -> int:
    return int(lib().orc_num_threads())


def _sfx(dtype) -> str:
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return "f32"
    if dtype == np.float64:
        return "f64"
    raise TypeError(f"oracle: unsupported dtype {dtype}")


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def _real(dtype, v):
    return ctypes.c_float(v) if np.dtype(dtype) == np.float32 else ctypes.c_double(v)


_i64 = ctypes.c_int64


def fht(x):
    """out = x @ H_D, unnormalised, natural order."""
    x = np.ascontiguousarray(x)
    B, D = x.shape
    assert D & (D - 1) == 0
    out = np.empty_like(x)
    getattr(lib(), "orc_fht_" + _sfx(x.dtype))(_p(x), _p(out), _i64(B), _i64(D))
    return out


def bh4(x, w):
    """x [B,D], w [R,J,D/bs,bs,bs] -> [B,R*D]."""
    x = np.ascontiguousarray(x)
    w = _c(w, x.dtype)
    B, D = x.shape
    R, J, NB, bs, bs2 = w.shape
    assert bs == bs2 and NB * bs == D
    out = np.empty((B, R * D), dtype=x.dtype)
    getattr(lib(), "orc_bh4_" + _sfx(x.dtype))(
        _p(x), _p(w), _p(out), _i64(B), _i64(D), _i64(R), _i64(J), _i64(bs))
    return out


def projection(x, w, bias, out_dim, decay=0.7):
    """BH4 module forward: x [B,H] -> z [B,out_dim]."""
    x = np.ascontiguousarray(x)
    w = _c(w, x.dtype)
    bias = None if bias is None else _c(bias, x.dtype)
    B, H = x.shape
    R, J, NB, bs, _ = w.shape
    D = NB * bs
    assert H <= D and out_dim <= R * D
    z = np.empty((B, out_dim), dtype=x.dtype)
    getattr(lib(), "orc_projection_" + _sfx(x.dtype))(
        _p(x), _p(w), _p(bias), _p(z), _i64(B), _i64(H), _i64(D), _i64(R), _i64(J),
        _i64(bs), _i64(out_dim), _real(x.dtype, decay))
    return z


def code_score(z):
    """z [..., k] -> (code int32 [...], score [...])."""
    z = np.ascontiguousarray(z)
    k = z.shape[-1]
    N = z.size // k
    codes = np.empty(z.shape[:-1], dtype=np.int32)
    scores = np.empty(z.shape[:-1], dtype=z.dtype)
    getattr(lib(), "orc_code_score_" + _sfx(z.dtype))(_p(z), _p(codes), _p(scores), _i64(N), _i64(k))
    return codes, scores


def code_score_bwd(z, g_score):
    z = np.ascontiguousarray(z)
    g_score = _c(g_score, z.dtype)
    k = z.shape[-1]
    N = z.size // k
    g_z = np.empty_like(z)
    getattr(lib(), "orc_code_score_bwd_" + _sfx(z.dtype))(_p(z), _p(g_score), _p(g_z), _i64(N), _i64(k))
    return g_z


def gather_add(idx, src, w):
    """out[b] = sum_i w[b,i] * src[idx[b,i]]."""
    src = np.ascontiguousarray(src)
    idx = _c(idx, np.int32)
    w = _c(w, src.dtype)
    B, I = idx.shape
    Sz, Dv = src.shape
    assert idx.min(initial=0) >= 0 and idx.max(initial=0) < Sz
    out = np.empty((B, Dv), dtype=src.dtype)
    getattr(lib(), "orc_gather_add_" + _sfx(src.dtype))(
        _p(idx), _p(src), _p(w), _p(out), _i64(B), _i64(I), _i64(Dv))
    return out


def gather_add_bf16(idx, src_bits, w):
    """src_bits: uint16 bfloat16 bit patterns [Sz,Dv]; accumulate in w.dtype."""
    src_bits = _c(src_bits, np.uint16)
    idx = _c(idx, np.int32)
    w = np.ascontiguousarray(w)
    B, I = idx.shape
    Sz, Dv = src_bits.shape
    assert idx.min(initial=0) >= 0 and idx.max(initial=0) < Sz
    out = np.empty((B, Dv), dtype=w.dtype)
    getattr(lib(), "orc_gather_add_bf16_" + _sfx(w.dtype))(
        _p(idx), _p(src_bits), _p(w), _p(out), _i64(B), _i64(I), _i64(Dv))
    return out


def indexed_inner_product(idx, g, src):
    src = np.ascontiguousarray(src)
    g = _c(g, src.dtype)
    idx = _c(idx, np.int32)
    B, I = idx.shape
    Sz, Dv = src.shape
    assert idx.min(initial=0) >= 0 and idx.max(initial=0) < Sz
    out = np.empty((B, I), dtype=src.dtype)
    getattr(lib(), "orc_indexed_inner_product_" + _sfx(src.dtype))(
        _p(idx), _p(g), _p(src), _p(out), _i64(B), _i64(I), _i64(Dv))
    return out


def scatter_add(idx, g, w, out_size):
    g = np.ascontiguousarray(g)
    w = _c(w, g.dtype)
    idx = _c(idx, np.int32)
    B, I = idx.shape
    Dv = g.shape[1]
    assert idx.min(initial=0) >= 0 and idx.max(initial=0) < out_size
    out = np.empty((out_size, Dv), dtype=g.dtype)
    getattr(lib(), "orc_scatter_add_" + _sfx(g.dtype))(
        _p(idx), _p(g), _p(w), _p(out), _i64(B), _i64(I), _i64(out_size), _i64(Dv))
    return out


def layernorm(x, gamma, beta, eps):
    x = np.ascontiguousarray(x)
    B, H = x.shape
    out = np.empty_like(x)
    getattr(lib(), "orc_layernorm_" + _sfx(x.dtype))(
        _p(x), _p(_c(gamma, x.dtype)), _p(_c(beta, x.dtype)), _real(x.dtype, eps), _p(out), _i64(B), _i64(H))
    return out


def lookup_ffn(x, ln_w, ln_b, eps, proj_w, proj_b, tables, bias, decay=0.7, return_parts=False):
    """Whole layer.  x [B,H]; proj_w [R,J,D/bs,bs,bs]; tables [T,S,Do]."""
    x = np.ascontiguousarray(x)
    dt = x.dtype
    B, H = x.shape
    proj_w = _c(proj_w, dt)
    R, J, NB, bs, _ = proj_w.shape
    D = NB * bs
    tables = _c(tables, dt)
    T, S, Do = tables.shape
    k = int(S).bit_length() - 1
    assert 1 << k == S and T * k <= R * D
    out = np.empty((B, Do), dtype=dt)
    z = np.empty((B, T * k), dtype=dt)
    codes = np.empty((B, T), dtype=np.int32)
    scores = np.empty((B, T), dtype=dt)
    getattr(lib(), "orc_lookup_ffn_" + _sfx(dt))(
        _p(x), _p(_c(ln_w, dt)), _p(_c(ln_b, dt)), _real(dt, eps),
        _p(proj_w), _p(None if proj_b is None else _c(proj_b, dt)), _real(dt, decay),
        _p(tables), _p(None if bias is None else _c(bias, dt)), _p(out),
        _p(z), _p(codes), _p(scores),
        _i64(B), _i64(H), _i64(D), _i64(R), _i64(J), _i64(bs), _i64(T), _i64(k), _i64(Do))
    if return_parts:
        return out, z, codes, scores
    return out


def bf16_round(x):
    """float32 -> bfloat16 bit patterns (round to nearest even), as uint16."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    rounded = u + (0x7FFF + ((u >> 16) & 1))
    return (rounded >> 16).astype(np.uint16)


def bf16_widen(bits):
    return (np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def load_ref(name):
    """Load oracle/_ref/<name>.so (the reference's own x86 kernel, compiled by
    build_ref.sh) as a Python module, or return None when it was not built."""
    path = os.path.join(_HERE, "_ref", name + ".so")
    if not os.path.exists(path):
        return None
    import torch  # noqa: F401  (the extension links against libtorch)
    spec = importlib.util.spec_from_file_location(name, path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod
