"""torch custom ops (namespace ``lookupffn``) over the C ABI of liblookupffn_hip.so.

Each op checks shapes and dtypes on the host, allocates its outputs with
``torch.empty`` on the inputs' device, and launches on torch's current stream.
Only a GPU ("CUDA" dispatch key, which is HIP on ROCm) implementation is
registered: calling an op with CPU tensors fails in the dispatcher.  Fake
(meta) implementations let the ops be traced.
"""
from __future__ import annotations

from typing import Tuple

import ctypes

import torch

from . import _lib

_L = torch.library.Library("lookupffn", "DEF")


def _is_pow2(v: int) -> bool:
    return v > 0 and (v & (v - 1)) == 0


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def _dev_guard(t: torch.Tensor):
    """Make t's device current for the launch; free when it already is (the usual case)."""
    idx = t.device.index
    if idx is None or idx == torch.cuda.current_device():
        return _NO_GUARD
    return torch.cuda.device(t.device)


def _sum_partials(parts_a: torch.Tensor, parts_b: torch.Tensor = None):
    """Column sums of one or two [P, n] arrays of per-workgroup partial sums in one launch, fixed
    order of additions (the backward kernels' weight and bias gradients)."""
    P, na = parts_a.shape
    nb = 0 if parts_b is None else parts_b.shape[1]
    assert parts_a.is_contiguous() and (parts_b is None or (parts_b.is_contiguous() and parts_b.shape[0] == P))
    if P > COLUMN_SUM_CHUNK_ROWS * 4:
        # many rows (a gradient over all tokens): a first pass over chunks of rows on many workgroups
        chunks = (P + COLUMN_SUM_CHUNK_ROWS - 1) // COLUMN_SUM_CHUNK_ROWS
        chunks = (P + ((P + chunks - 1) // chunks) - 1) // ((P + chunks - 1) // chunks)     # no empty chunk
        mid_a = torch.empty(chunks, na, dtype=torch.float32, device=parts_a.device)
        mid_b = None if parts_b is None else torch.empty(chunks, nb, dtype=torch.float32, device=parts_a.device)
        with _dev_guard(parts_a):
            rc = _lib.load().lffn_sum_partials_f32(_lib.ptr(parts_a), _lib.ptr(mid_a), na, _lib.ptr(parts_b),
                                                   _lib.ptr(mid_b), nb, P, chunks, _lib.stream_of(parts_a))
        _lib.check(rc, f"lffn_sum_partials_f32(P={P}, n_a={na}, n_b={nb}, chunks={chunks})")
        parts_a, parts_b, P = mid_a, mid_b, chunks
    out_a = torch.empty(na, dtype=torch.float32, device=parts_a.device)
    out_b = None if parts_b is None else torch.empty(nb, dtype=torch.float32, device=parts_a.device)
    with _dev_guard(parts_a):
        rc = _lib.load().lffn_sum_partials_f32(_lib.ptr(parts_a), _lib.ptr(out_a), na, _lib.ptr(parts_b),
                                               _lib.ptr(out_b), nb, P, 1, _lib.stream_of(parts_a))
    _lib.check(rc, f"lffn_sum_partials_f32(P={P}, n_a={na}, n_b={nb})")
    return out_a, out_b


COLUMN_SUM_CHUNK_ROWS = 256


def column_sums(g: torch.Tensor) -> torch.Tensor:
    """g.sum(0) of a contiguous fp32 [B, n] array on the GPU with n % 4 == 0 (a bias gradient over all
    tokens), reproducible; other inputs go to torch."""
    if (g.is_cuda and g.dim() == 2 and g.dtype == torch.float32 and g.is_contiguous() and g.shape[1] % 4 == 0
            and 1 <= g.shape[0] <= 65535 * COLUMN_SUM_CHUNK_ROWS and g.data_ptr() % 16 == 0
            and not torch.compiler.is_compiling()):
        return _sum_partials(g)[0]
    return g.sum(dim=0)


# ----------------------------------------------------------------------------- fht

_L.define("fht(Tensor x) -> Tensor")


def _fht_impl(x: torch.Tensor) -> torch.Tensor:
    """float32, float16 or bfloat16 rows; the 16-bit forms compute in fp32 and round once."""
    _lib.require_gpu(x)
    assert x.dim() == 2 and x.is_contiguous()
    assert x.dtype in (torch.float32, torch.float16, torch.bfloat16)
    B, D = x.shape
    out = torch.empty_like(x)
    name = {torch.float32: "lffn_fht_f32", torch.float16: "lffn_fht_f16", torch.bfloat16: "lffn_fht_bf16"}[x.dtype]
    with _dev_guard(x):
        rc = getattr(_lib.load(), name)(_lib.ptr(x), _lib.ptr(out), B, D, _lib.stream_of(x))
    _lib.check(rc, f"{name}(B={B}, D={D})")
    return out


_L.impl("fht", _fht_impl, "CUDA")


@torch.library.register_fake("lookupffn::fht")
def _(x):
    return torch.empty_like(x)


# ----------------------------------------------------------------------------- bh4_diag

_L.define("bh4_diag(Tensor x, Tensor diag) -> Tensor")


def _bh4_diag_impl(x: torch.Tensor, diag: torch.Tensor) -> torch.Tensor:
    _lib.require_gpu(x, diag)
    assert x.dim() == 2 and diag.dim() == 3
    assert x.dtype == torch.float32 and diag.dtype == torch.float32
    assert x.is_contiguous() and diag.is_contiguous()
    B, H = x.shape
    R, J, D = diag.shape
    assert H <= D
    out = torch.empty(B, R * D, dtype=torch.float32, device=x.device)
    with _dev_guard(x):
        rc = _lib.load().lffn_bh4_diag_f32(_lib.ptr(x), _lib.ptr(diag), _lib.ptr(out), B, H, D, R, J,
                                           _lib.stream_of(x))
    _lib.check(rc, f"lffn_bh4_diag_f32(B={B}, H={H}, D={D}, R={R}, J={J})")
    return out


_L.impl("bh4_diag", _bh4_diag_impl, "CUDA")


@torch.library.register_fake("lookupffn::bh4_diag")
def _(x, diag):
    return x.new_empty(x.shape[0], diag.shape[0] * diag.shape[2])


# ----------------------------------------------------------------------------- bh4_block

_L.define("bh4_fold(Tensor w) -> Tensor")


def _bh4_fold_impl(w: torch.Tensor) -> torch.Tensor:
    _lib.require_gpu(w)
    assert w.dim() == 5 and w.dtype == torch.float32 and w.is_contiguous()
    R, J, NB, bs, bs2 = w.shape
    assert bs == bs2
    out = torch.empty_like(w)
    with _dev_guard(w):
        rc = _lib.load().lffn_bh4_fold_f32(_lib.ptr(w), _lib.ptr(out), R, J, NB, bs, _lib.stream_of(w))
    _lib.check(rc, f"lffn_bh4_fold_f32(R={R}, J={J}, num_block={NB}, block_size={bs})")
    return out


_L.impl("bh4_fold", _bh4_fold_impl, "CUDA")


@torch.library.register_fake("lookupffn::bh4_fold")
def _(w):
    return torch.empty_like(w)


_L.define("bh4_block(Tensor x, Tensor w_folded) -> Tensor")


def _bh4_block_impl(x: torch.Tensor, w_folded: torch.Tensor) -> torch.Tensor:
    _lib.require_gpu(x, w_folded)
    assert x.dim() == 2 and w_folded.dim() == 5
    assert x.dtype == torch.float32 and w_folded.dtype == torch.float32
    assert x.is_contiguous() and w_folded.is_contiguous()
    B, H = x.shape
    R, J, NB, bs, _ = w_folded.shape
    D = NB * bs
    assert H <= D
    out = torch.empty(B, R * D, dtype=torch.float32, device=x.device)
    with _dev_guard(x):
        rc = _lib.load().lffn_bh4_block_f32(_lib.ptr(x), _lib.ptr(w_folded), _lib.ptr(out), B, H, D, R, J, bs,
                                            _lib.stream_of(x))
    _lib.check(rc, f"lffn_bh4_block_f32(B={B}, H={H}, D={D}, R={R}, J={J}, block_size={bs})")
    return out


_L.impl("bh4_block", _bh4_block_impl, "CUDA")


@torch.library.register_fake("lookupffn::bh4_block")
def _(x, w_folded):
    return x.new_empty(x.shape[0], w_folded.shape[0] * w_folded.shape[2] * w_folded.shape[3])


# ----------------------------------------------------------------------------- ln_bh4_block_hash

_L.define("ln_bh4_block_hash(Tensor x, Tensor? ln_weight, Tensor? ln_bias, float ln_eps, Tensor w_folded, "
          "Tensor? bias, int T, float decay, float residual) -> (Tensor, Tensor)")


def _ln_bh4_block_hash_impl(x, ln_weight, ln_bias, ln_eps, w_folded, bias, T, decay, residual):
    _lib.require_gpu(x, ln_weight, ln_bias, w_folded, bias)
    assert x.dim() == 2 and w_folded.dim() == 5
    assert x.dtype == torch.float32 and w_folded.dtype == torch.float32
    assert x.is_contiguous() and w_folded.is_contiguous()
    B, H = x.shape
    R, J, NB, bs, _ = w_folded.shape
    D = NB * bs
    assert H <= D and T * 8 <= R * D
    for t in (ln_weight, ln_bias):
        if t is not None:
            assert t.dtype == torch.float32 and t.is_contiguous() and t.numel() == H
    assert (ln_weight is None) == (ln_bias is None)
    if bias is not None:
        assert bias.dtype == torch.float32 and bias.is_contiguous() and bias.numel() == T * 8
    codes = torch.empty(B, T, dtype=torch.int32, device=x.device)
    scores = torch.empty(B, T, dtype=torch.float32, device=x.device)
    with _dev_guard(x):
        rc = _lib.load().lffn_ln_bh4_block_hash_f32(
            _lib.ptr(x), _lib.ptr(ln_weight), _lib.ptr(ln_bias), ln_eps, _lib.ptr(w_folded), _lib.ptr(bias),
            _lib.ptr(codes), _lib.ptr(scores), B, H, D, R, J, T, bs, decay, residual, _lib.stream_of(x))
    _lib.check(rc, f"lffn_ln_bh4_block_hash_f32(B={B}, H={H}, D={D}, R={R}, J={J}, T={T}, block_size={bs})")
    return codes, scores


_L.impl("ln_bh4_block_hash", _ln_bh4_block_hash_impl, "CUDA")


@torch.library.register_fake("lookupffn::ln_bh4_block_hash")
def _(x, ln_weight, ln_bias, ln_eps, w_folded, bias, T, decay, residual):
    return (torch.empty(x.shape[0], T, dtype=torch.int32, device=x.device),
            torch.empty(x.shape[0], T, dtype=torch.float32, device=x.device))


# ----------------------------------------------------------------------------- bh4_block training

_L.define("bh4_fold_mode(Tensor w, int mode) -> Tensor")


def _bh4_fold_mode_impl(w: torch.Tensor, mode: int) -> torch.Tensor:
    """w: [..., 64, 64] blocks.  mode 0 / 1: the forward / backward kernels' fetch order,
    mode 2: natural order (gradient w.r.t. folded weights -> gradient w.r.t. weights)."""
    _lib.require_gpu(w)
    assert w.dim() >= 2 and w.shape[-1] == w.shape[-2] and w.dtype == torch.float32 and w.is_contiguous()
    bs = w.shape[-1]
    nblk = w.numel() // (bs * bs)
    out = torch.empty_like(w)
    with _dev_guard(w):
        rc = _lib.load().lffn_bh4_fold_mode_f32(_lib.ptr(w), _lib.ptr(out), nblk, bs, mode, _lib.stream_of(w))
    _lib.check(rc, f"lffn_bh4_fold_mode_f32(num_blocks={nblk}, block_size={bs}, mode={mode})")
    return out


_L.impl("bh4_fold_mode", _bh4_fold_mode_impl, "CUDA")


@torch.library.register_fake("lookupffn::bh4_fold_mode")
def _(w, mode):
    return torch.empty_like(w)


_L.define("bh4_block_hash_train(Tensor x, Tensor w_folded, Tensor? bias, int T, float decay, float residual)"
          " -> (Tensor, Tensor, Tensor, Tensor)")


def _bh4_block_hash_train_impl(x, w_folded, bias, T, decay, residual):
    """-> (codes [B,T], scores [B,T], z [B,T*8], stage_inputs [R,J-1,B,D])."""
    _lib.require_gpu(x, w_folded, bias)
    assert x.dim() == 2 and w_folded.dim() == 5
    assert x.dtype == torch.float32 and w_folded.dtype == torch.float32
    assert x.is_contiguous() and w_folded.is_contiguous()
    B, H = x.shape
    R, J, NB, bs, _ = w_folded.shape
    D = NB * bs
    assert H <= D and T * 8 <= R * D
    if bias is not None:
        assert bias.dtype == torch.float32 and bias.is_contiguous() and bias.numel() == T * 8
    codes = torch.empty(B, T, dtype=torch.int32, device=x.device)
    scores = torch.empty(B, T, dtype=torch.float32, device=x.device)
    z = torch.empty(B, T * 8, dtype=torch.float32, device=x.device)
    stage_in = torch.empty(R, max(J - 1, 0), B, D, dtype=torch.float32, device=x.device)
    with _dev_guard(x):
        rc = _lib.load().lffn_bh4_block_hash_train_f32(
            _lib.ptr(x), _lib.ptr(w_folded), _lib.ptr(bias), _lib.ptr(codes), _lib.ptr(scores), _lib.ptr(z),
            _lib.ptr(stage_in) if J > 1 else None, B, H, D, R, J, T, bs, decay, residual, _lib.stream_of(x))
    _lib.check(rc, f"lffn_bh4_block_hash_train_f32(B={B}, H={H}, D={D}, R={R}, J={J}, T={T})")
    return codes, scores, z, stage_in


_L.impl("bh4_block_hash_train", _bh4_block_hash_train_impl, "CUDA")


@torch.library.register_fake("lookupffn::bh4_block_hash_train")
def _(x, w_folded, bias, T, decay, residual):
    B = x.shape[0]
    R, J, NB, bs, _ = w_folded.shape
    return (torch.empty(B, T, dtype=torch.int32, device=x.device), x.new_empty(B, T), x.new_empty(B, T * 8),
            x.new_empty(R, max(J - 1, 0), B, NB * bs))


_L.define("ln_bh4_block_hash_train(Tensor x, Tensor ln_w, Tensor ln_b, float eps, Tensor w_folded, Tensor? bias, int T, "
          "float decay, float residual) -> (Tensor, Tensor, Tensor, Tensor, Tensor)")


def _ln_bh4_block_hash_train_impl(x, ln_w, ln_b, eps, w_folded, bias, T, decay, residual):
    """LayerNorm inside the kernel -> (codes [B,T], scores [B,T], z [B,T*8], stage_inputs [R,J-1,B,D],
    row_stats [B,2] = every row's mean and 1/sigma)."""
    _lib.require_gpu(x, ln_w, ln_b, w_folded, bias)
    assert x.dim() == 2 and w_folded.dim() == 5
    for t in (x, ln_w, ln_b, w_folded):
        assert t.dtype == torch.float32 and t.is_contiguous()
    B, H = x.shape
    R, J, NB, bs, _ = w_folded.shape
    D = NB * bs
    assert H <= D and T * 8 <= R * D and ln_w.numel() == H and ln_b.numel() == H
    if bias is not None:
        assert bias.dtype == torch.float32 and bias.is_contiguous() and bias.numel() == T * 8
    codes = torch.empty(B, T, dtype=torch.int32, device=x.device)
    scores = torch.empty(B, T, dtype=torch.float32, device=x.device)
    z = torch.empty(B, T * 8, dtype=torch.float32, device=x.device)
    stage_in = torch.empty(R, max(J - 1, 0), B, D, dtype=torch.float32, device=x.device)
    stats = torch.empty(B, 2, dtype=torch.float32, device=x.device)
    with _dev_guard(x):
        rc = _lib.load().lffn_ln_bh4_block_hash_train_f32(
            _lib.ptr(x), _lib.ptr(ln_w), _lib.ptr(ln_b), eps, _lib.ptr(w_folded), _lib.ptr(bias), _lib.ptr(codes),
            _lib.ptr(scores), _lib.ptr(z), _lib.ptr(stage_in) if J > 1 else None, _lib.ptr(stats), B, H, D, R, J, T, bs,
            decay, residual, _lib.stream_of(x))
    _lib.check(rc, f"lffn_ln_bh4_block_hash_train_f32(B={B}, H={H}, D={D}, R={R}, J={J}, T={T})")
    return codes, scores, z, stage_in, stats


_L.impl("ln_bh4_block_hash_train", _ln_bh4_block_hash_train_impl, "CUDA")


@torch.library.register_fake("lookupffn::ln_bh4_block_hash_train")
def _(x, ln_w, ln_b, eps, w_folded, bias, T, decay, residual):
    B = x.shape[0]
    R, J, NB, bs, _ = w_folded.shape
    return (torch.empty(B, T, dtype=torch.int32, device=x.device), x.new_empty(B, T), x.new_empty(B, T * 8),
            x.new_empty(R, max(J - 1, 0), B, NB * bs), x.new_empty(B, 2))


_L.define("ln_bh4_block_wgrad(Tensor stage_grads, Tensor x, Tensor ln_w, Tensor ln_b, Tensor row_stats, Tensor stage_inputs, "
          "int R, int J) -> Tensor")


def _ln_bh4_block_wgrad_impl(stage_grads, x, ln_w, ln_b, row_stats, stage_inputs, R, J):
    """bh4_block_wgrad with LayerNorm(x) as the input of every repeat's first stage, formed on load."""
    _lib.require_gpu(stage_grads, x, ln_w, ln_b, row_stats, stage_inputs)
    for t in (stage_grads, x, ln_w, ln_b, row_stats, stage_inputs):
        assert t.dtype == torch.float32 and t.is_contiguous()
    S, B, D = stage_grads.shape
    assert S == R * J and x.shape[0] == B and stage_inputs.numel() == R * (J - 1) * B * D
    assert tuple(row_stats.shape) == (B, 2) and ln_w.numel() == x.shape[1] and ln_b.numel() == x.shape[1]
    g = torch.zeros(S, D // 64, 64, 64, dtype=torch.float32, device=x.device)
    with _dev_guard(x):
        rc = _lib.load().lffn_ln_bh4_block_wgrad_f32(_lib.ptr(stage_grads), _lib.ptr(x), _lib.ptr(ln_w), _lib.ptr(ln_b),
                                                     _lib.ptr(row_stats), _lib.ptr(stage_inputs), _lib.ptr(g), B, x.shape[1],
                                                     D, R, J, 64, _lib.stream_of(x))
    _lib.check(rc, f"lffn_ln_bh4_block_wgrad_f32(B={B}, H={x.shape[1]}, D={D}, R={R}, J={J})")
    return g


_L.impl("ln_bh4_block_wgrad", _ln_bh4_block_wgrad_impl, "CUDA")


@torch.library.register_fake("lookupffn::ln_bh4_block_wgrad")
def _(stage_grads, x, ln_w, ln_b, row_stats, stage_inputs, R, J):
    S, B, D = stage_grads.shape
    return x.new_empty(S, D // 64, 64, 64)


_L.define("bh4_block_bwd(Tensor g_z, Tensor w_folded_t, int H, float decay, float residual) -> (Tensor, Tensor)")


def _bh4_block_bwd_impl(g_z, w_folded_t, H, decay, residual):
    """-> (g_x [R,B,H], stage_grads [R,J,B,D])."""
    _lib.require_gpu(g_z, w_folded_t)
    assert g_z.dim() == 2 and g_z.dtype == torch.float32 and g_z.is_contiguous() and g_z.shape[1] % 8 == 0
    assert w_folded_t.dim() == 5 and w_folded_t.dtype == torch.float32 and w_folded_t.is_contiguous()
    B = g_z.shape[0]
    T = g_z.shape[1] // 8
    R, J, NB, bs, _ = w_folded_t.shape
    D = NB * bs
    g_x = torch.empty(R, B, H, dtype=torch.float32, device=g_z.device)
    stage_g = torch.empty(R, J, B, D, dtype=torch.float32, device=g_z.device)
    with _dev_guard(g_z):
        rc = _lib.load().lffn_bh4_block_bwd_f32(_lib.ptr(g_z), _lib.ptr(w_folded_t), _lib.ptr(g_x), _lib.ptr(stage_g),
                                                B, H, D, R, J, T, bs, decay, residual, _lib.stream_of(g_z))
    _lib.check(rc, f"lffn_bh4_block_bwd_f32(B={B}, H={H}, D={D}, R={R}, J={J}, T={T})")
    return g_x, stage_g


_L.impl("bh4_block_bwd", _bh4_block_bwd_impl, "CUDA")


@torch.library.register_fake("lookupffn::bh4_block_bwd")
def _(g_z, w_folded_t, H, decay, residual):
    R, J, NB, bs, _ = w_folded_t.shape
    return g_z.new_empty(R, g_z.shape[0], H), g_z.new_empty(R, J, g_z.shape[0], NB * bs)


_L.define("bh4_block_wgrad(Tensor stage_grads, Tensor x, Tensor stage_inputs, int R, int J) -> Tensor")


def _bh4_block_wgrad_impl(stage_grads, x, stage_inputs, R, J):
    """[R*J, D/64, 64, 64]: per stage and block, the sum over the tokens of (stage gradient)^T (stage input),
    in the folded basis.  stage_grads [R*J, B, D]; x [B, H]; stage_inputs [R, J-1, B, D]."""
    _lib.require_gpu(stage_grads, x, stage_inputs)
    for t in (stage_grads, x, stage_inputs):
        assert t.dtype == torch.float32 and t.is_contiguous()
    S, B, D = stage_grads.shape
    assert S == R * J and x.shape[0] == B and stage_inputs.numel() == R * (J - 1) * B * D
    g = torch.zeros(S, D // 64, 64, 64, dtype=torch.float32, device=x.device)
    with _dev_guard(x):
        rc = _lib.load().lffn_bh4_block_wgrad_f32(_lib.ptr(stage_grads), _lib.ptr(x), _lib.ptr(stage_inputs), _lib.ptr(g), B,
                                                  x.shape[1], D, R, J, 64, _lib.stream_of(x))
    _lib.check(rc, f"lffn_bh4_block_wgrad_f32(B={B}, H={x.shape[1]}, D={D}, R={R}, J={J})")
    return g


_L.impl("bh4_block_wgrad", _bh4_block_wgrad_impl, "CUDA")


@torch.library.register_fake("lookupffn::bh4_block_wgrad")
def _(stage_grads, x, stage_inputs, R, J):
    S, B, D = stage_grads.shape
    return x.new_empty(S, D // 64, 64, 64)


_L.define("lookup_ffn_fused(Tensor x, Tensor ln_w, Tensor ln_b, float eps, Tensor diag, Tensor? pbias, Tensor tables, "
          "Tensor? obias, Tensor? residual, float decay, float residual_coef) -> Tensor")


def _lookup_ffn_fused_impl(x, ln_w, ln_b, eps, diag, pbias, tables, obias, residual, decay, residual_coef):
    """The whole layer in one launch (PL/lookup.py:99-108): LayerNorm, diagonal BH4, mix, bias, 8-bit
    code + score, gather-add of the T rows, output bias, optional residual [B, Do]."""
    _lib.require_gpu(x, ln_w, ln_b, diag, tables)
    B, H = x.shape
    R, J, D = diag.shape
    T, S, Do = tables.shape
    for t in (x, ln_w, ln_b, diag, tables, pbias, obias, residual):
        assert t is None or (t.dtype == torch.float32 and t.is_contiguous())
    assert ln_w.numel() == H and ln_b.numel() == H
    assert pbias is None or pbias.numel() == T * 8
    assert obias is None or obias.numel() == Do
    assert residual is None or tuple(residual.shape) == (B, Do)
    out = torch.empty(B, Do, dtype=torch.float32, device=x.device)
    with _dev_guard(x):
        rc = _lib.load().lffn_lookup_ffn_fused_f32(
            _lib.ptr(x), _lib.ptr(ln_w), _lib.ptr(ln_b), eps, _lib.ptr(diag), _lib.ptr(pbias), _lib.ptr(tables),
            _lib.ptr(obias), _lib.ptr(residual), _lib.ptr(out), B, H, D, R, J, T, S, Do, decay, residual_coef,
            _lib.stream_of(x))
    _lib.check(rc, f"lffn_lookup_ffn_fused_f32(B={B}, H={H}, D={D}, R={R}, J={J}, T={T}, S={S}, Do={Do})")
    return out


_L.impl("lookup_ffn_fused", _lookup_ffn_fused_impl, "CUDA")


# The inference path of the layer calls the implementations below directly: outside torch.compile
# the dispatcher adds nothing but a few microseconds per call, which is the larger part of a step
# at small batches.
def ln_project_hash_direct(*args):
    return _ln_project_hash_impl(*args)


def ln_bh4_block_hash_direct(*args):
    return _ln_bh4_block_hash_impl(*args)


def lookup_gather_direct(*args):
    return _lookup_gather_impl(*args)


def lookup_ffn_fused_direct(x, ln_w, ln_b, eps, diag, pbias, tables, obias, residual, decay, residual_coef):
    """lookup_ffn_fused for a caller that has already checked the parameters (LookupFFN caches that):
    no dispatcher, no per-call checks beyond x itself.  The layer's launch is a few microseconds, so
    at small batches the host side of a call is most of its time."""
    if torch.compiler.is_compiling():
        return torch.ops.lookupffn.lookup_ffn_fused(x, ln_w, ln_b, eps, diag, pbias, tables, obias, residual,
                                                    decay, residual_coef)
    assert x.dtype == torch.float32 and x.is_cuda and x.is_contiguous() and x.device == tables.device
    B, H = x.shape
    R, J, D = diag.shape
    T, S, Do = tables.shape
    assert H == ln_w.numel() and (residual is None or (residual.dtype == torch.float32 and residual.is_contiguous()
                                                        and tuple(residual.shape) == (B, Do)))
    out = torch.empty((B, Do), dtype=torch.float32, device=x.device)
    with _dev_guard(x):
        rc = _lib.load().lffn_lookup_ffn_fused_f32(
            x.data_ptr(), ln_w.data_ptr(), ln_b.data_ptr(), eps, diag.data_ptr(),
            None if pbias is None else pbias.data_ptr(), tables.data_ptr(),
            None if obias is None else obias.data_ptr(), None if residual is None else residual.data_ptr(),
            out.data_ptr(), B, H, D, R, J, T, S, Do, decay, residual_coef, _lib.stream_of(x))
    if rc != 0:
        _lib.check(rc, f"lffn_lookup_ffn_fused_f32(B={B}, H={H}, D={D}, R={R}, J={J}, T={T}, S={S}, Do={Do})")
    return out


def fused_layer_block(ln_w, ln_b, eps, diag, pbias, tables, obias, decay, residual_coef):
    """The parameter block of lffn_lookup_ffn_fused_layer_f32 for a set of (checked, contiguous, fp32, same-device)
    parameters, with the entry point and a byref to the block: what lookup_ffn_fused_block takes.  The tensors
    must outlive the block (LookupFFN keeps both in one cache entry)."""
    R, J, D = diag.shape
    T, S, Do = tables.shape
    blk = _lib.FusedLayer(ln_w.data_ptr(), ln_b.data_ptr(), diag.data_ptr(), None if pbias is None else pbias.data_ptr(),
                          tables.data_ptr(), None if obias is None else obias.data_ptr(), ln_w.numel(), D, R, J, T, S, Do,
                          eps, decay, residual_coef)
    return (_lib.load().lffn_lookup_ffn_fused_layer_f32, ctypes.byref(blk), blk, ln_w.numel(), Do, tables.device)


def lookup_ffn_fused_block(block, x, residual):
    """lookup_ffn_fused_direct through the parameter block: six arguments cross the foreign-function interface
    instead of twenty-one."""
    fn, ref, _keep, H, Do, device = block
    if x.dtype != torch.float32 or x.dim() != 2 or x.shape[1] != H or x.device != device or not x.is_contiguous():
        raise ValueError("x: contiguous fp32 [B, H] on the parameters' device")
    B = x.shape[0]
    out = torch.empty((B, Do), dtype=torch.float32, device=device)
    with _dev_guard(x):
        rc = fn(ref, x.data_ptr(), None if residual is None else residual.data_ptr(), out.data_ptr(), B, _lib.stream_of(x))
    if rc != 0:
        _lib.check(rc, f"lffn_lookup_ffn_fused_layer_f32(B={B}, H={H}, Do={Do})")
    return out


@torch.library.register_fake("lookupffn::lookup_ffn_fused")
def _(x, ln_w, ln_b, eps, diag, pbias, tables, obias, residual, decay, residual_coef):
    return x.new_empty(x.shape[0], tables.shape[2])


LN_BWD_PARTIALS = 512

_L.define("layer_norm_bwd(Tensor x, Tensor? weight, float eps, Tensor g_y) -> (Tensor, Tensor, Tensor)")


def _layer_norm_bwd_impl(x, weight, eps, g_y):
    """Backward of LayerNorm over the last dimension of x [B, H]; g_y is [R, B, H] (the R gradients are
    added up).  -> (g_x [B, H], g_weight [H], g_bias [H])."""
    _lib.require_gpu(x, g_y)
    B, H = x.shape
    assert g_y.dim() == 3 and tuple(g_y.shape[1:]) == (B, H)
    for t in (x, weight, g_y):
        assert t is None or (t.dtype == torch.float32 and t.is_contiguous())
    R = g_y.shape[0]
    n = max(1, min(LN_BWD_PARTIALS, (B + 3) // 4))
    g_x = torch.empty_like(x)
    part = torch.empty(2, n, H, dtype=torch.float32, device=x.device)
    with _dev_guard(x):
        rc = _lib.load().lffn_layer_norm_bwd_f32(_lib.ptr(x), _lib.ptr(weight), eps, _lib.ptr(g_y), _lib.ptr(g_x),
                                                 _lib.ptr(part[0]), _lib.ptr(part[1]), B, H, R, n, _lib.stream_of(x))
    _lib.check(rc, f"lffn_layer_norm_bwd_f32(B={B}, H={H}, R={R})")
    g_w, g_b = _sum_partials(part[0], part[1])
    return g_x, g_w, g_b


_L.impl("layer_norm_bwd", _layer_norm_bwd_impl, "CUDA")


@torch.library.register_fake("lookupffn::layer_norm_bwd")
def _(x, weight, eps, g_y):
    return torch.empty_like(x), x.new_empty(x.shape[1]), x.new_empty(x.shape[1])


# ----------------------------------------------------------------------------- mix_code_score

_L.define("mix_code_score(Tensor y, Tensor x, Tensor? bias, int T, int k, int D, float decay, float residual)"
          " -> (Tensor, Tensor)")


def _mix_code_score_impl(y, x, bias, T, k, D, decay, residual):
    _lib.require_gpu(y, x, bias)
    assert y.dim() == 2 and x.dim() == 2 and y.shape[0] == x.shape[0]
    assert y.dtype == torch.float32 and x.dtype == torch.float32
    assert y.is_contiguous() and x.is_contiguous()
    B, ldy = y.shape
    H = x.shape[1]
    assert H <= D and T * k <= ldy
    if bias is not None:
        assert bias.dtype == torch.float32 and bias.is_contiguous() and bias.numel() == T * k
    codes = torch.empty(B, T, dtype=torch.int32, device=y.device)
    scores = torch.empty(B, T, dtype=torch.float32, device=y.device)
    with _dev_guard(y):
        rc = _lib.load().lffn_mix_code_score_f32(_lib.ptr(y), _lib.ptr(x), _lib.ptr(bias), _lib.ptr(codes),
                                                 _lib.ptr(scores), B, T, k, H, D, ldy, decay, residual,
                                                 _lib.stream_of(y))
    _lib.check(rc, f"lffn_mix_code_score_f32(B={B}, T={T}, k={k}, H={H}, D={D}, ldy={ldy})")
    return codes, scores


_L.impl("mix_code_score", _mix_code_score_impl, "CUDA")


@torch.library.register_fake("lookupffn::mix_code_score")
def _(y, x, bias, T, k, D, decay, residual):
    return (torch.empty(y.shape[0], T, dtype=torch.int32, device=y.device),
            torch.empty(y.shape[0], T, dtype=torch.float32, device=y.device))


# ----------------------------------------------------------------------------- project_hash

_L.define("project_hash(Tensor x, Tensor diag, Tensor? bias, int T, float decay, float residual, bool keep_z)"
          " -> (Tensor, Tensor, Tensor)")


def _project_hash_impl(x, diag, bias, T, decay, residual, keep_z):
    _lib.require_gpu(x, diag, bias)
    assert x.dim() == 2 and diag.dim() == 3
    assert x.dtype == torch.float32 and diag.dtype == torch.float32
    assert x.is_contiguous() and diag.is_contiguous()
    B, H = x.shape
    R, J, D = diag.shape
    assert H <= D and T * 8 <= R * D
    if bias is not None:
        assert bias.dtype == torch.float32 and bias.is_contiguous() and bias.numel() == T * 8
    codes = torch.empty(B, T, dtype=torch.int32, device=x.device)
    scores = torch.empty(B, T, dtype=torch.float32, device=x.device)
    z = torch.empty((B, T * 8) if keep_z else (0,), dtype=torch.float32, device=x.device)
    with _dev_guard(x):
        rc = _lib.load().lffn_project_hash_f32(
            _lib.ptr(x), _lib.ptr(diag), _lib.ptr(bias), _lib.ptr(z) if keep_z else None,
            _lib.ptr(codes), _lib.ptr(scores), B, H, D, R, J, T, decay, residual, _lib.stream_of(x))
    _lib.check(rc, f"lffn_project_hash_f32(B={B}, H={H}, D={D}, R={R}, J={J}, T={T})")
    return codes, scores, z


_L.impl("project_hash", _project_hash_impl, "CUDA")


@torch.library.register_fake("lookupffn::project_hash")
def _(x, diag, bias, T, decay, residual, keep_z):
    B = x.shape[0]
    return (x.new_empty(B, T, dtype=torch.int32), x.new_empty(B, T),
            x.new_empty((B, T * 8) if keep_z else (0,)))


_L.define("project_hash_bwd(Tensor x, Tensor diag, Tensor z, Tensor g_score, float decay, float residual, "
          "Tensor? ln_weight=None, Tensor? ln_bias=None, float ln_eps=0.0) -> (Tensor, Tensor, Tensor)")

PROJECT_BWD_PARTIALS = 512      # workgroups per repeat: two per compute unit


def _project_hash_bwd_impl(x, diag, z, g_score, decay, residual, ln_weight=None, ln_bias=None, ln_eps=0.0):
    """-> (grad x [B,H], grad diag [R,J,D], grad bias [T*8]).  With ln_weight / ln_bias the projection's
    input is LayerNorm(x), formed on load, and the first result is [R,B,H]: the gradient w.r.t. that
    LayerNorm output, one slab per repeat (layer_norm_bwd adds them)."""
    _lib.require_gpu(x, diag, z, g_score, ln_weight, ln_bias)
    for t in (x, diag, z, g_score, ln_weight, ln_bias):
        assert t is None or (t.dtype == torch.float32 and t.is_contiguous())
    assert (ln_weight is None) == (ln_bias is None)
    B, H = x.shape
    R, J, D = diag.shape
    T = g_score.shape[1]
    assert tuple(z.shape) == (B, T * 8) and g_score.shape[0] == B
    nparts = max(1, min(PROJECT_BWD_PARTIALS, (B + 3) // 4))
    g_x = torch.empty(R, B, H, dtype=torch.float32, device=x.device)
    part_d = torch.empty(nparts, R, J, D, dtype=torch.float32, device=x.device)
    part_b = torch.empty(nparts, R * D, dtype=torch.float32, device=x.device)
    if B > 0 and ln_weight is not None:
        assert ln_weight.numel() == H and ln_bias.numel() == H
        with _dev_guard(x):
            rc = _lib.load().lffn_ln_project_hash_bwd_f32(
                _lib.ptr(x), _lib.ptr(ln_weight), _lib.ptr(ln_bias), ln_eps, _lib.ptr(diag), _lib.ptr(z),
                _lib.ptr(g_score), _lib.ptr(g_x), _lib.ptr(part_d), _lib.ptr(part_b), B, H, D, R, J, T, nparts,
                decay, residual, _lib.stream_of(x))
        _lib.check(rc, f"lffn_ln_project_hash_bwd_f32(B={B}, H={H}, D={D}, R={R}, J={J}, T={T})")
    elif B > 0:
        with _dev_guard(x):
            rc = _lib.load().lffn_project_hash_bwd_f32(
                _lib.ptr(x), _lib.ptr(diag), _lib.ptr(z), _lib.ptr(g_score), _lib.ptr(g_x), _lib.ptr(part_d),
                _lib.ptr(part_b), B, H, D, R, J, T, nparts, decay, residual, _lib.stream_of(x))
        _lib.check(rc, f"lffn_project_hash_bwd_f32(B={B}, H={H}, D={D}, R={R}, J={J}, T={T})")
    else:
        part_d.zero_(); part_b.zero_()
    g_d, g_b = _sum_partials(part_d.view(nparts, R * J * D), part_b)
    if ln_weight is not None:
        return g_x, g_d.view(R, J, D), g_b[:T * 8]
    return (g_x[0] if R == 1 else g_x.sum(0)), g_d.view(R, J, D), g_b[:T * 8]


_L.impl("project_hash_bwd", _project_hash_bwd_impl, "CUDA")


@torch.library.register_fake("lookupffn::project_hash_bwd")
def _(x, diag, z, g_score, decay, residual, ln_weight=None, ln_bias=None, ln_eps=0.0):
    g_x = torch.empty_like(x) if ln_weight is None else x.new_empty((diag.shape[0],) + tuple(x.shape))
    return g_x, torch.empty_like(diag), x.new_empty(z.shape[1])


_L.define("ln_project_hash(Tensor x, Tensor ln_weight, Tensor ln_bias, float eps, Tensor diag, Tensor? bias, "
          "int T, float decay, float residual, bool keep_z) -> (Tensor, Tensor, Tensor)")


def _ln_project_hash_impl(x, ln_weight, ln_bias, eps, diag, bias, T, decay, residual, keep_z):
    _lib.require_gpu(x, ln_weight, ln_bias, diag, bias)
    assert x.dim() == 2 and diag.dim() == 3
    assert x.dtype == torch.float32 and diag.dtype == torch.float32
    assert ln_weight.dtype == torch.float32 and ln_bias.dtype == torch.float32
    assert x.is_contiguous() and diag.is_contiguous() and ln_weight.is_contiguous() and ln_bias.is_contiguous()
    B, H = x.shape
    R, J, D = diag.shape
    assert H <= D and T * 8 <= R * D and ln_weight.numel() == H and ln_bias.numel() == H
    if bias is not None:
        assert bias.dtype == torch.float32 and bias.is_contiguous() and bias.numel() == T * 8
    codes = torch.empty(B, T, dtype=torch.int32, device=x.device)
    scores = torch.empty(B, T, dtype=torch.float32, device=x.device)
    z = torch.empty((B, T * 8) if keep_z else (0,), dtype=torch.float32, device=x.device)
    with _dev_guard(x):
        rc = _lib.load().lffn_ln_project_hash_f32(
            _lib.ptr(x), _lib.ptr(ln_weight), _lib.ptr(ln_bias), eps, _lib.ptr(diag), _lib.ptr(bias),
            _lib.ptr(z) if keep_z else None, _lib.ptr(codes), _lib.ptr(scores),
            B, H, D, R, J, T, decay, residual, _lib.stream_of(x))
    _lib.check(rc, f"lffn_ln_project_hash_f32(B={B}, H={H}, D={D}, R={R}, J={J}, T={T})")
    return codes, scores, z


_L.impl("ln_project_hash", _ln_project_hash_impl, "CUDA")


@torch.library.register_fake("lookupffn::ln_project_hash")
def _(x, ln_weight, ln_bias, eps, diag, bias, T, decay, residual, keep_z):
    B = x.shape[0]
    return (x.new_empty(B, T, dtype=torch.int32), x.new_empty(B, T),
            x.new_empty((B, T * 8) if keep_z else (0,)))


# ----------------------------------------------------------------------------- code_score

_L.define("code_score(Tensor z) -> (Tensor, Tensor)")


def _code_score_impl(z: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    _lib.require_gpu(z)
    assert z.dim() >= 1 and z.dtype == torch.float32 and z.is_contiguous()
    k = z.shape[-1]
    N = z.numel() // max(k, 1)
    codes = torch.empty(z.shape[:-1], dtype=torch.int32, device=z.device)
    scores = torch.empty(z.shape[:-1], dtype=torch.float32, device=z.device)
    with _dev_guard(z):
        rc = _lib.load().lffn_code_score_f32(_lib.ptr(z), _lib.ptr(codes), _lib.ptr(scores), N, k,
                                             _lib.stream_of(z))
    _lib.check(rc, f"lffn_code_score_f32(N={N}, k={k})")
    return codes, scores


_L.impl("code_score", _code_score_impl, "CUDA")


@torch.library.register_fake("lookupffn::code_score")
def _(z):
    return z.new_empty(z.shape[:-1], dtype=torch.int32), z.new_empty(z.shape[:-1])


_L.define("code_score_bwd(Tensor z, Tensor g_score) -> Tensor")


def _code_score_bwd_impl(z: torch.Tensor, g_score: torch.Tensor) -> torch.Tensor:
    _lib.require_gpu(z, g_score)
    assert z.dtype == torch.float32 and g_score.dtype == torch.float32
    assert z.is_contiguous() and g_score.is_contiguous()
    assert tuple(g_score.shape) == tuple(z.shape[:-1])
    k = z.shape[-1]
    N = z.numel() // max(k, 1)
    g_z = torch.empty_like(z)
    with _dev_guard(z):
        rc = _lib.load().lffn_code_score_bwd_f32(_lib.ptr(z), _lib.ptr(g_score), _lib.ptr(g_z), N, k,
                                                 _lib.stream_of(z))
    _lib.check(rc, f"lffn_code_score_bwd_f32(N={N}, k={k})")
    return g_z


_L.impl("code_score_bwd", _code_score_bwd_impl, "CUDA")


@torch.library.register_fake("lookupffn::code_score_bwd")
def _(z, g_score):
    return torch.empty_like(z)


# ----------------------------------------------------------------------------- gather-add family

def _check_gather_args(indexes, rows, vector_dim):
    assert indexes.dim() == 2 and indexes.dtype == torch.int32 and indexes.is_contiguous()
    assert vector_dim % 64 == 0, vector_dim
    assert rows >= 1


_L.define("gather_add(Tensor indexes, Tensor source, Tensor weights) -> Tensor")


def _gather_add_impl(indexes, source, weights):
    _lib.require_gpu(indexes, source, weights)
    assert source.dim() == 2 and source.is_contiguous()
    assert weights.dtype == torch.float32 and weights.is_contiguous()
    assert tuple(weights.shape) == tuple(indexes.shape)
    B, I = indexes.shape
    S, Dv = source.shape
    _check_gather_args(indexes, S, Dv)
    out = torch.empty(B, Dv, dtype=torch.float32, device=source.device)
    lib = _lib.load()
    if source.dtype == torch.float32:
        fn, name = lib.lffn_gather_add_f32, "lffn_gather_add_f32"
    elif source.dtype == torch.bfloat16:
        fn, name = lib.lffn_gather_add_bf16, "lffn_gather_add_bf16"
    elif source.dtype == torch.float16:
        fn, name = lib.lffn_gather_add_f16, "lffn_gather_add_f16"
    else:
        raise NotImplementedError(f"gather_add: source dtype {source.dtype} (float32, bfloat16 and float16 rows are built)")
    with _dev_guard(source):
        rc = fn(_lib.ptr(indexes), _lib.ptr(source), _lib.ptr(weights), _lib.ptr(out), B, I, S, Dv,
                _lib.stream_of(source))
    _lib.check(rc, f"{name}(B={B}, I={I}, S={S}, Dv={Dv})")
    return out


_L.impl("gather_add", _gather_add_impl, "CUDA")


@torch.library.register_fake("lookupffn::gather_add")
def _(indexes, source, weights):
    return weights.new_empty(indexes.shape[0], source.shape[1])


# The inference path of the layer at many tokens: the projection kernel writes the gather kernel's record
# stream itself (no [B, T] codes and scores, no packing kernel).  Plain functions, no operator: the
# records are a private hand-over between the two kernels.
_RECORDS_PLANS = {}


ROWS_F32, ROWS_BF16, ROWS_F16 = 0, 1, 2      # the C ABI's row_format values


def row_format(dtype):
    """The C ABI's row_format for a table dtype, or None for a dtype no gather kernel is built for."""
    return {torch.float32: ROWS_F32, torch.bfloat16: ROWS_BF16, torch.float16: ROWS_F16}.get(dtype)


def lookup_gather_records_plan(B, T, S, Do, fmt=ROWS_F32):
    """(tokens per workgroup, record stride in tokens, bytes of the stream) when the record-stream form of
    the gather is the one to use for this shape and row format, else None.  Host-side query, cached."""
    key = (B, T, S, Do, fmt)
    hit = _RECORDS_PLANS.get(key, False)
    if hit is not False:
        return hit
    tokens, stride, nbytes = ctypes.c_int32(0), ctypes.c_int64(0), ctypes.c_int64(0)
    _lib.check(_lib.load().lffn_lookup_gather_records_plan_rows(B, T, S, Do, fmt, ctypes.byref(tokens), ctypes.byref(stride),
                                                                ctypes.byref(nbytes)), "lffn_lookup_gather_records_plan_rows")
    plan = (tokens.value, stride.value, nbytes.value) if nbytes.value > 0 else None
    if len(_RECORDS_PLANS) < 4096:
        _RECORDS_PLANS[key] = plan
    return plan


def _require(cond, what):
    """Argument checks of the *_direct helpers (no operator dispatcher in front of them): a real exception,
    also under ``python -O``."""
    if not cond:
        raise ValueError(what)


def ln_project_hash_records_direct(x, ln_w, ln_b, eps, diag, pbias, T, decay, residual, plan):
    """LayerNorm + diagonal BH4 + mix + 8-bit hash of x [B, H], written as the record stream of `plan`
    (from lookup_gather_records_plan) instead of codes and scores.  The caller has checked the parameters
    (fp32, contiguous, on x's device)."""
    _require(x.dtype == torch.float32 and x.is_cuda and x.is_contiguous() and x.dim() == 2, "x: contiguous fp32 [B, H] on the GPU")
    B, H = x.shape
    R, J, D = diag.shape
    _require(H == ln_w.numel() and T * 8 <= R * D and T % 2 == 0 and plan[1] >= B, "shapes do not fit the record plan")
    records = torch.empty(plan[2] // 4, dtype=torch.int32, device=x.device)
    with _dev_guard(x):
        rc = _lib.load().lffn_ln_project_hash_records_f32(
            x.data_ptr(), ln_w.data_ptr(), ln_b.data_ptr(), eps, diag.data_ptr(), None if pbias is None else pbias.data_ptr(),
            records.data_ptr(), plan[1], plan[0], B, H, D, R, J, T, decay, residual, _lib.stream_of(x))
    if rc != 0:
        _lib.check(rc, f"lffn_ln_project_hash_records_f32(B={B}, H={H}, D={D}, R={R}, J={J}, T={T})")
    return records


def ln_bh4_block_hash_records_direct(x, ln_w, ln_b, eps, w_folded, pbias, T, decay, residual, plan):
    """The same for BH4 with 64 x 64 blocks (folded weights [R, J, D/64, 64, 64]) on the matrix cores."""
    _require(x.dtype == torch.float32 and x.is_cuda and x.is_contiguous() and x.dim() == 2, "x: contiguous fp32 [B, H] on the GPU")
    B, H = x.shape
    R, J, NB, bs, _ = w_folded.shape
    D = NB * bs
    _require(H == ln_w.numel() and T * 8 <= R * D and T % 2 == 0 and plan[1] >= B, "shapes do not fit the record plan")
    records = torch.empty(plan[2] // 4, dtype=torch.int32, device=x.device)
    with _dev_guard(x):
        rc = _lib.load().lffn_ln_bh4_block_hash_records_f32(
            x.data_ptr(), ln_w.data_ptr(), ln_b.data_ptr(), eps, w_folded.data_ptr(), None if pbias is None else pbias.data_ptr(),
            records.data_ptr(), plan[1], plan[0], B, H, D, R, J, T, bs, decay, residual, _lib.stream_of(x))
    if rc != 0:
        _lib.check(rc, f"lffn_ln_bh4_block_hash_records_f32(B={B}, H={H}, D={D}, R={R}, J={J}, T={T})")
    return records


def lookup_gather_records_direct(records, plan, tables, bias, residual, B):
    """out[b] = residual[b] + bias + sum_t score * row, from the record stream written for `plan` (which was
    made for the tables' row format)."""
    T, S, Do = tables.shape
    fmt = row_format(tables.dtype)
    _require(fmt is not None and tables.is_contiguous() and records.numel() * 4 >= plan[2],
             "tables: contiguous float32, bfloat16 or float16; records: at least the plan's bytes")
    _require(residual is None or (residual.dtype == torch.float32 and residual.is_contiguous()
                                  and residual.device == tables.device and tuple(residual.shape) == (B, Do)),
             "residual: contiguous fp32 [B, Do] on the tables' device")
    out = torch.empty(B, Do, dtype=torch.float32, device=tables.device)
    with _dev_guard(tables):
        rc = _lib.load().lffn_lookup_gather_records_rows(
            records.data_ptr(), plan[1], tables.data_ptr(), None if bias is None else bias.data_ptr(),
            None if residual is None else residual.data_ptr(), out.data_ptr(), B, T, S, Do, fmt, plan[0], _lib.stream_of(tables))
    if rc != 0:
        _lib.check(rc, f"lffn_lookup_gather_records_rows(B={B}, T={T}, S={S}, Do={Do}, row_format={fmt})")
    return out


_L.define("lookup_gather(Tensor code, Tensor score, Tensor tables, Tensor? bias, Tensor? residual=None) -> Tensor")


def _lookup_gather_impl(code, score, tables, bias, residual=None):
    _lib.require_gpu(code, score, tables, bias, residual)
    assert tables.dim() == 3 and tables.is_contiguous()
    assert score.dtype == torch.float32 and score.is_contiguous()
    assert tuple(score.shape) == tuple(code.shape)
    B, T = code.shape
    T2, S, Do = tables.shape
    assert T2 == T and _is_pow2(S)
    _check_gather_args(code, T * S, Do)
    if bias is not None:
        assert bias.dtype == torch.float32 and bias.is_contiguous() and bias.numel() == Do
    if residual is not None:
        assert residual.dtype == torch.float32 and residual.is_contiguous() and tuple(residual.shape) == (B, Do)
    out = torch.empty(B, Do, dtype=torch.float32, device=tables.device)
    lib = _lib.load()
    fmt = row_format(tables.dtype)
    if fmt is None:
        raise NotImplementedError(f"lookup_gather: table dtype {tables.dtype} (float32, bfloat16 and float16 are built)")
    # many tokens: the four-lanes-per-token form, which wants a workspace for its record stream; a few
    # thousand: the table-split form, which wants one for its partial outputs
    ws_bytes = ctypes.c_int64(0)
    _lib.check(lib.lffn_lookup_gather_workspace_bytes(B, T, S, Do, fmt, ctypes.byref(ws_bytes)),
               "lffn_lookup_gather_workspace_bytes")
    sfx = ("f32", "bf16", "f16")[fmt]
    with _dev_guard(tables):
        if ws_bytes.value > 0 or fmt == ROWS_F16:
            name = "lffn_lookup_gather_ws_" + sfx
            ws = torch.empty(ws_bytes.value, dtype=torch.uint8, device=tables.device) if ws_bytes.value > 0 else None
            rc = getattr(lib, name)(_lib.ptr(code), _lib.ptr(score), _lib.ptr(tables), _lib.ptr(bias), _lib.ptr(residual),
                                    _lib.ptr(out), _lib.ptr(ws), ws_bytes.value, B, T, S, Do, _lib.stream_of(tables))
        else:
            name = "lffn_lookup_gather_residual_" + sfx
            rc = getattr(lib, name)(_lib.ptr(code), _lib.ptr(score), _lib.ptr(tables), _lib.ptr(bias), _lib.ptr(residual),
                                    _lib.ptr(out), B, T, S, Do, _lib.stream_of(tables))
    _lib.check(rc, f"{name}(B={B}, T={T}, S={S}, Do={Do})")
    return out


_L.impl("lookup_gather", _lookup_gather_impl, "CUDA")


@torch.library.register_fake("lookupffn::lookup_gather")
def _(code, score, tables, bias, residual=None):
    return score.new_empty(code.shape[0], tables.shape[2])


_L.define("indexed_inner_product(Tensor indexes, Tensor source_1, Tensor source_2) -> Tensor")


def _inner_impl(indexes, source_1, source_2):
    """fp32 inputs, or both half (the reference's reduced-precision call): the result is fp32 either way."""
    _lib.require_gpu(indexes, source_1, source_2)
    assert source_1.dim() == 2 and source_2.dim() == 2
    assert source_1.dtype == source_2.dtype and source_2.dtype in (torch.float32, torch.float16), \
        (source_1.dtype, source_2.dtype)
    assert source_1.is_contiguous() and source_2.is_contiguous()
    B, I = indexes.shape
    S, Dv = source_2.shape
    assert source_1.shape[0] == B and source_1.shape[1] == Dv
    _check_gather_args(indexes, S, Dv)
    out = torch.empty(B, I, dtype=torch.float32, device=source_2.device)
    lib = _lib.load()
    fn, name = ((lib.lffn_indexed_inner_product_f16, "lffn_indexed_inner_product_f16")
                if source_2.dtype == torch.float16 else
                (lib.lffn_indexed_inner_product_f32, "lffn_indexed_inner_product_f32"))
    with _dev_guard(source_2):
        rc = fn(_lib.ptr(indexes), _lib.ptr(source_1), _lib.ptr(source_2), _lib.ptr(out), B, I, S, Dv,
                _lib.stream_of(source_2))
    _lib.check(rc, f"{name}(B={B}, I={I}, S={S}, Dv={Dv})")
    return out


_L.impl("indexed_inner_product", _inner_impl, "CUDA")


@torch.library.register_fake("lookupffn::indexed_inner_product")
def _(indexes, source_1, source_2):
    return source_1.new_empty(indexes.shape, dtype=torch.float32)


_L.define("scatter_add(Tensor indexes, Tensor source, Tensor weights, int output_size) -> Tensor")


def _scatter_impl(indexes, source, weights, output_size):
    """source fp32 or half (the reference's reduced-precision call); weights and the result fp32."""
    _lib.require_gpu(indexes, source, weights)
    assert source.dim() == 2 and source.dtype in (torch.float32, torch.float16) and source.is_contiguous()
    assert weights.dtype == torch.float32 and weights.is_contiguous()
    assert tuple(weights.shape) == tuple(indexes.shape)
    B, I = indexes.shape
    Dv = source.shape[1]
    assert source.shape[0] == B
    _check_gather_args(indexes, output_size, Dv)
    out = torch.zeros(output_size, Dv, dtype=torch.float32, device=source.device)
    lib = _lib.load()
    fn, name = ((lib.lffn_scatter_add_f16, "lffn_scatter_add_f16") if source.dtype == torch.float16 else
                (lib.lffn_scatter_add_f32, "lffn_scatter_add_f32"))
    with _dev_guard(source):
        rc = fn(_lib.ptr(indexes), _lib.ptr(source), _lib.ptr(weights), _lib.ptr(out), B, I, output_size, Dv,
                _lib.stream_of(source))
    _lib.check(rc, f"{name}(B={B}, I={I}, out={output_size}, Dv={Dv})")
    return out


_L.impl("scatter_add", _scatter_impl, "CUDA")


@torch.library.register_fake("lookupffn::scatter_add")
def _(indexes, source, weights, output_size):
    return source.new_empty(output_size, source.shape[1], dtype=torch.float32)


# Below this many multiply-adds (B * T * Do) the LDS-accumulating scatter is the faster one
# (measured: 16384 x 32 x 768 and 16384 x 128 x 256 favour the sorted form, 2048 x 128 x 768 does not).
SORTED_SCATTER_MIN_WORK = 4 * 10 ** 8

_L.define("lookup_scatter(Tensor code, Tensor score, Tensor g, int S) -> Tensor")


def _lookup_scatter_impl(code, score, g, S):
    _lib.require_gpu(code, score, g)
    assert g.dim() == 2 and g.dtype == torch.float32 and g.is_contiguous()
    assert score.dtype == torch.float32 and score.is_contiguous()
    assert tuple(score.shape) == tuple(code.shape)
    B, T = code.shape
    Do = g.shape[1]
    assert g.shape[0] == B and _is_pow2(S)
    _check_gather_args(code, max(T * S, 1), Do)
    out = torch.empty(T, S, Do, dtype=torch.float32, device=g.device)     # fully overwritten by the kernel
    lib = _lib.load()
    ws_bytes = ctypes.c_int64(0)
    _lib.check(lib.lffn_lookup_scatter_workspace_bytes(B, T, S, Do, ctypes.byref(ws_bytes)), "lffn_lookup_scatter_workspace_bytes")
    with _dev_guard(g):
        if ws_bytes.value > 0 and B * T * Do >= SORTED_SCATTER_MIN_WORK:
            # sort the tokens of every table by code, then sum rows in registers: no atomics
            ws = torch.empty(ws_bytes.value, dtype=torch.uint8, device=g.device)
            rc = lib.lffn_lookup_scatter_sorted_f32(_lib.ptr(code), _lib.ptr(score), _lib.ptr(g), _lib.ptr(out), _lib.ptr(ws),
                                                    ws_bytes.value, B, T, S, Do, 0, _lib.stream_of(g))
            _lib.check(rc, f"lffn_lookup_scatter_sorted_f32(B={B}, T={T}, S={S}, Do={Do})")
        else:
            rc = lib.lffn_lookup_scatter_f32(_lib.ptr(code), _lib.ptr(score), _lib.ptr(g), _lib.ptr(out),
                                             B, T, S, Do, 0, _lib.stream_of(g))
            _lib.check(rc, f"lffn_lookup_scatter_f32(B={B}, T={T}, S={S}, Do={Do})")
    return out


_L.impl("lookup_scatter", _lookup_scatter_impl, "CUDA")


@torch.library.register_fake("lookupffn::lookup_scatter")
def _(code, score, g, S):
    return g.new_empty(code.shape[1], S, g.shape[1])


_L.define("lookup_backward(Tensor code, Tensor score, Tensor g, Tensor tables) -> (Tensor, Tensor)")


def lookup_backward_is_fused(B, T, S, Do):
    """Both gradients of the gather go through one call (lffn_lookup_backward_f32: the sorted scatter and the
    score gradient sharing one slice-major copy of g) for this shape."""
    if B * T * Do < SORTED_SCATTER_MIN_WORK or Do % 64 != 0:
        return False
    ws_bytes = ctypes.c_int64(0)
    _lib.check(_lib.load().lffn_lookup_scatter_workspace_bytes(B, T, S, Do, ctypes.byref(ws_bytes)),
               "lffn_lookup_scatter_workspace_bytes")
    return ws_bytes.value > 0


def _lookup_backward_impl(code, score, g, tables):
    """(grad_score [B, T], grad_tables [T, S, Do]) of out = sum_t score * tables[t, code]; g = grad of out."""
    _lib.require_gpu(code, score, g, tables)
    assert g.dim() == 2 and g.dtype == torch.float32 and g.is_contiguous()
    assert score.dtype == torch.float32 and score.is_contiguous() and tuple(score.shape) == tuple(code.shape)
    assert tables.dim() == 3 and tables.dtype == torch.float32 and tables.is_contiguous()
    B, T = code.shape
    Tt, S, Do = tables.shape
    assert Tt == T and g.shape[0] == B and g.shape[1] == Do and _is_pow2(S)
    _check_gather_args(code, max(T * S, 1), Do)
    if not lookup_backward_is_fused(B, T, S, Do):
        return _lookup_inner_impl(code, g, tables), _lookup_scatter_impl(code, score, g, S)
    lib = _lib.load()
    ws_bytes = ctypes.c_int64(0)
    _lib.check(lib.lffn_lookup_scatter_workspace_bytes(B, T, S, Do, ctypes.byref(ws_bytes)), "lffn_lookup_scatter_workspace_bytes")
    grad_score = torch.empty(B, T, dtype=torch.float32, device=g.device)          # both fully overwritten
    grad_tables = torch.empty(T, S, Do, dtype=torch.float32, device=g.device)
    ws = torch.empty(ws_bytes.value, dtype=torch.uint8, device=g.device)
    with _dev_guard(g):
        rc = lib.lffn_lookup_backward_f32(_lib.ptr(code), _lib.ptr(score), _lib.ptr(g), _lib.ptr(tables), _lib.ptr(grad_score),
                                          _lib.ptr(grad_tables), _lib.ptr(ws), ws_bytes.value, B, T, S, Do, 0, _lib.stream_of(g))
    _lib.check(rc, f"lffn_lookup_backward_f32(B={B}, T={T}, S={S}, Do={Do})")
    return grad_score, grad_tables


_L.impl("lookup_backward", _lookup_backward_impl, "CUDA")


@torch.library.register_fake("lookupffn::lookup_backward")
def _(code, score, g, tables):
    return g.new_empty(code.shape[0], code.shape[1]), g.new_empty(tables.shape)


_L.define("lookup_inner(Tensor code, Tensor g, Tensor tables) -> Tensor")


def _lookup_inner_impl(code, g, tables):
    _lib.require_gpu(code, g, tables)
    assert g.dim() == 2 and g.dtype == torch.float32 and g.is_contiguous()
    assert tables.dim() == 3 and tables.dtype == torch.float32 and tables.is_contiguous()
    B, T = code.shape
    Tt, S, Do = tables.shape
    assert Tt == T and g.shape[0] == B and g.shape[1] == Do and _is_pow2(S)
    _check_gather_args(code, max(T * S, 1), Do)
    out = torch.empty(B, T, dtype=torch.float32, device=g.device)     # fully overwritten by the kernels
    with _dev_guard(g):
        rc = _lib.load().lffn_lookup_inner_f32(_lib.ptr(code), _lib.ptr(g), _lib.ptr(tables), _lib.ptr(out),
                                               B, T, S, Do, _lib.stream_of(g))
    _lib.check(rc, f"lffn_lookup_inner_f32(B={B}, T={T}, S={S}, Do={Do})")
    return out


_L.impl("lookup_inner", _lookup_inner_impl, "CUDA")


@torch.library.register_fake("lookupffn::lookup_inner")
def _(code, g, tables):
    return g.new_empty(code.shape[0], code.shape[1])


fht = torch.ops.lookupffn.fht
bh4_diag = torch.ops.lookupffn.bh4_diag
bh4_fold = torch.ops.lookupffn.bh4_fold
bh4_block = torch.ops.lookupffn.bh4_block
mix_code_score = torch.ops.lookupffn.mix_code_score
bh4_fold_mode = torch.ops.lookupffn.bh4_fold_mode
bh4_block_hash_train = torch.ops.lookupffn.bh4_block_hash_train
bh4_block_bwd = torch.ops.lookupffn.bh4_block_bwd
bh4_block_wgrad = torch.ops.lookupffn.bh4_block_wgrad
ln_bh4_block_hash_train = torch.ops.lookupffn.ln_bh4_block_hash_train
ln_bh4_block_wgrad = torch.ops.lookupffn.ln_bh4_block_wgrad
lookup_ffn_fused = torch.ops.lookupffn.lookup_ffn_fused
layer_norm_bwd = torch.ops.lookupffn.layer_norm_bwd
ln_bh4_block_hash = torch.ops.lookupffn.ln_bh4_block_hash
project_hash = torch.ops.lookupffn.project_hash
project_hash_bwd = torch.ops.lookupffn.project_hash_bwd
ln_project_hash = torch.ops.lookupffn.ln_project_hash
code_score = torch.ops.lookupffn.code_score
code_score_bwd = torch.ops.lookupffn.code_score_bwd
gather_add = torch.ops.lookupffn.gather_add
lookup_gather = torch.ops.lookupffn.lookup_gather
indexed_inner_product = torch.ops.lookupffn.indexed_inner_product
scatter_add = torch.ops.lookupffn.scatter_add
lookup_scatter = torch.ops.lookupffn.lookup_scatter
lookup_backward = torch.ops.lookupffn.lookup_backward
lookup_inner = torch.ops.lookupffn.lookup_inner
