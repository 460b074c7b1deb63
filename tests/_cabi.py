"""Test helper: call the C ABI of liblookupffn_hip.so directly (ctypes), with
torch tensors used only as device memory.  Inputs are numpy arrays, outputs come
back as numpy arrays, so a parity test reads: oracle(numpy) vs cabi(numpy)."""
import ctypes

import numpy as np
import torch

from lookupffn_amd import _lib

DEV = "cuda:0"


def dev(a):
    if a is None:
        return None
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:    # bfloat16 bit patterns
        return torch.from_numpy(a.view(np.int16)).to(DEV)
    return torch.from_numpy(a).to(DEV)


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def _call(name, *args):
    stream = torch.cuda.current_stream().cuda_stream
    rc = getattr(_lib.load(), name)(*args, stream)
    assert rc == 0, f"{name} returned {rc}: {_lib.load().lffn_error_string(rc).decode()}"


def p(t):
    return None if t is None else t.data_ptr()


def fht(x):
    xd = dev(x)
    out = torch.empty_like(xd)
    _call("lffn_fht_f32", p(xd), p(out), x.shape[0], x.shape[1])
    return host(out)


def fht16(bits, bf16=False, in_place=False):
    """bits: uint16 patterns of half (or bfloat16) rows."""
    xd = dev(bits)
    out = xd if in_place else torch.full_like(xd, -1)
    _call("lffn_fht_bf16" if bf16 else "lffn_fht_f16", p(xd), p(out), bits.shape[0], bits.shape[1])
    return host(out).view(np.uint16)


def fht_inplace(x):
    xd = dev(x)
    _call("lffn_fht_f32", p(xd), p(xd), x.shape[0], x.shape[1])
    return host(xd)


def bh4_diag(x, diag):
    xd, dd = dev(x), dev(diag)
    B, H = x.shape
    R, J, D = diag.shape
    out = torch.empty(B, R * D, dtype=torch.float32, device=DEV)
    _call("lffn_bh4_diag_f32", p(xd), p(dd), p(out), B, H, D, R, J)
    return host(out)


def bh4_block(x, w):
    """fold + fused kernel; w: [R, J, NB, 64, 64]."""
    xd, wd = dev(x), dev(w)
    B, H = x.shape
    R, J, NB, bs, _ = w.shape
    wf = torch.empty_like(wd)
    _call("lffn_bh4_fold_f32", p(wd), p(wf), R, J, NB, bs)
    out = torch.full((B, R * NB * bs), float("nan"), dtype=torch.float32, device=DEV)
    _call("lffn_bh4_block_f32", p(xd), p(wf), p(out), B, H, NB * bs, R, J, bs)
    return host(out), host(wf)


def ln_bh4_block_hash(x, ln_w, ln_b, eps, w, bias, T, decay=0.7):
    """fold + the one-kernel front end; w: [R, J, NB, 64, 64]; ln_w None: no LayerNorm."""
    xd, lw, lb, wd, bd = dev(x), dev(ln_w), dev(ln_b), dev(w), dev(bias)
    B, H = x.shape
    R, J, NB, bs, _ = w.shape
    wf = torch.empty_like(wd)
    _call("lffn_bh4_fold_f32", p(wd), p(wf), R, J, NB, bs)
    codes = torch.full((B, T), -1, dtype=torch.int32, device=DEV)
    scores = torch.full((B, T), float("nan"), dtype=torch.float32, device=DEV)
    _call("lffn_ln_bh4_block_hash_f32", p(xd), p(lw), p(lb), float(np.float32(eps)), p(wf), p(bd), p(codes), p(scores),
          B, H, NB * bs, R, J, T, bs, float(np.float32(decay)), float(np.float32(1 - decay)))
    return host(codes), host(scores)


def bh4_fold_mode(w, mode):
    wd = dev(w)
    out = torch.full_like(wd, float("nan"))
    _call("lffn_bh4_fold_mode_f32", p(wd), p(out), w.size // (64 * 64), 64, mode)
    return host(out)


def bh4_block_train(x, w, bias, T, decay=0.7):
    """-> codes, scores, z, stage_inputs [R, J-1, B, D]"""
    xd, wd, bd = dev(x), dev(w), dev(bias)
    B, H = x.shape
    R, J, NB, bs, _ = w.shape
    D = NB * bs
    wf = torch.empty_like(wd)
    _call("lffn_bh4_fold_mode_f32", p(wd), p(wf), R * J * NB, bs, 0)
    codes = torch.full((B, T), -1, dtype=torch.int32, device=DEV)
    scores = torch.full((B, T), float("nan"), dtype=torch.float32, device=DEV)
    z = torch.full((B, T * 8), float("nan"), dtype=torch.float32, device=DEV)
    st = torch.full((R, max(J - 1, 1), B, D), float("nan"), dtype=torch.float32, device=DEV)
    _call("lffn_bh4_block_hash_train_f32", p(xd), p(wf), p(bd), p(codes), p(scores), p(z), p(st), B, H, D, R, J, T, bs,
          float(np.float32(decay)), float(np.float32(1 - decay)))
    return host(codes), host(scores), host(z), host(st)[:, :J - 1]


def ln_bh4_block_train(x, ln_w, ln_b, eps, w, bias, T, decay=0.7):
    """-> codes, scores, z, stage_inputs [R, J-1, B, D], row_stats [B, 2]"""
    xd, lw, lb, wd, bd = dev(x), dev(ln_w), dev(ln_b), dev(w), dev(bias)
    B, H = x.shape
    R, J, NB, bs, _ = w.shape
    D = NB * bs
    wf = torch.empty_like(wd)
    _call("lffn_bh4_fold_mode_f32", p(wd), p(wf), R * J * NB, bs, 0)
    codes = torch.full((B, T), -1, dtype=torch.int32, device=DEV)
    scores = torch.full((B, T), float("nan"), dtype=torch.float32, device=DEV)
    z = torch.full((B, T * 8), float("nan"), dtype=torch.float32, device=DEV)
    st = torch.full((R, max(J - 1, 1), B, D), float("nan"), dtype=torch.float32, device=DEV)
    stats = torch.full((B, 2), float("nan"), dtype=torch.float32, device=DEV)
    _call("lffn_ln_bh4_block_hash_train_f32", p(xd), p(lw), p(lb), float(np.float32(eps)), p(wf), p(bd), p(codes), p(scores),
          p(z), p(st), p(stats), B, H, D, R, J, T, bs, float(np.float32(decay)), float(np.float32(1 - decay)))
    return host(codes), host(scores), host(z), host(st)[:, :J - 1], host(stats)


def ln_bh4_block_wgrad(stage_grads, x, ln_w, ln_b, stats, stage_inputs, R, J):
    sg, xd, lw, lb, sd, si = dev(stage_grads), dev(x), dev(ln_w), dev(ln_b), dev(stats), dev(stage_inputs)
    S, B, D = stage_grads.shape
    g = torch.zeros(S, D // 64, 64, 64, dtype=torch.float32, device=DEV)
    _call("lffn_ln_bh4_block_wgrad_f32", p(sg), p(xd), p(lw), p(lb), p(sd), p(si), p(g), B, x.shape[1], D, R, J, 64)
    return host(g)


def bh4_block_bwd(g_z, w, H, decay=0.7):
    """-> g_x [R, B, H], stage_grads [R, J, B, D]"""
    gd, wd = dev(g_z), dev(w)
    B = g_z.shape[0]
    T = g_z.shape[1] // 8
    R, J, NB, bs, _ = w.shape
    D = NB * bs
    wt = torch.empty_like(wd)
    _call("lffn_bh4_fold_mode_f32", p(wd), p(wt), R * J * NB, bs, 1)
    g_x = torch.full((R, B, H), float("nan"), dtype=torch.float32, device=DEV)
    sg = torch.full((R, J, B, D), float("nan"), dtype=torch.float32, device=DEV)
    _call("lffn_bh4_block_bwd_f32", p(gd), p(wt), p(g_x), p(sg), B, H, D, R, J, T, bs,
          float(np.float32(decay)), float(np.float32(1 - decay)))
    return host(g_x), host(sg)


def bh4_block_wgrad(stage_grads, x, stage_inputs, R, J, init=None):
    sg, xd, si = dev(stage_grads), dev(x), dev(stage_inputs)
    S, B, D = stage_grads.shape
    g = torch.zeros(S, D // 64, 64, 64, dtype=torch.float32, device=DEV) if init is None else dev(init)
    _call("lffn_bh4_block_wgrad_f32", p(sg), p(xd), p(si), p(g), B, x.shape[1], D, R, J, 64)
    return host(g)


def lookup_ffn_fused(x, ln_w, ln_b, eps, diag, pbias, tables, obias, residual, decay=0.7):
    xd, dd, td = dev(x), dev(diag), dev(tables)
    lw, lb = (None, None) if ln_w is None else (dev(ln_w), dev(ln_b))
    pb = None if pbias is None else dev(pbias)
    ob = None if obias is None else dev(obias)
    rs = None if residual is None else dev(residual)
    B, H = x.shape
    R, J, D = diag.shape
    T, S, Do = tables.shape
    out = torch.full((B, Do), float("nan"), dtype=torch.float32, device=DEV)
    _call("lffn_lookup_ffn_fused_f32", p(xd), p(lw), p(lb), float(np.float32(eps)), p(dd), p(pb), p(td), p(ob), p(rs),
          p(out), B, H, D, R, J, T, S, Do, float(np.float32(decay)), float(np.float32(1 - decay)))
    return host(out)


def lookup_ffn_fused_layer(x, ln_w, ln_b, eps, diag, pbias, tables, obias, residual, decay=0.7):
    """lffn_lookup_ffn_fused_layer_f32: the same call with the parameters in a struct lffn_fused_layer."""
    xd, dd, td = dev(x), dev(diag), dev(tables)
    lw, lb = (None, None) if ln_w is None else (dev(ln_w), dev(ln_b))
    pb, ob, rs = dev(pbias), dev(obias), dev(residual)
    B, H = x.shape
    R, J, D = diag.shape
    T, S, Do = tables.shape
    blk = _lib.FusedLayer(p(lw), p(lb), p(dd), p(pb), p(td), p(ob), H, D, R, J, T, S, Do, float(np.float32(eps)),
                          float(np.float32(decay)), float(np.float32(1 - decay)))
    out = torch.full((B, Do), float("nan"), dtype=torch.float32, device=DEV)
    _call("lffn_lookup_ffn_fused_layer_f32", ctypes.byref(blk), p(xd), p(rs), p(out), B)
    return host(out)


def layer_norm_bwd(x, w, eps, g_y, num_partials=7):
    xd, gd = dev(x), dev(g_y)
    wd = None if w is None else dev(w)
    R, B, H = g_y.shape
    g_x = torch.full((B, H), float("nan"), dtype=torch.float32, device=DEV)
    pw = torch.full((num_partials, H), float("nan"), dtype=torch.float32, device=DEV)
    pb = torch.full((num_partials, H), float("nan"), dtype=torch.float32, device=DEV)
    _call("lffn_layer_norm_bwd_f32", p(xd), p(wd), float(np.float32(eps)), p(gd), p(g_x), p(pw), p(pb), B, H, R, num_partials)
    return host(g_x), host(pw).astype(np.float64).sum(0), host(pb).astype(np.float64).sum(0)


def mix_code_score(y, x, bias, T, k, D, decay=0.7):
    yd, xd, bd = dev(y), dev(x), dev(bias)
    B, ldy = y.shape
    H = x.shape[1]
    codes = torch.full((B, T), -1, dtype=torch.int32, device=DEV)
    scores = torch.full((B, T), float("nan"), dtype=torch.float32, device=DEV)
    _call("lffn_mix_code_score_f32", p(yd), p(xd), p(bd), p(codes), p(scores), B, T, k, H, D, ldy,
          float(decay), float(1 - decay))
    return host(codes), host(scores)


def project_hash(x, diag, bias, T, decay=0.7, keep_z=True):
    xd, dd, bd = dev(x), dev(diag), dev(bias)
    B, H = x.shape
    R, J, D = diag.shape
    codes = torch.full((B, T), -1, dtype=torch.int32, device=DEV)
    scores = torch.full((B, T), float("nan"), dtype=torch.float32, device=DEV)
    z = torch.full((B, T * 8), float("nan"), dtype=torch.float32, device=DEV) if keep_z else None
    _call("lffn_project_hash_f32", p(xd), p(dd), p(bd), p(z), p(codes), p(scores), B, H, D, R, J, T,
          float(np.float32(decay)), float(np.float32(1 - decay)))
    return host(codes), host(scores), (host(z) if keep_z else None)


def ln_project_hash(x, ln_w, ln_b, eps, diag, bias, T, decay=0.7):
    xd, wd, bd2, dd, bd = dev(x), dev(ln_w), dev(ln_b), dev(diag), dev(bias)
    B, H = x.shape
    R, J, D = diag.shape
    codes = torch.full((B, T), -1, dtype=torch.int32, device=DEV)
    scores = torch.full((B, T), float("nan"), dtype=torch.float32, device=DEV)
    z = torch.full((B, T * 8), float("nan"), dtype=torch.float32, device=DEV)
    _call("lffn_ln_project_hash_f32", p(xd), p(wd), p(bd2), float(np.float32(eps)), p(dd), p(bd), p(z), p(codes),
          p(scores), B, H, D, R, J, T, float(np.float32(decay)), float(np.float32(1 - decay)))
    return host(codes), host(scores), host(z)


def code_score(z):
    zd = dev(z)
    k = z.shape[-1]
    N = z.size // k
    codes = torch.full(z.shape[:-1], -1, dtype=torch.int32, device=DEV)
    scores = torch.full(z.shape[:-1], float("nan"), dtype=torch.float32, device=DEV)
    _call("lffn_code_score_f32", p(zd), p(codes), p(scores), N, k)
    return host(codes), host(scores)


def code_score_bwd(z, g):
    zd, gd = dev(z), dev(g)
    k = z.shape[-1]
    out = torch.full(z.shape, float("nan"), dtype=torch.float32, device=DEV)
    _call("lffn_code_score_bwd_f32", p(zd), p(gd), p(out), z.size // k, k)
    return host(out)


def gather_add(idx, src, w, bf16=False, fmt=None):
    """fmt (ROWS_*) overrides bf16; 16-bit rows are given as uint16 bit patterns."""
    idd, sd, wd = dev(idx), dev(src), dev(w)
    B, I = idx.shape
    S, Dv = src.shape
    out = torch.full((B, Dv), float("nan"), dtype=torch.float32, device=DEV)
    if fmt is None:
        fmt = ROWS_BF16 if bf16 else ROWS_F32
    _call(("lffn_gather_add_f32", "lffn_gather_add_bf16", "lffn_gather_add_f16")[fmt], p(idd), p(sd), p(wd), p(out), B, I, S, Dv)
    return host(out)


def lookup_gather(code, score, tables, bias=None, bf16=False, plan=None, residual=None, in_place=False):
    """plan = (tables_per_buffer, tokens_per_workgroup) runs exactly that kernel; residual [B, Do] is
    added inside the kernel (in_place: the residual buffer is also the output)."""
    cd, sd, td, bd = dev(code), dev(score), dev(tables), dev(bias)
    B, T = code.shape
    _, S, Do = tables.shape
    out = torch.full((B, Do), float("nan"), dtype=torch.float32, device=DEV)
    if residual is not None:
        assert plan is None
        rd = dev(residual)
        if in_place:
            out = rd
        _call("lffn_lookup_gather_residual_bf16" if bf16 else "lffn_lookup_gather_residual_f32",
              p(cd), p(sd), p(td), p(bd), p(rd), p(out), B, T, S, Do)
    elif plan is None:
        _call("lffn_lookup_gather_bf16" if bf16 else "lffn_lookup_gather_f32",
              p(cd), p(sd), p(td), p(bd), p(out), B, T, S, Do)
    else:
        _call("lffn_lookup_gather_planned_bf16" if bf16 else "lffn_lookup_gather_planned_f32",
              p(cd), p(sd), p(td), p(bd), p(out), B, T, S, Do, plan[0], plan[1])
    return host(out)


def lookup_gather_workspace_bytes(B, T, S, Do, bf16=False):
    """bf16: False / True, or a row format (ROWS_*)."""
    n = ctypes.c_int64(-1)
    assert _lib.load().lffn_lookup_gather_workspace_bytes(B, T, S, Do, int(bf16), ctypes.byref(n)) == 0
    return n.value


def lookup_gather_ws(code, score, tables, bias=None, bf16=False, residual=None, ws_bytes=None):
    """The workspace form; ws_bytes None = what lffn_lookup_gather_workspace_bytes asks for."""
    cd, sd, td, bd = dev(code), dev(score), dev(tables), dev(bias)
    rd = None if residual is None else dev(residual)
    B, T = code.shape
    _, S, Do = tables.shape
    if ws_bytes is None:
        ws_bytes = lookup_gather_workspace_bytes(B, T, S, Do, bf16)
    ws = torch.full((max(ws_bytes, 16) // 4,), float("nan"), dtype=torch.float32, device=DEV)
    out = torch.full((B, Do), float("nan"), dtype=torch.float32, device=DEV)
    _call("lffn_lookup_gather_ws_bf16" if bf16 else "lffn_lookup_gather_ws_f32",
          p(cd), p(sd), p(td), p(bd), p(rd), p(out), p(ws) if ws_bytes else None, ws_bytes, B, T, S, Do)
    return host(out)


def lookup_gather_ws_planned(code, score, tables, plan, bias=None, residual=None, ws_bytes=None):
    """Exactly the kernel `plan` = (tables_per_buffer, tokens_per_workgroup), with a workspace (fp32 rows);
    ws_bytes None = room for the record stream of form 3.  Returns (status, output)."""
    cd, sd, td, bd = dev(code), dev(score), dev(tables), dev(bias)
    rd = None if residual is None else dev(residual)
    B, T = code.shape
    _, S, Do = tables.shape
    if ws_bytes is None:
        ws_bytes = 6 * T * (B + 2048)
    ws = torch.full((max(ws_bytes, 16) // 4,), float("nan"), dtype=torch.float32, device=DEV)
    out = torch.full((B, Do), float("nan"), dtype=torch.float32, device=DEV)
    rc = _lib.load().lffn_lookup_gather_ws_planned_f32(p(cd), p(sd), p(td), p(bd), p(rd), p(out), p(ws) if ws_bytes else None,
                                                       ws_bytes, B, T, S, Do, plan[0], plan[1], None)
    torch.cuda.synchronize()
    return rc, host(out)


ROWS_F32, ROWS_BF16, ROWS_F16 = 0, 1, 2


def rows_of(tables_f32, fmt):
    """fp32 tables in the row format `fmt`: (what the kernel is given, the values it multiplies as float64)."""
    import oracle
    if fmt == ROWS_F32:
        return tables_f32, tables_f32.astype(np.float64)
    if fmt == ROWS_BF16:
        bits = oracle.bf16_round(tables_f32.reshape(-1, tables_f32.shape[-1])).reshape(tables_f32.shape)
        return bits, oracle.bf16_widen(bits.reshape(-1, bits.shape[-1])).reshape(bits.shape).astype(np.float64)
    half = tables_f32.astype(np.float16)
    return half.view(np.uint16), half.astype(np.float64)


def lookup_gather_ws_planned_rows(code, score, tables, fmt, plan, bias=None, residual=None, ws_bytes=None):
    """lffn_lookup_gather_ws_planned_rows: exactly the kernel `plan` on rows of format `fmt` (tables: fp32, or
    uint16 bit patterns of bfloat16 / half).  Returns (status, output)."""
    cd, sd, td, bd = dev(code), dev(score), dev(tables), dev(bias)
    rd = None if residual is None else dev(residual)
    B, T = code.shape
    _, S, Do = tables.shape
    if ws_bytes is None:
        ws_bytes = 6 * T * (B + 2048)
    ws = torch.full((max(ws_bytes, 16) // 4,), float("nan"), dtype=torch.float32, device=DEV)
    out = torch.full((B, Do), float("nan"), dtype=torch.float32, device=DEV)
    rc = _lib.load().lffn_lookup_gather_ws_planned_rows(p(cd), p(sd), p(td), p(bd), p(rd), p(out), p(ws) if ws_bytes else None,
                                                        ws_bytes, B, T, S, Do, fmt, plan[0], plan[1], None)
    torch.cuda.synchronize()
    return rc, host(out)


def lookup_gather_ws_f16(code, score, tables_bits, bias=None, residual=None, ws_bytes=None):
    cd, sd, td, bd = dev(code), dev(score), dev(tables_bits), dev(bias)
    rd = None if residual is None else dev(residual)
    B, T = code.shape
    _, S, Do = tables_bits.shape
    if ws_bytes is None:
        ws_bytes = lookup_gather_workspace_bytes(B, T, S, Do, ROWS_F16)
    ws = torch.full((max(ws_bytes, 16) // 4,), float("nan"), dtype=torch.float32, device=DEV)
    out = torch.full((B, Do), float("nan"), dtype=torch.float32, device=DEV)
    _call("lffn_lookup_gather_ws_f16", p(cd), p(sd), p(td), p(bd), p(rd), p(out), p(ws) if ws_bytes else None, ws_bytes,
          B, T, S, Do)
    return host(out)


def lookup_gather_ws_plan(B, T, S, Do, fmt=0, ws_bytes=1 << 40):
    form = ctypes.c_int32(-1)
    tokens = _lib.load().lffn_lookup_gather_ws_plan(B, T, S, Do, fmt, ws_bytes, ctypes.byref(form))
    return form.value, tokens


def lookup_gather_records_plan_rows(B, T, S, Do, fmt):
    tokens, stride, nbytes = ctypes.c_int32(-1), ctypes.c_int64(-1), ctypes.c_int64(-1)
    assert _lib.load().lffn_lookup_gather_records_plan_rows(B, T, S, Do, fmt, ctypes.byref(tokens), ctypes.byref(stride),
                                                            ctypes.byref(nbytes)) == 0
    return tokens.value, stride.value, nbytes.value


def lookup_gather_records_plan(B, T, S, Do):
    tokens, stride, nbytes = ctypes.c_int32(-1), ctypes.c_int64(-1), ctypes.c_int64(-1)
    assert _lib.load().lffn_lookup_gather_records_plan(B, T, S, Do, ctypes.byref(tokens), ctypes.byref(stride),
                                                       ctypes.byref(nbytes)) == 0
    return tokens.value, stride.value, nbytes.value


def record_slots(B, tokens):
    """Where the records of tokens 0..B-1 sit among a table pair's, for a gather of `tokens` tokens per
    workgroup: a tile is passes of 16 wavefronts x 16 tokens (group p*16 + w of the tile = pass p of wavefront
    w), a wavefront's records of all its passes are contiguous, wavefronts and tiles follow each other."""
    npm1 = (tokens - 1) // 256
    n_last = tokens // 16 - 16 * npm1
    b = np.arange(B, dtype=np.int64)
    tile, r = b // tokens, b % tokens
    group = r // 16
    wave, pas = group % 16, group // 16
    return tile * tokens + 16 * (npm1 * wave + np.minimum(wave, n_last)) + pas * 16 + r % 16


def records_of_tokens(rec, T, stride, B, tokens):
    """The record stream as [T/2, B, 3] words (token order)."""
    return rec.reshape(T // 2, stride, 3)[:, record_slots(B, tokens), :]


def layer_through_records(x, ln_w, ln_b, eps, diag, pbias, tables, obias, residual=None, decay=0.7, plan=None):
    """lffn_ln_project_hash_records_f32 followed by lffn_lookup_gather_records_f32; returns (output, records)."""
    B, H = x.shape
    R, J, D = diag.shape
    T, S, Do = tables.shape
    tokens, stride, nbytes = plan if plan is not None else lookup_gather_records_plan(B, T, S, Do)
    assert nbytes > 0
    xd, wd, bd, dd, pd, td, od = dev(x), dev(ln_w), dev(ln_b), dev(diag), dev(pbias), dev(tables), dev(obias)
    rd = None if residual is None else dev(residual)
    rec = torch.full((nbytes // 4,), -1, dtype=torch.int32, device=DEV)
    out = torch.full((B, Do), float("nan"), dtype=torch.float32, device=DEV)
    _call("lffn_ln_project_hash_records_f32", p(xd), p(wd), p(bd), eps, p(dd), p(pd), p(rec), stride, tokens, B, H, D, R, J, T,
          decay, 1.0 - decay)
    _call("lffn_lookup_gather_records_f32", p(rec), stride, p(td), p(od), p(rd), p(out), B, T, S, Do, tokens)
    return host(out), rec.cpu().numpy().view(np.uint32)


def lookup_gather_plan(B, T, S, Do, bf16=False):
    kind = ctypes.c_int32(-1)
    tokens = _lib.load().lffn_lookup_gather_plan(B, T, S, Do, int(bf16), ctypes.byref(kind))
    return kind.value, tokens


def indexed_inner_product(idx, g, src):
    idd, gd, sd = dev(idx), dev(g), dev(src)
    B, I = idx.shape
    S, Dv = src.shape
    out = torch.full((B, I), float("nan"), dtype=torch.float32, device=DEV)
    half = src.dtype == np.uint16              # half bit patterns for g and src: the reduced-precision call
    assert (g.dtype == np.uint16) == half
    _call("lffn_indexed_inner_product_f16" if half else "lffn_indexed_inner_product_f32",
          p(idd), p(gd), p(sd), p(out), B, I, S, Dv)
    return host(out)


def scatter_add(idx, g, w, out_size, init=None):
    idd, gd, wd = dev(idx), dev(g), dev(w)
    B, I = idx.shape
    Dv = g.shape[1]
    out = torch.zeros(out_size, Dv, dtype=torch.float32, device=DEV) if init is None else dev(init)
    _call("lffn_scatter_add_f16" if g.dtype == np.uint16 else "lffn_scatter_add_f32",     # uint16: half bit patterns
          p(idd), p(gd), p(wd), p(out), B, I, out_size, Dv)
    return host(out)


def lookup_scatter(code, score, g, S, accumulate=False, init=None):
    cd, sd, gd = dev(code), dev(score), dev(g)
    B, T = code.shape
    Do = g.shape[1]
    if init is None:
        out = torch.full((T, S, Do), float("nan"), dtype=torch.float32, device=DEV)   # must be fully overwritten
    else:
        out = dev(init)
    _call("lffn_lookup_scatter_f32", p(cd), p(sd), p(gd), p(out), B, T, S, Do, 1 if accumulate else 0)
    return host(out)


def lookup_scatter_workspace_bytes(B, T, S, Do):
    n = ctypes.c_int64(-1)
    rc = _lib.load().lffn_lookup_scatter_workspace_bytes(B, T, S, Do, ctypes.byref(n))
    assert rc == 0
    return n.value


def lookup_scatter_sorted(code, score, g, S, accumulate=False, init=None):
    cd, sd, gd = dev(code), dev(score), dev(g)
    B, T = code.shape
    Do = g.shape[1]
    nbytes = lookup_scatter_workspace_bytes(B, T, S, Do)
    assert nbytes > 0
    ws = torch.full((nbytes // 4,), 0x7f7f7f7f, dtype=torch.int32, device=DEV)      # scratch: any contents
    if init is None:
        out = torch.full((T, S, Do), float("nan"), dtype=torch.float32, device=DEV)   # must be fully overwritten
    else:
        out = dev(init)
    _call("lffn_lookup_scatter_sorted_f32", p(cd), p(sd), p(gd), p(out), p(ws), nbytes, B, T, S, Do, 1 if accumulate else 0)
    return host(out)


def lookup_backward(code, score, g, tables, accumulate=False, init=None, want=(True, True)):
    """lffn_lookup_backward_f32 -> (grad_score [B, T] or None, grad_tables [T, S, Do] or None)."""
    cd, sd, gd, td = dev(code), dev(score), dev(g), dev(tables)
    B, T = code.shape
    _, S, Do = tables.shape
    nbytes = lookup_scatter_workspace_bytes(B, T, S, Do)
    assert nbytes > 0
    ws = torch.full((nbytes // 4,), 0x7f7f7f7f, dtype=torch.int32, device=DEV)      # scratch: any contents
    gs = torch.full((B, T), float("nan"), dtype=torch.float32, device=DEV) if want[0] else None
    gt = None
    if want[1]:
        gt = torch.full((T, S, Do), float("nan"), dtype=torch.float32, device=DEV) if init is None else dev(init)
    _call("lffn_lookup_backward_f32", p(cd), p(sd), p(gd), p(td), p(gs), p(gt), p(ws), nbytes, B, T, S, Do,
          1 if accumulate else 0)
    return (None if gs is None else host(gs)), (None if gt is None else host(gt))


def lookup_inner(code, g, tables):
    cd, gd, td = dev(code), dev(g), dev(tables)
    B, T = code.shape
    _, S, Do = tables.shape
    out = torch.full((B, T), float("nan"), dtype=torch.float32, device=DEV)   # must be fully overwritten
    _call("lffn_lookup_inner_f32", p(cd), p(gd), p(td), p(out), B, T, S, Do)
    return host(out)


def sum_partials(parts_a, parts_b=None, chunks=1):
    """-> column sums of one or two [P, n] arrays, one row of sums per chunk of rows."""
    ad, bd = dev(parts_a), dev(parts_b)
    P, na = parts_a.shape
    nb = 0 if parts_b is None else parts_b.shape[1]
    oa = torch.full((chunks, na), float("nan"), dtype=torch.float32, device=DEV)
    ob = None if parts_b is None else torch.full((chunks, nb), float("nan"), dtype=torch.float32, device=DEV)
    _call("lffn_sum_partials_f32", p(ad), p(oa), na, p(bd), p(ob), nb, P, chunks)
    if chunks == 1:
        return host(oa)[0], (None if ob is None else host(ob)[0])
    return host(oa), (None if ob is None else host(ob))


def project_hash_bwd(x, diag, z, g_score, ln_w=None, ln_b=None, eps=1e-5, decay=0.7, nparts=64):
    """-> g_x [R, B, H] (w.r.t. the LayerNorm output when ln_w is given), grad diag [R, J, D], grad bias [R*D]."""
    xd, dd, zd, gd, lw, lb = dev(x), dev(diag), dev(z), dev(g_score), dev(ln_w), dev(ln_b)
    B, H = x.shape
    R, J, D = diag.shape
    T = g_score.shape[1]
    g_x = torch.full((R, B, H), float("nan"), dtype=torch.float32, device=DEV)
    part_d = torch.full((nparts, R, J, D), float("nan"), dtype=torch.float32, device=DEV)
    part_b = torch.full((nparts, R * D), float("nan"), dtype=torch.float32, device=DEV)
    dc, rc = float(np.float32(decay)), float(np.float32(1 - decay))
    if ln_w is None:
        _call("lffn_project_hash_bwd_f32", p(xd), p(dd), p(zd), p(gd), p(g_x), p(part_d), p(part_b),
              B, H, D, R, J, T, nparts, dc, rc)
    else:
        _call("lffn_ln_project_hash_bwd_f32", p(xd), p(lw), p(lb), float(np.float32(eps)), p(dd), p(zd), p(gd), p(g_x),
              p(part_d), p(part_b), B, H, D, R, J, T, nparts, dc, rc)
    torch.cuda.synchronize()
    return host(g_x), part_d.double().sum(0).cpu().numpy(), part_b.double().sum(0).cpu().numpy()
