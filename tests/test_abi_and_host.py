"""CPU-only checks of the boundary and host logic: the C-ABI library loads and
exports every symbol include/lookupffn_hip.h declares, argument validation
returns error codes without touching a GPU, and the module surface keeps the
reference's parameter names, shapes and config attributes (PL/lookup.py:10-130).
No kernel is launched here.
"""
import ctypes
import os
import re
from argparse import Namespace

import pytest
import torch

import lookupffn_amd
from lookupffn_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    hdr = open(os.path.join(ROOT, "include", "lookupffn_hip.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    return sorted(set(re.findall(r"\b(lffn_\w+)\s*\(", hdr)))


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(_lib.LIB_PATH)
    names = _declared()
    assert len(names) >= 12
    for n in names:
        assert hasattr(lib, n), n
    assert names == sorted(_lib.exported_symbols())


def test_version_and_error_strings():
    lib = _lib.load()
    assert lib.lffn_version() == _lib.ABI_VERSION
    for code in (0, -1, -2, -3, -99):
        assert len(lib.lffn_error_string(code)) > 0


def test_argument_validation_needs_no_gpu():
    lib = _lib.load()
    # null pointers
    assert lib.lffn_fht_f32(None, None, 4, 8, None) == _lib.LFFN_ERR_BAD_ARG
    assert lib.lffn_gather_add_f32(None, None, None, None, 4, 2, 8, 64, None) == _lib.LFFN_ERR_BAD_ARG
    assert lib.lffn_indexed_inner_product_f16(256, None, 256, 256, 4, 2, 8, 64, None) == _lib.LFFN_ERR_BAD_ARG
    assert lib.lffn_scatter_add_f16(256, 256, 256, None, 4, 2, 8, 64, None) == _lib.LFFN_ERR_BAD_ARG
    assert lib.lffn_indexed_inner_product_f16(256, 256, 256, 256, 4, 2, 8, 96, None) == _lib.LFFN_ERR_UNSUPPORTED  # Dv % 64
    assert lib.lffn_scatter_add_f16(256, 258, 256, 256, 4, 2, 8, 64, None) == _lib.LFFN_ERR_BAD_ARG          # misaligned g
    assert lib.lffn_scatter_add_f16(None, None, None, None, 0, 2, 8, 64, None) == _lib.LFFN_ERR_BAD_ARG      # null g, out
    # unsupported shapes (pointers are never dereferenced on the host)
    assert lib.lffn_fht_f32(256, 256, 4, 2048, None) == _lib.LFFN_ERR_UNSUPPORTED
    assert lib.lffn_fht_f32(256, 256, 4, 48, None) == _lib.LFFN_ERR_UNSUPPORTED      # not a power of two
    assert lib.lffn_gather_add_f32(256, 256, 256, 256, 4, 2, 8, 96, None) == _lib.LFFN_ERR_UNSUPPORTED  # Dv % 64
    assert lib.lffn_code_score_f32(256, 256, 256, 4, 0, None) == _lib.LFFN_ERR_UNSUPPORTED
    assert lib.lffn_code_score_f32(256, 256, 256, 4, 25, None) == _lib.LFFN_ERR_UNSUPPORTED
    assert lib.lffn_lookup_gather_f32(256, 256, 256, None, 256, 4, 2, 100, 64, None) == _lib.LFFN_ERR_UNSUPPORTED  # S
    # misaligned output
    assert lib.lffn_fht_f32(256, 260, 4, 8, None) == _lib.LFFN_ERR_BAD_ARG
    # T*8 > R*D
    assert lib.lffn_project_hash_f32(256, 256, None, None, 256, 256, 4, 16, 16, 1, 4, 3, 0.7, 0.3, None) \
        == _lib.LFFN_ERR_BAD_ARG
    # empty batches succeed without a launch
    assert lib.lffn_fht_f32(256, 256, 0, 8, None) == _lib.LFFN_OK
    assert lib.lffn_gather_add_f32(256, 256, 256, 256, 0, 2, 8, 64, None) == _lib.LFFN_OK
    assert lib.lffn_code_score_f32(256, 256, 256, 0, 8, None) == _lib.LFFN_OK


def test_argument_validation_of_the_backward_and_block_entry_points():
    lib = _lib.load()
    U, A, OK = _lib.LFFN_ERR_UNSUPPORTED, _lib.LFFN_ERR_BAD_ARG, _lib.LFFN_OK
    P = 256                                    # a non-null, 16-byte aligned "pointer" that is never dereferenced
    # indexed inner product on table-local codes
    assert lib.lffn_lookup_inner_f32(None, None, None, None, 4, 2, 16, 64, None) == A
    assert lib.lffn_lookup_inner_f32(P, P, P, P, 4, 2, 100, 64, None) == U          # S not a power of two
    assert lib.lffn_lookup_inner_f32(P, P, P, P, 4, 2, 16, 96, None) == U           # Do % 64
    assert lib.lffn_lookup_inner_f32(P, P + 4, P, P, 4, 2, 16, 64, None) == A       # misaligned g
    assert lib.lffn_lookup_inner_f32(P, P, P, P, 0, 2, 16, 64, None) == OK
    # scatter-add on table-local codes
    assert lib.lffn_lookup_scatter_f32(P, P, P, P, 4, 2, 100, 64, 0, None) == U
    # BH4 with 64 x 64 blocks
    assert lib.lffn_bh4_fold_f32(P, P + 1024, 1, 4, 16, 32, None) == U              # block size other than 64
    assert lib.lffn_bh4_fold_f32(P, P, 1, 4, 16, 64, None) == A                     # in place
    assert lib.lffn_bh4_block_f32(P, P, P, 4, 768, 2048, 1, 4, 64, None) == U       # D > 1024
    assert lib.lffn_bh4_block_f32(P, P, P, 4, 770, 1024, 1, 4, 64, None) == U       # H % 4
    assert lib.lffn_bh4_block_f32(P, P, P, 4, 2000, 1024, 1, 4, 64, None) == A      # H > D
    assert lib.lffn_bh4_block_f32(P, P, P, 0, 768, 1024, 1, 4, 64, None) == OK
    assert lib.lffn_ln_bh4_block_hash_f32(P, None, None, 0.0, P, None, P, P, 4, 768, 1024, 1, 4, 200, 64,
                                          0.7, 0.3, None) == A                      # T*8 > R*D
    assert lib.lffn_ln_bh4_block_hash_f32(P, P, None, 1e-5, P, None, P, P, 4, 768, 1024, 1, 4, 128, 64,
                                          0.7, 0.3, None) == A                      # LayerNorm weight without bias
    assert lib.lffn_ln_bh4_block_hash_f32(P, None, None, 0.0, P, None, P, P, 0, 768, 1024, 1, 4, 128, 64,
                                          0.7, 0.3, None) == OK
    # column sums of partial sums
    assert lib.lffn_sum_partials_f32(P, P, 6, None, None, 0, 16, 1, None) == U          # n % 4
    assert lib.lffn_sum_partials_f32(P, P, 8, None, None, 4, 16, 1, None) == A          # second array missing
    assert lib.lffn_sum_partials_f32(P, P + 4, 8, None, None, 0, 16, 1, None) == A      # misaligned
    assert lib.lffn_sum_partials_f32(P, P, 8, None, None, 0, 0, 1, None) == A           # no partials
    assert lib.lffn_sum_partials_f32(P, P, 8, None, None, 0, 16, 17, None) == A         # more chunks than rows
    assert lib.lffn_sum_partials_f32(P, P, 8, None, None, 0, 10, 8, None) == A          # ceil(10/8) = 2 rows: chunk 5.. empty
    assert lib.lffn_sum_partials_f32(None, None, 0, None, None, 0, 16, 1, None) == OK   # nothing to add
    # mix + hash
    assert lib.lffn_mix_code_score_f32(P, P, None, P, P, 4, 8, 25, 64, 64, 256, 0.7, 0.3, None) == U   # k > 24
    assert lib.lffn_mix_code_score_f32(P, P, None, P, P, 4, 40, 8, 64, 64, 256, 0.7, 0.3, None) == A   # T*k > ldy
    assert lib.lffn_mix_code_score_f32(P, P, None, P, P, 0, 8, 8, 64, 64, 256, 0.7, 0.3, None) == OK
    # 16-bit transform
    assert lib.lffn_fht_f16(P, P, 4, 2048, None) == U
    assert lib.lffn_fht_bf16(P, P + 2, 4, 64, None) == A                            # 8-byte alignment
    assert lib.lffn_fht_f16(P, P, 0, 64, None) == OK
    # block-64 training kernels
    assert lib.lffn_bh4_fold_mode_f32(P, P + 1 << 20, 4, 64, 3, None) == U                 # mode
    assert lib.lffn_bh4_fold_mode_f32(P, P, 4, 64, 1, None) == A                           # in place
    assert lib.lffn_bh4_fold_mode_f32(P, P + 4096, 0, 64, 1, None) == OK
    assert lib.lffn_bh4_block_hash_train_f32(P, P, None, P, P, None, P, 4, 768, 1024, 1, 4, 128, 64,
                                             0.7, 0.3, None) == A                          # z is required
    assert lib.lffn_bh4_block_bwd_f32(P, P, P, P, 4, 768, 1024, 1, 4, 200, 64, 0.7, 0.3, None) == A   # T*8 > R*D
    assert lib.lffn_bh4_block_bwd_f32(P, P, P, P, 0, 768, 1024, 1, 4, 128, 64, 0.7, 0.3, None) == OK
    assert lib.lffn_bh4_block_wgrad_f32(P, P, P, P, 4, 768, 1024, 1, 4, 32, None) == U       # block size
    assert lib.lffn_bh4_block_wgrad_f32(P, P, P, P, 4, 770, 1024, 1, 4, 64, None) == U       # H % 4
    assert lib.lffn_bh4_block_wgrad_f32(P, P, None, P, 4, 768, 1024, 1, 4, 64, None) == A    # stage inputs needed
    assert lib.lffn_bh4_block_wgrad_f32(P, P, P, P, 4, 1088, 1024, 1, 4, 64, None) == A      # H > D
    assert lib.lffn_bh4_block_wgrad_f32(P, P, P, P, 0, 768, 1024, 1, 4, 64, None) == OK
    assert lib.lffn_project_hash_bwd_f32(P, P, P, P, P, P, P, 4, 64, 64, 1, 4, 8, 1, 0.7, 0.3, None) == U   # D < 256
    assert lib.lffn_project_hash_bwd_f32(P, P, P, P, P, P, P, 4, 768, 1024, 1, 5, 128, 1, 0.7, 0.3, None) == U  # J > 4
    lb = lib.lffn_ln_project_hash_bwd_f32
    assert lb(P, None, P, 1e-5, P, P, P, P, P, P, 4, 768, 1024, 1, 4, 128, 1, 0.7, 0.3, None) == A    # no LayerNorm weight
    assert lb(P, P, P + 4, 1e-5, P, P, P, P, P, P, 4, 768, 1024, 1, 4, 128, 1, 0.7, 0.3, None) == A   # misaligned bias
    assert lb(P, P, P, 1e-5, P, P, P, P, P, P, 4, 768, 1024, 1, 5, 128, 1, 0.7, 0.3, None) == U       # J > 4
    assert lib.lffn_lookup_scatter_sorted_f32(P, P, P, P, P, 1 << 30, 16, 4, 1024, 64, 0, None) == U    # S > 512
    assert lib.lffn_lookup_scatter_sorted_f32(P, P, P, P, P, 1 << 30, 16, 4, 16, 48, 0, None) == U      # Do % 32
    assert lib.lffn_lookup_scatter_sorted_f32(P, P, P, P, P, 64, 16, 4, 16, 64, 0, None) == A           # workspace too small
    assert lib.lffn_lookup_scatter_sorted_f32(P, P, P, P, None, 1 << 30, 16, 4, 16, 64, 0, None) == A
    assert lib.lffn_lookup_scatter_workspace_bytes(16, 4, 16, 64, None) == A
    # whole layer in one launch
    assert lib.lffn_lookup_ffn_fused_f32(P, P, P, 1e-5, P, P, P, P, P, P, 4, 64, 64, 1, 4, 8, 256, 64, 0.7, 0.3, None) == U   # D < 256
    assert lib.lffn_lookup_ffn_fused_f32(P, P, P, 1e-5, P, P, P, P, P, P, 4, 256, 256, 1, 4, 32, 128, 64, 0.7, 0.3, None) == U  # S < 256
    assert lib.lffn_lookup_ffn_fused_f32(P, P, P, 1e-5, P, P, P, P, P, P, 4, 256, 256, 1, 4, 32, 256, 66, 0.7, 0.3, None) == U  # Do % 4
    assert lib.lffn_lookup_ffn_fused_f32(P, P, None, 1e-5, P, P, P, P, P, P, 4, 256, 256, 1, 4, 32, 256, 64, 0.7, 0.3, None) == A
    assert lib.lffn_lookup_ffn_fused_f32(P, P, P, 1e-5, P, P, P, P, P, P, 4, 256, 256, 1, 4, 40, 256, 64, 0.7, 0.3, None) == A  # T*8 > R*D
    assert lib.lffn_lookup_ffn_fused_f32(P, P, P, 1e-5, P, P, P, P, P, P, 0, 256, 256, 1, 4, 32, 256, 64, 0.7, 0.3, None) == OK
    # LayerNorm backward
    assert lib.lffn_layer_norm_bwd_f32(P, P, 1e-5, P, P, P, P, 4, 1028, 1, 8, None) == U      # H > 1024
    assert lib.lffn_layer_norm_bwd_f32(P, P, 1e-5, P, P, P, P, 4, 770, 1, 8, None) == U       # H % 4
    assert lib.lffn_layer_norm_bwd_f32(P, P, 1e-5, P, P, P, None, 4, 768, 1, 8, None) == A    # partials: both or none
    assert lib.lffn_layer_norm_bwd_f32(P, P, 1e-5, P, P, P, P, 4, 768, 1, 0, None) == A
    # gather with a workspace
    assert lib.lffn_lookup_gather_workspace_bytes(2048, 128, 256, 768, 0, None) == A
    assert lib.lffn_lookup_gather_ws_f32(P, P, P, None, None, P, None, 64, 4, 2, 16, 64, None) == A     # bytes without a workspace
    assert lib.lffn_lookup_gather_ws_f32(P, P, P, None, None, P + 4, None, 0, 4, 2, 16, 64, None) == A
    # gather with residual
    assert lib.lffn_lookup_gather_residual_f32(P, P, P, None, P + 4, P, 4, 2, 16, 64, None) == A


def _config(**kw):
    base = dict(hidden_size=48, ffn_num_table=8, ffn_table_size=256, layer_norm_eps=1e-5,
                projection_type="bh4", block_size=1)
    base.update(kw)
    return Namespace(**base)


def test_workspace_queries_are_host_side_plans():
    """The workspace sizes are decided on the host from the shape alone (no GPU needed): which
    shapes take the table-split gather and the sorted scatter, and how much scratch they want."""
    lib = _lib.load()

    def gather_ws(B, T, S, Do, bf16=0):
        n = ctypes.c_int64(-1)
        assert lib.lffn_lookup_gather_workspace_bytes(B, T, S, Do, bf16, ctypes.byref(n)) == 0
        return n.value

    def scatter_ws(B, T, S, Do):
        n = ctypes.c_int64(-1)
        assert lib.lffn_lookup_scatter_workspace_bytes(B, T, S, Do, ctypes.byref(n)) == 0
        return n.value

    # RoBERTa-base tables: a few thousand tokens split the tables over 4 or 8 workgroups per unit
    assert gather_ws(2048, 128, 256, 768) == 4 * 2048 * 768 * 4
    assert gather_ws(1024, 128, 256, 768) == 8 * 1024 * 768 * 4
    assert gather_ws(4096, 128, 256, 768) == 4 * 4096 * 768 * 4
    # enough tokens to fill the chip without a split, too few tokens or tables for it to pay, bad shapes
    for shape in ((16384, 128, 128, 768), (256, 32, 256, 256), (4096, 16, 256, 768),
                  (2048, 128, 512, 768), (2048, 128, 256, 100), (0, 128, 256, 768)):
        assert gather_ws(*shape) == 0, shape
    # 16-bit rows (1 bfloat16, 2 half): the record stream as well, from 16384 tokens on at these tables
    for fmt in (1, 2):
        assert gather_ws(16384, 128, 256, 768, fmt) == 64 * (16384 + 2048) * 12
        assert gather_ws(16384, 512, 256, 1024, fmt) == 256 * (16384 + 2048) * 12
        assert gather_ws(8192, 128, 256, 768, fmt) == 0
    # many tokens, fp32 rows, 256-row tables, an even number of them: the four-lanes-per-token kernel, which
    # wants 12 bytes per (token, table pair) for its record stream (whole token tiles: up to 2048 tokens more)
    assert gather_ws(16384, 128, 256, 768) == 64 * (16384 + 2048) * 12
    assert gather_ws(8192, 128, 256, 768) == 64 * (8192 + 2048) * 12
    assert gather_ws(32768, 128, 256, 512) == 64 * (32768 + 2048) * 12
    assert gather_ws(65536, 128, 256, 768) == 64 * (65536 + 2048) * 12                              # one launch, no pieces
    assert gather_ws(16384, 512, 256, 1024) == 256 * (16384 + 2048) * 12                            # 537 MB of tables
    # which gather kernel a shape gets is a host-side decision as well: (tables per LDS buffer, tokens per workgroup)
    def plan(B, T, S, Do, bf16=0):
        kind = ctypes.c_int32(-1)
        tokens = lib.lffn_lookup_gather_plan(B, T, S, Do, bf16, ctypes.byref(kind))
        return kind.value, tokens

    assert plan(16384, 128, 256, 768) == (1, 832)               # RoBERTa-base: 240 workgroups in one round
    assert plan(16384, 512, 256, 1024) == (1, 1024)             # 537 MB of tables: 256 workgroups in one round
    assert plan(16384, 512, 256, 1024, 1) == (1, 512)           # the same in bf16 rows
    assert plan(32768, 128, 256, 512) == (1, 1024)              # the reference's compare.py shape
    assert plan(8192, 128, 256, 768) == (2, 1024)               # fewer tokens: two tables per buffer
    assert plan(256, 32, 256, 256) == (0, 0)                    # too few tokens to stage tables: token-major
    assert plan(16384, 128, 512, 768) == (0, 0)                 # tables too long for the LDS buffers
    # what the workspace entry points run, given a workspace: (form, tokens per workgroup); form 3 = four lanes
    # per token from a record stream, 4 = table split
    def ws_plan(B, T, S, Do, fmt=0, ws=1 << 40):
        form = ctypes.c_int32(-1)
        tokens = lib.lffn_lookup_gather_ws_plan(B, T, S, Do, fmt, ws, ctypes.byref(form))
        return form.value, tokens

    assert ws_plan(16384, 128, 256, 768) == (3, 1648)           # RoBERTa-base: 10 tiles of 103 groups of 16 tokens x 24 slices
    assert ws_plan(16384, 512, 256, 1024) == (3, 2048)
    assert ws_plan(16384, 512, 256, 1024, 1) == (3, 1024) and ws_plan(16384, 512, 256, 1024, 2) == (3, 1024)
    assert ws_plan(16384, 128, 256, 768, 0, 0) == plan(16384, 128, 256, 768)       # no workspace: the plain entry's kernel
    assert ws_plan(2048, 128, 256, 768) == (4, 512)             # table split
    assert ws_plan(2048, 128, 256, 768, 2) == (0, 0)            # half rows, few tokens: token-major
    assert ws_plan(256, 32, 256, 256) == (0, 0)
    assert lib.lffn_lookup_gather_ws_plan(16384, 128, 256, 768, 3, 0, None) == _lib.LFFN_ERR_BAD_ARG
    # sorted scatter: pairs + offsets + transposed codes and scores + packed gradient, for at most 16384 tokens
    one = scatter_ws(16384, 128, 256, 768)
    assert one >= 16384 * 128 * 8 + 16384 * 768 * 4
    assert scatter_ws(1 << 20, 128, 256, 768) == one
    assert scatter_ws(100, 128, 256, 768) < one
    for shape in ((0, 4, 16, 64), (16, 0, 16, 64), (16, 4, 1024, 64), (16, 4, 16, 48)):
        assert scatter_ws(*shape) == 0, shape


def test_gather_plans_are_consistent_over_a_grid_of_shapes():
    """Host-side sweep of the three gather queries over 15 000 shapes (ragged token counts, odd table
    counts, every row format).  Whenever the workspace entry point would run the four-lanes-per-token
    kernel, the record stream its plan describes fits the workspace the size query asked for, the tile
    is one the kernel is built for and a table pair's records cover every token slot of every tile; the stand-alone
    record plan obeys the same rules (it may choose the form for more shapes: its records come from the
    projection kernel, so it does not count a packing kernel)."""
    lib = _lib.load()
    passes_built = {0: (4, 5, 6, 7, 8), 1: (4,), 2: (4,)}
    seen = {}

    def check_tile(fmt, B, T, S, tokens, stride, nbytes):
        assert S == 256 and T % 2 == 0
        assert tokens % 16 == 0 and 16 <= tokens <= 2048
        np_ = -(-tokens // 256)
        assert np_ in passes_built[fmt], (fmt, tokens)
        ntiles = -(-B // tokens)
        assert stride == ntiles * tokens and stride % 16 == 0       # whole tiles: 16-byte copies stay aligned
        assert B <= stride < B + 2048
        assert nbytes == 6 * T * stride

    for B in (1, 15, 16, 255, 256, 1000, 2047, 2048, 3000, 4096, 5000, 8192, 10000, 12000, 16383, 16384,
              16385, 20000, 32768, 50000, 65536, 100000, 262144):
        for T in (2, 3, 16, 32, 128, 130, 512):
            for S in (16, 64, 128, 256):
                for Do in (64, 128, 192, 256, 512, 768, 1024, 2048):
                    for fmt in (0, 1, 2):
                        shape = (B, T, S, Do, fmt)
                        nb = ctypes.c_int64(-1)
                        assert lib.lffn_lookup_gather_workspace_bytes(B, T, S, Do, fmt, ctypes.byref(nb)) == 0, shape
                        assert nb.value >= 0
                        form = ctypes.c_int32(-1)
                        tokens = lib.lffn_lookup_gather_ws_plan(B, T, S, Do, fmt, nb.value, ctypes.byref(form))
                        assert form.value in (0, 1, 2, 3, 4) and tokens >= 0, shape
                        seen[form.value] = seen.get(form.value, 0) + 1
                        tpw, rs, by = ctypes.c_int32(-1), ctypes.c_int64(-1), ctypes.c_int64(-1)
                        assert lib.lffn_lookup_gather_records_plan_rows(B, T, S, Do, fmt, ctypes.byref(tpw),
                                                                        ctypes.byref(rs), ctypes.byref(by)) == 0, shape
                        if form.value == 3:
                            # the workspace form packs the same stream: same tile, and it fits what was asked for
                            assert tpw.value == tokens, shape
                            assert by.value <= nb.value, shape
                        if tpw.value:
                            check_tile(fmt, B, T, S, tpw.value, rs.value, by.value)
                        else:
                            assert rs.value == 0 and by.value == 0 and form.value != 3, shape
                        if form.value == 0:
                            assert tokens == 0, shape
                        if nb.value == 0:
                            assert form.value in (0, 1, 2), shape       # nothing that needs a workspace
    assert all(seen.get(f, 0) > 100 for f in (0, 1, 2, 3, 4)), seen    # the grid reaches every form


def test_module_surface_matches_reference_names_and_shapes():
    m = lookupffn_amd.LookupFFN(_config(hidden_size=768, ffn_num_table=128, block_size=64), 768)
    sd = m.state_dict()
    assert set(sd) == {"LayerNorm.weight", "LayerNorm.bias", "hash.projection.weight",
                       "hash.projection.bias", "tables", "bias"}
    assert tuple(sd["tables"].shape) == (128, 256, 768)
    assert tuple(sd["bias"].shape) == (768,)
    # D = 1024, R = ceil(128*8/1024) = 1, 4 stages, 16 blocks of 64x64  (PL/lookup.py:18-23)
    assert tuple(sd["hash.projection.weight"].shape) == (1, 4, 16, 64, 64)
    assert tuple(sd["hash.projection.bias"].shape) == (1024,)
    assert m.hash.code_length == 8 and m.hash.total_dim == 1024
    p = m.hash.projection
    assert (p.padded_in_dim, p.num_repeat, p.num_block, p.decay_coeff) == (1024, 1, 16, 0.7)
    big = lookupffn_amd.BH4(1024, 4096, 1)
    assert big.num_repeat == 4 and tuple(big.weight.shape) == (4, 4, 1024, 1, 1)


def test_dense_projection_and_bad_projection_type():
    m = lookupffn_amd.Hashing(_config(projection_type="dense"))
    assert isinstance(m.projection, torch.nn.Linear)
    with pytest.raises(NotImplementedError):
        lookupffn_amd.Hashing(_config(projection_type="other"))
    with pytest.raises(AssertionError):
        lookupffn_amd.LookupFFN(_config(ffn_table_size=100), 64)       # PL/lookup.py:88


def test_cpu_tensors_fail_loudly():
    m = lookupffn_amd.LookupFFN(_config(), 64).eval()
    with pytest.raises(RuntimeError, match="GPU only"):
        m(torch.randn(3, 48))
    with pytest.raises(RuntimeError, match="GPU only"):
        lookupffn_amd.gather(torch.zeros(2, 2, dtype=torch.int32), torch.ones(2, 2), torch.ones(4, 64), False)
    with pytest.raises(RuntimeError, match="GPU only"):
        lookupffn_amd.compute_code_score(torch.randn(2, 3, 8), False)
    with pytest.raises((RuntimeError, NotImplementedError)):
        lookupffn_amd.hadamard(torch.randn(2, 8))       # no CPU kernel registered for the op


def test_slow_torch_hooks_match_closed_forms():
    # use_torch=True keeps the reference's slow formulas; they run on any device
    import scipy.linalg
    x = torch.randn(3, 16, dtype=torch.float64)
    want = x @ torch.tensor(scipy.linalg.hadamard(16), dtype=torch.float64)
    assert torch.allclose(lookupffn_amd.hadamard(x, use_torch=True), want)
    z = torch.tensor([[[1.0, -1, 1, -1, 0, 2, -3, 4]]])
    code, score = lookupffn_amd.compute_code_score_torch(z)
    assert code.item() == 0b10100101
    idx = torch.tensor([[0, 3], [2, 2]], dtype=torch.int32)
    src = torch.arange(4 * 64, dtype=torch.float32).reshape(4, 64)
    w = torch.tensor([[1.0, 2.0], [0.5, 0.5]])
    out = lookupffn_amd.weighted_gather_add(idx, src, w, use_torch=True)
    assert torch.equal(out[0], src[0] + 2 * src[3]) and torch.equal(out[1], src[2])


def test_ops_have_fake_implementations():
    # shape inference without a device (meta tensors)
    x = torch.empty(5, 48, device="meta")
    diag = torch.empty(1, 4, 64, device="meta")
    c, s, z = torch.ops.lookupffn.project_hash(x, diag, None, 8, 0.7, 0.3, True)
    assert c.shape == (5, 8) and c.dtype == torch.int32 and s.shape == (5, 8) and z.shape == (5, 64)
    t = torch.empty(8, 256, 64, device="meta")
    assert torch.ops.lookupffn.lookup_gather(c, s, t, None).shape == (5, 64)
    assert torch.ops.lookupffn.fht(torch.empty(3, 64, device="meta")).shape == (3, 64)


def _encoder_config(**kw):
    base = dict(hidden_size=64, num_attention_heads=4, attention_head_size=16, attention_probs_dropout_prob=0.1,
                hidden_dropout_prob=0.1, layer_norm_eps=1e-5, num_hidden_layers=2, vocab_size=100,
                max_position_embeddings=32, type_vocab_size=1, pad_token_id=1,
                ffn_num_table=8, ffn_table_size=256, projection_type="bh4", block_size=1)
    base.update(kw)
    return Namespace(**base)


def test_encoder_parameter_names_match_reference():
    # names a reference checkpoint of PL/encoder.py's Lookup model carries (after the
    # "model." prefix is stripped, roberta_to_hf_checkpoint.py:102-111)
    m = lookupffn_amd.Lookup(_encoder_config())
    keys = set(m.state_dict())
    for k in ["embeddings.word_embeddings.weight", "embeddings.position_embeddings.weight",
              "embeddings.token_type_embeddings.weight", "embeddings.LayerNorm.weight",
              "encoder.LayerNorm.bias", "encoder.layer.0.attention.LayerNorm.weight",
              "encoder.layer.0.attention.query.weight", "encoder.layer.0.attention.key.bias",
              "encoder.layer.0.attention.value.weight", "encoder.layer.0.attention.dense.weight",
              "encoder.layer.1.FFN.LayerNorm.weight", "encoder.layer.1.FFN.hash.projection.weight",
              "encoder.layer.1.FFN.hash.projection.bias", "encoder.layer.1.FFN.tables", "encoder.layer.1.FFN.bias"]:
        assert k in keys, k
    assert tuple(m.state_dict()["embeddings.position_embeddings.weight"].shape) == (34, 64)   # max_position + 2
    assert len(keys) == 5 + 2 + 2 * (2 + 8 + 6)


def test_attention_fused_equals_literal_formula_on_cpu():
    # the attention block is plain torch and runs anywhere; the fused evaluation must
    # equal the reference's literal matmul-softmax-matmul (PL/layer.py:55-64)
    torch.manual_seed(0)
    cfg = _encoder_config()
    att = lookupffn_amd.Attention(cfg).eval().double()
    x = torch.randn(3, 10, 64, dtype=torch.float64)
    mask = torch.ones(3, 10)
    mask[1, 7:] = 0
    att.fused = True
    a = att(x, mask)
    att.fused = False
    b = att(x, mask)
    # the module computes attention in float32 whatever the input dtype, as the reference does
    assert torch.allclose(a, b, rtol=1e-5, atol=1e-6)
    emb = lookupffn_amd.RobertaEmbeddings(cfg).eval()
    ids = torch.randint(0, 100, (2, 5))
    pos = torch.arange(5)[None].expand(2, 5)
    out = emb(ids, torch.zeros_like(ids), pos)
    want = torch.nn.functional.layer_norm(
        emb.word_embeddings.weight[ids] + emb.token_type_embeddings.weight[0] + emb.position_embeddings.weight[pos + 2],
        (64,), emb.LayerNorm.weight, emb.LayerNorm.bias, 1e-5)
    assert torch.allclose(out, want, atol=1e-6)
