"""GPU parity: every C-ABI entry point against the CPU oracle on the same seeded
inputs (sizes the oracle finishes in seconds), against the committed golden
fixtures, and at the BASELINE.json shapes through size-independent properties.

Tolerances (stated once, used below):
  * FHT / BH4 mixing: <= 1e-5 of the largest reference magnitude; in fact the
    kernel runs the reference's butterfly order with one rounding per stage, so
    the float32 oracle is matched bit for bit and the tests assert that.
  * codes: bit-exact given identical z.
  * scores and their gradient: <= 2e-6 relative (exp differs by <= 1 ulp).
  * gather-add fp32 and inner product: <= 1e-5 of the largest reference magnitude
    (fused multiply-add vs multiply-then-add).
  * bf16 tables: <= 1e-5 against the oracle on the same bf16 table, <= 1e-2
    against the fp32-table result.
  * scatter-add: <= 1e-5 of the largest magnitude (atomic order is free).
"""
import json
import math
import os

import numpy as np
import pytest
import torch

import oracle

from tests import _cabi as cabi

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _need_gpu():
    assert torch.cuda.is_available(), "GPU tests need an MI355X"
    yield


@pytest.fixture(scope="module")
def golden(golden_dir):
    with open(os.path.join(golden_dir, "lookupffn_golden.json")) as f:
        return json.load(f)


def relmax(got, want):
    want = np.asarray(want, dtype=np.float64)
    scale = max(np.abs(want).max(), 1e-30)
    return float(np.abs(np.asarray(got, dtype=np.float64) - want).max() / scale)


# ----------------------------------------------------------------------------- FHT

def test_fht_golden(golden):
    for D, g in golden["hadamard"].items():
        x = np.array(g["x"], dtype=np.float32)
        assert np.array_equal(cabi.fht(x), np.array(g["xH"], dtype=np.float32))


@pytest.mark.parametrize("D", [4, 8, 16, 32, 64, 128, 256, 512, 1024])
@pytest.mark.parametrize("B", [1, 7, 300])
def test_fht_matches_oracle(B, D):
    rng = np.random.RandomState(B * 10007 + D)
    x = rng.randn(B, D).astype(np.float32)
    want64 = oracle.fht(x.astype(np.float64))
    got = cabi.fht(x)
    assert relmax(got, want64) <= 1e-5
    assert np.array_equal(got, oracle.fht(x))           # same order, one rounding per stage
    assert np.array_equal(cabi.fht_inplace(x), got)


def test_fht_integer_inputs_exact_and_involution():
    rng = np.random.RandomState(5)
    D = 1024
    x = rng.randint(-8, 9, size=(64, D)).astype(np.float32)
    y = cabi.fht(x)
    import scipy.linalg
    assert np.array_equal(y.astype(np.float64), x.astype(np.float64) @ scipy.linalg.hadamard(D))
    assert np.array_equal(cabi.fht(y), D * x)            # H.H = D.I, exact on integers
    e = np.zeros((1, D), np.float32); e[0, 0] = 1
    assert np.array_equal(cabi.fht(e), np.ones((1, D), np.float32))


def test_fht_full_size_properties():
    # BASELINE.json config 2 shape: 16384 x 1024; linearity + Parseval + involution
    rng = np.random.RandomState(6)
    B, D = 16384, 1024
    x = rng.randn(B, D).astype(np.float32)
    y = cabi.fht(x)
    n_in = (x.astype(np.float64) ** 2).sum(1)
    n_out = (y.astype(np.float64) ** 2).sum(1)
    assert np.abs(n_out / (D * n_in) - 1).max() < 1e-5
    assert relmax(cabi.fht(y), D * x.astype(np.float64)) <= 1e-5
    sub = rng.choice(B, 64, replace=False)
    assert np.array_equal(y[sub], oracle.fht(x[sub]))


@pytest.mark.parametrize("D", [4, 16, 64, 256, 512, 1024])
@pytest.mark.parametrize("bf16", [False, True])
def test_fht_16bit_storage(D, bf16):
    """Half / bfloat16 rows: fp32 butterflies, one rounding on the store.  Against the float64
    transform of the same 16-bit inputs the error is that one rounding (2^-11 resp. 2^-8
    relative) plus fp32 rounding of the sums; small integers come out exactly."""
    import scipy.linalg
    rng = np.random.RandomState(D + int(bf16))
    B = 37
    x32 = rng.randn(B, D).astype(np.float32)
    if bf16:
        bits = oracle.bf16_round(x32)
        xin = oracle.bf16_widen(bits).astype(np.float64)
        widen, eps = (lambda b: oracle.bf16_widen(b).astype(np.float64)), 2.0 ** -8
    else:
        h = x32.astype(np.float16)
        bits = h.view(np.uint16)
        xin = h.astype(np.float64)
        widen, eps = (lambda b: b.view(np.float16).astype(np.float64)), 2.0 ** -11
    want = xin @ scipy.linalg.hadamard(D)
    got = widen(cabi.fht16(bits, bf16=bf16))
    scale = np.abs(want).max()
    assert np.all(np.abs(got - want) <= eps * np.abs(want) + 2e-6 * scale)
    assert np.array_equal(widen(cabi.fht16(bits, bf16=bf16, in_place=True)), got)
    # exact on small integers (every sum is representable)
    xi = rng.randint(-2, 3, size=(B, D)).astype(np.float32)
    if D <= 64:
        ib = oracle.bf16_round(xi) if bf16 else xi.astype(np.float16).view(np.uint16)
        assert np.array_equal(widen(cabi.fht16(ib, bf16=bf16)), xi.astype(np.float64) @ scipy.linalg.hadamard(D))


# ----------------------------------------------------------------------------- BH4 diag / projection + hash

@pytest.mark.parametrize("H,D,R,J", [(256, 256, 1, 4), (768, 1024, 1, 4), (1024, 1024, 4, 4), (48, 64, 2, 1),
                                      (100, 128, 1, 3), (6, 8, 1, 2), (511, 512, 2, 4)])
def test_bh4_diag_matches_oracle(H, D, R, J):
    rng = np.random.RandomState(H + D + R)
    B = 37
    x = rng.randn(B, H).astype(np.float32)
    diag = (rng.randn(R, J, D) / math.sqrt(D)).astype(np.float32)
    xp = np.concatenate([x, np.zeros((B, D - H), np.float32)], axis=1)
    want = oracle.bh4(xp, diag.reshape(R, J, D, 1, 1))
    got = cabi.bh4_diag(x, diag)
    assert np.array_equal(got, want)
    want64 = oracle.bh4(xp.astype(np.float64), diag.reshape(R, J, D, 1, 1).astype(np.float64))
    assert relmax(got, want64) <= 1e-5


# (B, H, D, R, J): every block count the kernel is built for (D/64 = 1..16), ragged token counts
# around the 32-token tile, zero padding H < D, several repeats, stage counts other than 4
BH4_BLOCK_CASES = [(37, 256, 256, 1, 4), (100, 768, 1024, 1, 4), (33, 1024, 1024, 4, 4), (1, 64, 64, 2, 4),
                   (64, 100, 128, 1, 3), (31, 512, 512, 2, 1), (0, 64, 64, 1, 4)]


@pytest.mark.parametrize("B,H,D,R,J", BH4_BLOCK_CASES)
def test_bh4_block_matches_oracle(B, H, D, R, J):
    import scipy.linalg
    rng = np.random.RandomState(B + H + D + R + J)
    NB = D // 64
    x = rng.randn(B, H).astype(np.float32)
    w = (rng.randn(R, J, NB, 64, 64) / math.sqrt(64 * D)).astype(np.float32)     # PL/lookup.py:22-23
    got, folded = cabi.bh4_block(x, w)
    # the folded weights are H_64 applied down the output index, exact up to fp32 rounding, stored
    # per block as [o/16][(i%16)/4][i/16][o%16][i%4]
    want_f = np.einsum("po,rjnoi->rjnpi", scipy.linalg.hadamard(64).astype(np.float64), w.astype(np.float64))
    unpacked = folded.reshape(R, J, NB, 4, 4, 4, 16, 4).transpose(0, 1, 2, 3, 6, 5, 4, 7).reshape(R, J, NB, 64, 64)
    assert relmax(unpacked, want_f) <= 1e-6
    if B == 0:
        assert got.shape == (0, R * D)
        return
    assert not np.isnan(got).any()
    xp = np.concatenate([x, np.zeros((B, D - H), np.float32)], axis=1)
    want64 = oracle.bh4(xp.astype(np.float64), w.astype(np.float64))
    assert relmax(got, want64) <= 1e-5
    # no further from the truth than the reference's own order of operations in fp32 (x3)
    ref32 = oracle.bh4(xp, w)
    assert relmax(got, want64) <= max(3 * relmax(ref32, want64), 2e-6)


def test_bh4_block_exact_on_integers():
    # identity blocks scaled by powers of two: every product and sum is exact, so the result is
    # the plain transform applied J times, bit for bit
    import scipy.linalg
    rng = np.random.RandomState(12)
    B, D, J = 40, 512, 2
    NB = D // 64
    x = rng.randint(-4, 5, size=(B, D)).astype(np.float32)
    w = np.zeros((1, J, NB, 64, 64), np.float32)
    for j in range(J):
        for n in range(NB):
            w[0, j, n] = np.eye(64, dtype=np.float32)[rng.permutation(64)] * (2.0 ** rng.randint(-2, 1))
    got, _ = cabi.bh4_block(x, w)
    want = x.astype(np.float64)
    for j in range(J):
        want = np.einsum("bni,noi->bno", want.reshape(B, NB, 64), w[0, j].astype(np.float64)).reshape(B, D)
        want = want @ scipy.linalg.hadamard(D)
    assert np.array_equal(got.astype(np.float64), want)


@pytest.mark.parametrize("B,H,D,R,T,k", [(50, 768, 1024, 1, 128, 8), (33, 1024, 1024, 4, 512, 8), (20, 100, 128, 2, 30, 8),
                                          (17, 256, 256, 1, 21, 12), (9, 64, 64, 3, 48, 4), (5, 30, 32, 1, 3, 7),
                                          (0, 64, 64, 1, 8, 8)])
def test_mix_code_score_matches_oracle(B, H, D, R, T, k):
    rng = np.random.RandomState(B + H + D + R + T + k)
    y = rng.randn(B, R * D).astype(np.float32)
    x = rng.randn(B, H).astype(np.float32)
    bias = (0.05 * rng.randn(T * k)).astype(np.float32)
    codes, scores = cabi.mix_code_score(y, x, bias, T, k, D)
    if B == 0:
        assert codes.shape == (0, T)
        return
    xp = np.concatenate([x, np.zeros((B, D - H), np.float32)], axis=1)
    # PL/lookup.py:36-37 in fp32, operation by operation
    z = (np.float32(0.7) * y + np.float32(1 - 0.7) * np.tile(xp, (1, R)))[:, :T * k] + bias
    want_c, want_s = oracle.code_score(z.reshape(B, T, k))
    assert np.array_equal(codes, want_c)
    np.testing.assert_allclose(scores, want_s, rtol=2e-6)
    # without bias
    codes0, scores0 = cabi.mix_code_score(y, x, None, T, k, D)
    z0 = (np.float32(0.7) * y + np.float32(1 - 0.7) * np.tile(xp, (1, R)))[:, :T * k]
    want_c0, want_s0 = oracle.code_score(z0.reshape(B, T, k))
    assert np.array_equal(codes0, want_c0)
    np.testing.assert_allclose(scores0, want_s0, rtol=2e-6)


@pytest.mark.parametrize("B,H,D,R,T,with_ln", [(100, 768, 1024, 1, 128, True), (70, 1024, 1024, 4, 512, True),
                                                (45, 256, 256, 1, 32, False), (33, 100, 128, 2, 30, True),
                                                (64, 512, 512, 2, 100, False), (1, 64, 64, 1, 8, True),
                                                (0, 64, 64, 1, 8, True)])
def test_ln_bh4_block_hash_matches_oracle(B, H, D, R, T, with_ln):
    """(LayerNorm ->) BH4 with 64 x 64 blocks -> mix -> hash in one kernel, against the float64
    oracle: y is rounded differently from the reference's order (1e-5), so a code may differ
    only where the true z is that close to 0; scores are compared where the codes agree."""
    rng = np.random.RandomState(B + H + D + R + T)
    J, NB = 4, D // 64
    x = (rng.randn(B, H) * 1.5 + 0.3).astype(np.float32)
    ln_w = (1 + 0.1 * rng.randn(H)).astype(np.float32) if with_ln else None
    ln_b = (0.1 * rng.randn(H)).astype(np.float32) if with_ln else None
    w = (rng.randn(R, J, NB, 64, 64) / math.sqrt(64 * D)).astype(np.float32)
    bias = (0.05 * rng.randn(T * 8)).astype(np.float32)
    codes, scores = cabi.ln_bh4_block_hash(x, ln_w, ln_b, 1e-5, w, bias, T)
    if B == 0:
        assert codes.shape == (0, T)
        return
    h64 = oracle.layernorm(x.astype(np.float64), ln_w, ln_b, 1e-5) if with_ln else x.astype(np.float64)
    z64 = oracle.projection(h64, w.astype(np.float64), bias.astype(np.float64), T * 8, 0.7).reshape(B, T, 8)
    code64, score64 = oracle.code_score(z64)
    scale = np.abs(z64).max()
    assert (codes >= 0).all() and not np.isnan(scores).any()          # every entry written
    same = codes == code64
    assert same.mean() >= 0.995
    # where a code differs, some z of that group is within rounding of zero
    assert np.all(np.abs(z64[~same]).min(axis=-1) <= 2e-5 * scale)
    np.testing.assert_allclose(scores[same], score64[same], rtol=3e-4)
    # the same codes and scores as the three-step path on the GPU (LayerNorm in torch, the BH4
    # kernel, the mix + hash kernel) wherever those codes agree with the truth
    if with_ln:
        h_gpu = torch.nn.functional.layer_norm(torch.tensor(x, device="cuda:0"), (H,),
                                               torch.tensor(ln_w, device="cuda:0"),
                                               torch.tensor(ln_b, device="cuda:0"), 1e-5).cpu().numpy()
    else:
        h_gpu = x
    y, _ = cabi.bh4_block(h_gpu, w)
    c3, s3 = cabi.mix_code_score(y, h_gpu, bias, T, 8, D)
    both = same & (c3 == code64)
    np.testing.assert_allclose(scores[both], s3[both], rtol=1e-4)
    if not with_ln:
        # identical inputs to the identical operations: bit for bit
        assert np.array_equal(codes, c3) and np.array_equal(scores, s3)


def test_bh4_fold_modes():
    import scipy.linalg
    rng = np.random.RandomState(77)
    w = rng.randn(3, 2, 64, 64).astype(np.float32)
    want = np.einsum("po,rnoi->rnpi", scipy.linalg.hadamard(64).astype(np.float64), w.astype(np.float64))
    f0 = cabi.bh4_fold_mode(w, 0).reshape(3, 2, 4, 4, 4, 16, 4).transpose(0, 1, 2, 5, 4, 3, 6).reshape(3, 2, 64, 64)
    assert relmax(f0, want) <= 1e-6                        # [o/16][(i%16)/4][i/16][o%16][i%4]
    f1 = cabi.bh4_fold_mode(w, 1).reshape(3, 2, 4, 4, 4, 16, 4)      # [i/16][(o%16)/4][o/16][i%16][o%4]
    f1 = f1.transpose(0, 1, 4, 3, 6, 2, 5).reshape(3, 2, 64, 64)     # -> [o/16, (o%16)/4, o%4][i/16, i%16]
    assert relmax(f1, want) <= 1e-6
    assert relmax(cabi.bh4_fold_mode(w, 2), want) <= 1e-6


@pytest.mark.parametrize("B,H,D,R,T", [(70, 768, 1024, 1, 128), (33, 256, 256, 2, 64), (40, 500, 512, 1, 64),
                                        (17, 64, 64, 1, 8), (50, 1024, 1024, 4, 512)])
def test_bh4_block_training_kernels_match_float64(B, H, D, R, T):
    """Forward with saved stage inputs, and the backward kernel, against the chain written out in
    float64: u_{s+1} = (W_s u_s) H_D per block; backwards q = G H_D, G <- W_s^T q."""
    import scipy.linalg
    rng = np.random.RandomState(B + H + D + R + T)
    J, NB = 4, D // 64
    x = rng.randn(B, H).astype(np.float32)
    w = (rng.randn(R, J, NB, 64, 64) / math.sqrt(64 * D)).astype(np.float32)
    bias = (0.05 * rng.randn(T * 8)).astype(np.float32)
    codes, scores, z, stage_in = cabi.bh4_block_train(x, w, bias, T)
    HD = scipy.linalg.hadamard(D).astype(np.float64)
    HN = scipy.linalg.hadamard(NB).astype(np.float64) if NB > 1 else np.ones((1, 1))
    xp = np.concatenate([x.astype(np.float64), np.zeros((B, D - H))], axis=1)
    w64 = w.astype(np.float64)
    us = np.zeros((R, J + 1, B, D))
    for r in range(R):
        us[r, 0] = xp
        for j in range(J):
            v = np.einsum("bni,noi->bno", us[r, j].reshape(B, NB, 64), w64[r, j]).reshape(B, D)
            us[r, j + 1] = v @ HD
    z64 = (0.7 * np.concatenate([us[r, J] for r in range(R)], axis=1) + 0.3 * np.tile(xp, (1, R)))[:, :T * 8] + bias
    scale = np.abs(z64).max()
    assert np.abs(z - z64).max() <= 1e-5 * scale
    for r in range(R):
        for j in range(1, J):
            assert relmax(stage_in[r, j - 1], us[r, j]) <= 1e-5
    # the codes and scores of the kernel's own z, exactly
    code_z, score_z = oracle.code_score(z.reshape(B, T, 8))
    assert np.array_equal(codes, code_z)
    np.testing.assert_allclose(scores, score_z, rtol=2e-6)
    # same codes and scores as the inference form
    c2, s2 = cabi.ln_bh4_block_hash(x, None, None, 0.0, w, bias, T)
    assert np.array_equal(codes, c2) and np.array_equal(scores, s2)

    g_z = rng.randn(B, T * 8).astype(np.float32)
    g_x, stage_g = cabi.bh4_block_bwd(g_z, w, H)
    gzp = np.concatenate([g_z.astype(np.float64), np.zeros((B, R * D - T * 8))], axis=1)
    for r in range(R):
        G = 0.7 * gzp[:, r * D:(r + 1) * D]
        for j in range(J - 1, -1, -1):
            P = np.einsum("mn,bno->bmo", HN, G.reshape(B, NB, 64)).reshape(B, D)
            assert relmax(stage_g[r, j], P) <= 1e-5, (r, j)
            q = G @ HD
            G = np.einsum("bno,noi->bni", q.reshape(B, NB, 64), w64[r, j]).reshape(B, D)
        want_x = G[:, :H] + 0.3 * gzp[:, r * D:r * D + H]
        assert relmax(g_x[r], want_x) <= 1e-5, r


@pytest.mark.parametrize("B,H,D,R,T", [(70, 768, 1024, 1, 128), (33, 256, 256, 2, 64), (600, 500, 512, 1, 64)])
def test_ln_bh4_block_training_kernels(B, H, D, R, T):
    """LayerNorm inside the training forward (lffn_ln_bh4_block_hash_train_f32) and formed again on load in the
    weight gradient (lffn_ln_bh4_block_wgrad_f32): against the same kernels without LayerNorm fed the normalised rows."""
    rng = np.random.RandomState(B + H + T)
    J, bs = 4, 64
    x = (rng.randn(B, H) * 1.5 + 0.3).astype(np.float32)
    ln_w = (1 + 0.1 * rng.randn(H)).astype(np.float32)
    ln_b = (0.1 * rng.randn(H)).astype(np.float32)
    w = (rng.randn(R, J, D // bs, bs, bs) / math.sqrt(bs * D)).astype(np.float32)
    bias = (0.05 * rng.randn(T * 8)).astype(np.float32)
    codes, scores, z, st, stats = cabi.ln_bh4_block_train(x, ln_w, ln_b, 1e-5, w, bias, T)
    # the rows' statistics against float64
    x64 = x.astype(np.float64)
    mean, var = x64.mean(1), x64.var(1)
    np.testing.assert_allclose(stats[:, 0], mean, rtol=0, atol=1e-6 * np.abs(x).max())
    np.testing.assert_allclose(stats[:, 1], 1 / np.sqrt(var + 1e-5), rtol=2e-6)
    # LayerNorm from the kernel's own statistics, its operations in fp32: the rows the kernel multiplied
    h = ((x - stats[:, :1]) * stats[:, 1:2] * ln_w + ln_b).astype(np.float32)
    assert relmax(h, oracle.layernorm(x64, ln_w, ln_b, 1e-5)) <= 1e-5
    # the same kernel without LayerNorm on those rows: the same codes, scores, z and stage inputs
    codes2, scores2, z2, st2 = cabi.bh4_block_train(h, w, bias, T)
    assert np.array_equal(z, z2) and np.array_equal(codes, codes2) and np.array_equal(scores, scores2)
    assert np.array_equal(st, st2)
    # the hash form used for inference runs the same LayerNorm: the same codes
    codes3, scores3 = cabi.ln_bh4_block_hash(x, ln_w, ln_b, 1e-5, w, bias, T)
    assert np.array_equal(codes, codes3) and np.array_equal(scores, scores3)
    # weight gradient: LayerNorm on load against the plain kernel on the normalised rows
    sg = rng.randn(R * J, B, D).astype(np.float32)
    g_ln = cabi.ln_bh4_block_wgrad(sg, x, ln_w, ln_b, stats, st.reshape(R, J - 1, B, D), R, J)
    g_plain = cabi.bh4_block_wgrad(sg, h, st.reshape(R, J - 1, B, D), R, J)
    assert relmax(g_ln, g_plain) <= 1e-5


@pytest.mark.parametrize("B,H,D,R,J", [(1000, 1024, 1024, 1, 2), (515, 768, 1024, 2, 2), (70, 100, 256, 1, 3),
                                       (2050, 512, 512, 1, 1), (3, 64, 64, 2, 1), (0, 64, 64, 1, 2)])
def test_bh4_block_wgrad_matches_float64(B, H, D, R, J):
    rng = np.random.RandomState(B + D + H)
    NB = D // 64
    sg = rng.randn(R * J, B, D).astype(np.float32)
    x = rng.randn(B, H).astype(np.float32)
    si = rng.randn(R, max(J - 1, 1), B, D).astype(np.float32)[:, :J - 1]
    xp = np.concatenate([x.astype(np.float64), np.zeros((B, D - H))], axis=1)
    want = np.stack([np.einsum("bno,bni->noi", sg[r * J + j].astype(np.float64).reshape(B, NB, 64),
                               (xp if j == 0 else si[r, j - 1].astype(np.float64)).reshape(B, NB, 64))
                     for r in range(R) for j in range(J)])
    got = cabi.bh4_block_wgrad(sg, x, np.ascontiguousarray(si), R, J)
    if B == 0:
        assert not got.any()
        return
    assert relmax(got, want) <= 1e-5
    init = rng.randn(R * J, NB, 64, 64).astype(np.float32)
    assert relmax(cabi.bh4_block_wgrad(sg, x, np.ascontiguousarray(si), R, J, init=init), want + init) <= 1e-5   # accumulates


# (B, H, D, R, J, T, Do): the whole layer in one launch; ragged token counts around the four tokens
# of a workgroup, H < D, several repeats, table counts around the eight loads in flight, output
# widths below, at and above the 256 columns of a pass
FUSED_LAYER_CASES = [(256, 256, 256, 1, 4, 32, 256), (5, 200, 256, 1, 4, 30, 64), (131, 768, 1024, 1, 4, 128, 768),
                     (9, 512, 512, 2, 3, 100, 260), (1, 300, 512, 1, 1, 7, 4)]


@pytest.mark.parametrize("B,H,D,R,J,T,Do", FUSED_LAYER_CASES)
@pytest.mark.parametrize("with_ln", [True, False])
def test_lookup_ffn_fused_matches_the_two_kernel_form(B, H, D, R, J, T, Do, with_ln):
    rng = np.random.RandomState(B + H + T + Do)
    S = 256
    x = rng.randn(B, H).astype(np.float32)
    ln_w = (1.0 + 0.1 * rng.randn(H)).astype(np.float32) if with_ln else None
    ln_b = (0.1 * rng.randn(H)).astype(np.float32) if with_ln else None
    diag = (rng.choice([-1.0, 1.0], size=(R, J, D)) / np.sqrt(D)).astype(np.float32)
    pbias = (0.01 * rng.randn(T * 8)).astype(np.float32)
    tables = (0.02 * rng.randn(T, S, Do)).astype(np.float32)
    obias = (0.001 * rng.randn(Do)).astype(np.float32)
    res = rng.randn(B, Do).astype(np.float32)
    if with_ln:
        code, score, _ = cabi.ln_project_hash(x, ln_w, ln_b, 1e-5, diag, pbias, T)
    else:
        code, score, _ = cabi.project_hash(x, diag, pbias, T)
    idx = code + (np.arange(T, dtype=np.int32) * S)[None]
    want = oracle.gather_add(idx, tables.reshape(T * S, Do).astype(np.float64), score.astype(np.float64))
    got = cabi.lookup_ffn_fused(x, ln_w, ln_b, 1e-5, diag, pbias, tables, obias, res)
    assert not np.isnan(got).any()
    assert relmax(got, want + obias + res) <= 1e-5       # same codes and scores (same kernel body), fp32 row sums
    # the same call with the parameters handed over in a struct lffn_fused_layer
    assert np.array_equal(got, cabi.lookup_ffn_fused_layer(x, ln_w, ln_b, 1e-5, diag, pbias, tables, obias, res))
    got = cabi.lookup_ffn_fused(x, ln_w, ln_b, 1e-5, diag, None, tables, None, None)
    if with_ln:
        code, score, _ = cabi.ln_project_hash(x, ln_w, ln_b, 1e-5, diag, np.zeros(T * 8, np.float32), T)
    else:
        code, score, _ = cabi.project_hash(x, diag, np.zeros(T * 8, np.float32), T)
    idx = code + (np.arange(T, dtype=np.int32) * S)[None]
    want = oracle.gather_add(idx, tables.reshape(T * S, Do).astype(np.float64), score.astype(np.float64))
    assert relmax(got, want) <= 1e-5


@pytest.mark.parametrize("B,H,R", [(1000, 768, 1), (37, 1024, 4), (5, 4, 1), (300, 260, 2), (0, 64, 1), (64, 512, 1)])
@pytest.mark.parametrize("affine", [True, False])
def test_layer_norm_bwd_matches_float64(B, H, R, affine):
    rng = np.random.RandomState(B + H + R)
    x = (rng.randn(B, H) * 2 + 0.5).astype(np.float32)
    w = (1 + 0.2 * rng.randn(H)).astype(np.float32) if affine else None
    gy = rng.randn(R, B, H).astype(np.float32)
    eps = 1e-5
    x64, g = x.astype(np.float64), gy.astype(np.float64).sum(0)
    mean = x64.mean(1, keepdims=True)
    rstd = 1.0 / np.sqrt(x64.var(1, keepdims=True) + eps)
    xh = (x64 - mean) * rstd
    gw = g * (w.astype(np.float64) if affine else 1.0)
    want_x = rstd * (gw - gw.mean(1, keepdims=True) - xh * (gw * xh).mean(1, keepdims=True))
    got_x, got_w, got_b = cabi.layer_norm_bwd(x, w, eps, gy)
    if B == 0:
        assert not got_w.any() and not got_b.any()
        return
    assert relmax(got_x, want_x) <= 2e-5
    assert relmax(got_w, (g * xh).sum(0)) <= 2e-5
    assert relmax(got_b, g.sum(0)) <= 2e-5


def test_sign_diagonal_fht_exact():
    # the BASELINE.json "random +-1 sign diagonal from seed": one round, exact on integers
    rng = np.random.RandomState(8)
    B, D = 33, 1024
    x = rng.randint(-8, 9, size=(B, D)).astype(np.float32)
    s = (2 * rng.randint(0, 2, size=(1, 1, D)) - 1).astype(np.float32)
    import scipy.linalg
    want = (x * s[0, 0]).astype(np.float64) @ scipy.linalg.hadamard(D)
    assert np.array_equal(cabi.bh4_diag(x, s).astype(np.float64), want)


@pytest.mark.parametrize("H,D,R,T", [(256, 256, 1, 32), (768, 1024, 1, 128), (1024, 1024, 4, 512),
                                      (48, 64, 1, 5), (100, 128, 2, 30), (8, 8, 1, 1)])
def test_project_hash_matches_oracle(H, D, R, T):
    rng = np.random.RandomState(H * 3 + T)
    B, J = 41, 4
    x = rng.randn(B, H).astype(np.float32)
    diag = (rng.randn(R, J, D) / math.sqrt(D)).astype(np.float32)
    bias = (0.1 * rng.randn(T * 8)).astype(np.float32)
    z_want = oracle.projection(x, diag.reshape(R, J, D, 1, 1), bias, T * 8, np.float32(0.7))
    code_want, score_want = oracle.code_score(z_want.reshape(B, T, 8))
    codes, scores, z = cabi.project_hash(x, diag, bias, T)
    assert np.array_equal(z, z_want)                      # identical operations in identical order
    assert np.array_equal(codes, code_want)               # so the codes are bit-exact end to end
    np.testing.assert_allclose(scores, score_want, rtol=2e-6, atol=0)
    codes2, scores2, _ = cabi.project_hash(x, diag, bias, T, keep_z=False)
    assert np.array_equal(codes2, codes) and np.array_equal(scores2, scores)
    codes3, _, z3 = cabi.project_hash(x, diag, None, T)
    z_nb = oracle.projection(x, diag.reshape(R, J, D, 1, 1), None, T * 8, np.float32(0.7))
    assert np.array_equal(z3, z_nb) and np.array_equal(codes3, oracle.code_score(z_nb.reshape(B, T, 8))[0])


@pytest.mark.parametrize("H,D,R,T", [(256, 256, 1, 32), (768, 1024, 1, 128), (1024, 1024, 4, 512), (100, 128, 2, 30),
                                      (48, 64, 1, 5), (6, 8, 1, 1)])
def test_ln_project_hash_matches_oracle(H, D, R, T):
    """LayerNorm fused into the projection kernel.  Its sums run in another order than
    the oracle's (and torch's), so h and z agree to rounding: z within 1e-5 of the
    float64 truth, a code may differ only where the true z is within that rounding of 0."""
    rng = np.random.RandomState(H + 7 * T)
    B, J = 300, 4
    x = (rng.randn(B, H) * 1.5 + 0.3).astype(np.float32)
    ln_w = (1 + 0.1 * rng.randn(H)).astype(np.float32)
    ln_b = (0.1 * rng.randn(H)).astype(np.float32)
    diag = ((2 * rng.randint(0, 2, size=(R, J, D)) - 1) / math.sqrt(D)).astype(np.float32)
    bias = (0.05 * rng.randn(T * 8)).astype(np.float32)
    h64 = oracle.layernorm(x.astype(np.float64), ln_w, ln_b, 1e-5)
    z64 = oracle.projection(h64, diag.reshape(R, J, D, 1, 1).astype(np.float64), bias.astype(np.float64), T * 8, 0.7)
    code64, score64 = oracle.code_score(z64.reshape(B, T, 8))
    codes, scores, z = cabi.ln_project_hash(x, ln_w, ln_b, 1e-5, diag, bias, T)
    scale = np.abs(z64).max()
    assert np.abs(z - z64).max() <= 1e-5 * scale
    flipped = (z.reshape(B, T, 8) > 0) != (z64.reshape(B, T, 8) > 0)
    assert np.all(np.abs(z64.reshape(B, T, 8)[flipped]) <= 1e-5 * scale)
    same = codes == code64
    assert same.mean() >= 0.999
    np.testing.assert_allclose(scores[same], score64[same], rtol=2e-4)   # |z| enters the score: 1e-5*scale on z
    # the kernel's own codes and scores are those of its own z, exactly
    code_z, score_z = oracle.code_score(z.reshape(B, T, 8))
    assert np.array_equal(codes, code_z)
    np.testing.assert_allclose(scores, score_z, rtol=2e-6)
    # against the two-kernel path (torch LayerNorm on the GPU, then the projection kernel)
    h_gpu = torch.nn.functional.layer_norm(torch.tensor(x, device="cuda:0"), (H,), torch.tensor(ln_w, device="cuda:0"),
                                           torch.tensor(ln_b, device="cuda:0"), 1e-5).cpu().numpy()
    _, _, z2 = cabi.project_hash(h_gpu, diag, bias, T)
    assert np.abs(z - z2).max() <= 1e-5 * scale


# (B, H, D, R, T, Do, forced plan or None): config 2's layer shape; a token count that ends inside a tile, a
# workgroup of the projection kernel and a quad; two repeats of a short transform (rows shared by four
# tokens per wavefront); an odd number of table pairs
# what lffn_lookup_gather_records_plan picks at configs 2 and 3: (tokens per workgroup, record stride, bytes)
CONFIG2_RECORD_PLAN = (1648, 16480, 6 * 128 * 16480)        # 10 tiles of 103 groups of 16 tokens x 24 slices
CONFIG3_RECORD_PLAN = (2048, 16384, 6 * 512 * 16384)        # 8 tiles x 32 slices
RECORD_LAYERS = [(16384, 768, 1024, 1, 128, 768, None), (4099, 768, 1024, 1, 128, 768, (1024, 5120)),
                 (5000, 100, 128, 2, 30, 128, (1536, 6144)), (2050, 64, 64, 1, 6, 64, (2048, 4096)),
                 # config 3's layer shape (four repeats of the transform, 512 tables, 4 KB rows, 2048-token tiles)
                 (4099, 1024, 1024, 4, 512, 1024, (2048, 6144))]


@pytest.mark.parametrize("B,H,D,R,T,Do,plan", RECORD_LAYERS)
def test_layer_through_the_record_stream_matches_the_two_kernel_form(B, H, D, R, T, Do, plan):
    """lffn_ln_project_hash_records_f32 + lffn_lookup_gather_records_f32: the records hold exactly the codes
    and scores lffn_ln_project_hash_f32 writes, in the layout the gather kernel reads, and the output is
    that of the gather on those codes and scores (bit for bit against the workspace entry point where both
    run the same tile size; against the float64 sum on a sample)."""
    rng = np.random.RandomState(B + H + T)
    S, J = 256, 4
    x = (rng.randn(B, H) * 1.5 + 0.3).astype(np.float32)
    ln_w = (1 + 0.1 * rng.randn(H)).astype(np.float32)
    ln_b = (0.1 * rng.randn(H)).astype(np.float32)
    diag = ((2 * rng.randint(0, 2, size=(R, J, D)) - 1) / math.sqrt(D)).astype(np.float32)
    pbias = (0.05 * rng.randn(T * 8)).astype(np.float32)
    tables = (0.02 * rng.randn(T, S, Do)).astype(np.float32)
    obias = (0.001 * rng.randn(Do)).astype(np.float32)
    res = rng.randn(B, Do).astype(np.float32)
    if plan is None:
        plan = cabi.lookup_gather_records_plan(B, T, S, Do)[:2]
        assert plan == CONFIG2_RECORD_PLAN[:2]
    tokens, stride = plan
    full_plan = (tokens, stride, 6 * T * stride)
    got, rec = cabi.layer_through_records(x, ln_w, ln_b, 1e-5, diag, pbias, tables, obias, residual=res, plan=full_plan)
    assert not np.isnan(got).any()
    codes, scores, _ = cabi.ln_project_hash(x, ln_w, ln_b, 1e-5, diag, pbias, T)
    # the records, word for word
    rec = cabi.records_of_tokens(rec, T, stride, B, tokens)                      # [T/2, B, 3]
    swap = ((np.arange(B) & 2) != 0)[None, :]
    c0, c1 = codes[:, 0::2].T, codes[:, 1::2].T                                  # [T/2, B]
    s0, s1 = scores[:, 0::2].T, scores[:, 1::2].T
    assert np.array_equal(np.ascontiguousarray(rec[:, :, 0]).view(np.float32), np.where(swap, s1, s0))
    assert np.array_equal(np.ascontiguousarray(rec[:, :, 1]).view(np.float32), np.where(swap, s0, s1))
    assert np.array_equal(rec[:, :, 2], np.where(swap, c1 | (c0 << 8), c0 | (c1 << 8)).astype(np.uint32))
    # the output: the same kernel at the same tile size through the workspace entry point, bit for bit
    rc, want_same = cabi.lookup_gather_ws_planned(codes, scores, tables, (3, tokens), bias=obias, residual=res)
    assert rc == 0 and np.array_equal(got, want_same)
    # and the float64 sum over the kernel's own codes and scores, on a sample
    sub = np.unique(np.concatenate([rng.choice(B, 96, replace=False), np.arange(B - 40, B), np.arange(0, 8)]))
    idx = codes[sub] + (np.arange(T, dtype=np.int32) * S)[None]
    want = oracle.gather_add(idx, tables.reshape(T * S, Do).astype(np.float64), scores[sub].astype(np.float64))
    assert relmax(got[sub], want + obias + res[sub]) <= 1e-5


@pytest.mark.parametrize("B,H,D,R,T,Do,tokens", [(4099, 768, 1024, 1, 128, 768, 1024), (2050, 256, 256, 2, 60, 128, 2048),
                                                   (3000, 64, 64, 1, 8, 64, 1536)])
def test_block_layer_through_the_record_stream(B, H, D, R, T, Do, tokens):
    """lffn_ln_bh4_block_hash_records_f32: the records hold the codes and scores lffn_ln_bh4_block_hash_f32
    writes, and the gather from them equals the gather kernel run on those codes and scores."""
    rng = np.random.RandomState(B + H + T + 1)
    S, J, bs = 256, 4, 64
    x = (rng.randn(B, H) * 1.5 + 0.3).astype(np.float32)
    ln_w = (1 + 0.1 * rng.randn(H)).astype(np.float32)
    ln_b = (0.1 * rng.randn(H)).astype(np.float32)
    w = (rng.randn(R, J, D // bs, bs, bs) / math.sqrt(bs * D)).astype(np.float32)
    pbias = (0.05 * rng.randn(T * 8)).astype(np.float32)
    tables = (0.02 * rng.randn(T, S, Do)).astype(np.float32)
    obias = (0.001 * rng.randn(Do)).astype(np.float32)
    wf = cabi.bh4_fold_mode(w, 0).reshape(w.shape)           # the forward fold (what lffn_bh4_fold_f32 writes)
    codes, scores = cabi.ln_bh4_block_hash(x, ln_w, ln_b, 1e-5, w, pbias, T)
    stride = -(-B // tokens) * tokens
    rec = torch.full((3 * (T // 2) * stride,), -1, dtype=torch.int32, device="cuda:0")
    out = torch.full((B, Do), float("nan"), dtype=torch.float32, device="cuda:0")
    d = cabi.dev
    xd, lw, lb, wd, pd, td, od = d(x), d(ln_w), d(ln_b), d(wf), d(pbias), d(tables), d(obias)
    cabi._call("lffn_ln_bh4_block_hash_records_f32", cabi.p(xd), cabi.p(lw), cabi.p(lb), float(np.float32(1e-5)), cabi.p(wd),
               cabi.p(pd), cabi.p(rec), stride, tokens, B, H, D, R, J, T, bs, float(np.float32(0.7)), float(np.float32(1 - 0.7)))
    cabi._call("lffn_lookup_gather_records_f32", cabi.p(rec), stride, cabi.p(td), cabi.p(od), None, cabi.p(out), B, T, S, Do, tokens)
    r = cabi.records_of_tokens(rec.cpu().numpy().view(np.uint32), T, stride, B, tokens)
    swap = ((np.arange(B) & 2) != 0)[None, :]
    c0, c1 = codes[:, 0::2].T, codes[:, 1::2].T
    s0, s1 = scores[:, 0::2].T, scores[:, 1::2].T
    assert np.array_equal(np.ascontiguousarray(r[:, :, 0]).view(np.float32), np.where(swap, s1, s0))
    assert np.array_equal(np.ascontiguousarray(r[:, :, 1]).view(np.float32), np.where(swap, s0, s1))
    assert np.array_equal(r[:, :, 2], np.where(swap, c1 | (c0 << 8), c0 | (c1 << 8)).astype(np.uint32))
    rc, want = cabi.lookup_gather_ws_planned(codes, scores, tables, (3, tokens), bias=obias)
    assert rc == 0 and np.array_equal(cabi.host(out), want)


def test_record_stream_plan_and_refusals():
    from lookupffn_amd import _lib
    lib = _lib.load()
    assert cabi.lookup_gather_records_plan(16384, 128, 256, 768) == CONFIG2_RECORD_PLAN
    assert cabi.lookup_gather_records_plan(16384, 512, 256, 1024) == CONFIG3_RECORD_PLAN
    for shape in ((256, 32, 256, 256), (16384, 128, 128, 768), (16384, 127, 256, 768), (0, 128, 256, 768)):
        assert cabi.lookup_gather_records_plan(*shape) == (0, 0, 0), shape
    # (records, stride, tables, bias, residual, out, B, T, S, Do, tokens): refused before any launch
    bad = lambda *a: lib.lffn_lookup_gather_records_f32(256, *a, None)
    assert bad(4096, 256, None, None, 256, 3000, 20, 256, 256, 1000) == _lib.LFFN_ERR_BAD_ARG            # not whole passes
    assert bad(4096, 256, None, None, 256, 3000, 20, 256, 256, 512) == _lib.LFFN_ERR_UNSUPPORTED         # two passes: not built
    assert bad(4096, 256, None, None, 256, 3000, 21, 256, 256, 1024) == _lib.LFFN_ERR_UNSUPPORTED        # odd T
    assert bad(3008, 256, None, None, 256, 3000, 20, 256, 256, 1024) == _lib.LFFN_ERR_BAD_ARG            # stride short of the last tile
    assert bad(3074, 256, None, None, 256, 3000, 20, 256, 256, 1024) == _lib.LFFN_ERR_BAD_ARG            # stride not a multiple of 4
    assert lib.lffn_lookup_gather_records_f32(260, 4096, 256, None, None, 256, 3000, 20, 256, 256, 1024, None) \
        == _lib.LFFN_ERR_BAD_ARG                                                                         # records not 16-byte aligned
    assert bad(4096, 256, None, None, 256, 3000, 20, 256, 256, 1032) == _lib.LFFN_ERR_BAD_ARG            # not whole groups of 16
    assert bad(8192, 256, None, None, 256, 3000, 20, 256, 256, 2304) == _lib.LFFN_ERR_UNSUPPORTED        # nine passes: not built
    assert bad(2048, 256, None, None, 256, 3000, 20, 256, 256, 1024) == _lib.LFFN_ERR_BAD_ARG            # stride < B
    # (x, ln_w, ln_b, eps, diag, bias, records, stride, tokens per workgroup, B, H, D, R, J, T, ...)
    assert lib.lffn_ln_project_hash_records_f32(256, 256, 256, 1e-5, 256, None, 256, 100, 1024, 300, 64, 64, 1, 4, 6, 0.7, 0.3, None) \
        == _lib.LFFN_ERR_BAD_ARG                                                                         # stride < a tile
    assert lib.lffn_ln_project_hash_records_f32(256, 256, 256, 1e-5, 256, None, 256, 1024, 1024, 300, 64, 64, 1, 4, 5, 0.7, 0.3, None) \
        == _lib.LFFN_ERR_BAD_ARG                                                                         # odd T
    assert lib.lffn_ln_project_hash_records_f32(256, 256, 256, 1e-5, 256, None, 256, 4096, 1000, 300, 64, 64, 1, 4, 6, 0.7, 0.3, None) \
        == _lib.LFFN_ERR_BAD_ARG                                                                         # tile not whole groups of 16
    assert lib.lffn_ln_bh4_block_hash_records_f32(256, 256, 256, 1e-5, 256, None, 256, 1024, 2064, 300, 64, 64, 1, 4, 6, 64, 0.7, 0.3, None) \
        == _lib.LFFN_ERR_BAD_ARG                                                                         # tile beyond 2048


@pytest.mark.parametrize("P,na,nb", [(1, 4, 0), (7, 64, 100), (512, 768, 768), (512, 4096, 1024), (1000, 260, 4),
                                      (129, 0, 72), (16, 8, 0)])
def test_sum_partials_matches_float64(P, na, nb):
    """The column sums of the backward kernels' partial sums: against float64, and bit-identical
    from call to call (fixed order of additions)."""
    rng = np.random.RandomState(P + na + nb)
    a = rng.randn(P, na).astype(np.float32)
    b = rng.randn(P, nb).astype(np.float32) if nb else None
    if na == 0:                                   # the first array may be the empty one
        got_b, _ = cabi.sum_partials(b)
        got_a = np.zeros(0, dtype=np.float32)
    else:
        got_a, got_b = cabi.sum_partials(a, b)
    assert got_a.shape == (na,)
    if na:
        want = a.astype(np.float64).sum(0)
        assert np.abs(got_a - want).max() <= 1e-6 * max(1.0, np.abs(a).sum(0).max())
        again, _ = cabi.sum_partials(a, b)
        assert np.array_equal(again, got_a)
    if nb:
        want = b.astype(np.float64).sum(0)
        assert np.abs(got_b - want).max() <= 1e-6 * max(1.0, np.abs(b).sum(0).max())


@pytest.mark.parametrize("P,n,chunks", [(1000, 68, 4), (16384, 768, 64), (257, 8, 257), (5000, 128, 7)])
def test_sum_partials_in_chunks_and_column_sums(P, n, chunks):
    """chunks > 1: one row of sums per chunk of ceil(P / chunks) consecutive rows (the first pass over
    a gradient with many rows); the package's column_sums strings two passes together."""
    rng = np.random.RandomState(P + n)
    a = rng.randn(P, n).astype(np.float32)
    rows = -(-P // chunks)
    if (chunks - 1) * rows >= P:
        pytest.skip("an empty chunk: rejected by the entry point")
    got, _ = cabi.sum_partials(a, chunks=chunks)
    want = np.stack([a[c * rows:(c + 1) * rows].astype(np.float64).sum(0) for c in range(chunks)])
    assert got.shape == (chunks, n)
    assert np.abs(got - want).max() <= 1e-6 * np.abs(a).sum(0).max()
    from lookupffn_amd import ops
    s = ops.column_sums(torch.tensor(a, device="cuda:0")).cpu().numpy()
    assert np.abs(s - a.astype(np.float64).sum(0)).max() <= 1e-6 * np.abs(a).sum(0).max()


@pytest.mark.parametrize("B,H,D,R,T", [(300, 768, 1024, 1, 128), (70, 256, 256, 2, 64), (33, 500, 512, 1, 40)])
def test_ln_project_hash_bwd_matches_the_backward_on_the_normalised_input(B, H, D, R, T):
    """LayerNorm formed on load inside the projection's backward: the same gradients as the plain
    backward kernel fed with the LayerNorm output (and the z of the forward with LayerNorm inside)."""
    rng = np.random.RandomState(B + H + T)
    J = 4
    x = (rng.randn(B, H) * 1.5 + 0.3).astype(np.float32)
    ln_w = (1 + 0.1 * rng.randn(H)).astype(np.float32)
    ln_b = (0.1 * rng.randn(H)).astype(np.float32)
    diag = (rng.randn(R, J, D) / math.sqrt(D)).astype(np.float32)
    bias = (0.05 * rng.randn(T * 8)).astype(np.float32)
    g_score = rng.randn(B, T).astype(np.float32)
    _, _, z = cabi.ln_project_hash(x, ln_w, ln_b, 1e-5, diag, bias, T)
    h = oracle.layernorm(x.astype(np.float64), ln_w, ln_b, 1e-5).astype(np.float32)
    want = cabi.project_hash_bwd(h, diag, z, g_score)
    got = cabi.project_hash_bwd(x, diag, z, g_score, ln_w, ln_b, 1e-5)
    for g, w in zip(got, want):
        assert g.shape == w.shape and not np.isnan(g).any()
        assert np.abs(g - w).max() <= 2e-5 * np.abs(w).max()


def test_project_hash_near_zero_flip_count():
    # end to end against the float64 truth: flips may only happen where |z| is tiny
    rng = np.random.RandomState(9)
    B, H, D, R, J, T = 2048, 768, 1024, 1, 4, 128
    x = rng.randn(B, H).astype(np.float32)
    diag = ((2 * rng.randint(0, 2, size=(R, J, D)) - 1) / math.sqrt(D)).astype(np.float32)
    codes, _, z = cabi.project_hash(x, diag, None, T)
    z64 = oracle.projection(x.astype(np.float64), diag.reshape(R, J, D, 1, 1).astype(np.float64), None, T * 8, 0.7)
    code64, _ = oracle.code_score(z64.reshape(B, T, 8))
    bits = (z.reshape(B, T, 8) > 0) != (z64.reshape(B, T, 8) > 0)
    flips = int(bits.sum())
    tiny = int((np.abs(z64) < 1e-6).sum())
    print(f"sign flips vs float64 truth: {flips} of {bits.size} (|z| < 1e-6: {tiny})")
    assert np.all(np.abs(z64.reshape(B, T, 8)[bits]) < 1e-5)
    assert (codes != code64).sum() <= flips


# ----------------------------------------------------------------------------- code + score

def test_code_golden(golden):
    z = np.array(golden["codes"]["z"], dtype=np.float32)
    codes, _ = cabi.code_score(z)
    assert np.array_equal(codes, np.array(golden["codes"]["code"], dtype=np.int32))
    for zz, want in zip(golden["score"]["z"], golden["score"]["score"]):
        _, s = cabi.code_score(np.array([zz], dtype=np.float32))
        assert abs(float(s[0]) - want) <= 2e-6 * max(1.0, abs(want))


@pytest.mark.parametrize("k", [1, 2, 3, 4, 7, 8, 11, 12, 16, 24])
def test_code_score_matches_oracle(k):
    rng = np.random.RandomState(k)
    z = rng.randn(257, 13, k).astype(np.float32)
    z[0, 0, : min(k, 3)] = [0.0, -0.0, np.nan][: min(k, 3)]
    code_want, score_want = oracle.code_score(z)
    codes, scores = cabi.code_score(z)
    assert np.array_equal(codes, code_want)
    ok = ~np.isnan(score_want)
    np.testing.assert_allclose(scores[ok], score_want[ok], rtol=2e-6, atol=0)
    assert np.array_equal(np.isnan(scores), np.isnan(score_want))


def test_code_score_bwd_matches_oracle():
    rng = np.random.RandomState(12)
    for k in (3, 4, 8, 12, 16):                       # 4, 8, 12, 16 take the vector kernel
        z = rng.randn(300, 9, k).astype(np.float32)
        z[0, 0, 0] = 0.0
        g = rng.randn(300, 9).astype(np.float32)
        want = oracle.code_score_bwd(z.astype(np.float64), g.astype(np.float64))
        got = cabi.code_score_bwd(z, g)
        np.testing.assert_allclose(got, want, rtol=2e-5, atol=1e-6)


# ----------------------------------------------------------------------------- gather-add

def _rand_gather(rng, B, T, S, Do):
    tables = (0.02 * rng.randn(T, S, Do)).astype(np.float32)
    code = rng.randint(0, S, size=(B, T)).astype(np.int32)
    idx = code + (np.arange(T, dtype=np.int32) * S)[None]
    w = (1.0 - rng.rand(B, T)).astype(np.float32)
    return tables, code, idx, w


def test_gather_golden(golden):
    g = golden["gather"]
    tables = np.array(g["tables"], dtype=np.float32)
    T, S, Do = tables.shape
    code = np.array(g["code"], dtype=np.int32)
    idx = code + (np.arange(T, dtype=np.int32) * S)[None]
    w = np.array(g["w"], dtype=np.float32)
    flat = tables.reshape(T * S, Do)
    want = np.array(g["out"], dtype=np.float32)
    assert np.array_equal(cabi.gather_add(idx, flat, w), want)
    assert np.array_equal(cabi.gather_add(idx, oracle.bf16_round(flat), w, bf16=True), want)
    gout = np.array(g["g_out"], dtype=np.float32)
    assert np.array_equal(cabi.indexed_inner_product(idx, gout, flat), np.array(g["g_w"], dtype=np.float32))
    assert np.array_equal(cabi.scatter_add(idx, gout, w, T * S).reshape(T, S, Do),
                          np.array(g["g_tables"], dtype=np.float32))


# (B, T, S, Do): config 1, ragged token counts, every lanes-per-token / vectors-per-lane tiling,
# index counts that are not multiples of the staging chunk or the unroll
GATHER_CASES = [(256, 32, 256, 256), (1, 2, 4, 64), (5, 6, 16, 128), (67, 10, 8, 192), (33, 130, 4, 768),
                (19, 64, 256, 1024), (9, 4, 8, 320), (130, 66, 16, 512), (3, 2, 2, 1920), (40, 128, 256, 768)]


@pytest.mark.parametrize("B,T,S,Do", GATHER_CASES)
def test_gather_add_matches_oracle(B, T, S, Do):
    rng = np.random.RandomState(B + T + Do)
    tables, code, idx, w = _rand_gather(rng, B, T, S, Do)
    flat = tables.reshape(T * S, Do)
    want64 = oracle.gather_add(idx, flat.astype(np.float64), w.astype(np.float64))
    want32 = oracle.gather_add(idx, flat, w)
    got = cabi.gather_add(idx, flat, w)
    assert relmax(got, want64) <= 1e-5
    assert relmax(got, want32) <= 1e-5
    # arbitrary (not per-table) indices, as the reference's own unit test draws them
    idx_any = rng.randint(0, T * S, size=(B, T)).astype(np.int32)
    assert relmax(cabi.gather_add(idx_any, flat, w), oracle.gather_add(idx_any, flat.astype(np.float64), w.astype(np.float64))) <= 1e-5
    # the layer's form: table-local codes, offset and bias folded in
    bias = (0.001 * rng.randn(Do)).astype(np.float32)
    if S & (S - 1) == 0:
        assert relmax(cabi.lookup_gather(code, w, tables, None), want64) <= 1e-5
        assert relmax(cabi.lookup_gather(code, w, tables, bias), want64 + bias) <= 1e-5


# (B, T, S, Do, bf16): shapes that the planner sends to the token-major kernel (0 tables per
# buffer), the one-table LDS kernel (1) and the two-table LDS kernel (2)
RESIDUAL_CASES = [(300, 20, 256, 256, False, 0), (16384, 8, 256, 768, False, 1), (4000, 12, 256, 768, False, 2),
                  (8192, 16, 256, 768, True, 2), (500, 6, 64, 128, True, 0)]


@pytest.mark.parametrize("B,T,S,Do,bf16,kind", RESIDUAL_CASES)
def test_lookup_gather_residual(B, T, S, Do, bf16, kind):
    assert cabi.lookup_gather_plan(B, T, S, Do, bf16)[0] == kind
    rng = np.random.RandomState(B + T + Do + 5)
    tables, code, idx, w = _rand_gather(rng, B, T, S, Do)
    bias = (0.001 * rng.randn(Do)).astype(np.float32)
    res = rng.randn(B, Do).astype(np.float32)
    tb = oracle.bf16_round(tables.reshape(T * S, Do)).reshape(T, S, Do) if bf16 else tables
    plain = cabi.lookup_gather(code, w, tb, bias, bf16=bf16)
    got = cabi.lookup_gather(code, w, tb, bias, bf16=bf16, residual=res)
    # the residual is one more fp32 addition on top of the plain result, element by element
    assert np.array_equal(got, plain + res)
    # in place: the residual buffer is the output buffer
    assert np.array_equal(cabi.lookup_gather(code, w, tb, bias, bf16=bf16, residual=res, in_place=True), got)
    # and the sum against the float64 oracle
    flat = oracle.bf16_widen(tb.reshape(T * S, Do)) if bf16 else tb.reshape(T * S, Do)
    want = oracle.gather_add(idx, flat.astype(np.float64), w.astype(np.float64)) + bias + res
    assert relmax(got, want) <= 1e-5


@pytest.mark.parametrize("B,T,S,Do", GATHER_CASES)
def test_gather_add_bf16_matches_oracle(B, T, S, Do):
    rng = np.random.RandomState(B + T + Do + 1)
    tables, code, idx, w = _rand_gather(rng, B, T, S, Do)
    flat = tables.reshape(T * S, Do)
    bits = oracle.bf16_round(flat)
    want_bf = oracle.gather_add_bf16(idx, bits, w.astype(np.float64))
    want_f32 = oracle.gather_add(idx, flat.astype(np.float64), w.astype(np.float64))
    got = cabi.gather_add(idx, bits, w, bf16=True)
    assert relmax(got, want_bf) <= 1e-5
    assert relmax(got, want_f32) <= 1e-2
    if S & (S - 1) == 0:
        assert relmax(cabi.lookup_gather(code, w, bits.reshape(T, S, Do), None, bf16=True), want_bf) <= 1e-5


# Every LDS-tiled gather kernel that is built: (tables per buffer, tokens per workgroup).
F32_PLANS = [(1, 256), (1, 512), (1, 832), (1, 1024), (2, 512), (2, 1024), (2, 1664), (2, 2048)]
BF16_PLANS = [(1, 256), (1, 512), (2, 512), (2, 1024)]
# (B, T, S, Do): ragged token counts, table counts that are odd / not multiples of the 8-
# and 16-table chunks, tables smaller than the LDS buffer, one and several token tiles
LDS_SHAPES = [(3000, 20, 256, 256), (4133, 5, 256, 384), (2049, 33, 64, 128), (1000, 17, 256, 128), (5000, 8, 32, 256)]


def _check_lds_gather(B, T, S, Do, bf16, plan):
    rng = np.random.RandomState(B + T + S + Do + 131 * plan[0] + plan[1])
    tables, code, idx, w = _rand_gather(rng, B, T, S, Do)
    bias = (0.001 * rng.randn(Do)).astype(np.float32)
    flat = tables.reshape(T * S, Do)
    src = oracle.bf16_round(flat) if bf16 else flat
    got = cabi.lookup_gather(code, w, src.reshape(T, S, Do), bias, bf16=bf16, plan=plan)
    assert not np.isnan(got).any()
    # a random sample of tokens plus the whole ragged tail
    sub = np.unique(np.concatenate([rng.choice(B, 96, replace=False), np.arange(B - 80, B), np.arange(0, 8)]))
    w64 = w[sub].astype(np.float64)
    if bf16:
        want = oracle.gather_add_bf16(idx[sub], src, w64) + bias
    else:
        want = oracle.gather_add(idx[sub], flat.astype(np.float64), w64) + bias
    assert relmax(got[sub], want) <= 1e-5
    # the LDS-tiled and the token-major kernels agree on every token
    assert relmax(got, cabi.gather_add(idx, src, w, bf16=bf16).astype(np.float64) + bias) <= 2e-6
    # codes are masked into their table: bits above log2(S) are ignored
    dirty = (code + S * rng.randint(0, 5, size=code.shape)).astype(np.int32)
    assert np.array_equal(cabi.lookup_gather(dirty, w, src.reshape(T, S, Do), bias, bf16=bf16, plan=plan), got)
    # no bias
    got_nb = cabi.lookup_gather(code, w, src.reshape(T, S, Do), None, bf16=bf16, plan=plan)
    assert relmax(got_nb[sub], want - bias) <= 1e-5


@pytest.mark.parametrize("bf16", [False, True])
def test_lookup_gather_takes_many_tokens_in_pieces(bf16):
    # from 32768 tokens on (tables that fit the cache) the entry point runs one launch per ~16384 tokens;
    # 40001 tokens: pieces of 20032 and 19969, with a residual and a bias, every token against the oracle
    rng = np.random.RandomState(77)
    B, T, S, Do = 40001, 6, 16, 128
    tables, code, idx, w = _rand_gather(rng, B, T, S, Do)
    bias = (0.001 * rng.randn(Do)).astype(np.float32)
    res = rng.randn(B, Do).astype(np.float32)
    flat = tables.reshape(T * S, Do)
    src = oracle.bf16_round(flat) if bf16 else flat
    got = cabi.lookup_gather(code, w, src.reshape(T, S, Do), bias, bf16=bf16, residual=res)
    if bf16:
        want = oracle.gather_add_bf16(idx, src, w.astype(np.float64))
    else:
        want = oracle.gather_add(idx, flat.astype(np.float64), w.astype(np.float64))
    assert relmax(got, want + bias + res) <= 1e-5


# (B, T, S, Do, bf16): shapes for which the workspace query asks for the table-split form (a few
# thousand tokens, enough tables to split): 2, 4 and 8 parts, ragged token counts, table counts
# that leave a short last part (200 = 64 + 64 + 64 + 8, 120 = 32 + 32 + 32 + 24, 200 = 112 + 88)
SPLIT_SHAPES = [(2048, 128, 256, 768, False), (1024, 128, 256, 768, False), (2500, 96, 256, 768, False),
                (2049, 200, 256, 768, False), (3000, 120, 64, 1024, False), (1500, 128, 64, 512, False),
                (5000, 128, 256, 768, True), (5001, 200, 256, 1024, True)]


@pytest.mark.parametrize("B,T,S,Do,bf16", SPLIT_SHAPES)
def test_lookup_gather_table_split_matches_oracle(B, T, S, Do, bf16):
    rng = np.random.RandomState(B + T + S + Do)
    tables, code, idx, w = _rand_gather(rng, B, T, S, Do)
    bias = (0.001 * rng.randn(Do)).astype(np.float32)
    res = rng.randn(B, Do).astype(np.float32)
    flat = tables.reshape(T * S, Do)
    src = oracle.bf16_round(flat) if bf16 else flat
    nbytes = cabi.lookup_gather_workspace_bytes(B, T, S, Do, bf16)
    assert nbytes > 0 and nbytes % (B * Do * 4) == 0                     # the split form is asked for
    got = cabi.lookup_gather_ws(code, w, src.reshape(T, S, Do), bias, bf16=bf16, residual=res)
    assert not np.isnan(got).any()
    sub = np.unique(np.concatenate([rng.choice(B, 128, replace=False), np.arange(B - 70, B), np.arange(0, 8)]))
    w64 = w[sub].astype(np.float64)
    want = oracle.gather_add_bf16(idx[sub], src, w64) if bf16 else oracle.gather_add(idx[sub], flat.astype(np.float64), w64)
    assert relmax(got[sub], want + bias + res[sub]) <= 1e-5
    # every token against the plain entry point (same rows, sums associated differently)
    plain = cabi.lookup_gather(code, w, src.reshape(T, S, Do), bias, bf16=bf16, residual=res)
    assert relmax(got, plain) <= 2e-6
    assert np.array_equal(got, cabi.lookup_gather_ws(code, w, src.reshape(T, S, Do), bias, bf16=bf16, residual=res))
    # without a workspace the entry point is the plain one
    assert np.array_equal(cabi.lookup_gather_ws(code, w, src.reshape(T, S, Do), bias, bf16=bf16, residual=res, ws_bytes=0), plain)
    # no bias, no residual
    got_nb = cabi.lookup_gather_ws(code, w, src.reshape(T, S, Do), None, bf16=bf16)
    assert relmax(got_nb[sub], want) <= 1e-5


def test_lookup_gather_workspace_query_is_zero_where_the_plain_form_is_as_fast():
    for shape in ((16384, 4, 256, 768), (8, 128, 256, 768), (4096, 16, 256, 768), (0, 4, 16, 64),
                  (16384, 128, 128, 768), (16384, 127, 256, 768)):
        assert cabi.lookup_gather_workspace_bytes(*shape) == 0, shape
    for shape in ((8192, 128, 256, 768), (16384, 4, 256, 768), (16384, 128, 128, 768)):
        assert cabi.lookup_gather_workspace_bytes(*shape, bf16=True) == 0, shape
    for shape in ((8192, 128, 256, 768), (2048, 32, 256, 768), (16384, 128, 128, 768)):     # half rows: token-major there
        assert cabi.lookup_gather_workspace_bytes(*shape, bf16=cabi.ROWS_F16) == 0, shape


# The four-lanes-per-token kernel (form 3), every tile size that is built, forced onto shapes it would not
# be chosen for.  (B, T, 256, Do): token counts that end inside a tile, a wavefront and a quad; 1 to 17
# table pairs; one column slice and several.
QUAD_PLANS = [(3, 1024), (3, 1536), (3, 1792), (3, 2048),
              # tiles whose last pass is short for some or most of a workgroup's wavefronts
              (3, 1648), (3, 784), (3, 2032), (3, 1296), (3, 1280), (3, 1200)]
QUAD_SHAPES = [(3000, 20, 256, 256), (4133, 6, 256, 384), (1793, 34, 256, 128), (1, 2, 256, 64), (2050, 8, 256, 192)]


@pytest.mark.parametrize("plan", QUAD_PLANS)
@pytest.mark.parametrize("B,T,S,Do", QUAD_SHAPES)
def test_lookup_gather_quad_kernels_match_oracle(B, T, S, Do, plan):
    rng = np.random.RandomState(B + T + S + Do + plan[1])
    tables, code, idx, w = _rand_gather(rng, B, T, S, Do)
    bias = (0.001 * rng.randn(Do)).astype(np.float32)
    res = rng.randn(B, Do).astype(np.float32)
    flat = tables.reshape(T * S, Do)
    rc, got = cabi.lookup_gather_ws_planned(code, w, tables, plan, bias=bias)
    assert rc == 0 and not np.isnan(got).any()
    want = oracle.gather_add(idx, flat.astype(np.float64), w.astype(np.float64)) + bias
    assert relmax(got, want) <= 1e-5
    dirty = (code + S * rng.randint(0, 5, size=code.shape)).astype(np.int32)      # bits above log2(S) are ignored
    assert np.array_equal(cabi.lookup_gather_ws_planned(dirty, w, tables, plan, bias=bias)[1], got)
    rc, got_r = cabi.lookup_gather_ws_planned(code, w, tables, plan, residual=res)
    assert rc == 0 and relmax(got_r, want - bias + res) <= 1e-5


# The same kernel on 16-bit rows (bfloat16 and half, fp32 sums): 64-column slices, 1024 tokens per workgroup
QUAD16_SHAPES = [(3000, 20, 256, 256), (4133, 6, 256, 384), (1793, 34, 256, 128), (1, 2, 256, 64), (2050, 8, 256, 192)]


@pytest.mark.parametrize("fmt", [cabi.ROWS_BF16, cabi.ROWS_F16])
@pytest.mark.parametrize("B,T,S,Do", QUAD16_SHAPES)
def test_lookup_gather_quad_kernels_16bit_rows_match_oracle(B, T, S, Do, fmt):
    rng = np.random.RandomState(B + T + S + Do + fmt)
    tables, code, idx, w = _rand_gather(rng, B, T, S, Do)
    bias = (0.001 * rng.randn(Do)).astype(np.float32)
    res = rng.randn(B, Do).astype(np.float32)
    bits, wide = cabi.rows_of(tables, fmt)
    rc, got = cabi.lookup_gather_ws_planned_rows(code, w, bits, fmt, (3, 1024), bias=bias)
    assert rc == 0 and not np.isnan(got).any()
    # the float64 sum over the 16-bit values the kernel reads: fp32 accumulation, 1e-5
    want = oracle.gather_add(idx, wide.reshape(T * S, Do), w.astype(np.float64)) + bias
    assert relmax(got, want) <= 1e-5
    # and 1e-2 against the sum over the fp32 values the rows were rounded from
    assert relmax(got, oracle.gather_add(idx, tables.reshape(T * S, Do).astype(np.float64), w.astype(np.float64)) + bias) <= 1e-2
    # every token against the token-major kernel on the same rows
    tm = cabi.gather_add(idx, bits.reshape(T * S, Do), w, fmt=fmt)
    assert relmax(got, tm.astype(np.float64) + bias) <= 2e-6
    dirty = (code + S * rng.randint(0, 5, size=code.shape)).astype(np.int32)      # bits above log2(S) are ignored
    assert np.array_equal(cabi.lookup_gather_ws_planned_rows(dirty, w, bits, fmt, (3, 1024), bias=bias)[1], got)
    rc, got_r = cabi.lookup_gather_ws_planned_rows(code, w, bits, fmt, (3, 1024), residual=res)
    assert rc == 0 and relmax(got_r, want - bias + res) <= 1e-5
    if fmt == cabi.ROWS_BF16:
        assert relmax(got, oracle.gather_add_bf16(idx, bits.reshape(T * S, Do), w) + bias) <= 1e-5


def test_lookup_gather_quad_16bit_refusals():
    from lookupffn_amd import _lib
    rng = np.random.RandomState(5)
    tables, code, idx, w = _rand_gather(rng, 300, 20, 256, 64)
    for fmt in (cabi.ROWS_BF16, cabi.ROWS_F16):
        bits, _ = cabi.rows_of(tables, fmt)
        assert cabi.lookup_gather_ws_planned_rows(code, w, bits, fmt, (3, 2048))[0] == _lib.LFFN_ERR_UNSUPPORTED   # 8 passes: fp32 rows only
        assert cabi.lookup_gather_ws_planned_rows(code, w, bits, fmt, (3, 1024), ws_bytes=0)[0] == _lib.LFFN_ERR_UNSUPPORTED
        assert cabi.lookup_gather_ws_planned_rows(code, w, bits, 3, (3, 1024))[0] == _lib.LFFN_ERR_BAD_ARG          # no such row format
    half, _ = cabi.rows_of(tables, cabi.ROWS_F16)
    assert cabi.lookup_gather_ws_planned_rows(code, w, half, cabi.ROWS_F16, (1, 256))[0] == _lib.LFFN_ERR_UNSUPPORTED   # not built for half rows
    rc, got = cabi.lookup_gather_ws_planned_rows(code, w, half, cabi.ROWS_F16, (0, 0))
    assert rc == 0 and np.array_equal(got, cabi.gather_add(idx, half.reshape(20 * 256, 64), w, fmt=cabi.ROWS_F16))


def test_lookup_gather_quad_refusals():
    from lookupffn_amd import _lib
    rng = np.random.RandomState(3)
    tables, code, idx, w = _rand_gather(rng, 300, 20, 256, 64)
    assert cabi.lookup_gather_ws_planned(code, w, tables, (3, 512))[0] == _lib.LFFN_ERR_UNSUPPORTED       # two passes: not built
    assert cabi.lookup_gather_ws_planned(code, w, tables, (3, 1000))[0] == _lib.LFFN_ERR_BAD_ARG
    assert cabi.lookup_gather_ws_planned(code, w, tables, (3, 1024), ws_bytes=0)[0] == _lib.LFFN_ERR_UNSUPPORTED   # no room for the records
    assert cabi.lookup_gather_ws_planned(code, w, tables, (3, 1024), ws_bytes=6 * 20 * 300)[0] == _lib.LFFN_ERR_UNSUPPORTED
    assert cabi.lookup_gather_ws_planned(code[:, :19].copy(), w[:, :19].copy(), tables[:19].copy(), (3, 1024))[0] == _lib.LFFN_ERR_UNSUPPORTED   # odd T
    t128 = np.ascontiguousarray(tables[:, :128])
    assert cabi.lookup_gather_ws_planned(code % 128, w, t128, (3, 1024))[0] == _lib.LFFN_ERR_UNSUPPORTED          # S != 256
    # the forms that need no workspace run through this entry point as well
    rc, got = cabi.lookup_gather_ws_planned(code, w, tables, (1, 256))
    assert rc == 0 and np.array_equal(got, cabi.lookup_gather(code, w, tables, plan=(1, 256)))
    # without a workspace argument the planned entry point refuses form 3
    lib = _lib.load()
    assert lib.lffn_lookup_gather_planned_f32(256, 256, 256, None, 256, 3000, 20, 256, 256, 3, 1024, None) == _lib.LFFN_ERR_UNSUPPORTED


# (B, T, S, Do): shapes for which the workspace query asks for the record stream of form 3: config 2,
# a token count that ends inside a tile and a quad, an odd number of table pairs, and several rounds of
# workgroups in one launch
QUAD_WS_SHAPES = [(16384, 128, 256, 768), (16001, 64, 256, 768), (20000, 30, 256, 512), (70001, 16, 256, 768)]


@pytest.mark.parametrize("B,T,S,Do", QUAD_WS_SHAPES)
def test_lookup_gather_record_stream_form_matches_oracle(B, T, S, Do):
    rng = np.random.RandomState(B + T + Do)
    tables, code, idx, w = _rand_gather(rng, B, T, S, Do)
    bias = (0.001 * rng.randn(Do)).astype(np.float32)
    res = rng.randn(B, Do).astype(np.float32)
    flat = tables.reshape(T * S, Do)
    nbytes = cabi.lookup_gather_workspace_bytes(B, T, S, Do)
    assert nbytes > 0 and nbytes % 12 == 0 and nbytes < B * Do * 4           # the record stream, not the table split
    got = cabi.lookup_gather_ws(code, w, tables, bias, residual=res)
    assert not np.isnan(got).any()
    sub = np.unique(np.concatenate([rng.choice(B, 128, replace=False), np.arange(B - 70, B), np.arange(0, 8)]))
    want = oracle.gather_add(idx[sub], flat.astype(np.float64), w[sub].astype(np.float64))
    assert relmax(got[sub], want + bias + res[sub]) <= 1e-5
    # every token against the plain entry point (same rows, the two tables of a pair added in either order)
    plain = cabi.lookup_gather(code, w, tables, bias, residual=res)
    assert relmax(got, plain) <= 2e-6
    # reproducible; a second call may reuse the workspace
    assert np.array_equal(got, cabi.lookup_gather_ws(code, w, tables, bias, residual=res))
    # without a workspace the entry point is the plain one; one that is too small for the batch is used for
    # what it can hold (pieces of a large batch) or not at all
    assert np.array_equal(cabi.lookup_gather_ws(code, w, tables, bias, residual=res, ws_bytes=0), plain)
    assert relmax(cabi.lookup_gather_ws(code, w, tables, bias, residual=res, ws_bytes=nbytes - 16), plain) <= 2e-6
    assert np.array_equal(cabi.lookup_gather_ws(code, w, tables, bias, residual=res, ws_bytes=1024), plain)
    # no bias, no residual
    assert relmax(cabi.lookup_gather_ws(code, w, tables, None)[sub], want) <= 1e-5


@pytest.mark.parametrize("plan", F32_PLANS)
@pytest.mark.parametrize("B,T,S,Do", LDS_SHAPES)
def test_lookup_gather_lds_kernels_match_oracle(B, T, S, Do, plan):
    _check_lds_gather(B, T, S, Do, False, plan)


@pytest.mark.parametrize("plan", BF16_PLANS)
@pytest.mark.parametrize("B,T,S,Do", LDS_SHAPES)
def test_lookup_gather_lds_kernels_bf16_match_oracle(B, T, S, Do, plan):
    _check_lds_gather(B, T, S, Do, True, plan)


def test_lookup_gather_plan_and_planned_entry():
    from lookupffn_amd import _lib
    # what the heuristic picks at the BASELINE.json shapes
    assert cabi.lookup_gather_plan(16384, 128, 256, 768) == (1, 832)            # config 2
    assert cabi.lookup_gather_plan(16384, 512, 256, 1024) == (1, 1024)          # config 3 fp32
    assert cabi.lookup_gather_plan(16384, 512, 256, 1024, bf16=True) == (1, 512)
    assert cabi.lookup_gather_plan(256, 32, 256, 256) == (0, 0)                 # config 1: token-major
    assert cabi.lookup_gather_plan(16384, 128, 512, 768) == (0, 0)              # S > 256
    # every plan the heuristic can return is one of the built kernels
    for B in (1024, 3000, 16384, 100000):
        for T in (4, 32, 128, 512):
            for Do in (64, 256, 768, 1024, 2048):
                for bf in (False, True):
                    kind, tokens = cabi.lookup_gather_plan(B, T, 256, Do, bf16=bf)
                    assert (kind, tokens) == (0, 0) or (kind, tokens) in (BF16_PLANS if bf else F32_PLANS)
    # a kernel that is not built, or a shape it cannot take, is refused before any launch
    lib = _lib.load()
    args = (256, 256, 256, None, 256, 3000, 20, 256, 256)
    assert lib.lffn_lookup_gather_planned_f32(*args, 1, 320, None) == _lib.LFFN_ERR_UNSUPPORTED      # 5 passes: not built
    assert lib.lffn_lookup_gather_planned_f32(*args, 1, 100, None) == _lib.LFFN_ERR_BAD_ARG          # not a multiple of 64
    assert lib.lffn_lookup_gather_planned_f32(*args, 3, 512, None) == _lib.LFFN_ERR_UNSUPPORTED      # two passes: not built
    assert lib.lffn_lookup_gather_planned_f32(*args, 4, 512, None) == _lib.LFFN_ERR_UNSUPPORTED      # no such kernel
    assert lib.lffn_lookup_gather_planned_bf16(*args, 2, 2048, None) == _lib.LFFN_ERR_UNSUPPORTED    # fp32 only
    big_s = (256, 256, 256, None, 256, 3000, 20, 512, 256)
    assert lib.lffn_lookup_gather_planned_f32(*big_s, 1, 512, None) == _lib.LFFN_ERR_UNSUPPORTED     # S > 256


def test_every_gather_form_and_the_inner_product_on_random_shapes():
    """Seeded sweep: every built table-major form (one or two tables per LDS buffer, every tile size,
    fp32 and bf16 rows) forced onto shapes it would not be chosen for (odd table counts, batches that
    end inside a tile or a wavefront, short tables, few tables), plus what the plan picks and the
    inner product, all against the float64 sum."""
    rng = np.random.RandomState(2024)

    def bf16_bits(a):
        u = a.astype(np.float32).view(np.uint32)
        return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)

    for it in range(24):
        bf = it % 3 == 2
        S = int(rng.choice([256, 256, 256, 128, 64, 16]))
        T = int(rng.randint(4, 36))
        Do = int(rng.choice([128, 256, 384, 768])) if bf else int(rng.choice([64, 128, 192, 256, 768]))
        B = int(rng.choice([1, 7, 63, 65, 257, 833, 1000]))
        tables = (0.1 * rng.randn(T, S, Do)).astype(np.float32)
        code = rng.randint(0, S, size=(B, T)).astype(np.int32)
        score = rng.rand(B, T).astype(np.float32)
        bias = (0.01 * rng.randn(Do)).astype(np.float32)
        tb = bf16_bits(tables) if bf else tables
        tv = (tb.astype(np.uint32) << 16).view(np.float32) if bf else tables
        rows = tv[np.arange(T)[None, :], code].astype(np.float64)                  # [B, T, Do]
        want = bias.astype(np.float64) + np.einsum("bt,btd->bd", score.astype(np.float64), rows)
        scale = np.abs(want).max()
        plans = [None]
        for kind in (1, 2):
            cols = (256 if kind == 1 else 128) // (2 if bf else 4)
            if Do % cols == 0:
                plans += [(kind, (64 if kind == 1 else 128) * np_) for np_ in ((4, 8) if bf else (4, 8, 13, 16))]
        for plan in plans:
            got = cabi.lookup_gather(code, score, tb, bias, bf16=bf, plan=plan)
            assert np.abs(got - want).max() <= 1e-5 * scale, (it, bf, B, T, S, Do, plan)
        if not bf:
            g = rng.randn(B, Do).astype(np.float32)
            want_i = np.einsum("bd,btd->bt", g.astype(np.float64), rows)
            got_i = cabi.lookup_inner(code, g, tables)
            assert np.abs(got_i - want_i).max() <= 1e-5 * np.abs(want_i).max(), (it, B, T, S, Do)


def test_four_lane_gather_and_record_layer_on_random_shapes():
    """Seeded sweep: the four-lanes-per-token gather at every tile size on ragged shapes (1 to 39 table
    pairs, token counts around the quad, wavefront, pass and tile boundaries, bias and residual on and
    off), the workspace entry point's own choice, and the layer through the record stream, all against
    float64 sums."""
    rng = np.random.RandomState(4242)
    S = 256
    for it in range(20):
        T = 2 * int(rng.randint(1, 40))
        Do = int(rng.choice([64, 128, 192, 256, 512, 768]))
        B = int(rng.choice([1, 2, 3, 5, 15, 17, 255, 257, 1023, 1025, 1791, 1793, 2047, 2049, 3000]))
        tables = (0.1 * rng.randn(T, S, Do)).astype(np.float32)
        code = rng.randint(0, S, size=(B, T)).astype(np.int32)
        score = rng.rand(B, T).astype(np.float32)
        bias = (0.01 * rng.randn(Do)).astype(np.float32) if rng.rand() < 0.7 else None
        res = rng.randn(B, Do).astype(np.float32) if rng.rand() < 0.5 else None
        want = np.einsum("bt,btd->bd", score.astype(np.float64), tables[np.arange(T)[None, :], code].astype(np.float64))
        want = want + (0 if bias is None else bias) + (0 if res is None else res)
        scale = np.abs(want).max()
        for tok in (1024, 1536, 1792, 2048, 1648, 784, 2032):
            rc, got = cabi.lookup_gather_ws_planned(code, score, tables, (3, tok), bias=bias, residual=res)
            assert rc == 0 and np.abs(got - want).max() <= 1e-5 * scale, (it, B, T, Do, tok)
        got = cabi.lookup_gather_ws(code, score, tables, bias, residual=res)
        assert np.abs(got - want).max() <= 1e-5 * scale, (it, B, T, Do)
    for it in range(8):
        D = int(rng.choice([64, 128, 256, 512, 1024]))
        R = int(rng.choice([1, 2])) if D <= 256 else 1
        H = int(rng.choice([D, D - 4, D // 2 + 4]))
        T = 2 * int(rng.randint(1, R * D // 16 + 1))
        Do = int(rng.choice([64, 128, 256]))
        B = int(rng.choice([1, 3, 5, 31, 33, 257, 1000, 2049]))
        tok = int(rng.choice([1024, 1536, 1792, 2048, 1648, 1008]))
        stride = -(-B // tok) * tok + 256
        x = (rng.randn(B, H) * 1.5 + 0.3).astype(np.float32)
        ln_w = (1 + 0.1 * rng.randn(H)).astype(np.float32)
        ln_b = (0.1 * rng.randn(H)).astype(np.float32)
        diag = ((2 * rng.randint(0, 2, size=(R, 4, D)) - 1) / math.sqrt(D)).astype(np.float32)
        pbias = (0.05 * rng.randn(T * 8)).astype(np.float32)
        tables = (0.1 * rng.randn(T, S, Do)).astype(np.float32)
        obias = (0.01 * rng.randn(Do)).astype(np.float32)
        got, _ = cabi.layer_through_records(x, ln_w, ln_b, 1e-5, diag, pbias, tables, obias, plan=(tok, stride, 6 * T * stride))
        codes, scores, _ = cabi.ln_project_hash(x, ln_w, ln_b, 1e-5, diag, pbias, T)
        want = obias + np.einsum("bt,btd->bd", scores.astype(np.float64), tables[np.arange(T)[None, :], codes].astype(np.float64))
        assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max(), (it, B, H, D, R, T, Do, tok)


def test_inner_product_four_lane_kernel_on_random_shapes():
    """Seeded sweep of lffn_lookup_inner_f32 over shapes that take the four-lanes-per-token kernel (S = 256,
    32 to 69 table pairs, 6 to 21 tiles of 1024 tokens: chunks of 2 or 4 pairs, last chunks of 1 to 3,
    ragged last tiles) against the token-major kernel on every entry and float64 sums on a sample."""
    rng = np.random.RandomState(777)
    S = 256
    for it in range(8):
        T = 2 * int(rng.randint(32, 70))
        Do = int(rng.choice([64, 128, 192]))
        B = int(rng.choice([6000, 7169, 8193, 12000, 16385, 20481]))
        tables = (0.1 * rng.randn(T, S, Do)).astype(np.float32)
        code = rng.randint(0, S, size=(B, T)).astype(np.int32)
        g = rng.randn(B, Do).astype(np.float32)
        got = cabi.lookup_inner(code, g, tables)
        assert not np.isnan(got).any(), (it, B, T, Do)
        idx = code + (np.arange(T, dtype=np.int32) * S)[None]
        flat = tables.reshape(T * S, Do)
        other = cabi.indexed_inner_product(idx, g, flat)
        scale = np.abs(other).max()
        assert np.abs(got.astype(np.float64) - other).max() <= 2e-6 * scale, (it, B, T, Do)
        sub = np.unique(np.concatenate([rng.choice(B, 64, replace=False), np.arange(B - 20, B), np.arange(1020, 1030)]))
        want = oracle.indexed_inner_product(idx[sub], g[sub].astype(np.float64), flat.astype(np.float64))
        assert np.abs(got[sub] - want).max() <= 1e-5 * np.abs(want).max(), (it, B, T, Do)


def test_gather_special_cases():
    rng = np.random.RandomState(30)
    tables, code, idx, w = _rand_gather(rng, 16, 8, 16, 128)
    flat = tables.reshape(-1, 128)
    onehot = np.zeros_like(w); onehot[:, 3] = 1.0
    assert np.array_equal(cabi.gather_add(idx, flat, onehot), flat[idx[:, 3]])
    np.testing.assert_allclose(cabi.gather_add(idx, np.ones_like(flat), w)[:, 5], w.astype(np.float64).sum(1), rtol=1e-6)
    # out-of-range indices are clamped, never dereferenced
    bad = idx.copy(); bad[0, 0] = -5; bad[1, 1] = 10 ** 6
    ref = idx.copy(); ref[0, 0] = 0; ref[1, 1] = flat.shape[0] - 1
    assert np.array_equal(cabi.gather_add(bad, flat, w), cabi.gather_add(ref, flat, w))
    # index count 0: zeros (or the bias)
    empty = cabi.gather_add(np.zeros((4, 0), np.int32), flat, np.zeros((4, 0), np.float32))
    assert np.array_equal(empty, np.zeros((4, 128), np.float32))


def test_gather_full_size_properties():
    # BASELINE.json config 2: 16384 tokens, 128 tables x 256 x 768 fp32
    rng = np.random.RandomState(31)
    B, T, S, Do = 16384, 128, 256, 768
    tables, code, idx, w = _rand_gather(rng, B, T, S, Do)
    flat = tables.reshape(T * S, Do)
    out = cabi.lookup_gather(code, w, tables, None)
    out_flat = cabi.gather_add(idx, flat, w)
    assert relmax(out_flat, out) <= 1e-6
    sub = rng.choice(B, 48, replace=False)
    want = oracle.gather_add(idx[sub], flat.astype(np.float64), w[sub].astype(np.float64))
    assert relmax(out[sub], want) <= 1e-5
    # linearity in the weights: G(a*w1 + w2) = a*G(w1) + G(w2)
    w2 = rng.rand(B, T).astype(np.float32)
    lhs = cabi.lookup_gather(code, (2 * w + w2).astype(np.float32), tables, None)
    rhs = 2 * out.astype(np.float64) + cabi.lookup_gather(code, w2, tables, None)
    assert relmax(lhs, rhs) <= 1e-5
    # checksum: sum_b out[b] = sum_{t,s} (sum_{b: code=s} w) * tables[t,s]
    cnt = np.zeros((T, S), np.float64)
    np.add.at(cnt, (np.broadcast_to(np.arange(T), (B, T)), code), w.astype(np.float64))
    want_sum = np.einsum("ts,tsd->d", cnt, tables.astype(np.float64))
    assert relmax(out.astype(np.float64).sum(0), want_sum) <= 1e-5


# ----------------------------------------------------------------------------- backward

@pytest.mark.parametrize("B,T,S,Do", [(256, 32, 256, 256), (5, 6, 16, 128), (67, 10, 8, 192), (33, 130, 4, 768),
                                      (9, 4, 8, 320), (3, 2, 2, 1920), (19, 64, 256, 1024)])
def test_backward_matches_oracle(B, T, S, Do):
    rng = np.random.RandomState(B + T + Do + 2)
    tables, code, idx, w = _rand_gather(rng, B, T, S, Do)
    flat = tables.reshape(T * S, Do)
    g = rng.randn(B, Do).astype(np.float32)
    want_w = oracle.indexed_inner_product(idx, g.astype(np.float64), flat.astype(np.float64))
    assert relmax(cabi.indexed_inner_product(idx, g, flat), want_w) <= 1e-5
    want_t = oracle.scatter_add(idx, g.astype(np.float64), w.astype(np.float64), T * S)
    got_t = cabi.scatter_add(idx, g, w, T * S)
    assert relmax(got_t, want_t) <= 1e-5
    # accumulates into what is already there
    init = rng.randn(T * S, Do).astype(np.float32)
    assert relmax(cabi.scatter_add(idx, g, w, T * S, init=init), want_t + init) <= 1e-5


@pytest.mark.parametrize("B,T,S,Do", [(256, 32, 256, 256), (5, 6, 16, 128), (67, 10, 8, 192), (33, 130, 4, 768),
                                      (9, 4, 8, 320), (3, 2, 2, 1920), (19, 64, 256, 1024), (70, 2, 4, 64)])
def test_backward_half_inputs_match_oracle(B, T, S, Do):
    """The reduced-precision calls of the backward (gradient rows and table rows in half, the place of
    gather_kernel_fp16.cu:64-184): every product is exact and the sums are fp32, so the results sit within
    1e-5 of the float64 oracle on the same half values (the reference rounds products and sums to half:
    bit parity with it is not defined, its atomics run in no fixed order)."""
    rng = np.random.RandomState(B + T + Do + 5)
    tables, code, idx, w = _rand_gather(rng, B, T, S, Do)
    flat_h = tables.reshape(T * S, Do).astype(np.float16)
    g_h = rng.randn(B, Do).astype(np.float16)
    want_w = oracle.indexed_inner_product(idx, g_h.astype(np.float64), flat_h.astype(np.float64))
    got_w = cabi.indexed_inner_product(idx, g_h.view(np.uint16), flat_h.view(np.uint16))
    assert relmax(got_w, want_w) <= 1e-5
    # the same numbers through the fp32 kernel: the two differ by fp32 summation order at most
    assert relmax(got_w, cabi.indexed_inner_product(idx, g_h.astype(np.float32), flat_h.astype(np.float32))) <= 2e-6
    want_t = oracle.scatter_add(idx, g_h.astype(np.float64), w.astype(np.float64), T * S)
    got_t = cabi.scatter_add(idx, g_h.view(np.uint16), w, T * S)
    assert relmax(got_t, want_t) <= 1e-5
    init = rng.randn(T * S, Do).astype(np.float32)
    assert relmax(cabi.scatter_add(idx, g_h.view(np.uint16), w, T * S, init=init), want_t + init) <= 1e-5
    # small integers: products and sums are exact in fp32 whatever the order, so equality is exact
    gi = rng.randint(-4, 5, size=(B, Do)).astype(np.float16)
    ri = rng.randint(-4, 5, size=(T * S, Do)).astype(np.float16)
    wi = rng.randint(-3, 4, size=(B, T)).astype(np.float32)
    assert np.array_equal(cabi.indexed_inner_product(idx, gi.view(np.uint16), ri.view(np.uint16)),
                          oracle.indexed_inner_product(idx, gi.astype(np.float64), ri.astype(np.float64)))
    assert np.array_equal(cabi.scatter_add(idx, gi.view(np.uint16), wi, T * S),
                          oracle.scatter_add(idx, gi.astype(np.float64), wi.astype(np.float64), T * S))


# (B, T, S, Do): odd table counts, tables smaller than the LDS
# slice, ragged token counts around the 64-token batches and 1024-token strides, and a
# table size (512) that takes the zero-fill + global-atomics path
SCATTER_CASES = [(256, 32, 256, 256), (1, 2, 4, 64), (63, 3, 16, 128), (65, 5, 256, 192), (1025, 7, 8, 64),
                 (2100, 6, 256, 128), (300, 1, 2, 64), (500, 4, 512, 128), (0, 4, 16, 64)]


@pytest.mark.parametrize("B,T,S,Do", SCATTER_CASES)
def test_lookup_scatter_matches_oracle(B, T, S, Do):
    rng = np.random.RandomState(B + T + S + Do)
    tables, code, idx, w = _rand_gather(rng, B, T, S, Do)
    g = rng.randn(B, Do).astype(np.float32)
    want = oracle.scatter_add(idx, g.astype(np.float64), w.astype(np.float64), T * S).reshape(T, S, Do)
    got = cabi.lookup_scatter(code, w, g, S)
    assert not np.isnan(got).any()                      # every row written, touched or not
    assert relmax(got, want) <= 1e-5 if B else np.array_equal(got, np.zeros_like(got))
    # accumulate into an existing buffer
    init = rng.randn(T, S, Do).astype(np.float32)
    assert relmax(cabi.lookup_scatter(code, w, g, S, accumulate=True, init=init), want + init) <= 1e-5
    # codes are masked into their table
    if B:
        dirty = (code + S * rng.randint(0, 4, size=code.shape)).astype(np.int32)
        assert relmax(cabi.lookup_scatter(dirty, w, g, S), want) <= 1e-5


# the sorted form: ragged token counts around the 8-entry steps, the 64-entry batches and the
# per-wavefront pieces, one code only (S = 1: every piece cuts the same bucket), few tokens in
# many codes (most buckets empty), 32-column slices beyond and below the eight XCDs
SORTED_CASES = [(256, 32, 256, 256), (1, 2, 4, 64), (63, 3, 16, 128), (65, 5, 256, 192), (1025, 7, 8, 64),
                (2100, 6, 256, 128), (300, 1, 2, 64), (500, 4, 512, 96), (4099, 3, 1, 32), (7, 2, 512, 32),
                (5000, 9, 64, 352), (16384 + 16384 + 100, 2, 16, 32)]      # the last: three chunks of tokens


@pytest.mark.parametrize("B,T,S,Do", SORTED_CASES)
def test_lookup_scatter_sorted_matches_oracle(B, T, S, Do):
    rng = np.random.RandomState(B + T + S + Do)
    tables, code, idx, w = _rand_gather(rng, B, T, S, Do)
    g = rng.randn(B, Do).astype(np.float32)
    want = oracle.scatter_add(idx, g.astype(np.float64), w.astype(np.float64), T * S).reshape(T, S, Do)
    got = cabi.lookup_scatter_sorted(code, w, g, S)
    assert not np.isnan(got).any()                      # every row written, touched or not
    assert relmax(got, want) <= 1e-5
    assert np.array_equal(got, cabi.lookup_scatter_sorted(code, w, g, S))        # fixed order of additions
    init = rng.randn(T, S, Do).astype(np.float32)
    assert relmax(cabi.lookup_scatter_sorted(code, w, g, S, accumulate=True, init=init), want + init) <= 1e-5
    dirty = (code + S * rng.randint(0, 4, size=code.shape)).astype(np.int32)      # codes are masked into their table
    assert np.array_equal(cabi.lookup_scatter_sorted(dirty, w, g, S), got)


def test_lookup_scatter_sorted_random_shapes():
    # seeded sweep: token counts around the 8-entry steps and the per-wavefront pieces, skewed and
    # uniform codes, one to many 32-column slices
    rng = np.random.RandomState(2024)
    for _ in range(16):
        B = int(rng.choice([1, 7, 8, 9, 63, 64, 65, 511, 513, 1000, 2047, 3001]))
        T = int(rng.randint(1, 8))
        S = int(rng.choice([1, 2, 8, 64, 256, 512]))
        Do = 32 * int(rng.randint(1, 10))
        code = (rng.zipf(1.3, size=(B, T)) % S).astype(np.int32) if rng.rand() < 0.5 else \
            rng.randint(0, S, size=(B, T)).astype(np.int32)
        w = rng.randn(B, T).astype(np.float32)
        g = rng.randn(B, Do).astype(np.float32)
        idx = code + (np.arange(T, dtype=np.int32) * S)[None]
        want = oracle.scatter_add(idx, g.astype(np.float64), w.astype(np.float64), T * S).reshape(T, S, Do)
        got = cabi.lookup_scatter_sorted(code, w, g, S)
        assert not np.isnan(got).any(), (B, T, S, Do)
        assert relmax(got, want) <= 1e-5, (B, T, S, Do)


def test_lookup_scatter_sorted_workspace_query():
    assert cabi.lookup_scatter_workspace_bytes(16384, 128, 256, 768) >= 16384 * 128 * 8
    assert cabi.lookup_scatter_workspace_bytes(1 << 20, 128, 256, 768) == cabi.lookup_scatter_workspace_bytes(16384, 128, 256, 768)
    for shape in ((0, 4, 16, 64), (16, 0, 16, 64), (16, 4, 1024, 64), (16, 4, 16, 48)):
        assert cabi.lookup_scatter_workspace_bytes(*shape) == 0


def test_lookup_scatter_sorted_full_size_zipf():
    # BASELINE.json config 5: config-2 shape, codes Zipf(1.1) over 256 entries (the hottest code takes ~18 % of the tokens)
    rng = np.random.RandomState(41)
    B, T, S, Do = 16384, 128, 256, 768
    p = 1.0 / np.arange(1, S + 1) ** 1.1
    p /= p.sum()
    code = rng.choice(S, size=(B, T), p=p).astype(np.int32)
    w = (1.0 - rng.rand(B, T)).astype(np.float32)
    g = rng.randn(B, Do).astype(np.float32)
    got = cabi.lookup_scatter_sorted(code, w, g, S)
    want_sum = w.astype(np.float64).T @ g.astype(np.float64)
    assert relmax(got.astype(np.float64).sum(1), want_sum) <= 1e-5
    for t in (0, 77, 127):
        want_t = oracle.scatter_add(code[:, t:t + 1], g.astype(np.float64), w[:, t:t + 1].astype(np.float64), S)
        assert relmax(got[t], want_t) <= 1e-5
    assert relmax(got, cabi.lookup_scatter(code, w, g, S)) <= 1e-5                # the LDS form


BACKWARD_CASES = [(256, 32, 256, 256), (65, 5, 256, 192), (4100, 16, 256, 768), (3000, 6, 64, 128), (2050, 3, 512, 64)]


@pytest.mark.parametrize("B,T,S,Do", BACKWARD_CASES)
def test_lookup_backward_matches_oracle_and_the_separate_entry_points(B, T, S, Do):
    """lffn_lookup_backward_f32: both gradients from one call and one workspace, against the float64 oracle and,
    bit for bit, against lffn_lookup_inner_f32 and lffn_lookup_scatter_sorted_f32."""
    rng = np.random.RandomState(B + T + S + Do)
    tables, code, idx, w = _rand_gather(rng, B, T, S, Do)
    g = rng.randn(B, Do).astype(np.float32)
    gs, gt = cabi.lookup_backward(code, w, g, tables)
    assert not np.isnan(gs).any() and not np.isnan(gt).any()
    flat = tables.reshape(T * S, Do)
    assert relmax(gs, oracle.indexed_inner_product(idx, g.astype(np.float64), flat.astype(np.float64))) <= 1e-5
    assert relmax(gt.reshape(T * S, Do), oracle.scatter_add(idx, g.astype(np.float64), w.astype(np.float64), T * S)) <= 1e-5
    assert np.array_equal(gt, cabi.lookup_scatter_sorted(code, w, g, S))
    assert relmax(gs, cabi.lookup_inner(code, g, tables)) <= 2e-6
    # either gradient alone; accumulation into an existing table gradient
    only_s, none_t = cabi.lookup_backward(code, w, g, tables, want=(True, False))
    assert none_t is None and relmax(only_s, gs) <= 2e-6          # (small shapes: the form with atomics, any order)
    none_s, only_t = cabi.lookup_backward(code, w, g, tables, want=(False, True))
    assert none_s is None and np.array_equal(only_t, gt)
    init = rng.randn(T, S, Do).astype(np.float32)
    _, acc = cabi.lookup_backward(code, w, g, tables, accumulate=True, init=init)
    assert np.array_equal(acc, cabi.lookup_scatter_sorted(code, w, g, S, accumulate=True, init=init))


def test_lookup_backward_full_size_zipf():
    """BASELINE.json config 5 through the one-call backward: config-2 shape, codes Zipf(1.1)."""
    rng = np.random.RandomState(41)
    B, T, S, Do = 16384, 128, 256, 768
    p = 1.0 / np.arange(1, S + 1) ** 1.1
    p /= p.sum()
    code = rng.choice(S, size=(B, T), p=p).astype(np.int32)
    w = (1.0 - rng.rand(B, T)).astype(np.float32)
    g = rng.randn(B, Do).astype(np.float32)
    tables = (0.02 * rng.randn(T, S, Do)).astype(np.float32)
    gs, gt = cabi.lookup_backward(code, w, g, tables)
    # table gradient: column sums, a few tables in full, the sorted entry point bit for bit
    assert relmax(gt.astype(np.float64).sum(1), w.astype(np.float64).T @ g.astype(np.float64)) <= 1e-5
    for t in (0, 77, 127):
        want_t = oracle.scatter_add(code[:, t:t + 1], g.astype(np.float64), w[:, t:t + 1].astype(np.float64), S)
        assert relmax(gt[t], want_t) <= 1e-5
    assert np.array_equal(gt, cabi.lookup_scatter_sorted(code, w, g, S))
    # score gradient: a token sample against the oracle, every (token, table) against the separate entry point
    # (the same additions in the same order: bit-identical), the duality with the forward, and a second call
    sub = np.unique(np.concatenate([rng.choice(B, 64, replace=False), np.arange(B - 40, B), np.arange(0, 8)]))
    idx = code + (np.arange(T, dtype=np.int32) * S)[None]
    want = oracle.indexed_inner_product(idx[sub], g[sub].astype(np.float64), tables.reshape(T * S, Do).astype(np.float64))
    assert relmax(gs[sub], want) <= 1e-5
    assert np.array_equal(gs, cabi.lookup_inner(code, g, tables))
    fwd = cabi.lookup_gather(code, w, tables, None)
    lhs = float((fwd.astype(np.float64) * g).sum())
    rhs = float((gs.astype(np.float64) * w).sum())
    assert abs(lhs - rhs) <= 1e-5 * max(abs(lhs), 1.0) * 10
    gs2, gt2 = cabi.lookup_backward(code, w, g, tables)
    assert np.array_equal(gs, gs2) and np.array_equal(gt, gt2)


def test_lookup_scatter_full_size_zipf_properties():
    # BASELINE.json config 5: config-2 shape, codes Zipf(1.1) over 256 entries
    rng = np.random.RandomState(41)
    B, T, S, Do = 16384, 128, 256, 768
    p = 1.0 / np.arange(1, S + 1) ** 1.1
    p /= p.sum()
    code = rng.choice(S, size=(B, T), p=p).astype(np.int32)
    w = (1.0 - rng.rand(B, T)).astype(np.float32)
    g = rng.randn(B, Do).astype(np.float32)
    got = cabi.lookup_scatter(code, w, g, S)
    # column sums: sum_s grad[t,s,:] = sum_b w[b,t] g[b,:]
    want_sum = w.astype(np.float64).T @ g.astype(np.float64)
    assert relmax(got.astype(np.float64).sum(1), want_sum) <= 1e-5
    # a few tables in full against the oracle (the hottest row takes ~18 % of the tokens)
    for t in (0, 77, 127):
        idx_t = code[:, t:t + 1]
        want_t = oracle.scatter_add(idx_t, g.astype(np.float64), w[:, t:t + 1].astype(np.float64), S)
        assert relmax(got[t], want_t) <= 1e-5
    # duality with the forward: <G(w), g> = <grad_tables, tables>
    tables = (0.02 * rng.randn(T, S, Do)).astype(np.float32)
    fwd = cabi.lookup_gather(code, w, tables, None)
    lhs = float((fwd.astype(np.float64) * g).sum())
    rhs = float((got.astype(np.float64) * tables).sum())
    assert abs(lhs - rhs) <= 1e-5 * max(abs(lhs), 1.0) * 10


# (B, T, S, Do): the LDS kernel needs ceil(B/256) * Do/64 >= 192 units, T >= 4 and S <= 256; the
# first rows take it with each token tile (832, 512, 256 tokens), ragged token counts, table counts
# that are no multiple of the 16-table chunk and tables smaller than the LDS slice; the next rows
# fall back to the token-major kernel.  The last rows take the four-lanes-per-token kernel (S = 256,
# T even, ceil(B/1024) * ceil(T/8) >= 200 workgroups with chunks of 4 table pairs, or
# ceil(B/1024) * ceil(T/4) >= 96 with chunks of 2): last chunks of 1, 3 and 2 pairs, a last tile of one
# token, a last chunk of 1 pair with chunks of 2.
INNER_CASES = [(16384, 20, 256, 768), (4100, 17, 256, 768), (3000, 5, 64, 1024), (12289, 33, 16, 768),
               (8191, 16, 256, 1536), (8191, 9, 128, 768), (256, 32, 256, 256), (1, 2, 4, 64), (65, 5, 256, 192),
               (500, 4, 512, 128), (2000, 3, 256, 1024), (0, 4, 16, 64),
               (20000, 82, 256, 64), (20481, 86, 256, 64), (24000, 76, 256, 128), (6000, 66, 256, 64),
               (4096, 128, 256, 192)]


@pytest.mark.parametrize("B,T,S,Do", INNER_CASES)
def test_lookup_inner_matches_oracle(B, T, S, Do):
    rng = np.random.RandomState(B + T + S + Do + 1)
    tables, code, idx, _ = _rand_gather(rng, B, T, S, Do)
    g = rng.randn(B, Do).astype(np.float32)
    got = cabi.lookup_inner(code, g, tables)
    if B == 0:
        assert got.shape == (0, T)
        return
    assert not np.isnan(got).any()                      # every entry written
    want = oracle.indexed_inner_product(idx, g.astype(np.float64), tables.reshape(T * S, Do).astype(np.float64))
    assert relmax(got, want) <= 1e-5
    # the same numbers as the flat-index entry point, up to the order of the additions
    assert relmax(got, cabi.indexed_inner_product(idx, g, tables.reshape(T * S, Do))) <= 1e-5
    # codes are masked into their table; a second call overwrites the first result
    dirty = (code + S * rng.randint(0, 4, size=code.shape)).astype(np.int32)
    assert relmax(cabi.lookup_inner(dirty, g, tables), want) <= 1e-5


def test_lookup_inner_is_reproducible_where_every_sum_has_one_owner():
    # the four-lanes-per-token kernel adds a (token, table)'s 24 slice sums in a fixed order in one
    # lane: two runs agree bit for bit (the form with atomics does not promise that)
    rng = np.random.RandomState(77)
    B, T, S, Do = 16384, 128, 256, 768
    tables, code, _, _ = _rand_gather(rng, B, T, S, Do)
    g = rng.randn(B, Do).astype(np.float32)
    first = cabi.lookup_inner(code, g, tables)
    for _ in range(12):
        assert np.array_equal(cabi.lookup_inner(code, g, tables), first)
    # where a token sits in the batch (tile, pass, quad) only changes the order in which its quad adds the
    # two halves of a 32-column slice
    perm = rng.permutation(B)
    moved = cabi.lookup_inner(np.ascontiguousarray(code[perm]), np.ascontiguousarray(g[perm]), tables)
    assert relmax(moved, first[perm].astype(np.float64)) <= 1e-6


def test_lookup_inner_full_size_duality():
    # BASELINE.json config 2 shape: <G(w), g> = sum_bt w[b,t] * grad_score[b,t], and linearity in g
    rng = np.random.RandomState(43)
    B, T, S, Do = 16384, 128, 256, 768
    tables, code, idx, w = _rand_gather(rng, B, T, S, Do)
    g = rng.randn(B, Do).astype(np.float32)
    got = cabi.lookup_inner(code, g, tables)
    fwd = cabi.lookup_gather(code, w, tables, None)
    lhs = float((fwd.astype(np.float64) * g).sum())
    rhs = float((got.astype(np.float64) * w).sum())
    assert abs(lhs - rhs) <= 1e-5 * max(abs(lhs), 1.0) * 10
    sub = slice(5000, 5200)
    want = oracle.indexed_inner_product(idx[sub], g[sub].astype(np.float64),
                                        tables.reshape(T * S, Do).astype(np.float64))
    assert relmax(got[sub], want) <= 1e-5
    assert relmax(cabi.lookup_inner(code, 2.0 * g, tables), 2.0 * got.astype(np.float64)) <= 1e-6


def test_half_backward_full_size_duality():
    """The half-precision backward operators at the config-2 size (16384 tokens x 128 rows each, 768 columns,
    Zipf(1.1) rows as in config 5): the forward, the inner product and the scatter-add are three views of one
    trilinear form, sum_bi w[b,i] <g[b], src[idx[b,i]]>, so their totals agree; samples against float64."""
    rng = np.random.RandomState(44)
    B, T, S, Do = 16384, 128, 256, 768
    p = 1.0 / np.arange(1, S + 1) ** 1.1
    p /= p.sum()
    code = rng.choice(S, size=(B, T), p=p).astype(np.int32)
    idx = code + (np.arange(T, dtype=np.int32) * S)[None]
    w = (1.0 - rng.rand(B, T)).astype(np.float32)
    src = (0.02 * rng.randn(T * S, Do)).astype(np.float16)
    g = rng.randn(B, Do).astype(np.float16)
    fwd = cabi.gather_add(idx, src.view(np.uint16), w, fmt=cabi.ROWS_F16)                       # [B, Do]
    inner = cabi.indexed_inner_product(idx, g.view(np.uint16), src.view(np.uint16))             # [B, T]
    scat = cabi.scatter_add(idx, g.view(np.uint16), w, T * S)                                   # [T*S, Do]
    a = float((fwd.astype(np.float64) * g.astype(np.float64)).sum())
    b = float((inner.astype(np.float64) * w).sum())
    c = float((scat.astype(np.float64) * src.astype(np.float64)).sum())
    scale = float(np.abs(inner.astype(np.float64) * w).sum())
    assert abs(a - b) <= 1e-5 * scale and abs(c - b) <= 1e-5 * scale
    sub = slice(7000, 7100)
    want = oracle.indexed_inner_product(idx[sub], g[sub].astype(np.float64), src.astype(np.float64))
    assert relmax(inner[sub], want) <= 1e-5
    # the hottest rows of a few tables against float64 sums over every token
    for t in (0, 77, 127):
        for c_ in (0, 1):
            hit = code[:, t] == c_
            want_row = (w[hit, t].astype(np.float64)[:, None] * g[hit].astype(np.float64)).sum(0)
            assert relmax(scat[t * S + c_], want_row) <= 1e-5


def test_scatter_duplicates_zipf():
    # heavy duplication of rows (BASELINE.json config 5 draws codes Zipf(1.1))
    rng = np.random.RandomState(40)
    B, T, S, Do = 2048, 16, 256, 256
    p = 1.0 / np.arange(1, S + 1) ** 1.1
    p /= p.sum()
    code = rng.choice(S, size=(B, T), p=p).astype(np.int32)
    idx = code + (np.arange(T, dtype=np.int32) * S)[None]
    w = (1.0 - rng.rand(B, T)).astype(np.float32)
    g = rng.randn(B, Do).astype(np.float32)
    want = oracle.scatter_add(idx, g.astype(np.float64), w.astype(np.float64), T * S)
    assert relmax(cabi.scatter_add(idx, g, w, T * S), want) <= 1e-5


# ----------------------------------------------------------------------------- config 3 at full size

@pytest.fixture(scope="module")
def config3():
    """BASELINE.json config 3: 16384 tokens, 512 tables x 256 entries x 1024 columns (537 MB of fp32
    rows, more than the Infinity Cache holds; 268 MB as bf16), weights uniform (0, 1]."""
    rng = np.random.default_rng(33)
    B, T, S, Do = 16384, 512, 256, 1024
    tables = rng.standard_normal((T, S, Do), dtype=np.float32)
    tables *= np.float32(0.02)
    code = rng.integers(0, S, size=(B, T), dtype=np.int32)
    idx = code + (np.arange(T, dtype=np.int32) * S)[None]
    w = (1.0 - rng.random((B, T), dtype=np.float32)).astype(np.float32)
    bias = (0.001 * rng.standard_normal(Do)).astype(np.float32)
    # a random sample of tokens, the first few and the whole tail of the last tile
    sub = np.unique(np.concatenate([rng.choice(B, 64, replace=False), np.arange(B - 40, B), np.arange(0, 8)]))
    # sum_b w[b,t] over the tokens with code s: what the all-token checksums are formed from
    cnt = np.zeros((T, S), np.float64)
    np.add.at(cnt, (np.broadcast_to(np.arange(T), (B, T)), code), w.astype(np.float64))
    return dict(B=B, T=T, S=S, Do=Do, tables=tables, code=code, idx=idx, w=w, bias=bias, sub=sub, cnt=cnt)


def _rows64(src_f32, idx):
    """The rows a sample of tokens reads, as a compact float64 table with re-numbered indices."""
    uniq, inv = np.unique(idx, return_inverse=True)
    return src_f32[uniq].astype(np.float64), inv.reshape(idx.shape).astype(np.int32)


@pytest.mark.parametrize("bf16", [False, True])
def test_config3_gather_full_size(config3, bf16):
    c = config3
    B, T, S, Do = c["B"], c["T"], c["S"], c["Do"]
    plan = cabi.lookup_gather_plan(B, T, S, Do, bf16)
    assert plan[0] in (1, 2), plan                       # a table-major LDS kernel, the planner's own choice
    flat = c["tables"].reshape(T * S, Do)
    src = oracle.bf16_round(flat) if bf16 else flat
    wide = oracle.bf16_widen(src) if bf16 else flat     # the values the kernel multiplies
    got = cabi.lookup_gather(c["code"], c["w"], src.reshape(T, S, Do), c["bias"], bf16=bf16)
    assert not np.isnan(got).any()
    sub = c["sub"]
    rows, ridx = _rows64(wide, c["idx"][sub])
    want = oracle.gather_add(ridx, rows, c["w"][sub].astype(np.float64)) + c["bias"]
    assert relmax(got[sub], want) <= 1e-5
    if bf16:
        rows32, _ = _rows64(flat, c["idx"][sub])
        assert relmax(got[sub], oracle.gather_add(ridx, rows32, c["w"][sub].astype(np.float64)) + c["bias"]) <= 1e-2
    # every token against the token-major kernel (same rows, the same order of additions)
    assert relmax(got, cabi.gather_add(c["idx"], src, c["w"], bf16=bf16).astype(np.float64) + c["bias"]) <= 2e-6
    # checksum over all tokens: sum_b out[b] = B * bias + sum_{t,s} cnt[t,s] * tables[t,s]
    want_sum = B * c["bias"].astype(np.float64)
    for t0 in range(0, T, 64):
        want_sum = want_sum + np.einsum("ts,tsd->d", c["cnt"][t0:t0 + 64], wide[t0 * S:(t0 + 64) * S].reshape(64, S, Do).astype(np.float64))
    assert relmax(got.astype(np.float64).sum(0), want_sum) <= 1e-5
    # a second launch gives the same bits (fixed order of additions)
    assert np.array_equal(got, cabi.lookup_gather(c["code"], c["w"], src.reshape(T, S, Do), c["bias"], bf16=bf16))


@pytest.mark.parametrize("fmt", [cabi.ROWS_F32, cabi.ROWS_BF16, cabi.ROWS_F16])
def test_config3_gather_record_stream_full_size(config3, fmt):
    """Config 3 through the form the layer and bench.py run there: lffn_lookup_gather_ws_* packs the record
    stream and launches the four-lanes-per-token kernel (fp32 rows: 2048-token tiles over 32 slices; bfloat16
    and half rows: 1024-token tiles over 16 slices of 64 columns; 256 table pairs)."""
    c = config3
    B, T, S, Do = c["B"], c["T"], c["S"], c["Do"]
    nbytes = cabi.lookup_gather_workspace_bytes(B, T, S, Do, fmt)
    assert nbytes > 0 and nbytes % 12 == 0 and nbytes < B * Do * 4            # the record stream, not the table split
    tokens = CONFIG3_RECORD_PLAN[0] if fmt == cabi.ROWS_F32 else 1024
    assert cabi.lookup_gather_records_plan_rows(B, T, S, Do, fmt) == (tokens, 16384, 6 * T * 16384)
    assert cabi.lookup_gather_ws_plan(B, T, S, Do, fmt, nbytes) == (3, tokens)
    bits, _ = cabi.rows_of(c["tables"], fmt)
    flat = bits.reshape(T * S, Do)
    widen = {cabi.ROWS_F32: lambda r: r, cabi.ROWS_BF16: oracle.bf16_widen, cabi.ROWS_F16: lambda r: r.view(np.float16)}[fmt]

    def ws_entry(residual=None):
        if fmt == cabi.ROWS_F16:
            return cabi.lookup_gather_ws_f16(c["code"], c["w"], bits, c["bias"], residual=residual)
        return cabi.lookup_gather_ws(c["code"], c["w"], bits, c["bias"], bf16=fmt == cabi.ROWS_BF16, residual=residual)
    got = ws_entry()
    assert not np.isnan(got).any()
    sub = c["sub"]
    uniq, inv = np.unique(c["idx"][sub], return_inverse=True)
    ridx = inv.reshape(c["idx"][sub].shape).astype(np.int32)
    want = oracle.gather_add(ridx, widen(flat[uniq]).astype(np.float64), c["w"][sub].astype(np.float64)) + c["bias"]
    assert relmax(got[sub], want) <= 1e-5
    if fmt != cabi.ROWS_F32:        # against the fp32 rows the 16-bit ones were rounded from
        rows32, _ = _rows64(c["tables"].reshape(T * S, Do), c["idx"][sub])
        assert relmax(got[sub], oracle.gather_add(ridx, rows32, c["w"][sub].astype(np.float64)) + c["bias"]) <= 1e-2
    # every token against the token-major kernel on the same rows (the two tables of a pair added in either order)
    assert relmax(got, cabi.gather_add(c["idx"], flat, c["w"], fmt=fmt).astype(np.float64) + c["bias"]) <= 2e-6
    # checksum over all tokens: sum_b out[b] = B * bias + sum_{t,s} cnt[t,s] * tables[t,s]
    want_sum = B * c["bias"].astype(np.float64)
    for t0 in range(0, T, 64):
        want_sum = want_sum + np.einsum("ts,tsd->d", c["cnt"][t0:t0 + 64],
                                        widen(flat[t0 * S:(t0 + 64) * S]).reshape(64, S, Do).astype(np.float64))
    assert relmax(got.astype(np.float64).sum(0), want_sum) <= 1e-5
    # a second launch gives the same bits; so does the same tile size named explicitly
    assert np.array_equal(got, ws_entry())
    rc, forced = cabi.lookup_gather_ws_planned_rows(c["code"], c["w"], bits, fmt, (3, tokens), bias=c["bias"])
    assert rc == 0 and np.array_equal(got, forced)
    # the residual goes into the store: the same sums plus the residual, rounded once more
    res = np.random.default_rng(36).standard_normal((B, Do), dtype=np.float32)
    assert np.array_equal(ws_entry(residual=res), got + res)


def test_config3_inner_product_full_size(config3):
    c = config3
    B, T, S, Do = c["B"], c["T"], c["S"], c["Do"]
    rng = np.random.default_rng(34)
    g = rng.standard_normal((B, Do), dtype=np.float32)
    got = cabi.lookup_inner(c["code"], g, c["tables"])
    assert not np.isnan(got).any()
    sub = c["sub"]
    flat = c["tables"].reshape(T * S, Do)
    rows, ridx = _rows64(flat, c["idx"][sub])
    want = oracle.indexed_inner_product(ridx, g[sub].astype(np.float64), rows)
    assert relmax(got[sub], want) <= 1e-5
    # every (token, table) against the token-major kernel
    assert relmax(got, cabi.indexed_inner_product(c["idx"], g, flat)) <= 1e-5
    # duality with the forward: <G(w), g> = sum_bt w[b,t] * grad_score[b,t]
    fwd = cabi.lookup_gather(c["code"], c["w"], c["tables"], None)
    lhs = float((fwd.astype(np.float64) * g).sum())
    rhs = float((got.astype(np.float64) * c["w"]).sum())
    assert abs(lhs - rhs) <= 1e-5 * max(abs(lhs), 1.0) * 10


def test_config3_scatter_full_size(config3):
    c = config3
    B, T, S, Do = c["B"], c["T"], c["S"], c["Do"]
    rng = np.random.default_rng(35)
    g = rng.standard_normal((B, Do), dtype=np.float32)
    got = cabi.lookup_scatter_sorted(c["code"], c["w"], g, S)
    assert not np.isnan(got).any()
    # column sums: sum_s grad[t,s,:] = sum_b w[b,t] g[b,:]
    want_sum = c["w"].astype(np.float64).T @ g.astype(np.float64)
    assert relmax(got.astype(np.float64).sum(1), want_sum) <= 1e-5
    # a few tables in full against the oracle
    for t in (0, 255, 511):
        want_t = oracle.scatter_add(c["code"][:, t:t + 1], g.astype(np.float64), c["w"][:, t:t + 1].astype(np.float64), S)
        assert relmax(got[t], want_t) <= 1e-5
    # the LDS form on the same inputs
    assert relmax(got, cabi.lookup_scatter(c["code"], c["w"], g, S)) <= 1e-5
    # duality with the forward: <G(w), g> = <grad_tables, tables>
    fwd = cabi.lookup_gather(c["code"], c["w"], c["tables"], None)
    lhs = float((fwd.astype(np.float64) * g).sum())
    rhs = float(np.einsum("tsd,tsd->", got.astype(np.float64), c["tables"].astype(np.float64)))
    assert abs(lhs - rhs) <= 1e-5 * max(abs(lhs), 1.0) * 10
