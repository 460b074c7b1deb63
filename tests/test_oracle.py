"""Pins the CPU oracle (oracle/) before anything is checked against it.

Each oracle function is checked against something that does not share its code:
the committed closed-form fixtures, scipy's Hadamard matrix (the reference's own
check, FHT/kernel.py:31-37), brute-force loops, torch library routines
(embedding_bag, layer_norm, einsum, autograd) and, where oracle/_ref was built,
the reference's own x86 kernels compiled from its sources.
"""
import json
import math
import os

import numpy as np
import pytest
import scipy.linalg
import torch

import oracle


@pytest.fixture(scope="module")
def golden(golden_dir):
    with open(os.path.join(golden_dir, "lookupffn_golden.json")) as f:
        return json.load(f)


# ----------------------------------------------------------------------------- FHT

def test_fht_golden(golden):
    for D, g in golden["hadamard"].items():
        x = np.array(g["x"], dtype=np.float32)
        want = np.array(g["xH"], dtype=np.float32)
        assert np.array_equal(oracle.fht(x), want)
        assert np.array_equal(oracle.fht(x.astype(np.float64)), want.astype(np.float64))
        H = np.array(g["H"], dtype=np.float64)
        assert np.array_equal(H, scipy.linalg.hadamard(int(D)))


@pytest.mark.parametrize("D", [1, 2, 4, 8, 32, 64, 256, 512, 1024])
def test_fht_matches_scipy_exactly_on_integers(D):
    rng = np.random.RandomState(D)
    x = rng.randint(-16, 17, size=(5, D)).astype(np.float32)
    H = scipy.linalg.hadamard(D).astype(np.float64) if D > 1 else np.ones((1, 1))
    want = x.astype(np.float64) @ H
    assert np.array_equal(oracle.fht(x).astype(np.float64), want)   # sums < 2^24: exact
    assert np.array_equal(oracle.fht(x.astype(np.float64)), want)


@pytest.mark.parametrize("D", [16, 256, 1024])
def test_fht_invariants(D):
    rng = np.random.RandomState(7)
    x = rng.randn(4, D)
    y = oracle.fht(x)
    np.testing.assert_allclose(oracle.fht(y), D * x, rtol=1e-12, atol=1e-9)      # H.H = D.I
    np.testing.assert_allclose((y ** 2).sum(1), D * (x ** 2).sum(1), rtol=1e-12)  # Parseval
    e0 = np.zeros((1, D)); e0[0, 0] = 1
    assert np.array_equal(oracle.fht(e0), np.ones((1, D)))
    e5 = np.zeros((1, D)); e5[0, 5] = 1
    assert np.array_equal(oracle.fht(e5)[0], scipy.linalg.hadamard(D)[5])           # row 5, natural order
    ones = np.ones((1, D))
    assert np.array_equal(oracle.fht(ones), D * e0)


def test_fht_f32_close_to_f64():
    rng = np.random.RandomState(3)
    x = rng.randn(64, 1024).astype(np.float32)
    want = x.astype(np.float64) @ scipy.linalg.hadamard(1024).astype(np.float64)
    got = oracle.fht(x)
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()


# ----------------------------------------------------------------------------- BH4

def _bh4_torch(x, w):
    """The reference's GPU formula (PL/bh4/kernel.py:23-36) in float64 with a matmul Hadamard."""
    x = torch.as_tensor(x, dtype=torch.float64)
    w = torch.as_tensor(w, dtype=torch.float64)
    B, D = x.shape
    BS = w.shape[-1]
    NB = D // BS
    H = torch.tensor(scipy.linalg.hadamard(D), dtype=torch.float64)
    out = []
    for i in range(w.shape[0]):
        y = x
        for j in range(w.shape[1]):
            y = torch.einsum("bni,noi->bno", y.reshape(B, NB, BS), w[i, j]).reshape(B, D)
            y = y @ H
        out.append(y)
    return torch.cat(out, dim=-1).numpy()


@pytest.mark.parametrize("D,bs,R,J", [(64, 1, 1, 4), (64, 16, 2, 4), (256, 64, 1, 4), (128, 1, 3, 1), (32, 32, 1, 2)])
def test_bh4_matches_einsum_hadamard(D, bs, R, J):
    rng = np.random.RandomState(D + bs)
    x = rng.randn(6, D)
    w = rng.randn(R, J, D // bs, bs, bs) / math.sqrt(bs * D)
    want = _bh4_torch(x, w)
    got64 = oracle.bh4(x, w)
    np.testing.assert_allclose(got64, want, rtol=1e-10, atol=1e-10 * np.abs(want).max())
    got32 = oracle.bh4(x.astype(np.float32), w.astype(np.float32))
    assert np.abs(got32 - want).max() <= 2e-5 * np.abs(want).max()


def test_bh4_block1_is_sign_diagonal_fht():
    rng = np.random.RandomState(11)
    D = 128
    x = rng.randint(-4, 5, size=(3, D)).astype(np.float32)
    s = (2 * rng.randint(0, 2, size=(1, 1, D, 1, 1)) - 1).astype(np.float32)
    want = (x * s.reshape(1, D)).astype(np.float64) @ scipy.linalg.hadamard(D)
    assert np.array_equal(oracle.bh4(x, s).astype(np.float64), want)


def test_projection_matches_module_formula():
    # PL/lookup.py:29-39 in torch float64
    rng = np.random.RandomState(5)
    B, H, D, R, J, bs, out_dim = 5, 48, 64, 2, 4, 1, 100
    x = rng.randn(B, H)
    w = rng.randn(R, J, D // bs, bs, bs) / math.sqrt(bs * D)
    bias = rng.randn(out_dim)
    xp = np.concatenate([x, np.zeros((B, D - H))], axis=1)
    want = 0.7 * _bh4_torch(xp, w) + (1 - 0.7) * np.tile(xp, (1, R))
    want = want[:, :out_dim] + bias
    got = oracle.projection(x, w, bias, out_dim, 0.7)
    np.testing.assert_allclose(got, want, rtol=1e-10, atol=1e-12)
    got32 = oracle.projection(x.astype(np.float32), w.astype(np.float32), bias.astype(np.float32), out_dim, 0.7)
    assert np.abs(got32 - want).max() <= 1e-5 * np.abs(want).max()


# ----------------------------------------------------------------------------- code + score

def test_code_golden_all_256_patterns(golden):
    z = np.array(golden["codes"]["z"], dtype=np.float32)
    code, _ = oracle.code_score(z)
    assert code.dtype == np.int32
    assert np.array_equal(code, np.array(golden["codes"]["code"], dtype=np.int32))


def test_score_golden(golden):
    for z, want in zip(golden["score"]["z"], golden["score"]["score"]):
        z64 = np.array([z], dtype=np.float64)
        _, s64 = oracle.code_score(z64)
        assert abs(s64[0] - want) <= 1e-14 * max(1.0, abs(want))
        _, s32 = oracle.code_score(z64.astype(np.float32))
        assert abs(float(s32[0]) - want) <= 2e-6 * max(1.0, abs(want))


def test_code_special_values():
    z = np.array([[0.0, -0.0, np.nan, 1e-30, -1e-30, np.inf, -np.inf, 1.0]], dtype=np.float32)
    code, _ = oracle.code_score(z)
    # only strictly positive entries set a bit: d = 3, 5, 7 -> 2^4 + 2^2 + 2^0
    assert code[0] == 16 + 4 + 1
    assert oracle.code_score(np.full((1, 8), 2.0, np.float32))[0][0] == 255
    assert oracle.code_score(np.full((1, 8), -2.0, np.float32))[0][0] == 0
    k1 = np.array([[0.8]], dtype=np.float64)
    _, s = oracle.code_score(k1)
    assert abs(s[0] - 0.8 / (1 + math.exp(-1.6))) < 1e-15


@pytest.mark.parametrize("k", [1, 3, 8, 11])
def test_code_score_brute_force(k):
    rng = np.random.RandomState(k)
    z = rng.randn(50, 7, k)
    code, score = oracle.code_score(z)
    for b in range(50):
        for t in range(7):
            c = 0
            for d in range(k):
                if z[b, t, d] > 0:
                    c |= 1 << (k - 1 - d)
            assert code[b, t] == c
            den = np.prod(1 + np.exp(-2 * np.abs(z[b, t])))
            assert abs(score[b, t] - np.abs(z[b, t]).sum() / den) < 1e-12


def test_code_score_matches_reference_torch_formula():
    # PL/compute_code_score/kernel.py:43-55 restated with torch library calls
    torch.manual_seed(0)
    z = torch.randn(300, 16, 8)
    mask = 2 ** torch.arange(7, -1, -1, dtype=z.dtype)
    code_t = ((z > 0).to(z.dtype) * mask).sum(-1).int()
    a = z.abs()
    score_t = a.sum(-1) / torch.prod(1 + torch.exp(-2 * a), dim=-1)
    code, score = oracle.code_score(z.numpy())
    assert np.array_equal(code, code_t.numpy())
    np.testing.assert_allclose(score, score_t.numpy(), rtol=2e-6)


def test_code_score_matches_reference_x86_kernel():
    ccs = oracle.load_ref("ccs_cpu")
    if ccs is None:
        pytest.skip("oracle/_ref/ccs_cpu.so not built (reference checkout absent)")
    torch.manual_seed(1)
    z = torch.randn(512, 32, 8)
    z[0, 0, :4] = 0.0
    codes = torch.empty(512, 32, dtype=torch.int)
    scores = torch.empty(512, 32, dtype=torch.float)
    ccs.compute_code_score(z, codes, scores)
    code, score = oracle.code_score(z.numpy())
    assert np.array_equal(code, codes.numpy())
    # same operations in the same order; the reference build may call exp in double
    np.testing.assert_allclose(score, scores.numpy(), rtol=1e-6, atol=0)


def test_code_score_bwd_matches_autograd():
    torch.manual_seed(2)
    z = torch.randn(40, 5, 8, dtype=torch.float64, requires_grad=True)
    a = z.abs()
    score = a.sum(-1) / torch.prod(1 + torch.exp(-2 * a), dim=-1)
    g = torch.randn(40, 5, dtype=torch.float64)
    score.backward(g)
    got = oracle.code_score_bwd(z.detach().numpy(), g.numpy())
    np.testing.assert_allclose(got, z.grad.numpy(), rtol=1e-10, atol=1e-12)
    got32 = oracle.code_score_bwd(z.detach().numpy().astype(np.float32), g.numpy().astype(np.float32))
    np.testing.assert_allclose(got32, z.grad.numpy(), rtol=2e-5, atol=1e-6)


# ----------------------------------------------------------------------------- gather-add and its backward

def _rand_gather(rng, B, T, S, Do, dtype=np.float32):
    tables = (0.02 * rng.randn(T, S, Do)).astype(dtype)
    code = rng.randint(0, S, size=(B, T)).astype(np.int32)
    idx = code + (np.arange(T, dtype=np.int32) * S)[None]
    w = (1.0 - rng.rand(B, T)).astype(dtype)
    return tables.reshape(T * S, Do), idx, w


def test_gather_golden(golden):
    g = golden["gather"]
    tables = np.array(g["tables"], dtype=np.float32)
    T, S, Do = tables.shape
    idx = np.array(g["code"], dtype=np.int32) + (np.arange(T, dtype=np.int32) * S)[None]
    w = np.array(g["w"], dtype=np.float32)
    flat = tables.reshape(T * S, Do)
    assert np.array_equal(oracle.gather_add(idx, flat, w), np.array(g["out"], dtype=np.float32))
    gout = np.array(g["g_out"], dtype=np.float32)
    assert np.array_equal(oracle.indexed_inner_product(idx, gout, flat), np.array(g["g_w"], dtype=np.float32))
    assert np.array_equal(oracle.scatter_add(idx, gout, w, T * S).reshape(T, S, Do),
                          np.array(g["g_tables"], dtype=np.float32))
    bits = oracle.bf16_round(flat)      # small integers are exact in bf16
    assert np.array_equal(oracle.gather_add_bf16(idx, bits, w), np.array(g["out"], dtype=np.float32))


def test_gather_matches_embedding_bag_and_autograd():
    rng = np.random.RandomState(21)
    flat, idx, w = _rand_gather(rng, 33, 6, 16, 64, np.float64)
    src_t = torch.tensor(flat, requires_grad=True)
    w_t = torch.tensor(w, requires_grad=True)
    out_t = torch.nn.functional.embedding_bag(torch.tensor(idx, dtype=torch.long), src_t,
                                              per_sample_weights=w_t, mode="sum")
    g = rng.randn(33, 64)
    out_t.backward(torch.tensor(g))
    np.testing.assert_allclose(oracle.gather_add(idx, flat, w), out_t.detach().numpy(), rtol=1e-12, atol=1e-14)
    np.testing.assert_allclose(oracle.indexed_inner_product(idx, g, flat), w_t.grad.numpy(), rtol=1e-12, atol=1e-14)
    np.testing.assert_allclose(oracle.scatter_add(idx, g, w, flat.shape[0]), src_t.grad.numpy(), rtol=1e-12, atol=1e-14)
    # float32 instantiation against the float64 truth
    o32 = oracle.gather_add(idx, flat.astype(np.float32), w.astype(np.float32))
    assert np.abs(o32 - out_t.detach().numpy()).max() <= 1e-5 * np.abs(out_t.detach().numpy()).max()


def test_gather_special_cases():
    rng = np.random.RandomState(22)
    flat, idx, w = _rand_gather(rng, 8, 4, 8, 64)
    onehot = np.zeros_like(w); onehot[:, 2] = 1.0
    assert np.array_equal(oracle.gather_add(idx, flat, onehot), flat[idx[:, 2]])       # row lookup
    const = np.ones_like(flat)
    np.testing.assert_allclose(oracle.gather_add(idx, const, w)[:, 0], w.astype(np.float64).sum(1), rtol=1e-6)
    # duplicate indices accumulate
    idx2 = np.zeros((1, 4), dtype=np.int32)
    assert np.array_equal(oracle.scatter_add(idx2, np.ones((1, 64), np.float32), np.ones((1, 4), np.float32), 2)[0],
                          np.full(64, 4.0, np.float32))


def test_gather_bf16_equals_f32_on_widened_table():
    rng = np.random.RandomState(23)
    flat, idx, w = _rand_gather(rng, 16, 4, 8, 128)
    bits = oracle.bf16_round(flat)
    wide = oracle.bf16_widen(bits)
    assert np.abs(wide - flat).max() <= 2 ** -8 * np.abs(flat).max()
    assert np.array_equal(bits, torch.tensor(flat).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16))
    assert np.array_equal(oracle.gather_add_bf16(idx, bits, w), oracle.gather_add(idx, wide, w))


def test_gather_matches_reference_x86_kernels():
    ga = oracle.load_ref("gather_add_cpu")
    if ga is None:
        pytest.skip("oracle/_ref/gather_add_cpu.so not built (reference checkout absent)")
    rng = np.random.RandomState(24)
    # the tiled kernel assumes table_size 256 and a token count divisible by 64
    # (PL/gather/cpu/torch_extension.cpp:66-72)
    flat, idx, w = _rand_gather(rng, 128, 8, 256, 64)
    ti, ts, tw = torch.tensor(idx), torch.tensor(flat), torch.tensor(w)
    want_scalar = ga.weighted_vector_gather_add_scalar(ti, ts, tw).numpy()
    want_tiled = ga.weighted_vector_gather_add_avx2_par(ti, ts, tw).numpy()
    got = oracle.gather_add(idx, flat, w)
    # same order of accumulation; the reference build may contract mul+add into fma
    assert np.abs(got - want_scalar).max() <= 1e-6 * np.abs(want_scalar).max()
    assert np.abs(got - want_tiled).max() <= 1e-6 * np.abs(want_tiled).max()


# ----------------------------------------------------------------------------- layer

def test_layernorm_matches_torch():
    rng = np.random.RandomState(31)
    x = rng.randn(9, 48)
    gam, bet = rng.randn(48), rng.randn(48)
    want = torch.nn.functional.layer_norm(torch.tensor(x), (48,), torch.tensor(gam), torch.tensor(bet), 1e-5).numpy()
    np.testing.assert_allclose(oracle.layernorm(x, gam, bet, 1e-5), want, rtol=1e-11, atol=1e-12)


def test_lookup_ffn_is_the_composition():
    rng = np.random.RandomState(32)
    B, H, T, S, Do, bs = 12, 48, 8, 256, 64, 1
    k = 8
    D, R = 64, 1
    x = rng.randn(B, H)
    ln_w, ln_b = 1 + 0.1 * rng.randn(H), 0.1 * rng.randn(H)
    pw = rng.randn(R, 4, D // bs, bs, bs) / math.sqrt(bs * D)
    pb = 0.01 * rng.randn(T * k)
    tables = 0.02 * rng.randn(T, S, Do)
    bias = 0.001 * rng.randn(Do)
    out, z, code, score = oracle.lookup_ffn(x, ln_w, ln_b, 1e-5, pw, pb, tables, bias, return_parts=True)
    h = torch.nn.functional.layer_norm(torch.tensor(x), (H,), torch.tensor(ln_w), torch.tensor(ln_b), 1e-5).numpy()
    z_w = oracle.projection(h, pw, pb, T * k, 0.7)
    np.testing.assert_allclose(z, z_w, rtol=1e-9, atol=1e-12)
    code_w, score_w = oracle.code_score(z_w.reshape(B, T, k))
    assert np.array_equal(code, code_w)
    idx = torch.tensor(code_w, dtype=torch.long) + torch.arange(T)[None] * S
    want = torch.nn.functional.embedding_bag(idx, torch.tensor(tables.reshape(T * S, Do)),
                                             per_sample_weights=torch.tensor(score_w), mode="sum").numpy() + bias
    np.testing.assert_allclose(out, want, rtol=1e-10, atol=1e-13)
