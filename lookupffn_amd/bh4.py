"""BH4 projection operators: the reference's ``bh4`` / ``hadamard`` surface
(PL/bh4/kernel.py, PL/bh4/fast_hadamard_transform/kernel.py) on the gfx950 kernels.

PL/ = src/roberta/models/prenorm_lookup/ in the reference checkout.
"""
from __future__ import annotations

import math

import torch
from torch.autograd import Function

from . import ops


def hadamard_transform(X: torch.Tensor) -> torch.Tensor:
    """Slow formula ``X @ H`` (fast_hadamard_transform/kernel.py:31-37), kept as
    the in-tree check behind ``hadamard(..., use_torch=True)``.  H is built from
    H[i,j] = (-1)^popcount(i & j)."""
    assert X.is_contiguous()
    assert len(X.shape) == 2
    D = X.shape[-1]
    assert int(2 ** int(math.log2(D))) == D
    i = torch.arange(D, device=X.device)
    bits = i[:, None] & i[None, :]
    pop = torch.zeros_like(bits)
    for s in range(max(1, D.bit_length())):
        pop += (bits >> s) & 1
    H = (1 - 2 * (pop & 1)).to(X.dtype)
    return torch.matmul(X, H)


def fast_hadamard_transform(X: torch.Tensor) -> torch.Tensor:
    """out = X @ H_D, unnormalised, natural order (fast_hadamard_transform/kernel.py:39-45)."""
    assert X.is_contiguous()
    assert len(X.shape) == 2
    assert X.dtype in (torch.float32, torch.float16, torch.bfloat16)
    assert int(2 ** int(math.log2(X.shape[-1]))) == X.shape[-1]
    return ops.fht(X)


def fast_hadamard_transform_dim512(X):
    """fast_hadamard_transform/kernel.py:17-22: half rows of 512.  Computed in fp32 with one
    rounding on the store (the reference rounds in half precision after every stage)."""
    assert X.is_contiguous()
    assert len(X.shape) == 2
    assert X.dtype == torch.float16
    assert X.shape[-1] == 512
    return ops.fht(X)


def fast_hadamard_transform_dim1024(X):
    """fast_hadamard_transform/kernel.py:24-29: half rows of 1024; see the 512 form."""
    assert X.is_contiguous()
    assert len(X.shape) == 2
    assert X.dtype == torch.float16
    assert X.shape[-1] == 1024
    return ops.fht(X)


class FastHadamardTransform(Function):
    """H is symmetric, so the backward is the same transform
    (fast_hadamard_transform/kernel.py:47-54)."""

    @staticmethod
    def forward(ctx, inp):
        return fast_hadamard_transform(inp.contiguous())

    @staticmethod
    def backward(ctx, grad_outputs):
        return fast_hadamard_transform(grad_outputs.contiguous())


class FastHadamardTransformDim512(Function):
    @staticmethod
    def forward(ctx, inp):
        return fast_hadamard_transform_dim512(inp.contiguous())

    @staticmethod
    def backward(ctx, grad_outputs):
        return fast_hadamard_transform_dim512(grad_outputs.contiguous())


class FastHadamardTransformDim1024(Function):
    @staticmethod
    def forward(ctx, inp):
        return fast_hadamard_transform_dim1024(inp.contiguous())

    @staticmethod
    def backward(ctx, grad_outputs):
        return fast_hadamard_transform_dim1024(grad_outputs.contiguous())


def hadamard(inp, use_torch=False):
    """fast_hadamard_transform/kernel.py:78-89 without the per-call warning print."""
    if use_torch:
        return hadamard_transform(inp)
    if inp.dtype == torch.float16:
        if inp.shape[-1] == 512:
            return FastHadamardTransformDim512.apply(inp)
        if inp.shape[-1] == 1024:
            return FastHadamardTransformDim1024.apply(inp)
    return FastHadamardTransform.apply(inp)


def bh4_cuda(x, w):
    """PL/bh4/kernel.py:23-36.  w: [R, 4, D/bs, bs, bs].

    Without autograd, block size 1 runs as one fused kernel (all stages and
    repeats in registers) and block size 64 (D <= 1024) as a weight-folding
    kernel plus one fused matrix-core kernel.  Otherwise each stage is the block-diagonal product
    followed by the transform kernel, differentiable through
    ``FastHadamardTransform``."""
    BS = w.shape[-1]
    B, D = x.shape
    NB = D // BS
    needs_grad = torch.is_grad_enabled() and (x.requires_grad or w.requires_grad)
    if BS == 1 and not needs_grad and x.dtype == torch.float32:
        return ops.bh4_diag(x.contiguous(), w.reshape(w.shape[0], w.shape[1], D).contiguous())
    if BS == 64 and D <= 1024 and not needs_grad and x.dtype == torch.float32:
        return ops.bh4_block(x.contiguous(), ops.bh4_fold(w.contiguous()))
    out = []
    for i in range(w.shape[0]):
        y = x
        for j in range(w.shape[1]):
            if BS == 1:
                y = y * w[i, j].reshape(1, D)
            else:
                y = y.reshape(B, NB, BS)
                y = torch.einsum("bni,noi->bno", y, w[i, j])
                y = y.reshape(B, D)
            y = hadamard(y)
        out.append(y)
    return torch.cat(out, dim=-1)


def bh4(x, w, training):
    """PL/bh4/kernel.py:10-21.  The reference sends CPU tensors in eval mode to
    its x86 extension; this package has no CPU path, so CPU tensors are an error
    in both modes."""
    if not (x.is_cuda and w.is_cuda):
        raise RuntimeError("bh4: lookupffn_amd runs on the GPU only (got a CPU tensor)")
    return bh4_cuda(x, w)
