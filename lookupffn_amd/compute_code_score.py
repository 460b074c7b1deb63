"""Code + score of the hash: the reference's ``compute_code_score`` surface
(PL/compute_code_score/kernel.py) on the gfx950 kernel."""
from __future__ import annotations

import torch
from torch.autograd import Function

from . import ops


def bin2dec(b, bits):
    """PL/compute_code_score/kernel.py:32-34 (MSB first)."""
    mask = 2 ** torch.arange(bits - 1, -1, -1, dtype=b.dtype, device=b.device)
    return torch.sum(mask * b, -1)


def compute_code_score_torch(hash_scores):
    """The reference's torch formula (PL/compute_code_score/kernel.py:43-55), kept as
    the in-tree slow check."""
    code_length = hash_scores.shape[-1]
    code = 2 * (hash_scores > 0).to(hash_scores.dtype) - 1
    code = bin2dec((code + 1) / 2, code_length).int()
    max_hash_scores = hash_scores.abs()
    denominator = torch.prod(1 + torch.exp(-2 * max_hash_scores), dim=-1)
    score = max_hash_scores.sum(dim=-1) / denominator
    return code, score


class ComputeCodeScore(Function):
    """One kernel for (code, score); the backward is the closed-form derivative
    of the score (the code is an integer and has no gradient).  The reference's
    class of this name is CPU-only with an unimplemented backward
    (PL/compute_code_score/kernel.py:57-65); on the GPU it relies on autograd
    through eight element-wise ops."""

    @staticmethod
    def forward(ctx, hash_scores):
        hash_scores = hash_scores.contiguous()
        code, score = ops.code_score(hash_scores)
        ctx.save_for_backward(hash_scores)
        ctx.mark_non_differentiable(code)
        return code, score

    @staticmethod
    def backward(ctx, grad_code, grad_score):
        (hash_scores,) = ctx.saved_tensors
        return ops.code_score_bwd(hash_scores, grad_score.contiguous())


def compute_code_score(hash_scores, training):
    """PL/compute_code_score/kernel.py:22-30: (code int32 [..., T], score float [..., T])."""
    if not hash_scores.is_cuda:
        raise RuntimeError("compute_code_score: lookupffn_amd runs on the GPU only (got a CPU tensor)")
    if hash_scores.dtype in (torch.float16, torch.bfloat16):
        # under autocast a dense projection hands over 16-bit z (the reference's torch formula takes
        # any float dtype, PL/compute_code_score/kernel.py:43-55): widened here, exactly, so the code is
        # that of the 16-bit values; the score comes back in float32 and autograd casts the gradient
        # of z back to the 16-bit type
        hash_scores = hash_scores.float()
    if hash_scores.dtype != torch.float32:
        raise NotImplementedError(f"compute_code_score: dtype {hash_scores.dtype} (float32, float16 and bfloat16 are taken)")
    return ComputeCodeScore.apply(hash_scores)
