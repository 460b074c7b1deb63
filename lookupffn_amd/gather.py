"""Weighted gather-add operators: the reference's ``gather`` /
``weighted_gather_add`` surface (PL/gather/kernel.py, PL/gather/cuda/kernel.py) on the
gfx950 kernels.  Rows may be float32, bfloat16 or float16; accumulation is float32.  The
reference's half-precision calls (every tensor half) are taken as well, forward and backward:
their sums are formed in float32 and rounded to half once."""
from __future__ import annotations

import math

import torch
from torch.autograd import Function
from torch.utils.checkpoint import checkpoint

from . import ops


def power2(val):
    return (2 ** int(round(math.log2(val)))) == val


def _check(indexes, a, b, names):
    assert indexes.is_contiguous()
    assert a.is_contiguous()
    assert b.is_contiguous()
    assert indexes.dtype == torch.int32, indexes.dtype
    assert len(indexes.shape) == 2, indexes.shape
    assert len(a.shape) == 2, a.shape
    assert len(b.shape) == 2, b.shape


def weighted_vector_gather_add(indexes, source, weights, use_torch=False):
    """outputs[b] = sum_i weights[b,i] * source[indexes[b,i]]   (PL/gather/cuda/kernel.py:22-70)."""
    _check(indexes, source, weights, "gather")
    assert source.dtype in [torch.float32, torch.bfloat16, torch.float16], source.dtype
    assert weights.dtype in [torch.float32, torch.float16], weights.dtype
    half_call = weights.dtype == torch.float16
    if half_call:
        # the reference's half-precision call (PL/gather/cuda/kernel.py:64-67): half rows, half weights, half
        # result.  Here the sums are fp32 and the result is rounded to half once
        assert source.dtype == torch.float16, source.dtype
    batch_size, index_size = indexes.shape
    source_size, vector_dim = source.shape
    assert weights.shape[0] == batch_size and weights.shape[1] == index_size
    assert index_size % 2 == 0, index_size
    assert vector_dim % 64 == 0, vector_dim

    if use_torch:
        indexes = indexes.long()

        def mini_batching(source, indexes, weights, batch_idx):
            outputs = source[indexes[batch_idx, :], :].reshape(index_size, vector_dim)
            return (outputs.to(weights.dtype) * weights[batch_idx, :, None]).sum(dim=0)

        output_list = []
        for batch_idx in range(batch_size):
            output_list.append(checkpoint(mini_batching, source, indexes, weights, batch_idx, use_reentrant=False))
        return torch.stack(output_list, dim=0)
    if half_call:
        return ops.gather_add(indexes, source, weights.float()).half()
    return ops.gather_add(indexes, source, weights)


def indexed_inner_product(indexes, source_1, source_2, use_torch=False):
    """outputs[b,i] = <source_1[b], source_2[indexes[b,i]]>   (PL/gather/cuda/kernel.py:72-122)."""
    _check(indexes, source_1, source_2, "inner")
    assert source_2.dtype in [torch.float32, torch.float16], source_2.dtype
    assert source_1.dtype == source_2.dtype, (source_1.dtype, source_2.dtype)
    half_call = source_2.dtype == torch.float16       # PL/gather/cuda/kernel.py:113-116: half in, half out
    batch_size, index_size = indexes.shape
    source_size, vector_dim = source_2.shape
    assert source_1.shape[0] == batch_size and source_1.shape[1] == vector_dim
    assert index_size % 2 == 0, index_size
    assert vector_dim % 64 == 0, vector_dim

    if use_torch:
        indexes = indexes.long()
        out = []
        for batch_idx in range(batch_size):
            rows = source_2[indexes[batch_idx, :], :].reshape(index_size, vector_dim)
            out.append((source_1[batch_idx, None, :] * rows).sum(dim=-1))
        return torch.stack(out, dim=0)
    out = ops.indexed_inner_product(indexes, source_1, source_2)      # fp32 sums of exact products
    return out.half() if half_call else out


def weighted_vector_scatter_add(indexes, source, weights, output_size, use_torch=False):
    """outputs[indexes[b,i]] += weights[b,i] * source[b]   (PL/gather/cuda/kernel.py:124-173)."""
    _check(indexes, source, weights, "scatter")
    assert source.dtype in [torch.float32, torch.float16], source.dtype
    assert weights.dtype == source.dtype, (source.dtype, weights.dtype)
    half_call = source.dtype == torch.float16         # PL/gather/cuda/kernel.py:164-167: half in, half out
    batch_size, index_size = indexes.shape
    _, vector_dim = source.shape
    assert weights.shape[0] == batch_size and weights.shape[1] == index_size
    assert source.shape[0] == batch_size
    assert index_size % 2 == 0, index_size
    assert vector_dim % 64 == 0, vector_dim

    if use_torch:
        indexes = indexes.long()
        outputs = torch.zeros(output_size, vector_dim, dtype=source.dtype, device=source.device)
        for batch_idx in range(batch_size):
            inst_source = (source[batch_idx, None, :] * weights[batch_idx, :, None]).reshape(index_size, -1)
            inst_indexes = indexes[batch_idx, :, None].repeat(1, vector_dim).reshape(index_size, -1)
            outputs.scatter_add_(0, inst_indexes, inst_source)
        return outputs
    if half_call:
        # fp32 products and sums (the reference multiplies and accumulates in half), one rounding at the end
        return ops.scatter_add(indexes, source, weights.float(), output_size).half()
    return ops.scatter_add(indexes, source, weights, output_size)


class WeightedVectorGatherAdd(Function):
    """PL/gather/cuda/kernel.py:175-202: backward returns (None, grad_source, grad_weights)."""

    @staticmethod
    def forward(ctx, indexes, source, weights):
        indexes, source, weights = indexes.contiguous(), source.contiguous(), weights.contiguous()
        ctx.save_for_backward(indexes, source, weights)
        return weighted_vector_gather_add(indexes, source, weights)

    @staticmethod
    def backward(ctx, grad_outputs):
        grad_outputs = grad_outputs.contiguous()
        indexes, source, weights = ctx.saved_tensors
        if source.dtype != weights.dtype or source.dtype == torch.bfloat16:
            # 16-bit rows under fp32 weights are inference formats; the reference's half call (rows, weights
            # and gradients all half, PL/gather/cuda/kernel.py:64-67,113-116,164-167) has its backward below
            raise NotImplementedError("backward through 16-bit rows with fp32 weights is not built (inference formats)")
        grad_outputs = grad_outputs.to(source.dtype)
        grad_weights = indexed_inner_product(indexes, grad_outputs, source)
        grad_source = weighted_vector_scatter_add(indexes, grad_outputs, weights, source.shape[0])
        return None, grad_source, grad_weights


def weighted_gather_add(indexes, source, weights, use_torch=False):
    """PL/gather/cuda/kernel.py:204-208."""
    if use_torch:
        return weighted_vector_gather_add(indexes, source, weights, use_torch=use_torch)
    return WeightedVectorGatherAdd.apply(indexes, source, weights)


def gather(indices, weights, tables, training):
    """PL/gather/kernel.py:11-25.  No CPU path: CPU tensors are an error in both modes."""
    if not (indices.is_cuda and weights.is_cuda and tables.is_cuda):
        raise RuntimeError("gather: lookupffn_amd runs on the GPU only (got a CPU tensor)")
    return weighted_gather_add(indices, tables, weights)


class LookupGather(Function):
    """The gather as the layer issues it (PL/lookup.py:120-130): codes are table-local,
    the offset ``arange(T) * S`` and the output bias (PL/lookup.py:108) are folded
    into the kernel, as is an optional residual [B, Do] added to the result.  Gradients: tables,
    scores, bias and residual."""

    @staticmethod
    def forward(ctx, code, score, tables, bias, residual):
        code, score, tables = code.contiguous(), score.contiguous(), tables.contiguous()
        ctx.save_for_backward(code, score, tables)
        ctx.has_bias = bias is not None
        ctx.has_residual = residual is not None
        return ops.lookup_gather(code, score, tables, None if bias is None else bias.contiguous(),
                                 None if residual is None else residual.contiguous())

    @staticmethod
    def backward(ctx, grad_outputs):
        code, score, tables = ctx.saved_tensors
        if tables.dtype != torch.float32:
            raise NotImplementedError("backward through 16-bit tables is not built (inference formats)")
        grad_outputs = grad_outputs.contiguous()
        T, S, Do = tables.shape
        if ctx.needs_input_grad[1] and ctx.needs_input_grad[2]:
            # one call: the score gradient and the sorted scatter share the slice-major copy of the gradient
            grad_score, grad_tables = ops.lookup_backward(code, score, grad_outputs, tables)
        else:
            grad_score = ops.lookup_inner(code, grad_outputs, tables) if ctx.needs_input_grad[1] else None
            grad_tables = ops.lookup_scatter(code, score, grad_outputs, S) if ctx.needs_input_grad[2] else None
        grad_bias = ops.column_sums(grad_outputs) if (ctx.has_bias and ctx.needs_input_grad[3]) else None
        grad_residual = grad_outputs if (ctx.has_residual and ctx.needs_input_grad[4]) else None
        return None, grad_score, grad_tables, grad_bias, grad_residual


def lookup_gather(code, score, tables, bias=None, residual=None):
    if not (code.is_cuda and score.is_cuda and tables.is_cuda):
        raise RuntimeError("lookup_gather: lookupffn_amd runs on the GPU only (got a CPU tensor)")
    return LookupGather.apply(code, score, tables, bias, residual)
