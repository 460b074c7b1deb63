"""``BH4``, ``Hashing`` and ``LookupFFN``: the module surface of the reference's
PL/lookup.py (PL/ = src/roberta/models/prenorm_lookup/), with the same
constructor arguments, ``config`` attribute names, parameter names and shapes
(so a reference state_dict loads unchanged), on the gfx950 kernels.

Inference (no gradient needed) with ``block_size == 1`` and 8-bit codes runs as
LayerNorm -> one fused projection+hash kernel -> one gather kernel.  Every other
case runs the same operator sequence as the reference, each operator on its
kernel and differentiable.
"""
from __future__ import annotations

import math

import numpy as np
import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops
from .bh4 import bh4
from .compute_code_score import compute_code_score
from .gather import gather, lookup_gather


class BH4(nn.Module):
    """PL/lookup.py:10-47."""

    def __init__(self, in_dim, out_dim, block_size, decay_coeff=0.7):
        super().__init__()
        self.in_dim = in_dim
        self.out_dim = out_dim
        self.block_size = block_size
        self.decay_coeff = decay_coeff

        self.padded_in_dim = int(2 ** math.ceil(math.log2(in_dim)))
        self.num_repeat = max(1, int(math.ceil(self.out_dim / self.padded_in_dim)))
        self.num_block = self.padded_in_dim // self.block_size

        coeff = math.sqrt(self.block_size * self.padded_in_dim)
        self.weight = nn.Parameter(
            torch.randn(self.num_repeat, 4, self.num_block, self.block_size, self.block_size) / coeff)
        self.bias = nn.Parameter(torch.zeros(self.out_dim))

    def extra_repr(self):
        return (f"in_dim={self.in_dim}, out_dim={self.out_dim}, block_size={self.block_size}, "
                f"decay_coeff={self.decay_coeff}")

    def _forward(self, x):
        batch_size, dim = x.shape
        if dim < self.padded_in_dim:
            padding_dim = self.padded_in_dim - dim
            x = torch.cat([x, torch.zeros(batch_size, padding_dim, dtype=x.dtype, device=x.device)],
                          dim=-1).contiguous()
        x = (self.decay_coeff * bh4(x, self.weight, training=self.training)
             + (1 - self.decay_coeff) * x.repeat(1, self.num_repeat))
        x = x[:, :self.out_dim].contiguous() + self.bias
        return x

    def forward(self, xs):
        shape = xs.shape[:-1]
        dim = xs.shape[-1]
        xs = xs.reshape(int(np.prod(shape)), dim)
        outputs = self._forward(xs)
        return outputs.reshape(*shape, self.out_dim)


class ProjectHash(torch.autograd.Function):
    """Diagonal BH4 -> mix -> bias -> 8-bit code + score as one differentiable operator:
    one kernel forward (z is kept), one kernel backward (the stages are recomputed in
    registers).  Same mathematics as BH4._forward + compute_code_score under autograd
    (PL/lookup.py:29-39, PL/compute_code_score/kernel.py:47-53); the code has no gradient."""

    @staticmethod
    def forward(ctx, x, weight, bias, T, decay):
        R, J = weight.shape[0], weight.shape[1]
        diag = weight.reshape(R, J, -1).contiguous()
        x = x.contiguous()
        code, score, z = ops.project_hash(x, diag, bias, T, float(decay), float(1 - decay), True)
        ctx.save_for_backward(x, diag, z)
        ctx.weight_shape = weight.shape
        ctx.has_bias = bias is not None
        ctx.decay = float(decay)
        ctx.mark_non_differentiable(code)
        return code, score

    @staticmethod
    def backward(ctx, _g_code, g_score):
        x, diag, z = ctx.saved_tensors
        g_x, g_diag, g_bias = ops.project_hash_bwd(x, diag, z, g_score.contiguous(), ctx.decay, 1 - ctx.decay)
        return (g_x if ctx.needs_input_grad[0] else None,
                g_diag.reshape(ctx.weight_shape) if ctx.needs_input_grad[1] else None,
                g_bias if (ctx.has_bias and ctx.needs_input_grad[2]) else None, None, None)


class BlockProjectHash(torch.autograd.Function):
    """BH4 with 64 x 64 blocks -> mix -> bias -> 8-bit code + score as one differentiable
    operator.  Forward: one matrix-core kernel that also keeps z and the input of every stage.
    Backward: the score derivative, one matrix-core kernel walking the stages down (grad x and
    the gradient in front of every block product), then the weight gradient: a matrix-core
    kernel summing, per block, those gradients against the saved stage inputs over the tokens,
    taken back through the 64-point transform.  Same mathematics as bh4_cuda + BH4._forward + compute_code_score under
    autograd (PL/bh4/kernel.py:23-36, PL/lookup.py:29-39)."""

    @staticmethod
    def forward(ctx, x, weight, bias, T, decay):
        x = x.contiguous()
        w = weight.contiguous()
        folded = ops.bh4_fold_mode(w, 0)
        code, score, z, stage_in = ops.bh4_block_hash_train(x, folded, bias, T, float(decay), float(1 - decay))
        ctx.save_for_backward(x, w, z, stage_in)
        ctx.has_bias = bias is not None
        ctx.decay = float(decay)
        ctx.mark_non_differentiable(code)
        return code, score

    @staticmethod
    def backward(ctx, _g_code, g_score):
        x, w, z, stage_in = ctx.saved_tensors
        R, J, NB, bs, _ = w.shape
        B, H = x.shape
        T = g_score.shape[1]
        g_z = ops.code_score_bwd(z.reshape(B, T, 8), g_score.contiguous()).reshape(B, T * 8)
        g_x, stage_g = ops.bh4_block_bwd(g_z, ops.bh4_fold_mode(w, 1), H, ctx.decay, 1 - ctx.decay)
        g_w = None
        if ctx.needs_input_grad[1]:
            # stage 0 reads x (zero beyond its H columns), stage j the saved input of that stage
            g_folded = ops.bh4_block_wgrad(stage_g.reshape(R * J, B, NB * bs), x, stage_in, R, J).view_as(w)
            g_w = ops.bh4_fold_mode(g_folded, 2)
        g_x = g_x[0] if R == 1 else g_x.sum(0)
        g_bias = ops.column_sums(g_z) if (ctx.has_bias and ctx.needs_input_grad[2]) else None
        return (g_x if ctx.needs_input_grad[0] else None, g_w, g_bias, None, None)


class Hashing(nn.Module):
    """PL/lookup.py:49-77."""

    def __init__(self, config):
        super().__init__()
        self.hidden_size = config.hidden_size
        self.num_table = config.ffn_num_table
        self.table_size = config.ffn_table_size
        self.code_length = int(math.log2(self.table_size))
        self.total_dim = self.num_table * self.code_length
        if config.projection_type == "bh4":
            self.projection = BH4(self.hidden_size, self.total_dim, block_size=config.block_size)
        elif config.projection_type == "dense":
            self.projection = nn.Linear(self.hidden_size, self.total_dim)
        else:
            raise NotImplementedError

    def can_fuse(self, x):
        """One-kernel projection+hash: diagonal BH4, 8-bit codes, fp32, no gradient."""
        p = self.projection
        needs_grad = torch.is_grad_enabled() and (
            x.requires_grad or any(q.requires_grad for q in self.parameters()))
        return (isinstance(p, BH4) and p.block_size == 1 and self.code_length == 8
                and p.padded_in_dim <= 1024 and p.padded_in_dim >= 8
                and x.dtype == torch.float32 and x.is_cuda and not needs_grad)

    def forward_fused(self, x, layer_norm=None):
        """One kernel: (LayerNorm ->) diagonal BH4 -> mix -> bias -> code + score."""
        p = self.projection
        diag = p.weight.reshape(p.num_repeat, p.weight.shape[1], p.padded_in_dim).contiguous()
        if layer_norm is not None:
            code, score, _ = ops.ln_project_hash(
                x.contiguous(), layer_norm.weight, layer_norm.bias, float(layer_norm.eps), diag, p.bias,
                self.num_table, float(p.decay_coeff), float(1 - p.decay_coeff), False)
        else:
            code, score, _ = ops.project_hash(
                x.contiguous(), diag, p.bias, self.num_table,
                float(p.decay_coeff), float(1 - p.decay_coeff), False)
        return code, score

    def can_fuse_block(self, x):
        """Two kernels for 64 x 64 blocks without gradient: all BH4 stages on the matrix
        cores, then mix + bias + code + score."""
        p = self.projection
        needs_grad = torch.is_grad_enabled() and (
            x.requires_grad or any(q.requires_grad for q in self.parameters()))
        return (isinstance(p, BH4) and p.block_size == 64 and 64 <= p.padded_in_dim <= 1024
                and p.in_dim % 4 == 0 and self.code_length <= 24
                and x.dtype == torch.float32 and x.is_cuda and not needs_grad)

    def folded_weight(self):
        """The BH4 weights with the 64-point transform applied (what ops.bh4_block takes), kept
        until the parameter is modified or moved.  Modifications are seen through the tensor's
        version counter, which in-place writes through ``.data`` (``w.data.add_(...)``, some
        hand-written optimizers) do not advance: after such a write call
        ``invalidate_folded_weight()``; switching the module between train() and eval() drops
        the cached copy as well."""
        w = self.projection.weight
        key = (w._version, w.data_ptr(), w.device)
        cached = getattr(self, "_folded", None)
        if cached is None or cached[0] != key:
            cached = (key, ops.bh4_fold(w.detach().contiguous()))
            self._folded = cached
        return cached[1]

    def invalidate_folded_weight(self):
        """Forget the folded copy of the BH4 weights: the next block-64 inference call folds again."""
        self._folded = None

    def train(self, mode=True):
        if mode != self.training:
            self._folded = None           # weights usually change between an eval and the next one
        return super().train(mode)

    def forward_block(self, x, layer_norm=None):
        """8-bit codes: one kernel, (LayerNorm ->) BH4 on the matrix cores -> mix -> bias ->
        code + score.  Other code lengths: the BH4 kernel, then mix + hash in a second one."""
        p = self.projection
        x = x.contiguous()
        if self.code_length == 8:
            lw = None if layer_norm is None else layer_norm.weight
            lb = None if layer_norm is None else layer_norm.bias
            eps = 0.0 if layer_norm is None else float(layer_norm.eps)
            return ops.ln_bh4_block_hash(x, lw, lb, eps, self.folded_weight(), p.bias, self.num_table,
                                         float(p.decay_coeff), float(1 - p.decay_coeff))
        if layer_norm is not None:
            x = layer_norm(x)
        y = ops.bh4_block(x, self.folded_weight())
        return ops.mix_code_score(y, x, p.bias, self.num_table, self.code_length, p.padded_in_dim,
                                  float(p.decay_coeff), float(1 - p.decay_coeff))

    def can_fuse_training(self, x):
        """The differentiable one-kernel form: diagonal BH4 with at most 4 stages, 8-bit codes,
        256 <= D <= 1024, fp32."""
        p = self.projection
        return (isinstance(p, BH4) and p.block_size == 1 and self.code_length == 8
                and 256 <= p.padded_in_dim <= 1024 and p.weight.shape[1] <= 4 and p.in_dim % 4 == 0
                and x.dtype == torch.float32 and x.is_cuda and p.weight.dtype == torch.float32)

    def can_fuse_block_training(self, x):
        """The differentiable matrix-core form: 64 x 64 blocks, 8-bit codes, D <= 1024, fp32."""
        p = self.projection
        return (isinstance(p, BH4) and p.block_size == 64 and self.code_length == 8
                and 64 <= p.padded_in_dim <= 1024 and p.in_dim % 4 == 0
                and x.dtype == torch.float32 and x.is_cuda and p.weight.dtype == torch.float32)

    def forward(self, x):
        B, D = x.shape
        if self.can_fuse(x):                      # no gradient needed: the inference kernels
            return self.forward_fused(x)
        if self.can_fuse_block(x):
            return self.forward_block(x)
        if self.can_fuse_training(x):
            p = self.projection
            return ProjectHash.apply(x, p.weight, p.bias, self.num_table, p.decay_coeff)
        if self.can_fuse_block_training(x):
            p = self.projection
            return BlockProjectHash.apply(x, p.weight, p.bias, self.num_table, p.decay_coeff)
        z = self.projection(x)
        z = z.reshape(B, self.num_table, self.code_length)
        code, score = compute_code_score(z, training=self.training)
        return code, score


class LayerNormFn(torch.autograd.Function):
    """torch's LayerNorm forward with a one-kernel backward (ops.layer_norm_bwd): mean and 1/sigma are
    recomputed from the input, the weight and bias gradients come out of the same pass."""

    @staticmethod
    def forward(ctx, x, weight, bias, eps):
        ctx.save_for_backward(x, weight)
        ctx.eps = float(eps)
        return F.layer_norm(x, (x.shape[-1],), weight, bias, eps)

    @staticmethod
    def backward(ctx, g_y):
        x, weight = ctx.saved_tensors
        g_x, g_w, g_b = ops.layer_norm_bwd(x, weight, ctx.eps, g_y.contiguous()[None])
        return (g_x if ctx.needs_input_grad[0] else None, g_w if ctx.needs_input_grad[1] else None,
                g_b if ctx.needs_input_grad[2] else None, None)


class LnProjectHash(torch.autograd.Function):
    """LayerNorm -> diagonal BH4 -> mix -> bias -> 8-bit code + score as one differentiable operator
    (PL/lookup.py:99, 29-39, PL/compute_code_score/kernel.py:47-53).  Forward: the inference kernel
    with z kept.  Backward: the projection's backward with LayerNorm recomputed on load, then the
    LayerNorm backward kernel; the normalised activations are never stored."""

    @staticmethod
    def forward(ctx, x, ln_weight, ln_bias, eps, weight, bias, T, decay):
        R, J = weight.shape[0], weight.shape[1]
        diag = weight.reshape(R, J, -1).contiguous()
        x = x.contiguous()
        code, score, z = ops.ln_project_hash(x, ln_weight, ln_bias, float(eps), diag, bias, T, float(decay),
                                             float(1 - decay), True)
        ctx.save_for_backward(x, ln_weight, ln_bias, diag, z)
        ctx.eps = float(eps)
        ctx.weight_shape = weight.shape
        ctx.has_bias = bias is not None
        ctx.decay = float(decay)
        ctx.mark_non_differentiable(code)
        return code, score

    @staticmethod
    def backward(ctx, _g_code, g_score):
        x, ln_weight, ln_bias, diag, z = ctx.saved_tensors
        g_h, g_diag, g_bias = ops.project_hash_bwd(x, diag, z, g_score.contiguous(), ctx.decay, 1 - ctx.decay,
                                                   ln_weight, ln_bias, ctx.eps)
        need = ctx.needs_input_grad
        g_x = g_lw = g_lb = None
        if need[0] or need[1] or need[2]:
            g_x, g_lw, g_lb = ops.layer_norm_bwd(x, ln_weight, ctx.eps, g_h)
        return (g_x if need[0] else None, g_lw if need[1] else None, g_lb if need[2] else None, None,
                g_diag.reshape(ctx.weight_shape) if need[4] else None,
                g_bias if (ctx.has_bias and need[5]) else None, None, None)


class LnBlockProjectHash(torch.autograd.Function):
    """LayerNorm -> BH4 with 64 x 64 blocks -> mix -> bias -> 8-bit code + score as one differentiable operator
    (PL/lookup.py:99 in front of PL/bh4/kernel.py:23-36 and PL/lookup.py:29-39).  Forward: BlockProjectHash's
    kernel with LayerNorm run on the token tile as it is loaded; it keeps every row's mean and 1/sigma
    instead of the normalised rows.  Backward: BlockProjectHash's, with the weight-gradient kernel forming
    LayerNorm(x) on load for the first stage of every repeat, then the LayerNorm backward kernel."""

    @staticmethod
    def forward(ctx, x, ln_weight, ln_bias, eps, weight, bias, T, decay):
        x = x.contiguous()
        w = weight.contiguous()
        folded = ops.bh4_fold_mode(w, 0)
        code, score, z, stage_in, stats = ops.ln_bh4_block_hash_train(x, ln_weight, ln_bias, float(eps), folded, bias, T,
                                                                      float(decay), float(1 - decay))
        ctx.save_for_backward(x, ln_weight, ln_bias, w, z, stage_in, stats)
        ctx.eps = float(eps)
        ctx.has_bias = bias is not None
        ctx.decay = float(decay)
        ctx.mark_non_differentiable(code)
        return code, score

    @staticmethod
    def backward(ctx, _g_code, g_score):
        x, ln_weight, ln_bias, w, z, stage_in, stats = ctx.saved_tensors
        R, J, NB, bs, _ = w.shape
        B, H = x.shape
        T = g_score.shape[1]
        need = ctx.needs_input_grad
        g_z = ops.code_score_bwd(z.reshape(B, T, 8), g_score.contiguous()).reshape(B, T * 8)
        g_h, stage_g = ops.bh4_block_bwd(g_z, ops.bh4_fold_mode(w, 1), H, ctx.decay, 1 - ctx.decay)
        g_w = None
        if need[4]:
            g_folded = ops.ln_bh4_block_wgrad(stage_g.reshape(R * J, B, NB * bs), x, ln_weight, ln_bias, stats, stage_in,
                                              R, J).view_as(w)
            g_w = ops.bh4_fold_mode(g_folded, 2)
        g_x = g_lw = g_lb = None
        if need[0] or need[1] or need[2]:
            g_x, g_lw, g_lb = ops.layer_norm_bwd(x, ln_weight, ctx.eps, g_h)      # adds the R repeats' gradients
        g_bias = ops.column_sums(g_z) if (ctx.has_bias and need[5]) else None
        return (g_x if need[0] else None, g_lw if need[1] else None, g_lb if need[2] else None, None, g_w, g_bias,
                None, None)


class LookupFFN(nn.Module):
    """PL/lookup.py:79-130."""

    def __init__(self, config, output_size):
        super().__init__()
        self.hidden_size = config.hidden_size
        self.output_size = output_size
        self.LayerNorm = nn.LayerNorm(self.hidden_size, eps=config.layer_norm_eps)

        self.num_table = config.ffn_num_table
        self.table_size = config.ffn_table_size
        assert (2 ** int(math.log2(self.table_size))) == self.table_size
        self.hash = Hashing(config)
        self.tables = nn.Parameter(0.02 * torch.randn(self.num_table, self.table_size, self.output_size))
        self.bias = nn.Parameter(0.001 * torch.randn(self.output_size))

    def __getstate__(self):
        # the cached parameter views are derived data: not pickled with the module
        state = super().__getstate__() if hasattr(super(), "__getstate__") else self.__dict__.copy()
        state = dict(state)
        state.pop("_inference_cache", None)
        return state

    def extra_repr(self):
        return (f"hidden_size={self.hidden_size}, num_table={self.num_table}, "
                f"table_size={self.table_size}, output_size={self.output_size}")

    # Up to this many tokens the one-launch form of the layer (a wavefront per token: LayerNorm,
    # projection, hash and the token's gather-add) beats the projection kernel followed by the
    # table-major gather, which stages every table slice in LDS and needs many tokens to pay for it.
    FUSED_LAYER_MAX_TOKENS = 512

    def _no_gradient_wanted(self, x):
        return not (torch.is_grad_enabled()
                    and (x.requires_grad or any(q.requires_grad for q in self.parameters())))

    def can_fuse_layer(self, x):
        """The one-launch form applies: few tokens, fp32 on the GPU, no gradient wanted, and parameters
        of the kind it is built for (diagonal BH4, 8-bit codes, 256-entry fp32 tables)."""
        if not (x.shape[0] <= self.FUSED_LAYER_MAX_TOKENS and x.is_cuda and x.dtype == torch.float32
                and self._no_gradient_wanted(x)):
            return False
        st = self._inference_state()
        return st is not None and st["one_launch"]

    def _inference_state(self):
        """What the inference kernels take from the parameters, or None when the parameters are not of
        a kind those kernels are built for; worked out once and kept until a parameter is replaced,
        moved or cast (in-place updates keep the storage, so the cached views stay good).  A launch
        is a few microseconds: re-deriving this on every call cost more than the kernels at small
        batches.  Keys: form ("diag": one kernel for LayerNorm + diagonal BH4 + hash; "block": the
        matrix-core kernel for 64 x 64 blocks), one_launch (the whole layer in one kernel is possible),
        and the detached parameter views."""
        p = self.hash.projection
        ln = self.LayerNorm
        params = (ln.weight, ln.bias, getattr(p, "weight", None), getattr(p, "bias", None), self.tables, self.bias)
        key = tuple((id(q), q.data_ptr(), q.dtype) if q is not None else None for q in params)
        cached = getattr(self, "_inference_cache", None)
        if cached is not None and cached[0] == key:
            return cached[1]
        small = (ln.weight, ln.bias, getattr(p, "weight", None), getattr(p, "bias", None), self.bias)
        ok = (isinstance(p, BH4) and self.hash.code_length == 8 and ln.elementwise_affine
              and ln.weight is not None and ln.bias is not None and p.in_dim == self.hidden_size
              and all(q is None or (q.dtype == torch.float32 and q.is_cuda and q.is_contiguous()
                                    and q.device == self.tables.device) for q in small)
              and self.tables.is_cuda and self.tables.is_contiguous()
              and ops.row_format(self.tables.dtype) is not None and self.output_size % 64 == 0)
        form = None
        if ok and p.block_size == 1 and 8 <= p.padded_in_dim <= 1024:
            form = "diag"
        elif ok and p.block_size == 64 and 64 <= p.padded_in_dim <= 1024 and p.in_dim % 4 == 0:
            form = "block"
        state = None
        if form is not None:
            state = dict(
                form=form,
                one_launch=(form == "diag" and p.padded_in_dim >= 256 and self.num_table <= 512
                            and self.table_size == 256 and self.tables.dtype == torch.float32),
                ln_w=ln.weight.detach(), ln_b=ln.bias.detach(), eps=float(ln.eps),
                diag=(p.weight.detach().reshape(p.num_repeat, p.weight.shape[1], p.padded_in_dim)
                      if form == "diag" else None),
                pbias=None if p.bias is None else p.bias.detach(), tables=self.tables.detach(),
                obias=self.bias.detach(), decay=float(p.decay_coeff), res_coef=float(1 - p.decay_coeff))
            if state["one_launch"]:
                state["block"] = ops.fused_layer_block(state["ln_w"], state["ln_b"], state["eps"], state["diag"], state["pbias"],
                                                       state["tables"], state["obias"], state["decay"], state["res_coef"])
        self._inference_cache = (key, state)
        return state

    def _forward_inference(self, x, residual, st):
        """No gradient wanted and parameters the inference kernels are built for: the entry points
        are called without the operator dispatcher or autograd (same kernels, same results)."""
        x = x.contiguous()
        if residual is not None:
            # forward() hands over fp32 of shape [tokens, output_size]; anything else is a caller's mistake
            if (residual.dtype != torch.float32 or residual.device != x.device
                    or tuple(residual.shape) != (x.shape[0], self.output_size)):
                raise ValueError("residual: fp32 [tokens, output_size] on the input's device")
            residual = residual.contiguous()
        if st["one_launch"] and x.shape[0] <= self.FUSED_LAYER_MAX_TOKENS:
            # small batches: the whole layer in one launch
            return ops.lookup_ffn_fused_block(st["block"], x, residual)
        if self.num_table % 2 == 0:
            # many tokens: the projection kernel writes the gather kernel's record stream directly
            plan = ops.lookup_gather_records_plan(x.shape[0], self.num_table, self.table_size, self.output_size,
                                                  ops.row_format(st["tables"].dtype))
            records = None
            if plan is not None and st["form"] == "diag" and st["diag"].shape[2] >= 16:
                records = ops.ln_project_hash_records_direct(x, st["ln_w"], st["ln_b"], st["eps"], st["diag"], st["pbias"],
                                                             self.num_table, st["decay"], st["res_coef"], plan)
            elif plan is not None and st["form"] == "block":
                records = ops.ln_bh4_block_hash_records_direct(x, st["ln_w"], st["ln_b"], st["eps"], self.hash.folded_weight(),
                                                               st["pbias"], self.num_table, st["decay"], st["res_coef"], plan)
            if records is not None:
                return ops.lookup_gather_records_direct(records, plan, st["tables"], st["obias"], residual, x.shape[0])
        if st["form"] == "diag":
            code, score, _ = ops.ln_project_hash_direct(x, st["ln_w"], st["ln_b"], st["eps"], st["diag"], st["pbias"],
                                                        self.num_table, st["decay"], st["res_coef"], False)
        else:
            code, score = ops.ln_bh4_block_hash_direct(x, st["ln_w"], st["ln_b"], st["eps"], self.hash.folded_weight(),
                                                       st["pbias"], self.num_table, st["decay"], st["res_coef"])
        return ops.lookup_gather_direct(code, score, st["tables"], st["obias"], residual)

    def _forward(self, hidden_states, residual=None):
        if (hidden_states.is_cuda and hidden_states.dtype == torch.float32 and not torch.compiler.is_compiling()
                and self._no_gradient_wanted(hidden_states)):
            st = self._inference_state()
            if st is not None:
                return self._forward_inference(hidden_states, residual, st)
        ln = self.LayerNorm
        ln_fusable = (ln.elementwise_affine and ln.weight is not None and ln.bias is not None
                      and ln.weight.dtype == torch.float32
                      and not (torch.is_grad_enabled() and (ln.weight.requires_grad or ln.bias.requires_grad)))
        if ln_fusable and self.hash.can_fuse(hidden_states):
            # inference: LayerNorm runs inside the projection kernel
            code, score = self.hash.forward_fused(hidden_states, layer_norm=ln)
        elif ln_fusable and self.hash.can_fuse_block(hidden_states):
            code, score = self.hash.forward_block(hidden_states, layer_norm=ln)
        else:
            ln_kernel_ok = (torch.is_grad_enabled() and hidden_states.is_cuda and hidden_states.dtype == torch.float32
                            and ln.elementwise_affine and ln.weight is not None and ln.bias is not None
                            and ln.weight.dtype == torch.float32 and self.hidden_size % 4 == 0
                            and self.hidden_size <= 1024)
            if ln_kernel_ok and self.hash.can_fuse_training(hidden_states):
                # training, diagonal BH4: LayerNorm inside the projection kernel forward and backward
                p = self.hash.projection
                code, score = LnProjectHash.apply(hidden_states, ln.weight, ln.bias, ln.eps, p.weight, p.bias,
                                                  self.num_table, p.decay_coeff)
            elif ln_kernel_ok and self.hash.can_fuse_block_training(hidden_states):
                # training, 64 x 64 blocks: LayerNorm inside the matrix-core kernel; the weight gradient forms it again on load
                p = self.hash.projection
                code, score = LnBlockProjectHash.apply(hidden_states, ln.weight, ln.bias, ln.eps, p.weight, p.bias,
                                                       self.num_table, p.decay_coeff)
            elif ln_kernel_ok:
                hidden_states = LayerNormFn.apply(hidden_states.contiguous(), ln.weight, ln.bias, ln.eps)
                code, score = self.hash(hidden_states)
            else:
                hidden_states = ln(hidden_states)
                code, score = self.hash(hidden_states)
        if self.output_size % 64 == 0 and ops.row_format(self.tables.dtype) is not None:
            # table-local codes, offset and bias folded into the gather kernel
            return lookup_gather(code, score.float(), self.tables, self.bias.float(), residual)
        outputs = self.gather(code, score, self.tables)
        outputs = outputs + self.bias
        return outputs if residual is None else outputs + residual

    def forward(self, hidden_states, residual=None):
        """PL/lookup.py:110-118.  ``residual`` (not in the reference; shape [..., output_size]) is
        added to the result inside the gather kernel: the encoder layer's "FFN(x) + x"."""
        if hidden_states.dim() == 2 and residual is None:
            # already [tokens, hidden]: nothing to reshape (at a few hundred tokens the layer is one launch of
            # a few microseconds and every view made here shows in its time)
            return self._forward(hidden_states, None)
        shape = hidden_states.shape[:-1]
        dim = hidden_states.shape[-1]
        tokens = math.prod(shape)
        hidden_states = hidden_states.reshape(tokens, dim)
        if residual is not None:
            residual = residual.reshape(tokens, self.output_size).float()
        outputs = self._forward(hidden_states, residual)
        return outputs.reshape(*shape, self.output_size)

    def gather(self, indexes, weights, tables):
        """PL/lookup.py:120-130: flat row numbers, then the general gather."""
        B, N = indexes.shape
        num_table, table_size, vector_dim = tables.shape
        assert weights.shape[0] == B
        assert weights.shape[1] == N
        indexes = indexes + torch.arange(num_table, device=indexes.device, dtype=indexes.dtype)[None] * table_size
        tables = tables.reshape(num_table * table_size, vector_dim)
        return gather(indexes, weights, tables, training=self.training)
