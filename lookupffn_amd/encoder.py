"""The caller of the hot path: the reference's pre-norm encoder with LookupFFN in
place of the feed-forward block (PL/layer.py, PL/encoder.py, and the embeddings
of src/roberta/models/postnorm.py:6-28), with the same module and parameter
names so that a reference state_dict loads unchanged.  Attention, embeddings
and LayerNorms are plain PyTorch-ROCm; only ``LookupFFN`` runs on the gfx950
kernels of this package.

``config`` carries the attributes the reference reads: hidden_size,
num_attention_heads, attention_head_size, attention_probs_dropout_prob,
hidden_dropout_prob, layer_norm_eps, num_hidden_layers, vocab_size,
max_position_embeddings, type_vocab_size, pad_token_id, plus LookupFFN's
(ffn_num_table, ffn_table_size, projection_type, block_size) and optionally
checkpoint_attention.
"""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch.utils.checkpoint import checkpoint

from .lookup import LookupFFN


class RobertaEmbeddings(nn.Module):
    """word + token-type + position embeddings, LayerNorm, dropout
    (src/roberta/models/postnorm.py:6-28); positions are offset by pad_token_id + 1."""

    def __init__(self, config):
        super().__init__()
        self.pad_token_id = config.pad_token_id
        self.word_embeddings = nn.Embedding(config.vocab_size, config.hidden_size)
        self.position_embeddings = nn.Embedding(config.max_position_embeddings + 2, config.hidden_size)
        self.token_type_embeddings = nn.Embedding(config.type_vocab_size, config.hidden_size)
        self.LayerNorm = nn.LayerNorm(config.hidden_size, eps=config.layer_norm_eps)
        self.dropout = nn.Dropout(config.hidden_dropout_prob)

    def forward(self, input_ids, token_type_ids, position_ids):
        x = (self.word_embeddings(input_ids)
             + self.token_type_embeddings(token_type_ids)
             + self.position_embeddings(position_ids + (self.pad_token_id + 1)))
        return self.dropout(self.LayerNorm(x))


class Attention(nn.Module):
    """Pre-norm multi-head self-attention (PL/layer.py:11-64): LayerNorm, q/k/v
    projections, softmax(q k^T / sqrt(d) - 1000 * (1 - mask)) v in float32, output
    projection.  ``fused=True`` evaluates the same expression with
    scaled_dot_product_attention; ``fused=False`` is the reference's literal
    sequence of matmuls."""

    def __init__(self, config, fused=True):
        super().__init__()
        self.num_attention_heads = config.num_attention_heads
        self.attention_head_size = config.attention_head_size
        self.all_head_size = self.num_attention_heads * self.attention_head_size
        self.dropout = nn.Dropout(config.attention_probs_dropout_prob)
        self.checkpoint_attention = bool(getattr(config, "checkpoint_attention", False))
        self.fused = fused

        self.LayerNorm = nn.LayerNorm(config.hidden_size, eps=config.layer_norm_eps)
        self.query = nn.Linear(config.hidden_size, config.hidden_size)
        self.key = nn.Linear(config.hidden_size, config.hidden_size)
        self.value = nn.Linear(config.hidden_size, config.hidden_size)
        self.dense = nn.Linear(config.hidden_size, config.hidden_size)

    def transpose_for_scores(self, x):
        return x.view(*x.shape[:-1], self.num_attention_heads, self.attention_head_size).permute(0, 2, 1, 3)

    def attention(self, query_layer, key_layer, value_layer, attention_mask):
        bias = -1000.0 * (1.0 - attention_mask[:, None, None, :].float())
        q, k, v = query_layer.float(), key_layer.float(), value_layer.float()
        if self.fused:
            ctx = F.scaled_dot_product_attention(q, k, v, attn_mask=bias,
                                                 dropout_p=self.dropout.p if self.training else 0.0)
        else:
            scale = self.attention_head_size ** 0.25
            probs = torch.softmax(torch.matmul(q / scale, (k / scale).transpose(-1, -2)) + bias, dim=-1)
            ctx = torch.matmul(self.dropout(probs), v)
        return ctx.to(value_layer.dtype)

    def forward(self, hidden_states, attention_mask):
        h = self.LayerNorm(hidden_states)
        q = self.transpose_for_scores(self.query(h))
        k = self.transpose_for_scores(self.key(h))
        v = self.transpose_for_scores(self.value(h))
        if self.checkpoint_attention:
            ctx = checkpoint(self.attention, q, k, v, attention_mask, use_reentrant=False)
        else:
            ctx = self.attention(q, k, v, attention_mask)
        ctx = ctx.permute(0, 2, 1, 3).contiguous()
        return self.dense(ctx.view(*ctx.shape[:-2], self.all_head_size))


class EncoderLayer(nn.Module):
    """attention + residual, LookupFFN + residual (PL/layer.py:66-78)."""

    def __init__(self, config):
        super().__init__()
        self.hidden_size = config.hidden_size
        self.FFN = LookupFFN(config, self.hidden_size)
        self.attention = Attention(config)
        self.dropout = nn.Dropout(p=config.hidden_dropout_prob)

    def forward(self, hidden_states, attention_mask):
        attn_output = self.dropout(self.attention(hidden_states, attention_mask)) + hidden_states
        if (not self.training or self.dropout.p == 0.0) and attn_output.dtype == torch.float32:
            # dropout is the identity: the residual add runs inside the FFN's gather kernel
            return self.FFN(attn_output, residual=attn_output)
        return self.dropout(self.FFN(attn_output)) + attn_output


class Encoder(nn.Module):
    """PL/encoder.py:9-19."""

    def __init__(self, config):
        super().__init__()
        self.layer = nn.ModuleList([EncoderLayer(config) for _ in range(config.num_hidden_layers)])
        self.LayerNorm = nn.LayerNorm(config.hidden_size, eps=config.layer_norm_eps)

    def forward(self, hidden_states, attention_mask):
        for layer_module in self.layer:
            hidden_states = layer_module(hidden_states, attention_mask)
        return self.LayerNorm(hidden_states)


class Lookup(nn.Module):
    """PL/encoder.py:21-37: embeddings + encoder; returns (sequence_output, {})."""

    def __init__(self, config):
        super().__init__()
        self.config = config
        self.embeddings = RobertaEmbeddings(config)
        self.encoder = Encoder(config)

    def forward(self, input_ids, token_type_ids, position_ids, attention_mask, **kwargs):
        embedding_output = self.embeddings(input_ids, token_type_ids, position_ids)
        return self.encoder(embedding_output, attention_mask), {}

    def get_input_embeddings(self):
        return self.embeddings.word_embeddings

    def set_input_embeddings(self, value):
        self.embeddings.word_embeddings = value
