"""Decoder-only language model built on `HierarchicalAttention`: the caller of the hot path.

Restates the model of the reference's training script
(hierarchical_attention_project/Hierarchical_Transformer_Pretrain.py:331-481) with the same
sub-module names, so its checkpoints (`model_state_dict`, optionally with a `module.` prefix)
load unchanged.  Differences: the feed-forward activation is selectable (the reference uses
ReLU), and the causal "mask" handed to the attention is a one-element tensor, because only its
presence is ever looked at (an N x N mask costs 16 MB at N=4096 and is never read).
"""
from __future__ import annotations

import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from .modules import HierarchicalAttention
from .ops import generate_span_input_Y


class PositionwiseFeedForward(nn.Module):
    def __init__(self, d_model: int, d_ff: int, dropout: float = 0.1, activation: str = "relu"):
        super().__init__()
        self.fc1 = nn.Linear(d_model, d_ff)
        self.fc2 = nn.Linear(d_ff, d_model)
        self.dropout = nn.Dropout(p=dropout)
        self.activation = {"relu": F.relu, "gelu": F.gelu}[activation]

    def forward(self, x):
        return self.fc2(self.dropout(self.activation(self.fc1(x))))


class PositionalEncoding(nn.Module):
    def __init__(self, d_model: int, dropout: float, max_len: int = 5000):
        super().__init__()
        self.dropout = nn.Dropout(p=dropout)
        pos = torch.arange(0.0, max_len).unsqueeze(1)
        freq = torch.exp(torch.arange(0.0, d_model, 2) * -(math.log(10000.0) / d_model))
        pe = torch.zeros(max_len, d_model)
        pe[:, 0::2] = torch.sin(pos * freq)
        pe[:, 1::2] = torch.cos(pos * freq)
        self.register_buffer("pe", pe.unsqueeze(0))

    def forward(self, x):
        return self.dropout(x + self.pe[:, :x.size(1), :].to(x.dtype))


class DecoderLayer(nn.Module):
    def __init__(self, d_model, num_heads, d_ff, dropout=0.1, window_size=16, activation="relu"):
        super().__init__()
        self.self_attn = HierarchicalAttention(d_model, num_heads, dropout, window_size=window_size)
        self.feed_forward = PositionwiseFeedForward(d_model, d_ff, dropout, activation)
        self.norm1 = nn.LayerNorm(d_model)
        self.norm2 = nn.LayerNorm(d_model)
        self.norm_y = nn.LayerNorm(d_model)
        # present in the reference's checkpoints, unused by its forward
        self.alpha_proj = nn.Linear(d_model, d_model)
        self.beta_proj = nn.Linear(d_model, d_model)
        self.dropout = nn.Dropout(dropout)

    def forward(self, x, y, mask=None, return_attention=False):
        # span nodes first: un-normalised leaves, normalised nodes; plain residual
        y = y + self.dropout(self.self_attn.cross_update_Y(x, y_in=self.norm_y(y)))
        # leaves: pre-norm attention over the window and the updated nodes
        nx = self.norm1(x)
        if return_attention:
            a, w = self.self_attn(nx, nx, nx, y=y, mask=mask, return_attention=True)
        else:
            a, w = self.self_attn(nx, nx, nx, y=y, mask=mask), None
        x = x + self.dropout(a)
        x = x + self.dropout(self.feed_forward(self.norm2(x)))
        return (x, y, w) if return_attention else (x, y)


class TransformerLM(nn.Module):
    def __init__(self, vocab_size, d_model, num_heads, d_ff, num_layers, dropout=0.1, window_size=16,
                 activation="relu", max_len=5000):
        super().__init__()
        self.embedding = nn.Embedding(vocab_size, d_model)
        self.pos_encoding = PositionalEncoding(d_model, dropout=dropout, max_len=max_len)
        self.layers = nn.ModuleList(
            [DecoderLayer(d_model, num_heads, d_ff, dropout, window_size, activation) for _ in range(num_layers)])
        self.fc_out = nn.Linear(d_model, vocab_size)
        self.fc_out.weight = self.embedding.weight  # tied
        self.d_model = d_model
        self.apply(self._init_weights)

    @staticmethod
    def _init_weights(m):
        if isinstance(m, nn.Linear):
            nn.init.normal_(m.weight, mean=0.0, std=0.02)
            if m.bias is not None:
                nn.init.zeros_(m.bias)
        elif isinstance(m, nn.Embedding):
            nn.init.normal_(m.weight, mean=0.0, std=0.02)

    def make_causal_mask(self, x):
        """Only `mask is not None` is ever tested downstream."""
        return torch.ones(1, 1, 1, 1, dtype=torch.bool, device=x.device)

    def forward(self, trg, return_attention=False):
        x = self.pos_encoding(self.embedding(trg) * math.sqrt(self.d_model))
        y = generate_span_input_Y(x)
        mask = self.make_causal_mask(trg)
        for layer in self.layers:
            if return_attention:
                x, y, _ = layer(x, y, mask=mask, return_attention=True)
            else:
                x, y = layer(x, y, mask=mask)
        return self.fc_out(x)

    def generate(self, src, start_token=2, max_len=50, temperature=1.0):
        """Samples up to `max_len` tokens after the prompt `src`, one full forward per token, and
        stops at the end-of-sequence id 3 (Hierarchical_Transformer_Pretrain.py:483-505).  As in the
        reference every forward needs a power-of-two length, so only prompts whose length stays a
        power of two while tokens are appended get past the first step."""
        self.eval()
        device = next(self.parameters()).device
        tokens = src.to(device)
        if tokens.dim() == 1:
            tokens = tokens.unsqueeze(0)
        with torch.no_grad():
            for _ in range(max_len):
                logits = self.forward(tokens)
                probs = torch.softmax(logits[:, -1, :] / temperature, dim=-1)
                nxt = torch.multinomial(probs, 1)
                tokens = torch.cat([tokens, nxt], dim=1)
                if nxt.item() == 3:
                    break
        return tokens

    def load_reference_checkpoint(self, state):
        """Loads a reference checkpoint dict (`{'model_state_dict': ...}` or a bare state dict,
        keys optionally prefixed with `module.`)."""
        sd = state.get("model_state_dict", state)
        sd = {(k[7:] if k.startswith("module.") else k): v for k, v in sd.items()}
        return self.load_state_dict(sd)
