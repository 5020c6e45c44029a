"""`HierarchicalAttention`: the nn.Module around the two ops.

Parameter names, shapes and method signatures follow the reference's
hierarchical_attention/modules/attention.py:10-270 so that its state dicts load
unchanged; the dense projections are torch's own `nn.Linear`, the tree build and
the span attention are the HIP kernels.
"""
from __future__ import annotations

import math
from typing import List, Optional

import torch
import torch.nn as nn

from ..ops.functional import build_parent_nodes, build_parents_forward, hierarchical_attention
from ..ops.topology import build_tree_topology


def _level_sizes(n_leaves: int) -> List[int]:
    sizes, cur = [], n_leaves
    while cur > 1:
        cur //= 2
        sizes.append(cur)
    return sizes


class HierarchicalAttention(nn.Module):
    def __init__(self, dim: int, num_heads: int, dropout: float = 0.1, window_size: int = 16):
        super().__init__()
        assert dim % num_heads == 0, "dim must be divisible by num_heads"
        self.dim, self.num_heads, self.head_dim = dim, num_heads, dim // num_heads
        self.window_size = window_size
        # bottom-up (span nodes)
        self.Wq_y = nn.Linear(dim, dim, bias=False)
        self.Wk_y = nn.Linear(dim, dim, bias=False)
        self.Wv_y = nn.Linear(dim, dim, bias=False)
        self.out_proj_y = nn.Linear(dim, dim)
        # top-down (leaves)
        self.Wq_x = nn.Linear(dim, dim, bias=False)
        self.Wk_x = nn.Linear(dim, dim, bias=False)
        self.Wv_x = nn.Linear(dim, dim, bias=False)
        self.out_proj_x = nn.Linear(dim, dim)
        self.dropout = nn.Dropout(dropout)
        # topology cache: one set of tables per (length, causal, device)
        self.cached_tables = None
        self.cached_seq_len = -1
        self.cached_is_causal = None
        self.sizes: Optional[List[int]] = None
        self.offsets: Optional[List[int]] = None

    # -- helpers -------------------------------------------------------------
    def _get_lookup_table(self, L: int, is_causal: bool, device: torch.device):
        t = self.cached_tables
        if (t is None or self.cached_seq_len != L or self.cached_is_causal != is_causal
                or t["forward_idx"].device != device):
            t = build_tree_topology(L, is_causal=is_causal, device=device)
            self.cached_tables, self.cached_seq_len, self.cached_is_causal = t, L, is_causal
        return t

    def _build_level_info(self, N: int):
        sizes = _level_sizes(N)
        offsets = [0]
        for s in sizes[:-1]:
            offsets.append(offsets[-1] + s)
        return sizes, offsets

    def _heads(self, t: torch.Tensor) -> torch.Tensor:
        return t.view(t.shape[0], -1, self.num_heads, self.head_dim)

    # -- bottom-up: leaves -> span nodes ----------------------------------------
    def cross_update_Y(self, x: torch.Tensor, y_in: torch.Tensor) -> torch.Tensor:
        B, N, D = x.shape
        assert y_in is not None, "y_in cannot be None"
        assert y_in.size(1) == N - 1, \
            f"y_in size {y_in.size(1)} mismatch! Expected N-1 ({N-1}) for N={N} leaves."
        if self.sizes is None or self.sizes[0] != N // 2:
            self.sizes, self.offsets = self._build_level_info(N)

        q_lv = torch.split(self._heads(self.Wq_y(y_in)), self.sizes, dim=1)
        k_lv = torch.split(self._heads(self.Wk_y(y_in)), self.sizes, dim=1)
        v_lv = torch.split(self._heads(self.Wv_y(y_in)), self.sizes, dim=1)

        # Without autograd the level outputs go straight into one [B, N-1, D] buffer (no
        # concatenation afterwards); with autograd each level is a differentiable op.
        direct = not (torch.is_grad_enabled() and (x.requires_grad or y_in.requires_grad
                                                    or self.Wq_y.weight.requires_grad))
        y_new = torch.empty((B, N - 1, D), dtype=x.dtype, device=x.device) if direct else None
        levels, src, off = [], x, 0
        for lvl, P in enumerate(self.sizes):
            k_c = self._heads(self.Wk_y(src))
            v_c = self.dropout(self._heads(self.Wv_y(src)))
            if lvl == 0:
                v_c = self.dropout(v_c)  # the leaf values pass through dropout twice
            if direct:
                dst = y_new[:, off:off + P]
                build_parents_forward(q_lv[lvl], k_lv[lvl], v_lv[lvl], k_c, v_c,
                                      out=dst.view(B, P, self.num_heads, self.head_dim))
                src = dst
            else:
                src = build_parent_nodes(q_lv[lvl], k_lv[lvl], v_lv[lvl], k_c, v_c).reshape(B, P, D)
                levels.append(src)
            off += P
        return self.out_proj_y(y_new if direct else torch.cat(levels, dim=1))

    # -- top-down: span nodes -> leaves -------------------------------------------
    def update_X_from_Y(self, x: torch.Tensor, y: torch.Tensor,
                        mask: Optional[torch.Tensor] = None) -> torch.Tensor:
        B, N, D = x.shape
        assert y is not None, "y (parents) cannot be None during top-down update"
        xy = torch.cat([x, y], dim=1)
        q = self._heads(self.Wq_x(x))
        k = self._heads(self.Wk_x(xy))
        v = self.dropout(self._heads(self.Wv_x(xy)))
        is_causal = mask is not None  # only the presence of a mask is looked at
        t = self._get_lookup_table(N, is_causal, x.device)
        heads = hierarchical_attention(q, k, v, t["forward_idx"], t["backward_gather"],
                                       t["forward_mask"] if is_causal else None, self.window_size)
        return self.out_proj_x(heads.view(B, N, D))

    def _standard_attention(self, Q, K, V, mask):
        scores = torch.matmul(Q, K.transpose(-1, -2)) / math.sqrt(Q.size(-1))
        if mask is not None:
            scores = scores.masked_fill(mask == 0, float("-inf"))
        attn = self.dropout(torch.softmax(scores, dim=-1))
        return torch.matmul(attn, V), attn

    def forward(self, query, key, value, y=None, mask=None, return_attention=False):
        B, Lq, D = query.shape
        if y is not None and Lq == key.size(1) == value.size(1):
            out = self.update_X_from_Y(query, y, mask)
            return (out, None) if return_attention else out
        # dense fallback when no span nodes are given or the lengths differ
        H, Dh = self.num_heads, self.head_dim
        Q = self.Wq_x(query).view(B, Lq, H, Dh).transpose(1, 2)
        K = self.Wk_x(key).view(B, key.size(1), H, Dh).transpose(1, 2)
        V = self.Wv_x(value).view(B, value.size(1), H, Dh).transpose(1, 2)
        ctx, attn = self._standard_attention(Q, K, V, mask)
        out = self.out_proj_x(ctx.transpose(1, 2).reshape(B, Lq, D))
        return (out, attn) if return_attention else out
