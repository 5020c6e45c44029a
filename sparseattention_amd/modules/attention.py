"""`HierarchicalAttention`: the nn.Module around the two ops.

Parameter names, shapes and method signatures follow the reference's
hierarchical_attention/modules/attention.py:10-270 so that its state dicts load
unchanged; the dense projections are torch's own `nn.Linear`, the tree build and
the span attention are the HIP kernels.
"""
from __future__ import annotations

import ctypes
import math
from typing import List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import _lib
from ..ops.functional import build_parent_nodes, hierarchical_attention, pack_kv_weights
from ..ops.topology import build_tree_topology


def _level_sizes(n_leaves: int) -> List[int]:
    sizes, cur = [], n_leaves
    while cur > 1:
        cur //= 2
        sizes.append(cur)
    return sizes


class _SpanLevels(torch.autograd.Function):
    """The level loop of `HierarchicalAttention.cross_update_Y` (reference
    hierarchical_attention/modules/attention.py:101-157, everything before out_proj_y) as one
    differentiable function on fused projections.  The reference gets the same gradients from
    autograd through 3 + 2L Linear layers and L `BuildParentNodesFunc`s (ops/functional.py:66-111)."""

    @staticmethod
    def forward(ctx, module, drop_p, x, y_in, wq, wk, wv):
        y_new, kept = module._span_levels(x, y_in, keep=True, drop_p=drop_p)
        # everything the backward reads goes through save_for_backward: an in-place write to one
        # of these tensors between forward and backward is then reported by autograd instead of
        # giving wrong gradients, and saved-tensor hooks (checkpointing, offloading) see them
        nl = len(kept["kvs"])
        ctx.save_for_backward(kept["x"], kept["y_in"], kept["qkv"], kept["blocks"], kept["w_qkv"], kept["w_kv"],
                              *kept["kvs"], *kept["masks"])
        ctx.module, ctx.levels, ctx.scales = module, nl, kept["scales"]
        ctx.in_dtypes = (x.dtype, y_in.dtype, wq.dtype)
        return y_new

    @staticmethod
    def backward(ctx, dy):
        saved = ctx.saved_tensors  # raises autograd's own error if they were freed or modified
        nl = ctx.levels
        kept = dict(zip(("x", "y_in", "qkv", "blocks", "w_qkv", "w_kv"), saved[:6]))
        kept["kvs"], kept["masks"], kept["scales"] = list(saved[6:6 + nl]), list(saved[6 + nl:]), ctx.scales
        dx, dy_in, dw = ctx.module._span_levels_backward(dy, kept)
        xd, yd, wd = ctx.in_dtypes
        D = dx.shape[-1]
        dw = dw.to(wd)
        return None, None, dx.to(xd), dy_in.to(yd), dw[:D], dw[D:2 * D], dw[2 * D:]


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
        self._fused = {}  # row-concatenated projection weights of the no-autograd path
        self.fuse_top_levels = True  # no-autograd path: the last levels in one launch where the shape allows
        self.fused_training = True   # autograd path: fused projections and one backward kernel per level

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

    _DIRECT_PROJECTION_MIN_ELEMENTS = 1 << 20

    def _heads(self, t: torch.Tensor) -> torch.Tensor:
        return t.view(t.shape[0], -1, self.num_heads, self.head_dim)

    def reset_fused_weights(self):
        """Drops the cached stacked / packed projection weights of the no-autograd path.  The cache
        notices optimizer steps, `load_state_dict`, `.to()` and `train()` by itself; call this after
        writing to a weight through `.data` (such writes leave no trace on the tensor)."""
        self._fused.clear()

    def _load_from_state_dict(self, *args, **kwargs):
        self._fused.clear()
        return super()._load_from_state_dict(*args, **kwargs)

    def _apply(self, fn, *args, **kwargs):
        self._fused.clear()
        return super()._apply(fn, *args, **kwargs)

    def train(self, mode: bool = True):
        self._fused.clear()
        return super().train(mode)

    def _fused_weight(self, name: str, layers, dtype: torch.dtype, packed: bool = False) -> torch.Tensor:
        """Weights of several bias-free projections, cast to `dtype` and stacked along the output
        dimension, so one GEMM computes them all (packed: key / value weights in the operand order
        of the fused upper levels); rebuilt when any of them has been written to or moved."""
        # (the parameter dictionary is read directly: Module.__getattr__ costs a microsecond per use)
        params = [m._parameters["weight"] for m in layers]
        key = tuple((w.data_ptr(), w._version, w.dtype) for w in params) + (dtype,)
        hit = self._fused.get(name)
        if hit is None or hit[0] != key:
            ws = [w.detach().to(dtype) for w in params]
            hit = (key, pack_kv_weights(ws[0], ws[1], self.num_heads) if packed else torch.cat(ws, dim=0))
            self._fused[name] = hit
        return hit[1]

    @staticmethod
    def _compute_dtype(t: torch.Tensor) -> torch.dtype:
        """Element type the projections produce: the autocast type inside `torch.autocast` (the
        reference's evaluation loop runs under it with fp32 activations and weights), else the
        activations' own type."""
        if t.is_cuda and torch.is_autocast_enabled("cuda"):
            return torch.get_autocast_dtype("cuda")
        return t.dtype

    def _needs_autograd(self, tensors, layers) -> bool:
        if not torch.is_grad_enabled():
            return False
        return any(t.requires_grad for t in tensors) or any(
            p.requires_grad for m in layers for p in m.parameters())

    def _span_levels(self, x: torch.Tensor, y_in: torch.Tensor, keep: bool = False, drop_p: float = 0.0):
        """The level loop of cross_update_Y on fused projections, without autograd: the three
        projections of the span nodes are one GEMM, the key/value projections of each level's
        children another, and each level's kernel reads its operands as column slices of those
        results.  Every level writes twice: a dense [B, P, D] block that feeds the next level's
        GEMM, and its slice of the level-concatenated [B, N-1, D] result (returned, before
        out_proj_y).  Unless `keep`, the last levels (few rows each) run as one launch that does
        their projections on chip.  `keep` returns what a backward pass needs as a dict; `drop_p`
        is the dropout probability applied to the children's values (the reference applies it
        twice to the leaves' values)."""
        B, N, D = x.shape
        H, Dh = self.num_heads, self.head_dim
        _lib.require_gpu(x, y_in)
        cdt = self._compute_dtype(x)
        x, y_in = x.to(cdt).contiguous(), y_in.to(cdt).contiguous()
        w_qkv = self._fused_weight("qkv_y", (self.Wq_y, self.Wk_y, self.Wv_y), cdt)
        qkv = F.linear(y_in, w_qkv)  # [B, N-1, 3D]
        w_kv = self._fused_weight("kv_y", (self.Wk_y, self.Wv_y), cdt)
        # every buffer the kernels address by raw pointer has the one element type
        assert qkv.dtype == cdt and qkv.is_contiguous(), "projection result has an unexpected layout"
        y_new = torch.empty((B, N - 1, D), dtype=cdt, device=x.device)
        blocks = torch.empty(B * (N - 1) * D, dtype=cdt, device=x.device)  # level-major
        # the level loop works on raw addresses: the operands are fixed column slices of qkv and
        # of each level's k/v projection, so no tensor views are made per level
        es = x.element_size()
        A = ctypes.c_int64 * 7
        row_strides = A(3 * D, 3 * D, 3 * D, 2 * D, 2 * D, D, D)
        fwd, code, stream = _lib.lib().hsa_build_parents_strided_fwd, _lib.dtype_code(x), _lib.stream_of(x)
        qkv_p, blk_p, out_p = qkv.data_ptr(), blocks.data_ptr(), y_new.data_ptr()
        # child rows the fused upper levels take (0: shape not handled)
        # (y_new's rows are 16-byte aligned: the fused upper levels may run as a launch per level)
        top_rows = 0 if keep or not self.fuse_top_levels else _lib.lib().hsa_cross_update_level_rows(B, H, Dh, code)
        kvs, masks, scales = [], [], []
        src, off = x, 0
        with _lib.on_device(x):
            for lvl, P in enumerate(self.sizes):
                if 2 * P <= top_rows:
                    # the remaining levels: fused projection + parent build, no GEMM launches
                    w_top = self._fused_weight("kv_y_packed", (self.Wk_y, self.Wv_y), cdt, packed=True)
                    assert src.dtype == cdt and src.is_contiguous() and w_top.dtype == cdt
                    rc = _lib.lib().hsa_cross_update_top_fwd(
                        src.data_ptr(), qkv_p + off * 3 * D * es, w_top.data_ptr(), out_p + off * D * es,
                        B, 2 * P, H, Dh, 0, (N - 1) * 3 * D, 3 * D, (N - 1) * D, D, code, stream)
                    _lib.check(rc, "hsa_cross_update_top_fwd")
                    break
                kv = F.linear(src, w_kv)  # [B, 2P, 2D]
                assert kv.dtype == cdt and kv.is_contiguous(), "projection result has an unexpected layout"
                if drop_p > 0:
                    # dropout on the value half: a saved boolean keep-mask (drawn in fp32) and one
                    # scale applied as a scalar, i.e. in fp32 with a single rounding of the product
                    # (a mask holding 1/keep_p in bf16 would scale by 1.109 instead of 1.111)
                    keep_p = 1.0 - drop_p
                    m = torch.rand((B, 2 * P, D), dtype=torch.float32, device=x.device) < keep_p
                    scale = 1.0 / keep_p
                    if lvl == 0:  # the leaves' values pass through dropout twice
                        m &= torch.rand((B, 2 * P, D), dtype=torch.float32, device=x.device) < keep_p
                        scale = scale * scale
                    kv[:, :, D:].mul_(m).mul_(scale)
                    masks.append(m)
                    scales.append(scale)
                par, kv_p, lvl_p = qkv_p + off * 3 * D * es, kv.data_ptr(), blk_p + B * off * D * es
                rc = fwd(par, par + D * es, par + 2 * D * es, kv_p, kv_p + D * es, lvl_p,
                         out_p + off * D * es, B, P, H, Dh,
                         A((N - 1) * 3 * D, (N - 1) * 3 * D, (N - 1) * 3 * D, 4 * P * D, 4 * P * D, P * D,
                           (N - 1) * D), row_strides, code, stream)
                _lib.check(rc, "hsa_build_parents_strided_fwd")
                if keep:
                    kvs.append(kv)
                src = blocks[B * off * D:B * (off + P) * D].view(B, P, D)
                off += P
        if not keep:
            return y_new
        return y_new, {"x": x, "y_in": y_in, "qkv": qkv, "blocks": blocks, "kvs": kvs, "masks": masks,
                       "scales": scales, "w_qkv": w_qkv, "w_kv": w_kv}

    def _span_levels_backward(self, dy: torch.Tensor, kept: dict):
        """Gradients of `_span_levels` with respect to x, y_in and the stacked q|k|v weights:
        per level one kernel (the three weights are recomputed, every gradient row written once
        into the fused layouts) and two GEMMs (input gradient and weight gradient of the fused
        key/value projection).  Returns (dx, dy_in, dW_qkv [3D, D] fp32)."""
        x, y_in, qkv, blocks = kept["x"], kept["y_in"], kept["qkv"], kept["blocks"]
        kvs, masks, w_qkv, w_kv = kept["kvs"], kept["masks"], kept["w_qkv"], kept["w_kv"]
        B, N, D = x.shape
        H, Dh = self.num_heads, self.head_dim
        cdt, es = x.dtype, x.element_size()
        dy = dy.to(cdt).contiguous()
        dqkv = torch.empty_like(qkv)
        dw_kv = torch.zeros((2 * D, D), dtype=torch.float32, device=x.device)
        A = ctypes.c_int64 * 11
        bwd, code, stream = _lib.lib().hsa_build_parents_strided_bwd, _lib.dtype_code(x), _lib.stream_of(x)
        rs = A(D, 3 * D, 3 * D, 3 * D, 2 * D, 2 * D, 3 * D, 3 * D, 3 * D, 2 * D, 2 * D)
        T3 = (N - 1) * 3 * D
        d_above, dx = None, None
        with _lib.on_device(x):
            for lvl in range(len(self.sizes) - 1, -1, -1):
                P, off = self.sizes[lvl], self.offsets[lvl]
                g = dy[:, off:off + P]
                g = (g + d_above) if d_above is not None else g.contiguous()
                kv = kvs[lvl]
                dkv = torch.empty_like(kv)
                par, dpar = qkv.data_ptr() + off * 3 * D * es, dqkv.data_ptr() + off * 3 * D * es
                kv_p, dkv_p = kv.data_ptr(), dkv.data_ptr()
                rc = bwd(g.data_ptr(), par, par + D * es, par + 2 * D * es, kv_p, kv_p + D * es,
                         dpar, dpar + D * es, dpar + 2 * D * es, dkv_p, dkv_p + D * es, B, P, H, Dh,
                         A(P * D, T3, T3, T3, 4 * P * D, 4 * P * D, T3, T3, T3, 4 * P * D, 4 * P * D), rs, code, stream)
                _lib.check(rc, "hsa_build_parents_strided_bwd")
                if masks:
                    dkv[:, :, D:].mul_(masks[lvl]).mul_(kept["scales"][lvl])
                src = x if lvl == 0 else blocks[B * self.offsets[lvl - 1] * D:B * off * D].view(B, 2 * P, D)
                dw_kv += torch.matmul(dkv.reshape(-1, 2 * D).t(), src.reshape(-1, D)).float()
                d_src = torch.matmul(dkv, w_kv)  # [B, 2P, D]
                if lvl == 0:
                    dx = d_src
                else:
                    d_above = d_src
        dy_in = torch.matmul(dqkv, w_qkv)
        dw_qkv = torch.matmul(dqkv.reshape(-1, 3 * D).t(), y_in.reshape(-1, D)).float()
        dw_qkv[D:] += dw_kv
        return dx, dy_in, dw_qkv

    # -- bottom-up: leaves -> span nodes ----------------------------------------
    def cross_update_Y(self, x: torch.Tensor, y_in: torch.Tensor) -> torch.Tensor:
        B, N, D = x.shape
        assert y_in is not None, "y_in cannot be None"
        assert y_in.size(1) == N - 1, \
            f"y_in size {y_in.size(1)} mismatch! Expected N-1 ({N-1}) for N={N} leaves."
        if self.sizes is None or self.sizes[0] != N // 2:
            self.sizes, self.offsets = self._build_level_info(N)

        grad = self._needs_autograd((x, y_in), (self.Wq_y, self.Wk_y, self.Wv_y))
        drop_p = self.dropout.p if self.training else 0.0
        if not grad and drop_p == 0:
            return self.out_proj_y(self._span_levels(x, y_in))
        if self.fused_training and x.is_cuda and N >= 2:
            # the same fused level loop as one differentiable function
            y_new = _SpanLevels.apply(self, drop_p, x, y_in, self.Wq_y.weight, self.Wk_y.weight, self.Wv_y.weight)
            return self.out_proj_y(y_new)

        q_lv = torch.split(self._heads(self.Wq_y(y_in)), self.sizes, dim=1)
        k_lv = torch.split(self._heads(self.Wk_y(y_in)), self.sizes, dim=1)
        v_lv = torch.split(self._heads(self.Wv_y(y_in)), self.sizes, dim=1)
        levels, src = [], x
        for lvl, P in enumerate(self.sizes):
            k_c = self._heads(self.Wk_y(src))
            v_c = self.dropout(self._heads(self.Wv_y(src)))
            if lvl == 0:
                v_c = self.dropout(v_c)  # the leaf values pass through dropout twice
            src = build_parent_nodes(q_lv[lvl], k_lv[lvl], v_lv[lvl], k_c, v_c).reshape(B, P, D)
            levels.append(src)
        return self.out_proj_y(torch.cat(levels, dim=1))

    # -- top-down: span nodes -> leaves -------------------------------------------
    def update_X_from_Y(self, x: torch.Tensor, y: torch.Tensor,
                        mask: Optional[torch.Tensor] = None) -> torch.Tensor:
        B, N, D = x.shape
        assert y is not None, "y (parents) cannot be None during top-down update"
        q = self._heads(self.Wq_x(x))
        grad = self._needs_autograd((x, y), (self.Wq_x, self.Wk_x, self.Wv_x))
        if (not grad and not (self.training and self.dropout.p > 0) and y.size(1) == N - 1
                and B * N * D >= self._DIRECT_PROJECTION_MIN_ELEMENTS):
            # leaves and span nodes are projected straight into their rows of the [B, 2N-1, D]
            # key / value buffers (batched GEMMs with a strided output): no concatenated input.
            # (Four GEMM launches instead of a copy and two: small inputs, where the launches cost
            # more host time than the copy costs the GPU, take the other branch.)
            # Everything is brought to the type of q first (under autocast the activations and
            # weights are fp32 while the projections come out in the autocast type; GEMMs with an
            # `out=` are not autocast)
            cdt = q.dtype
            xc, yc = x.to(cdt), y.to(cdt)
            k = torch.empty((B, 2 * N - 1, D), dtype=cdt, device=x.device)
            v = torch.empty_like(k)
            for lin, dst in ((self.Wk_x, k), (self.Wv_x, v)):
                wt = lin.weight.detach().to(cdt).t().unsqueeze(0).expand(B, D, D)
                torch.bmm(xc, wt, out=dst[:, :N])
                torch.bmm(yc, wt, out=dst[:, N:])
            k, v = self._heads(k), self._heads(v)
        else:
            xy = torch.cat([x, y], dim=1)
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
