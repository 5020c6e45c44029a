"""Functional ops: `build_parent_nodes`, `hierarchical_attention` (+ the fused tree build).

Call surface of the reference's hierarchical_attention/ops/functional.py:271-275.
Each op is a torch.autograd.Function whose forward allocates the output with
torch and enqueues a kernel of libhsa_gfx950.so on the current stream.
"""
from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import torch

from .. import _lib
from . import topology as _topo


def _is_canonical(idx_table: torch.Tensor, mask_table: Optional[torch.Tensor], N: int) -> Optional[bool]:
    """True/False = the tables are the canonical ones for N with that causal flag
    (known without touching the device); None = unknown table contents."""
    info = _topo.known_table(idx_table, "idx")
    if info is None or info[0] != N or idx_table.dtype != torch.int32:
        return None
    if mask_table is None:
        return False
    minfo = _topo.known_table(mask_table, "mask")
    if minfo is None or minfo[0] != N or not minfo[1]:
        return None
    return True


def verify_tables(idx_table: torch.Tensor, mask_table: Optional[torch.Tensor]) -> bool:
    """Compares tables of unknown origin with the canonical ones on the device (one
    host sync) and remembers the verdict, so that later calls take the fast path."""
    N, L = idx_table.shape
    if N < 1 or (N & (N - 1)) != 0 or L != N.bit_length() - 1:
        return False
    if _topo.known_other(idx_table) or _topo.known_other(mask_table):
        return False
    if torch.cuda.is_current_stream_capturing():
        return False  # the comparison synchronises: under graph capture unknown tables stay unknown
    canon = _topo.build_tree_topology(N, mask_table is not None, idx_table.device)
    ok = bool(torch.equal(idx_table.to(torch.int32), canon["forward_idx"]))
    if not ok:
        _topo.remember_other(idx_table)
    elif mask_table is not None:
        ok = bool(torch.equal(mask_table.to(torch.bool), canon["forward_mask"]))
        if not ok:
            _topo.remember_other(mask_table)
    if ok and idx_table.dtype == torch.int32:
        _topo._remember(idx_table, "idx", N, mask_table is not None)
        if mask_table is not None and mask_table.dtype == torch.bool:
            _topo._remember(mask_table, "mask", N, True)
    return ok


def attention_forward(Q, K, V, idx_table, mask_table=None, window_size: int = 16,
                      return_weights: bool = False, algo: str = "auto", out: Optional[torch.Tensor] = None):
    """Span attention forward on [B,N,H,D] / [B,M,H,D] tensors.

    Returns Out, or (Out, Weights [B,N,H,2R+1+L] fp32) with `return_weights`.
    `algo`: "auto" | "gather" | "tile".
    """
    _lib.require_gpu(Q, K, V, idx_table, mask_table)
    assert Q.dim() == 4 and K.dim() == 4 and V.dim() == 4, "Q, K, V must be [B, rows, H, D]"
    assert K.shape == V.shape, "K and V shapes differ"
    assert Q.dtype == K.dtype == V.dtype, "Q, K, V dtypes differ"
    B, N, H, D = Q.shape
    M = K.shape[1]
    assert K.shape[0] == B and K.shape[2] == H and K.shape[3] == D, "K shape does not match Q"
    assert idx_table.dim() == 2 and idx_table.shape[0] == N, "idx_table must be [N, levels]"
    L = idx_table.shape[1]
    R = int(window_size)
    assert R >= 0
    Q, K, V = Q.contiguous(), K.contiguous(), V.contiguous()
    if mask_table is not None:
        assert mask_table.shape == idx_table.shape, "mask_table shape mismatch"

    canon = _is_canonical(idx_table, mask_table, N)
    if canon is None and algo != "gather" and M >= 2 * N - 1:
        if verify_tables(idx_table, mask_table):
            canon = mask_table is not None
    if out is None:
        out = torch.empty_like(Q)
    else:
        assert out.shape == Q.shape and out.dtype == Q.dtype and out.is_contiguous() and out.is_cuda
    weights = (torch.empty((B, N, H, 2 * R + 1 + L), device=Q.device, dtype=torch.float32)
               if return_weights else None)
    if Q.numel() == 0:  # empty batch: nothing to launch
        return (out, weights) if return_weights else out
    lib = _lib.lib()
    with _lib.on_device(Q):
        if canon is not None and M >= 2 * N - 1:
            rc = lib.hsa_attn_fwd(_lib.ptr(Q), _lib.ptr(K), _lib.ptr(V), None, None, _lib.ptr(out),
                                  _lib.ptr(weights), B, N, M, H, D, L, R, int(canon),
                                  _lib.dtype_code(Q), _lib.algo_code(algo), _lib.stream_of(Q))
        else:
            idx32 = idx_table.to(torch.int32).contiguous()
            m8 = None
            if mask_table is not None:
                m8 = mask_table.contiguous()
                m8 = m8.view(torch.uint8) if m8.dtype == torch.bool else (m8 != 0).view(torch.uint8)
            rc = lib.hsa_attn_fwd(_lib.ptr(Q), _lib.ptr(K), _lib.ptr(V), _lib.ptr(idx32), _lib.ptr(m8),
                                  _lib.ptr(out), _lib.ptr(weights), B, N, M, H, D, L, R, 0,
                                  _lib.dtype_code(Q), _lib.algo_code(algo), _lib.stream_of(Q))
    _lib.check(rc, "hsa_attn_fwd")
    return (out, weights) if return_weights else out


def saved_state_backward_available(Q, K, window_size: int, causal: bool = True) -> bool:
    """Whether the one-pass backward (hsa_attn_bwd_saved) takes this problem on the canonical
    tables: then the forward should also keep its log-sum-exp (`attention_forward_lse`)."""
    if not Q.is_cuda or Q.dim() != 4:
        return False
    B, N, H, D = Q.shape
    if N < 1 or (N & (N - 1)) or Q.dtype not in (torch.float16, torch.bfloat16):
        return False
    return int(_lib.lib().hsa_attn_bwd_saved_workspace_bytes(B, N, K.shape[1], H, D, N.bit_length() - 1,
                                                            int(window_size), int(bool(causal)),
                                                            _lib.dtype_code(Q))) > 0


def attention_forward_lse(Q, K, V, window_size: int, causal: bool):
    """Span attention forward on the canonical tables that also returns the log-sum-exp of every
    (query, head)'s biased logits (log2 domain, [B, N, H] fp32), the state the one-pass backward
    works from.  Returns (Out, lse), or None where the kernel that writes it does not take the
    problem (the caller then uses `attention_forward`)."""
    _lib.require_gpu(Q, K, V)
    Q, K, V = Q.contiguous(), K.contiguous(), V.contiguous()
    B, N, H, D = Q.shape
    M, L = K.shape[1], N.bit_length() - 1
    if any(t.data_ptr() % 16 for t in (Q, K, V)):
        return None
    out = torch.empty_like(Q)
    lse = torch.empty((B, N, H), device=Q.device, dtype=torch.float32)
    with _lib.on_device(Q):
        rc = _lib.lib().hsa_attn_fwd_lse(_lib.ptr(Q), _lib.ptr(K), _lib.ptr(V), _lib.ptr(out), _lib.ptr(lse), B, N, M,
                                         H, D, L, int(window_size), int(bool(causal)), _lib.dtype_code(Q),
                                         _lib.stream_of(Q))
    if rc == -95:  # HSA_ERR_UNSUPPORTED: nothing was launched
        return None
    _lib.check(rc, "hsa_attn_fwd_lse")
    return out, lse


def attention_backward_saved(grad_out, Q, K, V, out, lse, window_size: int, causal: bool):
    """Gradients (dQ, dK, dV) in one pass from the forward's output and log-sum-exp."""
    _lib.require_gpu(grad_out, Q, K, V, out, lse)
    grad_out, Q, K, V, out, lse = (t.contiguous() for t in (grad_out, Q, K, V, out, lse))
    B, N, H, D = Q.shape
    M, L, R = K.shape[1], N.bit_length() - 1, int(window_size)
    assert lse.shape == (B, N, H) and lse.dtype == torch.float32 and out.shape == Q.shape
    dq, dk, dv = torch.empty_like(Q), torch.empty_like(K), torch.empty_like(V)
    lib = _lib.lib()
    nbytes = int(lib.hsa_attn_bwd_saved_workspace_bytes(B, N, M, H, D, L, R, int(bool(causal)), _lib.dtype_code(Q)))
    ws = torch.empty((max(nbytes, 4) + 3) // 4, device=Q.device, dtype=torch.float32)
    with _lib.on_device(Q):
        rc = lib.hsa_attn_bwd_saved(_lib.ptr(Q), _lib.ptr(K), _lib.ptr(V), _lib.ptr(out), _lib.ptr(lse),
                                    _lib.ptr(grad_out), _lib.ptr(dq), _lib.ptr(dk), _lib.ptr(dv), _lib.ptr(ws),
                                    ws.numel() * 4, B, N, M, H, D, L, R, int(bool(causal)), _lib.dtype_code(Q),
                                    _lib.stream_of(Q))
    _lib.check(rc, "hsa_attn_bwd_saved")
    return dq, dk, dv


def _rows_dense(t: torch.Tensor) -> bool:
    if t.is_contiguous():
        return True
    B, rows, H, D = t.shape
    return t.stride(3) == 1 and t.stride(2) == D and (rows == 1 or t.stride(1) == H * D)


def _batch_stride(t: torch.Tensor) -> int:
    """Element stride between batches of a [B, rows, H, D] tensor whose rows are dense."""
    B, rows, H, D = t.shape
    assert _rows_dense(t), "rows of the tensor must be dense [rows, H, D]"
    return t.stride(0) if B > 1 else rows * H * D


def _dense_rows(t: torch.Tensor) -> torch.Tensor:
    """The tensor itself when each batch's rows are dense (a level slice of a larger buffer
    qualifies: only the batch stride differs), else a contiguous copy."""
    return t if _rows_dense(t) else t.contiguous()


def build_parents_forward(Q_p, K_p, V_p, K_c, V_c, return_weights: bool = False,
                          out: Optional[torch.Tensor] = None):
    """One level of the parent build on [B,P,H,D] / [B,2P,H,D] tensors.  Inputs may be level
    slices of larger buffers (dense rows, any batch stride); `out` may be such a slice too."""
    _lib.require_gpu(Q_p, K_p, V_p, K_c, V_c, out)
    Q_p, K_p, V_p, K_c, V_c = (_dense_rows(t) for t in (Q_p, K_p, V_p, K_c, V_c))
    B, P, H, D = Q_p.shape
    assert K_c.shape[1] == 2 * P, "Child count mismatch"
    assert K_p.shape == Q_p.shape and V_p.shape == Q_p.shape, "parent K/V shape mismatch"
    assert V_c.shape == K_c.shape and K_c.shape[0] == B and K_c.shape[2:] == Q_p.shape[2:], \
        "child K/V shape mismatch"
    assert Q_p.dtype == K_p.dtype == V_p.dtype == K_c.dtype == V_c.dtype, "dtype mismatch"
    if out is None:
        out = torch.empty((B, P, H, D), dtype=Q_p.dtype, device=Q_p.device)
    else:
        assert out.shape == (B, P, H, D) and out.dtype == Q_p.dtype and _rows_dense(out)
    weights = torch.empty((B, P, H, 3), device=Q_p.device, dtype=Q_p.dtype) if return_weights else None
    if Q_p.numel() == 0:
        return (out, weights) if return_weights else out
    with _lib.on_device(Q_p):
        rc = _lib.lib().hsa_build_parents_fwd(
            _lib.ptr(Q_p), _lib.ptr(K_p), _lib.ptr(V_p), _lib.ptr(K_c), _lib.ptr(V_c), _lib.ptr(out),
            _lib.ptr(weights), B, P, H, D, _batch_stride(Q_p), _batch_stride(K_p), _batch_stride(V_p),
            _batch_stride(K_c), _batch_stride(V_c), _batch_stride(out), _lib.dtype_code(Q_p),
            _lib.stream_of(Q_p))
    _lib.check(rc, "hsa_build_parents_fwd")
    return (out, weights) if return_weights else out


def build_parents_strided(Q_p, K_p, V_p, K_c, V_c, out: torch.Tensor,
                          out2: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One level of the parent build on operands that are column slices of wider matrices
    (thirds of a fused q/k/v projection, halves of a fused k/v projection): each [B, rows, H, D]
    view needs dense heads (strides D, 1) only; row and batch strides are free.  The result goes
    to `out` and, if given, to `out2` as well.  No autograd."""
    ts = (Q_p, K_p, V_p, K_c, V_c, out) + ((out2,) if out2 is not None else ())
    _lib.require_gpu(*ts)
    B, P, H, D = Q_p.shape
    assert K_c.shape == (B, 2 * P, H, D) and V_c.shape == K_c.shape, "Child count mismatch"
    assert K_p.shape == Q_p.shape and V_p.shape == Q_p.shape and out.shape == Q_p.shape
    assert out2 is None or out2.shape == Q_p.shape
    bs, rs = [0] * 7, [0] * 7
    for i, t in enumerate(ts):
        assert t.dtype == Q_p.dtype, "dtype mismatch"
        assert t.stride(3) == 1 and t.stride(2) == D and t.stride(1) >= H * D, \
            "heads of every operand must be dense"
        rs[i] = t.stride(1)
        bs[i] = t.stride(0) if B > 1 else t.shape[1] * t.stride(1)
    A = ctypes.c_int64 * 7
    with _lib.on_device(Q_p):
        rc = _lib.lib().hsa_build_parents_strided_fwd(
            _lib.ptr(Q_p), _lib.ptr(K_p), _lib.ptr(V_p), _lib.ptr(K_c), _lib.ptr(V_c), _lib.ptr(out),
            _lib.ptr(out2), B, P, H, D, A(*bs), A(*rs), _lib.dtype_code(Q_p), _lib.stream_of(Q_p))
    _lib.check(rc, "hsa_build_parents_strided_fwd")
    return out


def fused_top_rows(num_heads: int, head_dim: int, dtype: torch.dtype) -> int:
    """Largest number of child rows `cross_update_top` takes for this head layout (0: the
    layout is not handled and every level has to go through `build_parents_strided`)."""
    if dtype not in (torch.float16, torch.bfloat16):
        return 0
    code = 1 if dtype == torch.float16 else 2
    return int(_lib.lib().hsa_cross_update_top_rows(num_heads, head_dim, code))


def pack_kv_weights(w_k: torch.Tensor, w_v: torch.Tensor, num_heads: int) -> torch.Tensor:
    """Key and value projection weights ([dim, dim] each, row = output feature) in the operand
    order `cross_update_top` streams them in.  Repack whenever the weights change."""
    _lib.require_gpu(w_k, w_v)
    dim = w_k.shape[0]
    assert w_k.shape == (dim, dim) and w_v.shape == (dim, dim) and w_k.dtype == w_v.dtype
    w_k, w_v = w_k.contiguous(), w_v.contiguous()
    packed = torch.empty(2 * dim * dim, dtype=w_k.dtype, device=w_k.device)
    with _lib.on_device(w_k):
        rc = _lib.lib().hsa_cross_update_pack_weights(
            _lib.ptr(w_k), _lib.ptr(w_v), _lib.ptr(packed), num_heads, dim // num_heads,
            _lib.dtype_code(w_k), _lib.stream_of(w_k))
    _lib.check(rc, "hsa_cross_update_pack_weights")
    return packed


def cross_update_top(src: torch.Tensor, qkv: torch.Tensor, w_packed: torch.Tensor, out: torch.Tensor,
                     num_heads: int) -> torch.Tensor:
    """Every level from `src` up to the root in one launch: per level the children are projected
    with the key / value weights (`w_packed` from `pack_kv_weights`), the parents are built, and
    the parents are the next level's children.

    src [B, C, dim] dense; qkv [B, C-1, 3*dim] the parents' q | k | v, level after level, root
    last; out [B, C-1, dim] numbered alike.  qkv and out may be row slices of larger tensors."""
    _lib.require_gpu(src, qkv, w_packed, out)
    B, C, dim = src.shape
    H, Dh = num_heads, dim // num_heads
    assert src.is_contiguous() and w_packed.is_contiguous() and w_packed.numel() == 2 * dim * dim
    assert qkv.shape == (B, C - 1, 3 * dim) and out.shape == (B, C - 1, dim)
    assert qkv.stride(2) == 1 and out.stride(2) == 1
    assert src.dtype == qkv.dtype == w_packed.dtype == out.dtype, "dtype mismatch"
    with _lib.on_device(src):
        rc = _lib.lib().hsa_cross_update_top_fwd(
            _lib.ptr(src), _lib.ptr(qkv), _lib.ptr(w_packed), _lib.ptr(out), B, C, H, Dh, 0,
            qkv.stride(0) if B > 1 else 0, qkv.stride(1) if C > 2 else 0,
            out.stride(0) if B > 1 else 0, out.stride(1) if C > 2 else 0,
            _lib.dtype_code(src), _lib.stream_of(src))
    _lib.check(rc, "hsa_cross_update_top_fwd")
    return out


def build_tree(Q_p, K_p, V_p, K_leaf, V_leaf, out: Optional[torch.Tensor] = None,
               out2: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Every tree level in one call: level 1 from the leaves, level l+1 from level l's
    outputs used as both child keys and child values.

    Q_p, K_p, V_p [B, N-1, H, D] are level-concatenated (level 1 first, root last) and so
    is the result.  Tensors may be batch-strided slices of larger buffers (for instance
    `out = K_full[:, N:]`) as long as each batch's rows are dense.  `out2`, if given,
    receives a second copy of the result (for instance `V_full[:, N:]`).
    """
    _lib.require_gpu(Q_p, K_p, V_p, K_leaf, V_leaf, out, out2)
    B, N, H, D = K_leaf.shape
    assert N >= 2 and (N & (N - 1)) == 0, "leaf count must be a power of 2"
    assert Q_p.shape == (B, N - 1, H, D) and K_p.shape == Q_p.shape and V_p.shape == Q_p.shape
    assert V_leaf.shape == K_leaf.shape
    if out is None:
        out = torch.empty((B, N - 1, H, D), dtype=Q_p.dtype, device=Q_p.device)
    assert out.shape == Q_p.shape and out.dtype == Q_p.dtype
    if out2 is not None:
        assert out2.shape == Q_p.shape and out2.dtype == Q_p.dtype
    if K_leaf.numel() == 0:
        return out
    ts = [Q_p, K_p, V_p, K_leaf, V_leaf]
    for i, t in enumerate(ts):
        if not (t.stride(3) == 1 and t.stride(2) == D and t.stride(1) == H * D):
            ts[i] = t.contiguous()
    Q_p, K_p, V_p, K_leaf, V_leaf = ts
    with _lib.on_device(Q_p):
        rc = _lib.lib().hsa_build_tree_fwd(
            _lib.ptr(Q_p), _lib.ptr(K_p), _lib.ptr(V_p), _lib.ptr(K_leaf), _lib.ptr(V_leaf), _lib.ptr(out),
            _lib.ptr(out2), B, N, H, D, _batch_stride(Q_p), _batch_stride(K_p), _batch_stride(V_p),
            _batch_stride(K_leaf), _batch_stride(V_leaf), _batch_stride(out),
            _batch_stride(out2) if out2 is not None else 0, _lib.dtype_code(Q_p), _lib.stream_of(Q_p))
    _lib.check(rc, "hsa_build_tree_fwd")
    return out


def build_parents_backward(grad_out, Q_p, K_p, V_p, K_c, V_c):
    """Gradients (dQ_p, dK_p, dV_p, dK_c, dV_c) of one parent-build level."""
    _lib.require_gpu(grad_out, Q_p, K_p, V_p, K_c, V_c)
    grad_out, Q_p, K_p, V_p, K_c, V_c = (t.contiguous() for t in (grad_out, Q_p, K_p, V_p, K_c, V_c))
    B, P, H, D = Q_p.shape
    dq, dkp, dvp = torch.empty_like(Q_p), torch.empty_like(K_p), torch.empty_like(V_p)
    dkc, dvc = torch.empty_like(K_c), torch.empty_like(V_c)
    if Q_p.numel() == 0:
        return dq, dkp, dvp, dkc, dvc
    with _lib.on_device(Q_p):
        rc = _lib.lib().hsa_build_parents_bwd(
            _lib.ptr(grad_out), _lib.ptr(Q_p), _lib.ptr(K_p), _lib.ptr(V_p), _lib.ptr(K_c), _lib.ptr(V_c),
            _lib.ptr(dq), _lib.ptr(dkp), _lib.ptr(dvp), _lib.ptr(dkc), _lib.ptr(dvc), B, P, H, D,
            _lib.dtype_code(Q_p), _lib.stream_of(Q_p))
    _lib.check(rc, "hsa_build_parents_bwd")
    return dq, dkp, dvp, dkc, dvc


def attention_backward(grad_out, Q, K, V, window_size: int, causal: bool, algo: str = "auto"):
    """Gradients (dQ, dK, dV) of the span attention for the canonical tables of N = Q.shape[1]."""
    _lib.require_gpu(grad_out, Q, K, V)
    grad_out, Q, K, V = (t.contiguous() for t in (grad_out, Q, K, V))
    B, N, H, D = Q.shape
    M = K.shape[1]
    L = N.bit_length() - 1
    R = int(window_size)
    dq, dk, dv = torch.empty_like(Q), torch.empty_like(K), torch.empty_like(V)
    if Q.numel() == 0:
        return dq, dk, dv
    lib = _lib.lib()
    if algo == "auto" and any(t.data_ptr() % 16 for t in (grad_out, Q, K, V)):
        algo = "gather"  # the tile kernels move 16-byte pieces
    nbytes = int(lib.hsa_attn_bwd_workspace_bytes(B, N, M, H, D, L, R, _lib.dtype_code(Q), _lib.algo_code(algo)))
    ws = torch.empty((max(nbytes, 4) + 3) // 4, device=Q.device, dtype=torch.float32)
    with _lib.on_device(Q):
        rc = lib.hsa_attn_bwd(_lib.ptr(Q), _lib.ptr(K), _lib.ptr(V), _lib.ptr(grad_out), _lib.ptr(dq),
                              _lib.ptr(dk), _lib.ptr(dv), _lib.ptr(ws), ws.numel() * 4, B, N, M, H, D,
                              L, R, int(bool(causal)), _lib.dtype_code(Q), _lib.algo_code(algo), _lib.stream_of(Q))
    _lib.check(rc, "hsa_attn_bwd")
    return dq, dk, dv


def attention_backward_tables(grad_out, Q, K, V, idx_table, mask_table, gather_table, window_size: int):
    """Gradients (dQ, dK, dV) of the span attention from the caller's own tables, as the
    reference's backward computes them (hierarchical_attention/ops/functional.py:171-264): key
    rows and dead slots from `idx_table` / `mask_table`, each node row's first attending query
    from column 0 of `gather_table`; the window is causal when a mask table is given."""
    _lib.require_gpu(grad_out, Q, K, V, idx_table, gather_table)
    grad_out, Q, K, V = (t.contiguous() for t in (grad_out, Q, K, V))
    B, N, H, D = Q.shape
    M = K.shape[1]
    assert idx_table.dim() == 2 and idx_table.shape[0] == N, "idx_table must be [N, L]"
    L = idx_table.shape[1]
    assert gather_table.dim() == 2 and gather_table.shape[1] >= 3 and gather_table.shape[0] >= min(M, 2 * N - 1), \
        "gather_table must hold a row of three entries per key row"
    idx = idx_table.to(torch.int32).contiguous()
    gat = gather_table.to(torch.int32)[:, :3].contiguous()
    m8 = None
    if mask_table is not None:
        assert mask_table.shape == idx_table.shape, "mask_table must have idx_table's shape"
        m8 = mask_table.to(torch.bool).contiguous().view(torch.uint8)
    R = int(window_size)
    dq, dk, dv = torch.empty_like(Q), torch.empty_like(K), torch.empty_like(V)
    if Q.numel() == 0:
        return dq, dk, dv
    ws = torch.empty(2 * B * N * H * (2 * R + 1 + L) + 4, device=Q.device, dtype=torch.float32)
    lib = _lib.lib()
    with _lib.on_device(Q):
        rc = lib.hsa_attn_bwd_tables(_lib.ptr(Q), _lib.ptr(K), _lib.ptr(V), _lib.ptr(grad_out), _lib.ptr(idx),
                                     _lib.ptr(m8), _lib.ptr(gat), _lib.ptr(dq), _lib.ptr(dk), _lib.ptr(dv),
                                     _lib.ptr(ws), ws.numel() * 4, B, N, M, H, D, L, R,
                                     int(mask_table is not None), _lib.dtype_code(Q), _lib.stream_of(Q))
    _lib.check(rc, "hsa_attn_bwd_tables")
    return dq, dk, dv


class BuildParentNodesFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, Q_p, K_p, V_p, K_c, V_c):
        # the backward recomputes the three weights, so only the inputs are kept
        ctx.save_for_backward(Q_p, K_p, V_p, K_c, V_c)
        return build_parents_forward(Q_p, K_p, V_p, K_c, V_c)

    @staticmethod
    def backward(ctx, grad_output):
        return build_parents_backward(grad_output, *ctx.saved_tensors)


# Which backward `hierarchical_attention` uses.  Two formulations exist: two passes over Q, dO and
# the leaf K / V (any shape the tile kernels take), and one pass that works from the forward's
# output and one log-sum-exp per (query, head), which the forward then keeps (16-bit types; 32 / 64
# channels per head with window radius up to 16, or up to 32 with the causal mask; 128 channels
# with the causal mask).  The one pass moves less (0.76 of the two passes' HBM
# traffic at B8 H8 N2048 D64) and measured faster on every shape tried (50.8 against 56.4 us there,
# 29.6 against 34.7 us at B16 H8 N512, 64.0 against 68.9 us at B2 H16 N8192 D32, 53.8 against 58.7 us
# at B8 H8 N2048 without the causal mask).
#   None (default): the one pass wherever it is built
#   True / False:   the same / never
# Process-wide; read when the forward runs.
one_pass_backward = None


def _use_one_pass(Q, K, window_size, causal) -> bool:
    if one_pass_backward is False or not saved_state_backward_available(Q, K, window_size, causal):
        return False
    return True


class HierarchicalAttentionFunc(torch.autograd.Function):
    """Forward + backward of the span attention (reference: HierarchicalAttentionFunc,
    hierarchical_attention/ops/functional.py:116-264, which keeps Q, K, V, the tables and its
    Weights tensor for the backward).  Kept here: Q, K, V and, where the one-pass backward is
    used (`one_pass_backward`), the output and one log-sum-exp per (query, head)."""

    @staticmethod
    def forward(ctx, Q, K, V, idx_table, gather_table, mask_table=None, window_size=16):
        if not any(ctx.needs_input_grad[:3]):
            return attention_forward(Q, K, V, idx_table, mask_table, window_size)
        N = Q.shape[1]
        canon = _is_canonical(idx_table, mask_table, N)
        if canon is None and K.shape[1] >= 2 * N - 1 and verify_tables(idx_table, mask_table):
            canon = mask_table is not None
        ctx.canonical = canon
        ctx.window_size = int(window_size)
        ctx.saved_state = False
        if (canon is not None and K.shape[1] >= 2 * N - 1 and Q.dtype == K.dtype == V.dtype
                and K.shape == V.shape and _use_one_pass(Q, K, window_size, canon)):
            res = attention_forward_lse(Q, K, V, window_size, canon)
            if res is not None:
                out, lse = res
                ctx.saved_state = True
                ctx.save_for_backward(Q, K, V, out, lse)
                return out
        out = attention_forward(Q, K, V, idx_table, mask_table, window_size)
        if canon is None and gather_table is not None:
            # tables of the caller's own: the backward reads them like the reference's does
            ctx.has_mask = mask_table is not None
            ctx.save_for_backward(Q, K, V, idx_table, gather_table, *([mask_table] if ctx.has_mask else []))
        else:
            ctx.save_for_backward(Q, K, V)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        if ctx.canonical is None:
            if len(ctx.saved_tensors) < 5:
                raise NotImplementedError(
                    "hierarchical_attention backward with tables other than build_tree_topology's needs the "
                    "gather_table that goes with them (the reference's backward kernels read it too)")
            Q, K, V, idx_table, gather_table = ctx.saved_tensors[:5]
            mask_table = ctx.saved_tensors[5] if ctx.has_mask else None
            dq, dk, dv = attention_backward_tables(grad_output, Q, K, V, idx_table, mask_table, gather_table,
                                                   ctx.window_size)
            return dq, dk, dv, None, None, None, None
        if ctx.saved_state:
            Q, K, V, out, lse = ctx.saved_tensors
            if all(t.data_ptr() % 16 == 0 for t in (grad_output.contiguous(), Q, K, V, out)):
                dq, dk, dv = attention_backward_saved(grad_output, Q, K, V, out, lse, ctx.window_size, ctx.canonical)
                return dq, dk, dv, None, None, None, None
        else:
            Q, K, V = ctx.saved_tensors
        dq, dk, dv = attention_backward(grad_output, Q, K, V, ctx.window_size, ctx.canonical)
        return dq, dk, dv, None, None, None, None


def build_parent_nodes(Q_p, K_p, V_p, K_c, V_c):
    """Parent i attends over {itself, children 2i and 2i+1}; returns [B, P, H, D]."""
    return BuildParentNodesFunc.apply(Q_p, K_p, V_p, K_c, V_c)


def hierarchical_attention(Q, K, V, idx_table, gather_table, mask_table=None, window_size=16):
    """Each leaf query attends to keys n-R..n+R plus one tree node per level.
    `mask_table is None` selects the non-causal mode; `gather_table` is unused by the
    forward pass."""
    return HierarchicalAttentionFunc.apply(Q, K, V, idx_table, gather_table, mask_table, window_size)
