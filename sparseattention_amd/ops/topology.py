"""Tree topology tables and the initial span nodes.

Same call surface as the reference's hierarchical_attention/ops/topology.py
(`build_tree_topology` :6-150, `generate_span_input_Y` :153-169); the tables are
produced from closed forms by the C library (host loop for CPU tensors, a fill
kernel for GPU tensors) instead of a sequence of tensor ops.
"""
from __future__ import annotations

import weakref
from typing import Dict, Optional

import torch

from .. import _lib

# Tables this module produced (or later verified) are remembered so that the
# attention op can skip reading them and use the closed form on chip.
# id(tensor) -> (weakref, version, kind, N, causal)
_KNOWN: Dict[int, tuple] = {}


def _remember(t: torch.Tensor, kind: str, n: int, causal: bool):
    key = id(t)
    _KNOWN[key] = (weakref.ref(t, lambda _r, k=key: _KNOWN.pop(k, None)), t._version, kind, n, causal)


# Tables of unknown origin that were compared with the canonical ones and differ:
# id(tensor) -> (weakref, version).  Saves the comparison (a host sync) on later calls.
_KNOWN_OTHER: Dict[int, tuple] = {}


def remember_other(t: torch.Tensor):
    key = id(t)
    _KNOWN_OTHER[key] = (weakref.ref(t, lambda _r, k=key: _KNOWN_OTHER.pop(k, None)), t._version)


def known_other(t: Optional[torch.Tensor]) -> bool:
    """True if `t` was found to differ from the canonical table and has not been written since."""
    if t is None:
        return False
    rec = _KNOWN_OTHER.get(id(t))
    return rec is not None and rec[0]() is t and rec[1] == t._version


def known_table(t: Optional[torch.Tensor], kind: str):
    """(N, causal) if `t` is an unmodified canonical table of that kind, else None."""
    if t is None:
        return None
    rec = _KNOWN.get(id(t))
    if rec is None or rec[0]() is not t or rec[1] != t._version or rec[2] != kind:
        return None
    return rec[3], rec[4]


def build_tree_topology(seq_len: int, is_causal: bool = True, device="cuda",
                        dtype=torch.int32) -> Dict[str, torch.Tensor]:
    """Lookup tables of the complete binary tree over `seq_len` leaves.

    forward_idx  [N, L]     row of the sibling/uncle node each leaf attends to per level
    forward_mask [N, L]     bool, True = masked (the neighbour lies in the future); all
                            False when not causal
    backward_gather [2N-1,3] (start, end, level): leaf range under each node's sibling,
                            -1 rows for the root and (causal) for right-hand nodes
    """
    assert (seq_len & (seq_len - 1)) == 0, "seq_len must be power of 2"
    assert seq_len >= 1
    L = seq_len.bit_length() - 1
    dev = torch.device(device)
    idx = torch.empty((seq_len, L), dtype=torch.int32, device=dev)
    msk = torch.empty((seq_len, L), dtype=torch.uint8, device=dev)
    gat = torch.empty((2 * seq_len - 1, 3), dtype=torch.int32, device=dev)
    lib = _lib.lib()
    if dev.type == "cuda":
        with _lib.on_device(idx):
            rc = lib.hsa_topology_device(seq_len, int(bool(is_causal)), _lib.ptr(idx), _lib.ptr(msk),
                                         _lib.ptr(gat), _lib.stream_of(idx))
    else:
        rc = lib.hsa_topology_host(seq_len, int(bool(is_causal)), _lib.ptr(idx), _lib.ptr(msk), _lib.ptr(gat))
    _lib.check(rc, "hsa_topology")
    fmask = msk.view(torch.bool)
    if dtype != torch.int32:
        idx = idx.to(dtype)
        gat = gat.to(dtype)
    _remember(idx, "idx", seq_len, bool(is_causal))
    _remember(fmask, "mask", seq_len, bool(is_causal))
    return {"forward_idx": idx, "forward_mask": fmask, "backward_gather": gat}


class _SpanInputY(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        B, N, C = x.shape
        x = x.contiguous()
        y = torch.empty((B, N - bin(N).count("1"), C), dtype=x.dtype, device=x.device)
        with _lib.on_device(x):
            rc = _lib.lib().hsa_span_input_y(_lib.ptr(x), _lib.ptr(y), B, N, C, _lib.dtype_code(x),
                                             _lib.stream_of(x))
        _lib.check(rc, "hsa_span_input_y")
        ctx.leaves = N
        return y

    @staticmethod
    def backward(ctx, dy):
        B, M, C = dy.shape
        dy = dy.contiguous()
        N = ctx.leaves
        dx = torch.empty((B, N, C), dtype=dy.dtype, device=dy.device)
        with _lib.on_device(dy):
            rc = _lib.lib().hsa_span_input_y_bwd(_lib.ptr(dy), _lib.ptr(dx), B, N, C, _lib.dtype_code(dy),
                                                 _lib.stream_of(dy))
        _lib.check(rc, "hsa_span_input_y_bwd")
        return dx


def generate_span_input_Y(x: torch.Tensor) -> Optional[torch.Tensor]:
    """Initial span nodes: pairwise means level by level, [B, N, C] -> [B, N-1, C] (any N: an unpaired
    last row of a level has no parent, N - popcount(N) rows in all)."""
    B, N, C = x.shape
    if N < 2:
        return None
    _lib.require_gpu(x)
    _lib.dtype_code(x)
    return _SpanInputY.apply(x)
