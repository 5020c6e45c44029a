"""CPU oracle for the hierarchical sparse attention forward path.

THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only the test-suite, the smoke
check and the benchmark's `cpu_baseline` leg may import it; the shipped package
never does (it fails loudly when its HIP library is missing instead).

Everything here is a restatement, in plain PyTorch/NumPy on the CPU, of the
algorithm the reference implements.  Each function names the reference lines it
follows.  Paths are relative to the reference checkout.

Pinning status (what independent evidence each function is checked against in
tests/test_oracle.py):

  topology_tables        closed forms, scalar climb (`topology_scalar`), counting
                         invariants, the C brute force                    PINNED
  attention_ref          dense softmax with log-multiplicity bias through
                         torch's scaled_dot_product_attention, per-query
                         Python brute force, the C brute force, closed-form
                         special cases (Q=0, constant V, N=2, causal row 0)  PINNED
  build_parent_nodes_ref F.softmax closed form, Q=0 mean, C brute force   PINNED
  span_input_y_ref       block-mean closed form                           PINNED
  cross_update_y_ref /   scalar per-parent / per-query loops written from the module's
  update_x_from_y_ref    definition with random, distinct weights and biases; the
                         uniform-softmax closed forms (Wq = 0: a linear recursion in
                         Wv, leaves reach level l through Wv^l / 3^l); identity-
                         projection reductions to the op oracles
                         (tests/test_oracle_modules.py)                   PINNED
  lm_forward_ref         (oracle/lm_ref.py) no layers = tied read-out of the scaled,
                         position-encoded embedding; silent attention = pre-norm FFN
                         stack; one layer wired by hand from the pinned module
                         oracles, told apart from four mis-wirings; causality
                         (tests/test_oracle_modules.py)                   PINNED
"""
from __future__ import annotations

import math
from typing import Dict, Optional, Tuple

import numpy as np
import torch
import torch.nn.functional as F


# ---------------------------------------------------------------------------
# Topology
# ---------------------------------------------------------------------------
def topology_tables(seq_len: int, is_causal: bool = True) -> Dict[str, np.ndarray]:
    """Vectorised "climb via the neighbour" construction of the three tables.

    Follows hierarchical_attention/ops/topology.py:6-150:
      * forward table, lines 30-59 (neighbour = sibling of the parent of the
        previous neighbour; future test `pair < n_next`; `max_valid` guard),
      * subtree ranges / node levels, lines 65-100,
      * gather table, lines 103-122.
    Returns int32 `forward_idx [N,L]`, bool `forward_mask [N,L]`,
    int32 `backward_gather [2N-1,3]`.
    """
    assert seq_len >= 1 and (seq_len & (seq_len - 1)) == 0, "seq_len must be power of 2"
    n_nodes = 2 * seq_len - 1
    levels = int(math.log2(seq_len))
    max_valid = n_nodes - 2

    fwd_idx = np.full((seq_len, levels), -1, dtype=np.int32)
    fwd_mask = np.zeros((seq_len, levels), dtype=bool)
    cur = np.arange(seq_len, dtype=np.int64)
    for lvl in range(levels):
        if lvl == 0:
            nxt = cur ^ 1
            pair = cur
        else:
            parent = cur // 2 + seq_len
            nxt = parent ^ 1
            pair = parent
        valid = nxt <= max_valid
        future = pair < nxt
        fwd_idx[:, lvl] = np.where(valid, nxt, fwd_idx[:, lvl])
        if is_causal:
            fwd_mask[:, lvl] = np.where(valid, future, fwd_mask[:, lvl])
        cur = nxt

    rng = np.zeros((n_nodes, 2), dtype=np.int64)
    node_level = np.zeros(n_nodes, dtype=np.int64)
    rng[:seq_len, 0] = np.arange(seq_len)
    rng[:seq_len, 1] = np.arange(seq_len) + 1
    start, count = 0, seq_len
    for lvl in range(levels):
        nstart, ncount = start + count, count // 2
        parents = np.arange(nstart, nstart + ncount)
        left = start + 2 * np.arange(ncount)
        rng[parents, 0] = rng[left, 0]
        rng[parents, 1] = rng[left + 1, 1]
        node_level[parents] = lvl + 1
        start, count = nstart, ncount

    nodes = np.arange(n_nodes)
    sib = np.minimum(nodes ^ 1, n_nodes - 1)
    take = (sib > nodes) if is_causal else (sib != nodes)
    take &= sib != nodes
    gather = np.full((n_nodes, 3), -1, dtype=np.int32)
    gather[take, 0] = rng[sib[take], 0]
    gather[take, 1] = rng[sib[take], 1]
    gather[take, 2] = node_level[take]
    return {"forward_idx": fwd_idx, "forward_mask": fwd_mask, "backward_gather": gather}


def topology_scalar(seq_len: int) -> Tuple[np.ndarray, np.ndarray]:
    """Per-leaf scalar climb; returns (idx_map int64 [N,L], causal_mask bool [N,L]).

    Follows hierarchical_attention_project/Hierarchical_Attention_Triton_Test.py:40-104
    (the table builder of the reference's own PyTorch checker): the mask is
    filled regardless of mode and only applied by the caller when causal.
    """
    assert (seq_len & (seq_len - 1)) == 0
    n_nodes = 2 * seq_len - 1
    max_valid = n_nodes - 2
    levels = int(math.log2(seq_len))
    idx = np.full((seq_len, levels), -1, dtype=np.int64)
    msk = np.zeros((seq_len, levels), dtype=bool)
    for n in range(seq_len):
        cur = n
        for lvl in range(levels):
            if lvl == 0:
                nxt, pair = cur ^ 1, cur
            else:
                nxt, pair = (cur // 2 + seq_len) ^ 1, cur // 2 + seq_len
            if nxt > max_valid:
                break
            if pair < nxt:
                msk[n, lvl] = True
            idx[n, lvl] = nxt
            cur = nxt
    return idx, msk


# ---------------------------------------------------------------------------
# Span attention (window + tree neighbours)
# ---------------------------------------------------------------------------
def attention_ref(Q: torch.Tensor, K: torch.Tensor, V: torch.Tensor,
                  idx_table, mask_table=None, window_size: int = 16,
                  compute_dtype: Optional[torch.dtype] = None,
                  return_weights: bool = False, chunk: int = 4096, query_range=None):
    """Gather + einsum + softmax form of the leaf update.

    Follows hierarchical_attention_project/Hierarchical_Attention_Triton_Test.py:277-337
    (window indices :161-187) and, for the `-1` entries and the op-level calling
    convention (`mask_table is None` means non-causal), the kernel
    hierarchical_attention/ops/triton/sparse_attn.py:40-43,96-117.

    Q [B,N,H,D]; K,V [B,M,H,D] (M = 2N-1 in normal use); idx_table [N,L] ints;
    mask_table [N,L] bool or None.  Returns Out [B,N,H,D] in `compute_dtype`
    (default: Q's dtype, which reproduces the reference's stage-wise rounding),
    and optionally Weights [B,N,H,2R+1+L] (window slots first, then levels).
    `query_range=(lo, hi)` evaluates only queries lo..hi-1 (the other output rows are left
    uninitialised): a bounded sample for timing long sequences.
    """
    B, N, H, D = Q.shape
    R = int(window_size)
    dt = compute_dtype or Q.dtype
    causal = mask_table is not None
    idx_t = torch.as_tensor(np.asarray(idx_table)).long()
    msk_t = torch.as_tensor(np.asarray(mask_table)).bool() if causal else None
    Lv = idx_t.shape[1]

    Qt = Q.to(dt).permute(0, 2, 1, 3)           # [B,H,N,D]
    Kt = K.to(dt).permute(0, 2, 1, 3)
    Vt = V.to(dt).permute(0, 2, 1, 3)
    out = torch.empty(B, H, N, D, dtype=dt)
    wts = torch.empty(B, H, N, 2 * R + 1 + Lv, dtype=dt) if return_weights else None
    offs = torch.arange(-R, R + 1)
    q_lo, q_hi = query_range if query_range is not None else (0, N)
    for s in range(q_lo, q_hi, chunk):
        e = min(q_hi, s + chunk)
        rows = torch.arange(s, e).unsqueeze(1)
        swa = rows + offs.unsqueeze(0)                      # [n, 2R+1]
        valid = (swa >= 0) & (swa < N)
        safe = swa.clamp(0, N - 1)
        q = Qt[:, :, s:e]
        swa_k = Kt[:, :, safe, :]                           # [B,H,n,W,D]
        swa_v = Vt[:, :, safe, :]
        logit_w = torch.einsum('b h l x d, b h l n d -> b h l n', q.unsqueeze(3), swa_k)
        logit_w = logit_w / math.sqrt(D)
        logit_w = logit_w.masked_fill(~valid[None, None], float('-inf'))
        if causal:
            logit_w = logit_w.masked_fill((safe > rows)[None, None], float('-inf'))

        it = idx_t[s:e]
        dead = it < 0
        it_safe = it.clamp(min=0)
        hk = Kt[:, :, it_safe, :]
        hv = Vt[:, :, it_safe, :]
        logit_h = torch.einsum('b h l x d, b h l n d -> b h l n', q.unsqueeze(3), hk)
        logit_h = logit_h / math.sqrt(D)
        logit_h = logit_h.masked_fill(dead[None, None], float('-inf'))
        if causal:
            logit_h = logit_h.masked_fill(msk_t[s:e][None, None], float('-inf'))

        logits = torch.cat([logit_w, logit_h], dim=3)
        vals = torch.cat([swa_v, hv], dim=3)
        mx = logits.max(dim=-1, keepdim=True)[0]
        w = F.softmax(logits - mx, dim=-1)
        out[:, :, s:e] = torch.einsum('b h l n, b h l n d -> b h l d', w, vals)
        if return_weights:
            wts[:, :, s:e] = w
    out = out.permute(0, 2, 1, 3).contiguous()
    if return_weights:
        return out, wts.permute(0, 2, 1, 3).contiguous()
    return out


def slot_multiplicity(N: int, idx_table, mask_table, window_size: int, n_keys: int) -> torch.Tensor:
    """mult[n, j] = how many attention slots of query n point at key row j.

    The multiset view of hierarchical_attention/ops/triton/sparse_attn.py:96-130:
    window slots (in range, and not in the future when causal) plus live tree
    slots.  Used by `attention_dense`.
    """
    R = int(window_size)
    causal = mask_table is not None
    idx = np.asarray(idx_table).astype(np.int64)
    mult = torch.zeros(N, n_keys, dtype=torch.float64)
    for n in range(N):
        lo = max(0, n - R)
        hi = min(N - 1, n if causal else n + R)
        mult[n, lo:hi + 1] += 1
        for l in range(idx.shape[1]):
            m = int(idx[n, l])
            if m < 0:
                continue
            if causal and bool(np.asarray(mask_table)[n, l]):
                continue
            mult[n, m] += 1
    return mult


def attention_dense(Q, K, V, idx_table, mask_table=None, window_size: int = 16) -> torch.Tensor:
    """Independent dense formulation: softmax(QK^T/sqrt(D) + log mult) V in fp64
    through torch's own scaled_dot_product_attention.  A slot multiset softmax
    equals a dense softmax whose additive bias is log(multiplicity)."""
    B, N, H, D = Q.shape
    mult = slot_multiplicity(N, idx_table, mask_table, window_size, K.shape[1])
    bias = torch.where(mult > 0, mult.log(), torch.full_like(mult, float('-inf')))
    q = Q.double().permute(0, 2, 1, 3)
    k = K.double().permute(0, 2, 1, 3)
    v = V.double().permute(0, 2, 1, 3)
    o = F.scaled_dot_product_attention(q, k, v, attn_mask=bias[None, None])
    return o.permute(0, 2, 1, 3).contiguous()


# ---------------------------------------------------------------------------
# BuildParentNodes
# ---------------------------------------------------------------------------
def build_parent_nodes_ref(Q_p, K_p, V_p, K_c, V_c, compute_dtype: Optional[torch.dtype] = None,
                           return_weights: bool = False):
    """Three-way attention of each parent over {itself, child 2i, child 2i+1}.

    Follows hierarchical_attention_project/Hierarchical_Attention_Triton_Test.py:239-251
    (pool = cat[parent, child pair], matmul logits / sqrt(Dh), F.softmax, matmul)
    in the op layout [B,P,H,D] / [B,2P,H,D] of
    hierarchical_attention/ops/functional.py:30-63.  The kernel's `+1e-9` in the
    denominator (ops/triton/build_parents.py:72) changes results by < 1e-9
    relative and is not reproduced here.
    """
    B, P, H, D = Q_p.shape
    assert K_c.shape[1] == 2 * P, "Child count mismatch"
    dt = compute_dtype or Q_p.dtype
    q = Q_p.to(dt).permute(0, 2, 1, 3)                              # [B,H,P,D]
    kp = K_p.to(dt).permute(0, 2, 1, 3)
    vp = V_p.to(dt).permute(0, 2, 1, 3)
    kc = K_c.to(dt).permute(0, 2, 1, 3).reshape(B, H, P, 2, D)
    vc = V_c.to(dt).permute(0, 2, 1, 3).reshape(B, H, P, 2, D)
    k_pool = torch.cat([kp.unsqueeze(3), kc], dim=3)               # [B,H,P,3,D]
    v_pool = torch.cat([vp.unsqueeze(3), vc], dim=3)
    logits = torch.matmul(q.unsqueeze(3), k_pool.transpose(-1, -2)) / math.sqrt(D)
    w = F.softmax(logits, dim=-1)                                   # [B,H,P,1,3]
    o = torch.matmul(w, v_pool).squeeze(3)                          # [B,H,P,D]
    o = o.permute(0, 2, 1, 3).contiguous()
    if return_weights:
        return o, w.squeeze(3).permute(0, 2, 1, 3).contiguous()
    return o


def build_tree_ref(Q_p, K_p, V_p, K_leaf, V_leaf, compute_dtype=None) -> torch.Tensor:
    """Whole tree by iterating the op level by level with an identity map between
    levels: children of level l+1 are level l's outputs, used as both K and V.
    Q_p,K_p,V_p [B,N-1,H,D] are level-concatenated (level 1 first, root last);
    returns the level-concatenated outputs [B,N-1,H,D]."""
    B, N, H, D = K_leaf.shape
    outs, kc, vc, off, P = [], K_leaf, V_leaf, 0, N // 2
    while P >= 1:
        o = build_parent_nodes_ref(Q_p[:, off:off + P], K_p[:, off:off + P], V_p[:, off:off + P],
                                   kc, vc, compute_dtype=compute_dtype)
        o = o.to(Q_p.dtype)
        outs.append(o)
        kc = vc = o
        off += P
        P //= 2
    return torch.cat(outs, dim=1)


# ---------------------------------------------------------------------------
# Y initialisation and the module-level compositions
# ---------------------------------------------------------------------------
def span_input_y_ref(x: torch.Tensor) -> Optional[torch.Tensor]:
    """Level-by-level pairwise means (hierarchical_attention/ops/topology.py:153-169)."""
    B, N, D = x.shape
    levels, cur = [], x
    while cur.size(1) > 1:
        n = cur.size(1)
        even = n - (n % 2)
        pairs = cur[:, :even, :].reshape(B, even // 2, 2, D)
        par = 0.5 * pairs[:, :, 0, :] + 0.5 * pairs[:, :, 1, :]
        levels.append(par)
        cur = par
    if not levels:
        return None
    return torch.cat(levels, dim=1)


def cross_update_y_ref(x, y_in, w: Dict[str, torch.Tensor], num_heads: int) -> torch.Tensor:
    """Bottom-up parent update, eval mode (dropout = identity).

    Follows hierarchical_attention/modules/attention.py:79-162 (same as the
    checker's :201-256): whole-tree parent projections, leaf K/V projected once,
    each further level re-projects the previous level's merged-head output.
    `w` holds Wq_y/Wk_y/Wv_y weights and out_proj_y weight+bias by state-dict name.
    """
    B, N, D = x.shape
    H, Dh = num_heads, D // num_heads
    assert y_in.size(1) == N - 1
    qp = F.linear(y_in, w["Wq_y.weight"]).view(B, -1, H, Dh)
    kp = F.linear(y_in, w["Wk_y.weight"]).view(B, -1, H, Dh)
    vp = F.linear(y_in, w["Wv_y.weight"]).view(B, -1, H, Dh)
    src, off, P, outs = x, 0, N // 2, []
    while P >= 1:
        kc = F.linear(src, w["Wk_y.weight"]).view(B, -1, H, Dh)
        vc = F.linear(src, w["Wv_y.weight"]).view(B, -1, H, Dh)
        o = build_parent_nodes_ref(qp[:, off:off + P], kp[:, off:off + P], vp[:, off:off + P], kc, vc)
        src = o.reshape(B, P, D)
        outs.append(src)
        off += P
        P //= 2
    return F.linear(torch.cat(outs, dim=1), w["out_proj_y.weight"], w["out_proj_y.bias"])


def update_x_from_y_ref(x, y, w: Dict[str, torch.Tensor], num_heads: int, window_size: int,
                        causal: bool) -> torch.Tensor:
    """Top-down leaf update (hierarchical_attention/modules/attention.py:165-220,
    checker :258-341): cat[x,y] -> Wq_x/Wk_x/Wv_x -> span attention -> out_proj_x."""
    B, N, D = x.shape
    H, Dh = num_heads, D // num_heads
    xy = torch.cat([x, y], dim=1)
    q = F.linear(x, w["Wq_x.weight"]).view(B, N, H, Dh)
    k = F.linear(xy, w["Wk_x.weight"]).view(B, -1, H, Dh)
    v = F.linear(xy, w["Wv_x.weight"]).view(B, -1, H, Dh)
    t = topology_tables(N, causal)
    o = attention_ref(q, k, v, t["forward_idx"], t["forward_mask"] if causal else None, window_size)
    return F.linear(o.reshape(B, N, D), w["out_proj_x.weight"], w["out_proj_x.bias"])
