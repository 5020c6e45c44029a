"""Pins the CPU oracle against independent formulations (no GPU, no reference import).

The reference ships no golden vectors for this path, so each oracle function is
checked against evidence a plausible mistake would break: closed forms, a dense
library formulation, brute force, and hand-computable special cases.
"""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle


def closed_form_tables(N, causal):
    L = N.bit_length() - 1
    n = np.arange(N)[:, None]
    l = np.arange(L)[None, :]
    off = np.where(l == 0, 0, 2 * N - (N >> np.maximum(l - 1, 0)))
    idx = (off + ((n >> l) ^ 1)).astype(np.int32)
    mask = (((n >> l) & 1) == 0) & causal
    gather = np.full((2 * N - 1, 3), -1, np.int32)
    for lv in range(L + 1):
        o = 0 if lv == 0 else 2 * N - (N >> (lv - 1))
        for j in range(N >> lv):
            i = o + j
            if i == 2 * N - 2 or (causal and j & 1):
                continue
            gather[i] = (((j ^ 1) << lv), ((j ^ 1) + 1) << lv, lv)
    return idx, mask, gather


@pytest.mark.parametrize("N", [1, 2, 4, 8, 32, 256, 2048])
@pytest.mark.parametrize("causal", [True, False])
def test_topology_closed_form_and_scalar(N, causal, bf):
    t = oracle.topology_tables(N, causal)
    idx, mask, gather = closed_form_tables(N, causal)
    assert t["forward_idx"].dtype == np.int32
    np.testing.assert_array_equal(t["forward_idx"], idx)
    np.testing.assert_array_equal(t["forward_mask"], mask)
    np.testing.assert_array_equal(t["backward_gather"], gather)
    if N <= 256:
        sidx, smask = oracle.topology_scalar(N)
        np.testing.assert_array_equal(sidx, idx)
        np.testing.assert_array_equal(smask & causal, mask)
    bidx, bmask, bgather = bf.topology(N, causal)
    np.testing.assert_array_equal(bidx, idx)
    np.testing.assert_array_equal(bmask, mask)
    np.testing.assert_array_equal(bgather, gather)


@pytest.mark.parametrize("N", [4, 64, 1024])
def test_topology_invariants(N):
    L = N.bit_length() - 1
    t = oracle.topology_tables(N, True)
    idx, mask = t["forward_idx"], t["forward_mask"]
    assert idx.min() >= 0 and idx.max() <= 2 * N - 3          # never the root, never -1
    assert set(np.unique(idx)) == set(range(2 * N - 2))       # every non-root node is someone's neighbour
    for l in range(L):
        _, counts = np.unique(idx[:, l], return_counts=True)
        assert (counts == (1 << l)).all()                     # a level-l node serves 2^l leaves
    pop = np.array([bin(n).count("1") for n in range(N)])
    np.testing.assert_array_equal(mask.sum(1), L - pop)       # masked levels = zero bits of n
    g = t["backward_gather"]
    assert (g[2 * N - 2] == -1).all()
    # sibling leaf ranges tile the leaves level by level
    live = g[g[:, 0] >= 0]
    assert ((live[:, 1] - live[:, 0]) == (1 << live[:, 2])).all()


def _rand(B, N, H, D, seed=0, M=None):
    g = torch.Generator().manual_seed(seed)
    M = M or 2 * N - 1
    return (torch.randn(B, N, H, D, generator=g), torch.randn(B, M, H, D, generator=g),
            torch.randn(B, M, H, D, generator=g))


@pytest.mark.parametrize("N,R", [(2, 1), (8, 0), (8, 3), (16, 16), (64, 5), (256, 8)])
@pytest.mark.parametrize("causal", [True, False])
def test_attention_three_formulations_agree(N, R, causal, bf):
    B, H, D = 2, 3, 16
    Q, K, V = _rand(B, N, H, D, seed=N + R)
    t = oracle.topology_tables(N, causal)
    m = t["forward_mask"] if causal else None
    ref = oracle.attention_ref(Q, K, V, t["forward_idx"], m, R, compute_dtype=torch.float64)
    dense = oracle.attention_dense(Q, K, V, t["forward_idx"], m, R)
    brute, bw = bf.attention(Q, K, V, t["forward_idx"], m, R, want_weights=True)
    assert (ref - dense).abs().max() < 1e-12
    assert np.abs(ref.numpy() - brute).max() < 2e-6
    _, w = oracle.attention_ref(Q, K, V, t["forward_idx"], m, R, compute_dtype=torch.float64,
                                return_weights=True)
    assert np.abs(w.numpy() - bw).max() < 1e-6
    assert torch.allclose(w.sum(-1), torch.ones_like(w.sum(-1)))


def test_attention_python_bruteforce_small():
    """Per-query loops written from the slot definition, N=16."""
    B, N, H, D, R = 1, 16, 2, 8, 2
    Q, K, V = _rand(B, N, H, D, seed=5)
    for causal in (True, False):
        t = oracle.topology_tables(N, causal)
        got = oracle.attention_ref(Q, K, V, t["forward_idx"], t["forward_mask"] if causal else None, R,
                                   compute_dtype=torch.float64)
        L = N.bit_length() - 1
        for n in range(N):
            rows = [j for j in range(n - R, n + R + 1) if 0 <= j < N and (not causal or j <= n)]
            for l in range(L):
                if causal and ((n >> l) & 1) == 0:
                    continue
                off = 0 if l == 0 else 2 * N - (N >> (l - 1))
                rows.append(off + ((n >> l) ^ 1))
            for h in range(H):
                s = torch.stack([(Q[0, n, h].double() * K[0, r, h].double()).sum() for r in rows]) / math.sqrt(D)
                p = torch.softmax(s, 0)
                want = sum(p[i] * V[0, r, h].double() for i, r in enumerate(rows))
                assert (got[0, n, h] - want).abs().max() < 1e-12


def test_attention_special_cases():
    B, N, H, D, R = 1, 32, 2, 8, 4
    Q, K, V = _rand(B, N, H, D, seed=9)
    tc = oracle.topology_tables(N, True)
    tn = oracle.topology_tables(N, False)
    # causal row 0 sees only itself
    out = oracle.attention_ref(Q, K, V, tc["forward_idx"], tc["forward_mask"], R)
    assert torch.allclose(out[:, 0], V[:, 0], atol=1e-6)
    # constant V -> that constant
    Vc = torch.full_like(V, 0.75)
    out = oracle.attention_ref(Q, K, Vc, tn["forward_idx"], None, R)
    assert torch.allclose(out, torch.full_like(out, 0.75), atol=1e-6)
    # Q = 0 -> multiplicity-weighted mean of the attended rows (sibling leaf twice)
    out = oracle.attention_ref(torch.zeros_like(Q), K, V, tn["forward_idx"], None, R,
                               compute_dtype=torch.float64)
    mult = oracle.slot_multiplicity(N, tn["forward_idx"], None, R, 2 * N - 1)
    assert mult[5, 4] == 2 and mult[5, 5] == 1 and mult[4, 5] == 2
    want = torch.einsum("nj,bjhd->bnhd", mult / mult.sum(1, keepdim=True), V.double())
    assert (out - want).abs().max() < 1e-12
    # R = 0, non causal: {self} + L nodes, every slot once
    mult0 = oracle.slot_multiplicity(N, tn["forward_idx"], None, 0, 2 * N - 1)
    assert (mult0.sum(1) == 1 + 5).all() and mult0.max() == 1
    # N = 2 by hand: query 1 causal attends {0 (window), 1 (self), 0 (level-0 sibling)}
    Q2, K2, V2 = _rand(1, 2, 1, 4, seed=3)
    t2 = oracle.topology_tables(2, True)
    o2 = oracle.attention_ref(Q2, K2, V2, t2["forward_idx"], t2["forward_mask"], 1, compute_dtype=torch.float64)
    s = torch.stack([(Q2[0, 1, 0].double() * K2[0, j, 0].double()).sum() / 2.0 for j in (0, 1, 0)])
    p = torch.softmax(s, 0)
    V2 = V2.double()
    want = p[0] * V2[0, 0, 0] + p[1] * V2[0, 1, 0] + p[2] * V2[0, 0, 0]
    assert (o2[0, 1, 0] - want).abs().max() < 1e-12


def test_attention_dead_slots_minus_one():
    """-1 entries are dead slots (kernel semantics), not a wrap to the last row."""
    B, N, H, D, R = 1, 8, 1, 4, 1
    Q, K, V = _rand(B, N, H, D, seed=2)
    t = oracle.topology_tables(N, False)
    idx = t["forward_idx"].copy()
    idx[:, 2] = -1
    got = oracle.attention_ref(Q, K, V, idx, None, R, compute_dtype=torch.float64)
    dense = oracle.attention_dense(Q, K, V, idx, None, R)
    assert (got - dense).abs().max() < 1e-12
    full = oracle.attention_ref(Q, K, V, t["forward_idx"], None, R, compute_dtype=torch.float64)
    assert (got - full).abs().max() > 1e-3


@pytest.mark.parametrize("P", [1, 4, 33])
def test_build_parents(P, bf):
    B, H, D = 2, 3, 16
    g = torch.Generator().manual_seed(P)
    qp, kp, vp = (torch.randn(B, P, H, D, generator=g) for _ in range(3))
    kc, vc = (torch.randn(B, 2 * P, H, D, generator=g) for _ in range(2))
    got, w = oracle.build_parent_nodes_ref(qp, kp, vp, kc, vc, compute_dtype=torch.float64, return_weights=True)
    # closed form per element
    qd, kpd, kcd, vpd, vcd = (t.double() for t in (qp, kp, kc, vp, vc))
    s = torch.stack([(qd * kpd).sum(-1), (qd * kcd[:, 0::2]).sum(-1), (qd * kcd[:, 1::2]).sum(-1)], -1) / math.sqrt(D)
    p = F.softmax(s, -1)
    want = p[..., 0:1] * vpd + p[..., 1:2] * vcd[:, 0::2] + p[..., 2:3] * vcd[:, 1::2]
    assert (got - want).abs().max() < 1e-12
    assert (w - p).abs().max() < 1e-12
    brute, bw = bf.build_parents(qp, kp, vp, kc, vc, want_weights=True)
    assert np.abs(got.numpy() - brute).max() < 1e-6
    assert np.abs(p.numpy() - bw).max() < 1e-6
    # zero query -> plain mean of the three value rows
    z = oracle.build_parent_nodes_ref(torch.zeros_like(qp), kp, vp, kc, vc)
    assert torch.allclose(z, (vp + vc[:, 0::2] + vc[:, 1::2]) / 3, atol=1e-6)


def test_build_tree_composition():
    B, N, H, D = 1, 8, 2, 4
    g = torch.Generator().manual_seed(1)
    qp, kp, vp = (torch.randn(B, N - 1, H, D, generator=g) for _ in range(3))
    kl, vl = (torch.randn(B, N, H, D, generator=g) for _ in range(2))
    out = oracle.build_tree_ref(qp, kp, vp, kl, vl)
    o1 = oracle.build_parent_nodes_ref(qp[:, :4], kp[:, :4], vp[:, :4], kl, vl)
    o2 = oracle.build_parent_nodes_ref(qp[:, 4:6], kp[:, 4:6], vp[:, 4:6], o1, o1)
    o3 = oracle.build_parent_nodes_ref(qp[:, 6:7], kp[:, 6:7], vp[:, 6:7], o2, o2)
    assert torch.equal(out, torch.cat([o1, o2, o3], 1))


def test_span_input_y_block_means():
    B, N, C = 2, 16, 5
    x = torch.randn(B, N, C, dtype=torch.float64)
    y = oracle.span_input_y_ref(x)
    assert y.shape == (B, N - 1, C)
    off = 0
    for lvl in range(1, 5):
        cnt = N >> lvl
        want = x.view(B, cnt, 1 << lvl, C).mean(2)
        assert (y[:, off:off + cnt] - want).abs().max() < 1e-12
        off += cnt
    assert oracle.span_input_y_ref(torch.randn(1, 1, 3)) is None


def test_module_compositions_reduce_to_ops():
    """With identity projections and zero bias the module-level oracles are the op oracles."""
    B, N, H, Dh, R = 1, 16, 2, 4, 2
    D = H * Dh
    g = torch.Generator().manual_seed(4)
    x = torch.randn(B, N, D, generator=g)
    y = torch.randn(B, N - 1, D, generator=g)
    eye = torch.eye(D)
    w = {k: eye for k in ["Wq_y.weight", "Wk_y.weight", "Wv_y.weight", "out_proj_y.weight",
                          "Wq_x.weight", "Wk_x.weight", "Wv_x.weight", "out_proj_x.weight"]}
    w["out_proj_y.bias"] = torch.zeros(D)
    w["out_proj_x.bias"] = torch.zeros(D)
    yh = y.view(B, N - 1, H, Dh)
    xh = x.view(B, N, H, Dh)
    got = oracle.cross_update_y_ref(x, y, w, H)
    want = oracle.build_tree_ref(yh, yh, yh, xh, xh).reshape(B, N - 1, D)
    assert torch.allclose(got, want, atol=1e-6)
    for causal in (True, False):
        t = oracle.topology_tables(N, causal)
        got = oracle.update_x_from_y_ref(x, y, w, H, R, causal)
        xy = torch.cat([x, y], 1).view(B, 2 * N - 1, H, Dh)
        want = oracle.attention_ref(xh, xy, xy, t["forward_idx"], t["forward_mask"] if causal else None, R)
        assert torch.allclose(got, want.reshape(B, N, D), atol=1e-6)


def test_oracle_gradients_are_true_derivatives():
    """The backward parity tests differentiate the oracle with autograd; check that against
    finite differences on tiny fp64 problems."""
    g = torch.Generator().manual_seed(0)
    B, N, H, D, R = 1, 8, 1, 4, 2
    q = torch.randn(B, N, H, D, generator=g, dtype=torch.float64, requires_grad=True)
    k = torch.randn(B, 2 * N - 1, H, D, generator=g, dtype=torch.float64, requires_grad=True)
    v = torch.randn(B, 2 * N - 1, H, D, generator=g, dtype=torch.float64, requires_grad=True)
    t = oracle.topology_tables(N, True)
    f = lambda a, b, c: oracle.attention_ref(a, b, c, t["forward_idx"], t["forward_mask"], R)
    assert torch.autograd.gradcheck(f, (q, k, v), eps=1e-6, atol=1e-6)
    qp, kp, vp = (torch.randn(1, 2, 1, 4, generator=g, dtype=torch.float64, requires_grad=True) for _ in range(3))
    kc, vc = (torch.randn(1, 4, 1, 4, generator=g, dtype=torch.float64, requires_grad=True) for _ in range(2))
    assert torch.autograd.gradcheck(oracle.build_parent_nodes_ref, (qp, kp, vp, kc, vc), eps=1e-6, atol=1e-6)


# ---------------------------------------------------------------- committed vectors
def _golden():
    import os
    return np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "small_case.npz"))


@pytest.mark.parametrize("causal", [True, False])
def test_oracle_matches_committed_vectors(causal):
    """tests/golden/small_case.npz (written by the scalar brute force) against the torch oracle."""
    g = _golden()
    tag = "causal" if causal else "full"
    t = oracle.topology_tables(64, causal)
    np.testing.assert_array_equal(t["forward_idx"], g["idx_" + tag])
    np.testing.assert_array_equal(t["forward_mask"], g["mask_" + tag])
    np.testing.assert_array_equal(t["backward_gather"], g["gather_" + tag])
    q, k, v = (torch.from_numpy(g[n]) for n in "qkv")
    out, w = oracle.attention_ref(q, k, v, t["forward_idx"], t["forward_mask"] if causal else None,
                                  int(g["radius"]), compute_dtype=torch.float64, return_weights=True)
    assert (out.double() - torch.from_numpy(g["attn_out_" + tag]).double()).abs().max() < 1e-6
    assert (w.double() - torch.from_numpy(g["attn_weights_" + tag]).double()).abs().max() < 1e-6
    ops = [torch.from_numpy(g[n]) for n in ("qp", "kp", "vp", "kc", "vc")]
    po, pw = oracle.build_parent_nodes_ref(*ops, compute_dtype=torch.float64, return_weights=True)
    assert (po.double() - torch.from_numpy(g["parents_out"]).double()).abs().max() < 1e-6
    assert (pw.double() - torch.from_numpy(g["parents_weights"]).double()).abs().max() < 1e-6

