"""Pins the module-level oracles (`cross_update_y_ref`, `update_x_from_y_ref`, `lm_forward_ref`)
with weights that can be told apart (random, non-symmetric, non-zero biases), against
  * scalar loops written here from the module's definition (one parent / one query / one head at a
    time, numpy only, no oracle function involved),
  * closed forms of special cases (zero query weights make every softmax uniform, so the result is
    a linear recursion in the value weights),
  * for the language model: hand-computable reductions (no layers; zeroed attention outputs).
Each test names the slips it was checked to catch.  No GPU, no reference import.

Reference: hierarchical_attention/modules/attention.py:79-220,
hierarchical_attention_project/Hierarchical_Transformer_Pretrain.py:331-481."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle

DT = torch.float64


def _weights(D, seed, names):
    g = torch.Generator().manual_seed(seed)
    w = {}
    for n in names:
        w[n + ".weight"] = torch.randn(D, D, generator=g, dtype=DT) * 0.7
    return w, g


def _module_weights(D, seed):
    w, g = _weights(D, seed, ["Wq_y", "Wk_y", "Wv_y", "out_proj_y", "Wq_x", "Wk_x", "Wv_x", "out_proj_x"])
    w["out_proj_y.bias"] = torch.randn(D, generator=g, dtype=DT)
    w["out_proj_x.bias"] = torch.randn(D, generator=g, dtype=DT)
    return w, g


def _softmax(s):
    e = np.exp(s - s.max())
    return e / e.sum()


# ------------------------------------------------------------------ cross_update_Y
def cross_update_scalar(x, y, w, H):
    """modules/attention.py:79-162 one parent and one head at a time.  x [N,D], y [N-1,D] numpy."""
    N, D = x.shape
    Dh = D // H
    Wq, Wk, Wv = (w[n + ".weight"].numpy() for n in ("Wq_y", "Wk_y", "Wv_y"))
    children = x                      # rows of the level below, un-projected
    rows, off, P = [], 0, N // 2
    while P >= 1:
        level = np.zeros((P, D))
        for i in range(P):
            node = y[off + i]
            q, kp, vp = Wq @ node, Wk @ node, Wv @ node                  # :101-103 (y = W x, nn.Linear)
            kc = [Wk @ children[2 * i], Wk @ children[2 * i + 1]]        # :116 / :141
            vc = [Wv @ children[2 * i], Wv @ children[2 * i + 1]]        # :117 / :142
            for h in range(H):
                s = slice(h * Dh, (h + 1) * Dh)
                logits = np.array([q[s] @ kp[s], q[s] @ kc[0][s], q[s] @ kc[1][s]]) / math.sqrt(Dh)
                p = _softmax(logits)
                level[i, s] = p[0] * vp[s] + p[1] * vc[0][s] + p[2] * vc[1][s]
        rows.append(level)
        children = level              # :157 the merged-head output is the next level's input
        off += P
        P //= 2
    cat = np.concatenate(rows, 0)
    return cat @ w["out_proj_y.weight"].numpy().T + w["out_proj_y.bias"].numpy()


@pytest.mark.parametrize("shape", [(8, 2, 3), (16, 3, 2), (2, 1, 4)])
def test_cross_update_y_ref_against_scalar_loops(shape):
    """Random distinct weights.  Checked to fail when the oracle swaps Wk_y / Wv_y, drops the
    out_proj_y bias, feeds level l+1 the un-projected or the leaf-level rows, or splits heads
    in a different channel order."""
    N, H, Dh = shape
    D = H * Dh
    w, g = _module_weights(D, seed=N)
    x = torch.randn(2, N, D, generator=g, dtype=DT)
    y = torch.randn(2, N - 1, D, generator=g, dtype=DT)
    got = oracle.cross_update_y_ref(x, y, w, H)
    for b in range(2):
        want = cross_update_scalar(x[b].numpy(), y[b].numpy(), w, H)
        assert np.abs(got[b].numpy() - want).max() < 1e-10


def test_cross_update_y_ref_uniform_softmax_closed_form():
    """Wq_y = 0 makes every 3-way softmax uniform, so level l is a linear recursion:
    out_l[i] = Wv (y_l[i] + c_{2i} + c_{2i+1}) / 3 with c = x at level 1 and c = out_{l-1} above,
    i.e. the leaves enter level l through Wv^l / 3^l.  Fails on a skipped re-projection, on values
    taken through Wk_y, and on a dropped bias; the key weights drop out entirely."""
    N, H, Dh = 16, 2, 3
    D = H * Dh
    w, g = _module_weights(D, seed=3)
    w["Wq_y.weight"] = torch.zeros(D, D, dtype=DT)
    x = torch.randn(1, N, D, generator=g, dtype=DT)
    y = torch.randn(1, N - 1, D, generator=g, dtype=DT)
    Wv = w["Wv_y.weight"]
    c, off, P, rows = x[0], 0, N // 2, []
    while P >= 1:
        lvl = (y[0, off:off + P] + c[0::2] + c[1::2]) @ Wv.T / 3.0
        rows.append(lvl)
        c, off, P = lvl, off + P, P // 2
    want = torch.cat(rows) @ w["out_proj_y.weight"].T + w["out_proj_y.bias"]
    got = oracle.cross_update_y_ref(x, y, w, H)
    assert (got[0] - want).abs().max() < 1e-10
    # the root sees leaf 0 through Wv four times and a factor 3^-4
    w0 = dict(w)
    w0["out_proj_y.weight"] = torch.eye(D, dtype=DT)
    w0["out_proj_y.bias"] = torch.zeros(D, dtype=DT)
    e = torch.zeros(1, N, D, dtype=DT)
    e[0, 0] = torch.randn(D, generator=g, dtype=DT)
    root = oracle.cross_update_y_ref(e, torch.zeros(1, N - 1, D, dtype=DT), w0, H)[0, -1]
    assert (root - torch.linalg.matrix_power(Wv, 4) @ e[0, 0] / 81.0).abs().max() < 1e-12


# ------------------------------------------------------------------ update_X_from_Y
def update_x_scalar(x, y, w, H, R, causal):
    """modules/attention.py:165-220 + the slot definition of ops/triton/sparse_attn.py:8-179, one
    query and one head at a time.  x [N,D], y [N-1,D] numpy."""
    N, D = x.shape
    Dh = D // H
    L = N.bit_length() - 1
    xy = np.concatenate([x, y], 0)                                    # :178 leaves first, then nodes
    Q = x @ w["Wq_x.weight"].numpy().T
    K = xy @ w["Wk_x.weight"].numpy().T
    V = xy @ w["Wv_x.weight"].numpy().T
    heads = np.zeros((N, D))
    for n in range(N):
        rows = [j for j in range(n - R, n + R + 1) if 0 <= j < N and (not causal or j <= n)]
        for l in range(L):
            off = 0 if l == 0 else 2 * N - (N >> (l - 1))
            if not (causal and ((n >> l) & 1) == 0):
                rows.append(off + ((n >> l) ^ 1))                     # a multiset: the sibling leaf twice
        for h in range(H):
            s = slice(h * Dh, (h + 1) * Dh)
            p = _softmax(np.array([Q[n, s] @ K[r, s] for r in rows]) / math.sqrt(Dh))
            heads[n, s] = sum(pi * V[r, s] for pi, r in zip(p, rows))
    return heads @ w["out_proj_x.weight"].numpy().T + w["out_proj_x.bias"].numpy()


@pytest.mark.parametrize("shape", [(8, 2, 3, 2), (16, 2, 2, 0), (16, 1, 4, 5), (2, 2, 2, 1)])
@pytest.mark.parametrize("causal", [True, False])
def test_update_x_from_y_ref_against_scalar_loops(shape, causal):
    """Random distinct weights.  Checked to fail when the oracle swaps Wk_x / Wv_x, drops the
    out_proj_x bias, concatenates [y, x] instead of [x, y], or projects the queries from xy."""
    N, H, Dh, R = shape
    D = H * Dh
    w, g = _module_weights(D, seed=N + R)
    x = torch.randn(2, N, D, generator=g, dtype=DT)
    y = torch.randn(2, N - 1, D, generator=g, dtype=DT)
    got = oracle.update_x_from_y_ref(x, y, w, H, R, causal)
    for b in range(2):
        want = update_x_scalar(x[b].numpy(), y[b].numpy(), w, H, R, causal)
        assert np.abs(got[b].numpy() - want).max() < 1e-10


def test_update_x_from_y_ref_uniform_softmax_closed_form():
    """Wq_x = 0: every live slot gets the same weight, so a query's result is
    out_proj_x(Wv_x · mean over its slot multiset of [x; y] rows) + bias."""
    N, H, Dh, R = 8, 2, 2, 1
    D = H * Dh
    w, g = _module_weights(D, seed=9)
    w["Wq_x.weight"] = torch.zeros(D, D, dtype=DT)
    x = torch.randn(1, N, D, generator=g, dtype=DT)
    y = torch.randn(1, N - 1, D, generator=g, dtype=DT)
    xy = torch.cat([x, y], 1)[0]
    got = oracle.update_x_from_y_ref(x, y, w, H, R, causal=False)[0]
    for n in range(N):
        rows = [j for j in range(n - R, n + R + 1) if 0 <= j < N]
        rows += [(0 if l == 0 else 2 * N - (N >> (l - 1))) + ((n >> l) ^ 1) for l in range(3)]
        mean = xy[rows].mean(0)
        want = w["out_proj_x.weight"] @ (w["Wv_x.weight"] @ mean) + w["out_proj_x.bias"]
        assert (got[n] - want).abs().max() < 1e-12


# ------------------------------------------------------------------ the language model
def _lm_state(V, d, H, ff, layers, seed, max_len=64):
    """A state dict with the reference model's key names (Pretrain.py:358-447) and random
    contents, LayerNorm weights and every bias included."""
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=DT) * 0.3
    sd = {"embedding.weight": r(V, d), "fc_out.bias": r(V)}
    sd["fc_out.weight"] = sd["embedding.weight"]
    pos = torch.arange(0.0, max_len, dtype=DT).unsqueeze(1)
    freq = torch.exp(torch.arange(0.0, d, 2, dtype=DT) * -(math.log(10000.0) / d))
    pe = torch.zeros(max_len, d, dtype=DT)
    pe[:, 0::2], pe[:, 1::2] = torch.sin(pos * freq), torch.cos(pos * freq)
    sd["pos_encoding.pe"] = pe.unsqueeze(0)
    for i in range(layers):
        p = "layers.%d." % i
        for n in ("Wq_y", "Wk_y", "Wv_y", "Wq_x", "Wk_x", "Wv_x", "out_proj_y", "out_proj_x"):
            sd[p + "self_attn." + n + ".weight"] = r(d, d)
        sd[p + "self_attn.out_proj_y.bias"], sd[p + "self_attn.out_proj_x.bias"] = r(d), r(d)
        for n in ("norm1", "norm2", "norm_y"):
            sd[p + n + ".weight"], sd[p + n + ".bias"] = 1 + r(d), r(d)
        sd[p + "feed_forward.fc1.weight"], sd[p + "feed_forward.fc1.bias"] = r(ff, d), r(ff)
        sd[p + "feed_forward.fc2.weight"], sd[p + "feed_forward.fc2.bias"] = r(d, ff), r(d)
    return sd


def _embed(sd, ids):
    d = sd["embedding.weight"].shape[1]
    return sd["embedding.weight"][ids] * math.sqrt(d) + sd["pos_encoding.pe"][0, :ids.shape[1]]


def test_lm_forward_ref_without_layers_is_the_tied_readout():
    """Zero layers: logits = (Emb[ids]·sqrt(d) + PE) · Emb^T + b  (Pretrain.py:443,464-481).
    Fails without the sqrt(d) scale, without the positional term, with an untied read-out or
    without its bias."""
    V, d = 11, 8
    sd = _lm_state(V, d, 2, 16, 0, seed=0)
    ids = torch.tensor([[3, 1, 4, 1, 5, 9, 2, 6], [5, 3, 5, 8, 9, 7, 9, 3]])
    got = oracle.lm_forward_ref(sd, ids, 2, 0, 2)
    want = _embed(sd, ids) @ sd["embedding.weight"].T + sd["fc_out.bias"]
    assert (got - want).abs().max() < 1e-12
    # untied fc_out.weight in the dict must not be consulted: the embedding matrix is the read-out
    sd2 = dict(sd)
    sd2["fc_out.weight"] = torch.zeros(V, d, dtype=DT)
    assert torch.equal(oracle.lm_forward_ref(sd2, ids, 2, 0, 2), got)


@pytest.mark.parametrize("activation", ["relu", "gelu"])
def test_lm_forward_ref_with_silent_attention_is_a_pre_norm_ffn_stack(activation):
    """out_proj_x / out_proj_y weights zero, biases kept: the attention contributes its bias only,
    so a layer is x <- x + b_x ; x <- x + fc2(act(fc1(LN2(x)))) with torch's own layer_norm, and
    the span nodes never reach the logits.  Fails on post-norm, on a missing residual, on the
    wrong activation, on LN2 applied before the attention residual."""
    V, d, H, ff, layers = 13, 8, 2, 12, 2
    sd = _lm_state(V, d, H, ff, layers, seed=1)
    for i in range(layers):
        sd["layers.%d.self_attn.out_proj_x.weight" % i] = torch.zeros(d, d, dtype=DT)
        sd["layers.%d.self_attn.out_proj_y.weight" % i] = torch.zeros(d, d, dtype=DT)
    ids = torch.tensor([[1, 2, 3, 4, 5, 6, 7, 8]])
    got = oracle.lm_forward_ref(sd, ids, H, layers, 2, activation=activation)
    x = _embed(sd, ids)
    act = F.relu if activation == "relu" else F.gelu
    for i in range(layers):
        p = "layers.%d." % i
        x = x + sd[p + "self_attn.out_proj_x.bias"]
        h = F.layer_norm(x, (d,), sd[p + "norm2.weight"], sd[p + "norm2.bias"])
        h = act(h @ sd[p + "feed_forward.fc1.weight"].T + sd[p + "feed_forward.fc1.bias"])
        x = x + h @ sd[p + "feed_forward.fc2.weight"].T + sd[p + "feed_forward.fc2.bias"]
    want = x @ sd["embedding.weight"].T + sd["fc_out.bias"]
    assert (got - want).abs().max() < 1e-10
    other = oracle.lm_forward_ref(sd, ids, H, layers, 2, activation="gelu" if activation == "relu" else "relu")
    assert (other - got).abs().max() > 1e-3


def test_lm_forward_ref_layer_wiring():
    """One full layer against the (pinned) module oracles wired by hand as Pretrain.py:379-431
    does: cross_update_Y gets the UN-normalised leaves and norm_y(span nodes), its result is added
    to the un-normalised span nodes; the attention gets norm1(leaves) and the updated,
    un-normalised span nodes; causal.  The alternatives a slip would produce (normalised leaves
    into cross_update_Y, normalised span nodes into the attention, the old span nodes, non-causal)
    are evaluated too and must differ from the oracle, so the comparison can tell them apart."""
    V, d, H, ff, R = 17, 8, 2, 16, 2
    sd = _lm_state(V, d, H, ff, 1, seed=2)
    ids = torch.tensor([[0, 5, 2, 7, 3, 8, 1, 16, 4, 4, 9, 10, 11, 12, 13, 14]])
    got = oracle.lm_forward_ref(sd, ids, H, 1, R, activation="gelu")
    p = "layers.0."
    w = {k[len(p + "self_attn."):]: v for k, v in sd.items() if k.startswith(p + "self_attn.")}
    ln = lambda t, n: F.layer_norm(t, (d,), sd[p + n + ".weight"], sd[p + n + ".bias"])

    def layer(leaves_for_cross, nodes_for_attn, causal=True):
        x = _embed(sd, ids)
        y0 = oracle.span_input_y_ref(x)
        y1 = y0 + oracle.cross_update_y_ref(leaves_for_cross(x), ln(y0, "norm_y"), w, H)
        x = x + oracle.update_x_from_y_ref(ln(x, "norm1"), nodes_for_attn(y0, y1), w, H, R, causal)
        h = F.gelu(ln(x, "norm2") @ sd[p + "feed_forward.fc1.weight"].T + sd[p + "feed_forward.fc1.bias"])
        x = x + h @ sd[p + "feed_forward.fc2.weight"].T + sd[p + "feed_forward.fc2.bias"]
        return x @ sd["embedding.weight"].T + sd["fc_out.bias"]

    want = layer(lambda x: x, lambda y0, y1: y1)
    assert (got - want).abs().max() < 1e-10
    slips = [layer(lambda x: ln(x, "norm1"), lambda y0, y1: y1),
             layer(lambda x: x, lambda y0, y1: ln(y1, "norm_y")),
             layer(lambda x: x, lambda y0, y1: y0),
             layer(lambda x: x, lambda y0, y1: y1, causal=False)]
    for s in slips:
        assert (s - got).abs().max() > 1e-3


def test_lm_forward_ref_is_causal():
    """A causal model's logits at position n do not change when later tokens change
    (window keys j <= n, tree slots masked by `forward_mask`, span nodes covering the future
    are never attended: Pretrain.py:458-461 hands every layer a mask)."""
    V, d, H, ff, R = 19, 8, 2, 16, 3
    sd = _lm_state(V, d, H, ff, 2, seed=3)
    ids = torch.randint(0, V, (1, 16), generator=torch.Generator().manual_seed(0))
    a = oracle.lm_forward_ref(sd, ids, H, 2, R)
    ids2 = ids.clone()
    ids2[0, 11:] = (ids2[0, 11:] + 1) % V
    b = oracle.lm_forward_ref(sd, ids2, H, 2, R)
    assert (a[0, :11] - b[0, :11]).abs().max() < 1e-12
    assert (a[0, 11:] - b[0, 11:]).abs().max() > 1e-3
