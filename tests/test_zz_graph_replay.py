"""HIP-graph capture of the path: the entry points allocate nothing, never synchronise and launch
on the stream they are given, so sequences of calls replay from a graph.  Collected last: these
tests also exercise torch's own kernels under capture."""
import pytest
import torch

import sparseattention_amd as sa
from sparseattention_amd.ops import functional as fn

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_step_replays_from_a_hip_graph():
    """Tree build + span attention captured once into a graph (the entry points allocate nothing,
    never synchronise and launch on the stream they are given), replayed on fresh inputs with
    eager work and synchronisations between the replays; every replay equals the eager result."""
    B, N, H, D, R = 2, 256, 4, 64, 16
    g = torch.Generator().manual_seed(5)
    mk = lambda rows: torch.randn(B, rows, H, D, generator=g).to(torch.bfloat16).to(DEV)
    t = sa.build_tree_topology(N, True, device=DEV)
    q, qp, kp, vp = mk(N), mk(N - 1), mk(N - 1), mk(N - 1)
    kfull = torch.zeros(B, 2 * N - 1, H, D, dtype=torch.bfloat16, device=DEV)
    vfull = torch.zeros_like(kfull)
    out = torch.zeros(B, N, H, D, dtype=torch.bfloat16, device=DEV)

    def step():
        sa.build_tree(qp, kp, vp, kfull[:, :N], vfull[:, :N], out=kfull[:, N:], out2=vfull[:, N:])
        fn.attention_forward(q, kfull, vfull, t["forward_idx"], t["forward_mask"], R, out=out)

    kfull[:, :N], vfull[:, :N] = mk(N), mk(N)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()                                   # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    # the recorded tree build is the one-launch kernel with arrival counters of its own (the eager
    # warm-up above made the counter array's address known): bit for bit the eager result
    _replays_equal_eager(graph, step, mk, q, qp, kp, vp, kfull, vfull, out, N)
    # and the multi-launch build agrees with it to the rounding of one multiply-add
    from sparseattention_amd import _lib
    nodes = kfull[:, N:].clone()
    assert _lib.lib().hsa_build_tree_tune(0, -1) == 0
    try:
        sa.build_tree(qp, kp, vp, kfull[:, :N], vfull[:, :N], out=kfull[:, N:], out2=vfull[:, N:])
        torch.cuda.synchronize()
    finally:
        assert _lib.lib().hsa_build_tree_tune(1, -1) == 0
    assert (nodes.float() - kfull[:, N:].float()).abs().max() <= 2e-2


def test_two_graphs_with_tree_builds_replay_side_by_side():
    """Two recorded tree builds have arrival counters of their own: their graphs replay on two
    streams at the same time, repeatedly, and both keep giving the eager result."""
    B, N, H, D = 4, 2048, 8, 64
    data = []
    for i in range(2):
        g = torch.Generator().manual_seed(40 + i)
        data.append([torch.randn(B, rows, H, D, generator=g).to(torch.bfloat16).to(DEV) for rows in (N - 1, N - 1, N - 1, N, N)])
    want = [sa.build_tree(*d) for d in data]       # eager: also makes the counter array's address known
    torch.cuda.synchronize()
    outs = [torch.zeros_like(w) for w in want]
    graphs = []
    for i in range(2):
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr):
            sa.build_tree(*data[i], out=outs[i])
        graphs.append(gr)
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for rep in range(5):
        for o in outs:
            o.zero_()
        torch.cuda.synchronize()
        for i in range(2):
            with torch.cuda.stream(streams[i]):
                graphs[i].replay()
        torch.cuda.synchronize()
        for i in range(2):
            assert torch.equal(outs[i], want[i]), "graph %d, replay %d" % (i, rep)


def _replays_equal_eager(graph, step, mk, q, qp, kp, vp, kfull, vfull, out, N):
    for rep in range(4):
        for buf, rows in ((q, N), (qp, N - 1), (kp, N - 1), (vp, N - 1)):
            buf.copy_(mk(rows))
        kfull[:, :N].copy_(mk(N))
        vfull[:, :N].copy_(mk(N))
        graph.replay()
        torch.cuda.synchronize()
        got, nodes = out.clone(), kfull[:, N:].clone()
        out.zero_()
        kfull[:, N:].zero_()
        step()                                   # eager, same inputs
        torch.cuda.synchronize()
        assert torch.equal(got, out) and torch.equal(nodes, kfull[:, N:]), "replay %d differs" % rep


def test_lm_forward_replays_from_a_hip_graph():
    """The whole decoder forward (projections by torch, tree and attention by the HIP kernels,
    fused upper levels included) captured into one graph; replays on new token ids, with eager
    forwards and synchronisations in between, equal the eager logits bit for bit."""
    torch.manual_seed(0)
    V, N, B = 211, 256, 2
    model = sa.TransformerLM(V, 256, 4, 512, 2, dropout=0.0, window_size=8, activation="gelu", max_len=N)
    model = model.to(DEV).to(torch.bfloat16).eval()
    tok = torch.randint(0, V, (B, N), device=DEV)
    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                model(tok)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = model(tok)
        for rep in range(3):
            tok.copy_(torch.randint(0, V, (B, N), device=DEV))
            graph.replay()
            torch.cuda.synchronize()
            got = out.clone()
            want = model(tok)
            torch.cuda.synchronize()
            assert torch.equal(got, want), "replay %d differs" % rep


def test_lm_full_benchmark_shape_properties():
    """The decoder-LM benchmark configuration at its FULL shape (6 layers, d_model 512, 8 heads,
    FFN 2048 GELU, vocabulary 50257, bf16, batch 8, 4096 tokens, window 16, random weights): too
    large for the CPU oracle, so what the model's definition fixes is checked: finite logits;
    causality (changing the token at position n leaves the logits of every earlier position bit
    for bit as they were, and changes position n); a HIP-graph replay of the forward reproduces
    the eager logits bit for bit."""
    torch.manual_seed(0)
    V, d, H, ff, layers, N, B, R = 50257, 512, 8, 2048, 6, 4096, 8, 16
    model = sa.TransformerLM(V, d, H, ff, layers, dropout=0.0, window_size=R, activation="gelu", max_len=N)
    model = model.to(DEV).to(torch.bfloat16).eval()
    tok = torch.randint(0, V, (B, N), generator=torch.Generator().manual_seed(0)).to(DEV)
    with torch.no_grad():
        base = model(tok)
        assert base.shape == (B, N, V) and base.dtype == torch.bfloat16
        assert bool(torch.isfinite(base).all())
        n = 2500
        tok2 = tok.clone()
        tok2[:, n] = (tok2[:, n] + 1) % V
        other = model(tok2)
        assert torch.equal(other[:, :n], base[:, :n]), "a later token changed earlier logits"
        assert not torch.equal(other[:, n], base[:, n])
        del other
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            model(tok)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = model(tok)
        for rep in range(2):
            out.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, base), "replay %d differs from the eager forward" % rep
