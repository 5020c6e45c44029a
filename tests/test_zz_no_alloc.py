"""`hsa_attn_bwd_static`: the span-attention backward whose scratch is a buffer inside the
library's device image, for callers that cannot allocate.  Called through the C ABI and compared
bit for bit with `hsa_attn_bwd` on a caller-provided workspace (same kernels, deterministic), on
two calls in a row, the second on a smaller problem, so that whatever the first call left in the
shared buffer must not leak into the second.  Collected last."""
import pytest
import torch

import oracle
from sparseattention_amd import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _inputs(B, N, H, D, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    mk = lambda rows: torch.randn(B, rows, H, D, generator=g).to(dtype)
    return mk(N), mk(2 * N - 1), mk(2 * N - 1), mk(N)


def _both(lib, case, causal, algo):
    """(dq, dk, dv) from hsa_attn_bwd with a torch workspace, and from hsa_attn_bwd_static."""
    B, N, H, D, R, dtype = case
    q, k, v, go = (t.to(DEV) for t in _inputs(B, N, H, D, dtype, seed=N + R))
    L = N.bit_length() - 1
    M = 2 * N - 1
    code, st = _lib.dtype_code(q), _lib.stream_of(q)
    a = _lib.algo_code(algo)
    nbytes = int(lib.hsa_attn_bwd_workspace_bytes(B, N, M, H, D, L, R, code, a))
    assert nbytes <= lib.hsa_attn_bwd_static_capacity()
    ws = torch.empty(nbytes // 4 + 1, dtype=torch.float32, device=DEV)
    want = [torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)]
    got = [torch.full_like(q, float("nan")), torch.full_like(k, float("nan")), torch.full_like(v, float("nan"))]
    rc = lib.hsa_attn_bwd(_lib.ptr(q), _lib.ptr(k), _lib.ptr(v), _lib.ptr(go), *map(_lib.ptr, want), _lib.ptr(ws),
                          ws.numel() * 4, B, N, M, H, D, L, R, int(causal), code, a, st)
    _lib.check(rc, "hsa_attn_bwd")
    rc = lib.hsa_attn_bwd_static(_lib.ptr(q), _lib.ptr(k), _lib.ptr(v), _lib.ptr(go), *map(_lib.ptr, got),
                                 B, N, M, H, D, L, R, int(causal), code, a, st)
    _lib.check(rc, "hsa_attn_bwd_static")
    torch.cuda.synchronize()
    return (q, k, v, go), want, got


@pytest.mark.parametrize("algo", ["auto", "gather"])
def test_static_scratch_backward_matches_workspace_backward(algo):
    lib = _lib.lib()
    big = (2, 1024, 4, 64, 16, torch.bfloat16)     # tile kernels: per-block partial rows for levels >= 4
    small = (1, 64, 3, 64, 5, torch.bfloat16)      # second call, smaller: reuses the start of the buffer
    for case in (big, small):
        for causal in (True, False):
            inp, want, got = _both(lib, case, causal, algo)
            for name, w, g in zip(("dQ", "dK", "dV"), want, got):
                assert torch.equal(w, g), "%s differs (case %s, causal %s, %s)" % (name, case, causal, algo)
    # and the small case against the oracle's autograd, to the gradient bar of the other tests
    B, N, H, D, R, dtype = small
    (q, k, v, go), _, got = _both(lib, small, True, algo)
    o = oracle.topology_tables(N, True)
    qr, kr, vr = (t.cpu().double().requires_grad_(True) for t in (q, k, v))
    oracle.attention_ref(qr, kr, vr, o["forward_idx"], o["forward_mask"], R).backward(go.cpu().double())
    for name, g, r in zip(("dQ", "dK", "dV"), got, (qr.grad, kr.grad, vr.grad)):
        err = float((g.double().cpu() - r).abs().max())
        assert err <= 3e-2 * max(1.0, float(r.abs().max())), "%s vs oracle: %.3e" % (name, err)


def test_static_scratch_backward_fp32_and_limit():
    lib = _lib.lib()
    inp, want, got = _both(lib, (1, 128, 2, 32, 4, torch.float32), True, "auto")
    for w, g in zip(want, got):
        assert torch.equal(w, g)
    # a problem whose workspace exceeds the built-in buffer is refused, nothing is launched
    B, N, H, D, R = 8, 8192, 8, 64, 16
    L, M = 13, 2 * N - 1
    assert lib.hsa_attn_bwd_workspace_bytes(B, N, M, H, D, L, R, 2, 0) > lib.hsa_attn_bwd_static_capacity()
    dummy = torch.empty(16, device=DEV)
    rc = lib.hsa_attn_bwd_static(*([_lib.ptr(dummy)] * 7), B, N, M, H, D, L, R, 1, 2, 0, _lib.stream_of(dummy))
    assert rc == -95
    assert b"scratch" in lib.hsa_last_error()


def test_static_scratch_backward_records_into_a_graph():
    """After the set-up call the static entry is nothing but kernel launches: it can be recorded
    into a HIP graph; every replay (with eager work and synchronisations in between) reproduces
    the eager gradients bit for bit."""
    lib = _lib.lib()
    assert lib.hsa_attn_bwd_static_capacity() > 0          # resolves the buffer's address on this GPU
    B, N, H, D, R, dtype = 2, 512, 4, 64, 16, torch.bfloat16
    q, k, v, go = (t.to(DEV) for t in _inputs(B, N, H, D, dtype, seed=7))
    L, M = N.bit_length() - 1, 2 * N - 1
    code = _lib.dtype_code(q)
    outs = [torch.zeros_like(q), torch.zeros_like(k), torch.zeros_like(v)]

    def call():
        rc = lib.hsa_attn_bwd_static(_lib.ptr(q), _lib.ptr(k), _lib.ptr(v), _lib.ptr(go), *map(_lib.ptr, outs),
                                     B, N, M, H, D, L, R, 1, code, 0, _lib.stream_of(q))
        _lib.check(rc, "hsa_attn_bwd_static")

    call()
    torch.cuda.synchronize()
    want = [t.clone() for t in outs]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for rep in range(3):
        for t in outs:
            t.fill_(float("nan"))      # eager work between the replays (a fill kernel, no memset node)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, w, g in zip(("dQ", "dK", "dV"), want, outs):
            assert torch.equal(w, g), "%s differs on replay %d" % (name, rep)
