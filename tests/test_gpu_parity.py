"""GPU parity: every kernel, called through the C ABI, against the CPU oracle on the same
seeded inputs.  Tolerances: fp32 1e-5 max-abs; bf16/fp16 2e-2 abs + 1e-2 relative against
the oracle evaluated in fp64 on the rounded inputs; index tables bit-exact."""
import math

import numpy as np
import pytest
import torch

import oracle
import sparseattention_amd as sa
from conftest import error_figures, report
from sparseattention_amd import _lib
from sparseattention_amd.ops import functional as fn

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16, torch.float16]


def tol(dtype):
    return (1e-5, 0.0) if dtype == torch.float32 else (2e-2, 1e-2)


def assert_close(got, want, dtype, what=""):
    atol, rtol = tol(dtype)
    got = got.detach().double().cpu()
    want = want.double()
    err = (got - want).abs()
    bound = atol + rtol * want.abs()
    bad = err > bound
    assert not bad.any(), "%s: %d elements out of tolerance, max abs err %.3e (dtype %s)" % (
        what, int(bad.sum()), float(err.max()), dtype)


@pytest.fixture
def tile_knobs():
    """Sets launch parameters of the tile kernels for one test and restores the defaults."""
    from sparseattention_amd import _lib

    def set_knobs(sb, wpb, swizzle, alternate):
        assert _lib.lib().hsa_attn_tile_tune(sb, wpb, swizzle, alternate) == 0
    yield set_knobs
    assert _lib.lib().hsa_attn_tile_tune(0, 0, 1, 1) == 0


@pytest.fixture
def top_knob():
    """Chooses between one launch per level (0) and the single launch (1) of the span-node update's
    upper levels for one test and restores the default."""
    from sparseattention_amd import _lib

    def set_knob(single_launch):
        assert _lib.lib().hsa_cross_update_top_tune(single_launch) == 0
    yield set_knob
    assert _lib.lib().hsa_cross_update_top_tune(0) == 0


def make_qkv(B, N, H, D, dtype, seed=0, scale=1.0, M=None):
    g = torch.Generator().manual_seed(seed)
    M = M or 2 * N - 1
    q = (torch.randn(B, N, H, D, generator=g) * scale).to(dtype)
    k = (torch.randn(B, M, H, D, generator=g) * scale).to(dtype)
    v = (torch.randn(B, M, H, D, generator=g) * scale).to(dtype)
    return q, k, v


# ---------------------------------------------------------------- topology
@pytest.mark.parametrize("N", [1, 2, 16, 2048, 65536])
@pytest.mark.parametrize("causal", [True, False])
def test_topology_device_bit_exact(N, causal):
    t = sa.build_tree_topology(N, causal, device=DEV)
    o = oracle.topology_tables(N, causal)
    assert t["forward_idx"].dtype == torch.int32 and t["forward_mask"].dtype == torch.bool
    np.testing.assert_array_equal(t["forward_idx"].cpu().numpy(), o["forward_idx"])
    np.testing.assert_array_equal(t["forward_mask"].cpu().numpy(), o["forward_mask"])
    np.testing.assert_array_equal(t["backward_gather"].cpu().numpy(), o["backward_gather"])


# ---------------------------------------------------------------- span attention, gather kernel
CASES = [  # B, N, H, D, R
    (2, 2, 1, 8, 1),
    (1, 8, 3, 16, 0),
    (2, 16, 2, 32, 3),
    (2, 64, 5, 64, 8),
    (1, 128, 2, 128, 40),      # 2R+1+L = 88 slots: more than one lane pass
    (2, 256, 4, 32, 8),        # the CPU plumbing configuration
    (1, 32, 2, 20, 2),         # head_dim not a power of two
]


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("causal", [True, False])
def test_attention_gather_vs_oracle(case, dtype, causal):
    B, N, H, D, R = case
    q, k, v = make_qkv(B, N, H, D, dtype, seed=N + R)
    t = sa.build_tree_topology(N, causal, device=DEV)
    o = oracle.topology_tables(N, causal)
    m_dev = t["forward_mask"] if causal else None
    out, w = fn.attention_forward(q.to(DEV), k.to(DEV), v.to(DEV), t["forward_idx"], m_dev, R,
                                  return_weights=True, algo="gather")
    assert out.dtype == dtype and out.shape == q.shape and w.dtype == torch.float32
    want, ww = oracle.attention_ref(q, k, v, o["forward_idx"], o["forward_mask"] if causal else None, R,
                                    compute_dtype=torch.float64, return_weights=True)
    assert_close(out, want, dtype, "out")
    assert (w.double().cpu() - ww).abs().max() < (1e-6 if dtype == torch.float32 else 2e-2)
    assert torch.allclose(w.sum(-1), torch.ones_like(w.sum(-1)), atol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_custom_tables_with_dead_slots(dtype):
    """Arbitrary neighbour tables: -1 entries, an arbitrary mask, more key rows than 2N-1."""
    B, N, H, D, R, M = 2, 32, 3, 16, 2, 80
    q, k, v = make_qkv(B, N, H, D, dtype, seed=11, M=M)
    rng = np.random.default_rng(0)
    L = 6
    idx = rng.integers(0, M, size=(N, L)).astype(np.int32)
    idx[rng.random((N, L)) < 0.2] = -1
    mask = rng.random((N, L)) < 0.3
    idx_d = torch.from_numpy(idx).to(DEV)
    mask_d = torch.from_numpy(mask).to(DEV)
    for m_np, m_dev in ((mask, mask_d), (None, None)):
        out = sa.hierarchical_attention(q.to(DEV), k.to(DEV), v.to(DEV), idx_d, None, m_dev, R)
        want = oracle.attention_ref(q, k, v, idx, m_np, R, compute_dtype=torch.float64)
        assert_close(out, want, dtype, "custom tables")


def test_attention_unknown_canonical_table_is_verified_once():
    N, R = 64, 4
    q, k, v = make_qkv(1, N, 2, 32, torch.float32, seed=3)
    o = oracle.topology_tables(N, True)
    idx_d = torch.from_numpy(o["forward_idx"]).to(DEV)        # same contents, unknown origin
    mask_d = torch.from_numpy(o["forward_mask"]).to(DEV)
    assert fn._is_canonical(idx_d, mask_d, N) is None
    out = sa.hierarchical_attention(q.to(DEV), k.to(DEV), v.to(DEV), idx_d, None, mask_d, R)
    assert fn._is_canonical(idx_d, mask_d, N) is True
    want = oracle.attention_ref(q, k, v, o["forward_idx"], o["forward_mask"], R, compute_dtype=torch.float64)
    assert_close(out, want, torch.float32)


def test_attention_inputs_untouched_and_noncontiguous():
    N, R = 32, 3
    q, k, v = make_qkv(2, N, 2, 16, torch.float32, seed=8)
    qd = q.to(DEV).transpose(1, 2).contiguous().transpose(1, 2)      # non-contiguous view
    kd, vd = k.to(DEV), v.to(DEV)
    kc, vc = kd.clone(), vd.clone()
    t = sa.build_tree_topology(N, True, device=DEV)
    out = sa.hierarchical_attention(qd, kd, vd, t["forward_idx"], t["backward_gather"], t["forward_mask"], R)
    assert torch.equal(kd, kc) and torch.equal(vd, vc) and out.is_contiguous()
    o = oracle.topology_tables(N, True)
    want = oracle.attention_ref(q, k, v, o["forward_idx"], o["forward_mask"], R, compute_dtype=torch.float64)
    assert_close(out, want, torch.float32)


def test_timed_entry_point_same_output_and_a_kernel_interval():
    """hsa_attn_fwd_timed: identical result, and the two events bracket the kernel itself."""
    import ctypes
    from sparseattention_amd import _lib
    B, N, H, D, R = 2, 256, 4, 64, 8
    L, M = 8, 2 * N - 1
    q, k, v = make_qkv(B, N, H, D, torch.bfloat16, seed=3)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    t = sa.build_tree_topology(N, True, device=DEV)
    want = fn.attention_forward(qd, kd, vd, t["forward_idx"], t["forward_mask"], R)
    lib = _lib.lib()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(); e1.record()          # creates the underlying HIP events
    torch.cuda.synchronize()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for algo in (_lib.ATTN_TILE, _lib.ATTN_GATHER):
        out = torch.zeros_like(qd)
        rc = lib.hsa_attn_fwd_timed(_lib.ptr(qd), _lib.ptr(kd), _lib.ptr(vd), None, None, _lib.ptr(out), None,
                                    B, N, M, H, D, L, R, 1, _lib.HSA_BF16, algo, st,
                                    ctypes.c_void_p(e0.cuda_event), ctypes.c_void_p(e1.cuda_event))
        assert rc == 0, lib.hsa_last_error()
        torch.cuda.synchronize()
        ref = want if algo == _lib.ATTN_TILE else fn.attention_forward(qd, kd, vd, t["forward_idx"],
                                                                       t["forward_mask"], R, algo="gather")
        assert torch.equal(out, ref)
        assert 0.0 < e0.elapsed_time(e1) < 50.0
    # a plain call afterwards is not affected by the events of the timed one
    assert torch.equal(fn.attention_forward(qd, kd, vd, t["forward_idx"], t["forward_mask"], R), want)
    assert lib.hsa_attn_fwd_timed(_lib.ptr(qd), _lib.ptr(kd), _lib.ptr(vd), None, None, _lib.ptr(out), None,
                                  B, N, M, H, D, L, R, 1, _lib.HSA_BF16, 0, st, None, None) == -22


def test_empty_batch_gives_empty_outputs():
    N, H, D = 16, 2, 8
    t = sa.build_tree_topology(N, True, device=DEV)
    z = lambda rows: torch.zeros(0, rows, H, D, device=DEV, requires_grad=True)
    q, k, v = z(N), z(2 * N - 1), z(2 * N - 1)
    out = sa.hierarchical_attention(q, k, v, t["forward_idx"], t["backward_gather"], t["forward_mask"], 2)
    assert out.shape == (0, N, H, D)
    out.sum().backward()
    assert q.grad.shape == q.shape and k.grad.shape == k.shape
    par = sa.build_parent_nodes(z(4), z(4), z(4), z(8), z(8))
    assert par.shape == (0, 4, H, D)
    par.sum().backward()
    assert sa.build_tree(z(N - 1), z(N - 1), z(N - 1), z(N), z(N)).shape == (0, N - 1, H, D)


@pytest.mark.parametrize("causal", [True, False])
def test_kernels_match_committed_vectors(causal):
    """tests/golden/small_case.npz: tables bit-exact, fp32 outputs and weights within 1e-5."""
    import os
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "small_case.npz"))
    tag = "causal" if causal else "full"
    t = sa.build_tree_topology(64, causal, device=DEV)
    np.testing.assert_array_equal(t["forward_idx"].cpu().numpy(), g["idx_" + tag])
    np.testing.assert_array_equal(t["forward_mask"].cpu().numpy(), g["mask_" + tag])
    np.testing.assert_array_equal(t["backward_gather"].cpu().numpy(), g["gather_" + tag])
    q, k, v = (torch.from_numpy(g[n]).to(DEV) for n in "qkv")
    out, w = fn.attention_forward(q, k, v, t["forward_idx"], t["forward_mask"] if causal else None,
                                  int(g["radius"]), return_weights=True)
    assert (out.cpu() - torch.from_numpy(g["attn_out_" + tag])).abs().max() < 1e-5
    assert (w.cpu() - torch.from_numpy(g["attn_weights_" + tag])).abs().max() < 1e-5
    ops = [torch.from_numpy(g[n]).to(DEV) for n in ("qp", "kp", "vp", "kc", "vc")]
    po, pw = fn.build_parents_forward(*ops, return_weights=True)
    assert (po.cpu() - torch.from_numpy(g["parents_out"])).abs().max() < 1e-5
    assert (pw.cpu() - torch.from_numpy(g["parents_weights"])).abs().max() < 1e-5
    # bf16 on the same vectors, at its own tolerance
    qb, kb, vb = (x.to(torch.bfloat16) for x in (q, k, v))
    ob = fn.attention_forward(qb, kb, vb, t["forward_idx"], t["forward_mask"] if causal else None,
                              int(g["radius"]))
    # the committed answer belongs to the fp32 inputs; the bf16 kernel sees rounded inputs, so its
    # bar (2e-2 + 1e-2 |ref|) is taken against the oracle on those rounded inputs
    o = oracle.topology_tables(64, causal)
    ref = oracle.attention_ref(qb.cpu(), kb.cpu(), vb.cpu(), o["forward_idx"], o["forward_mask"] if causal else None,
                               int(g["radius"]), compute_dtype=torch.float64)
    assert_close(ob, ref, torch.bfloat16, "bf16 on the committed inputs")


# ---------------------------------------------------------------- parent build
@pytest.mark.parametrize("shape", [(2, 1, 1, 8), (2, 5, 3, 16), (1, 64, 8, 64), (2, 16, 4, 128), (1, 7, 2, 20),
                                   (3, 33, 12, 64)])
@pytest.mark.parametrize("dtype", DTYPES)
def test_build_parents_vs_oracle(shape, dtype):
    B, P, H, D = shape
    g = torch.Generator().manual_seed(P * 7 + D)
    qp, kp, vp = (torch.randn(B, P, H, D, generator=g).to(dtype) for _ in range(3))
    kc, vc = (torch.randn(B, 2 * P, H, D, generator=g).to(dtype) for _ in range(2))
    out, w = fn.build_parents_forward(*(t.to(DEV) for t in (qp, kp, vp, kc, vc)), return_weights=True)
    assert out.dtype == dtype and w.dtype == dtype and w.shape == (B, P, H, 3)
    want, ww = oracle.build_parent_nodes_ref(qp, kp, vp, kc, vc, compute_dtype=torch.float64, return_weights=True)
    assert_close(out, want, dtype, "bpn out")
    assert (w.double().cpu() - ww).abs().max() < (1e-6 if dtype == torch.float32 else 1e-2)
    # the public op
    out2 = sa.build_parent_nodes(*(t.to(DEV) for t in (qp, kp, vp, kc, vc)))
    assert torch.equal(out, out2)


@pytest.mark.parametrize("shape", [(2, 5, 3, 16), (3, 32, 8, 64), (1, 1, 2, 128), (2, 7, 2, 20)])
@pytest.mark.parametrize("dtype", DTYPES)
def test_build_parents_column_slices(shape, dtype):
    """Operands that are thirds / halves of wider matrices (fused projections): same bits as the
    dense call, both outputs written, bytes around the outputs untouched."""
    B, P, H, D = shape
    g = torch.Generator().manual_seed(P + D)
    qkv = torch.randn(B, P, 3, H, D, generator=g).to(dtype).to(DEV)
    kv = torch.randn(B, 2 * P, 2, H, D, generator=g).to(dtype).to(DEV)
    big = torch.full((B, P + 3, H, D), 7.0, dtype=dtype, device=DEV)
    out = torch.empty(B, P, H, D, dtype=dtype, device=DEV)
    got = fn.build_parents_strided(qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], kv[:, :, 0], kv[:, :, 1],
                                   out=out, out2=big[:, 2:2 + P])
    ops = [t.contiguous() for t in (qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], kv[:, :, 0], kv[:, :, 1])]
    dense = fn.build_parents_forward(*ops)
    assert got is out and torch.equal(out, dense) and torch.equal(big[:, 2:2 + P], dense)
    assert (big[:, :2] == 7).all() and (big[:, 2 + P:] == 7).all()
    want = oracle.build_parent_nodes_ref(*(t.cpu() for t in ops), compute_dtype=torch.float64)
    assert_close(out, want, dtype, "bpn column slices")
    with pytest.raises(AssertionError):
        fn.build_parents_strided(qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], kv[:, :P, 0], kv[:, :P, 1], out=out)


@pytest.mark.parametrize("B,C,H,Dh", [(2, 64, 8, 64), (3, 32, 4, 32), (1, 2, 2, 64), (2, 16, 2, 128), (2, 32, 4, 128),
                                      (1, 8, 16, 32), (2, 64, 12, 32)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("single", [0, 1])
def test_cross_update_top_levels(B, C, H, Dh, dtype, single, top_knob):
    """All levels above C rows in one call (one fused launch per level, or a single launch):
    against the mathematics in fp64 (projection, 3-way softmax, level after level) and against the
    level-by-level kernels."""
    top_knob(single)
    dim = H * Dh
    assert C <= fn.fused_top_rows(H, Dh, dtype)
    g = torch.Generator().manual_seed(C + H)
    src = torch.randn(B, C, dim, generator=g).clamp(-1, 1).to(dtype)
    big = torch.randn(B, C + 4, 3 * dim, generator=g).clamp(-1, 1).to(dtype)   # parents' rows sit at 3..C+1
    w = (torch.randn(2 * dim, dim, generator=g) / dim ** 0.5).to(dtype)
    qkv = big[:, 3:3 + C - 1]
    outbig = torch.full((B, C + 1, dim), 5.0, dtype=dtype, device=DEV)
    bigd = big.to(DEV)
    wp = fn.pack_kv_weights(w[:dim].to(DEV), w[dim:].to(DEV), H)
    got = fn.cross_update_top(src.to(DEV), bigd[:, 3:3 + C - 1], wp, outbig[:, 1:C], H)
    assert (outbig[:, 0] == 5).all() and (outbig[:, C] == 5).all()
    # fp64 on the same 16-bit inputs
    cur, off, P, want = src.double(), 0, C // 2, []
    while P >= 1:
        kv = torch.nn.functional.linear(cur, w.double()).view(B, 2 * P, 2, H, Dh)
        par = qkv[:, off:off + P].double().view(B, P, 3, H, Dh)
        o = oracle.build_parent_nodes_ref(par[:, :, 0], par[:, :, 1], par[:, :, 2], kv[:, :, 0], kv[:, :, 1])
        cur = o.reshape(B, P, dim)
        want.append(cur)
        off, P = off + P, P // 2
    want = torch.cat(want, dim=1)
    report("cross_update_top_levels %s" % ((B, C, H, Dh, str(dtype), single),), **error_figures(got, want))
    # measured max-abs error: 8.4e-3 (bf16), 9.4e-4 (fp16) over these shapes; bar = 2.5 x that
    assert (got.double().cpu() - want).abs().max() < (2.1e-2 if dtype == torch.bfloat16 else 2.4e-3)
    # level by level on the GPU (each level's projection rounded to the element type, as here)
    cur, off, P, ref = src.to(DEV), 0, C // 2, []
    while P >= 1:
        kv = torch.nn.functional.linear(cur, w.to(DEV)).view(B, 2 * P, 2, H, Dh)
        par = bigd[:, 3 + off:3 + off + P].view(B, P, 3, H, Dh)
        o = torch.empty(B, P, H, Dh, dtype=dtype, device=DEV)
        fn.build_parents_strided(par[:, :, 0], par[:, :, 1], par[:, :, 2], kv[:, :, 0], kv[:, :, 1], out=o)
        cur = o.view(B, P, dim)
        ref.append(cur)
        off, P = off + P, P // 2
    assert (got.float() - torch.cat(ref, dim=1).float()).abs().max() < 2e-2


@pytest.mark.parametrize("B,C,H,Dh", [(2, 64, 8, 64), (2, 32, 12, 64), (3, 16, 4, 128), (1, 64, 16, 32)])
def test_cross_update_top_both_forms_agree(B, C, H, Dh, top_knob):
    """One launch per level and the single launch round at the same places: same bits.  Result rows
    that do not allow 16-byte reads (odd row stride) take the single launch by themselves."""
    dim = H * Dh
    g = torch.Generator().manual_seed(7 * C + H)
    src = torch.randn(B, C, dim, generator=g).clamp(-1, 1).to(torch.bfloat16).to(DEV)
    qkv = torch.randn(B, C - 1, 3 * dim, generator=g).clamp(-1, 1).to(torch.bfloat16).to(DEV)
    w = (torch.randn(2 * dim, dim, generator=g) / dim ** 0.5).to(torch.bfloat16).to(DEV)
    wp = fn.pack_kv_weights(w[:dim], w[dim:], H)
    outs = []
    for single in (0, 1):
        top_knob(single)
        outs.append(fn.cross_update_top(src, qkv, wp, torch.empty(B, C - 1, dim, dtype=torch.bfloat16, device=DEV), H))
    assert torch.equal(outs[0], outs[1])
    top_knob(0)
    wide = torch.full((B, C - 1, dim + 4), 3.0, dtype=torch.bfloat16, device=DEV)
    got = fn.cross_update_top(src, qkv, wp, wide[:, :, :dim], H)
    assert torch.equal(got, outs[0]) and (wide[:, :, dim:] == 3).all()


@pytest.mark.parametrize("B,C,H,Dh", [(1, 1024, 4, 64), (2, 256, 8, 64), (1, 128, 2, 128)])
def test_cross_update_top_many_rows_per_level_launches(B, C, H, Dh, top_knob):
    """More children than the single launch holds: one launch per level takes them in 16-row tiles
    (against the level-by-level kernels); the single launch refuses."""
    dim = H * Dh
    assert C > fn.fused_top_rows(H, Dh, torch.bfloat16)
    g = torch.Generator().manual_seed(C + H)
    src = torch.randn(B, C, dim, generator=g).clamp(-1, 1).to(torch.bfloat16).to(DEV)
    qkv = torch.randn(B, C - 1, 3 * dim, generator=g).clamp(-1, 1).to(torch.bfloat16).to(DEV)
    w = (torch.randn(2 * dim, dim, generator=g) / dim ** 0.5).to(torch.bfloat16).to(DEV)
    wp = fn.pack_kv_weights(w[:dim], w[dim:], H)
    got = fn.cross_update_top(src, qkv, wp, torch.empty(B, C - 1, dim, dtype=torch.bfloat16, device=DEV), H)
    cur, off, P, ref = src, 0, C // 2, []
    while P >= 1:
        kv = torch.nn.functional.linear(cur, w).view(B, 2 * P, 2, H, Dh)
        par = qkv[:, off:off + P].view(B, P, 3, H, Dh)
        o = torch.empty(B, P, H, Dh, dtype=torch.bfloat16, device=DEV)
        fn.build_parents_strided(par[:, :, 0], par[:, :, 1], par[:, :, 2], kv[:, :, 0], kv[:, :, 1], out=o)
        cur = o.view(B, P, dim)
        ref.append(cur)
        off, P = off + P, P // 2
    assert (got.float() - torch.cat(ref, dim=1).float()).abs().max() < 2e-2
    top_knob(1)
    with pytest.raises(sa.HsaError):
        fn.cross_update_top(src, qkv, wp, torch.empty(B, C - 1, dim, dtype=torch.bfloat16, device=DEV), H)
    lib = _lib.lib()
    assert lib.hsa_cross_update_level_rows(B, H, Dh, _lib.HSA_BF16) == fn.fused_top_rows(H, Dh, torch.bfloat16)
    top_knob(0)
    # heads whose weights fit the LDS hand every level over; 128-channel heads while B * C <= 8192
    assert lib.hsa_cross_update_level_rows(1, 8, 64, _lib.HSA_BF16) == 1 << 20
    assert lib.hsa_cross_update_level_rows(8, 8, 64, _lib.HSA_BF16) == 1 << 20
    assert lib.hsa_cross_update_level_rows(8, 16, 64, _lib.HSA_BF16) == 1024     # 256 KiB of weights per head
    assert lib.hsa_cross_update_level_rows(1, 4, 128, _lib.HSA_BF16) == 8192
    assert lib.hsa_cross_update_level_rows(8, 4, 128, _lib.HSA_BF16) == 1024
    assert lib.hsa_cross_update_level_tune(-1, 4096) == 0
    assert lib.hsa_cross_update_level_rows(8, 8, 64, _lib.HSA_BF16) == 512
    assert lib.hsa_cross_update_level_tune(-1, 0) == 0
    assert lib.hsa_cross_update_level_rows(4096, 4, 128, _lib.HSA_BF16) == fn.fused_top_rows(4, 128, torch.bfloat16)
    assert lib.hsa_cross_update_level_rows(1, 3, 24, _lib.HSA_BF16) == 0


@pytest.mark.parametrize("B,C,H,Dh", [(8, 1024, 8, 64), (8, 512, 8, 64), (2, 1024, 8, 64), (16, 256, 4, 32), (4, 512, 2, 128),
                                      (8, 256, 6, 64), (3, 128, 4, 64),
                                      # several groups of row tiles per workgroup, the weights resident in LDS
                                      (8, 2048, 8, 64), (16, 1024, 8, 64), (6, 4096, 8, 64), (2, 4096, 6, 64), (4, 2048, 8, 32)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_cross_update_levels_weights_staged_per_workgroup(B, C, H, Dh, dtype):
    """Large levels run on the kernels that keep a head's weights in LDS (staged in chunks per
    workgroup: two row tiles per wavefront or one, one or two workgroups per CU, chunks of four or
    eight k-steps, a model width that is no multiple of 256; or resident while a workgroup walks
    several groups of row tiles, an uneven share of groups included): bit-identical to the launch
    per wavefront and row tile, which rounds at the same places, and close to the level-by-level
    kernels."""
    dim = H * Dh
    g = torch.Generator().manual_seed(C + H + B)
    src = torch.randn(B, C, dim, generator=g).clamp(-1, 1).to(dtype).to(DEV)
    qkv = torch.randn(B, C - 1, 3 * dim, generator=g).clamp(-1, 1).to(dtype).to(DEV)
    w = (torch.randn(2 * dim, dim, generator=g) / dim ** 0.5).to(dtype).to(DEV)
    wp = fn.pack_kv_weights(w[:dim], w[dim:], H)
    lib = _lib.lib()
    outs = {}
    try:
        for min_tiles in (0, 1):   # never / every level with at least one 16-row tile
            assert lib.hsa_cross_update_level_tune(min_tiles, -1) == 0
            outs[min_tiles] = fn.cross_update_top(src, qkv, wp, torch.empty(B, C - 1, dim, dtype=dtype, device=DEV), H)
    finally:
        assert lib.hsa_cross_update_level_tune(8, -1) == 0
    assert torch.equal(outs[0], outs[1])
    cur, off, P, ref = src, 0, C // 2, []
    while P >= 1:
        kv = torch.nn.functional.linear(cur, w).view(B, 2 * P, 2, H, Dh)
        par = qkv[:, off:off + P].view(B, P, 3, H, Dh)
        o = torch.empty(B, P, H, Dh, dtype=dtype, device=DEV)
        fn.build_parents_strided(par[:, :, 0], par[:, :, 1], par[:, :, 2], kv[:, :, 0], kv[:, :, 1], out=o)
        cur = o.view(B, P, dim)
        ref.append(cur)
        off, P = off + P, P // 2
    assert (outs[1].float() - torch.cat(ref, dim=1).float()).abs().max() < 2e-2


def test_cross_update_top_shapes_not_handled(top_knob):
    top_knob(1)   # the single launch: more rows than it holds are refused
    assert fn.fused_top_rows(8, 64, torch.float32) == 0
    assert fn.fused_top_rows(3, 24, torch.bfloat16) == 0
    assert fn.fused_top_rows(8, 64, torch.bfloat16) == 64 and fn.fused_top_rows(8, 128, torch.bfloat16) == 32
    z = torch.zeros(1, 128, 512, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(sa.HsaError):
        fn.cross_update_top(z, torch.zeros(1, 127, 1536, dtype=torch.bfloat16, device=DEV),
                            torch.zeros(1024 * 512, dtype=torch.bfloat16, device=DEV),
                            torch.zeros(1, 127, 512, dtype=torch.bfloat16, device=DEV), 8)


def test_build_parents_child_count_assert():
    z = torch.zeros(1, 4, 1, 8, device=DEV)
    with pytest.raises(AssertionError):
        sa.build_parent_nodes(z, z, z, z, z)


@pytest.mark.parametrize("N,H,D", [(2, 4, 64), (4, 4, 64), (8, 1, 8), (16, 3, 20), (64, 4, 64), (128, 12, 64),
                                   (512, 4, 64), (1024, 2, 128), (32, 1, 520)])
@pytest.mark.parametrize("dtype", DTYPES)
def test_build_tree_vs_oracle(N, H, D, dtype):
    B = 2
    g = torch.Generator().manual_seed(N)
    qp, kp, vp = (torch.randn(B, N - 1, H, D, generator=g).to(dtype) for _ in range(3))
    kl, vl = (torch.randn(B, N, H, D, generator=g).to(dtype) for _ in range(2))
    out = sa.build_tree(*(t.to(DEV) for t in (qp, kp, vp, kl, vl)))
    want = oracle.build_tree_ref(qp, kp, vp, kl, vl, compute_dtype=torch.float64)
    # each level is rounded to the element type before feeding the next one in both
    assert_close(out, want, dtype, "tree")
    # writing straight into the node rows of a K_full buffer
    kfull = torch.zeros(B, 2 * N - 1, H, D, dtype=dtype, device=DEV)
    kfull[:, :N] = kl.to(DEV)
    vfull = torch.zeros_like(kfull)
    sa.build_tree(*(t.to(DEV) for t in (qp, kp, vp)), kfull[:, :N], vl.to(DEV), out=kfull[:, N:],
                  out2=vfull[:, N:])
    assert torch.equal(kfull[:, N:], out) and torch.equal(vfull[:, N:], out)
    assert torch.equal(kfull[:, :N], kl.to(DEV)) and not vfull[:, :N].any()


@pytest.fixture
def tree_knobs():
    """Sets how hsa_build_tree_fwd runs for one test and restores the defaults."""
    from sparseattention_amd import _lib

    def set_knobs(single_launch, threads):
        assert _lib.lib().hsa_build_tree_tune(single_launch, threads) == 0
    yield set_knobs
    assert _lib.lib().hsa_build_tree_tune(1, 0) == 0


# shapes chosen so that the single launch finishes 0..4 levels inside a workgroup and closes the
# rest in one, two or several rounds of "last workgroup to arrive" (N=16384 with 16 heads of 128:
# two subtrees per workgroup, four rounds)
FUSED_TREE_CASES = [(2, 8, 8, 64), (3, 64, 8, 64), (2, 512, 8, 64), (8, 2048, 8, 64), (1, 16384, 16, 128),
                    (2, 1024, 2, 64), (2, 256, 1, 32), (1, 4096, 4, 128), (2, 2048, 16, 64), (1, 8192, 8, 32)]


@pytest.mark.parametrize("case", FUSED_TREE_CASES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("threads", [0, 64, 128, 256, 512])
def test_build_tree_single_launch(case, dtype, threads, tree_knobs):
    """The whole tree in one launch against the oracle and against the multi-launch path, for
    every workgroup size; run twice on the same buffers (the arrival counters must be back at
    zero after a launch)."""
    B, N, H, D = case
    g = torch.Generator().manual_seed(N + H)
    qp, kp, vp = (torch.randn(B, N - 1, H, D, generator=g).to(dtype).to(DEV) for _ in range(3))
    kl, vl = (torch.randn(B, N, H, D, generator=g).to(dtype).to(DEV) for _ in range(2))
    tree_knobs(0, -1)
    stepwise = sa.build_tree(qp, kp, vp, kl, vl)
    tree_knobs(2, threads)
    out2 = torch.empty_like(stepwise)
    fused = sa.build_tree(qp, kp, vp, kl, vl, out2=out2)
    again = sa.build_tree(qp, kp, vp, kl, vl)
    assert torch.equal(fused, again) and torch.equal(fused, out2)
    want = oracle.build_tree_ref(qp.cpu(), kp.cpu(), vp.cpu(), kl.cpu(), vl.cpu(), compute_dtype=torch.float64)
    assert_close(fused, want, dtype, "single launch")
    # same arithmetic in both paths: they may differ by the rounding of one fused multiply-add
    atol = 1e-6 if dtype == torch.float32 else 2e-2
    assert (fused.float() - stepwise.float()).abs().max() <= atol


def test_build_tree_long_sequence_against_level_by_level():
    """B1 H16 N65536 D128 bf16, both node copies written (537 MB: the size from which the multi-launch
    build stores with the streaming hint): every level against the one-level op applied to the
    tree's own previous level, so that nothing but one level's rounding separates the two."""
    B, H, N, D = 1, 16, 65536, 128
    g = torch.Generator(device=DEV).manual_seed(5)
    mk = lambda rows: torch.randn(B, rows, H, D, generator=g, device=DEV, dtype=torch.float32).to(torch.bfloat16)
    qp, kp, vp = mk(N - 1), mk(N - 1), mk(N - 1)
    kfull = torch.zeros(B, 2 * N - 1, H, D, dtype=torch.bfloat16, device=DEV)
    vfull = torch.zeros_like(kfull)
    kfull[:, :N] = mk(N)
    vfull[:, :N] = mk(N)
    sa.build_tree(qp, kp, vp, kfull[:, :N], vfull[:, :N], out=kfull[:, N:], out2=vfull[:, N:])
    assert torch.equal(kfull[:, N:], vfull[:, N:])
    kc, vc, off = kfull[:, :N], vfull[:, :N], 0
    for lvl in range(1, N.bit_length()):
        P = N >> lvl
        want = sa.build_parent_nodes(qp[:, off:off + P], kp[:, off:off + P], vp[:, off:off + P], kc, vc)
        got = kfull[:, N + off:N + off + P]
        assert (got.float() - want.float()).abs().max() <= 2e-2, "level %d" % lvl
        kc = vc = got
        off += P
    assert off == N - 1


def test_build_tree_single_launch_on_concurrent_streams(tree_knobs):
    """Launches on different streams overlap on the GPU and must not share arrival counters:
    four streams each build their own tree several times while the others run."""
    tree_knobs(2, 512)
    B, N, H, D = 4, 2048, 8, 64
    streams = [torch.cuda.Stream() for _ in range(4)]
    data, outs = [], []
    for i in range(4):
        g = torch.Generator().manual_seed(100 + i)
        data.append([torch.randn(B, rows, H, D, generator=g).to(torch.bfloat16).to(DEV)
                     for rows in (N - 1, N - 1, N - 1, N, N)])
        outs.append([torch.empty(B, N - 1, H, D, dtype=torch.bfloat16, device=DEV) for _ in range(6)])
    torch.cuda.synchronize()
    for rep in range(6):
        for i, st in enumerate(streams):
            with torch.cuda.stream(st):
                sa.build_tree(*data[i], out=outs[i][rep])
    torch.cuda.synchronize()
    tree_knobs(0, -1)
    for i in range(4):
        want = sa.build_tree(*data[i])
        for rep in range(6):
            assert (outs[i][rep].float() - want.float()).abs().max() <= 2e-2, "stream %d repetition %d" % (i, rep)
            assert torch.equal(outs[i][rep], outs[i][0])


# ---------------------------------------------------------------- initial span nodes
@pytest.mark.parametrize("shape", [(2, 2, 8), (1, 64, 48), (2, 4096, 512), (1, 128, 7),
                                   # lengths that are no power of two, as the reference accepts them
                                   # (hierarchical_attention/ops/topology.py:158-162): an unpaired last row
                                   # of a level has no parent
                                   (2, 3, 8), (1, 5, 4), (2, 100, 24), (1, 1023, 16), (1, 4097, 8), (2, 33, 5)])
@pytest.mark.parametrize("dtype", DTYPES)
def test_span_input_y_bit_exact(shape, dtype):
    B, N, C = shape
    x = torch.randn(B, N, C, generator=torch.Generator().manual_seed(N)).to(dtype)
    y = sa.generate_span_input_Y(x.to(DEV))
    want = oracle.span_input_y_ref(x)
    assert y.dtype == dtype and y.shape == (B, N - bin(N).count("1"), C)
    assert torch.equal(y.cpu(), want)
    assert sa.generate_span_input_Y(x[:, :1].to(DEV)) is None


# ---------------------------------------------------------------- module
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("causal", [True, False])
def test_module_vs_oracle(dtype, causal):
    B, N, dim, H, R = 2, 64, 128, 4, 4
    torch.manual_seed(0)
    m = sa.HierarchicalAttention(dim, H, dropout=0.0, window_size=R).eval()
    x = torch.randn(B, N, dim).clamp(-1, 1)
    y = torch.randn(B, N - 1, dim).clamp(-1, 1)
    w32 = {k: v.detach().clone() for k, v in m.state_dict().items()}
    md = m.to(DEV).to(dtype)
    xd, yd = x.to(DEV).to(dtype), y.to(DEV).to(dtype)
    # oracle on the rounded parameters / inputs, in fp64 for a tight comparison
    wr = {k: v.to(dtype).double() for k, v in w32.items()}
    xr, yr = x.to(dtype).double(), y.to(dtype).double()
    with torch.no_grad():
        y_new = md.cross_update_Y(xd, yd)
        want_y = oracle.cross_update_y_ref(xr, yr, wr, H)
        mask = torch.ones(B, N, dtype=torch.bool, device=DEV) if causal else None
        out = md(xd, xd, xd, y=yd, mask=mask)
        want = oracle.update_x_from_y_ref(xr, yr, wr, H, R, causal)
    # GEMM chains (the reference's own bar is 1e-2..5e-2); measured max-abs error in bf16: 2.3e-3
    # (fp32: 3e-7); bar = 2.5 x that
    atol = 1e-4 if dtype == torch.float32 else 6e-3
    report("module_vs_oracle %s causal=%s" % (dtype, causal), y=error_figures(y_new, want_y), out=error_figures(out, want))
    assert (y_new.double().cpu() - want_y).abs().max() < atol
    assert (out.double().cpu() - want).abs().max() < atol
    assert md(xd, xd, xd, y=yd, mask=mask, return_attention=True)[1] is None


@pytest.mark.parametrize("N,dim,H", [(128, 64, 4), (256, 256, 4), (2, 128, 2), (512, 256, 2)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_module_fused_projection_path_matches_level_by_level_path(dtype, N, dim, H):
    """Without autograd the span-node update runs on fused projections (and, for 16-bit heads of
    32/64/128 channels, its last levels in one launch: the 256- and 512-leaf cases go through
    both kinds of level); with autograd it runs one projection and one differentiable op per
    level.  Same result, and the oracle's."""
    B = 2
    torch.manual_seed(1)
    m = sa.HierarchicalAttention(dim, H, dropout=0.0, window_size=4).to(DEV).to(dtype).eval()
    x = torch.randn(B, N, dim, device=DEV).clamp(-1, 1).to(dtype)
    y = torch.randn(B, N - 1, dim, device=DEV).clamp(-1, 1).to(dtype)
    with torch.no_grad():
        fused = m.cross_update_Y(x, y)
        again = m.cross_update_Y(x, y)      # cached stacked weights
        with torch.no_grad():
            m.Wk_y.weight.mul_(1.0)           # a write invalidates the cache, values unchanged
        third = m.cross_update_Y(x, y)
    stepwise = m.cross_update_Y(x.requires_grad_(True), y)
    assert stepwise.requires_grad and not fused.requires_grad
    assert torch.equal(fused, again) and torch.equal(fused, third)
    # measured in bf16: 2.5e-3 against the oracle, 2.0e-3 (one rounding step) between the paths;
    # bar = 2.5 x that
    tol = 1e-5 if dtype == torch.float32 else 6e-3
    assert (fused.float() - stepwise.detach().float()).abs().max() < tol
    w = {k: v.detach().double().cpu() for k, v in m.state_dict().items()}
    want = oracle.cross_update_y_ref(x.detach().double().cpu(), y.double().cpu(), w, H)
    report("module_fused_vs_stepwise %s N=%d dim=%d" % (dtype, N, dim), oracle=error_figures(fused, want),
           paths=error_figures(fused, stepwise))
    assert (fused.double().cpu() - want).abs().max() < (1e-4 if dtype == torch.float32 else 6e-3)
    m.fuse_top_levels = False
    with torch.no_grad():
        unfused_top = m.cross_update_Y(x.detach(), y)
    assert (fused.float() - unfused_top.float()).abs().max() < tol


# ---------------------------------------------------------------- the configurations of the benchmark
def _bf_check(bf, q, k, v, N, R, causal, out, dtype):
    o = oracle.topology_tables(N, causal)
    want = bf.attention(q.float().numpy(), k.float().numpy(), v.float().numpy(), o["forward_idx"],
                        o["forward_mask"] if causal else None, R)
    assert_close(out, torch.from_numpy(want), dtype, "full-size")
    return error_figures(out, torch.from_numpy(want)), torch.from_numpy(want)


def _north_star_bars(f, what, low=None):
    """The two bf16 bars, each on its own.  Max-abs <= 2e-2 holds everywhere and is asserted as
    it stands.  Max-rel <= 1e-2 (over the elements whose reference is at least 0.1 in size) is
    asserted where it holds; on N(0,1) inputs it cannot: an output near 0.1 is a sum of terms of
    size 1, each weight rounded to bf16 (relative 2^-9) as in the reference's own arithmetic, so
    absolute errors of 1..2e-3 are relative errors of 1..2e-2 there.  In that case `low` holds
    the figures of the reference's algorithm evaluated in bf16 by torch on the same inputs, and
    the kernel must be at least as close to the fp64 result as that."""
    assert f["max_abs"] <= 2e-2, "%s: max abs err %.3e" % (what, f["max_abs"])
    if low is None:
        assert f["max_rel"] <= 1e-2, "%s: max rel err %.3e" % (what, f["max_rel"])
    else:
        assert f["max_abs"] <= low["max_abs"] and f["max_rel"] <= max(1e-2, low["max_rel"]), \
            "%s: kernel %s vs the reference's algorithm in bf16 %s" % (what, f, low)


def _bf16_reference_figures(q, k, v, N, R, causal, want):
    """Error figures of the reference's algorithm evaluated in bf16 by torch on the CPU (gather,
    einsum, softmax, einsum: every stage rounds to bf16) against `want`, on the first two batch
    elements."""
    o = oracle.topology_tables(N, causal)
    low = oracle.attention_ref(q[:2], k[:2], v[:2], o["forward_idx"], o["forward_mask"] if causal else None, R)
    assert low.dtype == torch.bfloat16
    return error_figures(low, want[:2])


@pytest.mark.parametrize("causal", [True, False])
def test_cfg2_gather_full_size(causal, bf):
    B, H, N, D, R = 16, 8, 512, 64, 8
    q, k, v = make_qkv(B, N, H, D, torch.bfloat16, seed=0, scale=1.0 / 8)
    t = sa.build_tree_topology(N, causal, device=DEV)
    out = fn.attention_forward(q.to(DEV), k.to(DEV), v.to(DEV), t["forward_idx"],
                               t["forward_mask"] if causal else None, R, algo="gather")
    _bf_check(bf, q, k, v, N, R, causal, out, torch.bfloat16)


# ---------------------------------------------------------------- span attention, MFMA tile kernel
TILE_CASES = [  # B, N, H, D, R
    (2, 16, 2, 64, 1),
    (1, 32, 3, 64, 16),
    (2, 64, 8, 64, 8),
    (2, 256, 4, 64, 16),
    (1, 512, 12, 64, 20),
    (1, 128, 2, 128, 32),
    (2, 64, 2, 128, 5),
    (1, 64, 2, 64, 0),
    (2, 128, 4, 32, 8),
    (1, 64, 3, 32, 20),
    (1, 1024, 8, 32, 16),
    (1, 1024, 2, 128, 32),
    (1, 2048, 1, 64, 16),
]
# window radius above 32: four or five leaf blocks per query block with the causal mask, seven or
# nine without it
TILE_CASES_WIDE = [(2, 256, 4, 64, 48), (1, 512, 2, 64, 64), (1, 128, 2, 128, 50), (2, 256, 3, 32, 64), (1, 64, 2, 64, 33),
                   (1, 1024, 2, 64, 40), (1, 32, 2, 32, 64), (2, 512, 2, 128, 64), (1, 64, 1, 128, 33)]


@pytest.mark.parametrize("case", TILE_CASES_WIDE)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("strip", [None, "1", "2"])
def test_attention_tile_wide_window(case, dtype, strip, tile_knobs):
    """Windows of radius 33..64 stay on the tile kernel, with and without the causal mask, and the
    automatic choice is the tile kernel."""
    B, N, H, D, R = case
    if strip is not None:
        tile_knobs(int(strip), -1, -1, -1)
    q, k, v = make_qkv(B, N, H, D, dtype, seed=N + R + D)
    t = sa.build_tree_topology(N, True, device=DEV)
    o = oracle.topology_tables(N, True)
    out = fn.attention_forward(q.to(DEV), k.to(DEV), v.to(DEV), t["forward_idx"], t["forward_mask"], R, algo="tile")
    want = oracle.attention_ref(q, k, v, o["forward_idx"], o["forward_mask"], R, compute_dtype=torch.float64)
    assert_close(out, want, dtype, "tile, wide causal window")
    tn = sa.build_tree_topology(N, False, device=DEV)
    on = oracle.topology_tables(N, False)
    want = oracle.attention_ref(q, k, v, on["forward_idx"], None, R, compute_dtype=torch.float64)
    out = fn.attention_forward(q.to(DEV), k.to(DEV), v.to(DEV), tn["forward_idx"], None, R, algo="tile")
    assert_close(out, want, dtype, "tile, wide window, not causal")
    auto = fn.attention_forward(q.to(DEV), k.to(DEV), v.to(DEV), tn["forward_idx"], None, R)
    assert torch.equal(auto, out), "automatic choice, wide window, not causal"


@pytest.mark.parametrize("case", TILE_CASES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("strip", [None, "1", "2", "4", "4-same-direction", "8", "8-same-direction"])
def test_attention_tile_vs_oracle(case, dtype, causal, strip, tile_knobs):
    """Strip length forced to 1 / 2 / 4 query blocks, or to 8 (two runs of four blocks per
    wavefront, where the window radius allows it: bit-identical to strips of four), and the
    dispatcher's own choice.  Longer strips alternate their walking direction between neighbours
    unless told otherwise."""
    B, N, H, D, R = case
    alt = 1
    if strip is not None:
        alt = 0 if strip.endswith("same-direction") else 1
        tile_knobs(int(strip.split("-")[0]), -1, -1, alt)
    q, k, v = make_qkv(B, N, H, D, dtype, seed=N + R + D)
    t = sa.build_tree_topology(N, causal, device=DEV)
    o = oracle.topology_tables(N, causal)
    out = fn.attention_forward(q.to(DEV), k.to(DEV), v.to(DEV), t["forward_idx"],
                               t["forward_mask"] if causal else None, R, algo="tile")
    want = oracle.attention_ref(q, k, v, o["forward_idx"], o["forward_mask"] if causal else None, R,
                                compute_dtype=torch.float64)
    assert_close(out, want, dtype, "tile")
    if strip is not None and int(strip.split("-")[0]) > 4:
        tile_knobs(4, -1, -1, alt)
        four = fn.attention_forward(q.to(DEV), k.to(DEV), v.to(DEV), t["forward_idx"],
                                    t["forward_mask"] if causal else None, R, algo="tile")
        assert torch.equal(out, four), "two runs of four blocks against strips of four"


@pytest.mark.parametrize("case", TILE_CASES + [(1, 256, 2, 64, 48), (1, 64, 2, 32, 24), (1, 128, 2, 128, 40), (2, 512, 2, 64, 64),
                                              (1, 256, 2, 128, 64), (2, 64, 1, 128, 33)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("causal", [True, False])
def test_attention_tile_weights_vs_oracle(case, dtype, causal):
    """The tile kernel's softmax weights [B, N, H, 2R+1+L] (fp32; window slots first, then one
    per level; dead slots zero; the sibling leaf's weight split over its two slots) and its
    output, against the oracle; every row of weights sums to one."""
    B, N, H, D, R = case
    L = N.bit_length() - 1
    if 2 * R + 1 + L > 2 * D + 16:
        pytest.skip("a row of weights does not fit the wavefront's staging area")
    q, k, v = make_qkv(B, N, H, D, dtype, seed=N + R + D)
    t = sa.build_tree_topology(N, causal, device=DEV)
    o = oracle.topology_tables(N, causal)
    out, w = fn.attention_forward(q.to(DEV), k.to(DEV), v.to(DEV), t["forward_idx"],
                                  t["forward_mask"] if causal else None, R, return_weights=True, algo="tile")
    want, want_w = oracle.attention_ref(q, k, v, o["forward_idx"], o["forward_mask"] if causal else None, R,
                                        compute_dtype=torch.float64, return_weights=True)
    assert w.dtype == torch.float32 and w.shape == (B, N, H, 2 * R + 1 + L)
    assert_close(out, want, dtype, "tile output with weights")
    assert (w.double().cpu() - want_w).abs().max() < 2e-5
    assert (w.sum(-1) - 1).abs().max() < 1e-5
    assert ((want_w == 0) <= (w.cpu() == 0)).all()      # dead slots are exact zeros
    # the gather kernel's weights agree
    _, wg = fn.attention_forward(q.to(DEV), k.to(DEV), v.to(DEV), t["forward_idx"],
                                 t["forward_mask"] if causal else None, R, return_weights=True, algo="gather")
    assert (w - wg).abs().max() < 2e-5


@pytest.mark.parametrize("seed", range(40))
def test_attention_random_shapes(seed):
    """Seeded random shapes through whichever kernel the dispatcher picks, against the oracle."""
    rng = np.random.default_rng(1000 + seed)
    N = int(2 ** rng.integers(1, 10))
    D = int(rng.choice([8, 16, 20, 32, 64, 128]))
    H = int(rng.integers(1, 6))
    B = int(rng.integers(1, 3))
    R = int(rng.integers(0, 40)) if seed < 24 else int(rng.integers(0, 70))
    causal = bool(rng.integers(0, 2))
    dtype = [torch.float32, torch.bfloat16, torch.float16][int(rng.integers(0, 3))]
    q, k, v = make_qkv(B, N, H, D, dtype, seed=seed)
    t = sa.build_tree_topology(N, causal, device=DEV)
    o = oracle.topology_tables(N, causal)
    out = sa.hierarchical_attention(q.to(DEV), k.to(DEV), v.to(DEV), t["forward_idx"], t["backward_gather"],
                                    t["forward_mask"] if causal else None, R)
    want = oracle.attention_ref(q, k, v, o["forward_idx"], o["forward_mask"] if causal else None, R,
                                compute_dtype=torch.float64)
    assert_close(out, want, dtype, "B%d N%d H%d D%d R%d causal=%s %s" % (B, N, H, D, R, causal, dtype))


F32_TILE_CASES = [(1, 16, 2, 64, 3), (2, 64, 3, 64, 16), (1, 256, 4, 32, 8), (2, 128, 2, 64, 20), (1, 512, 5, 32, 32),
                  (1, 64, 2, 64, 0), (2, 1024, 8, 64, 16),
                  # head size 128: strips of one block (two where the window is causal and at most one block wide)
                  (1, 16, 2, 128, 3), (2, 256, 3, 128, 16), (1, 128, 2, 128, 32), (1, 2048, 8, 128, 16),
                  (1, 64, 1, 128, 0)]


@pytest.mark.parametrize("case", F32_TILE_CASES)
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("strip", [None, "1", "2", "4"])
def test_attention_tile_fp32_vs_oracle(case, causal, strip, tile_knobs):
    """fp32 tensors on the fp32 matrix instructions: the 1e-5 bar against the fp64 oracle."""
    B, N, H, D, R = case
    if strip is not None:
        tile_knobs(int(strip), -1, -1, -1)
    q, k, v = make_qkv(B, N, H, D, torch.float32, seed=N + R + D)
    t = sa.build_tree_topology(N, causal, device=DEV)
    o = oracle.topology_tables(N, causal)
    out = fn.attention_forward(q.to(DEV), k.to(DEV), v.to(DEV), t["forward_idx"],
                               t["forward_mask"] if causal else None, R, algo="tile")
    want = oracle.attention_ref(q, k, v, o["forward_idx"], o["forward_mask"] if causal else None, R,
                                compute_dtype=torch.float64)
    assert_close(out, want, torch.float32, "fp32 tile")
    gath = fn.attention_forward(q.to(DEV), k.to(DEV), v.to(DEV), t["forward_idx"],
                                t["forward_mask"] if causal else None, R, algo="gather")
    assert (out - gath).abs().max() < 2e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("algo", ["tile", "gather"])
def test_attention_peaked_softmax(dtype, algo):
    """Scores of a few hundred in magnitude (one key takes nearly all the weight): the running
    maximum keeps exp2 in range, masked slots stay exactly zero."""
    B, N, H, D, R = 1, 128, 2, 64, 16
    q, k, v = make_qkv(B, N, H, D, dtype, seed=11, scale=6.0)
    t = sa.build_tree_topology(N, True, device=DEV)
    o = oracle.topology_tables(N, True)
    out = fn.attention_forward(q.to(DEV), k.to(DEV), v.to(DEV), t["forward_idx"], t["forward_mask"], R, algo=algo)
    want = oracle.attention_ref(q, k, v, o["forward_idx"], o["forward_mask"], R, compute_dtype=torch.float64)
    assert torch.isfinite(out).all()
    if dtype == torch.float32:
        assert (out.double().cpu() - want).abs().max() < 2e-4      # |V| ~ 6, scores ~ 300: fp32 rounding of the scores
    else:
        # a 16-bit score of magnitude 300 carries an absolute error of order 1: compare where one key dominates
        w = oracle.attention_ref(q, k, v, o["forward_idx"], o["forward_mask"], R, compute_dtype=torch.float64,
                                 return_weights=True)[1]
        sure = w.max(dim=-1).values > 0.9999                          # [B, N, H]
        assert sure.float().mean() > 0.3
        err = (out.double().cpu() - want).abs().amax(dim=-1)
        assert (err[sure] < 0.1).all()


def test_tile_is_the_default_for_the_headline_shape():
    from sparseattention_amd import _lib
    assert _lib.lib().hsa_attn_fwd_uses_tile(2048, 4095, 8, 64, 11, 16, _lib.HSA_BF16, 1, 0) == 1
    assert _lib.lib().hsa_attn_fwd_uses_tile(2048, 4095, 8, 64, 11, 16, _lib.HSA_F32, 1, 0) == 1
    assert _lib.lib().hsa_attn_fwd_uses_tile(2048, 4095, 8, 128, 11, 16, _lib.HSA_F32, 1, 0) == 1
    assert _lib.lib().hsa_attn_fwd_uses_tile(2048, 4095, 8, 48, 11, 16, _lib.HSA_F32, 1, 0) == 0
    assert _lib.lib().hsa_attn_fwd_uses_tile(2048, 4095, 8, 128, 11, 16, _lib.HSA_F32, 1, 1) == 0
    assert _lib.lib().hsa_attn_fwd_uses_tile(2048, 4095, 8, 64, 11, 16, _lib.HSA_BF16, 0, 0) == 0


@pytest.mark.parametrize("causal", [True, False])
def test_cfg2_tile_full_size(causal, bf):
    B, H, N, D, R = 16, 8, 512, 64, 8
    q, k, v = make_qkv(B, N, H, D, torch.bfloat16, seed=0, scale=1.0 / 8)
    t = sa.build_tree_topology(N, causal, device=DEV)
    out = sa.hierarchical_attention(q.to(DEV), k.to(DEV), v.to(DEV), t["forward_idx"], t["backward_gather"],
                                    t["forward_mask"] if causal else None, R)
    f, _ = _bf_check(bf, q, k, v, N, R, causal, out, torch.bfloat16)
    report("cfg2_tile_full_size causal=%s" % causal, **f)
    _north_star_bars(f, "cfg2")


@pytest.mark.parametrize("causal", [True, False])
def test_cfg3_headline_full_size(causal, bf):
    """B8 H8 N2048 d64 bf16 R16 with the parents built by the tree kernel."""
    B, H, N, D, R = 8, 8, 2048, 64, 16
    g = torch.Generator().manual_seed(0)
    mk = lambda rows: torch.randn(B, rows, H, D, generator=g).to(torch.bfloat16)
    q, kl, vl, qp, kp, vp = mk(N), mk(N), mk(N), mk(N - 1), mk(N - 1), mk(N - 1)
    kfull = torch.empty(B, 2 * N - 1, H, D, dtype=torch.bfloat16, device=DEV)
    vfull = torch.empty_like(kfull)
    kfull[:, :N] = kl.to(DEV)
    vfull[:, :N] = vl.to(DEV)
    sa.build_tree(qp.to(DEV), kp.to(DEV), vp.to(DEV), kfull[:, :N], vfull[:, :N], out=kfull[:, N:],
                  out2=vfull[:, N:])
    tree = oracle.build_tree_ref(qp, kp, vp, kl, vl, compute_dtype=torch.float64)
    assert_close(kfull[:, N:], tree, torch.bfloat16, "tree")
    t = sa.build_tree_topology(N, causal, device=DEV)
    out = sa.hierarchical_attention(q.to(DEV), kfull, vfull, t["forward_idx"], t["backward_gather"],
                                    t["forward_mask"] if causal else None, R)
    f, want = _bf_check(bf, q, kfull.cpu(), vfull.cpu(), N, R, causal, out, torch.bfloat16)
    low = _bf16_reference_figures(q, kfull.cpu(), vfull.cpu(), N, R, causal, want)
    f_tree = error_figures(kfull[:, N:], tree)
    low_tree = error_figures(oracle.build_tree_ref(qp[:2], kp[:2], vp[:2], kl[:2], vl[:2]), tree[:2])
    report("cfg3_headline_full_size causal=%s" % causal, tree=f_tree, reference_in_bf16=low,
           reference_tree_in_bf16=low_tree, **f)
    _north_star_bars(f, "cfg3", low)
    _north_star_bars(f_tree, "cfg3 tree", low_tree)
    out_g = fn.attention_forward(q.to(DEV), kfull, vfull, t["forward_idx"],
                                 t["forward_mask"] if causal else None, R, algo="gather")
    assert (out.float() - out_g.float()).abs().max() < 2e-2


# ---------------------------------------------------------------- the language model around the ops
@pytest.mark.parametrize("activation", ["relu", "gelu"])
def test_transformer_lm_vs_oracle(activation):
    V, d, H, ff, layers, N, B, R = 211, 64, 4, 128, 2, 64, 2, 4
    torch.manual_seed(1)
    m = sa.TransformerLM(V, d, H, ff, layers, dropout=0.0, window_size=R, activation=activation, max_len=128).eval()
    tok = torch.randint(0, V, (B, N), generator=torch.Generator().manual_seed(2))
    sd = {k: v.detach().clone() for k, v in m.state_dict().items()}
    with torch.no_grad():
        got = m.to(DEV)(tok.to(DEV))
    want = oracle.lm_forward_ref(sd, tok, H, layers, R, activation)
    assert got.shape == (B, N, V)
    assert (got.double().cpu() - want).abs().max() < 2e-4


# ---------------------------------------------------------------- long-sequence stress (size-independent checks)
@pytest.mark.parametrize("shape", [(1, 16, 65536, 128, 32), (1, 1, 1 << 20, 64, 16)])
def test_long_sequence_properties(shape, tile_knobs):
    """B1 H16 N65536 D128 bf16 R32 (the long-sequence stress shape) and a 2^20-leaf tree (20 levels,
    the far tree block nearly full): too large for the gather oracle in seconds, so check what
    the mathematics fixes plus a brute-force sample of rows."""
    B, H, N, D, R = shape
    g = torch.Generator().manual_seed(0)
    q = torch.randn(B, N, H, D, generator=g).to(torch.bfloat16)
    k = torch.randn(B, 2 * N - 1, H, D, generator=g).to(torch.bfloat16)
    v = torch.randn(B, 2 * N - 1, H, D, generator=g).to(torch.bfloat16)
    t = sa.build_tree_topology(N, True, device=DEV)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    out = sa.hierarchical_attention(qd, kd, vd, t["forward_idx"], t["backward_gather"], t["forward_mask"], R)
    # causal row 0 attends only itself
    assert torch.equal(out[:, 0], vd[:, 0])
    # constant values come back unchanged whatever the weights are
    const = torch.full_like(vd, 0.5)
    oc = sa.hierarchical_attention(qd, kd, const, t["forward_idx"], t["backward_gather"], t["forward_mask"], R)
    assert (oc.float() - 0.5).abs().max() < 4e-3
    # brute force on a sample of rows spread over the sequence (first, last, block borders)
    rows = sorted(set([0, 1, 15, 16, 17, 31, 32, 33, 63, 64, 65, 1023, 1024, 4095, 4096, 32767, 32768, 65534, 65535,
                       N // 2 - 1, N // 2, N - 2, N - 1] + list(range(7, N, N // 16 + 3))))
    o = oracle.topology_tables(N, True)
    sel = torch.tensor(rows)
    outs = []
    for n in rows:
        L = o["forward_idx"].shape[1]
        live = [int(o["forward_idx"][n, l]) for l in range(L) if not o["forward_mask"][n, l]]
        keys = list(range(max(0, n - R), n + 1)) + live
        qf = q[0, n].double()                      # [H, D]
        kf = k[0, keys].double()                   # [S, H, D]
        vf = v[0, keys].double()
        s = torch.einsum("hd,shd->hs", qf, kf) / math.sqrt(D)
        p = torch.softmax(s, dim=-1)
        outs.append(torch.einsum("hs,shd->hd", p, vf))
    want = torch.stack(outs).unsqueeze(0)
    assert_close(out[:, sel], want, torch.bfloat16, "cfg5 sampled rows")
    f = error_figures(out[:, sel], want)
    assert f["max_abs"] <= 2e-2
    # the last 512 queries in full: the kernel against the fp64 oracle, beside the reference's
    # algorithm evaluated in bf16 by torch against the same
    lo, hi = N - 512, N
    blk = oracle.attention_ref(q, k, v, o["forward_idx"], o["forward_mask"], R, compute_dtype=torch.float64,
                               query_range=(lo, hi))[:, lo:hi]
    low = error_figures(oracle.attention_ref(q, k, v, o["forward_idx"], o["forward_mask"], R,
                                             query_range=(lo, hi))[:, lo:hi], blk)
    f_blk = error_figures(out[:, lo:hi], blk)
    report("long_sequence_properties %s" % (shape,), sampled_rows=f, last_512_queries=f_blk, reference_in_bf16=low)
    _north_star_bars(f_blk, "long sequence, last 512 queries", low)
    # the gather kernel agrees with the tile kernel at this size
    og = fn.attention_forward(qd, kd, vd, t["forward_idx"], t["forward_mask"], R, algo="gather")
    assert (og.float() - out.float()).abs().max() < 2e-2
    del og
    # at this size a wavefront walks two runs of four blocks: the same bits as strips of four, and
    # as strips of eight forced (whatever the automatic choice is)
    for strip in (4, 8):
        tile_knobs(strip, -1, -1, -1)
        forced = fn.attention_forward(qd, kd, vd, t["forward_idx"], t["forward_mask"], R, algo="tile")
        assert torch.equal(forced, out), "strips of %d blocks" % strip


# ---------------------------------------------------------------- backward passes
def _grad_close(got, want, dtype, what):
    got = got.detach().double().cpu()
    scale = max(1.0, float(want.abs().max()))
    atol = 2e-5 if dtype == torch.float32 else 3e-2
    err = float((got - want).abs().max())
    assert err <= atol * scale, "%s: max abs err %.3e (scale %.2f, dtype %s)" % (what, err, scale, dtype)


@pytest.mark.parametrize("case", [(2, 8, 2, 16, 2, None), (1, 64, 3, 32, 5, None), (2, 128, 4, 64, 16, None),
                                  (1, 32, 2, 20, 0, None), (1, 16, 2, 16, 20, 40), (1, 16, 2, 64, 3, None),
                                  (2, 256, 3, 64, 32, 600), (1, 1024, 2, 64, 0, None), (1, 64, 12, 64, 9, None),
                                  (1, 128, 2, 128, 32, None), (2, 32, 3, 128, 7, None), (2, 256, 4, 32, 16, None),
                                  (1, 128, 8, 32, 32, None), (1, 2048, 2, 64, 16, None), (1, 512, 3, 32, 20, None),
                                  (2, 4096, 1, 64, 8, None),
                                  # window radius 33..64: tile passes with the causal mask, gather formulation without
                                  (1, 256, 2, 64, 48, None), (2, 128, 3, 32, 64, None), (1, 128, 2, 128, 40, None),
                                  (1, 1024, 4, 64, 64, None)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("causal", [True, False])
def test_attention_backward_vs_oracle_autograd(case, dtype, causal):
    B, N, H, D, R, M = case
    q, k, v = make_qkv(B, N, H, D, dtype, seed=7 * N + R, M=M)
    go = torch.randn(B, N, H, D, generator=torch.Generator().manual_seed(3)).to(dtype)
    o = oracle.topology_tables(N, causal)
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    ref = oracle.attention_ref(qr, kr, vr, o["forward_idx"], o["forward_mask"] if causal else None, R)
    ref.backward(go.double())
    t = sa.build_tree_topology(N, causal, device=DEV)
    qd, kd, vd = (x.to(DEV).requires_grad_(True) for x in (q, k, v))
    out = sa.hierarchical_attention(qd, kd, vd, t["forward_idx"], t["backward_gather"],
                                    t["forward_mask"] if causal else None, R)
    out.backward(go.to(DEV))
    assert qd.grad.dtype == dtype and kd.grad.shape == k.shape
    _grad_close(qd.grad, qr.grad, dtype, "dQ")
    _grad_close(kd.grad, kr.grad, dtype, "dK")
    _grad_close(vd.grad, vr.grad, dtype, "dV")
    # the gather formulation explicitly (the default picks the tile kernels when eligible)
    dq, dk, dv = fn.attention_backward(go.to(DEV), qd.detach(), kd.detach(), vd.detach(), R, causal, algo="gather")
    _grad_close(dq, qr.grad, dtype, "dQ gather")
    _grad_close(dk, kr.grad, dtype, "dK gather")
    _grad_close(dv, vr.grad, dtype, "dV gather")


F32_BWD_TILE_CASES = [(1, 16, 2, 64, 3), (2, 64, 3, 64, 16), (1, 256, 4, 32, 8), (2, 128, 2, 32, 16), (1, 64, 2, 64, 0),
                      (1, 1024, 8, 64, 16), (1, 4096, 2, 32, 12), (2, 128, 1, 64, 7),
                      (2, 256, 2, 64, 22), (1, 512, 3, 64, 32), (2, 128, 2, 32, 17), (1, 64, 2, 32, 32), (1, 32, 1, 64, 25),
                      (1, 16, 1, 128, 5), (1, 64, 2, 128, 8), (2, 128, 2, 128, 16), (1, 256, 1, 128, 32), (1, 512, 2, 128, 20)]


@pytest.mark.parametrize("case", F32_BWD_TILE_CASES)
@pytest.mark.parametrize("causal", [True, False])
def test_attention_backward_tile_fp32(case, causal):
    """fp32 gradients on the fp32 matrix instructions: against autograd through the fp64 oracle and
    against the per-query gather formulation."""
    B, N, H, D, R = case
    q, k, v = make_qkv(B, N, H, D, torch.float32, seed=5 * N + R + D)
    go = torch.randn(B, N, H, D, generator=torch.Generator().manual_seed(4))
    o = oracle.topology_tables(N, causal)
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    oracle.attention_ref(qr, kr, vr, o["forward_idx"], o["forward_mask"] if causal else None, R).backward(go.double())
    args = (go.to(DEV), q.to(DEV), k.to(DEV), v.to(DEV), R, causal)
    dq, dk, dv = fn.attention_backward(*args, algo="tile")
    for name, got, want in (("dQ", dq, qr.grad), ("dK", dk, kr.grad), ("dV", dv, vr.grad)):
        _grad_close(got, want, torch.float32, name)
    gq, gk, gv = fn.attention_backward(*args, algo="gather")
    for got, other in ((dq, gq), (dk, gk), (dv, gv)):
        assert (got - other).abs().max() <= 4e-5 * max(1.0, float(other.abs().max()))


def test_attention_backward_tile_fp32_limits():
    """Shapes outside the fp32 tile backward are refused with algo="tile" and run on the gather kernels otherwise."""
    q, k, v = make_qkv(1, 64, 2, 64, torch.float32, seed=2)
    go = torch.randn(1, 64, 2, 64)
    args = (go.to(DEV), q.to(DEV), k.to(DEV), v.to(DEV), 40, True)
    with pytest.raises(_lib.HsaError):
        fn.attention_backward(*args, algo="tile")
    fn.attention_backward(*args)


@pytest.mark.parametrize("seed", range(32))
def test_attention_backward_random_shapes(seed):
    """Seeded random shapes through whichever backward kernels the dispatcher picks (tile passes with
    strips of four or of one block, fp32 tile passes, gather formulation), against autograd through
    the oracle."""
    rng = np.random.default_rng(2000 + seed)
    N = int(2 ** rng.integers(1, 10))
    D = int(rng.choice([16, 20, 32, 64, 128]))
    H = int(rng.integers(1, 5))
    B = int(rng.integers(1, 3))
    R = int(rng.integers(0, 36)) if seed < 16 else int(rng.integers(0, 70))
    causal = bool(rng.integers(0, 2))
    dtype = [torch.float32, torch.bfloat16, torch.float16][int(rng.integers(0, 3))]
    q, k, v = make_qkv(B, N, H, D, dtype, seed=seed)
    go = torch.randn(B, N, H, D, generator=torch.Generator().manual_seed(seed)).to(dtype)
    o = oracle.topology_tables(N, causal)
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    oracle.attention_ref(qr, kr, vr, o["forward_idx"], o["forward_mask"] if causal else None, R).backward(go.double())
    dq, dk, dv = fn.attention_backward(go.to(DEV), q.to(DEV), k.to(DEV), v.to(DEV), R, causal)
    what = "B%d N%d H%d D%d R%d causal=%s %s" % (B, N, H, D, R, causal, dtype)
    _grad_close(dq, qr.grad, dtype, "dQ " + what)
    _grad_close(dk, kr.grad, dtype, "dK " + what)
    _grad_close(dv, vr.grad, dtype, "dV " + what)


@pytest.mark.parametrize("seed", range(12))
def test_build_tree_random_shapes(seed, tree_knobs):
    """Seeded random shapes of the whole-tree build, one launch where possible and level passes, against
    the oracle."""
    rng = np.random.default_rng(3000 + seed)
    N = int(2 ** rng.integers(1, 12))
    D = int(rng.choice([8, 20, 32, 64, 128]))
    H = int(rng.choice([1, 2, 3, 4, 8, 16]))
    B = int(rng.integers(1, 4))
    dtype = [torch.float32, torch.bfloat16, torch.float16][int(rng.integers(0, 3))]
    g = torch.Generator().manual_seed(seed)
    qp, kp, vp = (torch.randn(B, N - 1, H, D, generator=g).to(dtype) for _ in range(3))
    kl, vl = (torch.randn(B, N, H, D, generator=g).to(dtype) for _ in range(2))
    want = oracle.build_tree_ref(qp, kp, vp, kl, vl, compute_dtype=torch.float64)
    dev = [t.to(DEV) for t in (qp, kp, vp, kl, vl)]
    for mode in (2, 0):
        tree_knobs(mode, 0 if mode else -1)
        out = sa.build_tree(*dev)
        assert_close(out, want, dtype, "B%d N%d H%d D%d %s mode %d" % (B, N, H, D, dtype, mode))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("causal", [True, False])
def test_attention_backward_wide_window_128_channels_both_formulations(dtype, causal):
    """Window radius 33..64 at 128 channels per head: the tile passes and the gather formulation
    agree, and the automatic choice is the tile passes."""
    B, N, H, D, R = 2, 512, 2, 128, 56
    q, k, v = make_qkv(B, N, H, D, dtype, seed=77)
    go = torch.randn(B, N, H, D, generator=torch.Generator().manual_seed(8)).to(dtype)
    args = (go.to(DEV), q.to(DEV), k.to(DEV), v.to(DEV), R)
    tile = fn.attention_backward(*args, causal, algo="tile")
    gath = fn.attention_backward(*args, causal, algo="gather")
    for a, b in zip(tile, gath):
        assert (a.float() - b.float()).abs().max() <= 4e-2 * max(1.0, float(b.float().abs().max()))
    auto = fn.attention_backward(*args, causal)
    for a, b in zip(auto, tile):
        assert torch.equal(a, b)


SAVED_BWD_CASES = [(2, 64, 2, 64, 16), (1, 128, 3, 64, 5), (2, 256, 4, 32, 16), (1, 512, 2, 64, 0), (2, 1024, 8, 64, 16),
                   (1, 2048, 2, 32, 9), (3, 64, 1, 32, 1), (1, 128, 1, 32, 16), (1, 4096, 3, 64, 13),
                   # window radius 17..32: two blocks of neighbours, with the causal mask only
                   (2, 64, 2, 64, 32), (1, 128, 3, 64, 17), (2, 256, 2, 32, 32), (1, 1024, 4, 64, 25), (1, 2048, 1, 32, 20),
                   # 128 channels per head: two wavefronts per head, with the causal mask only
                   (1, 64, 2, 128, 16), (2, 128, 1, 128, 32), (1, 512, 2, 128, 9), (1, 1024, 3, 128, 32), (2, 256, 2, 128, 20)]


@pytest.mark.parametrize("case", SAVED_BWD_CASES)
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_attention_backward_from_saved_forward_state(case, causal, dtype, tile_knobs):
    """The one-pass backward (hsa_attn_bwd_saved) on the forward's output and log-sum-exp
    (hsa_attn_fwd_lse): gradients against autograd through the fp64 oracle and against the
    two-pass backward, the forward's output against the plain forward (bit for bit), and the
    log-sum-exp against the oracle's logits.  One strip (no neighbours), first / last strips and
    inner strips all occur."""
    B, N, H, D, R = case
    if (R > 16 or D == 128) and not causal:
        qz = torch.zeros(B, N, H, D, dtype=dtype, device=DEV)
        assert not fn.saved_state_backward_available(qz, torch.zeros(B, 2 * N - 1, H, D, dtype=dtype, device=DEV), R, False)
        return
    q, k, v = make_qkv(B, N, H, D, dtype, seed=5 * N + R)
    go = torch.randn(B, N, H, D, generator=torch.Generator().manual_seed(N + R)).to(dtype)
    o = oracle.topology_tables(N, causal)
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    want_out, want_w = oracle.attention_ref(qr, kr, vr, o["forward_idx"], o["forward_mask"] if causal else None, R,
                                            return_weights=True)
    want_out.backward(go.double())
    qd, kd, vd, gd = q.to(DEV), k.to(DEV), v.to(DEV), go.to(DEV)
    assert fn.saved_state_backward_available(qd, kd, R, causal)
    out, lse = fn.attention_forward_lse(qd, kd, vd, R, causal)
    t = sa.build_tree_topology(N, causal, device=DEV)
    plain = fn.attention_forward(qd, kd, vd, t["forward_idx"], t["forward_mask"] if causal else None, R)
    assert torch.equal(out, plain)
    # strips of eight blocks (two runs of four per wavefront, long sequences) give the same bits
    tile_knobs(8, -1, -1, -1)
    out8, lse8 = fn.attention_forward_lse(qd, kd, vd, R, causal)
    tile_knobs(0, -1, -1, -1)
    assert torch.equal(out8, out) and torch.equal(lse8, lse)
    # lse: log2 of the sum over slots of 2^(logit * log2(e) / sqrt(D)), the sibling leaf counted twice
    L = N.bit_length() - 1
    idx = torch.as_tensor(o["forward_idx"]).long()
    n = torch.arange(N)
    sc = torch.full((B, N, H, 2 * R + 1 + L), float("-inf"), dtype=torch.float64)
    for w in range(2 * R + 1):
        j = n + w - R
        ok = (j >= 0) & (j < N) & ((j <= n) if causal else torch.ones_like(j, dtype=torch.bool))
        jj = j.clamp(0, N - 1)
        s = torch.einsum("bnhd,bnhd->bnh", q.double(), k.double()[:, jj]) / math.sqrt(D)
        sc[..., w] = torch.where(ok[None, :, None], s, torch.full_like(s, float("-inf")))
    for l in range(L):
        live = ~torch.as_tensor(o["forward_mask"])[:, l] if causal else torch.ones(N, dtype=torch.bool)
        s = torch.einsum("bnhd,bnhd->bnh", q.double(), k.double()[:, idx[:, l]]) / math.sqrt(D)
        sc[..., 2 * R + 1 + l] = torch.where(live[None, :, None], s, torch.full_like(s, float("-inf")))
    want_lse = torch.logsumexp(sc, dim=-1) / math.log(2.0)
    assert (lse.double().cpu() - want_lse).abs().max() < 2e-2
    got = fn.attention_backward_saved(gd, qd, kd, vd, out, lse, R, causal)
    two = fn.attention_backward(gd, qd, kd, vd, R, causal)
    # strips of four and of eight query blocks per wavefront (eight: one neighbour's block per 128
    # queries, the far tree block changes in the middle of the strip)
    # (16 and 32: long sequences; more tree levels are final inside the strip)
    for strip in (4, 8, 16, 32):
        assert _lib.lib().hsa_attn_bwd_saved_tune(strip) == 0
        try:
            forced = fn.attention_backward_saved(gd, qd, kd, vd, out, lse, R, causal)
        finally:
            _lib.lib().hsa_attn_bwd_saved_tune(0)
        for name, g1, ref in zip(("dQ", "dK", "dV"), forced, (qr.grad, kr.grad, vr.grad)):
            _grad_close(g1, ref, dtype, "%s one pass, strips of %d, causal=%s" % (name, strip, causal))
    for name, g1, g2, ref in zip(("dQ", "dK", "dV"), got, two, (qr.grad, kr.grad, vr.grad)):
        _grad_close(g1, ref, dtype, "%s one pass, causal=%s" % (name, causal))
        scale = max(1.0, float(ref.abs().max()))
        assert (g1.float() - g2.float()).abs().max() <= 2e-2 * scale, "%s: one pass vs two passes" % name
    # and through the autograd function: the switch forces either formulation, the default is the
    # one pass wherever it is built
    for flag, ref in ((False, two), (True, got), (None, got)):
        qa, ka, va = (x.clone().requires_grad_(True) for x in (qd, kd, vd))
        fn.one_pass_backward = flag
        try:
            sa.hierarchical_attention(qa, ka, va, t["forward_idx"], t["backward_gather"],
                                      t["forward_mask"] if causal else None, R).backward(gd)
        finally:
            fn.one_pass_backward = None
        for a, g1 in zip((qa.grad, ka.grad, va.grad), ref):
            assert torch.equal(a, g1)


def test_attention_backward_saved_state_limits():
    """Shapes the one-pass backward does not take report it instead of launching."""
    q = torch.zeros(1, 64, 2, 64, dtype=torch.bfloat16, device=DEV)
    k = torch.zeros(1, 127, 2, 64, dtype=torch.bfloat16, device=DEV)
    assert fn.saved_state_backward_available(q, k, 16)
    assert not fn.saved_state_backward_available(q, k, 17, False)               # radius above one block without the mask
    assert fn.saved_state_backward_available(q, k, 32, True) and not fn.saved_state_backward_available(q, k, 33, True)
    assert not fn.saved_state_backward_available(q.float(), k.float(), 16)      # fp32
    assert not fn.saved_state_backward_available(q[:, :32], k[:, :63], 16)      # fewer than 64 leaves
    q128, k128 = (torch.zeros(1, rows, 2, 128, dtype=torch.bfloat16, device=DEV) for rows in (64, 127))
    assert fn.saved_state_backward_available(q128, k128, 16, True)
    assert not fn.saved_state_backward_available(q128, k128, 16, False)         # 128 channels without the mask
    q256, k256 = (torch.zeros(1, rows, 2, 256, dtype=torch.bfloat16, device=DEV) for rows in (64, 127))
    assert not fn.saved_state_backward_available(q256, k256, 16, True)
    lib = _lib.lib()
    d = _lib.ptr(q)
    rc = lib.hsa_attn_bwd_saved(d, d, d, d, d, d, d, d, d, d, 1 << 20, 1, 64, 127, 2, 64, 6, 17, 0, 2, _lib.stream_of(q))
    assert rc == -95 and b"one-pass" in lib.hsa_last_error()


WIDE_BWD_CASES = [(2, 512, 4, 64, 56), (1, 256, 2, 64, 33), (2, 128, 3, 32, 64), (1, 1024, 2, 32, 40),
                  (1, 32, 2, 64, 48), (1, 64, 1, 64, 64), (1, 16, 2, 32, 50), (1, 2048, 2, 64, 64),
                  (1, 256, 2, 128, 40), (2, 128, 2, 128, 64), (1, 64, 1, 128, 33), (1, 1024, 1, 128, 56)]


@pytest.mark.parametrize("case", WIDE_BWD_CASES)
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_attention_backward_wide_window_tile_passes(case, causal, dtype):
    """Window radius 33..64, with and without the causal mask (up to nine leaf blocks per query
    block; strips of four blocks and of one; at 128 channels without the mask one block per
    wavefront): the tile passes against autograd through the oracle."""
    B, N, H, D, R = case
    q, k, v = make_qkv(B, N, H, D, dtype, seed=3 * N + R)
    go = torch.randn(B, N, H, D, generator=torch.Generator().manual_seed(R)).to(dtype)
    o = oracle.topology_tables(N, causal)
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    oracle.attention_ref(qr, kr, vr, o["forward_idx"], o["forward_mask"] if causal else None, R).backward(go.double())
    args = (go.to(DEV), q.to(DEV), k.to(DEV), v.to(DEV), R, causal)
    tile = fn.attention_backward(*args, algo="tile")
    for name, got, want in zip(("dQ", "dK", "dV"), tile, (qr.grad, kr.grad, vr.grad)):
        _grad_close(got, want, dtype, name + " wide window, causal=%s" % causal)
    auto = fn.attention_backward(*args)
    for a, b in zip(auto, tile):
        assert torch.equal(a, b), "the automatic choice is the tile passes"


@pytest.mark.parametrize("causal", [True, False])
def test_attention_backward_long_sequence_upper_levels(causal):
    """65536 leaves, 16 levels: a node near the root collects its gradient from tens of thousands
    of queries (the reference keeps a repro script for the magnitude of exactly these gradients,
    triton_kernel/reproduce_issue_v2.py).  The tile passes (per-strip partial rows summed by the
    key pass's trailing workgroups) against the per-key gather formulation, level by level."""
    B, N, H, D, R = 1, 65536, 2, 64, 16
    g = torch.Generator(device=DEV).manual_seed(9)
    mk = lambda rows: torch.randn(B, rows, H, D, generator=g, device=DEV).to(torch.bfloat16)
    q, k, v, go = mk(N), mk(2 * N - 1), mk(2 * N - 1), mk(N)
    tile = fn.attention_backward(go, q, k, v, R, causal, algo="tile")
    gath = fn.attention_backward(go, q, k, v, R, causal, algo="gather")
    off = N
    for lvl in range(1, N.bit_length()):
        rows = N >> lvl
        for a, b, name in ((tile[1], gath[1], "dK"), (tile[2], gath[2], "dV")):
            x, y = a[:, off:off + rows].float(), b[:, off:off + rows].float()
            scale = max(1.0, float(y.abs().max()))
            assert (x - y).abs().max() <= 3e-2 * scale, "%s level %d (scale %.1f)" % (name, lvl, scale)
        off += rows
    assert (tile[0].float() - gath[0].float()).abs().max() <= 3e-2 * max(1.0, float(gath[0].float().abs().max()))
    # the root row is attended by nobody
    assert not tile[1][:, 2 * N - 2].any() and not tile[2][:, 2 * N - 2].any()
    # the one-pass formulation with its automatic strip length and with strips of 16 and 32 query
    # blocks (levels up to 8 / 9 finished inside a strip, the rest from partial rows)
    out, lse = fn.attention_forward_lse(q, k, v, R, causal)
    for knob in (0, 16, 32):
        assert _lib.lib().hsa_attn_bwd_saved_tune(knob) == 0
        try:
            one = fn.attention_backward_saved(go, q, k, v, out, lse, R, causal)
        finally:
            _lib.lib().hsa_attn_bwd_saved_tune(0)
        off = N
        for lvl in range(1, N.bit_length()):
            rows = N >> lvl
            for a, b, name in ((one[1], gath[1], "dK"), (one[2], gath[2], "dV")):
                x, y = a[:, off:off + rows].float(), b[:, off:off + rows].float()
                scale = max(1.0, float(y.abs().max()))
                assert (x - y).abs().max() <= 3e-2 * scale, "one pass, knob %d: %s level %d (scale %.1f)" % (knob, name, lvl, scale)
            off += rows
        assert (one[0].float() - gath[0].float()).abs().max() <= 3e-2 * max(1.0, float(gath[0].float().abs().max()))
        assert not one[1][:, 2 * N - 2].any() and not one[2][:, 2 * N - 2].any()


def test_attention_backward_unknown_tables_need_their_gather_table():
    N = 16
    q, k, v = make_qkv(1, N, 1, 16, torch.float32, seed=1, M=40)
    idx = torch.randint(0, 40, (N, 4), dtype=torch.int32).to(DEV)
    qd = q.to(DEV).requires_grad_(True)
    out = sa.hierarchical_attention(qd, k.to(DEV), v.to(DEV), idx, None, None, 2)
    with pytest.raises(NotImplementedError):
        out.sum().backward()


@pytest.mark.parametrize("case", [(2, 32, 3, 16, 2, 70), (1, 64, 2, 64, 5, 127), (2, 16, 1, 20, 0, 31), (1, 128, 4, 32, 16, 300)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("causal", [True, False])
def test_attention_backward_from_caller_tables(case, dtype, causal):
    """Tables that are not build_tree_topology's (dead -1 slots, extra masked slots, node rows
    whose gather entry says nobody attends them, more key rows than 2N-1): the backward reads the
    caller's idx / mask / gather tables like the reference's does; against autograd through the
    fp64 oracle, directly and through the autograd function."""
    B, N, H, D, R, M = case
    L = N.bit_length() - 1
    q, k, v = make_qkv(B, N, H, D, dtype, seed=3 * N + R, M=M)
    go = torch.randn(B, N, H, D, generator=torch.Generator().manual_seed(R + 1)).to(dtype)
    o = oracle.topology_tables(N, causal)
    rng = np.random.default_rng(N + R)
    idx = np.array(o["forward_idx"], dtype=np.int32).copy()
    mask = np.array(o["forward_mask"], dtype=bool).copy() if causal else None
    gather = np.array(o["backward_gather"], dtype=np.int32).copy()
    idx[rng.random(idx.shape) < 0.15] = -1                     # dead slots
    if causal:
        mask |= rng.random(mask.shape) < 0.1                   # more masked slots
    # a few node rows nobody attends: their queries' slots die, the gather entry says -1
    for row in rng.choice(np.arange(N, 2 * N - 2), size=min(3, N - 2), replace=False):
        lvl = 1
        while row >= 2 * N - (N >> lvl):
            lvl += 1
        first = int(gather[row, 0])
        if first >= 0:
            idx[first:first + (1 << lvl), lvl] = -1
        gather[row] = -1
    if M > gather.shape[0]:
        gather = np.concatenate([gather, -np.ones((M - gather.shape[0], 3), np.int32)])
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    oracle.attention_ref(qr, kr, vr, idx, mask, R).backward(go.double())
    idx_d, gat_d = torch.from_numpy(idx).to(DEV), torch.from_numpy(gather).to(DEV)
    mask_d = torch.from_numpy(mask).to(DEV) if causal else None
    got = fn.attention_backward_tables(go.to(DEV), q.to(DEV), k.to(DEV), v.to(DEV), idx_d, mask_d, gat_d, R)
    for name, g1, ref in zip(("dQ", "dK", "dV"), got, (qr.grad, kr.grad, vr.grad)):
        _grad_close(g1, ref, dtype, "%s from the caller's tables, causal=%s" % (name, causal))
    qa, ka, va = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
    sa.hierarchical_attention(qa, ka, va, idx_d, gat_d, mask_d, R).backward(go.to(DEV))
    for a, g1 in zip((qa.grad, ka.grad, va.grad), got):
        assert torch.equal(a, g1)


@pytest.mark.parametrize("shape", [(2, 1, 1, 8), (2, 5, 3, 16), (1, 64, 8, 64), (2, 16, 4, 128), (1, 7, 2, 20)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_build_parents_backward_vs_oracle_autograd(shape, dtype):
    B, P, H, D = shape
    g = torch.Generator().manual_seed(P + D)
    qp, kp, vp = (torch.randn(B, P, H, D, generator=g).to(dtype) for _ in range(3))
    kc, vc = (torch.randn(B, 2 * P, H, D, generator=g).to(dtype) for _ in range(2))
    go = torch.randn(B, P, H, D, generator=g).to(dtype)
    refs = [t.double().requires_grad_(True) for t in (qp, kp, vp, kc, vc)]
    oracle.build_parent_nodes_ref(*refs).backward(go.double())
    devs = [t.to(DEV).requires_grad_(True) for t in (qp, kp, vp, kc, vc)]
    sa.build_parent_nodes(*devs).backward(go.to(DEV))
    for name, d, r in zip(["dQp", "dKp", "dVp", "dKc", "dVc"], devs, refs):
        _grad_close(d.grad, r.grad, dtype, name)


@pytest.mark.parametrize("N", [64, 100, 37, 3])
@pytest.mark.parametrize("C", [24, 7, 512])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_span_input_y_backward(dtype, N, C):
    B = 2
    x = torch.randn(B, N, C, generator=torch.Generator().manual_seed(0)).to(dtype)
    gy = torch.randn(B, N - bin(N).count("1"), C, generator=torch.Generator().manual_seed(1)).to(dtype)
    xr = x.double().requires_grad_(True)
    oracle.span_input_y_ref(xr).backward(gy.double())
    xd = x.to(DEV).requires_grad_(True)
    sa.generate_span_input_Y(xd).backward(gy.to(DEV))
    _grad_close(xd.grad, xr.grad, dtype, "dx")


def test_module_trains_end_to_end_like_the_oracle():
    """One backward through cross_update_Y + forward of the module: parameter and input
    gradients against autograd through the CPU oracle with the same weights."""
    B, N, dim, H, R = 2, 32, 64, 4, 3
    torch.manual_seed(0)
    m = sa.HierarchicalAttention(dim, H, dropout=0.0, window_size=R)
    x = torch.randn(B, N, dim).clamp(-1, 1)
    y = torch.randn(B, N - 1, dim).clamp(-1, 1)
    w = {k: v.detach().double().requires_grad_(True) for k, v in m.state_dict().items()}
    xr, yr = x.double().requires_grad_(True), y.double().requires_grad_(True)
    y2 = oracle.cross_update_y_ref(xr, yr, w, H)
    ref = oracle.update_x_from_y_ref(xr, y2, w, H, R, causal=True)
    ref.square().sum().backward()
    md = m.to(DEV)
    xd, yd = x.to(DEV).requires_grad_(True), y.to(DEV).requires_grad_(True)
    out = md(xd, xd, xd, y=md.cross_update_Y(xd, yd), mask=torch.ones(1, device=DEV))
    out.square().sum().backward()
    assert (out.detach().double().cpu() - ref.detach()).abs().max() < 1e-4
    _grad_close(xd.grad, xr.grad, torch.float32, "dx")
    _grad_close(yd.grad, yr.grad, torch.float32, "dy")
    for name, p in md.named_parameters():
        _grad_close(p.grad, w[name].grad, torch.float32, name)
