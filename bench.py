#!/usr/bin/env python3
"""Benchmark of the hierarchical sparse attention forward path on one MI355X.

A step = one pass of the hot path over one batch of synthetic input resident in HBM:
the bottom-up tree build (every BuildParentNodes level) that produces the node rows of
K_full / V_full, followed by the span attention forward.  Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg3|cfg2|cfg5]
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

WORKLOADS = {
    # name: (B, H, N, D, R, input scale, description)
    "cfg2": (16, 8, 512, 64, 8, 1.0 / 8, "B16 H8 N512 d64 bf16 SWA8 causal"),
    "cfg3": (8, 8, 2048, 64, 16, 1.0, "B8 H8 N2048 d64 bf16 SWA16 causal, parents built by the tree kernel"),
    "cfg5": (1, 16, 65536, 128, 32, 1.0, "B1 H16 N65536 d128 bf16 SWA32 causal"),
}
HBM_PEAK_GBS = 8000.0


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=300)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--workload", default="cfg3", choices=sorted(WORKLOADS) + ["cfg4"])
    ap.add_argument("--noncausal", action="store_true")
    ap.add_argument("--seq-len", type=int, default=0, help="override the workload's N (a power of two)")
    ap.add_argument("--attention-only", action="store_true",
                    help="a step is the span attention alone, on span nodes drawn i.i.d. like the leaves "
                         "(isolates the attention kernel; the tree build is not run)")
    ap.add_argument("--sets", type=int, default=0, help="buffer sets to rotate through (0 = enough to exceed 512 MB)")
    ap.add_argument("--streams", type=int, default=2,
                    help="HIP streams the steps alternate between (each step is an independent batch)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=15.0)
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch a plain 64 MiB -> 64 MiB copy kernel 10 times (reference for HBM counters)")
    return ap.parse_args()


def cpu_baseline(B, H, N, D, R, causal, scale, budget_s):
    """Times the CPU restatement of the reference's PyTorch algorithm (tree build level by
    level + gather/einsum span attention) on this host's cores, bf16 tensors like the GPU run."""
    import torch
    import oracle
    cores = os.cpu_count() or 1
    cores = min(cores, 16) if os.environ.get("OMP_NUM_THREADS") is None else int(os.environ["OMP_NUM_THREADS"])
    torch.set_num_threads(cores)
    g = torch.Generator().manual_seed(0)
    bs = min(B, 2)   # bounded sample: a slice of the batch, same N/H/D/R
    mk = lambda rows: (torch.randn(bs, rows, H, D, generator=g) * scale).to(torch.bfloat16)
    q, kl, vl, qp, kp, vp = mk(N), mk(N), mk(N), mk(N - 1), mk(N - 1), mk(N - 1)
    t = oracle.topology_tables(N, causal)
    m = t["forward_mask"] if causal else None

    def one():
        tree = oracle.build_tree_ref(qp, kp, vp, kl, vl)
        kf = torch.cat([kl, tree], 1)
        vf = torch.cat([vl, tree], 1)
        return oracle.attention_ref(q, kf, vf, t["forward_idx"], m, R)

    one()
    times, t_end = [], time.perf_counter() + budget_s
    while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 50):
        t0 = time.perf_counter()
        one()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    res = {"value": bs * N * H / med, "unit": "head-queries/s", "cores": cores, "kind": "port",
           "sample": "%d of %d batches of the same workload (bf16, torch CPU, %d threads), median of %d passes"
                     % (bs, B, cores, len(times))}
    res["cfg1_fp32"] = cpu_plumbing_case(oracle, cores)
    return res


def cpu_plumbing_case(oracle, cores):
    """The CPU-runnable configuration (B2 H4 N256 head 32, fp32, radius 8, causal and not): the CPU
    restatement timed in full and compared with the GPU kernel on the same seeded inputs."""
    import torch
    from sparseattention_amd.ops import functional as fn
    import sparseattention_amd as sa
    B, H, N, D, R = 2, 4, 256, 32, 8
    g = torch.Generator().manual_seed(0)
    q = torch.randn(B, N, H, D, generator=g)
    k = torch.randn(B, 2 * N - 1, H, D, generator=g)
    v = torch.randn(B, 2 * N - 1, H, D, generator=g)
    out = {"B": B, "H": H, "N": N, "D": D, "window_radius": R, "cores": cores}
    for causal in (True, False):
        t = oracle.topology_tables(N, causal)
        m = t["forward_mask"] if causal else None
        ts = []
        for _ in range(7):
            t0 = time.perf_counter()
            want = oracle.attention_ref(q, k, v, t["forward_idx"], m, R)
            ts.append(time.perf_counter() - t0)
        ts = sorted(ts[2:])  # two warm-ups, median of five
        td = sa.build_tree_topology(N, causal, device="cuda:0")
        got = fn.attention_forward(q.cuda(), k.cuda(), v.cuda(), td["forward_idx"],
                                   td["forward_mask"] if causal else None, R)
        tag = "causal" if causal else "noncausal"
        out[tag + "_cpu_head_queries_per_s"] = B * N * H / ts[len(ts) // 2]
        out[tag + "_gpu_vs_cpu_max_abs_err"] = (got.cpu() - want).abs().max().item()
    return out


def lm_forward_bench(args):
    """cfg4: forward of the 6-layer decoder LM (d_model 512, 8 heads, FFN 2048 GELU, vocab 50257,
    bf16, B=8, N=4096, window 16, random weights, token ids uniform over the vocabulary)."""
    import torch
    import sparseattention_amd as sa
    from sparseattention_amd.ops import functional as fn
    from sparseattention_amd.modules import attention as attn_mod

    dev = torch.device("cuda:0")
    B, N, V, d, H, ff, layers, R = 8, 4096, 50257, 512, 8, 2048, 6, 16
    torch.manual_seed(0)
    model = sa.TransformerLM(V, d, H, ff, layers, dropout=0.0, window_size=R, activation="gelu", max_len=N)
    model = model.to(dev).to(torch.bfloat16).eval()
    tok = torch.randint(0, V, (B, N), generator=torch.Generator().manual_seed(0)).to(dev)
    K = min(args.steps, 20)
    W = max(10, min(args.warmup, 20))  # the first forwards also grow the allocator's pools
    with torch.no_grad():
        for _ in range(W):
            model(tok)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(K):
            model(tok)
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / K
        # time share of the tree side (cross_update_Y: projections + one kernel per level) and of
        # the span attention op: the same forward with an event pair around each call
        spans = {"cross_update_Y": [], "hierarchical_attention": []}
        cls = attn_mod.HierarchicalAttention
        orig_c, orig_h = cls.cross_update_Y, attn_mod.hierarchical_attention

        def timed(name, f):
            def g(*a, **k):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                r = f(*a, **k)
                e1.record()
                spans[name].append((e0, e1))
                return r
            return g

        cls.cross_update_Y = timed("cross_update_Y", orig_c)
        attn_mod.hierarchical_attention = timed("hierarchical_attention", orig_h)
        model(tok)
        torch.cuda.synchronize()
        cls.cross_update_Y, attn_mod.hierarchical_attention = orig_c, orig_h

        # the same forward captured once into a HIP graph and replayed (no host work per launch);
        # a replay must reproduce the eager logits bit for bit, else the figure is not reported
        graph_ms = None
        eager = model(tok)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            model(tok)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            captured = model(tok)
        graph.replay()
        torch.cuda.synchronize()
        if torch.equal(captured, eager):
            t0 = time.perf_counter()
            for _ in range(K):
                graph.replay()
            torch.cuda.synchronize()
            graph_ms = (time.perf_counter() - t0) * 1e3 / K
            if not torch.equal(captured, eager):
                graph_ms = None
    share = {k: sum(a.elapsed_time(b) for a, b in v) for k, v in spans.items()}
    print(json.dumps({
        "metric": "LM forward tokens/sec, 6L d512 h8 ffn2048 GELU vocab50257 bf16 B8 N4096 SWA16",
        "value": B * N / (ms * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "cfg4: decoder LM forward, random init, eval mode"},
        "detail": {"ms_in_cross_update_Y_event_pairs": share["cross_update_Y"],
                   "ms_in_hierarchical_attention_event_pairs": share["hierarchical_attention"],
                   "hip_graph_replay_ms_per_forward": graph_ms,
                   "calls_cross_update_Y": len(spans["cross_update_Y"]),
                   "calls_hierarchical_attention": len(spans["hierarchical_attention"])}}))


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU only: this build has no multi-GPU path (every (batch, head) is "
              "independent, so the path would shard over batch or heads without any exchange). "
              "Re-run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    import torch
    from sparseattention_amd import _lib
    import sparseattention_amd as sa

    if args.workload == "cfg4":
        return lm_forward_bench(args)
    B, H, N, D, R, scale, desc = WORKLOADS[args.workload]
    if args.seq_len:
        assert args.seq_len >= 64 and args.seq_len & (args.seq_len - 1) == 0, "--seq-len must be a power of two >= 64"
        desc = desc.replace("N%d" % N, "N%d" % args.seq_len)
        N = args.seq_len
    causal = not args.noncausal
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    lib = _lib.lib()
    L = N.bit_length() - 1
    M = 2 * N - 1
    e = 2
    set_bytes = e * B * H * D * (N + 2 * M + N + 3 * (N - 1))
    nsets = args.sets or max(3, -(-512 * 2**20 // set_bytes))

    stream = torch.cuda.current_stream(dev)
    st = ctypes.c_void_p(stream.cuda_stream)
    # Steps are independent batches: they alternate between `--streams` HIP streams (default
    # priority), so one step's short-of-work kernels (the top of the tree runs on 64 of 256 CUs)
    # overlap the next step's streaming kernels.  A buffer set always goes to the same stream, so
    # two steps that touch the same buffers are ordered.
    nstreams = max(1, args.streams)
    while nsets % nstreams:
        nsets += 1
    side = [torch.cuda.Stream(device=dev) for _ in range(nstreams)] if nstreams > 1 else [stream]
    side_st = [ctypes.c_void_p(x.cuda_stream) for x in side]
    g = torch.Generator().manual_seed(0)
    sets = []
    for _ in range(nsets):
        mk = lambda rows: (torch.randn(B, rows, H, D, generator=g) * scale).to(torch.bfloat16).to(dev)
        s = {"q": mk(N), "qp": mk(N - 1), "kp": mk(N - 1), "vp": mk(N - 1),
             "kfull": torch.empty(B, M, H, D, dtype=torch.bfloat16, device=dev),
             "vfull": torch.empty(B, M, H, D, dtype=torch.bfloat16, device=dev),
             "out": torch.empty(B, N, H, D, dtype=torch.bfloat16, device=dev)}
        s["kfull"][:, :N] = mk(N)
        s["vfull"][:, :N] = mk(N)
        sets.append(s)
    torch.cuda.synchronize()  # the inputs were written on the current stream

    P = lambda t: ctypes.c_void_p(t.data_ptr())
    node_off = N * H * D * e
    full_bs = M * H * D

    def tree_args(s, st):
        return (P(s["qp"]), P(s["kp"]), P(s["vp"]), P(s["kfull"]), P(s["vfull"]),
                ctypes.c_void_p(s["kfull"].data_ptr() + node_off), ctypes.c_void_p(s["vfull"].data_ptr() + node_off),
                B, N, H, D, 0, 0, 0, full_bs, full_bs, full_bs, full_bs, _lib.HSA_BF16, st)

    def attn_args(s, st):
        return (P(s["q"]), P(s["kfull"]), P(s["vfull"]), None, None, P(s["out"]), None,
                B, N, M, H, D, L, R, int(causal), _lib.HSA_BF16, _lib.ATTN_AUTO, st)

    targs = [tree_args(s, st) for s in sets]          # everything on the current stream
    aargs = [attn_args(s, st) for s in sets]
    targs_p = [tree_args(s, side_st[i % nstreams]) for i, s in enumerate(sets)]   # set i on stream i % nstreams
    aargs_p = [attn_args(s, side_st[i % nstreams]) for i, s in enumerate(sets)]
    assert lib.hsa_attn_fwd_uses_tile(N, M, H, D, L, R, _lib.HSA_BF16, 1, 0) == 1

    # HIP events whose timestamps are the attention kernel's own begin and end (attached to the
    # dispatch by hsa_attn_fwd_timed), one pair per step
    hip = ctypes.CDLL("libamdhip64.so")
    hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
    hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]

    def new_event():
        ev = ctypes.c_void_p()
        assert hip.hipEventCreate(ctypes.byref(ev)) == 0
        return ev

    def elapsed_ms(a, b):
        ms = ctypes.c_float()
        assert hip.hipEventElapsedTime(ctypes.byref(ms), a, b) == 0
        return ms.value

    kev = [(new_event(), new_event()) for _ in range(args.steps)]

    if args.attention_only:
        for s_ in sets:
            s_["kfull"][:, N:] = (torch.randn(B, N - 1, H, D, generator=g) * scale).to(torch.bfloat16).to(dev)
            s_["vfull"][:, N:] = (torch.randn(B, N - 1, H, D, generator=g) * scale).to(torch.bfloat16).to(dev)
        torch.cuda.synchronize()
    tree_fwd = (lambda *a: 0) if args.attention_only else lib.hsa_build_tree_fwd

    def step(i, ev=None):
        rc = tree_fwd(*targs[i % nsets])
        if ev is None:
            rc |= lib.hsa_attn_fwd(*aargs[i % nsets])
        else:
            rc |= lib.hsa_attn_fwd_timed(*aargs[i % nsets], ev[0], ev[1])
        return rc

    def step_p(i):
        rc = tree_fwd(*targs_p[i % nsets])
        rc |= lib.hsa_attn_fwd(*aargs_p[i % nsets])
        return rc

    for i in range(args.warmup):
        assert step_p(i) == 0, lib.hsa_last_error()
    torch.cuda.synchronize()

    # --- timed region: exactly K steps between two synchronisations -----------------------
    K = args.steps
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    rc = 0
    for i in range(K):
        rc |= step_p(i)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    assert rc == 0, lib.hsa_last_error()
    ms_per_step = (t1 - t0) * 1e3 / K

    # --- the same K steps one after the other on a single stream (the latency of a step) ----
    for i in range(min(args.warmup, 10)):
        rc |= step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(K):
        rc |= step(i)
    torch.cuda.synchronize()
    serial_ms_per_step = (time.perf_counter() - t0) * 1e3 / K
    assert rc == 0, lib.hsa_last_error()

    # --- duration of the dominant kernel: the same K steps once more, every attention dispatch
    #     carrying its own pair of HIP events (kept out of the region above because an
    #     event-carrying dispatch costs the step about 3 us of completion handling) ---------
    for i in range(K):
        rc |= step(i, kev[i])
    torch.cuda.synchronize()
    assert rc == 0, lib.hsa_last_error()
    attn_kernel_ms = sorted(elapsed_ms(a, b) for a, b in kev)
    attn_avg_ms = sum(attn_kernel_ms) / K

    # --- K launches of one entry point between one pair of HIP events on the launch stream
    #     (same buffers, same rotation): kernel durations plus the gaps between launches ------
    def launches_ms(fn, arglist):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for i in range(K):
            fn(*arglist[i % nsets])
        e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / K

    attn_b2b_ms = launches_ms(lib.hsa_attn_fwd, aargs)
    tree_b2b_ms = launches_ms(lib.hsa_build_tree_fwd, targs)

    # --- backward of the span attention (next-row kernel), same rotation of inputs ----------------
    gq = torch.randn(B, N, H, D, device=dev).to(torch.bfloat16)
    dq_, dk_, dv_ = torch.empty_like(gq), torch.empty_like(sets[0]["kfull"]), torch.empty_like(sets[0]["kfull"])
    wsb = int(lib.hsa_attn_bwd_workspace_bytes(B, N, M, H, D, L, R, _lib.HSA_BF16, _lib.ATTN_AUTO))
    wsp = torch.empty(max(wsb, 4) // 4 + 1, device=dev, dtype=torch.float32)
    bargs = [(P(s["q"]), P(s["kfull"]), P(s["vfull"]), P(gq), P(dq_), P(dk_), P(dv_), P(wsp), wsp.numel() * 4,
              B, N, M, H, D, L, R, int(causal), _lib.HSA_BF16, _lib.ATTN_AUTO, st) for s in sets]
    for i in range(3):
        assert lib.hsa_attn_bwd(*bargs[i % nsets]) == 0, lib.hsa_last_error()
    attn_bwd_ms = launches_ms(lib.hsa_attn_bwd, bargs)

    # --- the same K steps with an event pair around every attention launch (each pair adds
    #     ~5 us of idle time around the kernel, so this is reported as detail only) ----------
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(K)]
    torch.cuda.synchronize()
    for i in range(K):
        a = i % nsets
        tree_fwd(*targs[a])
        ev[i][0].record(stream)
        lib.hsa_attn_fwd(*aargs[a])
        ev[i][1].record(stream)
    torch.cuda.synchronize()
    attn_ms = sorted(a.elapsed_time(b) for a, b in ev)
    attn_instep_avg_ms = sum(attn_ms) / K
    attn_instep_med_ms = attn_ms[K // 2]

    if args.calibrate_copy:
        n = 64 * 2**20 // 2
        src = [torch.randn(n, device=dev).to(torch.bfloat16) for _ in range(5)]
        dst = [torch.empty(n, device=dev, dtype=torch.bfloat16) for _ in range(5)]
        for i in range(10):
            dst[i % 5].copy_(src[i % 5])
        torch.cuda.synchronize()

    # HBM bytes per launch of the attention kernel as counted by rocprofv3 --pmc FETCH_SIZE /
    # WRITE_SIZE (scaled by a plain copy of known size); recorded under profiles/
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "attn_tile_%s_traffic.json" % args.workload)
    if os.path.exists(tpath):
        rec = json.load(open(tpath))
        if rec.get("causal") == causal and not args.seq_len:
            traffic = rec["traffic_bytes_per_launch"]

    head_queries = B * N * H
    attn_bytes = e * B * H * D * (N + 2 * M + N)             # Q + K_full + V_full + Out
    tree_bytes = e * B * H * D * (3 * (N - 1) + 2 * N + 2 * (N - 1))  # Qp,Kp,Vp + leaves + two copies out
    achieved = attn_bytes / (attn_avg_ms * 1e-3) / 1e9
    result = {
        "metric": "attn fwd queries/sec + % HBM roofline, B8 H8 N2048 d64 bf16 SWA16",
        "value": head_queries / (ms_per_step * 1e-3),
        "unit": "head-queries/s",
        "n_gpus": 1, "steps": K, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "%s: %s; step = tree build + span attention forward on one batch; independent batches alternate between %d HIP streams" % (args.workload, desc, nstreams),
                   "B": B, "H": H, "N": N, "D": D, "window_radius": R, "causal": causal,
                   "buffer_sets_rotated": nsets, "bytes_per_set": set_bytes, "streams": nstreams},
        "roofline": {"bound": "hbm", "kernel": "attn_tile_kernel (span attention forward)",
                     "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": traffic,
                     "algorithmic_bytes_per_launch": attn_bytes, "avg_launch_ms": attn_avg_ms,
                     "median_launch_ms": attn_kernel_ms[K // 2], "min_launch_ms": attn_kernel_ms[0],
                     "timing": "HIP events attached to each attention dispatch (kernel begin/end) over a repeat of the K timed steps"},
        "detail": {"single_stream_ms_per_step": serial_ms_per_step,
                   "single_stream_head_queries_per_s": head_queries / (serial_ms_per_step * 1e-3),
                   "attn_only_head_queries_per_s": head_queries / (attn_avg_ms * 1e-3),
                   "attn_back_to_back_ms_incl_launch_gaps": attn_b2b_ms,
                   "tree_build_avg_launch_ms": tree_b2b_ms,
                   "tree_algorithmic_bytes": tree_bytes,
                   "tree_GBps": tree_bytes / (tree_b2b_ms * 1e-3) / 1e9,
                   "attn_backward_avg_ms": attn_bwd_ms,
                   "attn_backward_algorithmic_bytes": e * B * H * D * (2 * N + 2 * M + N + 2 * M),
                   "attn_ms_in_step_event_pair_avg": attn_instep_avg_ms,
                   "attn_ms_in_step_event_pair_median": attn_instep_med_ms},
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(B, H, N, D, R, causal, scale, args.cpu_seconds)
    if args.attention_only:
        result["config"]["workload"] = result["config"]["workload"].replace(
            "step = tree build + span attention forward", "step = span attention forward alone (i.i.d. span nodes)")
    if args.workload != "cfg3" or not causal or args.seq_len or args.attention_only:
        result["metric"] = "attn fwd queries/sec + % HBM roofline, " + desc
    print(json.dumps(result))


if __name__ == "__main__":
    main()
