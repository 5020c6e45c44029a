"""Writes tests/golden/small_case.npz: inputs and known answers of a small case of every op on
the path (N=64 leaves, 2 heads of 16 channels, radius 3, fp32), computed by the scalar
double-precision brute force oracle/hsa_oracle_bf.c, slot by slot from the definition.

These are regression vectors of this repository's own checker (the reference ships none and was
not run); the tests compare both the torch oracle and the HIP kernels with them, so a change to
either that alters results shows up against a file that does not move.

    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle.bruteforce import BruteForce  # noqa: E402


def main():
    bf = BruteForce()
    rng = np.random.default_rng(20240607)
    B, N, H, D, R = 1, 64, 2, 16, 3
    M = 2 * N - 1
    q = rng.standard_normal((B, N, H, D)).astype(np.float32)
    k = rng.standard_normal((B, M, H, D)).astype(np.float32)
    v = rng.standard_normal((B, M, H, D)).astype(np.float32)
    out = {"q": q, "k": k, "v": v, "radius": np.int32(R)}
    for causal in (True, False):
        idx, mask, gather = bf.topology(N, causal)
        tag = "causal" if causal else "full"
        out["idx_" + tag], out["mask_" + tag], out["gather_" + tag] = idx, mask, gather
        o, w = bf.attention(q, k, v, idx, mask if causal else None, R, want_weights=True)
        out["attn_out_" + tag], out["attn_weights_" + tag] = o.astype(np.float32), w.astype(np.float32)
    P = 8
    qp, kp, vp = (rng.standard_normal((B, P, H, D)).astype(np.float32) for _ in range(3))
    kc, vc = (rng.standard_normal((B, 2 * P, H, D)).astype(np.float32) for _ in range(2))
    po, pw = bf.build_parents(qp, kp, vp, kc, vc, want_weights=True)
    out.update(qp=qp, kp=kp, vp=vp, kc=kc, vc=vc, parents_out=po.astype(np.float32),
               parents_weights=pw.astype(np.float32))
    path = os.path.join(HERE, "small_case.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
