"""ctypes binding of the brute-force C oracle (oracle/hsa_oracle_bf.c).

TEST INFRASTRUCTURE ONLY.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libhsa_oracle_bf.so")


def build_bruteforce(force: bool = False) -> str:
    src = os.path.join(_HERE, "hsa_oracle_bf.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["gcc", "-O2", "-fopenmp", "-shared", "-fPIC", "-o", _SO, src, "-lm"])
    return _SO


def _f32(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32))


class BruteForce:
    """Scalar double-precision loops; inputs are converted to contiguous fp32."""

    def __init__(self):
        self.lib = ctypes.CDLL(build_bruteforce())

    @staticmethod
    def _p(a):
        return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None

    def attention(self, Q, K, V, idx, mask, R, want_weights=False):
        Q, K, V = _f32(Q), _f32(K), _f32(V)
        B, N, H, D = Q.shape
        M = K.shape[1]
        idx = np.ascontiguousarray(np.asarray(idx, dtype=np.int32))
        L = idx.shape[1]
        m8 = None if mask is None else np.ascontiguousarray(np.asarray(mask).astype(np.uint8))
        out = np.empty_like(Q)
        w = np.empty((B, N, H, 2 * R + 1 + L), dtype=np.float32) if want_weights else None
        self.lib.hsa_oracle_attention(self._p(Q), self._p(K), self._p(V), self._p(idx), self._p(m8),
                                      self._p(out), self._p(w), B, N, M, H, D, L, int(R))
        return (out, w) if want_weights else out

    def build_parents(self, qp, kp, vp, kc, vc, want_weights=False):
        qp, kp, vp, kc, vc = map(_f32, (qp, kp, vp, kc, vc))
        B, P, H, D = qp.shape
        assert kc.shape[1] == 2 * P
        out = np.empty_like(qp)
        w = np.empty((B, P, H, 3), dtype=np.float32) if want_weights else None
        self.lib.hsa_oracle_build_parents(self._p(qp), self._p(kp), self._p(vp), self._p(kc), self._p(vc),
                                          self._p(out), self._p(w), B, P, H, D)
        return (out, w) if want_weights else out

    def topology(self, N, causal):
        L = int(N).bit_length() - 1
        idx = np.empty((N, L), dtype=np.int32)
        mask = np.empty((N, L), dtype=np.uint8)
        gather = np.empty((2 * N - 1, 3), dtype=np.int32)
        self.lib.hsa_oracle_topology(int(N), int(bool(causal)), self._p(idx), self._p(mask), self._p(gather))
        return idx, mask.astype(bool), gather
