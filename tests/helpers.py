"""Shared helpers for the parity tests."""
import math

import numpy as np


def gemm_tol(K, a, b):
    """The parity bound of the path: 1e-4 * sqrt(K) * max|a| * max|b|."""
    return 1e-4 * math.sqrt(max(K, 1)) * float(np.max(np.abs(a))) * float(np.max(np.abs(b)))


def seq_matmul_f32(a, b):
    """C[i, j] = sum over k = 0..K-1, in that order, of separately rounded f32
    products added to an f32 accumulator that starts at +0.0 -- what an
    unblocked i-k-j loop without FMA contraction produces."""
    a = np.asarray(a, dtype=np.float32)
    b = np.asarray(b, dtype=np.float32)
    m, k = a.shape
    n = b.shape[1]
    c = np.zeros((m, n), dtype=np.float32)
    for kk in range(k):
        prod = (a[:, kk:kk + 1] * b[kk:kk + 1, :]).astype(np.float32)
        c = (c + prod).astype(np.float32)
    return c


def max_err(x, y):
    return float(np.max(np.abs(np.asarray(x, dtype=np.float64) - np.asarray(y, dtype=np.float64)))) if np.size(x) else 0.0
