"""Shared helpers for the GPU parity tests."""
import numpy as np


def gemm_tolerance(K):
    """Max relative error allowed by the acceptance criterion: 1e-4 up to K = 4096, growing with
    sqrt(K / 4096) above."""
    return 1e-4 * max(1.0, float(np.sqrt(K / 4096.0)))


def gemm_errors(C, Cref, Cabs):
    """(i) max|C - Cref| / max|Cref| and (ii) max over entries of |C - Cref| / sum_k |a||b|."""
    C = np.asarray(C, np.float64)
    diff = np.abs(C - Cref)
    e1 = diff.max() / max(np.abs(Cref).max(), 1e-300)
    e2 = (diff / np.maximum(Cabs, 1e-300)).max()
    return float(e1), float(e2)


def cfg2_tensor(rng, rows=128, cols=40000):
    """fp32 N(0, 0.02^2) with 1 % of the entries replaced by N(0, 0.5^2) outliers."""
    x = rng.normal(0.0, 0.02, rows * cols).astype(np.float32)
    k = (rows * cols) // 100
    idx = rng.choice(rows * cols, k, replace=False)
    x[idx] = rng.normal(0.0, 0.5, k).astype(np.float32)
    return x.reshape(rows, cols)
