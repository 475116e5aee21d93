"""The reference's operator bound for a dequant-GEMV against an independent double dot product
(tests/tensor/gemma3_metal_tests.cpp:454-470): |y - sum x*w| <= gamma / (1 - gamma) * sum|x*w| + 1e-6
with gamma = (K / 32 + 32) * eps_f32 for the decode kernels and gamma = (K + 8) * eps_f32 for the
matrix (prefill) path (:1280-1285).  The dequantised weights come from the oracle's block decode,
which is pinned bit for bit against the compiled reference."""
import numpy as np

EPS = float(np.finfo(np.float32).eps)


def dense_weight(gfo, dtype, w, K, N):
    """[N, K] float64 matrix of the canonical block stream w."""
    return gfo.dequant(dtype, w).reshape(N, K).astype(np.float64)


def exact_dot(dense, x):
    """(double dot products [rows, N], sum of absolute products [rows, N])."""
    xd = x.astype(np.float64)
    return xd @ dense.T, np.abs(xd) @ np.abs(dense).T


def operator_bound(abs_sum, K, matrix_path=False):
    gamma = ((K + 8) if matrix_path else (K // 32 + 32)) * EPS
    return gamma / (1.0 - gamma) * abs_sum + 1.0e-6


def assert_within_operator_bound(gfo, dtype, w, x, y, K, N, rows=None, matrix_path=False, dense=None):
    """y [len(rows), N] against the double dot of x[rows]; returns the worst error / bound ratio."""
    dense = dense_weight(gfo, dtype, w, K, N) if dense is None else dense
    xs = x if rows is None else x[list(rows)]
    ref, abs_sum = exact_dot(dense, xs)
    bound = operator_bound(abs_sum, K, matrix_path)
    err = np.abs(np.asarray(y, np.float64) - ref)
    worst = float((err / bound).max())
    assert worst <= 1.0, (dtype, K, N, worst)
    return worst
