"""Writes tests/golden/small_cases.npz: small inputs with fp64 expected outputs.

The reference ships no numeric vectors for this path (its tests generate CUDA
text and never compare values), so these fixtures are computed here with plain
numpy in float64 -- independently of oracle/ -- and pin the oracle itself.
Run:  python tests/golden/make_golden.py
"""
import os

import numpy as np


def softmax64(x):
    e = np.exp(x - x.max(axis=-1, keepdims=True))
    return e / e.sum(axis=-1, keepdims=True)


def main():
    rng = np.random.default_rng(20240607)
    out = {}
    # matmul: three small shapes (short, odd and long K)
    for name, (m, n, k) in {"mm_a": (64, 48, 8), "mm_b": (37, 53, 29), "mm_c": (40, 64, 160)}.items():
        A = rng.uniform(-1, 1, (m, k)).astype(np.float32)
        B = rng.uniform(-1, 1, (k, n)).astype(np.float32)
        out[name + "_A"], out[name + "_B"] = A, B
        out[name + "_C"] = A.astype(np.float64) @ B.astype(np.float64)
    # batched matmul, all four layouts
    A = rng.standard_normal((2, 3, 10, 7)).astype(np.float32)
    B = rng.standard_normal((2, 3, 7, 5)).astype(np.float32)
    out["bmm_A"], out["bmm_B"] = A, B
    out["bmm_C"] = A.astype(np.float64) @ B.astype(np.float64)
    # softmax
    X = rng.standard_normal((4, 9, 33)).astype(np.float32) * 3
    out["sm_X"] = X
    out["sm_Y"] = softmax64(X.astype(np.float64))
    # attention, with and without scale / causal mask
    Q = rng.standard_normal((2, 2, 40, 16)).astype(np.float32)
    K = rng.standard_normal((2, 2, 40, 16)).astype(np.float32)
    V = rng.standard_normal((2, 2, 40, 16)).astype(np.float32)
    out["at_Q"], out["at_K"], out["at_V"] = Q, K, V
    q64, k64, v64 = (t.astype(np.float64) for t in (Q, K, V))
    s = q64 @ np.swapaxes(k64, -1, -2)
    out["at_O_plain"] = softmax64(s) @ v64
    out["at_O_scaled"] = softmax64(s * 0.25) @ v64
    mask = np.triu(np.ones((40, 40), dtype=bool), 1)
    sc = np.where(mask, -np.inf, s * 0.25)
    out["at_O_causal"] = softmax64(sc) @ v64
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "small_cases.npz"), **out)


if __name__ == "__main__":
    main()
