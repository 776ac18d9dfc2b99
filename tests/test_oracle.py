"""Pins the CPU oracle (oracle/kcg_oracle.c).

The reference holds no numeric vectors for this path, so every oracle function
is pinned by what the mathematics fixes: closed forms exact in fp32, brute
force in float64 (independent numpy code and the committed fixtures under
tests/golden/), invariants, and special cases chosen so that a dropped term, a
wrong index, a transposed operand or a wrong accumulation order fails.
"""
import os

import numpy as np
import pytest

from conftest import rel_err

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "small_cases.npz"))


# ------------------------------------------------------------------ matmul
def test_matmul_identity_exact(oracle):
    rng = np.random.default_rng(0)
    A = rng.standard_normal((33, 33)).astype(np.float32)
    I = np.eye(33, dtype=np.float32)
    assert np.array_equal(oracle.matmul(A, I), A)
    assert np.array_equal(oracle.matmul(I, A), A)


def test_matmul_all_ones_is_K(oracle):
    for K in (1, 7, 1000, 4096):
        C = oracle.matmul(np.ones((3, K), np.float32), np.ones((K, 5), np.float32))
        assert np.array_equal(C, np.full((3, 5), K, np.float32))


def test_matmul_small_integers_exact(oracle):
    rng = np.random.default_rng(1)
    A = rng.integers(-8, 9, (19, 40)).astype(np.float32)
    B = rng.integers(-8, 9, (40, 23)).astype(np.float32)
    expect = (A.astype(np.int64) @ B.astype(np.int64)).astype(np.float32)
    assert np.array_equal(oracle.matmul(A, B), expect)
    assert np.array_equal(oracle.matmul(A, B, literal=True), expect)


def test_matmul_not_transposed(oracle):
    # A[i,k] = i, B = first row of ones: C[i,j] = i for every j.  A transposed
    # operand or swapped indices gives a different pattern.
    M, K, N = 6, 4, 5
    A = np.repeat(np.arange(M, dtype=np.float32)[:, None], K, axis=1)
    B = np.zeros((K, N), np.float32)
    B[0, :] = 1
    C = oracle.matmul(A, B)
    assert np.array_equal(C, np.repeat(np.arange(M, dtype=np.float32)[:, None], N, axis=1))
    # rank-1: C = u v^T
    u = np.arange(1, 8, dtype=np.float32)[:, None]
    v = np.arange(1, 4, dtype=np.float32)[None, :]
    assert np.array_equal(oracle.matmul(u, v), u @ v)


def test_matmul_accumulation_order_is_ascending_k(oracle):
    # fp32 addition is not associative: with a = [1e8, 1, -1e8] (b = 1)
    # ascending order gives ((0+1e8)+1)-1e8 = 0, descending gives ((0-1e8)+1)+1e8 = 0
    # too, so use four terms: [1, 1e8, -1e8, 1]: ascending ((1+1e8)-1e8)+1 = 1
    # (the first 1 is absorbed), pairwise (1+1e8)+(-1e8+1) = 0, exact sum = 2.
    A = np.array([[1.0, 1e8, -1e8, 1.0]], np.float32)
    B = np.ones((4, 1), np.float32)
    assert oracle.matmul(A, B)[0, 0] == np.float32(1.0)
    assert oracle.matmul(A, B, literal=True)[0, 0] == np.float32(1.0)


def test_matmul_mul_and_add_round_separately(oracle):
    # (1+2^-12)^2 = 1 + 2^-11 + 2^-24; the product rounds to 1 + 2^-11 in fp32.
    # acc = -(1+2^-11) first, then the product: separate roundings give exactly 0,
    # a fused multiply-add would give 2^-24.
    x = np.float32(1 + 2.0 ** -12)
    A = np.array([[-(1 + 2.0 ** -11), x]], np.float32)
    B = np.array([[1.0], [x]], np.float32)
    assert oracle.matmul(A, B)[0, 0] == np.float32(0.0)
    assert oracle.matmul(A, B, literal=True)[0, 0] == np.float32(0.0)


def test_matmul_reordered_equals_literal_bitwise(oracle):
    rng = np.random.default_rng(2)
    for (M, N, K) in [(5, 7, 3), (64, 48, 100), (33, 130, 257)]:
        A = rng.standard_normal((M, K)).astype(np.float32)
        B = rng.standard_normal((K, N)).astype(np.float32)
        assert np.array_equal(oracle.matmul(A, B), oracle.matmul(A, B, literal=True))
        assert np.array_equal(oracle.matmul_rows(A, B, 2, M - 1), oracle.matmul(A, B)[2:M - 1])


def test_matmul_golden_fp64(oracle):
    for name in ("mm_a", "mm_b", "mm_c"):
        C = oracle.matmul(GOLD[name + "_A"], GOLD[name + "_B"])
        assert max(rel_err(C, GOLD[name + "_C"])) < 5e-6


def test_matmul_row_permutation_invariance(oracle):
    rng = np.random.default_rng(3)
    A = rng.standard_normal((40, 64)).astype(np.float32)
    B = rng.standard_normal((64, 24)).astype(np.float32)
    perm = rng.permutation(40)
    assert np.array_equal(oracle.matmul(A[perm], B), oracle.matmul(A, B)[perm])


# -------------------------------------------------------------------- relu
def test_relu_exact(oracle):
    x = np.array([-3.0, -0.0, 0.0, 2.5, -np.inf, np.inf, np.nan, -1e-45, 1e-45], np.float32)
    y = oracle.relu(x)
    assert np.array_equal(y[[0, 1, 2, 3, 4, 5, 7, 8]],
                          np.array([0, 0, 0, 2.5, 0, np.inf, 0, 1e-45], np.float32))
    assert np.isnan(y[6])                       # arith.maxf propagates NaN
    assert not np.signbit(y[1])                 # maxf(+0, -0) = +0


# ----------------------------------------------------------- batched matmul
def test_batched_matmul_layouts(oracle):
    A, B, C = GOLD["bmm_A"], GOLD["bmm_B"], GOLD["bmm_C"]
    At = np.ascontiguousarray(np.swapaxes(A, -1, -2))
    Bt = np.ascontiguousarray(np.swapaxes(B, -1, -2))
    for ta, tb, a, b in [(0, 0, A, B), (0, 1, A, Bt), (1, 0, At, B), (1, 1, At, Bt)]:
        got = oracle.batched_matmul(a, ta, b, tb)
        assert got.shape == C.shape
        assert max(rel_err(got, C)) < 5e-6
    # the four layouts run the same products in the same order: bit-identical
    ref = oracle.batched_matmul(A, 0, B, 0)
    assert np.array_equal(ref, oracle.batched_matmul(At, 1, Bt, 1))


def test_batched_matmul_batches_are_independent(oracle):
    rng = np.random.default_rng(4)
    A = rng.standard_normal((3, 6, 5)).astype(np.float32)
    B = rng.standard_normal((3, 5, 4)).astype(np.float32)
    C = oracle.batched_matmul(A, 0, B, 0)
    for b in range(3):
        assert np.array_equal(C[b], oracle.matmul(A[b], B[b]))


# ----------------------------------------------------------------- softmax
def test_softmax_closed_forms(oracle):
    y = oracle.softmax(np.full((3, 8), 2.5, np.float32))
    assert np.allclose(y, 1 / 8, rtol=1e-6)
    a, b = 0.7, -1.3
    y = oracle.softmax(np.array([[a, b]], np.float32))
    assert abs(y[0, 0] - 1 / (1 + np.exp(b - a))) < 1e-6
    assert abs(y[0, 1] - 1 / (1 + np.exp(a - b))) < 1e-6


def test_softmax_rows_sum_to_one_and_shift_invariant(oracle):
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((6, 50)) * 2).astype(np.float32)
    y = oracle.softmax(x)
    assert np.allclose(y.sum(-1), 1, atol=1e-5)
    y2 = oracle.softmax(x + np.float32(3.0))
    assert max(rel_err(y2, y)) < 1e-5
    got = oracle.softmax(GOLD["sm_X"])
    assert max(rel_err(got, GOLD["sm_Y"])) < 1e-5


def test_softmax_has_no_max_shift(oracle):
    # The reference computes exp(x)/sum(exp(x)) with no max subtraction
    # (src/Frontend/Operators.cc:504-534): x = 100 overflows expf to inf -> NaN.
    with np.errstate(all="ignore"):
        y = oracle.softmax(np.array([[100.0, 0.0]], np.float32))
    assert np.isnan(y[0, 0])


# -------------------------------------------------------------------- fmha
def _qkv(rng, shape):
    return [rng.standard_normal(shape).astype(np.float32) for _ in range(3)]


def test_fmha_equals_three_operator_graph(oracle):
    # BatchedMatmul(Q,K^T) -> Softmax -> BatchedMatmul(P,V), scale 1, no mask
    rng = np.random.default_rng(6)
    Q, K, V = _qkv(rng, (2, 2, 24, 8))
    Q *= 0.5
    S = oracle.batched_matmul(Q, 0, K, 1)
    P = oracle.softmax(S)
    O3 = oracle.batched_matmul(P, 0, V, 0)
    assert np.array_equal(oracle.fmha(Q, K, V, scale=1.0, causal=False, stable=False), O3)


def test_fmha_golden_fp64(oracle):
    Q, K, V = GOLD["at_Q"], GOLD["at_K"], GOLD["at_V"]
    for stable in (False, True):
        assert max(rel_err(oracle.fmha(Q, K, V, 1.0, False, stable), GOLD["at_O_plain"])) < 2e-5
        assert max(rel_err(oracle.fmha(Q, K, V, 0.25, False, stable), GOLD["at_O_scaled"])) < 2e-5
        assert max(rel_err(oracle.fmha(Q, K, V, 0.25, True, stable), GOLD["at_O_causal"])) < 2e-5


def test_fmha_v_ones_gives_ones(oracle):
    rng = np.random.default_rng(7)
    Q, K, _ = _qkv(rng, (1, 2, 30, 16))
    O = oracle.fmha(Q, K, np.ones_like(Q), scale=0.25, causal=True)
    assert np.allclose(O, 1, atol=1e-5)


def test_fmha_k_zero_gives_means(oracle):
    rng = np.random.default_rng(8)
    Q, _, V = _qkv(rng, (1, 1, 20, 8))
    K0 = np.zeros_like(Q)
    O = oracle.fmha(Q, K0, V, scale=1.0, causal=False)
    assert max(rel_err(O, np.broadcast_to(V.mean(2, keepdims=True), V.shape))) < 1e-5
    Oc = oracle.fmha(Q, K0, V, scale=1.0, causal=True)
    prefix = np.cumsum(V.astype(np.float64), 2) / np.arange(1, 21)[None, None, :, None]
    assert max(rel_err(Oc, prefix)) < 1e-5


def test_fmha_causal_first_row_and_mask_direction(oracle):
    rng = np.random.default_rng(9)
    Q, K, V = _qkv(rng, (1, 1, 12, 8))
    O = oracle.fmha(Q, K, V, scale=0.3, causal=True)
    assert np.allclose(O[0, 0, 0], V[0, 0, 0], atol=1e-6)       # row 0 sees key 0 only
    # changing a future key must not change an earlier row
    K2, V2 = K.copy(), V.copy()
    K2[0, 0, 7:] += 5
    V2[0, 0, 7:] -= 3
    O2 = oracle.fmha(Q, K2, V2, scale=0.3, causal=True)
    assert np.array_equal(O2[0, 0, :7], O[0, 0, :7])
    assert not np.array_equal(O2[0, 0, 7:], O[0, 0, 7:])


def test_fmha_one_hot_key_selection(oracle):
    # Q = K = 30 * one-hot rows: softmax is (numerically) a selection of key i.
    S, D = 8, 8
    E = (np.eye(S, D) * 30).astype(np.float32)[None, None]
    V = np.arange(S * D, dtype=np.float32).reshape(1, 1, S, D)
    O = oracle.fmha(E, E, V, scale=1.0, causal=False, stable=True)
    assert np.allclose(O, V, atol=1e-4)


def test_fmha_stable_equals_literal_and_scale_applies_to_logits(oracle):
    rng = np.random.default_rng(10)
    Q, K, V = _qkv(rng, (1, 2, 33, 16))
    a = oracle.fmha(Q, K, V, scale=0.25, causal=False, stable=False)
    b = oracle.fmha(Q, K, V, scale=0.25, causal=False, stable=True)
    assert max(rel_err(a, b)) < 1e-5
    # scale multiplies the logits: scaling Q by 0.25 (exact in fp32) is the same
    c = oracle.fmha(Q * np.float32(0.25), K, V, scale=1.0, causal=False, stable=False)
    assert max(rel_err(a, c)) < 1e-5


def test_fmha_heads_and_batches_independent(oracle):
    rng = np.random.default_rng(11)
    Q, K, V = _qkv(rng, (2, 3, 17, 8))
    O = oracle.fmha(Q, K, V, scale=0.35, causal=True)
    perm = [2, 0, 1]
    Op = oracle.fmha(Q[:, perm], K[:, perm], V[:, perm], scale=0.35, causal=True)
    assert np.array_equal(Op, O[:, perm])
    one = oracle.fmha(Q[1:2, 1:2], K[1:2, 1:2], V[1:2, 1:2], scale=0.35, causal=True)
    assert np.array_equal(one[0, 0], O[1, 1])


def test_fmha_rows_subset(oracle):
    rng = np.random.default_rng(12)
    Q, K, V = _qkv(rng, (1, 2, 40, 8))
    full = oracle.fmha(Q, K, V, scale=0.3, causal=True)
    part = oracle.fmha(Q, K, V, scale=0.3, causal=True, rows=(10, 25))
    assert np.array_equal(part, full[:, :, 10:25])


# -------------------------------------------------------------------- bf16
def test_bf16_conversions(oracle):
    from kernelcodegen_amd import inputs
    x = np.array([1.0, 1.00390625, 1.0078125, 1.01171875, -2.5, 3.0e38, 1e-40, np.inf], np.float32)
    b = oracle.f32_to_bf16(x)
    # 1 + 2^-8 is a tie -> even (1.0); 1 + 3*2^-8 is a tie -> even (1 + 2^-6)
    assert b[0] == 0x3F80 and b[1] == 0x3F80 and b[2] == 0x3F81 and b[3] == 0x3F82
    assert np.array_equal(b, inputs.to_bf16_bits(x))
    back = oracle.bf16_to_f32(b)
    assert np.array_equal(back, inputs.bf16_bits_to_f32(b))
    assert np.array_equal(oracle.f32_to_bf16(back), b)           # idempotent
    assert np.isnan(oracle.bf16_to_f32(oracle.f32_to_bf16(np.array([np.nan], np.float32))))[0]


def test_fmha_bf16_is_fp32_algorithm_on_widened_inputs(oracle):
    from kernelcodegen_amd import inputs
    rng = np.random.default_rng(13)
    Q, K, V = [inputs.to_bf16_bits(t) for t in _qkv(rng, (1, 2, 20, 16))]
    got = oracle.fmha(Q, K, V, scale=0.25, causal=True)
    ref = oracle.fmha(inputs.bf16_bits_to_f32(Q), inputs.bf16_bits_to_f32(K),
                      inputs.bf16_bits_to_f32(V), scale=0.25, causal=True)
    assert np.array_equal(got, ref)
