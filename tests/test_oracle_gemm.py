"""Pins the GEMM oracle (oracle/gemm_oracle.py + gemm_oracle.c) without any reference vectors --
the reference holds none for this path -- by what the mathematics fixes: exact integer cases,
closed forms, algebraic identities that a transposed operand, a dropped k term or a wrong stride
would break, and mutual agreement of four independent routines (numpy float32, numpy float64,
plain-C k-ordered fp32, plain-C float64, plain-C dot products, Python big integers)."""

import numpy as np
import pytest

from oracle import gemm_oracle as go


@pytest.fixture(scope="module", autouse=True)
def _built():
    go.build()


def rand(shape, seed):
    return np.random.default_rng(seed).uniform(-1, 1, shape).astype(np.float32)


@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (3, 5, 7), (8, 8, 8), (13, 2, 31), (2, 17, 1)])
def test_exact_integer_cases_match_bigint_arithmetic(M, N, K):
    A, B = go.make_inputs(M, N, K, seed=M * 100 + N * 10 + K, distribution="integer")
    exact = np.array(go.gemm_exact(A, B), dtype=np.float64)
    for routine in (go.gemm_f32, go.gemm_f64, go.c_gemm_f32, go.c_gemm_f64, go.c_gemm_naive):
        assert np.array_equal(np.asarray(routine(A, B), dtype=np.float64), exact), routine.__name__


def test_non_square_operands_are_not_transposed():
    # A = e_i e_j^T picks row j of B into row i of C; any transposition lands elsewhere.
    M, N, K = 4, 6, 5
    B = np.arange(K * N, dtype=np.float32).reshape(K, N)
    for i in range(M):
        for j in range(K):
            A = np.zeros((M, K), np.float32)
            A[i, j] = 1
            for routine in (go.gemm_f32, go.c_gemm_f32, go.c_gemm_f64, go.c_gemm_naive):
                C = np.asarray(routine(A, B))
                expect = np.zeros((M, N))
                expect[i] = B[j]
                assert np.array_equal(C, expect), (routine.__name__, i, j)


def test_closed_forms():
    n = 37
    B = rand((n, 23), 1)
    eye = np.eye(n, dtype=np.float32)
    assert np.array_equal(go.c_gemm_f32(eye, B), B)
    assert np.array_equal(go.c_gemm_naive(eye, B), B)
    assert np.array_equal(go.c_gemm_f64(eye, B), B.astype(np.float64))
    ones = go.c_gemm_f32(np.ones((9, 300), np.float32), np.ones((300, 11), np.float32))
    assert np.all(ones == 300.0)
    # rank-1: (u 1^T)(1 v^T) = K u v^T with u, v small integers -> exact
    u = np.arange(1, 8, dtype=np.float32)[:, None]
    v = np.arange(1, 6, dtype=np.float32)[None, :]
    K = 50
    C = go.c_gemm_f32(np.repeat(u, K, axis=1), np.repeat(v, K, axis=0))
    assert np.array_equal(C, K * (u @ v))


def test_transpose_identity_and_linearity():
    A, B = rand((19, 33), 2), rand((33, 27), 3)
    C = go.c_gemm_f64(A, B)
    Ct = go.c_gemm_f64(np.ascontiguousarray(B.T), np.ascontiguousarray(A.T))
    assert np.allclose(C, Ct.T, rtol=0, atol=1e-12)
    A2 = rand((19, 33), 4)
    lhs = go.c_gemm_f64((A + A2).astype(np.float32), B)
    # (A + A2) is rounded to fp32 first, so compare against the same rounded operand
    rhs = go.gemm_f64((A + A2).astype(np.float32), B)
    assert np.allclose(lhs, rhs, rtol=0, atol=1e-12)
    assert np.allclose(go.c_gemm_f64(A, B) + go.c_gemm_f64(A2, B),
                       go.gemm_f64(A.astype(np.float64) + A2.astype(np.float64), B), atol=1e-12)


def test_all_routines_agree_on_random_input():
    A, B = go.make_inputs(70, 50, 129, seed=5)
    C64 = go.gemm_f64(A, B)
    assert np.allclose(go.c_gemm_f64(A, B), C64, rtol=0, atol=1e-12)
    bound = 1e-4 * np.sqrt(129)
    for routine in (go.gemm_f32, go.c_gemm_f32, go.c_gemm_naive):
        assert np.max(np.abs(routine(A, B) - C64)) < bound * 0.1
    # the naive routine rounds the float64 dot product once: it is the correctly rounded answer
    assert np.array_equal(go.c_gemm_naive(A, B), C64.astype(np.float32))


def test_leading_dimensions_and_accumulate():
    big_a, big_b = rand((10, 40), 6), rand((40, 30), 7)
    A, B = big_a[:, :17], big_b[:17, :21]          # views with ld > width
    assert np.array_equal(go.c_gemm_f32(A, B), go.c_gemm_f32(np.ascontiguousarray(A), np.ascontiguousarray(B)))
    C0 = rand((10, 21), 8)
    out = C0.copy()
    go.c_gemm_f32(A, B, out=out, accumulate=True)
    assert np.allclose(out, C0 + go.gemm_f32(A, B), atol=1e-5)
    out64 = C0.astype(np.float64)
    go.c_gemm_f64(A, B, out=out64, accumulate=True)
    assert np.allclose(out64, C0 + go.gemm_f64(A, B), atol=1e-12)


def test_empty_dimensions():
    assert go.c_gemm_f32(np.zeros((0, 4), np.float32), np.zeros((4, 3), np.float32)).shape == (0, 3)
    C = go.c_gemm_f32(np.zeros((2, 0), np.float32), np.zeros((0, 3), np.float32))
    assert C.shape == (2, 3) and np.all(C == 0)


def test_error_report_accepts_good_and_rejects_bad():
    A, B = go.make_inputs(64, 48, 200, seed=9)
    good = go.gemm_f32(A, B)
    rep = go.error_report(good, A, B)
    assert rep["ok"] and rep["normwise"] == 0.0
    bad = good.copy()
    bad[3, 5] += 1.0                      # one wrong element: elementwise bound catches it
    assert not go.error_report(bad, A, B)["ok"]
    drift = good * (1 + 5e-5)             # small relative drift everywhere: normwise bound catches it
    assert not go.error_report(drift.astype(np.float32), A, B)["ok"]
    nan = good.copy()
    nan[0, 0] = np.nan
    assert not go.error_report(nan, A, B)["ok"]
    # dropped last k term
    assert not go.error_report(go.gemm_f32(A[:, :-1], B[:-1]), A, B)["ok"]
    cmp = go.c_compare(good, go.gemm_f64(A, B))
    assert cmp["max_abs"] == pytest.approx(rep["max_abs"], rel=1e-12)


def test_make_inputs_is_seeded_and_in_range():
    A1, B1 = go.make_inputs(8, 9, 10, seed=3)
    A2, B2 = go.make_inputs(8, 9, 10, seed=3)
    assert np.array_equal(A1, A2) and np.array_equal(B1, B2)
    assert A1.dtype == np.float32 and A1.min() >= -1 and A1.max() < 1
    Ai, _ = go.make_inputs(8, 9, 10, seed=3, distribution="integer")
    assert set(np.unique(Ai)).issubset(set(range(10)))
    An, _ = go.make_inputs(200, 9, 200, seed=3, distribution="normal")
    assert abs(float(An.mean())) < 0.05 and abs(float(An.std()) - 1) < 0.05


def golden_cases():
    import json
    from pathlib import Path
    return json.loads((Path(__file__).resolve().parent / "golden" / "gemm_exact_cases.json").read_text())


@pytest.mark.parametrize("case", golden_cases(), ids=lambda c: c["name"])
def test_committed_exact_cases(case):
    """Known answers computed with Python integers (tests/golden/make_gemm_golden.py): every routine of the
    oracle reproduces them bit for bit, also through a transposed copy of B."""
    A, B = np.array(case["A"], np.float32), np.array(case["B"], np.float32)
    C = np.array(case["C"], np.float64)
    assert A.shape == (case["M"], case["K"]) and B.shape == (case["K"], case["N"]) and C.shape == (case["M"], case["N"])
    for routine in (go.gemm_f32, go.gemm_f64, go.c_gemm_f32, go.c_gemm_f64, go.c_gemm_naive):
        assert np.array_equal(np.asarray(routine(A, B), dtype=np.float64), C), routine.__name__
    assert np.array_equal(np.array(go.gemm_exact(A, B), dtype=np.float64), C)
