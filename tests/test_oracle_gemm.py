"""Pins the GEMM references of the oracle (restating test/kahan.cu) with closed forms, the
reference's own known-answer patterns and brute force in exact arithmetic on small shapes."""
from fractions import Fraction

import numpy as np
import pytest


def _f32(x):
    return np.float32(x)


def _kahan_bruteforce(A, B):
    """Scalar float32 re-evaluation of test/kahan.cu:16-26 with numpy scalars (round after every op)."""
    M, K = A.shape
    N = B.shape[1]
    C = np.zeros((M, N), np.float32)
    for m in range(M):
        for n in range(N):
            s, d = _f32(0), _f32(0)
            for k in range(K):
                y = _f32(_f32(A[m, k] * B[k, n]) - d)
                t = _f32(s + y)
                d = _f32(_f32(t - s) - y)
                s = t
            C[m, n] = s
    return C


def test_kahan_matches_scalar_bruteforce_unfused(oracle, rng):
    A = rng.normal(0, 1, (5, 37)).astype(np.float32)
    B = rng.normal(0, 1, (37, 7)).astype(np.float32)
    assert (oracle.kahan_gemm(A, B, fused=False) == _kahan_bruteforce(A, B)).all()


def test_kahan_fused_equals_unfused_on_fp16_inputs(oracle, rng):
    # products of fp16 (or bf16) values are exact in fp32, so contracting a*b-diff into an FMA changes nothing
    A = rng.normal(0, 1, (16, 200)).astype(np.float16).astype(np.float32)
    B = rng.normal(0, 1, (200, 24)).astype(np.float16).astype(np.float32)
    assert (oracle.kahan_gemm(A, B, fused=True) == oracle.kahan_gemm(A, B, fused=False)).all()


def test_kahan_compensation_beats_naive_fp32(oracle):
    # 1 + 4096 * 2^-24: a plain fp32 running sum stays at 1, the compensated one recovers the tail
    K = 4097
    A = np.full((1, K), 2.0 ** -12, np.float32)
    A[0, 0] = 1.0
    B = np.full((K, 1), 2.0 ** -12, np.float32)
    B[0, 0] = 1.0
    exact = 1.0 + 4096 * 2.0 ** -24
    assert oracle.kahan_gemm(A, B)[0, 0] == np.float32(exact)
    naive = np.float32(0)
    for k in range(K):
        naive = np.float32(naive + np.float32(A[0, k] * B[k, 0]))
    assert naive == np.float32(1.0)


def test_double_gemm_against_exact_rationals(oracle, rng):
    A = rng.normal(0, 1, (4, 23)).astype(np.float16).astype(np.float32)
    B = rng.normal(0, 1, (23, 5)).astype(np.float16).astype(np.float32)
    C = oracle.double_gemm(A, B)
    for m in range(4):
        for n in range(5):
            exact = sum(Fraction(float(A[m, k])) * Fraction(float(B[k, n])) for k in range(23))
            assert C[m, n] == np.float32(float(exact))  # 23 fp16 products sum exactly in double


def test_kahan_close_to_double_reference(oracle, rng):
    A = rng.uniform(-1, 1, (64, 1024)).astype(np.float16).astype(np.float32)
    B = rng.uniform(-1, 1, (1024, 48)).astype(np.float16).astype(np.float32)
    k, d = oracle.kahan_gemm(A, B), oracle.double_gemm(A, B)
    assert np.abs(k - d).max() <= 2 * np.spacing(np.abs(d).max())


def test_identity_corner_known_answer(oracle):
    # reference KAT (examples/004.fp16.mm.ldmatrix.cu:6750-6775): A = I on a limit x limit corner,
    # B = row*limit + col there, zero elsewhere  =>  the corner of C equals B exactly
    M = N = K = 64
    limit = 16
    A = np.zeros((M, K), np.float32)
    B = np.zeros((K, N), np.float32)
    A[:limit, :limit] = np.eye(limit)
    B[:limit, :limit] = np.arange(limit * limit).reshape(limit, limit)
    for C in (oracle.kahan_gemm(A, B), oracle.double_gemm(A, B)):
        assert (C[:limit, :limit] == B[:limit, :limit]).all() and C[limit:].sum() == 0 and C[:, limit:].sum() == 0


def test_all_ones_gives_k(oracle):
    for K in (16, 512, 2048):
        C = oracle.kahan_gemm(np.ones((8, K), np.float32), np.ones((K, 8), np.float32))
        assert (C == K).all()


def test_transposed_layout_is_bit_identical(oracle, rng):
    A = rng.normal(0, 1, (32, 300)).astype(np.float32)
    B = rng.normal(0, 1, (300, 40)).astype(np.float32)
    for fused in (True, False):
        assert (oracle.kahan_gemm(A, B, fused) == oracle.kahan_gemm_bt(A, np.ascontiguousarray(B.T), fused)).all()


def test_a_transposed_operand_or_wrong_index_is_detected(oracle, rng):
    # guards the checks above: the sort of mistake they are meant to catch does change the result
    A = rng.normal(0, 1, (8, 8)).astype(np.float32)
    B = rng.normal(0, 1, (8, 8)).astype(np.float32)
    assert not np.allclose(oracle.kahan_gemm(A, B), oracle.kahan_gemm(A, B.T.copy()))
