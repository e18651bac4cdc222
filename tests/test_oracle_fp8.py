"""Pins the FP8 path of the oracle: quantiser invariants, exact-arithmetic evaluation of the
blockwise GEMM on small shapes, the reference's B = I known-answer test and idempotence of the
fused re-quantisation."""
from fractions import Fraction

import numpy as np
import pytest


def _round_f32(fr):
    """Correctly rounded (nearest even) float32 of a Fraction."""
    if fr == 0:
        return np.float32(0)
    sign = -1 if fr < 0 else 1
    a = abs(fr)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    e = max(e, -126)
    q = a / Fraction(2) ** (e - 23)  # in units of the ulp
    n = q.numerator // q.denominator
    rem = q - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and n % 2 == 1):
        n += 1
    return np.float32(sign * float(Fraction(n) * Fraction(2) ** (e - 23)))


def test_round_f32_helper():
    for v in (1.0, 1.0 + 2.0 ** -24, 1.0 + 3 * 2.0 ** -24, 0.1, 1e-40, 3.0e38):
        assert _round_f32(Fraction(v)) == np.float32(v)


@pytest.mark.parametrize("quant_m,transpose", [(1, True), (1, False), (128, False), (128, True)])
def test_quantiser_invariants(oracle, rng, quant_m, transpose):
    M, N = 200, 384  # ragged rows for the 128-row blocks
    x = rng.normal(0, 1, (M, N)).astype(np.float32)
    x[:, 17] *= 20
    x[5, :128] = 0  # an all-zero 1x128 block
    x[128:200, 256:384] = 0  # an all-zero (ragged) 128x128 block
    q, s = oracle.quant_fp8(x, quant_m, transpose)
    dec = oracle.e4m3_decode(q)
    assert np.isfinite(dec).all() and np.abs(dec).max() <= 448
    for bi in range(-(-M // quant_m)):
        for bj in range(N // 128):
            blk = x[bi * quant_m:(bi + 1) * quant_m, bj * 128:(bj + 1) * 128]
            sc = s[bj, bi] if transpose else s[bi, bj]
            amax = np.abs(blk).max()
            assert sc == np.float32(amax) / np.float32(448)
            qb = dec[bi * quant_m:(bi + 1) * quant_m, bj * 128:(bj + 1) * 128]
            if amax == 0:
                assert sc == 0 and (q[bi * quant_m:(bi + 1) * quant_m, bj * 128:(bj + 1) * 128] == 0).all()
                continue
            # the block's extreme element lands exactly on +-448
            i, j = np.unravel_index(np.abs(blk).argmax(), blk.shape)
            assert abs(qb[i, j]) == 448
            # round-to-nearest: error at most half a code step (in units of the scale)
            ulp = np.where(np.abs(qb) < 2.0 ** -6, 2.0 ** -9, 2.0 ** (np.floor(np.log2(np.maximum(np.abs(qb), 2.0 ** -6))) - 3))
            assert (np.abs(blk / sc - qb) <= 0.5 * ulp * (1 + 1e-6) + 1e-7).all()


def test_quantiser_scale_layouts(oracle, rng):
    x = rng.normal(0, 1, (256, 256)).astype(np.float32)
    q1, s1 = oracle.quant_fp8(x, 1, True)
    q2, s2 = oracle.quant_fp8(x, 1, False)
    assert (q1 == q2).all() and s1.shape == (2, 256) and s2.shape == (256, 2) and (s1 == s2.T).all()
    q3, s3 = oracle.quant_fp8(x, 128, False)
    q4, s4 = oracle.quant_fp8(x, 128, True)
    assert (q3 == q4).all() and s3.shape == (2, 2) and s4.shape == (2, 256) and (s4[:, :2] == s3.T).all()
    assert np.allclose(oracle.dequant_fp8(q1, s1, 1, True), x, atol=np.abs(x).max() / 448 * 17)


def _exact_reference(oracle, Aq, As, Bq, Bs, promote, assoc):
    """Same promotion order, but every partial sum in exact rational arithmetic and every fp32
    operation rounded explicitly."""
    M, K = Aq.shape
    N = Bq.shape[0]
    da = oracle.e4m3_decode(Aq)
    db = oracle.e4m3_decode(Bq)
    C = np.zeros((M, N), np.float32)
    for m in range(M):
        for n in range(N):
            acc = np.float32(0)
            for kb in range(K // 128):
                a_s, b_s = As[kb, m], Bs[n // 128, kb]
                for c0 in range(kb * 128, kb * 128 + 128, promote):
                    p = sum(Fraction(float(da[m, k])) * Fraction(float(db[n, k])) for k in range(c0, c0 + promote))
                    p = _round_f32(p)
                    if assoc == 0:
                        t = np.float32(p * a_s)
                        acc = _round_f32(Fraction(float(t)) * Fraction(float(b_s)) + Fraction(float(acc)))
                    else:
                        s = np.float32(a_s * b_s)
                        acc = _round_f32(Fraction(float(p)) * Fraction(float(s)) + Fraction(float(acc)))
            C[m, n] = acc
    return C


@pytest.mark.parametrize("promote,assoc", [(128, 1), (32, 1), (32, 0)])
def test_fp8_gemm_against_exact_arithmetic(oracle, rng, promote, assoc):
    M, N, K = 3, 130, 256
    A = rng.normal(0, 1, (M, K)).astype(np.float32)
    A[:, 40] *= 20
    W = rng.normal(0, 0.02, (N, K)).astype(np.float32)
    Aq, As = oracle.quant_fp8(A, 1, True)
    Bq, Bs = oracle.quant_fp8(W, 128, False)
    got = oracle.fp8_gemm(Aq, As, Bq, Bs, promote=promote, assoc=assoc)
    ref = _exact_reference(oracle, Aq, As, Bq, Bs, promote, assoc)
    assert (got == ref).all()
    # and the quantised product approximates the unquantised one
    assert np.abs(got - A @ W.T).max() < 0.1 * np.abs(A @ W.T).max()


def test_fp8_gemm_promotion_orders_agree_to_rounding(oracle, rng):
    from helpers import fp8_inputs
    Aq, As, Bq, Bs = fp8_inputs(oracle, 64, 256, 1024)
    c128 = oracle.fp8_gemm(Aq, As, Bq, Bs, 128, 1)
    c32 = oracle.fp8_gemm(Aq, As, Bq, Bs, 32, 1)
    c32b = oracle.fp8_gemm(Aq, As, Bq, Bs, 32, 0)
    amax = np.abs(c128).max()
    assert np.abs(c128 - c32).max() <= 1e-5 * amax and np.abs(c32 - c32b).max() <= 1e-5 * amax


def test_b_identity_known_answer(oracle, rng):
    # reference KAT (examples/005.fp8.mm.cu:2620-2634): A random, B = I  =>  C == dequant(A);
    # and because C's 1x128 groups coincide with A's, re-quantising C gives back A's codes and scales
    M = N = K = 256
    A = rng.uniform(-5, 5, (M, K)).astype(np.float32)
    Aq, As = oracle.quant_fp8(A, 1, True)
    Bq, Bs = oracle.quant_fp8(np.eye(N, K, dtype=np.float32), 128, False)
    assert (Bq[np.arange(N), np.arange(N)] == 0x7E).all() and (Bs[0, 0], Bs[0, 1]) == (np.float32(1) / np.float32(448), 0)
    for promote in (32, 128):
        C = oracle.fp8_gemm(Aq, As, Bq, Bs, promote=promote)
        deq = oracle.dequant_fp8(Aq, As, 1, True)
        assert np.abs(C - deq).max() <= 4 * np.spacing(np.abs(deq).max())
        Cq, Cs = oracle.requant_c_1x128(C)
        assert (Cq == Aq).all()
        assert np.abs(Cs - As).max() <= 1e-6 * As.max()


@pytest.mark.parametrize("reciprocal", [True, False])
def test_requant_is_idempotent(oracle, rng, reciprocal):
    C = rng.normal(0, 3, (64, 384)).astype(np.float32)
    C[7, 128:256] = 0
    Cq, Cs = oracle.requant_c_1x128(C, reciprocal=reciprocal)
    assert (Cq[7, 128:256] == 0).all() and Cs[1, 7] == 0
    deq = oracle.e4m3_decode(Cq) * np.repeat(Cs.T, 128, axis=1)
    Cq2, Cs2 = oracle.requant_c_1x128(deq, reciprocal=reciprocal)
    assert (Cq2 == Cq).all() and np.abs(Cs2 - Cs).max() <= 1e-6 * Cs.max()
    # the two reference forms (multiply by 448/amax vs divide by the scale) differ by at most one code step
    Cq_other, _ = oracle.requant_c_1x128(C, reciprocal=not reciprocal)
    assert np.abs(oracle.e4m3_code_index(Cq) - oracle.e4m3_code_index(Cq_other)).max() <= 1


def test_requant_zero_guard_versus_reference_nan(oracle):
    C = np.zeros((2, 128), np.float32)
    q_guard, s = oracle.requant_c_1x128(C, zero_guard=True)
    q_ref, _ = oracle.requant_c_1x128(C, zero_guard=False)
    assert (q_guard == 0).all() and (s == 0).all()
    assert (q_ref == 0x7F).all()  # the reference's unguarded 0 * inf = NaN


def test_requant_overflowing_reciprocal(oracle):
    """A group whose amax lies below 448 / FLT_MAX (about 2^-119): 448.f / amax is +inf.  The reference's arithmetic then
    writes +-448 for every non-zero element and NaN for the zeros; under the guard the group's codes are 0 next to the
    scale amax / 448 (v * 0: a negative element gives -0, code 0x80), and a group just above the limit is quantised as usual (its amax element reaches 448)."""
    tiny = np.float32(2.0 ** -121)
    C = np.zeros((3, 128), np.float32)
    C[0, :4] = [tiny, -tiny / 2, 0.0, tiny / 4]
    C[1, :3] = [np.float32(1e-36), np.float32(-5e-37), 0.0]      # also below 1.3166e-36
    C[2, :3] = [np.float32(2.0 ** -118), np.float32(-2.0 ** -119), 0.0]  # reciprocal finite
    with np.errstate(over="ignore", invalid="ignore", divide="ignore"):
        q_ref, _ = oracle.requant_c_1x128(C, zero_guard=False)
        q, s = oracle.requant_c_1x128(C, zero_guard=True)
    assert list(q_ref[0, :4]) == [0x7E, 0xFE, 0x7F, 0x7E]
    assert ((q[0] & 0x7F) == 0).all() and ((q[1] & 0x7F) == 0).all()  # signed zeros: v * 0
    assert q[0, 1] == 0x80 and q[0, 0] == 0
    assert s[0, 0] == np.float32(tiny) / np.float32(448.0) and s[0, 1] == np.float32(1e-36) / np.float32(448.0)
    assert q[2, 0] == 0x7E and q[2, 1] == 0xF6 and q[2, 2] == 0  # 448 and -224
    assert (q[2] == q_ref[2]).all()
