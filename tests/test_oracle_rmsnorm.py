"""The oracle's RMSNorm (no reference kernel: README.md:16 only plans to fuse it) pinned by the mathematics:
float64 evaluation of x / sqrt(mean(x^2) + eps) * w, unit mean square of the output, exact invariance under
power-of-two scaling of the input when eps = 0 (every operation then scales exactly), and the documented
summation order on a case where the order decides the last bit."""
import numpy as np


def test_against_float64(oracle):
    rng = np.random.default_rng(1)
    for K in (128, 2560, 4096, 9728, 132):
        x = (rng.standard_normal((7, K)) * 3).astype(np.float32)
        w = rng.uniform(0.5, 1.5, K).astype(np.float32)
        y = oracle.rmsnorm(x, w, 1e-6)
        x64 = x.astype(np.float64)
        want = x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + 1e-6) * w.astype(np.float64)
        assert y.dtype == np.float32 and np.all(np.abs(y - want) <= 4e-7 * np.abs(want) + 1e-30)


def test_unit_mean_square_and_weight(oracle):
    rng = np.random.default_rng(2)
    x = (rng.standard_normal((5, 2560)) * 17).astype(np.float32)
    y = oracle.rmsnorm(x, np.ones(2560, np.float32), 0.0)
    assert np.allclose((y.astype(np.float64) ** 2).mean(axis=1), 1.0, rtol=1e-6)
    w = np.full(2560, 0.25, np.float32)
    assert np.array_equal(oracle.rmsnorm(x, w, 0.0), y * np.float32(0.25))      # exact: a power of two
    # eps dominates a zero row: no NaN, y = 0
    z = oracle.rmsnorm(np.zeros((1, 256), np.float32), np.ones(256, np.float32), 1e-6)
    assert np.array_equal(z, np.zeros((1, 256), np.float32))


def test_power_of_two_scaling_is_exact_without_eps(oracle):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((4, 1024)).astype(np.float32)
    w = rng.uniform(0.5, 1.5, 1024).astype(np.float32)
    y = oracle.rmsnorm(x, w, 0.0)
    for k in (-7, 3, 12):
        assert np.array_equal(oracle.rmsnorm(x * np.float32(2.0 ** k), w, 0.0), y)


def test_documented_summation_order(oracle):
    """The sum of squares in the documented order (256 interleaved partial sums of fused multiply-adds, an xor
    butterfly inside each group of 64, then (G0 + G1) + (G2 + G3)), restated with exact rationals rounded to fp32
    after every operation."""
    from fractions import Fraction
    rng = np.random.default_rng(4)
    K = 2560
    x = rng.standard_normal((1, K)).astype(np.float32)

    def f32(v):
        return np.float32(v)

    def fma(a, b, c):  # exactly rounded a*b+c
        return np.float32(float(Fraction(float(a)) * Fraction(float(b)) + Fraction(float(c))))

    p = [np.float32(0)] * 256
    for c in range(K // 4):
        for e in range(4):
            v = x[0, 4 * c + e]
            p[c % 256] = fma(v, v, p[c % 256])
    G = []
    for g in range(4):
        pg = p[64 * g:64 * g + 64]
        for step in (32, 16, 8, 4, 2, 1):
            pg = [f32(pg[l] + pg[l ^ step]) for l in range(64)]
        G.append(pg[0])
    total = f32(f32(G[0] + G[1]) + f32(G[2] + G[3]))
    ms = f32(total / np.float32(K))
    r = f32(np.float32(1.0) / np.sqrt(f32(ms + np.float32(1e-6))))
    w = np.ones(K, np.float32)
    want = (x[0] * r) * w
    assert np.array_equal(oracle.rmsnorm(x, w, 1e-6)[0], want)


def test_rmsnorm_quant_is_the_quantiser_applied_to_the_norm(oracle):
    rng = np.random.default_rng(5)
    x = rng.standard_normal((9, 512)).astype(np.float32)
    w = rng.uniform(0.5, 1.5, 512).astype(np.float32)
    q, s = oracle.rmsnorm_quant(x, w, 1e-6)
    q2, s2 = oracle.quant_fp8(oracle.rmsnorm(x, w, 1e-6), 1, True)
    assert np.array_equal(q, q2) and np.array_equal(s, s2) and s.shape == (4, 9)
