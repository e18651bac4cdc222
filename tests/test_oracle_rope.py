"""Pins the oracle's per-head RMSNorm + rotary embedding (no reference kernel: README.md:16 only plans the fusion)
against what the mathematics fixes, so that a wrong sign, a wrong pairing (interleaved instead of rotate-half), a
missing norm weight or a head-kind mix-up fails here."""
import numpy as np
import pytest


def _tables(rows, theta=1e6):
    inv = theta ** (-np.arange(64, dtype=np.float64) / 64.0)
    ang = np.arange(rows, dtype=np.float64)[:, None] * inv[None, :]
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


def _reference_f64(x, qw, kw, eps, cos, sin, pos, n_q, n_kv):
    """The published formulation (rotate-half RoPE as in the Qwen/Llama model code): y = x * cos + rotate_half(x) * sin,
    with cos / sin repeated over both halves and rotate_half(x) = cat(-x[64:], x[:64]); RMSNorm per head first."""
    x = x.astype(np.float64)
    M, N = x.shape
    H = n_q + 2 * n_kv
    y = x.reshape(M, H, 128).copy()
    for h in range(n_q + n_kv):
        v = y[:, h, :]
        w = qw if h < n_q else kw
        if w is not None:
            v = v / np.sqrt((v * v).mean(axis=1, keepdims=True) + eps) * w.astype(np.float64)[None, :]
        c = np.concatenate([cos[pos], cos[pos]], axis=1).astype(np.float64)
        s = np.concatenate([sin[pos], sin[pos]], axis=1).astype(np.float64)
        rot = np.concatenate([-v[:, 64:], v[:, :64]], axis=1)
        y[:, h, :] = v * c + rot * s
    return y.reshape(M, N)


@pytest.mark.parametrize("n_q,n_kv,norm", [(32, 8, True), (4, 4, False), (2, 1, True), (1, 1, True)])
def test_matches_float64_rotate_half(oracle, n_q, n_kv, norm):
    rng = np.random.default_rng(n_q * 10 + n_kv)
    M, N = 9, (n_q + 2 * n_kv) * 128
    x = (rng.standard_normal((M, N)) * 3).astype(np.float32)
    qw = rng.uniform(0.5, 1.5, 128).astype(np.float32) if norm else None
    kw = rng.uniform(0.5, 1.5, 128).astype(np.float32) if norm else None
    cos, sin = _tables(4096)
    pos = rng.integers(0, 4096, M).astype(np.int32)
    y = oracle.qk_norm_rope(x, qw, kw, 1e-6, cos, sin, pos, n_q, n_kv)
    ref = _reference_f64(x, qw, kw, 1e-6, cos, sin, pos, n_q, n_kv)
    assert np.max(np.abs(y - ref)) <= 2e-6 * np.max(np.abs(ref))
    # value heads are copied bit for bit
    assert np.array_equal(y[:, (n_q + n_kv) * 128:].view(np.uint32), x[:, (n_q + n_kv) * 128:].view(np.uint32))


def test_query_and_key_heads_use_their_own_norm_weight(oracle):
    rng = np.random.default_rng(1)
    n_q, n_kv, M = 3, 2, 4
    x = rng.standard_normal((M, (n_q + 2 * n_kv) * 128)).astype(np.float32)
    cos, sin = _tables(16)
    pos = np.zeros(M, np.int32)  # angle 0: rope is the identity, what remains is the norm
    qw = np.full(128, 2.0, np.float32)
    kw = np.full(128, 0.5, np.float32)
    y = oracle.qk_norm_rope(x, qw, kw, 0.0, cos, sin, pos, n_q, n_kv).reshape(M, -1, 128)
    rms = np.sqrt((y.astype(np.float64) ** 2).mean(axis=2))
    assert np.allclose(rms[:, :n_q], 2.0, rtol=1e-6) and np.allclose(rms[:, n_q:n_q + n_kv], 0.5, rtol=1e-6)
    # only one of the two weights given: the other kind is not normalised
    y2 = oracle.qk_norm_rope(x, qw, None, 0.0, cos, sin, pos, n_q, n_kv).reshape(M, -1, 128)
    assert np.array_equal(y2[:, n_q:], x.reshape(M, -1, 128)[:, n_q:])
    assert np.array_equal(y2[:, :n_q], y[:, :n_q])


def test_angle_zero_is_the_identity_and_quarter_turn_swaps_halves(oracle):
    rng = np.random.default_rng(2)
    n_q, n_kv, M = 2, 1, 3
    x = rng.standard_normal((M, 4 * 128)).astype(np.float32)
    cos = np.stack([np.ones(64), np.zeros(64)]).astype(np.float32)
    sin = np.stack([np.zeros(64), np.ones(64)]).astype(np.float32)
    y0 = oracle.qk_norm_rope(x, None, None, 1e-6, cos, sin, np.zeros(M, np.int32), n_q, n_kv)
    assert np.array_equal(y0, x)
    y1 = oracle.qk_norm_rope(x, None, None, 1e-6, cos, sin, np.ones(M, np.int32), n_q, n_kv).reshape(M, 4, 128)
    xr = x.reshape(M, 4, 128)
    # a quarter turn: (lo, hi) -> (-hi, lo) exactly, for query and key heads only
    assert np.array_equal(y1[:, :3, :64], -xr[:, :3, 64:]) and np.array_equal(y1[:, :3, 64:], xr[:, :3, :64])
    assert np.array_equal(y1[:, 3], xr[:, 3])


def test_exact_inverse_with_dyadic_angles_and_norm_preservation(oracle):
    """cos = 0.6, sin = 0.8 is not dyadic, so use the 3-4-5 triangle scaled: c = 3, s = 4 gives y = 5 * rotation,
    all products exact for small integers; rotating back with (c, -s) returns 25 x exactly."""
    rng = np.random.default_rng(3)
    n_q, n_kv, M = 1, 1, 5
    x = rng.integers(-64, 64, (M, 3 * 128)).astype(np.float32)
    cos = np.stack([np.full(64, 3.0), np.full(64, 3.0)]).astype(np.float32)
    sin = np.stack([np.full(64, 4.0), np.full(64, -4.0)]).astype(np.float32)
    y = oracle.qk_norm_rope(x, None, None, 0.0, cos, sin, np.zeros(M, np.int32), n_q, n_kv)
    back = oracle.qk_norm_rope(y, None, None, 0.0, cos, sin, np.ones(M, np.int32), n_q, n_kv)
    assert np.array_equal(back[:, :256], 25.0 * x[:, :256])
    # per-pair norm: |y_pair|^2 = 25 |x_pair|^2, exactly in these integers
    xs = x[:, :256].reshape(M, 2, 2, 64).astype(np.float64)
    ys = y[:, :256].reshape(M, 2, 2, 64).astype(np.float64)
    assert np.array_equal((ys ** 2).sum(axis=2), 25.0 * (xs ** 2).sum(axis=2))


def test_positions_are_clamped_to_the_table(oracle):
    rng = np.random.default_rng(4)
    x = rng.standard_normal((3, 3 * 128)).astype(np.float32)
    cos, sin = _tables(8)
    a = oracle.qk_norm_rope(x, None, None, 1e-6, cos, sin, np.array([-5, 100, 7], np.int32), 1, 1)
    b = oracle.qk_norm_rope(x, None, None, 1e-6, cos, sin, np.array([0, 7, 7], np.int32), 1, 1)
    assert np.array_equal(a, b)


def test_sum_of_squares_order_is_the_documented_one(oracle):
    """A head whose partial sums differ by many orders of magnitude gives different fp32 totals for different
    summation orders; rebuild the documented order (fma chain of four per lane, xor butterfly 16, 8, 4, 2, 1) in numpy."""
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((6, 128)) * np.exp(rng.uniform(-12, 12, (6, 128)))).astype(np.float32)
    w = np.ones(128, np.float32)
    cos = np.ones((1, 64), np.float32)
    sin = np.zeros((1, 64), np.float32)
    xx = np.concatenate([x, np.zeros((6, 256), np.float32)], axis=1)
    y = oracle.qk_norm_rope(xx, w, w, 1e-6, cos, sin, np.zeros(6, np.int32), 1, 1)[:, :128]
    for m in range(6):
        part = np.zeros(32, np.float32)
        for l in range(32):
            acc = 0.0  # exact fma: float64 holds x*x + acc of two fp32 values with one rounding to fp32 afterwards
            for e in range(4):
                v = float(x[m, 4 * l + e])
                acc = float(np.float32(np.float64(v) * np.float64(v) + np.float64(acc)))
            part[l] = acc
        for step in (16, 8, 4, 2, 1):
            part = (part + part[np.arange(32) ^ step]).astype(np.float32)
        r = np.float32(1.0) / np.sqrt(np.float32(part[0] / np.float32(128.0) + np.float32(1e-6)))
        want = (x[m] * r) * w
        assert np.array_equal(y[m].view(np.uint32), want.astype(np.float32).view(np.uint32))
