"""The oracle's SwiGLU (silu(gate) * up in fp32) has no reference kernel to follow -- the reference only plans the
fusion (README.md:16) -- so it is pinned by the mathematics: known values of x / (1 + exp(-x)), the algebraically
different tanh form evaluated in float64, the limits, and the gate/up order."""
import numpy as np


def test_known_values(oracle):
    g = np.array([[0.0, 1.0, -1.0, 2.0]], np.float32)
    u = np.array([[3.0, 1.0, 1.0, -2.0]], np.float32)
    h = oracle.swiglu(np.concatenate([g, u], axis=1))
    want = np.array([[0.0, 0.7310585786300049, -0.2689414213699951, -2 * 1.7615941559557649]])
    assert np.allclose(h, want, rtol=3e-7, atol=0)
    # gate first, up second: swapping the halves is a different function
    h2 = oracle.swiglu(np.concatenate([u, g], axis=1))
    assert not np.allclose(h, h2)
    assert np.isclose(oracle.swiglu(np.array([[1.0, 2.0]], np.float32))[0, 0], 2 * 0.7310585786300049, rtol=3e-7)
    assert np.isclose(oracle.swiglu(np.array([[2.0, 1.0]], np.float32))[0, 0], 1.7615941559557649, rtol=3e-7)


def test_against_tanh_form_in_float64(oracle):
    rng = np.random.default_rng(3)
    g = (rng.standard_normal((64, 256)) * 4).astype(np.float32)
    u = (rng.standard_normal((64, 256)) * 2).astype(np.float32)
    h = oracle.swiglu(np.concatenate([g, u], axis=1))
    g64, u64 = g.astype(np.float64), u.astype(np.float64)
    want = g64 * 0.5 * (1.0 + np.tanh(0.5 * g64)) * u64
    assert h.dtype == np.float32
    assert np.all(np.abs(h - want) <= 4e-7 * np.abs(want) + 1e-37)


def test_limits_and_shape(oracle):
    big = np.array([[80.0, -80.0, 200.0, -200.0, 7.0, 7.0, 7.0, 7.0]], np.float32)
    h = oracle.swiglu(big)
    assert h.shape == (1, 4)
    assert h[0, 0] == np.float32(80.0 * 7.0) and h[0, 2] == np.float32(200.0 * 7.0)   # silu(x) -> x
    assert abs(h[0, 1]) < 1e-30 and h[0, 3] == 0.0                                     # silu(-x) -> -0
    assert np.all(np.isfinite(h))


def test_requant_is_the_plain_epilogue_applied_to_h(oracle):
    rng = np.random.default_rng(4)
    C = rng.standard_normal((8, 512)).astype(np.float32) * 3
    q, s = oracle.swiglu_requant(C)
    q2, s2 = oracle.requant_c_1x128(oracle.swiglu(C))
    assert q.shape == (8, 256) and s.shape == (2, 8)
    assert np.array_equal(q, q2) and np.array_equal(s, s2)
    # every 1x128 group of h reaches +-448 (code 0x7E / 0xFE) and scale == amax / 448
    h = oracle.swiglu(C)
    amax = np.abs(h).reshape(8, 2, 128).max(-1)
    assert np.array_equal(s, (amax / np.float32(448.0)).T.astype(np.float32))
    assert np.all(((q & 0x7F) == 0x7E).reshape(8, 2, 128).any(-1))
