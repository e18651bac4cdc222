"""Shared helpers of the test-suite: seeded inputs of the benchmark configurations and tolerance checks."""
import numpy as np


def fp16_inputs_uniform(M, N, K, seed=1):
    """cfg1: A, B ~ U(-1, 1), filled A then B in row-major order from one generator
    (the fill order of test/fp16_mm_test.cc:16-20), rounded to fp16."""
    rng = np.random.default_rng(seed)
    A = rng.uniform(-1.0, 1.0, (M, K)).astype(np.float32).astype(np.float16)
    B = rng.uniform(-1.0, 1.0, (K, N)).astype(np.float32).astype(np.float16)
    return A, B


def fp16_inputs_normal(M, N, K, seed=2):
    """cfg2: A ~ N(0,1), B ~ N(0,0.02), fp16."""
    rng = np.random.default_rng(seed)
    A = rng.standard_normal((M, K), dtype=np.float32).astype(np.float16)
    B = (rng.standard_normal((K, N), dtype=np.float32) * np.float32(0.02)).astype(np.float16)
    return A, B


def fp8_inputs(oracle, M, N, K, seed=3):
    """cfg3: A ~ N(0,1) with 1% of the K channels x20 -> 1x128 quant; B ~ N(0,0.02) [K,N] ->
    transposed [N,K] -> 128x128 quant.  Quantised by the CPU oracle (deterministic bytes)."""
    rng = np.random.default_rng(seed)
    A = rng.standard_normal((M, K), dtype=np.float32)
    nout = max(1, -(-K // 100))
    cols = rng.choice(K, nout, replace=False)
    A[:, cols] *= np.float32(20.0)
    B = rng.standard_normal((K, N), dtype=np.float32) * np.float32(0.02)
    Aq, As = oracle.quant_fp8(A, 1, True)
    Bq, Bs = oracle.quant_fp8(np.ascontiguousarray(B.T), 128, False)
    return Aq, As, Bq, Bs


def assert_fp16_close(got, ref, what=""):
    """FP16 GEMM bar: |d| <= 1e-3 + 1e-2 * |ref| element-wise (fp32 Kahan reference)."""
    got = np.asarray(got, dtype=np.float32)
    err = np.abs(got - ref)
    tol = 1e-3 + 1e-2 * np.abs(ref)
    bad = err > tol
    assert not bad.any(), "%s: %d of %d elements outside 1e-3 + 1e-2*|ref| (max err %g)" % (what, bad.sum(), bad.size, err.max())


def row_block_amax(ref):
    M, N = ref.shape
    nb = N // 128
    return np.abs(ref).reshape(M, nb, 128).max(-1).repeat(128, axis=1)


def assert_fp8_gemm_close(got, ref, what=""):
    """FP8 GEMM fp32/bf16 bar: |d| <= 2e-2 * max(|ref|, row-block amax * 2^-7).  The floor keeps the
    relative test meaningful where a sum cancels to (almost) zero."""
    got = np.asarray(got, dtype=np.float32)
    err = np.abs(got - ref)
    tol = 2e-2 * np.maximum(np.abs(ref), row_block_amax(ref) * 2.0 ** -7)
    bad = err > tol
    assert not bad.any(), "%s: %d of %d elements outside 2e-2 relative (max err %g)" % (what, bad.sum(), bad.size, err.max())


def assert_fused_close(oracle, cq, cs, rq, rs, what=""):
    """Fused-quant bar: codes within 1 e4m3 code step on >= 99.9% of elements, scales within 1e-3 relative."""
    d = np.abs(oracle.e4m3_code_index(cq) - oracle.e4m3_code_index(rq))
    frac = float((d <= 1).mean())
    assert frac >= 0.999, "%s: only %.5f of the codes within one e4m3 step" % (what, frac)
    rel = np.abs(cs - rs) / np.maximum(np.abs(rs), 1e-30)
    rel = np.where(rs == 0, np.abs(cs), rel)
    assert rel.max() <= 1e-3, "%s: scale relative error %g" % (what, rel.max())
