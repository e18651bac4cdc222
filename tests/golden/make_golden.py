#!/usr/bin/env python3
"""Writes the golden fixtures of the test-suite (inputs + expected outputs of the CPU oracle).

    python tests/golden/make_golden.py

The reference stores no golden vectors of its own (its tests print error statistics and assert
nothing, test/fp16_mm_test.cc:63-82), so these fixtures are produced by this repository's
oracle, which tests/test_oracle_*.py pin against closed forms and exact arithmetic.  They guard
against drift of the oracle and give the GPU tests inputs with byte-stable expected outputs.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle  # noqa: E402


def main():
    rng = np.random.default_rng(20240601)
    # FP16 GEMM 128 x 128 x 80 (K not a multiple of 32: exercises the K tail), fp16 and bf16 inputs
    A = rng.uniform(-1, 1, (128, 80)).astype(np.float32)
    B = rng.uniform(-1, 1, (80, 128)).astype(np.float32)
    a16, b16 = oracle.f32_to_f16_bits(A), oracle.f32_to_f16_bits(B)
    abf, bbf = oracle.f32_to_bf16_bits(A), oracle.f32_to_bf16_bits(B)
    np.savez_compressed(os.path.join(HERE, "fp16_gemm_128x128x80.npz"),
                        a_f16=a16, b_f16=b16, c_f16_kahan=oracle.kahan_gemm(oracle.f16_bits_to_f32(a16), oracle.f16_bits_to_f32(b16)),
                        a_bf16=abf, b_bf16=bbf, c_bf16_kahan=oracle.kahan_gemm(oracle.bf16_bits_to_f32(abf), oracle.bf16_bits_to_f32(bbf)))
    # quantiser: ragged rows, an outlier column, a zero block
    x = rng.normal(0, 1, (130, 256)).astype(np.float32)
    x[:, 77] *= 20
    x[3, 128:] = 0
    q1, s1 = oracle.quant_fp8(x, 1, True)
    q128, s128 = oracle.quant_fp8(x, 128, False)
    np.savez_compressed(os.path.join(HERE, "quant_130x256.npz"), x=x, q_1x128=q1, s_1x128_t=s1, q_128x128=q128, s_128x128=s128)
    # FP8 blockwise GEMM 128 x 256 x 256 and a skinny M = 5 case on the same weights
    X = rng.normal(0, 1, (128, 256)).astype(np.float32)
    X[:, [9, 200]] *= 20
    W = rng.normal(0, 0.02, (256, 256)).astype(np.float32)
    Aq, As = oracle.quant_fp8(X, 1, True)
    Bq, Bs = oracle.quant_fp8(W, 128, False)
    C = oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128)
    Cq, Cs = oracle.requant_c_1x128(C)
    A5q, A5s = oracle.quant_fp8(X[:5], 1, True)
    C5 = oracle.fp8_gemm(A5q, A5s, Bq, Bs, promote=128)
    C5q, C5s = oracle.requant_c_1x128(C5)
    np.savez_compressed(os.path.join(HERE, "fp8_gemm_128x256x256.npz"), aq=Aq, a_scale_t=As, bq_t=Bq, b_scale=Bs, c_f32=C,
                        c_bf16=oracle.f32_to_bf16_bits(C), cq=Cq, c_scale_t=Cs, a5q=A5q, a5_scale_t=A5s, c5_f32=C5, c5q=C5q, c5_scale_t=C5s)
    # offline layouts: the pre-shuffled image of a 48 x 384 weight block and a 128 x 256 byte transpose
    bt = rng.integers(0, 256, (48, 384), dtype=np.uint8)
    t_in = rng.integers(0, 256, (128, 256), dtype=np.uint8)
    np.savez_compressed(os.path.join(HERE, "layout_48x384.npz"), bt=bt, bp=oracle.preshuffle_b(bt), t_in=t_in,
                        t_out=oracle.transpose_aligned_128(t_in))
    # SwiGLU output of a gate_up-like GEMM 128 x 512 x 256 (256 gate + 256 up columns; the gate scales are raised so
    # that silu leaves its linear range)
    Xs = rng.normal(0, 1, (128, 256)).astype(np.float32)
    Xs[:, [3, 131]] *= 20
    Ws = rng.normal(0, 0.02, (512, 256)).astype(np.float32)
    Sq, Ss = oracle.quant_fp8(Xs, 1, True)
    Wq, Wsc = oracle.quant_fp8(Ws, 128, False)
    Wsc[:2] *= np.float32(40.0)
    Cg = oracle.fp8_gemm(Sq, Ss, Wq, Wsc, promote=128)
    Hq, Hs = oracle.swiglu_requant(Cg)
    np.savez_compressed(os.path.join(HERE, "swiglu_128x512x256.npz"), aq=Sq, a_scale_t=Ss, bq_t=Wq, b_scale=Wsc, c_f32=Cg, h_f32=oracle.swiglu(Cg),
                        hq=Hq, h_scale_t=Hs)
    # per-head RMSNorm + RoPE behind a QKV projection: 2 query, 1 key, 1 value head, positions beyond both table ends
    xr = (rng.standard_normal((16, 4 * 128)) * 3).astype(np.float32)
    qw = rng.uniform(0.5, 1.5, 128).astype(np.float32)
    kw = rng.uniform(0.5, 1.5, 128).astype(np.float32)
    inv = 1e6 ** (-np.arange(64, dtype=np.float64) / 64.0)
    ang = np.arange(48, dtype=np.float64)[:, None] * inv[None, :]
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    pos = rng.integers(-2, 52, 16).astype(np.int32)
    yr = oracle.qk_norm_rope(xr, qw, kw, 1e-6, cos, sin, pos, 2, 1)
    yq, ys = oracle.requant_c_1x128(yr)
    np.savez_compressed(os.path.join(HERE, "qk_norm_rope_16x512.npz"), x=xr, qw=qw, kw=kw, cos=cos, sin=sin, pos=pos, y=yr, y_bf16=oracle.f32_to_bf16_bits(yr),
                        yq=yq, y_scale_t=ys)
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    main()
