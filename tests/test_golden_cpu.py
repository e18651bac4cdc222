"""The committed golden fixtures are what the oracle produces today (guards against drift)."""
import os

import numpy as np

G = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def test_fp16_fixture(oracle):
    d = np.load(os.path.join(G, "fp16_gemm_128x128x80.npz"))
    assert (oracle.kahan_gemm(oracle.f16_bits_to_f32(d["a_f16"]), oracle.f16_bits_to_f32(d["b_f16"])) == d["c_f16_kahan"]).all()
    assert (oracle.kahan_gemm(oracle.bf16_bits_to_f32(d["a_bf16"]), oracle.bf16_bits_to_f32(d["b_bf16"])) == d["c_bf16_kahan"]).all()
    # closed-form cross-check of the stored result: float64 matmul of the same fp16 values
    ref = oracle.f16_bits_to_f32(d["a_f16"]).astype(np.float64) @ oracle.f16_bits_to_f32(d["b_f16"]).astype(np.float64)
    assert np.abs(d["c_f16_kahan"] - ref).max() <= 2e-6


def test_quant_fixture(oracle):
    d = np.load(os.path.join(G, "quant_130x256.npz"))
    q, s = oracle.quant_fp8(d["x"], 1, True)
    assert (q == d["q_1x128"]).all() and (s == d["s_1x128_t"]).all()
    q, s = oracle.quant_fp8(d["x"], 128, False)
    assert (q == d["q_128x128"]).all() and (s == d["s_128x128"]).all()
    assert (d["q_1x128"][3, 128:] == 0).all() and d["s_1x128_t"][1, 3] == 0


def test_fp8_fixture(oracle):
    d = np.load(os.path.join(G, "fp8_gemm_128x256x256.npz"))
    C = oracle.fp8_gemm(d["aq"], d["a_scale_t"], d["bq_t"], d["b_scale"], promote=128)
    assert (C == d["c_f32"]).all()
    Cq, Cs = oracle.requant_c_1x128(C)
    assert (Cq == d["cq"]).all() and (Cs == d["c_scale_t"]).all()
    assert (oracle.f32_to_bf16_bits(C) == d["c_bf16"]).all()
    C5 = oracle.fp8_gemm(d["a5q"], d["a5_scale_t"], d["bq_t"], d["b_scale"], promote=128)
    assert (C5 == d["c5_f32"]).all() and (C5 == C[:5]).all()  # rows are independent
    # closed-form cross-check: dequantise and multiply in float64
    A = oracle.dequant_fp8(d["aq"], d["a_scale_t"], 1, True).astype(np.float64)
    W = oracle.dequant_fp8(d["bq_t"], d["b_scale"], 128, False).astype(np.float64)
    assert np.abs(C - A @ W.T).max() <= 1e-5 * np.abs(C).max()


def test_layout_fixture(oracle):
    d = np.load(os.path.join(G, "layout_48x384.npz"))
    assert np.array_equal(oracle.preshuffle_b(d["bt"]), d["bp"]) and np.array_equal(oracle.unshuffle_b(d["bp"]), d["bt"])
    assert np.array_equal(d["t_out"], d["t_in"].T)
    # spot value fixed by the layout's definition: row 17 (= row 1 of row group 1), chunk 5 of slice 2 sits in block
    # (1, 2) at row 1's line, chunk 5 ^ swz(1) = 5 ^ 0
    blk = d["bp"].reshape(-1)[(1 * 3 + 2) * 2048:(1 * 3 + 2 + 1) * 2048]
    assert np.array_equal(blk[1 * 128 + 5 * 16:1 * 128 + 6 * 16], d["bt"][17, 2 * 128 + 5 * 16:2 * 128 + 6 * 16])


def test_swiglu_fixture(oracle):
    d = np.load(os.path.join(G, "swiglu_128x512x256.npz"))
    C = oracle.fp8_gemm(d["aq"], d["a_scale_t"], d["bq_t"], d["b_scale"], promote=128)
    assert (C == d["c_f32"]).all()
    h = oracle.swiglu(C)
    # exp may differ by an ulp between numpy builds / CPUs: hold the stored activation to 2 ulp, not to the bit
    assert np.all(np.abs(h - d["h_f32"]) <= 2.4e-7 * np.abs(d["h_f32"]) + 1e-38)
    assert np.abs(C[:, :256]).max() > 2.0, "the fixture does not leave silu's linear range"
    hq, hs = oracle.swiglu_requant(C)
    step = np.abs(oracle.e4m3_code_index(hq) - oracle.e4m3_code_index(d["hq"]))
    assert (step <= 1).all() and (step == 0).mean() >= 0.9999
    assert np.all(np.abs(hs - d["h_scale_t"]) <= 1e-6 * np.abs(d["h_scale_t"]))
    # closed-form cross-check of the stored activation: float64, tanh form
    g, u = C[:, :256].astype(np.float64), C[:, 256:].astype(np.float64)
    assert np.all(np.abs(d["h_f32"] - g * 0.5 * (1 + np.tanh(g / 2)) * u) <= 4e-7 * np.abs(g * u) + 1e-37)


def test_qk_norm_rope_fixture(oracle):
    d = np.load(os.path.join(G, "qk_norm_rope_16x512.npz"))
    y = oracle.qk_norm_rope(d["x"], d["qw"], d["kw"], 1e-6, d["cos"], d["sin"], d["pos"], 2, 1)
    assert np.array_equal(y.view(np.uint32), d["y"].view(np.uint32))
    assert np.array_equal(oracle.f32_to_bf16_bits(y), d["y_bf16"])
    yq, ys = oracle.requant_c_1x128(y)
    assert np.array_equal(yq, d["yq"]) and np.array_equal(ys.view(np.uint32), d["y_scale_t"].view(np.uint32))
    assert d["pos"].min() < 0 and d["pos"].max() >= d["cos"].shape[0], "the fixture does not exercise the clamp"
    # closed-form cross-check of the stored result: float64 norm + rotate-half rotation
    x = d["x"].astype(np.float64).reshape(16, 4, 128)
    p = np.clip(d["pos"], 0, d["cos"].shape[0] - 1)
    c, s = d["cos"][p].astype(np.float64), d["sin"][p].astype(np.float64)
    ref = x.copy()
    for h, w in ((0, d["qw"]), (1, d["qw"]), (2, d["kw"])):
        v = x[:, h] / np.sqrt((x[:, h] ** 2).mean(axis=1, keepdims=True) + 1e-6) * w.astype(np.float64)
        ref[:, h, :64] = v[:, :64] * c - v[:, 64:] * s
        ref[:, h, 64:] = v[:, 64:] * c + v[:, :64] * s
    assert np.abs(d["y"].reshape(16, 4, 128) - ref).max() <= 2e-6 * np.abs(ref).max()
