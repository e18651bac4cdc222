"""More than one round of 256 x 256 tiles with a partly filled last round: the launch gives the columns of the whole rounds
to 256 x 256 tiles and the rest to 128 x 256 tiles (one kernel).  Every tile adds the same 128-K slices in the same order,
so the results must equal the 128 x 128 tiles' bit for bit, in every output kind, across the seam between the two ranges."""
import numpy as np
import pytest
import torch

from helpers import assert_fp8_gemm_close

pytestmark = pytest.mark.gpu
T256, T128x256, T128 = 0, 1, 3


def _inputs(oracle, M, N, K, seed=0):
    rng = np.random.default_rng(seed + M + N + K)
    X = rng.standard_normal((M, K)).astype(np.float32)
    X[:, ::29] *= 7
    W = (rng.standard_normal((N, K)) * 0.03).astype(np.float32)
    Aq, As = oracle.quant_fp8(X, 1, True)
    Bq, Bs = oracle.quant_fp8(W, 128, False)
    Bs = (Bs * (1 + (np.arange(Bs.shape[0], dtype=np.float32) % 7))[:, None]).astype(np.float32)  # column blocks told apart
    return Aq, As, Bq, Bs


# (M, N): 260 tiles = 256 + 4 columns' worth; 608 tiles (the Qwen3-4B gate_up shape at M = 2048); 2 x 129 = 258
@pytest.mark.parametrize("M,N,K,pre,check_oracle", [(512, 33280, 256, False, True), (2048, 19456, 384, True, False), (512, 33024, 128, True, False)])
def test_equals_the_128x128_tiles(lib, oracle, M, N, K, pre, check_oracle):
    Aq, As, Bq, Bs = _inputs(oracle, M, N, K)
    dA, dAs, dBs = (torch.from_numpy(a).cuda() for a in (Aq, As, Bs))
    dB = torch.from_numpy(Bq).cuda()
    if pre:
        dB = lib.preshuffle_weight(dB)
    kw = dict(split_k=1, b_preshuffled=pre)
    C0 = torch.full((M, N), float("nan"), device="cuda")
    C3 = torch.empty((M, N), device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(dA, dAs, dB, dBs, C0, M, N, K, tile=T256, **kw)
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(dA, dAs, dB, dBs, C3, M, N, K, tile=T128, **kw)
    torch.cuda.synchronize()
    assert torch.equal(C0.view(torch.int32), C3.view(torch.int32)), "fp32 differs from the 128 x 128 tiles"
    if check_oracle:
        rows = np.r_[0:40, M - 40:M]
        assert_fp8_gemm_close(C0.cpu().numpy()[rows], oracle.fp8_gemm(Aq[rows], np.ascontiguousarray(As[:, rows]), Bq, Bs, promote=128), "hybrid tiles")
    del C3
    Y0 = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_bf16(dA, dAs, dB, dBs, Y0, M, N, K, tile=T256, **kw)
    torch.cuda.synchronize()
    assert torch.equal(Y0.view(torch.int16), C0.to(torch.bfloat16).view(torch.int16)), "bf16 != RNE(fp32)"
    del Y0
    Q0 = torch.full((M, N), 0x7F, dtype=torch.uint8, device="cuda")
    S0 = torch.full((N // 128, M), float("nan"), device="cuda")
    Q3, S3 = torch.empty_like(Q0), torch.empty_like(S0)
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(dA, dAs, dB, dBs, Q0, S0, M, N, K, tile=T256, **kw)
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(dA, dAs, dB, dBs, Q3, S3, M, N, K, tile=T128, **kw)
    torch.cuda.synchronize()
    assert torch.equal(Q0, Q3) and torch.equal(S0.view(torch.int32), S3.view(torch.int32)), "fused quantisation differs"
    del Q0, Q3
    H0 = torch.full((M, N // 2), 0x7F, dtype=torch.uint8, device="cuda")
    G0 = torch.full((N // 256, M), float("nan"), device="cuda")
    H1, G1 = torch.empty_like(H0), torch.empty_like(G0)
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__swiglu__C_1x128__output_fp8(dA, dAs, dB, dBs, H0, G0, M, N, K, tile=T256, **kw)
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__swiglu__C_1x128__output_fp8(dA, dAs, dB, dBs, H1, G1, M, N, K, tile=T128x256, **kw)
    torch.cuda.synchronize()
    assert torch.equal(H0, H1) and torch.equal(G0.view(torch.int32), G1.view(torch.int32)), "SwiGLU output differs from the 128 x 256 tiles"


def test_head_and_residual_epilogues_across_the_seam(lib, oracle):
    """The QKV + per-head norm + RoPE and the residual-add epilogues in the two-shape launch against the 128 x 128 tiles."""
    g = lambda a: torch.from_numpy(a).cuda()
    rng = np.random.default_rng(5)
    # 16 x 24 = 384 tiles of 256 x 256: 256 in large tiles, the last 8 tile columns (16 of 48 heads) in 128 x 256 tiles
    M, K, n_q, n_kv = 4096, 256, 32, 8
    N = (n_q + 2 * n_kv) * 128
    Aq, As, Bq, Bs = _inputs(oracle, M, N, K, 1)
    qw, kw = rng.uniform(0.5, 1.5, 128).astype(np.float32), rng.uniform(0.5, 1.5, 128).astype(np.float32)
    ang = rng.uniform(0, 6.28, (64, 64)).astype(np.float32)
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    pos = rng.integers(0, 64, M).astype(np.int32)
    args = (g(Aq), g(As), g(Bq), g(Bs), g(qw), g(kw), 1e-6, g(cos), g(sin), g(pos), n_q, n_kv, M, N, K)
    y0 = lib.fp8_gemm_qkv_rope(*args, tile=T256, split_k=1)
    y3 = lib.fp8_gemm_qkv_rope(*args, tile=T128, split_k=1)
    q0, s0 = lib.fp8_gemm_qkv_rope(*args, out_fp8=True, tile=T256, split_k=1)
    q3, s3 = lib.fp8_gemm_qkv_rope(*args, out_fp8=True, tile=T128, split_k=1)
    torch.cuda.synchronize()
    assert torch.equal(y0.view(torch.int16), y3.view(torch.int16)) and torch.equal(q0, q3) and torch.equal(s0.view(torch.int32), s3.view(torch.int32))
    # 32 x 10 = 320 tiles: 256 + 2 tile columns; hidden = bf16(C + residual), then norm + quantiser
    M, N, K = 8192, 2560, 256
    Aq, As, Bq, Bs = _inputs(oracle, M, N, K, 2)
    res = torch.from_numpy(rng.standard_normal((M, N)).astype(np.float32)).cuda().to(torch.bfloat16)
    w = g(rng.uniform(0.5, 1.5, N).astype(np.float32))
    h0, h3 = torch.empty_like(res), torch.empty_like(res)
    qa, sa = lib.fp8_gemm_add_rmsnorm_quant(g(Aq), g(As), g(Bq), g(Bs), res, h0, w, 1e-6, M, N, K, tile=T256, split_k=1)
    qb, sb = lib.fp8_gemm_add_rmsnorm_quant(g(Aq), g(As), g(Bq), g(Bs), res, h3, w, 1e-6, M, N, K, tile=T128, split_k=1)
    torch.cuda.synchronize()
    assert torch.equal(h0.view(torch.int16), h3.view(torch.int16)) and torch.equal(qa, qb) and torch.equal(sa.view(torch.int32), sb.view(torch.int32))


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("M,N,K,bt", [(512, 33280, 96, False), (2048, 19456, 64, True), (512, 33024, 80, False)])
def test_fp16_gemm_two_shape_launch(lib, oracle, dt, M, N, K, bt):
    """The FP16 / BF16 GEMM takes the same launch form; every tile adds the K steps in the same order, so the result must
    equal the 128 x 128 tiles' bit for bit (K = 80, 96: the K-tail path as well)."""
    T = torch.float16 if dt == "f16" else torch.bfloat16
    rng = np.random.default_rng(M + N + K)
    A = torch.from_numpy(rng.uniform(-1, 1, (M, K)).astype(np.float32)).cuda().to(T)
    B = torch.from_numpy(rng.uniform(-1, 1, (K, N)).astype(np.float32)).cuda().to(T)
    Bx = B.t().contiguous() if bt else B
    C0 = torch.full((M, N), float("nan"), dtype=T, device="cuda")
    C3 = torch.empty((M, N), dtype=T, device="cuda")
    lib.fp16_gemm(A, Bx, C0, b_transposed=bt, tile=T256)
    lib.fp16_gemm(A, Bx, C3, b_transposed=bt, tile=T128)
    torch.cuda.synchronize()
    assert torch.equal(C0.view(torch.int16), C3.view(torch.int16))
    rows = np.r_[0:16, M - 16:M]
    ref = oracle.kahan_gemm(A[rows].float().cpu().numpy(), B.float().cpu().numpy())
    got = C0[rows].float().cpu().numpy()
    assert np.all(np.abs(got - ref) <= 1e-3 + 1e-2 * np.abs(ref))
