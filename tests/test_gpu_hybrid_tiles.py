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
