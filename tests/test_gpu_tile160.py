"""The 128 x 160 tile of the FP8 GEMM (outputs without 1x128 groups: fp32, bf16, residual add).  Its waves straddle two
weight-scale blocks, at every alignment (tile columns start 0, 32, 64 or 96 columns into a block).  The K loop adds the same
slices in the same order as every other tile, so its fp32 result must equal the 128 x 128 tile's bit for bit."""
import numpy as np
import pytest
import torch

from helpers import assert_fp8_gemm_close

pytestmark = pytest.mark.gpu
T128, T160 = 3, 5


def _inputs(oracle, M, N, K, seed=0):
    rng = np.random.default_rng(seed + M + N + K)
    X = rng.standard_normal((M, K)).astype(np.float32)
    X[:, ::41] *= 9
    W = (rng.standard_normal((N, K)) * 0.03).astype(np.float32)
    Bq, Bs = oracle.quant_fp8(W, 128, False)
    # weight-scale blocks of very different size: taking the wrong block for a fragment would be off by a factor
    Bs = (Bs * (1 + np.arange(Bs.shape[0], dtype=np.float32))[:, None]).astype(np.float32)
    Aq, As = oracle.quant_fp8(X, 1, True)
    return Aq, As, Bq, Bs


@pytest.mark.parametrize("M,N,K,split,pre", [(128, 640, 128, 1, False), (128, 1280, 256, 1, True), (256, 2560, 512, 1, True), (128, 640, 1024, 3, False),
                                             (384, 640, 384, 1, False), (128, 2560, 4096, 2, False), (512, 1920, 256, 1, False)])
def test_matches_the_oracle_and_the_128x128_tile(lib, oracle, M, N, K, split, pre):
    Aq, As, Bq, Bs = _inputs(oracle, M, N, K)
    dA, dAs, dBs = (torch.from_numpy(a).cuda() for a in (Aq, As, Bs))
    dB = torch.from_numpy(Bq).cuda()
    if pre:
        dB = lib.preshuffle_weight(dB)
    ws = torch.full((8 * M * N * 4,), 0xFF, dtype=torch.uint8, device="cuda")
    C5 = torch.full((M, N), float("nan"), device="cuda")
    C3 = torch.empty((M, N), device="cuda")
    kw = dict(workspace=ws, split_k=split, b_preshuffled=pre)
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(dA, dAs, dB, dBs, C5, M, N, K, tile=T160, **kw)
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(dA, dAs, dB, dBs, C3, M, N, K, tile=T128, **kw)
    Y5 = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_bf16(dA, dAs, dB, dBs, Y5, M, N, K, tile=T160, **kw)
    torch.cuda.synchronize()
    assert_fp8_gemm_close(C5.cpu().numpy(), oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128), "128x160 tile")
    assert torch.equal(C5.view(torch.int32), C3.view(torch.int32)), "differs from the 128 x 128 tile"
    assert torch.equal(Y5.view(torch.int16), C5.to(torch.bfloat16).view(torch.int16)), "bf16 != RNE(fp32)"


@pytest.mark.parametrize("dt", ["f32", "bf16", "f16"])
def test_residual_add_epilogue(lib, oracle, dt):
    """Through llmmm_fp8_gemm_add_rmsnorm_quant: hidden == T(C32 + residual), codes and scales == the oracle's norm + quantiser."""
    T = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}[dt]
    M, N, K = 256, 1280, 384
    Aq, As, Bq, Bs = _inputs(oracle, M, N, K, 5)
    dA, dAs, dB, dBs = (torch.from_numpy(a).cuda() for a in (Aq, As, Bq, Bs))
    rng = np.random.default_rng(9)
    res = torch.from_numpy((rng.standard_normal((M, N)) * 2).astype(np.float32)).cuda().to(T)
    w = rng.uniform(0.5, 1.5, N).astype(np.float32)
    C = torch.empty((M, N), device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(dA, dAs, dB, dBs, C, M, N, K, tile=T160, split_k=1)
    hid = torch.empty_like(res)
    q, s = lib.fp8_gemm_add_rmsnorm_quant(dA, dAs, dB, dBs, res, hid, torch.from_numpy(w).cuda(), 1e-6, M, N, K, tile=T160, split_k=1)
    torch.cuda.synchronize()
    want = torch.from_numpy(C.cpu().numpy() + res.float().cpu().numpy()).to(T)
    view = torch.int32 if dt == "f32" else torch.int16
    assert torch.equal(hid.cpu().view(view), want.view(view))
    rq, rs = oracle.rmsnorm_quant(want.float().numpy(), w, 1e-6)
    assert np.array_equal(q.cpu().numpy(), rq) and np.array_equal(s.cpu().numpy().view(np.uint32), rs.view(np.uint32))


def test_chosen_where_it_saves_a_round_and_refused_for_grouped_outputs(lib):
    from llmmm_amd import _lib
    # 2560 columns at M = 2048: 320 tiles of 128 x 128 (two rounds of 256 CUs) against 256 of 128 x 160
    assert lib.query_config(_lib.OUT_BF16, 2048, 2560, 4096)[0] == T160
    assert lib.query_config(_lib.OUT_F32, 2048, 2560, 9728)[0] == T160
    assert lib.query_config(_lib.OUT_FP8Q, 2048, 2560, 4096)[0] != T160   # the fused quantisation needs whole 1x128 groups
    assert lib.query_config(_lib.OUT_BF16, 1024, 2560, 4096)[0] != T160   # one round either way
    M, N, K = 128, 640, 128
    A = torch.zeros((M, K), dtype=torch.uint8, device="cuda")
    As = torch.ones((1, M), device="cuda")
    B = torch.zeros((N, K), dtype=torch.uint8, device="cuda")
    Bs = torch.ones((N // 128, 1), device="cuda")
    Cq, Cs = torch.empty((M, N), dtype=torch.uint8, device="cuda"), torch.empty((N // 128, M), device="cuda")
    with pytest.raises(RuntimeError, match="no fp8 output"):
        lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(A, As, B, Bs, Cq, Cs, M, N, K, tile=T160)
    C = torch.empty((M, 256), device="cuda")
    with pytest.raises(RuntimeError, match="not aligned"):
        lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(A, As, torch.zeros((256, K), dtype=torch.uint8, device="cuda"), torch.ones((2, 1), device="cuda"), C,
                                                                     M, 256, K, tile=T160)
    h = torch.zeros((256, 640), dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError, match="unknown tile"):
        lib.fp16_gemm(h[:, :256].contiguous(), torch.zeros((256, 640), dtype=torch.float16, device="cuda"), tile=T160)
