"""RMSNorm fused in front of the 1x128 activation quantiser, through the C ABI, against the oracle.  The kernel
takes the sum of squares in the order the oracle documents, and every other operation is a correctly rounded IEEE
one, so codes and scales are compared bit for bit."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


# both kernels (a workgroup per row with 3 or 10 chunks per thread for K <= 10240, a wavefront per row above) must
# give the oracle's bits
@pytest.mark.parametrize("M,K", [(1, 2560), (16, 2560), (5, 128), (77, 4096), (2048, 2560), (33, 9728), (3, 384), (520, 4096), (600, 9728),
                                 (513, 128), (12, 10240 + 128), (70, 16384)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_bit_exact_against_oracle(lib, oracle, M, K, dtype):
    rng = np.random.default_rng(M * 7 + K)
    x = (rng.standard_normal((M, K)) * 3).astype(np.float32)
    x[:, ::97] *= 20
    if M > 2:
        x[2, :] = 0  # a zero row: eps keeps r finite, y = 0, scales 0, codes 0
    w = rng.uniform(0.5, 1.5, K).astype(np.float32)
    tx = torch.from_numpy(x).cuda().to(dtype)
    x_in = tx.float().cpu().numpy()  # the values the kernel sees
    q, s = lib.rmsnorm_quantize_activation(tx, torch.from_numpy(w).cuda(), 1e-6)
    torch.cuda.synchronize()
    rq, rs = oracle.rmsnorm_quant(x_in, w, 1e-6)
    assert np.array_equal(s.cpu().numpy().view(np.uint32), rs.view(np.uint32)), "scales differ"
    assert np.array_equal(q.cpu().numpy(), rq), "codes differ"


def test_feeds_the_gemm(lib, oracle):
    """End to end: rmsnorm + quant on the GPU, then the FP8 GEMM, against the oracle's chain."""
    from helpers import assert_fp8_gemm_close
    M, N, K = 16, 512, 1024
    rng = np.random.default_rng(9)
    x = rng.standard_normal((M, K)).astype(np.float32)
    w = rng.uniform(0.5, 1.5, K).astype(np.float32)
    W = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    Bq, Bs = oracle.quant_fp8(W, 128, False)
    Aq, As = lib.rmsnorm_quantize_activation(torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda(), 1e-6)
    C = torch.empty((M, N), dtype=torch.float32, device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(Aq, As, torch.from_numpy(Bq).cuda(), torch.from_numpy(Bs).cuda(), C, M, N, K)
    torch.cuda.synchronize()
    rq, rs = oracle.rmsnorm_quant(x, w, 1e-6)
    assert_fp8_gemm_close(C.cpu().numpy(), oracle.fp8_gemm(rq, rs, Bq, Bs, promote=128), "rmsnorm -> gemm")


def test_errors(lib):
    x = torch.zeros((4, 100), device="cuda")
    with pytest.raises(RuntimeError, match="M or N or K are not aligned."):
        lib.rmsnorm_quantize_activation(x, torch.ones(100, device="cuda"), 1e-6)
    with pytest.raises(RuntimeError, match="T is not supported."):
        lib.rmsnorm_quantize_activation(torch.zeros((4, 128), device="cuda", dtype=torch.float64), torch.ones(128, device="cuda"), 1e-6)
