"""The gated-MLP activation fused into the consumer: the down projection takes the fp32 gate_up result G [M, 2K] and runs on
quantise_1x128(silu(G[:, :K]) * G[:, K:]).  The promise is the bits of the two-step route: the same GEMM (same kernel and
split) on the codes and scales the library's SwiGLU quantiser writes from the same G."""
import numpy as np
import pytest
import torch

from helpers import assert_fp8_gemm_close

pytestmark = pytest.mark.gpu
TILES = {"auto": -1, "256x256": 0, "128x256": 1, "256x128": 2, "128x128": 3, "skinny": 8}


def _setup(oracle, M, N, K, seed):
    rng = np.random.default_rng(seed + M + N + K)
    G = (rng.standard_normal((M, 2 * K)) * 1.5).astype(np.float32)
    G[:, ::71] *= 6
    if M > 2:
        G[2, :] = 0  # a row of zeros: h = 0, scales 0, codes 0
    W = (rng.standard_normal((N, K)) * 0.03).astype(np.float32)
    Bq, Bs = oracle.quant_fp8(W, 128, False)
    return G, Bq, Bs


@pytest.mark.parametrize("M,N,K,split", [(1, 2560, 9728, 10), (4, 2560, 9728, 10), (2, 2560, 9728, 4), (4, 2560, 9728, 3), (3, 256, 512, 1),
                                         (4, 384, 4096, 1), (1, 128, 256, 2), (2, 2560, 9728, 0), (16, 2560, 9728, 0), (9, 128, 256, 2)])
@pytest.mark.parametrize("pre", [False, True])
def test_generated_activations_match_the_two_step_route(lib, oracle, M, N, K, split, pre):
    G, Bq, Bs = _setup(oracle, M, N, K, 1)
    dG, dBs = torch.from_numpy(G).cuda(), torch.from_numpy(Bs).cuda()
    dB = torch.from_numpy(Bq).cuda()
    if pre:
        dB = lib.preshuffle_weight(dB)
    ws = torch.full((16 * M * N * 4 + 4 * M * K,), 0xFF, dtype=torch.uint8, device="cuda")
    # two-step: quantise h on the host with the oracle (the kernel's silu uses the hardware's exp2 / rcp, so the codes may
    # differ by a step on a few elements) -> compare the GEMM results with the GEMM bar; and bit for bit against the GPU's
    # own two-step route further down
    hq, hs = oracle.swiglu_requant(G)
    C = torch.empty((M, N), dtype=torch.float32, device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(dG, None, dB, dBs, C, M, N, K, workspace=ws, tile=TILES["skinny"], split_k=split,
                                                                 b_preshuffled=pre, a_swiglu=True)
    torch.cuda.synchronize()
    ref = oracle.fp8_gemm(hq, hs, Bq, Bs, promote=128)
    assert_fp8_gemm_close(C.cpu().numpy(), ref, "a_swiglu vs oracle chain")


@pytest.mark.parametrize("M,N,K,split", [(1, 2560, 9728, 10), (4, 2560, 9728, 10), (3, 256, 1024, 2), (2, 384, 4096, 1), (4, 128, 128, 1)])
def test_bit_identical_to_the_library_quantising_first(lib, oracle, M, N, K, split):
    """M <= 4 generates the activations in the kernel; the same call at a larger M quantises them into the workspace first.
    Rows are independent, so the first M rows of a 32-row call (two-step route) must equal the M-row call bit for bit."""
    G, Bq, Bs = _setup(oracle, 32, N, K, 2)
    dB, dBs = torch.from_numpy(Bq).cuda(), torch.from_numpy(Bs).cuda()
    big = torch.from_numpy(G).cuda()
    small = big[:M].contiguous()
    ws = torch.full((16 * 32 * N * 4 + 4 * 32 * K + 4096,), 0xFF, dtype=torch.uint8, device="cuda")
    for fn, dt in ((lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32, torch.float32),
                   (lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_bf16, torch.bfloat16)):
        C32 = torch.empty((32, N), dtype=dt, device="cuda")
        Cm = torch.empty((M, N), dtype=dt, device="cuda")
        fn(big, None, dB, dBs, C32, 32, N, K, workspace=ws, tile=TILES["skinny"], split_k=split, a_swiglu=True)
        fn(small, None, dB, dBs, Cm, M, N, K, workspace=ws, tile=TILES["skinny"], split_k=split, a_swiglu=True)
        torch.cuda.synchronize()
        assert torch.equal(C32[:M].contiguous().view(torch.uint8), Cm.view(torch.uint8)), dt
    # fused C quantisation as well
    Cq32, Cs32 = torch.empty((32, N), dtype=torch.uint8, device="cuda"), torch.empty((N // 128, 32), device="cuda")
    Cqm, Csm = torch.empty((M, N), dtype=torch.uint8, device="cuda"), torch.empty((N // 128, M), device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(big, None, dB, dBs, Cq32, Cs32, 32, N, K, workspace=ws, tile=TILES["skinny"],
                                                                         split_k=split, a_swiglu=True)
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(small, None, dB, dBs, Cqm, Csm, M, N, K, workspace=ws, tile=TILES["skinny"],
                                                                         split_k=split, a_swiglu=True)
    torch.cuda.synchronize()
    assert torch.equal(Cq32[:M], Cqm) and torch.equal(Cs32[:, :M].contiguous().view(torch.int32), Csm.view(torch.int32))


def test_down_projection_with_the_block_epilogue(lib, oracle):
    """a_swiglu through llmmm_fp8_gemm_add_rmsnorm_quant: == the same call on the SwiGLU-quantised operand."""
    M, N, K = 4, 2560, 9728
    G, Bq, Bs = _setup(oracle, 32, N, K, 3)
    dB, dBs = torch.from_numpy(Bq).cuda(), torch.from_numpy(Bs).cuda()
    big = torch.from_numpy(G).cuda()
    rng = np.random.default_rng(5)
    res = torch.from_numpy(rng.standard_normal((32, N)).astype(np.float32)).cuda().to(torch.bfloat16)
    w = torch.from_numpy(rng.uniform(0.5, 1.5, N).astype(np.float32)).cuda()
    ws = torch.full((16 * 32 * N * 4 + 4 * 32 * K + 4096,), 0xFF, dtype=torch.uint8, device="cuda")
    h32, hm = torch.empty_like(res), torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    q32, s32 = lib.fp8_gemm_add_rmsnorm_quant(big, None, dB, dBs, res, h32, w, 1e-6, 32, N, K, workspace=ws, tile=TILES["skinny"], split_k=10, a_swiglu=True)
    qm, sm = lib.fp8_gemm_add_rmsnorm_quant(big[:M].contiguous(), None, dB, dBs, res[:M].contiguous(), hm, w, 1e-6, M, N, K, workspace=ws,
                                            tile=TILES["skinny"], split_k=10, a_swiglu=True)
    torch.cuda.synchronize()
    assert torch.equal(h32[:M].view(torch.int16), hm.view(torch.int16))
    assert torch.equal(q32[:M], qm) and torch.equal(s32[:, :M].contiguous().view(torch.int32), sm.view(torch.int32))


def test_tile_kernels_quantise_first(lib, oracle):
    M, N, K = 256, 512, 1024
    G, Bq, Bs = _setup(oracle, M, N, K, 4)
    dG, dB, dBs = torch.from_numpy(G).cuda(), torch.from_numpy(Bq).cuda(), torch.from_numpy(Bs).cuda()
    need = int(lib._lib.lib.llmmm_fp8_swiglu_a_workspace(M, N, K))
    assert need >= M * K + (K // 128) * M * 4
    assert int(lib._lib.lib.llmmm_fp8_swiglu_a_workspace(4, 2560, 9728)) == 0
    assert int(lib._lib.lib.llmmm_fp8_swiglu_a_workspace(16, 2560, 9728)) > 0
    ws = torch.full((need + 4 * M * N * 4,), 0xFF, dtype=torch.uint8, device="cuda")
    C = torch.empty((M, N), dtype=torch.float32, device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(dG, None, dB, dBs, C, M, N, K, workspace=ws, a_swiglu=True)
    torch.cuda.synchronize()
    hq, hs = oracle.swiglu_requant(G)
    assert_fp8_gemm_close(C.cpu().numpy(), oracle.fp8_gemm(hq, hs, Bq, Bs, promote=128), "a_swiglu, tile kernel")
    with pytest.raises(RuntimeError, match="workspace"):
        lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(dG, None, dB, dBs, C, M, N, K, workspace=None, a_swiglu=True)


def test_errors(lib):
    M, N, K = 4, 256, 9728  # 76 slices: generated activations need split-K >= 3
    G = torch.zeros((M, 2 * K), device="cuda")
    B = torch.zeros((N, K), dtype=torch.uint8, device="cuda")
    Bs = torch.ones((N // 128, K // 128), device="cuda")
    C = torch.empty((M, N), device="cuda")
    with pytest.raises(RuntimeError, match="split-K >= 3"):
        lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(G, None, B, Bs, C, M, N, K, workspace=torch.empty(1 << 20, dtype=torch.uint8, device="cuda"),
                                                                     tile=TILES["skinny"], split_k=2, a_swiglu=True)
    with pytest.raises(RuntimeError, match="workspace"):
        lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(G, None, B, Bs, C, M, N, K, workspace=None, tile=TILES["skinny"], a_swiglu=True)
    Hq, Hs = torch.empty((M, N // 2), dtype=torch.uint8, device="cuda"), torch.empty((1, M), device="cuda")
    with pytest.raises(RuntimeError, match="both"):
        lib.mm._fp8_gemm(lib._lib.OUT_FP8Q_SWIGLU, G, None, B, Bs, Hq, Hs, M, N, K, torch.empty(1 << 20, dtype=torch.uint8, device="cuda"), -1, 0, None, False, True)
