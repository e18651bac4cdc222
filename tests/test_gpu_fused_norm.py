"""A projection back to the hidden size with the decoder block's epilogue behind it (residual add, RMSNorm, 1x128
quantisation) in one call, through the C ABI.  The fused call promises the bits of its parts: the hidden state equals
T(C32 + residual) with C32 the fp32 output of the plain GEMM run with the same kernel and split, and codes and scales
equal the oracle's RMSNorm + quantiser on that hidden state."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

_TORCH = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}
TILES = {"auto": -1, "256x256": 0, "128x256": 1, "256x128": 2, "128x128": 3, "skinny": 8}


def _operands(oracle, M, N, K, seed):
    rng = np.random.default_rng(seed)
    X = rng.standard_normal((M, K)).astype(np.float32)
    X[:, ::61] *= 12
    W = (rng.standard_normal((N, K)) * 0.03).astype(np.float32)
    Aq, As = oracle.quant_fp8(X, 1, True)
    Bq, Bs = oracle.quant_fp8(W, 128, False)
    res = (rng.standard_normal((M, N)) * 2).astype(np.float32)
    res[:, ::89] *= 15
    w = rng.uniform(0.5, 1.5, N).astype(np.float32)
    return Aq, As, Bq, Bs, res, w


def _check(lib, oracle, M, N, K, dt, tile, split, pre=False, inplace=False, seed=0):
    Aq, As, Bq, Bs, res, w = _operands(oracle, M, N, K, seed + M + N + K)
    dA, dAs, dBs = (torch.from_numpy(a).cuda() for a in (Aq, As, Bs))
    dB = torch.from_numpy(Bq).cuda()
    if pre:
        dB = lib.preshuffle_weight(dB)
    # the plain GEMM with the same kernel and split gives the fp32 values the fused epilogue adds the residual to
    # (both calls get room for 16 planes, so that a split the library picks itself is the same in both)
    ws = torch.full((16 * M * N * 4,), 0xFF, dtype=torch.uint8, device="cuda")
    C = torch.empty((M, N), dtype=torch.float32, device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(dA, dAs, dB, dBs, C, M, N, K, workspace=ws, tile=tile, split_k=split, b_preshuffled=pre)
    ws.fill_(0xFF)
    tres = torch.from_numpy(res).cuda().to(_TORCH[dt])
    res_seen = tres.float().cpu().numpy()
    hidden = tres if inplace else torch.full((M, N), 7.0, dtype=_TORCH[dt], device="cuda")
    q, s = lib.fp8_gemm_add_rmsnorm_quant(dA, dAs, dB, dBs, tres, hidden, torch.from_numpy(w).cuda(), 1e-6, M, N, K, workspace=ws, tile=tile,
                                          split_k=split, b_preshuffled=pre)
    torch.cuda.synchronize()
    h32 = C.cpu().numpy() + res_seen  # one correctly rounded fp32 addition per element, as in the kernel
    want_hidden = torch.from_numpy(h32).to(_TORCH[dt])
    got = hidden.cpu()
    assert torch.equal(got.view(torch.int32 if dt == "f32" else torch.int16), want_hidden.view(torch.int32 if dt == "f32" else torch.int16)), "hidden state differs"
    rq, rs = oracle.rmsnorm_quant(want_hidden.float().numpy(), w, 1e-6)
    assert np.array_equal(s.cpu().numpy().view(np.uint32), rs.view(np.uint32)), "scales differ"
    assert np.array_equal(q.cpu().numpy(), rq), "codes differ"
    return dA, dAs, dB, dBs, hidden, w, q, s


# the weight-streaming kernel (M <= 128): O and down projections of the decode shapes, split and unsplit, ragged M
@pytest.mark.parametrize("M,N,K,split", [(1, 2560, 4096, 0), (16, 2560, 9728, 0), (5, 2560, 4096, 1), (16, 2560, 4096, 4), (77, 2560, 9728, 0),
                                         (128, 2560, 4096, 0), (3, 128, 128, 0), (9, 10240, 256, 2), (33, 3072 + 128, 512, 0)])
@pytest.mark.parametrize("dt", ["bf16", "f32"])
def test_streaming_kernel(lib, oracle, M, N, K, split, dt):
    _check(lib, oracle, M, N, K, dt, TILES["skinny"], split)


# the tile kernels in plane mode (one plane and split-K)
@pytest.mark.parametrize("M,N,K,tile,split", [(256, 2560, 4096, "auto", 0), (128, 2560, 1024, "128x128", 1), (128, 2560, 1024, "128x128", 3),
                                              (512, 2560, 512, "256x256", 0), (256, 2560, 9728, "128x256", 2), (2048, 2560, 256, "auto", 0)])
@pytest.mark.parametrize("dt", ["bf16", "f16"])
def test_tile_kernels(lib, oracle, M, N, K, tile, split, dt):
    _check(lib, oracle, M, N, K, dt, TILES[tile], split)


def test_unsplit_tile_kernels_add_the_residual_themselves(lib, oracle):
    """Without split the tile kernel's epilogue adds the residual and the norm kernel follows: no planes, no workspace
    (a 16-byte dummy here), the same bits."""
    assert lib._lib.lib.llmmm_fp8_gemm_add_rmsnorm_quant_workspace(2048, 2560, 4096) == 0
    for dt in ("f32", "bf16", "f16"):
        for tile in ("128x128", "256x128", "128x256", "256x256"):
            M, N, K = 256, 512, 384
            Aq, As, Bq, Bs, res, w = _operands(oracle, M, N, K, 3)
            dA, dAs, dB, dBs = (torch.from_numpy(a).cuda() for a in (Aq, As, Bq, Bs))
            C = torch.empty((M, N), dtype=torch.float32, device="cuda")
            lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(dA, dAs, dB, dBs, C, M, N, K, tile=TILES[tile], split_k=1)
            hidden = torch.from_numpy(res).cuda().to(_TORCH[dt])  # in place
            seen = hidden.float().cpu().numpy()
            tiny = torch.empty(16, dtype=torch.uint8, device="cuda")
            q, s = lib.fp8_gemm_add_rmsnorm_quant(dA, dAs, dB, dBs, hidden, hidden, torch.from_numpy(w).cuda(), 1e-6, M, N, K, workspace=tiny,
                                                  tile=TILES[tile], split_k=1)
            torch.cuda.synchronize()
            want = torch.from_numpy(C.cpu().numpy() + seen).to(_TORCH[dt])
            view = torch.int32 if dt == "f32" else torch.int16
            assert torch.equal(hidden.cpu().view(view), want.view(view)), (dt, tile)
            rq, rs = oracle.rmsnorm_quant(want.float().numpy(), w, 1e-6)
            assert np.array_equal(s.cpu().numpy().view(np.uint32), rs.view(np.uint32)) and np.array_equal(q.cpu().numpy(), rq), (dt, tile)


def test_preshuffled_weights_and_in_place_residual(lib, oracle):
    _check(lib, oracle, 16, 2560, 4096, "bf16", TILES["auto"], 0, pre=True, inplace=True)
    _check(lib, oracle, 256, 2560, 1024, "bf16", TILES["auto"], 0, pre=True, inplace=True)


def test_equals_the_separate_calls(lib, oracle):
    """The library's own choice of kernel: fused call == GEMM (fp32) + host add + rmsnorm_quantize_activation, bit for bit."""
    M, N, K = 16, 2560, 9728
    dA, dAs, dB, dBs, hidden, w, q, s = _check(lib, oracle, M, N, K, "bf16", TILES["auto"], 0, seed=5)
    q2, s2 = lib.rmsnorm_quantize_activation(hidden, torch.from_numpy(w).cuda(), 1e-6)
    torch.cuda.synchronize()
    assert torch.equal(q, q2) and torch.equal(s.view(torch.int32), s2.view(torch.int32))


def test_workspace_and_errors(lib):
    M, N, K = 48, 2560, 4096  # (up to 16 rows this shape runs in column strips, which need no workspace)
    need = lib._lib.lib.llmmm_fp8_gemm_add_rmsnorm_quant_workspace(M, N, K)
    assert need >= M * N * 4 and need % (M * N * 4) == 0
    A = torch.zeros((M, K), dtype=torch.uint8, device="cuda")
    As = torch.ones((K // 128, M), device="cuda")
    B = torch.zeros((N, K), dtype=torch.uint8, device="cuda")
    Bs = torch.ones((N // 128, K // 128), device="cuda")
    res = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    w = torch.ones(N, device="cuda")
    small = torch.empty(M * N * 4 - 16, dtype=torch.uint8, device="cuda")
    with pytest.raises(RuntimeError, match="workspace"):
        lib.fp8_gemm_add_rmsnorm_quant(A, As, B, Bs, res, res, w, 1e-6, M, N, K, workspace=small)
    # one plane is enough for the library's choice: the split shrinks to the workspace
    one = torch.empty(M * N * 4, dtype=torch.uint8, device="cuda")
    q, s = lib.fp8_gemm_add_rmsnorm_quant(A, As, B, Bs, res, res, w, 1e-6, M, N, K, workspace=one)
    torch.cuda.synchronize()
    assert int(q.max()) == 0 and float(s.abs().max()) == 0.0
    with pytest.raises(RuntimeError, match="workspace"):
        lib.fp8_gemm_add_rmsnorm_quant(A, As, B, Bs, res, res, w, 1e-6, M, N, K, workspace=one, split_k=2)
    with pytest.raises(RuntimeError, match="T is not supported."):
        lib.fp8_gemm_add_rmsnorm_quant(A, As, B, Bs, res.double(), res.double(), w, 1e-6, M, N, K)
    with pytest.raises(RuntimeError, match="10240"):
        lib.fp8_gemm_add_rmsnorm_quant(torch.zeros((M, 128), dtype=torch.uint8, device="cuda"), torch.ones((1, M), device="cuda"),
                                       torch.zeros((10368, 128), dtype=torch.uint8, device="cuda"), torch.ones((81, 1), device="cuda"),
                                       torch.zeros((M, 10368), dtype=torch.bfloat16, device="cuda"), torch.zeros((M, 10368), dtype=torch.bfloat16, device="cuda"),
                                       torch.ones(10368, device="cuda"), 1e-6, M, 10368, 128)
