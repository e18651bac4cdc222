"""The decoder block's epilogue fused into the consumer: a projection stops at its fp32 planes (llmmm_fp8_gemm_planes), and the
next projection's kernel sums them, adds the residual, stores the hidden state, normalises and quantises its own A operand.
The promise is the bits of the producer-side route: llmmm_fp8_gemm_add_rmsnorm_quant with the same kernel and split, followed
by the same second GEMM on the codes and scales it returns."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
SKINNY = 8
_T = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}


def _weights(oracle, rng, N, K, scale=0.03):
    q, s = oracle.quant_fp8((rng.standard_normal((N, K)) * scale).astype(np.float32), 128, False)
    return torch.from_numpy(q).cuda(), torch.from_numpy(s).cuda()


def _case(lib, oracle, M, H, K1, N2, split1, split2, dt, seed=0, rope=False):
    rng = np.random.default_rng(seed + M + H + K1 + N2)
    X = rng.standard_normal((M, K1)).astype(np.float32)
    X[:, ::37] *= 8
    Aq, As = oracle.quant_fp8(X, 1, True)
    dA, dAs = torch.from_numpy(Aq).cuda(), torch.from_numpy(As).cuda()
    W1, W1s = _weights(oracle, rng, H, K1)
    W2, W2s = _weights(oracle, rng, N2, H)
    res = torch.from_numpy((rng.standard_normal((M, H)) * 2).astype(np.float32)).cuda().to(_T[dt])
    w = torch.from_numpy(rng.uniform(0.5, 1.5, H).astype(np.float32)).cuda()
    ws = torch.full((16 * M * max(H, N2) * 4 + (1 << 16),), 0xFF, dtype=torch.uint8, device="cuda")
    # producer-side route
    hid_ref = torch.empty_like(res)
    q, s = lib.fp8_gemm_add_rmsnorm_quant(dA, dAs, W1, W1s, res, hid_ref, w, 1e-6, M, H, K1, workspace=ws, tile=SKINNY, split_k=split1)
    # consumer-side route
    planes, S = lib.fp8_gemm_planes(dA, dAs, W1, W1s, M, H, K1, tile=SKINNY, split_k=split1,
                                    planes=torch.full((16, M, H), float("nan"), dtype=torch.float32, device="cuda"))
    assert S == max(split1, 1) or split1 == 0
    hid = torch.full_like(res, 3.0)
    a2 = lib.PlanesRmsnorm(planes, S, res, hid, w, 1e-6)
    if rope:
        n_kv = 1
        n_q = N2 // 128 - 2
        cos = torch.from_numpy(np.cos(np.arange(64 * 32).reshape(32, 64) * 0.01).astype(np.float32)).cuda()
        sin = torch.from_numpy(np.sin(np.arange(64 * 32).reshape(32, 64) * 0.01).astype(np.float32)).cuda()
        pos = torch.arange(M, dtype=torch.int32, device="cuda")
        hw = torch.ones(128, device="cuda")
        ref = lib.fp8_gemm_qkv_rope(q, s, W2, W2s, hw, hw, 1e-6, cos, sin, pos, n_q, n_kv, M, N2, H, workspace=ws, tile=SKINNY, split_k=split2)
        ws.fill_(0xFF)
        got = lib.fp8_gemm_qkv_rope(a2, None, W2, W2s, hw, hw, 1e-6, cos, sin, pos, n_q, n_kv, M, N2, H, workspace=ws, tile=SKINNY, split_k=split2)
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), ref.view(torch.int16)), "second GEMM (rope) differs"
    else:
        ref = torch.empty((M, N2), dtype=torch.float32, device="cuda")
        got = torch.empty((M, N2), dtype=torch.float32, device="cuda")
        lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(q, s, W2, W2s, ref, M, N2, H, workspace=ws, tile=SKINNY, split_k=split2)
        ws.fill_(0xFF)
        lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(a2, None, W2, W2s, got, M, N2, H, workspace=ws, tile=SKINNY, split_k=split2)
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int32), ref.view(torch.int32)), "second GEMM differs"
    view = torch.int32 if dt == "f32" else torch.int16
    assert torch.equal(hid.view(view), hid_ref.view(view)), "hidden state differs"


# Qwen3-4B: O projection (K = 4096, split 8) -> gate_up (N = 19456, no split); down (K = 9728, split 10) -> QKV (N = 6144, split 5)
@pytest.mark.parametrize("M", [1, 2, 3, 4])
@pytest.mark.parametrize("dt", ["bf16", "f32"])
def test_generated_in_the_consumer_kernel(lib, oracle, M, dt):
    _case(lib, oracle, M, 2560, 4096, 19456, 8, 1, dt)
    _case(lib, oracle, M, 2560, 9728, 6144, 10, 5, dt)


@pytest.mark.parametrize("M,H,K1,N2,s1,s2,dt", [(1, 128, 128, 128, 1, 1, "f16"), (4, 3072, 256, 256, 2, 3, "f16"), (2, 384, 512, 384, 4, 1, "bf16"),
                                                (3, 1024, 1024, 512, 0, 0, "f32")])
def test_small_and_odd_shapes(lib, oracle, M, H, K1, N2, s1, s2, dt):
    _case(lib, oracle, M, H, K1, N2, s1, s2, dt, seed=3)


def test_rope_consumer(lib, oracle):
    _case(lib, oracle, 1, 2560, 9728, 6144, 10, 5, "bf16", rope=True)
    _case(lib, oracle, 4, 2560, 9728, 6144, 10, 5, "bf16", rope=True)


@pytest.mark.parametrize("M,H", [(8, 2560), (16, 2560), (2, 4096)])
def test_larger_shapes_quantise_first(lib, oracle, M, H):
    """M > 4 or K > 3072: the library runs the fused reduce + norm + quantise kernel into the workspace; same bits."""
    _case(lib, oracle, M, H, 1024, 512, 4, 2, "bf16", seed=7)


def test_errors(lib, oracle):
    M, H, K1, N2 = 2, 256, 256, 256
    rng = np.random.default_rng(0)
    W1, W1s = _weights(oracle, rng, H, K1)
    W2, W2s = _weights(oracle, rng, N2, H)
    A = torch.zeros((M, K1), dtype=torch.uint8, device="cuda")
    As = torch.ones((K1 // 128, M), device="cuda")
    planes, S = lib.fp8_gemm_planes(A, As, W1, W1s, M, H, K1, tile=SKINNY, split_k=2)
    assert S == 2
    res = torch.zeros((M, H), dtype=torch.bfloat16, device="cuda")
    w = torch.ones(H, device="cuda")
    C = torch.empty((M, N2), device="cuda")
    # an in-place hidden state cannot be generated by every workgroup: the quantise-first route takes over and needs its scratch
    with pytest.raises(RuntimeError, match="workspace"):
        lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(lib.PlanesRmsnorm(planes, S, res, res, w, 1e-6), None, W2, W2s, C, M, N2, H, tile=SKINNY)
    with pytest.raises(RuntimeError, match="splits"):
        lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(lib.PlanesRmsnorm(planes, 0, res, torch.empty_like(res), w, 1e-6), None, W2, W2s, C, M, N2, H,
                                                                     tile=SKINNY)
    # planes buffer too small for an explicit split
    with pytest.raises(RuntimeError, match="workspace"):
        lib.fp8_gemm_planes(A, As, W1, W1s, M, H, K1, tile=SKINNY, split_k=2, planes=torch.empty((1, M, H), device="cuda"))
    # zero operands: hidden == residual, codes 0
    hid = torch.full_like(res, 5.0)
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(lib.PlanesRmsnorm(planes, S, res, hid, w, 1e-6), None, W2, W2s, C, M, N2, H, tile=SKINNY)
    torch.cuda.synchronize()
    assert float(hid.float().abs().max()) == 0.0 and float(C.abs().max()) == 0.0


def test_in_place_hidden_state_falls_back_to_the_two_kernel_route(lib, oracle):
    M, H, K1, N2 = 2, 2560, 1024, 512
    rng = np.random.default_rng(11)
    Aq, As = oracle.quant_fp8(rng.standard_normal((M, K1)).astype(np.float32), 1, True)
    dA, dAs = torch.from_numpy(Aq).cuda(), torch.from_numpy(As).cuda()
    W1, W1s = _weights(oracle, rng, H, K1)
    W2, W2s = _weights(oracle, rng, N2, H)
    res = torch.from_numpy(rng.standard_normal((M, H)).astype(np.float32)).cuda().to(torch.bfloat16)
    w = torch.from_numpy(rng.uniform(0.5, 1.5, H).astype(np.float32)).cuda()
    planes, S = lib.fp8_gemm_planes(dA, dAs, W1, W1s, M, H, K1, tile=SKINNY, split_k=4)
    ws = torch.full((1 << 20,), 0xFF, dtype=torch.uint8, device="cuda")
    out_of_place, in_place = torch.empty((M, N2), device="cuda"), torch.empty((M, N2), device="cuda")
    hid = torch.empty_like(res)
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(lib.PlanesRmsnorm(planes, S, res, hid, w, 1e-6), None, W2, W2s, out_of_place, M, N2, H,
                                                                 workspace=ws, tile=SKINNY, split_k=1)
    res2 = res.clone()
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(lib.PlanesRmsnorm(planes, S, res2, res2, w, 1e-6), None, W2, W2s, in_place, M, N2, H,
                                                                 workspace=ws, tile=SKINNY, split_k=1)
    torch.cuda.synchronize()
    assert torch.equal(res2.view(torch.int16), hid.view(torch.int16))
    assert torch.equal(in_place.view(torch.int32), out_of_place.view(torch.int32))
