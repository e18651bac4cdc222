"""Library-chosen configurations over a seeded spread of shapes: whatever tile, split count, pipeline depth or
K-chunking the heuristics pick -- with the workspace the library asks for, and with none -- every output kind
must meet its bar against the oracle.  (The explicit-configuration tests live in test_gpu_fp8.py,
test_gpu_swiglu.py and test_gpu_layout.py; this file guards the selection logic in between.)"""
import numpy as np
import pytest
import torch

from helpers import assert_fp8_gemm_close, assert_fused_close, fp8_inputs

pytestmark = pytest.mark.gpu


def _shapes():
    rng = np.random.default_rng(20250101)
    out = []
    small_m = [1, 2, 7, 16, 17, 31, 32, 48, 64, 65, 100, 127, 128]
    for i in range(26):
        M = int(small_m[i % len(small_m)])
        N = int(rng.integers(1, 9)) * 256
        K = int(rng.integers(1, 25)) * 128
        out.append((M, N, K))
    for i in range(10):
        M = int(rng.integers(1, 5)) * 128
        N = int(rng.integers(1, 7)) * 256
        K = int(rng.integers(1, 17)) * 128
        out.append((M, N, K))
    out += [(1, 256, 9728), (16, 512, 9728), (128, 256, 9728), (64, 2560, 128), (128, 2560, 256), (256, 256, 6144)]
    return out


@pytest.mark.parametrize("M,N,K", _shapes())
@pytest.mark.parametrize("with_ws", [True, False])
def test_auto_configuration(lib, oracle, M, N, K, with_ws):
    Aq, As, Bq, Bs = fp8_inputs(oracle, M, N, K, seed=M * 131 + N + K)
    Bs = Bs.copy()
    Bs[: N // 256] *= np.float32(40.0)  # gate half: leaves silu's linear range
    ref = oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128)
    t = [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in (Aq, As, Bq, Bs)]
    what = "auto M=%d N=%d K=%d ws=%s" % (M, N, K, with_ws)

    def ws(kind):
        return lib.make_workspace(kind, M, N, K) if with_ws else None

    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    Cb = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    Cq = torch.full((M, N), 0x55, dtype=torch.uint8, device="cuda")
    Cs = torch.full((N // 128, M), -1.0, dtype=torch.float32, device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(*t, C, M, N, K, workspace=ws(0))
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_bf16(*t, Cb, M, N, K, workspace=ws(1))
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(*t, Cq, Cs, M, N, K, workspace=ws(2))
    torch.cuda.synchronize()
    C = C.cpu().numpy()
    assert_fp8_gemm_close(C, ref, what + " fp32")
    cb = Cb.view(torch.int16).cpu().numpy().view(np.uint16)
    assert_fp8_gemm_close(oracle.bf16_bits_to_f32(cb), ref, what + " bf16")
    rq, rs = oracle.requant_c_1x128(ref)
    assert_fused_close(oracle, Cq.cpu().numpy(), Cs.cpu().numpy(), rq, rs, what + " fused")
    # SwiGLU: small M needs a workspace by contract; without one the call must fail cleanly, not compute garbage
    Hq = torch.full((M, N // 2), 0x55, dtype=torch.uint8, device="cuda")
    Hs = torch.full((N // 256, M), -1.0, dtype=torch.float32, device="cuda")
    f = lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__swiglu__C_1x128__output_fp8
    if not with_ws and (M % 128 != 0 or lib.query_config(3, M, N, K)[0] == 8):
        with pytest.raises(RuntimeError, match="workspace"):
            f(*t, Hq, Hs, M, N, K, workspace=None)
        return
    f(*t, Hq, Hs, M, N, K, workspace=ws(3))
    torch.cuda.synchronize()
    hq, hs = oracle.swiglu_requant(ref)
    assert_fused_close(oracle, Hq.cpu().numpy(), Hs.cpu().numpy(), hq, hs, what + " swiglu")
