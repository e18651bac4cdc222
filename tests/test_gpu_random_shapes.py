"""Seeded random shapes -- the Qwen3-4B projections at random M and arbitrary (N, K) multiples of 128 -- through the
auto-configured entry points with the workspaces their query functions ask for, against the oracle: whatever kernel,
split, row grouping or tile the library picks for a shape, results meet the bars and rows behind M stay untouched."""
import numpy as np
import pytest
import torch

from helpers import assert_fp8_gemm_close, assert_fused_close

pytestmark = pytest.mark.gpu
QWEN = [(6144, 2560), (2560, 4096), (19456, 2560), (2560, 9728)]


def _case(oracle, lib, rng, qwen):
    M = int(rng.choice([rng.integers(1, 129), rng.integers(1, 129), 128 * rng.integers(1, 4)]))
    if qwen:
        N, K = QWEN[int(rng.integers(0, 4))]
        if N == 19456:
            M = min(M, 128)  # keeps the oracle's share of the run short
    else:
        N, K = int(128 * rng.integers(1, 25)), int(128 * rng.integers(1, 25))
    X = rng.standard_normal((M, K)).astype(np.float32)
    X[:, ::31] *= 8
    W = (rng.standard_normal((N, K)) * 0.03).astype(np.float32)
    Aq, As = oracle.quant_fp8(X, 1, True)
    Bq, Bs = oracle.quant_fp8(W, 128, False)
    dev = [torch.from_numpy(a).cuda() for a in (Aq, As, Bq, Bs)]
    pre = bool(rng.random() < 0.5)
    if pre:
        dev[2] = lib.preshuffle_weight(dev[2])
    return M, N, K, pre, dev, oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128)


@pytest.mark.parametrize("seed,qwen", [(1, True), (2, True), (3, True), (4, False), (5, False)])
def test_plain_outputs(lib, oracle, seed, qwen):
    from llmmm_amd import _lib
    rng = np.random.default_rng(seed)
    for _ in range(8):
        M, N, K, pre, (dA, dAs, dB, dBs), ref = _case(oracle, lib, rng, qwen)
        what = "M %d N %d K %d pre %d fp32 %s fp8q %s" % (M, N, K, pre, lib.query_config(_lib.OUT_F32, M, N, K), lib.query_config(_lib.OUT_FP8Q, M, N, K))
        C = torch.full((M + 1, N), float("nan"), device="cuda")
        Y = torch.full((M + 1, N), float("nan"), dtype=torch.bfloat16, device="cuda")
        Q = torch.full((M + 1, N), 0x7F, dtype=torch.uint8, device="cuda")
        S = torch.full((N // 128, M), float("nan"), device="cuda")
        lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(dA, dAs, dB, dBs, C[:M], M, N, K, b_preshuffled=pre,
                                                                     workspace=lib.make_workspace(_lib.OUT_F32, M, N, K))
        lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_bf16(dA, dAs, dB, dBs, Y[:M], M, N, K, b_preshuffled=pre,
                                                                     workspace=lib.make_workspace(_lib.OUT_BF16, M, N, K))
        lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(dA, dAs, dB, dBs, Q[:M], S, M, N, K, b_preshuffled=pre,
                                                                             workspace=lib.make_workspace(_lib.OUT_FP8Q, M, N, K))
        torch.cuda.synchronize()
        assert torch.isnan(C[M:]).all() and torch.isnan(Y[M:].float()).all() and (Q[M:] == 0x7F).all(), what + ": a row behind M was written"
        assert_fp8_gemm_close(C[:M].cpu().numpy(), ref, what)
        assert torch.equal(Y[:M], C[:M].to(torch.bfloat16)), what + ": bf16 output is not RNE(fp32 output)"
        rq, rs = oracle.requant_c_1x128(ref)
        assert_fused_close(oracle, Q[:M].cpu().numpy(), S.cpu().numpy(), rq, rs, what)


@pytest.mark.parametrize("seed", [11, 12])
def test_residual_add_rmsnorm_quant_on_o_and_down(lib, oracle, seed):
    rng = np.random.default_rng(seed)
    for _ in range(6):
        M = int(rng.choice([rng.integers(1, 129), 128 * rng.integers(1, 4)]))
        N, K = QWEN[1] if rng.random() < 0.5 else QWEN[3]
        X = rng.standard_normal((M, K)).astype(np.float32)
        W = (rng.standard_normal((N, K)) * 0.03).astype(np.float32)
        Aq, As = oracle.quant_fp8(X, 1, True)
        Bq, Bs = oracle.quant_fp8(W, 128, False)
        dA, dAs, dB, dBs = (torch.from_numpy(a).cuda() for a in (Aq, As, Bq, Bs))
        ref = oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128)
        res = torch.from_numpy((rng.standard_normal((M, N)) * 2).astype(np.float32)).cuda().to(torch.bfloat16)
        w = rng.uniform(0.5, 1.5, N).astype(np.float32)
        hidden = torch.full((M + 1, N), 7.0, dtype=torch.bfloat16, device="cuda")
        q, s = lib.fp8_gemm_add_rmsnorm_quant(dA, dAs, dB, dBs, res, hidden[:M], torch.from_numpy(w).cuda(), 1e-6, M, N, K)
        torch.cuda.synchronize()
        what = "M %d N %d K %d" % (M, N, K)
        assert (hidden[M:] == 7.0).all(), what + ": a row behind M was written"
        h = hidden[:M].float().cpu().numpy()
        want = ref + res.float().cpu().numpy()
        # the GEMM bar on the projection, plus half a bf16 step for the stored hidden state
        tol = 2e-2 * np.maximum(np.abs(ref), np.abs(ref).reshape(M, N // 128, 128).max(-1).repeat(128, axis=1) * 2.0 ** -7) + 2.0 ** -8 * np.abs(want) + 1e-6
        assert (np.abs(h - want) <= tol).all(), what + ": hidden state"
        rq, rs = oracle.rmsnorm_quant(h, w, 1e-6)  # bit-exact on the stored hidden state
        assert np.array_equal(q.cpu().numpy(), rq) and np.array_equal(s.cpu().numpy().view(np.uint32), rs.view(np.uint32)), what


@pytest.mark.parametrize("M", [1, 2, 4, 8, 16, 32])
@pytest.mark.parametrize("N,K", [(2560, 9728), (2560, 4096)])
def test_generated_activations_with_the_queried_workspaces(lib, oracle, M, N, K):
    """The down projection on silu(gate) * up made by the library (a_swiglu) through every entry point that takes it, each
    with exactly the buffers its size queries ask for -- the Python mirror's defaults.  These shapes run in column strips
    with quantised activations and in the split-K form with generated ones; the queries must cover the latter."""
    from llmmm_amd import _lib
    rng = np.random.default_rng(100 + M + K)
    G = (rng.standard_normal((M, 2 * K)) * 1.5).astype(np.float32)
    W = (rng.standard_normal((N, K)) * 0.03).astype(np.float32)
    Bq, Bs = oracle.quant_fp8(W, 128, False)
    hq, hs = oracle.swiglu_requant(G)
    ref = oracle.fp8_gemm(hq, hs, Bq, Bs, promote=128)
    dG, dB, dBs = torch.from_numpy(G).cuda(), torch.from_numpy(Bq).cuda(), torch.from_numpy(Bs).cuda()
    raw = _lib.lib
    a_ws = int(raw.llmmm_fp8_swiglu_a_workspace(M, N, K))
    # plain GEMM, fp32 output: llmmm_fp8_gemm_workspace + llmmm_fp8_swiglu_a_workspace bytes
    need = int(raw.llmmm_fp8_gemm_workspace(_lib.OUT_F32, M, N, K)) + a_ws
    ws = torch.full((max(need, 16),), 0xFF, dtype=torch.uint8, device="cuda")[:max(need, 1)] if need else None
    C = torch.full((M, N), float("nan"), device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(dG, None, dB, dBs, C, M, N, K, workspace=ws, a_swiglu=True)
    torch.cuda.synchronize()
    assert_fp8_gemm_close(C.cpu().numpy(), ref, "a_swiglu fp32, M %d" % M)
    # planes only: the defaults of the mirror are the queried sizes
    planes, splits = lib.fp8_gemm_planes(dG, None, dB, dBs, M, N, K, a_swiglu=True)
    torch.cuda.synchronize()
    assert splits >= 1 and planes.numel() * 4 == int(raw.llmmm_fp8_gemm_planes_bytes(M, N, K))
    assert_fp8_gemm_close(planes.view(-1)[:splits * M * N].view(splits, M, N).sum(0).cpu().numpy(), ref, "a_swiglu planes, M %d" % M)
    # projection + residual add + RMSNorm + quantiser
    res = torch.from_numpy(rng.standard_normal((M, N)).astype(np.float32)).cuda().to(torch.bfloat16)
    w = rng.uniform(0.5, 1.5, N).astype(np.float32)
    hidden = torch.empty_like(res)
    q, s = lib.fp8_gemm_add_rmsnorm_quant(dG, None, dB, dBs, res, hidden, torch.from_numpy(w).cuda(), 1e-6, M, N, K, a_swiglu=True)
    torch.cuda.synchronize()
    h = hidden.float().cpu().numpy()
    want = ref + res.float().cpu().numpy()
    tol = 2e-2 * np.maximum(np.abs(ref), np.abs(ref).reshape(M, N // 128, 128).max(-1).repeat(128, axis=1) * 2.0 ** -7) + 2.0 ** -8 * np.abs(want) + 1e-6
    assert (np.abs(h - want) <= tol).all(), "a_swiglu hidden state, M %d" % M
    rq, rs = oracle.rmsnorm_quant(h, w, 1e-6)
    assert np.array_equal(q.cpu().numpy(), rq) and np.array_equal(s.cpu().numpy().view(np.uint32), rs.view(np.uint32))
