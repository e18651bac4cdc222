"""A single tile row of fewer than 128 rows in the 128 x 128 FP8 tiles (64 < M < 128 on shapes whose M = 128 the tune
table gives to those tiles; any M < 128 when the tile is named).  Rows beyond M are computed from copies of the last
row and never stored: the result must equal the weight-streaming kernel's bit for bit (both add the same 128-K slices
in the same order) and nothing may be written behind row M - 1 (guard rows of NaN behind every output).  A sits in front of
rows of NaN codes: a lane that fetched a row other than its own (clamped) one for a stored output would show up as NaN."""
import numpy as np
import pytest
import torch

from helpers import assert_fp8_gemm_close

pytestmark = pytest.mark.gpu
T128, SKINNY = 3, 8


def _inputs(oracle, M, N, K, seed=0):
    rng = np.random.default_rng(seed + M + N + K)
    X = rng.standard_normal((M, K)).astype(np.float32)
    X[:, ::37] *= 11
    W = (rng.standard_normal((N, K)) * 0.03).astype(np.float32)
    Aq, As = oracle.quant_fp8(X, 1, True)
    Bq, Bs = oracle.quant_fp8(W, 128, False)
    return Aq, As, Bq, Bs


@pytest.mark.parametrize("M,N,K,split,pre", [(96, 256, 512, 1, False), (65, 1280, 1024, 1, True), (127, 512, 2560, 4, False), (1, 256, 256, 1, False),
                                             (100, 2560, 1280, 2, True), (17, 128, 128, 1, False), (112, 19456, 256, 1, False)])
def test_tail_rows_match_the_weight_streaming_kernel(lib, oracle, M, N, K, split, pre):
    Aq, As, Bq, Bs = _inputs(oracle, M, N, K)
    # A sits in front of rows that decode to NaN (0x7f is the e4m3 NaN code)
    dA_all = torch.full((M + 8, K), 0x7F, dtype=torch.uint8, device="cuda")
    dA_all[:M] = torch.from_numpy(Aq).cuda()
    dA = dA_all[:M]
    dAs = torch.from_numpy(As).cuda()
    dB, dBs = torch.from_numpy(Bq).cuda(), torch.from_numpy(Bs).cuda()
    if pre:
        dB = lib.preshuffle_weight(dB)
    ws = torch.full((8 * M * N * 4,), 0xFF, dtype=torch.uint8, device="cuda")
    kw = dict(workspace=ws, split_k=split, b_preshuffled=pre)
    guard = 4
    C = torch.full((M + guard, N), float("nan"), device="cuda")
    Cr = torch.empty((M, N), device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(dA, dAs, dB, dBs, C[:M], M, N, K, tile=T128, **kw)
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(dA, dAs, dB, dBs, Cr, M, N, K, tile=SKINNY, **kw)
    Y = torch.full((M + guard, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_bf16(dA, dAs, dB, dBs, Y[:M], M, N, K, tile=T128, **kw)
    Q = torch.full((M + guard, N), 0x7F, dtype=torch.uint8, device="cuda")
    Qs = torch.full((N // 128, M), float("nan"), device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(dA, dAs, dB, dBs, Q[:M], Qs, M, N, K, tile=T128, **kw)
    Qr = torch.empty((M, N), dtype=torch.uint8, device="cuda")
    Qsr = torch.empty((N // 128, M), device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(dA, dAs, dB, dBs, Qr, Qsr, M, N, K, tile=SKINNY, **kw)
    torch.cuda.synchronize()
    assert_fp8_gemm_close(C[:M].cpu().numpy(), oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128), "row tail")
    assert torch.equal(C[:M].view(torch.int32), Cr.view(torch.int32)), "differs from the weight-streaming kernel"
    assert torch.isnan(C[M:]).all() and torch.isnan(Y[M:].float()).all() and (Q[M:] == 0x7F).all(), "rows behind M were written"
    assert torch.equal(Y[:M].view(torch.int16), C[:M].to(torch.bfloat16).view(torch.int16)), "bf16 != RNE(fp32)"
    assert torch.equal(Q[:M], Qr) and torch.equal(Qs.view(torch.int32), Qsr.view(torch.int32)), "fused quantisation differs"


def test_table_routes_64_to_127_rows_like_128(lib):
    from llmmm_amd import _lib
    # gate_up and down of Qwen3-4B: M = 128 runs in 128 x 128 tiles, and so do 65 .. 127 rows
    for n, k in ((19456, 2560), (2560, 9728)):
        want = lib.query_config(_lib.OUT_FP8Q, 128, n, k)
        assert want[0] == T128
        for m in (65, 96, 127) if n == 19456 else (97, 112, 127):
            assert lib.query_config(_lib.OUT_FP8Q, m, n, k) == want
    # ... unless the table holds a weight-streaming entry measured between 65 and 127 rows (down up to 96 rows: four splits of
    # 32-row groups beat the tiles)
    for m in (65, 80, 96):
        assert lib.query_config(_lib.OUT_FP8Q, m, 2560, 9728) == (SKINNY, 4)
    # an unsplit entry (gate_up: enough column groups to fill the chip) already takes 33 .. 64 rows; a split one (down) does not
    for m in (33, 48, 64):
        assert lib.query_config(_lib.OUT_FP8Q, m, 19456, 2560) == lib.query_config(_lib.OUT_FP8Q, 128, 19456, 2560)
    assert lib.query_config(_lib.OUT_FP8Q, 32, 19456, 2560)[0] == SKINNY
    assert lib.query_config(_lib.OUT_FP8Q, 64, 2560, 9728)[0] == SKINNY


def test_swiglu_and_planes_entry_points_on_tail_rows(lib, oracle):
    """gate_up at M = 96 goes through the tiles' fp32 plane and the reduce kernel's SwiGLU; the result must equal M = 16-row
    blocks of the weight-streaming kernel (same planes, same reduce)."""
    M, N, K = 96, 19456, 2560
    Aq, As, Bq, Bs = _inputs(oracle, M, N, K, 3)
    dA, dAs, dB, dBs = (torch.from_numpy(a).cuda() for a in (Aq, As, Bq, Bs))
    ws = torch.empty(8 * M * N * 4, dtype=torch.uint8, device="cuda")
    H = torch.empty((M, N // 2), dtype=torch.uint8, device="cuda")
    Hs = torch.empty((N // 256, M), device="cuda")
    Hr, Hsr = torch.empty_like(H), torch.empty_like(Hs)
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__swiglu__C_1x128__output_fp8(dA, dAs, dB, dBs, H, Hs, M, N, K, workspace=ws)
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__swiglu__C_1x128__output_fp8(dA, dAs, dB, dBs, Hr, Hsr, M, N, K, workspace=ws, tile=SKINNY, split_k=1)
    torch.cuda.synchronize()
    assert torch.equal(H, Hr) and torch.equal(Hs.view(torch.int32), Hsr.view(torch.int32))


def test_untuned_shapes_between_64_and_128_rows(lib, oracle):
    """Shapes the tune table does not know: large weight matrices go to one row of 128 x 128 tiles, small ones stay with the
    weight-streaming kernel; both against the oracle, the SwiGLU output included."""
    from llmmm_amd import _lib
    assert lib.query_config(_lib.OUT_FP8Q, 96, 6144, 4096)[0] == T128      # 25 MB of weights
    assert lib.query_config(_lib.OUT_FP8Q, 128, 6144, 4096)[0] == T128
    assert lib.query_config(_lib.OUT_FP8Q, 96, 4096, 4096)[0] == SKINNY    # 17 MB
    assert lib.query_config(_lib.OUT_FP8Q, 128, 2048, 2048)[0] == SKINNY
    assert lib.query_config(_lib.OUT_FP8Q, 64, 6144, 4096)[0] == SKINNY
    M, N, K = 90, 6144, 4096
    Aq, As, Bq, Bs = _inputs(oracle, M, N, K, 9)
    dA, dAs, dB, dBs = (torch.from_numpy(a).cuda() for a in (Aq, As, Bq, Bs))
    ref = oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128)
    C = torch.empty((M, N), device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(dA, dAs, dB, dBs, C, M, N, K)
    H = torch.empty((M, N // 2), dtype=torch.uint8, device="cuda")
    Hs = torch.empty((N // 256, M), device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__swiglu__C_1x128__output_fp8(dA, dAs, dB, dBs, H, Hs, M, N, K,
                                                                                 workspace=lib.make_workspace(_lib.OUT_FP8Q_SWIGLU, M, N, K))
    Hr, Hsr = torch.empty_like(H), torch.empty_like(Hs)
    ws = torch.empty(8 * M * N * 4, dtype=torch.uint8, device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__swiglu__C_1x128__output_fp8(dA, dAs, dB, dBs, Hr, Hsr, M, N, K, workspace=ws, tile=SKINNY, split_k=4)
    torch.cuda.synchronize()
    assert_fp8_gemm_close(C.cpu().numpy(), ref, "untuned row tail")
    # the two routes split K differently (fp32 sums in another order): codes may differ by one step where a value sits on a boundary
    same = (H == Hr).float().mean().item()
    assert same > 0.999 and torch.allclose(Hs, Hsr, rtol=1e-3)


@pytest.mark.parametrize("M", [65, 96, 127])
@pytest.mark.parametrize("N,K", [(2560, 9728), (10240, 2048)])
def test_add_rmsnorm_quant_on_tail_rows_with_the_queried_workspace(lib, oracle, M, N, K):
    """The residual + RMSNorm + quantiser entry point on a row tail, tuned (down projection: split tiles) and untuned
    (one unsplit row of 128 x 128 tiles, which has no epilogue of its own and needs one plane), with exactly the
    workspace its query function asks for: hidden == T(C32 + residual), codes and scales == the oracle's on that."""
    from llmmm_amd import _lib
    # (the down projection up to 96 rows: the table sends it to the weight-streaming kernel in four splits -- the same property)
    assert lib.query_config(_lib.OUT_F32, M, N, K)[0] == (SKINNY if (N, K) == (2560, 9728) and M <= 96 else T128)
    need = _lib.lib.llmmm_fp8_gemm_add_rmsnorm_quant_workspace(M, N, K)
    assert need >= M * N * 4
    Aq, As, Bq, Bs = _inputs(oracle, M, N, K, 5)
    rng = np.random.default_rng(M)
    res = (rng.standard_normal((M, N)) * 2).astype(np.float32)
    w = rng.uniform(0.5, 1.5, N).astype(np.float32)
    dA, dAs, dB, dBs = (torch.from_numpy(a).cuda() for a in (Aq, As, Bq, Bs))
    C = torch.empty((M, N), device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(dA, dAs, dB, dBs, C, M, N, K, workspace=lib.make_workspace(_lib.OUT_F32, M, N, K))
    tres = torch.from_numpy(res).cuda().to(torch.bfloat16)
    hidden = torch.full((M + 2, N), 7.0, dtype=torch.bfloat16, device="cuda")
    ws = torch.full((need,), 0xFF, dtype=torch.uint8, device="cuda")
    q, s = lib.fp8_gemm_add_rmsnorm_quant(dA, dAs, dB, dBs, tres, hidden[:M], torch.from_numpy(w).cuda(), 1e-6, M, N, K, workspace=ws)
    torch.cuda.synchronize()
    want = torch.from_numpy(C.cpu().numpy() + tres.float().cpu().numpy()).to(torch.bfloat16)
    assert torch.equal(hidden[:M].cpu().view(torch.int16), want.view(torch.int16)) and (hidden[M:] == 7.0).all()
    rq, rs = oracle.rmsnorm_quant(want.float().numpy(), w, 1e-6)
    assert np.array_equal(q.cpu().numpy(), rq) and np.array_equal(s.cpu().numpy().view(np.uint32), rs.view(np.uint32))


@pytest.mark.parametrize("M", [65, 127])
@pytest.mark.parametrize("n_q,n_kv,K", [(136, 8, 2560), (48, 8, 2560)])
def test_qkv_rope_on_tail_rows_with_the_queried_workspace(lib, oracle, M, n_q, n_kv, K):
    from llmmm_amd import _lib
    N = (n_q + 2 * n_kv) * 128
    assert lib.query_config(_lib.OUT_F32, M, N, K)[0] == T128
    need = _lib.lib.llmmm_fp8_gemm_qkv_rope_workspace(M, N, K)
    assert need >= M * N * 4
    Aq, As, Bq, Bs = _inputs(oracle, M, N, K, 7)
    rng = np.random.default_rng(M + N)
    qw, kw = (rng.uniform(0.5, 1.5, 128).astype(np.float32) for _ in range(2))
    ang = np.arange(512, dtype=np.float64)[:, None] * (1e6 ** (-np.arange(64) / 64.0))[None, :]
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    pos = rng.integers(0, 512, M).astype(np.int32)
    g = lambda a: torch.from_numpy(a).cuda()
    dA, dAs, dB, dBs = g(Aq), g(As), g(Bq), g(Bs)
    C = torch.empty((M, N), device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(dA, dAs, dB, dBs, C, M, N, K, workspace=lib.make_workspace(_lib.OUT_F32, M, N, K))
    ws = torch.full((need,), 0xFF, dtype=torch.uint8, device="cuda")
    out = lib.fp8_gemm_qkv_rope(dA, dAs, dB, dBs, g(qw), g(kw), 1e-6, g(cos), g(sin), g(pos), n_q, n_kv, M, N, K, workspace=ws)
    torch.cuda.synchronize()
    want = oracle.qk_norm_rope(C.cpu().numpy(), qw, kw, 1e-6, cos, sin, pos, n_q, n_kv)
    assert np.array_equal(out.view(torch.int16).cpu().numpy().view(np.uint16), oracle.f32_to_bf16_bits(want))
