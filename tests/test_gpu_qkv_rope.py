"""The QKV projection with per-head RMSNorm and rotary embedding fused behind it, through the C ABI.  The second kernel
promises the oracle's bits on the fp32 GEMM result of the same kernel and split: bf16 output == RNE(oracle), fp8 output
== the oracle's 1x128 re-quantisation (reciprocal form) of the oracle's rotated heads."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
TILES = {"auto": -1, "256x256": 0, "128x256": 1, "256x128": 2, "128x128": 3, "skinny": 8}


def _tables(rows, theta=1e6):
    inv = theta ** (-np.arange(64, dtype=np.float64) / 64.0)
    ang = np.arange(rows, dtype=np.float64)[:, None] * inv[None, :]
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


def _run(lib, oracle, M, K, n_q, n_kv, tile, split, norm=True, pre=False, seed=0, rows=4096):
    N = (n_q + 2 * n_kv) * 128
    rng = np.random.default_rng(seed + M + N + K)
    X = rng.standard_normal((M, K)).astype(np.float32)
    X[:, ::53] *= 10
    W = (rng.standard_normal((N, K)) * 0.05).astype(np.float32)
    Aq, As = oracle.quant_fp8(X, 1, True)
    Bq, Bs = oracle.quant_fp8(W, 128, False)
    qw = rng.uniform(0.5, 1.5, 128).astype(np.float32) if norm else None
    kw = rng.uniform(0.5, 1.5, 128).astype(np.float32) if norm else None
    cos, sin = _tables(rows)
    pos = rng.integers(0, rows, M).astype(np.int32)
    if M > 3:
        pos[1], pos[2] = -3, rows + 10  # clamped to the table
    g = lambda a: None if a is None else torch.from_numpy(a).cuda()
    dA, dAs, dB, dBs = g(Aq), g(As), g(Bq), g(Bs)
    if pre:
        dB = lib.preshuffle_weight(dB)
    ws = torch.full((16 * M * N * 4,), 0xFF, dtype=torch.uint8, device="cuda")
    C = torch.empty((M, N), dtype=torch.float32, device="cuda")
    # the fp32 result of the kernel the fused call runs: with the library's own choice that is the choice for 1x128-grouped
    # outputs (heads are such groups), not the column strips a plain fp32 output takes at decode sizes
    from llmmm_amd import _lib
    plain_tile = lib.query_config(_lib.OUT_FP8Q, M, N, K)[0] if tile == TILES["auto"] and split == 0 else tile
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(dA, dAs, dB, dBs, C, M, N, K, workspace=ws, tile=plain_tile, split_k=split, b_preshuffled=pre)
    torch.cuda.synchronize()
    want = oracle.qk_norm_rope(C.cpu().numpy(), qw, kw, 1e-6, cos, sin, pos, n_q, n_kv)
    args = (dA, dAs, dB, dBs, g(qw), g(kw), 1e-6, g(cos), g(sin), g(pos), n_q, n_kv, M, N, K)
    kw_ = dict(workspace=ws, tile=tile, split_k=split, b_preshuffled=pre)
    ws.fill_(0xFF)
    out = lib.fp8_gemm_qkv_rope(*args, **kw_)
    ws.fill_(0xFF)
    q, s = lib.fp8_gemm_qkv_rope(*args, out_fp8=True, **kw_)
    torch.cuda.synchronize()
    assert np.array_equal(out.view(torch.int16).cpu().numpy().view(np.uint16), oracle.f32_to_bf16_bits(want)), "bf16 output differs"
    rq, rs = oracle.requant_c_1x128(want)
    assert np.array_equal(s.cpu().numpy().view(np.uint32), rs.view(np.uint32)), "scales differ"
    assert np.array_equal(q.cpu().numpy(), rq), "codes differ"
    return want


# Qwen3-4B geometry (32 query, 8 key/value heads, K = 2560) at decode sizes, and small geometries with odd head counts
@pytest.mark.parametrize("M,K,n_q,n_kv,split", [(1, 2560, 32, 8, 0), (16, 2560, 32, 8, 0), (5, 2560, 32, 8, 1), (16, 2560, 32, 8, 5), (77, 2560, 32, 8, 0),
                                                (128, 2560, 32, 8, 0), (3, 128, 1, 1, 0), (9, 512, 3, 2, 2), (33, 384, 5, 1, 0)])
def test_streaming_kernel(lib, oracle, M, K, n_q, n_kv, split):
    _run(lib, oracle, M, K, n_q, n_kv, TILES["skinny"], split)


@pytest.mark.parametrize("M,K,n_q,n_kv,tile,split", [(256, 2560, 32, 8, "auto", 0), (128, 512, 4, 2, "128x128", 1), (128, 1024, 4, 2, "128x128", 3),
                                                     (512, 512, 4, 2, "256x256", 0), (256, 2560, 32, 8, "128x256", 2), (2048, 256, 32, 8, "auto", 0)])
def test_tile_kernels(lib, oracle, M, K, n_q, n_kv, tile, split):
    _run(lib, oracle, M, K, n_q, n_kv, TILES[tile], split)


def test_unsplit_tile_kernels_need_no_workspace(lib, oracle):
    """Without split the tile kernels apply norm and rope to their accumulators: no planes, no workspace, same bits."""
    M, K, n_q, n_kv = 256, 1024, 6, 1
    N = (n_q + 2 * n_kv) * 128
    assert lib._lib.lib.llmmm_fp8_gemm_qkv_rope_workspace(2048, 6144, 2560) == 0
    rng = np.random.default_rng(21)
    Aq, As = oracle.quant_fp8(rng.standard_normal((M, K)).astype(np.float32), 1, True)
    Bq, Bs = oracle.quant_fp8((rng.standard_normal((N, K)) * 0.05).astype(np.float32), 128, False)
    qw, kw = rng.uniform(0.5, 1.5, 128).astype(np.float32), rng.uniform(0.5, 1.5, 128).astype(np.float32)
    cos, sin = _tables(512)
    pos = rng.integers(0, 512, M).astype(np.int32)
    g = lambda a: torch.from_numpy(a).cuda()
    dA, dAs, dB, dBs = g(Aq), g(As), g(Bq), g(Bs)
    C = torch.empty((M, N), dtype=torch.float32, device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(dA, dAs, dB, dBs, C, M, N, K, split_k=1)
    torch.cuda.synchronize()
    want = oracle.qk_norm_rope(C.cpu().numpy(), qw, kw, 1e-6, cos, sin, pos, n_q, n_kv)
    for tile in ("auto", "128x128", "256x128", "256x256"):
        tiny = torch.empty(16, dtype=torch.uint8, device="cuda")
        out = lib.fp8_gemm_qkv_rope(dA, dAs, dB, dBs, g(qw), g(kw), 1e-6, g(cos), g(sin), g(pos), n_q, n_kv, M, N, K, workspace=tiny, tile=TILES[tile])
        q, s = lib.fp8_gemm_qkv_rope(dA, dAs, dB, dBs, g(qw), g(kw), 1e-6, g(cos), g(sin), g(pos), n_q, n_kv, M, N, K, out_fp8=True, workspace=tiny,
                                     tile=TILES[tile])
        torch.cuda.synchronize()
        assert np.array_equal(out.view(torch.int16).cpu().numpy().view(np.uint16), oracle.f32_to_bf16_bits(want)), tile
        rq, rs = oracle.requant_c_1x128(want)
        assert np.array_equal(s.cpu().numpy().view(np.uint32), rs.view(np.uint32)) and np.array_equal(q.cpu().numpy(), rq), tile


def test_without_norm_and_with_preshuffled_weights(lib, oracle):
    _run(lib, oracle, 16, 2560, 32, 8, TILES["auto"], 0, norm=False, pre=True)
    _run(lib, oracle, 256, 1024, 6, 1, TILES["auto"], 0, norm=True, pre=True)


def test_rope_commutes_with_the_oracle_of_the_whole_chain(lib, oracle):
    """Against the oracle's own GEMM (not the GPU's fp32 result): the fused-output bar of the GEMM carries over, since
    norm and rotation are well conditioned -- |d| <= 2e-2 relative to the head's largest value."""
    M, K, n_q, n_kv = 16, 1024, 4, 2
    N = (n_q + 2 * n_kv) * 128
    rng = np.random.default_rng(77)
    X = rng.standard_normal((M, K)).astype(np.float32)
    W = (rng.standard_normal((N, K)) * 0.05).astype(np.float32)
    Aq, As = oracle.quant_fp8(X, 1, True)
    Bq, Bs = oracle.quant_fp8(W, 128, False)
    qw = np.ones(128, np.float32)
    cos, sin = _tables(64)
    pos = np.arange(M, dtype=np.int32)
    want = oracle.qk_norm_rope(oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128), qw, qw, 1e-6, cos, sin, pos, n_q, n_kv)
    g = lambda a: torch.from_numpy(a).cuda()
    out = lib.fp8_gemm_qkv_rope(g(Aq), g(As), g(Bq), g(Bs), g(qw), g(qw), 1e-6, g(cos), g(sin), g(pos), n_q, n_kv, M, N, K)
    torch.cuda.synchronize()
    got = out.float().cpu().numpy().reshape(M, -1, 128)
    ref = want.reshape(M, -1, 128)
    bound = 2e-2 * np.abs(ref).max(axis=2, keepdims=True) + 1e-6
    assert np.all(np.abs(got - ref) <= bound)


def test_errors(lib):
    M, K, n_q, n_kv = 16, 256, 2, 1
    N = 4 * 128
    z8 = lambda *s: torch.zeros(s, dtype=torch.uint8, device="cuda")
    f = lambda *s: torch.ones(s, device="cuda")
    pos = torch.zeros(M, dtype=torch.int32, device="cuda")
    args = lambda **o: (z8(M, K), f(K // 128, M), z8(N, K), f(N // 128, K // 128), f(128), f(128), 1e-6, f(8, 64), f(8, 64), pos)
    with pytest.raises(RuntimeError, match="n_q_heads"):
        lib.fp8_gemm_qkv_rope(*args(), 3, 1, M, N, K)
    with pytest.raises(RuntimeError, match="workspace"):
        lib.fp8_gemm_qkv_rope(*args(), n_q, n_kv, M, N, K, workspace=torch.empty(64, dtype=torch.uint8, device="cuda"))
    out = lib.fp8_gemm_qkv_rope(*args(), n_q, n_kv, M, N, K)
    torch.cuda.synchronize()
    assert float(out.float().abs().max()) == 0.0
