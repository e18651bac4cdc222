"""The weight-streaming kernel in column strips (LLMMM_TILE_STRIP): a workgroup owns 16 columns over all of K (32 where 16-column
strips would be more than the CUs and the weight matrix is small), its waves split K and add their partial sums in wave
order -- one launch, no workspace.  Against the oracle at the GEMM bar;
bit-identical run to run; bf16 == RNE(fp32); pre-shuffled weights give the same bits; rows behind M are never written."""
import ctypes

import numpy as np
import pytest
import torch

from helpers import assert_fp8_gemm_close, fp8_inputs

pytestmark = pytest.mark.gpu
STRIP, SKINNY = 9, 8


def _run(lib, Aq, As, Bq, Bs, M, N, K, pre=False, tile=STRIP, guard=3):
    t = [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in (Aq, As, Bq, Bs)]
    if pre:
        t[2] = lib.preshuffle_weight(t[2])
    C = torch.full((M + guard, N), float("nan"), dtype=torch.float32, device="cuda")
    Cb = torch.full((M + guard, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(*t, C[:M], M, N, K, tile=tile, b_preshuffled=pre)
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_bf16(*t, Cb[:M], M, N, K, tile=tile, b_preshuffled=pre)
    torch.cuda.synchronize()
    assert torch.isnan(C[M:]).all() and torch.isnan(Cb[M:].float()).all(), "rows behind M were written"
    return C[:M].clone(), Cb[:M].clone()


# K / 128 from 8 (one slice per wave) over uneven shares (20 slices: 2 or 3 per wave; 76: 9 or 10) to 8 per wave and more
@pytest.mark.parametrize("M,N,K", [(1, 2560, 4096), (16, 2560, 9728), (16, 6144, 2560), (5, 256, 1024), (32, 2560, 4096), (17, 128, 1152),
                                   (1, 128, 8192), (9, 512, 10240), (31, 384, 2560),
                                   # 32-column strips: 6144 x 2560 above; four waves per fragment with a tail slice, two row blocks, exactly 256 strips
                                   (3, 4608, 1152), (24, 4608, 1152), (1, 8192, 1024), (16, 6144, 4096),
                                   # 448 16-column strips of a matrix too large for wide ones: two workgroups on most CUs
                                   (3, 7168, 5120)])
def test_against_oracle(lib, oracle, M, N, K):
    Aq, As, Bq, Bs = fp8_inputs(oracle, M, N, K, seed=M + N + K)
    ref = oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128)
    C, Cb = _run(lib, Aq, As, Bq, Bs, M, N, K)
    assert_fp8_gemm_close(C.cpu().numpy(), ref, "strip %dx%dx%d" % (M, N, K))
    assert torch.equal(Cb, C.to(torch.bfloat16)), "bf16 output is not RNE(fp32 output)"
    C2, Cb2 = _run(lib, Aq, As, Bq, Bs, M, N, K)
    assert torch.equal(C.view(torch.int32), C2.view(torch.int32)) and torch.equal(Cb.view(torch.int16), Cb2.view(torch.int16)), "not the same bits run to run"
    Cp, _ = _run(lib, Aq, As, Bq, Bs, M, N, K, pre=True)
    assert torch.equal(C.view(torch.int32), Cp.view(torch.int32)), "pre-shuffled weights give other bits"
    # the split-K form adds the same slices in another order: equal within the bar, and exactly equal where every
    # slice but one of a row is zero (nothing to reorder)
    Cs_, _ = _run(lib, Aq, As, Bq, Bs, M, N, K, tile=SKINNY)
    assert_fp8_gemm_close(Cs_.cpu().numpy(), ref, "split form")


def test_single_nonzero_slice_is_exact(lib, oracle):
    """With one non-zero slice per row the sum has one term: strips, the split-K form and the oracle agree bit for bit."""
    M, N, K = 16, 256, 2048
    Aq, As, Bq, Bs = fp8_inputs(oracle, M, N, K, seed=3)
    keep = np.arange(M) % (K // 128)
    for m in range(M):
        for kb in range(K // 128):
            if kb != keep[m]:
                Aq[m, kb * 128:(kb + 1) * 128] = 0
    ref = oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128)
    C, _ = _run(lib, Aq, As, Bq, Bs, M, N, K)
    Cs_, _ = _run(lib, Aq, As, Bq, Bs, M, N, K, tile=SKINNY)
    assert torch.equal(C.view(torch.int32), Cs_.view(torch.int32))
    assert np.abs(C.cpu().numpy() - ref).max() <= 1e-4 * np.abs(ref).max()


def _strips_pay(m, n, k, fused):
    """The library's rule, restated: strips where measured faster than split-K + reduce (256 CUs)."""
    plain = m <= 8 or (m <= 16 and k <= 4096)
    if n // 16 <= 256:
        return m * k <= 65536 and m <= 16 if fused else plain
    if n % 32 == 0 and n // 32 <= 256 and n * k <= 32 << 20:   # 32-column strips
        return m <= 4 if fused else plain
    if 448 <= n // 16 <= 512:                                   # two 16-column strips on (nearly) every CU
        return m * k <= (65536 if fused else 131072)
    return False


def test_the_library_picks_strips_where_it_used_to_split(lib):
    from llmmm_amd import _lib
    for n, k in ((2560, 4096), (2560, 9728), (6144, 2560)):
        for m in (1, 4, 8, 16, 32):
            want = (STRIP, 1) if _strips_pay(m, n, k, False) else None  # every strip re-reads the activations: small M only
            for kind in (_lib.OUT_BF16, _lib.OUT_F32):
                got = lib.query_config(kind, m, n, k)
                assert got == want if want else got[0] == SKINNY and got[1] > 1
            # the 1x128-grouped output takes strips too (M <= 16: the strips of a column group exchange their row maxima; the
            # exchange costs about what the reduce launch did); what the split-K form would run in is what the size queries answer for
            got8 = lib.query_config(_lib.OUT_FP8Q, m, n, k)
            assert got8 == (STRIP, 1) if _strips_pay(m, n, k, True) else got8[0] == SKINNY and got8[1] > 1
            split8 = lib.workspace_bytes(_lib.OUT_FP8Q, m, n, k) // (m * n * 4)
            assert split8 > 1
            # the size queries cannot see a call's cfg: they answer for the split-K form, which a strip shape falls back to
            # when its activations are generated by the kernel (at least ceil(K / 128 / 32) splits then)
            planes = max(split8, -(-(k // 128) // 32)) * m * n * 4
            assert lib.workspace_bytes(_lib.OUT_BF16, m, n, k) == (planes if want else got[1] * m * n * 4)
            raw = _lib.lib
            assert raw.llmmm_fp8_gemm_planes_bytes(m, n, k) == planes
            if n <= 10240:
                assert raw.llmmm_fp8_gemm_add_rmsnorm_quant_workspace(m, n, k) == planes
            assert raw.llmmm_fp8_gemm_qkv_rope_workspace(m, n, k) > 0
    assert lib.query_config(_lib.OUT_BF16, 1, 19456, 2560) == (SKINNY, 1)   # enough column groups: no split to replace
    # other model families: wide strips on small matrices, paired narrow ones at 8192 columns, none for a round and a quarter
    for n, k in ((6144, 4096), (5120, 5120), (8192, 8192), (5120, 13824), (7168, 5120), (8192, 28672)):
        for m in (1, 4, 8, 16):
            for kind, fused in ((_lib.OUT_BF16, False), (_lib.OUT_FP8Q, True)):
                got = lib.query_config(kind, m, n, k)
                assert got == (STRIP, 1) if _strips_pay(m, n, k, fused) else got[0] == SKINNY and got[1] > 1, (m, n, k, fused, got)


@pytest.mark.parametrize("M,N,K", [(1, 2560, 4096), (8, 2560, 9728), (16, 2560, 4096), (8, 5120, 5120)])  # (the last: 32-column strips)
@pytest.mark.parametrize("dt", ["bf16", "f32", "f16"])
def test_residual_add_and_planes_entry_points_take_strips(lib, oracle, M, N, K, dt):
    """llmmm_fp8_gemm_add_rmsnorm_quant on a strip shape: hidden == T(C32 + residual) with C32 the strip kernel's fp32 output,
    codes and scales == the oracle's RMSNorm + quantiser of that hidden state, no workspace; in place too.
    llmmm_fp8_gemm_planes: one plane, the same fp32 values."""
    tdt = {"bf16": torch.bfloat16, "f32": torch.float32, "f16": torch.float16}[dt]
    Aq, As, Bq, Bs = fp8_inputs(oracle, M, N, K, seed=K + M)
    rng = np.random.default_rng(M)
    res = (rng.standard_normal((M, N)) * 2).astype(np.float32)
    w = rng.uniform(0.5, 1.5, N).astype(np.float32)
    t = [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in (Aq, As, Bq, Bs)]
    C, _ = _run(lib, Aq, As, Bq, Bs, M, N, K)
    tres = torch.from_numpy(res).cuda().to(tdt)
    want = torch.from_numpy(C.cpu().numpy() + tres.float().cpu().numpy()).to(tdt)
    tiny = torch.empty(16, dtype=torch.uint8, device="cuda")
    for inplace in (False, True):
        r = tres.clone()
        hidden = r if inplace else torch.full((M + 1, N), 7.0, dtype=tdt, device="cuda")[:M]
        q, s = lib.fp8_gemm_add_rmsnorm_quant(*t, r, hidden, torch.from_numpy(w).cuda(), 1e-6, M, N, K, workspace=tiny)
        torch.cuda.synchronize()
        bits = torch.int32 if dt == "f32" else torch.int16
        assert torch.equal(hidden.cpu().view(bits), want.view(bits)), "hidden state differs"
        rq, rs = oracle.rmsnorm_quant(want.float().numpy(), w, 1e-6)
        assert np.array_equal(q.cpu().numpy(), rq) and np.array_equal(s.cpu().numpy().view(np.uint32), rs.view(np.uint32))
    planes, splits = lib.fp8_gemm_planes(*t, M, N, K)
    torch.cuda.synchronize()
    assert splits == 1 and torch.equal(planes.reshape(-1)[:M * N].view(torch.int32), C.reshape(-1).view(torch.int32))


def test_refusals(lib):
    from llmmm_amd import _lib
    raw = _lib.lib
    fake = ctypes.c_void_p(0x1000)
    cfg = _lib.GemmCfg(STRIP, 0, 0, 0)
    args = (fake, fake, fake, fake, fake, fake)
    assert raw.llmmm_fp8_gemm_ex(_lib.OUT_FP8Q, *args, 17, 2560, 4096, None, 0, ctypes.byref(cfg), None) == _lib.ERR_INVALID_ARGUMENT  # fp8 output: M <= 16
    assert raw.llmmm_fp8_gemm_ex(_lib.OUT_FP8Q_SWIGLU, *args, 16, 2560, 4096, None, 0, ctypes.byref(cfg), None) == _lib.ERR_INVALID_ARGUMENT
    assert raw.llmmm_fp8_gemm_ex(_lib.OUT_F32, *args, 33, 2560, 4096, None, 0, ctypes.byref(cfg), None) == _lib.ERR_INVALID_ARGUMENT
    assert raw.llmmm_fp8_gemm_ex(_lib.OUT_F32, *args, 16, 2560, 896, None, 0, ctypes.byref(cfg), None) == _lib.ERR_INVALID_ARGUMENT
    cfg = _lib.GemmCfg(STRIP, 4, 0, 0)
    assert raw.llmmm_fp8_gemm_ex(_lib.OUT_F32, *args, 16, 2560, 4096, fake, 1 << 24, ctypes.byref(cfg), None) == _lib.ERR_INVALID_ARGUMENT
