"""llmmm_fp8_gemm_static_ws (the FP8 GEMM whose split-K planes live in a fixed array inside the library, for callers
that cannot allocate) against llmmm_fp8_gemm with a caller's workspace: bit for bit, on two calls in a row that share
the array, the second smaller than the first, and against the oracle at the fused-output bar."""
import ctypes

import numpy as np
import pytest
import torch

from helpers import assert_fp8_gemm_close, assert_fused_close, fp8_inputs

pytestmark = pytest.mark.gpu


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


def _both(raw, out_kind, M, N, K, t, stream):
    """One call of each entry point on the same device operands; returns the two (C, Cs) pairs as numpy arrays."""
    from llmmm_amd import _lib
    need = raw.llmmm_fp8_gemm_workspace(out_kind, M, N, K)
    assert need <= _lib.STATIC_WS_BYTES, "the case must fit the built-in array"
    assert need > 0 or out_kind != _lib.OUT_FP8Q, "the fused-quant case must split K"  # (fp32 / bf16 may run in column strips: no planes)
    ws = torch.full((max(need, 16),), 0xA5, dtype=torch.uint8, device="cuda")
    dt = {0: torch.float32, 1: torch.bfloat16, 2: torch.uint8}[out_kind]
    outs = []
    for static in (False, True):
        C = torch.full((M, N), 0x55 if dt == torch.uint8 else float("nan"), dtype=dt, device="cuda")
        Cs = torch.full((N // 128, M), -1.0, dtype=torch.float32, device="cuda")
        if static:
            rc = raw.llmmm_fp8_gemm_static_ws(out_kind, _p(t[0]), _p(t[1]), _p(t[2]), _p(t[3]), _p(C), _p(Cs), M, N, K, stream)
        else:
            rc = raw.llmmm_fp8_gemm(out_kind, _p(t[0]), _p(t[1]), _p(t[2]), _p(t[3]), _p(C), _p(Cs), M, N, K, _p(ws), need, stream)
        assert rc == 0, raw.llmmm_last_error().decode()
        torch.cuda.synchronize()
        bits = C.view(torch.int16) if dt == torch.bfloat16 else C
        outs.append((bits.cpu().numpy(), Cs.cpu().numpy()))
    return outs


def test_static_workspace_matches_caller_workspace(oracle):
    from llmmm_amd import _lib
    raw = _lib.lib
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # first the larger problem (64 x 6144 x 2560, split 5: 7.9 MB of planes for every output kind), then a smaller one
    # (1 x 2560 x 4096, split 8: 80 KB for the fused output) that finds the first call's partial sums still in the array
    for M, N, K, seed in ((64, 6144, 2560, 11), (1, 2560, 4096, 12)):
        Aq, As, Bq, Bs = fp8_inputs(oracle, M, N, K, seed=seed)
        t = [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in (Aq, As, Bq, Bs)]
        ref = oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128)
        for out_kind in (_lib.OUT_FP8Q, _lib.OUT_F32, _lib.OUT_BF16):
            (c0, s0), (c1, s1) = _both(raw, out_kind, M, N, K, t, stream)
            what = "%dx%dx%d out %d" % (M, N, K, out_kind)
            assert (c0.view(np.uint8) == c1.view(np.uint8)).all(), what + ": outputs differ between the two entry points"
            if out_kind == _lib.OUT_FP8Q:
                assert (s0.view(np.uint32) == s1.view(np.uint32)).all(), what + ": scales differ between the two entry points"
                rq, rs = oracle.requant_c_1x128(ref)
                assert_fused_close(oracle, c1, s1, rq, rs, what)
            elif out_kind == _lib.OUT_F32:
                assert_fp8_gemm_close(c1, ref, what)
            else:
                assert_fp8_gemm_close(oracle.bf16_bits_to_f32(c1.view(np.uint16)), ref, what)


def test_static_workspace_rejects_what_does_not_fit():
    from llmmm_amd import _lib
    raw = _lib.lib
    M, N, K = 1024, 2560, 9728  # the down projection at M = 1024 runs in three splits: 3 x 1024 x 2560 floats = 31 MB
    assert raw.llmmm_fp8_gemm_workspace(_lib.OUT_FP8Q, M, N, K) > _lib.STATIC_WS_BYTES
    fake = ctypes.c_void_p(0x1000)
    rc = raw.llmmm_fp8_gemm_static_ws(_lib.OUT_FP8Q, fake, fake, fake, fake, fake, fake, M, N, K, None)
    assert rc == _lib.ERR_WORKSPACE and b"built-in array" in raw.llmmm_last_error()


def test_static_workspace_call_is_capturable_and_allocates_nothing(oracle):
    """After one warm-up call on a shape that needs no planes at all (so the warm-up itself cannot have been what resolved
    the array for a split-K shape), a split-K call is captured into a HIP graph: the capture must succeed (torch captures in the
    mode in which an allocation or a synchronising runtime query on any thread fails the capture), an eager call must leave
    the device's free memory where it was, and every replay -- with eager
    work and synchronisations between them -- must reproduce the eager call's bits."""
    from llmmm_amd import _lib
    raw = _lib.lib
    M, N, K = 16, 2560, 4096
    assert raw.llmmm_fp8_gemm_workspace(_lib.OUT_FP8Q, M, N, K) > 0
    Aq, As, Bq, Bs = fp8_inputs(oracle, M, N, K, seed=21)
    t = [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in (Aq, As, Bq, Bs)]
    wM, wN, wK = 256, 256, 256  # one unsplit tile: no planes
    assert raw.llmmm_fp8_gemm_workspace(_lib.OUT_FP8Q, wM, wN, wK) == 0
    wa, was, wb, wbs = [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in fp8_inputs(oracle, wM, wN, wK, seed=22)]
    wc = torch.empty((wM, wN), dtype=torch.uint8, device="cuda")
    wcs = torch.empty((wN // 128, wM), dtype=torch.float32, device="cuda")
    C = torch.full((M, N), 0x55, dtype=torch.uint8, device="cuda")
    Cs = torch.full((N // 128, M), -1.0, dtype=torch.float32, device="cuda")
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        st = ctypes.c_void_p(side.cuda_stream)
        assert raw.llmmm_fp8_gemm_static_ws(_lib.OUT_FP8Q, _p(wa), _p(was), _p(wb), _p(wbs), _p(wc), _p(wcs), wM, wN, wK, st) == 0  # warm-up
        side.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            rc = raw.llmmm_fp8_gemm_static_ws(_lib.OUT_FP8Q, _p(t[0]), _p(t[1]), _p(t[2]), _p(t[3]), _p(C), _p(Cs), M, N, K,
                                              ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0, raw.llmmm_last_error().decode()
    torch.cuda.synchronize()
    # an eager call of the same shape leaves the device's free memory where it was (hipMemGetInfo around it)
    free0 = torch.cuda.mem_get_info()[0]
    assert raw.llmmm_fp8_gemm_static_ws(_lib.OUT_FP8Q, _p(t[0]), _p(t[1]), _p(t[2]), _p(t[3]), _p(C), _p(Cs), M, N, K, None) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0, "device memory was allocated by the call"
    # the eager result, through the caller's-workspace form
    need = raw.llmmm_fp8_gemm_workspace(_lib.OUT_FP8Q, M, N, K)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    Ce, Cse = torch.empty_like(C), torch.empty_like(Cs)
    assert raw.llmmm_fp8_gemm(_lib.OUT_FP8Q, _p(t[0]), _p(t[1]), _p(t[2]), _p(t[3]), _p(Ce), _p(Cse), M, N, K, _p(ws), need, None) == 0
    torch.cuda.synchronize()
    for rep in range(3):
        C.fill_(0x55)
        Cs.fill_(-1.0)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(C, Ce) and torch.equal(Cs.view(torch.int32), Cse.view(torch.int32)), "replay %d differs from the eager call" % rep
