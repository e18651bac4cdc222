"""The peak-rate probes run, leave their sink untouched and report rates of the right order of magnitude (they are
measurement aids: the test only guards against a probe that no longer executes its loop)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_probes_run(lib):
    from llmmm_amd import _lib
    raw = _lib.lib
    sink = torch.zeros(4, device="cuda")
    ops = torch.zeros(32768, dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    for kind in (_lib.DTYPE_F16, _lib.DTYPE_BF16, _lib.PROBE_FP8):
        for _ in range(3):
            assert raw.llmmm_probe_mfma(kind, ops.data_ptr(), sink.data_ptr(), 1024, 500, st) == 0
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        assert raw.llmmm_probe_mfma(kind, ops.data_ptr(), sink.data_ptr(), 1024, 500, st) == 0
        e1.record()
        torch.cuda.synchronize()
        tflops = raw.llmmm_probe_mfma_flops(kind, 1024, 500) / e0.elapsed_time(e1) * 1e-9
        assert 300 < tflops < 6000, (kind, tflops)
    buf = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").random_(0, 255)
    for _ in range(3):
        assert raw.llmmm_probe_hbm_read(buf.data_ptr(), buf.numel(), sink.data_ptr(), 2048, st) == 0
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    assert raw.llmmm_probe_hbm_read(buf.data_ptr(), buf.numel(), sink.data_ptr(), 2048, st) == 0
    e1.record()
    torch.cuda.synchronize()
    gbs = buf.numel() / e0.elapsed_time(e1) * 1e-6
    assert 1000 < gbs < 9000, gbs
    assert (sink == 0).all()


@pytest.mark.parametrize("kind", ["fp8", "fp16"])
def test_phase_probes_give_the_product_kernels_results_and_ordered_stamps(lib, oracle, kind):
    """The phase-accounting builds of the 256 x 256 tile kernels: same output bits as the product kernels, and for every wave
    five clock readings in order (entry <= first operands <= end of the K loop <= last store issued <= stores acknowledged)."""
    import ctypes
    from llmmm_amd import _lib
    raw = _lib.lib
    M, N, K = 512, 768, 1024
    nbytes = raw.llmmm_probe_phases_bytes(M, N)
    assert nbytes == (M // 256) * (N // 256) * 8 * 12 * 8
    stamps = torch.zeros(nbytes // 8, dtype=torch.int64, device="cuda")
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    if kind == "fp8":
        from helpers import fp8_inputs
        Aq, As, Bq, Bs = (torch.from_numpy(a).cuda() for a in fp8_inputs(oracle, M, N, K, seed=9))
        C0 = torch.empty((M, N), dtype=torch.uint8, device="cuda")
        S0 = torch.empty((N // 128, M), device="cuda")
        C1, S1 = torch.zeros_like(C0), torch.zeros_like(S0)
        lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(Aq, As, Bq, Bs, C0, S0, M, N, K, tile=_lib.TILE_256x256)
        assert raw.llmmm_probe_fp8_gemm_phases(p(Aq), p(As), p(Bq), p(Bs), p(C1), p(S1), M, N, K, p(stamps), nbytes, st) == 0
        torch.cuda.synchronize()
        assert torch.equal(C0, C1) and torch.equal(S0, S1)
    else:
        g = torch.Generator(device="cuda").manual_seed(3)
        A = torch.randn((M, K), generator=g, device="cuda").half()
        B = torch.randn((K, N), generator=g, device="cuda").half()
        C0 = lib.fp16_gemm(A, B, tile=_lib.TILE_256x256)
        C1 = torch.zeros_like(C0)
        assert raw.llmmm_probe_fp16_gemm_phases(_lib.DTYPE_F16, p(A), p(B), p(C1), M, N, K, p(stamps), nbytes, st) == 0
        torch.cuda.synchronize()
        assert torch.equal(C0, C1)
    rec = stamps.cpu().numpy().reshape(-1, 12)
    for col in (0, 1):  # the 100 MHz clock and the shader's cycle counter
        t = rec[:, col:10:2]
        assert (t[:, 0] > 0).all() and (np.diff(t, axis=1) >= 0).all()
    assert (rec[:, 10] >= 0).all() and (rec[:, 10] <= rec[:, 5] - rec[:, 3]).all()  # waits lie inside the K loop
    small = torch.zeros(8, dtype=torch.int64, device="cuda")
    assert raw.llmmm_probe_fp16_gemm_phases(_lib.DTYPE_F16, p(C1), p(C1), p(C1), M, N, K, p(small), 64, st) == _lib.ERR_WORKSPACE
