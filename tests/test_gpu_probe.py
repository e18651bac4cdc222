"""The peak-rate probes run, leave their sink untouched and report rates of the right order of magnitude (they are
measurement aids: the test only guards against a probe that no longer executes its loop)."""
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
