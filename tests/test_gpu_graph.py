"""Every entry point is one or two plain kernel launches on the caller's stream: captured into a HIP graph and
replayed several times -- with eager work and synchronisations in between -- each replay must reproduce the eager
result bit for bit (split-K runs included: their planes are plain scratch, rewritten by every call)."""
import numpy as np
import pytest
import torch

from helpers import fp8_inputs

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("M,split_k,kind", [(16, 5, "fp8q"), (1, 1, "fp8q"), (128, 4, "fp8q"), (256, 2, "fp8q"), (256, 1, "fp8q"),
                                            (16, 3, "swiglu"), (256, 1, "swiglu"), (128, 1, "swiglu")])
def test_graph_replays_match_eager(lib, oracle, M, split_k, kind):
    N, K = 1024, 1536
    Aq, As, Bq, Bs = fp8_inputs(oracle, M, N, K, seed=90 + M)
    t = [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in (Aq, As, Bq, Bs)]
    n_out = N // 2 if kind == "swiglu" else N
    ws = torch.empty(max(split_k, 1) * M * N * 4, dtype=torch.uint8, device="cuda")
    f = (lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__swiglu__C_1x128__output_fp8 if kind == "swiglu"
         else lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8)

    def run(Cq, Cs):
        f(*t, Cq, Cs, M, N, K, workspace=ws, split_k=split_k)

    eager_q = torch.empty((M, n_out), dtype=torch.uint8, device="cuda")
    eager_s = torch.empty((n_out // 128, M), dtype=torch.float32, device="cuda")
    run(eager_q, eager_s)
    torch.cuda.synchronize()
    gq, gs = torch.empty_like(eager_q), torch.empty_like(eager_s)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run(gq, gs)  # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        run(gq, gs)
    for rep in range(4):
        gq.fill_(0x55)
        gs.fill_(-1.0)
        ws.fill_(0xFF)  # eager work between the replays; the planes hold garbage again
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(gq, eager_q) and torch.equal(gs, eager_s), "replay %d differs from the eager result" % rep
        x = torch.randn(1 << 16, device="cuda")
        (x * 2).sum().item()  # unrelated eager work and a synchronisation


def test_graph_of_the_other_entry_points(lib, oracle):
    """FP16 GEMM, the quantiser, RMSNorm + quantiser and the weight pre-shuffle in one graph."""
    rng = np.random.default_rng(3)
    A = torch.from_numpy(rng.uniform(-1, 1, (256, 256)).astype(np.float16)).cuda()
    B = torch.from_numpy(rng.uniform(-1, 1, (256, 256)).astype(np.float16)).cuda()
    X = torch.from_numpy(rng.standard_normal((64, 512)).astype(np.float32)).cuda()
    w = torch.ones(512, device="cuda")
    Wq = torch.from_numpy(rng.integers(0, 256, (256, 512), dtype=np.uint8)).cuda()
    from llmmm_amd import _lib
    raw = _lib.lib
    C = torch.empty((256, 256), dtype=torch.float16, device="cuda")
    q1, s1 = torch.empty((64, 512), dtype=torch.uint8, device="cuda"), torch.empty((4, 64), device="cuda")
    q2, s2 = torch.empty_like(q1), torch.empty_like(s1)
    Wp = torch.empty_like(Wq)

    def run():
        st = torch.cuda.current_stream().cuda_stream
        assert raw.llmmm_fp16_gemm(0, A.data_ptr(), B.data_ptr(), C.data_ptr(), 256, 256, 256, 0, st) == 0
        assert raw.llmmm_quant_fp8(_lib.QUANT_1x128_T, X.data_ptr(), q1.data_ptr(), s1.data_ptr(), 64, 512, st) == 0
        assert raw.llmmm_rmsnorm_quant_fp8(_lib.DTYPE_F32, X.data_ptr(), w.data_ptr(), 1e-6, q2.data_ptr(), s2.data_ptr(), 64, 512, st) == 0
        assert raw.llmmm_fp8_preshuffle_b(Wq.data_ptr(), Wp.data_ptr(), 256, 512, st) == 0

    run()
    torch.cuda.synchronize()
    want = [x.clone() for x in (C, q1, s1, q2, s2, Wp)]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()
    torch.cuda.current_stream().wait_stream(side)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        run()
    for rep in range(3):
        for x in (C, q1, s1, q2, s2, Wp):
            x.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for got, exp in zip((C, q1, s1, q2, s2, Wp), want):
            assert torch.equal(got, exp), "replay %d" % rep
