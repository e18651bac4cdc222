"""The auto-tune driver on the GPU: tune_shape measures its candidates for a small shape and names one that the library
accepts; what it would write for that shape is a valid table row."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("M,N,K", [(16, 512, 1024), (128, 512, 1024)])
def test_tune_shape_returns_a_runnable_candidate(lib, oracle, M, N, K):
    from llmmm_amd import _lib, tune
    tile, split, results = tune.tune_shape(M, N, K, iters=5, rotate_bytes=8 << 20, verbose=False)
    assert (tile, split) in results and len(results) >= 3 and all(v > 0 for v in results.values())
    assert results[(tile, split)] == min(results.values())
    if M <= 64:
        assert tile == _lib.TILE_SKINNY and 1 <= split <= K // 128
    # the winner runs through the C ABI and meets the oracle
    import numpy as np
    from helpers import assert_fused_close, fp8_inputs
    Aq, As, Bq, Bs = fp8_inputs(oracle, M, N, K, seed=5)
    t = [torch.from_numpy(a).cuda() for a in (Aq, As, Bq, Bs)]
    Cq = torch.empty((M, N), dtype=torch.uint8, device="cuda")
    Cs = torch.empty((N // 128, M), dtype=torch.float32, device="cuda")
    ws = torch.empty(max(1, split) * M * N * 4, dtype=torch.uint8, device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(*t, Cq, Cs, M, N, K, workspace=ws, tile=tile, split_k=split)
    torch.cuda.synchronize()
    rq, rs = oracle.requant_c_1x128(oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128))
    assert_fused_close(oracle, Cq.cpu().numpy(), Cs.cpu().numpy(), rq, rs, "tuned candidate")
    rows = ([(M, N, K, split)], []) if tile == _lib.TILE_SKINNY else ([], [(M, N, K, tile, split)])
    assert tune.parse_file(tune.render_file(rows[0], rows[1], []))[:2] == rows


def test_tune_fp16_shape_returns_a_runnable_tile(lib, oracle):
    """The FP16 side of the driver: every tile that divides the shape is timed, the winner runs and meets the Kahan oracle."""
    import numpy as np
    from helpers import assert_fp16_close, fp16_inputs_uniform
    from llmmm_amd import tune
    M, N, K = 256, 512, 544
    best, results = tune.tune_fp16_shape(M, N, K, iters=5, verbose=False)
    assert best in results and len(results) == 5 and results[best] == min(results.values())
    A, B = fp16_inputs_uniform(M, N, K, seed=9)
    C = lib.fp16_gemm(torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda(), tile=best)
    torch.cuda.synchronize()
    assert_fp16_close(C.cpu().numpy(), oracle.kahan_gemm(A, B), "tuned fp16 tile")
    assert tune.parse_file(tune.render_file([], [], [(M, N, K, best, 1)]))[2] == [(M, N, K, best, 1)]


@pytest.mark.parametrize("N,K,tuned", [(4096, 14336, True), (5120, 5120, True), (8192, 8192, True),
                                       (6144, 6144, False), (12288, 4096, False), (9216, 3072, False)])
def test_the_library_choice_is_close_to_the_measured_best(lib, N, K, tuned):
    """Decode-sized M on projections of model families other than the one the kernels were developed on: three shapes the
    compiled-in table lists (a table hit) and three it has never seen (the heuristics).  The configuration the library
    picks by itself must run within 15 % of the best of the split counts timed here, on this GPU, in the same process --
    weights rotated over more copies than the caches hold, as the tune driver times them."""
    from llmmm_amd import _lib, mm, tune
    M = 16
    tile, split = lib.query_config(_lib.OUT_FP8Q, M, N, K)
    assert tile in (_lib.TILE_SKINNY, _lib.TILE_STRIP)
    rows = [r for r in tune.parse_header(open(tune.os.path.join(tune.HERE, "csrc", "tune_table.h")).read())[0] if r[1:3] == (N, K)]
    assert bool(rows) == tuned, "the test's idea of what the table lists is out of date"
    copies = max(2, -(-(512 << 20) // (N * K)))
    Aq, As, weights = tune._inputs(M, N, K, copies)
    Cq = torch.empty((M, N), dtype=torch.uint8, device="cuda")
    Cs = torch.empty((N // 128, M), dtype=torch.float32, device="cuda")
    ws = torch.empty(16 * M * N * 4, dtype=torch.uint8, device="cuda")

    def time_of(**cfg):
        state = {"i": 0}

        def step():
            Bq, Bs = weights[state["i"] % copies]
            state["i"] += 1
            mm.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(Aq, As, Bq, Bs, Cq, Cs, M, N, K, workspace=ws, **cfg)
        return min(tune._time_ms(step, 30, graph=True) for _ in range(2))

    auto = time_of()
    cands = {s: time_of(tile=_lib.TILE_SKINNY, split_k=s) for s in (1, 2, 3, 4, 5, 6, 8, 10) if s <= K // 256}
    best = min(cands, key=cands.get)
    if auto > 1.15 * cands[best]:  # a timing, not a result: one more look at both before calling it
        auto, cands[best] = min(auto, time_of()), min(cands[best], time_of(tile=_lib.TILE_SKINNY, split_k=best))
    assert auto <= 1.15 * cands[best], "M %d N %d K %d: the library's %s takes %.2f us, %d splits %.2f us" % (M, N, K, (tile, split), auto * 1e3, best, cands[best] * 1e3)
