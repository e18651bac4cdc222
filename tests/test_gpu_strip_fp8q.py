"""The fused 1x128 re-quantisation of C from column strips (decode-sized M on the projections with few column groups):
one launch, in which the workgroups of a 128-column group (eight 16-column strips, or four 32-column ones) exchange their
row maxima through device memory.
Codes and scales must be the oracle's re-quantisation of the strip kernel's own fp32 result bit for bit -- launch after
launch on one stream with changing inputs (a stale maximum from an earlier launch would show as a wrong scale), in
replayed graphs, on several streams at once -- and no wave may ever have hit the bound on its wait."""
import ctypes

import numpy as np
import pytest
import torch

from helpers import assert_fused_close, fp8_inputs

pytestmark = pytest.mark.gpu
STRIP, SKINNY = 9, 8


def _dev(*arrs):
    return [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in arrs]


def _timeouts():
    from llmmm_amd import _lib
    n = ctypes.c_uint(99)
    assert _lib.lib.llmmm_probe_strip_exchange_timeouts(ctypes.byref(n)) == 0
    return n.value


def _fused(lib, t, M, N, K, pre=False, tile=STRIP, guard=2):
    Cq = torch.full((M + guard, N), 0x55, dtype=torch.uint8, device="cuda")
    Cs = torch.full((N // 128, M), -1.0, dtype=torch.float32, device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(*t, Cq[:M], Cs, M, N, K, tile=tile, b_preshuffled=pre)
    return Cq, Cs


def _check(oracle, lib, t, M, N, K, Cq, Cs, what, pre=False):
    C32 = torch.empty((M, N), dtype=torch.float32, device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(*t, C32, M, N, K, tile=STRIP, b_preshuffled=pre)
    torch.cuda.synchronize()
    assert (Cq[M:] == 0x55).all(), what + ": rows behind M were written"
    oq, os_ = oracle.requant_c_1x128(C32.cpu().numpy())
    got_q, got_s = Cq[:M].cpu().numpy(), Cs.cpu().numpy()
    assert (got_s.view(np.uint32) == os_.view(np.uint32)).all(), what + ": scales differ from amax / 448 of the kernel's own fp32 result"
    assert (got_q == oq).all(), what + ": codes differ from requant(own fp32) at %s" % np.argwhere(got_q != oq)[:5].tolist()


# K / 128 from 8 (one slice per wave) over uneven shares (20, 76 slices: tail slices) to 80; one, three and 48 column groups
@pytest.mark.parametrize("M,N,K", [(1, 2560, 4096), (16, 2560, 4096), (1, 6144, 2560), (16, 6144, 2560), (1, 2560, 9728), (8, 2560, 9728),
                                   (5, 128, 1024), (3, 384, 10240), (16, 256, 1152),
                                   # 32-column strips (6144 x 2560 above): tail slices, exactly 256 strips, a larger K
                                   (3, 4608, 1152), (16, 4608, 1152), (2, 8192, 1024), (16, 6144, 4096),
                                   # 448 16-column strips (56 groups) of a matrix too large for wide ones: two workgroups on most CUs
                                   (2, 7168, 5120)])
@pytest.mark.parametrize("pre", [False, True])
def test_against_oracle(lib, oracle, M, N, K, pre):
    Aq, As, Bq, Bs = fp8_inputs(oracle, M, N, K, seed=M + N + K)
    t = _dev(Aq, As, Bq, Bs)
    if pre:
        t[2] = lib.preshuffle_weight(t[2])
    Cq, Cs = _fused(lib, t, M, N, K, pre)
    what = "fused strips %dx%dx%d pre %d" % (M, N, K, pre)
    _check(oracle, lib, t, M, N, K, Cq, Cs, what, pre)
    ref = oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128)
    rq, rs = oracle.requant_c_1x128(ref)
    assert_fused_close(oracle, Cq[:M].cpu().numpy(), Cs.cpu().numpy(), rq, rs, what)
    assert _timeouts() == 0


def test_back_to_back_launches_with_changing_inputs(lib, oracle):
    """Twelve launches on one stream with no synchronisation between them, the activations scaled differently for each
    (so every launch has other row maxima) and two shapes taking turns -- one in 16-column strips, the other in 32-column
    ones, groups 0 .. 19 of the exchange area serving both, so a width that left a group's slots in a state the other
    cannot read would show: every launch must deliver the scales of its own inputs."""
    shapes = [(16, 2560, 4096), (4, 6144, 2560)]
    cases = []
    for j in range(12):
        M, N, K = shapes[j % 2]
        Aq, As, Bq, Bs = fp8_inputs(oracle, M, N, K, seed=50 + j % 2)
        As = (As * np.float32(2.0 ** (j - 6))).astype(np.float32)
        cases.append((M, N, K, _dev(Aq, As, Bq, Bs)))
    outs = [_fused(lib, t, M, N, K) for M, N, K, t in cases]
    torch.cuda.synchronize()
    for j, ((M, N, K, t), (Cq, Cs)) in enumerate(zip(cases, outs)):
        _check(oracle, lib, t, M, N, K, Cq, Cs, "launch %d" % j)
    assert _timeouts() == 0


def test_graph_replays_and_two_streams(lib, oracle):
    """A captured launch replayed four times with the activations rewritten between the replays, eager work and
    synchronisations in between, and a second stream (an exchange area of its own) running the same shape concurrently."""
    M, N, K = 16, 2560, 4096
    base = fp8_inputs(oracle, M, N, K, seed=77)
    t = _dev(*base)
    other = _dev(*fp8_inputs(oracle, M, N, K, seed=78))
    Cq = torch.full((M, N), 0x55, dtype=torch.uint8, device="cuda")
    Cs = torch.full((N // 128, M), -1.0, dtype=torch.float32, device="cuda")
    side, side2 = torch.cuda.Stream(), torch.cuda.Stream()
    with torch.cuda.stream(side):
        lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(*t, Cq, Cs, M, N, K)  # warm-up outside the capture
        side.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(*t, Cq, Cs, M, N, K)
    torch.cuda.synchronize()
    for rep in range(4):
        t[1].copy_(torch.from_numpy((base[1] * np.float32(3.0 ** rep)).astype(np.float32)))
        Cq.fill_(0x55)
        torch.cuda.synchronize()
        with torch.cuda.stream(side2):
            o_q, o_s = _fused(lib, other, M, N, K, guard=0)
        g.replay()
        torch.cuda.synchronize()
        _check(oracle, lib, t, M, N, K, Cq, Cs, "replay %d" % rep)
        _check(oracle, lib, other, M, N, K, o_q, o_s, "second stream, round %d" % rep)
    assert _timeouts() == 0


def test_library_choice_and_fallbacks(lib, oracle):
    """Auto configuration takes strips for these shapes; the split-K form named explicitly still works and agrees within
    the fused bar (other summation order); M = 17 is refused for the strips' fp8 output."""
    from llmmm_amd import _lib
    M, N, K = 4, 2560, 9728
    assert lib.query_config(_lib.OUT_FP8Q, M, N, K) == (STRIP, 1)
    assert lib.query_config(_lib.OUT_FP8Q, 16, N, K)[0] == SKINNY and lib.query_config(_lib.OUT_FP8Q, 8, 6144, 2560)[0] == SKINNY
    Aq, As, Bq, Bs = fp8_inputs(oracle, M, N, K, seed=5)
    t = _dev(Aq, As, Bq, Bs)
    Cq = torch.full((M, N), 0x55, dtype=torch.uint8, device="cuda")
    Cs = torch.full((N // 128, M), -1.0, dtype=torch.float32, device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(*t, Cq, Cs, M, N, K)  # auto, no workspace needed
    _check(oracle, lib, t, M, N, K, Cq, Cs, "auto")
    ws = lib.make_workspace(_lib.OUT_FP8Q, M, N, K)
    Sq, Ss = torch.empty_like(Cq), torch.empty_like(Cs)
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(*t, Sq, Ss, M, N, K, tile=SKINNY, workspace=ws)
    torch.cuda.synchronize()
    assert_fused_close(oracle, Sq.cpu().numpy(), Ss.cpu().numpy(), Cq.cpu().numpy(), Cs.cpu().numpy(), "split-K form vs strips")
    with pytest.raises(RuntimeError):
        lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(*_dev(*fp8_inputs(oracle, 17, 256, 1024, seed=1)),
                                                                             torch.empty((17, 256), dtype=torch.uint8, device="cuda"),
                                                                             torch.empty((2, 17), dtype=torch.float32, device="cuda"), 17, 256, 1024, tile=STRIP)
    assert _timeouts() == 0


def test_more_streams_than_exchange_areas(lib, oracle):
    """Every stream the library meets gets an exchange area of its own; there are 32.  Forty streams, one call each with the
    caller's workspace at hand: the calls beyond the areas take the split-K form (two kernels) -- every result meets the
    fused bar, and those that ran in strips equal the first stream's bit for bit."""
    from llmmm_amd import _lib
    M, N, K = 8, 2560, 4096
    Aq, As, Bq, Bs = fp8_inputs(oracle, M, N, K, seed=123)
    t = _dev(Aq, As, Bq, Bs)
    ws = lib.make_workspace(_lib.OUT_FP8Q, M, N, K)
    assert ws is not None
    rq, rs = oracle.requant_c_1x128(oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128))
    streams = [torch.cuda.Stream() for _ in range(40)]
    outs = []
    for st in streams:
        Cq = torch.full((M, N), 0x55, dtype=torch.uint8, device="cuda")
        Cs = torch.full((N // 128, M), -1.0, dtype=torch.float32, device="cuda")
        with torch.cuda.stream(st):
            lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(*t, Cq, Cs, M, N, K, workspace=ws)
        st.synchronize()  # the calls beyond the areas share the one workspace: one after the other
        outs.append((Cq.cpu().numpy(), Cs.cpu().numpy()))
    same = 0
    for q, s in outs:
        assert_fused_close(oracle, q, s, rq, rs, "stream")
        same += int((q == outs[0][0]).all() and (s.view(np.uint32) == outs[0][1].view(np.uint32)).all())
    assert same >= 1  # (how many streams found an area depends on what ran in this process before)
    assert _timeouts() == 0


def test_non_finite_operands_and_tiny_groups(lib, oracle):
    """NaN codes in A and B, an infinite activation scale, a row of zeros and a row whose results are so small that
    448 / amax overflows: the exchanged maxima never become NaN (fmaxf drops it), an infinite maximum travels as it is,
    and codes and scales are the oracle's re-quantisation of the strip kernel's own fp32 result bit for bit."""
    M, N, K = 16, 384, 1024
    Aq, As, Bq, Bs = fp8_inputs(oracle, M, N, K, seed=31)
    Aq[3, 130] = 0x7F        # row 3: NaN in every column
    Bq[200, 300] = 0xFF      # column 200: NaN in every row
    As[1, 9] = np.inf        # row 9, second slice
    As[0, 13] = 1e38         # row 13: some sums overflow
    Aq[5] = 0                # row 5: all zeros
    k0 = 37
    Bq[:, k0] = np.random.default_rng(2).choice(np.array([0x00, 0x01, 0x81, 0x02], np.uint8), N)
    Bs[:] = np.float32(2.0 ** -44)
    Aq[7] = 0
    Aq[7, k0] = 0x01
    As[:, 7] = np.float32(2.0 ** -60)   # row 7: |C| <= 2^-121
    t = _dev(Aq, As, Bq, Bs)
    Cq, Cs = _fused(lib, t, M, N, K)
    _check(oracle, lib, t, M, N, K, Cq, Cs, "non-finite operands")
    q, s = Cq[:M].cpu().numpy(), Cs.cpu().numpy()
    assert (q[3] == 0x7F).all() and (q[:, 200] == 0x7F).all()
    keep = np.arange(N) != 200  # (0 * NaN = NaN in column 200)
    assert (q[5, keep] == 0).all() and (s[:, 5] == 0).all()
    assert ((q[7, keep] & 0x7F) == 0).all() and (s[:, 7] > 0).all() and (s[:, 7] < 1e-38).all()
    assert np.isinf(s[:, 9]).any()
    assert _timeouts() == 0


def test_beside_a_kernel_that_fills_the_chip(lib, oracle):
    """The strips of a group wait for each other, so they rely on all of them being dispatched.  While another stream runs
    256 x 256-tile GEMMs -- one workgroup per CU, whose LDS leaves no room for a strip beside it -- the strips get CUs only as
    GEMM workgroups end, a few at a time: every launch must still deliver the bits of an undisturbed one, and no wait may
    have run into its bound."""
    M, N, K = 16, 2560, 4096
    Aq, As, Bq, Bs = fp8_inputs(oracle, M, N, K, seed=9)
    t = _dev(Aq, As, Bq, Bs)
    ref_q, ref_s = _fused(lib, t, M, N, K, guard=0)
    torch.cuda.synchronize()
    A = torch.randn(4096, 4096, device="cuda", dtype=torch.float16)
    B = torch.randn(4096, 4096, device="cuda", dtype=torch.float16)
    C = torch.empty_like(A)
    big, small = torch.cuda.Stream(), torch.cuda.Stream()
    outs = [_fused(lib, t, M, N, K, guard=0) for _ in range(40)]  # buffers made (and filled once) ahead of the contended run
    for q, s in outs:
        q.fill_(0x55), s.fill_(-1.0)
    torch.cuda.synchronize()
    with torch.cuda.stream(big):
        for _ in range(30):
            lib.fp16_mm(A, B, C, 4096, 4096, 4096)
    with torch.cuda.stream(small):
        for q, s in outs:
            lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(*t, q, s, M, N, K, tile=STRIP)
    torch.cuda.synchronize()
    for q, s in outs:
        assert torch.equal(q, ref_q) and torch.equal(s.view(torch.int32), ref_s.view(torch.int32))
    assert _timeouts() == 0
