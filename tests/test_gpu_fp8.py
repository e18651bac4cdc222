"""GPU parity tests of the FP8 blockwise GEMM (fp32 / bf16 output and fused C re-quantisation),
MFMA tile kernels and the small-M split-K kernel, through the C ABI, against the oracle.

Bars: fp32/bf16 output within 2e-2 relative (floored at row-block amax * 2^-7); fused output:
codes within one e4m3 step on >= 99.9 % of the elements, scales within 1e-3 relative."""
import os

import numpy as np
import pytest
import torch

from helpers import assert_fp8_gemm_close, assert_fused_close, fp8_inputs

pytestmark = pytest.mark.gpu
G = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
TILES = {"auto": -1, "256x256": 0, "128x256": 1, "256x128": 2, "128x128": 3}


def _gpu(*arrs):
    return [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in arrs]


def _run_all(lib, Aq, As, Bq, Bs, tile=-1, split_k=0, use_ws=True):
    M, K = Aq.shape
    N = Bq.shape[0]
    t = _gpu(Aq, As, Bq, Bs)
    ws = lib.make_workspace(2, M, N, K) if use_ws else None
    if use_ws and split_k > 1:  # an explicit split: split_k partial planes; poisoned, the library must not rely on their content
        ws = torch.full((split_k * M * N * 4,), 0xFF, dtype=torch.uint8, device="cuda")
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    Cb = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    Cq = torch.full((M, N), 0x55, dtype=torch.uint8, device="cuda")
    Cs = torch.full((N // 128, M), -1.0, dtype=torch.float32, device="cuda")
    kw = dict(workspace=ws, tile=tile, split_k=split_k)
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(*t, C, M, N, K, **kw)
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_bf16(*t, Cb, M, N, K, **kw)
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(*t, Cq, Cs, M, N, K, **kw)
    torch.cuda.synchronize()
    out = [C.cpu().numpy(), Cb.view(torch.int16).cpu().numpy().view(np.uint16), Cq.cpu().numpy(), Cs.cpu().numpy()]
    from llmmm_amd import _lib
    if tile == -1 and split_k == 0 and lib.query_config(_lib.OUT_F32, M, N, K)[0] != lib.query_config(_lib.OUT_FP8Q, M, N, K)[0]:
        # decode sizes: the library runs outputs without 1x128 groups in column strips and the fused output in the split-K
        # form -- other kernels, other summation orders.  The fp32 result of the fused output's own kernel, for the
        # bit-for-bit property below:
        Cx = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(*t, Cx, M, N, K, workspace=ws, tile=lib.query_config(_lib.OUT_FP8Q, M, N, K)[0])
        torch.cuda.synchronize()
        out.append(Cx.cpu().numpy())
    return tuple(out)


def _check_all(oracle, out, ref, what):
    C, Cb, Cq, Cs = out[:4]
    assert_fp8_gemm_close(C, ref, what + " fp32")
    # bf16 output is defined as the round-to-nearest-even cast of the fp32 result
    assert (Cb == oracle.f32_to_bf16_bits(C)).all(), what + " bf16 is not RNE(fp32 output)"
    assert_fp8_gemm_close(oracle.bf16_bits_to_f32(Cb), ref, what + " bf16")
    rq, rs = oracle.requant_c_1x128(ref)
    assert_fused_close(oracle, Cq, Cs, rq, rs, what + " fused")
    # the fused epilogue is exactly the oracle's re-quantisation applied to the kernel's own fp32 result
    own = out[4] if len(out) > 4 else C
    assert_fp8_gemm_close(own, ref, what + " fp32 of the fused output's kernel")
    oq, os_ = oracle.requant_c_1x128(own)
    assert (Cq == oq).all() and (Cs.view(np.uint32) == os_.view(np.uint32)).all(), what + " fused != requant(own fp32)"


@pytest.mark.parametrize("tile", ["256x256", "128x256", "256x128", "128x128"])
def test_tile_kernels_against_oracle(lib, oracle, tile):
    M, N, K = 512, 768, 1152  # 9 slices: odd count exercises both LDS stages' tails
    Aq, As, Bq, Bs = fp8_inputs(oracle, M, N, K, seed=3)
    ref = oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128)
    _check_all(oracle, _run_all(lib, Aq, As, Bq, Bs, tile=TILES[tile]), ref, "tile " + tile)


@pytest.mark.parametrize("tile", ["256x256", "128x128"])
@pytest.mark.parametrize("split", [2, 3, 7])
def test_tile_kernels_split_k(lib, oracle, tile, split):
    """Split-K of the tile kernels: partial planes added in split order by the reduce kernel;
    uneven slice counts per split (9 slices over 2, 3 and 7 splits)."""
    M, N, K = 256, 512, 1152
    Aq, As, Bq, Bs = fp8_inputs(oracle, M, N, K, seed=77)
    ref = oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128)
    out = _run_all(lib, Aq, As, Bq, Bs, tile=TILES[tile], split_k=split)
    _check_all(oracle, out, ref, "tile %s split %d" % (tile, split))
    again = _run_all(lib, Aq, As, Bq, Bs, tile=TILES[tile], split_k=split)
    assert all((a == b).all() for a, b in zip(out[1:], again[1:])) and (out[0].view(np.uint32) == again[0].view(np.uint32)).all()


@pytest.mark.parametrize("K", [128, 256, 384, 512, 640])
def test_short_k(lib, oracle, K):
    """1 to 5 slices through the 256x256 tile kernel: prologue-only, odd and even slice counts."""
    M, N = 256, 512
    Aq, As, Bq, Bs = fp8_inputs(oracle, M, N, K, seed=40 + K)
    ref = oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128)
    _check_all(oracle, _run_all(lib, Aq, As, Bq, Bs, tile=TILES["256x256"]), ref, "K=%d" % K)


@pytest.mark.parametrize("K", [128, 256, 384, 512, 640, 1152])
@pytest.mark.parametrize("tile,M", [("128x128", 128), ("128x256", 128), ("256x128", 256)])
def test_short_k_single_tile_row(lib, oracle, tile, M, K):
    """One tile row (M = BM): the 32-row-wave tiles stream the weights through their deep pipeline (3 or 4 stages);
    1 to 9 slices cover a K range shorter than the pipeline, equal to it, and longer."""
    N = 512
    Aq, As, Bq, Bs = fp8_inputs(oracle, M, N, K, seed=60 + K)
    ref = oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128)
    _check_all(oracle, _run_all(lib, Aq, As, Bq, Bs, tile=TILES[tile]), ref, "tile %s M=%d K=%d" % (tile, M, K))
    _check_all(oracle, _run_all(lib, Aq, As, Bq, Bs, tile=TILES[tile], split_k=2 if K >= 256 else 1), ref, "tile %s M=%d K=%d split" % (tile, M, K))


@pytest.mark.parametrize("tile", ["128x256", "256x128", "128x128"])
def test_small_tiles_with_more_workgroups_than_cus(lib, oracle, tile):
    """More than 256 workgroups: the 32-row-wave tiles run their two-stage form (two workgroups per CU) instead of
    the deep pipeline that the smaller test shapes get."""
    M, N, K = 2048, 4352, 384
    Aq, As, Bq, Bs = fp8_inputs(oracle, M, N, K, seed=77)
    ref = oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128)
    _check_all(oracle, _run_all(lib, Aq, As, Bq, Bs, tile=TILES[tile]), ref, "tile %s, 272+ workgroups" % tile)


def test_single_slice(lib, oracle):
    Aq, As, Bq, Bs = fp8_inputs(oracle, 128, 128, 128, seed=11)
    _check_all(oracle, _run_all(lib, Aq, As, Bq, Bs), oracle.fp8_gemm(Aq, As, Bq, Bs), "K=128")


def test_golden_fixture(lib, oracle):
    d = np.load(os.path.join(G, "fp8_gemm_128x256x256.npz"))
    out = _run_all(lib, d["aq"], d["a_scale_t"], d["bq_t"], d["b_scale"])
    _check_all(oracle, out, d["c_f32"], "golden 128x256x256")
    assert_fused_close(oracle, out[2], out[3], d["cq"], d["c_scale_t"], "golden fused")
    out5 = _run_all(lib, d["a5q"], d["a5_scale_t"], d["bq_t"], d["b_scale"])
    _check_all(oracle, out5, d["c5_f32"], "golden skinny M=5")
    assert_fused_close(oracle, out5[2], out5[3], d["c5q"], d["c5_scale_t"], "golden skinny fused")


def test_b_identity_known_answer(lib, oracle):
    # reference KAT (examples/005.fp8.mm.cu:2620-2634): B = I  =>  C == dequant(A), Cq == Aq, Cs == As
    M = N = K = 256
    rng = np.random.default_rng(21)
    A = rng.uniform(-5, 5, (M, K)).astype(np.float32)
    Aq, As = oracle.quant_fp8(A, 1, True)
    Bq, Bs = oracle.quant_fp8(np.eye(N, K, dtype=np.float32), 128, False)
    C, Cb, Cq, Cs = _run_all(lib, Aq, As, Bq, Bs)[:4]
    deq = oracle.dequant_fp8(Aq, As, 1, True)
    assert np.abs(C - deq).max() <= 4 * np.spacing(np.abs(deq).max())
    assert (Cq == Aq).all()
    assert np.abs(Cs - As).max() <= 1e-6 * As.max()


def test_zero_blocks_give_zero_codes_and_scales(lib, oracle):
    # a 1x128 group of zeros: the reference's unguarded 0 * (448/0) yields NaN codes (0x7F); this
    # library emits code 0 and scale 0 (documented deviation)
    Aq, As, Bq, Bs = fp8_inputs(oracle, 128, 256, 256, seed=5)
    Aq[7] = 0
    As[:, 7] = 0
    Bq[128:] = 0
    Bs[1] = 0
    C, Cb, Cq, Cs = _run_all(lib, Aq, As, Bq, Bs)[:4]
    assert not C[7].any() and not C[:, 128:].any()
    assert not Cq[7].any() and not Cq[:, 128:].any() and not Cs[:, 7].any() and not Cs[1].any()
    assert np.isfinite(oracle.e4m3_decode(Cq)).all()


@pytest.mark.parametrize("M", [1, 2, 15, 16, 17, 33, 64, 65, 96, 128])
@pytest.mark.parametrize("split", [1, 3, 8])
def test_skinny_kernel_against_oracle(lib, oracle, M, split):
    N, K = 384, 1024
    Aq, As, Bq, Bs = fp8_inputs(oracle, M, N, K, seed=M)
    ref = oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128)
    _check_all(oracle, _run_all(lib, Aq, As, Bq, Bs, tile=8, split_k=split), ref, "skinny M=%d S=%d" % (M, split))


@pytest.mark.parametrize("M", [17, 32, 33, 64, 65, 100, 128])
def test_skinny_row_groups_over_an_unsplit_long_k(lib, oracle, M):
    """K = 2560 unsplit: 20 slices of 32 rows are 80 KB of staged activations, so the rows go in groups of 32 (gridDim.z up to 4),
    each with its own fused epilogue.  Against the oracle, and bit for bit against one row of 128 x 128 tiles (no split on
    either side: the same additions in the same order)."""
    N, K = 512, 2560
    Aq, As, Bq, Bs = fp8_inputs(oracle, M, N, K, seed=100 + M)
    ref = oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128)
    got = _run_all(lib, Aq, As, Bq, Bs, tile=8, split_k=1)
    _check_all(oracle, got, ref, "skinny row groups M=%d" % M)
    tiles = _run_all(lib, Aq, As, Bq, Bs, tile=3, split_k=1)  # LLMMM_TILE_128x128
    for a, b in zip(got[:4], tiles[:4]):
        assert np.array_equal(np.asarray(a).view(np.uint8), np.asarray(b).view(np.uint8)), "differs from the 128 x 128 tiles"


def test_skinny_without_workspace_does_not_split(lib, oracle):
    Aq, As, Bq, Bs = fp8_inputs(oracle, 4, 256, 2560, seed=8)
    ref = oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128)
    _check_all(oracle, _run_all(lib, Aq, As, Bq, Bs, use_ws=False), ref, "skinny no workspace")


def test_split_k_is_deterministic_and_reusable(lib, oracle):
    # fixed-order reduction: bit-identical results run after run on the same (never initialised) workspace
    M, N, K = 16, 2560, 4096
    Aq, As, Bq, Bs = fp8_inputs(oracle, M, N, K, seed=4)
    t = _gpu(Aq, As, Bq, Bs)
    ws = lib.make_workspace(2, M, N, K)
    outs = []
    for _ in range(5):
        Cq = torch.empty((M, N), dtype=torch.uint8, device="cuda")
        Cs = torch.empty((N // 128, M), dtype=torch.float32, device="cuda")
        C = torch.empty((M, N), dtype=torch.float32, device="cuda")
        lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(*t, Cq, Cs, M, N, K, workspace=ws)
        lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(*t, C, M, N, K, workspace=ws)
        outs.append((Cq.clone(), Cs.clone(), C.clone()))
    torch.cuda.synchronize()
    for o in outs[1:]:
        assert all(torch.equal(a, b) for a, b in zip(o, outs[0]))
    assert_fp8_gemm_close(outs[0][2].cpu().numpy(), oracle.fp8_gemm(Aq, As, Bq, Bs), "split-K auto")


@pytest.mark.parametrize("name,N,K", [("qkv", 6144, 2560), ("o", 2560, 4096), ("gate_up", 19456, 2560), ("down", 2560, 9728)])
@pytest.mark.parametrize("M", [1, 16])
def test_cfg5_decode_shapes(lib, oracle, name, N, K, M):
    # the Qwen3-4B projection shapes at M in {1, 16}: full shapes, oracle on the whole (small-M) product
    Aq, As, Bq, Bs = fp8_inputs(oracle, M, N, K, seed=hash(name) % 1000)
    ref = oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128)
    _check_all(oracle, _run_all(lib, Aq, As, Bq, Bs), ref, "%s M=%d" % (name, M))


def _slab_check(lib, oracle, M, N, K, rows, seed, dist="cfg3"):
    """Full-size run on GPU-quantised inputs, all three outputs; the oracle checks a row slab, properties the rest.
    dist "cfg3": A ~ N(0,1) with 1 % of the K channels x 20, B ~ N(0, 0.02); "reference": both operands
    u / (|v| + 1) with u, v ~ U(-5, 5), the inputs of the reference's own driver (examples/005.fp8.mm.opt.cu:521-527)."""
    g = torch.Generator(device="cuda").manual_seed(seed)
    if dist == "cfg3":
        X = torch.randn((M, K), generator=g, device="cuda")
        X[:, torch.randperm(K, generator=g, device="cuda")[:max(1, -(-K // 100))]] *= 20
        W = torch.randn((N, K), generator=g, device="cuda") * 0.02
    else:
        def u(*shape):
            return torch.rand(shape, generator=g, device="cuda") * 10 - 5
        X = u(M, K) / (u(M, K).abs() + 1)
        W = u(N, K) / (u(N, K).abs() + 1)
    Aq, As = lib.quantize_activation(X)
    Bq, Bs = lib.quantize_weight(W)
    C = torch.empty((M, N), dtype=torch.float32, device="cuda")
    Cb = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    Cq = torch.empty((M, N), dtype=torch.uint8, device="cuda")
    Cs = torch.empty((N // 128, M), dtype=torch.float32, device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(Aq, As, Bq, Bs, C, M, N, K)
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_bf16(Aq, As, Bq, Bs, Cb, M, N, K)
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(Aq, As, Bq, Bs, Cq, Cs, M, N, K)
    torch.cuda.synchronize()
    r = torch.from_numpy(rows).cuda()
    ref = oracle.fp8_gemm(Aq[r].cpu().numpy(), As[:, r].contiguous().cpu().numpy(), Bq.cpu().numpy(), Bs.cpu().numpy(), promote=128)
    assert_fp8_gemm_close(C[r].cpu().numpy(), ref, "slab fp32")
    assert_fp8_gemm_close(Cb[r].float().cpu().numpy(), ref, "slab bf16")
    rq, rs = oracle.requant_c_1x128(ref)
    assert_fused_close(oracle, Cq[r].cpu().numpy(), Cs[:, r].contiguous().cpu().numpy(), rq, rs, "slab fused")
    # properties over the whole output: the bf16 output is the fp32 output rounded to nearest even (the same kernel
    # and split produce both), every 1x128 group has a code of magnitude 448 (its amax element),
    # scales equal amax/448 of the fp32 result, and re-quantising the dequantised output is the identity
    assert torch.equal(Cb, C.to(torch.bfloat16)), "bf16 output is not RNE(fp32 output)"
    dec = Cq.view(torch.float8_e4m3fn).float()
    assert (dec.abs().reshape(M, N // 128, 128).amax(-1) == 448).all()
    amax = C.abs().reshape(M, N // 128, 128).amax(-1)
    assert ((Cs.t() - amax / 448.0).abs() <= 1e-6 * amax / 448.0).all()  # torch's own division may differ in the last bit
    deq = dec * Cs.t().repeat_interleave(128, dim=1)
    assert (deq - C).abs().max() <= amax.max() / 448 * 16.5
    q2, s2 = lib.quantize_activation(deq)
    assert (q2.view(torch.float8_e4m3fn).float() - dec).abs().max() == 0 or torch.equal(q2, Cq)


def test_cfg3_cfg4_4096_full_size(lib, oracle):
    _slab_check(lib, oracle, 4096, 4096, 4096, np.r_[0:48, 2040:2088, 4048:4096], seed=3)


@pytest.mark.parametrize("name,N,K", [("qkv", 6144, 2560), ("o", 2560, 4096), ("gate_up", 19456, 2560), ("down", 2560, 9728)])
@pytest.mark.parametrize("M", [128, 2048])
def test_cfg5_prefill_shapes(lib, oracle, name, N, K, M):
    # every Qwen3-4B projection at its stated (N, K): whatever tile, hybrid launch or split the library picks for it
    _slab_check(lib, oracle, M, N, K, np.r_[0:32, M // 2 - 16:M // 2 + 16, M - 32:M] if M > 128 else np.r_[0:32, M - 32:M], seed=17)


def test_reference_driver_shape_4096x7168x2048(lib, oracle):
    # the one non-square problem the reference's own driver runs (examples/005.fp8.mm.opt.cu:515), with its inputs
    _slab_check(lib, oracle, 4096, 7168, 2048, np.r_[0:32, 2040:2072, 4064:4096], seed=0, dist="reference")


@pytest.mark.parametrize("tile,split", [("256x256", 0), ("128x128", 0), ("128x128", 2), (8, 1), (8, 3)])
def test_non_finite_operands(lib, oracle, tile, split):
    """NaN codes in A and in B and an infinite activation scale: the fp32 result is NaN / infinite exactly where the
    oracle's is, and the fused output is the oracle's re-quantisation of it bit for bit -- NaN elements give code
    0x7F whatever their sign, an infinite element makes the group's scale infinite and every finite element of the
    group a signed zero (examples/005.fp8.mm.opt.cu:439-454 evaluated on such values)."""
    skinny = tile == 8
    M, N, K = (48 if skinny else 256), 512, 512
    Aq, As, Bq, Bs = fp8_inputs(oracle, M, N, K, seed=31)
    Aq[3, 130] = 0x7F       # row 3: NaN in every column group
    Aq[5, 7] = 0xFF
    Bq[200, 300] = 0x7F     # column 200: NaN in every row
    As[1, 9] = np.inf       # row 9, second slice: infinite partial sums (NaN where that slice's sum is zero)
    As[2, 11] = -np.inf
    As[0, 13] = 1e38        # row 13: some sums overflow to infinity, their neighbours in the same 1x128 group stay finite
    ref = oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128)
    assert np.isnan(ref[3]).all() and np.isnan(ref[:, 200]).all() and np.isinf(ref[9]).any()
    assert np.isinf(ref[13, :128]).any() and np.isfinite(ref[13, :128]).any()
    C, Cb, Cq, Cs = _run_all(lib, Aq, As, Bq, Bs, tile=tile if skinny else TILES[tile], split_k=split)[:4]
    what = "tile %s split %d" % (tile, split)
    assert (np.isnan(C) == np.isnan(ref)).all(), what + ": NaN pattern differs from the oracle's"
    inf = np.isinf(ref)
    assert (np.isinf(C) == inf).all() and (np.sign(C[inf]) == np.sign(ref[inf])).all(), what + ": infinities differ"
    fin = np.isfinite(ref)
    assert_fp8_gemm_close(np.where(fin, C, 0), np.where(fin, ref, 0), what)
    assert (Cb == oracle.f32_to_bf16_bits(C))[fin].all()
    oq, os_ = oracle.requant_c_1x128(C)
    assert (Cq == oq).all(), what + ": fused codes differ from requant(own fp32) at %s" % np.argwhere(Cq != oq)[:5].tolist()
    assert (Cs.view(np.uint32) == os_.view(np.uint32)).all()
    assert (Cq[3] == 0x7F).all() and (Cq[:, 200] == 0x7F).all()


@pytest.mark.parametrize("tile,split", [("256x256", 0), ("128x128", 0), ("128x128", 2), (8, 1), (8, 2)])
def test_groups_whose_reciprocal_scale_overflows(lib, oracle, tile, split):
    """Rows whose results are so small (|C| <= 2^-120) that 448 / amax is not a finite fp32 number: every epilogue that
    multiplies by the reciprocal -- the tile kernels' own, the split-K reduce kernel, the weight-streaming kernel's -- must
    treat such a group like a group of zeros (codes 0, scale amax / 448) instead of writing NaN codes; the rows next to
    them are quantised as usual.  Bit for bit against the oracle's re-quantisation of the kernel's own fp32 result."""
    skinny = tile == 8
    M, N, K = (16 if skinny else 256), 256, 256
    Aq, As, Bq, Bs = fp8_inputs(oracle, M, N, K, seed=91)
    rng = np.random.default_rng(5)
    k0 = 37
    Bq[:, k0] = rng.choice(np.array([0x00, 0x01, 0x81, 0x02, 0x82], np.uint8), N)  # 0, +-2^-9, +-2^-8
    Bs[:] = np.float32(2.0 ** -44)
    for m in (0, 5):  # one non-zero activation (2^-9) with scale 2^-60: |C| in {0, 2^-122, 2^-121}
        Aq[m] = 0
        Aq[m, k0] = 0x01
        As[:, m] = np.float32(2.0 ** -60)
    ref = oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128)
    assert 0 < np.abs(ref[0]).max() <= 2.0 ** -120 and np.abs(ref[1]).max() > 2.0 ** -100
    C, Cb, Cq, Cs = _run_all(lib, Aq, As, Bq, Bs, tile=tile if skinny else TILES[tile], split_k=split)[:4]
    what = "tile %s split %d" % (tile, split)
    assert (C[[0, 5]] == ref[[0, 5]]).all(), what + ": one product per sum, nothing to round"
    oq, os_ = oracle.requant_c_1x128(C)
    assert (Cq == oq).all(), what + ": fused codes differ from requant(own fp32) at %s" % np.argwhere(Cq != oq)[:5].tolist()
    assert (Cs.view(np.uint32) == os_.view(np.uint32)).all(), what + ": scales"
    assert ((Cq[[0, 5]] & 0x7F) == 0).all() and (Cs[:, [0, 5]] > 0).all()
    assert (np.abs(oracle.e4m3_decode(Cq[1])).reshape(-1, 128).max(-1) == 448).all()
