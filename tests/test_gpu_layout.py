"""Offline layout helpers on the GPU, through the C ABI: the weight pre-shuffle into MFMA operand
order (counterpart of construct_m16n8k32_B_layout, src/base/base.cu:222-271) and
transpose_matrix__aligned_128 (src/base/base.cu:124-153).  Byte work: everything is bit-exact.

* the pre-shuffle equals the oracle's image, and the inverse restores the input exactly (the
  reference's own check of its permutation, examples/005.fp8.mm.opt.cu:710-765);
* every FP8 GEMM kernel gives bit-identical results from pre-shuffled and from row-major weights;
* the transpose equals numpy's, as the reference's test compares bytes
  (test/transpose_matrix__aligned_128_test.cc:16-35)."""
import numpy as np
import pytest
import torch

from helpers import fp8_inputs

pytestmark = pytest.mark.gpu
TILES = {"256x256": 0, "128x256": 1, "256x128": 2, "128x128": 3, "skinny": 8}


@pytest.mark.parametrize("N,K", [(16, 128), (48, 384), (2560, 4096), (6144, 2560), (304, 640)])
def test_preshuffle_equals_oracle_and_inverts(lib, oracle, N, K):
    rng = np.random.default_rng(N + K)
    x = rng.integers(0, 256, (N, K), dtype=np.uint8)
    tx = torch.from_numpy(x).cuda()
    tp = torch.full((N, K), 0x55, dtype=torch.uint8, device="cuda")
    lib.construct_mfma_B_layout(tp, tx, N, K)
    back = torch.full((N, K), 0xAA, dtype=torch.uint8, device="cuda")
    lib.restore_B_layout(back, tp, N, K)
    torch.cuda.synchronize()
    assert np.array_equal(tp.cpu().numpy(), oracle.preshuffle_b(x))
    assert np.array_equal(back.cpu().numpy(), x)
    assert np.array_equal(tx.cpu().numpy(), x), "the source was modified"


@pytest.mark.parametrize("dtype", [np.uint8, np.float32])
@pytest.mark.parametrize("M,N", [(128, 128), (256, 384), (4096, 2560), (128, 9728)])
def test_transpose_equals_numpy(lib, oracle, M, N, dtype):
    rng = np.random.default_rng(M + N)
    x = rng.integers(0, 256, (M, N), dtype=np.uint8) if dtype is np.uint8 else rng.standard_normal((M, N), dtype=np.float32)
    tx = torch.from_numpy(x).cuda()
    ty = torch.empty((N, M), dtype=tx.dtype, device="cuda")
    lib.transpose_matrix__aligned_128(ty, tx, M, N)
    torch.cuda.synchronize()
    ref = oracle.transpose_aligned_128(x)
    assert np.array_equal(ty.cpu().numpy().view(np.uint8), ref.view(np.uint8))


def test_transpose_round_trip_full_size(lib):
    """Full-size case through a size-independent property: transposing twice is the identity."""
    M, N = 4096, 19456
    x = torch.randint(0, 256, (M, N), dtype=torch.uint8, device="cuda")
    y = torch.empty((N, M), dtype=torch.uint8, device="cuda")
    z = torch.empty((M, N), dtype=torch.uint8, device="cuda")
    lib.transpose_matrix__aligned_128(y, x, M, N)
    lib.transpose_matrix__aligned_128(z, y, N, M)
    torch.cuda.synchronize()
    assert torch.equal(z, x) and torch.equal(y, x.t().contiguous())


def test_alignment_errors(lib):
    a = torch.zeros((128, 256), dtype=torch.uint8, device="cuda")
    b = torch.zeros((128, 256), dtype=torch.uint8, device="cuda")
    with pytest.raises(RuntimeError, match="K must be greater than 0 and divisible by 128."):
        lib.construct_mfma_B_layout(b, a, 256, 100)
    with pytest.raises(RuntimeError, match="M or N can't be divided 128."):
        lib.transpose_matrix__aligned_128(b, a, 100, 256)
    with pytest.raises(RuntimeError, match="T is not supported."):
        lib.transpose_matrix__aligned_128(b.view(torch.int16), a.view(torch.int16), 128, 128)


def _run_three(lib, t, M, N, K, tile, split_k, pre):
    ws = torch.full((max(split_k, 1) * M * N * 4,), 0xFF, dtype=torch.uint8, device="cuda") if split_k > 1 else lib.make_workspace(2, M, N, K)
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    Cb = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    Cq = torch.full((M, N), 0x55, dtype=torch.uint8, device="cuda")
    Cs = torch.full((N // 128, M), -1.0, dtype=torch.float32, device="cuda")
    kw = dict(workspace=ws, tile=tile, split_k=split_k, b_preshuffled=pre)
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(*t, C, M, N, K, **kw)
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_bf16(*t, Cb, M, N, K, **kw)
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(*t, Cq, Cs, M, N, K, **kw)
    torch.cuda.synchronize()
    return C, Cb.view(torch.int16), Cq, Cs


@pytest.mark.parametrize("tile,M,split_k", [("256x256", 512, 1), ("128x256", 384, 1), ("256x128", 512, 1), ("128x128", 384, 1),
                                             ("256x256", 256, 3), ("128x128", 128, 2), ("128x256", 128, 1), ("256x128", 256, 1), ("256x256", 256, 1),
                                             ("skinny", 1, 1), ("skinny", 16, 3), ("skinny", 33, 1), ("skinny", 64, 8),
                                             ("skinny", 100, 1), ("skinny", 128, 3)])
def test_gemm_bit_identical_over_both_weight_layouts(lib, oracle, tile, M, split_k):
    N, K = 768, 1152
    Aq, As, Bq, Bs = fp8_inputs(oracle, M, N, K, seed=11)
    t_rows = [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in (Aq, As, Bq, Bs)]
    t_pre = list(t_rows)
    t_pre[2] = lib.preshuffle_weight(t_rows[2])
    rows = _run_three(lib, t_rows, M, N, K, TILES[tile], split_k, False)
    pre = _run_three(lib, t_pre, M, N, K, TILES[tile], split_k, True)
    for a, b, what in zip(rows, pre, ("fp32", "bf16", "codes", "scales")):
        assert not torch.isnan(a.float()).any() if what == "fp32" else True
        assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), "%s differs between the weight layouts (tile %s, M %d, split %d)" % (what, tile, M, split_k)
    # and the row-major result is the oracle's (the full parity bars live in test_gpu_fp8.py)
    ref = oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128)
    err = np.abs(rows[0].cpu().numpy() - ref)
    assert (err <= 2e-2 * np.maximum(np.abs(ref), np.abs(ref).max() * 2.0 ** -7)).all()


def test_decode_shape_pre_shuffled_against_oracle(lib, oracle):
    """Qwen3-4B gate_up at M = 16 (the shape the pre-shuffle is for), auto configuration, against the oracle."""
    from helpers import assert_fused_close
    M, N, K = 16, 19456, 2560
    Aq, As, Bq, Bs = fp8_inputs(oracle, M, N, K, seed=12)
    t = [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in (Aq, As, Bq, Bs)]
    t[2] = lib.preshuffle_weight(t[2])
    Cq = torch.full((M, N), 0x55, dtype=torch.uint8, device="cuda")
    Cs = torch.full((N // 128, M), -1.0, dtype=torch.float32, device="cuda")
    lib.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(*t, Cq, Cs, M, N, K, workspace=lib.make_workspace(2, M, N, K),
                                                                         b_preshuffled=True)
    torch.cuda.synchronize()
    rq, rs = oracle.requant_c_1x128(oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128))
    assert_fused_close(oracle, Cq.cpu().numpy(), Cs.cpu().numpy(), rq, rs, "gate_up M=16 pre-shuffled")


def test_golden_fixture(lib):
    import os
    d = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "layout_48x384.npz"))
    bt = torch.from_numpy(d["bt"]).cuda()
    bp = torch.empty_like(bt)
    lib.construct_mfma_B_layout(bp, bt, 48, 384)
    t_in = torch.from_numpy(d["t_in"]).cuda()
    t_out = torch.empty((256, 128), dtype=torch.uint8, device="cuda")
    lib.transpose_matrix__aligned_128(t_out, t_in, 128, 256)
    torch.cuda.synchronize()
    assert np.array_equal(bp.cpu().numpy(), d["bp"]) and np.array_equal(t_out.cpu().numpy(), d["t_out"])
