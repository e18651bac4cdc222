"""GPU quantiser (through the C ABI) against the oracle: bit-exact codes and scales."""
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
G = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _run(lib, x, quant_m, transpose, sshape):
    M, N = x.shape
    q = torch.full((M, N), 0x55, dtype=torch.uint8, device="cuda")
    s = torch.full(sshape, -1.0, dtype=torch.float32, device="cuda")
    lib.fp8_blockwise_symmetric_quantization(torch.from_numpy(x).cuda(), q, s, M, N, quant_m, 128, transpose)
    torch.cuda.synchronize()
    return q.cpu().numpy(), s.cpu().numpy()


@pytest.mark.parametrize("M,N", [(512, 1024), (77, 384), (1, 2560), (16, 128), (130, 260), (300, 132), (1, 4)])
@pytest.mark.parametrize("quant_m,transpose", [(1, True), (1, False), (128, False), (128, True)])
def test_bit_exact_against_oracle(lib, oracle, M, N, quant_m, transpose):
    rng = np.random.default_rng(M * 1000 + N)
    x = rng.normal(0, 1, (M, N)).astype(np.float32)
    x[:, ::37] *= 20
    if M > 3:
        x[3, :] = 0
    rq, rs = oracle.quant_fp8(x, quant_m, transpose)
    q, s = _run(lib, x, quant_m, transpose, rs.shape)
    assert (q == rq).all()
    if quant_m == 128 and transpose:
        # row stride M with only ceil(M/128) entries used per row (the reference's layout)
        mb = -(-M // 128)
        assert (s[:, :mb].view(np.uint32) == rs[:, :mb].view(np.uint32)).all()
    else:
        assert (s.view(np.uint32) == rs.view(np.uint32)).all()


def test_golden_fixture(lib):
    d = np.load(os.path.join(G, "quant_130x256.npz"))
    q, s = _run(lib, d["x"], 1, True, d["s_1x128_t"].shape)
    assert (q == d["q_1x128"]).all() and (s == d["s_1x128_t"]).all()
    q, s = _run(lib, d["x"], 128, False, d["s_128x128"].shape)
    assert (q == d["q_128x128"]).all() and (s == d["s_128x128"]).all()


def test_special_values(lib, oracle):
    x = np.zeros((4, 128), np.float32)
    x[1, :] = 448.0
    x[1, 5] = -448.0
    x[2, 0] = 1e30
    x[2, 1] = -3e29
    x[2, 2] = 1e-30
    x[3, :] = np.float32(1e-40)  # denormal amax: scale underflows, codes stay finite
    rq, rs = oracle.quant_fp8(x, 1, True)
    q, s = _run(lib, x, 1, True, rs.shape)
    assert (q == rq).all() and (s.view(np.uint32) == rs.view(np.uint32)).all()
    assert (q[0] == 0).all() and s[0, 0] == 0


def test_full_size_activation_and_weight(lib, oracle):
    # cfg3 shapes: activations 4096x4096 (1x128, transposed scales), weights 4096x4096 (128x128)
    g = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randn((4096, 4096), generator=g, device="cuda")
    x[:, torch.randperm(4096, generator=g, device="cuda")[:41]] *= 20
    q, s = lib.quantize_activation(x)
    wq, ws = lib.quantize_weight(x * 0.02)
    torch.cuda.synchronize()
    xs = x[:256].cpu().numpy()
    rq, rs = oracle.quant_fp8(xs, 1, True)
    assert (q[:256].cpu().numpy() == rq).all() and (s[:, :256].cpu().numpy() == rs).all()
    rq, rs = oracle.quant_fp8((x * 0.02)[:256].cpu().numpy(), 128, False)
    assert (wq[:256].cpu().numpy() == rq).all() and (ws[:2].cpu().numpy() == rs).all()
    # size-independent invariant over the whole matrix: |q| <= 448 and every 1x128 block reaches +-448
    dec = q.view(torch.float8_e4m3fn).float().abs().reshape(4096, 32, 128).amax(-1)
    assert (dec == 448).all()


def test_quotients_on_rounding_boundaries(lib, oracle):
    """The quantiser decides most codes from x * rcp(s) and divides only where that cannot settle the rounding.  Rows
    built to sit on the boundaries: quotients that are exact ties of the 3-bit mantissa (power-of-two scales, so the tie
    survives the division), and, for arbitrary scales, values up to three fp32 steps either side of every tie."""
    vals = oracle.e4m3_decode(np.arange(0, 0x7F, dtype=np.uint8)).astype(np.float64)  # every finite code >= 0
    mids = ((vals[:-1] + vals[1:]) / 2).astype(np.float32)                             # 126 ties, exact in fp32
    rng = np.random.default_rng(11)
    rows = []

    def row(v, amax):
        r = np.zeros(384, np.float32)
        for gi, sign in enumerate((1.0, -1.0, None)):
            sg = np.float32(sign) if sign else (rng.integers(0, 2, 126) * 2 - 1).astype(np.float32)
            r[gi * 128] = amax                      # every 128-column group has the same amax, hence the same scale
            r[gi * 128 + 1:gi * 128 + 127] = v * sg
        rows.append(r)

    for k in (-20, -3, 0, 5, 30):                   # s = 2^k exactly
        row(mids * np.float32(2.0 ** k), np.float32(448.0 * 2.0 ** k))
    for amax in (300.0, 1.0, 7.3e-4, 5.1e6, 447.99):
        amax = np.float32(amax)
        s = np.float32(amax / np.float32(448.0))
        for step in range(-3, 4):
            x = (mids.astype(np.float64) * float(s)).astype(np.float32)
            for _ in range(abs(step)):
                x = np.nextafter(x, np.float32(np.inf if step > 0 else -np.inf), dtype=np.float32)
            x[np.abs(x) > amax] = 0
            row(x, amax)
    x = np.stack(rows)
    rq, rs = oracle.quant_fp8(x, 1, True)
    q, s = _run(lib, x, 1, True, rs.shape)
    assert (s.view(np.uint32) == rs.view(np.uint32)).all()
    assert (q == rq).all(), "codes differ at %s" % (np.argwhere(q != rq)[:5],)
    assert len(np.unique(rq)) > 200                 # the rows do exercise the whole code range
    q128, s128 = _run(lib, x, 128, False, oracle.quant_fp8(x, 128, False)[1].shape)
    rq128, rs128 = oracle.quant_fp8(x, 128, False)
    assert (q128 == rq128).all() and (s128.view(np.uint32) == rs128.view(np.uint32)).all()
    # the same rows through the RMSNorm-fused quantiser (both of its kernels: K = 384 and a long row)
    for reps in (1, 32):
        xx = np.tile(x, (1, reps))
        w = rng.uniform(0.5, 2.0, xx.shape[1]).astype(np.float32)
        rq2, rs2 = oracle.rmsnorm_quant(xx, w, 1e-6)
        q2, s2 = lib.rmsnorm_quantize_activation(torch.from_numpy(xx).cuda(), torch.from_numpy(w).cuda(), 1e-6)
        torch.cuda.synchronize()
        assert (q2.cpu().numpy() == rq2).all() and (s2.cpu().numpy().view(np.uint32) == rs2.view(np.uint32)).all()


def test_non_finite_values_follow_the_reference(lib, oracle):
    """NaN and infinities through every quantiser layout, bit for bit against the oracle's restatement of the reference's
    arithmetic (examples/005.fp8.mm.cu:456, :474-485): a NaN never enters the block maximum and its code is 0x7F
    whatever its sign; an infinity makes the scale infinite, so finite elements become signed zeros and the infinite
    ones inf / inf = NaN -> 0x7F; a block that holds nothing but NaN keeps the maximum's seed (float)INT_MIN."""
    rng = np.random.default_rng(5)
    x = rng.normal(0, 1, (256, 384)).astype(np.float32)
    nan = np.array([0x7FC00000, 0xFFC00000, 0x7F800001, 0xFF800001, 0x7FFFFFFF], np.uint32).view(np.float32)
    x[0, :5] = nan                      # NaNs of both signs, quiet and signalling, among ordinary values
    x[1, 7] = np.inf                    # an infinite maximum
    x[1, 9] = -np.inf
    x[1, 11] = nan[1]
    x[2, 128:256] = nan[0]              # a 1x128 block of nothing but NaN
    x[3, 130] = -np.inf
    x[3, 131] = -3.0
    x[128:256, 256:384] = nan[1]        # a 128x128 block of nothing but NaN
    x[130, 0] = 3e38                    # near the largest finite value: scale stays finite
    x[131, 1] = 1e-45                   # the smallest subnormal beside ordinary values
    for quant_m, transpose in ((1, True), (1, False), (128, False), (128, True)):
        rq, rs = oracle.quant_fp8(x, quant_m, transpose)
        q, s = _run(lib, x, quant_m, transpose, rs.shape)
        bad = np.argwhere(q != rq)
        assert bad.size == 0, "quant_m %d transpose %s: codes differ at %s (got %s, oracle %s)" % (
            quant_m, transpose, bad[:5].tolist(), q[tuple(bad[:5].T)], rq[tuple(bad[:5].T)])
        if quant_m == 128 and transpose:
            assert (s[:, :2].view(np.uint32) == rs[:, :2].view(np.uint32)).all()
        else:
            assert (s.view(np.uint32) == rs.view(np.uint32)).all()
    rq, rs = oracle.quant_fp8(x, 1, True)
    assert rq[0, 0] == 0x7F and rq[0, 1] == 0x7F and rq[1, 7] == 0x7F and rq[1, 9] == 0x7F and rq[1, 0] in (0, 0x80)
    assert rs[1, 2] < 0 and (rq[2, 128:256] == 0x7F).all()
