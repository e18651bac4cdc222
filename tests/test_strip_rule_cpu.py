"""Where the library runs a decode-sized FP8 GEMM in column strips (one launch) instead of split-K + reduce: the rule of
`strips_pay` in csrc/capi.cpp restated from the measurements it encodes, against `llmmm_fp8_gemm_query` -- no GPU needed
(the library assumes the 256 CUs of an MI355X when it finds no device)."""
import pytest

STRIP, SKINNY = 9, 8


def strips_pay(m, n, k, fused):
    plain = m <= 8 or (m <= 16 and k <= 4096)
    if n // 16 <= 256:                                          # at most one 16-column strip per CU
        return m * k <= 65536 and m <= 16 if fused else plain
    if n % 32 == 0 and n // 32 <= 256 and n * k <= 32 << 20:    # 32-column strips
        return m <= 4 if fused else plain
    if 448 <= n // 16 <= 512:                                   # two 16-column strips on (nearly) every CU
        return m * k <= (65536 if fused else 131072)
    return False


# the Qwen3-4B projections that split K, and shapes of other families on both sides of every branch of the rule
@pytest.mark.parametrize("n,k", [(2560, 4096), (2560, 9728), (6144, 2560), (6144, 4096), (5120, 5120), (8192, 8192), (5120, 13824),
                                 (7168, 5120), (8192, 28672), (4096, 14336), (3584, 18944), (4608, 3584)])
def test_strips_where_measured_faster(n, k):
    import llmmm_amd
    from llmmm_amd import _lib
    for m in (1, 2, 4, 6, 8, 16):
        for kind, fused in ((_lib.OUT_BF16, False), (_lib.OUT_F32, False), (_lib.OUT_FP8Q, True)):
            got = llmmm_amd.query_config(kind, m, n, k)
            if strips_pay(m, n, k, fused):
                assert got == (STRIP, 1), (m, n, k, fused, got)
            else:
                assert got[0] == SKINNY and got[1] > 1, (m, n, k, fused, got)


def test_no_strips_where_nothing_is_split():
    import llmmm_amd
    from llmmm_amd import _lib
    assert llmmm_amd.query_config(_lib.OUT_FP8Q, 1, 19456, 2560) == (SKINNY, 1)  # 152 column groups fill the chip unsplit
    assert llmmm_amd.query_config(_lib.OUT_FP8Q, 17, 2560, 4096)[0] == SKINNY    # the exchange handles one 16-row block
    assert llmmm_amd.query_config(_lib.OUT_FP8Q_SWIGLU, 1, 19456, 2560)[0] == SKINNY
