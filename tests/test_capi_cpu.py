"""The C-ABI library without a GPU: it loads, exports every symbol that include/llmmm.h declares,
and rejects bad arguments before any device work -- with the reference's exception texts
(src/mm/fp16/mm.cu:15-21, examples/005.fp8.mm.cu:2490-2492).  No compute call is made here."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols(headers=("llmmm.h", "llmmm_probe.h")):
    names = set()
    for h in headers:
        text = open(os.path.join(ROOT, "include", h)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names.update(re.findall(r"LLMMM_API\s+[\w\s\*]+?\b(llmmm_\w+)\s*\(", text))
    return sorted(names)


def test_probes_are_declared_apart_from_the_drop_in_surface():
    """The boundary header declares no instrumentation: every llmmm_probe_* lives in llmmm_probe.h, nothing else does."""
    assert not [n for n in _declared_symbols(("llmmm.h",)) if n.startswith("llmmm_probe_")]
    probes = _declared_symbols(("llmmm_probe.h",))
    assert probes and all(n.startswith("llmmm_probe_") for n in probes)


def test_library_exports_every_declared_symbol():
    from llmmm_amd import _lib
    names = _declared_symbols()
    assert len(names) >= 10
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), "libllmmm.so does not export " + n
    assert sorted(_lib.SIGNATURES) == names, "llmmm_amd._lib.SIGNATURES and include/llmmm.h + llmmm_probe.h disagree"


def test_error_strings_are_the_reference_texts():
    from llmmm_amd._lib import lib
    assert lib.llmmm_error_string(1) == b"M or N or K are not aligned."
    assert lib.llmmm_error_string(2) == b"T is not supported."
    assert lib.llmmm_error_string(0) == b"ok"
    assert lib.llmmm_version() >= 100


FAKE = ctypes.c_void_p(0x1000)  # 16-byte aligned, never dereferenced: validation fails first


def test_fp16_validation_without_device():
    from llmmm_amd import _lib
    lib = _lib.lib
    f = lib.llmmm_fp16_gemm
    assert f(0, FAKE, FAKE, FAKE, 100, 256, 256, 0, None) == _lib.ERR_NOT_ALIGNED
    assert f(0, FAKE, FAKE, FAKE, 256, 200, 256, 0, None) == _lib.ERR_NOT_ALIGNED
    assert f(0, FAKE, FAKE, FAKE, 256, 256, 24, 0, None) == _lib.ERR_NOT_ALIGNED
    assert f(7, FAKE, FAKE, FAKE, 256, 256, 256, 0, None) == _lib.ERR_UNSUPPORTED_TYPE
    assert f(0, FAKE, FAKE, FAKE, 256, 256, 256, 5, None) == _lib.ERR_INVALID_ARGUMENT
    assert f(0, None, FAKE, FAKE, 256, 256, 256, 0, None) == _lib.ERR_INVALID_ARGUMENT
    assert f(0, ctypes.c_void_p(0x1004), FAKE, FAKE, 256, 256, 256, 0, None) == _lib.ERR_INVALID_ARGUMENT
    assert f(0, FAKE, FAKE, FAKE, 0, 256, 256, 0, None) == _lib.ERR_INVALID_ARGUMENT
    assert f(0, FAKE, FAKE, FAKE, -256, 256, 256, 0, None) == _lib.ERR_INVALID_ARGUMENT
    cfg = _lib.GemmCfg(_lib.TILE_256x256, 0)
    assert lib.llmmm_fp16_gemm_ex(0, FAKE, FAKE, FAKE, 128, 256, 256, 0, ctypes.byref(cfg), None) == _lib.ERR_NOT_ALIGNED
    cfg = _lib.GemmCfg(99, 0)
    assert lib.llmmm_fp16_gemm_ex(0, FAKE, FAKE, FAKE, 256, 256, 256, 0, ctypes.byref(cfg), None) == _lib.ERR_INVALID_ARGUMENT


def test_fp8_validation_without_device():
    from llmmm_amd import _lib
    lib = _lib.lib
    f = lib.llmmm_fp8_gemm
    args = (FAKE, FAKE, FAKE, FAKE, FAKE, FAKE)
    assert f(2, *args, 128, 100, 256, None, 0, None) == _lib.ERR_NOT_ALIGNED
    assert f(2, *args, 128, 128, 200, None, 0, None) == _lib.ERR_NOT_ALIGNED
    assert f(2, *args, 200, 128, 256, None, 0, None) == _lib.ERR_NOT_ALIGNED  # 128 < M, M % 128 != 0
    assert f(9, *args, 128, 128, 256, None, 0, None) == _lib.ERR_INVALID_ARGUMENT
    assert f(2, FAKE, FAKE, FAKE, FAKE, FAKE, None, 128, 128, 256, None, 0, None) == _lib.ERR_INVALID_ARGUMENT  # Cs missing
    assert f(0, None, FAKE, FAKE, FAKE, FAKE, None, 128, 128, 256, None, 0, None) == _lib.ERR_INVALID_ARGUMENT
    assert f(2, *args, 0, 128, 256, None, 0, None) == _lib.ERR_INVALID_ARGUMENT
    # explicit split-K with a workspace that is too small
    cfg = _lib.GemmCfg(_lib.TILE_SKINNY, 4)
    assert lib.llmmm_fp8_gemm_ex(2, *args, 16, 256, 1024, FAKE, 3 * 16 * 256 * 4, ctypes.byref(cfg), None) == _lib.ERR_WORKSPACE
    assert b"workspace" in lib.llmmm_last_error()
    cfg = _lib.GemmCfg(_lib.TILE_SKINNY, 1)
    assert lib.llmmm_fp8_gemm_ex(2, *args, 256, 256, 1024, None, 0, ctypes.byref(cfg), None) == _lib.ERR_INVALID_ARGUMENT


def test_quant_validation_without_device():
    from llmmm_amd import _lib
    lib = _lib.lib
    assert lib.llmmm_quant_fp8(0, FAKE, FAKE, FAKE, 16, 130, None) == _lib.ERR_NOT_ALIGNED
    assert lib.llmmm_quant_fp8(9, FAKE, FAKE, FAKE, 16, 128, None) == _lib.ERR_INVALID_ARGUMENT
    assert lib.llmmm_quant_fp8(0, None, FAKE, FAKE, 16, 128, None) == _lib.ERR_INVALID_ARGUMENT
    assert lib.llmmm_quant_fp8(0, FAKE, FAKE, FAKE, 0, 128, None) == _lib.ERR_INVALID_ARGUMENT


def test_workspace_sizes_and_config_queries():
    import llmmm_amd
    from llmmm_amd import _lib
    # a shape with a tile per CU never splits and needs no workspace; split configurations need S partial planes
    assert llmmm_amd.workspace_bytes(_lib.OUT_FP8Q, 4096, 4096, 4096) == 0
    for (n, k) in [(6144, 2560), (2560, 4096), (19456, 2560), (2560, 9728)]:
        for m in (1, 16):
            tile, split = llmmm_amd.query_config(_lib.OUT_FP8Q, m, n, k)
            assert tile in (_lib.TILE_SKINNY, _lib.TILE_STRIP) and 1 <= split <= min(32, k // 128)
            if tile == _lib.TILE_SKINNY:
                assert llmmm_amd.workspace_bytes(_lib.OUT_FP8Q, m, n, k) == (0 if split == 1 else split * m * n * 4)
            else:  # column strips need no planes; the query answers for the split-K form a call may fall back to
                assert split == 1 and llmmm_amd.workspace_bytes(_lib.OUT_FP8Q, m, n, k) >= 2 * m * n * 4
        for m in (128, 2048):
            tile, split = llmmm_amd.query_config(_lib.OUT_FP8Q, m, n, k)
            tiles = (_lib.TILE_256x256, _lib.TILE_128x256, _lib.TILE_256x128, _lib.TILE_128x128)
            assert tile in tiles + ((_lib.TILE_SKINNY,) if m == 128 else ())
            if tile in tiles:
                assert 1 <= split <= 8
            assert llmmm_amd.workspace_bytes(_lib.OUT_FP8Q, m, n, k) == (0 if split == 1 else split * m * n * 4)
    assert llmmm_amd.query_config(_lib.OUT_FP8Q, 4096, 4096, 4096) == (_lib.TILE_256x256, 1)
    with pytest.raises(RuntimeError, match="M or N or K are not aligned."):
        llmmm_amd.query_config(_lib.OUT_FP8Q, 200, 4096, 4096)


def test_python_mirror_raises_like_the_reference():
    import torch
    import llmmm_amd
    a = torch.zeros((256, 256), dtype=torch.float32)
    with pytest.raises(RuntimeError, match="T is not supported."):
        llmmm_amd.fp16_mm(a, a, a, 256, 256, 256)
    h = torch.zeros((256, 256), dtype=torch.float16)
    for (m, n, k) in [(128, 256, 256), (256, 128, 256), (256, 256, 8)]:
        with pytest.raises(RuntimeError, match="M or N or K are not aligned."):
            llmmm_amd.fp16_mm(h, h, h, m, n, k)  # the reference's rule: M, N % 256, K % 16
    with pytest.raises(TypeError):
        llmmm_amd.fp16_mm(h, h, h, 256, 256, 256)  # host tensors are not device pointers
    with pytest.raises(ValueError):
        llmmm_amd.fp8_blockwise_symmetric_quantization(a, a, a, 256, 256, 64)  # QUANT_M must be 1 or 128


def test_missing_library_fails_loudly(tmp_path, monkeypatch):
    # the product has no fallback: without libllmmm.so the binding refuses to load
    from llmmm_amd import _lib
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libllmmm.so"))
    with pytest.raises(ImportError, match="no fallback"):
        _lib.load()


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "llmmm_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "import oracle" not in text and "from oracle" not in text and "liboracle" not in text, f


def test_layout_helpers_validation_without_device():
    """Texts of src/base/base.cu:127-129 ("M or N can't be divided 128.") and :265-267 ("K must be ...")."""
    from llmmm_amd import _lib
    lib = _lib.lib
    A, B = ctypes.c_void_p(0x100000), ctypes.c_void_p(0x900000)
    for f in (lib.llmmm_fp8_preshuffle_b, lib.llmmm_fp8_unshuffle_b):
        assert f(A, B, 128, 100, None) == _lib.ERR_NOT_ALIGNED
        assert lib.llmmm_last_error() == b"K must be greater than 0 and divisible by 128."
        assert f(A, B, 24, 128, None) == _lib.ERR_NOT_ALIGNED
        assert f(A, B, 0, 128, None) == _lib.ERR_INVALID_ARGUMENT
        assert f(None, B, 128, 128, None) == _lib.ERR_INVALID_ARGUMENT
        assert f(A, ctypes.c_void_p(0x900004), 128, 128, None) == _lib.ERR_INVALID_ARGUMENT
        assert f(A, A, 128, 128, None) == _lib.ERR_INVALID_ARGUMENT  # in place
        assert f(A, ctypes.c_void_p(0x100000 + 128 * 64), 128, 128, None) == _lib.ERR_INVALID_ARGUMENT  # overlap
    t = lib.llmmm_transpose
    assert t(1, A, B, 128, 100, None) == _lib.ERR_NOT_ALIGNED
    assert lib.llmmm_last_error() == b"M or N can't be divided 128."
    assert t(4, A, B, 200, 128, None) == _lib.ERR_NOT_ALIGNED
    assert t(2, A, B, 128, 128, None) == _lib.ERR_UNSUPPORTED_TYPE
    assert t(4, A, A, 128, 128, None) == _lib.ERR_INVALID_ARGUMENT
    assert t(4, None, B, 128, 128, None) == _lib.ERR_INVALID_ARGUMENT
    # an unknown weight layout is rejected before any launch
    cfg = _lib.GemmCfg(_lib.TILE_AUTO, 0, 7)
    args = (FAKE, FAKE, FAKE, FAKE, FAKE, FAKE)
    assert lib.llmmm_fp8_gemm_ex(2, *args, 128, 128, 256, None, 0, ctypes.byref(cfg), None) == _lib.ERR_INVALID_ARGUMENT
    q = _lib.GemmCfg(5, 5, 5)
    assert lib.llmmm_fp8_gemm_query(2, 128, 128, 256, ctypes.byref(q)) == _lib.OK and q.b_layout == _lib.FP8_B_ROWS


def test_swiglu_validation_without_device():
    from llmmm_amd import _lib
    lib = _lib.lib
    args = (FAKE, FAKE, FAKE, FAKE, FAKE, FAKE)
    f = lib.llmmm_fp8_gemm
    assert f(_lib.OUT_FP8Q_SWIGLU, *args, 256, 384, 256, None, 0, None) == _lib.ERR_NOT_ALIGNED   # N % 256 != 0
    assert f(_lib.OUT_FP8Q_SWIGLU, FAKE, FAKE, FAKE, FAKE, FAKE, None, 256, 512, 256, None, 0, None) == _lib.ERR_INVALID_ARGUMENT  # Cs missing
    assert f(_lib.OUT_FP8Q_SWIGLU, *args, 16, 512, 256, None, 0, None) == _lib.ERR_WORKSPACE       # small M always needs a plane
    assert b"workspace" in lib.llmmm_last_error()
    assert f(4, *args, 256, 512, 256, None, 0, None) == _lib.ERR_INVALID_ARGUMENT
    # the workspace query covers the plane the small-M path needs, and an unsplit tile run needs none
    assert lib.llmmm_fp8_gemm_workspace(_lib.OUT_FP8Q_SWIGLU, 16, 19456, 2560) >= 16 * 19456 * 4
    assert lib.llmmm_fp8_gemm_workspace(_lib.OUT_FP8Q_SWIGLU, 4096, 4096, 4096) == 0
    # an unsplit SwiGLU run is given a 256-column tile
    q = _lib.GemmCfg()
    assert lib.llmmm_fp8_gemm_query(_lib.OUT_FP8Q_SWIGLU, 2048, 2560, 9728, ctypes.byref(q)) == _lib.OK
    assert q.split_k > 1 or q.tile in (_lib.TILE_256x256, _lib.TILE_128x256)
    cfg = _lib.GemmCfg(_lib.TILE_128x128, 1, 0)
    assert lib.llmmm_fp8_gemm_ex(_lib.OUT_FP8Q_SWIGLU, *args, 256, 512, 256, None, 0, ctypes.byref(cfg), None) == _lib.ERR_WORKSPACE
    # decode-sized M on a wide N: a 128-column tile through one fp32 plane, and the workspace query says so
    assert lib.llmmm_fp8_gemm_query(_lib.OUT_FP8Q_SWIGLU, 128, 19456, 2560, ctypes.byref(q)) == _lib.OK
    if q.tile in (_lib.TILE_128x128, _lib.TILE_256x128):
        assert lib.llmmm_fp8_gemm_workspace(_lib.OUT_FP8Q_SWIGLU, 128, 19456, 2560) >= 128 * 19456 * 4


def test_rmsnorm_quant_validation_without_device():
    from llmmm_amd import _lib
    lib = _lib.lib
    f = lib.llmmm_rmsnorm_quant_fp8
    eps = ctypes.c_float(1e-6)
    assert f(_lib.DTYPE_F32, FAKE, FAKE, eps, FAKE, FAKE, 4, 100, None) == _lib.ERR_NOT_ALIGNED
    assert f(7, FAKE, FAKE, eps, FAKE, FAKE, 4, 128, None) == _lib.ERR_UNSUPPORTED_TYPE
    assert f(_lib.DTYPE_BF16, None, FAKE, eps, FAKE, FAKE, 4, 128, None) == _lib.ERR_INVALID_ARGUMENT
    assert f(_lib.DTYPE_BF16, FAKE, FAKE, ctypes.c_float(-1.0), FAKE, FAKE, 4, 128, None) == _lib.ERR_INVALID_ARGUMENT
    assert f(_lib.DTYPE_BF16, FAKE, FAKE, ctypes.c_float(float("nan")), FAKE, FAKE, 4, 128, None) == _lib.ERR_INVALID_ARGUMENT
    assert f(_lib.DTYPE_F16, FAKE, FAKE, eps, FAKE, FAKE, 0, 128, None) == _lib.ERR_INVALID_ARGUMENT
    assert f(_lib.DTYPE_F16, ctypes.c_void_p(0x1008), FAKE, eps, FAKE, FAKE, 4, 128, None) == _lib.ERR_INVALID_ARGUMENT


def test_gemm_add_rmsnorm_quant_validation_without_device():
    from llmmm_amd import _lib
    lib = _lib.lib
    f = lib.llmmm_fp8_gemm_add_rmsnorm_quant
    eps = ctypes.c_float(1e-6)
    M, N, K = 48, 2560, 4096  # (up to 16 rows this shape runs in column strips, which need no workspace)
    plane = M * N * 4

    def call(dtype=_lib.DTYPE_BF16, res=FAKE, n=N, k=K, ws=FAKE, wsz=plane, cfg=None, e=eps, m=M):
        return f(FAKE, FAKE, FAKE, FAKE, dtype, res, FAKE, FAKE, e, FAKE, FAKE, m, n, k, ws, wsz, cfg, None)

    assert call(dtype=9) == _lib.ERR_UNSUPPORTED_TYPE
    assert call(n=2500) == _lib.ERR_NOT_ALIGNED
    assert call(k=100) == _lib.ERR_NOT_ALIGNED
    assert call(res=None) == _lib.ERR_INVALID_ARGUMENT
    assert call(n=10240 + 128) == _lib.ERR_INVALID_ARGUMENT
    assert call(e=ctypes.c_float(-1.0)) == _lib.ERR_INVALID_ARGUMENT
    assert call(ws=None, wsz=0) == _lib.ERR_WORKSPACE
    assert call(wsz=plane - 4) == _lib.ERR_WORKSPACE
    assert call(cfg=ctypes.byref(_lib.GemmCfg(_lib.TILE_SKINNY, 2, 0))) == _lib.ERR_WORKSPACE  # an explicit split never shrinks
    assert call(cfg=ctypes.byref(_lib.GemmCfg(_lib.TILE_64x128, 1, 0)), m=256, wsz=256 * N * 4) == _lib.ERR_INVALID_ARGUMENT
    assert call(cfg=ctypes.byref(_lib.GemmCfg(_lib.TILE_256x256, 1, 0)), m=128, wsz=128 * N * 4) == _lib.ERR_NOT_ALIGNED
    need = lib.llmmm_fp8_gemm_add_rmsnorm_quant_workspace(M, N, K)
    assert need >= plane and need % plane == 0
    assert lib.llmmm_fp8_gemm_add_rmsnorm_quant_workspace(M, 100, K) == 0


def test_qkv_rope_validation_without_device():
    from llmmm_amd import _lib
    lib = _lib.lib
    f = lib.llmmm_fp8_gemm_qkv_rope
    eps = ctypes.c_float(1e-6)
    M, N, K = 16, 6144, 2560
    plane = M * N * 4

    def call(kind=_lib.OUT_BF16, out=FAKE, sc=FAKE, qw=FAKE, kw=FAKE, cos=FAKE, rows=64, pos=FAKE, nq=32, nkv=8, n=N, k=K, ws=FAKE, wsz=plane):
        return f(kind, FAKE, FAKE, FAKE, FAKE, out, sc, qw, kw, eps, cos, FAKE, rows, pos, nq, nkv, M, n, k, ws, wsz, None, None)

    assert call(kind=_lib.OUT_F32) == _lib.ERR_INVALID_ARGUMENT
    assert call(k=100) == _lib.ERR_NOT_ALIGNED
    assert call(nq=31) == _lib.ERR_INVALID_ARGUMENT          # head counts must add up to N / 128
    assert call(out=None) == _lib.ERR_INVALID_ARGUMENT
    assert call(kind=_lib.OUT_FP8Q, sc=None) == _lib.ERR_INVALID_ARGUMENT
    assert call(rows=0) == _lib.ERR_INVALID_ARGUMENT
    assert call(pos=None) == _lib.ERR_INVALID_ARGUMENT
    assert call(pos=ctypes.c_void_p(0x1002)) == _lib.ERR_INVALID_ARGUMENT
    assert call(cos=ctypes.c_void_p(0x1008)) == _lib.ERR_INVALID_ARGUMENT
    assert call(ws=None, wsz=0) == _lib.ERR_WORKSPACE
    assert call(wsz=plane - 4) == _lib.ERR_WORKSPACE
    assert lib.llmmm_fp8_gemm_qkv_rope_workspace(M, N, K) >= plane


def test_a_layout_validation_without_device():
    from llmmm_amd import _lib
    lib = _lib.lib
    M, N, K = 4, 2560, 9728

    def call(cfg, As=None, ws=FAKE, wsz=1 << 30, kind=_lib.OUT_F32, m=M):
        return lib.llmmm_fp8_gemm_ex(kind, FAKE, As, FAKE, FAKE, FAKE, FAKE, m, N, K, ws, wsz, ctypes.byref(cfg), None)

    assert call(_lib.GemmCfg(-1, 0, 0, 7)) == _lib.ERR_INVALID_ARGUMENT                       # unknown A layout
    assert call(_lib.GemmCfg(-1, 0, 0, 0)) == _lib.ERR_INVALID_ARGUMENT                       # quantised A needs its scales
    assert call(_lib.GemmCfg(-1, 0, 0, 1), kind=_lib.OUT_FP8Q_SWIGLU) == _lib.ERR_INVALID_ARGUMENT  # SwiGLU on both sides
    assert call(_lib.GemmCfg(_lib.TILE_SKINNY, 2, 0, 1)) == _lib.ERR_INVALID_ARGUMENT        # 76 slices: split-K >= 3
    assert call(_lib.GemmCfg(_lib.TILE_SKINNY, 0, 0, 1), ws=None, wsz=0) == _lib.ERR_WORKSPACE
    assert call(_lib.GemmCfg(_lib.TILE_SKINNY, 0, 0, 1), m=32, ws=None, wsz=0) == _lib.ERR_WORKSPACE  # M > 4: quantises into the workspace
    assert lib.llmmm_fp8_swiglu_a_workspace(4, N, K) == 0
    assert lib.llmmm_fp8_swiglu_a_workspace(32, N, K) >= 32 * K + (K // 128) * 32 * 4


def test_planes_and_planes_rmsnorm_validation_without_device():
    from llmmm_amd import _lib
    lib = _lib.lib
    M, N, K = 1, 2560, 4096
    splits = ctypes.c_int(0)
    f = lib.llmmm_fp8_gemm_planes
    need = lib.llmmm_fp8_gemm_planes_bytes(M, N, K)
    assert need >= M * N * 4 and need % (M * N * 4) == 0
    assert f(FAKE, FAKE, FAKE, FAKE, M, N, K, None, need, ctypes.byref(splits), None, 0, None, None) == _lib.ERR_INVALID_ARGUMENT
    assert f(FAKE, FAKE, FAKE, FAKE, M, N, K, FAKE, need, None, None, 0, None, None) == _lib.ERR_INVALID_ARGUMENT
    assert f(FAKE, FAKE, FAKE, FAKE, M, 100, K, FAKE, need, ctypes.byref(splits), None, 0, None, None) == _lib.ERR_NOT_ALIGNED
    assert f(FAKE, FAKE, FAKE, FAKE, M, N, K, FAKE, M * N * 4 - 4, ctypes.byref(splits), None, 0, None, None) == _lib.ERR_WORKSPACE
    cfg2 = _lib.GemmCfg(_lib.TILE_SKINNY, 2, 0, 0)
    assert f(FAKE, FAKE, FAKE, FAKE, M, N, K, FAKE, M * N * 4, ctypes.byref(splits), None, 0, ctypes.byref(cfg2), None) == _lib.ERR_WORKSPACE
    # the descriptor of a_layout = PLANES_RMSNORM is validated on the host
    K2, N2 = 2560, 6144
    cfg = _lib.GemmCfg(_lib.TILE_SKINNY, 0, 0, _lib.FP8_A_PLANES_RMSNORM)

    def call(d):
        return lib.llmmm_fp8_gemm_ex(_lib.OUT_F32, ctypes.byref(d), None, FAKE, FAKE, FAKE, None, M, N2, K2, FAKE, 1 << 30, ctypes.byref(cfg), None)

    good = dict(planes=0x1000, splits=8, hidden_dtype=_lib.DTYPE_BF16, residual=0x2000, hidden_out=0x3000, norm_weight=0x4000, eps=1e-6)
    assert call(_lib.APlanesRmsnorm(**dict(good, planes=None))) == _lib.ERR_INVALID_ARGUMENT
    assert call(_lib.APlanesRmsnorm(**dict(good, splits=0))) == _lib.ERR_INVALID_ARGUMENT
    assert call(_lib.APlanesRmsnorm(**dict(good, hidden_dtype=9))) == _lib.ERR_UNSUPPORTED_TYPE
    assert call(_lib.APlanesRmsnorm(**dict(good, eps=-1.0))) == _lib.ERR_INVALID_ARGUMENT
    assert call(_lib.APlanesRmsnorm(**dict(good, residual=0x2004))) == _lib.ERR_INVALID_ARGUMENT
    assert lib.llmmm_fp8_planes_rmsnorm_a_workspace(2, N2, K2) == 2 * N2 * 4  # the kernel generates: one fp32 plane for outputs other than fp32
    assert lib.llmmm_fp8_planes_rmsnorm_a_workspace(16, N2, K2) > 0


def test_the_64x128_tile_is_fp16_only():
    from llmmm_amd import _lib
    lib = _lib.lib
    args = (FAKE, FAKE, FAKE, FAKE, FAKE, FAKE)
    cfg = _lib.GemmCfg(_lib.TILE_64x128, 1, 0)
    assert lib.llmmm_fp8_gemm_ex(2, *args, 256, 256, 256, None, 0, ctypes.byref(cfg), None) == _lib.ERR_INVALID_ARGUMENT


def test_probe_validation_without_device():
    from llmmm_amd import _lib
    lib = _lib.lib
    a32 = ctypes.c_void_p(0x2000)
    assert lib.llmmm_probe_mfma(5, a32, FAKE, 256, 10, None) == _lib.ERR_UNSUPPORTED_TYPE
    assert lib.llmmm_probe_mfma(0, None, FAKE, 256, 10, None) == _lib.ERR_INVALID_ARGUMENT
    assert lib.llmmm_probe_mfma(0, ctypes.c_void_p(0x2010), FAKE, 256, 10, None) == _lib.ERR_INVALID_ARGUMENT
    assert lib.llmmm_probe_mfma(0, a32, FAKE, 0, 10, None) == _lib.ERR_INVALID_ARGUMENT
    assert lib.llmmm_probe_mfma(0, a32, FAKE, 256, 0, None) == _lib.ERR_INVALID_ARGUMENT
    assert lib.llmmm_probe_hbm_read(a32, 100, FAKE, 256, None) == _lib.ERR_INVALID_ARGUMENT
    assert lib.llmmm_probe_hbm_read(None, 1024, FAKE, 256, None) == _lib.ERR_INVALID_ARGUMENT
    # FLOP of a launch: workgroups x 8 waves x iters x (16 MFMAs x 16384 | 8 MFMAs x 65536)
    assert lib.llmmm_probe_mfma_flops(0, 256, 10) == 256 * 8 * 10 * 16 * 16384.0
    assert lib.llmmm_probe_mfma_flops(_lib.PROBE_FP8, 256, 10) == 256 * 8 * 10 * 8 * 65536.0
    assert lib.llmmm_probe_mfma_flops(9, 256, 10) == 0.0


def _no_gpu_here():
    import torch
    return not torch.cuda.is_available()


@pytest.mark.skipif(not _no_gpu_here(), reason="passes validation with made-up pointers: only where no device can be reached")
@pytest.mark.parametrize("N,K", [(2560, 4096), (19456, 2560), (10240, 2048), (6144, 2560), (4096, 14336)])
@pytest.mark.parametrize("M", [1, 16, 65, 96, 127, 128, 256, 2048])
def test_queried_workspace_is_accepted_by_the_fused_entry_points(M, N, K):
    """The size a *_workspace query returns must pass the workspace checks of its call, row tails included (64 < M < 128
    routed to an unsplit 128 x 128 tile has no epilogue of its own and needs one fp32 plane).  Without a device the call
    gets as far as the launch (LLMMM_ERR_RUNTIME); a workspace complaint would come before that."""
    from llmmm_amd import _lib
    lib = _lib.lib
    eps = ctypes.c_float(1e-6)
    if N <= 10240:
        need = lib.llmmm_fp8_gemm_add_rmsnorm_quant_workspace(M, N, K)
        ws = FAKE if need else None
        rc = lib.llmmm_fp8_gemm_add_rmsnorm_quant(FAKE, FAKE, FAKE, FAKE, _lib.DTYPE_BF16, FAKE, FAKE, FAKE, eps, FAKE, FAKE, M, N, K, ws, need, None, None)
        assert rc == _lib.ERR_RUNTIME, lib.llmmm_last_error()
    heads = N // 128
    if heads >= 3 and (heads - 2) % 1 == 0:
        nkv = 1 if heads < 12 else 8
        nq = heads - 2 * nkv
        need = lib.llmmm_fp8_gemm_qkv_rope_workspace(M, N, K)
        ws = FAKE if need else None
        rc = lib.llmmm_fp8_gemm_qkv_rope(_lib.OUT_BF16, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, eps, FAKE, FAKE, 64, FAKE, nq, nkv, M, N, K,
                                         ws, need, None, None)
        assert rc == _lib.ERR_RUNTIME, lib.llmmm_last_error()


def test_planes_rmsnorm_descriptor_needs_no_16_byte_alignment():
    """The A argument of cfg.a_layout = PLANES_RMSNORM is a host structure of pointer alignment (8): one at an address
    that is 8 modulo 16 is as good as any.  The device pointers inside it are still checked."""
    from llmmm_amd import _lib
    lib = _lib.lib
    buf = (ctypes.c_char * (ctypes.sizeof(_lib.APlanesRmsnorm) + 32))()
    base = ctypes.addressof(buf)
    addr = base + ((8 - base) % 16)
    assert addr % 16 == 8
    d = _lib.APlanesRmsnorm.from_address(addr)
    d.planes, d.splits, d.hidden_dtype, d.residual, d.hidden_out, d.norm_weight, d.eps = 0x1000, 8, _lib.DTYPE_BF16, 0x2000, 0x3000, 0x4000, 1e-6
    cfg = _lib.GemmCfg(_lib.TILE_SKINNY, 0, 0, _lib.FP8_A_PLANES_RMSNORM)
    M, N, K = 1, 6144, 2560

    def call():
        return lib.llmmm_fp8_gemm_ex(_lib.OUT_F32, ctypes.c_void_p(addr), None, FAKE, FAKE, FAKE, None, M, N, K, None, 0, ctypes.byref(cfg), None)

    d.residual = 0x2004  # a misaligned device pointer inside the descriptor is still refused ...
    assert call() == _lib.ERR_INVALID_ARGUMENT and b"16-byte aligned" in lib.llmmm_last_error()
    d.residual = 0x2000
    d.splits = 0         # ... and so is a bad field, which shows that validation went past the alignment of A itself
    assert call() == _lib.ERR_INVALID_ARGUMENT and b"splits" in lib.llmmm_last_error()
    # the fused entry points take the same route
    d.splits = 99
    rc = lib.llmmm_fp8_gemm_qkv_rope(_lib.OUT_BF16, ctypes.c_void_p(addr), None, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, ctypes.c_float(1e-6), FAKE, FAKE, 64, FAKE,
                                     32, 8, M, N, K, FAKE, 1 << 20, ctypes.byref(cfg), None)
    assert rc == _lib.ERR_INVALID_ARGUMENT and b"splits" in lib.llmmm_last_error()


@pytest.mark.skipif(not _no_gpu_here(), reason="passes validation with made-up pointers: only where no device can be reached")
@pytest.mark.parametrize("N,K", [(2560, 9728), (2560, 4096), (6144, 2560), (19456, 2560), (4096, 14336)])
@pytest.mark.parametrize("M", [1, 2, 4, 8, 16, 32, 128])
@pytest.mark.parametrize("a_layout", [1, 2])
def test_queried_sizes_hold_for_generated_activations(M, N, K, a_layout):
    """A call whose activations the library makes itself (cfg.a_layout = SWIGLU_F32 or PLANES_RMSNORM) never runs in
    column strips, so the size queries -- which cannot see cfg -- must cover the split-K form of a strip-capable shape
    (2560 x 9728 at M <= 4 needs three planes for generated activations).  Each entry point gets exactly the queried
    sizes and must get as far as the launch (LLMMM_ERR_RUNTIME without a device)."""
    from llmmm_amd import _lib
    lib = _lib.lib
    eps = ctypes.c_float(1e-6)
    if a_layout == _lib.FP8_A_PLANES_RMSNORM and K > 10240:
        pytest.skip("the fused norm handles rows of at most 10240 columns")
    a_ws = (lib.llmmm_fp8_swiglu_a_workspace if a_layout == _lib.FP8_A_SWIGLU_F32 else lib.llmmm_fp8_planes_rmsnorm_a_workspace)(M, N, K)
    cfg = _lib.GemmCfg(_lib.TILE_AUTO, 0, 0, a_layout)
    if a_layout == _lib.FP8_A_PLANES_RMSNORM:
        d = _lib.APlanesRmsnorm()
        d.planes, d.splits, d.hidden_dtype, d.residual, d.hidden_out, d.norm_weight, d.eps = 0x1000, 4, _lib.DTYPE_BF16, 0x2000, 0x3000, 0x4000, 1e-6
        A = ctypes.cast(ctypes.pointer(d), ctypes.c_void_p)
    else:
        A = FAKE

    def ws(n):
        return (FAKE if n else None), n

    # the plain GEMM, every output kind
    for out in (_lib.OUT_F32, _lib.OUT_BF16, _lib.OUT_FP8Q):
        need = lib.llmmm_fp8_gemm_workspace(out, M, N, K) + a_ws
        rc = lib.llmmm_fp8_gemm_ex(out, A, None, FAKE, FAKE, FAKE, FAKE, M, N, K, *ws(need), ctypes.byref(cfg), None)
        assert rc == _lib.ERR_RUNTIME, (out, lib.llmmm_last_error())
    # planes only
    pb = lib.llmmm_fp8_gemm_planes_bytes(M, N, K)
    splits = ctypes.c_int(0)
    rc = lib.llmmm_fp8_gemm_planes(A, None, FAKE, FAKE, M, N, K, FAKE, pb, ctypes.byref(splits), *ws(a_ws), ctypes.byref(cfg), None)
    assert rc == _lib.ERR_RUNTIME, lib.llmmm_last_error()
    # projection + residual add + RMSNorm + quantiser
    if N <= 10240:
        need = lib.llmmm_fp8_gemm_add_rmsnorm_quant_workspace(M, N, K) + a_ws
        rc = lib.llmmm_fp8_gemm_add_rmsnorm_quant(A, None, FAKE, FAKE, _lib.DTYPE_BF16, FAKE, FAKE, FAKE, eps, FAKE, FAKE, M, N, K, *ws(need),
                                                  ctypes.byref(cfg), None)
        assert rc == _lib.ERR_RUNTIME, lib.llmmm_last_error()
    # QKV + per-head norm + rope
    heads = N // 128
    nkv = 1 if heads < 12 else 8
    need = lib.llmmm_fp8_gemm_qkv_rope_workspace(M, N, K) + a_ws
    rc = lib.llmmm_fp8_gemm_qkv_rope(_lib.OUT_BF16, A, None, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, eps, FAKE, FAKE, 64, FAKE, heads - 2 * nkv, nkv, M, N, K,
                                     *ws(need), ctypes.byref(cfg), None)
    assert rc == _lib.ERR_RUNTIME, lib.llmmm_last_error()
