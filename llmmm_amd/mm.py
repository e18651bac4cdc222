"""Host entry points of the matrix-multiplication path, mirroring the reference's launchers.

Same names, argument order and error behaviour as the reference's C++ functions
(``LLMMM::fp16_mm`` src/mm/fp16/mm.h:9-10; the FP8 launchers examples/005.fp8.mm.cu:217-225,
:547-549, :2467-2476), taking torch CUDA tensors where the reference takes raw device pointers.
Everything goes through the C ABI of ``libllmmm.so``; torch only owns the memory and the stream.
"""
import ctypes

import torch

from . import _lib
from ._lib import GemmCfg, check, lib

_FP8_DTYPES = (torch.uint8, torch.float8_e4m3fn)


def _stream(stream):
    if stream is None:
        return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    if isinstance(stream, torch.cuda.Stream):
        return ctypes.c_void_p(stream.cuda_stream)
    return ctypes.c_void_p(int(stream))


def _ptr(t, what, dtypes=None, numel=None):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise TypeError("%s must be a CUDA tensor" % what)
    if not t.is_contiguous():
        raise ValueError("%s must be contiguous" % what)
    if dtypes is not None and t.dtype not in dtypes:
        raise RuntimeError("T is not supported.")
    if numel is not None and t.numel() < numel:
        raise ValueError("%s holds %d elements, %d needed" % (what, t.numel(), numel))
    return ctypes.c_void_p(t.data_ptr())


def _dtype_code(t):
    if t.dtype == torch.float16:
        return _lib.DTYPE_F16
    if t.dtype == torch.bfloat16:
        return _lib.DTYPE_BF16
    raise RuntimeError("T is not supported.")  # src/mm/fp16/mm.cu:15-17


# ------------------------------------------------------------------------------------- FP16 / BF16
def fp16_mm(A, B, C, M, N, K, stream=None):
    """``LLMMM::fp16_mm<T>(A, B, C, M, N, K, stream)`` (src/mm/fp16/mm.cu:6-42).

    A [M,K], B [K,N], C [M,N] row-major, T = float16 or bfloat16, fp32 accumulation.
    Raises RuntimeError("M or N or K are not aligned.") unless M % 256 == 0, N % 256 == 0 and
    K % 16 == 0 (the reference's rule, mm.cu:19-21) and RuntimeError("T is not supported.")
    for other element types.  Asynchronous on ``stream`` (default: torch's current stream)."""
    code = _dtype_code(A)
    if B.dtype != A.dtype or C.dtype != A.dtype:
        raise RuntimeError("T is not supported.")
    if not (M % 256 == 0 and N % 256 == 0 and K % 16 == 0):
        raise RuntimeError("M or N or K are not aligned.")
    check(lib.llmmm_fp16_gemm(code, _ptr(A, "A", numel=M * K), _ptr(B, "B", numel=K * N), _ptr(C, "C", numel=M * N), M, N, K,
                              _lib.B_ROW_MAJOR, _stream(stream)))


def fp16_gemm(A, B, C=None, b_transposed=False, tile=_lib.TILE_AUTO, stream=None):
    """C = A @ B (or A @ Bt.T when ``b_transposed``) through ``llmmm_fp16_gemm_ex``.

    The library's own (wider) shape rule applies: M, N multiples of 128, K of 16."""
    code = _dtype_code(A)
    M, K = A.shape
    N = B.shape[0] if b_transposed else B.shape[1]
    if (B.shape[1] if b_transposed else B.shape[0]) != K or B.dtype != A.dtype:
        raise ValueError("shape or dtype mismatch between A and B")
    if C is None:
        C = torch.empty((M, N), dtype=A.dtype, device=A.device)
    cfg = GemmCfg(tile, 0)
    check(lib.llmmm_fp16_gemm_ex(code, _ptr(A, "A"), _ptr(B, "B"), _ptr(C, "C", (A.dtype,), M * N), M, N, K,
                                 _lib.B_TRANSPOSED if b_transposed else _lib.B_ROW_MAJOR, ctypes.byref(cfg), _stream(stream)))
    return C


# ------------------------------------------------------------------------------------- FP8 quantiser
def fp8_blockwise_symmetric_quantization(x, q, scale, M, N, quant_m, quant_n=128, scale_transpose=False, stream=None):
    """``fp8_blockwise_symmetric_quantization<QUANT_M, QUANT_N, SCALE_TRANSPOSE>(x, q, scale, M, N, stream)``
    (examples/005.fp8.mm.cu:547-563).  quant_m in {1, 128}, quant_n == 128 (its static_asserts)."""
    if quant_m not in (1, 128) or quant_n != 128:
        raise ValueError("QUANT_M must be 1 or 128 and QUANT_N 128")
    kind = {(1, True): _lib.QUANT_1x128_T, (128, False): _lib.QUANT_128x128, (1, False): _lib.QUANT_1x128,
            (128, True): _lib.QUANT_128x128_T}[(quant_m, bool(scale_transpose))]
    nb = (N + 127) // 128
    n_scale = nb * M if scale_transpose else ((M + quant_m - 1) // quant_m) * nb
    check(lib.llmmm_quant_fp8(kind, _ptr(x, "x", (torch.float32,), M * N), _ptr(q, "q", _FP8_DTYPES, M * N),
                              _ptr(scale, "scale", (torch.float32,), n_scale), M, N, _stream(stream)))


def quantize_activation(x, stream=None):
    """1x128 quantisation with transposed scales: returns (codes uint8 [M,K], scales [K/128... ceil, M])."""
    M, K = x.shape
    q = torch.empty((M, K), dtype=torch.uint8, device=x.device)
    s = torch.empty(((K + 127) // 128, M), dtype=torch.float32, device=x.device)
    fp8_blockwise_symmetric_quantization(x, q, s, M, K, 1, 128, True, stream)
    return q, s


def quantize_weight(wt, stream=None):
    """128x128 quantisation of a transposed weight Wt [N,K]: (codes [N,K], scales [ceil(N/128), ceil(K/128)])."""
    N, K = wt.shape
    q = torch.empty((N, K), dtype=torch.uint8, device=wt.device)
    s = torch.empty(((N + 127) // 128, (K + 127) // 128), dtype=torch.float32, device=wt.device)
    fp8_blockwise_symmetric_quantization(wt, q, s, N, K, 128, 128, False, stream)
    return q, s


def rmsnorm_quantize_activation(x, weight, eps, stream=None):
    """RMSNorm fused in front of the activation quantiser (the fusion the reference plans, README.md:16):
    x [M,K] float32 / bfloat16 / float16, weight [K] float32 -> (codes uint8 [M,K], scales float32 [K/128, M]) of
    ``x / sqrt(mean(x^2) + eps) * weight``, ready to be the A operand of the FP8 GEMM."""
    M, K = x.shape
    code = {torch.float32: _lib.DTYPE_F32, torch.bfloat16: _lib.DTYPE_BF16, torch.float16: _lib.DTYPE_F16}.get(x.dtype)
    if code is None:
        raise RuntimeError("T is not supported.")
    q = torch.empty((M, K), dtype=torch.uint8, device=x.device)
    s = torch.empty(((K + 127) // 128, M), dtype=torch.float32, device=x.device)
    check(lib.llmmm_rmsnorm_quant_fp8(code, _ptr(x, "x"), _ptr(weight, "weight", (torch.float32,), K), ctypes.c_float(eps), _ptr(q, "q"),
                                      _ptr(s, "scale"), M, K, _stream(stream)))
    return q, s


# ------------------------------------------------------------------------------------- FP8 GEMM
def workspace_bytes(out_kind, M, N, K):
    return int(lib.llmmm_fp8_gemm_workspace(out_kind, M, N, K))


def make_workspace(out_kind, M, N, K, device="cuda", stream=None):
    """Allocate a split-K workspace for this shape (None when none is needed); plain scratch, no initialisation."""
    n = workspace_bytes(out_kind, M, N, K)
    if n == 0:
        return None
    return torch.empty(n, dtype=torch.uint8, device=device)


def query_config(out_kind, M, N, K):
    cfg = GemmCfg()
    check(lib.llmmm_fp8_gemm_query(out_kind, M, N, K, ctypes.byref(cfg)))
    return cfg.tile, cfg.split_k


class PlanesRmsnorm:
    """The A operand of a projection whose input is the RMSNorm of a hidden state still in pieces (llmmm_a_planes_rmsnorm):
    ``planes`` [splits, M, K] float32 from :func:`fp8_gemm_planes`, ``residual`` / ``hidden_out`` [M, K] (float32, bfloat16 or
    float16; different tensors for M <= 4), ``norm_weight`` [K] float32."""

    def __init__(self, planes, splits, residual, hidden_out, norm_weight, eps):
        self.planes, self.splits, self.residual, self.hidden_out, self.norm_weight, self.eps = planes, splits, residual, hidden_out, norm_weight, eps

    def c_struct(self, M, K):
        code = {torch.float32: _lib.DTYPE_F32, torch.bfloat16: _lib.DTYPE_BF16, torch.float16: _lib.DTYPE_F16}.get(self.residual.dtype)
        if code is None or self.hidden_out.dtype != self.residual.dtype:
            raise RuntimeError("T is not supported.")
        return _lib.APlanesRmsnorm(_ptr(self.planes, "planes", (torch.float32,), self.splits * M * K).value, self.splits, code,
                                   _ptr(self.residual, "residual", numel=M * K).value, _ptr(self.hidden_out, "hidden_out", numel=M * K).value,
                                   _ptr(self.norm_weight, "norm_weight", (torch.float32,), K).value, self.eps)


def _a_operand(A, As, M, K, a_swiglu):
    """(A pointer, As pointer, a_layout, keep-alive) of the A operand: quantised codes + transposed scales, the fp32 gate_up result
    [M, 2K] (a_swiglu), or a :class:`PlanesRmsnorm`."""
    kb = K // 128 if K % 128 == 0 else 0
    if isinstance(A, PlanesRmsnorm):
        st = A.c_struct(M, K)
        return ctypes.cast(ctypes.pointer(st), ctypes.c_void_p), None, _lib.FP8_A_PLANES_RMSNORM, st
    if a_swiglu:
        return _ptr(A, "A (fp32 gate_up result)", (torch.float32,), M * 2 * K), None, _lib.FP8_A_SWIGLU_F32, None
    return _ptr(A, "A", _FP8_DTYPES, M * K), _ptr(As, "A_scale_transposed", (torch.float32,), kb * M), _lib.FP8_A_QUANTISED, None


def _a_workspace_bytes(A, M, N, K, a_swiglu):
    """Workspace bytes the A operand adds to a call's own: 0 for quantised codes, the library's answer for an operand it makes."""
    if isinstance(A, PlanesRmsnorm):
        return int(lib.llmmm_fp8_planes_rmsnorm_a_workspace(M, N, K))
    return int(lib.llmmm_fp8_swiglu_a_workspace(M, N, K)) if a_swiglu else 0


def _fp8_gemm(out_kind, A, As, Bt, Bs, C, Cs, M, N, K, workspace, tile, split_k, stream, b_preshuffled=False, a_swiglu=False):
    kb = K // 128 if K % 128 == 0 else 0
    c_dtypes = {_lib.OUT_F32: (torch.float32,), _lib.OUT_BF16: (torch.bfloat16,), _lib.OUT_FP8Q: _FP8_DTYPES, _lib.OUT_FP8Q_SWIGLU: _FP8_DTYPES}[out_kind]
    n_out = N // 2 if out_kind == _lib.OUT_FP8Q_SWIGLU else N  # SwiGLU halves the width
    a_p, as_p, a_layout, _keep = _a_operand(A, As, M, K, a_swiglu)
    b_p = _ptr(Bt, "B_transposed", _FP8_DTYPES, N * K)
    bs_p = _ptr(Bs, "B_scale_transposed", (torch.float32,), ((N + 127) // 128) * kb)
    c_p = _ptr(C, "C", c_dtypes, M * n_out)
    cs_p = _ptr(Cs, "C_scale_transposed", (torch.float32,), ((n_out + 127) // 128) * M) if out_kind in (_lib.OUT_FP8Q, _lib.OUT_FP8Q_SWIGLU) else None
    ws_p, ws_n = (ctypes.c_void_p(workspace.data_ptr()), workspace.numel() * workspace.element_size()) if workspace is not None else (None, 0)
    cfg = GemmCfg(tile, split_k, _lib.FP8_B_PRESHUFFLED if b_preshuffled else _lib.FP8_B_ROWS, a_layout)
    check(lib.llmmm_fp8_gemm_ex(out_kind, a_p, as_p, b_p, bs_p, c_p, cs_p, M, N, K, ws_p, ws_n, ctypes.byref(cfg), _stream(stream)))


def fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(A, A_scale_transposed, B_transposed, B_scale_transposed, C, M, N, K,
                                                             stream=None, workspace=None, tile=_lib.TILE_AUTO, split_k=0,
                                                             b_preshuffled=False, a_swiglu=False):
    """examples/005.fp8.mm.cu:217-246.  C [M,N] float32.  ``b_preshuffled``: B_transposed is the image written by
    :func:`construct_mfma_B_layout` instead of row-major [N,K] (same results, bit for bit).  ``a_swiglu``: A is the fp32
    result [M, 2K] of a gate_up projection and the GEMM runs on quantise(silu(gate) * up) (A_scale_transposed: None)."""
    _fp8_gemm(_lib.OUT_F32, A, A_scale_transposed, B_transposed, B_scale_transposed, C, None, M, N, K, workspace, tile, split_k, stream,
              b_preshuffled, a_swiglu)


def fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_bf16(A, A_scale_transposed, B_transposed, B_scale_transposed, C, M, N, K,
                                                             stream=None, workspace=None, tile=_lib.TILE_AUTO, split_k=0,
                                                             b_preshuffled=False, a_swiglu=False):
    """The fp32 variant's result rounded to bfloat16 (no reference kernel; same signature)."""
    _fp8_gemm(_lib.OUT_BF16, A, A_scale_transposed, B_transposed, B_scale_transposed, C, None, M, N, K, workspace, tile, split_k, stream,
              b_preshuffled, a_swiglu)


def fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(A, A_scale_transposed, B_transposed, B_scale_transposed, C,
                                                                     C_scale_transposed, M, N, K, stream=None, workspace=None,
                                                                     tile=_lib.TILE_AUTO, split_k=0, b_preshuffled=False, a_swiglu=False):
    """examples/005.fp8.mm.cu:2467-2500 / examples/005.fp8.mm.opt.cu:468-508.  C e4m3 codes [M,N],
    C_scale_transposed float32 [N/128, M]."""
    _fp8_gemm(_lib.OUT_FP8Q, A, A_scale_transposed, B_transposed, B_scale_transposed, C, C_scale_transposed, M, N, K, workspace, tile,
              split_k, stream, b_preshuffled, a_swiglu)


def fp8_gemm_blockwise_quant_A_1x128__B_128x128__swiglu__C_1x128__output_fp8(A, A_scale_transposed, B_transposed, B_scale_transposed, C,
                                                                             C_scale_transposed, M, N, K, stream=None, workspace=None,
                                                                             tile=_lib.TILE_AUTO, split_k=0, b_preshuffled=False):
    """The gate_up projection of a gated MLP with the activation fused in front of the C quantisation (the fusion
    the reference plans, README.md:16; no reference kernel).  B_transposed [N,K] holds the gate rows in [0, N/2) and
    the up rows in [N/2, N); C = e4m3 codes of silu(gate) * up [M, N/2], C_scale_transposed float32 [N/256, M].
    M <= 128 needs a workspace (``make_workspace(OUT_FP8Q_SWIGLU, ...)``).  (The other way to fuse the activation is on the
    consumer's side: run gate_up with fp32 output and pass it to the down projection with ``a_swiglu=True``.)"""
    _fp8_gemm(_lib.OUT_FP8Q_SWIGLU, A, A_scale_transposed, B_transposed, B_scale_transposed, C, C_scale_transposed, M, N, K, workspace,
              tile, split_k, stream, b_preshuffled)


def fp8_gemm_add_rmsnorm_quant(A, A_scale_transposed, B_transposed, B_scale_transposed, residual, hidden_out, norm_weight, eps, M, N, K,
                               stream=None, workspace=None, tile=_lib.TILE_AUTO, split_k=0, b_preshuffled=False, a_swiglu=False):
    """A projection back to the hidden size (O, down) with the decoder block's epilogue behind it (the fusion the reference
    plans, README.md:16): ``hidden_out = residual + A @ B`` (stored in the residual's dtype; may be the same tensor), then
    RMSNorm(hidden_out) * norm_weight quantised 1x128 with transposed scales.  Returns (codes uint8 [M,N], scales float32
    [N/128, M]): the A operand of the next projection, bit-identical to ``rmsnorm_quantize_activation(hidden_out, ...)``."""
    code = {torch.float32: _lib.DTYPE_F32, torch.bfloat16: _lib.DTYPE_BF16, torch.float16: _lib.DTYPE_F16}.get(residual.dtype)
    if code is None or hidden_out.dtype != residual.dtype:
        raise RuntimeError("T is not supported.")
    kb = K // 128 if K % 128 == 0 else 0
    if workspace is None:
        n = int(lib.llmmm_fp8_gemm_add_rmsnorm_quant_workspace(M, N, K)) + _a_workspace_bytes(A, M, N, K, a_swiglu)
        workspace = torch.empty(max(n, 16), dtype=torch.uint8, device=residual.device)
    q = torch.empty((M, N), dtype=torch.uint8, device=residual.device)
    s = torch.empty(((N + 127) // 128, M), dtype=torch.float32, device=residual.device)
    a_p, as_p, a_layout, _keep = _a_operand(A, A_scale_transposed, M, K, a_swiglu)
    cfg = GemmCfg(tile, split_k, _lib.FP8_B_PRESHUFFLED if b_preshuffled else _lib.FP8_B_ROWS, a_layout)
    check(lib.llmmm_fp8_gemm_add_rmsnorm_quant(
        a_p, as_p,
        _ptr(B_transposed, "B_transposed", _FP8_DTYPES, N * K), _ptr(B_scale_transposed, "B_scale_transposed", (torch.float32,), ((N + 127) // 128) * kb),
        code, _ptr(residual, "residual", numel=M * N), _ptr(hidden_out, "hidden_out", numel=M * N), _ptr(norm_weight, "norm_weight", (torch.float32,), N),
        ctypes.c_float(eps), _ptr(q, "q"), _ptr(s, "q_scale"), M, N, K, ctypes.c_void_p(workspace.data_ptr()),
        workspace.numel() * workspace.element_size(), ctypes.byref(cfg), _stream(stream)))
    return q, s


def fp8_gemm_planes(A, A_scale_transposed, B_transposed, B_scale_transposed, M, N, K, planes=None, stream=None, workspace=None, tile=_lib.TILE_AUTO,
                    split_k=0, b_preshuffled=False, a_swiglu=False):
    """A projection that stops at its fp32 partial sums: returns (planes float32 [>= splits, M, N], splits).  Feed them to the next
    projection as a :class:`PlanesRmsnorm` (residual add, RMSNorm and quantisation then happen in that projection's kernel)."""
    if planes is None:
        planes = torch.empty(max(int(lib.llmmm_fp8_gemm_planes_bytes(M, N, K)) // 4, max(split_k, 1) * M * N), dtype=torch.float32,
                             device=B_transposed.device)
    kb = K // 128 if K % 128 == 0 else 0
    if workspace is None and _a_workspace_bytes(A, M, N, K, a_swiglu):
        workspace = torch.empty(_a_workspace_bytes(A, M, N, K, a_swiglu), dtype=torch.uint8, device=B_transposed.device)
    a_p, as_p, a_layout, _keep = _a_operand(A, A_scale_transposed, M, K, a_swiglu)
    cfg = GemmCfg(tile, split_k, _lib.FP8_B_PRESHUFFLED if b_preshuffled else _lib.FP8_B_ROWS, a_layout)
    splits = ctypes.c_int(0)
    ws_p, ws_n = (ctypes.c_void_p(workspace.data_ptr()), workspace.numel() * workspace.element_size()) if workspace is not None else (None, 0)
    check(lib.llmmm_fp8_gemm_planes(a_p, as_p, _ptr(B_transposed, "B_transposed", _FP8_DTYPES, N * K),
                                    _ptr(B_scale_transposed, "B_scale_transposed", (torch.float32,), ((N + 127) // 128) * kb), M, N, K,
                                    _ptr(planes, "planes", (torch.float32,), M * N), planes.numel() * 4, ctypes.byref(splits), ws_p, ws_n, ctypes.byref(cfg),
                                    _stream(stream)))
    return planes, splits.value


def fp8_gemm_qkv_rope(A, A_scale_transposed, B_transposed, B_scale_transposed, q_norm_weight, k_norm_weight, eps, cos_table, sin_table, positions,
                      n_q_heads, n_kv_heads, M, N, K, out_fp8=False, stream=None, workspace=None, tile=_lib.TILE_AUTO, split_k=0,
                      b_preshuffled=False):
    """The QKV projection with per-head RMSNorm (weights [128] or None) and rotate-half RoPE of the query and key heads fused
    behind it (planned by the reference, README.md:16).  Heads are 128 wide; cos_table / sin_table [rows, 64] float32,
    positions [M] int32.  Returns the bf16 tensor [M,N], or (codes uint8 [M,N], scales float32 [N/128, M]) with out_fp8."""
    dev = B_transposed.device
    kb = K // 128 if K % 128 == 0 else 0
    if workspace is None:
        n = int(lib.llmmm_fp8_gemm_qkv_rope_workspace(M, N, K)) + _a_workspace_bytes(A, M, N, K, False)
        workspace = torch.empty(max(n, 16), dtype=torch.uint8, device=dev)
    out = torch.empty((M, N), dtype=torch.uint8 if out_fp8 else torch.bfloat16, device=dev)
    sc = torch.empty(((N + 127) // 128, M), dtype=torch.float32, device=dev) if out_fp8 else None
    rows = cos_table.shape[0]
    a_p, as_p, a_layout, _keep = _a_operand(A, A_scale_transposed, M, K, False)
    cfg = GemmCfg(tile, split_k, _lib.FP8_B_PRESHUFFLED if b_preshuffled else _lib.FP8_B_ROWS, a_layout)
    check(lib.llmmm_fp8_gemm_qkv_rope(
        _lib.OUT_FP8Q if out_fp8 else _lib.OUT_BF16, a_p, as_p,
        _ptr(B_transposed, "B_transposed", _FP8_DTYPES, N * K), _ptr(B_scale_transposed, "B_scale_transposed", (torch.float32,), ((N + 127) // 128) * kb),
        _ptr(out, "out"), _ptr(sc, "out_scale") if out_fp8 else None,
        _ptr(q_norm_weight, "q_norm_weight", (torch.float32,), 128) if q_norm_weight is not None else None,
        _ptr(k_norm_weight, "k_norm_weight", (torch.float32,), 128) if k_norm_weight is not None else None, ctypes.c_float(eps),
        _ptr(cos_table, "cos_table", (torch.float32,), rows * 64), _ptr(sin_table, "sin_table", (torch.float32,), rows * 64), rows,
        _ptr(positions, "positions", (torch.int32,), M), n_q_heads, n_kv_heads, M, N, K, ctypes.c_void_p(workspace.data_ptr()),
        workspace.numel() * workspace.element_size(), ctypes.byref(cfg), _stream(stream)))
    return (out, sc) if out_fp8 else out


# ------------------------------------------------------------------------------------- offline layout helpers
def construct_mfma_B_layout(dst, src_transposed, N, K, stream=None):
    """The role of ``LLMMM::construct_m16n8k32_B_layout(dst, src_transposed, N, K, stream)``
    (src/base/base.h:13, src/base/base.cu:222-271): the weights Bt [N,K] e4m3, permuted once into the order the
    matrix instructions read them in -- here the 16x16x128 MFMA operand image of gfx950, consumed by the FP8 GEMMs
    with ``b_preshuffled=True``.  Raises RuntimeError("K must be greater than 0 and divisible by 128.") like the
    reference (base.cu:265-267)."""
    check(lib.llmmm_fp8_preshuffle_b(_ptr(src_transposed, "src_transposed", _FP8_DTYPES, N * K), _ptr(dst, "dst", _FP8_DTYPES, N * K), N, K,
                                     _stream(stream)))


def restore_B_layout(dst_transposed, src, N, K, stream=None):
    """Exact inverse of :func:`construct_mfma_B_layout` (the reference checks its permutation the same way,
    examples/005.fp8.mm.opt.cu:710-765)."""
    check(lib.llmmm_fp8_unshuffle_b(_ptr(src, "src", _FP8_DTYPES, N * K), _ptr(dst_transposed, "dst_transposed", _FP8_DTYPES, N * K), N, K,
                                    _stream(stream)))


def preshuffle_weight(bq, stream=None):
    """Bt [N,K] e4m3 codes -> a new tensor holding the pre-shuffled image (same shape and dtype)."""
    N, K = bq.shape
    out = torch.empty_like(bq)
    construct_mfma_B_layout(out, bq, N, K, stream)
    return out


def transpose_matrix__aligned_128(dst, src, M, N, stream=None):
    """``LLMMM::transpose_matrix__aligned_128<T>(dst, src, M, N, stream)`` (src/base/base.cu:124-153): dst [N,M] =
    transpose of src [M,N] for 1-byte (e4m3) and 4-byte (float) elements.  Raises
    RuntimeError("M or N can't be divided 128.") unless both are multiples of 128 (base.cu:127-129)."""
    if src.dtype != dst.dtype or src.element_size() not in (1, 4):
        raise RuntimeError("T is not supported.")
    check(lib.llmmm_transpose(src.element_size(), _ptr(src, "src", numel=M * N), _ptr(dst, "dst", numel=M * N), M, N, _stream(stream)))
