"""CPU oracle for the LLMMM matrix-multiplication path: numpy front-end of ``oracle.c``.

TEST INFRASTRUCTURE ONLY.  Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline``
leg of ``bench.py`` may import this package; the product library (``llmmm_amd``) never does.

Every function restates a piece of the reference (file:line given at the C definition in
``oracle.c``); what pins each of them is listed in the header of that file.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")


def build(force=False):
    """Compile ``oracle.c`` with gcc (OpenMP, no contraction, no fast-math)."""
    src = os.path.join(_HERE, "oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


def _load():
    build()  # no-op unless the library is missing or older than oracle.c
    lib = ctypes.CDLL(_LIB_PATH)
    c = ctypes
    f32p, u8p, u16p = c.POINTER(c.c_float), c.POINTER(c.c_uint8), c.POINTER(c.c_uint16)
    sig = {
        "oracle_num_threads": (c.c_int, []),
        "oracle_set_num_threads": (None, [c.c_int]),
        "oracle_f16_to_f32": (c.c_float, [c.c_uint16]),
        "oracle_f32_to_f16": (c.c_uint16, [c.c_float]),
        "oracle_bf16_to_f32": (c.c_float, [c.c_uint16]),
        "oracle_f32_to_bf16": (c.c_uint16, [c.c_float]),
        "oracle_e4m3_decode": (c.c_float, [c.c_uint8]),
        "oracle_e4m3_encode": (c.c_uint8, [c.c_float]),
        "oracle_kahan_gemm": (None, [f32p, f32p, f32p, c.c_int, c.c_int, c.c_int, c.c_int]),
        "oracle_kahan_gemm_bt": (None, [f32p, f32p, f32p, c.c_int, c.c_int, c.c_int, c.c_int]),
        "oracle_double_gemm": (None, [f32p, f32p, f32p, c.c_int, c.c_int, c.c_int]),
        "oracle_quant_fp8": (None, [f32p, u8p, f32p, c.c_int, c.c_int, c.c_int, c.c_int]),
        "oracle_dequant_fp8": (None, [u8p, f32p, f32p, c.c_int, c.c_int, c.c_int, c.c_int]),
        "oracle_fp8_gemm": (c.c_int, [u8p, f32p, u8p, f32p, f32p, c.c_int, c.c_int, c.c_int, c.c_int, c.c_int]),
        "oracle_requant_c_1x128": (None, [f32p, u8p, f32p, c.c_int, c.c_int, c.c_int, c.c_int]),
        "oracle_rmsnorm": (None, [f32p, f32p, c.c_float, f32p, c.c_int, c.c_int]),
        "oracle_qk_norm_rope": (None, [f32p, f32p, f32p, c.c_float, f32p, f32p, c.c_int, c.POINTER(c.c_int32), c.c_int, c.c_int, f32p, c.c_int]),
        "oracle_e4m3_encode_n": (None, [f32p, u8p, c.c_size_t]),
        "oracle_e4m3_decode_n": (None, [u8p, f32p, c.c_size_t]),
        "oracle_f32_to_f16_n": (None, [f32p, u16p, c.c_size_t]),
        "oracle_f16_to_f32_n": (None, [u16p, f32p, c.c_size_t]),
        "oracle_f32_to_bf16_n": (None, [f32p, u16p, c.c_size_t]),
        "oracle_bf16_to_f32_n": (None, [u16p, f32p, c.c_size_t]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    return lib


_lib = _load()


def _p(a, ct):
    return a.ctypes.data_as(ctypes.POINTER(ct))


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _u8(a):
    a = np.ascontiguousarray(a)
    assert a.dtype == np.uint8, a.dtype
    return a


def num_threads():
    return int(_lib.oracle_num_threads())


def set_num_threads(n):
    _lib.oracle_set_num_threads(int(n))


# ----------------------------------------------------------------------------- scalar formats
def e4m3_decode(codes):
    """uint8 e4m3 codes -> float32 (NaN for 0x7F / 0xFF)."""
    q = _u8(codes)
    out = np.empty(q.shape, np.float32)
    _lib.oracle_e4m3_decode_n(_p(q, ctypes.c_uint8), _p(out, ctypes.c_float), q.size)
    return out


def e4m3_encode(x):
    """float32 -> e4m3 codes, RNE, saturate-to-finite, NaN -> 0x7F."""
    x = _f32(x)
    out = np.empty(x.shape, np.uint8)
    _lib.oracle_e4m3_encode_n(_p(x, ctypes.c_float), _p(out, ctypes.c_uint8), x.size)
    return out


def f32_to_f16_bits(x):
    x = _f32(x)
    out = np.empty(x.shape, np.uint16)
    _lib.oracle_f32_to_f16_n(_p(x, ctypes.c_float), _p(out, ctypes.c_uint16), x.size)
    return out


def f16_bits_to_f32(h):
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, np.float32)
    _lib.oracle_f16_to_f32_n(_p(h, ctypes.c_uint16), _p(out, ctypes.c_float), h.size)
    return out


def f32_to_bf16_bits(x):
    x = _f32(x)
    out = np.empty(x.shape, np.uint16)
    _lib.oracle_f32_to_bf16_n(_p(x, ctypes.c_float), _p(out, ctypes.c_uint16), x.size)
    return out


def bf16_bits_to_f32(h):
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, np.float32)
    _lib.oracle_bf16_to_f32_n(_p(h, ctypes.c_uint16), _p(out, ctypes.c_float), h.size)
    return out


def e4m3_code_index(codes):
    """Monotone integer order of e4m3 values: index(a) < index(b) <=> value(a) < value(b).

    +0 and -0 share index 0; NaN codes map to +-127 (outside the finite range +-126)."""
    c = np.asarray(codes, dtype=np.uint8).astype(np.int32)
    mag = c & 0x7F
    return np.where(c & 0x80, -mag, mag)


# ----------------------------------------------------------------------------- GEMM references
def kahan_gemm(A, B, fused=True):
    """fp32 Kahan-compensated C = A[M,K] @ B[K,N] (test/kahan.cu:16-26)."""
    A, B = _f32(A), _f32(B)
    M, K = A.shape
    K2, N = B.shape
    assert K == K2
    C = np.empty((M, N), np.float32)
    _lib.oracle_kahan_gemm(_p(A, ctypes.c_float), _p(B, ctypes.c_float), _p(C, ctypes.c_float), M, N, K, int(fused))
    return C


def kahan_gemm_bt(A, Bt, fused=True):
    """Same arithmetic with B given as Bt[N,K]."""
    A, Bt = _f32(A), _f32(Bt)
    M, K = A.shape
    N, K2 = Bt.shape
    assert K == K2
    C = np.empty((M, N), np.float32)
    _lib.oracle_kahan_gemm_bt(_p(A, ctypes.c_float), _p(Bt, ctypes.c_float), _p(C, ctypes.c_float), M, N, K, int(fused))
    return C


def double_gemm(A, B):
    """fp32 products accumulated in double (test/kahan.cu:48-55)."""
    A, B = _f32(A), _f32(B)
    M, K = A.shape
    K2, N = B.shape
    assert K == K2
    C = np.empty((M, N), np.float32)
    _lib.oracle_double_gemm(_p(A, ctypes.c_float), _p(B, ctypes.c_float), _p(C, ctypes.c_float), M, N, K)
    return C


# ----------------------------------------------------------------------------- FP8 path
def scale_shape(M, N, quant_m, scale_transpose):
    nb = (N + 127) // 128
    mb = (M + quant_m - 1) // quant_m
    if scale_transpose:
        # the reference strides the transposed layout by M also for 128-row blocks
        # (examples/005.fp8.mm.cu:532-533), so the buffer is [nb, M] with only M/128 used per row
        return (nb, M)
    return (mb, nb)


def quant_fp8(x, quant_m, scale_transpose):
    """examples/005.fp8.mm.cu:439-545.  Returns (codes uint8 [M,N], scales float32)."""
    x = _f32(x)
    M, N = x.shape
    assert quant_m in (1, 128)
    q = np.empty((M, N), np.uint8)
    s = np.zeros(scale_shape(M, N, quant_m, scale_transpose), np.float32)
    _lib.oracle_quant_fp8(_p(x, ctypes.c_float), _p(q, ctypes.c_uint8), _p(s, ctypes.c_float), M, N, quant_m,
                          int(scale_transpose))
    return q, s


def dequant_fp8(q, s, quant_m, scale_transpose):
    q = _u8(q)
    s = _f32(s)
    M, N = q.shape
    x = np.empty((M, N), np.float32)
    _lib.oracle_dequant_fp8(_p(q, ctypes.c_uint8), _p(s, ctypes.c_float), _p(x, ctypes.c_float), M, N, quant_m,
                            int(scale_transpose))
    return x


def fp8_gemm(Aq, As, Bt, Bs, promote=128, assoc=1):
    """Blockwise-scaled GEMM, fp32 result (examples/005.fp8.mm.cu:176-199 / :885-902).

    Aq [M,K] codes, As [K/128,M], Bt [N,K] codes, Bs [ceil(N/128),K/128]."""
    Aq, Bt, As, Bs = _u8(Aq), _u8(Bt), _f32(As), _f32(Bs)
    M, K = Aq.shape
    N, K2 = Bt.shape
    assert K == K2 and As.shape == (K // 128, M) and Bs.shape == ((N + 127) // 128, K // 128), (As.shape, Bs.shape)
    C = np.empty((M, N), np.float32)
    rc = _lib.oracle_fp8_gemm(_p(Aq, ctypes.c_uint8), _p(As, ctypes.c_float), _p(Bt, ctypes.c_uint8),
                              _p(Bs, ctypes.c_float), _p(C, ctypes.c_float), M, N, K, promote, assoc)
    if rc:
        raise RuntimeError("M or N or K are not aligned.")
    return C


def requant_c_1x128(C, reciprocal=True, zero_guard=True):
    """Fused-epilogue arithmetic (examples/005.fp8.mm.opt.cu:401-462): (Cq [M,N], Cs [ceil(N/128), M])."""
    C = _f32(C)
    M, N = C.shape
    Cq = np.empty((M, N), np.uint8)
    Cs = np.empty(((N + 127) // 128, M), np.float32)
    _lib.oracle_requant_c_1x128(_p(C, ctypes.c_float), _p(Cq, ctypes.c_uint8), _p(Cs, ctypes.c_float), M, N,
                                int(reciprocal), int(zero_guard))
    return Cq, Cs


def swiglu(C):
    """h[m, j] = silu(C[m, j]) * C[m, N/2 + j] in fp32, silu(x) = x / (1 + exp(-x)): the gated-MLP activation
    between the gate_up and down projections (gate columns first, up columns second).  The reference has no such
    kernel -- fusing SiLU into the GEMM is on its plan (README.md:16) -- so this definition is the build's own;
    pinned by tests/test_oracle_swiglu.py (known values, the tanh form in float64, limits, gate/up asymmetry)."""
    C = _f32(C)
    half = C.shape[1] // 2
    assert C.shape[1] == 2 * half
    g, u = C[:, :half], C[:, half:]
    with np.errstate(over="ignore"):
        e = np.exp(-g)  # float32
    return ((g / (np.float32(1.0) + e)) * u).astype(np.float32)


def swiglu_requant(C):
    """(Cq [M, N/2], Cs [N/256, M]): the fused epilogue's 1x128 quantisation applied to swiglu(C)."""
    return requant_c_1x128(swiglu(C))


def rmsnorm(x, w, eps):
    """y = x / sqrt(mean(x^2) + eps) * w in fp32, rows of x [M,K] (K % 4 == 0), w [K].  No reference kernel
    (README.md:16 plans the fusion); the summation order is that of 256 GPU lanes, see oracle.c."""
    x, w = _f32(x), _f32(w)
    M, K = x.shape
    assert K % 4 == 0 and w.shape == (K,)
    y = np.empty((M, K), np.float32)
    _lib.oracle_rmsnorm(_p(x, ctypes.c_float), _p(w, ctypes.c_float), ctypes.c_float(eps), _p(y, ctypes.c_float), M, K)
    return y


def rmsnorm_quant(x, w, eps):
    """RMSNorm followed by the activation quantiser (1x128, transposed scales): (q [M,K], s [ceil(K/128), M])."""
    return quant_fp8(rmsnorm(x, w, eps), 1, True)


def qk_norm_rope(x, qw, kw, eps, cos, sin, pos, n_q, n_kv):
    """Per-head RMSNorm (head size 128; weights qw / kw [128] or None) and rotate-half RoPE of the query and key heads
    of a QKV projection result x [M, (n_q + 2 n_kv) * 128]; cos / sin [rows, 64] fp32, pos [M] int32.  No reference
    kernel (README.md:16 plans the fusion); arithmetic order in oracle.c."""
    x = _f32(x)
    M, N = x.shape
    assert N == (n_q + 2 * n_kv) * 128
    cos, sin = _f32(cos), _f32(sin)
    assert cos.shape == sin.shape and cos.shape[1] == 64
    pos = np.ascontiguousarray(pos, dtype=np.int32)
    assert pos.shape == (M,)
    qw = None if qw is None else _f32(qw)
    kw = None if kw is None else _f32(kw)
    y = np.empty((M, N), np.float32)
    _lib.oracle_qk_norm_rope(_p(x, ctypes.c_float), None if qw is None else _p(qw, ctypes.c_float), None if kw is None else _p(kw, ctypes.c_float),
                             ctypes.c_float(eps), _p(cos, ctypes.c_float), _p(sin, ctypes.c_float), cos.shape[0], _p(pos, ctypes.c_int32), n_q, n_kv,
                             _p(y, ctypes.c_float), M)
    return y


# ----------------------------------------------------------------------------- offline layouts
def operand_swizzle_rows16(r):
    """Chunk XOR of row r (0..15) in the 16-row x 128-byte MFMA operand image of the pre-shuffled
    weights: 16-byte chunk c of row r sits at r*128 + ((c ^ swz(r)) << 4)."""
    r = np.asarray(r)
    return ((r >> 1) & 7) ^ ((((r >> 2) ^ (r >> 3)) & 1) << 1)


def preshuffle_b(Bt):
    """The pre-shuffled image of Bt [N,K] (1-byte elements; N % 16 == 0, K % 128 == 0), returned in Bt's shape.

    The MI355X counterpart of construct_m16n8k32_B_layout (src/base/base.cu:222-271): block
    (n/16, k/128) of 2 KB at ((n/16) * (K/128) + k/128) * 2048 holds its 16 rows x 128 bytes with the
    chunks of row r XOR-ed by operand_swizzle_rows16(r).  Pinned by tests/test_oracle_layout.py
    (bijection, block and row confinement, conflict-free operand reads) and, on the GPU, by the
    bit-identity of GEMM results over both layouts."""
    Bt = _u8(Bt)
    N, K = Bt.shape
    if N % 16 or K % 128:
        raise RuntimeError("K must be greater than 0 and divisible by 128." if K % 128 else "N must be divisible by 16.")
    src = Bt.reshape(N // 16, 16, K // 128, 8, 16).transpose(0, 2, 1, 3, 4)  # [rg, kb, r, c, byte]
    out = np.empty_like(src)
    r = np.arange(16)
    swz = operand_swizzle_rows16(r)
    for c in range(8):
        out[:, :, r, c ^ swz, :] = src[:, :, r, c, :]
    return np.ascontiguousarray(out).reshape(N, K)


def unshuffle_b(Bp):
    """Inverse of preshuffle_b."""
    Bp = _u8(Bp)
    N, K = Bp.shape
    img = Bp.reshape(N // 16, K // 128, 16, 8, 16)
    out = np.empty_like(img)
    r = np.arange(16)
    swz = operand_swizzle_rows16(r)
    for c in range(8):
        out[:, :, r, c, :] = img[:, :, r, c ^ swz, :]
    return np.ascontiguousarray(out.transpose(0, 2, 1, 3, 4)).reshape(N, K)


def transpose_aligned_128(src):
    """transpose_matrix__aligned_128 (src/base/base.cu:124-153): dst[n, m] = src[m, n], M and N multiples of 128."""
    M, N = src.shape
    if M % 128 or N % 128:
        raise RuntimeError("M or N can't be divided 128.")
    return np.ascontiguousarray(src.T)
