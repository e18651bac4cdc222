/*
 * llmmm.h -- C ABI of the MI355X (gfx950) implementation of LLMMM's matrix-multiplication core.
 *
 * Every entry point takes plain device pointers and sizes, allocates nothing, never
 * synchronises the device and enqueues its work on the caller's HIP stream (passed as void*,
 * NULL = default stream), exactly like the reference's host launchers.  All functions return
 * LLMMM_OK or one of the LLMMM_ERR_* codes below; argument errors are detected before any
 * device work is enqueued.  The C++ drop-in shims in include/llmmm/mm/ turn non-zero codes into
 * the std::runtime_error the reference throws.
 *
 * Data layouts (row-major everywhere, as in the reference):
 *   FP16/BF16 GEMM  A[m*K+k], B[k*N+n] (or Bt[n*K+k]), C[m*N+n]      src/mm/fp16/mm.cuh:102,103,236
 *   FP8 GEMM        A[m*K+k] e4m3, As[(k/128)*M+m], Bt[n*K+k] e4m3,
 *                   Bs[(n/128)*(K/128)+k/128], C[m*N+n], Cs[(n/128)*M+m]
 *                                                                    examples/005.fp8.mm.cu:131,157,168,212,774,2698
 *   e4m3 = OCP FP8 E4M3 (bias 7, max 448, no inf, NaN 0x7F/0xFF), the format of __nv_fp8_e4m3.
 */
#ifndef LLMMM_H
#define LLMMM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LLMMM_API __attribute__((visibility("default")))

/* ---- status codes ---------------------------------------------------------------------- */
#define LLMMM_OK 0
#define LLMMM_ERR_NOT_ALIGNED 1      /* "M or N or K are not aligned."   src/mm/fp16/mm.cu:19-21 */
#define LLMMM_ERR_UNSUPPORTED_TYPE 2 /* "T is not supported."            src/mm/fp16/mm.cu:15-17 */
#define LLMMM_ERR_INVALID_ARGUMENT 3 /* null / misaligned pointer, non-positive size, bad enum    */
#define LLMMM_ERR_WORKSPACE 4        /* workspace missing or too small for the chosen split-K     */
#define LLMMM_ERR_RUNTIME 5          /* a HIP call failed (the reference prints and exits,        */
                                     /* src/util/macro.h:26-33; here the caller decides)          */

/* ---- enums ----------------------------------------------------------------------------- */
#define LLMMM_DTYPE_F16 0  /* half            src/mm/fp16/mm.cu:44 */
#define LLMMM_DTYPE_BF16 1 /* __nv_bfloat16   src/mm/fp16/mm.cu:45-46 */
#define LLMMM_DTYPE_F32 2  /* float: input type of the quantisers only */

#define LLMMM_B_ROW_MAJOR 0  /* B[K,N], the reference layout (src/mm/fp16/mm.cuh:103) */
#define LLMMM_B_TRANSPOSED 1 /* Bt[N,K]; an extension, same arithmetic */

#define LLMMM_OUT_F32 0  /* ...__output_fp32              examples/005.fp8.mm.cu:217-225 */
#define LLMMM_OUT_BF16 1 /* same result rounded to bf16 (no reference kernel; RNE cast of the fp32 result) */
#define LLMMM_OUT_FP8Q 2 /* ...__C_1x128__output_fp8      examples/005.fp8.mm.cu:2467-2476 */
#define LLMMM_OUT_FP8Q_SWIGLU 3 /* SiLU(gate) * up, then the same 1x128 quantisation; no reference kernel: the
                                   fusion the reference plans next (README.md:16).  See llmmm_fp8_gemm. */

#define LLMMM_QUANT_1x128_T 0   /* <1,128,true>    activations: scale[(n/128)*M + m]           examples/005.fp8.mm.cu:2686 */
#define LLMMM_QUANT_128x128 1   /* <128,128,false> weights:     scale[(m/128)*ceil(N/128)+n/128] examples/005.fp8.mm.cu:2739 */
#define LLMMM_QUANT_1x128 2     /* <1,128,false>                scale[m*ceil(N/128) + n/128] */
#define LLMMM_QUANT_128x128_T 3 /* <128,128,true>               scale[(n/128)*M + m/128] */

/* Kernel selection for llmmm_fp8_gemm_ex / llmmm_fp16_gemm_ex (the auto-tune driver's knobs).
 * tile: LLMMM_TILE_AUTO or one of the explicit ids; split_k: 0 = auto, >= 1 explicit. */
#define LLMMM_TILE_AUTO (-1)
#define LLMMM_TILE_256x256 0
#define LLMMM_TILE_128x256 1
#define LLMMM_TILE_256x128 2
#define LLMMM_TILE_128x128 3
#define LLMMM_TILE_64x128 4 /* FP16/BF16 GEMM only: small problems */
#define LLMMM_TILE_128x160 5 /* FP8 GEMM only, N % 160 == 0, fp32 / bf16 / residual-add outputs (no 1x128-grouped epilogue):
                              * 2560-column outputs in 16 tiles per row -- one tile per CU at M = 2048 */
#define LLMMM_TILE_SKINNY 8 /* M <= 128 weight-streaming kernel */
#define LLMMM_TILE_STRIP 9  /* FP8 GEMM, M <= 32, K >= 1024, fp32 / bf16 / residual-add outputs, and the 1x128-grouped fp8 output for
                             * M <= 16: the weight-streaming kernel in strips of 16 or 32 columns over all of K -- the K split
                             * happens inside the workgroup, one launch, no workspace */

/* Weight layout of the FP8 GEMM's B operand (llmmm_gemm_cfg.b_layout). */
#define LLMMM_FP8_B_ROWS 0        /* Bt[N,K] row-major, the reference layout (examples/005.fp8.mm.cu:157) */
#define LLMMM_FP8_B_PRESHUFFLED 1 /* the image llmmm_fp8_preshuffle_b writes */

/* What the FP8 GEMM's A argument points at (llmmm_gemm_cfg.a_layout). */
#define LLMMM_FP8_A_QUANTISED 0  /* A [M,K] e4m3 + As [K/128, M]: the reference's operand (examples/005.fp8.mm.cu:157) */
#define LLMMM_FP8_A_SWIGLU_F32 1 /* A is the fp32 result G [M, 2K] of a gate_up projection (llmmm_fp8_gemm with LLMMM_OUT_F32), As is
                                  * ignored: the GEMM runs on quantise_1x128(silu(G[:, :K]) * G[:, K:]), which the kernel makes itself --
                                  * see llmmm_fp8_swiglu_a_workspace */

#define LLMMM_FP8_A_PLANES_RMSNORM 2 /* A points at a llmmm_a_planes_rmsnorm (host memory): the operand is the RMSNorm of a hidden
                                      * state that is still in pieces, see llmmm_fp8_gemm_planes */

typedef struct llmmm_gemm_cfg {
  int tile;
  int split_k;
  int b_layout; /* FP8 only: LLMMM_FP8_B_ROWS (0, the default) or LLMMM_FP8_B_PRESHUFFLED; the FP16 GEMM ignores it */
  int a_layout; /* FP8 only: LLMMM_FP8_A_QUANTISED (0, the default), LLMMM_FP8_A_SWIGLU_F32 or LLMMM_FP8_A_PLANES_RMSNORM */
} llmmm_gemm_cfg;

/* ---- FP16 / BF16 GEMM -------------------------------------------------------------------
 * Replaces  template<T> void LLMMM::fp16_mm(const T* A, const T* B, T* C, int M, int N, int K,
 *                                           cudaStream_t)      src/mm/fp16/mm.h:9-10, mm.cu:6-42.
 * C = A * B with fp32 accumulation, result rounded (nearest even) to the input type.
 * Requires M % 128 == 0, N % 128 == 0, K % 16 == 0 (the reference: M,N % 256, K % 16; the C++
 * shim enforces the reference's stricter rule).  Pointers must be 16-byte aligned. */
LLMMM_API int llmmm_fp16_gemm(int dtype, const void* A, const void* B, void* C, int M, int N, int K, int b_layout, void* stream);
LLMMM_API int llmmm_fp16_gemm_ex(int dtype, const void* A, const void* B, void* C, int M, int N, int K, int b_layout,
                                 const llmmm_gemm_cfg* cfg, void* stream);

/* ---- FP8 blockwise GEMM -----------------------------------------------------------------
 * Replaces  fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(A, A_scale_transposed,
 *             B_transposed, B_scale_transposed, C, M, N, K, stream)   examples/005.fp8.mm.cu:217-246
 * and       fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(..., C,
 *             C_scale_transposed, M, N, K, stream)                    examples/005.fp8.mm.cu:2467-2500,
 *                                                                     examples/005.fp8.mm.opt.cu:468-508.
 * C is float* (OUT_F32), bf16* (OUT_BF16) or e4m3 uint8_t* (OUT_FP8Q); Cs is only used (and
 * required) for OUT_FP8Q.  N % 128 == 0 and K % 128 == 0 are required.  M % 128 == 0 runs the
 * MFMA tile kernels (the reference's domain); 1 <= M < 128 runs the weight-streaming kernel
 * (so does M = 128 when LLMMM_TILE_SKINNY is requested through llmmm_fp8_gemm_ex).  Other M are
 * rejected as not aligned.
 * LLMMM_OUT_FP8Q_SWIGLU (the gate_up projection of a gated MLP): Bt holds the gate rows in [0, N/2) and the
 * up rows in [N/2, N) (N % 256 == 0; Bs covers all N rows as usual).  With C32 = the fp32 result above,
 * h[m,j] = silu(C32[m,j]) * C32[m,N/2+j], silu(x) = x / (1 + exp(-x)) in fp32 (hardware exp2 and
 * reciprocal, each within about an ulp), and the output is h quantised per 1x128 like OUT_FP8Q:
 * C = e4m3 uint8_t[M, N/2], Cs = float[(N/2)/128, M].  For M <= 128 this output always goes
 * through the workspace (at least one plane of M * N floats is required).
 * Split-K: shapes with too few tiles or column groups to fill the GPU split K over several
 * workgroups; each split stores a plane of fp32 partial sums into `workspace` and a second
 * kernel adds the planes in split order (a fixed order: results do not depend on timing) and
 * applies the epilogue.  `workspace` is plain scratch of llmmm_fp8_gemm_workspace() bytes, needs
 * no initialisation and holds nothing between calls.  With workspace == NULL (or one too small
 * for the split the library would pick) K is split less or not at all; an explicit
 * cfg->split_k that does not fit is an error.  Calls that share a workspace must be ordered on
 * one stream. */
LLMMM_API int llmmm_fp8_gemm(int out_kind, const void* A, const float* As, const void* Bt, const float* Bs, void* C, float* Cs,
                             int M, int N, int K, void* workspace, size_t workspace_bytes, void* stream);
LLMMM_API int llmmm_fp8_gemm_ex(int out_kind, const void* A, const float* As, const void* Bt, const float* Bs, void* C, float* Cs,
                                int M, int N, int K, void* workspace, size_t workspace_bytes, const llmmm_gemm_cfg* cfg,
                                void* stream);
/* Bytes of workspace that the configuration the library picks for this shape and output needs
 * (0 when it neither splits K nor goes through a plane); an explicit split_k = S needs S * M * N * 4 bytes.  No
 * reference counterpart: split-K is "still to do" there (README.md:22). */
LLMMM_API size_t llmmm_fp8_gemm_workspace(int out_kind, int M, int N, int K);
/* The configuration llmmm_fp8_gemm would use for this shape (tune table, then heuristic). */
LLMMM_API int llmmm_fp8_gemm_query(int out_kind, int M, int N, int K, llmmm_gemm_cfg* cfg);

/* The same GEMM for callers that cannot allocate device memory and have no workspace to pass: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  The split-K
 * planes live in a fixed array of LLMMM_STATIC_WS_BYTES inside the library's device image (every GPU the library runs on
 * holds its own copy until the process ends); the call allocates and frees nothing and is otherwise
 * llmmm_fp8_gemm(out_kind, ..., workspace of llmmm_fp8_gemm_workspace(out_kind, M, N, K) bytes), bit for bit.  Shapes
 * whose planes need more than LLMMM_STATIC_WS_BYTES return LLMMM_ERR_WORKSPACE (never a silently smaller split).  All
 * calls on one GPU share that GPU's array: calls that overlap in time on one GPU (different streams, different
 * threads) race on it -- order them on one stream.  The array's address is looked up on the first call per device
 * (one runtime query, not capturable): make one call per device before capturing. */
#define LLMMM_STATIC_WS_BYTES (16u << 20)
LLMMM_API int llmmm_fp8_gemm_static_ws(int out_kind, const void* A, const float* As, const void* Bt, const float* Bs, void* C, float* Cs,
                                       int M, int N, int K, void* stream);

/* ---- FP8 blockwise quantiser ------------------------------------------------------------
 * Replaces  template<int QUANT_M, int QUANT_N, bool SCALE_TRANSPOSE>
 *           void fp8_blockwise_symmetric_quantization(const float* x, __nv_fp8_e4m3* q,
 *                float* scale, int M, int N, cudaStream_t)             examples/005.fp8.mm.cu:547-563.
 * x [M,N] fp32 -> q [M,N] e4m3 + scales (layout per `kind`).  Any M; N % 4 == 0. */
LLMMM_API int llmmm_quant_fp8(int kind, const float* x, void* q, float* scale, int M, int N, void* stream);

/* RMSNorm fused in front of the activation quantiser -- the "RMSNorm + fp8 dynamic quant" fusion the reference plans
 * (README.md:16); it has no kernel for it.  x [M,K] (in_dtype: LLMMM_DTYPE_F32, _BF16 or _F16), weight [K] fp32:
 *   y = x / sqrt(mean_k(x^2) + eps) * weight   (fp32),   then   q, scale = 1x128 quantisation of y as by
 * llmmm_quant_fp8(LLMMM_QUANT_1x128_T): q [M,K] e4m3, scale [(k/128)*M + m] -- the A / A_scale_transposed pair of
 * llmmm_fp8_gemm.  K % 128 == 0; x, weight and q 16-byte aligned.  The sum of squares is taken in a fixed order
 * (documented at the kernel), so results are reproducible bit for bit. */
LLMMM_API int llmmm_rmsnorm_quant_fp8(int in_dtype, const void* x, const float* weight, float eps, void* q, float* scale, int M, int K,
                                      void* stream);

/* Decoder-block epilogue fused behind a projection back to the hidden size (O, down) -- the "RMSNorm + fp8 dynamic
 * quant fused into MM" of the reference's plan (README.md:16); no reference kernel.  With C32 = the fp32 result of the
 * blockwise GEMM of llmmm_fp8_gemm (same operands, same layouts):
 *   h          = C32 + residual                          (fp32; residual [M,N] of hidden_dtype)
 *   hidden_out = hidden_dtype(h)                         (the new residual stream; may be the same buffer as residual)
 *   q, q_scale = llmmm_rmsnorm_quant_fp8(hidden_out, norm_weight, eps)   -- bit for bit what the separate call gives
 * so the next projection's A operand leaves this call.  Small M (the weight-streaming kernel) and split-K runs go
 * through fp32 planes in `workspace` (llmmm_fp8_gemm_add_rmsnorm_quant_workspace bytes), which one kernel sums in split
 * order, adds the residual to, normalises and quantises; an unsplit tile kernel adds the residual in its own epilogue,
 * the norm + quantiser kernel follows, and no workspace is needed (the query function then returns 0).
 * hidden_dtype: LLMMM_DTYPE_F32 / _BF16 / _F16.  N % 128 == 0, N <= 10240, K % 128 == 0, M as for llmmm_fp8_gemm.
 * cfg may be NULL (library's choice of kernel and split). */
LLMMM_API int    llmmm_fp8_gemm_add_rmsnorm_quant(const void* A, const float* As, const void* Bt, const float* Bs, int hidden_dtype,
                                                  const void* residual, void* hidden_out, const float* norm_weight, float eps, void* q,
                                                  float* q_scale, int M, int N, int K, void* workspace, size_t workspace_bytes,
                                                  const llmmm_gemm_cfg* cfg, void* stream);
LLMMM_API size_t llmmm_fp8_gemm_add_rmsnorm_quant_workspace(int M, int N, int K);

/* The QKV projection with what stands between it and attention fused behind it -- per-head RMSNorm (the q_norm / k_norm
 * of Qwen3) and rotary position embedding; "RMSNorm, RoPE fused into MM" is on the reference's plan (README.md:16), no
 * reference kernel.  Heads are 128 columns wide: columns [0, n_q_heads*128) are query heads, the next n_kv_heads*128 key
 * heads, the last n_kv_heads*128 value heads; N = (n_q_heads + 2 n_kv_heads) * 128.  With C32 the fp32 GEMM result:
 *   query / key head x (128 values of row m):
 *     x <- x / sqrt(mean(x^2) + eps) * w          w = q_norm_weight / k_norm_weight [128]; skipped when that pointer is NULL
 *     p  = clamp(positions[m], 0, table_rows-1)   positions [M] int32; cos_table / sin_table [table_rows, 64] fp32
 *     y[i]    = x[i]    * cos[p,i] - x[i+64] * sin[p,i]        (rotate-half pairing, i < 64)
 *     y[i+64] = x[i+64] * cos[p,i] + x[i]    * sin[p,i]
 *   value heads: y = x.
 * out_kind LLMMM_OUT_BF16: out [M,N] bf16.  LLMMM_OUT_FP8Q: out [M,N] e4m3 and out_scale [N/128, M] -- one scale per row
 * and head (the 1x128 rule of the fused C quantisation), for an FP8 attention.
 * Small M (the weight-streaming kernel) and split-K runs go through fp32 planes in `workspace`
 * (llmmm_fp8_gemm_qkv_rope_workspace bytes), where the second kernel takes the place of the split-K reduce kernel, so norm
 * and rope cost no launch of their own; an unsplit tile kernel applies them to its accumulators and needs no workspace
 * (the query function then returns 0).  Both routes perform the same operations in the same order: the results agree
 * bit for bit with each other for equal fp32 sums. */
LLMMM_API int    llmmm_fp8_gemm_qkv_rope(int out_kind, const void* A, const float* As, const void* Bt, const float* Bs, void* out,
                                         float* out_scale, const float* q_norm_weight, const float* k_norm_weight, float eps,
                                         const float* cos_table, const float* sin_table, int table_rows, const int* positions,
                                         int n_q_heads, int n_kv_heads, int M, int N, int K, void* workspace, size_t workspace_bytes,
                                         const llmmm_gemm_cfg* cfg, void* stream);
LLMMM_API size_t llmmm_fp8_gemm_qkv_rope_workspace(int M, int N, int K);

/* The gated-MLP activation fused into the *consumer*: with cfg.a_layout = LLMMM_FP8_A_SWIGLU_F32, llmmm_fp8_gemm_ex and
 * llmmm_fp8_gemm_add_rmsnorm_quant (the down projection) take the fp32 gate_up result G [M, 2K] as their A argument and run on
 * h = silu(G[:, :K]) * G[:, K:] quantised 1x128 -- the operand LLMMM_OUT_FP8Q_SWIGLU would have written, bit for bit (planned by
 * the reference, README.md:16; no reference kernel).  For M <= 4 every workgroup of the weight-streaming kernel makes the
 * slices of h it needs while its first weights are in flight, so the activation costs no launch (gate_up: one kernel with fp32
 * output; down: its usual kernels; K / 128 / split_k <= 32).  Otherwise the library quantises h into the front of the workspace
 * first, which then must hold llmmm_fp8_swiglu_a_workspace(M, N, K) bytes (0 when the kernel does it itself) on top of what
 * the GEMM wants. */
LLMMM_API size_t llmmm_fp8_swiglu_a_workspace(int M, int N, int K);

/* The block epilogue fused into the *consumer* (single-stream decode).  llmmm_fp8_gemm_planes runs a projection back to the
 * hidden size (O, down) and stops at its fp32 partial sums: `planes` [*splits][M][N] (llmmm_fp8_gemm_planes_bytes bytes hold
 * the library's choice of split; with less room the split shrinks; cfg as for llmmm_fp8_gemm_ex, `workspace` only serves an
 * a_layout that has to be quantised first).  The next projection (QKV, gate_up; any FP8 entry point) then takes
 * cfg.a_layout = LLMMM_FP8_A_PLANES_RMSNORM and a llmmm_a_planes_rmsnorm in place of A (As ignored; K of that call = N of
 * the planes), and runs on
 *   h = sum of the planes in split order + residual;  hidden_out = hidden_dtype(h);  A = quantise_1x128(rmsnorm(hidden_out) * w)
 * -- exactly the hidden state, codes and scales llmmm_fp8_gemm_add_rmsnorm_quant delivers, bit for bit.  For M <= 2 and
 * K <= 3072 every workgroup of the weight-streaming kernel makes the operand itself while its first weights are in flight
 * (no reduce kernel, no norm kernel: one launch per projection), provided hidden_out is a buffer of its own, not the
 * residual, and there are at most 10 planes.  Otherwise the library runs the fused reduce + norm + quantise kernel into the
 * front of the workspace first (llmmm_fp8_planes_rmsnorm_a_workspace extra bytes, or M * K + K / 128 * M * 4 rounded up to
 * 256 each when one of the provisos fails).  The generating kernel writes fp32 only; for another output kind its result passes
 * through one fp32 plane, which llmmm_fp8_planes_rmsnorm_a_workspace counts in (M * N * 4 bytes where the kernel generates).
 * The size queries of this header answer for every a_layout: a shape that would run in column strips with quantised
 * activations runs in the split-K form with generated ones, and the queries return what that form needs.
 * Planned by the reference (README.md:16), no reference kernel. */
typedef struct llmmm_a_planes_rmsnorm {
  const float* planes;      /* [splits][M][K] fp32, from llmmm_fp8_gemm_planes */
  int          splits;
  int          hidden_dtype; /* LLMMM_DTYPE_F32 / _BF16 / _F16 */
  const void*  residual;    /* [M, K] */
  void*        hidden_out;  /* [M, K] */
  const float* norm_weight; /* [K] */
  float        eps;
} llmmm_a_planes_rmsnorm;
LLMMM_API int    llmmm_fp8_gemm_planes(const void* A, const float* As, const void* Bt, const float* Bs, int M, int N, int K, float* planes,
                                       size_t planes_bytes, int* splits, void* workspace, size_t workspace_bytes, const llmmm_gemm_cfg* cfg,
                                       void* stream);
LLMMM_API size_t llmmm_fp8_gemm_planes_bytes(int M, int N, int K);
LLMMM_API size_t llmmm_fp8_planes_rmsnorm_a_workspace(int M, int N, int K);

/* ---- offline layout helpers --------------------------------------------------------------
 * llmmm_fp8_preshuffle_b takes the role of  construct_m16n8k32_B_layout(dst, src_transposed, N, K,
 * stream)  (src/base/base.h:13, src/base/base.cu:222-271): a one-off permutation of the weights
 * Bt[N,K] e4m3 into the order the matrix instructions consume them in.  The byte order is this
 * library's (MFMA 16x16x128 on gfx950), not the reference's mma.m16n8k32 one: Bp consists of
 * 2 KB blocks, block (n/16, k/128) at ((n/16) * (K/128) + k/128) * 2048, each the LDS image of
 * its 16 rows x 128 bytes (16-byte chunk c of row r at r*128 + ((c ^ swz(r)) << 4), with
 * swz(r) = ((r >> 1) & 7) ^ ((((r >> 2) ^ (r >> 3)) & 1) << 1)).  Every FP8 GEMM entry point
 * accepts it through cfg->b_layout = LLMMM_FP8_B_PRESHUFFLED, with the scales Bs unchanged;
 * results are bit-identical to the row-major layout's.  llmmm_fp8_unshuffle_b is the exact inverse.
 * N % 16 == 0 and K % 128 == 0 (the reference's text "K must be greater than 0 and divisible by
 * 128." is left in llmmm_last_error); src and dst must not overlap.
 * llmmm_transpose replaces  transpose_matrix__aligned_128<T>(dst, src, M, N, stream)
 * (src/base/base.h:9, src/base/base.cu:124-153) for sizeof(T) = 1 (e4m3) and 4 (float):
 * dst[n*M+m] = src[m*N+n]; M % 128 == 0 and N % 128 == 0 ("M or N can't be divided 128."). */
LLMMM_API int llmmm_fp8_preshuffle_b(const void* Bt, void* Bp, int N, int K, void* stream);
LLMMM_API int llmmm_fp8_unshuffle_b(const void* Bp, void* Bt, int N, int K, void* stream);
LLMMM_API int llmmm_transpose(int elem_size, const void* src, void* dst, int M, int N, void* stream);

/* Measurement probes (register-only MFMA loops, a streaming read, the product kernels built with clock readings) are
 * exported by the same library but declared in a header of their own, llmmm_probe.h: they are instrumentation, not
 * part of the drop-in surface. */

/* ---- misc ------------------------------------------------------------------------------- */
LLMMM_API const char* llmmm_error_string(int code); /* the reference's exception texts for codes 1 and 2 */
LLMMM_API const char* llmmm_last_error(void);       /* thread-local detail of the last failure */
LLMMM_API int         llmmm_version(void);

#ifdef __cplusplus
}
#endif
#endif /* LLMMM_H */
