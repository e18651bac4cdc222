// Internal interface between the C-ABI layer (capi.cpp) and the gfx950 kernel files.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

// Tile ids (LLMMM_TILE_*) and enum values are those of the public header.
#include "../../include/llmmm.h"

namespace llmmm {

// dtype: 0 = fp16, 1 = bf16.  b_layout: 0 = B[K,N] row-major, 1 = Bt[N,K].
hipError_t fp16_gemm_launch(int dtype, int b_layout, int tile, const void* A, const void* B, void* C, int M, int N, int K,
                            hipStream_t stream);

// out_kind: 0 = fp32, 1 = bf16, 2 = e4m3 codes + per-1x128 scales, 3 = SwiGLU (silu(C[:, :N/2]) * C[:, N/2:]) as codes + scales.  S > 1 splits K over S
// workgroups per tile (S <= K/128): `planes` then holds S * M * N floats of partial sums, added
// in split order by a second kernel that also runs the epilogue.  planes != nullptr with S == 1 takes the
// same two-kernel route through one plane (the SwiGLU output from a 128-column tile).  C == nullptr (with planes): only
// the planes are written, no reduce kernel is launched.
// b_layout: LLMMM_FP8_B_ROWS (Bt[N,K] row-major) or LLMMM_FP8_B_PRESHUFFLED (the image fp8_preshuffle_launch writes).
hipError_t fp8_gemm_launch(int out_kind, int tile, int b_layout, const void* A, const float* As, const void* Bt, const float* Bs,
                           void* C, float* Cs, int M, int N, int K, int S, float* planes, hipStream_t stream);

// C = epilogue(planes[0] + planes[1] + ... + planes[S-1]) (that order), planes of M * N floats each.
// Per-head RMSNorm + rotary embedding behind a QKV projection (heads of 128 columns: n_q query, n_kv key, n_kv value).
struct Fp8HeadOp {
  const float* qw         = nullptr;  // norm weights [128] of the query / key heads, nullptr: no norm
  const float* kw         = nullptr;
  const float* cos_t      = nullptr;  // [table_rows, 64]
  const float* sin_t      = nullptr;
  const int*   pos        = nullptr;  // [M] row of the tables, clamped
  float        eps        = 0.f;
  int          table_rows = 0;
  int          n_q        = 0;
  int          n_kv       = 0;
  const void*  residual   = nullptr;  // fp8_gemm_add_residual_launch only: [M, N] of the hidden dtype
  unsigned long long* stamps = nullptr;  // fp8_gemm_phases_launch only: PHASE_STAMPS clock readings per wave (see there)
};
// A tile kernel (no split) with the head op in its epilogue; out_kind LLMMM_OUT_BF16 or LLMMM_OUT_FP8Q.
hipError_t fp8_gemm_qk_rope_launch(int out_kind, int tile, int b_layout, const void* A, const float* As, const void* Bt, const float* Bs, void* C,
                                   float* Cs, int M, int N, int K, const Fp8HeadOp& op, hipStream_t stream);
// A tile kernel (no split) whose epilogue stores hidden = T(C + residual), T = hidden_dtype (LLMMM_DTYPE_*); hidden may be
// the residual buffer.
hipError_t fp8_gemm_add_residual_launch(int hidden_dtype, int tile, int b_layout, const void* A, const float* As, const void* Bt, const float* Bs,
                                        const void* residual, void* hidden, int M, int N, int K, hipStream_t stream);
// Behind a QKV projection whose kernel wrote S fp32 planes: ordered plane sum, per-head RMSNorm (qw / kw [128] or
// nullptr) and rotate-half RoPE (cos / sin tables [table_rows, 64], positions [M]) of the n_q query and n_kv key heads
// of 128 columns, value heads untouched; out_kind LLMMM_OUT_BF16 or LLMMM_OUT_FP8Q (1x128 = per-head scales).
hipError_t fp8_planes_qk_norm_rope_launch(int out_kind, const float* planes, int S, void* C, float* Cs, const float* qw, const float* kw, float eps,
                                          const float* cos_t, const float* sin_t, int table_rows, const int* pos, int n_q, int n_kv, int M,
                                          hipStream_t stream);
// Where a launch of the 256 x 256 tile kernels spends its time: the kernel of fp8_gemm_launch(LLMMM_OUT_FP8Q, LLMMM_TILE_256x256,
// row-major weights) / fp16_gemm_launch(256 x 256 tile, row-major B) built with clock readings at five points of every
// wave -- entry, first operands in LDS (end of the prologue), end of the K loop, last store issued, stores acknowledged.
// stamps[(workgroup * 8 + wave) * PHASE_RECORD + 2 * p] = s_memrealtime (a constant 100 MHz clock) at point p and
// [.. + 2 * p + 1] = s_memtime (shader clock cycles); [.. + PHASE_STAMPS] = the shader cycles the wave spent in the K loop's
// waits for its loads and for the other waves (the barrier of every stage); [.. + PHASE_STAMPS + 1] = the part of that spent
// waiting for its own loads (and LDS reads).  M and N
// multiples of 256.  The results are the product kernels'.
constexpr int PHASE_POINTS = 5, PHASE_STAMPS = 2 * PHASE_POINTS, PHASE_RECORD = PHASE_STAMPS + 2;
hipError_t fp8_gemm_phases_launch(const void* A, const float* As, const void* Bt, const float* Bs, void* C, float* Cs, int M, int N, int K,
                                  unsigned long long* stamps, hipStream_t stream);
hipError_t fp16_gemm_phases_launch(int dtype, const void* A, const void* B, void* C, int M, int N, int K, unsigned long long* stamps, hipStream_t stream);

hipError_t fp8_splitk_reduce_launch(int out_kind, const float* planes, int S, void* C, float* Cs, int M, int N, hipStream_t stream);

// M <= 128 (row groups of 64); S splits of K.  partial == nullptr (S must be 1): complete result in C / Cs.
// Otherwise only the S partial planes `partial` [S][M][N] fp32 are written; run fp8_splitk_reduce_launch behind it.
hipError_t fp8_skinny_launch(int out_kind, int b_layout, const void* A, const float* As, const void* Bt, const float* Bs, void* C,
                             float* Cs, int M, int N, int K, int S, float* partial, hipStream_t stream);

// The weight-streaming kernel in column strips: a workgroup owns 16 output columns over all of K, its eight waves split K and
// add their sums in LDS in wave order -- one launch, no planes, deterministic.  M <= STRIP_MAX_M, N % 16 == 0,
// K % 128 == 0, K >= 1024; out_kind LLMMM_OUT_F32 or LLMMM_OUT_BF16 (no 1x128-grouped outputs: a strip holds an eighth
// of a group).  hipErrorInvalidValue outside these limits.
constexpr int STRIP_MAX_M = 32;
int strip_fragments(int N, int K);  // 16-column fragments per strip the launchers below will use for this shape: 1 or 2
hipError_t fp8_strip_launch(int out_kind, int b_layout, const void* A, const float* As, const void* Bt, const float* Bs, void* C, int M, int N, int K,
                            hipStream_t stream);
// The fused 1x128 re-quantisation from column strips (M <= 16, N % 128 == 0, at most STRIP_XCH_MAX_GROUPS column groups): one
// launch; the eight strips of a group exchange their row maxima through area `xarea` (0 .. STRIP_XCH_AREAS - 1) of a small
// array in the library's device image.  Launches that use the same area must not overlap.
constexpr int STRIP_XCH_AREAS = 32, STRIP_XCH_MAX_GROUPS = 256;
hipError_t fp8_strip_fp8q_launch(int b_layout, const void* A, const float* As, const void* Bt, const float* Bs, void* C, float* Cs, int M, int N, int K,
                                 int xarea, hipStream_t stream);
hipError_t strip_exchange_timeouts(unsigned* out);  // waves that ever gave up waiting in that exchange (synchronises)
// The same with hidden = T(C + residual) as its output (T = hidden_dtype, LLMMM_DTYPE_*; hidden may be the residual buffer).
hipError_t fp8_strip_add_residual_launch(int hidden_dtype, int b_layout, const void* A, const float* As, const void* Bt, const float* Bs, const void* residual,
                                         void* hidden, int M, int N, int K, hipStream_t stream);

// What the weight-streaming kernel needs to make its activations from a hidden state that is still in pieces.
constexpr int SKINNY_GEN_MAX_PLANES = 10;
struct SkinnyGenA {
  const float* planes   = nullptr;  // [splits][M][K] fp32 partial sums of the projection before
  const void*  residual = nullptr;  // [M, K] of the hidden dtype
  void*        hidden   = nullptr;  // [M, K] out: hidden dtype(sum + residual); must not alias the residual
  const float* w        = nullptr;  // [K] RMSNorm weights
  float        eps      = 0.f;
  int          splits   = 0;
};
// The kernel with A = quantise_1x128(rmsnorm(hidden) * w), hidden = T(sum of planes + residual): M <= 2, K <= 3072, at most SKINNY_GEN_MAX_PLANES planes, fp32
// output (C, or planes `partial` as above).  hipErrorInvalidValue outside these limits.
hipError_t fp8_skinny_rmsnorm_a_launch(int hidden_dtype, int b_layout, const SkinnyGenA& ag, const void* Bt, const float* Bs, float* C, int M, int N, int K,
                                       int S, float* partial, hipStream_t stream);

// The same kernel making its activations itself from the fp32 gate_up result G [M, 2K]: A = quantise_1x128(silu(G[:, :K]) *
// G[:, K:]), M <= 16, at most 32 slices of 128 per split (hipErrorInvalidValue otherwise).  partial as above.
hipError_t fp8_skinny_swiglu_a_launch(int out_kind, int b_layout, const float* G, const void* Bt, const float* Bs, void* C, float* Cs, int M, int N,
                                      int K, int S, float* partial, hipStream_t stream);

// Weights Bt[N,K] e4m3 (N % 16 == 0, K % 128 == 0) -> 2 KB blocks in MFMA operand order, or back (inverse != 0).
hipError_t fp8_preshuffle_launch(int inverse, const void* src, void* dst, int N, int K, hipStream_t stream);

// dst[N,M] = transpose(src[M,N]) for 1-byte or 4-byte elements; M % 128 == 0, N % 128 == 0.
hipError_t transpose_launch(int elem_size, const void* src, void* dst, int M, int N, hipStream_t stream);

hipError_t quant_fp8_launch(int quant_m, int transpose, const float* x, void* q, float* scale, int M, int N, hipStream_t stream);

// RMSNorm + 1x128 quantisation with transposed scales; x [M,K] of in_dtype (LLMMM_DTYPE_*), w [K] fp32, K % 128 == 0.
hipError_t rmsnorm_quant_launch(int in_dtype, const void* x, const float* w, float eps, void* q, float* scale, int M, int K,
                                hipStream_t stream);

// Peak-rate probes (probe.hip).  kind: 0 = f16, 1 = bf16 (16x16x32), 2 = fp8 e4m3 (16x16x128); operands: 32 KB of operand bits.
hipError_t probe_mfma_launch(int kind, const void* operands, float* sink, int workgroups, int iters, hipStream_t stream);
double     probe_mfma_flops(int kind, int workgroups, int iters);
hipError_t probe_stream_read_launch(const void* src, size_t bytes, float* sink, int workgroups, hipStream_t stream);

// hidden = T(sum of S planes [S][M][N] + residual); q, scale = quant_1x128_T(RMSNorm(hidden) * w).  N % 128 == 0, N <= 10240;
// residual and hidden may be the same buffer.
hipError_t planes_add_rmsnorm_quant_launch(int hidden_dtype, const float* planes, int S, const void* residual, void* hidden, const float* w,
                                           float eps, void* q, float* scale, int M, int N, hipStream_t stream);

// Compute units of the device (hipDeviceProp_t::multiProcessorCount of the device that is current on first use; 256 when
// there is none): what "a round of the chip" means to the tile heuristics and the two-shape launches.
int num_cus();

// Leaves the text in the calling thread's llmmm_last_error() and returns `code` (capi.cpp).
int report_error(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

hipError_t fill_u32_launch(uint32_t* p, uint32_t value, size_t n, hipStream_t stream);

}  // namespace llmmm
