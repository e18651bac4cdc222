// The reference's offline layout helpers (src/base/base.h:8-13) with their signatures unchanged
// (device pointers, stream last, std::runtime_error with the reference's texts on misuse):
//
//   transpose_matrix__aligned_128<T>(dst, src, M, N, stream)            src/base/base.cu:124-155
//        dst [N,M] = transpose of src [M,N]; sizeof(T) must be 1 or 4; "M or N can't be divided 128."
//   construct_m16n8k32_B_layout(dst, src_transposed, N, K, stream)      src/base/base.cu:222-271
//        the one-off permutation of the weights Bt [N,K] into the order the matrix instructions
//        consume them in; "K must be greater than 0 and divisible by 128."
//
// The second keeps its name so that a caller's weight-preparation step compiles unchanged, but the
// byte order it produces is this library's -- the 16x16x128 MFMA operand image of gfx950 (see
// llmmm.h) -- not NVIDIA's mma.m16n8k32 fragment order; the result is what the FP8 GEMM entry
// points take with cfg.b_layout = LLMMM_FP8_B_PRESHUFFLED.  construct_mfma_B_layout is the same
// function under a name that says so, restore_B_layout its exact inverse.  The reference's
// construct_m16n8k32_A_layout has no counterpart: activations are produced at run time, by the
// quantiser or by a fused epilogue, already in the row-major order the kernels read.
#pragma once
#include <hip/hip_runtime.h>
#include <stdexcept>
#include <string>

#include "../../llmmm.h"

namespace LLMMM {

namespace detail_base {
inline void throw_on_error(int code)
{
  if (code == LLMMM_OK) return;
  if (code == LLMMM_ERR_NOT_ALIGNED || code == LLMMM_ERR_UNSUPPORTED_TYPE) throw std::runtime_error(llmmm_last_error());
  throw std::runtime_error(std::string(llmmm_error_string(code)) + ": " + llmmm_last_error());
}
}  // namespace detail_base

template <typename T>
void transpose_matrix__aligned_128(T* dst, T* src, int M, int N, hipStream_t stream)
{
  static_assert(sizeof(T) == 1 || sizeof(T) == 4, "sizeof(T) must be 1 or 4");  // src/base/base.cu:151
  detail_base::throw_on_error(llmmm_transpose((int)sizeof(T), src, dst, M, N, (void*)stream));
}

template <typename FP8>
void construct_mfma_B_layout(FP8* dst, const FP8* src_transposed, int N, int K, hipStream_t stream)
{
  static_assert(sizeof(FP8) == 1, "one byte per element");
  detail_base::throw_on_error(llmmm_fp8_preshuffle_b(src_transposed, dst, N, K, (void*)stream));
}

template <typename FP8>
void construct_m16n8k32_B_layout(FP8* dst, const FP8* src_transposed, int N, int K, hipStream_t stream)
{
  construct_mfma_B_layout(dst, src_transposed, N, K, stream);
}

template <typename FP8>
void restore_B_layout(FP8* dst_transposed, const FP8* src, int N, int K, hipStream_t stream)
{
  static_assert(sizeof(FP8) == 1, "one byte per element");
  detail_base::throw_on_error(llmmm_fp8_unshuffle_b(src, dst_transposed, N, K, (void*)stream));
}

}  // namespace LLMMM
