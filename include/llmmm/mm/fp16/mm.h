// Drop-in for the reference's src/mm/fp16/mm.h:9-10 on MI355X:
//
//   namespace LLMMM { template<typename T> void fp16_mm(const T* A, const T* B, T* C,
//                                                       int M, int N, int K, hipStream_t stream); }
//
// T is _Float16 / __half (the reference's `half`) or __bf16 / hip_bfloat16 / __hip_bfloat16 (its
// `__nv_bfloat16`).  Same contract as src/mm/fp16/mm.cu:6-42: device pointers, row-major A[M,K],
// B[K,N], C[M,N], asynchronous on `stream`, no allocation, no synchronisation, and
// std::runtime_error("T is not supported.") / ("M or N or K are not aligned.") unless
// M % 256 == 0, N % 256 == 0, K % 16 == 0.  Header-only shim over the C ABI (llmmm.h).
#pragma once
#include <hip/hip_runtime.h>
#include <stdexcept>
#include <type_traits>

#include "../../../llmmm.h"

namespace LLMMM {

namespace detail {
template <typename T>
struct fp16_dtype {
  static constexpr int value = -1;
};
template <>
struct fp16_dtype<_Float16> {
  static constexpr int value = LLMMM_DTYPE_F16;
};
template <>
struct fp16_dtype<__bf16> {
  static constexpr int value = LLMMM_DTYPE_BF16;
};
#if defined(HIP_INCLUDE_HIP_HIP_FP16_H) || defined(__HIP_FP16_H__) || defined(HIP_INCLUDE_HIP_AMD_DETAIL_HIP_FP16_H)
template <>
struct fp16_dtype<__half> {
  static constexpr int value = LLMMM_DTYPE_F16;
};
#endif
#if defined(_HIP_INCLUDE_HIP_AMD_DETAIL_HIP_BF16_H_)
template <>
struct fp16_dtype<__hip_bfloat16> {
  static constexpr int value = LLMMM_DTYPE_BF16;
};
#endif

inline void throw_on_error(int code)
{
  if (code == LLMMM_OK) return;
  if (code == LLMMM_ERR_NOT_ALIGNED || code == LLMMM_ERR_UNSUPPORTED_TYPE) throw std::runtime_error(llmmm_error_string(code));
  throw std::runtime_error(std::string(llmmm_error_string(code)) + ": " + llmmm_last_error());
}
}  // namespace detail

template <typename T>
void fp16_mm(const T* A, const T* B, T* C, int M, int N, int K, hipStream_t stream)
{
  if (detail::fp16_dtype<T>::value < 0) throw std::runtime_error("T is not supported.");
  // the reference's tiling rule (BLOCK 256 x 256, LOOP_K 16: src/mm/fp16/mm.cu:9-21)
  if (!(M % 256 == 0 && N % 256 == 0 && K % 16 == 0)) throw std::runtime_error("M or N or K are not aligned.");
  detail::throw_on_error(llmmm_fp16_gemm(detail::fp16_dtype<T>::value, A, B, C, M, N, K, LLMMM_B_ROW_MAJOR, (void*)stream));
}

}  // namespace LLMMM
