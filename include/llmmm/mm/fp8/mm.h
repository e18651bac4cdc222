// The reference's FP8 launchers, promoted from examples/005.fp8.mm*.cu into the library with
// their signatures unchanged (device pointers, stream last, std::runtime_error on misuse):
//
//   fp8_blockwise_symmetric_quantization<QUANT_M, QUANT_N, SCALE_TRANSPOSE>(x, q, scale, M, N, stream)
//                                                                   examples/005.fp8.mm.cu:547-549
//   fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(A, A_scale_transposed, B_transposed,
//        B_scale_transposed, C, M, N, K, stream)                    examples/005.fp8.mm.cu:217-225
//   fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(A, A_scale_transposed, B_transposed,
//        B_scale_transposed, C, C_scale_transposed, M, N, K, stream)
//                                   examples/005.fp8.mm.cu:2467-2476, examples/005.fp8.mm.opt.cu:468-508
//   ...__output_bf16: the fp32 variant's result rounded to bf16 (no reference kernel).
//
// fp8_t stands for the reference's __nv_fp8_e4m3: one byte of OCP E4M3.  The launchers are templates over that
// one-byte type, so a caller holding __hip_fp8_e4m3* (the natural port of __nv_fp8_e4m3*, <hip/hip_fp8.h>), uint8_t* or
// LLMMM::fp8_t* passes its pointers as they are.  The launchers follow the
// reference's rule M % 128 == 0, N % 128 == 0, K % 128 == 0 (examples/005.fp8.mm.cu:2490-2492) and
// additionally accept 1 <= M <= 128 (decode), which the reference does not cover.  The reference
// signatures have no workspace argument, so the split-K scratch of the small-M shapes comes from a
// buffer kept per host thread and stream: the caller's, handed over once with LLMMM::set_fp8_workspace
// (then nothing here allocates or waits, as in the reference), or else one the shim allocates with
// hipMalloc on first need, grows when a later call needs more and frees when the thread ends.  Calls
// on one stream are ordered, so one buffer per stream is race-free; a call that has to allocate must
// not happen inside a stream capture -- set a workspace first, or run each shape once before capturing.
// The buffers are keyed by the stream handle: before hipStreamDestroy call LLMMM::release_fp8_workspace(stream)
// on every thread that used the shims on it, or a later stream that gets the same handle inherits the entry.
#pragma once
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdexcept>
#include <type_traits>
#include <string>
#include <unordered_map>
#include <stdint.h>

#include "../../../llmmm.h"

namespace LLMMM {

struct fp8_t {
  unsigned char bits;  // OCP FP8 E4M3 code
};
static_assert(sizeof(fp8_t) == 1, "fp8_t must be one byte");

namespace detail8 {
inline void throw_on_error(int code)
{
  if (code == LLMMM_OK) return;
  if (code == LLMMM_ERR_NOT_ALIGNED || code == LLMMM_ERR_UNSUPPORTED_TYPE) throw std::runtime_error(llmmm_error_string(code));
  throw std::runtime_error(std::string(llmmm_error_string(code)) + ": " + llmmm_last_error());
}

// Scratch for the split-K planes of a shim call, private to this host thread and stream.  Either the caller's own buffer
// (LLMMM::set_fp8_workspace: the shim then never allocates, frees or waits) or one the shim allocates on first need, grows
// when a later call needs more (hipFree waits for the device, so no kernel still uses the old one) and frees when the
// thread ends.
struct WorkspaceSlots {
  struct Slot {
    void*  ptr    = nullptr;
    size_t bytes  = 0;
    bool   caller = false;  // the caller's buffer: never freed here
  };
  std::unordered_map<hipStream_t, Slot> slots;
  // (The main thread's thread-local objects are destroyed before any static destructor or atexit handler runs, i.e.
  // while the HIP runtime is still loaded; a thread that ends later than that gets hipErrorDeinitialized, which is
  // ignored like every other error here -- the process is going away.)
  ~WorkspaceSlots()
  {
    for (auto& kv : slots)
      if (kv.second.ptr && !kv.second.caller) (void)hipFree(kv.second.ptr);
  }
};
inline WorkspaceSlots& workspace_slots()
{
  static thread_local WorkspaceSlots w;
  return w;
}

// The buffer for a call that needs `need` bytes; *have = what the library may use of it.  A caller's buffer that is
// smaller than `need` is passed on as it is: llmmm_fp8_gemm then splits K less, or not at all, where the kernel can.
// The SwiGLU output at M <= 128 (or from a 128-column tile) cannot: it needs one whole fp32 plane, M * N * 4 bytes, and
// the call throws "workspace missing or too small" without it.
inline void* cached_workspace(hipStream_t stream, size_t need, size_t* have)
{
  *have = 0;
  if (need == 0) return nullptr;
  WorkspaceSlots::Slot& s = workspace_slots().slots[stream];
  if (s.caller) {
    *have = s.bytes;
    return s.ptr;
  }
  if (s.bytes < need) {
    size_t want = size_t(1) << 20;
    while (want < need) want <<= 1;
    if (s.ptr) (void)hipFree(s.ptr);
    s.ptr = nullptr, s.bytes = 0;
    const hipError_t e = hipMalloc(&s.ptr, want);
    if (e != hipSuccess) throw std::runtime_error(std::string("workspace allocation failed: ") + hipGetErrorString(e));
    s.bytes = want;
  }
  *have = s.bytes;
  return s.ptr;
}

inline void gemm(int out_kind, const void* A, const float* As, const void* Bt, const float* Bs, void* C, float* Cs, int M, int N, int K, hipStream_t stream)
{
  const size_t need = llmmm_fp8_gemm_workspace(out_kind, M, N, K);  // 0 for shapes that run unsplit (and for invalid ones)
  size_t       have = 0;
  void*        ws   = cached_workspace(stream, need, &have);
  throw_on_error(llmmm_fp8_gemm(out_kind, A, As, Bt, Bs, C, Cs, M, N, K, ws, have, (void*)stream));
}
}  // namespace detail8

// Hands the launchers of this header a split-K workspace for calls of the calling thread on `stream`: device memory of
// `bytes` bytes, 16-byte aligned, plain scratch, which must stay valid until it is replaced or withdrawn
// (set_fp8_workspace(stream, nullptr, 0): back to a buffer of the shim's own, allocated on the next need; one it held
// before the caller's came was freed when the caller's arrived -- hipFree synchronises, so set the workspace before any capture).
// With a workspace set, the reference-signature launchers honour the reference's contract to the letter -- no
// allocation, no free, no synchronisation (src/mm/fp16/mm.cu:6-42) -- and can be captured into a HIP graph on first use.
// llmmm_fp8_gemm_workspace(out_kind, M, N, K) gives the size a shape wants; with less, K is split less or not at all.
// The reference has no such call (its kernels never split K, README.md:22).
inline void set_fp8_workspace(hipStream_t stream, void* workspace, size_t bytes)
{
  auto& slots = detail8::workspace_slots().slots;
  auto  it    = slots.find(stream);
  if (workspace && bytes) {
    if (reinterpret_cast<uintptr_t>(workspace) & 15u) throw std::runtime_error("invalid argument: workspace must be 16-byte aligned");
    if (it != slots.end() && it->second.ptr && !it->second.caller) (void)hipFree(it->second.ptr);  // the shim's own buffer gives way
    detail8::WorkspaceSlots::Slot& s = slots[stream];
    s.ptr = workspace, s.bytes = bytes, s.caller = true;
  }
  else if (it != slots.end() && it->second.caller)
    slots.erase(it);
}

// Withdraws whatever the calling thread keeps for `stream` -- the caller's buffer or the shim's own (freed: hipFree
// synchronises) -- so that the handle can be destroyed and reused.  No counterpart in the reference (no workspace there).
inline void release_fp8_workspace(hipStream_t stream)
{
  auto& slots = detail8::workspace_slots().slots;
  auto  it    = slots.find(stream);
  if (it == slots.end()) return;
  if (it->second.ptr && !it->second.caller) (void)hipFree(it->second.ptr);
  slots.erase(it);
}

// F8 below: any one-byte type that holds an OCP E4M3 code (LLMMM::fp8_t, __hip_fp8_e4m3, uint8_t).
template <typename F8>
using if_fp8_t = typename std::enable_if<sizeof(F8) == 1 && !std::is_void<F8>::value, int>::type;

template <int QUANT_M, int QUANT_N, bool SCALE_TRANSPOSE, typename F8, if_fp8_t<F8> = 0>
void fp8_blockwise_symmetric_quantization(const float* x, F8* q, float* scale, int M, int N, hipStream_t stream)
{
  static_assert(QUANT_M == 1 || QUANT_M == 128, "QUANT_M must be 1 or 128");  // examples/005.fp8.mm.cu:551-552
  static_assert(QUANT_N == 128, "QUANT_N must be 128");
  constexpr int kind = QUANT_M == 1 ? (SCALE_TRANSPOSE ? LLMMM_QUANT_1x128_T : LLMMM_QUANT_1x128)
                                    : (SCALE_TRANSPOSE ? LLMMM_QUANT_128x128_T : LLMMM_QUANT_128x128);
  detail8::throw_on_error(llmmm_quant_fp8(kind, x, q, scale, M, N, (void*)stream));
}

template <typename F8, if_fp8_t<F8> = 0>
void fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(const F8* A, const float* A_scale_transposed, const F8* B_transposed,
                                                              const float* B_scale_transposed, float* C, int M, int N, int K, hipStream_t stream)
{
  detail8::gemm(LLMMM_OUT_F32, A, A_scale_transposed, B_transposed, B_scale_transposed, C, nullptr, M, N, K, stream);
}

template <typename F8, if_fp8_t<F8> = 0>
void fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_bf16(const F8* A, const float* A_scale_transposed, const F8* B_transposed,
                                                              const float* B_scale_transposed, void* C, int M, int N, int K, hipStream_t stream)
{
  detail8::gemm(LLMMM_OUT_BF16, A, A_scale_transposed, B_transposed, B_scale_transposed, C, nullptr, M, N, K, stream);
}

template <typename F8, if_fp8_t<F8> = 0>
void fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(const F8* A, const float* A_scale_transposed, const F8* B_transposed,
                                                                      const float* B_scale_transposed, F8* C, float* C_scale_transposed, int M,
                                                                      int N, int K, hipStream_t stream)
{
  detail8::gemm(LLMMM_OUT_FP8Q, A, A_scale_transposed, B_transposed, B_scale_transposed, C, C_scale_transposed, M, N, K, stream);
}

// RMSNorm fused in front of the 1x128 activation quantiser (planned by the reference, README.md:16; no reference
// kernel): q, scale = quantise<1,128,true>(x / sqrt(mean(x^2) + eps) * weight).  T = float, __half/_Float16 or a
// 2-byte bfloat16 type; weight is fp32.
template <typename T, typename F8, if_fp8_t<F8> = 0>
void rmsnorm_fp8_blockwise_symmetric_quantization(const T* x, const float* weight, float eps, F8* q, float* scale, int M, int K,
                                                  hipStream_t stream)
{
  constexpr int dtype = sizeof(T) == 4 ? LLMMM_DTYPE_F32 : (std::is_same<T, _Float16>::value || std::is_same<T, __half>::value) ? LLMMM_DTYPE_F16 : LLMMM_DTYPE_BF16;
  static_assert(sizeof(T) == 4 || sizeof(T) == 2, "T must be float, half or bfloat16");
  detail8::throw_on_error(llmmm_rmsnorm_quant_fp8(dtype, x, weight, eps, q, scale, M, K, (void*)stream));
}

// The gate_up projection of a gated MLP with silu(gate) * up fused in front of the C quantisation -- the
// fusion the reference plans (README.md:16), no reference kernel.  B_transposed [N,K]: gate rows in
// [0, N/2), up rows in [N/2, N); C [M, N/2] e4m3, C_scale_transposed [N/256, M].
template <typename F8, if_fp8_t<F8> = 0>
void fp8_gemm_blockwise_quant_A_1x128__B_128x128__swiglu__C_1x128__output_fp8(const F8* A, const float* A_scale_transposed, const F8* B_transposed,
                                                                              const float* B_scale_transposed, F8* C, float* C_scale_transposed,
                                                                              int M, int N, int K, hipStream_t stream)
{
  detail8::gemm(LLMMM_OUT_FP8Q_SWIGLU, A, A_scale_transposed, B_transposed, B_scale_transposed, C, C_scale_transposed, M, N, K, stream);
}

// A projection back to the hidden size (O, down) with the decoder block's epilogue behind it -- residual add, the next
// RMSNorm and the 1x128 quantisation (planned by the reference, README.md:16; no reference kernel):
//   hidden_out = T(A @ B + residual);  q, q_scale = quantise<1,128,true>(rmsnorm(hidden_out) * norm_weight)
// hidden_out may be the residual buffer.  workspace: llmmm_fp8_gemm_add_rmsnorm_quant_workspace(M, N, K) bytes.
template <typename T, typename F8, if_fp8_t<F8> = 0>
void fp8_gemm_blockwise_quant_A_1x128__B_128x128__add_rmsnorm__output_fp8(const F8* A, const float* A_scale_transposed, const F8* B_transposed,
                                                                          const float* B_scale_transposed, const T* residual, T* hidden_out,
                                                                          const float* norm_weight, float eps, F8* q, float* q_scale, int M, int N,
                                                                          int K, void* workspace, size_t workspace_bytes, hipStream_t stream)
{
  constexpr int dtype = sizeof(T) == 4 ? LLMMM_DTYPE_F32 : (std::is_same<T, _Float16>::value || std::is_same<T, __half>::value) ? LLMMM_DTYPE_F16 : LLMMM_DTYPE_BF16;
  static_assert(sizeof(T) == 4 || sizeof(T) == 2, "T must be float, half or bfloat16");
  detail8::throw_on_error(llmmm_fp8_gemm_add_rmsnorm_quant(A, A_scale_transposed, B_transposed, B_scale_transposed, dtype, residual, hidden_out, norm_weight,
                                                           eps, q, q_scale, M, N, K, workspace, workspace_bytes, nullptr, (void*)stream));
}

// The QKV projection with per-head RMSNorm (q_norm / k_norm weights [128], either may be nullptr) and the rotate-half
// rotary embedding of the query and key heads fused behind it (planned by the reference, README.md:16; no reference
// kernel).  Heads of 128 columns: n_q_heads query, n_kv_heads key, n_kv_heads value; cos / sin fp32 [table_rows, 64];
// positions [M].  C: bf16 [M, N].  workspace: llmmm_fp8_gemm_qkv_rope_workspace(M, N, K) bytes (0 at prefill sizes).
template <typename F8, if_fp8_t<F8> = 0>
void fp8_gemm_blockwise_quant_A_1x128__B_128x128__qk_norm_rope__output_bf16(const F8* A, const float* A_scale_transposed,
                                                                                   const F8* B_transposed, const float* B_scale_transposed, void* C,
                                                                                   const float* q_norm_weight, const float* k_norm_weight, float eps,
                                                                                   const float* cos_table, const float* sin_table, int table_rows,
                                                                                   const int* positions, int n_q_heads, int n_kv_heads, int M, int N,
                                                                                   int K, void* workspace, size_t workspace_bytes, hipStream_t stream)
{
  detail8::throw_on_error(llmmm_fp8_gemm_qkv_rope(LLMMM_OUT_BF16, A, A_scale_transposed, B_transposed, B_scale_transposed, C, nullptr, q_norm_weight,
                                                  k_norm_weight, eps, cos_table, sin_table, table_rows, positions, n_q_heads, n_kv_heads, M, N, K,
                                                  workspace, workspace_bytes, nullptr, (void*)stream));
}

}  // namespace LLMMM
