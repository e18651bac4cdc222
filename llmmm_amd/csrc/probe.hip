// Peak-rate microbenchmarks for gfx950: what the matrix pipes and the HBM deliver on this very part, next to the
// nominal figures a roofline is priced against.  Counterpart of the reference's register-only MMA loop
// test_fp8_peak_work (examples/005.fp8.test.cu:19-71), which it uses to find the tensor-core rate of its GPU.
//
//  * mfma_peak_kernel: 8 waves per workgroup, each issuing v_mfma back to back on eight independent accumulator
//    fragments (enough to cover the instruction's latency) from operands held in registers -- no LDS, no memory
//    traffic.  The operand bits come from a caller-supplied buffer: the rate this part sustains depends on them
//    (zeros run at the full clock; random data draws more power and the clock drops), and a GEMM's roofline
//    on real data is the random-operand figure.
//  * stream_read_kernel: every byte of a buffer read once with non-temporal 16-byte loads, nothing written.
#include "device_common.hip.h"
#include "kernels.h"

namespace llmmm {

enum { PROBE_F16 = 0, PROBE_BF16 = 1, PROBE_FP8 = 2 };

template <int KIND>
__global__ void __launch_bounds__(512) mfma_peak_kernel(const i32x8* __restrict__ operands, float* __restrict__ sink, int iters)
{
  // two operand fragments per lane, different for every lane of the workgroup
  i32x8 a = operands[threadIdx.x], b = operands[512 + threadIdx.x];
  f32x4 acc[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) acc[u] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < iters; ++it) {
    asm volatile("" : "+v"(a), "+v"(b));  // opaque: the loop body may not be folded
    if constexpr (KIND == PROBE_FP8) {
#pragma unroll
      for (int u = 0; u < 8; ++u) acc[u] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, acc[u], 0, 0, 0, 0, 0, 0);
    }
    else {
      union {
        i32x8  w;
        f16x8  h[2];
        bf16x8 bf[2];
      } ua, ub;
      ua.w = a;
      ub.w = b;
#pragma unroll
      for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          if constexpr (KIND == PROBE_F16)
            acc[u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ua.h[half], ub.h[half], acc[u], 0, 0, 0);
          else
            acc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ua.bf[half], ub.bf[half], acc[u], 0, 0, 0);
        }
    }
  }
  float s = 0.f;
#pragma unroll
  for (int u = 0; u < 8; ++u) s += acc[u][0] + acc[u][1] + acc[u][2] + acc[u][3];
  if (s == 12345.678f) sink[0] = s;  // never true for the operand patterns in use; keeps the loop alive
}

// FLOP of one launch of mfma_peak_kernel: workgroups x 8 waves x iters x MFMAs per iteration x 2 * 16 * 16 * k.
double probe_mfma_flops(int kind, int workgroups, int iters)
{
  const double per_iter = kind == PROBE_FP8 ? 8.0 * (2.0 * 16 * 16 * 128) : 16.0 * (2.0 * 16 * 16 * 32);
  return (double)workgroups * 8.0 * (double)iters * per_iter;
}

hipError_t probe_mfma_launch(int kind, const void* operands, float* sink, int workgroups, int iters, hipStream_t stream)
{
  const dim3 grid(workgroups), block(512);
  switch (kind) {
    case PROBE_F16: hipLaunchKernelGGL(mfma_peak_kernel<PROBE_F16>, grid, block, 0, stream, (const i32x8*)operands, sink, iters); break;
    case PROBE_BF16: hipLaunchKernelGGL(mfma_peak_kernel<PROBE_BF16>, grid, block, 0, stream, (const i32x8*)operands, sink, iters); break;
    case PROBE_FP8: hipLaunchKernelGGL(mfma_peak_kernel<PROBE_FP8>, grid, block, 0, stream, (const i32x8*)operands, sink, iters); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

__global__ void __launch_bounds__(512) stream_read_kernel(const i32x4* __restrict__ src, float* __restrict__ sink, size_t vecs)
{
  // workgroup w reads the contiguous range [w * per, (w + 1) * per) of 16-byte vectors, eight loads in flight per lane
  const size_t per  = (vecs + gridDim.x - 1) / gridDim.x;
  const size_t beg  = (size_t)blockIdx.x * per;
  const size_t end  = beg + per < vecs ? beg + per : vecs;
  i32x4        acc  = {0, 0, 0, 0};
  for (size_t i = beg + threadIdx.x; i < end; i += 8 * 512) {
    i32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const size_t j = i + (size_t)u * 512;
      v[u]           = __builtin_nontemporal_load(src + (j < end ? j : end - 1));
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) acc ^= v[u];
  }
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x5eed5eed) sink[0] = 1.f;  // practically never; keeps the loads alive
}

hipError_t probe_stream_read_launch(const void* src, size_t bytes, float* sink, int workgroups, hipStream_t stream)
{
  hipLaunchKernelGGL(stream_read_kernel, dim3(workgroups), dim3(512), 0, stream, (const i32x4*)src, sink, bytes / 16);
  return hipGetLastError();
}

}  // namespace llmmm
