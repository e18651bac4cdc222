// Offline data-layout helpers for gfx950: the weight pre-shuffle into MFMA operand order and the
// 128-aligned matrix transpose.
//
// The reference prepares its FP8 operands offline with construct_m16n8k32_{A,B}_layout
// (src/base/base.cu:157-273), a permutation of every 128x128 block into the register order of
// NVIDIA's mma.m16n8k32 fragments, and transposes weights with transpose_matrix__aligned_128
// (src/base/base.cu:10-155).  The permutation here plays the same role for
// v_mfma_f32_16x16x128_f8f6f4 on gfx950 and is not the reference's byte order:
//
//   Bp is a sequence of 2 KB blocks, block (rg, kb) at ((rg * K/128) + kb) * 2048, holding rows
//   16*rg .. 16*rg+15 and bytes 128*kb .. 128*kb+127 of Bt[N,K] as the LDS image the GEMM
//   kernels read their operand fragments from (the SWZ_ROWS16 placement of device_common.hip.h):
//   byte b of 16-byte chunk c of row r sits at  r*128 + ((c ^ swz(r)) << 4) + b.
//
// A kernel then fills LDS with plain linear 1 KB bursts (lane l copies bytes 16*l .. 16*l+15 of a
// half block), and a wave that streams one 16-row group through all of K reads one contiguous
// run of K/128 * 2 KB instead of sixteen rows that lie K bytes apart.
#include "device_common.hip.h"
#include "kernels.h"

namespace llmmm {

// One wavefront moves one 1 KB half block: eight rows x 128 bytes on the row-major side, one
// linear 1 KB burst on the pre-shuffled side.  Consecutive wavefronts walk along K first.
template <bool INVERSE>
__global__ void __launch_bounds__(256) fp8_preshuffle_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, int N, int K)
{
  const int  lane = threadIdx.x & 63;
  const long w    = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int  KB   = K >> 7;
  const long halves = (long)(N >> 4) * KB * 2;
  if (w >= halves) return;
  const int        half = (int)(w & 1);
  const long       blk  = w >> 1;  // = rg * KB + kb
  const int        kb   = (int)(blk % KB);
  const long       rg   = blk / KB;
  const KMajorLane p    = kmajor_lane<SWZ_ROWS16>(half, lane);
  const size_t     rowmajor = (size_t)(rg * 16 + p.row) * K + (size_t)kb * 128 + p.chunk * 16;
  const size_t     shuffled = (size_t)blk * 2048 + half * 1024 + lane * 16;
  if constexpr (INVERSE)
    *(i32x4*)(dst + rowmajor) = *(const i32x4*)(src + shuffled);
  else
    *(i32x4*)(dst + shuffled) = *(const i32x4*)(src + rowmajor);
}

hipError_t fp8_preshuffle_launch(int inverse, const void* src, void* dst, int N, int K, hipStream_t stream)
{
  const long halves = (long)(N / 16) * (K / 128) * 2;
  const dim3 grid((unsigned)((halves + 3) / 4)), block(256);
  if (inverse)
    hipLaunchKernelGGL(fp8_preshuffle_kernel<true>, grid, block, 0, stream, (const uint8_t*)src, (uint8_t*)dst, N, K);
  else
    hipLaunchKernelGGL(fp8_preshuffle_kernel<false>, grid, block, 0, stream, (const uint8_t*)src, (uint8_t*)dst, N, K);
  return hipGetLastError();
}

// dst[n*M + m] = src[m*N + n] for M and N multiples of 128 (transpose_matrix__aligned_128,
// src/base/base.cu:125-155, for 1-byte and 4-byte elements).  A workgroup transposes one block
// through LDS so that both the reads and the writes cover whole row segments.
// 4-byte elements: 64 x 64 block, row pitch 65 words (a column then touches 64 different banks).
__global__ void __launch_bounds__(256) transpose32_kernel(const uint32_t* __restrict__ src, uint32_t* __restrict__ dst, int M, int N)
{
  __shared__ uint32_t tile[64 * 65];
  const int           m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
  const int           tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
#pragma unroll
  for (int j = 0; j < 16; ++j) tile[(4 * j + ty) * 65 + tx] = src[(size_t)(m0 + 4 * j + ty) * N + n0 + tx];
  __syncthreads();
#pragma unroll
  for (int j = 0; j < 16; ++j) dst[(size_t)(n0 + 4 * j + ty) * M + m0 + tx] = tile[tx * 65 + 4 * j + ty];
}

// 1-byte elements: 128 x 128 block, four bytes per lane on the global side (32 lanes = one
// 128-byte row segment), the transposition done by the byte-granular LDS writes.
__global__ void __launch_bounds__(256) transpose8_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, int M, int N)
{
  constexpr int      PITCH = 132;
  __shared__ __attribute__((aligned(4))) uint8_t tile[128 * PITCH];  // tile[n][m]
  const int          m0 = blockIdx.y * 128, n0 = blockIdx.x * 128;
  const int          c = threadIdx.x & 31, ty = threadIdx.x >> 5;
#pragma unroll
  for (int u = 0; u < 16; ++u) {
    const int      r = 8 * u + ty;
    const uint32_t v = *(const uint32_t*)(src + (size_t)(m0 + r) * N + n0 + 4 * c);
#pragma unroll
    for (int j = 0; j < 4; ++j) tile[(4 * c + j) * PITCH + r] = (uint8_t)(v >> (8 * j));
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < 16; ++u) {
    const int r = 8 * u + ty;
    *(uint32_t*)(dst + (size_t)(n0 + r) * M + m0 + 4 * c) = *(const uint32_t*)(tile + r * PITCH + 4 * c);
  }
}

hipError_t transpose_launch(int elem_size, const void* src, void* dst, int M, int N, hipStream_t stream)
{
  if (elem_size == 1)
    hipLaunchKernelGGL(transpose8_kernel, dim3(N / 128, M / 128), dim3(256), 0, stream, (const uint8_t*)src, (uint8_t*)dst, M, N);
  else if (elem_size == 4)
    hipLaunchKernelGGL(transpose32_kernel, dim3(N / 64, M / 64), dim3(256), 0, stream, (const uint32_t*)src, (uint32_t*)dst, M, N);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

}  // namespace llmmm
