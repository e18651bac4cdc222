// Blockwise symmetric FP8 (OCP e4m3) quantiser for gfx950.
//
// Replaces fp8_blockwise_symmetric_quantization<QUANT_M, 128, SCALE_TRANSPOSE>
// (reference: examples/005.fp8.mm.cu:439-563): per block amax -> s = amax / 448.f ->
// q = e4m3(s ? x / s : 0), the code of the IEEE-correct fp32 quotient (q_pack_quotients_e4m3x4 below
// finds it without dividing wherever the rounding is not in doubt), round-to-nearest-even and
// saturation to +-448; a block of zeros gives s = 0 and q = 0.  Scale layouts:
//   QUANT_M == 1:   transposed s[(n/128)*M + m]      plain s[m*ceil(N/128) + n/128]
//   QUANT_M == 128: transposed s[(n/128)*M + m/128]  plain s[(m/128)*ceil(N/128) + n/128]
// (row stride M in both transposed forms, as written at :494 and :532).
// HBM-bound: x is read once (4 B/element) and q written once (1 B/element); the 128x128 form
// keeps its block in registers between the amax pass and the conversion.
// Rows may be ragged (any M); N must be a multiple of 4 (float4 accesses, as in the reference).
#include "device_common.hip.h"
#include "kernels.h"

namespace llmmm {

// e4m3 codes of v[0..3] / s (s != 0, |v[e]| <= 448 s up to rounding), equal bit for bit to converting the correctly
// rounded fp32 quotients -- without dividing, almost always.  An IEEE fp32 division costs about ten vector instructions
// per element and made the quantisers ALU-bound (the same element rate from bf16 and from fp32 inputs).  Instead:
// t = v * rcp(s) lies within 2^-22 (relative) of the exact quotient and of its fp32 rounding; if t (1 - 2^-21) and
// t (1 + 2^-21), which bracket both, convert to the same code, then -- the conversion being monotone -- so does the
// correctly rounded quotient.  Otherwise (a quotient within 2^-20 of a rounding boundary of the 3-bit mantissa: about
// 3 in 10^5 elements), or when s is so small or large that rcp(s) leaves the normal range, the lane divides.
// No clamp on the fast path: |t| < 448 (1 + 2^-20), and everything below 464 converts to 448.
// Non-finite values follow the reference's arithmetic: a NaN element gives 0x7F (on the fast path both brackets
// convert to the hardware's NaN code, which e4m3x4_nan_codes_to_7f turns into 0x7F); an infinite or negative scale
// (a block that holds an infinity, or nothing but NaN) fails the range test and the lane divides.
__device__ __forceinline__ uint32_t q_pack_quotients_e4m3x4(f32x4 v, float s)
{
  const float y  = __builtin_amdgcn_rcpf(s);
  const float dn = 1.0f - 0x1p-21f, up = 1.0f + 0x1p-21f;
  f32x4       t;
#pragma unroll
  for (int e = 0; e < 4; ++e) t[e] = v[e] * y;
  int lo = __builtin_amdgcn_cvt_pk_fp8_f32(t[0] * dn, t[1] * dn, 0, false);
  lo     = __builtin_amdgcn_cvt_pk_fp8_f32(t[2] * dn, t[3] * dn, lo, true);
  int hi = __builtin_amdgcn_cvt_pk_fp8_f32(t[0] * up, t[1] * up, 0, false);
  hi     = __builtin_amdgcn_cvt_pk_fp8_f32(t[2] * up, t[3] * up, hi, true);
  if (lo == hi && s >= 0x1p-100f && s <= 0x1p100f) return e4m3x4_nan_codes_to_7f((uint32_t)lo);
  return pack_e4m3x4_sat(v[0] / s, v[1] / s, v[2] / s, v[3] / s);
}

// The reference starts its block maximum from (float)INT_MIN (examples/005.fp8.mm.cu:456) and its comparison never
// takes a NaN, so a block that holds nothing but NaN keeps that seed: scale INT_MIN / 448, codes 0x7F.  fmaxf drops
// NaN operands the same way.
constexpr float QUANT_AMAX_SEED = -2147483648.f;

__device__ __forceinline__ float amax4(float m, f32x4 v)
{
  return fmaxf(fmaxf(m, fmaxf(__builtin_fabsf(v[0]), __builtin_fabsf(v[1]))), fmaxf(__builtin_fabsf(v[2]), __builtin_fabsf(v[3])));
}

// 1 x 128 blocks.  Half a wavefront (32 lanes x float4) owns one block; a workgroup of 256
// threads covers 8 consecutive rows of one 128-column group per step and strides over rows.
template <bool TRANSPOSE>
__global__ void __launch_bounds__(256) quant_1x128_kernel(const float* __restrict__ x, uint8_t* __restrict__ q,
                                                          float* __restrict__ scale, int M, int N, int rows_per_wg)
{
  const int tid   = threadIdx.x;
  const int sub   = tid >> 5;        // which of the 8 rows of a step
  const int l32   = tid & 31;
  const int nb    = blockIdx.x;      // 128-column group
  const int n     = nb * 128 + l32 * 4;
  const int nbn   = (N + 127) >> 7;
  const int mbeg  = blockIdx.y * rows_per_wg;
  const int mend  = min(M, mbeg + rows_per_wg);
  const bool live = n < N;
  // four rows per thread and pass: their loads go out together, before the first row's cross-lane amax and divisions
  constexpr int U = 4;
  for (int m0 = mbeg + sub; m0 < mend; m0 += 8 * U) {
    f32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int m = m0 + 8 * u;
      v[u]        = f32x4{0.f, 0.f, 0.f, 0.f};
      if (live && m < mend) v[u] = __builtin_nontemporal_load((const f32x4*)(x + (size_t)m * N + n));
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int m = m0 + 8 * u;
      if (m >= mend) break;  // uniform over the half-wavefront that shares the row
      float a = QUANT_AMAX_SEED;
      if (live) a = amax4(a, v[u]);
      a       = wave_xor_max(a, 1);
      a       = wave_xor_max(a, 2);
      a       = wave_xor_max(a, 4);
      a       = wave_xor_max(a, 8);
      a       = wave_xor_max(a, 16);
      const float s = a / 448.f;
      uint32_t    c = 0;
      if (s != 0.f) c = q_pack_quotients_e4m3x4(v[u], s);
      if (live) *(uint32_t*)(q + (size_t)m * N + n) = c;
      if (l32 == 0) {
        if (TRANSPOSE)
          scale[(size_t)nb * M + m] = s;
        else
          scale[(size_t)m * nbn + nb] = s;
      }
    }
  }
}

// 128 x 128 blocks: one workgroup of 256 threads per block, 16 float4 per thread in registers.
template <bool TRANSPOSE>
__global__ void __launch_bounds__(256) quant_128x128_kernel(const float* __restrict__ x, uint8_t* __restrict__ q,
                                                            float* __restrict__ scale, int M, int N)
{
  __shared__ float wmax[4];
  const int tid  = threadIdx.x;
  const int l32  = tid & 31;
  const int sub  = tid >> 5;
  const int nb   = blockIdx.x;
  const int mb   = blockIdx.y;
  const int n    = nb * 128 + l32 * 4;
  const int nbn  = (N + 127) >> 7;
  const bool live = n < N;
  f32x4     v[16];
  float     a = QUANT_AMAX_SEED;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int m = mb * 128 + r * 8 + sub;
    v[r]        = f32x4{0.f, 0.f, 0.f, 0.f};
    if (live && m < M) {
      v[r] = __builtin_nontemporal_load((const f32x4*)(x + (size_t)m * N + n));
      a    = amax4(a, v[r]);
    }
  }
  a = wave_xor_max(a, 1);
  a = wave_xor_max(a, 2);
  a = wave_xor_max(a, 4);
  a = wave_xor_max(a, 8);
  a = wave_xor_max(a, 16);
  a = wave_xor_max(a, 32);
  if ((tid & 63) == 0) wmax[tid >> 6] = a;
  __syncthreads();
  a             = fmaxf(fmaxf(wmax[0], wmax[1]), fmaxf(wmax[2], wmax[3]));
  const float s = a / 448.f;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int m = mb * 128 + r * 8 + sub;
    uint32_t  c = 0;
    if (s != 0.f) c = q_pack_quotients_e4m3x4(v[r], s);
    if (live && m < M) *(uint32_t*)(q + (size_t)m * N + n) = c;
  }
  if (tid == 0) {
    if (TRANSPOSE)
      scale[(size_t)nb * M + mb] = s;
    else
      scale[(size_t)mb * nbn + nb] = s;
  }
}

// RMSNorm fused in front of the 1 x 128 activation quantiser (the "RMSNorm + fp8 dynamic quant" fusion the reference
// plans, README.md:16; no reference kernel):
//   y[m,k] = (x[m,k] * r) * w[k],  r = 1 / sqrt(sum_k x[m,k]^2 / K + eps),  then q, s = quant_1x128(y), scales transposed.
// The sum of squares has one fixed order, which the CPU oracle restates, so that results are bit-exact and do not
// depend on which of the two kernels below runs: the row is cut into chunks of four elements; chunk c belongs to
// virtual lane c % 256, which accumulates its chunks in ascending order with one fused multiply-add per element;
// the 256 partial sums are combined per group of 64 by an xor butterfly (32, 16, .. 1) and the four group sums as
// (G0 + G1) + (G2 + G3).  A second pass normalises and quantises: a 128-column group is 32 consecutive chunks =
// half a wavefront in either kernel, so its amax needs five cross-lane steps.  HBM traffic: x once, q once.
//   * rmsnorm_quant_row_kernel:   one 256-thread workgroup per row (a thread is a virtual lane), the row held in
//     registers: K <= 10240.  Measured at K = 2560 against a wavefront per row: 3.2 instead of 8.2 us at M = 16 (a
//     single wavefront works through the row's 40 divisions per lane on its own), 6.9 instead of 9.4 us at M = 2048.
//   * rmsnorm_quant_1x128_kernel: one wavefront per row (a lane plays four virtual lanes), the row read twice:
//     longer rows.
// One chunk (4 elements) per lane of row m: normalise, take the amax of the 128-column group (the 32 chunks of this
// half of the wavefront), quantise, store codes and the group's scale.
__device__ __forceinline__ void rmsnorm_quant_chunk(f32x4 v, float r, const float* __restrict__ w, uint8_t* __restrict__ q,
                                                    float* __restrict__ scale, int m, int M, int K, int c, int chunks, int lane)
{
  const bool live = c < chunks;
  f32x4      y    = {0.f, 0.f, 0.f, 0.f};
  if (live) {
    const f32x4 wv = *(const f32x4*)(w + 4 * c);
#pragma unroll
    for (int e = 0; e < 4; ++e) y[e] = (v[e] * r) * wv[e];
  }
  float a = amax4(0.f, y);
  a       = wave_xor_max(a, 1);
  a       = wave_xor_max(a, 2);
  a       = wave_xor_max(a, 4);
  a       = wave_xor_max(a, 8);
  a       = wave_xor_max(a, 16);
  const float s  = a / 448.f;
  uint32_t    cd = 0;
  if (s != 0.f) cd = q_pack_quotients_e4m3x4(y, s);
  if (live) {
    *(uint32_t*)(q + (size_t)m * K + 4 * c) = cd;
    if ((lane & 31) == 0) scale[(size_t)(c >> 5) * M + m] = s;
  }
}

// One wavefront per row, any K: the row is read twice (the second time from the L2).  A lane plays the four
// virtual lanes lane, lane + 64, lane + 128, lane + 192.
template <typename IN_T>
__global__ void __launch_bounds__(256) rmsnorm_quant_1x128_kernel(const IN_T* __restrict__ x, const float* __restrict__ w, float eps,
                                                                  uint8_t* __restrict__ q, float* __restrict__ scale, int M, int K)
{
  const int lane = threadIdx.x & 63;
  const int m    = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (m >= M) return;  // whole wavefronts leave: no barrier below
  const IN_T* xr      = x + (size_t)m * K;
  const int   chunks  = K >> 2;
  float       part[4] = {0.f, 0.f, 0.f, 0.f};
  for (int c0 = 0; c0 < chunks; c0 += 256) {
#pragma unroll
    for (int gidx = 0; gidx < 4; ++gidx) {
      const int c = c0 + 64 * gidx + lane;
      if (c < chunks) {
        const f32x4 v = load_row4<IN_T>(xr + 4 * c);
#pragma unroll
        for (int e = 0; e < 4; ++e) part[gidx] = __builtin_fmaf(v[e], v[e], part[gidx]);
      }
    }
  }
#pragma unroll
  for (int step = 32; step >= 1; step >>= 1)
#pragma unroll
    for (int gidx = 0; gidx < 4; ++gidx) part[gidx] = part[gidx] + wave_xor_get(part[gidx], step);
  const float acc = (part[0] + part[1]) + (part[2] + part[3]);
  const float ms  = acc / (float)K;
  const float r   = 1.0f / __builtin_sqrtf(ms + eps);
  // second pass: lanes beyond the row's end still take part in the cross-lane maxima (with zeros)
  for (int c0 = 0; c0 < chunks; c0 += 64) {
    const int c = c0 + lane;
    f32x4     v = {0.f, 0.f, 0.f, 0.f};
    if (c < chunks) v = load_row4<IN_T>(xr + 4 * c);
    rmsnorm_quant_chunk(v, r, w, q, scale, m, M, K, c, chunks, lane);
  }
}

// One workgroup of 256 threads per row: thread t is virtual lane t and owns chunks t, t + 256, ...  NI = chunks per
// thread held in registers (K <= 1024 * NI).
template <typename IN_T, int NI>
__global__ void __launch_bounds__(256) rmsnorm_quant_row_kernel(const IN_T* __restrict__ x, const float* __restrict__ w, float eps,
                                                                uint8_t* __restrict__ q, float* __restrict__ scale, int M, int K)
{
  __shared__ float group_sum[4];
  const int   t      = threadIdx.x;
  const int   m      = blockIdx.x;
  const IN_T* xr     = x + (size_t)m * K;
  const int   chunks = K >> 2;
  f32x4       held[NI], wv[NI];
  float       acc = 0.f;
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int c = t + 256 * i;
    held[i]     = f32x4{0.f, 0.f, 0.f, 0.f};
    wv[i]       = f32x4{0.f, 0.f, 0.f, 0.f};
    if (c < chunks) {
      held[i] = load_row4<IN_T>(xr + 4 * c);
      wv[i]   = *(const f32x4*)(w + 4 * c);
    }
  }
#pragma unroll
  for (int i = 0; i < NI; ++i)
    if (t + 256 * i < chunks) {
#pragma unroll
      for (int e = 0; e < 4; ++e) acc = __builtin_fmaf(held[i][e], held[i][e], acc);
    }
#pragma unroll
  for (int step = 32; step >= 1; step >>= 1) acc = acc + wave_xor_get(acc, step);
  if ((t & 63) == 0) group_sum[t >> 6] = acc;
  __syncthreads();
  const float total = (group_sum[0] + group_sum[1]) + (group_sum[2] + group_sum[3]);
  const float ms    = total / (float)K;
  const float r     = 1.0f / __builtin_sqrtf(ms + eps);
  float       amax[NI];
#pragma unroll
  for (int i = 0; i < NI; ++i) {
#pragma unroll
    for (int e = 0; e < 4; ++e) held[i][e] = (held[i][e] * r) * wv[i][e];  // zeros beyond the row's end
    amax[i] = amax4(0.f, held[i]);
  }
#pragma unroll
  for (int step = 1; step <= 16; step <<= 1)
#pragma unroll
    for (int i = 0; i < NI; ++i) amax[i] = wave_xor_max(amax[i], step);
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int   c  = t + 256 * i;
    const float sc = amax[i] / 448.f;
    uint32_t    cd = 0;
    if (sc != 0.f) cd = q_pack_quotients_e4m3x4(held[i], sc);
    if (c < chunks) {
      *(uint32_t*)(q + (size_t)m * K + 4 * c) = cd;
      if ((t & 31) == 0) scale[(size_t)(c >> 5) * M + m] = sc;
    }
  }
}

// The decoder-block epilogue behind a projection back to the hidden size (O, down), in one kernel behind the GEMM's
// fp32 planes:  h = (plane 0 + plane 1 + ... in split order) + residual,  hidden = T(h) (the new residual stream),
// y = RMSNorm(float(hidden)) * weight,  q, s = quant_1x128(y) -- the A operand of the next projection.  It takes the
// place of the split-K reduce kernel and of the separate RMSNorm + quantiser launch; the norm sees the rounded hidden
// state, exactly what a separate kernel reading `hidden` would see, and follows the same fixed summation order
// (rmsnorm_quant_row_kernel), so its codes and scales are those of the unfused sequence, bit for bit.
// One 256-thread workgroup per row; N <= 1024 * NI columns.
template <typename T, int NI>
__global__ void __launch_bounds__(256) planes_add_rmsnorm_quant_kernel(const float* __restrict__ planes, int S, const T* residual, T* hidden,
                                                                       const float* __restrict__ w, float eps, uint8_t* __restrict__ q,
                                                                       float* __restrict__ scale, int M, int N)
{
  __shared__ float group_sum[4];
  const int    t      = threadIdx.x;
  const int    m      = blockIdx.x;
  const int    chunks = N >> 2;
  const size_t plane  = (size_t)M * N;
  f32x4        held[NI], wv[NI];
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    held[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    wv[i]   = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  // Everything that does not depend on the planes is requested first; then the planes, W of them in flight per chunk,
  // summed in split order (0 + p0 + p1 + ...: the order of the split-K reduce kernel).  Threads past the end of the
  // row load its last chunk and drop it.
  f32x4 rv[NI];
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int c = min(t + 256 * i, chunks - 1);
    rv[i]       = load_row4<T>(residual + (size_t)m * N + 4 * c);
    wv[i]       = *(const f32x4*)(w + 4 * c);
  }
  constexpr int W = NI <= 3 ? 8 : 2;
  for (int s0 = 0; s0 < S; s0 += W) {
    f32x4 p[W][NI];
#pragma unroll
    for (int u = 0; u < W; ++u)
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int c = min(t + 256 * i, chunks - 1);
        p[u][i]     = __builtin_nontemporal_load((const f32x4*)(planes + (size_t)min(s0 + u, S - 1) * plane + (size_t)m * N + 4 * c));
      }
#pragma unroll
    for (int u = 0; u < W; ++u)
      if (s0 + u < S) {
#pragma unroll
        for (int i = 0; i < NI; ++i) held[i] += p[u][i];
      }
  }
  float acc = 0.f;
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int c = t + 256 * i;
    if (c < chunks) {
      const f32x4 h = held[i] + rv[i];
      store_row4<T>(hidden + (size_t)m * N + 4 * c, h);
      // the norm reads the hidden state as stored (rounded to T)
      if constexpr (sizeof(T) == 4)
        held[i] = h;
      else {
#pragma unroll
        for (int e = 0; e < 4; ++e) held[i][e] = (float)(T)h[e];
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) acc = __builtin_fmaf(held[i][e], held[i][e], acc);
    }
    else
      held[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
#pragma unroll
  for (int step = 32; step >= 1; step >>= 1) acc = acc + wave_xor_get(acc, step);
  if ((t & 63) == 0) group_sum[t >> 6] = acc;
  __syncthreads();
  const float total = (group_sum[0] + group_sum[1]) + (group_sum[2] + group_sum[3]);
  const float ms    = total / (float)N;
  const float r     = 1.0f / __builtin_sqrtf(ms + eps);
  float       amax[NI];
#pragma unroll
  for (int i = 0; i < NI; ++i) {
#pragma unroll
    for (int e = 0; e < 4; ++e) held[i][e] = (held[i][e] * r) * wv[i][e];
    amax[i] = amax4(0.f, held[i]);
  }
#pragma unroll
  for (int step = 1; step <= 16; step <<= 1)
#pragma unroll
    for (int i = 0; i < NI; ++i) amax[i] = wave_xor_max(amax[i], step);
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int   c  = t + 256 * i;
    const float sc = amax[i] / 448.f;
    uint32_t    cd = 0;
    if (sc != 0.f) cd = q_pack_quotients_e4m3x4(held[i], sc);
    if (c < chunks) {
      *(uint32_t*)(q + (size_t)m * N + 4 * c) = cd;
      if ((t & 31) == 0) scale[(size_t)(c >> 5) * M + m] = sc;
    }
  }
}

hipError_t planes_add_rmsnorm_quant_launch(int hidden_dtype, const float* planes, int S, const void* residual, void* hidden, const float* w,
                                           float eps, void* q, float* scale, int M, int N, hipStream_t stream)
{
#define LLMMM_GO(T)                                                                                                                        \
  {                                                                                                                                        \
    if (N <= 1024 * 3)                                                                                                                     \
      hipLaunchKernelGGL((planes_add_rmsnorm_quant_kernel<T, 3>), dim3(M), dim3(256), 0, stream, planes, S, (const T*)residual, (T*)hidden, \
                         w, eps, (uint8_t*)q, scale, M, N);                                                                                \
    else                                                                                                                                   \
      hipLaunchKernelGGL((planes_add_rmsnorm_quant_kernel<T, 10>), dim3(M), dim3(256), 0, stream, planes, S, (const T*)residual,           \
                         (T*)hidden, w, eps, (uint8_t*)q, scale, M, N);                                                                    \
  }
  if (N > 1024 * 10) return hipErrorInvalidValue;
  switch (hidden_dtype) {
    case LLMMM_DTYPE_F16: LLMMM_GO(_Float16) break;
    case LLMMM_DTYPE_BF16: LLMMM_GO(__bf16) break;
    case LLMMM_DTYPE_F32: LLMMM_GO(float) break;
    default: return hipErrorInvalidValue;
  }
#undef LLMMM_GO
  return hipGetLastError();
}

hipError_t rmsnorm_quant_launch(int in_dtype, const void* x, const float* w, float eps, void* q, float* scale, int M, int K,
                                hipStream_t stream)
{
  const dim3 grid((M + 3) / 4), block(256);
#define LLMMM_NORM_GO(T)                                                                                                               \
  {                                                                                                                                    \
    if (K <= 1024 * 3)                                                                                                                 \
      hipLaunchKernelGGL((rmsnorm_quant_row_kernel<T, 3>), dim3(M), block, 0, stream, (const T*)x, w, eps, (uint8_t*)q, scale, M, K);   \
    else if (K <= 1024 * 10)                                                                                                           \
      hipLaunchKernelGGL((rmsnorm_quant_row_kernel<T, 10>), dim3(M), block, 0, stream, (const T*)x, w, eps, (uint8_t*)q, scale, M, K);  \
    else                                                                                                                               \
      hipLaunchKernelGGL((rmsnorm_quant_1x128_kernel<T>), grid, block, 0, stream, (const T*)x, w, eps, (uint8_t*)q, scale, M, K);       \
  }
  switch (in_dtype) {
    case LLMMM_DTYPE_F16: LLMMM_NORM_GO(_Float16) break;
    case LLMMM_DTYPE_BF16: LLMMM_NORM_GO(__bf16) break;
    case LLMMM_DTYPE_F32: LLMMM_NORM_GO(float) break;
    default: return hipErrorInvalidValue;
  }
#undef LLMMM_NORM_GO
  return hipGetLastError();
}

__global__ void fill_u32_kernel(uint32_t* p, uint32_t value, size_t n)
{
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = value;
}

hipError_t fill_u32_launch(uint32_t* p, uint32_t value, size_t n, hipStream_t stream)
{
  hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, p, value, n);
  return hipGetLastError();
}

hipError_t quant_fp8_launch(int quant_m, int transpose, const float* x, void* q, float* scale, int M, int N, hipStream_t stream)
{
  const int nbn = (N + 127) / 128;
  if (quant_m == 1) {
    // enough workgroups to fill the chip, at least 8 rows each
    int rows_per_wg = 64;
    while (rows_per_wg > 8 && (long)nbn * ((M + rows_per_wg - 1) / rows_per_wg) < 2048) rows_per_wg >>= 1;
    dim3 grid(nbn, (M + rows_per_wg - 1) / rows_per_wg);
    if (transpose)
      hipLaunchKernelGGL(quant_1x128_kernel<true>, grid, dim3(256), 0, stream, x, (uint8_t*)q, scale, M, N, rows_per_wg);
    else
      hipLaunchKernelGGL(quant_1x128_kernel<false>, grid, dim3(256), 0, stream, x, (uint8_t*)q, scale, M, N, rows_per_wg);
  }
  else {
    dim3 grid(nbn, (M + 127) / 128);
    if (transpose)
      hipLaunchKernelGGL(quant_128x128_kernel<true>, grid, dim3(256), 0, stream, x, (uint8_t*)q, scale, M, N);
    else
      hipLaunchKernelGGL(quant_128x128_kernel<false>, grid, dim3(256), 0, stream, x, (uint8_t*)q, scale, M, N);
  }
  return hipGetLastError();
}

}  // namespace llmmm
