// Small-M (decode) FP8 blockwise GEMM for gfx950: weight streaming with deterministic split-K.
//
// Same arithmetic and layouts as fp8_gemm.hip (reference math: examples/005.fp8.mm.cu:885-902,
// fused epilogue examples/005.fp8.mm.opt.cu:401-462) for M <= 64 rows, a range the reference
// does not cover (its launchers require M % 128 == 0, examples/005.fp8.mm.opt.cu:492; split-K
// is listed as unfinished in README.md:22).
//
//  * HBM-bound: every byte of Bt[N,K] is read exactly once, straight from global memory into
//    the MFMA operand registers (no LDS).  One wavefront owns 16 weight rows; per 128-K slice
//    lane (g = lane/16, i = lane%16) loads bytes [16g,16g+16) and [64+16g,64+16g+16) of row i,
//    so each of the two load instructions touches 64 contiguous bytes per row.  The activation
//    operand uses the same k -> register mapping, which is all the MFMA needs.
//  * A workgroup = 8 waves = one 128-column quantisation group; grid.y = number of K splits.
//  * split-K: each split writes its fp32 partial tile to the workspace; the workgroup that
//    arrives last at the group's counter adds the partials in split order 0..S-1 (fixed order,
//    independent of arrival) and runs the epilogue.  Nobody waits on anybody.
#include "device_common.hip.h"
#include "kernels.h"

namespace llmmm {

enum { SK_OUT_F32 = 0, SK_OUT_BF16 = 1, SK_OUT_FP8Q = 2 };

__device__ __forceinline__ uint32_t sk_pack_e4m3x4(float a, float b, float c, float d)
{
  a     = __builtin_amdgcn_fmed3f(a, -448.f, 448.f);
  b     = __builtin_amdgcn_fmed3f(b, -448.f, 448.f);
  c     = __builtin_amdgcn_fmed3f(c, -448.f, 448.f);
  d     = __builtin_amdgcn_fmed3f(d, -448.f, 448.f);
  int v = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
  v     = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, v, true);
  return (uint32_t)v;
}

template <int MBLK, int OUT>
__global__ void __launch_bounds__(512)
fp8_skinny_kernel(const uint8_t* __restrict__ A, const float* __restrict__ As, const uint8_t* __restrict__ Bt,
                  const float* __restrict__ Bs, void* __restrict__ Cv, float* __restrict__ Cs, int M, int N, int K, int S,
                  float* __restrict__ partial, unsigned* __restrict__ counters)
{
  constexpr int UNROLL = 4;
  __shared__ float    wave_amax[8][MBLK][16];
  __shared__ unsigned is_last;

  const int tid  = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g    = lane >> 4;
  const int i    = lane & 15;
  const int ng   = blockIdx.x;
  const int sp   = blockIdx.y;
  const int KB   = K >> 7;
  const int kb0  = sp * KB / S;  // KB * S is small: 32-bit arithmetic (a 64-bit divide costs hundreds of scalar ops)
  const int kb1  = (sp + 1) * KB / S;

  const int      nrow = ng * 128 + wave * 16 + i;
  const uint8_t* wp   = Bt + (size_t)nrow * K + 16 * g;
  const float*   bsp  = Bs + (size_t)ng * KB;

  f32x4 acc[MBLK];
#pragma unroll
  for (int mb = 0; mb < MBLK; ++mb) acc[mb] = f32x4{0.f, 0.f, 0.f, 0.f};

  for (int kb = kb0; kb < kb1; kb += UNROLL) {
    i32x4 w0[UNROLL], w1[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      if (kb + u < kb1) {
        w0[u] = __builtin_nontemporal_load((const i32x4*)(wp + (size_t)(kb + u) * 128));
        w1[u] = __builtin_nontemporal_load((const i32x4*)(wp + (size_t)(kb + u) * 128 + 64));
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      if (kb + u < kb1) {
        const float sb = bsp[kb + u];
        union {
          i32x4 h[2];
          i32x8 v;
        } wf;
        wf.h[0] = w0[u];
        wf.h[1] = w1[u];
#pragma unroll
        for (int mb = 0; mb < MBLK; ++mb) {
          const int m = mb * 16 + i;
          union {
            i32x4 h[2];
            i32x8 v;
          } af;
          float s = 0.f;
          if (m < M) {
            const uint8_t* ap = A + (size_t)m * K + (size_t)(kb + u) * 128 + 16 * g;
            af.h[0]           = *(const i32x4*)ap;
            af.h[1]           = *(const i32x4*)(ap + 64);
            s                 = As[(size_t)(kb + u) * M + m] * sb;
          }
          else {
            af.h[0] = i32x4{0, 0, 0, 0};
            af.h[1] = i32x4{0, 0, 0, 0};
          }
          const f32x4 z = {0.f, 0.f, 0.f, 0.f};
          const f32x4 p = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf.v, af.v, z, 0, 0, 0, 0, 0, 0);
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[mb][r] = __builtin_fmaf(p[r], s, acc[mb][r]);
        }
      }
    }
  }

  // lane (g, i): row m = mb*16 + i, columns ncol .. ncol+3
  const int ncol = ng * 128 + wave * 16 + 4 * g;

  if (S > 1) {
    // Partials travel through device-coherent (agent-scope, relaxed) stores and loads, which
    // write through / read past the per-XCD L2.  That makes full release/acquire fences
    // unnecessary: a fence at agent scope writes back and invalidates the whole L2 of the XCD,
    // which costs far more than this kernel's entire run.
#pragma unroll
    for (int mb = 0; mb < MBLK; ++mb) {
      const int m = mb * 16 + i;
      if (m < M) {
        float* dst = partial + ((size_t)sp * M + m) * N + ncol;
#pragma unroll
        for (int r = 0; r < 4; ++r) __hip_atomic_store(dst + r, acc[mb][r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0): this wave's partial stores are acknowledged
    __syncthreads();
    if (tid == 0) {
      const unsigned old = __hip_atomic_fetch_add(counters + ng, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      is_last            = (old == (unsigned)(S - 1));
    }
    __syncthreads();
    if (!is_last) return;
#pragma unroll
    for (int mb = 0; mb < MBLK; ++mb) {
      const int m = mb * 16 + i;
      f32x4     t = {0.f, 0.f, 0.f, 0.f};
      if (m < M) {
        for (int s = 0; s < S; ++s) {  // fixed order 0..S-1, whoever arrived last
          const float* src = partial + ((size_t)s * M + m) * N + ncol;
#pragma unroll
          for (int r = 0; r < 4; ++r) t[r] += __hip_atomic_load(src + r, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
      acc[mb] = t;
    }
    if (tid == 0) __hip_atomic_store(counters + ng, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
  }

  if constexpr (OUT == SK_OUT_F32) {
    float* C = (float*)Cv;
#pragma unroll
    for (int mb = 0; mb < MBLK; ++mb) {
      const int m = mb * 16 + i;
      if (m < M) *(f32x4*)(C + (size_t)m * N + ncol) = acc[mb];
    }
  }
  else if constexpr (OUT == SK_OUT_BF16) {
    __bf16* C = (__bf16*)Cv;
    typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
#pragma unroll
    for (int mb = 0; mb < MBLK; ++mb) {
      const int m = mb * 16 + i;
      bf16x4    o;
#pragma unroll
      for (int r = 0; r < 4; ++r) o[r] = (__bf16)acc[mb][r];
      if (m < M) *(bf16x4*)(C + (size_t)m * N + ncol) = o;
    }
  }
  else {
    uint8_t* C = (uint8_t*)Cv;
#pragma unroll
    for (int mb = 0; mb < MBLK; ++mb) {
      float a = fmaxf(fmaxf(__builtin_fabsf(acc[mb][0]), __builtin_fabsf(acc[mb][1])),
                      fmaxf(__builtin_fabsf(acc[mb][2]), __builtin_fabsf(acc[mb][3])));
      a       = wave_xor_max(a, 16);
      a       = wave_xor_max(a, 32);
      if (g == 0) wave_amax[wave][mb][i] = a;
    }
    __syncthreads();
#pragma unroll
    for (int mb = 0; mb < MBLK; ++mb) {
      const int m    = mb * 16 + i;
      float     amax = 0.f;
#pragma unroll
      for (int w = 0; w < 8; ++w) amax = fmaxf(amax, wave_amax[w][mb][i]);
      const float scale = amax / 448.f;
      const float inv   = amax > 0.f ? 448.f / amax : 0.f;
      if (m < M) {
        *(uint32_t*)(C + (size_t)m * N + ncol) =
          sk_pack_e4m3x4(acc[mb][0] * inv, acc[mb][1] * inv, acc[mb][2] * inv, acc[mb][3] * inv);
        if (wave == 0 && g == 0) Cs[(size_t)ng * M + m] = scale;
      }
    }
  }
}

template <int MBLK, int OUT>
static hipError_t launch_skinny(const void* A, const float* As, const void* Bt, const float* Bs, void* C, float* Cs, int M,
                                int N, int K, int S, float* partial, unsigned* counters, hipStream_t stream)
{
  hipLaunchKernelGGL((fp8_skinny_kernel<MBLK, OUT>), dim3(N / 128, S), dim3(512), 0, stream, (const uint8_t*)A, As,
                     (const uint8_t*)Bt, Bs, C, Cs, M, N, K, S, partial, counters);
  return hipGetLastError();
}

template <int OUT>
static hipError_t dispatch_skinny(const void* A, const float* As, const void* Bt, const float* Bs, void* C, float* Cs, int M,
                                  int N, int K, int S, float* partial, unsigned* counters, hipStream_t stream)
{
  if (M <= 16) return launch_skinny<1, OUT>(A, As, Bt, Bs, C, Cs, M, N, K, S, partial, counters, stream);
  if (M <= 32) return launch_skinny<2, OUT>(A, As, Bt, Bs, C, Cs, M, N, K, S, partial, counters, stream);
  if (M <= 64) return launch_skinny<4, OUT>(A, As, Bt, Bs, C, Cs, M, N, K, S, partial, counters, stream);
  return hipErrorInvalidValue;
}

hipError_t fp8_skinny_launch(int out_kind, const void* A, const float* As, const void* Bt, const float* Bs, void* C, float* Cs,
                             int M, int N, int K, int S, float* partial, unsigned* counters, hipStream_t stream)
{
  switch (out_kind) {
    case SK_OUT_F32: return dispatch_skinny<SK_OUT_F32>(A, As, Bt, Bs, C, Cs, M, N, K, S, partial, counters, stream);
    case SK_OUT_BF16: return dispatch_skinny<SK_OUT_BF16>(A, As, Bt, Bs, C, Cs, M, N, K, S, partial, counters, stream);
    case SK_OUT_FP8Q: return dispatch_skinny<SK_OUT_FP8Q>(A, As, Bt, Bs, C, Cs, M, N, K, S, partial, counters, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace llmmm
