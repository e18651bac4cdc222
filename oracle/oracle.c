/*
 * CPU oracle for the LLMMM matrix-multiplication path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the arithmetic of the reference's GPU kernels so that the
 * HIP kernels of this repository can be checked against it.  It is never linked into, called
 * from or shipped with the product library: only tests, the smoke check and the cpu_baseline
 * leg of the benchmark may use it.
 *
 * The reference cannot be compiled here (CUDA C++ with SM89 inline PTX; no nvcc), so there is
 * no reference build to compare with; every function below is pinned by closed forms,
 * invariants and exhaustive tables in tests/test_oracle_*.py instead:
 *
 *   oracle_kahan_gemm        test/kahan.cu:16-26             pinned: identity/all-ones KATs, brute force in
 *                                                            Python ints/fractions on tiny shapes, agreement
 *                                                            with oracle_double_gemm
 *   oracle_double_gemm       test/kahan.cu:48-55             pinned: exact rational arithmetic on tiny shapes
 *   oracle_e4m3_decode/encode  cuda_fp8.h __nv_fp8_e4m3 (CUDA toolkit, version unpinned by the reference;
 *                            OCP FP8 E4M3, RNE, saturate-to-finite, NaN->0x7F)
 *                                                            pinned: exhaustive 256-code table from the OCP
 *                                                            spec, decode->encode identity, all midpoints,
 *                                                            saturation, torch.float8_e4m3fn cross-check
 *   oracle_quant_fp8         examples/005.fp8.mm.cu:439-545  pinned: invariants (amax element -> +-448,
 *                                                            |x-q*s| <= half ulp, zero block -> s=0,q=0)
 *   oracle_fp8_gemm          examples/005.fp8.mm.cu:176-199 (per-32 promotion),
 *                            examples/005.fp8.mm.cu:885-902 (per-128 promotion)
 *                                                            pinned: B = I known-answer test
 *                                                            (examples/005.fp8.mm.cu:2620-2634), exact
 *                                                            rational evaluation on small shapes
 *   oracle_requant_c_1x128   examples/005.fp8.mm.opt.cu:401-462 (reciprocal form) and
 *                            examples/005.fp8.mm.cu:759-774 (division form)
 *                                                            pinned: idempotence, B = I => Cq == Aq
 *
 *   oracle_rmsnorm           no reference kernel (fusing RMSNorm into the quantiser is on the reference's
 *                            plan, README.md:16): y = x / sqrt(mean(x^2) + eps) * w in fp32, the sum of squares
 *                            taken in the order of 256 GPU lanes (see the function)
 *                                                            pinned: float64 evaluation, exact invariance under
 *                                                            power-of-two scaling (eps = 0), unit mean square
 *
 *   oracle_qk_norm_rope      no reference kernel (fusing RMSNorm and RoPE into the GEMM is on the reference's plan,
 *                            README.md:16): per-head RMSNorm (head size 128) and rotary embedding of the query and key
 *                            heads of a QKV projection, value heads untouched
 *                                                            pinned: float64 evaluation of the rotate-half formula,
 *                                                            identity at angle 0, quarter turn, exact inverse
 *                                                            and pair norm on an integer 3-4-5 rotation, the
 *                                                            documented summation order rebuilt in numpy
 *
 * Compile with -ffp-contract=off: every fused multiply-add below is written explicitly.
 */
#include <math.h>
#include <stdint.h>
#include <stddef.h>
#include <string.h>
#include <stdlib.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

ORACLE_API int oracle_num_threads(void)
{
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

ORACLE_API void oracle_set_num_threads(int n)
{
#ifdef _OPENMP
  if (n > 0) omp_set_num_threads(n);
#else
  (void)n;
#endif
}

/* ------------------------------------------------------------------ scalar formats */

/* IEEE binary16 -> binary32 (exact). Counterpart of float(half), test/fp16_mm_test.cc:64. */
ORACLE_API float oracle_f16_to_f32(uint16_t h)
{
  uint32_t sign = (uint32_t)(h >> 15) << 31;
  int      e    = (h >> 10) & 31;
  uint32_t m    = h & 1023u;
  float    v;
  if (e == 31) {
    uint32_t bits = sign | 0x7f800000u | (m << 13);
    memcpy(&v, &bits, 4);
    return v;
  }
  if (e == 0)
    v = ldexpf((float)m, -24);
  else
    v = ldexpf((float)(1024u + m), e - 25);
  return sign ? -v : v;
}

/* binary32 -> binary16, round-to-nearest-even, overflow to inf.  Counterpart of half(float),
 * test/fp16_mm_test.cc:43 and the epilogue cast at src/mm/fp16/mm.cuh:427. */
ORACLE_API uint16_t oracle_f32_to_f16(float f)
{
  uint32_t x;
  memcpy(&x, &f, 4);
  uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  uint32_t ax   = x & 0x7fffffffu;
  if (ax >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | ((ax > 0x7f800000u) ? 0x200u : 0u));
  if (ax >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* >= 65520 rounds to inf */
  if (ax < 0x33000001u) return sign;                        /* <= 2^-25 rounds to zero (tie to even) */
  int      e = (int)(ax >> 23) - 127;
  uint32_t m = (ax & 0x7fffffu) | 0x800000u; /* 24-bit significand */
  int      shift;                            /* bits to drop */
  uint32_t base;
  if (e >= -14) {
    shift = 13;
    base  = (uint32_t)(e + 15) << 10;
    m &= 0x7fffffu;
  }
  else {
    shift = 13 + (-14 - e);
    base  = 0;
  }
  uint32_t keep = m >> shift;
  uint32_t rem  = m & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (keep & 1u))) keep += 1u;
  return (uint16_t)(sign | (base + keep)); /* carry into the exponent is the correct result */
}

ORACLE_API float oracle_bf16_to_f32(uint16_t h)
{
  uint32_t bits = (uint32_t)h << 16;
  float    v;
  memcpy(&v, &bits, 4);
  return v;
}

/* binary32 -> bfloat16, round-to-nearest-even (NaN kept quiet).  Counterpart of
 * __nv_bfloat16(float), src/mm/fp16/mm.cu:44-46. */
ORACLE_API uint16_t oracle_f32_to_bf16(float f)
{
  uint32_t x;
  memcpy(&x, &f, 4);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
  uint32_t lsb = (x >> 16) & 1u;
  x += 0x7fffu + lsb;
  return (uint16_t)(x >> 16);
}

/* OCP FP8 E4M3 (e4m3fn): 1-4-3, bias 7, no infinity, NaN = S.1111.111, max finite 448. */
ORACLE_API float oracle_e4m3_decode(uint8_t c)
{
  int   s = c >> 7, e = (c >> 3) & 15, m = c & 7;
  float v;
  if (e == 15 && m == 7) return NAN;
  if (e == 0)
    v = ldexpf((float)m, -9);
  else
    v = ldexpf((float)(8 + m), e - 10);
  return s ? -v : v;
}

/* float -> e4m3, round-to-nearest-even, saturate to +-448 (also for +-inf), NaN -> 0x7F.
 * Behaviour of __nv_fp8_e4m3(float) = __nv_cvt_float_to_fp8(x, __NV_SATFINITE, __NV_E4M3),
 * call sites examples/005.fp8.mm.cu:482-485, examples/005.fp8.mm.opt.cu:445-454. */
ORACLE_API uint8_t oracle_e4m3_encode(float f)
{
  uint32_t x;
  memcpy(&x, &f, 4);
  uint8_t  sign = (uint8_t)((x >> 24) & 0x80u);
  uint32_t ax   = x & 0x7fffffffu;
  if (ax > 0x7f800000u) return 0x7f; /* NaN: CUDA returns 0x7F regardless of sign */
  float a;
  memcpy(&a, &ax, 4);
  if (a >= 464.0f) return (uint8_t)(sign | 0x7e); /* 464 = midpoint(448, 480) ties to even = 480 -> saturates */
  if (a > 448.0f) return (uint8_t)(sign | 0x7e);  /* rounds down to 448 */
  if (a < ldexpf(1.0f, -10)) return sign;         /* below half the min subnormal -> 0 */
  if (a == ldexpf(1.0f, -10)) return sign;        /* tie between 0 and 2^-9 -> even (0) */
  int e;
  (void)frexpf(a, &e); /* a = fr * 2^e, fr in [0.5,1) -> unbiased exponent e-1 */
  int ue = e - 1;
  if (ue < -6) ue = -6;                          /* subnormal range shares the 2^-6 scale */
  float    q    = ldexpf(a, 3 - ue);             /* a in units of the spacing 2^(ue-3); exact */
  float    fl   = floorf(q);
  float    rem  = q - fl;
  uint32_t keep = (uint32_t)fl;
  if (rem > 0.5f || (rem == 0.5f && (keep & 1u))) keep += 1u;
  /* keep is in [8,16] for normals (16 = carry), [0,8] for subnormals */
  uint32_t code;
  if (ue == -6 && keep < 8u)
    code = keep; /* subnormal */
  else {
    if (keep == 16u) {
      keep = 8u;
      ue += 1;
    }
    code = ((uint32_t)(ue + 7) << 3) | (keep - 8u);
  }
  if (code > 0x7eu) code = 0x7eu;
  return (uint8_t)(sign | code);
}

/* ------------------------------------------------------------------ FP16-path GEMM references */

/* test/kahan.cu:16-26.  A [M,K], B [K,N], C [M,N], all fp32 row-major.
 * fused != 0 evaluates y as fmaf(a, b, -diff): nvcc contracts `A[k]*B[k*N] - diff` into one FMA
 * under its default --fmad=true (the reference's CMakeLists.txt:19 does not disable it).  For
 * inputs that are fp16 or bf16 values the product is exact in fp32 and both forms agree. */
ORACLE_API void oracle_kahan_gemm(const float* A, const float* B, float* C, int M, int N, int K, int fused)
{
#pragma omp parallel for schedule(static)
  for (int m = 0; m < M; ++m) {
    float* sum  = (float*)calloc((size_t)N, sizeof(float));
    float* diff = (float*)calloc((size_t)N, sizeof(float));
    const float* a = A + (size_t)m * K;
    for (int k = 0; k < K; ++k) {
      const float  ak = a[k];
      const float* b  = B + (size_t)k * N;
      if (fused) {
        for (int n = 0; n < N; ++n) {
          float y = fmaf(ak, b[n], -diff[n]);
          float t = sum[n] + y;
          diff[n] = (t - sum[n]) - y;
          sum[n]  = t;
        }
      }
      else {
        for (int n = 0; n < N; ++n) {
          float y = ak * b[n] - diff[n];
          float t = sum[n] + y;
          diff[n] = (t - sum[n]) - y;
          sum[n]  = t;
        }
      }
    }
    memcpy(C + (size_t)m * N, sum, (size_t)N * sizeof(float));
    free(sum);
    free(diff);
  }
}

/* test/kahan.cu:48-55: the product is formed in fp32 (float * float), widened, and added to a
 * double accumulator in ascending k; the result is rounded to fp32 on the store. */
ORACLE_API void oracle_double_gemm(const float* A, const float* B, float* C, int M, int N, int K)
{
#pragma omp parallel for schedule(static)
  for (int m = 0; m < M; ++m) {
    double*      sum = (double*)calloc((size_t)N, sizeof(double));
    const float* a   = A + (size_t)m * K;
    for (int k = 0; k < K; ++k) {
      const float  ak = a[k];
      const float* b  = B + (size_t)k * N;
      for (int n = 0; n < N; ++n) {
        float p = ak * b[n];
        sum[n] += (double)p;
      }
    }
    for (int n = 0; n < N; ++n) C[(size_t)m * N + n] = (float)sum[n];
    free(sum);
  }
}

/* Same as oracle_kahan_gemm but B is given transposed, Bt [N,K] (B[k][n] = Bt[n][k]); the
 * arithmetic and its order are identical, so the result is bit-identical to the [K,N] form. */
ORACLE_API void oracle_kahan_gemm_bt(const float* A, const float* Bt, float* C, int M, int N, int K, int fused)
{
#pragma omp parallel for schedule(static)
  for (int m = 0; m < M; ++m) {
    const float* a = A + (size_t)m * K;
    for (int n = 0; n < N; ++n) {
      const float* b   = Bt + (size_t)n * K;
      float        sum = 0.0f, diff = 0.0f;
      for (int k = 0; k < K; ++k) {
        float y = fused ? fmaf(a[k], b[k], -diff) : (a[k] * b[k] - diff);
        float t = sum + y;
        diff    = (t - sum) - y;
        sum     = t;
      }
      C[(size_t)m * N + n] = sum;
    }
  }
}

/* ------------------------------------------------------------------ FP8 blockwise quantiser */

/* examples/005.fp8.mm.cu:439-545.  x [M,N] fp32 -> q [M,N] e4m3 + scales.
 * quant_m is 1 (one scale per row and 128-column group) or 128 (one per 128x128 block);
 * the 128-wide column groups and 128-tall row groups may be ragged at the edges (the kernel
 * guards rows with `m < M`, :468; columns are assumed a multiple of 4 by its float4 loads).
 * scale layouts:
 *   quant_m == 1,  transposed:  s[(n/128)*M + m]              (:494)
 *   quant_m == 1,  plain:       s[m*ceil(N/128) + n/128]      (:497)
 *   quant_m == 128, transposed: s[(n/128)*M + m/128]          (:532-533; row stride M as written)
 *   quant_m == 128, plain:      s[(m/128)*ceil(N/128) + n/128] (:536-538)
 * amax starts from (float)INT_MIN (:456) so a block of zeros yields amax 0, s 0 and q 0;
 * s = amax / 448.f (:479, :516); q = e4m3(s ? x / s : 0) (:482-485, :523-528). */
ORACLE_API void oracle_quant_fp8(const float* x, uint8_t* q, float* scale, int M, int N, int quant_m,
                                 int scale_transpose)
{
  const int nb = (N + 127) / 128;
  const int mb = (M + quant_m - 1) / quant_m;
#pragma omp parallel for schedule(static)
  for (int bi = 0; bi < mb; ++bi) {
    for (int bj = 0; bj < nb; ++bj) {
      int   m0 = bi * quant_m, m1 = m0 + quant_m < M ? m0 + quant_m : M;
      int   n0 = bj * 128, n1 = n0 + 128 < N ? n0 + 128 : N;
      float amax = (float)(-2147483647 - 1);
      for (int m = m0; m < m1; ++m)
        for (int n = n0; n < n1; ++n) {
          float v = fabsf(x[(size_t)m * N + n]);
          amax    = (amax < v) ? v : amax;
        }
      float s = amax / 448.0f;
      for (int m = m0; m < m1; ++m)
        for (int n = n0; n < n1; ++n) {
          float v                 = x[(size_t)m * N + n];
          q[(size_t)m * N + n] = oracle_e4m3_encode(s ? v / s : 0.0f);
        }
      /* both block heights index the scale by the block-row bi = m / quant_m */
      if (scale_transpose)
        scale[(size_t)bj * M + bi] = s; /* row stride M as written at :494 and :532 */
      else
        scale[(size_t)bi * nb + bj] = s;
    }
  }
}

/* ------------------------------------------------------------------ FP8 blockwise GEMM */

/* C[m,n] = sum_kb  partial(kb) * As[kb,m] * Bs[n/128,kb]
 *   A  [M,K] e4m3,  As [K/128, M] fp32,  Bt [N,K] e4m3 (B transposed),  Bs [ceil(N/128), K/128] fp32,
 *   C  [M,N] fp32.
 * promote == 32  follows examples/005.fp8.mm.cu:176-199: each 32-K tensor-core product is rounded to
 *                fp32 and promoted on its own;  assoc == 0: acc += (p*As)*Bs (:194),
 *                assoc == 1: acc += p*(As*Bs) (:369-370, all later variants).
 * promote == 128 follows examples/005.fp8.mm.cu:885-902: the four 32-K products of a slice accumulate
 *                inside the tensor-core accumulator and are promoted once, acc += p*(As*Bs).
 * The partial sums are evaluated exactly (products of e4m3 values are multiples of 2^-18 below
 * 2^18, so a double holds any 128-term sum exactly) and rounded once to fp32: the ideal value of
 * a hardware dot-product unit whose internal order is unspecified.  The promotion itself is one
 * FMA per slice (nvcc's default contraction of `acc += p * s`).
 * M, N are arbitrary; K must be a multiple of 128. */
ORACLE_API int oracle_fp8_gemm(const uint8_t* A, const float* As, const uint8_t* Bt, const float* Bs, float* C, int M,
                               int N, int K, int promote, int assoc)
{
  if (K % 128 != 0 || (promote != 32 && promote != 128)) return 1;
  const int kb_n = K / 128;
  float     lut[256];
  for (int i = 0; i < 256; ++i) lut[i] = oracle_e4m3_decode((uint8_t)i);
#pragma omp parallel for schedule(static)
  for (int m = 0; m < M; ++m) {
    float* arow = (float*)malloc((size_t)K * sizeof(float));
    for (int k = 0; k < K; ++k) arow[k] = lut[A[(size_t)m * K + k]];
    for (int n = 0; n < N; ++n) {
      const uint8_t* b   = Bt + (size_t)n * K;
      float          acc = 0.0f;
      for (int kb = 0; kb < kb_n; ++kb) {
        const float as = As[(size_t)kb * M + m];
        const float bs = Bs[(size_t)(n / 128) * kb_n + kb];
        if (promote == 128) {
          double p = 0.0;
          for (int k = kb * 128; k < kb * 128 + 128; ++k) p += (double)arow[k] * (double)lut[b[k]];
          acc = fmaf((float)p, as * bs, acc);
        }
        else {
          for (int c = 0; c < 4; ++c) {
            double p = 0.0;
            for (int k = kb * 128 + c * 32; k < kb * 128 + c * 32 + 32; ++k) p += (double)arow[k] * (double)lut[b[k]];
            if (assoc == 0)
              acc = fmaf((float)p * as, bs, acc);
            else
              acc = fmaf((float)p, as * bs, acc);
          }
        }
      }
      C[(size_t)m * N + n] = acc;
    }
    free(arow);
  }
  return 0;
}

/* Fused C re-quantisation, examples/005.fp8.mm.opt.cu:401-462.
 * For every row m and 128-column group nb: amax = max|C|, scale = amax/448.f,
 * reciprocal != 0: Cq = e4m3(C * (448.f/amax))  (opt.cu:439-454)
 * reciprocal == 0: Cq = e4m3(C / scale)         (examples/005.fp8.mm.cu:759-769)
 * Cs[nb*M + m] = scale (opt.cu:458-461).
 * zero_guard != 0 (this repository's kernels): a group whose 448.f/amax is not finite -- all zeros, or amax below
 *                  2^-119 so that the reciprocal overflows -- gives codes 0 next to its scale amax/448;
 * zero_guard == 0: the reference's unguarded arithmetic (0 * inf = NaN -> 0x7F; with an overflowing reciprocal
 *                  +-448 for every non-zero element).
 * Non-finite C: a NaN element never enters the maximum.  (In the reference a thread's chain
 * `max_val > |c| ? max_val : |c|`, opt.cu:413, keeps a NaN only when it is the last value that thread compares, and the
 * cross-lane `max()` steps behind it, opt.cu:415-416 and :432, drop it again: fmaxf semantics.  Only a group that holds
 * nothing but NaN differs: NaN scale there, scale 0 here under the zero guard.)  A NaN element's code is 0x7F; an
 * infinite element gives amax = scale = inf and 448/amax = 0, so finite elements become (signed) zeros and the
 * infinite ones 0 * inf = NaN -> 0x7F, as in the reference. */
ORACLE_API void oracle_requant_c_1x128(const float* C, uint8_t* Cq, float* Cs, int M, int N, int reciprocal,
                                       int zero_guard)
{
  const int nb_n = (N + 127) / 128;
#pragma omp parallel for schedule(static)
  for (int m = 0; m < M; ++m) {
    for (int nb = 0; nb < nb_n; ++nb) {
      int   n0 = nb * 128, n1 = n0 + 128 < N ? n0 + 128 : N;
      float amax = 0.0f;
      for (int n = n0; n < n1; ++n) {
        float v = fabsf(C[(size_t)m * N + n]);
        if (v > amax) amax = v; /* a NaN is never taken, see above */
      }
      float scale = amax / 448.0f;
      float inv   = 448.0f / amax;
      for (int n = n0; n < n1; ++n) {
        float v = C[(size_t)m * N + n];
        float r;
        if (zero_guard && !(inv < INFINITY))
          r = v * 0.0f; /* amax == 0, or so small that 448 / amax overflows: zeros, a NaN stays a NaN (code 0x7F) */
        else
          r = reciprocal ? v * inv : v / scale;
        Cq[(size_t)m * N + n] = oracle_e4m3_encode(r);
      }
      Cs[(size_t)nb * M + m] = scale;
    }
  }
}

/* Dequantise helper for tests: x = decode(q) * s with s looked up as in oracle_quant_fp8
 * (quant_m == 1 transposed layout or quant_m == 128 plain layout only). */
ORACLE_API void oracle_dequant_fp8(const uint8_t* q, const float* scale, float* x, int M, int N, int quant_m,
                                   int scale_transpose)
{
  const int nb = (N + 127) / 128;
#pragma omp parallel for schedule(static)
  for (int m = 0; m < M; ++m)
    for (int n = 0; n < N; ++n) {
      int   bi = m / quant_m, bj = n / 128;
      float s  = scale_transpose ? scale[(size_t)bj * M + bi] : scale[(size_t)bi * nb + bj];
      x[(size_t)m * N + n] = oracle_e4m3_decode(q[(size_t)m * N + n]) * s;
    }
}

/* Bulk converters so Python does not loop. */
ORACLE_API void oracle_e4m3_encode_n(const float* x, uint8_t* q, size_t n)
{
  for (size_t i = 0; i < n; ++i) q[i] = oracle_e4m3_encode(x[i]);
}
ORACLE_API void oracle_e4m3_decode_n(const uint8_t* q, float* x, size_t n)
{
  for (size_t i = 0; i < n; ++i) x[i] = oracle_e4m3_decode(q[i]);
}
ORACLE_API void oracle_f32_to_f16_n(const float* x, uint16_t* h, size_t n)
{
  for (size_t i = 0; i < n; ++i) h[i] = oracle_f32_to_f16(x[i]);
}
ORACLE_API void oracle_f16_to_f32_n(const uint16_t* h, float* x, size_t n)
{
  for (size_t i = 0; i < n; ++i) x[i] = oracle_f16_to_f32(h[i]);
}
ORACLE_API void oracle_f32_to_bf16_n(const float* x, uint16_t* h, size_t n)
{
  for (size_t i = 0; i < n; ++i) h[i] = oracle_f32_to_bf16(x[i]);
}
ORACLE_API void oracle_bf16_to_f32_n(const uint16_t* h, float* x, size_t n)
{
  for (size_t i = 0; i < n; ++i) x[i] = oracle_bf16_to_f32(h[i]);
}

/* Per-head RMSNorm and rotary position embedding behind a QKV projection (heads of 128 columns: n_q query heads, then
 * n_kv key heads, then n_kv value heads; N = (n_q + 2 n_kv) * 128).  No reference kernel (README.md:16 plans the
 * fusion); the arithmetic order is this build's definition, chosen so that 32 GPU lanes per head reproduce it:
 *   norm (query heads with qw, key heads with kw; skipped when the weight pointer is NULL): lane l of 32 owns columns
 *     4l .. 4l+3 and accumulates acc = fma(x, x, acc) over them in ascending order from 0; the 32 partial sums are
 *     combined by a butterfly (p[l] += p[l ^ 16], then ^8, ^4, ^2, ^1); r = 1 / sqrt(total / 128 + eps);
 *     x <- (x * r) * w[col]                                (w has 128 entries, shared by all heads of a kind)
 *   rope (query and key heads; rotate-half pairing of column i with column i + 64, i < 64; angle row
 *     p = clamp(pos[m], 0, table_rows - 1) of the cos / sin tables [table_rows, 64]):
 *     y[i]      = fma(x[i],      cos[p,i], -(x[i + 64] * sin[p,i]))
 *     y[i + 64] = fma(x[i + 64], cos[p,i],   x[i]      * sin[p,i])
 *   value heads: y = x. */
ORACLE_API void oracle_qk_norm_rope(const float* x, const float* qw, const float* kw, float eps, const float* cos_t, const float* sin_t,
                                    int table_rows, const int32_t* pos, int n_q, int n_kv, float* y, int M)
{
  const int N = (n_q + 2 * n_kv) * 128;
#pragma omp parallel for schedule(static)
  for (int m = 0; m < M; ++m) {
    int p = pos[m];
    if (p < 0) p = 0;
    if (p > table_rows - 1) p = table_rows - 1;
    const float* c = cos_t + (size_t)p * 64;
    const float* s = sin_t + (size_t)p * 64;
    for (int h = 0; h < n_q + 2 * n_kv; ++h) {
      const float* xr = x + (size_t)m * N + h * 128;
      float*       yr = y + (size_t)m * N + h * 128;
      if (h >= n_q + n_kv) {
        for (int i = 0; i < 128; ++i) yr[i] = xr[i];
        continue;
      }
      float        v[128];
      const float* w = h < n_q ? qw : kw;
      for (int i = 0; i < 128; ++i) v[i] = xr[i];
      if (w) {
        float part[32];
        for (int l = 0; l < 32; ++l) {
          float acc = 0.f;
          for (int e = 0; e < 4; ++e) acc = fmaf(v[4 * l + e], v[4 * l + e], acc);
          part[l] = acc;
        }
        for (int step = 16; step >= 1; step >>= 1) {
          float t[32];
          for (int l = 0; l < 32; ++l) t[l] = part[l] + part[l ^ step];
          for (int l = 0; l < 32; ++l) part[l] = t[l];
        }
        const float r = 1.0f / sqrtf(part[0] / 128.0f + eps);
        for (int i = 0; i < 128; ++i) v[i] = (v[i] * r) * w[i];
      }
      for (int i = 0; i < 64; ++i) {
        const float lo = v[i], hi = v[i + 64];
        yr[i]      = fmaf(lo, c[i], -(hi * s[i]));
        yr[i + 64] = fmaf(hi, c[i], lo * s[i]);
      }
    }
  }
}

/* RMSNorm in fp32: y[m,k] = (x[m,k] * r) * w[k], r = 1 / sqrt(sum_k x[m,k]^2 / K + eps).
 * No reference kernel (README.md:16 plans the fusion); the arithmetic order is this build's definition, chosen so
 * that GPU wavefronts reproduce it bit for bit: the row is cut into chunks of 4 consecutive elements; chunk c belongs
 * to virtual lane c % 256, which accumulates its chunks in ascending order with one fused multiply-add per element
 * (acc = fma(x, x, acc), elements of a chunk in ascending order); each group of 64 virtual lanes combines its partial
 * sums by a butterfly (p[l] += p[l ^ 32], then ^16, ^8, ^4, ^2, ^1), and the four group sums are added as
 * (G0 + G1) + (G2 + G3).  Division by K, the square root and the reciprocal are correctly rounded IEEE operations.
 * K % 4 == 0. */
ORACLE_API void oracle_rmsnorm(const float* x, const float* w, float eps, float* y, int M, int K)
{
#pragma omp parallel for schedule(static)
  for (int m = 0; m < M; ++m) {
    const float* xr = x + (size_t)m * K;
    float        p[256];
    for (int l = 0; l < 256; ++l) p[l] = 0.f;
    const int chunks = K / 4;
    for (int c = 0; c < chunks; ++c)
      for (int e = 0; e < 4; ++e) p[c & 255] = fmaf(xr[4 * c + e], xr[4 * c + e], p[c & 255]);
    float G[4];
    for (int g = 0; g < 4; ++g) {
      float* pg = p + 64 * g;
      for (int step = 32; step >= 1; step >>= 1) {
        float t[64];
        for (int l = 0; l < 64; ++l) t[l] = pg[l] + pg[l ^ step];
        for (int l = 0; l < 64; ++l) pg[l] = t[l];
      }
      G[g] = pg[0];
    }
    const float total = (G[0] + G[1]) + (G[2] + G[3]);
    const float ms    = total / (float)K;
    const float r     = 1.0f / sqrtf(ms + eps);
    for (int k = 0; k < K; ++k) y[(size_t)m * K + k] = (xr[k] * r) * w[k];
  }
}
