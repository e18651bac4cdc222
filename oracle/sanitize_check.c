/* Test infrastructure: runs every entry point of the CPU oracle on ragged shapes with buffers of exactly the
 * documented sizes, in a build with AddressSanitizer and UndefinedBehaviorSanitizer (make sanitize_check), so that an
 * index that leaves a buffer or an undefined conversion aborts the run.  Prints "sanitize ok" at the end. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include "oracle.c"

static float* randf(size_t n, unsigned* s, float scale)
{
  float* p = (float*)malloc(n * sizeof(float));
  for (size_t i = 0; i < n; ++i) {
    *s   = *s * 1664525u + 1013904223u;
    p[i] = ((float)(*s >> 8) / 16777216.0f * 2.0f - 1.0f) * scale;
  }
  return p;
}

int main(void)
{
  unsigned s = 7;
  /* FP16-path references: odd sizes */
  {
    const int M = 5, N = 7, K = 19;
    float *A = randf((size_t)M * K, &s, 1.f), *B = randf((size_t)K * N, &s, 1.f), *Bt = randf((size_t)N * K, &s, 1.f);
    float* C = (float*)malloc((size_t)M * N * sizeof(float));
    oracle_kahan_gemm(A, B, C, M, N, K, 0);
    oracle_kahan_gemm(A, B, C, M, N, K, 1);
    oracle_kahan_gemm_bt(A, Bt, C, M, N, K, 1);
    oracle_double_gemm(A, B, C, M, N, K);
    free(A), free(B), free(Bt), free(C);
  }
  /* quantiser: ragged rows and columns, all four scale layouts, non-finite values */
  {
    const int M = 130, N = 260, nb = (N + 127) / 128, mb = (M + 127) / 128;
    float*    x = randf((size_t)M * N, &s, 3.f);
    x[3]        = NAN, x[N + 5] = INFINITY, x[2 * N] = -INFINITY;
    uint8_t* q  = (uint8_t*)malloc((size_t)M * N);
    float*   sc = (float*)malloc((size_t)nb * M * sizeof(float)); /* the largest of the four layouts */
    float*   y  = (float*)malloc((size_t)M * N * sizeof(float));
    oracle_quant_fp8(x, q, sc, M, N, 1, 1);
    oracle_dequant_fp8(q, sc, y, M, N, 1, 1);
    oracle_quant_fp8(x, q, sc, M, N, 1, 0);
    oracle_quant_fp8(x, q, sc, M, N, 128, 1);
    float* sc2 = (float*)malloc((size_t)mb * nb * sizeof(float));
    oracle_quant_fp8(x, q, sc2, M, N, 128, 0);
    oracle_dequant_fp8(q, sc2, y, M, N, 128, 0);
    free(x), free(q), free(sc), free(sc2), free(y);
  }
  /* FP8 GEMM, both promotion orders, ragged M and N; fused re-quantisation in its three forms */
  {
    const int M = 5, N = 200, K = 256, kb = K / 128, nb = (N + 127) / 128;
    float *   xa = randf((size_t)M * K, &s, 2.f), *xb = randf((size_t)N * K, &s, 0.05f);
    uint8_t * Aq = (uint8_t*)malloc((size_t)M * K), *Bq = (uint8_t*)malloc((size_t)N * K), *Cq = (uint8_t*)malloc((size_t)M * N);
    float *   As = (float*)malloc((size_t)kb * M * sizeof(float)), *Bs = (float*)malloc((size_t)nb * kb * sizeof(float));
    float *   C = (float*)malloc((size_t)M * N * sizeof(float)), *Cs = (float*)malloc((size_t)nb * M * sizeof(float));
    oracle_quant_fp8(xa, Aq, As, M, K, 1, 1);
    oracle_quant_fp8(xb, Bq, Bs, N, K, 128, 0);
    if (oracle_fp8_gemm(Aq, As, Bq, Bs, C, M, N, K, 128, 1) || oracle_fp8_gemm(Aq, As, Bq, Bs, C, M, N, K, 32, 0) || oracle_fp8_gemm(Aq, As, Bq, Bs, C, M, N, K, 32, 1)) return 1;
    if (!oracle_fp8_gemm(Aq, As, Bq, Bs, C, M, N, 100, 128, 1)) return 1; /* K % 128 != 0 is refused */
    C[1] = NAN, C[N + 2] = INFINITY;
    oracle_requant_c_1x128(C, Cq, Cs, M, N, 1, 1);
    oracle_requant_c_1x128(C, Cq, Cs, M, N, 0, 1);
    oracle_requant_c_1x128(C, Cq, Cs, M, N, 1, 0);
    free(xa), free(xb), free(Aq), free(Bq), free(Cq), free(As), free(Bs), free(C), free(Cs);
  }
  /* RMSNorm; per-head norm + rope with clamped positions */
  {
    const int M = 3, K = 384;
    float *   x = randf((size_t)M * K, &s, 2.f), *w = randf(K, &s, 1.f), *y = (float*)malloc((size_t)M * K * sizeof(float));
    oracle_rmsnorm(x, w, 1e-6f, y, M, K);
    const int n_q = 1, n_kv = 1, rows = 4;
    float *   qw = randf(128, &s, 1.f), *kw = randf(128, &s, 1.f), *ct = randf((size_t)rows * 64, &s, 1.f), *st = randf((size_t)rows * 64, &s, 1.f);
    int32_t   pos[3] = {-5, 2, 99};
    oracle_qk_norm_rope(x, qw, kw, 1e-6f, ct, st, rows, pos, n_q, n_kv, y, M);
    oracle_qk_norm_rope(x, NULL, NULL, 1e-6f, ct, st, rows, pos, n_q, n_kv, y, M);
    free(x), free(w), free(y), free(qw), free(kw), free(ct), free(st);
  }
  /* scalar and bulk converters over every code / a spread of values */
  {
    float    f[8] = {0.f, -0.f, 1e-30f, -448.f, 465.f, INFINITY, -INFINITY, NAN};
    uint8_t  q[8];
    uint16_t h[8];
    float    back[8];
    oracle_e4m3_encode_n(f, q, 8);
    oracle_e4m3_decode_n(q, back, 8);
    oracle_f32_to_f16_n(f, h, 8);
    oracle_f16_to_f32_n(h, back, 8);
    oracle_f32_to_bf16_n(f, h, 8);
    oracle_bf16_to_f32_n(h, back, 8);
    for (int c = 0; c < 256; ++c) (void)oracle_e4m3_encode(oracle_e4m3_decode((uint8_t)c));
    for (int c = 0; c < 65536; c += 7) (void)oracle_f32_to_f16(oracle_f16_to_f32((uint16_t)c)), (void)oracle_f32_to_bf16(oracle_bf16_to_f32((uint16_t)c));
  }
  puts("sanitize ok");
  return 0;
}
