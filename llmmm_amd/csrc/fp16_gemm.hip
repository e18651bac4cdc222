// FP16 / BF16 GEMM for gfx950:  C[M,N] = A[M,K] * B,  fp32 accumulation, output rounded to T.
//
// Replaces the kernel behind LLMMM::fp16_mm<T> (reference: src/mm/fp16/mm.cu:6-42 launching
// src/mm/fp16/mm.cuh:657-684).  Layouts follow the reference: A[m*K+k] (mm.cuh:102),
// B[k*N+n] (mm.cuh:103), C[m*N+n] (mm.cuh:236).  A second B layout, Bt[n*K+k], is an extension.
//
// Design (nothing here is translated from the reference's mma.sync/ldmatrix code):
//  * one workgroup computes a BM x BN tile, one wavefront a 64(m) x 128(n) sub-tile built from
//    v_mfma_f32_32x32x16_{f16,bf16}; the MFMA is issued with B as the row operand and A as the
//    column operand so that each lane ends up with 4 consecutive n of one row m (packed stores);
//  * K advances 32 elements per stage (64 bytes per tile row, (BM+BN)*64 bytes of LDS) and four
//    stages form a ring that LDS-direct global loads fill three stages ahead of the MFMAs
//    (no staging registers, no ds_write);
//  * the single workgroup barrier of a stage sits between its two 16-wide k-steps: by then
//    every wave has pulled the stage's operands into registers, so the barrier both frees the
//    stage's buffer for the load of stage +4 and publishes stage +1, whose first fragments are
//    fetched right behind it -- no wave ever waits on an LDS read it has just issued;
//  * A (and Bt) tiles are K-major and read with ds_read_b128 through the SWZ_ROW64 placement;
//    a row-major B tile is kept as [k][n] and read with the transposing ds_read_b64_tr_b16,
//    its 64-byte column chunks XOR-ed with k&3;
//  * workgroup ids are remapped so that the tiles resident on one XCD share A/B panels in its L2.
#include "device_common.hip.h"
#include "kernels.h"

namespace llmmm {

template <typename T>
struct Mfma16;
template <>
struct Mfma16<_Float16> {
  typedef f16x8 vec;
  static __device__ __forceinline__ f32x16 run(vec x, vec y, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(x, y, c, 0, 0, 0); }
};
template <>
struct Mfma16<__bf16> {
  typedef bf16x8 vec;
  static __device__ __forceinline__ f32x16 run(vec x, vec y, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, c, 0, 0, 0); }
};

template <typename T, int BM, int BN, bool B_NK>
struct Fp16Tile {
  static constexpr int WAVES_M = BM / 64;
  static constexpr int WAVES_N = BN / 128;
  static constexpr int NW      = WAVES_M * WAVES_N;
  static constexpr int NT      = NW * 64;
  static constexpr int BK      = 32;              // elements of K per stage
  static constexpr int A_BYTES = BM * 64;         // K-major, 64 bytes per row
  static constexpr int B_BYTES = BN * 64;         // either layout: 32 x BN x 2 bytes
  static constexpr int B_ROW   = BN * 2;          // row pitch of the [k][n] layout
  static constexpr int STAGE   = A_BYTES + B_BYTES;
  static constexpr int A_LOADS = (BM / 16) / NW;  // 1024-byte groups per wave
  static constexpr int B_LOADS = (BN / 16) / NW;
  static constexpr int LOADS   = A_LOADS + B_LOADS;
  // wave-uniform step between two loads of a wave
  static constexpr int ROWS_PER_LOAD    = 16 * NW;        // K-major tiles: tile rows
  static constexpr int B_KROWS_PER_GRP  = 1024 / B_ROW;   // [k][n] tile: k rows per 1 KB group
  static constexpr int B_KROWS_PER_LOAD = B_KROWS_PER_GRP * NW;
};

// Issue the LDS-direct loads of one stage.  `kleft` = K - k0 (elements still to go); a stage
// whose K range is cut short zero-fills the missing part so that the MFMAs need no masking.
// All loads of a wave share one per-lane offset: they differ by a wave-uniform row (or k) step
// that the swizzles do not see.  The loads are inline assembly with the wave-uniform part of the
// address in SGPRs: no vector ALU work goes into addresses, and the compiler -- which would
// turn every wait it inserts into "all loads done" while it knows of an LDS-direct load in
// flight -- never sees them; the kernel places the s_waitcnt vmcnt itself.
__device__ __forceinline__ void sload_lds_16B(const void* sbase, unsigned voff, unsigned lds_addr)
{
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "s"(lds_addr) : "memory");
}
template <typename T, int BM, int BN, bool B_NK, bool KTAIL>
__device__ __forceinline__ void fp16_issue_stage(char LLMMM_LDS* lds, unsigned lds_addr, const T* __restrict__ Ag, const T* __restrict__ Bg,
                                                 unsigned a_off, int a_k, unsigned b_off, int b_k, int K, int N, int wave,
                                                 int lane, int kleft)
{
  typedef Fp16Tile<T, BM, BN, B_NK> TC;
  // without a K tail (K % 32 == 0) the loads are unconditional: straight-line code keeps the
  // compiler's wait-count bookkeeping exact
  const bool full = !KTAIL || kleft >= TC::BK;
#pragma unroll
  for (int i = 0; i < TC::A_LOADS; ++i) {
    char LLMMM_LDS* dst = lds + (wave + i * TC::NW) * 1024;
    if (full || a_k < kleft)
      sload_lds_16B(Ag + (size_t)(TC::ROWS_PER_LOAD * i) * K, a_off * 2u, lds_addr + (wave + i * TC::NW) * 1024);
    else
      *(i32x4 LLMMM_LDS*)(dst + lane * 16) = i32x4{0, 0, 0, 0};
  }
  char LLMMM_LDS* ldsB = lds + TC::A_BYTES;
#pragma unroll
  for (int i = 0; i < TC::B_LOADS; ++i) {
    char LLMMM_LDS* dst = ldsB + (wave + i * TC::NW) * 1024;
    if constexpr (B_NK) {
      if (full || b_k < kleft)
        sload_lds_16B(Bg + (size_t)(TC::ROWS_PER_LOAD * i) * K, b_off * 2u, lds_addr + TC::A_BYTES + (wave + i * TC::NW) * 1024);
      else
        *(i32x4 LLMMM_LDS*)(dst + lane * 16) = i32x4{0, 0, 0, 0};
    }
    else {
      if (full || b_k + TC::B_KROWS_PER_LOAD * i < kleft)
        sload_lds_16B(Bg + (size_t)(TC::B_KROWS_PER_LOAD * i) * N, b_off * 2u, lds_addr + TC::A_BYTES + (wave + i * TC::NW) * 1024);
      else
        *(i32x4 LLMMM_LDS*)(dst + lane * 16) = i32x4{0, 0, 0, 0};
    }
  }
}

// Operand fragments of one 16-wide k-step (ks = 0 or 1 inside a stage): a[mf] = 32 rows of A,
// b[nf] = 32 rows of B^T.
template <typename T, int BM, int BN, bool B_NK>
__device__ __forceinline__ void fp16_read_frags(const char LLMMM_LDS* lds, int a_rd, const int (&b_rd)[4], int ks,
                                                typename Mfma16<T>::vec (&a)[2], typename Mfma16<T>::vec (&b)[4])
{
  typedef Fp16Tile<T, BM, BN, B_NK> TC;
  typedef typename Mfma16<T>::vec   vec;
  const char LLMMM_LDS*             ldsA = lds;
  const char LLMMM_LDS*             ldsB = lds + TC::A_BYTES;
#pragma unroll
  for (int mf = 0; mf < 2; ++mf) a[mf] = *(const vec LLMMM_LDS*)(ldsA + (a_rd ^ (ks << 5)) + mf * 2048);
#pragma unroll
  for (int nf = 0; nf < 4; ++nf) {
    if constexpr (B_NK) {
      b[nf] = *(const vec LLMMM_LDS*)(ldsB + (b_rd[0] ^ (ks << 5)) + nf * 2048);
    }
    else {
      union {
        i16x4 h[2];
        vec   v;
      } u;
      u.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((i16x4 LLMMM_LDS*)(ldsB + b_rd[nf] + (ks * 16) * TC::B_ROW));
      u.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((i16x4 LLMMM_LDS*)(ldsB + b_rd[nf] + (ks * 16 + 4) * TC::B_ROW));
      b[nf]  = u.v;
    }
  }
}

// Half of a k-step: the 4 MFMAs of fragments nf = 2h, 2h+1.
template <typename T>
__device__ __forceinline__ void fp16_mfma_half(int h, const typename Mfma16<T>::vec (&a)[2], const typename Mfma16<T>::vec (&b)[4],
                                               f32x16 (&acc)[4][2])
{
#pragma unroll
  for (int nf = 2 * h; nf < 2 * h + 2; ++nf)
#pragma unroll
    for (int mf = 0; mf < 2; ++mf) acc[nf][mf] = Mfma16<T>::run(b[nf], a[mf], acc[nf][mf]);
}

template <typename T, int BM, int BN, bool B_NK, bool KTAIL>
__global__ void __launch_bounds__((BM / 64) * (BN / 128) * 64)
fp16_gemm_kernel(const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C, int M, int N, int K, int tiles_m, int tiles_n)
{
  typedef Fp16Tile<T, BM, BN, B_NK> TC;
  typedef typename Mfma16<T>::vec   vec;
  __shared__ __attribute__((aligned(1024))) char lds_raw[4 * TC::STAGE];  // the ring of four stages

  const int tid  = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm   = wave % TC::WAVES_M;
  const int wn   = wave / TC::WAVES_M;
  int       tm, tn;
  tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;

  // ---- loader setup
  const KMajorLane lp    = kmajor_lane<SWZ_ROW64>(wave, lane);
  const unsigned   a_off = (unsigned)(lp.row * K + lp.chunk * 8);
  const int        a_k   = lp.chunk * 8;
  unsigned         b_off;
  int              b_k;
  if constexpr (B_NK) {
    b_off = a_off;
    b_k   = a_k;
  }
  else {
    const int k     = wave * TC::B_KROWS_PER_GRP + (lane * 16) / TC::B_ROW;
    const int pbyte = (lane * 16) % TC::B_ROW;
    const int ch    = (pbyte >> 6) ^ (k & 3);
    b_off           = (unsigned)(k * N + ((ch << 6) + (pbyte & 63)) / 2);
    b_k             = k;
  }
  const T* Ag = A + (size_t)m0 * K;
  const T* Bg = B_NK ? B + (size_t)n0 * K : B + n0;

  // ---- operand read setup (byte offsets inside a stage)
  const int hi   = lane >> 5;
  const int a_rd = kmajor_offset<SWZ_ROW64>(wm * 64 + (lane & 31), hi);
  int       b_rd[4];
  if constexpr (B_NK) {
    b_rd[0] = kmajor_offset<SWZ_ROW64>(wn * 128 + (lane & 31), hi);
    b_rd[1] = b_rd[2] = b_rd[3] = 0;
  }
  else {
    const int blk = lane >> 4, i = lane & 15;
#pragma unroll
    for (int nf = 0; nf < 4; ++nf)
      b_rd[nf] = (8 * (blk >> 1) + (i >> 2)) * TC::B_ROW + (((wn * 4 + nf) ^ (i >> 2)) << 6) + (blk & 1) * 32 + (i & 3) * 8;
  }

  f32x16 acc[4][2];
#pragma unroll
  for (int nf = 0; nf < 4; ++nf)
#pragma unroll
    for (int mf = 0; mf < 2; ++mf)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[nf][mf][r] = 0.0f;

  const int    KT          = (K + TC::BK - 1) / TC::BK;
  const int    full_stages = K / TC::BK;
  const size_t b_step      = B_NK ? (size_t)TC::BK : (size_t)TC::BK * N;

  char LLMMM_LDS* const lds      = (char LLMMM_LDS*)lds_raw;
  char LLMMM_LDS* const ring[4]  = {lds, lds + TC::STAGE, lds + 2 * TC::STAGE, lds + 3 * TC::STAGE};
  const unsigned        lds_base = (unsigned)(size_t)lds;  // the same buffers as LDS byte addresses, for the loader
  const unsigned ring_addr[4]    = {lds_base, lds_base + TC::STAGE, lds_base + 2 * TC::STAGE, lds_base + 3 * TC::STAGE};

#define LLMMM_ISSUE(stage, buf)                                                                                              \
  fp16_issue_stage<T, BM, BN, B_NK, KTAIL>(ring[buf], ring_addr[buf], Ag + (size_t)(stage) * TC::BK, Bg + (size_t)(stage) * b_step, a_off, a_k, b_off, \
                                    b_k, K, N, wave, lane, K - (stage) * TC::BK)

  // prologue: stages 0..2 in flight, stage 0 landed and published, then stage 3 behind the barrier
  LLMMM_ISSUE(0, 0);
  if (1 < KT) LLMMM_ISSUE(1, 1);
  if (2 < KT) LLMMM_ISSUE(2, 2);
  wait_vmcnt<0>();
  __builtin_amdgcn_s_barrier();
  if (3 < KT) LLMMM_ISSUE(3, 3);

  vec a0[2], b0[4], a1[2], b1[4];
  fp16_read_frags<T, BM, BN, B_NK>(ring[0], a_rd, b_rd, 0, a0, b0);

  // One stage s (in ring[u]).  STEADY = "stages s+1 .. s+4 exist and are full" (straight-line code).
  // The LDS reads of the next k-step are issued between the two MFMA halves of the current one:
  // by the time their data is needed four MFMAs (>= 128 cycles) have been issued behind them.
  // (While LDS-direct loads are in flight the compiler only ever waits for *all* LDS reads, so a
  // read must never be issued right before a wait.)
#define LLMMM_STAGE(STEADY, s, u)                                                                                  \
  {                                                                                                                \
    fp16_mfma_half<T>(0, a0, b0, acc);                                                                             \
    __builtin_amdgcn_sched_barrier(0);                                                                             \
    fp16_read_frags<T, BM, BN, B_NK>(ring[u], a_rd, b_rd, 1, a1, b1);                                              \
    __builtin_amdgcn_sched_barrier(0);                                                                             \
    fp16_mfma_half<T>(1, a0, b0, acc);                                                                             \
    __builtin_amdgcn_sched_barrier(0);                                                                             \
    /* every LDS read of stage s has been issued; once they are back (lgkmcnt(0), part of each wait below) the */ \
    /* barrier hands ring[u] to the loader and publishes stage s+1 */                                             \
    if (STEADY || (s) + 3 < full_stages)                                                                           \
      wait_vmcnt<2 * TC::LOADS>(); /* stages s+2 and s+3 may still be in flight */                                 \
    else if ((s) + 2 < full_stages)                                                                                \
      wait_vmcnt<TC::LOADS>();                                                                                     \
    else                                                                                                           \
      wait_vmcnt<0>();                                                                                             \
    __builtin_amdgcn_s_barrier();                                                                                  \
    if (STEADY || (s) + 4 < KT) LLMMM_ISSUE((s) + 4, u);                                                           \
    fp16_mfma_half<T>(0, a1, b1, acc);                                                                             \
    __builtin_amdgcn_sched_barrier(0);                                                                             \
    /* unconditional: after the last stage this reads a stale buffer and the result is unused */                  \
    fp16_read_frags<T, BM, BN, B_NK>(ring[((u) + 1) & 3], a_rd, b_rd, 0, a0, b0);                                  \
    __builtin_amdgcn_sched_barrier(0);                                                                             \
    fp16_mfma_half<T>(1, a1, b1, acc);                                                                             \
    __builtin_amdgcn_sched_barrier(0);                                                                             \
  }

  int kt = 0;
  for (; kt + 8 <= full_stages; kt += 4) {
    LLMMM_STAGE(true, kt + 0, 0)
    LLMMM_STAGE(true, kt + 1, 1)
    LLMMM_STAGE(true, kt + 2, 2)
    LLMMM_STAGE(true, kt + 3, 3)
  }
  for (; kt < KT; kt += 4) {
    if (kt + 0 < KT) LLMMM_STAGE(false, kt + 0, 0)
    if (kt + 1 < KT) LLMMM_STAGE(false, kt + 1, 1)
    if (kt + 2 < KT) LLMMM_STAGE(false, kt + 2, 2)
    if (kt + 3 < KT) LLMMM_STAGE(false, kt + 3, 3)
  }
#undef LLMMM_STAGE
#undef LLMMM_ISSUE

  // ---- epilogue: lane holds, for row m = ..+lane%32, the columns 8*(r/4) + 4*(lane/32) + r%4.
  // Stored straight from this layout, one instruction would write 16 bytes to each of 32 rows,
  // and the memory pipeline pays per row segment.  Instead every wave lays its 64 x 128 result
  // out row-major (256-byte rows, 16-byte chunks XOR-ed with the row so that the ds_read_b128
  // below is conflict-free) in a private 16 KB piece of the ring and stores whole rows, 16
  // bytes per lane.  Behind the last stage's barrier no wave reads operands any more and every
  // load has landed, so the ring is free.
  {
    typedef T             tx4 __attribute__((ext_vector_type(4)));
    char LLMMM_LDS* const stg = lds + wave * 16384;
#pragma unroll
    for (int mf = 0; mf < 2; ++mf) {
      const int r = mf * 32 + (lane & 31);
#pragma unroll
      for (int nf = 0; nf < 4; ++nf)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const f32x16& v = acc[nf][mf];
          tx4           o;
          o[0] = (T)v[4 * q + 0];
          o[1] = (T)v[4 * q + 1];
          o[2] = (T)v[4 * q + 2];
          o[3] = (T)v[4 * q + 3];
          *(tx4 LLMMM_LDS*)(stg + r * 256 + (((nf * 4 + q) ^ (r & 15)) << 4) + 8 * hi) = o;
        }
    }
    T* cbase = C + (size_t)(m0 + wm * 64) * N + n0 + wn * 128;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const int   r = 4 * j + (lane >> 4), ch = lane & 15;
      const i32x4 v = *(const i32x4 LLMMM_LDS*)(stg + r * 256 + ((ch ^ (r & 15)) << 4));
      *(i32x4*)(cbase + (size_t)r * N + ch * 8) = v;
    }
  }
}

// --------------------------------------------------------------------------------------------- host
template <typename T, int BM, int BN, bool B_NK>
static hipError_t launch_fp16(const void* A, const void* B, void* C, int M, int N, int K, hipStream_t stream)
{
  typedef Fp16Tile<T, BM, BN, B_NK> TC;
  const int tiles_m = M / BM, tiles_n = N / BN;
  if (K % TC::BK)
    hipLaunchKernelGGL((fp16_gemm_kernel<T, BM, BN, B_NK, true>), dim3(tiles_m * tiles_n), dim3(TC::NT), 0, stream, (const T*)A,
                       (const T*)B, (T*)C, M, N, K, tiles_m, tiles_n);
  else
    hipLaunchKernelGGL((fp16_gemm_kernel<T, BM, BN, B_NK, false>), dim3(tiles_m * tiles_n), dim3(TC::NT), 0, stream, (const T*)A,
                       (const T*)B, (T*)C, M, N, K, tiles_m, tiles_n);
  return hipGetLastError();
}

template <typename T, bool B_NK>
static hipError_t dispatch_fp16(int tile, const void* A, const void* B, void* C, int M, int N, int K, hipStream_t stream)
{
  switch (tile) {
    case LLMMM_TILE_256x256: return launch_fp16<T, 256, 256, B_NK>(A, B, C, M, N, K, stream);
    case LLMMM_TILE_128x256: return launch_fp16<T, 128, 256, B_NK>(A, B, C, M, N, K, stream);
    case LLMMM_TILE_256x128: return launch_fp16<T, 256, 128, B_NK>(A, B, C, M, N, K, stream);
    case LLMMM_TILE_128x128: return launch_fp16<T, 128, 128, B_NK>(A, B, C, M, N, K, stream);
    default: return hipErrorInvalidValue;
  }
}

hipError_t fp16_gemm_launch(int dtype, int b_layout, int tile, const void* A, const void* B, void* C, int M, int N, int K,
                            hipStream_t stream)
{
  if (dtype == 0)
    return b_layout ? dispatch_fp16<_Float16, true>(tile, A, B, C, M, N, K, stream)
                    : dispatch_fp16<_Float16, false>(tile, A, B, C, M, N, K, stream);
  return b_layout ? dispatch_fp16<__bf16, true>(tile, A, B, C, M, N, K, stream)
                  : dispatch_fp16<__bf16, false>(tile, A, B, C, M, N, K, stream);
}

}  // namespace llmmm
