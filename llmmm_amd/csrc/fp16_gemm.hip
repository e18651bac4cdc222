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
//  * K advances 64 elements (128 bytes per tile row) per stage; two LDS stages are filled by
//    LDS-direct global loads (no staging registers, no ds_write) while the other one is consumed;
//  * A (and Bt) tiles are K-major and read with ds_read_b128 through the XOR swizzle of
//    device_common.hip.h; a row-major B tile is kept as [k][n] and read with the transposing
//    ds_read_b64_tr_b16, its 64-byte column chunks XOR-ed with k&3;
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

// Logical tile id -> (tm, tn).  Hardware hands consecutive workgroup ids to the 8 XCDs in turn,
// so ids congruent mod 8 share an L2: give each XCD a contiguous run of the grouped order
// (GROUP_M tile rows swept along n), whose members reuse the same few A and B panels.
__device__ __forceinline__ void tile_coords(int wg, int tiles_m, int tiles_n, int& tm, int& tn)
{
  const int tiles = tiles_m * tiles_n;
  int       L     = wg;
  if ((tiles & 7) == 0) L = (wg & 7) * (tiles >> 3) + (wg >> 3);
  constexpr int GROUP_M = 4;
  const int     per     = GROUP_M * tiles_n;
  const int     group   = L / per;
  const int     first   = group * GROUP_M;
  const int     gm      = (tiles_m - first) < GROUP_M ? (tiles_m - first) : GROUP_M;
  const int     in      = L - group * per;
  tm                    = first + in % gm;
  tn                    = in / gm;
}

template <typename T, int BM, int BN, bool B_NK>
struct Fp16Tile {
  static constexpr int WAVES_M = BM / 64;
  static constexpr int WAVES_N = BN / 128;
  static constexpr int NW      = WAVES_M * WAVES_N;
  static constexpr int NT      = NW * 64;
  static constexpr int BK      = 64;             // elements of K per stage
  static constexpr int A_BYTES = BM * 128;       // K-major, 128 bytes per row
  static constexpr int B_BYTES = BN * 128;       // either layout: 64 x BN x 2 bytes
  static constexpr int B_ROW   = BN * 2;         // row pitch of the [k][n] layout
  static constexpr int STAGE   = A_BYTES + B_BYTES;
  static constexpr int A_LOADS = (BM / 8) / NW;  // 1024-byte groups per wave
  static constexpr int B_LOADS = (B_BYTES / 1024) / NW;
};

// Issue the LDS-direct loads of one stage.  `kleft` = K - k0 (elements still to go); a stage
// whose K range is cut short zero-fills the missing part so that the MFMAs need no masking.
template <typename T, int BM, int BN, bool B_NK>
__device__ __forceinline__ void fp16_issue_stage(char LLMMM_LDS* lds, const T* __restrict__ Ag, const T* __restrict__ Bg,
                                                 const int (&a_off)[Fp16Tile<T, BM, BN, B_NK>::A_LOADS],
                                                 const int (&a_chunk)[Fp16Tile<T, BM, BN, B_NK>::A_LOADS],
                                                 const int (&b_off)[Fp16Tile<T, BM, BN, B_NK>::B_LOADS],
                                                 const int (&b_kc)[Fp16Tile<T, BM, BN, B_NK>::B_LOADS], int wave, int lane,
                                                 int kleft)
{
  typedef Fp16Tile<T, BM, BN, B_NK> TC;
  const bool full = kleft >= TC::BK;
#pragma unroll
  for (int i = 0; i < TC::A_LOADS; ++i) {
    const int         g   = wave + i * TC::NW;
    char LLMMM_LDS*   dst = lds + g * 1024;
    if (full || a_chunk[i] * 8 < kleft)
      load_lds_16B(Ag + a_off[i], dst);
    else
      *(i32x4 LLMMM_LDS*)(dst + lane * 16) = i32x4{0, 0, 0, 0};
  }
  char LLMMM_LDS* ldsB = lds + TC::A_BYTES;
#pragma unroll
  for (int i = 0; i < TC::B_LOADS; ++i) {
    const int       g   = wave + i * TC::NW;
    char LLMMM_LDS* dst = ldsB + g * 1024;
    // b_kc: K-major layout -> first k of the lane's chunk; [k][n] layout -> the lane's k row
    if (full || b_kc[i] < kleft)
      load_lds_16B(Bg + b_off[i], dst);
    else
      *(i32x4 LLMMM_LDS*)(dst + lane * 16) = i32x4{0, 0, 0, 0};
  }
}

// Operand fragments of one 16-wide k-step: a[mf] = 32 rows of A, b[nf] = 32 rows of B^T.
template <typename T, int BM, int BN, bool B_NK>
__device__ __forceinline__ void fp16_read_frags(const char LLMMM_LDS* ldsA, const char LLMMM_LDS* ldsB, const int (&a_rd)[2],
                                                const int (&b_rd)[4], int ks, typename Mfma16<T>::vec (&a)[2],
                                                typename Mfma16<T>::vec (&b)[4])
{
  typedef Fp16Tile<T, BM, BN, B_NK> TC;
  typedef typename Mfma16<T>::vec   vec;
#pragma unroll
  for (int mf = 0; mf < 2; ++mf) a[mf] = *(const vec LLMMM_LDS*)(ldsA + (a_rd[mf] ^ (ks << 5)));
#pragma unroll
  for (int nf = 0; nf < 4; ++nf) {
    if constexpr (B_NK) {
      b[nf] = *(const vec LLMMM_LDS*)(ldsB + (b_rd[nf] ^ (ks << 5)));
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

// One stage = four k-steps; the fragments of step ks+1 are fetched while step ks multiplies.
template <typename T, int BM, int BN, bool B_NK>
__device__ __forceinline__ void fp16_compute_stage(const char LLMMM_LDS* lds, const int (&a_rd)[2], const int (&b_rd)[4],
                                                   f32x16 (&acc)[4][2])
{
  typedef Fp16Tile<T, BM, BN, B_NK> TC;
  typedef typename Mfma16<T>::vec   vec;
  const char LLMMM_LDS*             ldsA = lds;
  const char LLMMM_LDS*             ldsB = lds + TC::A_BYTES;
  vec                               a[2][2], b[2][4];
  fp16_read_frags<T, BM, BN, B_NK>(ldsA, ldsB, a_rd, b_rd, 0, a[0], b[0]);
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) {
    const int cur = ks & 1;
    if (ks + 1 < 4) fp16_read_frags<T, BM, BN, B_NK>(ldsA, ldsB, a_rd, b_rd, ks + 1, a[cur ^ 1], b[cur ^ 1]);
    __builtin_amdgcn_sched_barrier(0);  // all reads of step ks+1 are in flight before step ks multiplies
#pragma unroll
    for (int nf = 0; nf < 4; ++nf)
#pragma unroll
      for (int mf = 0; mf < 2; ++mf) acc[nf][mf] = Mfma16<T>::run(b[cur][nf], a[cur][mf], acc[nf][mf]);
    __builtin_amdgcn_sched_barrier(0);
  }
}

template <typename T, int BM, int BN, bool B_NK>
__global__ void __launch_bounds__((BM / 64) * (BN / 128) * 64)
fp16_gemm_kernel(const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C, int M, int N, int K, int tiles_m, int tiles_n)
{
  typedef Fp16Tile<T, BM, BN, B_NK> TC;
  __shared__ __attribute__((aligned(1024))) char lds0[TC::STAGE];
  __shared__ __attribute__((aligned(1024))) char lds1[TC::STAGE];

  const int tid  = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm   = wave % TC::WAVES_M;
  const int wn   = wave / TC::WAVES_M;
  int       tm, tn;
  tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;

  // ---- loader setup: element offsets (relative to the tile's first row / column) per load
  int a_off[TC::A_LOADS], a_chunk[TC::A_LOADS], b_off[TC::B_LOADS], b_kc[TC::B_LOADS];
#pragma unroll
  for (int i = 0; i < TC::A_LOADS; ++i) {
    const KMajorLane p = kmajor_lane<SWZ_ROWS32>(wave + i * TC::NW, lane);
    a_off[i]           = p.row * K + p.chunk * 8;
    a_chunk[i]         = p.chunk;
  }
#pragma unroll
  for (int i = 0; i < TC::B_LOADS; ++i) {
    const int g = wave + i * TC::NW;
    if constexpr (B_NK) {
      const KMajorLane p = kmajor_lane<SWZ_ROWS32>(g, lane);
      b_off[i]           = p.row * K + p.chunk * 8;
      b_kc[i]            = p.chunk * 8;
    }
    else {
      constexpr int ROWS_PER_GROUP = 1024 / TC::B_ROW;
      const int     k              = g * ROWS_PER_GROUP + (lane * 16) / TC::B_ROW;
      const int     pbyte          = (lane * 16) % TC::B_ROW;
      const int     ch             = (pbyte >> 6) ^ (k & 3);
      b_off[i]                     = k * N + ((ch << 6) + (pbyte & 63)) / 2;
      b_kc[i]                      = k;
    }
  }
  const T* Ag = A + (size_t)m0 * K;
  const T* Bg = B_NK ? B + (size_t)n0 * K : B + n0;

  // ---- operand read setup (byte offsets inside a stage)
  int a_rd[2], b_rd[4];
  const int hi = lane >> 5;
#pragma unroll
  for (int mf = 0; mf < 2; ++mf) {
    const int r = wm * 64 + mf * 32 + (lane & 31);
    a_rd[mf]    = kmajor_phys_row<SWZ_ROWS32>(r) * 128 + ((hi ^ kmajor_swz<SWZ_ROWS32>(r)) << 4);
  }
#pragma unroll
  for (int nf = 0; nf < 4; ++nf) {
    if constexpr (B_NK) {
      const int r = wn * 128 + nf * 32 + (lane & 31);
      b_rd[nf]    = kmajor_phys_row<SWZ_ROWS32>(r) * 128 + ((hi ^ kmajor_swz<SWZ_ROWS32>(r)) << 4);
    }
    else {
      const int blk = lane >> 4, i = lane & 15;
      const int ch  = wn * 4 + nf;
      b_rd[nf] = (8 * (blk >> 1) + (i >> 2)) * TC::B_ROW + ((ch ^ (i >> 2)) << 6) + (blk & 1) * 32 + (i & 3) * 8;
    }
  }

  f32x16 acc[4][2];
#pragma unroll
  for (int nf = 0; nf < 4; ++nf)
#pragma unroll
    for (int mf = 0; mf < 2; ++mf)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[nf][mf][r] = 0.0f;

  const int    KT      = (K + TC::BK - 1) / TC::BK;
  const size_t b_step  = B_NK ? (size_t)TC::BK : (size_t)TC::BK * N;
  char LLMMM_LDS* const s0 = (char LLMMM_LDS*)lds0;
  char LLMMM_LDS* const s1 = (char LLMMM_LDS*)lds1;

  fp16_issue_stage<T, BM, BN, B_NK>(s0, Ag, Bg, a_off, a_chunk, b_off, b_kc, wave, lane, K);
  for (int kt = 0; kt < KT; kt += 2) {
    // even stage: data in lds0, prefetch into lds1
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0), lgkmcnt(0): this wave's loads / zero-fills have landed
    __syncthreads();
    if (kt + 1 < KT)
      fp16_issue_stage<T, BM, BN, B_NK>(s1, Ag + (size_t)(kt + 1) * TC::BK, Bg + (size_t)(kt + 1) * b_step, a_off, a_chunk, b_off,
                                        b_kc, wave, lane, K - (kt + 1) * TC::BK);
    fp16_compute_stage<T, BM, BN, B_NK>(s0, a_rd, b_rd, acc);
    if (kt + 1 < KT) {
      __builtin_amdgcn_s_waitcnt(0x0070);
      __syncthreads();
      if (kt + 2 < KT)
        fp16_issue_stage<T, BM, BN, B_NK>(s0, Ag + (size_t)(kt + 2) * TC::BK, Bg + (size_t)(kt + 2) * b_step, a_off, a_chunk,
                                          b_off, b_kc, wave, lane, K - (kt + 2) * TC::BK);
      fp16_compute_stage<T, BM, BN, B_NK>(s1, a_rd, b_rd, acc);
    }
  }

  // ---- epilogue: lane holds, for row m = ..+lane%32, the columns 8*(r/4) + 4*(lane/32) + r%4
  const int m = m0 + wm * 64 + (lane & 31);
#pragma unroll
  for (int mf = 0; mf < 2; ++mf) {
    T* crow = C + (size_t)(m + mf * 32) * N + n0 + wn * 128 + 4 * hi;
#pragma unroll
    for (int nf = 0; nf < 4; ++nf)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        typedef T       tx4 __attribute__((ext_vector_type(4)));
        const f32x16&   v = acc[nf][mf];
        tx4             o;
        o[0] = (T)v[4 * q + 0];
        o[1] = (T)v[4 * q + 1];
        o[2] = (T)v[4 * q + 2];
        o[3] = (T)v[4 * q + 3];
        *(tx4*)(crow + nf * 32 + q * 8) = o;
      }
  }
}

// --------------------------------------------------------------------------------------------- host
template <typename T, int BM, int BN, bool B_NK>
static hipError_t launch_fp16(const void* A, const void* B, void* C, int M, int N, int K, hipStream_t stream)
{
  typedef Fp16Tile<T, BM, BN, B_NK> TC;
  const int tiles_m = M / BM, tiles_n = N / BN;
  hipLaunchKernelGGL((fp16_gemm_kernel<T, BM, BN, B_NK>), dim3(tiles_m * tiles_n), dim3(TC::NT), 0, stream, (const T*)A,
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
