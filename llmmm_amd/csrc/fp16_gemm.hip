// FP16 / BF16 GEMM for gfx950:  C[M,N] = A[M,K] * B,  fp32 accumulation, output rounded to T.
//
// Replaces the kernel behind LLMMM::fp16_mm<T> (reference: src/mm/fp16/mm.cu:6-42 launching
// src/mm/fp16/mm.cuh:657-684).  Layouts follow the reference: A[m*K+k] (mm.cuh:102),
// B[k*N+n] (mm.cuh:103), C[m*N+n] (mm.cuh:236).  A second B layout, Bt[n*K+k], is an extension.
//
// Design (nothing here is translated from the reference's mma.sync/ldmatrix code):
//  * one workgroup computes a BM x BN tile, one wavefront a 64(m) x 128(n) sub-tile built from
//    v_mfma_f32_16x16x32_{f16,bf16}.  On this power-limited part the 16x16x32 shape sustains
//    about 16 % more FLOP/s than 32x32x16 on random operands (same peak, less energy per
//    FLOP), which is why it is used although it needs twice the instructions.  The MFMA is
//    issued with B as the row operand and A as the column operand, so that each lane ends up
//    with 4 consecutive n of one row m;
//  * K advances 32 elements per stage = one MFMA k-step (64 bytes per tile row, (BM+BN)*64 bytes
//    of LDS) and four stages form a ring that LDS-direct global loads fill three stages ahead
//    of the MFMAs (no staging registers, no ds_write);
//  * the single workgroup barrier of a stage sits in its middle, between the MFMAs of the wave's
//    left and right 64 columns: by then every wave has pulled the stage's operands into
//    registers, so the barrier both frees the stage's buffer for the load of stage +4 and
//    publishes stage +1, whose first fragments are fetched right behind it -- no wave ever waits
//    on an LDS read it has just issued;
//  * A (and Bt) tiles are K-major and read with one ds_read_b128 per 16-row fragment (chunk
//    XOR-ed with row bit 3: conflict-free); a row-major B tile is kept as [k][n] and read with
//    the transposing ds_read_b64_tr_b16, its 32-byte column chunks XOR-ed with k bits 0, 1, 3;
//  * the epilogue lays each wave's result out row-major in LDS and stores whole rows;
//  * workgroup ids are remapped so that the tiles resident on one XCD share A/B panels in its L2.
#include "device_common.hip.h"
#include "kernels.h"

namespace llmmm {

template <typename T>
struct Mfma32;
template <>
struct Mfma32<_Float16> {
  typedef f16x8 vec;
  static __device__ __forceinline__ f32x4 run(vec x, vec y, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(x, y, c, 0, 0, 0); }
};
template <>
struct Mfma32<__bf16> {
  typedef bf16x8 vec;
  static __device__ __forceinline__ f32x4 run(vec x, vec y, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(x, y, c, 0, 0, 0); }
};

// WM = rows of a wave's sub-tile (64, 32 or 16); its columns are always 128.
template <typename T, int BM, int BN, int WM, bool B_NK>
struct Fp16Tile {
  static constexpr int MF      = WM / 16;  // 16-row fragments per wave
  static constexpr int WAVES_M = BM / WM;
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

// K-major tile of 64-byte rows read as 16-row fragments: lanes 16g..16g+15 take 16 consecutive
// rows at chunk g.  Four rows fill a 256-byte bank row; XOR-ing row bit 3 into chunk bit 1 keeps
// the 16 lanes of every ds_read_b128 pass on 16 different 16-byte slots.
__device__ __forceinline__ int k64_swz(int r) { return ((r >> 3) & 1) << 1; }
__device__ __forceinline__ int k64_offset(int r, int c) { return r * 64 + ((c ^ k64_swz(r)) << 4); }
// [k][n] tile: the 32-byte column chunk of row k is XOR-ed with k bits 0, 1 and 3, which keeps
// the 4 x 4 row/chunk patches of a transposing 64-bit read on different banks.
__device__ __forceinline__ int kn_swz(int k) { return (k & 3) | (((k >> 3) & 1) << 2); }

// LDS-direct load as inline assembly with the wave-uniform part of the address in SGPRs: no
// vector ALU work goes into addresses, and the compiler -- which would turn every wait it
// inserts into "all loads done" while it knows of an LDS-direct load in flight -- never sees
// it; the kernel places the s_waitcnt vmcnt itself.
__device__ __forceinline__ void sload_lds_16B(const void* sbase, unsigned voff, unsigned lds_addr)
{
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "s"(lds_addr) : "memory");
}

// Per-lane loader state.  The loads of a wave for the K-major tiles share one byte offset (they
// differ by a wave-uniform row step that the swizzle does not see); those of the [k][n] tile
// get one offset each, because their k step may flip the swizzle.
template <int B_LOADS>
struct Fp16Loader {
  unsigned a_off;          // bytes
  int      a_k;            // k offset (elements) of the lane's chunk inside a stage
  unsigned b_off[B_LOADS]; // bytes
  int      b_k[B_LOADS];   // K-major: k offset of the chunk; [k][n]: k row of the lane
};

// Issue the LDS-direct loads of one stage.  `kleft` = K - k0 (elements still to go); a stage
// whose K range is cut short zero-fills the missing part so that the MFMAs need no masking.
template <typename T, int BM, int BN, int WM, bool B_NK, bool KTAIL>
__device__ __forceinline__ void fp16_issue_stage(char LLMMM_LDS* lds, unsigned lds_addr, const T* __restrict__ Ag, const T* __restrict__ Bg,
                                                 const Fp16Loader<Fp16Tile<T, BM, BN, WM, B_NK>::B_LOADS>& ld, int K, int N, int wave, int lane,
                                                 int kleft)
{
  typedef Fp16Tile<T, BM, BN, WM, B_NK> TC;
  // without a K tail (K % 32 == 0) the loads are unconditional straight-line code
  const bool full = !KTAIL || kleft >= TC::BK;
#pragma unroll
  for (int i = 0; i < TC::A_LOADS; ++i) {
    if (full || ld.a_k < kleft)
      sload_lds_16B(Ag + (size_t)(TC::ROWS_PER_LOAD * i) * K, ld.a_off, lds_addr + (wave + i * TC::NW) * 1024);
    else
      *(i32x4 LLMMM_LDS*)(lds + (wave + i * TC::NW) * 1024 + lane * 16) = i32x4{0, 0, 0, 0};
  }
#pragma unroll
  for (int i = 0; i < TC::B_LOADS; ++i) {
    const unsigned dst = TC::A_BYTES + (wave + i * TC::NW) * 1024;
    if (full || ld.b_k[i] < kleft) {
      if constexpr (B_NK)
        sload_lds_16B(Bg + (size_t)(TC::ROWS_PER_LOAD * i) * K, ld.b_off[i], lds_addr + dst);
      else
        sload_lds_16B(Bg + (size_t)(TC::B_KROWS_PER_LOAD * i) * N, ld.b_off[i], lds_addr + dst);
    }
    else
      *(i32x4 LLMMM_LDS*)(lds + dst + lane * 16) = i32x4{0, 0, 0, 0};
  }
}

// The 16-row A fragments of a stage.
template <typename T, int MF>
__device__ __forceinline__ void fp16_read_a(const char LLMMM_LDS* lds, int a_rd, typename Mfma32<T>::vec (&a)[MF])
{
  typedef typename Mfma32<T>::vec vec;
#pragma unroll
  for (int mf = 0; mf < MF; ++mf) a[mf] = *(const vec LLMMM_LDS*)(lds + a_rd + mf * 1024);
}
// Four 16-column B fragments: nf = 4*half .. 4*half+3.
template <typename T, int BM, int BN, int WM, bool B_NK>
__device__ __forceinline__ void fp16_read_b(const char LLMMM_LDS* lds, const int (&b_rd)[8], int half, typename Mfma32<T>::vec (&b)[4])
{
  typedef Fp16Tile<T, BM, BN, WM, B_NK> TC;
  typedef typename Mfma32<T>::vec   vec;
  const char LLMMM_LDS*             ldsB = lds + TC::A_BYTES;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int nf = 4 * half + q;
    if constexpr (B_NK) {
      b[q] = *(const vec LLMMM_LDS*)(ldsB + b_rd[0] + nf * 1024);
    }
    else {
      union {
        i16x4 h[2];
        vec   v;
      } u;
      u.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((i16x4 LLMMM_LDS*)(ldsB + b_rd[nf]));
      u.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((i16x4 LLMMM_LDS*)(ldsB + b_rd[nf] + 4 * TC::B_ROW));
      b[q]   = u.v;
    }
  }
}

// 2 * MF MFMAs: fragments nf = 4*half + 2*part, +1 against the wave's row fragments.
template <typename T, int MF>
__device__ __forceinline__ void fp16_mfma8(int half, int part, const typename Mfma32<T>::vec (&a)[MF], const typename Mfma32<T>::vec (&b)[4],
                                           f32x4 (&acc)[8][MF])
{
#pragma unroll
  for (int q = 2 * part; q < 2 * part + 2; ++q)
#pragma unroll
    for (int mf = 0; mf < MF; ++mf) acc[4 * half + q][mf] = Mfma32<T>::run(b[q], a[mf], acc[4 * half + q][mf]);
}

// The kernel's body for tile `tile_index` of the tiles_m x tiles_n tiles of the column range that starts at n_base (0 and
// the whole matrix for the plain kernel); lds_raw: the workgroup's ring of four stages.
// STAMP: the phase-accounting build -- clock readings at five points of every wave, stored to `stamps` at the end.
template <typename T, int BM, int BN, int WM, bool B_NK, bool KTAIL, bool STAMP = false>
__device__ __forceinline__ void fp16_gemm_body(const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C, int M, int N, int K, int tiles_m,
                                               int tiles_n, char LLMMM_LDS* lds_raw, int tile_index, int n_base, unsigned long long* stamps = nullptr)
{
  typedef Fp16Tile<T, BM, BN, WM, B_NK> TC;
  typedef typename Mfma32<T>::vec   vec;
  constexpr int                     MF = TC::MF;
  PhaseClock                        ph[STAMP ? PHASE_POINTS : 1];
  unsigned long long                wait_cycles = 0, load_wait_cycles = 0;  // STAMP: shader cycles in the K loop's "loads landed + barrier" waits; of which for the loads
  if constexpr (STAMP) ph[0] = phase_clock();

  const int tid  = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm   = wave % TC::WAVES_M;
  const int wn   = wave / TC::WAVES_M;
  int       tm, tn;
  tile_coords(tile_index, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = n_base + tn * BN;

  // ---- loader setup: lane -> what the 16 bytes at (1 KB group base + 16*lane) must hold
  Fp16Loader<TC::B_LOADS> ld;
  {
    const int r = wave * 16 + (lane >> 2);          // tile row of the first group; later groups add 16*NW rows
    const int c = (lane & 3) ^ k64_swz(r);          // logical chunk placed at physical chunk lane%4
    ld.a_off    = (unsigned)(r * K + c * 8) * 2u;
    ld.a_k      = c * 8;
#pragma unroll
    for (int i = 0; i < TC::B_LOADS; ++i) {
      if constexpr (B_NK) {
        ld.b_off[i] = ld.a_off;
        ld.b_k[i]   = ld.a_k;
      }
      else {
        const int k     = (wave + i * TC::NW) * TC::B_KROWS_PER_GRP + (lane * 16) / TC::B_ROW;
        const int pbyte = (lane * 16) % TC::B_ROW;
        const int ch    = (pbyte >> 5) ^ kn_swz(k);  // logical 32-byte chunk stored at physical chunk pbyte/32
        // the base pointer of load i already advances by B_KROWS_PER_LOAD * i rows
        ld.b_off[i] = (unsigned)((k - i * TC::B_KROWS_PER_LOAD) * N + ((ch << 5) + (pbyte & 31)) / 2) * 2u;
        ld.b_k[i]   = k;
      }
    }
  }
  const T* Ag = A + (size_t)m0 * K;
  const T* Bg = B_NK ? B + (size_t)n0 * K : B + n0;

  // ---- operand read setup (byte offsets inside a stage).  lane = (g = lane/16, i = lane%16):
  // row i of a 16-row fragment, k = 8g .. 8g+7
  const int g    = lane >> 4;
  const int li   = lane & 15;
  const int a_rd = k64_offset(wm * WM + li, g);
  int       b_rd[8];
  if constexpr (B_NK) {
    b_rd[0] = k64_offset(wn * 128 + li, g);
#pragma unroll
    for (int nf = 1; nf < 8; ++nf) b_rd[nf] = 0;
  }
  else {
    // transposing read: inside the 16-lane block, lane j supplies the 8 bytes (4 columns) j%4 of k row 8g + j/4
    const int k = 8 * g + (li >> 2);
#pragma unroll
    for (int nf = 0; nf < 8; ++nf) b_rd[nf] = k * TC::B_ROW + (((wn * 8 + nf) ^ kn_swz(k)) << 5) + (li & 3) * 8;
  }

  f32x4 acc[8][MF];
#pragma unroll
  for (int nf = 0; nf < 8; ++nf)
#pragma unroll
    for (int mf = 0; mf < MF; ++mf) acc[nf][mf] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int    KT          = (K + TC::BK - 1) / TC::BK;
  const int    full_stages = K / TC::BK;
  const size_t b_step      = B_NK ? (size_t)TC::BK : (size_t)TC::BK * N;

  char LLMMM_LDS* const lds      = (char LLMMM_LDS*)lds_raw;
  char LLMMM_LDS* const ring[4]  = {lds, lds + TC::STAGE, lds + 2 * TC::STAGE, lds + 3 * TC::STAGE};
  const unsigned        lds_base = (unsigned)(size_t)lds;  // the same buffers as LDS byte addresses, for the loader
  const unsigned ring_addr[4]    = {lds_base, lds_base + TC::STAGE, lds_base + 2 * TC::STAGE, lds_base + 3 * TC::STAGE};

#define LLMMM_ISSUE(stage, buf)                                                                                                     \
  fp16_issue_stage<T, BM, BN, WM, B_NK, KTAIL>(ring[buf], ring_addr[buf], Ag + (size_t)(stage) * TC::BK, Bg + (size_t)(stage) * b_step, ld, K, \
                                           N, wave, lane, K - (stage) * TC::BK)

  // prologue: stages 0..2 in flight, stage 0 landed and published, then stage 3 behind the barrier
  LLMMM_ISSUE(0, 0);
  if (1 < KT) LLMMM_ISSUE(1, 1);
  if (2 < KT) LLMMM_ISSUE(2, 2);
  if (!KTAIL && 2 < KT)
    wait_vmcnt<2 * TC::LOADS>();  // only stage 0 has to be here; stages 1 and 2 stay in flight
  else
    wait_vmcnt<0>();
  __builtin_amdgcn_s_barrier();
  if constexpr (STAMP) ph[1] = phase_clock();
  if (3 < KT) LLMMM_ISSUE(3, 3);

  vec aX[MF], aY[MF], bL[4], bR[4];  // A fragments of the current / next stage; B fragments of the left / right 64 columns
  fp16_read_a<T, MF>(ring[0], a_rd, aX);
  fp16_read_b<T, BM, BN, WM, B_NK>(ring[0], b_rd, 0, bL);

  // One stage s (in ring[u]) with its A fragments in aC; aN receives those of stage s+1.
  // STEADY = "stages s+1 .. s+4 exist and are full" (straight-line code).  LDS reads are always
  // issued between two groups of 8 MFMAs, a whole group (>= 128 cycles) before their data is used.
#define LLMMM_STAGE(STEADY, s, u, aC, aN)                                                                          \
  {                                                                                                                \
    fp16_mfma8<T, MF>(0, 0, aC, bL, acc);                                                                              \
    __builtin_amdgcn_sched_barrier(0);                                                                             \
    fp16_read_b<T, BM, BN, WM, B_NK>(ring[u], b_rd, 1, bR);                                                            \
    __builtin_amdgcn_sched_barrier(0);                                                                             \
    fp16_mfma8<T, MF>(0, 1, aC, bL, acc);                                                                              \
    __builtin_amdgcn_sched_barrier(0);                                                                             \
    /* every LDS read of stage s has been issued; once they are back (lgkmcnt(0), part of each wait below) the */ \
    /* barrier hands ring[u] to the loader and publishes stage s+1 */                                             \
    unsigned long long tw_ = 0;                                                                                    \
    if constexpr (STAMP) tw_ = __builtin_amdgcn_s_memtime();                                                       \
    if (STEADY || (s) + 3 < full_stages)                                                                           \
      wait_vmcnt<2 * TC::LOADS>(); /* stages s+2 and s+3 may still be in flight */                                 \
    else if ((s) + 2 < full_stages)                                                                                \
      wait_vmcnt<TC::LOADS>();                                                                                     \
    else                                                                                                           \
      wait_vmcnt<0>();                                                                                             \
    if constexpr (STAMP) load_wait_cycles += __builtin_amdgcn_s_memtime() - tw_;                                   \
    __builtin_amdgcn_s_barrier();                                                                                  \
    if constexpr (STAMP) wait_cycles += __builtin_amdgcn_s_memtime() - tw_;                                        \
    if (STEADY || (s) + 4 < KT) LLMMM_ISSUE((s) + 4, u);                                                           \
    fp16_mfma8<T, MF>(1, 0, aC, bR, acc);                                                                              \
    __builtin_amdgcn_sched_barrier(0);                                                                             \
    /* unconditional: after the last stage this reads a stale buffer and the result is unused */                  \
    fp16_read_a<T, MF>(ring[((u) + 1) & 3], a_rd, aN);                                                   \
    fp16_read_b<T, BM, BN, WM, B_NK>(ring[((u) + 1) & 3], b_rd, 0, bL);                                                \
    __builtin_amdgcn_sched_barrier(0);                                                                             \
    fp16_mfma8<T, MF>(1, 1, aC, bR, acc);                                                                              \
    __builtin_amdgcn_sched_barrier(0);                                                                             \
  }

  int kt = 0;
  for (; kt + 8 <= full_stages; kt += 4) {
    LLMMM_STAGE(true, kt + 0, 0, aX, aY)
    LLMMM_STAGE(true, kt + 1, 1, aY, aX)
    LLMMM_STAGE(true, kt + 2, 2, aX, aY)
    LLMMM_STAGE(true, kt + 3, 3, aY, aX)
  }
  for (; kt < KT; kt += 4) {
    if (kt + 0 < KT) LLMMM_STAGE(false, kt + 0, 0, aX, aY)
    if (kt + 1 < KT) LLMMM_STAGE(false, kt + 1, 1, aY, aX)
    if (kt + 2 < KT) LLMMM_STAGE(false, kt + 2, 2, aX, aY)
    if (kt + 3 < KT) LLMMM_STAGE(false, kt + 3, 3, aY, aX)
  }
#undef LLMMM_STAGE
#undef LLMMM_ISSUE
  if constexpr (STAMP) ph[2] = phase_clock();

  // ---- epilogue: lane (g, li) holds rows m = .. + mf*16 + li, columns nf*16 + 4g + r.
  // Stored straight from this layout, one instruction would write 8 bytes to each of 16 rows,
  // and the memory pipeline pays per row segment.  Instead every wave lays its 64 x 128 result
  // out row-major (256-byte rows, 16-byte chunks XOR-ed with the row so that the ds_read_b128
  // below is conflict-free) in a private 16 KB piece of the ring and stores whole rows, 16
  // bytes per lane.  Behind the last stage's barrier no wave reads operands any more and every
  // load has landed, so the ring is free.
  {
    typedef T             tx4 __attribute__((ext_vector_type(4)));
    char LLMMM_LDS* const stg = lds + wave * (WM * 256);
#pragma unroll
    for (int mf = 0; mf < MF; ++mf) {
      const int r = mf * 16 + li;
#pragma unroll
      for (int nf = 0; nf < 8; ++nf) {
        const f32x4 v = acc[nf][mf];
        tx4         o;
        o[0] = (T)v[0];
        o[1] = (T)v[1];
        o[2] = (T)v[2];
        o[3] = (T)v[3];
        *(tx4 LLMMM_LDS*)(stg + r * 256 + (((nf * 2 + (g >> 1)) ^ (r & 15)) << 4) + 8 * (g & 1)) = o;
      }
    }
    T* cbase = C + (size_t)(m0 + wm * WM) * N + n0 + wn * 128;
#pragma unroll
    for (int j = 0; j < WM / 4; ++j) {
      const int   r = 4 * j + (lane >> 4), ch = lane & 15;
      const i32x4 v = *(const i32x4 LLMMM_LDS*)(stg + r * 256 + ((ch ^ (r & 15)) << 4));
      *(i32x4*)(cbase + (size_t)r * N + ch * 8) = v;
    }
  }
  if constexpr (STAMP) {
    ph[3] = phase_clock();
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the stores are acknowledged
    ph[4] = phase_clock();
    if (lane == 0) {
      unsigned long long* o = stamps + ((size_t)tile_index * TC::NW + wave) * PHASE_RECORD;
#pragma unroll
      for (int p = 0; p < PHASE_POINTS; ++p) o[2 * p] = ph[p].real, o[2 * p + 1] = ph[p].cycles;
      o[PHASE_STAMPS] = wait_cycles, o[PHASE_STAMPS + 1] = load_wait_cycles;
    }
  }
}

template <typename T>
__global__ void __launch_bounds__(512)
fp16_gemm_phases_kernel(const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C, int M, int N, int K, int tiles_m, int tiles_n,
                        unsigned long long* stamps)
{
  __shared__ __attribute__((aligned(1024))) char lds_raw[4 * Fp16Tile<T, 256, 256, 64, false>::STAGE];
  fp16_gemm_body<T, 256, 256, 64, false, false, true>(A, B, C, M, N, K, tiles_m, tiles_n, (char LLMMM_LDS*)lds_raw, blockIdx.x, 0, stamps);
}

template <typename T, int BM, int BN, int WM, bool B_NK, bool KTAIL>
__global__ void __launch_bounds__((BM / WM) * (BN / 128) * 64)
fp16_gemm_kernel(const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C, int M, int N, int K, int tiles_m, int tiles_n)
{
  __shared__ __attribute__((aligned(1024))) char lds_raw[4 * Fp16Tile<T, BM, BN, WM, B_NK>::STAGE];  // the ring of four stages
  fp16_gemm_body<T, BM, BN, WM, B_NK, KTAIL>(A, B, C, M, N, K, tiles_m, tiles_n, (char LLMMM_LDS*)lds_raw, blockIdx.x, 0);
}

// 256 x 256 tiles whose number is not a multiple of the 256 CUs end with a round that keeps part of the chip busy for a
// whole tile's time (2048 x 19456: 608 tiles, the third round 96 of them).  One launch of both shapes: the columns that fill
// whole rounds go to 256 x 256 tiles (workgroups 0 .. tiles_m_big * cols_big - 1, dispatched first), the remaining columns
// to twice as many 128 x 256 tiles -- the same eight waves, ring and K loop, half the rows per wave, the same results.
template <typename T, bool B_NK, bool KTAIL>
__global__ void __launch_bounds__(512)
fp16_gemm_hybrid_kernel(const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C, int M, int N, int K, int tiles_m_big, int cols_big,
                        int cols_small)
{
  static_assert(Fp16Tile<T, 128, 256, 32, B_NK>::STAGE <= Fp16Tile<T, 256, 256, 64, B_NK>::STAGE, "the small tiles fit the large tiles' ring");
  __shared__ __attribute__((aligned(1024))) char lds_raw[4 * Fp16Tile<T, 256, 256, 64, B_NK>::STAGE];
  const int n_big = tiles_m_big * cols_big;
  if ((int)blockIdx.x < n_big)
    fp16_gemm_body<T, 256, 256, 64, B_NK, KTAIL>(A, B, C, M, N, K, tiles_m_big, cols_big, (char LLMMM_LDS*)lds_raw, blockIdx.x, 0);
  else
    fp16_gemm_body<T, 128, 256, 32, B_NK, KTAIL>(A, B, C, M, N, K, 2 * tiles_m_big, cols_small, (char LLMMM_LDS*)lds_raw, (int)blockIdx.x - n_big,
                                                 cols_big * 256);
}

// --------------------------------------------------------------------------------------------- host
template <typename T, int BM, int BN, int WM, bool B_NK>
static hipError_t launch_fp16(const void* A, const void* B, void* C, int M, int N, int K, hipStream_t stream)
{
  typedef Fp16Tile<T, BM, BN, WM, B_NK> TC;
  const int tiles_m = M / BM, tiles_n = N / BN;
  if constexpr (BM == 256 && BN == 256) {
    // more than one round of the chip with a partly filled last one: whole rounds in 256 x 256 tiles, the remaining
    // columns in 128 x 256 tiles, if those fit one round (fp16_gemm_hybrid_kernel)
    const int  cus   = num_cus();
    const long tiles = (long)tiles_m * tiles_n, full = tiles / cus * cus;
    if (tiles > cus && tiles_m > 1 && full % tiles_m == 0) {
      const int cols_big = (int)(full / tiles_m), cols_small = tiles_n - cols_big;
      if (cols_small > 0 && (long)cols_small * tiles_m * 2 <= cus) {
        const dim3 grid(tiles_m * cols_big + 2 * tiles_m * cols_small);
        if (K % TC::BK)
          hipLaunchKernelGGL((fp16_gemm_hybrid_kernel<T, B_NK, true>), grid, dim3(512), 0, stream, (const T*)A, (const T*)B, (T*)C, M, N, K, tiles_m,
                             cols_big, cols_small);
        else
          hipLaunchKernelGGL((fp16_gemm_hybrid_kernel<T, B_NK, false>), grid, dim3(512), 0, stream, (const T*)A, (const T*)B, (T*)C, M, N, K, tiles_m,
                             cols_big, cols_small);
        return hipGetLastError();
      }
    }
  }
  if (K % TC::BK)
    hipLaunchKernelGGL((fp16_gemm_kernel<T, BM, BN, WM, B_NK, true>), dim3(tiles_m * tiles_n), dim3(TC::NT), 0, stream, (const T*)A,
                       (const T*)B, (T*)C, M, N, K, tiles_m, tiles_n);
  else
    hipLaunchKernelGGL((fp16_gemm_kernel<T, BM, BN, WM, B_NK, false>), dim3(tiles_m * tiles_n), dim3(TC::NT), 0, stream, (const T*)A,
                       (const T*)B, (T*)C, M, N, K, tiles_m, tiles_n);
  return hipGetLastError();
}

template <typename T, bool B_NK>
static hipError_t dispatch_fp16(int tile, const void* A, const void* B, void* C, int M, int N, int K, hipStream_t stream)
{
  // the 256 x 256 tile uses eight 64-row waves; the smaller tiles 32-row waves, which doubles the
  // waves per SIMD (measured 10-45 % faster than 64-row waves on those tiles)
  switch (tile) {
    case LLMMM_TILE_256x256: return launch_fp16<T, 256, 256, 64, B_NK>(A, B, C, M, N, K, stream);
    case LLMMM_TILE_128x256: return launch_fp16<T, 128, 256, 32, B_NK>(A, B, C, M, N, K, stream);
    case LLMMM_TILE_256x128: return launch_fp16<T, 256, 128, 32, B_NK>(A, B, C, M, N, K, stream);
    case LLMMM_TILE_128x128: return launch_fp16<T, 128, 128, 32, B_NK>(A, B, C, M, N, K, stream);
    case LLMMM_TILE_64x128: return launch_fp16<T, 64, 128, 16, B_NK>(A, B, C, M, N, K, stream);  // four 16-row waves: small problems
    default: return hipErrorInvalidValue;
  }
}

hipError_t fp16_gemm_phases_launch(int dtype, const void* A, const void* B, void* C, int M, int N, int K, unsigned long long* stamps, hipStream_t stream)
{
  if (M % 256 || N % 256 || K % 32 || !stamps) return hipErrorInvalidValue;
  const int tiles_m = M / 256, tiles_n = N / 256;
  if (dtype == 0)
    hipLaunchKernelGGL((fp16_gemm_phases_kernel<_Float16>), dim3(tiles_m * tiles_n), dim3(512), 0, stream, (const _Float16*)A, (const _Float16*)B, (_Float16*)C, M,
                       N, K, tiles_m, tiles_n, stamps);
  else
    hipLaunchKernelGGL((fp16_gemm_phases_kernel<__bf16>), dim3(tiles_m * tiles_n), dim3(512), 0, stream, (const __bf16*)A, (const __bf16*)B, (__bf16*)C, M, N, K,
                       tiles_m, tiles_n, stamps);
  return hipGetLastError();
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
