// Small-M (decode) FP8 blockwise GEMM for gfx950: weight streaming with deterministic split-K.
//
// Same arithmetic and layouts as fp8_gemm.hip (reference math: examples/005.fp8.mm.cu:885-902,
// fused epilogue examples/005.fp8.mm.opt.cu:401-462) for M <= 128 rows (in groups of 64), a range the reference
// does not cover (its launchers require M % 128 == 0, examples/005.fp8.mm.opt.cu:492; split-K
// is listed as unfinished in README.md:22).
//
//  * HBM-bound: every byte of Bt[N,K] is read exactly once.  One wavefront owns 16 weight rows;
//    per 128-K slice it moves their 16 x 128 bytes global -> LDS with two LDS-direct loads that
//    each cover 8 whole rows (full 128-byte lines per instruction), into a wave-private ring of
//    D slots, and reads the MFMA operand back with two conflict-free ds_read_b128.  The
//    activation rows go straight from global memory (L2) into the other operand's registers.
//  * A workgroup = 8 waves = one 128-column quantisation group; grid.y = number of K splits.
//  * split-K: each split stores its fp32 plane of partial sums (plain stores) and is done; the
//    reduce kernel of fp8_gemm.hip, launched behind it, adds the planes in split order 0..S-1
//    (fixed order, independent of arrival) and runs the epilogue.  An in-kernel "last arriver
//    reduces" scheme was measured slower: its device-scope stores, counter and re-reads put three
//    dependent memory round trips on the critical path of every column group.
//  * The activation rows a workgroup needs (16..64 rows x the K range of its split) are staged
//    in LDS once, before the loop, whenever they fit beside the ring; every wave then reads its
//    operand fragments from there instead of re-fetching them from L2 slice by slice.
#include "device_common.hip.h"
#include "kernels.h"

namespace llmmm {

enum { SK_OUT_F32 = 0, SK_OUT_BF16 = 1, SK_OUT_FP8Q = 2 };

// What one 128-K slice needs besides the weights: the activation rows (straight into the MFMA
// operand registers) and both scales.  Rows beyond M are clamped to M-1 (a valid address, no
// divergence); their products are computed and never stored.
template <int MBLK, bool APRE>
struct SkinnySlot {
  i32x4 a[APRE ? 1 : MBLK][2];  // unused when the activations were staged in LDS up front (APRE)
  float sa[MBLK];
  float sb;
};

// Weights: the wave's 16 rows x 128 bytes of a slice travel global -> LDS with two LDS-direct
// loads of 1 KB each.  A load covers 8 whole rows, so every 128-byte line is fetched by one
// instruction in full; the SWZ_ROWS16 placement makes the operand read-back conflict-free.
// One wave-private ring slot = 2 KB; no workgroup barrier is involved.
constexpr int SKINNY_LOADS_PER_SLOT_BASE = 2;  // LDS-direct loads; + 3 (or 1, with APRE) per 16 activation rows

// The weight stream is read once and never again: its loads carry the non-temporal hint, which
// keeps the stream from displacing the (re-used) activations and scales in the caches and was
// measured 0.7-0.8 us faster per launch on every decode shape.
__device__ __forceinline__ void skinny_stream_lds_16B(const void* gptr, unsigned lds_addr)
{
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt" ::"v"(gptr), "s"(lds_addr) : "memory");
}

// All vector-memory loads of a slot, in a fixed order, as inline assembly (see device_common.hip.h):
// the kernel counts them itself.
template <int MBLK, bool APRE, bool SA_LDS = false>
__device__ __forceinline__ void skinny_fetch(SkinnySlot<MBLK, APRE>& t, unsigned ring_slot, const uint8_t* wrow, int w_kstep,
                                             unsigned w_off0, unsigned w_off1, const uint8_t* const (&ap)[MBLK], const float* const (&asp)[MBLK],
                                             const float* bsp, int kb, int M)
{
  skinny_stream_lds_16B(wrow + (size_t)kb * w_kstep + w_off0, ring_slot);
  skinny_stream_lds_16B(wrow + (size_t)kb * w_kstep + w_off1, ring_slot + 1024);
#pragma unroll
  for (int mb = 0; mb < MBLK; ++mb) {
    if constexpr (!APRE) {
      asm_load_16B(t.a[mb][0], ap[mb] + (size_t)kb * 128);
      asm_load_16B(t.a[mb][1], ap[mb] + (size_t)kb * 128 + 16);
    }
    if constexpr (!SA_LDS) asm_load_f32(t.sa[mb], asp[mb] + (size_t)kb * M);
  }
  t.sb = bsp[kb];
}

// s_waitcnt vmcnt(N) that also "touches" the slot's registers, so that nothing reading them can
// be moved in front of it.
template <int N, int MBLK, bool APRE, bool SA_LDS = false>
__device__ __forceinline__ void skinny_wait(SkinnySlot<MBLK, APRE>& t)
{
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  if constexpr (SA_LDS) {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");  // the slot holds no registers of its own: everything it waits for lands in LDS
  }
  else if constexpr (APRE) {
    if constexpr (MBLK == 1)
      asm volatile("s_waitcnt vmcnt(%1)" : "+v"(t.sa[0]) : "n"(N) : "memory");
    else if constexpr (MBLK == 2)
      asm volatile("s_waitcnt vmcnt(%2)" : "+v"(t.sa[0]), "+v"(t.sa[1]) : "n"(N) : "memory");
    else if constexpr (MBLK == 4)
      asm volatile("s_waitcnt vmcnt(%4)" : "+v"(t.sa[0]), "+v"(t.sa[1]), "+v"(t.sa[2]), "+v"(t.sa[3]) : "n"(N) : "memory");
    else
      asm volatile("s_waitcnt vmcnt(%8)"
                   : "+v"(t.sa[0]), "+v"(t.sa[1]), "+v"(t.sa[2]), "+v"(t.sa[3]), "+v"(t.sa[4]), "+v"(t.sa[5]), "+v"(t.sa[6]), "+v"(t.sa[7])
                   : "n"(N)
                   : "memory");
  }
  else if constexpr (MBLK == 1)
    asm volatile("s_waitcnt vmcnt(%3)" : "+v"(t.a[0][0]), "+v"(t.a[0][1]), "+v"(t.sa[0]) : "n"(N) : "memory");
  else if constexpr (MBLK == 2)
    asm volatile("s_waitcnt vmcnt(%6)"
                 : "+v"(t.a[0][0]), "+v"(t.a[0][1]), "+v"(t.sa[0]), "+v"(t.a[1][0]), "+v"(t.a[1][1]), "+v"(t.sa[1])
                 : "n"(N)
                 : "memory");
  else if constexpr (MBLK == 4)
    asm volatile("s_waitcnt vmcnt(%12)"
                 : "+v"(t.a[0][0]), "+v"(t.a[0][1]), "+v"(t.sa[0]), "+v"(t.a[1][0]), "+v"(t.a[1][1]), "+v"(t.sa[1]), "+v"(t.a[2][0]),
                   "+v"(t.a[2][1]), "+v"(t.sa[2]), "+v"(t.a[3][0]), "+v"(t.a[3][1]), "+v"(t.sa[3])
                 : "n"(N)
                 : "memory");
}

// With APRE the activation fragments come from the workgroup's staged copy: a_slice points at
// the MBLK x 2 KB block of this slice, a_rd is the lane's SWZ_ROWS16 offset of (row i, chunk 2g).
// With SA_LDS the row scales of the slice come from LDS as well (sa_slice: 16 floats, row i at [i]).
template <int MBLK, bool APRE, bool SA_LDS = false>
__device__ __forceinline__ void skinny_consume(const SkinnySlot<MBLK, APRE>& t, const char LLMMM_LDS* ring_slot, int w_rd, bool valid,
                                               f32x4 (&acc)[MBLK], const char LLMMM_LDS* a_slice, int a_rd, const float LLMMM_LDS* sa_slice = nullptr,
                                               int row = 0)
{
  union {
    i32x4 h[2];
    i32x8 v;
  } wf, af;
  wf.h[0] = *(const i32x4 LLMMM_LDS*)(ring_slot + w_rd);
  wf.h[1] = *(const i32x4 LLMMM_LDS*)(ring_slot + (w_rd ^ 16));
#pragma unroll
  for (int mb = 0; mb < MBLK; ++mb) {
    if constexpr (APRE) {
      af.h[0] = *(const i32x4 LLMMM_LDS*)(a_slice + mb * 2048 + a_rd);
      af.h[1] = *(const i32x4 LLMMM_LDS*)(a_slice + mb * 2048 + (a_rd ^ 16));
    }
    else {
      af.h[0] = t.a[mb][0];
      af.h[1] = t.a[mb][1];
    }
    float sa;
    if constexpr (SA_LDS)
      sa = sa_slice[row];
    else
      sa = t.sa[mb];
    const float s = valid ? sa * t.sb : 0.f;
    const f32x4 z = {0.f, 0.f, 0.f, 0.f};
    const f32x4 p = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf.v, af.v, z, 0, 0, 0, 0, 0, 0);
#pragma unroll
    for (int r = 0; r < 4; ++r) acc[mb][r] = __builtin_fmaf(p[r], s, acc[mb][r]);
  }
}

// D = ring depth = slices in flight per wave.  The host picks the largest D that does not exceed
// the number of slices of the shortest split.
// ASTG = bytes of LDS in which the workgroup stages its activation rows for the whole K range
// of its split before the loop starts (0: the rows are fetched slice by slice into registers).
// AGEN: the activations are not given quantised -- the workgroup makes them itself from the fp32 result G [M, 2K] of
// the gate_up projection: h = silu(G[:, :K]) * G[:, K:], quantised 1x128, for the 16 rows and the K range it works on
// (the arithmetic of the reduce kernel's SwiGLU output, so the codes and scales are the ones that kernel would have
// written).  M <= 16.  A (then: G) and As (unused) keep their places in the argument list.
// AGEN == 2: the activations are the RMSNorm of a hidden state that is itself still in pieces -- the fp32 planes of the
// projection before (summed in split order), plus the residual: h = sum + residual, hidden = HT(h) (stored by workgroup
// (0, 0, 0); it must not alias the residual, which every workgroup reads), A = quantise_1x128(rmsnorm(hidden) * w), in the
// arithmetic and order of planes_add_rmsnorm_quant_kernel, bit for bit.  M <= 2, K <= 3072 (the row lives in registers),
// at most SKINNY_GEN_MAX_PLANES planes.
template <int MBLK, int OUT, int D, int ASTG, int AGEN = 0, typename HT = float>
__global__ void __launch_bounds__(512)
fp8_skinny_kernel(const uint8_t* __restrict__ A, const float* __restrict__ As, const uint8_t* __restrict__ Bt,
                  const float* __restrict__ Bs, void* __restrict__ Cv, float* __restrict__ Cs, int M, int N, int K, int S,
                  float* __restrict__ partial, int bpre, SkinnyGenA ag)
{
  constexpr bool APRE  = ASTG > 0;
  static_assert(AGEN == 0 || (MBLK == 1 && APRE), "generated activations: 16 rows, staged in LDS");
  constexpr int  LOADS = SKINNY_LOADS_PER_SLOT_BASE + (AGEN != 0 ? 0 : (APRE ? 1 : 3) * MBLK);  // vector-memory loads per slot, issued in slot order
  static_assert(D * LOADS < 64, "vmcnt is a 6-bit counter");
  static_assert(MBLK <= 4 || APRE, "128-row groups only with staged activations");
  __shared__ __attribute__((aligned(1024))) char a_stage[APRE ? ASTG : 16];
  // one array per ring slot, so that the compiler can tell the slots apart
  __shared__ __attribute__((aligned(1024))) char ring0[8 * 2048];
  __shared__ __attribute__((aligned(1024))) char ring1[8 * 2048];
  __shared__ __attribute__((aligned(1024))) char ring2[D > 2 ? 8 * 2048 : 16];
  __shared__ __attribute__((aligned(1024))) char ring3[D > 2 ? 8 * 2048 : 16];
  __shared__ __attribute__((aligned(1024))) char ring4[D > 4 ? 8 * 2048 : 16];
  __shared__ __attribute__((aligned(1024))) char ring5[D > 4 ? 8 * 2048 : 16];
  __shared__ __attribute__((aligned(1024))) char ring6[D > 4 ? 8 * 2048 : 16];
  __shared__ __attribute__((aligned(1024))) char ring7[D > 4 ? 8 * 2048 : 16];
  __shared__ float    wave_amax[8][MBLK][16];
  __shared__ float    a_scale[AGEN != 0 ? (ASTG / 2048) * 16 : 1];  // AGEN: the generated row scales, [slice][row]
  __shared__ float    gen_sum[AGEN == 2 ? 8 : 1];                        // AGEN == 2: sums of squares of the 64-lane groups, two rows

  const int tid  = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g    = lane >> 4;
  const int i    = lane & 15;
  const int ng   = blockIdx.x;
  const int sp   = blockIdx.y;
  const int m0   = blockIdx.z * (16 * MBLK);  // row groups of 16 * MBLK rows: gridDim.z = number of groups
  const int KB   = K >> 7;
  const int kb0  = sp * KB / S;  // KB * S is small: 32-bit arithmetic (a 64-bit divide costs hundreds of scalar ops)
  const int kb1  = (sp + 1) * KB / S;

  char LLMMM_LDS* const ring[8] = {(char LLMMM_LDS*)ring0 + wave * 2048, (char LLMMM_LDS*)ring1 + wave * 2048,
                                   (char LLMMM_LDS*)ring2 + wave * 2048, (char LLMMM_LDS*)ring3 + wave * 2048,
                                   (char LLMMM_LDS*)ring4 + wave * 2048, (char LLMMM_LDS*)ring5 + wave * 2048,
                                   (char LLMMM_LDS*)ring6 + wave * 2048, (char LLMMM_LDS*)ring7 + wave * 2048};
  unsigned ring_addr[8];  // the same slots as wave-uniform LDS byte addresses, for the loader
#pragma unroll
  for (int u = 0; u < 8; ++u) ring_addr[u] = __builtin_amdgcn_readfirstlane((unsigned)(size_t)ring[u]);

  // weights: loader lane -> (row, chunk) of the 1 KB group it fills; reader lane (g, i) -> row i, chunks 2g, 2g+1
  // pre-shuffled weights (bpre, layout.hip): the wave's 16 rows x 128 bytes of a slice are one 2 KB block that
  // already is the ring slot's image, and the blocks of consecutive slices follow each other
  const uint8_t*   wrow = Bt + (size_t)(ng * 128 + wave * 16) * K;
  const KMajorLane l0   = kmajor_lane<SWZ_ROWS16>(0, lane);
  const KMajorLane l1   = kmajor_lane<SWZ_ROWS16>(1, lane);
  const unsigned   w_off0   = bpre ? (unsigned)lane * 16u : (unsigned)(l0.row * K + l0.chunk * 16);
  const unsigned   w_off1   = bpre ? 1024u + (unsigned)lane * 16u : (unsigned)(l1.row * K + l1.chunk * 16);
  const int        w_kstep  = bpre ? 2048 : 128;
  const int        w_rd   = kmajor_offset<SWZ_ROWS16>(i, 2 * g);
  const float*     bsp    = Bs + (size_t)ng * KB;
  const uint8_t*   ap[MBLK];
  const float*     asp[MBLK];
#pragma unroll
  for (int mb = 0; mb < MBLK; ++mb) {
    const int m = min(m0 + mb * 16 + i, M - 1);
    ap[mb]      = A + (size_t)m * K + 32 * g;  // same k -> register mapping as the weights: bytes 32g .. 32g+31
    asp[mb]     = As + m;
  }

  f32x4 acc[MBLK];
#pragma unroll
  for (int mb = 0; mb < MBLK; ++mb) acc[mb] = f32x4{0.f, 0.f, 0.f, 0.f};

  // Activation staging: the 16*MBLK rows x (kb1 - kb0) slices this workgroup needs, as one
  // SWZ_ROWS16 tile of MBLK x 2 KB per slice, fetched once by LDS-direct loads of 8 whole rows
  // (1 KB units dealt round-robin to the waves) instead of once per wave and slice.  They are
  // the oldest loads in flight, so "at most D*LOADS outstanding" after the ring prologue means
  // they have landed.
  const char LLMMM_LDS* const a_tile = (const char LLMMM_LDS*)a_stage;
  const int                   a_rd   = kmajor_offset<SWZ_ROWS16>(i, 2 * g);
  if constexpr (APRE && AGEN == 0) {
    const unsigned a_addr = (unsigned)(size_t)(char LLMMM_LDS*)a_stage;
    const int      units  = (kb1 - kb0) * 2 * MBLK;
    for (int u = wave; u < units; u += 8) {
      const int j = u / (2 * MBLK), within = u - j * (2 * MBLK);
      const int r = within * 8 + (lane >> 3);
      const int c = (lane & 7) ^ kmajor_swz<SWZ_ROWS16>(r);
      const int m = min(m0 + r, M - 1);
      asm_load_lds_16B(A + (size_t)m * K + (size_t)(kb0 + j) * 128 + c * 16, a_addr + j * (MBLK * 2048) + within * 1024);
    }
  }

  // Software pipeline, D slices in flight per wave, all vector-memory loads issued strictly in
  // slot order so that "at most n loads outstanding" pins down which slots have landed.
  // Slice indices beyond the split are clamped to its last slice (a repeated, cached load) and
  // consumed with a zero scale; the last pass issues nothing and counts its waits down.
  // AGEN == 2: everything the generated operand needs is requested first, as hand-counted loads like the ring's, so that
  // it is the oldest traffic in flight: "at most D * LOADS outstanding" behind the ring prologue then means it has landed,
  // and the norm runs while the first weights are still on their way.
  constexpr int GP = SKINNY_GEN_MAX_PLANES;  // all planes are requested up front (the split counts in use are 1 .. 10)
  i32x4         g_res[AGEN == 2 ? 3 : 1], g_w[AGEN == 2 ? 3 : 1], g_p[AGEN == 2 ? GP : 1][AGEN == 2 ? 3 : 1];
  i32x2         g_res2[AGEN == 2 ? 3 : 1];  // the residual chunk of a 2-byte hidden type (nothing may read these before the wait)
  if constexpr (AGEN == 2) {
    const int    vl = tid & 255, r = min(tid >> 8, M - 1), chunks = K >> 2;
    const size_t pplane = (size_t)M * K;
    // Straight-line code, every load unconditional: a register written by a load the compiler cannot see in flight must
    // not pass through a copy before the counted wait, and conditional definitions invite such copies.  Loads that
    // are not needed (waves without a row of their own, planes beyond the split count) all read one common address
    // instead, which costs a single cache line per instruction.
    const bool  own  = (tid >> 8) < M;
    const char* idle = (const char*)ag.w;
#pragma unroll
    for (int u = 0; u < 3; ++u) {
      const int   c  = min(vl + 256 * u, chunks - 1);
      const char* rp = (const char*)((const HT*)ag.residual + (size_t)r * K + 4 * c);
      if constexpr (sizeof(HT) == 4)
        asm_load_16B(g_res[u], own ? rp : idle);
      else
        asm_load_8B(g_res2[u], own ? rp : idle);
      asm_load_16B(g_w[u], own ? (const char*)(ag.w + 4 * c) : idle);
    }
#pragma unroll
    for (int v = 0; v < GP; ++v)
#pragma unroll
      for (int u = 0; u < 3; ++u) {
        const int   c  = min(vl + 256 * u, chunks - 1);
        const char* pp = (const char*)(ag.planes + (size_t)min(v, ag.splits - 1) * pplane + (size_t)r * K + 4 * c);
        asm_load_16B(g_p[v][u], own && v < ag.splits ? pp : idle);
      }
  }
  // AGEN == 1: likewise the gate and up values of the first four (row, slice) tasks of every half-wave (all of them for
  // M * slices <= 64; later batches use ordinary loads)
  i32x4 g_gate[AGEN == 1 ? 4 : 1], g_up[AGEN == 1 ? 4 : 1];
  if constexpr (AGEN == 1) {
    const float* G    = (const float*)A;
    const int    rows = min(M, 16), tasks = (kb1 - kb0) * rows;
#pragma unroll
    for (int u = 0; u < 4; ++u) {  // unconditional loads (see above); tasks that do not exist read G's first bytes
      const int    t  = (tid >> 5) + 16 * u, tc = min(t, tasks - 1);
      const int    j  = tc / rows, r = tc - j * rows;
      const float* gp = G + (size_t)r * 2 * K + (size_t)(kb0 + j) * 128 + 4 * (tid & 31);
      asm_load_16B(g_gate[u], t < tasks ? gp : G);
      asm_load_16B(g_up[u], t < tasks ? gp + K : G);
    }
  }
  SkinnySlot<MBLK, APRE> slot[D];
#pragma unroll
  for (int u = 0; u < D; ++u) {
    skinny_fetch<MBLK, APRE, AGEN != 0>(slot[u], ring_addr[u], wrow, w_kstep, w_off0, w_off1, ap, asp, bsp, min(kb0 + u, kb1 - 1), M);
    __builtin_amdgcn_sched_barrier(0);
  }
  if constexpr (AGEN == 2) {
    HT*          hid    = (HT*)ag.hidden;
    const int    vl     = tid & 255, rsel = tid >> 8;  // 256 virtual lanes per row; rows 0 and 1 side by side (M <= 2)
    const int    chunks = K >> 2, nsl = kb1 - kb0;
    const size_t pplane = (size_t)M * K;
    const bool   writer = blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0;
    const int    r      = min(rsel, M - 1);
    const bool   live   = rsel < M;
    for (int x = tid; x < nsl * 128; x += 512) *(i32x4 LLMMM_LDS*)((char LLMMM_LDS*)a_stage + x * 16) = i32x4{0, 0, 0, 0};
    for (int x = tid; x < nsl * 16; x += 512) a_scale[x] = 0.f;
    // The operand's loads are in once at most the ring's D * LOADS loads are outstanding.  Every destination register of
    // those early loads is an in/out operand of the wait itself, so the values the code below reads are, to the compiler,
    // results of this instruction: nothing that uses them can be placed in front of it.  (One statement per chunk column:
    // twelve 128-bit operands each; the second and third find the count already met.)
    static_assert(GP == 10, "the operand list below names ten planes");
#pragma unroll
    for (int u = 0; u < 3; ++u) {
      if constexpr (sizeof(HT) == 4)
        asm volatile("s_waitcnt vmcnt(%12)"
                     : "+v"(g_res[u]), "+v"(g_w[u]), "+v"(g_p[0][u]), "+v"(g_p[1][u]), "+v"(g_p[2][u]), "+v"(g_p[3][u]), "+v"(g_p[4][u]), "+v"(g_p[5][u]),
                       "+v"(g_p[6][u]), "+v"(g_p[7][u]), "+v"(g_p[8][u]), "+v"(g_p[9][u])
                     : "n"(D * LOADS)
                     : "memory");
      else
        asm volatile("s_waitcnt vmcnt(%12)"
                     : "+v"(g_res2[u]), "+v"(g_w[u]), "+v"(g_p[0][u]), "+v"(g_p[1][u]), "+v"(g_p[2][u]), "+v"(g_p[3][u]), "+v"(g_p[4][u]), "+v"(g_p[5][u]),
                       "+v"(g_p[6][u]), "+v"(g_p[7][u]), "+v"(g_p[8][u]), "+v"(g_p[9][u])
                     : "n"(D * LOADS)
                     : "memory");
    }
    f32x4 held[3], rv[3], wv[3];
#pragma unroll
    for (int u = 0; u < 3; ++u) {
      wv[u] = __builtin_bit_cast(f32x4, g_w[u]);
      if constexpr (sizeof(HT) == 4)
        rv[u] = __builtin_bit_cast(f32x4, g_res[u]);
      else {
        typedef HT     ht4 __attribute__((ext_vector_type(4)));
        const ht4      t  = __builtin_bit_cast(ht4, g_res2[u]);
        rv[u]             = f32x4{(float)t[0], (float)t[1], (float)t[2], (float)t[3]};
      }
      held[u] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int v = 0; v < GP; ++v)
      if (v < ag.splits) {
#pragma unroll
        for (int u = 0; u < 3; ++u) held[u] += __builtin_bit_cast(f32x4, g_p[v][u]);
      }
    float acc = 0.f;
#pragma unroll
    for (int u = 0; u < 3; ++u) {
      const int c = vl + 256 * u;
      if (c < chunks) {
        const f32x4 h = held[u] + rv[u];
        if (writer && live) store_row4<HT>(hid + (size_t)r * K + 4 * c, h);
        if constexpr (sizeof(HT) == 4)
          held[u] = h;
        else {
#pragma unroll
          for (int e = 0; e < 4; ++e) held[u][e] = (float)(HT)h[e];  // the norm reads the hidden state as stored
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) acc = __builtin_fmaf(held[u][e], held[u][e], acc);
      }
      else
        held[u] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int step = 32; step >= 1; step >>= 1) acc = acc + wave_xor_get(acc, step);
    if (lane == 0) gen_sum[wave] = acc;
    __syncthreads();  // (also: the zero fill is complete)
    const float total = (gen_sum[4 * rsel] + gen_sum[4 * rsel + 1]) + (gen_sum[4 * rsel + 2] + gen_sum[4 * rsel + 3]);
    const float ms    = total / (float)K;
    const float rn    = 1.0f / __builtin_sqrtf(ms + ag.eps);
#pragma unroll
    for (int u = 0; u < 3; ++u) {
      const int c = vl + 256 * u;
      const int j = (c >> 5) - kb0;  // the chunk's 128-column block as a slice of this workgroup
      // only the blocks of this workgroup's K range are quantised (uniform over the 32 lanes that share a block)
      if (c < chunks && live && j >= 0 && j < nsl) {
#pragma unroll
        for (int e = 0; e < 4; ++e) held[u][e] = (held[u][e] * rn) * wv[u][e];
        float a = fmaxf(fmaxf(fmaxf(0.f, __builtin_fabsf(held[u][0])), __builtin_fabsf(held[u][1])), fmaxf(__builtin_fabsf(held[u][2]), __builtin_fabsf(held[u][3])));
#pragma unroll
        for (int step = 1; step <= 16; step <<= 1) a = wave_xor_max(a, step);
        const float sc = a / 448.f;
        uint32_t    cd = 0;
        if (sc != 0.f) cd = pack_e4m3x4_sat(held[u][0] / sc, held[u][1] / sc, held[u][2] / sc, held[u][3] / sc);
        *(uint32_t LLMMM_LDS*)((char LLMMM_LDS*)a_stage + j * 2048 + kmajor_offset<SWZ_ROWS16>(r, (c & 31) >> 2) + (c & 3) * 4) = cd;
        if ((c & 31) == 0) a_scale[j * 16 + r] = sc;
      }
    }
    __syncthreads();  // the staged tile is complete
  }
  else if constexpr (AGEN == 1) {
    // Half a wavefront per (row, slice) task, a lane per four columns of the slice.
    const float* G   = (const float*)A;
    const int    l32 = tid & 31;
    if (M < 16) {  // rows M .. 15 of every slice: zero codes, zero scales (their products are never stored)
      for (int x = tid; x < (kb1 - kb0) * 128; x += 512) *(i32x4 LLMMM_LDS*)((char LLMMM_LDS*)a_stage + x * 16) = i32x4{0, 0, 0, 0};
      for (int x = tid; x < (kb1 - kb0) * 16; x += 512) a_scale[x] = 0.f;
      __syncthreads();
    }
    // (row, slice) tasks are dealt round-robin to the 16 half-waves: for M = 1 every half-wave has one slice to make.
    // The first batch was requested in front of the ring prologue: once at most D * LOADS loads are outstanding it is in.
    const int nsl = kb1 - kb0, rows = min(M, 16), tasks = nsl * rows;
    // (the early loads' destinations are in/out operands of the wait: what is read below is, to the compiler, its result)
    asm volatile("s_waitcnt vmcnt(%8)"
                 : "+v"(g_gate[0]), "+v"(g_up[0]), "+v"(g_gate[1]), "+v"(g_up[1]), "+v"(g_gate[2]), "+v"(g_up[2]), "+v"(g_gate[3]), "+v"(g_up[3])
                 : "n"(D * LOADS)
                 : "memory");
    for (int t0 = tid >> 5; t0 < tasks; t0 += 16 * 4) {  // four tasks of a half-wave per batch
      f32x4 gv[4], uv[4];
      if (t0 < 16) {
#pragma unroll
        for (int u = 0; u < 4; ++u) gv[u] = __builtin_bit_cast(f32x4, g_gate[u]), uv[u] = __builtin_bit_cast(f32x4, g_up[u]);
      }
      else {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int    t  = min(t0 + 16 * u, tasks - 1), j = t / rows, r = t - j * rows;
          const float* gp = G + (size_t)r * 2 * K + (size_t)(kb0 + j) * 128 + 4 * l32;
          gv[u]           = *(const f32x4*)gp;
          uv[u]           = *(const f32x4*)(gp + K);
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int t = t0 + 16 * u;
        if (t < tasks) {  // uniform over the half-wave
          const int j = t / rows, r = t - j * rows;
          f32x4     h;
#pragma unroll
          for (int q = 0; q < 4; ++q) h[q] = silu_mul(gv[u][q], uv[u][q]);
          float a = fmaxf(fmaxf(fmaxf(0.f, __builtin_fabsf(h[0])), __builtin_fabsf(h[1])), fmaxf(__builtin_fabsf(h[2]), __builtin_fabsf(h[3])));
#pragma unroll
          for (int step = 1; step <= 16; step <<= 1) a = wave_xor_max(a, step);
          const float scale = a / 448.f;
          const float inv   = requant_inv(a);
          *(uint32_t LLMMM_LDS*)((char LLMMM_LDS*)a_stage + j * 2048 + kmajor_offset<SWZ_ROWS16>(r, l32 >> 2) + (l32 & 3) * 4) =
            pack_e4m3x4_in_range(h[0] * inv, h[1] * inv, h[2] * inv, h[3] * inv);
          if (l32 == 0) a_scale[j * 16 + r] = scale;
        }
      }
    }
    __syncthreads();
  }
  else if constexpr (APRE) {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(D * LOADS) : "memory");
    __syncthreads();  // every wave's share of the staged activations is in LDS
  }
  int kb = kb0;
  for (; kb + D < kb1; kb += D) {  // passes followed by another pass: consume a slot, refill it
#pragma unroll
    for (int u = 0; u < D; ++u) {
      skinny_wait<(D - 1) * LOADS, MBLK, APRE, AGEN != 0>(slot[u]);
      skinny_consume<MBLK, APRE, AGEN != 0>(slot[u], ring[u], w_rd, true, acc, a_tile + (kb + u - kb0) * (MBLK * 2048), a_rd,
                                       (const float LLMMM_LDS*)a_scale + (AGEN != 0 ? (kb + u - kb0) * 16 : 0), i);
      __builtin_amdgcn_sched_barrier(0);
      skinny_fetch<MBLK, APRE, AGEN != 0>(slot[u], ring_addr[u], wrow, w_kstep, w_off0, w_off1, ap, asp, bsp, min(kb + u + D, kb1 - 1), M);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
#define LLMMM_LAST(u)                                                              \
  if constexpr ((u) < D) {                                                         \
    skinny_wait<(D - 1 - (u)) * LOADS, MBLK, APRE, AGEN != 0>(slot[u]);                 \
    skinny_consume<MBLK, APRE, AGEN != 0>(slot[u], ring[u], w_rd, kb + (u) < kb1, acc,  \
                               a_tile + (min(kb + (u), kb1 - 1) - kb0) * (MBLK * 2048), a_rd, \
                               (const float LLMMM_LDS*)a_scale + (AGEN != 0 ? (min(kb + (u), kb1 - 1) - kb0) * 16 : 0), i); \
    __builtin_amdgcn_sched_barrier(0);                                             \
  }
  LLMMM_LAST(0) LLMMM_LAST(1) LLMMM_LAST(2) LLMMM_LAST(3) LLMMM_LAST(4) LLMMM_LAST(5) LLMMM_LAST(6) LLMMM_LAST(7)
#undef LLMMM_LAST

  // lane (g, i): row m = mb*16 + i, columns ncol .. ncol+3
  const int ncol = ng * 128 + wave * 16 + 4 * g;

  if (partial != nullptr) {
    // split-K (or an epilogue that lives in the second kernel only, S >= 1): this workgroup only stores its
    // plane of partial sums; a second kernel adds the planes in split order 0..S-1 and runs the
    // epilogue (fixed order, whatever the arrival order)
#pragma unroll
    for (int mb = 0; mb < MBLK; ++mb) {
      const int m = m0 + mb * 16 + i;
      if (m < M) *(f32x4*)(partial + ((size_t)sp * M + m) * N + ncol) = acc[mb];
    }
    return;
  }

  if constexpr (OUT == SK_OUT_F32) {
    float* C = (float*)Cv;
#pragma unroll
    for (int mb = 0; mb < MBLK; ++mb) {
      const int m = m0 + mb * 16 + i;
      if (m < M) *(f32x4*)(C + (size_t)m * N + ncol) = acc[mb];
    }
  }
  else if constexpr (OUT == SK_OUT_BF16) {
    __bf16* C = (__bf16*)Cv;
    typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
#pragma unroll
    for (int mb = 0; mb < MBLK; ++mb) {
      const int m = m0 + mb * 16 + i;
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
      float a = fmaxf(fmaxf(fmaxf(0.f, __builtin_fabsf(acc[mb][0])), __builtin_fabsf(acc[mb][1])),
                      fmaxf(__builtin_fabsf(acc[mb][2]), __builtin_fabsf(acc[mb][3])));
      a       = wave_xor_max(a, 16);
      a       = wave_xor_max(a, 32);
      if (g == 0) wave_amax[wave][mb][i] = a;
    }
    __syncthreads();
#pragma unroll
    for (int mb = 0; mb < MBLK; ++mb) {
      const int m    = m0 + mb * 16 + i;
      float     amax = 0.f;
#pragma unroll
      for (int w = 0; w < 8; ++w) amax = fmaxf(amax, wave_amax[w][mb][i]);
      const float scale = amax / 448.f;
      const float inv   = requant_inv(amax);
      if (m < M) {
        *(uint32_t*)(C + (size_t)m * N + ncol) =
          pack_e4m3x4_in_range(acc[mb][0] * inv, acc[mb][1] * inv, acc[mb][2] * inv, acc[mb][3] * inv);
        if (wave == 0 && g == 0) Cs[(size_t)ng * M + m] = scale;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------
// Column strips: one launch for the shapes whose few 128-column groups make the kernel above split K over several
// workgroups and leave the sum to a second kernel (the 2560-column projections O and down, QKV).  A workgroup owns 16
// output columns -- one wave's worth of weight rows -- over ALL of K; its eight waves take eight consecutive ranges of
// 128-K slices, each with the wave-private ring of the kernel above, and their partial sums meet in LDS, where they are
// added in wave order 0 .. 7: a fixed order, so results are the same run after run, with no planes, no workspace and no
// second launch.  N / 16 workgroups (160 for 2560 columns) stream the weights at the rate N / 128 x S workgroups of the
// split kernel did.  A strip holds an eighth of a 1x128 quantisation group, so this form serves the outputs without
// such groups: fp32, bf16, and hidden = T(C + residual) for the projections that end a decoder block.
// The activations come straight from global memory (L2) into the operand registers, slice by slice (M <= 32 rows).
// With CF = 2 a workgroup owns two adjacent 16-column fragments (a 32-column strip): waves 2 ks and 2 ks + 1 take K range ks
// of 4 for fragment 0 and 1 -- half the workgroups, for shapes whose 16-column strips would outnumber the CUs.
//
// The fused 1x128 re-quantisation (ST_OUT_FP8Q, M <= 16) needs the row maximum over a whole 128-column group, i.e. over
// the eight 16-column fragments -- eight workgroups, or four of two fragments -- that share the group.  They exchange just
// that: the wave that finishes a fragment publishes the maxima of its 16 columns (16 rows x 4 bytes) in a small exchange
// area in device memory and reads the other seven fragments' back, all with device-scope atomic stores and loads and no fence (nothing else is shared, and the values carry
// their own "written" mark), then quantises its own columns with the group's scale.  Against the split-K form this
// saves the second launch and the fp32 planes' round trip; it costs one store -> load hand-off through memory.
//
// The exchange area: g_strip_xch[area][buffer][group][fragment][row], zero when the library is loaded.  A slot holds
// (bits of the maximum) + 1 -- never 0, the maxima being non-negative floats and never NaN -- or 0 for "not written
// in this launch".  Two buffers take turns: a launch works in the buffer that holds zeros and, first of all, every
// fragment zeroes its own 16 slots of the other buffer (which its previous launch filled), so the next launch finds
// that one clean.  Which buffer is which, a fragment's wave reads off the fragment's own row-0 slot at kernel entry --
// written by no one but that fragment's wave, and all eight fragments of a group take part in every launch that touches
// the group, whatever the strip width, so they agree.  Nothing is reset from the host, nothing counts arrivals, and a
// captured graph can be replayed at will.  Launches that share an area must not overlap: the host gives every stream an
// area of its own (llmmm::strip_exchange_area) and keeps the split-K form for streams beyond the number of areas.
//
// Waiting for other workgroups is safe here because workgroups are dispatched in the order of their ids and the
// workgroups of a group have consecutive ids: whenever a wave waits, all workgroups with smaller ids have been
// dispatched, so the group with the smallest id that is still incomplete can always make progress.  The wait is bounded
// all the same (XCH_SPIN_TICKS of the 100 MHz clock): a wave that gives up counts itself in g_strip_xch_timeouts, which
// the host can read (llmmm_probe_strip_exchange_timeouts), and finishes with whatever it has -- every wave always
// reaches the end of the kernel.
constexpr int                XCH_AREAS = STRIP_XCH_AREAS, XCH_GROUPS = STRIP_XCH_MAX_GROUPS;
constexpr unsigned long long XCH_SPIN_TICKS = 2000000ull;  // 20 ms
static __device__ unsigned   g_strip_xch[XCH_AREAS][2][XCH_GROUPS][8][16];
static __device__ unsigned   g_strip_xch_timeouts;

enum { ST_OUT_F32 = 0, ST_OUT_BF16 = 1, ST_OUT_ADD = 2, ST_OUT_FP8Q = 3 };

// CF = 16-column fragments of a strip (1 or 2): with CF = 2 a workgroup owns 32 columns -- wave w takes fragment w % 2 and
// the K range (w / 2) of four -- so that N / 32 workgroups cover outputs whose N / 16 strips would be more than the CUs
// (a second round of workgroups costs more than the narrower K split: 6144 columns are 384 strips or 192 wide ones).
template <int MBLK, int OUT, int D, bool TAIL, typename HT, int CF = 1>
__global__ void __launch_bounds__(512)
fp8_strip_kernel(const uint8_t* __restrict__ A, const float* __restrict__ As, const uint8_t* __restrict__ Bt, const float* __restrict__ Bs,
                 void* __restrict__ Cv, const HT* __restrict__ residual, int M, int N, int K, int bpre, float* __restrict__ Cs, int xarea)
{
  static_assert(OUT != ST_OUT_FP8Q || MBLK == 1, "the exchange handles one 16-row block");
  static_assert(CF == 1 || CF == 2, "16 or 32 columns per workgroup");
  constexpr int KS = 8 / CF;  // K ranges per column fragment
  constexpr int LOADS = SKINNY_LOADS_PER_SLOT_BASE + 3 * MBLK;
  static_assert((D + (TAIL ? 1 : 0)) * LOADS < 64, "vmcnt is a 6-bit counter");
  static_assert(D >= 2 && D <= 4, "ring depths in use");
  __shared__ __attribute__((aligned(1024))) char ring0[8 * 2048];
  __shared__ __attribute__((aligned(1024))) char ring1[8 * 2048];
  __shared__ __attribute__((aligned(1024))) char ring2[D > 2 ? 8 * 2048 : 16];
  __shared__ __attribute__((aligned(1024))) char ring3[D > 3 ? 8 * 2048 : 16];
  __shared__ __attribute__((aligned(1024))) char tail_slot[TAIL ? 8 * 2048 : 16];
  __shared__ f32x4 part[8][MBLK][64];  // the waves' partial sums, lane for lane

  const int tid  = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g    = lane >> 4;
  const int i    = lane & 15;
  const int cf   = wave % CF;            // the wave's column fragment
  const int ks   = wave / CF;            // ... and its K range
  const int n0   = blockIdx.x * 16 * CF + 16 * cf;  // the wave's first column
  const int KB   = K >> 7;
  // K is dealt in whole slices: every wave takes q = KB / KS consecutive slices through its ring (q >= 1: the host checks
  // KB >= 8), and the KB % KS slices behind them go one each to the first K ranges as a "tail" slice, requested before
  // anything else and consumed last -- so the ring never runs over slices that are not the wave's own.  TAIL = (KB % KS != 0).
  const int q    = KB / KS;
  const int kb0  = ks * q, kb1 = kb0 + q;
  const int kbt  = KS * q + ks;          // the wave's tail slice ...
  const bool has_tail = kbt < KB;        // ... if there is one (otherwise the last slice is fetched in its place and not used)

  char LLMMM_LDS* const ring[4] = {(char LLMMM_LDS*)ring0 + wave * 2048, (char LLMMM_LDS*)ring1 + wave * 2048,
                                   (char LLMMM_LDS*)ring2 + wave * 2048, (char LLMMM_LDS*)ring3 + wave * 2048};
  char LLMMM_LDS* const tail = (char LLMMM_LDS*)tail_slot + wave * 2048;
  unsigned ring_addr[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) ring_addr[u] = __builtin_amdgcn_readfirstlane((unsigned)(size_t)ring[u]);
  const unsigned tail_addr = __builtin_amdgcn_readfirstlane((unsigned)(size_t)tail);

  // the strip's 16 weight rows: row-major Bt[N,K], or the pre-shuffled image, whose 2 KB blocks of consecutive slices follow each other
  const uint8_t*   wrow    = Bt + (size_t)n0 * K;
  const KMajorLane l0      = kmajor_lane<SWZ_ROWS16>(0, lane);
  const KMajorLane l1      = kmajor_lane<SWZ_ROWS16>(1, lane);
  const unsigned   w_off0  = bpre ? (unsigned)lane * 16u : (unsigned)(l0.row * K + l0.chunk * 16);
  const unsigned   w_off1  = bpre ? 1024u + (unsigned)lane * 16u : (unsigned)(l1.row * K + l1.chunk * 16);
  const int        w_kstep = bpre ? 2048 : 128;
  const int        w_rd    = kmajor_offset<SWZ_ROWS16>(i, 2 * g);
  const float*     bsp     = Bs + (size_t)(n0 >> 7) * KB;
  const uint8_t*   ap[MBLK];
  const float*     asp[MBLK];
#pragma unroll
  for (int mb = 0; mb < MBLK; ++mb) {
    const int m = min(mb * 16 + i, M - 1);  // rows beyond M repeat the last row; their sums are never stored
    ap[mb]      = A + (size_t)m * K + 32 * g;
    asp[mb]     = As + m;
  }
  f32x4 acc[MBLK];
#pragma unroll
  for (int mb = 0; mb < MBLK; ++mb) acc[mb] = f32x4{0.f, 0.f, 0.f, 0.f};

  // ST_OUT_FP8Q: the strip's own row-0 slot of exchange buffer 0 (non-zero: the strip's last launch worked in buffer 0),
  // requested before everything else (the oldest load in flight: it has landed whenever a ring slot has) and looked at
  // in the epilogue
  unsigned own_mark = 0u;
  if constexpr (OUT == ST_OUT_FP8Q) {
    const int frag = blockIdx.x * CF + cf;  // the 16-column fragment whose epilogue this wave may run: slot frag % 8 of group frag / 8
    asm volatile("global_load_dword %0, %1, off sc1" : "=v"(own_mark) : "v"(&g_strip_xch[xarea][0][frag >> 3][frag & 7][0]) : "memory");
  }

  // the tail slice first (the oldest loads in flight: landed whenever a ring slot has), then the wave's q slices through
  // its ring, D in flight (the pipeline of fp8_skinny_kernel)
  SkinnySlot<MBLK, false> tslot;
  if constexpr (TAIL) {
    skinny_fetch<MBLK, false>(tslot, tail_addr, wrow, w_kstep, w_off0, w_off1, ap, asp, bsp, min(kbt, KB - 1), M);
    __builtin_amdgcn_sched_barrier(0);
  }
  SkinnySlot<MBLK, false> slot[D];
#pragma unroll
  for (int u = 0; u < D; ++u) {
    skinny_fetch<MBLK, false>(slot[u], ring_addr[u], wrow, w_kstep, w_off0, w_off1, ap, asp, bsp, min(kb0 + u, kb1 - 1), M);
    __builtin_amdgcn_sched_barrier(0);
  }
  int kb = kb0;
  for (; kb + D < kb1; kb += D) {
#pragma unroll
    for (int u = 0; u < D; ++u) {
      skinny_wait<(D - 1) * LOADS, MBLK, false>(slot[u]);
      skinny_consume<MBLK, false>(slot[u], ring[u], w_rd, true, acc, nullptr, 0);
      __builtin_amdgcn_sched_barrier(0);
      skinny_fetch<MBLK, false>(slot[u], ring_addr[u], wrow, w_kstep, w_off0, w_off1, ap, asp, bsp, min(kb + u + D, kb1 - 1), M);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
#define LLMMM_LAST(u)                                                                 \
  if constexpr ((u) < D) {                                                            \
    skinny_wait<(D - 1 - (u)) * LOADS, MBLK, false>(slot[u]);                          \
    skinny_consume<MBLK, false>(slot[u], ring[u], w_rd, kb + (u) < kb1, acc, nullptr, 0); \
    __builtin_amdgcn_sched_barrier(0);                                                \
  }
  LLMMM_LAST(0) LLMMM_LAST(1) LLMMM_LAST(2) LLMMM_LAST(3)
#undef LLMMM_LAST
  if constexpr (TAIL) {
    skinny_wait<0, MBLK, false>(tslot);  // (long landed; ties its registers to this point)
    skinny_consume<MBLK, false>(tslot, tail, w_rd, has_tail, acc, nullptr, 0);
  }

#pragma unroll
  for (int mb = 0; mb < MBLK; ++mb) part[wave][mb][lane] = acc[mb];
  __syncthreads();
  if (wave >= MBLK * CF) return;  // wave mb * CF + c finishes column fragment c of the 16-row block mb
  const int mb = wave / CF;       // (wave % CF = cf: the fragment whose K ranges this wave summed one of)
  f32x4     v  = part[cf][mb][lane];
#pragma unroll
  for (int w = 1; w < KS; ++w) v += part[w * CF + cf][mb][lane];  // K ranges in order: the same sum whatever the waves' timing
  const int m = mb * 16 + i, ncol = n0 + 4 * g;  // lane (g, i): row m, columns ncol .. ncol + 3
  if constexpr (OUT == ST_OUT_FP8Q) {
    // (waves 0 .. CF-1 only, each on its own 16-column fragment exactly as a 16-column strip would be -- strips of either
    // width leave an area in the same state; rows beyond M take part with whatever their sums are: their maxima are
    // exchanged and never used)
    float a = fmaxf(fmaxf(fmaxf(0.f, __builtin_fabsf(v[0])), __builtin_fabsf(v[1])), fmaxf(__builtin_fabsf(v[2]), __builtin_fabsf(v[3])));
    a       = wave_xor_max(a, 16);
    a       = wave_xor_max(a, 32);  // the fragment's maximum of row i, in all four lanes that hold the row
    const int frag = blockIdx.x * CF + cf, grp = frag >> 3, strip = frag & 7;
    asm volatile("s_waitcnt vmcnt(0)" : "+v"(own_mark)::"memory");  // long landed; ties the register to this point
    const int cur = own_mark != 0u ? 1 : 0;  // the buffer this fragment did not fill last time (both clean: buffer 0)
    unsigned* mine_cur  = &g_strip_xch[xarea][cur][grp][strip][0];
    unsigned* mine_prev = &g_strip_xch[xarea][cur ^ 1][grp][strip][0];
    if (g == 0) {
      __hip_atomic_store(mine_prev + i, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(mine_cur + i, __builtin_bit_cast(unsigned, a) + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    // lane l polls rows 2 (l % 8), 2 (l % 8) + 1 of fragment l / 8: the group's 128 slots, 8 bytes per lane
    const unsigned long long* src = (const unsigned long long*)&g_strip_xch[xarea][cur][grp][0][0] + lane;
    unsigned long long        w;
    const unsigned long long  t0 = __builtin_amdgcn_s_memrealtime();
    for (;;) {
      w = __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const bool missing = (unsigned)w == 0u || (unsigned)(w >> 32) == 0u;
      if (__builtin_amdgcn_ballot_w64(missing) == 0ull) break;
      if (__builtin_amdgcn_s_memrealtime() - t0 > XCH_SPIN_TICKS) {  // (uniform: one clock reading per wave)
        if (lane == 0) atomicAdd(&g_strip_xch_timeouts, 1u);
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    float r0 = __builtin_bit_cast(float, (unsigned)w - 1u), r1 = __builtin_bit_cast(float, (unsigned)(w >> 32) - 1u);
#pragma unroll
    for (int step = 8; step <= 32; step <<= 1) r0 = wave_xor_max(r0, step), r1 = wave_xor_max(r1, step);  // over the group's fragments
    const float e0 = __shfl(r0, i >> 1, 64), e1 = __shfl(r1, i >> 1, 64);
    const float amax = (i & 1) ? e1 : e0;  // the group's maximum of row i
    const float scale = amax / 448.f;
    const float inv   = requant_inv(amax);
    if (m < M) {
      *(uint32_t*)((uint8_t*)Cv + (size_t)m * N + ncol) = pack_e4m3x4_in_range(v[0] * inv, v[1] * inv, v[2] * inv, v[3] * inv);
      if (strip == 0 && g == 0) Cs[(size_t)grp * M + m] = scale;
    }
    return;
  }
  if (m >= M) return;
  if constexpr (OUT == ST_OUT_F32)
    *(f32x4*)((float*)Cv + (size_t)m * N + ncol) = v;
  else if constexpr (OUT == ST_OUT_BF16)
    store_row4<__bf16>((__bf16*)Cv + (size_t)m * N + ncol, v);
  else {
    const f32x4 r = load_row4<HT>(residual + (size_t)m * N + ncol);
    store_row4<HT>((HT*)Cv + (size_t)m * N + ncol, v + r);  // one fp32 addition per element, then the hidden type's rounding
  }
}

// Ring depth: of 4, 3 and 2 the one that runs over the fewest slices beyond the q slices of a wave (a pass past
// the end re-fetches the last slice: wasted loads cost more here than a shallow ring -- down at M = 1, 9 slices per
// wave: 8.3 us with an 8-deep ring, 6.5 us with a 2-deep one); the deeper ring on ties.
// Strip width: 16 columns; 32 when 16-column strips would be more than the CUs, 32-column ones are not, and the weight
// matrix is small enough that a launch is short (measured, bf16 output at M = 1, us, 16 / 32 columns: 6144 x 2560 5.0 / 4.9,
// 6144 x 4096 6.2 / 5.9, 5120 x 5120 7.5 / 6.6 -- but 8192 x 8192, 67 MB, 11.8 / 13.3: 512 narrow strips sit two to a
// CU and pull more between them than one wide strip does).
int strip_fragments(int N, int K)
{
  return (N / 16 > num_cus() && N % 32 == 0 && N / 32 <= num_cus() && (long)N * K <= (32L << 20)) ? 2 : 1;
}
template <int MBLK, int OUT, typename HT, int CF>
static hipError_t launch_strip_cf(const void* A, const float* As, const void* Bt, const float* Bs, void* C, const void* residual, int M, int N, int K, int bpre,
                                  hipStream_t stream, float* Cs, int xarea)
{
  constexpr int KS = 8 / CF;
  const int  q = (K / 128) / KS;
  const dim3 grid(N / (16 * CF)), block(512);
  int        best = 2, waste = 1 << 30;
  for (int d = 4; d >= 2; --d) {
    const int w = (q + d - 1) / d * d - q;
    if (w < waste) best = d, waste = w;
  }
  const bool tail = (K / 128) % KS != 0;
#define LLMMM_GO(D)                                                                                                                                         \
  if (tail)                                                                                                                                                 \
    hipLaunchKernelGGL((fp8_strip_kernel<MBLK, OUT, D, true, HT, CF>), grid, block, 0, stream, (const uint8_t*)A, As, (const uint8_t*)Bt, Bs, C, (const HT*)residual, \
                       M, N, K, bpre, Cs, xarea);                                                                                                           \
  else                                                                                                                                                      \
    hipLaunchKernelGGL((fp8_strip_kernel<MBLK, OUT, D, false, HT, CF>), grid, block, 0, stream, (const uint8_t*)A, As, (const uint8_t*)Bt, Bs, C, (const HT*)residual, \
                       M, N, K, bpre, Cs, xarea)
  if (best == 4) {
    LLMMM_GO(4);
  }
  else if (best == 3) {
    LLMMM_GO(3);
  }
  else {
    LLMMM_GO(2);
  }
#undef LLMMM_GO
  return hipGetLastError();
}
template <int MBLK, int OUT, typename HT>
static hipError_t launch_strip(const void* A, const float* As, const void* Bt, const float* Bs, void* C, const void* residual, int M, int N, int K, int bpre,
                               hipStream_t stream, float* Cs = nullptr, int xarea = 0)
{
  return strip_fragments(N, K) == 2 ? launch_strip_cf<MBLK, OUT, HT, 2>(A, As, Bt, Bs, C, residual, M, N, K, bpre, stream, Cs, xarea)
                                 : launch_strip_cf<MBLK, OUT, HT, 1>(A, As, Bt, Bs, C, residual, M, N, K, bpre, stream, Cs, xarea);
}

hipError_t fp8_strip_launch(int out_kind, int b_layout, const void* A, const float* As, const void* Bt, const float* Bs, void* C, int M, int N, int K,
                            hipStream_t stream)
{
  if (M < 1 || M > STRIP_MAX_M || N % 16 || K % 128 || K / 128 < 8) return hipErrorInvalidValue;
  const int bpre = b_layout == LLMMM_FP8_B_PRESHUFFLED;
  if (out_kind == LLMMM_OUT_F32)
    return M <= 16 ? launch_strip<1, ST_OUT_F32, float>(A, As, Bt, Bs, C, nullptr, M, N, K, bpre, stream)
                   : launch_strip<2, ST_OUT_F32, float>(A, As, Bt, Bs, C, nullptr, M, N, K, bpre, stream);
  if (out_kind == LLMMM_OUT_BF16)
    return M <= 16 ? launch_strip<1, ST_OUT_BF16, float>(A, As, Bt, Bs, C, nullptr, M, N, K, bpre, stream)
                   : launch_strip<2, ST_OUT_BF16, float>(A, As, Bt, Bs, C, nullptr, M, N, K, bpre, stream);
  return hipErrorInvalidValue;
}

// The fused 1x128 re-quantisation in column strips (M <= 16, at most STRIP_XCH_MAX_GROUPS column groups): one launch, the
// fragments of a group agreeing on the row maxima through exchange area `xarea` (see above the kernel).
hipError_t fp8_strip_fp8q_launch(int b_layout, const void* A, const float* As, const void* Bt, const float* Bs, void* C, float* Cs, int M, int N, int K,
                                 int xarea, hipStream_t stream)
{
  if (M < 1 || M > 16 || N % 128 || N / 128 > XCH_GROUPS || K % 128 || K / 128 < 8 || xarea < 0 || xarea >= XCH_AREAS || !Cs) return hipErrorInvalidValue;
  return launch_strip<1, ST_OUT_FP8Q, float>(A, As, Bt, Bs, C, nullptr, M, N, K, b_layout == LLMMM_FP8_B_PRESHUFFLED, stream, Cs, xarea);
}

// Waves that gave up waiting in the exchange since the library was loaded (0 on a healthy device); synchronises.
hipError_t strip_exchange_timeouts(unsigned* out)
{
  return hipMemcpyFromSymbol(out, HIP_SYMBOL(g_strip_xch_timeouts), sizeof(unsigned), 0, hipMemcpyDeviceToHost);
}

template <typename HT>
static hipError_t strip_add(int b_layout, const void* A, const float* As, const void* Bt, const float* Bs, const void* residual, void* hidden, int M, int N, int K,
                            hipStream_t stream)
{
  const int bpre = b_layout == LLMMM_FP8_B_PRESHUFFLED;
  return M <= 16 ? launch_strip<1, ST_OUT_ADD, HT>(A, As, Bt, Bs, hidden, residual, M, N, K, bpre, stream)
                 : launch_strip<2, ST_OUT_ADD, HT>(A, As, Bt, Bs, hidden, residual, M, N, K, bpre, stream);
}

hipError_t fp8_strip_add_residual_launch(int hidden_dtype, int b_layout, const void* A, const float* As, const void* Bt, const float* Bs, const void* residual,
                                         void* hidden, int M, int N, int K, hipStream_t stream)
{
  if (M < 1 || M > STRIP_MAX_M || N % 16 || K % 128 || K / 128 < 8) return hipErrorInvalidValue;
  switch (hidden_dtype) {
    case LLMMM_DTYPE_F32: return strip_add<float>(b_layout, A, As, Bt, Bs, residual, hidden, M, N, K, stream);
    case LLMMM_DTYPE_BF16: return strip_add<__bf16>(b_layout, A, As, Bt, Bs, residual, hidden, M, N, K, stream);
    case LLMMM_DTYPE_F16: return strip_add<_Float16>(b_layout, A, As, Bt, Bs, residual, hidden, M, N, K, stream);
    default: return hipErrorInvalidValue;
  }
}

template <int MBLK, int OUT, int D, int ASTG>
static hipError_t launch_skinny(const void* A, const float* As, const void* Bt, const float* Bs, void* C, float* Cs, int M,
                                int N, int K, int S, float* partial, int bpre, hipStream_t stream)
{
  hipLaunchKernelGGL((fp8_skinny_kernel<MBLK, OUT, D, ASTG>), dim3(N / 128, S, (M + 16 * MBLK - 1) / (16 * MBLK)), dim3(512), 0, stream,
                     (const uint8_t*)A, As, (const uint8_t*)Bt, Bs, C, Cs, M, N, K, S, partial, bpre, SkinnyGenA{});
  return hipGetLastError();
}

// Generated activations (AGEN): M <= 16, the K range of a split must fit the staging buffer.
template <int OUT>
static hipError_t dispatch_skinny_agen(const float* G, const void* Bt, const float* Bs, void* C, float* Cs, int M, int N, int K, int S, float* partial,
                                       int bpre, hipStream_t stream)
{
  const int KB = K / 128, slices = KB / S, longest = (KB + S - 1) / S, need = 2048 * longest;
  if (M > 16 || need > 65536) return hipErrorInvalidValue;
#define LLMMM_GO(D, ASTG)                                                                                                                   \
  {                                                                                                                                         \
    hipLaunchKernelGGL((fp8_skinny_kernel<1, OUT, D, ASTG, 1>), dim3(N / 128, S, 1), dim3(512), 0, stream, (const uint8_t*)G, (const float*)nullptr, \
                       (const uint8_t*)Bt, Bs, C, Cs, M, N, K, S, partial, bpre, SkinnyGenA{});                                            \
    return hipGetLastError();                                                                                                               \
  }
  if (slices >= 8 && need <= 28672) LLMMM_GO(8, 28672);
  if (slices >= 4) LLMMM_GO(4, 65536);
  LLMMM_GO(2, 65536);
#undef LLMMM_GO
}

hipError_t fp8_skinny_swiglu_a_launch(int out_kind, int b_layout, const float* G, const void* Bt, const float* Bs, void* C, float* Cs, int M, int N,
                                      int K, int S, float* partial, hipStream_t stream)
{
  const int bpre = b_layout == LLMMM_FP8_B_PRESHUFFLED;
  switch (out_kind) {
    case SK_OUT_F32: return dispatch_skinny_agen<SK_OUT_F32>(G, Bt, Bs, C, Cs, M, N, K, S, partial, bpre, stream);
    case SK_OUT_BF16: return dispatch_skinny_agen<SK_OUT_BF16>(G, Bt, Bs, C, Cs, M, N, K, S, partial, bpre, stream);
    case SK_OUT_FP8Q: return dispatch_skinny_agen<SK_OUT_FP8Q>(G, Bt, Bs, C, Cs, M, N, K, S, partial, bpre, stream);
    default: return hipErrorInvalidValue;
  }
}

template <typename HT>
static hipError_t dispatch_skinny_gen2(const SkinnyGenA& ag, const void* Bt, const float* Bs, float* C, int M, int N, int K, int S, float* partial, int bpre,
                                       hipStream_t stream)
{
  const int KB = K / 128, slices = KB / S, longest = (KB + S - 1) / S, need = 2048 * longest;
  if (M > 2 || K > 3072 || need > 65536 || ag.splits < 1 || ag.splits > SKINNY_GEN_MAX_PLANES || ag.hidden == ag.residual) return hipErrorInvalidValue;
#define LLMMM_GO(D, ASTG)                                                                                                                       \
  {                                                                                                                                             \
    hipLaunchKernelGGL((fp8_skinny_kernel<1, SK_OUT_F32, D, ASTG, 2, HT>), dim3(N / 128, S, 1), dim3(512), 0, stream, (const uint8_t*)nullptr,  \
                       (const float*)nullptr, (const uint8_t*)Bt, Bs, (void*)C, (float*)nullptr, M, N, K, S, partial, bpre, ag);                \
    return hipGetLastError();                                                                                                                   \
  }
  if (slices >= 8 && need <= 28672) LLMMM_GO(8, 28672);
  if (slices >= 4) LLMMM_GO(4, 65536);
  LLMMM_GO(2, 65536);
#undef LLMMM_GO
}

hipError_t fp8_skinny_rmsnorm_a_launch(int hidden_dtype, int b_layout, const SkinnyGenA& ag, const void* Bt, const float* Bs, float* C, int M, int N, int K,
                                       int S, float* partial, hipStream_t stream)
{
  const int bpre = b_layout == LLMMM_FP8_B_PRESHUFFLED;
  switch (hidden_dtype) {
    case LLMMM_DTYPE_F32: return dispatch_skinny_gen2<float>(ag, Bt, Bs, C, M, N, K, S, partial, bpre, stream);
    case LLMMM_DTYPE_BF16: return dispatch_skinny_gen2<__bf16>(ag, Bt, Bs, C, M, N, K, S, partial, bpre, stream);
    case LLMMM_DTYPE_F16: return dispatch_skinny_gen2<_Float16>(ag, Bt, Bs, C, M, N, K, S, partial, bpre, stream);
    default: return hipErrorInvalidValue;
  }
}

// Ring depth D: the largest that does not exceed the slices of the shortest split.  Activation
// staging: whenever the rows of the longest split fit next to the ring (28 KB beside the
// 8-deep ring, 64 KB beside a 4-deep one); otherwise the per-slice register path.
template <int OUT>
static hipError_t dispatch_skinny(const void* A, const float* As, const void* Bt, const float* Bs, void* C, float* Cs, int M,
                                  int N, int K, int S, float* partial, int bpre, hipStream_t stream)
{
  const int KB     = K / 128;
  const int slices = KB / S;              // of the shortest split
  const int longest = (KB + S - 1) / S;   // of the longest
#define LLMMM_GO(MBLK, D, ASTG) return launch_skinny<MBLK, OUT, D, ASTG>(A, As, Bt, Bs, C, Cs, M, N, K, S, partial, bpre, stream)
  if (M <= 16) {
    const int need = 2048 * longest;
    if (slices >= 8 && need <= 28672) LLMMM_GO(1, 8, 28672);
    if (slices >= 4 && need <= 65536) LLMMM_GO(1, 4, 65536);
    if (need <= 65536) LLMMM_GO(1, 2, 65536);
    if (slices >= 8) LLMMM_GO(1, 8, 0);
    if (slices >= 4) LLMMM_GO(1, 4, 0);
    LLMMM_GO(1, 2, 0);
  }
  if (M <= 32) {
    const int need = 2 * 2048 * longest;
    if (slices >= 4 && need <= 65536) LLMMM_GO(2, 4, 65536);
    if (need <= 65536) LLMMM_GO(2, 2, 65536);
    if (slices >= 4 && need <= 81920) LLMMM_GO(2, 4, 81920);  // 20 slices (K = 2560 unsplit): 80 KB beside a 4-deep ring
    if (slices >= 4) LLMMM_GO(2, 4, 0);
    LLMMM_GO(2, 2, 0);
  }
  if (M > 64 && M <= 128 && 8 * 2048 * longest <= 65536) {  // one pass over the weights for all rows
    if (slices >= 4) LLMMM_GO(8, 4, 65536);
    LLMMM_GO(8, 2, 65536);
  }
  if (M <= 128) {  // two row groups of (up to) 64 when M > 64
    const int need = 4 * 2048 * longest;
    if (slices >= 4 && need <= 65536) LLMMM_GO(4, 4, 65536);
    if (need <= 65536) LLMMM_GO(4, 2, 65536);
    // K ranges too long to stage 64 rows of: row groups of 32 whose rows still fit (every group streams the weights of
    // its columns again, from L2) -- 128 x 6144 x 2560 unsplit: 10.6 us in four groups, one launch, against 13.3 us in
    // five splits + reduce and 42 us with the activations fetched per wave and slice
    if (slices >= 4 && 2 * 2048 * longest <= 81920) LLMMM_GO(2, 4, 81920);
    if (slices >= 4) LLMMM_GO(4, 4, 0);
    LLMMM_GO(4, 2, 0);
  }
#undef LLMMM_GO
  return hipErrorInvalidValue;
}

hipError_t fp8_skinny_launch(int out_kind, int b_layout, const void* A, const float* As, const void* Bt, const float* Bs, void* C,
                             float* Cs, int M, int N, int K, int S, float* partial, hipStream_t stream)
{
  const int bpre = b_layout == LLMMM_FP8_B_PRESHUFFLED;
  switch (out_kind) {
    case SK_OUT_F32: return dispatch_skinny<SK_OUT_F32>(A, As, Bt, Bs, C, Cs, M, N, K, S, partial, bpre, stream);
    case SK_OUT_BF16: return dispatch_skinny<SK_OUT_BF16>(A, As, Bt, Bs, C, Cs, M, N, K, S, partial, bpre, stream);
    case SK_OUT_FP8Q: return dispatch_skinny<SK_OUT_FP8Q>(A, As, Bt, Bs, C, Cs, M, N, K, S, partial, bpre, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace llmmm
