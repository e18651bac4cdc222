// FP8 (OCP e4m3) blockwise-scaled GEMM for gfx950 with fp32 / bf16 output, the fused per-1x128
// re-quantisation of C, or the same re-quantisation of silu(gate) * up (SwiGLU) for a gate_up projection.
//
//   C[m,n] = sum_kb ( sum_{k in 128-slice kb} Aq[m,k] * Bq[n,k] ) * As[kb,m] * Bs[n/128,kb]
//
// Replaces the reference kernels fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32
// (examples/005.fp8.mm.cu:51-246) and ...__C_1x128__output_fp8 (canonical form
// examples/005.fp8.mm.opt.cu:177-465).  Layouts as there: A [M,K] e4m3, A_scale_transposed
// [K/128,M], B_transposed [N,K] e4m3, B_scale [N/128,K/128], C [M,N], C_scale_transposed
// [N/128,M] (examples/005.fp8.mm.cu:131,157,168,212,774).
//
// Design:
//  * v_mfma_f32_16x16x128_f8f6f4 (both operands e4m3): one instruction covers one 128-wide
//    quantisation slice of a 16x16 output block, started from C = 0, so the slice's partial sum
//    comes back as 4 fp32 registers per lane;
//  * the slice scale As[kb,m]*Bs[nb,kb] is applied with one v_fma_f32 per accumulator
//    (promotion once per 128-K slice, the order of examples/005.fp8.mm.cu:885-902); Bt is the
//    row operand and A the column operand, so a lane owns one row m and its scale is a single
//    register per 16-row fragment;
//  * one stage = one slice: a BM x 128 B tile of A and a BN x 128 B tile of Bt, both K-major,
//    land in LDS by LDS-direct loads (two stages in flight; three or four with the slice scales in the
//    stage when a single tile row streams the weights) and are read with ds_read_b128 through the
//    SWZ_ROWS16 placement; the weights may also arrive pre-shuffled into that placement (layout.hip);
//  * split-K: gridDim.y workgroups per tile write fp32 planes, and a second kernel adds them in split
//    order and runs the epilogue (fixed order: results do not depend on timing);
//  * fused epilogue (examples/005.fp8.mm.opt.cu:401-462): a wavefront owns 64 rows x one whole
//    128-column quantisation group, so the row amax needs the lane's 32 values and two
//    cross-lane steps; scale = amax/448, codes = e4m3(C * (448/amax)), saturating.
//    A group of zeros yields scale 0 and codes 0 (the reference's unguarded 0*inf gives NaN codes).
#include <type_traits>
#include "device_common.hip.h"
#include "kernels.h"

namespace llmmm {

enum { OUT_F32 = 0, OUT_BF16 = 1, OUT_FP8Q = 2, OUT_SWIGLU = 3,
       // internal: the bf16 / e4m3 epilogues behind the per-head RMSNorm + RoPE of a QKV projection (Fp8HeadOp)
       OUT_ROPE_BF16 = 4, OUT_ROPE_FP8Q = 5,
       // internal: hidden = T(C + residual), T = float / bf16 / fp16 (Fp8HeadOp::residual, the output goes to Cv)
       OUT_ADD_F32 = 6, OUT_ADD_BF16 = 7, OUT_ADD_F16 = 8 };

__device__ __forceinline__ f32x4 mfma_fp8_k128(i32x8 x, i32x8 y)
{
  const f32x4 z = {0.f, 0.f, 0.f, 0.f};
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(x, y, z, 0, 0, 0, 0, 0, 0);
}

// WM = rows of a wave's sub-tile (64 or 32); its columns are 128, one quantisation group -- or, in the 160-column tile
// (BN = 160: 2560-column outputs in 16 tiles per row, one per CU at M = 2048), 160, which straddle two weight-scale blocks.
template <int BM, int BN, int WM>
struct Fp8Tile {
  static constexpr int MF      = WM / 16;  // 16-row fragments per wave
  static constexpr int WN      = BN % 128 == 0 ? 128 : BN;  // columns of a wave
  static constexpr int NF      = WN / 16;                   // 16-column fragments per wave
  static constexpr int WAVES_M = BM / WM;
  static constexpr int WAVES_N = BN / WN;
  static constexpr int NW      = WAVES_M * WAVES_N;
  static constexpr int NT      = NW * 64;
  static constexpr int A_BYTES = BM * 128;
  static constexpr int B_BYTES = BN * 128;
  static constexpr int STAGE   = A_BYTES + B_BYTES;
  static constexpr int A_LOADS = (BM / 8) / NW;
  static constexpr int B_LOADS = (BN / 8) / NW;
};

// Operand and scale loads of the main loop are written as inline assembly, with a wave-uniform
// base in SGPRs and one constant per-lane byte offset, and the kernel places its own s_waitcnt:
// the compiler then never sees an LDS-direct load in flight (it would turn every wait it
// inserts into "all loads done"), and no vector ALU work goes into addresses.
__device__ __forceinline__ void fp8_load_lds_16B(const void* sbase, unsigned voff, unsigned lds_addr)
{
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "s"(lds_addr) : "memory");
}
// The same load with the non-temporal hint, for weights that only one workgroup reads (a single
// tile row): streamed through, they do not displace the activations and scales every workgroup
// shares.  Measured: about 1 us faster at M = 128 on the N = 19456 and K = 9728 shapes -- and 10-50 %
// slower wherever several tile rows re-read the weights from the L2, so only used for one row.
__device__ __forceinline__ void fp8_load_lds_16B_nt(const void* sbase, unsigned voff, unsigned lds_addr)
{
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt" ::"v"(voff), "s"(sbase), "s"(lds_addr) : "memory");
}
template <int IMM>
__device__ __forceinline__ void fp8_load_f32(float& dst, const void* sbase, unsigned voff)
{
  asm volatile("global_load_dword %0, %1, %2 offset:%3" : "=v"(dst) : "v"(voff), "s"(sbase), "n"(IMM) : "memory");
}

// Load i (0 .. A_LOADS + B_LOADS - 1) of a wave for one stage.  All loads of a wave share one
// per-lane offset: load i covers tile rows 8*(wave + i*NW) .. +7, and the SWZ_ROWS16 placement
// only looks at row bits 0..3, so moving by 8*NW (>= 16) rows changes nothing but the
// wave-uniform row base.
//
// Pre-shuffled weights (layout.hip) hold the same LDS image as consecutive 1 KB half blocks: half
// block h of row group rg and slice kb at ((rg * K/128 + kb) * 2 + h) * 1024.  Rows 8*NW apart
// are then 8*NW*K bytes apart as well, so only the per-lane offset (16 * lane instead of
// row * K + chunk * 16, the wave's own rows folded into the base) and the step from slice to
// slice (2048 instead of 128 bytes) differ between the two layouts.
//
// MT (a last tile row with fewer than BM rows of A): the lanes of load i whose row lies beyond the matrix fetch its
// last row instead, so the per-lane offset differs from load to load -- a_tail[i], relative to the tile's first row.
template <int BM, int BN, int WM, bool BNT, int I, bool MT = false>
__device__ __forceinline__ void fp8_issue_load(unsigned lds_stage, const uint8_t* Ag, const uint8_t* Bg, unsigned a_off, unsigned b_off, int K, size_t b_hi, int wave,
                                               const unsigned* a_tail = nullptr)
{
  typedef Fp8Tile<BM, BN, WM> TC;
  // b_hi: extra byte offset of the tile's upper half of weight rows (0 unless the two halves come from different row ranges)
  const size_t b_skip = I - TC::A_LOADS >= TC::B_LOADS / 2 ? b_hi : 0;
  if constexpr (I < TC::A_LOADS) {
    if constexpr (MT)
      fp8_load_lds_16B(Ag, a_tail[I], lds_stage + (wave + I * TC::NW) * 1024);
    else
      fp8_load_lds_16B(Ag + (size_t)(8 * TC::NW * I) * K, a_off, lds_stage + (wave + I * TC::NW) * 1024);
  }
  else if constexpr (I < TC::A_LOADS + TC::B_LOADS) {
    if constexpr (BNT)
      fp8_load_lds_16B_nt(Bg + (size_t)(8 * TC::NW * (I - TC::A_LOADS)) * K + b_skip, b_off, lds_stage + TC::A_BYTES + (wave + (I - TC::A_LOADS) * TC::NW) * 1024);
    else
      fp8_load_lds_16B(Bg + (size_t)(8 * TC::NW * (I - TC::A_LOADS)) * K + b_skip, b_off, lds_stage + TC::A_BYTES + (wave + (I - TC::A_LOADS) * TC::NW) * 1024);
  }
}
template <int BM, int BN, int WM, bool BNT, int FIRST, int COUNT, bool MT = false>
__device__ __forceinline__ void fp8_issue_loads(unsigned lds_stage, const uint8_t* Ag, const uint8_t* Bg, unsigned a_off, unsigned b_off, int K, size_t b_hi, int wave,
                                                const unsigned* a_tail = nullptr)
{
  if constexpr (COUNT > 0) {
    fp8_issue_load<BM, BN, WM, BNT, FIRST, MT>(lds_stage, Ag, Bg, a_off, b_off, K, b_hi, wave, a_tail);
    fp8_issue_loads<BM, BN, WM, BNT, FIRST + 1, COUNT - 1, MT>(lds_stage, Ag, Bg, a_off, b_off, K, b_hi, wave, a_tail);
  }
}
// The slice scales of the lane's four 16-row fragments and of the wave's column group.
// (TWO: a 160-column wave also takes the scale of the next weight block, Bs_elem2.)
template <int MF, bool TWO = false>
__device__ __forceinline__ void fp8_issue_scales(float (&sa)[MF], float& sb, const float* As_slice, unsigned row_off, const float* Bs_elem, unsigned zero,
                                                 float* sb2 = nullptr, const float* Bs_elem2 = nullptr)
{
  fp8_load_f32<0>(sa[0], As_slice, row_off);
  fp8_load_f32<64>(sa[1], As_slice, row_off);
  if constexpr (MF == 4) {
    fp8_load_f32<128>(sa[2], As_slice, row_off);
    fp8_load_f32<192>(sa[3], As_slice, row_off);
  }
  fp8_load_f32<0>(sb, Bs_elem, zero);
  if constexpr (TWO) fp8_load_f32<0>(*sb2, Bs_elem2, zero);
}

// 32 bytes of one row: chunk 2g at rd0 and chunk 2g+1 at rd1 (= rd0 ^ 16); `imm` selects the
// 16-row fragment (a multiple of 2048 bytes, which the swizzle does not see).
__device__ __forceinline__ i32x8 fp8_read_frag(const char LLMMM_LDS* tile, int rd0, int rd1, int imm)
{
  union {
    i32x4 h[2];
    i32x8 v;
  } u;
  u.h[0] = *(const i32x4 LLMMM_LDS*)(tile + rd0 + imm);
  u.h[1] = *(const i32x4 LLMMM_LDS*)(tile + rd1 + imm);
  return u.v;
}

// What a slice issues for its successor while it computes.
struct Fp8Next {
  unsigned       lds_stage;  // LDS byte address of the stage buffer to fill
  const uint8_t* Ag;         // tile's A rows / Bt rows at the next slice's k offset
  const uint8_t* Bg;
  const float*   As_slice;   // As + kb_next * M
  const float*   Bs_elem;    // &Bs[nb, kb_next]
  const float*   Bs_elem2;   // 160-column waves: &Bs[nb + 1, kb_next]
  const char*    sc_ptr;     // deep pipeline only: this lane's scale of the slice being requested (see fp8_scale_load_lds)
};

// Deep pipeline: the slice scales travel with the stage.  One 4-byte LDS-direct load per wave and slice: lanes
// 0 .. WM-1 fetch As[kb, row] of the wave's rows, the other lanes all fetch Bs[nb, kb]; lane l's value lands at
// lds_addr + 4*l, so the wave later reads its row scales at 4*(16*mf + i) and the column-group scale at 128.
__device__ __forceinline__ void fp8_scale_load_lds(const char* lane_ptr, unsigned lds_addr)
{
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(lane_ptr), "s"(lds_addr) : "memory");
}

// One 128-K slice of the wave's WM x 128 sub-tile.  s[mf] = As[kb, row] * Bs[nb, kb].
// With LOAD, the next stage's loads go out two or more per fragment step during the first four
// steps (spread, so that no wave sits in the memory pipeline's issue queue while its matrix
// work waits, and early enough to land within the slice), its scales during the fifth.
// 160-column waves (NF = 10): fragments nf < nfb lie in the first weight-scale block and take s, the others s2.
template <int BM, int BN, int WM, bool BNT, bool LOAD, bool SCALE_LDS = false, bool MT = false>
__device__ __forceinline__ void fp8_compute_stage(const char LLMMM_LDS* lds, int a_rd0, int a_rd1, int b_rd0, int b_rd1,
                                                  const float (&s)[WM / 16], f32x4 (&acc)[Fp8Tile<BM, BN, WM>::NF][WM / 16], const Fp8Next& nx, unsigned lane_off,
                                                  unsigned b_lane_off, unsigned row_off, unsigned zero, int K, size_t b_hi, int wave, float (&sa_next)[WM / 16],
                                                  float& sb_next, const float (&s2)[WM / 16], int nfb, float& sb2_next, const unsigned* a_tail = nullptr)
{
  constexpr int MF = WM / 16;
  typedef Fp8Tile<BM, BN, WM> TC;
  constexpr int  NF  = TC::NF;
  constexpr bool TWO = NF != 8;
  constexpr int           NL   = TC::A_LOADS + TC::B_LOADS;
  constexpr int           LPG  = (NL + 3) / 4;
  const char LLMMM_LDS*   ldsA = lds;
  const char LLMMM_LDS*   ldsB = lds + TC::A_BYTES;
  i32x8                   a[MF], b[2];
  f32x4                   p[2][MF];
  // the first MFMA needs b[0] and a[0] only: they are requested first (pinned: the scheduler would otherwise put all of A
  // in front), so that it waits for four LDS reads instead of eleven while all eight waves read at once behind the barrier
  b[0] = fp8_read_frag(ldsB, b_rd0, b_rd1, 0);
  a[0] = fp8_read_frag(ldsA, a_rd0, a_rd1, 0);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int mf = 1; mf < MF; ++mf) a[mf] = fp8_read_frag(ldsA, a_rd0, a_rd1, mf * 2048);
#pragma unroll
  for (int nf = 0; nf < NF; ++nf) {
    const int cur = nf & 1;
    if (nf + 1 < NF) b[cur ^ 1] = fp8_read_frag(ldsB, b_rd0, b_rd1, (nf + 1) * 2048);
    if constexpr (LOAD) {
      if (nf == 0) fp8_issue_loads<BM, BN, WM, BNT, 0, LPG, MT>(nx.lds_stage, nx.Ag, nx.Bg, lane_off, b_lane_off, K, b_hi, wave, a_tail);
      if (nf == 1) fp8_issue_loads<BM, BN, WM, BNT, LPG, LPG, MT>(nx.lds_stage, nx.Ag, nx.Bg, lane_off, b_lane_off, K, b_hi, wave, a_tail);
      if (nf == 2) fp8_issue_loads<BM, BN, WM, BNT, 2 * LPG, LPG, MT>(nx.lds_stage, nx.Ag, nx.Bg, lane_off, b_lane_off, K, b_hi, wave, a_tail);
      if (nf == 3) fp8_issue_loads<BM, BN, WM, BNT, 3 * LPG, LPG, MT>(nx.lds_stage, nx.Ag, nx.Bg, lane_off, b_lane_off, K, b_hi, wave, a_tail);
      if (nf == 4) {
        if constexpr (SCALE_LDS)
          fp8_scale_load_lds(nx.sc_ptr, nx.lds_stage + TC::STAGE + wave * 256);
        else
          fp8_issue_scales<MF, TWO>(sa_next, sb_next, nx.As_slice, row_off, nx.Bs_elem, zero, &sb2_next, nx.Bs_elem2);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int mf = 0; mf < MF; ++mf) p[cur][mf] = mfma_fp8_k128(b[cur], a[mf]);
    if (nf > 0) {
#pragma unroll
      for (int mf = 0; mf < MF; ++mf) {
        const float sc = TWO ? (nf - 1 < nfb ? s[mf] : s2[mf]) : s[mf];
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[nf - 1][mf][r] = __builtin_fmaf(p[cur ^ 1][mf][r], sc, acc[nf - 1][mf][r]);
      }
      // Pin the promotion here (an empty asm the optimiser cannot move or sink), then ask for
      // MFMA, 4 FMA, MFMA, 4 FMA ...: the FMAs of fragment nf-1 run under the MFMAs of fragment nf.
#pragma unroll
      for (int mf = 0; mf < MF; ++mf) asm volatile("" : "+v"(acc[nf - 1][mf]));
#pragma unroll
      for (int mf = 0; mf < MF; ++mf) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
#pragma unroll
  for (int mf = 0; mf < MF; ++mf) {
    const float sc = TWO ? (NF - 1 < nfb ? s[mf] : s2[mf]) : s[mf];
#pragma unroll
    for (int r = 0; r < 4; ++r) acc[NF - 1][mf][r] = __builtin_fmaf(p[(NF - 1) & 1][mf][r], sc, acc[NF - 1][mf][r]);
  }
#pragma unroll
  for (int mf = 0; mf < MF; ++mf) asm volatile("" : "+v"(acc[NF - 1][mf]));
}

// SwiGLU exchange: the fragments mf = SEND0 .. SEND0 + MF/2 - 1 go to the partner wave through LDS, lane for lane.
template <int MF, int SEND0>
__device__ __forceinline__ void swiglu_send(const f32x4 (&acc)[8][MF], char LLMMM_LDS* region, int lane)
{
#pragma unroll
  for (int nf = 0; nf < 8; ++nf)
#pragma unroll
    for (int h = 0; h < MF / 2; ++h) *(f32x4 LLMMM_LDS*)(region + ((h * 8 + nf) * 64 + lane) * 16) = acc[nf][SEND0 + h];
}

// The kept fragments mf = KEEP0 .. (own values: gate if IS_GATE, else up) meet the partner's values of the same
// rows and columns: h = silu(gate) * up, then the fused 1x128 quantisation of h exactly as for plain C
// (examples/005.fp8.mm.opt.cu:401-462), staged row-major in `stg` and stored as whole 128-byte rows.
template <int MF, int KEEP0, bool IS_GATE>
__device__ __forceinline__ void swiglu_finish(const f32x4 (&acc)[8][MF], const f32x4 (&other)[8][MF / 2], char LLMMM_LDS* stg, uint8_t* C,
                                              float* Cs_col, int ldc, int row0, int col0, int lane)
{
  constexpr int MH = MF / 2;
  const int     g = lane >> 4, li = lane & 15;
#pragma unroll
  for (int h = 0; h < MH; ++h) {
    f32x4 v[8];
    float amax = 0.f;
#pragma unroll
    for (int nf = 0; nf < 8; ++nf)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float mine = acc[nf][KEEP0 + h][q], theirs = other[nf][h][q];
        v[nf][q]         = IS_GATE ? silu_mul(mine, theirs) : silu_mul(theirs, mine);
        amax             = fmaxf(amax, __builtin_fabsf(v[nf][q]));
      }
    amax              = wave_xor_max(amax, 16);
    amax              = wave_xor_max(amax, 32);
    const float scale = amax / 448.f;
    const float inv   = requant_inv(amax);
    const int   r     = h * 16 + li;
#pragma unroll
    for (int nf = 0; nf < 8; ++nf)
      *(uint32_t LLMMM_LDS*)(stg + r * 128 + ((nf ^ ((r >> 1) & 7)) << 4) + 4 * g) =
        pack_e4m3x4_in_range(v[nf][0] * inv, v[nf][1] * inv, v[nf][2] * inv, v[nf][3] * inv);
    if (g == 0) Cs_col[row0 + KEEP0 * 16 + r] = scale;
  }
#pragma unroll
  for (int j = 0; j < MH * 2; ++j) {
    const int   r = 8 * j + (lane >> 3), c = lane & 7;
    const i32x4 x = *(const i32x4 LLMMM_LDS*)(stg + r * 128 + ((c ^ ((r >> 1) & 7)) << 4));
    *(i32x4*)(C + (size_t)(row0 + KEEP0 * 16 + r) * ldc + col0 + c * 16) = x;
  }
}

// Per-head RMSNorm + rotary embedding on the accumulators of one wave, which hold WM rows x one whole head (128
// columns): lane (g, li) owns row mf*16 + li, columns nf*16 + 4g + q.  Same arithmetic, in the same order, as
// fp8_planes_qk_norm_rope_kernel: the 4-column chunk c = nf*4 + g is that kernel's lane c, so the butterfly over chunk
// bits 4, 3, 2 runs over nf inside the lane (all eight results are equal, one is computed) and bits 1, 0 over g across
// lanes (xor 32, xor 16); column i < 64 and its partner i + 64 are fragments nf and nf + 4 of the same lane.
//
// The cos / sin values a lane needs (four 16-byte pieces of each table per row) come through the wave's private piece
// of the idle operand buffers, `tab` (MF * 4 KB), by LDS-direct loads whose lane l lands at +16 l -- the lane layout the
// rotation reads them back in.  Half of the rows per pass, every load of a pass in flight at once and none of them
// holding registers: fetched into registers instead, the 128 accumulator registers leave room for a few pieces at a
// time and the epilogue pays one L2 round trip after the other (2048 x 6144 x 2560: 43 us with, 33.6 us without rope).
template <int MF>
__device__ __forceinline__ void qk_norm_rope_fragments(f32x4 (&acc)[8][MF], const Fp8HeadOp& op, int head, int row0, int lane, char LLMMM_LDS* tab)
{
  if (head >= op.n_q + op.n_kv) return;  // value head (wave-uniform)
  constexpr int MFP = MF / 2;            // 16-row fragments per pass
  static_assert(MF % 2 == 0, "two passes");
  const int      g = lane >> 4, li = lane & 15;
  const unsigned tab_addr = (unsigned)(size_t)tab;
  unsigned       toff[MF];  // byte offset of the lane's first piece in either table
#pragma unroll
  for (int mf = 0; mf < MF; ++mf) toff[mf] = (unsigned)min(max(op.pos[row0 + mf * 16 + li], 0), op.table_rows - 1) * 256u + 16u * g;
  // pass h: pieces (m, nf, table) of fragments mf = h * MFP + m at tab + ((m * 4 + nf) * 2 + table) * 1024
#define LLMMM_ROPE_FETCH(H)                                                                                  \
  _Pragma("unroll") for (int m = 0; m < MFP; ++m) _Pragma("unroll") for (int nf = 0; nf < 4; ++nf) {         \
    fp8_load_lds_16B(op.cos_t, toff[(H) * MFP + m] + 64u * nf, tab_addr + ((m * 4 + nf) * 2 + 0) * 1024);    \
    fp8_load_lds_16B(op.sin_t, toff[(H) * MFP + m] + 64u * nf, tab_addr + ((m * 4 + nf) * 2 + 1) * 1024);    \
  }
#define LLMMM_ROPE_ROTATE(H)                                                                                 \
  _Pragma("unroll") for (int m = 0; m < MFP; ++m) {                                                          \
    const int mf = (H) * MFP + m;                                                                            \
    _Pragma("unroll") for (int nf = 0; nf < 4; ++nf) {                                                       \
      const f32x4 cs = *(const f32x4 LLMMM_LDS*)(tab + ((m * 4 + nf) * 2 + 0) * 1024 + lane * 16);           \
      const f32x4 sn = *(const f32x4 LLMMM_LDS*)(tab + ((m * 4 + nf) * 2 + 1) * 1024 + lane * 16);           \
      _Pragma("unroll") for (int q = 0; q < 4; ++q) {                                                        \
        const float lo = acc[nf][mf][q], hi = acc[nf + 4][mf][q];                                            \
        const float t1 = hi * sn[q], t2 = lo * sn[q];                                                        \
        acc[nf][mf][q]     = __builtin_fmaf(lo, cs[q], -t1);                                                 \
        acc[nf + 4][mf][q] = __builtin_fmaf(hi, cs[q], t2);                                                  \
      }                                                                                                      \
    }                                                                                                        \
  }
  LLMMM_ROPE_FETCH(0)
  const float* nw = head < op.n_q ? op.qw : op.kw;
  if (nw != nullptr) {
    float r[MF];
#pragma unroll
    for (int mf = 0; mf < MF; ++mf) {
      float p[8];
#pragma unroll
      for (int nf = 0; nf < 8; ++nf) {
        float a = 0.f;
#pragma unroll
        for (int q = 0; q < 4; ++q) a = __builtin_fmaf(acc[nf][mf][q], acc[nf][mf][q], a);
        p[nf] = a;
      }
      float t = ((p[0] + p[4]) + (p[2] + p[6])) + ((p[1] + p[5]) + (p[3] + p[7]));
      t       = t + wave_xor_get(t, 32);
      t       = t + wave_xor_get(t, 16);
      r[mf]   = 1.0f / __builtin_sqrtf(t / 128.0f + op.eps);
    }
#pragma unroll
    for (int nf = 0; nf < 8; ++nf) {
      const f32x4 w = *(const f32x4*)(nw + nf * 16 + 4 * g);
#pragma unroll
      for (int mf = 0; mf < MF; ++mf)
#pragma unroll
        for (int q = 0; q < 4; ++q) acc[nf][mf][q] = (acc[nf][mf][q] * r[mf]) * w[q];
    }
  }
  wait_vmcnt<0>();
  LLMMM_ROPE_ROTATE(0)
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the first pass has been read: its slots may be refilled
  LLMMM_ROPE_FETCH(1)
  wait_vmcnt<0>();
  LLMMM_ROPE_ROTATE(1)
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // read before the caller stages its output in the same memory
#undef LLMMM_ROPE_FETCH
#undef LLMMM_ROPE_ROTATE
}

// LDS bytes of one workgroup of fp8_gemm_body<BM, BN, WM, *, BMODE>: two operand stages, or the deep pipeline's three or four
// stages with 256 bytes of scales per wave each.
template <int BM, int BN, int WM, int BMODE>
constexpr int fp8_lds_bytes()
{
  typedef Fp8Tile<BM, BN, WM> TC;
  const bool deep    = (BMODE & 4) != 0 && WM == 32;
  const int  stage_d = TC::STAGE + TC::NW * 256;
  return !deep ? 2 * TC::STAGE : (4 * stage_d <= 160 * 1024 ? 4 : 3) * stage_d;
}

// BMODE bit 0 (BPRE): Bt is the pre-shuffled image of the weights (layout.hip) instead of row-major [N, K].
// BMODE bit 1 (BNT): the weight loads carry the non-temporal hint (one tile row: every weight byte is read once).
// BMODE bit 2 (DEEP, 32-row-wave tiles only): the launch has at most one workgroup per CU, which then runs a deeper pipeline.
template <int BM, int BN, int WM, int OUT, int BMODE>
__device__ __forceinline__ void fp8_gemm_body(const uint8_t* __restrict__ A, const float* __restrict__ As, const uint8_t* __restrict__ Bt,
                                              const float* __restrict__ Bs, void* __restrict__ Cv, float* __restrict__ Cs, int M, int N, int K,
                                              int tiles_m, int tiles_n, const Fp8HeadOp& op, char LLMMM_LDS* lds, int tile_index, int n_base)
{
  // tile_index: this workgroup's tile among the tiles_m x tiles_n tiles of the column range that starts at n_base (0 and
  // the whole matrix for the plain kernel; SwiGLU counts n_base in gate columns); lds: the workgroup's operand buffers
  typedef Fp8Tile<BM, BN, WM> TC;
  constexpr int  MF   = TC::MF;
  constexpr int  NF   = TC::NF;
  constexpr bool TWO  = NF != 8;  // 160-column waves straddle two weight-scale blocks
  static_assert(!TWO || (OUT == OUT_F32 || OUT == OUT_BF16 || OUT == OUT_ADD_F32 || OUT == OUT_ADD_BF16 || OUT == OUT_ADD_F16),
                "the 160-column tile has no 1x128-grouped epilogues");
  constexpr bool BPRE = (BMODE & 1) != 0, BNT = (BMODE & 2) != 0;
  // A launch with at most one workgroup per CU (few tiles: decode-sized or mid-sized M) leaves the workgroups
  // waiting on memory latency, not on the matrix pipe, and the LDS a second workgroup would have used lies idle:
  // the 32-row-wave tiles then run a deeper pipeline -- as many stages as fit the LDS instead of two, the slice
  // scales travelling with the stage.  (With two workgroups per CU the two-stage form is faster: 29 vs 38 us on
  // 2048 x 2560 x 4096 in 128 x 128 tiles.)
  constexpr bool DEEP    = (BMODE & 4) != 0 && WM == 32;
  // BMODE bit 3 (MT, deep 128 x 128 tiles with the fp32 / bf16 / fp8 outputs only): M is not a multiple of BM; the rows
  // of the last tile row beyond the matrix are computed from copies of its last row and never stored.
  constexpr bool MT      = (BMODE & 8) != 0;
  // BMODE bit 4 (STAMP): the phase-accounting build -- clock readings at five points of every wave, stored to op.stamps at the end
  constexpr bool STAMP   = (BMODE & 16) != 0;
  PhaseClock     ph[STAMP ? PHASE_POINTS : 1];
  unsigned long long wait_cycles = 0;  // STAMP: shader cycles this wave spent in the K loop's "loads landed + barrier" waits (slices 1 ..)
  unsigned long long load_wait_cycles = 0;  // ... of which for its own loads (the rest: for the other waves at the barrier)
  if constexpr (STAMP) ph[0] = phase_clock();
  static_assert(!MT || (DEEP && BM == 128 && BN == 128 && (OUT == OUT_F32 || OUT == OUT_BF16 || OUT == OUT_FP8Q)), "row tails: deep 128 x 128 tiles only");
  constexpr int  STAGE_D = TC::STAGE + TC::NW * 256;                 // operands + 256 bytes of scales per wave
  constexpr int  NST     = !DEEP ? 2 : (4 * STAGE_D <= 160 * 1024 ? 4 : 3);
  static_assert(fp8_lds_bytes<BM, BN, WM, BMODE>() == (DEEP ? NST * STAGE_D : 2 * TC::STAGE), "the kernels size the buffers with fp8_lds_bytes");

  const int tid  = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm   = wave % TC::WAVES_M;
  const int wn   = wave / TC::WAVES_M;
  int       tm, tn;
  tile_coords(tile_index, tiles_m, tiles_n, tm, tn);
  // SwiGLU output: the tile's two 128-column halves are the gate columns n0 .. n0+127 and the up columns
  // N/2 + n0 .. of the same 128 output columns, so the weight rows of the upper half start N/2 - 128 rows further on
  constexpr bool SWIGLU = OUT == OUT_SWIGLU;
  static_assert(!SWIGLU || BN == 256, "the SwiGLU epilogue pairs the two 128-column halves of a 256-wide tile");
  const int    m0   = tm * BM, n0 = n_base + (SWIGLU ? tn * 128 : tn * BN);
  const size_t b_hi = SWIGLU ? (size_t)((N >> 1) - 128) * K : 0;
  const int    KB   = K >> 7;
  // split-K: gridDim.y workgroups share a tile, each taking a contiguous run of slices and (the
  // host only splits the fp32 instantiation) writing its partial sums to its own [M, N] plane
  // of C; a second kernel adds the planes in order.  gridDim.y == 1: the whole K range.
  const int S   = gridDim.y;
  const int sp  = blockIdx.y;
  const int kb0 = sp * KB / S;
  const int KBL = (sp + 1) * KB / S - kb0;  // slices of this workgroup (>= 1: the host keeps S <= KB)

  const KMajorLane lp       = kmajor_lane<SWZ_ROWS16>(wave, lane);
  const unsigned   lane_off = (unsigned)(lp.row * K + lp.chunk * 16);
  const uint8_t*   Ag       = A + (size_t)m0 * K + (size_t)kb0 * 128;
  // pre-shuffled: row 8*wave of the tile starts half block (wave & 1) of row group n0/16 + wave/2
  constexpr int    B_KSTEP    = BPRE ? 2048 : 128;  // bytes from one slice to the next
  const unsigned   b_lane_off = BPRE ? (unsigned)lane * 16u : lane_off;
  const uint8_t*   Bg         = BPRE ? Bt + (size_t)(n0 + 16 * (wave >> 1)) * K + (wave & 1) * 1024 + (size_t)kb0 * 2048
                                     : Bt + (size_t)n0 * K + (size_t)kb0 * 128;

  // operand reads: lane = (g = lane/16, i = lane%16) takes row i of a 16-row fragment and the
  // 32 bytes k = 32g .. 32g+31 (chunks 2g and 2g+1)
  const int g     = lane >> 4;
  const int a_rd0 = kmajor_offset<SWZ_ROWS16>(wm * WM + (lane & 15), 2 * g), a_rd1 = a_rd0 ^ 16;
  const int b_rd0 = kmajor_offset<SWZ_ROWS16>(wn * TC::WN + (lane & 15), 2 * g), b_rd1 = b_rd0 ^ 16;

  f32x4 acc[NF][MF];
#pragma unroll
  for (int nf = 0; nf < NF; ++nf)
#pragma unroll
    for (int mf = 0; mf < MF; ++mf) acc[nf][mf] = f32x4{0.f, 0.f, 0.f, 0.f};

  // scales: As[kb*M + m] for the lane's 4 rows, Bs[(n/128)*KB + kb] for the wave's column group
  const int      mrow    = m0 + wm * WM + (lane & 15);
  const unsigned row_off = (unsigned)mrow * 4u;
  const float*   Bsp     = Bs + (size_t)((n0 >> 7) + (SWIGLU ? wn * (N >> 8) : wn)) * KB + kb0;
  // 160-column waves: columns n0 .. n0+159 lie in weight-scale blocks n0/128 and n0/128 + 1; the first nfb fragments
  // (16 columns each) belong to the former
  const float*   Bsp2    = Bsp + (TWO ? KB : 0);
  const int      nfb     = TWO ? (128 - (n0 & 127)) >> 4 : NF;
  const float*   Asl     = As + (size_t)kb0 * M;
  unsigned       zero    = 0;
  asm volatile("" : "+v"(zero));  // a VGPR holding 0: the per-lane offset of the wave-uniform Bs load
  float sa_next[MF], sb_next, sb2_next = 0.f;

  const unsigned lds0 = (unsigned)(size_t)(char LLMMM_LDS*)lds;
  char LLMMM_LDS* const s0 = (char LLMMM_LDS*)lds;

  if constexpr (DEEP) {
    constexpr int PER = TC::A_LOADS + TC::B_LOADS + 1;  // vector-memory loads of a wave per slice
    unsigned a_tail[TC::A_LOADS];  // MT: per-load offsets with the row clamped to the matrix
#pragma unroll
    for (int i = 0; i < TC::A_LOADS; ++i) a_tail[i] = MT ? (unsigned)(min(lp.row + 8 * TC::NW * i, M - 1 - m0) * K + lp.chunk * 16) : 0u;
    static_assert((NST - 2) * PER < 64, "vmcnt is a 6-bit counter");
    // this lane's scale source: a row scale (stride M floats per slice) or the column-group scale (stride 1)
    const bool     row_lane = lane < WM;
    const char*    sc_ptr   = row_lane ? (const char*)(Asl + (MT ? min(m0 + wm * WM + lane, M - 1) : m0 + wm * WM + lane)) : (const char*)(TWO && lane >= 48 ? Bsp2 : Bsp);
    const unsigned sc_step  = row_lane ? (unsigned)M * 4u : 4u;
    // prologue: slices 0 .. NST-2 (a K range shorter than that repeats its last slice into the spare stages)
#pragma unroll
    for (int u = 0; u < NST - 1; ++u) {
      const int kk = min(u, KBL - 1);
      fp8_issue_loads<BM, BN, WM, BNT, 0, TC::A_LOADS + TC::B_LOADS, MT>(lds0 + u * STAGE_D, Ag + (size_t)kk * 128, Bg + (size_t)kk * B_KSTEP, lane_off,
                                                                         b_lane_off, K, b_hi, wave, a_tail);
      fp8_scale_load_lds(sc_ptr + (size_t)kk * sc_step, lds0 + u * STAGE_D + TC::STAGE + wave * 256);
    }
    const char* sc_next = sc_ptr + (size_t)(NST - 1) * sc_step;
    unsigned    cur     = 0;  // byte offset of the stage being computed
    const float LLMMM_LDS* const my_scales = (const float LLMMM_LDS*)(s0 + TC::STAGE + wave * 256);
#define LLMMM_FP8_DEEP_SLICE(LOAD, WAIT)                                                                                          \
  {                                                                                                                               \
    wait_vmcnt<(WAIT)>();                                                                                                         \
    __syncthreads();                                                                                                              \
    const float LLMMM_LDS* sc_ = (const float LLMMM_LDS*)((const char LLMMM_LDS*)my_scales + cur);                                \
    float                  s[MF], s2[MF];                                                                                         \
    const float            sb_ = sc_[32], sb2_ = sc_[48];                                                                         \
    _Pragma("unroll") for (int mf = 0; mf < MF; ++mf) {                                                                            \
      const float sa_ = sc_[mf * 16 + (lane & 15)];                                                                               \
      s[mf] = sa_ * sb_, s2[mf] = sa_ * sb2_;                                                                                     \
    }                                                                                                                             \
    Fp8Next nx;                                                                                                                   \
    nx.lds_stage = lds0 + (cur == 0 ? (NST - 1) * STAGE_D : cur - STAGE_D);                                                       \
    nx.Ag        = Ag + (size_t)(kc + NST - 1) * 128;                                                                             \
    nx.Bg        = Bg + (size_t)(kc + NST - 1) * B_KSTEP;                                                                         \
    nx.As_slice  = nullptr;                                                                                                       \
    nx.Bs_elem   = nullptr;                                                                                                       \
    nx.Bs_elem2  = nullptr;                                                                                                       \
    nx.sc_ptr    = sc_next;                                                                                                       \
    fp8_compute_stage<BM, BN, WM, BNT, LOAD, true, MT>(s0 + cur, a_rd0, a_rd1, b_rd0, b_rd1, s, acc, nx, lane_off, b_lane_off, row_off, zero, K, \
                                                       b_hi, wave, sa_next, sb_next, s2, nfb, sb2_next, a_tail);                  \
    cur = cur + STAGE_D == NST * STAGE_D ? 0 : cur + STAGE_D;                                                                     \
  }
    int kc = 0;
    for (; kc + (NST - 1) < KBL; ++kc) {  // slices that still have a slice NST-1 ahead of them to request
      LLMMM_FP8_DEEP_SLICE(true, (NST - 2) * PER)
      sc_next += sc_step;
    }
    // the last (up to) NST-1 slices request nothing more: the waits count down
    if (kc < KBL) { LLMMM_FP8_DEEP_SLICE(false, (NST - 2) * PER) ++kc; }
    if (kc < KBL) { LLMMM_FP8_DEEP_SLICE(false, (NST - 3) * PER) ++kc; }
    if constexpr (NST == 4)
      if (kc < KBL) { LLMMM_FP8_DEEP_SLICE(false, 0) ++kc; }
#undef LLMMM_FP8_DEEP_SLICE
    wait_vmcnt<0>();  // repeats of the last slice that a short K range left in flight
  }
  else {
  fp8_issue_loads<BM, BN, WM, BNT, 0, TC::A_LOADS + TC::B_LOADS>(lds0, Ag, Bg, lane_off, b_lane_off, K, b_hi, wave);
  fp8_issue_scales<MF, TWO>(sa_next, sb_next, Asl, row_off, Bsp, zero, &sb2_next, Bsp2);

  // One slice: wait for this wave's loads of the slice (all of them were issued at least half a
  // slice ago), meet the other waves, then compute it while the loads of the next one go out.
#define LLMMM_FP8_SLICE(LOAD, CUR, NXT_LDS, KC)                                                                                   \
  {                                                                                                                               \
    unsigned long long tw_ = 0;                                                                                                   \
    if constexpr (STAMP) tw_ = __builtin_amdgcn_s_memtime();                                                                      \
    wait_vmcnt<0>();                                                                                                              \
    if constexpr (STAMP)                                                                                                          \
      if ((KC) != 0) load_wait_cycles += __builtin_amdgcn_s_memtime() - tw_;                                                      \
    if constexpr (MF == 4)                                                                                                        \
      asm volatile("" : "+v"(sa_next[0]), "+v"(sa_next[1]), "+v"(sa_next[2]), "+v"(sa_next[MF - 1]), "+v"(sb_next));              \
    else                                                                                                                          \
      asm volatile("" : "+v"(sa_next[0]), "+v"(sa_next[1]), "+v"(sb_next));                                                       \
    if constexpr (TWO) asm volatile("" : "+v"(sb2_next));                                                                         \
    __syncthreads();                                                                                                              \
    if constexpr (STAMP) {                                                                                                        \
      if ((KC) == 0)                                                                                                              \
        ph[1] = phase_clock();                                                                                                    \
      else                                                                                                                        \
        wait_cycles += __builtin_amdgcn_s_memtime() - tw_;                                                                        \
    }                                                                                                                             \
    float s[MF], s2[MF];                                                                                                          \
    _Pragma("unroll") for (int mf = 0; mf < MF; ++mf) s[mf] = sa_next[mf] * sb_next, s2[mf] = sa_next[mf] * sb2_next;              \
    Fp8Next nx;                                                                                                                   \
    nx.lds_stage = NXT_LDS;                                                                                                       \
    nx.Ag        = Ag + (size_t)((KC) + 1) * 128;                                                                                 \
    nx.Bg        = Bg + (size_t)((KC) + 1) * B_KSTEP;                                                                               \
    nx.As_slice  = Asl + (size_t)((KC) + 1) * M;                                                                                  \
    nx.Bs_elem   = Bsp + (KC) + 1;                                                                                                \
    nx.Bs_elem2  = Bsp2 + (KC) + 1;                                                                                               \
    fp8_compute_stage<BM, BN, WM, BNT, LOAD>(CUR, a_rd0, a_rd1, b_rd0, b_rd1, s, acc, nx, lane_off, b_lane_off, row_off, zero, K, b_hi, wave, sa_next, \
                                    sb_next, s2, nfb, sb2_next);                                                                  \
  }

  unsigned cur = 0;  // byte offset of the stage being computed: 0 or STAGE
  for (int kc = 0; kc < KBL - 1; ++kc) {
    LLMMM_FP8_SLICE(true, s0 + cur, lds0 + (TC::STAGE - cur), kc)
    cur = TC::STAGE - cur;
  }
  LLMMM_FP8_SLICE(false, s0 + cur, 0u, KBL - 1)
#undef LLMMM_FP8_SLICE
  }

  // ---- epilogue.  lane (g, i): row m = .. + mf*16 + i, columns n = nf*16 + 4g + r.
  // Written straight from this layout, one store instruction would touch 16 rows with 16..64
  // bytes each; the memory pipeline pays per row segment, not per byte.  So every wave first
  // lays its WM x 128 result out row-major in a private 16 KB piece of the (now idle) operand
  // buffers -- 16-byte chunks XOR-ed with row bits so that neither the writes nor the
  // ds_read_b128 reads conflict -- and stores it back out 16 bytes per lane, whole rows at a time.
  if constexpr (STAMP) ph[2] = phase_clock();
  __syncthreads();  // every wave is done reading the last operand stage
  // WM rows of up to 256 bytes (fp32 goes 16 rows at a time); 160-column waves pad their rows by 16 bytes instead of XOR-ing chunks
  constexpr int         RS32 = TC::WN * 4 + 16, RS16 = TC::WN * 2 + 16;  // padded row strides of the 160-column staging
  char LLMMM_LDS* const stg  = s0 + wave * (TWO ? (16 * RS32 > WM * RS16 ? 16 * RS32 : WM * RS16) : WM * 256);
  const int             row0 = m0 + wm * WM;
  const int             col0 = n0 + wn * TC::WN;
  const int             li   = lane & 15;
  if constexpr (OUT == OUT_ROPE_BF16 || OUT == OUT_ROPE_FP8Q) qk_norm_rope_fragments<MF>(acc, op, col0 >> 7, row0, lane, stg);
  if constexpr (TWO) {
    // 160-column waves: the same staging with padded rows instead of the chunk XOR (a row is 40 or 20 chunks, not a power
    // of two), 16-byte chunks dealt to the lanes in row-major order
    constexpr int CH32 = TC::WN / 4, CH16 = TC::WN / 8;  // 16-byte chunks per row: fp32, 2-byte types
    if constexpr (OUT == OUT_BF16) {
      __bf16* C = (__bf16*)Cv;
      typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
#pragma unroll
      for (int mf = 0; mf < MF; ++mf) {
        const int r = mf * 16 + li;
#pragma unroll
        for (int nf = 0; nf < NF; ++nf) {
          bf16x4 o;
#pragma unroll
          for (int q = 0; q < 4; ++q) o[q] = (__bf16)acc[nf][mf][q];
          *(bf16x4 LLMMM_LDS*)(stg + r * RS16 + nf * 32 + 8 * g) = o;
        }
      }
#pragma unroll
      for (int j = 0; j < (WM * CH16) / 64; ++j) {
        const int   idx = j * 64 + lane, r = idx / CH16, c = idx - r * CH16;
        const i32x4 v   = *(const i32x4 LLMMM_LDS*)(stg + r * RS16 + c * 16);
        *(i32x4*)(C + (size_t)(row0 + r) * N + col0 + c * 8) = v;
      }
    }
    else {
      // fp32 planes / fp32 output, or hidden = T(C + residual)
#pragma unroll
      for (int mf = 0; mf < MF; ++mf) {
#pragma unroll
        for (int nf = 0; nf < NF; ++nf) *(f32x4 LLMMM_LDS*)(stg + li * RS32 + nf * 64 + 16 * g) = acc[nf][mf];
#pragma unroll
        for (int j = 0; j < (16 * CH32) / 64; ++j) {
          const int    idx = j * 64 + lane, r = idx / CH32, c = idx - r * CH32;
          const f32x4  v   = *(const f32x4 LLMMM_LDS*)(stg + r * RS32 + c * 16);
          const size_t at  = (size_t)(row0 + 16 * mf + r) * N + col0 + c * 4;
          if constexpr (OUT == OUT_F32)
            *(f32x4*)((float*)Cv + (size_t)sp * M * N + at) = v;
          else {
            typedef typename std::conditional<OUT == OUT_ADD_F32, float, typename std::conditional<OUT == OUT_ADD_BF16, __bf16, _Float16>::type>::type T;
            store_row4<T>((T*)Cv + at, v + load_row4<T>((const T*)op.residual + at));
          }
        }
      }
    }
  }
  else if constexpr (OUT == OUT_F32) {
    float* C = (float*)Cv + (size_t)sp * M * N;
#pragma unroll
    for (int mf = 0; mf < MF; ++mf) {  // 16 rows x 512 B per round
#pragma unroll
      for (int nf = 0; nf < 8; ++nf) *(f32x4 LLMMM_LDS*)(stg + li * 512 + (((nf * 4 + g) ^ ((li & 7) << 1)) << 4)) = acc[nf][mf];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int   r = 2 * j + (lane >> 5), c = lane & 31;
        const f32x4 v = *(const f32x4 LLMMM_LDS*)(stg + r * 512 + ((c ^ ((r & 7) << 1)) << 4));
        if (!MT || row0 + 16 * mf + r < M) *(f32x4*)(C + (size_t)(row0 + 16 * mf + r) * N + col0 + c * 4) = v;
      }
    }
  }
  else if constexpr (OUT == OUT_ADD_F32 || OUT == OUT_ADD_BF16 || OUT == OUT_ADD_F16) {
    // the fp32 staging of OUT_F32; each lane then adds the residual to its four columns in fp32 and stores T(sum)
    typedef typename std::conditional<OUT == OUT_ADD_F32, float, typename std::conditional<OUT == OUT_ADD_BF16, __bf16, _Float16>::type>::type T;
    const T* res = (const T*)op.residual;
    T*       H   = (T*)Cv;
#pragma unroll
    for (int mf = 0; mf < MF; ++mf) {
#pragma unroll
      for (int nf = 0; nf < 8; ++nf) *(f32x4 LLMMM_LDS*)(stg + li * 512 + (((nf * 4 + g) ^ ((li & 7) << 1)) << 4)) = acc[nf][mf];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int    r   = 2 * j + (lane >> 5), c = lane & 31;
        const f32x4  v   = *(const f32x4 LLMMM_LDS*)(stg + r * 512 + ((c ^ ((r & 7) << 1)) << 4));
        const size_t idx = (size_t)(row0 + 16 * mf + r) * N + col0 + c * 4;
        store_row4<T>(H + idx, v + load_row4<T>(res + idx));
      }
    }
  }
  else if constexpr (OUT == OUT_BF16 || OUT == OUT_ROPE_BF16) {
    __bf16* C = (__bf16*)Cv;
    typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
#pragma unroll
    for (int mf = 0; mf < MF; ++mf) {
      const int r = mf * 16 + li;
#pragma unroll
      for (int nf = 0; nf < 8; ++nf) {
        bf16x4 o;
#pragma unroll
        for (int q = 0; q < 4; ++q) o[q] = (__bf16)acc[nf][mf][q];
        *(bf16x4 LLMMM_LDS*)(stg + r * 256 + (((nf * 2 + (g >> 1)) ^ (r & 15)) << 4) + 8 * (g & 1)) = o;
      }
    }
#pragma unroll
    for (int j = 0; j < WM / 4; ++j) {
      const int   r = 4 * j + (lane >> 4), c = lane & 15;
      const i32x4 v = *(const i32x4 LLMMM_LDS*)(stg + r * 256 + ((c ^ (r & 15)) << 4));
      if (!MT || row0 + r < M) *(i32x4*)(C + (size_t)(row0 + r) * N + col0 + c * 8) = v;
    }
  }
  else if constexpr (OUT == OUT_SWIGLU) {
    // Waves (wm, 0) hold the gate half and waves (wm, 1) the up half of the same WM rows x 128 output columns.
    // Each sends the partner the 16-row fragments it does not keep (the gate wave keeps the first half of them,
    // the up wave the second), so that all eight waves share the activation work and each owns whole rows.
    constexpr int         MH      = MF / 2;
    char LLMMM_LDS* const xmine   = s0 + wave * (MH * 8192);
    const int             partner = wm + (1 - wn) * TC::WAVES_M;
    const char LLMMM_LDS* xtheirs = s0 + partner * (MH * 8192);
    if (wn == 0)
      swiglu_send<MF, MH>(acc, xmine, lane);
    else
      swiglu_send<MF, 0>(acc, xmine, lane);
    __syncthreads();
    f32x4 other[8][MH];
#pragma unroll
    for (int nf = 0; nf < 8; ++nf)
#pragma unroll
      for (int h = 0; h < MH; ++h) other[nf][h] = *(const f32x4 LLMMM_LDS*)(xtheirs + ((h * 8 + nf) * 64 + lane) * 16);
    __syncthreads();  // every wave has read its partner's fragments: the regions are free for the output staging
    uint8_t*  C    = (uint8_t*)Cv;
    const int half = N >> 1;
    if (wn == 0)
      swiglu_finish<MF, 0, true>(acc, other, xmine, C, Cs + (size_t)(n0 >> 7) * M, half, row0, n0, lane);
    else
      swiglu_finish<MF, MH, false>(acc, other, xmine, C, Cs + (size_t)(n0 >> 7) * M, half, row0, n0, lane);
  }
  else {
    uint8_t* C = (uint8_t*)Cv;
#pragma unroll
    for (int mf = 0; mf < MF; ++mf) {
      float amax = 0.f;
#pragma unroll
      for (int nf = 0; nf < 8; ++nf)
#pragma unroll
        for (int q = 0; q < 4; ++q) amax = fmaxf(amax, __builtin_fabsf(acc[nf][mf][q]));
      amax              = wave_xor_max(amax, 16);
      amax              = wave_xor_max(amax, 32);
      const float scale = amax / 448.f;
      const float inv   = requant_inv(amax);
      const int   r     = mf * 16 + li;
#pragma unroll
      for (int nf = 0; nf < 8; ++nf) {
        const f32x4 v = acc[nf][mf];
        *(uint32_t LLMMM_LDS*)(stg + r * 128 + ((nf ^ ((r >> 1) & 7)) << 4) + 4 * g) = pack_e4m3x4_in_range(v[0] * inv, v[1] * inv, v[2] * inv, v[3] * inv);
      }
      if (g == 0 && (!MT || row0 + r < M)) Cs[(size_t)((n0 >> 7) + wn) * M + row0 + r] = scale;
    }
#pragma unroll
    for (int j = 0; j < WM / 8; ++j) {
      const int   r = 8 * j + (lane >> 3), c = lane & 7;
      const i32x4 v = *(const i32x4 LLMMM_LDS*)(stg + r * 128 + ((c ^ ((r >> 1) & 7)) << 4));
      if (!MT || row0 + r < M) *(i32x4*)(C + (size_t)(row0 + r) * N + col0 + c * 16) = v;
    }
  }
  if constexpr (STAMP) {
    ph[3] = phase_clock();
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the stores are acknowledged
    ph[4] = phase_clock();
    if (lane == 0) {
      unsigned long long* o = op.stamps + ((size_t)tile_index * TC::NW + wave) * PHASE_RECORD;
#pragma unroll
      for (int p = 0; p < PHASE_POINTS; ++p) o[2 * p] = ph[p].real, o[2 * p + 1] = ph[p].cycles;
      o[PHASE_STAMPS] = wait_cycles, o[PHASE_STAMPS + 1] = load_wait_cycles;
    }
  }
}

template <int BM, int BN, int WM, int OUT, int BMODE>
__global__ void __launch_bounds__((BM / WM) * (BN / 128) * 64)
fp8_gemm_kernel(const uint8_t* __restrict__ A, const float* __restrict__ As, const uint8_t* __restrict__ Bt,
                const float* __restrict__ Bs, void* __restrict__ Cv, float* __restrict__ Cs, int M, int N, int K, int tiles_m,
                int tiles_n, Fp8HeadOp op)
{
  __shared__ __attribute__((aligned(1024))) char lds[fp8_lds_bytes<BM, BN, WM, BMODE>()];
  fp8_gemm_body<BM, BN, WM, OUT, BMODE>(A, As, Bt, Bs, Cv, Cs, M, N, K, tiles_m, tiles_n, op, (char LLMMM_LDS*)lds, blockIdx.x, 0);
}

// 256 x 256 tiles leave the last round of the chip partly filled when their number is not a multiple of the 256 CUs
// (M = 2048, N = 19456: 608 tiles, the third round 96 of them).  This launch gives the columns that fill whole rounds to
// 256 x 256 tiles and the remaining ones to twice as many 128 x 256 tiles (the same eight waves and K loop, half the
// rows per wave; same results bit for bit): the last round then runs on up to all CUs for half as long.  Workgroups
// 0 .. tiles_m_big * cols_big - 1 are the large tiles (dispatched first), the rest the small ones of the column range
// behind them.
template <int OUT, int BPRE>
__global__ void __launch_bounds__(512)
fp8_gemm_hybrid_kernel(const uint8_t* __restrict__ A, const float* __restrict__ As, const uint8_t* __restrict__ Bt,
                       const float* __restrict__ Bs, void* __restrict__ Cv, float* __restrict__ Cs, int M, int N, int K, int tiles_m_big,
                       int cols_big, int cols_small, Fp8HeadOp op)
{
  static_assert(fp8_lds_bytes<128, 256, 32, BPRE>() <= fp8_lds_bytes<256, 256, 64, BPRE>(), "the small tiles fit the large tiles' buffers");
  __shared__ __attribute__((aligned(1024))) char lds[fp8_lds_bytes<256, 256, 64, BPRE>()];
  const int n_big = tiles_m_big * cols_big;
  if ((int)blockIdx.x < n_big)
    fp8_gemm_body<256, 256, 64, OUT, BPRE>(A, As, Bt, Bs, Cv, Cs, M, N, K, tiles_m_big, cols_big, op, (char LLMMM_LDS*)lds, blockIdx.x, 0);
  else
    fp8_gemm_body<128, 256, 32, OUT, BPRE>(A, As, Bt, Bs, Cv, Cs, M, N, K, 2 * tiles_m_big, cols_small, op, (char LLMMM_LDS*)lds,
                                           (int)blockIdx.x - n_big, cols_big * (OUT == OUT_SWIGLU ? 128 : 256));
}

// Sum of S planes at one position, added in plane order 0 .. S-1.  W planes are in flight at a time; positions
// beyond S repeat the last plane and are not added.
template <int W>
__device__ __forceinline__ void reduce_planes_chunk(f32x4& v, const float* src, int s0, int S, size_t plane)
{
  f32x4 t[W];
#pragma unroll
  for (int u = 0; u < W; ++u) t[u] = __builtin_nontemporal_load((const f32x4*)(src + (size_t)min(s0 + u, S - 1) * plane));
#pragma unroll
  for (int u = 0; u < W; ++u)
    if (s0 + u < S) v += t[u];
}
// One memory round trip for up to 16 planes (the split counts in use are 2 .. 10).
__device__ __forceinline__ f32x4 reduce_planes(const float* src, int S, size_t plane)
{
  f32x4 v = {0.f, 0.f, 0.f, 0.f};
  if (S <= 4)
    reduce_planes_chunk<4>(v, src, 0, S, plane);
  else if (S <= 8)
    reduce_planes_chunk<8>(v, src, 0, S, plane);
  else
    for (int s0 = 0; s0 < S; s0 += 16) reduce_planes_chunk<16>(v, src, s0, S, plane);
  return v;
}

// Second kernel of a split-K run: C = epilogue(sum over s = 0..S-1, in that order, of plane s).
// Half a wavefront (32 lanes x 4 columns) owns one row of one 128-column group, which is also
// one quantisation group of the fused output; a workgroup of 256 threads covers 8 rows per step.
// The arithmetic of each epilogue is that of fp8_gemm_kernel, so a split run only differs from an
// unsplit one by the (fixed) order of the fp32 additions.
template <int OUT>
__global__ void __launch_bounds__(256)
fp8_splitk_reduce_kernel(const float* __restrict__ planes, int S, void* __restrict__ Cv, float* __restrict__ Cs, int M, int N,
                         int rows_per_wg)
{
  const int    tid   = threadIdx.x;
  const int    sub   = tid >> 5;
  const int    l32   = tid & 31;
  const int    nb    = blockIdx.x;
  const int    n     = nb * 128 + l32 * 4;
  const int    mbeg  = blockIdx.y * rows_per_wg;
  const int    mend  = min(M, mbeg + rows_per_wg);
  const size_t plane = (size_t)M * N;
  for (int m = mbeg + sub; m < mend; m += 8) {
    const float* src = planes + (size_t)m * N + n;
    f32x4        v   = reduce_planes(src, S, plane);
    if constexpr (OUT == OUT_SWIGLU) {
      // v = the gate columns; the up columns of the same outputs lie N/2 further on.  h = silu(gate) * up.
      const f32x4 up = reduce_planes(src + (N >> 1), S, plane);
#pragma unroll
      for (int q = 0; q < 4; ++q) v[q] = silu_mul(v[q], up[q]);
    }
    if constexpr (OUT == OUT_F32) {
      *(f32x4*)((float*)Cv + (size_t)m * N + n) = v;
    }
    else if constexpr (OUT == OUT_BF16) {
      typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
      bf16x4         o;
#pragma unroll
      for (int q = 0; q < 4; ++q) o[q] = (__bf16)v[q];
      *(bf16x4*)((__bf16*)Cv + (size_t)m * N + n) = o;
    }
    else {  // e4m3 codes + 1x128 scales, of C or (SwiGLU) of h, whose rows are N/2 wide
      const int ldc = OUT == OUT_SWIGLU ? (N >> 1) : N;
      float a = fmaxf(fmaxf(fmaxf(0.f, __builtin_fabsf(v[0])), __builtin_fabsf(v[1])), fmaxf(__builtin_fabsf(v[2]), __builtin_fabsf(v[3])));
      a       = wave_xor_max(a, 1);
      a       = wave_xor_max(a, 2);
      a       = wave_xor_max(a, 4);
      a       = wave_xor_max(a, 8);
      a       = wave_xor_max(a, 16);
      const float scale = a / 448.f;
      const float inv   = requant_inv(a);
      *(uint32_t*)((uint8_t*)Cv + (size_t)m * ldc + n) = pack_e4m3x4_in_range(v[0] * inv, v[1] * inv, v[2] * inv, v[3] * inv);
      if (l32 == 0) Cs[(size_t)nb * M + m] = scale;
    }
  }
}

// The second kernel behind a QKV projection: ordered plane sum, then per-head RMSNorm and rotary embedding of the
// query and key heads (heads of 128 columns: n_q query, n_kv key, n_kv value heads), then the bf16 or e4m3 + 1x128
// epilogue of the reduce kernel -- a head is exactly one quantisation group.  Half a wavefront owns one row of one
// head, lane l the columns 4l .. 4l+3:
//   norm  (weight pointer of the head's kind not null): acc = fma(x, x, acc) over the lane's four columns, xor
//         butterfly 16, 8, 4, 2, 1, r = 1 / sqrt(total / 128 + eps), x = (x * r) * w
//   rope  rotate-half: column i pairs with column i + 64, which lane l ^ 16 holds at the same register index;
//         lo' = fma(lo, cos, -(hi * sin)), hi' = fma(hi, cos, lo * sin), angle row clamp(pos[m], 0, table_rows - 1)
template <int OUT>
__global__ void __launch_bounds__(256)
fp8_planes_qk_norm_rope_kernel(const float* __restrict__ planes, int S, void* __restrict__ Cv, float* __restrict__ Cs,
                               const float* __restrict__ qw, const float* __restrict__ kw, float eps, const float* __restrict__ cos_t,
                               const float* __restrict__ sin_t, int table_rows, const int* __restrict__ pos, int n_q, int n_kv, int M, int N,
                               int rows_per_wg)
{
  static_assert(OUT == OUT_BF16 || OUT == OUT_FP8Q, "bf16 or e4m3 output");
  const int    tid    = threadIdx.x;
  const int    sub    = tid >> 5;
  const int    l32    = tid & 31;
  const int    head   = blockIdx.x;
  const int    n      = head * 128 + l32 * 4;
  const int    mbeg   = blockIdx.y * rows_per_wg;
  const int    mend   = min(M, mbeg + rows_per_wg);
  const size_t plane  = (size_t)M * N;
  const bool   rotate = head < n_q + n_kv;
  const float* nw     = head < n_q ? qw : (rotate ? kw : nullptr);
  f32x4        w4     = {1.f, 1.f, 1.f, 1.f};
  if (nw != nullptr) w4 = *(const f32x4*)(nw + l32 * 4);
  const int  ti = (l32 & 15) * 4;  // first of the lane's four angle indices
  const bool lo = l32 < 16;
  for (int m = mbeg + sub; m < mend; m += 8) {
    f32x4 cs = {1.f, 1.f, 1.f, 1.f}, sn = {0.f, 0.f, 0.f, 0.f};
    if (rotate) {
      const int p = min(max(pos[m], 0), table_rows - 1);
      cs          = *(const f32x4*)(cos_t + (size_t)p * 64 + ti);
      sn          = *(const f32x4*)(sin_t + (size_t)p * 64 + ti);
    }
    f32x4 v = reduce_planes(planes + (size_t)m * N + n, S, plane);
    if (nw != nullptr) {
      float acc = 0.f;
#pragma unroll
      for (int q = 0; q < 4; ++q) acc = __builtin_fmaf(v[q], v[q], acc);
#pragma unroll
      for (int step = 16; step >= 1; step >>= 1) acc = acc + wave_xor_get(acc, step);
      const float r = 1.0f / __builtin_sqrtf(acc / 128.0f + eps);
#pragma unroll
      for (int q = 0; q < 4; ++q) v[q] = (v[q] * r) * w4[q];
    }
    if (rotate) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float other = wave_xor_get(v[q], 16);
        const float t     = other * sn[q];
        v[q]              = __builtin_fmaf(v[q], cs[q], lo ? -t : t);
      }
    }
    if constexpr (OUT == OUT_BF16) {
      typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
      bf16x4         o;
#pragma unroll
      for (int q = 0; q < 4; ++q) o[q] = (__bf16)v[q];
      *(bf16x4*)((__bf16*)Cv + (size_t)m * N + n) = o;
    }
    else {
      float a = fmaxf(fmaxf(fmaxf(0.f, __builtin_fabsf(v[0])), __builtin_fabsf(v[1])), fmaxf(__builtin_fabsf(v[2]), __builtin_fabsf(v[3])));
#pragma unroll
      for (int step = 1; step <= 16; step <<= 1) a = wave_xor_max(a, step);
      const float scale = a / 448.f;
      const float inv   = requant_inv(a);
      *(uint32_t*)((uint8_t*)Cv + (size_t)m * N + n) = pack_e4m3x4_in_range(v[0] * inv, v[1] * inv, v[2] * inv, v[3] * inv);
      if (l32 == 0) Cs[(size_t)head * M + m] = scale;
    }
  }
}

// --------------------------------------------------------------------------------------------- host
template <int OUT>
static hipError_t launch_reduce(const float* planes, int S, void* C, float* Cs, int M, int N, hipStream_t stream)
{
  const int groups      = OUT == OUT_SWIGLU ? N / 256 : N / 128;  // 128-column groups of the output
  int       rows_per_wg = 8;
  while (rows_per_wg < 64 && (long)groups * ((M + 2 * rows_per_wg - 1) / (2 * rows_per_wg)) >= 2048) rows_per_wg *= 2;
  hipLaunchKernelGGL((fp8_splitk_reduce_kernel<OUT>), dim3(groups, (M + rows_per_wg - 1) / rows_per_wg), dim3(256), 0, stream, planes,
                     S, C, Cs, M, N, rows_per_wg);
  return hipGetLastError();
}

template <int BM, int BN, int WM, int OUT>
static auto pick_kernel(int bmode) -> decltype(&fp8_gemm_kernel<BM, BN, WM, OUT, 0>)
{
  if (bmode & 8) {  // a row tail: deep 128 x 128 tiles with the fp32 / bf16 / fp8 outputs
    if constexpr (BM == 128 && BN == 128 && WM == 32 && (OUT == OUT_F32 || OUT == OUT_BF16 || OUT == OUT_FP8Q))
      return (bmode & 1) ? fp8_gemm_kernel<BM, BN, WM, OUT, 15> : fp8_gemm_kernel<BM, BN, WM, OUT, 14>;
    else
      return nullptr;
  }
  if constexpr (WM != 32) bmode &= 3;  // only the 32-row-wave tiles have a deep form
  switch (bmode) {
    case 1: return fp8_gemm_kernel<BM, BN, WM, OUT, 1>;
    case 2: return fp8_gemm_kernel<BM, BN, WM, OUT, 2>;
    case 3: return fp8_gemm_kernel<BM, BN, WM, OUT, 3>;
    case 4: return fp8_gemm_kernel<BM, BN, WM, OUT, WM == 32 ? 4 : 0>;
    case 5: return fp8_gemm_kernel<BM, BN, WM, OUT, WM == 32 ? 5 : 1>;
    case 6: return fp8_gemm_kernel<BM, BN, WM, OUT, WM == 32 ? 6 : 2>;
    case 7: return fp8_gemm_kernel<BM, BN, WM, OUT, WM == 32 ? 7 : 3>;
    default: return fp8_gemm_kernel<BM, BN, WM, OUT, 0>;
  }
}

template <int BM, int BN, int WM, int OUT>
static hipError_t launch_fp8(const void* A, const float* As, const void* Bt, const float* Bs, void* C, float* Cs, int M, int N,
                             int K, int S, float* planes, bool bpre, const Fp8HeadOp& op, hipStream_t stream)
{
  typedef Fp8Tile<BM, BN, WM> TC;
  const int tiles_m = (M + BM - 1) / BM, tiles_n = N / BN;
  if (M % BM != 0 && tiles_m != 1) return hipErrorInvalidValue;  // a row tail: M < BM only (one tile row, the deep form)
  // one tile row: the weights are read once (streamed, deep); at most one workgroup per CU: deep
  const int  cus        = num_cus();
  const bool one_per_cu = (long)tiles_m * tiles_n * (S < 1 ? 1 : S) <= cus;
  const int  bmode      = (bpre ? 1 : 0) | (tiles_m == 1 ? 2 | 4 : 0) | (one_per_cu ? 4 : 0) | (M % BM != 0 ? 8 : 0);
  if (S <= 1 && planes == nullptr) {
    if constexpr (OUT == OUT_SWIGLU && BN != 256) {
      return hipErrorInvalidValue;  // unsplit SwiGLU needs a 256-wide tile (the host picks one)
    }
    else {
      if constexpr (BM == 256 && BN == 256) {
        // more than one round of the chip with a partly filled last one: whole rounds in 256 x 256 tiles, the remaining
        // columns in 128 x 256 tiles, if those fit one round (fp8_gemm_hybrid_kernel)
        const long tiles = (long)tiles_m * tiles_n;
        const long full  = tiles / cus * cus;
        if (tiles > cus && tiles_m > 1 && full % tiles_m == 0) {
          const int cols_big = (int)(full / tiles_m), cols_small = tiles_n - cols_big;
          if (cols_small > 0 && (long)cols_small * tiles_m * 2 <= cus) {
            const dim3 grid(tiles_m * cols_big + 2 * tiles_m * cols_small);
            if (bpre)
              hipLaunchKernelGGL((fp8_gemm_hybrid_kernel<OUT, 1>), grid, dim3(512), 0, stream, (const uint8_t*)A, As, (const uint8_t*)Bt, Bs, C, Cs, M,
                                 N, K, tiles_m, cols_big, cols_small, op);
            else
              hipLaunchKernelGGL((fp8_gemm_hybrid_kernel<OUT, 0>), grid, dim3(512), 0, stream, (const uint8_t*)A, As, (const uint8_t*)Bt, Bs, C, Cs, M,
                                 N, K, tiles_m, cols_big, cols_small, op);
            return hipGetLastError();
          }
        }
      }
      const auto kernel = pick_kernel<BM, BN, WM, OUT>(bmode);
      if (kernel == nullptr) return hipErrorInvalidValue;
      hipLaunchKernelGGL(kernel, dim3(tiles_m * tiles_n), dim3(TC::NT), 0, stream, (const uint8_t*)A, As, (const uint8_t*)Bt, Bs, C, Cs,
                         M, N, K, tiles_m, tiles_n, op);
      return hipGetLastError();
    }
  }
  // split-K (or planes != nullptr with S = 1: an epilogue that only the second kernel has): S partial planes from
  // the fp32 instantiation, then the ordered sum + epilogue
  if constexpr (OUT >= OUT_ROPE_BF16) {
    return hipErrorInvalidValue;  // these epilogues have second kernels of their own behind planes
  }
  else {
    if (S < 1) S = 1;
    const auto kernel = pick_kernel<BM, BN, WM, OUT_F32>(bmode);
    if (kernel == nullptr) return hipErrorInvalidValue;
    hipLaunchKernelGGL(kernel, dim3(tiles_m * tiles_n, S), dim3(TC::NT), 0, stream, (const uint8_t*)A, As, (const uint8_t*)Bt, Bs,
                       (void*)planes, (float*)nullptr, M, N, K, tiles_m, tiles_n, op);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || C == nullptr) return e;  // C == nullptr: the caller consumes the planes itself
    return launch_reduce<OUT>(planes, S, C, Cs, M, N, stream);
  }
}

template <int OUT>
static hipError_t dispatch_fp8(int tile, const void* A, const float* As, const void* Bt, const float* Bs, void* C, float* Cs,
                               int M, int N, int K, int S, float* planes, bool bpre, const Fp8HeadOp& op, hipStream_t stream)
{
  // the 256 x 256 tile uses eight 64-row waves; the smaller tiles 32-row waves (twice the waves per SIMD)
  switch (tile) {
    case LLMMM_TILE_256x256: return launch_fp8<256, 256, 64, OUT>(A, As, Bt, Bs, C, Cs, M, N, K, S, planes, bpre, op, stream);
    case LLMMM_TILE_128x256: return launch_fp8<128, 256, 32, OUT>(A, As, Bt, Bs, C, Cs, M, N, K, S, planes, bpre, op, stream);
    case LLMMM_TILE_256x128: return launch_fp8<256, 128, 32, OUT>(A, As, Bt, Bs, C, Cs, M, N, K, S, planes, bpre, op, stream);
    case LLMMM_TILE_128x128: return launch_fp8<128, 128, 32, OUT>(A, As, Bt, Bs, C, Cs, M, N, K, S, planes, bpre, op, stream);
    case LLMMM_TILE_128x160:
      // no 1x128-grouped epilogue: fp32 (also the planes of a split run), bf16 and residual-add outputs only
      if constexpr (OUT == OUT_F32 || OUT == OUT_BF16 || OUT == OUT_ADD_F32 || OUT == OUT_ADD_BF16 || OUT == OUT_ADD_F16)
        return launch_fp8<128, 160, 32, OUT>(A, As, Bt, Bs, C, Cs, M, N, K, S, planes, bpre, op, stream);
      else
        return hipErrorInvalidValue;
    default: return hipErrorInvalidValue;
  }
}

hipError_t fp8_gemm_launch(int out_kind, int tile, int b_layout, const void* A, const float* As, const void* Bt, const float* Bs,
                           void* C, float* Cs, int M, int N, int K, int S, float* planes, hipStream_t stream)
{
  const bool bpre = b_layout == LLMMM_FP8_B_PRESHUFFLED;
  switch (out_kind) {
    case OUT_F32: return dispatch_fp8<OUT_F32>(tile, A, As, Bt, Bs, C, Cs, M, N, K, S, planes, bpre, Fp8HeadOp{}, stream);
    case OUT_BF16: return dispatch_fp8<OUT_BF16>(tile, A, As, Bt, Bs, C, Cs, M, N, K, S, planes, bpre, Fp8HeadOp{}, stream);
    case OUT_FP8Q: return dispatch_fp8<OUT_FP8Q>(tile, A, As, Bt, Bs, C, Cs, M, N, K, S, planes, bpre, Fp8HeadOp{}, stream);
    case OUT_SWIGLU: return dispatch_fp8<OUT_SWIGLU>(tile, A, As, Bt, Bs, C, Cs, M, N, K, S, planes, bpre, Fp8HeadOp{}, stream);
    default: return hipErrorInvalidValue;
  }
}

hipError_t fp8_gemm_phases_launch(const void* A, const float* As, const void* Bt, const float* Bs, void* C, float* Cs, int M, int N, int K,
                                  unsigned long long* stamps, hipStream_t stream)
{
  if (M % 256 || N % 256 || K % 128 || !stamps) return hipErrorInvalidValue;
  Fp8HeadOp op;
  op.stamps = stamps;
  const int tiles_m = M / 256, tiles_n = N / 256;
  hipLaunchKernelGGL((fp8_gemm_kernel<256, 256, 64, OUT_FP8Q, 16>), dim3(tiles_m * tiles_n), dim3(512), 0, stream, (const uint8_t*)A, As, (const uint8_t*)Bt, Bs, C,
                     Cs, M, N, K, tiles_m, tiles_n, op);
  return hipGetLastError();
}

hipError_t fp8_gemm_qk_rope_launch(int out_kind, int tile, int b_layout, const void* A, const float* As, const void* Bt, const float* Bs, void* C,
                                   float* Cs, int M, int N, int K, const Fp8HeadOp& op, hipStream_t stream)
{
  const bool bpre = b_layout == LLMMM_FP8_B_PRESHUFFLED;
  if (N != (op.n_q + 2 * op.n_kv) * 128) return hipErrorInvalidValue;
  switch (out_kind) {
    case OUT_BF16: return dispatch_fp8<OUT_ROPE_BF16>(tile, A, As, Bt, Bs, C, Cs, M, N, K, 1, nullptr, bpre, op, stream);
    case OUT_FP8Q: return dispatch_fp8<OUT_ROPE_FP8Q>(tile, A, As, Bt, Bs, C, Cs, M, N, K, 1, nullptr, bpre, op, stream);
    default: return hipErrorInvalidValue;
  }
}

hipError_t fp8_gemm_add_residual_launch(int hidden_dtype, int tile, int b_layout, const void* A, const float* As, const void* Bt, const float* Bs,
                                        const void* residual, void* hidden, int M, int N, int K, hipStream_t stream)
{
  const bool bpre = b_layout == LLMMM_FP8_B_PRESHUFFLED;
  Fp8HeadOp  op;
  op.residual = residual;
  switch (hidden_dtype) {
    case LLMMM_DTYPE_F32: return dispatch_fp8<OUT_ADD_F32>(tile, A, As, Bt, Bs, hidden, nullptr, M, N, K, 1, nullptr, bpre, op, stream);
    case LLMMM_DTYPE_BF16: return dispatch_fp8<OUT_ADD_BF16>(tile, A, As, Bt, Bs, hidden, nullptr, M, N, K, 1, nullptr, bpre, op, stream);
    case LLMMM_DTYPE_F16: return dispatch_fp8<OUT_ADD_F16>(tile, A, As, Bt, Bs, hidden, nullptr, M, N, K, 1, nullptr, bpre, op, stream);
    default: return hipErrorInvalidValue;
  }
}

hipError_t fp8_splitk_reduce_launch(int out_kind, const float* planes, int S, void* C, float* Cs, int M, int N, hipStream_t stream)
{
  switch (out_kind) {
    case OUT_F32: return launch_reduce<OUT_F32>(planes, S, C, Cs, M, N, stream);
    case OUT_BF16: return launch_reduce<OUT_BF16>(planes, S, C, Cs, M, N, stream);
    case OUT_FP8Q: return launch_reduce<OUT_FP8Q>(planes, S, C, Cs, M, N, stream);
    case OUT_SWIGLU: return launch_reduce<OUT_SWIGLU>(planes, S, C, Cs, M, N, stream);
    default: return hipErrorInvalidValue;
  }
}

hipError_t fp8_planes_qk_norm_rope_launch(int out_kind, const float* planes, int S, void* C, float* Cs, const float* qw, const float* kw, float eps,
                                          const float* cos_t, const float* sin_t, int table_rows, const int* pos, int n_q, int n_kv, int M,
                                          hipStream_t stream)
{
  const int heads = n_q + 2 * n_kv, N = heads * 128;
  int       rows_per_wg = 8;
  while (rows_per_wg < 64 && (long)heads * ((M + 2 * rows_per_wg - 1) / (2 * rows_per_wg)) >= 2048) rows_per_wg *= 2;
  const dim3 grid(heads, (M + rows_per_wg - 1) / rows_per_wg);
  if (out_kind == OUT_BF16)
    hipLaunchKernelGGL((fp8_planes_qk_norm_rope_kernel<OUT_BF16>), grid, dim3(256), 0, stream, planes, S, C, Cs, qw, kw, eps, cos_t, sin_t,
                       table_rows, pos, n_q, n_kv, M, N, rows_per_wg);
  else if (out_kind == OUT_FP8Q)
    hipLaunchKernelGGL((fp8_planes_qk_norm_rope_kernel<OUT_FP8Q>), grid, dim3(256), 0, stream, planes, S, C, Cs, qw, kw, eps, cos_t, sin_t,
                       table_rows, pos, n_q, n_kv, M, N, rows_per_wg);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

}  // namespace llmmm
