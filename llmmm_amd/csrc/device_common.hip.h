// Device-side building blocks shared by the gfx950 GEMM kernels: vector types, the LDS tile
// layout with its bank-conflict-free swizzle, the direct global->LDS tile loader and small
// wavefront helpers.  gfx950 (CDNA4) only: 64-wide wavefronts, 160 KB LDS, 64 LDS banks.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace llmmm {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));

#define LLMMM_LDS __attribute__((address_space(3)))
#define LLMMM_GLOBAL __attribute__((address_space(1)))

// ---------------------------------------------------------------------------------------------
// K-major operand tiles in LDS (FP8): a tile row holds 128 bytes of the K extent as eight 16-byte chunks;
// row r / chunk c lives at  r * 128 + ((c ^ swz(r)) << 4).
// ds_read_b128 serves a wavefront in four passes of 16 lanes -- {0-3,12-15,20-23,24-27},
// {4-11,16-19,28-31} and the same two sets + 32 (measured on gfx950) -- and a pass is
// conflict-free when its 16 lanes touch 16 different 16-byte slots of the 256-byte bank row.
// SWZ_ROWS16 is matched to the lane -> (row, chunk) pattern of the 16x16x128 fp8 MFMA operands: lanes 16g..16g+15 read
// 16 consecutive rows at chunk 2g (+1).  The chunk is XOR-ed with row bits 1..3 and, for rows 4..11 of every 16, with
// 2, which cancels the chunk difference between the two halves of a pass.
// ---------------------------------------------------------------------------------------------
enum { SWZ_ROWS16 = 1 };

template <int SWZ>
struct KMajor {
  static_assert(SWZ == SWZ_ROWS16, "one placement only");
  static constexpr int ROW    = 128;  // bytes per tile row
  static constexpr int CHUNKS = ROW / 16;
  static constexpr int ROWS_PER_KB = 1024 / ROW;              // tile rows covered by one 1 KB load
};

template <int SWZ>
__device__ __forceinline__ int kmajor_swz(int r)
{
  return ((r >> 1) & 7) ^ ((((r >> 2) ^ (r >> 3)) & 1) << 1);
}
template <int SWZ>
__device__ __forceinline__ int kmajor_offset(int r, int c)
{
  return r * KMajor<SWZ>::ROW + ((c ^ kmajor_swz<SWZ>(r)) << 4);
}

// One wave copies 1024 bytes of a tile with a single LDS-direct load: lane l owns the 16 bytes
// at lds_group + 16*l, and fetches the logical (row, chunk) that the swizzle places there.
struct KMajorLane {
  int row;    // logical tile row this lane fetches
  int chunk;  // logical 16-byte chunk within the row
};
template <int SWZ>
__device__ __forceinline__ KMajorLane kmajor_lane(int group, int lane)
{
  KMajorLane p;
  p.row   = group * KMajor<SWZ>::ROWS_PER_KB + lane / KMajor<SWZ>::CHUNKS;
  p.chunk = (lane % KMajor<SWZ>::CHUNKS) ^ kmajor_swz<SWZ>(p.row);
  return p;
}

// 16 bytes per lane, global -> LDS without passing through registers (lane l's data lands at lds_addr + 16*l), written
// as inline assembly so that it stays invisible to the compiler's wait-count bookkeeping.
// While an LDS-direct load that the compiler knows about is in flight, every wait it inserts on
// its own becomes "all loads done", which defeats a deep software pipeline; kernels that keep
// many slices in flight issue all their vector-memory loads through these helpers and place the
// s_waitcnt themselves.  lds_addr is the wave-uniform LDS byte address (goes to M0).
__device__ __forceinline__ void asm_load_lds_16B(const void* gptr, unsigned lds_addr)
{
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gptr), "s"(lds_addr) : "memory");
}
__device__ __forceinline__ void asm_load_16B(i32x4& dst, const void* gptr)
{
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(dst) : "v"(gptr) : "memory");
}
__device__ __forceinline__ void asm_load_8B(i32x2& dst, const void* gptr)
{
  asm volatile("global_load_dwordx2 %0, %1, off" : "=v"(dst) : "v"(gptr) : "memory");
}
__device__ __forceinline__ void asm_load_f32(float& dst, const void* gptr)
{
  asm volatile("global_load_dword %0, %1, off" : "=v"(dst) : "v"(gptr) : "memory");
}

// s_waitcnt vmcnt(N) lgkmcnt(0): at most N of this wave's vector-memory loads still in flight,
// every LDS access done.  simm16 = vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] << 14.
template <int N>
__device__ __forceinline__ void wait_vmcnt()
{
  static_assert(N >= 0 && N < 64, "vmcnt out of range");
  __builtin_amdgcn_s_waitcnt((N & 15) | 0x70 | ((N >> 4) << 14));
}

// Clock readings for the phase-accounting builds of the tile kernels: the constant 100 MHz counter and the shader's cycle
// counter (scalar reads; the values are stored with ordinary vector stores at the end of the kernel).
struct PhaseClock {
  unsigned long long real, cycles;
};
__device__ __forceinline__ PhaseClock phase_clock()
{
  PhaseClock c;
  c.real   = __builtin_amdgcn_s_memrealtime();
  c.cycles = __builtin_amdgcn_s_memtime();
  return c;
}

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

// The value lane (l ^ mask) holds, for mask = 1, 2, 4, 8, 16 or 32 (a compile-time constant at every call site once
// inlined).  No LDS address computation and, for 1, 2 and 32, no trip through the LDS crossbar at all:
//   1, 2     DPP quad permutes (a VALU move),
//   4 .. 16  ds_swizzle in bit-mask mode (xor inside each group of 32 lanes),
//   32       v_permlane32_swap exchanges the upper 32 lanes of its first register with the lower 32 lanes of its second:
//            from (v, v) it returns r[0] = the lower half of v in both halves, r[1] = the upper half in both halves.
__device__ __forceinline__ float wave_xor_get(float v, int mask)
{
  const int iv = __builtin_bit_cast(int, v);
  switch (mask) {
    case 1: return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(iv, 0xB1, 0xf, 0xf, true));  // quad_perm [1,0,3,2]
    case 2: return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(iv, 0x4E, 0xf, 0xf, true));  // quad_perm [2,3,0,1]
    case 4: return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(iv, (4 << 10) | 0x1f));
    case 8: return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(iv, (8 << 10) | 0x1f));
    case 16: return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(iv, (16 << 10) | 0x1f));
    case 32: {
      const auto r = __builtin_amdgcn_permlane32_swap((unsigned)iv, (unsigned)iv, false, false);
      // lanes 0..31 want the upper half (r[1]), lanes 32..63 the lower half (r[0])
      return __builtin_bit_cast(float, (__lane_id() < 32) ? r[1] : r[0]);
    }
    default: return __shfl_xor(v, mask, 64);
  }
}

__device__ __forceinline__ float wave_xor_max(float v, int mask)
{
  return fmaxf(v, wave_xor_get(v, mask));
}

// ---------------------------------------------------------------------------------------------
// fp32 -> OCP e4m3, four codes per dword, as the reference's __nv_fp8_e4m3(float) gives them (round to nearest even,
// saturate to +-448, every NaN -> 0x7F; examples/005.fp8.mm.cu:482-485, examples/005.fp8.mm.opt.cu:445-454).
// v_cvt_pk_fp8_f32 rounds to nearest even and converts everything below 464 to 448, but writes 0xFF for a NaN of
// either sign and sign | 0x7F for larger magnitudes and infinities (measured).
// ---------------------------------------------------------------------------------------------
// Bytes whose low seven bits are all ones (the two NaN codes) lose their sign bit; other bytes are unchanged.
__device__ __forceinline__ uint32_t e4m3x4_nan_codes_to_7f(uint32_t c)
{
  const uint32_t m = ((c & 0x7F7F7F7Fu) + 0x01010101u) & 0x80808080u;
  return c & ~m;
}
// For values that are NaN or lie within +-448 (1 + 2^-20): quotients by a block's own scale, products with
// 448 / amax.  No clamp is needed then, and the only 0x7F / 0xFF bytes the hardware writes stand for NaN.
__device__ __forceinline__ uint32_t pack_e4m3x4_in_range(float a, float b, float c, float d)
{
  int v = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
  v     = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, v, true);
  return e4m3x4_nan_codes_to_7f((uint32_t)v);
}
// For any value: clamped to +-448 first (v_med3_f32 turns a NaN into a bound, so NaN is put back by hand).
__device__ __forceinline__ uint32_t pack_e4m3x4_sat(float a, float b, float c, float d)
{
  const uint32_t nan = (a != a ? 0x000000FFu : 0u) | (b != b ? 0x0000FF00u : 0u) | (c != c ? 0x00FF0000u : 0u) | (d != d ? 0xFF000000u : 0u);
  a     = __builtin_amdgcn_fmed3f(a, -448.f, 448.f);
  b     = __builtin_amdgcn_fmed3f(b, -448.f, 448.f);
  c     = __builtin_amdgcn_fmed3f(c, -448.f, 448.f);
  d     = __builtin_amdgcn_fmed3f(d, -448.f, 448.f);
  int v = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
  v     = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, v, true);
  return ((uint32_t)v & ~nan) | (0x7F7F7F7Fu & nan);
}

// 448 / amax of the fused re-quantisation (examples/005.fp8.mm.opt.cu:439-446), or 0 where that quotient is not finite: a
// group of zeros (the reference multiplies by 448 / 0 and writes NaN codes) and a group so small -- amax below 2^-119 --
// that the reciprocal overflows (the reference then writes +-448 for every non-zero element and NaN for the zeros).
// Such a group gets codes 0 (a NaN element stays NaN, 0x7F) next to its scale amax / 448; with a finite reciprocal every
// product lies within +-448 (1 + 2^-20), which is what pack_e4m3x4_in_range asks for.
__device__ __forceinline__ float requant_inv(float amax)
{
  const float inv = 448.f / amax;
  return inv < __builtin_inff() ? inv : 0.f;
}

// Four consecutive row elements of type float / bf16 / fp16 <-> fp32 (one 16- or 8-byte access).
template <typename IN_T>
__device__ __forceinline__ f32x4 load_row4(const IN_T* p);
template <>
__device__ __forceinline__ f32x4 load_row4<float>(const float* p)
{
  return *(const f32x4*)p;
}
template <>
__device__ __forceinline__ f32x4 load_row4<__bf16>(const __bf16* p)
{
  typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
  const bf16x4   v = *(const bf16x4*)p;
  return f32x4{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
}
template <>
__device__ __forceinline__ f32x4 load_row4<_Float16>(const _Float16* p)
{
  const f16x4 v = *(const f16x4*)p;
  return f32x4{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
}

template <typename T>
__device__ __forceinline__ void store_row4(T* p, f32x4 v);
template <>
__device__ __forceinline__ void store_row4<float>(float* p, f32x4 v)
{
  *(f32x4*)p = v;
}
template <>
__device__ __forceinline__ void store_row4<__bf16>(__bf16* p, f32x4 v)
{
  typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
  *(bf16x4*)p = bf16x4{(__bf16)v[0], (__bf16)v[1], (__bf16)v[2], (__bf16)v[3]};
}
template <>
__device__ __forceinline__ void store_row4<_Float16>(_Float16* p, f32x4 v)
{
  *(f16x4*)p = f16x4{(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
}

// silu(g) * u with the hardware's exp2 and reciprocal (each within about one ulp of fp32): far below the
// resolution of the e4m3 codes the result is quantised to.  g -> -inf gives -0, g -> +inf gives g * u.
__device__ __forceinline__ float silu_mul(float g, float u)
{
  const float e = __builtin_amdgcn_exp2f(g * -1.44269504088896340736f);  // exp(-g)
  return g * __builtin_amdgcn_rcpf(1.f + e) * u;
}

}  // namespace llmmm
