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
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));

#define LLMMM_LDS __attribute__((address_space(3)))
#define LLMMM_GLOBAL __attribute__((address_space(1)))

// ---------------------------------------------------------------------------------------------
// K-major operand tiles.  A tile is R rows, each row holding 128 bytes of the K extent (64 fp16
// or 128 fp8 values) as eight 16-byte chunks.  Row r / chunk c lives at
//     phys_row(r) * 128 + ((c ^ swz(r)) << 4).
// ds_read_b128 serves a wavefront in four passes of 16 lanes -- {0-3,12-15,20-23,24-27},
// {4-11,16-19,28-31} and the same two sets + 32 (measured on gfx950) -- and a pass is
// conflict-free when its 16 lanes touch 16 different 16-byte slots of the 256-byte bank row.
// Two placements are used, each matched to the lane -> (row, chunk) pattern of one MFMA shape:
//   SWZ_ROWS32: lanes 0-31 read 32 consecutive rows at one chunk, lanes 32-63 another chunk
//               (32x32x16 f16/bf16 operands).  Rows of a pair are swapped when bit 3 is set
//               and the chunk is XOR-ed with row bits 1..3 and 4..6.
//   SWZ_ROWS16: lanes 16g..16g+15 read 16 consecutive rows at chunk 2g (+1)
//               (16x16x128 fp8 operands).  The chunk is XOR-ed with row bits 1..3 and, for
//               rows 4..11 of every 16, with 2, which cancels the chunk difference between
//               the two halves of a pass.
// ---------------------------------------------------------------------------------------------
enum { SWZ_ROWS32 = 0, SWZ_ROWS16 = 1 };

template <int SWZ>
__device__ __forceinline__ int kmajor_phys_row(int r)
{
  return SWZ == SWZ_ROWS32 ? (r ^ ((r >> 3) & 1)) : r;
}
template <int SWZ>
__device__ __forceinline__ int kmajor_swz(int r)
{
  return SWZ == SWZ_ROWS32 ? (((r >> 1) ^ (r >> 4)) & 7) : (((r >> 1) & 7) ^ ((((r >> 2) ^ (r >> 3)) & 1) << 1));
}
template <int SWZ>
__device__ __forceinline__ int kmajor_offset(int r, int c)
{
  return kmajor_phys_row<SWZ>(r) * 128 + ((c ^ kmajor_swz<SWZ>(r)) << 4);
}

// One wave copies eight tile rows (1024 bytes of LDS) with a single LDS-direct load: lane l
// owns the 16 bytes at lds_group + 16*l, and fetches the logical (row, chunk) that the swizzle
// places there.
struct KMajorLane {
  int row;    // logical tile row this lane fetches
  int chunk;  // logical 16-byte chunk within the 128-byte row
};
template <int SWZ>
__device__ __forceinline__ KMajorLane kmajor_lane(int group, int lane)
{
  const int  prow = group * 8 + (lane >> 3);
  const int  row  = kmajor_phys_row<SWZ>(prow);  // both placements are involutions on the row index
  KMajorLane p;
  p.row   = row;
  p.chunk = (lane & 7) ^ kmajor_swz<SWZ>(row);
  return p;
}

// 16 bytes per lane, global -> LDS without passing through registers.  lds_base must be
// wave-uniform; lane l's data lands at lds_base + 16*l.
__device__ __forceinline__ void load_lds_16B(const void* gptr, void LLMMM_LDS* lds_base)
{
  __builtin_amdgcn_global_load_lds((const void LLMMM_GLOBAL*)gptr, lds_base, 16, 0, 0);
}

__device__ __forceinline__ float wave_xor_max(float v, int mask)
{
  return fmaxf(v, __shfl_xor(v, mask, 64));
}

}  // namespace llmmm
