// Offline auto-tune results, compiled in.  Regenerate with `python -m llmmm_amd.tune` on an
// MI355X; shapes that are not listed fall back to the heuristics in capi.cpp.
// (The reference only sketches this interface: `tune(N, K)` in src/mm/fp32/impl.h:20-23.)
#pragma once
#include "kernels.h"

namespace llmmm {

struct SkinnyTune {
  int m_max;  // entry applies to M <= m_max
  int N, K;
  int split_k;
};
struct TileTune {
  int M, N, K;
  int tile;
};

// FP8 weight-streaming kernel (M <= 64): Qwen3-4B projections.
static const SkinnyTune kSkinnyTune[] = {
  {64, 6144, 2560, 10},   // QKV
  {64, 2560, 4096, 16},   // O
  {64, 19456, 2560, 4},   // gate_up
  {64, 2560, 9728, 19},   // down
};

// FP8 MFMA tile kernels (M % 128 == 0).
static const TileTune kTileTune[] = {
  {4096, 4096, 4096, LLMMM_TILE_256x256},
};

// FP16/BF16 MFMA tile kernels.
static const TileTune kFp16TileTune[] = {
  {4096, 4096, 4096, LLMMM_TILE_256x256},
  {1024, 1024, 1024, LLMMM_TILE_128x128},
};

}  // namespace llmmm
