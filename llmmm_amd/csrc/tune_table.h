// Offline auto-tune results, compiled in.  Regenerate with `python -m llmmm_amd.tune --write` on an
// MI355X; shapes that are not listed fall back to the heuristics in capi.cpp.
// (The reference only sketches this interface: `tune(N, K)` in src/mm/fp32/impl.h:20-23.)
#pragma once
#include "kernels.h"

namespace llmmm {

struct SkinnyTune {
  int m_max;  // entry applies to M <= m_max (entries are ordered by m_max per shape)
  int N, K;
  int split_k;
};
struct TileTune {
  int M, N, K;
  int tile;
  int split_k;  // 0 = heuristic
};

// FP8 weight-streaming kernel (M <= 128).
static const SkinnyTune kSkinnyTune[] = {
  {1, 2560, 4096, 8},
  {16, 2560, 4096, 8},
  {64, 2560, 4096, 8},
  {128, 2560, 4096, 4},
  {1, 2560, 9728, 10},
  {16, 2560, 9728, 10},
  {64, 2560, 9728, 10},
  {96, 2560, 9728, 4},
  {1, 6144, 2560, 5},
  {16, 6144, 2560, 5},
  {64, 6144, 2560, 5},
  {128, 6144, 2560, 1},
  {1, 19456, 2560, 1},
  {16, 19456, 2560, 1},
  {32, 19456, 2560, 1},
};

// FP8 MFMA tile kernels (M % 128 == 0).
static const TileTune kTileTune[] = {
  {4096, 4096, 4096, 0, 1},
  {2048, 6144, 2560, 0, 1},
  {2048, 2560, 4096, 3, 1},
  {64, 19456, 2560, 3, 1},
  {128, 19456, 2560, 3, 1},
  {2048, 19456, 2560, 0, 1},
  {128, 2560, 9728, 3, 8},
  {2048, 2560, 9728, 3, 1},
  {256, 6144, 2560, 3, 1},
  {512, 6144, 2560, 3, 1},
  {1024, 6144, 2560, 3, 1},
  {256, 2560, 4096, 3, 4},
  {512, 2560, 4096, 3, 3},
  {1024, 2560, 4096, 3, 1},
  {256, 19456, 2560, 3, 1},
  {512, 19456, 2560, 0, 1},
  {1024, 19456, 2560, 0, 1},
  {256, 2560, 9728, 3, 6},
  {512, 2560, 9728, 3, 3},
  {1024, 2560, 9728, 3, 3},
};

// FP16/BF16 MFMA tile kernels.
static const TileTune kFp16TileTune[] = {
  {1024, 1024, 1024, 4, 1},
  {2048, 2048, 2048, 3, 1},
  {4096, 4096, 4096, 0, 1},
  {4096, 6144, 2048, 0, 1},
  {4096, 2048, 12288, 1, 1},
  {2048, 19456, 2560, 0, 1},
  {2048, 2560, 9728, 1, 1},
};

}  // namespace llmmm

