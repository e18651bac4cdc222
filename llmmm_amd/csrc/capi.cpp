// C-ABI layer: argument validation, kernel selection (tune table, then heuristic) and launch.
// Mirrors the reference's host launchers: no allocation, no synchronisation, work enqueued on
// the caller's stream (src/mm/fp16/mm.cu:6-42, examples/005.fp8.mm.cu:2466-2500).
#include "../../include/llmmm.h"
#include "../../include/llmmm_probe.h"
#include "kernels.h"
#include "tune_table.h"

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>
#include <vector>

namespace {

thread_local char g_last_error[256] = "";

int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
int fail(int code, const char* fmt, ...)
{
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

}  // namespace

int llmmm::num_cus()
{
  static const int n = [] {
    int            dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0) return prop.multiProcessorCount;
    (void)hipGetLastError();  // no device: not an error of the call that asked
    return 256;
  }();
  return n;
}

// The same for the other files of the library (declared in kernels.h).
int llmmm::report_error(int code, const char* fmt, ...)
{
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

namespace {

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

constexpr int    MAX_SPLIT_K     = 32;
// Compute units of the current device (llmmm::num_cus: read from the runtime once; 256, the MI355X, where no device
// can be asked -- the size queries also work without one).
#define NUM_CUS (llmmm::num_cus())

constexpr int SKINNY_MAX_M = 128;  // rows the weight-streaming kernel takes

int max_split_for(int K) { return (K / 128) < MAX_SPLIT_K ? (K / 128) : MAX_SPLIT_K; }

// Split count for the weight-streaming kernel when the tune table has no entry: about one
// workgroup (one 128-column group x one split) per CU -- what the measured
// Qwen3-4B shapes settle on -- every split at least two 128-K slices long, but short enough
// that the activation rows of a split can be staged in LDS (64 KB: 32 slices of 16 rows).
int heuristic_split(int M, int N, int K)
{
  const int groups = N / 128, kb = K / 128;
  // whole workgroups per CU, never more workgroups than CUs (96 column groups in three splits are 288 workgroups, a
  // second round: 16 x 12288 x 4096 took 18.6 us so, 13.1 us in two splits), and no more than eight splits: beyond that
  // the planes and the reduce kernel cost more than the shorter streams give (3072 x 8192 at M = 16: 9.8 us in ten, 8.5 in eight)
  int s = NUM_CUS / groups;
  if (s > 8) s = 8;
  if (s > kb / 2) s = kb / 2;
  const int mblk = M <= 16 ? 1 : M <= 32 ? 2 : M <= 64 ? 4 : 8;
  const int cap  = 32 / mblk;  // slices whose rows fit the staging area
  if (s < (kb + cap - 1) / cap) s = (kb + cap - 1) / cap;
  if (s > MAX_SPLIT_K) s = MAX_SPLIT_K;
  if (s > kb) s = kb;
  if (s < 1) s = 1;
  return s;
}

// Tile for the MFMA kernels: fewest "waves" of workgroups over the 256 CUs, weighted by tile
// area and a mild efficiency penalty for the smaller tiles (less operand reuse per byte of LDS).
int heuristic_tile(int M, int N)
{
  static const struct {
    int   id, bm, bn, per_cu;
    float eff;
  } cand[] = {{LLMMM_TILE_256x256, 256, 256, 1, 1.00f},
              {LLMMM_TILE_128x256, 128, 256, 1, 0.85f},
              {LLMMM_TILE_256x128, 256, 128, 1, 0.85f},
              {LLMMM_TILE_128x128, 128, 128, 2, 0.90f}};
  int   best      = -1;
  float best_cost = 0.f;
  for (const auto& c : cand) {
    if (M % c.bm || N % c.bn) continue;
    const long  tiles = (long)(M / c.bm) * (N / c.bn);
    const long  slots = (long)NUM_CUS * c.per_cu;
    float       waves = (float)((tiles + slots - 1) / slots);
    if (c.id == LLMMM_TILE_256x256) {
      // a launch of 256 x 256 tiles fills a partly empty last round with half-size tiles where it can (the same
      // conditions as launch_fp8 / launch_fp16 in the kernel files): that round then costs half
      const long tm = M / 256, tn = N / 256, full = tiles / NUM_CUS * NUM_CUS;
      if (tiles > NUM_CUS && tm > 1 && full % tm == 0 && tn - full / tm > 0 && (tn - full / tm) * tm * 2 <= NUM_CUS) waves -= 0.5f;
    }
    // More 128 x 128 tiles than CUs put two on some CUs, and on weights that come from HBM -- as a layer's weights do in a
    // model -- that costs 6-32 % against half as many 256 x 128 tiles, one per CU, whose tile rows re-read the weights half
    // as often (us, weights rotated over more copies than the caches hold / one copy; 128 x 128 | 256 x 128 | 128 x 256:
    // 2048 x 2560 x 9728 85.3 / 64.0 | 64.5 / 62.6 | 66.4 / 62.2; 1024 x 6144 x 2560 27.9 / 21.3 | 22.4 / 21.6 | 23.6 / 21.4;
    // 512 x 10240 x 8192 73.0 / 55.0 | 57.9 / 53.3 | 59.7 / 53.0; 256 x 19456 x 2560 29.1 / 20.5 | 25.8 / 24.0 | 26.0 / 20.9).
    // Up to one tile per CU the small tile stays ahead (1024 x 4096 x 4096: 26.8 | 31.7 | 30.6 cold).
    float eff = c.eff;
    if (c.id == LLMMM_TILE_128x128 && tiles > NUM_CUS) eff = 0.74f;
    if (c.id == LLMMM_TILE_256x128) eff = 0.86f;  // (ahead of 128 x 256 on weights from HBM: 256 x 22016 x 4096 34.0 against 40.0 us)
    const float cost  = waves * c.per_cu * c.bm * c.bn / eff;
    if (best < 0 || cost < best_cost) {
      best      = c.id;
      best_cost = cost;
    }
  }
  return best;
}

// The FP16 / BF16 kernels' tile for shapes the table does not list: the most tiles any CU gets (two 128 x 128 tiles share
// a CU side by side, but it then takes as long as for both) times the tile's area, over a measured efficiency relative
// to the 256 x 256 tile (4096^3: 111.6 us in 256 x 256, 127.6 in 128 x 256, 131.9 in 256 x 128, 146.8 in 128 x 128).  Picks
// the measured best on every shape of the tune driver's list, e.g. 128 x 256 for 2048 x 2560 x 9728 (115 us; 144 in
// 128 x 128, 182 in 256 x 256) and for 4096 x 2048 x 12288 (184 us; 229 in 256 x 256).
int heuristic_tile_fp16(int M, int N)
{
  static const struct {
    int   id, bm, bn;
    float eff;
  } cand[] = {{LLMMM_TILE_256x256, 256, 256, 1.00f}, {LLMMM_TILE_128x256, 128, 256, 0.875f}, {LLMMM_TILE_256x128, 256, 128, 0.85f}, {LLMMM_TILE_128x128, 128, 128, 0.74f}};
  int   best      = -1;
  float best_cost = 0.f;
  for (const auto& c : cand) {
    if (M % c.bm || N % c.bn) continue;
    const long tiles  = (long)(M / c.bm) * (N / c.bn);
    float      rounds = (float)((tiles + NUM_CUS - 1) / NUM_CUS);
    if (c.id == LLMMM_TILE_256x256) {  // a partly filled last round runs in half-size tiles where launch_fp16 can arrange it
      const long tm = M / 256, tn = N / 256, full = tiles / NUM_CUS * NUM_CUS;
      if (tiles > NUM_CUS && tm > 1 && full % tm == 0 && tn - full / tm > 0 && (tn - full / tm) * tm * 2 <= NUM_CUS) rounds -= 0.5f;
    }
    const float cost = rounds * c.bm * c.bn / c.eff;
    if (best < 0 || cost < best_cost) best = c.id, best_cost = cost;
  }
  return best;
}

constexpr int MAX_TILE_SPLIT = 8;

bool tile_dims(int tile, int& bm, int& bn);

// Split-K factor for the MFMA tile kernels: only when the tiles alone leave most of the chip idle -- at most about one
// workgroup per CU, every split at least two slices long -- and only when the shorter K loop pays for the fp32 planes'
// round trip and the second launch.  The estimate (microseconds): a 128 x 128 x 128 slice of a lone workgroup takes
// about 0.5 us (measured: 2048..19456-column outputs at M = 128..512), larger tiles in proportion; the reduce launch
// costs about 3 us and S planes are written and read at about 4 TB/s.  (M = 256, N = 6144, K = 2560 in 96 tiles:
// 14.3 us unsplit, 18.9 us in two splits; M = 256, N = 2560, K = 9728 in 40 tiles: 40 us unsplit, 18.6 us in six.)
int heuristic_tile_split(int tile, int M, int N, int K)
{
  int bm, bn;
  if (!tile_dims(tile, bm, bn)) return 1;
  const int tiles = (M / bm) * (N / bn), kb = K / 128;
  int       smax  = NUM_CUS / tiles;
  if (smax > kb / 2) smax = kb / 2;
  if (smax > MAX_TILE_SPLIT) smax = MAX_TILE_SPLIT;
  const double t_slice  = 0.5 * (double)bm * bn / (128.0 * 128.0);
  const double plane_us = (double)M * N * 4.0 * 2.0 / 4.0e6;  // one plane written and read
  int          best     = 1;
  double       best_us  = kb * t_slice;
  for (int s = 2; s <= smax; ++s) {
    const double us = ((kb + s - 1) / s) * t_slice + 3.0 + s * plane_us;
    if (us < best_us) best = s, best_us = us;
  }
  return best;
}
bool tile_dims(int tile, int& bm, int& bn)
{
  switch (tile) {
    case LLMMM_TILE_256x256: bm = 256; bn = 256; return true;
    case LLMMM_TILE_128x256: bm = 128; bn = 256; return true;
    case LLMMM_TILE_256x128: bm = 256; bn = 128; return true;
    case LLMMM_TILE_128x128: bm = 128; bn = 128; return true;
    case LLMMM_TILE_64x128: bm = 64; bn = 128; return true;  // FP16/BF16 only
    case LLMMM_TILE_128x160: bm = 128; bn = 160; return true;  // FP8 only, outputs without 1x128 groups
    default: return false;
  }
}

// ---- tune tables: entries read at run time from the file LLMMM_TUNE_FILE names (if any) come first, the compiled-in
// table (tune_table.h) second.  File format, one entry per line, '#' starts a comment:
//   skinny <m_max> <N> <K> <split_k>          FP8 weight-streaming kernel, applies to M <= m_max
//   tile   <M> <N> <K> <tile id> <split_k>    FP8 MFMA tile kernels (tile ids: LLMMM_TILE_*; split_k 0 = heuristic)
//   fp16   <M> <N> <K> <tile id>              FP16 / BF16 GEMM
// (`python -m llmmm_amd.tune --write-file PATH` writes it.)  The reference only hints at tuning: tune(N, K),
// src/mm/fp32/impl.h:20-23.
struct TuneOverride {
  std::vector<llmmm::SkinnyTune> skinny;
  std::vector<llmmm::TileTune>   tile, fp16;
};
const TuneOverride& tune_override()
{
  static const TuneOverride t = [] {
    TuneOverride o;
    const char*  path = getenv("LLMMM_TUNE_FILE");
    if (!path || !*path) return o;
    FILE* f = fopen(path, "r");
    if (!f) {
      fprintf(stderr, "llmmm: LLMMM_TUNE_FILE=%s cannot be read; using the built-in table\n", path);
      return o;
    }
    char line[256];
    int  lineno = 0;
    while (fgets(line, sizeof(line), f)) {
      ++lineno;
      if (!strchr(line, '\n') && !feof(f)) {
        // longer than the buffer: no entry is, so the whole line is dropped (its tail must not be read as a new entry)
        int ch;
        while ((ch = fgetc(f)) != EOF && ch != '\n') {}
        fprintf(stderr, "llmmm: %s:%d: line too long, ignored\n", path, lineno);
        continue;
      }
      if (char* h = strchr(line, '#')) *h = 0;
      char kind[16];
      int  a, b, c, d, e;
      const int n = sscanf(line, "%15s %d %d %d %d %d", kind, &a, &b, &c, &d, &e);
      if (n <= 0) continue;  // blank
      int bm, bn;
      if (n == 5 && !strcmp(kind, "skinny") && a >= 1 && a <= SKINNY_MAX_M && b > 0 && c > 0 && d >= 1 && d <= MAX_SPLIT_K)
        o.skinny.push_back({a, b, c, d});
      // (a tile must divide the shape it is entered for -- an entry that does not would turn a call the heuristic serves
      // into "not aligned"; the one exception is a row tail: fewer than 128 rows in 128 x 128 tiles)
      else if (n == 6 && !strcmp(kind, "tile") && a > 0 && b > 0 && c > 0 && tile_dims(d, bm, bn) && d != LLMMM_TILE_64x128 && d != LLMMM_TILE_128x160 && e >= 0 &&
               e <= MAX_SPLIT_K && b % bn == 0 && (a % bm == 0 || (a < 128 && d == LLMMM_TILE_128x128)))
        o.tile.push_back({a, b, c, d, e});
      else if (n == 5 && !strcmp(kind, "fp16") && a > 0 && b > 0 && c > 0 && tile_dims(d, bm, bn) && d != LLMMM_TILE_128x160 && a % bm == 0 && b % bn == 0)
        o.fp16.push_back({a, b, c, d, 1});
      else
        fprintf(stderr, "llmmm: %s:%d: not a tune entry, ignored\n", path, lineno);
    }
    fclose(f);
    return o;
  }();
  return t;
}

// FP8 tile kernels: the entry of this exact shape; failing that, for an (N, K) the tables know at other M, the tile of the
// entry nearest in M (by ratio, less than a factor of two away) whose tile divides this M -- its split count does not carry over (it depends on how many
// tiles M makes), the heuristic decides that.  false: nothing known about (N, K).
template <typename Table>
bool lookup_tile_in(const Table& table, int M, int N, int K, int* tile, int* split, double* best_ratio)
{
  bool found = false;
  for (const auto& e : table) {
    if (e.N != N || e.K != K) continue;
    int bm, bn;
    if (!tile_dims(e.tile, bm, bn) || N % bn) continue;
    // (an entry for fewer than 128 rows is a row tail of 128 x 128 tiles and speaks for exactly its M)
    if (M % bm && !(M < 128 && e.M == M && e.tile == LLMMM_TILE_128x128)) continue;
    if (e.M < 128 && e.M != M) continue;
    const double ratio = e.M > M ? (double)e.M / M : (double)M / e.M;
    if (ratio < *best_ratio) {
      *best_ratio = ratio, *tile = e.tile, *split = e.M == M ? e.split_k : 0;
      found = true;
    }
  }
  return found;
}
bool lookup_tile(int M, int N, int K, int* tile, int* split, bool exact_only = false)
{
  // (beyond a factor of two in M the tile count changes too much for the tuned tile to say anything: M = 8192 on the
  // 2560-column projections runs 7 % faster in the heuristic's 256 x 256 tiles than in the 128 x 128 ones tuned at M = 2048)
  const double limit = exact_only ? 1.0 + 1e-9 : 2.0;
  double       best  = limit;
  if (lookup_tile_in(tune_override().tile, M, N, K, tile, split, &best) && best == 1.0) return true;  // an exact entry of the file wins
  double best2 = best;
  int    t2 = 0, s2 = 0;
  if (lookup_tile_in(llmmm::kTileTune, M, N, K, &t2, &s2, &best2) && best2 < best) *tile = t2, *split = s2, best = best2;
  return best < limit;
}
bool lookup_skinny(int M, int N, int K, int* split, int* m_max = nullptr)
{
  for (const auto& e : tune_override().skinny)
    if (e.N == N && e.K == K && M <= e.m_max) return *split = e.split_k, (m_max ? *m_max = e.m_max : 0), true;
  for (const auto& e : llmmm::kSkinnyTune)
    if (e.N == N && e.K == K && M <= e.m_max) return *split = e.split_k, (m_max ? *m_max = e.m_max : 0), true;
  return false;
}
bool lookup_fp16_tile(int M, int N, int K, int* tile)
{
  // (an entry whose tile does not divide the shape is no entry: the heuristic decides)
  auto fits = [&](int t) {
    int bm, bn;
    return tile_dims(t, bm, bn) && M % bm == 0 && N % bn == 0;
  };
  for (const auto& e : tune_override().fp16)
    if (e.M == M && e.N == N && e.K == K && fits(e.tile)) return *tile = e.tile, true;
  for (const auto& e : llmmm::kFp16TileTune)
    if (e.M == M && e.N == N && e.K == K && fits(e.tile)) return *tile = e.tile, true;
  return false;
}

int choose_fp8(int M, int N, int K, llmmm_gemm_cfg* cfg)
{
  if (M <= 0 || N <= 0 || K <= 0) return fail(LLMMM_ERR_INVALID_ARGUMENT, "M, N and K must be positive (got %d, %d, %d)", M, N, K);
  if (N % 128 || K % 128) return fail(LLMMM_ERR_NOT_ALIGNED, "M or N or K are not aligned.");
  cfg->tile     = -1;
  cfg->split_k  = 0;
  cfg->b_layout = LLMMM_FP8_B_ROWS;
  cfg->a_layout = LLMMM_FP8_A_QUANTISED;
  {
    int t, sp;  // an entry for exactly this shape (one for fewer than 128 rows can only name the 128 x 128 tile: a row tail)
    if (lookup_tile(M, N, K, &t, &sp, true) && (M % 128 == 0 || (M < 128 && t == LLMMM_TILE_128x128))) cfg->tile = t, cfg->split_k = sp;
  }
  // 64 < M < 128 with a weight-streaming entry measured in that range (m_max < 128): it was timed against the row-tail
  // tiles below and won (2560 x 9728 up to 96 rows: 13.0 us in four splits of 32-row groups, 14.5 us in tiles)
  if (cfg->tile < 0 && M > 64 && M < 128) {
    int sp, mm;
    if (lookup_skinny(M, N, K, &sp, &mm) && mm < 128) cfg->tile = LLMMM_TILE_SKINNY, cfg->split_k = sp;
  }
  // 64 < M < 128: where the table gives M = 128 to 128 x 128 tiles, the same tiles take the shorter matrix too (the
  // rows of the tile beyond M are computed and not stored) -- 96 x 19456 x 2560: 20 us instead of 33 us in the
  // weight-streaming kernel, whose eight 16-row blocks per wave are bound by their LDS reads and fp32 planes
  // (where that entry is unsplit -- enough column groups to fill the chip, i.e. a large weight matrix -- already from 33
  // rows on: 19456 x 2560 at M = 48 / 64: 15.9 / 16.7 us in tiles, 18.0 / 19.5 us streaming in three splits; at 32: 15.3 / 15.5)
  if (cfg->tile < 0 && M > 32 && M < 128) {
    int t, sp;
    if (lookup_tile(128, N, K, &t, &sp, true) && t == LLMMM_TILE_128x128 && (M > 64 || sp <= 1)) cfg->tile = t, cfg->split_k = sp;
  }
  if (cfg->tile < 0 && M <= SKINNY_MAX_M) {
    int sp;
    if (lookup_skinny(M, N, K, &sp)) cfg->tile = LLMMM_TILE_SKINNY, cfg->split_k = sp;
    // untuned shapes: the weight-streaming kernel up to 64 rows; above that only while the weight matrix is small -- its
    // eight 16-row blocks per wave and its fp32 planes grow with M, and from about 20 MB of weights on, one row of 128 x 128
    // tiles (a row tail for M < 128) is faster (measured at M = 96, us, streaming / tiles: N x K = 4096 x 4096 12.4 / 14.2,
    // 6144 x 4096 19.9 / 16.0, 4096 x 14336 39.4 / 22.1, 28672 x 4096 66.7 / 27.1)
    // (from 40 MB on the tiles win from 33 rows on, as on the tuned 19456 x 2560)
    if (cfg->tile < 0) cfg->tile = (M <= 32 || (long)N * K < 20000000L || (M <= 64 && (long)N * K < 40000000L)) ? LLMMM_TILE_SKINNY : LLMMM_TILE_128x128;
  }
  if (cfg->tile < 0) {
    if (M % 128) return fail(LLMMM_ERR_NOT_ALIGNED, "M or N or K are not aligned.");
    // an (N, K) that was tuned at other M: the tile of the nearest tuned M; otherwise the heuristic
    int t, sp;
    if (lookup_tile(M, N, K, &t, &sp))
      cfg->tile = t, cfg->split_k = sp;
    else
      cfg->tile = heuristic_tile(M, N);
  }
  if (cfg->tile == LLMMM_TILE_SKINNY) {
    if (cfg->split_k <= 0) cfg->split_k = heuristic_split(M, N, K);
  }
  else if (cfg->split_k <= 0)
    cfg->split_k = heuristic_tile_split(cfg->tile, M < 128 ? 128 : M, N, K);
  return LLMMM_OK;
}

// The SwiGLU output.  In the tile kernels the activation is either fused into the epilogue of a 256-column tile
// (whose two halves are the gate and the up columns of the same outputs), or -- with a 128-column tile, or
// whenever K is split -- applied by the reduce kernel to fp32 planes in the workspace.  The second way costs a
// round trip of M * N floats, which only pays while that is small and the 256-column tiles would leave
// most of the chip idle (decode-sized M).
constexpr size_t SWIGLU_PLANE_LIMIT = 16u << 20;

// Outputs without 1x128 groups (fp32, bf16, residual add) may use the 160-column tile: when 128 x 128 tiles were chosen,
// are not split, and 160-column ones need fewer rounds of the chip -- 2560 columns at M = 2048: 320 tiles (two rounds,
// the second a quarter full) against 256 (one).  Measured on O / down at M = 2048: 30.0 -> 26.9 us, 64.0 -> 55.8 us.
void prefer_wide_tile(llmmm_gemm_cfg* cfg, int M, int N)
{
  // (or 256 x 128 tiles, which the table and the heuristic name where 128 x 128 ones would sit two to a CU: one 128 x 160 tile
  // per CU is as fast on weights from HBM and faster on cached ones -- 1024 x 5120 x 2560, us: 19.8 / 19.0 against 21.3 / 20.9)
  if ((cfg->tile != LLMMM_TILE_128x128 && cfg->tile != LLMMM_TILE_256x128) || cfg->split_k > 1 || N % 640 || M % 128) return;
  const long t128 = (long)(M / 128) * (N / 128), t160 = (long)(M / 128) * (N / 160);
  if ((t160 + NUM_CUS - 1) / NUM_CUS < (t128 + NUM_CUS - 1) / NUM_CUS) cfg->tile = LLMMM_TILE_128x160;
}

// The weight-streaming kernel in column strips (one launch, the K split inside the workgroup) takes what the split-K
// form of that kernel would otherwise do in two launches, for the outputs it has: no 1x128 groups.
bool strip_fits(int M, int N, int K) { return M >= 1 && M <= llmmm::STRIP_MAX_M && N % 16 == 0 && K % 128 == 0 && K / 128 >= 8; }
// Where strips beat the split-K form with its second kernel (measured, pre-shuffled weights; `fused` = with the 1x128
// quantisation, whose exchange between the strips of a column group costs 1.4 - 1.6 us, about what the reduce launch did).
// Every strip reads all M activation rows over all of K, so the strips' cost grows with M while the split form's hardly does.
//  * at most one 16-column strip per CU (2560 and 4096 columns): plain outputs up to M = 8, up to 16 for K <= 4096; fused
//    while M * K <= 65536 (2560 x 4096, us, strips / split + reduce: 5.4 / 6.5 at M = 1, 6.6 / 7.0 at 16; 2560 x 9728: 8.0 / 8.4
//    at M = 1, 9.1 / 9.0 at 8);
//  * more, but 32-column strips fit one round and the matrix is small (llmmm::strip_fragments; 6144 x 2560, 6144 x 4096,
//    5120 x 5120): plain outputs as above (6144 x 4096 at M = 16: 7.5 / 8.8), fused up to M = 4 (6144 x 2560: 6.2 / 6.65 at M = 1,
//    7.0 / 6.7 at 8; 6144 x 4096: 7.2 / 8.65 and 7.8 / 8.7; 5120 x 5120: 7.9 / 8.4 and 8.7 / 8.55);
//  * two 16-column strips on (nearly) every CU -- between 1.75 and 2 per CU, which share it side by side (8192 x 8192, 512
//    strips: 13.2 / 15.1 fused at M = 1, 14.3 / 15.3 at 8, 16.5 / 15.3 at 16; 7168 x 5120, 448 strips: 10.3 / 11.7 at M = 1;
//    8192 x 28672: 39.9 / 39.5 at M = 1 and 40.7 / 37.6 at 4, hence the same M * K bound as above);
//  * otherwise not: 5120 x 13824 at M = 1 takes 19.5 us in 320 strips, a round and a quarter, and 14.8 us in six splits
//    (5120 x 17408: 21.4 / 17.5; 10240 x 8192, 640 strips: 17.9 / 18.1).
bool strips_pay(int M, int N, int K, bool fused)
{
  const long cus = NUM_CUS, s16 = N / 16;
  const bool plain_ok = M <= 8 || (M <= 16 && K <= 4096);
  if (s16 <= cus) return fused ? (long)M * K <= 65536 : plain_ok;
  if (llmmm::strip_fragments(N, K) == 2) return fused ? M <= 4 : plain_ok;
  if (s16 <= 2 * cus && s16 * 8 >= 2 * cus * 7) return (long)M * K <= (fused ? 65536 : 131072);  // (plain: 8192 x 8192 up to M = 16)
  return false;
}
// Plain outputs, one 16-column strip per CU, measured against the split form (bf16 out, us, strips / split + reduce):
// O 4.0 / 6.2 (M = 1), 4.9 / 6.5 (8), 5.6 / 6.8 (16), 7.7 / 7.3 (32); down 6.7 / 8.2, 7.7 / 8.9, 9.4 / 9.1, 13.7 / 9.7.
void prefer_strip(llmmm_gemm_cfg* cfg, int M, int N, int K)
{
  if (cfg->tile == LLMMM_TILE_SKINNY && cfg->split_k > 1 && strip_fits(M, N, K) && strips_pay(M, N, K, false)) cfg->tile = LLMMM_TILE_STRIP, cfg->split_k = 1;
}

// The fused 1x128 output in column strips (one launch; the strips of a column group exchange their row maxima through
// device memory, fp8_skinny.hip): M <= 16 and few enough column groups for the exchange area.
bool strip_fp8q_fits(int M, int N, int K) { return strip_fits(M, N, K) && M <= 16 && N % 128 == 0 && N / 128 <= llmmm::STRIP_XCH_MAX_GROUPS; }
void prefer_strip_fp8q(llmmm_gemm_cfg* cfg, int M, int N, int K)
{
  if (cfg->tile == LLMMM_TILE_SKINNY && cfg->split_k > 1 && strip_fp8q_fits(M, N, K) && strips_pay(M, N, K, true)) cfg->tile = LLMMM_TILE_STRIP, cfg->split_k = 1;
}

// The exchange area of a stream (0 .. STRIP_XCH_AREAS - 1): launches on one stream are ordered, so they may share an
// area; every stream the library meets gets one of its own, for the life of the process, and streams beyond the number
// of areas get -1 -- their calls keep the split-K form.  Host bookkeeping only: nothing here touches the device.
int strip_exchange_area(void* stream)
{
  static std::mutex mu;
  static void*      owner[llmmm::STRIP_XCH_AREAS];
  static int        used = 0;
  std::lock_guard<std::mutex> lock(mu);
  for (int i = 0; i < used; ++i)
    if (owner[i] == stream) return i;
  if (used == llmmm::STRIP_XCH_AREAS) return -1;
  owner[used] = stream;
  return used++;
}

// The split the weight-streaming kernel runs this shape in when it is the split-K form after all (tune table, then heuristic).
int skinny_split_for(int M, int N, int K)
{
  int sp;
  return lookup_skinny(M, N, K, &sp) ? sp : heuristic_split(M, N, K);
}

// Planes a strip-capable shape needs when the call turns out not to run in strips after all: activations the kernel makes
// itself (cfg.a_layout) and explicit splits belong to the split-K form, and generated activations need a split whose K
// range fits the staging buffer.  The size queries cannot see the caller's cfg, so they answer for this case.
size_t strip_fallback_plane_bytes(int M, int N, int K)
{
  int s = skinny_split_for(M, N, K);
  const int kb = K / 128, min_split = (kb + 31) / 32;  // = agen_min_split(K)
  if (s < min_split) s = min_split;
  if (s > max_split_for(K)) s = max_split_for(K);
  return (size_t)(s < 1 ? 1 : s) * M * N * sizeof(float);
}

int choose_fp8_out(int out_kind, int M, int N, int K, llmmm_gemm_cfg* cfg)
{
  const int rc = choose_fp8(M, N, K, cfg);
  if (rc) return rc;
  if (out_kind == LLMMM_OUT_F32 || out_kind == LLMMM_OUT_BF16) prefer_wide_tile(cfg, M, N), prefer_strip(cfg, M, N, K);
  if (out_kind == LLMMM_OUT_FP8Q) prefer_strip_fp8q(cfg, M, N, K);
  if (out_kind == LLMMM_OUT_FP8Q_SWIGLU) {
    if (N % 256) return fail(LLMMM_ERR_NOT_ALIGNED, "M or N or K are not aligned.");
    if (cfg->tile != LLMMM_TILE_SKINNY && cfg->split_k <= 1) {
      const bool narrow      = cfg->tile == LLMMM_TILE_256x128 || cfg->tile == LLMMM_TILE_128x128;
      const long wide_tiles  = (long)(M / 128) * (N / 256);
      const bool small_plane = (size_t)M * N * sizeof(float) <= SWIGLU_PLANE_LIMIT;
      if (small_plane && wide_tiles < NUM_CUS / 2) {
        if (!narrow) cfg->tile = LLMMM_TILE_128x128;  // through one fp32 plane, twice the workgroups
      }
      else if (narrow && M % 128 == 0)  // (a row tail stays with the 128 x 128 tiles and the plane)
        cfg->tile = (M % 256 == 0 && (long)(M / 256) * (N / 256) >= NUM_CUS) ? LLMMM_TILE_256x256 : LLMMM_TILE_128x256;
    }
  }
  return LLMMM_OK;
}

}  // namespace

extern "C" {

const char* llmmm_error_string(int code)
{
  switch (code) {
    case LLMMM_OK: return "ok";
    case LLMMM_ERR_NOT_ALIGNED: return "M or N or K are not aligned.";
    case LLMMM_ERR_UNSUPPORTED_TYPE: return "T is not supported.";
    case LLMMM_ERR_INVALID_ARGUMENT: return "invalid argument";
    case LLMMM_ERR_WORKSPACE: return "workspace missing or too small";
    case LLMMM_ERR_RUNTIME: return "HIP runtime error";
    default: return "unknown error";
  }
}

const char* llmmm_last_error(void) { return g_last_error; }

int llmmm_version(void) { return 100; }

int llmmm_fp16_gemm_ex(int dtype, const void* A, const void* B, void* C, int M, int N, int K, int b_layout,
                       const llmmm_gemm_cfg* cfg, void* stream)
{
  if (dtype != LLMMM_DTYPE_F16 && dtype != LLMMM_DTYPE_BF16) return fail(LLMMM_ERR_UNSUPPORTED_TYPE, "T is not supported.");
  if (b_layout != LLMMM_B_ROW_MAJOR && b_layout != LLMMM_B_TRANSPOSED)
    return fail(LLMMM_ERR_INVALID_ARGUMENT, "unknown B layout %d", b_layout);
  if (M <= 0 || N <= 0 || K <= 0) return fail(LLMMM_ERR_INVALID_ARGUMENT, "M, N and K must be positive (got %d, %d, %d)", M, N, K);
  if (M % 128 || N % 128 || K % 16) return fail(LLMMM_ERR_NOT_ALIGNED, "M or N or K are not aligned.");
  if (!A || !B || !C) return fail(LLMMM_ERR_INVALID_ARGUMENT, "null pointer");
  if (!aligned16(A) || !aligned16(B) || !aligned16(C)) return fail(LLMMM_ERR_INVALID_ARGUMENT, "pointers must be 16-byte aligned");
  if ((long)M * K >= (1L << 31) || (long)N * K >= (1L << 31) || (long)M * N >= (1L << 31))
    return fail(LLMMM_ERR_INVALID_ARGUMENT, "matrix has 2^31 or more elements");
  int tile = cfg ? cfg->tile : LLMMM_TILE_AUTO;
  if (tile == LLMMM_TILE_AUTO) {
    if (!lookup_fp16_tile(M, N, K, &tile)) tile = LLMMM_TILE_AUTO;
    if (tile == LLMMM_TILE_AUTO) {
      tile = heuristic_tile_fp16(M, N);
      // small problems: 128 x 128 tiles on at most half of the CUs -> twice as many 64 x 128 tiles of four 16-row
      // waves (1024^3: 8.0 instead of 11.3 us; from 160 tiles of 128 x 128 on, the larger tile wins again)
      if (tile == LLMMM_TILE_128x128 && (long)(M / 128) * (N / 128) <= NUM_CUS / 2) tile = LLMMM_TILE_64x128;
    }
  }
  int bm, bn;
  if (!tile_dims(tile, bm, bn) || tile == LLMMM_TILE_128x160) return fail(LLMMM_ERR_INVALID_ARGUMENT, "unknown tile id %d", tile);
  if (M % bm || N % bn) return fail(LLMMM_ERR_NOT_ALIGNED, "M or N or K are not aligned.");
  const hipError_t e = llmmm::fp16_gemm_launch(dtype, b_layout, tile, A, B, C, M, N, K, (hipStream_t)stream);
  if (e != hipSuccess) return fail(LLMMM_ERR_RUNTIME, "fp16 gemm launch: %s", hipGetErrorString(e));
  return LLMMM_OK;
}

int llmmm_fp16_gemm(int dtype, const void* A, const void* B, void* C, int M, int N, int K, int b_layout, void* stream)
{
  return llmmm_fp16_gemm_ex(dtype, A, B, C, M, N, K, b_layout, nullptr, stream);
}

int llmmm_fp8_gemm_query(int out_kind, int M, int N, int K, llmmm_gemm_cfg* cfg)
{
  if (out_kind < LLMMM_OUT_F32 || out_kind > LLMMM_OUT_FP8Q_SWIGLU) return fail(LLMMM_ERR_INVALID_ARGUMENT, "unknown output kind %d", out_kind);
  if (!cfg) return fail(LLMMM_ERR_INVALID_ARGUMENT, "null cfg");
  return choose_fp8_out(out_kind, M, N, K, cfg);
}

size_t llmmm_fp8_gemm_workspace(int out_kind, int M, int N, int K)
{
  if (M <= 0 || N <= 0 || K <= 0 || N % 128 || K % 128) return 0;
  llmmm_gemm_cfg cfg;
  if (choose_fp8_out(out_kind, M, N, K, &cfg) != LLMMM_OK) return 0;
  if (cfg.tile == LLMMM_TILE_STRIP) return strip_fallback_plane_bytes(M, N, K);  // strips need none; a call with generated activations leaves them
  const int  s       = cfg.split_k;  // the split the library would pick (an explicit cfg->split_k = S needs S planes)
  const bool narrow  = cfg.tile == LLMMM_TILE_256x128 || cfg.tile == LLMMM_TILE_128x128;
  const bool a_plane = out_kind == LLMMM_OUT_FP8Q_SWIGLU && (cfg.tile == LLMMM_TILE_SKINNY || narrow);  // SwiGLU outside a 256-column tile
  if (s <= 1 && !a_plane) return 0;
  return (size_t)(s < 1 ? 1 : s) * M * N * sizeof(float);
}

// cfg.a_layout = LLMMM_FP8_A_SWIGLU_F32: the weight-streaming kernel makes the activations itself for M <= 4 when a
// split's K range fits its staging buffer (32 slices of 128); otherwise h is quantised into the front of the workspace.
// (Every column group's workgroup repeats the activation work of its K range, so its cost grows with M: measured on the
// Qwen3-4B down projection, +0.8 us at M = 1, +1.8 at M = 4, +2.5 at M = 8, +4.6 at M = 16, against the 2.4 us that the
// separate SwiGLU quantiser launch costs.  The kernel itself takes up to 16 rows.)
constexpr int AGEN_MAX_M = 4, AGEN_MAX_SLICES = 32;
static size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }
static size_t swiglu_a_bytes(int M, int K) { return align256((size_t)M * K) + align256((size_t)(K / 128) * M * sizeof(float)); }
static int agen_min_split(int K) { return ((K / 128) + AGEN_MAX_SLICES - 1) / AGEN_MAX_SLICES; }

size_t llmmm_fp8_swiglu_a_workspace(int M, int N, int K)
{
  llmmm_gemm_cfg cfg;
  if (choose_fp8(M, N, K, &cfg) != LLMMM_OK) return 0;
  if (cfg.tile == LLMMM_TILE_SKINNY && M <= AGEN_MAX_M) return 0;
  return swiglu_a_bytes(M, K);
}

// How a call gets its A operand: given quantised (agen 0), generated by the weight-streaming kernel from the fp32 gate_up
// result (1) or from a hidden state still in pieces (2, with what the kernel needs in `ag`).
struct APrep {
  int               agen         = 0;
  int               hidden_dtype = 0;
  llmmm::SkinnyGenA ag;
};
constexpr int AGEN2_MAX_M = 2, AGEN2_MAX_K = 3072;

size_t llmmm_fp8_planes_rmsnorm_a_workspace(int M, int N, int K)
{
  llmmm_gemm_cfg cfg;
  if (choose_fp8(M, N, K, &cfg) != LLMMM_OK) return 0;
  // (the generating kernel writes fp32 only: any other output kind goes through one fp32 plane and the reduce kernel, and
  // an unsplit call has no plane in llmmm_fp8_gemm_workspace's answer -- this one covers it)
  if (cfg.tile == LLMMM_TILE_SKINNY && M <= AGEN2_MAX_M && K <= AGEN2_MAX_K) return (size_t)M * N * sizeof(float);
  return swiglu_a_bytes(M, K);  // the same codes + scales block
}

// Resolves a_layout for a call whose kernel choice is `tile`: either the kernel generates A (prep->agen != 0; A is not
// used as an operand pointer any more), or the operand is quantised into the front of the workspace now and A / As /
// workspace are redirected to it.
static int prepare_a(const llmmm_gemm_cfg* user, int tile, const void*& A, const float*& As, int M, int K, void*& workspace, size_t& workspace_bytes,
                     void* stream, APrep* prep)
{
  *prep = APrep();
  if (!user || user->a_layout == LLMMM_FP8_A_QUANTISED) return LLMMM_OK;
  if (user->a_layout != LLMMM_FP8_A_SWIGLU_F32 && user->a_layout != LLMMM_FP8_A_PLANES_RMSNORM)
    return fail(LLMMM_ERR_INVALID_ARGUMENT, "unknown A layout %d", user->a_layout);
  if ((long)M * 2 * K >= (1L << 31)) return fail(LLMMM_ERR_INVALID_ARGUMENT, "matrix has 2^31 or more elements");
  const llmmm_a_planes_rmsnorm* d = nullptr;
  if (user->a_layout == LLMMM_FP8_A_PLANES_RMSNORM) {
    d = (const llmmm_a_planes_rmsnorm*)A;  // a host structure
    if (!d->planes || !d->residual || !d->hidden_out || !d->norm_weight) return fail(LLMMM_ERR_INVALID_ARGUMENT, "null pointer");
    if (d->hidden_dtype != LLMMM_DTYPE_F16 && d->hidden_dtype != LLMMM_DTYPE_BF16 && d->hidden_dtype != LLMMM_DTYPE_F32)
      return fail(LLMMM_ERR_UNSUPPORTED_TYPE, "T is not supported.");
    if (d->splits < 1 || d->splits > MAX_SPLIT_K) return fail(LLMMM_ERR_INVALID_ARGUMENT, "splits must be 1..%d (got %d)", MAX_SPLIT_K, d->splits);
    if (!(d->eps >= 0.f)) return fail(LLMMM_ERR_INVALID_ARGUMENT, "eps must be non-negative");
    if (K > 10240) return fail(LLMMM_ERR_INVALID_ARGUMENT, "the fused norm handles rows of at most 10240 columns (got %d)", K);
    if (!aligned16(d->planes) || !aligned16(d->residual) || !aligned16(d->hidden_out) || !aligned16(d->norm_weight))
      return fail(LLMMM_ERR_INVALID_ARGUMENT, "pointers must be 16-byte aligned");
    // (every generating workgroup reads the residual while one writes the hidden state: an in-place update takes the
    // quantise-first route below, where one workgroup owns each row)
    if (tile == LLMMM_TILE_SKINNY && M <= AGEN2_MAX_M && K <= AGEN2_MAX_K && d->splits <= llmmm::SKINNY_GEN_MAX_PLANES && d->hidden_out != d->residual) {
      prep->agen         = 2;
      prep->hidden_dtype = d->hidden_dtype;
      prep->ag.planes = d->planes, prep->ag.residual = d->residual, prep->ag.hidden = d->hidden_out, prep->ag.w = d->norm_weight;
      prep->ag.eps = d->eps, prep->ag.splits = d->splits;
      return LLMMM_OK;
    }
  }
  else if (tile == LLMMM_TILE_SKINNY && M <= AGEN_MAX_M) {
    prep->agen = 1;
    return LLMMM_OK;
  }
  const size_t need = swiglu_a_bytes(M, K);
  if (!workspace || workspace_bytes < need)
    return fail(LLMMM_ERR_WORKSPACE, "workspace holds %zu bytes, quantising the activations first needs %zu", workspace ? workspace_bytes : (size_t)0, need);
  if (!aligned16(workspace)) return fail(LLMMM_ERR_INVALID_ARGUMENT, "workspace must be 16-byte aligned");
  uint8_t*   hq = (uint8_t*)workspace;
  float*     hs = (float*)(hq + align256((size_t)M * K));
  hipError_t e;
  if (d)
    e = llmmm::planes_add_rmsnorm_quant_launch(d->hidden_dtype, d->planes, d->splits, d->residual, d->hidden_out, d->norm_weight, d->eps, hq, hs, M, K,
                                               (hipStream_t)stream);
  else
    e = llmmm::fp8_splitk_reduce_launch(LLMMM_OUT_FP8Q_SWIGLU, (const float*)A, 1, hq, hs, M, 2 * K, (hipStream_t)stream);
  if (e != hipSuccess) return fail(LLMMM_ERR_RUNTIME, "activation quantiser launch: %s", hipGetErrorString(e));
  A               = hq;
  As              = hs;
  workspace       = hq + need;
  workspace_bytes = workspace_bytes - need;
  if (workspace_bytes == 0) workspace = nullptr;
  return LLMMM_OK;
}

int llmmm_fp8_gemm_ex(int out_kind, const void* A, const float* As, const void* Bt, const float* Bs, void* C, float* Cs, int M,
                      int N, int K, void* workspace, size_t workspace_bytes, const llmmm_gemm_cfg* user, void* stream)
{
  if (out_kind < LLMMM_OUT_F32 || out_kind > LLMMM_OUT_FP8Q_SWIGLU) return fail(LLMMM_ERR_INVALID_ARGUMENT, "unknown output kind %d", out_kind);
  const bool     swiglu = out_kind == LLMMM_OUT_FP8Q_SWIGLU;
  llmmm_gemm_cfg cfg;
  const int      rc = choose_fp8_out(out_kind, M, N, K, &cfg);
  if (rc) return rc;
  const bool a_swiglu = user && user->a_layout == LLMMM_FP8_A_SWIGLU_F32;
  const bool a_made   = user && user->a_layout != LLMMM_FP8_A_QUANTISED;  // A is not the quantised operand: As is not used
  if (!A || (!As && !a_made) || !Bt || !Bs || !C) return fail(LLMMM_ERR_INVALID_ARGUMENT, "null pointer");
  if (a_swiglu && swiglu) return fail(LLMMM_ERR_INVALID_ARGUMENT, "SwiGLU on both the A operand and the output");
  if ((out_kind == LLMMM_OUT_FP8Q || swiglu) && !Cs) return fail(LLMMM_ERR_INVALID_ARGUMENT, "C_scale_transposed is required for fp8 output");
  // (with a_layout = PLANES_RMSNORM, A is a host structure: prepare_a checks the device pointers inside it)
  const bool a_host = user && user->a_layout == LLMMM_FP8_A_PLANES_RMSNORM;
  if ((!a_host && !aligned16(A)) || !aligned16(Bt) || !aligned16(C)) return fail(LLMMM_ERR_INVALID_ARGUMENT, "pointers must be 16-byte aligned");
  if ((long)M * K >= (1L << 31) || (long)N * K >= (1L << 31) || (long)M * N >= (1L << 31))
    return fail(LLMMM_ERR_INVALID_ARGUMENT, "matrix has 2^31 or more elements");
  if (user) {
    // (a named weight-streaming kernel where the library would have taken tiles: the split is that kernel's own heuristic)
    if (user->tile == LLMMM_TILE_SKINNY && cfg.tile == LLMMM_TILE_STRIP)
      cfg.split_k = skinny_split_for(M, N, K);  // (the split-K form named where the library would have taken strips)
    else if (user->tile == LLMMM_TILE_SKINNY && cfg.tile != LLMMM_TILE_SKINNY && M <= SKINNY_MAX_M)
      cfg.split_k = heuristic_split(M, N, K);
    if (user->tile != LLMMM_TILE_AUTO) cfg.tile = user->tile;
    if (user->split_k > 0) cfg.split_k = user->split_k;
    if (user->b_layout != LLMMM_FP8_B_ROWS && user->b_layout != LLMMM_FP8_B_PRESHUFFLED)
      return fail(LLMMM_ERR_INVALID_ARGUMENT, "unknown B layout %d", user->b_layout);
    cfg.b_layout = user->b_layout;
  }
  hipError_t e;
  APrep      prep;
  if (cfg.tile == LLMMM_TILE_SKINNY && M > SKINNY_MAX_M) return fail(LLMMM_ERR_INVALID_ARGUMENT, "the weight-streaming kernel handles M <= %d", SKINNY_MAX_M);
  const int rca = prepare_a(user, cfg.tile, A, As, M, K, workspace, workspace_bytes, stream, &prep);
  if (rca) return rca;
  const int agen = prep.agen;
  if (cfg.tile == LLMMM_TILE_STRIP && (agen || (user && user->split_k > 1))) {
    // generated activations and an explicit split are the split-K form's: a strip the library picked itself gives way, one asked for is refused
    if (user && user->tile == LLMMM_TILE_STRIP) return fail(LLMMM_ERR_INVALID_ARGUMENT, "the column-strip kernel takes quantised activations and does not split K over workgroups");
    cfg.tile = LLMMM_TILE_SKINNY;
    if (!(user && user->split_k > 0)) cfg.split_k = skinny_split_for(M, N, K);
  }
  int xarea = -1;
  if (cfg.tile == LLMMM_TILE_STRIP && out_kind == LLMMM_OUT_FP8Q && strip_fp8q_fits(M, N, K) && (xarea = strip_exchange_area(stream)) < 0 &&
      !(user && user->tile == LLMMM_TILE_STRIP)) {
    // more streams than exchange areas: a strip the library picked itself gives way to the split-K form
    cfg.tile    = LLMMM_TILE_SKINNY;
    cfg.split_k = skinny_split_for(M, N, K);
  }
  if (cfg.tile == LLMMM_TILE_STRIP) {
    if (out_kind == LLMMM_OUT_FP8Q) {
      if (!strip_fp8q_fits(M, N, K))
        return fail(LLMMM_ERR_INVALID_ARGUMENT, "the column-strip kernel quantises C for M <= 16, K >= 1024 and at most %d column groups", llmmm::STRIP_XCH_MAX_GROUPS);
      if (xarea < 0) return fail(LLMMM_ERR_INVALID_ARGUMENT, "the column-strip kernel's fp8 output serves %d streams per process", llmmm::STRIP_XCH_AREAS);
      e = llmmm::fp8_strip_fp8q_launch(cfg.b_layout, A, As, Bt, Bs, C, Cs, M, N, K, xarea, (hipStream_t)stream);
    }
    else {
      if (out_kind != LLMMM_OUT_F32 && out_kind != LLMMM_OUT_BF16) return fail(LLMMM_ERR_INVALID_ARGUMENT, "the column-strip kernel has fp32, bf16 and fp8 (1x128) outputs only");
      if (!strip_fits(M, N, K)) return fail(LLMMM_ERR_INVALID_ARGUMENT, "the column-strip kernel handles M <= %d and K >= 1024", llmmm::STRIP_MAX_M);
      e = llmmm::fp8_strip_launch(out_kind, cfg.b_layout, A, As, Bt, Bs, C, M, N, K, (hipStream_t)stream);
    }
  }
  else if (cfg.tile == LLMMM_TILE_SKINNY) {
    int split = cfg.split_k;
    if (split > max_split_for(K)) split = max_split_for(K);
    if (split < 1) split = 1;
    if (!workspace) split = 1;  // documented: no workspace, no split
    const int min_split = agen ? agen_min_split(K) : 1;  // generated activations: a split's K range must fit the staging buffer
    if (split < min_split) {
      if ((user && user->split_k > 0) || !workspace)
        return fail(user && user->split_k > 0 ? LLMMM_ERR_INVALID_ARGUMENT : LLMMM_ERR_WORKSPACE,
                    "generated activations need split-K >= %d for K = %d (at most %d slices of 128 per split), and a workspace for it", min_split, K, AGEN_MAX_SLICES);
      split = min_split;
    }
    float* partial = nullptr;
    if (swiglu && !workspace) return fail(LLMMM_ERR_WORKSPACE, "the SwiGLU output at M <= %d needs a workspace of at least M * N floats", SKINNY_MAX_M);
    if (split > 1 && !(user && user->split_k > 0)) {
      // a split the library chose itself shrinks to what the caller's workspace holds
      const size_t room = workspace_bytes / ((size_t)M * N * sizeof(float));
      if ((size_t)split > room) split = room < 2 ? 1 : (int)room;
      if (split < min_split) split = min_split;  // (fails the size check below)
    }
    // (the norm-generating kernel only writes fp32: any other output goes through one plane and the reduce kernel)
    if (split > 1 || swiglu || (agen == 2 && out_kind != LLMMM_OUT_F32)) {
      const size_t need = (size_t)split * M * N * sizeof(float);
      if (!workspace || workspace_bytes < need) return fail(LLMMM_ERR_WORKSPACE, "workspace holds %zu bytes, split-K %d needs %zu", workspace ? workspace_bytes : (size_t)0, split, need);
      if (!aligned16(workspace)) return fail(LLMMM_ERR_INVALID_ARGUMENT, "workspace must be 16-byte aligned");
      partial = (float*)workspace;
    }
    if (agen == 2)
      e = llmmm::fp8_skinny_rmsnorm_a_launch(prep.hidden_dtype, cfg.b_layout, prep.ag, Bt, Bs, (float*)C, M, N, K, split, partial, (hipStream_t)stream);
    else if (agen)
      e = llmmm::fp8_skinny_swiglu_a_launch(partial ? LLMMM_OUT_F32 : out_kind, cfg.b_layout, (const float*)A, Bt, Bs, C, Cs, M, N, K, split, partial,
                                            (hipStream_t)stream);
    else
      e = llmmm::fp8_skinny_launch(partial ? LLMMM_OUT_F32 : out_kind, cfg.b_layout, A, As, Bt, Bs, C, Cs, M, N, K, split, partial, (hipStream_t)stream);
    if (e == hipSuccess && partial) e = llmmm::fp8_splitk_reduce_launch(out_kind, partial, split, C, Cs, M, N, (hipStream_t)stream);
  }
  else {
    int bm, bn;
    if (!tile_dims(cfg.tile, bm, bn) || cfg.tile == LLMMM_TILE_64x128) return fail(LLMMM_ERR_INVALID_ARGUMENT, "unknown tile id %d", cfg.tile);
    if (cfg.tile == LLMMM_TILE_128x160 && (out_kind == LLMMM_OUT_FP8Q || swiglu)) {
      // its waves straddle the 1x128 groups of the fused quantisation: a tile the library picked itself gives way, one asked for is refused
      if (user && user->tile == LLMMM_TILE_128x160) return fail(LLMMM_ERR_INVALID_ARGUMENT, "the 128 x 160 tile has no fp8 output");
      cfg.tile = LLMMM_TILE_128x128;
      tile_dims(cfg.tile, bm, bn);
    }
    // (128 x 128 tiles also take a single tile row of fewer than 128 rows)
    if ((M % bm && !(cfg.tile == LLMMM_TILE_128x128 && M < 128)) || N % bn) return fail(LLMMM_ERR_NOT_ALIGNED, "M or N or K are not aligned.");
    if (user && user->tile != LLMMM_TILE_AUTO && user->split_k <= 0) cfg.split_k = heuristic_tile_split(cfg.tile, M < bm ? bm : M, N, K);
    int split = cfg.split_k;
    if (split > K / 128) split = K / 128;
    if (split > MAX_SPLIT_K) split = MAX_SPLIT_K;
    if (split < 1 || !workspace) split = 1;  // documented: no workspace, no split
    float* planes = nullptr;
    if (split > 1 && !(user && user->split_k > 0)) {
      // a split the library chose itself shrinks to what the caller's workspace holds
      const size_t plane = (size_t)M * N * sizeof(float);
      const size_t room  = workspace_bytes / plane;
      if ((size_t)split > room) split = room < 2 ? 1 : (int)room;
    }
    if (swiglu && split <= 1 && bn != 256 && (!workspace || workspace_bytes < (size_t)M * N * sizeof(float))) {
      // no room for the fp32 plane a 128-column tile needs: the fused epilogue of a 256-column tile instead
      if ((user && user->tile != LLMMM_TILE_AUTO) || M % 128)
        return fail(LLMMM_ERR_WORKSPACE, "the SwiGLU output from a 128-column tile needs a workspace of M * N floats");
      cfg.tile = LLMMM_TILE_128x256;
      bn       = 256;
    }
    if (split > 1 || (swiglu && bn != 256)) {
      const size_t need = (size_t)split * M * N * sizeof(float);
      if (workspace_bytes < need) return fail(LLMMM_ERR_WORKSPACE, "workspace holds %zu bytes, split-K %d needs %zu", workspace_bytes, split, need);
      if (!aligned16(workspace)) return fail(LLMMM_ERR_INVALID_ARGUMENT, "workspace must be 16-byte aligned");
      planes = (float*)workspace;
    }
    e = llmmm::fp8_gemm_launch(out_kind, cfg.tile, cfg.b_layout, A, As, Bt, Bs, C, Cs, M, N, K, split, planes, (hipStream_t)stream);
  }
  if (e != hipSuccess) return fail(LLMMM_ERR_RUNTIME, "fp8 gemm launch: %s", hipGetErrorString(e));
  return LLMMM_OK;
}

int llmmm_fp8_gemm(int out_kind, const void* A, const float* As, const void* Bt, const float* Bs, void* C, float* Cs, int M, int N,
                   int K, void* workspace, size_t workspace_bytes, void* stream)
{
  return llmmm_fp8_gemm_ex(out_kind, A, As, Bt, Bs, C, Cs, M, N, K, workspace, workspace_bytes, nullptr, stream);
}

int llmmm_quant_fp8(int kind, const float* x, void* q, float* scale, int M, int N, void* stream)
{
  if (kind < LLMMM_QUANT_1x128_T || kind > LLMMM_QUANT_128x128_T) return fail(LLMMM_ERR_INVALID_ARGUMENT, "unknown quantiser kind %d", kind);
  if (M <= 0 || N <= 0) return fail(LLMMM_ERR_INVALID_ARGUMENT, "M and N must be positive (got %d, %d)", M, N);
  if (N % 4) return fail(LLMMM_ERR_NOT_ALIGNED, "M or N or K are not aligned.");
  if (!x || !q || !scale) return fail(LLMMM_ERR_INVALID_ARGUMENT, "null pointer");
  if (!aligned16(x) || (reinterpret_cast<uintptr_t>(q) & 3u)) return fail(LLMMM_ERR_INVALID_ARGUMENT, "x must be 16-byte and q 4-byte aligned");
  if ((long)M * N >= (1L << 31)) return fail(LLMMM_ERR_INVALID_ARGUMENT, "matrix has 2^31 or more elements");
  const int quant_m   = (kind == LLMMM_QUANT_1x128_T || kind == LLMMM_QUANT_1x128) ? 1 : 128;
  const int transpose = (kind == LLMMM_QUANT_1x128_T || kind == LLMMM_QUANT_128x128_T) ? 1 : 0;
  const hipError_t e  = llmmm::quant_fp8_launch(quant_m, transpose, x, q, scale, M, N, (hipStream_t)stream);
  if (e != hipSuccess) return fail(LLMMM_ERR_RUNTIME, "quantiser launch: %s", hipGetErrorString(e));
  return LLMMM_OK;
}

int llmmm_rmsnorm_quant_fp8(int in_dtype, const void* x, const float* weight, float eps, void* q, float* scale, int M, int K, void* stream)
{
  if (in_dtype != LLMMM_DTYPE_F16 && in_dtype != LLMMM_DTYPE_BF16 && in_dtype != LLMMM_DTYPE_F32) return fail(LLMMM_ERR_UNSUPPORTED_TYPE, "T is not supported.");
  if (M <= 0 || K <= 0) return fail(LLMMM_ERR_INVALID_ARGUMENT, "M and K must be positive (got %d, %d)", M, K);
  if (K % 128) return fail(LLMMM_ERR_NOT_ALIGNED, "M or N or K are not aligned.");
  if (!x || !weight || !q || !scale) return fail(LLMMM_ERR_INVALID_ARGUMENT, "null pointer");
  if (!(eps >= 0.f)) return fail(LLMMM_ERR_INVALID_ARGUMENT, "eps must be non-negative");
  if (!aligned16(x) || !aligned16(weight) || !aligned16(q)) return fail(LLMMM_ERR_INVALID_ARGUMENT, "pointers must be 16-byte aligned");
  if ((long)M * K >= (1L << 31)) return fail(LLMMM_ERR_INVALID_ARGUMENT, "matrix has 2^31 or more elements");
  const hipError_t e = llmmm::rmsnorm_quant_launch(in_dtype, x, weight, eps, q, scale, M, K, (hipStream_t)stream);
  if (e != hipSuccess) return fail(LLMMM_ERR_RUNTIME, "rmsnorm + quantiser launch: %s", hipGetErrorString(e));
  return LLMMM_OK;
}

int llmmm_probe_mfma(int kind, const void* operands, float* sink, int workgroups, int iters, void* stream)
{
  if (kind < 0 || kind > LLMMM_PROBE_FP8) return fail(LLMMM_ERR_UNSUPPORTED_TYPE, "T is not supported.");
  if (!operands || !sink) return fail(LLMMM_ERR_INVALID_ARGUMENT, "null pointer");
  if (!aligned16(operands) || (reinterpret_cast<uintptr_t>(operands) & 31u)) return fail(LLMMM_ERR_INVALID_ARGUMENT, "operands must be 32-byte aligned");
  if (workgroups <= 0 || workgroups > 65536 || iters <= 0) return fail(LLMMM_ERR_INVALID_ARGUMENT, "workgroups must be 1..65536 and iters positive");
  const hipError_t e = llmmm::probe_mfma_launch(kind, operands, sink, workgroups, iters, (hipStream_t)stream);
  if (e != hipSuccess) return fail(LLMMM_ERR_RUNTIME, "probe launch: %s", hipGetErrorString(e));
  return LLMMM_OK;
}

double llmmm_probe_mfma_flops(int kind, int workgroups, int iters)
{
  if (kind < 0 || kind > LLMMM_PROBE_FP8 || workgroups <= 0 || iters <= 0) return 0.0;
  return llmmm::probe_mfma_flops(kind, workgroups, iters);
}

int llmmm_probe_hbm_read(const void* src, size_t bytes, float* sink, int workgroups, void* stream)
{
  if (!src || !sink) return fail(LLMMM_ERR_INVALID_ARGUMENT, "null pointer");
  if (!aligned16(src) || bytes == 0 || bytes % 16) return fail(LLMMM_ERR_INVALID_ARGUMENT, "src must be 16-byte aligned and bytes a positive multiple of 16");
  if (workgroups <= 0 || workgroups > 65536) return fail(LLMMM_ERR_INVALID_ARGUMENT, "workgroups must be 1..65536");
  const hipError_t e = llmmm::probe_stream_read_launch(src, bytes, sink, workgroups, (hipStream_t)stream);
  if (e != hipSuccess) return fail(LLMMM_ERR_RUNTIME, "probe launch: %s", hipGetErrorString(e));
  return LLMMM_OK;
}

// Workspace of the entry points whose epilogue runs either inside an unsplit tile kernel (no planes) or in a second
// kernel behind fp32 planes: the same decision as resolve_plane_cfg takes for a call without cfg.  A single tile row of
// fewer than 128 rows (64 < M < 128 in 128 x 128 tiles) has no epilogue of its own and always goes through one plane.
static size_t plane_route_workspace(int M, int N, int K, bool wide_ok)
{
  if (M <= 0 || N <= 0 || K <= 0 || N % 128 || K % 128) return 0;
  llmmm_gemm_cfg cfg;
  if (choose_fp8(M, N, K, &cfg) != LLMMM_OK) return 0;
  if (wide_ok) prefer_wide_tile(&cfg, M, N), prefer_strip(&cfg, M, N, K);
  if (cfg.tile == LLMMM_TILE_STRIP) return strip_fallback_plane_bytes(M, N, K);  // strips need none (epilogue inside the kernel); a call with generated activations leaves them
  int split = cfg.split_k < 1 ? 1 : cfg.split_k;
  if (split > max_split_for(K)) split = max_split_for(K);
  int bm = 0, bn = 0;
  if (cfg.tile != LLMMM_TILE_SKINNY && tile_dims(cfg.tile, bm, bn) && M % bm == 0 && split == 1) return 0;  // epilogue inside the tile kernel
  return (size_t)split * M * N * sizeof(float);
}

int llmmm_probe_strip_exchange_timeouts(unsigned* count)
{
  if (!count) return fail(LLMMM_ERR_INVALID_ARGUMENT, "null pointer");
  const hipError_t e = llmmm::strip_exchange_timeouts(count);
  if (e != hipSuccess) return fail(LLMMM_ERR_RUNTIME, "reading the exchange's time-out counter: %s", hipGetErrorString(e));
  return LLMMM_OK;
}

size_t llmmm_probe_phases_bytes(int M, int N)
{
  if (M <= 0 || N <= 0 || M % 256 || N % 256) return 0;
  return (size_t)(M / 256) * (N / 256) * 8 * llmmm::PHASE_RECORD * sizeof(unsigned long long);
}

int llmmm_probe_fp8_gemm_phases(const void* A, const float* As, const void* Bt, const float* Bs, void* C, float* Cs, int M, int N, int K, void* stamps,
                                size_t stamps_bytes, void* stream)
{
  if (M <= 0 || N <= 0 || K <= 0) return fail(LLMMM_ERR_INVALID_ARGUMENT, "M, N and K must be positive (got %d, %d, %d)", M, N, K);
  if (M % 256 || N % 256 || K % 128) return fail(LLMMM_ERR_NOT_ALIGNED, "M or N or K are not aligned.");
  if (!A || !As || !Bt || !Bs || !C || !Cs || !stamps) return fail(LLMMM_ERR_INVALID_ARGUMENT, "null pointer");
  if (!aligned16(A) || !aligned16(Bt) || !aligned16(C) || !aligned16(stamps)) return fail(LLMMM_ERR_INVALID_ARGUMENT, "pointers must be 16-byte aligned");
  if (stamps_bytes < llmmm_probe_phases_bytes(M, N)) return fail(LLMMM_ERR_WORKSPACE, "stamps holds %zu bytes, %zu needed", stamps_bytes, llmmm_probe_phases_bytes(M, N));
  const hipError_t e = llmmm::fp8_gemm_phases_launch(A, As, Bt, Bs, C, Cs, M, N, K, (unsigned long long*)stamps, (hipStream_t)stream);
  if (e != hipSuccess) return fail(LLMMM_ERR_RUNTIME, "probe launch: %s", hipGetErrorString(e));
  return LLMMM_OK;
}

int llmmm_probe_fp16_gemm_phases(int dtype, const void* A, const void* B, void* C, int M, int N, int K, void* stamps, size_t stamps_bytes, void* stream)
{
  if (dtype != LLMMM_DTYPE_F16 && dtype != LLMMM_DTYPE_BF16) return fail(LLMMM_ERR_UNSUPPORTED_TYPE, "T is not supported.");
  if (M <= 0 || N <= 0 || K <= 0) return fail(LLMMM_ERR_INVALID_ARGUMENT, "M, N and K must be positive (got %d, %d, %d)", M, N, K);
  if (M % 256 || N % 256 || K % 32) return fail(LLMMM_ERR_NOT_ALIGNED, "M or N or K are not aligned.");
  if (!A || !B || !C || !stamps) return fail(LLMMM_ERR_INVALID_ARGUMENT, "null pointer");
  if (!aligned16(A) || !aligned16(B) || !aligned16(C) || !aligned16(stamps)) return fail(LLMMM_ERR_INVALID_ARGUMENT, "pointers must be 16-byte aligned");
  if (stamps_bytes < llmmm_probe_phases_bytes(M, N)) return fail(LLMMM_ERR_WORKSPACE, "stamps holds %zu bytes, %zu needed", stamps_bytes, llmmm_probe_phases_bytes(M, N));
  const hipError_t e = llmmm::fp16_gemm_phases_launch(dtype, A, B, C, M, N, K, (unsigned long long*)stamps, (hipStream_t)stream);
  if (e != hipSuccess) return fail(LLMMM_ERR_RUNTIME, "probe launch: %s", hipGetErrorString(e));
  return LLMMM_OK;
}

size_t llmmm_fp8_gemm_add_rmsnorm_quant_workspace(int M, int N, int K) { return plane_route_workspace(M, N, K, true); }

// Kernel and split for the entry points whose epilogue lives in a second kernel behind fp32 planes, chosen and
// validated as llmmm_fp8_gemm_ex does.  split == 0 on return: a tile kernel without split, which `allow_direct`
// callers run with the epilogue inside the kernel (no planes, no workspace); otherwise split >= 1 planes are needed
// and the workspace has been checked to hold them.
struct PlaneCfg {
  int  tile = 0, split = 0, b_layout = 0;
  bool  skinny = false;
  bool  strip  = false;  // the weight-streaming kernel in column strips: one launch, its fp32 result is the one "plane"
  APrep prep;
};
static int resolve_plane_cfg(const void*& A, const float*& As, const void* Bt, const float* Bs, int M, int N, int K, void*& workspace,
                             size_t& workspace_bytes, const llmmm_gemm_cfg* user, bool allow_direct, PlaneCfg* out, void* stream, bool wide_ok = true)
{
  llmmm_gemm_cfg cfg;
  const int      rc = choose_fp8(M, N, K, &cfg);
  if (rc) return rc;
  if (wide_ok) prefer_wide_tile(&cfg, M, N);
  // (wide_ok also stands for "no 1x128-grouped epilogue behind the GEMM": the callers that may take column strips.  Not with
  // activations the kernel has to make itself, nor against an explicit split.)
  if (wide_ok && !(user && (user->a_layout != LLMMM_FP8_A_QUANTISED || user->split_k > 0 || user->tile != LLMMM_TILE_AUTO))) prefer_strip(&cfg, M, N, K);
  const bool a_made = user && user->a_layout != LLMMM_FP8_A_QUANTISED;
  if (!A || (!As && !a_made) || !Bt || !Bs) return fail(LLMMM_ERR_INVALID_ARGUMENT, "null pointer");
  const bool a_host = user && user->a_layout == LLMMM_FP8_A_PLANES_RMSNORM;  // a host structure, checked by prepare_a
  if ((!a_host && !aligned16(A)) || !aligned16(Bt)) return fail(LLMMM_ERR_INVALID_ARGUMENT, "pointers must be 16-byte aligned");
  if ((long)M * K >= (1L << 31) || (long)N * K >= (1L << 31) || (long)M * N >= (1L << 31))
    return fail(LLMMM_ERR_INVALID_ARGUMENT, "matrix has 2^31 or more elements");
  if (user) {
    // (a named weight-streaming kernel where the library would have taken tiles: the split is that kernel's own heuristic)
    if (user->tile == LLMMM_TILE_SKINNY && cfg.tile != LLMMM_TILE_SKINNY && M <= SKINNY_MAX_M) cfg.split_k = heuristic_split(M, N, K);
    if (user->tile != LLMMM_TILE_AUTO) cfg.tile = user->tile;
    if (user->split_k > 0) cfg.split_k = user->split_k;
    if (user->b_layout != LLMMM_FP8_B_ROWS && user->b_layout != LLMMM_FP8_B_PRESHUFFLED)
      return fail(LLMMM_ERR_INVALID_ARGUMENT, "unknown B layout %d", user->b_layout);
    cfg.b_layout = user->b_layout;
  }
  int bm = 0, bn = 0;
  const bool skinny = cfg.tile == LLMMM_TILE_SKINNY;
  if (cfg.tile == LLMMM_TILE_STRIP) {
    if (!wide_ok) return fail(LLMMM_ERR_INVALID_ARGUMENT, "the column-strip kernel cannot hold whole heads");
    if (a_made || (user && user->split_k > 1)) return fail(LLMMM_ERR_INVALID_ARGUMENT, "the column-strip kernel takes quantised activations and does not split K over workgroups");
    if (!strip_fits(M, N, K)) return fail(LLMMM_ERR_INVALID_ARGUMENT, "the column-strip kernel handles M <= %d and K >= 1024", llmmm::STRIP_MAX_M);
    out->prep = APrep();
    out->tile = cfg.tile, out->b_layout = cfg.b_layout, out->skinny = false, out->strip = true;
    if (allow_direct) {
      out->split = 0;  // the caller's epilogue is the strip kernel's own (residual add): no planes
      return LLMMM_OK;
    }
    const size_t plane1 = (size_t)M * N * sizeof(float);
    if (!workspace || workspace_bytes < plane1) return fail(LLMMM_ERR_WORKSPACE, "workspace holds %zu bytes, one fp32 plane needs %zu", workspace ? workspace_bytes : (size_t)0, plane1);
    if (!aligned16(workspace)) return fail(LLMMM_ERR_INVALID_ARGUMENT, "workspace must be 16-byte aligned");
    out->split = 1;
    return LLMMM_OK;
  }
  if (skinny) {
    if (M > SKINNY_MAX_M) return fail(LLMMM_ERR_INVALID_ARGUMENT, "the weight-streaming kernel handles M <= %d", SKINNY_MAX_M);
  }
  else {
    if (!tile_dims(cfg.tile, bm, bn) || cfg.tile == LLMMM_TILE_64x128) return fail(LLMMM_ERR_INVALID_ARGUMENT, "unknown tile id %d", cfg.tile);
    if ((M % bm && !(cfg.tile == LLMMM_TILE_128x128 && M < 128)) || N % bn) return fail(LLMMM_ERR_NOT_ALIGNED, "M or N or K are not aligned.");
    if (user && user->tile != LLMMM_TILE_AUTO && user->split_k <= 0) cfg.split_k = heuristic_tile_split(cfg.tile, M < bm ? bm : M, N, K);
  }
  // the A operand given as the fp32 gate_up result: generated by the kernel, or quantised into the front of the workspace now
  const int rca = prepare_a(user, cfg.tile, A, As, M, K, workspace, workspace_bytes, stream, &out->prep);
  if (rca) return rca;
  int split = cfg.split_k < 1 ? 1 : cfg.split_k;
  if (split > max_split_for(K)) split = max_split_for(K);
  const size_t plane    = (size_t)M * N * sizeof(float);
  const bool   explicit_split = user && user->split_k > 0;
  const int    min_split = out->prep.agen ? agen_min_split(K) : 1;
  if (split < min_split) {
    if (explicit_split) return fail(LLMMM_ERR_INVALID_ARGUMENT, "generated activations need split-K >= %d for K = %d", min_split, K);
    split = min_split;
  }
  out->tile = cfg.tile, out->b_layout = cfg.b_layout, out->skinny = skinny;
  // (a row tail -- M < 128 in 128 x 128 tiles -- has no direct epilogues: always through planes)
  if (allow_direct && !skinny && M % bm == 0 && (split == 1 || (!explicit_split && (!workspace || workspace_bytes < 2 * plane)))) {
    out->split = 0;  // also when a split the library chose itself finds no room for two planes
    return LLMMM_OK;
  }
  if (!workspace || workspace_bytes < plane) return fail(LLMMM_ERR_WORKSPACE, "workspace holds %zu bytes, one fp32 plane needs %zu", workspace ? workspace_bytes : (size_t)0, plane);
  if (!aligned16(workspace)) return fail(LLMMM_ERR_INVALID_ARGUMENT, "workspace must be 16-byte aligned");
  if ((size_t)split * plane > workspace_bytes) {
    if (explicit_split) return fail(LLMMM_ERR_WORKSPACE, "workspace holds %zu bytes, split-K %d needs %zu", workspace_bytes, split, (size_t)split * plane);
    split = (int)(workspace_bytes / plane);  // a split the library chose itself shrinks to the workspace (>= 1: checked above)
    if (split < min_split) return fail(LLMMM_ERR_WORKSPACE, "workspace holds %zu bytes, generated activations need split-K %d: %zu", workspace_bytes, min_split, (size_t)min_split * plane);
  }
  out->split = split;
  return LLMMM_OK;
}

static int launch_into_planes(const PlaneCfg& pc, const void* A, const float* As, const void* Bt, const float* Bs, int M, int N, int K,
                              void* workspace, void* stream)
{
  float*     planes = (float*)workspace;
  hipError_t e;
  if (pc.strip)
    e = llmmm::fp8_strip_launch(LLMMM_OUT_F32, pc.b_layout, A, As, Bt, Bs, planes, M, N, K, (hipStream_t)stream);
  else if (pc.skinny && pc.prep.agen == 2)
    e = llmmm::fp8_skinny_rmsnorm_a_launch(pc.prep.hidden_dtype, pc.b_layout, pc.prep.ag, Bt, Bs, nullptr, M, N, K, pc.split, planes, (hipStream_t)stream);
  else if (pc.skinny && pc.prep.agen == 1)
    e = llmmm::fp8_skinny_swiglu_a_launch(LLMMM_OUT_F32, pc.b_layout, (const float*)A, Bt, Bs, nullptr, nullptr, M, N, K, pc.split, planes, (hipStream_t)stream);
  else if (pc.skinny)
    e = llmmm::fp8_skinny_launch(LLMMM_OUT_F32, pc.b_layout, A, As, Bt, Bs, nullptr, nullptr, M, N, K, pc.split, planes, (hipStream_t)stream);
  else
    e = llmmm::fp8_gemm_launch(LLMMM_OUT_F32, pc.tile, pc.b_layout, A, As, Bt, Bs, nullptr, nullptr, M, N, K, pc.split, planes, (hipStream_t)stream);
  if (e != hipSuccess) return fail(LLMMM_ERR_RUNTIME, "fp8 gemm launch: %s", hipGetErrorString(e));
  return LLMMM_OK;
}

size_t llmmm_fp8_gemm_planes_bytes(int M, int N, int K)
{
  if (M <= 0 || N <= 0 || K <= 0 || N % 128 || K % 128) return 0;
  llmmm_gemm_cfg cfg;
  if (choose_fp8(M, N, K, &cfg) != LLMMM_OK) return 0;
  const size_t own = (size_t)(cfg.split_k < 1 ? 1 : cfg.split_k) * M * N * sizeof(float);
  prefer_strip(&cfg, M, N, K);  // (strips write one plane; a call with generated activations leaves them for the split-K form)
  if (cfg.tile == LLMMM_TILE_STRIP) {
    const size_t fb = strip_fallback_plane_bytes(M, N, K);
    return fb > own ? fb : own;
  }
  return own;
}

int llmmm_fp8_gemm_planes(const void* A, const float* As, const void* Bt, const float* Bs, int M, int N, int K, float* planes, size_t planes_bytes,
                          int* splits, void* workspace, size_t workspace_bytes, const llmmm_gemm_cfg* user, void* stream)
{
  if (!splits || !planes) return fail(LLMMM_ERR_INVALID_ARGUMENT, "null pointer");
  llmmm_gemm_cfg probe;
  int            rc = choose_fp8(M, N, K, &probe);
  if (rc) return rc;
  llmmm_gemm_cfg inner;
  inner.tile = LLMMM_TILE_AUTO, inner.split_k = 0, inner.b_layout = LLMMM_FP8_B_ROWS, inner.a_layout = LLMMM_FP8_A_QUANTISED;
  if (user) inner = *user;
  if (inner.a_layout != LLMMM_FP8_A_QUANTISED) {
    // an operand the library has to quantise first goes to `workspace` (the planes have a buffer of their own); one the
    // kernel generates is resolved a second time inside resolve_plane_cfg, which launches nothing for it
    if (!A) return fail(LLMMM_ERR_INVALID_ARGUMENT, "null pointer");
    const int tile = inner.tile != LLMMM_TILE_AUTO ? inner.tile : probe.tile;
    APrep     prep;
    rc = prepare_a(&inner, tile, A, As, M, K, workspace, workspace_bytes, stream, &prep);
    if (rc) return rc;
    if (prep.agen == 0) inner.a_layout = LLMMM_FP8_A_QUANTISED;
  }
  PlaneCfg pc;
  void*    pw = planes;
  size_t   pb = planes_bytes;
  rc = resolve_plane_cfg(A, As, Bt, Bs, M, N, K, pw, pb, &inner, false, &pc, stream);
  if (rc) return rc;
  rc = launch_into_planes(pc, A, As, Bt, Bs, M, N, K, pw, stream);
  if (rc) return rc;
  *splits = pc.split;
  return LLMMM_OK;
}

int llmmm_fp8_gemm_add_rmsnorm_quant(const void* A, const float* As, const void* Bt, const float* Bs, int hidden_dtype, const void* residual,
                                     void* hidden_out, const float* norm_weight, float eps, void* q, float* q_scale, int M, int N, int K,
                                     void* workspace, size_t workspace_bytes, const llmmm_gemm_cfg* user, void* stream)
{
  if (hidden_dtype != LLMMM_DTYPE_F16 && hidden_dtype != LLMMM_DTYPE_BF16 && hidden_dtype != LLMMM_DTYPE_F32)
    return fail(LLMMM_ERR_UNSUPPORTED_TYPE, "T is not supported.");
  llmmm_gemm_cfg probe;
  const int      rc0 = choose_fp8(M, N, K, &probe);  // shape checks first, with the reference's texts
  if (rc0) return rc0;
  if (N > 10240) return fail(LLMMM_ERR_INVALID_ARGUMENT, "the fused norm handles rows of at most 10240 columns (got %d)", N);
  if (!residual || !hidden_out || !norm_weight || !q || !q_scale) return fail(LLMMM_ERR_INVALID_ARGUMENT, "null pointer");
  if (!(eps >= 0.f)) return fail(LLMMM_ERR_INVALID_ARGUMENT, "eps must be non-negative");
  if (!aligned16(residual) || !aligned16(hidden_out) || !aligned16(norm_weight) || !aligned16(q))
    return fail(LLMMM_ERR_INVALID_ARGUMENT, "pointers must be 16-byte aligned");
  PlaneCfg pc;
  int      rc = resolve_plane_cfg(A, As, Bt, Bs, M, N, K, workspace, workspace_bytes, user, true, &pc, stream);
  if (rc) return rc;
  if (pc.split == 0) {
    // a tile kernel without split, or column strips: the residual is added in its epilogue, the norm + quantiser kernel follows on the
    // stored hidden state (the same two operations on the same values as behind planes, without the fp32 round trip)
    hipError_t e = pc.strip ? llmmm::fp8_strip_add_residual_launch(hidden_dtype, pc.b_layout, A, As, Bt, Bs, residual, hidden_out, M, N, K, (hipStream_t)stream)
                            : llmmm::fp8_gemm_add_residual_launch(hidden_dtype, pc.tile, pc.b_layout, A, As, Bt, Bs, residual, hidden_out, M, N, K, (hipStream_t)stream);
    if (e == hipSuccess) e = llmmm::rmsnorm_quant_launch(hidden_dtype, hidden_out, norm_weight, eps, q, q_scale, M, N, (hipStream_t)stream);
    if (e != hipSuccess) return fail(LLMMM_ERR_RUNTIME, "fp8 gemm + add, rmsnorm + quantiser launch: %s", hipGetErrorString(e));
    return LLMMM_OK;
  }
  rc = launch_into_planes(pc, A, As, Bt, Bs, M, N, K, workspace, stream);
  if (rc) return rc;
  const hipError_t e = llmmm::planes_add_rmsnorm_quant_launch(hidden_dtype, (const float*)workspace, pc.split, residual, hidden_out, norm_weight, eps, q,
                                                              q_scale, M, N, (hipStream_t)stream);
  if (e != hipSuccess) return fail(LLMMM_ERR_RUNTIME, "add + rmsnorm + quantiser launch: %s", hipGetErrorString(e));
  return LLMMM_OK;
}

size_t llmmm_fp8_gemm_qkv_rope_workspace(int M, int N, int K) { return plane_route_workspace(M, N, K, false); }

int llmmm_fp8_gemm_qkv_rope(int out_kind, const void* A, const float* As, const void* Bt, const float* Bs, void* out, float* out_scale,
                            const float* q_norm_weight, const float* k_norm_weight, float eps, const float* cos_table, const float* sin_table,
                            int table_rows, const int* positions, int n_q_heads, int n_kv_heads, int M, int N, int K, void* workspace,
                            size_t workspace_bytes, const llmmm_gemm_cfg* user, void* stream)
{
  if (out_kind != LLMMM_OUT_BF16 && out_kind != LLMMM_OUT_FP8Q) return fail(LLMMM_ERR_INVALID_ARGUMENT, "output kind %d: bf16 or fp8 (1x128) only", out_kind);
  llmmm_gemm_cfg probe;
  const int      rc0 = choose_fp8(M, N, K, &probe);
  if (rc0) return rc0;
  if (n_q_heads < 1 || n_kv_heads < 1 || (long)(n_q_heads + 2L * n_kv_heads) * 128 != N)
    return fail(LLMMM_ERR_INVALID_ARGUMENT, "N = %d is not (n_q_heads + 2 n_kv_heads) * 128 with %d query and %d key/value heads", N, n_q_heads, n_kv_heads);
  if (!out || !cos_table || !sin_table || !positions) return fail(LLMMM_ERR_INVALID_ARGUMENT, "null pointer");
  if (out_kind == LLMMM_OUT_FP8Q && !out_scale) return fail(LLMMM_ERR_INVALID_ARGUMENT, "out_scale is required for fp8 output");
  if (table_rows < 1) return fail(LLMMM_ERR_INVALID_ARGUMENT, "the cos / sin tables need at least one row");
  if (!(eps >= 0.f)) return fail(LLMMM_ERR_INVALID_ARGUMENT, "eps must be non-negative");
  if (!aligned16(out) || !aligned16(cos_table) || !aligned16(sin_table) || (q_norm_weight && !aligned16(q_norm_weight)) ||
      (k_norm_weight && !aligned16(k_norm_weight)) || (reinterpret_cast<uintptr_t>(positions) & 3u))
    return fail(LLMMM_ERR_INVALID_ARGUMENT, "pointers must be 16-byte aligned (positions: 4-byte)");
  PlaneCfg pc;
  int      rc = resolve_plane_cfg(A, As, Bt, Bs, M, N, K, workspace, workspace_bytes, user, true, &pc, stream, false);
  if (rc) return rc;
  if (pc.tile == LLMMM_TILE_128x160) return fail(LLMMM_ERR_INVALID_ARGUMENT, "the 128 x 160 tile cannot hold whole heads");
  if (pc.split == 0) {  // a tile kernel without split: norm and rope run on the accumulators, no planes
    llmmm::Fp8HeadOp op;
    op.qw = q_norm_weight, op.kw = k_norm_weight, op.cos_t = cos_table, op.sin_t = sin_table, op.pos = positions;
    op.eps = eps, op.table_rows = table_rows, op.n_q = n_q_heads, op.n_kv = n_kv_heads;
    const hipError_t e = llmmm::fp8_gemm_qk_rope_launch(out_kind, pc.tile, pc.b_layout, A, As, Bt, Bs, out, out_scale, M, N, K, op, (hipStream_t)stream);
    if (e != hipSuccess) return fail(LLMMM_ERR_RUNTIME, "fp8 gemm + qk-norm + rope launch: %s", hipGetErrorString(e));
    return LLMMM_OK;
  }
  rc = launch_into_planes(pc, A, As, Bt, Bs, M, N, K, workspace, stream);
  if (rc) return rc;
  const hipError_t e = llmmm::fp8_planes_qk_norm_rope_launch(out_kind, (const float*)workspace, pc.split, out, out_scale, q_norm_weight, k_norm_weight, eps,
                                                             cos_table, sin_table, table_rows, positions, n_q_heads, n_kv_heads, M, (hipStream_t)stream);
  if (e != hipSuccess) return fail(LLMMM_ERR_RUNTIME, "qk-norm + rope launch: %s", hipGetErrorString(e));
  return LLMMM_OK;
}

static int preshuffle(int inverse, const void* src, void* dst, int N, int K, void* stream)
{
  if (N <= 0 || K <= 0) return fail(LLMMM_ERR_INVALID_ARGUMENT, "N and K must be positive (got %d, %d)", N, K);
  if (K % 128) return fail(LLMMM_ERR_NOT_ALIGNED, "K must be greater than 0 and divisible by 128.");
  if (N % 16) return fail(LLMMM_ERR_NOT_ALIGNED, "N must be divisible by 16.");
  if (!src || !dst) return fail(LLMMM_ERR_INVALID_ARGUMENT, "null pointer");
  if (!aligned16(src) || !aligned16(dst)) return fail(LLMMM_ERR_INVALID_ARGUMENT, "pointers must be 16-byte aligned");
  if ((long)N * K >= (1L << 31)) return fail(LLMMM_ERR_INVALID_ARGUMENT, "matrix has 2^31 or more elements");
  const char *a = (const char*)src, *b = (const char*)dst;
  if (a < b + (size_t)N * K && b < a + (size_t)N * K) return fail(LLMMM_ERR_INVALID_ARGUMENT, "source and destination overlap");
  const hipError_t e = llmmm::fp8_preshuffle_launch(inverse, src, dst, N, K, (hipStream_t)stream);
  if (e != hipSuccess) return fail(LLMMM_ERR_RUNTIME, "pre-shuffle launch: %s", hipGetErrorString(e));
  return LLMMM_OK;
}

int llmmm_fp8_preshuffle_b(const void* Bt, void* Bp, int N, int K, void* stream) { return preshuffle(0, Bt, Bp, N, K, stream); }
int llmmm_fp8_unshuffle_b(const void* Bp, void* Bt, int N, int K, void* stream) { return preshuffle(1, Bp, Bt, N, K, stream); }

int llmmm_transpose(int elem_size, const void* src, void* dst, int M, int N, void* stream)
{
  if (elem_size != 1 && elem_size != 4) return fail(LLMMM_ERR_UNSUPPORTED_TYPE, "T is not supported.");
  if (M <= 0 || N <= 0) return fail(LLMMM_ERR_INVALID_ARGUMENT, "M and N must be positive (got %d, %d)", M, N);
  if (M % 128 || N % 128) return fail(LLMMM_ERR_NOT_ALIGNED, "M or N can't be divided 128.");
  if (!src || !dst) return fail(LLMMM_ERR_INVALID_ARGUMENT, "null pointer");
  if ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 3u) return fail(LLMMM_ERR_INVALID_ARGUMENT, "pointers must be 4-byte aligned");
  if ((long)M * N >= (1L << 31)) return fail(LLMMM_ERR_INVALID_ARGUMENT, "matrix has 2^31 or more elements");
  const size_t bytes = (size_t)M * N * elem_size;
  const char * a = (const char*)src, *b = (const char*)dst;
  if (a < b + bytes && b < a + bytes) return fail(LLMMM_ERR_INVALID_ARGUMENT, "source and destination overlap");
  const hipError_t e = llmmm::transpose_launch(elem_size, src, dst, M, N, (hipStream_t)stream);
  if (e != hipSuccess) return fail(LLMMM_ERR_RUNTIME, "transpose launch: %s", hipGetErrorString(e));
  return LLMMM_OK;
}

}  // extern "C"
