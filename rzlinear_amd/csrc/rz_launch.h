// Host-side launch of the contraction kernels; one translation unit per element type.
#pragma once

#include <atomic>

#include "../../include/rzlinear.h"
#include "rz_common.h"

namespace rz {

// Every planning function takes the caller's tuning overrides (all zero = automatic); nothing
// here reads the environment or keeps state, so a workspace query and the launch that follows
// it decide alike.
static inline rz_tuning tuning_or_default(const rz_tuning* t) {
  rz_tuning d = {};
  return t != nullptr ? *t : d;
}
static inline bool tuning_valid(const rz_tuning& t) {
  return (t.tile == 0 || t.tile == 32 || t.tile == 64 || t.tile == 128 || t.tile == 256) && (t.stages == 0 || t.stages == 1) &&
         (t.lds_image == 0 || t.lds_image == -1) && (t.window >= -1 && t.window <= 1) &&
         (t.split >= -1 && t.split <= 16) && (t.clamp == 0 || t.clamp == -1) &&
         (t.fold >= -1 && t.fold <= 2) && (t.fold_tiles == 0 || t.fold_tiles == -1) && (t.finish == 0 || t.finish == -1) && t.poll_limit >= 0;
}

// Kernels that use more than the default 64 KB of LDS need their limit raised once per kernel
// and device; `done` is that kernel's bit set of devices already served.
static inline hipError_t raise_lds_limit(const void* kernel, std::atomic<uint64_t>& done) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const uint64_t bit = 1ull << (dev & 63);
  if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
  if (e == hipSuccess) done.fetch_or(bit, std::memory_order_release);
  return e;
}

static constexpr int kComputeUnits = 256;
// Number of workgroups of the small tile that fills the compute units a few times over.
static constexpr int kTargetWorkgroups = 1024;

// Contracted elements per kernel step that every slice of a cut contraction must be a multiple
// of: 128 bytes, and 256 for the 16-bit 128 tile, whose eight-wavefront form takes 256-byte steps
// (a slice that began in the middle of such a step would start between two hashed tiles).
static inline int slice_unit(int tile, int elem_bytes, bool weight_grad = false) {
  if (elem_bytes == 4 && tile <= 64 && !weight_grad) return 64;   // (fp32 forward / input-grad, 64 and 32 x 64 tiles: 256-byte steps as well)
  return ((tile == 128 && elem_bytes == 2) ? 256 : 128) / elem_bytes;
}

// Tile codes: 64, 128, 256 are square C tiles; 32 stands for the 32 x 64 tile of the fp32 forward /
// input-grad kernels, for batches whose rows would leave the last 64-row tile at most half full
// (M = 32, 96, 160: that half would be padding).
static inline int tile_cols(int t) { return t == 32 ? 64 : t; }
static inline long long tile_count(int I, int J, int t) {
  return (long long)((I + t - 1) / t) * ((J + tile_cols(t) - 1) / tile_cols(t));
}

// Rate of `wgs` equal workgroups on the chip relative to a full one, when a compute unit runs at
// `lo` with one workgroup resident and at `hi` with `slots` (linear in between).  The hardware
// deals workgroups out evenly, so the busiest compute unit holds c = ceil(wgs / CUs) of them; up to
// `slots` they run side by side and finish together after c * w / e(c), while the chip's work is
// wgs * w: the rate is (wgs / CUs) * e(c) / c.  (320 workgroups on 256 compute units leave 64 of
// them with two: the launch takes as long as 512 would.)  Beyond `slots` per compute unit the
// workgroups go in rounds of CUs * slots and a last, partly filled round costs a full one.
static inline double occupancy_rate(double wgs, int slots, double lo, double hi, int knee = 0) {
  const double per_cu = wgs / kComputeUnits;
  if (per_cu <= 1.0) return lo * per_cu;
  // (`knee`: the number of resident workgroups from which the compute unit runs at `hi`, if fewer than `slots`)
  const double full = knee > 1 ? knee : slots;
  auto e = [&](double c) { return full > 1 ? lo + (hi - lo) * (c < full ? (c - 1.0) / (full - 1.0) : 1.0) : hi; };
  if (per_cu <= slots) {
    const double c = (double)((long long)(per_cu + 0.999999));
    return per_cu * e(c) / c;
  }
  const double cap = (double)kComputeUnits * slots;
  const double rounds = (double)((long long)((wgs + cap - 1) / cap));
  return hi * wgs / (rounds * cap);
}

// Relative throughput of a tile shape at a given number of workgroups, from measurements on
// MI355X (256 tile at one workgroup per compute unit = 1).  16-bit types: the 128 tile reaches
// 0.51 with one workgroup per compute unit and 0.75 with two or more, the 64 tile 0.16 and 0.33
// (four or more).  fp32 is bound by the slower fp32 MFMA rate, so the small tiles lose far less:
// 0.86 / 0.90 and 0.45 / 0.80.  How the number of workgroups enters: occupancy_rate above.
static inline double tile_score_full(int I, int J, int t, int elem_bytes) {
  const double wgs = (double)tile_count(I, J, t);
  const bool f32 = elem_bytes == 4;
  const int slots = (t == 256) ? 1 : (t == 128 ? 2 : 4);          // resident workgroups per CU
  const double lo = (t == 256) ? 1.0 : (t == 128 ? (f32 ? 0.86 : 0.51) : (f32 ? 0.45 : 0.16));  // one workgroup per CU
  const double hi = (t == 256) ? 1.0 : (t == 128 ? (f32 ? 0.90 : 0.75) : (f32 ? 0.80 : 0.33));  // `slots` per CU
  return occupancy_rate(wgs, slots, lo, hi);
}
// ... times the share of a tile grid's MFMA work that is not padding
static inline double tile_score(int I, int J, int t, int elem_bytes) {
  const double wgs = (double)tile_count(I, J, t);
  return tile_score_full(I, J, t, elem_bytes) * ((double)I * (double)J) / (wgs * t * t);
}

// Relative throughput of `wgs` workgroups of tile t (see tile_score_full, which this restates for
// a workgroup count that includes the slices of a cut contraction).
// (store_op: the figures of forward / input-grad as they are now — fp32 staged directly, 16-bit fitted
//  again with them; weight-grad keeps its own)
static inline double tile_rate(double wgs, int t, int elem_bytes, double lo64_f32 = 0.60, bool store_op = false) {
  const bool f32 = elem_bytes == 4;
  if (f32 && store_op) {
    // fp32 forward / input-grad, staged directly: every tile runs the MFMA pipe at the 256 tile's rate
    // once its loop is under way, at one workgroup per compute unit already (eight wavefronts); what a
    // smaller tile costs is the longer fill and drain per workgroup, which plan_split prices per slice.
    // (the 32 x 64 tile, four wavefronts, needs a second workgroup on the compute unit for that: 0.7 alone —
    //  M = 8, K = N = 8192: 256 workgroups 51 us, 512 45 us; M = 16, K = 4096, N = 11008: 172 workgroups 46 us,
    //  688 34 us)
    if (t == 32) return occupancy_rate(wgs, 4, 0.7, 1.0, 2);
    // (the 64 tile alone on a compute unit: 0.85 — M = 96, K = N = 4096 in two slices, 256 workgroups: 48 us)
    return occupancy_rate(wgs, t == 256 ? 1 : 2, t == 64 ? 0.85 : 1.0, 1.0);
  }
  // (32 x 64, four wavefronts: half a 64 workgroup's work in about its time, up to eight resident)
  if (t == 32) return occupancy_rate(wgs, 8, 0.40, 0.80);
  // (the 16-bit 128 tile in its eight-wavefront form — up to one and a half workgroups per compute unit, see
  //  kernel_form — has a compute unit to itself and runs at 0.80 there; beyond one per compute unit that
  //  means a second round: K = N = 10240, M = 128: 80 tiles whole 92 us, in two slices 55, three 43, four 62)
  if (!f32 && store_op && t == 128 && wgs <= kComputeUnits * 3 / 2) return occupancy_rate(wgs, 1, 0.80, 0.80);
  const int slots = (t == 256) ? 1 : (t == 128 ? 2 : 4);
  // (the 16-bit 64 tile: 0.29 with one workgroup per compute unit, 0.40 from two on — K = N = 10240, M = 128:
  //  320 workgroups 93 us, 640 68 us; M = 512, K = 4096, N = 1024 in four slices 16 us)
  const double lo = (t == 256) ? 1.0 : (t == 128 ? (f32 ? 0.86 : 0.51) : (f32 ? lo64_f32 : (store_op ? 0.29 : 0.24)));
  const double hi = (t == 256) ? 1.0 : (t == 128 ? (f32 ? 0.90 : 0.75) : (f32 ? 0.80 : (store_op ? 0.40 : 0.33)));
  return occupancy_rate(wgs, slots, lo, hi, (t == 64 && !f32) ? 2 : 0);
}

// C-tile edge for a contraction with an I x J result: the best-scoring of 256, 128, 64.
static inline int pick_tile(int I, int J, int elem_bytes, const rz_tuning& tuning) {
  if (tuning.tile) return (tuning.tile == 32 && elem_bytes != 4) ? 64 : tuning.tile;
  int best = 256;
  double best_score = tile_score(I, J, 256, elem_bytes);
  const int others[2] = {128, 64};
  for (int t : others) {
    const double sc = tile_score(I, J, t, elem_bytes);
    if (sc > best_score * 1.02) {   // prefer the larger tile on a near tie
      best = t;
      best_score = sc;
    }
  }
  return best;
}

// Weight-grad without any scatter in the contraction kernel: X^T.dY is stored tile by tile and a
// second kernel, whose workgroups own windows of hashed_weight, folds the tiles into dHW.
// (the fold kernel reads a kilobyte per wavefront from any 4-byte boundary: up to 1032 bytes before and after the tiles)
static constexpr size_t kFoldMarginBytes = 2048;

struct FoldPlan {
  int use;
  int small;             // few tiles: the kernel whose workgroups each look at every tile (no windows in LDS, no shares)
  int window, windows;   // floats per window (a multiple of 1024, at most 32768) and their number
  int shares;            // workgroups per window, each with an equal part of the window's tiles and an image of its own
  int tile_bytes;        // bytes of a stored element of X^T.dY: 4, or 2 (the layer's 16-bit dtype, see fold_tile_bytes)
  size_t tiles_bytes;    // the tile-by-tile X^T.dY: slices * tiles * BK*BN elements, with a margin before and after
  size_t partial_bytes;  // shares images of dHW (none with a single share: the fold kernel writes dHW)
  size_t offsets_bytes;  // where every tile starts in hashed_weight, one int32 per tile
};

// What the contraction kernel stores the tiles of X^T.dY as for the fold: floats — or, when the layer
// and its dHW are both 16-bit, the layer's dtype: the sum over M is complete (fp32) by then and the
// fold adds the stored values up in fp32 again, so this costs one more rounding per stored value (the
// reference rounds the running sum at every atomic add, RzLinearBackward.py:364-371) and halves the
// bytes written and read back, which is what the fold costs.
static inline int fold_tile_bytes(int elem_bytes, bool dhw_f32, const rz_tuning& t) {
  return (elem_bytes == 2 && !dhw_f32 && t.fold_tiles != -1) ? 2 : 4;
}

// The windows of hashed_weight that the fold kernel's workgroups own (a function of H alone: a layer
// plan lists every window's tiles).
static inline void fold_geometry(int H, int* window, int* windows) {
  const int kWindowMax = 32768, kThreads = 1024;
  int n = (int)(((long long)H + kWindowMax - 1) / kWindowMax);
  // from half a window per compute unit on, the windows are cut so that whole rounds of workgroups
  // come out, and every workgroup writes its window of dHW itself (no shares, no images)
  if (n * 2 >= kComputeUnits) n = (n + kComputeUnits - 1) / kComputeUnits * kComputeUnits;
  *window = (int)(((((long long)H + n - 1) / n) + kThreads - 1) / kThreads * kThreads);
  *windows = (int)(((long long)H + *window - 1) / *window);
}

static inline FoldPlan plan_fold(int K, int N, int H, int BK, int BN, int slices, bool windowed = false, int tile_bytes = 4) {
  FoldPlan f = {};
  f.tile_bytes = tile_bytes;
  const long long E = (long long)BK * BN;
  const long long tiles = (long long)((K + BK - 1) / BK) * ((N + BN - 1) / BN);
  // (element indices of the buffer are 32-bit in the kernels; the fold lists slices entries per tile)
  if (E > 16384 || slices > 64 || (long long)slices * tiles * E >= (1LL << 31)) return f;
  // (few tiles over a hashed_weight of up to 2^18 elements: measured 5 to 8 us; with a larger one every
  //  workgroup would still look at every tile for the handful that reach it, and the windowed kernel or
  //  the window kernel do better — K = 2048, N = 4096, H = 2^20: 20 us against the window kernel's 25 in all)
  if (tiles <= 4096 && H <= (1 << 18) && !windowed) {
    // every workgroup of 256 threads owns 256 elements of dHW
    f.small = 1;
    f.window = 256;
    f.windows = (H + f.window - 1) / f.window;
    f.shares = 1;
    f.tiles_bytes = (((size_t)slices * tiles * E * (size_t)tile_bytes + 255) & ~(size_t)255) + 2 * kFoldMarginBytes;
    f.partial_bytes = 0;
    f.offsets_bytes = ((size_t)tiles * sizeof(int32_t) + 255) & ~(size_t)255;
    f.use = 1;
    return f;
  }
  fold_geometry(H, &f.window, &f.windows);
  // (a workgroup fills a compute unit: no more workgroups than compute units, or two would wait for a second round)
  long long shares = f.windows * 2 >= kComputeUnits ? 1 : kComputeUnits / f.windows;
  if (shares > slices * tiles / 8) shares = slices * tiles / 8;   // a share is worth a workgroup from some tiles on
  if (shares < 1) shares = 1;
  f.shares = (int)shares;
  f.tiles_bytes = (((size_t)slices * tiles * E * (size_t)tile_bytes + 255) & ~(size_t)255) + 2 * kFoldMarginBytes;
  const size_t pitch = (size_t)((H + 3) & ~3);
  f.partial_bytes = f.shares > 1 ? ((size_t)f.shares * pitch * sizeof(float) + 255) & ~(size_t)255 : 0;
  f.offsets_bytes = ((size_t)tiles * sizeof(int32_t) + 255) & ~(size_t)255;
  f.use = 1;
  return f;
}

// How the weight-grad contraction C[K,N] = X^T.dY over M is cut into workgroups, and how the
// finished tiles reach dHW.
struct WeightGradPlan {
  int tile;          // C tile edge (128 or 256)
  int splits;        // slices of the reduction over M (blockIdx.y)
  int r_chunk;       // rows of M per slice, a multiple of the R step
  long long workgroups;
  int image_pitch;   // > 0: every workgroup first sums its tiles into an fp32 image of dHW held
                     // in LDS and stores it as one partial image; a second kernel adds the
                     // partial images up.  0: tiles go to dHW by global atomics.
  FoldPlan fold;        // fold.use: no scatter in the contraction kernel at all (tile-by-tile output)
  double fold_us;       // ... and roughly how long the whole weight-grad then takes, in microseconds
  size_t workspace_bytes;   // partial images, or the fp32 image for the atomics (16-bit dHW)
  // bias gradient computed in the same pass: partial column sums of dY, one row per
  // (slice, tile row), stored behind the first `workspace_bytes` of the workspace
  int colsum_rows, colsum_pitch;
  size_t colsum_bytes;
  bool lds_image() const { return image_pitch > 0; }
};

// LDS bytes of a compute unit that an fp32 image of dHW may take (the rest holds the small
// offset table of the scatter); the image reuses the operand stages, which are dead by then.
static constexpr size_t kMaxImageBytes = 147456;

static inline long long tile_cover(int K, int N, int t) {
  return (long long)((K + t - 1) / t) * ((N + t - 1) / t) * t * t;
}

// Slices of M for the 128 and 256 tiles with LDS images: as many as fill the compute units once.  A
// few workgroups beyond one per compute unit would make a second round that costs as much as the
// first (300 workgroups take as long as 512), so the count stays at or below the compute units
// (K = N = 2560, M = 2048 bf16: 3 slices x 100 tiles 57.9 us, 2 slices 46.8 us).
static inline long long image_slices(long long tiles, long long r_steps) {
  long long want = (kComputeUnits + tiles - 1) / tiles;
  if (want > 1 && tiles * want > kComputeUnits) want--;
  if (want > r_steps) want = r_steps;
  return want < 1 ? 1 : want;
}

// How well C tiles fill their rounds of workgroups, relative to an ideal distribution.  256 tiles
// go one to a compute unit in rounds of that many.  128 tiles go two to a compute unit; the
// busiest compute unit gets c = ceil(tiles / CUs) of them and works through them in pairs, a
// last odd one alone in about half the time of a pair.
static inline double filled_256(long long tiles) {
  return (double)tiles / (double)((tiles + kComputeUnits - 1) / kComputeUnits * kComputeUnits);
}
static inline double filled_128(long long tiles) {
  const long long c = (tiles + kComputeUnits - 1) / kComputeUnits;
  return ((double)tiles / (2.0 * kComputeUnits)) / ((double)(c / 2) + (c % 2 ? 0.52 : 0.0));
}
// fp32: the 128 tile in pairs runs at this fraction of the 256 tile's rate (weight-grad, measured:
// 4096^2 1067 against 1012 us in one round each; K = N = 5120, M = 4096: 1831 against 2000 us,
// 1600 tiles in seven half-rounds against 400 in two rounds)
static constexpr double kPairRate128F32 = 0.955;

static inline WeightGradPlan plan_weight_grad(int M, int K, int N, int H, int BK, int BN, int elem_bytes,
                                              const rz_tuning& t, int tile_bytes = 4) {
  WeightGradPlan pl;
  const int pitch = (H + 3) & ~3;
  const bool image = t.lds_image != -1 && (size_t)pitch * sizeof(float) <= kMaxImageBytes;
  if (t.tile) {
    pl.tile = t.tile == 32 ? 64 : t.tile;   // (the 32 x 64 tile serves forward / input-grad only)
  } else if (image) {
    // with the LDS image the M loop can be cut freely (a slice costs one partial image), so
    // the pipelined 256 tile is used unless it would mostly compute padding
    pl.tile = 64;
    if (tile_cover(K, N, 128) * 10 <= tile_cover(K, N, 64) * 13) pl.tile = 128;
    if (tile_cover(K, N, 256) * 10 <= tile_cover(K, N, pl.tile) * 13) pl.tile = 256;
    // a short M cut over many slices leaves a 256 workgroup a few steps between its prologue
    // and its scatter: the 128 tile then has less to set up and to scatter per workgroup
    // (fp32, M = 2048, K = N = 1024: 53.0 -> 47.5 us; M = 512, K = N = 2048: 51.8 -> 48.4 us; 2048^3 and
    //  M = 16384, K = 512, N = 1024 stay with the 256 tile: 135.8 against 138.8 us, 137 either way)
    const long long tiles256 = tile_count(K, N, 256);
    const int step256 = slice_unit(256, elem_bytes, true);
    const bool cover128 = tile_cover(K, N, 128) * 10 <= tile_cover(K, N, 256) * 13;
    if (pl.tile == 256 && elem_bytes == 4 && tiles256 < kComputeUnits &&
        (long long)((M + step256 - 1) / step256) * tiles256 < 16LL * kComputeUnits && cover128)
      pl.tile = 128;
    // (two 128 workgroups fit a compute unit only while two images fit its LDS: K = N = 10240, M = 2048,
    //  H = 36000: 3849 us against 3583 us with the 256 tile)
    if (pl.tile == 256 && elem_bytes == 4 && cover128 && tiles256 >= kComputeUnits && (size_t)pitch * sizeof(float) <= 78 * 1024) {
      // fp32, at least as many 256 tiles as compute units: the two tiles by how they fill their
      // rounds (K = N = 10240 is six rounds and a quarter of the one, twelve and a half pairs of
      // the other: M = 2048 3520 -> 3317 us, M = 4096 6972 -> 6486 us; K = N = 6000, M = 1024:
      // 848 -> 698 us); the image stores of paired workgroups are half hidden behind each other
      const long long tiles128 = tile_count(K, N, 128);
      const double work_us = 2.0 * (double)M * K * N / 137e6, image_us = (double)pitch * 8.0 / 5e6;
      const double t256 = work_us / filled_256(tiles256) + (double)tiles256 * image_us;
      const double t128 = work_us / (kPairRate128F32 * filled_128(tiles128)) + 0.5 * (double)tiles128 * image_us;
      if (t128 < t256 * 0.99) pl.tile = 128;
    }
    if (pl.tile == 256 && elem_bytes == 2 && cover128) {
      // 16-bit: the two tiles by estimated time.  Fitted on MI355X (weight-grad, 256 workgroups):
      // a 256 workgroup pays about 5.5 steps of 64 rows for its fill, its image rounds and the
      // store of its image, whatever the length of its loop; the 128 tile in its eight-wavefront
      // form (steps of 128 rows, up to 384 workgroups) runs at 0.82 of the 256 tile's rate and
      // pays about 4 of its steps.  Both write one image per workgroup.  (2048^3: 32.4 -> 30.5 us;
      // M = 8192, K = N = 2048 stays with the 256 tile: 72.8 against 82.1 us.)
      const long long tiles128 = tile_count(K, N, 128);
      const long long s256 = image_slices(tiles256, (M + 63) / 64), s128 = image_slices(tiles128, (M + 127) / 128);
      const long long w256 = tiles256 * s256, w128 = tiles128 * s128;
      if (w128 <= kComputeUnits * 3 / 2) {
        auto filled = [](long long w, long long cap) { return (double)w / (double)((w + cap - 1) / cap * cap); };
        const double st256 = (double)(((M + 63) / 64 + s256 - 1) / s256), st128 = (double)(((M + 127) / 128 + s128 - 1) / s128);
        const double work_us = 2.0 * (double)M * K * N / 1200e6;
        const double image_us = (double)pitch * 8.0 / 5e6;   // written once, read once
        const double t256 = work_us * (st256 + 5.5) / st256 / filled(w256, kComputeUnits) + (double)w256 * image_us;
        const double t128 = work_us * (st128 + 4.0) / st128 / (0.82 * filled(w128, kComputeUnits)) + (double)w128 * image_us;
        if (t128 < t256 * 0.97) pl.tile = 128;
      }
    }
  } else {
    pl.tile = pick_tile(K, N, elem_bytes, t);
    // fp32 with the tiles stored for the fold kernel: by how the two tiles fill their rounds when
    // there are at least as many 256 tiles as compute units (K = N = 10240: M = 128 455 -> 401 us,
    // M = 1024 1938 -> 1797 us, M = 4096 7002 -> 6449 us; K = N = 4096, one round exactly, stays
    // with the 256 tile: 1043 against 1085 us); with fewer, a short M takes the 128 tile, whose
    // paired workgroups hide each other's stores
    if (pl.tile == 256 && elem_bytes == 4 && t.fold != -1 && plan_fold(K, N, H, BK, BN, 1).use) {
      const long long t256 = tile_count(K, N, 256), t128 = tile_count(K, N, 128);
      if (t256 >= kComputeUnits ? kPairRate128F32 * filled_128(t128) > filled_256(t256) * 1.01 : M <= 2048) pl.tile = 128;
    }
  }
  const long long tiles = (long long)((K + pl.tile - 1) / pl.tile) * ((N + pl.tile - 1) / pl.tile);
  const int TR = slice_unit(pl.tile, elem_bytes, true);
  const int r_steps = (M + TR - 1) / TR;
  // split the reduction over M when there are too few W tiles to fill the chip
  // (one workgroup per compute unit for the 128 tile too: a second one per compute unit would come
  //  with twice the partial images to write and to add up — 1024^3: bf16 22.3 -> 20.4 us, fp32 37.0 -> 33.9 us)
  const long long target = (pl.tile >= 128) ? kComputeUnits : kTargetWorkgroups;
  long long want = (target + tiles - 1) / tiles;
  if (want > r_steps) want = r_steps;
  if (want < 1) want = 1;
  if (image && pl.tile >= 128) want = image_slices(tiles, r_steps);
  if (!image) {
    // every slice repeats the K*N adds of the scatter (global atomics, about 5.4 ps each, some 70 %
    // of which the contraction does not hide): the number of slices with the least estimated time
    if (want > 8) want = 8;
    const double peak = elem_bytes == 4 ? 137e6 : 1150e6;   // flop per microsecond of the 256 tile on a full chip
    double best_us = 0.0;
    long long best = 1;
    for (long long w = 1; w <= want; w++) {
      const long long per = (r_steps + w - 1) / w;
      if ((r_steps + per - 1) / per != w) continue;
      const double steps = (double)per * (TR * elem_bytes / 128);
      const double us = 2.0 * (double)M * K * N / (peak * tile_rate((double)tiles * w, pl.tile, elem_bytes) * steps / (steps + 2.0)) +
                        (double)w * K * N * 3.8e-6;
      if (best_us == 0.0 || us < best_us * 0.97) {
        best_us = us;
        best = w;
      }
    }
    want = best;
  }
  const int steps_per = (int)((r_steps + want - 1) / want);
  pl.splits = (r_steps + steps_per - 1) / steps_per;
  pl.r_chunk = steps_per * TR;
  pl.workgroups = tiles * pl.splits;
  pl.image_pitch = image ? pitch : 0;
  pl.fold = FoldPlan{};
  pl.fold_us = 0.0;
  if (!image && t.fold != -1) {
    const FoldPlan f = plan_fold(K, N, H, BK, BN, pl.splits, t.fold == 2, tile_bytes);
    if (f.use) {
      // what the two ways cost beyond the contraction itself, in microseconds: the part of the
      // K*N global atomics per slice that the contraction does not hide (2.8 to 5.2 ps each,
      // measured), against reading the tiles back (their stores overlap the contraction, unless
      // it is shorter than they are), writing and reading the images, and two more launches
      const double elems = (double)pl.splits * (double)K * (double)N;
      // (fp32, K = N = 10240: the contraction takes 427 us at M = 256, 805 us at M = 512)
      const double product_us = 2.0 * (double)M * K * N / (elem_bytes == 4 ? 145e6 : 900e6);
      const double store_us = elems * tile_bytes / 4.0e6;
      // (K*N atomics take about 5.2 ps each; a long contraction hides up to 2.4 ps of that — K = 2048,
      //  N = 8192, bf16: M = 128 87 us in all against 57 us folded, M = 1024 108 against 79 us)
      const double hidden = 0.45 * product_us < elems * 2.4e-6 ? 0.45 * product_us : elems * 2.4e-6;
      const double atomics_us = elems * 5.2e-6 - hidden;
      // (a workgroup of the fold kernel reads some 20 GB/s: few workgroups cannot use the memory system; all of
      //  them together 6 TB/s of fp32 tiles — K = N = 10240: 85 us — and 4.7 TB/s of 16-bit ones — 58 us —
      //  where the instructions per load set the pace)
      const double read_bytes = elems * tile_bytes * (1.0 + (double)BK * BN / f.window);
      const double all_us = (read_bytes + 2.0 * (double)f.partial_bytes) / (tile_bytes == 4 ? 6.0e6 : 4.7e6);
      const double one_us = read_bytes / ((double)f.windows * f.shares) / (tile_bytes == 4 ? 24e3 : 19e3);
      // (few tiles: every element is read once, by a kernel of a few microseconds; it is taken even where
      //  the atomics would be a little faster — K = N = 1024: 5 us against 3 us on top of the contraction —
      //  because it adds in a fixed order: the same bits on every call)
      const double fold_us = f.small ? (store_us > product_us ? store_us - product_us : 0.0) + elems * tile_bytes / 4.5e6 + 5.0
                                     : (store_us > product_us ? store_us - product_us : 0.0) + (all_us > one_us ? all_us : one_us) + 10.0;
      if (t.fold >= 1 || f.small || fold_us < atomics_us) {
        pl.fold = f;
        // (for the comparison with the window kernel: every round of workgroups of the contraction
        //  kernel also pays its fill, drain and store — about 5 us for a round of 256 tiles, 10 us
        //  in fp32, in proportion to the tile's area — which matters when M is small)
        const double round_us = (elem_bytes == 4 ? 10.0 : 5.0) * (double)pl.tile * pl.tile / 65536.0;
        // (a contraction shorter than the stores of its tiles takes the time of the stores — fp32, K = N = 10240,
        //  H = 2^20, M = 32: 220 us in all)
        const double contraction_us = product_us + round_us * (double)((pl.workgroups + kComputeUnits - 1) / kComputeUnits);
        pl.fold_us = (contraction_us > store_us ? contraction_us : store_us) + fold_us - (store_us > product_us ? store_us - product_us : 0.0);
      }
    }
  }
  size_t ws = 0;
  if (pl.fold.use) ws = pl.fold.tiles_bytes + pl.fold.partial_bytes + pl.fold.offsets_bytes;
  else if (pl.image_pitch > 0) ws = (size_t)pl.workgroups * pl.image_pitch * sizeof(float);
  else if (elem_bytes == 2) ws = (size_t)H * sizeof(float);   // fp32 image for the atomics
  pl.workspace_bytes = (ws + 255) & ~(size_t)255;
  pl.colsum_rows = pl.splits * ((K + pl.tile - 1) / pl.tile);
  pl.colsum_pitch = ((N + pl.tile - 1) / pl.tile) * pl.tile;
  pl.colsum_bytes = (size_t)pl.colsum_rows * pl.colsum_pitch * sizeof(float);
  return pl;
}

// Weight-grad by windows of dHW (rz_window.h): used when hashed_weight is too large for one
// LDS image and the contraction over M is short, so that the K*N global atomics of the scatter
// kernel would dominate.
struct WindowPlan {
  bool use;
  int window;    // elements of dHW per workgroup
  int windows;   // workgroups
  long long tiles;   // W tiles (entries of the offset table the kernel scans)
};
static constexpr int kWindowFloats = 25600;   // LDS floats a workgroup can hold next to its staging

// Hashed tiles that the window kernel serves: 32 to 256 rows, 32 to 128 columns.  Its unit of work is 32
// rows by min(BN, 64) columns of a tile; a tile has window_units of them, unit u = strip * parts + part
// starting at off + window_unit_start and spanning window_unit_span elements of hashed_weight.
static inline bool window_tile_supported(int BK, int BN) {
  return (BN == 32 || BN == 64 || BN == 128) && (BK == 32 || BK == 64 || BK == 128 || BK == 256);
}
static inline int window_unit_cols(int BN) { return BN < 64 ? BN : 64; }
static inline int window_units(int BK, int BN) { return (BK / 32) * (BN / window_unit_cols(BN)); }
static inline int window_unit_span(int BN) { return 31 * BN + window_unit_cols(BN); }
static inline long long window_unit_start(int BN, int u) {
  const int parts = BN / window_unit_cols(BN);
  return (long long)(u / parts) * (32 * BN) + (long long)(u % parts) * window_unit_cols(BN);
}

// Size and number of the windows for a hashed_weight of H elements (a function of H alone: a
// layer plan built once per layer holds the strip lists of exactly these windows).
static inline void window_geometry(int H, int* window, int* windows) {
  // one workgroup per compute unit when the windows can be that large, else whole rounds
  const long long rounds = ((long long)H + (long long)kWindowFloats * kComputeUnits - 1) /
                           ((long long)kWindowFloats * kComputeUnits);
  long long w = (((long long)H + rounds * kComputeUnits - 1) / (rounds * kComputeUnits) + 3) & ~3LL;
  if (w < 1024) w = 1024;                        // tiny windows would each redo most tiles
  *window = (int)w;
  *windows = (int)(((long long)H + w - 1) / w);
}

// planned: the caller holds a layer plan, so the kernel neither hashes the tile offsets nor scans
// them for its strips (some 25 us less, measured at K = N = 10240).
static inline WindowPlan plan_window(int M, int K, int N, int H, int BK, int BN, int elem_bytes, const rz_tuning& t,
                                     const WeightGradPlan& other, bool planned = false) {
  WindowPlan pl = {false, 0, 0, 0};
  if (t.window == -1 || !window_tile_supported(BK, BN)) return pl;
  const long long tiles = (long long)((K + BK - 1) / BK) * ((N + BN - 1) / BN);
  if (tiles > (1 << 20)) return pl;              // every workgroup scans every tile's offset
  pl.tiles = tiles;
  window_geometry(H, &pl.window, &pl.windows);
  const long long w = pl.window;
  // Rough times in microseconds, fitted to measurements at K = N = 10240, H = 6.5 M on MI355X.
  // Scatter kernel: K*N atomics at about 184 G/s plus the product.  Window kernel: every
  // workgroup works through tiles * (window + tile) / H tiles; a tile costs about 0.31 us plus
  // 0.18 us (16-bit), or 0.43 us plus 0.63 us (fp32: the fp32 MFMA rate), per 32 rows of M (the
  // operands of every tile come out of L2 again: tiles that share a window share no rows or
  // columns of W; a wavefront has three groups of rows in flight, which is what its registers hold).
  const double chunks = (double)((M + 31) / 32);
  // (in units of 64 x 64 tiles, i.e. of two strips of 64 columns: the figures below were fitted on those;
  //  32-column tiles take the time of 64-column ones — their units are half empty)
  const double per_wg = (double)tiles * ((double)w + (double)BK * BN) / (double)H * ((double)BK / 64.0) * (BN > 64 ? BN / 64.0 : 1.0);
  const double wg_rounds = (double)((pl.windows + kComputeUnits - 1) / kComputeUnits);
  // (rows of X or dY that are not whole 16-byte pieces are fetched element by element: about 2.2 times the
  //  time per tile — M = 256, K = 10239, N = 10240, bf16: 411 us against 190 us with K = 10240)
  const int vec = 16 / elem_bytes;
  const double by_elements = (K % vec == 0 && N % vec == 0) ? 1.0 : 2.2;
  double t_window = wg_rounds * per_wg * by_elements * ((elem_bytes == 4 ? 0.43 + 0.63 * chunks : 0.31 + 0.18 * chunks)) + (planned ? 5.0 : 28.0);
  // Every element of dHW receives K*N / H tiles, and the adds into one place of a window go in a
  // fixed order, one after the other: with many tiles per element that chain is what takes the
  // time, about 1.7 us a link (K = 2048, N = 8192, H = 200000: 84 links, 158 us at M = 32 — folded
  // 57 us; K = N = 10240, H = 200000: 524 links, 1048 us).
  // (fp32, K = N = 10240, H = 2^20, M = 32: 100 links, 260 us — folded 220 us)
  const double chain_us = (elem_bytes == 4 ? 2.4 : 1.7) * (double)K * (double)N / (double)H + 10.0;
  if (t_window < chain_us) t_window = chain_us;
  // ... against what the contraction kernel's plan would take: the fold, or the atomic scatter
  const double t_scatter = 0.9 * (double)K * N / 184e3 + 2.0 * M * (double)K * N / 800e6;
  const double t_other = other.fold.use ? other.fold_us : t_scatter;
  pl.use = t.window == 1 || t_window < t_other;
  return pl;
}

// A layer plan: what the weight-grad of one layer needs of its hash and nothing else (it depends on
// K, N, H, the tile and the hash constants, not on M, the element type or the data), computed once
// on the host and kept by the caller in device memory.  int32 words:
//   [0, 16)   header: magic, version, K, N, H, BK, BN, hash_levels, tiles, windows, window,
//             entries, strips per tile, checksum of the hash constants (layer_plan_hash_sum),
//             fold windows, fold window
//   offsets   [tiles]           where every W tile starts in hashed_weight (index tk * tiles_n + tn)
//   start     [windows + 1]     first entry of every window of the window kernel (window_geometry)
//   list      [capacity]        the units of work (tile * units per tile + unit: 32 rows by up to 64 columns of
//                               a tile, see window_units) that meet the window, ascending
//   offs      [capacity]        ... and where each starts in hashed_weight
//   fold_start [fold windows + 1]  first entry of every window of the fold kernel (fold_geometry)
//   fold_list  [fold capacity]     the tiles that meet the window, in the order in which the fold kernel's
//                                  own search numbers them (fold_rank_order)
// The first two lists exist for the tiles the window kernel supports (windows = 0 otherwise).
static constexpr int32_t kLayerPlanMagic = 0x525a4c50, kLayerPlanVersion = 2;
static constexpr int kLayerPlanHeader = 16;
// What a plan's header says of the hash constants that its offsets were computed with (the kernels
// that read a plan compare it with their own call's constants).
__host__ __device__ static inline int32_t layer_plan_hash_sum(const HashParams& h) {
  uint32_t s = 2166136261u;
  const uint32_t v[8] = {h.R0, h.R1, h.R2, h.R3, h.R4, h.R5, h.R7, (uint32_t)h.levels};
  for (int i = 0; i < 8; i++) s = (s ^ v[i]) * 16777619u;
  return (int32_t)(s & 0x7fffffffu);
}
// header words 2..7 and 13 against a call (K, N, H, BK, BN, hash_levels, constants)
__host__ __device__ static inline bool layer_plan_matches(const int32_t* hd, int K, int N, int H, const HashParams& h) {
  return hd[0] == kLayerPlanMagic && hd[2] == K && hd[3] == N && hd[4] == H && hd[5] == h.BK && hd[6] == h.BN &&
         hd[7] == h.levels && hd[13] == layer_plan_hash_sum(h);
}
struct LayerPlanLayout {
  bool ok;
  int tiles, windows, window, strips_per_tile, strip_elems;   // (units per tile, elements a unit spans)
  long long capacity;                 // list entries reserved (an upper bound of those used)
  int fold_window, fold_windows;
  long long fold_capacity;
  size_t offsets_at, start_at, list_at, offs_at, fold_start_at, fold_list_at, words;
};
static inline LayerPlanLayout layer_plan_layout(int K, int N, int H, int BK, int BN) {
  LayerPlanLayout l = {};
  const long long tiles = (long long)((K + BK - 1) / BK) * ((N + BN - 1) / BN);
  if (tiles > (1 << 22)) return l;
  l.tiles = (int)tiles;
  auto round16 = [](size_t v) { return (v + 15) & ~(size_t)15; };
  l.offsets_at = kLayerPlanHeader;
  l.start_at = round16(l.offsets_at + (size_t)tiles);
  if (window_tile_supported(BK, BN) && tiles <= (1 << 20)) {
    window_geometry(H, &l.window, &l.windows);
    l.strips_per_tile = window_units(BK, BN);
    l.strip_elems = window_unit_span(BN);
    // a unit that spans strip_elems consecutive elements meets at most ceil(strip_elems / window) + 1 windows
    l.capacity = tiles * l.strips_per_tile * ((l.strip_elems + l.window - 1) / l.window + 1);
  }
  l.list_at = round16(l.start_at + (size_t)l.windows + 1);
  l.offs_at = round16(l.list_at + (size_t)l.capacity);
  // a tile of BK * BN consecutive elements meets at most ceil(BK * BN / window) + 1 fold windows
  fold_geometry(H, &l.fold_window, &l.fold_windows);
  l.fold_capacity = tiles * (((long long)BK * BN + l.fold_window - 1) / l.fold_window + 1);
  l.fold_start_at = round16(l.offs_at + (size_t)l.capacity);
  l.fold_list_at = round16(l.fold_start_at + (size_t)l.fold_windows + 1);
  l.words = round16(l.fold_list_at + (size_t)l.fold_capacity);
  l.ok = l.words < (1u << 30);
  return l;
}

// Forward / input-grad with few C tiles and a long contraction (skinny batches): R is cut into
// slices over blockIdx.y, every slice writes an fp32 partial result, a second kernel adds them.
struct SplitPlan {
  int tile;
  int splits;        // 1 = no split, no workspace
  int r_chunk;
  size_t workspace_bytes;
  double est_us;     // what the model expects the launch(es) to take
};

// Slices up to which a cut contraction is finished by its own kernel (GemmParams::finish; 0: never).  The
// slice that comes last at a tile reads the others' planes by itself, four bytes per lane and load, after
// an atomic's round trip: that pays up to four slices, where the rows of a tile are real (a batch of
// fewer rows than the tile has is finished in 3 us by a second kernel too), and with the 256 tile only
// where the planes are large.  Measured, forward, GPU-bound (finished in the kernel / second kernel):
// bf16 K = N = 10240: M = 128, 128 tile, three slices 47 / 54 us; M = 32 49 / 46; M = 1024, 256 tile 252 / 260;
// M = 128, 256 tile 104 / 93.  M = 128, K = 2048, N = 8192: 128 tile, three slices 14.7 / 20.8 us.
// M = 64, K = N = 4096: 64 tile, four slices 12.7 / 13.6; 128 tile 21.3 / 18.4.  Six slices at M = 32: 52 / 40.
// The 32 x 64 tile has two wavefronts to read with: two slices.
static inline int finish_slices(int tile, int I, int J) {
  if (I < (tile == 32 ? 32 : tile)) return 0;
  if (tile == 256 && (double)I * J * 4.0 < 16.0e6) return 0;
  return tile == 32 ? 2 : kFinishSlices;
}

// Tile and number of slices together: the pair with the least estimated time.  A slice pays the
// fill and drain of its pipeline (about three steps), the cut pays the fp32 partial planes
// (written, read back) and the launch of the kernel that adds them.
static inline SplitPlan plan_split(int I, int J, int R, int elem_bytes, const rz_tuning& t, int depth = 0) {
  SplitPlan best = {};
  double best_us = 0.0;
  const double peak = elem_bytes == 4 ? 149e6 : 1150e6;   // flop per microsecond of the 256 tile on a full chip
  const int tiles_of[4] = {256, 128, 64, 32};
  // (an override that asks for the 32 x 64 tile where it does not exist gets the 64 tile)
  const int forced = (t.tile == 32 && elem_bytes != 4) ? 64 : t.tile;
  for (int tile : tiles_of) {
    if (forced && tile != forced) continue;
    // (the 32 x 64 tile: fp32 only, and only where 64-row tiles would end in a tile at most half full —
    //  K = N = 10240: M = 96 259 -> 232 us, M = 160 428 -> 353 us, M = 288 668 -> 620 us)
    if (tile == 32 && !forced && (elem_bytes != 4 || (I > 32 && (I - 1) % 64 >= 32))) continue;
    const int TR = slice_unit(tile, elem_bytes);
    const long long tiles = tile_count(I, J, tile);
    const int r_steps = (R + TR - 1) / TR;
    const double useful = (double)I * (double)J / ((double)tiles * tile * tile_cols(tile));
    // fp32 staged directly (complete tiles, or ragged ones with rows of 16 bytes and more): see tile_rate;
    // a workgroup's fill and drain cost about 2, 8 and 12 steps of 128 bytes for the tiles of 256, 128
    // and 64 / 32 x 64 (4096^3: 941, 986, 1016 us; M = 4096, K = N = 1024: 128 tile 76 us, 64 tile 82 us;
    // 1024^3: 64 tile 23.8 us, 128 tile cut in four 35 us).  The bounds-checked form, which only shapes
    // with shorter rows or an override still take, keeps the older pricing.
    const bool whole = I % tile == 0 && J % tile_cols(tile) == 0 && R % TR == 0;
    const bool direct = elem_bytes == 4 && (whole || (t.clamp != -1 && R * elem_bytes >= 16));
    const double lo64 = whole ? 0.67 : 0.60;
    const double fill = !direct ? 2.0 : tile == 256 ? 2.0 : tile == 128 ? 8.0 : 12.0;
    double whole_us = 0.0;
    for (int want = 1; want <= 16; want++) {
      if (want > 1 && t.split == -1) break;
      // (a kernel of a dozen microseconds is not worth cutting: the second launch and the short loops
      //  cost what the idle compute units would have gained — fp32, M = 32 and 96, K = N = 1024: 13 us
      //  whole, 15 us cut in eight or four)
      if (want > 1 && direct && whole_us <= 16.0 && t.split <= 0) break;
      const int steps_per = (r_steps + want - 1) / want;
      const int slices = (r_steps + steps_per - 1) / steps_per;
      if (slices != want) continue;                           // (the same cut as a smaller `want`)
      if (t.split > 0 && slices != t.split) continue;         // (an override asks for exactly that many slices)
      if (slices > 1 && steps_per * (TR * elem_bytes / 128) < 4 && t.split <= 0) break;   // slices of a few steps are all fill and drain
      const double steps = (double)steps_per * (TR * elem_bytes / 128);
      const double rate = peak * tile_rate((double)tiles * slices, tile, elem_bytes, lo64, direct || elem_bytes == 2) * useful * steps / (steps + fill);
      double us = 2.0 * (double)I * (double)J * (double)R / rate + 4.0;
      // (up to finish_slices the kernel finishes its own tiles: every plane is written, all but one are read
      //  back by the finishing workgroups, and no second kernel is launched — worth a couple of microseconds
      //  and a plane; fp32, M = 16384, K = 512, N = 1024 input-grad, planes of 33 MB: the 256 tile in two
      //  slices 155 us against the whole 128 tile's 136)
      if (slices > 1 && slices <= finish_slices(tile, I, J) && t.finish != -1) us += (2.0 * slices - 1.0) * (double)I * J * 4.0 / 4.0e6 + 2.0;
      else if (slices > 1) us += (2.0 * slices * (double)I * J * 4.0 + (double)I * J * elem_bytes) / 4.0e6 + (direct ? 3.0 : 4.0);
      else whole_us = us;
      // (near ties go to the larger tile and the fewer slices, which come first)
      if (best.tile == 0 || us < best_us * 0.97) {
        best.tile = tile;
        best.splits = slices;
        best.r_chunk = steps_per * TR;
        best_us = us;
      }
    }
  }
  // (16-bit: a problem that some tile does whole in a dozen microseconds is not cut — M = 128, K = N = 1024:
  //  64 tile whole 10.2 us; every cut, finished in the kernel or not, 12 to 16 us)
  if (elem_bytes == 2 && t.split == 0 && best.splits > 1 && depth == 0) {
    rz_tuning whole_only = t;
    whole_only.split = -1;
    const SplitPlan w = plan_split(I, J, R, elem_bytes, whole_only, 1);
    if (w.est_us <= 14.0) return w;
  }
  if (best.tile == 0 && t.split > 0) {   // (no cut comes out at exactly that many slices: the library's own choice)
    rz_tuning free_cut = t;
    free_cut.split = 0;
    return plan_split(I, J, R, elem_bytes, free_cut);
  }
  best.workspace_bytes = best.splits > 1 ? (size_t)best.splits * (size_t)I * (size_t)J * sizeof(float) : 0;
  best.est_us = best_us;
  return best;
}

// Which instantiation of the contraction kernel runs a launch: C tile, wavefronts, LDS stages,
// whether every tile and step is complete (no bounds checks), whether a ragged shape still
// takes direct staging with edge pieces fetched from inside the operands, and the contracted
// elements per step that follow from those.  One function decides for the launch and for
// rz_plan_query.
struct KernelForm {
  int tile, waves, stages;
  bool full, clamp;
  int step;
};

static inline KernelForm kernel_form(int op, int I, int J, int R, int chunk, int tile, long long workgroups,
                                     int elem_bytes, const rz_tuning& t) {
  KernelForm f;
  f.tile = tile;
  f.stages = (tile == 128 && t.stages == 1) ? 1 : 2;
  // 128 tile: with about one workgroup per compute unit, eight wavefronts (two per SIMD, 64 x 32
  // each) hide latency better than four of 64 x 64; with more workgroups resident the
  // four-wavefront form does less LDS traffic per flop
  // 64 tile: four wavefronts; fp32 forward / input-grad take eight (two groups that share every R
  // step: a second wavefront per SIMD keeps the MFMA pipe fed while the first waits for LDS)
  f.waves = tile == 256 ? 8
            : tile == 32 ? 4
            : tile == 64 ? ((elem_bytes == 4 && op != kWeightGrad) ? 8 : 4)
                         : (f.stages == 1 ? 4 : (workgroups <= kComputeUnits * 3 / 2 ? 8 : 4));
  // (32-bit: every two-stage form stages directly; 16-bit: the tiles of 128 and more)
  const bool direct_capable = f.stages == 2 && (elem_bytes == 4 || tile >= 128);
  const int step_plain = elem_bytes == 4 ? slice_unit(tile, elem_bytes, op == kWeightGrad) : 128 / elem_bytes;
  const int step_direct = (direct_capable && elem_bytes == 2 && tile == 128 && f.waves == 8) ? 256 / elem_bytes : step_plain;
  f.full = (I % tile == 0) && (J % tile_cols(tile) == 0) && (R % step_direct == 0) && (chunk % step_direct == 0);
  // a plain operand's rows must hold at least one 16-byte piece (a piece that straddles the end of a
  // row is handled in the kernel; a row shorter than a piece is not)
  const int vec = 16 / elem_bytes;
  const bool pieces_ok = op == kWeightGrad ? (I >= vec && J >= vec) : R >= vec;
  f.clamp = !f.full && direct_capable && pieces_ok && t.clamp != -1;
  f.step = (f.full || f.clamp) ? step_direct : step_plain;
  return f;
}

// Fills in the tiling fields of `p` and enqueues the kernel for `op` on `stream`; weight-grad
// takes its plan (tile, split of M, scatter mode) from `plan`, the others ignore it.
// (forward / input-grad take tile and split from `split`, or pick a tile and do not split).
hipError_t launch_gemm_f32(int op, GemmParams p, const WeightGradPlan* plan, const SplitPlan* split,
                           const rz_tuning& tuning, hipStream_t stream);
hipError_t launch_gemm_bf16(int op, GemmParams p, const WeightGradPlan* plan, const SplitPlan* split,
                            const rz_tuning& tuning, hipStream_t stream);
hipError_t launch_gemm_f16(int op, GemmParams p, const WeightGradPlan* plan, const SplitPlan* split,
                           const rz_tuning& tuning, hipStream_t stream);

struct WindowParams;
// Enqueues the windowed weight-grad kernel; p.window and the tile grid must come from plan_window.
hipError_t launch_window_f32(const WindowParams& p, int windows, hipStream_t stream);
hipError_t launch_window_bf16(const WindowParams& p, int windows, hipStream_t stream);
hipError_t launch_window_f16(const WindowParams& p, int windows, hipStream_t stream);

}  // namespace rz
