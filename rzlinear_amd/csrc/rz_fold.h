// Fold kernel of the weight gradient: dHW[h] = sum of the elements of X^T.dY that hash to h, from
// X^T.dY stored tile by tile (GemmParams::tiles_out).  The transpose of the reference's scatter
// (python/rz_linear/impl/RzLinearBackward.py:190-218 adds every BLOCK_SIZE_K x BLOCK_SIZE_N tile at
// its hashed offset with atomics): here a workgroup OWNS a window of hashed_weight, looks for the
// tiles that land in it and adds them up in LDS.  No atomics anywhere, and the order of the
// additions is fixed (the order of the workgroup's tile list), so the result is the same on every call.
//
// A hashed tile is BK*BN contiguous elements of hashed_weight and BK*BN contiguous floats of the
// tile-by-tile buffer (of which only the part inside K x N is read), so its reads are whole cache lines whatever its offset.  Inside the
// workgroup thread i owns the window positions i, i + 1024, i + 2048, ...: for every tile it
// reads the elements that fall on its own positions (consecutive threads, consecutive addresses)
// and adds them with plain LDS read-add-write.  No two threads ever touch the same LDS word, so
// no barrier is needed between tiles.
//
// A window is at most 32768 floats (128 KB of LDS).  When hashed_weight has fewer windows than
// the chip has compute units, `shares` workgroups share a window: each takes an equal part of the
// window's tiles and writes its own partial image; reduce_partials_kernel adds the images.
// With a single share the workgroup writes its window of dHW itself.
#pragma once

#include <hip/hip_runtime.h>

#include "../../include/rzlinear.h"
#include "rz_common.h"

namespace rz {

struct FoldParams {
  const float* tiles;   // [slices][tiles_k * tiles_n][BK * BN]
  const int32_t* offsets;   // [tiles_k * tiles_n] where every tile starts in hashed_weight (hashed once, by another kernel)
  float* partial;       // [shares][pitch]: every workgroup writes its window of its share's image ...
  void* out;            // ... or, with a single share (partial == null), its window of dHW itself:
  int out_dtype;        //     an rz_dtype code,
  int accumulate;       //     added to what dHW holds, if set
  HashParams h;
  int H, pitch;
  int K, N;             // extent of X^T.dY: what a tile holds beyond it was never written and is not read
  int tiles_k, tiles_n, slices;
  int window;           // floats per window, a multiple of kFoldThreads
  int windows, shares;
};

static constexpr int kFoldThreads = 1024;
static constexpr int kFoldList = 2048;       // entries of the tile list in LDS
static constexpr int kFoldScan = 32;         // tile indices per thread and listing pass
static constexpr int kFoldWindowMax = 32768;

static inline size_t fold_lds_bytes(int window) {
  return (size_t)window * sizeof(float) + 3 * kFoldList * sizeof(int) + 32 * sizeof(int);
}

// LPE: loads per list entry and thread, BK*BN / 1024 (1 for smaller tiles: then only the first
// BK*BN threads of an entry have an element).  A round of 16 loads per thread is issued before
// its additions.
template <int LPE>
__global__ __launch_bounds__(kFoldThreads) void fold_tiles_kernel(const FoldParams p) {
  extern __shared__ __align__(16) float fold_lds[];
  float* img = fold_lds;
  int* list_at = reinterpret_cast<int*>(fold_lds + p.window);   // first float of the entry's tile
  int* list_rel = list_at + kFoldList;                           // where the tile starts, relative to the window
  int* list_lim = list_rel + kFoldList;                          // rows | columns << 16 of the tile inside K x N
  int* wave_sum = list_lim + kFoldList;                          // [16] per-wavefront counts, [16] = total
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int win = blockIdx.x % p.windows, share = blockIdx.x / p.windows;
  const int w0 = win * p.window;
  const int wlen = (p.H - w0) < p.window ? (p.H - w0) : p.window;
  const int E = p.h.BK * p.h.BN, eshift = p.h.bk_shift + p.h.bn_shift;
  const int ntiles = p.tiles_k * p.tiles_n;
  for (int q = tid; q < p.window; q += kFoldThreads) img[q] = 0.f;   // (own positions only)

  // bit j: tile first + i + 1024 j (below `stop`) lands in the window; the offsets are fetched together
  auto scan = [&](int first, int stop) -> unsigned {
    unsigned mask = 0u;
#pragma unroll
    for (int j = 0; j < kFoldScan; j++) {
      // (no branch around the loads: they are issued together)
      const int id = first + tid + j * kFoldThreads;
      const int rel = p.offsets[id < stop ? id : stop - 1] - w0;
      mask |= (id < stop && rel > -E && rel < wlen) ? 1u << j : 0u;
    }
    return mask;
  };
  // sum over the workgroup, and over the wavefronts before this one (two barriers)
  auto total_of = [&](int incl, int* before) -> int {
    __syncthreads();   // (earlier reads of wave_sum, and of the list, are over)
    if (lane == 63) wave_sum[wave] = incl;
    __syncthreads();
    int sum = 0;
    *before = 0;
    for (int v = 0; v < kFoldThreads / 64; v++) {
      const int c = wave_sum[v];
      if (v < wave) *before += c;
      sum += c;
    }
    return sum;
  };
  auto wave_scan = [&](int mine) -> int {   // inclusive
    int incl = mine;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int up = __shfl_up(incl, d, 64);
      if (lane >= d) incl += up;
    }
    return incl;
  };

  // The window's tiles are numbered in a fixed order (pass by pass, thread by thread); the share
  // takes an equal part of the numbers: the workgroups of a window then have the same work to
  // within a tile, whatever the hash does.
  int rank_lo = 0, rank_hi = 0x7fffffff;
  if (p.shares > 1) {
    int mine = 0, before;
    for (int first = 0; first < ntiles; first += kFoldScan * kFoldThreads) mine += __popc(scan(first, ntiles));
    const int all = total_of(wave_scan(mine), &before);
    rank_lo = (int)((long long)share * all / p.shares);
    rank_hi = (int)((long long)(share + 1) * all / p.shares);
  }
  int lo = 0, seen = 0;                    // tiles [0, lo) hold `seen` tiles of the window
  int span = kFoldScan * kFoldThreads;
  while (lo < ntiles && seen < rank_hi) {   // (uniform: every thread of the workgroup goes round together)
    if (span > ntiles - lo) span = ntiles - lo;
    // --- list the share's tiles among [lo, lo + span) ---------------------------------------------
    unsigned mask = scan(lo, lo + span);
    const int mine = __popc(mask);
    const int incl = wave_scan(mine);
    int before;
    const int found = total_of(incl, &before);
    const int want_lo = rank_lo > seen ? rank_lo : seen;
    const int want_hi = rank_hi < seen + found ? rank_hi : seen + found;
    const int total = (want_hi > want_lo ? want_hi - want_lo : 0) * p.slices;
    if (total > kFoldList) {   // does not fit: look at half the range (a range of kFoldList / slices tiles always fits)
      span = (span + 1) / 2;
      continue;
    }
    int rank = seen + before + incl - mine;   // of this thread's first tile
    while (mask != 0u) {
      const int j = __ffs(mask) - 1;
      mask &= mask - 1u;
      if (rank >= want_lo && rank < want_hi) {
        const int id = lo + tid + j * kFoldThreads;
        const int rel = p.offsets[id] - w0;
        const int tk = id / p.tiles_n, tn = id - tk * p.tiles_n;
        const int rows = (p.K - tk * p.h.BK) < p.h.BK ? (p.K - tk * p.h.BK) : p.h.BK;
        const int cols = (p.N - tn * p.h.BN) < p.h.BN ? (p.N - tn * p.h.BN) : p.h.BN;
        for (int s = 0; s < p.slices; s++) {
          list_at[(rank - want_lo) * p.slices + s] = (s * ntiles + id) << eshift;
          list_rel[(rank - want_lo) * p.slices + s] = rel;
          list_lim[(rank - want_lo) * p.slices + s] = rows | cols << 16;
        }
      }
      rank++;
    }
    seen += found;
    __syncthreads();
    // --- add the listed tiles into the window -------------------------------------------------
    // Rounds of 16 loads per thread (16 / LPE entries); the next round's loads are in flight
    // while this round's values are added, in list order.  Lane u of every wavefront fetches
    // entry u of the round from the list; the entries are then uniform values (scalar registers).
    constexpr int kRound = 16 / LPE;
    struct Round {
      float v[16];
      int q[16];      // window position of v[f], -1: none
      bool clash;     // (uniform) two tiles of the round overlap: their adds must stay in order
    };
    auto issue = [&](int t, Round& r) {
      const bool have = lane < kRound && t + lane < total;
      const int my_rel = have ? list_rel[t + lane] : -(1 << 29);   // (far away: no element lands in the window)
      const int my_at = have ? list_at[t + lane] : 0;
      const int my_lim = have ? list_lim[t + lane] : 0;
      bool meets = false;
#pragma unroll
      for (int d = 1; d < kRound; d++) {
        const int other = __shfl_down(my_rel, d, 64);
        const int gap = my_rel - other;
        meets |= have && lane + d < kRound && gap < E && gap > -E;
      }
      r.clash = __ballot(meets) != 0ull;
#pragma unroll
      for (int f = 0; f < 16; f++) {
        const int rel = __builtin_amdgcn_readlane(my_rel, f / LPE), at = __builtin_amdgcn_readlane(my_at, f / LPE);
        const int lim = __builtin_amdgcn_readlane(my_lim, f / LPE);
        const int e = ((tid - rel) & (kFoldThreads - 1)) + (f % LPE) * kFoldThreads;   // my (f % LPE)-th element of the tile
        const int pos = rel + e;                                                       // (pos % 1024 == tid)
        // (in the window, and inside K x N: the contraction wrote nothing beyond its own C tiles)
        const bool ok = e < E && pos >= 0 && pos < wlen && (e >> p.h.bn_shift) < (lim & 0xffff) &&
                        (e & (p.h.BN - 1)) < (lim >> 16);
        // (every thread loads, those without an element the tile's first float: with no branch
        //  around the loads their number is fixed, and the wait for this round's values can leave
        //  the next round's in flight)
        const float x = p.tiles[(uint32_t)(ok ? at + e : at)];
        r.v[f] = ok ? x : 0.f;
        r.q[f] = ok ? pos : -1;
      }
    };
    // (plain read-add-write: LDS float atomics are several times slower, and nobody else touches
    //  this thread's words)
    auto add = [&](const Round& r) {
      if (!r.clash) {   // all positions of the round differ: read them together
        float cur[16];
#pragma unroll
        for (int f = 0; f < 16; f++) cur[f] = img[r.q[f] >= 0 ? r.q[f] : tid];
#pragma unroll
        for (int f = 0; f < 16; f++)
          if (r.q[f] >= 0) img[r.q[f]] = cur[f] + r.v[f];
      } else {
#pragma unroll
        for (int f = 0; f < 16; f++)
          if (r.q[f] >= 0) img[r.q[f]] += r.v[f];
      }
    };
    Round r0, r1;
    issue(0, r0);
    for (int t = 0; t < total; t += 2 * kRound) {
      issue(t + kRound, r1);
      add(r0);
      issue(t + 2 * kRound, r0);
      add(r1);
    }
    lo += span;
  }
  // --- the window of this share's image ---------------------------------------------------------
  if (p.partial != nullptr) {
    float* out = p.partial + (size_t)share * (size_t)p.pitch + w0;
    for (int q = tid; q < wlen; q += kFoldThreads) out[q] = img[q];
  } else if (p.out_dtype == RZ_F32) {
    float* out = reinterpret_cast<float*>(p.out) + w0;
    for (int q = tid; q < wlen; q += kFoldThreads) out[q] = img[q] + (p.accumulate ? out[q] : 0.f);
  } else if (p.out_dtype == RZ_BF16) {
    bf16_t* out = reinterpret_cast<bf16_t*>(p.out) + w0;
    for (int q = tid; q < wlen; q += kFoldThreads)
      out[q] = ElemTraits<bf16_t>::from_float(img[q] + (p.accumulate ? ElemTraits<bf16_t>::to_float(out[q]) : 0.f));
  } else {
    f16_t* out = reinterpret_cast<f16_t*>(p.out) + w0;
    for (int q = tid; q < wlen; q += kFoldThreads)
      out[q] = ElemTraits<f16_t>::from_float(img[q] + (p.accumulate ? ElemTraits<f16_t>::to_float(out[q]) : 0.f));
  }
}

}  // namespace rz
