// Fold kernel of the weight gradient: dHW[h] = sum of the elements of X^T.dY that hash to h, from
// X^T.dY stored tile by tile (GemmParams::tiles_out).  The transpose of the reference's scatter
// (python/rz_linear/impl/RzLinearBackward.py:190-218 adds every BLOCK_SIZE_K x BLOCK_SIZE_N tile at
// its hashed offset with atomics): here a workgroup OWNS a window of hashed_weight, looks for the
// tiles that land in it and adds them up in LDS.  No atomics anywhere, and the order of the
// additions is fixed (the order of the workgroup's tile list), so the result is the same on every call.
//
// A hashed tile is BK*BN contiguous elements of hashed_weight and BK*BN contiguous floats of the
// tile-by-tile buffer, so its reads are whole cache lines whatever its offset.  The list holds
// the tiles in runs of at most 2048 elements.  The window is cut into blocks of 256 positions (of
// 512 where the tiles are kept in a 16-bit type): sixteen bytes of tile elements per lane;
// wavefront w owns the blocks w, w + 16, w + 32, ..., and inside a block lane l owns the four
// (eight) positions from 4 l (8 l) on.  A run meets at most nine blocks in a row, so at most one of a
// wavefront's: the wavefront walks down the list, skips the runs that miss its blocks, and for
// each of the others reads the elements that fall on its block with ONE 16-byte load per lane
// (from a scalar base: the run starts anywhere, on an element's boundary) and adds them with
// 16-byte LDS reads, additions and 16-byte LDS writes.  What a run needs per
// wavefront is scalar arithmetic; no two lanes ever touch the same LDS word, so the wavefronts
// need no barrier between runs and each goes down the list at its own pace.  Only the blocks
// at the two ends of a run, and runs of tiles that stick out of K x N (whose buffer holds floats
// that the contraction never wrote), need their elements masked one by one: a branch of its
// own; there, lanes wholly outside the run re-fetch floats of the run, so that a block costs no
// memory traffic beyond the run's own cache lines.  The loads reach up to one element short of
// sixteen bytes before and after a run (an empty slot of a round reads the buffer's first kilobyte):
// the buffer is allocated with a margin on both sides.
//
// A window is at most 32768 floats (128 KB of LDS).  When hashed_weight has fewer windows than
// the chip has compute units, `shares` workgroups share a window: each takes an equal part of the
// window's tiles and writes its own partial image; reduce_partials_kernel adds the images.
// With a single share the workgroup writes its window of dHW itself.
#pragma once

#include <hip/hip_runtime.h>

#include "../../include/rzlinear.h"
#include "rz_common.h"
#include "rz_launch.h"

namespace rz {

struct FoldParams {
  const void* tiles;    // [slices][tiles_k * tiles_n][BK * BN], floats or elements of a 16-bit dtype (the kernels' TT)
  const int32_t* offsets;   // [tiles_k * tiles_n] where every tile starts in hashed_weight (hashed once, by another kernel;
                            // null for the few-tiles kernel: it hashes them itself)
  const int32_t* plan_header;   // `offsets` belongs to a layer plan (else null): its header, checked against this call's
  const int32_t* plan_start;    // the plan's list of every window's tiles (else null: the kernel looks for them): [windows + 1] ...
  const int32_t* plan_list;     // ... and the tile indices, in the order in which the kernel's own search numbers them
  int plan_capacity;            // ... of which the plan has room for this many
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
static constexpr int kFoldList = 2048;       // entries of the run list in LDS
static constexpr int kFoldScan = 64;         // tile indices per thread and listing pass (one bit each of a 64-bit mask)
static constexpr int kFoldWindowMax = 32768;
static constexpr int kFoldRun = 2048;        // floats of a run at most (tiles are powers of two: whole runs)
static constexpr int kFoldRound = 8;         // runs whose loads a wavefront issues together
// (a wavefront's block of window positions: sixteen bytes of tile elements per lane — see FoldRaw)

static inline size_t fold_lds_bytes(int window) {
  return (size_t)window * sizeof(float) + 3 * kFoldList * sizeof(int) + 32 * sizeof(int);
}

typedef float fold_f4 __attribute__((ext_vector_type(4)));
typedef float fold_f4u __attribute__((ext_vector_type(4), aligned(4)));
typedef uint16_t fold_h8 __attribute__((ext_vector_type(8)));
typedef uint16_t fold_h8u __attribute__((ext_vector_type(8), aligned(2)));

// The sixteen bytes of consecutive tile elements that a lane loads at a time, as they lie in memory
// (TT = float: four, bf16_t or f16_t: eight), and as floats.
template <typename TT> struct FoldRaw {
  typedef fold_h8 type;
  typedef fold_h8u unaligned;
  static constexpr int kPer = 8;
};
template <> struct FoldRaw<float> {
  typedef fold_f4 type;
  typedef fold_f4u unaligned;
  static constexpr int kPer = 4;
};
template <typename TT>
__device__ __forceinline__ void fold_widen(typename FoldRaw<TT>::type raw, float* v) {
#pragma unroll
  for (int f = 0; f < FoldRaw<TT>::kPer; f++) {
    if constexpr (sizeof(TT) == 4) {
      v[f] = raw[f];
    } else {
      TT e;
      const uint16_t bits = raw[f];
      __builtin_memcpy(&e, &bits, 2);
      v[f] = ElemTraits<TT>::to_float(e);
    }
  }
}

template <typename TT>
__global__ __launch_bounds__(kFoldThreads) void fold_tiles_kernel(const FoldParams p) {
  extern __shared__ __align__(16) float fold_lds[];
  float* img = fold_lds;
  int* list_at = reinterpret_cast<int*>(fold_lds + p.window);   // first float of the run in the buffer
  int* list_rel = list_at + kFoldList;                           // where the run starts, relative to the window
  int* list_lim = list_rel + kFoldList;                          // (rows - 1) | (columns - 1) << 14 of the tile inside K x N | run << 28
  int* wave_sum = list_lim + kFoldList;                          // [16] per-wavefront counts, [16] = total
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  constexpr int kPer = FoldRaw<TT>::kPer;          // window positions of a lane inside a block
  constexpr int kFoldBlock = 64 * kPer;            // ... and of the block: 256 or 512
  constexpr int kBlockShift = kPer == 4 ? 8 : 9;
  const int lane_e = lane * kPer;
  const unsigned lane16 = lane * 16;
  const int win = blockIdx.x % p.windows, share = blockIdx.x / p.windows;
  const int w0 = win * p.window;
  const int wlen = (p.H - w0) < p.window ? (p.H - w0) : p.window;
  const int E = p.h.BK * p.h.BN, eshift = p.h.bk_shift + p.h.bn_shift;
  const int ntiles = p.tiles_k * p.tiles_n;
  const int run = E < kFoldRun ? E : kFoldRun, runs = E / run;   // (E is a power of two)
  const int per_tile = p.slices * runs;                          // list entries of a tile
  const int full_lim = (p.h.BK - 1) | (p.h.BN - 1) << 14;
  // Offsets from a plan that was built for another layer, tile or hash would be in range and
  // wrong: then the image is NaN and nothing is added (what the output paths below store).
  const bool plan_ok = p.plan_header == nullptr ||
                       (layer_plan_matches(p.plan_header, p.K, p.N, p.H, p.h) &&
                        (p.plan_list == nullptr || (p.plan_header[14] == p.windows && p.plan_header[15] == p.window)));   // (uniform)
  for (int q = tid; q < p.window; q += kFoldThreads) img[q] = plan_ok ? 0.f : __builtin_nanf("");   // (own positions only)

  // bit j: tile first + i + 1024 j (below `stop`) lands in the window.  The offsets are fetched
  // sixteen at a time, by loads that depend on no condition (one load under a branch per index
  // would cost a round trip to the L2 each); batches wholly beyond `stop` are skipped.
  auto scan = [&](int first, int stop) -> unsigned long long {
    unsigned long long mask = 0ull;
    constexpr int kBatch = 16;
#pragma unroll
    for (int c = 0; c < kFoldScan / kBatch; c++) {
      if (first + c * kBatch * kFoldThreads >= stop) break;   // (uniform)
      int rel[kBatch];
#pragma unroll
      for (int j = 0; j < kBatch; j++) {
        const int id = first + tid + (c * kBatch + j) * kFoldThreads;
        rel[j] = p.offsets[id < stop ? id : stop - 1];
      }
#pragma unroll
      for (int j = 0; j < kBatch; j++) {
        const int id = first + tid + (c * kBatch + j) * kFoldThreads, r = rel[j] - w0;
        mask |= (unsigned long long)((id < stop) & (r > -E) & (r < wlen)) << (c * kBatch + j);
      }
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

  // The window's tiles are numbered in a fixed order that depends on nothing but the table of
  // offsets: pass by pass of kFoldScan * kFoldThreads tile indices, and inside a pass wavefront by
  // wavefront, thread by thread, bit by bit of the thread's mask.  A share takes an equal part of
  // the numbers, so the workgroups of a window have the same work to within a tile whatever the
  // hash does, and — every share numbering alike — their parts are a partition of the window's tiles.
  const int cap = kFoldList / per_tile;    // tiles whose runs the list holds at a time (at least four)
  // the runs of tile `id`, the at-th tile of the list
  auto put = [&](int at, int id) {
    const int rel = p.offsets[id] - w0;
    const int tk = id / p.tiles_n, tn = id - tk * p.tiles_n;
    const int rows = (p.K - tk * p.h.BK) < p.h.BK ? (p.K - tk * p.h.BK) : p.h.BK;
    const int cols = (p.N - tn * p.h.BN) < p.h.BN ? (p.N - tn * p.h.BN) : p.h.BN;
    for (int s = 0; s < p.slices; s++)
      for (int c = 0; c < runs; c++) {
        const int slot = (at * p.slices + s) * runs + c;
        list_at[slot] = ((s * ntiles + id) << eshift) + c * run;
        list_rel[slot] = rel + c * run;
        list_lim[slot] = (rows - 1) | (cols - 1) << 14 | c << 28;
      }
  };
  auto walk = [&](int total) {
    // --- add the listed runs into the window ---------------------------------------------------
    // Every wavefront on its own: lane u holds entry u of a chunk of 64 list entries; the entries
    // that meet one of the wavefront's blocks are taken in list order, in rounds of kFoldRound;
    // the next round's loads are in flight while this round's values are added.  What describes
    // an entry to the wavefront is uniform (scalar registers).
    struct Round {
      typename FoldRaw<TT>::type v[kFoldRound];   // (as loaded: widened when added, so that the loads stay in flight)
      int pos[kFoldRound];   // window position of the block
      int e0[kFoldRound];    // float of the run that falls on the block's first position (-255 .. run - 1)
      int lim[kFoldRound];   // the entry's, -1: no entry
    };
    unsigned long long todo = 0ull;   // entries of the chunk that this wavefront still has to add
    int next = 0;                     // first list entry behind the chunk
    int c_pos = 0, c_e0 = 0, c_off = 0, c_lim = 0;
    auto refill = [&]() {
      while (todo == 0ull && next < total) {   // (uniform)
        const int t = next + lane;
        const bool have = t < total;
        const int rel = have ? list_rel[t] : 0, at = have ? list_at[t] : 0;
        c_lim = have ? list_lim[t] : 0;
        const int first = rel >> kBlockShift;          // (arithmetic shift: the block of the run's first float)
        const int b = first + ((wave - first) & 15);   // the wavefront's only block among the sixteen from there on
        c_pos = b * kFoldBlock;
        c_e0 = c_pos - rel;
        c_off = at + c_e0;
        todo = __ballot(have && b >= 0 && c_pos < wlen && c_e0 < run);
        next += 64;
      }
    };
    auto issue = [&](Round& r) {
#pragma unroll
      for (int u = 0; u < kFoldRound; u++) {
        const bool any = todo != 0ull;
        const int src = any ? (int)__builtin_ctzll(todo) : 0;
        todo &= todo - 1ull;
        const int off = __builtin_amdgcn_readlane(c_off, src), lim = __builtin_amdgcn_readlane(c_lim, src);
        r.pos[u] = __builtin_amdgcn_readlane(c_pos, src);
        r.e0[u] = __builtin_amdgcn_readlane(c_e0, src);
        r.lim[u] = any ? lim : -1;
        // (every slot loads, an empty one the buffer's first floats: with no branch around the
        //  loads their number is fixed, and the wait for this round's values can leave the next
        //  round's in flight)
        const char* first = reinterpret_cast<const char*>(p.tiles) + (any ? (long long)off : 0ll) * (long long)sizeof(TT);   // (scalar)
        unsigned mine = lane16;   // offset of the lane's elements from the block's first, in bytes
        if (any && (r.e0[u] < 0 || r.e0[u] + kFoldBlock > run)) {   // (uniform) an end of the run:
          // lanes that lie wholly outside the run fetch floats of the run that other lanes fetch
          // anyway (their values count as zero below) instead of a neighbouring tile's
          const int e = r.e0[u] + lane_e;
          const int inside = e <= -kPer ? 0 : (e >= run ? max(run - kPer, r.e0[u]) : e);
          mine = (unsigned)(inside - r.e0[u]) * (unsigned)sizeof(TT);
        }
        // (read once and never again: a load that leaves the caches to the offsets and to the
        //  contraction's stores still on their way to memory — K = N = 10240: 129 -> 111 us)
        r.v[u] = __builtin_nontemporal_load(reinterpret_cast<const typename FoldRaw<TT>::unaligned*>(
            first + mine));
      }
    };
    // (plain read-add-write: LDS float atomics are several times slower, and nobody else touches
    //  this lane's words; runs that overlap are added one after the other, in list order)
    auto add = [&](const Round& r) {
#pragma unroll
      for (int u = 0; u < kFoldRound; u++) {
        if (r.lim[u] == -1) continue;   // (uniform)
        float v[kPer];
        fold_widen<TT>(r.v[u], v);
        const int lim = r.lim[u];
        if (r.e0[u] < 0 || r.e0[u] + kFoldBlock > run) {   // (uniform) an end of the run: what is not the run's counts as zero
          const unsigned e = (unsigned)(r.e0[u] + lane_e);   // (a float before the run wraps round to a large number)
#pragma unroll
          for (int f = 0; f < kPer; f++) v[f] = e + (unsigned)f < (unsigned)run ? v[f] : 0.f;
        }
        if ((lim & 0x0fffffff) != full_lim) {   // (uniform) a tile that sticks out of K x N: what lies outside was never written
          asm volatile("" ::: "memory");   // (keeps this arithmetic out of the common path)
          const int rows = (lim & 0x3fff) + 1, cols = ((lim >> 14) & 0x3fff) + 1, base = (lim >> 28) * run;
#pragma unroll
          for (int f = 0; f < kPer; f++) {
            const int in_tile = base + r.e0[u] + lane_e + f;
            const bool ok = ((in_tile >> p.h.bn_shift) < rows) & ((in_tile & (p.h.BN - 1)) < cols);
            v[f] = ok ? v[f] : 0.f;
          }
        }
        fold_f4* at = reinterpret_cast<fold_f4*>(img + r.pos[u] + lane_e);
#pragma unroll
        for (int g = 0; g < kPer / 4; g++) {
          fold_f4 w = at[g];
#pragma unroll
          for (int f = 0; f < 4; f++) w[f] += v[4 * g + f];
          at[g] = w;
        }
      }
    };
    Round r0, r1;
    refill();
    issue(r0);
    while (true) {   // (uniform per wavefront; no barrier inside)
      refill();
      if (todo == 0ull) {   // (nothing left to load: no round of empty slots, whose loads would still be waited for)
        add(r0);
        break;
      }
      issue(r1);
      add(r0);
      refill();
      if (todo == 0ull) {
        add(r1);
        break;
      }
      issue(r0);
      add(r1);
    }
  };

  if (p.plan_list != nullptr) {
    // The layer plan lists the window's tiles, numbered as below: nothing to look for.
    // (what a plan says is kept inside the plan and inside the table of offsets whatever it holds: a
    //  spoilt plan gives a wrong dHW, never an access out of bounds)
    const int begin = min(max(p.plan_start[win], 0), p.plan_capacity);
    const int all = plan_ok ? min(max(p.plan_start[win + 1], begin), p.plan_capacity) - begin : 0;
    const int want_lo = (int)((long long)share * all / p.shares), want_hi = (int)((long long)(share + 1) * all / p.shares);
    for (int chunk_lo = want_lo; chunk_lo < want_hi; chunk_lo += cap) {   // (uniform)
      const int chunk_hi = (chunk_lo + cap) < want_hi ? (chunk_lo + cap) : want_hi;
      if (chunk_lo != want_lo) __syncthreads();   // (the wavefronts are done reading the previous chunk's list)
      for (int q = chunk_lo + tid; q < chunk_hi; q += kFoldThreads) put(q - chunk_lo, min(max(p.plan_list[begin + q], 0), ntiles - 1));
      __syncthreads();
      walk((chunk_hi - chunk_lo) * per_tile);
    }
  }
  int rank_lo = 0, rank_hi = 0x7fffffff;
  if (p.shares > 1 && p.plan_list == nullptr) {
    int mine = 0, before;
    for (int first = 0; first < ntiles; first += kFoldScan * kFoldThreads) mine += __popcll(scan(first, ntiles));
    const int all = total_of(wave_scan(mine), &before);
    rank_lo = (int)((long long)share * all / p.shares);
    rank_hi = (int)((long long)(share + 1) * all / p.shares);
  }
  int lo = plan_ok && p.plan_list == nullptr ? 0 : ntiles, seen = 0;   // tiles [0, lo) hold `seen` tiles of the window
  while (lo < ntiles && seen < rank_hi) {   // (uniform: every thread of the workgroup goes round together)
    const int span = (ntiles - lo) < kFoldScan * kFoldThreads ? (ntiles - lo) : kFoldScan * kFoldThreads;
    const unsigned long long pass_mask = scan(lo, lo + span);
    const int mine = __popcll(pass_mask);
    const int incl = wave_scan(mine);
    int before;
    const int found = total_of(incl, &before);
    const int first_rank = seen + before + incl - mine;   // of this thread's first tile
    const int want_lo = rank_lo > seen ? rank_lo : seen;
    const int want_hi = rank_hi < seen + found ? rank_hi : seen + found;
    seen += found;
    lo += span;
    // The share's tiles of this pass, `cap` numbers at a time (the numbering does not depend on
    // how many fit the list, so a share that needs several chunks still takes exactly its part).
    for (int chunk_lo = want_lo; chunk_lo < want_hi; chunk_lo += cap) {   // (uniform)
      const int chunk_hi = (chunk_lo + cap) < want_hi ? (chunk_lo + cap) : want_hi;
      const int total = (chunk_hi - chunk_lo) * per_tile;
      if (chunk_lo != want_lo) __syncthreads();   // (the wavefronts are done reading the previous chunk's list)
      unsigned long long mask = pass_mask;
      int rank = first_rank;
      while (mask != 0ull) {
        const int j = __ffsll((long long)mask) - 1;
        mask &= mask - 1ull;
        if (rank >= chunk_lo && rank < chunk_hi) put(rank - chunk_lo, lo - span + tid + j * kFoldThreads);
        rank++;
      }
      __syncthreads();
      walk(total);
    }
  }
  // --- the window of this share's image ---------------------------------------------------------
  __syncthreads();   // (the words below were added up by other threads)
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

// ---- the same sum for a layer of few tiles ------------------------------------------------------
// With a few thousand tiles at most, every workgroup can afford to look at every tile offset, and
// the machinery above (windows in LDS, shares, run lists walked by wavefronts) costs more than it
// saves: a 1024 x 1024 layer has 256 tiles and a hashed_weight of 65536 elements, and its whole
// gradient is a few microseconds of reading.  Here a workgroup of 256 threads owns 256
// consecutive elements of dHW, one per thread; it lists the tiles whose
// slice meets its elements (ascending tile index: two barriers per 1024 tiles) and every thread
// then walks down the list and adds what each tile holds for its element — loads of 64 consecutive
// floats per wavefront, fixed order of additions (tile by tile, slice by slice),
// no atomics, every element of dHW written once.
static constexpr int kFoldSmallThreads = 256;
static constexpr int kFoldSmallTiles = 4096;   // tiles at most: the list in LDS can hold every one of them

template <typename TT>
__global__ __launch_bounds__(kFoldSmallThreads) void fold_small_kernel(const FoldParams p) {
  constexpr int PER = 1;   // elements of dHW per thread
  __shared__ int list_id[kFoldSmallTiles];     // tiles that meet this workgroup's elements, ascending
  __shared__ int list_rel[kFoldSmallTiles];    // ... and where each starts, relative to the first element
  __shared__ int wave_count[kFoldSmallThreads / 64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  constexpr int kSpan = kFoldSmallThreads * PER;
  const int h0 = blockIdx.x * kSpan;
  const int span = (p.H - h0) < kSpan ? (p.H - h0) : kSpan;
  const int E = p.h.BK * p.h.BN, eshift = p.h.bk_shift + p.h.bn_shift;
  const int ntiles = p.tiles_k * p.tiles_n;
  const bool plan_ok = p.plan_header == nullptr || layer_plan_matches(p.plan_header, p.K, p.N, p.H, p.h);   // (uniform)
  // (the offsets are fetched whether or not the header turns out to match — the caller vouches for the plan's
  //  size, so the reads stay inside it — so that the two fetches travel together; a plan that does not
  //  match lists nothing)
  const bool even = p.K % p.h.BK == 0 && p.N % p.h.BN == 0;   // (uniform) every tile lies inside K x N
  int listed = 0;
  for (int first = 0; first < ntiles; first += 4 * kFoldSmallThreads) {
    // thread t looks at the tiles first + 4 t .. first + 4 t + 3 (ascending over the threads)
    int rel[4];
    unsigned hit = 0u;
#pragma unroll
    for (int u = 0; u < 4; u++) {
      const int id = first + 4 * tid + u;
      const int idc = id < ntiles ? id : ntiles - 1;
      // (without a table, the few offsets a thread needs are hashed on the spot)
      rel[u] = (p.offsets != nullptr ? p.offsets[idc] : (int)tile_offset(p.h, (uint32_t)(idc / p.tiles_n), (uint32_t)(idc % p.tiles_n))) - h0;
      hit |= (unsigned)((id < ntiles) & (rel[u] > -E) & (rel[u] < span) & plan_ok) << u;
    }
    const int mine = __popc(hit);
    int incl = mine;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int up = __shfl_up(incl, d, 64);
      if (lane >= d) incl += up;
    }
    __syncthreads();   // (the counts of the previous round have been read)
    if (lane == 63) wave_count[wave] = incl;
    __syncthreads();
    int at = listed + incl - mine;
    for (int w = 0; w < kFoldSmallThreads / 64; w++) {
      const int c = wave_count[w];
      if (w < wave) at += c;
      listed += c;
    }
#pragma unroll
    for (int u = 0; u < 4; u++)
      if ((hit >> u) & 1u) {
        list_id[at] = first + 4 * tid + u;
        list_rel[at] = rel[u];
        at++;
      }
  }
  __syncthreads();
  float acc[PER];
#pragma unroll
  for (int j = 0; j < PER; j++) acc[j] = plan_ok ? 0.f : __builtin_nanf("");
  // The list is taken 32 / PER tiles at a time: all loads of a batch are issued before the first value is
  // used (a load per tile under its own branch would wait out one memory latency after the other: 17
  // tiles took 10 us that way), and the values are added in list order.  A thread that a tile does not
  // reach loads the tile buffer's first float instead and adds zero.
  constexpr int kBatch = 32 / PER;
  for (int e0 = 0; e0 < listed; e0 += kBatch) {   // (uniform)
    unsigned off[kBatch][PER];
    bool ok[kBatch][PER];
#pragma unroll
    for (int u = 0; u < kBatch; u++) {
      const int e = e0 + u < listed ? e0 + u : listed - 1;
      const int id = list_id[e], rel = list_rel[e];
      // rows and columns of the tile inside K x N (what lies beyond was never written)
      int rows = p.h.BK, cols = p.h.BN;
      if (!even) {
        const int tk = id / p.tiles_n, tn = id - tk * p.tiles_n;
        rows = (p.K - tk * p.h.BK) < p.h.BK ? (p.K - tk * p.h.BK) : p.h.BK;
        cols = (p.N - tn * p.h.BN) < p.h.BN ? (p.N - tn * p.h.BN) : p.h.BN;
      }
      const bool whole = rows == p.h.BK && cols == p.h.BN;
#pragma unroll
      for (int j = 0; j < PER; j++) {
        const int x = tid + j * kFoldSmallThreads - rel;   // element of the tile that lands on this thread's j-th element
        ok[u][j] = e0 + u < listed && x >= 0 && x < E && tid + j * kFoldSmallThreads < span &&
                   (whole || ((x >> p.h.bn_shift) < rows && (x & (p.h.BN - 1)) < cols));
        off[u][j] = ok[u][j] ? ((unsigned)id << eshift) + (unsigned)x : 0u;
      }
    }
    for (int sl = 0; sl < p.slices; sl++) {
      const TT* base = reinterpret_cast<const TT*>(p.tiles) + (((size_t)sl * ntiles) << eshift);
      TT v[kBatch][PER];
#pragma unroll
      for (int u = 0; u < kBatch; u++)
#pragma unroll
        for (int j = 0; j < PER; j++) v[u][j] = base[off[u][j]];
#pragma unroll
      for (int u = 0; u < kBatch; u++)
#pragma unroll
        for (int j = 0; j < PER; j++) acc[j] += ok[u][j] ? ElemTraits<TT>::to_float(v[u][j]) : 0.f;
    }
  }
#pragma unroll
  for (int j = 0; j < PER; j++) {
    const int pos = tid + j * kFoldSmallThreads;
    if (pos >= span) continue;
    const int q = h0 + pos;
    if (p.out_dtype == RZ_F32) {
      float* out = reinterpret_cast<float*>(p.out);
      out[q] = acc[j] + (p.accumulate ? out[q] : 0.f);
    } else if (p.out_dtype == RZ_BF16) {
      bf16_t* out = reinterpret_cast<bf16_t*>(p.out);
      out[q] = ElemTraits<bf16_t>::from_float(acc[j] + (p.accumulate ? ElemTraits<bf16_t>::to_float(out[q]) : 0.f));
    } else {
      f16_t* out = reinterpret_cast<f16_t*>(p.out);
      out[q] = ElemTraits<f16_t>::from_float(acc[j] + (p.accumulate ? ElemTraits<f16_t>::to_float(out[q]) : 0.f));
    }
  }
}

}  // namespace rz
