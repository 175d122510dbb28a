// Weight-grad for a hashed_weight too large for one LDS image, with a short contraction
// (small M): every workgroup owns a WINDOW of dHW and pulls in the tiles that touch it.
//
// The scatter kernel adds K*N values into dHW with global atomics, which cost the same
// however small M is (K = N = 10240: 105 M atomics, about 0.57 ms on MI355X, for a product
// that takes microseconds).  Here a workgroup keeps dHW[w0, w0 + window) as an fp32 image in
// LDS, finds the W tiles whose slice [off, off + BK*BN) meets that range by scanning the table
// of tile offsets (hashed into the workspace by a small kernel of the same call) and lists them,
// cut into strips of 32 rows, in ascending order — or, when the caller holds a layer plan, reads
// that list from it (offsets and lists depend on the layer alone).  Then
// every WAVEFRONT takes strips from the list on its own: it computes the whole X^T.dY product
// of a strip — the operands are small and stay in L2; a wavefront fetches its own operand
// pieces (16-bit types: 16-byte pieces through a small LDS area of its own and the LDS
// transpose read; otherwise the MFMA fragments element by element in their register layout),
// so no wavefront waits for another — and adds the part inside the window with plain LDS
// read-add-write.  Slices of different
// tiles may overlap: a tile is added only after every earlier tile of the list whose slice
// meets its own has been added (a flag per list entry, polled in LDS), so the summation order
// of every element is the list order whatever the timing.  Finally the window is stored: every
// element of dHW is written exactly once, with no atomics and no clearing pass.  A tile that
// straddles a window boundary is computed by both neighbours.
#pragma once

#include <type_traits>

#include "rz_gemm.h"
#include "rz_launch.h"

namespace rz {

struct WindowParams {
  const void* X;
  const void* dY;
  void* dHW;
  const int32_t* offsets;   // offset of every W tile, index tk * tiles_n + tn
  // From a layer plan (null: every workgroup finds its strips by scanning `offsets`): the strips
  // that meet window b are entries [plan_start[b], plan_start[b + 1]) of plan_list (tile *
  // strips per tile + strip, ascending) and plan_offs (where each starts in hashed_weight).
  const int32_t* plan_start;
  const int32_t* plan_list;
  const int32_t* plan_offs;
  const int32_t* plan_header;   // shapes, tile, hash (words 2..7, 13) and window (10): checked against this call's
  int M, K, N, H;
  int64_t ldx, lddy;
  float scale;
  HashParams h;
  int window;        // elements of dHW per workgroup (a multiple of 4)
  int tiles_k, tiles_n;
  int accumulate;    // dHW += gradient instead of dHW = gradient
  int out_f32;       // dHW is fp32 whatever T is
  int poll_limit;    // looks at the flags of earlier strips before a wavefront gives up (kWindowPollLimit)
};

// How often a wavefront looks at the flags of the earlier strips it must wait for before it gives
// up.  A look takes at least 64 clocks (the sleep between two), so the limit is some seconds —
// far beyond any real wait (a strip's product takes microseconds) and still an end.
static constexpr int kWindowPollLimit = 1 << 24;

// The hashed tile is BK x TBN: TBN (32, 64 or 128) at compile time — it is the row pitch of a tile's
// slice of hashed_weight — BK (a multiple of 32) at run time.  The unit of work is 32 rows by UC =
// min(TBN, 64) columns of a tile: strip s (rows 32 s .. 32 s + 31) of a 128-column tile is two
// units side by side.  Unit u = s * parts + part of a tile at `off` starts at off + 32 * TBN * s +
// UC * part and its rows are TBN apart: from its first to its last element it spans kUnitSpan =
// 31 * TBN + UC elements (all of them its own when the tile is no wider than 64).  A wavefront
// holds the unit's 32x32 blocks in registers.
// STAGED (K and N multiples of the 16-byte piece): operands travel as 16-byte pieces through the
// wavefront's staging area (a quarter of the load instructions per byte for fp32, an eighth for the
// 16-bit types); otherwise fragments are loaded element by element.
template <typename T, int TBN, bool STAGED>
struct WindowKernel {
  static_assert(TBN == 32 || TBN == 64 || TBN == 128, "tiles of 32, 64 or 128 columns");
  typedef ElemTraits<T> Tr;
  typedef typename Mfma<T>::Frag Frag;
  static constexpr int kThreads = 1024;
  static constexpr int kWaves = kThreads / 64;
  static constexpr int UC = TBN < 64 ? TBN : 64;         // columns of a unit
  static constexpr int kParts = TBN / UC;                // units side by side in a strip of a tile
  static constexpr int kUnitSpan = 31 * TBN + UC;        // elements of hashed_weight from a unit's first to its last
  static constexpr int kMaxUnits = 16;                   // units of a tile at most (BK <= 256)
  static constexpr int BI = 1, BJ = UC / 32;             // blocks of a unit
  static constexpr int KS = Tr::kMfmaK;                  // rows of M one MFMA contracts (16 or 2)
  // rows of M loaded ahead as one group (16 wavefronts per compute unit leave 128 registers each)
  static constexpr int kGroupRows = sizeof(T) == 4 ? 8 : 16;
  static constexpr int GS = kGroupRows / KS;             // MFMA steps per group
  static constexpr int kBatch = STAGED ? 8 : 4;           // tile offsets a lane loads at a time
  // Items (one group of rows of one strip) whose operand loads are in flight while one is being
  // multiplied, plus that one: a ring of register sets.  An item is a few loads and a few MFMAs,
  // so a wavefront's rate is (items in flight) / (memory latency).
  static constexpr int kDepth = (STAGED || sizeof(T) == 4) ? 3 : 2;
  static constexpr bool k16 = sizeof(T) == 2;
  // staged: a wavefront's own staging area, one group of rows of X (32 columns) and of dY (TBN
  // columns), 3 KB; the list is kept shorter to make room for it next to the window
  static constexpr int VEC = Tr::kVec;                   // elements of a 16-byte piece
  static constexpr int kStageX = kGroupRows * 32, kStageElems = STAGED ? kStageX + kGroupRows * UC : 8;
  static constexpr int kList = 960;   // capacity of the list of units found
  static_assert(!STAGED || (64 * VEC == kGroupRows * 32), "one piece of X and BJ of dY per lane and group");

  struct Smem {
    int list[kList];              // units found in this pass (tile id * units per tile + unit), ascending
    int offs[kList];              // ... their offsets in hashed_weight
    int done[kList];              // ... and whether they have been added to the window
    int count[2][kWaves];
    int spoilt;                   // a wavefront gave up waiting for an earlier strip: the window is stored as NaN
    alignas(16) T stage[kWaves][kStageElems];
    alignas(16) float window[4];  // the image of dHW[w0, w0 + window) starts here, then 64
                                  // dump slots
  };
  static constexpr size_t kFixedBytes = offsetof(Smem, window) + sizeof(float) * 64;   // + dump slots

  // MFMA fragment of a 32-wide block of a row-major matrix (rows = the contracted dimension M).
  //   16-bit: lane l holds rows m0 + r0 + (l >> 5) * 8 + j, j = 0..7, of column (l & 31)
  //   fp32  : lane l holds row m0 + r0 + (l >> 5) of column (l & 31)
  // `rows` points at row m0 (a row of the matrix) and the first column of the strip (clamped into
  // the matrix); `lane_col` is the lane's column inside the strip, or 0 with col_ok = false when
  // that column lies outside the matrix.  whole = every row of the group exists, the usual
  // case.  Whatever is outside reads an element inside the matrix instead and is replaced by zero.
  static __device__ __forceinline__ Frag load_frag(const T* __restrict__ rows, int64_t ld, int r0, int m0, int M,
                                                   int lane, int lane_col, bool col_ok, bool whole) {
    const int mg = lane >> 5;
    if constexpr (sizeof(T) == 4) {
      const bool ok = col_ok && (whole || m0 + r0 + mg < M);
      const float v = reinterpret_cast<const float*>(rows)[ok ? (uint32_t)((r0 + mg) * (int)ld + lane_col) : 0u];
      return ok ? v : 0.f;
    } else {
      const uint16_t* r16 = reinterpret_cast<const uint16_t*>(rows);
      u32x4_t f = {0u, 0u, 0u, 0u};
      if (whole) {
        // the rows j are a uniform distance apart: uniform base per row, one lane offset
        // (a lane outside the matrix has lane_col = 0: it reads the strip's first column)
        const uint32_t off = (uint32_t)(mg * 8 * (int)ld + lane_col);
#pragma unroll
        for (int j = 0; j < 8; j++) {
          const uint32_t v = (r16 + (int64_t)(r0 + j) * ld)[off];
          f[j >> 1] |= (col_ok ? v : 0u) << (16 * (j & 1));
        }
      } else {
#pragma unroll
        for (int j = 0; j < 8; j++) {
          const bool ok = col_ok && (m0 + r0 + mg * 8 + j < M);
          const uint32_t v = r16[ok ? (uint32_t)((r0 + mg * 8 + j) * (int)ld + lane_col) : 0u];
          f[j >> 1] |= (ok ? v : 0u) << (16 * (j & 1));
        }
      }
      return f;
    }
  }

  static __device__ void run(const WindowParams& p, Smem& sm) {
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    float* __restrict__ win = sm.window;
    const long long w0 = (long long)blockIdx.x * p.window;
    const int wlen = (p.H - w0) < p.window ? (int)(p.H - w0) : p.window;
    const T* __restrict__ gX = static_cast<const T*>(p.X);
    const T* __restrict__ gdY = static_cast<const T*>(p.dY);

    for (int i = tid * 4; i < p.window; i += kThreads * 4) {
      const float4 z = {0.f, 0.f, 0.f, 0.f};
      *reinterpret_cast<float4*>(win + i) = z;
    }
    if (tid == 0) sm.spoilt = 0;   // (read after the barriers of the rounds below)

    const int total = p.tiles_k * p.tiles_n;
    const int ngroups = (p.M + kGroupRows - 1) / kGroupRows;
    const int units = (p.h.BK >> 5) * kParts;               // units of a tile (a power of two, at most kMaxUnits)
    const int ushift = __builtin_ctz(units);

    f32x16_t acc[BI][BJ];
#pragma unroll
    for (int a = 0; a < BI; a++)
#pragma unroll
      for (int b = 0; b < BJ; b++)
#pragma unroll
        for (int e = 0; e < 16; e++) acc[a][b][e] = 0.f;
    // kDepth register sets: the fragments of the next groups are loaded while this one is multiplied
    Frag fa[kDepth][GS][BI], fb[kDepth][GS][BJ];
    // 16-bit staged path: the raw 16-byte pieces instead (one of X, two of dY per lane and group)
    u32x4_t px[kDepth], py[kDepth][BJ];
    // element offset of this lane's piece of X, and of its BJ pieces of dY, from the first row of a group
    const int lane_x = STAGED ? (lane / (32 / VEC)) * (int)p.ldx + (lane % (32 / VEC)) * VEC : 0;
    int lane_y[BJ];
#pragma unroll
    for (int q = 0; q < BJ; q++)
      lane_y[q] = STAGED ? (lane / (UC / VEC) + q * (64 / (UC / VEC))) * (int)p.lddy + (lane % (UC / VEC)) * VEC : 0;

    // Listing the units that meet the window, in ascending (tile, unit) order.  The tile ids of
    // a range [lo, hi) are dealt to the wavefronts in contiguous chunks; every wavefront first
    // counts the units of its chunk that meet the window, the counts are added up (one
    // barrier), then it examines its chunk again and writes its units behind those of the
    // wavefronts before it.  Normally the range is the whole table and the list (kList entries)
    // takes every hit; if it would overflow, the range is halved until its hits fit, and the
    // rest of the table follows in further rounds.  (A range of one tile has at most kMaxUnits
    // hits, so the halving ends.)
    auto unit_start = [&](int off, int u) -> long long {
      return (long long)off + (long long)(u / kParts) * (32 * TBN) + (u % kParts) * UC;
    };
    auto units_of = [&](int id, int off) -> unsigned {
      // bit u: unit u of tile id meets the window (id < 0: no tile)
      unsigned hits = 0u;
      for (int u = 0; u < units; u++) {   // (uniform)
        const long long so = unit_start(off, u);
        hits |= (unsigned)(id >= 0 && so < w0 + wlen && so + kUnitSpan > w0) << u;
      }
      return hits;
    };
    auto wave_sum = [&](int v) -> int {
#pragma unroll
      for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d, 64);
      return v;
    };
    const bool planned = p.plan_start != nullptr;   // (uniform)
    if (planned) {
      // A plan built for another layer would send the loads below anywhere: refuse it, loudly
      // (the window of dHW becomes NaN), instead of reading outside X and dY.
      const int32_t* hd = p.plan_header;
      if (!layer_plan_matches(hd, p.K, p.N, p.H, p.h) || hd[6] != TBN || hd[10] != p.window || hd[12] != units) {
        const float nan = __builtin_nanf("");
        if (p.out_f32 || sizeof(T) == 4) {
          for (int i = tid; i < wlen; i += kThreads) (static_cast<float*>(p.dHW) + w0)[i] = nan;
        } else {
          for (int i = tid; i < wlen; i += kThreads) (static_cast<T*>(p.dHW) + w0)[i] = Tr::from_float(nan);
        }
        return;
      }
    }
    // (what a plan says is kept inside the plan, the tiles and hashed_weight whatever it holds: a spoilt plan
    //  gives a wrong dHW, never an access out of bounds)
    const int plan_entries = planned ? p.plan_header[11] : 0;
    const int plan_lo = planned ? min(max(p.plan_start[blockIdx.x], 0), plan_entries) : 0;
    const int plan_n = planned ? min(max(p.plan_start[blockIdx.x + 1], plan_lo), plan_entries) - plan_lo : 0;
    const int list_total = planned ? plan_n : total;   // what the rounds below work through: entries, or tile ids
    int lo = 0;
    while (lo < list_total) {
      int hi = total, found = 0, chunk = 0;
      if (planned) {
        // the next kList entries of this window's precomputed list (same order as the scan finds them)
        found = plan_n - lo < kList ? plan_n - lo : kList;
        __syncthreads();   // (the previous round's list is no longer read)
        for (int i = tid; i < found; i += kThreads) {
          sm.list[i] = min(max(p.plan_list[plan_lo + lo + i], 0), (total << ushift) - 1);
          sm.offs[i] = min(max(p.plan_offs[plan_lo + lo + i], 0), p.H - 1);
          sm.done[i] = 0;
        }
        hi = lo + found;
      } else {
        for (;;) {
          chunk = (hi - lo + kWaves - 1) / kWaves;
          const int begin = lo + wave * chunk, end = begin + chunk < hi ? begin + chunk : hi;
          int mine = 0;
          for (int id0 = begin; id0 < end; id0 += 64 * kBatch) {
            // a lane's next kBatch offsets are loaded together (one memory latency, not kBatch)
            int offv[kBatch];
  #pragma unroll
            for (int u = 0; u < kBatch; u++) {
              const int id = id0 + u * 64 + lane;
              offv[u] = id < end ? p.offsets[id] : 0;
            }
  #pragma unroll
            for (int u = 0; u < kBatch; u++) {
              const int id = id0 + u * 64 + lane;
              mine += __popc(units_of(id < end ? id : -1, offv[u]));
            }
          }
          mine = wave_sum(mine);
          __syncthreads();   // (the counts of the previous attempt or round have been read)
          if (lane == 0) sm.count[0][wave] = mine;
          __syncthreads();
          found = 0;
  #pragma unroll
          for (int w = 0; w < kWaves; w++) found += __builtin_amdgcn_readfirstlane(sm.count[0][w]);
          if (found <= kList) break;
          hi = lo + (hi - lo) / 2;   // (found > kList >= kMaxUnits, so the range holds at least two tiles)
        }
        {
          int at = 0;
  #pragma unroll
          for (int w = 0; w < kWaves; w++) at += (w < wave) ? __builtin_amdgcn_readfirstlane(sm.count[0][w]) : 0;
          const int begin = lo + wave * chunk, end = begin + chunk < hi ? begin + chunk : hi;
          for (int id0 = begin; id0 < end; id0 += 64 * kBatch) {
            int offv[kBatch];
  #pragma unroll
            for (int u = 0; u < kBatch; u++) {
              const int id = id0 + u * 64 + lane;
              offv[u] = id < end ? p.offsets[id] : 0;
            }
  #pragma unroll
            for (int u = 0; u < kBatch; u++) {
              const int id = id0 + u * 64 + lane;
              unsigned hits = units_of(id < end ? id : -1, offv[u]);
              // the units of the lanes below me (tiles with smaller ids), then my own in order
              const int c = __popc(hits);
              int incl = c;
  #pragma unroll
              for (int d = 1; d < 64; d <<= 1) {
                const int up = __shfl_up(incl, d, 64);
                if (lane >= d) incl += up;
              }
              int mine = at + incl - c;
              while (hits != 0u) {
                const int un = __builtin_ctz(hits);
                hits &= hits - 1u;
                sm.list[mine] = (id << ushift) + un;
                sm.offs[mine] = (int)unit_start(offv[u], un);
                sm.done[mine] = 0;
                mine++;
              }
              at += __shfl(incl, 63, 64);
            }
          }
        }
      }
      lo = hi;
      __syncthreads();   // list complete, flags cleared

      // ---- every wavefront works through list entries wave, wave + kWaves, ... on its own ----
      // An item is one group of rows of M of one tile.  No barrier in here: a wavefront that
      // waits for an earlier tile's flag must never be waited for by the owner of that tile.
      const int my_tiles = found > wave ? (found - wave + kWaves - 1) / kWaves : 0;
      const int items = my_tiles * ngroups;
      int ft = 0, fg = 0;      // tile ordinal and group of the next item to load
      // The loads of an item are issued unconditionally, in straight-line code: the compiler
      // counts outstanding loads along every path, and a fetch under a branch would make it wait
      // for ALL loads at the first use behind the join — the item just requested included.
      // Beyond the wavefront's last item the last strip is fetched again (valid addresses, in
      // cache; what arrives is multiplied into accumulators that nobody reads any more).
      // Staged form: what a fetch needs of its strip is worked out once per strip and kept in
      // scalar registers (the strip's first column in X and in dY, whether all its columns
      // exist), and what it needs of the lane once per kernel (lane_x / lane_y: element
      // offset of the lane's piece from the group's first row); an item then costs two scalar
      // multiply-adds and three loads with a uniform base.  Only groups with rows beyond M and
      // strips at the edge of the matrix take the path with per-lane checks.
      // (offsets, not pointers: a pointer carried round the loop would lose its address space
      //  and turn the loads into flat ones, which also count as LDS traffic)
      int strip_x = 0, strip_k0 = 0, strip_n0 = 0;
      bool strip_whole = false;
      // which of a lane's pieces of the group at row m0 of the unit at (k0, n0) lie inside the matrices
      auto pieces_inside = [&](int m0, int k0, int n0, bool& okx, bool (&oky)[BJ]) {
        constexpr int PX = 32 / VEC, PY = UC / VEC;
        okx = m0 + lane / PX < p.M && k0 + (lane % PX) * VEC < p.K;
        const bool col_ok = n0 + (lane % PY) * VEC < p.N;
#pragma unroll
        for (int q = 0; q < BJ; q++) oky[q] = m0 + lane / PY + q * (64 / PY) < p.M && col_ok;
      };
      // ... and the same for the strip being multiplied
      int mult_k0 = 0, mult_n0 = 0;
      bool mult_whole = false;
      auto fetch_next = [&](auto set) {
        constexpr int S = decltype(set)::value;
        if constexpr (STAGED) {
          if (fg == 0) {   // (uniform) a new strip
            const int ftc = ft < my_tiles ? ft : my_tiles - 1;
            const int v = __builtin_amdgcn_readfirstlane(sm.list[wave + ftc * kWaves]);
            const int id = v >> ushift, un = v & (units - 1);
            const int tk = id / p.tiles_n, tn = id - tk * p.tiles_n;
            strip_k0 = tk * p.h.BK + (un / kParts) * 32;   // the unit's first row of W
            strip_n0 = tn * TBN + (un % kParts) * UC;      // ... and first column
            strip_whole = strip_k0 + 32 <= p.K && strip_n0 + UC <= p.N;
            // (a strip that begins beyond K contributes nothing; its base is kept inside the matrix)
            strip_x = strip_k0 < p.K ? strip_k0 : p.K - 1;
          }
          const int m0 = fg * kGroupRows;
          const T* rows_x = gX + ((int64_t)m0 * p.ldx + strip_x);
          const T* rows_y = gdY + ((int64_t)m0 * p.lddy + strip_n0);
          const T* src_x = rows_x + lane_x;
          const T* src_y[BJ];
#pragma unroll
          for (int q = 0; q < BJ; q++) src_y[q] = rows_y + lane_y[q];
          if (!(strip_whole && m0 + kGroupRows <= p.M)) {   // (uniform, rare)
            // a piece outside the matrix is fetched from inside it (and replaced by zero when the
            // item is multiplied, where the same checks are made again: nothing about a set is
            // carried round the ring but its data)
            // (the empty statement keeps this block out of the usual path: its arithmetic would
            //  otherwise be carried out for every item and thrown away)
            asm volatile("" ::: "memory");
            bool okx, oky[BJ];
            pieces_inside(m0, strip_k0, strip_n0, okx, oky);
            src_x = okx ? src_x : gX + (int64_t)m0 * p.ldx;
#pragma unroll
            for (int q = 0; q < BJ; q++) src_y[q] = oky[q] ? src_y[q] : gdY + (int64_t)m0 * p.lddy;
          }
          __builtin_memcpy(&px[S], src_x, 16);
#pragma unroll
          for (int q = 0; q < BJ; q++) __builtin_memcpy(&py[S][q], src_y[q], 16);
          if (++fg == ngroups) {
            fg = 0;
            ft++;
          }
          return;
        }
        {
          const int ftc = ft < my_tiles ? ft : my_tiles - 1;
          const int v = __builtin_amdgcn_readfirstlane(sm.list[wave + ftc * kWaves]);
          const int id = v >> ushift, un = v & (units - 1);
          const int tk = id / p.tiles_n, tn = id - tk * p.tiles_n;
          const int k0 = tk * p.h.BK + (un / kParts) * 32;   // the unit's first row of W
          const int n0 = tn * TBN + (un % kParts) * UC;      // ... and first column
          const int m0 = fg * kGroupRows;
          const bool whole = m0 + kGroupRows <= p.M;
          // (a strip that begins beyond K contributes nothing; its base is kept inside the matrix)
          const T* rows_x = gX + (int64_t)m0 * p.ldx + (int64_t)(k0 < p.K ? k0 : p.K - 1);
          const T* rows_y = gdY + (int64_t)m0 * p.lddy + (int64_t)(n0 < p.N ? n0 : p.N - 1);
#pragma unroll
          for (int a = 0; a < BI; a++) {
            const int col = a * 32 + (lane & 31);
            const bool ok = k0 + col < p.K;
#pragma unroll
            for (int s = 0; s < GS; s++)
              fa[S][s][a] = load_frag(rows_x, p.ldx, s * KS, m0, p.M, lane, ok ? col : 0, ok, whole);
          }
#pragma unroll
          for (int b = 0; b < BJ; b++) {
            const int col = b * 32 + (lane & 31);
            const bool ok = n0 + col < p.N;
#pragma unroll
            for (int s = 0; s < GS; s++)
              fb[S][s][b] = load_frag(rows_y, p.lddy, s * KS, m0, p.M, lane, ok ? col : 0, ok, whole);
          }
          if (++fg == ngroups) {
            fg = 0;
            ft++;
          }
        }
      };
      // add the finished strip of list entry `e` into the window, after the earlier strips whose
      // slices meet its own, and raise its flag
      auto add_tile = [&](int e) {
        const int tile_off = __builtin_amdgcn_readfirstlane(sm.offs[e]);
        // lane l looks at the earlier entries l, l + 64, ...: straight-line LDS reads, no branches.
        // The wait is bounded: an entry only waits for earlier ones, whose owners wait for still
        // earlier ones, so it ends by itself; should a flag never come all the same (a list that
        // is not what this kernel expects), the wavefront gives up after kPollLimit looks, marks
        // the window as spoilt and goes on, so that every wavefront reaches the end of the kernel.
        for (int polls = 0;; polls++) {
          bool pending = false;
          for (int f = lane; f < e; f += 64) {
            const int d = sm.offs[f] - tile_off;
            const int dn = __hip_atomic_load(&sm.done[f], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            pending |= (d < kUnitSpan) & (d > -kUnitSpan) & (dn == 0);
          }
          if (!__any(pending)) break;
          if (polls >= p.poll_limit) {   // (uniform)
            if (lane == 0) __hip_atomic_store(&sm.spoilt, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            break;
          }
          __builtin_amdgcn_s_sleep(1);
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        const int rel = (int)((long long)tile_off - w0);   // (offsets and window starts are below 2^31)
        if (rel >= 0 && rel + kUnitSpan <= wlen) {
          // the whole unit lies inside the window (the usual case): no checks, constant offsets
#pragma unroll
          for (int b = 0; b < BJ; b++) {
            float* at = win + rel + ((lane >> 5) * 4) * TBN + b * 32 + (lane & 31);
            // (eight elements at a time: 16 wavefronts per compute unit leave few registers)
#pragma unroll
            for (int half = 0; half < 2; half++) {
              float cur[8];
#pragma unroll
              for (int q = 0; q < 8; q++) {
                const int i = half * 8 + q;
                cur[q] = at[((i >> 2) * 8 + (i & 3)) * TBN];
              }
#pragma unroll
              for (int q = 0; q < 8; q++) {
                const int i = half * 8 + q;
                at[((i >> 2) * 8 + (i & 3)) * TBN] = cur[q] + acc[0][b][i] * p.scale;
                acc[0][b][i] = 0.f;
              }
            }
          }
        } else {
          // elements outside the window go to a dump slot behind it: no branches, so the reads
          // and the writes of a block go out back to back (the addresses of a lane are distinct;
          // the dump slots are shared between wavefronts, their contents are never used)
          const int dump = p.window + lane;
#pragma unroll
          for (int b = 0; b < BJ; b++) {
            const int base = rel + ((lane >> 5) * 4) * TBN + b * 32 + (lane & 31);
            // (eight elements at a time: 16 wavefronts per compute unit leave few registers)
#pragma unroll
            for (int half = 0; half < 2; half++) {
              int at[8];
              float cur[8];
#pragma unroll
              for (int q = 0; q < 8; q++) {
                const int i = half * 8 + q;
                const int x = base + ((i >> 2) * 8 + (i & 3)) * TBN;
                at[q] = (x >= 0 && x < wlen) ? x : dump;
                cur[q] = win[at[q]];
              }
#pragma unroll
              for (int q = 0; q < 8; q++) {
                const int i = half * 8 + q;
                win[at[q]] = cur[q] + acc[0][b][i] * p.scale;
                acc[0][b][i] = 0.f;
              }
            }
          }
        }
        if (lane == 0) __hip_atomic_store(&sm.done[e], 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
      };
      int pt = 0, pg = 0;      // tile ordinal and group of the item being multiplied
      auto item = [&](auto set) {
        constexpr int S = decltype(set)::value;
        // the set freed by the previous item takes the loads of the item kDepth - 1 ahead
        fetch_next(std::integral_constant<int, (S + kDepth - 1) % kDepth>{});
        if constexpr (STAGED) {
          {
            // pieces -> this wavefront's staging area (LDS operations of one wavefront are carried
            // out in order, so neither the reads below nor the next group's writes need a barrier)
            T* st = sm.stage[wave];
            const u32x4_t z = {0u, 0u, 0u, 0u};
            constexpr int PX = 32 / VEC, PY = UC / VEC;
            // (pieces outside the matrix become zero; the usual set has none: a uniform branch, no selects)
            u32x4_t wx = px[S], wy[BJ];
#pragma unroll
            for (int q = 0; q < BJ; q++) wy[q] = py[S][q];
            if (pg == 0) {   // (uniform) a new unit
              const int ptc = pt < my_tiles ? pt : my_tiles - 1;
              const int v = __builtin_amdgcn_readfirstlane(sm.list[wave + ptc * kWaves]);
              const int id = v >> ushift, un = v & (units - 1), tk = id / p.tiles_n;
              mult_k0 = tk * p.h.BK + (un / kParts) * 32;
              mult_n0 = (id - tk * p.tiles_n) * TBN + (un % kParts) * UC;
              mult_whole = mult_k0 + 32 <= p.K && mult_n0 + UC <= p.N;
            }
            if (!(mult_whole && (pg + 1) * kGroupRows <= p.M)) {
              asm volatile("" ::: "memory");
              bool okx, oky[BJ];
              pieces_inside(pg * kGroupRows, mult_k0, mult_n0, okx, oky);
              wx = okx ? wx : z;
#pragma unroll
              for (int q = 0; q < BJ; q++) wy[q] = oky[q] ? wy[q] : z;
            }
            *reinterpret_cast<u32x4_t*>(st + (lane / PX) * 32 + (lane % PX) * VEC) = wx;
            if constexpr (k16) {
#pragma unroll
              for (int q = 0; q < BJ; q++) {
                const int r = lane / PY + (64 / PY) * q, pc = lane % PY;
                // 64-column units: dY rows are two 64-byte chunks, swapped in every other pair of rows, so
                // that the four rows of a transpose read fall on different banks; 32-column units lie as X does
                if constexpr (UC == 64)
                  *reinterpret_cast<u32x4_t*>(st + kStageX + r * UC + ((((pc >> 2) ^ ((r >> 1) & 1)) << 5) | ((pc & 3) << 3))) = wy[q];
                else
                  *reinterpret_cast<u32x4_t*>(st + kStageX + r * UC + pc * VEC) = wy[q];
              }
              // fragments by the LDS transpose read: within 16 lanes, lane c receives column c of a
              // 4 x 16 block whose rows the lanes address four-per-row
              typedef s16x4_t __attribute__((address_space(3))) * lds_s16x4_ptr;
              const int g = lane >> 4, jl = lane & 15;
              const int row = 8 * (g >> 1) + (jl >> 2), col = 16 * (g & 1) + 4 * (jl & 3);
              auto tr_frag = [&](const T* at, int pitch) -> Frag {
                const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(at));
                const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(at + 4 * pitch));
                const u32x2_t l2 = __builtin_bit_cast(u32x2_t, lo), h2 = __builtin_bit_cast(u32x2_t, hi);
                u32x4_t f = {l2[0], l2[1], h2[0], h2[1]};
                return f;
              };
              const Frag a = tr_frag(st + row * 32 + col, 32);
              Frag b[BJ];
#pragma unroll
              for (int j = 0; j < BJ; j++)
                b[j] = UC == 64 ? tr_frag(st + kStageX + row * UC + (((j ^ ((row >> 1) & 1)) << 5) | col), UC)
                                : tr_frag(st + kStageX + row * UC + col, UC);
#pragma unroll
              for (int j = 0; j < BJ; j++) acc[0][j] = Mfma<T>::run(a, b[j], acc[0][j]);
            } else {
              // fp32: the two 128-byte halves of a dY row are swapped in every other row, so that the
              // two rows of an MFMA step (lanes 0-31 and 32-63) lie on different banks
#pragma unroll
              for (int q = 0; q < BJ; q++) {
                const int r = lane / PY + (64 / PY) * q, c = (lane % PY) * VEC;
                *reinterpret_cast<u32x4_t*>(st + kStageX + r * UC + (UC == 64 ? (c ^ ((r & 1) << 5)) : c)) = wy[q];
              }
              // fragments: lane l holds row 2 s + (l >> 5), column l & 31 of the block
              const int mg = lane >> 5, cl = lane & 31;
              Frag a[GS], b[GS][BJ];
#pragma unroll
              for (int g = 0; g < GS; g++) {
                a[g] = st[(2 * g + mg) * 32 + cl];
#pragma unroll
                for (int j = 0; j < BJ; j++) b[g][j] = st[kStageX + (2 * g + mg) * UC + (UC == 64 ? (((j ^ mg) << 5) | cl) : cl)];
              }
#pragma unroll
              for (int g = 0; g < GS; g++)
#pragma unroll
                for (int j = 0; j < BJ; j++) acc[0][j] = Mfma<T>::run(a[g], b[g][j], acc[0][j]);
            }
            if (pt < my_tiles && ++pg == ngroups) {
              add_tile(wave + pt * kWaves);
              pg = 0;
              pt++;
            }
            return;
          }
        }
#pragma unroll
        for (int s = 0; s < GS; s++)
#pragma unroll
          for (int a = 0; a < BI; a++)
#pragma unroll
            for (int b = 0; b < BJ; b++) acc[a][b] = Mfma<T>::run(fa[S][s][a], fb[S][s][b], acc[a][b]);
        if (pt < my_tiles && ++pg == ngroups) {
          add_tile(wave + pt * kWaves);
          pg = 0;
          pt++;
        }
      };
      if (my_tiles > 0) {
        // whole turns of the ring: the up to kDepth - 1 items past the end are padding (see fetch_next)
        static_assert(kDepth >= 2 && kDepth <= 8, "the ring below is written out for up to eight sets");
        auto each_set = [&](auto&& f, auto count) {   // f(0), ..., f(count - 1) with compile-time arguments
          constexpr int C = decltype(count)::value;
          f(std::integral_constant<int, 0>{});
          if constexpr (C > 1) f(std::integral_constant<int, 1>{});
          if constexpr (C > 2) f(std::integral_constant<int, 2>{});
          if constexpr (C > 3) f(std::integral_constant<int, 3>{});
          if constexpr (C > 4) f(std::integral_constant<int, 4>{});
          if constexpr (C > 5) f(std::integral_constant<int, 5>{});
          if constexpr (C > 6) f(std::integral_constant<int, 6>{});
          if constexpr (C > 7) f(std::integral_constant<int, 7>{});
        };
        each_set(fetch_next, std::integral_constant<int, kDepth - 1>{});
        for (int i = 0; i < items; i += kDepth) each_set(item, std::integral_constant<int, kDepth>{});
        // (the padding items have left rubbish in the accumulators)
#pragma unroll
        for (int a = 0; a < BI; a++)
#pragma unroll
          for (int b = 0; b < BJ; b++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[a][b][e] = 0.f;
      }
      __syncthreads();   // every strip of the list has been added
    }

    // store the window: dHW[w0 + i] (+)= image[i], each element exactly once
    __syncthreads();   // (a window that no strip meets has passed no barrier since it was cleared)
    if (sm.spoilt) {   // (uniform) the order of the adds was not kept: say so in the result
      const float nan = __builtin_nanf("");
      for (int i = tid; i < wlen; i += kThreads) win[i] = nan;
      __syncthreads();
    }
    if (p.out_f32 || sizeof(T) == 4) {
      float* out = static_cast<float*>(p.dHW) + w0;
      for (int i = tid; i < wlen; i += kThreads) out[i] = win[i] + (p.accumulate ? out[i] : 0.f);
    } else {
      T* out = static_cast<T*>(p.dHW) + w0;
      for (int i = tid; i < wlen; i += kThreads)
        out[i] = Tr::from_float(win[i] + (p.accumulate ? Tr::to_float(out[i]) : 0.f));
    }
  }
};

template <typename T, int TBN, bool STAGED>
__global__ __launch_bounds__((WindowKernel<T, TBN, STAGED>::kThreads)) void rz_window_kernel(WindowParams p) {
  typedef WindowKernel<T, TBN, STAGED> K;
  extern __shared__ __attribute__((aligned(16))) unsigned char rz_window_smem[];
  K::run(p, *reinterpret_cast<typename K::Smem*>(rz_window_smem));
}

}  // namespace rz
