// Weight-grad for a hashed_weight too large for one LDS image, with a short contraction
// (small M): every workgroup owns a WINDOW of dHW and pulls in the tiles that touch it.
//
// The scatter kernel adds K*N values into dHW with global atomics, which cost the same
// however small M is (K = N = 10240: 105 M atomics, about 0.57 ms on MI355X, for a product
// that takes microseconds).  Here a workgroup keeps dHW[w0, w0 + window) as an fp32 image in
// LDS, finds the W tiles whose slice [off, off + BK*BN) meets that range by scanning the table
// of tile offsets (hashed into the workspace by a small kernel of the same call; nothing is
// kept between calls), computes each such tile's
// X^T.dY product — operands are small and stay in L2 — and adds the part inside the window
// with plain LDS read-add-write; barriers separate the adds of different tiles, whose slices
// may overlap.  Finally the window is stored: every element of dHW is written exactly once, in
// a fixed summation order (ascending tile id), with no atomics and no clearing pass.  A tile
// that straddles a window boundary is computed by both neighbours.
#pragma once

#include "rz_gemm.h"

namespace rz {

struct WindowParams {
  const void* X;
  const void* dY;
  void* dHW;
  const int32_t* offsets;   // offset of every W tile, index tk * tiles_n + tn
  int M, K, N, H;
  int64_t ldx, lddy;
  float scale;
  HashParams h;
  int window;        // elements of dHW per workgroup (a multiple of 4)
  int tiles_k, tiles_n;
  int accumulate;    // dHW += gradient instead of dHW = gradient
  int out_f32;       // dHW is fp32 whatever T is
};

// TBK x TBN is the hashed tile (compile time).  A workgroup is kTeams teams of one wavefront
// per 32x32 block of a tile.  The teams multiply different tiles at the same time (several
// wavefronts per SIMD hide each other's latencies) and then add them into the window one
// team after the other, in list order.
template <typename T, int TBK, int TBN>
struct WindowKernel {
  // the operand staging (padded LDS layouts, transpose reads) of the contraction kernel
  typedef GemmKernel<T, kWeightGrad, TBK, TBN, TBK / 32, TBN / 32, 1, false> G;
  typedef typename G::LA LA;
  typedef typename G::LB LB;
  typedef typename Mfma<T>::Frag Frag;
  static constexpr int kTeamThreads = G::kThreads;
  static constexpr int kTeams = sizeof(T) == 4 ? 2 : 4;
  static constexpr int kThreads = kTeamThreads * kTeams;
  static constexpr int kWaves = kThreads / 64;
  static constexpr int VEC = G::VEC;
  static constexpr int kRows = 32;                 // rows of M per staged chunk
  static constexpr int kPiecesA = kRows * LA::kCpr / kTeamThreads;
  static constexpr int kPiecesB = kRows * LB::kCpr / kTeamThreads;
  static_assert(kRows * LA::kCpr % kTeamThreads == 0 && kRows * LB::kCpr % kTeamThreads == 0, "chunk must split evenly");
  static_assert(kRows % G::KS == 0 && kRows <= G::TR, "chunk rows must suit the fragment reads");
  static constexpr int kList = kThreads;           // capacity of the list of tiles found
  static constexpr int kBatch = 8;                 // tile offsets a thread loads at a time

  struct Smem {
    alignas(16) T a[kTeams][kRows * LA::kPitch];
    alignas(16) T b[kTeams][kRows * LB::kPitch];
    int list[kList];              // ids of the tiles found in this pass, ascending
    int offs[kList];              // ... and their offsets in hashed_weight
    int count[2][kWaves];
    alignas(16) float window[4];  // the image of dHW[w0, w0 + window) starts here, then 64
                                  // dump slots
  };
  static constexpr size_t kFixedBytes = offsetof(Smem, window) + sizeof(float) * 64;   // + dump slots

  static __device__ void run(const WindowParams& p, Smem& sm) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int team = wave / (kTeamThreads / 64), ttid = tid % kTeamThreads;
    const int twave = wave % (kTeamThreads / 64);
    const int wave_i = twave / (TBN / 32), wave_j = twave % (TBN / 32);
    float* __restrict__ win = sm.window;
    const long long w0 = (long long)blockIdx.x * p.window;
    const int wlen = (p.H - w0) < p.window ? (int)(p.H - w0) : p.window;
    const T* __restrict__ gX = static_cast<const T*>(p.X);
    const T* __restrict__ gdY = static_cast<const T*>(p.dY);

    for (int i = tid * 4; i < p.window; i += kThreads * 4) {
      const float4 z = {0.f, 0.f, 0.f, 0.f};
      *reinterpret_cast<float4*>(win + i) = z;
    }

    const int total = p.tiles_k * p.tiles_n;
    const int nchunks = (p.M + kRows - 1) / kRows;
    f32x16_t acc;
#pragma unroll
    for (int e = 0; e < 16; e++) acc[e] = 0.f;
    u32x4_t ra[kPiecesA], rb[kPiecesB];

    // 16 bytes at (row, col) of a row-major matrix, zero outside it.  When the column limit is a
    // multiple of the vector width (`aligned`, the same for all threads) a piece is inside or
    // outside as a whole: the load is then issued unconditionally from a clamped address, and
    // the zero is selected only when the piece goes to LDS — nothing between the load and the
    // next commit touches the loaded registers, so the load stays in flight that long.
    auto piece = [&](const T* base, int64_t ld, int row, int row_lim, int col, int col_lim, bool aligned,
                     bool& ok) -> u32x4_t {
      ok = true;
      if (!aligned) return load_plain<T, false>(base, ld, row, row_lim, col, col_lim);
      ok = row < row_lim && col < col_lim;
      u32x4_t v;
      __builtin_memcpy(&v, base + (ok ? (int64_t)row * ld + col : 0), 16);
      return v;
    };
    const bool aligned = (p.K % VEC == 0) && (p.N % VEC == 0);
    bool oka[kPiecesA], okb[kPiecesB];
    // global -> registers: chunk c (rows of M) of the X and dY tiles of W tile `id`
    auto fetch = [&](int id, int c) {
      const int tk = id / p.tiles_n, tn = id - tk * p.tiles_n;
      const int m0 = c * kRows;
#pragma unroll
      for (int q = 0; q < kPiecesA; q++) {
        const int pc = ttid + q * kTeamThreads;
        ra[q] = piece(gX, p.ldx, m0 + pc / LA::kCpr, p.M, tk * TBK + (pc % LA::kCpr) * VEC, p.K, aligned, oka[q]);
      }
#pragma unroll
      for (int q = 0; q < kPiecesB; q++) {
        const int pc = ttid + q * kTeamThreads;
        rb[q] = piece(gdY, p.lddy, m0 + pc / LB::kCpr, p.M, tn * TBN + (pc % LB::kCpr) * VEC, p.N, aligned, okb[q]);
      }
    };
    auto commit = [&]() {
      const u32x4_t z = {0u, 0u, 0u, 0u};
#pragma unroll
      for (int q = 0; q < kPiecesA; q++) {
        const int pc = ttid + q * kTeamThreads;
        G::template lds_put<kRStrided, LA>(sm.a[team], pc / LA::kCpr, pc % LA::kCpr, oka[q] ? ra[q] : z);
      }
#pragma unroll
      for (int q = 0; q < kPiecesB; q++) {
        const int pc = ttid + q * kTeamThreads;
        G::template lds_put<kRStrided, LB>(sm.b[team], pc / LB::kCpr, pc % LB::kCpr, okb[q] ? rb[q] : z);
      }
    };
    auto compute = [&]() {
#pragma unroll
      for (int ks = 0; ks < kRows / G::KS; ks++) {
        const Frag fa = G::template lds_frag<kRStrided, LA>(sm.a[team], wave_i * 32, ks, lane);
        const Frag fb = G::template lds_frag<kRStrided, LB>(sm.b[team], wave_j * 32, ks, lane);
        acc = Mfma<T>::run(fa, fb, acc);
      }
    };
    // add this wavefront's finished 32x32 block of the tile at offset `tile_off` into the
    // window and clear it; all reads first, then the adds, then all writes (the 16 addresses of
    // a lane are distinct)
    auto add_to_window = [&](int tile_off) {
      // (offsets and window starts are below 2^31, so their difference fits an int)
      const int base = (int)((long long)tile_off - w0) + (wave_i * 32 + (lane >> 5) * 4) * TBN + wave_j * 32 + (lane & 31);
      // elements outside the window go to a dump slot behind it: no branches, so
      // the 16 reads and the 16 writes each go out back to back
      const int dump = p.window + lane;   // (shared between wavefronts: its contents are never used)
      int at[16];
      float cur[16];
#pragma unroll
      for (int e = 0; e < 16; e++) {
        const int a = base + ((e >> 2) * 8 + (e & 3)) * TBN;
        at[e] = (a >= 0 && a < wlen) ? a : dump;
        cur[e] = win[at[e]];
      }
#pragma unroll
      for (int e = 0; e < 16; e++) {
        win[at[e]] = cur[e] + acc[e] * p.scale;
        acc[e] = 0.f;
      }
    };

    // The tile ids are examined kThreads at a time; the tiles that meet the window are appended
    // to the list in ascending order (ballot + prefix inside a wavefront, counts across them).
    // With a hash that spreads the tiles evenly the list holds every hit after one sweep; if
    // it could overflow, the tiles found so far are worked through first.
    int next_id = 0;
    int parity = 0;   // the counts are double-buffered: one barrier per batch of ids
    while (next_id < total) {
      int found = 0;
      while (next_id < total && found + kThreads <= kList) {
        // a thread's next kBatch offsets are loaded together (one memory latency, not kBatch)
        int batch_off[kBatch];
#pragma unroll
        for (int j = 0; j < kBatch; j++) {
          const int id = next_id + j * kThreads + tid;
          batch_off[j] = p.offsets[id < total ? id : total - 1];
        }
#pragma unroll
        for (int j = 0; j < kBatch; j++) {
          if (!(next_id < total && found + kThreads <= kList)) break;   // (the same for all threads)
          const int my_id = next_id + tid;
          const long long my_off = batch_off[j];
          const bool hit = my_id < total && my_off < w0 + wlen && my_off + TBK * TBN > w0;
          const unsigned long long mask = __ballot(hit);
          if (lane == 0) sm.count[parity][wave] = __popcll(mask);
          __syncthreads();   // (first time round: also the cleared window, the finished list)
          int before = 0, batch = 0;
#pragma unroll
          for (int w = 0; w < kWaves; w++) {
            const int c = __builtin_amdgcn_readfirstlane(sm.count[parity][w]);
            before += (w < wave) ? c : 0;
            batch += c;
          }
          if (hit) {
            const int at = found + before + __popcll(mask & ((1ull << lane) - 1ull));
            sm.list[at] = my_id;
            sm.offs[at] = (int)my_off;
          }
          found += batch;
          next_id += kThreads;
          parity ^= 1;
        }
      }
      __syncthreads();   // list complete

      // Round r: team t takes list entry r * kTeams + t.  Every team runs the same number of
      // chunks per round, so the barriers below are reached by all wavefronts together; a team
      // without a tile only keeps step.
      const int rounds = (found + kTeams - 1) / kTeams;
      int entry = team;                                     // this team's current list entry
      if (entry < found) fetch(sm.list[entry], 0);
      for (int r = 0; r < rounds; r++) {
        const bool have = entry < found;
        const int tile_off = have ? __builtin_amdgcn_readfirstlane(sm.offs[entry]) : 0;
        for (int c = 0; c < nchunks; c++) {
          if (have) commit();
          __syncthreads();   // staged chunks visible
          // the next chunk's global loads fly during this chunk's product
          if (c + 1 < nchunks) {
            if (have) fetch(sm.list[entry], c + 1);
          } else if (entry + kTeams < found) {
            fetch(sm.list[entry + kTeams], 0);
          }
          if (have) compute();
          if (c + 1 < nchunks) __syncthreads();   // fragments read: the stages may be overwritten
        }
        // Tiles whose slices overlap must not be added at the same time.  With a large
        // hashed_weight the kTeams tiles of a round rarely overlap: then all teams add at once;
        // otherwise one team after the other.  (The decision depends on the offsets alone, so
        // the summation order stays a function of the problem.)
        bool overlap = false;
        {
          int round_off[kTeams];
#pragma unroll
          for (int t = 0; t < kTeams; t++) {
            const int e = r * kTeams + t;
            round_off[t] = e < found ? __builtin_amdgcn_readfirstlane(sm.offs[e]) : -1;
          }
#pragma unroll
          for (int t = 0; t < kTeams; t++)
#pragma unroll
            for (int u = t + 1; u < kTeams; u++) {
              const int d = round_off[t] - round_off[u];
              overlap |= round_off[t] >= 0 && round_off[u] >= 0 && d < TBK * TBN && d > -TBK * TBN;
            }
        }
        if (!overlap) {
          if (have) add_to_window(tile_off);
          __syncthreads();
        } else {
          for (int turn = 0; turn < kTeams; turn++) {
            if (turn == team && have) add_to_window(tile_off);
            __syncthreads();
          }
        }
        entry += kTeams;
      }
    }
    __syncthreads();

    // store the window: dHW[w0 + i] (+)= image[i], each element exactly once
    if (p.out_f32 || sizeof(T) == 4) {
      float* out = static_cast<float*>(p.dHW) + w0;
      for (int i = tid; i < wlen; i += kThreads) out[i] = win[i] + (p.accumulate ? out[i] : 0.f);
    } else {
      T* out = static_cast<T*>(p.dHW) + w0;
      for (int i = tid; i < wlen; i += kThreads)
        out[i] = ElemTraits<T>::from_float(win[i] + (p.accumulate ? ElemTraits<T>::to_float(out[i]) : 0.f));
    }
  }
};

template <typename T, int TBK, int TBN>
__global__ __launch_bounds__((WindowKernel<T, TBK, TBN>::kThreads)) void rz_window_kernel(WindowParams p) {
  typedef WindowKernel<T, TBK, TBN> K;
  extern __shared__ __attribute__((aligned(16))) unsigned char rz_window_smem[];
  K::run(p, *reinterpret_cast<typename K::Smem*>(rz_window_smem));
}

}  // namespace rz
