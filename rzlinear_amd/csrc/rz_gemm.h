// One MFMA-tiled kernel template for the three RzLinear contractions on gfx950.
//
// A workgroup of WI*WJ wavefronts owns a TI x TJ tile of C and walks the contracted
// dimension R in steps of TR (128 bytes of R per step, 256 for some forms: see TR below).  Per step the A and B tiles are staged
// in LDS and read from there as MFMA fragments.  The hashed operand (W) is fetched as 16-byte
// pieces of hashed_weight at off(tk,tn) + kk*BN + nn; the pieces may start at any element, so
// the loads are unaligned and rely on the hardware's unaligned global access.  Tile offsets
// are hashed into an LDS table sixteen steps at a time, all threads sharing the work, so the
// integer modulos cost every wavefront the same small share and stay off the critical path.
// With direct staging everything a load address needs apart from the step is computed once per
// thread (a 32-bit byte offset per piece); the step only moves a uniform base in scalar
// registers, and a hashed piece adds its tile's table entry.
//
// Register staging (the 16-bit 64 tile, rows shorter than 16 bytes, the single-stage form):
// global -> registers (issued one or two steps ahead) -> LDS (one or two stages).  LDS layouts
// (X = I or J extent of the operand)
//   16-bit, R contiguous in the source : [X][TR + 8]   fragment = one ds_read_b128 per lane
//   16-bit, X contiguous in the source : [TR][X + 32]  fragment = two ds_read_b64_tr_b16
//       (the LDS transpose read returns, to lane c of a 16-lane group, column c of a 4 x 16
//        block whose rows the group's lanes address four-per-row; 32 lanes touch 4 rows x 64
//        bytes, and the 64-byte row skew of this pitch keeps those on distinct banks)
//   fp32                                : [TR][X + pad], one ds_read_b32 per lane; a source
//       with R contiguous is transposed while it is written (pad 1), else copied (pad 4)
//
// Direct staging (16-bit types: the 128 and 256 tiles; fp32: every tile; two stages; complete
// tiles, or ragged ones with CLAMP below): the tiles go global -> LDS with
// direct-to-LDS loads, no registers and no LDS write instructions in between.  Such a load
// puts the 64 lanes' 16-byte pieces at consecutive LDS addresses, so rows cannot be padded;
// the stages are unpadded and swizzled instead, and the swizzle is applied on the global side
// (each lane fetches the piece that belongs at its LDS slot):
//   R contiguous : [X][TR], row = 8 pieces; piece p of row x sits at slot p ^ ((x >> 1) & 7)
//                  (16 pieces with the 256-byte R step: slot p ^ (x & 15))
//   X contiguous : [TR][X], row = X/32 units of 32 elements; unit u of row r sits at u ^ (r & 3)
//                  (fp32: u ^ ((r >> 2) & 1))
// Both keep the fragment reads free of bank conflicts.  fp32 fragments of a directly staged tile
// cover eight elements of R at a time, four MFMAs per pair of blocks: MFMA j of the four contracts
// elements j (lanes 0-31) and 4 + j (lanes 32-63) — any pairing of the two halves is a valid sum as
// long as A and B use the same one — so a lane's four values are one 16-byte piece where R is
// contiguous (one ds_read_b128) and four ds_read_b32 of one column where X is.
#pragma once

#include <type_traits>

#include "rz_common.h"

#ifndef RZ_F32_DIRECT
#define RZ_F32_DIRECT 1
#endif

namespace rz {

enum Layout { kRContig = 0, kRStrided = 1 };

template <typename T> struct Mfma;
template <> struct Mfma<float> {
  typedef float Frag;
  static __device__ __forceinline__ f32x16_t run(Frag a, Frag b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
  }
};
template <> struct Mfma<bf16_t> {
  typedef u32x4_t Frag;
  static __device__ __forceinline__ f32x16_t run(Frag a, Frag b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                   __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  }
};
template <> struct Mfma<f16_t> {
  typedef u32x4_t Frag;
  static __device__ __forceinline__ f32x16_t run(Frag a, Frag b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a),
                                                  __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  }
};

// 16 bytes of a plain row-major matrix at (row, col..col+VEC), zero where out of range
// (FULL: the caller guarantees the piece is in range, no checks).
template <typename T, bool FULL>
__device__ __forceinline__ u32x4_t load_plain(const T* __restrict__ base, int64_t ld, int row,
                                              int row_lim, int col, int col_lim) {
  constexpr int VEC = ElemTraits<T>::kVec;
  u32x4_t v = {0u, 0u, 0u, 0u};
  if constexpr (FULL) {
    __builtin_memcpy(&v, base + (int64_t)row * ld + col, 16);
    return v;
  }
  if (row < row_lim && col < col_lim) {
    const T* p = base + (int64_t)row * ld + col;
    if (col + VEC <= col_lim) {
      __builtin_memcpy(&v, p, 16);
    } else {
#pragma unroll
      for (int e = 0; e < VEC; e++) {
        if (col + e < col_lim) {
          if constexpr (sizeof(T) == 2) {
            uint16_t b;
            __builtin_memcpy(&b, p + e, 2);
            v[e >> 1] |= (uint32_t)b << (16 * (e & 1));
          } else {
            uint32_t b;
            __builtin_memcpy(&b, p + e, 4);
            v[e] = b;
          }
        }
      }
    }
  }
  return v;
}

// Zero the elements e of a 16-byte piece with col + e >= col_lim.
template <typename T>
__device__ __forceinline__ u32x4_t mask_tail(u32x4_t v, int col, int col_lim) {
  constexpr int VEC = ElemTraits<T>::kVec;
  if (col + VEC > col_lim) {
#pragma unroll
    for (int e = 0; e < VEC; e++) {
      if (col + e >= col_lim) {
        if constexpr (sizeof(T) == 2) v[e >> 1] &= (e & 1) ? 0x0000ffffu : 0xffff0000u;
        else v[e] = 0u;
      }
    }
  }
  return v;
}

// The elements sh .. VEC - 1 of a 16-byte piece moved down to positions 0 .. VEC - 1 - sh, zeros above
// (1 <= sh < VEC; 16-bit: VEC = 8, 32-bit: VEC = 4).
__device__ __forceinline__ u32x4_t shift_down_32(u32x4_t v, int sh) {
  u32x4_t r;
#pragma unroll
  for (int e = 0; e < 4; e++) r[e] = (e + sh == 1) ? v[1] : (e + sh == 2) ? v[2] : (e + sh == 3) ? v[3] : 0u;
  return r;
}
__device__ __forceinline__ u32x4_t shift_down_16(u32x4_t v, int sh) {
  const uint64_t lo = (uint64_t)v[0] | (uint64_t)v[1] << 32, hi = (uint64_t)v[2] | (uint64_t)v[3] << 32;
  const int bits = sh * 16;
  const uint64_t olo = bits >= 64 ? hi >> (bits - 64) : (lo >> bits) | (hi << (64 - bits));
  const uint64_t ohi = bits >= 64 ? 0ull : hi >> bits;
  u32x4_t r = {(uint32_t)olo, (uint32_t)(olo >> 32), (uint32_t)ohi, (uint32_t)(ohi >> 32)};
  return r;
}

// COLSUM (weight-grad only): also sum the columns of B (dY) for the bias gradient.
// CLAMP (with FULL = false): ragged shapes.  The last R step may be partial (its excess is
// cleared in LDS) and the C tile grid may have ragged edges.  Tiles are then still staged directly: a piece that
// would start outside the operand is fetched from the nearest row / piece inside it (hashed
// pieces need nothing: every tile index hashes to a valid slice).  What such a piece holds
// only reaches rows or columns of C that the bounds-checked epilogue never stores.
// Rows of a plain operand need not be whole 16-byte pieces either (any K, N >= 8): the piece that
// straddles the end of a row is fetched as it lies, reaching into the next row — except in the
// operand's LAST row, where that would read beyond the operand: there the piece is fetched so that
// it ends with the row, and one thread puts it right in LDS afterwards (a second, guarded load,
// shifted into place).  Where R is the contiguous dimension the excess elements of the straddling
// piece are cleared in LDS in every row, like the pieces wholly beyond R.
// WK (forward / input-grad): WK groups of WI x WJ wavefronts share a C tile; group g multiplies
// the g-th part of every R step and the groups' accumulators are added through LDS at the end.
// For a tile with one wavefront per SIMD (fp32, 64 x 64) this puts a second wavefront on every
// SIMD, which fills the MFMA pipe while the first waits for its fragments.
template <typename T, int OP, int TI, int TJ, int WI, int WJ, int NSTAGE, bool FULL, bool COLSUM = false,
          bool CLAMP = false, int WK = 1>
struct GemmKernel {
  static_assert(WK == 1 || (OP != kWeightGrad && NSTAGE == 2), "the R step is shared out only by the pipelined store kernels");
  static_assert(!(FULL && CLAMP), "complete tiles need no clamping");
  static_assert(!COLSUM || OP == kWeightGrad, "column sums belong to the weight-grad contraction");
  typedef ElemTraits<T> Tr;
  static constexpr int kThreads = 64 * WI * WJ * WK;
  static constexpr int VEC = Tr::kVec;
  static constexpr bool k16 = (Tr::kBytes == 2);
  // R step: 128 bytes of R — except the directly staged 128 tile with eight wavefronts, which
  // is used at about one workgroup per compute unit and has LDS to spare: it takes 256 bytes
  // per step, halving the barriers per flop (8 % faster at 2048^3).
  static constexpr bool kLongStep = Tr::kBytes == 2 && (FULL || CLAMP) && NSTAGE == 2 && TI == 128 && TJ == 128 &&
                                    WI * WJ == 8;
  // ... and the fp32 tiles of at most 64 rows in forward / input-grad, whose 128-byte step is over in
  // 0.4 us — less than a load from L2 takes, so that loads issued two steps ahead arrive late, and
  // half as many barriers per flop (1024^3: forward 30.2 -> 28.3 us, input-grad 27.1 -> 25.9 us;
  // the four-wavefront weight-grad form lost 3 % with it and keeps the short step)
  static constexpr bool kLongStepF32 = Tr::kBytes == 4 && NSTAGE == 2 && TI <= 64 && OP != kWeightGrad;
  static constexpr int TR = ((kLongStep || kLongStepF32) ? 256 : 128) / Tr::kBytes;
  static constexpr int kPpr = TR / (16 / Tr::kBytes);   // 16-byte pieces per R-contiguous row (8 or 16)
  // swizzle of an R-contiguous direct stage: piece p of row x sits at slot p ^ row_swizzle(x)
  static __device__ __forceinline__ int row_swizzle(int row) { return kPpr == 16 ? (row & 15) : ((row >> 1) & 7); }
  // swizzle of an X-contiguous direct stage: the unit of 32 elements u of row r sits at u ^ unit_swizzle(r)
  // (32-bit: rows r and r + 4, which the two halves of a wavefront read together, land in different banks)
  static __device__ __forceinline__ int unit_swizzle(int row) { return Tr::kBytes == 2 ? (row & 3) : ((row >> 2) & 1); }
  static __device__ __forceinline__ int strided_at(int row, int col, int pitch) {
    return row * pitch + ((((col >> 5) ^ unit_swizzle(row)) << 5) | (col & 31));
  }
  static __device__ __forceinline__ u32x4_t shift_down(u32x4_t v, int sh) {
    return Tr::kBytes == 2 ? shift_down_16(v, sh) : shift_down_32(v, sh);
  }
  static constexpr int A_LAYOUT = (OP == kWeightGrad) ? kRStrided : kRContig;
  static constexpr int B_LAYOUT = (OP == kInputGrad) ? kRContig : kRStrided;
  static constexpr int WTI = TI / WI, WTJ = TJ / WJ;   // wavefront tile
  static constexpr int MI = WTI / 32, MJ = WTJ / 32;   // 32x32 MFMA blocks per wavefront
  static_assert(WTI % 32 == 0 && WTJ % 32 == 0, "wavefront tile must be a multiple of 32");

  // direct-to-LDS staging (see the head of this file)
  static constexpr bool kDirect16 = k16 && (FULL || CLAMP) && NSTAGE == 2 && TI >= 128 && TJ >= 128;
  // fp32, complete tiles: the same staging; a "sub-step" is then eight elements of R (four MFMAs per
  // pair of blocks), and a fragment holds a lane's four values of it
  static constexpr bool kDirect32 = !k16 && RZ_F32_DIRECT && (FULL || CLAMP) && NSTAGE == 2 && TJ >= 64;
  static constexpr bool kDirect = kDirect16 || kDirect32;
  static constexpr int KS = kDirect32 ? 8 : Tr::kMfmaK;
  typedef typename std::conditional<kDirect32, f32x4_t, typename Mfma<T>::Frag>::type Frag;
  static __device__ __forceinline__ f32x16_t mma(Frag a, Frag b, f32x16_t c) {
    if constexpr (kDirect32) {
#pragma unroll
      for (int j = 0; j < 4; j++) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j], b[j], c, 0, 0, 0);
      return c;
    } else {
      return Mfma<T>::run(a, b, c);
    }
  }

  template <int LAYOUT, int TX> struct Lds {
    static constexpr int kPitch = kDirect ? (LAYOUT == kRContig ? TR : TX)
                                  : k16   ? (LAYOUT == kRContig ? TR + 8 : TX + 32)
                                          : (LAYOUT == kRContig ? TX + 1 : TX + 4);
    static constexpr int kRows = ((k16 || kDirect) && LAYOUT == kRContig) ? TX : TR;
    static constexpr int kElems = ((kPitch * kRows + 7) / 8) * 8;
    static_assert(!kDirect32 || LAYOUT == kRContig || (TX >= 64 && TX <= 256), "a direct load instruction fills whole rows of two or more 128-byte units");
    // source tile as seen by the global loads
    static constexpr int kSrcRows = (LAYOUT == kRContig) ? TX : TR;
    static constexpr int kSrcCols = (LAYOUT == kRContig) ? TR : TX;
    static constexpr int kCpr = kSrcCols / VEC;                 // 16-byte pieces per source row
    static constexpr int kPieces = kSrcRows * kCpr / kThreads;  // pieces per thread
    static_assert(kSrcRows * kCpr % kThreads == 0, "tile must split evenly over the threads");
    // a thread's pieces are kPieces consecutive source rows (else: interleaved over the tile)
    static constexpr bool kBlocked = (k16 || LAYOUT == kRStrided) && (kThreads % kCpr == 0) &&
                                     (kPieces == 1 || kPieces == 2 || kPieces == 4 || kPieces == 8 ||
                                      kPieces == 16);
  };
  typedef Lds<A_LAYOUT, TI> LA;
  typedef Lds<B_LAYOUT, TJ> LB;

  // offset table: kOffSlots windows (one per R step; two banks of kOffBank steps, one in use
  // while the other is refilled) of kOffWindow entries; the weight-grad epilogue reuses it for
  // the (TI/16) x (TJ/16) tiles of its C tile
  static constexpr int kOffSlots = 32;    // two banks of kOffBank steps
  static constexpr int kOffBank = 16;
  static constexpr int kOffWindow = (TR / 16) * (TJ / 16);
  static constexpr int kOffEntries = (OP == kWeightGrad) ? (TI / 16) * (TJ / 16) : kOffSlots * kOffWindow;
  static constexpr int kTurnEntries = 65;   // weight-grad, behind the offsets: the round of up to 64 hashed tiles, and the number of rounds

  struct Smem {
    alignas(16) T a[NSTAGE][LA::kElems];
    alignas(16) T b[NSTAGE][LB::kElems];
    int off[kOffEntries];
  };
  // after the last R step the operand stages are dead; weight-grad may keep an fp32 image of
  // dHW there
  static constexpr size_t kImageBytes = sizeof(T) * NSTAGE * (size_t)(LA::kElems + LB::kElems);

  // ---- LDS write of one staged piece -------------------------------------------------------
  template <int LAYOUT, typename L>
  static __device__ __forceinline__ void lds_put(T* lds, int srow, int scc, u32x4_t v) {
    if constexpr (k16 || LAYOUT == kRStrided) {
      *reinterpret_cast<u32x4_t*>(lds + srow * L::kPitch + scc * VEC) = v;
    } else {
      // fp32, R contiguous in the source: transpose to [r][x]
#pragma unroll
      for (int e = 0; e < 4; e++)
        reinterpret_cast<uint32_t*>(lds)[(scc * 4 + e) * L::kPitch + srow] = v[e];
    }
  }

  // ---- MFMA fragment of the 32-wide block starting at x_base, R sub-step ks ------------------
  template <int LAYOUT, typename L>
  static __device__ __forceinline__ Frag lds_frag(const T* lds, int x_base, int ks, int lane) {
    if constexpr (kDirect32) {
      // sub-step ks = elements 8 ks .. 8 ks + 7 of the R step; MFMA j of the sub-step contracts
      // elements 8 ks + j and 8 ks + 4 + j (the lower and the upper half of the wavefront): any
      // pairing does, as long as both operands use the same one, and this one makes a lane's four
      // values one 16-byte piece where R is contiguous
      const float* f = reinterpret_cast<const float*>(lds);
      if constexpr (LAYOUT == kRContig) {
        const int row = x_base + (lane & 31), piece = ks * 2 + (lane >> 5);
        return *reinterpret_cast<const f32x4_t*>(f + row * L::kPitch + ((piece ^ row_swizzle(row)) << 2));
      } else {
        // rows 8 ks + 4 h .. + 3 (h = lane / 32), 32 consecutive columns: the 128-byte unit u of row r
        // sits at u ^ ((r >> 2) & 1), so that the two halves of the wavefront read different banks
        const int col = x_base + (lane & 31), row = ks * 8 + (lane >> 5) * 4;
        const float* at = f + strided_at(row, col, L::kPitch);
        f32x4_t v = {at[0], at[L::kPitch], at[2 * L::kPitch], at[3 * L::kPitch]};
        return v;
      }
    } else if constexpr (!k16) {
      return reinterpret_cast<const float*>(lds)[(ks * 2 + (lane >> 5)) * L::kPitch + x_base +
                                                 (lane & 31)];
    } else if constexpr (LAYOUT == kRContig) {
      const int row = x_base + (lane & 31), piece = ks * 2 + (lane >> 5);
      if constexpr (kDirect)
        return *reinterpret_cast<const u32x4_t*>(lds + row * L::kPitch + ((piece ^ row_swizzle(row)) << 3));
      return *reinterpret_cast<const u32x4_t*>(lds + row * L::kPitch + piece * 8);
    } else {
      const int g = lane >> 4, jl = lane & 15;
      const int row = ks * 16 + 8 * (g >> 1) + (jl >> 2), col = x_base + 16 * (g & 1) + 4 * (jl & 3);
      // (row + 4 has the same swizzle as row, so the second read is one pitch-multiple further)
      const T* p = kDirect ? lds + strided_at(row, col, L::kPitch) : lds + row * L::kPitch + col;
      typedef s16x4_t __attribute__((address_space(3))) * lds_s16x4_ptr;
      const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p));
      const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p + 4 * L::kPitch));
      const u32x2_t l2 = __builtin_bit_cast(u32x2_t, lo), h2 = __builtin_bit_cast(u32x2_t, hi);
      u32x4_t r = {l2[0], l2[1], h2[0], h2[1]};
      return r;
    }
  }

  // ---- hashed tiles touched by one R step ---------------------------------------------------
  struct OffWindow { int tk0, tn0, ntn, count; };
  static __device__ __forceinline__ OffWindow off_window(const HashParams& h, int x0_k, int span_k,
                                                         int x0_n, int span_n) {
    OffWindow w;
    w.tk0 = x0_k >> h.bk_shift;
    w.tn0 = x0_n >> h.bn_shift;
    const int ntk = (span_k >> h.bk_shift) > 0 ? (span_k >> h.bk_shift) : 1;
    w.ntn = (span_n >> h.bn_shift) > 0 ? (span_n >> h.bn_shift) : 1;
    w.count = ntk * w.ntn;
    return w;
  }
  static __device__ __forceinline__ void off_fill(int* tab, const HashParams& h, const OffWindow& w,
                                                  int tid) {
    if (tid < w.count)
      tab[tid] = (int)tile_offset(h, (uint32_t)(w.tk0 + tid / w.ntn), (uint32_t)(w.tn0 + tid % w.ntn));
  }

  // Element index in hashed_weight of W[k, n] through the offset table (k, n inside the window).
  static __device__ __forceinline__ int hashed_index(const HashParams& h, const int* tab,
                                                     const OffWindow& w, int k, int n) {
    const int off = tab[((k >> h.bk_shift) - w.tk0) * w.ntn + ((n >> h.bn_shift) - w.tn0)];
    return off + (k & (h.BK - 1)) * h.BN + (n & (h.BN - 1));
  }

  // 16 bytes of W starting at element `idx` of hashed_weight; zero outside K x N.
  static __device__ __forceinline__ u32x4_t load_hashed(const T* __restrict__ hw, int idx, int k,
                                                        int K, int n, int N) {
    u32x4_t v = {0u, 0u, 0u, 0u};
    if (FULL || (k < K && n < N)) {
      __builtin_memcpy(&v, hw + idx, 16);
      if constexpr (!FULL) v = mask_tail<T>(v, n, N);
    }
    return v;
  }

  static __device__ __forceinline__ void run(const GemmParams& p, Smem& sm) {
    run_item(p, sm, threadIdx.x, blockIdx.x, blockIdx.y, gridDim.x);
  }

  // One C tile (workgroup id `bx` of `gx`, as the hardware deals them to the XCDs) and slice `by`
  // of the contracted dimension.
  static __device__ __forceinline__ void run_item(const GemmParams& p, Smem& sm, const int tid, int bx, int by, int gx) {
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // (uniform: lives in a scalar register)
    const int wave_k = wave / (WI * WJ);                 // which part of every R step
    const int wave_i = (wave % (WI * WJ)) / WJ, wave_j = wave % WJ;
    // Offset in the C tile of a wavefront's 32x32 block (a, b).  Forward and input-grad give a
    // wavefront one contiguous WTI x WTJ sub-tile (whole cache lines per store).  Weight-grad
    // deals the blocks round-robin instead, so that the blocks of one hashed tile belong to
    // different wavefronts and its scatter round is shared between them.
    auto blk_i = [&](int a) -> int { return (OP == kWeightGrad) ? (a * WI + wave_i) * 32 : wave_i * WTI + a * 32; };
    auto blk_j = [&](int b) -> int { return (OP == kWeightGrad) ? (b * WJ + wave_j) * 32 : wave_j * WTJ + b * 32; };

    // Workgroup ids are dealt round-robin to the 8 XCDs; renumber so that each XCD (one L2)
    // gets a contiguous run of tiles, then walk tiles with J fastest (forward/input-grad
    // share the streamed A panel) or in square-ish groups (weight-grad streams both).
    int id = bx;
    {
      const int nwg = gx, per = nwg >> 3, rem = nwg & 7, x = id & 7, q = id >> 3;
      id = x * per + (x < rem ? x : rem) + q;
    }
    int ti, tj;
    if constexpr (OP == kWeightGrad) {
      constexpr int G = 8;
      const int in_group = G * p.tiles_j;
      const int first = (id / in_group) * G;
      const int gsz = (p.tiles_i - first) < G ? (p.tiles_i - first) : G;
      ti = first + (id % in_group) % gsz;
      tj = (id % in_group) / gsz;
    } else {
      ti = id / p.tiles_j;
      tj = id % p.tiles_j;
    }
    const int i0 = ti * TI, j0 = tj * TJ;
    const int r_begin = by * p.r_chunk;
    const int r_end = (r_begin + p.r_chunk) < p.R ? (r_begin + p.r_chunk) : p.R;
    const int steps = (r_end - r_begin + TR - 1) / TR;

    const T* __restrict__ gA = static_cast<const T*>(p.A);
    const T* __restrict__ gB = static_cast<const T*>(p.B);
    const T* __restrict__ gHW = static_cast<const T*>(p.HW);

    f32x16_t acc[MI][MJ];
#pragma unroll
    for (int a = 0; a < MI; a++)
#pragma unroll
      for (int b = 0; b < MJ; b++)
#pragma unroll
        for (int e = 0; e < 16; e++) acc[a][b][e] = 0.f;

    u32x4_t ra[LA::kPieces], rb[LB::kPieces];
    // elements of the last R step that lie beyond R (ragged contraction, direct staging)
    const int tail = CLAMP ? steps * TR - (r_end - r_begin) : 0;
    // elements of the piece that straddles the end of an operand's rows (0: rows are whole pieces):
    // along R in forward / input-grad, along I (X) and J (dY) in weight-grad
    const int rag_r = (CLAMP && OP != kWeightGrad) ? (p.R & (VEC - 1)) : 0;
    const int rag_i = (CLAMP && OP == kWeightGrad) ? (p.I & (VEC - 1)) : 0;
    const int rag_j = (CLAMP && OP == kWeightGrad) ? (p.J & (VEC - 1)) : 0;
    // the step that holds the operands' last row is issued piece by piece and put right in LDS
    const bool slow_last = CLAMP && (tail > 0 || ((rag_i | rag_j) != 0 && r_end == p.R));

    // Bias gradient (COLSUM): the tiles_i workgroups of one tile column and slice stage the same
    // rows of dY, so they take turns: the workgroup whose turn it is adds the rows of that R
    // step, from the registers on their way into LDS (direct staging: from the LDS stage), into
    // per-thread column sums.  A thread's pieces sit in one 16-byte column position, so VEC
    // sums per thread suffice.
    static_assert(!COLSUM || kThreads % LB::kCpr == 0, "a thread's pieces must share their columns");
    float colsum[VEC];
#pragma unroll
    for (int e = 0; e < VEC; e++) colsum[e] = 0.f;
    int colsum_turn = COLSUM ? (r_begin / TR) % p.tiles_i : 0;

    auto window = [&](int step) -> OffWindow {
      const int r0 = r_begin + step * TR;
      if constexpr (OP == kForward) return off_window(p.h, r0, TR, j0, TJ);
      else return off_window(p.h, j0, TJ, r0, TR);
    };
    // hash the tiles of R step `step` into its slot of the offset table
    // Hash the tiles of the kOffBank steps from `first` on into their slots of the offset table,
    // all threads sharing the work (the integer modulos of the hash are long instruction
    // sequences: done in bulk, every wavefront pays the same small share every kOffBank steps).
    // With direct staging an entry is the tile offset plus the part of the within-tile offset
    // that belongs to the step (a step inside a larger hashed tile starts r0 & (B - 1) rows /
    // columns into it).
    auto hash_bulk = [&](int first) {
      if constexpr (OP != kWeightGrad) {
        if (first < steps) {
          const OffWindow w0 = window(first);              // count and ntn are the same for every step
          const int cshift = __builtin_ctz(w0.count);     // (a power of two)
          const int total = kOffBank << cshift;
          for (int e = tid; e < total; e += kThreads) {
            const int step = first + (e >> cshift), t = e & (w0.count - 1);
            if (step < steps) {
              const OffWindow w = window(step);
              int v = (int)tile_offset(p.h, (uint32_t)(w.tk0 + t / w.ntn), (uint32_t)(w.tn0 + t % w.ntn));
              if constexpr (kDirect) {
                const int r0 = r_begin + step * TR;
                v += (OP == kForward) ? (r0 & (p.h.BK - 1) & ~(TR - 1)) * p.h.BN : (r0 & (p.h.BN - 1) & ~(TR - 1));
              }
              sm.off[(step & (kOffSlots - 1)) * kOffWindow + t] = v;
            }
          }
        }
      }
    };
    // in the main loops: at the first step of a bank, refill the other bank for the steps after it
    auto hash_ahead = [&](int s) {
      if constexpr (OP != kWeightGrad) {
        if (s > 0 && (s & (kOffBank - 1)) == 0) hash_bulk(s + kOffBank);
      }
    };
    // Which 16-byte pieces of a source tile a thread moves.  A thread owns kPieces consecutive
    // rows at one column position: the rows are a constant pitch apart (cheap addresses), and,
    // being at most 16 rows aligned to their count, they lie in ONE hashed tile, so a hashed
    // operand needs a single table lookup per thread and step.  (fp32 tiles whose source has R
    // contiguous are transposed on their way into LDS; they keep the interleaved mapping, which
    // spreads that scatter over the banks.)
    auto piece_row = [&](auto L, int q) -> int {
      typedef decltype(L) LL;
      if constexpr (LL::kBlocked) return (tid / LL::kCpr) * LL::kPieces + q;
      else return (tid + q * kThreads) / LL::kCpr;
    };
    auto piece_cc = [&](auto L, int q) -> int {
      typedef decltype(L) LL;
      if constexpr (LL::kBlocked) return tid % LL::kCpr;
      else return (tid + q * kThreads) % LL::kCpr;
    };
    // global -> registers for R step `step`
    auto fetch = [&](int step) {
      const int r0 = r_begin + step * TR;
#pragma unroll
      for (int q = 0; q < LA::kPieces; q++) {
        const int srow = piece_row(LA{}, q), scol = piece_cc(LA{}, q) * VEC;
        if constexpr (A_LAYOUT == kRContig)
          ra[q] = load_plain<T, FULL>(gA, p.lda, i0 + srow, p.I, r0 + scol, r_end);
        else
          ra[q] = load_plain<T, FULL>(gA, p.lda, r0 + srow, r_end, i0 + scol, p.I);
      }
      if constexpr (OP == kWeightGrad) {
#pragma unroll
        for (int q = 0; q < LB::kPieces; q++) {
          const int srow = piece_row(LB{}, q), scol = piece_cc(LB{}, q) * VEC;
          rb[q] = load_plain<T, FULL>(gB, p.ldb, r0 + srow, r_end, j0 + scol, p.J);
        }
      } else {
        const OffWindow w = window(step);
        const int* tab = sm.off + (step & (kOffSlots - 1)) * kOffWindow;
        int idx[LB::kPieces];
        if constexpr (LB::kBlocked) {
          // one lookup: the thread's rows are consecutive rows k of one hashed tile
          const int srow = piece_row(LB{}, 0), scol = piece_cc(LB{}, 0) * VEC;
          const int k = (OP == kForward) ? r0 + srow : j0 + srow;
          const int n = (OP == kForward) ? j0 + scol : r0 + scol;
          const int idx0 = hashed_index(p.h, tab, w, k, n);
#pragma unroll
          for (int q = 0; q < LB::kPieces; q++) idx[q] = idx0 + q * p.h.BN;
        } else {
          // all table lookups first (one LDS round trip), then the loads
#pragma unroll
          for (int q = 0; q < LB::kPieces; q++) {
            const int srow = piece_row(LB{}, q), scol = piece_cc(LB{}, q) * VEC;
            const int k = (OP == kForward) ? r0 + srow : j0 + srow;
            const int n = (OP == kForward) ? j0 + scol : r0 + scol;
            idx[q] = hashed_index(p.h, tab, w, k, n);
          }
        }
#pragma unroll
        for (int q = 0; q < LB::kPieces; q++) {
          const int srow = piece_row(LB{}, q), scol = piece_cc(LB{}, q) * VEC;
          if constexpr (OP == kForward)
            rb[q] = load_hashed(gHW, idx[q], r0 + srow, r_end, j0 + scol, p.J);
          else
            rb[q] = load_hashed(gHW, idx[q], j0 + srow, p.J, r0 + scol, r_end);
        }
      }
    };
    // registers -> LDS stage `st`
    auto commit = [&](int st) {
#pragma unroll
      for (int q = 0; q < LA::kPieces; q++)
        lds_put<A_LAYOUT, LA>(sm.a[st], piece_row(LA{}, q), piece_cc(LA{}, q), ra[q]);
#pragma unroll
      for (int q = 0; q < LB::kPieces; q++)
        lds_put<B_LAYOUT, LB>(sm.b[st], piece_row(LB{}, q), piece_cc(LB{}, q), rb[q]);
      if constexpr (COLSUM) {
        // commits happen once per R step, in step order
        if (colsum_turn == ti) {
#pragma unroll
          for (int q = 0; q < LB::kPieces; q++) {
            T elems[VEC];
            __builtin_memcpy(elems, &rb[q], 16);
#pragma unroll
            for (int e = 0; e < VEC; e++) colsum[e] += Tr::to_float(elems[e]);
          }
        }
        colsum_turn = (colsum_turn + 1 == p.tiles_i) ? 0 : colsum_turn + 1;
      }
    };
    // Direct staging: the same sums out of the dY tile in LDS stage `st`.  Thread (g, c) =
    // (tid / kCpr, tid % kCpr) adds rows g, g + groups, ... of the 16-byte column position c
    // (16-bit: the rows are a multiple of four apart, so they share one swizzle).
    auto colsum_from_stage = [&](int st) {
      constexpr int kGroups = kThreads / LB::kCpr;
      static_assert(!(COLSUM && kDirect) || (TR % kGroups == 0 && (!k16 || kGroups % 4 == 0)), "rows must share a swizzle");
      if (colsum_turn == ti) {
        const int g = tid / LB::kCpr, c = tid % LB::kCpr;
#pragma unroll
        for (int i = 0; i < TR / kGroups; i++) {
          const int row = g + i * kGroups;
          T elems[VEC];
          __builtin_memcpy(elems, sm.b[st] + strided_at(row, c * VEC, LB::kPitch), 16);
#pragma unroll
          for (int e = 0; e < VEC; e++) colsum[e] += Tr::to_float(elems[e]);
        }
      }
      colsum_turn = (colsum_turn + 1 == p.tiles_i) ? 0 : colsum_turn + 1;
    };
    // Direct staging: where a lane's q-th load instruction of a tile fetches from.  The
    // instruction with index n = wave * kPieces + q fills LDS bytes [1024 n, 1024 n + 1024) of
    // the stage, lane i the 16 bytes at 16 i; (row, col) is the source piece that the swizzled
    // layout keeps there.
    auto direct_src = [&](auto L, int layout, int q, int& row, int& col) {
      typedef decltype(L) LL;
      const int n = wave * LL::kPieces + q;
      if (layout == kRContig) {
        row = n * (64 / kPpr) + lane / kPpr;
        col = ((lane % kPpr) ^ row_swizzle(row)) * VEC;
      } else {
        constexpr int kSlots = LL::kPitch / VEC;        // 16-byte slots per row
        row = n * (64 / kSlots) + lane / kSlots;
        const int slot = lane % kSlots;
        constexpr int kPpu = 32 / VEC;                  // 16-byte slots per unit of 32 elements
        col = (((slot / kPpu) ^ unit_swizzle(row)) << 5) | ((slot % kPpu) * VEC);
      }
    };
    auto direct_load = [&](const T* src, const T* stage, int q, int pieces) {
      // the LDS address goes through M0 and must be the same for the whole wavefront
      typedef const T __attribute__((address_space(3)))* lds_ptr;
      const uint32_t dst = __builtin_amdgcn_readfirstlane(
          (uint32_t)(uintptr_t)(lds_ptr)(stage) + (uint32_t)((wave * pieces + q) * 1024));
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(dst), "v"(src)
                   : "memory", "m0");
    };
    // the same load with the address split into a uniform 64-bit base (scalar registers) and a
    // per-lane 32-bit byte offset: the offsets are computed once, the base moves with the step
    auto direct_load_so = [&](const void* base, uint32_t voff, const T* stage, int q, int pieces) {
      typedef const T __attribute__((address_space(3)))* lds_ptr;
      const uint32_t dst = __builtin_amdgcn_readfirstlane(
          (uint32_t)(uintptr_t)(lds_ptr)(stage) + (uint32_t)((wave * pieces + q) * 1024));
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(voff), "s"(base)
                   : "memory", "m0");
    };
    // the plain tiles of R step `step` -> LDS stage `st`, addresses computed in full (used for
    // the last, partial step of a ragged contraction, whose pieces beyond R are redirected)
    auto direct_issue_plain_slow = [&](int step, int st) {
      const int r0 = r_begin + step * TR;
#pragma unroll
      for (int q = 0; q < LA::kPieces; q++) {
        int row, col;
        direct_src(LA{}, A_LAYOUT, q, row, col);
        // (CLAMP: rows / 16-byte columns beyond I come from the last one inside)
        const int gi = (A_LAYOUT == kRContig) ? i0 + row : i0 + col;
        const int ci = !CLAMP ? gi : (A_LAYOUT == kRContig) ? (gi < p.I ? gi : p.I - 1) : (gi < p.I ? gi : p.I - VEC);
        // (CLAMP weight-grad: rows of the last, partial R step beyond R come from row R - 1 and
        //  are cleared in LDS before they are used, see clear_tail)
        const int gr = r0 + row;
        const int cr = (CLAMP && OP == kWeightGrad && gr >= p.R) ? p.R - 1 : gr;
        // (CLAMP forward / input-grad: pieces of the last, partial R step beyond R come from the
        //  last piece inside and are cleared in LDS as well)
        const int gc = r0 + col;
        int cc = (CLAMP && gc >= p.R) ? p.R - VEC : gc;
        int ca = ci;
        if constexpr (CLAMP) {
          // the piece that straddles the end of the operand's last row ends with the row (see clear_tail)
          if (A_LAYOUT == kRContig && rag_r && ci == p.I - 1 && gc < p.R && gc + VEC > p.R) cc = p.R - VEC;
          if (A_LAYOUT == kRStrided && rag_i && cr == p.R - 1 && gi < p.I && gi + VEC > p.I) ca = p.I - VEC;
        }
        const T* src = (A_LAYOUT == kRContig) ? gA + (int64_t)ci * p.lda + cc
                                              : gA + (int64_t)cr * p.lda + ca;
        direct_load(src, sm.a[st], q, LA::kPieces);
      }
      if constexpr (OP == kWeightGrad) {
#pragma unroll
        for (int q = 0; q < LB::kPieces; q++) {
          int row, col;
          direct_src(LB{}, B_LAYOUT, q, row, col);
          const int gj = j0 + col;
          int cj = (!CLAMP || gj < p.J) ? gj : p.J - VEC;
          const int gr = r0 + row;
          const int cr = (CLAMP && gr >= p.R) ? p.R - 1 : gr;
          if (CLAMP && rag_j && cr == p.R - 1 && gj < p.J && gj + VEC > p.J) cj = p.J - VEC;
          direct_load(gB + (int64_t)cr * p.ldb + cj, sm.b[st], q, LB::kPieces);
        }
      }
    };
    // Step-invariant part of every direct load of this thread, computed once.
    //   plain operand : byte offset of the piece from the tile's first element of the step
    //                   (edge clamping of ragged tile grids included: it does not depend on the step)
    //   hashed operand: which entry of the step's offset window the piece's tile is, and the
    //                   byte offset of the piece inside its tile.  A step starts on a multiple of
    //                   TR, so with the hashed tile's extent along R a power of two, (r0 + x) &
    //                   (B - 1) = (r0 & (B - 1)) + (x & (B - 1)) when B >= TR, and r0 drops out
    //                   when B < TR; the step's part is uniform and is added to the table entries
    //                   when they are hashed (see hash_bulk).
    uint32_t a_voff[kDirect ? LA::kPieces : 1], b_voff[kDirect ? LB::kPieces : 1];
    int b_tab[kDirect ? LB::kPieces : 1];
    if constexpr (kDirect) {
#pragma unroll
      for (int q = 0; q < LA::kPieces; q++) {
        int row, col;
        direct_src(LA{}, A_LAYOUT, q, row, col);
        if constexpr (A_LAYOUT == kRContig) {
          const int gi = i0 + row;
          const int ci = (!CLAMP || gi < p.I) ? row : p.I - 1 - i0;
          a_voff[q] = (uint32_t)(((int64_t)ci * p.lda + col) * (int64_t)sizeof(T));
        } else {
          const int gi = i0 + col;
          // (an offset is unsigned: a tile with fewer than VEC columns inside I has no whole piece of its
          //  own to repeat and repeats its first, straddling one)
          const int ci = (!CLAMP || gi < p.I) ? col : (p.I - VEC - i0 > 0 ? p.I - VEC - i0 : 0);
          a_voff[q] = (uint32_t)(((int64_t)row * p.lda + ci) * (int64_t)sizeof(T));
        }
      }
#pragma unroll
      for (int q = 0; q < LB::kPieces; q++) {
        int row, col;
        direct_src(LB{}, B_LAYOUT, q, row, col);
        if constexpr (OP == kWeightGrad) {
          const int gj = j0 + col;
          const int cj = (!CLAMP || gj < p.J) ? col : (p.J - VEC - j0 > 0 ? p.J - VEC - j0 : 0);
          b_voff[q] = (uint32_t)(((int64_t)row * p.ldb + cj) * (int64_t)sizeof(T));
          b_tab[q] = 0;
        } else {
          // (k, n) of the piece relative to the step's first row / column of W
          // (forward: k = r0 + row, n = j0 + col; input-grad: k = j0 + row, n = r0 + col)
          const int dk = row, dn = col;
          const int kk = (OP == kForward) ? (p.h.BK >= TR ? dk : (dk & (p.h.BK - 1))) : ((j0 + dk) & (p.h.BK - 1));
          const int nn = (OP == kForward) ? ((j0 + dn) & (p.h.BN - 1)) : (p.h.BN >= TR ? dn : (dn & (p.h.BN - 1)));
          b_voff[q] = (uint32_t)((kk * p.h.BN + nn) * (int)sizeof(T));
          const int tk_rel = (OP == kForward) ? (p.h.BK >= TR ? 0 : (dk >> p.h.bk_shift)) : (((j0 + dk) >> p.h.bk_shift) - (j0 >> p.h.bk_shift));
          const int tn_rel = (OP == kForward) ? (((j0 + dn) >> p.h.bn_shift) - (j0 >> p.h.bn_shift)) : (p.h.BN >= TR ? 0 : (dn >> p.h.bn_shift));
          const int ntn = (OP == kForward) ? ((TJ >> p.h.bn_shift) > 0 ? (TJ >> p.h.bn_shift) : 1)
                                           : ((TR >> p.h.bn_shift) > 0 ? (TR >> p.h.bn_shift) : 1);
          b_tab[q] = tk_rel * ntn + tn_rel;
        }
      }
    }
    // a uniform pointer, said to be one (two scalar registers): the base operand of the loads above
    auto uniform_ptr = [&](const T* ptr) -> const T* {
      const uint64_t v = (uint64_t)(uintptr_t)ptr;
      const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
      const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
      return (const T*)(uintptr_t)(((uint64_t)hi << 32) | lo);
    };
    // all tiles of R step `step` -> LDS stage `st`
    auto direct_issue = [&](int step, int st) {
      const int r0 = r_begin + step * TR;
      if (CLAMP && slow_last && step == steps - 1) {   // (uniform) the partial last step, or the one with the operands' last row
        direct_issue_plain_slow(step, st);
      } else {
        // first element of the A tile of this step (uniform)
        const T* a_base = uniform_ptr((A_LAYOUT == kRContig) ? gA + (int64_t)i0 * p.lda + r0 : gA + (int64_t)r0 * p.lda + i0);
#pragma unroll
        for (int q = 0; q < LA::kPieces; q++) direct_load_so(a_base, a_voff[q], sm.a[st], q, LA::kPieces);
        if constexpr (OP == kWeightGrad) {
          const T* b_base = uniform_ptr(gB + (int64_t)r0 * p.ldb + j0);
#pragma unroll
          for (int q = 0; q < LB::kPieces; q++) direct_load_so(b_base, b_voff[q], sm.b[st], q, LB::kPieces);
        }
      }
      if constexpr (OP != kWeightGrad) {
        const int* tab = sm.off + (step & (kOffSlots - 1)) * kOffWindow;
        const T* hw_base = uniform_ptr(gHW);
        uint32_t off[LB::kPieces];
#pragma unroll
        for (int q = 0; q < LB::kPieces; q++) off[q] = (uint32_t)tab[b_tab[q]];   // all lookups first, then the loads
#pragma unroll
        for (int q = 0; q < LB::kPieces; q++)
          direct_load_so(hw_base, off[q] * (uint32_t)sizeof(T) + b_voff[q], sm.b[st], q, LB::kPieces);
      }
    };
    // CLAMP, last R step: once every wavefront's loads of that step have landed (the caller has just
    // passed a barrier), the part of both stages beyond R — fetched from inside the operands, or
    // from tiles beyond the tile grid — is set to zero: whole rows where X is contiguous; where R is,
    // the trailing 16-byte pieces of every row and the excess elements of a piece that straddles R.
    // The straddling piece of an operand's last row (fetched so that it ends with the row, lest the
    // load reach beyond the operand) is fetched again here, through registers, and shifted into
    // place.  A second barrier makes all that visible.  Happens at most once per workgroup.
    auto clear_tail = [&](int st) {
      if constexpr (CLAMP) {
        if (slow_last) {
          const u32x4_t z = {0u, 0u, 0u, 0u};
          // `plain`: the operand's rows lie in memory as they are (not hashed); g, ld: the operand;
          // x0, ext: the tile's first index and the operand's extent along X
          auto clear = [&](auto L, int layout, T* stage, bool plain, const T* g, int64_t ld, int x0, int ext, int rag_x) {
            typedef decltype(L) LL;
            if (layout == kRStrided) {
              const int first = TR - tail;
              for (int i = tid; i < tail * (LL::kPitch / VEC); i += kThreads)
                *reinterpret_cast<u32x4_t*>(stage + first * LL::kPitch + i * VEC) = z;
              // the operand's last row (the last one before `first`), the piece that straddles its end
              const int c = ext - rag_x - x0;
              if (plain && rag_x && r_end == p.R && c >= 0 && c < LL::kPitch && tid == 0) {
                const int row = first - 1;
                u32x4_t v;
                __builtin_memcpy(&v, g + (int64_t)(p.R - 1) * ld + (ext - VEC), 16);
                *reinterpret_cast<u32x4_t*>(stage + strided_at(row, c, LL::kPitch)) = shift_down(v, VEC - rag_x);
              }
            } else {
              const int pieces = tail / VEC, first = TR / VEC - pieces;
              for (int i = tid; i < LL::kRows * pieces; i += kThreads) {
                const int row = i / pieces, pz = first + i % pieces;
                *reinterpret_cast<u32x4_t*>(stage + row * LL::kPitch + (pz ^ row_swizzle(row)) * VEC) = z;
              }
              if (rag_r) {
                const int pz = first - 1;   // the piece that straddles R
                for (int row = tid; row < LL::kRows; row += kThreads) {
                  u32x4_t* at = reinterpret_cast<u32x4_t*>(stage + row * LL::kPitch + (pz ^ row_swizzle(row)) * VEC);
                  u32x4_t v;
                  if (plain && x0 + row >= ext - 1) {   // the operand's last row, and the rows beyond that repeat it
                    __builtin_memcpy(&v, g + (int64_t)(ext - 1) * ld + (p.R - VEC), 16);
                    v = shift_down(v, VEC - rag_r);
                  } else {
                    v = mask_tail<T>(*at, 0, rag_r);
                  }
                  *at = v;
                }
              }
            }
          };
          clear(LA{}, A_LAYOUT, sm.a[st], true, gA, p.lda, i0, p.I, rag_i);
          clear(LB{}, B_LAYOUT, sm.b[st], OP == kWeightGrad, gB, p.ldb, j0, p.J, rag_j);
          __syncthreads();
        }
      }
    };
    // MFMAs of one R step out of LDS stage `st`; fragments are read one sub-step ahead
    auto compute = [&](int st) {
      constexpr int NKS = TR / KS;
      Frag fa[2][MI], fb[2][MJ];
      auto frags = [&](int ks, int buf) {
#pragma unroll
        for (int a = 0; a < MI; a++)
          fa[buf][a] = lds_frag<A_LAYOUT, LA>(sm.a[st], blk_i(a), ks, lane);
#pragma unroll
        for (int b = 0; b < MJ; b++)
          fb[buf][b] = lds_frag<B_LAYOUT, LB>(sm.b[st], blk_j(b), ks, lane);
      };
      frags(0, 0);
#pragma unroll
      for (int ks = 0; ks < NKS; ks++) {
        if (ks + 1 < NKS) frags(ks + 1, (ks + 1) & 1);
#pragma unroll
        for (int a = 0; a < MI; a++)
#pragma unroll
          for (int b = 0; b < MJ; b++)
            acc[a][b] = mma(fa[ks & 1][a], fb[ks & 1][b], acc[a][b]);
        // scheduling hint: spread the LDS reads of the next sub-step between this sub-step's
        // MFMAs (one read after each MFMA), so that their latency hides behind matrix work
        constexpr int kReads = (k16 && A_LAYOUT == kRStrided ? 2 : 1) * MI +
                               (k16 && B_LAYOUT == kRStrided ? 2 : 1) * MJ;
        constexpr int kMfmas = MI * MJ;
        if (ks + 1 < NKS) {
#pragma unroll
          for (int i = 0; i < kMfmas; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // 1 MFMA
            // its share of the LDS reads (compile-time: the loop is unrolled)
            if ((kReads * (i + 1)) / kMfmas - (kReads * i) / kMfmas == 1)
              __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            else if ((kReads * (i + 1)) / kMfmas - (kReads * i) / kMfmas == 2)
              __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            else if ((kReads * (i + 1)) / kMfmas - (kReads * i) / kMfmas == 3)
              __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);
          }
        } else {
          __builtin_amdgcn_sched_group_barrier(0x008, kMfmas, 0);
        }
      }
    };

    if (steps > 0) {
      hash_bulk(0);
      hash_bulk(kOffBank);
      if constexpr (OP != kWeightGrad) __syncthreads();
      if constexpr (!kDirect) fetch(0);
    }
    if constexpr (NSTAGE == 1) {
      // one LDS stage: write it, read it, two barriers per step; relies on several
      // workgroups per compute unit to overlap the phases
      for (int s = 0; s < steps; s++) {
        commit(0);
        __syncthreads();
        if (s + 1 < steps) fetch(s + 1);
        hash_ahead(s);
        compute(0);
        __syncthreads();
      }
    } else {
      // Two LDS stages and a software pipeline with ONE barrier per R step.  While the MFMAs
      // of step s run out of stage s&1, the same instruction stream carries, between them:
      //   sub-step 0      the LDS writes of step s+1 (registers loaded during step s-1)
      //   sub-step 1      the global loads of step s+2 and the hashing of step s+4
      //   every sub-step  the LDS reads of the next sub-step's fragments
      // The barrier sits before the last sub-step: by then every wavefront has issued (and
      // waited for) its last reads of stage s&1 and has written stage (s+1)&1, so the last
      // sub-step can already read the first fragments of step s+1, and the next step's writes
      // into stage s&1 are safe.
      // With direct staging the side jobs shrink to one: right after the barrier of step s,
      // when stage s&1 has been read for the last time, the direct-to-LDS loads of step s+2
      // are issued into it; they have a whole step to land and are waited for just before the
      // barrier of step s+1.
      constexpr int NKS = TR / KS / WK;   // sub-steps of this wavefront's part of an R step
      // fp32: left to itself the compiler moves a sub-step's fragment reads down to just before
      // the MFMAs that use them (read, wait, four MFMAs).  Holding them a sub-step ahead, as
      // written, is faster in the 64 tile (1024^3: 28.7 -> 27.4 us forward, 33.8 -> 31.4 us
      // weight-grad) and in the 256 tile's input-grad (M = 32768, K = N = 2048: 2110 -> 2003 us),
      // slower elsewhere (4096^3 forward 996 -> 1031 us; the 128 tile at 2048^3 154 -> 164 us).
      constexpr bool kPinFrags = !kDirect && sizeof(T) == 4 && (TI == 64 || (TI == 256 && OP == kInputGrad));
      static_assert(NKS >= 3 && NKS * KS * WK == TR, "pipeline needs at least three sub-steps per R step");
      const int ks0 = wave_k * NKS;
      Frag fa[2][MI], fb[2][MJ];
      auto frags = [&](int st, int ks, int buf) {
#pragma unroll
        for (int a = 0; a < MI; a++)
          fa[buf][a] = lds_frag<A_LAYOUT, LA>(sm.a[st], blk_i(a), ks0 + ks, lane);
#pragma unroll
        for (int b = 0; b < MJ; b++)
          fb[buf][b] = lds_frag<B_LAYOUT, LB>(sm.b[st], blk_j(b), ks0 + ks, lane);
      };
      auto mfmas = [&](int buf) {
#pragma unroll
        for (int a = 0; a < MI; a++)
#pragma unroll
          for (int b = 0; b < MJ; b++) acc[a][b] = mma(fa[buf][a], fb[buf][b], acc[a][b]);
      };
      // one R step; the flags say which of the side jobs still exist near the end of the loop
      // `late` staggers the side jobs of the two wavefronts that share a SIMD: one does them
      // during the first sub-steps, the other during the last ones, so that while one issues
      // LDS writes and global loads the other keeps the MFMA pipe fed.
      auto step = [&](int s, auto late, auto do_commit, auto do_fetch, auto has_next) {
        constexpr int kCommitAt = decltype(late)::value ? NKS - 2 : 0;
        constexpr int kFetchAt = kCommitAt;   // right behind the LDS writes that free the registers
        const int st = s & 1;
        // (its few threads branch, which ends a scheduling region: keep it out of the MFMA stream)
        if constexpr (decltype(do_fetch)::value) hash_ahead(s);
#pragma unroll
        for (int ks = 0; ks < NKS; ks++) {
          if (ks + 1 < NKS) {
            frags(st, ks + 1, (ks + 1) & 1);
            if constexpr (kPinFrags) __builtin_amdgcn_sched_barrier(0);
          } else {
            if constexpr (kDirect) {
              // the loads of step s+1 (the only ones in flight) must have landed
              if constexpr (decltype(has_next)::value) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            }
            __syncthreads();
            if constexpr (kDirect) {
              // stage st has been read for the last time: refill it for step s+2
              if constexpr (decltype(do_fetch)::value) direct_issue(s + 2, st);
              // (no refill left = the next step is the last one: it may be a partial step)
              if constexpr (decltype(has_next)::value && !decltype(do_fetch)::value) clear_tail(st ^ 1);
            }
            if constexpr (decltype(has_next)::value) frags(st ^ 1, 0, (ks + 1) & 1);
          }
          if constexpr (kDirect && COLSUM) {
            if (ks == 1) colsum_from_stage(st);   // once per R step, in step order
          }
          if constexpr (!kDirect) {
            if (ks == kCommitAt) {
              if constexpr (decltype(do_commit)::value) commit(st ^ 1);
            }
            if (ks == kFetchAt) {
              if constexpr (decltype(do_fetch)::value) fetch(s + 2);
            }
          }
          mfmas(ks & 1);
        }
      };
      auto loop = [&](auto late) {
        int s = 0;
        for (; s + 2 < steps; s++) step(s, late, std::true_type{}, std::true_type{}, std::true_type{});
        if (s + 1 < steps) {
          step(s, late, std::true_type{}, std::false_type{}, std::true_type{});
          s++;
        }
        step(s, late, std::false_type{}, std::false_type{}, std::false_type{});
      };
      if (steps > 0) {
        if constexpr (kDirect) {
          direct_issue(0, 0);
          if (steps > 1) {
            direct_issue(1, 1);
            // loads complete in order: all but the last step's worth have landed
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LA::kPieces + LB::kPieces) : "memory");
          } else {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
          }
        } else {
          commit(0);
          if (steps > 1) fetch(1);
        }
        __syncthreads();
        if constexpr (kDirect) {
          if (steps == 1) clear_tail(0);
        }
        frags(0, 0, 0);
        // wavefronts w and w + 4 of a workgroup share a SIMD
        if (kThreads == 512 && wave >= 4) loop(std::true_type{});
        else loop(std::false_type{});
      }
    }

    // ---- epilogue ---------------------------------------------------------------------------
    // accumulator element e of a 32x32 block: row (e/4)*8 + (lane/32)*4 + e%4, column lane%32
    if constexpr (OP == kWeightGrad) {
      const bool image_mode = p.image_pitch > 0;
      float* image = reinterpret_cast<float*>(&sm);   // aliases the operand stages
      __syncthreads();                                 // every wavefront is done reading them
      if constexpr (COLSUM) {
        // combine the threads that share columns (fixed order), one row of partial sums out
        constexpr int kGroups = kThreads / LB::kCpr;
        static_assert(sizeof(float) * kGroups * TJ <= sizeof(Smem), "column sums must fit the stages");
#pragma unroll
        for (int e = 0; e < VEC; e++) image[(tid / LB::kCpr) * TJ + (tid % LB::kCpr) * VEC + e] = colsum[e];
        __syncthreads();
        for (int c = tid; c < TJ; c += kThreads) {
          float s = 0.f;
          for (int g = 0; g < kGroups; g++) s += image[g * TJ + c];
          p.colsum[((size_t)by * p.tiles_i + ti) * (size_t)p.colsum_pitch + j0 + c] = s;
        }
        __syncthreads();
      }
      if (image_mode) {
        const float4 z = {0.f, 0.f, 0.f, 0.f};
        for (int i = tid * 4; i < p.image_pitch; i += kThreads * 4) *reinterpret_cast<float4*>(image + i) = z;
      }
      // offset table of this C tile's hashed tiles: behind the image (which may be larger
      // than the operand stages), else in its usual place
      int* etab = image_mode ? reinterpret_cast<int*>(image + p.image_pitch) : sm.off;
      const OffWindow w = off_window(p.h, i0, TI, j0, TJ);
      const bool tiled = p.tiles_out != nullptr;
      for (int t = tid; t < w.count; t += kThreads) {
        const int tk = w.tk0 + t / w.ntn, tn = w.tn0 + t % w.ntn;
        if (tiled)   // where the tile starts in the tile-by-tile output (-1: the C tile reaches beyond the grid)
          etab[t] = (tk < p.out_tiles_k && tn < p.out_tiles_n)
                        ? ((by * p.out_tiles_k + tk) * p.out_tiles_n + tn) << (p.h.bk_shift + p.h.bn_shift)
                        : -1;
        else
          etab[t] = (int)tile_offset(p.h, (uint32_t)tk, (uint32_t)tn);
      }
      __syncthreads();
      // No scatter: the accumulators are stored plainly, hashed tile by hashed tile (whole tiles:
      // zeros where a tile reaches beyond K x N); the fold kernel adds the tiles into dHW.
      auto store_tiles = [&](auto narrow) {
        // (narrow: the tiles are kept in the layer's 16-bit dtype — each value rounded once here, added up in fp32 by the fold)
        constexpr bool kNarrow = decltype(narrow)::value;
        T* const out16 = reinterpret_cast<T*>(p.tiles_out);
#pragma unroll
        for (int a = 0; a < MI; a++)
#pragma unroll
          for (int b = 0; b < MJ; b++) {
            const int n = j0 + blk_j(b) + (lane & 31);
            int base[4];
#pragma unroll
            for (int g = 0; g < 4; g++) {
              const int k = i0 + blk_i(a) + g * 8 + (lane >> 5) * 4;
              const int start = etab[((k >> p.h.bk_shift) - w.tk0) * w.ntn + ((n >> p.h.bn_shift) - w.tn0)];
              base[g] = start < 0 ? -1 : start + (k & (p.h.BK - 1)) * p.h.BN + (n & (p.h.BN - 1));
            }
#pragma unroll
            for (int e = 0; e < 16; e++) {
              const int k = i0 + blk_i(a) + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
              const bool inside = FULL || (k < p.I && n < p.J);
              if (FULL || base[e >> 2] >= 0) {
                const float v = inside ? acc[a][b][e] * p.scale : 0.f;
                const uint32_t at = (uint32_t)(base[e >> 2] + (e & 3) * p.h.BN);
                if constexpr (kNarrow) out16[at] = Tr::from_float(v);
                else p.tiles_out[at] = v;
              }
            }
          }
      };
      // Scatter-add of the accumulators.  The four rows e&3 of a row group (e>>2) are adjacent
      // rows of one hashed tile (tiles are at least 16 rows), so one table lookup per row
      // group gives all four addresses; the lookups of a 32x32 block are issued together and
      // the adds follow back to back.
      auto scatter = [&](float* target) {
        if (steps <= 0) return;
#pragma unroll
        for (int a = 0; a < MI; a++)
#pragma unroll
          for (int b = 0; b < MJ; b++) {
            const int n = j0 + blk_j(b) + (lane & 31);
            int base[4];
            bool ok[4];
#pragma unroll
            for (int g = 0; g < 4; g++) {
              const int k = i0 + blk_i(a) + g * 8 + (lane >> 5) * 4;
              ok[g] = FULL || (k < p.I && n < p.J);
              base[g] = etab[((k >> p.h.bk_shift) - w.tk0) * w.ntn + ((n >> p.h.bn_shift) - w.tn0)] +
                        (k & (p.h.BK - 1)) * p.h.BN + (n & (p.h.BN - 1));
            }
#pragma unroll
            for (int e = 0; e < 16; e++) {
              const int k = i0 + blk_i(a) + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
              if (FULL || (ok[e >> 2] && k < p.I))
                unsafeAtomicAdd(target + base[e >> 2] + (e & 3) * p.h.BN, acc[a][b][e] * p.scale);
            }
          }
      };
      if (tiled) {
        if (sizeof(T) == 2 && p.tiles_out_16) store_tiles(std::true_type{});   // (uniform)
        else store_tiles(std::false_type{});
      } else if (image_mode) {
        // Tiles of one workgroup overlap in hashed_weight: sum them in an LDS image of dHW
        // first, then store the image as this workgroup's partial result.
        if (p.h.bk_shift >= 5 && p.h.bn_shift >= 5) {
          // Every 32x32 accumulator block lies inside one hashed tile, whose BK*BN addresses
          // are all distinct.  LDS float atomics are slow, so instead the tiles of the window
          // take turns: in a round only the blocks of that round's tile(s) are added, with plain
          // read-add-write, and a barrier separates the rounds.
          int blk_tile[MI][MJ], blk_base[MI][MJ];
#pragma unroll
          for (int a = 0; a < MI; a++)
#pragma unroll
            for (int b = 0; b < MJ; b++) {
              const int k0 = i0 + blk_i(a), n0 = j0 + blk_j(b);
              const int t = __builtin_amdgcn_readfirstlane(((k0 >> p.h.bk_shift) - w.tk0) * w.ntn +
                                                           ((n0 >> p.h.bn_shift) - w.tn0));
              blk_tile[a][b] = t;
              blk_base[a][b] = etab[t] + ((k0 & (p.h.BK - 1)) + (lane >> 5) * 4) * p.h.BN +
                               ((n0 + (lane & 31)) & (p.h.BN - 1));
            }
          // With many hashed tiles per C tile, tiles whose slices do not meet may share a round:
          // a tile's round is one later than the latest round of the EARLIER tiles that meet its
          // slice (round 0 if none does), so every element still receives its adds in tile order
          // and the result has the same bits as with one round per tile.  The first wavefront
          // works the rounds out, tile by tile: lane j keeps the tiles of round j as a bit mask.
          int rounds = w.count;
          const bool levelled = w.count > 16 && w.count <= 64;
          if (levelled) {
            int* turn = etab + kOffEntries;             // [count] rounds, then their number
            if (wave == 0) {
              const int off_u = lane < w.count ? etab[lane] : 0;
              const int extent = p.h.BK * p.h.BN;
              unsigned long long members = 0ull;
              int my_turn = 0, turns = 1;
              for (int t = 0; t < w.count; t++) {
                const int d = off_u - __builtin_amdgcn_readlane(off_u, t);
                const unsigned long long meets = __ballot(lane < t && d < extent && d > -extent);
                const unsigned long long busy = __ballot((members & meets) != 0ull);   // rounds with a tile that meets t
                const int k = busy ? 64 - __builtin_clzll(busy) : 0;
                if (lane == k) members |= 1ull << t;
                if (lane == t) my_turn = k;
                turns = k + 1 > turns ? k + 1 : turns;
              }
              if (lane < w.count) turn[lane] = my_turn;
              if (lane == 0) turn[64] = turns;
            }
            __syncthreads();
            rounds = __builtin_amdgcn_readfirstlane(turn[64]);
#pragma unroll
            for (int a = 0; a < MI; a++)
#pragma unroll
              for (int b = 0; b < MJ; b++) blk_tile[a][b] = __builtin_amdgcn_readfirstlane(turn[blk_tile[a][b]]);
          }
          for (int t = 0; t < rounds; t++) {
            if (steps > 0) {
#pragma unroll
              for (int a = 0; a < MI; a++)
#pragma unroll
                for (int b = 0; b < MJ; b++) {
                  if (blk_tile[a][b] == t) {
                    const int k0 = i0 + blk_i(a) + (lane >> 5) * 4;
                    const bool col_ok = FULL || (j0 + blk_j(b) + (lane & 31) < p.J);
                    float cur[16];
#pragma unroll
                    for (int e = 0; e < 16; e++)
                      cur[e] = image[blk_base[a][b] + ((e >> 2) * 8 + (e & 3)) * p.h.BN];
#pragma unroll
                    for (int e = 0; e < 16; e++)
                      if (FULL || (col_ok && k0 + (e >> 2) * 8 + (e & 3) < p.I))
                        image[blk_base[a][b] + ((e >> 2) * 8 + (e & 3)) * p.h.BN] =
                            cur[e] + acc[a][b][e] * p.scale;
                  }
                }
            }
            __syncthreads();
          }
        } else {
          scatter(image);
          __syncthreads();
        }
        float* dst = p.scatter + ((size_t)by * gx + bx) * (size_t)p.image_pitch;
        for (int i = tid * 4; i < p.image_pitch; i += kThreads * 4)
          *reinterpret_cast<float4*>(dst + i) = *reinterpret_cast<const float4*>(image + i);
      } else {
        scatter(p.scatter);
      }
    } else {
      if constexpr (WK > 1) {
        // add up the groups' accumulators: groups 1.. park theirs in the dead operand stages,
        // group 0 adds them (fixed order) and stores the tile
        float* park = reinterpret_cast<float*>(&sm);
        static_assert(sizeof(float) * (WK - 1) * TI * TJ <= sizeof(Smem), "the accumulators must fit the stages");
        __syncthreads();   // every wavefront is done reading the stages
        const int slot = ((wave % (WI * WJ)) * MI * MJ) * 16 * 64 + lane;
        if (wave_k > 0) {
#pragma unroll
          for (int a = 0; a < MI; a++)
#pragma unroll
            for (int b = 0; b < MJ; b++)
#pragma unroll
              for (int e = 0; e < 16; e++)
                park[(wave_k - 1) * TI * TJ + slot + ((a * MJ + b) * 16 + e) * 64] = acc[a][b][e];
        }
        __syncthreads();
        if (wave_k == 0) {
#pragma unroll
          for (int g = 1; g < WK; g++)
#pragma unroll
            for (int a = 0; a < MI; a++)
#pragma unroll
              for (int b = 0; b < MJ; b++)
#pragma unroll
                for (int e = 0; e < 16; e++)
                  acc[a][b][e] += park[(g - 1) * TI * TJ + slot + ((a * MJ + b) * 16 + e) * 64];
        }
      }
      // (of several groups of wavefronts that shared the R steps, the first holds the sums and stores)
      const bool writer = wave_k == 0;   // (uniform)
      float out_scale = p.scale;
      const T* __restrict__ gBias = static_cast<const T*>(p.bias);
      // optional bias of this lane's columns, added in fp32 before the single rounding
      float bias[MJ];
#pragma unroll
      for (int b = 0; b < MJ; b++) {
        const int col = j0 + blk_j(b) + (lane & 31);
        bias[b] = 0.f;
        if (gBias != nullptr && (FULL || col < p.J)) bias[b] = Tr::to_float(gBias[col]);
      }
      if (p.partial != nullptr) {
        // R is split over the slices `by` (few C tiles, long R): this slice's scaled fp32 partial
        // result goes to its own [I][J] plane.  The planes are added up by a second kernel — or,
        // with a counter per C tile (p.finish), by the slice that arrives at the tile last: it
        // adds the planes in slice order, its own from its registers (the same bits it stored),
        // so the sum does not depend on who came last; nobody waits for anybody.
        float* __restrict__ gP = p.partial + (size_t)by * (size_t)p.I * (size_t)p.J;
        const bool finishing = p.finish != nullptr;   // (uniform)
        if (writer) {
#pragma unroll
          for (int a = 0; a < MI; a++) {
#pragma unroll
            for (int e = 0; e < 16; e++) {
              const int row = i0 + blk_i(a) + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
#pragma unroll
              for (int b = 0; b < MJ; b++) {
                const int col = j0 + blk_j(b) + (lane & 31);
                if (FULL || (row < p.I && col < p.J)) {
                  if (finishing) store_agent_f32(gP + (size_t)row * p.J + col, acc[a][b][e] * p.scale);
                  else gP[(size_t)row * p.J + col] = acc[a][b][e] * p.scale;
                }
              }
            }
          }
        }
        if (!finishing) return;
        const int slices = (int)gridDim.y;
        unsigned* counter = p.finish + (size_t)ti * (size_t)p.tiles_j + tj;
        int* arrived = reinterpret_cast<int*>(&sm);   // (the stages are dead)
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this wavefront's part of the plane is where the others will look
        __syncthreads();
        if (tid == 0) *arrived = (int)__hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (*arrived != slices - 1) return;   // (uniform) another slice will finish this tile
        if (tid == 0) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // (as the next launch expects it)
        if (!writer) return;
        const size_t plane = (size_t)p.I * (size_t)p.J;
#pragma unroll
        for (int a = 0; a < MI; a++) {
#pragma unroll
          for (int b = 0; b < MJ; b++) {
            const int col = j0 + blk_j(b) + (lane & 31);
            // (half a block at a time: the other slices' values of eight rows are fetched before the first is
            //  used — a whole block's would cost registers that the two-workgroup forms do not have)
#pragma unroll
            for (int h = 0; h < 2; h++) {
              float v[kFinishSlices][8];
#pragma unroll
              for (int sl = 0; sl < kFinishSlices; sl++) {
                if (sl < slices && sl != by) {   // (uniform)
#pragma unroll
                  for (int e = 0; e < 8; e++) {
                    const int row = i0 + blk_i(a) + (h * 2 + (e >> 2)) * 8 + (lane >> 5) * 4 + (e & 3);
                    v[sl][e] = (FULL || (row < p.I && col < p.J)) ? load_agent_f32(p.partial + (size_t)sl * plane + (size_t)row * p.J + col) : 0.f;
                  }
                }
              }
              float sum[8];
#pragma unroll
              for (int e = 0; e < 8; e++) sum[e] = 0.f;
#pragma unroll
              for (int sl = 0; sl < kFinishSlices; sl++) {
                if (sl == by) {
#pragma unroll
                  for (int e = 0; e < 8; e++) sum[e] += __fmul_rn(acc[a][b][h * 8 + e], p.scale);   // (the product as it was stored: not fused into the add)
                } else if (sl < slices) {
#pragma unroll
                  for (int e = 0; e < 8; e++) sum[e] += v[sl][e];
                }
              }
              // (the bias joins the fp32 sum as in the second kernel: an add of its own, rounded to fp32,
              //  not part of a fused multiply-add that rounds straight to the output type)
#pragma unroll
              for (int e = 0; e < 8; e++) acc[a][b][h * 8 + e] = __fadd_rn(sum[e], bias[b]);
            }
          }
        }
        out_scale = 1.f;
#pragma unroll
        for (int b = 0; b < MJ; b++) bias[b] = 0.f;
      }
      if (!writer) return;
      T* __restrict__ gC = static_cast<T*>(p.C);
      // the column blocks of a row go out back to back, so that the halves of a cache line
      // reach L2 together.  A large C is stored with streaming stores: nothing here reads it
      // again, and kept in L2 it would push out the operand panels that the workgroups of the
      // next round still share (ffn input-grad, 64 MB of dX: 883 -> 861 us).
      auto store_c = [&](auto streaming) {
#pragma unroll
        for (int a = 0; a < MI; a++) {
#pragma unroll
          for (int e = 0; e < 16; e++) {
            const int row = i0 + blk_i(a) + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
#pragma unroll
            for (int b = 0; b < MJ; b++) {
              const int col = j0 + blk_j(b) + (lane & 31);
              if (FULL || (row < p.I && col < p.J)) {
                const T value = Tr::from_float(acc[a][b][e] * out_scale + bias[b]);
                T* dst = gC + (int64_t)row * p.ldc + col;
                if constexpr (!decltype(streaming)::value) *dst = value;
                else if constexpr (sizeof(T) == 4) __builtin_nontemporal_store(value, dst);
                else __builtin_nontemporal_store(value.bits, &dst->bits);
              }
            }
          }
        }
      };
      if (p.stream_c) store_c(std::true_type{});
      else store_c(std::false_type{});
    }
  }
};

template <typename T, int OP, int TI, int TJ, int WI, int WJ, int NSTAGE, bool FULL, bool COLSUM, bool CLAMP, int WK = 1>
__global__ __launch_bounds__(64 * WI * WJ * WK) void rz_gemm_kernel(GemmParams p) {
  typedef GemmKernel<T, OP, TI, TJ, WI, WJ, NSTAGE, FULL, COLSUM, CLAMP, WK> K;
  extern __shared__ __attribute__((aligned(16))) unsigned char rz_smem_raw[];
  K::run(p, *reinterpret_cast<typename K::Smem*>(rz_smem_raw));
}

}  // namespace rz
