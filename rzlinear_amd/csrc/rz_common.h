// Shared device/host definitions of the gfx950 RzLinear kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace rz {

// ---- element types -------------------------------------------------------------------------
// 16-bit floats travel as raw uint16_t; only the MFMA builtins and the final conversion care
// which format they are.
struct bf16_t { uint16_t bits; };
struct f16_t { uint16_t bits; };

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(4))) short s16x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;

template <typename T> struct ElemTraits;
template <> struct ElemTraits<float> {
  static constexpr int kBytes = 4;
  static constexpr int kVec = 4;        // elements per 16-byte chunk
  static constexpr int kMfmaK = 2;      // contraction depth of one v_mfma_f32_32x32x2_f32
  static __device__ __forceinline__ float from_float(float v) { return v; }
  static __device__ __forceinline__ float to_float(float v) { return v; }
};
template <> struct ElemTraits<bf16_t> {
  static constexpr int kBytes = 2;
  static constexpr int kVec = 8;
  static constexpr int kMfmaK = 16;     // v_mfma_f32_32x32x16_bf16
  static __device__ __forceinline__ bf16_t from_float(float v) {
    __bf16 b = (__bf16)v;               // round to nearest even
    bf16_t r;
    __builtin_memcpy(&r.bits, &b, 2);
    return r;
  }
  static __device__ __forceinline__ float to_float(bf16_t v) {
    uint32_t u = (uint32_t)v.bits << 16;
    float f;
    __builtin_memcpy(&f, &u, 4);
    return f;
  }
};
template <> struct ElemTraits<f16_t> {
  static constexpr int kBytes = 2;
  static constexpr int kVec = 8;
  static constexpr int kMfmaK = 16;     // v_mfma_f32_32x32x16_f16
  static __device__ __forceinline__ f16_t from_float(float v) {
    _Float16 h = (_Float16)v;
    f16_t r;
    __builtin_memcpy(&r.bits, &h, 2);
    return r;
  }
  static __device__ __forceinline__ float to_float(f16_t v) {
    _Float16 h;
    __builtin_memcpy(&h, &v.bits, 2);
    return (float)h;
  }
};

// ---- tile hash -----------------------------------------------------------------------------
// off(tk,tn) = (((tk*R3 + tn*R2 + R1) % R0) * R0 + ((tk*R7 + tn*R5 + R4) % R0)) % (H - BK*BN)
// (levels == 1 keeps only the first term).  The host checks that every intermediate stays
// below 2^31, so unsigned 32-bit arithmetic equals the reference's signed 32-bit arithmetic.
// levels == 3 is the legacy generation's tile hash: the first term alone, evaluated in 64-bit
// integers (its prime is close to 2^31), modulo H - BK*BN + 1; `range` then holds that value.
struct HashParams {
  uint32_t R0, R1, R2, R3, R4, R5, R7;
  uint32_t range;      // H - BK*BN  (legacy hash: H - BK*BN + 1)
  int bk_shift, bn_shift;
  int BK, BN;
  int levels;
};

__host__ __device__ __forceinline__ uint32_t tile_offset(const HashParams& h, uint32_t tk,
                                                         uint32_t tn) {
  if (h.levels == 3)
    return (uint32_t)((((uint64_t)tk * h.R3 + (uint64_t)tn * h.R2 + h.R1) % h.R0) % h.range);
  const uint32_t hi = (tk * h.R3 + tn * h.R2 + h.R1) % h.R0;
  if (h.levels == 1) return hi % h.range;
  const uint32_t lo = (tk * h.R7 + tn * h.R5 + h.R4) % h.R0;
  return (hi * h.R0 + lo) % h.range;
}

// ---- the three contractions as one GEMM shape ----------------------------------------------
// C[I,J] = sum_r A(i,r) * B(r,j)
//   forward      I=M J=N R=K   A = X  (rows i, contiguous r)   B = W tiles (rows r=k, contiguous j=n)
//   input-grad   I=M J=K R=N   A = dY (rows i, contiguous r)   B = W tiles (rows j=k, contiguous r=n)
//   weight-grad  I=K J=N R=M   A = X  (rows r=m, contiguous i) B = dY      (rows r=m, contiguous j)
enum Op { kForward = 0, kInputGrad = 1, kWeightGrad = 2 };

// Slices of a cut contraction whose values the kernel that finishes its own tiles holds at a time
// (GemmParams::finish; see finish_slices in rz_launch.h).
static constexpr int kFinishSlices = 4;

struct GemmParams {
  const void* A;
  const void* B;      // plain B operand (weight-grad) — else unused
  const void* HW;     // hashed weight (forward, input-grad)
  void* C;            // plain output (forward, input-grad)
  int stream_c;       // ... stored with streaming (non-temporal) stores: for outputs far larger than the L2
  const void* bias;   // optional [J] vector added to every row of C (forward), or null
  float* partial;     // forward/input-grad with R split over blockIdx.y: fp32 partial results
                      // [slices][I][J] (scaled, no bias) instead of C; null = no split
  unsigned* finish;   // ... with one counter per C tile (zero between launches): the slice that arrives
                      // last at a tile adds the slices up itself and stores C (+ bias); null = a second
                      // kernel does
  float* scatter;     // weight-grad target: fp32 image of dHW (direct atomics), or the
                      // per-workgroup partial images [workgroups][image_pitch] (LDS mode)
  int image_pitch;    // > 0 selects the LDS mode: floats per partial image (H rounded up to 4)
  float* tiles_out;   // weight-grad, non-null: no scatter at all; the C tile (scaled X^T.dY) is stored
                      // hashed tile by hashed tile, tile (tk, tn) of slice s as BK*BN contiguous floats
                      // at ((s * tiles_k + tk) * tiles_n + tn) * BK*BN (only the part inside K x N is defined), and a
                      // second kernel folds the tiles into dHW
  int tiles_out_16;   // ... as elements of the layer's 16-bit dtype instead of floats (same element indices)
  int out_tiles_k, out_tiles_n;   // ... its tile grid: ceil(K / BK) x ceil(N / BN)
  float* colsum;      // weight-grad that also yields the bias gradient: partial column sums of B
                      // (dY), one row per (slice, tile row): [slices * tiles_i][colsum_pitch]
  int colsum_pitch;   // floats per row of colsum (J rounded up to the tile)
  int I, J, R;
  int64_t lda, ldb, ldc;
  int tiles_i, tiles_j;
  int r_chunk;        // rows of R handled by one blockIdx.y slice (multiple of the R step)
  float scale;
  HashParams h;
};

// Loads and stores at agent scope: for data that another workgroup of the SAME kernel wrote or will
// read (such accesses go to the point where the GPU's L2 caches agree; a wavefront that has waited
// for its own stores may then tell the others, through an atomic, that they are there).
__device__ __forceinline__ void store_agent_f32(float* at, float v) {
  __hip_atomic_store(at, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_agent_f32(const float* at) {
  return __hip_atomic_load(at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace rz
