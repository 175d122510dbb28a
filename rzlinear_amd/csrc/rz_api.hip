// C ABI of librzlinear: argument checks, the host-side tile hash, small utility kernels
// (materialise, device-side offsets, zero fill, fp32 -> element conversion) and dispatch to
// the contraction kernels.
#include "../../include/rzlinear.h"

#include <atomic>

#include "rz_common.h"
#include "rz_fold.h"
#include "rz_launch.h"
#include "rz_window.h"

namespace rz {

static int ilog2_exact(int v) {
  int s = 0;
  while ((1 << s) < v) s++;
  return ((1 << s) == v) ? s : -1;
}

static int check_tile(int BK, int BN) {
  if (BK < 16 || BK > 256 || BN < 16 || BN > 256) return RZ_ERR_BAD_TILE;
  if (ilog2_exact(BK) < 0 || ilog2_exact(BN) < 0) return RZ_ERR_BAD_TILE;
  return RZ_OK;
}

// Validates the hash inputs and fills HashParams.  The reference evaluates the hash in
// signed 32-bit arithmetic; reject inputs whose intermediates would not fit, rather than
// silently computing something else.
static int make_hash(HashParams* h, int K, int N, int H, int BK, int BN, const int32_t* R,
                     int levels) {
  if (R == nullptr) return RZ_ERR_NULL_POINTER;
  if (K < 1 || N < 1 || H < 1) return RZ_ERR_BAD_SHAPE;
  int st = check_tile(BK, BN);
  if (st != RZ_OK) return st;
  if (levels != RZ_HASH_ONE_LEVEL && levels != RZ_HASH_TWO_LEVEL && levels != RZ_HASH_LEGACY)
    return RZ_ERR_BAD_ARGUMENT;
  const bool legacy = levels == RZ_HASH_LEGACY;
  if (legacy ? (long long)H < (long long)BK * BN : (long long)H <= (long long)BK * BN)
    return RZ_ERR_HASH_RANGE;
  for (int i = 0; i < 8; i++)
    if (R[i] < 0) return RZ_ERR_BAD_ARGUMENT;
  if (R[0] < 1) return RZ_ERR_BAD_ARGUMENT;
  const long long lim = 2147483647LL;
  const long long TK = ((long long)K + BK - 1) / BK, TN = ((long long)N + BN - 1) / BN;
  if (!legacy) {   // the legacy hash is evaluated in 64-bit integers and cannot overflow them
    if (TK * R[3] + TN * R[2] + R[1] > lim) return RZ_ERR_HASH_OVERFLOW;
    if (TK * R[7] + TN * R[5] + R[4] > lim) return RZ_ERR_HASH_OVERFLOW;
    if (levels == 2 && ((long long)R[0] - 1) * R[0] + (R[0] - 1) > lim) return RZ_ERR_HASH_OVERFLOW;
  }
  h->R0 = (uint32_t)R[0];
  h->R1 = (uint32_t)R[1];
  h->R2 = (uint32_t)R[2];
  h->R3 = (uint32_t)R[3];
  h->R4 = (uint32_t)R[4];
  h->R5 = (uint32_t)R[5];
  h->R7 = (uint32_t)R[7];
  h->range = (uint32_t)(H - BK * BN + (legacy ? 1 : 0));
  h->BK = BK;
  h->BN = BN;
  h->bk_shift = ilog2_exact(BK);
  h->bn_shift = ilog2_exact(BN);
  h->levels = levels;
  return RZ_OK;
}

// Row pitches are limited so that a tile's rows stay within the 32-bit byte offsets of the kernels'
// load addresses (256 rows of 2^23 four-byte elements are 2^33 bytes: the limit is per element type below).
static bool pitch_ok(int64_t ld, int elem_bytes) { return ld > 0 && ld * elem_bytes * 256 < (1LL << 32); }

static int dtype_bytes(int dtype) {
  switch (dtype) {
    case RZ_F32: return 4;
    case RZ_BF16:
    case RZ_F16: return 2;
    default: return 0;
  }
}

static hipError_t launch_gemm(int dtype, int op, const GemmParams& p, const WeightGradPlan* plan,
                              const SplitPlan* split, const rz_tuning& tuning, hipStream_t s) {
  switch (dtype) {
    case RZ_F32: return launch_gemm_f32(op, p, plan, split, tuning, s);
    case RZ_BF16: return launch_gemm_bf16(op, p, plan, split, tuning, s);
    case RZ_F16: return launch_gemm_f16(op, p, plan, split, tuning, s);
    default: return hipErrorInvalidValue;
  }
}

// ---- utility kernels ------------------------------------------------------------------------
__global__ void tile_offsets_kernel(int32_t* out, int TK, int TN, HashParams h) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t < TK * TN) out[t] = (int32_t)tile_offset(h, (uint32_t)(t / TN), (uint32_t)(t % TN));
}

// One workgroup per W tile: the slice is copied row by row, clipped at K and N.
template <typename E>
__global__ void materialize_kernel(const E* __restrict__ hw, E* __restrict__ W, int K, int N, int TN,
                                   int64_t ldw, HashParams h) {
  const int tk = blockIdx.x / TN, tn = blockIdx.x % TN;
  const uint32_t off = tile_offset(h, (uint32_t)tk, (uint32_t)tn);
  const int elems = h.BK * h.BN;
  for (int e = threadIdx.x; e < elems; e += blockDim.x) {
    const int kk = e >> h.bn_shift, nn = e & (h.BN - 1);
    const int k = tk * h.BK + kk, n = tn * h.BN + nn;
    if (k < K && n < N) W[(int64_t)k * ldw + n] = hw[off + e];
  }
}

__global__ void fill_zero_kernel(uint32_t* p, size_t words) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < words; i += stride) p[i] = 0u;
}

// dst[i] = src[i] (+ dst[i] when ACC), converted to the element type.
template <typename T, bool ACC>
__global__ void convert_from_f32_kernel(const float* __restrict__ src, T* __restrict__ dst, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = ElemTraits<T>::from_float(src[i] + (ACC ? ElemTraits<T>::to_float(dst[i]) : 0.f));
}

// dHW[h] = sum over the partial images of part[p][h] (+ dHW[h] when ACC), converted to the
// element type.  A workgroup of 256 threads owns 256 / GROUPS groups of four slots; GROUPS thread
// groups each add up every GROUPS-th partial image (all their loads in flight together when
// there are at most eight each), then the groups are combined through LDS in a fixed order, so the
// result does not depend on scheduling.
template <typename T, bool ACC, int GROUPS>
__global__ __launch_bounds__(256) void reduce_partials_kernel(const float* __restrict__ part,
                                                              T* __restrict__ out, int H, int pitch,
                                                              int nparts) {
  constexpr int kSlots = 256 / GROUPS;
  __shared__ float4 sums[GROUPS][kSlots];
  const int q = threadIdx.x % kSlots, g = threadIdx.x / kSlots;
  const int slot = (blockIdx.x * kSlots + q) * 4;
  float4 s = {0.f, 0.f, 0.f, 0.f};
  if (slot < pitch) {
    // eight loads in flight per thread; the order of the additions stays fixed
#pragma unroll 8
    for (int p = g; p < nparts; p += GROUPS) {
      const float4 v = *reinterpret_cast<const float4*>(part + (size_t)p * pitch + slot);
      s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
  }
  sums[g][q] = s;
  __syncthreads();
  if (g == 0 && slot < pitch) {
    for (int i = 1; i < GROUPS; i++) {
      const float4 v = sums[i][q];
      s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
    const float r[4] = {s.x, s.y, s.z, s.w};
#pragma unroll
    for (int e = 0; e < 4; e++)
      if (slot + e < H)
        out[slot + e] = ElemTraits<T>::from_float(r[e] + (ACC ? ElemTraits<T>::to_float(out[slot + e]) : 0.f));
  }
}

// dbias[n] = sum over the rows of part[row][n], converted to the element type.  A workgroup owns
// 64 columns; four thread groups each add up every fourth row (eight loads in flight), then
// the groups are combined through LDS in a fixed order.
template <typename T>
__global__ __launch_bounds__(256) void reduce_colsum_kernel(const float* __restrict__ part,
                                                            T* __restrict__ out, int N, int pitch, int rows) {
  __shared__ float sums[4][64];
  const int c = threadIdx.x & 63, g = threadIdx.x >> 6;
  const int n = blockIdx.x * 64 + c;
  float s = 0.f;
  if (n < N) {
#pragma unroll 8
    for (int r = g; r < rows; r += 4) s += part[(size_t)r * pitch + n];
  }
  sums[g][c] = s;
  __syncthreads();
  if (g == 0 && n < N) out[n] = ElemTraits<T>::from_float((sums[0][c] + sums[1][c]) + (sums[2][c] + sums[3][c]));
}

// dbias[n] = sum over the rows m of dY[m][n], for the weight-grad forms that do not stage dY
// tile by tile (the window kernel: short M).  A workgroup owns 64 columns; four thread groups
// each add up every fourth row, then the groups are combined through LDS in a fixed order.
template <typename T, typename O>
__global__ __launch_bounds__(256) void colsum_rows_kernel(const T* __restrict__ dY, int64_t ld, O* __restrict__ out,
                                                          int N, int M) {
  __shared__ float sums[4][64];
  const int c = threadIdx.x & 63, g = threadIdx.x >> 6;
  const int n = blockIdx.x * 64 + c;
  float s = 0.f;
  if (n < N) {
#pragma unroll 8
    for (int m = g; m < M; m += 4) s += ElemTraits<T>::to_float(dY[(int64_t)m * ld + n]);
  }
  sums[g][c] = s;
  __syncthreads();
  if (g == 0 && n < N) out[n] = ElemTraits<O>::from_float((sums[0][c] + sums[1][c]) + (sums[2][c] + sums[3][c]));
}

static void launch_colsum_rows(int dtype, int out_dtype, const void* dY, int64_t ld, void* out, int N, int M,
                               hipStream_t s) {
  const dim3 grid((N + 63) / 64), block(256);
  if (dtype == RZ_F32)
    hipLaunchKernelGGL((colsum_rows_kernel<float, float>), grid, block, 0, s, (const float*)dY, ld, (float*)out, N, M);
  else if (dtype == RZ_BF16 && out_dtype == RZ_F32)
    hipLaunchKernelGGL((colsum_rows_kernel<bf16_t, float>), grid, block, 0, s, (const bf16_t*)dY, ld, (float*)out, N, M);
  else if (dtype == RZ_BF16)
    hipLaunchKernelGGL((colsum_rows_kernel<bf16_t, bf16_t>), grid, block, 0, s, (const bf16_t*)dY, ld, (bf16_t*)out, N, M);
  else if (out_dtype == RZ_F32)
    hipLaunchKernelGGL((colsum_rows_kernel<f16_t, float>), grid, block, 0, s, (const f16_t*)dY, ld, (float*)out, N, M);
  else
    hipLaunchKernelGGL((colsum_rows_kernel<f16_t, f16_t>), grid, block, 0, s, (const f16_t*)dY, ld, (f16_t*)out, N, M);
}

// C[i][j] = sum over the slices of part[s][i][j] (+ bias[j]), converted to the element type.
template <typename T>
__global__ __launch_bounds__(256) void reduce_slices_kernel(const float* __restrict__ part,
                                                            T* __restrict__ C, const T* __restrict__ bias,
                                                            int I, int J, int64_t ldc, int slices) {
  const size_t plane = (size_t)I * (size_t)J;
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= plane) return;
  const int i = (int)(idx / J), j = (int)(idx % J);
  float s = 0.f;
  for (int k = 0; k < slices; k++) s += part[(size_t)k * plane + idx];
  if (bias != nullptr) s += ElemTraits<T>::to_float(bias[j]);
  C[(int64_t)i * ldc + j] = ElemTraits<T>::from_float(s);
}

template <typename T>
static hipError_t reduce_slices(const float* part, void* C, const void* bias, int I, int J, int64_t ldc,
                                int slices, hipStream_t s) {
  const size_t plane = (size_t)I * (size_t)J;
  const size_t blocks = (plane + 255) / 256;
  if (blocks > 0x7fffffffULL) return hipErrorInvalidValue;
  hipLaunchKernelGGL(reduce_slices_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, s, part, (T*)C,
                     (const T*)bias, I, J, ldc, slices);
  return hipGetLastError();
}

static hipError_t reduce_slices_dtype(int dtype, const float* part, void* C, const void* bias, int I, int J,
                                      int64_t ldc, int slices, hipStream_t s) {
  switch (dtype) {
    case RZ_F32: return reduce_slices<float>(part, C, bias, I, J, ldc, slices, s);
    case RZ_BF16: return reduce_slices<bf16_t>(part, C, bias, I, J, ldc, slices, s);
    case RZ_F16: return reduce_slices<f16_t>(part, C, bias, I, J, ldc, slices, s);
    default: return hipErrorInvalidValue;
  }
}

// ---- counters of the cut contractions that finish in one kernel ---------------------------------
// One 32-bit counter per tile of the output (GemmParams::finish), in a file-scope device array: zero
// when the library is loaded, and set back to zero by the workgroup that finishes a tile.  The array
// is divided among streams: the first sixteen streams per device that launch such a contraction each
// get a part of their own, for good; launches on one stream run one after the other and leave their
// counters at zero, so every launch of a stream starts at the first counter of the stream's part, and
// launches on different streams, which may run at the same time, never share a counter.  A stream
// beyond the sixteenth, a stream under capture (its kernels will run again later, on whatever stream the
// graph is launched on) and an output of more tiles than a part has counters get the second kernel
// instead.  In host code the array's name is a handle for hipGetSymbolAddress, looked up once per
// device with that device current.
static constexpr unsigned kFinishStreams = 16, kFinishPerStream = 4096;
static constexpr unsigned kFinishCounters = kFinishStreams * kFinishPerStream;
static constexpr int kFinishMaxDevices = 64;
static __device__ __align__(256) unsigned finish_counters[kFinishCounters];
static std::atomic<unsigned*> finish_counters_ptr[kFinishMaxDevices];
static std::atomic<uintptr_t> finish_owner[kFinishMaxDevices][kFinishStreams];   // stream handle + 1 (0: nobody's yet)

// Counters for a launch with `tiles` output tiles on stream s, or null (the caller then launches the second kernel).
static unsigned* finish_counters_for(long long tiles, hipStream_t s) {
  if (tiles < 1 || tiles > (long long)kFinishPerStream) return nullptr;
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &capture) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  if (capture != hipStreamCaptureStatusNone) return nullptr;
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kFinishMaxDevices) return nullptr;
  unsigned* base = finish_counters_ptr[dev].load(std::memory_order_acquire);
  if (base == nullptr) {
    void* q = nullptr;
    if (hipGetSymbolAddress(&q, HIP_SYMBOL(finish_counters)) != hipSuccess || q == nullptr) {
      (void)hipGetLastError();
      return nullptr;
    }
    base = static_cast<unsigned*>(q);
    finish_counters_ptr[dev].store(base, std::memory_order_release);   // (a racing thread stores the same value)
  }
  const uintptr_t key = reinterpret_cast<uintptr_t>(s) + 1;   // (the null stream has a part like any other)
  for (unsigned i = 0; i < kFinishStreams; i++) {
    uintptr_t owner = finish_owner[dev][i].load(std::memory_order_acquire);
    if (owner == 0 && finish_owner[dev][i].compare_exchange_strong(owner, key, std::memory_order_acq_rel)) owner = key;
    if (owner == key) return base + i * kFinishPerStream;
  }
  return nullptr;
}

// Forward (op kForward) or input-grad through one code path: p holds the operands; with a
// workspace the contraction may be split over R (skinny problems).
static int run_plain_op(int op, int dtype, GemmParams p, const void* bias, void* workspace,
                        size_t workspace_bytes, bool may_split, const rz_tuning& tuning, hipStream_t s) {
  // an output of more than twice an L2 goes out with streaming stores (a smaller one may still be
  // in cache when the next kernel reads it)
  p.stream_c = (size_t)p.I * (size_t)p.J * dtype_bytes(dtype) >= ((size_t)8 << 20) ? 1 : 0;
  if (may_split) {
    // tile and slices are chosen together
    const SplitPlan sp = plan_split(p.I, p.J, p.R, dtype_bytes(dtype), tuning);
    if (sp.splits > 1) {
      if (workspace == nullptr || workspace_bytes < sp.workspace_bytes) return RZ_ERR_WORKSPACE;
      p.partial = (float*)workspace;
      // the slice that arrives last at a tile finishes it (adds the slices in slice order, then the
      // bias: the bits of the second kernel's sum) — unless told otherwise, or out of counters
      p.finish = (tuning.finish != -1 && sp.splits <= finish_slices(sp.tile, p.I, p.J)) ? finish_counters_for(tile_count(p.I, p.J, sp.tile), s) : nullptr;
      p.bias = p.finish != nullptr ? bias : nullptr;
      if (launch_gemm(dtype, op, p, nullptr, &sp, tuning, s) != hipSuccess) return RZ_ERR_LAUNCH;
      if (p.finish != nullptr) return RZ_OK;
      return reduce_slices_dtype(dtype, p.partial, p.C, bias, p.I, p.J, p.ldc, sp.splits, s) == hipSuccess
                 ? RZ_OK : RZ_ERR_LAUNCH;
    }
    p.bias = bias;
    return launch_gemm(dtype, op, p, nullptr, &sp, tuning, s) == hipSuccess ? RZ_OK : RZ_ERR_LAUNCH;
  }
  p.bias = bias;
  return launch_gemm(dtype, op, p, nullptr, nullptr, tuning, s) == hipSuccess ? RZ_OK : RZ_ERR_LAUNCH;
}

static hipError_t zero_words(void* p, size_t bytes, hipStream_t s) {
  // bytes is a multiple of 4 for every caller (fp32 images)
  const size_t words = bytes / 4;
  if (words == 0) return hipSuccess;
  size_t blocks = (words + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)blocks), dim3(256), 0, s, (uint32_t*)p, words);
  return hipGetLastError();
}

// Launchers over the output element type (an rz_dtype code) of the weight-grad tail kernels.
template <bool ACC>
static void launch_reduce_partials(int out_dtype, const float* part, void* out, int H, int pitch, int nparts,
                                   hipStream_t s) {
  // (16 groups of 16 slots; 32 groups of 8 slots — twice the workgroups, every load of a thread in
  //  flight at once — were no faster: 7.0 against 5.7 us for 256 images of 67 KB)
  constexpr int GROUPS = 16, kSlots = 256 / GROUPS;
  const dim3 grid((pitch / 4 + kSlots - 1) / kSlots), block(256);
  if (out_dtype == RZ_F32)
    hipLaunchKernelGGL((reduce_partials_kernel<float, ACC, GROUPS>), grid, block, 0, s, part, (float*)out, H, pitch, nparts);
  else if (out_dtype == RZ_BF16)
    hipLaunchKernelGGL((reduce_partials_kernel<bf16_t, ACC, GROUPS>), grid, block, 0, s, part, (bf16_t*)out, H, pitch, nparts);
  else
    hipLaunchKernelGGL((reduce_partials_kernel<f16_t, ACC, GROUPS>), grid, block, 0, s, part, (f16_t*)out, H, pitch, nparts);
}

// (tile_dtype: what the contraction kernel stored the tiles as — floats, or the layer's 16-bit dtype)
static hipError_t launch_fold_small(const FoldParams& fp, int tile_dtype, hipStream_t s) {
  const long long tiles = (long long)fp.tiles_k * fp.tiles_n;
  if (fp.partial != nullptr || fp.out == nullptr || fp.shares != 1 || tiles > kFoldSmallTiles ||
      fp.window != kFoldSmallThreads || (long long)fp.windows * fp.window < fp.H)
    return hipErrorInvalidValue;
  const dim3 grid((unsigned)fp.windows), block(kFoldSmallThreads);
  if (tile_dtype == RZ_BF16) hipLaunchKernelGGL(fold_small_kernel<bf16_t>, grid, block, 0, s, fp);
  else if (tile_dtype == RZ_F16) hipLaunchKernelGGL(fold_small_kernel<f16_t>, grid, block, 0, s, fp);
  else hipLaunchKernelGGL(fold_small_kernel<float>, grid, block, 0, s, fp);
  return hipGetLastError();
}

template <typename TT>
static hipError_t launch_fold_as(const FoldParams& fp, hipStream_t s) {
  static std::atomic<uint64_t> raised{0};
  const size_t lds = fold_lds_bytes(fp.window);
  const int E = fp.h.BK * fp.h.BN, runs = E > kFoldRun ? E / kFoldRun : 1;
  if ((fp.partial == nullptr && (fp.shares != 1 || fp.out == nullptr)) || fp.window <= 0 || fp.window % kFoldThreads != 0 || fp.window > kFoldWindowMax ||
      fp.slices * runs * 4 > kFoldList || runs > 8 || fp.h.BK > 16384 || fp.h.BN > 16384 || (long long)fp.windows * fp.window < fp.H)
    return hipErrorInvalidValue;
  if (lds > 64 * 1024) {
    hipError_t e = raise_lds_limit(reinterpret_cast<const void*>(fold_tiles_kernel<TT>), raised);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(fold_tiles_kernel<TT>, dim3((unsigned)(fp.windows * fp.shares)), dim3(kFoldThreads), lds, s, fp);
  return hipGetLastError();
}

static hipError_t launch_fold(const FoldParams& fp, int tile_dtype, hipStream_t s) {
  return tile_dtype == RZ_BF16 ? launch_fold_as<bf16_t>(fp, s)
         : tile_dtype == RZ_F16 ? launch_fold_as<f16_t>(fp, s)
                                : launch_fold_as<float>(fp, s);
}

template <bool ACC>
static void launch_convert(int out_dtype, const float* src, void* dst, int n, hipStream_t s) {
  const dim3 grid((n + 255) / 256), block(256);
  if (out_dtype == RZ_BF16)
    hipLaunchKernelGGL((convert_from_f32_kernel<bf16_t, ACC>), grid, block, 0, s, src, (bf16_t*)dst, n);
  else if (out_dtype == RZ_F16)
    hipLaunchKernelGGL((convert_from_f32_kernel<f16_t, ACC>), grid, block, 0, s, src, (f16_t*)dst, n);
  else
    hipLaunchKernelGGL((convert_from_f32_kernel<float, ACC>), grid, block, 0, s, src, (float*)dst, n);
}

static void launch_reduce_colsum(int out_dtype, const float* part, void* out, int N, int pitch, int rows,
                                 hipStream_t s) {
  const dim3 grid((N + 63) / 64), block(256);
  if (out_dtype == RZ_F32)
    hipLaunchKernelGGL(reduce_colsum_kernel<float>, grid, block, 0, s, part, (float*)out, N, pitch, rows);
  else if (out_dtype == RZ_BF16)
    hipLaunchKernelGGL(reduce_colsum_kernel<bf16_t>, grid, block, 0, s, part, (bf16_t*)out, N, pitch, rows);
  else
    hipLaunchKernelGGL(reduce_colsum_kernel<f16_t>, grid, block, 0, s, part, (f16_t*)out, N, pitch, rows);
}

static inline size_t round256(size_t b) { return (b + 255) & ~(size_t)255; }

// Workspace layout of a weight-grad call: [main][column sums].  main = the partial images (LDS
// image mode), the tile-by-tile X^T.dY followed by the fold kernel's images, the table of tile
// offsets (window kernel) or, for the atomic scatter into a 16-bit dHW, its fp32 image.
struct WeightGradWorkspace {
  size_t main_bytes, total_bytes;
};
static WeightGradWorkspace weight_grad_workspace(const WeightGradPlan& plan, const WindowPlan& window, int H,
                                                 bool dhw_f32, bool with_dbias, bool planned = false) {
  WeightGradWorkspace w;
  if (window.use) w.main_bytes = planned ? 0 : round256((size_t)window.tiles * sizeof(int32_t));  // tile offsets
  else if (plan.image_pitch > 0 || plan.fold.use) w.main_bytes = plan.workspace_bytes;
  else w.main_bytes = dhw_f32 ? 0 : round256((size_t)H * sizeof(float));
  // (the window kernel does not stage dY by tile columns: its bias gradient is a pass of its own)
  w.total_bytes = w.main_bytes + (with_dbias && !window.use ? plan.colsum_bytes : 0);
  return w;
}

// dHW (and optionally dbias) of one layer; see rz_weight_grad_ex in the header.
static int weight_grad_impl(const void* X, const void* dY, void* dHW, void* dbias, void* workspace,
                            size_t workspace_bytes, int M, int K, int N, int H, int BK, int BN,
                            const int32_t R[8], float init_factor, int64_t ldx, int64_t lddy, int dtype,
                            unsigned flags, void* stream, int hash_levels = RZ_HASH_TWO_LEVEL,
                            const rz_tuning* tuning_arg = nullptr, const int32_t* layer_plan = nullptr,
                            size_t layer_plan_bytes = 0) {
  if (X == nullptr || dY == nullptr || dHW == nullptr) return RZ_ERR_NULL_POINTER;
  if (dtype_bytes(dtype) == 0) return RZ_ERR_BAD_DTYPE;
  if (M < 1 || ldx < K || lddy < N) return RZ_ERR_BAD_SHAPE;
  if (!pitch_ok(ldx, dtype_bytes(dtype)) || !pitch_ok(lddy, dtype_bytes(dtype))) return RZ_ERR_BAD_SHAPE;
  if (flags & ~(unsigned)(RZ_WG_ACCUMULATE | RZ_WG_DHW_F32 | RZ_WG_DBIAS_F32)) return RZ_ERR_BAD_ARGUMENT;
  const rz_tuning tuning = tuning_or_default(tuning_arg);
  if (!tuning_valid(tuning)) return RZ_ERR_BAD_ARGUMENT;
  GemmParams p = {};
  int st = make_hash(&p.h, K, N, H, BK, BN, R, hash_levels);
  if (st != RZ_OK) return st;
  const bool accumulate = (flags & RZ_WG_ACCUMULATE) != 0;
  const int dhw_dtype = (flags & RZ_WG_DHW_F32) ? RZ_F32 : dtype;
  const int dbias_dtype = (flags & RZ_WG_DBIAS_F32) ? RZ_F32 : dtype;
  const WeightGradPlan plan = plan_weight_grad(M, K, N, H, BK, BN, dtype_bytes(dtype), tuning,
                                               fold_tile_bytes(dtype_bytes(dtype), dhw_dtype == RZ_F32, tuning));
  // a layer plan (device memory, built for exactly this K, N, H, tile and hash) replaces the
  // per-call hashing of the tile offsets and the window kernel's search for its strips
  const bool planned = layer_plan != nullptr;
  LayerPlanLayout lay = {};
  if (planned) {
    lay = layer_plan_layout(K, N, H, BK, BN);
    if (!lay.ok || layer_plan_bytes != lay.words * sizeof(int32_t)) return RZ_ERR_BAD_ARGUMENT;
  }
  WindowPlan wp = {};
  if (!plan.lds_image()) wp = plan_window(M, K, N, H, BK, BN, dtype_bytes(dtype), tuning, plan, planned && lay.windows > 0);
  const WeightGradWorkspace ws = weight_grad_workspace(plan, wp, H, dhw_dtype == RZ_F32, dbias != nullptr, planned);
  if (ws.total_bytes > 0 && (workspace == nullptr || workspace_bytes < ws.total_bytes)) return RZ_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  p.A = X;
  p.B = dY;
  p.I = K;
  p.J = N;
  p.R = M;
  p.lda = ldx;
  p.ldb = lddy;
  p.scale = init_factor;
  if (dbias != nullptr && !wp.use) p.colsum = reinterpret_cast<float*>(static_cast<char*>(workspace) + ws.main_bytes);
  if (wp.use) {
    // large hashed_weight, short contraction: windows of dHW instead of K*N atomics.  The
    // tile offsets are hashed once into the workspace; every workgroup scans them.
    {
      WindowParams w = {};
      if (planned) {
        if (lay.windows != wp.windows || lay.window != wp.window) return RZ_ERR_BAD_ARGUMENT;
        w.offsets = layer_plan + lay.offsets_at;
        w.plan_start = layer_plan + lay.start_at;
        w.plan_list = layer_plan + lay.list_at;
        w.plan_offs = layer_plan + lay.offs_at;
        w.plan_header = layer_plan;
      } else {
        const int TK = (K + BK - 1) / BK, TN = (N + BN - 1) / BN;
        hipLaunchKernelGGL(tile_offsets_kernel, dim3((TK * TN + 255) / 256), dim3(256), 0, s, (int32_t*)workspace,
                           TK, TN, p.h);
        if (hipGetLastError() != hipSuccess) return RZ_ERR_LAUNCH;
        w.offsets = (const int32_t*)workspace;
      }
      w.X = X; w.dY = dY; w.dHW = dHW;
      w.M = M; w.K = K; w.N = N; w.H = H;
      w.ldx = ldx; w.lddy = lddy;
      w.scale = init_factor;
      w.h = p.h;
      w.window = wp.window;
      w.tiles_k = (K + BK - 1) / BK;
      w.tiles_n = (N + BN - 1) / BN;
      w.accumulate = accumulate ? 1 : 0;
      w.out_f32 = dhw_dtype == RZ_F32 ? 1 : 0;
      w.poll_limit = tuning.poll_limit > 0 ? tuning.poll_limit : kWindowPollLimit;
      hipError_t e = dtype == RZ_F32 ? launch_window_f32(w, wp.windows, s)
                     : dtype == RZ_BF16 ? launch_window_bf16(w, wp.windows, s)
                                        : launch_window_f16(w, wp.windows, s);
      if (e != hipSuccess) return RZ_ERR_LAUNCH;
      if (dbias != nullptr) {
        launch_colsum_rows(dtype, dbias_dtype, dY, lddy, dbias, N, M, s);
        if (hipGetLastError() != hipSuccess) return RZ_ERR_LAUNCH;
      }
      return RZ_OK;
    }
  }
  if (plan.fold.use) {
    // no scatter in the contraction: X^T.dY goes to the workspace tile by tile, the fold kernel's
    // workgroups each add up the tiles that land in their window of hashed_weight (per share of
    // the tiles), and the shares' images are added up (no atomics, fixed summation order)
    const FoldPlan& f = plan.fold;
    p.scatter = nullptr;
    p.tiles_out = (float*)((char*)workspace + kFoldMarginBytes);   // (the fold kernel's loads reach a few floats beyond the tiles)
    p.tiles_out_16 = f.tile_bytes == 2 ? 1 : 0;
    if (p.tiles_out_16 && dtype_bytes(dtype) != 2) return RZ_ERR_BAD_ARGUMENT;   // (cannot happen: see fold_tile_bytes)
    const int tile_dtype = p.tiles_out_16 ? dtype : RZ_F32;
    p.out_tiles_k = (K + BK - 1) / BK;
    p.out_tiles_n = (N + BN - 1) / BN;
    if (launch_gemm(dtype, kWeightGrad, p, &plan, nullptr, tuning, s) != hipSuccess) return RZ_ERR_LAUNCH;
    FoldParams fp;
    fp.tiles = p.tiles_out;
    fp.plan_header = nullptr;
    fp.plan_start = nullptr;
    fp.plan_list = nullptr;
    fp.plan_capacity = 0;
    if (planned) {
      fp.offsets = layer_plan + lay.offsets_at;
      fp.plan_header = layer_plan;
      if (!f.small && lay.fold_windows == f.windows && lay.fold_window == f.window) {
        fp.plan_start = layer_plan + lay.fold_start_at;
        fp.plan_list = layer_plan + lay.fold_list_at;
        fp.plan_capacity = (int)lay.fold_capacity;
      }
    } else if (f.small) {
      fp.offsets = nullptr;   // (the kernel hashes the few offsets it needs)
    } else {
      int32_t* offsets = (int32_t*)((char*)workspace + f.tiles_bytes + f.partial_bytes);
      hipLaunchKernelGGL(tile_offsets_kernel, dim3((p.out_tiles_k * p.out_tiles_n + 255) / 256), dim3(256), 0, s, offsets,
                         p.out_tiles_k, p.out_tiles_n, p.h);
      if (hipGetLastError() != hipSuccess) return RZ_ERR_LAUNCH;
      fp.offsets = offsets;
    }
    fp.partial = f.shares > 1 ? (float*)((char*)workspace + f.tiles_bytes) : nullptr;
    fp.out = dHW;
    fp.out_dtype = dhw_dtype;
    fp.accumulate = accumulate ? 1 : 0;
    fp.h = p.h;
    fp.H = H;
    fp.pitch = (H + 3) & ~3;
    fp.K = K;
    fp.N = N;
    fp.tiles_k = p.out_tiles_k;
    fp.tiles_n = p.out_tiles_n;
    fp.slices = plan.splits;
    fp.window = f.window;
    fp.windows = f.windows;
    fp.shares = f.shares;
    if ((f.small ? launch_fold_small(fp, tile_dtype, s) : launch_fold(fp, tile_dtype, s)) != hipSuccess) return RZ_ERR_LAUNCH;
    if (f.shares > 1) {
      if (accumulate) launch_reduce_partials<true>(dhw_dtype, fp.partial, dHW, H, fp.pitch, f.shares, s);
      else launch_reduce_partials<false>(dhw_dtype, fp.partial, dHW, H, fp.pitch, f.shares, s);
    }
  } else if (plan.image_pitch > 0) {
    // every workgroup sums its tiles into an LDS image of dHW and stores it as a partial image;
    // the partial images are then added up (no global atomics, fixed summation order)
    p.scatter = (float*)workspace;
    if (launch_gemm(dtype, kWeightGrad, p, &plan, nullptr, tuning, s) != hipSuccess) return RZ_ERR_LAUNCH;
    if (accumulate) launch_reduce_partials<true>(dhw_dtype, p.scatter, dHW, H, plan.image_pitch, (int)plan.workgroups, s);
    else launch_reduce_partials<false>(dhw_dtype, p.scatter, dHW, H, plan.image_pitch, (int)plan.workgroups, s);
  } else {
    // hashed_weight too large for an LDS image: tiles go to an fp32 image of dHW by global
    // atomics; an fp32 dHW is its own image (and, accumulating, needs no clearing)
    float* image = (dhw_dtype == RZ_F32) ? (float*)dHW : (float*)workspace;
    if (!(accumulate && dhw_dtype == RZ_F32) &&
        zero_words(image, (size_t)H * sizeof(float), s) != hipSuccess)
      return RZ_ERR_LAUNCH;
    p.scatter = image;
    if (launch_gemm(dtype, kWeightGrad, p, &plan, nullptr, tuning, s) != hipSuccess) return RZ_ERR_LAUNCH;
    if (dhw_dtype != RZ_F32) {
      if (accumulate) launch_convert<true>(dhw_dtype, image, dHW, H, s);
      else launch_convert<false>(dhw_dtype, image, dHW, H, s);
    }
  }
  if (hipGetLastError() != hipSuccess) return RZ_ERR_LAUNCH;
  if (dbias != nullptr) {
    launch_reduce_colsum(dbias_dtype, p.colsum, dbias, N, plan.colsum_pitch, plan.colsum_rows, s);
    if (hipGetLastError() != hipSuccess) return RZ_ERR_LAUNCH;
  }
  return RZ_OK;
}

}  // namespace rz

using namespace rz;

// ---- scratch memory of the entry point that allocates nothing ---------------------------------
// A file-scope device array stands in for the caller's workspace.  Every GPU that loads the
// library holds its own copy, at its own address, until the process ends.  In host code the
// array's NAME is only a handle for hipGetSymbolAddress — never a device address; the address
// is looked up once per device (with that device current) and kept here.
static constexpr size_t kScratchBytes = 32u << 20;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
static constexpr int kMaxDevices = 64;
static std::atomic<void*> scratch_ptr[kMaxDevices];

// Device address of the current device's scratch array, or null (status in *st) if it cannot be
// had.  `owned` is memory of the call (its dHW): the kernels will run where it lives, so it must be
// device memory of the current device, or they would be handed another GPU's array.
static void* scratch_of_current_device(const void* owned, int* st) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    *st = RZ_ERR_LAUNCH;
    return nullptr;
  }
  hipPointerAttribute_t attr;
  if (hipPointerGetAttributes(&attr, owned) != hipSuccess || attr.type != hipMemoryTypeDevice || attr.device != dev) {
    (void)hipGetLastError();   // (a pointer HIP does not know leaves an error behind: it is reported here, not later)
    *st = RZ_ERR_BAD_ARGUMENT;
    return nullptr;
  }
  void* p = scratch_ptr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) {
      *st = RZ_ERR_LAUNCH;
      return nullptr;
    }
    scratch_ptr[dev].store(p, std::memory_order_release);   // (a racing thread stores the same value)
  }
  *st = RZ_OK;
  return p;
}

extern "C" {

#define RZ_API __attribute__((visibility("default")))

RZ_API int rz_version(void) { return 500; }

RZ_API const char* rz_status_string(int status) {
  switch (status) {
    case RZ_OK: return "ok";
    case RZ_ERR_NULL_POINTER: return "null pointer argument";
    case RZ_ERR_BAD_SHAPE: return "bad shape: M, K, N must be >= 1 and every row pitch >= the row length";
    case RZ_ERR_BAD_TILE: return "BLOCK_SIZE_K and BLOCK_SIZE_N must be powers of two in [16, 256]";
    case RZ_ERR_HASH_RANGE: return "hashed_weight too small: need H > BLOCK_SIZE_K * BLOCK_SIZE_N";
    case RZ_ERR_BAD_DTYPE: return "unsupported dtype (expected float32, bfloat16 or float16)";
    case RZ_ERR_HASH_OVERFLOW: return "hash intermediates exceed int32 for these constants and dimensions";
    case RZ_ERR_WORKSPACE: return "workspace missing or smaller than rz_weight_grad_workspace_bytes";
    case RZ_ERR_LAUNCH: return "HIP kernel launch failed";
    case RZ_ERR_BAD_ARGUMENT: return "bad argument";
    case RZ_ERR_SCRATCH_LIMIT: return "problem needs more scratch memory than the library's static 32 MiB: use the entry point that takes a workspace";
    default: return "unknown status";
  }
}

RZ_API int rz_tile_offsets(int32_t* out, int K, int N, int H, int BK, int BN, const int32_t R[8],
                           int hash_levels) {
  if (out == nullptr) return RZ_ERR_NULL_POINTER;
  HashParams h;
  int st = make_hash(&h, K, N, H, BK, BN, R, hash_levels);
  if (st != RZ_OK) return st;
  const int TK = (K + BK - 1) / BK, TN = (N + BN - 1) / BN;
  for (int tk = 0; tk < TK; tk++)
    for (int tn = 0; tn < TN; tn++)
      out[(size_t)tk * TN + tn] = (int32_t)tile_offset(h, (uint32_t)tk, (uint32_t)tn);
  return RZ_OK;
}

RZ_API int rz_tile_offsets_device(int32_t* d_out, int K, int N, int H, int BK, int BN,
                                  const int32_t R[8], int hash_levels, void* stream) {
  if (d_out == nullptr) return RZ_ERR_NULL_POINTER;
  HashParams h;
  int st = make_hash(&h, K, N, H, BK, BN, R, hash_levels);
  if (st != RZ_OK) return st;
  const int TK = (K + BK - 1) / BK, TN = (N + BN - 1) / BN;
  const int total = TK * TN;
  hipLaunchKernelGGL(tile_offsets_kernel, dim3((total + 255) / 256), dim3(256), 0,
                     (hipStream_t)stream, d_out, TK, TN, h);
  return hipGetLastError() == hipSuccess ? RZ_OK : RZ_ERR_LAUNCH;
}

static int forward_impl(const void* X, const void* HW, const void* bias, void* Y, void* workspace,
                        size_t workspace_bytes, bool may_split, int M, int K, int N, int H, int BK, int BN,
                        const int32_t R[8], float init_factor, int64_t ldx, int64_t ldy, int dtype,
                        void* stream, int hash_levels = RZ_HASH_TWO_LEVEL, const rz_tuning* tuning_arg = nullptr) {
  if (X == nullptr || HW == nullptr || Y == nullptr) return RZ_ERR_NULL_POINTER;
  if (dtype_bytes(dtype) == 0) return RZ_ERR_BAD_DTYPE;
  if (M < 1 || ldx < K || ldy < N || !pitch_ok(ldx, dtype_bytes(dtype)) || !pitch_ok(ldy, dtype_bytes(dtype))) return RZ_ERR_BAD_SHAPE;
  const rz_tuning tuning = tuning_or_default(tuning_arg);
  if (!tuning_valid(tuning)) return RZ_ERR_BAD_ARGUMENT;
  GemmParams p = {};
  int st = make_hash(&p.h, K, N, H, BK, BN, R, hash_levels);
  if (st != RZ_OK) return st;
  p.A = X;
  p.HW = HW;
  p.C = Y;
  p.I = M;
  p.J = N;
  p.R = K;
  p.lda = ldx;
  p.ldc = ldy;
  p.scale = init_factor;
  return run_plain_op(kForward, dtype, p, bias, workspace, workspace_bytes, may_split, tuning, (hipStream_t)stream);
}

static int input_grad_impl(const void* dY, const void* HW, void* dX, void* workspace, size_t workspace_bytes,
                           bool may_split, int M, int K, int N, int H, int BK, int BN, const int32_t R[8],
                           float init_factor, int64_t lddy, int64_t lddx, int dtype, void* stream,
                           int hash_levels = RZ_HASH_TWO_LEVEL, const rz_tuning* tuning_arg = nullptr) {
  if (dY == nullptr || HW == nullptr || dX == nullptr) return RZ_ERR_NULL_POINTER;
  if (dtype_bytes(dtype) == 0) return RZ_ERR_BAD_DTYPE;
  if (M < 1 || lddy < N || lddx < K || !pitch_ok(lddy, dtype_bytes(dtype)) || !pitch_ok(lddx, dtype_bytes(dtype))) return RZ_ERR_BAD_SHAPE;
  const rz_tuning tuning = tuning_or_default(tuning_arg);
  if (!tuning_valid(tuning)) return RZ_ERR_BAD_ARGUMENT;
  GemmParams p = {};
  int st = make_hash(&p.h, K, N, H, BK, BN, R, hash_levels);
  if (st != RZ_OK) return st;
  p.A = dY;
  p.HW = HW;
  p.C = dX;
  p.I = M;
  p.J = K;
  p.R = N;
  p.lda = lddy;
  p.ldc = lddx;
  p.scale = init_factor;
  return run_plain_op(kInputGrad, dtype, p, nullptr, workspace, workspace_bytes, may_split, tuning,
                      (hipStream_t)stream);
}

RZ_API int rz_forward_bias(const void* X, const void* HW, const void* bias, void* Y, int M, int K,
                           int N, int H, int BK, int BN, const int32_t R[8], float init_factor,
                           int64_t ldx, int64_t ldy, int dtype, void* stream) {
  return forward_impl(X, HW, bias, Y, nullptr, 0, false, M, K, N, H, BK, BN, R, init_factor, ldx, ldy, dtype,
                      stream);
}

RZ_API int rz_forward(const void* X, const void* HW, void* Y, int M, int K, int N, int H, int BK,
                      int BN, const int32_t R[8], float init_factor, int64_t ldx, int64_t ldy,
                      int dtype, void* stream) {
  return forward_impl(X, HW, nullptr, Y, nullptr, 0, false, M, K, N, H, BK, BN, R, init_factor, ldx, ldy,
                      dtype, stream);
}

RZ_API size_t rz_forward_hashed_workspace_bytes(int M, int K, int N, int H, int BK, int BN, int dtype,
                                                const rz_tuning* tuning) {
  (void)H; (void)BK; (void)BN;
  const int eb = dtype_bytes(dtype);
  const rz_tuning t = tuning_or_default(tuning);
  if (eb == 0 || M < 1 || K < 1 || N < 1 || !tuning_valid(t)) return 0;
  return plan_split(M, N, K, eb, t).workspace_bytes;
}

RZ_API size_t rz_forward_workspace_bytes(int M, int K, int N, int H, int BK, int BN, int dtype) {
  return rz_forward_hashed_workspace_bytes(M, K, N, H, BK, BN, dtype, nullptr);
}

RZ_API int rz_forward_ws(const void* X, const void* HW, const void* bias, void* Y, void* workspace,
                         size_t workspace_bytes, int M, int K, int N, int H, int BK, int BN,
                         const int32_t R[8], float init_factor, int64_t ldx, int64_t ldy, int dtype,
                         void* stream) {
  return forward_impl(X, HW, bias, Y, workspace, workspace_bytes, true, M, K, N, H, BK, BN, R, init_factor,
                      ldx, ldy, dtype, stream);
}

RZ_API int rz_input_grad(const void* dY, const void* HW, void* dX, int M, int K, int N, int H,
                         int BK, int BN, const int32_t R[8], float init_factor, int64_t lddy,
                         int64_t lddx, int dtype, void* stream) {
  return input_grad_impl(dY, HW, dX, nullptr, 0, false, M, K, N, H, BK, BN, R, init_factor, lddy, lddx,
                         dtype, stream);
}

RZ_API size_t rz_input_grad_hashed_workspace_bytes(int M, int K, int N, int H, int BK, int BN, int dtype,
                                                   const rz_tuning* tuning) {
  (void)H; (void)BK; (void)BN;
  const int eb = dtype_bytes(dtype);
  const rz_tuning t = tuning_or_default(tuning);
  if (eb == 0 || M < 1 || K < 1 || N < 1 || !tuning_valid(t)) return 0;
  return plan_split(M, K, N, eb, t).workspace_bytes;
}

RZ_API size_t rz_input_grad_workspace_bytes(int M, int K, int N, int H, int BK, int BN, int dtype) {
  return rz_input_grad_hashed_workspace_bytes(M, K, N, H, BK, BN, dtype, nullptr);
}

RZ_API int rz_input_grad_ws(const void* dY, const void* HW, void* dX, void* workspace,
                            size_t workspace_bytes, int M, int K, int N, int H, int BK, int BN,
                            const int32_t R[8], float init_factor, int64_t lddy, int64_t lddx, int dtype,
                            void* stream) {
  return input_grad_impl(dY, HW, dX, workspace, workspace_bytes, true, M, K, N, H, BK, BN, R, init_factor,
                         lddy, lddx, dtype, stream);
}

RZ_API size_t rz_weight_grad_workspace_bytes(int M, int K, int N, int H, int BK, int BN, int dtype) {
  return rz_weight_grad_ex_workspace_bytes(M, K, N, H, BK, BN, dtype, 0u, 0);
}

RZ_API int rz_weight_grad(const void* X, const void* dY, void* dHW, void* workspace,
                          size_t workspace_bytes, int M, int K, int N, int H, int BK, int BN,
                          const int32_t R[8], float init_factor, int64_t ldx, int64_t lddy,
                          int dtype, void* stream) {
  return weight_grad_impl(X, dY, dHW, nullptr, workspace, workspace_bytes, M, K, N, H, BK, BN, R,
                          init_factor, ldx, lddy, dtype, 0u, stream);
}

RZ_API int rz_weight_grad_static(const void* X, const void* dY, void* dHW, int M, int K, int N, int H, int BK,
                                 int BN, const int32_t R[8], float init_factor, int64_t ldx, int64_t lddy,
                                 int dtype, void* stream) {
  // the same kernels and checks as rz_weight_grad; only the workspace differs.  The plan is the
  // same too, except that the fold (whose tile-by-tile buffer takes 4*K*N bytes and more) gives
  // way to the scatter kernel when it does not fit the scratch array.
  rz_tuning tuning = {};
  if (dtype_bytes(dtype) != 0 && M >= 1 && K >= 1 && N >= 1 && H >= 1) {
    if (rz_weight_grad_hashed_workspace_bytes(M, K, N, H, BK, BN, dtype, 0u, 0, &tuning) > kScratchBytes) {
      tuning.fold = -1;
      if (rz_weight_grad_hashed_workspace_bytes(M, K, N, H, BK, BN, dtype, 0u, 0, &tuning) > kScratchBytes)
        return RZ_ERR_SCRATCH_LIMIT;
    }
  }
  // (argument errors are reported as rz_weight_grad reports them, before the device is looked at)
  if (X == nullptr || dY == nullptr || dHW == nullptr) return RZ_ERR_NULL_POINTER;
  if (dtype_bytes(dtype) == 0) return RZ_ERR_BAD_DTYPE;
  if (M < 1 || ldx < K || lddy < N) return RZ_ERR_BAD_SHAPE;
  HashParams h;
  int st = make_hash(&h, K, N, H, BK, BN, R, RZ_HASH_TWO_LEVEL);
  if (st != RZ_OK) return st;
  void* ws = scratch_of_current_device(dHW, &st);
  if (ws == nullptr) return st;
  return weight_grad_impl(X, dY, dHW, nullptr, ws, kScratchBytes, M, K, N, H, BK, BN, R, init_factor, ldx, lddy,
                          dtype, 0u, stream, RZ_HASH_TWO_LEVEL, &tuning);
}

RZ_API size_t rz_weight_grad_hashed_workspace_bytes(int M, int K, int N, int H, int BK, int BN, int dtype,
                                                    unsigned flags, int with_dbias, const rz_tuning* tuning) {
  const int eb = dtype_bytes(dtype);
  const rz_tuning t = tuning_or_default(tuning);
  if (eb == 0 || M < 1 || K < 1 || N < 1 || H < 1 || !tuning_valid(t)) return 0;
  if (check_tile(BK, BN) != RZ_OK) return 0;
  const bool dhw_f32 = (flags & RZ_WG_DHW_F32) != 0 || dtype == RZ_F32;
  const WeightGradPlan plan = plan_weight_grad(M, K, N, H, BK, BN, eb, t, fold_tile_bytes(eb, dhw_f32, t));
  WindowPlan wp = {};
  if (!plan.lds_image()) wp = plan_window(M, K, N, H, BK, BN, eb, t, plan);
  return weight_grad_workspace(plan, wp, H, dhw_f32, with_dbias != 0).total_bytes;
}

RZ_API size_t rz_weight_grad_ex_workspace_bytes(int M, int K, int N, int H, int BK, int BN, int dtype,
                                                unsigned flags, int with_dbias) {
  return rz_weight_grad_hashed_workspace_bytes(M, K, N, H, BK, BN, dtype, flags, with_dbias, nullptr);
}

RZ_API int rz_weight_grad_ex(const void* X, const void* dY, void* dHW, void* dbias, void* workspace,
                             size_t workspace_bytes, int M, int K, int N, int H, int BK, int BN,
                             const int32_t R[8], float init_factor, int64_t ldx, int64_t lddy,
                             int dtype, unsigned flags, void* stream) {
  return weight_grad_impl(X, dY, dHW, dbias, workspace, workspace_bytes, M, K, N, H, BK, BN, R,
                          init_factor, ldx, lddy, dtype, flags, stream);
}

RZ_API int rz_forward_hashed(const void* X, const void* HW, const void* bias, void* Y, void* workspace,
                             size_t workspace_bytes, int M, int K, int N, int H, int BK, int BN,
                             const int32_t R[8], int hash_levels, float init_factor, int64_t ldx,
                             int64_t ldy, int dtype, const rz_tuning* tuning, void* stream) {
  return forward_impl(X, HW, bias, Y, workspace, workspace_bytes, true, M, K, N, H, BK, BN, R, init_factor,
                      ldx, ldy, dtype, stream, hash_levels, tuning);
}

RZ_API int rz_input_grad_hashed(const void* dY, const void* HW, void* dX, void* workspace,
                                size_t workspace_bytes, int M, int K, int N, int H, int BK, int BN,
                                const int32_t R[8], int hash_levels, float init_factor, int64_t lddy,
                                int64_t lddx, int dtype, const rz_tuning* tuning, void* stream) {
  return input_grad_impl(dY, HW, dX, workspace, workspace_bytes, true, M, K, N, H, BK, BN, R, init_factor,
                         lddy, lddx, dtype, stream, hash_levels, tuning);
}

RZ_API int rz_weight_grad_hashed(const void* X, const void* dY, void* dHW, void* dbias, void* workspace,
                                 size_t workspace_bytes, int M, int K, int N, int H, int BK, int BN,
                                 const int32_t R[8], int hash_levels, float init_factor, int64_t ldx,
                                 int64_t lddy, int dtype, unsigned flags, const rz_tuning* tuning, void* stream) {
  return weight_grad_impl(X, dY, dHW, dbias, workspace, workspace_bytes, M, K, N, H, BK, BN, R,
                          init_factor, ldx, lddy, dtype, flags, stream, hash_levels, tuning);
}

RZ_API size_t rz_layer_plan_bytes(int K, int N, int H, int BK, int BN) {
  if (K < 1 || N < 1 || H < 1 || check_tile(BK, BN) != RZ_OK || (long long)H <= (long long)BK * BN) return 0;
  const LayerPlanLayout l = layer_plan_layout(K, N, H, BK, BN);
  return l.ok ? l.words * sizeof(int32_t) : 0;
}

RZ_API int rz_layer_plan_build(void* plan_host, size_t plan_bytes, int K, int N, int H, int BK, int BN,
                               const int32_t R[8], int hash_levels) {
  if (plan_host == nullptr) return RZ_ERR_NULL_POINTER;
  HashParams h;
  int st = make_hash(&h, K, N, H, BK, BN, R, hash_levels);
  if (st != RZ_OK) return st;
  const LayerPlanLayout l = layer_plan_layout(K, N, H, BK, BN);
  if (!l.ok || plan_bytes != l.words * sizeof(int32_t)) return RZ_ERR_BAD_ARGUMENT;
  int32_t* w = static_cast<int32_t*>(plan_host);
  for (size_t i = 0; i < l.words; i++) w[i] = 0;
  const int TK = (K + BK - 1) / BK, TN = (N + BN - 1) / BN;
  int32_t* offsets = w + l.offsets_at;
  for (int tk = 0; tk < TK; tk++)
    for (int tn = 0; tn < TN; tn++) offsets[(size_t)tk * TN + tn] = (int32_t)tile_offset(h, (uint32_t)tk, (uint32_t)tn);
  long long entries = 0;
  if (l.windows > 0) {
    // counting sort of (window, strip) pairs by window; visiting the strips in ascending order
    // keeps every window's list ascending, which is the order the kernel's own search produces
    int32_t* start = w + l.start_at;
    int32_t* list = w + l.list_at;
    int32_t* offs = w + l.offs_at;
    auto for_each_pair = [&](auto&& f) {
      for (int id = 0; id < l.tiles; id++)
        for (int sidx = 0; sidx < l.strips_per_tile; sidx++) {
          const long long so = (long long)offsets[id] + window_unit_start(BN, sidx);
          const long long first = so / l.window, last = (so + l.strip_elems - 1) / l.window;
          for (long long b = first; b <= last && b < l.windows; b++) f((int)b, id * l.strips_per_tile + sidx, (int32_t)so);
        }
    };
    for_each_pair([&](int b, int, int32_t) { start[b + 1]++; });
    for (int b = 0; b < l.windows; b++) start[b + 1] += start[b];
    entries = start[l.windows];
    if (entries > l.capacity) return RZ_ERR_BAD_ARGUMENT;   // (cannot happen: see layer_plan_layout)
    // (start[b] is advanced while the lists are filled and restored afterwards)
    for_each_pair([&](int b, int strip, int32_t so) {
      list[start[b]] = strip;
      offs[start[b]] = so;
      start[b]++;
    });
    for (int b = l.windows; b > 0; b--) start[b] = start[b - 1];
    start[0] = 0;
  }
  {
    // The fold kernel's lists, by the same counting sort.  The tiles are visited in the order in which the
    // kernel's own search numbers them (pass by pass of kFoldScan * kFoldThreads tile indices; inside a pass
    // thread by thread, and tile t + 1024 j of the pass is bit j of thread t), so that a window's tiles are
    // added in the same order, and come out in the same bits, with a plan and without.
    int32_t* start = w + l.fold_start_at;
    int32_t* list = w + l.fold_list_at;
    const long long E = (long long)BK * BN;
    auto for_each_pair = [&](auto&& f) {
      for (int first = 0; first < l.tiles; first += kFoldScan * kFoldThreads)
        for (int t = 0; t < kFoldThreads; t++)
          for (int j = 0; j < kFoldScan; j++) {
            const long long id = (long long)first + t + (long long)j * kFoldThreads;
            if (id >= l.tiles) break;
            const long long off = offsets[id];
            for (long long b = off / l.fold_window; b <= (off + E - 1) / l.fold_window && b < l.fold_windows; b++) f((int)b, (int)id);
          }
    };
    for_each_pair([&](int b, int) { start[b + 1]++; });
    for (int b = 0; b < l.fold_windows; b++) start[b + 1] += start[b];
    if (start[l.fold_windows] > l.fold_capacity) return RZ_ERR_BAD_ARGUMENT;   // (cannot happen: see layer_plan_layout)
    for_each_pair([&](int b, int id) { list[start[b]++] = id; });
    for (int b = l.fold_windows; b > 0; b--) start[b] = start[b - 1];
    start[0] = 0;
  }
  const int32_t header[kLayerPlanHeader] = {kLayerPlanMagic, kLayerPlanVersion, K, N, H, BK, BN, hash_levels, l.tiles,
                                            l.windows, l.window, (int32_t)entries, l.strips_per_tile,
                                            layer_plan_hash_sum(h), l.fold_windows, l.fold_window};
  for (int i = 0; i < kLayerPlanHeader; i++) w[i] = header[i];
  return RZ_OK;
}

RZ_API int rz_weight_grad_planned(const void* X, const void* dY, void* dHW, void* dbias, void* workspace,
                                  size_t workspace_bytes, const void* layer_plan, size_t layer_plan_bytes, int M,
                                  int K, int N, int H, int BK, int BN, const int32_t R[8], int hash_levels,
                                  float init_factor, int64_t ldx, int64_t lddy, int dtype, unsigned flags,
                                  const rz_tuning* tuning, void* stream) {
  if (layer_plan == nullptr) return RZ_ERR_NULL_POINTER;
  return weight_grad_impl(X, dY, dHW, dbias, workspace, workspace_bytes, M, K, N, H, BK, BN, R, init_factor, ldx,
                          lddy, dtype, flags, stream, hash_levels, tuning, static_cast<const int32_t*>(layer_plan),
                          layer_plan_bytes);
}

RZ_API int rz_plan_query(int op, int M, int K, int N, int H, int BK, int BN, int dtype, unsigned flags,
                         int with_dbias, const rz_tuning* tuning, int32_t out[8]) {
  (void)with_dbias;
  if (out == nullptr) return RZ_ERR_NULL_POINTER;
  const bool planned = (flags & RZ_PLAN_WITH_LAYER_PLAN) != 0;
  const int eb = dtype_bytes(dtype);
  if (eb == 0) return RZ_ERR_BAD_DTYPE;
  if (M < 1 || K < 1 || N < 1 || H < 1) return RZ_ERR_BAD_SHAPE;
  const rz_tuning t = tuning_or_default(tuning);
  if (!tuning_valid(t)) return RZ_ERR_BAD_ARGUMENT;
  int st = check_tile(BK, BN);
  if (st != RZ_OK) return st;
  for (int i = 0; i < 8; i++) out[i] = 0;
  if (op == kWeightGrad) {
    const bool dhw_f32 = (flags & RZ_WG_DHW_F32) != 0 || dtype == RZ_F32;
    const WeightGradPlan plan = plan_weight_grad(M, K, N, H, BK, BN, eb, t, fold_tile_bytes(eb, dhw_f32, t));
    WindowPlan wp = {};
    if (!plan.lds_image())
      wp = plan_window(M, K, N, H, BK, BN, eb, t, plan, planned && layer_plan_layout(K, N, H, BK, BN).windows > 0);
    if (wp.use) {
      out[0] = 0; out[1] = 1; out[2] = M; out[3] = 32; out[4] = 4; out[5] = wp.windows; out[7] = wp.windows;
      return RZ_OK;
    }
    const KernelForm f = kernel_form(op, K, N, M, plan.r_chunk, plan.tile, plan.workgroups, eb, t);
    out[0] = plan.tile; out[1] = plan.splits; out[2] = plan.r_chunk; out[3] = f.step;
    out[4] = plan.fold.use ? 5 : plan.image_pitch > 0 ? 2 : 3;
    out[5] = (int32_t)plan.workgroups;
    if (plan.fold.use) {
      out[6] = plan.fold.shares;
      out[7] = plan.fold.windows;
    }
    return RZ_OK;
  }
  if (op != kForward && op != kInputGrad) return RZ_ERR_BAD_ARGUMENT;
  const int I = M, J = op == kForward ? N : K, R = op == kForward ? K : N;
  const SplitPlan sp = plan_split(I, J, R, eb, t);
  const bool cut = sp.splits > 1;
  const int chunk = cut ? sp.r_chunk : R;
  const KernelForm f = kernel_form(op, I, J, R, chunk, sp.tile, tile_count(I, J, sp.tile) * sp.splits, eb, t);
  out[0] = sp.tile; out[1] = sp.splits; out[2] = chunk; out[3] = f.step; out[4] = cut ? 1 : 0;
  out[5] = (int32_t)(tile_count(I, J, sp.tile) * sp.splits);
  out[6] = (cut && t.finish != -1 && sp.splits <= finish_slices(sp.tile, I, J) && tile_count(I, J, sp.tile) <= (long long)kFinishPerStream) ? 1 : 0;
  return RZ_OK;
}

RZ_API int rz_materialize(const void* HW, void* W, int K, int N, int H, int BK, int BN,
                          const int32_t R[8], int hash_levels, int64_t ldw, int dtype, void* stream) {
  if (HW == nullptr || W == nullptr) return RZ_ERR_NULL_POINTER;
  if (dtype_bytes(dtype) == 0) return RZ_ERR_BAD_DTYPE;
  if (ldw < N) return RZ_ERR_BAD_SHAPE;
  HashParams h;
  int st = make_hash(&h, K, N, H, BK, BN, R, hash_levels);
  if (st != RZ_OK) return st;
  const int TK = (K + BK - 1) / BK, TN = (N + BN - 1) / BN;
  if ((long long)TK * TN > 0x7fffffffLL) return RZ_ERR_BAD_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == RZ_F32)
    hipLaunchKernelGGL(materialize_kernel<uint32_t>, dim3(TK * TN), dim3(256), 0, s,
                       (const uint32_t*)HW, (uint32_t*)W, K, N, TN, ldw, h);
  else
    hipLaunchKernelGGL(materialize_kernel<uint16_t>, dim3(TK * TN), dim3(256), 0, s,
                       (const uint16_t*)HW, (uint16_t*)W, K, N, TN, ldw, h);
  return hipGetLastError() == hipSuccess ? RZ_OK : RZ_ERR_LAUNCH;
}

}  // extern "C"
