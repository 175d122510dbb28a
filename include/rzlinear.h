/*
 * librzlinear — C ABI of the MI355X (gfx950) RzLinear hot path.
 *
 * RzLinear is a linear layer whose logical weight W[K,N] is never stored: tile
 * (tk,tn) of W, BK x BN elements, is the contiguous slice
 *     hashed_weight[off(tk,tn) : off(tk,tn) + BK*BN]     viewed row-major [BK,BN]
 * of a 1-D parameter hashed_weight[H].  The three device entry points compute
 *     forward      Y   = (X  . W  ) * init_factor
 *     input-grad   dX  = (dY . W^T) * init_factor
 *     weight-grad  dHW = scatter_add over tiles of (X^T . dY) * init_factor
 * without materialising W.
 *
 * Conventions shared by every entry point
 *   - plain pointers and sizes only; device pointers are HIP device memory that
 *     the caller owns; no entry point allocates or frees device memory or
 *     synchronises with the host; work is enqueued on `stream` (a hipStream_t
 *     passed as void*, NULL = the default stream).
 *   - matrices are row-major with unit column stride; `ld*` is the row pitch in
 *     ELEMENTS.  Any M, K, N >= 1 is accepted (edge tiles read as zero).
 *   - R[8] are the hash constants: R[0] = P (prime), R[1..7] in [0,P).  R[6] is
 *     carried but takes part in no formula, exactly as in the reference.
 *   - BK, BN: powers of two in [16, 256]; H > BK*BN.
 *   - return value: RZ_OK (0) or a negative rz_status; never throws.
 *
 * Reference interface that each entry point replaces is cited as
 * file:line of the reference checkout (python/rz_linear/...).
 */
#ifndef RZLINEAR_H
#define RZLINEAR_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum rz_status {
  RZ_OK = 0,
  RZ_ERR_NULL_POINTER = -1,
  RZ_ERR_BAD_SHAPE = -2,       /* M, K, N < 1, ld too small (or 256 rows of it beyond 4 GB), sizes beyond int32 tiling */
  RZ_ERR_BAD_TILE = -3,        /* BK/BN not a power of two in [16,256] */
  RZ_ERR_HASH_RANGE = -4,      /* H <= BK*BN  (reference: assert H > BLOCK_SIZE_K*BLOCK_SIZE_N) */
  RZ_ERR_BAD_DTYPE = -5,
  RZ_ERR_HASH_OVERFLOW = -6,   /* hash intermediates would leave int32 (reference computes in int32) */
  RZ_ERR_WORKSPACE = -7,       /* workspace missing or too small */
  RZ_ERR_LAUNCH = -8,          /* HIP reported a launch error */
  RZ_ERR_BAD_ARGUMENT = -9,
  RZ_ERR_SCRATCH_LIMIT = -10   /* rz_weight_grad_static: the problem needs more than the static scratch */
} rz_status;

typedef enum rz_dtype {
  RZ_F32 = 0,
  RZ_BF16 = 1,
  RZ_F16 = 2
} rz_dtype;

/* Which tile hash an entry point with a `hash_levels` argument evaluates. */
typedef enum rz_hash {
  RZ_HASH_ONE_LEVEL = 1,  /* ((tk*R3 + tn*R2 + R1) % R0) % (H - BK*BN)          impl/RzLinearIdx.py:70-71 */
  RZ_HASH_TWO_LEVEL = 2,  /* the hash of the three kernels                       impl/RzLinearForward.py:316 */
  RZ_HASH_LEGACY = 3      /* ((tk*R3 + tn*R2 + R1) % R0) % (H - BK*BN + 1) in 64-bit integers: the tiled
                             location of the legacy generation (16 x 16 tiles, prime 2038074743),
                             /rz_linear_kernel.cu:34-36,:56-64; R4..R7 unused; H >= BK*BN suffices */
} rz_hash;

/*
 * Optional tuning overrides of the entry points that take a `const rz_tuning*` (NULL or an
 * all-zero struct = the library decides everything, which is what callers want; the overrides
 * exist so that tests and benchmarks can reach every kernel form).  The library reads no
 * environment variable and keeps no settings between calls: what a call does is a function of
 * its arguments alone, and a workspace query answers for the same tuning it is given.
 * No counterpart in the reference, whose tile choice is the autotuner's.
 */
typedef struct rz_tuning {
  int tile;       /* C-tile edge of the contraction kernels: 0 = automatic, 64, 128 or 256; 32 = the 32 x 64
                     tile of fp32 forward / input-grad (elsewhere it reads as 64) */
  int stages;     /* 0 = automatic, 1 = the single-stage form of the 128 tile */
  int lds_image;  /* weight-grad: 0 = automatic, -1 = never sum tiles in an LDS image of dHW */
  int window;     /* weight-grad: 0 = automatic, 1 = dHW by windows whenever possible, -1 = never */
  int split;      /* forward / input-grad: 0 = automatic, -1 = never split the contraction, 2 .. 16 = into exactly
                     that many slices where such a cut exists */
  int clamp;      /* ragged shapes: 0 = automatic, -1 = always the bounds-checked kernels */
  int fold;       /* weight-grad with a hashed_weight too large for LDS: 0 = automatic, 1 = X^T.dY stored
                     tile by tile and folded into dHW by a second kernel whenever possible, 2 = the same
                     with the windowed fold kernel even for the few tiles that have a kernel of their own,
                     -1 = never */
  int fold_tiles; /* weight-grad by the fold, 16-bit layer with a 16-bit dHW: 0 = automatic (X^T.dY is stored tile by
                     tile in the layer's dtype: half the bytes written and read back; every stored value is
                     rounded once more than in fp32, the sum over M and the sum of the tiles stay fp32),
                     -1 = always fp32 tiles */
  int finish;     /* forward / input-grad with a cut contraction: 0 = automatic (the slice that arrives last at a
                     tile of the output adds the slices' partial results up and stores it: no second kernel),
                     -1 = always a second kernel; the results are the same bits either way.  The arrivals are
                     counted in a device array that the library owns and divides among streams: each of the
                     first sixteen streams per device that launch such a contraction keeps a part of its own,
                     so calls on different streams never share a counter; a further stream, a stream under
                     capture and an output of more than 4096 tiles get the second kernel */
  int poll_limit; /* weight-grad by windows: 0 = default; > 0 = how often a wavefront looks at the flags of the
                     earlier strips it waits for before it gives up and the window is stored as NaN (a bounded
                     wait; tests set a tiny value to see every wavefront leave the kernel all the same) */
} rz_tuning;

/* Library / ABI version (major*10000 + minor*100 + patch). */
int rz_version(void);

/* Human-readable text for a status code (static storage). */
const char* rz_status_string(int status);

/*
 * Tile offsets on the HOST, bit-exact integer hash.
 *   hash_levels = 2:  off = (((tk*R3 + tn*R2 + R1) % R0) * R0 + ((tk*R7 + tn*R5 + R4) % R0)) % (H - BK*BN)
 *       replaces the inline hash of rz_linear_forward_core           impl/RzLinearForward.py:316,:349
 *       rz_linear_backward_weight_grad_core                           impl/RzLinearBackward.py:369
 *       rz_linear_backward_input_grad_core                            impl/RzLinearBackward.py:686,:716
 *   hash_levels = 1:  off = ((tk*R3 + tn*R2 + R1) % R0) % (H - BK*BN)
 *       replaces the hash of rz_linear_idx_kernel                     impl/RzLinearIdx.py:70-71
 *   hash_levels = 3:  the legacy generation's tiled location (see rz_hash)
 *       replaces location_tiled                                       /rz_linear_kernel.cu:56-64
 * out has ceil(K/BK)*ceil(N/BN) entries, index tk*ceil(N/BN) + tn.
 */
int rz_tile_offsets(int32_t* out, int K, int N, int H, int BK, int BN, const int32_t R[8],
                    int hash_levels);

/*
 * Forward: Y[M,N] = (X[M,K] . W) * init_factor.
 * Replaces rz_linear_forward_tl                                       impl/RzLinearForward.py:6-85
 * (kernel rz_linear_forward_core                                      impl/RzLinearForward.py:271-357).
 * X, HW, Y are device pointers of element type `dtype`; Y is fully overwritten.
 */
int rz_forward(const void* X, const void* HW, void* Y, int M, int K, int N, int H, int BK, int BN,
               const int32_t R[8], float init_factor, int64_t ldx, int64_t ldy, int dtype,
               void* stream);

/*
 * Forward with the layer's bias fused into the store: Y = (X . W) * init_factor + bias[N]
 * (bias of element type `dtype`, may be NULL = rz_forward).  The sum is formed in fp32 and
 * rounded once.  Replaces the launcher above plus the separate `x + self._bias` of the module,
 * python/rz_linear/RzLinear.py:93-94.
 */
int rz_forward_bias(const void* X, const void* HW, const void* bias, void* Y, int M, int K, int N,
                    int H, int BK, int BN, const int32_t R[8], float init_factor, int64_t ldx,
                    int64_t ldy, int dtype, void* stream);

/*
 * Input gradient: dX[M,K] = (dY[M,N] . W^T) * init_factor.
 * Replaces rz_linear_backward_input_grad_tl                           impl/RzLinearBackward.py:374-449
 * (kernel rz_linear_backward_input_grad_core                          impl/RzLinearBackward.py:642-727).
 */
int rz_input_grad(const void* dY, const void* HW, void* dX, int M, int K, int N, int H, int BK,
                  int BN, const int32_t R[8], float init_factor, int64_t lddy, int64_t lddx,
                  int dtype, void* stream);

/*
 * Forward / input-grad that may split the contraction: with few output tiles and a long
 * contracted dimension (skinny batches such as M = 32 against K = N = 10240) the work is cut
 * into slices that write fp32 partial results to `workspace`, and a second kernel adds them
 * (plus bias) into the output.  *_workspace_bytes returns the size needed (0 = no split; then
 * these calls equal rz_forward_bias / rz_input_grad and workspace may be NULL).  No
 * counterpart in the reference, whose kernels never split (impl/RzLinearForward.py:37-40,
 * impl/RzLinearBackward.py:407-410).
 */
size_t rz_forward_workspace_bytes(int M, int K, int N, int H, int BK, int BN, int dtype);
int rz_forward_ws(const void* X, const void* HW, const void* bias, void* Y, void* workspace,
                  size_t workspace_bytes, int M, int K, int N, int H, int BK, int BN,
                  const int32_t R[8], float init_factor, int64_t ldx, int64_t ldy, int dtype,
                  void* stream);
size_t rz_input_grad_workspace_bytes(int M, int K, int N, int H, int BK, int BN, int dtype);
int rz_input_grad_ws(const void* dY, const void* HW, void* dX, void* workspace,
                     size_t workspace_bytes, int M, int K, int N, int H, int BK, int BN,
                     const int32_t R[8], float init_factor, int64_t lddy, int64_t lddx, int dtype,
                     void* stream);

/*
 * Bytes of device workspace rz_weight_grad needs for this problem (0 when none).
 * When hashed_weight is small enough for an fp32 image of dHW to fit the LDS of a compute
 * unit, every workgroup stores one partial image ([workgroups][H rounded up to 4] floats) that
 * a second kernel adds up.  Otherwise one of three: with many W tiles per element of dHW the
 * contraction stores X^T.dY tile by tile (4 * ceil(K/BK)*BK * ceil(N/BN)*BN bytes per slice of M)
 * and a second kernel folds the tiles into dHW (plus a few images of dHW and one int32 offset
 * per W tile); with M small against K*N, dHW is computed in windows and the workspace holds
 * only the offsets; with few tiles the 16-bit types need an fp32 image of dHW (H floats) for
 * atomic adds and fp32 needs nothing.  The size depends on M: ask again when the batch size
 * changes.
 */
size_t rz_weight_grad_workspace_bytes(int M, int K, int N, int H, int BK, int BN, int dtype);

/*
 * Weight gradient: dHW[H] = sum over tiles (tk,tn) of (X^T . dY)[tile] * init_factor added at
 * off(tk,tn); dHW is zeroed and fully overwritten by the call (element type `dtype`).
 * Replaces rz_linear_backward_weight_grad_tl                          impl/RzLinearBackward.py:23-97
 * (kernel rz_linear_backward_weight_grad_core                         impl/RzLinearBackward.py:291-371).
 * Accumulation and the scatter are done in fp32 for every dtype (one exception: a 16-bit layer with a
 * 16-bit dHW on the fold path keeps the complete fp32 sums over M in its own dtype between the two
 * kernels — one more rounding per stored value, still added up in fp32; see rz_tuning.fold_tiles — where
 * the reference rounds the running sum at every atomic add).  The LDS-image, fold and
 * window paths add in a fixed order (plain read-add-write in LDS, ordered by barriers, by list
 * order or by flags; partial images are added in index order): the same inputs give the same
 * bits on every call.  Two cases leave the summation order across tiles open, as the reference
 * does everywhere: the global-atomic path (hashed tiles of more than 16384 elements over a
 * hashed_weight too large for LDS, or where rz_tuning asks for it), and hashed tiles of 16 rows or
 * 16 columns on the LDS-image path (an MFMA block then spans several hashed tiles whose slices may
 * overlap, and they are added into the image with LDS atomics).
 */
int rz_weight_grad(const void* X, const void* dY, void* dHW, void* workspace,
                   size_t workspace_bytes, int M, int K, int N, int H, int BK, int BN,
                   const int32_t R[8], float init_factor, int64_t ldx, int64_t lddy, int dtype,
                   void* stream);

/*
 * rz_weight_grad without a workspace argument and without any allocation: the partial images,
 * the offset table or the fp32 image that rz_weight_grad keeps in the caller's workspace live in
 * a 32 MiB device array that is part of the library (every GPU that loads the library holds its
 * own copy until the process ends).  No counterpart in the reference; it is for callers that
 * cannot allocate: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  Same arguments, results and status codes as rz_weight_grad otherwise.  A problem
 * for which rz_weight_grad would store X^T.dY tile by tile in more than 32 MiB takes the scatter
 * kernel with global atomics instead; a problem that needs more than 32 MiB even so is refused
 * with RZ_ERR_SCRATCH_LIMIT (at M = N = K = 4096, H = 16778 the need is 17 MB).  The first call on a device looks the array's
 * address up (make that call outside a graph capture).  The array used is that of the CURRENT device, which must be
 * the device that holds dHW (and the other operands, and the stream): a call whose dHW lives on another device, or is
 * not device memory at all, is refused with RZ_ERR_BAD_ARGUMENT.  All calls on one GPU share the one array:
 * calls that overlap in time on the same GPU — different streams, or different host threads —
 * race on it and must be serialised by the caller; calls on one stream are ordered and safe.
 * Nothing in the array needs to survive between calls, and each call writes what it reads.
 */
int rz_weight_grad_static(const void* X, const void* dY, void* dHW, int M, int K, int N, int H, int BK,
                          int BN, const int32_t R[8], float init_factor, int64_t ldx, int64_t lddy,
                          int dtype, void* stream);

/*
 * Weight gradient for training loops that own their gradient buffers, optionally with the
 * bias gradient from the same pass over dY.
 *   flags (bitwise or):
 *     RZ_WG_ACCUMULATE  dHW += gradient instead of dHW = gradient.  Several layers may share one
 *                       hashed_weight (python/rz_linear/RzLinear.py:54-58); accumulating here
 *                       saves autograd's separate add over H and the clearing of dHW.
 *     RZ_WG_DHW_F32     dHW is fp32 whatever `dtype` is (fp32 master gradients).
 *     RZ_WG_DBIAS_F32   dbias is fp32 whatever `dtype` is.
 *   dbias (may be NULL): dbias[N] = column sums of dY — the gradient of the bias that
 *     python/rz_linear/RzLinear.py:93-94 adds, which autograd otherwise computes with a second
 *     pass over dY.  Always overwritten; not scaled by init_factor (the bias is added after it).
 *     The sums come from the dY tiles that the contraction stages anyway, in a fixed order.
 * With flags = 0 and dbias = NULL this is rz_weight_grad.  The workspace size depends on the
 * options: ask rz_weight_grad_ex_workspace_bytes with the same flags and with_dbias = (dbias != NULL).
 * Extends rz_linear_backward_weight_grad_tl                           impl/RzLinearBackward.py:23-97,
 * which always overwrites a fresh buffer of the input's dtype.
 */
#define RZ_WG_ACCUMULATE 1u
#define RZ_WG_DHW_F32 2u
#define RZ_WG_DBIAS_F32 4u
size_t rz_weight_grad_ex_workspace_bytes(int M, int K, int N, int H, int BK, int BN, int dtype,
                                         unsigned flags, int with_dbias);
int rz_weight_grad_ex(const void* X, const void* dY, void* dHW, void* dbias, void* workspace,
                      size_t workspace_bytes, int M, int K, int N, int H, int BK, int BN,
                      const int32_t R[8], float init_factor, int64_t ldx, int64_t lddy, int dtype,
                      unsigned flags, void* stream);

/*
 * The three contractions with an explicit tile hash (rz_hash) and optional tuning overrides.
 * hash_levels = RZ_HASH_TWO_LEVEL and tuning = NULL give rz_forward_ws / rz_input_grad_ws /
 * rz_weight_grad_ex (same flags).  RZ_HASH_LEGACY runs a hashed_weight laid out by the legacy
 * generation — its forward /rz_linear_kernel.cu:245-338 and backward :516-592 in tiled mode —
 * with BK = BN = 16 and the constants of /RzLinear.py:70-75 (larger tiles follow the same
 * formula).  The workspace size is asked with the same tuning (and flags) as the call.
 */
size_t rz_forward_hashed_workspace_bytes(int M, int K, int N, int H, int BK, int BN, int dtype,
                                         const rz_tuning* tuning);
int rz_forward_hashed(const void* X, const void* HW, const void* bias, void* Y, void* workspace,
                      size_t workspace_bytes, int M, int K, int N, int H, int BK, int BN,
                      const int32_t R[8], int hash_levels, float init_factor, int64_t ldx, int64_t ldy,
                      int dtype, const rz_tuning* tuning, void* stream);
size_t rz_input_grad_hashed_workspace_bytes(int M, int K, int N, int H, int BK, int BN, int dtype,
                                            const rz_tuning* tuning);
int rz_input_grad_hashed(const void* dY, const void* HW, void* dX, void* workspace,
                         size_t workspace_bytes, int M, int K, int N, int H, int BK, int BN,
                         const int32_t R[8], int hash_levels, float init_factor, int64_t lddy,
                         int64_t lddx, int dtype, const rz_tuning* tuning, void* stream);
size_t rz_weight_grad_hashed_workspace_bytes(int M, int K, int N, int H, int BK, int BN, int dtype,
                                             unsigned flags, int with_dbias, const rz_tuning* tuning);
int rz_weight_grad_hashed(const void* X, const void* dY, void* dHW, void* dbias, void* workspace,
                          size_t workspace_bytes, int M, int K, int N, int H, int BK, int BN,
                          const int32_t R[8], int hash_levels, float init_factor, int64_t ldx,
                          int64_t lddy, int dtype, unsigned flags, const rz_tuning* tuning, void* stream);

/*
 * Layer plan: the part of a weight-grad call that depends only on the layer — K, N, H, the tile
 * and the hash constants — and not on the batch: where every W tile starts in hashed_weight and,
 * for every window of dHW that the window kernel or the fold kernel works on, the ordered list of
 * tile strips (of tiles) that land in it.  Without a plan every weight-grad call on a large
 * hashed_weight hashes the tile offsets again and every workgroup searches them for its strips or
 * tiles (some 25 us of an 85 us call at M = 32, K = N = 10240; 5 us of the fold kernel's 60 to 90);
 * with one it reads its list.  The result is the same bit for bit.
 *   rz_layer_plan_bytes   size of the plan (0: bad arguments)
 *   rz_layer_plan_build   fills plan_host[plan_bytes] on the HOST (no device is touched); the
 *                         caller copies it to device memory once and keeps it with the layer
 *   rz_weight_grad_planned  rz_weight_grad_hashed with that device copy; the workspace is asked
 *                         for as for rz_weight_grad_hashed (never more is needed).  The plan must
 *                         have been built for the same K, N, H, BK, BN, R and hash_levels: the
 *                         size is checked on the host; the plan's header (shapes, tile, hash and a
 *                         checksum of R) is checked by the kernels that read it, which store NaN
 *                         into dHW instead of following a plan of another layer.
 * No counterpart in the reference, whose kernels hash every tile offset on every call
 * (impl/RzLinearBackward.py:369).
 */
size_t rz_layer_plan_bytes(int K, int N, int H, int BK, int BN);
int rz_layer_plan_build(void* plan_host, size_t plan_bytes, int K, int N, int H, int BK, int BN,
                        const int32_t R[8], int hash_levels);
int rz_weight_grad_planned(const void* X, const void* dY, void* dHW, void* dbias, void* workspace,
                           size_t workspace_bytes, const void* layer_plan, size_t layer_plan_bytes, int M,
                           int K, int N, int H, int BK, int BN, const int32_t R[8], int hash_levels,
                           float init_factor, int64_t ldx, int64_t lddy, int dtype, unsigned flags,
                           const rz_tuning* tuning, void* stream);

/*
 * How a call would be carried out (host-side, touches no device): which C tile, how many
 * slices of the contracted dimension and how long each, which kernel form.  op: 0 = forward,
 * 1 = input-grad, 2 = weight-grad (flags / with_dbias as for rz_weight_grad_hashed, else 0).
 * RZ_PLAN_WITH_LAYER_PLAN in flags: answer for a call that carries a layer plan (rz_weight_grad_planned), which
 * changes what the window kernel costs and hence when it is taken.
 * Fills out[8] = { C-tile edge, slices, contracted elements per slice, contracted elements per
 * kernel step, mode, workgroups, workgroups per window of the fold kernel (mode 5; mode 1: 1 if the kernel
 * finishes its own tiles, 0 if a second kernel adds the slices up; else 0), windows of dHW
 * (modes 4 and 5, else 0) } with mode 0 = plain store, 1 = split contraction with
 * fp32 partial planes, 2 = weight-grad through LDS images of dHW, 3 = weight-grad by global
 * atomics, 4 = weight-grad by windows of dHW, 5 = weight-grad stored tile by tile and folded
 * into dHW by a second kernel.  For tests of the planning logic and for tuning; no counterpart in the
 * reference.
 */
#define RZ_PLAN_WITH_LAYER_PLAN 0x100u
int rz_plan_query(int op, int M, int K, int N, int H, int BK, int BN, int dtype, unsigned flags,
                  int with_dbias, const rz_tuning* tuning, int32_t out[8]);

/*
 * Materialise W[K,N] (row pitch ldw) from hashed_weight; edge tiles are clipped.
 * Replaces rz_linear_idx_tl                                           impl/RzLinearIdx.py:6-45
 * (kernel rz_linear_idx_kernel                                        impl/RzLinearIdx.py:48-77),
 * which uses hash_levels = 1; hash_levels = 2 gives the W that the three kernels above see.
 */
int rz_materialize(const void* HW, void* W, int K, int N, int H, int BK, int BN,
                   const int32_t R[8], int hash_levels, int64_t ldw, int dtype, void* stream);

/*
 * Tile offsets computed on the DEVICE into d_out[ceil(K/BK)*ceil(N/BN)] (int32), same
 * formulas as rz_tile_offsets; lets a test compare the device hash bit for bit.
 */
int rz_tile_offsets_device(int32_t* d_out, int K, int N, int H, int BK, int BN,
                           const int32_t R[8], int hash_levels, void* stream);

/*
 * Fused optimiser steps over a parameter vector of n elements (the hashed_weight that one or
 * several layers share, or a bias): parameter, gradient and state are read and written once.
 * No counterpart in the reference, which leaves the update to torch.optim; the rules are
 * torch.optim.SGD's (momentum, dampening, weight_decay, nesterov) and torch.optim.Adam's /
 * AdamW's (decoupled != 0), amsgrad off.  param_dtype is an rz_dtype; grad_dtype is the same or
 * RZ_F32 (a gradient accumulated in fp32, RZ_WG_DHW_F32).  grad is multiplied by grad_scale
 * first (1 / loss scale, 1 / number of micro-batches; 1.0f = none).  State buffers are fp32.
 * master (optional) is an fp32 copy of the parameter that carries the update; the parameter
 * then receives its rounded value (16-bit parameters, whose small updates would otherwise be
 * rounded away).  rz_sgd_step: momentum_buf may be NULL when momentum == 0; first_step != 0
 * makes the buffer start as the gradient, as torch does.  rz_adam_step: step counts from 1.
 */
int rz_sgd_step(void* param, const void* grad, float* momentum_buf, float* master, int64_t n,
                int param_dtype, int grad_dtype, float lr, float momentum, float dampening,
                float weight_decay, int nesterov, int first_step, float grad_scale, void* stream);
int rz_adam_step(void* param, const void* grad, float* exp_avg, float* exp_avg_sq, float* master, int64_t n,
                 int param_dtype, int grad_dtype, float lr, float beta1, float beta2, float eps,
                 float weight_decay, int decoupled, int step, float grad_scale, void* stream);

/*
 * Measurement aid, no counterpart in the reference: the MFMA rate this GPU sustains on the
 * matrix work of the contraction kernels' inner loop when nothing else is in the way.  Launches
 * `workgroups` workgroups of eight wavefronts (one per compute unit fits); every wavefront issues
 * steps * 32 MFMA 32x32x16 on eight accumulator blocks, i.e. a launch is
 * workgroups * 8 * steps * 32 * 32768 flop.  mode 0: operands stay in registers; mode 1: fragments
 * come out of LDS (six 1 KB reads per eight MFMA, one barrier per step), as in the real loop.
 * operands: 64 KB of 16-bit values of `dtype` (RZ_BF16 or RZ_F16) in device memory — the clock
 * under matrix load depends on how much the operand bits toggle, so pass values like the real
 * data's.  out: workgroups * 512 floats (written, meaningless).  ticks: 2 * workgroups uint64:
 * shader clocks and ticks of the constant 100 MHz clock that the first wavefront of each
 * workgroup spent in the loop, which gives the shader clock under this load.  bench.py times
 * the launches and reports the result next to the roofline of the data sheet's peak.
 */
int rz_mfma_probe(const void* operands, void* out, void* ticks, int workgroups, int steps, int mode,
                  int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* RZLINEAR_H */
