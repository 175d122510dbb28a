/*
 * CPU restatement of the RzLinear hot path (tile hash, forward, input-grad,
 * weight-grad, materialise).  TEST INFRASTRUCTURE ONLY: this file is the checker
 * that the HIP kernels are compared against.  Nothing in the product package may
 * link, load or call it; only tests, the smoke check and the CPU-baseline leg of
 * the benchmark do.
 *
 * Every function follows the loop structure of the reference's device kernels
 * (one program per output tile, a loop over tiles of the contracted dimension,
 * masks that read out-of-range rows/columns as zero) and accumulates in double,
 * so that it can referee both the fp32 and the 16-bit kernels.
 *
 * Reference lines restated (paths relative to the reference checkout):
 *   tile offset, two-level hash   python/rz_linear/impl/RzLinearForward.py:316,:349
 *                                 python/rz_linear/impl/RzLinearBackward.py:369,:686,:716
 *   tile offset, one-level hash   python/rz_linear/impl/RzLinearIdx.py:70-71
 *   element address in a tile     python/rz_linear/impl/RzLinearForward.py:312-313
 *   forward                       python/rz_linear/impl/RzLinearForward.py:271-357
 *   input-grad                    python/rz_linear/impl/RzLinearBackward.py:642-727
 *   weight-grad                   python/rz_linear/impl/RzLinearBackward.py:291-371
 *   materialise                   python/rz_linear/impl/RzLinearIdx.py:48-77
 *
 * Parity status: pinned.  The reference ships no golden vectors for the two-level
 * hash (its own forward/backward tests no longer match its launcher signatures),
 * so vectors were produced once by running the reference's own Triton kernels under
 * Triton's CPU interpreter (tests/golden/make_reference_vectors.py ->
 * tests/golden/reference_vectors.npz); forward, input-grad and weight-grad here
 * agree with them to fp32 rounding.  Independent of that, tests/test_oracle.py
 * holds hand-evaluated offsets, degenerate hashes, the identity-input trick,
 * torch.autograd through a gather and brute force on tiny shapes.
 * The one-level materialiser is pinned by the formula inside the reference's
 * test_get_idx (python/tests/test_rz_linear.py:21-33).
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define RZ_EXPORT __attribute__((visibility("default")))

/* R[0]=P (prime), R[1..7] random in [0,P); R[6] takes part in no formula. */
RZ_EXPORT int64_t rz_oracle_tile_offset(int64_t tk, int64_t tn, int64_t H, int64_t BK,
                                        int64_t BN, const int32_t *R, int hash_levels) {
  const int64_t R0 = R[0];
  const int64_t range = H - BK * BN; /* precondition H > BK*BN, RzLinearForward.py:28 */
  const int64_t hi = (tk * R[3] + tn * R[2] + R[1]) % R0;
  /* legacy generation: one level, 64-bit, range + 1 (/rz_linear_kernel.cu:34-36,:56-64) */
  if (hash_levels == 3) return hi % (range + 1);
  if (hash_levels == 1) return hi % range; /* RzLinearIdx.py:70-71 */
  const int64_t lo = (tk * R[7] + tn * R[5] + R[4]) % R0;
  return (hi * R0 + lo) % range;
}

/* out[tk*TN + tn], TK = ceil(K/BK), TN = ceil(N/BN).  Returns 0, or -1 when the
 * precondition H > BK*BN fails, or -2 when an intermediate would leave int32
 * (the reference evaluates the hash in 32-bit integers). */
RZ_EXPORT int rz_oracle_tile_offsets(int64_t *out, int64_t K, int64_t N, int64_t H, int64_t BK,
                                     int64_t BN, const int32_t *R, int hash_levels) {
  if (hash_levels == 3 ? H < BK * BN : H <= BK * BN) return -1;
  const int64_t TK = (K + BK - 1) / BK, TN = (N + BN - 1) / BN;
  const int64_t lim = 2147483647LL;
  const int64_t R0 = R[0];
  if (hash_levels != 3) { /* the legacy hash is evaluated in 64-bit integers */
    if ((TK * (int64_t)R[3] + TN * (int64_t)R[2] + R[1]) > lim) return -2;
    if ((TK * (int64_t)R[7] + TN * (int64_t)R[5] + R[4]) > lim) return -2;
    if (hash_levels != 1 && (R0 - 1) * R0 + (R0 - 1) > lim) return -2;
  }
  for (int64_t tk = 0; tk < TK; tk++)
    for (int64_t tn = 0; tn < TN; tn++)
      out[tk * TN + tn] = rz_oracle_tile_offset(tk, tn, H, BK, BN, R, hash_levels);
  return 0;
}

/* W[k,n] = hw[off(k/BK, n/BN) + (k%BK)*BN + n%BN]   (RzLinearForward.py:312-313) */
RZ_EXPORT int rz_oracle_materialize(const double *hw, double *W, int64_t K, int64_t N, int64_t H,
                                    int64_t BK, int64_t BN, const int32_t *R, int hash_levels) {
  if (H <= BK * BN) return -1;
  for (int64_t k = 0; k < K; k++)
    for (int64_t n = 0; n < N; n++) {
      int64_t off = rz_oracle_tile_offset(k / BK, n / BN, H, BK, BN, R, hash_levels);
      W[k * N + n] = hw[off + (k % BK) * BN + (n % BN)];
    }
  return 0;
}

/* Y[M,N] = (X[M,K] . W) * f, one "program" per (row, tile column), a loop over
 * K tiles that re-hashes at every step (RzLinearForward.py:329-349), the mask
 * k<K, n<N giving zeros (:338-341), the scale at the store (:357). */
RZ_EXPORT int rz_oracle_forward(const double *X, const double *hw, double *Y, int64_t M, int64_t K,
                                int64_t N, int64_t H, int64_t BK, int64_t BN, const int32_t *R,
                                double f) {
  if (H <= BK * BN) return -1;
  const int64_t TK = (K + BK - 1) / BK, TN = (N + BN - 1) / BN;
  double *acc = (double *)malloc(sizeof(double) * BN);
  for (int64_t m = 0; m < M; m++)
    for (int64_t tn = 0; tn < TN; tn++) {
      memset(acc, 0, sizeof(double) * BN);
      for (int64_t tk = 0; tk < TK; tk++) {
        const double *tile = hw + rz_oracle_tile_offset(tk, tn, H, BK, BN, R, 2);
        for (int64_t kk = 0; kk < BK && tk * BK + kk < K; kk++) {
          const double a = X[m * K + tk * BK + kk];
          const double *row = tile + kk * BN;
          for (int64_t nn = 0; nn < BN; nn++) acc[nn] += a * row[nn];
        }
      }
      for (int64_t nn = 0; nn < BN && tn * BN + nn < N; nn++) Y[m * N + tn * BN + nn] = acc[nn] * f;
    }
  free(acc);
  return 0;
}

/* dX[M,K] = (dY[M,N] . W^T) * f: program (row, tile row tk) loops over N tiles
 * and reads the same slice transposed (RzLinearBackward.py:679-681,:696-716). */
RZ_EXPORT int rz_oracle_input_grad(const double *dY, const double *hw, double *dX, int64_t M,
                                   int64_t K, int64_t N, int64_t H, int64_t BK, int64_t BN,
                                   const int32_t *R, double f) {
  if (H <= BK * BN) return -1;
  const int64_t TK = (K + BK - 1) / BK, TN = (N + BN - 1) / BN;
  double *acc = (double *)malloc(sizeof(double) * BK);
  for (int64_t m = 0; m < M; m++)
    for (int64_t tk = 0; tk < TK; tk++) {
      memset(acc, 0, sizeof(double) * BK);
      for (int64_t tn = 0; tn < TN; tn++) {
        const double *tile = hw + rz_oracle_tile_offset(tk, tn, H, BK, BN, R, 2);
        for (int64_t nn = 0; nn < BN && tn * BN + nn < N; nn++) {
          const double g = dY[m * N + tn * BN + nn];
          for (int64_t kk = 0; kk < BK; kk++) acc[kk] += g * tile[kk * BN + nn];
        }
      }
      for (int64_t kk = 0; kk < BK && tk * BK + kk < K; kk++) dX[m * K + tk * BK + kk] = acc[kk] * f;
    }
  free(acc);
  return 0;
}

/* dHW[H]: one program per W tile reduces X^T.dY over all of M, then adds the whole
 * BKxBN tile (out-of-range rows/columns are zero) times f into the slice of the
 * zero-initialised output (RzLinearBackward.py:344-371, zeros at :47-48). */
RZ_EXPORT int rz_oracle_weight_grad(const double *X, const double *dY, double *dHW, int64_t M,
                                    int64_t K, int64_t N, int64_t H, int64_t BK, int64_t BN,
                                    const int32_t *R, double f) {
  if (H <= BK * BN) return -1;
  const int64_t TK = (K + BK - 1) / BK, TN = (N + BN - 1) / BN;
  double *c = (double *)malloc(sizeof(double) * BK * BN);
  memset(dHW, 0, sizeof(double) * H);
  for (int64_t tk = 0; tk < TK; tk++)
    for (int64_t tn = 0; tn < TN; tn++) {
      memset(c, 0, sizeof(double) * BK * BN);
      for (int64_t m = 0; m < M; m++)
        for (int64_t kk = 0; kk < BK && tk * BK + kk < K; kk++) {
          const double a = X[m * K + tk * BK + kk];
          const double *g = dY + m * N + tn * BN;
          double *crow = c + kk * BN;
          for (int64_t nn = 0; nn < BN && tn * BN + nn < N; nn++) crow[nn] += a * g[nn];
        }
      double *dst = dHW + rz_oracle_tile_offset(tk, tn, H, BK, BN, R, 2);
      for (int64_t i = 0; i < BK * BN; i++) dst[i] += c[i] * f;
    }
  free(c);
  return 0;
}
