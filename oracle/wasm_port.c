/*
 * wasm_port.c -- single-core C restatement of the loop nests the reference's Wasm backend
 * generates for f32 matmul and matvec.  TEST / BASELINE INFRASTRUCTURE ONLY: it is timed as the
 * "port" CPU baseline next to the GPU numbers and never called by the product.
 *
 * What is restated (paths relative to the reference tree):
 *   - tiled-SIMD reduction: 128-row x 128-column x K=64 tiles, a 4-row x 4-vector micro tile of
 *     f32x4 accumulators, partial sums parked in the output between K tiles
 *       plan    src/backend/wasm/tilePlan.ts:38-45, 278-304
 *       loops   src/backend/wasm/codegen.ts:874-967, 560-694
 *   - K-SIMD reduction (matvec): 4 rows at a time, one f32x4 accumulator per row running along
 *     K with 4x unrolling, lanes summed l0+l1+l2+l3 at the end
 *       plan    src/backend/wasm/tilePlan.ts:306-334
 *       loops   src/backend/wasm/codegen.ts:744-872
 * In Node the backend runs these on the calling thread (no Worker => no pool,
 * src/backend/wasm/parallel.ts:14-19, 262-266), so one core is the faithful setting.
 * Products are combined with a separate multiply and add (the path taken when the engine does
 * not validate relaxed-madd, src/backend/wasm/codegen.ts:318-322).
 *
 * Parity unpinned at the bit level: only a live run of the reference could fix the exact f32
 * sums; tests compare this file with an f64 GEMM under a K-scaled bound.
 */

#include <stdint.h>
#include <string.h>

typedef float f32x4 __attribute__((vector_size(16), aligned(4)));

static inline f32x4 splat(float x) { return (f32x4){x, x, x, x}; }
static inline f32x4 loadu(const float *p) {
  f32x4 v;
  memcpy(&v, p, 16);
  return v;
}
static inline void storeu(float *p, f32x4 v) { memcpy(p, &v, 16); }

static int64_t pow2_at_most(int64_t max) { /* findPow2(0, max) in src/utils.ts:298-307 */
  int64_t r = 1;
  while (2 * r <= max) r *= 2;
  return r;
}

/* C[M,N] = A[M,K] . B[K,N], all row-major f32.  Requires N % 4 == 0 (the SIMD path's own guard);
 * returns non-zero otherwise. */
int jo_wasm_matmul_f32(const float *A, const float *B, float *C, int64_t M, int64_t N, int64_t K) {
  if (N % 4 != 0 || M < 1 || K < 1) return 1;
  int64_t tile_rows = M / 2 < 1 ? 1 : (M / 2 > 128 ? 128 : M / 2);
  tile_rows = pow2_at_most(tile_rows);
  int64_t tile_vecs = N / 4 / 2 < 1 ? 1 : (N / 4 / 2 > 32 ? 32 : N / 4 / 2);
  tile_vecs = pow2_at_most(tile_vecs);
  const int64_t tile_cols = tile_vecs * 4;
  int64_t tile_k = 1;
  for (int64_t d = K < 64 ? K : 64; d > 1; d--)
    if (K % d == 0) { tile_k = d; break; }
  int64_t micro_rows = 1;
  for (int64_t d = 4; d > 1; d--)
    if (tile_rows % d == 0 && M % d == 0) { micro_rows = d; break; }
  const int64_t micro_vecs = tile_vecs < 4 ? tile_vecs : 4;

  for (int64_t row_tile = 0; row_tile < M; row_tile += tile_rows) {
    const int64_t row_end = row_tile + tile_rows < M ? row_tile + tile_rows : M;
    for (int64_t col_tile = 0; col_tile < N; col_tile += tile_cols) {
      const int64_t col_end = col_tile + tile_cols < N ? col_tile + tile_cols : N;
      for (int64_t k0 = 0; k0 < K; k0 += tile_k) {
        const int64_t k1 = k0 + tile_k;
        for (int64_t r0 = row_tile; r0 + micro_rows <= row_end; r0 += micro_rows) {
          int64_t col = col_tile;
          for (; col + micro_vecs * 4 <= col_end; col += micro_vecs * 4) {
            f32x4 acc[4][4];
            for (int64_t r = 0; r < micro_rows; r++)
              for (int64_t v = 0; v < micro_vecs; v++)
                acc[r][v] = k0 == 0 ? splat(0.0f) : loadu(C + (r0 + r) * N + col + 4 * v);
            for (int64_t k = k0; k < k1; k++) {
              f32x4 b[4];
              for (int64_t v = 0; v < micro_vecs; v++) b[v] = loadu(B + k * N + col + 4 * v);
              for (int64_t r = 0; r < micro_rows; r++) {
                const f32x4 a = splat(A[(r0 + r) * K + k]);
                for (int64_t v = 0; v < micro_vecs; v++) acc[r][v] = a * b[v] + acc[r][v];
              }
            }
            for (int64_t r = 0; r < micro_rows; r++)
              for (int64_t v = 0; v < micro_vecs; v++) storeu(C + (r0 + r) * N + col + 4 * v, acc[r][v]);
          }
          for (; col < col_end; col += 4) { /* leftover single vectors */
            for (int64_t r = 0; r < micro_rows; r++) {
              f32x4 acc = k0 == 0 ? splat(0.0f) : loadu(C + (r0 + r) * N + col);
              for (int64_t k = k0; k < k1; k++) acc = splat(A[(r0 + r) * K + k]) * loadu(B + k * N + col) + acc;
              storeu(C + (r0 + r) * N + col, acc);
            }
          }
        }
      }
    }
  }
  return 0;
}

/* y[M] = W[M,K] . x[K], row-major f32, K % 4 == 0. */
int jo_wasm_matvec_f32(const float *W, const float *x, float *y, int64_t M, int64_t K) {
  if (K % 4 != 0) return 1;
  int64_t unroll = 1;
  for (int64_t d = 4; d > 1; d--)
    if ((K / 4) % d == 0) { unroll = d; break; }
  int64_t micro_rows = 1;
  for (int64_t d = 4; d > 1; d--)
    if (M % d == 0) { micro_rows = d; break; }
  for (int64_t r0 = 0; r0 < M; r0 += micro_rows) {
    f32x4 acc[4] = {splat(0.0f), splat(0.0f), splat(0.0f), splat(0.0f)};
    for (int64_t k = 0; k < K; k += 4 * unroll) {
      for (int64_t u = 0; u < unroll; u++) {
        const f32x4 xv = loadu(x + k + 4 * u);
        for (int64_t r = 0; r < micro_rows; r++) acc[r] = loadu(W + (r0 + r) * K + k + 4 * u) * xv + acc[r];
      }
    }
    for (int64_t r = 0; r < micro_rows; r++) y[r0 + r] = ((acc[r][0] + acc[r][1]) + acc[r][2]) + acc[r][3];
  }
  return 0;
}
