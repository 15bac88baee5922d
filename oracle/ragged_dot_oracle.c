/* CPU oracle for tokamax.ragged_dot in plain C -- TEST INFRASTRUCTURE ONLY.
 *
 * A second, independent restatement (next to ragged_dot_oracle.py) of the
 * reference's tile scheduler and of its XLA ragged dot, used by the tests to
 * cross-check the NumPy oracle and by bench.py as the single-thread CPU leg.
 * Nothing in the shipped library links or loads this file.
 *
 * Follows, in the reference tree:
 *   oracle_group_offsets   tokamax/_src/ops/ragged_dot/pallas_mosaic_gpu_common.py:119-121
 *   oracle_create_aligned  tokamax/_src/ops/ragged_dot/pallas_mosaic_gpu_common.py:119-151
 *   oracle_ragged_dot_f32  tokamax/_src/ops/ragged_dot/base.py:291-360 (mode 0/1/2 = the three
 *                          dimension-number sets at base.py:40-54), f32 accumulation
 * Pins: the scheduler against the literal vectors of pallas_mosaic_gpu_common_test.py:27-84;
 * the GEMM against brute force / library GEMM special cases (see tests/test_oracle.py).
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static int32_t imax(int32_t a, int32_t b) { return a > b ? a : b; }
static int32_t imin(int32_t a, int32_t b) { return a < b ? a : b; }

/* offsets[G+1] = exclusive prefix sum of max(group_sizes, 0). */
void oracle_group_offsets(const int32_t* group_sizes, int64_t G, int32_t* offsets) {
  int32_t acc = 0;
  offsets[0] = 0;
  for (int64_t g = 0; g < G; ++g) {
    acc += imax(group_sizes[g], 0);
    offsets[g + 1] = acc;
  }
}

/* Six arrays of tid_size int32 each, laid out back to back in `out`:
 * group_id, block_start, actual_start, actual_end, start_within_block, actual_size.
 * Returns the number of tasks that belong to non-empty groups. */
int32_t oracle_create_aligned(const int32_t* group_sizes, int64_t G, int32_t tile, int32_t tid_size,
                              int32_t align_tile, int32_t* out) {
  int32_t* starts = (int32_t*)malloc(sizeof(int32_t) * (size_t)(G + 1));
  int32_t* start_tasks = (int32_t*)malloc(sizeof(int32_t) * (size_t)(G + 1));
  oracle_group_offsets(group_sizes, G, starts);
  start_tasks[0] = 0;
  for (int64_t g = 0; g < G; ++g) {
    int32_t sz = imax(group_sizes[g], 0);
    int32_t aligned = (starts[g] / align_tile) * align_tile;
    int32_t end = starts[g] + sz;
    int32_t nb = sz == 0 ? 0 : (end - aligned + tile - 1) / tile;
    start_tasks[g + 1] = start_tasks[g] + nb;
  }
  int32_t* group_id = out;
  int32_t* block_start = out + tid_size;
  int32_t* actual_start = out + 2 * (int64_t)tid_size;
  int32_t* actual_end = out + 3 * (int64_t)tid_size;
  int32_t* start_within = out + 4 * (int64_t)tid_size;
  int32_t* actual_size = out + 5 * (int64_t)tid_size;
  for (int32_t t = 0; t < tid_size; ++t) {
    /* searchsorted(group_end_tasks[:-1], t, side="right"): count of entries <= t among the
     * first G-1 end-task values (end_task[g] == start_tasks[g+1]). */
    int32_t g = 0;
    while (g < G - 1 && start_tasks[g + 1] <= t) ++g;
    int32_t sz = imax(group_sizes[g], 0);
    int32_t aligned = (starts[g] / align_tile) * align_tile;
    int32_t end = starts[g] + sz;
    int32_t bs = aligned + tile * (t - start_tasks[g]);
    int32_t vs = imax(bs, starts[g]);
    int32_t ve = imin(bs + tile, end);
    group_id[t] = g;
    block_start[t] = bs;
    actual_start[t] = vs;
    actual_end[t] = ve;
    start_within[t] = vs - bs;
    actual_size[t] = imax(0, ve - vs);
  }
  int32_t n = start_tasks[G];
  free(starts);
  free(start_tasks);
  return n;
}

/* mode 0: out[m,n]   = lhs[m,k]  . rhs[g,k,n]      (rows of group g use rhs[g])
 * mode 1: out[m,k]   = lhs[m,n]  . rhs[g,k,n]^T
 * mode 2: out[g,k,n] = lhs[rows_g,k]^T . rhs[rows_g,n]
 * All row-major f32, f32 accumulation in index order; rows >= sum(sizes) give zeros. */
void oracle_ragged_dot_f32(const float* lhs, const float* rhs, const int32_t* group_sizes, float* out,
                           int64_t m, int64_t k, int64_t n, int64_t G, int32_t mode) {
  int32_t* off = (int32_t*)malloc(sizeof(int32_t) * (size_t)(G + 1));
  oracle_group_offsets(group_sizes, G, off);
  if (mode == 0) {
    memset(out, 0, sizeof(float) * (size_t)(m * n));
    for (int64_t g = 0; g < G; ++g) {
      int64_t s = off[g], e = off[g + 1] < m ? off[g + 1] : m;
      const float* w = rhs + g * k * n;
      for (int64_t i = s; i < e; ++i) {
        float* o = out + i * n;
        for (int64_t kk = 0; kk < k; ++kk) {
          float a = lhs[i * k + kk];
          const float* wr = w + kk * n;
          for (int64_t j = 0; j < n; ++j) o[j] += a * wr[j];
        }
      }
    }
  } else if (mode == 1) {
    memset(out, 0, sizeof(float) * (size_t)(m * k));
    for (int64_t g = 0; g < G; ++g) {
      int64_t s = off[g], e = off[g + 1] < m ? off[g + 1] : m;
      const float* w = rhs + g * k * n;
      for (int64_t i = s; i < e; ++i)
        for (int64_t kk = 0; kk < k; ++kk) {
          float acc = 0.f;
          for (int64_t j = 0; j < n; ++j) acc += lhs[i * n + j] * w[kk * n + j];
          out[i * k + kk] = acc;
        }
    }
  } else {
    memset(out, 0, sizeof(float) * (size_t)(G * k * n));
    for (int64_t g = 0; g < G; ++g) {
      int64_t s = off[g], e = off[g + 1] < m ? off[g + 1] : m;
      float* o = out + g * k * n;
      for (int64_t i = s; i < e; ++i)
        for (int64_t kk = 0; kk < k; ++kk) {
          float a = lhs[i * k + kk];
          for (int64_t j = 0; j < n; ++j) o[kk * n + j] += a * rhs[i * n + j];
        }
    }
  }
  free(off);
}
