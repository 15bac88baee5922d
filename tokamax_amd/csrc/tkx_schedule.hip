// Group-offset prefix sum + tile scheduler: one workgroup, everything in LDS.
//
// Produces, bit for bit, what the reference's GroupInfo.create_aligned computes with XLA ops
// (tokamax/_src/ops/ragged_dot/pallas_mosaic_gpu_common.py:119-151), plus the group offsets and
// the number of tasks that belong to non-empty groups, which the GEMM kernels use to skip the rest.
#include "tkx_common.h"

namespace tkx {
namespace {

constexpr int kThreads = 256;

// Exclusive scan of `partial` (one value per thread) across the workgroup; returns this thread's
// exclusive prefix and writes the grand total to *total. `buf` holds 2*kThreads ints.
__device__ inline int32_t block_exclusive_scan(int32_t v, int32_t* buf, int32_t* total) {
  const int t = threadIdx.x;
  int32_t* a = buf;
  int32_t* b = buf + kThreads;
  a[t] = v;
  __syncthreads();
  for (int d = 1; d < kThreads; d <<= 1) {
    int32_t x = a[t];
    if (t >= d) x += a[t - d];
    b[t] = x;
    __syncthreads();
    int32_t* tmp = a;
    a = b;
    b = tmp;
  }
  int32_t incl = a[t];
  *total = a[kThreads - 1];
  __syncthreads();
  return incl - v;
}

// `group_offset` (device pointer to one int32, or null for 0) and `num_global`: group_sizes has
// num_global entries and the G groups scheduled here are its entries [offset, offset + G) (the
// expert-parallel shard of experimental/gmm_v2/gmm_v2_test.py:44-101); entries outside
// [0, num_global) count as empty, and the rows of the groups before `offset` are skipped.
__global__ __launch_bounds__(kThreads) void schedule_kernel(const int32_t* __restrict__ group_sizes, int32_t G,
                                                             const int32_t* __restrict__ group_offset, int32_t num_global,
                                                             int32_t tile, int32_t tid_size, int32_t align_tile,
                                                             int32_t span_width, int32_t* __restrict__ ws,
                                                             int64_t off_offsets, int64_t off_gid, int64_t off_bstart,
                                                             int64_t off_astart, int64_t off_aend, int64_t off_swb,
                                                             int64_t off_asize, int64_t off_sfirst, int64_t off_swidth,
                                                             int64_t off_split_counters) {
  extern __shared__ int32_t smem[];
  int32_t* scan_buf = smem;                         // 2*kThreads
  int32_t* starts = smem + 2 * kThreads;            // G+1 : exclusive cumsum of clamped sizes
  int32_t* start_tasks = starts + (G + 1);          // G+1 : exclusive cumsum of blocks per group
  const int t = threadIdx.x;
  for (int i = t; i < kSplitUnits; i += kThreads) ws[off_split_counters + i] = 0;  // arrival counters of a split launch
  const int per = (G + kThreads - 1) / kThreads;
  const int lo = min(t * per, G), hi = min(lo + per, G);

  const int32_t goff = group_offset != nullptr ? group_offset[0] : 0;
  auto size_of = [&](int g) -> int32_t {
    const int64_t j = (int64_t)goff + g;
    return j >= 0 && j < num_global ? max(group_sizes[j], 0) : 0;
  };
  // pass 0: rows of the groups before the first one of this shard
  int32_t local = 0;
  const int32_t before = min(max(goff, 0), num_global);
  for (int j = t; j < before; j += kThreads) local += max(group_sizes[j], 0);
  int32_t lead;
  block_exclusive_scan(local, scan_buf, &lead);

  // pass 1: group starts
  local = 0;
  for (int g = lo; g < hi; ++g) local += size_of(g);
  int32_t total_rows;
  int32_t run = lead + block_exclusive_scan(local, scan_buf, &total_rows);
  total_rows += lead;
  for (int g = lo; g < hi; ++g) {
    starts[g] = run;
    run += size_of(g);
  }
  if (t == 0) starts[G] = total_rows;
  __syncthreads();

  // pass 2: blocks per group -> first task of each group
  auto blocks_of = [&](int g) -> int32_t {
    int32_t sz = size_of(g);
    int32_t aligned = (starts[g] / align_tile) * align_tile;
    return sz == 0 ? 0 : (starts[g] + sz - aligned + tile - 1) / tile;
  };
  local = 0;
  for (int g = lo; g < hi; ++g) local += blocks_of(g);
  int32_t num_tasks;
  run = block_exclusive_scan(local, scan_buf, &num_tasks);
  for (int g = lo; g < hi; ++g) {
    start_tasks[g] = run;
    run += blocks_of(g);
  }
  if (t == 0) {
    start_tasks[G] = num_tasks;
    ws[0] = num_tasks;
    ws[1] = total_rows;
    ws[2] = lead;
  }
  __syncthreads();

  for (int g = t; g <= G; g += kThreads) ws[off_offsets + g] = starts[g];

  // pass 3: tasks. group = #{ j < G-1 : end_task[j] <= task }, end_task[j] == start_tasks[j+1].
  for (int task = t; task < tid_size; task += kThreads) {
    int l = 0, h = G - 1;  // search in start_tasks[1 .. G-1]
    while (l < h) {
      int mid = (l + h) >> 1;
      if (start_tasks[mid + 1] <= task) l = mid + 1; else h = mid;
    }
    const int g = l;
    const int32_t sz = size_of(g);
    const int32_t aligned = (starts[g] / align_tile) * align_tile;
    const int32_t end = starts[g] + sz;
    const int32_t bs = aligned + tile * (task - start_tasks[g]);
    const int32_t vs = max(bs, starts[g]);
    const int32_t ve = min(bs + tile, end);
    ws[off_gid + task] = g;
    ws[off_bstart + task] = bs;
    ws[off_astart + task] = vs;
    ws[off_aend + task] = ve;
    ws[off_swb + task] = vs - bs;
    ws[off_asize + task] = max(0, ve - vs);
    // Span of this task: the group's T tasks are cut into ceil(T / span_width) spans of nearly equal
    // width, so that the tasks that run side by side on an n-panel all use the same group's weights.
    int32_t sfirst = task, swidth = 1;
    // (Sizes that add up to more than m rows make more tasks than slots: spans end with the slots, so that the
    // launch order, which walks whole spans, stays inside the arrays.)
    const int32_t T = min(start_tasks[g + 1], tid_size) - start_tasks[g], idx = task - start_tasks[g];
    if (task < num_tasks && idx < T) {
      const int32_t nspans = (T + span_width - 1) / span_width;
      const int32_t base = T / nspans, extra = T - base * nspans;  // the first `extra` spans are one wider
      const int32_t wide = extra * (base + 1);
      if (idx < wide) {
        swidth = base + 1;
        sfirst = idx / swidth * swidth;
      } else {
        swidth = base;
        sfirst = wide + (idx - wide) / base * base;
      }
      sfirst += start_tasks[g];
    }
    ws[off_sfirst + task] = sfirst;
    ws[off_swidth + task] = swidth;
  }
}

}  // namespace

int32_t launch_schedule(const int32_t* group_sizes, int64_t G, const int32_t* group_offset, int64_t num_global, int64_t m,
                        int32_t block_m, int32_t align_tile, int32_t span_width, int32_t* ws, const WsLayout& L,
                        hipStream_t stream) {
  (void)m;
  const size_t smem = sizeof(int32_t) * (size_t)(2 * kThreads + 2 * (G + 1));
  if (smem > 64 * 1024) return set_error(TKX_ERR_UNSUPPORTED, "num_groups=%lld too large for the scheduler", (long long)G);
  if (num_global < 0 || num_global > 0x7fffffffLL) return set_error(TKX_ERR_INVALID, "bad number of group sizes");
  schedule_kernel<<<1, kThreads, smem, stream>>>(group_sizes, (int32_t)G, group_offset, (int32_t)num_global, block_m, L.tid_size, align_tile,
                                                span_width < 1 ? 1 : span_width, ws, L.offsets, L.task[0], L.task[1],
                                                L.task[2], L.task[3], L.task[4], L.task[5], L.task[6], L.task[7],
                                                L.split_counters);
  TKX_HIP_CHECK(hipGetLastError());
  return TKX_OK;
}

}  // namespace tkx
