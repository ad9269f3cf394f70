// Rulebook list form, processing order, dirty-site propagation.
#include <algorithm>

#include "common.h"
#include "grid.h"

namespace insc {

__global__ void pairs_flag_kernel(const int32_t *__restrict__ nbr, int64_t N, int K, int32_t *__restrict__ flags) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= N * K) return;
  int64_t k = t / N, o = t % N;
  flags[t] = nbr[o * K + k] >= 0 ? 1 : 0;
}

__global__ void pairs_write_kernel(const int32_t *__restrict__ nbr, int64_t N, int K,
                                   const int32_t *__restrict__ pos, const int32_t *__restrict__ total,
                                   int32_t *__restrict__ counts, int32_t *__restrict__ pairs, int64_t cap) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= N * K) return;
  int64_t k = t / N, o = t % N;
  int v = nbr[o * K + k];
  int p = pos[t];
  if (v >= 0 && p < cap) {
    pairs[2 * (int64_t)p] = v;
    pairs[2 * (int64_t)p + 1] = (int)o;
  }
  if (o == 0) {
    int end = (k + 1 < K) ? pos[(k + 1) * N] : *total;
    counts[k] = end - p;
  }
}


// sort key, 40 bits (five 8-bit radix passes): batch parity | Morton code of the 64^3 block, four
// bits per axis | neighbour pattern (27 bits).  Sites with the same pattern inside a block end up
// in the same tiles, so a tile skips the offsets none of its rows has; larger blocks give purer
// tiles (the gather locality they cost matters less than the matrix-core work they save).  The
// order is a heuristic only: blocks 1024 voxels apart and batches of equal parity share groups,
// which costs some locality and nothing else.
__global__ void order_key_kernel(const int32_t *__restrict__ coords, const int32_t *__restrict__ nbr, int64_t first,
                                 int64_t n, uint64_t *__restrict__ keys, int32_t *__restrict__ vals) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n) return;
  const int64_t i = first + t;
  int4 c = reinterpret_cast<const int4 *>(coords)[i];
  uint32_t m = 0;
  for (int k = 0; k < 27; k++) m |= (nbr[i * 27 + k] >= 0 ? 1u : 0u) << k;
  keys[t] = order_key(c, m);
  vals[t] = (int)i;
}

__global__ void offset_key_kernel(const int32_t *__restrict__ order, const int32_t *__restrict__ offset, int64_t n,
                                  uint64_t *__restrict__ keys, int32_t *__restrict__ vals) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n) return;
  const int s = order ? order[t] : (int)t;
  keys[t] = (uint64_t)(offset[s] & 7);
  vals[t] = s;
}

// the two key kernels for several scales in one launch each (blockIdx.y = scale)
struct OrderBuildJobDev {
  const int32_t *coords, *nbr, *offset, *order;
  uint64_t *keys;
  int32_t *vals;
  int64_t n;
};
struct OrderBuildBatchDev {
  OrderBuildJobDev job[SORT_BATCH_MAX_JOBS];
};
__global__ void order_key_batch_kernel(OrderBuildBatchDev b) {
  const OrderBuildJobDev &j = b.job[blockIdx.y];
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= j.n) return;
  const int4 c = reinterpret_cast<const int4 *>(j.coords)[t];
  uint32_t m = 0;
  for (int k = 0; k < 27; k++) m |= (j.nbr[t * 27 + k] >= 0 ? 1u : 0u) << k;
  j.keys[t] = order_key(c, m);
  j.vals[t] = (int)t;
}
__global__ void offset_key_batch_kernel(OrderBuildBatchDev b) {
  const OrderBuildJobDev &j = b.job[blockIdx.y];
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= j.n) return;
  const int s = j.order[t];
  j.keys[t] = (uint64_t)(j.offset[s] & 7);
  j.vals[t] = s;
}

__global__ void mark_kernel(const int32_t *__restrict__ site_of_point, int64_t P, uint8_t *__restrict__ mask) {
  int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= P) return;
  int s = site_of_point[p];
  if (s >= 0) mask[s] = 1;
}

__global__ void dilate3_kernel(const int32_t *__restrict__ nbr, const uint8_t *__restrict__ mask_in,
                               uint8_t *__restrict__ mask_out, const int32_t *__restrict__ d_n, int64_t n_upper) {
  int64_t n = d_n ? min((int64_t)*d_n, n_upper) : n_upper;
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n * 27) return;
  int64_t i = t / 27;
  if (!mask_in[i]) return;
  int j = nbr[t];
  if (j >= 0) mask_out[j] = 1;
}

__global__ void parents_kernel(const int32_t *__restrict__ parent, const uint8_t *__restrict__ mask_fine,
                               uint8_t *__restrict__ mask_coarse, const int32_t *__restrict__ d_n, int64_t n_upper) {
  int64_t n = d_n ? min((int64_t)*d_n, n_upper) : n_upper;
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  if (mask_fine[i] && parent[i] >= 0) mask_coarse[parent[i]] = 1;
}

__global__ void children_kernel(const int32_t *__restrict__ parent, const uint8_t *__restrict__ mask_coarse,
                                uint8_t *__restrict__ mask_fine, const int32_t *__restrict__ d_n, int64_t n_upper) {
  int64_t n = d_n ? min((int64_t)*d_n, n_upper) : n_upper;
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  if (parent[i] >= 0 && mask_coarse[parent[i]]) mask_fine[i] = 1;
}

__global__ void or_kernel(const uint8_t *__restrict__ a, const uint8_t *__restrict__ b, uint8_t *__restrict__ out,
                          const int32_t *__restrict__ d_n, int64_t n_upper) {
  int64_t n = d_n ? min((int64_t)*d_n, n_upper) : n_upper;
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  out[i] = (a[i] | b[i]) ? 1 : 0;
}

__global__ void compact_flag_kernel(const uint8_t *__restrict__ mask, const int32_t *__restrict__ order,
                                    const int32_t *__restrict__ d_n, int64_t n_upper, int32_t *__restrict__ flags) {
  int64_t n = d_n ? min((int64_t)*d_n, n_upper) : n_upper;
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n_upper) return;
  int f = 0;
  if (t < n) {
    int s = order ? order[t] : (int)t;
    f = (s >= 0 && mask[s]) ? 1 : 0;
  }
  flags[t] = f;
}

__global__ void compact_write_kernel(const uint8_t *__restrict__ mask, const int32_t *__restrict__ order,
                                     const int32_t *__restrict__ d_n, int64_t n_upper,
                                     const int32_t *__restrict__ pos, int32_t *__restrict__ rows) {
  int64_t n = d_n ? min((int64_t)*d_n, n_upper) : n_upper;
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n) return;
  int s = order ? order[t] : (int)t;
  if (s >= 0 && mask[s]) rows[pos[t]] = s;
}

}  // namespace insc

namespace insc {

int order_build_batch(const OrderBuildJob *jobs, int n_jobs, hipStream_t s) {
  if (n_jobs <= 0) return INSC_OK;
  if (n_jobs > SORT_BATCH_MAX_JOBS) {
    set_error("order_build_batch: at most %d scales", SORT_BATCH_MAX_JOBS);
    return INSC_ERR_ARG;
  }
  size_t bytes = 0;
  int64_t n_max = 0;
  for (int i = 0; i < n_jobs; i++) {
    if (jobs[i].n < 1 || jobs[i].n > SORT_BATCH_MAX_N || !jobs[i].g || !jobs[i].nbr || !jobs[i].order || !jobs[i].pos ||
        (jobs[i].offset && (!jobs[i].bo_order || !jobs[i].bo_pos))) {
      set_error("order_build_batch: bad job %d", i);
      return INSC_ERR_ARG;
    }
    bytes += ((sizeof(uint64_t) + sizeof(int32_t)) * (size_t)jobs[i].n + 511) & ~(size_t)255;
    n_max = std::max(n_max, jobs[i].n);
  }
  void *ws;
  int rc = workspace(WS_API, s, bytes, &ws);
  if (rc) return rc;
  char *p = (char *)ws;
  OrderBuildBatchDev b;
  SortJob sj[SORT_BATCH_MAX_JOBS];
  for (int i = 0; i < n_jobs; i++) {
    uint64_t *keys = (uint64_t *)p;
    int32_t *vals = (int32_t *)(keys + jobs[i].n);
    p += ((sizeof(uint64_t) + sizeof(int32_t)) * (size_t)jobs[i].n + 511) & ~(size_t)255;
    b.job[i] = OrderBuildJobDev{insc_grid_coords(jobs[i].g), jobs[i].nbr, jobs[i].offset, jobs[i].order, keys, vals, jobs[i].n};
    sj[i] = SortJob{keys, vals, jobs[i].order, jobs[i].pos, jobs[i].n};
  }
  hipLaunchKernelGGL(order_key_batch_kernel, dim3(grid_for(n_max, 256), (unsigned)n_jobs), dim3(256), 0, s, b);
  INSC_LAUNCH_CHECK();
  if ((rc = sort_pairs_u64_into_batch(sj, n_jobs, ORDER_KEY_BITS, s))) return rc;
  // the orders grouped by the position inside the parent cell, for the scales that have a coarser one
  OrderBuildBatchDev b2;
  int n2 = 0;
  n_max = 0;
  for (int i = 0; i < n_jobs; i++) {
    if (!jobs[i].offset) continue;
    b2.job[n2] = b.job[i];
    sj[n2] = SortJob{b.job[i].keys, b.job[i].vals, jobs[i].bo_order, jobs[i].bo_pos, jobs[i].n};
    n_max = std::max(n_max, jobs[i].n);
    n2++;
  }
  if (n2 == 0) return INSC_OK;
  hipLaunchKernelGGL(offset_key_batch_kernel, dim3(grid_for(n_max, 256), (unsigned)n2), dim3(256), 0, s, b2);
  INSC_LAUNCH_CHECK();
  return sort_pairs_u64_into_batch(sj, n2, 3, s);
}

}  // namespace insc

using namespace insc;

extern "C" {

int insc_rulebook_pairs(const int32_t *d_nbr, int64_t N, int K, int32_t *d_counts, int32_t *d_pairs,
                        int64_t pairs_capacity, int64_t *h_total, void *stream) {
  INSC_REQUIRE(N >= 0 && K > 0 && K <= 64 && pairs_capacity >= 0, INSC_ERR_ARG, "insc_rulebook_pairs: bad sizes");
  INSC_REQUIRE(d_counts && (N == 0 || (d_nbr && (d_pairs || pairs_capacity == 0))), INSC_ERR_ARG,
               "insc_rulebook_pairs: null pointer");
  INSC_REQUIRE(N * K < (1ll << 31), INSC_ERR_ARG, "insc_rulebook_pairs: N*K too large");
  hipStream_t s = (hipStream_t)stream;
  if (N == 0) {
    int rc = insc_fill_i32(d_counts, K, 0, stream);
    if (rc) return rc;
    if (h_total) *h_total = 0;
    return INSC_OK;
  }
  void *ws;
  int rc = workspace(WS_API, s, sizeof(int32_t) * (size_t)(N * K + 64), &ws);
  if (rc) return rc;
  int32_t *flags = (int32_t *)ws;
  int32_t *total = flags + N * K;
  const unsigned nb = grid_for(N * K, 256, 1ll << 30);
  hipLaunchKernelGGL(pairs_flag_kernel, dim3(nb), dim3(256), 0, s, d_nbr, N, K, flags);
  INSC_LAUNCH_CHECK();
  rc = scan_exclusive_i32(flags, flags, N * K, total, s);
  if (rc) return rc;
  hipLaunchKernelGGL(pairs_write_kernel, dim3(nb), dim3(256), 0, s, d_nbr, N, K, flags, total, d_counts, d_pairs,
                     pairs_capacity);
  INSC_LAUNCH_CHECK();
  int32_t h = 0;
  if (h_total || true) {
    INSC_HIP(hipMemcpyAsync(&h, total, sizeof(int32_t), hipMemcpyDeviceToHost, s));
    INSC_HIP(hipStreamSynchronize(s));
    if (h_total) *h_total = h;
    INSC_REQUIRE(h <= pairs_capacity, INSC_ERR_CAPACITY, "insc_rulebook_pairs: %d pairs exceed capacity %lld", h,
                 (long long)pairs_capacity);
  }
  return INSC_OK;
}

int insc_order_build(const insc_grid *g, const int32_t *d_nbr, int64_t first, int64_t n, int32_t *d_order,
                     void *stream) {
  INSC_REQUIRE(g && first >= 0 && n >= 0 && first + n <= insc_grid_capacity(g), INSC_ERR_ARG,
               "insc_order_build: bad arguments");
  INSC_REQUIRE(n == 0 || (d_nbr && d_order), INSC_ERR_ARG, "insc_order_build: null pointer");
  if (n == 0) return INSC_OK;
  hipStream_t s = (hipStream_t)stream;
  void *ws;
  int rc = workspace(WS_API, s, (sizeof(uint64_t) + sizeof(int32_t)) * (size_t)n, &ws);
  if (rc) return rc;
  uint64_t *keys = (uint64_t *)ws;
  int32_t *ids = (int32_t *)(keys + n);  // (the unsorted site ids: the sort delivers into d_order, no copy back)
  hipLaunchKernelGGL(order_key_kernel, dim3(grid_for(n, 256)), dim3(256), 0, s, insc_grid_coords(g), d_nbr, first, n,
                     keys, ids);
  INSC_LAUNCH_CHECK();
  return sort_pairs_u64_into(keys, ids, d_order + first, n, ORDER_KEY_BITS, s);
}

int insc_order_build_scales(const insc_grid *const *grids, const int32_t *const *d_nbr, const int32_t *const *d_offset,
                            const int64_t *n, int n_scales, int32_t *const *d_order, int32_t *const *d_pos,
                            int32_t *const *d_bo_order, int32_t *const *d_bo_pos, void *stream) {
  INSC_REQUIRE(grids && d_nbr && n && d_order && d_pos && n_scales >= 1 && n_scales <= SORT_BATCH_MAX_JOBS, INSC_ERR_ARG,
               "insc_order_build_scales: 1..%d scales, no null array", SORT_BATCH_MAX_JOBS);
  OrderBuildJob jobs[SORT_BATCH_MAX_JOBS];
  for (int i = 0; i < n_scales; i++) {
    INSC_REQUIRE(grids[i] && n[i] >= 1 && n[i] <= SORT_BATCH_MAX_N && n[i] <= insc_grid_capacity(grids[i]), INSC_ERR_ARG,
                 "insc_order_build_scales: scale %d has %lld sites (1..%lld, within the grid's capacity)", i,
                 (long long)n[i], (long long)SORT_BATCH_MAX_N);
    const int32_t *off = d_offset ? d_offset[i] : nullptr;
    INSC_REQUIRE(d_nbr[i] && d_order[i] && d_pos[i] && (!off || (d_bo_order && d_bo_pos && d_bo_order[i] && d_bo_pos[i])),
                 INSC_ERR_ARG, "insc_order_build_scales: null pointer at scale %d", i);
    jobs[i] = OrderBuildJob{grids[i], d_nbr[i], off, n[i], d_order[i], d_pos[i], off ? d_bo_order[i] : nullptr,
                            off ? d_bo_pos[i] : nullptr};
  }
  return order_build_batch(jobs, n_scales, (hipStream_t)stream);
}

int insc_order_by_offset(const int32_t *d_order, const int32_t *d_offset, int64_t n, int32_t *d_out, void *stream) {
  INSC_REQUIRE(n >= 0 && (n == 0 || (d_offset && d_out)), INSC_ERR_ARG, "insc_order_by_offset: bad arguments");
  if (n == 0) return INSC_OK;
  hipStream_t s = (hipStream_t)stream;
  void *ws;
  int rc = workspace(WS_API, s, (sizeof(uint64_t) + sizeof(int32_t)) * (size_t)n, &ws);
  if (rc) return rc;
  uint64_t *keys = (uint64_t *)ws;
  int32_t *ids = (int32_t *)(keys + n);
  hipLaunchKernelGGL(offset_key_kernel, dim3(grid_for(n, 256)), dim3(256), 0, s, d_order, d_offset, n, keys, ids);
  INSC_LAUNCH_CHECK();
  return sort_pairs_u64_into(keys, ids, d_out, n, 3, s);
}

int insc_dirty_mark(const int32_t *d_site_of_point, int64_t P, uint8_t *d_mask, void *stream) {
  INSC_REQUIRE(P >= 0 && (P == 0 || (d_site_of_point && d_mask)), INSC_ERR_ARG, "insc_dirty_mark: bad arguments");
  if (P == 0) return INSC_OK;
  hipLaunchKernelGGL(mark_kernel, dim3(grid_for(P, 256)), dim3(256), 0, (hipStream_t)stream, d_site_of_point, P,
                     d_mask);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

int insc_dirty_dilate3(const int32_t *d_nbr, const uint8_t *d_mask_in, uint8_t *d_mask_out, const int32_t *d_n,
                       int64_t n_upper, void *stream) {
  INSC_REQUIRE(n_upper >= 0 && (n_upper == 0 || (d_nbr && d_mask_in && d_mask_out)), INSC_ERR_ARG,
               "insc_dirty_dilate3: bad arguments");
  if (n_upper == 0) return INSC_OK;
  hipLaunchKernelGGL(dilate3_kernel, dim3(grid_for(n_upper * 27, 256, 1ll << 30)), dim3(256), 0, (hipStream_t)stream,
                     d_nbr, d_mask_in, d_mask_out, d_n, n_upper);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

int insc_dirty_parents(const int32_t *d_parent, const uint8_t *d_mask_fine, uint8_t *d_mask_coarse,
                       const int32_t *d_n_fine, int64_t n_upper, void *stream) {
  INSC_REQUIRE(n_upper >= 0 && (n_upper == 0 || (d_parent && d_mask_fine && d_mask_coarse)), INSC_ERR_ARG,
               "insc_dirty_parents: bad arguments");
  if (n_upper == 0) return INSC_OK;
  hipLaunchKernelGGL(parents_kernel, dim3(grid_for(n_upper, 256)), dim3(256), 0, (hipStream_t)stream, d_parent,
                     d_mask_fine, d_mask_coarse, d_n_fine, n_upper);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

int insc_dirty_children(const int32_t *d_parent, const uint8_t *d_mask_coarse, uint8_t *d_mask_fine,
                        const int32_t *d_n_fine, int64_t n_upper, void *stream) {
  INSC_REQUIRE(n_upper >= 0 && (n_upper == 0 || (d_parent && d_mask_fine && d_mask_coarse)), INSC_ERR_ARG,
               "insc_dirty_children: bad arguments");
  if (n_upper == 0) return INSC_OK;
  hipLaunchKernelGGL(children_kernel, dim3(grid_for(n_upper, 256)), dim3(256), 0, (hipStream_t)stream, d_parent,
                     d_mask_coarse, d_mask_fine, d_n_fine, n_upper);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

int insc_dirty_or(const uint8_t *d_a, const uint8_t *d_b, uint8_t *d_out, const int32_t *d_n, int64_t n_upper,
                  void *stream) {
  INSC_REQUIRE(n_upper >= 0 && (n_upper == 0 || (d_a && d_b && d_out)), INSC_ERR_ARG, "insc_dirty_or: bad arguments");
  if (n_upper == 0) return INSC_OK;
  hipLaunchKernelGGL(or_kernel, dim3(grid_for(n_upper, 256)), dim3(256), 0, (hipStream_t)stream, d_a, d_b, d_out,
                     d_n, n_upper);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

int insc_dirty_compact(const uint8_t *d_mask, const int32_t *d_order, const int32_t *d_n, int64_t n_upper,
                       int32_t *d_rows, int32_t *d_count, int64_t *h_count, void *stream) {
  INSC_REQUIRE(n_upper >= 0 && d_count && (n_upper == 0 || (d_mask && d_rows)), INSC_ERR_ARG,
               "insc_dirty_compact: bad arguments");
  hipStream_t s = (hipStream_t)stream;
  if (n_upper == 0) {
    int rc = insc_fill_i32(d_count, 1, 0, stream);
    if (rc) return rc;
    if (h_count) *h_count = 0;
    return INSC_OK;
  }
  void *ws;
  int rc = workspace(WS_API, s, sizeof(int32_t) * (size_t)n_upper, &ws);
  if (rc) return rc;
  int32_t *flags = (int32_t *)ws;
  const unsigned nb = grid_for(n_upper, 256);
  hipLaunchKernelGGL(compact_flag_kernel, dim3(nb), dim3(256), 0, s, d_mask, d_order, d_n, n_upper, flags);
  INSC_LAUNCH_CHECK();
  rc = scan_exclusive_i32(flags, flags, n_upper, d_count, s);
  if (rc) return rc;
  hipLaunchKernelGGL(compact_write_kernel, dim3(nb), dim3(256), 0, s, d_mask, d_order, d_n, n_upper, flags, d_rows);
  INSC_LAUNCH_CHECK();
  if (h_count) {
    int32_t h = 0;
    INSC_HIP(hipMemcpyAsync(&h, d_count, sizeof(int32_t), hipMemcpyDeviceToHost, s));
    INSC_HIP(hipStreamSynchronize(s));
    *h_count = h;
  }
  return INSC_OK;
}

}  // extern "C"
