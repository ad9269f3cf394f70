// Device-wide exclusive scan and stable LSD radix sort.  These replace the CUDPP scan /
// compact / radix-sort calls the reference leans on (CUDA/CUDPPWrapper.hpp:30-217).
#include <algorithm>

#include "common.h"

namespace insc {

constexpr int SCAN_THREADS = 256;
constexpr int SCAN_ITEMS = 8;
constexpr int SCAN_TILE = SCAN_THREADS * SCAN_ITEMS;

__device__ __forceinline__ int wave_incl_scan(int v) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    int t = __shfl_up(v, d, 64);
    if (lane >= d) v += t;
  }
  return v;
}

// exclusive scan of one value per thread across a 256-thread block; returns block total
__device__ __forceinline__ int block_excl_scan(int v, int *total, int *lds /*[4]*/) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  int inc = wave_incl_scan(v);
  if (lane == 63) lds[w] = inc;
  __syncthreads();
  int off = 0, tot = 0;
#pragma unroll
  for (int i = 0; i < SCAN_THREADS / 64; i++) {
    int s = lds[i];
    if (i < w) off += s;
    tot += s;
  }
  __syncthreads();
  *total = tot;
  return off + inc - v;
}

__global__ __launch_bounds__(SCAN_THREADS) void scan_block_sums(const int32_t *__restrict__ in, int64_t n,
                                                                int32_t *__restrict__ bsums) {
  __shared__ int lds[4];
  int64_t base = (int64_t)blockIdx.x * SCAN_TILE + (int64_t)threadIdx.x * SCAN_ITEMS;
  int s = 0;
#pragma unroll
  for (int i = 0; i < SCAN_ITEMS; i++)
    if (base + i < n) s += in[base + i];
  int tot;
  block_excl_scan(s, &tot, lds);
  if (threadIdx.x == 0) bsums[blockIdx.x] = tot;
}

// single block: exclusive scan of bsums[0..nb) in place, total to *total (if non-null)
__global__ __launch_bounds__(SCAN_THREADS) void scan_bsums(int32_t *__restrict__ bsums, int64_t nb,
                                                           int32_t *__restrict__ total) {
  __shared__ int lds[4];
  int carry = 0;
  for (int64_t base = 0; base < nb; base += SCAN_THREADS) {
    int64_t i = base + threadIdx.x;
    int v = (i < nb) ? bsums[i] : 0;
    int tot;
    int ex = block_excl_scan(v, &tot, lds);
    if (i < nb) bsums[i] = carry + ex;
    carry += tot;
  }
  if (threadIdx.x == 0 && total) *total = carry;
}

__global__ __launch_bounds__(SCAN_THREADS) void scan_final(const int32_t *__restrict__ in, int32_t *__restrict__ out,
                                                           int64_t n, const int32_t *__restrict__ bsums) {
  __shared__ int lds[4];
  int64_t base = (int64_t)blockIdx.x * SCAN_TILE + (int64_t)threadIdx.x * SCAN_ITEMS;
  int v[SCAN_ITEMS];
  int s = 0;
#pragma unroll
  for (int i = 0; i < SCAN_ITEMS; i++) {
    v[i] = (base + i < n) ? in[base + i] : 0;
    s += v[i];
  }
  int tot;
  int ex = block_excl_scan(s, &tot, lds) + bsums[blockIdx.x];
#pragma unroll
  for (int i = 0; i < SCAN_ITEMS; i++) {
    if (base + i < n) out[base + i] = ex;
    ex += v[i];
  }
}

// scan_final for up to SCAN_FUSED_MAX_BLOCKS blocks: every block adds up the sums of the blocks before it by
// itself (at most 16 loads per thread) instead of reading them from a scan that a launch of its own made;
// the last block leaves the grand total.
constexpr int SCAN_FUSED_MAX_BLOCKS = 4096;
__global__ __launch_bounds__(SCAN_THREADS) void scan_final_fused(const int32_t *__restrict__ in, int32_t *__restrict__ out,
                                                                 int64_t n, const int32_t *__restrict__ bsums,
                                                                 int32_t *__restrict__ total) {
  __shared__ int lds[4];
  __shared__ int pre_w[4];
  int pre = 0;
  for (int i = threadIdx.x; i < (int)blockIdx.x; i += SCAN_THREADS) pre += bsums[i];
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) pre += __shfl_xor(pre, d, 64);
  if ((threadIdx.x & 63) == 0) pre_w[threadIdx.x >> 6] = pre;
  int64_t base = (int64_t)blockIdx.x * SCAN_TILE + (int64_t)threadIdx.x * SCAN_ITEMS;
  int v[SCAN_ITEMS];
  int s = 0;
#pragma unroll
  for (int i = 0; i < SCAN_ITEMS; i++) {
    v[i] = (base + i < n) ? in[base + i] : 0;
    s += v[i];
  }
  int tot;
  int ex = block_excl_scan(s, &tot, lds);  // (its barriers also publish pre_w)
  const int before = pre_w[0] + pre_w[1] + pre_w[2] + pre_w[3];
  ex += before;
#pragma unroll
  for (int i = 0; i < SCAN_ITEMS; i++) {
    if (base + i < n) out[base + i] = ex;
    ex += v[i];
  }
  if (total && blockIdx.x == gridDim.x - 1 && threadIdx.x == 0) *total = before + tot;
}

__global__ void scan_zero_total(int32_t *total) { *total = 0; }

// Short inputs (the digit counts of a radix pass, the rows of a coarse scale): one workgroup of 1024
// threads, up to 32 consecutive values per thread, one launch instead of three.
constexpr int SCAN_ONE_THREADS = 1024;
constexpr int SCAN_ONE_ITEMS = 32;
constexpr int SCAN_ONE_MAX = SCAN_ONE_THREADS * SCAN_ONE_ITEMS;
__device__ __forceinline__ void scan_one_block_body(const int32_t *__restrict__ in, int32_t *__restrict__ out, int n,
                                                    int32_t *__restrict__ total, int *wsum /*[SCAN_ONE_THREADS / 64]*/) {
  const int per = (n + SCAN_ONE_THREADS - 1) / SCAN_ONE_THREADS;  // <= SCAN_ONE_ITEMS
  const int base = threadIdx.x * per;
  int v[SCAN_ONE_ITEMS];
  int sum = 0;
#pragma unroll
  for (int i = 0; i < SCAN_ONE_ITEMS; i++) {
    v[i] = (i < per && base + i < n) ? in[base + i] : 0;
    sum += v[i];
  }
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int inc = wave_incl_scan(sum);
  if (lane == 63) wsum[w] = inc;
  __syncthreads();  // (also: every value has been read before the first one is written - in may be out)
  int off = 0, tot = 0;
#pragma unroll
  for (int i = 0; i < SCAN_ONE_THREADS / 64; i++) {
    const int t = wsum[i];
    if (i < w) off += t;
    tot += t;
  }
  int ex = off + inc - sum;
#pragma unroll
  for (int i = 0; i < SCAN_ONE_ITEMS; i++) {
    if (i < per && base + i < n) out[base + i] = ex;
    ex += v[i];
  }
  if (threadIdx.x == 0 && total) *total = tot;
}
__global__ __launch_bounds__(SCAN_ONE_THREADS) void scan_one_block(const int32_t *__restrict__ in,
                                                                   int32_t *__restrict__ out, int n,
                                                                   int32_t *__restrict__ total) {
  __shared__ int wsum[SCAN_ONE_THREADS / 64];
  scan_one_block_body(in, out, n, total, wsum);
}

int scan_exclusive_i32(const int32_t *in, int32_t *out, int64_t n, int32_t *total, hipStream_t s) {
  if (n <= 0) {
    if (total) {
      hipLaunchKernelGGL(scan_zero_total, dim3(1), dim3(1), 0, s, total);
      INSC_LAUNCH_CHECK();
    }
    return INSC_OK;
  }
  if (n <= SCAN_ONE_MAX) {
    hipLaunchKernelGGL(scan_one_block, dim3(1), dim3(SCAN_ONE_THREADS), 0, s, in, out, (int)n, total);
    INSC_LAUNCH_CHECK();
    return INSC_OK;
  }
  int64_t nb = cdiv(n, SCAN_TILE);
  void *ws;
  int rc = workspace(WS_SCAN, s, sizeof(int32_t) * (size_t)nb, &ws);
  if (rc) return rc;
  int32_t *bsums = (int32_t *)ws;
  hipLaunchKernelGGL(scan_block_sums, dim3((unsigned)nb), dim3(SCAN_THREADS), 0, s, in, n, bsums);
  if (nb <= SCAN_FUSED_MAX_BLOCKS) {
    hipLaunchKernelGGL(scan_final_fused, dim3((unsigned)nb), dim3(SCAN_THREADS), 0, s, in, out, n, bsums, total);
  } else {
    hipLaunchKernelGGL(scan_bsums, dim3(1), dim3(SCAN_THREADS), 0, s, bsums, nb, total);
    hipLaunchKernelGGL(scan_final, dim3((unsigned)nb), dim3(SCAN_THREADS), 0, s, in, out, n, bsums);
  }
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

// ---------------------------------------------------------------------------------------
// radix sort: 8 bits per pass, 256 threads x 8 rounds per block, stable
// ---------------------------------------------------------------------------------------
constexpr int SORT_THREADS = 256;
constexpr int SORT_ROUNDS = 8;
constexpr int SORT_TILE = SORT_THREADS * SORT_ROUNDS;
constexpr int SORT_FUSED_MAX_BLOCKS = 256;  // up to this many blocks (524 288 pairs) every scatter block sums the counts itself

// counts[digit * nb + block] for the scan over all counts, or - BY_BLOCK - counts[block * 256 + digit] for
// a scatter that adds them up itself
template <bool BY_BLOCK>
__device__ __forceinline__ void sort_hist_body(const uint64_t *__restrict__ keys, int64_t n, int shift,
                                               int32_t *__restrict__ counts, int nb, int *h /*[256]*/) {
  h[threadIdx.x] = 0;
  __syncthreads();
  int64_t base = (int64_t)blockIdx.x * SORT_TILE;
#pragma unroll
  for (int r = 0; r < SORT_ROUNDS; r++) {
    int64_t i = base + r * SORT_THREADS + threadIdx.x;
    if (i < n) atomicAdd(&h[(int)((keys[i] >> shift) & 255)], 1);
  }
  __syncthreads();
  if (BY_BLOCK)
    counts[(int64_t)blockIdx.x * 256 + threadIdx.x] = h[threadIdx.x];
  else
    counts[(int64_t)threadIdx.x * nb + blockIdx.x] = h[threadIdx.x];
}
template <bool FUSED>
__global__ __launch_bounds__(SORT_THREADS) void sort_hist(const uint64_t *__restrict__ keys, int64_t n, int shift,
                                                          int32_t *__restrict__ counts, int nb) {
  __shared__ int h[256];
  sort_hist_body<FUSED>(keys, n, shift, counts, nb, h);
}

// inv (nullable): the inverse of the permutation that vals_out receives, inv[vals_out[i]] = i
// offsets: the scanned counts, [digit * nb + block]; or - RAW - the counts themselves, [block * 256 + digit]:
// thread t then adds up the counts of digit t over the blocks (before this one, and all) and the block
// scans the digit totals, in place of a scan launch between the histogram and the scatter.
template <bool RAW>
__device__ __forceinline__ void sort_scatter_body(const uint64_t *__restrict__ keys_in,
                                                  const int32_t *__restrict__ vals_in, uint64_t *__restrict__ keys_out,
                                                  int32_t *__restrict__ vals_out, int32_t *__restrict__ inv, int64_t n,
                                                  int shift, const int32_t *__restrict__ offsets, int nb, int *base,
                                                  int (*wcount)[256]) {
  const int t = threadIdx.x, lane = t & 63, w = t >> 6;
  if (RAW) {
    int before = 0, total = 0;
    for (int b0 = 0; b0 < nb; b0 += 16) {  // (sixteen loads in flight at a time)
      int c[16];
#pragma unroll
      for (int u = 0; u < 16; u++) c[u] = b0 + u < nb ? offsets[(int64_t)(b0 + u) * 256 + t] : 0;
#pragma unroll
      for (int u = 0; u < 16; u++) {
        if (b0 + u < (int)blockIdx.x) before += c[u];
        total += c[u];
      }
    }
    const int inc = wave_incl_scan(total);
    if (lane == 63) wcount[0][w] = inc;
    __syncthreads();
    int off = 0;
    for (int i = 0; i < w; i++) off += wcount[0][i];
    base[t] = off + inc - total + before;
    __syncthreads();  // (wcount is cleared below)
  } else {
    base[t] = offsets[(int64_t)t * nb + blockIdx.x];
  }
  const int64_t tile = (int64_t)blockIdx.x * SORT_TILE;
  for (int r = 0; r < SORT_ROUNDS; r++) {
#pragma unroll
    for (int i = 0; i < SORT_THREADS / 64; i++) wcount[i][t] = 0;
    __syncthreads();
    int64_t i = tile + r * SORT_THREADS + t;
    bool valid = i < n;
    uint64_t key = valid ? keys_in[i] : 0;
    int val = valid ? vals_in[i] : 0;
    int digit = (int)((key >> shift) & 255);
    // lanes of this wave holding the same digit
    uint64_t peers = __ballot(valid);
#pragma unroll
    for (int b = 0; b < 8; b++) {
      uint64_t m = __ballot((digit >> b) & 1);
      peers &= ((digit >> b) & 1) ? m : ~m;
    }
    int rank_in_wave = __popcll(peers & ((1ull << lane) - 1ull));
    if (valid && rank_in_wave == 0) wcount[w][digit] = __popcll(peers);
    __syncthreads();
    if (valid) {
      int rank = base[digit] + rank_in_wave;
      for (int i2 = 0; i2 < w; i2++) rank += wcount[i2][digit];
      keys_out[rank] = key;
      vals_out[rank] = val;
      if (inv) inv[val] = rank;
    }
    __syncthreads();
    int add = 0;
#pragma unroll
    for (int i2 = 0; i2 < SORT_THREADS / 64; i2++) add += wcount[i2][t];
    base[t] += add;
    __syncthreads();
  }
}
template <bool FUSED>
__global__ __launch_bounds__(SORT_THREADS) void sort_scatter(const uint64_t *__restrict__ keys_in,
                                                             const int32_t *__restrict__ vals_in,
                                                             uint64_t *__restrict__ keys_out,
                                                             int32_t *__restrict__ vals_out, int64_t n, int shift,
                                                             const int32_t *__restrict__ offsets, int nb) {
  __shared__ int base[256];
  __shared__ int wcount[SORT_THREADS / 64][256];
  sort_scatter_body<FUSED>(keys_in, vals_in, keys_out, vals_out, nullptr, n, shift, offsets, nb, base, wcount);
}

// Several sorts of the same key width, pass by pass in the same launches (blockIdx.y = job): two
// launches per pass whatever the number of jobs (the scatter adds up the digit counts itself).  Jobs of at
// most SORT_BATCH_MAX_N pairs, i.e. 128 blocks whose counts every scatter block reads.
struct SortJobDev {
  uint64_t *k[2];
  int32_t *v[2];
  int32_t *vals_out, *inv, *counts;
  int64_t n;
  int nb;
};
struct SortBatchDev {
  SortJobDev job[SORT_BATCH_MAX_JOBS];
};
__global__ __launch_bounds__(SORT_THREADS) void sort_hist_batch(SortBatchDev b, int shift, int src) {
  __shared__ int h[256];
  const SortJobDev &j = b.job[blockIdx.y];
  if ((int)blockIdx.x >= j.nb) return;
  sort_hist_body<true>(j.k[src], j.n, shift, j.counts, j.nb, h);
}
__global__ __launch_bounds__(SORT_THREADS) void sort_scatter_batch(SortBatchDev b, int shift, int src, int last) {
  __shared__ int base[256];
  __shared__ int wcount[SORT_THREADS / 64][256];
  const SortJobDev &j = b.job[blockIdx.y];
  if ((int)blockIdx.x >= j.nb) return;
  sort_scatter_body<true>(j.k[src], j.v[src], j.k[src ^ 1], last ? j.vals_out : j.v[src ^ 1], last ? j.inv : nullptr, j.n,
                          shift, j.counts, j.nb, base, wcount);
}

int sort_pairs_u64(uint64_t *keys, int32_t *vals, int64_t n, int key_bits, hipStream_t s) {
  if (n <= 1 || key_bits <= 0) return INSC_OK;
  if (key_bits > 64) key_bits = 64;
  const int passes = (key_bits + 7) / 8;
  const int64_t nb64 = cdiv(n, SORT_TILE);
  if (nb64 > (1 << 22)) {
    set_error("sort_pairs_u64: n=%lld too large", (long long)n);
    return INSC_ERR_ARG;
  }
  const int nb = (int)nb64;
  size_t off_keys = 0;
  size_t off_vals = off_keys + sizeof(uint64_t) * (size_t)n;
  size_t off_cnt = (off_vals + sizeof(int32_t) * (size_t)n + 255) & ~(size_t)255;
  size_t bytes = off_cnt + sizeof(int32_t) * 256 * (size_t)nb;
  void *ws;
  int rc = workspace(WS_SORT, s, bytes, &ws);
  if (rc) return rc;
  uint64_t *k2 = (uint64_t *)((char *)ws + off_keys);
  int32_t *v2 = (int32_t *)((char *)ws + off_vals);
  int32_t *counts = (int32_t *)((char *)ws + off_cnt);
  uint64_t *kin = keys, *kout = k2;
  int32_t *vin = vals, *vout = v2;
  for (int p = 0; p < passes; p++) {
    int shift = 8 * p;
    if (nb <= SORT_FUSED_MAX_BLOCKS) {  // (the scatter adds up the digit counts itself: two launches per pass)
      hipLaunchKernelGGL(sort_hist<true>, dim3(nb), dim3(SORT_THREADS), 0, s, kin, n, shift, counts, nb);
      hipLaunchKernelGGL(sort_scatter<true>, dim3(nb), dim3(SORT_THREADS), 0, s, kin, vin, kout, vout, n, shift, counts, nb);
    } else {
      hipLaunchKernelGGL(sort_hist<false>, dim3(nb), dim3(SORT_THREADS), 0, s, kin, n, shift, counts, nb);
      rc = scan_exclusive_i32(counts, counts, 256 * (int64_t)nb, nullptr, s);
      if (rc) return rc;
      hipLaunchKernelGGL(sort_scatter<false>, dim3(nb), dim3(SORT_THREADS), 0, s, kin, vin, kout, vout, n, shift, counts, nb);
    }
    INSC_LAUNCH_CHECK();
    uint64_t *tk = kin; kin = kout; kout = tk;
    int32_t *tv = vin; vin = vout; vout = tv;
  }
  if (kin != keys) {
    INSC_HIP(hipMemcpyAsync(keys, kin, sizeof(uint64_t) * (size_t)n, hipMemcpyDeviceToDevice, s));
    INSC_HIP(hipMemcpyAsync(vals, vin, sizeof(int32_t) * (size_t)n, hipMemcpyDeviceToDevice, s));
  }
  return INSC_OK;
}

// The same sort with the values delivered into another array: vals_out gets the values in key order,
// keys and vals_in are scratch afterwards.  No copy at the end, whatever the number of passes.
int sort_pairs_u64_into(uint64_t *keys, int32_t *vals_in, int32_t *vals_out, int64_t n, int key_bits, hipStream_t s) {
  if (n <= 0) return INSC_OK;
  if (key_bits > 64) key_bits = 64;
  const int passes = key_bits <= 0 ? 0 : (key_bits + 7) / 8;
  if (n == 1 || passes == 0) {
    INSC_HIP(hipMemcpyAsync(vals_out, vals_in, sizeof(int32_t) * (size_t)n, hipMemcpyDeviceToDevice, s));
    return INSC_OK;
  }
  const int64_t nb64 = cdiv(n, SORT_TILE);
  if (nb64 > (1 << 22)) {
    set_error("sort_pairs_u64_into: n=%lld too large", (long long)n);
    return INSC_ERR_ARG;
  }
  const int nb = (int)nb64;
  size_t off_keys = 0;
  size_t off_vals = off_keys + sizeof(uint64_t) * (size_t)n;
  size_t off_cnt = (off_vals + sizeof(int32_t) * (size_t)n + 255) & ~(size_t)255;
  size_t bytes = off_cnt + sizeof(int32_t) * 256 * (size_t)nb;
  void *ws;
  int rc = workspace(WS_SORT, s, bytes, &ws);
  if (rc) return rc;
  uint64_t *k2 = (uint64_t *)((char *)ws + off_keys);
  int32_t *v2 = (int32_t *)((char *)ws + off_vals);
  int32_t *counts = (int32_t *)((char *)ws + off_cnt);
  uint64_t *kin = keys, *kout = k2;
  int32_t *vin = vals_in, *vout = v2;
  for (int p = 0; p < passes; p++) {
    const int shift = 8 * p;
    const bool last = p + 1 == passes;
    // (the keys of the last pass go where they would have gone; nobody reads them)
    if (nb <= SORT_FUSED_MAX_BLOCKS) {
      hipLaunchKernelGGL(sort_hist<true>, dim3(nb), dim3(SORT_THREADS), 0, s, kin, n, shift, counts, nb);
      hipLaunchKernelGGL(sort_scatter<true>, dim3(nb), dim3(SORT_THREADS), 0, s, kin, vin, kout, last ? vals_out : vout, n,
                         shift, counts, nb);
    } else {
      hipLaunchKernelGGL(sort_hist<false>, dim3(nb), dim3(SORT_THREADS), 0, s, kin, n, shift, counts, nb);
      rc = scan_exclusive_i32(counts, counts, 256 * (int64_t)nb, nullptr, s);
      if (rc) return rc;
      hipLaunchKernelGGL(sort_scatter<false>, dim3(nb), dim3(SORT_THREADS), 0, s, kin, vin, kout, last ? vals_out : vout, n,
                         shift, counts, nb);
    }
    INSC_LAUNCH_CHECK();
    uint64_t *tk = kin; kin = kout; kout = tk;
    int32_t *tv = vin; vin = vout; vout = tv;
  }
  return INSC_OK;
}

int sort_pairs_u64_into_batch(const SortJob *jobs, int n_jobs, int key_bits, hipStream_t s) {
  if (n_jobs <= 0) return INSC_OK;
  if (n_jobs > SORT_BATCH_MAX_JOBS || key_bits <= 0 || key_bits > 64) {
    set_error("sort_pairs_u64_into_batch: %d jobs, %d key bits", n_jobs, key_bits);
    return INSC_ERR_ARG;
  }
  const int passes = (key_bits + 7) / 8;
  SortBatchDev b;
  size_t bytes = 0;
  int nb_max = 0;
  for (int i = 0; i < n_jobs; i++) {
    if (jobs[i].n < 1 || jobs[i].n > SORT_BATCH_MAX_N) {
      set_error("sort_pairs_u64_into_batch: job %d has %lld pairs (1..%lld)", i, (long long)jobs[i].n,
                (long long)SORT_BATCH_MAX_N);
      return INSC_ERR_ARG;
    }
    bytes += (sizeof(uint64_t) + sizeof(int32_t)) * (size_t)jobs[i].n + 256 * sizeof(int32_t) * (size_t)cdiv(jobs[i].n, SORT_TILE) + 768;
  }
  void *ws;
  int rc = workspace(WS_SORT, s, bytes, &ws);
  if (rc) return rc;
  char *p = (char *)ws;
  auto take = [&](size_t nbytes) -> void * {
    void *r = p;
    p += (nbytes + 255) & ~(size_t)255;
    return r;
  };
  for (int i = 0; i < n_jobs; i++) {
    SortJobDev &j = b.job[i];
    j.n = jobs[i].n;
    j.nb = (int)cdiv(j.n, SORT_TILE);
    nb_max = std::max(nb_max, j.nb);
    j.k[0] = jobs[i].keys;
    j.v[0] = jobs[i].vals_in;
    j.k[1] = (uint64_t *)take(sizeof(uint64_t) * (size_t)j.n);
    j.v[1] = (int32_t *)take(sizeof(int32_t) * (size_t)j.n);
    j.counts = (int32_t *)take(sizeof(int32_t) * 256 * (size_t)j.nb);
    j.vals_out = jobs[i].vals_out;
    j.inv = jobs[i].inv_out;
  }
  for (int pass = 0; pass < passes; pass++) {
    const int src = pass & 1, last = pass + 1 == passes;
    hipLaunchKernelGGL(sort_hist_batch, dim3((unsigned)nb_max, (unsigned)n_jobs), dim3(SORT_THREADS), 0, s, b, 8 * pass, src);
    hipLaunchKernelGGL(sort_scatter_batch, dim3((unsigned)nb_max, (unsigned)n_jobs), dim3(SORT_THREADS), 0, s, b, 8 * pass, src,
                       last);
    INSC_LAUNCH_CHECK();
  }
  return INSC_OK;
}

}  // namespace insc

extern "C" {

int insc_scan_exclusive_i32(const int32_t *d_in, int32_t *d_out, int64_t n, int32_t *d_total, void *stream) {
  INSC_REQUIRE(n >= 0 && ((d_in && d_out) || n == 0), INSC_ERR_ARG, "insc_scan_exclusive_i32: bad arguments");
  return insc::scan_exclusive_i32(d_in, d_out, n, d_total, (hipStream_t)stream);
}

int insc_sort_pairs_u64(uint64_t *d_keys, int32_t *d_vals, int64_t n, int key_bits, void *stream) {
  INSC_REQUIRE(n >= 0 && ((d_keys && d_vals) || n == 0), INSC_ERR_ARG, "insc_sort_pairs_u64: bad arguments");
  INSC_REQUIRE(key_bits >= 0 && key_bits <= 64, INSC_ERR_ARG, "insc_sort_pairs_u64: key_bits %d", key_bits);
  return insc::sort_pairs_u64(d_keys, d_vals, n, key_bits, (hipStream_t)stream);
}

}  // extern "C"
